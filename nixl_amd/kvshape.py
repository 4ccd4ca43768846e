"""Sizes of a paged KV cache, from which the descriptor lists of a KV transfer get their shape.

The arithmetic is the one of the reference's KV benchmark models
(benchmark/kvbench/models/llama3_1.py:62-95, deepseek_r1.py:69-109, qwen3.py:64-104,
gpt_oss.py:63-103, utils.py:23-40): bytes of KV cache per token, bytes of one IO request for a
given tensor/pipeline split and access pattern, and requests per batch.  `paged_kv_layout`
then states what a block-granular transfer looks like in memory: one descriptor per (layer,
K or V, block), which is how bench.py and the tests lay out their pools.

Model parameters are those of the reference's example files
(benchmark/kvbench/examples/model_*.yaml); `Strategy` carries the fields of its strategy
files (examples/block-tp1-pp1.yaml and siblings).
"""
import math
from dataclasses import dataclass

# bytes per element (models/utils.py:23-33)
PRECISION_BYTES = {"fp8": 1, "int8": 1, "fp16": 2, "bfloat16": 2}


def precision_size(precision):
    try:
        return PRECISION_BYTES[precision]
    except KeyError:
        raise ValueError(f"Unsupported precision: {precision}") from None


@dataclass
class Strategy:
    """The strategy / runtime / system sections of a kvbench configuration file."""
    tp_size: int = 1
    pp_size: int = 1
    model_quant_mode: str = "fp8"
    kvcache_quant_mode: str = "fp8"
    access_pattern: str = "block"  # "block": one request spans the layers of a pipeline stage; "layer": one layer
    page_size: int = 16
    isl: int = 1000
    osl: int = 100
    num_requests: int = 10


class _GqaModel:
    """Grouped-query attention: layers x KV heads x head dimension x {K, V}."""

    def __init__(self, name, num_layers, num_kv_heads, head_dim, strategy=None):
        self.model_name = name
        self.num_layers = num_layers
        self.num_kv_heads = num_kv_heads
        self.query_head_dimension = head_dim
        self.strategy = strategy or Strategy()

    def get_kv_size_per_token(self, token_count=1):
        # these models size their cache by model_quant_mode (llama3_1.py:74, qwen3.py:84, gpt_oss.py:83)
        return int(self.num_layers * self.num_kv_heads * self.query_head_dimension * 2 *
                   precision_size(self.strategy.model_quant_mode) * token_count)

    def get_io_size(self, page_size=1):
        per_layer = int(self.get_kv_size_per_token() / self.num_layers)
        if per_layer <= 0:
            raise ValueError("Invalid KV Size: 0")
        io_size = int(per_layer / self.strategy.tp_size)
        if self.strategy.access_pattern == "block":
            io_size = int(io_size * (self.num_layers / self.strategy.pp_size))
        return int(io_size * page_size)


class Llama31(_GqaModel):
    """models/llama3_1.py: KV heads = query heads / queries per group."""

    def __init__(self, name, num_layers, num_query_heads_with_mha, query_head_dimension, gqa_num_queries_in_group,
                 strategy=None):
        super().__init__(name, num_layers, num_query_heads_with_mha / gqa_num_queries_in_group, query_head_dimension,
                         strategy)


class Qwen3(_GqaModel):
    """models/qwen3.py."""


class GptOss(_GqaModel):
    """models/gpt_oss.py."""


class DeepSeekR1:
    """models/deepseek_r1.py: multi-head latent attention keeps one latent vector plus the rope
    part per token and layer, sized by kvcache_quant_mode."""

    def __init__(self, name, num_layers, rope_mla_dimension, mla_latent_vector_dimension, strategy=None):
        self.model_name = name
        self.num_layers = num_layers
        self.rope_mla_dimension = rope_mla_dimension
        self.mla_latent_vector_dimension = mla_latent_vector_dimension
        self.strategy = strategy or Strategy()

    def get_kv_size_per_token(self, token_count=1):
        return int((self.rope_mla_dimension + self.mla_latent_vector_dimension) *
                   precision_size(self.strategy.kvcache_quant_mode) * self.num_layers) * token_count

    def get_io_size(self, page_size=1):
        kv_size = self.get_kv_size_per_token()
        if kv_size <= 0:
            raise ValueError("Invalid KV Size: 0")
        io_size = int(kv_size / self.num_layers) / self.strategy.tp_size
        if self.strategy.access_pattern == "block":
            io_size = io_size * math.ceil(self.num_layers / self.strategy.pp_size)
        return int(io_size * page_size)


# benchmark/kvbench/examples/model_*.yaml
def model(name, strategy=None):
    table = {
        "LLAMA3.1_8B": lambda: Llama31("LLAMA3.1_8B", 32, 32, 128, 4, strategy),
        "LLAMA3.1_70B": lambda: Llama31("LLAMA3.1_70B", 80, 64, 128, 8, strategy),
        "DEEPSEEK_R1": lambda: DeepSeekR1("DEEPSEEK_R1", 61, 64, 512, strategy),
        "QWEN3_8B": lambda: Qwen3("QWEN3_8B", 36, 8, 128, strategy),
        "GPT_OSS_20B": lambda: GptOss("GPT_OSS_20B", 24, 8, 64, strategy),
    }
    try:
        return table[name.upper()]()
    except KeyError:
        raise ValueError(f"unknown model {name!r}; known: {sorted(table)}") from None


def get_batch_size(m, io_size):
    """Requests per batch (models/utils.py:36-40)."""
    return math.ceil(m.get_kv_size_per_token(int(m.strategy.isl)) / io_size * m.strategy.num_requests)


@dataclass
class PagedKvLayout:
    layers: int
    sub_blocks_per_layer: int  # 2 (K and V) for attention with separate keys and values, 1 for a latent cache
    bytes_per_sub_block: int  # one descriptor
    tokens_per_block: int

    @property
    def descriptors_per_block(self):
        return self.layers * self.sub_blocks_per_layer

    @property
    def bytes_per_block(self):
        return self.descriptors_per_block * self.bytes_per_sub_block


def paged_kv_layout(m, tokens_per_block=None, precision=None):
    """What moving one KV block means as descriptors: per layer, K and V each hold
    tokens_per_block x (KV size per token and layer / 2) bytes.  `precision` overrides the
    strategy's quantisation (the benchmark pools hold bf16)."""
    tokens = tokens_per_block or m.strategy.page_size
    per_token_layer = m.get_kv_size_per_token() // m.num_layers
    if precision is not None:
        quant = m.strategy.kvcache_quant_mode if isinstance(m, DeepSeekR1) else m.strategy.model_quant_mode
        per_token_layer = per_token_layer // precision_size(quant) * precision_size(precision)
    subs = 1 if isinstance(m, DeepSeekR1) else 2
    return PagedKvLayout(m.num_layers, subs, per_token_layer // subs * tokens, tokens)
