"""The KV-size arithmetic that fixes the descriptor shape of a paged-KV transfer, pinned on
every known answer the reference's own test holds (benchmark/kvbench/test/test_kvcache.py:
32-76 for bytes per token, :79-102 for bytes per IO request; strategy values from
benchmark/kvbench/examples/{block,layer}-tp*-pp*.yaml: fp8 model and cache, page size 16)."""
import pytest

from nixl_amd import kvshape


def _strategy(pattern, tp, pp):
    return kvshape.Strategy(tp_size=tp, pp_size=pp, access_pattern=pattern)


KV_PER_TOKEN = (
    [("LLAMA3.1_8B", "block", 1, pp, 65536) for pp in (1, 2, 4, 8)]
    + [("LLAMA3.1_8B", "block", 8, pp, 65536) for pp in (2, 4, 8, 16, 32)]
    + [("LLAMA3.1_8B", "layer", 1, pp, 65536) for pp in (1, 2, 4, 8)]
    + [("LLAMA3.1_70B", "block", 1, pp, 163840) for pp in (1, 2, 4, 8)]
    + [("LLAMA3.1_70B", "block", 8, pp, 163840) for pp in (2, 4, 8, 16, 32)]
    + [("LLAMA3.1_70B", "layer", 1, pp, 163840) for pp in (1, 2, 4, 8)]
    + [("DEEPSEEK_R1", "block", 8, pp, 35136) for pp in (2, 4, 8, 16, 32)]
)


@pytest.mark.parametrize("name, pattern, tp, pp, want", KV_PER_TOKEN)
def test_kv_bytes_per_token_known_answers(name, pattern, tp, pp, want):
    assert kvshape.model(name, _strategy(pattern, tp, pp)).get_kv_size_per_token(1) == want


IO_SIZE = (
    [("LLAMA3.1_70B", "block", 8, pp, want) for pp, want in ((2, 10240), (4, 5120), (8, 2560), (16, 1280), (32, 640))]
    + [("LLAMA3.1_70B", "layer", 8, pp, 256) for pp in (2, 4, 8, 16, 32)]
)


@pytest.mark.parametrize("name, pattern, tp, pp, want", IO_SIZE)
def test_io_request_bytes_known_answers(name, pattern, tp, pp, want):
    assert kvshape.model(name, _strategy(pattern, tp, pp)).get_io_size() == want


def test_token_count_scales_and_other_families():
    m = kvshape.model("LLAMA3.1_8B")
    assert m.get_kv_size_per_token(1000) == 65536 * 1000
    # grouped-query families from their definition: layers x KV heads x head dim x {K, V} x bytes
    assert kvshape.model("QWEN3_8B").get_kv_size_per_token() == 36 * 8 * 128 * 2
    assert kvshape.model("GPT_OSS_20B").get_kv_size_per_token() == 24 * 8 * 64 * 2
    bf16 = kvshape.Strategy(model_quant_mode="bfloat16")
    assert kvshape.model("LLAMA3.1_8B", bf16).get_kv_size_per_token() == 2 * 65536
    # DeepSeek sizes its cache by the cache's quantisation, not the model's (deepseek_r1.py:82)
    assert kvshape.model("DEEPSEEK_R1", bf16).get_kv_size_per_token() == 35136
    assert kvshape.model("DEEPSEEK_R1", kvshape.Strategy(kvcache_quant_mode="fp16")).get_kv_size_per_token() == 2 * 35136
    with pytest.raises(ValueError):
        kvshape.model("LLAMA3.1_8B", kvshape.Strategy(model_quant_mode="fp4")).get_kv_size_per_token()
    with pytest.raises(ValueError):
        kvshape.model("nope")
    # requests per batch (models/utils.py:36-40): ceil(KV bytes of the input sequence / request bytes x requests)
    m = kvshape.model("LLAMA3.1_70B", _strategy("block", 8, 2))
    assert kvshape.get_batch_size(m, m.get_io_size(16)) == -(-163840 * 1000 * 10 // (10240 * 16))


def test_paged_layout_of_the_benchmark_configuration():
    """The KV benchmark's shape follows from the model: Llama-3.1-8B, 16 tokens per block, bf16:
    32 layers x {K, V} descriptors of 8 heads x 128 x 2 B x 16 tokens = 32 KiB per block."""
    lay = kvshape.paged_kv_layout(kvshape.model("LLAMA3.1_8B"), 16, "bfloat16")
    assert (lay.layers, lay.sub_blocks_per_layer, lay.bytes_per_sub_block) == (32, 2, 32768)
    assert lay.descriptors_per_block == 64 and lay.bytes_per_block == 2 << 20
    assert 1024 * lay.descriptors_per_block == 65536  # descriptors of a 1024-block request
    fp8 = kvshape.paged_kv_layout(kvshape.model("LLAMA3.1_8B"))
    assert fp8.bytes_per_sub_block == 16384 and fp8.tokens_per_block == 16
    mla = kvshape.paged_kv_layout(kvshape.model("DEEPSEEK_R1"), 64)
    assert (mla.layers, mla.sub_blocks_per_layer, mla.bytes_per_sub_block) == (61, 1, 576 * 64)
