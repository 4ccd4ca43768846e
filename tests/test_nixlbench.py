"""The nixlbench-style harness: flag handling, sweep order, report format and the byte check,
on the CPU with the per-descriptor memcpy backend; on the GPU with the HIP backend."""
import io

import pytest

from nixl_amd import nixlbench


def _run(argv):
    out = io.StringIO()
    rc, results = nixlbench.main(argv, out)
    return rc, results, out.getvalue()


COMMON = ["--start_block_size", "4096", "--max_block_size", "16384", "--start_batch_size", "4", "--max_batch_size", "16",
          "--num_iter", "12", "--warmup_iter", "2", "--check_consistency"]


@pytest.mark.parametrize("extra", [[], ["--prepared_xfer"], ["--op_type", "READ", "--pipeline_depth", "2"],
                                   ["--recreate_xfer", "--randomize_location_mode", "blockaligned"]])
def test_sweep_on_cpu_backend(oracle_plugin_dir, extra):
    rc, results, text = _run(["--backend", "MEMCPY", "--plugin_dir", oracle_plugin_dir, "--initiator_seg_type", "DRAM",
                              "--target_seg_type", "DRAM"] + COMMON + extra)
    assert rc == 0, text
    # block sizes double on the outside, batch sizes on the inside (utils.cpp sweep order)
    assert [(r["block"], r["batch"]) for r in results] == [(b, n) for b in (4096, 8192, 16384) for n in (4, 8, 16)]
    assert all(r["consistent"] is True and r["gbps"] > 0 for r in results)
    lines = text.splitlines()
    assert lines[1].split()[:6] == ["Block", "Size", "(B)", "Batch", "Size", "B/W"]
    assert len([l for l in lines if l.endswith("consistency: ok")]) == 9


def test_threads_share_a_point_on_cpu_backend(oracle_plugin_dir):
    """--num_threads: each thread drives its own requests over its own part of the buffers
    (benchmark/nixlbench/src/worker/nixl/nixl_worker.cpp:1847-1879); every thread's bytes are
    checked, the report has one line a point."""
    rc, results, text = _run(["--backend", "MEMCPY", "--plugin_dir", oracle_plugin_dir, "--initiator_seg_type", "DRAM",
                              "--target_seg_type", "DRAM", "--num_threads", "3", "--pipeline_depth", "2"] + COMMON)
    assert rc == 0, text
    assert len(results) == 9 and all(r["consistent"] is True and r["threads"] == 3 and r["gbps"] > 0 for r in results)
    assert "3 threads" in text.splitlines()[0]
    with pytest.raises(SystemExit):
        nixlbench.parse(["--num_threads", "5", "--num_iter", "12"])


def test_bad_flags_are_rejected():
    with pytest.raises(SystemExit):
        nixlbench.parse(["--start_block_size", "8192", "--max_block_size", "4096"])
    with pytest.raises(SystemExit):
        nixlbench.parse(["--max_block_size", str(1 << 30), "--max_batch_size", "64", "--total_buffer_size", str(1 << 30)])


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [["--prepared_xfer"], ["--op_type", "READ", "--pipeline_depth", "4"]])
def test_sweep_on_hip_backend(cuda, extra):
    rc, results, text = _run(["--backend", "HIP"] + COMMON + extra)
    assert rc == 0, text
    assert len(results) == 9 and all(r["consistent"] is True for r in results)


@pytest.mark.gpu
def test_threads_on_hip_backend(cuda):
    rc, results, text = _run(["--backend", "HIP", "--backend_params", "num_streams=2", "--num_threads", "2", "--prepared_xfer"]
                             + COMMON)
    assert rc == 0, text
    assert len(results) == 9 and all(r["consistent"] is True and r["threads"] == 2 for r in results)


@pytest.mark.gpu
def test_hip_backend_pinned_host_to_vram(cuda):
    rc, results, text = _run(["--backend", "HIP", "--initiator_seg_type", "DRAM", "--target_seg_type", "VRAM"] + COMMON)
    assert rc == 0, text
