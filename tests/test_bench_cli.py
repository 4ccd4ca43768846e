"""bench.py's command-line contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                          timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_counter_file_of_the_profiler_is_read_per_kernel(tmp_path):
    """bench.py takes its live traffic figure from rocprofv3's counter_collection.csv: median over the copy
    kernel's dispatches, the yardstick kernel apart, other kernels and counters ignored."""
    sys.path.insert(0, ROOT)
    import bench
    rows = [("copy_uniform_kernel<1, 4, 1>(x)", "A", 10.0), ("copy_uniform_kernel<1, 4, 1>(x)", "A", 30.0),
            ("copy_uniform_kernel<1, 4, 1>(x)", "A", 20.0), ("copy_uniform_kernel<1, 4, 1>(x)", "B", 7.0),
            ("void at::native::vectorized_elementwise_kernel<4, at::native::CUDAFunctorOnSelf_add<int>, a>(b)", "A", 5.0),
            ("void at::native::vectorized_elementwise_kernel<4, at::native::CUDAFunctorOnSelf_add<int>, a>(b)", "A", 6.0),
            ("void at::native::vectorized_elementwise_kernel<4, at::native::CUDAFunctorOnSelf_add<int>, a>(b)", "B", 2.0),
            ("some_other_kernel(y)", "A", 1e9), ("copy_uniform_kernel<1, 4, 1>(x)", "C", 1e9)]
    path = tmp_path / "t_counter_collection.csv"
    with open(path, "w") as f:
        f.write('"Dispatch_Id","Kernel_Name","Counter_Name","Counter_Value"\n')
        for i, (k, c, v) in enumerate(rows):
            f.write(f'{i},"{k}","{c}",{v}\n')
    kernel, yard, n = bench.counter_samples(str(path), ["A", "B"])
    assert kernel == {"A": 20.0, "B": 7.0} and yard == {"A": 6.0, "B": 2.0} and n == 3
    assert bench.counter_samples(str(path), ["A", "D"]) is None


def test_phase_timers_are_read_from_the_debug_lines():
    """bench.py's breakdown of a request made through prepXfer comes from the debug lines of the
    agent and of the plugin: one entry per request and phase, other lines ignored."""
    sys.path.insert(0, ROOT)
    import bench
    text = "\n".join([
        "[nixl D] backend HIP: prepared 524288 descriptors into 1 strides",
        "[nixl D] makeXferReq: merged 65536 indices into 65536 descriptors in 128.5 us",
        "[nixl D] HIP backend: prepXfer of 65536 descriptors (blocks): block pass 124.525 us, plan from records 8.03 us, "
        "rest (general lowering, event, stream) 0.611 us",
        "[nixl D] makeXferReq: merged 65536 indices into 65472 descriptors in 1.3e+02 us",
        "[nixl D] HIP backend: prepXfer of 65472 descriptors (general): block pass 0 us, plan from records 0 us, "
        "rest (general lowering, event, stream) 2500.5 us"])
    phases, paths = bench.parse_prep_debug_lines(text)
    assert phases == {"agent_expand_index_pairs": [128.5, 130.0], "plugin_block_pass": [124.525, 0.0],
                      "plugin_plan_from_records": [8.03, 0.0], "plugin_rest": [0.611, 2500.5]}
    assert paths == ["blocks", "general"]


def test_counter_file_is_read_for_several_kernels_at_once(tmp_path):
    """The expert-parallel traffic figures: medians per kernel tag from one counter file, a tag
    without samples left out, the yardstick apart."""
    sys.path.insert(0, ROOT)
    import bench
    rows = [("void (anonymous namespace)::ll_bits_kernel<false, 1>(a)", "A", 3.0),
            ("void (anonymous namespace)::ll_bits_kernel<true, 4>(a)", "A", 100.0),
            ("void (anonymous namespace)::ll_dispatch_kernel<true>(a)", "A", 10.0),
            ("void (anonymous namespace)::ll_dispatch_kernel<true>(a)", "A", 30.0),
            ("void (anonymous namespace)::ll_dispatch_kernel<true>(a)", "A", 20.0),
            ("void at::native::vectorized_elementwise_kernel<4, at::native::CUDAFunctorOnSelf_add<int>, a>(b)", "A", 8.0)]
    path = tmp_path / "t_counter_collection.csv"
    with open(path, "w") as f:
        f.write('"Dispatch_Id","Kernel_Name","Counter_Name","Counter_Value"\n')
        for i, (k, c, v) in enumerate(rows):
            f.write(f'{i},"{k}","{c}",{v}\n')
    medians, yard = bench.counter_medians(str(path), ["A"], ["ll_bits_kernel<false", "ll_dispatch_kernel<true>", "ll_scales_kernel"])
    assert medians == {"ll_bits_kernel<false": {"A": 3.0}, "ll_dispatch_kernel<true>": {"A": 20.0}} and yard == {"A": 8.0}
