"""Host-side checks of the benchmark driver that need no GPU."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode != 0
    assert "one GPU" in p.stderr and p.stdout.strip() == ""


def test_unknown_workload_lists_the_known_ones():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "nope"], capture_output=True, text=True)
    assert p.returncode != 0
    for name in ("decode_fp8_32k_32layers", "prefill_fp8_512x4608_32layers", "copy_calibration"):
        assert name in p.stderr


def test_workload_tables_state_the_configurations_algorithmic_work():
    sys.path.insert(0, ROOT)
    from vulkanforge_amd import workloads
    head = workloads.DECODE["decode_fp8_32k_32layers"]
    assert head.kv_bytes_step() == 2 * 32768 * 8 * 128 * 32                      # K and V of every visible key once, 32 layers
    assert head.kv_bytes_layer(0) == 67_108_864
    pf = workloads.PREFILL["prefill_fp8_512x4608_32layers"]
    assert pf.flops_layer() == sum(4096 + i + 1 for i in range(512)) * 32 * 4 * 128
    sliding = workloads.DECODE["decode_f16_hd256_sliding_12layers"]
    assert [sliding.layer_window(i) for i in range(6)] == [4096] * 5 + [0]        # five sliding layers, then a global one
    assert json.dumps({"ok": True})                                               # (bench lines are plain JSON)


def test_calibration_library_loads_and_exports_what_the_benchmark_calls():
    # (no device work: symbols only)
    import ctypes
    lib = ctypes.CDLL(os.path.join(ROOT, "vulkanforge_amd", "libvfkv_calib.so"))
    for name in ("vfkv_calib_stream_read", "vfkv_calib_pattern_read", "vfkv_calib_empty"):
        assert hasattr(lib, name), name
    with open(os.path.join(ROOT, "bench.py")) as f:
        text = f.read()
    import re
    for name in set(re.findall(r"calib\.(vfkv_calib_\w+)", text)):
        assert hasattr(lib, name), name
