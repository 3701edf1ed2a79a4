"""The drop-in claim at the source level, on the CPU: tests/callsite/call_site.cpp -- a translation unit that calls
heuristic_prepare with the reference's 40 arguments (multi_head_cache_attention.h:107-148), the stage functions,
kv_cache_reorder / kv_cache_invert_reorder, dynamic_batching_rotary_position_embedding and row_parallel_linear
through the reference's prototypes -- is compiled with g++ against include/pmx_hip/*.h, linked with libpmx_hip.so and run.  No GPU: the
prepare step is host code and the stage calls are made on an empty batch."""
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_reference_style_call_site_compiles_links_and_runs(pkg, hip_lib, tmp_path):
    lib_dir = os.path.dirname(pkg._lib.LIB_PATH)
    exe = str(tmp_path / "call_site")
    cmd = ["g++", "-std=c++17", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
           "-I" + os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "callsite", "call_site.cpp"), "-o", exe,
           "-L" + lib_dir, "-l:libpmx_hip.so", "-L/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-3000:]
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    out = dict(line.split("=", 1) if line.count("=") == 1 else (line, "") for line in r.stdout.splitlines())
    lines = r.stdout.splitlines()
    assert lines[0] == "prepare rc=0"
    scale = float(np.float32(1.0 / np.sqrt(np.float32(128))))
    pieces = 256 + 128  # one workgroup of four waves per CU on 256 CUs, one group of eight kv heads; one more piece per sequence
    assert lines[1] == ("prefill_batches=0 q_stride_s=4096 k_stride_s=1024 o_stride_s=4096 num_kv_repeats=4 "
                        "attn_scale=%.9g decoding_algo=3 multi_block=256 workspace_size=%d" % (scale, pieces * 32 * 130 * 4))
    assert lines[2] == "device_prop kept by pointer: 1"
    assert lines[3] == "bad heads rc=2"
    assert lines[4] == "idle prepare rc=0 kvstore=0 decode=0 prefill=0 forward=0"
    assert lines[5] == "reorder(no pages)=0 invert(no pages)=0"
    assert lines[6] == "rope(empty batch)=0"
    assert lines[7] == "kvcache(empty batch)=0"
    assert lines[8] == "linear(no rows)=0 linear(not parallel)=2"
    assert lines[9] == "linear_ref(no rows)=0 linear_ref(null comm)=0 linear_ref(two ranks)=2"
    assert out is not None
