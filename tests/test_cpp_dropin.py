"""The C++ drop-in headers (blitz_scale_amd/cpp) used the way the reference's worker uses its own:
a hipcc-built program runs a prefill and a decode step of one layer and checks them against the CPU
checker.  The binary is built on the CPU side (build_cpp_test) and only executed on the GPU box."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_dropin")
LAYER_BIN = os.path.join(ROOT, "tests", "cpp", "layer_step")
ORDER_BIN = os.path.join(ROOT, "tests", "cpp", "test_reference_order")


def build_cpp_test():
    import oracle
    oracle.build()
    cpp = os.path.join(ROOT, "blitz_scale_amd", "cpp")
    cmd = ["/opt/rocm/bin/hipcc", "--offload-arch=gfx950", "-O2", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-I", os.path.join(ROOT, "include"), "-I", cpp, "-I", os.path.join(cpp, "kernel"),
           os.path.join(ROOT, "tests", "cpp", "test_dropin.cpp"), "-o", BIN,
           "-L", os.path.join(ROOT, "blitz_scale_amd", "lib"), "-lbz_hip", "-L", os.path.join(ROOT, "oracle"), "-lbz_oracle",
           "-Wl,-rpath,$ORIGIN/../../blitz_scale_amd/lib", "-Wl,-rpath,$ORIGIN/../../oracle"]
    out = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in out.stderr.splitlines() if "packed-fp32-ops" not in l)
    if out.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    # the layer step with every GEMM on hipBLASLt (blitz_scale_amd/cpp/util/hipblaslt_gemm.h)
    cmd2 = cmd[:cmd.index(os.path.join(ROOT, "tests", "cpp", "test_dropin.cpp"))] + [
        os.path.join(ROOT, "tests", "cpp", "layer_step.cpp"), "-o", LAYER_BIN,
        "-L", os.path.join(ROOT, "blitz_scale_amd", "lib"), "-lbz_hip", "-L", "/opt/rocm/lib", "-lhipblaslt",
        "-L", os.path.join(ROOT, "oracle"), "-lbz_oracle_omp",
        "-Wl,-rpath,$ORIGIN/../../blitz_scale_amd/lib", "-Wl,-rpath,$ORIGIN/../../oracle"]
    out = subprocess.run(cmd2, capture_output=True, text=True)
    err = "\n".join(l for l in out.stderr.splitlines() if "packed-fp32-ops" not in l)
    if out.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    # the reference's own call order and argument lists against the checker's kRoPELlama mode, two models on two threads
    i = cmd.index(os.path.join(ROOT, "tests", "cpp", "test_dropin.cpp"))
    cmd3 = cmd[:i] + [os.path.join(ROOT, "tests", "cpp", "test_reference_order.cpp"), "-o", ORDER_BIN, "-pthread"] + cmd[i + 3:]
    out = subprocess.run(cmd3, capture_output=True, text=True)
    err = "\n".join(l for l in out.stderr.splitlines() if "packed-fp32-ops" not in l)
    if out.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + err)
    return BIN


def test_headers_compile_and_link_without_a_gpu():
    assert os.path.exists(build_cpp_test()) and os.path.exists(LAYER_BIN) and os.path.exists(ORDER_BIN)


@pytest.mark.gpu
def test_reference_call_order_gives_rope_llama_results():
    """prefill attention -> 4-argument store; 3-argument append -> 5-argument decode, raw q/k/v, header defaults only."""
    if not os.path.exists(ORDER_BIN):
        build_cpp_test()
    out = subprocess.run([ORDER_BIN], capture_output=True, text=True, timeout=120)
    print(out.stdout, out.stderr)
    assert out.returncode == 0 and "PASS" in out.stdout


@pytest.mark.gpu
def test_layer_prefill_and_decode_through_the_cpp_headers():
    if not os.path.exists(BIN):
        build_cpp_test()
    out = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(out.stdout, out.stderr)
    assert out.returncode == 0 and "PASS" in out.stdout


@pytest.mark.gpu
def test_layer_decode_step_with_hipblaslt_gemms():
    if not os.path.exists(LAYER_BIN):
        build_cpp_test()
    out = subprocess.run([LAYER_BIN], capture_output=True, text=True, timeout=300)
    print(out.stdout, out.stderr)
    assert out.returncode == 0 and "PASS" in out.stdout
