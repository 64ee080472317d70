"""The C++ host layer (ROCm memory manager, device context, bundle helpers)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SELFTEST = os.path.join(ROOT, "execution-ucx_amd", "lib", "host_selftest")
REFERENCE = "/root/reference"


def test_host_layer_without_device(pkg):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    assert os.path.exists(SELFTEST), "build the host self-test with `make -C execution-ucx_amd host`"
    out = subprocess.run([SELFTEST, "--no-device"], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "host_selftest ok" in out.stdout


def test_host_layer_compiles_against_the_reference_headers():
    """Only where the execution-ucx tree is mounted (never on the GPU box)."""
    if not os.path.exists(os.path.join(REFERENCE, "ucx_context", "ucx_context_data.hpp")):
        pytest.skip("reference tree not present")
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-DAXON_ROCM_IN_REFERENCE_TREE",
           "-I", REFERENCE, "-I", os.path.join(ROOT, "include"),
           "-I", os.path.join(ROOT, "execution-ucx_amd", "host"),
           os.path.join(ROOT, "tests", "cpp", "in_tree_compile_check.cpp")]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr


@pytest.mark.gpu
def test_host_layer_on_device(gpu):
    out = subprocess.run([SELFTEST], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "host_selftest ok" in out.stdout


@pytest.mark.gpu
def test_receive_adapters_against_the_reference_classes(gpu):
    """oracle/_ref/adapters_selftest (tests/cpp/adapters_selftest.cpp, built by oracle/Makefile
    where the execution-ucx tree is mounted, with its real ucx_context_data.hpp and
    ucx_memory_resource.cpp): PackTensors -> ToUcxBuffer -> ReceiveBufferFor -> memcpy ->
    ToUcxBufferVec and RocmBundleReceivePolicy on the device, views against the reference's own
    to_buffer_vec, payload against the oracle's pack, every pool block released once."""
    exe = os.path.join(ROOT, "oracle", "_ref", "adapters_selftest")
    assert os.path.exists(exe), "oracle/_ref/adapters_selftest is missing: run __graft_entry__.build() " \
                                "where the reference tree is mounted"
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "adapters_selftest ok" in out.stdout


@pytest.mark.gpu
def test_am_bundle_surface_against_the_reference_classes(gpu):
    """oracle/_ref/am_surface_selftest (tests/cpp/am_surface_selftest.cpp): connection_send /
    connection_recv / connection_recv_header / connection_recv_buffer of
    host/loopback_am_context.hpp with the reference's real UcxBuffer, UcxHeader, UcxAmData,
    UcxAmIovec and UcxBufferVec.  The host bundle of 64 fp32 tensors and a device bundle go
    PackTensors -> connection_send -> connection_recv_header -> ReceiveBufferFor ->
    connection_recv_buffer -> UnpackTensors with the payload compared against the oracle's
    pack; then the reference's edge rules, its iov and divide-by-two known answers, and
    cancellation."""
    exe = os.path.join(ROOT, "oracle", "_ref", "am_surface_selftest")
    assert os.path.exists(exe), "oracle/_ref/am_surface_selftest is missing: run __graft_entry__.build() " \
                                "where the reference tree is mounted"
    out = subprocess.run([exe], capture_output=True, text=True, timeout=180)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "am_surface_selftest ok" in out.stdout


def test_planner_and_header_codec_under_sanitizers(tmp_path):
    """tests/cpp/plan_fuzz.cpp against a planner compiled with AddressSanitizer and
    UBSan (host code only; the kernels' object file is linked as built): random tensor
    descriptors through every inspection call, and mutated headers through the
    decoder, which must refuse them or accept only what re-encodes to the same bytes."""
    pkgdir = os.path.join(ROOT, "execution-ucx_amd")
    objs = [os.path.join(pkgdir, "build", n) for n in
            ("axr_runtime.cpp.o", "axr_loopback.cpp.o", "axr_kernels.hip.o")]
    hipcc, clang = "/opt/rocm/bin/hipcc", "/opt/rocm/llvm/bin/clang++"
    if not all(os.path.exists(p) for p in objs + [hipcc, clang]):
        pytest.skip("needs the library's object files (make -C execution-ucx_amd) and the ROCm compilers")
    inc = ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(pkgdir, "csrc")]
    san = ["-fsanitize=address", "-fsanitize=undefined", "-fno-sanitize-recover=undefined"]
    plan_o, fuzz_o, exe = (str(tmp_path / n) for n in ("axr_plan.o", "plan_fuzz.o", "plan_fuzz"))
    host_san = [x for flag in san for x in ("-Xarch_host", flag)]
    steps = [
        [hipcc, "--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-fPIC", *host_san,
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", *inc,
         "-x", "hip", "-c", os.path.join(pkgdir, "csrc", "axr_plan.cpp"), "-o", plan_o],
        [clang, "-O1", "-g", "-std=c++17", *san, *inc, "-c",
         os.path.join(ROOT, "tests", "cpp", "plan_fuzz.cpp"), "-o", fuzz_o],
        [hipcc, "--offload-arch=gfx950", *san[:2], "-fno-gpu-sanitize", fuzz_o, plan_o, *objs,
         "-o", exe, "-lpthread"],
    ]
    for cmd in steps:
        out = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        assert out.returncode == 0, out.stderr[-3000:]
    out = subprocess.run([exe, "7", "1200"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, (out.stdout + out.stderr)[-3000:]
    assert "plan_fuzz ok" in out.stdout


def test_loopback_context_under_thread_sanitizer(tmp_path):
    """tests/cpp/loopback_stress.cpp with the loopback context and the runtime shim
    compiled with ThreadSanitizer (host code only, host memory only): four senders, one
    receiver and a thread that creates and destroys contexts, all at once."""
    pkgdir = os.path.join(ROOT, "execution-ucx_amd")
    objs = [os.path.join(pkgdir, "build", n) for n in ("axr_plan.cpp.o", "axr_kernels.hip.o")]
    hipcc, clang = "/opt/rocm/bin/hipcc", "/opt/rocm/llvm/bin/clang++"
    if not all(os.path.exists(p) for p in objs + [hipcc, clang]):
        pytest.skip("needs the library's object files (make -C execution-ucx_amd) and the ROCm compilers")
    inc = ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(pkgdir, "csrc")]
    built = []
    for name in ("axr_loopback", "axr_runtime"):
        built.append(str(tmp_path / (name + ".o")))
        cmd = [hipcc, "--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-fPIC",
               "-Xarch_host", "-fsanitize=thread", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", *inc,
               "-x", "hip", "-c", os.path.join(pkgdir, "csrc", name + ".cpp"), "-o", built[-1]]
        out = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        assert out.returncode == 0, out.stderr[-3000:]
    stress_o, exe = str(tmp_path / "loopback_stress.o"), str(tmp_path / "loopback_stress")
    for cmd in ([clang, "-O1", "-g", "-std=c++17", "-fsanitize=thread", *inc, "-c",
                 os.path.join(ROOT, "tests", "cpp", "loopback_stress.cpp"), "-o", stress_o],
                [hipcc, "--offload-arch=gfx950", "-fsanitize=thread", "-fno-gpu-sanitize", stress_o, *built, *objs,
                 "-o", exe, "-lpthread"]):
        out = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        assert out.returncode == 0, out.stderr[-3000:]
    out = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0 and "ThreadSanitizer" not in out.stderr, (out.stdout + out.stderr)[-4000:]
    assert "loopback_stress ok 2500" in out.stdout      # 4 x 400, then 3 x 300 on a shared context


def test_host_copy_helper_under_sanitizers(tmp_path):
    """tests/cpp/host_copy_check.cpp: the threaded copy of the staging paths against plain
    memcpy for random piece lists and 1 to 16 threads, with the runtime shim compiled with
    AddressSanitizer and UBSan (host code only, no GPU)."""
    pkgdir = os.path.join(ROOT, "execution-ucx_amd")
    objs = [os.path.join(pkgdir, "build", n) for n in
            ("axr_plan.cpp.o", "axr_loopback.cpp.o", "axr_kernels.hip.o")]
    hipcc, clang = "/opt/rocm/bin/hipcc", "/opt/rocm/llvm/bin/clang++"
    if not all(os.path.exists(p) for p in objs + [hipcc, clang]):
        pytest.skip("needs the library's object files (make -C execution-ucx_amd) and the ROCm compilers")
    inc = ["-I", os.path.join(ROOT, "include"), "-I", os.path.join(pkgdir, "csrc")]
    runtime_o, check_o, exe = (str(tmp_path / n) for n in ("axr_runtime.o", "host_copy_check.o", "host_copy_check"))
    steps = [
        [hipcc, "--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-fPIC",
         "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", *inc,
         "-x", "hip", "-c", os.path.join(pkgdir, "csrc", "axr_runtime.cpp"), "-o", runtime_o],
        [clang, "-O1", "-g", "-std=c++17", "-fsanitize=address,undefined", *inc, "-c",
         os.path.join(ROOT, "tests", "cpp", "host_copy_check.cpp"), "-o", check_o],
        [hipcc, "--offload-arch=gfx950", "-fsanitize=address", "-fsanitize=undefined", "-fno-gpu-sanitize",
         check_o, runtime_o, *objs, "-o", exe, "-lpthread"],
    ]
    for cmd in steps:
        out = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        assert out.returncode == 0, out.stderr[-3000:]
    out = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, (out.stdout + out.stderr)[-3000:]
    assert "host_copy_check ok" in out.stdout
