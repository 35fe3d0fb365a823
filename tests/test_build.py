"""The build of the HIP libraries: what it reads from the compiler's report, and that no kernel of
the libraries in the tree spills registers to memory (such a kernel passes every numerical test and
runs ten times slower)."""

from __future__ import annotations

import json
import subprocess

from mini_llm_runtime_amd.kernels import build


def test_spilled_registers_are_read_from_the_compiler_report(monkeypatch):
    report = "\n".join([
        "a.hip:10:1: remark: Function Name: _Zkernel_one [-Rpass-analysis=kernel-resource-usage]",
        "   10 | __global__ void kernel_one(int n) {",
        "      | ^",
        "a.hip:10:1: remark:     VGPRs: 128 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:10:1: remark:     VGPRs Spill: 301 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:90:1: remark: Function Name: _Zkernel_two [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:90:1: remark:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:90:1: remark:     VGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]",
        "a.hip:5:3: warning: something else",
    ])
    logged = []
    monkeypatch.setattr(build, "log", logged.append)
    monkeypatch.setattr(
        subprocess, "run", lambda *a, **k: subprocess.CompletedProcess(a, 0, stdout=report, stderr=None)
    )
    assert build._run(["hipcc"], "compiling a.hip") == {"_Zkernel_one": 301, "_Zkernel_two": 0}
    assert any("warning: something else" in line and "remark" not in line for line in logged)
    assert not any("__global__" in line or "| ^" in line for line in logged)
    assert any("_Zkernel_one spills 301" in line for line in logged)


def test_no_kernel_of_the_built_libraries_spills():
    """Read from what the last build of each library wrote beside it (a library built before the build
    kept count has nothing to say)."""
    folder = build.build_dir()
    for module in build.all_modules():
        stamp = build.library_path(module, folder).with_suffix(".json")
        if not stamp.exists():
            continue
        data = json.loads(stamp.read_text())
        if "kernels" not in data:
            continue
        assert data["kernels"] > 0, f"{stamp.name}: the compiler reported no kernel"
        assert data["spilling_kernels"] == {}, f"{stamp.name}: kernels that spill registers: {data['spilling_kernels']}"


def test_kernel_choice_for_the_benchmark_shapes():
    """The choice of a product kernel is host code and answers without a GPU: the shapes of the three
    benchmark models get the tilings that the measurements behind the estimates chose.  (The numbers are
    those of `mlr_gemm_bf16`'s `kernel` argument.)"""
    import ctypes

    path = build.library_path(build.CORE, build.build_dir())
    if not path.exists() or not build.is_current(build.CORE):
        import pytest

        pytest.skip("the core library is not built from the present sources")
    lib = ctypes.CDLL(str(path))
    for fn in (lib.mlr_gemm_bf16_kernel, lib.mlr_gemm_bf16_slices):
        fn.argtypes, fn.restype = [ctypes.c_int] * 4, ctypes.c_int
    chosen = lambda m, n, k, most: lib.mlr_gemm_bf16_kernel(m, n, k, lib.mlr_gemm_bf16_slices(m, n, k, most))
    # up to 64 tokens: the row-splitting kernel for the 0.5B products, tiles of 64 tokens whose width
    # makes one round over the compute units for the gate-up of the 7B (160 features) and 32B (224) shapes
    assert chosen(8, 9728, 896, 1) == 16 and chosen(8, 896, 4864, 8) == 16
    assert chosen(64, 37888, 3584, 1) == 65 and chosen(8, 37888, 3584, 1) == 65
    assert chosen(64, 55296, 5120, 1) == 67 and chosen(8, 55296, 5120, 1) == 67
    assert chosen(64, 9728, 896, 1) == 62 and chosen(8, 151936, 896, 1) == 14
    # a prompt of 2,048 tokens: tiles of 256 tokens, 320 features wide for the 0.5B gate-up (one round),
    # 160 for the 7B query/key/value width, square for the large products
    assert chosen(2048, 9728, 896, 1) == 48
    assert chosen(2048, 4608, 3584, 1) == 47
    assert chosen(2048, 37888, 3584, 1) == 45 and chosen(2048, 55296, 5120, 1) == 45
    assert lib.mlr_gemm_bf16_slices(2048, 3584, 18944, 4) == 2 and chosen(2048, 3584, 18944, 4) == 45
    # in between, tiles of 64 tokens for a large matrix cut along k, the staged ones for a small one
    assert chosen(128, 3584, 18944, 4) == 64 and chosen(192, 2048, 1536, 4) == 11
    # every answer is a kernel that exists, whatever the shape
    known = {16, 14, 11, 22, 23, 44, 45, 46, 47, 48, 62, 63, 64, 65, 66, 67, 68}
    for m in (1, 5, 16, 17, 33, 64, 65, 100, 257, 1000, 5000):
        for n, k in ((8, 8), (100, 40), (517, 96), (896, 896), (4608, 3584), (151936, 896), (59136, 8192)):
            for most in (1, 4, 16):
                assert chosen(m, n, k, most) in known
