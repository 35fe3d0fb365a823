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
