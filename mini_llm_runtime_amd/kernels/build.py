"""Compiling the HIP sources for gfx950 with hipcc into shared libraries.

A *module* is one shared library made from some sources and preprocessor
definitions.  `core` holds every kernel that does not depend on a model's head
size; `attention_d<D>` holds the MFMA attention kernels for one head size and is
only built when a model with that head size is loaded.  Libraries are kept in
`csrc/_build/` beside the sources (or, when that folder cannot be written, in a
per-user folder under the system's temporary directory) with a stamp of the
sources' hash, and are rebuilt when the stamp does not match.  While compiling, a
line is printed for every file and every few seconds.
"""

from __future__ import annotations

import hashlib
import json
import os
import re
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from dataclasses import dataclass, field
from pathlib import Path
from typing import Optional, Sequence

CSRC = Path(__file__).resolve().parents[1] / "csrc"
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # packed float32 instructions are kept out of all device code
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # matrix-core accumulators in ordinary vector registers: every kernel here fits in 256 of
    # them, and the separate accumulator file costs a copy per element whenever the vector
    # ALU touches an accumulator (softmax rescaling, epilogues)
    "-mllvm",
    "-amdgpu-mfma-vgpr-form",
]
@dataclass(frozen=True)
class Module:
    name: str
    sources: tuple[str, ...]
    defines: tuple[str, ...] = field(default_factory=tuple)
    headers: tuple[str, ...] = ("api.h", "common.h", "mfma.h", "gemm_epilogue.h")  # what the sources include: part of the stamp


CORE = Module(
    "core",
    (
        "elementwise.hip",
        "gemm_simple.hip",
        "gemm_mfma.hip",
        "gemm_fused.hip",
        "gemm_stream.hip",
        "attention_simple.hip",
        "sampling.hip",
    ),
)


DEFAULT_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 128, 256)


def attention_module(head_dim: int) -> Module:
    """The MFMA attention kernels for one head size (a multiple of 16 within 16..256)."""
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise ValueError("the MFMA attention kernels take head sizes in steps of 16 up to 256")
    return Module(
        f"attention_d{head_dim}", ("attention_mfma.hip",), (f"MLR_HEAD_DIM={head_dim}",), ("common.h", "mfma.h")
    )


def all_modules() -> list[Module]:
    """Every module a default build compiles: the core library and the attention
    kernels of the usual head sizes (other sizes are compiled when a model needs them)."""
    return [CORE] + [attention_module(d) for d in DEFAULT_HEAD_DIMS]


def log(message: str) -> None:
    print(f"[mini_llm_runtime_amd] {message}", file=sys.stderr, flush=True)


def find_hipcc() -> str:
    for candidate in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if candidate and Path(candidate).exists():
            return candidate
    raise RuntimeError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); the HIP kernels cannot be built")


def _writable(folder: Path) -> bool:
    try:
        folder.mkdir(parents=True, exist_ok=True)
        probe = folder / f".probe{os.getpid()}"
        probe.write_text("x")
        probe.unlink()
        return True
    except OSError:
        return False


def build_dir() -> Path:
    override = os.environ.get("MLR_BUILD_DIR")
    if override:
        folder = Path(override)
        folder.mkdir(parents=True, exist_ok=True)
        return folder
    in_tree = CSRC / "_build"
    if _writable(in_tree):
        return in_tree
    fallback = Path(tempfile.gettempdir()) / f"mini_llm_runtime_amd_build_{os.getuid()}"
    fallback.mkdir(parents=True, exist_ok=True)
    return fallback


def _source_hash(module: Module) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS).encode())
    h.update(" ".join(module.defines).encode())
    for name in list(module.sources) + list(module.headers):
        path = CSRC / name
        if path.exists():
            h.update(name.encode())
            h.update(path.read_bytes())
    return h.hexdigest()


def library_path(module: Module, folder: Optional[Path] = None) -> Path:
    return (folder or build_dir()) / f"libmlr_{module.name}.so"


def is_current(module: Module, folder: Optional[Path] = None) -> bool:
    lib = library_path(module, folder)
    stamp = lib.with_suffix(".json")
    if not lib.exists() or not stamp.exists():
        return False
    try:
        return json.loads(stamp.read_text()).get("hash") == _source_hash(module)
    except (OSError, ValueError):
        return False


# The compiler reports every kernel's registers: a kernel that spills them to memory still
# computes the right thing, ten times slower, so the build counts the spills and says so.
RESOURCE_REMARKS = "-Rpass-analysis=kernel-resource-usage"
_KERNEL_NAME = re.compile(r"remark: Function Name: (\S+)")
_KERNEL_SPILL = re.compile(r"remark:\s+VGPRs Spill: (\d+)")
_SOURCE_CONTEXT = re.compile(r"^\s*\d*\s*\|")


def _run(cmd: Sequence[str], what: str) -> dict[str, int]:
    """Runs a compiler command; returns {kernel: spilled vector registers} for the kernels it reported."""
    env = dict(os.environ)
    # hipcc and clang want a writable HOME/TMPDIR for their temporary files
    if not env.get("HOME") or not os.access(env.get("HOME", ""), os.W_OK):
        env["HOME"] = tempfile.gettempdir()
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if proc.returncode != 0:
        raise RuntimeError(f"{what} failed (exit {proc.returncode}):\n$ {' '.join(cmd)}\n{proc.stdout}")
    noise = "is not a recognized feature for this target"
    spills: dict[str, int] = {}
    kernel, rest, in_report = None, [], False
    for line in proc.stdout.splitlines():
        named = _KERNEL_NAME.search(line)
        if named:
            kernel = named.group(1)
            spills.setdefault(kernel, 0)
        spilled = _KERNEL_SPILL.search(line)
        if spilled and kernel is not None:
            spills[kernel] = max(spills[kernel], int(spilled.group(1)))
        if "[-Rpass-analysis=kernel-resource-usage]" in line:
            in_report = True  # the source line and the caret under it belong to the report
            continue
        if in_report and _SOURCE_CONTEXT.match(line):
            continue
        in_report = False
        if line.strip() and noise not in line:
            rest.append(line)
    if rest:
        log(f"{what}: " + "\n".join(rest))
    for name, count in spills.items():
        if count:
            log(f"{what}: kernel {name} spills {count} vector registers to memory")
    return spills


def build_module(module: Module, *, force: bool = False, jobs: int = 8) -> Path:
    """Compile and link one module; returns the library's path."""
    folder = build_dir()
    lib = library_path(module, folder)
    if not force and is_current(module, folder):
        return lib
    hipcc = find_hipcc()
    started = time.time()
    log(f"building {lib.name} for {ARCH} ({len(module.sources)} files) in {folder}")
    objects = [folder / f"{module.name}_{Path(s).stem}.o" for s in module.sources]
    done = threading.Event()

    def heartbeat() -> None:
        while not done.wait(10.0):
            log(f"  still compiling {lib.name} ... {time.time() - started:.0f} s")

    beat = threading.Thread(target=heartbeat, daemon=True)
    beat.start()
    try:
        defines = [f"-D{d}" for d in module.defines]

        def compile_one(pair: tuple[str, Path]) -> dict[str, int]:
            src, obj = pair
            log(f"  hipcc {src}")
            return _run(
                [hipcc, *FLAGS, RESOURCE_REMARKS, *defines, "-I", str(CSRC), "-c", str(CSRC / src), "-o", str(obj)],
                f"compiling {src}",
            )

        with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(objects)))) as pool:
            reports = list(pool.map(compile_one, zip(module.sources, objects)))
        kernels = {name: count for report in reports for name, count in report.items()}
        tmp = lib.with_suffix(f".tmp{os.getpid()}.so")
        _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objects)], f"linking {lib.name}")
        os.replace(tmp, lib)
        lib.with_suffix(".json").write_text(json.dumps({
            "hash": _source_hash(module), "arch": ARCH, "kernels": len(kernels),
            "spilling_kernels": {name: count for name, count in kernels.items() if count},
        }))
    finally:
        done.set()
    log(f"built {lib.name} in {time.time() - started:.1f} s")
    return lib


def ensure_module(module: Module) -> Path:
    """The module's library, building it first if it is missing or stale."""
    if is_current(module):
        return library_path(module)
    return build_module(module)
