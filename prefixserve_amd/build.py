"""Compiles and loads the two native libraries of the package.

* ``_core``: the host-side cache bookkeeping (C++17 + pybind11), built with g++.
* ``libpsamd_kernels.so``: every device kernel (HIP, gfx950 only), built with hipcc and
  called through ``ctypes`` with raw pointers and a stream handle.

Both are built in-tree under ``prefixserve_amd/_lib`` (or, when the package folder is
not writable, under a per-user temporary folder). ``ensure_*`` loads what is built and
compiles only when nothing is; ``build_all(force=True)`` always compiles. A build prints
a line per file so that a first call in a fresh checkout shows progress.
"""

from __future__ import annotations

import ctypes
import importlib.machinery
import importlib.util
import os
import shutil
import subprocess
import sys
import sysconfig
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path
from types import ModuleType

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
GPU_ARCH = "gfx950"

CORE_SOURCES = ["core/page_pool.cpp", "core/prefix_tree.cpp", "core/step_pack.cpp", "core/bindings.cpp"]
KERNEL_LIB = "libpsamd_kernels.so"

HIPCC_FLAGS = [
    f"--offload-arch={GPU_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # Packed fp32 instructions are kept out of every kernel of this library.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
    # Matrix-core results stay in ordinary vector registers: the softmax and epilogues read
    # them at once, and copies to and from the accumulator file were a fifth of all vector
    # instructions in the attention kernels.
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
]


class BuildError(RuntimeError):
    pass


def _say(msg: str) -> None:
    print(f"[prefixserve_amd build] {msg}", file=sys.stderr, flush=True)


def _writable(d: Path) -> bool:
    try:
        d.mkdir(parents=True, exist_ok=True)
        probe = d / f".probe-{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return True
    except OSError:
        return False


def lib_dir() -> Path:
    """Where built libraries live: in-tree if possible."""
    override = os.environ.get("PREFIXSERVE_AMD_LIB_DIR")
    if override:
        d = Path(override)
        d.mkdir(parents=True, exist_ok=True)
        return d
    d = PKG_DIR / "_lib"
    if _writable(d):
        return d
    d = Path(tempfile.gettempdir()) / f"prefixserve_amd-lib-{os.getuid()}"
    d.mkdir(parents=True, exist_ok=True)
    return d


def _existing(name: str) -> Path | None:
    """A built library: in the folder ``PREFIXSERVE_AMD_LIB_DIR`` names if it is set, else
    in-tree, else in the per-user fallback folder."""
    override = os.environ.get("PREFIXSERVE_AMD_LIB_DIR")
    if override:
        p = Path(override) / name
        return p if p.exists() else None
    for d in (PKG_DIR / "_lib", Path(tempfile.gettempdir()) / f"prefixserve_amd-lib-{os.getuid()}"):
        p = d / name
        if p.exists():
            return p
    return None


def _run(cmd: list[str], what: str) -> None:
    t0 = time.time()
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise BuildError(f"{what} failed ({proc.returncode}):\n{' '.join(cmd)}\n{proc.stdout}\n{proc.stderr}")
    _say(f"{what}: {time.time() - t0:.1f}s")


def _find(tool: str, fallbacks: list[str]) -> str:
    found = shutil.which(tool)
    if found:
        return found
    for f in fallbacks:
        if Path(f).exists():
            return f
    raise BuildError(f"{tool} not found (looked on PATH and in {fallbacks})")


def core_module_name() -> str:
    return "_core" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so")


# Every warning is an error, in the module and in the check program alike.
CORE_WARNINGS = ["-Wall", "-Wextra", "-Wshadow", "-Wconversion", "-Wsign-conversion", "-Werror"]
SANITIZE_FLAGS = ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer", "-O1", "-g"]


def build_core() -> Path:
    import pybind11

    gxx = _find("g++", ["/usr/bin/g++"])
    out = lib_dir() / core_module_name()
    tmp = out.with_suffix(out.suffix + f".tmp{os.getpid()}")
    cmd = [
        gxx, "-O2", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden", *CORE_WARNINGS,
        # Python's and pybind11's headers as system headers: their own warnings are not this package's errors.
        "-isystem", sysconfig.get_paths()["include"], "-isystem", pybind11.get_include(), f"-I{CSRC / 'core'}",
        *[str(CSRC / s) for s in CORE_SOURCES], "-o", str(tmp),
    ]
    _run(cmd, "host cache core (g++)")
    os.replace(tmp, out)
    return out


def build_core_program(main_source: Path, out: Path, sanitize: bool = False, what: str = "core check program") -> Path:
    """A standalone program from ``main_source`` and the core's sources without the Python
    bindings, for checks of the core that run without an interpreter: with ``sanitize`` the
    address and undefined-behaviour sanitizers are compiled in (host code only; a sanitized
    Python module would need the sanitizer's runtime loaded before the interpreter)."""
    gxx = _find("g++", ["/usr/bin/g++"])
    sources = [str(CSRC / s) for s in CORE_SOURCES if not s.endswith("bindings.cpp")]
    cmd = [gxx, "-std=c++17", *CORE_WARNINGS, *(SANITIZE_FLAGS if sanitize else ["-O2"]), f"-I{CSRC / 'core'}",
           str(main_source), *sources, "-o", str(out)]
    _run(cmd, f"{what}{' (sanitizers)' if sanitize else ''}")
    return out


def kernel_sources() -> list[Path]:
    return sorted((CSRC / "kernels").glob("*.hip"))


def build_kernels() -> Path:
    hipcc = _find("hipcc", ["/opt/rocm/bin/hipcc"])
    out = lib_dir() / KERNEL_LIB
    obj_dir = lib_dir() / "obj"
    obj_dir.mkdir(parents=True, exist_ok=True)
    srcs = kernel_sources()
    if not srcs:
        raise BuildError(f"no kernel sources under {CSRC / 'kernels'}")
    _say(f"compiling {len(srcs)} HIP sources for {GPU_ARCH} ...")

    extra = os.environ.get("PREFIXSERVE_AMD_HIPCC_FLAGS", "").split()

    def one(src: Path) -> Path:
        obj = obj_dir / (src.stem + ".o")
        _run([hipcc, *HIPCC_FLAGS, *extra, f"-I{CSRC / 'kernels'}", "-c", str(src), "-o", str(obj)],
             f"hipcc {src.name}")
        return obj

    workers = max(1, min(len(srcs), (os.cpu_count() or 2), 8))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        objs = list(pool.map(one, srcs))
    tmp = out.with_suffix(f".tmp{os.getpid()}")
    _run([hipcc, f"--offload-arch={GPU_ARCH}", "-shared", "-fPIC", *[str(o) for o in objs], "-o", str(tmp)],
         "link " + KERNEL_LIB)
    os.replace(tmp, out)
    shutil.rmtree(obj_dir, ignore_errors=True)
    return out


def build_extension(sources: list[Path], out: Path) -> Path:
    """A shared library of device kernels from HIP sources of one's own, compiled with the flags
    the package's kernels are compiled with (``csrc/kernels`` is on the include path, so
    ``common.h`` may be used): what a part that brings a kernel of its own builds and then hands
    to ``HipOps.load_extension``. Its entry points are ``extern "C"``, take the stream first
    and return 0 or an error code."""
    hipcc = _find("hipcc", ["/opt/rocm/bin/hipcc"])
    out = Path(out)
    out.parent.mkdir(parents=True, exist_ok=True)
    tmp = out.with_suffix(f".tmp{os.getpid()}")
    _run([hipcc, *HIPCC_FLAGS, f"-I{CSRC / 'kernels'}", "-shared", *[str(s) for s in sources], "-o", str(tmp)],
         f"hipcc {' '.join(Path(s).name for s in sources)} -> {out.name}")
    os.replace(tmp, out)
    return out


def build_all(force: bool = True) -> None:
    if force or _existing(core_module_name()) is None:
        build_core()
    if force or _existing(KERNEL_LIB) is None:
        build_kernels()


_core_mod: ModuleType | None = None
_kernel_lib: ctypes.CDLL | None = None


def ensure_core() -> ModuleType:
    """The ``_core`` extension module, compiled first if no built file exists."""
    global _core_mod
    if _core_mod is not None:
        return _core_mod
    path = _existing(core_module_name())
    if path is None:
        _say("host cache core is not built yet; compiling it now")
        path = build_core()
    name = "prefixserve_amd._core"
    loader = importlib.machinery.ExtensionFileLoader(name, str(path))
    spec = importlib.util.spec_from_file_location(name, str(path), loader=loader)
    assert spec is not None
    mod = importlib.util.module_from_spec(spec)
    loader.exec_module(mod)
    sys.modules[name] = mod
    _core_mod = mod
    return mod


def ensure_kernels() -> ctypes.CDLL:
    """The kernel library, compiled first if no built file exists. Raises if it cannot be
    built or loaded: there is no other implementation to fall back to."""
    global _kernel_lib
    if _kernel_lib is not None:
        return _kernel_lib
    path = _existing(KERNEL_LIB)
    if path is None:
        _say("device kernels are not built yet; compiling them now (about a minute)")
        path = build_kernels()
    try:
        _kernel_lib = ctypes.CDLL(str(path))
    except OSError as e:
        raise BuildError(f"cannot load {path}: {e}") from e
    return _kernel_lib
