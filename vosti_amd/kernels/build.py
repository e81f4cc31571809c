"""Compiles the native libraries in-tree.

Three shared libraries and one program are built from ``vosti_amd/csrc``:

* ``libvosti_bf16.so`` and ``libvosti_f32.so``: the gfx950 kernels, the same
  sources compiled with ``-DVK_BF16`` or ``-DVK_F32`` (hipcc);
* ``libvosti_host.so``: the cache manager, the scheduler, the architectures' reading of config.json and
  the rules that every host of the kernels shares (g++, no GPU code);
* ``libvosti_engine.so``: the native engine (``csrc/engine`` but its command
  line; g++ against the HIP runtime, linked against ``libvosti_host.so``, so that
  a process has one cache manager, one scheduler and one registry of
  architectures; it loads the kernel library of the chosen precision from its own
  folder), with a C interface (``capi.cpp``) that ``vosti_amd.engine.NativeEngine``
  drives;
* ``vosti_engine``: the engine's command line (``main.cpp``), linked against the two.

A library is rebuilt when the hash of its sources, headers and flags differs
from the one recorded beside it.  ``ensure()``
builds only the library that is asked for, so a first call compiles what the
chosen precision needs and nothing else; it prints a line per compiled file so
that a long first build is visibly alive.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE_DIR = Path(__file__).resolve().parent.parent
CSRC = PACKAGE_DIR / "csrc"
GPU_ARCH = "gfx950"
GPU_LIBS = {"bf16": "VK_BF16", "f32": "VK_F32"}

HIPCC_FLAGS = [
    f"--offload-arch={GPU_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
HOST_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-Wall", "-Wextra", "-ffp-contract=off"]


def _writable_dir(preferred: Path, fallback_name: str) -> Path:
    try:
        preferred.mkdir(parents=True, exist_ok=True)
        probe = preferred / f".probe{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return preferred
    except OSError:
        d = Path(tempfile.gettempdir()) / f"vosti_amd_{os.getuid()}" / fallback_name
        d.mkdir(parents=True, exist_ok=True)
        return d


def lib_dir() -> Path:
    return _writable_dir(PACKAGE_DIR / "_lib", "lib")


def build_dir() -> Path:
    return _writable_dir(PACKAGE_DIR.parent / "_build", "build")


def _file_name(name: str) -> str:
    if name == "engine":
        return "vosti_engine"
    return "libvosti_engine.so" if name == "engine_lib" else f"libvosti_{name}.so"


def lib_path(name: str) -> Path:
    """Path of a built library or program: the in-tree one if present, else the fallback location."""
    in_tree = PACKAGE_DIR / "_lib" / _file_name(name)
    if in_tree.exists():
        return in_tree
    return lib_dir() / _file_name(name)


def rocm_root() -> Path:
    return Path(os.environ.get("ROCM_PATH") or "/opt/rocm")


def _sources(name: str) -> tuple[list[Path], list[Path]]:
    host = CSRC / "host"
    if name == "host":
        return sorted(host.glob("*.cpp")), sorted(host.glob("*.h"))
    if name in ("engine", "engine_lib"):
        engine = CSRC / "engine"
        headers = sorted(engine.glob("*.h")) + sorted(host.glob("*.h"))
        if name == "engine":
            return [engine / "main.cpp"], headers
        return [p for p in sorted(engine.glob("*.cpp")) if p.name != "main.cpp"], headers
    return sorted(CSRC.glob("*.hip")), sorted(CSRC.glob("*.h"))


def _flags(name: str) -> list[str]:
    if name == "host":
        return HOST_FLAGS
    if name in ("engine", "engine_lib"):
        return HOST_FLAGS + ["-I", str(rocm_root() / "include")]
    return HIPCC_FLAGS + [f"-D{GPU_LIBS[name]}"]


def source_hash(name: str) -> str:
    srcs, hdrs = _sources(name)
    h = hashlib.sha256()
    h.update(repr(_flags(name)).encode())
    for p in srcs + hdrs:
        h.update(p.name.encode())
        h.update(p.read_bytes())
    return h.hexdigest()


def is_current(name: str) -> bool:
    lib = lib_path(name)
    stamp = Path(str(lib) + ".srchash")
    return lib.exists() and stamp.exists() and stamp.read_text().strip() == source_hash(name)


def _find(tool: str, *candidates: str) -> str:
    for c in (shutil.which(tool), *candidates):
        if c and os.path.exists(c):
            return c
    raise RuntimeError(f"{tool} not found; it is needed to compile vosti_amd's native code")


def _run(cmd: list[str], what: str) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"compiling {what} failed:\n{' '.join(cmd)}\n{proc.stdout}")


def build(name: str, verbose: bool = True) -> Path:
    """Compile library ``name`` ('bf16', 'f32', 'host', 'engine_lib') or the program 'engine' unconditionally."""
    srcs, _ = _sources(name)
    if not srcs:
        raise RuntimeError(f"no sources for library {name!r} under {CSRC}")
    obj_dir = build_dir() / name
    obj_dir.mkdir(parents=True, exist_ok=True)
    if name in ("host", "engine", "engine_lib"):
        compiler = _find("g++", "/usr/bin/g++")
    else:
        compiler = _find("hipcc", "/opt/rocm/bin/hipcc")
    flags = _flags(name)
    t0 = time.time()

    def compile_one(src: Path) -> Path:
        obj = obj_dir / (src.stem + ".o")
        _run([compiler, *flags, "-I", str(src.parent), "-c", str(src), "-o", str(obj)], src.name)
        if verbose:
            print(f"[vosti_amd build] {name}: compiled {src.name} ({time.time() - t0:.0f}s)", file=sys.stderr, flush=True)
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)), 16))
    with ThreadPoolExecutor(workers) as pool:
        objs = list(pool.map(compile_one, srcs))
    out = lib_dir() / _file_name(name)
    # The engine's library is linked against the host library and the program against both; they find each
    # other in their own folder at run time ($ORIGIN), or where they were when this was linked.
    needs = {"engine_lib": ["host"], "engine": ["engine_lib", "host"]}.get(name, [])
    deps: list[str] = []
    for dep in needs:
        dep_path = ensure(dep, verbose)
        deps += ["-L", str(dep_path.parent), f"-l{dep_path.name[3:-3]}", f"-Wl,-rpath,{dep_path.parent}"]
    if needs:
        deps.append("-Wl,-rpath,$ORIGIN")
    if name == "engine":
        tmp = out.with_name(f"{out.name}.tmp{os.getpid()}")
        rocm_lib = str(rocm_root() / "lib")
        _run([compiler, "-o", str(tmp), *map(str, objs), *deps, "-L", rocm_lib, "-lamdhip64", "-ldl", f"-Wl,-rpath,{rocm_lib}"], out.name)
        os.replace(tmp, out)
        Path(str(out) + ".srchash").write_text(source_hash(name) + "\n")
        if verbose:
            print(f"[vosti_amd build] {name}: linked {out} ({time.time() - t0:.0f}s)", file=sys.stderr, flush=True)
        return out
    tmp = out.with_suffix(f".tmp{os.getpid()}.so")
    link = [compiler, "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    if name == "engine_lib":
        rocm_lib = str(rocm_root() / "lib")
        link += [*deps, "-L", rocm_lib, "-lamdhip64", "-ldl", f"-Wl,-rpath,{rocm_lib}"]
    elif name != "host":
        link.insert(1, f"--offload-arch={GPU_ARCH}")
    _run(link, out.name)
    # A kernel whose host-side stub the compiler left out shows as an undefined symbol only when the
    # library is loaded: find out now, not at the first use on a GPU.
    try:
        ctypes.CDLL(str(tmp), mode=os.RTLD_NOW)
    except OSError as e:
        tmp.unlink(missing_ok=True)
        raise RuntimeError(f"{out.name} was linked but does not load: {e}") from None
    os.replace(tmp, out)
    Path(str(out) + ".srchash").write_text(source_hash(name) + "\n")
    if verbose:
        print(f"[vosti_amd build] {name}: linked {out} ({time.time() - t0:.0f}s)", file=sys.stderr, flush=True)
    return out


def ensure(name: str, verbose: bool = True) -> Path:
    """Return the path of an up-to-date library, compiling it (and what it is linked against) if needed."""
    for dep in {"engine_lib": ["host"], "engine": ["host", "engine_lib"]}.get(name, []):
        ensure(dep, verbose)
    if is_current(name):
        return lib_path(name)
    if verbose:
        print(f"[vosti_amd build] {name}: compiling native code (first use)", file=sys.stderr, flush=True)
    return build(name, verbose)


def build_plugin(source: str | Path, out: str | Path) -> Path:
    """Compiles one C++ file that registers part kinds or architectures with the native engine into a shared
    library for ``load_plugin`` (host compiler; the engine's headers are csrc/engine and csrc/host).  What it
    uses of the engine is resolved when it is loaded into a process that holds the engine."""
    compiler = _find("g++", "/usr/bin/g++")
    out = Path(out)
    _run([compiler, *HOST_FLAGS, "-shared", "-I", str(CSRC / "engine"), "-I", str(CSRC / "host"), "-I", str(rocm_root() / "include"),
          str(source), "-o", str(out)], Path(source).name)
    return out


def build_all(verbose: bool = True) -> None:
    for name in ("host", "engine_lib", "engine", "bf16", "f32"):
        build(name, verbose)


if __name__ == "__main__":
    build_all()
