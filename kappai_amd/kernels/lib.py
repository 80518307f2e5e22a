"""Building and loading the HIP libraries.

Every ``csrc/<name>.hip`` becomes one shared library ``csrc/_build/<name>.so`` for gfx950,
compiled with hipcc the first time one of its kernels is called and loaded through
ctypes.  There is no other implementation behind these kernels: if hipcc or a library is
missing, the call fails with an error that says so.
"""
from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import stat
import subprocess
import sys
import tempfile
import threading
import time
from pathlib import Path
from typing import Dict, List, Optional

CSRC = Path(__file__).resolve().parent.parent / "csrc"
GPU_ARCH = "gfx950"
# packed fp32 instructions are switched off for all device code of this package
HIPCC_FLAGS = ["-O3", "-std=c++17", f"--offload-arch={GPU_ARCH}", "-shared", "-fPIC",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument", "-Wno-pass-failed"]
LIBRARIES = ["elementwise", "gemm", "shortconv", "attention", "sampling", "engine", "engine_api"]
# libraries made of more sources than the one of their own name
EXTRA_SOURCES = {"engine": ["engine_parts"]}


def _python_flags() -> List[str]:
    """What a library that talks to the interpreter is compiled and linked with."""
    import sysconfig
    flags = [f"-I{sysconfig.get_paths()['include']}"]
    libdir = sysconfig.get_config_var("LIBDIR")
    if libdir:
        flags.append(f"-L{libdir}")
    version = sysconfig.get_config_var("LDVERSION") or sysconfig.get_python_version()
    return flags + [f"-lpython{version}", "-ldl"]


# flags of single libraries beside HIPCC_FLAGS: name -> function that returns them
EXTRA_FLAGS = {"engine_api": _python_flags}
# libraries compiled once per value of a constant: name -> (constant, values built ahead)
VARIANT_LIBRARIES = {"attention_mfma": ("HEAD_DIM", [16, 32, 48, 64, 80, 128, 256])}


class KernelBuildError(RuntimeError):
    pass


class KernelLaunchError(RuntimeError):
    pass


_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise KernelBuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): the "
                           "HIP kernels of kappai_amd cannot be built, and there is no other path")


def _defines_flags(defines) -> List[str]:
    return [f"-D{k}={v}" for k, v in sorted((defines or {}).items())]


def _built_name(name: str, defines) -> str:
    return name + "".join(f"__{k}{v}" for k, v in sorted((defines or {}).items()))


def _sources(name: str) -> List[Path]:
    return [CSRC / f"{n}.hip" for n in [name] + EXTRA_SOURCES.get(name, [])]


def _source_hash(name: str, defines=None, sources=None) -> str:
    h = hashlib.sha256()
    for p in list(sources or _sources(name)) + sorted(CSRC.glob("*.h")):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    h.update(" ".join(HIPCC_FLAGS + _defines_flags(defines) + _extra_flags(name)).encode())
    return h.hexdigest()


def _extra_flags(name: str) -> List[str]:
    return EXTRA_FLAGS[name]() if name in EXTRA_FLAGS else []


def _tree_build_dir() -> Path:
    return CSRC / "_build"


def _private_temp_dir(create: bool):
    """A build folder under the temp folder for a source tree that cannot be written: made with
    mode 0700, and used only if it is a real folder of this user that nobody else can write
    (anything else there could hold a library that somebody else put in place).  None when it is
    not there (``create`` false) ; an error when it is there but not ours alone."""
    uid = os.getuid() if hasattr(os, "getuid") else 0
    d = Path(tempfile.gettempdir()) / f"kappai_amd_build_{uid}"
    if create:
        try:
            os.mkdir(d, 0o700)
        except FileExistsError:
            pass
    try:
        st = os.lstat(d)
    except FileNotFoundError:
        return None
    if not stat.S_ISDIR(st.st_mode) or st.st_uid != uid or st.st_mode & 0o022:
        raise KernelBuildError(
            f"{d} is not a folder of user {uid} that only they can write (owner {st.st_uid}, "
            f"mode {stat.S_IMODE(st.st_mode):o}): refusing to build or load kernels there")
    return d


def _dir_writable(d: Path) -> bool:
    try:
        d.mkdir(parents=True, exist_ok=True)
        fd, probe = tempfile.mkstemp(prefix=".probe_", dir=d)
        os.close(fd)
        os.unlink(probe)
        return True
    except OSError:
        return False


def _build_dirs(create: bool = False) -> List[Path]:
    """Where built libraries live: the source tree's own ``_build``; the private temp folder
    only when the tree cannot be written."""
    tree = _tree_build_dir()
    if _dir_writable(tree):
        return [tree]
    dirs = [tree] if tree.is_dir() else []
    tmp = _private_temp_dir(create)
    if tmp is not None:
        dirs.append(tmp)
    return dirs


def _writable_build_dir() -> Path:
    for d in _build_dirs(create=True):
        if _dir_writable(d):
            return d
    raise KernelBuildError("no writable folder for the built kernels: tried "
                           f"{_tree_build_dir()} and a private folder under "
                           f"{tempfile.gettempdir()}")


def _find_built(built: str, want_hash: str):
    for d in _build_dirs():
        so, tag = d / f"{built}.so", d / f"{built}.hash"
        if so.is_file() and tag.is_file() and tag.read_text().strip() == want_hash:
            return so
    return None


def compile_library(name: str, verbose: bool = True, defines=None, sources=None,
                    out_dir: Optional[Path] = None) -> Path:
    """Compile ``csrc/<name>.hip`` (with the other sources of its library) now, whether or not a
    built library is there.  ``sources`` / ``out_dir``: a library of somebody else's
    (``library_at``)."""
    srcs = list(sources or _sources(name))
    for src in srcs:
        if not src.is_file():
            raise KernelBuildError(f"{src}: no such kernel source")
    out_dir = out_dir or _writable_build_dir()
    built = _built_name(name, defines)
    so, tag = out_dir / f"{built}.so", out_dir / f"{built}.hash"
    tmp = out_dir / f".{built}.{os.getpid()}.{threading.get_ident()}.so"
    cmd = [_hipcc(), *HIPCC_FLAGS, *_defines_flags(defines), f"-I{CSRC}", *map(str, srcs), "-o",
           str(tmp), *_extra_flags(name)]
    what = " + ".join(src.name for src in srcs) + (
        " (" + ", ".join(f"{k}={v}" for k, v in sorted(defines.items())) + ")" if defines else "")
    if verbose:
        print(f"[kappai_amd] compiling {what} for {GPU_ARCH} ...", file=sys.stderr, flush=True)
    t0 = time.time()
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    while True:
        try:
            out, _ = proc.communicate(timeout=20)
            break
        except subprocess.TimeoutExpired:
            if verbose:
                print(f"[kappai_amd] ... still compiling {what} ({time.time() - t0:.0f} s)",
                      file=sys.stderr, flush=True)
    if proc.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise KernelBuildError(f"hipcc failed on {what}:\n{out}")
    os.replace(tmp, so)
    tag.write_text(_source_hash(name, defines, srcs))
    if verbose:
        print(f"[kappai_amd] built {so.name} in {time.time() - t0:.1f} s", file=sys.stderr,
              flush=True)
    return so


def build_all(verbose: bool = True, force: bool = True) -> None:
    """Compile every library (used by the build check); in parallel threads."""
    errors = []

    def work(n, defines):
        try:
            if force or _find_built(_built_name(n, defines), _source_hash(n, defines)) is None:
                compile_library(n, verbose, defines)
        except Exception as exc:  # noqa: BLE001 - collected and raised below
            errors.append(exc)

    jobs = [(n, None) for n in LIBRARIES]
    for n, (const, values) in VARIANT_LIBRARIES.items():
        jobs += [(n, {const: v}) for v in values]
    threads = [threading.Thread(target=work, args=job) for job in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    if errors:
        raise errors[0]


def library(name: str, **defines) -> ctypes.CDLL:
    """The loaded library ``name`` (compiled with ``defines`` as -D constants); compiled
    first if no up-to-date build exists."""
    if not defines:
        lib = _loaded.get(name)          # every kernel launch comes through here
        if lib is not None:
            return lib
    built = _built_name(name, defines)
    lib = _loaded.get(built)
    if lib is not None:
        return lib
    with _lock:
        lib = _loaded.get(built)
        if lib is not None:
            return lib
        so = _find_built(built, _source_hash(name, defines))
        if so is None:
            so = compile_library(name, defines=defines)
        try:
            lib = ctypes.CDLL(str(so))
        except OSError as exc:
            raise KernelBuildError(f"cannot load {so}: {exc}") from exc
        _loaded[built] = lib
        return lib


def library_at(source, build: bool = True, force: bool = False) -> ctypes.CDLL:
    """The library of one ``.hip`` file that lives outside this package (a part of somebody
    else's, with its kernel and the function that runs it from C): compiled like the package's
    own, with ``csrc`` on the include path, into ``_build`` beside the source, and loaded."""
    src = Path(source).resolve()
    key = f"@{src}"
    lib = _loaded.get(key)
    if lib is not None and not force:
        return lib
    with _lock:
        out_dir = src.parent / "_build"
        want = _source_hash(src.stem, None, [src])
        so, tag = out_dir / f"{src.stem}.so", out_dir / f"{src.stem}.hash"
        fresh = so.is_file() and tag.is_file() and tag.read_text().strip() == want
        if force or not fresh:
            if not build:
                raise KernelBuildError(f"{so} is missing or older than its source")
            out_dir.mkdir(parents=True, exist_ok=True)
            compile_library(src.stem, sources=[src], out_dir=out_dir)
        try:
            lib = ctypes.CDLL(str(so))
        except OSError as exc:
            raise KernelBuildError(f"cannot load {so}: {exc}") from exc
        _loaded[key] = lib
        return lib


def check(status: int, what: str) -> None:
    if status != 0:
        raise KernelLaunchError(f"{what}: HIP error {status}")
