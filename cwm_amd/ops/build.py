"""Compiles the HIP sources under `cwm_amd/csrc` for gfx950 and loads them.

Each source file becomes one shared library next to the package
(`cwm_amd/_lib/<name>[__DEF_VAL...].so`), built with plain `hipcc` and loaded with
ctypes.  A library is built when it is first asked for and is missing or older than
its sources (a digest of the sources and flags is kept beside it), so a fresh
checkout compiles exactly the kernels that the model at hand uses.  While hipcc
runs, a line is printed to stderr every few seconds.

There is no fallback: if a library cannot be built or loaded, `KernelBuildError`
is raised and nothing runs.
"""

from __future__ import annotations

import ctypes
import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from typing import Dict, Iterable, Mapping, Optional, Tuple

CSRC_DIR = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "csrc"))
_IN_TREE_LIB_DIR = os.path.normpath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "_lib"))

GPU_ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={GPU_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]

# flags of single sources (none at present)
EXTRA_FLAGS: Dict[str, Tuple[str, ...]] = {}

# source file (without .hip) -> macro sets that `build_all` compiles ahead of time
SOURCES: Dict[str, Tuple[Mapping[str, int], ...]] = {
    "rowwise": ({},),
    "rope_kv": ({},),
    "attention_simple": ({},),
    "gemm_f32": ({},),
    "gemm_f32_stream": ({},),
    "sampling": ({},),
    "gemm_bf16_stream": ({},),
    "gemm_bf16_tile": ({},),
    "ceilings": ({},),
    "attention_mfma": tuple({"HEAD_DIM": hd} for hd in (16, 32, 48, 64, 80, 96, 128, 256)),
}


class KernelBuildError(RuntimeError):
    pass


_loaded: Dict[str, ctypes.CDLL] = {}
_lock = threading.Lock()


def register_source(name: str, variants: Iterable[Mapping[str, int]] = ({},)) -> None:
    """Declare a source file of `csrc` and the macro sets `build_all` compiles."""
    SOURCES[name] = tuple(dict(v) for v in variants)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise KernelBuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


_lib_dir_cache: Optional[str] = None


def _lib_dir() -> str:
    global _lib_dir_cache
    if _lib_dir_cache is None:
        _lib_dir_cache = _choose_lib_dir()
    return _lib_dir_cache


def _choose_lib_dir() -> str:
    override = os.environ.get("CWM_AMD_LIB_DIR")
    if override:
        os.makedirs(override, exist_ok=True)
        return override
    try:
        os.makedirs(_IN_TREE_LIB_DIR, exist_ok=True)
        probe = os.path.join(_IN_TREE_LIB_DIR, f".write_probe_{os.getpid()}_{threading.get_ident()}")
        with open(probe, "w"):
            pass
        os.remove(probe)
        return _IN_TREE_LIB_DIR
    except OSError:
        fallback = os.path.join(tempfile.gettempdir(), f"cwm_amd_lib_{os.getuid()}")
        os.makedirs(fallback, exist_ok=True)
        return fallback


def _variant_tag(defines: Mapping[str, int]) -> str:
    return "".join(f"__{k}_{defines[k]}" for k in sorted(defines))  # letters, digits and underscores only: a plain file name


def _digest(name: str, defines: Mapping[str, int]) -> str:
    h = hashlib.sha256()
    for fname in sorted(os.listdir(CSRC_DIR)):
        if fname == f"{name}.hip" or fname.endswith(".h"):
            with open(os.path.join(CSRC_DIR, fname), "rb") as fh:
                h.update(fname.encode())
                h.update(fh.read())
    h.update(" ".join([*HIPCC_FLAGS, *EXTRA_FLAGS.get(name, ())]).encode())
    h.update(_variant_tag(defines).encode())
    return h.hexdigest()


def library_path(name: str, defines: Optional[Mapping[str, int]] = None) -> str:
    return os.path.join(_lib_dir(), f"{name}{_variant_tag(defines or {})}.so")


def _find_built(name: str, defines: Mapping[str, int], digest: str) -> Optional[str]:
    """A library whose digest matches, in the in-tree folder or the one in use."""
    tag = _variant_tag(defines)
    for folder in dict.fromkeys((_IN_TREE_LIB_DIR, _lib_dir())):
        path = os.path.join(folder, f"{name}{tag}.so")
        stamp = path + ".digest"
        if os.path.isfile(path) and os.path.isfile(stamp):
            try:
                with open(stamp, "r") as fh:
                    if fh.read().strip() == digest:
                        return path
            except OSError:
                pass
    return None


def build(name: str, defines: Optional[Mapping[str, int]] = None, force: bool = False, quiet: bool = False) -> str:
    """Compile `csrc/<name>.hip` (with -D macros) unless an up-to-date library exists."""
    defines = dict(defines or {})
    src = os.path.join(CSRC_DIR, f"{name}.hip")
    if not os.path.isfile(src):
        raise KernelBuildError(f"no such kernel source: {src}")
    digest = _digest(name, defines)
    if not force:
        found = _find_built(name, defines, digest)
        if found:
            return found
    out = library_path(name, defines)
    tmp = f"{out}.tmp{os.getpid()}"
    cmd = [_hipcc(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(name, ()), *[f"-D{k}={v}" for k, v in sorted(defines.items())], "-I", CSRC_DIR, src, "-o", tmp]
    label = os.path.basename(out)
    if not quiet:
        print(f"[cwm_amd] compiling {label} for {GPU_ARCH} ...", file=sys.stderr, flush=True)
    start = time.time()
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())
    proc = subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    output = []

    def _drain() -> None:
        assert proc.stdout is not None
        for line in proc.stdout:
            output.append(line)

    reader = threading.Thread(target=_drain, daemon=True)
    reader.start()
    last = start
    while proc.poll() is None:
        time.sleep(0.2)
        if not quiet and time.time() - last > 10:
            last = time.time()
            print(f"[cwm_amd] ... still compiling {label} ({int(last - start)} s)", file=sys.stderr, flush=True)
    reader.join()
    text = "".join(line for line in output if "packed-fp32-ops" not in line)
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise KernelBuildError(f"hipcc failed for {name}.hip (exit {proc.returncode}):\n{text}")
    os.replace(tmp, out)
    with open(out + ".digest", "w") as fh:
        fh.write(digest)
    if not quiet:
        print(f"[cwm_amd] built {label} in {time.time() - start:.1f} s", file=sys.stderr, flush=True)
    return out


def load(name: str, defines: Optional[Mapping[str, int]] = None) -> ctypes.CDLL:
    """The library of `csrc/<name>.hip`, built first if need be."""
    if defines is None:
        lib = _loaded.get(name)  # the common case, on every launch: no lock, no tag
        if lib is not None:
            return lib
    key = name + _variant_tag(defines or {})
    with _lock:
        lib = _loaded.get(key)
        if lib is None:
            path = build(name, defines)
            try:
                lib = ctypes.CDLL(path)
            except OSError as exc:
                raise KernelBuildError(f"cannot load {path}: {exc}") from None
            lib.cwm_error_message.restype = ctypes.c_char_p
            _loaded[key] = lib
        return lib


def build_all(force: bool = True, jobs: int = 4) -> None:
    """Compile every registered source and variant (what `__graft_entry__.build` calls)."""
    from concurrent.futures import ThreadPoolExecutor

    work = [(name, dict(v)) for name, variants in SOURCES.items() for v in variants]
    _lib_dir()
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        futures = [pool.submit(build, name, v, force) for name, v in work]
        for fut in futures:
            fut.result()


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
