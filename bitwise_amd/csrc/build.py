"""Building and loading the gfx950 kernel library.

The sources are compiled with hipcc straight to one shared library with a C interface
(no code translation step, no torch C++ API).  The library lives beside the sources; if
that folder cannot be written, a per-user folder under the temporary directory is used.
A stamp file holds a hash of the sources, so a stale library is rebuilt and a current one
is loaded as it is.
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
from typing import List, Optional

HERE = Path(__file__).resolve().parent
SOURCES = ["elementwise.hip", "gemm_f32.hip", "gemm_bf16.hip", "attention_f32.hip", "attention_bf16.hip",
           "fused_decode.hip", "sampling.hip"]
HEADERS = ["common.h", "api.h", "layout.h", "gemm_bf16_skinny.h", "gemm_bf16_tiles.h", "gemm_bf16_rows.h",
           "gemm_bf16_phases.h"]
LIB_NAME = "libbitwise_hip.so"
# -ffp-contract=off: a multiply-add is fused only where the source says fmaf.  Packed 32-bit
# float instructions are switched off for the device pass.
FLAGS = ["--offload-arch=gfx950", "-O3", "-ffp-contract=off", "-fPIC", "-std=c++17",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

_lib: Optional[ctypes.CDLL] = None


class KernelLibraryError(RuntimeError):
    pass


def source_stamp() -> str:
    h = hashlib.sha256()
    for name in SOURCES + HEADERS:
        h.update(name.encode())
        h.update((HERE / name).read_bytes())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()


def _candidate_dirs() -> List[Path]:
    uid = os.getuid() if hasattr(os, "getuid") else 0
    return [HERE, Path(tempfile.gettempdir()) / f"bitwise_amd_build_{uid}"]


def _find_current() -> Optional[Path]:
    stamp = source_stamp()
    for d in _candidate_dirs():
        lib, st = d / LIB_NAME, d / (LIB_NAME + ".stamp")
        if lib.exists() and st.exists() and st.read_text().strip() == stamp:
            return lib
    return None


def _hipcc() -> Optional[str]:
    return shutil.which("hipcc") or (str(Path("/opt/rocm/bin/hipcc")) if Path("/opt/rocm/bin/hipcc").exists() else None)


def _say(msg: str) -> None:
    print(f"[bitwise_amd build] {msg}", file=sys.stderr, flush=True)


def build(force: bool = False, verbose: bool = True) -> Path:
    """Compile every kernel source for gfx950 and link the library; returns its path."""
    if not force:
        cur = _find_current()
        if cur is not None:
            return cur
    hipcc = _hipcc()
    if hipcc is None:
        raise KernelLibraryError("the kernel library is not built and hipcc was not found to build it")
    out_dir = None
    for d in _candidate_dirs():
        try:
            d.mkdir(parents=True, exist_ok=True)
            probe = d / f".probe_{os.getpid()}"
            probe.write_text("x")
            probe.unlink()
            out_dir = d
            break
        except OSError:
            continue
    if out_dir is None:
        raise KernelLibraryError("no writable folder for the kernel library")
    obj_dir = out_dir / "_build"
    obj_dir.mkdir(exist_ok=True)
    env = dict(os.environ)
    env.setdefault("HOME", str(out_dir))        # hipcc wants some HOME; an empty one will do
    t0 = time.time()
    if verbose:
        _say(f"compiling {len(SOURCES)} kernel sources for gfx950 into {out_dir} (about a minute)")

    def compile_one(name: str) -> str:
        obj = obj_dir / (Path(name).stem + ".o")
        cmd = [hipcc, *FLAGS, "-c", str(HERE / name), "-o", str(obj)]
        p = subprocess.run(cmd, capture_output=True, text=True, env=env, cwd=str(HERE))
        if p.returncode != 0:
            raise KernelLibraryError(f"hipcc failed on {name}:\n{p.stderr[-4000:]}")
        if verbose:
            _say(f"compiled {name} ({time.time() - t0:.0f} s)")
        return str(obj)

    with ThreadPoolExecutor(max_workers=min(6, len(SOURCES))) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    tmp_lib = out_dir / (LIB_NAME + f".tmp{os.getpid()}")
    # -z defs: a kernel template that the host pass failed to instantiate (it can do so without a
    # word) leaves an undefined symbol; better the link fails here than the load on the GPU box
    p = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-z,defs", "-o", str(tmp_lib), *objs],
                       capture_output=True, text=True, env=env)
    if p.returncode != 0:
        raise KernelLibraryError(f"linking the kernel library failed:\n{p.stderr[-4000:]}")
    os.replace(tmp_lib, out_dir / LIB_NAME)
    (out_dir / (LIB_NAME + ".stamp")).write_text(source_stamp())
    if verbose:
        _say(f"built {out_dir / LIB_NAME} in {time.time() - t0:.0f} s")
    return out_dir / LIB_NAME


def load() -> ctypes.CDLL:
    """The kernel library, built first if there is no current one.  Fails loudly otherwise."""
    global _lib
    if _lib is None:
        path = _find_current() or build()
        try:
            _lib = ctypes.CDLL(str(path))
        except OSError as e:
            raise KernelLibraryError(f"cannot load {path}: {e}") from None
    return _lib


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
