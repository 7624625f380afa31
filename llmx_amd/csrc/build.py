"""Builds the gfx950 kernel library with hipcc and finds it again.

The library is a plain shared object with a C ABI (no Python headers), built in
the tree beside its sources so that it travels with the checkout.  `load_path`
returns what is built when its stamp (a hash of sources and flags) is the
current one and compiles otherwise; `build` always compiles.  Where the source tree cannot be written the library goes to a
per-user folder under the system's temporary directory.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
LIB_NAME = "libllmx_kernels.so"
ARCH = "gfx950"
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    # packed fp32 arithmetic is kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unused-command-line-argument",
]


class BuildError(RuntimeError):
    pass


def sources() -> list[Path]:
    return sorted(HERE.glob("*.hip"))


def _stamp() -> str:
    h = hashlib.sha256()
    for p in sorted(list(HERE.glob("*.hip")) + list(HERE.glob("*.h"))):
        h.update(p.name.encode())
        h.update(p.read_bytes())
    h.update(" ".join(FLAGS).encode())
    return h.hexdigest()


def _say(text: str) -> None:
    print(f"llmx_amd: {text}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); the kernel library cannot be built")


def _writable(d: Path) -> bool:
    try:
        d.mkdir(parents=True, exist_ok=True)
        probe = d / f".probe{os.getpid()}"
        probe.write_bytes(b"")
        probe.unlink()
        return True
    except OSError:
        return False


def _fallback_dir() -> Path:
    return Path(tempfile.gettempdir()) / f"llmx_amd_build_{os.getuid()}_{_stamp()[:16]}"


def lib_candidates() -> list[Path]:
    return [HERE / LIB_NAME, _fallback_dir() / LIB_NAME]


def build(verbose: bool = True) -> Path:
    """Compile every kernel source for gfx950 and link the library; returns its path."""
    hipcc = _hipcc()
    out_dir = HERE if _writable(HERE / "_build") else _fallback_dir()
    obj_dir = out_dir / "_build"
    obj_dir.mkdir(parents=True, exist_ok=True)
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # hipcc wants a HOME for its caches
    srcs = sources()
    if not srcs:
        raise BuildError(f"no kernel sources under {HERE}")
    t0 = time.time()

    def compile_one(src: Path) -> Path:
        obj = obj_dir / (src.stem + ".o")
        cmd = [hipcc, *FLAGS, "-c", str(src), "-o", str(obj)]
        if verbose:
            _say(f"compiling {src.name} for {ARCH} ...")
        r = subprocess.run(cmd, capture_output=True, text=True, env=env, cwd=str(HERE))
        if r.returncode != 0:
            raise BuildError(f"hipcc failed on {src.name}:\n{r.stderr[-4000:]}")
        return obj

    workers = max(1, min(len(srcs), int(os.environ.get("MAX_JOBS", "8")), 16))
    with ThreadPoolExecutor(workers) as pool:
        objs = list(pool.map(compile_one, srcs))
    lib = out_dir / LIB_NAME
    tmp = out_dir / (LIB_NAME + f".tmp{os.getpid()}")
    cmd = [hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    if verbose:
        _say(f"linking {lib.name} ...")
    r = subprocess.run(cmd, capture_output=True, text=True, env=env)
    if r.returncode != 0:
        raise BuildError(f"hipcc failed to link {LIB_NAME}:\n{r.stderr[-4000:]}")
    os.replace(tmp, lib)
    (out_dir / (LIB_NAME + ".stamp")).write_text(_stamp())
    if verbose:
        _say(f"built {lib} in {time.time() - t0:.1f} s")
    return lib


def load_path(verbose: bool = True) -> Path:
    """The built library; compiled now if none is there or if what is there was built from other sources or flags."""
    want = _stamp()
    for lib in lib_candidates():
        if lib.exists():
            stamp = lib.with_name(LIB_NAME + ".stamp")
            if stamp.exists() and stamp.read_text() == want:
                return lib
            if verbose:
                _say(f"{lib} was not built from the current sources: building again")
            break
    return build(verbose=verbose)


if __name__ == "__main__":
    print(build())
