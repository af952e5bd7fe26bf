"""Building and loading the HIP kernels.

The sources under ``csrc/`` are compiled with hipcc for gfx950 into shared libraries under
``csrc/_build/`` (or, if the checkout cannot be written to, under the temporary folder) and loaded
with ctypes.  A library is named after a hash of its sources and flags, so a changed source is built
again and an up-to-date library is loaded as it is.  There is no fallback: if a library cannot be
built or loaded, the error says so and nothing runs.

Libraries:
  ``core``              every kernel that does not depend on the head size
  ``attention_hd<N>``   the matrix-core attention kernels, compiled for one head size
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
from concurrent.futures import ThreadPoolExecutor, wait
from pathlib import Path

from . import profile

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc",
         # packed 32-bit float instructions are kept out of generated code on purpose
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option"]

CORE_SOURCES = ["elementwise.hip", "linear.hip", "rope_store.hip", "attention_simple.hip", "sampling.hip",
                "linear_mfma.hip", "linear_ring.hip", "linear_wide.hip", "linear_wide_store_32.hip", "linear_wide_store_64.hip",
                "linear_wide_gated_32.hip", "linear_wide_gated_64.hip", "linear_wide_store_128.hip", "linear_wide_gated_128.hip", "linear_mid.hip",
                "weights_prep.hip", "linear_tile.hip"]
ATTENTION_SOURCES = ["attention_mfma.hip"]
HEADERS = ["common.h", "mfma.h", "linear_thin.h", "linear_wide.h", "attention_api.h"]


class KernelBuildError(RuntimeError):
    pass


class KernelError(RuntimeError):
    """A kernel entry point refused its arguments or a launch failed."""


_lock = threading.Lock()
_loaded: dict[str, ctypes.CDLL] = {}


def _say(msg: str) -> None:
    print(f"[palm_infra_amd] {msg}", file=sys.stderr, flush=True)


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise KernelBuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin); the HIP kernels "
                           "cannot be built and there is no other path")


def build_dir() -> Path:
    """In the checkout if it can be written to, else a folder of this user under the temporary one."""
    local = CSRC / "_build"
    try:
        local.mkdir(parents=True, exist_ok=True)
        probe = local / f".probe{os.getpid()}"
        probe.write_text("")
        probe.unlink()
        return local
    except OSError:
        d = Path(tempfile.gettempdir()) / f"palm_infra_amd_build_{os.getuid()}"
        d.mkdir(parents=True, exist_ok=True)
        return d


def _existing(names) -> list[str]:
    return [n for n in names if (CSRC / n).is_file()]


def _digest(sources, defines) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + sorted(defines)).encode())
    for name in sorted(_existing(list(sources) + HEADERS)):
        h.update(name.encode())
        h.update((CSRC / name).read_bytes())
    return h.hexdigest()[:16]


def library_path(name: str, sources, defines=()) -> Path:
    return build_dir() / f"libpalm_{name}_{_digest(sources, defines)}.so"


def _find_built(name: str, sources, defines) -> Path | None:
    """An up-to-date library, in the checkout or in the temporary folder."""
    fname = f"libpalm_{name}_{_digest(sources, defines)}.so"
    for d in (CSRC / "_build", Path(tempfile.gettempdir()) / f"palm_infra_amd_build_{os.getuid()}"):
        if (d / fname).is_file():
            return d / fname
    return None


def _compile(name: str, sources, defines, force: bool) -> Path:
    sources = _existing(sources)
    if not sources:
        raise KernelBuildError(f"library {name}: none of its sources exist under {CSRC}")
    if not force:
        found = _find_built(name, sources, defines)
        if found is not None:
            return found
    out = library_path(name, sources, defines)
    hipcc = _hipcc()
    work = out.parent / f"obj_{name}_{os.getpid()}"
    work.mkdir(parents=True, exist_ok=True)
    env = dict(os.environ)
    env.setdefault("HOME", str(out.parent))   # hipcc wants a home for its caches
    t0 = time.time()
    _say(f"compiling {name} ({len(sources)} files) for {ARCH} ...")

    def one(src: str) -> Path:
        obj = work / (src.replace(".hip", "") + ".o")
        cmd = [hipcc, *FLAGS, *[f"-D{d}" for d in defines], "-c", str(CSRC / src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise KernelBuildError(f"hipcc failed on {src}:\n{r.stderr[-4000:]}")
        _say(f"  {src} done ({time.time() - t0:.0f} s)")
        return obj

    try:
        with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
            jobs = [pool.submit(one, src) for src in sources]
            pending = set(jobs)
            while pending:                               # a line now and then, so that a long compile is seen to be alive
                done, pending = wait(pending, timeout=15)
                if pending and not done:
                    _say(f"  still compiling, {len(pending)} of {len(jobs)} files to go ({time.time() - t0:.0f} s)")
            objs = [j.result() for j in jobs]
        tmp = out.with_suffix(f".tmp{os.getpid()}")
        r = subprocess.run([hipcc, "-shared", "-fPIC", f"--offload-arch={ARCH}", "-fno-gpu-rdc",
                            *[str(o) for o in objs], "-o", str(tmp)], capture_output=True, text=True, env=env)
        if r.returncode != 0:
            raise KernelBuildError(f"linking {out.name} failed:\n{r.stderr[-4000:]}")
        os.replace(tmp, out)
    finally:
        shutil.rmtree(work, ignore_errors=True)
    # libraries of older sources are of no use any more
    for old in out.parent.glob(f"libpalm_{name}_*.so"):
        if old != out:
            try:
                old.unlink()
            except OSError:
                pass
    _say(f"built {out.name} in {time.time() - t0:.0f} s")
    return out


def _spec(name: str):
    if name == "core":
        return CORE_SOURCES, ()
    if name.startswith("attention_hd"):
        hd = int(name[len("attention_hd"):])
        return ATTENTION_SOURCES, (f"PALM_HEAD_DIM={hd}",)
    raise KeyError(name)


def build(name: str, force: bool = False) -> Path:
    sources, defines = _spec(name)
    with _lock:
        return _compile(name, sources, defines, force)


def load(name: str) -> ctypes.CDLL:
    """The library, built first if no up-to-date build exists."""
    with _lock:
        if name in _loaded:
            return _loaded[name]
        sources, defines = _spec(name)
        path = _compile(name, sources, defines, force=False)
        try:
            lib = ctypes.CDLL(str(path))
        except OSError as e:
            raise KernelBuildError(f"cannot load {path}: {e}") from None
        lib.palm_last_error.restype = ctypes.c_char_p
        _loaded[name] = lib
        return lib


def loaded_paths() -> list[str]:
    return sorted(getattr(lib, "_name", "?") for lib in _loaded.values())


def call(lib: ctypes.CDLL, fn_name: str, *args) -> None:
    fn = getattr(lib, fn_name)
    recorder = profile.active()
    rc = fn(*args) if recorder is None else recorder.around(fn_name, lambda: fn(*args))
    if rc != 0:
        raise KernelError(f"{fn_name}: {lib.palm_last_error().decode(errors='replace')}")
