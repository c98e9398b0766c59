"""Compiles the HIP sources under ``csrc/`` for gfx950 into shared libraries.

There is one core library (every kernel whose code does not depend on the model's sizes) and
*variant* libraries: a source compiled with ``-D`` macros for one concrete size (for instance
one head size of the MFMA attention kernels).  A variant is built the first time a model needs
it, so a first call compiles what that model needs and nothing else.

Libraries live in ``csrc/_build/`` inside the package when that is writable, else in a per-user
folder under the system's temporary directory.  A stamp file beside each library holds a hash of
its sources and flags; a library whose stamp does not match is rebuilt.
"""

from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path
from typing import Dict, Iterable, List, Optional, Sequence

CSRC = Path(__file__).resolve().parent.parent / "csrc"
ARCH = "gfx950"

CORE_NAME = "torchllms_amd_core"
CORE_SOURCES = [
    "elementwise.hip",
    "attention_generic.hip",
    "gemm_f32.hip",
    "gemm_stream.hip",
    "gemm_wide.hip",
    "sampling.hip",
]
HEADERS = ["common.h", "qkv_epilogue.h", "no_alloc.h"]

HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    # packed 32-bit float instructions are kept out of all device code
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    # gemm_wide.hip sets m0 in its own assembly and says so in the clobber list; the compiler warns
    # about that once per instantiation (hundreds of lines at a user's first call)
    "-Wno-inline-asm",
]


class BuildError(RuntimeError):
    pass


def _log(msg: str) -> None:
    print(f"[torchllms_amd build] {msg}", file=sys.stderr, flush=True)


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


def build_dir() -> Path:
    """The folder libraries are built into: in-tree when writable, else a per-user temp folder."""
    override = os.environ.get("TORCHLLMS_AMD_BUILD_DIR")
    candidates = [Path(override)] if override else []
    candidates.append(CSRC / "_build")
    candidates.append(Path(tempfile.gettempdir()) / f"torchllms_amd_build_{os.getuid()}")
    for cand in candidates:
        try:
            cand.mkdir(parents=True, exist_ok=True)
            probe = cand / f".probe_{os.getpid()}"
            probe.write_text("")
            probe.unlink()
            return cand
        except OSError:
            continue
    raise BuildError(f"no writable build folder among {[str(c) for c in candidates]}")


def _existing_library(lib_name: str) -> Optional[Path]:
    """A library built earlier, looked for in every folder ``build_dir`` may have chosen."""
    override = os.environ.get("TORCHLLMS_AMD_BUILD_DIR")
    folders = [Path(override)] if override else []
    folders += [CSRC / "_build", Path(tempfile.gettempdir()) / f"torchllms_amd_build_{os.getuid()}"]
    for folder in folders:
        p = folder / f"lib{lib_name}.so"
        if p.is_file():
            return p
    return None


def _hash(sources: Sequence[str], defines: Sequence[str]) -> str:
    h = hashlib.sha256()
    for name in list(sources) + HEADERS:
        h.update(name.encode())
        h.update((CSRC / name).read_bytes())
    h.update(" ".join(HIPCC_FLAGS + list(defines)).encode())
    return h.hexdigest()


def _run(cmd: List[str], what: str) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines() if "is not a recognized feature for this target" not in line
    )
    if proc.returncode != 0:
        raise BuildError(f"{what} failed (exit {proc.returncode}):\n{' '.join(cmd)}\n{out}")
    if out.strip():
        _log(f"{what}:\n{out}")


def build_library(lib_name: str, sources: Sequence[str], defines: Sequence[str] = (), force: bool = False) -> Path:
    """Compile ``sources`` (names under csrc/) into ``lib<lib_name>.so``; return its path."""
    digest = _hash(sources, defines)
    if not force:
        have = _existing_library(lib_name)
        if have is not None:
            stamp = have.with_suffix(".stamp")
            if stamp.is_file() and stamp.read_text().strip() == digest:
                return have
    hipcc = find_hipcc()
    out_dir = build_dir()
    lib = out_dir / f"lib{lib_name}.so"
    _log(f"compiling {lib.name} for {ARCH} from {len(sources)} source file(s) into {out_dir}")
    t0 = time.time()
    stop = threading.Event()

    def heartbeat():
        while not stop.wait(20.0):
            _log(f"... still compiling {lib.name} ({time.time() - t0:.0f} s)")

    beat = threading.Thread(target=heartbeat, daemon=True)
    beat.start()
    try:
        objs = []

        def compile_one(src: str) -> Path:
            # the process id keeps two processes that build the same library at once (two first calls from
            # one checkout) out of each other's files; the library itself is moved into place whole
            obj = out_dir / f"{lib_name}.{Path(src).stem}.{os.getpid()}.o"
            _run([hipcc, *HIPCC_FLAGS, *defines, "-I", str(CSRC), "-c", str(CSRC / src), "-o", str(obj)], f"compile {src}")
            return obj

        workers = max(1, min(len(sources), int(os.environ.get("MAX_JOBS", "8")), 16))
        with ThreadPoolExecutor(max_workers=workers) as pool:
            objs = list(pool.map(compile_one, sources))
        tmp = out_dir / f"lib{lib_name}.{os.getpid()}.tmp.so"
        _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)], f"link {lib.name}")
        os.replace(tmp, lib)
        lib.with_suffix(".stamp").write_text(digest)
        for o in objs:
            try:
                o.unlink()
            except OSError:
                pass
    finally:
        stop.set()
    _log(f"built {lib.name} in {time.time() - t0:.1f} s")
    return lib


def build_core(force: bool = False) -> Path:
    return build_library(CORE_NAME, CORE_SOURCES, force=force)


#: variant libraries: name pattern, source, macro that carries the size
VARIANTS: Dict[str, Dict[str, str]] = {}


def register_variant(kind: str, source: str, macro: str) -> None:
    VARIANTS[kind] = {"source": source, "macro": macro}


def variant_name(kind: str, value: int) -> str:
    return f"torchllms_amd_{kind}_{value}"


def build_variant(kind: str, value: int, force: bool = False) -> Path:
    v = VARIANTS[kind]
    return build_library(variant_name(kind, value), [v["source"]], defines=[f"-D{v['macro']}={value}"], force=force)


register_variant("attn_decode", "attention_decode.hip", "TL_HEAD_DIM")
register_variant("attn_prefill", "attention_prefill.hip", "TL_HEAD_DIM")
# the roofline micro-benchmarks of bench.py (one library; the macro only names its version)
register_variant("peaks", "peaks.hip", "TL_PEAKS")

#: sizes compiled ahead of time by ``build_all`` (tests, the smoke run and the benchmark use these)
PREBUILT_VARIANTS: Dict[str, Iterable[int]] = {"attn_decode": (32, 64, 128, 256), "attn_prefill": (32, 64, 128, 256), "peaks": (1,)}


def stale_libraries() -> List[str]:
    """Names of libraries that were built earlier and whose sources or flags have changed since:
    their next use compiles them again.  Libraries that were never built are not named."""
    wanted = [(CORE_NAME, CORE_SOURCES, [])]
    for kind, values in PREBUILT_VARIANTS.items():
        v = VARIANTS[kind]
        wanted += [(variant_name(kind, value), [v["source"]], [f"-D{v['macro']}={value}"]) for value in values]
    stale = []
    for lib_name, sources, defines in wanted:
        have = _existing_library(lib_name)
        if have is None:
            continue
        stamp = have.with_suffix(".stamp")
        if not stamp.is_file() or stamp.read_text().strip() != _hash(sources, defines):
            stale.append(lib_name)
    return stale


def build_all(force: bool = False) -> List[Path]:
    """Everything the tests, the smoke run and the benchmark load."""
    out = [build_core(force=force)]
    for kind, values in PREBUILT_VARIANTS.items():
        for value in values:
            out.append(build_variant(kind, value, force=force))
    return out


if __name__ == "__main__":
    for p in build_all(force="--force" in sys.argv):
        print(p)
