"""Compiles the HIP sources under csrc/ for gfx950 into shared libraries, one per
(source, element type), and finds them again.

A library's file name carries a digest of the sources it was built from, so a library
that is found is never stale; what is missing is compiled on first use (only the
libraries that the running model's element type needs), with a progress line per
library.  Libraries are written next to the sources (csrc/_build/) when that folder
can be written, else under NANO_VLLM_AMD_BUILD_DIR or the system's temporary folder.
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
from typing import Dict, Iterable, List, Optional, Tuple

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "csrc")
ARCH = "gfx950"

# module -> (source file, element types it is compiled for; None = no element type)
MODULES: Dict[str, Tuple[str, Tuple[Optional[str], ...]]] = {
    "embed": ("embed.hip", ("bf16", "f32")),
    "norm": ("norm.hip", ("bf16", "f32")),
    "activation": ("activation.hip", ("bf16", "f32")),
    "rope": ("rope.hip", ("bf16", "f32")),
    "attn_generic": ("attn_generic.hip", ("bf16", "f32")),
    "gemm": ("gemm.hip", ("bf16", "f32")),
    "gemm_skinny": ("gemm_skinny.hip", ("bf16",)),
    "gemm_team": ("gemm_team.hip", ("bf16",)),
    "gemm_tile": ("gemm_tile.hip", ("bf16",)),
    "attn_decode": ("attn_decode.hip", ("bf16",)),
    "attn_prefill": ("attn_prefill.hip", ("bf16",)),
    "sample": ("sample.hip", (None,)),
}

_HEADERS = ("common.h",)
_FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", "-fvisibility=hidden",
          # hipcc -O3 forms packed-float instructions by itself; they are switched off
          # for every kernel here (a device flag: the host pass reports it as unknown).
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


class BuildError(RuntimeError):
    pass


def _digest(source: str, dtype: Optional[str]) -> str:
    h = hashlib.sha256()
    for name in (source,) + _HEADERS + tuple(sorted(_extra_headers(source))):
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode())
            h.update(f.read())
    h.update(" ".join(_FLAGS).encode())
    h.update((dtype or "-").encode())
    return h.hexdigest()[:12]


def _extra_headers(source: str) -> List[str]:
    """Headers of csrc/ that the source includes besides common.h."""
    out = []
    with open(os.path.join(CSRC, source)) as f:
        for line in f:
            line = line.strip()
            if line.startswith('#include "'):
                name = line.split('"')[1]
                if name not in _HEADERS and os.path.isfile(os.path.join(CSRC, name)):
                    out.append(name)
    return out


def _writable(folder: str) -> bool:
    try:
        os.makedirs(folder, exist_ok=True)
        probe = tempfile.NamedTemporaryFile(dir=folder, delete=True)
        probe.close()
        return True
    except OSError:
        return False


def build_dirs() -> List[str]:
    """Folders that may hold libraries, in the order they are searched."""
    dirs = [os.path.join(CSRC, "_build")]
    env = os.environ.get("NANO_VLLM_AMD_BUILD_DIR")
    if env:
        dirs.append(env)
    dirs.append(os.path.join(tempfile.gettempdir(), f"nano_vllm_amd-{os.getuid()}"))
    return dirs


def _file_name(module: str, dtype: Optional[str]) -> str:
    source, dtypes = MODULES[module]
    if dtype not in dtypes:
        raise BuildError(f"kernel module {module!r} has no build for element type {dtype!r}")
    tag = f"_{dtype}" if dtype else ""
    return f"nva_{module}{tag}.{_digest(source, dtype)}.so"


def find_library(module: str, dtype: Optional[str]) -> Optional[str]:
    name = _file_name(module, dtype)
    for d in build_dirs():
        path = os.path.join(d, name)
        if os.path.isfile(path):
            return path
    return None


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand):
            return cand
    raise BuildError("hipcc was not found (PATH, HIPCC, /opt/rocm/bin): the HIP kernels cannot be compiled")


def _compile(module: str, dtype: Optional[str], out_dir: str) -> str:
    source, _ = MODULES[module]
    name = _file_name(module, dtype)
    final = os.path.join(out_dir, name)
    tmp = os.path.join(out_dir, f".{name}.{os.getpid()}.tmp")
    cmd = [_hipcc(), f"--offload-arch={ARCH}"] + _FLAGS
    if dtype:
        cmd.append("-DNVA_" + dtype.upper())
    cmd += [os.path.join(CSRC, source), "-o", tmp]
    env = dict(os.environ)
    env.setdefault("HOME", out_dir)          # hipcc wants a home for its temporary files
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, cwd=out_dir)
    if proc.returncode != 0:
        raise BuildError(f"hipcc failed for {source} ({dtype}):\n{proc.stdout}")
    os.replace(tmp, final)
    # older builds of the same library are of no use any more
    prefix = name.split(".")[0] + "."
    for other in os.listdir(out_dir):
        if other.startswith(prefix) and other.endswith(".so") and other != name:
            try:
                os.remove(os.path.join(out_dir, other))
            except OSError:
                pass
    return final


def ensure_built(wanted: Iterable[Tuple[str, Optional[str]]], force: bool = False, quiet: bool = False,
                 jobs: Optional[int] = None) -> Dict[Tuple[str, Optional[str]], str]:
    """Returns {(module, dtype): path}, compiling what is missing (everything if force)."""
    wanted = list(dict.fromkeys(wanted))
    found: Dict[Tuple[str, Optional[str]], str] = {}
    todo = []
    for key in wanted:
        path = None if force else find_library(*key)
        if path:
            found[key] = path
        else:
            todo.append(key)
    if not todo:
        return found
    out_dir = next((d for d in build_dirs() if _writable(d)), None)
    if out_dir is None:
        raise BuildError(f"no writable folder for compiled kernels among {build_dirs()}")
    jobs = jobs or max(1, min(len(todo), int(os.environ.get("MAX_JOBS", "0")) or (os.cpu_count() or 4), 16))
    say = (lambda *a: None) if quiet else (lambda *a: print(*a, file=sys.stderr, flush=True))
    say(f"[nano_vllm_amd] compiling {len(todo)} kernel librar{'y' if len(todo) == 1 else 'ies'} "
        f"for {ARCH} into {out_dir} ({jobs} at a time)")
    t0 = time.time()
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        futures = {pool.submit(_compile, m, d, out_dir): (m, d) for m, d in todo}
        pending = set(futures)
        done_count = 0
        while pending:
            import concurrent.futures as cf
            finished, pending = cf.wait(pending, timeout=20, return_when=cf.FIRST_COMPLETED)
            for fut in finished:
                key = futures[fut]
                found[key] = fut.result()
                done_count += 1
                say(f"[nano_vllm_amd]   {done_count}/{len(todo)} {key[0]}{'/' + key[1] if key[1] else ''} "
                    f"built after {time.time() - t0:.0f} s")
            if not finished:
                say(f"[nano_vllm_amd]   still compiling ({len(pending)} left, {time.time() - t0:.0f} s)")
    return found


def all_targets() -> List[Tuple[str, Optional[str]]]:
    return [(m, d) for m, (_, dtypes) in MODULES.items() for d in dtypes]


def targets_for(dtype: str) -> List[Tuple[str, Optional[str]]]:
    """What a model of one element type ("bf16" or "f32") needs."""
    out = []
    for m, (_, dtypes) in MODULES.items():
        if dtype in dtypes:
            out.append((m, dtype))
        elif None in dtypes:
            out.append((m, None))
    return out


def build_all(force: bool = True, quiet: bool = False):
    return ensure_built(all_targets(), force=force, quiet=quiet)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv or True)
