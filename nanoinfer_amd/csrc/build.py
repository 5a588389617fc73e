"""Compile the HIP sources of this folder for gfx950 into shared libraries and find them again.

A library is named ``<name>-<hash>.so`` where the hash covers the sources, the headers, the
defines and the compiler flags, so a stale build is never loaded: when a source changes the
name changes and the library is compiled again at its first use.  Libraries are written beside
the sources (``_lib/``) when that folder can be written, else under the temporary folder.
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
from typing import Dict, Iterable, List, Optional

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"
FLAGS = ["-O3", "-std=c++17", "-shared", "-fPIC", f"--offload-arch={ARCH}",
         # packed float32 arithmetic is kept out of the generated code
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-unused-value", "-Wno-unknown-warning-option"]
HEADERS = ["common.h", "attention_api.h"]


class BuildError(RuntimeError):
    pass


def find_hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.isfile(cand) and os.access(cand, os.X_OK):
            return cand
    raise BuildError("hipcc was not found (looked at $HIPCC, PATH and /opt/rocm/bin): "
                     "the HIP kernels of nanoinfer_amd cannot be compiled")


def _digest(sources: Iterable[str], defines: Dict[str, object]) -> str:
    h = hashlib.sha256()
    for rel in list(sources) + HEADERS:
        with open(os.path.join(HERE, rel), "rb") as fh:
            h.update(rel.encode())
            h.update(fh.read())
    h.update(repr(sorted(defines.items())).encode())
    h.update(repr(FLAGS).encode())
    return h.hexdigest()[:12]


def _lib_dirs() -> List[str]:
    dirs = [os.path.join(HERE, "_lib")]
    uid = os.getuid() if hasattr(os, "getuid") else 0
    dirs.append(os.path.join(tempfile.gettempdir(), f"nanoinfer_amd-lib-{uid}"))
    return dirs


def library_path(name: str, sources: List[str], defines: Optional[Dict[str, object]] = None,
                 force: bool = False, verbose: bool = True) -> str:
    """Path of the built library; compiles it when it is not there (or when ``force``)."""
    defines = defines or {}
    fname = f"{name}-{_digest(sources, defines)}.so"
    if not force:
        for d in _lib_dirs():
            p = os.path.join(d, fname)
            if os.path.isfile(p):
                return p
    out_dir = None
    for d in _lib_dirs():
        try:
            os.makedirs(d, exist_ok=True)
            probe = os.path.join(d, f".w{os.getpid()}-{threading.get_ident()}")
            with open(probe, "w"):
                pass
            os.remove(probe)
            out_dir = d
            break
        except OSError:
            continue
    if out_dir is None:
        raise BuildError(f"no writable folder for compiled kernels among {_lib_dirs()}")
    out = os.path.join(out_dir, fname)
    tmp = out + f".tmp{os.getpid()}-{threading.get_ident()}"
    cmd = [find_hipcc()] + FLAGS + [f"-D{k}={v}" for k, v in sorted(defines.items())] + \
          [f"-I{HERE}"] + [os.path.join(HERE, s) for s in sources] + ["-o", tmp]
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())  # the compiler wants a home for its caches
    if verbose:
        print(f"[nanoinfer_amd] compiling {name} for {ARCH} ...", file=sys.stderr, flush=True)
    t0 = time.time()
    stop = threading.Event()

    def _tick():
        while not stop.wait(20.0):
            print(f"[nanoinfer_amd] still compiling {name} ({time.time() - t0:.0f} s)", file=sys.stderr, flush=True)

    ticker = threading.Thread(target=_tick, daemon=True)
    if verbose:
        ticker.start()
    try:
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    finally:
        stop.set()
    if proc.returncode != 0:
        if os.path.exists(tmp):
            os.remove(tmp)
        raise BuildError(f"hipcc failed for {name}:\n{' '.join(cmd)}\n{proc.stdout}")
    os.replace(tmp, out)
    # drop older builds of the same library
    for f in os.listdir(out_dir):
        if f.startswith(name + "-") and f.endswith(".so") and f != fname:
            try:
                os.remove(os.path.join(out_dir, f))
            except OSError:
                pass
    if verbose:
        print(f"[nanoinfer_amd] compiled {name} in {time.time() - t0:.1f} s -> {out}", file=sys.stderr, flush=True)
    return out


# What the framework is made of.  Attention is compiled per head size.
CORE = ("ni_ops", ["ops.hip"], {})
SAMPLING = ("ni_sampling", ["sampling.hip"], {})
SKINNY = ("ni_skinny_gemm", ["gemv.hip"], {})
COMMON_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 160, 256)


def attention_target(head_dim: int):
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise BuildError(f"head size {head_dim} is not supported by the attention kernels: "
                         "it must be a multiple of 16 between 16 and 256")
    return (f"ni_attention_hd{head_dim}", ["attention.hip"], {"HEAD_DIM": head_dim})


def attention_mfma_target(head_dim: int):
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise BuildError(f"head size {head_dim} is not supported by the matrix-core attention kernel: "
                         "it must be a multiple of 16 between 16 and 256")
    return (f"ni_attention_mfma_hd{head_dim}", ["attention_mfma.hip"], {"HEAD_DIM": head_dim})


def attention_mfma_f32_target(head_dim: int):
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise BuildError(f"head size {head_dim} is not supported by the float32 matrix-core attention kernel: "
                         "it must be a multiple of 16 between 16 and 256")
    return (f"ni_attention_mfma_f32_hd{head_dim}", ["attention_mfma_f32.hip"], {"HEAD_DIM": head_dim})


def build_all(head_dims: Iterable[int] = COMMON_HEAD_DIMS, force: bool = True, verbose: bool = True,
              jobs: Optional[int] = None) -> List[str]:
    """Compile every library (attention for the given head sizes)."""
    targets = [CORE, SAMPLING, SKINNY] + [attention_target(h) for h in head_dims] + \
        [attention_mfma_target(h) for h in head_dims] + \
        [attention_mfma_f32_target(h) for h in head_dims]
    # the compiler runs in processes of its own: a few at a time (the longest, the skinny product, first)
    from concurrent.futures import ThreadPoolExecutor
    workers = max(1, min(8, (os.cpu_count() or 2) // 2 if jobs is None else int(jobs)))
    order = sorted(range(len(targets)), key=lambda i: targets[i] is not SKINNY)
    paths: List[Optional[str]] = [None] * len(targets)
    with ThreadPoolExecutor(max_workers=workers) as pool:
        futures = {i: pool.submit(library_path, *targets[i], force=force, verbose=verbose) for i in order}
        for i, f in futures.items():
            paths[i] = f.result()
    return paths
