"""Shared pieces of the GPU tests: model folders made once per session, the plain reference for a
token list, and the one definition of "equal beyond rounding"."""
import functools
import os
import shutil
import tempfile

import torch

import plain_llama as P
from tiny_configs import ALL

# max |engine - plain| / max |plain| over the compared logits.  Fixed when the first kernels ran
# (measured then: float32 below 1e-6, bfloat16 below 8e-3 on these configurations).
TOL = {"float32": 2e-5, "bfloat16": 2e-2}
# The same row by row: max |engine - plain| of a row / max |plain| of THAT row, so that a row of small
# logits cannot hide behind the largest logit of another.  Fixed when this bound was added, from
# what the suite showed then (the worst row of all comparisons: float32 6e-6, bfloat16 1.7e-2).
ROW_TOL = {"float32": 2e-5, "bfloat16": 3e-2}
worst_row_seen = {"float32": 0.0, "bfloat16": 0.0}

_folders = {}
_root = None


def model_folder(name: str, stored: str = "float32", seed: int = 7, **init) -> str:
    """A random-weights model folder for tiny configuration ``name`` (made once, in a temp folder).
    ``init`` replaces fields of the architecture's rule for drawing the weights (``overrides=...``)."""
    global _root
    key = (name, stored, seed, repr(sorted(init.items())))
    if key not in _folders:
        import nanoinfer_amd  # noqa: F401
        from nanoinfer_amd.weights.loader import make_random_model

        if _root is None:
            _root = tempfile.mkdtemp(prefix="nanoinfer-tests-")
            import atexit
            atexit.register(shutil.rmtree, _root, ignore_errors=True)
        _folders[key] = make_random_model(os.path.join(_root, f"{name}-{stored}-{seed}-{len(_folders)}"), ALL[name], seed,
                                          dtype=stored, **init)
    return _folders[key]


@functools.lru_cache(maxsize=None)
def _plain_model(folder: str, as_bf16: bool):
    config, tensors = P.read_model_folder(folder)
    return config, (P.round_to_bfloat16(tensors) if as_bf16 else tensors)


@functools.lru_cache(maxsize=None)
def plain_logits(folder: str, tokens: tuple, dtype: str) -> torch.Tensor:
    """Logits of the whole sequence by the plain implementation; for a bfloat16 engine the
    matrices are rounded to bfloat16 first, as the engine holds them."""
    config, tensors = _plain_model(folder, dtype == "bfloat16")
    return P.forward(config, tensors, list(tokens))


def random_tokens(vocab: int, n: int, seed: int):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randint(0, vocab, (n,), generator=g).tolist())


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float((got.double().cpu() - want).abs().max() / want.abs().max())


def assert_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what: str = "") -> None:
    assert tuple(got.shape) == tuple(want.shape), f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    diff = (got.double().cpu() - want).abs()
    err = float(diff.max() / want.abs().max())
    if diff.dim() == 2:
        per_row = diff.max(dim=-1).values / want.abs().max(dim=-1).values
        worst_row_seen[dtype] = max(worst_row_seen[dtype], float(per_row.max()))
        if not float(per_row.max()) <= ROW_TOL[dtype]:
            row = int(per_row.argmax())
            raise AssertionError(f"{what}: row {row} of {diff.shape[0]} is off by {float(per_row[row]):.3e} of its own "
                                 f"largest logit, beyond {ROW_TOL[dtype]:.0e} ({dtype})")
    if not err <= TOL[dtype]:
        row = int(diff.max(dim=-1).values.argmax()) if diff.dim() == 2 else -1
        raise AssertionError(f"{what}: relative error {err:.3e} exceeds {TOL[dtype]:.0e} ({dtype}); "
                             f"worst row {row} of {diff.shape[0] if diff.dim() == 2 else 1}; "
                             f"first row beyond tolerance "
                             f"{int((diff.max(dim=-1).values / want.abs().max() > TOL[dtype]).nonzero()[0]) if diff.dim() == 2 else -1}")
