"""Tensors of a model folder, by name, checked against what the model's parts ask for.

The reference trusts running offsets into its own file format and validates neither size nor
shape (src/model/llama.cpp:568-706).  Here the parts state the names and shapes they need, the
file states what it holds, and every difference is reported in ONE error: tensors that are
missing, tensors nobody asked for, tensors of the wrong shape.

Types: a tensor is handed on as stored (bfloat16 stays bfloat16, float32 stays float32, float16
is widened to float32, integer tables become int32); the parts place matrices in the compute type
and one-dimensional parameters in float32.
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, List, Tuple

import torch

from ..config.model_config import read_config_json
from ..config.spec import ModelSpec
from ..registry import architecture_of, get_part
from .safetensors_io import SafetensorsFile, WeightFileError, write_safetensors, write_safetensors_streamed


class WeightMismatchError(WeightFileError):
    """The checkpoint does not hold exactly the tensors the model needs."""

    def __init__(self, path: str, missing: List[str], unexpected: List[str],
                 wrong_shape: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]]):
        self.path = path
        self.missing = missing
        self.unexpected = unexpected
        self.wrong_shape = wrong_shape
        lines = [f"{path} does not match the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shape ({len(wrong_shape)}): " + ", ".join(
                f"{n} is {list(got)}, expected {list(want)}" for n, want, got in wrong_shape))
        super().__init__("\n".join(lines))


def expected_tensors(spec: ModelSpec) -> Dict[str, Tuple[int, ...]]:
    """Name -> shape of every tensor the parts of ``spec`` ask for (a name asked for twice, as
    by a tied head, must be asked for with one shape)."""
    requests = list(get_part("embedding", spec.embedding.kind).weight_requests(spec.embedding))
    for b in spec.blocks:
        requests += get_part("block", b.kind).weight_requests(b)
    requests += get_part("norm", spec.final_norm.kind).weight_requests(spec.final_norm)
    requests += get_part("head", spec.head.kind).weight_requests(spec.head)
    out: Dict[str, Tuple[int, ...]] = {}
    for r in requests:
        shape = tuple(int(s) for s in r.shape)
        if r.name in out and out[r.name] != shape:
            raise WeightFileError(f"tensor {r.name!r} is asked for with shapes {out[r.name]} and {shape}")
        out[r.name] = shape
    return out


def _as_stored(t: torch.Tensor) -> torch.Tensor:
    if t.dtype in (torch.bfloat16, torch.float32):
        return t
    if t.dtype in (torch.float16, torch.float64):
        return t.to(torch.float32)
    if t.dtype in (torch.int64, torch.int16, torch.int8, torch.uint8, torch.int32):
        return t.to(torch.int32)
    raise WeightFileError(f"tensor type {t.dtype} cannot be used")


INDEX_NAME = "model.safetensors.index.json"


class _Checkpoint:
    """The tensors of a model folder by name: one ``model.safetensors``, or the shards that
    ``model.safetensors.index.json`` names (its ``weight_map``: tensor name -> file name)."""

    def __init__(self, folder: str):
        single = os.path.join(folder, "model.safetensors")
        index = os.path.join(folder, INDEX_NAME)
        self.files: Dict[str, SafetensorsFile] = {}
        self.where: Dict[str, str] = {}
        if os.path.isfile(single) or not os.path.isfile(index):
            self.path = single
            f = self.files[single] = SafetensorsFile(single)
            self.where = {n: single for n in f.names()}
            return
        self.path = index
        try:
            with open(index) as fh:
                weight_map = json.load(fh)["weight_map"]
        except (OSError, ValueError, KeyError) as e:
            raise WeightFileError(f"{index}: not a shard index with a weight_map ({e})") from None
        for name, shard in weight_map.items():
            path = os.path.join(folder, str(shard))
            if path not in self.files:
                self.files[path] = SafetensorsFile(path)
            self.where[name] = path
        listed = set(weight_map)
        for path, f in self.files.items():
            for n in f.names():
                if n not in listed:
                    self.where.setdefault(n, path)      # a tensor the index forgot is still "unexpected", not lost
        absent = sorted(n for n, path in self.where.items() if n not in self.files[path].names())
        if absent:
            raise WeightFileError(f"{index}: tensors named in the index are not in their shards: {absent}")

    def names(self):
        return self.where.keys()

    def shape(self, name: str):
        return self.files[self.where[name]].shape(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self.files[self.where[name]].tensor(name)


def load_tensors(folder: str, spec: ModelSpec) -> Dict[str, torch.Tensor]:
    """The tensors ``spec`` needs from the checkpoint in ``folder`` (CPU views of the mapped files):
    ``model.safetensors``, or the shards listed in ``model.safetensors.index.json``."""
    f = _Checkpoint(folder)
    path = f.path
    want = expected_tensors(spec)
    have = set(f.names())
    missing = sorted(n for n in want if n not in have)
    unexpected = []
    for n in sorted(have - set(want)):
        orig = spec.duplicates.get(n)
        if orig in have and tuple(f.shape(n)) == tuple(f.shape(orig)) and torch.equal(f.tensor(n), f.tensor(orig)):
            continue  # a second copy of a tensor the model shares
        if any(n.endswith(suffix) for suffix in spec.ignorable_suffixes):
            continue  # a buffer that exporters write along and the model does not use
        unexpected.append(n)
    wrong = sorted((n, want[n], f.shape(n)) for n in want if n in have and tuple(f.shape(n)) != want[n])
    if missing or unexpected or wrong:
        raise WeightMismatchError(path, missing, unexpected, wrong)
    return {n: _as_stored(f.tensor(n)) for n in want}


def check_tensors(spec: ModelSpec, tensors: Dict[str, torch.Tensor], where: str = "the tensors given") -> Dict[str, torch.Tensor]:
    """Tensors handed over directly (no file) checked as a checkpoint's are: every tensor the parts of
    ``spec`` ask for is there with its shape and none besides, or ONE error names all that differ."""
    want = expected_tensors(spec)
    missing = sorted(n for n in want if n not in tensors)
    unexpected = sorted(n for n in tensors if n not in want
                        and not any(n.endswith(suffix) for suffix in spec.ignorable_suffixes))
    wrong = sorted((n, want[n], tuple(tensors[n].shape)) for n in want if n in tensors and tuple(tensors[n].shape) != want[n])
    if missing or unexpected or wrong:
        raise WeightMismatchError(where, missing, unexpected, wrong)
    return {n: _as_stored(tensors[n]) for n in want}


def write_model_folder(folder: str, config_json: Dict[str, Any], tensors: Dict[str, torch.Tensor],
                       shards: int = 1) -> str:
    """``config.json`` and the checkpoint: one ``model.safetensors``, or ``shards`` files and their index."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(config_json, fh, indent=2)
    if shards <= 1:
        write_safetensors(os.path.join(folder, "model.safetensors"), tensors, {"format": "pt"})
        return folder
    names = list(tensors)
    per = -(-len(names) // shards)
    weight_map, total = {}, 0
    for i in range(shards):
        part = {n: tensors[n] for n in names[i * per:(i + 1) * per]}
        if not part:
            continue
        fname = f"model-{i + 1:05d}-of-{shards:05d}.safetensors"
        write_safetensors(os.path.join(folder, fname), part, {"format": "pt"})
        for n, t in part.items():
            weight_map[n] = fname
            total += t.numel() * t.element_size()
    with open(os.path.join(folder, INDEX_NAME), "w") as fh:
        json.dump({"metadata": {"total_size": total}, "weight_map": weight_map}, fh, indent=2)
    return folder


_TORCH_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def make_random_model(folder: str, config_json: Dict[str, Any], seed: int, dtype: str = "bfloat16",
                      shards: int = 1, device=None, **init) -> str:
    """Random-weights mode: write ``config.json`` and ``model.safetensors`` (or ``shards`` files and
    their index) for the architecture that ``config_json`` names, from a seed.  ``dtype`` is the type
    every tensor is stored in.  What is drawn is the architecture's :class:`InitRule`, of which
    ``init`` may replace fields (``matrix_std=...``); which tensors exist, and their shapes, is what
    the parts of the model ask for.  Every element is a function of (seed, tensor name, element
    index), so the file does not depend on where it is made: with a GPU (``device``; default: the
    current one when there is one) large tensors are generated there and streamed to the file piece
    by piece, which a model of tens of gigabytes needs; without, numpy gives the same bits."""
    if dtype not in _TORCH_DTYPES:
        raise WeightFileError(f"dtype {dtype!r} is not one of {sorted(_TORCH_DTYPES)}")
    import dataclasses

    from . import random_init

    arch = architecture_of(config_json)
    cfg = arch.config_from_dict(config_json)
    spec = arch.build_spec(cfg)
    rule = dataclasses.replace(arch.init, **init) if init else arch.init
    store = _TORCH_DTYPES[dtype]
    if device is None and torch.cuda.is_available():
        device = torch.device("cuda", torch.cuda.current_device())
    entries = []
    for name, shape in expected_tensors(spec).items():
        mean, std = rule.mean_std(name, shape)
        entries.append((name, store, shape,
                        lambda name=name, shape=shape, mean=mean, std=std:
                        random_init.pieces(seed, name, shape, mean, std, store, device)))
    out = dict(cfg.to_dict())
    out["torch_dtype"] = "bfloat16" if store == torch.bfloat16 else "float32"
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(out, fh, indent=2)
    if shards <= 1:
        write_safetensors_streamed(os.path.join(folder, "model.safetensors"), entries, {"format": "pt"})
        return folder
    per = -(-len(entries) // shards)
    weight_map, total = {}, 0
    for i in range(shards):
        part = entries[i * per:(i + 1) * per]
        if not part:
            continue
        fname = f"model-{i + 1:05d}-of-{shards:05d}.safetensors"
        write_safetensors_streamed(os.path.join(folder, fname), part, {"format": "pt"})
        for name, dt, shape, _ in part:
            weight_map[name] = fname
            n = 1
            for d in shape:
                n *= int(d)
            total += n * (2 if dt == torch.bfloat16 else 4)
    with open(os.path.join(folder, INDEX_NAME), "w") as fh:
        json.dump({"metadata": {"total_size": total}, "weight_map": weight_map}, fh, indent=2)
    return folder


def read_model_folder(folder: str):
    """``(architecture, typed configuration, spec)`` of a model folder, chosen by ``config.json``."""
    raw = read_config_json(folder)
    arch = architecture_of(raw)
    cfg = arch.config_from_dict(raw)
    return arch, cfg, arch.build_spec(cfg)
