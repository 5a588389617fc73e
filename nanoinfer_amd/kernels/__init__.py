"""Python face of the HIP kernels: loads the compiled libraries through ``ctypes`` and checks,
on the host, that operand shapes, types and devices are what each kernel and its grid assume.

There is no fallback: when a library cannot be built or loaded, or a tensor is not on the GPU,
the call raises.  Matrix products are the one thing taken from a library (``torch.matmul`` ->
rocBLAS/hipBLASLt), as the reference takes them from cuBLAS (src/op/kernels/cuda/matmul_kernel.cu:76-86).
"""
from __future__ import annotations

import ctypes
import functools
from typing import Dict, Optional

import torch

from ..csrc import build as _build


class KernelError(RuntimeError):
    pass


_DTYPE_CODE = {torch.float32: 0, torch.bfloat16: 1}
_libs: Dict[str, ctypes.CDLL] = {}


def _load(target) -> ctypes.CDLL:
    name, sources, defines = target
    lib = _libs.get(name)
    if lib is None:
        path = _build.library_path(name, sources, defines)
        try:
            lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load the compiled kernels {path}: {e}") from e
        _libs[name] = lib
    return lib


def core() -> ctypes.CDLL:
    return _load(_build.CORE)


def sampling_lib() -> ctypes.CDLL:
    return _load(_build.SAMPLING)


def skinny_lib() -> ctypes.CDLL:
    return _load(_build.SKINNY)


def attention_lib(head_dim: int) -> ctypes.CDLL:
    return _load(_build.attention_target(head_dim))


def attention_mfma_lib(head_dim: int) -> ctypes.CDLL:
    return _load(_build.attention_mfma_target(head_dim))


def attention_mfma_f32_lib(head_dim: int) -> ctypes.CDLL:
    return _load(_build.attention_mfma_f32_target(head_dim))


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise KernelError(f"compute type {dtype} is not supported (float32 or bfloat16)") from None


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> ctypes.c_void_p:
    """The current stream of the current device as the kernels' launch argument (the raw handle is
    asked for directly: building a Stream object costs more than a small kernel's launch)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _gpu(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    """Host-side check of one kernel operand; the message is built only when the check fails."""
    if not t.is_cuda:
        raise KernelError(f"{name} must live on the GPU (no CPU fallback exists)")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, is {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} must have shape {tuple(shape)}, has {tuple(t.shape)}")


def _check(err: int, what: str) -> None:
    if err != 0:
        raise KernelError(f"{what}: launch failed with HIP error {err}")


# ------------------------------------------------------------------ row-wise / element-wise

def embedding(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out[t] = table[ids[t]]`` as float32; ``ids`` were range-checked by the caller."""
    T = ids.shape[0]
    vocab, d = table.shape
    _gpu(ids, "ids", torch.int32, (T,))
    _gpu(table, "table")
    _gpu(out, "out", torch.float32, (T, d))
    _check(core().ni_embedding(_ptr(ids), _ptr(table), _ptr(out), T, d, vocab, dtype_code(table.dtype), _stream()),
           "embedding")
    return out


def add_rmsnorm(h: torch.Tensor, pending: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``h += pending`` (when no ``rows``) and ``out = rmsnorm(h) * weight``; with ``rows`` only those
    rows are read and ``h`` stays as it is.  ``pending`` is [T, d] of the output's type, or float32
    [S, T, d]: S addends (the shares of a product whose K range was cut), added in their order."""
    T, d = h.shape
    _gpu(h, "h", torch.float32)
    _gpu(weight, "weight", torch.float32, (d,))
    n = T if rows is None else rows.shape[0]
    _gpu(out, "out", None, (n, d))
    addends, float_addends = 1, 0
    if pending is not None:
        if pending.dim() == 3:
            _gpu(pending, "pending", torch.float32, (pending.shape[0], T, d))
            addends, float_addends = pending.shape[0], 1
        else:
            _gpu(pending, "pending", out.dtype, (T, d))
    if rows is not None:
        _gpu(rows, "rows", torch.int32, (n,))
    _check(core().ni_add_rmsnorm(_ptr(h), _ptr(pending), addends, float_addends, ctypes.c_size_t(T * d), _ptr(weight),
                                 _ptr(out), _ptr(rows), n, d, ctypes.c_float(eps), dtype_code(out.dtype), _stream()),
           "add_rmsnorm")
    return out


def rope_table(inv_freq: torch.Tensor, max_pos: int):
    """cos and sin of ``pos * inv_freq[p]`` in float32, each ``[max_pos, len(inv_freq)]``."""
    _gpu(inv_freq, "inv_freq", torch.float32)
    half = inv_freq.shape[0]
    cos = torch.empty(max_pos, half, dtype=torch.float32, device=inv_freq.device)
    sin = torch.empty_like(cos)
    _check(core().ni_rope_table(_ptr(inv_freq), _ptr(cos), _ptr(sin), max_pos, half, _stream()), "rope_table")
    return cos, sin


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, cos: Optional[torch.Tensor],
                  sin: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor], kpool: Optional[torch.Tensor],
                  vpool: Optional[torch.Tensor], H: int, KVH: int, hd: int) -> None:
    """Rotate the query and key heads of ``qkv`` ([T, (H+2KVH)*hd]) and store keys and values in
    the pools ([pages, KVH, page_size, hd]) at ``slot_mapping`` (absent: nothing is stored)."""
    T = qkv.shape[0]
    _gpu(qkv, "qkv", None, (T, (H + 2 * KVH) * hd))
    _gpu(positions, "positions", torch.int32, (T,))
    rot = 0
    if cos is not None:
        rot = 2 * cos.shape[1]
        if not (rot <= hd):
            raise KernelError(f"rotary size {rot} exceeds the head size {hd}")
        _gpu(cos, "cos", torch.float32)
        _gpu(sin, "sin", torch.float32, cos.shape)
    page_size = 1
    if slot_mapping is not None:
        _gpu(slot_mapping, "slot_mapping", torch.int32, (T,))
        if not (kpool is not None and vpool is not None):
            raise KernelError("a slot mapping needs both pools")
        _gpu(kpool, "kpool", qkv.dtype)
        _gpu(vpool, "vpool", qkv.dtype, kpool.shape)
        if not (kpool.dim() == 4 and kpool.shape[1] == KVH and kpool.shape[3] == hd):
            raise KernelError(f"pool must be [pages, {KVH}, page_size, {hd}], is {tuple(kpool.shape)}")
        page_size = kpool.shape[2]
    _check(core().ni_rope_kv_write(_ptr(qkv), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(slot_mapping),
                                   _ptr(kpool), _ptr(vpool), T, H, KVH, hd, rot, page_size,
                                   dtype_code(qkv.dtype), _stream()), "rope_kv_write")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out = silu(gate_up[:, :I]) * gate_up[:, I:]``."""
    T, two_i = gate_up.shape
    if not (two_i % 2 == 0):
        raise KernelError("gate_up needs an even width")
    _gpu(gate_up, "gate_up")
    _gpu(out, "out", gate_up.dtype, (T, two_i // 2))
    _check(core().ni_swiglu(_ptr(gate_up), _ptr(out), T, two_i // 2, dtype_code(gate_up.dtype), _stream()), "swiglu")
    return out


def random_normal(out: torch.Tensor, key: int, start: int, mean: float, std: float) -> torch.Tensor:
    """``out[i] = mean + std * n(key, start + i)`` for the flat tensor ``out`` (float32 or bfloat16):
    the counter-based normal stream of :mod:`nanoinfer_amd.weights.random_init`, same bits as its
    numpy routine."""
    _gpu(out, "out")
    if not (out.dim() == 1 and 0 <= int(key) < 2 ** 64 and int(start) >= 0):
        raise KernelError("random_normal fills a flat tensor from a 64-bit key and a non-negative start")
    _check(core().ni_random_normal(_ptr(out), ctypes.c_size_t(out.numel()), ctypes.c_uint64(int(key)),
                                   ctypes.c_uint64(int(start)), ctypes.c_float(mean), ctypes.c_float(std),
                                   dtype_code(out.dtype), _stream()), "random_normal")
    return out


# ------------------------------------------------------------------ attention

def choose_splits(n_tokens: int, kv_heads: int, group: int, max_keys: int) -> int:
    """How many pieces the key range of every token is cut into, so that a small batch still
    fills the 256 compute units.  One piece never holds fewer than 256 keys."""
    chunks = (group + 3) // 4
    items = max(1, n_tokens * kv_heads * chunks)
    want = max(1, 512 // items)
    return int(max(1, min(want, (max_keys + 255) // 256, 64)))


def _token_attention_checks(qkv, kpool, vpool, block_table, seq_of_token, positions, out, H, KVH, hd, nsplit, workspace):
    T = qkv.shape[0]
    _gpu(qkv, "qkv")
    if not (qkv.shape[1] >= H * hd):
        raise KernelError("qkv is narrower than the query heads")
    if not (H % KVH == 0):
        raise KernelError(f"{H} query heads do not divide into {KVH} kv heads")
    _gpu(kpool, "kpool", qkv.dtype)
    _gpu(vpool, "vpool", qkv.dtype, kpool.shape)
    if not (kpool.dim() == 4 and kpool.shape[1] == KVH and kpool.shape[3] == hd):
        raise KernelError(f"pool must be [pages, {KVH}, page_size, {hd}], is {tuple(kpool.shape)}")
    _gpu(block_table, "block_table", torch.int32)
    if not (block_table.dim() == 2):
        raise KernelError("block_table must be [sequences, pages]")
    _gpu(seq_of_token, "seq_of_token", torch.int32, (T,))
    _gpu(positions, "positions", torch.int32, (T,))
    _gpu(out, "out", qkv.dtype, (T, H * hd))
    part_o = part_ml = None
    if nsplit > 1:
        need = T * H * nsplit * (hd + 2)
        if not (workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need):
            raise KernelError(f"attention workspace of {need} floats needed for {nsplit} splits")
        _gpu(workspace, "workspace")
        flat = workspace.view(-1)
        part_o = flat[: T * H * nsplit * hd]
        part_ml = flat[T * H * nsplit * hd: need]
    return T, part_o, part_ml


def token_attention(qkv: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, block_table: torch.Tensor,
                    seq_of_token: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, H: int, KVH: int,
                    hd: int, scale: float, window: Optional[int], nsplit: int,
                    workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of every token of ``qkv`` over the paged cache of its sequence.

    ``qkv`` is [T, >= H*hd] with the (rotated) query heads first; the pools already hold the keys
    and values of all positions up to each token's own.  ``workspace`` (float32, at least
    ``T*H*nsplit*(hd+2)`` elements) is needed when ``nsplit > 1``.
    """
    T, part_o, part_ml = _token_attention_checks(qkv, kpool, vpool, block_table, seq_of_token, positions, out,
                                                 H, KVH, hd, nsplit, workspace)
    lib = attention_lib(hd)
    _check(lib.ni_token_attention(_ptr(qkv), qkv.shape[1], _ptr(kpool), _ptr(vpool), _ptr(block_table),
                                  block_table.shape[1], _ptr(seq_of_token), _ptr(positions), _ptr(out),
                                  _ptr(part_o), _ptr(part_ml), T, H, KVH, kpool.shape[2],
                                  int(window) if window else 0, ctypes.c_float(scale), nsplit,
                                  dtype_code(qkv.dtype), _stream()), "token_attention")
    return out


def mfma_token_splits(n_tokens: int, kv_heads: int, group: int, max_keys: int) -> int:
    """Into how many runs the matrix-core kernel for single tokens cuts every key range.  Up to a
    workgroup per compute unit: enough runs to give every unit one, none shorter than 256 keys
    (measured at batches 1 to 64 and contexts of 2,100 and 8,200 keys).  Beyond that the units
    that get one workgroup more than the others set the time, each drawing the same ~37 GB/s
    whatever runs on it: 264 workgroups take 42 us where 256 take 26.  Two runs each even that out
    a little where they leave the fullest unit three halves instead of two wholes (37 us there;
    more runs lose to their own start-up and to the kernel that merges them)."""
    units = COMPUTE_UNITS
    items = max(1, n_tokens * kv_heads * ((group + 15) // 16))
    if items <= units:
        return int(max(1, min(units // items, max_keys // 256, 64)))
    whole = -(-items // units)                       # workgroups on the fullest unit, uncut
    halves = -(-2 * items // units)                  # and with two runs each
    return 2 if max_keys >= 512 and halves / 2 + 0.2 < whole else 1


def mfma_token_attention(qkv: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, block_table: torch.Tensor,
                         seq_of_token: torch.Tensor, positions: torch.Tensor, out: torch.Tensor, H: int, KVH: int,
                         hd: int, scale: float, window: Optional[int], nsplit: int,
                         workspace: Optional[torch.Tensor] = None, merge: bool = True) -> torch.Tensor:
    """:func:`token_attention` on the matrix cores (types and head sizes that :func:`mfma_token_ok`
    takes): the query heads of a kv head are the rows of the products, the wavefronts of a
    workgroup share out the keys.  With ``nsplit > 1`` and ``merge=False`` the partial results of
    the key runs are left in ``workspace`` for :func:`skinny_gemm_merged` and ``out`` is not written."""
    if not (mfma_token_ok(qkv.dtype, hd)):
        raise KernelError(f"mfma_token_attention does not take {qkv.dtype} with head size {hd}")
    if not (qkv.shape[1] % (16 // qkv.element_size()) == 0):
        raise KernelError("rows of qkv are not aligned to 16 bytes")
    T, part_o, part_ml = _token_attention_checks(qkv, kpool, vpool, block_table, seq_of_token, positions, out,
                                                 H, KVH, hd, nsplit, workspace)
    if qkv.dtype == torch.float32:
        launch = attention_mfma_f32_lib(hd).ni_mfma_token_attention_f32
    else:
        if not (kpool.numel() // hd < 2 ** 32):
            raise KernelError("the matrix-core attention kernels number the rows of a pool in 32 bits")
        launch = attention_mfma_lib(hd).ni_mfma_token_attention
    _check(launch(_ptr(qkv), qkv.shape[1], _ptr(kpool), _ptr(vpool), _ptr(block_table), block_table.shape[1],
                  _ptr(seq_of_token), _ptr(positions), _ptr(out), _ptr(part_o), _ptr(part_ml), T, H, KVH, kpool.shape[2],
                  int(window) if window else 0, ctypes.c_float(scale), nsplit, _stream()), "mfma_token_attention")
    if nsplit > 1 and merge:
        _check(attention_lib(hd).ni_merge_splits(_ptr(part_o), _ptr(part_ml), _ptr(out), T, H, nsplit,
                                                 dtype_code(out.dtype), _stream()), "merge_splits")
    return out


def mfma_attention_ok(dtype: torch.dtype, hd: int) -> bool:
    """Whether a matrix-core attention kernel for prompt portions takes this type and head size:
    bfloat16 and float32, head sizes in steps of 16 up to 256."""
    return dtype in (torch.bfloat16, torch.float32) and hd % 16 == 0 and 16 <= hd <= 256


def mfma_token_ok(dtype: torch.dtype, hd: int) -> bool:
    """Whether a matrix-core kernel for single tokens takes this type and head size: bfloat16 with
    head sizes in steps of 32, float32 in steps of 16."""
    if dtype == torch.bfloat16:
        return hd % 32 == 0 and 32 <= hd <= 256
    return dtype == torch.float32 and hd % 16 == 0 and 16 <= hd <= 256


COMPUTE_UNITS = 256      # of an MI355X


def _heads_per_tile(group: int) -> int:
    return 16 if group >= 16 else 8 if group > 4 else 4 if group > 2 else 2 if group > 1 else 1


def mfma_tile_tokens(hd: int, group: int, n_tokens: Optional[int] = None, kv_heads: int = 1,
                     dtype: torch.dtype = torch.bfloat16) -> int:
    """Tokens of one tile of the matrix-core attention kernel for ``group`` query heads per kv head.
    A wavefront owns one block of 16 rows, or two where the head size leaves registers for them.
    More blocks share every staged key among more rows and give a wavefront more independent work,
    but fewer tiles fill the chip less evenly (the kernel pairs long tiles with short ones, in a workgroup
    or over the two workgroups of a compute unit): two blocks are taken where a step of ``n_tokens``
    tokens still has one and a half such tiles for every compute unit (measured at head size 64, one
    block : two blocks in us: 1,024 tokens 19.8 : 24.0, 1,536 tokens 41.8 : 37.0, 2,048 tokens 44.2 : 43.2,
    2,560 tokens 100.4 : 78.6, 3,072 tokens 117.2 : 95.3, 4,096 tokens 150.8 : 108.0).  Without ``n_tokens``:
    the smallest tile.  The float32 kernel has one tile size."""
    if dtype == torch.float32:
        return int(attention_mfma_f32_lib(hd).ni_mfma_attention_f32_tile_tokens(int(group)))
    lib = attention_mfma_lib(hd)
    hpt = _heads_per_tile(group)
    blocks = 1
    if n_tokens is not None:
        chunks = (group + hpt - 1) // hpt
        for b in (2,):
            if b <= int(lib.ni_mfma_attention_max_blocks()) and \
                    2 * (n_tokens // (4 * b * 16 // hpt)) * kv_heads * chunks >= 3 * COMPUTE_UNITS:
                blocks = b
                break
    return int(lib.ni_mfma_attention_tile_tokens(int(group), blocks))


def mfma_plan(hd: int, group: int, kv_heads: int, n_tokens: int, max_q_len: int, max_keys: int,
              dtype: torch.dtype = torch.bfloat16):
    """Tile size and number of key runs for the matrix-core attention of a step of ``n_tokens``
    tokens whose longest portion has ``max_q_len`` and whose rows read at most ``max_keys`` keys:
    ``(tile_tokens, nsplit)``, ``nsplit`` None where :func:`mfma_splits` is to decide from the
    number of tiles.  Tiles of two blocks a wavefront are taken for long prompts
    (:func:`mfma_tile_tokens`), and for one portion alone that stands far into its sequence (the
    keys before it at least as many as its own, judged from ``max_keys`` rounded up to a power of
    two so that a recorded step and its eager twin decide alike): its tiles are then of like length
    and need no pairing, and cutting their keys into runs of 512 or more fills the chip (measured at
    head size 64: 512 tokens at context 2,048 take 36.8 us with one block and no cut, 30.8 with two
    blocks and four runs; at context 4,096 68.4 and 45.7)."""
    if dtype == torch.float32:
        return mfma_tile_tokens(hd, group, dtype=dtype), None
    small = mfma_tile_tokens(hd, group)
    tile = mfma_tile_tokens(hd, group, n_tokens, kv_heads)
    if tile != small:
        return tile, None
    lib = attention_mfma_lib(hd)
    hpt = _heads_per_tile(group)
    per_tile = kv_heads * ((group + hpt - 1) // hpt)
    bound = max(256, 1 << max(0, int(max_keys) - 1).bit_length())
    if int(lib.ni_mfma_attention_max_blocks()) >= 2 and n_tokens == max_q_len and bound >= 4 * n_tokens - 2:
        items = max(1, n_tokens // (2 * small)) * per_tile
        nsplit = min(-(-2 * COMPUTE_UNITS // items), bound // 512, 16)
        if nsplit >= 1 and items * nsplit >= 2 * COMPUTE_UNITS:
            return 2 * small, int(nsplit)
    return small, None


def build_q_tiles(q_start, q_len, context_len, tile_tokens: int):
    """Cut the portions of a step (host lists: first row, length, context after the step) into
    tiles of at most ``tile_tokens`` tokens: flat list of (sequence, first row, tokens, first position),
    the tiles with the most keys before them first (the kernel deals them out in that order)."""
    tiles = []
    for s, (row, n, total) in enumerate(zip(q_start, q_len, context_len)):
        first = total - n
        for t0 in range(0, n, tile_tokens):
            tiles.append((s, row + t0, min(tile_tokens, n - t0), first + t0))
    tiles.sort(key=lambda t: -(t[3] + t[2]))
    return [x for t in tiles for x in t]


def mfma_splits(n_tiles: int, kv_heads: int, group: int, max_keys: int) -> int:
    """Into how many runs the matrix-core kernel cuts the keys of every tile.  Cutting costs a
    second kernel that merges the runs, and float32 partial results in between: a step with many
    tiles is cut only into runs of 2,048 keys or more, up to about a thousand workgroups (measured
    for portions of 512 tokens at contexts of 512 to 8,192), and not at all once it has two tiles for
    every compute unit (2,048 tokens in tiles of 32 at contexts of 4,096 / 8,192 / 32,768: 88 / 180 / 721 us
    uncut, 99 / 192 / 741 in two runs; 1,024 tokens, one tile a unit: 75 / 142 uncut, 64 / 114 in two);
    a step with fewer tiles than the chip has compute units, into runs of 512 keys or more until
    every unit has one."""
    hpt = _heads_per_tile(group)
    items = max(1, n_tiles * kv_heads * ((group + hpt - 1) // hpt))
    many = min(1024 // items if items < 2 * COMPUTE_UNITS else 1, max_keys // 2048)
    few = min(COMPUTE_UNITS // items, max_keys // 512)
    return int(max(1, min(max(many, few), 16)))


def mfma_attention(qkv: torch.Tensor, kpool: torch.Tensor, vpool: torch.Tensor, block_table: torch.Tensor,
                   tiles: torch.Tensor, out: torch.Tensor, H: int, KVH: int, hd: int, scale: float,
                   window: Optional[int], nsplit: int = 1, workspace: Optional[torch.Tensor] = None,
                   tile_tokens: Optional[int] = None) -> torch.Tensor:
    """Attention of prompt portions on the matrix cores, in bfloat16 or in true float32 (a kernel
    each).  ``tiles`` is int32 [n, 4] from :func:`build_q_tiles` with ``tile_tokens`` tokens a tile (a
    size that :func:`mfma_tile_tokens` gives for the type; default: its smallest); the pools already
    hold the keys and values of every position of the step.  ``workspace`` (float32,
    ``T*H*nsplit*(hd+2)`` elements) is needed when ``nsplit > 1``."""
    T = qkv.shape[0]
    dtype = qkv.dtype
    _gpu(qkv, "qkv")
    if not (mfma_attention_ok(dtype, hd)):
        raise KernelError(f"mfma_attention does not take {dtype} with head size {hd}")
    if not (H >= 1 and KVH >= 1 and H % KVH == 0):
        raise KernelError(f"{H} query heads do not divide into {KVH} kv heads")
    smallest = mfma_tile_tokens(hd, H // KVH, dtype=dtype)
    tile_tokens = smallest if tile_tokens is None else int(tile_tokens)
    blocks = tile_tokens // smallest
    most = 1 if dtype == torch.float32 else int(attention_mfma_lib(hd).ni_mfma_attention_max_blocks())
    if not (blocks * smallest == tile_tokens and 1 <= blocks <= most):
        raise KernelError(f"mfma_attention has no tiles of {tile_tokens} tokens at head size {hd} in {dtype} "
                          f"(the smallest has {smallest})")
    if not (qkv.shape[1] >= H * hd and qkv.shape[1] % 8 == 0):
        raise KernelError("qkv is narrower than the query heads or its rows are unaligned")
    _gpu(kpool, "kpool", dtype)
    _gpu(vpool, "vpool", dtype, kpool.shape)
    if not (kpool.dim() == 4 and kpool.shape[1] == KVH and kpool.shape[3] == hd):
        raise KernelError(f"pool must be [pages, {KVH}, page_size, {hd}], is {tuple(kpool.shape)}")
    if not (kpool.numel() // hd < 2 ** 32):
        raise KernelError("the matrix-core attention kernels number the rows of a pool in 32 bits")
    _gpu(block_table, "block_table", torch.int32)
    _gpu(tiles, "tiles", torch.int32)
    if not (tiles.dim() == 2 and tiles.shape[1] == 4):
        raise KernelError("tiles must be [n, 4]")
    _gpu(out, "out", dtype, (T, H * hd))
    if not (1 <= nsplit <= 64):
        raise KernelError(f"mfma_attention cuts the keys into 1 to 64 runs, not {nsplit}")
    part_o = part_ml = None
    if nsplit > 1:
        need = T * H * nsplit * (hd + 2)
        if not (workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need):
            raise KernelError(f"attention workspace of {need} floats needed for {nsplit} splits")
        _gpu(workspace, "workspace")
        flat = workspace.view(-1)
        part_o = flat[: T * H * nsplit * hd]
        part_ml = flat[T * H * nsplit * hd: need]
    if dtype == torch.float32:
        _check(attention_mfma_f32_lib(hd).ni_mfma_attention_f32(
            _ptr(qkv), qkv.shape[1], _ptr(kpool), _ptr(vpool), _ptr(block_table), block_table.shape[1], _ptr(tiles),
            tiles.shape[0], _ptr(out), _ptr(part_o), _ptr(part_ml), H, KVH, kpool.shape[2],
            int(window) if window else 0, ctypes.c_float(scale), nsplit, _stream()), "mfma_attention (float32)")
    else:
        _check(attention_mfma_lib(hd).ni_mfma_attention(
            _ptr(qkv), qkv.shape[1], _ptr(kpool), _ptr(vpool), _ptr(block_table), block_table.shape[1], _ptr(tiles),
            tiles.shape[0], _ptr(out), _ptr(part_o), _ptr(part_ml), H, KVH, kpool.shape[2],
            int(window) if window else 0, ctypes.c_float(scale), nsplit, blocks, _stream()), "mfma_attention")
    if nsplit > 1:
        _check(attention_lib(hd).ni_merge_splits(_ptr(part_o), _ptr(part_ml), _ptr(out), T, H, nsplit,
                                                 dtype_code(out.dtype), _stream()), "merge_splits")
    return out


# ------------------------------------------------------------------ sampling

def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    R, V = logits.shape
    _gpu(logits, "logits", torch.float32)
    if out is None:
        out = torch.empty(R, dtype=torch.int32, device=logits.device)
    _gpu(out, "out", torch.int32, (R,))
    part_val = torch.empty(R, 32, dtype=torch.float32, device=logits.device)
    part_idx = torch.empty(R, 32, dtype=torch.int32, device=logits.device)
    _check(sampling_lib().ni_argmax(_ptr(logits), _ptr(out), _ptr(part_val), _ptr(part_idx), R, V, _stream()), "argmax")
    return out


def sample(logits: torch.Tensor, work: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, penalty: torch.Tensor, pen_ids: torch.Tensor, pen_off: torch.Tensor,
           uniform: torch.Tensor, out: torch.Tensor, uses_top_k: bool = True, uses_top_p: bool = True,
           pen_count: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row of ``logits`` [R, V]: repetition penalty on the tokens ``pen_ids[pen_off[r]:
    pen_off[r+1]]``, temperature, top-k, softmax, top-p, and the token at which the cumulative mass
    in vocabulary order reaches ``uniform[r]`` times the kept mass; rows with temperature <= 0 take
    the largest (penalised) logit.  ``work`` [R, V] is scratch.  ``uses_top_k`` / ``uses_top_p``
    may be False when no row asks for it: their launches are then left out.  With ``pen_count``
    (int32 [R]) row r's penalised tokens are the first ``pen_count[r]`` from ``pen_off[r]`` on, and
    the chosen token is appended to them and counted, for the next draw of the same rows: the
    caller leaves room behind every row's tokens."""
    R, V = logits.shape
    _gpu(logits, "logits", torch.float32)
    _gpu(work, "work", torch.float32, (R, V))
    for name, t, dt in (("temperature", temperature, torch.float32), ("top_k", top_k, torch.int32),
                        ("top_p", top_p, torch.float32), ("penalty", penalty, torch.float32),
                        ("uniform", uniform, torch.float32), ("out", out, torch.int32)):
        _gpu(t, name, dt, (R,))
    _gpu(pen_off, "pen_off", torch.int32, (R + 1,))
    _gpu(pen_ids, "pen_ids", torch.int32)
    if pen_count is not None:
        _gpu(pen_count, "pen_count", torch.int32, (R,))
    lib = sampling_lib()
    P = int(lib.ni_sample_parts(R, V))
    # per-part results, two sets of per-part histograms, the decisions of the levels
    scratch = torch.empty(R * P * 5 + 2 * R * P * 256 + R * 16, dtype=torch.int32, device=logits.device)
    parts, hist, state = scratch[: R * P * 5], scratch[R * P * 5: R * P * 5 + 2 * R * P * 256], scratch[-R * 16:]
    _check(lib.ni_sample(_ptr(logits), _ptr(work), _ptr(temperature), _ptr(top_k), _ptr(top_p),
                         _ptr(penalty), _ptr(pen_ids), _ptr(pen_off), _ptr(pen_count), _ptr(uniform), _ptr(out),
                         _ptr(parts), _ptr(hist), _ptr(state), R, V, P, int(bool(uses_top_k)), int(bool(uses_top_p)),
                         _stream()), "sample")
    return out


# ------------------------------------------------------------------ matrix product (library)

SKINNY_MAX_ROWS = 64        # what the kernel takes
SKINNY_BEST_ROWS = 16       # up to here the skinny product beats the library's on this chip whatever the matrix


def skinny_wins(M: int, K: int, dtype: torch.dtype, weight=None) -> bool:
    """Whether the skinny product is the faster one for M rows of K elements (measured at the 1B
    sizes, bfloat16).  Up to 16 rows always.  From 17 to 64 rows (re-tiled matrices only) every
    workgroup reads the rows of x that belong to its columns' K range anew: that is worth it while
    x is small beside the matrix, which ends at rows of more than 4,096 elements and over 32 rows
    (the [2048, 8192] matrix: 20.8 us against the library's 19.5 at 64 rows, 14.0 : 13.7 at 32,
    while [2048, 2048] takes 7.0 : 8.7 and the stacked [16384, 2048] with SwiGLU 21.8 : 25.5)."""
    if not skinny_ok(M, K, dtype):
        return False
    if M <= SKINNY_BEST_ROWS:
        return True
    if not (isinstance(weight, Weight) and weight.tiles is not None):
        return False
    if dtype == torch.float32:
        # float32 rows are twice the bytes and a workgroup holds half the tiles, so what the workgroups load of x is
        # twice the matrix and more.  Measured in recorded steps (us, skinny : library, with the SwiGLU kernel where the
        # fusion saves it), layer sizes of the 1B / 3B / 8B shapes: only rows of 2,048 elements gain or tie
        # ([2048, 2048] at 32 rows 10.7 : 10.1, stacked [16384, 2048] 36.7 : 35.4; at 64 rows 17.0 : 13.2 and 57.8 : 44.2);
        # [16384, 3072] at 32 rows 52.9 : 51.2, at 64 rows 81.9 : 60.7; [3072, 8192] 41.2 : 30.6 and 61.1 : 45.2;
        # [28672, 4096] 122.8 : 103.6 and 197.7 : 141.9; [4096, 14336] 72.3 : 57.9 and 107.5 : 86.2
        return K <= 2048 and (M <= 32 or weight.rows.shape[0] < 8192)
    return M <= 32 or K <= 4096
FUSE_NORMS = True           # residual sums and norms ride on the skinny products of a decode step where they can
ADDENDS_IN_PROLOGUE = True  # the shares of a cut product are added by the next normalising prologue and residual epilogue
MERGE_IN_PRODUCT = True     # the key runs of a decode step's attention are merged by the output product where it can
SPLIT_K = True              # products of 17 to 64 rows on matrices of few tiles are cut along K, the next norm adds the shares
DEFER_NORMS = True          # a product onto the residual stream leaves h * w and sums of squares for the next norm, whose division the product behind it makes


def tile_weight(w: torch.Tensor) -> torch.Tensor:
    """``w`` [N, K] re-laid for the skinny product: [tile of 16 rows][128-byte piece][lane][32 bytes]
    with lane = 16 * (which 32 bytes of the piece) + (row in the tile), zero-padded to whole tiles
    and pieces.  Flat, same type and device as ``w``."""
    N, Kd = w.shape
    el = 8 if w.dtype == torch.float32 else 16
    ch = 4 * el
    Np, Kp = (N + 15) // 16 * 16, (Kd + ch - 1) // ch * ch
    if (Np, Kp) != (N, Kd):
        padded = torch.zeros(Np, Kp, dtype=w.dtype, device=w.device)
        padded[:N, :Kd] = w
        w = padded
    return w.view(Np // 16, 16, Kp // ch, 4, el).permute(0, 2, 3, 1, 4).contiguous().view(-1)


class Weight:
    """A matrix [out, in] as the products want it: ``rows`` as stored (for the library product of
    many rows) and, optionally, ``tiles`` in the order the skinny product streams it."""

    __slots__ = ("rows", "tiles", "rows_t")

    def __init__(self, rows: torch.Tensor, tiled: bool = True):
        self.rows = rows
        self.rows_t = rows.t()        # the view the library product takes, made once
        self.tiles = tile_weight(rows) if tiled and rows.dtype in (torch.float32, torch.bfloat16) else None

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype


def _rows_and_tiles(weight):
    if isinstance(weight, Weight):
        return weight.rows, weight.tiles
    return weight, None
_library_calls = 0


def library_calls() -> int:
    """How many library routines (matrix products) ran inside steps so far.  A step in whose recording
    the count has moved is replayed against eager runs before the recording is used."""
    return _library_calls


def note_library_call() -> None:
    """For a part that calls a library routine of its own inside a step (a product, a reduction):
    say so, so that a recording of the step is tried against eager runs before it is used (some
    library routines record nodes that do not replay faithfully)."""
    global _library_calls
    _library_calls += 1



def skinny_ok(M: int, K: int, dtype: torch.dtype) -> bool:
    """Whether the hand-written skinny product takes this shape: at most 64 rows, rows of W that
    split into whole 32-byte lane loads."""
    return 0 < M <= SKINNY_MAX_ROWS and K % (8 if dtype == torch.float32 else 16) == 0


def _tiles_per_group(n_out: int) -> int:
    tiles = (n_out + 15) // 16
    return 4 if tiles >= 2048 else (2 if tiles >= 512 else 1)


class NormedInput:
    """The input of a product given as the float32 residual stream ``h`` [M, K] together with the
    weight and eps of the RMSNorm that stands before the product: the skinny product normalises the
    rows in its prologue instead of a kernel of its own (:func:`norm_prologue_ok` says when).
    ``pending``: float32 addends [S, M, K] that ``h`` has not received yet (the shares of a product
    whose K range was cut); the rows are normalised as ``(h + pending[0]) + pending[1]`` and ``h``
    is left as it is: whoever adds into ``h`` next (the residual epilogue of a later product, given
    the same addends) brings them in."""

    __slots__ = ("h", "weight", "eps", "dtype", "pending")

    def __init__(self, h: torch.Tensor, weight: torch.Tensor, eps: float, dtype: torch.dtype,
                 pending: Optional[torch.Tensor] = None):
        self.h, self.weight, self.eps, self.dtype, self.pending = h, weight, float(eps), dtype, pending

    @property
    def shape(self):
        return self.h.shape

    @property
    def device(self):
        return self.h.device


class NormSpec:
    """Weight and eps of an RMSNorm, for a product onto the residual stream that is to leave the norm's
    input half done behind (:class:`ScaledInput`)."""

    __slots__ = ("weight", "eps")

    def __init__(self, weight: torch.Tensor, eps: float):
        self.weight, self.eps = weight, float(eps)


class ScaledInput:
    """The input of a product that stands behind an RMSNorm, as the product before the norm left it:
    ``x`` [M, K] = ``h * weight`` in the compute type (not yet divided by the rows' root mean squares) and
    ``ss`` float32 [M, parts], the sums of ``h^2`` over the columns of each of that product's workgroups.
    ``RMSNorm(h) . W^T = ((h * w) . W^T) / rms(h)`` row by row: the skinny product multiplies ``x`` and
    divides in its epilogue, so no kernel normalises and none reads ``h`` for it.  The residual stream
    itself is complete (nothing is pending), so whoever cannot take this computes the norm of ``h``."""

    __slots__ = ("x", "ss", "norm")

    def __init__(self, x: torch.Tensor, ss: torch.Tensor, norm: NormSpec):
        self.x, self.ss, self.norm = x, ss, norm

    @property
    def shape(self):
        return self.x.shape

    @property
    def dtype(self):
        return self.x.dtype

    @property
    def device(self):
        return self.x.device

    def made_for(self, weight: torch.Tensor, eps: float) -> bool:
        """Whether this is the input of the norm with that weight tensor and eps."""
        return self.norm.weight is weight and self.norm.eps == float(eps)


DEFER_PARTS_MAX = 256        # sums of squares a row may come in (the kernels' bound)


@functools.lru_cache(maxsize=None)
def _residual_parts(M: int, N: int, K: int) -> int:
    return int(skinny_lib().ni_skinny_residual_parts(int(M), int(N), int(K), _tiles_per_group(N)))


def leaves_scaled_ok(M: int, K: int, dtype: torch.dtype, weight) -> bool:
    """Whether a product of M rows of K elements onto the residual stream should leave a :class:`ScaledInput`
    for the next norm; it then runs whole (its K range uncut) with the residual epilogue.  Measured in decode
    steps of the 1B / 3B / 8B shapes against the ways it replaces (ms a step without : with).  Up to 16 rows
    where the product runs whole anyway: the product behind the norm then needs neither a normalising
    prologue (every workgroup reading all of h) nor a norm kernel (1B bfloat16 at batch 8 / 12 / 16
    0.926 : 0.901, 1.057 : 1.008, 1.162 : 1.097, batch 1 the same; 1B float32 at batch 12 / 16 1.916 : 1.865,
    1.997 : 1.941; 3B bfloat16 at batch 1 / 8 / 16 2.101 : 1.981, 2.412 : 2.275, 2.980 : 2.845).  Not where the
    product would be cut along K to fill the chip (the down product of the 1B shape): whole it loses more than
    the norm saves (1B at batch 1 0.742 : 0.776, float32 at batch 8 1.622 : 1.722).  From 17 to 32 rows the
    products with rows of up to 4,096 elements (the o products), which whole beat their K shares plus the norm
    kernel that adds them (1B at batch 24 / 32 1.263 : 1.251, 1.400 : 1.389); past 32 rows they do not."""
    if not (DEFER_NORMS and isinstance(weight, Weight) and weight.tiles is not None and skinny_ok(M, K, dtype)):
        return False
    if _residual_parts(M, weight.rows.shape[0], K) > DEFER_PARTS_MAX:
        return False
    if M <= SKINNY_BEST_ROWS:
        if skinny_ksplit(M, K, dtype, weight)[0] == 1:
            return True
        # A matrix of few tiles and long rows, which would be cut along K to fill the chip (the down product of the 1B
        # shape): whole, it fills the chip by halved tiles instead (two workgroups a tile, each loading all of x),
        # which costs more than the cut and, from five rows on in bfloat16, less than what the next product saves
        # without a prologue that adds the shares or a norm kernel (a step of the 1B shape at batch 1 / 4 / 6 / 8 / 16,
        # cut : whole, 0.747 : 0.772, 0.818 : 0.823, 0.871 : 0.857, 0.903 : 0.890, 1.118 : 1.095; in float32, whose
        # matrices are twice the bytes, 1.364 : 1.504, 1.455 : 1.573, 1.613 : 1.717, 1.948 : 2.024)
        N = weight.rows.shape[0]
        return (dtype == torch.bfloat16 and M >= 5 and _tiles_per_group(N) == 1 and (N + 15) // 16 <= DEFER_PARTS_MAX // 2 and K >= 4096)
    return M <= 32 and K <= 4096 and skinny_wins(M, K, dtype, weight)


def takes_scaled_ok(M: int, K: int, dtype: torch.dtype, weight) -> bool:
    """Whether the skinny product of M rows with this matrix can take a :class:`ScaledInput` for x."""
    return (DEFER_NORMS and isinstance(weight, Weight) and weight.tiles is not None
            and skinny_wins(M, K, dtype, weight))


def _scaled_args(x: "ScaledInput", M: int, Kd: int):
    """(x, ss, parts, eps) of a scaled input, checked, for a kernel's arguments."""
    _gpu(x.x, "x", None, (M, Kd))
    _gpu(x.ss, "sums of squares", torch.float32)
    if not (x.ss.dim() == 2 and x.ss.shape[0] == M and 1 <= x.ss.shape[1] <= DEFER_PARTS_MAX):
        raise KernelError(f"sums of squares {tuple(x.ss.shape)} against [{M}, at most {DEFER_PARTS_MAX}]")
    return x.x, x.ss, int(x.ss.shape[1]), x.norm.eps


@functools.lru_cache(maxsize=None)
def _prologue_sizes_ok(M: int, K: int, code: int) -> bool:
    return bool(skinny_lib().ni_skinny_prologue_ok(M, K, code))


@functools.lru_cache(maxsize=None)
def prologue_addends() -> int:
    """How many pending addends the normalising prologue can add to its rows of h."""
    return int(skinny_lib().ni_skinny_prologue_addends())


def norm_prologue_ok(M: int, K: int, dtype: torch.dtype, weight, addends: int = 0, swiglu: bool = False) -> bool:
    """Whether the skinny product can take RMSNorm(h) for its input: at most eight rows (every
    workgroup normalises all of them: beyond that the norm as a kernel of its own is faster), a
    re-tiled matrix, rows short enough for the normalised operand to stay in registers.  With
    ``addends`` pending addends of h (:class:`NormedInput`): at most :func:`prologue_addends`, and a
    matrix of whose tiles a workgroup takes at most two (``swiglu``: a stacked gate/up matrix)."""
    if not (isinstance(weight, Weight) and weight.tiles is not None and dtype in _DTYPE_CODE
            and _prologue_sizes_ok(int(M), int(K), dtype_code(dtype))):
        return False
    if addends == 0:
        return True
    n_out = weight.rows.shape[0] // 2 if swiglu else weight.rows.shape[0]
    return addends <= prologue_addends() and _tiles_per_group(n_out) <= 2


def _check_addends(pending: Optional[torch.Tensor], M: int, width: int):
    """(pointer, count) of pending addends [S, M, width] in float32, for a kernel's arguments."""
    if pending is None:
        return None, 0
    _gpu(pending, "pending addends", torch.float32)
    if not (pending.dim() == 3 and pending.shape[1] == M and pending.shape[2] == width and 1 <= pending.shape[0] <= 16):
        raise KernelError(f"pending addends {tuple(pending.shape)} against [S <= 16, {M}, {width}]")
    return pending, int(pending.shape[0])


def skinny_ksplit(M: int, K: int, dtype: torch.dtype, weight):
    """(shares, tiles per workgroup) for a product of rows onto the residual stream whose K
    range is worth cutting: a matrix of few 16-row tiles (the [2048, K] matrices of the 1B shape have
    128) leaves half the chip idle with one workgroup a tile, and every compute unit that does work
    loads all of x.  Cut into shares the product runs on about 256 workgroups, each loading its share
    of x only; the shares' float32 sums are added by the kernel that adds the product to the residual
    stream.  Measured at the 1B shape (us): [2048, 8192] at 64 rows 20.9 -> 12.0 (the library 20.4), at
    32 rows 14.2 -> 9.1, at 16 rows 12.7 -> 8.1, at 9 rows 9.8 -> 7.5; [2048, 2048] at 64 rows 7.3 -> 5.5,
    at 32 rows 5.0 -> 4.0, at 16 rows 4.65 -> 4.4.  Up to 16 rows only rows of 4,096 elements or more are
    cut.  Up to eight rows the next product normalises in its prologue, which is worth more than the cut:
    there the product goes in the two shares that this prologue can add to its rows of h by itself
    (:class:`NormedInput` with ``pending``; the residual epilogue that follows brings them into h), which
    needs no kernel for the sum ([2048, 8192] at 8 rows 11.7 -> 8.3 us, at one row 9.6 -> 8.0; a decode
    step of the 1B shape 1.011 -> 0.982 ms at batch 8, 0.802 -> 0.776 at batch 1).  Float32 rows are cut by
    the same rule (a decode step of the 1B shape in float32: 4.51 -> 4.23 ms at batch 64, 3.18 -> 2.86 at
    32, 2.42 -> 2.27 at 16; before, the [2048, 8192] matrix at more than 32 rows went to the library,
    41.6 us a layer).  (1, .): not cut."""
    if not (SPLIT_K and isinstance(weight, Weight) and weight.tiles is not None
            and 1 <= M <= SKINNY_MAX_ROWS and skinny_ok(M, K, dtype)):
        return 1, 1
    N = weight.rows.shape[0]
    most = 16
    if M <= SKINNY_BEST_ROWS:
        if K < 4096:
            return 1, 1
        if _prologue_sizes_ok(int(M), int(N), dtype_code(dtype)):
            # the next product can normalise in its prologue: cut into as many shares as that prologue adds
            # to its rows of h (where it cannot, float32 rows of 8,192 elements are cut even so: the matrix
            # is twice the bytes, the cut gains more than the prologue)
            most = prologue_addends() if ADDENDS_IN_PROLOGUE else (16 if dtype == torch.float32 and K >= 8192 else 1)
    if dtype == torch.float32 and M > SKINNY_BEST_ROWS and N > 2048:
        # float32 past 16 rows: only matrices of at most 128 tiles gain by the cut; the library's product is faster on the
        # others ([3072, 8192] at 64 rows in two shares 54.6 us against 45.2, [4096, 4096] 33.5 : 26.8, [4096, 14336] 93.8 : 86.2)
        return 1, 1
    # two tiles a workgroup (half the workgroups' loads of x, twice the shares) past 32 rows of 4,096 elements or more,
    # and in bfloat16 from 17 rows of 3,072 or more (product and the norm kernel behind it in us at 17 / 32 rows, whole or
    # one tile a workgroup : two, [3072, 8192] 22.2 : 19.1 / 21.3 : 19.1, [4096, 14336] 32.0 : 28.1 / 33.4 : 28.6, [2048, 8192]
    # 12.9 : 12.5 / 13.4 : 12.9; [3072, 3072] at 48 / 64 rows 11.4 : 10.7 / 12.7 : 11.4)
    per = 2 if (M > 32 and K >= 4096) or (dtype == torch.bfloat16 and M > SKINNY_BEST_ROWS and K >= 3072) else 1
    groups = -(-((N + 15) // 16) // per)
    pieces = (K + 63) // 64
    # as many shares as keep the workgroups within one to a compute unit (192 groups in two shares are one and a
    # half rounds: measured slower), each share at least sixteen pieces
    shares = max(1, min(COMPUTE_UNITS // groups, pieces // 16, most))
    return shares, (per if shares > 1 else 1)


def skinny_gemm_ksplit(x: torch.Tensor, weight, shares: int, per_group: int) -> torch.Tensor:
    """``x . weight^T`` as ``shares`` float32 addends [shares, M, N] (see :func:`skinny_ksplit`)."""
    M, Kd = x.shape
    rows, tiles = _rows_and_tiles(weight)
    N = rows.shape[0]
    _gpu(x, "x", rows.dtype)
    _gpu(rows, "weight", None, (N, Kd))
    if not (tiles is not None and 1 <= M <= SKINNY_MAX_ROWS and skinny_ok(M, Kd, x.dtype) and 1 <= shares <= 16):
        raise KernelError(f"the product in shares does not take M={M}, K={Kd}, {shares} shares with this matrix")
    out = torch.empty(shares, M, N, dtype=torch.float32, device=x.device)
    _check(skinny_lib().ni_skinny_gemm_ksplit(_ptr(x), _ptr(tiles), _ptr(out), M, N, Kd, int(per_group), int(shares),
                                              dtype_code(x.dtype), _stream()), "skinny_gemm_ksplit")
    return out


def residual_epilogue_ok(M: int, K: int, dtype: torch.dtype, weight) -> bool:
    """Whether a product can go to the float32 residual stream without a kernel of its own for the
    sum: added by the skinny product's epilogue, or left as float32 shares for the next norm."""
    if not (isinstance(weight, Weight) and weight.tiles is not None):
        return False
    return skinny_wins(M, K, dtype, weight) or skinny_ksplit(M, K, dtype, weight)[0] > 1


def residual_takes_addends(M: int, K: int, dtype: torch.dtype, weight) -> bool:
    """Whether the product that goes into the residual stream can bring pending addends of the
    stream in with it (``linear(..., residual=h, pending=...)``): the decode step's kernel with the
    residual epilogue, not the product in shares."""
    return (isinstance(weight, Weight) and weight.tiles is not None and M <= SKINNY_BEST_ROWS
            and skinny_wins(M, K, dtype, weight) and skinny_ksplit(M, K, dtype, weight)[0] == 1)


def _check_normed(x: NormedInput, Kd: int) -> None:
    _gpu(x.h, "h", torch.float32)
    if not (x.h.dim() == 2 and x.h.shape[1] == Kd):
        raise KernelError(f"normed input {tuple(x.h.shape)} against K={Kd}")
    _gpu(x.weight, "norm weight", torch.float32, (Kd,))


def skinny_gemm(x, weight, out: torch.Tensor, swiglu: bool = False, residual: bool = False,
                pending: Optional[torch.Tensor] = None, leave: Optional[NormSpec] = None):
    """``x . weight^T`` for at most 64 rows of ``x``, streaming ``weight`` once (MFMA).  ``out``
    may be float32 for bfloat16 inputs.  With ``swiglu`` the weight is a stacked [2I, K] matrix
    (gate rows, then up rows) and ``out`` [M, I] receives ``silu(gate) * up``.  With ``residual``
    ``out`` is the float32 residual stream [M, N] and the product is added into it, after the
    ``pending`` addends [S, M, N] that the stream has not received yet (at most 16 rows).  ``x`` may
    be a :class:`NormedInput` or a :class:`ScaledInput`.  With ``residual`` and ``leave`` (the norm that
    stands behind the stream) a :class:`ScaledInput` for that norm is returned."""
    normed = isinstance(x, NormedInput)
    scaled = isinstance(x, ScaledInput)
    M, Kd = x.shape
    dtype = x.dtype
    rows, tiles = _rows_and_tiles(weight)
    N = rows.shape[0]
    _gpu(rows, "weight", dtype)
    if not (rows.shape[1] == Kd):
        raise KernelError(f"skinny_gemm: {tuple(x.shape)} x {tuple(rows.shape)}^T")
    if not (skinny_ok(M, Kd, dtype)):
        raise KernelError(f"skinny_gemm does not take M={M}, K={Kd} in {dtype}")
    if swiglu and tiles is not None and (N // 2) % 16:
        tiles = None          # gate and up halves do not start on tile boundaries: stream the rows as stored
    if swiglu:
        if not (N % 2 == 0):
            raise KernelError("a stacked gate/up matrix needs an even number of rows")
        if not (not residual):
            raise KernelError("swiglu and residual exclude each other")
        _gpu(out, "out", dtype, (M, N // 2))
        epi = 2
    elif residual:
        if not (tiles is not None):
            raise KernelError("the residual epilogue needs a re-tiled matrix")
        _gpu(out, "out", torch.float32, (M, N))
        epi = 3
    else:
        if not (out.dtype in (dtype, torch.float32)):
            raise KernelError(f"out must be {dtype} or float32")
        _gpu(out, "out", None, (M, N))
        epi = 1 if (out.dtype == torch.float32 and dtype != torch.float32) else 0
    if pending is not None and not (residual and M <= SKINNY_BEST_ROWS):
        raise KernelError("pending addends go with the residual epilogue of at most 16 rows")
    if leave is not None and not residual:
        raise KernelError("only a product onto the residual stream leaves the next norm's input behind")
    if scaled and (residual or tiles is None):
        raise KernelError("a scaled input goes into a product with a re-tiled matrix that does not add into the stream")
    pend, n_pend = _check_addends(pending, M, N)
    per_group = _tiles_per_group(N // 2 if swiglu else N)
    if tiles is None and per_group == 4 and M <= 12:
        # the widest matrices as stored (the head over the vocabulary): few rows stream fastest with fewer tiles a
        # workgroup (measured at [128256, 2048], us for 1 / 2 / 4 tiles: one row 83.9 / 87.4 / 90.3, four rows
        # 86.0 / 87.3 / 94.3, eight rows 97.9 / 90.5 / 94.1, twelve 109.9 / 98.8 / 100.0, sixteen 118.6 / 103.2 / 100.5)
        per_group = 1 if M <= 4 else 2
    if swiglu and M > SKINNY_BEST_ROWS and tiles is not None:
        # past 16 rows a workgroup that multiplies two pairs of gate and up tiles halves the loads of x, which
        # every workgroup brings in whole (measured, one pair : two pairs in us, at [16384, 2048]: 17 rows 15.9 : 15.9,
        # 32 rows 16.6 : 16.2, 64 rows 21.3 : 18.9; at [16384, 3072]: 17 rows 22.1 : 21.4, 32 rows 23.4 : 21.1, 64 rows
        # 29.6 : 24.5; at [28672, 4096]: 17 rows 49.1 : 48.2, 32 rows 54.6 : 48.4, 64 rows 67.4 : 54.4)
        per_group = max(per_group, 4)
    if normed:
        h_pend, h_n = _check_addends(x.pending, M, Kd)
        if not (tiles is not None and norm_prologue_ok(M, Kd, dtype, weight, h_n, swiglu) and epi in (0, 2)):
            raise KernelError(f"the normalising prologue does not take M={M}, K={Kd} in {dtype} with this matrix and epilogue")
        _check_normed(x, Kd)
        _check(skinny_lib().ni_skinny_gemm_normed(_ptr(x.h), _ptr(x.weight), ctypes.c_float(x.eps), _ptr(tiles), _ptr(out),
                                                  M, N, Kd, epi, per_group, dtype_code(dtype), _ptr(h_pend), h_n, _stream()),
               "skinny_gemm_normed")
        return out
    xn = next_w = ss = None
    parts, eps, left = 0, 0.0, None
    if scaled:
        x, ss, parts, eps = _scaled_args(x, M, Kd)
    elif leave is not None:
        _gpu(leave.weight, "next norm weight", torch.float32, (N,))
        parts = _residual_parts(M, N, Kd)
        xn = torch.empty(M, N, dtype=dtype, device=out.device)
        ss = torch.empty(M, parts, dtype=torch.float32, device=out.device)
        next_w, left = leave.weight, ScaledInput(xn, ss, leave)
    _gpu(x, "x")
    _check(skinny_lib().ni_skinny_gemm(_ptr(x), _ptr(rows if tiles is None else tiles), _ptr(out), M, N, Kd, epi,
                                       per_group, 0 if tiles is None else 1, dtype_code(dtype), _ptr(pend), n_pend,
                                       _ptr(xn), _ptr(next_w), _ptr(ss), parts, ctypes.c_float(eps), _stream()), "skinny_gemm")
    return left if left is not None else out


def skinny_merge_ok(M: int, H: int, hd: int, nsplit: int, dtype: torch.dtype, weight) -> bool:
    """Whether the product of an attention's output with ``weight`` can merge the attention's
    ``nsplit`` key runs in its prologue: bfloat16, a re-tiled matrix, few rows, and heads and runs
    whose weights fit the workgroup's LDS."""
    if not (isinstance(weight, Weight) and weight.tiles is not None and dtype == torch.bfloat16):
        return False
    return bool(skinny_lib().ni_skinny_merge_ok(int(M), int(H), int(hd), int(nsplit), dtype_code(dtype)))


def skinny_merge_wins(M: int, H: int, hd: int, nsplit: int, dtype: torch.dtype, weight) -> bool:
    """Whether merging in the product's prologue is also the faster way.  Every workgroup of the
    product reads all partial results of all rows, 4 * nsplit times the bytes of the merged rows,
    through its compute unit's one path of 64 bytes a cycle: that beats the merge kernel's launch
    for one or two rows (measured at the 1B shape: a decode step at batch 1 0.819 -> 0.792 ms, at
    batch 2 the same, at batch 4 0.894 -> 0.910, at batch 8 1.003 -> 1.051)."""
    return M * nsplit <= 16 and skinny_merge_ok(M, H, hd, nsplit, dtype, weight)


def skinny_gemm_merged(workspace: torch.Tensor, nsplit: int, M: int, H: int, hd: int, weight, out: torch.Tensor,
                       residual: bool = False, pending: Optional[torch.Tensor] = None, leave: Optional[NormSpec] = None):
    """``attn . weight^T`` where ``attn`` [M, H*hd] is still in the pieces that an attention kernel
    left in ``workspace`` for ``nsplit`` key runs (float32: outputs [M, H, nsplit, hd], then
    (maximum, sum) pairs [M, H, nsplit, 2]): the runs are merged in the product's prologue, with the
    numbers the merge kernel gives.  ``out`` as for :func:`skinny_gemm`, with ``residual`` the
    float32 residual stream (and ``pending`` what it has not received yet)."""
    rows, tiles = _rows_and_tiles(weight)
    N = rows.shape[0]
    dtype = rows.dtype
    if not skinny_merge_ok(M, H, hd, nsplit, dtype, weight):
        raise KernelError(f"the merging prologue does not take M={M}, {H} heads of {hd}, {nsplit} runs in {dtype}")
    _gpu(rows, "weight", dtype, (N, H * hd))
    need = M * H * nsplit * (hd + 2)
    _gpu(workspace, "workspace", torch.float32)
    if not (workspace.numel() >= need):
        raise KernelError(f"attention workspace of {need} floats needed for {nsplit} splits")
    flat = workspace.view(-1)
    part_o, part_ml = flat[: M * H * nsplit * hd], flat[M * H * nsplit * hd: need]
    if residual:
        _gpu(out, "out", torch.float32, (M, N))
    else:
        _gpu(out, "out", dtype, (M, N))
    if pending is not None and not residual:
        raise KernelError("pending addends go with the residual epilogue")
    pend, n_pend = _check_addends(pending, M, N)
    xn = next_w = ss = left = None
    parts = 0
    if leave is not None:
        if not residual:
            raise KernelError("only a product onto the residual stream leaves the next norm's input behind")
        _gpu(leave.weight, "next norm weight", torch.float32, (N,))
        parts = (N + 15) // 16
        xn = torch.empty(M, N, dtype=dtype, device=out.device)
        ss = torch.empty(M, parts, dtype=torch.float32, device=out.device)
        next_w, left = leave.weight, ScaledInput(xn, ss, leave)
    _check(skinny_lib().ni_skinny_gemm_merged(_ptr(part_o), _ptr(part_ml), nsplit, H, hd, _ptr(tiles), _ptr(out), M, N,
                                              3 if residual else 0, dtype_code(dtype), _ptr(pend), n_pend,
                                              _ptr(xn), _ptr(next_w), _ptr(ss), parts, _stream()),
           "skinny_gemm_merged")
    return left if left is not None else out


def qkv_rope_ok(M: int, K: int, hd: int, rotary_dim: int, dtype: torch.dtype) -> bool:
    """Whether the product with a stacked [q; k; v] matrix can rotate and store in its epilogue:
    few rows, a head size that splits into pairs of 16-wide tiles, the whole head rotated."""
    return skinny_ok(M, K, dtype) and hd % 32 == 0 and rotary_dim == hd


def qkv_rope_wins(M: int, K: int, dtype: torch.dtype) -> bool:
    """Whether that fused product is also faster than the library's product and the rotation kernel behind it.
    In bfloat16 always (17 to 64 rows of the 1B / 3B / 8B shapes: 7.2 : 12.9, 13.0 : 16.5, 20.7 : 21.8 us at 64 rows).
    In float32 for rows of up to 2,048 elements, and for up to 16 rows of 4,096 or more: the 3B shape's
    [5120, 3072] takes 29.5 : 22.4 at 8 rows and 41.2 : 33.1 at 64 (a float32 decode step of that shape at batch 8:
    4.72 ms fused, 4.62 with the library), the 8B shape's [6144, 4096] 28.1 : 27.9 and 56.2 : 43.1 (a step at batch 8:
    7.91 ms fused, 8.13 with the library; at batch 64 the library gains)."""
    return dtype != torch.float32 or K <= 2048 or (M <= SKINNY_BEST_ROWS and K >= 4096)


def skinny_qkv_rope(x, w_qkv, positions: torch.Tensor, cos: torch.Tensor,
                    sin: torch.Tensor, slot_mapping: Optional[torch.Tensor], kpool: Optional[torch.Tensor],
                    vpool: Optional[torch.Tensor], H: int, KVH: int, hd: int) -> torch.Tensor:
    """``x . w_qkv^T`` for few rows with rotation and cache write fused in: returns the rotated
    queries [M, H*hd]; rotated keys and plain values go straight into the pools at ``slot_mapping``.
    ``x`` may be a :class:`NormedInput`."""
    normed = isinstance(x, NormedInput)
    M, Kd = x.shape
    dtype = x.dtype
    rows, tiles = _rows_and_tiles(w_qkv)
    ss, parts, eps = None, 0, 0.0
    if isinstance(x, ScaledInput):
        if tiles is None:
            raise KernelError("a scaled input goes into a product with a re-tiled matrix")
        x, ss, parts, eps = _scaled_args(x, M, Kd)
    _gpu(rows, "w_qkv", dtype, ((H + 2 * KVH) * hd, Kd))
    if not (qkv_rope_ok(M, Kd, hd, 2 * cos.shape[1], dtype)):
        raise KernelError(f"skinny_qkv_rope does not take M={M}, K={Kd}, hd={hd}")
    _gpu(positions, "positions", torch.int32, (M,))
    _gpu(cos, "cos", torch.float32)
    _gpu(sin, "sin", torch.float32, cos.shape)
    page_size = 1
    if slot_mapping is not None:
        _gpu(slot_mapping, "slot_mapping", torch.int32, (M,))
        _gpu(kpool, "kpool", dtype)
        _gpu(vpool, "vpool", dtype, kpool.shape)
        if not (kpool.dim() == 4 and kpool.shape[1] == KVH and kpool.shape[3] == hd):
            raise KernelError(f"pool must be [pages, {KVH}, page_size, {hd}], is {tuple(kpool.shape)}")
        page_size = kpool.shape[2]
    pend, n_pend = None, 0
    if normed:
        pend, n_pend = _check_addends(x.pending, M, Kd)
        if not (norm_prologue_ok(M, Kd, dtype, w_qkv, min(n_pend, prologue_addends()))) or n_pend > prologue_addends():
            raise KernelError(f"the normalising prologue does not take M={M}, K={Kd} in {dtype} with {n_pend} addends")
        _check_normed(x, Kd)
        x_ptr, h_ptr, nw_ptr, eps = None, _ptr(x.h), _ptr(x.weight), x.eps
        device = x.h.device
    else:
        _gpu(x, "x")
        x_ptr, h_ptr, nw_ptr = _ptr(x), None, None
        device = x.device
    q = torch.empty(M, H * hd, dtype=dtype, device=device)
    _check(skinny_lib().ni_skinny_qkv_rope(x_ptr, h_ptr, nw_ptr, ctypes.c_float(eps), _ptr(rows if tiles is None else tiles),
                                           _ptr(q), _ptr(positions), _ptr(cos), _ptr(sin), _ptr(slot_mapping), _ptr(kpool),
                                           _ptr(vpool), M, Kd, H, KVH, hd, page_size, 0 if tiles is None else 1,
                                           dtype_code(dtype), _ptr(pend), n_pend, _ptr(ss), parts, _stream()), "skinny_qkv_rope")
    return q


def linear(x, weight, out_dtype: Optional[torch.dtype] = None, residual: Optional[torch.Tensor] = None,
           pending: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None, leave: Optional[NormSpec] = None):
    """``x . weight^T`` with ``weight`` stored [out, in].  Few rows go to the hand-written skinny
    product; many rows to the library (rocBLAS/hipBLASLt), where float32 inputs are multiplied in
    true float32 (the reduced-precision matrix modes of the library are switched off at import).
    ``out_dtype`` float32 keeps the float32 accumulators of a bfloat16 product.  ``x`` may be a
    :class:`NormedInput` where :func:`norm_prologue_ok` holds.  With ``residual`` (the float32
    residual stream, where :func:`residual_epilogue_ok` holds) the product is added into it and
    nothing is returned, or (17 to 64 rows on a matrix of few tiles, :func:`skinny_ksplit`) it is
    returned as float32 addends [S, M, N] that the next norm adds to the stream.  ``pending``: addends
    that ``residual`` has not received yet and that the product brings in with it (where
    :func:`residual_takes_addends` holds).  ``out``: where a plain product is to be written ([M, N] of the
    output type) instead of a new tensor.  ``leave`` (with ``residual``, where :func:`leaves_scaled_ok`
    holds; ignored elsewhere): the norm that stands behind the stream; the product then runs whole and
    returns a :class:`ScaledInput` for that norm.  ``x`` may itself be a :class:`ScaledInput` where
    :func:`takes_scaled_ok` holds."""
    rows, _ = _rows_and_tiles(weight)
    if out is not None and (isinstance(x, (NormedInput, ScaledInput)) or residual is not None):
        raise KernelError("out= goes with a plain product")
    if isinstance(x, ScaledInput):
        if residual is not None or not takes_scaled_ok(x.shape[0], x.shape[1], x.dtype, weight):
            raise KernelError("this product cannot take a scaled input")
        y = torch.empty(x.shape[0], rows.shape[0], dtype=out_dtype or x.dtype, device=x.device)
        return skinny_gemm(x, weight, y)
    if isinstance(x, NormedInput):
        if not (residual is None):
            raise KernelError("a normed input and a residual output in one product are not compiled")
        out = torch.empty(x.shape[0], rows.shape[0], dtype=x.dtype, device=x.device)
        return skinny_gemm(x, weight, out)
    if not (x.is_cuda and rows.is_cuda):
        raise KernelError("linear needs GPU tensors")
    if not (x.dtype == rows.dtype):
        raise KernelError(f"linear: activation {x.dtype} and weight {rows.dtype} differ")
    if not (x.dim() == 2 and x.shape[1] == rows.shape[1]):
        raise KernelError(f"linear: {tuple(x.shape)} x {tuple(rows.shape)}^T")
    if residual is not None:
        if not (residual_epilogue_ok(x.shape[0], x.shape[1], x.dtype, weight)):
            raise KernelError("the residual epilogue does not take this product")
        if leave is not None and leaves_scaled_ok(x.shape[0], x.shape[1], x.dtype, weight):
            if pending is not None and x.shape[0] > SKINNY_BEST_ROWS:
                raise KernelError("this product cannot bring the residual stream's pending addends in")
            return skinny_gemm(x, weight, residual, residual=True, pending=pending, leave=leave)
        if pending is not None and not residual_takes_addends(x.shape[0], x.shape[1], x.dtype, weight):
            raise KernelError("this product cannot bring the residual stream's pending addends in")
        shares, per = skinny_ksplit(x.shape[0], x.shape[1], x.dtype, weight)
        if shares > 1:
            return skinny_gemm_ksplit(x, weight, shares, per)      # addends for the next norm
        skinny_gemm(x, weight, residual, residual=True, pending=pending)
        return None
    if pending is not None:
        raise KernelError("pending addends go with a residual output")
    out_dtype = out_dtype or x.dtype
    if out is not None:
        _gpu(out, "out", out_dtype, (x.shape[0], rows.shape[0]))
    if skinny_wins(x.shape[0], x.shape[1], x.dtype, weight):
        if out is None:
            out = torch.empty(x.shape[0], rows.shape[0], dtype=out_dtype, device=x.device)
        return skinny_gemm(x, weight, out)
    rows_t = weight.rows_t if isinstance(weight, Weight) else rows.t()
    global _library_calls
    _library_calls += 1
    if out_dtype != x.dtype:
        return torch.mm(x, rows_t, out_dtype=out_dtype) if out is None else torch.mm(x, rows_t, out_dtype=out_dtype, out=out)
    return torch.mm(x, rows_t) if out is None else torch.mm(x, rows_t, out=out)


def swiglu_takes_scaled(M: int, K: int, dtype: torch.dtype, weight_gate_up) -> bool:
    """Whether :func:`linear_swiglu` can take a :class:`ScaledInput` of M rows: the fused skinny product on a
    re-tiled stacked matrix whose halves start on tile boundaries."""
    return takes_scaled_ok(M, K, dtype, weight_gate_up) and (weight_gate_up.shape[0] // 2) % 16 == 0


def linear_swiglu(x, weight_gate_up) -> torch.Tensor:
    """``silu(x . Wg^T) * (x . Wu^T)`` for the stacked matrix [Wg; Wu]: fused into the product for
    few rows, product then the SwiGLU kernel for many.  ``x`` may be a :class:`NormedInput`, or a
    :class:`ScaledInput` where :func:`swiglu_takes_scaled` holds."""
    inter = weight_gate_up.shape[0] // 2
    out = torch.empty(x.shape[0], inter, dtype=x.dtype, device=x.device)
    if isinstance(x, ScaledInput) and not swiglu_takes_scaled(x.shape[0], x.shape[1], x.dtype, weight_gate_up):
        raise KernelError("this product cannot take a scaled input")
    # (past 16 rows only a matrix whose halves start on tile boundaries is streamed re-tiled)
    if isinstance(x, NormedInput) or (skinny_wins(x.shape[0], x.shape[1], x.dtype, weight_gate_up)
                                      and (x.shape[0] <= SKINNY_BEST_ROWS or inter % 16 == 0)):
        return skinny_gemm(x, weight_gate_up, out, swiglu=True)
    global _library_calls
    _library_calls += 1
    rows_t = weight_gate_up.rows_t if isinstance(weight_gate_up, Weight) else weight_gate_up.t()
    return swiglu(torch.mm(x, rows_t), out)


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible: nanoinfer_amd runs on an MI355X only and has no CPU path")
    return torch.device("cuda", torch.cuda.current_device())


torch.backends.cuda.matmul.allow_tf32 = False
torch.backends.cudnn.allow_tf32 = False
