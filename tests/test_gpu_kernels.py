"""Each HIP kernel alone against its plain reference, at sizes other than the engine's tests use:
widths and vocabularies that are no power of two, head sizes in steps of 16, odd page sizes."""
import math
import random

import numpy as np
import pytest
import torch

import plain_llama as P

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# kernels do float32 arithmetic on exactly the given inputs; what is left is summation order
# (float32) plus the rounding of the stored result (bfloat16: 2^-9 relative)
KTOL = {"float32": 3e-6, "bfloat16": 6e-3}


def dev(t, dtype=None):
    return t.to("cuda", dtype) if dtype is not None else t.to("cuda")


def rel(got, want):
    return float((got.double().cpu() - want.double()).abs().max() / max(1e-30, float(want.double().abs().max())))


@pytest.fixture(scope="module")
def K():
    from nanoinfer_amd import kernels
    return kernels


def test_missing_gpu_tensor_is_refused(K):
    with pytest.raises(K.KernelError):
        K.embedding(torch.zeros(2, dtype=torch.int32), torch.zeros(4, 4), torch.zeros(2, 4))
    with pytest.raises(Exception) as e:
        K.attention_lib(40)                       # not a multiple of 16: refused with a reason, never run
    assert "multiple of 16" in str(e.value)
    with pytest.raises(Exception):
        K.attention_lib(272)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_weights_kernel_gives_the_bits_of_the_host_routine(K, dtype):
    """Every element is a function of (key, index): the kernel and numpy agree bit for bit, at
    any start (also beyond 32 bits) and for mean and deviation of both kinds of tensor."""
    from nanoinfer_amd.weights import random_init as R
    for name, start, count, mean, std in (("model.embed_tokens.weight", 0, 300001, 0.0, 0.02),
                                          ("model.norm.weight", 12345, 70000, 1.0, 0.05),
                                          ("x", (1 << 35) + 7, 4099, -3.0, 2.5), ("y", 0, 1, 0.0, 1.0)):
        key = R.tensor_key(5, name)
        want = R.normal_cpu(key, start, count, mean, std, DT[dtype])
        got = K.random_normal(torch.empty(count, dtype=DT[dtype], device="cuda"), key, start, mean, std).cpu()
        assert torch.equal(got.view(torch.int16 if dtype == "bfloat16" else torch.int32),
                           want.view(torch.int16 if dtype == "bfloat16" else torch.int32)), (name, start)
    with pytest.raises(K.KernelError):
        K.random_normal(torch.empty(2, 2, device="cuda"), 1, 0, 0.0, 1.0)


def test_large_tensors_of_a_random_model_are_made_on_the_gpu_with_the_same_bits(tmp_path, monkeypatch):
    from nanoinfer_amd.weights import random_init as R
    from nanoinfer_amd.weights.loader import make_random_model
    from tiny_configs import TINY_B
    cpu = make_random_model(str(tmp_path / "cpu"), TINY_B, seed=8, dtype="bfloat16", device=None)
    monkeypatch.setattr(R, "GPU_WORTH_IT", 1000)         # now every matrix goes through the kernel
    monkeypatch.setattr(R, "PIECE", 50000)
    made = []
    original = R.normal_gpu
    monkeypatch.setattr(R, "normal_gpu", lambda *a: (made.append(a[2]), original(*a))[1])
    gpu = make_random_model(str(tmp_path / "gpu"), TINY_B, seed=8, dtype="bfloat16")
    assert made and max(made) == 50000
    assert open(str(tmp_path / "cpu" / "model.safetensors"), "rb").read() == \
        open(str(tmp_path / "gpu" / "model.safetensors"), "rb").read()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding(K, dtype):
    g = torch.Generator().manual_seed(0)
    table = torch.randn(1003, 70, generator=g).to(DT[dtype])
    ids = torch.randint(0, 1003, (37,), generator=g).to(torch.int32)
    out = K.embedding(dev(ids), dev(table), torch.empty(37, 70, device="cuda"))
    assert torch.equal(out.cpu(), P.embedding(table.float(), ids.tolist()).float())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [1, 50, 257, 2048, 4100])
def test_add_rmsnorm(K, dtype, d):
    g = torch.Generator().manual_seed(d)
    T = 9
    h = torch.randn(T, d, generator=g) * 3
    pending = torch.randn(T, d, generator=g).to(DT[dtype])
    w = 1 + 0.1 * torch.randn(d, generator=g)
    eps = 3e-6
    hd, out = dev(h.clone()), torch.empty(T, d, device="cuda", dtype=DT[dtype])
    K.add_rmsnorm(hd, dev(pending), dev(w), eps, out)
    total = h.double() + pending.double()
    assert rel(hd, total) < 1e-6                                     # the residual stream moved on, in float32
    assert rel(out, P.rmsnorm(total, w, eps)) < KTOL[dtype]
    # reference vector: [1..d], weight 1 (test/test_op/test_layer_rmsnorm.cpp:112-136)
    x = torch.arange(1, d + 1, dtype=torch.float32)[None]
    out1 = K.add_rmsnorm(dev(x.clone()), None, dev(torch.ones(d)), 1e-5, torch.empty(1, d, device="cuda", dtype=DT[dtype]))
    assert rel(out1, x.double() / math.sqrt(float((x.double() ** 2).mean()) + 1e-5)) < KTOL[dtype]
    # gathered rows leave h alone and may repeat a row
    rows = torch.tensor([4, 0, 4, 8], dtype=torch.int32)
    hd2 = dev(h.clone())
    out2 = K.add_rmsnorm(hd2, dev(pending), dev(w), eps, torch.empty(4, d, device="cuda", dtype=DT[dtype]), dev(rows))
    assert torch.equal(hd2.cpu(), h)
    assert rel(out2, P.rmsnorm(total[rows.long()], w, eps)) < KTOL[dtype]
    # five float32 addends (the shares of a product cut along K), added in their order
    shares = torch.randn(5, T, d, generator=g)
    hd3 = dev(h.clone())
    out3 = K.add_rmsnorm(hd3, dev(shares), dev(w), eps, torch.empty(T, d, device="cuda", dtype=DT[dtype]))
    in_order = h.clone()
    for a in range(5):
        in_order += shares[a]
    assert torch.equal(hd3.cpu(), in_order)                          # bit for bit: the same additions in the same order
    assert rel(out3, P.rmsnorm(in_order.double(), w, eps)) < KTOL[dtype]


def test_rope_table_holds_the_sines_of_position_times_frequency(K):
    """The table against numbers: cos and sin of pos * f in float64, for frequencies that come from
    nowhere but this test (a geometric run, and the worked llama3 numbers of tests/rope_literals.py)."""
    from rope_literals import CASES
    runs = [np.array([1.0 / 3.7 ** p for p in range(24)], dtype=np.float32)]
    runs += [np.array([value for _, value in pairs.values()], dtype=np.float32) for _, _, _, pairs in CASES]
    for inv in runs:
        n = 3000
        cos, sin = K.rope_table(dev(torch.from_numpy(inv)), n)
        assert cos.shape == sin.shape == (n, len(inv))
        angle = (np.arange(n, dtype=np.float32)[:, None] * inv[None, :]).astype(np.float64)     # the product is float32
        assert float((sin.double().cpu() - torch.from_numpy(np.sin(angle))).abs().max()) < 2e-6
        assert float((cos.double().cpu() - torch.from_numpy(np.cos(angle))).abs().max()) < 2e-6
    assert bool((sin[0] == 0).all()) and bool((cos[0] == 1).all())


def plain_rotate_half(x, sin, cos, rot):
    """[T, heads, hd] with pairs (j, j + rot/2) inside the first rot dims."""
    half = rot // 2
    x = x.double()
    out = x.clone()
    s, c = sin[:, None, :], cos[:, None, :]
    out[..., :half] = x[..., :half] * c - x[..., half:rot] * s
    out[..., half:rot] = x[..., :half] * s + x[..., half:rot] * c
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,KVH,hd,rot,ps", [(4, 2, 16, 16, 4), (6, 1, 32, 32, 8), (5, 5, 48, 24, 5), (8, 2, 128, 128, 16),
                                               (3, 3, 64, 32, 8), (2, 1, 80, 48, 4)])
def test_rope_and_cache_write(K, dtype, H, KVH, hd, rot, ps):
    g = torch.Generator().manual_seed(hd)
    T, pages = 11, 9
    qkv = torch.randn(T, (H + 2 * KVH) * hd, generator=g).to(DT[dtype])
    positions = torch.tensor([0, 1, 2, 3, 40, 41, 7, 300, 301, 302, 5], dtype=torch.int32)
    inv = P.rope_frequencies(rot, 10000.0, None)
    cos, sin = K.rope_table(dev(torch.from_numpy(inv)), 512)
    slots = torch.tensor(random.Random(0).sample(range(pages * ps), T), dtype=torch.int32)
    kpool = torch.full((pages, KVH, ps, hd), 9.0, dtype=DT[dtype], device="cuda")
    vpool = torch.full((pages, KVH, ps, hd), 9.0, dtype=DT[dtype], device="cuda")
    buf = dev(qkv.clone())
    K.rope_kv_write(buf, dev(positions), cos, sin, dev(slots), kpool, vpool, H, KVH, hd)
    s, c = P.rope_tables(positions.tolist(), inv)
    q_ref = plain_rotate_half(qkv[:, :H * hd].reshape(T, H, hd), s, c, rot)
    k_ref = plain_rotate_half(qkv[:, H * hd:(H + KVH) * hd].reshape(T, KVH, hd), s, c, rot)
    v_ref = qkv[:, (H + KVH) * hd:].reshape(T, KVH, hd).double()
    assert rel(buf[:, :H * hd].reshape(T, H, hd), q_ref) < KTOL[dtype]
    assert torch.equal(buf[:, H * hd:].cpu(), qkv[:, H * hd:])                       # k and v columns are left as they were
    kp, vp = kpool.cpu(), vpool.cpu()
    touched = torch.zeros(pages, ps, dtype=torch.bool)
    for t in range(T):
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        touched[page, off] = True
        assert rel(kp[page, :, off, :], k_ref[t]) < KTOL[dtype]
        assert torch.equal(vp[page, :, off, :].double(), v_ref[t])
    assert bool((kp.float()[~touched[:, None, :].expand(pages, KVH, ps)] == 9.0).all())   # nothing else was written
    # the flat address is ((page * KVH + head) * page_size + slot) * hd, the pool's declared order
    t0 = 3
    page, off = int(slots[t0]) // ps, int(slots[t0]) % ps
    flat = vpool.view(-1)
    addr = ((page * KVH + (KVH - 1)) * ps + off) * hd
    assert torch.equal(flat[addr:addr + hd].cpu().double(), v_ref[t0, KVH - 1])


def test_rope_quarter_turn_vector(K):
    # test/test_cuda_kernel/test_rope_kernel.cpp:20-118 in this engine's pairing: sin 1, cos 0 turns (2, 2) into (-2, 2)
    qkv = torch.full((1, 3 * 16), 2.0, device="cuda")
    cos = torch.zeros(2, 8, device="cuda")
    sin = torch.ones(2, 8, device="cuda")
    K.rope_kv_write(qkv, dev(torch.tensor([1], dtype=torch.int32)), cos, sin, None, None, None, 1, 1, 16)
    assert torch.equal(qkv[0, :8].cpu(), torch.full((8,), -2.0)) and torch.equal(qkv[0, 8:16].cpu(), torch.full((8,), 2.0))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_swiglu(K, dtype):
    g = torch.Generator().manual_seed(1)
    for width in (137, 136, 140, 4096):          # one element at a time, 16-byte vectors of either type, a long row
        gu = (torch.randn(7, 2 * width, generator=g) * 3).to(DT[dtype])
        gu[0, :4] = torch.tensor([-100.0, 100.0, -30.0, 0.0]).to(DT[dtype])     # the exponential overflows and underflows
        out = K.swiglu(dev(gu), torch.empty(7, width, device="cuda", dtype=DT[dtype]))
        assert bool(torch.isfinite(out).all())
        assert rel(out, P.swiglu(gu[:, :width].double(), gu[:, width:].double())) < KTOL[dtype], width
    one = K.swiglu(torch.ones(1, 2, device="cuda"), torch.empty(1, 1, device="cuda"))
    assert abs(float(one) - 0.7310586) < 1e-6                          # test/test_op/test_layer_swiglu.cpp:65-108


# ------------------------------------------------------------------ attention over pages

def paged_case(K, dtype, H, KVH, hd, ps, lens, q_lens, window, seed, nsplit, boost=None, kernel="token", blocks=1):
    """Sequences of ``lens`` keys each; the last ``q_lens`` of each are this step's queries.  The
    cache is filled through a shuffled block table; everything else in the pools is NaN so that a
    read outside a sequence's own keys poisons the result."""
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    pages_per = [-(-n // ps) for n in lens]
    total_pages = sum(pages_per) + 3
    ids = list(range(total_pages))
    rng.shuffle(ids)
    width = max(pages_per)
    table = torch.full((B, width), -1, dtype=torch.int32)
    kpool = torch.full((total_pages, KVH, ps, hd), float("nan"))
    vpool = torch.full((total_pages, KVH, ps, hd), float("nan"))
    ks, vs, qs, seq_of, positions = [], [], [], [], []
    at = 0
    for b, n in enumerate(lens):
        k = torch.randn(n, KVH, hd, generator=g).to(DT[dtype]).float()
        v = torch.randn(n, KVH, hd, generator=g).to(DT[dtype]).float()
        q = torch.randn(n, H, hd, generator=g).to(DT[dtype]).float()
        if boost is not None:
            bb, key_at, query_at, factor = boost
            if bb == b:
                # the inputs stay exactly representable in the compute type
                k[key_at] = (k[key_at] * factor).to(DT[dtype]).float()
                q[query_at] = (k[key_at].repeat_interleave(H // KVH, 0) / factor * 4).to(DT[dtype]).float()
        for p in range(pages_per[b]):
            table[b, p] = ids[at]
            lo, hi = p * ps, min(n, (p + 1) * ps)
            kpool[ids[at], :, :hi - lo] = k[lo:hi].transpose(0, 1)
            vpool[ids[at], :, :hi - lo] = v[lo:hi].transpose(0, 1)
            at += 1
        ks.append(k), vs.append(v), qs.append(q)
        if window:
            # keys that the window of the step's first query has passed: their pages may have been given
            # back and hold anything; here NaN, so that a kernel that as much as multiplies them by zero shows
            for i in range(max(0, n - q_lens[b] + 1 - window)):
                kpool[int(table[b, i // ps]), :, i % ps] = float("nan")
                vpool[int(table[b, i // ps]), :, i % ps] = float("nan")
        for i in range(n - q_lens[b], n):
            seq_of.append(b), positions.append(i)
    T = len(seq_of)
    qkv = torch.zeros(T, (H + 2 * KVH) * hd)
    row = 0
    for b, n in enumerate(lens):
        for i in range(n - q_lens[b], n):
            qkv[row, :H * hd] = qs[b][i].reshape(-1)
            row += 1
    out = torch.empty(T, H * hd, device="cuda", dtype=DT[dtype])
    ws = torch.empty(max(1, T * H * nsplit * (hd + 2)), device="cuda") if nsplit > 1 else None
    if kernel == "mfma":
        starts = [sum(q_lens[:b]) for b in range(B)]
        tile_tokens = K.mfma_tile_tokens(hd, H // KVH, dtype=DT[dtype]) * blocks      # a wavefront owns `blocks` blocks of 16 rows
        flat = K.build_q_tiles(starts, q_lens, lens, tile_tokens)
        tiles = dev(torch.tensor(flat, dtype=torch.int32).view(-1, 4))
        K.mfma_attention(dev(qkv, DT[dtype]), dev(kpool, DT[dtype]), dev(vpool, DT[dtype]), dev(table), tiles, out,
                         H, KVH, hd, 1.0 / math.sqrt(hd), window, nsplit, ws, tile_tokens)
    else:
        fn = {"token": K.token_attention, "mfma_token": K.mfma_token_attention}[kernel]
        fn(dev(qkv, DT[dtype]), dev(kpool, DT[dtype]), dev(vpool, DT[dtype]), dev(table),
           dev(torch.tensor(seq_of, dtype=torch.int32)), dev(torch.tensor(positions, dtype=torch.int32)),
           out, H, KVH, hd, 1.0 / math.sqrt(hd), window, nsplit, ws)
    want = torch.cat([P.causal_attention(qs[b], ks[b], vs[b], range(n), window=window)[n - q_lens[b]:].reshape(q_lens[b], H * hd)
                      for b, n in enumerate(lens)])
    return out, want, (qs, ks, vs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,KVH,hd,ps", [(4, 2, 16, 16), (6, 1, 32, 8), (5, 5, 48, 5), (32, 8, 64, 16), (3, 3, 80, 16),
                                         (8, 2, 96, 4), (2, 1, 112, 16), (16, 2, 128, 16), (2, 2, 256, 16)])
def test_attention_head_sizes_and_groups(K, dtype, H, KVH, hd, ps):
    lens, q_lens = [1, 37, 130, 64], [1, 37, 2, 1]
    for nsplit, kernel in ((1, "token"), (3, "token")):
        out, want, _ = paged_case(K, dtype, H, KVH, hd, ps, lens, q_lens, None, hd + nsplit, nsplit, kernel=kernel)
        assert not torch.isnan(out).any(), "a key outside the sequence's own pages was read"
        assert rel(out, want) < KTOL[dtype], (H, KVH, hd, ps, nsplit, kernel)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_window_edges(K, dtype):
    for window in (1, 7, 16, 33):
        out, want, _ = paged_case(K, dtype, 4, 2, 32, 8, [50, 9, 33], [50, 9, 2], window, window, 1)
        assert not torch.isnan(out).any()
        assert rel(out, want) < KTOL[dtype], window
    out, want, _ = paged_case(K, dtype, 4, 2, 32, 8, [300], [1], 200, 3, 4)
    assert rel(out, want) < KTOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_finds_a_far_key_among_hundreds(K, dtype):
    """One early key is made to match the last query: the output must be that key's value, which
    random keys would never show.  Key 37 sits in the middle of a page, key 16 on a page's first
    slot, key 15 on a page's last; splits cut the range in other places."""
    for key_at in (37, 16, 15, 0, 699):
        for nsplit in (1, 5):
            out, want, (qs, ks, vs) = paged_case(K, dtype, 8, 2, 64, 16, [700], [1], None, 9, nsplit,
                                                 boost=(0, key_at, 699, 6.0))
            assert rel(out, want) < KTOL[dtype]
            got = out.double().cpu().reshape(8, 64)
            expect = vs[0][key_at].double().repeat_interleave(4, 0)
            assert float((got - expect).abs().max()) < 0.05, key_at     # the one key took all the weight


@pytest.mark.parametrize("kernel", ["token", "mfma", "mfma_token"])
def test_attention_block_table_longer_than_one_segment(K, kernel):
    """The kernels keep 1,024 entries of a block table in LDS at a time.  With pages of one or
    three slots a range of 2,500 keys needs several such segments; a boosted key is placed in the
    first, at the seam and in the last, so that a segment read through the wrong entries shows."""
    n = 2500
    for i, (ps, key_at) in enumerate(((1, 5), (1, 1023), (1, 1024), (1, 2499), (3, 3071 % n), (3, 1))):
        out, want, (qs, ks, vs) = paged_case(K, "bfloat16", 4, 2, 64, ps, [n, 40], [3, 2], None, ps + key_at, 1,
                                             boost=(0, key_at, n - 1, 6.0), kernel=kernel,
                                             blocks=(1, 2)[i % 2] if kernel == "mfma" else 1)
        assert not torch.isnan(out).any()
        assert rel(out, want) < KTOL["bfloat16"], (ps, key_at)
        got = out.double().cpu()[2].reshape(4, 64)
        expect = vs[0][key_at].double().repeat_interleave(2, 0)
        assert float((got - expect).abs().max()) < 0.05, (ps, key_at)


# ---- the matrix-core kernel for prompt portions (bfloat16)

@pytest.mark.parametrize("H,KVH,hd,ps", [(4, 2, 32, 8), (6, 1, 32, 8), (32, 8, 64, 16), (16, 2, 128, 16), (2, 2, 256, 16),
                                         (3, 3, 96, 4), (32, 1, 64, 16), (5, 5, 64, 5), (12, 4, 64, 16),
                                         # odd multiples of 16: the last 16 dims of a head go through a product of their own
                                         (4, 2, 16, 16), (5, 5, 48, 5), (6, 2, 80, 16), (2, 1, 112, 16), (16, 1, 144, 8), (3, 3, 240, 16)])
def test_mfma_attention_head_sizes_and_groups(K, H, KVH, hd, ps):
    # whole prompts, portions that start in the middle of a sequence, single tokens beside them, tile edges
    lens, q_lens = [1, 37, 130, 64, 200, 17], [1, 37, 2, 1, 77, 16]
    for blocks in (1, 2, 4):
        if blocks > mfma_max_blocks(K, hd):
            with pytest.raises(K.KernelError, match="no tiles of"):
                paged_case(K, "bfloat16", H, KVH, hd, ps, lens, q_lens, None, hd + H, 1, kernel="mfma", blocks=blocks)
            continue
        for nsplit in (1, 3):
            out, want, _ = paged_case(K, "bfloat16", H, KVH, hd, ps, lens, q_lens, None, hd + H, nsplit, kernel="mfma",
                                      blocks=blocks)
            assert not torch.isnan(out).any(), "a key outside the sequence's own pages took part"
            assert rel(out, want) < KTOL["bfloat16"], (H, KVH, hd, ps, nsplit, blocks)


def mfma_max_blocks(K, hd):
    return int(K.attention_mfma_lib(hd).ni_mfma_attention_max_blocks())


def test_mfma_tile_size_and_splits_follow_the_step(K):
    # 32 query heads on 8 kv heads, head size 64: tiles of 16 tokens, or of 32 where that leaves 384 tiles (one and a
    # half for every compute unit)
    assert K.mfma_tile_tokens(64, 4) == 16
    assert K.mfma_tile_tokens(64, 4, 1535, 8) == 16 and K.mfma_tile_tokens(64, 4, 1536, 8) == 32
    assert K.mfma_tile_tokens(64, 4, 2048, 8) == 32
    assert K.mfma_tile_tokens(64, 4, 4096, 8) == 32
    assert K.mfma_tile_tokens(64, 4, 100, 8) == 16
    assert K.mfma_tile_tokens(128, 4, 8192, 8) == 16        # head size 128 leaves registers for one block only
    assert K.mfma_tile_tokens(256, 1, 8192, 8) == 64        # one head a tile: 4 wavefronts x 16 tokens, one block
    # many tiles: runs of 2,048 keys or more; fewer tiles than compute units: runs of 512 or more
    assert K.mfma_splits(128, 8, 4, 2048) == 1
    assert K.mfma_splits(64, 8, 4, 32768) == 1 and K.mfma_splits(63, 8, 4, 32768) == 2     # two tiles a compute unit: uncut
    assert K.mfma_splits(32, 8, 4, 8192) == 4
    assert K.mfma_splits(8, 8, 4, 2048) == 4
    assert K.mfma_splits(8, 8, 4, 300) == 1
    assert K.mfma_splits(1, 1, 1, 10 ** 6) == 16
    # single tokens: a workgroup for every compute unit, then two runs where that evens out the units' load
    assert [K.mfma_token_splits(b, 8, 4, 2170) for b in (1, 8, 16, 32, 33, 48, 56, 64)] == [8, 4, 2, 1, 2, 2, 1, 1]
    assert K.mfma_token_splits(40, 8, 4, 300) == 1 and K.mfma_token_splits(1, 8, 4, 100000) == 32
    # one portion alone far into its sequence: two blocks and runs of 512 keys or more, if that fills the chip
    assert K.mfma_plan(64, 4, 8, 512, 512, 2048) == (32, 4) == K.mfma_plan(64, 4, 8, 512, 512, 1100)
    assert K.mfma_plan(64, 4, 8, 512, 512, 1024) == (16, None)        # the keys before it may be as few as its own
    assert K.mfma_plan(64, 4, 8, 512, 512, 5000) == (32, 4)
    assert K.mfma_plan(64, 4, 8, 1024, 1024, 1024) == (16, None)      # a whole prompt: short and long tiles, paired
    assert K.mfma_plan(64, 4, 8, 2048, 2048, 2048) == (32, None)
    assert K.mfma_plan(64, 4, 8, 4096, 4096, 4096) == (32, None)
    assert K.mfma_plan(64, 4, 8, 512, 300, 2048) == (16, None)        # several portions in the step
    assert K.mfma_plan(128, 4, 8, 512, 512, 2048) == (16, None)       # head size 128 has one block only


@pytest.mark.parametrize("H,KVH,hd,ps", [(4, 2, 32, 8), (6, 1, 32, 8), (32, 8, 64, 16), (16, 2, 128, 16), (2, 2, 256, 16),
                                         (3, 3, 96, 4), (40, 2, 64, 16), (5, 5, 64, 5), (12, 4, 160, 16)])
def test_mfma_token_attention_head_sizes_and_groups(K, H, KVH, hd, ps):
    # the kernel for single tokens: rows are the query heads of a kv head (20 of them: two chunks of 16)
    lens, q_lens = [1, 37, 130, 64, 300, 33], [1, 37, 2, 1, 3, 1]
    for dtype in ("bfloat16", "float32"):
        for nsplit in (1, 3):
            out, want, _ = paged_case(K, dtype, H, KVH, hd, ps, lens, q_lens, None, hd + H, nsplit, kernel="mfma_token")
            assert not torch.isnan(out).any(), "a key outside the sequence's own pages took part"
            assert rel(out, want) < KTOL[dtype], (dtype, H, KVH, hd, ps, nsplit)


@pytest.mark.parametrize("H,KVH,hd,ps", [(4, 2, 16, 16), (5, 5, 48, 5), (3, 3, 80, 16), (2, 1, 112, 16), (24, 8, 128, 16), (34, 2, 64, 8)])
def test_mfma_token_attention_in_float32_at_its_own_head_sizes(K, H, KVH, hd, ps):
    # head sizes in steps of 16, which the bfloat16 kernel does not take; 17 heads a group: two chunks of 16
    lens, q_lens = [1, 37, 130, 64, 300, 33, 17], [1, 37, 2, 1, 3, 1, 1]
    assert K.mfma_token_ok(torch.float32, hd) and K.mfma_token_ok(torch.bfloat16, hd) == (hd % 32 == 0)
    for nsplit in (1, 2, 5):
        out, want, _ = paged_case(K, "float32", H, KVH, hd, ps, lens, q_lens, None, hd + H, nsplit, kernel="mfma_token")
        assert not torch.isnan(out).any(), "a key outside the sequence's own pages took part"
        assert rel(out, want) < KTOL["float32"], (H, KVH, hd, ps, nsplit)


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_mfma_token_attention_window_and_far_key(K, dtype):
    for window in (1, 7, 16, 33, 100):
        out, want, _ = paged_case(K, dtype, 4, 2, 32, 8, [150, 9, 33], [150, 9, 2], window, window, 1, kernel="mfma_token")
        assert not torch.isnan(out).any()
        assert rel(out, want) < KTOL[dtype], window
    for window, nsplit in ((300, 3), (129, 2), (600, 4)):      # windows cut into runs: the first run starts inside a step
        out, want, _ = paged_case(K, dtype, 8, 2, 64, 16, [901, 333], [2, 1], window, window, nsplit, kernel="mfma_token")
        assert not torch.isnan(out).any()
        assert rel(out, want) < KTOL[dtype], window
    for key_at in (37, 16, 15, 0, 31, 32, 127, 128, 698):
        out, want, (qs, ks, vs) = paged_case(K, dtype, 8, 2, 64, 16, [700], [1], None, 9, 1 + key_at % 4,
                                             boost=(0, key_at, 699, 6.0), kernel="mfma_token")
        assert rel(out, want) < KTOL[dtype]
        got = out.double().cpu()[-1].reshape(8, 64)
        expect = vs[0][key_at].double().repeat_interleave(4, 0)
        assert float((got - expect).abs().max()) < 0.05, key_at


@pytest.mark.parametrize("blocks", [1, 2])
def test_mfma_attention_window_and_far_key(K, blocks):
    for window in (1, 7, 16, 33, 100):
        out, want, _ = paged_case(K, "bfloat16", 4, 2, 32, 8, [150, 9, 33], [150, 9, 2], window, window, 1, kernel="mfma",
                                  blocks=blocks)
        assert not torch.isnan(out).any()
        assert rel(out, want) < KTOL["bfloat16"], window
    for key_at in (37, 16, 15, 0, 31, 32, 698):
        # 5 queries, or 90 so that the large tiles are full and the last one is not
        for n_q in (5, 90):
            out, want, (qs, ks, vs) = paged_case(K, "bfloat16", 8, 2, 64, 16, [700], [n_q], None, 9, 1 + key_at % 4,
                                                 boost=(0, key_at, 699, 6.0), kernel="mfma", blocks=blocks)
            assert rel(out, want) < KTOL["bfloat16"]
            got = out.double().cpu()[-1].reshape(8, 64)
            expect = vs[0][key_at].double().repeat_interleave(4, 0)
            assert float((got - expect).abs().max()) < 0.05, key_at
    # a window long enough that whole turns of the step ring lie inside every row's key range (the steps that run
    # without masks), its start and the rows' own positions at their edges; the passed pages hold no finite number
    for window, lens, q_lens in ((400, [900, 40], [90, 40]), (300, [901], [5]), (129, [700, 333], [64, 33]), (600, [777], [1])):
        out, want, _ = paged_case(K, "bfloat16", 8, 2, 64, 16, lens, q_lens, window, window + lens[0], 1, kernel="mfma",
                                  blocks=blocks)
        assert not torch.isnan(out).any()
        assert rel(out, want) < KTOL["bfloat16"], window
    with pytest.raises(Exception):
        K.attention_mfma_lib(40)
    assert K.mfma_token_ok(torch.float32, 48) and not K.mfma_token_ok(torch.bfloat16, 48) and K.mfma_attention_ok(torch.bfloat16, 48)
    assert K.mfma_attention_ok(torch.float32, 48) and not K.mfma_attention_ok(torch.float32, 40) and not K.mfma_attention_ok(torch.bfloat16, 40)
    # the kernel for single tokens is not compiled for the odd multiples of 16: asked all the same, it refuses
    with pytest.raises(K.KernelError):
        K.mfma_token_attention(torch.zeros(1, 8 * 48, device="cuda", dtype=torch.bfloat16), *[None] * 6, 4, 2, 48, 1.0, None, 1)


@pytest.mark.parametrize("hd,blocks", [(16, 1), (16, 2), (48, 1), (48, 2), (80, 1), (112, 1)])
def test_mfma_attention_window_and_far_key_at_odd_multiples_of_16(K, hd, blocks):
    """The bfloat16 kernel for prompt portions at head sizes 16, 48, 80 and 112: windows whose passed pages hold no
    finite number, and one far key that takes all the weight of the last query (a key that differs from its
    neighbours in its last 16 dims only would be lost by a kernel that forgot them: here every dim counts)."""
    for window in (1, 7, 33, 100):
        out, want, _ = paged_case(K, "bfloat16", 4, 2, hd, 8, [150, 9, 33], [150, 9, 2], window, window + hd, 1, kernel="mfma",
                                  blocks=blocks)
        assert not torch.isnan(out).any()
        assert rel(out, want) < KTOL["bfloat16"], window
    for key_at in (37, 16, 0, 31, 32, 698):
        for n_q in (5, 90):
            out, want, (qs, ks, vs) = paged_case(K, "bfloat16", 8, 2, hd, 16, [700], [n_q], None, 9 + hd, 1 + key_at % 4,
                                                 boost=(0, key_at, 699, 6.0 if hd >= 48 else 10.0), kernel="mfma", blocks=blocks)
            assert rel(out, want) < KTOL["bfloat16"]
            got = out.double().cpu()[-1].reshape(8, hd)
            expect = vs[0][key_at].double().repeat_interleave(4, 0)
            assert float((got - expect).abs().max()) < 0.05, key_at
    # the last 16 dims alone decide: two keys that agree everywhere else
    g = torch.Generator().manual_seed(hd)
    n, H, KVH = 64, 2, 1
    k = torch.zeros(n, KVH, hd)
    k[:, 0, hd - 16:] = torch.randn(n, 16, generator=g).to(torch.bfloat16).float()
    v = torch.randn(n, KVH, hd, generator=g).to(torch.bfloat16).float()
    q = torch.zeros(n, H, hd)
    q[:, :, hd - 16:] = (k[:, :, hd - 16:] * 8).to(torch.bfloat16).float()
    kpool, vpool = k.transpose(0, 1)[None].contiguous(), v.transpose(0, 1)[None].contiguous()       # one page of 64 slots
    qkv = torch.zeros(n, (H + 2 * KVH) * hd)
    qkv[:, :H * hd] = q.reshape(n, -1)
    tile_tokens = K.mfma_tile_tokens(hd, H // KVH) * blocks
    tiles = dev(torch.tensor(K.build_q_tiles([0], [n], [n], tile_tokens), dtype=torch.int32).view(-1, 4))
    out = torch.empty(n, H * hd, device="cuda", dtype=torch.bfloat16)
    K.mfma_attention(dev(qkv, torch.bfloat16), dev(kpool, torch.bfloat16), dev(vpool, torch.bfloat16),
                     dev(torch.zeros(1, 1, dtype=torch.int32)), tiles, out, H, KVH, hd, 1.0 / math.sqrt(hd), None, 1, None, tile_tokens)
    want = P.causal_attention(q, k, v, range(n)).reshape(n, H * hd)
    assert rel(out, want) < KTOL["bfloat16"]
    assert float((want - v.double().mean(0).reshape(1, hd).repeat(1, H)).abs().max()) > 0.3      # far from the plain mean of the values


@pytest.mark.parametrize("blocks", [1, 2])
def test_mfma_attention_more_tiles_than_the_chip_holds(K, blocks):
    """A prompt of 4,200 tokens, 16 query heads on 8 kv heads: with tiles of 32 tokens more tiles than the chip holds
    workgroups, dealt out in three rounds (with 64 tokens: two); with 1,100 tokens every tile has a workgroup of its
    own and the upper half of the grid walks the list backwards.  Rows picked from the start, the end and the middle of
    the prompt against the plain formula."""
    H, KVH, hd, ps = 16, 8, 64, 16
    for n in (4200, 1100):
        g = torch.Generator().manual_seed(n + blocks)
        q = torch.randn(n, H, hd, generator=g).bfloat16().float()
        k = torch.randn(n, KVH, hd, generator=g).bfloat16().float()
        v = torch.randn(n, KVH, hd, generator=g).bfloat16().float()
        pages = -(-n // ps)
        order = torch.randperm(pages, generator=g)
        kpool = torch.full((pages + 2, KVH, ps, hd), float("nan"))
        vpool = torch.full((pages + 2, KVH, ps, hd), float("nan"))
        pad = pages * ps - n
        kp = torch.cat([k, torch.zeros(pad, KVH, hd)]).view(pages, ps, KVH, hd).transpose(1, 2)
        vp = torch.cat([v, torch.zeros(pad, KVH, hd)]).view(pages, ps, KVH, hd).transpose(1, 2)
        kpool[order], vpool[order] = kp, vp
        table = order.to(torch.int32).view(1, pages)
        qkv = torch.cat([q.reshape(n, H * hd), torch.zeros(n, 2 * KVH * hd)], dim=1)
        tile_tokens = K.mfma_tile_tokens(hd, H // KVH) * blocks
        tiles = dev(torch.tensor(K.build_q_tiles([0], [n], [n], tile_tokens), dtype=torch.int32).view(-1, 4))
        out = torch.empty(n, H * hd, device="cuda", dtype=torch.bfloat16)
        K.mfma_attention(dev(qkv, torch.bfloat16), dev(kpool, torch.bfloat16), dev(vpool, torch.bfloat16), dev(table), tiles, out,
                         H, KVH, hd, 1.0 / math.sqrt(hd), None, 1, None, tile_tokens)
        got = out.float().cpu().view(n, H, hd)
        assert not torch.isnan(got).any()
        rows = sorted(set([0, 1, 15, 16, 31, 32, 33, 63, 64, 65, n // 2, n // 2 + 17, n - 65, n - 33, n - 2, n - 1]
                          + torch.randint(0, n, (24,), generator=g).tolist()))
        for t in rows:
            for h in (0, 3, H - 1):
                kk, vv = k[:t + 1, h // (H // KVH)].double(), v[:t + 1, h // (H // KVH)].double()
                w = torch.softmax(kk @ q[t, h].double() / math.sqrt(hd), dim=0)
                assert float((got[t, h].double() - w @ vv).abs().max()) < 2e-2, (n, t, h)


# ---- the matrix-core kernel for prompt portions in float32

@pytest.mark.parametrize("H,KVH,hd,ps", [(4, 2, 16, 16), (6, 1, 32, 8), (5, 5, 48, 5), (32, 8, 64, 16), (3, 3, 80, 16),
                                         (8, 2, 96, 4), (2, 1, 112, 16), (16, 2, 128, 16), (2, 2, 256, 16), (32, 1, 64, 16),
                                         (12, 4, 64, 3)])
def test_mfma_attention_float32_head_sizes_and_groups(K, H, KVH, hd, ps):
    # whole prompts, portions that start in the middle of a sequence, single tokens beside them, tile edges
    lens, q_lens = [1, 37, 130, 64, 200, 17], [1, 37, 2, 1, 77, 16]
    for nsplit in (1, 3):
        out, want, _ = paged_case(K, "float32", H, KVH, hd, ps, lens, q_lens, None, hd + H, nsplit, kernel="mfma")
        assert not torch.isnan(out).any(), "a key outside the sequence's own pages took part"
        assert rel(out, want) < KTOL["float32"], (H, KVH, hd, ps, nsplit)
    with pytest.raises(K.KernelError, match="no tiles of"):
        paged_case(K, "float32", H, KVH, hd, ps, lens, q_lens, None, 1, 1, kernel="mfma", blocks=2)


def test_mfma_attention_float32_window_and_far_key(K):
    for window in (1, 7, 16, 33, 100):
        for nsplit in (1, 2):
            out, want, _ = paged_case(K, "float32", 4, 2, 32, 8, [150, 9, 33], [150, 9, 2], window, window, nsplit,
                                      kernel="mfma")
            assert not torch.isnan(out).any()
            assert rel(out, want) < KTOL["float32"], (window, nsplit)
    for key_at in (37, 16, 15, 0, 31, 32, 698):
        for n_q in (5, 90):
            out, want, (qs, ks, vs) = paged_case(K, "float32", 8, 2, 64, 16, [700], [n_q], None, 9, 1 + key_at % 4,
                                                 boost=(0, key_at, 699, 6.0), kernel="mfma")
            assert rel(out, want) < KTOL["float32"]
            got = out.double().cpu()[-1].reshape(8, 64)
            expect = vs[0][key_at].double().repeat_interleave(4, 0)
            assert float((got - expect).abs().max()) < 0.05, key_at


def test_mfma_attention_float32_block_table_longer_than_one_segment(K):
    n = 2500
    for ps, key_at in ((1, 5), (1, 1023), (1, 1024), (1, 2499), (3, 3071 % n), (3, 1)):
        out, want, (qs, ks, vs) = paged_case(K, "float32", 4, 2, 64, ps, [n, 40], [3, 2], None, ps + key_at, 1,
                                             boost=(0, key_at, n - 1, 6.0), kernel="mfma")
        assert not torch.isnan(out).any()
        assert rel(out, want) < KTOL["float32"], (ps, key_at)
        got = out.double().cpu()[2].reshape(4, 64)
        expect = vs[0][key_at].double().repeat_interleave(2, 0)
        assert float((got - expect).abs().max()) < 0.05, (ps, key_at)


def test_attention_uniform_keys_reference_vector(K):
    # test/test_cuda_kernel/test_paged_attention_kernel.cpp:18-84: K = 0.1, V = 0.2, ctx 10, hd 128, 4 heads on 2 -> 0.2
    H, KVH, hd, ps = 4, 2, 128, 16
    kpool = torch.full((2, KVH, ps, hd), 0.1, device="cuda")
    vpool = torch.full((2, KVH, ps, hd), 0.2, device="cuda")
    qkv = torch.full((1, (H + 2 * KVH) * hd), 0.3, device="cuda")
    out = torch.empty(1, H * hd, device="cuda")
    K.token_attention(qkv, kpool, vpool, dev(torch.tensor([[1, 0]], dtype=torch.int32)),
                      dev(torch.tensor([0], dtype=torch.int32)), dev(torch.tensor([9], dtype=torch.int32)), out,
                      H, KVH, hd, 1 / math.sqrt(hd), None, 1)
    assert float((out - 0.2).abs().max()) < 1e-6


# ------------------------------------------------------------------ sampling

def test_argmax_planted_maxima_and_ties(K):
    # test/test_cuda_kernel/test_argmax_kernel.cpp:18-65
    V = 10000
    rows = torch.zeros(6, V)
    for r, at in enumerate((100, 5000, 9999, 0)):
        rows[r, at] = 10.0
    rows[4, 7] = rows[4, 3] = rows[4, 9000] = 2.0          # equal maxima: the lowest index
    rows[5] = -1.0
    rows[5, 4321] = -0.5
    assert K.argmax(dev(rows)).tolist() == [100, 5000, 9999, 0, 3, 4321]
    g = torch.Generator().manual_seed(0)
    big = torch.randn(3, 128256, generator=g)
    assert K.argmax(dev(big)).tolist() == big.argmax(-1).tolist()


def sample_rows(K, logits, temperature, top_k, top_p, penalty, generated, uniform):
    R, V = logits.shape
    pen_ids, pen_off = [], [0]
    for g in generated:
        pen_ids += sorted(set(g))
        pen_off.append(len(pen_ids))
    f32, i32 = torch.float32, torch.int32
    out = torch.empty(R, dtype=i32, device="cuda")
    K.sample(dev(logits), torch.empty(R, V, device="cuda"), dev(torch.tensor(temperature, dtype=f32)),
             dev(torch.tensor(top_k, dtype=i32)), dev(torch.tensor(top_p, dtype=f32)), dev(torch.tensor(penalty, dtype=f32)),
             dev(torch.tensor(pen_ids or [0], dtype=i32)), dev(torch.tensor(pen_off, dtype=i32)),
             dev(torch.tensor(uniform, dtype=f32)), out)
    return out.tolist()


def plain_pick(logits, temperature, top_k, top_p, penalty, generated, u):
    l = logits.double()
    if penalty != 1.0:
        l = P.repetition_penalty(l, generated, penalty)
    if temperature <= 0:
        return P.argmax(l)
    l = P.temperature_scale(l, temperature)
    return P.inverse_cdf(P.filtered_distribution(l, top_k, top_p), u)


@pytest.mark.parametrize("V", [50, 1000, 5003, 40000])
def test_sampling_matches_plain(K, V):
    g = torch.Generator().manual_seed(V)
    rng = random.Random(V)
    cases = []
    for _ in range(48):
        cases.append(dict(temperature=rng.choice([0.0, 0.5, 0.8, 1.0, 1.7]), top_k=rng.choice([0, 0, 1, 5, 40]),
                          top_p=rng.choice([1.0, 1.0, 0.9, 0.5, 0.1]), penalty=rng.choice([1.0, 1.0, 1.3]),
                          generated=[rng.randrange(V) for _ in range(rng.randint(0, 6))],
                          u=(rng.randrange(1, 1 << 20)) / float(1 << 20)))
    logits = torch.randn(len(cases), V, generator=g) * 2.5
    got = sample_rows(K, logits, [c["temperature"] for c in cases], [c["top_k"] for c in cases],
                      [c["top_p"] for c in cases], [c["penalty"] for c in cases], [c["generated"] for c in cases],
                      [c["u"] for c in cases])
    for r, c in enumerate(cases):
        want = plain_pick(logits[r], c["temperature"], c["top_k"], c["top_p"], c["penalty"], c["generated"], c["u"])
        if got[r] != want:
            # a draw that falls within rounding of a boundary of the cumulative distribution may take
            # either neighbour: accept only if u is that close to the boundary between the two
            l = logits[r].double()
            if c["penalty"] != 1.0:
                l = P.repetition_penalty(l, c["generated"], c["penalty"])
            probs = P.filtered_distribution(P.temperature_scale(l, c["temperature"]), c["top_k"], c["top_p"])
            cum = torch.cumsum(probs, 0)
            lo, hi = sorted((got[r], want))
            assert probs[got[r]] > 0 and abs(float(cum[lo]) - c["u"]) < 1e-5, (r, c, got[r], want)


def test_sampling_at_the_family_vocabulary(K):
    # eight rows of 128,256 logits: 32 workgroups share a row
    V = 128256
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(8, V, generator=g) * 3
    opts = [(0.8, 0, 1.0, 1.0), (1.0, 50, 1.0, 1.0), (0.7, 0, 0.9, 1.0), (1.2, 200, 0.5, 1.3), (0.0, 0, 1.0, 1.0),
            (0.0, 0, 1.0, 2.0), (1.5, 1, 1.0, 1.0), (0.9, 1000, 0.99, 1.0)]
    generated = [[], [], [5], [int(logits[3].argmax()), 7, 7], [], [int(logits[5].argmax())], [], []]
    us = [0.37, 0.81, 0.05, 0.66, 0.5, 0.5, 0.93, 0.999]
    got = sample_rows(K, logits, [o[0] for o in opts], [o[1] for o in opts], [o[2] for o in opts], [o[3] for o in opts], generated, us)
    for r, (t, k, p, pen) in enumerate(opts):
        want = plain_pick(logits[r], t, k, p, pen, generated[r], us[r])
        if got[r] != want:
            l = logits[r].double()
            if pen != 1.0:
                l = P.repetition_penalty(l, generated[r], pen)
            probs = P.filtered_distribution(P.temperature_scale(l, t), k, p)
            cum = torch.cumsum(probs, 0)
            lo = min(got[r], want)
            assert t > 0 and probs[got[r]] > 0 and abs(float(cum[lo]) - us[r]) < 1e-5, (r, got[r], want)
    assert got[5] != int(logits[5].argmax())         # the penalised maximum lost


def test_sampling_closed_forms(K):
    V = 10
    logits = torch.tensor([[2.0, -1.0, 3.0, 0.0, -2.0, 1.0, 0.5, -0.5, 1.5, -1.5]]).repeat(5, 1)
    # top-k 1 is argmax whatever u; a tiny temperature too; greedy with a penalty moves the maximum
    got = sample_rows(K, logits, [1.0, 1e-4, 0.0, 0.0, 1.0], [1, 0, 0, 0, 0], [1.0, 1.0, 1.0, 1.0, 0.3],
                      [1.0, 1.0, 1.0, 10.0, 1.0], [[], [], [], [2], []], [0.99, 0.5, 0.5, 0.5, 0.7])
    assert got[:3] == [2, 2, 2]
    assert got[3] == 0                      # 3.0 / 10 = 0.3 < 2.0: the penalised token loses
    assert got[4] == 2                      # top-p 0.3: the most probable token alone carries it
    # same seed, same token; other u, possibly other token, but always inside the top-k set
    logits = torch.randn(1, 777, generator=torch.Generator().manual_seed(4)).repeat(64, 1)
    us = [(i + 1) / 64 for i in range(64)]
    got = sample_rows(K, logits, [1.0] * 64, [5] * 64, [1.0] * 64, [1.0] * 64, [[]] * 64, us)
    top5 = set(logits[0].topk(5).indices.tolist())
    assert set(got) <= top5 and len(set(got)) > 1
    again = sample_rows(K, logits, [1.0] * 64, [5] * 64, [1.0] * 64, [1.0] * 64, [[]] * 64, us)
    assert again == got


def test_sampling_keeps_the_penalised_tokens_of_a_run(K):
    """With a count of its own on the device, a row's list of penalised tokens takes every token the
    row is given, and the next call over the same rows penalises it: three calls in a row equal three
    calls whose lists the host has extended."""
    V, R = 3000, 3
    g = torch.Generator().manual_seed(11)
    logits = [torch.randn(R, V, generator=g) * 2 for _ in range(3)]
    for lg in logits:
        lg[0] *= 0.05
        lg[0, 7] = 30.0            # row 0 (greedy, penalty 5): 7 wins once, then its penalised logit 6 still does,
        lg[0, 9] = 6.5             # unless 9 has not been chosen yet
    temperature, top_k, top_p, penalty = [0.0, 0.9, 1.0], [0, 20, 0], [1.0, 1.0, 0.7], [5.0, 1.4, 1.0]
    us = [[0.5, 0.3, 0.9], [0.5, 0.6, 0.2], [0.5, 0.1, 0.4]]
    start = [[], [5, 6], [1]]
    want, lists = [], [list(x) for x in start]
    for i in range(3):
        got = sample_rows(K, logits[i], temperature, top_k, top_p, penalty, lists, us[i])
        want.append(got)
        for r in range(R):
            lists[r].append(got[r])
    assert [w[0] for w in want] == [7, 9, 7]
    f32, i32 = torch.float32, torch.int32
    pen_ids, pen_off = [], [0]
    for x in start:
        pen_ids += sorted(set(x)) + [0] * 3
        pen_off.append(len(pen_ids))
    ids, off = dev(torch.tensor(pen_ids, dtype=i32)), dev(torch.tensor(pen_off, dtype=i32))
    count = dev(torch.tensor([len(set(x)) for x in start], dtype=i32))
    opts = [dev(torch.tensor(temperature, dtype=f32)), dev(torch.tensor(top_k, dtype=i32)), dev(torch.tensor(top_p, dtype=f32)),
            dev(torch.tensor(penalty, dtype=f32))]
    for i in range(3):
        out = torch.empty(R, dtype=i32, device="cuda")
        K.sample(dev(logits[i]), torch.empty(R, V, device="cuda"), *opts, ids, off, dev(torch.tensor(us[i], dtype=f32)), out,
                 pen_count=count)
        assert out.tolist() == want[i], i
    assert count.tolist() == [len(set(x)) + 3 for x in start]
    assert ids.tolist()[0:3] == [w[0] for w in want]


# ------------------------------------------------------------------ skinny matrix product

def _skinny_case(Kmod, dtype, M, N, Kd):
    g = torch.Generator().manual_seed(M * 1000 + N + Kd)
    x = torch.randn(M, Kd, generator=g).to(DT[dtype])
    w = (torch.randn(N, Kd, generator=g) / math.sqrt(Kd)).to(DT[dtype])
    want = x.double() @ w.double().t()
    if not Kmod.skinny_ok(M, Kd, DT[dtype]):
        with pytest.raises(Kmod.KernelError):
            Kmod.skinny_gemm(dev(x), dev(w), torch.empty(M, N, device="cuda", dtype=DT[dtype]))
        return
    out = Kmod.skinny_gemm(dev(x), dev(w), torch.empty(M, N, device="cuda", dtype=DT[dtype]))
    assert rel(out, want) < KTOL[dtype], "store"
    out32 = Kmod.skinny_gemm(dev(x), dev(w), torch.empty(M, N, device="cuda", dtype=torch.float32))
    assert rel(out32, want) < 3e-6, "float32 out"
    if N % 2 == 0:
        act = Kmod.skinny_gemm(dev(x), dev(w), torch.empty(M, N // 2, device="cuda", dtype=DT[dtype]), swiglu=True)
        assert rel(act, P.swiglu(want[:, :N // 2], want[:, N // 2:])) < KTOL[dtype], "swiglu"
    assert rel(Kmod.linear(dev(x), dev(w)), want) < KTOL[dtype]
    # the re-tiled copy of the matrix gives the same sums in the same order
    tiled = Kmod.Weight(dev(w))
    assert tiled.tiles is not None and tiled.tiles.numel() >= w.numel()
    assert torch.equal(Kmod.skinny_gemm(dev(x), tiled, torch.empty(M, N, device="cuda", dtype=DT[dtype])), out)
    assert torch.equal(Kmod.skinny_gemm(dev(x), tiled, torch.empty(M, N, device="cuda", dtype=torch.float32)), out32)
    if N % 2 == 0:
        assert torch.equal(Kmod.skinny_gemm(dev(x), tiled, torch.empty(M, N // 2, device="cuda", dtype=DT[dtype]), swiglu=True), act)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M,N,Kd", [(1, 16, 16), (5, 50, 64), (16, 1000, 192), (17, 778, 2048), (40, 2064, 528),
                                    (64, 96, 8192), (8, 128256, 64), (3, 33, 48), (33, 40000, 256), (2, 34, 24)])
def test_skinny_product(K, dtype, M, N, Kd):
    _skinny_case(K, dtype, M, N, Kd)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M,N,Kd", [(1, 32, 64), (5, 50, 192), (16, 1000, 528), (8, 4096, 2048), (3, 778, 1024), (16, 96, 48),
                                    (2, 64, 4096), (6, 1000, 528), (7, 96, 48), (9, 64, 256), (5, 33008, 48)])
def test_skinny_product_with_norm_prologue_and_residual_epilogue(K, dtype, M, N, Kd):
    """RMSNorm(h) as the input of a product (store and SwiGLU epilogues), and a product added into
    the residual stream, against the plain steps in float64.  Row widths that are no multiple of a
    128-byte piece (528, 48) put the zero padding of the re-tiled matrix to work."""
    g = torch.Generator().manual_seed(M * 77 + N + Kd)
    h = torch.randn(M, Kd, generator=g) * 3
    nw = 1 + 0.1 * torch.randn(Kd, generator=g)
    eps = 2e-6
    w = (torch.randn(N, Kd, generator=g) / math.sqrt(Kd)).to(DT[dtype])
    W = K.Weight(dev(w))
    xn = P.rmsnorm(h.double(), nw, eps)
    ok = K.norm_prologue_ok(M, Kd, DT[dtype], W)
    assert ok == (Kd <= 2048 and M <= 8), "up to eight rows of up to 2,048 elements are taken"
    assert not K.norm_prologue_ok(9, Kd, DT[dtype], W) and not K.norm_prologue_ok(M, Kd, DT[dtype], dev(w))
    normed = K.NormedInput(dev(h), dev(nw), eps, DT[dtype])
    if not ok:      # refused with a reason, never run
        with pytest.raises(K.KernelError):
            K.skinny_gemm(normed, W, torch.empty(M, N, device="cuda", dtype=DT[dtype]))
    else:
        # the operand is rounded to the compute type after the norm, as the separate kernel rounds its output
        xr = xn.to(DT[dtype]).double()
        want = xr @ w.double().t()
        out = K.skinny_gemm(normed, W, torch.empty(M, N, device="cuda", dtype=DT[dtype]))
        assert rel(out, want) < KTOL[dtype], "normed, store"
        assert rel(K.linear(normed, W), want) < KTOL[dtype]
        if N % 32 == 0:
            act = K.skinny_gemm(normed, W, torch.empty(M, N // 2, device="cuda", dtype=DT[dtype]), swiglu=True)
            assert rel(act, P.swiglu(want[:, :N // 2], want[:, N // 2:])) < KTOL[dtype], "normed, swiglu"
            assert rel(K.linear_swiglu(normed, W), P.swiglu(want[:, :N // 2], want[:, N // 2:])) < KTOL[dtype]
        # the same numbers as norm kernel + product, up to the order of the sum of squares
        x_sep = K.add_rmsnorm(dev(h.clone()), None, dev(nw), eps, torch.empty(M, Kd, device="cuda", dtype=DT[dtype]))
        sep = K.skinny_gemm(x_sep, W, torch.empty(M, N, device="cuda", dtype=DT[dtype]))
        assert rel(out, sep.double().cpu()) < KTOL[dtype]
    # residual epilogue: stream += x . W^T, in float32, other columns and rows untouched
    x = torch.randn(M, Kd, generator=g).to(DT[dtype])
    stream = torch.randn(M + 2, N, generator=g)
    buf = dev(stream.clone())
    assert K.residual_epilogue_ok(M, Kd, DT[dtype], W) and not K.residual_epilogue_ok(M, Kd, DT[dtype], dev(w))
    shares = K.skinny_ksplit(M, Kd, DT[dtype], W)[0]
    assert (shares > 1) == (Kd >= 4096), "long rows on a matrix of few tiles go in shares, for the next norm or prologue to add"
    addends = K.linear(dev(x), W, residual=buf[:M])
    if shares > 1:
        assert addends.shape == (shares, M, N) and addends.dtype == torch.float32 and torch.equal(buf.cpu(), stream)
        assert rel(addends.double().sum(0), x.double() @ w.double().t()) < 3e-6
    else:
        assert addends is None
        assert rel(buf[:M], stream[:M].double() + x.double() @ w.double().t()) < 3e-6
    assert torch.equal(buf[M:].cpu(), stream[M:])
    with pytest.raises(K.KernelError):
        K.skinny_gemm(normed, dev(w), torch.empty(M, N, device="cuda", dtype=DT[dtype]))       # needs the re-tiled matrix


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M,d,Ko,N2,S", [(1, 64, 32, 96, 0), (5, 192, 528, 1000, 2), (8, 2048, 2048, 256, 0), (16, 100 * 16, 48, 64, 1),
                                         (3, 4096, 512, 128, 0), (24, 528, 64, 160, 0), (33, 2064, 192, 96, 0), (64, 2048, 2048, 512, 0),
                                         (48, 272, 4096, 64, 0), (12, 3072, 256, 64, 2), (32, 2048, 2048, 512, 0),
                                         (20, 3072, 3072, 256, 0), (8, 2048, 8192, 64, 2), (17, 272, 4112, 64, 0),
                                         (16, 528, 4096, 64, 0), (4, 2048, 8192, 64, 0), (13, 2560, 4112, 96, 1),
                                         (9, 2040, 4096, 64, 0), (7, 24, 4096, 64, 1)])
def test_a_norm_done_in_two_halves_by_the_products_around_it(K, dtype, M, d, Ko, N2, S):
    """A product onto the residual stream leaves ``h * w`` and every workgroup's sums of squares of its columns
    behind; the product after the norm takes them and divides by the rows' root mean squares in its epilogue
    (store, float32 store, SwiGLU, rotation + cache write).  Against the plain steps in float64: stream, then
    RMSNorm, rounded to the compute type, then the product.  With addends that the stream has not received (S),
    widths that are no multiple of a tile or a piece, and one to four blocks of rows."""
    g = torch.Generator().manual_seed(M * 131 + d + Ko)
    dt = DT[dtype]
    h = torch.randn(M + 1, d, generator=g) * 2
    x = torch.randn(M, Ko, generator=g).to(dt)
    wo = (torch.randn(d, Ko, generator=g) / math.sqrt(Ko)).to(dt)
    nw = 1 + 0.1 * torch.randn(d, generator=g)
    eps = 3e-6
    pend = torch.randn(S, M, d, generator=g) if S else None
    Wo = K.Weight(dev(wo))
    # up to 16 rows a product that would not be cut along K anyway (or, in bfloat16 from five rows on, one of long rows
    # on few tiles, which then runs on halved tiles), up to 32 one with rows of up to 4,096 elements
    halved = dtype == "bfloat16" and M >= 5 and d <= 128 * 16 and Ko >= 4096
    assert K.leaves_scaled_ok(M, Ko, dt, Wo) == (K.skinny_ksplit(M, Ko, dt, Wo)[0] == 1 or halved if M <= 16 else
                                                 (M <= 32 and Ko <= 4096 and K.skinny_wins(M, Ko, dt, Wo)))
    if dtype == "bfloat16":     # (in float32 the skinny kernels stream rows of up to 2,048 elements only, past 16 rows)
        assert K.leaves_scaled_ok(M, Ko, dt, Wo) == ((M, Ko) not in ((33, 192), (64, 2048), (48, 4096), (4, 8192), (17, 4112)))
    else:
        assert not K.leaves_scaled_ok(M, Ko, dt, Wo) or (M, Ko) not in ((8, 8192), (16, 4096), (4, 8192))
    assert not K.leaves_scaled_ok(M, Ko, dt, dev(wo)), "only a re-tiled matrix"
    if not K.leaves_scaled_ok(M, Ko, dt, Wo):
        if K.residual_epilogue_ok(M, Ko, dt, Wo):       # the product goes its other way, whatever is asked for the norm
            assert not isinstance(K.linear(dev(x), Wo, residual=dev(h.clone())[:M], leave=K.NormSpec(dev(nw), eps)),
                                  K.ScaledInput)
        return
    stream = dev(h.clone())
    spec = K.NormSpec(dev(nw), eps)
    args = (dev(x), None if pend is None else dev(pend))
    for size in (M * 64, M * 256, M * d):       # what the product allocates for itself starts out as NaN, not as zeros
        del_me = torch.full((size,), float("nan"), device="cuda")
        del del_me
    left = K.linear(args[0], Wo, residual=stream[:M], pending=args[1], leave=spec)
    assert isinstance(left, K.ScaledInput) and left.made_for(spec.weight, eps) and not left.made_for(dev(nw), eps)
    want_h = h[:M].double() + x.double() @ wo.double().t()
    if pend is not None:
        want_h = (h[:M].double() + pend.double().sum(0)) + x.double() @ wo.double().t()
    assert rel(stream[:M], want_h) < 3e-6 and torch.equal(stream[M:].cpu(), h[M:]), "the stream itself, and no other row"
    got_h = stream[:M].double().cpu()
    assert rel(left.x, got_h * nw.double()) < KTOL[dtype], "h * w"
    assert left.ss.shape[0] == M and rel(left.ss.double().sum(1), (got_h ** 2).sum(1)) < 3e-6, "sums of squares"
    xn = P.rmsnorm(got_h, nw, eps).to(dt).double()
    # the products behind the norm: what the kernel is to compute, ((h * w rounded to the compute type) . W^T) / rms(h),
    # and, beside it, the plain order (norm, rounded, then the product), from which it differs by how the operand's
    # elements are rounded (each once in both orders; in float32 not at all)
    w2 = (torch.randn(N2, d, generator=g) / math.sqrt(d)).to(dt)
    W2 = K.Weight(dev(w2))
    inv_rms = 1.0 / torch.sqrt((got_h ** 2).mean(dim=1, keepdim=True) + eps)
    want = ((got_h * nw.double()).to(dt).double() @ w2.double().t()) * inv_rms
    plain_order = xn @ w2.double().t()
    assert rel(want, plain_order) < (1e-6 if dtype == "float32" else 1e-2)
    takes = K.takes_scaled_ok(M, d, dt, W2)
    assert takes == K.skinny_wins(M, d, dt, W2)
    if not takes:
        with pytest.raises(K.KernelError):
            K.linear(left, W2)
        return
    assert rel(K.linear(left, W2), want) < KTOL[dtype], "store"
    assert rel(K.linear(left, W2, out_dtype=torch.float32), want) < KTOL[dtype], "float32 store"
    if N2 % 32 == 0:
        assert K.swiglu_takes_scaled(M, d, dt, W2)
        assert rel(K.linear_swiglu(left, W2), P.swiglu(want[:, :N2 // 2], want[:, N2 // 2:])) < KTOL[dtype], "swiglu"
    with pytest.raises(K.KernelError):
        K.linear(left, dev(w2))                 # as stored: not taken
    # rotation and cache write behind the norm: the same queries and pages as from the normalised rows
    H, KVH, hd, ps = 2, 1, 32, 4
    wq = (torch.randn((H + 2 * KVH) * hd, d, generator=g) / math.sqrt(d)).to(dt)
    Wq = K.Weight(dev(wq))
    if K.qkv_rope_ok(M, d, hd, hd, dt) and K.takes_scaled_ok(M, d, dt, Wq):
        cos, sin = K.rope_table(dev(torch.rand(hd // 2, generator=g)), 128)
        pos = dev(torch.arange(M, dtype=torch.int32) + 7)
        slots = dev(torch.randperm(M + 3, generator=g)[:M].to(torch.int32))
        pools = [[torch.zeros(-(-(M + 3) // ps), KVH, ps, hd, device="cuda", dtype=dt) for _ in range(2)] for _ in range(2)]
        q_scaled = K.skinny_qkv_rope(left, Wq, pos, cos, sin, slots, pools[0][0], pools[0][1], H, KVH, hd)
        q_plain = K.skinny_qkv_rope(dev(xn.to(dt)), Wq, pos, cos, sin, slots, pools[1][0], pools[1][1], H, KVH, hd)
        scale = float(q_plain.double().abs().max())
        assert float((q_scaled.double() - q_plain.double()).abs().max()) < KTOL[dtype] * scale
        for a, b in zip(pools[0], pools[1]):
            assert float((a.double() - b.double()).abs().max()) < KTOL[dtype] * max(scale, float(b.double().abs().max()))
            assert float(b.double().abs().max()) > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M,N,Kd", [(17, 96, 2048), (33, 778, 528), (64, 2064, 192), (40, 50, 4096), (24, 64, 8192), (64, 2048, 8192),
                                    (20, 3000, 2048), (48, 272, 4112)])
def test_skinny_product_of_17_to_64_rows_adds_into_the_residual_stream(K, dtype, M, N, Kd):
    """The kernel for 17 to 64 rows (re-tiled matrix, x through LDS): the residual epilogue, rows
    that are no multiple of 16, a tile past the matrix, a row width that is no multiple of a piece."""
    g = torch.Generator().manual_seed(M * 31 + N + Kd)
    w = (torch.randn(N, Kd, generator=g) / math.sqrt(Kd)).to(DT[dtype])
    W = K.Weight(dev(w))
    x = torch.randn(M, Kd, generator=g).to(DT[dtype])
    stream = torch.randn(M + 3, N, generator=g)
    buf = dev(stream.clone())
    assert not K.skinny_wins(M, Kd, DT[dtype], dev(w)), "past 16 rows only a re-tiled matrix is streamed"
    ok = K.residual_epilogue_ok(M, Kd, DT[dtype], W)
    assert ok == (K.skinny_wins(M, Kd, DT[dtype], W) or K.skinny_ksplit(M, Kd, DT[dtype], W)[0] > 1)
    assert ok
    got = K.linear(dev(x), W, residual=buf[:M])
    shares, per = K.skinny_ksplit(M, Kd, DT[dtype], W)
    groups = -(-((N + 15) // 16) // per)
    assert 1 <= shares <= 16 and (shares == 1 or (shares * groups <= 256 and Kd // 64 // shares >= 16)), \
        "a cut leaves no more than a workgroup for every compute unit and at least sixteen pieces a share"
    if shares > 1:
        # the K range was cut: float32 addends for the next norm, the stream itself untouched
        assert got.dtype == torch.float32 and tuple(got.shape) == (shares, M, N)
        assert torch.equal(buf.cpu(), stream)
        total = buf[:M].double() + got.double().sum(0)
        # ... which adds them in its pass: h += sum of the addends, out = rmsnorm(h)
        nw = 1 + 0.1 * torch.randn(N, generator=g)
        out = K.add_rmsnorm(buf[:M], got, dev(nw), 1e-5, torch.empty(M, N, device="cuda", dtype=DT[dtype]))
        assert rel(buf[:M], total.cpu()) < 1e-6
        assert rel(out, P.rmsnorm(total.cpu(), nw, 1e-5)) < KTOL[dtype]
        picked = dev(torch.tensor([M - 1, 0, 3], dtype=torch.int32))
        buf2 = dev(stream.clone())
        out = K.add_rmsnorm(buf2[:M], got, dev(nw), 1e-5, torch.empty(3, N, device="cuda", dtype=DT[dtype]), picked)
        assert rel(out, P.rmsnorm(total.cpu(), nw, 1e-5)[[M - 1, 0, 3]]) < KTOL[dtype] and torch.equal(buf2.cpu(), stream)
    else:
        assert got is None
        total = buf[:M].double()
    assert rel(total, stream[:M].double() + x.double() @ w.double().t()) < 3e-6
    assert torch.equal(buf[M:].cpu(), stream[M:]), "rows past the batch were written"
    assert rel(K.linear(dev(x), W), x.double() @ w.double().t()) < KTOL[dtype]


@pytest.mark.parametrize("M,N,Kd,shares", [(9, 2048, 8192, 2), (16, 96, 4096, 4), (12, 272, 4112, 4), (8, 2048, 8192, 2),
                                           (1, 2048, 8192, 2), (8, 96, 4096, 2), (8, 3072, 8192, 1), (1, 4096, 14336, 1),
                                           (12, 3072, 8192, 1), (16, 2048, 2048, 1), (8, 2048, 2048, 1)])
def test_long_products_of_up_to_16_rows_are_cut_where_the_chip_has_room(K, M, N, Kd, shares):
    """Up to 16 bfloat16 rows of 4,096 elements or more onto the residual stream go in shares of K
    where the shares still make no more workgroups than the chip has compute units (not the 192
    tiles of the 3B shape in two shares): as many as fit past eight rows, where the norm that
    follows is a kernel of its own; two up to eight rows, which the next product's normalising
    prologue adds to its rows itself."""
    g = torch.Generator().manual_seed(M + N + Kd)
    w = (torch.randn(N, Kd, generator=g) / math.sqrt(Kd)).to(torch.bfloat16)
    W = K.Weight(dev(w))
    x = torch.randn(M, Kd, generator=g).to(torch.bfloat16)
    stream = torch.randn(M + 1, N, generator=g)
    buf = dev(stream.clone())
    assert K.skinny_ksplit(M, Kd, torch.bfloat16, W)[0] == shares
    got = K.linear(dev(x), W, residual=buf[:M])
    if shares == 1:
        assert got is None
        total = buf[:M].double().cpu()
    else:
        assert tuple(got.shape) == (shares, M, N) and got.dtype == torch.float32 and torch.equal(buf.cpu(), stream)
        total = stream[:M].double() + got.double().sum(0).cpu()
    assert rel(total, stream[:M].double() + x.double() @ w.double().t()) < 3e-6
    assert torch.equal(buf[M:].cpu(), stream[M:])


@pytest.mark.parametrize("M,H,hd,N,runs", [(1, 32, 64, 2048, 8), (8, 32, 64, 2048, 4), (3, 8, 128, 528, 8), (5, 24, 32, 96, 2),
                                           (4, 6, 80, 272, 3), (8, 16, 128, 64, 4), (2, 1, 16, 48, 5), (1, 12, 96, 40, 16)])
@pytest.mark.parametrize("residual", [False, True])
def test_skinny_product_merges_the_key_runs_of_an_attention(K, M, H, hd, N, runs, residual):
    # The attention's partial results go straight into the output product.  One run of one head
    # dominates by e^12 and one is empty (maximum "minus infinity", sum 0), so that a wrong weight or
    # a mixed-up index of (row, head, run) shows.
    g = torch.Generator().manual_seed(M * 1000 + H * 10 + runs)
    part_o = torch.randn(M, H, runs, hd, generator=g) * 5
    part_m = torch.randn(M, H, runs, generator=g) * 3
    part_l = torch.rand(M, H, runs, generator=g) * 50 + 1
    part_m[M - 1, H // 2, runs - 1] += 12.0
    part_m[0, 0, 0], part_l[0, 0, 0], part_o[0, 0, 0] = -1.0e30 * math.log(2.0), 0.0, 0.0
    w = torch.randn(N, H * hd, generator=g) / math.sqrt(H * hd)
    wt = K.Weight(dev(w, torch.bfloat16))
    assert K.skinny_merge_ok(M, H, hd, runs, torch.bfloat16, wt)
    ws = dev(torch.cat([part_o.reshape(-1), torch.stack([part_m, part_l], -1).reshape(-1)]))
    f = torch.exp(part_m.double() - part_m.double().amax(-1, keepdim=True))
    attn = ((part_o.double() * f[..., None]).sum(2) / (part_l.double() * f).sum(-1, keepdim=True)).reshape(M, H * hd)
    want = attn.to(torch.bfloat16).double() @ w.to(torch.bfloat16).double().t()
    if residual:
        h0 = torch.randn(M, N, generator=g)
        out = dev(h0.clone())
        K.skinny_gemm_merged(ws, runs, M, H, hd, wt, out, residual=True)
        got = out.cpu().double() - h0.double()
    else:
        out = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
        got = K.skinny_gemm_merged(ws, runs, M, H, hd, wt, out).cpu().double()
    assert rel(got, want) < KTOL["bfloat16"], (M, H, hd, N, runs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M,N,Kd,S", [(1, 64, 2048, 2), (8, 96, 2048, 2), (4, 1000, 528, 1), (5, 64, 192, 2), (7, 3072, 2048, 2),
                                      (2, 32, 48, 1), (8, 128, 1024, 2)])
def test_pending_addends_of_the_residual_stream_ride_on_the_products(K, dtype, M, N, Kd, S):
    """The shares of a cut product, which h has not received yet: the normalising prologue normalises
    (h + p0) + p1 and leaves h alone, the residual epilogue stores ((h + p0) + p1) + product.  Both
    give the very numbers of the same kernels run on a stream that a plain sum has updated before."""
    g = torch.Generator().manual_seed(M * 31 + N + Kd + S)
    h = torch.randn(M, Kd, generator=g) * 3
    pend = torch.randn(S, M, Kd, generator=g) * 2
    summed = h.clone()
    for a in range(S):
        summed += pend[a]
    nw = 1 + 0.1 * torch.randn(Kd, generator=g)
    eps = 3e-6
    w = (torch.randn(N, Kd, generator=g) / math.sqrt(Kd)).to(DT[dtype])
    W = K.Weight(dev(w))
    assert K.prologue_addends() == 2
    assert K.norm_prologue_ok(M, Kd, DT[dtype], W, S) and not K.norm_prologue_ok(M, Kd, DT[dtype], W, 3)
    h_dev = dev(h)
    with_addends = K.NormedInput(h_dev, dev(nw), eps, DT[dtype], dev(pend))
    plain = K.NormedInput(dev(summed), dev(nw), eps, DT[dtype])
    out = lambda n: torch.empty(M, n, device="cuda", dtype=DT[dtype])
    got, want = K.skinny_gemm(with_addends, W, out(N)), K.skinny_gemm(plain, W, out(N))
    assert torch.equal(got, want), "normed with addends, store"
    assert rel(got, P.rmsnorm(summed.double(), nw, eps).to(DT[dtype]).double() @ w.double().t()) < KTOL[dtype]
    assert torch.equal(K.linear(with_addends, W), want)
    if N % 32 == 0:
        assert K.norm_prologue_ok(M, Kd, DT[dtype], W, S, swiglu=True)
        assert torch.equal(K.linear_swiglu(with_addends, W), K.linear_swiglu(plain, W)), "normed with addends, swiglu"
    assert torch.equal(h_dev.cpu(), h), "the prologue leaves h as it is"
    # the residual epilogue: the stream's own addends [S, M, N] first, then the product
    x = torch.randn(M, Kd, generator=g).to(DT[dtype])
    stream = torch.randn(M + 1, N, generator=g)
    owed = torch.randn(S, M, N, generator=g)
    assert K.residual_takes_addends(M, Kd, DT[dtype], W)
    got = dev(stream.clone())
    assert K.linear(dev(x), W, residual=got[:M], pending=dev(owed)) is None
    want = stream.clone()
    for a in range(S):
        want[:M] += owed[a]
    want = dev(want)
    K.linear(dev(x), W, residual=want[:M])
    assert torch.equal(got, want), "residual with addends"
    with pytest.raises(K.KernelError):
        K.linear(dev(x), W, pending=dev(owed))                                    # nothing to add them into
    with pytest.raises(K.KernelError):
        K.linear(dev(x), W, residual=got[:M], pending=dev(owed[:, :, :N - 16]))   # of another width
    with pytest.raises(K.KernelError):
        K.skinny_gemm(K.NormedInput(h_dev, dev(nw), eps, DT[dtype], dev(torch.zeros(3, M, Kd))), W, out(N))   # more than it holds


def test_pending_addends_with_rotation_and_with_merged_key_runs(K):
    """The same for the product that rotates and writes the cache (normalising prologue) and for the output
    product that merges an attention's key runs (residual epilogue)."""
    g = torch.Generator().manual_seed(5)
    for dtype, M, H, KVH, hd, Kd in (("bfloat16", 8, 32, 8, 64, 2048), ("float32", 3, 4, 2, 32, 192), ("bfloat16", 1, 6, 1, 32, 528)):
        h = torch.randn(M, Kd, generator=g) * 2
        pend = torch.randn(2, M, Kd, generator=g)
        summed = (h + pend[0]) + pend[1]
        nw = 1 + 0.1 * torch.randn(Kd, generator=g)
        W = K.Weight(dev((torch.randn((H + 2 * KVH) * hd, Kd, generator=g) / math.sqrt(Kd)).to(DT[dtype])))
        positions = dev(torch.randint(0, 500, (M,), generator=g).to(torch.int32))
        slots = dev(torch.tensor(random.Random(2).sample(range(32), M), dtype=torch.int32))
        cos, sin = K.rope_table(dev(torch.from_numpy(P.rope_frequencies(hd, 10000.0, None))), 512)
        results = []
        for x in (K.NormedInput(dev(h), dev(nw), 1e-5, DT[dtype], dev(pend)), K.NormedInput(dev(summed), dev(nw), 1e-5, DT[dtype])):
            kp = torch.zeros(2, KVH, 16, hd, dtype=DT[dtype], device="cuda")
            vp = torch.zeros_like(kp)
            results.append((K.skinny_qkv_rope(x, W, positions, cos, sin, slots, kp, vp, H, KVH, hd), kp, vp))
        for a, b in zip(*results):
            assert torch.equal(a, b), dtype
    M, H, hd, N, runs = 2, 32, 64, 2048, 8
    part_o = torch.randn(M, H, runs, hd, generator=g)
    ml = torch.stack([torch.randn(M, H, runs, generator=g), torch.rand(M, H, runs, generator=g) + 1], -1)
    ws = dev(torch.cat([part_o.reshape(-1), ml.reshape(-1)]))
    wt = K.Weight(dev(torch.randn(N, H * hd, generator=g) / 45, torch.bfloat16))
    stream, owed = torch.randn(M, N, generator=g), torch.randn(2, M, N, generator=g)
    got = dev(stream.clone())
    K.skinny_gemm_merged(ws, runs, M, H, hd, wt, got, residual=True, pending=dev(owed))
    want = dev((stream + owed[0]) + owed[1])
    K.skinny_gemm_merged(ws, runs, M, H, hd, wt, want, residual=True)
    assert torch.equal(got, want)


def test_what_the_merging_prologue_refuses(K):
    wt = K.Weight(dev(torch.zeros(64, 2048), torch.bfloat16))
    assert K.skinny_merge_ok(8, 32, 64, 4, torch.bfloat16, wt)
    assert not K.skinny_merge_ok(9, 32, 64, 4, torch.bfloat16, wt)          # more rows than the prologue stages
    assert not K.skinny_merge_ok(8, 32, 64, 1, torch.bfloat16, wt)          # nothing to merge
    assert not K.skinny_merge_ok(8, 32, 64, 17, torch.bfloat16, wt)         # more runs than it holds
    assert K.skinny_merge_ok(1, 32, 64, 16, torch.bfloat16, wt) and K.skinny_merge_ok(4, 32, 64, 8, torch.bfloat16, wt)
    assert not K.skinny_merge_ok(8, 32, 64, 5, torch.bfloat16, wt)          # eight rows: four runs fit a thread's registers
    assert not K.skinny_merge_ok(3, 32, 64, 9, torch.bfloat16, wt)          # four rows: eight runs
    assert not K.skinny_merge_ok(8, 48, 64, 4, torch.bfloat16, wt)          # rows of 3,072 elements: past the compiled size
    assert not K.skinny_merge_ok(8, 32, 64, 4, torch.float32, wt)
    # and where it is taken: one or two rows, beyond that the merge kernel is the faster way
    assert K.skinny_merge_wins(1, 32, 64, 8, torch.bfloat16, wt) and K.skinny_merge_wins(2, 32, 64, 8, torch.bfloat16, wt)
    assert not K.skinny_merge_wins(8, 32, 64, 4, torch.bfloat16, wt) and not K.skinny_merge_wins(3, 32, 64, 8, torch.bfloat16, wt)
    assert not K.skinny_merge_ok(8, 32, 64, 4, torch.bfloat16, K.Weight(dev(torch.zeros(64, 2048), torch.bfloat16), tiled=False))
    with pytest.raises(K.KernelError, match="merging prologue"):
        K.skinny_gemm_merged(torch.zeros(1 << 20, device="cuda"), 17, 8, 32, 64, wt, torch.empty(8, 64, device="cuda", dtype=torch.bfloat16))
    with pytest.raises(K.KernelError, match="workspace"):
        K.skinny_gemm_merged(torch.zeros(100, device="cuda"), 4, 8, 32, 64, wt, torch.empty(8, 64, device="cuda", dtype=torch.bfloat16))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whichever_product_is_chosen_equals_the_plain_one(K, dtype):
    """``K.linear`` and ``K.linear_swiglu`` choose between the skinny kernels (whole, or cut along K into
    float32 shares) and the library by rules that were measured and may be measured again.  Whatever
    they choose, for row counts and widths on both sides of every rule: the result is the plain product,
    onto the residual stream as well as into a tensor of its own."""
    g = torch.Generator().manual_seed(5)
    dt = DT[dtype]
    paths = set()
    for N, Kd in ((32, 8192), (2048, 2048), (48, 3072), (4096, 4096), (40, 2040 if dtype == "float32" else 2032)):
        w = (torch.randn(N, Kd, generator=g) / math.sqrt(Kd)).to(dt)
        W = K.Weight(dev(w))
        for M in (1, 8, 9, 16, 17, 32, 33, 40, 64, 65, 130):
            x = torch.randn(M, Kd, generator=g).to(dt)
            want = x.double() @ w.double().t()
            calls = K.library_calls()
            assert rel(K.linear(dev(x), W), want) < KTOL[dtype], (M, N, Kd)
            paths.add("library" if K.library_calls() != calls else "skinny")
            if K.residual_epilogue_ok(M, Kd, dt, W):
                h0 = torch.randn(M, N, generator=g)
                h = dev(h0.clone())
                out = K.linear(dev(x), W, residual=h)
                if out is None:
                    total = h
                    paths.add("residual")
                else:       # float32 shares for the next norm to add
                    assert out.dtype == torch.float32 and out.dim() == 3 and out.shape[0] == K.skinny_ksplit(M, Kd, dt, W)[0] > 1
                    assert torch.equal(h.cpu(), h0)
                    total = h + out.sum(0)
                    paths.add("shares")
                assert rel(total, h0.double() + want) < KTOL[dtype], (M, N, Kd)
    for inter, Kd in ((8192, 2048), (136, 96)):
        w = (torch.randn(2 * inter, Kd, generator=g) / math.sqrt(Kd)).to(dt)
        W = K.Weight(dev(w))
        for M in (8, 17, 32, 33, 64, 65):
            x = torch.randn(M, Kd, generator=g).to(dt)
            gu = x.double() @ w.double().t()
            assert rel(K.linear_swiglu(dev(x), W), P.swiglu(gu[:, :inter], gu[:, inter:])) < KTOL[dtype], (M, inter, Kd)
    assert paths == {"library", "skinny", "residual", "shares"}        # the cases did reach every way
    # what no rule may change: more than 64 rows never go to the skinny kernels, and a matrix that is not
    # re-tiled has no residual epilogue past 16 rows (the library's product adds into nothing)
    assert not K.skinny_wins(65, 2048, dt, K.Weight(dev(torch.zeros(32, 2048)), tiled=True))
    plain = dev(torch.zeros(32, 8192))
    assert not K.residual_epilogue_ok(40, 8192, dt, plain)
    with pytest.raises(K.KernelError):
        K.linear(dev(torch.zeros(40, 8192)).to(dt), plain.to(dt), residual=dev(torch.zeros(40, 32)))


def test_skinny_product_reference_vector(K):
    # test/test_cuda_kernel/test_matmul_kernel.cpp:30-99: ones x 0.5 with K = 128 gives 64
    out = K.skinny_gemm(torch.ones(3, 128, device="cuda"), torch.full((7, 128), 0.5, device="cuda"),
                        torch.empty(3, 7, device="cuda"))
    assert torch.all(out == 64.0)
    # many rows go to the library, in true float32
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(300, 1024, generator=g), torch.randn(512, 1024, generator=g) / 32
    assert rel(K.linear(dev(x), dev(w)), x.double() @ w.double().t()) < 3e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M,H,KVH,hd,Kd,ps", [(1, 4, 2, 32, 64, 8), (8, 32, 8, 64, 2048, 16), (5, 6, 1, 32, 192, 8),
                                             (40, 3, 3, 128, 96, 4), (64, 8, 2, 96, 256, 16), (14, 32, 8, 64, 2048, 16),
                                             (2, 24, 8, 128, 1024, 16), (16, 8, 8, 64, 2048, 16),
                                             # pairs of tiles x blocks of 32 rows past 256 workgroups: three and four
                                             # blocks of sixteen rows a workgroup instead; and just below: dealt out
                                             (64, 24, 8, 128, 512, 16), (40, 32, 8, 128, 256, 16), (33, 40, 8, 64, 128, 8),
                                             # 17 to 32 rows: sixteen a workgroup where that keeps within 256 workgroups
                                             (24, 32, 8, 64, 2048, 16), (32, 6, 1, 32, 192, 8), (20, 24, 8, 128, 1024, 16)])
def test_product_with_rotation_and_cache_write(K, dtype, M, H, KVH, hd, Kd, ps):
    """The fused epilogue against the plain steps: product, rotation of pairs (j, j + hd/2), write by slot."""
    g = torch.Generator().manual_seed(M + hd)
    x = torch.randn(M, Kd, generator=g).to(DT[dtype])
    w = (torch.randn((H + 2 * KVH) * hd, Kd, generator=g) / math.sqrt(Kd)).to(DT[dtype])
    positions = torch.randint(0, 500, (M,), generator=g).to(torch.int32)
    pages = -(-M // ps) + 2
    slots = torch.tensor(random.Random(1).sample(range(pages * ps), M), dtype=torch.int32)
    inv = P.rope_frequencies(hd, 10000.0, None)
    cos, sin = K.rope_table(dev(torch.from_numpy(inv)), 512)
    kpool = torch.full((pages, KVH, ps, hd), 7.0, dtype=DT[dtype], device="cuda")
    vpool = torch.full((pages, KVH, ps, hd), 7.0, dtype=DT[dtype], device="cuda")
    assert K.qkv_rope_ok(M, Kd, hd, hd, DT[dtype])
    q = K.skinny_qkv_rope(dev(x), dev(w), dev(positions), cos, sin, dev(slots), kpool, vpool, H, KVH, hd)
    W = K.Weight(dev(w))
    if K.norm_prologue_ok(M, Kd, DT[dtype], W):
        # the same product taken on RMSNorm(h): queries and pages as from the norm kernel's output
        h = torch.randn(M, Kd, generator=g) * 2
        nw = 1 + 0.1 * torch.randn(Kd, generator=g)
        x_sep = K.add_rmsnorm(dev(h.clone()), None, dev(nw), 1e-5, torch.empty(M, Kd, device="cuda", dtype=DT[dtype]))
        kp1, vp1 = torch.zeros_like(kpool), torch.zeros_like(vpool)
        q1 = K.skinny_qkv_rope(x_sep, W, dev(positions), cos, sin, dev(slots), kp1, vp1, H, KVH, hd)
        kp2, vp2 = torch.zeros_like(kpool), torch.zeros_like(vpool)
        q2 = K.skinny_qkv_rope(K.NormedInput(dev(h), dev(nw), 1e-5, DT[dtype]), W, dev(positions), cos, sin, dev(slots),
                               kp2, vp2, H, KVH, hd)
        for got, want_t in ((q2, q1), (kp2, kp1), (vp2, vp1)):
            assert rel(got, want_t.double().cpu()) < KTOL[dtype]
    qkv = x.double() @ w.double().t()
    s, c = P.rope_tables(positions.tolist(), inv)
    q_ref = plain_rotate_half(qkv[:, :H * hd].reshape(M, H, hd), s, c, hd)
    k_ref = plain_rotate_half(qkv[:, H * hd:(H + KVH) * hd].reshape(M, KVH, hd), s, c, hd)
    v_ref = qkv[:, (H + KVH) * hd:].reshape(M, KVH, hd)
    assert rel(q.reshape(M, H, hd), q_ref) < KTOL[dtype]
    kp, vp = kpool.cpu().double(), vpool.cpu().double()
    touched = torch.zeros(pages, ps, dtype=torch.bool)
    scale_k, scale_v = float(k_ref.abs().max()), float(v_ref.abs().max())
    for t in range(M):
        page, off = int(slots[t]) // ps, int(slots[t]) % ps
        touched[page, off] = True
        assert float((kp[page, :, off] - k_ref[t]).abs().max()) < KTOL[dtype] * scale_k
        assert float((vp[page, :, off] - v_ref[t]).abs().max()) < KTOL[dtype] * scale_v
    untouched = ~touched[:, None, :].expand(pages, KVH, ps)
    assert bool((kp[untouched] == 7.0).all()) and bool((vp[untouched] == 7.0).all())
    # without a slot mapping nothing is stored, the queries are the same
    k2 = torch.full_like(kpool, 3.0)
    q2 = K.skinny_qkv_rope(dev(x), dev(w), dev(positions), cos, sin, None, None, None, H, KVH, hd)
    assert torch.equal(q2, q) and bool((k2 == 3.0).all())
    # the re-tiled matrix: same queries, same pages
    k3, v3 = torch.full_like(kpool, 7.0), torch.full_like(vpool, 7.0)
    q3 = K.skinny_qkv_rope(dev(x), K.Weight(dev(w)), dev(positions), cos, sin, dev(slots), k3, v3, H, KVH, hd)
    assert torch.equal(q3, q) and torch.equal(k3, kpool) and torch.equal(v3, vpool)
    assert not K.qkv_rope_ok(M, Kd, 48, 48, DT[dtype]) and not K.qkv_rope_ok(M, Kd, hd, hd // 2, DT[dtype])
