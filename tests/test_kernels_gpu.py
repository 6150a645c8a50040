"""Each HIP kernel alone against a plain 32-bit reference, at other sizes than the
engine's: widths and vocabularies that are no power of two, head sizes in steps of 16,
several head groupings and page sizes.  Inputs are made so that faults show: one key
far away or at a page's or a window's edge carries the whole result."""
import math

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from qwen_engine_amd.kernels import ops
    ops.load_library()
    return ops


def rand(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def close(got, want, dtype, scale=None):
    got, want = got.float().cpu(), want.float().cpu()
    s = float(want.abs().max()) if scale is None else scale
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    err = float((got - want).abs().max())
    assert err <= tol * max(s, 1e-6), f"error {err} beside scale {s}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding(ops, dtype):
    table = rand(331, 80, seed=1, dtype=dtype)
    ids = torch.tensor([0, 330, 5, 5, 17, 200], dtype=torch.int32)
    out = ops.embedding(ids.to(DEV), table.to(DEV))
    assert out.dtype == torch.float32
    assert torch.equal(out.cpu(), P.embedding(ids, table).float())     # a copy: exact


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [77, 80, 1024, 3000, 9000])
def test_rmsnorm_plain_fused_and_gathered(ops, dtype, H):
    h = rand(7, H, seed=2, scale=3.0)
    w = 1 + rand(H, seed=3, scale=0.1)
    delta = rand(7, H, seed=4, dtype=dtype)
    eps = 1e-5
    close(ops.rmsnorm(h.to(DEV), w.to(DEV), eps, dtype), P.rms_norm(h, w, eps), dtype)
    hd = h.to(DEV)
    out = ops.rmsnorm(hd, w.to(DEV), eps, dtype, delta=delta.to(DEV))
    total = h + delta.float()
    close(out, P.rms_norm(total, w, eps), dtype)
    assert torch.equal(hd.cpu(), total)                                # the residual sum, in 32-bit
    rows = torch.tensor([6, 0, 3], dtype=torch.int32)
    hd = h.to(DEV)
    out = ops.rmsnorm(hd, w.to(DEV), eps, dtype, delta=delta.to(DEV), rows=rows.to(DEV))
    close(out, P.rms_norm(total[rows.long()], w, eps), dtype)
    assert torch.equal(hd.cpu(), h)                                    # gathered: h is left alone


def test_rmsnorm_eps_is_inside_the_root(ops):
    h = torch.full((1, 64), 2.0)
    out = ops.rmsnorm(h.to(DEV), torch.ones(64, device=DEV), 5.0, torch.float32)
    torch.testing.assert_close(out.cpu(), torch.full((1, 64), 2.0 / 3.0))


@pytest.mark.parametrize("M,N,K", [(1, 500, 96), (5, 331, 80), (64, 64, 64), (130, 77, 200), (3, 2048, 1024)])
@pytest.mark.parametrize("dt_x,dt_w,dt_o", [(torch.float32, torch.float32, torch.float32),
                                            (torch.bfloat16, torch.bfloat16, torch.bfloat16),
                                            (torch.bfloat16, torch.bfloat16, torch.float32),
                                            (torch.bfloat16, torch.float32, torch.bfloat16)])
def test_gemm_generic(ops, M, N, K, dt_x, dt_w, dt_o):
    x, w = rand(M, K, seed=5, dtype=dt_x), rand(N, K, seed=6, dtype=dt_w, scale=0.1)
    bias = rand(N, seed=7)
    want = P.linear(x.double(), w.double())
    got = ops.gemm(x.to(DEV), w.to(DEV), out_dtype=dt_o, algo=ops.ALGO_GENERIC)
    assert got.dtype == dt_o
    close(got, want, dt_o)
    got = ops.gemm(x.to(DEV), w.to(DEV), bias.to(DEV), out_dtype=dt_o, algo=ops.ALGO_GENERIC)
    close(got, want + bias.double(), dt_o)


def test_float32_gemm_keeps_what_reduced_precision_loses(ops):
    # 1 + 2^-12 is exact in float32, lost in bfloat16 or tf32-like modes
    x = torch.full((2, 64), 1.0 + 2.0 ** -12)
    w = torch.ones(3, 64)
    got = ops.gemm(x.to(DEV), w.to(DEV)).cpu()
    assert torch.equal(got, torch.full((2, 3), 64.0 * (1.0 + 2.0 ** -12)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul(ops, dtype):
    gu = rand(9, 2 * 112, seed=8, dtype=dtype, scale=2.0)
    got = ops.silu_mul(gu.to(DEV))
    g, u = gu[:, :112].float(), gu[:, 112:].float()
    close(got, P.silu_mul(g, u), dtype)
    ones = torch.cat([g, torch.ones_like(g)], dim=1).to(dtype)
    close(ops.silu_mul(ones.to(DEV)), torch.nn.functional.silu(ones[:, :112].float()), dtype)


def paged_cache(k, v, page, perm_seed, dtype, extra_pages=3):
    """k, v [L, Hkv, D] -> (cache [pages, 2, Hkv, P, D], block table row) with shuffled pages.
    A key tile is [P][D]; a value tile is stored transposed, [D][P]."""
    L, hkv, d = k.shape
    n = (L + page - 1) // page
    g = torch.Generator().manual_seed(perm_seed)
    ids = torch.randperm(n + extra_pages, generator=g)[:n]
    cache = torch.full((n + extra_pages, 2, hkv, page, d), float("nan")).to(dtype)
    vt = cache[:, 1].view(-1, hkv, d, page)               # the same memory, seen as [D][P] tiles
    for pos in range(L):
        cache[ids[pos // page], 0, :, pos % page] = k[pos]
        vt[ids[pos // page], :, :, pos % page] = v[pos]
    return cache, ids.to(torch.int32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,d,page", [(4, 2, 16, 4), (6, 1, 32, 8), (6, 2, 48, 16), (8, 8, 64, 1),
                                           (3, 3, 80, 5), (16, 8, 128, 16), (2, 1, 256, 64)])
def test_attention_over_pages(ops, dtype, hq, hkv, d, page):
    """Two requests in one batch: a portion of 9 tokens after 140 cached ones, and a decoded token
    at position 70.  Pages are shuffled and unused pages hold NaN."""
    scale = 1 / math.sqrt(d)
    lens = [(140, 9), (70, 1)]
    qs, pos, seq, tables, caches, want = [], [], [], [], [], []
    base_page = 0
    for b, (before, n) in enumerate(lens):
        L = before + n
        k, v = rand(L, hkv, d, seed=10 + b, dtype=dtype), rand(L, hkv, d, seed=20 + b, dtype=dtype)
        q = rand(n, hq, d, seed=30 + b, dtype=dtype)
        cache, ids = paged_cache(k, v, page, 40 + b, dtype)
        tables.append(ids + base_page)
        base_page += cache.shape[0]
        caches.append(cache)
        qs.append(q)
        pos += list(range(before, L))
        seq += [b] * n
        want.append(P.attention(q.float(), k.float(), v.float(), scale))
    width = max(len(t) for t in tables)
    table = torch.full((2, width), -1, dtype=torch.int32)
    for b, t in enumerate(tables):
        table[b, :len(t)] = t
    out = ops.attention(torch.cat(qs).to(DEV), torch.cat(caches).to(DEV),
                        torch.tensor(pos, dtype=torch.int32, device=DEV),
                        torch.tensor(seq, dtype=torch.int32, device=DEV), table.to(DEV), scale)
    assert not torch.isnan(out.float()).any()
    close(out, torch.cat(want), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [4, 16])
@pytest.mark.parametrize("key_pos", [0, 3, 4, 63, 64, 127, 128, 511, 700])
def test_one_far_key_among_hundreds_decides(ops, dtype, page, key_pos):
    """A query at position 700 whose score with one key stands out returns that key's value:
    a kernel that skips or misplaces a key (a page's edge, a chunk's edge, the first or the
    last key) returns something else."""
    hq = hkv = 2
    d, L = 32, 701
    k = rand(L, hkv, d, seed=50, dtype=dtype, scale=0.1)
    v = rand(L, hkv, d, seed=51, dtype=dtype)
    q = rand(1, hq, d, seed=52, dtype=dtype)
    k[key_pos] = (q[0].float() * 8).to(dtype)               # score ~ 8 |q|^2 / sqrt(d): far above the rest
    cache, ids = paged_cache(k, v, page, 53, dtype)
    out = ops.attention(q.to(DEV), cache.to(DEV), torch.tensor([L - 1], dtype=torch.int32, device=DEV),
                        torch.zeros(1, dtype=torch.int32, device=DEV), ids[None].to(DEV), 1 / math.sqrt(d))
    want = P.attention(q.float(), k.float(), v.float(), 1 / math.sqrt(d))
    close(out, want, dtype)
    assert float((want[0] - v[key_pos].float()).abs().max()) < 0.05     # the input does what it is meant to


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 5, 64, 65, 100])
def test_window_edge(ops, dtype, window):
    """The key just inside the window decides the result when it stands out; the key just
    outside must not, however large its score."""
    hq, hkv, d, L, page = 4, 2, 16, 300, 8
    scale = 1 / math.sqrt(d)
    q = rand(1, hq, d, seed=60, dtype=dtype)
    for standout in (L - window, L - window - 1):           # inside, outside
        k = rand(L, hkv, d, seed=61, dtype=dtype, scale=0.1)
        v = rand(L, hkv, d, seed=62, dtype=dtype)
        if standout >= 0:
            k[standout, 0] = (q[0, 0].float() * 8).to(dtype)
            k[standout, 1] = (q[0, 2].float() * 8).to(dtype)
        cache, ids = paged_cache(k, v, page, 63, dtype)
        # pages that the window has passed are given back: the table holds -1 there
        first_live = max(0, L - 1 - window + 1) // page
        ids = ids.clone()
        ids[:first_live] = -1
        out = ops.attention(q.to(DEV), cache.to(DEV), torch.tensor([L - 1], dtype=torch.int32, device=DEV),
                            torch.zeros(1, dtype=torch.int32, device=DEV), ids[None].to(DEV), scale, window=window)
        want = P.attention(q.float(), k.float(), v.float(), scale, window=window)
        close(out, want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,d,page", [(4, 2, 16, 4), (6, 1, 32, 8), (6, 2, 48, 16), (16, 8, 128, 16), (2, 2, 80, 3)])
def test_qk_norm_rope_store(ops, dtype, hq, hkv, d, page):
    T, pages, eps = 11, 9, 1e-5
    width = (hq + 2 * hkv) * d
    qkv = rand(T, width, seed=70, dtype=dtype)
    qw, kw = 1 + rand(d, seed=71, scale=0.1), 1 + rand(d, seed=72, scale=0.1)
    table = P.rope_table(10000.0, d, 64)
    pos = torch.tensor([0, 1, 2, 3, 40, 41, 63, 7, 8, 9, 10], dtype=torch.int32)
    slots = torch.tensor([5 * page + 0, 5 * page + 1, 2 * page + page - 1, 0, 1, 8 * page + page - 1,
                          3 * page, 4 * page, -1, 6 * page, 7 * page], dtype=torch.int32)
    if page == 1:
        slots = torch.arange(T, dtype=torch.int32)
    slots = torch.where(slots >= pages * page, torch.tensor(-1, dtype=torch.int32), slots)
    cache = torch.zeros(pages, 2, hkv, page, d, dtype=dtype, device=DEV)
    q_out = ops.qk_rope_store(qkv.to(DEV), hq, hkv, d, pos.to(DEV), qw.to(DEV), kw.to(DEV), eps,
                              table.to(DEV), slots.to(DEV), cache, page)
    x = qkv.float()
    q = x[:, :hq * d].view(T, hq, d)
    k = x[:, hq * d:(hq + hkv) * d].view(T, hkv, d)
    v = x[:, (hq + hkv) * d:].view(T, hkv, d)
    q_ref = P.apply_rope(table, pos, P.rms_norm(q, qw, eps))
    k_ref = P.apply_rope(table, pos, P.rms_norm(k, kw, eps))
    close(q_out, q_ref, dtype)
    want = torch.zeros(pages, 2, hkv, page, d)
    want_vt = want[:, 1].view(pages, hkv, d, page)         # value tiles are [D][P]
    for t in range(T):
        s = int(slots[t])
        if s >= 0:
            want[s // page, 0, :, s % page] = k_ref[t]
            want_vt[s // page, :, :, s % page] = v[t]
    close(cache, want, dtype)
    assert torch.equal(cache[:, 1].float().cpu(), want[:, 1].to(dtype).float())      # values are copied exactly
    # the steps apart: norm only into the packed form, then rotation and store from it
    packed = ops.qk_rope_store(qkv.to(DEV), hq, hkv, d, None, qw.to(DEV), kw.to(DEV), eps, None, None, None,
                               page, packed=True)
    close(packed[:, :hq], P.rms_norm(q, qw, eps), dtype)
    close(packed[:, hq:hq + hkv], P.rms_norm(k, kw, eps), dtype)
    assert torch.equal(packed[:, hq + hkv:].cpu().float(), v.to(dtype).float())
    no_norm = ops.qk_rope_store(qkv.to(DEV), hq, hkv, d, pos.to(DEV), None, None, 0.0, table.to(DEV), None, None, page)
    close(no_norm, P.apply_rope(table, pos, q), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hq,hkv,d,page", [(16, 8, 128, 16), (4, 2, 64, 32), (12, 4, 16, 16), (6, 1, 128, 20), (20, 20, 32, 8)])
def test_qk_norm_rope_store_of_many_tokens(ops, dtype, hq, hkv, d, page):
    """Enough tokens for the kernel that takes a token per block and writes values by tiles of 16
    tokens: a prompt from a page's start, one from the middle of a page, tokens whose slots are
    scattered, tokens without a slot, and a last tile of fewer than 16 tokens."""
    eps = 1e-6
    lens = [(0, 150), (page // 2 + 1, 100), (3, 16)]                  # (first position, tokens) of three requests
    T = sum(n for _, n in lens) + 24
    width = (hq + 2 * hkv) * d
    assert T * (hq + 2 * hkv) > 2048
    qkv = rand(T, width, seed=73, dtype=dtype)
    qw, kw = 1 + rand(d, seed=74, scale=0.1), 1 + rand(d, seed=75, scale=0.1)
    table = P.rope_table(10000.0, d, 256)
    pages = 40
    perm = torch.randperm(pages, generator=torch.Generator().manual_seed(76)).tolist()
    pos, slots = [], []
    for first, n in lens:                                             # consecutive slots through pages of its own
        mine = [perm.pop() for _ in range((first + n + page - 1) // page)]
        for p_ in range(first, first + n):
            pos.append(p_)
            slots.append(mine[p_ // page] * page + p_ % page)
    free = [pg * page + o for pg in perm[:4] for o in range(page)]
    g = torch.Generator().manual_seed(77)
    pick = torch.randperm(len(free), generator=g)[:24].tolist()
    for i in range(24):                                               # scattered, and every fifth without a slot
        pos.append(100 + i)
        slots.append(-1 if i % 5 == 4 else free[pick[i]])
    pos, slots = torch.tensor(pos, dtype=torch.int32), torch.tensor(slots, dtype=torch.int32)
    cache = torch.zeros(pages, 2, hkv, page, d, dtype=dtype, device=DEV)
    q_out = ops.qk_rope_store(qkv.to(DEV), hq, hkv, d, pos.to(DEV), qw.to(DEV), kw.to(DEV), eps,
                              table.to(DEV), slots.to(DEV), cache, page)
    x = qkv.float()
    q = x[:, :hq * d].view(T, hq, d)
    k = x[:, hq * d:(hq + hkv) * d].view(T, hkv, d)
    v = x[:, (hq + hkv) * d:].view(T, hkv, d)
    close(q_out, P.apply_rope(table, pos, P.rms_norm(q, qw, eps)), dtype)
    k_ref = P.apply_rope(table, pos, P.rms_norm(k, kw, eps))
    want = torch.zeros(pages, 2, hkv, page, d)
    want_vt = want[:, 1].view(pages, hkv, d, page)
    for t in range(T):
        s = int(slots[t])
        if s >= 0:
            want[s // page, 0, :, s % page] = k_ref[t]
            want_vt[s // page, :, :, s % page] = v[t]
    close(cache, want, dtype)
    assert torch.equal(cache[:, 1].float().cpu(), want[:, 1].to(dtype).float())      # values are copied exactly


@pytest.mark.parametrize("hq,hkv,d,page", [(6, 2, 128, 16), (5, 3, 64, 32), (4, 1, 16, 16)])
@pytest.mark.parametrize("norm,rope,bias", [(True, True, False), (False, True, True), (True, False, True)])
def test_norm_rotation_and_cache_write_from_partial_products(ops, hq, hkv, d, page, norm, rope, bias):
    """The projection as three 32-bit partial products (+ bias): the kernel adds them in order, rounds
    to bfloat16 and goes on as on a stored projection, to the bit.  Tokens in runs of 16 side by
    side in a page (values written by tiles), a run across a page's edge, scattered slots, a token
    without a slot."""
    bf = torch.bfloat16
    width, T, eps = (hq + 2 * hkv) * d, 260, 1e-6
    parts = torch.stack([rand(T, width, seed=610 + i, scale=0.6) for i in range(3)])
    b = rand(width, seed=613) if bias else None
    summed = parts[0] + parts[1] + parts[2]
    qkv = (summed + b if bias else summed).to(bf)
    qw = 1 + rand(d, seed=614, scale=0.1) if norm else None
    kw = 1 + rand(d, seed=615, scale=0.1) if norm else None
    table = P.rope_table(10000.0, d, 600) if rope else None
    pages = 40
    g = torch.Generator().manual_seed(616)
    second = (3 * page + 200 + page - 1) // page * page + page + page // 2
    slots = list(range(3 * page, 3 * page + 200)) + [second + i for i in range(28)]   # 200 in a row, 28 from the middle of a page
    free = [s_ for s_ in torch.randperm(pages * page, generator=g).tolist() if s_ not in set(slots)]
    slots += free[:T - len(slots)]
    slots[100] = -1
    positions = torch.randint(0, 600, (T,), generator=g).to(torch.int32)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    dev = lambda t: None if t is None else t.to(DEV)
    caches = [torch.full((pages, 2, hkv, page, d), 7.0, dtype=bf, device=DEV) for _ in range(2)]
    assert ops.qk_rope_store_parts_supported(d, dev(table))
    q1 = ops.qk_rope_store_parts(parts.to(DEV), dev(b), hq, hkv, d, positions.to(DEV) if rope else None, dev(qw), dev(kw),
                                 eps, dev(table), i32(slots), caches[0], page)
    q2 = ops.qk_rope_store(qkv.to(DEV), hq, hkv, d, positions.to(DEV) if rope else None, dev(qw), dev(kw), eps, dev(table),
                           i32(slots), caches[1], page)
    assert torch.equal(q1, q2) and torch.equal(caches[0], caches[1])
    assert not torch.equal(caches[0], torch.full_like(caches[0], 7.0))
    # a rotation over part of the head is not taken
    if rope and d >= 32:
        assert not ops.qk_rope_store_parts_supported(d, P.rope_table(10000.0, d // 2, 10))


@pytest.mark.parametrize("hq,hkv,page,K", [(16, 8, 16, 1024), (3, 2, 32, 96), (5, 1, 16, 160)])
@pytest.mark.parametrize("norm,rope,bias", [(True, True, False), (False, True, True), (True, False, False),
                                            (False, False, False)])
def test_qkv_product_with_norm_rotation_and_cache_write_inside(ops, hq, hkv, page, K, norm, rope, bias):
    """The tiled product that norms, rotates and writes the cache from its own result, in every
    tile shape, against the plain functions and against the product followed by the separate
    kernel (the same arithmetic on the same rounded product: equal to the bit).  Tokens: a prompt
    from a page's start (runs of 16 side by side), one from the middle of a page, scattered
    slots, tokens without a slot; the number of tokens is no multiple of a tile."""
    bf, d, eps = torch.bfloat16, 128, 1e-6
    lens = [(0, 200), (page // 2 + 1, 100), (3, 16)]
    T = sum(n for _, n in lens) + 24
    width = (hq + 2 * hkv) * d
    assert T * (hq + 2 * hkv) > 2048                                  # (the separate kernel is then the one with the same order of sums)
    x = rand(T, K, seed=600, dtype=bf)
    w = rand(width, K, seed=601, dtype=bf, scale=1.0 / math.sqrt(K))
    b = rand(width, seed=602, scale=0.5) if bias else None
    qw = 1 + rand(d, seed=603, scale=0.1) if norm else None
    kw = 1 + rand(d, seed=604, scale=0.1) if norm else None
    table = P.rope_table(10000.0, d, 256) if rope else None
    pages = 40
    perm = torch.randperm(pages, generator=torch.Generator().manual_seed(605)).tolist()
    pos, slots = [], []
    for first, n in lens:
        mine = [perm.pop() for _ in range((first + n + page - 1) // page)]
        for p_ in range(first, first + n):
            pos.append(p_)
            slots.append(mine[p_ // page] * page + p_ % page)
    free = [pg * page + o for pg in perm[:4] for o in range(page)]
    pick = torch.randperm(len(free), generator=torch.Generator().manual_seed(606))[:24].tolist()
    for i in range(24):
        pos.append(100 + i)
        slots.append(-1 if i % 5 == 4 else free[pick[i]])
    pos, slots = torch.tensor(pos, dtype=torch.int32), torch.tensor(slots, dtype=torch.int32)
    dev = lambda t: None if t is None else t.to(DEV)
    # the product and the separate kernel
    cache2 = torch.zeros(pages, 2, hkv, page, d, dtype=bf, device=DEV)
    qkv = ops.gemm(x.to(DEV), w.to(DEV), dev(b))
    q2 = ops.qk_rope_store(qkv, hq, hkv, d, dev(pos) if rope else None, dev(qw), dev(kw), eps, dev(table),
                           dev(slots), cache2, page)
    # the plain functions on the rounded product
    y = qkv.float().cpu()
    qr = y[:, :hq * d].view(T, hq, d)
    kr = y[:, hq * d:(hq + hkv) * d].view(T, hkv, d)
    if norm:
        qr, kr = P.rms_norm(qr, qw, eps), P.rms_norm(kr, kw, eps)
    if rope:
        qr, kr = P.apply_rope(table, pos, qr), P.apply_rope(table, pos, kr)
    assert ops.gemm_qkv_supported(x.to(DEV), w.to(DEV), cache2, hq, dev(table))
    for tile in (0, 64, 128, 256, 512):
        cache = torch.zeros(pages, 2, hkv, page, d, dtype=bf, device=DEV)
        q = ops.gemm_qkv(x.to(DEV), w.to(DEV), dev(b), hq, cache, dev(pos) if rope else None, dev(qw), dev(kw), eps,
                         dev(table), dev(slots), tile=tile)
        close(q, qr, bf)
        assert torch.equal(q, q2), f"tile {tile}: q differs from the separate kernel's"
        assert torch.equal(cache, cache2), f"tile {tile}: the cache differs from the separate kernel's"
    # without slots nothing is written
    cache = torch.zeros(pages, 2, hkv, page, d, dtype=bf, device=DEV)
    q = ops.gemm_qkv(x.to(DEV), w.to(DEV), dev(b), hq, cache, dev(pos) if rope else None, dev(qw), dev(kw), eps,
                     dev(table), None)
    assert torch.equal(q, q2) and not bool(cache.any())
    assert not ops.gemm_qkv_supported(x[:64].to(DEV), w.to(DEV), cache, hq, dev(table))      # few rows: not this kernel's


def test_argmax_takes_the_lowest_index_on_ties(ops):
    logits = rand(5, 50000, seed=80)
    logits[0, 49999] = 9.0
    logits[1, 0] = 9.0
    logits[2, 777] = logits[2, 40001] = 9.0                  # a tie: the lower index wins
    logits[3] = -3.0                                         # all equal
    logits[4, 255] = logits[4, 256] = 9.0                    # a tie across two threads' strides
    got = ops.argmax(logits.to(DEV)).cpu().tolist()
    assert got == [49999, 0, 777, 0, 255]
    assert got == P.greedy(logits)
    odd = rand(3, 331, seed=81)
    assert ops.argmax(odd.to(DEV)).cpu().tolist() == P.greedy(odd)
    wide = rand(7, 151936, seed=85)                          # the two-stage form for wide vocabularies
    wide[1, 2047] = wide[1, 2048] = wide[1, 151935] = 9.0    # ties across spans
    wide[2, 151935] = 9.0
    wide[3] = 1.5
    got = ops.argmax(wide.to(DEV)).cpu().tolist()
    assert got == P.greedy(wide) and got[1] == 2047 and got[2] == 151935 and got[3] == 0


def test_temperature_sampling_is_the_inverse_cdf(ops):
    V = 331
    logits = rand(64, V, seed=82, scale=2.0)
    temps = torch.tensor([0.7, 1.0, 1.5, 0.2] * 16)
    us = torch.rand(64, generator=torch.Generator().manual_seed(83))
    us[0], us[1] = 0.0, 1.0 - 2.0 ** -24
    got = ops.sample(logits.to(DEV), temps.to(DEV), us.to(DEV)).cpu().tolist()
    cdf = torch.softmax(logits.double() / temps.double()[:, None], dim=-1).cumsum(-1)
    for r, tok in enumerate(got):
        lo = float(cdf[r, tok - 1]) if tok > 0 else 0.0
        hi = float(cdf[r, tok])
        assert lo - 1e-5 <= float(us[r]) <= hi + 1e-5, (r, tok, lo, float(us[r]), hi)
    # a low temperature approaches greedy
    cold = ops.sample(logits.to(DEV), torch.full((64,), 1e-3, device=DEV), us.to(DEV)).cpu().tolist()
    assert cold == P.greedy(logits)
    # frequencies follow the distribution
    row = torch.tensor([[2.0, 1.0, 0.0, -1.0, 0.5]]).repeat(4000, 1)
    u = torch.rand(4000, generator=torch.Generator().manual_seed(84))
    draws = ops.sample(row.to(DEV), torch.ones(4000, device=DEV), u.to(DEV)).cpu()
    freq = torch.bincount(draws, minlength=5).double() / 4000
    assert (freq - torch.softmax(row[0].double(), -1)).abs().max() < 0.03


def test_kernels_refuse_what_they_do_not_take(ops):
    x = torch.zeros(4, 8, device=DEV)
    with pytest.raises(ops.KernelError):
        ops.gemm(x, torch.zeros(3, 9, device=DEV))                       # inner sizes differ
    with pytest.raises(ops.KernelError):
        ops.gemm(x, torch.zeros(3, 8, device=DEV, dtype=torch.bfloat16))  # 32-bit activations, 16-bit weights
    with pytest.raises(ops.KernelError):
        ops.gemm(x.t(), torch.zeros(3, 4, device=DEV))                   # not contiguous
    with pytest.raises(ops.KernelError):
        ops.rmsnorm(x, torch.ones(7, device=DEV), 1e-6, torch.float32)
    with pytest.raises(ops.KernelError):
        ops.embedding(torch.zeros(3, dtype=torch.int64, device=DEV), x)  # ids must be int32
    q = torch.zeros(1, 3, 16, device=DEV)
    cache = torch.zeros(2, 2, 2, 4, 16, device=DEV)
    i32 = lambda *v: torch.tensor(v, dtype=torch.int32, device=DEV)
    with pytest.raises(ops.KernelError):
        ops.attention(q, cache, i32(0), i32(0), i32(0)[None], 1.0)       # 3 heads on 2 kv heads
    big = torch.zeros(1, 2, 272, device=DEV)
    with pytest.raises(ops.KernelError):
        ops.attention(big, torch.zeros(2, 2, 2, 4, 272, device=DEV), i32(0), i32(0), i32(0)[None], 1.0)
    with pytest.raises(ops.KernelError):
        ops.silu_mul(torch.zeros(2, 7, device=DEV))


# ---- the MFMA kernels of the bfloat16 mode -------------------------------------------------------
@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(64, 64), (500, 96), (331, 160), (4096, 1024), (1024, 3072)])
def test_gemm_for_few_rows(ops, M, N, K):
    bf = torch.bfloat16
    x, w = rand(M, K, seed=90, dtype=bf), rand(N, K, seed=91, dtype=bf, scale=0.1)
    bias = rand(N, seed=92)
    assert ops.gemm_fused_supported(x.to(DEV), w.to(DEV))
    want = P.linear(x.double(), w.double())
    for dt_o in (bf, torch.float32):
        got = ops.gemm(x.to(DEV), w.to(DEV), out_dtype=dt_o, algo=ops.ALGO_FAST)
        close(got, want, dt_o if dt_o == bf else torch.float32, scale=float(want.abs().max()))
    close(ops.gemm(x.to(DEV), w.to(DEV), bias.to(DEV), algo=ops.ALGO_FAST), want + bias.double(), bf)
    # added into the 32-bit stream
    h = rand(M, N, seed=93)
    hd = h.to(DEV)
    ops.gemm(x.to(DEV), w.to(DEV), out=hd, epilogue=ops.EPI_RESIDUAL)
    close(hd, h.double() + want, torch.float32, scale=float(want.abs().max()))
    # cut along K into partial products, which the norm adds up
    for splits in (0, 1, 3):
        parts = ops.gemm(x.to(DEV), w.to(DEV), epilogue=ops.EPI_PARTIAL, splits=splits)
        assert parts.dtype == torch.float32 and parts.dim() == 3 and (splits == 0 or parts.shape[0] == splits)
        close(parts.sum(0), want, torch.float32, scale=float(want.abs().max()))
    hd = h.to(DEV)
    nw = 1 + rand(N, seed=96, scale=0.1)
    normed = ops.rmsnorm(hd, nw.to(DEV), 1e-6, bf, delta=parts)
    total = h.double() + parts.double().cpu().sum(0)
    close(hd, total, torch.float32)
    close(normed, P.rms_norm(total.float(), nw, 1e-6), bf)


@pytest.mark.parametrize("N", [48, 8192])
@pytest.mark.parametrize("K", [512, 1536, 2048, 2560, 5120])
def test_gemm_for_few_rows_over_rounds_of_chunks(ops, N, K):
    """The kernel for few rows has a form for blocks whose waves read their chunks of K in one round and a form
    that runs several rounds with the next round's loads in flight (pairs of rounds, then one or two): K from
    one round to five or more, with and without a cut along K, for one to four tiles of 16 rows of x and for
    one and two tiles of outputs a block; silu.mul in both layouts of gate and up.  In 64-bit on drawn columns."""
    bf = torch.bfloat16
    g = torch.Generator().manual_seed(1000 * N + K)
    w = (torch.randn(N, K, generator=g) * 0.05).to(bf)
    wd = w.to(DEV)
    cols = torch.randint(0, N, (192,), generator=g) if N > 192 else torch.arange(N)
    wc, cd = w[cols].double(), cols.to(DEV)
    half = N // 2
    w_il = ops.interleave_gate_up(wd[:half], wd[half:]) if half % 32 == 0 else None
    for M in (1, 8, 16, 17, 32, 33, 49, 64):
        x = torch.randn(M, K, generator=g).to(bf)
        xd = x.to(DEV)
        want = x.double() @ wc.t()
        scale = float(want.abs().max())
        got = ops.gemm(xd, wd, out_dtype=torch.float32, algo=ops.ALGO_FAST)[:, cd]
        assert float((got.double().cpu() - want).abs().max()) <= 3e-6 * scale, ("store", M)
        for splits in (2, 3):
            parts = ops.gemm(xd, wd, epilogue=ops.EPI_PARTIAL, splits=splits)
            assert float((parts.sum(0)[:, cd].double().cpu() - want).abs().max()) <= 3e-6 * scale, ("partial", splits, M)
        gu = x.double() @ w.double().t()
        want_g = P.silu_mul(gu[:, :half], gu[:, half:])
        got = ops.gemm(xd, wd, epilogue=ops.EPI_SILU_MUL, out_dtype=torch.float32)
        assert float((got.double().cpu() - want_g).abs().max()) <= 1e-5 * float(want_g.abs().max()), ("silu", M)
        if w_il is not None and ops.gemm_silu_supported(xd, w_il):
            got = ops.gemm(xd, w_il, epilogue=ops.EPI_SILU_MUL_IL, out_dtype=torch.float32)
            assert float((got.double().cpu() - want_g).abs().max()) <= 1e-5 * float(want_g.abs().max()), ("silu, interleaved", M)


@pytest.mark.parametrize("N,K", [(8201, 2112), (9000, 2080), (8200, 4160)])
def test_gemm_for_few_rows_whose_sizes_are_no_multiples_of_the_tiles(ops, N, K):
    """A matrix large enough for the whole-line loads whose last tile of rows is partly beyond the matrix, with
    a K of 33 and 65 lines and with one that is no whole number of lines (which takes the other form), for
    row counts inside the first and the third tile of 16: every output, in 64-bit."""
    bf = torch.bfloat16
    g = torch.Generator().manual_seed(N + K)
    w = (torch.randn(N, K, generator=g) * 0.05).to(bf)
    wd = w.to(DEV)
    for M in (1, 3, 11, 16, 40):
        x = torch.randn(M, K, generator=g).to(bf)
        want = x.double() @ w.double().t()
        scale = float(want.abs().max())
        got = ops.gemm(x.to(DEV), wd, out_dtype=torch.float32)
        assert float((got.double().cpu() - want).abs().max()) <= 3e-6 * scale, ("store", M)
        for splits in (2, 4):
            parts = ops.gemm(x.to(DEV), wd, epilogue=ops.EPI_PARTIAL, splits=splits)
            assert float((parts.sum(0).double().cpu() - want).abs().max()) <= 3e-6 * scale, ("partial", splits, M)


@pytest.mark.parametrize("M", [1, 8, 40, 64])
@pytest.mark.parametrize("I,K", [(160, 96), (112, 64), (3072, 1024)])
def test_gemm_with_silu_mul(ops, M, I, K):
    bf = torch.bfloat16
    x, w = rand(M, K, seed=94, dtype=bf), rand(2 * I, K, seed=95, dtype=bf, scale=0.2)
    got = ops.gemm(x.to(DEV), w.to(DEV), epilogue=ops.EPI_SILU_MUL)
    gu = P.linear(x.double(), w.double())
    close(got, P.silu_mul(gu[:, :I], gu[:, I:]), bf)


def test_gemm_for_few_rows_refuses_other_shapes(ops):
    bf = torch.bfloat16
    x = torch.zeros(4, 80, dtype=bf, device=DEV)             # K = 80 is no multiple of 32
    w = torch.zeros(16, 80, dtype=bf, device=DEV)
    assert not ops.gemm_fused_supported(x, w)
    with pytest.raises(ops.KernelError):
        ops.gemm(x, w, algo=ops.ALGO_FAST)
    ops.gemm(x, w)                                           # the generic kernel takes it
    big = torch.zeros(65, 64, dtype=bf, device=DEV)
    assert not ops.gemm_fused_supported(big, torch.zeros(16, 64, dtype=bf, device=DEV))
    f = torch.zeros(4, 64, device=DEV)
    assert not ops.gemm_fused_supported(f, torch.zeros(16, 64, device=DEV))


@pytest.mark.parametrize("hq,hkv,d,page", [(16, 8, 128, 16), (8, 8, 64, 16), (32, 4, 128, 32), (16, 1, 64, 64), (6, 2, 128, 16)])
@pytest.mark.parametrize("window", [0, 200])
def test_decode_attention_kernel(ops, hq, hkv, d, page, window):
    """Five requests with one new token each, at positions that end inside a tile, at a tile's and at
    a split's edge; pages shuffled, unwritten parts of pages hold NaN."""
    bf = torch.bfloat16
    scale = 1 / math.sqrt(d)
    positions = [0, 15, 16, 127, 128, 700]
    qs, tables, caches, want = [], [], [], []
    base = 0
    for b, p in enumerate(positions):
        L = p + 1
        k, v = rand(L, hkv, d, seed=100 + b, dtype=bf), rand(L, hkv, d, seed=200 + b, dtype=bf)
        q = rand(1, hq, d, seed=300 + b, dtype=bf)
        cache, ids = paged_cache(k, v, page, 400 + b, bf)
        tables.append(ids + base)
        base += cache.shape[0]
        caches.append(cache)
        qs.append(q)
        want.append(P.attention(q.float(), k.float(), v.float(), scale, window=window or None))
    width = max(len(t) for t in tables)
    table = torch.full((len(positions), width), -1, dtype=torch.int32)
    for b, t in enumerate(tables):
        table[b, :len(t)] = t
    B = len(positions)
    qd, cd = torch.cat(qs).to(DEV), torch.cat(caches).to(DEV)
    assert ops.attention_decode_supported(qd, cd)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    out = ops.attention(qd, cd, i32(positions), i32(list(range(B))), table.to(DEV), scale, window=window,
                        dec_tokens=i32(list(range(B))), max_dec_position=max(positions))
    assert not torch.isnan(out.float()).any()
    close(out, torch.cat(want), bf)
    # a subset through the decode kernel, the rest through the generic one: every row is written once
    out2 = ops.attention(qd, cd, i32(positions), i32(list(range(B))), table.to(DEV), scale, window=window,
                         dec_tokens=i32([5, 1, 3]), max_dec_position=700, other_tokens=i32([0, 2, 4]))
    close(out2, torch.cat(want), bf)
    # the hint that some requests' first keys are read by others chooses between two kinds of loads: the same bits
    out3 = ops.attention(qd, cd, i32(positions), i32(list(range(B))), table.to(DEV), scale, window=window,
                         dec_tokens=i32(list(range(B))), max_dec_position=max(positions),
                         shared_keys=i32([0, 16, 0, 64, 129, 300]))
    assert torch.equal(out3, out)
    with pytest.raises(ops.KernelError):                      # an entry per row of the table
        ops.attention(qd, cd, i32(positions), i32(list(range(B))), table.to(DEV), scale, window=window,
                      dec_tokens=i32(list(range(B))), max_dec_position=max(positions), shared_keys=i32([0, 16]))


@pytest.mark.parametrize("hq,hkv,d,page", [(16, 8, 128, 16), (4, 4, 64, 16), (8, 1, 128, 32), (6, 2, 64, 48), (16, 1, 64, 16)])
@pytest.mark.parametrize("window", [0, 40])
@pytest.mark.parametrize("norm,rope", [(True, True), (False, True), (True, False)])
def test_decode_attention_with_norm_rotation_and_cache_write_inside(ops, hq, hkv, d, page, window, norm, rope):
    """Single new tokens at positions that are first in the cache, first of a page, first and last
    of a split of 128 keys and in the middle of one: the kernel that norms and rotates q and k
    itself, takes the new key and value from registers and writes them to the cache, against the
    plain functions; and against the separate kernels on the same operands."""
    bf = torch.bfloat16
    scale, eps = 1 / math.sqrt(d), 1e-6
    positions = [0, 1, page, 127, 128, 129, 255, 256, 300, 700]
    B = len(positions)
    width = (hq + 2 * hkv) * d
    qkv = rand(B, width, seed=510, dtype=bf)
    qw = 1 + rand(d, seed=511, scale=0.1) if norm else None
    kw = 1 + rand(d, seed=512, scale=0.1) if norm else None
    table = P.rope_table(10000.0, d, 1024) if rope else None
    caches, tables, slots, want, k_new, base = [], [], [], [], [], 0
    for b, p in enumerate(positions):
        L = p + 1
        k, v = rand(L, hkv, d, seed=520 + b, dtype=bf), rand(L, hkv, d, seed=540 + b, dtype=bf)
        x = qkv[b].float()
        q_b = x[:hq * d].view(1, hq, d)
        k_b = x[hq * d:(hq + hkv) * d].view(1, hkv, d)
        v_b = x[(hq + hkv) * d:].view(1, hkv, d)
        pos_b = torch.tensor([p], dtype=torch.int32)
        if norm:
            q_b, k_b = P.rms_norm(q_b, qw, eps), P.rms_norm(k_b, kw, eps)
        if rope:
            q_b, k_b = P.apply_rope(table, pos_b, q_b), P.apply_rope(table, pos_b, k_b)
        q_b, k_b = q_b.to(bf).float(), k_b.to(bf).float()
        k_new.append(k_b[0])
        keys = torch.cat([k[:p].float(), k_b]) if p else k_b
        vals = torch.cat([v[:p].float(), v_b]) if p else v_b
        want.append(P.attention(q_b, keys, vals, scale, window=window or None))
        # the cache holds the keys before p; the slot of p itself holds NaN until the kernel writes it
        k[p], v[p] = float("nan"), float("nan")
        cache, ids = paged_cache(k, v, page, 560 + b, bf)
        tables.append(ids + base)
        slots.append(int(ids[p // page] + base) * page + p % page)
        base += cache.shape[0]
        caches.append(cache)
    slots[4] = -1                                            # one token without a slot: nothing is written for it
    cache = torch.cat(caches)
    width_t = max(len(t) for t in tables)
    tab = torch.full((B, width_t), -1, dtype=torch.int32)
    for b, t in enumerate(tables):
        tab[b, :len(t)] = t
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    dev = lambda t: None if t is None else t.to(DEV)
    cd = cache.to(DEV)
    assert ops.attention_decode_fused_supported(qkv.to(DEV), cd, hq, dev(table))
    out = ops.attention_decode_fused(qkv.to(DEV), hq, cd, i32(positions), i32(list(range(B))), tab.to(DEV), scale,
                                     window, i32(list(range(B))), max(positions), dev(qw), dev(kw), eps, dev(table),
                                     i32(slots))
    assert not torch.isnan(out.float()).any()
    close(out, torch.cat(want), bf)
    # the cache afterwards: the new key (normed, rotated) and value at the slot, nothing else touched
    after = cd.cpu()
    vt_after = after[:, 1].reshape(after.shape[0], hkv, d, page)
    x = qkv.float()
    for b, p in enumerate(positions):
        s = slots[b]
        if s < 0:
            continue
        close(after[s // page, 0, :, s % page], k_new[b], bf)
        assert torch.equal(vt_after[s // page, :, :, s % page].float(), x[b, (hq + hkv) * d:].view(hkv, d))
    untouched = torch.ones_like(cache, dtype=torch.bool)
    vt_mask = untouched[:, 1].view(cache.shape[0], hkv, d, page)
    for s in slots:
        if s >= 0:
            untouched[s // page, 0, :, s % page] = False
            vt_mask[s // page, :, :, s % page] = False
    same = (after == cache) | (torch.isnan(after.float()) & torch.isnan(cache.float()))
    assert bool(same[untouched].all())
    # the separate kernels on the same operands give the same rows (to rounding of the norm's sum)
    cd2 = cache.to(DEV)
    q2 = ops.qk_rope_store(qkv.to(DEV), hq, hkv, d, i32(positions) if rope else None, dev(qw), dev(kw), eps, dev(table),
                           i32(slots), cd2, page)
    out2 = ops.attention(q2, cd2, i32(positions), i32(list(range(B))), tab.to(DEV), scale, window=window,
                         dec_tokens=i32([b for b in range(B) if slots[b] >= 0]), max_dec_position=max(positions))
    rows = [b for b in range(B) if slots[b] >= 0]
    close(out[rows], out2[rows].float().cpu(), bf)
    # without a list of rows every row is taken, in order: the same results to the bit
    out3 = ops.attention_decode_fused(qkv.to(DEV), hq, cache.to(DEV), i32(positions), i32(list(range(B))), tab.to(DEV),
                                      scale, window, None, max(positions), dev(qw), dev(kw), eps, dev(table), i32(slots))
    assert torch.equal(out3, out)
    # ... and with the hint that other requests read some requests' first keys too (another kind of load there)
    out4 = ops.attention_decode_fused(qkv.to(DEV), hq, cache.to(DEV), i32(positions), i32(list(range(B))), tab.to(DEV),
                                      scale, window, None, max(positions), dev(qw), dev(kw), eps, dev(table), i32(slots),
                                      shared_keys=i32([(64 * b) % 200 for b in range(B)]))
    assert torch.equal(out4, out)


@pytest.mark.parametrize("key_pos", [0, 15, 16, 127, 128, 255, 256, 1000, 1023])
def test_decode_kernel_one_far_key_decides(ops, key_pos):
    bf = torch.bfloat16
    hq, hkv, d, L, page = 4, 2, 128, 1024, 16
    k = rand(L, hkv, d, seed=500, dtype=bf, scale=0.1)
    v = rand(L, hkv, d, seed=501, dtype=bf)
    q = rand(1, hq, d, seed=502, dtype=bf)
    k[key_pos, 0] = (q[0, 1].float() * 4).to(bf)            # head 1 of group 0, head 3 of group 1
    k[key_pos, 1] = (q[0, 3].float() * 4).to(bf)
    cache, ids = paged_cache(k, v, page, 503, bf)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    out = ops.attention(q.to(DEV), cache.to(DEV), i32([L - 1]), i32([0]), ids[None].to(DEV), 1 / math.sqrt(d),
                        dec_tokens=i32([0]), max_dec_position=L - 1)
    want = P.attention(q.float(), k.float(), v.float(), 1 / math.sqrt(d))
    close(out, want, bf)
    assert float((want[0, 1] - v[key_pos, 0].float()).abs().max()) < 0.05


@pytest.mark.parametrize("M,N,K", [(65, 64, 64), (128, 128, 64), (200, 331, 96), (257, 500, 160), (2048, 1024, 1024),
                                   (300, 3072, 1024), (130, 152, 2048), (17, 200, 64), (33, 40000, 96)])
def test_gemm_tiled_mfma(ops, M, N, K):
    bf = torch.bfloat16
    x, w = rand(M, K, seed=110, dtype=bf), rand(N, K, seed=111, dtype=bf, scale=0.1)
    bias = rand(N, seed=112)
    want = P.linear(x.double(), w.double())
    got = ops.gemm(x.to(DEV), w.to(DEV), algo=ops.ALGO_FAST)
    close(got, want, bf)
    for rows in (64, 65, 128, 256, 512):                     # every tile shape on every size (512: 256 x 256; 65: 64 rows, k step 128)
        close(ops.gemm(x.to(DEV), w.to(DEV), algo=ops.ALGO_TILE + rows), want, bf)
        close(ops.gemm(x.to(DEV), w.to(DEV), bias.to(DEV), out_dtype=torch.float32, algo=ops.ALGO_TILE + rows),
              want + bias.double(), torch.float32, scale=float(want.abs().max()))
    got32 = ops.gemm(x.to(DEV), w.to(DEV), bias.to(DEV), out_dtype=torch.float32, algo=ops.ALGO_FAST)
    close(got32, want + bias.double(), torch.float32, scale=float(want.abs().max()))
    # the generic kernel on the same operands agrees to accumulation order
    close(ops.gemm(x.to(DEV), w.to(DEV), out_dtype=torch.float32, algo=ops.ALGO_GENERIC), want, torch.float32,
          scale=float(want.abs().max()))
    with pytest.raises(ops.KernelError):
        ops.gemm(torch.zeros(100, 76, dtype=bf, device=DEV), torch.zeros(8, 76, dtype=bf, device=DEV), algo=ops.ALGO_FAST)


@pytest.mark.parametrize("M", [17, 40, 64])
def test_gemm_of_few_rows_against_a_large_matrix(ops, M):
    """17 to 64 rows against a matrix of 16 M elements or more go through the tiled kernel (the one
    for few rows reads mostly activations there): plain, cut along K into partial products, and
    with silu.mul over interleaved gate|up rows."""
    bf = torch.bfloat16
    N, K = 4224, 4096
    x, w = rand(M, K, seed=180, dtype=bf), rand(N, K, seed=181, dtype=bf, scale=0.05)
    bias = rand(N, seed=182)
    want = P.linear(x.double(), w.double())
    xd, wd = x.to(DEV), w.to(DEV)
    close(ops.gemm(xd, wd), want, bf)
    close(ops.gemm(xd, wd, bias.to(DEV), out_dtype=torch.float32), want + bias.double(), torch.float32,
          scale=float(want.abs().max()))
    for splits in (0, 1, 5, 16):
        parts = ops.gemm(xd, wd, epilogue=ops.EPI_PARTIAL, splits=splits)
        assert parts.dtype == torch.float32 and parts.dim() == 3 and (splits == 0 or parts.shape[0] == splits)
        close(parts.sum(0), want, torch.float32, scale=float(want.abs().max()))
    # the norm adds the parts up, as after the attention and the feed-forward
    h = rand(M, N, seed=183)
    hd = h.to(DEV)
    nw = 1 + rand(N, seed=184, scale=0.1)
    parts = ops.gemm(xd, wd, epilogue=ops.EPI_PARTIAL)
    normed = ops.rmsnorm(hd, nw.to(DEV), 1e-6, bf, delta=parts)
    total = h.double() + parts.double().cpu().sum(0)
    close(hd, total, torch.float32)
    close(normed, P.rms_norm(total.float(), nw, 1e-6), bf)
    # gate|up: 2 * 2112 rows of 4096
    I = N // 2
    g, u = w[:I], w[I:]
    wil = ops.interleave_gate_up(g.to(DEV), u.to(DEV))
    assert ops.gemm_silu_supported(xd, wil)
    got = ops.gemm(xd, wil, epilogue=ops.EPI_SILU_MUL_IL)
    close(got, P.silu_mul(P.linear(x.double(), g.double()), P.linear(x.double(), u.double())), bf)


@pytest.mark.parametrize("hq,hkv,d,page", [(16, 8, 128, 16), (4, 4, 64, 16), (8, 1, 128, 32), (6, 2, 64, 64), (8, 2, 128, 48)])
@pytest.mark.parametrize("window", [0, 40, 17])
def test_prefill_attention_kernel(ops, hq, hkv, d, page, window):
    """Three requests in one batch: a whole prompt of 75 tokens, a portion of 37 tokens after 100
    cached ones, and one of 2 tokens after 15; beside a decoded token.  Pages shuffled, unwritten
    parts of pages NaN."""
    bf = torch.bfloat16
    scale = 1 / math.sqrt(d)
    lens = [(0, 75), (100, 37), (15, 2), (33, 1)]
    qs, pos, seq, tables, caches, want, portions, dec, other = [], [], [], [], [], [], [], [], []
    base, row = 0, 0
    R = ops.prefill_tile_rows(hq, hkv)
    assert R == 32 // (hq // hkv) if (hq // hkv) in (1, 2, 4, 8, 16, 32) else R == 32
    for b, (before, n) in enumerate(lens):
        L = before + n
        k, v = rand(L, hkv, d, seed=120 + b, dtype=bf), rand(L, hkv, d, seed=130 + b, dtype=bf)
        q = rand(n, hq, d, seed=140 + b, dtype=bf)
        cache, ids = paged_cache(k, v, page, 150 + b, bf)
        tables.append(ids + base)
        base += cache.shape[0]
        caches.append(cache)
        qs.append(q)
        pos += list(range(before, L))
        seq += [b] * n
        want.append(P.attention(q.float(), k.float(), v.float(), scale, window=window or None))
        if n == 1:
            dec.append(row)
        else:
            other += list(range(row, row + n))
            portions.append((row, n))
        row += n
    from qwen_engine_amd.parts.attention import prefill_tiles
    tiles = torch.tensor(prefill_tiles(portions, R), dtype=torch.int32).view(-1, 2).tolist()
    width = max(len(t) for t in tables)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    for b, t in enumerate(tables):
        table[b, :len(t)] = t
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    for groups in (0, 1, 2):                     # wave groups a block: chosen by the kernel, one, two
        out = ops.attention(torch.cat(qs).to(DEV), torch.cat(caches).to(DEV), i32(pos), i32(seq), table.to(DEV), scale,
                            window=window, dec_tokens=i32(dec), max_dec_position=33, other_tokens=i32(other),
                            other_tiles=i32(tiles), prefill_groups=groups)
        assert not torch.isnan(out.float()).any()
        close(out, torch.cat(want), bf)


@pytest.mark.parametrize("rows_per_tile", [16, 32, 4])
def test_prefill_tiles_made_on_the_device(ops, rows_per_tile):
    """The tile list cut from portions that lie on the device equals the list made on the host, filled up
    with groups of no rows; a portion of no rows gives none."""
    from qwen_engine_amd.parts.attention import prefill_tiles
    for portions in ([(0, 75)], [(3, 0), (3, 500)], [(8, 37), (45, 91)], [(0, 1), (1, 2), (3, 300)], [(16, 127), (143, 385)]):
        want = prefill_tiles([p for p in portions if p[1] > 0], rows_per_tile)
        groups = len(want) // 8
        dev = torch.tensor(portions, dtype=torch.int32, device=DEV)
        got = ops.prefill_tiles_on_device(dev, rows_per_tile, groups + 2).cpu()
        assert got.shape == (4 * (groups + 2), 2)
        assert got[:4 * groups].flatten().tolist() == want
        assert got[4 * groups:, 1].tolist() == [0] * 8                       # groups of no rows
        assert int(got[:, 0].min()) >= 0 and int(got[:, 0].max()) < portions[-1][0] + max(portions[-1][1], 1)


@pytest.mark.parametrize("key_pos", [0, 15, 16, 200, 255, 256, 299])
def test_prefill_kernel_one_far_key_decides(ops, key_pos):
    """Rows 256..299 of a request; the row at position 299 (and every row at or after the key)
    returns the value of the one key that stands out."""
    bf = torch.bfloat16
    hq, hkv, d, L, page, first = 2, 1, 128, 300, 16, 256
    k = rand(L, hkv, d, seed=160, dtype=bf, scale=0.1)
    v = rand(L, hkv, d, seed=161, dtype=bf)
    direction = rand(d, seed=162)
    q = (direction[None, None, :] + 0.05 * rand(L - first, hq, d, seed=163)).to(bf)
    k[key_pos, 0] = (direction * 4).to(bf)
    cache, ids = paged_cache(k, v, page, 164, bf)
    n = L - first
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    from qwen_engine_amd.parts.attention import prefill_tiles
    tiles = torch.tensor(prefill_tiles([(0, n)], ops.prefill_tile_rows(hq, hkv)), dtype=torch.int32).view(-1, 2).tolist()
    want = P.attention(q.float(), k.float(), v.float(), 1 / math.sqrt(d))
    for groups in (1, 2):
        out = ops.attention(q.to(DEV), cache.to(DEV), i32(list(range(first, L))), i32([0] * n), ids[None].to(DEV),
                            1 / math.sqrt(d), dec_tokens=i32([]), other_tokens=i32(list(range(n))),
                            other_tiles=i32(tiles), prefill_groups=groups)
        close(out, want, bf)
    last_seen = max(key_pos, first) - first
    assert float((want[last_seen:, 0] - v[key_pos, 0].float()).abs().max()) < 0.05


@pytest.mark.parametrize("hq,hkv,d,page", [(16, 8, 128, 16), (4, 4, 64, 16), (8, 1, 128, 32), (6, 2, 64, 64)])
@pytest.mark.parametrize("window", [0, 200, 70])
def test_prefill_attention_over_key_segments(ops, hq, hkv, d, page, window):
    """The keys cut into segments of 64 to 512 (and as the kernel chooses): a portion of 300 rows after
    700 cached tokens, a whole prompt of 330 and two rows after 513, beside a decoded token.  Blocks
    whose keys lie in one segment write their rows themselves, the others leave partial results
    that the merge adds; the first key of the first request stands out for its first head, so every
    row of that head (that still sees it) gets its weight from the first segment."""
    bf = torch.bfloat16
    scale = 1 / math.sqrt(d)
    lens = [(700, 300), (0, 330), (513, 2), (90, 1)]
    qs, pos, seq, tables, caches, want, portions, dec, other = [], [], [], [], [], [], [], [], []
    base, row = 0, 0
    R = ops.prefill_tile_rows(hq, hkv)
    direction = rand(d, seed=119)
    for b, (before, n) in enumerate(lens):
        L = before + n
        k, v = rand(L, hkv, d, seed=120 + b, dtype=bf, scale=0.3), rand(L, hkv, d, seed=130 + b, dtype=bf)
        q = rand(n, hq, d, seed=140 + b, dtype=bf)
        if b == 0:
            q[:, 0] = (direction[None] + 0.05 * rand(n, d, seed=118)).to(bf)
            k[0, 0] = (direction * 4).to(bf)
        cache, ids = paged_cache(k, v, page, 150 + b, bf)
        tables.append(ids + base)
        base += cache.shape[0]
        caches.append(cache)
        qs.append(q)
        pos += list(range(before, L))
        seq += [b] * n
        want.append(P.attention(q.float(), k.float(), v.float(), scale, window=window or None))
        if b == 0 and not window:
            assert float((want[-1][:, 0] - v[0, 0].float()).abs().max()) < 0.05
        if n == 1:
            dec.append(row)
        else:
            other += list(range(row, row + n))
            portions.append((row, n))
        row += n
    from qwen_engine_amd.parts.attention import prefill_tiles
    tiles = torch.tensor(prefill_tiles(portions, R), dtype=torch.int32).view(-1, 2).tolist()
    width = max(len(t) for t in tables)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    for b, t in enumerate(tables):
        table[b, :len(t)] = t
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    args = (torch.cat(qs).to(DEV), torch.cat(caches).to(DEV), i32(pos), i32(seq), table.to(DEV), scale)
    whole = ops.attention(*args, window=window, dec_tokens=i32(dec), max_dec_position=90, other_tokens=i32(other),
                          other_tiles=i32(tiles), max_other_keys=1000, prefill_segment_keys=0)
    close(whole, torch.cat(want), bf)
    for seg, groups in ((64, 1), (64, 2), (128, 0), (256, 2), (512, 1), (512, 2), (960, 0), (-1, 0)):
        out = ops.attention(*args, window=window, dec_tokens=i32(dec), max_dec_position=90, other_tokens=i32(other),
                            other_tiles=i32(tiles), prefill_groups=groups, max_other_keys=1000 if seg != 960 else 1024,
                            prefill_segment_keys=seg)
        assert not torch.isnan(out.float()).any(), (seg, groups)
        close(out, torch.cat(want), bf)
        # rows whose keys lie in one segment come from the same sums as without segments
        if seg == 512 and groups == 2:
            assert torch.equal(out[300:630], whole[300:630])                 # the whole prompt of 330: keys 0 .. 329
    # a caller that does not know the positions names the row that sees the most keys (row 299, at
    # position 999): the kernels cut by its position, as the host would have
    by_row = ops.attention(*args, window=window, dec_tokens=i32(dec), max_dec_position=90, other_tokens=i32(other),
                           other_tiles=i32(tiles), other_keys_row=299)
    by_host = ops.attention(*args, window=window, dec_tokens=i32(dec), max_dec_position=90, other_tokens=i32(other),
                            other_tiles=i32(tiles), max_other_keys=1000)
    close(by_row, torch.cat(want), bf)
    assert torch.equal(by_row, by_host)
    with pytest.raises(ops.KernelError):
        ops.attention(*args, other_tokens=i32(other), dec_tokens=i32(dec), max_dec_position=90, other_tiles=i32(tiles),
                      max_other_keys=1000, prefill_segment_keys=100)
    with pytest.raises(ops.KernelError):
        ops.attention(*args, other_tokens=i32(other), dec_tokens=i32(dec), max_dec_position=90, other_tiles=i32(tiles),
                      other_keys_row=len(pos))


@pytest.mark.parametrize("M", [1, 8, 64, 65, 200, 1024])
@pytest.mark.parametrize("I,K", [(160, 96), (192, 64), (3072, 1024)])
def test_gemm_with_silu_mul_over_interleaved_rows(ops, M, I, K):
    """gate and up rows in alternating blocks of 32: the kernel for few rows and the tiled one both
    find the gate and the up of an output side by side; so does the separate silu.mul kernel."""
    bf = torch.bfloat16
    g, u = rand(I, K, seed=170, dtype=bf, scale=0.2), rand(I, K, seed=171, dtype=bf, scale=0.2)
    x = rand(M, K, seed=172, dtype=bf)
    w = ops.interleave_gate_up(g, u)
    assert torch.equal(w[:32], g[:32]) and torch.equal(w[32:64], u[:32]) and torch.equal(w[64:96], g[32:64])
    want = P.silu_mul(P.linear(x.double(), g.double()), P.linear(x.double(), u.double()))
    assert ops.gemm_silu_supported(x.to(DEV), w.to(DEV)) == (K % 32 == 0 or M > 64)
    if ops.gemm_silu_supported(x.to(DEV), w.to(DEV)):
        close(ops.gemm(x.to(DEV), w.to(DEV), epilogue=ops.EPI_SILU_MUL_IL), want, bf)
        if M > 64:
            for rows in (64, 65, 128, 256, 512):
                close(ops.gemm(x.to(DEV), w.to(DEV), epilogue=ops.EPI_SILU_MUL_IL, algo=ops.ALGO_TILE + rows), want, bf)
    gu = ops.gemm(x.to(DEV), w.to(DEV), algo=ops.ALGO_GENERIC)
    close(ops.silu_mul(gu, interleaved=True), want, bf)


@pytest.mark.parametrize("I,K,cuts_wanted", [(4096, 2048, 4), (2048, 4096, 8)])
@pytest.mark.parametrize("M", [17, 40, 64])
def test_gemm_of_few_rows_against_a_large_matrix(ops, M, I, K, cuts_wanted):
    """17 to 64 rows against 16 M weights and more go through the tiled kernel: gate|up with silu.mul in a
    tile shape of its own, the others as partial products in as many cuts of K as the kernel asks for.  With
    rows of 8192 bytes (K = 4096) every block starts its walk along K at another step."""
    bf = torch.bfloat16
    g, u = rand(I, K, seed=180, dtype=bf, scale=0.2), rand(I, K, seed=181, dtype=bf, scale=0.2)
    x = rand(M, K, seed=182, dtype=bf)
    w = ops.interleave_gate_up(g, u).to(DEV)
    want = P.silu_mul(P.linear(x.double(), g.double()), P.linear(x.double(), u.double()))
    close(ops.gemm(x.to(DEV), w, epilogue=ops.EPI_SILU_MUL_IL), want, bf)
    close(ops.gemm(x.to(DEV), w, epilogue=ops.EPI_SILU_MUL_IL, algo=ops.ALGO_TILE + 64), want, bf)
    wd = torch.cat([g, u]).to(DEV)                           # [8192, 2048]: 64 tile columns, so 4 cuts; [4096, 4096]: 32, so 8
    cuts = ops.gemm_branch_splits(x.to(DEV), wd)
    assert cuts == cuts_wanted
    parts = ops.gemm(x.to(DEV), wd, epilogue=ops.EPI_PARTIAL, splits=cuts)
    assert parts.shape == (cuts, M, 2 * I) and parts.dtype == torch.float32
    want = P.linear(x.double(), torch.cat([g, u]).double())
    close(parts.sum(0), want, torch.float32, scale=float(want.abs().max()))


@pytest.mark.parametrize("L", [4096, 4097, 8300])
def test_decode_kernel_with_more_than_32_splits(ops, L):
    """A token at position L - 1 over 32, 33 and 65 splits of 128 keys: the merge kernel sums eight of a
    wave's splits at a time and goes round again beyond 32 splits, and its first pass over the maxima
    goes round again beyond 64.  In each of four head groups one key carries the result: the first
    key, one in the middle, the last key of split 31, and the token's own."""
    bf = torch.bfloat16
    hq, hkv, d, page = 8, 4, 128, 16
    k = rand(L, hkv, d, seed=510, dtype=bf, scale=0.1)
    v = rand(L, hkv, d, seed=511, dtype=bf)
    q = rand(1, hq, d, seed=512, dtype=bf)
    far = [0, L // 2 + 5, 4095, L - 1]
    for kvh, key_pos in enumerate(far):
        k[key_pos, kvh] = (q[0, 2 * kvh].float() * 4).to(bf)
    cache, ids = paged_cache(k, v, page, 513, bf)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    out = ops.attention(q.to(DEV), cache.to(DEV), i32([L - 1]), i32([0]), ids[None].to(DEV), 1 / math.sqrt(d),
                        dec_tokens=i32([0]), max_dec_position=L - 1)
    want = P.attention(q.float(), k.float(), v.float(), 1 / math.sqrt(d))
    close(out, want, bf)
    for kvh, key_pos in enumerate(far):
        assert float((want[0, 2 * kvh] - v[key_pos, kvh].float()).abs().max()) < 0.05
    # several rows whose graphs share the largest position: a shorter one leaves its last splits empty
    positions = [L - 1, 130, 4000]
    qs = rand(3, hq, d, seed=514, dtype=bf)
    table = ids[None].repeat(3, 1)
    out = ops.attention(qs.to(DEV), cache.to(DEV), i32(positions), i32([0, 1, 2]), table.to(DEV), 1 / math.sqrt(d),
                        dec_tokens=i32([0, 1, 2]), max_dec_position=L - 1)
    want = torch.cat([P.attention(qs[i:i + 1].float(), k[:p + 1].float(), v[:p + 1].float(), 1 / math.sqrt(d))
                      for i, p in enumerate(positions)])
    close(out, want, bf)


@pytest.mark.parametrize("M", [1, 2, 5, 8, 16, 64])
@pytest.mark.parametrize("K", [1024, 1056])
def test_gemm_for_few_rows_against_the_whole_vocabulary(ops, M, K):
    """The head's product at the family's vocabulary: [M, K] against [151936, K], 32-bit logits,
    compared in 64-bit on the first and last columns and on 3000 drawn ones.  Up to 16 rows (one tile
    of rows; K = 1024: whole lines of 128 bytes a load, one tile of outputs a block; K = 1056, an odd
    number of chunks of 32: one tile a block up to 8 rows, four from 9 on) a row's logits are the same
    bits whatever else is in the batch."""
    bf = torch.bfloat16
    N = 151936
    x, w = rand(M, K, seed=520, dtype=bf), rand(N, K, seed=521, dtype=bf, scale=0.02)
    got = ops.gemm(x.to(DEV), w.to(DEV), out_dtype=torch.float32).cpu()
    assert got.shape == (M, N) and torch.isfinite(got).all()
    if M <= 16:
        alone = ops.gemm(x[M - 1:].to(DEV), w.to(DEV), out_dtype=torch.float32).cpu()
        assert torch.equal(alone[0], got[M - 1])
    cols = torch.cat([torch.arange(0, 80), torch.arange(N - 120, N),
                      torch.randint(0, N, (3000,), generator=torch.Generator().manual_seed(522))])
    want = x.double() @ w[cols].double().t()
    close(got[:, cols], want, torch.float32, scale=float(want.abs().max()))
    # the same through the generic 32-bit kernel, on 32-bit copies of the operands
    got32 = ops.gemm(x.float().to(DEV), w.float().to(DEV), out_dtype=torch.float32, algo=ops.ALGO_GENERIC).cpu()
    close(got32[:, cols], want, torch.float32, scale=float(want.abs().max()))


@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("N,K", [(4096, 1024), (512, 96), (336, 160), (2048, 4096), (64, 8192)])
def test_gemm_with_the_norm_as_its_prologue(ops, M, N, K):
    """The product of few rows that norms the 32-bit stream itself gives, to the bit, what the norm
    kernel followed by the product gives: the same arithmetic in the same order.  Also with a bias,
    with silu.mul over gate|up rows (both layouts), and against the plain norm and product."""
    bf = torch.bfloat16
    h = rand(M, K, seed=530, scale=3.0).to(DEV)
    nw = (1 + rand(K, seed=531, scale=0.2)).to(DEV)
    w = rand(N, K, seed=532, dtype=bf, scale=0.1).to(DEV)
    bias = rand(N, seed=533).to(DEV)
    eps = 1e-5
    # (the normed rows lie in shared memory as bfloat16, with 8 elements of padding a row: up to 136 KB)
    assert ops.gemm_norm_supported(M, w) == (M * (K + 8) * 2 <= 136 * 1024)
    if not ops.gemm_norm_supported(M, w):
        with pytest.raises(ops.KernelError):
            ops.gemm(h, w, norm_weight=nw, norm_eps=eps)
        return
    x = ops.rmsnorm(h, nw, eps, bf)
    for b in (None, bias):
        for dt_o in (bf, torch.float32):
            fused = ops.gemm(h, w, b, out_dtype=dt_o, norm_weight=nw, norm_eps=eps)
            assert fused.dtype == dt_o and torch.equal(fused, ops.gemm(x, w, b, out_dtype=dt_o))
    close(x, P.rms_norm(h.cpu().double(), nw.cpu().double(), eps), bf)            # the norm kernel itself
    want = P.linear(x.cpu().double(), w.cpu().double())
    close(ops.gemm(h, w, out_dtype=torch.float32, norm_weight=nw, norm_eps=eps), want, torch.float32,
          scale=float(want.abs().max()))
    # with the residual sum inside as well: the partial products of the branch before are added to the
    # stream in order, normed and multiplied, and the sums are written to a second buffer
    for S in (1, 4):
        parts = rand(S, M, K, seed=534, scale=1.5).to(DEV)
        h2 = h.clone()
        x2 = ops.rmsnorm(h2, nw, eps, bf, delta=parts)                 # (adds the parts into h2)
        summed = torch.full_like(h, float("nan"))
        fused = ops.gemm(h, w, bias, norm_weight=nw, norm_eps=eps, delta=parts, stream_out=summed)
        assert torch.equal(summed, h2) and torch.equal(fused, ops.gemm(x2, w, bias))
    with pytest.raises(ops.KernelError):
        ops.gemm(h, w, norm_weight=nw, norm_eps=eps, delta=parts, stream_out=h)     # over the stream that is read
    if N % 64 == 0:
        fused = ops.gemm(h, w, epilogue=ops.EPI_SILU_MUL_IL, norm_weight=nw, norm_eps=eps)
        assert fused.shape == (M, N // 2) and torch.equal(fused, ops.gemm(x, w, epilogue=ops.EPI_SILU_MUL_IL))
    fused = ops.gemm(h, w, epilogue=ops.EPI_SILU_MUL, norm_weight=nw, norm_eps=eps)
    assert torch.equal(fused, ops.gemm(x, w, epilogue=ops.EPI_SILU_MUL))
    g, u = want[:, :N // 2], want[:, N // 2:]
    close(fused, P.silu_mul(g, u), bf)


def test_gemm_norm_prologue_refuses_what_it_does_not_take(ops):
    bf = torch.bfloat16
    w = rand(64, 64, seed=540, dtype=bf).to(DEV)
    nw = torch.ones(64, device=DEV)
    assert not ops.gemm_norm_supported(17, w)                            # more than 16 rows
    assert not ops.gemm_norm_supported(4, w.float())                     # 32-bit weights
    assert not ops.gemm_norm_supported(16, torch.zeros(32, 8192, dtype=bf, device=DEV))     # rows too long for shared memory
    assert not ops.gemm_norm_supported(2, torch.zeros(32, 16384, dtype=bf, device=DEV))     # beyond the norm kernel's own layout
    with pytest.raises(ops.KernelError):
        ops.gemm(torch.zeros(17, 64, device=DEV), w, norm_weight=nw, norm_eps=1e-6)
    with pytest.raises(ops.KernelError):                                 # the stream is 32-bit
        ops.gemm(torch.zeros(4, 64, device=DEV, dtype=bf), w, norm_weight=nw, norm_eps=1e-6)
    with pytest.raises(ops.KernelError):                                 # partial products do not go with it
        ops.gemm(torch.zeros(4, 64, device=DEV), w, epilogue=ops.EPI_PARTIAL, norm_weight=nw, norm_eps=1e-6)


@pytest.mark.parametrize("hq,hkv,d,page", [(4, 2, 16, 4), (6, 1, 32, 3), (6, 2, 48, 16), (40, 2, 64, 5), (3, 3, 80, 1),
                                           (16, 8, 128, 16), (2, 1, 256, 64), (34, 1, 16, 8)])
@pytest.mark.parametrize("window", [0, 37])
def test_float32_attention_on_the_matrix_units(ops, hq, hkv, d, page, window):
    """The float32 kernel on the matrix units (heads as columns, 16 keys a tile, any page size, more
    than 16 heads a group in several waves) against the plain attention and against the
    one-wave-a-head kernel, which sums in another order: portions and single tokens of three
    requests, one of them starting at position 0; unused pages and the ends of pages hold NaN."""
    scale = 0.7 / math.sqrt(d)
    lens = [(140, 9), (70, 1), (0, 21)]
    qs, pos, seq, tables, caches, want = [], [], [], [], [], []
    base_page = 0
    for b, (before, n) in enumerate(lens):
        L = before + n
        k, v = rand(L, hkv, d, seed=610 + b), rand(L, hkv, d, seed=620 + b)
        q = rand(n, hq, d, seed=630 + b)
        cache, ids = paged_cache(k, v, page, 640 + b, torch.float32)
        tables.append(ids + base_page)
        base_page += cache.shape[0]
        caches.append(cache)
        qs.append(q)
        pos += list(range(before, L))
        seq += [b] * n
        want.append(P.attention(q, k, v, scale, window=window or None))
    width = max(len(t) for t in tables)
    table = torch.full((len(lens), width), -1, dtype=torch.int32)
    for b, t in enumerate(tables):
        table[b, :len(t)] = t
    args = (torch.cat(qs).to(DEV), torch.cat(caches).to(DEV), torch.tensor(pos, dtype=torch.int32, device=DEV),
            torch.tensor(seq, dtype=torch.int32, device=DEV), table.to(DEV), scale)
    out = ops.attention(*args, window=window)
    assert not torch.isnan(out).any()
    close(out, torch.cat(want), torch.float32)
    try:
        ops.use_matrix_f32(False)
        other = ops.attention(*args, window=window)
    finally:
        ops.use_matrix_f32(True)
    close(other, torch.cat(want), torch.float32)
    assert not torch.equal(other, out) or d == 16          # (two kernels, two orders of the sums)
    # a subset of the rows, as the engine asks for when the others go to another kernel
    rows = torch.tensor([0, 9, 10, 30], dtype=torch.int32, device=DEV)
    part = torch.full_like(out, float("nan"))
    q_all = args[0]
    from qwen_engine_amd.kernels.ops import load_library, _DT
    lib = load_library()
    rc = lib.qe_attention(q_all.data_ptr(), part.data_ptr(), args[1].data_ptr(), args[2].data_ptr(), args[3].data_ptr(),
                          args[4].data_ptr(), args[4].shape[1], rows.data_ptr(), 4, hq, hkv, d, page, scale, window, 0,
                          torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(part[rows.long()], out[rows.long()]) and torch.isnan(part[1]).all()


@pytest.mark.parametrize("M,N,K", [(1, 500, 96), (5, 331, 80), (64, 64, 64), (130, 77, 200), (3, 2048, 1024), (257, 130, 30),
                                   (70, 65, 17), (2048, 192, 1024)])
def test_float32_gemm_on_the_matrix_units(ops, M, N, K):
    """The float32 product on the matrix units against the 64-bit product, tighter than the vector
    units' kernel needs, and against that kernel; rows give the same bits whatever else is in the batch."""
    x, w = rand(M, K, seed=650), rand(N, K, seed=651, scale=0.1)
    bias = rand(N, seed=652)
    want = P.linear(x.double(), w.double())
    got = ops.gemm(x.to(DEV), w.to(DEV))
    close(got, want, torch.float32)
    close(ops.gemm(x.to(DEV), w.to(DEV), bias.to(DEV)), want + bias.double(), torch.float32)
    try:
        ops.use_matrix_f32(False)
        other = ops.gemm(x.to(DEV), w.to(DEV))
    finally:
        ops.use_matrix_f32(True)
    close(other, want, torch.float32)
    # a row alone and the same row among the others: the same bits
    alone = ops.gemm(x[M // 2:M // 2 + 1].to(DEV), w.to(DEV))
    assert torch.equal(alone[0], got[M // 2])
