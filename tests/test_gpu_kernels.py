"""Each kernel alone against its plain torch version (tests/reference_ops.py), at sizes other
than the tiny models': widths and vocabularies that are no power of two, head sizes in steps
of 16, odd head counts and groups, several page sizes, in float32 and bfloat16."""
import random

import numpy as np
import pytest
import torch

import reference_ops as ref
from lucciola_amd.kernels import ops
from lucciola_amd.kernels.ops import AttentionBatch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-6) if dtype == torch.float32 else dict(rtol=1.6e-2, atol=1e-3)


def close(got, want, dtype, scale=1.0, atol=None):
    t = tol(dtype)
    torch.testing.assert_close(got.double().cpu(), want.double().cpu(), rtol=t["rtol"],
                               atol=t["atol"] * scale if atol is None else atol)


def attention_atol(dtype, v_cache):
    """The matrix-core kernels round the softmax weights to bfloat16 before the P.V product:
    each weight is off by at most 2^-9 of itself, so an output (a convex combination of value
    rows) is off by at most 2^-9 max|v|, beside its own rounding."""
    return None if dtype == torch.float32 else float(v_cache.abs().max()) * 2.0 ** -9


def rnd(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H,V", [(1, 16, 7), (5, 200, 331), (130, 1000, 50)])
def test_embedding(dtype, T, H, V):
    table = rnd(V, H, dtype=dtype, seed=1)
    ids = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(2)).int().to(DEV)
    got = ops.embedding(ids, table)
    assert got.dtype == torch.float32
    assert torch.equal(got, ref.embedding(ids, table))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,n", [(1, 16), (7, 200), (33, 1000), (3, 4100)])
def test_rmsnorm_with_residual(dtype, T, n):
    h = rnd(T, n, seed=3, scale=2.0)
    delta = rnd(T, n, dtype=dtype, seed=4)
    w = 1 + rnd(n, seed=5, scale=0.1)
    h_ref = h.clone()
    want = ref.rmsnorm(h_ref, delta, w, 1e-5, dtype)
    got = ops.rmsnorm(h, delta, w, 1e-5, dtype)
    torch.testing.assert_close(h, h_ref, rtol=1e-6, atol=1e-6)     # the stream took the sum
    close(got, want, dtype)
    # without a pending branch, and at chosen rows only (the stream must stay untouched)
    h2 = rnd(T, n, seed=6)
    keep = h2.clone()
    rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
    got = ops.rmsnorm(h2, delta, w, 1e-6, dtype, rows=rows)
    want = ref.rmsnorm(keep.clone(), delta, w, 1e-6, dtype, rows=rows)
    assert torch.equal(h2, keep)
    close(got, want, dtype)
    close(ops.rmsnorm(h2, None, w, 1e-6, dtype), ref.rmsnorm(keep.clone(), None, w, 1e-6, dtype), dtype)


def test_rmsnorm_eps_matters():
    x = torch.full((1, 64), 1e-3, device=DEV)
    w = torch.ones(64, device=DEV)
    a = ops.rmsnorm(x.clone(), None, w, 1e-6, torch.float32)
    b = ops.rmsnorm(x.clone(), None, w, 1e-5, torch.float32)
    assert abs(float(a[0, 0]) - 1e-3 / (2e-6) ** 0.5) < 1e-3
    assert abs(float(b[0, 0]) - 1e-3 / (1.1e-5) ** 0.5) < 1e-3


@pytest.mark.parametrize("dt_x,dt_w,dt_o", [
    (torch.float32, torch.float32, torch.float32), (torch.float32, torch.bfloat16, torch.float32),
    (torch.bfloat16, torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.bfloat16, torch.float32),
    (torch.bfloat16, torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 331, 72), (65, 130, 200), (64, 64, 16), (17, 1000, 257),
                                   (16, 200, 1030), (9, 70, 515)])
def test_gemm_generic(dt_x, dt_w, dt_o, M, N, K):
    x = rnd(M, K, dtype=dt_x, seed=7)
    w = rnd(N, K, dtype=dt_w, seed=8)
    got = ops.gemm(x, w, dt_o)
    want = ref.gemm(x, w, dt_o)
    close(got, want, dt_o, scale=K ** 0.5)


@pytest.mark.parametrize("K", [600, 601, 256, 77])
def test_gemm_generic_same_bits_for_any_number_of_rows(K):
    """A row's float32 product has the same bits alone (tiles of 16 rows, K shared out over
    workgroups), among a few dozen rows and among a thousand (tiles of 64 rows, K not shared)."""
    x = rnd(1100, K, seed=11)
    w = rnd(3700, K, seed=12)
    whole = ops.gemm(x, w, torch.float32)
    close(whole, ref.gemm(x, w, torch.float32), torch.float32, scale=K ** 0.5)
    for first, count in ((0, 7), (500, 1), (1084, 16), (30, 40)):
        rows = ops.gemm(x[first:first + count].contiguous(), w, torch.float32)
        assert torch.equal(rows, whole[first:first + count]), (first, count)


def make_rope_table(positions, rot, theta):
    i = torch.arange(rot // 2, dtype=torch.float64)
    inv = 1.0 / theta ** (2 * i / rot)
    ang = torch.arange(positions, dtype=torch.float64)[:, None] * inv[None]
    return torch.cat([ang.cos(), ang.sin()], 1).float().to(DEV)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page", [(4, 2, 16, 4), (6, 2, 48, 16), (5, 5, 32, 8), (8, 1, 128, 16),
                                           (3, 1, 80, 2), (2, 2, 256, 32), (32, 8, 128, 16), (3, 3, 128, 4)])
def test_qk_norm_rope_write(dtype, nh, nkv, d, page):
    T, pages = 37, 40
    qkv = rnd(T, (nh + 2 * nkv) * d, dtype=dtype, seed=9)
    qw, kw = 1 + rnd(d, seed=10, scale=0.2), 1 + rnd(d, seed=11, scale=0.2)
    positions = torch.randint(0, 500, (T,), generator=torch.Generator().manual_seed(12)).int().to(DEV)
    table = make_rope_table(512, d, 10000.0)
    slots = torch.randperm(pages * page, generator=torch.Generator().manual_seed(13))[:T].int()
    slots[5] = -1
    slots = slots.to(DEV)
    kc = torch.zeros(pages, nkv, page, d, dtype=dtype, device=DEV)
    vc = torch.zeros(pages, nkv, d, page, dtype=dtype, device=DEV)
    qkv_ref, kc_ref, vc_ref = qkv.clone(), kc.clone(), vc.clone()
    ref.qk_norm_rope_write(qkv_ref, nh, nkv, d, qw, kw, 1e-6, positions, table, kc_ref, vc_ref, slots, page)
    ops.qk_norm_rope_write(qkv, nh, nkv, d, qw, kw, 1e-6, positions, table, kc, vc, slots, page)
    close(qkv, qkv_ref, dtype)
    close(kc, kc_ref, dtype)
    assert torch.equal(vc, vc_ref)
    # no norm, no rotation, no cache: nothing changes
    again = qkv.clone()
    ops.qk_norm_rope_write(again, nh, nkv, d, None, None, 0.0, None, None, None, None, None, page)
    assert torch.equal(again, qkv)


def paged_case(lengths, new, nh, nkv, d, page, dtype, seed, spare=3):
    """Requests with ``lengths[r]`` cached tokens of which the last ``new[r]`` are this step's."""
    rng = random.Random(seed)
    R = len(lengths)
    need = sum(-(-n // page) for n in lengths)
    ids = list(range(need + spare))
    rng.shuffle(ids)
    kc = rnd(need + spare, nkv, page, d, dtype=dtype, seed=seed + 1)
    vc = rnd(need + spare, nkv, d, page, dtype=dtype, seed=seed + 2)
    mb = max(-(-n // page) for n in lengths)
    table = torch.full((R, mb), -1, dtype=torch.int32)
    for r, n in enumerate(lengths):
        for j in range(-(-n // page)):
            table[r, j] = ids.pop()
    tok_req, positions, q_start = [], [], [0]
    for r, (n, k) in enumerate(zip(lengths, new)):
        tok_req += [r] * k
        positions += list(range(n - k, n))
        q_start.append(q_start[-1] + k)
    T = len(tok_req)
    qkv = rnd(T, (nh + 2 * nkv) * d, dtype=dtype, seed=seed + 3)
    dec = np.asarray([[q_start[r], r, lengths[r] - 1, 0] for r in range(R) if new[r] == 1], dtype=np.int32).reshape(-1, 4)
    dec_lengths = np.asarray([lengths[r] for r in range(R) if new[r] == 1], dtype=np.int64)
    items = ops._decode_items(dec, dec_lengths)       # the planner's list of work items, taken where a test asks
    tiles = []
    for r in range(R):
        if new[r] > 1:
            for t0 in range(0, new[r], 64):
                tiles += [r, q_start[r] + t0, min(64, new[r] - t0), lengths[r] - new[r] + t0]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    batch = AttentionBatch(tok_req=i32(tok_req), positions=i32(positions), block_table=table.to(DEV),
                           q_start=i32(q_start), ctx_len=i32(lengths), num_decode=len(dec),
                           decode_rows=torch.from_numpy(dec).to(DEV), prefill_tiles=i32(tiles).view(-1, 4),
                           decode_items=torch.from_numpy(items).to(DEV),
                           decode_longest=int(dec_lengths.max()) if len(dec) else 0,
                           decode_total=int(dec_lengths.sum()), max_ctx=max(lengths), all_decode=len(dec) == R)
    return qkv, batch, kc, vc


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page,window", [
    (4, 2, 16, 4, 0), (6, 2, 48, 16, 0), (8, 1, 32, 8, 0), (5, 5, 80, 16, 0), (32, 8, 128, 16, 0),
    (6, 2, 48, 16, 24), (4, 4, 64, 8, 5), (2, 1, 256, 16, 0), (4, 2, 64, 16, 0), (6, 2, 96, 16, 24),
    (16, 1, 32, 16, 0), (32, 8, 128, 16, 40), (12, 4, 128, 16, 7), (10, 2, 128, 16, 0), (5, 1, 128, 16, 33)])
def test_attention_mixed_batch(dtype, nh, nkv, d, page, window):
    lengths = [1, 300, 17, 64, 130]
    new = [1, 1, 17, 2, 70]
    qkv, batch, kc, vc = paged_case(lengths, new, nh, nkv, d, page, dtype, seed=20)
    got = ops.attention(qkv, batch, kc, vc, nh, nkv, d, page, d ** -0.5, window)
    want = ref.attention(qkv.cpu(), AttentionBatch(batch.tok_req.cpu(), batch.positions.cpu(),
                                                   batch.block_table.cpu()),
                         kc.cpu(), vc.cpu(), nh, nkv, d, page, d ** -0.5, window)
    close(got, want, dtype, atol=attention_atol(dtype, vc))
    # the general kernel with several rows to a workgroup: rows of one request together, the others
    # (a workgroup's rows straddle two requests) one after the other; every row the same bits
    lib = ops.library()
    lib.lc_attention_generic_rows(4)
    try:
        assert torch.equal(ops.attention(qkv, batch, kc, vc, nh, nkv, d, page, d ** -0.5, window), got)
    finally:
        lib.lc_attention_generic_rows(0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d,page,window", [(6, 2, 48, 16, 0), (6, 2, 48, 16, 700), (10, 2, 20, 8, 0),
                                                   (4, 4, 128, 16, 1100)])
def test_attention_general_kernel_same_bits_alone_and_in_a_prompt(dtype, nh, nkv, d, page, window):
    """The last tokens of a long prompt, once as rows of the whole prompt (one workgroup works
    through all their keys) and once alone (the keys are shared out over workgroups and joined
    by a second kernel): the same bits, and both near the plain result."""
    if dtype == torch.bfloat16 and ops.library().lc_attn_bf16_supported(nh, nkv, d, page):
        pytest.skip("these sizes have a matrix-core kernel in bfloat16")
    length, whole, alone = 1500, 700, 5
    qkv, batch, kc, vc = paged_case([length], [whole], nh, nkv, d, page, dtype, seed=26)
    got = ops.attention(qkv, batch, kc, vc, nh, nkv, d, page, d ** -0.5, window)
    want = ref.attention(qkv.cpu(), AttentionBatch(batch.tok_req.cpu(), batch.positions.cpu(),
                                                   batch.block_table.cpu()),
                         kc.cpu(), vc.cpu(), nh, nkv, d, page, d ** -0.5, window)
    close(got, want, dtype, atol=attention_atol(dtype, vc))
    _, few, kc2, vc2 = paged_case([length], [alone], nh, nkv, d, page, dtype, seed=26)
    assert torch.equal(kc2, kc) and torch.equal(few.block_table, batch.block_table)
    tail = ops.attention(qkv[-alone:].contiguous(), few, kc, vc, nh, nkv, d, page, d ** -0.5, window)
    assert torch.equal(tail, got[-alone:])
    # several rows of the prompt to a workgroup, which share every key and value they load (what a
    # large prompt gets by itself); once with an odd number of rows, whose last workgroup has one
    lib = ops.library()
    lib.lc_attention_generic_rows(4)
    try:
        shared = ops.attention(qkv, batch, kc, vc, nh, nkv, d, page, d ** -0.5, window)
        odd = ops.attention(qkv[1:].contiguous(), AttentionBatch(batch.tok_req[1:].contiguous(),
                                                                 batch.positions[1:].contiguous(),
                                                                 batch.block_table),
                            kc, vc, nh, nkv, d, page, d ** -0.5, window)
    finally:
        lib.lc_attention_generic_rows(0)
    assert torch.equal(shared, got)
    assert torch.equal(odd, got[1:])


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_far_key_stands_out(dtype):
    """One key among many hundreds gets a large score: the output must be its value row, so a
    kernel that drops or misplaces far keys fails."""
    nh, nkv, d, page = 4, 2, 32, 16
    for far in (0, 15, 16, 511, 777):
        qkv, batch, kc, vc = paged_case([900], [1], nh, nkv, d, page, dtype, seed=30)
        table = batch.block_table[0].tolist()
        q = torch.zeros(1, nh + 2 * nkv, d, dtype=dtype, device=DEV)
        q[0, :nh, 3] = 40.0
        kc[table[far // page], :, far % page, :] = 0
        kc[table[far // page], :, far % page, 3] = 40.0
        got = ops.attention(q.view(1, -1), batch, kc, vc, nh, nkv, d, page, d ** -0.5, 0).view(nh, d)
        for h in range(nh):
            close(got[h], vc[table[far // page], h // 2, :, far % page], dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(1, 8), (5, 200), (70, 1001)])
def test_swiglu(dtype, T, I):
    gu = rnd(T, 2 * I, dtype=dtype, seed=40, scale=3.0)
    close(ops.swiglu(gu), ref.swiglu(gu), dtype)
    z = torch.zeros(1, 2 * I, dtype=dtype, device=DEV)
    assert float(ops.swiglu(z).abs().max()) == 0.0


@pytest.mark.parametrize("V", [7, 331, 151936])
def test_sampling(V):
    logits = rnd(6, V, seed=50, scale=2.0)
    logits[1, V // 2] = logits[1, 0] = 50.0            # a tie: the lowest index wins
    got = ops.sample(logits)
    assert got.tolist() == logits.argmax(dim=1).tolist()
    assert int(got[1]) == 0
    temps = torch.tensor([0.7, 0.0, 1.3, 0.7, 2.0, 0.05], device=DEV)
    us = torch.tensor([0.0, 0.3, 0.999999, 0.5, 0.25, 0.9], device=DEV)
    got = ops.sample(logits, temps, us).tolist()
    want = ref.sample(logits.cpu(), temps.cpu(), us.cpu()).tolist()
    p = torch.softmax(logits.double().cpu() / temps.double().cpu().clamp(min=1e-9)[:, None], 1)
    cdf = p.cumsum(1)
    for r in range(6):
        if got[r] != want[r]:   # only a float32-rounding neighbour of the boundary may differ
            lo = cdf[r, min(got[r], want[r])]
            assert abs(float(lo) - float(us[r])) < 1e-4, (r, got[r], want[r])
    assert got[1] == 0


def test_sampling_follows_the_distribution():
    logits = torch.tensor([[0.0, 1.0, 2.0, -1.0, 0.5]], device=DEV).repeat(4000, 1).contiguous()
    temps = torch.full((4000,), 0.7, device=DEV)
    us = torch.rand(4000, generator=torch.Generator().manual_seed(1)).to(DEV)
    got = ops.sample(logits, temps, us)
    freq = torch.bincount(got.cpu().long(), minlength=5).double() / 4000
    p = torch.softmax(logits[0].double().cpu() / 0.7, 0)
    assert float((freq - p).abs().max()) < 0.03


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M,N,K", [(1, 16, 128), (8, 100, 256), (17, 4096, 1024), (64, 331, 384),
                                   (65, 128, 128), (128, 257, 512), (300, 1000, 640), (2048, 512, 1024),
                                   (3, 151936 // 8, 256), (33, 4096, 4096), (64, 6144, 1024), (48, 100, 128),
                                   (20, 24576, 256), (600, 3000, 256), (2, 331, 512), (13, 16400, 256),
                                   (16, 24576, 128), (12, 16384, 2048), (40, 24576, 1024), (64, 20000, 1152),
                                   (33, 30000, 1024), (64, 38000, 1024), (50, 51200, 1024)])
def test_gemm_bf16_matrix_cores(out_dtype, M, N, K):
    x = rnd(M, K, dtype=torch.bfloat16, seed=60)
    w = rnd(N, K, dtype=torch.bfloat16, seed=61)
    assert ops._fast_gemm_ok(M, N, K)
    got = ops.gemm(x, w, out_dtype)
    want = ref.gemm(x, w, out_dtype)
    close(got, want, out_dtype, scale=K ** 0.5)


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12])
@pytest.mark.parametrize("M,N,K", [(1, 16, 128), (70, 130, 128), (257, 300, 256), (300, 1000, 640),
                                   (513, 257, 384), (64, 128, 1024), (1000, 520, 2048), (100, 400, 128)])
def test_gemm_bf16_every_tile_shape(tile, M, N, K):
    """Each tile shape of the tiled kernel at sizes that leave ragged edges in both directions,
    from two k-blocks (fewer than the ring of stages holds) to many; with and without the SwiGLU
    epilogue, bfloat16 and float32 output."""
    x = rnd(M, K, dtype=torch.bfloat16, seed=63)
    w = rnd(N, K, dtype=torch.bfloat16, seed=64)
    assert ops._fast_gemm_ok(M, N, K)
    ops.force_gemm_tile(tile)
    try:
        got16 = ops.gemm(x, w, torch.bfloat16)
        got32 = ops.gemm(x, w, torch.float32)
        fused = ops.gemm_swiglu(x, w[:N // 16 * 16]) if N >= 16 else None
    finally:
        ops.force_gemm_tile(-1)
    close(got16, ref.gemm(x, w, torch.bfloat16), torch.bfloat16, scale=K ** 0.5)
    close(got32, ref.gemm(x, w, torch.float32), torch.float32, scale=K ** 0.5)
    if fused is not None:
        full = x.double() @ w[:N // 16 * 16].double().T
        blocks = full.view(M, -1, 2, 8)
        g, u = blocks[:, :, 0, :].reshape(M, -1), blocks[:, :, 1, :].reshape(M, -1)
        close(fused, (g / (1 + torch.exp(-g)) * u).to(torch.bfloat16), torch.bfloat16, scale=K ** 0.5)


@pytest.mark.parametrize("tile,M,N,K", [(4, 2000, 10200, 1024), (2, 2048, 10240, 1024), (3, 1990, 6520, 2048),
                                        (-1, 2048, 10240, 5120), (6, 570, 24500, 1024), (5, 760, 12000, 1024)])
def test_gemm_bf16_last_round_cut_along_k(tile, M, N, K):
    """Sizes whose tiles fill the CUs once or twice and leave a small rest: the rest's tiles
    are cut along K and summed by a second kernel.  Plain and with the SwiGLU epilogue,
    bfloat16 and float32 output, ragged edges."""
    x = rnd(M, K, dtype=torch.bfloat16, seed=65, scale=0.5)
    w = rnd(N, K, dtype=torch.bfloat16, seed=66, scale=0.5)
    ops.force_gemm_tile(tile)
    try:
        assert ops.library().lc_gemm_bf16_workspace(M, N, K) > 0      # the cut is really taken
        got16 = ops.gemm(x, w, torch.bfloat16)
        got32 = ops.gemm(x, w, torch.float32)
        fused = ops.gemm_swiglu(x, w[:N // 16 * 16])
    finally:
        ops.force_gemm_tile(-1)
    want = x.float() @ w.float().T
    close(got32, want, torch.float32, scale=K ** 0.5)
    close(got16, want.to(torch.bfloat16), torch.bfloat16, scale=K ** 0.5)
    blocks = want[:, :N // 16 * 16].double().view(M, -1, 2, 8)
    g, u = blocks[:, :, 0, :].reshape(M, -1), blocks[:, :, 1, :].reshape(M, -1)
    close(fused, (g / (1 + torch.exp(-g)) * u).to(torch.bfloat16), torch.bfloat16, scale=K ** 0.5)


@pytest.mark.parametrize("M,H,K,N2", [(1, 5120, 128, 6160), (8, 5120, 256, 10250), (16, 6272, 384, 5130),
                                      (1, 128, 128, 48), (2, 384, 256, 1000), (5, 256, 640, 272), (8, 4096, 512, 2064),
                                      (11, 640, 128, 16), (12, 16384, 6272, 16416), (12, 8192, 128, 48), (16, 1152, 384, 130),
                                      (8, 4096, 12288, 6144), (3, 1024, 1536, 2064), (16, 4096, 4096, 4112), (2, 512, 9216, 528)])
@pytest.mark.parametrize("runs", [2, 0])
def test_norm_folded_into_the_products_around_it(M, H, K, N2, runs):
    """Up to 16 rows: the product before a norm adds its result to the stream and leaves
    bf16(h * weight) and the pieces of the rows' sums of squares; the product after it applies
    the rows' factors to its sums.  Each piece is checked against the plain formulas, and the
    chain against norm-then-product; the first norm of a model has no product before it."""
    if not runs and K % 512 and H % 512:
        pytest.skip("neither product would read w in runs")
    ops.gemm_runs(runs)
    try:
        norm_folded_case(M, H, K, N2)
    finally:
        ops.gemm_runs(True)


def norm_folded_case(M, H, K, N2):
    eps = 3e-6
    h = rnd(M, H, seed=70, scale=2.0)
    x = rnd(M, K, dtype=torch.bfloat16, seed=71)
    w = rnd(H, K, dtype=torch.bfloat16, seed=72, scale=K ** -0.5)
    g = 1 + rnd(H, seed=73, scale=0.2)
    w2 = rnd(N2, H, dtype=torch.bfloat16, seed=74, scale=H ** -0.5)
    pending = ops.gemm(x, w, torch.bfloat16, defer=True)
    assert isinstance(pending, ops.PendingProduct)
    h_want = h.double() + x.double() @ w.double().T
    h_got = h.clone()
    rows = ops.rmsnorm(h_got, pending, g, eps, torch.bfloat16, scaled=True)
    assert isinstance(rows, ops.ScaledRows) and rows.count == rows.pieces.shape[0]
    torch.testing.assert_close(h_got.double(), h_want, rtol=1e-5, atol=1e-5)
    close(rows.x, (h_got.double() * g.double()).to(torch.bfloat16), torch.bfloat16)
    torch.testing.assert_close(rows.pieces[:, :M].double().sum(0), (h_got.double() ** 2).sum(1), rtol=1e-5, atol=0)
    normed = h_got.double() * torch.rsqrt((h_got.double() ** 2).mean(1, keepdim=True) + eps) * g.double()
    close(ops.value(rows), normed.to(torch.bfloat16), torch.bfloat16)
    # the product takes the rounded rows h * g and applies the factors to its float32 sums
    factors = torch.rsqrt((h_got.double() ** 2).mean(1, keepdim=True) + eps)
    full = (rows.x.double() @ w2.double().T) * factors
    got = ops.gemm(rows, w2, torch.bfloat16)
    close(got, full.to(torch.bfloat16), torch.bfloat16, scale=2.0)
    w2e = w2[:N2 // 16 * 16]
    blocks = full[:, :N2 // 16 * 16].view(M, -1, 2, 8)
    gate, up = blocks[:, :, 0, :].reshape(M, -1), blocks[:, :, 1, :].reshape(M, -1)
    close(ops.gemm_swiglu(rows, w2e), (gate / (1 + torch.exp(-gate)) * up).to(torch.bfloat16), torch.bfloat16, scale=2.0)
    # and the chain is the product of the normed rows, up to the rounding of those rows to bfloat16
    exact = normed @ w2.double().T
    assert float((got.double() - exact).norm() / exact.norm()) < 6e-3
    # the same rows from the norm kernel alone (no product before it), with and without a branch to add
    for delta in (None, rnd(M, H, dtype=torch.bfloat16, seed=75)):
        h2 = h.clone()
        alone = ops.rmsnorm(h2, delta, g, eps, torch.bfloat16, scaled=True)
        assert isinstance(alone, ops.ScaledRows) and alone.count == 1
        h2_want = h.double() + (0 if delta is None else delta.double())
        torch.testing.assert_close(h2.double(), h2_want, rtol=1e-6, atol=1e-6)
        normed2 = h2.double() * torch.rsqrt((h2.double() ** 2).mean(1, keepdim=True) + eps) * g.double()
        exact2 = normed2 @ w2.double().T
        assert float((ops.gemm(alone, w2, torch.bfloat16).double() - exact2).norm() / exact2.norm()) < 6e-3
    # whoever does not ask for scaled rows gets tensors, and the pending product is added all the same
    h3 = h.clone()
    plain_rows = ops.rmsnorm(h3, ops.gemm(x, w, torch.bfloat16, defer=True), g, eps, torch.bfloat16)
    assert isinstance(plain_rows, torch.Tensor)
    torch.testing.assert_close(h3.double(), h_want, rtol=2e-2, atol=2e-2)   # the branch was rounded to bfloat16 first
    # more than 16 rows (unless the product is cut along K anyway), float32, or a width the
    # matrix-core kernels do not take: nothing is deferred
    more = ops.gemm(rnd(17, K, dtype=torch.bfloat16), w, torch.bfloat16, defer=True)
    assert isinstance(more, ops.PendingProduct) == (ops.library().lc_gemm_bf16_shares(17, H, K) > 1)
    assert isinstance(ops.gemm(x.float(), w.float(), torch.float32, defer=True), torch.Tensor)
    assert isinstance(ops.rmsnorm(rnd(M, 72), None, 1 + rnd(72), eps, torch.bfloat16, scaled=True), torch.Tensor)


def test_gemm_bf16_one_hot_rows_and_columns():
    """x picks single columns of w: the product must return exactly those entries, so a wrong
    operand layout (rows, k order) shows as a wrong element, not as a small error."""
    M, N, K = 40, 48, 256
    w = rnd(N, K, dtype=torch.bfloat16, seed=62)
    x = torch.zeros(M, K, dtype=torch.bfloat16, device=DEV)
    cols = [(7 * m + 3) % K for m in range(M)]
    for m, c in enumerate(cols):
        x[m, c] = 1.0
    got = ops.gemm(x, w, torch.float32)
    want = w.float()[:, cols].T.contiguous()
    assert torch.equal(got, want)
    xb = torch.zeros(200, K, dtype=torch.bfloat16, device=DEV)
    cols = [(11 * m + 5) % K for m in range(200)]
    for m, c in enumerate(cols):
        xb[m, c] = 1.0
    assert torch.equal(ops.gemm(xb, w, torch.float32), w.float()[:, cols].T.contiguous())


@pytest.mark.parametrize("nh,nkv,d,window", [(32, 8, 128, 0), (8, 2, 64, 0), (4, 4, 96, 1000), (16, 1, 32, 0)])
def test_attention_bf16_long_contexts(nh, nkv, d, window):
    """Decode over thousands of keys (the pages are shared out over several workgroups and
    joined) beside a long prompt portion with history."""
    lengths = [5000, 1, 17, 2049, 700]
    new = [1, 1, 1, 1, 300]
    qkv, batch, kc, vc = paged_case(lengths, new, nh, nkv, d, 16, torch.bfloat16, seed=70)
    assert ops.library().lc_attn_bf16_supported(nh, nkv, d, 16)
    got = ops.attention(qkv, batch, kc, vc, nh, nkv, d, 16, d ** -0.5, window)
    want = ref.attention(qkv.cpu(), AttentionBatch(batch.tok_req.cpu(), batch.positions.cpu(),
                                                   batch.block_table.cpu()),
                         kc.cpu(), vc.cpu(), nh, nkv, d, 16, d ** -0.5, window)
    close(got, want, torch.bfloat16, atol=attention_atol(torch.bfloat16, vc))


def test_slow_paths_say_so_once(capfd):
    """A large bfloat16 product whose K the matrix-core kernels do not take, and bfloat16
    attention with pages that are no multiple of 16, run through the general kernels, right,
    and say so on stderr the first time."""
    ops._said.clear()
    x = torch.randn(5, 2056, device=DEV).bfloat16()
    w = torch.randn(2048, 2056, device=DEV).bfloat16()
    for _ in range(2):
        got = ops.gemm(x, w)
    close(got, ref.gemm(x.cpu(), w.cpu()), torch.bfloat16)
    qkv, batch, kc, vc = paged_case([40], [40], 4, 2, 64, 8, torch.bfloat16, seed=3)
    for _ in range(2):
        ops.attention(qkv, batch, kc, vc, 4, 2, 64, 8, 64 ** -0.5, 0)
    err = capfd.readouterr().err
    assert err.count("product with w [2048, 2056] has no matrix-core kernel") == 1
    assert err.count("pages of 8 tokens has no matrix-core kernel") == 1
    ops.gemm(torch.randn(5, 2048, device=DEV).bfloat16(), torch.randn(2048, 2048, device=DEV).bfloat16())
    assert "no matrix-core" not in capfd.readouterr().err


@pytest.mark.parametrize("nh,nkv,window", [(8, 2, 0), (4, 2, 100), (6, 1, 33), (2, 1, 0), (10, 2, 0), (3, 1, 50),
                                           (15, 3, 0)])
def test_attention_prefill_of_heads_of_128_in_pairs(nh, nkv, window):
    """Heads of 128 go in pairs of one kv head (of an odd number from three on, the last pair is
    a single head) to the prefill kernel built from 32x32x16 products: whole prompts, portions after a history, rows that do not fill a tile,
    a window whose edge cuts through groups of keys, against the plain formulas and against the
    general kernel."""
    d = 128
    lengths = [700, 64, 333, 1, 2049, 95]
    new = [700, 64, 130, 1, 300, 31]
    qkv, batch, kc, vc = paged_case(lengths, new, nh, nkv, d, 16, torch.bfloat16, seed=75)
    want = ref.attention(qkv.cpu(), AttentionBatch(batch.tok_req.cpu(), batch.positions.cpu(),
                                                   batch.block_table.cpu()),
                         kc.cpu(), vc.cpu(), nh, nkv, d, 16, d ** -0.5, window)
    lib = ops.library()
    try:
        lib.lc_attn_prefill_wide(1)
        got = ops.attention(qkv, batch, kc, vc, nh, nkv, d, 16, d ** -0.5, window)
        lib.lc_attn_prefill_wide(0)
        general = ops.attention(qkv, batch, kc, vc, nh, nkv, d, 16, d ** -0.5, window)
    finally:
        lib.lc_attn_prefill_wide(1)
    close(got, want, torch.bfloat16, atol=attention_atol(torch.bfloat16, vc))
    close(general, want, torch.bfloat16, atol=attention_atol(torch.bfloat16, vc))
    # a far key that stands out, in the first group of keys of a long tile
    q2, b2, k2, v2 = paged_case([1500], [1500], nh, nkv, d, 16, torch.bfloat16, seed=76)
    table = b2.block_table[0].tolist()
    far = 37
    k2[table[far // 16], :, far % 16, :] = 0
    k2[table[far // 16], :, far % 16, 5] = 30.0
    q2.view(1500, nh + 2 * nkv, d)[1400:, :nh, :] = 0
    q2.view(1500, nh + 2 * nkv, d)[1400:, :nh, 5] = 30.0
    out = ops.attention(q2, b2, k2, v2, nh, nkv, d, 16, d ** -0.5, 0).view(1500, nh, d)
    for h in range(nh):
        close(out[1450, h], v2[table[far // 16], h // (nh // nkv), :, far % 16], torch.bfloat16)


@pytest.mark.parametrize("nh,nkv,d,window,rot,normed", [(32, 8, 128, 0, 128, True), (6, 2, 96, 24, 96, True),
                                                        (8, 1, 64, 0, 32, False), (4, 4, 32, 0, 0, True),
                                                        (16, 1, 32, 0, 32, True)])
@pytest.mark.parametrize("waves,deep,items", [(0, 1, False), (4, 1, False), (4, 0, False), (8, 1, False),
                                              (0, 1, "always"), (4, 1, "always")])
def test_attention_decode_with_prologue_in_the_kernel(nh, nkv, d, window, rot, normed, waves, deep, items):
    """A step of single tokens with raw q, k, v: the decode kernel norms, rotates and writes
    the cache itself.  Output and cache must equal those of the separate kernel followed by
    the plain decode kernel, for short and long contexts (one or many shares of the pages),
    a token at a page's first and last place, part of the head rotated or none; with workgroups
    of four and of eight waves, the four-wave ones with two pages in flight and with one; with
    every request's pages in the same number of shares, and cut into the planner's work items."""
    lib = ops.library()
    lib.lc_attn_decode_waves(waves)
    lib.lc_attn_decode_deep(deep)
    ops.decode_by_items(items)
    try:
        decode_prologue_case(nh, nkv, d, window, rot, normed)
    finally:
        lib.lc_attn_decode_waves(0)
        lib.lc_attn_decode_deep(1)
        ops.decode_by_items(True)


def decode_prologue_case(nh, nkv, d, window, rot, normed):
    lengths = [1, 16, 17, 300, 2049, 5000, 33]
    qkv, batch, kc, vc = paged_case(lengths, [1] * len(lengths), nh, nkv, d, 16, torch.bfloat16, seed=90)
    assert ops.library().lc_attn_bf16_supported(nh, nkv, d, 16)
    qw = (1 + 0.1 * rnd(d, seed=91)) if normed else None
    kw = (1 + 0.1 * rnd(d, seed=92)) if normed else None
    table = None
    if rot:
        ang = torch.arange(6000, dtype=torch.float64)[:, None] * (10000.0 ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot))
        table = torch.cat([ang.cos(), ang.sin()], 1).float().to(DEV)
    slots = torch.tensor([int(batch.block_table[r, (n - 1) // 16]) * 16 + (n - 1) % 16
                          for r, n in enumerate(lengths)], dtype=torch.int32, device=DEV)
    # separately
    qkv1, kc1, vc1 = qkv.clone(), kc.clone(), vc.clone()
    ops.qk_norm_rope_write(qkv1, nh, nkv, d, qw, kw, 1e-6, batch.positions, table, kc1, vc1, slots, 16)
    want = ops.attention(qkv1, batch, kc1, vc1, nh, nkv, d, 16, d ** -0.5, window)
    # in the kernel
    qkv2, kc2, vc2 = qkv.clone(), kc.clone(), vc.clone()
    got = ops.attention(qkv2, batch, kc2, vc2, nh, nkv, d, 16, d ** -0.5, window,
                        ops.QKPrologue(qw, kw, 1e-6, table, slots))
    assert torch.equal(qkv2, qkv)                       # raw input untouched
    assert torch.equal(kc2, kc1) and torch.equal(vc2, vc1)
    close(got, want, torch.bfloat16, atol=attention_atol(torch.bfloat16, vc1))
    assert float((got.float() - want.float()).abs().max()) <= 2.0 ** -7 * float(want.float().abs().max())
    # no cache write asked for: the cache stays as it was, q is still prepared
    kc3, vc3 = kc1.clone(), vc1.clone()
    got3 = ops.attention(qkv.clone(), batch, kc3, vc3, nh, nkv, d, 16, d ** -0.5, window,
                         ops.QKPrologue(qw, kw, 1e-6, table, None))
    assert torch.equal(kc3, kc1) and torch.equal(vc3, vc1)
    close(got3, want, torch.bfloat16, atol=attention_atol(torch.bfloat16, vc1))


@pytest.mark.parametrize("nh,nkv,d,window,rot,normed", [(32, 8, 128, 0, 128, True), (12, 4, 128, 40, 128, True),
                                                        (6, 6, 128, 0, 0, True), (4, 2, 128, 0, 128, False),
                                                        (6, 2, 96, 24, 96, True), (8, 1, 64, 0, 32, False)])
def test_attention_mixed_step_with_raw_q(nh, nkv, d, window, rot, normed):
    """Portions of prompts beside single tokens, q, k, v raw: a kernel of its own prepares k and
    v; where the head size allows (128, rotated whole or not at all) it leaves q alone and both
    attention kernels norm and rotate their q themselves, elsewhere it prepares q too.  Either
    way the output is that of preparing everything first, and the caches agree to the bit."""
    lengths = [1, 70, 300, 2049, 16, 150, 5000, 64]
    new = [1, 70, 1, 130, 16, 2, 1, 1]
    qkv, batch, kc, vc = paged_case(lengths, new, nh, nkv, d, 16, torch.bfloat16, seed=95)
    qw = (1 + 0.1 * rnd(d, seed=96)) if normed else None
    kw = (1 + 0.1 * rnd(d, seed=97)) if normed else None
    table = None
    if rot:
        ang = torch.arange(6000, dtype=torch.float64)[:, None] * (10000.0 ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot))
        table = torch.cat([ang.cos(), ang.sin()], 1).float().to(DEV)
    pos = batch.positions.tolist()
    req = batch.tok_req.tolist()
    slots = torch.tensor([int(batch.block_table[r, p // 16]) * 16 + p % 16 for r, p in zip(req, pos)],
                         dtype=torch.int32, device=DEV)
    qkv1, kc1, vc1 = qkv.clone(), kc.clone(), vc.clone()
    ops.qk_norm_rope_write(qkv1, nh, nkv, d, qw, kw, 1e-6, batch.positions, table, kc1, vc1, slots, 16)
    want = ops.attention(qkv1, batch, kc1, vc1, nh, nkv, d, 16, d ** -0.5, window)
    qkv2, kc2, vc2 = qkv.clone(), kc.clone(), vc.clone()
    got = ops.attention(qkv2, batch, kc2, vc2, nh, nkv, d, 16, d ** -0.5, window,
                        ops.QKPrologue(qw, kw, 1e-6, table, slots))
    assert torch.equal(kc2, kc1) and torch.equal(vc2, vc1)
    own_q = bool(ops.library().lc_attn_prefill_prepares_q(d, rot))
    assert own_q == (d == 128)
    q_cols = nh * d
    assert torch.equal(qkv2[:, :q_cols], (qkv if own_q else qkv1)[:, :q_cols])     # q raw or prepared
    assert torch.equal(qkv2[:, q_cols:q_cols + nkv * d], qkv1[:, q_cols:q_cols + nkv * d])   # k prepared
    close(got, want, torch.bfloat16, atol=attention_atol(torch.bfloat16, vc1))
    assert float((got.float() - want.float()).abs().max()) <= 2.0 ** -6 * float(want.float().abs().max())


@pytest.mark.parametrize("lengths,new", [([70], [70]), ([102, 33], [70, 33]), ([40 + 50], [50]), ([64, 16, 200], [64, 16, 100]),
                                         ([2048], [2048])])
def test_k_and_v_alone_page_by_page(lengths, new):
    """q left to the attention kernels, heads of 128: where 16 rows of the batch fill one page
    in order the values are turned round in LDS and written as one piece, elsewhere row by row
    (a portion that starts in the middle of a page, a second request whose rows do not start
    at a multiple of 16, the ragged end).  Caches and k in place must equal the plain version's,
    q must stay raw."""
    nh, nkv, d, page = 6, 3, 128, 16
    qkv, batch, kc, vc = paged_case(lengths, new, nh, nkv, d, page, torch.bfloat16, seed=98)
    kw = 1 + 0.1 * rnd(d, seed=99)
    qw = 1 + 0.1 * rnd(d, seed=100)
    ang = torch.arange(4096, dtype=torch.float64)[:, None] * (10000.0 ** (-torch.arange(d // 2, dtype=torch.float64) * 2 / d))
    table = torch.cat([ang.cos(), ang.sin()], 1).float().to(DEV)
    pos, req = batch.positions.tolist(), batch.tok_req.tolist()
    slots = torch.tensor([int(batch.block_table[r, p // page]) * page + p % page for r, p in zip(req, pos)],
                         dtype=torch.int32, device=DEV)
    got_qkv, got_k, got_v = qkv.clone(), kc.clone(), vc.clone()
    ops.qk_norm_rope_write(got_qkv, nh, nkv, d, qw, kw, 1e-6, batch.positions, table, got_k, got_v, slots, page,
                           skip_q=True)
    want_qkv, want_k, want_v = qkv.clone(), kc.clone(), vc.clone()
    ref.qk_norm_rope_write(want_qkv, nh, nkv, d, qw, kw, 1e-6, batch.positions, table, want_k, want_v, slots, page)
    assert torch.equal(got_qkv[:, :nh * d], qkv[:, :nh * d])
    assert torch.equal(got_v, want_v)                          # copies
    close(got_k, want_k, torch.bfloat16)
    close(got_qkv[:, nh * d:(nh + nkv) * d], want_qkv[:, nh * d:(nh + nkv) * d], torch.bfloat16)
    # and to the bit what the kernel for all heads writes
    all_qkv, all_k, all_v = qkv.clone(), kc.clone(), vc.clone()
    ops.qk_norm_rope_write(all_qkv, nh, nkv, d, qw, kw, 1e-6, batch.positions, table, all_k, all_v, slots, page)
    assert torch.equal(got_k, all_k) and torch.equal(got_v, all_v)


@pytest.mark.parametrize("M,I,K", [(1, 16, 128), (8, 200, 256), (33, 1000, 128), (64, 96, 384), (65, 136, 256),
                                   (300, 520, 128), (2048, 256, 256), (40, 2048, 1024), (64, 12288, 512),
                                   (2, 72, 640), (14, 8200, 256), (16, 8192, 128)])
def test_gemm_with_swiglu_epilogue(M, I, K):
    """gate and up interleaved in blocks of 8 rows, silu(gate) * up formed in the epilogue."""
    x = rnd(M, K, dtype=torch.bfloat16, seed=80, scale=0.5)
    gate = rnd(I, K, dtype=torch.bfloat16, seed=81, scale=0.2)
    up = rnd(I, K, dtype=torch.bfloat16, seed=82, scale=0.2)
    w = ops.interleave_gate_up(gate, up)
    assert torch.equal(w[:8], gate[:8]) and torch.equal(w[8:16], up[:8]) and torch.equal(w[16:24], gate[8:16])
    assert ops.gemm_swiglu_supported(torch.bfloat16, w, K)
    got = ops.gemm_swiglu(x, w)
    g, u = x.double() @ gate.double().T, x.double() @ up.double().T
    want = (g / (1 + torch.exp(-g)) * u).to(torch.bfloat16)
    close(got, want, torch.bfloat16, scale=0.5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("d,page,new", [(32, 16, 1), (32, 16, 40), (48, 8, 1), (64, 16, 70)])
def test_attention_window_edge(dtype, d, page, new):
    """The key just outside the window gets a huge score and a value of its own: if the window
    were one position too wide the output would be that value.  The key just inside gets the
    same treatment and must win."""
    nh, nkv, window, length = 2, 1, 37, 200
    for inside in (False, True):
        qkv, batch, kc, vc = paged_case([length], [new], nh, nkv, d, page, dtype, seed=90)
        table = batch.block_table[0].tolist()
        qkv.zero_()
        q = qkv.view(new, nh + 2 * nkv, d)
        q[:, :nh, 5] = 30.0
        p_last = length - 1                              # the last query's position
        j = p_last - window + (1 if inside else 0)       # first visible key is p - window + 1
        kc[table[j // page], 0, j % page, :] = 0
        kc[table[j // page], 0, j % page, 5] = 30.0
        vc[table[j // page], 0, :, j % page] = 7.0
        got = ops.attention(qkv, batch, kc, vc, nh, nkv, d, page, d ** -0.5, window)[-1].float()
        if inside:
            assert float((got - 7.0).abs().max()) < 0.1
        else:
            assert float(got.abs().max()) < 5.0          # a mix of ordinary values, not the marked one


@pytest.mark.parametrize("shape", [-1, 0, 1, 2, 3])
@pytest.mark.parametrize("M,N,K", [(3, 8240, 128), (8, 16400, 512), (16, 8208, 4096), (5, 9000, 5120), (9, 24576, 6144),
                                   (1, 48, 256), (7, 4112, 1024)])
def test_gemm_bf16_few_rows_every_shape(M, N, K, shape):
    """Every shape of the kernel for up to 16 rows, chosen by size and forced; among the sizes,
    more column tiles than the CUs hold workgroups, where a workgroup takes several tiles and
    its waves keep their part of x in registers (one, two or three k blocks a wave, the last
    ones partly unused).  Plain, with the SwiGLU epilogue, with scaled rows, float32 output."""
    ops.force_gemm_skinny(shape)
    try:
        few_rows_case(M, N, K)
    finally:
        ops.force_gemm_skinny(-1)


@pytest.mark.parametrize("even", [True, False])
@pytest.mark.parametrize("M,N,K", [(1, 5120, 256), (2, 6150, 384), (8, 5120, 8192), (16, 5136, 128), (5, 6150, 4096),
                                   (9, 10250, 5120), (3, 4100, 128), (12, 7170, 6272), (8, 16001, 256)])
def test_gemm_bf16_few_rows_cut_evenly(M, N, K, even):
    """Numbers of columns that items of 16 rows of w would spread unevenly over the CUs (one and
    a quarter a CU, one and a half, two and a half): N is cut into equal items of fewer rows, whose
    last block of 16 is partly idle; with and without that, every epilogue."""
    ops.gemm_even_rows(even)
    try:
        few_rows_case(M, N, K)
    finally:
        ops.gemm_even_rows(True)


@pytest.mark.parametrize("runs", [2, 1, 0])
@pytest.mark.parametrize("M,N,K", [(8, 6144, 4096), (1, 4096, 512), (16, 24576, 1024), (5, 4112, 12288), (13, 1000, 2560),
                                   (8, 151936, 1024), (2, 300, 16384)])
def test_gemm_bf16_few_rows_in_runs(M, N, K, runs):
    """Up to 16 rows and K a multiple of 512: w is read in runs of 1 KB through LDS (one tile a
    workgroup with x streamed beside w, or several with x kept in registers) at every size (2),
    where w is large (1), or, switched off (0), as the matrix-core operand lies.  Every epilogue."""
    ops.gemm_runs(runs)
    try:
        few_rows_case(M, N, K)
    finally:
        ops.gemm_runs(True)


def few_rows_case(M, N, K):
    x = rnd(M, K, dtype=torch.bfloat16, seed=80)
    w = rnd(N, K, dtype=torch.bfloat16, seed=81, scale=K ** -0.5)
    want = x.double() @ w.double().T
    close(ops.gemm(x, w, torch.float32), want.float(), torch.float32, scale=4.0)
    close(ops.gemm(x, w, torch.bfloat16), want.to(torch.bfloat16), torch.bfloat16, scale=2.0)
    even = N // 16 * 16
    blocks = want[:, :even].reshape(M, -1, 2, 8)
    gate, up = blocks[:, :, 0, :].reshape(M, -1), blocks[:, :, 1, :].reshape(M, -1)
    close(ops.gemm_swiglu(x, w[:even]), (gate / (1 + torch.exp(-gate)) * up).to(torch.bfloat16), torch.bfloat16, scale=2.0)
    h = rnd(M, K, seed=82, scale=1.5)
    g = 1 + rnd(K, seed=83, scale=0.2)
    rows = ops.rmsnorm(h, None, g, 1e-6, torch.bfloat16, scaled=True)
    factors = torch.rsqrt((h.double() ** 2).mean(1, keepdim=True) + 1e-6)
    close(ops.gemm(rows, w, torch.bfloat16), ((rows.x.double() @ w.double().T) * factors).to(torch.bfloat16),
          torch.bfloat16, scale=2.0)


@pytest.mark.parametrize("M,H,K", [(40, 512, 2048), (64, 4096, 4096), (100, 384, 1024), (17, 1152, 1536)])
@pytest.mark.parametrize("small", [1, 0])
def test_norm_sums_the_shares_of_a_product_cut_along_k(M, H, K, small):
    """More than 16 rows and few tiles: the product before a norm is cut along K; its shares
    stay float32 and the norm kernel adds them to the stream itself (all rows, and chosen rows
    with the stream left alone)."""
    ops.library().lc_gemm_bf16_small_partials(small)     # up to 64 rows: tiles of 64 x 64 or of 64 x 128
    try:
        norm_of_shares_case(M, H, K)
    finally:
        ops.library().lc_gemm_bf16_small_partials(1)


def norm_of_shares_case(M, H, K):
    eps = 1e-6
    h = rnd(M, H, seed=90, scale=2.0)
    x = rnd(M, K, dtype=torch.bfloat16, seed=91)
    w = rnd(H, K, dtype=torch.bfloat16, seed=92, scale=K ** -0.5)
    g = 1 + rnd(H, seed=93, scale=0.2)
    assert ops.library().lc_gemm_bf16_shares(M, H, K) > 1
    pending = ops.gemm(x, w, torch.bfloat16, defer=True)
    assert isinstance(pending, ops.PendingProduct)
    h_want = h.double() + x.double() @ w.double().T
    normed = h_want * torch.rsqrt((h_want ** 2).mean(1, keepdim=True) + eps) * g.double()
    rows = torch.tensor([M - 1, 0, 3], dtype=torch.int32, device=DEV)
    h_rows = h.clone()
    got_rows = ops.rmsnorm(h_rows, pending, g, eps, torch.bfloat16, rows=rows)
    assert torch.equal(h_rows, h)
    close(got_rows, normed[rows.long()].to(torch.bfloat16), torch.bfloat16)
    h_got = h.clone()
    got = ops.rmsnorm(h_got, pending, g, eps, torch.bfloat16, scaled=True)
    assert isinstance(got, torch.Tensor)
    torch.testing.assert_close(h_got.double(), h_want, rtol=1e-5, atol=1e-5)
    close(got, normed.to(torch.bfloat16), torch.bfloat16)
    close(ops.value(pending), (x.double() @ w.double().T).to(torch.bfloat16), torch.bfloat16, scale=2.0)


def test_feed_tokens():
    gen = torch.Generator().manual_seed(5)
    ids = torch.randint(0, 1000, (37,), generator=gen, dtype=torch.int32)
    sampled = torch.randint(0, 1000, (9,), generator=gen, dtype=torch.int32)
    source = torch.full((37,), -1, dtype=torch.int32)
    source[[0, 5, 6, 36]] = torch.tensor([3, 8, 3, 0], dtype=torch.int32)
    want = ids.clone()
    ref.feed_tokens(want, source, sampled)
    got = ids.to(DEV)
    ops.feed_tokens(got, source.to(DEV), sampled.to(DEV))
    assert torch.equal(got.cpu(), want)
    with pytest.raises(ops.KernelError):
        ops.feed_tokens(got, source.to(DEV)[:5], sampled.to(DEV))


@pytest.mark.parametrize("nh,nkv,d,window,lengths,new", [
    (32, 8, 128, 0, [8192], [576]),               # pairs of heads, four shares
    (32, 8, 128, 0, [5000, 1], [100, 1]),         # single heads, eight shares, a decode token beside
    (8, 2, 64, 0, [5000, 3000], [100, 70]),
    (4, 4, 96, 1000, [6000], [130]),              # a window: the shares cover its pages only
    (16, 1, 32, 0, [4100, 700], [64, 3]),
    (32, 8, 128, 0, [900], [576])])               # no more than a share's worth of keys: not cut
def test_attention_prefill_shares_of_the_keys(nh, nkv, d, window, lengths, new):
    """A portion of a prompt after a long history is few tiles with many keys each: the tiles'
    pages are shared out over several workgroups and joined, as the decode kernel does it."""
    qkv, batch, kc, vc = paged_case(lengths, new, nh, nkv, d, 16, torch.bfloat16, seed=77)
    nt = batch.prefill_tiles.shape[0]
    splits = ops.library().lc_attn_prefill_splits(nt, nh, nkv, batch.max_ctx)
    assert (splits > 1) == (max(lengths) >= 2048)
    got = ops.attention(qkv, batch, kc, vc, nh, nkv, d, 16, d ** -0.5, window)
    want = ref.attention(qkv.cpu(), AttentionBatch(batch.tok_req.cpu(), batch.positions.cpu(),
                                                   batch.block_table.cpu()),
                         kc.cpu(), vc.cpu(), nh, nkv, d, 16, d ** -0.5, window)
    close(got, want, torch.bfloat16, atol=attention_atol(torch.bfloat16, vc))


@pytest.mark.parametrize("nh,nkv,d,window", [(32, 8, 128, 0), (6, 2, 96, 700), (8, 1, 64, 0), (4, 2, 32, 0)])
@pytest.mark.parametrize("waves,items", [(0, False), (4, False), (0, "always"), (0, True)])
def test_attention_decode_of_many_requests_of_unequal_length(nh, nkv, d, window, waves, items):
    """So many requests that each gets one workgroup per kv head (of eight waves then), lengths
    from one token to thousands; also with workgroups of four waves, which walk their pages
    with two in flight: every number of pages a wave, from none on, the first and the last turn
    of the three sets of page registers; and through the planner's list of work items, which cuts
    the long requests into more shares than the short ones."""
    rng = random.Random(5)
    lengths = [rng.choice([1, 15, 16, 17, 100, 700, 2100, 3000]) for _ in range(70)]
    lengths[:14] = [16 * 4 * n + k for n in range(7) for k in (1, 16)]     # 0 to 6 whole rounds of four waves, and one page more
    qkv, batch, kc, vc = paged_case(lengths, [1] * len(lengths), nh, nkv, d, 16, torch.bfloat16, seed=95)
    if nkv >= 8:
        assert ops.library().lc_attn_decode_splits(len(lengths), nkv, max(lengths)) == 1
    ops.library().lc_attn_decode_waves(waves)
    ops.decode_by_items(items)
    try:
        got = ops.attention(qkv, batch, kc, vc, nh, nkv, d, 16, d ** -0.5, window)
    finally:
        ops.library().lc_attn_decode_waves(0)
        ops.decode_by_items(True)
    want = ref.attention(qkv.cpu(), AttentionBatch(batch.tok_req.cpu(), batch.positions.cpu(),
                                                   batch.block_table.cpu()),
                         kc.cpu(), vc.cpu(), nh, nkv, d, 16, d ** -0.5, window)
    close(got, want, torch.bfloat16, atol=attention_atol(torch.bfloat16, vc))


@pytest.mark.parametrize("nh,nkv,window,rot,normed,count", [(32, 8, 0, 128, True, 5), (12, 4, 40, 128, True, 1),
                                                            (4, 4, 0, 0, False, 3), (16, 2, 0, 128, False, 8)])
def test_attention_decode_takes_q_k_v_as_shares_of_a_product(nh, nkv, window, rot, normed, count):
    """A step of single tokens whose q/k/v product was cut along K: the decode kernel sums the
    float32 shares as it reads them.  Output and caches equal, to the bit, those of summing the
    shares first (in their order, rounded to bfloat16) and handing the kernel the sum."""
    d = 128
    lengths = [1, 16, 17, 300, 2049, 5000, 33]
    T = len(lengths)
    _, batch, kc, vc = paged_case(lengths, [1] * T, nh, nkv, d, 16, torch.bfloat16, seed=97)
    width = (nh + 2 * nkv) * d
    partials = rnd(count, T, width, seed=98, scale=count ** -0.5)
    shares = ops.ProductShares(partials, torch.bfloat16)
    summed = shares.value()
    plain = torch.zeros(T, width, device=DEV)
    for s in range(count):
        plain += partials[s]
    assert torch.equal(summed, plain.to(torch.bfloat16))
    qw = (1 + 0.1 * rnd(d, seed=91)) if normed else None
    kw = (1 + 0.1 * rnd(d, seed=92)) if normed else None
    table = make_rope_table(6000, rot, 10000.0) if rot else None
    slots = torch.tensor([int(batch.block_table[r, (n - 1) // 16]) * 16 + (n - 1) % 16
                          for r, n in enumerate(lengths)], dtype=torch.int32, device=DEV)
    assert ops.attention_takes_shares(batch, T, nh, nkv, d, 16, torch.bfloat16, rot)
    kc1, vc1 = kc.clone(), vc.clone()
    want = ops.attention(summed.clone(), batch, kc1, vc1, nh, nkv, d, 16, d ** -0.5, window,
                         ops.QKPrologue(qw, kw, 1e-6, table, slots))
    kc2, vc2 = kc.clone(), vc.clone()
    got = ops.attention(shares, batch, kc2, vc2, nh, nkv, d, 16, d ** -0.5, window,
                        ops.QKPrologue(qw, kw, 1e-6, table, slots))
    assert torch.equal(got, want)
    assert torch.equal(kc2, kc1) and torch.equal(vc2, vc1)
    # where the kernel cannot (a prompt portion in the step), the shares are summed first
    _, mixed, kc3, vc3 = paged_case([40, 9], [1, 4], nh, nkv, d, 16, torch.bfloat16, seed=99)
    assert not ops.attention_takes_shares(mixed, 5, nh, nkv, d, 16, torch.bfloat16, rot)
    part5 = rnd(2, 5, width, seed=100)
    slots5 = torch.tensor([int(mixed.block_table[0, 2]) * 16 + 7] +
                          [int(mixed.block_table[1, 0]) * 16 + i for i in range(5, 9)], dtype=torch.int32, device=DEV)
    a = ops.attention(ops.ProductShares(part5, torch.bfloat16), mixed, kc3.clone(), vc3.clone(), nh, nkv, d, 16,
                      d ** -0.5, window, ops.QKPrologue(qw, kw, 1e-6, table, slots5))
    b = ops.attention(ops.ProductShares(part5, torch.bfloat16).value(), mixed, kc3.clone(), vc3.clone(), nh, nkv, d,
                      16, d ** -0.5, window, ops.QKPrologue(qw, kw, 1e-6, table, slots5))
    assert torch.equal(a, b)


def test_decode_attention_keeps_its_page_registers_in_registers():
    """The decode kernel's walk with two pages in flight fills its page registers with loads that
    the compiler does not count; that is only sound while none of them is spilled.  The library asks
    its compiled kernels and must find them without scratch memory (else it would quietly walk with
    one page in flight)."""
    for d in (32, 64, 96, 128):
        assert ops.library().lc_attn_decode_deep_ok(d) == 1


def test_runs_kernel_keeps_its_ring_of_x_in_registers():
    """The form of the runs kernel that fills a ring of registers with hand-counted loads is
    only sound while the compiler keeps that ring in registers; the library asks its compiled
    kernels and must find them without scratch memory (else it would quietly run the slower
    kernel)."""
    assert ops.library().lc_gemm_bf16_runs_ring_ok() == 1
