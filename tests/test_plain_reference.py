"""What fixes the plain implementation (tests/plain_qwen3.py) beside the reference's text:
special cases that reduce to a library routine, invariants, and the vectors the reference's own
files hold.  Each is chosen so that a plausible mistake fails it (a wrong pairing or sign in
the rotation, a norm in the wrong place, a wrong kv-head map, an off-by-one in the mask)."""
import math

import pytest
import torch
import torch.nn.functional as F

import configs
import plain_qwen3 as plain
from helpers import random_weights

F64 = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64)


def test_embedding_is_row_lookup():
    table = rnd(11, 6)
    ids = [3, 0, 10, 3]
    assert torch.equal(plain.embedding(ids, table), F.embedding(torch.tensor(ids), table))


def test_linear_is_x_times_w_transposed_without_bias():
    x, w = rnd(5, 7), rnd(4, 7, seed=1)
    torch.testing.assert_close(plain.linear(x, w), F.linear(x, w))


def test_rmsnorm_reduces_to_the_library_routine():
    x, w = rnd(6, 20), 1 + 0.1 * rnd(20, seed=1)
    for eps in (1e-6, 1e-5, 1e-2):
        torch.testing.assert_close(plain.rmsnorm(x, w, eps), F.rms_norm(x, (20,), w, eps))
    unit = plain.rmsnorm(x, torch.ones(20, dtype=F64), 0.0)
    torch.testing.assert_close((unit * unit).mean(-1), torch.ones(6, dtype=F64))
    # eps sits inside the square root, added to the MEAN of squares (not to the sum)
    tiny = torch.full((1, 4), 1e-3, dtype=F64)
    got = plain.rmsnorm(tiny, torch.ones(4, dtype=F64), 1e-6)
    torch.testing.assert_close(got, tiny / math.sqrt(1e-6 + 1e-6))


def test_rope_position_zero_is_identity_and_norms_are_kept():
    x = rnd(3, 2, 16)
    torch.testing.assert_close(plain.rope(x, [0, 0, 0], 1e4), x)
    y = plain.rope(x, [5, 17, 300], 1e4)
    half = 8
    torch.testing.assert_close(y[..., :half] ** 2 + y[..., half:] ** 2,
                               x[..., :half] ** 2 + x[..., half:] ** 2)


def test_rope_pairs_i_with_i_plus_half():
    # src/kernels/rope.cu:46-48: the partner of feature i is i + d/2, not i + 1
    d = 8
    x = torch.zeros(1, 1, d, dtype=F64)
    x[0, 0, 1] = 1.0
    y = plain.rope(x, [3], 100.0)[0, 0]
    angle = 3 / 100.0 ** (2 * 1 / d)
    want = torch.zeros(d, dtype=F64)
    want[1], want[1 + d // 2] = math.cos(angle), math.sin(angle)      # x cos, +x sin (rope.cu:55-56)
    torch.testing.assert_close(y, want)
    # the second half rotates back into the first with a minus sign
    x = torch.zeros(1, 1, d, dtype=F64)
    x[0, 0, 1 + d // 2] = 1.0
    y = plain.rope(x, [3], 100.0)[0, 0]
    want = torch.zeros(d, dtype=F64)
    want[1], want[1 + d // 2] = -math.sin(angle), math.cos(angle)
    torch.testing.assert_close(y, want)


def test_rope_depends_on_distances_only():
    q, k = rnd(1, 1, 32), rnd(1, 1, 32, seed=1)
    for theta in (1e4, 1e6):
        a = (plain.rope(q, [40], theta) * plain.rope(k, [33], theta)).sum()
        b = (plain.rope(q, [7], theta) * plain.rope(k, [0], theta)).sum()
        torch.testing.assert_close(a, b)
    # and theta matters
    assert not torch.allclose(plain.rope(q, [40], 1e4), plain.rope(q, [40], 1e6))


@pytest.mark.parametrize("nh,nkv", [(4, 4), (4, 2), (8, 1), (6, 2)])
def test_attention_reduces_to_the_library_routine(nh, nkv):
    T, d = 9, 16
    q, k, v = rnd(T, nh, d), rnd(T, nkv, d, seed=1), rnd(T, nkv, d, seed=2)
    got = plain.attention(q, k, v, list(range(T)))
    kk = k.repeat_interleave(nh // nkv, dim=1)      # kv head of query head h is h // (nh // nkv)
    vv = v.repeat_interleave(nh // nkv, dim=1)
    want = F.scaled_dot_product_attention(q.transpose(0, 1), kk.transpose(0, 1), vv.transpose(0, 1),
                                          is_causal=True).transpose(0, 1)
    torch.testing.assert_close(got, want)


def test_attention_special_cases():
    d = 8
    q, k, v = rnd(1, 2, d), rnd(1, 1, d, seed=1), rnd(1, 1, d, seed=2)
    out = plain.attention(q, k, v, [5])                 # one key: the output is its value
    torch.testing.assert_close(out[0, 0], v[0, 0])
    torch.testing.assert_close(out[0, 1], v[0, 0])
    # one head, no mask effect on the last row: plain softmax(q k^T / sqrt(d)) v
    T = 6
    q, k, v = rnd(T, 1, d), rnd(T, 1, d, seed=3), rnd(T, 1, d, seed=4)
    last = plain.attention(q, k, v, list(range(T)))[-1, 0]
    w = torch.softmax(k[:, 0] @ q[-1, 0] / math.sqrt(d), 0)
    torch.testing.assert_close(last, w @ v[:, 0])
    # the first row sees only itself
    torch.testing.assert_close(plain.attention(q, k, v, list(range(T)))[0, 0], v[0, 0])


def test_attention_window_counts_the_query_itself():
    """The reference has no sliding window (its kernels mask by position only,
    src/kernels/attention.cu:90-92), so what a window means here is the engine's own choice and
    parity is unpinned: a query at p sees the w positions p - w + 1 .. p.  What pins the plain
    form: a window of one leaves each row its own value, a window as long as the sequence is
    no window, and a key that every query loves stops counting exactly w positions later."""
    T, d, w = 12, 8, 4
    q1, k1, v1 = rnd(T, 2, d), rnd(T, 1, d, seed=1), rnd(T, 1, d, seed=2)
    torch.testing.assert_close(plain.attention(q1, k1, v1, list(range(T)), window=1),
                               v1.expand(T, 2, d).contiguous())
    loved = 3
    q2, k2, v2 = torch.zeros(T, 1, d, dtype=torch.float64), torch.zeros(T, 1, d, dtype=torch.float64), rnd(T, 1, d, seed=5)
    q2[:, 0, 0] = 50.0
    k2[loved, 0, 0] = 50.0
    seen = plain.attention(q2, k2, v2, list(range(T)), window=w)
    for t in range(loved, T):
        if t - loved < w:       # still inside the window: the loved key takes all the weight
            torch.testing.assert_close(seen[t, 0], v2[loved, 0])
        else:                   # w positions later it is gone: the mean of the window's values
            torch.testing.assert_close(seen[t, 0], v2[t - w + 1:t + 1, 0].mean(0))
    q, k, v = rnd(T, 1, d), rnd(T, 1, d, seed=1), rnd(T, 1, d, seed=2)
    got = plain.attention(q, k, v, list(range(T)), window=w)
    for t in range(T):
        lo = max(0, t - w + 1)                          # w positions: t - w + 1 .. t
        wts = torch.softmax(k[lo:t + 1, 0] @ q[t, 0] / math.sqrt(d), 0)
        torch.testing.assert_close(got[t, 0], wts @ v[lo:t + 1, 0])
    torch.testing.assert_close(plain.attention(q, k, v, list(range(T)), window=T),
                               plain.attention(q, k, v, list(range(T))))


def test_swiglu_is_silu_times_up():
    g, u = rnd(4, 10) * 3, rnd(4, 10, seed=1)
    torch.testing.assert_close(plain.swiglu(g, u), F.silu(g) * u)
    assert float(plain.swiglu(torch.zeros(3, dtype=F64), u[0, :3]).abs().max()) == 0.0


def test_softmax_vectors_of_the_reference():
    # learn/softmax.cc:8 feeds [1, 2, 3, 4]; learn/softmax.cc:44-46 feeds 1..1024
    for x in (torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=F64), torch.arange(1, 1025, dtype=F64)):
        p = torch.softmax(x, 0)
        cdf = p.cumsum(0)
        for u in (0.0, 0.3, 0.77, 0.999):
            tok = plain.sample_token(x, 1.0, u)
            assert cdf[tok] > u and (tok == 0 or cdf[tok - 1] <= u)
        assert plain.sample_token(x, 0.0, 0.5) == len(x) - 1
        assert plain.sample_token(x, 1e-3, 0.5) == len(x) - 1     # temperature -> 0 is the argmax


@pytest.mark.parametrize("key", ["A", "B", "C", "D"])
def test_residual_wiring(key):
    cfg, _, seed = configs.ALL[key]
    w = {k: v.clone() for k, v in random_weights(cfg, seed).items()}
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    full = plain.forward(cfg, w, ids)
    # both branches silenced: the logits are head(norm(embedding))
    for name in w:
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            w[name] = torch.zeros_like(w[name])
    head = w.get("lm_head.weight", w["model.embed_tokens.weight"])
    want = plain.linear(plain.rmsnorm(plain.embedding(ids, w["model.embed_tokens.weight"]),
                                      w["model.norm.weight"], cfg["rms_norm_eps"]), head)
    torch.testing.assert_close(plain.forward(cfg, w, ids), want)
    assert not torch.allclose(full, want)


@pytest.mark.parametrize("key", ["A", "B", "C", "D"])
def test_shifting_all_positions_changes_nothing(key):
    cfg, _, seed = configs.ALL[key]
    w = random_weights(cfg, seed)
    ids = [7, 7, 2, 9, 1, 0, 3, 3, 8, 5, 4, 6] * 3
    torch.testing.assert_close(plain.forward(cfg, w, ids, first_position=0),
                               plain.forward(cfg, w, ids, first_position=37), rtol=1e-9, atol=1e-11)


def test_causality_and_heads():
    cfg, _, seed = configs.ALL["B"]
    w = random_weights(cfg, seed)
    ids = list(range(20))
    a = plain.forward(cfg, w, ids)
    b = plain.forward(cfg, w, ids[:12] + [99] * 8)
    torch.testing.assert_close(a[:12], b[:12])           # later tokens do not reach back
    assert not torch.allclose(a[12:], b[12:])
    # tied and separate heads differ only in the last product
    cfg_a, _, seed_a = configs.ALL["A"]
    wa = random_weights(cfg_a, seed_a)
    assert "lm_head.weight" not in wa
    wa2 = dict(wa)
    wa2["lm_head.weight"] = wa["model.embed_tokens.weight"]
    torch.testing.assert_close(plain.forward(cfg_a, wa, ids[:5]),
                               plain.forward(dict(cfg_a, tie_word_embeddings=False), wa2, ids[:5]))


def test_window_of_config_c_matters():
    cfg, _, seed = configs.ALL["C"]
    w = random_weights(cfg, seed)
    ids = [i % 50 for i in range(60)]
    with_window = plain.forward(cfg, w, ids)
    without = plain.forward(dict(cfg, use_sliding_window=False,
                                 layer_types=["full_attention"] * 4), w, ids)
    torch.testing.assert_close(with_window[:24], without[:24])      # inside the first window
    assert not torch.allclose(with_window[40:], without[40:])
