"""Plain torch versions of every kernel in ``lucciola_amd.kernels.ops``, with the same
signatures and memory layouts (paged caches, block tables, slot lists).  They compute in
float64 and round once to the output dtype.  Two uses: each GPU kernel is tested alone against
its function here, and CPU tests put these in place of the kernels to exercise the step
function, the cache and the scheduler without a GPU.  Nothing under ``lucciola_amd`` imports
this file.
"""
import torch

F64 = torch.float64


def embedding(ids, table, scale=1.0):
    return table[ids.long()].to(torch.float32) * scale


def rmsnorm(h, delta, weight, eps, out_dtype, rows=None, scaled=False):   # never hands out scaled rows
    if rows is None:
        if delta is not None:
            h += delta.to(torch.float32)
        v = h.to(F64)
    else:
        v = h[rows.long()].to(F64)
        if delta is not None:
            v = (h[rows.long()] + delta[rows.long()].to(torch.float32)).to(F64)
    inv = torch.rsqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    return (v * inv * weight.to(F64)).to(out_dtype)


def rmsnorm_act(x, weight, eps):
    v = x.to(F64)
    inv = torch.rsqrt((v * v).mean(dim=-1, keepdim=True) + eps)
    return (v * inv * weight.to(F64)).to(x.dtype)


def gemm(x, w, out_dtype=None, defer=False, shares=False):   # never defers, never hands out shares
    return (x.to(F64) @ w.to(F64).T).to(out_dtype or x.dtype)


def qk_norm_rope_write(qkv, nh, nkv, d, q_weight, k_weight, eps, positions, rope_table,
                       k_cache, v_cache, slots, page_size):
    T = qkv.shape[0]
    x = qkv.view(T, nh + 2 * nkv, d)
    q, k, v = x[:, :nh].to(F64), x[:, nh:nh + nkv].to(F64), x[:, nh + nkv:]
    if q_weight is not None:
        q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * q_weight.to(F64)
        k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * k_weight.to(F64)
    if rope_table is not None:
        rot = rope_table.shape[1]
        half = rot // 2
        cs = rope_table[positions.long()].to(F64)
        cos, sin = cs[:, None, :half], cs[:, None, half:]

        def rotate(t):
            a, b = t[..., :half], t[..., half:rot]
            return torch.cat([a * cos - b * sin, a * sin + b * cos, t[..., rot:]], dim=-1)
        q, k = rotate(q), rotate(k)
    x[:, :nh] = q.to(qkv.dtype)
    x[:, nh:nh + nkv] = k.to(qkv.dtype)
    if k_cache is not None and slots is not None:
        for t in range(T):
            s = int(slots[t])
            if s < 0:
                continue
            page, off = divmod(s, page_size)
            k_cache[page, :, off, :] = x[t, nh:nh + nkv]
            v_cache[page, :, :, off] = v[t]


def attention(qkv, batch, k_cache, v_cache, nh, nkv, d, page_size, scale, window=0, prologue=None):
    if prologue is not None:
        qk_norm_rope_write(qkv, nh, nkv, d, prologue.q_weight, prologue.k_weight, prologue.eps,
                           batch.positions, prologue.rope_table, k_cache, v_cache, prologue.slots,
                           page_size)
    T = qkv.shape[0]
    q = qkv.view(T, nh + 2 * nkv, d)[:, :nh].to(F64)
    out = torch.zeros(T, nh, d, dtype=F64, device=qkv.device)
    group = nh // nkv
    tok_req = batch.tok_req.tolist()
    positions = batch.positions.tolist()
    tables = batch.block_table.tolist()
    for t in range(T):
        p = positions[t]
        lo = max(0, p - window + 1) if window else 0
        table = tables[tok_req[t]]
        js = list(range(lo, p + 1))
        pages = torch.tensor([table[j // page_size] for j in js], dtype=torch.long)
        assert (pages >= 0).all(), "attention reads a page that was given back"
        offs = torch.tensor([j % page_size for j in js], dtype=torch.long)
        keys = k_cache[pages, :, offs, :].to(F64)      # [n, nkv, d]
        vals = v_cache[pages, :, :, offs].to(F64)
        for h in range(nh):
            s = (keys[:, h // group, :] @ q[t, h]) * scale
            w = torch.softmax(s, dim=0)
            out[t, h] = w @ vals[:, h // group, :]
    return out.reshape(T, nh * d).to(qkv.dtype)


def swiglu(gu):
    I = gu.shape[1] // 2
    g, u = gu[:, :I].to(F64), gu[:, I:].to(F64)
    return (g / (1 + torch.exp(-g)) * u).to(gu.dtype)


def sample(logits, temperature=None, uniform=None):
    R = logits.shape[0]
    out = torch.empty(R, dtype=torch.int32, device=logits.device)
    for r in range(R):
        t = float(temperature[r]) if temperature is not None else 0.0
        if t <= 0:
            out[r] = int(torch.argmax(logits[r]))
            continue
        z = logits[r].to(F64) / t
        p = torch.exp(z - z.max())
        cdf = torch.cumsum(p, 0)
        target = float(uniform[r]) * float(cdf[-1])
        out[r] = int(min(int(torch.searchsorted(cdf, torch.tensor(target, dtype=F64), right=True)),
                         logits.shape[1] - 1))
    return out


def attention_takes_shares(*args, **kwargs):
    return False


def feed_tokens(ids, source, sampled):
    take = source >= 0
    ids[take] = sampled[source[take].long()]


ALL = ("feed_tokens", "attention_takes_shares", "embedding", "rmsnorm", "rmsnorm_act", "gemm", "qk_norm_rope_write", "attention",
       "swiglu", "sample")


def install(monkeypatch):
    """Put these functions in place of the kernels (CPU tests of the engine's host logic)."""
    from lucciola_amd.kernels import ops
    for name in ALL:
        monkeypatch.setattr(ops, name, globals()[name])
