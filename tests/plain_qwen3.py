"""A plain, slow implementation of the Qwen3 dense decoder: whole sequences, no cache, one
function for each part, float64 on the CPU.  Written from the formulas of the reference's
kernels (each function cites file:line of the reference's tree); it shares no code with the
engine under ``lucciola_amd`` and is what the engine is compared with.
"""
import hashlib
import math

import numpy as np
import torch

F64 = torch.float64


def embedding(ids, table):
    """out[t, :] = table[ids[t], :]   (src/kernels/embedding.cu:22-38)"""
    return table[torch.as_tensor(ids, dtype=torch.long)].to(F64)


def rmsnorm(x, weight, eps):
    """y_i = x_i * rsqrt(sum_j x_j^2 / n + eps) * w_i over the last dimension
    (src/kernels/rmsnorm.cu:56-97: sum of squares :60-69, rsqrtf(sum/hidden + eps) :77,
    val * rms * w :94)."""
    x = x.to(F64)
    n = x.shape[-1]
    inv = 1.0 / torch.sqrt((x * x).sum(dim=-1, keepdim=True) / n + eps)
    return x * inv * weight.to(F64)


def linear(x, weight):
    """Y[m, n] = sum_k X[m, k] * W[n, k], no bias   (src/kernels/linear.cu:24-52)"""
    return x.to(F64) @ weight.to(F64).T


def rope(x, positions, theta):
    """x: [T, heads, d].  For pair i in [0, d/2): freq = 1 / theta^(2i/d); angle = pos * freq;
    (x[i], x[i + d/2]) -> (x[i] cos - x[i+d/2] sin, x[i] sin + x[i+d/2] cos)
    (src/kernels/rope.cu:28-60: freq :33-34, angle :35, halves :46-48, rotation :55-56)."""
    x = x.to(F64)
    d = x.shape[-1]
    half = d // 2
    i = torch.arange(half, dtype=F64)
    freq = 1.0 / torch.pow(torch.tensor(float(theta), dtype=F64), 2.0 * i / d)
    angle = torch.as_tensor(positions, dtype=F64)[:, None] * freq[None, :]   # [T, d/2]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1)


def attention(q, k, v, positions, scale=None, window=None):
    """q: [T, nh, d]; k, v: [T, nkv, d]; one sequence, token t at absolute position
    positions[t] (increasing).  kv head of query head h is h // (nh // nkv)
    (src/kernels/attention.cu:53); score = q . k * scale with scale = 1/sqrt(d) (:60-66);
    a query sees the keys at positions <= its own (:90-92) and, with a window w, only those at
    positions > its own - w; softmax with the maximum subtracted (:88-106); out = P . v
    (:129-144)."""
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    T, nh, d = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    pos = torch.as_tensor(positions, dtype=torch.long)
    out = torch.zeros(T, nh, d, dtype=F64)
    for h in range(nh):
        kh = h // group
        s = (q[:, h, :] @ k[:, kh, :].T) * scale                 # [T, T]
        visible = pos[None, :] <= pos[:, None]
        if window:
            visible &= pos[None, :] > pos[:, None] - window
        s = s.masked_fill(~visible, float("-inf"))
        s = s - s.max(dim=-1, keepdim=True).values
        p = torch.exp(s)
        p = p / p.sum(dim=-1, keepdim=True)
        out[:, h, :] = p @ v[:, kh, :]
    return out


def swiglu(gate, up):
    """silu(g) * u with silu(g) = g / (1 + exp(-g))   (src/kernels/swiglu.cu:8,31-35)"""
    gate, up = gate.to(F64), up.to(F64)
    return gate / (1.0 + torch.exp(-gate)) * up


def attention_block(x, w, prefix, cfg, positions, window=None, kv_from=None):
    """Projections -> per-head RMSNorm of q and k over head_dim with one [d] weight each ->
    rotary on q and k -> attention -> output projection (src/qwen.cc:592-738; QK-norm before
    the rotation :617-644).  Returns (output, (k, v)); ``kv_from`` replaces this block's own
    keys and values (a site that reads another site's cache)."""
    T = x.shape[0]
    nh, nkv, d = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_norm_eps"], cfg["rope_theta"]
    q = linear(x, w[prefix + "q_proj.weight"]).view(T, nh, d)
    q = rope(rmsnorm(q, w[prefix + "q_norm.weight"], eps), positions, theta)
    if kv_from is None:
        k = linear(x, w[prefix + "k_proj.weight"]).view(T, nkv, d)
        v = linear(x, w[prefix + "v_proj.weight"]).view(T, nkv, d)
        k = rope(rmsnorm(k, w[prefix + "k_norm.weight"], eps), positions, theta)
    else:
        k, v = kv_from
    o = attention(q, k, v, positions, window=window).reshape(T, nh * d)
    return linear(o, w[prefix + "o_proj.weight"]), (k, v)


def mlp_block(x, w, prefix):
    """down(silu(gate(x)) * up(x))   (src/qwen.cc:762-794)"""
    return linear(swiglu(linear(x, w[prefix + "gate_proj.weight"]),
                         linear(x, w[prefix + "up_proj.weight"])),
                  w[prefix + "down_proj.weight"])


def normalize_config(cfg):
    cfg = dict(cfg)
    cfg.setdefault("num_key_value_heads", cfg["num_attention_heads"])       # src/qwen.cc:53-54
    cfg.setdefault("head_dim", cfg["hidden_size"] // cfg["num_attention_heads"])  # :55-56
    cfg.setdefault("rms_norm_eps", 1e-6)     # the reference's literal, src/qwen.cc:588
    cfg.setdefault("rope_theta", 1e6)        # the reference's literal, src/qwen.cc:636
    return cfg


def layer_windows(cfg):
    L = cfg["num_hidden_layers"]
    types = cfg.get("layer_types")
    if types is None:
        use = cfg.get("use_sliding_window", False) and cfg.get("sliding_window") is not None
        first = cfg.get("max_window_layers", L)
        types = ["sliding_attention" if use and i >= first else "full_attention" for i in range(L)]
    return [cfg.get("sliding_window") if t == "sliding_attention" else None for t in types]


def forward(cfg, weights, ids, first_position=0, run_order=None):
    """Logits [T, vocab] (float64) of one whole sequence.  Pre-norm residual wiring
    (src/qwen.cc:574-589,741-759,797-798): r = h; x = norm_in(h); h = attn(x) + r; r = h;
    x = norm_post(h); h = mlp(x) + r; then the final norm and the head (src/qwen.cc:851-882),
    the head being the embedding table when there is no lm_head.weight (src/qwen.cc:80-84).
    ``run_order``: list of (layer, cache_of) pairs; default every layer once, in order."""
    cfg = normalize_config(cfg)
    eps = cfg["rms_norm_eps"]
    T = len(ids)
    positions = list(range(first_position, first_position + T))
    windows = layer_windows(cfg)
    if run_order is None:
        run_order = [(i, None) for i in range(cfg["num_hidden_layers"])]
    h = embedding(ids, weights["model.embed_tokens.weight"])
    kvs = []
    for layer, cache_of in run_order:
        p = f"model.layers.{layer}."
        x = rmsnorm(h, weights[p + "input_layernorm.weight"], eps)
        a, kv = attention_block(x, weights, p + "self_attn.", cfg, positions, windows[layer],
                                kv_from=None if cache_of is None else kvs[cache_of])
        kvs.append(kv)
        h = h + a
        x = rmsnorm(h, weights[p + "post_attention_layernorm.weight"], eps)
        h = h + mlp_block(x, weights, p + "mlp.")
    x = rmsnorm(h, weights["model.norm.weight"], eps)
    head = weights.get("lm_head.weight")
    if head is None or cfg.get("tie_word_embeddings", False):
        head = weights["model.embed_tokens.weight"]
    return linear(x, head)


def greedy(cfg, weights, prompt, new_tokens):
    """Greedy generation by running the whole sequence again for every token; ties go to the
    lowest index."""
    ids = list(prompt)
    out = []
    for _ in range(new_tokens):
        logits = forward(cfg, weights, ids)[-1]
        tok = int(torch.argmax(logits))
        out.append(tok)
        ids.append(tok)
    return out


def sample_token(logits, temperature, u):
    """Temperature sampling by inverse CDF: p = softmax(logits / temperature); the token is
    the first index whose cumulative probability exceeds u * sum(p)."""
    if temperature <= 0:
        return int(torch.argmax(logits))
    z = logits.to(F64) / temperature
    p = torch.exp(z - z.max())
    cdf = torch.cumsum(p, 0)
    return int(torch.searchsorted(cdf, torch.tensor(u, dtype=F64) * cdf[-1], right=True).clamp(max=len(p) - 1))


def random_weight(seed, name, shape, std, plus_one=False):
    """The engine's random weights, computed again in numpy (the reference has no random
    weights, src/qwen.cc:69-84; the recipe is the engine's own and is written out here from
    its description, not from its code): a value depends on (seed, tensor name, element
    index) only.  key = mix(seed xor first 8 bytes of sha256(name), little-endian);
    h_j = mix(key + (3 i + j + 1) * G) for j = 0..2; z = (sum of the twelve 16-bit fields of
    the h_j - 6 * 65535) / 65536; value = float32(z * std) (+ 1), mix being splitmix64's
    finaliser and G its increment.  Returns float32."""
    G, M1, M2 = np.uint64(0x9E3779B97F4A7C15), np.uint64(0xBF58476D1CE4E5B9), np.uint64(0x94D049BB133111EB)

    def mix(x):
        x = x + G
        x = (x ^ (x >> np.uint64(30))) * M1
        x = (x ^ (x >> np.uint64(27))) * M2
        return x ^ (x >> np.uint64(31))

    with np.errstate(over="ignore"):
        start = (int(seed) % (1 << 64)) ^ int.from_bytes(hashlib.sha256(name.encode()).digest()[:8], "little")
        key = mix(np.array([start], dtype=np.uint64))[0]
        count = int(np.prod(shape)) if len(shape) else 1
        i = np.arange(count, dtype=np.uint64)
        total = np.zeros(count, dtype=np.int64)
        for j in (1, 2, 3):
            h = mix(key + (i * np.uint64(3) + np.uint64(j)) * G)
            for shift in (0, 16, 32, 48):
                total += ((h >> np.uint64(shift)) & np.uint64(0xFFFF)).astype(np.int64)
    z = ((total - 6 * 65535).astype(np.float32) / np.float32(65536.0)) * np.float32(std)
    if plus_one:
        z = z + np.float32(1.0)
    return z.astype(np.float32).reshape(shape)
