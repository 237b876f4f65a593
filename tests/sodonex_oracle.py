"""A plain float64 implementation of the Sodonex design, written from its
equations: one function per mechanism, whole sequences only (no cache, no
state, no batching), no code shared with the framework. The tests compare the
framework's step function, cache and kernels with it.

Notation: T tokens, d the model width, H query heads, G key/value heads,
D the per-head query/key size; weights are [out, in] and applied as W x.
"""
import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------ mechanisms
def rms(x, eps):
    """x over the root of (its mean square + eps), along the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose gain is one number for all coordinates."""
    return rms(x, eps) * g


def token_shift(h, mu):
    """h_t + (h_{t-1} - h_t) * mu per coordinate; the token before the first is zero."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]])
    return h + (prev - h) * mu


def short_conv(u, w):
    """Causal per-channel convolution: y_t = sum_j w[:, j] u_{t - taps + 1 + j},
    zeros before the start. u [T, C], w [C, taps]."""
    T, taps = u.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u])
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + pad[j:j + T] * w[:, j]
    return y


def rotate_half(x, dims, base):
    """x [T, heads, D]: in every head entry i < dims/2 pairs with entry
    i + dims/2 and the pair turns by position * base^(-2i/dims); entries from
    ``dims`` on pass through."""
    T = x.shape[0]
    half = dims // 2
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = torch.arange(T, dtype=F64)[:, None] * f[None, :]
    c, s = a.cos()[:, None, :], a.sin()[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def chunk_sigmoid_attention(q, k, v, scale, pb, chunk):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv]. Query i sees key
    j <= i of its own chunk (i // chunk == j // chunk); a visible key weighs
    sigmoid(score + pb[h]) and the weights are not normalised."""
    T, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    i = torch.arange(T)
    seen = (i[None, :] <= i[:, None]) & ((i[None, :] // chunk) == (i[:, None] // chunk))
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // rep
        s = q[:, h] @ k[:, g].T * scale + pb[h]
        w = torch.sigmoid(s) * seen
        out[:, h] = w @ v[:, g]
    return out


def attention_mixer(h, sd, p, m, eps):
    """The whole mixer on its (token-shifted) input h [T, d]."""
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    W = lambda n: sd[p + n].to(F64)
    q = h @ W("q").T + W("q.b")
    k = h @ W("k").T + W("k.b")
    q, k = short_conv(q, W("q.conv")), short_conv(k, W("k.conv"))
    v = k.view(T, G, D)                               # the values: keys after the convolution
    q = (rms(q, eps) * W("q.norm")).view(T, H, D)     # one norm over the whole projection
    k = (rms(k, eps) * W("k.norm")).view(T, G, D)
    r = m["rot"]
    q, k = rotate_half(q, r["dims"], r["base"]), rotate_half(k, r["dims"], r["base"])
    o = chunk_sigmoid_attention(q, k, v, m["scale"], W("pb"), m["mask"]["size"])
    gate = torch.sigmoid(h @ W("g").T)                # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, -1) @ W("o").T + W("o.b")


def route(h, sd, p, f):
    """Top experts by router logit; weights = softmax over the chosen logits."""
    z = h @ sd[p + "router"].to(F64).T + sd[p + "router.b"].to(F64)
    top = z.topk(f["router"]["top"], dim=-1)
    return top.indices, torch.softmax(top.values, dim=-1)


def moe(h, sd, p, f):
    idx, wt = route(h, sd, p, f)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wt[t]):
            up = sd[f"{p}e{e}.up"].to(F64) @ h[t]
            out[t] += w * (sd[f"{p}e{e}.down"].to(F64) @ torch.relu(up).pow(2))
    return out


def forward(cfg, sd, toks, layers_out=False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after
    every layer when asked)."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = sd["embed"].to(F64)[torch.tensor(toks)] * cfg["embedding"]["scale"]
    trail = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        assert L["type"] == "attention"
        h = token_shift(x, sd[p + "shift"].to(F64))
        y = attention_mixer(h, sd, p + "mix.", L["mixer"], eps)
        x = x + mult * scalar_norm(y, sd[p + "norm1"].to(F64), eps)
        if L.get("mlp"):
            y = moe(x, sd, p + "mlp.", L["mlp"])
            x = x + mult * scalar_norm(y, sd[p + "norm2"].to(F64), eps)
        trail.append(x)
    logits = scalar_norm(x, sd["final.norm"].to(F64), eps) @ sd["head"].to(F64).T
    return (logits, torch.stack(trail)) if layers_out else logits


# -------------------------------------------------- small configurations / weights
def attn(heads=4, kv_heads=2, dim=16, taps=4, chunk=8, dims=8, base=10000.0, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "conv": taps,
            "mask": {"size": chunk}, "rot": {"dims": dims, "base": base},
            "scale": dim ** -0.5 if scale is None else scale}


def moe_ff(experts=6, top=2, ff=24):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def make_config(layers, width=48, vocab=120, eps=1e-5, mult=0.4, embed_scale=3.0):
    return {"architecture": "Sodonex", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "residual_mult": mult, "embedding": {"scale": embed_scale},
            "layers": [{"type": "attention", "mixer": m, "mlp": f} for m, f in layers]}


def make_weights(cfg, seed=0):
    """Seeded bf16 weights in checkpoint naming."""
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]
    sd = {}

    def mat(name, rows, cols, gain=1.0):
        sd[name] = (torch.randn(rows, cols, generator=g) * gain / math.sqrt(cols)).to(torch.bfloat16)

    def vec(name, n, mean=0.0, std=0.1):
        sd[name] = (mean + torch.randn(n, generator=g) * std).to(torch.bfloat16)

    def one(name, mean=1.0, std=0.1):
        sd[name] = torch.tensor(mean + std * torch.randn((), generator=g).item(),
                                dtype=torch.bfloat16)

    sd["embed"] = (torch.randn(cfg["vocab"], d, generator=g) / math.sqrt(d)).to(torch.bfloat16)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, D = m["heads"], m["kv_heads"], m["dim"]
        one(p + "norm1")
        vec(p + "shift", d, 0.4, 0.25)
        mat(p + "mix.q", H * D, d, 2.0); vec(p + "mix.q.b", H * D)
        mat(p + "mix.k", G * D, d, 2.0); vec(p + "mix.k.b", G * D)
        sd[p + "mix.q.conv"] = (torch.randn(H * D, m["conv"], generator=g) * 0.5).to(torch.bfloat16)
        sd[p + "mix.k.conv"] = (torch.randn(G * D, m["conv"], generator=g) * 0.5).to(torch.bfloat16)
        vec(p + "mix.q.norm", H * D, 1.0); vec(p + "mix.k.norm", G * D, 1.0)
        vec(p + "mix.pb", H, -1.0, 0.5)
        mat(p + "mix.g", H, d, 2.0)
        mat(p + "mix.o", d, H * D, 2.0); vec(p + "mix.o.b", d)
        f = L.get("mlp")
        if f:
            one(p + "norm2")
            for e in range(f["router"]["experts"]):
                mat(f"{p}mlp.e{e}.up", f["expert"]["ff"], d, 2.0)
                mat(f"{p}mlp.e{e}.down", d, f["expert"]["ff"], 2.0)
            mat(p + "mlp.router", f["router"]["experts"], d, 4.0)
            vec(p + "mlp.router.b", f["router"]["experts"], 0.0, 0.3)
    one("final.norm")
    mat("head", cfg["vocab"], d, 2.0)
    return sd
