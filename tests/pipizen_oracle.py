"""A plain, slow float64 implementation of the Pipizen design, one function per
mechanism, written from the design's equations. It shares no code with the
product path (``loqa_hub_amd``): it is what the tests compare the framework to.

Notation: x is the residual stream [T, width]; every sequence is processed
alone, token by token where a recurrence or a cache is involved.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def _w(sd, name):
    return sd[name].to(F64)


def dyt(x, sd, name):
    """Dynamic Tanh: tanh(alpha x) * w + b (no mean, no variance)."""
    return torch.tanh(_w(sd, name + ".alpha") * x) * _w(sd, name) + _w(sd, name + ".b")


def rms_unit(x, weight, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def rotary_angles(rot: dict, positions: torch.Tensor):
    """(cos, sin) [T, dims/2] with the YaRN frequency blend and magnitude."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def dim_of(t):
            return dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(base))
        lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
        hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    a = positions.to(F64)[:, None] * f[None, :]
    return torch.cos(a) * mag, torch.sin(a) * mag


def rotate_pairs(x, cos, sin, dims):
    """x [T, ..., n]: the first ``dims`` entries rotate as (2i, 2i+1) pairs."""
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    while cos.dim() < u.dim():
        cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def latent_kv(h, sd, pre, m, eps, positions):
    """The cached pair of a latent-attention layer: (c [T, rank], k_rot [T, rot_dim])."""
    R, Dr = m["kv_rank"], m["rot_dim"]
    z = h @ _w(sd, pre + "dkv").T
    c = rms_unit(z[:, :R], _w(sd, pre + "dkv.norm"), eps)
    cos, sin = rotary_angles(m["rot"], positions)
    kr = rotate_pairs(z[:, R:R + Dr], cos, sin, int(m["rot"]["dims"]))
    return c, kr


def latent_attention(h, sd, pre, m, positions, c, kr):
    """Causal softmax attention with a sink over the latent cache (c, kr) of
    the same sequence; h [T, width] are the queries' inputs at ``positions``
    and row j of the cache is position j."""
    H, D, Dr, Dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ _w(sd, pre + "q").T).view(T, H, D + Dr)
    cos, sin = rotary_angles(m["rot"], positions)
    q_rot = rotate_pairs(q[..., D:], cos, sin, int(m["rot"]["dims"]))
    k_un = (c @ _w(sd, pre + "uk").T).view(-1, H, D)
    val = (c @ _w(sd, pre + "uv").T).view(-1, H, Dv)
    sink = _w(sd, pre + "sink")
    out = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        n = int(positions[t]) + 1
        for hh in range(H):
            s = (k_un[:n, hh] @ q[t, hh, :D] + kr[:n] @ q_rot[t, hh]) * float(m["scale"])
            mx = torch.maximum(s.max(), sink[hh])
            e = torch.exp(s - mx)
            den = e.sum() + torch.exp(sink[hh] - mx)
            out[t, hh] = (e / den) @ val[:n, hh]
    return out.reshape(T, H * Dv) @ _w(sd, pre + "o").T


def lightning(h, sd, pre, m, eps, state=None):
    """Linear attention with a per-head decay; returns (y, state)."""
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(h @ _w(sd, pre + "q").T).view(T, H, D)
    k = silu(h @ _w(sd, pre + "k").T).view(T, H, D)
    v = silu(h @ _w(sd, pre + "v").T).view(T, H, Dv)
    decay = torch.tensor(m["decay"], dtype=F64)
    S = torch.zeros(H, D, Dv, dtype=F64) if state is None else state.clone()
    o = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hde,hd->he", S, q[t])
    y = rms_unit(o.reshape(T, H * Dv), _w(sd, pre + "norm"), eps)
    y = y * torch.sigmoid(h @ _w(sd, pre + "g").T)
    return y @ _w(sd, pre + "o").T, S


def gated_ff(h, sd, pre):
    return (silu(h @ _w(sd, pre + "gate").T) * (h @ _w(sd, pre + "up").T)) @ _w(sd, pre + "down").T


def route(h, sd, pre, r):
    """Chosen experts and their weights, per token: lists of (index, weight)."""
    E, n_id, top = r["experts"], r.get("identity", 0), r["top"]
    s = torch.softmax(h @ _w(sd, pre + "router").T, dim=-1)
    choice = s + _w(sd, pre + "correction") if (pre + "correction") in sd else s.clone()
    g = r.get("groups")
    if g:
        per = (E + n_id) // g["count"]
        gs = choice.view(-1, g["count"], per).max(-1).values
        keep = gs.topk(g["keep"], dim=-1).indices
        allowed = torch.zeros_like(gs, dtype=torch.bool).scatter_(1, keep, True)
        choice = choice.masked_fill(~allowed.repeat_interleave(per, dim=1), -math.inf)
    idx = choice.topk(top, dim=-1).indices
    return idx, s.gather(1, idx)


def moe(h, sd, pre, mlp):
    r = mlp["router"]
    E = r["experts"]
    idx, wt = route(h, sd, pre, r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wt[t]):
            if e >= E:
                out[t] += w * h[t]
            else:
                out[t] += w * gated_ff(h[t:t + 1], sd, f"{pre}e{e}.")[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, sd, pre + "shared.")
    return out


def forward(cfg: dict, sd: dict, tokens: list[int], return_layers: bool = False):
    """Logits [T, vocab] of one whole sequence (float64)."""
    eps = float(cfg["norm"]["eps"])
    T = len(tokens)
    pos = torch.arange(T)
    x = _w(sd, "embed")[torch.tensor(tokens)]
    caches: dict[int, tuple] = {}
    layers = []
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = dyt(x, sd, p + "norm1")
        if L["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                caches[i] = latent_kv(h, sd, p + "mix.", m, eps, pos)
                src = i
            y = latent_attention(h, sd, p + "mix.", m, pos, *caches[src])
        elif L["type"] == "lightning":
            y, _ = lightning(h, sd, p + "mix.", m, eps)
        else:
            raise ValueError(L["type"])
        x = x + dyt(y, sd, p + "norm1b")
        if L.get("mlp"):
            h = dyt(x, sd, p + "norm2")
            y = gated_ff(h, sd, p + "mlp.") if L["mlp"]["kind"] == "dense" else \
                moe(h, sd, p + "mlp.", L["mlp"])
            x = x + dyt(y, sd, p + "norm2b")
        layers.append(x.clone())
    logits = dyt(x, sd, "final.norm") @ _w(sd, "head").T
    return (logits, torch.stack(layers)) if return_layers else logits


# --------------------------------------------------------------------------
# Test fixtures: small configurations (config.json form) and seeded weights in
# checkpoint naming, made here so that the tests do not lean on the product's
# own generators.
def latent(heads=3, dim=16, rot_dim=8, vdim=12, kv_rank=24, *, dims=None, scaling=True,
           kv_from=None, base=10000.0, scale=None):
    rot = {"base": base, "dims": rot_dim if dims is None else dims}
    if scaling:
        rot["scaling"] = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "rot": rot, "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def lightning_layer(heads=2, dim=16, vdim=24, decay=None):
    decay = decay or [0.5 + 0.49 * i / max(1, heads - 1) for i in range(heads)]
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def moe_ff(experts=6, identity=2, top=2, count=4, keep=2, ff=24, shared=40):
    f = {"kind": "moe", "expert": {"ff": ff},
         "router": {"experts": experts, "identity": identity, "top": top,
                    "groups": {"count": count, "keep": keep}}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def make_config(layers, width=48, vocab=120, eps=1e-5):
    out = []
    for mixer, mlp in layers:
        L = dict(mixer)
        L["mlp"] = mlp
        out.append(L)
    return {"architecture": "Pipizen", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "layers": out}


def make_weights(cfg: dict, seed: int = 0) -> dict:
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]
    sd = {}

    def mat(name, rows, cols, gain=1.5):
        sd[name] = (torch.randn(rows, cols, generator=g) * gain / cols ** 0.5).to(torch.bfloat16)

    def vec(name, n, mean, std):
        sd[name] = (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    def norm(name):
        vec(name, d, 1.0, 0.2)
        vec(name + ".b", d, 0.0, 0.1)
        sd[name + ".alpha"] = torch.tensor(0.4 + 0.8 * float(torch.rand((), generator=g)),
                                           dtype=torch.bfloat16)

    sd["embed"] = torch.randn(cfg["vocab"], d, generator=g).to(torch.bfloat16)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        norm(p + "norm1"); norm(p + "norm1b")
        if L["type"] == "latent_attention":
            mat(p + "mix.q", m["heads"] * (m["dim"] + m["rot_dim"]), d, 3.0)
            if m.get("kv_from") is None:
                mat(p + "mix.dkv", m["kv_rank"] + m["rot_dim"], d, 3.0)
                vec(p + "mix.dkv.norm", m["kv_rank"], 1.0, 0.2)
            mat(p + "mix.uk", m["heads"] * m["dim"], m["kv_rank"], 2.0)
            mat(p + "mix.uv", m["heads"] * m["vdim"], m["kv_rank"], 2.0)
            vec(p + "mix.sink", m["heads"], 1.0, 1.0)
            mat(p + "mix.o", d, m["heads"] * m["vdim"], 2.0)
        else:
            mat(p + "mix.q", m["heads"] * m["dim"], d)
            mat(p + "mix.k", m["heads"] * m["dim"], d)
            mat(p + "mix.v", m["heads"] * m["vdim"], d, 2.0)
            mat(p + "mix.g", m["heads"] * m["vdim"], d)
            vec(p + "mix.norm", m["heads"] * m["vdim"], 1.0, 0.2)
            mat(p + "mix.o", d, m["heads"] * m["vdim"], 2.0)
        f = L.get("mlp")
        if not f:
            continue
        norm(p + "norm2"); norm(p + "norm2b")
        if f["kind"] == "dense":
            mat(p + "mlp.gate", f["ff"], d, 2.0); mat(p + "mlp.up", f["ff"], d, 2.0)
            mat(p + "mlp.down", d, f["ff"], 2.0)
        else:
            r = f["router"]
            n = r["experts"] + r.get("identity", 0)
            for e in range(r["experts"]):
                mat(f"{p}mlp.e{e}.gate", f["expert"]["ff"], d, 2.0)
                mat(f"{p}mlp.e{e}.up", f["expert"]["ff"], d, 2.0)
                mat(f"{p}mlp.e{e}.down", d, f["expert"]["ff"], 4.0)
            mat(p + "mlp.router", n, d, 4.0)
            # corrections large enough to change choices, some of them negative
            vec(p + "mlp.correction", n, -0.05, 0.15)
            if f.get("shared"):
                mat(p + "mlp.shared.gate", f["shared"]["ff"], d, 2.0)
                mat(p + "mlp.shared.up", f["shared"]["ff"], d, 2.0)
                mat(p + "mlp.shared.down", d, f["shared"]["ff"], 2.0)
    norm("final.norm")
    mat("head", cfg["vocab"], d, 2.0)
    return sd
