"""Sodonex: a decoder-only language model whose config.json lists its layers
one by one. A layer is

    x <- x + m * norm1(mixer(shift(x)))        x <- x + m * norm2(ff(x))

with the norm on the sublayer's OUTPUT only (RMS norm with a single gain for
all coordinates) and ``m`` a model-wide residual multiplier. The mixer's input
is token-shifted (a learned per-coordinate blend with the previous token's
row). The mixer is attention without softmax:

* q and k projections with biases, each followed by a short causal
  convolution per channel, then one RMS norm over the whole projection, then
  rotate-half rotary positions on the first ``rot.dims`` entries of each head;
* no value projection: the value vectors are the convolved keys, taken before
  their norm and rotation;
* a query sees the earlier keys of its own chunk of ``mask.size`` positions;
  a visible key weighs sigmoid(q . k * scale + bias_h), and the weights are
  used as they are, without dividing by their sum;
* each head's output is multiplied by sigmoid of a per-head gate projection of
  the mixer's input before the output projection (with bias).

The feed-forward is a mixture of experts: the ``top`` largest router logits
(f32, with bias) choose the experts, weighed by the softmax over the chosen
logits; an expert is down(relu(up x)^2).

MI355X layout, in the manner of the other decoders: a flat [T, width] token
batch (prompt portions beside decode tokens), an f32 residual stream updated
inside the norm launch, q | k | gate as ONE projection GEMM, the K / V pages on
the shared block pool, and the per-sequence rows (previous mixer input,
convolution tails) in f32 state slots. Plain GEMMs go to the vendor library;
everything around them is this repository's HIP (``ops/seqmix.py``).
"""
from __future__ import annotations

import torch

from .. import ops
from ..ops import seqmix
from .configs import SodonexConfig


class SodonexWeights:
    """Device weights in the fused layouts, from a state dict in checkpoint
    naming (``embed``, ``l<i>.norm1|norm2|shift``, ``l<i>.mix.*``,
    ``l<i>.mlp.*``, ``final.norm``, ``head``)."""

    def __init__(self, cfg: SodonexConfig, sd: dict, device, dtype=torch.bfloat16,
                 max_positions: int = 8192):
        self.cfg, self.dtype, self.device = cfg, dtype, torch.device(device)
        self.max_positions = max_positions
        dev = self.device

        def W(name):            # a projection matrix in the activation dtype
            return sd[name].to(dev, dtype).contiguous()

        def F(name):            # small vectors the f32 paths read
            return sd[name].to(dev, torch.float32).contiguous()

        def S(name):            # a single number
            return float(sd[name].float().reshape(-1)[0])

        d = cfg.d_model
        self.embed = sd["embed"].to(dev, torch.float32).contiguous()
        if self.embed.shape != (cfg.vocab_size, d):
            raise ValueError("embed does not match vocab x width")
        self.head = sd["head"].to(dev, torch.float32).contiguous()
        self.final_norm = S("final.norm")
        self._tables: dict[tuple, torch.Tensor] = {}
        self.layers: list[dict] = []
        for i, lc in enumerate(cfg.layers):
            p, m = f"l{i}.", lc.mixer
            H, G, D = m.heads, m.kv_heads, m.dim
            L: dict = {"norm1": S(p + "norm1"), "shift": F(p + "shift")}
            wq, wk, wg = W(p + "mix.q"), W(p + "mix.k"), W(p + "mix.g")
            if wq.shape != (H * D, d) or wk.shape != (G * D, d) or wg.shape != (H, d):
                raise ValueError(f"layer {i}: projection shapes do not match the config")
            # q | k | gate rows as one GEMM (the gate has no bias); zero rows pad
            # the output to a multiple of 8 columns so that its rows stay
            # 16-byte aligned for the kernels that read them
            pad = -H % 8
            L["wqkg"] = torch.cat([wq, wk, wg, torch.zeros(pad, d, dtype=dtype, device=dev)]
                                  ).contiguous()
            L["bqkg"] = torch.cat([W(p + "mix.q.b"), W(p + "mix.k.b"),
                                   torch.zeros(H + pad, dtype=dtype, device=dev)]).contiguous()
            conv = torch.cat([F(p + "mix.q.conv"), F(p + "mix.k.conv")])
            if conv.shape != ((H + G) * D, m.taps):
                raise ValueError(f"layer {i}: convolution weights do not match the config")
            L["conv"] = conv.t().contiguous()                 # tap-major [taps, C]
            L["q_norm"], L["k_norm"] = F(p + "mix.q.norm"), F(p + "mix.k.norm")
            L["pb"] = F(p + "mix.pb")
            L["wo"], L["bo"] = W(p + "mix.o"), W(p + "mix.o.b")
            if L["wo"].shape != (d, H * m.vdim):
                raise ValueError(f"layer {i}: output projection does not match the config")
            L["cos_sin"] = self._table(m.rot)
            f = lc.mlp
            if f is not None:
                L["norm2"] = S(p + "norm2")
                L["router"], L["router_b"] = F(p + "mlp.router"), F(p + "mlp.router.b")
                if L["router"].shape != (f.experts, d):
                    raise ValueError(f"layer {i}: router does not match the config")
                L["e_up"] = torch.stack([W(f"{p}mlp.e{e}.up") for e in range(f.experts)]).contiguous()
                L["e_down"] = torch.stack([W(f"{p}mlp.e{e}.down")
                                           for e in range(f.experts)]).contiguous()
                if L["e_up"].shape != (f.experts, f.ff, d):
                    raise ValueError(f"layer {i}: expert shapes do not match the config")
            self.layers.append(L)

    def _table(self, rot) -> torch.Tensor:
        key = (rot.dims, rot.base)
        if key not in self._tables:
            self._tables[key] = seqmix.rope_table_half(rot.dims, self.max_positions, rot.base,
                                                       self.device)
        return self._tables[key]

    @classmethod
    def random(cls, cfg: SodonexConfig, device, seed: int = 0, dtype=torch.bfloat16,
               max_positions: int = 8192) -> "SodonexWeights":
        return cls(cfg, random_state_dict(cfg, seed), device, dtype, max_positions)


def random_state_dict(cfg: SodonexConfig, seed: int = 0) -> dict:
    """Seeded random weights in checkpoint naming (bf16), scaled so that
    activations stay O(1) through the stack; used by tests, smoke and bench."""
    g = torch.Generator().manual_seed(seed)
    d = cfg.d_model
    sd: dict = {}

    def mat(name, rows, cols, gain=1.0):
        sd[name] = (torch.randn(rows, cols, generator=g) * gain / cols ** 0.5).to(torch.bfloat16)

    def vec(name, n, mean=0.0, std=0.1):
        sd[name] = (mean + torch.randn(n, generator=g) * std).to(torch.bfloat16)

    def one(name):
        sd[name] = torch.tensor(1.0 + 0.1 * torch.randn((), generator=g).item(),
                                dtype=torch.bfloat16)

    sd["embed"] = (torch.randn(cfg.vocab_size, d, generator=g) / d ** 0.5).to(torch.bfloat16)
    for i, lc in enumerate(cfg.layers):
        p, m = f"l{i}.", lc.mixer
        H, G, D = m.heads, m.kv_heads, m.dim
        one(p + "norm1")
        vec(p + "shift", d, 0.4, 0.2)
        mat(p + "mix.q", H * D, d, 2.0); vec(p + "mix.q.b", H * D)
        mat(p + "mix.k", G * D, d, 2.0); vec(p + "mix.k.b", G * D)
        sd[p + "mix.q.conv"] = (torch.randn(H * D, m.taps, generator=g) * 0.5).to(torch.bfloat16)
        sd[p + "mix.k.conv"] = (torch.randn(G * D, m.taps, generator=g) * 0.5).to(torch.bfloat16)
        vec(p + "mix.q.norm", H * D, 1.0); vec(p + "mix.k.norm", G * D, 1.0)
        vec(p + "mix.pb", H, -1.0, 0.5)
        mat(p + "mix.g", H, d, 2.0)
        mat(p + "mix.o", d, H * m.vdim, 2.0); vec(p + "mix.o.b", d)
        f = lc.mlp
        if f is None:
            continue
        one(p + "norm2")
        for e in range(f.experts):
            mat(f"{p}mlp.e{e}.up", f.ff, d, 2.0)
            mat(f"{p}mlp.e{e}.down", d, f.ff, 2.0)
        mat(p + "mlp.router", f.experts, d, 3.0)
        vec(p + "mlp.router.b", f.experts, 0.0, 0.2)
    one("final.norm")
    mat("head", cfg.vocab_size, d, 2.0)
    return sd


def config_to_json(cfg: SodonexConfig) -> dict:
    """The config.json of ``cfg`` (the inverse of ``sodonex_config_from_json``)."""
    layers = []
    for lc in cfg.layers:
        m, f = lc.mixer, lc.mlp
        mx = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
              "conv": m.taps, "mask": {"size": m.chunk}, "scale": m.scale,
              "rot": {"dims": m.rot.dims, "base": m.rot.base}}
        mlp = None if f is None else {"kind": "moe", "expert": {"ff": f.ff},
                                      "router": {"experts": f.experts, "top": f.top}}
        layers.append({"type": lc.kind, "mixer": mx, "mlp": mlp})
    return {"architecture": "Sodonex", "vocab": cfg.vocab_size, "width": cfg.d_model,
            "norm": {"eps": cfg.norm_eps}, "residual_mult": cfg.residual_mult,
            "embedding": {"scale": cfg.embed_scale}, "layers": layers}


class SodonexModel:
    """The step function: one pass of a flat token batch through all layers,
    reading and extending the paged K / V cache and the row-state slots."""

    hybrid = True

    def __init__(self, w: SodonexWeights):
        self.w, self.cfg = w, w.cfg

    # the cache manager sizes its storage from this
    def cache_spec(self) -> dict:
        kv, rows = {}, {}
        d = self.cfg.d_model
        for i, lc in enumerate(self.cfg.layers):
            m = lc.mixer
            kv[i] = (m.kv_heads * m.dim, m.kv_heads * m.vdim)
            # the previous mixer input, and the last taps - 1 projected q | k rows
            rows[i] = {"prev": (d,), "tail": (m.taps - 1, (m.heads + m.kv_heads) * m.dim)}
        return {"latent": {}, "state": {}, "kv": kv, "rows": rows}

    def embed(self, tokens: torch.Tensor) -> torch.Tensor:
        x = torch.nn.functional.embedding(tokens.long(), self.w.embed)
        return x * self.cfg.embed_scale

    def forward(self, meta, cache, trail: list | None = None) -> torch.Tensor:
        """f32 logits [len(meta.logit_idx), vocab] of one step. ``meta``: the
        engine's StepMeta; ``cache``: a HybridCache. ``trail`` collects the
        residual stream after every layer (tests)."""
        w, cfg, dt = self.w, self.cfg, self.w.dtype
        x = self.embed(meta.tokens).contiguous()
        T = x.shape[0]
        eps, mult = cfg.norm_eps, cfg.residual_mult
        for i, (lc, L) in enumerate(zip(cfg.layers, w.layers)):
            m, st = lc.mixer, cache.rows[i]
            H, G, D = m.heads, m.kv_heads, m.dim
            h = seqmix.token_shift(x, L["shift"], st["prev"], meta.state_slots, meta.cu_q,
                                   meta.positions, dt)
            u = ops.linear(h, L["wqkg"], L["bqkg"])
            kc, vc = cache.kv[i]
            q = seqmix.conv_norm_rope_append(u, L["conv"], st["tail"], meta.state_slots, meta.cu_q,
                                             meta.positions, L["q_norm"], L["k_norm"], eps,
                                             L["cos_sin"], m.rot.dims, H, G, D, kc, vc, meta.slots,
                                             dt)
            # every reader of this step's row state is done: store the new rows
            seqmix.seq_state_save(x, u, st["prev"], st["tail"], meta.state_slots, meta.cu_q,
                                  meta.positions)
            o = seqmix.sigmoid_attention(q, kc, vc, meta.cu_q, meta.ctx_lens, meta.block_tables,
                                         meta.positions, L["pb"],
                                         u[:, (H + G) * D:(H + G) * D + H], m.scale,
                                         m.chunk, H, G, D, meta.max_q)
            y = ops.linear(o, L["wo"], L["bo"])
            f = lc.mlp
            xa = seqmix.scalar_rms_add(x, y, L["norm1"], eps, mult, dt if f is not None else None)
            if f is not None:
                y = self._moe(f, L, xa)
                seqmix.scalar_rms_add(x, y, L["norm2"], eps, mult, None)
            if trail is not None:
                trail.append(x.clone())
        hf = seqmix.scalar_rms_norm(x, w.final_norm, eps, row_idx=meta.logit_idx)
        return ops.linear(hf, w.head)

    @staticmethod
    def _moe(f, L, h) -> torch.Tensor:
        z = ops.linear(h.float(), L["router"])
        idx, wt = seqmix.moe_route(z, None, 1, 1, f.top, bias=L["router_b"], top_softmax=True)
        return seqmix.moe_experts(h, idx, wt, L["e_up"], L["e_down"], gated=False)
