"""Entry points of the sequence-mixer ops of the hybrid decoders: Dynamic-Tanh
norm, latent (compressed-KV) attention with a softmax sink over a paged latent
cache, decayed linear attention with a carried per-sequence state, and the
grouped top-k expert router with its expert feed-forward.

As everywhere in ``ops``: GPU tensors run the HIP kernels
(``csrc/kernels/norm_dyt.hip``, ``attn_latent.hip``, ``lightning.hip``,
``moe.hip``), CPU tensors the f32 PyTorch references (the CPU test tier and the
numerics oracle of the GPU tests). Activations are bfloat16 or float32
(``_DT``); the residual stream, scores, softmax, recurrent state, router and
norm statistics are f32 in both.
"""
from __future__ import annotations

import torch

from . import reference as ref
from ._lib import check, kernels, ptr, stream_ptr

_DT = {torch.bfloat16: 0, torch.float32: 1}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"activation dtype {t.dtype} is not supported") from None


def _f32c(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise TypeError(f"{name} must be contiguous float32")


def _i32c(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise TypeError(f"{name} must be contiguous int32")


class DytParams:
    """One Dynamic-Tanh norm: f32 weight and bias vectors and the scalar alpha."""
    __slots__ = ("w", "b", "alpha")

    def __init__(self, w: torch.Tensor, b: torch.Tensor, alpha: float):
        self.w, self.b, self.alpha = w.float().contiguous(), b.float().contiguous(), float(alpha)

    def tup(self):
        return self.w, self.b, self.alpha


def dyt_norm(x: torch.Tensor, p: DytParams, out_dtype, row_idx: torch.Tensor | None = None
             ) -> torch.Tensor:
    """y = tanh(alpha x) * w + b over rows of x [rows, d] (f32 or an activation
    dtype); ``row_idx`` (int64) gathers rows in the same launch."""
    if not x.is_cuda:
        return ref.dyt_norm(x, p.w, p.b, p.alpha, out_dtype, row_idx)
    assert x.dim() == 2 and x.is_contiguous()
    d = x.shape[1]
    rows = x.shape[0] if row_idx is None else row_idx.numel()
    if row_idx is not None:
        assert row_idx.dtype == torch.int64 and row_idx.is_contiguous()
    assert p.w.numel() == d and p.b.numel() == d
    y = torch.empty(rows, d, dtype=out_dtype, device=x.device)
    if rows:
        check(kernels().loqa_dyt_norm(ptr(x), _dt(x), ptr(row_idx), ptr(p.w), ptr(p.b), p.alpha,
                                      ptr(y), _dt(y), rows, d, stream_ptr(x)), "dyt_norm")
    return y


def dyt_add_norm(resid: torch.Tensor, y: torch.Tensor, post: DytParams,
                 nxt: DytParams | None, out_dtype) -> torch.Tensor | None:
    """The fused residual step: resid (f32, in place) += dyt(y; post), and in
    the same launch h = dyt(resid; nxt) for the next sublayer (None: no h)."""
    if not resid.is_cuda:
        return ref.dyt_add_norm(resid, y, post.tup(), None if nxt is None else nxt.tup(), out_dtype)
    _f32c(resid, "resid")
    assert y.shape == resid.shape and y.is_contiguous()
    rows, d = resid.shape
    h = torch.empty(rows, d, dtype=out_dtype, device=resid.device) if nxt is not None else None
    if rows:
        check(kernels().loqa_dyt_add_norm(
            ptr(resid), ptr(y), _dt(y), ptr(post.w), ptr(post.b), post.alpha,
            ptr(nxt.w) if nxt else None, ptr(nxt.b) if nxt else None, nxt.alpha if nxt else 0.0,
            ptr(h), _dt(h) if h is not None else 0, rows, d, stream_ptr(resid)), "dyt_add_norm")
    return h


def rope_table_pairs(dims: int, max_pos: int, base: float, yarn: tuple | None = None,
                     device=None) -> torch.Tensor:
    """(cos, sin) table of the interleaved rotary layout, optionally YaRN-scaled
    (see :func:`reference.rope_table_pairs`); built once at load time."""
    return ref.rope_table_pairs(dims, max_pos, base, yarn, device)


def latent_append(z: torch.Tensor, norm_w: torch.Tensor, eps: float, positions: torch.Tensor,
                  cos_sin: torch.Tensor, cache: torch.Tensor, slots: torch.Tensor, R: int,
                  dims: int) -> None:
    """RMS-norm the latent part of z [T, R + Dr], rotate its rotary key part and
    store both in the paged latent cache [blocks, BLK, R + Dr] (one launch)."""
    if not z.is_cuda:
        return ref.latent_append(z, norm_w, eps, positions, cos_sin, cache, slots, R, dims)
    T, W = z.shape
    assert z.stride(1) == 1 and cache.is_contiguous() and cache.dtype == z.dtype
    assert cache.shape[2] == W and 0 < R <= W and dims % 2 == 0 and dims <= W - R
    _f32c(norm_w, "norm_w"); _f32c(cos_sin, "cos_sin"); _i32c(positions, "positions")
    _i32c(slots, "slots")
    assert norm_w.numel() == R and cos_sin.shape[1] * 2 == dims
    assert positions.numel() >= T and slots.numel() >= T
    if T:
        check(kernels().loqa_latent_append(
            ptr(z), _dt(z), z.stride(0), ptr(norm_w), eps, ptr(positions), ptr(cos_sin),
            cos_sin.shape[0], ptr(cache), cache.shape[1], cache.shape[0], ptr(slots), T, R, W - R,
            dims, stream_ptr(z)), "latent_append")


def latent_attention(qa: torch.Tensor, qr: torch.Tensor, cache: torch.Tensor, cu_q: torch.Tensor,
                     ctx_lens: torch.Tensor, block_tables: torch.Tensor, positions: torch.Tensor,
                     cos_sin: torch.Tensor, sink: torch.Tensor | None, scale: float, R: int,
                     dims: int, max_ctx: int = 0, out: torch.Tensor | None = None) -> torch.Tensor:
    """Causal attention over the paged latent cache, all heads sharing each
    cached row: score = (qa . c + rot(qr) . k_rot) * scale; softmax with
    ``sink`` [H] (f32, optional) in the denominator; out = sum_j p_j c_j.
    qa [H, T, R] (queries already folded into latent space), qr [T, H, Dr]
    (unrotated; may be a strided view), out [H, T, R]."""
    H, T, _ = qa.shape
    if out is None:
        out = torch.empty(H, T, R, dtype=qa.dtype, device=qa.device)
    if not qa.is_cuda:
        return ref.latent_attention(qa, qr, cache, cu_q, ctx_lens, block_tables, positions,
                                    cos_sin, sink, scale, R, dims, out)
    Dr = cache.shape[2] - R
    assert qa.shape[2] == R and qa.stride(2) == 1 and qr.shape == (T, H, Dr) and qr.stride(2) == 1
    assert qa.dtype == cache.dtype == qr.dtype == out.dtype and cache.is_contiguous()
    assert out.is_contiguous() and out.shape == (H, T, R)
    _i32c(cu_q, "cu_q"); _i32c(ctx_lens, "ctx_lens"); _i32c(block_tables, "block_tables")
    _i32c(positions, "positions"); _f32c(cos_sin, "cos_sin")
    if sink is not None:
        _f32c(sink, "sink")
        assert sink.numel() == H
    B = ctx_lens.numel()
    assert cu_q.numel() == B + 1 and block_tables.shape[0] == B and positions.numel() >= T
    # few query rows over a long context: split the keys over workgroups
    hg = (H + 3) // 4
    ns = 1 if T * hg >= 512 else max(1, min(32, -(-int(max_ctx) // 128), 1024 // max(1, T * hg)))
    ws = torch.empty(ns * T * H * (R + 2), dtype=torch.float32, device=qa.device) if ns > 1 else None
    if T:
        check(kernels().loqa_latent_attention(
            ptr(qa), qa.stride(1), qa.stride(0), ptr(qr), qr.stride(0), qr.stride(1), _dt(qa),
            ptr(cache), cache.shape[1], cache.shape[0], ptr(cu_q), ptr(ctx_lens), ptr(block_tables),
            block_tables.shape[1], ptr(positions), ptr(cos_sin), cos_sin.shape[0], ptr(sink),
            float(scale), B, H, T, R, Dr, dims, ptr(out), ns, ptr(ws), stream_ptr(qa)),
            "latent_attention")
    return out


PREFILL_DK = (64, 128, 192, 256)     # head sizes the matrix-core prompt kernel is built for
PREFILL_DV = (64, 128)


def prefill_head_sizes(dk: int, dv: int) -> tuple[int, int] | None:
    """The (padded) key and value head sizes of the prompt-pass kernel for a
    model's sizes, or None when it does not cover them."""
    a = next((x for x in PREFILL_DK if x >= dk), None)
    b = next((x for x in PREFILL_DV if x >= dv), None)
    return None if a is None or b is None else (a, b)


def latent_gather(cache: torch.Tensor, block_tables: torch.Tensor, cu_k: torch.Tensor,
                  total_k: int, max_ctx: int, R: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Every sequence's cached rows in position order, as contiguous latents
    [total_k, R] and rotary key parts [total_k, Dr] (bf16, GPU)."""
    assert cache.is_cuda and cache.dtype == torch.bfloat16 and cache.is_contiguous()
    _i32c(block_tables, "block_tables"); _i32c(cu_k, "cu_k")
    B, Dr = block_tables.shape[0], cache.shape[2] - R
    assert cu_k.numel() == B + 1
    cl = torch.empty(total_k, R, dtype=cache.dtype, device=cache.device)
    kr = torch.empty(total_k, Dr, dtype=cache.dtype, device=cache.device)
    check(kernels().loqa_latent_gather(ptr(cache), cache.shape[1], ptr(block_tables),
                                       block_tables.shape[1], ptr(cu_k), B, int(max_ctx), R, Dr,
                                       ptr(cl), ptr(kr), stream_ptr(cache)), "latent_gather")
    return cl, kr


def latent_kfill_(k: torch.Tensor, kr: torch.Tensor, D: int) -> None:
    """k [L, H, DK] (bf16): every head's entries D .. D + Dr take kr [L, Dr]."""
    L, H, DK = k.shape
    Dr = kr.shape[1]
    assert k.is_contiguous() and kr.is_contiguous() and kr.shape[0] == L and D + Dr <= DK
    assert k.dtype == kr.dtype == torch.bfloat16
    check(kernels().loqa_latent_kfill(ptr(k), ptr(kr), L, H, DK, D, Dr, stream_ptr(k)),
          "latent_kfill")


def rope_pairs_(x: torch.Tensor, off: int, dims: int, positions: torch.Tensor,
                cos_sin: torch.Tensor) -> None:
    """Rotate in place the interleaved pairs x[t, h, off : off + dims] (bf16)."""
    T, H, _ = x.shape
    assert x.dtype == torch.bfloat16 and x.stride(2) == 1 and off + dims <= x.shape[2]
    _i32c(positions, "positions"); _f32c(cos_sin, "cos_sin")
    assert cos_sin.shape[1] * 2 == dims and positions.numel() >= T
    check(kernels().loqa_rope_pairs(ptr(x), x.stride(0), x.stride(1), T, H, off, dims,
                                    ptr(positions), ptr(cos_sin), cos_sin.shape[0], stream_ptr(x)),
          "rope_pairs")


def latent_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_q: torch.Tensor,
                   cu_k: torch.Tensor, positions: torch.Tensor, sink: torch.Tensor | None,
                   scale: float, max_q: int) -> torch.Tensor:
    """Causal flash attention of a prompt pass on the matrix cores: q [T, H, DK]
    (rotated), k [L, H, DK], v [L, H, DV] per-head keys / values of the
    gathered contexts (``cu_k``), a query at absolute position p sees keys
    0 .. p of its sequence; ``sink`` [H] joins the softmax denominator.
    Returns [T, H * DV] (bf16)."""
    T, H, DK = q.shape
    DV = v.shape[2]
    assert q.is_cuda and q.dtype == k.dtype == v.dtype == torch.bfloat16
    assert q.stride(2) == 1 and q.stride(1) == DK and k.is_contiguous() and v.is_contiguous()
    assert k.shape[1:] == (H, DK) and v.shape[:2] == k.shape[:2]
    assert DK in PREFILL_DK and DV in PREFILL_DV
    _i32c(cu_q, "cu_q"); _i32c(cu_k, "cu_k"); _i32c(positions, "positions")
    B = cu_q.numel() - 1
    assert cu_k.numel() == B + 1
    if sink is not None:
        _f32c(sink, "sink")
    o = torch.empty(T, H * DV, dtype=q.dtype, device=q.device)
    check(kernels().loqa_latent_prefill(ptr(q), q.stride(0), ptr(k), ptr(v), ptr(o), ptr(cu_q),
                                        ptr(cu_k), ptr(positions), ptr(sink), float(scale), B, H,
                                        int(max_q), DK, DV, stream_ptr(q)), "latent_prefill")
    return o


def lightning_scan(qkv: torch.Tensor, H: int, D: int, Dv: int, state: torch.Tensor,
                   state_slots: torch.Tensor, cu_q: torch.Tensor, positions: torch.Tensor,
                   decay: torch.Tensor) -> torch.Tensor:
    """Decayed linear attention over a flat token batch: per sequence and head
    S <- decay_h S + k v^T, o = S^T q, token by token in f32, with q, k, v the
    SiLU of the first columns of ``qkv`` [T, >= 2 H D + H Dv]. ``state`` [slots,
    H, D, Dv] f32 carries S between steps (a sequence whose first position in
    this step is 0 starts from zero). Returns o f32 [T, H Dv]. Prompt portions
    and single decode tokens take the same kernel and the same order of
    operations, so the result does not depend on how a prompt was cut."""
    if not qkv.is_cuda:
        return ref.lightning_scan(qkv, H, D, Dv, state, state_slots, cu_q, positions, decay)
    T = qkv.shape[0]
    assert qkv.stride(1) == 1 and qkv.shape[1] >= 2 * H * D + H * Dv
    _f32c(state, "state"); _f32c(decay, "decay")
    assert state.shape[1:] == (H, D, Dv) and decay.numel() == H
    _i32c(state_slots, "state_slots"); _i32c(cu_q, "cu_q"); _i32c(positions, "positions")
    B = state_slots.numel()
    assert cu_q.numel() == B + 1
    o = torch.empty(T, H * Dv, dtype=torch.float32, device=qkv.device)
    if T:
        # SiLU of q | k | v once, in f32 (every column block of a head shares q and k)
        n = 2 * H * D + H * Dv
        act = torch.empty(T, n, dtype=torch.float32, device=qkv.device)
        k, st = kernels(), stream_ptr(qkv)
        check(k.loqa_lightning_prep(ptr(qkv), _dt(qkv), qkv.stride(0), T, n, ptr(act), st),
              "lightning_prep")
        check(k.loqa_lightning_scan(ptr(act), n, H, D, Dv, ptr(state), state.shape[0],
                                    ptr(state_slots), ptr(cu_q), ptr(positions), ptr(decay), ptr(o),
                                    B, T, st), "lightning_scan")
    return o


def gated_rmsnorm(o: torch.Tensor, w: torch.Tensor, gate: torch.Tensor, eps: float,
                  out_dtype) -> torch.Tensor:
    """y = rmsnorm(o) * w * sigmoid(gate) over whole rows of o f32 [T, n];
    ``gate`` [T, n] may be a column slice of a wider projection."""
    if not o.is_cuda:
        return ref.gated_rmsnorm(o, w, gate, eps, out_dtype)
    _f32c(o, "o"); _f32c(w, "w")
    T, n = o.shape
    assert gate.shape == (T, n) and gate.stride(1) == 1 and w.numel() == n
    y = torch.empty(T, n, dtype=out_dtype, device=o.device)
    if T:
        check(kernels().loqa_gated_rmsnorm(ptr(o), ptr(w), ptr(gate), _dt(gate), gate.stride(0), eps,
                                           ptr(y), _dt(y), T, n, stream_ptr(o)), "gated_rmsnorm")
    return y


def silu_mul_any(x: torch.Tensor) -> torch.Tensor:
    """[gate | up] -> silu(gate) * up for bf16 or f32 activations."""
    if not x.is_cuda:
        return ref.silu_mul(x)
    assert x.dim() == 2 and x.is_contiguous() and x.shape[1] % 2 == 0
    T, F2 = x.shape
    y = torch.empty(T, F2 // 2, dtype=x.dtype, device=x.device)
    if T:
        check(kernels().loqa_silu_mul_any(ptr(x), _dt(x), T, F2 // 2, ptr(y), stream_ptr(x)),
              "silu_mul_any")
    return y


def moe_route(z: torch.Tensor, correction: torch.Tensor | None, n_groups: int, keep: int,
              top: int, bias: torch.Tensor | None = None, top_softmax: bool = False
              ) -> tuple[torch.Tensor, torch.Tensor]:
    """Router decisions from f32 logits z [T, E] (+ ``bias`` [E]). Default:
    softmax scores, choice by score + ``correction`` limited to the ``keep``
    best of ``n_groups`` groups of neighbouring experts, weights = the plain
    scores (not renormalised). ``top_softmax``: the ``top`` largest logits are
    chosen and weighed by the softmax over the chosen logits only.
    Returns (idx int32 [T, top], weight f32 [T, top])."""
    if not z.is_cuda:
        return ref.moe_route(z, correction, n_groups, keep, top, bias, top_softmax)
    _f32c(z, "z")
    T, E = z.shape
    assert E % max(1, n_groups) == 0 and 0 < top <= E and E <= 1024
    for v, name in ((correction, "correction"), (bias, "bias")):
        if v is not None:
            _f32c(v, name)
            assert v.numel() == E
    idx = torch.empty(T, top, dtype=torch.int32, device=z.device)
    wt = torch.empty(T, top, dtype=torch.float32, device=z.device)
    if T:
        check(kernels().loqa_moe_route(ptr(z), ptr(correction), ptr(bias), int(top_softmax), E,
                                       max(1, n_groups), min(keep, max(1, n_groups)), top, ptr(idx),
                                       ptr(wt), T, stream_ptr(z)), "moe_route")
    return idx, wt


def moe_experts(h: torch.Tensor, idx: torch.Tensor, wt: torch.Tensor, w_gate_up: torch.Tensor,
                w_down: torch.Tensor, gated: bool = True) -> torch.Tensor:
    """Weighted sum of every token's chosen experts, f32 [T, d]. Experts below
    E = w_gate_up.shape[0] are feed-forwards: gated (w_gate_up [E, 2F, d] with
    gate rows then up rows, SwiGLU) or not (w_gate_up [E, F, d], the square of
    relu), w_down [E, d, F]; an index >= E is an identity expert. On the GPU: a
    device-side plan (tokens grouped by expert, no host round trip), a grouped
    up GEMM with the activation as its epilogue, a grouped down GEMM, and a
    combine launch that applies the weights in f32."""
    if not h.is_cuda:
        return ref.moe_experts(h, idx, wt, w_gate_up, w_down, h.dtype, gated)
    T, d = h.shape
    E, F2, _ = w_gate_up.shape
    F = F2 // 2 if gated else F2
    top = idx.shape[1]
    assert h.is_contiguous() and w_gate_up.is_contiguous() and w_down.is_contiguous()
    assert w_gate_up.dtype == h.dtype == w_down.dtype and w_down.shape == (E, d, F)
    assert w_gate_up.shape[2] == d
    _i32c(idx, "idx"); _f32c(wt, "wt")
    dev = h.device
    P = T * top
    out = torch.empty(T, d, dtype=torch.float32, device=dev)
    if T == 0:
        return out
    # plan: offsets[E + 1] of each expert's segment, perm[P] pair ids sorted by
    # expert (identity pairs last, past offsets[E]), pos[P] = where each pair sits
    plan = torch.empty(E + 2 + 2 * P, dtype=torch.int32, device=dev)
    act = torch.empty(P, F, dtype=h.dtype, device=dev)
    y = torch.empty(P, d, dtype=h.dtype, device=dev)
    k, st = kernels(), stream_ptr(h)
    check(k.loqa_moe_plan(ptr(idx), P, E, ptr(plan), st), "moe_plan")
    check(k.loqa_moe_grouped_gemm(ptr(h), _dt(h), ptr(w_gate_up), ptr(plan), P, E, top, d, F,
                                  1 if gated else 2, ptr(act), st), "moe_up")
    check(k.loqa_moe_grouped_gemm(ptr(act), _dt(h), ptr(w_down), ptr(plan), P, E, top, F, d, 0,
                                  ptr(y), st), "moe_down")
    check(k.loqa_moe_combine(ptr(h), ptr(y), _dt(h), ptr(idx), ptr(wt), ptr(plan), T, top, E, d,
                             ptr(out), st), "moe_combine")
    return out


# ---------------------------------------------------------------------------
# Per-sequence row state (token shift, convolution tails), chunked sigmoid
# attention over paged K/V, scalar-gain RMS norm on the residual step
# (csrc/kernels/seq_rows.hip, attn_sigmoid.hip, norm_scalar.hip)
def rope_table_half(dims: int, max_pos: int, base: float, device=None) -> torch.Tensor:
    """(cos, sin) table of the rotate-half rotary layout, built once at load time."""
    return ref.rope_table_half(dims, max_pos, base, device)


def _seq_args(state_slots, cu_q, positions, T):
    _i32c(state_slots, "state_slots"); _i32c(cu_q, "cu_q"); _i32c(positions, "positions")
    B = state_slots.numel()
    assert cu_q.numel() == B + 1 and positions.numel() >= T
    return B


def token_shift(x: torch.Tensor, mu: torch.Tensor, prev: torch.Tensor, state_slots: torch.Tensor,
                cu_q: torch.Tensor, positions: torch.Tensor, out_dtype) -> torch.Tensor:
    """h_t = x_t + (x_{t-1} - x_t) * mu over a flat token batch x f32 [T, d];
    the row before a feed's first token is ``prev[slot]`` f32 [slots, d] (zeros
    when the feed starts at position 0). ``prev`` is not written here
    (:func:`seq_state_save` does, once every reader of the step is done)."""
    if not x.is_cuda:
        return ref.token_shift(x, mu, prev, state_slots, cu_q, positions, out_dtype)
    _f32c(x, "x"); _f32c(mu, "mu"); _f32c(prev, "prev")
    T, d = x.shape
    assert mu.numel() == d and prev.shape[1] == d
    B = _seq_args(state_slots, cu_q, positions, T)
    h = torch.empty(T, d, dtype=out_dtype, device=x.device)
    if T:
        check(kernels().loqa_token_shift(ptr(x), ptr(mu), ptr(prev), prev.shape[0], ptr(state_slots),
                                         ptr(cu_q), ptr(positions), B, T, d, ptr(h), _dt(h),
                                         stream_ptr(x)), "token_shift")
    return h


def seq_state_save(x: torch.Tensor | None, u: torch.Tensor, prev: torch.Tensor | None,
                   tail: torch.Tensor, state_slots: torch.Tensor, cu_q: torch.Tensor,
                   positions: torch.Tensor) -> None:
    """The step's row state: prev[slot] = the last row of each feed of x f32
    [T, d]; tail[slot] f32 [taps - 1, C] = the last taps - 1 rows of the
    projections u[:, :C] (older rows move up under a shorter feed)."""
    if not u.is_cuda:
        return ref.seq_state_save(x, u, prev, tail, state_slots, cu_q, positions)
    T = u.shape[0]
    _f32c(tail, "tail")
    keep, C = tail.shape[1], tail.shape[2]
    assert u.stride(1) == 1 and u.shape[1] >= C
    d = 0
    if prev is not None:
        _f32c(x, "x"); _f32c(prev, "prev")
        d = x.shape[1]
        assert prev.shape == (tail.shape[0], d) and x.shape[0] == T
    B = _seq_args(state_slots, cu_q, positions, T)
    if T:
        check(kernels().loqa_seq_state_save(ptr(x), d, ptr(u), _dt(u), u.stride(0), ptr(prev),
                                            ptr(tail), tail.shape[0], keep, C, ptr(state_slots),
                                            ptr(cu_q), ptr(positions), B, stream_ptr(u)),
              "seq_state_save")


def conv_norm_rope_append(u: torch.Tensor, conv_w: torch.Tensor, tail: torch.Tensor,
                          state_slots: torch.Tensor, cu_q: torch.Tensor, positions: torch.Tensor,
                          q_norm: torch.Tensor, k_norm: torch.Tensor, eps: float,
                          cos_sin: torch.Tensor, dims: int, H: int, G: int, D: int,
                          k_cache: torch.Tensor, v_cache: torch.Tensor, slots: torch.Tensor,
                          out_dtype) -> torch.Tensor:
    """One launch between the q | k projection and attention: short causal
    convolution per channel (f32 weights conv_w tap-major [taps, (H + G) D]; the
    rows before a feed come from ``tail[slot]``), v = the convolved k, RMS norm of q
    and of k over the whole projection, rotate-half rotary on the first
    ``dims`` entries of every head, k into its paged cache [blocks, BLK, G D]
    and v into its transposed pages [blocks, G D, BLK]; returns q [T, H D]."""
    if not u.is_cuda:
        return ref.conv_norm_rope_append(u, conv_w, tail, state_slots, cu_q, positions, q_norm,
                                         k_norm, eps, cos_sin, dims, H, G, D, k_cache, v_cache,
                                         slots, out_dtype)
    T = u.shape[0]
    taps, C = conv_w.shape
    assert C == (H + G) * D and u.stride(1) == 1 and u.shape[1] >= C
    _f32c(conv_w, "conv_w"); _f32c(tail, "tail"); _f32c(q_norm, "q_norm"); _f32c(k_norm, "k_norm")
    _f32c(cos_sin, "cos_sin"); _i32c(slots, "slots")
    assert tail.shape[1:] == (taps - 1, C) and q_norm.numel() == H * D and k_norm.numel() == G * D
    assert dims % 2 == 0 and dims <= D and (dims == 0 or cos_sin.shape[1] * 2 == dims)
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.shape[2] == G * D and k_cache.dtype == v_cache.dtype == out_dtype
    assert v_cache.shape == (k_cache.shape[0], G * D, k_cache.shape[1])
    assert slots.numel() >= T
    B = _seq_args(state_slots, cu_q, positions, T)
    q = torch.empty(T, H * D, dtype=out_dtype, device=u.device)
    if T:
        check(kernels().loqa_conv_norm_rope_append(
            ptr(u), _dt(u), u.stride(0), ptr(conv_w), taps, ptr(tail), tail.shape[0],
            ptr(state_slots), ptr(cu_q), ptr(positions), B, T, ptr(q_norm), ptr(k_norm), eps,
            ptr(cos_sin), cos_sin.shape[0], dims, H, G, D, ptr(k_cache), ptr(v_cache),
            k_cache.shape[1], k_cache.shape[0], ptr(slots), ptr(q), _dt(q), stream_ptr(u)),
            "conv_norm_rope_append")
    return q


SIGMOID_MFMA_D = (64, 128)        # head sizes the matrix-core form is built for


def sigmoid_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      cu_q: torch.Tensor, ctx_lens: torch.Tensor, block_tables: torch.Tensor,
                      positions: torch.Tensor, head_bias: torch.Tensor, gate: torch.Tensor | None,
                      scale: float, chunk: int, H: int, G: int, D: int, max_q: int = 0,
                      matrix_cores: bool | None = None) -> torch.Tensor:
    """Attention without softmax over paged K [blocks, BLK, G D] and transposed
    V pages [blocks, G D, BLK]: a query at
    position p sees keys j <= p - with ``chunk`` > 0 only those of its own chunk
    (j // chunk == p // chunk, counted from the sequence's start) - and a
    visible key weighs sigmoid(q . k * scale + head_bias[h]) (f32, not
    normalised over keys). Head h's output is multiplied by sigmoid(gate[t, h])
    (``gate`` [T, H], may be a column slice). q [T, H D] -> [T, H D]. Prompt
    portions, decode tokens and mixed batches take the same launch; every
    output sums its keys in ascending position order whatever the batch."""
    if not q.is_cuda:
        return ref.sigmoid_attention(q, k_cache, v_cache, cu_q, ctx_lens, block_tables, positions,
                                     head_bias, gate, scale, chunk, H, G, D, q.dtype)
    T = q.shape[0]
    assert q.is_contiguous() and q.shape[1] == H * D and H % G == 0
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.shape[2] == G * D and k_cache.dtype == v_cache.dtype == q.dtype
    assert v_cache.shape == (k_cache.shape[0], G * D, k_cache.shape[1])
    _i32c(cu_q, "cu_q"); _i32c(ctx_lens, "ctx_lens"); _i32c(block_tables, "block_tables")
    _i32c(positions, "positions"); _f32c(head_bias, "head_bias")
    B = ctx_lens.numel()
    assert cu_q.numel() == B + 1 and block_tables.shape[0] == B and positions.numel() >= T
    assert head_bias.numel() == H
    gs = 0
    if gate is not None:
        assert gate.shape == (T, H) and gate.stride(1) == 1 and gate.dtype == q.dtype
        gs = gate.stride(0)
    o = torch.empty(T, H * D, dtype=q.dtype, device=q.device)
    if matrix_cores is None:
        matrix_cores = max_q >= 16
    mfma = bool(matrix_cores) and q.dtype == torch.bfloat16 and D in SIGMOID_MFMA_D
    if T:
        check(kernels().loqa_sigmoid_attention(
            ptr(q), _dt(q), ptr(k_cache), ptr(v_cache), k_cache.shape[1], k_cache.shape[0],
            ptr(cu_q), ptr(ctx_lens), ptr(block_tables), block_tables.shape[1], ptr(positions),
            ptr(head_bias), ptr(gate), gs, float(scale), int(chunk), B, T, H, G, D, int(max_q),
            int(mfma), ptr(o), stream_ptr(q)), "sigmoid_attention")
    return o


def scalar_rms_add(resid: torch.Tensor, y: torch.Tensor, g: float, eps: float, mult: float,
                   out_dtype=None) -> torch.Tensor | None:
    """The residual step with a norm on the sublayer's output only: resid (f32,
    in place) += mult * y / rms(y) * g with ONE gain g for all coordinates; the
    same launch returns resid in ``out_dtype`` for the next sublayer's GEMMs
    (None: nothing; float32: resid itself)."""
    if not resid.is_cuda:
        ref.scalar_rms_add(resid, y, g, eps, mult, None)
        if out_dtype is None:
            return None
        return resid if out_dtype == torch.float32 else resid.to(out_dtype)
    _f32c(resid, "resid")
    assert y.shape == resid.shape and y.is_contiguous()
    rows, d = resid.shape
    copy = out_dtype is not None and out_dtype != torch.float32
    h = torch.empty(rows, d, dtype=out_dtype, device=resid.device) if copy else None
    if rows:
        check(kernels().loqa_scalar_rms_add(ptr(resid), ptr(y), _dt(y), float(g) * float(mult),
                                            float(eps), ptr(h), rows, d, stream_ptr(resid)),
              "scalar_rms_add")
    return h if copy else (resid if out_dtype == torch.float32 else None)


def scalar_rms_norm(x: torch.Tensor, g: float, eps: float, row_idx: torch.Tensor | None = None
                    ) -> torch.Tensor:
    """f32 rows of x / rms(x) * g for x f32 [rows, d]; ``row_idx`` (int64)
    gathers rows in the same launch."""
    if not x.is_cuda:
        return ref.scalar_rms_norm(x, g, eps, row_idx)
    _f32c(x, "x")
    d = x.shape[1]
    rows = x.shape[0] if row_idx is None else row_idx.numel()
    if row_idx is not None:
        assert row_idx.dtype == torch.int64 and row_idx.is_contiguous()
    y = torch.empty(rows, d, dtype=torch.float32, device=x.device)
    if rows:
        check(kernels().loqa_scalar_rms_norm(ptr(x), ptr(row_idx), float(g), float(eps), ptr(y), rows,
                                             d, stream_ptr(x)), "scalar_rms_norm")
    return y
