"""The Sodonex family through the framework (registry, weights, engine step,
hybrid cache, scheduler) against the plain float64 oracle in
``sodonex_oracle.py``. Every test builds its own small configuration and
seeded weights. The same tests run on the CPU (reference ops) and, marked
``gpu``, on the HIP kernels.
"""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import sodonex_oracle as O
from loqa_hub_amd.engine.llm_engine import GenRequest, LLMEngine
from loqa_hub_amd.models.configs import sodonex_config_from_json
from loqa_hub_amd.models.registry import family_of, lm_config_from_json
from loqa_hub_amd.models.sodonex import SodonexWeights, config_to_json, random_state_dict
from loqa_hub_amd.ops import seqmix

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
TOL = {torch.float32: 2e-4, torch.bfloat16: 6e-2}
F64 = torch.float64


def engine(cfg_json, sd, device, dtype=torch.float32, max_tokens=256, block=16, max_seqs=4):
    cfg = lm_config_from_json(cfg_json, "t")
    w = SodonexWeights(cfg, sd, device, dtype, max_positions=max_tokens)
    return LLMEngine(cfg, device, weights=w, max_seqs=max_seqs, max_seq_len=max_tokens,
                     block_size=block, num_blocks=max_tokens // block, use_graphs=False, dtype=dtype)


def rel_err(got: torch.Tensor, want: torch.Tensor, q: float = 1.0) -> float:
    """RMS difference (mean removed per row) over the RMS of the wanted logits:
    the worst row, or the ``q`` quantile of the rows."""
    d = got.double().cpu() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()).quantile(q))


def feed(eng, seq, toks, cuts):
    """Feed ``toks`` to one sequence in portions of ``cuts`` sizes (cycled);
    returns the logits of every position."""
    out, i, k = [], 0, 0
    while i < len(toks):
        n = min(cuts[k % len(cuts)], len(toks) - i)
        out.append(eng.step_logits([seq], [toks[i:i + n]], [list(range(n))]))
        i, k = i + n, k + 1
    return torch.cat(out)


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# layers of unequal sizes: grouped heads, one key/value head, as many key/value
# heads as heads, no feed-forward, one tap, a chunk that is no power of two
FULL = [(O.attn(), O.moe_ff()),
        (O.attn(heads=6, kv_heads=1, dim=8, taps=2, chunk=5, dims=8), None),
        (O.attn(heads=2, kv_heads=2, dim=24, taps=3, chunk=16, dims=4, base=50.0),
         O.moe_ff(experts=3, top=3, ff=8)),
        (O.attn(heads=3, kv_heads=1, dim=16, taps=1, chunk=11, dims=0), O.moe_ff(experts=9, top=1))]


@pytest.fixture(scope="module")
def full_model():
    cfg = O.make_config(FULL)
    return cfg, O.make_weights(cfg, 1)


def test_registry_reads_config(full_model):
    cfg_json, _ = full_model
    cfg = lm_config_from_json(json.loads(json.dumps(cfg_json)))
    assert family_of(cfg).name == "sodonex" and family_of(cfg_json).hybrid
    assert cfg.n_layers == len(FULL) and cfg.layers[1].mlp is None
    assert cfg.layers[1].mixer.chunk == 5 and cfg.layers[3].mixer.taps == 1
    assert cfg.layers[2].mlp.top == 3 and cfg.layers[2].mlp.act == "relu2"
    assert cfg.residual_mult == cfg_json["residual_mult"]
    assert config_to_json(cfg)["layers"] == json.loads(json.dumps(cfg_json))["layers"]
    for key, val in (("kv_heads", 3), ("vdim", 8)):
        bad = json.loads(json.dumps(cfg_json))
        bad["layers"][0]["mixer"][key] = val
        with pytest.raises(ValueError):
            sodonex_config_from_json(bad)
    sd = random_state_dict(cfg, 0)
    assert sd["l0.norm1"].dim() == 0 and sd["l3.mix.q.conv"].shape == (48, 1)


# ------------------------------------------------------ each mechanism alone
def _meta(lens, starts, device):
    cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32)
    pos = torch.cat([s + torch.arange(n) for n, s in zip(lens, starts)]).to(torch.int32)
    return cu.to(device), pos.to(device)


@pytest.mark.parametrize("device", DEVICES)
def test_token_shift_and_saved_row(device):
    g = torch.Generator().manual_seed(0)
    d, n = 40, 23
    x = torch.randn(n, d, generator=g)
    mu = torch.rand(d, generator=g)
    want = O.token_shift(x.double(), mu.double())
    for cuts in ([n], [1] * n, [2, 7, 1, 13]):
        prev = torch.full((3, d), 99.0, device=device)       # a dirty slot
        tail = torch.zeros(3, 0, 1, device=device)
        slot = torch.tensor([1], dtype=torch.int32, device=device)
        got, at = [], 0
        for c in cuts:
            cu, pos = _meta([c], [at], device)
            xs = x[at:at + c].to(device).contiguous()
            got.append(seqmix.token_shift(xs, mu.to(device), prev, slot, cu, pos, torch.float32))
            seqmix.seq_state_save(xs, xs, prev, tail, slot, cu, pos)
            at += c
        assert (torch.cat(got).cpu().double() - want).abs().max() < 1e-6, cuts
        assert torch.equal(prev[1].cpu(), x[-1]) and float(prev[0, 0]) == 99.0


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("extra", [3, 8], ids=["rows_unaligned", "rows_aligned"])
@pytest.mark.parametrize("taps,dims", [(4, 8), (1, 16), (2, 0), (7, 4)])
def test_conv_norm_rotary_append(device, taps, dims, extra):
    """The launch between the projection and attention, fed in portions (some
    shorter than the convolution) into scattered page slots: q, the cached k
    and the cached v (= the convolved k before norm and rotation)."""
    g = torch.Generator().manual_seed(taps)
    H, G, D, n, eps, base = 3, 2, 16, 19, 1e-5, 100.0
    C = (H + G) * D
    u = torch.randn(n, C + extra, generator=g)                # more columns ride along
    cw = torch.randn(C, taps, generator=g) * 0.5
    qn, kn = torch.rand(H * D, generator=g) + 0.5, torch.rand(G * D, generator=g) + 0.5
    y = O.short_conv(u[:, :C].double(), cw.double())
    wq = O.rotate_half((O.rms(y[:, :H * D], eps) * qn.double()).view(n, H, D), dims, base)
    wk = O.rotate_half((O.rms(y[:, H * D:], eps) * kn.double()).view(n, G, D), dims, base)
    table = seqmix.rope_table_half(dims, 64, base, device)
    for cuts in ([n], [1] * n, [2, 1, 9, 3, 4]):
        kc, vc = torch.zeros(4, 8, G * D, device=device), torch.zeros(4, G * D, 8, device=device)
        tail = torch.full((2, taps - 1, C), 7.0, device=device)
        slot = torch.tensor([1], dtype=torch.int32, device=device)
        where = torch.randperm(32, generator=g)[:n].to(torch.int32)
        got, at = [], 0
        for c in cuts:
            cu, pos = _meta([c], [at], device)
            us = u[at:at + c].to(device)
            got.append(seqmix.conv_norm_rope_append(
                us, cw.t().contiguous().to(device), tail, slot, cu, pos, qn.to(device), kn.to(device), eps, table,
                dims, H, G, D, kc, vc, where[at:at + c].to(device), torch.float32))
            seqmix.seq_state_save(None, us, None, tail, slot, cu, pos)
            at += c
        rows = where.long()
        assert (torch.cat(got).cpu().double() - wq.reshape(n, -1)).abs().max() < 2e-5, cuts
        assert (kc.view(32, -1)[rows].cpu().double() - wk.reshape(n, -1)).abs().max() < 2e-5
        vrows = vc.transpose(1, 2).reshape(32, -1)[rows]           # value pages are [G D, BLK]
        assert (vrows.cpu().double() - y[:, H * D:]).abs().max() < 2e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,chunk", [(4, 2, 16, 8), (3, 3, 8, 5), (6, 2, 64, 48), (2, 1, 24, 1),
                                         (4, 4, 128, 40), (2, 2, 16, 0), (5, 1, 32, 64)])
def test_sigmoid_attention_op(device, H, G, D, chunk):
    """The attention op on a batch of three unequal sequences (one decoding a
    single token at the first position of a chunk) against the oracle: keys
    beyond the chunk's edge weigh nothing, keys inside are not normalised."""
    g = torch.Generator().manual_seed(H * D + chunk)
    blk, lens = 16, [37, 50, 81]
    feeds = [37, 1, 30]
    if chunk:
        lens[1] = 3 * chunk + 1                                # position 3 * chunk: sees itself only
    scale = D ** -0.5
    pb = torch.randn(H, generator=g)
    nblk = sum(-(-n // blk) for n in lens)
    kc, vc = torch.zeros(nblk, blk, G * D), torch.zeros(nblk, G * D, blk)
    order = torch.randperm(nblk, generator=g).tolist()
    bt = torch.zeros(3, 16, dtype=torch.int32)
    qs, want, gates = [], [], []
    for b, n in enumerate(lens):
        q = torch.randn(n, H, D, generator=g)
        k = torch.randn(n, G, D, generator=g)
        v = torch.randn(n, G, D, generator=g)
        gate = torch.randn(n, H, generator=g)
        o = O.chunk_sigmoid_attention(q.double(), k.double(), v.double(), scale, pb.double(),
                                      chunk if chunk else 10 ** 6)
        o = o * torch.sigmoid(gate.double())[:, :, None]
        for i in range(-(-n // blk)):
            page = order.pop()
            bt[b, i] = page
            m = min(blk, n - i * blk)
            kc[page, :m] = k[i * blk:i * blk + m].reshape(m, -1)
            vc[page, :, :m] = v[i * blk:i * blk + m].reshape(m, -1).T
        f = feeds[b]
        qs.append(q[n - f:].reshape(f, -1)); gates.append(gate[n - f:]); want.append(o[n - f:].reshape(f, -1))
    cu, pos = _meta(feeds, [n - f for n, f in zip(lens, feeds)], device)
    got = seqmix.sigmoid_attention(
        torch.cat(qs).to(device), kc.to(device), vc.to(device), cu,
        torch.tensor(lens, dtype=torch.int32, device=device), bt.to(device), pos, pb.to(device),
        torch.cat(gates).to(device), scale, chunk, H, G, D, max(feeds))
    want = torch.cat(want)
    assert (got.cpu().double() - want).abs().max() / want.abs().max() < 1e-5


@pytest.mark.parametrize("device", DEVICES)
def test_router_top_softmax(device):
    g = torch.Generator().manual_seed(0)
    for E, top in [(10, 3), (5, 5), (7, 1), (130, 4)]:
        h = torch.randn(33, 16, generator=g)
        sd = {"r.router": torch.randn(E, 16, generator=g), "r.router.b": torch.randn(E, generator=g)}
        idx, wt = O.route(h.double(), sd, "r.", {"router": {"experts": E, "top": top}})
        z = (h @ sd["r.router"].T).to(device)
        gi, gw = seqmix.moe_route(z, None, 1, 1, top, bias=sd["r.router.b"].to(device),
                                  top_softmax=True)
        gi, gw = gi.cpu().long(), gw.cpu().double()
        for t in range(33):
            assert set(gi[t].tolist()) == set(idx[t].tolist())
            a = dict(zip(gi[t].tolist(), gw[t].tolist()))
            for e, w in zip(idx[t].tolist(), wt[t].tolist()):
                assert abs(a[e] - w) < 1e-5
            assert abs(sum(a.values()) - 1.0) < 1e-5


@pytest.mark.parametrize("device", DEVICES)
def test_scalar_norm_residual_step(device):
    g = torch.Generator().manual_seed(2)
    for d in (24, 320, 700, 2500):
        x, y = torch.randn(9, d, generator=g), torch.randn(9, d, generator=g) * 3
        want = x.double() + 0.3 * O.scalar_norm(y.double(), 1.7, 1e-5)
        r = x.clone().to(device)
        h = seqmix.scalar_rms_add(r, y.to(device), 1.7, 1e-5, 0.3, torch.bfloat16)
        assert (r.cpu().double() - want).abs().max() < 1e-5
        assert torch.equal(h.cpu(), r.cpu().to(torch.bfloat16))
        rows = torch.tensor([8, 0, 3], device=device)
        n = seqmix.scalar_rms_norm(r, 0.9, 1e-5, rows)
        assert (n.cpu().double() - O.scalar_norm(want[[8, 0, 3]], 0.9, 1e-5)).abs().max() < 1e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("layer", [
    (O.attn(), None),
    (O.attn(heads=4, kv_heads=1, dim=64, chunk=16, dims=16), None),      # matrix-core head size
    (O.attn(heads=2, kv_heads=2, dim=8, taps=1, chunk=1, dims=8), None),  # every token alone
    (O.attn(heads=5, kv_heads=5, dim=12, taps=6, chunk=100, dims=2), None),   # one chunk holds all
    (O.attn(), O.moe_ff()),
    (O.attn(), O.moe_ff(experts=4, top=4, ff=40)),
    (O.attn(), O.moe_ff(experts=70, top=2, ff=8)),
], ids=["grouped", "one_kv_head", "chunk_of_one", "wide_chunk", "moe", "moe_all", "moe_many"])
def test_single_layer(device, layer):
    cfg = O.make_config([layer], width=40, vocab=90)
    sd = O.make_weights(cfg, 3)
    toks = tokens(37, 90, 5)
    want, trail = O.forward(cfg, sd, toks, layers_out=True)
    eng = engine(cfg, sd, device)
    s = eng.open_sequence()
    got = eng.step_logits([s], [toks], [list(range(len(toks)))])
    assert rel_err(got, want) < TOL[torch.float32]
    # the residual stream after the layer, through the model's own step function
    max_q, max_ctx, host = eng._meta([eng.open_sequence()], [toks], decode=False)
    meta = eng._build_meta(eng._to_device(host), max_q, max_ctx, False)
    seen = []
    eng.model.forward(meta, eng.kv, trail=seen)
    assert (seen[0].cpu().double() - trail[0]).abs().max() / trail[0].abs().max() < 1e-5


# ------------------------------------------- whole model, cuts, batches, reuse
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_prompt(device, dtype, full_model):
    cfg, sd = full_model
    toks = tokens(70, cfg["vocab"], 11)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device, dtype)
    got = eng.step_logits([eng.open_sequence()], [toks], [list(range(len(toks)))])
    if dtype == torch.float32:
        assert rel_err(got, want) < TOL[dtype]
    else:
        # single rows move under 16-bit rounding when a router logit is nearly
        # tied: the typical row is what is pinned
        assert rel_err(got, want, 0.5) < TOL[dtype] and rel_err(got, want, 0.9) < 0.25


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2, 7], [16], [17, 1, 1, 30], [5, 64]],
                         ids=lambda c: "x".join(map(str, c)))
def test_portions_and_decode(device, cuts, full_model):
    """Token-by-token decoding and portions of any size (down to two tokens,
    shorter than the convolutions, across page borders at 16 and chunk edges at
    5, 8, 11 and 16) give the whole prompt's logits."""
    cfg, sd = full_model
    toks = tokens(53, cfg["vocab"], 12)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device)
    got = feed(eng, eng.open_sequence(), toks, cuts)
    assert rel_err(got, want) < TOL[torch.float32]


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_and_reuse(device, full_model):
    """Four unequal requests, portions beside single tokens in one step; two
    end early and two new ones take over their pages and state slots. Every
    request's logits equal the ones it gets alone (oracle)."""
    cfg, sd = full_model
    V = cfg["vocab"]
    reqs = {n: tokens(L, V, 20 + i) for i, (n, L) in
            enumerate([("a", 41), ("b", 1), ("c", 18), ("d", 33), ("e", 25), ("f", 47)])}
    want = {n: O.forward(cfg, sd, t) for n, t in reqs.items()}
    eng = engine(cfg, sd, device, max_tokens=192, max_seqs=4)
    plan = {"a": [7, 1, 1, 16, 2, 1, 13], "b": [1], "c": [2, 15, 1], "d": [16, 16, 1],
            "e": [3, 1, 21], "f": [30, 1, 16]}
    at = {n: 0 for n in reqs}
    live, waiting, got = {}, ["a", "b", "c", "d", "e", "f"], {n: [] for n in reqs}
    steps = 0
    while waiting or live:
        while waiting and len(live) < 4:
            n = waiting.pop(0)
            live[n] = eng.open_sequence()
        names = list(live)
        feeds, wants = [], []
        for n in names:
            k = plan[n].pop(0)
            feeds.append(reqs[n][at[n]:at[n] + k])
            wants.append(list(range(k)))
            at[n] += k
        out = eng.step_logits([live[n] for n in names], feeds, wants)
        o = 0
        for n, f in zip(names, feeds):
            got[n].append(out[o:o + len(f)])
            o += len(f)
            if at[n] == len(reqs[n]):
                eng.close_sequence(live.pop(n))
        steps += 1
    assert steps > 5
    for n in reqs:
        assert rel_err(torch.cat(got[n]), want[n]) < TOL[torch.float32], n
    assert eng.kv.pool.free_blocks() == 192 // 16 and eng.kv.slots.free_slots() == 4


@pytest.mark.parametrize("device", DEVICES)
def test_slot_and_pages_reused_clean(device, full_model):
    """A sequence that takes over used pages and a slot whose rows hold another
    sequence's last tokens starts from nothing; a sequence left out of a step
    goes on from its own rows."""
    cfg, sd = full_model
    eng = engine(cfg, sd, device, max_tokens=64, max_seqs=1)
    a, b = tokens(60, cfg["vocab"], 31), tokens(29, cfg["vocab"], 32)
    s = eng.open_sequence()
    eng.step_logits([s], [a], [[]])
    with pytest.raises(RuntimeError):
        eng.open_sequence()                                   # the only slot is taken
    eng.close_sequence(s)
    s = eng.open_sequence()
    got = feed(eng, s, b, [4, 1])
    assert rel_err(got, O.forward(cfg, sd, b)) < TOL[torch.float32]
    eng2 = engine(cfg, sd, device, max_tokens=128, max_seqs=2)
    s1, s2 = eng2.open_sequence(), eng2.open_sequence()
    g1 = [eng2.step_logits([s1, s2], [a[:9], b[:20]], [list(range(9)), []])]
    eng2.step_logits([s2], [b[20:]], [[]])                    # s1 sits this step out
    g1.append(eng2.step_logits([s1], [a[9:40]], [list(range(31))]))
    assert rel_err(torch.cat(g1), O.forward(cfg, sd, a[:40])) < TOL[torch.float32]


def _echo_model(chunk, taps=1):
    """One layer whose attention answers 'which token opened my chunk': the
    key of the probed token scores far above the others, so a chunk edge that
    is one token off, or a lost key, changes the logits by much more than the
    tolerance."""
    cfg = O.make_config([(O.attn(heads=2, kv_heads=1, dim=16, taps=taps, chunk=chunk, dims=0,
                                 scale=1.5), None)], width=32, vocab=400, mult=1.0)
    sd = O.make_weights(cfg, 7)
    sd["l0.shift"] = torch.zeros(32, dtype=torch.bfloat16)
    sd["l0.mix.q.norm"] = torch.ones(32, dtype=torch.bfloat16)
    sd["l0.mix.k.norm"] = torch.ones(16, dtype=torch.bfloat16)
    sd["l0.mix.q.b"] = torch.zeros(32, dtype=torch.bfloat16)
    sd["l0.mix.k.b"] = torch.zeros(16, dtype=torch.bfloat16)
    sd["l0.mix.pb"] = torch.full((2,), -14.0, dtype=torch.bfloat16)   # only a matching key counts
    # the query of a token is the key of the same embedding flipped: a probe
    # whose embedding is the flip of token A's scores A's key highest
    wk = sd["l0.mix.k"].float()
    sd["l0.mix.q"] = torch.cat([wk.flip(1), wk.flip(1)]).to(torch.bfloat16)
    one = torch.zeros(16, taps)
    one[:, -1] = 1.0                               # the convolutions pass the current token through
    sd["l0.mix.q.conv"] = one.repeat(2, 1).to(torch.bfloat16)
    sd["l0.mix.k.conv"] = one.to(torch.bfloat16)
    return cfg, sd


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("chunk", [16, 24, 64])
def test_chunk_edges_in_prompts_and_decoding(device, chunk):
    """Probes just inside and just outside a chunk edge, and one far back: the
    probe placed in the marked token's chunk hears it, the probe one chunk later
    (also when the marked token is the previous position, a page border for
    chunk 16) does not; in whole prompts, portions and single-token decoding."""
    cfg, sd = _echo_model(chunk)
    n_chunks = 5
    mark_at = 2 * chunk                            # the first position of chunk 2
    for probe_at in (mark_at + 1, 3 * chunk - 1, 3 * chunk, 4 * chunk + 3):
        toks = list(range(1, n_chunks * chunk + 1))          # all different
        probe = 299
        sd["embed"][probe] = sd["embed"][toks[mark_at]].flip(0)
        toks[probe_at] = probe
        want = O.forward(cfg, sd, toks)[probe_at:probe_at + 1]
        other = list(toks)
        other[mark_at] = 298
        moved = O.forward(cfg, sd, other)[probe_at:probe_at + 1]
        inside = probe_at < 3 * chunk
        assert (rel_err(moved.float(), want) > 0.1) == inside      # heard only inside the chunk
        for cuts in ([len(toks)], [mark_at + 1, 1], [7], [probe_at, 1, 2]):
            eng = engine(cfg, sd, device, max_tokens=n_chunks * 64 if chunk == 64 else 256)
            got = feed(eng, eng.open_sequence(), toks, cuts)[probe_at:probe_at + 1]
            assert rel_err(got, want) < TOL[torch.float32], (probe_at, cuts)


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_taps(device):
    """The first tokens of a sequence: convolution taps and the shifted row
    before position 0 are zeros whatever the slot held; portions shorter than
    the convolution keep the tail in order."""
    cfg = O.make_config([(O.attn(heads=2, kv_heads=1, dim=8, taps=5, chunk=4, dims=4), O.moe_ff()),
                         (O.attn(heads=2, kv_heads=2, dim=8, taps=3, chunk=6, dims=8), None)],
                        width=24, vocab=50)
    sd = O.make_weights(cfg, 9)
    toks = tokens(14, 50, 2)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device, max_tokens=32, max_seqs=1)
    for cuts in ([1], [2], [3, 1], [14]):
        s = eng.open_sequence()
        assert rel_err(feed(eng, s, toks, cuts), want) < TOL[torch.float32], cuts
        eng.close_sequence(s)                                  # the next run reuses slot and pages


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_odd_sizes(device, dtype):
    """A width, vocabulary, head size and expert width that are no multiples of
    8 (no 16-byte rows anywhere), three query heads per key/value head."""
    cfg = O.make_config([(O.attn(heads=3, kv_heads=1, dim=10, taps=3, chunk=9, dims=6),
                          O.moe_ff(experts=5, top=2, ff=13)),
                         (O.attn(heads=6, kv_heads=2, dim=14, taps=2, chunk=4, dims=14), None)],
                        width=50, vocab=77)
    sd = O.make_weights(cfg, 8)
    toks = tokens(45, 77, 3)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device, dtype, max_tokens=64)
    got = feed(eng, eng.open_sequence(), toks, [20, 1, 1, 6, 17])
    if dtype == torch.float32:
        assert rel_err(got, want) < TOL[dtype]
    else:
        assert rel_err(got, want, 0.5) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode(device):
    """150 single-token steps over many chunks and pages."""
    cfg = O.make_config([(O.attn(heads=2, kv_heads=1, dim=8, taps=4, chunk=7, dims=4), None),
                         (O.attn(heads=4, kv_heads=2, dim=8, taps=2, chunk=32, dims=8),
                          O.moe_ff(experts=4, top=2, ff=16))], width=24, vocab=60)
    sd = O.make_weights(cfg, 4)
    toks = tokens(160, 60, 6)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device, max_tokens=160)
    got = feed(eng, eng.open_sequence(), toks, [10] + [1] * 150)
    assert rel_err(got, want) < TOL[torch.float32]


# ------------------------------------------- the engine's own entry points
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(device, full_model):
    """Schema-less requests through ``submit_batch`` (continuous batching:
    inline prompts, chunked prompts in mixed steps, decode steps) produce the
    oracle's greedy continuation."""
    cfg, sd = full_model
    V = cfg["vocab"]
    prompts = [tokens(n, V, 40 + i) for i, n in enumerate([5, 90, 23, 70])]
    n_new = 6

    def greedy(p):
        seq = list(p)
        for _ in range(n_new):
            seq.append(int(O.forward(cfg, sd, seq)[-1].argmax()))
        return seq[len(p):]
    want = [greedy(p) for p in prompts]
    eng = engine(cfg, sd, device, max_tokens=512, max_seqs=4)
    eng.chunk_prefill = 32          # prompts longer than inline_prefill go in 32-token chunks
    eng.inline_prefill = 8
    reqs = [GenRequest(p, None, max_new_tokens=n_new) for p in prompts]
    try:
        eng.submit_batch(reqs[:2]).result(timeout=300)
        f1 = eng.submit_batch(reqs[2:3])
        f2 = eng.submit_batch(reqs[3:])
        f1.result(timeout=300), f2.result(timeout=300)
    finally:
        eng.stop()
    for r, w in zip(reqs, want):
        assert r.done and r.grammar.emitted == w
    assert eng.kv.slots.free_slots() == 4


def test_generate_entry_point(full_model):
    cfg, sd = full_model
    p = tokens(12, cfg["vocab"], 50)
    eng = engine(cfg, sd, "cpu")
    r = eng.generate([GenRequest(p, None, max_new_tokens=3)])[0]
    seq = list(p)
    for _ in range(3):
        seq.append(int(O.forward(cfg, sd, seq)[-1].argmax()))
    assert r.grammar.emitted == seq[len(p):]


def test_trace_replay_program(tmp_path, full_model):
    """The replay command on a checkpoint folder: steps on stdin, logits files
    and ``done`` lines out; a request that sits out a step goes on later."""
    from loqa_hub_amd.models.loader import write_safetensors
    cfg, sd = full_model
    model = tmp_path / "m"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(cfg))
    write_safetensors(sd, str(model / "model.safetensors"))
    a, b = tokens(20, cfg["vocab"], 60), tokens(9, cfg["vocab"], 61)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:11], "want": [0, 10]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:8], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[11:], "want": [8]},
                                {"id": "b", "tokens": b[8:], "want": [0]}], "end": ["a", "b"]},
    ]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, "-m", "loqa_hub_amd.cli.trace_run", "--model", str(model),
                        "--dtype", "float32", "--out", str(out), "--max-tokens", "64",
                        "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                       capture_output=True, cwd=ROOT, timeout=300)
    assert p.returncode == 0, p.stderr
    assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == \
        ["done 0", "done 1", "done 2"]
    V = cfg["vocab"]
    wa, wb = O.forward(cfg, sd, a), O.forward(cfg, sd, b)
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V))
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V))
    assert not (out / "1.f32").exists()
    assert rel_err(g0, wa[[0, 10]]) < TOL[torch.float32]
    assert rel_err(g2, torch.stack([wa[19], wb[8]])) < TOL[torch.float32]


# ------------------------------------------- matrix-core paths (bf16, GPU only)
@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,chunk", [(6, 1, 64, 48), (4, 2, 128, 64), (40, 2, 64, 20),
                                         (3, 3, 64, 0), (12, 1, 128, 1000)])
def test_sigmoid_attention_matrix_cores(H, G, D, chunk):
    """The bf16 matrix-core form against the row form and the f64 oracle on a
    mixed batch: a long portion on top of a cached context that starts in the
    middle of a chunk, a short portion, and single decode tokens."""
    g = torch.Generator().manual_seed(H + D + chunk)
    blk, lens, feeds = 16, [150, 33, 70, 5], [101, 33, 1, 1]
    scale = D ** -0.5
    pb = torch.randn(H, generator=g) - 1.0
    nblk = sum(-(-n // blk) for n in lens)
    kc, vc = torch.zeros(nblk, blk, G * D), torch.zeros(nblk, G * D, blk)
    order = torch.randperm(nblk, generator=g).tolist()
    bt = torch.zeros(4, 16, dtype=torch.int32)
    qs, want, gates = [], [], []
    for b, n in enumerate(lens):
        q = torch.randn(n, H, D, generator=g).bfloat16()
        k = torch.randn(n, G, D, generator=g).bfloat16()
        v = torch.randn(n, G, D, generator=g).bfloat16()
        gate = torch.randn(n, H, generator=g).bfloat16()
        o = O.chunk_sigmoid_attention(q.double(), k.double(), v.double(), scale, pb.double(),
                                      chunk if chunk else 10 ** 6)
        o = o * torch.sigmoid(gate.double())[:, :, None]
        for i in range(-(-n // blk)):
            page = order.pop()
            bt[b, i] = page
            m = min(blk, n - i * blk)
            kc[page, :m] = k[i * blk:i * blk + m].reshape(m, -1).float()
            vc[page, :, :m] = v[i * blk:i * blk + m].reshape(m, -1).float().T
        f = feeds[b]
        qs.append(q[n - f:].reshape(f, -1)); gates.append(gate[n - f:]); want.append(o[n - f:].reshape(f, -1))
    cu, pos = _meta(feeds, [n - f for n, f in zip(lens, feeds)], "cuda")
    args = (torch.cat(qs).cuda(), kc.bfloat16().cuda(), vc.bfloat16().cuda(), cu,
            torch.tensor(lens, dtype=torch.int32).cuda(), bt.cuda(), pos, pb.cuda(),
            torch.cat(gates).cuda(), scale, chunk, H, G, D, max(feeds))
    rows = seqmix.sigmoid_attention(*args, matrix_cores=False).float().cpu()
    mfma = seqmix.sigmoid_attention(*args, matrix_cores=True).float().cpu()
    want = torch.cat(want)
    top = want.abs().max()
    assert (rows.double() - want).abs().max() / top < 1e-2
    assert (mfma.double() - want).abs().max() / top < 1e-2
    assert (mfma - rows).abs().max() / top < 1e-2


@pytest.mark.gpu
@pytest.mark.parametrize("T,d,F", [(333, 96, 64), (2100, 64, 64)], ids=["direct", "staged"])
def test_relu2_expert_gemm_matrix_cores(T, d, F):
    """The bf16 grouped expert GEMMs with the squared-relu epilogue on the
    matrix cores against the f32 reference: unequal expert loads, an empty
    expert, segments that do not fill a tile."""
    from loqa_hub_amd.ops import reference as ref
    g = torch.Generator().manual_seed(3)
    E, top = 7, 3
    h = torch.randn(T, d, generator=g).to(torch.bfloat16)
    wu = (torch.randn(E, F, d, generator=g) / d ** 0.5).to(torch.bfloat16)
    wd = (torch.randn(E, d, F, generator=g) / F ** 0.5).to(torch.bfloat16)
    idx = torch.randint(0, E, (T, top), generator=g).to(torch.int32)
    idx[idx == 4] = 5                                      # expert 4 gets nothing
    wt = torch.rand(T, top, generator=g)
    want = ref.moe_experts(h.float(), idx, wt, wu.float(), wd.float(), torch.float32, gated=False)
    got = seqmix.moe_experts(h.cuda(), idx.cuda(), wt.cuda(), wu.cuda(), wd.cuda(),
                             gated=False).cpu()
    err = (got - want).abs().max() / want.abs().max()
    assert err < 2e-2, float(err)
