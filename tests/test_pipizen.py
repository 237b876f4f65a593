"""The Pipizen family through the framework (registry, weights, engine step,
hybrid cache, scheduler) against the plain float64 oracle in
``pipizen_oracle.py``. Every test builds its own small configuration and
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

import pipizen_oracle as O
from loqa_hub_amd.engine.llm_engine import GenRequest, LLMEngine
from loqa_hub_amd.models.configs import pipizen_config_from_json
from loqa_hub_amd.models.pipizen import PipizenWeights
from loqa_hub_amd.models.registry import family_of, lm_config_from_json

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
TOL = {torch.float32: 2e-4, torch.bfloat16: 6e-2}


def engine(cfg_json, sd, device, dtype=torch.float32, max_tokens=256, block=16, max_seqs=4):
    cfg = lm_config_from_json(cfg_json, "t")
    w = PipizenWeights(cfg, sd, device, dtype, max_positions=max_tokens)
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


FULL = [(O.latent(), O.dense()),
        (O.lightning_layer(), O.moe_ff()),
        (O.latent(kv_from=0), None),
        (O.latent(heads=2, dim=8, rot_dim=12, vdim=20, kv_rank=40, dims=8, scaling=False),
         O.moe_ff(experts=5, identity=0, top=1, count=1, keep=1, shared=0)),
        (O.lightning_layer(heads=3, dim=24, vdim=40), O.dense(32)),
        (O.latent(heads=2, dim=8, rot_dim=12, vdim=20, kv_rank=40, dims=8, scaling=False,
                  kv_from=3), O.moe_ff(experts=9, identity=3, top=3, count=3, keep=2))]


@pytest.fixture(scope="module")
def full_model():
    cfg = O.make_config(FULL)
    return cfg, O.make_weights(cfg, 1)


def test_registry_reads_config(full_model):
    cfg_json, _ = full_model
    cfg = lm_config_from_json(json.loads(json.dumps(cfg_json)))
    assert family_of(cfg).name == "pipizen" and family_of(cfg_json).hybrid
    assert cfg.n_layers == len(FULL) and cfg.layers[2].mlp is None
    assert cfg.layers[5].mixer.kv_from == 3 and cfg.layers[3].mixer.rot.yarn is None
    assert cfg.layers[1].mlp.identity == 2 and cfg.layers[3].mlp.groups == 1
    assert family_of({"architectures": ["LlamaForCausalLM"], "num_attention_heads": 4,
                      "hidden_size": 64}).name == "llama"
    with pytest.raises(ValueError):
        bad = json.loads(json.dumps(cfg_json))
        bad["layers"][2]["mixer"]["kv_from"] = 1          # a lightning layer holds no latent cache
        pipizen_config_from_json(bad)


# ------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("layer", [
    (O.latent(), None),                                                   # sink, YaRN, folded q/k
    (O.latent(heads=1, dim=32, rot_dim=4, vdim=8, kv_rank=16, dims=2), None),   # rot.dims < rot_dim
    (O.latent(scaling=False, base=500.0), None),
    (O.latent(heads=2, dim=8, rot_dim=6, vdim=10, kv_rank=23, dims=4), None),    # odd row length
    (O.latent(heads=5, dim=8, rot_dim=8, vdim=6, kv_rank=26), None),   # rows not 16-byte multiples
    (O.lightning_layer(), None),
    (O.lightning_layer(heads=1, dim=72, vdim=80, decay=[0.999]), None),   # D, Dv beyond one tile
    (O.lightning_layer(heads=5, dim=8, vdim=8, decay=[0.1, 0.3, 0.6, 0.9, 1.0]), None),
    (O.lightning_layer(), O.dense()),
    (O.lightning_layer(), O.moe_ff()),
    (O.lightning_layer(), O.moe_ff(experts=4, identity=4, top=3, count=2, keep=1, shared=0)),
    (O.lightning_layer(), O.moe_ff(experts=70, identity=2, top=4, count=8, keep=3, ff=8)),
], ids=["latent", "latent_partrot", "latent_plain", "latent_odd", "latent_unaligned", "lightning", "lightning_wide",
        "lightning_decays", "dense", "moe", "moe_identity", "moe_many"])
def test_single_layer(device, layer):
    cfg = O.make_config([layer], width=40, vocab=90)
    sd = O.make_weights(cfg, 3)
    toks = tokens(37, 90, 5)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device)
    s = eng.open_sequence()
    got = eng.step_logits([s], [toks], [list(range(len(toks)))])
    assert rel_err(got, want) < TOL[torch.float32]


@pytest.mark.parametrize("device", DEVICES)
def test_router_choices(device):
    """Group limits, negative choice scores and identity experts: the chosen
    set and the weights equal the oracle's."""
    from loqa_hub_amd.ops import seqmix
    g = torch.Generator().manual_seed(0)
    for E, G, keep, top in [(12, 3, 2, 3), (8, 8, 3, 2), (6, 1, 1, 6), (64, 4, 1, 5)]:
        z = torch.randn(33, E, generator=g) * 2
        corr = torch.randn(E, generator=g) * 0.3 - 0.4     # mostly negative choice scores
        sd = {"router": torch.eye(E), "correction": corr}
        idx, wt = O.route(z.double(), {"r.router": torch.eye(E, dtype=torch.float64),
                                       "r.correction": corr}, "r.",
                          {"experts": E, "identity": 0, "top": top,
                           "groups": {"count": G, "keep": keep}})
        gi, gw = seqmix.moe_route(z.to(device), corr.to(device), G, keep, top)
        gi, gw = gi.cpu().long(), gw.cpu().double()
        for t in range(z.shape[0]):
            assert set(gi[t].tolist()) == set(idx[t].tolist())
            a = dict(zip(gi[t].tolist(), gw[t].tolist()))
            for e, w in zip(idx[t].tolist(), wt[t].tolist()):
                assert abs(a[e] - w) < 1e-6
        del sd


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
        # these weights are sharp (peaked attention, near-tied routers), so single
        # rows move a lot under 16-bit rounding: the typical row is what is pinned
        assert rel_err(got, want, 0.5) < 0.15 and rel_err(got, want, 0.25) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2, 7], [16], [17, 1, 1, 30], [5, 64]],
                         ids=lambda c: "x".join(map(str, c)))
def test_portions_and_decode(device, cuts, full_model):
    """Token-by-token decoding and portions of any size (down to two tokens,
    across page borders at 16) give the whole prompt's logits."""
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
    """A sequence that takes over a long-decayed state slot and used pages
    starts from nothing."""
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


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_stands_out(device):
    """One key hundreds of tokens back carries the answer: the query weights
    are tied to the key path so that the last token (a repeat of the far one)
    scores that key far above all others. Losing it changes the logits."""
    cfg = O.make_config([(O.latent(heads=2, dim=16, rot_dim=4, vdim=16, kv_rank=16, scale=3.0),
                          None)], width=32, vocab=300)
    sd = O.make_weights(cfg, 7)
    m = cfg["layers"][0]["mixer"]
    sd["l0.mix.dkv.norm"] = torch.ones(16, dtype=torch.bfloat16)
    sd["l0.mix.sink"] = torch.full((2,), -4.0, dtype=torch.bfloat16)
    sd["l0.norm1"] = torch.ones(32, dtype=torch.bfloat16)
    sd["l0.norm1.b"] = torch.zeros(32, dtype=torch.bfloat16)
    # unit key up-projection: the unrotated keys are the (unit-RMS) latents, so
    # among equal-length keys the one parallel to the query scores highest
    sd["l0.mix.uk"] = torch.eye(16).repeat(2, 1).to(torch.bfloat16)
    wq = sd["l0.mix.q"].float().view(2, 20, 32)
    for h in range(2):     # q_unrotated(x) = W_dkv flip(x): parallel to the key of flip(x)
        wq[h, :16] = sd["l0.mix.dkv"].float()[:16].flip(1)
        wq[h, 16:] = 0
    sd["l0.mix.q"] = wq.view(40, 32).to(torch.bfloat16)
    toks = list(range(1, 231))                 # all different
    far, probe = 3, 298                        # the far key sits within the first page
    sd["embed"][probe] = sd["embed"][toks[far]].flip(0)
    toks.append(probe)
    want = O.forward(cfg, sd, toks)[-1:]
    other = list(toks)
    other[far] = 299
    moved = O.forward(cfg, sd, other)[-1:]
    assert rel_err(moved.float(), want) > 0.2             # the far key matters
    for cuts in ([len(toks)], [200, 30, 1], [7]):
        eng = engine(cfg, sd, device, max_tokens=256)
        got = feed(eng, eng.open_sequence(), toks, cuts)[-1:]
        assert rel_err(got, want) < TOL[torch.float32], cuts
    assert m["heads"] == 2


@pytest.mark.parametrize("device", DEVICES)
def test_sink_counts_once(device):
    """A large sink drains most of the attention mass; leaving it out, scaling
    it or counting it per key would change the logits by far more than the
    tolerance."""
    layer = (O.latent(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=8), None)
    cfg = O.make_config([layer], width=24, vocab=50)
    sd = O.make_weights(cfg, 9)
    sd["l0.mix.sink"] = torch.tensor([6.0, 3.0], dtype=torch.bfloat16)
    toks = tokens(40, 50, 2)
    want = O.forward(cfg, sd, toks)
    no_sink = dict(sd)
    no_sink["l0.mix.sink"] = torch.tensor([-30.0, -30.0], dtype=torch.bfloat16)
    assert rel_err(O.forward(cfg, no_sink, toks).float(), want) > 0.05
    eng = engine(cfg, sd, device)
    assert rel_err(feed(eng, eng.open_sequence(), toks, [9, 1]), want) < TOL[torch.float32]


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_state(device):
    """150 single-token steps: the lightning state (one head without decay,
    one forgetting fast) and the latent pages stay exact."""
    cfg = O.make_config([(O.lightning_layer(heads=2, dim=8, vdim=8, decay=[1.0, 0.4]), None),
                         (O.latent(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=8), O.dense(16))],
                        width=24, vocab=60)
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
def test_prompt_path_matches_folded_attention(full_model):
    """bf16 on the GPU: prompt passes run latent attention on per-head keys and
    values (head sizes padded to the kernel's) while short feeds read the latent
    pages directly; both agree with each other within 16-bit rounding, for
    whole prompts, portions on top of a cached context and an unequal batch."""
    from loqa_hub_amd.models.pipizen import PipizenModel
    cfg = O.make_config([(O.latent(heads=3, dim=16, rot_dim=8, vdim=12, kv_rank=32), None),
                         (O.latent(heads=3, dim=16, rot_dim=8, vdim=12, kv_rank=32, kv_from=0),
                          O.dense(64)),
                         (O.latent(heads=2, dim=96, rot_dim=32, vdim=128, kv_rank=64, scaling=False),
                          None)], width=64, vocab=100)
    sd = O.make_weights(cfg, 5)
    a, b = tokens(150, 100, 1), tokens(40, 100, 2)
    want_a, want_b = O.forward(cfg, sd, a), O.forward(cfg, sd, b)
    outs = {}
    for name, min_q in (("prompt", 1), ("folded", 10 ** 9)):
        eng = engine(cfg, sd, "cuda", torch.bfloat16, max_tokens=256)
        assert "prompt_sizes" in eng.weights.layers[0]
        eng.model.prompt_min_q = min_q
        sa, sb = eng.open_sequence(), eng.open_sequence()
        got_a = [eng.step_logits([sa], [a[:70]], [list(range(70))])]
        o = eng.step_logits([sa, sb], [a[70:133], b[:39]], [list(range(63)), list(range(39))])
        got_a.append(o[:63])
        got_b = [o[63:]]
        o = eng.step_logits([sa, sb], [a[133:], b[39:]], [list(range(17)), [0]])
        got_a.append(o[:17])
        got_b.append(o[17:])
        outs[name] = (torch.cat(got_a), torch.cat(got_b))
    assert PipizenModel.prompt_min_q > 1
    for i, want in enumerate((want_a, want_b)):
        assert rel_err(outs["prompt"][i], outs["folded"][i].double().cpu(), 0.9) < 0.05
        assert rel_err(outs["prompt"][i], want, 0.5) < 0.06
        assert rel_err(outs["folded"][i], want, 0.5) < 0.06


@pytest.mark.gpu
@pytest.mark.parametrize("T,d,F", [(333, 96, 64), (700, 128, 192), (2100, 64, 64)],
                         ids=["direct", "staged", "staged_many_rows"])
def test_grouped_expert_gemm_matrix_cores(T, d, F):
    """The bf16 grouped expert GEMMs on the matrix cores (K a multiple of 32;
    prompt-sized batches stage the token rows in LDS) against the f32
    reference: unequal expert loads, an empty expert, identity experts,
    segments that do not fill a tile."""
    from loqa_hub_amd.ops import reference as ref
    from loqa_hub_amd.ops import seqmix
    g = torch.Generator().manual_seed(3)
    E, top = 7, 3
    h = torch.randn(T, d, generator=g).to(torch.bfloat16)
    wgu = (torch.randn(E, 2 * F, d, generator=g) / d ** 0.5).to(torch.bfloat16)
    wd = (torch.randn(E, d, F, generator=g) / F ** 0.5).to(torch.bfloat16)
    idx = torch.randint(0, E + 2, (T, top), generator=g).to(torch.int32)
    idx[idx == 4] = 5                                      # expert 4 gets nothing
    wt = torch.rand(T, top, generator=g)
    want = ref.moe_experts(h.float(), idx, wt, wgu.float(), wd.float(), torch.float32)
    got = seqmix.moe_experts(h.cuda(), idx.cuda(), wt.cuda(), wgu.cuda(), wd.cuda()).cpu()
    err = (got - want).abs().max() / want.abs().max()
    assert err < 2e-2, float(err)


@pytest.mark.gpu
@pytest.mark.parametrize("B", [1, 6, 24], ids=["narrow_blocks", "medium_blocks", "wide_blocks"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_lightning_scan_kernel_widths(B, dtype):
    """The scan kernel's column-block width follows the batch (8 / 16 / 32
    columns per workgroup): each against the f32 reference, with unequal
    sequences, a second step on top of the carried state, and slots in
    scrambled order."""
    from loqa_hub_amd.ops import reference as ref
    from loqa_hub_amd.ops import seqmix
    g = torch.Generator().manual_seed(B)
    H, D, Dv = 8, 16, 40
    n = 2 * H * D + 2 * H * Dv                       # q | k | v | gate columns
    slots = torch.randperm(B + 3, generator=g)[:B].to(torch.int32)
    decay = torch.linspace(0.3, 1.0, H)
    st_ref = torch.zeros(B + 3, H, D, Dv)
    st_gpu = st_ref.clone().cuda()
    pos0 = torch.zeros(B, dtype=torch.long)
    for lens in ([int(x) for x in torch.randint(1, 50, (B,), generator=g)], [1] * B):
        cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32)
        T = int(cu[-1])
        positions = torch.cat([pos0[b] + torch.arange(lens[b]) for b in range(B)]).to(torch.int32)
        qkv = (torch.randn(T, n, generator=g) * 0.7).to(dtype)
        want = ref.lightning_scan(qkv, H, D, Dv, st_ref, slots, cu, positions, decay)
        got = seqmix.lightning_scan(qkv.cuda(), H, D, Dv, st_gpu, slots.cuda(), cu.cuda(),
                                    positions.cuda(), decay.cuda())
        scale = want.abs().max()
        assert (got.cpu() - want).abs().max() / scale < 1e-5
        pos0 += torch.tensor(lens)
    assert (st_gpu.cpu() - st_ref).abs().max() / st_ref.abs().max() < 1e-5
