"""Telurax hybrid decoders through the engine (scheduler, paged cache, state slots, step function)
against the plain implementation in ``telurax_oracle.py``. Small configurations with random weights
made here; every test runs on the CPU ops and, marked ``gpu``, on the HIP kernels."""
import json
import math
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import telurax_oracle as oracle
from llm_consensus_amd._native import core
from llm_consensus_amd.engine.engine import Engine
from llm_consensus_amd.models.hybrid import DESIGNS, HybridModel, config_from_dict, config_to_dict
from llm_consensus_amd.models.registry import HYBRID_DESIGNS

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
BS = 16
ROOT = Path(__file__).resolve().parents[1]


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, identity=2, top=3, groups=4, keep=2, scale=1.5, ff=20, shared=24):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "identity": identity, "top": top, "scale": scale,
                       "groups": {"count": groups, "keep": keep}},
            "shared": {"ff": shared} if shared else None}


def latent(heads=3, dim=12, vdim=20, rank=24, scale=0.4, mlp=None):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale},
            "mlp": mlp}


def mlstm(heads=2, dim=10, vdim=14, cap=8.0, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": mlp}


def config(layers, width=40, vocab=67, eps=1e-5, embed_scale=0.7, logit_scale=0.3):
    return {"architecture": "Telurax", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": embed_scale}, "logit_scale": logit_scale, "layers": layers}


MIXED = config([latent(mlp=moe()), mlstm(mlp=dense()), mlstm(heads=1, dim=16, vdim=8, cap=3.0), latent(heads=2, dim=8, vdim=8, rank=16, mlp=dense(24)),
                mlstm(heads=3, dim=6, vdim=10, mlp=moe(experts=5, identity=0, top=2, groups=1, keep=1, shared=0))])


def build(cfg, device, dtype=torch.float32, seed=0, blocks=24, slots=4, weights=None, **kw):
    W = weights if weights is not None else oracle.random_weights(cfg, seed)
    model = HybridModel(config_from_dict(cfg, "test", {k: tuple(v.shape) for k, v in W.items()}), device, dtype)
    model.set_weights(lambda n: W[n])
    eng = Engine(model, num_kv_blocks=blocks, block_size=BS, max_batch_seqs=kw.pop("max_batch_seqs", slots),
                 state_slots=slots, max_model_len=blocks * BS, enable_prefix_cache=False,
                 use_graphs=kw.pop("use_graphs", False), pipeline_decode=kw.pop("pipeline_decode", False), **kw)
    return eng, W


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def replay_alone(eng, toks, cuts):
    """One request fed in portions of the given sizes (the rest one token at a time); all logits."""
    rid, at, out = eng.replay_open(), 0, []
    sizes = list(cuts) + [1] * (len(toks) - sum(cuts))
    for n in sizes:
        out.append(eng.replay_step([(rid, toks[at:at + n], list(range(n)))]))
        at += n
    eng.replay_close(rid)
    return np.concatenate(out)


def rel_err(got, want, close_calls=0):
    """Largest row error (mean taken off, RMS over the vocabulary, against the mean RMS of the wanted
    rows). ``close_calls``: that many of the worst rows are left out: in bf16 a router's close call
    can go the other way for a token, which changes that row for good and no other."""
    want = want.numpy() if hasattr(want, "numpy") else want
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    rows = np.sort(np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1)).mean())
    return float(rows[:len(rows) - close_calls].max() if close_calls < len(rows) else 0.0)


def calls(dtype, rows):
    return 0 if dtype == torch.float32 else max(1, rows // 25)


def limit(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


def _whole_prompt(cfg, device, dtype, name, cuts=None, seed=0):
    eng, W = build(cfg, device, dtype, seed=seed)
    toks = tokens(45 if cuts is None else sum(cuts) + 3, cfg["vocab"], 3)
    got = replay_alone(eng, toks, cuts or [len(toks)])
    assert rel_err(got, oracle.forward(cfg, W, toks), calls(dtype, len(toks))) < limit(dtype), name


def test_the_registry_names_the_designs_of_the_model_code():
    assert set(HYBRID_DESIGNS) == set(DESIGNS)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name,layers", [
    ("latent attention", [latent(), latent(heads=1, dim=7, vdim=5, rank=9, scale=1.1)]),
    ("latent widths the matrix-core kernel takes", [latent(heads=4, dim=16, vdim=16, rank=32), latent(heads=2, dim=8, vdim=24, rank=16)]),
    ("latent wider than a wave", [latent(heads=2, dim=8, vdim=8, rank=72)]),
    ("latent wider than the width", [latent(heads=2, dim=8, vdim=8, rank=300)]),
    ("mlstm", [mlstm(), mlstm(heads=3, dim=5, vdim=33, cap=2.0)]),
    ("mlstm without a cap, one head", [mlstm(heads=1, dim=40, vdim=3, cap=0.0)]),
    ("gated dense feed-forward", [mlstm(mlp=dense()), latent(mlp=dense(9))]),
    ("routed feed-forward", [latent(mlp=moe()), mlstm(mlp=moe(experts=7, identity=1, top=1, groups=2, keep=1, scale=2.5, shared=0))]),
    ("routed: no identity experts, one group", [mlstm(mlp=moe(experts=4, identity=0, top=4, groups=1, keep=1, ff=8, shared=8))]),
    ("routed: every group kept, many experts", [latent(mlp=moe(experts=66, identity=4, top=5, groups=7, keep=7, ff=4))]),
])
def test_each_mechanism_whole_prompt(device, dtype, name, layers):
    _whole_prompt(config(layers), device, dtype, name)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_depths_the_mfma_products_take(device, dtype):
    """Width 64 and feed-forwards of 128 / 64: in bf16 on the GPU the dense projections go through the packed
    MFMA kernels (depth a multiple of 64, fp32 epilogue)."""
    cfg = config([latent(heads=2, dim=32, vdim=32, rank=64, mlp=dense(128)), mlstm(heads=2, dim=32, vdim=32, mlp=moe(ff=64, shared=64)),
                  latent(heads=4, dim=16, vdim=16, rank=32, mlp=moe(shared=0))], width=64, vocab=70)
    _whole_prompt(cfg, device, dtype, "mfma depths", cuts=[40, 2, 17])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_deep_products_whose_outputs_are_no_multiple_of_32(device, dtype):
    """Width 1024: deep enough that the bf16 MFMA products of a few rows (and of a few hundred) split
    their depth over workgroups, while the fused projections, the vocabulary and the router have
    widths like 90 or 179. A long portion, a short one and decoded tokens."""
    cfg = config([latent(heads=3, dim=16, vdim=16, rank=32, mlp=moe(ff=64, shared=64)), mlstm(heads=2, dim=16, vdim=24, mlp=dense(64))],
                 width=1024, vocab=90)
    eng, W = build(cfg, device, dtype, blocks=24)
    toks = tokens(300, cfg["vocab"], 3)
    got = replay_alone(eng, toks, [270, 20])
    assert rel_err(got, oracle.forward(cfg, W, toks), calls(dtype, len(toks))) < limit(dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_constants_that_could_pass_for_one(device):
    """Scales of 1, an offset norm whose weights are far from zero, a large eps: none is assumed."""
    cfg = config([latent(scale=1.0, mlp=moe(scale=1.0)), mlstm(mlp=dense())], eps=0.05, embed_scale=1.0, logit_scale=1.0)
    W = oracle.random_weights(cfg, 4)
    for k in W:
        if k.endswith(("norm1", "norm2")) or k == "final.norm":
            W[k] = (W[k].float() * 5 - 0.5).to(W[k].dtype)
    eng, _ = build(cfg, device, weights=W)
    toks = tokens(30, cfg["vocab"], 9)
    assert rel_err(replay_alone(eng, toks, [17]), oracle.forward(cfg, W, toks)) < 2e-4
    other = config(cfg["layers"], eps=0.05, embed_scale=2.0, logit_scale=0.25)
    eng2, _ = build(other, device, weights=W)
    assert rel_err(replay_alone(eng2, toks, [17]), oracle.forward(other, W, toks)) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_residual_stream_after_every_layer(device):
    eng, W = build(MIXED, device)
    toks = tokens(20, MIXED["vocab"], 5)
    taps, rid = [], eng.replay_open()
    eng.replay_step([(rid, toks, [])], taps=taps)
    _, want = oracle.forward(MIXED, W, toks, return_layers=True)
    assert len(taps) == len(MIXED["layers"])
    for i, t in enumerate(taps):
        torch.testing.assert_close(t.cpu().double(), want[i], atol=2e-4, rtol=2e-4, msg=f"layer {i}")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cuts", [[], [1], [40], [2, 2, 3, 2, 17, 2], [11, 1, 1, 12, 13], [5, 7, 12, 16, 1, 15, 2]])
def test_portions_and_token_by_token_decoding(device, dtype, cuts):
    """The same logits whether the prompt comes whole, in portions down to two tokens (cut inside
    pages of 16), or one token at a time."""
    eng, W = build(MIXED, device, dtype)
    toks = tokens(70, MIXED["vocab"], 7)
    want = oracle.forward(MIXED, W, toks)
    assert rel_err(replay_alone(eng, toks, cuts), want, calls(dtype, len(toks))) < limit(dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_portions(device, dtype):
    """Portions of a few hundred tokens (the matrix memory scans them in parallel segments on the
    GPU), the second one continuing from the state and the maximum the first one left."""
    cfg = config([mlstm(mlp=dense()), latent(heads=2, dim=8, vdim=8, rank=16), mlstm(heads=1, dim=12, vdim=70, cap=4.0)])
    eng, W = build(cfg, device, dtype, blocks=30)
    toks = tokens(340, cfg["vocab"], 13)
    assert rel_err(replay_alone(eng, toks, [150, 180]), oracle.forward(cfg, W, toks)) < limit(dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_pages(device):
    cfg = config([latent(), mlstm(), latent(heads=2, dim=8, vdim=8, rank=16, mlp=moe())])
    eng, W = build(cfg, device)
    toks = tokens(100, cfg["vocab"], 11)
    assert rel_err(replay_alone(eng, toks, [3]), oracle.forward(cfg, W, toks)) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixed_batches_reused_pages_and_slots(device, dtype):
    """Up to four live requests, portions beside single tokens, in a pool too small for all of
    them at once: requests end, others take their pages and state slots."""
    eng, W = build(MIXED, device, dtype, blocks=12, slots=4)
    V = MIXED["vocab"]
    reqs = {n: tokens(L, V, 20 + i) for i, (n, L) in enumerate([("a", 50), ("b", 33), ("c", 1), ("d", 47), ("e", 40),
                                                                ("f", 18), ("g", 60)])}
    want = {n: oracle.forward(MIXED, W, t).numpy() for n, t in reqs.items()}
    sched = [[("a", 20), ("b", 2)], [("a", 1), ("b", 13), ("c", 1)], [("a", 1), ("b", 1), ("d", 30)],
             [("a", 28), ("d", 1)], [("b", 17), ("d", 16), ("e", 9)], [("e", 1)], [("e", 30), ("f", 18)],
             [("g", 33)], [("g", 1)], [("g", 26)]]
    at, rid, got = {n: 0 for n in reqs}, {}, {n: [] for n in reqs}
    free0 = eng.kvm.stats().blocks_free
    for step in sched:
        entries = []
        for n, k in step:
            if n not in rid:
                rid[n] = eng.replay_open()
            entries.append((rid[n], reqs[n][at[n]:at[n] + k], list(range(k))))
        lg = eng.replay_step(entries)
        o = 0
        for n, k in step:
            got[n].append(lg[o:o + k])
            o += k
            at[n] += k
            if at[n] == len(reqs[n]):
                eng.replay_close(rid[n])
    assert all(at[n] == len(reqs[n]) for n in reqs)
    assert eng.kvm.stats().blocks_free == free0 and eng.kvm.free_state_slots == 4
    for n in reqs:
        assert rel_err(np.concatenate(got[n]), want[n], calls(dtype, len(reqs[n])) if len(reqs[n]) > 1 else 0) < limit(dtype), n


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode_from", [0, 3, 18])
def test_causality_at_every_place_and_page_border(device, decode_from):
    """Attention only (nothing else carries a token forward), a flat softmax: a changed token moves
    the logits of its own row and of every later row, and of no earlier one, whether the rows run as
    a prompt or are decoded one by one. Pages of 16: places 15 / 16 and 31 / 32 are page borders."""
    cfg = config([latent(heads=2, dim=8, vdim=8, rank=16, scale=0.05), latent(heads=1, dim=6, vdim=10, rank=12, scale=0.05)])
    eng, W = build(cfg, device)
    toks = tokens(43, cfg["vocab"], 31)
    cuts = [decode_from] if decode_from else [len(toks)]
    base = replay_alone(eng, toks, cuts)
    assert rel_err(base, oracle.forward(cfg, W, toks)) < 2e-4
    for j in (0, 1, 15, 16, 17, 31, 32, 41, 42):
        alt = list(toks)
        alt[j] = (alt[j] + 1) % cfg["vocab"]
        moved = np.abs(replay_alone(eng, alt, cuts) - base).max(-1)
        assert (moved[:j] < 1e-6).all() and (moved[j:] > 2e-6).all(), j


@pytest.mark.parametrize("device", DEVICES)
def test_a_far_key_that_stands_out(device):
    """One key far back among hundreds carries the answer: with a large score scale single keys
    dominate the softmax rows, so dropping or misplacing one shows. The last rows are decoded."""
    cfg = config([latent(heads=1, dim=16, vdim=16, rank=16, scale=6.0)], vocab=50)
    eng, W = build(cfg, device, blocks=24)
    toks = tokens(330, cfg["vocab"], 41)
    H = oracle.forward(cfg, W, toks)
    assert rel_err(replay_alone(eng, toks, [300]), H) < 2e-4
    # the oracle's own softmax rows are peaked: the test would not pass with a key lost
    Wd = {k: v.double() for k, v in W.items()}
    x = Wd["embed"][toks] * cfg["embedding"]["scale"] + oracle.position_vectors(len(toks), cfg["width"])
    h = oracle.offset_norm(x, Wd["l0.norm1"], 1e-5)
    q = h @ Wd["l0.mix.q"].T
    c = oracle.unit_rms(h @ Wd["l0.mix.dkv"].T, 1e-5) * Wd["l0.mix.dkv.norm"]
    k = c @ Wd["l0.mix.uk"].T
    far = 0
    for i in range(300, len(toks)):                  # the decoded rows
        s = torch.softmax((k[:i + 1] @ q[i]) * 6.0, 0)
        far += int(float(s.max()) > 0.5 and int(s.argmax()) < 250)
    assert far >= 5


@pytest.mark.parametrize("device", DEVICES)
def test_the_memory_reaches_back_to_the_first_tokens(device):
    """mLSTM only, forget gates held open: the first token still moves the last logits after 150
    decoded tokens, and the engine agrees with the plain recurrence over all of them."""
    cfg = config([mlstm(heads=2, dim=8, vdim=8, cap=15.0)])
    W = oracle.random_weights(cfg, 2)
    W["l0.mix.f.b"] = torch.full_like(W["l0.mix.f.b"], 9.0)
    W["l0.mix.f"] = W["l0.mix.f"] * 0
    eng, _ = build(cfg, device, weights=W)
    toks = tokens(160, cfg["vocab"], 6)
    base = replay_alone(eng, toks, [10])
    assert rel_err(base, oracle.forward(cfg, W, toks)) < 2e-4
    alt = [(toks[0] + 1) % cfg["vocab"]] + toks[1:]
    assert np.abs(replay_alone(eng, alt, [10])[-1] - base[-1]).max() > 1e-4


@pytest.mark.parametrize("device", DEVICES)
def test_routing_choices_that_groups_and_corrections_decide(device):
    """Corrections large enough to change the choice, all of them negative (a group that is not kept
    must count as minus infinity, not as zero), and groups that exclude the best single expert of
    some token: the oracle's own choices confirm that each rule decides something here."""
    mlp = moe(experts=9, identity=3, top=3, groups=4, keep=2, scale=0.8)
    cfg = config([mlstm(mlp=mlp)])
    W = oracle.random_weights(cfg, 8)
    gen = torch.Generator().manual_seed(1)
    W["l0.mlp.correction"] = (-1.0 + 0.3 * torch.rand(12, generator=gen)).to(torch.bfloat16)
    eng, _ = build(cfg, device, weights=W)
    toks = tokens(60, cfg["vocab"], 12)
    assert rel_err(replay_alone(eng, toks, [40]), oracle.forward(cfg, W, toks)) < 2e-4
    Wd = {k: v.double() for k, v in W.items()}
    x = Wd["embed"][toks] * cfg["embedding"]["scale"] + oracle.position_vectors(len(toks), cfg["width"])
    x = x + oracle.mlstm(oracle.offset_norm(x, Wd["l0.norm1"], 1e-5), Wd, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    h = oracle.offset_norm(x, Wd["l0.norm2"], 1e-5)
    full = oracle.route(h, Wd, "l0.mlp.", mlp["router"])[0].sort(-1).values
    assert (full != oracle.route(h, Wd, "l0.mlp.", mlp["router"], use_groups=False)[0].sort(-1).values).any()
    assert (full != oracle.route(h, Wd, "l0.mlp.", mlp["router"], use_correction=False)[0].sort(-1).values).any()
    assert (full >= 9).any()                          # identity experts are chosen too


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_single_token_requests(device):
    eng, W = build(MIXED, device)
    for toks in ([7], [7, 7], tokens(3, MIXED["vocab"], 2)):
        assert rel_err(replay_alone(eng, toks, [len(toks)]), oracle.forward(MIXED, W, toks)) < 2e-4
        assert rel_err(replay_alone(eng, toks, []), oracle.forward(MIXED, W, toks)) < 2e-4


@pytest.mark.parametrize("device", DEVICES)
def test_pool_or_slots_exhausted_is_an_error_and_leaves_the_engine_usable(device):
    cfg = config([mlstm()])
    eng, W = build(cfg, device, blocks=2, slots=2)
    a, b, c = eng.replay_open(), eng.replay_open(), eng.replay_open()
    eng.replay_step([(a, [1, 2], []), (b, [3], [])])
    with pytest.raises(RuntimeError):
        eng.replay_step([(c, [4], [])])
    eng.replay_close(a)
    lg = eng.replay_step([(c, [4, 5], [1])])
    assert rel_err(lg, oracle.forward(cfg, W, [4, 5])[1:]) < 2e-4


def _greedy_oracle(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(oracle.forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_submit_and_the_scheduler(device, graphs):
    """More requests than state slots, prompts cut by the scheduler's token budget, decoding
    chains riding in the steps that prefill later prompts; recorded decode steps on the GPU."""
    if graphs and device == "cpu":
        pytest.skip("decode graphs are a GPU feature")
    eng, W = build(MIXED, device, blocks=40, slots=3, max_batch_seqs=3, max_prefill_tokens=24, use_graphs=graphs,
                   pipeline_decode=graphs)
    p = core.SamplingParams()
    p.temperature, p.max_new_tokens, p.ignore_eos = 0.0, 9, True
    prompts = [tokens(n, MIXED["vocab"], 50 + n) for n in (30, 5, 41, 1, 17)]
    rids = [eng.submit(pr, params=p) for pr in prompts]
    eng.run_until_done()
    for rid, pr in zip(rids, prompts):
        out = eng.pop_result(rid)
        assert out.token_ids[0] == _greedy_oracle(MIXED, W, pr, 9)
    assert eng.kvm.free_state_slots == 3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_serving_steps_launch_only_the_kernel_library(dtype):
    """Prompt portions, mixed steps, decode steps and replayed steps: PyTorch launches no kernel of
    its own in any of them (allocations, views and buffer copies aside)."""
    from llm_consensus_amd.utils.audit import AtenAudit

    cfg = config([latent(heads=2, dim=32, vdim=32, rank=64, mlp=dense(128)), mlstm(heads=2, dim=32, vdim=32, mlp=moe(ff=64, shared=64)),
                  latent(mlp=moe(shared=0)), mlstm()], width=64, vocab=70)
    eng, _ = build(cfg, "cuda:0", dtype, blocks=40, slots=3, max_batch_seqs=3, max_prefill_tokens=24)
    p = core.SamplingParams()
    p.temperature, p.max_new_tokens, p.ignore_eos = 0.7, 5, True

    def work():
        rids = [eng.submit(tokens(n, cfg["vocab"], n), params=p) for n in (30, 5, 41)]
        eng.run_until_done()
        rid = eng.replay_open()
        eng.replay_step([(rid, tokens(20, cfg["vocab"], 1), [0, 19])])
        eng.replay_step([(rid, [3], [0])])
        eng.replay_close(rid)
        return [eng.pop_result(r) for r in rids]

    work()
    torch.cuda.synchronize()
    with AtenAudit() as audit:
        outs = work()
        torch.cuda.synchronize()
    assert all(len(o.token_ids[0]) == 5 for o in outs)
    assert audit.kernels == {}, audit.kernels


def test_checkpoint_directory_through_the_registry_the_trace_tool_and_the_command_line(tmp_path, capsys):
    """A Telurax checkpoint directory is found by its config.json, loaded with the checkpoint's tensor
    names, replayed by ``bin/trace_run`` (two requests in one step, a request that ends and one that
    goes on) and answers a question through the command line."""
    from safetensors.torch import save_file

    from llm_consensus_amd import cli
    from llm_consensus_amd.models.loader import load_model
    from llm_consensus_amd.models.registry import resolve

    cfg = config([latent(mlp=moe()), mlstm(mlp=dense()), latent(heads=2, dim=8, vdim=8, rank=16)], width=32, vocab=300)
    W = oracle.random_weights(cfg, 3)
    ck = tmp_path / "telurax"
    ck.mkdir()
    (ck / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in W.items()}, str(ck / "model.safetensors"))
    assert resolve(str(ck)).name == "hybrid"
    m = load_model(str(ck), "cpu", dtype=torch.float32)
    assert [L.spec.type for L in m.layers] == ["latent_attention", "mlstm", "latent_attention"]
    assert config_to_dict(m.cfg)["layers"][0]["mlp"]["router"] == cfg["layers"][0]["mlp"]["router"]
    a, b = tokens(21, 300, 1), tokens(9, 300, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:17], "want": [0, 16]}, {"id": "b", "tokens": b[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[17:18], "want": [0]}, {"id": "b", "tokens": b[2:], "want": [6]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[18:], "want": [2]}], "end": ["a"]}]
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(ck), "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128", "--device", "cpu"], input="".join(json.dumps(s) + "\n" for s in steps),
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = oracle.forward(cfg, W, a).numpy(), oracle.forward(cfg, W, b).numpy()
    got = [np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, 300) for i in range(3)]
    assert rel_err(got[0], la[[0, 16]]) < 2e-4
    assert rel_err(got[1], np.stack([la[17], lb[8]])) < 2e-4
    assert rel_err(got[2], la[[20]]) < 2e-4
    toml = tmp_path / "e.toml"
    toml.write_text(f"""strategy = "majority_vote"
decision_mode = "logprob"
choices = "ABCD"
[sampling]
temperature = 0.0
max_new_tokens = 4
[models.h]
path = "{ck}"
[[members]]
name = "hybrid"
model = "h"
""")
    q = tmp_path / "q.txt"
    q.write_text("Which? A. a B. b C. c D. d\n")
    assert cli.main(["--config", str(toml), "--questions", str(q), "--device", "cpu", "--no-warm-up"]) == 0
    assert capsys.readouterr().out.strip()[-1] in "ABCD"


def test_random_checkpoint_writer_and_random_init(tmp_path):
    """The family's checkpoint writer and ``random_init`` (benchmarks, stand-ins) know the design's tensors: what
    one writes the loader reads back, and both models answer the same."""
    from llm_consensus_amd.models.loader import load_model, write_random_hybrid_checkpoint

    cfg = config_from_dict(config([mlstm(mlp=moe(shared=0)), latent(mlp=dense()), mlstm(), latent(mlp=moe())], width=24, vocab=80))
    ck = write_random_hybrid_checkpoint(cfg, str(tmp_path / "ck"), seed=7)
    assert json.loads((ck / "config.json").read_text())["architecture"] == "Telurax"
    a = load_model(str(ck), "cpu", dtype=torch.float32)
    b = HybridModel.random_init(cfg, "cpu", seed=7, dtype=torch.float32)
    assert a.cfg.layers == b.cfg.layers and (a.cfg.embed_scale, a.cfg.logit_scale) == (b.cfg.embed_scale, b.cfg.logit_scale)
    out = []
    for m in (a, b):
        eng = Engine(m, num_kv_blocks=8, block_size=BS, max_batch_seqs=2, state_slots=2, max_model_len=8 * BS,
                     enable_prefix_cache=False, use_graphs=False, pipeline_decode=False)
        out.append(replay_alone(eng, tokens(12, 80, 1), [7]))
    assert np.isfinite(out[0]).all() and np.abs(out[0]).max() > 0
    np.testing.assert_allclose(out[0], out[1], rtol=1e-6, atol=1e-6)
