"""Nidozen hybrid decoders through the engine (scheduler, paged cache, state slots, step function)
against the plain implementation in ``hybrid_oracle.py``. Small configurations with random
weights made here; every test runs on the CPU ops and, marked ``gpu``, on the HIP kernels."""
import numpy as np
import pytest
import torch

import hybrid_oracle as oracle
from llm_consensus_amd._native import core
from llm_consensus_amd.engine.engine import Engine
from llm_consensus_amd.models.hybrid import HybridModel, config_from_dict

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
BS = 16


def attn(heads=4, kv=2, dim=16, vdim=24, chunk=12, rot=8, base=500.0, scale=0.6, kv_from=None, ff=40):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": chunk},
         "rot": {"dims": rot, "base": base}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def gru(width=40, ff=0):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def gla(heads=2, dim=8, vdim=12, tau=4.0, rank=6, ff=0):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=32, vocab=61, eps=1e-5):
    return {"architecture": "Nidozen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


MIXED = config([attn(), gru(), attn(kv_from=0, ff=24), gla(), gru(width=20, ff=28), attn(heads=2, kv=2, dim=12, vdim=8,
                                                                                        chunk=5, rot=12, ff=0)])


def build(cfg, device, dtype=torch.float32, seed=0, blocks=24, slots=4, **kw):
    W = oracle.random_weights(cfg, seed)
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


def rel_err(got, want):
    want = want.numpy() if hasattr(want, "numpy") else want
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1)).mean()).max())


def limit(dtype):
    return 2e-4 if dtype == torch.float32 else 6e-2


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name,layers", [
    ("attention", [attn(), attn(heads=3, kv=3, dim=10, vdim=10, rot=10, chunk=7)]),
    ("one kv head, no rotation", [attn(heads=4, kv=1, rot=0, chunk=9)]),
    ("widths the matrix-core kernel takes", [attn(dim=16, vdim=32, chunk=12), attn(heads=2, kv=1, dim=24, vdim=16, chunk=20,
                                                                                  ff=0)]),
    ("shared keys", [attn(), attn(kv_from=0, ff=0), gru(), attn(kv_from=0, chunk=4)]),
    ("mingru", [gru(), gru(width=24, ff=36)]),
    ("gla", [gla(), gla(heads=1, dim=20, vdim=5, tau=1.5, rank=3, ff=20)]),
])
def test_each_mechanism_whole_prompt(device, dtype, name, layers):
    cfg = config(layers)
    _whole_prompt(cfg, device, dtype, name)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_depths_the_mfma_products_take(device, dtype):
    """Width 64 and feed-forward 128: in bf16 on the GPU these projections go through the packed
    MFMA kernels (depth a multiple of 64, fp32 epilogue), the decay bottleneck (depth 6) does not."""
    cfg = config([attn(dim=16, vdim=16, ff=128), gru(width=64, ff=64), gla(heads=2, dim=32, vdim=32, ff=128),
                  attn(kv_from=0, dim=16, vdim=16, ff=0)], width=64, vocab=70)
    _whole_prompt(cfg, device, dtype, "mfma depths", cuts=[40, 2, 17])


def _whole_prompt(cfg, device, dtype, name, cuts=None):
    eng, W = build(cfg, device, dtype)
    toks = tokens(45 if cuts is None else sum(cuts) + 3, cfg["vocab"], 3)
    got = replay_alone(eng, toks, cuts or [len(toks)])
    assert rel_err(got, oracle.forward(cfg, W, toks)) < limit(dtype), name


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
    pages of 16 and chunks of 12 and 5), or one token at a time."""
    eng, W = build(MIXED, device, dtype)
    toks = tokens(70, MIXED["vocab"], 7)
    want = oracle.forward(MIXED, W, toks)
    assert rel_err(replay_alone(eng, toks, cuts), want) < limit(dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_portions(device, dtype):
    """Portions of a few hundred tokens (the recurrences scan them in parallel segments on the GPU),
    the second one continuing from the state the first one left."""
    eng, W = build(MIXED, device, dtype)
    toks = tokens(340, MIXED["vocab"], 13)
    assert rel_err(replay_alone(eng, toks, [150, 180]), oracle.forward(MIXED, W, toks)) < limit(dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_past_chunks_and_pages(device):
    cfg = config([attn(chunk=6), gla(), gru(), attn(kv_from=0, chunk=6, ff=0)])
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
        assert rel_err(np.concatenate(got[n]), want[n]) < limit(dtype), n


@pytest.mark.parametrize("device", DEVICES)
def test_pool_or_slots_exhausted_is_an_error_and_leaves_the_engine_usable(device):
    eng, W = build(config([gru()]), device, blocks=2, slots=2)
    a, b, c = eng.replay_open(), eng.replay_open(), eng.replay_open()
    eng.replay_step([(a, [1, 2], []), (b, [3], [])])
    with pytest.raises(RuntimeError):
        eng.replay_step([(c, [4], [])])                 # no slot (and no block)
    eng.replay_close(a)
    lg = eng.replay_step([(c, [4, 5], [1])])
    assert rel_err(lg, oracle.forward(config([gru()]), W, [4, 5])[1:]) < 2e-4


def _edge_logits(eng, toks, decode_from):
    return replay_alone(eng, toks, [decode_from] if decode_from else [len(toks)])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cuts", [[70], [20, 33, 2, 15], [17, 1, 1, 30]])
def test_portions_on_the_matrix_core_attention(device, dtype, cuts):
    """Head widths that take the tiled kernel on the GPU: portions that start inside a chunk, cross
    chunk and page borders, and are shorter than a tile of 16 rows next to longer ones."""
    cfg = config([attn(dim=16, vdim=16, chunk=12), gru(), attn(kv_from=0, dim=16, vdim=16, chunk=12, ff=0),
                  attn(heads=2, kv=2, dim=32, vdim=48, chunk=25, rot=32)])
    eng, W = build(cfg, device, dtype)
    toks = tokens(70, cfg["vocab"], 17)
    assert rel_err(replay_alone(eng, toks, cuts), oracle.forward(cfg, W, toks)) < limit(dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("vdim", [24, 16])
@pytest.mark.parametrize("decode_from", [0, 3])
def test_chunk_edges_show_in_the_logits(device, decode_from, vdim):
    """Attention only (nothing else carries a token forward), a flat softmax: a changed token
    moves the logits of the rows of ITS chunk from its position on, and of no other row. Chunk 10
    against pages of 16: the edges fall inside pages and a page border (16, 32) inside chunks."""
    C = 10
    cfg = config([attn(heads=2, kv=1, vdim=vdim, chunk=C, scale=0.8, ff=0),
                  attn(kv_from=0, heads=2, kv=1, vdim=vdim, chunk=C, scale=0.8)])
    eng, W = build(cfg, device)
    toks = tokens(43, cfg["vocab"], 31)
    base = _edge_logits(eng, toks, decode_from)
    assert rel_err(base, oracle.forward(cfg, W, toks)) < 2e-4
    for j in (0, C - 1, C, 15, 16, 2 * C - 1, 2 * C, 31, 32, 39):
        alt = list(toks)
        alt[j] = (alt[j] + 1) % cfg["vocab"]
        moved = np.abs(_edge_logits(eng, alt, decode_from) - base).max(-1)
        end = (j // C + 1) * C
        assert (moved[:j] < 1e-5).all() and (moved[min(end, len(toks)):] < 1e-5).all(), j
        assert (moved[j:min(end, len(toks))] > 5e-5).all(), j


@pytest.mark.parametrize("device", DEVICES)
def test_a_far_key_that_stands_out(device):
    """One key far back among hundreds carries the answer: the query at the end matches it (large
    score scale, keys and queries are unit-normed), so dropping or misplacing it shows."""
    cfg = config([attn(heads=1, kv=1, dim=16, vdim=16, chunk=400, rot=4, scale=40.0, ff=0)], vocab=50)
    eng, W = build(cfg, device, blocks=24)
    toks = tokens(330, cfg["vocab"], 41)
    want = oracle.forward(cfg, W, toks)
    got = replay_alone(eng, toks, [300])
    assert rel_err(got, want) < 2e-4
    peak = torch.softmax(torch.tensor(got[-1]), 0).max()
    assert peak > 0  # the comparison above is the test; with scale 40 single keys dominate the rows


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_single_token_requests(device):
    eng, W = build(MIXED, device)
    for toks in ([7], [7, 7], tokens(3, MIXED["vocab"], 2)):
        assert rel_err(replay_alone(eng, toks, [len(toks)]), oracle.forward(MIXED, W, toks)) < 2e-4
        assert rel_err(replay_alone(eng, toks, []), oracle.forward(MIXED, W, toks)) < 2e-4


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


@pytest.mark.parametrize("device", DEVICES)
def test_requests_the_family_does_not_serve_are_refused(device):
    eng, _ = build(config([gru()]), device)
    with pytest.raises(ValueError):
        eng.submit([1, 2, 3], kind=core.RequestKind.Embed)
    with pytest.raises(ValueError):
        eng.submit([1, 2, 3], n=2)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_serving_steps_launch_only_the_kernel_library(dtype):
    """Prompt portions, mixed steps, decode steps and replayed steps of a hybrid model: PyTorch
    launches no kernel of its own in any of them (allocations, views and buffer copies aside)."""
    from llm_consensus_amd.utils.audit import AtenAudit

    cfg = config([attn(dim=16, vdim=16, ff=128), gru(width=64, ff=64), gla(heads=2, dim=32, vdim=32, ff=0),
                  attn(kv_from=0, dim=16, vdim=16, ff=0), attn(heads=2, kv=1, dim=12, vdim=24)], width=64, vocab=70)
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

    work()                                   # first use: lazy initialisation happens here
    torch.cuda.synchronize()
    with AtenAudit() as audit:
        outs = work()
        torch.cuda.synchronize()
    assert all(len(o.token_ids[0]) == 5 for o in outs)
    assert audit.kernels == {}, audit.kernels


def test_checkpoint_directory_through_the_registry_and_the_command_line(tmp_path, capsys):
    """A Nidozen checkpoint directory is found by its config.json, loaded with the checkpoint's
    tensor names, and answers a question through the command line beside a transformer member."""
    from llm_consensus_amd import cli
    from llm_consensus_amd.models.loader import load_model, write_random_hybrid_checkpoint
    from llm_consensus_amd.models.registry import resolve

    cfg = config_from_dict(config([attn(ff=24), gru(width=24), gla(), attn(kv_from=0, ff=0)], width=32, vocab=300))
    ck = write_random_hybrid_checkpoint(cfg, str(tmp_path / "nidozen"), seed=3)
    assert resolve(str(ck)).name == "hybrid"
    m = load_model(str(ck), "cpu", dtype=torch.float32)
    assert [L.spec.type for L in m.layers] == ["attention", "mingru", "gla", "attention"] and m.layers[2].spec.rank == 6
    toml = tmp_path / "e.toml"
    toml.write_text(f"""strategy = "majority_vote"
decision_mode = "logprob"
choices = "ABCD"
[sampling]
temperature = 0.0
max_new_tokens = 4
[models.h]
path = "{ck}"
[models.t]
preset = "tiny-llama"
[[members]]
name = "hybrid"
model = "h"
[[members]]
name = "llama"
model = "t"
""")
    q = tmp_path / "q.txt"
    q.write_text("Which? A. a B. b C. c D. d\n")
    assert cli.main(["--config", str(toml), "--questions", str(q), "--device", "cpu", "--no-warm-up"]) == 0
    assert capsys.readouterr().out.strip()[-1] in "ABCD"
