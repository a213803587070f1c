"""Dogidra through the engine: checkpoint folder -> registry -> runner ->
scheduler / block manager / state slots, against the float64 oracle in
tests/oracle_dogidra.py. Every test builds its own small configuration and
random weights. CPU runs the reference ops; gpu-marked variants run the HIP
kernels."""

import json
import os

import pytest
import torch

import oracle_dogidra as O
from dogidra_util import (TOL, close, make_cfg, make_engine, make_weights,
                          mixer, moe, rel_err, save_checkpoint)
from production_stack_amd.engine.models import registry
from production_stack_amd.engine.sampling import SamplingParams

pytestmark = pytest.mark.filterwarnings("ignore::UserWarning")

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = ["float32", "bfloat16"]

# four layers, the middle two run twice (six layer runs): windows of 20 and
# 13 positions with pooled blocks of 4 and 5 (5 does not divide the page of
# 16), rotary on part of a head and on all of it, with and without blended
# frequencies, key width != value width, recurrent widths 40 / 24, layers
# with and without a feed-forward or shared expert, three taps
STACK = [
    (mixer(4, 2, 16, 24, 20, 4, 0.3, 8, 100.0, (4.0, 32, 4.0, 1.0), 15.0, 40),
     moe(24, 5, 2, 1.5, 40)),
    (mixer(6, 3, 8, 8, 13, 5, 0.4, 8, 10000.0, None, 0.0, 24, 1.0, 1.0),
     moe(16, 4, 3, 2.25, 0)),
    (mixer(2, 1, 16, 8, 20, 4, 0.25, 4, 50.0, (2.0, 16, 2.0, 0.5), 22.0, 40,
           0.5, 1.5), None),
    (mixer(4, 4, 16, 16, 33, 16, 0.3, 16, 1000.0, (8.0, 64, 8.0, 1.0), 10.0,
           8), moe(24, 3, 1, 1.0, 24)),
]
LOOP = (1, 3, 2)
RUNS = 6
VOCAB = 97


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    cfg = make_cfg(STACK, width=64, vocab=VOCAB, taps=3, loop=LOOP)
    W = make_weights(cfg, seed=6)
    path = save_checkpoint(tmp_path_factory.mktemp("dg") / "m", cfg, W)
    return path, cfg, W


def tokens(n, seed, vocab=VOCAB):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def replay(eng, rid, toks, sizes):
    """Feed toks in portions of the given sizes (None = the rest); returns
    logits at every position."""
    out, at = [], 0
    for s in sizes:
        s = len(toks) - at if s is None else min(s, len(toks) - at)
        if s <= 0:
            continue
        last = at + s == len(toks)
        out.append(eng.replay_step(
            [(rid, toks[at:at + s], list(range(s)))],
            end=[rid] if last else []))
        at += s
    assert at == len(toks)
    return torch.cat(out)


# ---------------------------------------------------------------------------
def test_registry_reads_checkpoint_folder(ckpt):
    path, cfg, W = ckpt
    mc = registry.config_from_dir(path)
    assert mc.family == "dogidra" and mc.vocab_size == VOCAB
    assert mc.hidden_size == 64 and len(mc.layer_specs) == len(STACK)
    assert mc.has_recurrent_state and mc.loop == LOOP
    assert mc.embedding_scale == 5.0 and mc.tie_word_embeddings
    s0, s1, s2, s3 = mc.layer_specs
    assert s0.norm == "layer" and s0.input_conv == 3 and not s0.parallel
    m0 = s0.mixer
    assert (m0.kind, m0.combine, m0.left_scale, m0.right_scale) == (
        "pair", "weighted", 0.7, 0.6)
    a, b = m0.left, m0.right
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.window,
            a.window_pool, a.scale, a.softcap, a.rot_dims, a.rot_base,
            a.rot_layout, a.rot_scaling) == (
        "attention", 4, 2, 16, 24, 20, 4, 0.3, 15.0, 8, 100.0, "half",
        (4.0, 32.0, 4.0, 1.0))
    assert a.qk_norm_all and a.rope and not a.bias and not a.sink
    assert (b.kind, b.vdim) == ("mingru", 40)
    f0 = s0.mlp
    assert (f0.experts, f0.top, f0.route_scale, f0.shared_ff, f0.correction,
            f0.score, f0.act, f0.gated, f0.shared_gate, f0.renormalize) == (
        5, 2, 1.5, 40, True, "sigmoid", "relu2", False, False, False)
    assert s1.mixer.left.rot_scaling is None and s1.mixer.left.softcap == 0
    assert s1.mlp.shared_ff == 0 and s2.mlp is None
    assert s1.mlp.route_scale == 2.25
    assert "dogidra" in registry.FP32_FAMILIES
    model = registry.build_model(mc, "float32")
    assert [i for i, _ in model.runs] == [0, 1, 2, 1, 2, 3]
    assert [b for _, b in model.runs] == [False, True, False, True, False,
                                          False]
    assert len(model.cache_shapes()) == RUNS


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_prompt_and_every_layer_run(ckpt, device, dtype):
    path, cfg, W = ckpt
    toks = tokens(70, 1)
    layers = []
    want = O.forward(cfg, W, toks, layers)
    eng = make_engine(path, dtype, device)
    seen = {}
    eng.runner.model.residual_hook = lambda i, x: seen.__setitem__(
        i, x.detach().clone())
    got = replay(eng, "a", toks, [None])
    assert close(got, want, dtype)
    assert sorted(seen) == list(range(RUNS)) and len(layers) == RUNS
    for i in range(RUNS):
        assert seen[i].dtype == torch.float32     # fp32 residual stream
        assert close(seen[i], layers[i], dtype), i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens_and_single_token_prompt(ckpt, device, dtype):
    path, cfg, W = ckpt
    eng = make_engine(path, dtype, device)
    for n in (1, 2, 3, 5):
        toks = tokens(n, 10 + n)
        want = O.forward(cfg, W, toks)
        assert close(replay(eng, f"p{n}", toks, [None]), want, dtype)
        assert close(replay(eng, f"q{n}", toks, [1] * n), want, dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [
    [1] * 90, [2] * 45, [3, 2, 17, 2, 31, 2, None], [19, 1, 1, 1, None],
    [20, 20, 13, None], [33, 1, 33, None], [16, 16, 16, 16, 16, None],
    [24, 4, 5, 2, None]])
def test_portions_match_whole_prompt(ckpt, device, dtype, sizes):
    """Prefill against token-by-token decoding, and portions of several
    sizes down to two tokens, cut inside pages, windows and pooled blocks
    and exactly on their edges (windows of 13 / 20 / 33 positions, blocks
    of 4 / 5 / 16, pages of 16, convolutions reaching back over a cut)."""
    path, cfg, W = ckpt
    toks = tokens(90, 2)
    want = O.forward(cfg, W, toks)
    eng = make_engine(path, dtype, device)
    assert close(replay(eng, "a", toks, sizes), want, dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode_past_many_windows_and_blocks(ckpt, device):
    path, cfg, W = ckpt
    toks = tokens(260, 3)
    want = O.forward(cfg, W, toks)
    eng = make_engine(path, "float32", device)
    # a first portion of more than 128 rows routes through the sorted
    # expert dispatch, the single tokens through the all-experts path
    got = replay(eng, "a", toks, [137] + [1] * 123)
    assert rel_err(got, want) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_mixed_batches_reuse_pages_and_slots(ckpt, device, dtype):
    """Up to three live requests of unequal length per step, portions
    beside single tokens; the pool (3 slots, 12 pages) is smaller than the
    sum of all requests, so pages (keys, values, pooled blocks) and slots
    (recurrent state, convolution tails of every layer run) pass from
    finished requests to new ones. Every request must equal itself
    alone."""
    path, cfg, W = ckpt
    lens = {"a": 61, "b": 5, "c": 40, "d": 1, "e": 47, "f": 22}
    toks = {k: tokens(n, 30 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: O.forward(cfg, W, v) for k, v in toks.items()}
    eng = make_engine(path, dtype, device, blocks=12, max_seqs=3)
    plan = [
        [("a", 17), ("b", 2), ("c", 3)],
        [("a", 1), ("b", 3), ("c", 16)],          # b ends
        [("a", 2), ("d", 1), ("c", 1)],           # d: one-token request
        [("c", 20), ("e", 31)],                   # a sits out; c ends
        [("a", 41), ("e", 1), ("f", 2)],          # a ends
        [("e", 15), ("f", 20)],                   # both end
    ]
    at = {k: 0 for k in toks}
    got = {k: [] for k in toks}
    for step in plan:
        entries, end = [], []
        for rid, n in step:
            lo = at[rid]
            entries.append((rid, toks[rid][lo:lo + n], list(range(n))))
            at[rid] += n
            if at[rid] == lens[rid]:
                end.append(rid)
        out = eng.replay_step(entries, end=end)
        r0 = 0
        for rid, n in step:
            got[rid].append(out[r0:r0 + n])
            r0 += n
    assert at == lens
    bm = eng.block_manager
    assert bm.num_free == 12 and len(bm.free_slots) == 3   # all given back
    for k in toks:
        assert close(torch.cat(got[k]), want[k], dtype), k


def oracle_greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(O.forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("budget,blocks", [(1 << 20, 64), (7, 64), (24, 9)])
def test_greedy_generation_through_the_scheduler(ckpt, device, budget,
                                                 blocks):
    """LLMEngine.generate: the scheduler's own chunking (token budgets of
    7 and 24 cut the prompts into portions), continuous batching of three
    unequal requests, and with 9 pages preemption with recomputation, must
    all give the oracle's greedy continuation."""
    path, cfg, W = ckpt
    prompts = [tokens(45, 50), tokens(3, 51), tokens(28, 52)]
    n_new = 10
    want = [oracle_greedy(cfg, W, p, n_new) for p in prompts]
    eng = make_engine(path, "float32", device, blocks=blocks, max_seqs=3,
                      budget=budget)
    out = eng.generate(prompts, SamplingParams(
        max_tokens=n_new, temperature=0.0, ignore_eos=True))
    for i in range(3):
        assert out[f"offline-{i}"] == want[i], i
    assert eng.block_manager.num_free == blocks
    assert len(eng.block_manager.free_slots) == 3


OTHER_STACKS = [
    # (stack, width, vocab, eps, taps, loop, embedding scale)
    # one layer, nothing looped, no convolution; blocks of one position;
    # rotary over the whole head; both scales 1
    ([(mixer(2, 1, 16, 16, 6, 1, 0.25, 16, 50.0, (4.0, 16, 2.0, 1.0), 0.0,
             16, 1.0, 1.0), None)], 32, 41, 1e-6, 0, None, 1.0),
    # the whole stack looped three times; one tap; no window (plain
    # causal); no rotary code; as many key/value heads as query heads; a
    # router that picks one expert; widths no multiple of 8
    ([(mixer(3, 3, 12, 20, 0, 0, 0.3, 0, 1.0, None, 20.0, 36),
       moe(20, 3, 1, 1.0, 12)),
      (mixer(5, 1, 12, 20, 7, 3, 0.3, 6, 10.0, (2.0, 8, 2.0, 0.5), 0.0, 12),
       moe(12, 2, 2, 0.5, 0))],
     72, 53, 3e-4, 1, (0, 2, 3), 9.0),
    # a loop that runs once; a window of one position with blocks of two;
    # seven taps; blocks longer than a page (40 > 16); five query heads on
    # one key/value head; window without pooled blocks
    ([(mixer(5, 1, 20, 12, 1, 2, 0.22, 20, 1e6, (8.0, 32, 16.0, 2.0), 8.0,
             24), moe(16, 6, 2, 3.0, 8)),
      (mixer(2, 2, 8, 8, 9, 40, 0.35, 4, 10.0, None, 0.0, 70, 0.3, 2.0),
       None),
      (mixer(4, 2, 16, 8, 11, 0, 0.3, 8, 100.0, (4.0, 32, 4.0, 1.0), 0.0,
             8), moe(8, 4, 4, 1.0, 16))],
     60, 71, 1e-5, 7, (2, 3, 1), 3.0),
    # only the last layer looped, twice; an empty looped span elsewhere is
    # not needed: start == stop gives passes without layers
    ([(mixer(2, 2, 32, 32, 16, 16, 0.18, 32, 2e4, (3.0, 48, 16.0, 1.0), 25.0,
             48), moe(24, 4, 2, 1.75, 24)),
      (mixer(8, 2, 16, 8, 24, 8, 0.25, 16, 2e4, (3.0, 48, 16.0, 1.0), 25.0,
             40), moe(8, 7, 3, 1.0, 0))],
     64, 37, 1e-5, 5, (1, 2, 2), 7.0),
]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("which", range(len(OTHER_STACKS)))
def test_other_orders_and_sizes(tmp_path, device, dtype, which):
    stack, width, vocab, eps, taps, loop, scale = OTHER_STACKS[which]
    cfg = make_cfg(stack, width=width, vocab=vocab, eps=eps, taps=taps,
                   loop=loop, scale=scale)
    W = make_weights(cfg, seed=40 + which)
    path = save_checkpoint(tmp_path / f"o{which}", cfg, W)
    toks = tokens(80, 70 + which, vocab=vocab)
    want = O.forward(cfg, W, toks)
    eng = make_engine(path, dtype, device)
    assert close(replay(eng, "a", toks, [None]), want, dtype)
    assert close(replay(eng, "b", toks, [6, 1, 2, 30, 1, 1, None]), want,
                 dtype)
    # two requests side by side, cut differently
    half = replay_two(eng, toks, [9, 40, None], [33, 2, None])
    assert close(half[0], want, dtype) and close(half[1], want, dtype)


def replay_two(eng, toks, sizes_a, sizes_b):
    """The same tokens as two requests in shared steps with different
    cuts; returns both requests' logits at every position."""
    def cuts(sizes):
        out, at = [], 0
        for s in sizes:
            s = len(toks) - at if s is None else min(s, len(toks) - at)
            if s > 0:
                out.append((at, at + s))
                at += s
        return out
    ca, cb = cuts(sizes_a), cuts(sizes_b)
    got = {"x": [], "y": []}
    for step in range(max(len(ca), len(cb))):
        entries, end = [], []
        for rid, cc in (("x", ca), ("y", cb)):
            if step < len(cc):
                a, b = cc[step]
                entries.append((rid, toks[a:b], list(range(b - a))))
                if b == len(toks):
                    end.append(rid)
        out = eng.replay_step(entries, end=end)
        r0 = 0
        for rid, t, _ in entries:
            got[rid].append(out[r0:r0 + len(t)])
            r0 += len(t)
    return torch.cat(got["x"]), torch.cat(got["y"])


# ---------------------------------------------------------------------------
# a key made to stand out: at the window's edges, at a pooled block's edges,
# at page borders and far away
# ---------------------------------------------------------------------------
NEEDLE, PROBE = 3, 4


def needle_model(size, pool, width=32, vocab=23):
    """One layer whose attention half lets the PROBE token's query match
    the NEEDLE token's key far above every other pair (in head entries the
    rotary code leaves alone), the needle's value being large: whether and
    how (itself, or averaged into its block) the needle is visible decides
    the logits. The recurrent half and the convolution are switched off so
    that nothing else carries the needle forward."""
    stack = [(mixer(2, 1, 16, 8, size, pool, 2.0, 8, 100.0,
                    (4.0, 32, 4.0, 1.0), 0.0, 8, 1.0, 1.0), None)]
    cfg = make_cfg(stack, width=width, vocab=vocab, taps=2, loop=None,
                   scale=1.0)
    W = make_weights(cfg, seed=9)
    f32 = torch.float32
    emb = W["embed"].to(f32)
    emb[:, :2] = 0.0
    # rows of mean zero: the normed channels 0 and 1 of ordinary tokens
    # are exactly zero
    emb[:, 2:] -= emb[:, 2:].mean(1, keepdim=True)
    emb[NEEDLE] = 0.0
    emb[NEEDLE, 0] = 4.0
    emb[PROBE] = 0.0
    emb[PROBE, 1] = 4.0
    W["embed"] = emb.to(torch.bfloat16)
    bf = torch.bfloat16
    W["l0.norm1"] = torch.ones(width, dtype=bf)
    W["l0.norm1.b"] = torch.zeros(width, dtype=bf)
    W["l0.canon1"] = torch.zeros(width, 2, dtype=bf)
    q, k, v = (W[f"l0.mix.left.{n}"].to(f32) for n in "qkv")
    q[:, 1] = 0.0
    k[:, 0] = 0.0
    q[15::16] = 0.0
    k[15::16] = 0.0
    q[15::16, 1] = 6.0          # last entry of every query head
    k[15::16, 0] = 6.0          # last entry of the key head
    v[:, 0] = 3.0
    for n, t in (("q", q), ("k", k), ("v", v)):
        W[f"l0.mix.left.{n}"] = t.to(bf)
    W["l0.mix.left.q.norm"] = torch.ones(32, dtype=bf)
    W["l0.mix.left.k.norm"] = torch.ones(16, dtype=bf)
    W["l0.mix.right.o"] = torch.zeros_like(W["l0.mix.right.o"])
    return cfg, W


def needle_tokens(n, needle_at, probe_at, seed, vocab=23):
    g = torch.Generator().manual_seed(seed)
    t = torch.randint(5, vocab, (n,), generator=g).tolist()
    t[needle_at] = NEEDLE
    t[probe_at] = PROBE
    return t


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_window_and_block_edges_with_a_stand_out_key(tmp_path, device,
                                                     dtype):
    """The probe sits at position 99, the window holds 24 positions
    (76..99) and blocks hold 8, so blocks up to 64..71 are seen pooled and
    72..75 is not seen at all. The needle is put just inside the window
    (76), just outside (75, invisible), at the start of the unseen block
    (72), at the end of the last seen block (71), at that block's start on
    a page border (64), far back (2), and, without pooled blocks, at 2
    (invisible) - in prompt portions and in single decoded tokens."""
    for pool, spots in ((8, (76, 75, 72, 71, 64, 2)), (0, (76, 2))):
        cfg, W = needle_model(24, pool)
        path = save_checkpoint(tmp_path / f"n{pool}", cfg, W)
        eng = make_engine(path, dtype, device)
        seen = {}
        for spot in spots:
            toks = needle_tokens(104, spot, 99, 60)
            want = O.forward(cfg, W, toks)
            seen[spot] = want[99]
            for sizes in ([None], [90] + [1] * 14, [77, 2, 2, None],
                          [64, 35, 1, None], [72, 8, 8, 8, None]):
                got = replay(eng, f"r{spot}", toks, sizes)
                assert close(got, want, dtype), (pool, spot, sizes)
                assert rel_err(got[99:100], want[99:100]) < (
                    2e-4 if dtype == "float32" else 5e-2), (pool, spot)
        # the test has teeth: the probe's logits tell the cases apart
        assert rel_err(seen[76], seen[2]) > 0.05
        if pool:
            assert rel_err(seen[76], seen[75]) > 0.3      # window edge
            assert rel_err(seen[71], seen[72]) > 0.05     # block edge
            assert rel_err(seen[75], seen[72]) < 1e-3     # both unseen
            assert rel_err(seen[2], seen[75]) > 0.05      # far, but seen


def test_router_choice_uses_the_correction_not_the_weights(tmp_path):
    """Guards oracle and engine together: the correction moves the choice
    but not the weights; an unchosen expert never runs."""
    stack = [(mixer(2, 1, 8, 8, 6, 2, 0.3, 4, 10.0, None, 0.0, 8),
              moe(8, 3, 1, 2.0, 0))]
    cfg = make_cfg(stack, width=16, vocab=19, taps=2, loop=None)
    W = make_weights(cfg, seed=4)
    toks = tokens(24, 7, 19)
    base = O.forward(cfg, W, toks)
    W2 = dict(W)
    W2["l0.mlp.correction"] = torch.tensor(
        [5.0, -5.0, -5.0]).to(torch.bfloat16)          # always expert 0
    W3 = dict(W2)
    W3["l0.mlp.e1.down"] = torch.zeros_like(W["l0.mlp.e1.down"])
    W3["l0.mlp.e2.down"] = torch.zeros_like(W["l0.mlp.e2.down"])
    moved = O.forward(cfg, W2, toks)
    assert rel_err(moved, base) > 1e-3
    assert rel_err(O.forward(cfg, W3, toks), moved) == 0.0
    for k, w in enumerate((W, W2)):
        path = save_checkpoint(tmp_path / f"r{k}", cfg, w)
        eng = make_engine(path, "float32", "cpu")
        got = replay(eng, "a", toks, [7, 1, None])
        assert rel_err(got, O.forward(cfg, w, toks)) < 2e-4


def test_named_config_generates_deterministically():
    """The named tiny stack: random init, engine entry point, greedy."""
    from production_stack_amd.engine.config import (CacheConfig,
                                                    EngineConfig,
                                                    SchedulerConfig)
    from production_stack_amd.engine.engine import LLMEngine

    def run(budget):
        eng = LLMEngine(EngineConfig(
            model="tiny-dogidra", dtype="float32", max_model_len=256,
            enforce_eager=True,
            cache=CacheConfig(num_gpu_blocks=32, block_size=16),
            scheduler=SchedulerConfig(max_num_seqs=2,
                                      max_num_batched_tokens=budget,
                                      max_prefill_chunk=budget)),
            device="cpu")
        return eng.generate(
            [tokens(70, 1, 300), tokens(4, 2, 300)],
            SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))

    a, b = run(256), run(11)
    assert a == b and all(len(v) == 6 for v in a.values())


def test_trace_run_command(ckpt, tmp_path):
    """bin/trace_run end to end: JSON lines in, 'done' lines and logit
    files out, pool sized by --max-tokens, requests ended and replaced."""
    import subprocess
    import sys

    import numpy as np

    path, cfg, W = ckpt
    root = os.path.join(os.path.dirname(__file__), "..")
    ta, tb, tc = tokens(40, 80), tokens(7, 81), tokens(21, 82)
    steps = [
        {"step": 0, "entries": [
            {"id": "a", "tokens": ta[:33], "want": [0, 32]},
            {"id": "b", "tokens": tb, "want": [6]}], "end": ["b"]},
        {"step": 1, "entries": [
            {"id": "a", "tokens": ta[33:34], "want": []}], "end": []},
        {"step": 2, "entries": [
            {"id": "c", "tokens": tc, "want": [20]},
            {"id": "a", "tokens": ta[34:], "want": [5]}],
         "end": ["a", "c"]},
    ]
    out = tmp_path / "out"
    r = subprocess.run(
        [sys.executable, os.path.join(root, "bin", "trace_run"), "--model",
         path, "--dtype", "float32", "--out", str(out), "--max-tokens", "128",
         "--max-seqs", "2", "--device", "cpu"],
        input="\n".join(json.dumps(s) for s in steps) + "\n",
        capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    done = [ln for ln in r.stdout.splitlines() if ln.startswith("done ")]
    assert done == ["done 0", "done 1", "done 2"]
    assert not (out / "1.f32").exists()
    wa, wb, wc = (O.forward(cfg, W, t) for t in (ta, tb, tc))
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4")
                          .reshape(3, -1).copy())
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4")
                          .reshape(2, -1).copy())
    assert rel_err(g0, torch.stack([wa[0], wa[32], wb[6]])) < 2e-4
    assert rel_err(g2, torch.stack([wc[20], wa[39]])) < 2e-4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", DTYPES)
def test_decode_graph_replays_match_eager(ckpt, dtype):
    """Single-token steps replay a captured hipGraph (padded to a batch
    bucket, padding rows parked on the spare state slot; the routed
    feed-forwards take the all-experts path). Three requests of unequal
    length join and leave, so bucket sizes, padding rows and slots
    change between replays; eager prompt portions run in between. Every
    step's logits must match the eager engine's."""
    from production_stack_amd.engine.config import (CacheConfig,
                                                    EngineConfig,
                                                    SchedulerConfig)
    from production_stack_amd.engine.engine import LLMEngine

    path, cfg, W = ckpt

    def make(eager):
        return LLMEngine(EngineConfig(
            model=path, dtype=dtype, max_model_len=256, enforce_eager=eager,
            cache=CacheConfig(num_gpu_blocks=48, block_size=16,
                              enable_prefix_caching=False),
            scheduler=SchedulerConfig(max_num_seqs=4,
                                      max_num_batched_tokens=64)),
            device="cuda")

    graph, eager = make(False), make(True)
    assert graph.runner.graphs is not None and eager.runner.graphs is None
    prompts = [tokens(37, 90), tokens(5, 91), tokens(70, 92)]
    lens = [9, 14, 6]
    outs = []
    for eng in (graph, eager):
        got = {}
        seen = []
        orig = eng.runner.sample

        def spy(logits, seqs, _orig=orig, _seen=seen):
            _seen.append(logits.detach().float().cpu().clone())
            return _orig(logits, seqs)

        eng.runner.sample = spy
        for i, (p, n) in enumerate(zip(prompts, lens)):
            eng.add_request(f"r{i}", p, SamplingParams(
                max_tokens=n, temperature=0.0, ignore_eos=True))
        while eng.has_unfinished():
            for o in eng.step():
                got.setdefault(o.request_id, []).extend(o.new_token_ids)
        outs.append((got, seen))
    (g_tok, g_log), (e_tok, e_log) = outs
    assert len(g_log) == len(e_log) and len(g_log) >= max(lens)
    if dtype == "float32":
        assert g_tok == e_tok
    for a, b in zip(g_log, e_log):
        assert a.shape == b.shape
        if dtype == "float32":
            assert rel_err(a, b) < 2e-4
    want = [oracle_greedy(cfg, W, p, n) for p, n in zip(prompts, lens)]
    if dtype == "float32":
        assert [g_tok[f"r{i}"] for i in range(3)] == want
