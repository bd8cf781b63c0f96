"""GPU tests of the Gepilix serving path against the plain oracle (oracle/gepilix.py): each mechanism's kernel or module alone, then the model through the
registry, the slot cache and the ragged-batch scheduler -- whole prompts, token-by-token decoding, portions, unequal batches, reused slots, keys at the
chunks' and windows' edges, odd sizes, greedy generation, the trace replay program.  fp32 mode is held to fp32 rounding; bf16 mode to a few bf16
roundings of the logits' scale."""

import math

import pytest
import torch

from oracle import gepilix as O
from tests import gepilix_util as U

pytestmark = pytest.mark.gpu
_oracle_cache = {}
DEV = "cuda"
F32, F64, BF16, I32 = torch.float32, torch.float64, torch.bfloat16, torch.int32
TOL = {"float32": 3e-5, "bfloat16": 8e-2}


def dev_i32(x):
    return torch.tensor(x, dtype=I32).to(DEV)


def row_err(got, want):
    """The worst row's rms of the difference (mean removed) over the rms of the wanted rows."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()).max().item()


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def all_experts(cfg):
    """The same configuration with every expert chosen.  A top-k choice is no continuous function: where two router logits nearly tie, bf16 rounding
    upstream may pick the other expert, which says nothing about the kernels -- so the bf16 runs of whole models route every token to every expert (dispatch,
    weights, gated epilogue and the shared expert are all still there), and the choice itself is tested in fp32 and on the router kernel alone."""
    import copy

    cfg = copy.deepcopy(cfg)
    for layer in cfg["layers"]:
        if (layer.get("mlp") or {}).get("kind") == "moe":
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return cfg


def clear_tokens(cfg, w, n, seed, margin=1e-3):
    """Random tokens on which no router makes a close call at fp32 rounding: the seed is stepped until every token's gap exceeds ``margin``."""
    for k in range(40):
        toks = tokens(n, cfg["vocab"], seed + 1000 * k)
        gaps = []
        _oracle_cache[(id(w), str(cfg["layers"]), tuple(toks), False)] = O.forward(cfg, w, toks, F64, gaps=gaps)
        if not gaps or min(float(g_.min()) for g_ in gaps) > margin:
            return toks
    raise AssertionError("no token sequence without a close router call found")


@pytest.fixture(scope="module")
def checkpoint(tmp_path_factory):
    cs = U.make_config(U.default_layers())
    w = U.make_weights(cs, 11)
    return U.save(str(tmp_path_factory.mktemp("gepilix")), cs, w), cs[0], w


@pytest.fixture(scope="module")
def models(checkpoint, tmp_path_factory):
    """dtype -> (model, its configuration, weights): the bf16 model chooses every expert (``all_experts``), on the same weights."""
    from llm_quest_amd import registry

    folder, cfg, w = checkpoint
    every = all_experts(cfg)
    folder16 = U.save(str(tmp_path_factory.mktemp("gepilix16")), (every, None), w)
    return {"float32": (registry.load_model(folder, "float32", DEV), cfg, w), "bfloat16": (registry.load_model(folder16, "bfloat16", DEV), every, w)}


def oracle(cfg, w, toks, layers=False):
    key = (id(w), str(cfg["layers"]), tuple(toks), layers)
    if key not in _oracle_cache:
        _oracle_cache[key] = O.forward(cfg, w, toks, F64, return_layers=layers)
    return _oracle_cache[key]


def batch_of(model, **kw):
    from llm_quest_amd.generate import RaggedBatch

    return RaggedBatch(model, **kw)


# ------------------------------------------------------------------------------------------------------------------- the model through the scheduler
@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_whole_prompt_every_layer(models, dt):
    model, cfg, w = models[dt]
    toks = clear_tokens(cfg, w, 70, 1)
    want, layers = oracle(cfg, w, toks, layers=True)
    b = batch_of(model)
    got, got_layers = b.step([("a", toks)], [list(range(len(toks)))], return_layers=True)
    assert len(got_layers) == len(layers)
    for i, l in enumerate(got_layers):
        assert row_err(l, layers[i]) < TOL[dt], f"residual stream after layer {i}"
    assert row_err(got, want) < TOL[dt]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_token_by_token_from_the_first_token(models, dt):
    """Every token alone: the first token's shift reads zeros, convolutions read zeros before the start, every state starts at zero; chunks and windows
    fill and close one token at a time."""
    model, cfg, w = models[dt]
    toks = clear_tokens(cfg, w, 60, 2)
    want = oracle(cfg, w, toks)
    b = batch_of(model)
    got = torch.cat([b.step([("a", [t])]) for t in toks])
    assert row_err(got, want) < TOL[dt]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_portions_of_several_sizes(models, dt):
    """Portions down to one and two tokens: shorter than a convolution's taps, ending inside and exactly at a chunk's edge (chunks of 13 and 8 count from the
    sequence's first token, not from where the prompt was cut)."""
    model, cfg, w = models[dt]
    toks = clear_tokens(cfg, w, 90, 3)
    want = oracle(cfg, w, toks)
    b = batch_of(model)
    got, at = [], 0
    for n in [7, 2, 2, 1, 1, 33, 1, 9, 2, 32]:
        got.append(b.step([("a", toks[at : at + n])], [list(range(n))]))
        at += n
    assert at == len(toks)
    assert row_err(torch.cat(got), want) < TOL[dt]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_unequal_batch_equals_each_request_alone(models, dt):
    model, cfg, w = models[dt]
    lens, tail = [1, 41, 17, 66], 9
    seqs = [clear_tokens(cfg, w, n + tail, 10 + i) for i, n in enumerate(lens)]
    alone = []
    for s in seqs:
        b = batch_of(model)
        alone.append(b.step([("x", s)], [list(range(len(s)))]))
    b = batch_of(model, slots=2)  # fewer slots than sequences: the cache grows
    got = [[] for _ in seqs]
    out = b.step([(i, s[: lens[i]]) for i, s in enumerate(seqs)], [list(range(n)) for n in lens])
    at = 0
    for i, n in enumerate(lens):
        got[i].append(out[at : at + n])
        at += n
    live = list(range(len(seqs)))
    for k in range(tail):
        if k == 4:  # two requests leave early; the others go on
            for i in (0, 2):
                b.finish(i)
                live.remove(i)
        out = b.step([(i, [seqs[i][lens[i] + k]]) for i in live])
        for j, i in enumerate(live):
            got[i].append(out[j : j + 1])
    for i, s in enumerate(seqs):
        g = torch.cat(got[i])
        ref = alone[i][: g.shape[0]]  # (alone, the whole request is one prompt: in bf16 its last tokens take the prompt form of the kernels, here the one-token form)
        assert row_err(g, ref) < (1e-5 if dt == "float32" else 6e-2), f"request {i} in the batch differs from the request alone"
        assert row_err(g, oracle(cfg, w, s)[: g.shape[0]]) < TOL[dt]


def test_freed_slots_are_reused_without_leftovers(models):
    """A long sequence leaves key / value rows, recurrent states, convolution inputs and a shifted row behind; the next, shorter one takes its slot and must
    see none of them.  The cache starts small, so rows also grow while a sequence is alive."""
    model, cfg, w = models["float32"]
    b = batch_of(model, slots=1)
    b.cache.initial_chunk_size, b.cache.chunk_size = 4, 8
    long_, short = tokens(60, cfg["vocab"], 20), clear_tokens(cfg, w, 33, 21)
    b.step([("long", long_[:50])])
    for t in long_[50:]:
        b.step([("long", [t])])
    b.finish("long")
    got = [b.step([("short", short[:12])], [list(range(12))])] + [b.step([("short", [t])]) for t in short[12:]]
    assert b.cache.reuses >= 1 and b.cache.slots == 1
    assert row_err(torch.cat(got), oracle(cfg, w, short)) < TOL["float32"]


def test_long_decoding_passes_chunks_and_windows(models):
    """Decoded tokens walk past every window (7, 11 keys) and through dozens of chunks (8, 13 positions); the recurrent states are carried 200 steps."""
    model, cfg, w = models["float32"]
    toks = clear_tokens(cfg, w, 200, 30)
    b = batch_of(model)
    b.step([("a", toks[:5])])
    got = torch.cat([b.step([("a", [t])]) for t in toks[5:]])
    assert row_err(got, oracle(cfg, w, toks)[5:]) < TOL["float32"]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_other_sizes_odd_and_one(tmp_path, dt):
    """Sizes that are no multiples of 8 or of each other's: one head, one key head per query head, a chunk and a window of one key, a chunk and a window
    that never close, no cap, no frequency scaling, no mask entry at all, one block, one group, one tap (no convolution state), one expert chosen of two,
    no shared expert, unequal branch factors, a rotation of two entries, state and head sizes that differ, a layer without feed-forward first."""
    from llm_quest_amd import registry

    free = U.chunked(heads=2, kv_heads=2, dim=12, vdim=20, size=5, softcap=0.0)
    del free["mask"]
    layers = [(U.parallel(left=U.chunked(heads=1, kv_heads=1, dim=10, vdim=20, size=1, softcap=2.0), width=30, blocks=1, conv=1), None),
              (U.parallel_2(left=U.windowed(heads=6, kv_heads=2, dim=12, vdim=20, size=1, rot_dims=2, base=77.0, scaling=None, softcap=0.0), heads=1, vdim=18, state=10, groups=1,
                            norm_groups=1, conv=1, left_scale=1.0, right_scale=0.25), U.moe(experts=2, top=1, ff=20, shared=0)),
              (U.wkv(heads=1, dim=36, rank=1), U.dense(ff=18)),
              (U.parallel(left=free, width=60, blocks=5, conv=7), U.moe(experts=3, top=3, ff=33, shared=10)),
              (U.parallel_2(left=U.windowed(heads=3, kv_heads=1, dim=20, vdim=12, size=1000, rot_dims=20, scaling=(2.0, 1.0, 2.0, 16)), heads=6, vdim=10, state=34, groups=6,
                            norm_groups=3, conv=3), None),
              (U.wkv(heads=5, dim=12, rank=7), U.moe(experts=7, top=2, ff=12, shared=25))]
    cs = U.make_config(layers, width=100, vocab=77, eps=1e-6)
    w = U.make_weights(cs, 5)
    cfg = cs[0] if dt == "float32" else all_experts(cs[0])
    model = registry.load_model(U.save(str(tmp_path), (cfg, None), w), dt, DEV)
    toks = clear_tokens(cfg, w, 48, 6)
    want = oracle(cfg, w, toks)
    b = batch_of(model)
    got = [b.step([("a", toks[:29])], [list(range(29))])] + [b.step([("a", [t])]) for t in toks[29:]]
    assert row_err(torch.cat(got), want) < TOL[dt]


def test_wide_rows_and_wide_heads(tmp_path):
    """Rows wider than 512, attention heads of 136 | 72, a state of 136 key channels, recurrent heads of 96, value heads wider than 64."""
    from llm_quest_amd import registry

    layers = [(U.parallel(left=U.chunked(heads=2, kv_heads=1, dim=136, vdim=72, size=9), width=520, blocks=2, conv=3), U.dense(ff=64)),
              (U.wkv(heads=2, dim=96, rank=12), None),
              (U.parallel_2(left=U.windowed(heads=2, kv_heads=1, dim=40, vdim=72, size=17, rot_dims=16), heads=2, vdim=72, state=136, groups=1, norm_groups=2, conv=2), U.moe(ff=16, shared=16))]
    cs = U.make_config(layers, width=520, vocab=50)
    w = U.make_weights(cs, 9)
    for dt in ("float32", "bfloat16"):
        cfg = cs[0] if dt == "float32" else all_experts(cs[0])
        toks = clear_tokens(cfg, w, 40, 8)
        want = oracle(cfg, w, toks)
        model = registry.load_model(U.save(str(tmp_path / dt), (cfg, None), w), dt, DEV)
        b = batch_of(model)
        got = [b.step([("a", toks[:21])], [list(range(21))])] + [b.step([("a", [t])]) for t in toks[21:]]
        assert row_err(torch.cat(got), want) < TOL[dt]


def test_greedy_generation_through_the_entry_point(models):
    from llm_quest_amd.generate import generate_ragged

    model, cfg, w = models["float32"]
    prompts = [tokens(n, cfg["vocab"], 40 + n) for n in (4, 19, 9)]
    out = generate_ragged(model, prompts, max_gen=10)
    for p, gen in zip(prompts, out):
        assert len(gen) == 10
        seq = list(p)
        for t in gen:
            lg = O.forward(cfg, w, seq, F64)[-1]
            top = torch.topk(lg, 2)
            if int(top.indices[0]) != t:
                assert float(top.values[0] - top.values[1]) < 1e-4, "greedy token differs from the oracle's without a near tie"
                break
            seq.append(t)
    first = out[1][2]
    out2 = generate_ragged(model, prompts, max_gen=10, eos_ids=[first])
    assert out2[1] == out[1][: out[1].index(first)] and out2[0][: len(out2[0])] == out[0][: len(out2[0])]


def test_trace_replay_program_end_to_end(checkpoint, tmp_path):
    """bin/trace_run as a user runs it: a folder, steps on standard input (two prompts in one batch, then one token each, one request ending early and
    its slot taken by a third), logits files out -- against the oracle."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    folder32, cfg32, w = checkpoint
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    every = all_experts(cfg32)
    runs = {"float32": (folder32, cfg32), "bfloat16": (U.save(str(tmp_path / "every"), (every, None), w), every)}
    for dt, (folder, cfg) in runs.items():
        _replay(root, folder, cfg, w, dt, tmp_path / dt)


def _replay(root, folder, cfg, w, dt, out):
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    a, b, c = clear_tokens(cfg, w, 31, 50), clear_tokens(cfg, w, 9, 51), clear_tokens(cfg, w, 12, 52)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:28], "want": [0, 13, 27]}, {"id": "b", "tokens": b[:8], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[28:29], "want": [0]}, {"id": "b", "tokens": b[8:9], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[29:30], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "c", "tokens": c, "want": [11]}], "end": ["c"]},
             {"step": 4, "entries": [{"id": "a", "tokens": a[30:31], "want": [0]}], "end": ["a"]}]
    wa, wb, wc = oracle(cfg, w, a), oracle(cfg, w, b), oracle(cfg, w, c)
    want = {0: torch.stack([wa[0], wa[13], wa[27]]), 1: torch.stack([wa[28], wb[8]]), 3: wc[11:12], 4: wa[30:31]}
    res = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dt, "--out", str(out), "--max-tokens", "64"],
                         input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    assert [l for l in res.stdout.split("\n") if l.startswith("done")] == [f"done {i}" for i in range(5)]
    assert not (out / "2.f32").exists()
    for i, ref in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, cfg["vocab"]))
        assert got.shape == ref.shape and row_err(got, ref) < TOL[dt], (dt, i)


# ------------------------------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("width", [72, 100, 256, 520, 1000, 4100])
def test_residual_sum_branch_join_and_tanh_norm(width):
    from llm_quest_amd import kernels_seq as S

    g = torch.Generator().manual_seed(width)
    T, parts, eps = 9, 3, 1e-5
    r = lambda *s: torch.randn(*s, generator=g)
    x, ya, yb, y2 = r(T, width) * 3, r(T, width) * 40, r(T, width) * 0.01, r(T * parts, width)
    wa, wb, ls, w, b = r(width).abs() + 0.5, r(width).abs() + 0.5, r(width), r(width), r(width)
    alpha = 0.37
    d = lambda t: t.to(DEV)
    for ydt in (F32, BF16):
        a_, b_ = ya.to(ydt), yb.to(ydt)
        # both branches normed, expert rows, layer scale
        y = 0.5 * O.unit_rms(a_.double(), eps) * wa.double() + 0.5 * O.unit_rms(b_.double(), eps) * wb.double() + y2.double().reshape(T, parts, width).sum(1)
        v = x.double() + ls.double() * y
        x_out, h, h32 = S.dyt_sum(d(x), ya=d(a_), wa=d(wa), ca=0.5, yb=d(b_), wb=d(wb), cb=0.5, y2=d(y2), parts=parts, ls=d(ls), eps=eps, x_out=True, norm=(alpha, d(w), d(b)),
                                  out_dtype=BF16, want32=True)
        assert torch.allclose(x_out.cpu().double(), v, atol=3e-5)
        assert row_err(h32, O.dyn_tanh(v, alpha, w.double(), b.double())) < 3e-6 and torch.equal(h.cpu(), h32.cpu().to(BF16))
        # plain weighted branches (no norm); eps matters for the tiny branch above, not here
        v = x.double() + ls.double() * (0.8 * a_.double() + 1.7 * b_.double())
        x_out, h, _ = S.dyt_sum(d(x), ya=d(a_), ca=0.8, yb=d(b_), cb=1.7, ls=d(ls), x_out=True, norm=(alpha, d(w), d(b)), out_dtype=F32)
        assert torch.allclose(x_out.cpu().double(), v, atol=3e-5) and row_err(h, O.dyn_tanh(v, alpha, w.double(), b.double())) < 3e-6
    # the norm alone; the sum alone, in place; one summand on a view with a pitch of its own
    _, h, _ = S.dyt_sum(d(x), norm=(alpha, d(w), d(b)), out_dtype=F32)
    assert row_err(h, O.dyn_tanh(x.double(), alpha, w.double(), b.double())) < 3e-6
    xd = d(x)
    wide = d(torch.cat([ya, yb], dim=1))
    x_out, none, _ = S.dyt_sum(xd, ya=wide[:, width:], x_out=xd)
    assert none is None and x_out is xd and torch.allclose(xd.cpu().double(), x.double() + yb.double(), atol=3e-5)


def test_token_shift_reads_and_leaves_the_previous_row():
    from llm_quest_amd import kernels_seq as S

    g = torch.Generator().manual_seed(1)
    C, n_mix = 52, 5
    lens = [3, 1, 6]
    h = torch.randn(sum(lens), C, generator=g)
    mu = torch.rand(n_mix, C, generator=g)
    state = torch.randn(4, C, generator=g)
    slots = [2, 0, 3]
    st = state.clone().to(DEV)
    off = [0, 3, 4, 10]
    row_seq = sum([[i] * n for i, n in enumerate(lens)], [])
    out = S.token_shift(h.to(DEV), mu.to(DEV), st, dev_i32(row_seq), dev_i32(off), dev_i32(slots), F32).cpu()
    for i, n in enumerate(lens):
        rows = h[off[i] : off[i + 1]]
        prev = torch.cat([state[slots[i]][None], rows[:-1]])
        for m in range(n_mix):
            want = rows + (prev - rows) * mu[m]
            assert torch.allclose(out[off[i] : off[i + 1], m * C : (m + 1) * C], want, atol=1e-6)
        assert torch.equal(st[slots[i]].cpu(), rows[-1])
    assert torch.equal(st[1].cpu(), state[1])


def _attention_case(dt, size, chunked, past, n_new, H=4, G=2, d=24, dv=40, softcap=6.0, boost=None, seed=0):
    """One sequence with ``past`` cached keys and ``n_new`` new rows through the attention kernel against the oracle's masked softmax.  ``boost`` = (query
    position, key position): that query and key are made parallel and long, so that the key dominates the row if -- and only if -- it is visible."""
    from llm_quest_amd import kernels_seq as S

    g = torch.Generator().manual_seed(seed)
    n = past + n_new
    q, k, v = torch.randn(n, H, d, generator=g), torch.randn(n, G, d, generator=g), torch.randn(n, G, dv, generator=g)
    if boost:
        qi, kj = boost
        q[qi] = 6.0 * k[kj].repeat_interleave(H // G, dim=0)
        k[kj] = 3.0 * k[kj]
    scale = 0.3
    want = O.masked_attention(q.double(), k.double(), v.double(), scale, softcap, O.chunk_visible(size) if chunked else O.window_visible(size))[past:]
    kv_dt = BF16 if dt == "bfloat16" else F32
    row0 = 5
    cache = torch.zeros(row0 + n + 3, G * (d + dv), dtype=kv_dt, device=DEV)
    cache[row0 : row0 + n] = torch.cat([k.reshape(n, -1), v.reshape(n, -1)], dim=1).to(kv_dt).to(DEV)
    if dt == "bfloat16":
        kk, vv = k.to(BF16).double(), v.to(BF16).double()
        want = O.masked_attention(q.double(), kk, vv, scale, softcap, O.chunk_visible(size) if chunked else O.window_visible(size))[past:]
    qd = q[past:].reshape(n_new, H * d).contiguous().to(DEV)
    out = torch.empty(n_new, H * dv, dtype=kv_dt, device=DEV)
    i32 = dev_i32
    S.latent_attn(qd, cache, None, cache[:, G * d :], out, H, 2, d, 0, dv, d, d, dv, dv, (i32([0]), i32([n_new]), i32([past]), i32([row0]), i32([row0]), i32([row0])), n_new,
                  scale, max_keys=n, kv_rep=H // G, window=0 if chunked else size, softcap=softcap, chunk=size if chunked else 0)
    return out.float().cpu().reshape(n_new, H, dv), want


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("chunked", [True, False])
def test_attention_edges_of_chunks_and_windows(dt, chunked):
    """Prompts and one-token steps; sizes below, at and above the kernels' 64-key steps; keys far away among hundreds (one-token steps over long caches deal
    the visible range to several workgroups), the first key inside and the last key outside every edge made dominant."""
    tol = 2e-5 if dt == "float32" else 2e-2
    for size, past, n_new in [(13, 0, 70), (64, 0, 200), (100, 37, 90), (200, 700, 1), (200, 799, 1), (200, 800, 1), (7, 300, 1), (65, 129, 3), (1, 10, 5), (1000, 0, 150)]:
        got, want = _attention_case(dt, size, chunked, past, n_new, seed=size + past)
        assert row_err(got.reshape(n_new, -1), want.reshape(n_new, -1)) < tol, (size, past, n_new)
    for size, qi, n_new in [(50, 449, 1), (50, 450, 1), (50, 120, 121), (200, 999, 1), (64, 640, 1), (64, 703, 1)]:
        # the first visible key and the one just before it, each in turn dominant
        lo = qi // size * size if chunked else qi - size + 1
        for kj in (lo, lo - 1):
            got, want = _attention_case(dt, size, chunked, qi + 1 - n_new, n_new, boost=(qi, kj), seed=qi + kj)
            assert row_err(got.reshape(n_new, -1), want.reshape(n_new, -1)) < tol, (size, qi, kj)
    # a far key inside a chunk / window that holds hundreds
    got, want = _attention_case(dt, 512, chunked, 1000, 1, boost=(1000, 520), seed=3)
    assert row_err(got.reshape(1, -1), want.reshape(1, -1)) < tol


def test_head_gate_relu2_and_tanh_rows():
    from llm_quest_amd import kernels_seq as S

    g = torch.Generator().manual_seed(0)
    for n, group in ((70, 10), (64, 16)):
        wide = torch.randn(6, 2 * n, generator=g).to(DEV)
        x, gate = wide[:, 1 : n + 1], wide[:, n + 3 : n + 3 + n // group]
        got = S.unary_rows(x, S.UNARY_HEAD_GATE, gate=gate, group=group)
        want = x.double() * torch.sigmoid(gate.double()).repeat_interleave(group, dim=1)
        assert row_err(got, want) < 2e-6
        for kind, ref in ((S.UNARY_RELU2, lambda z: torch.relu(z) ** 2), (S.UNARY_TANH, torch.tanh)):
            assert row_err(S.unary_rows(wide[:, :n], kind), ref(wide[:, :n].double())) < 2e-6
            assert row_err(S.unary_rows(wide[:, :n].to(BF16), kind), ref(wide[:, :n].to(BF16).double())) < 5e-3


def _ragged(lens):
    off = [0]
    for n in lens:
        off.append(off[-1] + n)
    return off, sum([[i] * n for i, n in enumerate(lens)], [])


@pytest.mark.parametrize("H,dk,dv", [(3, 24, 24), (2, 40, 72), (1, 136, 20)])
def test_decay_bonus_attention_in_steps(H, dk, dv):
    """Two sequences in two steps of unequal portions against the oracle's token loop; the bonus made large so that a misplaced one shows."""
    from llm_quest_amd import kernels_seq as S

    g = torch.Generator().manual_seed(dk)
    lens = [19, 7]
    r_, k_, v_, z_ = (torch.randn(sum(lens), H * n, generator=g) for n in (dk, dk, dv, dk))
    z_ = z_ - 1.0
    u = torch.randn(H * dk, generator=g) * 3
    want = []
    at = 0
    for n in lens:
        sl = slice(at, at + n)
        r, k, v, dec = r_[sl].double().reshape(n, H, dk), k_[sl].double().reshape(n, H, dk), v_[sl].double().reshape(n, H, dv), torch.exp(-torch.exp(z_[sl].double())).reshape(n, H, dk)
        o = torch.zeros(n, H, dv, dtype=F64)
        for h in range(H):
            Sm = torch.zeros(dk, dv, dtype=F64)
            for t in range(n):
                kv = torch.outer(k[t, h], v[t, h])
                o[t, h] = (Sm + u.double().reshape(H, dk)[h][:, None] * kv).T @ r[t, h]
                Sm = dec[t, h][:, None] * Sm + kv
        want.append(o.reshape(n, -1))
        at += n
    state = torch.zeros(4, H, dk, dv, device=DEV)
    slots = dev_i32([3, 1])
    got = [[], []]
    for cuts in ([11, 2], [8, 5]):
        rows = []
        base = [0, lens[0]]
        done = [len(torch.cat(g_)) if g_ else 0 for g_ in got]
        idx = sum([list(range(base[i] + done[i], base[i] + done[i] + cuts[i])) for i in range(2)], [])
        off, _ = _ragged(cuts)
        o = S.decay_bonus_attention(r_[idx].to(DEV), k_[idx].to(DEV), v_[idx].to(DEV), z_[idx].to(DEV), u.to(DEV), dev_i32(off), slots, state, H, dk, dv).cpu()
        got[0].append(o[: cuts[0]])
        got[1].append(o[cuts[0] :])
    for i in range(2):
        assert row_err(torch.cat(got[i]), want[i]) < 2e-5


@pytest.mark.parametrize("H,G,N,P", [(4, 2, 24, 20), (6, 1, 16, 8), (2, 2, 136, 72)])
def test_state_space_duality_in_steps(H, G, N, P):
    from llm_quest_amd import kernels_seq as S

    g = torch.Generator().manual_seed(N)
    n, cut = 23, 14
    x, B, C, dt = torch.randn(n, H * P, generator=g), torch.randn(n, G * N, generator=g), torch.randn(n, G * N, generator=g), torch.randn(n, H, generator=g)
    dt_bias, A_log, D = torch.randn(H, generator=g), torch.randn(H, generator=g) * 0.5, torch.randn(H, generator=g)
    dtv = O.softplus(dt.double() + dt_bias.double())
    want = torch.zeros(n, H, P, dtype=F64)
    for h in range(H):
        Sm = torch.zeros(N, P, dtype=F64)
        gi = h // (H // G)
        for t in range(n):
            Sm = torch.exp(-torch.exp(A_log[h].double()) * dtv[t, h]) * Sm + dtv[t, h] * torch.outer(B[t].double().reshape(G, N)[gi], x[t].double().reshape(H, P)[h])
            want[t, h] = Sm.T @ C[t].double().reshape(G, N)[gi] + D[h].double() * x[t].double().reshape(H, P)[h]
    state = torch.zeros(2, H, N, P, device=DEV)
    d = lambda t: t.to(DEV)
    got = []
    for a, b in ((0, cut), (cut, n)):
        got.append(S.ssd(d(C[a:b]), d(B[a:b]), d(x[a:b]), d(dt[a:b]), d(dt_bias), d(A_log), d(D), dev_i32([0, b - a]), dev_i32([1]), state, H, G, N, P).cpu())
    assert row_err(torch.cat(got), want.reshape(n, -1)) < 2e-5
    assert float(state[0].abs().max()) == 0.0


def test_real_gated_recurrent_unit_in_steps():
    """Decays close to one (small lam) and close to zero; the state carried over three steps, one of a single token."""
    from llm_quest_amd import kernels_seq as S

    g = torch.Generator().manual_seed(2)
    C, nb, n = 60, 5, 31
    m = C // nb
    u, y = torch.randn(n, C, generator=g), torch.randn(n, C, generator=g)
    pr, pi = torch.randn(n, C, generator=g), torch.randn(n, C, generator=g)  # gate pre-activations per channel
    br, bi = torch.randn(C, generator=g), torch.randn(C, generator=g)
    lam = torch.linspace(-9.0, 3.0, C)
    r, i = torch.sigmoid(pr.double() + br.double()), torch.sigmoid(pi.double() + bi.double())
    a = torch.exp(-8.0 * r * O.softplus(lam.double()))
    Sm = torch.zeros(C, dtype=F64)
    want = torch.zeros(n, C, dtype=F64)
    for t in range(n):
        Sm = a[t] * Sm + torch.sqrt(1.0 - a[t] * a[t]) * i[t] * u[t].double()
        want[t] = Sm * O.gelu_tanh(y[t].double())
    lay = lambda r_, i_: torch.cat([r_.reshape(-1, nb, m), i_.reshape(-1, nb, m)], dim=2).reshape(-1, 2 * C)  # per block [recurrence gate | input gate]
    gates, gb = lay(pr, pi), lay(br[None], bi[None]).reshape(-1)
    state = torch.zeros(3, C, device=DEV)
    d = lambda t: t.contiguous().to(DEV)
    got = []
    for a_, b_ in ((0, 13), (13, 14), (14, n)):
        got.append(S.rglru(d(u[a_:b_]), d(gates[a_:b_]), d(gb), d(lam), d(y[a_:b_]), nb, dev_i32([0, b_ - a_]), dev_i32([2]), state, F32).cpu())
    assert row_err(torch.cat(got), want) < 2e-5
    assert torch.allclose(state[2].cpu().double(), Sm, atol=1e-5)


def test_gated_norm_in_groups_both_orders():
    from llm_quest_amd import kernels_seq as S

    g = torch.Generator().manual_seed(3)
    for n, groups in ((96, 4), (100, 1), (72, 72 // 8)):
        o, gate, w = torch.randn(7, n, generator=g) * 5, torch.randn(7, n, generator=g), torch.rand(n, generator=g) + 0.5
        od, gd, wd = o.double(), gate.double(), w.double()
        after = O.unit_rms(od.reshape(7, groups, -1), 1e-5).reshape(7, n) * wd * O.silu(gd)
        first = O.unit_rms((od * O.silu(gd)).reshape(7, groups, -1), 1e-5).reshape(7, n) * wd
        assert row_err(S.gated_groupnorm(o.to(DEV), w.to(DEV), gate.to(DEV), groups, 1e-5, F32), after) < 2e-6
        assert row_err(S.gated_groupnorm(o.to(DEV), w.to(DEV), gate.to(DEV), groups, 1e-5, F32, gate_first=True), first) < 2e-6


def test_router_weights_are_the_softmax_over_the_winners():
    from llm_quest_amd import kernels_seq as S

    g = torch.Generator().manual_seed(4)
    for E, top in ((8, 2), (5, 1), (70, 6), (3, 3)):
        logits, bias = torch.randn(33, E, generator=g) * 2, torch.randn(E, generator=g)
        ids, wts = S.moe_route(logits.to(DEV), bias.to(DEV), top, 1, 1, 1.0, softmax="chosen")
        val, idx = torch.topk(logits.double() + bias.double(), top, dim=-1)
        assert torch.equal(ids.cpu().long(), idx)
        assert torch.allclose(wts.cpu().double(), torch.softmax(val, dim=-1), atol=2e-6)


def test_rescaled_rotary_frequencies_and_short_convolution_with_bias():
    from llm_quest_amd import kernels_seq as S

    for dims, base, sc in ((12, 5000.0, (4.0, 1.0, 4.0, 64)), (64, 5e5, (8.0, 1.0, 4.0, 8192)), (6, 10.0, None), (32, 1e4, (2.0, 2.0, 16.0, 100))):
        scaling = dict(zip(("factor", "low", "high", "original"), sc)) if sc else None
        got = S.scaled_rope_frequencies(dims, base, scaling, "cpu")
        assert torch.allclose(got.double(), torch.tensor(O.scaled_frequencies(dims, base, scaling), dtype=F64), rtol=1e-6)
    g = torch.Generator().manual_seed(5)
    for C, taps in ((52, 4), (30, 1), (10, 7)):
        x, w, b = torch.randn(15, C, generator=g), torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
        want = O.causal_conv(x.double(), w.double(), b.double())
        state = torch.zeros(2, taps - 1, C, device=DEV) if taps > 1 else None
        got = []
        for a_, b_ in ((0, 2), (2, 3), (3, 15)):
            n = b_ - a_
            got.append(S.ragged_conv(x[a_:b_].to(DEV), w.to(DEV), state, dev_i32([0] * n), dev_i32([0, n]), dev_i32([1]), act=False, out_dtype=F32, bias=b.to(DEV)).cpu())
        assert row_err(torch.cat(got), want) < 2e-6
