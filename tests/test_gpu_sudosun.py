"""GPU tests of the Sudosun design in the layer-stack model class: every mechanism alone (one-layer models and single operators with planted
values), then whole models of small random configurations through the engine — against tests/sudosun_oracle.py (float64, whole sequences,
no cache, no pages, no slots).

f32 models must agree with the oracle to f32 rounding, bf16 models to bf16 rounding; and the logits of a position must not depend on how
its prompt was cut, on the rest of the batch or on the pages and state slots it got.
"""
import json
import math
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

from tests import sudosun_oracle as so
from tests.test_gpu_stack import BF16, F32, TOL, build, check, empty, from_dev, paged, raw, rel, to_dev, tokens_of
from vllm_rs_amd import _lib, checkpoint

pytestmark = pytest.mark.gpu

MOE = dict(kind="moe", expert=dict(ff=40), router=dict(experts=6, top=3, identity=3, groups=dict(count=3, keep=2)))
DENSE = dict(kind="dense", ff=72, limit=0.9)


def delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=4):
    return dict(type="delta", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv))


def lightning(heads=3, dim=24, vdim=16, decay=(0.6, 0.95, 0.999)):
    return dict(type="lightning", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)))


def parallel(heads=6, kv_heads=3, dim=16, vdim=24, size=70, dims=8, scaling=True, width=48, blocks=3, conv=4, scale=0.3, base=2000.0):
    left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if dims:
        left["rot"] = dict(base=base, dims=dims)
        if scaling:
            left["rot"]["scaling"] = dict(factor=3.0, original=48, fast=6.0, slow=1.5)
    if size:
        left["mask"] = dict(size=size)
    return dict(type="parallel", mixer=dict(left=left, right=dict(width=width, blocks=blocks, conv=conv)))


def config(layers, width=96, vocab=160, eps=1e-5, logit_scale=1.7):
    return dict(architecture="Sudosun", width=width, vocab=vocab, norm=dict(eps=eps), logit_scale=logit_scale, layers=layers)


def config_a():
    """every mixer and both feed-forwards, grouped q / k heads in the delta rule, key size != value size everywhere, rotary on part of a head,
    a window longer than a page and one shorter, a layer without feed-forward, a router without groups and identity experts, top 1"""
    return config([
        dict(parallel(), mlp=MOE),
        dict(delta(), mlp=DENSE),
        dict(lightning(), mlp=None),
        dict(parallel(heads=4, kv_heads=4, dim=24, vdim=16, size=9, dims=24, scaling=False, width=32, blocks=1, conv=2), mlp=dict(kind="moe", expert=dict(ff=24), router=dict(experts=4, top=1))),
        dict(delta(heads=2, kv_heads=2, dim=8, vdim=8, conv=1), mlp=MOE),
        dict(lightning(heads=2, dim=8, vdim=24, decay=(0.5, 0.9995)), mlp=DENSE),
    ])


def config_b():
    """sizes off every 16-byte path: width 50, heads of 5 / 7 / 6 channels, a window of 5 positions, convolutions of 3 taps, one gate block of
    7 channels, top = every router output"""
    moe = dict(kind="moe", expert=dict(ff=11), router=dict(experts=2, top=3, identity=1))
    return config([
        dict(lightning(heads=2, dim=6, vdim=5, decay=(0.8, 0.97)), mlp=moe),
        dict(parallel(heads=2, kv_heads=1, dim=6, vdim=7, size=5, dims=2, width=14, blocks=2, conv=3, scale=0.5, base=100.0), mlp=dict(kind="dense", ff=13, limit=2.5)),
        dict(delta(heads=2, kv_heads=1, dim=5, vdim=7, conv=3), mlp=None),
    ], width=50, vocab=70, eps=1e-6, logit_scale=0.6)


def agree(got, ref, dt, what=""):
    """a model's rows against the oracle's.  f32: every row to f32 rounding.  bf16: a close call of a router (a discrete choice) may turn
    a token, so the rows are judged one by one: the typical row to bf16 rounding, three in four within a few times that"""
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    got, ref = got.reshape(-1, got.shape[-1]), ref.reshape(-1, ref.shape[-1])
    rows = np.sqrt(((got - ref) ** 2).mean(-1)) / np.maximum(np.sqrt((ref ** 2).mean(-1)), 1e-30)
    if dt == F32:
        assert rows.max() < 2e-4 and rel(got, ref) < TOL[F32], (what, rows.max(), rel(got, ref))
    else:
        assert np.median(rows) < 5e-2 and np.quantile(rows, 0.75) < 8e-2, (what, float(np.median(rows)), float(np.quantile(rows, 0.75)))


def every(n):
    return list(range(n))


def only(tensors, branch):
    """a parallel mixer with one branch alone: the other branch's output norm weighs nothing"""
    off = "l0.mix.%s.out" % ("right" if branch == "left" else "left")
    tensors[off] = np.zeros_like(tensors[off])
    return tensors


# ------------------------------------------------------------------------------------------------ each mechanism alone
ALONE = {
    "delta": ([delta()], None),
    "delta-one-group-one-tap": ([delta(heads=3, kv_heads=1, dim=8, vdim=40, conv=1)], None),
    "delta-wide": ([delta(heads=2, kv_heads=2, dim=128, vdim=128, conv=3)], None),
    "lightning": ([lightning()], None),
    "lightning-one-head": ([lightning(heads=1, dim=64, vdim=48, decay=(0.97,))], None),
    "attention-branch": ([parallel()], "left"),
    "attention-branch-plain-causal": ([parallel(size=0, scaling=False)], "left"),
    "attention-branch-no-rotary": ([parallel(dims=0, size=33)], "left"),
    "recurrent-branch": ([parallel()], "right"),
    "recurrent-branch-one-block-one-tap": ([parallel(width=40, blocks=1, conv=1)], "right"),
    "parallel": ([parallel()], None),
    "dense": ([dict(lightning(), mlp=DENSE)], None),
    "experts": ([dict(lightning(), mlp=MOE)], None),
    "experts-top1-plain": ([dict(lightning(), mlp=dict(kind="moe", expert=dict(ff=24), router=dict(experts=7, top=1)))], None),
    "experts-all-chosen": ([dict(lightning(), mlp=dict(kind="moe", expert=dict(ff=24), router=dict(experts=3, top=5, identity=2)))], None),
}


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", sorted(ALONE))
def test_each_mechanism_alone(name, dt):
    """one layer of one kind (no feed-forward unless it is the subject): a 150-token prompt whole, then the same prompt in portions with
    single tokens between them — the layer's output and the logits against the oracle"""
    layers, branch = ALONE[name]
    layers = [dict(dict(mlp=None), **x) for x in layers]
    cfg = config(layers)
    tensors = so.random_tensors(cfg, 7)
    if branch:
        only(tensors, branch)
    toks = tokens_of(cfg, 150, 3)
    ref, lay = so.forward(cfg, tensors, toks, True)
    eng = build(cfg, tensors, dt, blocks=8, max_model_len=256)
    eng.layer_trace(True)
    got = eng.replay_step([(1, toks, every(150))], [1])
    trace = eng.read_layer_trace(150)
    eng.layer_trace(False)
    agree(trace[0], lay[0], dt, "layer")
    agree(got, ref, dt, "whole")
    rows, at = [], 0
    for c in (1, 2, 60, 1, 1, 5, 64, 1, 15):
        rows.append(eng.replay_step([(2, toks[at:at + c], every(c))], [2] if at + c == 150 else []))
        at += c
    eng.close()
    assert at == 150
    agree(np.concatenate(rows), ref, dt, "portions")
    assert rel(np.concatenate(rows), got) < (1e-5 if dt == F32 else 3e-2)


def test_first_tokens_of_a_sequence():
    """sequences of one, two and four tokens (shorter than the convolutions): whole and token by token; the recurrences start from zero
    also for the first token, the convolutions see zeros before it"""
    cfg = config([dict(parallel(conv=4), mlp=None), dict(delta(conv=4), mlp=None), dict(lightning(), mlp=None)])
    tensors = so.random_tensors(cfg, 9)
    eng = build(cfg, tensors, F32, blocks=4, max_model_len=128)
    for toks in ([5], [5, 5], [7, 5], [5, 7, 5, 5]):
        ref = so.forward(cfg, tensors, toks)
        whole = eng.replay_step([(1, toks, every(len(toks)))], [1])
        agree(whole, ref, F32, str(toks))
        one = np.stack([eng.replay_step([(2, toks[p:p + 1], [0])], [2] if p == len(toks) - 1 else [])[0] for p in range(len(toks))])
        agree(one, ref, F32, str(toks) + " token by token")
    eng.close()


@pytest.mark.parametrize("decode", [False, True], ids=["prompt", "decoded"])
@pytest.mark.parametrize("size", [7, 64, 70])
def test_window_edges(size, decode):
    """attention branch alone: a changed token reaches its own position and the size - 1 positions behind it and nothing beyond — exactly.
    Portions cut inside windows; decoding past the window."""
    cfg = config([dict(parallel(size=size, heads=4, kv_heads=2), mlp=None)])
    tensors = only(so.random_tensors(cfg, 11), "left")
    n = 3 * size + 5
    toks = tokens_of(cfg, n, 4)
    other = list(toks)
    at = size + size // 2
    other[at] = (toks[at] + 3) % cfg["vocab"]
    ref_a, ref_b = so.forward(cfg, tensors, toks), so.forward(cfg, tensors, other)
    eng = build(cfg, tensors, F32, blocks=8, max_model_len=320)

    def run(rid, t):
        if not decode:
            cuts = [size - 2, 5, size, n - 2 * size - 3]
            out, p = [], 0
            for i, c in enumerate(cuts):
                out.append(eng.replay_step([(rid, t[p:p + c], every(c))], [rid] if i == len(cuts) - 1 else []))
                p += c
            return np.concatenate(out)
        first = eng.replay_step([(rid, t[:3], every(3))], [])
        return np.concatenate([first] + [eng.replay_step([(rid, t[p:p + 1], [0])], [rid] if p == n - 1 else []) for p in range(3, n)])
    a, b = run(1, toks), run(2, other)
    eng.close()
    agree(a, ref_a, F32), agree(b, ref_b, F32)
    edge = at + size  # the first position that no longer sees the changed token
    changed = np.abs(a - b).max(-1)
    ref_changed = np.abs(ref_a - ref_b).max(-1)
    assert (changed[:at] == 0).all() and (changed[edge:] == 0).all() and (ref_changed[edge:] < 1e-12).all()
    assert (changed[at:edge] > 1e-6).all() and (ref_changed[at:edge] > 1e-6).all()
    assert rel(a[edge], ref_a[edge]) < 3e-5 and rel(a[edge - 1], ref_a[edge - 1]) < 3e-5


@pytest.mark.parametrize("kind", ["lightning", "delta", "recurrent-branch"])
def test_a_far_token_stays_in_the_state(kind):
    """a token hundreds of positions back reaches the last logits only through the state (slow decays): whole prompt, decoding across page
    borders and 2-token portions give the oracle's logits, which do depend on that token"""
    layer = {"lightning": lightning(heads=2, dim=16, vdim=16, decay=(0.9995, 0.999)),
             "delta": delta(heads=2, kv_heads=2, dim=64, vdim=16, conv=2),
             "recurrent-branch": parallel(size=4, width=32, blocks=2, conv=2)}[kind]
    cfg = config([dict(layer, mlp=None)])
    tensors = so.random_tensors(cfg, 13)
    if kind == "delta":  # slow decays: a strongly negative step-size bias; no writes to wear the state down
        tensors["l0.mix.dt_bias"] = so.bf16_round(np.full_like(tensors["l0.mix.dt_bias"], -9.0))
        tensors["l0.mix.b"] = np.zeros_like(tensors["l0.mix.b"])
    if kind == "recurrent-branch":  # decays close to one; the attention branch (a window of four) weighs nothing
        only(tensors, "right")
        tensors["l0.mix.right.lam"] = so.bf16_round(np.full_like(tensors["l0.mix.right.lam"], -8.0))
    n = 260 if kind == "delta" else 640
    toks = tokens_of(cfg, n, 5)
    other = list(toks)
    other[20] = (toks[20] + 1) % cfg["vocab"]
    if kind == "recurrent-branch":  # every token adds to the one state value of a channel: the two tokens compared keep embeddings of full
        # size, all others get small ones, so that the far token is not one among hundreds of equals
        tensors["embed"][:150] = so.bf16_round(tensors["embed"][:150] * 0.1)
        tensors["l0.norm1.b"] = np.zeros_like(tensors["l0.norm1.b"])
        toks = [t % 150 for t in toks]
        other = list(toks)
        toks[20], other[20] = 158, 159
    ref_a, ref_b = so.forward(cfg, tensors, toks)[-1], so.forward(cfg, tensors, other)[-1]
    felt = rel(ref_a, ref_b)
    assert felt > 1e-3
    eng = build(cfg, tensors, F32, blocks=24, max_model_len=704)
    whole = eng.replay_step([(1, other, [n - 1])], [1])[0]
    eng.replay_step([(2, other[:40], [])], [])
    for p in range(40, n - 1):
        eng.replay_step([(2, other[p:p + 1], [])], [])
    dec = eng.replay_step([(2, other[n - 1:], [0])], [2])[0]
    for p in range(0, n - 2, 2):
        eng.replay_step([(3, other[p:p + 2], [])], [])
    por = eng.replay_step([(3, other[n - 2:], [1])], [3])[0]
    eng.close()
    for got in (whole, dec, por):
        assert rel(got, ref_b) < min(1e-4, felt / 10) and rel(got, ref_a) > felt / 2


# ------------------------------------------------------------------------------------------------ whole models
@pytest.fixture(scope="module", params=[("a", F32), ("a", BF16), ("b", F32), ("b", BF16)], ids=["a-f32", "a-bf16", "b-f32", "b-bf16"])
def model(request):
    name, dt = request.param
    cfg = config_a() if name == "a" else config_b()
    tensors = so.random_tensors(cfg, 17 if name == "a" else 18)
    eng = build(cfg, tensors, dt, blocks=12, max_model_len=512, num_state_slots=4)
    yield cfg, tensors, dt, eng
    eng.close()


def test_layers_one_by_one(model):
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 90, 1)
    eng.layer_trace(True)
    got = eng.replay_step([(1, toks, every(90))], [1])
    trace = eng.read_layer_trace(90)
    eng.layer_trace(False)
    ref, layers = so.forward(cfg, tensors, toks, True)
    for i, x in enumerate(layers):
        agree(trace[i], x, dt, f"layer {i}")
    agree(got, ref, dt)


def test_prefill_against_token_by_token_decoding(model):
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 150, 2)
    ref = so.forward(cfg, tensors, toks)
    whole = eng.replay_step([(1, toks, every(150))], [1])
    agree(whole, ref, dt, "whole")
    one = np.stack([eng.replay_step([(2, toks[p:p + 1], [0])], [2] if p == 149 else [])[0] for p in range(150)])
    agree(one, ref, dt, "token by token")
    assert rel(one, whole) < (1e-5 if dt == F32 else 3e-2)


@pytest.mark.parametrize("sizes", [[2] * 30, [37, 3, 37, 2, 5], [64, 64, 2], [63, 2, 63, 2], [1, 5, 1, 1, 70, 1], [71, 9, 2, 70]])
def test_portions(model, sizes):
    """a prompt cut anywhere (down to two tokens, at and across page borders and window edges, shorter than the convolutions) gives the
    logits of the whole prompt"""
    cfg, tensors, dt, eng = model
    n = sum(sizes)
    toks = tokens_of(cfg, n, 3)
    whole = eng.replay_step([(1, toks, every(n))], [1])
    got, at = [], 0
    for i, c in enumerate(sizes):
        got.append(eng.replay_step([(2, toks[at:at + c], every(c))], [2] if i == len(sizes) - 1 else []))
        at += c
    got = np.concatenate(got)
    assert rel(got, whole) < (1e-5 if dt == F32 else 3e-2)
    agree(got, so.forward(cfg, tensors, toks), dt)


def test_unequal_batch_against_each_alone(model):
    cfg, tensors, dt, eng = model
    lens = [70, 3, 129, 1]
    prompts = [tokens_of(cfg, n, 10 + i) for i, n in enumerate(lens)]
    alone = [eng.replay_step([(1, p, every(len(p)))], [1]) for p in prompts]
    batch = eng.replay_step([(10 + i, p, every(len(p))) for i, p in enumerate(prompts)], [10, 11, 12, 13])
    tol = 1e-5 if dt == F32 else 3e-2
    at = 0
    for i, p in enumerate(prompts):
        assert rel(batch[at:at + len(p)], alone[i]) < tol, f"request {i} depends on its batch"
        at += len(p)
    cut = [n // 2 for n in lens]
    first = eng.replay_step([(20 + i, p[:c], every(c)) for i, (p, c) in enumerate(zip(prompts, cut)) if c], [])
    second = eng.replay_step([(20 + i, p[c:], every(len(p) - c)) for i, (p, c) in enumerate(zip(prompts, cut))], [20, 21, 22, 23])
    a1 = a2 = 0
    for i, (p, c) in enumerate(zip(prompts, cut)):
        got = np.concatenate([first[a1:a1 + c], second[a2:a2 + len(p) - c]])
        a1, a2 = a1 + c, a2 + len(p) - c
        assert rel(got, alone[i]) < tol, f"request {i} depends on its cut or its batch"


def test_mixed_steps_with_reused_pages_and_slots(model):
    """12 pages and 4 state slots for 8 requests that come and go: decoded tokens beside portions of prompts, a finished request's pages and
    slot taken by the next one at once; every logit row equals the request's own run"""
    cfg, tensors, dt, eng = model
    r = np.random.default_rng(4)
    lens = [130, 60, 200, 90, 33, 150, 64, 128]
    prompts = [tokens_of(cfg, n, 40 + i) for i, n in enumerate(lens)]
    ref = [so.forward(cfg, tensors, p) for p in prompts]
    waiting, live = list(range(len(prompts))), {}
    got_rows, ref_rows = [], []
    while waiting or live:
        while waiting and len(live) < 4 and sum((lens[i] + 63) // 64 for i in list(live) + [waiting[0]]) <= 12:
            live[waiting.pop(0)] = 0
        entries, ends, spans = [], [], []
        for i, at in live.items():
            left = lens[i] - at
            c = 1 if (at > 0 and r.random() < 0.5) else int(min(left, r.choice([2, 3, 17, 64, 100])))
            entries.append((1000 + i, prompts[i][at:at + c], every(c)))
            spans.append((i, at, c))
            if at + c == lens[i]:
                ends.append(1000 + i)
        out = eng.replay_step(entries, ends)
        o = 0
        for i, at, c in spans:
            got_rows.append(out[o:o + c]), ref_rows.append(ref[i][at:at + c])
            o += c
            live[i] = at + c
            if live[i] == lens[i]:
                del live[i]
    agree(np.concatenate(got_rows), np.concatenate(ref_rows), dt)


def test_a_fifth_request_waits_for_a_slot(model):
    cfg, tensors, dt, eng = model
    for i in range(4):
        eng.replay_step([(500 + i, [1, 2, 3], [])], [])
    with pytest.raises(RuntimeError, match="state slot"):
        eng.replay_step([(504, [1, 2, 3], [])], [])
    eng.replay_step([], [500, 501, 502, 503, 504])
    toks = tokens_of(cfg, 10, 1)
    agree(eng.replay_step([(505, toks, every(10))], [505]), so.forward(cfg, tensors, toks), dt)


def test_long_decoding(model):
    """310 decoded tokens behind a 20-token prompt: window edges, page borders and the states pass under decoded tokens"""
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 330, 5)
    ref = so.forward(cfg, tensors, toks)
    eng.replay_step([(1, toks[:20], [])], [])
    rows = [eng.replay_step([(1, toks[p:p + 1], [0])], [1] if p == len(toks) - 1 else [])[0] for p in range(20, len(toks))]
    agree(np.stack(rows), ref[20:], dt)


def test_long_prompt_in_one_step_and_in_portions():
    """a 1500-token prompt through heads of 64 / 128 channels (bf16 prompt steps of this size take the matrix-core attention and matrix
    kernels), whole and in three portions; logits also just inside and just outside the window of the first portion's last token"""
    cfg = config([dict(parallel(heads=4, kv_heads=2, dim=64, vdim=32, size=192, dims=32, width=64, blocks=2, scale=0.11), mlp=MOE),
                  dict(delta(heads=2, kv_heads=1, dim=64, vdim=64, conv=3), mlp=None),
                  dict(lightning(heads=2, dim=128, vdim=64, decay=(0.99, 0.9995)), mlp=DENSE)], width=128)
    tensors = so.random_tensors(cfg, 23)
    toks = tokens_of(cfg, 1500, 8)
    want = sorted(set(list(range(0, 1500, 47)) + [191, 192, 193, 699, 700, 890, 891, 1499]))
    ref = so.forward(cfg, tensors, toks)[want]
    for dt in (F32, BF16):
        eng = build(cfg, tensors, dt, blocks=48, max_model_len=1536)
        whole = eng.replay_step([(1, toks, want)], [1])
        agree(whole, ref, dt, "whole")
        parts, at = [], 0
        for c in (700, 40, 760):
            parts.append(eng.replay_step([(2, toks[at:at + c], [w - at for w in want if at <= w < at + c])], [2] if at + c == 1500 else []))
            at += c
        eng.close()
        parts = np.concatenate(parts)
        agree(parts, ref, dt, "portions")
        assert rel(parts, whole) < (1e-5 if dt == F32 else 3e-2)


@pytest.mark.parametrize("use_graph", [False, True], ids=["eager", "graphs"])
def test_greedy_generation_through_the_scheduler(use_graph):
    """Engine.generate: the engine's own scheduler, block manager with state slots, prefill and decode steps (captured decode graphs when
    asked) and its argmax — against the oracle's greedy continuation, f32 so that near ties do not decide.  Two slots for three requests:
    the third waits for a slot and takes a used one."""
    cfg = config_a()
    tensors = so.random_tensors(cfg, 19)
    eng = build(cfg, tensors, F32, blocks=16, max_model_len=256, use_graph=use_graph, num_state_slots=2)
    prompts = [tokens_of(cfg, n, 60 + n) for n in (5, 70, 31)]
    outs = eng.generate(prompts, max_tokens=12, ignore_eos=True)
    eng.close()
    for p, out in zip(prompts, outs):
        seq = list(p)
        for t in out:
            lg = so.forward(cfg, tensors, seq)[-1]
            top2 = np.sort(lg)[-2:]
            assert int(t) == int(lg.argmax()) or top2[1] - top2[0] < 1e-3, (len(p), len(seq))
            seq.append(int(t))
        assert len(out) == 12


def test_sampled_generation_stays_inside_the_top_k():
    """the framework's sampler on this design's logits (temperature, top-k 3): every sampled token is one of the three most likely by the
    oracle's logits for the sequence so far (or within rounding of the third), and a penalised run still finishes"""
    cfg = config_a()
    tensors = so.random_tensors(cfg, 21)
    eng = build(cfg, tensors, F32, blocks=16, max_model_len=256, num_state_slots=2)
    prompts = [tokens_of(cfg, n, 80 + n) for n in (9, 40)]
    outs = eng.generate(prompts, max_tokens=8, ignore_eos=True, sampling=dict(temperature=0.9, top_k=3, top_p=1.0))
    pen = eng.generate(prompts[:1], max_tokens=6, ignore_eos=True, sampling=dict(temperature=0.7, top_k=4, top_p=0.9, frequency_penalty=0.5, presence_penalty=0.2))
    eng.close()
    assert len(pen[0]) == 6
    for p, out in zip(prompts, outs):
        seq = list(p)
        assert len(out) == 8
        for t in out:
            lg = so.forward(cfg, tensors, seq)[-1]
            third = np.sort(lg)[-3]
            assert lg[int(t)] >= third - 1e-3, (len(p), len(seq))
            seq.append(int(t))


def test_synthetic_weights_and_state_plan():
    from vllm_rs_amd.engine import Engine
    cfg = checkpoint.parse_config(config_a())
    eng = Engine(cfg, max_num_seqs=4, max_model_len=256, kv_fraction=0.01, use_graph=False).init_synthetic()
    assert eng.num_gpu_blocks > 16
    out = eng.generate([list(range(1, 40)), list(range(3, 9))], max_tokens=5, ignore_eos=True)
    assert [len(o) for o in out] == [5, 5]
    eng.close()
    with pytest.raises(RuntimeError, match="prefix cache"):
        Engine(cfg, max_num_seqs=4, max_model_len=256, num_gpu_blocks=8, use_graph=False, enable_prefix_cache=True).init_synthetic()


def test_trace_runner_on_a_model_folder(tmp_path):
    """bin/trace_run as a user starts it: config.json + model.safetensors in a folder, steps on standard input (a prompt in portions beside
    another request's single tokens; a pool of three pages and two state slots used again), logits files out — against the oracle"""
    cfg = config_a()
    tensors = so.random_tensors(cfg, 31)
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfg))
    header, blobs, off = {}, [], 0
    for name, a in tensors.items():
        b = checkpoint.f32_to_bf16_bits(np.asarray(a, np.float32)).tobytes()
        header[name] = dict(dtype="BF16", shape=list(np.shape(a)), data_offsets=[off, off + len(b)])
        off += len(b)
        blobs.append(b)
    h = json.dumps(header).encode()
    (model_dir / "model.safetensors").write_bytes(struct.pack("<Q", len(h)) + h + b"".join(blobs))
    p1, p2, p3 = tokens_of(cfg, 100, 1), tokens_of(cfg, 40, 2), tokens_of(cfg, 64, 3)
    steps = [dict(entries=[dict(id="x", tokens=p1[:37], want=every(37)), dict(id="y", tokens=p2[:38], want=[])], end=[]),
             dict(entries=[dict(id="x", tokens=p1[37:99], want=every(62)), dict(id="y", tokens=p2[38:39], want=[0])], end=[]),
             dict(entries=[dict(id="y", tokens=p2[39:], want=[0])], end=["y"]),
             dict(entries=[dict(id="x", tokens=p1[99:], want=[0])], end=["x"]),
             dict(entries=[dict(id="z", tokens=p3, want=every(64))], end=["z"])]
    for i, s in enumerate(steps):
        s["step"] = i
    r1, r2, r3 = (so.forward(cfg, tensors, p) for p in (p1, p2, p3))
    want = [r1[:37], np.concatenate([r1[37:99], r2[38:39]]), r2[39:], r1[99:], r3]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dtype, dt in (("float32", F32), ("bfloat16", BF16)):
        out = tmp_path / ("out_" + dtype)
        r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(model_dir), "--dtype", dtype, "--out", str(out),
                            "--max-tokens", "192", "--max-seqs", "2"], input="\n".join(json.dumps(s) for s in steps).encode() + b"\n",
                           capture_output=True, timeout=110)
        assert r.returncode == 0, r.stderr.decode()[-1500:]
        assert [ln for ln in r.stdout.decode().split("\n") if ln.startswith("done")] == ["done %d" % i for i in range(5)]
        got = [np.fromfile(out / ("%d.f32" % i), "<f4").reshape(-1, cfg["vocab"]) for i in range(5)]
        assert [g.shape[0] for g in got] == [w.shape[0] for w in want]
        agree(np.concatenate(got), np.concatenate(want), dt, dtype)


# ------------------------------------------------------------------------------------------------ operators alone, planted values
def run_window_attention(L, q, positions, k, v, scale, window, sink, head_scale, gate, dt, decode, r, BS=64):
    Tq, H, dim = q.shape
    G, vdim = k.shape[1], v.shape[2]
    kc, vc, table = paged(k, v, BS, r, dt)
    sk = raw(sink, np.float32).ptr if sink is not None else None
    hs = raw(head_scale, np.float32).ptr if head_scale is not None else None
    if decode:
        res = []
        for i in range(Tq):
            o1 = empty(H * vdim * 4)
            qi = to_dev(q[i].reshape(1, H * dim), dt)
            gt = raw(gate[i:i + 1], np.float32).ptr if gate is not None else None
            L.vra_stack_op_attention_window(qi.ptr, H * dim, o1.ptr, kc.ptr, vc.ptr, raw([positions[i]], np.int64).ptr, raw(table, np.uint32).ptr,
                                            raw([positions[i] + 1], np.uint32).ptr, None, 1, 1, 1, H, G, dim, vdim, BS, len(table), scale, window, sk, hs, gt, H, dt, 0)
            check()
            res.append(from_dev(o1, (H, vdim), dt))
        return np.stack(res)
    out = empty(Tq * H * vdim * 4)
    gt = raw(gate, np.float32).ptr if gate is not None else None
    L.vra_stack_op_attention_window(to_dev(q.reshape(Tq, H * dim), dt).ptr, H * dim, out.ptr, kc.ptr, vc.ptr, raw(positions, np.int64).ptr,
                                    raw(table, np.uint32).ptr, raw([k.shape[0]], np.uint32).ptr, raw([0, Tq], np.uint32).ptr, 1, Tq, Tq, H, G, dim, vdim, BS,
                                    len(table), scale, window, sk, hs, gt, H, dt, 0)
    check()
    return from_dev(out, (Tq, H, vdim), dt)


def window_reference(q, k, v, scale, window, sink, head_scale, gate, positions):
    """all keys 0 .. Tk - 1 against queries at `positions` (the oracle's own function takes square prompts: here its parts are put together)"""
    Tk = k.shape[0]
    pos = np.asarray(positions)
    dist = pos[:, None] - np.arange(Tk)[None, :]
    vis = (dist >= 0) & ((dist < window) if window > 0 else True)
    H = q.shape[1]
    hs = scale * (np.ones(H) if head_scale is None else head_scale.astype(np.float64))
    sk = np.full(H, -1e30) if sink is None else sink.astype(np.float64)
    out = so.softmax_window_sink(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), hs, sk, vis)
    return out if gate is None else out * so.sigmoid(gate.astype(np.float64))[:, :, None]


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("decode", [False, True], ids=["prompt", "decoded"])
@pytest.mark.parametrize("window,dim,vdim", [(150, 32, 16), (64, 16, 8), (70, 64, 64), (1, 16, 8), (0, 24, 16)])
def test_window_planted_key(dt, decode, window, dim, vdim):
    """one key stands out among 900 (its value is a marker).  A query at the key's position or up to window - 1 positions behind it returns
    the marker — also across page borders; a query one position further, or before the key, does not feel it at all.  With a sink per
    head, a temperature per head and an output gate per head.  (bf16 prompts: matrix-core kernel for the first and third shape.)"""
    L = _lib.load()
    r = np.random.default_rng(window + dim)
    Tk, H, G = 900, 4, 2
    base_k = so.bf16_round((0.1 * r.standard_normal((Tk, G, dim))).astype(np.float32))
    base_v = so.bf16_round((0.1 * r.standard_normal((Tk, G, vdim))).astype(np.float32))
    u = np.zeros(dim, np.float32)
    u[3] = 1.0
    sink = np.array([-30.0, 0.0, 2.0, -5.0], np.float32)
    head_scale = np.array([1.0, 0.5, 2.0, 1.25], np.float32)
    w = window if window > 0 else Tk
    for j in (0, 63, 64, 400, 899 - min(w - 1, 5)):
        k, v = base_k.copy(), base_v.copy()
        k[j, :, :] = 16.0 * u  # score 8 * 16 * 0.25 = 32 (times the head's scale) against |scores| < 1 elsewhere
        v[j, :, :] = 5.0
        positions = sorted({p for p in (j - 1, j, j + 1, j + w - 2, j + w - 1, j + w, j + w + 1, 899) if 0 <= p < Tk})
        q = np.tile(8.0 * u, (len(positions), H, 1)).astype(np.float32)
        gate = r.standard_normal((len(positions), H)).astype(np.float32)
        got = run_window_attention(L, q, np.array(positions, np.int64), k, v, 0.25, window, sink, head_scale, gate, dt, decode, r)
        ref = window_reference(q, k, v, 0.25, window, sink, head_scale, gate, positions)
        for i, p in enumerate(positions):
            sees = j <= p < j + w
            g = 1.0 / (1.0 + np.exp(-gate[i].astype(np.float64)))
            if sees:
                assert np.abs(got[i] / g[:, None] - 5.0).max() < 3e-2, (j, p)
            else:
                assert np.abs(got[i]).max() < 1.0, (j, p)  # (small values only: the marker has no weight at all)
        assert rel(got, ref) < (2e-5 if dt == F32 else 6e-3)
    # a sink that towers over every score takes all the weight: the output vanishes; a sink far below changes nothing
    k, v = base_k.copy(), base_v.copy()
    positions = [0, 70, 899]
    q = np.tile(8.0 * u, (3, H, 1)).astype(np.float32)
    got = run_window_attention(L, q, np.array(positions, np.int64), k, v, 0.25, window, np.full(H, 60.0, np.float32), None, None, dt, decode, r)
    assert np.abs(got).max() < 1e-20
    a = run_window_attention(L, q, np.array(positions, np.int64), k, v, 0.25, window, np.full(H, -80.0, np.float32), None, None, dt, decode, r)
    assert rel(a, window_reference(q, k, v, 0.25, window, None, None, None, positions)) < (2e-5 if dt == F32 else 6e-3)


def run_scan_ex(L, q, k, v, decay, head_decay, beta, act, q_scale, cuts, slot, state, qk_rep=1):
    T, Hq, D = q.shape
    H, V = v.shape[1], v.shape[2]
    outs, at = [], 0
    for c in cuts:
        sl = slice(at, at + c)
        out = empty(c * H * V * 4)
        f = lambda a: raw(np.ascontiguousarray(a[sl].reshape(c, -1)), np.float32).ptr
        L.vra_stack_op_linear_scan_ex(f(q), Hq * D, f(k), Hq * D, f(v), H * V, f(decay) if decay is not None else None, H, 1 if decay is not None else 0, act,
                                      raw(head_decay, np.float32).ptr if head_decay is not None else None, f(beta) if beta is not None else None, H, q_scale,
                                      state.ptr, raw([slot], np.int32).ptr, raw(np.arange(at, at + c), np.int64).ptr,
                                      raw([0, c], np.uint32).ptr if c > 1 or at == 0 else None, out.ptr, H * V, 1, H, qk_rep, D, V, 0)
        check()
        outs.append(out.numpy(np.float32, (c, H, V)))
        at += c
    return np.concatenate(outs)


@pytest.mark.parametrize("form", ["silu-constant-decay", "delta-decay-per-head"])
@pytest.mark.parametrize("H,rep,D,V", [(2, 1, 8, 8), (3, 1, 5, 7), (4, 2, 16, 24), (2, 2, 128, 128), (1, 1, 200, 9), (2, 1, 24, 300)])
def test_linear_recurrence_forms(form, H, rep, D, V):
    """the recurrence kernel in the two forms of this design against the oracle's token loops: every lane grouping (key sizes 5 .. 200), value
    sizes off the workgroup's column count, grouped q / k heads; one whole step, and portions (down to one token, with single-token steps
    in the decode form) whose state waits in a slot that held another sequence's state before"""
    L = _lib.load()
    r = np.random.default_rng(D * 7 + V)
    T = 75
    q = r.standard_normal((T, H // rep, D)).astype(np.float32)
    k = (r.standard_normal((T, H // rep, D)) / math.sqrt(D)).astype(np.float32)
    v = r.standard_normal((T, H, V)).astype(np.float32)
    q64, k64, v64 = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    if form == "silu-constant-decay":
        head_decay = (0.8 + 0.19 * r.random(H)).astype(np.float32)
        ref = so.constant_decay_recurrence(np.repeat(so.silu(q64), rep, 1) * 0.5, np.repeat(so.silu(k64), rep, 1), so.silu(v64), head_decay.astype(np.float64))
        args = dict(decay=None, head_decay=head_decay, beta=None, act=1)
    else:
        k = k / np.sqrt((k * k).sum(-1, keepdims=True))
        g = (0.7 + 0.3 * r.random((T, H))).astype(np.float32)
        beta = r.random((T, H)).astype(np.float32)
        ref = so.delta_rule_recurrence(q64 * 0.5, k.astype(np.float64), v64, beta.astype(np.float64), g.astype(np.float64))
        args = dict(decay=g, head_decay=None, beta=beta, act=0)
    state = raw(r.standard_normal(3 * H * V * D).astype(np.float32) * 100.0, np.float32)  # (what earlier sequences left: must not be felt)
    run = lambda cuts, slot: run_scan_ex(L, q, k, v, args["decay"], args["head_decay"], args["beta"], args["act"], 0.5, cuts, slot, state, rep)
    whole = run([T], 1)
    assert rel(whole, ref) < 1e-5
    parts = run([1, 1, 2, 16, 1, 17, 32, 1, 4], 2)
    assert rel(parts, ref) < 1e-5 and np.abs(parts - whole).max() <= 1e-6 * np.abs(whole).max()
    assert rel(run([40, 35], 1), ref) < 1e-5  # the slot of the first run, used again


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("C,blocks,taps", [(48, 3, 4), (14, 2, 3), (200, 1, 1), (512, 4, 2)])
def test_convolution_and_gated_recurrence(dt, C, blocks, taps):
    """the short convolution with its state and the gated diagonal recurrence against the oracle, for two sequences of one step, whole and
    in portions (cuts shorter than the taps, single tokens in the decode form), the states waiting in slots that held other values; decays
    close to one included (lam far below zero)"""
    L = _lib.load()
    r = np.random.default_rng(C + taps)
    lens, bw = [53, 20], C // blocks
    w = (0.4 * r.standard_normal((C, taps)) + 0.3).astype(np.float32)
    bias = (0.2 * r.standard_normal(C)).astype(np.float32)
    lam = np.concatenate([np.full(C // 2, -9.0), r.standard_normal(C - C // 2)]).astype(np.float32)
    seqs = []
    for n in lens:
        x, gr, gi, y = (r.standard_normal((n, C)).astype(np.float32) for _ in range(4))
        u = so.causal_conv(x.astype(np.float64), w.astype(np.float64), bias.astype(np.float64))
        ref = so.gated_diagonal_recurrence(u, so.sigmoid(gr.astype(np.float64)), so.sigmoid(gi.astype(np.float64)), lam.astype(np.float64)) * so.gelu_tanh(y.astype(np.float64))
        seqs.append((x, gr, gi, y, u, ref))
    conv_state = raw(r.standard_normal(4 * max(taps - 1, 1) * C).astype(np.float32) * 50.0, np.float32)
    state = raw(r.standard_normal(4 * C).astype(np.float32) * 50.0, np.float32)

    def blocked(g):  # gate logits as the block-diagonal product leaves them: per block the recurrence gate's columns, then the input gate's
        gr, gi = g
        n = gr.shape[0]
        return np.concatenate([gr.reshape(n, blocks, bw), gi.reshape(n, blocks, bw)], -1).reshape(n, 2 * C)

    def run(cuts_per_seq, slots):
        got = [[] for _ in seqs]
        at = [0] * len(seqs)
        for step in range(max(len(c) for c in cuts_per_seq)):
            live = [s for s in range(len(seqs)) if step < len(cuts_per_seq[s])]
            cs = [cuts_per_seq[s][step] for s in live]
            T = sum(cs)
            decode_form = all(c == 1 for c in cs) and all(at[s] > 0 for s in live)
            cat = lambda i: np.concatenate([seqs[s][i][at[s]:at[s] + c] for s, c in zip(live, cs)])
            pos = np.concatenate([np.arange(at[s], at[s] + c) for s, c in zip(live, cs)]).astype(np.int64)
            cu = None if decode_form else raw(np.concatenate([[0], np.cumsum(cs)]), np.uint32).ptr
            sl = raw([slots[s] for s in live], np.int32).ptr
            ud = empty(T * C * 4)
            L.vra_stack_op_conv_rows(raw(cat(0), np.float32).ptr, C, C, taps, raw(w, np.float32).ptr, raw(bias, np.float32).ptr, conv_state.ptr, 0, ud.ptr, C,
                                     raw(pos, np.int64).ptr, cu, sl, T, len(live), 0)
            check()
            g = raw(blocked((cat(1), cat(2))), np.float32)
            out = empty(T * C * 4)
            L.vra_stack_op_gated_scan(ud.ptr, C, g.ptr, g.ptr + 4 * bw, 2 * C, bw, raw(cat(3), np.float32).ptr, C, raw(lam, np.float32).ptr, 8.0, state.ptr, sl,
                                      raw(pos, np.int64).ptr, cu, out.ptr, C, len(live), C, T, dt, 0)
            check()
            o = from_dev(out, (T, C), dt)
            uo = ud.numpy(np.float32, (T, C))
            o0 = 0
            for s, c in zip(live, cs):
                assert rel(uo[o0:o0 + c], seqs[s][4][at[s]:at[s] + c]) < 1e-6
                got[s].append(o[o0:o0 + c])
                o0 += c
                at[s] += c
        return [np.concatenate(g) for g in got]
    tol = 2e-5 if dt == F32 else 6e-3
    whole = run([[n] for n in lens], [1, 3])
    parts = run([[1, 2, 1, 1, 30, 1, 17], [2, 1, 1, 1, 15]], [3, 0])  # (slot 3 held the other sequence before)
    for s in range(len(seqs)):
        assert rel(whole[s], seqs[s][5]) < tol and rel(parts[s], seqs[s][5]) < tol
        assert rel(parts[s], whole[s]) < (1e-6 if dt == F32 else 6e-3)


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("W,E,ident,top,groups,keep", [(96, 6, 3, 3, 3, 2), (51, 3, 0, 3, 0, 0), (256, 36, 4, 1, 8, 3), (64, 6, 2, 4, 4, 1), (128, 70, 2, 3, 8, 3)])
def test_seam_with_dynamic_tanh_and_grouped_router(dt, W, E, ident, top, groups, keep):
    """x += D(c1 N(part1) + c2 N(part2); post), h = D(x; pre) with D = tanh(alpha v) w + b and N an RMS norm of the part's own; then pairs
    without a row and a weighted second part; the router: softmax over all outputs, choice by corrected score inside the best groups,
    weights = the plain scores, identity experts as expert -1 with their weights summed.  Planted: a towering logit inside a group that the
    correction pushes out; equal logits (the lower index wins)."""
    L = _lib.load()
    r = np.random.default_rng(W + E)
    T, eps, n = 9, 1e-5, E + ident
    f = lambda *s: r.standard_normal(s).astype(np.float32)
    x, p1, p2 = f(T, W), 3.0 * f(T, W), 0.2 * f(T, W)
    n1w, n2w, post, post_b, pre, pre_b = (1 + 0.2 * f(W)), (1 + 0.2 * f(W)), (1 + 0.2 * f(W)), 0.1 * f(W), (1 + 0.2 * f(W)), 0.1 * f(W)
    rw = so.bf16_round(3.0 * f(n, W) / math.sqrt(W))
    corr = (0.05 * f(n)).astype(np.float32)
    s = 0.5 * (so.rms(p1.astype(np.float64), eps) * n1w + so.rms(p2.astype(np.float64), eps) * n2w)
    x_ref = x + np.tanh(0.7 * s) * post + post_b
    h_ref = np.tanh(0.4 * x_ref) * pre + pre_b
    router = dict(experts=E, identity=ident, top=top)
    if groups:
        router["groups"] = dict(count=groups, keep=keep)
    chosen, wt = so.route(h_ref, router, {"router": rw.astype(np.float64), "correction": corr.astype(np.float64)}, "")
    xd, hd, h32 = raw(x, np.float32), empty(T * W * 4), empty(T * W * 4)
    pe, pwt, idw = empty(T * top * 4), empty(T * top * 4), empty(T * 4)
    d = lambda a: raw(a, np.float32).ptr

    def seam(xd, p1, n1, pw, pe_in, c1, p2, p2w, c2, n1w, n2w, post, post_b, pa, rw, corr):
        L.vra_stack_op_seam(xd.ptr, p1, n1, pw, pe_in, c1, p2, p2w, c2, n1w, n2w, 1, post, post_b, pa, d(pre), d(pre_b), 0.4, hd.ptr, h32.ptr, eps, T, W,
                            to_dev(rw, dt).ptr, d(corr), 1, n, top, groups, keep, ident, pe.ptr, pwt.ptr, idw.ptr, dt, 0)
        check()
        return pe.numpy(np.int32, (T, top)), pwt.numpy(np.float32, (T, top)), idw.numpy(np.float32, (T,))
    experts, weights, idsum = seam(xd, d(p1), 1, None, None, 0.5, d(p2), None, 0.5, d(n1w), d(n2w), d(post), d(post_b), 0.7, rw, corr)
    assert rel(xd.numpy(np.float32, (T, W)), x_ref) < 1e-6 and rel(h32.numpy(np.float32, (T, W)), h_ref) < 1e-6
    assert rel(from_dev(hd, (T, W), dt), h_ref) < (1e-6 if dt == F32 else 4e-3)
    for t in range(T):
        want = [int(e) if e < E else -1 for e in chosen[t]]
        assert sorted(experts[t].tolist()) == sorted(want), t
        assert np.allclose(np.sort(weights[t]), np.sort(wt[t]), atol=2e-6 if dt == F32 else 1e-2)
        assert abs(idsum[t] - sum(a for e, a in zip(chosen[t], wt[t]) if e >= E)) < (1e-5 if dt == F32 else 2e-2)
    # pairs without a row are left out (their rows hold NaN), the second part enters with its per-row weight
    n1 = 3
    q1 = f(T * n1, W)
    pw = r.random(T * n1).astype(np.float32)
    miss = (r.random(T * n1) < 0.4)
    q1[miss] = np.nan
    pe_in = np.where(miss, -1, 2).astype(np.int32)
    p2w = r.random(T).astype(np.float32)
    s = np.where(miss[:, None], 0.0, pw[:, None] * q1).reshape(T, n1, W).sum(1).astype(np.float64) + p2w[:, None] * p2
    x2 = raw(x, np.float32)
    seam(x2, d(q1), n1, d(pw), raw(pe_in, np.int32).ptr, 1.0, d(p2), d(p2w), 1.0, None, None, d(post), d(post_b), 0.7, rw, corr)
    assert rel(x2.numpy(np.float32, (T, W)), x + np.tanh(0.7 * s) * post + post_b) < 1e-6
    # planted logits: all rows of the router equal, so the logits are the same for every expert and the correction decides alone
    if groups and keep < groups and top <= (n // groups) * keep:
        per = n // groups
        c2 = np.zeros(n, np.float32)
        c2[n - 1] = 0.5          # the best corrected score sits in the last group ...
        c2[0] = 0.25             # ... the next in the first
        experts, weights, _ = seam(raw(x, np.float32), None, 1, None, None, 1.0, None, None, 1.0, None, None, None, None, 1.0, np.zeros((n, W), np.float32), c2)
        kept = [groups - 1, 0] + list(range(1, groups - 1))
        allowed = {e for g in kept[:keep] for e in range(g * per, (g + 1) * per)}
        for t in range(T):
            picked = {int(e) if e >= 0 else -1 for e in experts[t]}
            real = {e for e in picked if e >= 0}
            assert real <= allowed and np.allclose(weights[t], 1.0 / n, atol=1e-6)  # the weights are the plain scores: the correction is not in them
            assert (n - 1 in picked) if ident == 0 else (-1 in picked)
    # equal logits and no correction: the lowest indices win
    experts, weights, _ = seam(raw(x, np.float32), None, 1, None, None, 1.0, None, None, 1.0, None, None, None, None, 1.0, np.zeros((n, W), np.float32), np.zeros(n, np.float32))
    if not groups or keep >= groups or top <= n // groups:
        assert (experts == np.where(np.arange(top) < E, np.arange(top), -1)[None, :]).all() and np.allclose(weights, 1.0 / n)
