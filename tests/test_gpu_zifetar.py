"""GPU tests of the Zifetar design in the layer-stack model class: every mechanism alone (one-layer models), then whole models of small
random configurations through the engine — against tests/zifetar_oracle.py (float64, whole sequences, no cache, no pages, no slots).

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

from tests import zifetar_oracle as zo
from tests.test_gpu_stack import BF16, F32, TOL, build, rel, tokens_of
from vllm_rs_amd import checkpoint

pytestmark = pytest.mark.gpu

EMB = dict(scale=3.5, bigram=dict(buckets=53, mul_prev=11, mul_cur=5))
MOE = dict(kind="moe", expert=dict(ff=40), router=dict(experts=5, top=2))


def delta(heads=4, kv_heads=2, dim=16, vdim=24, conv=4):
    return dict(type="channel_delta", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv))


def retention(heads=3, dim=24, vdim=16, decay=(0.9, 0.99, 0.999), dims=16, base=5000.0):
    m = dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay))
    if dims:
        m["rot"] = dict(base=base, dims=dims)
    return dict(type="retention", mixer=m)


def parallel(heads=6, kv_heads=3, dim=16, vdim=24, size=70, dims=8, scaling=True, r_heads=2, r_dim=24, r_vdim=16, tau=8.0, ls=0.7, rs=1.2, scale=0.3):
    rot = dict(base=2000.0, dims=dims)
    if scaling:
        rot["scaling"] = dict(factor=4.0, low=1.0, high=3.0, original=48)
    left = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, rot=rot)
    if size:
        left["mask"] = dict(size=size)
    return dict(type="parallel", mixer=dict(left=left, right=dict(heads=r_heads, dim=r_dim, vdim=r_vdim, tau=tau), left_scale=ls, right_scale=rs))


def config(layers, width=96, vocab=160, eps=1e-5, emb=EMB):
    return dict(architecture="Zifetar", width=width, vocab=vocab, norm=dict(eps=eps), embedding=emb, layers=layers)


def config_a():
    """every mixer, grouped q / k heads in the delta rule, key size != value size everywhere, rotary on part of a head, a block mask longer
    than a page, a layer without feed-forward, top 1 and top = experts routers"""
    return config([
        dict(parallel(), mlp=MOE),
        dict(delta(), mlp=dict(kind="moe", expert=dict(ff=24), router=dict(experts=3, top=3))),
        dict(retention(), mlp=None),
        dict(parallel(heads=4, kv_heads=4, dim=24, vdim=16, size=0, dims=24, scaling=False, r_heads=3, r_dim=8, r_vdim=8, tau=2.0), mlp=MOE),
        dict(delta(heads=2, kv_heads=2, dim=8, vdim=8, conv=2), mlp=dict(kind="moe", expert=dict(ff=16), router=dict(experts=4, top=1))),
        dict(retention(heads=2, dim=8, vdim=24, decay=(0.5, 0.9995), dims=0), mlp=MOE),
    ])


def config_b():
    """sizes off every 16-byte path: width 50, heads of 5 / 7 / 6 channels, a block mask of 9 positions, convolutions of 3 taps"""
    moe = dict(kind="moe", expert=dict(ff=11), router=dict(experts=3, top=2))
    return config([
        dict(retention(heads=2, dim=6, vdim=5, decay=(0.8, 0.97), dims=4, base=100.0), mlp=moe),
        dict(parallel(heads=2, kv_heads=1, dim=6, vdim=7, size=9, dims=2, r_heads=2, r_dim=5, r_vdim=7, tau=3.0, ls=1.1, rs=0.4, scale=0.5), mlp=moe),
        dict(delta(heads=2, kv_heads=1, dim=5, vdim=7, conv=3), mlp=None),
    ], width=50, vocab=70, eps=1e-6, emb=dict(scale=2.0, bigram=dict(buckets=17, mul_prev=3, mul_cur=2)))


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


# ------------------------------------------------------------------------------------------------ each mechanism alone
ALONE = {
    "delta": [delta()],
    "delta-one-group-conv1": [delta(heads=3, kv_heads=1, dim=8, vdim=40, conv=1)],
    "delta-wide": [delta(heads=2, kv_heads=2, dim=128, vdim=128, conv=3)],
    "retention": [retention()],
    "retention-full-rotary": [retention(heads=2, dim=64, vdim=48, decay=(0.97, 0.999), dims=64, base=2e5)],
    "retention-no-rotary": [retention(dims=0)],
    "attention-branch": [parallel(rs=0.0)],
    "attention-branch-plain-causal": [parallel(size=0, scaling=False, rs=0.0)],
    "linear-branch": [parallel(ls=0.0)],
    "parallel": [parallel()],
    "experts": [dict(retention(), mlp=MOE)],
    "experts-top1": [dict(retention(), mlp=dict(kind="moe", expert=dict(ff=24), router=dict(experts=7, top=1)))],
}


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("name", sorted(ALONE))
def test_each_mechanism_alone(name, dt):
    """one layer of one kind (no feed-forward unless it is the subject): a 150-token prompt whole, then the same prompt in portions with
    single tokens between them — the layer's output and the logits against the oracle"""
    layers = [dict(dict(mlp=None), **x) for x in ALONE[name]]
    cfg = config(layers)
    tensors = zo.random_tensors(cfg, 7)
    toks = tokens_of(cfg, 150, 3)
    lay = []
    ref = zo.forward(cfg, tensors, toks, lay)
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


def test_embedding_pairs_and_first_token():
    """the token-pair row depends on the previous token also across a step's cut and in decoding; the first token takes the table's last row:
    sequences of one and two tokens, and the same token at position 0 and behind another one"""
    cfg = config([dict(retention(), mlp=None)])
    tensors = zo.random_tensors(cfg, 9)
    eng = build(cfg, tensors, F32, blocks=4, max_model_len=128)
    for toks in ([5], [5, 5], [7, 5], [5, 7, 5, 5]):
        ref = zo.forward(cfg, tensors, toks)
        whole = eng.replay_step([(1, toks, every(len(toks)))], [1])
        agree(whole, ref, F32, str(toks))
        one = np.stack([eng.replay_step([(2, toks[p:p + 1], [0])], [2] if p == len(toks) - 1 else [])[0] for p in range(len(toks))])
        agree(one, ref, F32, str(toks) + " token by token")
    a = zo.forward(cfg, tensors, [7, 5])[1]
    b = zo.forward(cfg, tensors, [9, 5])[1]
    assert np.abs(a - b).max() > 1e-3  # (the oracle's pair row does depend on the previous token)
    eng.close()


@pytest.mark.parametrize("decode", [False, True], ids=["prompt", "decoded"])
@pytest.mark.parametrize("size", [7, 64, 70])
def test_block_mask_edges(size, decode):
    """softmax branch alone: a changed token reaches the positions of its own block of `size` positions (and, through the pair table, its
    successor) and nothing behind the block's edge — exactly; the first position of a block sees one key.  Portions cut inside blocks."""
    cfg = config([dict(parallel(size=size, rs=0.0, heads=4, kv_heads=2), mlp=None)])
    tensors = zo.random_tensors(cfg, 11)
    n = 3 * size + 5
    toks = tokens_of(cfg, n, 4)
    other = list(toks)
    at = size + size // 2          # a token inside the second block
    other[at] = (toks[at] + 3) % cfg["vocab"]
    ref_a, ref_b = zo.forward(cfg, tensors, toks), zo.forward(cfg, tensors, other)
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
    edge = 2 * size
    changed = np.abs(a - b).max(-1)
    ref_changed = np.abs(ref_a - ref_b).max(-1)
    assert (changed[:at] == 0).all() and (changed[edge:] == 0).all() and (ref_changed[edge:] < 1e-12).all()
    assert (changed[at:edge] > 1e-5).all() and (ref_changed[at:edge] > 1e-5).all()
    # the first position of the third block: one key, its own; the last of the second: all of its block
    assert rel(a[edge], ref_a[edge]) < 3e-5 and rel(a[edge - 1], ref_a[edge - 1]) < 3e-5


@pytest.mark.parametrize("kind", ["retention", "delta", "linear-branch"])
def test_a_far_token_stays_in_the_state(kind):
    """a token hundreds of positions back reaches the last logits only through the matrix state (slow decays; the delta rule's writes wear
    it down faster, so its prompt is shorter): whole prompt, decoding across page borders and 2-token portions give the oracle's logits,
    which do depend on that token"""
    layer = {"retention": retention(heads=2, dim=16, vdim=16, decay=(0.9995, 0.999), dims=8),
             "delta": delta(heads=2, kv_heads=2, dim=64, vdim=16, conv=2),
             "linear-branch": parallel(ls=0.0, tau=64.0)}[kind]
    cfg = config([dict(layer, mlp=None)])
    tensors = zo.random_tensors(cfg, 13)
    if kind == "delta":  # slow decays: a strongly negative step-size bias; write strengths of one half
        tensors["l0.mix.dt_bias"] = zo.bf16_round(np.full_like(tensors["l0.mix.dt_bias"], -9.0))
        tensors["l0.mix.b"] = np.zeros_like(tensors["l0.mix.b"])
    if kind == "linear-branch":
        tensors["l0.mix.right.a2.b"] = zo.bf16_round(np.full_like(tensors["l0.mix.right.a2.b"], 6.0))
    n = 260 if kind == "delta" else 640
    toks = tokens_of(cfg, n, 5)
    other = list(toks)
    other[20] = (toks[20] + 1) % cfg["vocab"]
    ref_a, ref_b = zo.forward(cfg, tensors, toks)[-1], zo.forward(cfg, tensors, other)[-1]
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
    tensors = zo.random_tensors(cfg, 17 if name == "a" else 18, rank=8 if name == "a" else 3)
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
    layers = []
    ref = zo.forward(cfg, tensors, toks, layers)
    for i, x in enumerate(layers):
        agree(trace[i], x, dt, f"layer {i}")
    agree(got, ref, dt)


def test_prefill_against_token_by_token_decoding(model):
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 150, 2)
    ref = zo.forward(cfg, tensors, toks)
    whole = eng.replay_step([(1, toks, every(150))], [1])
    agree(whole, ref, dt, "whole")
    one = np.stack([eng.replay_step([(2, toks[p:p + 1], [0])], [2] if p == 149 else [])[0] for p in range(150)])
    agree(one, ref, dt, "token by token")
    assert rel(one, whole) < (1e-5 if dt == F32 else 3e-2)


@pytest.mark.parametrize("sizes", [[2] * 30, [37, 3, 37, 2, 5], [64, 64, 2], [63, 2, 63, 2], [1, 5, 1, 1, 70, 1], [71, 9, 2, 70]])
def test_portions(model, sizes):
    """a prompt cut anywhere (down to two tokens, at and across page borders and block-mask edges, shorter than the convolutions) gives
    the logits of the whole prompt"""
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
    agree(got, zo.forward(cfg, tensors, toks), dt)


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
    ref = [zo.forward(cfg, tensors, p) for p in prompts]
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
    agree(eng.replay_step([(505, toks, every(10))], [505]), zo.forward(cfg, tensors, toks), dt)


def test_long_decoding(model):
    """310 decoded tokens behind a 20-token prompt: block-mask edges, page borders and the state pass under decoded tokens"""
    cfg, tensors, dt, eng = model
    toks = tokens_of(cfg, 330, 5)
    ref = zo.forward(cfg, tensors, toks)
    eng.replay_step([(1, toks[:20], [])], [])
    rows = [eng.replay_step([(1, toks[p:p + 1], [0])], [1] if p == len(toks) - 1 else [])[0] for p in range(20, len(toks))]
    agree(np.stack(rows), ref[20:], dt)


def test_long_prompt_in_one_step_and_in_portions():
    """a 1500-token prompt through heads of 64 / 128 channels (bf16 prompt steps of this size take the matrix-core attention and matrix
    kernels), whole and in three portions"""
    cfg = config([dict(parallel(heads=4, kv_heads=2, dim=64, vdim=32, size=192, dims=32, r_heads=2, r_dim=32, r_vdim=64, scale=0.11), mlp=MOE),
                  dict(delta(heads=2, kv_heads=1, dim=64, vdim=64, conv=3), mlp=None),
                  dict(retention(heads=2, dim=128, vdim=64, decay=(0.99, 0.9995), dims=32), mlp=MOE)], width=128)
    tensors = zo.random_tensors(cfg, 23)
    toks = tokens_of(cfg, 1500, 8)
    want = list(range(0, 1500, 47)) + [191, 192, 193, 1499]
    want.sort()
    ref = zo.forward(cfg, tensors, toks)[want]
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
    tensors = zo.random_tensors(cfg, 19)
    eng = build(cfg, tensors, F32, blocks=16, max_model_len=256, use_graph=use_graph, num_state_slots=2)
    prompts = [tokens_of(cfg, n, 60 + n) for n in (5, 70, 31)]
    outs = eng.generate(prompts, max_tokens=12, ignore_eos=True)
    eng.close()
    for p, out in zip(prompts, outs):
        seq = list(p)
        for t in out:
            lg = zo.forward(cfg, tensors, seq)[-1]
            top2 = np.sort(lg)[-2:]
            assert int(t) == int(lg.argmax()) or top2[1] - top2[0] < 1e-3, (len(p), len(seq))
            seq.append(int(t))
        assert len(out) == 12


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
    tensors = zo.random_tensors(cfg, 31)
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
    r1, r2, r3 = (zo.forward(cfg, tensors, p) for p in (p1, p2, p3))
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
from tests.test_gpu_stack import check, empty, from_dev, paged, raw, to_dev  # noqa: E402
from vllm_rs_amd import _lib  # noqa: E402


def masked_softmax(q, k, v, scale, vis):
    """q [Tq, H, D] against ALL keys k [Tk, G, D] under the visibility matrix vis [Tq, Tk] (the oracle's attention takes square prompts)"""
    Tq, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((Tq, H, v.shape[-1]))
    for hd in range(H):
        g = hd // (H // G)
        s = np.where(vis, (q[:, hd] @ k[:, g].T) * scale, -np.inf)
        e = np.exp(s - s.max(-1, keepdims=True))
        out[:, hd] = (e / e.sum(-1, keepdims=True)) @ v[:, g]
    return out


def run_masked_attention(L, q, positions, k, v, scale, chunk, dt, decode, r, BS=64):
    Tq, H, dim = q.shape
    G, vdim = k.shape[1], v.shape[2]
    kc, vc, table = paged(k, v, BS, r, dt)
    if decode:
        res = []
        for i in range(Tq):
            o1 = empty(H * vdim * 4)
            qi = to_dev(q[i].reshape(1, H * dim), dt)
            L.vra_stack_op_attention_chunk(qi.ptr, H * dim, o1.ptr, kc.ptr, vc.ptr, raw([positions[i]], np.int64).ptr, raw(table, np.uint32).ptr,
                                           raw([positions[i] + 1], np.uint32).ptr, None, 1, 1, 1, H, G, dim, vdim, BS, len(table), scale, chunk, dt, 0)
            check()
            res.append(from_dev(o1, (H, vdim), dt))
        return np.stack(res)
    out = empty(Tq * H * vdim * 4)
    L.vra_stack_op_attention_chunk(to_dev(q.reshape(Tq, H * dim), dt).ptr, H * dim, out.ptr, kc.ptr, vc.ptr, raw(positions, np.int64).ptr,
                                   raw(table, np.uint32).ptr, raw([k.shape[0]], np.uint32).ptr, raw([0, Tq], np.uint32).ptr, 1, Tq, Tq, H, G, dim, vdim, BS,
                                   len(table), scale, chunk, dt, 0)
    check()
    return from_dev(out, (Tq, H, vdim), dt)


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("decode", [False, True], ids=["prompt", "decoded"])
@pytest.mark.parametrize("chunk,dim,vdim", [(150, 32, 16), (64, 16, 8), (70, 64, 64), (1, 16, 8)])
def test_block_mask_planted_key(dt, decode, chunk, dim, vdim):
    """one key stands out among 900 (its value is a marker).  A query in the key's own block of positions and not before it returns the
    marker — at the block's first and last position, across page borders; a query of the next block, or of the block before, or before
    the key inside its block, does not feel it at all.  (bf16 prompts: matrix-core kernel for the first and third shape, FMA otherwise.)"""
    L = _lib.load()
    r = np.random.default_rng(chunk + dim)
    Tk, H, G = 900, 4, 2
    base_k = zo.bf16_round((0.1 * r.standard_normal((Tk, G, dim))).astype(np.float32))
    base_v = zo.bf16_round((0.1 * r.standard_normal((Tk, G, vdim))).astype(np.float32))
    u = np.zeros(dim, np.float32)
    u[3] = 1.0
    for j in (0, chunk - 1, chunk, 3 * chunk + chunk // 2, (899 // chunk) * chunk):
        if j >= Tk:
            continue
        k, v = base_k.copy(), base_v.copy()
        k[j, :, :] = 16.0 * u  # score 8 * 16 * 0.25 = 32 against |scores| < 1 elsewhere
        v[j, :, :] = 5.0
        lo, hi = j // chunk * chunk, min((j // chunk + 1) * chunk, Tk)
        positions = sorted({p for p in (lo - 1, lo, j - 1, j, j + 1, hi - 1, hi, hi + 1, 899) if 0 <= p < Tk})
        q = np.tile(8.0 * u, (len(positions), H, 1)).astype(np.float32)
        got = run_masked_attention(L, q, np.array(positions, np.int64), k, v, 0.25, chunk, dt, decode, r)
        for i, p in enumerate(positions):
            sees = lo <= j <= p < hi
            if sees:
                assert np.abs(got[i] - 5.0).max() < 2e-2, (j, p)
            else:
                assert np.abs(got[i]).max() < 1.0, (j, p)  # (small values only: the marker has no weight at all)
        vis = np.array([[(kk <= p) and (kk // chunk == p // chunk) for kk in range(Tk)] for p in positions])
        ref = masked_softmax(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), 0.25, vis)
        assert rel(got, ref) < (2e-5 if dt == F32 else 6e-3)


def run_scan(L, q, k, v, decay, head_decay, beta, q_scale, cuts, slots, state, n_slots, qk_rep=1):
    """the recurrence over ONE sequence given in portions `cuts`, its state in slot `slots` of `state` (a device buffer that persists)"""
    T, Hq, D = q.shape
    H, V = v.shape[1], v.shape[2]
    outs, at = [], 0
    for c in cuts:
        sl = slice(at, at + c)
        out = empty(c * H * V * 4)
        f = lambda a: raw(np.ascontiguousarray(a[sl].reshape(c, -1)), np.float32).ptr
        L.vra_stack_op_linear_scan(f(q), Hq * D, f(k), Hq * D, f(v), H * V, f(decay) if decay is not None else None, H * D,
                                   raw(head_decay, np.float32).ptr if head_decay is not None else None, f(beta) if beta is not None else None, H, q_scale,
                                   state.ptr, raw([slots], np.int32).ptr, raw(np.arange(at, at + c), np.int64).ptr, raw([0, c], np.uint32).ptr if c > 1 or at == 0 else None,
                                   out.ptr, H * V, 1, H, qk_rep, D, V, 0)
        check()
        outs.append(out.numpy(np.float32, (c, H, V)))
        at += c
    return np.concatenate(outs)


@pytest.mark.parametrize("form", ["head-decay", "row-decay", "delta"])
@pytest.mark.parametrize("H,rep,D,V", [(2, 1, 8, 8), (3, 1, 5, 7), (4, 2, 16, 24), (2, 1, 64, 40), (2, 2, 128, 128), (1, 1, 200, 9), (2, 1, 24, 300)])
def test_linear_recurrence_alone(form, H, rep, D, V):
    """the recurrence kernel against the oracle's token loop: every lane grouping (key sizes 5 .. 200), value sizes off the workgroup's
    column count, grouped q / k heads; one whole step, and portions (down to one token, with single-token steps in the decode form) whose
    state waits in a slot that held another sequence's state before"""
    L = _lib.load()
    r = np.random.default_rng(D * 7 + V)
    T = 75
    q = r.standard_normal((T, H // rep, D)).astype(np.float32)
    k = (r.standard_normal((T, H // rep, D)) / math.sqrt(D)).astype(np.float32)
    v = r.standard_normal((T, H, V)).astype(np.float32)
    decay = head_decay = beta = None
    if form == "head-decay":
        head_decay = (0.8 + 0.19 * r.random(H)).astype(np.float32)
        dd = np.broadcast_to(head_decay[None, :, None], (T, H, D))
    else:
        decay = (0.7 + 0.3 * r.random((T, H, D))).astype(np.float32)
        dd = decay
    if form == "delta":
        beta = r.random((T, H)).astype(np.float32)
        k = k / np.sqrt((k * k).sum(-1, keepdims=True))
    ref = zo.linear_recurrence(np.repeat(q, rep, 1).astype(np.float64) * 0.5, np.repeat(k, rep, 1).astype(np.float64), v.astype(np.float64),
                               np.asarray(dd, np.float64), None if beta is None else beta.astype(np.float64))
    n_slots = 3
    state = raw(r.standard_normal(n_slots * H * V * D).astype(np.float32) * 100.0, np.float32)  # (what earlier sequences left: must not be felt)
    whole = run_scan(L, q, k, v, decay, head_decay, beta, 0.5, [T], 1, state, n_slots, rep)
    assert rel(whole, ref) < 1e-5
    parts = run_scan(L, q, k, v, decay, head_decay, beta, 0.5, [1, 1, 2, 16, 1, 17, 32, 1, 4], 2, state, n_slots, rep)
    assert rel(parts, ref) < 1e-5 and np.abs(parts - whole).max() <= 1e-6 * np.abs(whole).max()
    again = run_scan(L, q, k, v, decay, head_decay, beta, 0.5, [40, 35], 1, state, n_slots, rep)  # the slot of the first run, used again
    assert rel(again, ref) < 1e-5



@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("W,E,top", [(96, 5, 2), (51, 3, 3), (256, 40, 1), (64, 8, 4)])
def test_seam_norms_and_router(dt, W, E, top):
    """x += N(c1 sum_j w_j part_j + c2 part2; post), h = N(x; pre), router: biased logits on h, the `top` largest, softmax over those alone.
    One logit is planted far above the rest in some rows (its weight is then 1 up to e^-20) and two equal logits in another (the lower index wins)."""
    L = _lib.load()
    r = np.random.default_rng(W + E)
    T, n1, eps = 9, 3, 1e-5
    x = r.standard_normal((T, W)).astype(np.float32)
    p1 = r.standard_normal((T * n1, W)).astype(np.float32)
    pw = r.random(T * n1).astype(np.float32)
    p2 = r.standard_normal((T, W)).astype(np.float32)
    post, pre = (1 + 0.2 * r.standard_normal(W)).astype(np.float32), (1 + 0.2 * r.standard_normal(W)).astype(np.float32)
    rw = zo.bf16_round((r.standard_normal((E, W)) / math.sqrt(W)).astype(np.float32))
    rb = (0.3 * r.standard_normal(E)).astype(np.float32)
    s = 0.75 * (pw[:, None] * p1).reshape(T, n1, W).sum(1).astype(np.float64) + 1.25 * p2
    x_ref = x + zo.rms(s, eps) * post
    h_ref = zo.rms(x_ref, eps) * pre
    z = h_ref @ rw.T.astype(np.float64) + rb
    xd, hd = raw(x, np.float32), empty(T * W * 4)
    pe, pwt = empty(T * top * 4), empty(T * top * 4)
    L.vra_stack_op_sandwich_norm(xd.ptr, raw(p1, np.float32).ptr, n1, raw(pw, np.float32).ptr, 0.75, raw(p2, np.float32).ptr, 1.25, raw(post, np.float32).ptr,
                                 raw(pre, np.float32).ptr, hd.ptr, eps, T, W, to_dev(rw, dt).ptr, raw(rb, np.float32).ptr, E, top, pe.ptr, pwt.ptr, dt, 0)
    check()
    assert rel(xd.numpy(np.float32, (T, W)), x_ref) < 1e-6
    assert rel(from_dev(hd, (T, W), dt), h_ref) < (1e-6 if dt == F32 else 4e-3)
    experts, weights = pe.numpy(np.int32, (T, top)), pwt.numpy(np.float32, (T, top))
    for t in range(T):
        order = np.argsort(-z[t], kind="stable")[:top]
        gap = np.sort(z[t])[::-1]
        if top < E and gap[top - 1] - gap[top] < 1e-3:
            continue  # (a close call at the cut: either choice is right to rounding)
        assert sorted(experts[t].tolist()) == sorted(order.tolist()), t
        e = np.exp(z[t, experts[t]] - z[t, experts[t]].max())
        assert np.allclose(weights[t], e / e.sum(), atol=2e-5 if dt == F32 else 2e-2) and abs(weights[t].sum() - 1.0) < 1e-5
    # a towering logit takes all the weight; equal logits go to the lower index
    big = rb.copy()
    big[E - 1] = 40.0
    L.vra_stack_op_sandwich_norm(xd.ptr, None, 1, None, 1.0, None, 1.0, None, raw(pre, np.float32).ptr, hd.ptr, eps, T, W, to_dev(np.zeros((E, W), np.float32), dt).ptr,
                                 raw(big, np.float32).ptr, E, top, pe.ptr, pwt.ptr, dt, 0)
    check()
    experts, weights = pe.numpy(np.int32, (T, top)), pwt.numpy(np.float32, (T, top))
    assert (experts[:, 0] == E - 1).all() and (weights[:, 0] > 1.0 - 1e-6 * top).all()
    L.vra_stack_op_sandwich_norm(xd.ptr, None, 1, None, 1.0, None, 1.0, None, raw(pre, np.float32).ptr, hd.ptr, eps, T, W, to_dev(np.zeros((E, W), np.float32), dt).ptr,
                                 raw(np.zeros(E, np.float32), np.float32).ptr, E, top, pe.ptr, pwt.ptr, dt, 0)
    check()
    experts, weights = pe.numpy(np.int32, (T, top)), pwt.numpy(np.float32, (T, top))
    assert (experts == np.arange(top)[None, :]).all() and np.allclose(weights, 1.0 / top)
