"""CPU tests of the Zifetar design in the layer-stack model class: the reader of its config.json (every size and constant, optional
mechanisms), the native parser of the layer list it writes and the scheduler's state slots (host-only engine: no GPU touched), and the
float64 oracle's mechanisms checked by hand (tests/zifetar_oracle.py)."""
import ctypes as C
import math

import numpy as np
import pytest

from tests import zifetar_oracle as zo
from vllm_rs_amd import _lib, checkpoint
from vllm_rs_amd.engine import model_config


def small_config():
    moe = dict(kind="moe", expert=dict(ff=20), router=dict(experts=5, top=2))
    left = dict(heads=4, kv_heads=2, dim=8, vdim=6, scale=0.4, mask=dict(size=9), rot=dict(base=300.0, dims=4, scaling=dict(factor=4.0, low=1.0, high=3.0, original=32)))
    return dict(architecture="Zifetar", width=24, vocab=50, norm=dict(eps=1e-5), embedding=dict(scale=2.5, bigram=dict(buckets=19, mul_prev=7, mul_cur=3)), layers=[
        dict(type="parallel", mixer=dict(left=left, right=dict(heads=2, dim=6, vdim=5, tau=4.0), left_scale=0.5, right_scale=1.5), mlp=moe),
        dict(type="channel_delta", mixer=dict(heads=4, kv_heads=2, dim=6, vdim=5, conv=3), mlp=moe),
        dict(type="retention", mixer=dict(heads=2, dim=8, vdim=6, decay=[0.9, 0.99], rot=dict(base=100.0, dims=6)), mlp=None),
        dict(type="parallel", mixer=dict(left=dict(heads=2, dim=4, scale=0.5), right=dict(heads=1, dim=4, tau=1.0)), mlp=None),
    ])


def fields(line):
    return dict(kv.split("=") for kv in line.split()[1:])


def test_config_reader_takes_every_size_and_constant_from_the_config():
    cfg = checkpoint.parse_config(small_config())
    assert cfg["arch"] == "stack" and cfg["design"] == "Zifetar" and cfg["hidden_size"] == 24 and cfg["vocab_size"] == 50 and cfg["num_layers"] == 4
    lines = cfg["spec"].strip().split("\n")
    top = fields(lines[0])
    assert (top["block"], top["norm"], top["pos"], float(top["eps"]), float(top["norm_offset"]), float(top["embed_scale"])) == ("sandwich", "rms", "none", 1e-5, 1.0, 2.5)
    assert (int(top["pair_buckets"]), int(top["pair_mul_prev"]), int(top["pair_mul_cur"]), int(top["embed_norm"])) == (19, 7, 3, 1)
    l0, l1, l2, l3 = (fields(x) for x in lines[1:])
    assert (l0["mixer"], int(l0["heads"]), int(l0["kv_heads"]), int(l0["dim"]), int(l0["vdim"]), float(l0["scale"]), int(l0["chunk"])) == ("parallel", 4, 2, 8, 6, 0.4, 9)
    assert (int(l0["rot_dims"]), float(l0["rot_base"]), float(l0["rs_factor"]), float(l0["rs_low"]), float(l0["rs_high"]), float(l0["rs_original"])) == (4, 300.0, 4.0, 1.0, 3.0, 32.0)
    assert (int(l0["r_heads"]), int(l0["r_dim"]), int(l0["r_vdim"]), float(l0["tau"]), float(l0["left_scale"]), float(l0["right_scale"])) == (2, 6, 5, 4.0, 0.5, 1.5)
    assert (l0["mlp"], int(l0["ff"]), int(l0["experts"]), int(l0["top"]), l0["router"], l0["act"]) == ("moe", 20, 5, 2, "softmax", "silu")
    assert (l1["mixer"], int(l1["heads"]), int(l1["kv_heads"]), int(l1["dim"]), int(l1["vdim"]), int(l1["conv"])) == ("delta", 4, 2, 6, 5, 3)
    assert (l2["mixer"], int(l2["heads"]), l2["decay"], int(l2["rot_dims"]), float(l2["rot_base"]), l2["mlp"]) == ("retention", 2, "0.9,0.99", 6, 100.0, "none")
    # what the config leaves out is off or at its default: no mask, no rotary, no frequency scaling, kv_heads = heads, value size = key size
    assert int(l3["chunk"]) == 0 and int(l3["rot_dims"]) == 0 and "rs_factor" not in l3 and int(l3["kv_heads"]) == 2 and int(l3["vdim"]) == 4 and int(l3["r_vdim"]) == 4
    assert checkpoint.parse_config(small_config(), "float32")["dtype"] == checkpoint.F32


def test_config_reader_rejects_what_the_design_does_not_have():
    bad = small_config()
    bad["layers"][0]["type"] = "attention"
    with pytest.raises(ValueError):
        checkpoint.parse_config(bad)
    bad = small_config()
    bad["layers"][1]["mlp"]["kind"] = "dense"
    with pytest.raises(ValueError):
        checkpoint.parse_config(bad)
    with pytest.raises(ValueError):
        checkpoint.parse_config(small_config(), "float16")


def create(spec, cfg, slots=0):
    L = _lib.load()
    mc = model_config(cfg)
    ec = _lib.EngineConfig(block_size=64, max_num_seqs=4, max_model_len=256, num_gpu_blocks=8, prefill_chunk=8192, device=-1, num_state_slots=slots)
    h = L.vra_engine_create_spec(C.byref(mc), C.byref(ec), spec.encode())
    assert h
    return L, h


def test_native_parser_accepts_the_layer_list():
    cfg = checkpoint.parse_config(small_config())
    L, h = create(cfg["spec"], cfg)
    assert L.vra_engine_finalize_weights(h) == 0, L.vra_engine_last_error(h).decode()
    L.vra_engine_destroy(h)


@pytest.mark.parametrize("edit,why", [
    (lambda s: s.replace("block=sandwich", "block=sequential"), "sandwich blocks"),
    (lambda s: s.replace("decay=0.9,0.99", "decay=0.9"), "one decay per head"),
    (lambda s: s.replace("conv=3", "conv=0"), "conv >= 1"),
    (lambda s: s.replace("tau=4.0", "tau=0.0"), "tau > 0"),
    (lambda s: s.replace("rot_dims=6", "rot_dims=5"), "even rot_dims"),
    (lambda s: s.replace("heads=4 kv_heads=2 dim=6", "heads=3 kv_heads=2 dim=6"), "multiple of kv_heads"),
    (lambda s: s.replace("router=softmax", "router=dice", 1), "router is sigmoid or softmax"),
    (lambda s: s.replace("mixer=retention", "mixer=conv"), "unknown mixer"),
])
def test_native_parser_refuses_inconsistent_lists(edit, why):
    """the refusal surfaces at the first call that needs the model (loading a tensor), with the reason"""
    cfg = checkpoint.parse_config(small_config())
    L, h = create(edit(cfg["spec"]), cfg)
    a = np.zeros((50, 24), np.uint16)
    shape = (C.c_int64 * 2)(50, 24)
    assert L.vra_engine_load_tensor(h, b"embed", a.ctypes.data_as(C.c_void_p), shape, 2, 2) != 0
    assert why in L.vra_engine_last_error(h).decode()
    L.vra_engine_destroy(h)


def test_scheduler_hands_out_state_slots_and_takes_them_back():
    """two state slots, three requests: the scheduler batches two, the third waits although pages are free, and runs when a slot comes back"""
    cfg = checkpoint.parse_config(small_config())
    L, h = create(cfg["spec"], cfg, slots=2)
    assert L.vra_engine_finalize_weights(h) == 0, L.vra_engine_last_error(h).decode()
    rids = []
    for n in (5, 7, 3):
        p = np.arange(1, n + 1, dtype=np.uint32)
        rids.append(L.vra_engine_add_request(h, p.ctypes.data_as(C.c_void_p), n, 2, 1, None, 0))
    seen = []
    for _ in range(20):
        pf, m = C.c_int32(0), _lib.StepMeta()
        n = L.vra_engine_dry_schedule(h, C.byref(pf), C.byref(m))
        assert n >= 0, L.vra_engine_last_error(h).decode()
        if n == 0:
            if not L.vra_engine_has_unfinished(h):
                break
            continue
        seen.append(sorted(int(m.request_ids[i]) for i in range(n)))
        assert n <= 2
        t = np.full(n, 9, np.uint32)
        assert L.vra_engine_dry_commit(h, t.ctypes.data_as(C.c_void_p), n) == n
    assert seen[0] == sorted(rids[:2]) and any(rids[2] in s for s in seen[1:]) and not L.vra_engine_has_unfinished(h)
    assert all(L.vra_engine_request_finished(h, r) for r in rids)
    L.vra_engine_destroy(h)


# ------------------------------------------------------------------------------------------------ the oracle's mechanisms by hand
def test_norm_with_a_weight_around_zero():
    v = np.array([[3.0, 4.0]])
    assert np.allclose(zo.norm1p(v, np.array([0.0, 1.0]), 0.0), [[3.0 / math.sqrt(12.5), 2 * 4.0 / math.sqrt(12.5)]])
    assert np.allclose(zo.rms(np.array([[0.0, 0.0]]), 1e-6), 0.0)


def test_token_pair_rows():
    emb, table = np.arange(12.0).reshape(6, 2), 100.0 + np.arange(16.0).reshape(8, 2)
    x = zo.embed_tokens([4, 5, 4], emb, table, 2.0, 7, 3, 5)
    assert np.allclose(x[0], emb[4] * 2 + table[7])                      # the first token: the table's last row
    assert np.allclose(x[1], emb[5] * 2 + table[(4 * 3 + 5 * 5) % 7])    # previous token 4, token 5
    assert np.allclose(x[2], emb[4] * 2 + table[(5 * 3 + 4 * 5) % 7])


def test_rotary_half_layout_and_scaling():
    f = zo.rotary_freqs(4, 100.0)
    assert np.allclose(f, [1.0, 0.1])
    v = np.array([[[1.0, 2.0, 0.0, 0.0, 7.0]]])  # dimension 0 pairs with 2, 1 with 3; dimension 4 passes
    out = zo.rotate_half(v, [3], f)[0, 0]
    assert np.allclose(out, [math.cos(3.0), 2 * math.cos(0.3), math.sin(3.0), 2 * math.sin(0.3), 7.0])
    sc = dict(factor=8.0, low=1.0, high=4.0, original=64)
    fs, f0 = zo.rotary_freqs(16, 10000.0, sc), zo.rotary_freqs(16, 10000.0)
    wl = 2 * math.pi / f0
    assert np.allclose(fs[wl < 16], f0[wl < 16]) and np.allclose(fs[wl > 64], f0[wl > 64] / 8.0)
    mid = (wl >= 16) & (wl <= 64)
    assert mid.any() and np.all(fs[mid] < f0[mid]) and np.all(fs[mid] > f0[mid] / 8.0)


def test_short_convolution_and_unit_vectors():
    z = np.array([[1.0], [2.0], [3.0]])
    w = np.array([[0.5, -1.0, 2.0]])  # last column: the current token
    pre = np.array([2.0 * 1, -1.0 * 1 + 2.0 * 2, 0.5 * 1 - 1.0 * 2 + 2.0 * 3])
    assert np.allclose(zo.causal_conv_silu(z, w)[:, 0], pre / (1 + np.exp(-pre)))


def test_linear_recurrence_by_hand():
    q = np.array([[[1.0, 0.0]], [[1.0, 1.0]]])
    k = np.array([[[1.0, 0.0]], [[0.0, 1.0]]])
    v = np.array([[[2.0]], [[3.0]]])
    d = np.full((2, 1, 2), 0.5)
    o = zo.linear_recurrence(q, k, v, d)
    assert np.allclose(o[:, 0, 0], [2.0, 0.5 * 2.0 + 3.0])  # the read-out sees the current token's write; the old row decays once
    # delta rule: writing the same key twice with strength 1 and no decay replaces the value
    k2 = np.array([[[1.0, 0.0]], [[1.0, 0.0]]])
    o = zo.linear_recurrence(np.array([[[1.0, 0.0]], [[1.0, 0.0]]]), k2, v, np.ones((2, 1, 2)), beta=np.ones((2, 1)))
    assert np.allclose(o[:, 0, 0], [2.0, 3.0])
    o = zo.linear_recurrence(np.array([[[1.0, 0.0]], [[1.0, 0.0]]]), k2, v, np.ones((2, 1, 2)), beta=np.full((2, 1), 0.5))
    assert np.allclose(o[:, 0, 0], [1.0, 1.0 + 0.5 * (3.0 - 1.0)])


def test_block_mask_and_softmax():
    m = zo.chunk_visible(7, 3)
    assert m[2].tolist() == [True, True, True, False, False, False, False] and m[3].tolist() == [False, False, False, True, False, False, False]
    assert m[5].tolist() == [False, False, False, True, True, True, False] and zo.chunk_visible(3, 0)[2].all()
    q = np.zeros((2, 1, 1))
    out = zo.softmax_attention(q, np.zeros((2, 1, 1)), np.array([[[1.0]], [[3.0]]]), 1.0, zo.chunk_visible(2, 0))
    assert np.allclose(out[:, 0, 0], [1.0, 2.0])


def test_router_softmax_over_the_chosen_logits():
    W = 2
    w = {"router": np.array([[1.0, 0.0], [0.0, 1.0], [0.0, 0.0]]), "router.b": np.array([0.0, 0.0, 0.5])}
    for e, s in enumerate((1.0, 10.0, 100.0)):  # expert e multiplies by s: gate = up = identity-like, down picks the first channel
        w["e%d.gate" % e], w["e%d.up" % e], w["e%d.down" % e] = np.eye(W), np.eye(W) * s, np.eye(W)
    h = np.array([[2.0, 1.0]])  # logits 2, 1, 0.5: experts 0 and 1 are chosen
    out = zo.moe(h, dict(router=dict(experts=3, top=2)), w, "")
    p = math.exp(2.0) / (math.exp(2.0) + math.exp(1.0))
    act = h[0] / (1 + np.exp(-h[0])) * h[0]
    assert np.allclose(out[0], p * act * 1.0 + (1 - p) * act * 10.0)


def test_decay_forms():
    cfg = small_config()
    cfg["layers"] = cfg["layers"][:1]
    w = zo.random_tensors(cfg, 3)
    # sigmoid(z)^(1 / tau) stays in (0, 1) and grows with tau
    z = np.array([-3.0, 0.0, 3.0])
    a4, a9 = np.exp(np.log(zo.sigmoid(z)) / 4.0), np.exp(np.log(zo.sigmoid(z)) / 9.0)
    assert np.all(a4 < a9) and np.all(a9 < 1.0) and np.isclose(a4[1], 0.5 ** 0.25)
    assert zo.forward(cfg, w, [1, 2, 3]).shape == (3, 50)
    assert np.isclose(zo.softplus(np.array([0.0]))[0], math.log(2.0)) and np.isclose(zo.softplus(np.array([50.0]))[0], 50.0)
