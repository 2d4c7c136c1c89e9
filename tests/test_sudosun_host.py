"""CPU tests of the Sudosun design in the layer-stack model class: the reader of its config.json (every size and constant, optional
mechanisms), the native parser of the layer list it writes and the scheduler's state slots (host-only engine: no GPU touched), and the
float64 oracle's mechanisms checked by hand (tests/sudosun_oracle.py)."""
import ctypes as C
import math

import numpy as np
import pytest

from tests import sudosun_oracle as so
from vllm_rs_amd import _lib, checkpoint
from vllm_rs_amd.engine import model_config


def small_config():
    moe = dict(kind="moe", expert=dict(ff=20), router=dict(experts=7, top=3, identity=2, groups=dict(count=3, keep=2)))
    left = dict(heads=4, kv_heads=2, dim=8, vdim=6, scale=0.4, mask=dict(size=9),
                rot=dict(base=300.0, dims=4, scaling=dict(factor=3.0, original=32, fast=8.0, slow=2.0)))
    return dict(architecture="Sudosun", width=24, vocab=50, norm=dict(eps=1e-5), logit_scale=1.5, layers=[
        dict(type="parallel", mixer=dict(left=left, right=dict(width=18, blocks=3, conv=2)), mlp=moe),
        dict(type="delta", mixer=dict(heads=4, kv_heads=2, dim=6, vdim=5, conv=3), mlp=dict(kind="dense", ff=28, limit=0.75)),
        dict(type="lightning", mixer=dict(heads=2, dim=8, vdim=6, decay=[0.9, 0.99]), mlp=None),
        dict(type="parallel", mixer=dict(left=dict(heads=2, dim=4, scale=0.5), right=dict(width=8, blocks=1)),
             mlp=dict(kind="moe", expert=dict(ff=8), router=dict(experts=3, top=1))),
    ])


def fields(line):
    return dict(kv.split("=") for kv in line.split()[1:])


def test_config_reader_takes_every_size_and_constant_from_the_config():
    cfg = checkpoint.parse_config(small_config())
    assert cfg["arch"] == "stack" and cfg["design"] == "Sudosun" and cfg["hidden_size"] == 24 and cfg["vocab_size"] == 50 and cfg["num_layers"] == 4
    lines = cfg["spec"].strip().split("\n")
    top = fields(lines[0])
    assert (top["block"], top["norm"], top["pos"], float(top["eps"]), int(top["tie_head"]), float(top["logit_scale"])) == ("sandwich", "dyt", "none", 1e-5, 1, 1.5)
    l0, l1, l2, l3 = (fields(x) for x in lines[1:])
    assert (l0["mixer"], l0["right"], int(l0["heads"]), int(l0["kv_heads"]), int(l0["dim"]), int(l0["vdim"]), float(l0["scale"]), int(l0["window"])) == ("parallel", "rglru", 4, 2, 8, 6, 0.4, 9)
    assert (l0["rot_layout"], int(l0["rot_dims"]), float(l0["rot_base"]), float(l0["yarn_factor"]), float(l0["yarn_original"]), float(l0["yarn_fast"]), float(l0["yarn_slow"])) == ("pairs", 4, 300.0, 3.0, 32.0, 8.0, 2.0)
    assert (int(l0["r_width"]), int(l0["r_blocks"]), int(l0["r_conv"]), float(l0["left_scale"]), float(l0["right_scale"])) == (18, 3, 2, 0.5, 0.5)
    assert (int(l0["sink"]), int(l0["head_temp"]), int(l0["head_gate"]), int(l0["branch_norm"]), int(l0["qk_norm"]), int(l0["bias"])) == (1, 1, 1, 1, 1, 1)
    assert (l0["mlp"], int(l0["ff"]), int(l0["experts"]), int(l0["top"]), l0["router"], l0["act"], int(l0["identity"]), int(l0["groups"]), int(l0["keep"])) == ("moe", 20, 7, 3, "softmax_all", "silu", 2, 3, 2)
    assert (l1["mixer"], int(l1["lowrank"]), int(l1["heads"]), int(l1["kv_heads"]), int(l1["dim"]), int(l1["vdim"]), int(l1["conv"])) == ("delta", 0, 4, 2, 6, 5, 3)
    assert (l1["mlp"], int(l1["ff"]), float(l1["limit"])) == ("clamped", 28, 0.75)
    assert (l2["mixer"], int(l2["heads"]), l2["decay"], int(l2["dim"]), int(l2["vdim"]), l2["mlp"]) == ("lightning", 2, "0.9,0.99", 8, 6, "none")
    # what the config leaves out is off or at its default: no window, no rotary, no frequency scaling, kv_heads = heads, value size = key size,
    # one tap, no groups, no identity experts
    assert int(l3["window"]) == 0 and int(l3["rot_dims"]) == 0 and "yarn_factor" not in l3 and int(l3["kv_heads"]) == 2 and int(l3["vdim"]) == 4
    assert int(l3["r_conv"]) == 1 and int(l3["identity"]) == 0 and "groups" not in l3
    assert checkpoint.parse_config(small_config(), "float32")["dtype"] == checkpoint.F32


def test_config_reader_rejects_what_the_design_does_not_have():
    bad = small_config()
    bad["layers"][0]["type"] = "attention"
    with pytest.raises(ValueError):
        checkpoint.parse_config(bad)
    bad = small_config()
    bad["layers"][1]["mlp"]["kind"] = "gated"
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
    (lambda s: s.replace("r_width=18 r_blocks=3", "r_width=18 r_blocks=4"), "equal blocks"),
    (lambda s: s.replace("rot_dims=4", "rot_dims=3"), "even rot_dims"),
    (lambda s: s.replace("right=rglru", "right=lstm", 1), "right is gla or rglru"),
    (lambda s: s.replace("rot_layout=pairs", "rot_layout=thirds", 1), "rot_layout half or pairs"),
    (lambda s: s.replace("groups=3 keep=2", "groups=4 keep=2"), "groups must divide"),
    (lambda s: s.replace("groups=3 keep=2", "groups=3 keep=4"), "keep <= groups"),
    (lambda s: s.replace("router=softmax_all", "router=dice", 1), "router is sigmoid or softmax or softmax_all"),
    (lambda s: s.replace("mlp=clamped ff=28", "mlp=clamped ff=0"), "without ff"),
    (lambda s: s.replace("mixer=lightning", "mixer=thunder"), "unknown mixer"),
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
    L.vra_engine_destroy(h)


# ------------------------------------------------------------------------------------------------ the oracle's mechanisms by hand
def test_dynamic_tanh_has_no_statistics():
    w = {"n": np.array([2.0, 3.0]), "n.b": np.array([0.5, -0.5]), "n.alpha": np.array(0.25)}
    x = np.array([[4.0, -8.0], [400.0, 0.0]])
    out = so.dyt(x, w, "n")
    assert np.allclose(out[0], [2 * math.tanh(1.0) + 0.5, 3 * math.tanh(-2.0) - 0.5])
    assert np.allclose(out[1], [2.5, -0.5])  # a huge neighbour does not move the other entry


def test_rotary_neighbouring_pairs_and_yarn():
    cos, sin = so.rotary_table(dict(base=100.0, dims=4), [3])
    assert np.allclose(cos[0], [math.cos(3.0), math.cos(0.3)]) and np.allclose(sin[0], [math.sin(3.0), math.sin(0.3)])
    v = np.array([[[1.0, 0.0, 0.0, 2.0, 7.0]]])  # (0, 1) and (2, 3) are pairs; dimension 4 passes
    out = so.rotate_pairs(v, cos, sin)[0, 0]
    assert np.allclose(out, [math.cos(3.0), math.sin(3.0), -2 * math.sin(0.3), 2 * math.cos(0.3), 7.0])
    rot = dict(base=10000.0, dims=16, scaling=dict(factor=8.0, original=64, fast=4.0, slow=1.0))
    c1, s1 = so.rotary_table(rot, [1])
    ang = np.arctan2(s1[0], c1[0])
    f0 = 10000.0 ** (-2.0 * np.arange(8) / 16)
    turns = 64 * f0 / (2 * math.pi)
    assert np.allclose(ang[turns > 4.5], f0[turns > 4.5]) and np.allclose(ang[turns < 0.5], f0[turns < 0.5] / 8.0)
    assert np.allclose(np.hypot(c1[0], s1[0]), 0.1 * math.log(8.0) + 1.0)


def test_short_convolution_counts_from_zeros():
    z = np.array([[1.0], [2.0], [3.0]])
    w = np.array([[0.5, -1.0, 2.0]])  # last column: the current token
    assert np.allclose(so.causal_conv(z, w, np.array([10.0]))[:, 0], [10 + 2.0, 10 - 1.0 + 4.0, 10 + 0.5 - 2.0 + 6.0])


def test_recurrences_by_hand():
    q = np.array([[[1.0, 0.0]], [[1.0, 1.0]]])
    k = np.array([[[1.0, 0.0]], [[0.0, 1.0]]])
    v = np.array([[[2.0]], [[3.0]]])
    o = so.constant_decay_recurrence(q, k, v, [0.5])
    assert np.allclose(o[:, 0, 0], [2.0, 0.5 * 2.0 + 3.0])  # the read-out sees the current token's write; the old row decays once
    same = np.array([[[1.0, 0.0]], [[1.0, 0.0]]])
    o = so.delta_rule_recurrence(same, same, v, np.ones((2, 1)), np.ones((2, 1)))
    assert np.allclose(o[:, 0, 0], [2.0, 3.0])  # strength 1, no decay: the second write replaces the value
    o = so.delta_rule_recurrence(same, same, v, np.full((2, 1), 0.5), np.array([[1.0], [0.5]]))
    assert np.allclose(o[:, 0, 0], [1.0, 0.5 + 0.5 * (3.0 - 0.5)])  # decay first, then the write against what is left
    # the gated diagonal recurrence starts from zero also for the first token: its input arrives scaled by sqrt(1 - a^2)
    lam = np.array([0.0])
    a = math.exp(-8.0 * 0.5 * math.log(2.0))
    out = so.gated_diagonal_recurrence(np.array([[2.0], [0.0]]), np.array([[0.5], [0.5]]), np.array([[1.0], [1.0]]), lam)
    assert np.allclose(out[:, 0], [math.sqrt(1 - a * a) * 2.0, a * math.sqrt(1 - a * a) * 2.0])


def test_window_and_sink():
    vis = so.window_visible(range(6), 3)
    assert vis[4].tolist() == [False, False, True, True, True, False] and vis[1].tolist() == [True, True, False, False, False, False]
    assert so.window_visible(range(3), 0)[2].all()
    q, k = np.zeros((2, 1, 1)), np.zeros((2, 1, 1))
    v = np.array([[[1.0]], [[3.0]]])
    out = so.softmax_window_sink(q, k, v, np.array([1.0]), np.array([math.log(2.0)]), so.window_visible(range(2), 0))
    assert np.allclose(out[:, 0, 0], [1.0 / 3.0, 4.0 / 4.0])  # the sink weighs 2 beside keys of weight 1 and carries no value
    out = so.softmax_window_sink(q, k, v, np.array([1.0]), np.array([-1e9]), so.window_visible(range(2), 1))
    assert np.allclose(out[:, 0, 0], [1.0, 3.0])  # a window of one: the query's own position


def test_router_groups_correction_and_identity_experts():
    W = 2
    w = {"router": np.zeros((6, W)), "correction": np.zeros(6)}
    w["router"][:, 0] = [3.0, 0.0, 2.5, 0.0, 1.0, 2.0]
    r = dict(experts=4, identity=2, top=2, groups=dict(count=3, keep=2))
    h = np.array([[1.0, 0.0]])
    chosen, wt = so.route(h, r, w, "")
    s = np.exp(w["router"][:, 0]) / np.exp(w["router"][:, 0]).sum()
    assert chosen[0].tolist() == [0, 2] and np.allclose(wt[0], s[[0, 2]])  # groups {0,1} and {2,3} are best; weights are not renormalised
    w["correction"] = np.array([0.0, 0.0, -1.0, -1.0, 0.0, 0.0])  # the correction moves the choice, not the weights; group {2,3} drops out
    chosen, wt = so.route(h, r, w, "")
    assert chosen[0].tolist() == [0, 5] and np.allclose(wt[0], s[[0, 5]])
    for e in range(4):
        w["e%d.gate" % e], w["e%d.up" % e], w["e%d.down" % e] = np.eye(W), np.eye(W), np.eye(W) * 10.0 ** e
    out = so.ff_moe(h, dict(router=r), w, "")
    act = so.silu(h[0]) * h[0]
    assert np.allclose(out[0], s[0] * act + s[5] * h[0])  # expert 5 is an identity expert: its weight times the input itself


def test_clamped_dense_feed_forward():
    w = {"gate": np.array([[1.0], [1.0]]), "up": np.array([[1.0], [-1.0]]), "down": np.array([[1.0, 10.0]])}
    out = so.ff_dense(np.array([[5.0]]), dict(limit=2.0), w, "")
    g = 2.0 / (1 + math.exp(-1.702 * 2.0))
    assert np.allclose(out[0], [g * 3.0 + 10.0 * g * (-2.0 + 1.0)])


def test_whole_model_shapes():
    cfg = small_config()
    w = so.random_tensors(cfg, 3)
    lg, layers = so.forward(cfg, w, [1, 2, 3, 4, 5], True)
    assert lg.shape == (5, 50) and layers.shape == (4, 5, 24)
    assert so.forward(cfg, w, [1, 2, 3])[:3].shape == (3, 50) and np.allclose(so.forward(cfg, w, [1, 2, 3]), lg[:3])  # causal
