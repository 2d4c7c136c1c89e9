"""HuggingFace checkpoint ingestion for the native runtime: `config.json` → model config,
`*.safetensors` (single file or sharded `model.safetensors.index.json`, src/utils/mod.rs:90-111) → tensors under their
HF names, handed to `vra_engine_load_tensor` (which does the TP slicing and the int4 repack on the device).

Mirrors what the reference reads: `Config` (src/utils/config.rs:218-255), `QuantConfig` (:735-757; only 4-bit,
`desc_act = false` is accepted — src/utils/mod.rs:1316-1318), and the tensors of `WNA16::new`
(src/models/layers/wna16.rs:56-152: qweight / qzeros / scales / g_idx / bias; scales and bias are stored f16 and
cast to the model dtype, :97-109).  Pure host code: numpy + a 30-line safetensors reader (mmap, zero copy); no torch.
"""
import json
import mmap
import os
import struct

import numpy as np

BF16, F16, F32 = 0, 1, 2
_ST_DTYPES = {"BF16": (np.uint16, "bf16"), "F16": (np.uint16, "f16"), "F32": (np.float32, "f32"), "I32": (np.int32, "i32"),
              "U32": (np.uint32, "u32"), "I64": (np.int64, "i64"), "U8": (np.uint8, "u8"), "I8": (np.int8, "i8"),
              "U16": (np.uint16, "u16"), "I16": (np.int16, "i16"), "BOOL": (np.uint8, "bool"), "F64": (np.float64, "f64")}
ARCHS = {"LlamaForCausalLM": "llama", "MistralForCausalLM": "llama", "Qwen2ForCausalLM": "qwen2", "Qwen3ForCausalLM": "qwen3"}


def f32_to_bf16_bits(x):
    """round-to-nearest-even, NaN quieted — same rule as the kernels (common.cuh BF16::from_f32)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)


def read_safetensors(path):
    """-> dict name -> (numpy array view into an mmap, kind) with kind in {'bf16','f16','f32','i32',...}; 16-bit floats
    come back as uint16 bit patterns."""
    f = open(path, "rb")
    mm = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ)
    (hlen,) = struct.unpack("<Q", mm[:8])
    header = json.loads(mm[8:8 + hlen].decode("utf-8"))
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        if meta["dtype"] not in _ST_DTYPES:
            raise ValueError(f"{path}: tensor {name} has unsupported dtype {meta['dtype']}")
        npdt, kind = _ST_DTYPES[meta["dtype"]]
        b0, b1 = meta["data_offsets"]
        a = np.frombuffer(mm, dtype=npdt, count=(b1 - b0) // np.dtype(npdt).itemsize, offset=8 + hlen + b0)
        out[name] = (a.reshape(meta["shape"]), kind)
    return out


# Architectures whose config.json lists the layers one by one (key "architecture", a string): name -> parser to the dict of a
# layer-stack model (vllm_rs_amd/host/stack_model.h).  Their tensors keep the checkpoint's own names.
def _num(v):
    return repr(float(v))


def parse_ditilix(cfg_json, dtype=None):
    """Ditilix config.json -> cfg dict with arch "stack": sizes for the engine plus the spec text (one `stack` record, one `layer`
    record per entry of "layers") the native model class parses.  Every size and constant is taken from the config; keys the design
    makes optional (q_temp, softcap, kv_from, mlp, shared) switch their mechanism off when absent or null."""
    td = dtype or cfg_json.get("torch_dtype", "bfloat16")
    dt = {"bfloat16": BF16, "bf16": BF16, "float32": F32, "f32": F32, BF16: BF16, F32: F32}.get(td)
    if dt is None:
        raise ValueError(f"dtype {td!r}: a layer stack runs in bfloat16 or float32")
    norm = cfg_json.get("norm") or {}
    width, vocab, layers = int(cfg_json["width"]), int(cfg_json["vocab"]), cfg_json["layers"]
    lines = ["stack width=%d vocab=%d eps=%s groups=%d residual_mult=%s logit_scale=%s pos_base=%s" % (
        width, vocab, _num(norm.get("eps", 1e-6)), int(norm.get("groups", 1)), _num(cfg_json.get("residual_mult", 1.0)),
        _num(cfg_json.get("logit_scale", 1.0)), _num(10000.0))]
    heads = kv_heads = dim = 1
    for i, layer in enumerate(layers):
        if layer.get("type", "attention") != "attention":
            raise ValueError(f"layer {i}: mixer type {layer.get('type')!r} is not part of this design")
        mx = layer["mixer"]
        f = dict(heads=int(mx["heads"]), kv_heads=int(mx.get("kv_heads", mx["heads"])), dim=int(mx["dim"]), vdim=int(mx.get("vdim", mx["dim"])),
                 scale=_num(mx["scale"]) if mx.get("scale") is not None else _num(int(mx["dim"]) ** -0.5),
                 softcap=_num(mx.get("softcap") or 0.0), kv_from=int(mx["kv_from"]) if mx.get("kv_from") is not None else -1)
        qt = mx.get("q_temp")
        if qt:
            f.update(temp_coef=_num(qt["coef"]), temp_every=int(qt["every"]))
        mlp = layer.get("mlp")
        if not mlp:
            f.update(mlp="none")
        elif mlp["kind"] == "dense":
            f.update(mlp="dense", ff=int(mlp["ff"]))
        elif mlp["kind"] == "moe":
            f.update(mlp="moe", ff=int(mlp["expert"]["ff"]), limit=_num(mlp["expert"].get("limit") or 0.0),
                     experts=int(mlp["router"]["experts"]), top=int(mlp["router"].get("top", 1)))
            if mlp.get("shared"):
                f.update(shared_ff=int(mlp["shared"]["ff"]), shared_limit=_num(mlp["shared"].get("limit") or 0.0))
        else:
            raise ValueError(f"layer {i}: feed-forward kind {mlp['kind']!r} is not part of this design")
        lines.append("layer " + " ".join(f"{k}={v}" for k, v in f.items()))
        heads, kv_heads, dim = max(heads, f["heads"]), max(kv_heads, f["kv_heads"]), max(dim, f["dim"], f["vdim"])
    return dict(arch="stack", design="Ditilix", hidden_size=width, vocab_size=vocab, num_layers=len(layers), num_heads=heads, num_kv_heads=kv_heads,
                head_dim=dim, intermediate_size=0, max_position_embeddings=int(cfg_json.get("max_position_embeddings", 1 << 20)),
                rms_norm_eps=float(norm.get("eps", 1e-6)), rope_theta=10000.0, dtype=dt, quant_method=None, spec="\n".join(lines) + "\n")


def parse_gaperax(cfg_json, dtype=None):
    """Gaperax config.json -> cfg dict with arch "stack": sequential pre-norm blocks with a Dynamic Tanh norm, no position vector at the
    embedding, and per layer a latent attention (low-rank latents, rotary part with optional YaRN scaling, softmax sink) or an attention
    with sigmoid weights (distance penalty, window with kept first tokens, mixed heads, output gate), a gated gelu feed-forward or none,
    optionally the tensors of another layer ("weights_of").  Every size and constant comes from the config."""
    td = dtype or cfg_json.get("torch_dtype", "bfloat16")
    dt = {"bfloat16": BF16, "bf16": BF16, "float32": F32, "f32": F32, BF16: BF16, F32: F32}.get(td)
    if dt is None:
        raise ValueError(f"dtype {td!r}: a layer stack runs in bfloat16 or float32")
    norm = cfg_json.get("norm") or {}
    width, vocab, layers = int(cfg_json["width"]), int(cfg_json["vocab"]), cfg_json["layers"]
    lines = ["stack width=%d vocab=%d eps=%s block=sequential norm=dyt pos=none" % (width, vocab, _num(norm.get("eps", 1e-6)))]
    heads = kv_heads = dim = 1
    for i, layer in enumerate(layers):
        mx, kind = layer["mixer"], layer.get("type")
        f = dict(heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx.get("vdim", mx["dim"])),
                 scale=_num(mx["scale"]) if mx.get("scale") is not None else _num(int(mx["dim"]) ** -0.5))
        if kind == "latent_attention":
            rot = mx.get("rot") or {}
            f.update(mixer="latent", kv_heads=1, rot_dim=int(mx.get("rot_dim", 0)), kv_rank=int(mx["kv_rank"]), q_rank=int(mx["q_rank"]), sink=1,
                     rot_dims=int(rot.get("dims", mx.get("rot_dim", 0))), rot_base=_num(rot.get("base", 10000.0)))
            sc = rot.get("scaling")
            if sc:
                f.update(yarn_factor=_num(sc["factor"]), yarn_original=_num(sc["original"]), yarn_fast=_num(sc.get("fast", 32.0)),
                         yarn_slow=_num(sc.get("slow", 1.0)))
        elif kind == "attention":
            mask = mx.get("mask") or {}
            f.update(mixer="sigmoid", kv_heads=int(mx.get("kv_heads", mx["heads"])), window=int(mask.get("size", 0)),
                     keep_first=int(mask.get("keep_first", 0)), slope_exp=_num(8.0))
        else:
            raise ValueError(f"layer {i}: mixer type {kind!r} is not part of this design")
        if layer.get("weights_of") is not None:
            f.update(weights_of=int(layer["weights_of"]))
        mlp = layer.get("mlp")
        if not mlp:
            f.update(mlp="none")
        elif mlp["kind"] == "dense":
            f.update(mlp="gated", ff=int(mlp["ff"]))
        else:
            raise ValueError(f"layer {i}: feed-forward kind {mlp['kind']!r} is not part of this design")
        lines.append("layer " + " ".join(f"{k}={v}" for k, v in f.items()))
        heads, kv_heads, dim = max(heads, f["heads"]), max(kv_heads, f["kv_heads"]), max(dim, f["dim"], f["vdim"])
    return dict(arch="stack", design="Gaperax", hidden_size=width, vocab_size=vocab, num_layers=len(layers), num_heads=heads, num_kv_heads=kv_heads,
                head_dim=dim, intermediate_size=0, max_position_embeddings=int(cfg_json.get("max_position_embeddings", 1 << 20)),
                rms_norm_eps=float(norm.get("eps", 1e-6)), rope_theta=10000.0, dtype=dt, quant_method=None, spec="\n".join(lines) + "\n")


def parse_zifetar(cfg_json, dtype=None):
    """Zifetar config.json -> cfg dict with arch "stack": sandwich-norm blocks (an RMS norm before and after every sub-block, weights stored
    around zero), an embedding with a hashed token-pair table and a norm of its own, per layer one of three mixers that carry a state per
    sequence (gated delta rule, retention, softmax attention inside blocks of positions beside a gated linear attention) and a mixture of
    experts whose router takes a softmax over the chosen logits.  Every size and constant comes from the config; the ranks of the low-rank
    projections come from the tensors' shapes ("rank_a" / "rank_g" of a mixer only size synthetic weights)."""
    td = dtype or cfg_json.get("torch_dtype", "bfloat16")
    dt = {"bfloat16": BF16, "bf16": BF16, "float32": F32, "f32": F32, BF16: BF16, F32: F32}.get(td)
    if dt is None:
        raise ValueError(f"dtype {td!r}: a layer stack runs in bfloat16 or float32")
    norm = cfg_json.get("norm") or {}
    em = cfg_json.get("embedding") or {}
    bg = em.get("bigram") or {}
    width, vocab, layers = int(cfg_json["width"]), int(cfg_json["vocab"]), cfg_json["layers"]
    head = "stack width=%d vocab=%d eps=%s block=sandwich norm=rms pos=none norm_offset=1.0 embed_scale=%s embed_norm=1" % (
        width, vocab, _num(norm.get("eps", 1e-6)), _num(em.get("scale", 1.0)))
    if bg:
        head += " pair_buckets=%d pair_mul_prev=%d pair_mul_cur=%d" % (int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"]))
    lines = [head]
    heads = kv_heads = dim = 1

    def rot_fields(mx):
        rot = mx.get("rot") or {}
        f = dict(rot_dims=int(rot.get("dims", 0)), rot_base=_num(rot.get("base", 10000.0)))
        sc = rot.get("scaling")
        if sc:
            f.update(rs_factor=_num(sc["factor"]), rs_low=_num(sc["low"]), rs_high=_num(sc["high"]), rs_original=_num(sc["original"]))
        return f

    for i, layer in enumerate(layers):
        mx, kind = layer["mixer"], layer.get("type")
        if kind == "channel_delta":
            f = dict(mixer="delta", heads=int(mx["heads"]), kv_heads=int(mx.get("kv_heads", mx["heads"])), dim=int(mx["dim"]),
                     vdim=int(mx.get("vdim", mx["dim"])), conv=int(mx.get("conv", 1)), rank_a=int(mx.get("rank_a", 32)), rank_g=int(mx.get("rank_g", 32)))
        elif kind == "retention":
            f = dict(mixer="retention", heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx.get("vdim", mx["dim"])),
                     decay=",".join(_num(d) for d in mx["decay"]))
            f.update(rot_fields(mx))
        elif kind == "parallel":
            le, ri = mx["left"], mx["right"]
            f = dict(mixer="parallel", heads=int(le["heads"]), kv_heads=int(le.get("kv_heads", le["heads"])), dim=int(le["dim"]),
                     vdim=int(le.get("vdim", le["dim"])), scale=_num(le["scale"]) if le.get("scale") is not None else _num(int(le["dim"]) ** -0.5),
                     chunk=int((le.get("mask") or {}).get("size", 0)), qk_norm=1, bias=1,
                     r_heads=int(ri["heads"]), r_dim=int(ri["dim"]), r_vdim=int(ri.get("vdim", ri["dim"])), tau=_num(ri["tau"]),
                     rank_a=int(ri.get("rank_a", 32)), left_scale=_num(mx.get("left_scale", 1.0)), right_scale=_num(mx.get("right_scale", 1.0)))
            f.update(rot_fields(le))
        else:
            raise ValueError(f"layer {i}: mixer type {kind!r} is not part of this design")
        mlp = layer.get("mlp")
        if not mlp:
            f.update(mlp="none")
        elif mlp["kind"] == "moe":
            f.update(mlp="moe", ff=int(mlp["expert"]["ff"]), experts=int(mlp["router"]["experts"]), top=int(mlp["router"].get("top", 1)),
                     router="softmax", act="silu")
        else:
            raise ValueError(f"layer {i}: feed-forward kind {mlp['kind']!r} is not part of this design")
        lines.append("layer " + " ".join(f"{k}={v}" for k, v in f.items()))
        heads, kv_heads, dim = max(heads, f["heads"]), max(kv_heads, f.get("kv_heads", f["heads"])), max(dim, f["dim"], f["vdim"])
    return dict(arch="stack", design="Zifetar", hidden_size=width, vocab_size=vocab, num_layers=len(layers), num_heads=heads, num_kv_heads=kv_heads,
                head_dim=dim, intermediate_size=0, max_position_embeddings=int(cfg_json.get("max_position_embeddings", 1 << 20)),
                rms_norm_eps=float(norm.get("eps", 1e-6)), rope_theta=10000.0, dtype=dt, quant_method=None, spec="\n".join(lines) + "\n")


def parse_sudosun(cfg_json, dtype=None):
    """Sudosun config.json -> cfg dict with arch "stack": sandwich blocks whose four norms are Dynamic Tanh, a plain embedding whose table is
    also the head, per layer one of three mixers that carry a state per sequence (a gated delta rule with one decay per head, lightning
    attention with constant decays, softmax attention under a sliding window with a sink beside a real-gated diagonal recurrence) and a
    feed-forward that is dense (clamped gated form) or a mixture of experts (softmax over all router outputs, a correction for the choice,
    expert groups, identity experts).  Every size and constant comes from the config; the taps of the convolutions come from their tensors."""
    td = dtype or cfg_json.get("torch_dtype", "bfloat16")
    dt = {"bfloat16": BF16, "bf16": BF16, "float32": F32, "f32": F32, BF16: BF16, F32: F32}.get(td)
    if dt is None:
        raise ValueError(f"dtype {td!r}: a layer stack runs in bfloat16 or float32")
    norm = cfg_json.get("norm") or {}
    width, vocab, layers = int(cfg_json["width"]), int(cfg_json["vocab"]), cfg_json["layers"]
    lines = ["stack width=%d vocab=%d eps=%s block=sandwich norm=dyt pos=none tie_head=1 logit_scale=%s" % (
        width, vocab, _num(norm.get("eps", 1e-6)), _num(cfg_json.get("logit_scale", 1.0)))]
    heads = kv_heads = dim = 1
    for i, layer in enumerate(layers):
        mx, kind = layer["mixer"], layer.get("type")
        if kind == "delta":
            f = dict(mixer="delta", lowrank=0, heads=int(mx["heads"]), kv_heads=int(mx.get("kv_heads", mx["heads"])), dim=int(mx["dim"]),
                     vdim=int(mx.get("vdim", mx["dim"])), conv=int(mx.get("conv", 1)))
        elif kind == "lightning":
            f = dict(mixer="lightning", heads=int(mx["heads"]), dim=int(mx["dim"]), vdim=int(mx.get("vdim", mx["dim"])),
                     decay=",".join(_num(d) for d in mx["decay"]))
        elif kind == "parallel":
            le, ri = mx["left"], mx["right"]
            rot = le.get("rot") or {}
            f = dict(mixer="parallel", right="rglru", heads=int(le["heads"]), kv_heads=int(le.get("kv_heads", le["heads"])), dim=int(le["dim"]),
                     vdim=int(le.get("vdim", le["dim"])), scale=_num(le["scale"]) if le.get("scale") is not None else _num(int(le["dim"]) ** -0.5),
                     window=int((le.get("mask") or {}).get("size", 0)), qk_norm=1, bias=1, sink=1, head_temp=1, head_gate=1, branch_norm=1,
                     rot_layout="pairs", rot_dims=int(rot.get("dims", 0)), rot_base=_num(rot.get("base", 10000.0)),
                     r_width=int(ri["width"]), r_blocks=int(ri.get("blocks", 1)), r_conv=int(ri.get("conv", 1)), left_scale=_num(0.5), right_scale=_num(0.5))
            sc = rot.get("scaling")
            if sc:
                f.update(yarn_factor=_num(sc["factor"]), yarn_original=_num(sc["original"]), yarn_fast=_num(sc.get("fast", 32.0)),
                         yarn_slow=_num(sc.get("slow", 1.0)))
        else:
            raise ValueError(f"layer {i}: mixer type {kind!r} is not part of this design")
        mlp = layer.get("mlp")
        if not mlp:
            f.update(mlp="none")
        elif mlp["kind"] == "dense":
            f.update(mlp="clamped", ff=int(mlp["ff"]), limit=_num(mlp["limit"]))
        elif mlp["kind"] == "moe":
            r = mlp["router"]
            f.update(mlp="moe", ff=int(mlp["expert"]["ff"]), experts=int(r["experts"]), top=int(r.get("top", 1)), router="softmax_all", act="silu",
                     identity=int(r.get("identity", 0)))
            g = r.get("groups")
            if g:
                f.update(groups=int(g["count"]), keep=int(g["keep"]))
        else:
            raise ValueError(f"layer {i}: feed-forward kind {mlp['kind']!r} is not part of this design")
        lines.append("layer " + " ".join(f"{k}={v}" for k, v in f.items()))
        heads, kv_heads, dim = max(heads, f["heads"]), max(kv_heads, f.get("kv_heads", f["heads"])), max(dim, f["dim"], f["vdim"])
    return dict(arch="stack", design="Sudosun", hidden_size=width, vocab_size=vocab, num_layers=len(layers), num_heads=heads, num_kv_heads=kv_heads,
                head_dim=dim, intermediate_size=0, max_position_embeddings=int(cfg_json.get("max_position_embeddings", 1 << 20)),
                rms_norm_eps=float(norm.get("eps", 1e-6)), rope_theta=10000.0, dtype=dt, quant_method=None, spec="\n".join(lines) + "\n")


STACK_ARCHS = {"Ditilix": parse_ditilix, "Gaperax": parse_gaperax, "Zifetar": parse_zifetar, "Sudosun": parse_sudosun}


def parse_config(cfg_json, dtype=None):
    """HF config.json dict -> the dict `vllm_rs_amd.engine.model_config` consumes; raises on what the reference
    rejects (src/utils/mod.rs:1303-1330).  A config that names one of STACK_ARCHS under "architecture" goes to that design's parser."""
    if cfg_json.get("architecture") in STACK_ARCHS:
        return STACK_ARCHS[cfg_json["architecture"]](cfg_json, dtype)
    archs = cfg_json.get("architectures") or ["LlamaForCausalLM"]
    if archs[0] not in ARCHS:
        raise ValueError(f"architecture {archs[0]} is not on this path (supported: {sorted(ARCHS)})")
    td = dtype or cfg_json.get("torch_dtype", "bfloat16")
    dt = {"bfloat16": BF16, "bf16": BF16, "float16": F16, "half": F16, "f16": F16}.get(td if isinstance(td, str) else "", None)
    if dt is None:
        dt = td if td in (BF16, F16) else BF16
    heads = cfg_json["num_attention_heads"]
    out = dict(arch=ARCHS[archs[0]], hidden_size=cfg_json["hidden_size"], intermediate_size=cfg_json["intermediate_size"],
               num_layers=cfg_json["num_hidden_layers"], num_heads=heads, num_kv_heads=cfg_json.get("num_key_value_heads", heads),
               head_dim=cfg_json.get("head_dim") or cfg_json["hidden_size"] // heads, vocab_size=cfg_json["vocab_size"],
               max_position_embeddings=cfg_json.get("max_position_embeddings", 4096), rms_norm_eps=cfg_json.get("rms_norm_eps", 1e-5),
               rope_theta=float(cfg_json.get("rope_theta", (cfg_json.get("rope_parameters") or {}).get("rope_theta", 10000.0))),
               rope_scaling=cfg_json.get("rope_scaling"), tie_word_embeddings=bool(cfg_json.get("tie_word_embeddings", False)),
               attention_bias=bool(cfg_json.get("attention_bias", ARCHS[archs[0]] == "qwen2")), dtype=dt, quant_method=None)
    # Sliding-window attention (Mistral-7B-v0.1: 4096; llama.rs:46,284 passes config.sliding_window into attention and mask): wired into
    # the engine's forward since round 6 (vra_model_config.sliding_window).  A window that covers every position is full causal attention.
    sw = cfg_json.get("sliding_window")
    if sw and cfg_json.get("use_sliding_window", True) and int(sw) < int(out["max_position_embeddings"]):
        out["sliding_window"] = int(sw)
    q = cfg_json.get("quantization_config")
    if q:
        method = q.get("quant_method", "").lower()
        if method not in ("gptq", "awq"):
            raise ValueError(f"quant_method {method!r} is not on this path (gptq, awq)")
        if q.get("bits", 4) != 4:
            raise ValueError("only 4-bit GPTQ/AWQ checkpoints are supported (wna16.rs:154-160)")
        if q.get("desc_act", False):
            raise ValueError("desc_act=true checkpoints are rejected, as in the reference (src/utils/mod.rs:1316-1318)")
        if method == "gptq" and q.get("sym", True) is False:
            raise ValueError("asymmetric GPTQ goes through gemm_half_q_half_alt in the reference (f16 only); not wired into the engine")
        out.update(quant_method=method, group_size=q.get("group_size", 128))
    return out


def iter_tensors(model_dir):
    """yields (hf_name, array, kind) over every tensor of the checkpoint (sharded or not)."""
    idx = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.exists(idx):
        files = sorted(set(json.load(open(idx))["weight_map"].values()))
    else:
        files = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors files in {model_dir}")
    for fn in files:
        for name, (a, kind) in read_safetensors(os.path.join(model_dir, fn)).items():
            yield name, a, kind


def to_engine_tensor(name, a, kind, model_dtype):
    """checkpoint tensor -> what vra_engine_load_tensor expects: packed int tensors as they are, every float tensor
    as 16-bit patterns of the MODEL dtype (scales/bias are f16 on disk even for bf16 models: wna16.rs:97-109)."""
    if kind in ("i32", "u32"):
        return np.ascontiguousarray(a).view(np.uint32)
    if model_dtype == F32:  # 32-bit models (layer stacks): every float tensor widened exactly
        if kind == "f32":
            return np.ascontiguousarray(a, np.float32)
        if kind == "bf16":
            return np.ascontiguousarray((a.astype(np.uint32) << 16).view(np.float32))
        if kind == "f16":
            return a.view(np.float16).astype(np.float32)
        raise ValueError(f"{name}: cannot convert {kind} to float32")
    want = "bf16" if model_dtype == BF16 else "f16"
    if kind == want:
        return np.ascontiguousarray(a)
    if kind == "f16":
        f = a.view(np.float16).astype(np.float32)
    elif kind == "bf16":
        f = (a.astype(np.uint32) << 16).view(np.float32)
    elif kind == "f32":
        f = np.asarray(a, np.float32)
    else:
        raise ValueError(f"{name}: cannot convert {kind} to the model dtype")
    return f32_to_bf16_bits(f) if model_dtype == BF16 else f.astype(np.float16).view(np.uint16)


def load_pretrained(model_dir, dtype=None):
    """-> (cfg dict, generator of (name, engine-ready array)); rotary inv_freq buffers and unused tensors are skipped
    by the engine itself (unknown names are ignored there only if they end in `rotary_emb.inv_freq`)."""
    cfg = parse_config(json.load(open(os.path.join(model_dir, "config.json"))), dtype)

    def gen():
        for name, a, kind in iter_tensors(model_dir):
            if name.endswith("rotary_emb.inv_freq"):
                continue
            if name.endswith(".g_idx"):
                g = cfg.get("group_size", 128)
                K = a.shape[0]
                gg = g if g and g > 0 else K
                if not np.array_equal(np.asarray(a, np.int64), np.arange(K) // gg):
                    raise ValueError(f"{name}: non-trivial g_idx (act-order) is not supported (SURVEY Appendix A7)")
                continue
            yield name, to_engine_tensor(name, a, kind, cfg["dtype"])
    return cfg, gen()
