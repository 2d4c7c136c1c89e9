"""Throughput of a layer-stack model (Ditilix, Gaperax, Zifetar or Sudosun design) beside the dense bf16 Llama of the same widths —
`python bench.py --design ditilix|gaperax|zifetar|sudosun` (Sudosun also beside the Zifetar design of the same widths, its closest model;
Zifetar also beside the Ditilix mixture of experts of the same widths, the closest
model of its class).

Random weights of layer sizes that resemble a real model; for each size one JSON line with prefill tokens/s (one prompt of
`prefill_tokens`, best of three engine steps) and decode tokens/s (batches of 1 and 8 behind 512-token prompts, HIP-event time of
`steps` engine steps), for both models, with the model FLOPs per token and the weight bytes a decode step streams, so that both can be
priced against the same roofline (2.5 PFLOP/s dense bf16, 8 TB/s).
"""
import json
import time

import numpy as np


def stack_config(width, heads, kv_heads, dim, ff, layers, vocab, experts=0, top=2, expert_ff=0, shared_ff=0, share_kv=False):
    """config.json dict of a Ditilix model: layer 0 dense, the others mixtures of experts when `experts` > 0; with share_kv the second
    half of the layers reads the keys / values of the last layer of the first half"""
    mx = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, softcap=50.0, q_temp=dict(coef=0.1, every=1024))
    ls = []
    for i in range(layers):
        m = dict(mx)
        if share_kv and i >= (layers + 1) // 2:
            m["kv_from"] = (layers + 1) // 2 - 1
        if experts and i > 0:
            mlp = dict(kind="moe", expert=dict(ff=expert_ff, limit=7.0), router=dict(experts=experts, top=top))
            if shared_ff:
                mlp["shared"] = dict(ff=shared_ff, limit=7.0)
        else:
            mlp = dict(kind="dense", ff=ff)
        ls.append(dict(type="attention", mixer=m, mlp=mlp))
    return dict(architecture="Ditilix", width=width, vocab=vocab, residual_mult=0.5, logit_scale=1.0, norm=dict(eps=1e-6, groups=4), layers=ls)


def stack_costs(cj):
    """(matrix FLOPs per token without attention, weight bytes a one-token step reads) of a Ditilix config"""
    W, flops, wbytes = cj["width"], 0, 0
    for layer in cj["layers"]:
        mx, ml = layer["mixer"], layer["mlp"]
        n = mx["heads"] * mx["dim"] + (0 if mx.get("kv_from") is not None else mx["kv_heads"] * (mx["dim"] + mx["vdim"]))
        p = W * n + mx["heads"] * mx["vdim"] * W
        if ml["kind"] == "dense":
            act = p + 2 * W * ml["ff"]
        else:
            act = p + ml["router"]["top"] * 3 * W * ml["expert"]["ff"] + (3 * W * ml["shared"]["ff"] if ml.get("shared") else 0) + W * ml["router"]["experts"]
        flops += 2 * act
        wbytes += 2 * act
    head = cj["vocab"] * W
    return flops + 2 * head, wbytes + 2 * head


def gaperax_config(width, heads, kv_heads, dim, ff, layers, vocab, kv_rank, q_rank, rot_dim, window, keep_first):
    """config.json dict of a Gaperax model: every fourth layer (from the first) a latent attention, the others windowed sigmoid attention"""
    lat = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=dim, kv_rank=kv_rank, q_rank=q_rank, scale=(dim + rot_dim) ** -0.5,
               rot=dict(base=5e5, dims=rot_dim, scaling=dict(factor=8.0, original=8192, fast=32.0, slow=1.0)))
    sig = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, mask=dict(size=window, keep_first=keep_first))
    ls = [dict(type="latent_attention" if i % 4 == 0 else "attention", mixer=lat if i % 4 == 0 else sig, mlp=dict(kind="dense", ff=ff)) for i in range(layers)]
    return dict(architecture="Gaperax", width=width, vocab=vocab, norm=dict(eps=1e-6), layers=ls)


def gaperax_costs(cj):
    """(matrix FLOPs per token without attention, weight bytes a one-token step reads) of a Gaperax config"""
    W, n = cj["width"], 0
    for layer in cj["layers"]:
        mx = layer["mixer"]
        H, dim, vdim = mx["heads"], mx["dim"], mx["vdim"]
        if layer["type"] == "latent_attention":
            rd, kr, qr = mx["rot_dim"], mx["kv_rank"], mx["q_rank"]
            n += W * (qr + kr + rd) + qr * H * (dim + rd) + H * dim * kr + H * kr * vdim + H * vdim * W
        else:
            G = mx.get("kv_heads", H)
            n += W * (H * dim + G * dim + G * vdim + H * vdim) + H * vdim * W
        if layer.get("mlp"):
            n += 3 * W * layer["mlp"]["ff"]
    n += cj["vocab"] * W
    return 2 * n, 2 * n


def zifetar_config(width, heads, kv_heads, dim, layers, vocab, experts, top, expert_ff, chunk, rank):
    """config.json dict of a Zifetar model: layers in the order parallel, delta rule, retention, ...; every layer a mixture of experts"""
    rot = dict(base=2e5, dims=dim, scaling=dict(factor=4.0, low=1.0, high=8.0, original=4096))
    par = dict(left=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, mask=dict(size=chunk), rot=rot),
               right=dict(heads=heads // 2, dim=dim, vdim=dim, tau=8.0, rank_a=rank), left_scale=0.5, right_scale=1.0)
    dl = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, conv=4, rank_a=rank, rank_g=rank)
    ret = dict(heads=heads, dim=dim, vdim=dim, decay=[1.0 - 2.0 ** (-5.0 - 5.0 * h / max(heads - 1, 1)) for h in range(heads)], rot=dict(base=1e5, dims=dim))
    mlp = dict(kind="moe", expert=dict(ff=expert_ff), router=dict(experts=experts, top=top))
    kinds = [("parallel", par), ("channel_delta", dl), ("retention", ret)]
    ls = [dict(type=kinds[i % 3][0], mixer=kinds[i % 3][1], mlp=mlp) for i in range(layers)]
    return dict(architecture="Zifetar", width=width, vocab=vocab, norm=dict(eps=1e-6), embedding=dict(scale=width ** 0.5, bigram=dict(buckets=65521, mul_prev=257, mul_cur=3)),
                layers=ls)


def zifetar_costs(cj):
    """(matrix FLOPs per token without attention and recurrences, weight bytes a one-token step reads) of a Zifetar config"""
    W, n = cj["width"], 0
    for layer in cj["layers"]:
        mx = layer["mixer"]
        if layer["type"] == "parallel":
            le, ri = mx["left"], mx["right"]
            H, G, D, V = le["heads"], le["kv_heads"], le["dim"], le["vdim"]
            rh, rd, rv, ra = ri["heads"], ri["dim"], ri["vdim"], ri["rank_a"]
            n += W * (H * D + G * D + G * V + rh * (2 * rd + 2 * rv) + ra) + ra * rh * rd + (H * V + rh * rv) * W
        elif layer["type"] == "channel_delta":
            H, G, D, V, ra, rg = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"], mx["rank_a"], mx["rank_g"]
            n += W * (2 * G * D + H * V + H + ra + rg) + ra * H * D + rg * H * V + H * V * W
        else:
            H, D, V = mx["heads"], mx["dim"], mx["vdim"]
            n += W * (2 * H * D + 2 * H * V) + H * V * W
        if layer.get("mlp"):
            n += layer["mlp"]["router"]["top"] * 3 * W * layer["mlp"]["expert"]["ff"] + W * layer["mlp"]["router"]["experts"]
    n += cj["vocab"] * W
    return 2 * n, 2 * n


def sudosun_config(width, heads, kv_heads, dim, layers, vocab, experts, top, expert_ff, window, blocks):
    """config.json dict of a Sudosun model: layers in the order parallel, delta rule, lightning, ...; every layer a mixture of experts (four
    identity experts beside the real ones, four groups of which two may be chosen from)"""
    rot = dict(base=1e6, dims=dim // 2, scaling=dict(factor=8.0, original=4096, fast=16.0, slow=2.0))
    par = dict(left=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, mask=dict(size=window), rot=rot),
               right=dict(width=width, blocks=blocks, conv=4))
    dl = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, conv=4)
    li = dict(heads=heads, dim=dim, vdim=dim, decay=[1.0 - 2.0 ** (-5.0 - 5.0 * h / max(heads - 1, 1)) for h in range(heads)])
    mlp = dict(kind="moe", expert=dict(ff=expert_ff), router=dict(experts=experts, top=top, identity=4, groups=dict(count=4, keep=2)))
    kinds = [("parallel", par), ("delta", dl), ("lightning", li)]
    ls = [dict(type=kinds[i % 3][0], mixer=kinds[i % 3][1], mlp=mlp) for i in range(layers)]
    return dict(architecture="Sudosun", width=width, vocab=vocab, norm=dict(eps=1e-6), logit_scale=1.0, layers=ls)


def sudosun_costs(cj):
    """(matrix FLOPs per token without attention and recurrences, weight bytes a one-token step reads) of a Sudosun config"""
    W, n = cj["width"], 0
    for layer in cj["layers"]:
        mx = layer["mixer"]
        if layer["type"] == "parallel":
            le, ri = mx["left"], mx["right"]
            H, G, D, V, Wr = le["heads"], le["kv_heads"], le["dim"], le["vdim"], ri["width"]
            n += W * (H * D + G * D + G * V + H + 2 * Wr) + 2 * Wr * (Wr // ri["blocks"]) + (H * V + Wr) * W
        elif layer["type"] == "delta":
            H, G, D, V = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            n += W * (2 * G * D + 2 * H * V + 2 * H) + H * V * W
        else:
            H, D, V = mx["heads"], mx["dim"], mx["vdim"]
            n += W * (2 * H * D + 2 * H * V) + H * V * W
        mlp = layer.get("mlp")
        if mlp and mlp["kind"] == "moe":
            n += mlp["router"]["top"] * 3 * W * mlp["expert"]["ff"] + W * (mlp["router"]["experts"] + mlp["router"].get("identity", 0))
        elif mlp:
            n += 3 * W * mlp["ff"]
    n += cj["vocab"] * W
    return 2 * n, 2 * n


def llama_costs(cfg):
    H, D = cfg["hidden_size"], cfg["head_dim"]
    per = H * (cfg["num_heads"] + 2 * cfg["num_kv_heads"]) * D + cfg["num_heads"] * D * H + 3 * H * cfg["intermediate_size"]
    n = per * cfg["num_layers"] + cfg["vocab_size"] * H
    return 2 * n, 2 * n


def measure(eng, L, vocab, prefill_tokens, steps, warmup):
    def sync():
        L.vra_device_sync()
    r = np.random.default_rng(0)
    best = 1e9
    for _ in range(3):
        eng.add_request(r.integers(1, vocab - 1, prefill_tokens).astype(np.uint32), max_tokens=1, ignore_eos=True)
        sync()
        t0 = time.perf_counter()
        eng.step()
        sync()
        best = min(best, time.perf_counter() - t0)
        while eng.has_unfinished():
            eng.step()
    out = dict(prefill_tokens_per_s=prefill_tokens / best, prefill_ms=best * 1e3)
    for bs in (1, 8):
        for _ in range(bs):
            eng.add_request(r.integers(1, vocab - 1, 512).astype(np.uint32), max_tokens=warmup + steps + 8, ignore_eos=True)
        while True:
            n, is_prefill = eng.step()
            if not is_prefill and n == bs:
                break
        for _ in range(warmup):
            eng.step()
        sync()
        ms = eng.timed_decode(steps)
        sync()
        out[f"decode_bs{bs}_tokens_per_s"] = bs * steps / (ms / 1e3)
        out[f"decode_bs{bs}_ms_per_step"] = ms / steps
        while eng.has_unfinished():
            eng.step()
    return out


SIZES = {
    # name: (width, heads, kv_heads, head size, dense ff, layers, vocab, experts, top, expert ff, shared ff, share_kv)
    "dense-2048": (2048, 16, 4, 128, 8192, 4, 32000, 0, 0, 0, 0, False),
    "moe-2048": (2048, 16, 4, 128, 8192, 4, 32000, 16, 2, 1024, 2048, True),
    "dense-4096": (4096, 32, 8, 128, 14336, 2, 32000, 0, 0, 0, 0, False),
}


GAPERAX_SIZES = {
    # name: (width, heads, kv_heads, head size, ff, layers, vocab, kv latent, q latent, rotated part, window, kept first tokens)
    "gaperax-2048": (2048, 16, 4, 128, 8192, 4, 32000, 192, 768, 64, 1024, 16),
    "gaperax-4096": (4096, 32, 8, 128, 14336, 2, 32000, 192, 1536, 64, 1024, 16),
}


ZIFETAR_SIZES = {
    # name: (width, heads, kv_heads, head size, layers, vocab, experts, top, expert ff, block mask, rank of the low-rank projections)
    "zifetar-2048": (2048, 16, 4, 128, 3, 32000, 16, 2, 1024, 1024, 64),
    "zifetar-4096": (4096, 32, 8, 128, 3, 32000, 16, 2, 2048, 1024, 128),
}


SUDOSUN_SIZES = {
    # name: (width, heads, kv_heads, head size, layers, vocab, experts, top, expert ff, window, gate blocks of the recurrence)
    "sudosun-2048": (2048, 16, 4, 128, 3, 32000, 16, 2, 1024, 1024, 16),
    "sudosun-4096": (4096, 32, 8, 128, 3, 32000, 16, 2, 2048, 1024, 32),
}


def main(steps=64, warmup=8, prefill_tokens=2048, graph=True, sizes=None, design="ditilix"):
    from . import _lib, checkpoint
    from .engine import BF16, Engine
    L = _lib.load()
    lines = []
    table = GAPERAX_SIZES if design == "gaperax" else (ZIFETAR_SIZES if design == "zifetar" else (SUDOSUN_SIZES if design == "sudosun" else SIZES))
    for name in (sizes or table):
        if design == "sudosun":
            width, heads, kvh, dim, layers, vocab, experts, top, eff, window, blocks = table[name]
            cj = sudosun_config(width, heads, kvh, dim, layers, vocab, experts, top, eff, window, blocks)
            ff = 4 * width
        elif design == "zifetar":
            width, heads, kvh, dim, layers, vocab, experts, top, eff, chunk, rank = table[name]
            cj = zifetar_config(width, heads, kvh, dim, layers, vocab, experts, top, eff, chunk, rank)
            ff = 4 * width
        elif design == "gaperax":
            width, heads, kvh, dim, ff, layers, vocab, kr, qr, rd, window, keep_first = table[name]
            cj = gaperax_config(width, heads, kvh, dim, ff, layers, vocab, kr, qr, rd, window, keep_first)
        else:
            width, heads, kvh, dim, ff, layers, vocab, experts, top, eff, sff, share = table[name]
            cj = stack_config(width, heads, kvh, dim, ff, layers, vocab, experts, top, eff, sff, share)
        eng = Engine(checkpoint.parse_config(cj), num_gpu_blocks=512, max_num_seqs=8, max_model_len=4096, use_graph=graph).init_synthetic()
        res = dict(stack=measure(eng, L, vocab, prefill_tokens, steps, warmup))
        eng.close()
        res["stack"]["flops_per_token"], res["stack"]["weight_bytes_per_step"] = (
            sudosun_costs(cj) if design == "sudosun" else (zifetar_costs(cj) if design == "zifetar" else (gaperax_costs(cj) if design == "gaperax" else stack_costs(cj))))
        if design == "sudosun":  # the closest model of the same class: the Zifetar design of the same widths (state mixers, the same experts)
            zj = zifetar_config(width, heads, kvh, dim, layers, vocab, experts, top, eff, window, width // 32)
            eng = Engine(checkpoint.parse_config(zj), num_gpu_blocks=512, max_num_seqs=8, max_model_len=4096, use_graph=graph).init_synthetic()
            res["zifetar"] = measure(eng, L, vocab, prefill_tokens, steps, warmup)
            eng.close()
            res["zifetar"]["flops_per_token"], res["zifetar"]["weight_bytes_per_step"] = zifetar_costs(zj)
        if design == "zifetar":  # the closest model of the same class: softmax attention + the same mixture of experts in every layer
            dj = stack_config(width, heads, kvh, dim, ff, layers + 1, vocab, experts, top, eff, 0, False)
            dj["layers"] = dj["layers"][1:]
            eng = Engine(checkpoint.parse_config(dj), num_gpu_blocks=512, max_num_seqs=8, max_model_len=4096, use_graph=graph).init_synthetic()
            res["ditilix_moe"] = measure(eng, L, vocab, prefill_tokens, steps, warmup)
            eng.close()
            res["ditilix_moe"]["flops_per_token"], res["ditilix_moe"]["weight_bytes_per_step"] = stack_costs(dj)
        lcfg = dict(arch="llama", hidden_size=width, intermediate_size=ff, num_layers=layers, num_heads=heads, num_kv_heads=kvh, head_dim=dim,
                    vocab_size=vocab, max_position_embeddings=4096, rms_norm_eps=1e-5, rope_theta=10000.0, quant_method=None, dtype=BF16)
        eng = Engine(lcfg, num_gpu_blocks=512, max_num_seqs=8, max_model_len=4096, use_graph=graph).init_synthetic()
        res["llama_dense"] = measure(eng, L, vocab, prefill_tokens, steps, warmup)
        eng.close()
        res["llama_dense"]["flops_per_token"], res["llama_dense"]["weight_bytes_per_step"] = llama_costs(lcfg)
        for m in res.values():
            m["prefill_matrix_tflops"] = m["prefill_tokens_per_s"] * m["flops_per_token"] / 1e12
            m["decode_bs1_weight_gb_per_s"] = m["weight_bytes_per_step"] / (m["decode_bs1_ms_per_step"] / 1e3) / 1e9
        line = dict(metric="stack_vs_dense_llama", size=name, design={"gaperax": "Gaperax", "zifetar": "Zifetar", "sudosun": "Sudosun"}.get(design, "Ditilix"), dtype="bf16", data="synthetic", prefill_tokens=prefill_tokens,
                    decode_context=512, steps=steps, **res)
        print(json.dumps(line), flush=True)
        lines.append(line)
    return lines
