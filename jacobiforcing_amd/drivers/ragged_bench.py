#!/usr/bin/env python3
"""Prefill and decode throughput of a ragged model family (Lokizen, Vumalix, Bamanex, Mikipel) at sizes that resemble a real model's
layers, beside the package's closest existing model at equal width, depth, head sizes and active feed-forward width (Lokizen beside
Qwen2; Vumalix, Bamanex and Mikipel beside Lokizen and Qwen2) — random weights, synthetic tokens.

    python -m jacobiforcing_amd.drivers.ragged_bench [--design lokizen|vumalix|bamanex|mikipel] [--sizes small,medium] [--kernels]
    python bench.py --design lokizen            (the same, as one JSON line)

Per size: prefill = whole prompts in one step (tokens / s), decode = one token for each of ``--decode-batch`` requests at a
context of ``--context`` tokens (tokens / s).  ``--kernels`` adds each layer kernel alone at the size's shapes with its
algorithmic bytes and flops and the fraction of the chip's roofline (8 TB/s, 2.5 PFLOP/s bf16 matrix / 157 TFLOP/s float
vector) that its time amounts to, next to the like kernel of the Qwen2 forward (scaled-dot-product attention, the SwiGLU
launch, F.rms_norm)."""
from __future__ import annotations

import argparse
import json
import time

import torch
import torch.nn.functional as F

HBM_BPS, MATRIX_FLOPS, VECTOR_FLOPS = 8.0e12, 2.5e15, 157e12

SIZES = {
    # width, layers (alternating retention / attention), heads, kv_heads, dim, experts, top, ff, window, vocab
    "small": dict(width=1024, layers=4, heads=8, kv=2, dim=128, experts=16, top=4, ff=512, window=1024, vocab=32000),
    "medium": dict(width=2048, layers=8, heads=16, kv=4, dim=128, experts=32, top=4, ff=1024, window=2048, vocab=32000),
}


def lokizen_config(s):
    from ..modeling.lokizen import LokizenConfig
    H, D = s["heads"], s["dim"]
    moe = {"kind": "moe", "expert": {"ff": s["ff"]}, "router": {"experts": s["experts"], "top": s["top"], "scale": 1.0}}
    ret = {"type": "retention", "mlp": moe, "mixer": {"heads": H, "dim": D, "vdim": D, "rot": {"dims": D, "base": 1e6},
                                                       "decay": [1 - 2.0 ** (-5 - 3 * h / H) for h in range(H)]}}
    att = {"type": "attention", "mlp": moe, "mixer": {"heads": H, "kv_heads": s["kv"], "dim": D, "vdim": D, "scale": D ** -0.5, "bias_max": 4096,
                                                       "mask": {"size": s["window"], "keep_first": 4}}}
    return LokizenConfig.from_dict({"architecture": "Lokizen", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-5},
                                    "embedding": {"scale": 1.0}, "layers": [ret if i % 2 == 0 else att for i in range(s["layers"])]})


def qwen2_config(s):
    from ..modeling.qwen2 import Qwen2Config
    return Qwen2Config(vocab_size=s["vocab"], hidden_size=s["width"], intermediate_size=s["top"] * s["ff"], num_hidden_layers=s["layers"],
                       num_attention_heads=s["heads"], num_key_value_heads=s["kv"], head_dim=s["dim"], max_position_embeddings=1 << 16,
                       eos_token_id=s["vocab"] - 1, pad_token_id=s["vocab"] - 2)


def timed(fn, warmup=2, iters=5):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / iters


# Vumalix at the same widths, depths and head counts: latent attention and differential attention alternate; the differential
# maps have half of Lokizen's head size each, the latent has the rank of a head; the dense feed-forward has the experts' active width
VSIZES = {
    "small": dict(width=1024, layers=4, heads=8, kv=2, dim=64, vdim=128, lheads=8, ldim=64, rot=32, lvdim=64, kv_rank=128, q_rank=384,
                  window=1024, ff=2048, taps=4, vocab=32000),
    "medium": dict(width=2048, layers=8, heads=16, kv=4, dim=64, vdim=128, lheads=16, ldim=128, rot=64, lvdim=128, kv_rank=512, q_rank=768,
                   window=2048, ff=4096, taps=4, vocab=32000),
}


def vumalix_config(s):
    from ..modeling.vumalix import VumalixConfig
    mlp = {"kind": "dense", "ff": s["ff"]}
    lat = {"type": "latent_attention", "mlp": mlp,
           "mixer": {"heads": s["lheads"], "dim": s["ldim"], "rot_dim": s["rot"], "vdim": s["lvdim"], "kv_rank": s["kv_rank"], "q_rank": s["q_rank"],
                     "scale": (s["ldim"] + s["rot"]) ** -0.5, "mask": {"size": s["window"]}, "rot": {"dims": s["rot"], "base": 1e6}}}
    att = {"type": "attention", "mlp": mlp, "mixer": {"heads": s["heads"], "kv_heads": s["kv"], "dim": s["dim"], "vdim": s["vdim"], "scale": s["dim"] ** -0.5,
                                                       "diff": 0.3, "q_temp": {"coef": 0.1, "every": 256}}}
    return VumalixConfig.from_dict({"architecture": "Vumalix", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-6}, "canon": {"taps": s["taps"]},
                                    "layers": [lat if i % 2 == 0 else att for i in range(s["layers"])]})


def bench_lokizen(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    from ..modeling.lokizen import random_model
    model = random_model(lokizen_config(s), "cuda", dtype, max_positions=max(prompt_len, context) + 64)
    return bench_ragged(model, s["vocab"], prompts, prompt_len, decode_batch, context)


def bench_vumalix(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    from ..modeling.vumalix import random_model
    model = random_model(vumalix_config(s), "cuda", dtype, max_positions=max(prompt_len, context) + 64)
    return bench_ragged(model, s["vocab"], prompts, prompt_len, decode_batch, context)


def bench_ragged(model, vocab, prompts, prompt_len, decode_batch, context):
    from .. import layer_ops as LO
    dev = "cuda"
    s = {"vocab": vocab}
    page = 64
    per = -(-(max(prompt_len, context) + 1) // page)
    slots = max(prompts, decode_batch)
    cache = model.new_cache(slots * per, page, slots)
    tables = [list(range(b * per, (b + 1) * per)) for b in range(slots)]
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, s["vocab"], (prompts * prompt_len,), generator=g).to(dev)
    pre = LO.RaggedBatch.build([prompt_len] * prompts, [0] * prompts, list(range(prompts)), tables[:prompts], page, dev)
    last = torch.arange(prompts, device=dev) * prompt_len + prompt_len - 1
    t_pre = timed(lambda: model.forward(ids, pre, cache, last))
    # decode at `context`: the pool holds whatever the prompts left (random weights: the timing does not depend on the values)
    dec = LO.RaggedBatch.build([1] * decode_batch, [context] * decode_batch, list(range(decode_batch)), tables[:decode_batch], page, dev)
    dids = ids[:decode_batch].contiguous()
    t_dec = timed(lambda: model.forward(dids, dec, cache, None), warmup=3, iters=20)
    return {"prefill_tokens_per_s": prompts * prompt_len / t_pre, "prefill_ms": 1e3 * t_pre, "decode_tokens_per_s": decode_batch / t_dec,
            "decode_ms": 1e3 * t_dec}


def bench_qwen2(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    from ..modeling.qwen2 import Qwen2Model, Qwen2Weights, StaticKVCache
    dev = torch.device("cuda")
    cfg = qwen2_config(s)
    model = Qwen2Model(cfg, Qwen2Weights(cfg, dev, dtype=dtype))
    g = torch.Generator().manual_seed(0)

    def run(R, T, start, last_only):
        cache = StaticKVCache(cfg, R, start + T + 8, 0, 1, dev, dtype=dtype)          # row r of the batch is cache row r: attended in place
        ids = torch.randint(0, s["vocab"], (R, T), generator=g).to(dev)
        st = torch.full((R,), start, dtype=torch.int32, device=dev)
        pos = st.view(R, 1) + torch.arange(T, dtype=torch.int32, device=dev).view(1, T)
        rp = torch.arange(R, dtype=torch.int32, device=dev)
        idx = (torch.arange(R, dtype=torch.int32, device=dev) * T + T - 1) if last_only else None
        return lambda: model.forward(ids, pos, cache, row_prompt=rp, row_cand=rp * 0 - 1, row_len=st * 0 + T, kv_len_rows=st, any_candidates=False,
                                     s_cur=start + T, logit_index=idx, rows_in_place=True)

    t_pre = timed(run(prompts, prompt_len, 0, True))
    t_dec = timed(run(decode_batch, 1, context, False), warmup=3, iters=20)
    return {"prefill_tokens_per_s": prompts * prompt_len / t_pre, "prefill_ms": 1e3 * t_pre, "decode_tokens_per_s": decode_batch / t_dec,
            "decode_ms": 1e3 * t_dec}


def kernel_table(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    """Each layer kernel alone, prefill shape and decode shape: microseconds, algorithmic bytes / flops, fraction of the roofline
    (the larger of bytes / 8 TB/s and flops / peak, over the time)."""
    from .. import layer_ops as LO
    from .. import ops
    dev = "cuda"
    H, G, D, W, E, top, ff, win = s["heads"], s["kv"], s["dim"], s["width"], s["experts"], s["top"], s["ff"], s["window"]
    page, es = 64, 2
    per = -(-(max(prompt_len, context) + 1) // page)
    slots = max(prompts, decode_batch)
    tables = [list(range(b * per, (b + 1) * per)) for b in range(slots)]
    g = torch.Generator().manual_seed(0)
    rnd = lambda *sh: torch.randn(*sh, generator=g).to(dev).to(dtype)
    kc, vc = rnd(slots * per * page, G * D), rnd(slots * per * page, G * D)
    state = torch.zeros((slots, H, D, D), device=dev)
    decay = torch.full((H,), 0.99, device=dev)
    a = torch.arange(max(prompt_len, context) + 8, dtype=torch.float32, device=dev).view(-1, 1) * torch.rand(D // 2, device=dev).view(1, -1)
    cos, sin = a.cos().contiguous(), a.sin().contiguous()
    rel, talk = torch.randn(16, H, device=dev), torch.eye(H, device=dev)
    from ..modeling.lokizen import distance_bucket_table
    lut = torch.from_numpy(distance_bucket_table(16, 4096, max(prompt_len, context) + 8)).to(dev)
    rel, lut = rel[lut.long()].contiguous(), None                       # the bias laid out by distance, as the model passes it
    w_up, w_down = rnd(E, ff, W) * 0.02, rnd(E, W, ff) * 0.02
    out = {}

    def row(name, secs, nbytes, flops, peak):
        bound = max(nbytes / HBM_BPS, flops / peak)
        out[name] = {"us": round(1e6 * secs, 1), "MB": round(nbytes / 1e6, 2), "GFLOP": round(flops / 1e9, 2), "roofline_fraction": round(bound / secs, 4)}

    for phase, B, T, start in (("prefill", prompts, prompt_len, 0), ("decode", decode_batch, 1, context)):
        n = B * T
        batch = LO.RaggedBatch.build([T] * B, [start] * B, list(range(B)), tables[:B], page, dev)
        x, y, wn = torch.randn(n, W, device=dev), rnd(n, W), rnd(W)
        row(f"{phase}.add_rmsnorm", timed(lambda: LO.add_rmsnorm(x, y, None, wn, 1e-5, dtype)), n * W * (4 + 4 + es + es), 4.0 * n * W, VECTOR_FLOPS)
        q, gate = rnd(n, H * D), rnd(n, H * D)
        keys = sum(min(start + t + 1, win + 4) for t in range(T)) * B                       # visible (query, key) pairs per head
        kv_bytes = B * min(start + T, win + T) * 2 * G * D * es                              # every needed key / value row once
        t_att = timed(lambda: LO.attn_window(q, gate, kc, vc, batch, H, G, D, D, D ** -0.5, win, 4, rel, lut, talk))
        row(f"{phase}.attn_window", t_att, kv_bytes + 3 * n * H * D * es, 4.0 * keys * H * D, MATRIX_FLOPS)
        proj = rnd(n, 4 * H * D)
        t_ret = timed(lambda: LO.retention(proj, (0, H * D, 2 * H * D, 3 * H * D), batch, H, D, D, D, cos, sin, decay, 1e-5, state))
        row(f"{phase}.retention", t_ret, n * 5 * H * D * es + 2 * B * H * D * D * 4, 4.0 * n * H * D * D, VECTOR_FLOPS)
        h, z = rnd(n, W), torch.randn(n, E, device=dev)
        t_moe = timed(lambda: LO.moe_experts(h, z, None, top, 1.0, w_up, w_down))
        used = min(E, n * top)
        row(f"{phase}.moe_experts", t_moe, used * 2 * ff * W * es + n * W * es + n * top * W * 4, 4.0 * n * top * ff * W, MATRIX_FLOPS)
        # the like kernels of the Qwen2 forward at the same shapes
        S = start + T
        qh = rnd(B, G, (H // G) * T, D)
        Kf, Vf = rnd(B, G, S, D), rnd(B, G, S, D)
        bias = torch.zeros((B, 1, (H // G) * T, (S + 15) // 16 * 16), dtype=dtype, device=dev)[..., :S]
        t_sdpa = timed(lambda: F.scaled_dot_product_attention(qh, Kf, Vf, attn_mask=bias))
        pairs = B * sum(start + t + 1 for t in range(T))
        row(f"{phase}.qwen2.sdpa", t_sdpa, 2 * B * S * G * D * es + 2 * n * H * D * es, 4.0 * pairs * H * D, MATRIX_FLOPS)
        gu = rnd(n, 2 * top * ff)
        row(f"{phase}.qwen2.swiglu", timed(lambda: ops.swiglu(gu)), 3 * n * top * ff * es, 4.0 * n * top * ff, VECTOR_FLOPS)
        xb = rnd(n, W)
        row(f"{phase}.qwen2.rms_norm", timed(lambda: F.rms_norm(xb, (W,), wn, 1e-5)), 2 * n * W * es, 4.0 * n * W, VECTOR_FLOPS)
        wgu, wd = rnd(2 * top * ff, W), rnd(W, top * ff)
        t_mlp = timed(lambda: F.linear(ops.swiglu(F.linear(xb, wgu)), wd))
        row(f"{phase}.qwen2.mlp_gemms", t_mlp, 3 * top * ff * W * es + 2 * n * W * es, 6.0 * n * top * ff * W, MATRIX_FLOPS)
    return out


def kernel_table_vumalix(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    """Vumalix's layer kernels alone at the size's shapes, prefill and decode, each beside the like kernel of the closest model
    (Lokizen's windowed attention, its residual + norm launch, its whole-projection q/k norm; Qwen2's SwiGLU launch)."""
    from .. import layer_ops as LO
    from .. import ops
    dev = "cuda"
    W, H, G, D, Dv, ff, win, taps = s["width"], s["heads"], s["kv"], s["dim"], s["vdim"], s["ff"], s["window"], s["taps"]
    LH, LD, rd, LDv, R, Rq = s["lheads"], s["ldim"], s["rot"], s["lvdim"], s["kv_rank"], s["q_rank"]
    lk = SIZES_BY_WIDTH[W]
    KH, KG, KD = lk["heads"], lk["kv"], lk["dim"]
    page, es = 64, 2
    per = -(-(max(prompt_len, context) + 1) // page)
    slots = max(prompts, decode_batch)
    tables = [list(range(b * per, (b + 1) * per)) for b in range(slots)]
    g = torch.Generator().manual_seed(0)
    rnd = lambda *sh: torch.randn(*sh, generator=g).to(dev).to(dtype)
    tokens = slots * per * page
    kd, vd, lat = rnd(tokens, 2 * G * D), rnd(tokens, G * Dv), rnd(tokens, R + rd)
    kk, vk = rnd(tokens, KG * KD), rnd(tokens, KG * KD)
    a = torch.arange(max(prompt_len, context) + 8, dtype=torch.float32, device=dev).view(-1, 1) * torch.rand(rd // 2, device=dev).view(1, -1)
    cos, sin = a.cos().contiguous(), a.sin().contiguous()
    tail = torch.zeros((slots, taps - 1, W), device=dev)
    out = {}

    def row(name, secs, nbytes, flops, peak):
        bound = max(nbytes / HBM_BPS, flops / peak)
        out[name] = {"us": round(1e6 * secs, 1), "MB": round(nbytes / 1e6, 2), "GFLOP": round(flops / 1e9, 2), "roofline_fraction": round(bound / secs, 4)}

    for phase, B, T, start in (("prefill", prompts, prompt_len, 0), ("decode", decode_batch, 1, context)):
        n = B * T
        batch = LO.RaggedBatch.build([T] * B, [start] * B, list(range(B)), tables[:B], page, dev)
        causal = B * sum(start + t + 1 for t in range(T))                                       # visible (query, key) pairs per head, no window
        windowed = B * sum(min(start + t + 1, win) for t in range(T))
        span_c, span_w = B * (start + T), B * min(start + T, win + T)                              # pool rows a launch has to read once
        x, y, gw, wn = torch.randn(n, W, device=dev), rnd(n, W), torch.ones(1, device=dev), rnd(W)
        row(f"{phase}.norm_add", timed(lambda: LO.norm_add(x, y, gw, 1e-6, dtype)), n * W * (4 + 4 + es + es), 4.0 * n * W, VECTOR_FLOPS)
        row(f"{phase}.lokizen.add_rmsnorm", timed(lambda: LO.add_rmsnorm(x, y, None, wn, 1e-5, dtype)), n * W * (4 + 4 + es + es), 4.0 * n * W, VECTOR_FLOPS)
        cw = rnd(W, taps)
        row(f"{phase}.causal_conv", timed(lambda: LO.causal_conv(x, cw, batch, tail)), n * W * (4 + es), 2.0 * taps * n * W, VECTOR_FLOPS)
        z, coef = rnd(n, ff), torch.tensor([0.5, 0.3, 0.2, 0.1], device=dev)
        row(f"{phase}.polynorm", timed(lambda: LO.polynorm(z, coef, 1e-6)), 3 * n * ff * es, 12.0 * n * ff, VECTOR_FLOPS)
        gu = rnd(n, 2 * ff)
        row(f"{phase}.qwen2.swiglu", timed(lambda: ops.swiglu(gu)), 3 * n * ff * es, 4.0 * n * ff, VECTOR_FLOPS)
        # differential attention: norm + append, both maps' attention, combination
        proj = rnd(n, 2 * H * D + 2 * G * D + G * Dv)
        wq = rnd(D)
        sweep = LO.attn_sweep_tile_rows(dtype, 2 * H, 2 * G, D, Dv, kd, vd, G) > 0
        apart = 2 * H > LO.ATTN_MAX_HEADS_ONE_LAUNCH and not sweep
        t_hn = timed(lambda: LO.head_norm_append(proj, (0, 2 * H * D, 2 * H * D + 2 * G * D), H, G, 2, D, Dv, wq, wq, 1e-6, 0.1, 256, batch, kd, vd, apart))
        row(f"{phase}.head_norm_append", t_hn, 2 * n * (2 * H * D + 2 * G * D + G * Dv) * es, 6.0 * n * (2 * H + 2 * G) * D, VECTOR_FLOPS)
        pk = rnd(n, KH * KD + 2 * KG * KD)
        wqk, wkk = rnd(KH * KD), rnd(KG * KD)
        t_qk = timed(lambda: LO.qk_norm_append(pk, (0, KH * KD, KH * KD + KG * KD), KH, KG, KD, KD, wqk, wkk, 1e-5, kk, vk, batch.kv_slot))
        row(f"{phase}.lokizen.qk_norm_append", t_qk, 2 * n * (KH * KD + 2 * KG * KD) * es, 6.0 * n * (KH + KG) * KD, VECTOR_FLOPS)
        q = LO.head_norm_append(proj, (0, 2 * H * D, 2 * H * D + 2 * G * D), H, G, 2, D, Dv, wq, wq, 1e-6, 0.1, 256, batch, kd, vd, apart)

        def diff_attn():
            if sweep:
                return LO.attn_sweep(q, kd, vd, batch, 2 * H, 2 * G, D, Dv, D ** -0.5, 0, value_heads=G, float_out=True)
            if not apart:
                return LO.attn_window(q, None, kd, vd, batch, 2 * H, 2 * G, D, Dv, D ** -0.5, 0, 0, None, None, None, value_heads=G, float_out=True)
            return [LO.attn_window(q[mp], None, kd[:, mp * G * D:(mp + 1) * G * D], vd, batch, H, G, D, Dv, D ** -0.5, 0, 0, None, None, None, float_out=True)
                    for mp in range(2)]
        row(f"{phase}.attn_differential", timed(diff_attn), span_c * (2 * G * D + G * Dv) * es + n * 2 * H * (D * es + Dv * 4),
            2.0 * causal * 2 * H * (D + Dv), MATRIX_FLOPS)
        a12 = torch.randn(n, 2 * H * Dv, device=dev)
        row(f"{phase}.diff_combine", timed(lambda: LO.diff_combine(a12[:, :H * Dv], a12[:, H * Dv:], H, Dv, 0.4, 1e-6, 0.7, dtype)),
            n * H * Dv * (8 + es), 6.0 * n * H * Dv, VECTOR_FLOPS)
        # latent attention: norms + rotation + append, query packing, attention over the latent pool, gate
        pl = rnd(n, Rq + R + rd + LH * LDv)
        wlq, wlk = rnd(Rq), rnd(R)
        t_lp = timed(lambda: LO.latent_prep(pl, 0, Rq, Rq, R, rd, rd, wlq, wlk, 1e-6, batch, cos, sin, lat))
        row(f"{phase}.latent_prep", t_lp, 2 * n * (Rq + R + rd) * es, 6.0 * n * (Rq + R + rd), VECTOR_FLOPS)
        qa, ql = rnd(LH, n, R), rnd(n, LH * (LD + rd))
        row(f"{phase}.latent_q_pack", timed(lambda: LO.latent_q_pack(qa, ql, LH, LD, R, rd, rd, batch, cos, sin)), 2 * n * LH * (R + rd) * es,
            6.0 * n * LH * rd, VECTOR_FLOPS)
        qf = LO.latent_q_pack(qa, ql, LH, LD, R, rd, rd, batch, cos, sin)
        step = LO.ATTN_MAX_VALUE_WIDTH

        def latent_attn():
            if LO.attn_sweep_tile_rows(dtype, LH, 1, R + rd, R, lat, lat[:, :R]):
                return LO.attn_sweep(qf, lat, lat[:, :R], batch, LH, 1, R + rd, R, 0.1, win)
            return [LO.attn_window(qf, None, lat, lat[:, c0:min(R, c0 + step)], batch, LH, 1, R + rd, min(R, c0 + step) - c0, 0.1, win, 0, None, None, None)
                    for c0 in range(0, R, step)]
        row(f"{phase}.attn_latent", timed(latent_attn), span_w * (R + rd) * es + n * LH * (2 * R + rd) * es, 2.0 * windowed * LH * (2 * R + rd), MATRIX_FLOPS)
        ov = rnd(LH, n, LDv)
        row(f"{phase}.heads_gate", timed(lambda: LO.heads_gate(ov, pl[:, Rq + R + rd:])), 3 * n * LH * LDv * es, 6.0 * n * LH * LDv, VECTOR_FLOPS)
        # the like kernel of the closest model: Lokizen's windowed attention with its bias, head mixing and gate, at its own sizes
        ql2, gate = rnd(n, KH * KD), rnd(n, KH * KD)
        rel, talk = torch.randn(max(prompt_len, context) + 8, KH, device=dev), torch.eye(KH, device=dev)
        t_att = timed(lambda: LO.attn_window(ql2, gate, kk, vk, batch, KH, KG, KD, KD, KD ** -0.5, win, 4, rel, None, talk))
        row(f"{phase}.lokizen.attn_window", t_att, span_w * 2 * KG * KD * es + 3 * n * KH * KD * es, 4.0 * windowed * KH * KD, MATRIX_FLOPS)
    return out


SIZES_BY_WIDTH = {v["width"]: v for v in SIZES.values()}


# Bamanex at Lokizen's widths, depths, head counts and windows: every layer is attention; dense feed-forwards (of the experts' active
# width) and expert feed-forwards (Lokizen's expert count, choice size and width, plus a shared expert) alternate
def bamanex_config(s):
    from ..modeling.bamanex import BamanexConfig
    H, D = s["heads"], s["dim"]
    mixer = {"heads": H, "kv_heads": s["kv"], "dim": D, "vdim": D, "scale": D ** -0.5, "mask": {"size": s["window"]},
             "rot": {"dims": D // 2, "base": 1e6, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
    moe = {"kind": "moe", "expert": {"ff": s["ff"], "limit": 7.0}, "router": {"experts": s["experts"], "top": s["top"]}, "shared": {"ff": s["ff"], "limit": 7.0}}
    dense = {"kind": "dense", "ff": s["top"] * s["ff"]}
    return BamanexConfig.from_dict({"architecture": "Bamanex", "vocab": s["vocab"], "width": s["width"], "norm": {"eps": 1e-6}, "logit_scale": 1.0,
                                    "layers": [{"type": "attention", "mixer": mixer, "mlp": dense if i % 2 == 0 else moe} for i in range(s["layers"])]})


def bench_bamanex(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    from ..modeling.bamanex import random_model
    model = random_model(bamanex_config(s), "cuda", dtype, max_positions=max(prompt_len, context) + 64)
    return bench_ragged(model, s["vocab"], prompts, prompt_len, decode_batch, context)


def kernel_table_bamanex(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    """Bamanex's layer kernels alone at the size's shapes, prefill and decode, each beside the like kernel of the closest model
    (Lokizen's residual + norm launch, its whole-projection q/k norm, its windowed attention, its routed experts; Qwen2's SwiGLU
    launch)."""
    from .. import layer_ops as LO
    from .. import ops
    dev = "cuda"
    H, G, D, W, E, top, ff, win = s["heads"], s["kv"], s["dim"], s["width"], s["experts"], s["top"], s["ff"], s["window"]
    page, es = 64, 2
    per = -(-(max(prompt_len, context) + 1) // page)
    slots = max(prompts, decode_batch)
    tables = [list(range(b * per, (b + 1) * per)) for b in range(slots)]
    g = torch.Generator().manual_seed(0)
    rnd = lambda *sh: torch.randn(*sh, generator=g).to(dev).to(dtype)
    kc, vc = rnd(slots * per * page, G * D), rnd(slots * per * page, G * D)
    rd = D // 2
    a = torch.arange(max(prompt_len, context) + 8, dtype=torch.float32, device=dev).view(-1, 1) * torch.rand(rd // 2, device=dev).view(1, -1)
    cos, sin = a.cos().contiguous(), a.sin().contiguous()
    sink = torch.randn(H, device=dev)
    w_gu, w_up, w_down = rnd(E, 2 * ff, W) * 0.02, rnd(E, ff, W) * 0.02, rnd(E, W, ff) * 0.02
    out = {}

    def row(name, secs, nbytes, flops, peak):
        bound = max(nbytes / HBM_BPS, flops / peak)
        out[name] = {"us": round(1e6 * secs, 1), "MB": round(nbytes / 1e6, 2), "GFLOP": round(flops / 1e9, 2), "roofline_fraction": round(bound / secs, 4)}

    for phase, B, T, start in (("prefill", prompts, prompt_len, 0), ("decode", decode_batch, 1, context)):
        n = B * T
        batch = LO.RaggedBatch.build([T] * B, [start] * B, list(range(B)), tables[:B], page, dev)
        windowed = B * sum(min(start + t + 1, win) for t in range(T))                              # visible (query, key) pairs per head
        span_w = B * min(start + T, win + T)                                                       # pool rows a launch has to read once
        # residual sum of two scaled sublayer outputs + both norms  |  Lokizen: one addend, one norm
        x, y1, y2, wn = torch.randn(n, W, device=dev), rnd(n, W), rnd(n, W), rnd(W)
        ls, w1 = torch.rand(W, device=dev), torch.randn(W, device=dev) * 0.1
        row(f"{phase}.scaled_add_norms", timed(lambda: LO.scaled_add_norms(x, [(y1, ls), (y2, ls)], w1, w1, 1.0, 1e-6, dtype, two=True)),
            n * W * (4 + 4 + 4 * es), 8.0 * n * W, VECTOR_FLOPS)
        row(f"{phase}.lokizen.add_rmsnorm", timed(lambda: LO.add_rmsnorm(x, y1, None, wn, 1e-5, dtype)), n * W * (4 + 4 + es + es), 4.0 * n * W, VECTOR_FLOPS)
        # rotation + per-head unit norm + append  |  Lokizen: whole-projection norm + append
        proj = rnd(n, H * D + 2 * G * D + H)
        cols = (0, H * D, H * D + G * D)
        t_hn = timed(lambda: LO.head_norm_append(proj, cols, H, G, 1, D, D, None, None, 1e-6, 0.0, 1, batch, kc, vc, rot_dims=rd, cos=cos, sin=sin))
        row(f"{phase}.head_norm_append(rot)", t_hn, 2 * n * (H * D + 2 * G * D) * es, 10.0 * n * (H + G) * D, VECTOR_FLOPS)
        pk = rnd(n, H * D + 2 * G * D)
        wqk, wkk = rnd(H * D), rnd(G * D)
        t_qk = timed(lambda: LO.qk_norm_append(pk, cols, H, G, D, D, wqk, wkk, 1e-5, kc, vc, batch.kv_slot))
        row(f"{phase}.lokizen.qk_norm_append", t_qk, 2 * n * (H * D + 2 * G * D) * es, 6.0 * n * (H + G) * D, VECTOR_FLOPS)
        # attention with sink and head gate  |  Lokizen: window keeping first tokens, distance bias, mixed heads, element gate
        q = LO.head_norm_append(proj, cols, H, G, 1, D, D, None, None, 1e-6, 0.0, 1, batch, kc, vc, rot_dims=rd, cos=cos, sin=sin)
        hg = proj[:, H * D + 2 * G * D:]
        sweep = LO.attn_sweep_tile_rows(dtype, H, G, D, D, kc, vc) > 0

        def sink_attn():
            if sweep:
                return LO.attn_sweep(q, kc, vc, batch, H, G, D, D, D ** -0.5, win, sink=sink, gate=hg, gate_per_head=True)
            return LO.attn_window(q, hg, kc, vc, batch, H, G, D, D, D ** -0.5, win, 0, None, None, None, sink=sink, gate_per_head=True)
        row(f"{phase}.attn_sink_gate", timed(sink_attn), span_w * 2 * G * D * es + 2 * n * H * D * es, 4.0 * windowed * H * D, MATRIX_FLOPS)
        gate = rnd(n, H * D)
        rel, talk = torch.randn(max(prompt_len, context) + 8, H, device=dev), torch.eye(H, device=dev)
        t_att = timed(lambda: LO.attn_window(q, gate, kc, vc, batch, H, G, D, D, D ** -0.5, win, 4, rel, None, talk))
        row(f"{phase}.lokizen.attn_window", t_att, span_w * 2 * G * D * es + 3 * n * H * D * es, 4.0 * windowed * H * D, MATRIX_FLOPS)
        # gated activations  |  Qwen2's SwiGLU launch
        gu = rnd(n, 2 * top * ff)
        row(f"{phase}.gated_act(gelu)", timed(lambda: LO.gated_act(gu, 0, top * ff, top * ff, LO.ACT_GELU_TANH)), 3 * n * top * ff * es, 12.0 * n * top * ff, VECTOR_FLOPS)
        gs = rnd(n, 2 * ff + 8)                                # gate, linear branch, the token gate, zero columns up to a 16-byte border
        row(f"{phase}.gated_act(clamped, row gate)", timed(lambda: LO.gated_act(gs, 0, ff, ff, LO.ACT_CLAMPED_SWISH, 7.0, 1.702, 1.0, row_gate=gs[:, 2 * ff])),
            3 * n * ff * es, 10.0 * n * ff, VECTOR_FLOPS)
        row(f"{phase}.qwen2.swiglu", timed(lambda: ops.swiglu(gu)), 3 * n * top * ff * es, 4.0 * n * top * ff, VECTOR_FLOPS)
        g1 = rnd(n, 2 * ff)                                    # the same launch at the shared expert's width: the clamped unit's like at equal bytes
        row(f"{phase}.qwen2.swiglu(shared width)", timed(lambda: ops.swiglu(g1)), 3 * n * ff * es, 4.0 * n * ff, VECTOR_FLOPS)
        # routed experts: clamped gated units, softmax routing  |  Lokizen: relu^2 units, sigmoid routing
        h, z = rnd(n, W), torch.randn(n, E, device=dev)
        used = min(E, n * top)
        t_moe = timed(lambda: LO.moe_experts(h, z, None, top, 1.0, w_gu, w_down, route="softmax_renorm", renorm_eps=1e-20,
                                             gated=(LO.ACT_CLAMPED_SWISH, 7.0, 1.702, 1.0)))
        row(f"{phase}.moe_experts(gated)", t_moe, used * 3 * ff * W * es + n * W * es + n * top * W * 4, 6.0 * n * top * ff * W, MATRIX_FLOPS)
        t_moe = timed(lambda: LO.moe_experts(h, z, None, top, 1.0, w_up, w_down))
        row(f"{phase}.lokizen.moe_experts", t_moe, used * 2 * ff * W * es + n * W * es + n * top * W * 4, 4.0 * n * top * ff * W, MATRIX_FLOPS)
    return out


# Mikipel at Lokizen's widths, depths, head counts, head sizes and experts: the delta rule where Lokizen has retention, grouped-query
# attention and latent attention (Vumalix's latent sizes) taking turns where it has windowed attention; one dense feed-forward of the
# experts' active width, experts elsewhere; four taps
def mikipel_config(s):
    from ..modeling.mikipel import MikipelConfig
    H, G, D, W = s["heads"], s["kv"], s["dim"], s["width"]
    v = VSIZES["small" if W <= 1024 else "medium"]
    moe = {"kind": "moe", "expert": {"ff": s["ff"]}, "router": {"experts": s["experts"], "top": s["top"]}}
    dense = {"kind": "dense", "ff": s["top"] * s["ff"]}
    dlt = {"type": "delta", "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "conv": 4}}
    att = {"type": "attention", "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, "rot": {"dims": D, "base": 1e6, "scaling": {"factor": 8.0}}}}
    lat = {"type": "latent_attention", "mixer": {"heads": v["lheads"], "dim": v["ldim"], "rot_dim": v["rot"], "vdim": v["lvdim"], "kv_rank": v["kv_rank"],
                                                 "scale": (v["ldim"] + v["rot"]) ** -0.5, "rot": {"dims": v["rot"], "base": 1e6}}}
    order = [dlt, att, dlt, lat]
    return MikipelConfig.from_dict({"architecture": "Mikipel", "vocab": s["vocab"], "width": W, "norm": {"eps": 1e-6}, "embedding": {"scale": W ** 0.5},
                                    "residual_mult": 0.3, "logit_softcap": 30.0,
                                    "layers": [dict(order[i % 4], mlp=dense if i == 1 else moe) for i in range(s["layers"])]})


def bench_mikipel(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    from ..modeling.mikipel import random_model
    model = random_model(mikipel_config(s), "cuda", dtype, max_positions=max(prompt_len, context) + 64)
    return bench_ragged(model, s["vocab"], prompts, prompt_len, decode_batch, context)


def kernel_table_mikipel(s, prompts, prompt_len, decode_batch, context, dtype=torch.bfloat16):
    """Mikipel's layer kernels alone at the size's shapes, prefill and decode, each beside the like kernel of the closest model
    (Lokizen's residual + norm launch, its retention scan, its windowed attention, its routed experts; Vumalix's convolution; Qwen2's
    SwiGLU launch)."""
    from .. import layer_ops as LO
    from .. import ops
    dev = "cuda"
    H, G, D, W, E, top, ff, win, L = s["heads"], s["kv"], s["dim"], s["width"], s["experts"], s["top"], s["ff"], s["window"], s["layers"]
    page, es = 64, 2
    per = -(-(max(prompt_len, context) + 1) // page)
    slots = max(prompts, decode_batch)
    tables = [list(range(b * per, (b + 1) * per)) for b in range(slots)]
    g = torch.Generator().manual_seed(0)
    rnd = lambda *sh: torch.randn(*sh, generator=g).to(dev).to(dtype)
    kc, vc = rnd(slots * per * page, G * D), rnd(slots * per * page, G * D)
    a = torch.arange(max(prompt_len, context) + 8, dtype=torch.float32, device=dev).view(-1, 1) * torch.rand(D // 2, device=dev).view(1, -1)
    cos, sin = a.cos().contiguous(), a.sin().contiguous()
    state, decay = torch.zeros((slots, H, D, D), device=dev), torch.full((H,), 0.99, device=dev)
    a_log, dt_bias, nw = torch.zeros(H, device=dev), torch.zeros(H, device=dev), torch.ones(D, device=dev)
    C_ = 2 * G * D + H * D
    taps = 4
    ctail, stail, vtail = torch.zeros((slots, taps - 1, C_), device=dev), torch.zeros((slots, 1, W), device=dev), torch.zeros((slots, taps - 1, W), device=dev)
    w_gu, w_up, w_down = rnd(E, 2 * ff, W) * 0.02, rnd(E, ff, W) * 0.02, rnd(E, W, ff) * 0.02
    out = {}

    def row(name, secs, nbytes, flops, peak):
        bound = max(nbytes / HBM_BPS, flops / peak)
        out[name] = {"us": round(1e6 * secs, 1), "MB": round(nbytes / 1e6, 2), "GFLOP": round(flops / 1e9, 2), "roofline_fraction": round(bound / secs, 4)}

    for phase, B, T, start in (("prefill", prompts, prompt_len, 0), ("decode", decode_batch, 1, context)):
        n = B * T
        batch = LO.RaggedBatch.build([T] * B, [start] * B, list(range(B)), tables[:B], page, dev)
        causal = B * sum(start + t + 1 for t in range(T))                                       # visible (query, key) pairs per head
        windowed = B * sum(min(start + t + 1, win) for t in range(T))
        span_c, span_w = B * (start + T), B * min(start + T, win + T)                              # pool rows a launch has to read once
        # residual sum + mixture of the depths + norm (rounded and unrounded), at half depth and at full depth  |  Lokizen: one addend, one norm
        x, y1, y2, wn = torch.randn(n, W, device=dev), rnd(n, W), torch.randn(n, top, W, device=dev), torch.randn(W, device=dev)
        streams, mix, xo = torch.randn(L + 1, n, W, device=dev), torch.randn(L + 1, device=dev), torch.empty(n, W, device=dev)
        for d in (L // 2, L):
            row(f"{phase}.depth_mix_norm(depth {d})", timed(lambda: LO.depth_mix_norm(x, [(y1, None), (y2, None)], 0.3, streams, d, mix, xo, wn, 1e-6, dtype, want_float=True)),
                n * W * (4 + es + 4 * top + 4 + 4 * d + 4 + 4 + es + 4), (2.0 * d + 10) * n * W, VECTOR_FLOPS)
        row(f"{phase}.lokizen.add_rmsnorm", timed(lambda: LO.add_rmsnorm(x, y2, None, wn.to(dtype), 1e-5, dtype)), n * W * (4 + 4 * top + 4 + 4 + es), 4.0 * n * W, VECTOR_FLOPS)
        hf = torch.randn(n, W, device=dev)
        row(f"{phase}.token_shift", timed(lambda: LO.token_shift(hf, wn, batch, stail, dtype)), n * W * (4 + es), 3.0 * n * W, VECTOR_FLOPS)
        # short convolution + silu of q | k | v  |  Vumalix: convolution of the stream, added to it
        proj = rnd(n, C_ + H * D + 2 * H + (-(C_ + H * D + 2 * H)) % 8)
        cw = rnd(C_, taps)
        row(f"{phase}.short_conv(silu)", timed(lambda: LO.short_conv(proj, 0, C_, cw, batch, ctail, LO.ACT_SILU)), n * C_ * (es + 4), (2.0 * taps + 4) * n * C_, VECTOR_FLOPS)
        vw = rnd(W, taps)
        row(f"{phase}.vumalix.causal_conv", timed(lambda: LO.causal_conv(x, vw, batch, vtail)), n * W * (4 + es), 2.0 * taps * n * W, VECTOR_FLOPS)
        # gated delta rule  |  Lokizen: retention (fixed decay, no correction term)
        qkv = LO.short_conv(proj, 0, C_, cw, batch, ctail, LO.ACT_SILU)
        t_dl = timed(lambda: LO.delta_rule(qkv, (0, G * D, 2 * G * D), proj, (C_ + H * D, C_ + H * D + H, C_), a_log, dt_bias, nw, batch, H, G, D, D, 1e-6, D ** -0.5, 1e-6, state))
        row(f"{phase}.delta_rule", t_dl, n * (C_ * 4 + (2 * H * D + 2 * H) * es) + 2 * B * H * D * D * 4, 6.0 * n * H * D * D, VECTOR_FLOPS)
        pr = rnd(n, 4 * H * D)
        t_ret = timed(lambda: LO.retention(pr, (0, H * D, 2 * H * D, 3 * H * D), batch, H, D, D, D, cos, sin, decay, 1e-5, state))
        row(f"{phase}.lokizen.retention", t_ret, n * 5 * H * D * es + 2 * B * H * D * D * 4, 4.0 * n * H * D * D, VECTOR_FLOPS)
        # plain causal grouped-query attention (rotation + unit norm + append, then the one-sweep kernel)  |  Lokizen: windowed attention
        pa = rnd(n, H * D + 2 * G * D)
        cols = (0, H * D, H * D + G * D)
        t_hn = timed(lambda: LO.head_norm_append(pa, cols, H, G, 1, D, D, None, None, 1e-6, 0.0, 1, batch, kc, vc, rot_dims=D, cos=cos, sin=sin))
        row(f"{phase}.head_norm_append(rot)", t_hn, 2 * n * (H * D + 2 * G * D) * es, 10.0 * n * (H + G) * D, VECTOR_FLOPS)
        q = LO.head_norm_append(pa, cols, H, G, 1, D, D, None, None, 1e-6, 0.0, 1, batch, kc, vc, rot_dims=D, cos=cos, sin=sin)
        sweep = LO.attn_sweep_tile_rows(dtype, H, G, D, D, kc, vc) > 0
        t_at = timed(lambda: LO.attn_sweep(q, kc, vc, batch, H, G, D, D, D ** -0.5, 0) if sweep else LO.attn_window(q, None, kc, vc, batch, H, G, D, D, D ** -0.5, 0, 0, None, None, None))
        row(f"{phase}.attn_causal", t_at, span_c * 2 * G * D * es + 2 * n * H * D * es, 4.0 * causal * H * D, MATRIX_FLOPS)
        gate = rnd(n, H * D)
        rel, talk = torch.randn(max(prompt_len, context) + 8, H, device=dev), torch.eye(H, device=dev)
        t_lw = timed(lambda: LO.attn_window(q, gate, kc, vc, batch, H, G, D, D, D ** -0.5, win, 4, rel, None, talk))
        row(f"{phase}.lokizen.attn_window", t_lw, span_w * 2 * G * D * es + 3 * n * H * D * es, 4.0 * windowed * H * D, MATRIX_FLOPS)
        # latent attention without a query latent, neighbouring rotation pairs, no window
        v = VSIZES["small" if W <= 1024 else "medium"]
        LH, LD, rd, LDv, R = v["lheads"], v["ldim"], v["rot"], v["lvdim"], v["kv_rank"]
        lat = rnd(slots * per * page, R + rd)
        pl = rnd(n, LH * (LD + rd) + R + rd)
        wlk = rnd(R)
        al = torch.arange(max(prompt_len, context) + 8, dtype=torch.float32, device=dev).view(-1, 1) * torch.rand(rd // 2, device=dev).view(1, -1)
        lc, ls_ = al.cos().contiguous(), al.sin().contiguous()
        t_lp = timed(lambda: LO.latent_prep(pl, 0, 0, LH * (LD + rd), R, rd, rd, None, wlk, 1e-6, batch, lc, ls_, lat, pairing=LO.ROT_NEIGHBOURS))
        row(f"{phase}.latent_prep", t_lp, 2 * n * (R + rd) * es, 6.0 * n * (R + rd), VECTOR_FLOPS)
        qa, ql = rnd(LH, n, R), pl[:, :LH * (LD + rd)]
        row(f"{phase}.latent_q_pack", timed(lambda: LO.latent_q_pack(qa, ql, LH, LD, R, rd, rd, batch, lc, ls_, pairing=LO.ROT_NEIGHBOURS)), 2 * n * LH * (R + rd) * es,
            6.0 * n * LH * rd, VECTOR_FLOPS)
        qf = LO.latent_q_pack(qa, ql, LH, LD, R, rd, rd, batch, lc, ls_, pairing=LO.ROT_NEIGHBOURS)
        step = LO.ATTN_MAX_VALUE_WIDTH

        def latent_attn():
            if LO.attn_sweep_tile_rows(dtype, LH, 1, R + rd, R, lat, lat[:, :R]):
                return LO.attn_sweep(qf, lat, lat[:, :R], batch, LH, 1, R + rd, R, 0.1, 0)
            return [LO.attn_window(qf, None, lat, lat[:, c0:min(R, c0 + step)], batch, LH, 1, R + rd, min(R, c0 + step) - c0, 0.1, 0, 0, None, None, None)
                    for c0 in range(0, R, step)]
        row(f"{phase}.attn_latent", timed(latent_attn), span_c * (R + rd) * es + n * LH * (2 * R + rd) * es, 2.0 * causal * LH * (2 * R + rd), MATRIX_FLOPS)
        # activations  |  Qwen2's SwiGLU launch
        up = rnd(n, top * ff)
        row(f"{phase}.gated_act(gelu_erf, no linear branch)", timed(lambda: LO.gated_act(up, 0, -1, top * ff, LO.ACT_GELU_ERF)), 2 * n * top * ff * es, 10.0 * n * top * ff, VECTOR_FLOPS)
        gu = rnd(n, 2 * top * ff)
        row(f"{phase}.qwen2.swiglu", timed(lambda: ops.swiglu(gu)), 3 * n * top * ff * es, 4.0 * n * top * ff, VECTOR_FLOPS)
        # routed experts: silu units, softmax over the chosen logits  |  Lokizen: relu^2 units, sigmoid routing
        h, z = rnd(n, W), torch.randn(n, E, device=dev)
        used = min(E, n * top)
        t_moe = timed(lambda: LO.moe_experts(h, z, None, top, 1.0, w_gu, w_down, route="top_softmax", gated=(LO.ACT_SILU, 0.0, 1.0, 0.0)))
        row(f"{phase}.moe_experts(silu units)", t_moe, used * 3 * ff * W * es + n * W * es + n * top * W * 4, 6.0 * n * top * ff * W, MATRIX_FLOPS)
        t_moe = timed(lambda: LO.moe_experts(h, z, None, top, 1.0, w_up, w_down))
        row(f"{phase}.lokizen.moe_experts", t_moe, used * 2 * ff * W * es + n * W * es + n * top * W * 4, 4.0 * n * top * ff * W, MATRIX_FLOPS)
        zl = torch.randn(B, s["vocab"], device=dev)
        row(f"{phase}.softcap", timed(lambda: LO.softcap(zl, 30.0)), 2 * B * s["vocab"] * 4, 8.0 * B * s["vocab"], VECTOR_FLOPS)
    return out


def run_mikipel(sizes=("small", "medium"), prompts=4, prompt_len=2048, decode_batch=32, context=2048, kernels=True):
    res = {"bench": "ragged_family", "design": "Mikipel", "closest": "Lokizen", "dtype": "bf16", "data": "synthetic", "prompts": prompts,
           "prompt_len": prompt_len, "decode_batch": decode_batch, "context": context, "sizes": {}}
    for name in sizes:
        s = SIZES[name]
        entry = {"shape": s, "mikipel": bench_mikipel(s, prompts, prompt_len, decode_batch, context)}
        torch.cuda.empty_cache()
        entry["lokizen"] = bench_lokizen(s, prompts, prompt_len, decode_batch, context)
        torch.cuda.empty_cache()
        entry["qwen2"] = bench_qwen2(s, prompts, prompt_len, decode_batch, context)
        torch.cuda.empty_cache()
        if kernels:
            entry["kernels"] = kernel_table_mikipel(s, prompts, prompt_len, decode_batch, context)
            torch.cuda.empty_cache()
        res["sizes"][name] = entry
    return res


def run_bamanex(sizes=("small", "medium"), prompts=4, prompt_len=2048, decode_batch=32, context=2048, kernels=True):
    res = {"bench": "ragged_family", "design": "Bamanex", "closest": "Lokizen", "dtype": "bf16", "data": "synthetic", "prompts": prompts,
           "prompt_len": prompt_len, "decode_batch": decode_batch, "context": context, "sizes": {}}
    for name in sizes:
        s = SIZES[name]
        entry = {"shape": s, "bamanex": bench_bamanex(s, prompts, prompt_len, decode_batch, context)}
        torch.cuda.empty_cache()
        entry["lokizen"] = bench_lokizen(s, prompts, prompt_len, decode_batch, context)
        torch.cuda.empty_cache()
        entry["qwen2"] = bench_qwen2(s, prompts, prompt_len, decode_batch, context)
        torch.cuda.empty_cache()
        if kernels:
            entry["kernels"] = kernel_table_bamanex(s, prompts, prompt_len, decode_batch, context)
            torch.cuda.empty_cache()
        res["sizes"][name] = entry
    return res


def run_vumalix(sizes=("small", "medium"), prompts=4, prompt_len=2048, decode_batch=32, context=2048, kernels=True):
    res = {"bench": "ragged_family", "design": "Vumalix", "closest": "Lokizen", "dtype": "bf16", "data": "synthetic", "prompts": prompts,
           "prompt_len": prompt_len, "decode_batch": decode_batch, "context": context, "sizes": {}}
    for name in sizes:
        s = VSIZES[name]
        entry = {"shape": s, "vumalix": bench_vumalix(s, prompts, prompt_len, decode_batch, context)}
        torch.cuda.empty_cache()
        entry["lokizen"] = bench_lokizen(SIZES[name], prompts, prompt_len, decode_batch, context)
        torch.cuda.empty_cache()
        entry["qwen2"] = bench_qwen2(dict(SIZES[name], top=1, ff=s["ff"]), prompts, prompt_len, decode_batch, context)
        torch.cuda.empty_cache()
        if kernels:
            entry["kernels"] = kernel_table_vumalix(s, prompts, prompt_len, decode_batch, context)
            torch.cuda.empty_cache()
        res["sizes"][name] = entry
    return res


def run(sizes=("small", "medium"), prompts=4, prompt_len=2048, decode_batch=32, context=2048, kernels=True, design="lokizen"):
    if design.lower() == "vumalix":
        return run_vumalix(sizes, prompts, prompt_len, decode_batch, context, kernels)
    if design.lower() == "bamanex":
        return run_bamanex(sizes, prompts, prompt_len, decode_batch, context, kernels)
    if design.lower() == "mikipel":
        return run_mikipel(sizes, prompts, prompt_len, decode_batch, context, kernels)
    res = {"bench": "ragged_family", "design": "Lokizen", "closest": "Qwen2", "dtype": "bf16", "data": "synthetic", "prompts": prompts,
           "prompt_len": prompt_len, "decode_batch": decode_batch, "context": context, "sizes": {}}
    for name in sizes:
        s = SIZES[name]
        entry = {"shape": s, "lokizen": bench_lokizen(s, prompts, prompt_len, decode_batch, context)}
        torch.cuda.empty_cache()
        entry["qwen2"] = bench_qwen2(s, prompts, prompt_len, decode_batch, context)
        torch.cuda.empty_cache()
        if kernels:
            entry["kernels"] = kernel_table(s, prompts, prompt_len, decode_batch, context)
            torch.cuda.empty_cache()
        res["sizes"][name] = entry
    return res


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--design", default="lokizen", choices=("lokizen", "vumalix", "bamanex", "mikipel"))
    ap.add_argument("--sizes", default="small,medium")
    ap.add_argument("--prompts", type=int, default=4)
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--decode-batch", type=int, default=32)
    ap.add_argument("--context", type=int, default=2048)
    ap.add_argument("--no-kernels", action="store_true")
    a = ap.parse_args(argv)
    print(json.dumps(run(tuple(a.sizes.split(",")), a.prompts, a.prompt_len, a.decode_batch, a.context, not a.no_kernels, a.design)), flush=True)


if __name__ == "__main__":
    main()
