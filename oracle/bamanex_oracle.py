"""Plain, slow restatement of the Bamanex decoder in torch on the CPU, one function per mechanism.  Test infrastructure only:
nothing under ``jacobiforcing_amd/`` imports it and it shares no code with the package.  Every function works on ONE whole
sequence (tokens 0 .. T-1) in the dtype of its inputs (float32 or float64) and has no cache: position t simply sees what its
mask lets it see; a looped span of layers is simply run again.

The design: a float residual stream; every layer reads the stream through TWO zero-centred RMS norms (weight stored as w, applied
as 1 + w), one feeding the mixer and one the feed-forward, and adds both results — each scaled per channel — in one sum.  The
mixer is grouped-query attention with biased projections, a partial rotation whose frequencies are stretched for long wavelengths,
unit-RMS queries and keys, a sliding window, a per-head sink in the softmax's denominator and a per-head sigmoid gate.  The
feed-forward is either a gated dense layer (tanh-form gelu) or a mixture of experts with clamped gated units, softmax routing
renormalised over the chosen experts, and a gated shared expert.

Notation: ``h`` [T, width] what a sublayer reads, ``P`` a dict of a layer's tensors keyed by the name behind ``l<i>.`` (``mix.q``,
``mlp.up`` …), ``m`` the layer's ``mixer`` entry of config.json, ``f`` its ``mlp`` entry."""
from __future__ import annotations

import math

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def centred_norm(x, w, eps):
    """RMS norm whose stored weight is the deviation from one."""
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def stretched_frequencies(dims: int, base: float, scaling) -> list:
    """f_i = base^(-2i/dims), i < dims/2; with ``scaling`` {factor, low, high, original}: a frequency whose wavelength is shorter
    than original/high stays, one longer than original/low is divided by factor, and between the two the result slides from the
    divided to the kept frequency with s = (original/wavelength - low) / (high - low).  Written over the whole vector at once."""
    f = torch.tensor(float(base), dtype=torch.float64) ** (-torch.arange(0, dims, 2, dtype=torch.float64) / dims)
    if scaling:
        factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        turns = orig * f / (2.0 * math.pi)                               # how often the pair goes round within `original` positions
        s = ((turns - low) / (high - low)).clamp(0.0, 1.0)               # 0: long wavelengths, 1: short ones
        f = (1.0 - s) * f / factor + s * f
    return f.tolist()


def rotate_pairs(vec, position: int, freqs):
    """vec [.., d]: of the first 2 * len(freqs) entries, i and i + len(freqs) are a pair turned by position * freqs[i]; the angle is
    formed and its cosine / sine taken in float32."""
    half = len(freqs)
    a = torch.tensor(float(position), dtype=torch.float32) * torch.tensor(freqs, dtype=torch.float32)
    c, s = torch.cos(a).to(vec.dtype), torch.sin(a).to(vec.dtype)
    u, v = vec[..., :half], vec[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, vec[..., 2 * half:]], -1)


def sink_softmax(scores, sink):
    """Softmax over ``scores`` whose denominator holds one more term exp(sink): the weights sum to less than one."""
    top = torch.maximum(scores.max(), sink)
    e = torch.exp(scores - top)
    return e / (e.sum() + torch.exp(sink - top))


def gated_sink_attention(h, P, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    freqs = stretched_frequencies(int(rot.get("dims", 0)), float(rot.get("base", 10000.0)), rot.get("scaling"))
    size = (m.get("mask") or {}).get("size", 0) or T + 1
    q = (h @ P["mix.q"].T + P["mix.q.b"]).view(T, H, D)
    k = (h @ P["mix.k"].T + P["mix.k.b"]).view(T, G, D)
    v = (h @ P["mix.v"].T + P["mix.v.b"]).view(T, G, Dv)
    q = torch.stack([unit_rms(rotate_pairs(q[t], t, freqs), eps) for t in range(T)])
    k = torch.stack([unit_rms(rotate_pairs(k[t], t, freqs), eps) for t in range(T)])
    gate = torch.sigmoid(h @ P["mix.g"].T)                               # [T, H]
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for i in range(T):
        lo = max(0, i - size + 1)
        for hh in range(H):
            c = hh // (H // G)
            w = sink_softmax((k[lo:i + 1, c] @ q[i, hh]) * m["scale"], P["mix.sink"][hh])
            out[i, hh] = (w @ v[lo:i + 1, c]) * gate[i, hh]
    return out.reshape(T, H * Dv) @ P["mix.o"].T + P["mix.o.b"]


def dense_feed_forward(h, P, prefix="mlp."):
    return (gelu_tanh(h @ P[prefix + "gate"].T) * (h @ P[prefix + "up"].T)) @ P[prefix + "down"].T


def clamped_unit(h, P, prefix, limit):
    """An expert: the gate is capped from above, the linear branch from both sides and shifted by one."""
    g = torch.clamp(h @ P[prefix + "gate"].T, max=limit)
    u = torch.clamp(h @ P[prefix + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ P[prefix + "down"].T


def route(h, P, f):
    """(chosen experts [T, top], their weights [T, top]): softmax over all experts in float32, the largest ``top`` scores (ties: the
    lower index), renormalised over the chosen."""
    z = h.to(torch.float32) @ P["mlp.router"].to(torch.float32).T
    s = torch.softmax(z, -1)
    top = int(f["router"]["top"])
    ids = torch.zeros(h.shape[0], top, dtype=torch.long)
    for t in range(h.shape[0]):
        left = s[t].clone()
        for j in range(top):
            ids[t, j] = int(torch.argmax(left))                          # argmax returns the first of equal maxima
            left[ids[t, j]] = -1.0
    w = torch.gather(s, 1, ids)
    return ids, w / (w.sum(-1, keepdim=True) + 1e-20)


def expert_mixture(h, P, f):
    ids, w = route(h, P, f)
    out = torch.zeros(h.shape[0], P["mlp.e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            out[t] += w[t, j].to(h.dtype) * clamped_unit(h[t:t + 1], P, f"mlp.e{e}.", float(f["expert"]["limit"]))[0]
    if f.get("shared") is not None:
        out = out + torch.sigmoid(h @ P["mlp.shared.sg"].T) * clamped_unit(h, P, "mlp.shared.", float(f["shared"]["limit"]))
    return out


def feed_forward(h, P, f):
    return dense_feed_forward(h, P) if f.get("kind", "dense") == "dense" else expert_mixture(h, P, f)


def layer_tensors(tensors, i: int):
    p = f"l{i}."
    return {k[len(p):]: v for k, v in tensors.items() if k.startswith(p)}


def layer_order(cfg) -> list:
    """Layer indices in execution order: the looped span start .. stop-1 runs ``times`` times in a row."""
    n = len(cfg["layers"])
    lp = cfg.get("loop") or {}
    a, b, times = int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1))
    return list(range(a)) + list(range(a, b)) * (times if b > a else 0) + list(range(b, n))


def forward(cfg, tensors, tokens, dtype=torch.float64):
    """cfg: config.json as a dict.  Returns (logits [T, vocab], the stream after every layer run [runs, T, width])."""
    t = {k: v.to(dtype) for k, v in tensors.items()}
    eps = float(cfg["norm"]["eps"])
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    trace = []
    for li in layer_order(cfg):
        L, P = cfg["layers"][li], layer_tensors(t, li)
        if L["type"] != "attention":
            raise ValueError(f"layer {li}: unknown mixer {L['type']!r}")
        y = gated_sink_attention(centred_norm(x, P["norm1"], eps), P, L["mixer"], eps) * P["ls1"]
        if L.get("mlp") is not None:
            y = y + feed_forward(centred_norm(x, P["norm2"], eps), P, L["mlp"]) * P["ls2"]
        x = x + y
        trace.append(x.clone())
    logits = (centred_norm(x, t["final.norm"], eps) @ t["head"].T) * float(cfg.get("logit_scale", 1.0))
    return logits, torch.stack(trace)
