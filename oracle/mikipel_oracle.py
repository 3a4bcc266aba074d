"""Plain, slow restatement of the Mikipel decoder in torch on the CPU, one function per mechanism.  Test infrastructure only:
nothing under ``jacobiforcing_amd/`` imports it and it shares no code with the package.  Every function works on ONE whole
sequence (tokens 0 .. T-1) in the dtype of its inputs (float32 or float64) and has no cache: attention is a masked score
matrix, the recurrent mixer a loop over the tokens from a zero state.

Notation: ``h`` [T, width] a sublayer's input, ``P`` a dict of a layer's tensors keyed by the name behind ``l<i>.`` (``mix.q``,
``mlp.e3.up`` ...), ``m`` the layer's ``mixer`` entry and ``f`` its ``mlp`` entry of config.json."""
from __future__ import annotations

import math

import torch


def rms_norm(x, w=None, eps=1e-6):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def gelu_erf(z):
    return 0.5 * z * (1 + torch.erf(z / math.sqrt(2.0)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def token_shift(h, mu):
    """h_t + (h_(t-1) - h_t) * mu, with zeros in front of the first token."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


def angles(T, dims, base, factor=1.0, dtype=torch.float64):
    f = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(dims // 2)], dtype=dtype)
    return torch.arange(T, dtype=dtype).view(T, 1) * f.view(1, -1)                         # [T, dims/2]


def rotate_halves(x, a):
    """x [T, heads, >= dims]: dimension i pairs with i + dims/2; a [T, dims/2]."""
    half = a.shape[1]
    c, s = a.cos().unsqueeze(1), a.sin().unsqueeze(1)
    u, v, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
    return torch.cat([u * c - v * s, v * c + u * s, rest], -1)


def rotate_neighbours(x, a):
    """x [T, heads, >= dims]: dimension 2i pairs with 2i + 1; a [T, dims/2]."""
    half = a.shape[1]
    c, s = a.cos().unsqueeze(1), a.sin().unsqueeze(1)
    u, v, rest = x[..., 0:2 * half:2], x[..., 1:2 * half:2], x[..., 2 * half:]
    out = torch.stack([u * c - v * s, v * c + u * s], -1).flatten(-2)
    return torch.cat([out, rest], -1)


def causal_softmax(s):
    """s [heads, T, T] scores -> weights over the keys j <= i."""
    T = s.shape[-1]
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    return torch.softmax(s.masked_fill(~mask, float("-inf")), -1)


def attention_mixer(h, P, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ P["mix.q"].T).view(T, H, D)
    k = (h @ P["mix.k"].T).view(T, G, D)
    v = (h @ P["mix.v"].T).view(T, G, Dv)
    rot = m.get("rot") or {}
    if rot.get("dims", 0):
        a = angles(T, rot["dims"], rot["base"], (rot.get("scaling") or {}).get("factor", 1.0), h.dtype)
        q, k = rotate_halves(q, a), rotate_halves(k, a)
    q, k = rms_norm(q, None, eps), rms_norm(k, None, eps)
    rep = H // G
    k, v = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
    w = causal_softmax(torch.einsum("ihd,jhd->hij", q, k) * m["scale"])
    return torch.einsum("hij,jhd->ihd", w, v).reshape(T, H * Dv) @ P["mix.o"].T


def latent_attention_mixer(h, P, m, eps):
    """Keys and values the long way round: built per token and head from the latent."""
    T = h.shape[0]
    H, D, rd, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ P["mix.q"].T).view(T, H, D + rd)
    ckr = h @ P["mix.dkv"].T
    c = rms_norm(ckr[:, :R], P["mix.dkv.norm"], eps)
    kr = ckr[:, R:].view(T, 1, rd)
    rot = m.get("rot") or {}
    qr = q[..., D:]
    if rot.get("dims", 0):
        a = angles(T, rot["dims"], rot["base"], (rot.get("scaling") or {}).get("factor", 1.0), h.dtype)
        qr, kr = rotate_neighbours(qr, a), rotate_neighbours(kr, a)
    ku = (c @ P["mix.uk"].T).view(T, H, D)
    v = (c @ P["mix.uv"].T).view(T, H, Dv)
    s = torch.einsum("ihd,jhd->hij", q[..., :D], ku) + torch.einsum("ihd,jd->hij", qr, kr[:, 0])
    w = causal_softmax(s * m["scale"])
    return torch.einsum("hij,jhd->ihd", w, v).reshape(T, H * Dv) @ P["mix.o"].T


def short_conv(x, w):
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] * x_(t - taps + 1 + j), zeros before the start."""
    T, taps = x.shape[0], w.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x], 0)
    y = torch.zeros_like(x)
    for j in range(taps):
        y = y + xp[j:j + T] * w[:, j]
    return y


def delta_mixer(h, P, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(h @ P["mix.q"].T, P["mix.q.conv"])).view(T, G, D)
    k = silu(short_conv(h @ P["mix.k"].T, P["mix.k.conv"])).view(T, G, D)
    v = silu(short_conv(h @ P["mix.v"].T, P["mix.v.conv"])).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ P["mix.b"].T)                                                 # [T, H]
    g = torch.exp(-torch.exp(P["mix.A_log"]) * softplus(h @ P["mix.a"].T + P["mix.dt_bias"]))
    gate = (h @ P["mix.g"].T).view(T, H, Dv)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for hh in range(H):
        c = hh // (H // G)
        S = torch.zeros(D, Dv, dtype=h.dtype)
        for t in range(T):
            S = g[t, hh] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, c])
            S = S + torch.outer(k[t, c], u)
            out[t, hh] = S.T @ q[t, c]
    out = rms_norm(out, P["mix.norm"], eps) * silu(gate)
    return out.reshape(T, H * Dv) @ P["mix.o"].T


def route(z, top):
    """z [T, E] router logits -> (indices [T, top], weights [T, top]): the largest logits, softmax over the chosen ones only."""
    val, idx = torch.sort(z, dim=-1, descending=True, stable=True)
    return idx[:, :top], torch.softmax(val[:, :top], -1)


def feed_forward(h, P, f):
    if f is None:
        return torch.zeros_like(h)
    if f.get("kind", "dense") == "dense":
        return gelu_erf(h @ P["mlp.up"].T) @ P["mlp.down"].T
    idx, wt = route(h @ P["mlp.router"].T + P["mlp.router.b"], f["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, we in zip(idx[t].tolist(), wt[t]):
            p = f"mlp.e{e}."
            out[t] = out[t] + we * ((silu(P[p + "gate"] @ h[t]) * (P[p + "up"] @ h[t])) @ P[p + "down"].T)
    return out


MIXERS = {"attention": attention_mixer, "latent_attention": latent_attention_mixer, "delta": delta_mixer}


def forward(cfg: dict, tensors: dict, tokens, dtype=torch.float64, trace=None):
    """Logits [T, vocab] of one whole sequence.  ``trace``, when a list, receives the stream every layer hands on."""
    t = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    outs = [x]                                                   # the embedding output and every layer's own result
    for i, L in enumerate(cfg["layers"]):
        P = {k[len(f"l{i}."):]: v for k, v in t.items() if k.startswith(f"l{i}.")}
        h = rms_norm(x, P["norm1"], eps)
        y = x + mult * (MIXERS[L["type"]](token_shift(h, P["shift"]), P, L["mixer"], eps) + feed_forward(h, P, L.get("mlp")))
        outs.append(y)
        x = sum(P["dwa"][j] * outs[j] for j in range(i + 2))
        if trace is not None:
            trace.append(x.clone())
    z = rms_norm(x, t["final.norm"], eps) @ t["embed"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z
