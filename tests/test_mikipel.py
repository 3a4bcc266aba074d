"""Mikipel through the package (HIP layer kernels, paged pools, state slots with named tails, ragged step, scheduler, LLM.generate)
against the plain oracle ``oracle/mikipel_oracle.py``, which shares no code with it.  Small random models of several shapes; where
random weights would hide a fault (a far key among hundreds, a key at a page's border, an old write in a recurrent state) the weights
and inputs are chosen so that it shows.

CPU tests cover the oracle's own pieces, the config reader and the cache layout; everything that launches a kernel is marked ``gpu``."""
import json
import random

import numpy as np
import pytest
import torch

from oracle import mikipel_oracle as O
from jacobiforcing_amd.modeling import MODEL_REGISTRY, read_model_config
from jacobiforcing_amd.modeling import mikipel as MK

gpu = pytest.mark.gpu


# ---- model shapes -----------------------------------------------------------------------------------------------------------------
def attn(heads=6, kv=2, dim=24, vdim=40, dims=16, base=500.0, scale=0.3, factor=4.0):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if dims:
        m["rot"] = {"dims": dims, "base": base}
        if factor:
            m["rot"]["scaling"] = {"factor": factor}
    return {"type": "attention", "mixer": m}


def latent(heads=3, dim=16, rot_dim=8, vdim=24, rank=40, dims=8, base=300.0, scale=0.25, factor=0.0):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if dims:
        m["rot"] = {"dims": dims, "base": base}
        if factor:
            m["rot"]["scaling"] = {"factor": factor}
    return {"type": "latent_attention", "mixer": m}


def delta(heads=4, kv=2, dim=24, vdim=20, conv=3):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}}


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=24):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def make_cfg(layers, width=96, vocab=131, eps=1e-5, emb=2.5, mult=0.4, cap=9.0):
    d = {"architecture": "Mikipel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers, "embedding": {"scale": emb}, "residual_mult": mult}
    if cap:
        d["logit_softcap"] = cap
    return d


def shape_a():
    """All three mixers, dense and expert feed-forwards and a layer without one, grouped heads, a rotation over a part of the head with
    and without scaling, different head sizes for keys and values, convolutions of three taps and of one (none)."""
    return make_cfg([dict(latent(), mlp=dense()), dict(delta(), mlp=moe()), dict(attn(), mlp=None), dict(delta(heads=2, kv=2, dim=40, vdim=72, conv=1), mlp=dense(24)),
                     dict(attn(heads=4, kv=4, dim=16, vdim=16, dims=16, factor=0.0), mlp=moe(experts=3, top=3, ff=20))])


def shape_b():
    """One head; one expert chosen; no rotation in one layer; sizes that are no multiples of eight; no soft cap, no embedding scale, a
    residual multiplier of one; five taps; one key head under three heads of the recurrent mixer."""
    return make_cfg([dict(attn(heads=1, kv=1, dim=20, vdim=12, dims=0), mlp=moe(experts=3, top=1, ff=20)),
                     dict(latent(heads=5, dim=12, rot_dim=6, vdim=20, rank=24, dims=4, factor=8.0), mlp=None),
                     dict(delta(heads=3, kv=1, dim=16, vdim=8, conv=5), mlp=moe(experts=4, top=2, ff=33)),
                     dict(latent(heads=2, dim=8, rot_dim=10, vdim=8, rank=12, dims=0), mlp=dense(30))],
                    width=64, vocab=77, eps=1e-6, emb=1.0, mult=1.0, cap=0.0)


def shape_c():
    """Head sizes the matrix-core attention kernels take in bfloat16, many heads over few key heads, a single layer kind per layer pair."""
    return make_cfg([dict(attn(heads=8, kv=2, dim=64, vdim=64, dims=32, base=1e6, scale=0.125), mlp=dense(48)),
                     dict(latent(heads=8, dim=32, rot_dim=32, vdim=32, rank=64, dims=32, scale=0.125), mlp=moe(experts=9, top=2, ff=16)),
                     dict(delta(heads=4, kv=2, dim=64, vdim=64, conv=2), mlp=dense(64))], width=128, vocab=50, mult=0.5, cap=20.0)


SHAPES = {"a": shape_a, "b": shape_b, "c": shape_c}


def tensors_for(cfg_dict, seed):
    return MK.random_tensors(MK.MikipelConfig.from_dict(cfg_dict), seed)


def layer_tensors(t, i, dtype=torch.float64):
    return {k[len(f"l{i}."):]: v.to(dtype) for k, v in t.items() if k.startswith(f"l{i}.")}


def rel_err(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.sqrt(((got - want) ** 2).mean()) / max(np.sqrt((want ** 2).mean()), 1e-30))


F32_TOL, BF16_TOL = 2e-4, 6e-2


def rows_off(got, want, tol):
    """Fraction of rows (positions) whose own relative error is above ``tol``.  In bfloat16 a router's close call may go the other way
    for a token — and, through a recurrent state, for the tokens behind it — so a test over random routers bounds how many rows differ."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    err = np.sqrt(((got - want) ** 2).mean(-1)) / np.maximum(np.sqrt((want ** 2).mean(-1)), 1e-30)
    return float((err > tol).mean())


def toks(n, vocab, seed):
    return [random.Random(seed * 7919 + i).randrange(vocab) for i in range(n)]


# =====================================================================================================================================
# CPU: oracle pieces, config reader, cache layout
# =====================================================================================================================================
def test_registry_reads_the_architecture_key(tmp_path):
    assert MODEL_REGISTRY["Mikipel"][2] == "ragged"
    (tmp_path / "config.json").write_text(json.dumps(shape_a()))
    cfg = read_model_config(tmp_path)
    assert isinstance(cfg, MK.MikipelConfig) and cfg.family == "ragged" and cfg.num_hidden_layers == 5
    assert (cfg.embedding_scale, cfg.residual_mult, cfg.logit_softcap, cfg.norm_eps) == (2.5, 0.4, 9.0, 1e-5)
    b = MK.MikipelConfig.from_dict(shape_b())
    assert (b.embedding_scale, b.residual_mult, b.logit_softcap) == (1.0, 1.0, 0.0)


def test_config_rejects_what_the_design_does_not_have():
    for change in (lambda c: c["layers"][0].update(type="retention"), lambda c: c["layers"][0]["mlp"].update(kind="polynomial"),
                   lambda c: c["layers"][2]["mixer"].update(kv_heads=4), lambda c: c["layers"][2]["mixer"]["rot"].update(dims=26),
                   lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), lambda c: c["layers"][2]["mixer"]["rot"].update(dims=7),
                   lambda c: c["layers"][1]["mixer"].update(conv=9), lambda c: c["layers"][1]["mixer"].update(kv_heads=3),
                   lambda c: c["layers"][1]["mlp"]["router"].update(top=6)):
        bad = shape_a()
        change(bad)
        with pytest.raises(ValueError):
            MK.MikipelConfig.from_dict(bad)


def test_cache_layout_and_stacked_weights():
    cfg = MK.MikipelConfig.from_dict(shape_a())
    w = MK.MikipelWeights(cfg, tensors_for(shape_a(), 1), "cpu", torch.float32)
    specs = MK.MikipelModel(cfg, w, max_positions=16).cache_specs()
    assert [s.kind for s in specs] == ["kv", "state", "kv", "state", "kv"]
    assert (specs[0].k_width, specs[0].v_width) == (48, 0) and (specs[2].k_width, specs[2].v_width) == (48, 80)
    assert specs[1].state_shape == (4, 24, 20) and specs[1].tails == {"shift": (1, 96), "conv": (2, 2 * 48 + 80)}
    assert specs[3].tails == {"shift": (1, 96)} and all(s.tails["shift"] == (1, 96) for s in specs)          # one tap: no convolution tail
    l0, l1, l2 = w.layers[0], w.layers[1], w.layers[2]
    assert tuple(l0["w_in"].shape) == (3 * 24 + 48, 96) and l0["kv_col"] == 72 and tuple(l0["w_uk"].shape) == (3, 16, 40) and tuple(l0["w_uv"].shape) == (3, 40, 24)
    rows = 2 * 48 + 80 + 80 + 8                                                                  # q, k, v, gate, decay input, step input
    assert tuple(l1["w_in"].shape) == (rows, 96) and l1["pcols"] == (256, 260, 176) and tuple(l1["conv"].shape) == (176, 3)
    assert tuple(l2["w_in"].shape) == (6 * 24 + 48 + 80, 96) and l2["cols"] == (0, 144, 192)
    assert tuple(l1["w_gu"].shape) == (5, 48, 96) and l1["router"].dtype == torch.float32 and l1["router_b"].numel() == 5
    assert [w.layers[i]["dwa"].numel() for i in range(5)] == [2, 3, 4, 5, 6] and "w_up" not in l2 and "w_gu" not in l2
    from jacobiforcing_amd.engine.state_cache import PagedStateCache
    cache = PagedStateCache(specs, 4, 8, 3, "cpu", torch.float32)
    assert tuple(cache.tails[1]["conv"].shape) == (3, 2, 176) and tuple(cache.tails[4]["shift"].shape) == (3, 1, 96) and cache.v[0] is None
    assert tuple(cache.state[3].shape) == (3, 2, 40, 72) and cache.bytes() > 0


def test_oracle_pieces():
    g = torch.Generator().manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    z = torch.tensor([-3.0, 0.0, 0.5, 2.0], dtype=torch.float64)
    assert torch.allclose(O.gelu_erf(z), torch.nn.functional.gelu(z)) and torch.allclose(O.silu(z), torch.nn.functional.silu(z))
    assert torch.allclose(O.softplus(z), torch.nn.functional.softplus(z)) and float(O.softplus(torch.tensor(50.0, dtype=torch.float64))) == 50.0
    h, mu = rn(5, 7), torch.rand(7, generator=g, dtype=torch.float64)
    s = O.token_shift(h, mu)
    assert torch.allclose(s[0], h[0] * (1 - mu)) and torch.allclose(s[3], h[3] * (1 - mu) + h[2] * mu)
    assert torch.equal(O.token_shift(h, torch.zeros(7, dtype=torch.float64)), h)
    # both pairings keep lengths, leave the rest alone, do nothing at position 0 and differ from each other
    x, a = rn(4, 3, 10), O.angles(4, 6, 50.0, 2.0)
    assert torch.allclose(a[3], 3 * torch.tensor([1.0, 50.0 ** (-2 / 6), 50.0 ** (-4 / 6)], dtype=torch.float64) / 2.0)
    for rot in (O.rotate_halves, O.rotate_neighbours):
        r = rot(x, a)
        assert torch.allclose((r * r).sum(-1), (x * x).sum(-1)) and torch.equal(r[..., 6:], x[..., 6:]) and torch.allclose(r[0], x[0])
    assert not torch.allclose(O.rotate_halves(x, a)[1:], O.rotate_neighbours(x, a)[1:])
    u = O.rotate_neighbours(x, a)[2, 1]
    assert abs(float(u[2]) - float(x[2, 1, 2] * a[2, 1].cos() - x[2, 1, 3] * a[2, 1].sin())) < 1e-12
    v = O.rotate_halves(x, a)[2, 1]
    assert abs(float(v[4]) - float(x[2, 1, 4] * a[2, 1].cos() + x[2, 1, 1] * a[2, 1].sin())) < 1e-12
    # the convolution's last column is the current token's; the router's weights are a softmax over the chosen logits alone
    xs, w = rn(6, 3), rn(3, 4)
    y = O.short_conv(xs, w)
    assert torch.allclose(y[0], xs[0] * w[:, 3]) and torch.allclose(y[4], xs[4] * w[:, 3] + xs[3] * w[:, 2] + xs[2] * w[:, 1] + xs[1] * w[:, 0])
    idx, wt = O.route(torch.tensor([[0.1, 2.0, -1.0, 2.0, 1.5]], dtype=torch.float64), 3)
    assert idx.tolist() == [[1, 3, 4]] and torch.allclose(wt, torch.softmax(torch.tensor([[2.0, 2.0, 1.5]], dtype=torch.float64), -1))
    # the delta rule overwrites: after writing v along a unit key with step size one and no decay, reading along that key returns v
    m = {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 3, "conv": 1}
    one = torch.ones(1, 1, dtype=torch.float64)
    P = {"mix.q": torch.eye(4, dtype=torch.float64), "mix.k": torch.eye(4, dtype=torch.float64), "mix.v": torch.eye(4, dtype=torch.float64)[:3],
         "mix.q.conv": torch.ones(4, 1, dtype=torch.float64), "mix.k.conv": torch.ones(4, 1, dtype=torch.float64), "mix.v.conv": torch.ones(3, 1, dtype=torch.float64),
         "mix.b": 50 * torch.ones(1, 4, dtype=torch.float64), "mix.a": torch.zeros(1, 4, dtype=torch.float64), "mix.A_log": torch.tensor([-40.0], dtype=torch.float64),
         "mix.dt_bias": torch.zeros(1, dtype=torch.float64), "mix.g": 50 * torch.ones(3, 4, dtype=torch.float64), "mix.norm": torch.ones(3, dtype=torch.float64),
         "mix.o": torch.eye(3, dtype=torch.float64)}
    hh = torch.tensor([[3.0, 1.0, 2.0, 0.5]] * 2, dtype=torch.float64)
    out = O.delta_mixer(hh, P, m, 0.0)
    vv = O.silu(hh[0, :3])
    assert torch.allclose(out[0], out[1], atol=1e-9) and torch.allclose(out[0] / out[0].norm(), vv / vv.norm() , atol=1e-6) and float(one.sum()) == 1.0


# =====================================================================================================================================
# GPU: the package against the oracle
# =====================================================================================================================================
class Rig:
    """A model on the GPU with a pool of shuffled pages; runs steps of (request, tokens) and keeps the bookkeeping a test needs."""

    def __init__(self, cfg_dict, seed=0, dtype=torch.float32, page=8, pages=64, slots=4, tensors=None, max_positions=1024):
        from jacobiforcing_amd import layer_ops as LO
        self.LO = LO
        self.cfg_dict = cfg_dict
        self.cfg = MK.MikipelConfig.from_dict(cfg_dict)
        self.tensors = tensors or tensors_for(cfg_dict, seed)
        self.model = MK.MikipelModel(self.cfg, MK.MikipelWeights(self.cfg, self.tensors, "cuda", dtype), max_positions=max_positions)
        self.page = page
        self.cache = self.model.new_cache(pages, page, slots)
        self.free_pages = list(range(pages))
        random.Random(seed).shuffle(self.free_pages)
        self.free_slots = list(range(slots))[::-1]
        self.req = {}

    def poison(self):
        """Fill pools, states and tails with large values: whatever a kernel reads without having written it shows."""
        for t in self.cache.k + self.cache.v + self.cache.state + [x for d in self.cache.tails for x in d.values()]:
            if t is not None:
                t.fill_(1e4)

    def batch(self, entries):
        counts, starts, slots, tables, ids = [], [], [], [], []
        for key, tk in entries:
            r = self.req.setdefault(key, {"n": 0, "pages": [], "slot": None})
            if r["slot"] is None:
                r["slot"] = self.free_slots.pop()
            while len(r["pages"]) * self.page < r["n"] + len(tk):
                r["pages"].append(self.free_pages.pop())
            counts.append(len(tk)); starts.append(r["n"]); slots.append(r["slot"]); tables.append(r["pages"])
            ids += list(tk)
            r["n"] += len(tk)
        return self.LO.RaggedBatch.build(counts, starts, slots, tables, self.page, "cuda"), ids

    def step(self, entries, trace=None):
        """entries = [(key, tokens)]; returns logits [sum of tokens, vocab] (float, on the CPU)."""
        b, ids = self.batch(entries)
        return self.model.forward(torch.tensor(ids, device="cuda"), b, self.cache, None, trace).cpu()

    def end(self, key):
        r = self.req.pop(key)
        self.free_pages += r["pages"][::-1]
        self.free_slots.append(r["slot"])

    def oracle(self, tokens, trace=None):
        return O.forward(self.cfg_dict, self.tensors, list(tokens), torch.float64, trace)


@gpu
@pytest.mark.parametrize("W", [50, 96, 200, 1000, 2052])
def test_residual_sum_depth_mixture_and_norm(W):
    from jacobiforcing_amd import layer_ops as LO
    g = torch.Generator().manual_seed(W)
    rn = lambda *s: torch.randn(*s, generator=g)
    n = 5
    x, y1, y2, w, mix = rn(n, W), rn(n, W) * 3, rn(n, 3, W), rn(W), rn(4)
    streams = rn(5, n, W).cuda()
    before = streams.clone()
    own = x.double() + 0.3 * (y1.bfloat16().double() + y2.double().sum(1))
    mixed = sum(mix[j].double() * before[j].cpu().double() for j in range(3)) + mix[3].double() * own
    xo = torch.empty(n, W, device="cuda")
    o16, o32 = LO.depth_mix_norm(x.cuda(), [(y1.cuda().bfloat16(), None), (y2.cuda(), None)], 0.3, streams, 3, mix.cuda(), xo, w.cuda(), 1e-5, torch.bfloat16, want_float=True)
    assert rel_err(streams[3].cpu(), own) < 1e-6 and torch.equal(streams[:3], before[:3]) and torch.equal(streams[4], before[4])
    assert rel_err(xo.cpu(), mixed) < 1e-6 and rel_err(o32.cpu(), O.rms_norm(mixed, w.double(), 1e-5)) < 1e-6 and torch.equal(o16.cpu(), o32.cpu().bfloat16())
    # in place on the stream it reads; no mixture: the layer's own result goes on; float output alone
    xi = x.cuda()
    o = LO.depth_mix_norm(xi, [(y1.cuda(), None)], 2.0, streams, 1, None, xi, None, 1e-5, torch.float32)
    assert rel_err(xi.cpu(), x.double() + 2 * y1.double()) < 1e-6 and torch.equal(streams[1], xi) and rel_err(o.cpu(), O.rms_norm(x.double() + 2 * y1.double(), None, 1e-5)) < 1e-6
    # the norm alone (nothing written), the update alone (no stream kept), and eps inside the root
    keep = xi.clone()
    assert rel_err(LO.depth_mix_norm(xi, [], 0.3, None, -1, None, None, w.cuda(), 1e-5, torch.float32).cpu(), O.rms_norm(keep.cpu().double(), w.double(), 1e-5)) < 1e-6
    assert torch.equal(xi, keep)
    assert LO.depth_mix_norm(xi, [(y2.cuda(), None)], 0.5, None, -1, None, xo, None, 1e-5, None) is None and rel_err(xo.cpu(), keep.cpu().double() + 0.5 * y2.double().sum(1)) < 1e-6
    tiny = torch.full((1, W), 1e-4)
    assert rel_err(LO.depth_mix_norm(tiny.cuda(), [], 1.0, None, -1, None, None, w.cuda(), 1e-5, torch.float32).cpu(), O.rms_norm(tiny.double(), w.double(), 1e-5)) < 1e-6
    with pytest.raises(ValueError):
        LO.depth_mix_norm(x.cuda(), [(y1.cuda(), None)], 1.0, streams, 2, mix.cuda(), streams[1], None, 1e-5, None)      # the result inside what it is mixed from


@gpu
def test_token_shift_kernel_reads_and_moves_the_tail():
    from jacobiforcing_amd import layer_ops as LO
    g = torch.Generator().manual_seed(3)
    W = 70
    h, mu = torch.randn(7, W, generator=g), torch.rand(W, generator=g)
    tail = torch.randn(4, 1, W, generator=g)
    b = LO.RaggedBatch.build([3, 1, 2, 1], [0, 5, 2, 0], [2, 0, 3, 1], [[0], [1], [2], [3]], 8, "cuda")
    td = tail.cuda()
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 6e-3)):
        td.copy_(tail)
        out = LO.token_shift(h.cuda(), mu.cuda(), b, td, dtype).float().cpu()
        prev = torch.stack([torch.zeros(W), h[0], h[1], tail[0, 0], tail[3, 0], h[4], torch.zeros(W)])         # a start at position 0 never reads its slot
        assert rel_err(out, h.double() + (prev.double() - h.double()) * mu.double()) < tol
        assert torch.equal(td.cpu()[:, 0], torch.stack([h[3], h[6], h[2], h[5]]))
    # a step of single rows: the norm's launch shifts as well (the unrounded norm against the slot's tail, which it then replaces)
    x, w = torch.randn(4, W, generator=g), torch.randn(W, generator=g)
    b1 = LO.RaggedBatch.build([1, 1, 1, 1], [4, 0, 9, 1], [3, 1, 0, 2], [[0], [1], [2, 3], [4]], 8, "cuda")
    hn = O.rms_norm(x.double(), w.double(), 1e-5)
    prev = torch.stack([tail[3, 0], torch.zeros(W), tail[0, 0], tail[2, 0]]).double()
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 6e-3)):
        td.copy_(tail)
        o16, o32, sh = LO.depth_mix_norm(x.cuda(), [], 1.0, None, -1, None, None, w.cuda(), 1e-5, dtype, want_float=True, shift=(mu.cuda(), b1, td))
        assert rel_err(sh.float().cpu(), hn + (prev - hn) * mu.double()) < tol and rel_err(o32.cpu(), hn) < 1e-6 and o16.dtype == dtype
        assert rel_err(td.cpu()[[3, 1, 0, 2], 0], hn) < 1e-6
    with pytest.raises(ValueError):
        LO.depth_mix_norm(h.cuda(), [], 1.0, None, -1, None, None, None, 1e-5, torch.float32, shift=(mu.cuda(), b, td))       # a request with three rows


@gpu
@pytest.mark.parametrize("taps", [1, 2, 3, 4, 5, 8])
def test_short_convolution_across_portions(taps):
    from jacobiforcing_amd import layer_ops as LO
    g = torch.Generator().manual_seed(taps)
    C_, col, ld = 70, 3, 80
    xa, xb = torch.randn(23, ld, generator=g), torch.randn(12, ld, generator=g)
    w = torch.randn(C_, taps, generator=g)
    want = [O.silu(O.short_conv(x[:, col:col + C_].double(), w.double())) for x in (xa, xb)]
    plain = O.short_conv(xa[:, col:col + C_].double(), w.double())
    tail = torch.full((3, max(taps - 1, 1), C_), 1e4, device="cuda") if taps > 1 else None
    cuts = [(0, 9, 0, 1), (9, 10, 1, 3), (10, 19, 3, 4), (19, 23, 4, 12)]                        # portions beside single rows, shorter and longer than the taps
    got_a, got_b, got_p = [], [], []
    for a0, a1, b0, b1 in cuts:
        b = LO.RaggedBatch.build([a1 - a0, b1 - b0], [a0, b0], [2, 0], [[0, 1, 2], [3, 4]], 8, "cuda")
        x = torch.cat([xa[a0:a1], xb[b0:b1]]).cuda()
        y = LO.short_conv(x, col, C_, w.cuda(), b, tail, LO.ACT_SILU).cpu()
        got_a.append(y[:a1 - a0]); got_b.append(y[a1 - a0:])
    assert rel_err(torch.cat(got_a), want[0]) < 1e-6 and rel_err(torch.cat(got_b), want[1]) < 1e-6
    b = LO.RaggedBatch.build([23], [0], [1], [[0, 1, 2]], 8, "cuda")
    assert rel_err(LO.short_conv(xa.cuda(), col, C_, w.cuda(), b, tail, LO.ACT_NONE).cpu(), plain) < 1e-6
    xh = xa.cuda().bfloat16()
    wh = w.cuda().bfloat16()
    ref = O.silu(O.short_conv(xh.cpu().double()[:, col:col + C_], wh.cpu().double()))
    assert rel_err(LO.short_conv(xh, col, C_, wh, b, tail, LO.ACT_SILU).cpu(), ref) < 1e-6      # 16-bit inputs, float arithmetic and output


@gpu
@pytest.mark.parametrize("F_", [24, 100, 513])
def test_units_of_the_feed_forwards(F_):
    from jacobiforcing_amd import layer_ops as LO
    g = torch.Generator().manual_seed(F_)
    z = torch.randn(7, 2 * F_ + 3, generator=g) * 3
    zd = z.double()
    assert rel_err(LO.gated_act(z.cuda(), 1, -1, F_, LO.ACT_GELU_ERF).cpu(), O.gelu_erf(zd[:, 1:F_ + 1])) < 1e-6
    assert rel_err(LO.gated_act(z.cuda(), 0, F_, F_, LO.ACT_SILU).cpu(), O.silu(zd[:, :F_]) * zd[:, F_:2 * F_]) < 1e-6
    assert rel_err(LO.gated_act(z.cuda(), F_ + 1, 1, F_, LO.ACT_SILU).cpu(), O.silu(zd[:, F_ + 1:2 * F_ + 1]) * zd[:, 1:F_ + 1]) < 1e-6
    zb = z.cuda().bfloat16()
    assert rel_err(LO.gated_act(zb, 0, -1, F_, LO.ACT_GELU_ERF).float().cpu(), O.gelu_erf(zb.cpu().double()[:, :F_])) < 6e-3
    cap = LO.softcap((z * 4).cuda().contiguous(), 7.5).cpu()
    assert rel_err(cap, 7.5 * torch.tanh(zd * 4 / 7.5)) < 1e-6 and float(cap.abs().max()) <= 7.5


@gpu
@pytest.mark.parametrize("E,top,ff,W", [(5, 2, 24, 96), (3, 1, 20, 64), (4, 4, 33, 50), (16, 3, 64, 128)])
def test_router_and_experts_alone(E, top, ff, W, monkeypatch):
    from jacobiforcing_amd import layer_ops as LO
    cfg = make_cfg([dict(attn(), mlp=moe(experts=E, top=top, ff=ff))], width=W)
    t = tensors_for(cfg, E)
    P = layer_tensors(t, 0)
    h = torch.randn(70, W, generator=torch.Generator().manual_seed(2))
    h[3] = h[2]                                                                                 # equal rows choose equal experts
    f = cfg["layers"][0]["mlp"]
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        w = MK.MikipelWeights(MK.MikipelConfig.from_dict(cfg), t, "cuda", dtype).layers[0]
        hd = h.cuda().to(dtype)
        ref = O.feed_forward(hd.cpu().double(), P, f)
        for unfused in ("", "1"):                         # the unit in the up product's epilogue, and as a launch of its own
            monkeypatch.setenv("JL_MOE_UNFUSED_ACT", unfused)
            logits = torch.addmm(w["router_b"], hd.float(), w["router"].t())
            y = LO.moe_experts(hd, logits, None, top, 1.0, w["w_gu"], w["w_down"], route="top_softmax", gated=(LO.ACT_SILU, 0.0, 1.0, 0.0))
            assert tuple(y.shape) == (70, top, W) and y.dtype == torch.float32
            assert rows_off(y.sum(1).cpu(), ref, tol) <= (0.0 if dtype == torch.float32 else 0.05), (dtype, unfused)
        monkeypatch.delenv("JL_MOE_UNFUSED_ACT")
    # ties go to the lower index; the weights are the softmax over the chosen logits alone (a large logit left out changes nothing)
    from jacobiforcing_amd import _native as N
    z = torch.zeros(3, E)
    z[1, E - 1] = 1.0
    z[2] = torch.arange(E, dtype=torch.float32) * 0.7
    zc, ids, wts = z.cuda(), torch.empty((3, top), dtype=torch.int32, device="cuda"), torch.empty((3, top), device="cuda")
    N.check_layers(N.layers().jl_moe_route(zc.data_ptr(), None, 3, E, top, 1.0, ids.data_ptr(), wts.data_ptr(), N.JL_ROUTE_TOP_SOFTMAX, 0.0,
                                          torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert ids[0].tolist() == list(range(top)) and ids[1].tolist() == ([E - 1] + list(range(top - 1)))[:top]
    assert ids[2].tolist() == list(range(E - 1, E - 1 - top, -1))
    assert torch.allclose(wts.sum(1).cpu(), torch.ones(3), atol=1e-6)
    assert torch.allclose(wts[2].cpu(), torch.softmax(z[2, E - top:].flip(0), 0), atol=1e-6)


MIXER_SIZES = [attn(4, 2, 32, 64, 16), attn(8, 8, 64, 32, 64, factor=0.0), attn(3, 1, 24, 40, 12), attn(2, 1, 128, 128, 32, base=1e6), attn(12, 4, 16, 16, 8),
               attn(40, 1, 16, 32, 0), attn(1, 1, 20, 10, 6), attn(6, 3, 48, 20, 48),
               latent(3, 16, 8, 24, 40, 8), latent(8, 32, 32, 32, 64, 32), latent(1, 20, 6, 10, 33, 4, factor=2.0), latent(16, 64, 16, 64, 128, 16), latent(5, 8, 10, 8, 200, 0),
               latent(8, 64, 64, 128, 512, 24),
               delta(4, 2, 24, 20, 3), delta(2, 2, 40, 72, 1), delta(3, 1, 16, 8, 5), delta(4, 2, 64, 64, 4), delta(8, 8, 128, 128, 2), delta(1, 1, 200, 300, 4),
               delta(6, 2, 8, 260, 3)]


@gpu
@pytest.mark.parametrize("layer", MIXER_SIZES, ids=lambda L: L["type"][0] + "-".join(str(v) for v in L["mixer"].values() if not isinstance(v, (dict, float))))
def test_each_mixer_alone_in_portions_and_single_tokens(layer):
    """One mixer on the oracle's own inputs, float32 and bfloat16: a prompt's first part in one step, a second part that starts inside a
    page and inside a group of the recurrence, two tokens, then single tokens, then a long portion (the recurrence's form with the state's
    columns shared out), on shuffled pages and a poisoned slot."""
    W, T = 64, 84
    cfg = make_cfg([dict(layer, mlp=None)], width=W, vocab=40)
    t = tensors_for(cfg, 5)
    P = layer_tensors(t, 0)
    h = torch.randn(T, W, generator=torch.Generator().manual_seed(7))
    kind = layer["type"]
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
        rig = Rig(cfg, tensors=t, dtype=dtype, pages=16)
        rig.poison()
        hd = h.cuda().to(dtype)
        want = O.MIXERS[kind](hd.cpu().double(), P, layer["mixer"], 1e-5)
        run = {"attention": rig.model._attention, "latent_attention": rig.model._latent_attention, "delta": rig.model._delta}[kind]
        got, at = [], 0
        for n in (19, 14, 2, 1, 1, 1, 5, 41):
            b, _ = rig.batch([("r", [0] * n)])
            got.append(torch.nn.functional.linear(run(0, hd[at:at + n].contiguous(), b, rig.cache), rig.model.w.layers[0]["w_o"]).float().cpu())
            at += n
        assert rel_err(torch.cat(got), want) < tol, dtype


@gpu
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_prompt_and_every_layer(name):
    rig = Rig(SHAPES[name](), seed=3)
    t = toks(37, rig.cfg.vocab_size, 1)
    tr_o, tr_g = [], []
    want = rig.oracle(t, tr_o)
    got = rig.step([("r", t)], tr_g)
    assert len(tr_g) == len(tr_o) == rig.cfg.num_hidden_layers
    for li, (g_, o_) in enumerate(zip(tr_g, tr_o)):
        assert rel_err(g_.cpu(), o_) < F32_TOL, li
    assert rel_err(got, want) < F32_TOL
    rig.end("r")
    assert rel_err(rig.step([("again", t)]), want) < F32_TOL                                    # without the trace: the sums folded into the norms' launch
    if rig.cfg.logit_softcap:
        assert float(got.abs().max()) <= rig.cfg.logit_softcap


@gpu
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_prefill_equals_token_by_token_decoding(name):
    rig = Rig(SHAPES[name](), seed=5)
    rig.poison()
    t = toks(29, rig.cfg.vocab_size, 2)
    want = rig.oracle(t)
    got = torch.cat([rig.step([("r", [x])]) for x in t])
    assert rel_err(got, want) < F32_TOL
    assert rel_err(rig.step([("p", t)]), want) < F32_TOL


@gpu
@pytest.mark.parametrize("cuts", [[2] * 20, [1, 2, 3, 5, 8, 13, 7, 1], [7, 9, 8, 16], [39, 1], [3, 37], [8, 8, 8, 8, 8], [15, 17, 1, 7]])
def test_portions_of_any_size(cuts):
    """Portions down to two tokens, at and beside the edges of pages (8), of the recurrence's groups and of the convolution's runs (8)."""
    for name in ("a", "b"):
        rig = Rig(SHAPES[name](), seed=7)
        rig.poison()
        t = toks(sum(cuts), rig.cfg.vocab_size, 3)
        got, at = [], 0
        for n in cuts:
            got.append(rig.step([("r", t[at:at + n])]))
            at += n
        assert rel_err(torch.cat(got), rig.oracle(t)) < F32_TOL, name


@gpu
def test_unequal_requests_in_one_batch_equal_each_alone():
    for name in ("a", "b", "c"):
        rig = Rig(SHAPES[name](), seed=11, pages=96)
        V = rig.cfg.vocab_size
        seqs = {"x": toks(41, V, 4), "y": toks(3, V, 5), "z": toks(18, V, 6), "w": toks(70, V, 7)}
        plan = [[("x", 17), ("y", 1), ("w", 33)], [("x", 1), ("y", 2), ("z", 18), ("w", 1)], [("x", 23), ("w", 36)]]
        at, got = {k: 0 for k in seqs}, {k: [] for k in seqs}
        for step in plan:
            out = rig.step([(k, seqs[k][at[k]:at[k] + n]) for k, n in step])
            r0 = 0
            for k, n in step:
                got[k].append(out[r0:r0 + n]); r0 += n; at[k] += n
        for k, s in seqs.items():
            assert at[k] == len(s) and rel_err(torch.cat(got[k]), rig.oracle(s)) < F32_TOL, (name, k)


@gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32_TOL), (torch.bfloat16, BF16_TOL)])
def test_freed_pages_and_slots_are_used_again(dtype, tol):
    """Two slots, a pool that holds two requests: requests end, their pages and slots go to new ones; old keys, states, convolution
    inputs and shifted rows must not leak."""
    rig = Rig(shape_a(), seed=17, pages=12, slots=2, dtype=dtype)
    V = rig.cfg.vocab_size
    rig.poison()
    for rnd in range(4):
        a, b = toks(40 + rnd, V, 20 + rnd), toks(17 + 3 * rnd, V, 30 + rnd)
        ga = rig.step([("a", a[:25]), ("b", b[:1])])                                           # b starts with a single token in a used slot
        gb = rig.step([("a", a[25:]), ("b", b[1:])])
        got_a = torch.cat([ga[:25], gb[:len(a) - 25]])
        got_b = torch.cat([ga[25:], gb[len(a) - 25:]])
        if dtype == torch.float32:
            assert rel_err(got_a, rig.oracle(a)) < tol and rel_err(got_b, rig.oracle(b)) < tol, rnd
        else:
            assert rows_off(got_a, rig.oracle(a), tol) <= 0.1 and rows_off(got_b, rig.oracle(b), tol) <= 0.1, rnd
        used = set(rig.req["a"]["pages"]) | set(rig.req["b"]["pages"])
        rig.end("b"); rig.end("a")
        assert len(rig.free_pages) == 12 and len(used) >= 8


def peaked_model(kind):
    """One attention layer of either kind, no feed-forward, no shift, a sharp softmax, a rotation over a small part of the head; the
    layer's own result goes on alone.  Returns (cfg, tensors, hot query token, hot key token, scores): the pair of tokens whose unrotated
    score is the largest."""
    V = 40
    layer = attn(heads=2, kv=1, dim=16, vdim=16, dims=4, base=10000.0, scale=2.5, factor=0.0) if kind == "attention" else \
        latent(heads=2, dim=16, rot_dim=4, vdim=16, rank=32, dims=4, base=10000.0, scale=2.5)
    cfg = make_cfg([dict(layer, mlp=None)], width=32, vocab=V, emb=1.0, mult=1.0, cap=0.0)
    t = tensors_for(cfg, 23)
    t["l0.shift"] = torch.zeros(32)
    t["l0.dwa"] = torch.tensor([0.0, 1.0])
    eps = cfg["norm"]["eps"]
    h = O.rms_norm(t["embed"].double(), t["l0.norm1"].double(), eps)
    if kind == "attention":
        q = O.rms_norm((h @ t["l0.mix.q"].double().T).view(V, 2, 16), None, eps)[:, 0]
        k = O.rms_norm((h @ t["l0.mix.k"].double().T).view(V, 1, 16), None, eps)[:, 0]
        s = q[:, 4:] @ k[:, 4:].T
    else:
        q = (h @ t["l0.mix.q"].double().T).view(V, 2, 20)[:, 0, :16]
        c = O.rms_norm((h @ t["l0.mix.dkv"].double().T)[:, :32], t["l0.mix.dkv.norm"].double(), eps)
        s = q @ (c @ t["l0.mix.uk"].double().T).view(V, 2, 16)[:, 0].T
    qi, kj = divmod(int(s.argmax()), V)
    return cfg, t, qi, kj, s


@gpu
@pytest.mark.parametrize("kind", ["attention", "latent_attention"])
@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32_TOL), (torch.bfloat16, BF16_TOL)])
@pytest.mark.parametrize("place", [16, 23, 24, 0])
def test_a_far_key_among_hundreds(kind, dtype, tol, place):
    """Plain causal attention over many pages: the hot key sits up to 300 tokens back — at a page's first place, at its last place, at
    the next page's first, and at position 0 — and is read by a prompt's portion and by a single decoded token."""
    cfg, t, qi, kj, s = peaked_model(kind)
    dull = [x for x in np.argsort(s[qi].numpy())[:12].tolist() if x != kj]
    T = 300
    seq = [dull[i % len(dull)] for i in range(T)]
    seq[place], seq[T - 1], seq[T - 9] = kj, qi, qi
    rig = Rig(cfg, tensors=t, pages=64, dtype=dtype)
    got = rig.step([("r", seq[:121])])
    got = torch.cat([got, rig.step([("r", seq[121:T - 2])]), rig.step([("r", seq[T - 2:T - 1])]), rig.step([("r", seq[T - 1:])])])
    want = rig.oracle(seq)
    assert rel_err(got[-1], want[-1]) < tol and rel_err(got[T - 9], want[T - 9]) < tol and rel_err(got, want) < tol
    seq2 = list(seq)
    seq2[place] = dull[0]
    other = rig.oracle(seq2)
    assert rel_err(other[-1], want[-1]) > 0.05 and rel_err(other[T - 9], want[T - 9]) > 0.05     # the test would see the key missing


@gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32_TOL), (torch.bfloat16, BF16_TOL)])
def test_an_old_write_stays_in_the_recurrent_state(dtype, tol):
    """A delta layer that hardly decays: what token 3 wrote is still read 250 tokens later, through portions, a used slot and decoding."""
    cfg = make_cfg([dict(delta(heads=2, kv=1, dim=16, vdim=16, conv=2), mlp=None)], width=32, vocab=40, emb=1.0, mult=4.0, cap=0.0)
    t = tensors_for(cfg, 41)
    t["l0.mix.A_log"] = torch.full((2,), -9.0)
    t["l0.dwa"] = torch.tensor([0.0, 1.0])
    T = 256
    seq = toks(T, 40, 9)
    seq = [x % 4 for x in seq]                                                                  # few distinct keys: the state is written along them again and again
    seq[3] = 39
    rig = Rig(cfg, tensors=t, pages=48, dtype=dtype)
    rig.step([("old", toks(20, 40, 1))])
    rig.end("old")
    got = torch.cat([rig.step([("r", seq[:5])]), rig.step([("r", seq[5:130])]), rig.step([("r", seq[130:T - 3])])] + [rig.step([("r", [x])]) for x in seq[T - 3:]])
    want = rig.oracle(seq)
    assert rel_err(got, want) < tol and rel_err(got[-1], want[-1]) < tol
    seq2 = list(seq)
    seq2[3] = 0
    assert rel_err(rig.oracle(seq2)[-1], want[-1]) > 0.2
    t2 = dict(t)
    t2["l0.mix.A_log"] = torch.full((2,), 1.0)                                                  # with a fast decay the old write is gone: the test rests on the state
    assert rel_err(O.forward(cfg, t2, seq2, torch.float64)[-1], O.forward(cfg, t2, seq, torch.float64)[-1]) < 1e-6


@gpu
def test_the_first_tokens_of_a_sequence():
    """One, two and three tokens in a slot and on pages that hold another request's keys, state, convolution inputs and shifted row."""
    for name in ("a", "b"):
        rig = Rig(SHAPES[name](), seed=19, slots=1, pages=16)
        V = rig.cfg.vocab_size
        rig.step([("old", toks(30, V, 1))])
        rig.end("old")
        for n in (1, 2, 3):
            t = toks(n + 1, V, 50 + n)
            got = torch.cat([rig.step([("new", t[:n])]), rig.step([("new", t[n:])])])
            assert rel_err(got, rig.oracle(t)) < F32_TOL, (name, n)
            rig.end("new")


@gpu
def test_long_decoding():
    rig = Rig(shape_b(), seed=29, pages=64)
    t = toks(200, rig.cfg.vocab_size, 8)
    want = rig.oracle(t)
    got = [rig.step([("r", t[:40])])] + [rig.step([("r", [x])]) for x in t[40:]]
    assert rel_err(torch.cat(got), want) < F32_TOL and rel_err(got[-1], want[-1:]) < F32_TOL


def random_cfg(r):
    def rot(limit):
        if r.random() < 0.15:
            return 0, 0.0
        return r.choice([d for d in (2, 4, 6, 8, 12, 16, 24, 32) if d <= limit]), r.choice([0.0, 2.0, 8.0])
    layers = []
    for _ in range(r.choice([1, 2, 3, 4])):
        kind = r.choice(["attention", "latent_attention", "delta"])
        if kind == "attention":
            kv, D = r.choice([1, 2, 3]), r.choice([8, 16, 24, 32, 64])
            dims, factor = rot(D)
            L = attn(kv * r.choice([1, 2, 4]), kv, D, r.choice([D, 16, 32, 40]), dims, r.choice([50.0, 1e4, 1e6]), r.choice([D ** -0.5, 0.2]), factor)
        elif kind == "latent_attention":
            D, rd = r.choice([8, 16, 32]), r.choice([4, 8, 16, 32])
            dims, factor = rot(rd)
            L = latent(r.choice([1, 2, 4, 6]), D, rd, r.choice([D, 16, 24]), r.choice([16, 32, 40, 64, 96]), dims, r.choice([50.0, 1e4]), r.choice([(D + rd) ** -0.5, 0.2]), factor)
        else:
            kv = r.choice([1, 2, 3])
            L = delta(kv * r.choice([1, 2, 3]), kv, r.choice([8, 16, 24, 64]), r.choice([8, 16, 40, 64, 130]), r.choice([1, 2, 3, 4, 5]))
        k = r.random()
        E = r.choice([2, 4, 7])
        L["mlp"] = None if k < 0.2 else dense(r.choice([24, 56, 100])) if k < 0.55 else moe(E, r.choice([1, 2, E]), r.choice([16, 24, 40]))
        layers.append(L)
    return make_cfg(layers, width=r.choice([32, 48, 64, 100]), vocab=r.choice([30, 77, 131]), eps=r.choice([1e-5, 1e-6]), emb=r.choice([1.0, 3.0, 8.0]),
                    mult=r.choice([0.25, 0.5, 1.0]), cap=r.choice([0.0, 6.0, 30.0]))


@gpu
@pytest.mark.parametrize("seed", range(12))
def test_random_configurations_in_a_mixed_schedule(seed):
    """Random layer orders, head counts, sizes, taps and constants; two requests of unequal length in a random schedule of portions and
    single tokens, float32 and bfloat16."""
    r = random.Random(1000 + seed)
    cfg = random_cfg(r)
    t = tensors_for(cfg, seed)
    V = cfg["vocab"]
    seqs = {"x": toks(r.choice([9, 31, 60]), V, seed), "y": toks(r.choice([2, 17, 45]), V, seed + 100)}
    plan, at = [], {k: 0 for k in seqs}
    while any(at[k] < len(s) for k, s in seqs.items()):
        step = []
        for k, s in seqs.items():
            if at[k] < len(s) and r.random() < 0.8:
                n = min(len(s) - at[k], r.choice([1, 1, 2, 3, 7, 8, 9, 20, 40]))
                step.append((k, at[k], n)); at[k] += n
        if step:
            plan.append(step)
    want = {k: O.forward(cfg, t, s, torch.float64) for k, s in seqs.items()}
    for dtype in (torch.float32, torch.bfloat16):
        rig = Rig(cfg, tensors=t, dtype=dtype, pages=32, seed=seed)
        rig.poison()
        got = {k: [] for k in seqs}
        for step in plan:
            out = rig.step([(k, seqs[k][a:a + n]) for k, a, n in step])
            r0 = 0
            for k, a, n in step:
                got[k].append(out[r0:r0 + n]); r0 += n
        for k in seqs:
            if dtype == torch.float32:
                assert rel_err(torch.cat(got[k]), want[k]) < F32_TOL, (cfg, k)
            else:
                assert rows_off(torch.cat(got[k]), want[k], 0.1) <= 0.25, (cfg, k)


def _write_model(tmp_path, cfg_dict, tensors):
    from safetensors.torch import save_file
    (tmp_path / "config.json").write_text(json.dumps(cfg_dict))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()}, str(tmp_path / "model.safetensors"))
    return str(tmp_path)


def _oracle_greedy(cfg_dict, tensors, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(O.forward(cfg_dict, tensors, seq, torch.float64)[-1].argmax()))
    return seq[len(prompt):]


@gpu
def test_greedy_generation_through_the_engine_and_its_scheduler(tmp_path):
    """LLM.generate on a checkpoint directory: registry -> loader -> scheduler (prompts cut to the token budget, admissions limited by
    two slots, pages reused) -> ragged step -> argmax.  float32 so that the greedy choice is the oracle's."""
    from jacobiforcing_amd import LLM, SamplingParams
    cfg_dict = shape_a()
    tensors = tensors_for(cfg_dict, 31)
    path = _write_model(tmp_path, cfg_dict, tensors)
    V = cfg_dict["vocab"]
    prompts = [toks(n, V, 40 + n) for n in (70, 5, 33, 1)]
    llm = LLM(path, tokenizer_path="none", dtype="float32", kvcache_block_size=64, num_kvcache_blocks=4, max_num_seqs=2, max_model_len=128,
              max_num_batched_tokens=128, device="cuda")
    out = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=6, ignore_eos=True), use_tqdm=False)
    for p, o in zip(prompts, out):
        assert o["token_ids"] == _oracle_greedy(cfg_dict, tensors, p, 6)
    assert len(llm.scheduler.block_manager.free_block_ids) == 4 and len(llm.model_runner.free_rows) == 2
    # the same engine replays a given schedule: portions beside single tokens, requests that end, logits where asked
    a, b = prompts[0], prompts[2]
    l1 = llm.replay_step([("a", a[:40], [0, 39]), ("b", b[:2], [])])
    l2 = llm.replay_step([("a", a[40:], [29]), ("b", b[2:], [len(b) - 3])], end=["a"])
    l3 = llm.replay_step([("c", a, [len(a) - 1])], end=["b", "c"])
    wa, wb = O.forward(cfg_dict, tensors, a, torch.float64), O.forward(cfg_dict, tensors, b, torch.float64)
    assert tuple(l1.shape) == (2, V) and rel_err(l1.cpu(), wa[[0, 39]]) < F32_TOL
    assert rel_err(l2.cpu(), torch.stack([wa[69], wb[len(b) - 1]])) < F32_TOL and rel_err(l3.cpu(), wa[-1:]) < F32_TOL
    assert len(llm.scheduler.block_manager.free_block_ids) == 4 and len(llm.model_runner.free_rows) == 2


@gpu
def test_a_preempted_request_starts_again_from_an_empty_state(tmp_path):
    """Three pages for two requests that need five: the newer one is preempted while it decodes, gives pages and slot back and is
    prefilled again later — its recurrent state, convolution inputs and shifted rows start from nothing, the results are the oracle's."""
    from jacobiforcing_amd import LLM, SamplingParams
    cfg_dict = shape_a()
    tensors = tensors_for(cfg_dict, 43)
    path = _write_model(tmp_path, cfg_dict, tensors)
    V = cfg_dict["vocab"]
    prompts = [toks(100, V, 61), toks(60, V, 62)]
    llm = LLM(path, tokenizer_path="none", dtype="float32", kvcache_block_size=64, num_kvcache_blocks=3, max_num_seqs=2, max_model_len=192,
              max_num_batched_tokens=192, device="cuda")
    preempted = []
    keep = llm.scheduler.preempt
    llm.scheduler.preempt = lambda seq: (preempted.append(seq.seq_id), keep(seq))[1]
    out = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=30, ignore_eos=True), use_tqdm=False)
    assert preempted, "the pool was meant to run out"
    for p, o in zip(prompts, out):
        assert o["token_ids"] == _oracle_greedy(cfg_dict, tensors, p, 30)
    assert len(llm.scheduler.block_manager.free_block_ids) == 3 and len(llm.model_runner.free_rows) == 2


@gpu
def test_sampling_through_the_engine_follows_the_distribution(tmp_path):
    from jacobiforcing_amd import LLM, SamplingParams
    cfg_dict = shape_b()
    tensors = tensors_for(cfg_dict, 37)
    path = _write_model(tmp_path, cfg_dict, tensors)
    prompt = toks(9, cfg_dict["vocab"], 50)
    llm = LLM(path, tokenizer_path="none", dtype="float32", kvcache_block_size=64, num_kvcache_blocks=16, max_num_seqs=16, max_model_len=64,
              max_num_batched_tokens=64, device="cuda")
    torch.manual_seed(0)
    out = llm.generate([prompt] * 800, SamplingParams(temperature=1.0, max_tokens=1, ignore_eos=True), use_tqdm=False)
    p = torch.softmax(O.forward(cfg_dict, tensors, prompt, torch.float64)[-1], 0).numpy()
    counts = np.bincount([o["token_ids"][0] for o in out], minlength=len(p)) / 800.0
    assert 0.5 * np.abs(counts - p).sum() < 0.2                                                 # total variation of 800 draws over 77 ids
