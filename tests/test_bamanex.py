"""Bamanex through the package (HIP layer kernels, paged pools with one pool per layer run, ragged step, scheduler, LLM.generate)
against the plain oracle ``oracle/bamanex_oracle.py``, which shares no code with it.  Small random models of several shapes; where
random weights would hide a fault (a key at a window's edge, a far key among hundreds, a sink that is left out) the inputs are
chosen so that one score stands out.

CPU tests cover the oracle's own pieces, the config reader, the frequency table and the cache layout; everything that launches a
kernel is marked ``gpu``."""
import json
import math
import random

import numpy as np
import pytest
import torch

from oracle import bamanex_oracle as O
from jacobiforcing_amd.modeling import MODEL_REGISTRY, read_model_config
from jacobiforcing_amd.modeling import bamanex as BX

gpu = pytest.mark.gpu

STRETCH = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}


# ---- model shapes -----------------------------------------------------------------------------------------------------------------
def attn(heads=6, kv=2, dim=24, vdim=40, size=11, dims=16, base=500.0, scale=0.3, scaling=STRETCH):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if size:
        m["mask"] = {"size": size}
    if dims:
        m["rot"] = {"dims": dims, "base": base}
        if scaling:
            m["rot"]["scaling"] = dict(scaling)
    return {"type": "attention", "mixer": m}


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=24, limit=1.5, shared_ff=40, shared_limit=0.75):
    f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared_ff:
        f["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return f


def make_cfg(layers, width=96, vocab=131, eps=1e-5, loop=None, logit_scale=1.5):
    d = {"architecture": "Bamanex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers, "logit_scale": logit_scale}
    if loop:
        d["loop"] = dict(zip(("start", "stop", "times"), loop))
    return d


def shape_a():
    """Dense and expert feed-forwards, a layer without one, grouped key/value heads, a looped span of two layers run three times,
    different head sizes for keys and values, different limits and widths for routed and shared experts."""
    return make_cfg([dict(attn(), mlp=dense()), dict(attn(heads=4, kv=4, dim=16, vdim=16, size=7, dims=8), mlp=moe()),
                     dict(attn(heads=3, kv=1, dim=32, vdim=24, size=19, dims=32, scaling=None), mlp=None), dict(attn(size=5), mlp=moe(shared_ff=0, top=3))],
                    loop=(1, 3, 3))


def shape_b():
    """One head; one expert chosen; all experts chosen; a window of one token and none at all; no rotation; sizes that are no
    multiples of eight; nothing looped."""
    return make_cfg([dict(attn(heads=1, kv=1, dim=20, vdim=72, size=1, dims=12, base=10000.0), mlp=moe(experts=3, top=1, ff=20, shared_ff=12)),
                     dict(attn(heads=5, kv=5, dim=12, vdim=20, size=0, dims=0), mlp=moe(experts=4, top=4, ff=33, limit=0.5, shared_ff=33, shared_limit=2.5)),
                     dict(attn(heads=2, kv=1, dim=40, vdim=8, size=64, dims=40, base=50.0), mlp=dense(24))],
                    width=64, vocab=77, eps=1e-6, logit_scale=0.5)


def shape_c():
    """Many heads over few key/value heads, windows longer than any test sequence, the whole model inside the loop."""
    return make_cfg([dict(attn(heads=20, kv=5, dim=16, vdim=32, size=4096, dims=16), mlp=dense(48)),
                     dict(attn(heads=8, kv=2, dim=64, vdim=64, size=33, dims=32, base=1e6), mlp=moe(experts=9, top=2, ff=16, shared_ff=16))],
                    width=80, vocab=50, loop=(0, 2, 2), logit_scale=1.0)


SHAPES = {"a": shape_a, "b": shape_b, "c": shape_c}


def tensors_for(cfg_dict, seed):
    return BX.random_tensors(BX.BamanexConfig.from_dict(cfg_dict), seed)


def rel_err(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.sqrt(((got - want) ** 2).mean()) / max(np.sqrt((want ** 2).mean()), 1e-30))


F32_TOL, BF16_TOL = 2e-4, 6e-2


def rows_off(got, want, tol):
    """Fraction of rows (positions) whose own relative error is above ``tol``.  In bfloat16 a router's close call may go the other
    way for a token or two — such a token's row is simply another expert's, by much more than rounding — so a test over random
    routers bounds how many rows differ instead of their common error."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    err = np.sqrt(((got - want) ** 2).mean(-1)) / np.maximum(np.sqrt((want ** 2).mean(-1)), 1e-30)
    return float((err > tol).mean())


def toks(n, vocab, seed):
    return [random.Random(seed * 7919 + i).randrange(vocab) for i in range(n)]


# =====================================================================================================================================
# CPU: oracle pieces, config reader, frequency table, cache layout
# =====================================================================================================================================
def test_registry_reads_the_architecture_key(tmp_path):
    assert MODEL_REGISTRY["Bamanex"][2] == "ragged"
    (tmp_path / "config.json").write_text(json.dumps(shape_a()))
    cfg = read_model_config(tmp_path)
    assert isinstance(cfg, BX.BamanexConfig) and cfg.family == "ragged" and cfg.num_hidden_layers == 4 and cfg.logit_scale == 1.5
    assert cfg.runs() == [0, 1, 2, 1, 2, 1, 2, 3] == O.layer_order(shape_a())
    assert BX.BamanexConfig.from_dict(shape_b()).runs() == [0, 1, 2] and BX.BamanexConfig.from_dict(shape_c()).runs() == [0, 1, 0, 1]


def test_config_rejects_what_the_design_does_not_have():
    for change in (lambda c: c["layers"][0].update(type="retention"), lambda c: c["layers"][0]["mlp"].update(kind="polynomial"),
                   lambda c: c["layers"][0]["mixer"].update(kv_heads=4), lambda c: c["layers"][0]["mixer"]["rot"].update(dims=26),
                   lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), lambda c: c.update(loop={"start": 2, "stop": 9, "times": 2}),
                   lambda c: c["layers"][1]["mlp"]["router"].update(top=6)):
        bad = shape_a()
        change(bad)
        with pytest.raises(ValueError):
            BX.BamanexConfig.from_dict(bad)


def test_one_pool_per_layer_run_and_stacked_weights():
    cfg = BX.BamanexConfig.from_dict(shape_a())
    w = BX.BamanexWeights(cfg, tensors_for(shape_a(), 1), "cpu", torch.float32)
    specs = BX.BamanexModel(cfg, w, max_positions=16).cache_specs()
    assert len(specs) == 8 and [(s.k_width, s.v_width) for s in specs[:3]] == [(48, 80), (64, 64), (32, 24)] and specs[3].k_width == 64
    l0, l1, l3 = w.layers[0], w.layers[1], w.layers[3]
    # q, k, v and the six head gates, then zero rows up to a multiple of eight (the gates and the padding have no bias)
    assert tuple(l0["w_in"].shape) == (6 * 24 + 2 * 24 + 2 * 40 + 6 + 2, 96) and l0["cols"] == (0, 144, 192, 272) and float(l0["b_in"][-8:].abs().sum()) == 0
    assert float(l0["w_in"][-2:].abs().sum()) == 0 and float(l0["w_in"][-8:-2].abs().sum()) > 0
    assert tuple(l0["w_gu"].shape) == (112, 96) and tuple(l1["w_gu"].shape) == (5, 48, 96) and tuple(l1["w_sh"].shape) == (88, 96)
    assert "w_sh" not in l3 and "norm2" not in w.layers[2] and l0["norm1"].dtype == torch.float32 and l1["router"].dtype == torch.float32


def test_frequency_table_keeps_divides_and_blends():
    dims, base = 16, 500.0
    plain = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    got, want = BX.rotary_frequencies(dims, base, STRETCH), O.stretched_frequencies(dims, base, STRETCH)
    assert np.allclose(got, want, rtol=1e-12) and BX.rotary_frequencies(dims, base, None) == plain
    ratio = [g / p for g, p in zip(got, plain)]
    assert ratio[0] == 1.0 and ratio[1] == 1.0 and ratio[-1] == 1 / 8.0 and 1 / 8.0 < ratio[2] < 1.0      # all three branches occur
    # at the two edges the blend meets the kept and the divided frequency
    edge = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 2 * math.pi * 4}
    assert abs(BX.rotary_frequencies(2, 1.0, edge)[0] - 1.0) < 1e-12 and abs(O.stretched_frequencies(2, 1.0, edge)[0] - 1.0) < 1e-12


def test_oracle_pieces():
    g = torch.Generator().manual_seed(0)
    s = torch.randn(9, generator=g, dtype=torch.float64)
    w = O.sink_softmax(s, torch.tensor(0.3, dtype=torch.float64))
    assert abs(float(w.sum()) - float(torch.exp(s).sum() / (torch.exp(s).sum() + math.exp(0.3)))) < 1e-12
    assert abs(float(O.sink_softmax(s, torch.tensor(-80.0, dtype=torch.float64)).sum()) - 1.0) < 1e-12
    v = torch.randn(3, 10, generator=g, dtype=torch.float64)
    r = O.rotate_pairs(v, 17, [0.5, 0.01, 0.2])
    assert torch.allclose((r * r).sum(-1), (v * v).sum(-1)) and torch.equal(r[:, 6:], v[:, 6:]) and not torch.allclose(r[:, :6], v[:, :6])
    assert torch.equal(O.rotate_pairs(v, 0, [0.5, 0.01, 0.2]), v)
    z = torch.tensor([-3.0, 0.0, 2.0], dtype=torch.float64)
    assert torch.allclose(O.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    x = torch.randn(4, 12, generator=g, dtype=torch.float64)
    assert torch.allclose(O.centred_norm(x, torch.zeros(12, dtype=torch.float64), 0.0).pow(2).mean(-1), torch.ones(4, dtype=torch.float64))
    P = {"mlp.router": torch.randn(6, 12, generator=g, dtype=torch.float64)}
    ids, wt = O.route(x, P, {"router": {"experts": 6, "top": 3}})
    full = torch.softmax(x @ P["mlp.router"].T, -1)
    assert torch.allclose(wt.sum(-1).double(), torch.ones(4, dtype=torch.float64), atol=1e-6)
    assert all(set(ids[t].tolist()) == set(torch.topk(full[t], 3).indices.tolist()) for t in range(4))
    hi = torch.full((1, 12), 5.0, dtype=torch.float64)
    unit = {"u.gate": torch.eye(12, dtype=torch.float64), "u.up": -torch.eye(12, dtype=torch.float64), "u.down": torch.eye(12, dtype=torch.float64)}
    assert torch.allclose(O.clamped_unit(hi, unit, "u.", 2.0), torch.full((1, 12), 2.0 * torch.sigmoid(torch.tensor(3.404)).item() * (-2.0 + 1.0), dtype=torch.float64))


# =====================================================================================================================================
# GPU: the package against the oracle
# =====================================================================================================================================
class Rig:
    """A model on the GPU with a pool of shuffled pages; runs steps of (request, tokens) and keeps the bookkeeping a test needs."""

    def __init__(self, cfg_dict, seed=0, dtype=torch.float32, page=8, pages=64, slots=4, tensors=None, max_positions=1024):
        from jacobiforcing_amd import layer_ops as LO
        self.LO = LO
        self.cfg_dict = cfg_dict
        self.cfg = BX.BamanexConfig.from_dict(cfg_dict)
        self.tensors = tensors or tensors_for(cfg_dict, seed)
        self.model = BX.BamanexModel(self.cfg, BX.BamanexWeights(self.cfg, self.tensors, "cuda", dtype), max_positions=max_positions)
        self.page = page
        self.cache = self.model.new_cache(pages, page, slots)
        self.free_pages = list(range(pages))
        random.Random(seed).shuffle(self.free_pages)
        self.free_slots = list(range(slots))[::-1]
        self.req = {}

    def poison(self):
        """Fill the pools with large values: whatever a kernel reads without having written it shows."""
        for t in self.cache.k + self.cache.v:
            if t is not None:
                t.fill_(1e4)

    def step(self, entries, trace=None):
        """entries = [(key, tokens)]; returns logits [sum of tokens, vocab] (float, on the CPU)."""
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
        b = self.LO.RaggedBatch.build(counts, starts, slots, tables, self.page, "cuda")
        return self.model.forward(torch.tensor(ids, device="cuda"), b, self.cache, None, trace).cpu()

    def end(self, key):
        r = self.req.pop(key)
        self.free_pages += r["pages"][::-1]
        self.free_slots.append(r["slot"])

    def oracle(self, tokens):
        return O.forward(self.cfg_dict, self.tensors, list(tokens), torch.float64)


@gpu
@pytest.mark.parametrize("W", [96, 200, 1000])
def test_scaled_residual_sum_and_the_two_norms(W):
    from jacobiforcing_amd import layer_ops as LO
    g = torch.Generator().manual_seed(W)
    rn = lambda *s: torch.randn(*s, generator=g)
    x, y1, y2, y3, s1, s2, w1, w2 = rn(5, W), rn(5, W) * 3, rn(5, 3, W), rn(5, W), rn(W), rn(W), rn(W) * 0.2, rn(W) * 0.2
    new = x.double() + y1.double() * s1.double() + (y2.double().sum(1) + y3.double()) * s2.double()
    xd = x.cuda()
    o1, o2 = LO.scaled_add_norms(xd, [(y1.cuda(), s1.cuda()), (y2.cuda(), s2.cuda()), (y3.cuda(), s2.cuda())], w1.cuda(), w2.cuda(), 1.0, 1e-5,
                                 torch.float32, two=True)
    assert rel_err(xd.cpu(), new) < 1e-6
    assert rel_err(o1.cpu(), O.centred_norm(new, w1.double(), 1e-5)) < 1e-6 and rel_err(o2.cpu(), O.centred_norm(new, w2.double(), 1e-5)) < 1e-6
    # bfloat16 addends and outputs around a float stream; an addend without a scale; no addend at all; the update alone
    xb = x.cuda()
    ob = LO.scaled_add_norms(xb, [(y1.cuda().bfloat16(), None)], w1.cuda(), None, 1.0, 1e-5, torch.bfloat16)
    newb = x.double() + y1.bfloat16().double()
    assert xb.dtype == torch.float32 and rel_err(xb.cpu(), newb) < 1e-6 and rel_err(ob.float().cpu(), O.centred_norm(newb, w1.double(), 1e-5)) < 6e-3
    assert rel_err(LO.scaled_add_norms(xb, [], w2.cuda(), None, 1.0, 1e-5, torch.float32).cpu(), O.centred_norm(newb, w2.double(), 1e-5)) < 1e-6
    # the second norm in both forms: rounded for the products, unrounded for a float router
    p1, p2, p2f = LO.scaled_add_norms(xb, [], w1.cuda(), w2.cuda(), 1.0, 1e-5, torch.bfloat16, two=True, second_float=True)
    assert p2.dtype == torch.bfloat16 and p2f.dtype == torch.float32 and rel_err(p2f.cpu(), O.centred_norm(newb, w2.double(), 1e-5)) < 1e-6
    assert torch.equal(p2.cpu(), p2f.cpu().bfloat16()) and rel_err(p1.float().cpu(), O.centred_norm(newb, w1.double(), 1e-5)) < 6e-3
    q1, q2, q2f = LO.scaled_add_norms(xb, [], w1.cuda(), w2.cuda(), 1.0, 1e-5, torch.float32, two=True, second_float=True)
    assert q2f is q2 and q2.dtype == torch.float32
    assert LO.scaled_add_norms(xb, [(y3.cuda(), s1.cuda())], None, None, 1.0, 1e-5, None) is None
    assert rel_err(xb.cpu(), newb + y3.double() * s1.double()) < 1e-6
    tiny = torch.full((1, W), 1e-4)                                                            # eps inside the root decides here
    assert rel_err(LO.scaled_add_norms(tiny.cuda(), [], w1.cuda(), None, 1.0, 1e-5, torch.float32).cpu(), O.centred_norm(tiny.double(), w1.double(), 1e-5)) < 1e-6


@gpu
@pytest.mark.parametrize("F_", [24, 100, 513])
def test_gated_activations(F_):
    from jacobiforcing_amd import layer_ops as LO
    g = torch.Generator().manual_seed(F_)
    z = torch.randn(7, 2 * F_ + 3, generator=g) * 3
    zd = z.double()
    want = O.gelu_tanh(zd[:, :F_]) * zd[:, F_:2 * F_]
    assert rel_err(LO.gated_act(z.cuda(), 0, F_, F_, LO.ACT_GELU_TANH).cpu(), want) < 1e-6
    assert rel_err(LO.gated_act(z.cuda().bfloat16(), 0, F_, F_, LO.ACT_GELU_TANH).float().cpu(), O.gelu_tanh(z.bfloat16().double()[:, :F_]) * z.bfloat16().double()[:, F_:2 * F_]) < 6e-3
    # the clamped unit on columns that start at odd places: linear branch at 1, gate at F_ + 1, the row gate in the last column.  The
    # oracle's unit reads one input for both branches: [u | g] with selector matrices as its weights
    eye, zero = torch.eye(F_, dtype=torch.float64), torch.zeros(F_, F_, dtype=torch.float64)
    P = {"u.up": torch.cat([eye, zero], 1), "u.gate": torch.cat([zero, eye], 1), "u.down": eye}
    for limit in (0.5, 2.0, 7.0):                         # clamps that bite often, sometimes, hardly ever
        want = O.clamped_unit(zd[:, 1:2 * F_ + 1], P, "u.", limit)
        got = LO.gated_act(z.cuda(), F_ + 1, 1, F_, LO.ACT_CLAMPED_SWISH, limit, 1.702, 1.0)
        assert rel_err(got.cpu(), want) < 1e-6
        got = LO.gated_act(z.cuda(), F_ + 1, 1, F_, LO.ACT_CLAMPED_SWISH, limit, 1.702, 1.0, row_gate=z.cuda()[:, 2 * F_ + 2])
        assert rel_err(got.cpu(), want * torch.sigmoid(zd[:, 2 * F_ + 2:2 * F_ + 3])) < 1e-6
    assert rel_err(O.clamped_unit(zd[:, 1:2 * F_ + 1], P, "u.", 0.5), O.clamped_unit(zd[:, 1:2 * F_ + 1], P, "u.", 2.0)) > 0.05


@gpu
@pytest.mark.parametrize("E,top,ff,W", [(5, 2, 24, 96), (3, 1, 20, 64), (4, 4, 33, 50), (16, 3, 64, 128)])
def test_softmax_router_and_clamped_experts_alone(E, top, ff, W, monkeypatch):
    from jacobiforcing_amd import layer_ops as LO
    cfg = make_cfg([dict(attn(), mlp=moe(experts=E, top=top, ff=ff, limit=1.25, shared_ff=0))], width=W)
    t = tensors_for(cfg, E)
    P = {k: v.double() for k, v in O.layer_tensors(t, 0).items()}
    h = torch.randn(70, W, generator=torch.Generator().manual_seed(2))
    h[3] = h[2]                                                                                 # equal rows choose equal experts
    f = cfg["layers"][0]["mlp"]
    want = O.expert_mixture(h.double(), P, f)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        w = BX.BamanexWeights(BX.BamanexConfig.from_dict(cfg), t, "cuda", dtype).layers[0]
        hd = h.cuda().to(dtype)
        ref = want if dtype == torch.float32 else O.expert_mixture(h.bfloat16().double(), P, f)
        for unfused in ("", "1"):                         # the unit in the up product's epilogue, and as a launch of its own
            monkeypatch.setenv("JL_MOE_UNFUSED_ACT", unfused)
            y = LO.moe_experts(hd, torch.nn.functional.linear(hd.float(), w["router"]), None, top, 1.0, w["w_gu"], w["w_down"], route="softmax_renorm",
                               renorm_eps=1e-20, gated=(LO.ACT_CLAMPED_SWISH, 1.25, 1.702, 1.0))
            assert tuple(y.shape) == (70, top, W) and y.dtype == torch.float32
            assert rel_err(y.sum(1).cpu(), ref) < tol, (dtype, unfused)
        monkeypatch.delenv("JL_MOE_UNFUSED_ACT")
    # ties go to the lower index, and the weights of the chosen sum to one
    z = torch.zeros(2, E)
    z[1, E - 1] = 1.0
    zc, ids, wts = z.cuda(), torch.empty((2, top), dtype=torch.int32, device="cuda"), torch.empty((2, top), device="cuda")
    from jacobiforcing_amd import _native as N
    N.check_layers(N.layers().jl_moe_route(zc.data_ptr(), None, 2, E, top, 1.0, ids.data_ptr(), wts.data_ptr(), N.JL_ROUTE_SOFTMAX_RENORM, 1e-20,
                                          torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert ids[0].tolist() == list(range(top)) and ids[1].tolist() == ([E - 1] + list(range(top - 1)))[:top]
    assert torch.allclose(wts.sum(1).cpu(), torch.ones(2), atol=1e-6)


def one_layer(H, G, D, Dv, size, dims, W=64, scaling=STRETCH, scale=0.4, base=300.0):
    return make_cfg([dict(attn(heads=H, kv=G, dim=D, vdim=Dv, size=size, dims=dims, base=base, scale=scale, scaling=scaling), mlp=None)], width=W, vocab=40)


# head sizes that take the one-sweep matrix-core kernel in bfloat16 (D % 8 == 0, Dv % 32 == 0), the two-sweep one (H <= 16, Dv % 4 == 0),
# and the plain one; rotations over the whole head, a part of it in multiples of eight and not, and none
ATTN_SIZES = [(4, 2, 32, 64, 21, 16), (8, 8, 64, 32, 9, 64), (3, 1, 24, 40, 30, 12), (2, 1, 128, 128, 50, 32), (12, 4, 16, 16, 0, 8), (5, 5, 40, 96, 64, 40),
              (40, 1, 16, 32, 17, 0), (1, 1, 20, 10, 5, 6), (6, 3, 48, 20, 1, 48), (16, 2, 64, 128, 100, 24), (2, 2, 256, 64, 33, 128)]


@gpu
@pytest.mark.parametrize("H,G,D,Dv,size,dims", ATTN_SIZES)
def test_the_mixer_alone_in_portions_and_single_tokens(H, G, D, Dv, size, dims):
    """Rotation, unit norm, window, sink and head gate of one layer on the oracle's own inputs, float32 and bfloat16: a prompt's
    portion, a second portion that starts inside a page, then single tokens."""
    cfg = one_layer(H, G, D, Dv, size, dims)
    t = tensors_for(cfg, H + D)
    t["l0.mix.sink"] = t["l0.mix.sink"] + 2.0                                                   # sinks that take a good share of every row
    T, cuts = 150, [83, 40] + [1] * 27
    h = torch.randn(T, 64, generator=torch.Generator().manual_seed(1))
    m = cfg["layers"][0]["mixer"]
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
        rig = Rig(cfg, tensors=t, dtype=dtype, page=16, pages=24)
        rig.poison()
        hin = h.to(dtype)
        want = O.gated_sink_attention(hin.double(), {k: v.double() for k, v in O.layer_tensors(t, 0).items()}, m, 1e-5)
        got, at = [], 0
        for c in cuts:
            b = rig.LO.RaggedBatch.build([c], [at], [1], [[9, 3, 20, 11, 5, 0, 1, 2, 4, 6]], 16, "cuda")
            got.append(rig.model._attention(0, 0, hin[at:at + c].cuda(), b, rig.cache).float().cpu())
            at += c
        assert rel_err(torch.cat(got), want) < tol, dtype
    no_sink = dict(O.layer_tensors(t, 0), **{"mix.sink": torch.full((H,), -60.0)})
    assert rel_err(O.gated_sink_attention(h.double(), {k: v.double() for k, v in no_sink.items()}, m, 1e-5), want) > 0.05      # a sink left out shows


@gpu
@pytest.mark.parametrize("H,G,D,Dv", [(4, 2, 32, 64), (8, 8, 64, 32), (2, 1, 128, 128), (40, 1, 16, 32), (16, 2, 64, 128), (2, 2, 256, 64), (6, 2, 24, 96),
                                      (3, 1, 40, 128), (8, 2, 128, 128), (5, 1, 64, 32)])
@pytest.mark.parametrize("size", [0, 21, 100])
def test_long_portions_on_tiles_of_128_rows(H, G, D, Dv, size, monkeypatch):
    """bfloat16 steps whose requests bring many tokens run the one-sweep attention on tiles of up to 128 (query, head) rows, every
    wavefront with rows of its own: two unequal requests side by side, the second continuing from a position inside a page, tiles
    that end inside a request, windows shorter and longer than a tile, sinks that matter, the head gate."""
    from jacobiforcing_amd import _native as N
    from jacobiforcing_amd import layer_ops as LO
    monkeypatch.setattr(LO, "SWEEP_SPLIT_BELOW_GROUPS", 1)                                      # small steps too
    assert N.layers().jl_attn_sweep_wide_tile_rows(N.JL_BF16, H, G, G, D, Dv, G * D, G * Dv, 0) == 128 // min(H // G, 32)
    cfg = one_layer(H, G, D, Dv, size, 8)
    t = tensors_for(cfg, H + Dv)
    t["l0.mix.sink"] = t["l0.mix.sink"] + 2.0
    m = cfg["layers"][0]["mixer"]
    P = {k: v.double() for k, v in O.layer_tensors(t, 0).items()}
    ha = torch.randn(170, 64, generator=torch.Generator().manual_seed(1)).bfloat16()
    hb = torch.randn(107, 64, generator=torch.Generator().manual_seed(2)).bfloat16()
    want_a, want_b = O.gated_sink_attention(ha.double(), P, m, 1e-5), O.gated_sink_attention(hb.double(), P, m, 1e-5)
    rig = Rig(cfg, tensors=t, dtype=torch.bfloat16, page=16, pages=32)
    rig.poison()
    ta, tb = [9, 3, 20, 11, 5, 0, 1, 2, 4, 6, 30], [7, 8, 10, 12, 13, 14, 15]
    b0 = rig.LO.RaggedBatch.build([37], [0], [0], [tb], 16, "cuda")                               # the second request's first 37 tokens
    g0 = rig.model._attention(0, 0, hb[:37].cuda(), b0, rig.cache).float().cpu()
    b1 = rig.LO.RaggedBatch.build([170, 70], [0, 37], [1, 0], [ta, tb], 16, "cuda")
    g1 = rig.model._attention(0, 0, torch.cat([ha, hb[37:]]).cuda(), b1, rig.cache).float().cpu()
    assert rel_err(g1[:170], want_a) < 3e-2 and rel_err(torch.cat([g0, g1[170:]]), want_b) < 3e-2
    monkeypatch.setenv("JL_ATTN_NO_SWEEP", "1")                                                  # and the two kernels agree to rounding
    g2 = rig.model._attention(0, 0, torch.cat([ha, hb[37:]]).cuda(), b1, rig.cache).float().cpu()
    assert rel_err(g1, g2) < 2e-2


@gpu
@pytest.mark.parametrize("H,G,D,Dv", [(4, 1, 64, 64), (8, 2, 32, 96), (6, 2, 24, 40), (3, 3, 20, 12)])
@pytest.mark.parametrize("size", [0, 300])
def test_single_tokens_over_a_long_context_take_the_sink_once(H, G, D, Dv, size):
    """Decoding far into a context shares the keys of a tile out over workgroups; the sink belongs to one share only."""
    cfg = one_layer(H, G, D, Dv, size, 8)
    t = tensors_for(cfg, 3)
    t["l0.mix.sink"] = t["l0.mix.sink"] + 3.0
    T = 420
    h = torch.randn(T, 64, generator=torch.Generator().manual_seed(5))
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
        rig = Rig(cfg, tensors=t, dtype=dtype, page=64, pages=8)
        hin = h.to(dtype)
        want = O.gated_sink_attention(hin.double(), {k: v.double() for k, v in O.layer_tensors(t, 0).items()}, cfg["layers"][0]["mixer"], 1e-5)
        got, at = [], 0
        for c in [T - 3, 1, 1, 1]:
            b = rig.LO.RaggedBatch.build([c], [at], [0], [[5, 2, 7, 0, 3, 1, 6]], 64, "cuda")
            got.append(rig.model._attention(0, 0, hin[at:at + c].cuda(), b, rig.cache).float().cpu())
            at += c
        assert rel_err(torch.cat(got)[-3:], want[-3:]) < tol and rel_err(torch.cat(got), want) < tol, dtype


@gpu
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_each_feed_forward_alone(name):
    rig = Rig(SHAPES[name](), seed=3)
    h = torch.randn(37, rig.cfg.hidden_size, generator=torch.Generator().manual_seed(1))
    for li, L in enumerate(rig.cfg_dict["layers"]):
        if L.get("mlp") is None:
            continue
        P = {k: v.double() for k, v in O.layer_tensors(rig.tensors, li).items()}
        parts = rig.model._feed_forward(li, h.cuda())
        got = sum(y.float().sum(1) if y.dim() == 3 else y.float() for y, _ in parts)
        assert all(s is rig.model.w.layers[li]["ls2"] for _, s in parts)
        assert rel_err(got.cpu(), O.feed_forward(h.double(), P, L["mlp"])) < 1e-5, li


@gpu
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_prompt_and_every_layer_run(name):
    rig = Rig(SHAPES[name](), seed=5)
    t = toks(61, rig.cfg.vocab_size, 1)
    trace = []
    got = rig.step([("p", t)], trace)
    want, want_trace = rig.oracle(t)
    assert len(trace) == want_trace.shape[0] == len(rig.cfg.runs())
    for i, x in enumerate(trace):
        assert rel_err(x.cpu(), want_trace[i]) < 1e-5, f"layer run {i}"
    assert rel_err(got, want) < F32_TOL
    assert rel_err(Rig(SHAPES[name](), seed=5).step([("p", t)]), want) < F32_TOL                 # the same with the sums folded into the norms
    assert rel_err(Rig(SHAPES[name](), seed=5, dtype=torch.bfloat16).step([("p", t)]), want) < BF16_TOL


@gpu
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_prefill_equals_token_by_token_decoding(name):
    rig = Rig(SHAPES[name](), seed=7)
    t = toks(40, rig.cfg.vocab_size, 2)
    want, _ = rig.oracle(t)
    rig.poison()
    whole = rig.step([("whole", t)])
    single = torch.cat([rig.step([("single", [x])]) for x in t])
    assert rel_err(whole, want) < F32_TOL and rel_err(single, want) < F32_TOL and rel_err(single, whole) < F32_TOL


@gpu
@pytest.mark.parametrize("cuts", [[2] * 20, [1, 2, 3, 5, 8, 13, 7, 1], [7, 9, 8, 16], [39, 1], [3, 37]])
def test_portions_of_any_size(cuts):
    """Cuts inside pages and windows; portions of two tokens."""
    for name in ("a", "b"):
        rig = Rig(SHAPES[name](), seed=11)
        t = toks(sum(cuts), rig.cfg.vocab_size, 3)
        want, _ = rig.oracle(t)
        rig.poison()
        got, at = [], 0
        for c in cuts:
            got.append(rig.step([("r", t[at:at + c])]))
            at += c
        assert rel_err(torch.cat(got), want) < F32_TOL, name


@gpu
def test_unequal_requests_in_one_batch_equal_each_alone():
    rig = Rig(shape_a(), seed=13, pages=96)
    V = rig.cfg.vocab_size
    reqs = {"long": toks(70, V, 4), "mid": toks(23, V, 5), "one": toks(1, V, 6), "two": toks(2, V, 7)}
    want = {k: rig.oracle(v)[0] for k, v in reqs.items()}
    rig.poison()
    # step 1: portions of three prompts side by side; step 2: the rest of one, single tokens of the others, a new request
    s1 = rig.step([("long", reqs["long"][:50]), ("mid", reqs["mid"][:22]), ("one", reqs["one"])])
    s2 = rig.step([("long", reqs["long"][50:51]), ("two", reqs["two"]), ("mid", reqs["mid"][22:])])
    s3 = rig.step([("long", reqs["long"][51:])])
    got = {"long": torch.cat([s1[:50], s2[:1], s3]), "mid": torch.cat([s1[50:72], s2[3:4]]), "one": s1[72:73], "two": s2[1:3]}
    for k in reqs:
        assert rel_err(got[k], want[k]) < F32_TOL, k


@gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32_TOL), (torch.bfloat16, BF16_TOL)])
def test_freed_pages_and_slots_are_used_again(dtype, tol):
    """Two slots, a pool that holds two requests: requests end, their pages and slots go to new ones, old keys must not leak — in
    none of the passes of the looped span, which have pools of their own."""
    rig = Rig(shape_a(), seed=17, pages=12, slots=2, dtype=dtype)
    V = rig.cfg.vocab_size
    rig.poison()
    for rnd in range(4):
        a, b = toks(40 + rnd, V, 20 + rnd), toks(17 + 3 * rnd, V, 30 + rnd)
        ga = rig.step([("a", a[:25]), ("b", b[:1])])                                           # b starts with a single token on used pages
        gb = rig.step([("a", a[25:]), ("b", b[1:])])
        got_a = torch.cat([ga[:25], gb[:len(a) - 25]])
        got_b = torch.cat([ga[25:], gb[len(a) - 25:]])
        assert rel_err(got_a, rig.oracle(a)[0]) < tol and rel_err(got_b, rig.oracle(b)[0]) < tol, rnd
        used = set(rig.req["a"]["pages"]) | set(rig.req["b"]["pages"])
        rig.end("b"); rig.end("a")
        assert len(rig.free_pages) == 12 and len(used) >= 8


def peaked_model(size, D=16, Dv=16, dims=4, loop=None):
    """One attention layer (run once, or looped), no feed-forward, a sharp softmax, a rotation over a small part of the head.
    Returns (cfg, tensors, hot query token, hot key token, scores): the pair of tokens whose unrotated score is the largest."""
    cfg = make_cfg([dict(attn(heads=2, kv=1, dim=D, vdim=Dv, size=size, dims=dims, base=10000.0, scale=2.5), mlp=None)], width=32, vocab=40, loop=loop)
    t = tensors_for(cfg, 23)
    t["l0.mix.sink"] = torch.zeros(2)
    t["l0.mix.g"] = torch.zeros_like(t["l0.mix.g"])
    eps = cfg["norm"]["eps"]
    h = O.centred_norm(t["embed"].double(), t["l0.norm1"].double(), eps)
    q = O.unit_rms((h @ t["l0.mix.q"].double().T + t["l0.mix.q.b"].double()).view(40, 2, D), eps)[:, 0]
    k = O.unit_rms((h @ t["l0.mix.k"].double().T + t["l0.mix.k.b"].double()).view(40, 1, D), eps)[:, 0]
    s = q[:, dims:] @ k[:, dims:].T
    qi, kj = divmod(int(s.argmax()), 40)
    return cfg, t, qi, kj, s


@gpu
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("dtype,tol,D,Dv", [(torch.float32, F32_TOL, 16, 16), (torch.bfloat16, BF16_TOL, 16, 16), (torch.bfloat16, BF16_TOL, 32, 64)])
def test_a_key_just_inside_and_just_outside_the_window(decode, dtype, tol, D, Dv):
    size = 21
    cfg, t, qi, kj, s = peaked_model(size, D, Dv)
    dull = [x for x in np.argsort(s[qi].numpy())[:12].tolist() if x != kj]                         # keys the hot query ignores
    T = 70
    cases = {"window_in": T - 1 - (size - 1), "window_out": T - 1 - size, "page_border_in": 56, "first": 0, "near": T - 2}
    outs = {}
    for name, j in cases.items():
        seq = [dull[i % len(dull)] for i in range(T)]
        seq[j], seq[T - 1] = kj, qi
        rig = Rig(cfg, tensors=t, dtype=dtype)
        rig.poison()
        if decode:
            rig.step([("r", seq[:T - 9])])
            got = torch.cat([rig.step([("r", [x])]) for x in seq[T - 9:]])[-1]
        else:
            got = rig.step([("r", seq[:30]), ("other", seq[:11])])                               # a second request beside it
            got = rig.step([("r", seq[30:])])[-1]
        want = rig.oracle(seq)[0][-1]
        assert rel_err(got, want) < tol, name
        outs[name] = want
    # the inputs do show an edge that is one token off: a seen and an unseen hot key give different logits
    assert rel_err(outs["window_in"], outs["window_out"]) > 0.05 and rel_err(outs["page_border_in"], outs["window_out"]) > 0.05
    assert rel_err(outs["first"], outs["window_out"]) < 0.05                                     # both unseen: nearly the same


@gpu
@pytest.mark.parametrize("dtype,tol", [(torch.float32, F32_TOL), (torch.bfloat16, BF16_TOL)])
def test_a_far_key_among_hundreds(dtype, tol):
    """A window longer than the sequence over many pages: the hot key sits 280 tokens back, at a page's first place, and the layer
    runs twice (a pool per pass)."""
    cfg, t, qi, kj, s = peaked_model(400, loop=(0, 1, 2))
    dull = [x for x in np.argsort(s[qi].numpy())[:12].tolist() if x != kj]
    T = 300
    seq = [dull[i % len(dull)] for i in range(T)]
    seq[16], seq[T - 1] = kj, qi
    rig = Rig(cfg, tensors=t, pages=64, dtype=dtype)
    got = rig.step([("r", seq[:121])])
    got = torch.cat([got, rig.step([("r", seq[121:T - 2])]), rig.step([("r", seq[T - 2:T - 1])]), rig.step([("r", seq[T - 1:])])])
    want = rig.oracle(seq)[0]
    assert rel_err(got[-1], want[-1]) < tol and rel_err(got, want) < tol
    seq2 = list(seq)
    seq2[16] = dull[0]
    assert rel_err(rig.oracle(seq2)[0][-1], want[-1]) > 0.05
    near = json.loads(json.dumps(cfg))
    near["layers"][0]["mixer"]["mask"]["size"] = 283                                             # one token short of the hot key
    assert rel_err(O.forward(near, t, seq, torch.float64)[0][-1], want[-1]) > 0.05


@gpu
def test_the_first_tokens_of_a_sequence():
    """One, two and three tokens on pages that hold another request's keys."""
    for name in ("a", "b"):
        rig = Rig(SHAPES[name](), seed=19, slots=2, pages=16)
        V = rig.cfg.vocab_size
        rig.step([("old", toks(30, V, 1))])
        rig.end("old")
        for n in (1, 2, 3):
            t = toks(n + 1, V, 50 + n)
            got = torch.cat([rig.step([("new", t[:n])]), rig.step([("new", t[n:])])])
            assert rel_err(got, rig.oracle(t)[0]) < F32_TOL, (name, n)
            rig.end("new")


@gpu
def test_long_decoding_keeps_the_window():
    rig = Rig(shape_b(), seed=29, pages=64)
    t = toks(260, rig.cfg.vocab_size, 8)
    want, _ = rig.oracle(t)
    rig.poison()
    got = torch.cat([rig.step([("r", t[:20])])] + [rig.step([("r", [x])]) for x in t[20:]])
    assert rel_err(got, want) < F32_TOL and rel_err(got[-1], want[-1]) < F32_TOL
    rb = Rig(shape_b(), seed=29, pages=64, dtype=torch.bfloat16)
    gb = torch.cat([rb.step([("r", t[:20])])] + [rb.step([("r", [x])]) for x in t[20:]])
    assert rel_err(gb, want) < BF16_TOL


def random_shape(seed):
    """A random configuration: layer count and order, loop, head counts, sizes (multiples of eight and not), windows from one token
    to longer than the sequence, rotations, stretch constants, feed-forward kinds, expert counts, limits, logit scale."""
    r = random.Random(seed)
    layers = []
    for _ in range(r.choice([1, 2, 3, 4])):
        kind = r.random()
        if kind < 0.2:
            mlp = None
        elif kind < 0.55:
            mlp = dense(r.choice([8, 24, 40, 100]))
        else:
            E = r.choice([2, 3, 4, 8, 17])
            mlp = moe(experts=E, top=r.choice([t for t in (1, 2, 3, 4) if t <= E]), ff=r.choice([8, 12, 32, 48]), limit=r.choice([0.5, 1.0, 3.0, 7.0]),
                      shared_ff=r.choice([0, 8, 20, 64]), shared_limit=r.choice([0.5, 2.0, 6.0]))
        kv = r.choice([1, 2, 3, 4])
        D = r.choice([8, 16, 20, 24, 32, 64])
        stretch = None if r.random() < 0.3 else {"factor": r.choice([2.0, 4.0, 32.0]), "low": r.choice([0.5, 1.0, 2.0]), "high": r.choice([3.0, 4.0, 8.0]),
                                                 "original": r.choice([8, 32, 256, 4096])}
        layers.append(dict(attn(heads=kv * r.choice([1, 2, 3, 5]), kv=kv, dim=D, vdim=r.choice([8, 16, 32, 40, 64, 96]), size=r.choice([0, 1, 2, 5, 8, 9, 17, 40, 1000]),
                                dims=r.choice([d for d in (0, 2, 4, 8, 12, 16, 20, 24, 32, 64) if d <= D]), base=r.choice([100.0, 10000.0, 5e5]),
                                scale=r.choice([0.1, 0.25, 0.5]), scaling=stretch), mlp=mlp))
    n = len(layers)
    a = r.randrange(n + 1)
    b = r.randrange(a, n + 1)
    return make_cfg(layers, width=r.choice([32, 48, 64, 72, 100]), vocab=r.choice([17, 64, 131]), eps=r.choice([1e-5, 1e-6]),
                    loop=r.choice([None, (a, b, r.choice([1, 2, 3]))]), logit_scale=r.choice([0.5, 1.0, 3.0]))


@gpu
@pytest.mark.parametrize("seed", range(16))
def test_random_configurations_in_a_mixed_schedule(seed):
    """Two requests cut at random into portions and single tokens, side by side from poisoned pools, float32 and bfloat16."""
    cfg = random_shape(seed)
    r = random.Random(100 + seed)
    V = cfg["vocab"]
    a, b = toks(45, V, seed), toks(29, V, seed + 50)
    for dtype, tol in ((torch.float32, F32_TOL), (torch.bfloat16, 2 * BF16_TOL)):
        rig = Rig(cfg, seed=seed, dtype=dtype, pages=32)
        want_a, want_b = rig.oracle(a)[0], rig.oracle(b)[0]
        rig.poison()
        got_a, got_b, ia, ib = [], [], 0, 0
        while ia < len(a) or ib < len(b):
            na = min(len(a) - ia, r.choice([1, 1, 2, 3, 7, 16]))
            nb = min(len(b) - ib, r.choice([0, 1, 1, 2, 5, 11])) if ia > 6 else 0
            entries = ([("a", a[ia:ia + na])] if na else []) + ([("b", b[ib:ib + nb])] if nb else [])
            if not entries:
                entries, nb = [("b", b[ib:ib + 1])], 1
            out = rig.step(entries)
            got_a.append(out[:na]); got_b.append(out[na:])
            ia += na; ib += nb
        if dtype == torch.float32:
            assert rel_err(torch.cat(got_a), want_a) < tol and rel_err(torch.cat(got_b), want_b) < tol, (seed, dtype, cfg)
        else:
            assert rows_off(torch.cat(got_a), want_a, tol) <= 0.1 and rows_off(torch.cat(got_b), want_b, tol) <= 0.1, (seed, dtype, cfg)


def _write_model(tmp_path, cfg_dict, tensors):
    from safetensors.torch import save_file
    (tmp_path / "config.json").write_text(json.dumps(cfg_dict))
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()}, str(tmp_path / "model.safetensors"))
    return str(tmp_path)


def _oracle_greedy(cfg_dict, tensors, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(O.forward(cfg_dict, tensors, seq, torch.float64)[0][-1].argmax()))
    return seq[len(prompt):]


@gpu
def test_greedy_generation_through_the_engine_and_its_scheduler(tmp_path):
    """LLM.generate on a checkpoint directory: registry -> loader -> scheduler (prompts cut to the token budget, admissions
    limited by two slots, pages reused) -> ragged step -> argmax.  float32 so that the greedy choice is the oracle's."""
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
    wa, wb = O.forward(cfg_dict, tensors, a, torch.float64)[0], O.forward(cfg_dict, tensors, b, torch.float64)[0]
    assert tuple(l1.shape) == (2, V) and rel_err(l1.cpu(), wa[[0, 39]]) < F32_TOL
    assert rel_err(l2.cpu(), torch.stack([wa[69], wb[len(b) - 1]])) < F32_TOL and rel_err(l3.cpu(), wa[-1:]) < F32_TOL
    assert len(llm.scheduler.block_manager.free_block_ids) == 4 and len(llm.model_runner.free_rows) == 2


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
    p = torch.softmax(O.forward(cfg_dict, tensors, prompt, torch.float64)[0][-1], 0).numpy()
    counts = np.bincount([o["token_ids"][0] for o in out], minlength=len(p)) / 800.0
    assert 0.5 * np.abs(counts - p).sum() < 0.2                                                 # total variation of 800 draws over 77 ids
