"""Bamanex: a decoder with a float residual stream whose layers run their mixer and their feed-forward side by side on the SAME
stream — x += ls1 * mixer(norm1(x)) + ls2 * ff(norm2(x)), both norms zero-centred (weight stored as w, applied as 1 + w), ls1 / ls2
a scale per channel — and which may run a span of its layers several times with the same weights (every pass with a cache of
its own).

* mixer ``attention``: grouped-query attention with biased projections; rotary positions on the first ``rot.dims`` dimensions of
  every head (rotate-half pairs) with frequencies stretched for long wavelengths (unchanged below a wavelength of original/high,
  divided by ``factor`` above original/low, blended in between); queries and keys brought to unit RMS per head after the rotation;
  a sliding window; a learned sink per head in the softmax's denominator; a sigmoid gate per head on the heads' outputs.
* feed-forward ``dense``: down(gelu_tanh(gate h) * up h).
* feed-forward ``moe``: softmax router over all experts, the largest ``top`` chosen and renormalised; experts are clamped gated
  units down(g sigmoid(1.702 g) (u + 1)) with g = min(gate h, limit), u = clamp(up h, +-limit); a shared expert of the same form runs
  for every token behind a sigmoid gate of one number per token.

The forward runs one ragged batch (``layer_ops.RaggedBatch``): portions of prompts and single decoded tokens side by side, over
``engine.state_cache.PagedStateCache``.  Dense products are torch's (hipBLASLt / rocBLAS); everything else is a launch of
``libjf_layers.so`` / ``libjf_layers_seq.so``.  A layer's two sublayer outputs are folded, with their scales, into the launch that
forms the next layer's two norms.  With float32 weights every product is a true 32-bit one."""
from __future__ import annotations

import json
import math
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import layer_ops as LO
from ..engine.state_cache import PagedStateCache, RunSpec

SWISH_ALPHA, UNIT_SHIFT, ROUTER_RENORM_EPS = 1.702, 1.0, 1e-20       # constants of the design's clamped gated unit and router


@dataclass
class BamanexConfig:
    vocab_size: int
    hidden_size: int
    layers: List[Dict[str, Any]]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    max_position_embeddings: int = 1 << 20          # the design has no limit of its own: the engine's max_model_len decides
    eos_token_id: int = -1
    pad_token_id: int = 0
    family: str = "ragged"

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "BamanexConfig":
        lp = d.get("loop") or {}
        n = len(d["layers"])
        start, stop, times = int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1))
        if not (0 <= start <= stop <= n) or times < 1:
            raise ValueError(f"loop {lp} does not fit {n} layers")
        for i, L in enumerate(d["layers"]):
            if L["type"] != "attention":
                raise ValueError(f"layer {i}: unknown mixer {L['type']!r}")
            m = L["mixer"]
            if int(m["heads"]) % int(m["kv_heads"]):
                raise ValueError(f"layer {i}: {m['heads']} heads over {m['kv_heads']} key/value heads")
            dims = int((m.get("rot") or {}).get("dims", 0))
            if dims % 2 or dims > int(m["dim"]):
                raise ValueError(f"layer {i}: rot.dims {dims} must be even and at most dim {m['dim']}")
            f = L.get("mlp")
            if f is not None and f.get("kind", "dense") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward {f.get('kind')!r}")
            if f is not None and f.get("kind") == "moe" and not 1 <= int(f["router"]["top"]) <= int(f["router"]["experts"]):
                raise ValueError(f"layer {i}: top {f['router']['top']} of {f['router']['experts']} experts")
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), layers=d["layers"], loop_start=start, loop_stop=stop,
                   loop_times=times, norm_eps=float(d["norm"]["eps"]), logit_scale=float(d.get("logit_scale", 1.0)),
                   eos_token_id=int(d.get("eos_token_id", -1)), pad_token_id=int(d.get("pad_token_id", 0)))

    @classmethod
    def from_json(cls, path) -> "BamanexConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))

    def runs(self) -> List[int]:
        """Layer indices in execution order: the span loop_start .. loop_stop-1 runs loop_times times in a row."""
        a, b = self.loop_start, self.loop_stop
        return list(range(a)) + list(range(a, b)) * (self.loop_times if b > a else 0) + list(range(b, len(self.layers)))


def rotary_frequencies(dims: int, base: float, scaling: Optional[Dict[str, Any]]) -> List[float]:
    """Angle per position of pair i < dims/2: base^(-2i/dims), stretched by ``scaling`` {factor, low, high, original}: wavelengths
    below original/high keep their frequency, those above original/low get frequency/factor, and in between the two are blended
    with s = (original/wavelength - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength > orig / low:
                f = f / factor
            elif wavelength >= orig / high:
                s = (orig / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def _rot_key(m: Dict[str, Any]):
    rot = m.get("rot") or {}
    sc = rot.get("scaling") or None
    return (int(rot.get("dims", 0)), float(rot.get("base", 10000.0)),
            tuple(float(sc[k]) for k in ("factor", "low", "high", "original")) if sc else None)


class BamanexWeights:
    """Tensors by their checkpoint names (``embed``, ``l<i>.norm1``, ``l<i>.mix.q`` / ``.q.b`` …, ``l<i>.mlp.*``, ``l<i>.ls1``,
    ``final.norm``, ``head``), regrouped per layer for the forward: the mixer's input projections (q, k, v, head gate) stacked into
    one matrix with one bias vector, a dense feed-forward's gate and up stacked, every expert's gate rows stacked on its up rows
    ([E, 2*ff, W]), the shared expert's gate, up and token gate stacked; norm weights, channel scales, sinks and the router in
    float."""

    def __init__(self, cfg: BamanexConfig, tensors: Dict[str, torch.Tensor], device, dtype=torch.bfloat16):
        dev = torch.device(device)
        act = lambda k: tensors[k].to(device=dev, dtype=dtype).contiguous()
        f32 = lambda k: tensors[k].to(device=dev, dtype=torch.float32).contiguous()
        self.device, self.dtype = dev, dtype
        W = cfg.hidden_size
        self.embed, self.final_norm, self.head = act("embed"), f32("final.norm"), act("head")
        if tuple(self.embed.shape) != (cfg.vocab_size, W):
            raise ValueError(f"embed is {tuple(self.embed.shape)}, config says {(cfg.vocab_size, W)}")
        self.layers = []
        # a stacked matrix ends with zero rows up to a multiple of eight: the product's rows then start at 16-byte borders
        pad = lambda rows: torch.zeros(((-rows) % 8, W), dtype=dtype, device=dev)
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L["mixer"]
            H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
            rows = H * D + G * D + G * Dv + H
            w = dict(norm1=f32(p + "norm1"), ls1=f32(p + "ls1"), sink=f32(p + "mix.sink"), w_o=act(p + "mix.o"), b_o=act(p + "mix.o.b"),
                     w_in=torch.cat([act(p + "mix.q"), act(p + "mix.k"), act(p + "mix.v"), act(p + "mix.g"), pad(rows)], 0),
                     b_in=torch.cat([act(p + "mix.q.b"), act(p + "mix.k.b"), act(p + "mix.v.b"), torch.zeros(H + (-rows) % 8, dtype=dtype, device=dev)], 0),
                     cols=(0, H * D, H * D + G * D, H * D + G * D + G * Dv))
            if w["w_in"].shape[0] != rows + (-rows) % 8 or w["sink"].numel() != H or tuple(w["w_o"].shape) != (W, H * Dv):
                raise ValueError(f"layer {i}: the mixer's tensors do not fit heads={H} kv_heads={G} dim={D} vdim={Dv}")
            f = L.get("mlp")
            if f is not None:
                w.update(norm2=f32(p + "norm2"), ls2=f32(p + "ls2"))
                if f.get("kind", "dense") == "dense":
                    w.update(w_gu=torch.cat([act(p + "mlp.gate"), act(p + "mlp.up")], 0), w_down=act(p + "mlp.down"))
                    if w["w_gu"].shape[0] != 2 * int(f["ff"]):
                        raise ValueError(f"layer {i}: gate / up have {w['w_gu'].shape[0]} rows together, config says ff {f['ff']}")
                else:
                    E, ff = int(f["router"]["experts"]), int(f["expert"]["ff"])
                    w.update(router=f32(p + "mlp.router"),
                             w_gu=torch.stack([torch.cat([act(p + f"mlp.e{e}.gate"), act(p + f"mlp.e{e}.up")], 0) for e in range(E)]).contiguous(),
                             w_down=torch.stack([act(p + f"mlp.e{e}.down") for e in range(E)]).contiguous())
                    if tuple(w["w_gu"].shape) != (E, 2 * ff, W) or tuple(w["router"].shape) != (E, W):
                        raise ValueError(f"layer {i}: experts are {tuple(w['w_gu'].shape)}, config says {E} experts of ff {ff}")
                    if f.get("shared") is not None:
                        fs = int(f["shared"]["ff"])
                        w.update(w_sh=torch.cat([act(p + "mlp.shared.gate"), act(p + "mlp.shared.up"), act(p + "mlp.shared.sg").view(1, W), pad(2 * fs + 1)], 0),
                                 w_sh_down=act(p + "mlp.shared.down"))
                        if w["w_sh"].shape[0] != 2 * fs + 1 + (-(2 * fs + 1)) % 8:
                            raise ValueError(f"layer {i}: the shared expert's gate / up do not have the {fs} rows each that the config says")
            self.layers.append(w)

    @classmethod
    def from_safetensors(cls, cfg: BamanexConfig, model_dir, device, dtype=torch.bfloat16) -> "BamanexWeights":
        from safetensors import safe_open
        files = sorted(Path(model_dir).glob("*.safetensors"))
        if not files:
            raise FileNotFoundError(f"no *.safetensors under {model_dir}")
        tensors = {}
        for f in files:
            with safe_open(str(f), "pt", "cpu") as sf:
                for k in sf.keys():
                    tensors[k] = sf.get_tensor(k)
        return cls(cfg, tensors, device, dtype)

    @classmethod
    def random(cls, cfg: BamanexConfig, device, dtype=torch.bfloat16, seed: int = 0) -> "BamanexWeights":
        return cls(cfg, random_tensors(cfg, seed), device, dtype)


def random_tensors(cfg: BamanexConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's names (benchmarks and tests; bf16-representable float32 values)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.hidden_size
    rnd = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(torch.bfloat16).float()
    lin = lambda o, i: rnd(o, i, std=i ** -0.5)
    t = {"embed": rnd(cfg.vocab_size, W), "final.norm": rnd(W, std=0.1), "head": lin(cfg.vocab_size, W)}
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        t.update({p + "norm1": rnd(W, std=0.1), p + "ls1": (0.5 + 0.5 * torch.rand(W, generator=g)).to(torch.bfloat16).float(),
                  p + "mix.q": lin(H * D, W), p + "mix.q.b": rnd(H * D, std=0.1), p + "mix.k": lin(G * D, W), p + "mix.k.b": rnd(G * D, std=0.1),
                  p + "mix.v": lin(G * Dv, W), p + "mix.v.b": rnd(G * Dv, std=0.1), p + "mix.sink": rnd(H), p + "mix.g": lin(H, W),
                  p + "mix.o": lin(W, H * Dv), p + "mix.o.b": rnd(W, std=0.1)})
        f = L.get("mlp")
        if f is None:
            continue
        t.update({p + "norm2": rnd(W, std=0.1), p + "ls2": (0.5 + 0.5 * torch.rand(W, generator=g)).to(torch.bfloat16).float()})
        if f.get("kind", "dense") == "dense":
            t.update({p + "mlp.gate": lin(f["ff"], W), p + "mlp.up": lin(f["ff"], W), p + "mlp.down": lin(W, f["ff"])})
            continue
        E, ff = f["router"]["experts"], f["expert"]["ff"]
        t[p + "mlp.router"] = lin(E, W) * 2
        for e in range(E):
            t.update({p + f"mlp.e{e}.gate": lin(ff, W) * 2, p + f"mlp.e{e}.up": lin(ff, W) * 2, p + f"mlp.e{e}.down": lin(W, ff)})
        if f.get("shared") is not None:
            fs = f["shared"]["ff"]
            t.update({p + "mlp.shared.gate": lin(fs, W) * 2, p + "mlp.shared.up": lin(fs, W) * 2, p + "mlp.shared.down": lin(W, fs),
                      p + "mlp.shared.sg": lin(1, W)})
    return t


class BamanexModel:
    def __init__(self, cfg: BamanexConfig, weights: BamanexWeights, max_positions: int = 8192):
        self.cfg, self.w = cfg, weights
        self.device, self.dtype = weights.device, weights.dtype
        self.runs = cfg.runs()
        self._angles: Dict[tuple, tuple] = {}
        self.max_positions = 0
        self.reserve_positions(max_positions)

    # ---- what the cache must hold, one entry per layer run (a repeated layer has a pool per pass) ---------------------------------------
    def cache_specs(self) -> List[RunSpec]:
        return [RunSpec("kv", k_width=int(m["kv_heads"]) * int(m["dim"]), v_width=int(m["kv_heads"]) * int(m["vdim"]))
                for m in (self.cfg.layers[li]["mixer"] for li in self.runs)]

    def new_cache(self, num_pages: int, page_size: int, num_slots: int) -> PagedStateCache:
        return PagedStateCache(self.cache_specs(), num_pages, page_size, num_slots, self.device, self.dtype)

    # ---- rotation angles for every position the engine can reach: position * frequency, cosine and sine, all in float32 -----------------
    def reserve_positions(self, n: int) -> None:
        if n <= self.max_positions:
            return
        self.max_positions = int(n)
        self._angles.clear()
        for L in self.cfg.layers:
            key = _rot_key(L["mixer"])
            if key[0] and key not in self._angles:
                f = torch.tensor(rotary_frequencies(key[0], key[1], dict(zip(("factor", "low", "high", "original"), key[2])) if key[2] else None),
                                 dtype=torch.float32, device=self.device)
                a = torch.arange(n, dtype=torch.float32, device=self.device).view(n, 1) * f.view(1, -1)
                self._angles[key] = (a.cos().contiguous(), a.sin().contiguous())

    # ---- mixer -------------------------------------------------------------------------------------------------------------------------
    def _attention(self, run: int, li: int, h: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache) -> torch.Tensor:
        m, w, eps = self.cfg.layers[li]["mixer"], self.w.layers[li], self.cfg.norm_eps
        H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        key = _rot_key(m)
        cos, sin = self._angles[key] if key[0] else (None, None)
        proj = F.linear(h, w["w_in"], w["b_in"])
        kp, vp = cache.k[run], cache.v[run]
        q = LO.head_norm_append(proj, w["cols"][:3], H, G, 1, D, Dv, None, None, eps, 0.0, 1, batch, kp, vp, rot_dims=key[0], cos=cos, sin=sin)
        gate = proj[:, w["cols"][3]:w["cols"][3] + H]
        window, scale = int((m.get("mask") or {}).get("size", 0)), float(m["scale"])
        if LO.attn_sweep_tile_rows(self.dtype, H, G, D, Dv, kp, vp) > 0:      # bfloat16, head sizes the one-sweep matrix-core kernel takes
            a = LO.attn_sweep(q, kp, vp, batch, H, G, D, Dv, scale, window, sink=w["sink"], gate=gate, gate_per_head=True)
        else:
            a = LO.attn_window(q, gate, kp, vp, batch, H, G, D, Dv, scale, window, 0, None, None, None, sink=w["sink"], gate_per_head=True)
        return F.linear(a, w["w_o"], w["b_o"])

    # ---- feed-forward: the addends (tensor, channel scale) its result contributes to the residual sum -----------------------------------
    def _feed_forward(self, li: int, h: torch.Tensor, h_float: Optional[torch.Tensor] = None) -> list:
        """``h_float``: the same norm output unrounded (float), when the caller has it: the router reads that."""
        f, w = self.cfg.layers[li]["mlp"], self.w.layers[li]
        if f.get("kind", "dense") == "dense":
            ff = int(f["ff"])
            return [(F.linear(LO.gated_act(F.linear(h, w["w_gu"]), 0, ff, ff, LO.ACT_GELU_TANH), w["w_down"]), w["ls2"])]
        unit = lambda c: (LO.ACT_CLAMPED_SWISH, float(c["limit"]), SWISH_ALPHA, UNIT_SHIFT)
        out = [(LO.moe_experts(h, F.linear(h_float if h_float is not None else h.float(), w["router"]), None, int(f["router"]["top"]), 1.0, w["w_gu"], w["w_down"], route="softmax_renorm",
                               renorm_eps=ROUTER_RENORM_EPS, gated=unit(f["expert"])), w["ls2"])]
        if f.get("shared") is not None:                 # the token gate multiplies the activation: down() is linear, so the result is the gated output
            fs = int(f["shared"]["ff"])
            z = F.linear(h, w["w_sh"])
            out.append((F.linear(LO.gated_act(z, 0, fs, fs, *unit(f["shared"]), row_gate=z[:, 2 * fs]), w["w_sh_down"]), w["ls2"]))
        return out

    # ---- one step ----------------------------------------------------------------------------------------------------------------------
    @torch.inference_mode()
    def forward(self, ids: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache, logit_rows: Optional[torch.Tensor] = None,
                trace: Optional[list] = None) -> torch.Tensor:
        """ids int64 [N] (the batch's rows).  Returns float logits [N, vocab], or of the rows in ``logit_rows``.  ``trace``, when a
        list, receives the residual stream after every layer run (debugging and tests)."""
        cfg, w, eps, dt = self.cfg, self.w, self.cfg.norm_eps, self.dtype
        if batch.max_pos > self.max_positions:
            raise ValueError(f"position {batch.max_pos - 1} is beyond the {self.max_positions} positions the tables were reserved for")
        x, _ = LO.embed_scale(w.embed, ids, 1.0, False)
        pending: list = []                               # the previous layer's sublayer outputs, folded into the next norms' launch
        for run, li in enumerate(self.runs):
            L, lw = cfg.layers[li], w.layers[li]
            has_ff = L.get("mlp") is not None
            routed = has_ff and L["mlp"].get("kind", "dense") == "moe"      # a router reads its norm in float, the products the activation dtype
            hs = LO.scaled_add_norms(x, pending, lw["norm1"], lw["norm2"] if has_ff else None, 1.0, eps, dt, two=has_ff, second_float=routed)
            h1, h2, h2f = (hs if routed else (*hs, None)) if has_ff else (hs, None, None)
            pending = [(self._attention(run, li, h1, batch, cache), lw["ls1"])]
            if has_ff:
                pending += self._feed_forward(li, h2, h2f)
            if trace is not None:
                LO.scaled_add_norms(x, pending, None, None, 1.0, eps, None)
                pending = []
                trace.append(x.clone())
        hf = LO.scaled_add_norms(x, pending, w.final_norm, None, 1.0, eps, dt)
        if logit_rows is not None:
            hf = hf.index_select(0, logit_rows)
        return F.linear(hf, w.head).float() * cfg.logit_scale


def load_model_directory(model_dir, device, dtype=torch.bfloat16, max_positions: int = 8192):
    cfg = BamanexConfig.from_json(Path(model_dir) / "config.json")
    return cfg, BamanexModel(cfg, BamanexWeights.from_safetensors(cfg, model_dir, device, dtype), max_positions)


def random_model(cfg: BamanexConfig, device, dtype=torch.bfloat16, max_positions: int = 8192, seed: int = 0) -> BamanexModel:
    return BamanexModel(cfg, BamanexWeights.random(cfg, device, dtype, seed), max_positions)
