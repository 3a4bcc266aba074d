"""Mikipel: a decoder with a float residual stream whose layers run their mixer and their feed-forward side by side on ONE norm of
the stream — x + m * (mixer(shift(h)) + ff(h)), h = norm1(x), m one number — and hand on not their own result but a learned
mixture of the embedding output and the results of all layers so far (``dwa``: depth-weighted average).  The mixer reads h through a
token shift, h_t + (h_(t-1) - h_t) * mu per channel; the previous token's h is part of a request's state in every layer.

* mixer ``attention``: grouped-query attention, no biases; rotary positions on the first ``rot.dims`` dimensions of every head
  (rotate-half pairs, frequencies divided by ``rot.scaling.factor``); queries and keys brought to unit RMS per head after the rotation;
  plain causal softmax.
* mixer ``latent_attention``: keys and values through a normalised latent of ``kv_rank`` plus ONE rotary key part shared by the heads
  (neighbouring dimensions form the rotation's pairs) — only these two are cached; queries straight from the input.
* mixer ``delta``: the gated delta rule — q, k, v through a short causal convolution and silu, q and k unit vectors, a decay and a step
  size per head and token, a float state per head; the output normalised per head and gated by silu.
* feed-forward ``dense``: down(gelu(up h)) with the erf gelu; ``moe``: the largest router logits (with a bias) choose ``top`` experts
  down(silu(gate h) * up h), weighted by the softmax over the chosen logits; or none.
* output: the model's norm, the embedding table itself as the head, and a tanh soft cap.

The forward runs one ragged batch (``layer_ops.RaggedBatch``): portions of prompts and single decoded tokens side by side, over
``engine.state_cache.PagedStateCache``.  Dense products are torch's (hipBLASLt / rocBLAS); everything else is a launch of
``libjf_layers.so`` / ``libjf_layers_seq.so``.  A layer's sublayer outputs are folded into the launch that stores its result, mixes
the depths and forms the next layer's norm — and, in a step of single tokens, its token shift.  With float32 weights every product is a true 32-bit one."""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Dict, List, Optional

import torch
import torch.nn.functional as F

from .. import layer_ops as LO
from ..engine.state_cache import PagedStateCache, RunSpec

MIXERS = ("attention", "latent_attention", "delta")
UNIT_EPS = 1e-6                      # inside the root of the delta rule's unit vectors (a constant of the design)
MAX_TAPS = 8


@dataclass
class MikipelConfig:
    vocab_size: int
    hidden_size: int
    layers: List[Dict[str, Any]]
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    residual_mult: float = 1.0
    logit_softcap: float = 0.0                      # 0: no cap
    max_position_embeddings: int = 1 << 20          # the design has no limit of its own: the engine's max_model_len decides
    eos_token_id: int = -1
    pad_token_id: int = 0
    family: str = "ragged"

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MikipelConfig":
        for i, L in enumerate(d["layers"]):
            if L["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer {L['type']!r}")
            m = L["mixer"]
            if L["type"] in ("attention", "delta") and int(m["heads"]) % int(m.get("kv_heads", m["heads"])):
                raise ValueError(f"layer {i}: {m['heads']} heads over {m['kv_heads']} key heads")
            if L["type"] != "delta":
                dims = int((m.get("rot") or {}).get("dims", 0))
                limit = int(m["dim"] if L["type"] == "attention" else m["rot_dim"])
                if dims % 2 or dims > limit:
                    raise ValueError(f"layer {i}: rot.dims {dims} must be even and at most {limit}")
            elif not 1 <= int(m.get("conv", 1)) <= MAX_TAPS:
                raise ValueError(f"layer {i}: a convolution of {m['conv']} taps (1 .. {MAX_TAPS} are served)")
            f = L.get("mlp")
            if f is not None and f.get("kind", "dense") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward {f.get('kind')!r}")
            if f is not None and f.get("kind") == "moe" and not 1 <= int(f["router"]["top"]) <= int(f["router"]["experts"]):
                raise ValueError(f"layer {i}: top {f['router']['top']} of {f['router']['experts']} experts")
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), layers=d["layers"], norm_eps=float(d["norm"]["eps"]),
                   embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)), residual_mult=float(d.get("residual_mult", 1.0)),
                   logit_softcap=float(d.get("logit_softcap") or 0.0), eos_token_id=int(d.get("eos_token_id", -1)),
                   pad_token_id=int(d.get("pad_token_id", 0)))

    @classmethod
    def from_json(cls, path) -> "MikipelConfig":
        return cls.from_dict(json.loads(Path(path).read_text()))


def _rot_key(m: Dict[str, Any]):
    rot = m.get("rot") or {}
    return int(rot.get("dims", 0)), float(rot.get("base", 10000.0)), float((rot.get("scaling") or {}).get("factor", 1.0))


def _delta_sizes(m: Dict[str, Any]):
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    return H, int(m.get("kv_heads", H)), D, Dv, int(m.get("conv", 1))


class MikipelWeights:
    """Tensors by their checkpoint names (``embed``, ``l<i>.norm1``, ``l<i>.shift``, ``l<i>.dwa``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
    ``final.norm``), regrouped per layer for the forward: a mixer's input projections stacked into one matrix (ending with zero rows up
    to a multiple of eight, so that the product's rows start at 16-byte borders), the latent up-projections per head ([H, D, R] for keys,
    [H, R, Dv] for values), the three convolutions' taps stacked like their channels, every expert's gate rows on its up rows
    ([E, 2*ff, W]); norm weights, shift, depth weights, decay constants and the router in float."""

    def __init__(self, cfg: MikipelConfig, tensors: Dict[str, torch.Tensor], device, dtype=torch.bfloat16):
        dev = torch.device(device)
        act = lambda k: tensors[k].to(device=dev, dtype=dtype).contiguous()
        f32 = lambda k: tensors[k].to(device=dev, dtype=torch.float32).reshape(-1).contiguous()
        self.device, self.dtype = dev, dtype
        W = cfg.hidden_size
        self.embed, self.final_norm = act("embed"), f32("final.norm")
        if tuple(self.embed.shape) != (cfg.vocab_size, W):
            raise ValueError(f"embed is {tuple(self.embed.shape)}, config says {(cfg.vocab_size, W)}")
        self.layers = []

        def stack(i, names, want):
            rows = torch.cat([act(n) for n in names], 0)
            if rows.shape != (want, W):
                raise ValueError(f"layer {i}: the mixer's input projections are {tuple(rows.shape)}, the config's sizes give {(want, W)}")
            return torch.cat([rows, torch.zeros(((-want) % 8, W), dtype=dtype, device=dev)], 0) if want % 8 else rows

        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L["mixer"]
            w = dict(norm1=f32(p + "norm1"), shift=f32(p + "shift"), dwa=f32(p + "dwa"), w_o=act(p + "mix.o"))
            if w["dwa"].numel() != i + 2 or w["shift"].numel() != W or w["norm1"].numel() != W:
                raise ValueError(f"layer {i}: norm1 / shift have {W} entries and dwa {i + 2}")
            if L["type"] == "attention":
                H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
                w.update(w_in=stack(i, [p + "mix.q", p + "mix.k", p + "mix.v"], H * D + G * D + G * Dv), cols=(0, H * D, H * D + G * D))
                out_in = H * Dv
            elif L["type"] == "latent_attention":
                H, D, rd, Dv, R = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
                w.update(w_in=stack(i, [p + "mix.q", p + "mix.dkv"], H * (D + rd) + R + rd), kv_col=H * (D + rd), dkv_norm=act(p + "mix.dkv.norm"),
                         w_uk=act(p + "mix.uk").view(H, D, R).contiguous(), w_uv=act(p + "mix.uv").view(H, Dv, R).transpose(1, 2).contiguous())
                if w["dkv_norm"].numel() != R:
                    raise ValueError(f"layer {i}: dkv.norm has {w['dkv_norm'].numel()} entries, kv_rank is {R}")
                out_in = H * Dv
            else:
                H, G, D, Dv, taps = _delta_sizes(m)
                C_ = 2 * G * D + H * Dv
                w.update(w_in=stack(i, [p + "mix.q", p + "mix.k", p + "mix.v", p + "mix.g", p + "mix.a", p + "mix.b"], C_ + H * Dv + 2 * H),
                         pcols=(C_ + H * Dv, C_ + H * Dv + H, C_), conv=torch.cat([act(p + "mix.q.conv"), act(p + "mix.k.conv"), act(p + "mix.v.conv")], 0).contiguous(),
                         a_log=f32(p + "mix.A_log"), dt_bias=f32(p + "mix.dt_bias"), out_norm=f32(p + "mix.norm"))
                if tuple(w["conv"].shape) != (C_, taps) or w["a_log"].numel() != H or w["dt_bias"].numel() != H or w["out_norm"].numel() != Dv:
                    raise ValueError(f"layer {i}: the delta mixer's tensors do not fit heads={H} kv_heads={G} dim={D} vdim={Dv} conv={taps}")
                out_in = H * Dv
            if tuple(w["w_o"].shape) != (W, out_in):
                raise ValueError(f"layer {i}: mix.o is {tuple(w['w_o'].shape)}, the config's sizes give {(W, out_in)}")
            f = L.get("mlp")
            if f is not None and f.get("kind", "dense") == "dense":
                w.update(w_up=act(p + "mlp.up"), w_down=act(p + "mlp.down"))
                if tuple(w["w_up"].shape) != (int(f["ff"]), W):
                    raise ValueError(f"layer {i}: mlp.up is {tuple(w['w_up'].shape)}, config says ff {f['ff']}")
            elif f is not None:
                E, ff = int(f["router"]["experts"]), int(f["expert"]["ff"])
                w.update(router=tensors[p + "mlp.router"].to(device=dev, dtype=torch.float32).contiguous(), router_b=f32(p + "mlp.router.b"),
                         w_gu=torch.stack([torch.cat([act(p + f"mlp.e{e}.gate"), act(p + f"mlp.e{e}.up")], 0) for e in range(E)]).contiguous(),
                         w_down=torch.stack([act(p + f"mlp.e{e}.down") for e in range(E)]).contiguous())
                if tuple(w["w_gu"].shape) != (E, 2 * ff, W) or tuple(w["router"].shape) != (E, W) or w["router_b"].numel() != E:
                    raise ValueError(f"layer {i}: experts are {tuple(w['w_gu'].shape)}, config says {E} experts of ff {ff}")
            self.layers.append(w)

    @classmethod
    def from_safetensors(cls, cfg: MikipelConfig, model_dir, device, dtype=torch.bfloat16) -> "MikipelWeights":
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
    def random(cls, cfg: MikipelConfig, device, dtype=torch.bfloat16, seed: int = 0) -> "MikipelWeights":
        return cls(cfg, random_tensors(cfg, seed), device, dtype)


def random_tensors(cfg: MikipelConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Random tensors under the checkpoint's names (benchmarks and tests; bf16-representable float32 values)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.hidden_size
    rnd = lambda *s, std=1.0: (torch.randn(*s, generator=g) * std).to(torch.bfloat16).float()
    uni = lambda *s, lo=0.0, hi=1.0: (lo + (hi - lo) * torch.rand(*s, generator=g)).to(torch.bfloat16).float()
    lin = lambda o, i: rnd(o, i, std=i ** -0.5)
    one = lambda *s: (1 + torch.randn(*s, generator=g) * 0.1).to(torch.bfloat16).float()
    t = {"embed": rnd(cfg.vocab_size, W, std=W ** -0.5), "final.norm": one(W)}
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L["mixer"]
        dwa = rnd(i + 2, std=0.2)
        dwa[-1] += 1.0
        t.update({p + "norm1": one(W), p + "shift": uni(W), p + "dwa": dwa.to(torch.bfloat16).float()})
        if L["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            t.update({p + "mix.q": lin(H * D, W), p + "mix.k": lin(G * D, W), p + "mix.v": lin(G * Dv, W), p + "mix.o": lin(W, H * Dv)})
        elif L["type"] == "latent_attention":
            H, D, rd, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            t.update({p + "mix.q": lin(H * (D + rd), W), p + "mix.dkv": lin(R + rd, W), p + "mix.dkv.norm": one(R), p + "mix.uk": lin(H * D, R),
                      p + "mix.uv": lin(H * Dv, R), p + "mix.o": lin(W, H * Dv)})
        else:
            H, G, D, Dv, taps = _delta_sizes(m)
            t.update({p + "mix.q": lin(G * D, W), p + "mix.k": lin(G * D, W), p + "mix.v": lin(H * Dv, W), p + "mix.g": lin(H * Dv, W),
                      p + "mix.a": lin(H, W), p + "mix.b": lin(H, W), p + "mix.o": lin(W, H * Dv), p + "mix.norm": one(Dv),
                      p + "mix.A_log": uni(H, lo=-3.0, hi=1.0), p + "mix.dt_bias": rnd(H, std=1.0)})
            for k, c in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                t[p + f"mix.{k}.conv"] = rnd(c, taps, std=0.5)
        f = L.get("mlp")
        if f is None:
            continue
        if f.get("kind", "dense") == "dense":
            t.update({p + "mlp.up": lin(f["ff"], W), p + "mlp.down": lin(W, f["ff"])})
            continue
        E, ff = f["router"]["experts"], f["expert"]["ff"]
        t.update({p + "mlp.router": lin(E, W) * 2, p + "mlp.router.b": rnd(E, std=0.5)})
        for e in range(E):
            t.update({p + f"mlp.e{e}.gate": lin(ff, W), p + f"mlp.e{e}.up": lin(ff, W), p + f"mlp.e{e}.down": lin(W, ff)})
    return t


class MikipelModel:
    def __init__(self, cfg: MikipelConfig, weights: MikipelWeights, max_positions: int = 8192):
        self.cfg, self.w = cfg, weights
        self.device, self.dtype = weights.device, weights.dtype
        self._angles: Dict[tuple, tuple] = {}
        self.max_positions = 0
        self.reserve_positions(max_positions)

    # ---- what the cache must hold, one entry per layer: every layer carries the previous token's norm output (the token shift) ----------
    def cache_specs(self) -> List[RunSpec]:
        W, specs = self.cfg.hidden_size, []
        for L in self.cfg.layers:
            m, tails = L["mixer"], {"shift": (1, W)}
            if L["type"] == "attention":
                specs.append(RunSpec("kv", k_width=int(m["kv_heads"]) * int(m["dim"]), v_width=int(m["kv_heads"]) * int(m["vdim"]), tails=tails))
            elif L["type"] == "latent_attention":      # the latent and the shared rotary key; values are read out of the same rows
                specs.append(RunSpec("kv", k_width=int(m["kv_rank"]) + int(m["rot_dim"]), v_width=0, tails=tails))
            else:                                       # the float state per head, and the convolutions' last inputs
                H, G, D, Dv, taps = _delta_sizes(m)
                if taps > 1:
                    tails["conv"] = (taps - 1, 2 * G * D + H * Dv)
                specs.append(RunSpec("state", state_shape=(H, D, Dv), tails=tails))
        return specs

    def new_cache(self, num_pages: int, page_size: int, num_slots: int) -> PagedStateCache:
        return PagedStateCache(self.cache_specs(), num_pages, page_size, num_slots, self.device, self.dtype)

    # ---- rotation angles for every position the engine can reach: position * (frequency / factor), cosine and sine, all in float32 -------
    def reserve_positions(self, n: int) -> None:
        if n <= self.max_positions:
            return
        self.max_positions = int(n)
        self._angles.clear()
        for L in self.cfg.layers:
            if L["type"] == "delta":
                continue
            key = _rot_key(L["mixer"])
            if key[0] and key not in self._angles:
                dims, base, factor = key
                f = torch.tensor([base ** (-2.0 * k / dims) / factor for k in range(dims // 2)], dtype=torch.float32, device=self.device)
                a = torch.arange(n, dtype=torch.float32, device=self.device).view(n, 1) * f.view(1, -1)
                self._angles[key] = (a.cos().contiguous(), a.sin().contiguous())

    def _tables(self, m):
        key = _rot_key(m)
        return (key[0], *self._angles[key]) if key[0] else (0, None, None)

    # ---- mixers ------------------------------------------------------------------------------------------------------------------------
    def _attention(self, li: int, h: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache) -> torch.Tensor:
        m, w, eps = self.cfg.layers[li]["mixer"], self.w.layers[li], self.cfg.norm_eps
        H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        dims, cos, sin = self._tables(m)
        proj = F.linear(h, w["w_in"])
        kp, vp, scale = cache.k[li], cache.v[li], float(m["scale"])
        q = LO.head_norm_append(proj, w["cols"], H, G, 1, D, Dv, None, None, eps, 0.0, 1, batch, kp, vp, rot_dims=dims, cos=cos, sin=sin)
        if LO.attn_sweep_tile_rows(self.dtype, H, G, D, Dv, kp, vp) > 0:      # bfloat16, head sizes the one-sweep matrix-core kernel takes
            return LO.attn_sweep(q, kp, vp, batch, H, G, D, Dv, scale, 0)
        return LO.attn_window(q, None, kp, vp, batch, H, G, D, Dv, scale, 0, 0, None, None, None)

    def _latent_attention(self, li: int, h: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache) -> torch.Tensor:
        m, w, eps = self.cfg.layers[li]["mixer"], self.w.layers[li], self.cfg.norm_eps
        H, D, rd, Dv, R = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        dims, cos, sin = self._tables(m)
        n, pool, scale = h.shape[0], cache.k[li], float(m["scale"])
        proj = F.linear(h, w["w_in"])
        LO.latent_prep(proj, 0, 0, w["kv_col"], R, rd, dims, None, w["dkv_norm"], eps, batch, cos, sin, pool, pairing=LO.ROT_NEIGHBOURS)
        q = proj[:, :H * (D + rd)]
        qa = torch.bmm(q.view(n, H, D + rd)[:, :, :D].transpose(0, 1), w["w_uk"])                  # [H, N, R]: query . (W_uk c) = (W_uk^T query) . c
        qf = LO.latent_q_pack(qa, q, H, D, R, rd, dims, batch, cos, sin, pairing=LO.ROT_NEIGHBOURS)
        step = LO.ATTN_MAX_VALUE_WIDTH
        if LO.attn_sweep_tile_rows(self.dtype, H, 1, R + rd, R, pool, pool[:, :R]):                 # bfloat16, latents in multiples of 32 up to 512
            o = LO.attn_sweep(qf, pool, pool[:, :R], batch, H, 1, R + rd, R, scale, 0)
            ov = torch.bmm(o.view(n, H, R).transpose(0, 1), w["w_uv"])
        elif R <= step or self.dtype != torch.bfloat16:
            o = LO.attn_window(qf, None, pool, pool[:, :R], batch, H, 1, R + rd, R, scale, 0, 0, None, None, None)
            ov = torch.bmm(o.view(n, H, R).transpose(0, 1), w["w_uv"])                               # [H, N, Dv]
        else:           # a latent wider than the matrix-core kernel's value tile: a launch per column range of the latent
            ov = None
            for c0 in range(0, R, step):
                c1 = min(R, c0 + step)
                o = LO.attn_window(qf, None, pool, pool[:, c0:c1], batch, H, 1, R + rd, c1 - c0, scale, 0, 0, None, None, None)
                o = o.view(n, H, c1 - c0).transpose(0, 1)
                ov = torch.bmm(o, w["w_uv"][:, c0:c1]) if ov is None else torch.baddbmm(ov, o, w["w_uv"][:, c0:c1])
        return LO.heads_gate(ov, None)

    def _delta(self, li: int, h: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache) -> torch.Tensor:
        m, w = self.cfg.layers[li]["mixer"], self.w.layers[li]
        H, G, D, Dv, taps = _delta_sizes(m)
        proj = F.linear(h, w["w_in"])
        qkv = LO.short_conv(proj, 0, 2 * G * D + H * Dv, w["conv"], batch, cache.tails[li].get("conv"), LO.ACT_SILU)
        return LO.delta_rule(qkv, (0, G * D, 2 * G * D), proj, w["pcols"], w["a_log"], w["dt_bias"], w["out_norm"], batch, H, G, D, Dv, UNIT_EPS,
                             D ** -0.5, self.cfg.norm_eps, cache.state[li])

    # ---- feed-forward: the addends its result contributes to the residual sum -----------------------------------------------------------
    def _feed_forward(self, li: int, h: torch.Tensor, h_float: torch.Tensor) -> list:
        """``h_float``: the same norm output unrounded (float): the router reads that."""
        f, w = self.cfg.layers[li]["mlp"], self.w.layers[li]
        if f.get("kind", "dense") == "dense":
            ff = int(f["ff"])
            return [(F.linear(LO.gated_act(F.linear(h, w["w_up"]), 0, -1, ff, LO.ACT_GELU_ERF), w["w_down"]), None)]
        logits = torch.addmm(w["router_b"], h_float, w["router"].t())
        return [(LO.moe_experts(h, logits, None, int(f["router"]["top"]), 1.0, w["w_gu"], w["w_down"], route="top_softmax", gated=(LO.ACT_SILU, 0.0, 1.0, 0.0)), None)]

    # ---- one step ----------------------------------------------------------------------------------------------------------------------
    @torch.inference_mode()
    def forward(self, ids: torch.Tensor, batch: LO.RaggedBatch, cache: PagedStateCache, logit_rows: Optional[torch.Tensor] = None,
                trace: Optional[list] = None) -> torch.Tensor:
        """ids int64 [N] (the batch's rows).  Returns float logits [N, vocab], or of the rows in ``logit_rows``.  ``trace``, when a
        list, receives the stream every layer hands on (debugging and tests)."""
        cfg, w, eps, dt, mult = self.cfg, self.w, self.cfg.norm_eps, self.dtype, self.cfg.residual_mult
        if batch.max_pos > self.max_positions:
            raise ValueError(f"position {batch.max_pos - 1} is beyond the {self.max_positions} positions the tables were reserved for")
        n, W, nl = ids.numel(), cfg.hidden_size, len(cfg.layers)
        streams = torch.empty((nl + 1, n, W), dtype=torch.float32, device=self.device)      # the embedding output and every layer's own result
        LO.embed_scale(w.embed, ids, cfg.embedding_scale, False, out=streams[0])
        x, mixed = streams[0], torch.empty((n, W), dtype=torch.float32, device=self.device)
        pending: list = []                               # the previous layer's sublayer outputs, folded into the next norm's launch
        both = dt != torch.float32                       # a 16-bit norm for the products, the unrounded one for the shift and the router

        def hand_on(li: int, norm_w: Optional[torch.Tensor], out_dtype, unrounded: bool = False, shift=None):
            """Layer li - 1's result becomes stream li, the mixture of streams 0 .. li the new x; returns its norm (and, with ``shift``,
            the shifted norm from the same launch)."""
            nonlocal x, pending
            if not pending:
                return LO.depth_mix_norm(x, [], mult, None, -1, None, None, norm_w, eps, out_dtype, want_float=unrounded, shift=shift)
            r = LO.depth_mix_norm(x, pending, mult, streams, li, w.layers[li - 1]["dwa"], mixed, norm_w, eps, out_dtype, want_float=unrounded, shift=shift)
            x, pending = mixed, []
            return r

        single = max(batch.counts) == 1                  # every request brings one row (decoding): the shift rides in the norm's launch

        for li, L in enumerate(cfg.layers):
            lw = w.layers[li]
            if single:
                hs = hand_on(li, lw["norm1"], dt, unrounded=both, shift=(lw["shift"], batch, cache.tails[li]["shift"]))
                h, hf, shifted = hs if both else (hs[0], hs[0], hs[1])
            else:
                hs = hand_on(li, lw["norm1"], dt, unrounded=both)
                h, hf = hs if both else (hs, hs)
                shifted = LO.token_shift(hf, lw["shift"], batch, cache.tails[li]["shift"], dt)
            mixer = self._attention if L["type"] == "attention" else self._latent_attention if L["type"] == "latent_attention" else self._delta
            pending = [(F.linear(mixer(li, shifted, batch, cache), lw["w_o"]), None)]
            if L.get("mlp") is not None:
                pending += self._feed_forward(li, h, hf)
            if trace is not None:
                hand_on(li + 1, None, None)
                trace.append(x.clone())
        hl = hand_on(nl, w.final_norm, dt)
        if logit_rows is not None:
            hl = hl.index_select(0, logit_rows)
        z = F.linear(hl, w.embed).float()
        return LO.softcap(z, cfg.logit_softcap) if cfg.logit_softcap > 0 else z


def load_model_directory(model_dir, device, dtype=torch.bfloat16, max_positions: int = 8192):
    cfg = MikipelConfig.from_json(Path(model_dir) / "config.json")
    return cfg, MikipelModel(cfg, MikipelWeights.from_safetensors(cfg, model_dir, device, dtype), max_positions)


def random_model(cfg: MikipelConfig, device, dtype=torch.bfloat16, max_positions: int = 8192, seed: int = 0) -> MikipelModel:
    return MikipelModel(cfg, MikipelWeights.random(cfg, device, dtype, seed), max_positions)
