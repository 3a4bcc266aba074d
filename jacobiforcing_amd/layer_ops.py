"""torch-facing wrappers over ``libjf_layers.so`` (include/jf_layers.h): torch allocates and owns the memory, every operation
runs in the HIP library.  Shapes are checked here, on the host, before a launch.

A step's tokens form one ragged batch (``RaggedBatch``): N token rows, the rows of a request consecutive, with the per-request
records and tiles the kernels read."""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from . import _native as N


ATTN_SPLIT_BELOW_TILES, ATTN_SPLIT_WORKGROUPS = 128, 512     # attention: split a tile's keys while tiles x splits stays below ~2 per CU
ATTN_MAX_HEADS_ONE_LAUNCH, ATTN_MAX_VALUE_WIDTH = 16, 128   # what the matrix-core attention kernel takes in one workgroup
SWEEP_SPLIT_BELOW_GROUPS, SWEEP_SPLIT_WORKGROUPS = 512, 2048   # one-sweep attention: its workgroups are small (4 wavefronts, <= 32 rows)
SWEEP_WIDE_ROWS_PER_REQUEST = 16   # one-sweep attention: from this many tokens per request on average a step takes the 128-row tiles
RETENTION_CHUNK = 64          # tokens per chunk when a long portion's recurrence is cut into chunks that run side by side
DELTA_COLUMNS_FROM = 32       # delta rule: from this many tokens in a request's portion on, the state's columns are shared out over wavefronts


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream(device: torch.device):
    return C.c_void_p(torch.cuda.current_stream(device).cuda_stream) if device.type == "cuda" else None


def _code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return N.JL_F32
    if dt == torch.bfloat16:
        return N.JL_BF16
    raise ValueError(f"activations must be float32 or bfloat16, got {dt}")


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise ValueError(msg)


def _dev(t: torch.Tensor) -> None:
    if t.device.type != "cuda":
        raise N.NativeLibraryError("the layer kernels run on the GPU only (no CPU fallback)")


@dataclass
class RaggedBatch:
    """What one step runs: requests b = 0..B-1 with ``counts[b]`` new tokens from position ``starts[b]``, state slot ``slots[b]``
    and pages ``block_tables[b]``.  Device tensors: ``seq`` [B, 4] int32 {row0, count, pos0, slot}, ``kv_slot`` [N] int64 (pool
    token of every new row), ``tables`` [B, C] int32, ``row_req`` / ``pos`` [N] int32 (request and position of every row)."""
    B: int
    N: int
    counts: List[int]
    starts: List[int]
    seq: torch.Tensor
    kv_slot: torch.Tensor
    tables: torch.Tensor
    row_req: torch.Tensor
    pos: torch.Tensor
    page_size: int
    max_pos: int
    max_page: int
    max_slot: int
    _tiles: dict

    @classmethod
    def build(cls, counts: Sequence[int], starts: Sequence[int], slots: Sequence[int], block_tables: Sequence[Sequence[int]],
              page_size: int, device) -> "RaggedBatch":
        B = len(counts)
        row0 = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
        seq = np.stack([row0[:-1], np.asarray(counts), np.asarray(starts), np.asarray(slots)], 1).astype(np.int32).reshape(B, 4)
        C_ = max(1, max(len(t) for t in block_tables))
        bt = np.full((B, C_), -1, dtype=np.int32)
        kv = np.empty(int(row0[-1]), dtype=np.int64)
        row_pos = np.empty(int(row0[-1]), dtype=np.int32)
        for b in range(B):
            t = np.asarray(block_tables[b], dtype=np.int64)
            bt[b, :t.size] = t
            pos = starts[b] + np.arange(counts[b], dtype=np.int64)
            if counts[b] and (starts[b] + counts[b] + page_size - 1) // page_size > t.size:
                raise ValueError(f"request {b}: {t.size} pages do not hold {starts[b] + counts[b]} tokens")
            kv[row0[b]:row0[b + 1]] = t[pos // page_size] * page_size + pos % page_size
            row_pos[row0[b]:row0[b + 1]] = pos
        dev = torch.device(device)
        return cls(B=B, N=int(row0[-1]), counts=list(map(int, counts)), starts=list(map(int, starts)),
                   seq=torch.from_numpy(seq).to(dev), kv_slot=torch.from_numpy(kv).to(dev), tables=torch.from_numpy(bt).to(dev),
                   row_req=torch.from_numpy(np.repeat(np.arange(B, dtype=np.int32), np.asarray(counts, dtype=np.int64))).to(dev),
                   pos=torch.from_numpy(row_pos).to(dev),
                   page_size=int(page_size), max_pos=max(int(s) + int(c) for s, c in zip(starts, counts)), max_page=int(bt.max()),
                   max_slot=int(max(slots)), _tiles={})

    def chunks(self, size: int):
        """A portion of at least two chunks is cut into chunks of ``size`` tokens that the recurrent layers run side by side.
        None when no request of the step is that long.  Else (chunk records [chunks, 4] int32 {row0, count, pos0, chunk index},
        chunk lengths [chunks] int32, request records [B, 4] int32 {first chunk, chunks, pos0, slot})."""
        key = ("chunks", size)
        if key not in self._tiles:
            plan = None
            if max(self.counts) >= 2 * size:
                seq = self.seq.cpu().numpy()
                rec, req = [], []
                for b, (c, s) in enumerate(zip(self.counts, self.starts)):
                    req.append((len(rec), -(-c // size), s, int(seq[b, 3])))
                    for o in range(0, c, size):
                        rec.append((int(seq[b, 0]) + o, min(size, c - o), s + o, len(rec)))
                dev = self.seq.device
                rec = np.asarray(rec, dtype=np.int32).reshape(-1, 4)
                plan = (torch.from_numpy(rec).to(dev), torch.from_numpy(np.ascontiguousarray(rec[:, 1])).to(dev),
                        torch.from_numpy(np.asarray(req, dtype=np.int32).reshape(-1, 4)).to(dev))
            self._tiles[key] = plan
        return self._tiles[key]

    def tiles(self, tq: int) -> torch.Tensor:
        """[n_tiles, 4] int32 {b, first query position, count, first row}: each request's rows cut into runs of at most ``tq``."""
        t = self._tiles.get(tq)
        if t is None:
            rows, r0 = [], 0
            for b, (c, s) in enumerate(zip(self.counts, self.starts)):
                for o in range(0, c, tq):
                    rows.append((b, s + o, min(tq, c - o), r0 + o))
                r0 += c
            t = self._tiles[tq] = torch.tensor(rows, dtype=torch.int32, device=self.seq.device).reshape(-1, 4)
        return t


def embed_scale(embed: torch.Tensor, ids: torch.Tensor, scale: float, want_copy: bool,
                out: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Rows ``ids`` of ``embed`` times ``scale`` as float [N, W] (written into ``out`` when given), and a second copy with ``want_copy``."""
    _dev(embed)
    _need(embed.dim() == 2 and embed.is_contiguous() and ids.dtype == torch.int64 and ids.is_contiguous(), "embed_scale: embed [V, W], ids int64 [N]")
    n, W = ids.numel(), embed.shape[1]
    if out is not None:
        _need(out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (n, W), "embed_scale: out float [N, W]")
    x = out if out is not None else torch.empty((n, W), dtype=torch.float32, device=embed.device)
    x0 = torch.empty_like(x) if want_copy else None
    N.check_layers(N.layers().jl_embed_scale(_ptr(embed), _code(embed.dtype), _ptr(ids), n, W, float(scale), _ptr(x), _ptr(x0),
                                            _stream(embed.device)), "jl_embed_scale")
    return x, x0


def add_rmsnorm(x: torch.Tensor, y: Optional[torch.Tensor], x0: Optional[torch.Tensor], w: Optional[torch.Tensor], eps: float,
                out_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """x (float [N, W], in place) += y summed over its middle axis ([N, W] or [N, S, W], float or bf16) + x0; returns
    rms_norm(x) * w in ``out_dtype`` (None: the update only)."""
    _dev(x)
    n, W = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous(), "add_rmsnorm: x must be contiguous float32 [N, W]")
    cnt = 0
    if y is not None:
        _need(y.is_contiguous() and y.shape[0] == n and y.shape[-1] == W and y.dim() in (2, 3), "add_rmsnorm: y must be [N, W] or [N, S, W]")
        cnt = 1 if y.dim() == 2 else y.shape[1]
    if x0 is not None:
        _need(x0.shape == x.shape and x0.dtype == torch.float32 and x0.is_contiguous(), "add_rmsnorm: x0 must match x")
    out = None
    if out_dtype is not None:
        out = torch.empty((n, W), dtype=out_dtype, device=x.device)
        if w is not None:
            _need(w.dtype == out_dtype and w.numel() == W and w.is_contiguous(), "add_rmsnorm: the weight has the output's dtype and W entries")
    N.check_layers(N.layers().jl_add_rmsnorm(_ptr(x), _ptr(y), _code(y.dtype) if y is not None else 0, cnt, _ptr(x0), _ptr(w), float(eps),
                                            _ptr(out), _code(out_dtype or torch.float32), n, W, _stream(x.device)), "jl_add_rmsnorm")
    return out


def qk_norm_append(proj: torch.Tensor, cols: Tuple[int, int, int], H: int, G: int, D: int, Dv: int, wq: torch.Tensor, wk: torch.Tensor,
                   eps: float, k_cache: torch.Tensor, v_cache: torch.Tensor, kv_slot: torch.Tensor) -> torch.Tensor:
    _dev(proj)
    n, ld = proj.shape
    dt = proj.dtype
    _need(proj.is_contiguous() and kv_slot.dtype == torch.int64 and kv_slot.numel() == n, "qk_norm_append: proj [N, ld], one pool token per row")
    _need(wq.numel() == H * D and wk.numel() == G * D and wq.dtype == dt and wk.dtype == dt, "qk_norm_append: norm weights over the whole projections")
    _need(k_cache.dtype == dt and v_cache.dtype == dt and k_cache.is_contiguous() and v_cache.is_contiguous() and
          k_cache.shape[-1] == G * D and v_cache.shape[-1] == G * Dv and k_cache.shape[0] == v_cache.shape[0], "qk_norm_append: pools [tokens, G*D] / [tokens, G*Dv]")
    q = torch.empty((n, H * D), dtype=dt, device=proj.device)
    N.check_layers(N.layers().jl_qk_norm_append(_ptr(proj), _code(dt), n, ld, cols[0], cols[1], cols[2], H, G, D, Dv, _ptr(wq), _ptr(wk), float(eps),
                                               _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(kv_slot), _stream(proj.device)), "jl_qk_norm_append")
    return q


def _check_gate_sink(gate, sink, gate_per_head: bool, n: int, H: int, Dv: int, dt, what: str) -> None:
    if gate is not None:
        _need(gate.shape == (n, H if gate_per_head else H * Dv) and gate.stride(1) == 1 and gate.dtype == dt,
              f"{what}: gate [N, H*Dv], or [N, H] with one gate per head")
    if sink is not None:
        _need(sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == H, f"{what}: sink float [H]")


def attn_tile_rows(dtype: torch.dtype, H: int, G: int, D: int, Dv: int, k_ld: int = 0, v_ld: int = 0) -> int:
    tq = int(N.layers().jl_attn_tile_rows(_code(dtype), H, G, D, Dv, k_ld, v_ld))
    if tq <= 0:
        raise ValueError(f"attention sizes heads={H} kv_heads={G} dim={D} vdim={Dv} exceed the kernel's tile")
    return tq


def attn_window(q: torch.Tensor, gate: Optional[torch.Tensor], k_cache: torch.Tensor, v_cache: torch.Tensor, batch: RaggedBatch,
                H: int, G: int, D: int, Dv: int, scale: float, window: int, keep_first: int, rel: Optional[torch.Tensor],
                lut: Optional[torch.Tensor], talk: Optional[torch.Tensor], value_heads: int = 0, float_out: bool = False,
                sink: Optional[torch.Tensor] = None, gate_per_head: bool = False) -> torch.Tensor:
    """q [N, H*D]; gate a [N, H*Dv] view (column range of the projection output, row stride free; [N, H] with ``gate_per_head``) or
    None.  ``sink`` float [H]: one more term exp(sink_h) in every softmax denominator of head h.  Returns [N, H*Dv].
    The pools may be column ranges of wider rows (``v_cache`` may be a view into ``k_cache``).  ``value_heads`` (0: G) < G: key head
    c reads value head c % value_heads — several score maps over the same values.  ``float_out``: float outputs from bfloat16
    inputs (for what is subtracted or normalised next)."""
    _dev(q)
    dt = q.dtype
    n = q.shape[0]
    Gv = value_heads or G
    _need(q.is_contiguous() and q.shape[1] == H * D and n == batch.N, "attn_window: q [N, H*D] of the batch")
    _need(G % Gv == 0 and k_cache.dtype == dt and v_cache.dtype == dt and k_cache.dim() == 2 and v_cache.dim() == 2 and k_cache.shape[1] == G * D and
          v_cache.shape[1] == Gv * Dv and k_cache.stride(1) == 1 and v_cache.stride(1) == 1 and k_cache.shape[0] == v_cache.shape[0],
          "attn_window: pool dtype / widths")
    k_ld, v_ld = k_cache.stride(0), v_cache.stride(0)
    pool_tokens = k_cache.shape[0]
    _need(pool_tokens % batch.page_size == 0 and batch.max_page < pool_tokens // batch.page_size, "attn_window: a page lies outside the pool")
    _check_gate_sink(gate, sink, gate_per_head, n, H, Dv, dt, "attn_window")
    for t, shape in ((rel, None), (talk, (H, H))):
        if t is not None:
            _need(t.dtype == torch.float32 and t.is_contiguous() and (shape is None or tuple(t.shape) == shape), "attn_window: float tables")
    if rel is not None:                                  # rel [rows, H] with lut [positions] -> row, or rel [positions, H] by distance itself
        _need(rel.shape[1] == H and (lut is None or lut.dtype == torch.int32), "attn_window: rel [rows, H] (+ int32 lut)")
    tq = attn_tile_rows(dt, H, G, D, Dv, k_ld, v_ld)
    tiles = batch.tiles(tq)
    out = torch.empty((n, H * Dv), dtype=torch.float32 if float_out else dt, device=q.device)
    # few tiles with many keys (decoding): share each tile's keys out over workgroups until the chip is full
    splits, scratch = 1, None
    if tq == 32 and tiles.shape[0] < ATTN_SPLIT_BELOW_TILES:
        reach = batch.max_pos if window <= 0 else min(batch.max_pos, int(window) + int(keep_first) + tq)
        splits = max(1, min(-(-reach // 64), ATTN_SPLIT_WORKGROUPS // tiles.shape[0], 64))
        if splits > 1:
            scratch = torch.empty((int(N.layers().jl_attn_scratch_floats(tiles.shape[0], n, H, Dv, splits)),), dtype=torch.float32, device=q.device)
    q_pack = torch.empty((tiles.shape[0] * 32 * H * D,), dtype=dt, device=q.device) if tq == 32 else None
    a = N.AttnArgs(q=q.data_ptr(), gate=gate.data_ptr() if gate is not None else None, gate_ld=gate.stride(0) if gate is not None else 0,
                   k_cache=k_cache.data_ptr(), v_cache=v_cache.data_ptr(), out=out.data_ptr(), block_tables=batch.tables.data_ptr(),
                   tiles=tiles.data_ptr(), rel=rel.data_ptr() if rel is not None else None, lut=lut.data_ptr() if lut is not None else None,
                   talk=talk.data_ptr() if talk is not None else None, bt_stride=batch.tables.shape[1], n_tiles=tiles.shape[0],
                   lut_len=(lut.numel() if lut is not None else rel.shape[0]) if rel is not None else 0, page_size=batch.page_size, H=H, G=G, D=D, Dv=Dv, window=int(window),
                   keep_first=int(keep_first), TQ=tq, dtype=_code(dt), scale=float(scale), splits=splits, n_rows=n,
                   scratch=scratch.data_ptr() if scratch is not None else None,
                   q_pack=q_pack.data_ptr() if q_pack is not None else None, k_ld=k_ld, v_ld=v_ld, Gv=Gv,
                   out_dtype=N.JL_OUT_F32 if float_out and dt != torch.float32 else N.JL_OUT_SAME,
                   sink=sink.data_ptr() if sink is not None else None, gate_heads=int(gate_per_head))
    N.check_layers(N.layers().jl_attn_window(C.byref(a), _stream(q.device)), "jl_attn_window")
    return out


def attn_sweep_tile_rows(dtype: torch.dtype, H: int, G: int, D: int, Dv: int, k_cache: torch.Tensor, v_cache: torch.Tensor, value_heads: int = 0) -> int:
    """Queries per tile of the one-sweep kernel (heads in groups over a key head) for these sizes and pools; 0 when it does not
    take them."""
    if dtype != torch.bfloat16 or os.environ.get("JL_ATTN_NO_SWEEP"):                          # A/B switch for measurements
        return 0
    v_in_k = v_cache.data_ptr() == k_cache.data_ptr()
    return int(N.layers().jl_attn_sweep_tile_rows(_code(dtype), H, G, value_heads or G, D, Dv, k_cache.stride(0), v_cache.stride(0), int(v_in_k)))


def attn_sweep(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, batch: RaggedBatch, H: int, G: int, D: int, Dv: int, scale: float,
               window: int, value_heads: int = 0, float_out: bool = False, sink: Optional[torch.Tensor] = None,
               gate: Optional[torch.Tensor] = None, gate_per_head: bool = False) -> torch.Tensor:
    """Attention without bias or head mixing (``sink`` / ``gate`` as for ``attn_window``) in one sweep on the matrix cores: q [N, H*D] bfloat16, pools as for
    ``attn_window`` (column ranges of wider rows allowed); ``v_cache`` may be the first Dv columns of ``k_cache`` itself (one key
    head whose rows hold the values: the latent pool).  Returns [N, H*Dv].  Sizes as ``attn_sweep_tile_rows`` accepts them."""
    _dev(q)
    n = q.shape[0]
    Gv = value_heads or G
    _need(q.is_contiguous() and q.shape[1] == H * D and n == batch.N and H % G == 0 and G % Gv == 0, "attn_sweep: q [N, H*D] of the batch")
    _need(k_cache.dtype == q.dtype and v_cache.dtype == q.dtype and k_cache.dim() == 2 and v_cache.dim() == 2 and k_cache.shape[1] == G * D and
          v_cache.shape[1] == Gv * Dv and k_cache.stride(1) == 1 and v_cache.stride(1) == 1 and k_cache.shape[0] == v_cache.shape[0],
          "attn_sweep: pool dtype / widths")
    _need(k_cache.shape[0] % batch.page_size == 0 and batch.max_page < k_cache.shape[0] // batch.page_size, "attn_sweep: a page lies outside the pool")
    _check_gate_sink(gate, sink, gate_per_head, n, H, Dv, q.dtype, "attn_sweep")
    tq = attn_sweep_tile_rows(q.dtype, H, G, D, Dv, k_cache, v_cache, Gv)
    _need(tq > 0, f"attn_sweep: heads={H} kv_heads={G} dim={D} vdim={Dv} are not sizes of this kernel")
    tiles = batch.tiles(tq)
    out = torch.empty((n, H * Dv), dtype=torch.float32 if float_out else q.dtype, device=q.device)
    # few tiles with many keys (decoding): share each tile's keys out over workgroups until the chip is full
    groups = tiles.shape[0] * G * -(-(H // G) // 32)
    splits, scratch = 1, None
    if groups >= SWEEP_SPLIT_BELOW_GROUPS and n >= SWEEP_WIDE_ROWS_PER_REQUEST * batch.B:
        # long portions: tiles of up to 128 (query, head) rows, every wavefront keeps its rows to itself
        wide = int(N.layers().jl_attn_sweep_wide_tile_rows(_code(q.dtype), H, G, Gv, D, Dv, k_cache.stride(0), v_cache.stride(0),
                                                           int(v_cache.data_ptr() == k_cache.data_ptr())))
        if wide > 0:
            tq, tiles = wide, batch.tiles(wide)
    elif groups < SWEEP_SPLIT_BELOW_GROUPS:
        reach = batch.max_pos if window <= 0 else min(batch.max_pos, int(window) + tq)
        splits = max(1, min(-(-reach // 128), SWEEP_SPLIT_WORKGROUPS // groups, 64))
        if splits > 1:
            scratch = torch.empty((int(N.layers().jl_attn_sweep_scratch_floats(tiles.shape[0], H, G, Dv, splits)),), dtype=torch.float32, device=q.device)
    a = N.AttnArgs(q=q.data_ptr(), k_cache=k_cache.data_ptr(), v_cache=v_cache.data_ptr(), out=out.data_ptr(), block_tables=batch.tables.data_ptr(),
                   tiles=tiles.data_ptr(), bt_stride=batch.tables.shape[1], n_tiles=tiles.shape[0], page_size=batch.page_size, H=H, G=G, D=D, Dv=Dv,
                   window=int(window), TQ=tq, dtype=_code(q.dtype), scale=float(scale), n_rows=n, k_ld=k_cache.stride(0), v_ld=v_cache.stride(0), Gv=Gv,
                   splits=splits, scratch=scratch.data_ptr() if scratch is not None else None,
                   out_dtype=N.JL_OUT_F32 if float_out else N.JL_OUT_SAME, sink=sink.data_ptr() if sink is not None else None,
                   gate=gate.data_ptr() if gate is not None else None, gate_ld=gate.stride(0) if gate is not None else 0, gate_heads=int(gate_per_head))
    N.check_layers(N.layers().jl_attn_sweep(C.byref(a), _stream(q.device)), "jl_attn_sweep")
    return out


def retention(proj: torch.Tensor, cols: Tuple[int, int, int, int], batch: RaggedBatch, H: int, D: int, Dv: int, rot_dims: int,
              cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], decay: torch.Tensor, eps: float, state: torch.Tensor) -> torch.Tensor:
    """proj [N, ld] with q, k, v, gate at ``cols``; state [slots, H, D, Dv] float (updated in place).  Returns [N, H*Dv]."""
    _dev(proj)
    n, ld = proj.shape
    _need(proj.is_contiguous() and n == batch.N, "retention: proj [N, ld] of the batch")
    _need(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (H, D, Dv), "retention: state [slots, H, D, Dv] float")
    _need(batch.max_slot < state.shape[0], "retention: a slot lies outside the state")
    _need(decay.dtype == torch.float32 and decay.numel() == H, "retention: one decay per head")
    _need(max(cols[0], cols[1]) + H * D <= ld and max(cols[2], cols[3]) + H * Dv <= ld, "retention: columns do not fit the row")
    tl = 0
    if rot_dims:
        _need(cos is not None and cos.dtype == torch.float32 and cos.is_contiguous() and cos.shape == sin.shape and cos.shape[1] == rot_dims // 2,
              "retention: cos / sin [positions, rot_dims / 2] float")
        tl = cos.shape[0]
        _need(batch.max_pos <= tl, "retention: the angle tables are shorter than the batch's positions")
    out = torch.empty((n, H * Dv), dtype=proj.dtype, device=proj.device)
    L, st = N.layers(), _stream(proj.device)

    def scan(records, count, where, mode, what):
        N.check_layers(L.jl_retention(_ptr(proj), _code(proj.dtype), ld, cols[0], cols[1], cols[2], cols[3], _ptr(records), count, H, D, Dv,
                                      rot_dims, _ptr(cos), _ptr(sin), tl, _ptr(decay), float(eps), _ptr(where), _ptr(out), mode, st), what)

    plan = batch.chunks(RETENTION_CHUNK)
    if plan is None:                                    # decoded tokens and short portions: one scan per request
        scan(batch.seq, batch.B, state, 0, "jl_retention")
        return out
    chunk_rec, chunk_len, req = plan
    scratch = torch.empty((chunk_rec.shape[0], H, D, Dv), dtype=torch.float32, device=proj.device)
    scan(chunk_rec, chunk_rec.shape[0], scratch, 1, "jl_retention(local state)")
    N.check_layers(L.jl_retention_join(_ptr(req), batch.B, _ptr(chunk_len), H, D, Dv, _ptr(decay), _ptr(state), _ptr(scratch), st), "jl_retention_join")
    scan(chunk_rec, chunk_rec.shape[0], scratch, 2, "jl_retention(outputs)")
    return out


_ROUTES = {"sigmoid": N.JL_ROUTE_SIGMOID, "softmax_renorm": N.JL_ROUTE_SOFTMAX_RENORM, "top_softmax": N.JL_ROUTE_TOP_SOFTMAX}


def moe_experts(h: torch.Tensor, router_logits: torch.Tensor, correction: Optional[torch.Tensor], top: int, scale: float,
                w_up: torch.Tensor, w_down: torch.Tensor, route: str = "sigmoid", renorm_eps: float = 0.0,
                gated: Optional[Tuple[int, float, float, float]] = None) -> torch.Tensor:
    """Routed experts: h [N, W], router_logits float [N, E], w_down [E, W, ff].  Returns the weighted expert outputs per choice,
    float [N, top, W] (their sum over the middle axis is the layer's output).

    ``route`` "sigmoid": sigmoid scores, choice by score + correction, weights = score * scale; "softmax_renorm": softmax over all
    experts, the largest chosen, weights = score / (sum of the chosen + renorm_eps) * scale; "top_softmax": the largest logits chosen,
    weights = softmax over the chosen logits only, times scale.
    ``gated`` None: experts down(relu(up h)^2) with w_up [E, ff, W].  ``gated`` = (kind, limit, alpha, shift) of ``gated_act``: w_up
    [E, 2*ff, W] stacks every expert's gate rows on its linear rows, and the up product applies the unit in its epilogue."""
    _dev(h)
    n, W = h.shape
    E, ff = w_down.shape[0], w_down.shape[2]
    up_rows = 2 * ff if gated is not None else ff
    dev, dt = h.device, h.dtype
    _need(h.is_contiguous() and router_logits.dtype == torch.float32 and router_logits.is_contiguous() and tuple(router_logits.shape) == (n, E),
          "moe_experts: h [N, W], logits float [N, E]")
    _need(tuple(w_up.shape) == (E, up_rows, W) and tuple(w_down.shape) == (E, W, ff) and w_up.dtype == dt and w_down.dtype == dt and
          w_up.is_contiguous() and w_down.is_contiguous(), "moe_experts: expert weights [E, ff (2*ff when gated), W] / [E, W, ff] in the activation dtype")
    _need(route in _ROUTES and 1 <= top <= E, "moe_experts: route is 'sigmoid', 'softmax_renorm' or 'top_softmax', 1 <= top <= experts")
    if correction is not None:
        _need(correction.dtype == torch.float32 and correction.numel() == E, "moe_experts: correction float [E]")
    L, st = N.layers(), _stream(dev)
    ids = torch.empty((n, top), dtype=torch.int32, device=dev)
    wts = torch.empty((n, top), dtype=torch.float32, device=dev)
    N.check_layers(L.jl_moe_route(_ptr(router_logits), _ptr(correction), n, E, top, float(scale), _ptr(ids), _ptr(wts),
                                  _ROUTES[route], float(renorm_eps), st), "jl_moe_route")
    tm = int(L.jl_moe_tile_rows())
    rows = n * top
    max_tiles = rows // tm + E
    perm = torch.empty((rows,), dtype=torch.int32, device=dev)
    offsets = torch.empty((E + 1,), dtype=torch.int32, device=dev)
    tile_e = torch.empty((max_tiles,), dtype=torch.int32, device=dev)
    tile_r = torch.empty((max_tiles,), dtype=torch.int32, device=dev)
    N.check_layers(L.jl_moe_group(_ptr(ids), n, top, E, tm, _ptr(perm), _ptr(offsets), _ptr(tile_e), _ptr(tile_r), max_tiles, st), "jl_moe_group")
    if gated is not None and not os.environ.get("JL_MOE_UNFUSED_ACT"):          # the unit in the product's epilogue (A/B switch for measurements)
        act = torch.empty((rows, ff), dtype=dt, device=dev)
        N.check_layers(L.jl_moe_gemm_gated(_ptr(h), _ptr(w_up), _code(dt), W, ff, top, _ptr(perm), _ptr(offsets), _ptr(tile_e), _ptr(tile_r), max_tiles,
                                           int(gated[0]), float(gated[1]), float(gated[2]), float(gated[3]), _ptr(act), st), "jl_moe_gemm_gated")
    else:
        act = torch.empty((rows, up_rows), dtype=dt, device=dev)
        N.check_layers(L.jl_moe_gemm(_ptr(h), _ptr(w_up), _code(dt), N.JL_MOE_UP_PLAIN if gated is not None else N.JL_MOE_UP_RELU2, W, up_rows, top, _ptr(perm),
                                     _ptr(offsets), _ptr(tile_e), _ptr(tile_r), max_tiles, None, _ptr(act), st), "jl_moe_gemm(up)")
        if gated is not None:
            act = gated_act(act, 0, ff, ff, *gated)
    y = torch.empty((n, top, W), dtype=torch.float32, device=dev)
    N.check_layers(L.jl_moe_gemm(_ptr(act), _ptr(w_down), _code(dt), N.JL_MOE_DOWN, ff, W, top, _ptr(perm), _ptr(offsets), _ptr(tile_e), _ptr(tile_r), max_tiles,
                                 _ptr(wts), _ptr(y), st), "jl_moe_gemm(down)")
    return y


ACT_GELU_TANH, ACT_CLAMPED_SWISH, ACT_SILU, ACT_GELU_ERF, ACT_NONE = N.JL_ACT_GELU_TANH, N.JL_ACT_CLAMPED_SWISH, N.JL_ACT_SILU, N.JL_ACT_GELU_ERF, N.JL_ACT_NONE


def gated_act(z: torch.Tensor, g_col: int, u_col: int, F_: int, kind: int, limit: float = 0.0, alpha: float = 1.0, shift: float = 0.0,
              row_gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Gated activation of a feed-forward whose gate and linear branch are F_ columns each of one product z [N, ld], at g_col /
    u_col.  ACT_GELU_TANH: gelu_tanh(g) * u.  ACT_CLAMPED_SWISH: g' = min(g, limit), u' = clamp(u, +-limit), g' sigmoid(alpha g') (u' +
    shift).  ACT_SILU: g sigmoid(g) * u.  ACT_GELU_ERF: 0.5 g (1 + erf(g / sqrt 2)) * u.  ``u_col`` < 0: no linear branch (a plain
    activation of the F_ columns at g_col).  ``row_gate`` [N] or [N, 1] view (row stride free): the row is further multiplied by sigmoid(row_gate).  Returns [N, F_]."""
    _dev(z)
    u_col = -1 if u_col < 0 else u_col
    _need(z.dim() == 2 and z.stride(1) == 1 and 0 <= g_col and g_col + F_ <= z.shape[1] and u_col + F_ <= z.shape[1], "gated_act: z [N, ld] with both column ranges inside")
    n = z.shape[0]
    rg_ld = 0
    if row_gate is not None:
        _need(row_gate.dtype == z.dtype and row_gate.numel() == n and row_gate.shape[0] == n, "gated_act: one row gate per row, of z's dtype")
        rg_ld = row_gate.stride(0)
    out = torch.empty((n, F_), dtype=z.dtype, device=z.device)
    N.check_layers(N.layers().jl_gated_act(_ptr(z), _code(z.dtype), n, z.stride(0), g_col, u_col, F_, int(kind), float(limit), float(alpha), float(shift),
                                          _ptr(row_gate), rg_ld, _ptr(out), _stream(z.device)), "jl_gated_act")
    return out


def scaled_add_norms(x: torch.Tensor, addends: Sequence[Tuple[torch.Tensor, Optional[torch.Tensor]]], w1: Optional[torch.Tensor],
                     w2: Optional[torch.Tensor], w_offset: float, eps: float, out_dtype: Optional[torch.dtype], two: bool = False,
                     second_float: bool = False):
    """x (float [N, W], in place) += sum over ``addends`` (y, scale) of scale * y, y [N, W] or [N, S, W] (summed over S) float or
    bfloat16, scale float [W] or None; then, with ``out_dtype``, the RMS norm of the updated x with float weights stored around
    ``w_offset``: x / rms(x) * (w_offset + w1) — and the same with w2 when ``two`` (both sublayers of a layer read one stream).
    Returns None, the norm, or the pair of norms; with ``second_float`` (and a 16-bit ``out_dtype``) a third tensor: the second norm
    unrounded, in float (for a float router beside the experts' 16-bit products)."""
    _dev(x)
    n, W = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and len(addends) <= 3, "scaled_add_norms: x contiguous float32 [N, W], at most 3 addends")
    arr = (N.Addend * max(1, len(addends)))()
    for k, (y, sc) in enumerate(addends):
        _need(y.is_contiguous() and y.shape[0] == n and y.shape[-1] == W and y.dim() in (2, 3), "scaled_add_norms: an addend is [N, W] or [N, S, W]")
        if sc is not None:
            _need(sc.dtype == torch.float32 and sc.numel() == W and sc.is_contiguous(), "scaled_add_norms: a scale is float [W]")
        arr[k] = N.Addend(y=y.data_ptr(), dtype=_code(y.dtype), count=1 if y.dim() == 2 else y.shape[1], scale=sc.data_ptr() if sc is not None else None)
    for w in (w1, w2):
        if w is not None:
            _need(w.dtype == torch.float32 and w.numel() == W and w.is_contiguous(), "scaled_add_norms: norm weights are float [W]")
    out1 = torch.empty((n, W), dtype=out_dtype, device=x.device) if out_dtype is not None else None
    out2 = torch.empty((n, W), dtype=out_dtype, device=x.device) if out_dtype is not None and two else None
    out2f = torch.empty((n, W), dtype=torch.float32, device=x.device) if out2 is not None and second_float and out_dtype != torch.float32 else None
    N.check_layers(N.layers().jl_scaled_add_norms(_ptr(x), arr, len(addends), _ptr(w1), _ptr(w2), float(w_offset), float(eps), _ptr(out1), _ptr(out2),
                                                 _ptr(out2f), _code(out_dtype or torch.float32), n, W, _stream(x.device)), "jl_scaled_add_norms")
    if two and second_float:
        return out1, out2, out2f if out2f is not None else out2
    return (out1, out2) if two else out1


def norm_add(x: torch.Tensor, y: torch.Tensor, g: torch.Tensor, eps: float, out_dtype: Optional[torch.dtype]) -> Optional[torch.Tensor]:
    """x (float [N, W], in place) += rms_norm(y) * g, g a single float (a norm on a sublayer's OUTPUT).  Returns x in
    ``out_dtype`` (None: the update only)."""
    _dev(x)
    n, W = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous() and y.is_contiguous() and tuple(y.shape) == (n, W), "norm_add: x float [N, W], y [N, W]")
    _need(g.dtype == torch.float32 and g.numel() == 1, "norm_add: the weight is one float")
    out = torch.empty((n, W), dtype=out_dtype, device=x.device) if out_dtype is not None else None
    N.check_layers(N.layers().jl_norm_add(_ptr(x), _ptr(y), _code(y.dtype), _ptr(g), float(eps), _ptr(out), _code(out_dtype or torch.float32), n, W,
                                         _stream(x.device)), "jl_norm_add")
    return out


def polynorm(z: torch.Tensor, coef: torch.Tensor, eps: float) -> torch.Tensor:
    """c0 n(z) + c1 n(z^2) + c2 n(z^3) + c3 with n(u) = u / rms(u) over a row; z [N, F], coef four floats."""
    _dev(z)
    _need(z.dim() == 2 and z.is_contiguous() and coef.dtype == torch.float32 and coef.numel() == 4 and coef.is_contiguous(), "polynorm: z [N, F], coef float [4]")
    out = torch.empty_like(z)
    N.check_layers(N.layers().jl_polynorm(_ptr(z), _code(z.dtype), z.shape[0], z.shape[1], _ptr(coef), float(eps), _ptr(out), _stream(z.device)),
                   "jl_polynorm")
    return out


def causal_conv(x: torch.Tensor, w: torch.Tensor, batch: RaggedBatch, tail: Optional[torch.Tensor]) -> torch.Tensor:
    """x + (causal depthwise convolution of x over time, per request), from the float residual x [N, W] with w [W, taps]; ``tail``
    float [slots, taps - 1, W] carries every request's last inputs from step to step (updated here).  Returns [N, W] of w's dtype."""
    _dev(x)
    n, W = x.shape
    taps = w.shape[1]
    _need(x.dtype == torch.float32 and x.is_contiguous() and n == batch.N and w.is_contiguous() and w.shape[0] == W, "causal_conv: x float [N, W], w [W, taps]")
    if taps > 1:
        _need(tail is not None and tail.dtype == torch.float32 and tail.is_contiguous() and tuple(tail.shape[1:]) == (taps - 1, W) and
              batch.max_slot < tail.shape[0], "causal_conv: tail float [slots, taps - 1, W] with the batch's slots")
    out = torch.empty((n, W), dtype=w.dtype, device=x.device)
    L, st = N.layers(), _stream(x.device)
    N.check_layers(L.jl_causal_conv(_ptr(x), _ptr(w), _code(w.dtype), _ptr(batch.row_req), _ptr(batch.seq), _ptr(tail), n, W, taps, _ptr(out), st),
                   "jl_causal_conv")
    if taps > 1 and max(batch.counts) > 1:                  # single rows (decoding) have moved their tails in the launch above
        N.check_layers(L.jl_causal_conv_carry(_ptr(x), _ptr(batch.seq), batch.B, _ptr(tail), W, taps, st), "jl_causal_conv_carry")
    return out


def head_norm_append(proj: torch.Tensor, cols: Tuple[int, int, int], H: int, G: int, M: int, D: int, Dv: int, wq: Optional[torch.Tensor],
                     wk: Optional[torch.Tensor], eps: float, t_coef: float, t_every: int, batch: RaggedBatch, k_cache: torch.Tensor,
                     v_cache: torch.Tensor, maps_apart: bool = False, rot_dims: int = 0, cos: Optional[torch.Tensor] = None,
                     sin: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Per-head (and per score map) stage in front of attention: with ``rot_dims`` the rotation of q and k by position (rotate-half
    pairs on the first rot_dims dimensions of every head, angles from cos / sin [positions, rot_dims / 2] float), then the RMS norm
    of q and k over D (times wq / wk [D]; None: no weight), the query temperature by position, keys / values appended to the
    pools.  Returns q [N, M*H*D] map-major ([M, N, H*D] with ``maps_apart``: a contiguous query matrix per map); the key pool rows
    are [M, G, D] map-major."""
    _dev(proj)
    n, ld = proj.shape
    dt = proj.dtype
    _need(proj.is_contiguous() and n == batch.N, "head_norm_append: proj [N, ld] of the batch")
    for w in (wq, wk):
        _need(w is None or (w.numel() == D and w.dtype == dt), "head_norm_append: norm weights over one head")
    _need(rot_dims % 2 == 0 and 0 <= rot_dims <= D, "head_norm_append: the rotation takes an even number of dimensions up to D")
    _angle_tables(rot_dims, cos, sin, batch, "head_norm_append")
    _need(k_cache.dtype == dt and v_cache.dtype == dt and k_cache.is_contiguous() and v_cache.is_contiguous() and
          k_cache.shape[-1] == M * G * D and v_cache.shape[-1] == G * Dv and k_cache.shape[0] == v_cache.shape[0], "head_norm_append: pools [tokens, M*G*D] / [tokens, G*Dv]")
    q = torch.empty((M, n, H * D) if maps_apart else (n, M * H * D), dtype=dt, device=proj.device)
    N.check_layers(N.layers().jl_head_norm_append(_ptr(proj), _code(dt), n, ld, cols[0], cols[1], cols[2], H, G, M, D, Dv, _ptr(wq), _ptr(wk), float(eps),
                                                 float(t_coef), int(t_every), _ptr(batch.pos), _ptr(q), int(maps_apart), _ptr(k_cache), _ptr(v_cache),
                                                 _ptr(batch.kv_slot), int(rot_dims), _ptr(cos) if rot_dims else None, _ptr(sin) if rot_dims else None,
                                                 _stream(proj.device)), "jl_head_norm_append")
    return q


def diff_combine(a1: torch.Tensor, a2: torch.Tensor, H: int, Dv: int, lam: float, eps: float, out_scale: float, out_dtype: torch.dtype) -> torch.Tensor:
    """a1, a2 float [N, H*Dv] (two score maps' outputs; views with a common row stride) -> rms_norm_per_head(a1 - lam * a2) *
    out_scale, [N, H*Dv]."""
    _dev(a1)
    n = a1.shape[0]
    _need(a1.dtype == torch.float32 and a2.dtype == torch.float32 and tuple(a1.shape) == (n, H * Dv) and a2.shape == a1.shape and
          a1.stride(1) == 1 and a2.stride(1) == 1 and a1.stride(0) == a2.stride(0), "diff_combine: two float [N, H*Dv] with one row stride")
    out = torch.empty((n, H * Dv), dtype=out_dtype, device=a1.device)
    N.check_layers(N.layers().jl_diff_combine(_ptr(a1), _ptr(a2), a1.stride(0), n, H, Dv, float(lam), float(eps), float(out_scale), _ptr(out),
                                             _code(out_dtype), _stream(a1.device)), "jl_diff_combine")
    return out


def _angle_tables(rot_dims: int, cos, sin, batch: RaggedBatch, what: str) -> int:
    if not rot_dims:
        return 0
    _need(cos is not None and cos.dtype == torch.float32 and cos.is_contiguous() and cos.shape == sin.shape and cos.shape[1] == rot_dims // 2,
          f"{what}: cos / sin [positions, rot_dims / 2] float")
    _need(batch.max_pos <= cos.shape[0], f"{what}: the angle tables are shorter than the batch's positions")
    return cos.shape[0]


ROT_HALVES, ROT_NEIGHBOURS = N.JL_ROT_HALVES, N.JL_ROT_NEIGHBOURS      # which dimensions a rotation pairs: i with i + dims/2, or 2i with 2i + 1


def latent_prep(proj: torch.Tensor, q_col: int, Rq: int, kv_col: int, R: int, rd: int, rot_dims: int, wq: Optional[torch.Tensor], wkv: torch.Tensor,
                eps: float, batch: RaggedBatch, cos, sin, pool: torch.Tensor, pairing: int = N.JL_ROT_HALVES) -> Optional[torch.Tensor]:
    """Normalised query latent [N, Rq] (None with Rq = 0: a model without one); the pool row of every token becomes [normalised key/value
    latent | rotated shared key]."""
    _dev(proj)
    n, ld = proj.shape
    dt = proj.dtype
    _need(proj.is_contiguous() and n == batch.N and (Rq == 0 or (wq is not None and wq.numel() == Rq and wq.dtype == dt)) and wkv.numel() == R and wkv.dtype == dt,
          "latent_prep: proj [N, ld] of the batch, norm weights over the latents")
    _need(pool.dtype == dt and pool.is_contiguous() and pool.shape[-1] == R + rd, "latent_prep: pool [tokens, R + rd]")
    tl = _angle_tables(rot_dims, cos, sin, batch, "latent_prep")
    cq = torch.empty((n, Rq), dtype=dt, device=proj.device) if Rq else None
    N.check_layers(N.layers().jl_latent_prep(_ptr(proj), _code(dt), n, ld, q_col, Rq, kv_col, R, rd, rot_dims, _ptr(wq) if Rq else None, _ptr(wkv), float(eps),
                                            _ptr(batch.pos), _ptr(cos), _ptr(sin), tl, _ptr(cq), _ptr(pool), _ptr(batch.kv_slot), int(pairing),
                                            _stream(proj.device)), "jl_latent_prep")
    return cq


def latent_q_pack(qa: torch.Tensor, q: torch.Tensor, H: int, D: int, R: int, rd: int, rot_dims: int, batch: RaggedBatch, cos, sin,
                  pairing: int = N.JL_ROT_HALVES) -> torch.Tensor:
    """qa [H, N, R] (queries times the key up-projection), q [N, H*(D + rd)] (row stride free: a column range of a wider product) ->
    [N, H*(R + rd)] with the rotary part rotated."""
    _dev(q)
    n = q.shape[0]
    _need(q.stride(1) == 1 and qa.is_contiguous() and tuple(qa.shape) == (H, n, R) and q.shape[1] == H * (D + rd) and qa.dtype == q.dtype and n == batch.N,
          "latent_q_pack: qa [H, N, R], q [N, H*(D + rd)]")
    tl = _angle_tables(rot_dims, cos, sin, batch, "latent_q_pack")
    out = torch.empty((n, H * (R + rd)), dtype=q.dtype, device=q.device)
    N.check_layers(N.layers().jl_latent_q_pack(_ptr(qa), _ptr(q), q.stride(0), _code(q.dtype), n, H, D, R, rd, rot_dims, _ptr(batch.pos), _ptr(cos), _ptr(sin), tl,
                                              _ptr(out), int(pairing), _stream(q.device)), "jl_latent_q_pack")
    return out


def heads_gate(ov: torch.Tensor, gate: Optional[torch.Tensor]) -> torch.Tensor:
    """ov [H, N, Dv] -> [N, H*Dv], times sigmoid(gate) (a [N, H*Dv] view, row stride free)."""
    _dev(ov)
    H, n, Dv = ov.shape
    _need(ov.is_contiguous(), "heads_gate: ov [H, N, Dv] contiguous")
    if gate is not None:
        _need(gate.shape == (n, H * Dv) and gate.stride(1) == 1 and gate.dtype == ov.dtype, "heads_gate: gate [N, H*Dv]")
    out = torch.empty((n, H * Dv), dtype=ov.dtype, device=ov.device)
    N.check_layers(N.layers().jl_heads_gate(_ptr(ov), _ptr(gate), gate.stride(0) if gate is not None else 0, _code(ov.dtype), n, H, Dv, _ptr(out),
                                           _stream(ov.device)), "jl_heads_gate")
    return out


def _addends(addends, n: int, W: int, what: str):
    arr = (N.Addend * max(1, len(addends)))()
    for k, (y, sc) in enumerate(addends):
        _need(y.is_contiguous() and y.shape[0] == n and y.shape[-1] == W and y.dim() in (2, 3), f"{what}: an addend is [N, W] or [N, S, W]")
        if sc is not None:
            _need(sc.dtype == torch.float32 and sc.numel() == W and sc.is_contiguous(), f"{what}: a scale is float [W]")
        arr[k] = N.Addend(y=y.data_ptr(), dtype=_code(y.dtype), count=1 if y.dim() == 2 else y.shape[1], scale=sc.data_ptr() if sc is not None else None)
    return arr


def depth_mix_norm(x_in: torch.Tensor, addends: Sequence[Tuple[torch.Tensor, Optional[torch.Tensor]]], mult: float, streams: Optional[torch.Tensor],
                   depth: int, mix: Optional[torch.Tensor], x_out: Optional[torch.Tensor], w: Optional[torch.Tensor], eps: float,
                   out_dtype: Optional[torch.dtype], want_float: bool = False, shift: Optional[tuple] = None):
    """Residual update, weighted sum over the streams of all depths, RMS norm.  y = x_in + mult * sum of the addends ((tensor [N, W] or
    [N, S, W], channel scale or None), at most three).  With ``depth`` >= 0, y becomes streams[depth] (``streams`` float [depths, N, W]) and
    x_out = sum_{j <= depth} mix[j] * streams[j] (``mix`` float, at least depth + 1 entries; None: x_out = y); with ``depth`` < 0, x_out = y,
    or nothing is written when there are no addends.  Returns the norm of x_out (of x_in when nothing was written) times ``w`` (float
    [W] or None) in ``out_dtype`` — and, with ``want_float``, the same unrounded in float as a second result; None with neither.
    ``shift`` = (mu float [W], batch, tail float [slots, 1, W]): for a step in which every request brings ONE row, ``token_shift`` of the
    unrounded norm in the same launch; its result (``out_dtype``) is appended to what is returned."""
    _dev(x_in)
    n, W = x_in.shape
    _need(x_in.dtype == torch.float32 and x_in.is_contiguous() and len(addends) <= 3, "depth_mix_norm: x_in contiguous float32 [N, W], at most 3 addends")
    arr = _addends(addends, n, W, "depth_mix_norm")
    written = depth >= 0 or len(addends) > 0
    if written:
        _need(x_out is not None and x_out.dtype == torch.float32 and x_out.is_contiguous() and x_out.shape == x_in.shape, "depth_mix_norm: x_out float [N, W]")
    ld = 0
    if depth >= 0:
        _need(streams is not None and streams.dtype == torch.float32 and streams.is_contiguous() and streams.dim() == 3 and tuple(streams.shape[1:]) == (n, W) and
              depth < streams.shape[0], "depth_mix_norm: streams float [depths, N, W] with room for this depth")
        ld = n * W
        if mix is not None:
            _need(mix.dtype == torch.float32 and mix.is_contiguous() and mix.numel() >= depth + 1, "depth_mix_norm: mix float with depth + 1 entries")
    if w is not None:
        _need(w.dtype == torch.float32 and w.numel() == W and w.is_contiguous(), "depth_mix_norm: the norm weight is float [W]")
    out = torch.empty((n, W), dtype=out_dtype, device=x_in.device) if out_dtype is not None else None
    outf = torch.empty((n, W), dtype=torch.float32, device=x_in.device) if want_float else None
    mu = seq = tail = outs = None
    if shift is not None:
        mu, batch, tail = shift
        _need(out_dtype is not None and batch.N == n and batch.B == n and max(batch.counts) == 1, "depth_mix_norm: the shift in this launch needs one row per request")
        _need(mu.dtype == torch.float32 and mu.numel() == W and mu.is_contiguous() and tail.dtype == torch.float32 and tail.is_contiguous() and
              tail.numel() == tail.shape[0] * W and batch.max_slot < tail.shape[0], "depth_mix_norm: mu float [W], tail float [slots, 1, W] with the batch's slots")
        seq, outs = batch.seq, torch.empty((n, W), dtype=out_dtype, device=x_in.device)
    N.check_layers(N.layers().jl_depth_mix_norm(_ptr(x_in), arr, len(addends), float(mult), _ptr(streams) if depth >= 0 else None, ld, int(depth),
                                               _ptr(mix) if depth >= 0 else None, _ptr(x_out) if written else None, _ptr(w), float(eps), _ptr(out),
                                               _code(out_dtype or torch.float32), _ptr(outf), n, W, _ptr(mu), _ptr(seq), _ptr(tail), _ptr(outs),
                                               _stream(x_in.device)), "jl_depth_mix_norm")
    res = (out, outf) if want_float else out
    if shift is not None:
        return (*res, outs) if want_float else (res, outs)
    return res


def token_shift(h: torch.Tensor, mu: torch.Tensor, batch: RaggedBatch, tail: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """h + (h of the previous token - h) * mu: h float [N, W], mu float [W]; ``tail`` float [slots, 1, W] carries every request's last h
    from step to step (updated here; never read by a request that starts at position 0)."""
    _dev(h)
    n, W = h.shape
    _need(h.dtype == torch.float32 and h.is_contiguous() and n == batch.N and mu.dtype == torch.float32 and mu.numel() == W and mu.is_contiguous(),
          "token_shift: h float [N, W] of the batch, mu float [W]")
    _need(tail.dtype == torch.float32 and tail.is_contiguous() and tail.numel() == tail.shape[0] * W and batch.max_slot < tail.shape[0],
          "token_shift: tail float [slots, 1, W] with the batch's slots")
    out = torch.empty((n, W), dtype=out_dtype, device=h.device)
    N.check_layers(N.layers().jl_token_shift(_ptr(h), _ptr(mu), _ptr(batch.row_req), _ptr(batch.seq), _ptr(tail), n, W, _ptr(out), _code(out_dtype),
                                            _stream(h.device)), "jl_token_shift")
    return out


def softcap(z: torch.Tensor, cap: float) -> torch.Tensor:
    """cap * tanh(z / cap), in place on contiguous float z."""
    _dev(z)
    _need(z.dtype == torch.float32 and z.is_contiguous() and cap > 0, "softcap: contiguous float32 values and a positive cap")
    N.check_layers(N.layers().jl_softcap(_ptr(z), z.numel(), float(cap), _stream(z.device)), "jl_softcap")
    return z


def short_conv(x: torch.Tensor, col: int, C_: int, w: torch.Tensor, batch: RaggedBatch, tail: Optional[torch.Tensor], act: int = N.JL_ACT_SILU) -> torch.Tensor:
    """act(causal depthwise convolution over time, per request) of the columns col .. col + C_ of x [N, ld], with w [C_, taps]; float
    [N, C_].  ``tail`` float [slots, taps - 1, C_] carries every request's last inputs from step to step (updated here)."""
    _dev(x)
    n, ld = x.shape
    taps = w.shape[1]
    _need(x.is_contiguous() and n == batch.N and w.is_contiguous() and w.shape[0] == C_ and w.dtype == x.dtype and 0 <= col and col + C_ <= ld and 1 <= taps <= 8,
          "short_conv: x [N, ld] of the batch, w [C, taps <= 8] of its dtype, the columns inside the row")
    if taps > 1:
        _need(tail is not None and tail.dtype == torch.float32 and tail.is_contiguous() and tuple(tail.shape[1:]) == (taps - 1, C_) and
              batch.max_slot < tail.shape[0], "short_conv: tail float [slots, taps - 1, C] with the batch's slots")
    out = torch.empty((n, C_), dtype=torch.float32, device=x.device)
    N.check_layers(N.layers().jl_short_conv(_ptr(x), _code(x.dtype), ld, col, _ptr(w), _ptr(batch.row_req), _ptr(batch.seq), batch.B, max(batch.counts),
                                           _ptr(tail), n, C_, taps, int(act), _ptr(out), _stream(x.device)), "jl_short_conv")
    return out


def delta_rule(qkv: torch.Tensor, cols: Tuple[int, int, int], proj: torch.Tensor, pcols: Tuple[int, int, int], a_log: torch.Tensor, dt_bias: torch.Tensor,
               norm_w: torch.Tensor, batch: RaggedBatch, H: int, G: int, D: int, Dv: int, unit_eps: float, q_scale: float, eps: float,
               state: torch.Tensor) -> torch.Tensor:
    """Gated delta rule.  qkv float [N, *] holds q, k (G*D each) and v (H*Dv) at ``cols`` (after convolution and activation); proj [N, ld]
    holds the decay input a, the step input b (H each) and the gate (H*Dv) at ``pcols``; a_log, dt_bias float [H]; norm_w float [Dv];
    state [slots, H, D, Dv] float (updated in place).  Returns [N, H*Dv] of proj's dtype."""
    _dev(proj)
    n, ld = proj.shape
    _need(proj.is_contiguous() and n == batch.N and qkv.dtype == torch.float32 and qkv.is_contiguous() and qkv.shape[0] == n, "delta_rule: proj and float qkv of the batch")
    _need(H % G == 0 and max(cols[0], cols[1]) + G * D <= qkv.shape[1] and cols[2] + H * Dv <= qkv.shape[1] and max(pcols[0], pcols[1]) + H <= ld and
          pcols[2] + H * Dv <= ld, "delta_rule: columns do not fit the rows")
    _need(state.dtype == torch.float32 and state.is_contiguous() and tuple(state.shape[1:]) == (H, D, Dv) and batch.max_slot < state.shape[0],
          "delta_rule: state float [slots, H, D, Dv] with the batch's slots")
    for t, k in ((a_log, H), (dt_bias, H), (norm_w, Dv)):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.numel() == k, "delta_rule: a_log, dt_bias float [H], norm_w float [Dv]")
    out = torch.empty((n, H * Dv), dtype=proj.dtype, device=proj.device)
    long_portions = max(batch.counts) >= DELTA_COLUMNS_FROM and not os.environ.get("JL_DELTA_NO_COLUMNS")          # A/B switch for measurements
    raw = torch.empty((n, H * Dv), dtype=torch.float32, device=proj.device) if long_portions else None
    N.check_layers(N.layers().jl_delta_rule(_ptr(qkv), N.JL_F32, qkv.shape[1], cols[0], cols[1], cols[2], _ptr(proj), _code(proj.dtype), ld, pcols[0], pcols[1],
                                           pcols[2], _ptr(a_log), _ptr(dt_bias), _ptr(norm_w), _ptr(batch.seq), batch.B, n, H, G, D, Dv, float(unit_eps),
                                           float(q_scale), float(eps), _ptr(state), _ptr(raw), _ptr(out), _stream(proj.device)), "jl_delta_rule")
    return out
