"""Goganex decoder: pre-norm layers whose mixer reads a token-shifted input; the mixer is either
grouped-query attention (interleaved rotary pairs with rescaled frequencies, unit-RMS queries and
keys, a per-head temperature, a softmax sink of score 0) or a parallel pair — attention without
positions whose values are its unnormed keys, beside a minGRU — whose RMS-normed outputs are
averaged; a clamped gated feed-forward; a span of layers may run several times in a row with the
same weights, every run with a cache and state of its own.

Per layer run (the same code for prompts, portions of prompts, single decoded tokens and any mix
of them in one batch; only the attention launch differs):

    h, x  = shift_norm(x, pending)              H1 (HIP): pending residual add + RMS norm + token
                                                shift against the previous row / the kept state
    proj  = h @ [Wq; Wk; Wv]^T                  one GEMM for every projection that reads h
            (parallel: [Wq; Wk; Wz; Wx; Wg])
    q     = qk_prep(proj)                       H2 (HIP): rotary pairs, per-head unit RMS, keys and
                                                values -> the paged cache
    o     = gqa_attention(q)                    H3 (HIP): causal, grouped heads share each staged
                                                key tile; sink in the denominator; a decode step
                                                splits each row's keys over workgroups + a combine
    attention:  pending = o @ Wo^T
    parallel:   r = mingru_scan(proj)           H4 (HIP): gates, recurrence in fp32, output gate
                x += (norm(o @ Wo^T) + norm(r @ Wro^T)) / 2      H5 (HIP)
    h     = add_norm(x, pending)                H6 (HIP): residual add + RMS norm
    pending = limited_glu(h @ [Wgate; Wup]^T) @ Wdown^T          H7 (HIP) between two GEMMs

``pending`` is a branch output whose residual add is fused into the next norm launch. A decode
step (one row per sequence, the launch sequence the captured graph replays) runs its linears on
the skinny decode GEMM (shuffled weight copies, ``decode_weights``) and stores the shift state
inside H1; varlen steps use the library GEMMs and a separate state launch.

The residual stream, every norm, positions / angles, scores and softmax, the recurrence and its
gates are fp32 whatever the model dtype; the GEMM operands and the cache take the model dtype.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch
import torch.nn.functional as F

from ..ops import hybrid as Hy
from ..parallel.tp import TPInfo
from .config import ModelConfig, ParallelSpec, attention_of
from .llama import AttnMeta


@dataclass
class _Rows:
    """Row bookkeeping of one forward, derived once from the attention metadata."""
    row_seq: torch.Tensor
    start_pos: torch.Tensor
    cu_q: torch.Tensor
    slots: torch.Tensor


class GoganexModel:
    use_skinny = True          # decode steps run their linears on the skinny decode GEMM (A/B knob)
    fuse_adds = True           # residual adds ride in the next norm launch (A/B knob)
    matrix_attention = True    # layers whose shapes fit run the framework's matrix-core attention kernels
    accepts_hidden = False
    stateful = True            # keeps a per-sequence running state beside the paged cache

    def __init__(self, cfg: ModelConfig, weights: Dict[str, torch.Tensor], device, dtype=torch.bfloat16,
                 tp: Optional[TPInfo] = None):
        self.cfg = cfg
        self.w = weights
        self.tp = tp or TPInfo()
        if self.tp.size > 1:
            raise ValueError(f"{cfg.name}: tensor parallelism is not supported for this architecture")
        self.device = torch.device(device)
        self.dtype = dtype
        if dtype == torch.float32:      # true fp32 products: no reduced-precision matrix mode
            torch.backends.cuda.matmul.allow_tf32 = False
            torch.backends.cudnn.allow_tf32 = False
        top = max((attention_of(ls) for ls in cfg.layers), key=lambda m: m.heads)
        self.n_heads, self.n_kv_heads, self.head_dim = top.heads, top.kv_heads, top.dim
        f32 = torch.float32
        self.layers: Dict[int, Dict[str, torch.Tensor]] = {}
        for ls in cfg.layers:
            i = ls.source
            if i in self.layers:
                continue
            p = f"l{i}."
            lw = {k[len(p):]: v for k, v in weights.items() if k.startswith(p)}
            if isinstance(ls.mixer, ParallelSpec):
                # one GEMM for the five projections that read the mixer input
                lw["w_in"] = torch.cat([lw["mix.left.q"], lw["mix.left.k"], lw["mix.right.z"], lw["mix.right.x"],
                                        lw["mix.right.g"]]).contiguous()
                fp = ("mix.right.z.b", "mix.right.x.b", "mix.left.out", "mix.right.out")
            else:
                lw["w_in"] = torch.cat([lw["mix.q"], lw["mix.k"], lw["mix.v"]]).contiguous()
                fp = ("mix.temp",)
            if ls.ff:
                lw["w_gu"] = torch.cat([lw["mlp.gate"], lw["mlp.up"]]).contiguous()
            for n in ("norm1", "norm2", "shift") + fp:
                if n in lw:
                    lw[n] = lw[n].to(f32).contiguous()
            lw["inv_freq"] = Hy.rotary_table(attention_of(ls).rot, self.device)
            self.layers[i] = lw
        self.final_norm = weights["final.norm"].to(f32).contiguous()
        self._dec: Optional[Dict[int, Dict[str, torch.Tensor]]] = None
        self._split_ws: Optional[torch.Tensor] = None
        self._static: Dict[int, tuple] = {}
        self._ws: Dict[tuple, Hy.SplitWorkspace] = {}

    @property
    def kv_heads_local(self) -> int:
        return self.n_kv_heads

    # ---- cache ------------------------------------------------------------------------------------
    def cache_shapes(self):
        return [(a.kv_heads, a.dim, a.vdim) for a in map(attention_of, self.cfg.layers)]

    def matrix_layers(self, block_size: int, device, dtype):
        """Per layer run: whether its attention runs on the framework's bf16 matrix-core kernels
        (csrc/attention_prefill*.hip, attention_decode.hip, extended by the sink term): pages of
        32 tokens, equal key and value size of 64 or 128, up to 16 query heads per key / value
        head, the main extension built. Every other layer (and fp32) runs the family's own
        any-size kernel on a cache of plain rows."""
        from .. import ops
        ok = (self.matrix_attention and torch.device(device).type == "cuda" and dtype == torch.bfloat16
              and block_size == 32 and ops.native_available())
        return [bool(ok and a.dim == a.vdim and a.dim in (64, 128) and a.group <= 16 and a.scale > 0)
                for a in map(attention_of, self.cfg.layers)]

    def make_cache(self, num_blocks: int, block_size: int, device, dtype, n_slots: int):
        from ..engine.kv_cache import GroupedKVCache
        rec = [ls.mixer.right.width if isinstance(ls.mixer, ParallelSpec) else 0 for ls in self.cfg.layers]
        return GroupedKVCache(self.cache_shapes(), self.cfg.hidden, rec, num_blocks, block_size, device, dtype,
                              n_slots=n_slots, matrix_layout=self.matrix_layers(block_size, device, dtype))

    def cache_bytes_per_block(self, block_size: int, dtype_bytes: int) -> int:
        return sum(g * (dk + dv) for g, dk, dv in self.cache_shapes()) * block_size * dtype_bytes

    # ---- decode GEMMs -----------------------------------------------------------------------------
    _DEC_LINEARS = ("w_in", "mix.o", "mix.left.o", "mix.right.o", "w_gu", "mlp.down")

    def decode_weights(self, drop_originals: bool = False) -> Dict[int, Dict[str, torch.Tensor]]:
        """Fragment-shuffled copies of a layer's linears for the framework's skinny decode GEMM
        (csrc/gemm_skinny.hip: every wave load reads 1 KiB of contiguous weights), built once. Only
        on a GPU, in bf16, when the main extension is built and the shapes fit its tiles (K a
        multiple of 32, N of 16); a linear that does not fit keeps its row-major GEMM. The
        row-major tensors always stay (prompts use them): ``drop_originals`` is not honoured."""
        if self._dec is None:
            from .. import ops
            self._dec = {}
            ok = self.device.type == "cuda" and self.dtype == torch.bfloat16 and ops.native_available()
            for i, lw in self.layers.items():
                d = {}
                for n in self._DEC_LINEARS if ok else ():
                    W = lw.get(n)
                    if W is not None and W.shape[1] % 32 == 0 and W.shape[0] % 16 == 0:
                        d[n] = ops.shuffle_weight(W)
                self._dec[i] = d
            if ok:
                self._split_ws = ops.split_workspace(self.device)
        return self._dec

    def _linear(self, x: torch.Tensor, layer: int, name: str, skinny: bool) -> torch.Tensor:
        """x @ W^T: the skinny decode GEMM for a decode step of up to 32 rows, else the library GEMM."""
        if skinny:
            Ws = self._dec[layer].get(name)
            if Ws is not None:
                from .. import ops
                return ops.skinny_gemm(x, Ws, ops.PRO_PLAIN, ops.EPI_STORE, split_ws=self._split_ws,
                                       split_mode=ops.SPLIT_K | ops.SPLIT_BALANCE)
        return F.linear(x, self.layers[layer][name])

    # ---- forward ----------------------------------------------------------------------------------
    def _rows(self, positions: torch.Tensor, meta: AttnMeta) -> _Rows:
        dev = positions.device
        if meta.kind == "decode":
            B = positions.shape[0]
            st = self._static.get(B)
            if st is None:
                ar = torch.arange(B + 1, dtype=torch.int32, device=dev)
                st = self._static[B] = (ar[:B].contiguous(), ar, torch.stack([ar[:B], ar[:B]], 1).contiguous())
            return _Rows(st[0], positions.to(torch.int32), st[1], meta.state_slots)
        if meta.row_seq is None:
            lens = (meta.cu_q[1:] - meta.cu_q[:-1]).long()
            meta.row_seq = torch.repeat_interleave(torch.arange(lens.numel(), dtype=torch.int32, device=dev), lens)
        return _Rows(meta.row_seq, meta.start_pos, meta.cu_q, meta.state_slots)

    def _tiles(self, meta: AttnMeta, rows: int, b: _Rows) -> torch.Tensor:
        if meta.kind == "decode":
            return self._static[b.row_seq.shape[0]][2]
        cache = meta.latent_tiles if meta.latent_tiles is not None else {}
        meta.latent_tiles = cache
        t = cache.get(rows)
        if t is None:
            cu, sp = meta.host_rows if meta.host_rows is not None else (b.cu_q.cpu(), b.start_pos.cpu())
            t = cache[rows] = Hy.tile_map(cu, sp, rows).to(b.cu_q.device, non_blocking=True)
        return t

    def _scan_chunks(self, meta: AttnMeta, b: _Rows):
        """Work lists of the chunked recurrence scan for this batch (None: no long span)."""
        cache = meta.latent_tiles if meta.latent_tiles is not None else {}
        meta.latent_tiles = cache
        if "scan" not in cache:
            cu = meta.host_rows[0] if meta.host_rows is not None else b.cu_q.cpu()
            cache["scan"] = Hy.scan_chunks(cu, b.cu_q.device)
        return cache["scan"]

    def decode_splits(self, rows: int, kv_heads: int) -> int:
        """Key ranges per decoded row: about one workgroup per CU over rows x key/value heads."""
        if self.device.type != "cuda":
            return 1
        from .. import ops
        return int(max(1, min(64, ops.device_cus(self.device) // max(1, rows * kv_heads))))

    def _workspace(self, rows: int, a, splits: int) -> Optional[Hy.SplitWorkspace]:
        if splits <= 1:
            return None
        key = (rows, a.heads, a.vdim, splits)
        ws = self._ws.get(key)
        if ws is None:
            ws = self._ws[key] = Hy.SplitWorkspace(rows, a.heads, a.vdim, splits, self.device)
        return ws

    def _attend(self, proj, a, lw, l, positions, kv, meta, b, decode, v_off):
        """Queries / keys / values of ``proj`` -> cache -> attention output [T, heads * vdim]."""
        adt, T = self.dtype, proj.shape[0]
        if kv.matrix[l]:
            return self._attend_matrix(proj, a, lw, l, positions, kv, meta, b, decode, v_off)
        q = Hy.qk_prep(proj, a, 0, a.heads * a.dim, v_off, lw["inv_freq"], self.cfg.norm_eps, positions,
                       kv.k_layer(l), kv.v_layer(l), meta.slot_mapping, adt)
        splits = self.decode_splits(T, a.kv_heads) if decode else 1
        return Hy.gqa_attention(q, kv.k_layer(l), kv.v_layer(l), meta.block_tables, b.cu_q, b.start_pos, a.scale,
                                lw.get("mix.temp") if a.head_temp else None, a.sink,
                                tiles=self._tiles(meta, Hy.rows_per_tile(a.group), b) if proj.is_cuda else None,
                                num_splits=splits, workspace=self._workspace(T, a, splits), out_dtype=adt)

    def _attend_matrix(self, proj, a, lw, l, positions, kv, meta, b, decode, v_off):
        """The same on the framework's matrix-core kernels: the cache in their layout, the head
        temperature moved into the queries, the sink passed on."""
        from .. import ops
        T, dev = proj.shape[0], proj.device
        kc, vc = kv.k_layer(l), kv.v_layer(l)
        q = Hy.qk_prep(proj, a, 0, a.heads * a.dim, v_off, lw["inv_freq"], self.cfg.norm_eps, positions, kc, vc,
                       meta.slot_mapping, self.dtype, matrix_layout=True,
                       q_scale=lw.get("mix.temp") if a.head_temp else None)
        if decode:
            splits = ops.decode_splits(T, a.kv_heads)
            key = ("matrix", T, a.heads, a.dim, splits)
            ws = self._ws.get(key)
            if ws is None:
                ws = self._ws[key] = ops.DecodeWorkspace(T, a.heads, a.dim, splits, dev)
            o = ops.paged_attention_decode(q, kc, vc, meta.block_tables, meta.ctx_lens, a.scale, splits, ws, sink=a.sink)
        else:
            rows = ops.native().prefill_rows_per_tile(a.group, a.dim)
            cache = meta.latent_tiles if meta.latent_tiles is not None else {}
            meta.latent_tiles = cache
            tm = cache.get(("matrix", rows))
            if tm is None:
                cu, sp = meta.host_rows if meta.host_rows is not None else (b.cu_q.cpu(), b.start_pos.cpu())
                tm = cache[("matrix", rows)] = ops.prefill_tile_map(cu, rows, sp).to(dev, non_blocking=True)
            o = ops.prefill_attention(q, kc, vc, meta.block_tables, b.cu_q, b.start_pos, a.scale, tm, sink=a.sink)
        return o.reshape(T, a.heads * a.vdim)

    def forward(self, ids: torch.Tensor, positions: torch.Tensor, kv, meta: AttnMeta,
                hidden: Optional[torch.Tensor] = None, keep_layers: Optional[list] = None) -> torch.Tensor:
        """Logits [rows, vocab] fp32: every row of a decode step, ``meta.last_rows`` of a varlen
        step (all rows when it is None). ``keep_layers``: a list that receives the residual stream
        after every layer run (debugging / tests)."""
        cfg, adt = self.cfg, self.dtype
        eps = cfg.norm_eps
        T = ids.shape[0]
        b = self._rows(positions, meta)
        decode = meta.kind == "decode"
        skinny = decode and T <= 32 and ids.is_cuda and self.use_skinny and bool(self.decode_weights())
        x = F.embedding(ids, self.w["embed"]).float()
        if cfg.embed_scale != 1.0:
            x = x * cfg.embed_scale
        pend: Optional[torch.Tensor] = None     # a branch output whose residual add is still to come
        for l, ls in enumerate(cfg.layers):
            src, lw = ls.source, self.layers[ls.source]
            if pend is not None and not self.fuse_adds:
                x, pend = x + pend.float(), None
            h, x = Hy.shift_norm(x, pend, lw["norm1"], eps, lw["shift"], kv.shift[l], b.row_seq, positions, b.start_pos,
                                 b.slots, adt, shift_state=decode)
            pend = None
            if not decode:
                Hy.shift_state_update(x, lw["norm1"], eps, kv.shift[l], b.cu_q, b.slots)
            proj = self._linear(h, src, "w_in", skinny)
            if isinstance(ls.mixer, ParallelSpec):
                a, r = ls.mixer.left, ls.mixer.right
                o = self._attend(proj, a, lw, l, positions, kv, meta, b, decode, 0)
                off = (a.heads + a.kv_heads) * a.dim
                s = Hy.mingru_scan(proj, off, off + r.width, off + 2 * r.width, r.width, lw["mix.right.z.b"],
                                   lw["mix.right.x.b"], kv.rec[l], b.cu_q, b.start_pos, b.slots, adt,
                                   chunks=self._scan_chunks(meta, b) if proj.is_cuda and not decode else None)
                Hy.dual_norm_add_(x, self._linear(o, src, "mix.left.o", skinny), lw["mix.left.out"],
                                  self._linear(s, src, "mix.right.o", skinny), lw["mix.right.out"], eps)
            else:
                a = ls.mixer
                o = self._attend(proj, a, lw, l, positions, kv, meta, b, decode, (a.heads + a.kv_heads) * a.dim)
                pend = self._linear(o, src, "mix.o", skinny)
            if ls.ff:
                if pend is not None and not self.fuse_adds:
                    x, pend = x + pend.float(), None
                h = Hy.add_norm(x, pend, lw["norm2"], eps, adt)
                act = Hy.limited_glu(self._linear(h, src, "w_gu", skinny), ls.ff_limit, adt)
                pend = self._linear(act, src, "mlp.down", skinny)
            if keep_layers is not None:
                if pend is not None:
                    x, pend = x + pend.float(), None
                keep_layers.append(x.clone())
        if not decode and meta.last_rows is not None:
            x = x.index_select(0, meta.last_rows)
            pend = pend.index_select(0, meta.last_rows) if pend is not None else None
        xn = Hy.add_norm(x, pend, self.final_norm, eps, adt)
        return F.linear(xn, self.w["head"]).float()
