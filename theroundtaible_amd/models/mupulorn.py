"""Mupulorn decoder: latent attention with a softmax sink and an output gate, a causal input
convolution ahead of every sublayer, scalar-weight RMS norms around every sublayer, a PolyNorm
feed-forward, soft-capped logits. Layers are configured one by one and may run another layer's
weights (with a cache and state of their own).

Per layer (the same code for prompts, portions of prompts, single decoded tokens and any mix of
them in one batch; only the attention launch differs):

    h     = canon_norm(x)                       L1 (HIP): scalar RMS norm + conv over time (+ state)
    proj  = h @ [Wdq; Wdkv; Wg]^T               hipBLASLt, one GEMM for the three input projections
    cq    = latent_prep(proj)                   L2 (HIP): query-latent norm; KV-latent norm + rotary
                                                key part -> the paged latent cache
    q     = cq @ Wuq^T ; q_lat = q_nope . Wuk   hipBLASLt (batched over heads): the query moves
                                                into latent space, so keys are the cached rows
    o_lat = latent_attention(q_lat, q_rot)      L3 (HIP): causal, sink in the denominator, all heads
                                                of a row share each staged key tile (bf16: 32x32x16
                                                MFMA; fp32 and odd sizes: plain FMA); a decode step
                                                splits each row's keys over workgroups + a combine
    o     = gate_mul(o_lat . Wuv, proj)         hipBLASLt + L4 (HIP): sigmoid output gate
    x    += scalar_norm(o @ Wo^T)               hipBLASLt + L5 (HIP): post-norm + fp32 residual add
    h     = canon_norm(x)                       L1 (second convolution state)
    x    += scalar_norm(poly_norm(h @ Wup^T) @ Wdown^T)      hipBLASLt + L6 + L5

A decode step (one row per sequence, the launch sequence the captured graph replays) runs the five
linears on the skinny decode GEMM (shuffled weight copies, ``decode_weights``) and shifts the
convolution state inside L1; varlen steps use the library GEMMs and a separate state launch.

The residual stream, every norm, the convolution state, positions / angles, scores and softmax
are fp32 whatever the model dtype; the GEMM operands and the cache take the model dtype.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional

import torch
import torch.nn.functional as F

from ..ops import latent as L
from ..parallel.tp import TPInfo
from .config import ModelConfig
from .llama import AttnMeta


@dataclass
class _Rows:
    """Row bookkeeping of one forward, derived once from the attention metadata."""
    row_seq: torch.Tensor
    start_pos: torch.Tensor
    cu_q: torch.Tensor
    slots: torch.Tensor


class MupulornModel:
    use_skinny = True          # decode steps run their linears on the skinny decode GEMM (A/B knob)
    accepts_hidden = False
    stateful = True            # keeps a per-sequence running state beside the paged cache

    def __init__(self, cfg: ModelConfig, weights: Dict[str, torch.Tensor], device, dtype=torch.bfloat16,
                 tp: Optional[TPInfo] = None):
        self.cfg = cfg
        self.w = weights
        self.tp = tp or TPInfo()
        if self.tp.size > 1:
            raise ValueError(f"{cfg.name}: the latent cache is shared by all heads; tensor parallelism is not supported")
        self.device = torch.device(device)
        self.dtype = dtype
        if dtype == torch.float32:      # true fp32 products: no reduced-precision matrix mode
            torch.backends.cuda.matmul.allow_tf32 = False
            torch.backends.cudnn.allow_tf32 = False
        top = max((ls.mixer for ls in cfg.layers), key=lambda m: m.heads)
        self.n_heads, self.n_kv_heads, self.head_dim = top.heads, 1, cfg.head_dim
        f32 = torch.float32
        self.layers: Dict[int, Dict[str, torch.Tensor]] = {}
        for i, ls in enumerate(cfg.layers):
            if ls.source != i:
                continue
            p, m = f"l{i}.", ls.mixer
            lw = {k[len(p):]: v for k, v in weights.items() if k.startswith(p)}
            # one GEMM for the three projections that read the mixer input
            lw["w_in"] = torch.cat([lw["mix.dq"], lw["mix.dkv"], lw["mix.g"]]).contiguous()
            # per-head up-projections: q_lat[h] = q_nope[h] @ uk_h[h], o[h] = o_lat[h] @ uv_ht[h]
            lw["uk_h"] = lw["mix.uk"].view(m.heads, m.dim, m.kv_rank).contiguous()
            lw["uv_ht"] = lw["mix.uv"].view(m.heads, m.vdim, m.kv_rank).transpose(1, 2).contiguous()
            for n in ("norm1", "norm1b", "norm2", "norm2b", "mix.sink", "mlp.act", "mix.dq.norm", "mix.dkv.norm",
                      "canon1", "canon2"):
                if n in lw:
                    lw[n] = lw[n].to(f32).contiguous()
            self.layers[i] = lw
        self.final_norm = weights["final.norm"].to(f32)
        self._dec: Optional[Dict[int, Dict[str, torch.Tensor]]] = None
        self._split_ws: Optional[torch.Tensor] = None
        self._static: Dict[int, tuple] = {}
        self._ws: Dict[tuple, L.LatentWorkspace] = {}

    @property
    def kv_heads_local(self) -> int:
        return 1

    # ---- cache ------------------------------------------------------------------------------------
    def cache_row_dims(self):
        return [ls.mixer.cache_row for ls in self.cfg.layers]

    def make_cache(self, num_blocks: int, block_size: int, device, dtype, n_slots: int):
        from ..engine.kv_cache import LatentKVCache
        return LatentKVCache(self.cache_row_dims(), self.cfg.hidden, self.cfg.canon_taps, num_blocks, block_size,
                             device, dtype, n_slots=n_slots)

    def cache_bytes_per_block(self, block_size: int, dtype_bytes: int) -> int:
        return sum(self.cache_row_dims()) * block_size * dtype_bytes

    # ---- decode GEMMs -----------------------------------------------------------------------------
    _DEC_LINEARS = ("w_in", "mix.uq", "mix.o", "mlp.up", "mlp.down")

    def decode_weights(self, drop_originals: bool = False) -> Dict[int, Dict[str, torch.Tensor]]:
        """Fragment-shuffled copies of the five linears of a layer for the framework's skinny decode
        GEMM (csrc/gemm_skinny.hip: every wave load reads 1 KiB of contiguous weights), built once.
        Only on a GPU, in bf16, when the main extension is built and the shapes fit its tiles
        (K a multiple of 32, N of 16); a linear that does not fit keeps its row-major GEMM. The
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
            t = cache[rows] = L.tile_map(cu, sp, rows).to(b.cu_q.device, non_blocking=True)
        return t

    def decode_splits(self, rows: int) -> int:
        """Key ranges per decoded row: one workgroup per CU over the whole batch, at most 64 (a
        workgroup's time is its tile count; B = 8 x 4096 keys, 32 heads: 16 / 32 / 64 ranges take
        68 / 60 / 95 us with the combine — 64 ranges there are two rounds of workgroups)."""
        if self.device.type != "cuda":
            return 1
        from .. import ops
        return int(max(1, min(64, ops.device_cus(self.device) // max(1, rows))))

    def _workspace(self, rows: int, m, splits: int) -> Optional[L.LatentWorkspace]:
        if splits <= 1:
            return None
        key = (rows, m.heads, m.kv_rank, splits)
        ws = self._ws.get(key)
        if ws is None:
            ws = self._ws[key] = L.LatentWorkspace(rows, m.heads, m.kv_rank, splits, self.device)
        return ws

    def forward(self, ids: torch.Tensor, positions: torch.Tensor, kv, meta: AttnMeta,
                hidden: Optional[torch.Tensor] = None, keep_layers: Optional[list] = None) -> torch.Tensor:
        """Logits [rows, vocab] fp32: every row of a decode step, ``meta.last_rows`` of a varlen
        step (all rows when it is None). ``keep_layers``: a list that receives the residual stream
        after every layer (debugging / tests)."""
        cfg, adt = self.cfg, self.dtype
        eps = cfg.norm_eps
        T = ids.shape[0]
        b = self._rows(positions, meta)
        decode = meta.kind == "decode"
        splits = self.decode_splits(T) if decode else 1
        skinny = decode and T <= 32 and ids.is_cuda and self.use_skinny and bool(self.decode_weights())
        x = F.embedding(ids, self.w["embed"]).float()
        for l, ls in enumerate(cfg.layers):
            lw, m = self.layers[ls.source], ls.mixer
            conv, rows = kv.conv[l], kv.layer_rows(l)
            # (a decode step shifts the convolution state inside the same launch)
            h = L.canon_norm(x, lw["norm1"], eps, lw["canon1"], conv, 0, b.row_seq, positions, b.start_pos, b.slots, adt,
                             shift_state=decode)
            if not decode:
                L.canon_state_update(x, lw["norm1"], eps, lw["canon1"], conv, 0, b.cu_q, b.start_pos, b.slots)
            proj = self._linear(h, ls.source, "w_in", skinny)
            cq = L.latent_prep(proj, m, lw["mix.dq.norm"], lw["mix.dkv.norm"], eps, positions, rows,
                               meta.slot_mapping, adt)
            q = self._linear(cq, ls.source, "mix.uq", skinny).view(T, m.heads, m.dim + m.rot_dim)
            q_lat = torch.bmm(q[:, :, :m.dim].transpose(0, 1), lw["uk_h"])
            o_lat = L.latent_attention(q_lat, q, m, rows, meta.block_tables, b.cu_q, b.start_pos, lw["mix.sink"],
                                       tiles=self._tiles(meta, L.rows_per_tile(m.heads, m.kv_rank, m.rot_dim, adt), b)
                                       if x.is_cuda else None,
                                       num_splits=splits, workspace=self._workspace(T, m, splits), out_dtype=adt)
            o = torch.bmm(o_lat, lw["uv_ht"])
            og = L.gate_mul(o, proj, m.q_rank + m.cache_row, adt)
            L.scalar_norm_add_(x, self._linear(og, ls.source, "mix.o", skinny), lw["norm1b"], eps)
            if ls.ff:
                h = L.canon_norm(x, lw["norm2"], eps, lw["canon2"], conv, 1, b.row_seq, positions, b.start_pos,
                                 b.slots, adt, shift_state=decode)
                if not decode:
                    L.canon_state_update(x, lw["norm2"], eps, lw["canon2"], conv, 1, b.cu_q, b.start_pos, b.slots)
                a = L.poly_norm(self._linear(h, ls.source, "mlp.up", skinny), lw["mlp.act"], eps, adt)
                L.scalar_norm_add_(x, self._linear(a, ls.source, "mlp.down", skinny), lw["norm2b"], eps)
            if keep_layers is not None:
                keep_layers.append(x.clone())
        if not decode and meta.last_rows is not None:
            x = x.index_select(0, meta.last_rows)
        xn = L.scalar_rms_norm(x, self.final_norm, eps, adt)
        return L.logit_softcap(F.linear(xn, self.w["head"]), cfg.logit_scale, cfg.logit_softcap)
