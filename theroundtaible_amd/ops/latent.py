"""Ops of the latent-attention model family: scalar RMS norms, input convolutions with a running
state, the latent cache write, attention over the cached latents with a softmax sink, the output
gate, PolyNorm and the logit soft cap.

GPU tensors go to the HIP kernels of ``theroundtaible_amd._C_latent`` (``csrc/latent/``, built
in-tree by ``csrc/build.py``; :func:`ensure_built` compiles it on first use in a fresh checkout);
CPU tensors run the PyTorch statements in :mod:`.reference`. There is no silent fallback on a GPU.

Every kernel computes in fp32 and reads / writes bf16 or fp32 tensors as given; the residual
stream and the convolution state are always fp32.
"""
from __future__ import annotations

import os
import sys
from typing import Optional

import torch

from . import reference as ref

_NATIVE = None
_NATIVE_ERR: Optional[BaseException] = None

KEY_TILE = 64            # keys per attention tile (csrc/latent/latent_attention.hip)
MAX_LATENT = 512         # widest cached latent the attention kernels hold in registers


def native():
    global _NATIVE, _NATIVE_ERR
    if _NATIVE is None and _NATIVE_ERR is None:
        try:
            from .. import _C_latent  # type: ignore
            _NATIVE = _C_latent
        except BaseException as e:  # noqa: BLE001
            _NATIVE_ERR = e
    if _NATIVE is None:
        raise RuntimeError(f"theroundtaible_amd._C_latent (HIP kernels) is not built/importable: {_NATIVE_ERR}. "
                           f"Run `python csrc/build.py latent` (or __graft_entry__.build()).")
    return _NATIVE


def ensure_built(verbose: bool = False) -> None:
    """Compile the extension if it is missing or older than its sources (a fresh checkout's first
    GPU run); only this family's kernels are compiled."""
    global _NATIVE_ERR
    root = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    sys.path.insert(0, os.path.join(root, "csrc"))
    try:
        import build as csrc_build
        csrc_build.build_latent(verbose=verbose)
    finally:
        sys.path.pop(0)
    _NATIVE_ERR = None


def _gpu(t: torch.Tensor) -> bool:
    return t.is_cuda


def scalar_rms_norm(x, g, eps, out_dtype=None):
    if _gpu(x):
        out = torch.empty(x.shape, dtype=out_dtype or x.dtype, device=x.device)
        native().scalar_rms_norm(out, x.contiguous(), g, float(eps))
        return out
    return ref.scalar_rms_norm(x, g, eps, out_dtype)


def scalar_norm_add_(res, y, g, eps):
    if _gpu(res):
        native().scalar_norm_add(res, y.contiguous(), g, float(eps))
        return res
    return ref.scalar_norm_add_(res, y, g, eps)


def canon_norm(x, g, eps, w, conv, sub, row_seq, positions, start_pos, slots, out_dtype, shift_state=False):
    """``conv`` [n_slots, 2, taps - 1, W] fp32, ``sub`` 0 (mixer) / 1 (feed-forward).
    ``shift_state`` (only with ONE row per sequence, a decode step): the same launch also shifts
    every sequence's state by its row, so no :func:`canon_state_update` follows."""
    if _gpu(x):
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        native().canon_norm(out, x, g, float(eps), w, conv, int(sub), row_seq, positions, start_pos, slots,
                            bool(shift_state))
        return out
    out = ref.canon_norm(x, g, eps, w, conv[:, sub, :w.shape[1] - 1], row_seq, positions, start_pos, slots, out_dtype)
    if shift_state and w.shape[1] > 1:
        cu = torch.arange(x.shape[0] + 1, dtype=torch.int32)
        ref.canon_state_update(x, g, eps, conv[:, sub, :w.shape[1] - 1], cu, start_pos, slots)
    return out


def canon_state_update(x, g, eps, w, conv, sub, cu_q, start_pos, slots):
    """Runs AFTER :func:`canon_norm` of the same sublayer (it overwrites what that one reads)."""
    if w.shape[1] <= 1:
        return
    if _gpu(x):
        native().canon_state_update(x, g, float(eps), w, conv, int(sub), cu_q, start_pos, slots)
        return
    ref.canon_state_update(x, g, eps, conv[:, sub, :w.shape[1] - 1], cu_q, start_pos, slots)


def latent_prep(proj, spec, wq, wkv, eps, positions, cache_rows, slot_mapping, out_dtype):
    if _gpu(proj):
        cq = torch.empty(proj.shape[0], spec.q_rank, dtype=out_dtype, device=proj.device)
        native().latent_prep(cq, proj, spec.q_rank, spec.kv_rank, spec.rot_dim, wq, wkv, float(eps), positions,
                             float(spec.rot_base), spec.rot_dims, cache_rows, slot_mapping)
        return cq
    return ref.latent_prep(proj, spec.q_rank, spec.kv_rank, spec.rot_dim, wq, wkv, eps, positions, spec.rot_base,
                           spec.rot_dims, cache_rows, slot_mapping, out_dtype)


def rows_per_tile(heads: int, kv_rank: int, rot_dim: int, dtype) -> int:
    """Query rows one attention workgroup takes (all heads of each row share the staged key tile);
    the kernel's own rule (it depends on what fits the LDS)."""
    rows = int(native().latent_rows_per_tile(heads, kv_rank, rot_dim, dtype == torch.bfloat16))
    if rows <= 0:
        raise ValueError(f"latent attention: a cached row of {kv_rank + rot_dim} numbers does not fit the kernel's LDS tile")
    return rows


def tile_map(cu_q: torch.Tensor, start_pos: torch.Tensor, rows: int) -> torch.Tensor:
    """[n_tiles, 2] int32 (sequence, first row) of the varlen attention launch, heaviest first."""
    items = []
    cq, sp = cu_q.tolist(), start_pos.tolist()
    for s in range(len(sp)):
        for r in range(cq[s], cq[s + 1], rows):
            items.append((sp[s] + min(r + rows, cq[s + 1]) - cq[s], s, r))
    items.sort(key=lambda x: -x[0])
    return torch.tensor([(s, r) for _, s, r in items], dtype=torch.int32).reshape(-1, 2)


class LatentWorkspace:
    """Split-key scratch of the one-row-per-sequence (decode) attention launch: per (row, head,
    split) a partial output, running maximum and sum; static, so captured graphs can hold it."""

    def __init__(self, max_rows: int, heads: int, kv_rank: int, max_splits: int, device):
        self.max_rows, self.max_splits = max_rows, max_splits
        self.part_o = torch.empty(max_rows * heads * max_splits * kv_rank, dtype=torch.float32, device=device)
        self.part_ml = torch.empty(max_rows * heads * max_splits * 2, dtype=torch.float32, device=device)


def latent_attention(q_lat, q, spec, cache_rows, block_tables, cu_q, start_pos, sink, tiles=None,
                     num_splits: int = 1, workspace: Optional[LatentWorkspace] = None, out_dtype=None):
    """See :func:`.reference.latent_attention`. ``tiles``: :func:`tile_map` on the device (GPU);
    ``num_splits`` > 1 cuts every tile's keys into that many ranges merged by a second launch
    (one row per sequence: the decode step)."""
    out_dtype = out_dtype or q.dtype
    if _gpu(q):
        H, T, C = q_lat.shape
        if C > MAX_LATENT:
            raise ValueError(f"latent attention kernels hold at most {MAX_LATENT} latent dims per row, got {C}")
        out = torch.empty(H, T, C, dtype=out_dtype, device=q.device)
        rows = 1 if num_splits > 1 else rows_per_tile(H, C, q.shape[2] - spec.dim, q.dtype)
        if tiles is None:
            tiles = tile_map(cu_q.cpu(), start_pos.cpu(), rows).to(q.device)
        if num_splits > 1 and workspace is None:
            workspace = LatentWorkspace(T, H, C, num_splits, q.device)
        native().latent_attention(out, q_lat, q, spec.dim, cache_rows, block_tables, cu_q, start_pos, tiles, sink,
                                  float(spec.scale), float(spec.rot_base), spec.rot_dims, rows, int(num_splits),
                                  workspace.part_o if num_splits > 1 else None,
                                  workspace.part_ml if num_splits > 1 else None)
        return out
    return ref.latent_attention(q_lat, q, spec.dim, cache_rows, block_tables, cu_q, start_pos, sink, spec.scale,
                                spec.rot_base, spec.rot_dims, out_dtype)


def gate_mul(o, proj, g_off, out_dtype):
    if _gpu(o):
        H, T, Dv = o.shape
        out = torch.empty(T, H * Dv, dtype=out_dtype, device=o.device)
        native().gate_mul(out, o, proj, int(g_off))
        return out
    return ref.gate_mul(o, proj, g_off, out_dtype)


def poly_norm(z, coef, eps, out_dtype):
    if _gpu(z):
        out = torch.empty(z.shape, dtype=out_dtype, device=z.device)
        native().poly_norm(out, z.contiguous(), coef, float(eps))
        return out
    return ref.poly_norm(z, coef, eps, out_dtype)


def logit_softcap(logits, scale, cap):
    if _gpu(logits):
        out = torch.empty(logits.shape, dtype=torch.float32, device=logits.device)
        native().logit_softcap(out, logits.contiguous(), float(scale), float(cap))
        return out
    return ref.logit_softcap(logits, scale, cap)
