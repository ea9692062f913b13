"""HIP kernels of the latent-attention family against the PyTorch statements of the same ops
(theroundtaible_amd/ops/reference.py), in fp32 and bf16, at sizes that are not multiples of the
tile shapes."""
import math

import pytest
import torch

from theroundtaible_amd.models.config import LatentAttentionSpec
from theroundtaible_amd.ops import latent as L
from theroundtaible_amd.ops import reference as ref

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tol(dtype):
    return dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=2e-4, atol=2e-5)


def _rows_meta(lens, starts):
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    row_seq = torch.repeat_interleave(torch.arange(len(lens), dtype=torch.int32), torch.tensor(lens))
    pos = torch.cat([torch.arange(s, s + n) for s, n in zip(starts, lens)]).long()
    return (torch.tensor(cu, dtype=torch.int32), torch.tensor(starts, dtype=torch.int32), row_seq, pos)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W", [96, 200, 1030])
def test_scalar_norms(dtype, W):
    g = torch.Generator().manual_seed(W)
    x = torch.randn(37, W, generator=g) * 3
    y = (torch.randn(37, W, generator=g) * 2).to(dtype)
    gain = torch.tensor(1.7)
    a = L.scalar_rms_norm(x.to(DEV), gain.to(DEV), 1e-5, dtype).cpu()
    torch.testing.assert_close(a, ref.scalar_rms_norm(x, gain, 1e-5, dtype), **_tol(dtype))
    r = x.clone().to(DEV)
    L.scalar_norm_add_(r, y.to(DEV), gain.to(DEV), 1e-5)
    torch.testing.assert_close(r.cpu(), ref.scalar_norm_add_(x.clone(), y, gain, 1e-5), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_canon_norm_and_state(dtype, taps):
    g = torch.Generator().manual_seed(taps)
    W, lens, starts = 136, [9, 1, 2, 300, 1], [0, 5, 1, 17, 0]
    cu, sp, row_seq, pos = _rows_meta(lens, starts)
    x = torch.randn(sum(lens), W, generator=g)
    w = torch.randn(W, taps, generator=g) * 0.3
    conv = torch.randn(6, 2, max(taps - 1, 1), W, generator=g)
    slots = torch.tensor([4, 0, 2, 5, 1], dtype=torch.int32)
    gain = torch.tensor(0.8)
    for sub in (0, 1):
        want = ref.canon_norm(x, gain, 1e-5, w, conv[:, sub, :taps - 1], row_seq, pos, sp, slots, dtype)
        got = L.canon_norm(x.to(DEV), gain.to(DEV), 1e-5, w.to(DEV), conv.to(DEV), sub, row_seq.to(DEV), pos.to(DEV),
                           sp.to(DEV), slots.to(DEV), dtype)
        torch.testing.assert_close(got.cpu(), want, **_tol(dtype))
        cd, cc = conv.clone().to(DEV), conv.clone()
        L.canon_state_update(x.to(DEV), gain.to(DEV), 1e-5, w.to(DEV), cd, sub, cu.to(DEV), sp.to(DEV), slots.to(DEV))
        L.canon_state_update(x, gain, 1e-5, w, cc, sub, cu, sp, slots)
        torch.testing.assert_close(cd.cpu(), cc, rtol=1e-5, atol=1e-6)


def _spec(H, D, R, Dv, C, Q, rot_dims=None):
    return LatentAttentionSpec(H, D, R, Dv, C, Q, 10000.0, R if rot_dims is None else rot_dims, 1.0 / math.sqrt(D + R))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_prep(dtype):
    g = torch.Generator().manual_seed(1)
    m = _spec(3, 24, 10, 16, 72, 40, rot_dims=6)
    T, BS, NB = 50, 16, 9
    proj = torch.randn(T, m.q_rank + m.cache_row + 33, generator=g).to(dtype)
    wq, wkv = torch.rand(m.q_rank, generator=g) + 0.5, torch.rand(m.kv_rank, generator=g) + 0.5
    pos = torch.randint(0, 5000, (T,), generator=g)
    slots = torch.randperm(NB * BS, generator=g)[:T]
    c0 = torch.zeros(NB, BS, m.cache_row, dtype=dtype)
    c1 = c0.clone().to(DEV)
    want = ref.latent_prep(proj, m.q_rank, m.kv_rank, m.rot_dim, wq, wkv, 1e-5, pos, m.rot_base, m.rot_dims, c0, slots, dtype)
    got = L.latent_prep(proj.to(DEV), m, wq.to(DEV), wkv.to(DEV), 1e-5, pos.to(DEV), c1, slots.to(DEV), dtype)
    torch.testing.assert_close(got.cpu(), want, **_tol(dtype))
    torch.testing.assert_close(c1.cpu(), c0, **_tol(dtype))


def _attention_case(dtype, m, lens, starts, BS, seed, splits=1):
    g = torch.Generator().manual_seed(seed)
    cu, sp, row_seq, pos = _rows_meta(lens, starts)
    T, H, C, R = sum(lens), m.heads, m.kv_rank, m.rot_dim
    ctx = [s + n for s, n in zip(starts, lens)]
    nblk = [(c + BS - 1) // BS for c in ctx]
    NB = sum(nblk) + 3
    perm = torch.randperm(NB, generator=g).tolist()
    bt = torch.zeros(len(lens), max(nblk), dtype=torch.int32)
    at = 0
    for s, n in enumerate(nblk):
        bt[s, :n] = torch.tensor(perm[at:at + n], dtype=torch.int32)
        at += n
    cache = (torch.randn(NB, BS, C + R, generator=g) * 0.7).to(dtype)
    q_lat = torch.randn(H, T, C, generator=g).to(dtype)
    q = torch.randn(T, H, m.dim + R, generator=g).to(dtype)
    sink = torch.randn(H, generator=g)
    want = ref.latent_attention(q_lat, q, m.dim, cache, bt, cu, sp, sink, m.scale, m.rot_base, m.rot_dims, torch.float32)
    got = L.latent_attention(q_lat.to(DEV), q.to(DEV), m, cache.to(DEV), bt.to(DEV), cu.to(DEV), sp.to(DEV),
                             sink.to(DEV), num_splits=splits, out_dtype=dtype)
    torch.testing.assert_close(got.float().cpu(), want, **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 48, 32, 128), (3, 24, 10, 72), (5, 32, 0, 200), (40, 16, 8, 64), (2, 64, 32, 320),
                                   # bf16 shapes of the matrix-core kernel: latent 64 .. 512, rotary 0 .. 64, more
                                   # heads than one workgroup's 64 pairs
                                   (16, 128, 64, 512), (70, 32, 16, 64), (3, 32, 32, 192), (4, 16, 0, 256), (6, 32, 48, 384)])
def test_latent_attention_varlen(dtype, shape):
    H, D, R, C = shape
    m = _spec(H, D, R, 16, C, 32)
    _attention_case(dtype, m, [70, 1, 2, 300, 5, 1], [0, 129, 63, 17, 64, 0], 16, seed=H)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("splits", [2, 7, 32])
@pytest.mark.parametrize("shape", [(6, 32, 16, 96), (6, 32, 16, 128), (66, 16, 32, 512)])
def test_latent_attention_split_keys(dtype, splits, shape):
    H, D, R, C = shape
    m = _spec(H, D, R, 16, C, 32)
    _attention_case(dtype, m, [1, 1, 1, 1], [0, 63, 64, 700], 32, seed=splits, splits=splits)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gate_poly_softcap(dtype):
    g = torch.Generator().manual_seed(5)
    H, T, Dv = 5, 33, 24
    o = torch.randn(H, T, Dv, generator=g).to(dtype)
    proj = torch.randn(T, 17 + H * Dv, generator=g).to(dtype)
    torch.testing.assert_close(L.gate_mul(o.to(DEV), proj.to(DEV), 17, dtype).cpu(), ref.gate_mul(o, proj, 17, dtype),
                               **_tol(dtype))
    z = (torch.randn(T, 333, generator=g) * 2).to(dtype)
    coef = torch.tensor([0.7, -0.4, 0.2, 0.1])
    torch.testing.assert_close(L.poly_norm(z.to(DEV), coef.to(DEV), 1e-5, dtype).cpu(), ref.poly_norm(z, coef, 1e-5, dtype),
                               **_tol(dtype))
    lg = (torch.randn(T, 1000, generator=g) * 40).to(dtype)
    torch.testing.assert_close(L.logit_softcap(lg.to(DEV), 0.5, 30.0).cpu(), ref.logit_softcap(lg, 0.5, 30.0),
                               rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_canon_norm_shifts_state_in_decode_steps(taps):
    """One row per sequence: the fused launch gives the output AND the state of the two-launch form."""
    g = torch.Generator().manual_seed(taps)
    W, starts = 200, [0, 5, 1, 2, 300]
    cu, sp, row_seq, pos = _rows_meta([1] * 5, starts)
    x = torch.randn(5, W, generator=g)
    w = torch.randn(W, taps, generator=g) * 0.3
    conv = torch.randn(6, 2, max(taps - 1, 1), W, generator=g)
    slots = torch.tensor([4, 0, 2, 5, 1], dtype=torch.int32)
    gain = torch.tensor(0.8)
    cc = conv.clone()
    want = L.canon_norm(x, gain, 1e-5, w, cc, 1, row_seq, pos, sp, slots, torch.float32, shift_state=True)
    cd = conv.clone().to(DEV)
    got = L.canon_norm(x.to(DEV), gain.to(DEV), 1e-5, w.to(DEV), cd, 1, row_seq.to(DEV), pos.to(DEV), sp.to(DEV),
                       slots.to(DEV), torch.float32, shift_state=True)
    torch.testing.assert_close(got.cpu(), want, rtol=2e-4, atol=2e-5)
    torch.testing.assert_close(cd.cpu(), cc, rtol=1e-5, atol=1e-6)
