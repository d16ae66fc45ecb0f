"""GPU parity of the HIP layers Benarax is built from against their eager stand-ins (oracle/ref_benarax_modules.py),
layer by layer, in float32 and bfloat16, on a mixed step (prompt portions beside single rows, shuffled pages, state
slots in any order) with sizes that exercise the kernels' tails: widths that are no multiple of a vector, head sizes
between the register layouts, experts that get no row."""
import math

import pytest
import torch

import nanovllm_amd as nv
from buvalix_util import paged_context
from oracle import ref_benarax_modules as R

pytestmark = pytest.mark.gpu
DEV = "cuda"


def hip_layers():
    from nanovllm_amd.model.benarax import _default_layers
    return _default_layers()


def rel(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm().clamp_min(1e-30)).item()


def tol(dt):
    return 2e-6 if dt == torch.float32 else 1e-2


@pytest.fixture(params=[torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def dt(request):
    return request.param


@pytest.fixture
def step():
    n_q, n_k = [5, 1, 17, 2, 1], [5, 40, 30, 2, 9]
    ctx, pos = paged_context(n_q, n_k, 8, 40, 1, DEV, slots=[2, 0, 3, 1, 4])
    nv.set_context(ctx)
    yield sum(n_q), pos
    nv.set_context(None)


def rn(g, *s):
    return torch.randn(*s, generator=g).to(DEV)


@pytest.mark.parametrize("W,groups", [(96, 1), (96, 3), (100, 10), (2048, 4), (520, 13)])
def test_stream_boundary(dt, W, groups):
    L, g, T = hip_layers(), torch.Generator().manual_seed(W), 9
    x, add, parts, nm = rn(g, T, W), rn(g, T, W).to(dt), rn(g, T, 3, W), rn(g, T, W).to(dt)
    nw, w = rn(g, W), rn(g, W)
    xa, xb = x.clone(), x.clone()
    kw = dict(add=add, add_parts=parts, normed=nm, normed_weight=nw, mult=0.6, norm=w, groups=groups, eps=1e-5, out_dtype=dt,
              want_f32=True)
    ra, rb = L.stream_boundary(xa, **kw), R.stream_boundary(xb, **kw)
    assert rel(xa, xb) < 2e-6 and rel(ra[0], rb[0]) < 2e-6 and rel(ra[1], rb[1]) < tol(dt)
    xa, xb = x.clone(), x.clone()
    ca, cb = L.stream_boundary(xa, add=add, mult=0.5, copy_dtype=dt), R.stream_boundary(xb, add=add, mult=0.5, copy_dtype=dt)
    assert rel(xa, xb) < 2e-6 and rel(ca, cb) < tol(dt)
    assert rel(L.rms_norm_rows(add, w, 1e-5), R.rms_norm_rows(add, w, 1e-5)) < tol(dt)


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_causal_conv_add(dt, step, taps):
    L, g, (T, _), C = hip_layers(), torch.Generator().manual_seed(taps), step, 300
    ca, cb = L.CausalConvAdd(C, taps, device=DEV), R.CausalConvAdd(C, taps, device=DEV)
    wt = rn(g, C, taps)
    ca.weight.data.copy_(wt)
    cb.weight.data.copy_(wt)
    x, sa = rn(g, T, C), rn(g, 5, taps - 1, C)
    sb = sa.clone()
    assert rel(ca(x, sa, dt), cb(x, sb, dt)) < tol(dt)
    if taps > 1:
        assert rel(sa, sb) < 2e-6


def test_token_gate(dt):
    L, g = hip_layers(), torch.Generator().manual_seed(0)
    tab, ids, z = rn(g, 50, 70).to(dt), torch.randint(0, 50, (33,), generator=g).to(DEV), rn(g, 33, 14).to(dt)
    assert rel(L.TokenGate(28, 14)(z, tab, ids), R.TokenGate(28, 14)(z, tab, ids)) < tol(dt)


@pytest.mark.parametrize("H,D", [(3, 20), (2, 64), (1, 96), (2, 128), (1, 200)])
def test_general_delta_rule(dt, step, H, D):
    L, g, (T, _) = hip_layers(), torch.Generator().manual_seed(D), step
    da, db = L.GeneralDeltaRule(H, D, 1e-5, device=DEV), R.GeneralDeltaRule(H, D, 1e-5, device=DEV)
    for n in ("a_bias", "w_bias", "norm_weight"):
        v = rn(g, H * D)
        getattr(da, n).data.copy_(v)
        getattr(db, n).data.copy_(v)
    fused = rn(g, T, 6 * H * D).to(dt)                    # slices of one projection, as the model passes them
    r, k, v = (fused[:, i * H * D:(i + 1) * H * D].unflatten(1, (H, D)) for i in range(3))
    w_raw, a_raw, gate = (fused[:, i * H * D:(i + 1) * H * D] for i in range(3, 6))
    sa = rn(g, 5, H, D, D) * 0.3
    sb = sa.clone()
    assert rel(da(r, k, v, w_raw, a_raw, gate, sa), db(r, k, v, w_raw, a_raw, gate, sb)) < tol(dt)
    assert rel(sa, sb) < 1e-5


@pytest.mark.parametrize("H,rank,Rr,Dn,inter,scaling", [
    (4, 80, 16, 48, True, {"factor": 3.0, "fast": 16.0, "slow": 2.0, "original": 128}),     # key 96, value 80: tile kernel
    (3, 40, 8, 24, False, None),                                                            # single rows by 16-byte pieces
    (2, 64, 64, 32, False, None), (5, 18, 6, 10, True, None), (2, 192, 64, 128, True, None),
    (2, 320, 16, 40, False, None),                                                          # values wider than 256
    (2, 256, 64, 32, True, None)])                                                           # the largest tile shape (320 / 256)
@pytest.mark.parametrize("alias", [False, True], ids=["own-values", "values-in-keys"])
def test_latent_attention(dt, step, H, rank, Rr, Dn, inter, scaling, alias):
    L, g, (T, pos) = hip_layers(), torch.Generator().manual_seed(rank), step
    la = L.LatentAttention(H, rank, Rr, 0.1, 1e-5, 5000.0, scaling, interleaved=inter, device=DEV)
    lb = R.LatentAttention(H, rank, Rr, 0.1, 1e-5, 5000.0, scaling, interleaved=inter, device=DEV)
    v = rn(g, rank)
    la.latent_norm.data.copy_(v)
    lb.latent_norm.data.copy_(v)
    q, ql, ckv = rn(g, T, H, Dn + Rr).to(dt), rn(g, H, T, rank).to(dt).transpose(0, 1), rn(g, T, rank + Rr).to(dt)
    ka = rn(g, 40, 8, 1, rank + Rr).to(dt)
    kb = ka.clone()
    va, vb = (ka[..., :rank], kb[..., :rank]) if alias else (ka[..., :rank].contiguous().clone(), ka[..., :rank].contiguous().clone())
    oa, ob = la(q, ql, ckv, pos, ka, va), lb(q, ql, ckv, pos, kb, vb)
    assert rel(oa, ob) < (1e-5 if dt == torch.float32 else 2e-2)
    assert rel(ka, kb) < tol(dt) and rel(va, vb) < tol(dt)


@pytest.mark.parametrize("E,top,ff,T,W", [(14, 2, 56, 25, 96), (5, 3, 24, 25, 100), (8, 2, 40, 700, 96), (4, 4, 16, 3, 36),
                                          (12, 1, 72, 130, 256), (6, 2, 200, 2000, 128), (600, 3, 8, 40, 64), (70, 16, 8, 9, 32)])
def test_routed_experts(dt, E, top, ff, T, W):
    L, g = hip_layers(), torch.Generator().manual_seed(E)
    h, lg = rn(g, T, W).to(dt), rn(g, T, E)
    lg[:, E - 1] = -50.0                                  # an expert nobody chooses (unless every expert is chosen)
    gu, dn = (rn(g, E, 2 * ff, W) / math.sqrt(W)).to(dt), (rn(g, E, W, ff) / math.sqrt(ff)).to(dt)
    oa, ob = L.MoEExperts(top, 0.8)(h, lg, gu, dn), R.MoEExperts(top, 0.8)(h, lg, gu, dn)
    assert oa.shape == (T, top, W) and oa.dtype == torch.float32
    assert rel(oa, ob) < (1e-5 if dt == torch.float32 else 1e-2)


def test_general_delta_rule_many_pairs(dt):
    """Enough (sequence, head) pairs that every head stays in one workgroup (fewer pairs split a head's columns)."""
    L, g = hip_layers(), torch.Generator().manual_seed(3)
    B, H, D = 140, 4, 32
    n_q = [1] * (B - 2) + [3, 2]
    n_k = [q + (i % 5) for i, q in enumerate(n_q)]
    ctx, _ = paged_context(n_q, n_k, 8, 2 * B, 2, DEV, slots=list(range(B))[::-1])
    nv.set_context(ctx)
    T = sum(n_q)
    da, db = L.GeneralDeltaRule(H, D, 1e-5, device=DEV), R.GeneralDeltaRule(H, D, 1e-5, device=DEV)
    for n in ("a_bias", "w_bias", "norm_weight"):
        v = rn(g, H * D)
        getattr(da, n).data.copy_(v)
        getattr(db, n).data.copy_(v)
    r, k, v = (rn(g, T, H, D).to(dt) for _ in range(3))
    w_raw, a_raw, gate = (rn(g, T, H * D).to(dt) for _ in range(3))
    sa = rn(g, B, H, D, D) * 0.3
    sb = sa.clone()
    assert rel(da(r, k, v, w_raw, a_raw, gate, sa), db(r, k, v, w_raw, a_raw, gate, sb)) < max(tol(dt), 2e-5)
    assert rel(sa, sb) < 1e-5
    nv.set_context(None)
