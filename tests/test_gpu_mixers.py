"""GPU: every kernel of the second library against the eager stand-in of the same layer
(oracle/ref_mixer_modules.py), in float32 (tight) and bfloat16, on paged caches with shuffled blocks, state slots
that are not in batch order, prompt portions beside single tokens, and sizes that are not powers of two."""
import math

import pytest
import torch

import nanovllm_amd as nv
from nanovllm_amd import ops
from nanovllm_amd.layers import activation, attention, delta_rule, layernorm
from oracle import ref_mixer_modules as ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def _context(n_qs, n_ks, block_size, num_blocks, seed, slots=None):
    """Shuffled block tables for sequences with n_k tokens in the cache after this step, of which the last n_q are
    the step's rows."""
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(num_blocks, generator=g).tolist()
    need = [-(-n // block_size) for n in n_ks]
    assert sum(need) <= num_blocks
    width = max(need) + 1
    tables, nxt, slot_map, pos = [], 0, [], []
    for nq, nk, nb in zip(n_qs, n_ks, need):
        row = perm[nxt:nxt + nb]
        nxt += nb
        tables.append(row + [-1] * (width - nb))
        for p in range(nk - nq, nk):
            slot_map.append(row[p // block_size] * block_size + p % block_size)
            pos.append(p)
    cu = lambda xs: torch.tensor([0] + torch.tensor(xs).cumsum(0).tolist(), dtype=torch.int32, device=DEV)
    ctx = nv.CacheContext(slot_mapping=torch.tensor(slot_map, dtype=torch.int32, device=DEV), cu_seqlens_q=cu(n_qs),
                          cu_seqlens_k=cu(n_ks), max_seqlen_q=max(n_qs), max_seqlen_k=max(n_ks),
                          block_tables=torch.tensor(tables, dtype=torch.int32, device=DEV), block_size=block_size,
                          state_slots=None if slots is None else torch.tensor(slots, dtype=torch.int32, device=DEV))
    return ctx, torch.tensor(pos, dtype=torch.int64, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cols", [48, 256, 1000, 4096])
def test_add_layernorm_all_forms(dtype, cols):
    g = torch.Generator(device=DEV).manual_seed(cols)
    T = 37
    mk = lambda *s: torch.randn(*s, generator=g, device=DEV)
    a, b = layernorm.LayerNorm(cols, 1e-5, device=DEV), layernorm.LayerNorm(cols, 1e-5, device=DEV)
    ra, rb = ref.LayerNorm(cols, 1e-5, device=DEV), ref.LayerNorm(cols, 1e-5, device=DEV)
    with torch.no_grad():
        for m, r in ((a, ra), (b, rb)):
            m.weight.copy_(1 + 0.3 * mk(cols)); m.bias.copy_(0.2 * mk(cols))
            r.weight.copy_(m.weight); r.bias.copy_(m.bias)
    resid = 3 * mk(T, cols) + 2.0
    wide = (5 * mk(T, cols + 8)).to(dtype)
    h = wide[:, :cols]                                   # a row stride that is not the width
    extra = mk(T, cols)
    for use_h, use_extra, use_pre in [(0, 0, 1), (1, 0, 1), (1, 1, 1), (1, 0, 0), (0, 1, 0), (0, 1, 1)]:
        x, xr = resid.clone(), resid.clone()
        y = layernorm.residual_boundary(x, h if use_h else None, a if use_h else None, extra if use_extra else None,
                                        b if use_pre else None, dtype)
        yr = ref.residual_boundary(xr, h if use_h else None, ra if use_h else None, extra if use_extra else None,
                                   rb if use_pre else None, dtype)
        torch.testing.assert_close(x, xr, rtol=1e-5, atol=1e-5)
        if use_pre:
            torch.testing.assert_close(y.float(), yr.float(), **_tol(dtype))
        else:
            assert y is None


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gelu_tanh_and_mul(dtype):
    g = torch.Generator(device=DEV).manual_seed(1)
    x = (3 * torch.randn(19, 2 * 72 + 6, generator=g, device=DEV)).to(dtype)[:, :2 * 72]
    torch.testing.assert_close(activation.GeluTanhAndMul()(x).float(), ref.GeluTanhAndMul()(x).float(), **_tol(dtype))
    wide = (4 * torch.randn(33, 2 * 64, generator=g, device=DEV)).to(dtype)          # rows in 16-byte pieces
    wide[0, :8] = torch.tensor([-30.0, -9.0, -1.0, -1e-3, 0.0, 1e-3, 9.0, 30.0], device=DEV).to(dtype)
    torch.testing.assert_close(activation.GeluTanhAndMul()(wide).float(), ref.GeluTanhAndMul()(wide).float(), **_tol(dtype))


def _attention_pair(H, G, D, Dv, **kw):
    a = attention.ScoreModAttention(H, G, D, Dv, device=DEV, **kw)
    r = ref.ScoreModAttention(H, G, D, Dv, device=DEV, **kw)
    return a, r


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(8, 2, 96, 96), (4, 2, 64, 64), (6, 3, 40, 72), (5, 5, 128, 32), (2, 1, 24, 200)])
@pytest.mark.parametrize("flavour", ["rot_sink", "temp_bias", "plain"])
def test_scoremod_attention_mixed_batch(dtype, shape, flavour):
    H, G, D, Dv = shape
    bs, nb = 16, 40
    n_qs, n_ks = [1, 70, 2, 1, 33], [131, 70, 97, 1, 160]
    kw = dict(scale=D ** -0.5, softcap=20.0)
    if flavour == "rot_sink":
        kw.update(rot_dims=(D // 2) // 2 * 2, rot_base=5000.0, use_sink=True)
    elif flavour == "temp_bias":
        kw.update(temp_coef=0.7, temp_every=32)
    else:
        kw.update(softcap=0.0)
    a, r = _attention_pair(H, G, D, Dv, **kw)
    g = torch.Generator(device=DEV).manual_seed(H * 100 + D)
    if flavour == "rot_sink":
        with torch.no_grad():
            a.sink.copy_(torch.randn(H, generator=g, device=DEV) * 2)
            r.sink.copy_(a.sink)
    if flavour == "temp_bias":
        table = torch.randn(H, 50, generator=g, device=DEV)
        a.set_distance_bias(table)
        r.set_distance_bias(table)
    ctx, pos = _context(n_qs, n_ks, bs, nb, seed=3)
    T = sum(n_qs)
    mk = lambda *s: (torch.randn(*s, generator=g, device=DEV) * 1.5).to(dtype)
    kc, vc = mk(nb, bs, G, D), mk(nb, bs, G, Dv)
    kc_r, vc_r = kc.clone(), vc.clone()
    fused = mk(T, H * D + G * D + G * Dv + 8)             # q | k | v slices of one projection, as the model has them
    q = fused[:, :H * D].unflatten(1, (H, D))
    k = fused[:, H * D:H * D + G * D].unflatten(1, (G, D))
    v = fused[:, H * D + G * D:H * D + G * D + G * Dv].unflatten(1, (G, Dv))
    nv.set_context(ctx)
    o = a(q, k, v, pos, kc, vc)
    o_r = r(q, k, v, pos, kc_r, vc_r)
    nv.set_context(None)
    torch.testing.assert_close(kc.float(), kc_r.float(), **_tol(dtype))
    assert torch.equal(vc, vc_r)
    torch.testing.assert_close(o.float(), o_r.float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(4, 2, 96, 96), (2, 2, 128, 64), (4, 1, 32, 160), (2, 1, 256, 256)])
def test_scoremod_attention_long_portions_cross_query_and_key_tiles(dtype, shape):
    """Portions longer than the MFMA kernel's 64-query tile over caches longer than its 64-key tile, pages of 24
    (no multiple of either), single rows in between, and a sequence of 65 rows (one row into the second tile)."""
    H, G, D, Dv = shape
    bs, nb = 24, 60
    n_qs, n_ks = [200, 1, 130, 65, 2], [200, 77, 300, 65, 130]
    a, r = _attention_pair(H, G, D, Dv, scale=D ** -0.5, softcap=25.0, rot_dims=16, rot_base=1000.0, use_sink=True)
    g = torch.Generator(device=DEV).manual_seed(7)
    table = torch.randn(H, 90, generator=g, device=DEV)
    a.set_distance_bias(table)
    r.set_distance_bias(table)
    with torch.no_grad():
        a.sink.copy_(torch.randn(H, generator=g, device=DEV))
        r.sink.copy_(a.sink)
    ctx, pos = _context(n_qs, n_ks, bs, nb, seed=4)
    ctx.num_decode_seqs = 1
    T = sum(n_qs)
    mk = lambda *s: torch.randn(*s, generator=g, device=DEV).to(dtype)
    kc, vc = mk(nb, bs, G, D), mk(nb, bs, G, Dv)
    kc_r, vc_r = kc.clone(), vc.clone()
    q, k, v = mk(T, H, D), mk(T, G, D), mk(T, G, Dv)
    nv.set_context(ctx)
    o = a(q, k, v, pos, kc, vc)
    o_r = r(q, k, v, pos, kc_r, vc_r)
    nv.set_context(None)
    torch.testing.assert_close(o.float(), o_r.float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(8, 2, 96, 96), (16, 2, 64, 128), (12, 1, 32, 48), (3, 3, 20, 6), (4, 2, 128, 256)])
@pytest.mark.parametrize("lens", [[1500, 700, 1, 64, 65], [300] * 40])
def test_scoremod_attention_single_rows_key_slices_and_head_groups(dtype, shape, lens):
    """Pure decode steps: long contexts cut into key slices (some slices of the shorter sequences are empty), one
    key only, contexts of exactly one tile and one more, groups of 8 and 12 query heads per kv head, a head size
    that is no multiple of a 16-byte piece, and a batch large enough that nothing is sliced."""
    H, G, D, Dv = shape
    bs = 24
    nb = sum(-(-n // bs) for n in lens) + 2
    a, r = _attention_pair(H, G, D, Dv, scale=D ** -0.5, softcap=25.0, temp_coef=0.3, temp_every=100, use_sink=True)
    g = torch.Generator(device=DEV).manual_seed(9)
    table = torch.randn(H, 200, generator=g, device=DEV)
    a.set_distance_bias(table)
    r.set_distance_bias(table)
    with torch.no_grad():
        a.sink.copy_(torch.randn(H, generator=g, device=DEV) * 2)
        r.sink.copy_(a.sink)
    ctx, pos = _context([1] * len(lens), lens, bs, nb, seed=5)
    ctx.num_decode_seqs = len(lens)
    T = len(lens)
    mk = lambda *s: torch.randn(*s, generator=g, device=DEV).to(dtype)
    kc, vc = mk(nb, bs, G, D), mk(nb, bs, G, Dv)
    kc_r, vc_r = kc.clone(), vc.clone()
    q, k, v = mk(T, H, D), mk(T, G, D), mk(T, G, Dv)
    nv.set_context(ctx)
    o = a(q, k, v, pos, kc, vc)
    o_r = r(q, k, v, pos, kc_r, vc_r)
    nv.set_context(None)
    torch.testing.assert_close(o.float(), o_r.float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 3, 4])
@pytest.mark.parametrize("C", [200, 203])          # rows in 16-byte pieces, and a width that has none
def test_short_conv_in_portions_matches_one_pass(dtype, taps, C):
    slots_n = 5
    a, r = delta_rule.ShortConvSilu(C, taps, device=DEV), ref.ShortConvSilu(C, taps, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(taps)
    with torch.no_grad():
        a.weight.copy_(torch.randn(C, taps, generator=g, device=DEV))
        r.weight.copy_(a.weight)
    st = torch.full((slots_n, max(taps - 1, 0), C), 7.0, device=DEV).to(dtype)      # stale content of reused slots
    st_r = st.clone()
    lens = [11, 1, 6]
    xs = [torch.randn(n, C + 8, generator=g, device=DEV).to(dtype)[:, :C] for n in lens]
    slots = [3, 0, 4]
    cuts = [[1, 1, 2, 7], [1], [2, 1, 3]]                  # portions per sequence; step s takes the s-th of each
    done = [0, 0, 0]
    outs, outs_r = [[] for _ in lens], [[] for _ in lens]
    for s in range(4):
        live = [i for i in range(3) if s < len(cuts[i])]
        n_qs = [cuts[i][s] for i in live]
        n_ks = [done[i] + cuts[i][s] for i in live]
        ctx, _ = _context(n_qs, n_ks, 16, 16, seed=s, slots=[slots[i] for i in live])
        x = torch.cat([xs[i][done[i]:done[i] + cuts[i][s]] for i in live])
        nv.set_context(ctx)
        y, y_r = a(x, st), r(x, st_r)
        nv.set_context(None)
        o = 0
        for i, n in zip(live, n_qs):
            outs[i].append(y[o:o + n]); outs_r[i].append(y_r[o:o + n])
            o += n
            done[i] += n
    for i, n in enumerate(lens):
        whole = torch.nn.functional.silu(sum(
            torch.cat([torch.zeros(taps - 1, C, device=DEV), xs[i].float()])[j:j + n] * a.weight[:, j] for j in range(taps)))
        torch.testing.assert_close(torch.cat(outs[i]).float(), whole, **_tol(dtype))
        torch.testing.assert_close(torch.cat(outs[i]).float(), torch.cat(outs_r[i]).float(), **_tol(dtype))
    if taps > 1:
        torch.testing.assert_close(st[slots].float(), st_r[slots].float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 2, 64, 64), (4, 2, 32, 48), (6, 3, 128, 128), (3, 1, 24, 72), (2, 2, 192, 40)])
def test_gated_delta_rule_portions_and_slots(dtype, shape):
    H, G, D, Dv = shape
    a, r = delta_rule.GatedDeltaRule(H, G, D, Dv, 1e-5, device=DEV), ref.GatedDeltaRule(H, G, D, Dv, 1e-5, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(D + Dv)
    with torch.no_grad():
        a.A_log.copy_(torch.randn(H, generator=g, device=DEV) * 0.5 - 1.0)
        a.dt_bias.copy_(torch.randn(H * D, generator=g, device=DEV))
        a.norm_weight.copy_(1 + 0.2 * torch.randn(Dv, generator=g, device=DEV))
        r.load_state_dict(a.state_dict())
    state = torch.full((4, H, D, Dv), 3.0, device=DEV)                   # stale content of reused slots
    state_r = state.clone()
    mk = lambda *s: (torch.randn(*s, generator=g, device=DEV)).to(dtype)
    for step, (n_qs, n_ks, slots) in enumerate([([40, 1, 5], [40, 1, 5], [2, 0, 3]),
                                                ([1, 19, 2], [41, 20, 7], [2, 0, 3]),
                                                ([1, 3], [42, 3], [2, 1])]):      # slot 1: a new sequence
        ctx, _ = _context(n_qs, n_ks, 16, 16, seed=step, slots=slots)
        T = sum(n_qs)
        q, k, v = mk(T, G, D), mk(T, G, D), mk(T, H, Dv)
        a_raw, b_raw, gate = mk(T, H * D), mk(T, H), mk(T, H * Dv)
        nv.set_context(ctx)
        o = a(q, k, v, a_raw, b_raw, gate, state)
        o_r = r(q, k, v, a_raw, b_raw, gate, state_r)
        nv.set_context(None)
        torch.testing.assert_close(o.float(), o_r.float(), **(_tol(dtype) if dtype != torch.float32 else dict(rtol=1e-4, atol=1e-4)))
        torch.testing.assert_close(state[slots], state_r[slots], rtol=1e-4, atol=1e-4)
