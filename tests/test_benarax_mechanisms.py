"""Each mechanism of the Benarax layers alone, against the plain functions of oracle/ref_benarax.py, with inputs made
so that a fault shows: a key far back whose score stands out among hundreds, loud keys at the query's own position
(seen) and at the next one (not seen), norm groups of very different size, a state channel that never decays next to
one that forgets fast, a removal rate of one, experts that clamp, an expert nobody chooses.
CPU: the eager stand-ins (what the CPU engine tests run on); gpu: the HIP kernels."""
import math

import pytest
import torch

import nanovllm_amd as nv
from benarax_util import config, delta_layer, latent_layer, layer_namespace, moe, paged_context, random_checkpoint
from nanovllm_amd.model.benarax import BenaraxConfig, BenaraxForCausalLM
from oracle import ref_benarax as R

BACKENDS = [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def dev(request):
    return request.param


def one_layer(layer, dev, seed=0, edit=None, **cfg_kw):
    """A one-layer model in float32 with random weights (edited by `edit(ck)` before loading)."""
    cfg = config([layer], **cfg_kw)
    ck = random_checkpoint(cfg, seed)
    if edit is not None:
        edit(ck)
    model = BenaraxForCausalLM(BenaraxConfig.from_dict(cfg), layers=layer_namespace(dev), dtype=torch.float32, device=dev)
    model.load_tensors(ck)
    return model, cfg, ck


def in_portions(dev, fn, T, cuts, block_size=8, slot=1, n_slots=3):
    """Run fn(rows slice, positions) over one sequence in the given portions under a paged context."""
    nb = -(-T // block_size) + 2
    out, done = [], 0
    for n in cuts:
        ctx, pos = paged_context([n], [done + n], block_size, nb, 5, dev, slots=[slot])
        nv.set_context(ctx)
        out.append(fn(slice(done, done + n), pos).cpu())
        nv.set_context(None)
        done += n
    assert done == T
    return torch.cat(out)


def cuts_for(T):
    return [[T], [T - 40, 1, 2, 37], [2] * (T // 2) + [1] * (T % 2)] if T <= 90 else [[T], [T - 33, 1, 1, 31]]


# ------------------------------------------------------------------------------------------ stream boundary
@pytest.mark.parametrize("groups", [1, 2, 5, 10])
def test_grouped_norm_takes_every_part_by_itself(dev, groups):
    L = layer_namespace(dev)
    g = torch.Generator().manual_seed(groups)
    T, W = 7, 40
    x = torch.randn(T, W, generator=g)
    x[:, :W // groups] *= 300.0                     # one loud part must not quieten the others
    w = torch.randn(W, generator=g)
    h32, h = L.stream_boundary(x.clone().to(dev), norm=w.to(dev), groups=groups, eps=1e-5, out_dtype=torch.float32, want_f32=True)
    want = R.group_rms_norm(x, w, groups, 1e-5)
    torch.testing.assert_close(h.cpu(), want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(h32.cpu(), want, rtol=1e-5, atol=1e-5)
    if groups > 1:
        assert (h.cpu() - R.group_rms_norm(x, w, 1, 1e-5)).abs().max() > 0.5


def test_boundary_adds_parallel_sublayers_and_the_normed_side_input(dev):
    L = layer_namespace(dev)
    g = torch.Generator().manual_seed(3)
    T, W, m = 9, 24, 0.6
    x, a, y = torch.randn(T, W, generator=g), torch.randn(T, W, generator=g), torch.randn(T, W, generator=g) * 50
    parts, wn, w = torch.randn(T, 3, W, generator=g), torch.randn(W, generator=g), torch.randn(W, generator=g)
    xs = x.clone().to(dev)
    xb = L.stream_boundary(xs, add=a.to(dev), add_parts=parts.to(dev), mult=m, copy_dtype=torch.float32)
    x1 = x + m * (a + parts.sum(1))
    torch.testing.assert_close(xs.cpu(), x1, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(xb.cpu(), x1, rtol=1e-5, atol=1e-5)
    _, h = L.stream_boundary(xs, normed=y.to(dev), normed_weight=wn.to(dev), mult=m, norm=w.to(dev), groups=3, eps=1e-5,
                             out_dtype=torch.float32)
    x2 = x1 + m * R.rms_unit(y, 1e-5) * wn
    torch.testing.assert_close(xs.cpu(), x2, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(h.cpu(), R.group_rms_norm(x2, w, 3, 1e-5), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(L.rms_norm_rows(y.to(dev), wn.to(dev), 1e-5).cpu(), R.rms_unit(y, 1e-5) * wn, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("taps", [1, 2, 4, 6])
def test_convolution_carries_its_last_inputs_and_starts_from_zeros(dev, taps):
    L = layer_namespace(dev)
    g = torch.Generator().manual_seed(taps)
    T, C = 23, 20
    x, w = torch.randn(T, C, generator=g), torch.randn(C, taps, generator=g)
    conv = L.CausalConvAdd(C, taps, device=dev)
    with torch.no_grad():
        conv.weight.copy_(w)
    want = x + R.causal_conv(x, w)
    for cuts in ([T], [1] * T, [2] * 11 + [1], [3, 1, 1, 2, 9, 7]):
        state = torch.full((3, taps - 1, C), 7.0, device=dev)           # what a previous owner of the slot left
        got = in_portions(dev, lambda s, pos: conv(x[s].to(dev), state, torch.float32), T, cuts)
        torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-5)
        assert (state[0] == 7).all() and (state[2] == 7).all()          # other slots untouched


def test_token_gate_reads_its_own_columns(dev):
    L = layer_namespace(dev)
    g = torch.Generator().manual_seed(1)
    T, dim, V = 11, 6, 13
    z, table = torch.randn(T, dim, generator=g) * 2, torch.randn(V, 4 * dim, generator=g)
    ids = torch.randint(0, V, (T,), generator=g)
    for layer in (0, 2, 3):
        got = L.TokenGate(layer * dim, dim)(z.to(dev), table.to(dev), ids.to(dev)).cpu()
        torch.testing.assert_close(got, R.gelu_tanh(z) * table[ids, layer * dim:(layer + 1) * dim], rtol=1e-5, atol=1e-5)


# ------------------------------------------------------------------------------------------ generalized delta rule
def test_delta_rule_keeps_what_does_not_decay_and_removes_at_rate_one(dev):
    def edit(ck):
        ck["l0.mix.w0"][:] = -30.0                  # sigmoid -> 0: these channels never decay ...
        ck["l0.mix.w0"][5:9] = 30.0                 # ... these lose the most per token (exp(-exp(-1/2)))
        ck["l0.mix.w2"][:] = 0.0
        ck["l0.mix.a.b"][:] = -30.0                 # nothing is removed ...
        ck["l0.mix.a.b"][16:] = 30.0                # ... except in the second head, at rate one
        ck["l0.mix.a"][:] = 0.0
    model, cfg, ck = one_layer(delta_layer(heads=2, dim=16), dev, seed=2, edit=edit)
    mix, m = model.layers[0].mix, cfg["layers"][0]["mixer"]
    T, W = 260, cfg["width"]
    g = torch.Generator().manual_seed(4)
    h = torch.randn(T, W, generator=g)
    h[200:] = h[0]                                   # late tokens ask with the first token's vector
    want = R.general_delta(h, ck, "l0.mix.", m, cfg["norm"]["eps"], torch.float32)
    # the read-out 200 tokens later still depends on the first token
    h2 = h.clone()
    h2[0] = torch.randn(W, generator=g)
    assert (R.general_delta(h2, ck, "l0.mix.", m, cfg["norm"]["eps"], torch.float32)[250] - want[250]).abs().max() > 2e-3
    for cuts in cuts_for(T) + [[3] + [1] * (T - 3)]:
        state = torch.full((3, 2, 16, 16), 5.0, device=dev)
        got = in_portions(dev, lambda s, pos: mix(h[s].to(dev), pos, {"state": state}), T, cuts)
        torch.testing.assert_close(got, want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("heads,dim", [(1, 8), (3, 20), (2, 40), (1, 72)])
def test_delta_rule_sizes(dev, heads, dim):
    model, cfg, ck = one_layer(delta_layer(heads=heads, dim=dim), dev, seed=dim)
    T = 37
    h = torch.randn(T, cfg["width"], generator=torch.Generator().manual_seed(dim))
    want = R.general_delta(h, ck, "l0.mix.", cfg["layers"][0]["mixer"], cfg["norm"]["eps"], torch.float32)
    for cuts in ([T], [18, 1, 17, 1]):
        state = torch.zeros(3, heads, dim, dim, device=dev)
        got = in_portions(dev, lambda s, pos: model.layers[0].mix(h[s].to(dev), pos, {"state": state}), T, cuts)
        torch.testing.assert_close(got, want, rtol=2e-4, atol=2e-4)


# ------------------------------------------------------------------------------------------ latent attention
def latent_reference(q_rot, q_lat, c, k_rot, scale):
    s = (torch.einsum("ihd,jd->hij", q_lat, c) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * scale
    T = c.shape[0]
    s = s.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), float("-inf"))
    return torch.einsum("hij,jd->ihd", torch.softmax(s, -1), c)


@pytest.mark.parametrize("interleaved", [True, False])
def test_far_key_own_position_and_next_position(dev, interleaved):
    L = layer_namespace(dev)
    H, rank, Rr, Dq, T, eps = 3, 24, 8, 20, 300, 1e-5
    g = torch.Generator().manual_seed(7)
    q = torch.randn(T, H, Dq, generator=g) * 0.3
    q_lat = torch.randn(T, H, rank, generator=g) * 0.3
    ckv = torch.randn(T, rank + Rr, generator=g)
    lat_w = torch.randn(rank, generator=g) * 0.1 + 1.0
    # key 3, far back, is loud along one latent direction that the last queries ask for; query 150 asks for what the
    # keys at 150 (its own place: seen) and 151 (not seen) hold along another
    ckv[3, :rank] = 0.0
    ckv[3, 0] = 9.0
    q_lat[-5:, :, 0] = 6.0
    for j in (150, 151):
        ckv[j, :rank] = 0.0
        ckv[j, 1] = 9.0 if j == 150 else -9.0
    q_lat[150, :, 1] = 6.0
    q_lat[149, :, 1] = -6.0                        # would love key 151 (and 150 is the NEXT position for it)
    scaling = {"factor": 4.0, "fast": 16.0, "slow": 1.0, "original": 64} if interleaved else None
    attn = L.LatentAttention(H, rank, Rr, 0.7, eps, 50.0, scaling, interleaved=interleaved, device=dev)
    with torch.no_grad():
        attn.latent_norm.copy_(lat_w)
    freq, mag = R.rotary_frequencies(Rr, 50.0, scaling)
    pos = torch.arange(T)
    c = R.rms_unit(ckv[:, :rank], eps) * lat_w
    k_rot = R.rotary(ckv[:, None, rank:], pos, freq, mag, interleaved)[:, 0]
    q_rot = R.rotary(q[..., Dq - Rr:], pos, freq, mag, interleaved)
    want = latent_reference(q_rot, q_lat, c, k_rot, 0.7)
    w_far = torch.softmax((torch.einsum("hd,jd->hj", q_lat[-1], c) + torch.einsum("hd,jd->hj", q_rot[-1], k_rot)) * 0.7, -1)
    assert w_far[:, 3].min() > 0.5                   # the far key really carries the answer
    for cuts in cuts_for(T) + [[148, 1, 1, 1, 1, 148]]:
        nb = -(-T // 8) + 2
        kc = torch.full((nb, 8, 1, rank + Rr), 9.0, device=dev)
        vc = kc[..., :rank]                          # the values are the front of the key rows, as in the engine
        got = in_portions(dev, lambda s, p: attn(q[s].to(dev), q_lat[s].to(dev), ckv[s].to(dev), p, kc, vc), T, cuts)
        torch.testing.assert_close(got, want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("kind,kw", [("latent_attention", {}), ("latent_attention_2", {}),
                                     ("latent_attention", dict(heads=1, dim=16, rot_dim=16, vdim=4, q_rank=7, kv_rank=16)),
                                     ("latent_attention_2", dict(heads=5, dim=6, rot_dim=2, vdim=6, q_rank=30, kv_rank=9,
                                                                 scaling={"factor": 2.0, "fast": 4.0, "slow": 0.5, "original": 16}))])
def test_latent_mixer_equals_the_plain_form(dev, kind, kw):
    """The mixer as the model runs it (key up-projection applied to the query, value up-projection to the output)
    against keys and values expanded per head."""
    model, cfg, ck = one_layer(latent_layer(kind, **kw), dev, seed=9)
    m, T = cfg["layers"][0]["mixer"], 45
    h = torch.randn(T, cfg["width"], generator=torch.Generator().manual_seed(3))
    want = R.latent_attention(h, ck, "l0.mix.", m, cfg["norm"]["eps"], kind == "latent_attention", torch.float32)
    for cuts in cuts_for(T):
        nb = -(-T // 8) + 2
        kc = torch.zeros(nb, 8, 1, m["kv_rank"] + m["rot_dim"], device=dev)
        vc = torch.zeros(nb, 8, 1, m["kv_rank"], device=dev)
        got = in_portions(dev, lambda s, p: model.layers[0].mix(h[s].to(dev), p, (kc, vc)), T, cuts)
        torch.testing.assert_close(got, want, rtol=2e-4, atol=2e-4)


# ------------------------------------------------------------------------------------------ routed experts
@pytest.mark.parametrize("experts,top,ff,T", [(5, 2, 24, 33), (4, 1, 8, 5), (3, 3, 40, 70), (9, 4, 16, 1), (6, 2, 72, 400)])
def test_experts_route_clamp_and_weigh(dev, experts, top, ff, T):
    def edit(ck):
        ck["l0.mlp.router"][experts - 1] = 0.0       # nobody prefers the last expert ...
        ck["l0.mlp.router"][experts - 1, 0] = -20.0
        ck["l0.mlp.e0.gate"] *= 6.0                  # ... and the first one clamps
        ck["l0.mlp.e0.up"] *= 6.0
    model, cfg, ck = one_layer(delta_layer(mlp=moe(experts, top, ff, limit=0.75)), dev, seed=experts, edit=edit)
    g = torch.Generator().manual_seed(T)
    h = torch.randn(T, cfg["width"], generator=g)
    h[:, 0] = h[:, 0].abs() + 0.5
    want = R.moe(h, ck, "l0.mlp.", cfg["layers"][0]["mlp"], torch.float32)
    got = model.layers[0].mlp(h.to(dev))
    assert got.shape == (T, top, cfg["width"])
    torch.testing.assert_close(got.sum(1).cpu(), want, rtol=2e-4, atol=2e-4)
    logits = h @ ck["l0.mlp.router"].float().T
    if top < experts:
        assert (logits.topk(top, -1).indices != experts - 1).all()
