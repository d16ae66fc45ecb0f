"""Each mechanism of the Buvalix layers alone, against the plain functions of oracle/ref_buvalix.py, with inputs
made so that a fault shows: one key far back whose score stands out among hundreds, a sink that takes most of the
mass, a distance table with one loud row per bucket edge, a decay that is almost 1 next to one that forgets at once.
CPU: the eager stand-ins (what the CPU engine tests run on); gpu: the HIP kernels."""
import math

import pytest
import torch

import nanovllm_amd as nv
from buvalix_util import layer_namespace, paged_context
from nanovllm_amd.model.buvalix import distance_bias_table
from oracle import ref_buvalix as R

BACKENDS = [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def dev(request):
    return request.param


def run_attention(dev, attn, q, k, v, cuts, block_size=8):
    """Feed one sequence through the layer in the given portions; returns [T, H * Dv]."""
    T, G, D = k.shape
    Dv = v.shape[2]
    nb = -(-T // block_size) + 2
    kc = torch.full((nb, block_size, G, D), 9.0, device=dev)
    vc = torch.full((nb, block_size, G, Dv), -9.0, device=dev)
    out, done = [], 0
    table_seed = 5
    for n in cuts:
        ctx, pos = paged_context([n], [done + n], block_size, nb, table_seed, dev)
        nv.set_context(ctx)
        s = slice(done, done + n)
        out.append(attn(q[s].to(dev), k[s].to(dev), v[s].to(dev), pos, kc, vc).cpu())
        nv.set_context(None)
        done += n
    assert done == T
    return torch.cat(out)


def cuts_for(T):
    return [[T], [T - 40, 1, 2, 37], [1] * T] if T <= 80 else [[T], [T - 33, 1, 1, 31]]


def test_far_key_among_hundreds_with_rotary_sink_and_cap(dev):
    L = layer_namespace(dev)
    H, G, D, Dv, T = 4, 2, 16, 24, 300
    g = torch.Generator().manual_seed(0)
    q, k, v = torch.randn(T, H, D, generator=g) * 0.3, torch.randn(T, G, D, generator=g) * 0.3, torch.randn(T, G, Dv, generator=g)
    # un-rotated dimensions (8..15) carry a loud match between the last queries and key 3, and between query 150 and
    # key 149 / its own position (just inside) -- a key dropped or shifted by one changes the output by O(1)
    k[3, :, 8:] = 4.0
    q[-5:, :, 8:] = 4.0
    k[149, :, 8:] = -4.0
    q[150, :, 8:] = -4.0
    attn = L.ScoreModAttention(H, G, D, Dv, scale=0.25, softcap=30.0, rot_dims=8, rot_base=100.0, use_sink=True, device=dev)
    with torch.no_grad():
        attn.sink.copy_(torch.tensor([-2.0, 0.5, 3.0, 25.0]))         # the last head's sink outweighs most rows
    want = R.causal_attention(R.rotary_interleaved(q, torch.arange(T), 8, 100.0), R.rotary_interleaved(k, torch.arange(T), 8, 100.0),
                              v, 0.25, 30.0, sink=attn.sink.detach().cpu()).reshape(T, -1)
    # the sink really matters, and the far key really is seen
    no_sink = R.causal_attention(R.rotary_interleaved(q, torch.arange(T), 8, 100.0), R.rotary_interleaved(k, torch.arange(T), 8, 100.0),
                                 v, 0.25, 30.0).reshape(T, -1)
    assert (want - no_sink).abs().max() > 0.1
    for cuts in cuts_for(T):
        got = run_attention(dev, attn, q, k, v, cuts)
        torch.testing.assert_close(got, want, rtol=2e-4, atol=2e-4)


def test_distance_table_rows_and_query_temperature_edges(dev):
    L = layer_namespace(dev)
    H, G, D, Dv, T = 2, 1, 8, 8, 70
    rows, far, every = 10, 24.0, 9
    # buckets by the definition, at the edges: exact below rows/2, the last row from `far` on
    assert [R.distance_bucket(n, rows, far) for n in (0, 4, 5, 23, 24, 25, 500)] == [0, 4, 5, 9, 9, 9, 9]
    assert R.distance_bucket(6, rows, far) == 5 and R.distance_bucket(7, rows, far) == 6
    rel = torch.zeros(rows, H)
    rel[:, 0] = torch.tensor([0.0, 6.0, -6.0, 6.0, -6.0, 6.0, -6.0, 6.0, -6.0, 6.0])    # neighbouring rows disagree loudly
    rel[:, 1] = torch.linspace(-5, 5, rows)
    table = distance_bias_table(rel.to(dev), far)
    assert table.shape == (H, 25)
    for n in range(25):
        assert torch.equal(table[:, n].cpu(), rel[R.distance_bucket(n, rows, far)])
    g = torch.Generator().manual_seed(1)
    q, k, v = torch.randn(T, H, D, generator=g), torch.randn(T, G, D, generator=g), torch.randn(T, G, Dv, generator=g)
    attn = L.ScoreModAttention(H, G, D, Dv, scale=0.5, softcap=10.0, temp_coef=0.8, temp_every=every, device=dev)
    attn.set_distance_bias(table)
    temp = R.query_temperature(torch.arange(T), 0.8, every)
    assert temp[7] == 1.0 and temp[8] > 1.5 and temp[16] == temp[8] and temp[17] > temp[16]      # steps at p + 1 = 9, 18
    want = R.causal_attention(q * temp[:, None, None], k, v, 0.5, 10.0, rel=rel, far=far).reshape(T, -1)
    for cuts in cuts_for(T):
        got = run_attention(dev, attn, q, k, v, cuts)
        torch.testing.assert_close(got, want, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("taps", [2, 3, 5])
def test_short_convolution_first_tokens_and_portions(dev, taps):
    L = layer_namespace(dev)
    C, T = 12, 23
    g = torch.Generator().manual_seed(taps)
    x, w = torch.randn(T, C, generator=g), torch.randn(C, taps, generator=g)
    conv = L.ShortConvSilu(C, taps, device=dev)
    with torch.no_grad():
        conv.weight.copy_(w)
    want = R.short_conv_silu(x, w)
    for cuts in ([T], [1] * T, [2, 1, 1, 3, 16], [taps - 1, 1, T - taps]):
        state = torch.full((3, taps - 1, C), 50.0, device=dev)      # what a previous owner of the slot left
        out, done = [], 0
        for n in cuts:
            ctx, _ = paged_context([n], [done + n], 8, 8, 0, dev, slots=[1])
            nv.set_context(ctx)
            out.append(conv(x[done:done + n].to(dev), state).cpu())
            nv.set_context(None)
            done += n
        torch.testing.assert_close(torch.cat(out), want, rtol=1e-5, atol=1e-5)
        assert torch.all(state[0] == 50.0) and torch.all(state[2] == 50.0)


def test_gated_delta_rule_decays_heads_and_portions(dev):
    L = layer_namespace(dev)
    H, G, D, Dv, T = 4, 2, 10, 6, 40
    g = torch.Generator().manual_seed(3)
    q, k, v = torch.randn(T, G, D, generator=g), torch.randn(T, G, D, generator=g), torch.randn(T, H, Dv, generator=g)
    a_raw, b_raw, gate = torch.randn(T, H * D, generator=g), torch.randn(T, H, generator=g), torch.randn(T, H * Dv, generator=g)
    rule = L.GatedDeltaRule(H, G, D, Dv, 1e-5, device=dev)
    with torch.no_grad():
        rule.A_log.copy_(torch.tensor([-6.0, 0.0, 2.5, -1.0]))       # head 0 keeps almost everything, head 2 forgets at once
        rule.dt_bias.copy_(torch.randn(H * D, generator=g) * 2)
        rule.norm_weight.copy_(torch.randn(Dv, generator=g))
    rep = H // G
    qn = (q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5).repeat_interleave(rep, 1)
    kn = (k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)).repeat_interleave(rep, 1)
    decay = torch.exp(-torch.exp(rule.A_log.detach().cpu())[None, :, None]
                      * torch.nn.functional.softplus(a_raw + rule.dt_bias.detach().cpu()).view(T, H, D))
    assert decay[:, 0].min() > 0.9 and decay[:, 2].median() < 0.05
    o = R.gated_delta_channel(qn, kn, v, torch.sigmoid(b_raw), decay)
    want = (R.rms_unit(o, 1e-5) * rule.norm_weight.detach().cpu() * torch.sigmoid(gate).view(T, H, Dv)).reshape(T, -1)
    for cuts in ([T], [1] * T, [2, 17, 1, 20]):
        state = torch.full((2, H, D, Dv), 7.0, device=dev)
        out, done = [], 0
        for n in cuts:
            ctx, _ = paged_context([n], [done + n], 8, 8, 0, dev, slots=[1])
            nv.set_context(ctx)
            s = slice(done, done + n)
            out.append(rule(q[s].to(dev), k[s].to(dev), v[s].to(dev), a_raw[s].to(dev), b_raw[s].to(dev),
                            gate[s].to(dev), state).cpu())
            nv.set_context(None)
            done += n
        torch.testing.assert_close(torch.cat(out), want, rtol=2e-4, atol=2e-4)
        assert torch.all(state[0] == 7.0)


def test_layer_norm_boundary_and_gelu(dev):
    L = layer_namespace(dev)
    W, T = 44, 9
    g = torch.Generator().manual_seed(4)
    a, b = L.LayerNorm(W, 1e-3, device=dev), L.LayerNorm(W, 1e-3, device=dev)
    with torch.no_grad():
        for m in (a, b):
            m.weight.copy_(torch.randn(W, generator=g)); m.bias.copy_(torch.randn(W, generator=g))
    x, h, e = torch.randn(T, W, generator=g) * 4 + 3, torch.randn(T, W, generator=g), torch.randn(T, W, generator=g)
    xd = x.clone().to(dev)
    y = L.residual_boundary(xd, h.to(dev), a, e.to(dev), b, torch.float32)
    x_want = x + R.layer_norm(h, a.weight.detach().cpu(), a.bias.detach().cpu(), 1e-3) + e
    torch.testing.assert_close(xd.cpu(), x_want, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(y.cpu(), R.layer_norm(x_want, b.weight.detach().cpu(), b.bias.detach().cpu(), 1e-3), rtol=1e-5, atol=2e-5)
    z = torch.randn(T, 2 * 14, generator=g) * 3
    torch.testing.assert_close(L.GeluTanhAndMul()(z.to(dev)).cpu(), R.gelu_tanh(z[:, :14]) * z[:, 14:], rtol=1e-5, atol=1e-5)
    assert abs(R.gelu_tanh(torch.tensor(1.0)).item() - 0.5 * (1 + math.tanh(math.sqrt(2 / math.pi) * 1.044715))) < 1e-7
