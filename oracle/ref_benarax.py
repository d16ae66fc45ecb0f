"""Oracle (test infrastructure): a plain, slow restatement of the Benarax design, one function per mechanism,
whole sequences at a time, no cache and no batching.  It shares nothing with the product path: tests compare
the engine (paged latent cache, state slots, chunked prompts, mixed batches, HIP kernels) with these functions.

`dtype=torch.float32` computes everything in 32-bit.  With `torch.bfloat16` the matrix products take bfloat16
operands (fp32 accumulation, bfloat16 result) and everything the design keeps in 32-bit stays there: the residual
stream, norms, routers, rotary angles, attention scores and weights, and the whole recurrence with its gates.

A model is (cfg, weights): cfg the parsed config.json, weights a dict name -> tensor as stored.

The design in short.  x_0 = embed[token] * embedding.scale.  Every layer: h = groupnorm(x); the mixer reads
h + causalconv(h) and the feed-forward reads h; x += m * (mixer + ff); then a per-layer token table enters:
y = P (gelu_tanh(G x) * table[token]), x += m * rmsnorm(y) * w.  A span of layers may run several times with the same
weights (each pass with its own history).  logits = head groupnorm(x) * logit_scale.
"""
from __future__ import annotations

import math

import torch


def linear(x, w, b=None, dtype=torch.float32):
    return torch.nn.functional.linear(x.to(dtype), w.to(dtype), None if b is None else b.to(dtype))


def rms_unit(x, eps):
    x = x.float()
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_rms_norm(x, w, groups, eps):
    """Each of `groups` equal consecutive parts is divided by its own root mean square; then the weight."""
    T, W = x.shape
    y = rms_unit(x.float().view(T, groups, W // groups), eps).reshape(T, W)
    return y * w.float()


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_conv(h, w):
    """h [T, C], w [C, taps]: out_t = sum_j w[:, j] h_(t - taps + 1 + j), zeros before the start."""
    T, C = h.shape
    taps = w.shape[1]
    out = torch.zeros(T, C)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j].float() * h[s].float()
    return out


# ------------------------------------------------------------------------------------------ rotary
def rotary_frequencies(dims, base, scaling=None):
    """(frequencies [dims/2] float32, magnitude): base^(-2i/dims), optionally blended towards f / factor for the
    slowly turning pairs (a linear ramp between the pairs that make `fast` and `slow` turns over `original`
    positions), with cos and sin scaled by 0.1 ln(factor) + 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    mag = 1.0
    if scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        at = lambda turns: dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(at(float(scaling["fast"]))), 0)
        hi = min(math.ceil(at(float(scaling["slow"]))), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    return f.float(), mag


def rotary(x, positions, freq, mag, interleaved):
    """x [T, H, R] with R = 2 * len(freq): pairs (2i, 2i+1) when interleaved, else (i, i + R/2)."""
    x = x.float()
    ang = positions.float()[:, None] * freq[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    half = freq.numel()
    out = torch.empty_like(x)
    if interleaved:
        u, v = x[..., 0::2], x[..., 1::2]
        out[..., 0::2] = u * c - v * s
        out[..., 1::2] = v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:]
        out[..., :half] = u * c - v * s
        out[..., half:] = v * c + u * s
    return out


# ------------------------------------------------------------------------------------------ mixers
def latent_attention(h, W, p, m, eps, interleaved, dtype):
    """Queries and keys / values both go through a normalised low-rank latent; one rotated key part is shared by all
    heads; plain causal softmax."""
    T = h.shape[0]
    H, D, R, Dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = (rms_unit(linear(h, W[p + "dq"], dtype=dtype), eps) * W[p + "dq.norm"].float()).to(dtype)
    q = linear(cq, W[p + "uq"], dtype=dtype).float().view(T, H, D + R)
    kv = linear(h, W[p + "dkv"], dtype=dtype).float()
    c = (rms_unit(kv[:, :rank], eps) * W[p + "dkv.norm"].float()).to(dtype)
    freq, mag = rotary_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    k_rot = rotary(kv[:, None, rank:], pos, freq, mag, interleaved).to(dtype).float()       # [T, 1, R]
    q_rot = rotary(q[..., D:], pos, freq, mag, interleaved).to(dtype).float()
    k_plain = linear(c, W[p + "uk"], dtype=dtype).float().view(T, H, D)
    v = linear(c, W[p + "uv"], dtype=dtype).float().view(T, H, Dv)
    s = torch.einsum("ihd,jhd->hij", q[..., :D].to(dtype).float(), k_plain)
    s = (s + torch.einsum("ihd,jd->hij", q_rot, k_rot[:, 0])) * float(m["scale"])
    s = s.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), float("-inf"))
    o = torch.einsum("hij,jhd->ihd", torch.softmax(s, dim=-1), v).reshape(T, H * Dv)
    return linear(o, W[p + "o"], dtype=dtype)


def general_delta(h, W, p, m, eps, dtype):
    """Per head a state S [D, D] (key channel x value channel): S <- diag(w) S - (a * u)(u^T S) + k v^T with both
    terms reading the old state, u the unit key; read-out S^T r, unit rms per head, weight, output gate."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = linear(h, W[p + "r"], dtype=dtype).float().view(T, H, D)
    k = linear(h, W[p + "k"], dtype=dtype).float().view(T, H, D)
    v = linear(h, W[p + "v"], dtype=dtype).float().view(T, H, D)
    low = torch.tanh(linear(h, W[p + "w1"], dtype=dtype).float()).to(dtype)
    w_raw = linear(low, W[p + "w2"], dtype=dtype).float() + W[p + "w0"].float()
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(w_raw)).view(T, H, D)
    a = torch.sigmoid(linear(h, W[p + "a"], dtype=dtype).float() + W[p + "a.b"].float()).view(T, H, D)
    gate = torch.sigmoid(linear(h, W[p + "g"], dtype=dtype).float())
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, D, D)
    out = torch.zeros(T, H, D)
    for t in range(T):
        uS = torch.einsum("hk,hkv->hv", u[t], S)
        S = decay[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, r[t])
    o = rms_unit(out, eps).reshape(T, H * D) * W[p + "norm"].float() * gate
    return linear(o, W[p + "o"], dtype=dtype)


# ------------------------------------------------------------------------------------------ feed-forward
def moe(h, W, p, mlp, dtype, margins=None):
    """Router logits in 32-bit; the `top` largest choose the experts, weighted by a softmax over those logits only.
    Expert: g = min(G h, lim), u = clamp(U h, -lim, lim), down(g * sigmoid(1.702 g) * (u + 1)).
    margins: a list that receives, per token, how far the last chosen logit lies above the first one left out, in units
    of the token's logit spread (infinite when every expert is chosen)."""
    T = h.shape[0]
    top, lim = mlp["router"]["top"], float(mlp["expert"]["limit"])
    z = linear(h.to(dtype).float(), W[p + "router"].float())
    val, idx = z.topk(top, dim=-1)
    if margins is not None:
        if top < z.shape[1]:
            nxt = z.topk(top + 1, dim=-1).values[:, -1]
            margins.append((val[:, -1] - nxt) / z.std(dim=-1).clamp_min(1e-9))
        else:
            margins.append(torch.full((T,), float("inf")))
    wgt = torch.softmax(val, dim=-1)
    out = torch.zeros(T, W[p + "e0.down"].shape[0])
    for t in range(T):
        for j in range(top):
            e = f"{p}e{int(idx[t, j])}."
            g = linear(h[t:t + 1], W[e + "gate"], dtype=dtype).float().clamp(max=lim)
            u = linear(h[t:t + 1], W[e + "up"], dtype=dtype).float().clamp(-lim, lim)
            y = (g * torch.sigmoid(1.702 * g) * (u + 1)).to(dtype)
            out[t] += wgt[t, j] * linear(y, W[e + "down"], dtype=dtype).float()[0]
    return out


def token_side(x, tokens, W, i, dim, eps, dtype):
    """The per-layer token table's contribution (before the residual multiplier)."""
    p = f"l{i}.side."
    e = W["side.embed"][tokens, i * dim:(i + 1) * dim].float()
    g = (gelu_tanh(linear(x, W[p + "gate"], dtype=dtype).float()) * e).to(dtype)
    y = linear(g, W[p + "proj"], dtype=dtype).float()
    return rms_unit(y, eps) * W[p + "norm"].float()


# ------------------------------------------------------------------------------------------ the model
def layer_runs(cfg):
    n, loop = len(cfg["layers"]), cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(cfg, W, tokens, dtype=torch.float32, margins=None):
    """Returns (logits [T, vocab] float32, residual stream after every layer run [runs, T, width]).
    margins: a list that receives every run's router margins (see `moe`)."""
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps, groups, mult = float(cfg["norm"]["eps"]), int(cfg["norm"]["groups"]), float(cfg["residual_mult"])
    x = W["embed"][tokens].float() * float(cfg["embedding"]["scale"])
    streams = []
    for i in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        h32 = group_rms_norm(x, W[p + "norm1"], groups, eps)
        hm = h32
        if cfg.get("canon"):
            hm = h32 + causal_conv(h32, W[p + "canon1"])
        h, hm = h32.to(dtype), hm.to(dtype)
        if L["type"] == "general_delta":
            y = general_delta(hm, W, p + "mix.", L["mixer"], eps, dtype).float()
        else:
            y = latent_attention(hm, W, p + "mix.", L["mixer"], eps, L["type"] == "latent_attention", dtype).float()
        if L.get("mlp") is not None:
            y = y + moe(h, W, p + "mlp.", L["mlp"], dtype, margins)
        x = x + mult * y
        if cfg.get("token_side"):
            x = x + mult * token_side(x, tokens, W, i, int(cfg["token_side"]["dim"]), eps, dtype)
        streams.append(x.clone())
    y = group_rms_norm(x, W["final.norm"], groups, eps).to(dtype)
    logits = linear(y, W["head"], dtype=dtype).float() * float(cfg["logit_scale"])
    return logits, torch.stack(streams)
