"""Oracle (test infrastructure): a plain, slow restatement of the Buvalix design, one function per
mechanism, whole sequences at a time, no cache and no batching.  It shares nothing with the product
path: tests compare the engine (paged cache, state slots, chunked prompts, mixed batches, HIP kernels)
with these functions.

`dtype=torch.float32` computes everything in 32-bit.  With `torch.bfloat16` the matrix products take
bfloat16 operands (fp32 accumulation, bfloat16 result) and everything the design keeps in 32-bit stays there.

A model is (cfg, weights): cfg the parsed config.json, weights a dict name -> tensor as stored.
"""
from __future__ import annotations

import math

import torch


# ------------------------------------------------------------------------------------------ small pieces
def linear(x, w, b=None, dtype=torch.float32):
    """W x (+ b), operands in `dtype`, result in `dtype`."""
    y = torch.nn.functional.linear(x.to(dtype), w.to(dtype), None if b is None else b.to(dtype))
    return y


def layer_norm(x, w, b, eps):
    x = x.float()
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w.float() + b.float()


def rms_unit(x, eps):
    x = x.float()
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotary_interleaved(x, positions, dims, base):
    """x: [T, H, D]; rotates pairs (2i, 2i+1) of the first `dims` dimensions by positions * base^(-2i/dims)."""
    x = x.float()
    i = torch.arange(dims // 2, dtype=torch.float64)
    freq = (float(base) ** (-2.0 * i / dims)).float()                       # [dims/2]
    ang = positions.float()[:, None] * freq[None, :]                        # fp32 product
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Exact below rows/2, logarithmic up to `far`, then the last row."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def query_temperature(positions, coef, every):
    return 1.0 + coef * torch.log(torch.floor((positions.float() + 1.0) / every) + 1.0)


def causal_attention(q, k, v, scale, softcap=None, sink=None, rel=None, far=None):
    """q: [T, H, D], k: [T, G, D], v: [T, G, Dv], all fp32 scores.  sink: [H] extra denominator term;
    rel: [rows, H] distance bias with bucket(i - j)."""
    T, H, _ = q.shape
    G = k.shape[1]
    q, k, v = q.float(), k.float(), v.float()
    out = torch.zeros(T, H, v.shape[-1])
    idx = torch.arange(T)
    dist = (idx[:, None] - idx[None, :])
    visible = dist >= 0
    if rel is not None:
        rows = rel.shape[0]
        table = torch.tensor([distance_bucket(n, rows, far) for n in range(T)], dtype=torch.long)
        buckets = table[dist.clamp(min=0)]
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        if rel is not None:
            s = s + rel.float()[:, h][buckets]
        s = s.masked_fill(~visible, float("-inf"))
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink.float()[h].expand_as(m))
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink.float()[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def short_conv_silu(x, w, dtype=torch.float32):
    """x: [T, C]; w: [C, taps], last column multiplies the current token; zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, C, dtype=torch.float32), x.float()], 0)
    y = torch.zeros(T, C)
    for j in range(taps):
        y = y + xp[j:j + T] * w.float()[:, j]
    y = y.to(dtype).float()
    return torch.nn.functional.silu(y).to(dtype)


def gated_delta_channel(q, k, v, beta, g):
    """The recurrence of one head, written as three assignments per token t (S_t is [D, Dv], rows indexed by key channel):
        A   = Diag(g_t) S_{t-1}                 decay
        S_t = A + k_t (beta_t (v_t - A^T k_t))^T  delta-rule write
        o_t = S_t^T q_t                          read after the write
    q, k: [T, H, D]; v: [T, H, Dv]; beta: [T, H]; g: [T, H, D].  S_0 = 0, float32 throughout."""
    T, H, D = q.shape
    Dv = v.shape[-1]
    S = torch.zeros(H, D, Dv)
    out = torch.zeros(T, H, Dv)
    for t in range(T):
        S = S * g[t][:, :, None]
        u = beta[t][:, None] * (v[t] - torch.einsum("hdv,hd->hv", S, k[t]))
        S = S + k[t][:, :, None] * u[:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


# ------------------------------------------------------------------------------------------ mixers
def mixer_attention(h, positions, m, W, pre, dtype):
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = linear(h, W[pre + "q"], W[pre + "q.b"], dtype).view(T, H, D)
    k = linear(h, W[pre + "k"], W[pre + "k.b"], dtype).view(T, G, D)
    v = linear(h, W[pre + "v"], W[pre + "v.b"], dtype).view(T, G, Dv)
    q = rotary_interleaved(q, positions, m["rot"]["dims"], m["rot"]["base"]).to(dtype)
    k = rotary_interleaved(k, positions, m["rot"]["dims"], m["rot"]["base"]).to(dtype)
    o = causal_attention(q, k, v, m["scale"], m.get("softcap"), sink=W[pre + "sink"])
    return linear(o.reshape(T, H * Dv), W[pre + "o"], None, dtype)


def mixer_attention_2(h, positions, m, W, pre, dtype):
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = linear(h, W[pre + "q"], None, dtype).view(T, H, D)
    k = linear(h, W[pre + "k"], None, dtype).view(T, G, D)
    v = linear(h, W[pre + "v"], None, dtype).view(T, G, Dv)
    temp = query_temperature(positions, m["q_temp"]["coef"], m["q_temp"]["every"])
    q = (q.float() * temp[:, None, None]).to(dtype)
    o = causal_attention(q, k, v, m["scale"], m.get("softcap"), rel=W[pre + "rel"], far=m["bias_max"])
    return linear(o.reshape(T, H * Dv), W[pre + "o"], None, dtype)


def mixer_channel_delta(h, m, W, pre, eps, dtype):
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    rep = H // G
    q = short_conv_silu(linear(h, W[pre + "q"], None, dtype), W[pre + "q.conv"], dtype).float().view(T, G, D)
    k = short_conv_silu(linear(h, W[pre + "k"], None, dtype), W[pre + "k.conv"], dtype).float().view(T, G, D)
    v = short_conv_silu(linear(h, W[pre + "v"], None, dtype), W[pre + "v.conv"], dtype).float().view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q = q.repeat_interleave(rep, dim=1)
    k = k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(linear(h, W[pre + "b"], None, dtype).float())                                 # [T, H]
    a = linear(linear(h, W[pre + "a1"], None, dtype), W[pre + "a2"], None, dtype).float() + W[pre + "dt_bias"].float()
    rate = torch.exp(W[pre + "A_log"].float())[None, :, None]                                          # per head
    g = torch.exp(-rate * torch.nn.functional.softplus(a).view(T, H, D))
    o = gated_delta_channel(q, k, v, beta, g)                                                          # [T, H, Dv]
    gate = torch.sigmoid(linear(linear(h, W[pre + "g1"], None, dtype), W[pre + "g2"], None, dtype).float()).view(T, H, Dv)
    o = rms_unit(o, eps) * W[pre + "norm"].float() * gate
    return linear(o.reshape(T, H * Dv), W[pre + "o"], None, dtype)


def feed_forward(h, W, pre, dtype):
    gate = linear(h, W[pre + "gate"], None, dtype)
    up = linear(h, W[pre + "up"], None, dtype)
    act = (gelu_tanh(gate.float()) * up.float()).to(dtype)
    return linear(act, W[pre + "down"], None, dtype)


# ------------------------------------------------------------------------------------------ whole model
def layer_runs(cfg):
    """Layer indices in execution order, with a flag on the run that opens a repeated pass."""
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    runs = [(i, False) for i in range(loop["start"])]
    for p in range(loop["times"]):
        for i in range(loop["start"], loop["stop"]):
            runs.append((i, p > 0 and i == loop["start"]))
    runs += [(i, False) for i in range(loop["stop"], n)]
    return runs


def forward(cfg, W, tokens, dtype=torch.float32):
    """Returns (logits [T, vocab] fp32, residual stream after every layer run [runs, T, width])."""
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    x0 = W["embed"][tokens].float()
    x = x0.clone()
    streams = []
    for i, reopen in layer_runs(cfg):
        L = cfg["layers"][i]
        p = f"l{i}."
        if reopen:
            x = x + x0
        h = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps).to(dtype)
        if L["type"] == "attention":
            y = mixer_attention(h, positions, L["mixer"], W, p + "mix.", dtype)
        elif L["type"] == "attention_2":
            y = mixer_attention_2(h, positions, L["mixer"], W, p + "mix.", dtype)
        elif L["type"] == "channel_delta":
            y = mixer_channel_delta(h, L["mixer"], W, p + "mix.", eps, dtype)
        else:
            raise ValueError(L["type"])
        x = x + layer_norm(y, W[p + "norm1b"], W[p + "norm1b.b"], eps)
        if L.get("mlp") is not None:
            h = layer_norm(x, W[p + "norm2"], W[p + "norm2.b"], eps).to(dtype)
            y = feed_forward(h, W, p + "mlp.", dtype)
            x = x + layer_norm(y, W[p + "norm2b"], W[p + "norm2b.b"], eps)
        streams.append(x.clone())
    h = layer_norm(x, W["final.norm"], W["final.norm.b"], eps).to(dtype)
    logits = linear(h, W["head"], None, dtype).float()
    return logits, torch.stack(streams)
