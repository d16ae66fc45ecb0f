"""Oracle (test infrastructure): torch stand-ins for the layers of the second kernel library (LayerNorm on an
fp32 stream, score-modified paged attention, short convolution and gated delta rule with state slots, tanh-GELU
gate), with the same constructors and the same cache / state layouts as the HIP-backed modules.  They let the
whole engine (scheduler, block and slot managers, runner, model) run without a GPU, and give GPU tests an eager
reference per layer.  Device-agnostic, slow, written from the layer contracts; the product model never imports it."""
from __future__ import annotations

import math

import torch
import torch.nn as nn


def _ctx():
    import nanovllm_amd
    return nanovllm_amd.get_context()


class LayerNorm(nn.Module):
    def __init__(self, hidden_size, eps=1e-5, device=None):
        super().__init__()
        self.hidden_size, self.eps = hidden_size, eps
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=torch.float32, device=device))
        self.bias = nn.Parameter(torch.zeros(hidden_size, dtype=torch.float32, device=device))

    def normalize(self, x):
        x = x.float()
        mu = x.mean(-1, keepdim=True)
        var = ((x - mu) ** 2).mean(-1, keepdim=True)
        return (x - mu) / torch.sqrt(var + self.eps) * self.weight + self.bias

    def forward(self, x, out_dtype=torch.float32):
        return self.normalize(x).to(out_dtype)


def residual_boundary(resid, h=None, post=None, extra=None, pre=None, out_dtype=torch.float32):
    if h is not None:
        resid += post.normalize(h)
    if extra is not None:
        resid += extra
    return pre.normalize(resid).to(out_dtype) if pre is not None else None


class GeluTanhAndMul(nn.Module):
    def forward(self, x):
        g, u = x.float().chunk(2, dim=-1)
        return (0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g ** 3))) * u).to(x.dtype)


class ScoreModAttention(nn.Module):
    def __init__(self, num_heads, num_kv_heads, head_dim, v_head_dim, scale, softcap=0.0, rot_dims=0,
                 rot_base=10000.0, temp_coef=0.0, temp_every=0, use_sink=False, device=None):
        super().__init__()
        self.H, self.G, self.D, self.Dv = num_heads, num_kv_heads, head_dim, v_head_dim
        self.scale, self.softcap = float(scale), float(softcap or 0.0)
        self.rot_dims, self.rot_base = int(rot_dims), float(rot_base)
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        self.sink = nn.Parameter(torch.zeros(num_heads, dtype=torch.float32, device=device)) if use_sink else None
        self.dist_bias = None

    def set_distance_bias(self, table):
        self.dist_bias = None if table is None else table.float()

    def _rotate(self, x, positions):
        if not self.rot_dims:
            return x.float()
        n = self.rot_dims
        i = torch.arange(n // 2, dtype=torch.float64)
        f = (self.rot_base ** (-2.0 * i / n)).float().to(x.device)
        ang = positions.float()[:, None] * f[None, :]
        c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
        x = x.float().clone()
        a, b = x[..., 0:n:2].clone(), x[..., 1:n:2].clone()
        x[..., 0:n:2] = a * c - b * s
        x[..., 1:n:2] = b * c + a * s
        return x

    def forward(self, q, k, v, positions, k_cache, v_cache):
        ctx = _ctx()
        dt = q.dtype
        q, k = self._rotate(q, positions), self._rotate(k, positions)
        if self.temp_every:
            temp = 1.0 + self.temp_coef * torch.log(torch.floor((positions.float() + 1.0) / self.temp_every) + 1.0)
            q = q * temp[:, None, None]
        q = q.to(dt)
        bs = k_cache.shape[1]
        slots = ctx.slot_mapping.long()
        k_cache.view(-1, self.G, self.D)[slots] = k.to(dt)
        v_cache.view(-1, self.G, self.Dv)[slots] = v.to(dt)
        cu_q, cu_k = ctx.cu_seqlens_q.tolist(), ctx.cu_seqlens_k.tolist()
        out = torch.zeros(q.shape[0], self.H, self.Dv, dtype=torch.float32, device=q.device)
        for b in range(len(cu_q) - 1):
            nq, nk = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
            if nq == 0:
                continue
            pos_k = torch.arange(nk, device=q.device)
            rows = ctx.block_tables[b].long()[pos_k // bs] * bs + pos_k % bs
            kk = k_cache.view(-1, self.G, self.D)[rows].float()
            vv = v_cache.view(-1, self.G, self.Dv)[rows].float()
            pos_q = nk - nq + torch.arange(nq, device=q.device)
            dist = pos_q[:, None] - pos_k[None, :]
            for h in range(self.H):
                g = h // (self.H // self.G)
                s = (q[cu_q[b]:cu_q[b + 1], h].float() @ kk[:, g].T) * self.scale
                if self.softcap:
                    s = self.softcap * torch.tanh(s / self.softcap)
                if self.dist_bias is not None:
                    tab = self.dist_bias[h].to(q.device)
                    s = s + tab[dist.clamp(0, tab.numel() - 1)]
                s = s.masked_fill(dist < 0, float("-inf"))
                if self.sink is not None:
                    s = torch.cat([s, self.sink[h].expand(nq, 1)], dim=1)
                p = torch.softmax(s, dim=-1)[:, :nk]
                out[cu_q[b]:cu_q[b + 1], h] = p @ vv[:, g]
        return out.reshape(q.shape[0], self.H * self.Dv).to(dt)


class ShortConvSilu(nn.Module):
    def __init__(self, channels, taps, device=None):
        super().__init__()
        self.channels, self.taps = channels, taps
        self.weight = nn.Parameter(torch.zeros(channels, taps, dtype=torch.float32, device=device))

    def forward(self, x, conv_state):
        ctx = _ctx()
        cu_q, cu_k, slots = ctx.cu_seqlens_q.tolist(), ctx.cu_seqlens_k.tolist(), ctx.state_slots.tolist()
        keep = self.taps - 1
        y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        for b, slot in enumerate(slots):
            nq, nk = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
            if nq == 0:
                continue
            past = conv_state[slot].clone() if nk > nq else torch.zeros_like(conv_state[slot])
            if 0 < nk - nq < keep:                       # fewer inputs so far than the state has rows
                past[:keep - (nk - nq)] = 0
            seq = torch.cat([past, x[cu_q[b]:cu_q[b + 1]]], dim=0)
            acc = torch.zeros(nq, self.channels, dtype=torch.float32, device=x.device)
            for j in range(self.taps):
                acc += seq[j:j + nq].float() * self.weight[:, j]
            y[cu_q[b]:cu_q[b + 1]] = torch.nn.functional.silu(acc).to(x.dtype)
            conv_state[slot] = seq[seq.shape[0] - keep:]
        return y


class GatedDeltaRule(nn.Module):
    def __init__(self, num_heads, num_qk_heads, head_dim, v_head_dim, eps, device=None):
        super().__init__()
        self.H, self.G, self.D, self.Dv, self.eps = num_heads, num_qk_heads, head_dim, v_head_dim, eps
        f32 = dict(dtype=torch.float32, device=device)
        self.A_log = nn.Parameter(torch.zeros(num_heads, **f32))
        self.dt_bias = nn.Parameter(torch.zeros(num_heads * head_dim, **f32))
        self.norm_weight = nn.Parameter(torch.ones(v_head_dim, **f32))

    def forward(self, q, k, v, a_raw, b_raw, gate_raw, state):
        ctx = _ctx()
        cu_q, cu_k, slots = ctx.cu_seqlens_q.tolist(), ctx.cu_seqlens_k.tolist(), ctx.state_slots.tolist()
        T, H, D, Dv, rep = q.shape[0], self.H, self.D, self.Dv, self.H // self.G
        qf, kf = q.float(), k.float()
        qf = qf / torch.sqrt((qf * qf).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        kf = kf / torch.sqrt((kf * kf).sum(-1, keepdim=True) + 1e-6)
        qf, kf = qf.repeat_interleave(rep, dim=1), kf.repeat_interleave(rep, dim=1)
        beta = torch.sigmoid(b_raw.float())
        g = torch.exp(-torch.exp(self.A_log)[None, :, None]
                      * torch.nn.functional.softplus(a_raw.float() + self.dt_bias).view(T, H, D))
        out = torch.zeros(T, H, Dv, dtype=torch.float32, device=q.device)
        for b, slot in enumerate(slots):
            nq, nk = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
            if nq == 0:
                continue
            S = state[slot].clone() if nk > nq else torch.zeros_like(state[slot])
            for t in range(cu_q[b], cu_q[b + 1]):
                S = S * g[t][:, :, None]
                u = beta[t][:, None] * (v[t].float() - torch.einsum("hdv,hd->hv", S, kf[t]))
                S = S + kf[t][:, :, None] * u[:, None, :]
                out[t] = torch.einsum("hdv,hd->hv", S, qf[t])
            state[slot] = S
        out = out / torch.sqrt((out * out).mean(-1, keepdim=True) + self.eps) * self.norm_weight
        out = out * torch.sigmoid(gate_raw.float()).view(T, H, Dv)
        return out.reshape(T, H * Dv).to(q.dtype)
