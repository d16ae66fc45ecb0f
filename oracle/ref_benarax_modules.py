"""Oracle (test infrastructure): torch stand-ins for the layers Benarax is built from (grouped-norm stream boundary,
causal convolution with carried inputs, token gate, generalized delta rule with state slots, latent attention over
the paged latent cache, routed experts), with the same constructors and the same cache / state layouts as the
HIP-backed modules.  They let the whole engine run without a GPU and give GPU tests an eager reference per layer.
Device-agnostic, slow, written from the layer contracts; the product model never imports it."""
from __future__ import annotations

import math

import torch
import torch.nn as nn


def _ctx():
    import nanovllm_amd
    return nanovllm_amd.get_context()


def _unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm_rows(x, weight, eps):
    return (_unit_rms(x.float(), eps) * weight).to(x.dtype)


def stream_boundary(x, add=None, add_parts=None, normed=None, normed_weight=None, mult=1.0, norm=None, groups=1,
                    eps=1e-5, out_dtype=None, want_f32=False, copy_dtype=None):
    if add is not None or add_parts is not None:
        y = torch.zeros_like(x)
        if add is not None:
            y = y + add.float()
        if add_parts is not None:
            for j in range(add_parts.shape[1]):
                y = y + add_parts[:, j].float()
        x += mult * y
    if normed is not None:
        x += mult * (_unit_rms(normed.float(), eps) * normed_weight)
    if norm is not None:
        T, W = x.shape
        h32 = _unit_rms(x.view(T, groups, W // groups), eps).reshape(T, W) * norm
        return (h32 if want_f32 else None), h32.to(out_dtype or torch.float32)
    if copy_dtype is not None:
        return x.to(copy_dtype)
    return None


class CausalConvAdd(nn.Module):
    def __init__(self, channels, taps, device=None):
        super().__init__()
        self.channels, self.taps = channels, taps
        self.weight = nn.Parameter(torch.zeros(channels, taps, dtype=torch.float32, device=device))

    def forward(self, x, state, out_dtype):
        ctx = _ctx()
        cu_q, cu_k, slots = ctx.cu_seqlens_q.tolist(), ctx.cu_seqlens_k.tolist(), ctx.state_slots.tolist()
        keep = self.taps - 1
        y = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        for b, slot in enumerate(slots):
            nq, nk = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
            if nq == 0:
                continue
            past = state[slot].clone() if nk > nq else torch.zeros_like(state[slot])
            if 0 < nk - nq < keep:
                past[:keep - (nk - nq)] = 0
            seq = torch.cat([past, x[cu_q[b]:cu_q[b + 1]]], dim=0)
            acc = x[cu_q[b]:cu_q[b + 1]].clone()
            for j in range(self.taps):
                acc += seq[j:j + nq] * self.weight[:, j]
            y[cu_q[b]:cu_q[b + 1]] = acc.to(out_dtype)
            state[slot] = seq[seq.shape[0] - keep:]
        return y


class TokenGate(nn.Module):
    def __init__(self, offset, dim):
        super().__init__()
        self.offset, self.dim = offset, dim

    def forward(self, z, table, ids):
        e = table[ids, self.offset:self.offset + self.dim].float()
        z = z.float()
        g = 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))
        return (g * e).to(table.dtype)


class GeneralDeltaRule(nn.Module):
    def __init__(self, num_heads, head_dim, eps, decay_rate=math.exp(-0.5), key_eps=1e-6, device=None):
        super().__init__()
        self.H, self.D, self.eps, self.decay_rate, self.key_eps = num_heads, head_dim, eps, decay_rate, key_eps
        f32 = dict(dtype=torch.float32, device=device)
        self.a_bias = nn.Parameter(torch.zeros(num_heads * head_dim, **f32))
        self.w_bias = nn.Parameter(torch.zeros(num_heads * head_dim, **f32))
        self.norm_weight = nn.Parameter(torch.ones(num_heads * head_dim, **f32))

    def forward(self, r, k, v, w_raw, a_raw, gate_raw, state):
        ctx = _ctx()
        cu_q, cu_k, slots = ctx.cu_seqlens_q.tolist(), ctx.cu_seqlens_k.tolist(), ctx.state_slots.tolist()
        T, H, D = r.shape[0], self.H, self.D
        r, k, v = r.float(), k.float(), v.float()
        u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + self.key_eps)
        w = torch.exp(-self.decay_rate * torch.sigmoid(w_raw.float() + self.w_bias)).view(T, H, D)
        a = torch.sigmoid(a_raw.float() + self.a_bias).view(T, H, D)
        out = torch.zeros(T, H, D, dtype=torch.float32, device=r.device)
        for b, slot in enumerate(slots):
            nq, nk = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
            if nq == 0:
                continue
            S = state[slot].clone() if nk > nq else torch.zeros_like(state[slot])
            for t in range(cu_q[b], cu_q[b + 1]):
                uS = torch.einsum("hk,hkv->hv", u[t], S)
                S = w[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
                out[t] = torch.einsum("hkv,hk->hv", S, r[t])
            state[slot] = S
        out = _unit_rms(out, self.eps).reshape(T, H * D) * self.norm_weight * torch.sigmoid(gate_raw.float())
        return out.to(gate_raw.dtype)


def blended_frequencies(dims, base, scaling):
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


class LatentAttention(nn.Module):
    def __init__(self, num_heads, rank, rot_dim, scale, eps, rot_base=10000.0, rot_scaling=None, interleaved=True,
                 device=None):
        super().__init__()
        self.H, self.rank, self.R, self.scale, self.eps, self.interleaved = num_heads, rank, rot_dim, float(scale), eps, interleaved
        self.latent_norm = nn.Parameter(torch.ones(rank, dtype=torch.float32, device=device))
        f, self.mag = blended_frequencies(rot_dim, rot_base, rot_scaling)
        self.register_buffer("freq", f.to(device) if device is not None else f, persistent=False)

    def _rotate(self, x, positions):
        ang = positions.float()[:, None] * self.freq[None, :]
        c, s = (torch.cos(ang) * self.mag)[:, None, :], (torch.sin(ang) * self.mag)[:, None, :]
        x = x.float()
        out = torch.empty_like(x)
        half = self.R // 2
        if self.interleaved:
            a, b = x[..., 0::2], x[..., 1::2]
            out[..., 0::2], out[..., 1::2] = a * c - b * s, b * c + a * s
        else:
            a, b = x[..., :half], x[..., half:]
            out[..., :half], out[..., half:] = a * c - b * s, b * c + a * s
        return out

    def forward(self, q, q_lat, ckv, positions, k_cache, v_cache):
        ctx = _ctx()
        dt, T, H, rank, R = q.dtype, q.shape[0], self.H, self.rank, self.R
        c = (_unit_rms(ckv[:, :rank].float(), self.eps) * self.latent_norm).to(dt)
        k_rot = self._rotate(ckv[:, None, rank:], positions)[:, 0].to(dt)
        q_full = torch.cat([q_lat.float(), self._rotate(q[:, :, q.shape[2] - R:], positions)], dim=-1).to(dt)
        bs = k_cache.shape[1]
        slots = ctx.slot_mapping.long()
        k_cache.view(-1, rank + R)[slots] = torch.cat([c, k_rot], dim=-1)
        if v_cache.data_ptr() != k_cache.data_ptr():      # (else the values are the front of the key rows)
            v_cache.view(-1, rank)[slots] = c
        cu_q, cu_k = ctx.cu_seqlens_q.tolist(), ctx.cu_seqlens_k.tolist()
        out = torch.zeros(T, H, rank, dtype=torch.float32, device=q.device)
        for b in range(len(cu_q) - 1):
            nq, nk = cu_q[b + 1] - cu_q[b], cu_k[b + 1] - cu_k[b]
            if nq == 0:
                continue
            pos_k = torch.arange(nk, device=q.device)
            rows = ctx.block_tables[b].long()[pos_k // bs] * bs + pos_k % bs
            kk, vv = k_cache.view(-1, rank + R)[rows].float(), v_cache.reshape(-1, rank)[rows].float()
            pos_q = nk - nq + torch.arange(nq, device=q.device)
            s = torch.einsum("ihd,jd->hij", q_full[cu_q[b]:cu_q[b + 1]].float(), kk) * self.scale
            s = s.masked_fill((pos_q[:, None] < pos_k[None, :])[None], float("-inf"))
            out[cu_q[b]:cu_q[b + 1]] = torch.einsum("hij,jd->ihd", torch.softmax(s, dim=-1), vv)
        return out.to(dt)


class MoEExperts(nn.Module):
    def __init__(self, top, limit, alpha=1.702):
        super().__init__()
        self.top, self.limit, self.alpha = top, float(limit), float(alpha)

    def forward(self, h, logits, gate_up, down):
        T, ff, dt = h.shape[0], gate_up.shape[1] // 2, h.dtype
        val, idx = logits.float().topk(self.top, dim=-1)
        wgt = torch.softmax(val, dim=-1)
        out = torch.zeros(T, self.top, down.shape[1], dtype=torch.float32, device=h.device)
        for e in idx.unique().tolist():
            t, j = (idx == e).nonzero(as_tuple=True)
            gu = torch.nn.functional.linear(h[t], gate_up[e]).float()
            g, u = gu[:, :ff].clamp(max=self.limit), gu[:, ff:].clamp(-self.limit, self.limit)
            y = (g * torch.sigmoid(self.alpha * g) * (u + 1)).to(dt)
            out[t, j] = torch.nn.functional.linear(y, down[e]).float() * wgt[t, j][:, None]
        return out
