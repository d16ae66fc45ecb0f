"""Benarax: a decoder with a float32 residual stream, ONE grouped RMS norm per layer whose output feeds the token
mixer and the feed-forward side by side, a short causal convolution in front of every mixer, three kinds of mixer
chosen per layer, a mixture-of-experts feed-forward, a per-layer token table that enters the stream after the
feed-forward, and a span of layers that may run several times with shared weights.

  * `general_delta`       a recurrent mixer: per head a state S [D, D] with one decay and one removal rate per key
                          channel, S <- diag(w) S - (a * u)(u^T S) + k v^T (u the unit key), read out with r,
                          normalised per head, gated;
  * `latent_attention`    queries and keys / values through normalised low-rank latents; one rotated key part shared
                          by all heads; interleaved-pair rotary with blended (long-context) frequencies;
  * `latent_attention_2`  the same with the rotate-half pairing;
  * feed-forward          `top` of `experts` small clamped-GLU experts, weighted by a softmax over the chosen router
                          logits; absent where the config says null.

Per layer:  h = groupnorm(x);  x += m * (mixer(h + conv(h)) + ff(h));  x += m * rmsnorm(P (gelu(G x) * table[token])) * w.

Only the latent c and the shared rotated key are cached per token: attention runs in the latent space (the key
up-projection is applied to the query, the value up-projection to the attention output), i.e. as multi-query attention
with key size kv_rank + rot_dim and value size kv_rank over the framework's paged attention kernels.

Execution order ("runs"): the layers before loop.start once, the layers loop.start .. loop.stop-1 loop.times times in
a row, the rest once.  Every run has its own caches: the convolution's carried inputs (a state slot), and a paged
latent cache or the recurrence's state slot.

Every size and constant comes from config.json (`BenaraxConfig.from_dict`).  The model is built from the package's
layers (`layers=` swaps in stand-ins, as for the other models); the matrix products are torch's.  What the design keeps
in 32 bits is kept there also when the model runs in bfloat16: the residual stream, norms, router, rotary angles,
scores, the recurrence and its gates.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..engine.cache_spec import PagedKVSpec, SlotStateSpec
from ..utils.cache_context import get_context
from .buvalix import _FusedInputs, _linear

LATENT_KINDS = {"latent_attention": True, "latent_attention_2": False}      # kind -> interleaved rotary pairs


# ------------------------------------------------------------------------------------------------ configuration
@dataclass
class BenaraxMixerConfig:
    kind: str
    heads: int
    dim: int
    # latent attention only
    rot_dim: int = 0
    vdim: int = 0
    q_rank: int = 0
    kv_rank: int = 0
    scale: float = 0.0
    rot_base: float = 10000.0
    rot_scaling: dict | None = None


@dataclass
class BenaraxMoEConfig:
    experts: int
    top: int
    ff: int
    limit: float


@dataclass
class BenaraxLayerConfig:
    mixer: BenaraxMixerConfig
    mlp: BenaraxMoEConfig | None


@dataclass
class BenaraxConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    norm_groups: int
    residual_mult: float
    embedding_scale: float
    logit_scale: float
    canon_taps: int                  # 0: no input convolution
    side_dim: int                    # 0: no per-layer token table
    layers: list = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    eos_token_id: int | None = None
    max_position_embeddings: int | None = None

    @classmethod
    def from_dict(cls, d: dict) -> "BenaraxConfig":
        layers = []
        for L in d["layers"]:
            m, kind = L["mixer"], L["type"]
            mc = BenaraxMixerConfig(kind=kind, heads=int(m["heads"]), dim=int(m["dim"]))
            if kind in LATENT_KINDS:
                rot = m["rot"]
                mc.rot_dim, mc.vdim = int(m["rot_dim"]), int(m["vdim"])
                mc.q_rank, mc.kv_rank, mc.scale = int(m["q_rank"]), int(m["kv_rank"]), float(m["scale"])
                mc.rot_base, mc.rot_scaling = float(rot["base"]), rot.get("scaling")
                if int(rot.get("dims", mc.rot_dim)) != mc.rot_dim or mc.rot_dim % 2:
                    raise ValueError("the rotated part is rot_dim wide (even), and rot.dims must equal it")
            elif kind != "general_delta":
                raise ValueError(f"unknown mixer type {kind!r}")
            mlp = L.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "moe":
                    raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
                mlp = BenaraxMoEConfig(int(mlp["router"]["experts"]), int(mlp["router"]["top"]),
                                       int(mlp["expert"]["ff"]), float(mlp["expert"]["limit"]))
                if not 1 <= mlp.top <= mlp.experts:
                    raise ValueError("router.top must lie in 1 .. router.experts")
            layers.append(BenaraxLayerConfig(mc, mlp))
        loop = d.get("loop") or {}
        n = len(layers)
        cfg = cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                  norm_groups=int(d["norm"].get("groups", 1)), residual_mult=float(d.get("residual_mult", 1.0)),
                  embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                  logit_scale=float(d.get("logit_scale", 1.0)), canon_taps=int((d.get("canon") or {}).get("taps", 0)),
                  side_dim=int((d.get("token_side") or {}).get("dim", 0)), layers=layers,
                  loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
                  loop_times=int(loop.get("times", 1)), eos_token_id=d.get("eos_token_id"))
        if not (0 <= cfg.loop_start <= cfg.loop_stop <= n) or cfg.loop_times < 1:
            raise ValueError("loop must satisfy 0 <= start <= stop <= number of layers and times >= 1")
        if cfg.hidden_size % cfg.norm_groups:
            raise ValueError("norm.groups must divide the width")
        return cfg

    def runs(self) -> list[int]:
        """Layer indices in execution order."""
        return (list(range(self.loop_start)) + list(range(self.loop_start, self.loop_stop)) * self.loop_times
                + list(range(self.loop_stop, len(self.layers))))


def _default_layers():
    from ..layers import general_delta, latent_attention, moe, stream

    class _L:
        stream_boundary = staticmethod(stream.stream_boundary)
        rms_norm_rows = staticmethod(stream.rms_norm_rows)
        CausalConvAdd = stream.CausalConvAdd
        TokenGate = stream.TokenGate
        GeneralDeltaRule = general_delta.GeneralDeltaRule
        LatentAttention = latent_attention.LatentAttention
        MoEExperts = moe.MoEExperts
    return _L


# ------------------------------------------------------------------------------------------------ modules
class BenaraxGeneralDelta(nn.Module, _FusedInputs):
    _inputs = ("r", "k", "v", "a", "g", "w1")

    def __init__(self, m: BenaraxMixerConfig, width: int, eps: float, L, dtype, device):
        super().__init__()
        self.m = m
        n = m.heads * m.dim
        for name in ("r", "k", "v", "a", "g"):
            setattr(self, name, _linear(width, n, False, dtype, device))
        # the low-rank width is the file's (w1: [rank, width]); 1 here, resized when the weights arrive
        self.w1 = _linear(width, 1, False, dtype, device)
        self.w2 = _linear(1, n, False, dtype, device)
        self.o = _linear(n, width, False, dtype, device)
        self.rule = L.GeneralDeltaRule(m.heads, m.dim, eps, device=device)

    def cache_spec(self):
        return SlotStateSpec({"state": ((self.m.heads, self.m.dim, self.m.dim), torch.float32)})

    def finalize(self):
        if self.w2.weight.shape[1] != self.w1.weight.shape[0]:
            raise ValueError("low-rank decay projections do not chain")
        self._fuse(self._inputs)

    def forward(self, x, positions, cache):
        H, D = self.m.heads, self.m.dim
        r, k, v, a, g, w1 = self._project(x, self._inputs)
        w_raw = self.w2(torch.tanh(w1))
        o = self.rule(r.unflatten(1, (H, D)), k.unflatten(1, (H, D)), v.unflatten(1, (H, D)), w_raw, a, g,
                      cache["state"])
        return self.o(o)


class BenaraxLatentAttention(nn.Module, _FusedInputs):
    _inputs = ("dq", "dkv")

    def __init__(self, m: BenaraxMixerConfig, width: int, eps: float, L, dtype, device):
        super().__init__()
        self.m, self.eps, self._L = m, eps, L
        H = m.heads
        self.dq = _linear(width, m.q_rank, False, dtype, device)
        self.dkv = _linear(width, m.kv_rank + m.rot_dim, False, dtype, device)
        self.uq = _linear(m.q_rank, H * (m.dim + m.rot_dim), False, dtype, device)
        self.uk = _linear(m.kv_rank, H * m.dim, False, dtype, device)
        self.uv = _linear(m.kv_rank, H * m.vdim, False, dtype, device)
        self.o = _linear(H * m.vdim, width, False, dtype, device)
        self.dq_norm = nn.Parameter(torch.ones(m.q_rank, dtype=torch.float32, device=device))
        self.attn = L.LatentAttention(H, m.kv_rank, m.rot_dim, m.scale, eps, m.rot_base, m.rot_scaling,
                                      interleaved=LATENT_KINDS[m.kind], device=device)

    def cache_spec(self):
        # one key "head" [latent | rotated part]; the value of a token is the latent, i.e. the front of its key row
        return PagedKVSpec(1, self.m.kv_rank + self.m.rot_dim, self.m.kv_rank, value_in_key=True)

    def finalize(self):
        self._fuse(self._inputs)

    def forward(self, x, positions, cache):
        m, H = self.m, self.m.heads
        cq, ckv = self._project(x, self._inputs)
        q = self.uq(self._L.rms_norm_rows(cq, self.dq_norm, self.eps)).unflatten(1, (H, m.dim + m.rot_dim))
        # the key up-projection moves to the query: q_lat[t, h] = uk_h^T q_plain[t, h]
        q_lat = torch.bmm(q[:, :, :m.dim].transpose(0, 1), self.uk.weight.view(H, m.dim, m.kv_rank))      # [H, T, rank]
        o_lat = self.attn(q, q_lat.transpose(0, 1), ckv, positions, cache[0], cache[1])                   # [T, H, rank]
        # ... and the value up-projection to the output
        o = torch.bmm(o_lat.transpose(0, 1), self.uv.weight.view(H, m.vdim, m.kv_rank).transpose(1, 2))   # [H, T, vdim]
        return self.o(o.transpose(0, 1).reshape(x.shape[0], H * m.vdim))


class BenaraxMoE(nn.Module):
    def __init__(self, c: BenaraxMoEConfig, width: int, L, dtype, device):
        super().__init__()
        self.c = c
        self.router = nn.Parameter(torch.zeros(c.experts, width, dtype=torch.float32, device=device))
        # per expert [gate rows | up rows] x width, and down [width, ff]
        self.gate_up = nn.Parameter(torch.zeros(c.experts, 2 * c.ff, width, dtype=dtype, device=device))
        self.down = nn.Parameter(torch.zeros(c.experts, width, c.ff, dtype=dtype, device=device))
        self.experts = L.MoEExperts(c.top, c.limit)

    def forward(self, h, h32=None):
        """Returns the weighted expert outputs [T, top, width] float32; the stream update sums them.  The router reads
        the norm's float32 output where the step has it (h32), else h widened."""
        logits = F.linear(h32 if h32 is not None else h.float(), self.router)
        return self.experts(h, logits, self.gate_up, self.down)


class BenaraxSide(nn.Module):
    def __init__(self, width: int, dim: int, eps: float, index: int, L, dtype, device):
        super().__init__()
        self.gate = _linear(width, dim, False, dtype, device)
        self.proj = _linear(dim, width, False, dtype, device)
        self.norm = nn.Parameter(torch.ones(width, dtype=torch.float32, device=device))
        self.token_gate = L.TokenGate(index * dim, dim)


class BenaraxLayer(nn.Module):
    def __init__(self, index: int, lc: BenaraxLayerConfig, cfg: BenaraxConfig, L, dtype, device):
        super().__init__()
        W, eps = cfg.hidden_size, cfg.norm_eps
        self.norm1 = nn.Parameter(torch.ones(W, dtype=torch.float32, device=device))
        self.canon = L.CausalConvAdd(W, cfg.canon_taps, device=device) if cfg.canon_taps else None
        if lc.mixer.kind == "general_delta":
            self.mix = BenaraxGeneralDelta(lc.mixer, W, eps, L, dtype, device)
        else:
            self.mix = BenaraxLatentAttention(lc.mixer, W, eps, L, dtype, device)
        self.mlp = BenaraxMoE(lc.mlp, W, L, dtype, device) if lc.mlp is not None else None
        self.side = BenaraxSide(W, cfg.side_dim, eps, index, L, dtype, device) if cfg.side_dim else None


class BenaraxForCausalLM(nn.Module):
    #: the in-tree library this model's layers need (`nanovllm_amd._lib.build(target)`)
    kernel_library = "mixers"
    #: a cached prompt prefix cannot be taken over: the carried state at its end is not kept
    prefix_caching = False

    def __init__(self, cfg: BenaraxConfig, layers=None, dtype: torch.dtype = torch.bfloat16, device=None):
        super().__init__()
        L = layers if layers is not None else _default_layers()
        self.config, self.dtype, self._L = cfg, dtype, L
        self.embed = nn.Embedding(cfg.vocab_size, cfg.hidden_size, dtype=dtype, device=device)
        self.side_embed = None
        if cfg.side_dim:
            self.side_embed = nn.Parameter(torch.zeros(cfg.vocab_size, cfg.side_dim * len(cfg.layers), dtype=dtype,
                                                       device=device))
        self.layers = nn.ModuleList(BenaraxLayer(i, lc, cfg, L, dtype, device) for i, lc in enumerate(cfg.layers))
        self.final_norm = nn.Parameter(torch.ones(cfg.hidden_size, dtype=torch.float32, device=device))
        self.head = _linear(cfg.hidden_size, cfg.vocab_size, False, dtype, device)
        self._runs = cfg.runs()
        self._caches: list | None = None

    # ---- weights ----------------------------------------------------------------------------------------
    def checkpoint_names(self) -> dict[str, str]:
        """checkpoint tensor name -> parameter name of this module tree (the experts are stacked separately)."""
        names = {"embed": "embed.weight", "head": "head.weight", "final.norm": "final_norm"}
        if self.side_embed is not None:
            names["side.embed"] = "side_embed"
        for i, layer in enumerate(self.layers):
            p, t = f"l{i}.", f"layers.{i}."
            names[p + "norm1"] = t + "norm1"
            if layer.canon is not None:
                names[p + "canon1"] = t + "canon.weight"
            if self.config.layers[i].mixer.kind == "general_delta":
                for n in ("r", "k", "v", "a", "g", "w1", "w2", "o"):
                    names[p + "mix." + n] = t + f"mix.{n}.weight"
                names[p + "mix.a.b"] = t + "mix.rule.a_bias"
                names[p + "mix.w0"] = t + "mix.rule.w_bias"
                names[p + "mix.norm"] = t + "mix.rule.norm_weight"
            else:
                for n in ("dq", "uq", "dkv", "uk", "uv", "o"):
                    names[p + "mix." + n] = t + f"mix.{n}.weight"
                names[p + "mix.dq.norm"] = t + "mix.dq_norm"
                names[p + "mix.dkv.norm"] = t + "mix.attn.latent_norm"
            if layer.mlp is not None:
                names[p + "mlp.router"] = t + "mlp.router"
            if layer.side is not None:
                names[p + "side.gate"] = t + "side.gate.weight"
                names[p + "side.proj"] = t + "side.proj.weight"
                names[p + "side.norm"] = t + "side.norm"
        return names

    def load_tensors(self, tensors: dict[str, torch.Tensor]) -> None:
        """Copy checkpoint tensors (by checkpoint name) into the parameters.  The low-rank width of the decay
        projection is the file's; the experts of a layer are stacked into [experts, rows, cols] tensors."""
        names = self.checkpoint_names()
        params = dict(self.named_parameters())
        seen = set()
        with torch.no_grad():
            for i, layer in enumerate(self.layers):
                if layer.mlp is None:
                    continue
                for e in range(layer.mlp.c.experts):
                    p = f"l{i}.mlp.e{e}."
                    for n in ("gate", "up", "down"):
                        if p + n not in tensors:
                            raise KeyError(f"checkpoint lacks {p + n}")
                    gu = torch.cat([tensors[p + "gate"], tensors[p + "up"]], dim=0)
                    if gu.shape != layer.mlp.gate_up.shape[1:] or tensors[p + "down"].shape != layer.mlp.down.shape[1:]:
                        raise ValueError(f"{p}*: expert shapes do not match the configuration")
                    layer.mlp.gate_up[e].copy_(gu)
                    layer.mlp.down[e].copy_(tensors[p + "down"])
                    seen.update(p + n for n in ("gate", "up", "down"))
            for ck, pn in names.items():
                if ck not in tensors:
                    raise KeyError(f"checkpoint lacks {ck}")
                t, p = tensors[ck], params[pn]
                if t.shape != p.shape:
                    free = pn.endswith((".w1.weight", ".w2.weight"))
                    if not free or t.dim() != p.dim():
                        raise ValueError(f"{ck}: checkpoint shape {tuple(t.shape)} != parameter {tuple(p.shape)}")
                    p.data = torch.empty(t.shape, dtype=p.dtype, device=p.device)
                p.copy_(t)
                seen.add(ck)
        extra = sorted(set(tensors) - seen)
        if extra:
            raise KeyError(f"checkpoint has tensors the model does not know, e.g. {extra[:3]}")
        self.finalize()

    def finalize(self) -> "BenaraxForCausalLM":
        for layer in self.layers:
            layer.mix.finalize()
        return self

    # ---- caches -------------------------------------------------------------------------------------------
    def cache_specs(self) -> list:
        """Per run, in execution order: the convolution's carried inputs (when the design has one), then the mixer's
        paged latent cache or state."""
        cfg, specs = self.config, []
        for i in self._runs:
            if cfg.canon_taps:
                specs.append(SlotStateSpec({"inputs": ((cfg.canon_taps - 1, cfg.hidden_size), torch.float32)}))
            specs.append(self.layers[i].mix.cache_spec())
        return specs

    def bind_caches(self, caches: list) -> None:
        per = 2 if self.config.canon_taps else 1
        assert len(caches) == per * len(self._runs)
        self._caches = [(caches[per * r]["inputs"] if per == 2 else None, caches[per * r + per - 1])
                        for r in range(len(self._runs))]

    # ---- forward ------------------------------------------------------------------------------------------
    def forward(self, input_ids, positions, logits_rows=None, streams: list | None = None):
        """Returns float32 logits [T or len(logits_rows), vocab].  streams: a list that receives the residual stream
        after every run."""
        if self._caches is None:
            raise RuntimeError("caches are not bound: the model runs through the engine's cache and state manager")
        cfg, L, dt = self.config, self._L, self.dtype
        eps, groups, mult = cfg.norm_eps, cfg.norm_groups, cfg.residual_mult
        x = self.embed(input_ids).float() * cfg.embedding_scale
        ctx = get_context()
        h32, h = L.stream_boundary(x, norm=self.layers[self._runs[0]].norm1, groups=groups, eps=eps, out_dtype=dt,
                                   want_f32=cfg.canon_taps > 0)
        last = len(self._runs) - 1
        for run, i in enumerate(self._runs):
            layer = self.layers[i]
            ctx.layer_idx = run
            conv_state, cache = self._caches[run]
            hm = layer.canon(h32, conv_state, dt) if layer.canon is not None else h
            mix = layer.mix(hm, positions, cache)
            ff = layer.mlp(h, h32) if layer.mlp is not None else None
            nxt = self.layers[self._runs[run + 1]].norm1 if run < last else self.final_norm
            if run == last and logits_rows is not None and streams is None:
                # only the asked rows go on: the caches and states of this step are complete
                x, mix, input_ids = x[logits_rows], mix[logits_rows], input_ids[logits_rows]
                ff = ff[logits_rows] if ff is not None else None
                logits_rows = None
            want32 = cfg.canon_taps > 0 and run < last
            if layer.side is not None:
                xb = L.stream_boundary(x, add=mix, add_parts=ff, mult=mult, copy_dtype=dt)
                g = layer.side.token_gate(layer.side.gate(xb), self.side_embed, input_ids)
                y = layer.side.proj(g)
                if streams is not None:
                    L.stream_boundary(x, normed=y, normed_weight=layer.side.norm, mult=mult, eps=eps)
                    streams.append(x.clone())
                    h32, h = L.stream_boundary(x, norm=nxt, groups=groups, eps=eps, out_dtype=dt, want_f32=want32)
                else:
                    h32, h = L.stream_boundary(x, normed=y, normed_weight=layer.side.norm, mult=mult, norm=nxt,
                                               groups=groups, eps=eps, out_dtype=dt, want_f32=want32)
            else:
                if streams is not None:
                    L.stream_boundary(x, add=mix, add_parts=ff, mult=mult)
                    streams.append(x.clone())
                    h32, h = L.stream_boundary(x, norm=nxt, groups=groups, eps=eps, out_dtype=dt, want_f32=want32)
                else:
                    h32, h = L.stream_boundary(x, add=mix, add_parts=ff, mult=mult, norm=nxt, groups=groups, eps=eps,
                                               out_dtype=dt, want_f32=want32)
        if logits_rows is not None:
            h = h[logits_rows]
        return self.head(h).float() * cfg.logit_scale
