"""Buvalix: a decoder with a float32 residual stream, a LayerNorm before AND after every sublayer, three kinds
of token mixer chosen per layer, and a span of layers that may run several times with shared weights.

  * `attention`     grouped-query attention with biased projections, interleaved-pair rotary on the first
                    rot.dims dimensions, soft-capped scores and a learned per-head sink in the softmax denominator;
  * `attention_2`   no rotary: a position-dependent query temperature, soft-capped scores plus a learned per-head
                    bias by bucketed distance (exact buckets up close, logarithmic up to bias_max, then one row);
  * `channel_delta` a recurrent mixer: q / k / v through a short causal convolution and SiLU, then the gated delta
                    rule with one decay per head and key channel, a normalised read-out and an output gate;
  * feed-forward    down(gelu_tanh(gate x) * (up x)), absent where the config says null.

Execution order ("runs"): the layers before loop.start once, the layers loop.start .. loop.stop-1 loop.times times in
a row, the rest once.  Every run has its own paged KV cache or its own state slots (the weights are shared, the
history is not); before each repeated pass the embedding output is added to the stream again.

Every size and constant comes from config.json (`BuvalixConfig.from_dict`).  The model is built from the package's
layers (`layers=` swaps in stand-ins, as for the other model): LayerNorm / residual_boundary, ScoreModAttention,
ShortConvSilu, GatedDeltaRule, GeluTanhAndMul; the matrix products are torch's.  What the design keeps in 32 bits is
kept there also when the model runs in bfloat16: the residual stream, norms, scores, the recurrence and its gates.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..engine.cache_spec import PagedKVSpec, SlotStateSpec
from ..utils.cache_context import get_context


# ------------------------------------------------------------------------------------------------ configuration
@dataclass
class MixerConfig:
    kind: str
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float = 0.0
    softcap: float = 0.0
    rot_dims: int = 0
    rot_base: float = 10000.0
    temp_coef: float = 0.0
    temp_every: int = 0
    bias_max: float = 0.0
    conv: int = 0


@dataclass
class LayerConfig:
    mixer: MixerConfig
    ff: int | None          # None: the layer has no feed-forward sublayer


@dataclass
class BuvalixConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: list = field(default_factory=list)
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    eos_token_id: int | None = None
    max_position_embeddings: int | None = None      # the design has no position table: no bound

    @classmethod
    def from_dict(cls, d: dict) -> "BuvalixConfig":
        layers = []
        for L in d["layers"]:
            m, kind = L["mixer"], L["type"]
            mc = MixerConfig(kind=kind, heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                             vdim=int(m["vdim"]))
            if kind in ("attention", "attention_2"):
                mc.scale = float(m["scale"])
                mc.softcap = float(m.get("softcap") or 0.0)
            if kind == "attention":
                mc.rot_dims, mc.rot_base = int(m["rot"]["dims"]), float(m["rot"]["base"])
            elif kind == "attention_2":
                mc.temp_coef, mc.temp_every = float(m["q_temp"]["coef"]), int(m["q_temp"]["every"])
                mc.bias_max = float(m["bias_max"])
            elif kind == "channel_delta":
                mc.conv = int(m["conv"])
            else:
                raise ValueError(f"unknown mixer type {kind!r}")
            mlp = L.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") != "dense":
                raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
            layers.append(LayerConfig(mc, int(mlp["ff"]) if mlp is not None else None))
        loop = d.get("loop") or {}
        n = len(layers)
        cfg = cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                  layers=layers, loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
                  loop_times=int(loop.get("times", 1)), eos_token_id=d.get("eos_token_id"))
        if not (0 <= cfg.loop_start <= cfg.loop_stop <= n) or cfg.loop_times < 1:
            raise ValueError("loop must satisfy 0 <= start <= stop <= number of layers and times >= 1")
        return cfg

    def runs(self) -> list[tuple[int, bool]]:
        """(layer index, whether this run opens a repeated pass) in execution order."""
        out = [(i, False) for i in range(self.loop_start)]
        for p in range(self.loop_times):
            out += [(i, p > 0 and i == self.loop_start) for i in range(self.loop_start, self.loop_stop)]
        out += [(i, False) for i in range(self.loop_stop, len(self.layers))]
        return out


def distance_bias_table(rel: torch.Tensor, far: float) -> torch.Tensor:
    """Expand a bucketed table rel [rows, H] to one column per distance, [H, ceil(far) + 1]: distance n < rows/2 has
    its own row, larger ones share rows on a logarithmic scale that reaches the last row at `far`, and every distance
    from `far` on takes the last row (the attention kernel clamps the distance to the last column)."""
    rows = rel.shape[0]
    half = rows // 2
    n_dist = int(math.ceil(far)) + 1
    if far <= half or half < 1:
        raise ValueError(f"bias_max ({far}) must exceed half the number of table rows ({rows})")
    idx = []
    for n in range(n_dist):
        if n < half:
            idx.append(n)
        else:
            idx.append(min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half)))))
    return rel.float()[torch.tensor(idx, device=rel.device)].t().contiguous()


# ------------------------------------------------------------------------------------------------ modules
def _default_layers():
    from ..layers import activation, attention, delta_rule, layernorm

    class _L:
        LayerNorm = layernorm.LayerNorm
        residual_boundary = staticmethod(layernorm.residual_boundary)
        ScoreModAttention = attention.ScoreModAttention
        ShortConvSilu = delta_rule.ShortConvSilu
        GatedDeltaRule = delta_rule.GatedDeltaRule
        GeluTanhAndMul = activation.GeluTanhAndMul
    return _L


def _linear(n_in, n_out, bias, dtype, device):
    return nn.Linear(n_in, n_out, bias=bias, dtype=dtype, device=device)


class _FusedInputs:
    """Several projections of one input run as ONE matrix product: after `fuse()` the named nn.Linear weights are
    views of one [sum of outputs, inputs] tensor (names and values unchanged)."""

    def _fuse(self, names):
        mods = [getattr(self, n) for n in names]
        w = torch.cat([m.weight.data for m in mods], dim=0)
        has_bias = mods[0].bias is not None
        b = torch.cat([m.bias.data for m in mods], dim=0) if has_bias else None
        o = 0
        for m in mods:
            n = m.weight.shape[0]
            m.weight.data = w[o:o + n]
            if has_bias:
                m.bias.data = b[o:o + n]
            o += n
        self._fused_w, self._fused_b = w, b
        self._fused_sizes = [m.weight.shape[0] for m in mods]

    def _project(self, x, names):
        w = getattr(self, "_fused_w", None)
        if w is not None and w.device == x.device and w.dtype == x.dtype:
            return F.linear(x, w, self._fused_b).split(self._fused_sizes, dim=1)
        return tuple(getattr(self, n)(x) for n in names)


class BuvalixAttention(nn.Module, _FusedInputs):
    """Both attention mixers: `attention` (biases, rotary, sink) and `attention_2` (query temperature, distance bias)."""
    _inputs = ("q", "k", "v")

    def __init__(self, m: MixerConfig, width: int, L, dtype, device):
        super().__init__()
        self.m = m
        biased = m.kind == "attention"
        self.q = _linear(width, m.heads * m.dim, biased, dtype, device)
        self.k = _linear(width, m.kv_heads * m.dim, biased, dtype, device)
        self.v = _linear(width, m.kv_heads * m.vdim, biased, dtype, device)
        self.o = _linear(m.heads * m.vdim, width, False, dtype, device)
        self.attn = L.ScoreModAttention(m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.softcap, m.rot_dims,
                                        m.rot_base, m.temp_coef, m.temp_every, use_sink=biased, device=device)
        self.rel = None
        if m.kind == "attention_2":
            self.rel = nn.Parameter(torch.zeros(0, m.heads, dtype=torch.float32, device=device))   # rows from the file

    def cache_spec(self):
        return PagedKVSpec(self.m.kv_heads, self.m.dim, self.m.vdim)

    def finalize(self):
        self._fuse(self._inputs)
        if self.rel is not None:
            self.attn.set_distance_bias(distance_bias_table(self.rel.data, self.m.bias_max))

    def forward(self, x, positions, cache):
        m = self.m
        q, k, v = self._project(x, self._inputs)
        o = self.attn(q.unflatten(1, (m.heads, m.dim)), k.unflatten(1, (m.kv_heads, m.dim)),
                      v.unflatten(1, (m.kv_heads, m.vdim)), positions, cache[0], cache[1])
        return self.o(o)


class BuvalixChannelDelta(nn.Module, _FusedInputs):
    _inputs = ("q", "k", "v", "b", "a1", "g1")

    def __init__(self, m: MixerConfig, width: int, eps: float, L, dtype, device):
        super().__init__()
        self.m = m
        qk, vv = m.kv_heads * m.dim, m.heads * m.vdim
        self.q = _linear(width, qk, False, dtype, device)
        self.k = _linear(width, qk, False, dtype, device)
        self.v = _linear(width, vv, False, dtype, device)
        self.b = _linear(width, m.heads, False, dtype, device)
        # the low-rank widths are the files' (a1: [rank, width]); 1 here, resized when the weights arrive
        self.a1 = _linear(width, 1, False, dtype, device)
        self.a2 = _linear(1, m.heads * m.dim, False, dtype, device)
        self.g1 = _linear(width, 1, False, dtype, device)
        self.g2 = _linear(1, vv, False, dtype, device)
        self.o = _linear(vv, width, False, dtype, device)
        self.conv = L.ShortConvSilu(2 * qk + vv, m.conv, device=device)       # q | k | v channels in one launch
        self.rule = L.GatedDeltaRule(m.heads, m.kv_heads, m.dim, m.vdim, eps, device=device)
        self._qk, self._vv = qk, vv

    def cache_spec(self):
        m = self.m
        return SlotStateSpec({"conv": ((m.conv - 1, 2 * self._qk + self._vv), None),
                              "state": ((m.heads, m.dim, m.vdim), torch.float32)})

    def finalize(self):
        self._fuse(self._inputs)

    def forward(self, x, positions, cache):
        m, qk, vv = self.m, self._qk, self._vv
        w = getattr(self, "_fused_w", None)
        if w is not None and w.device == x.device and w.dtype == x.dtype:
            y = F.linear(x, w)
            qkv = y[:, :2 * qk + vv]
            b, a1, g1 = y[:, 2 * qk + vv:].split(self._fused_sizes[3:], dim=1)
        else:
            q, k, v, b, a1, g1 = self._project(x, self._inputs)
            qkv = torch.cat([q, k, v], dim=1)
        qkv = self.conv(qkv, cache["conv"])
        q = qkv[:, :qk].unflatten(1, (m.kv_heads, m.dim))
        k = qkv[:, qk:2 * qk].unflatten(1, (m.kv_heads, m.dim))
        v = qkv[:, 2 * qk:].unflatten(1, (m.heads, m.vdim))
        o = self.rule(q, k, v, self.a2(a1), b, self.g2(g1), cache["state"])
        return self.o(o)


class BuvalixMLP(nn.Module, _FusedInputs):
    _inputs = ("gate", "up")

    def __init__(self, width: int, ff: int, L, dtype, device):
        super().__init__()
        self.gate = _linear(width, ff, False, dtype, device)
        self.up = _linear(width, ff, False, dtype, device)
        self.down = _linear(ff, width, False, dtype, device)
        self.act = L.GeluTanhAndMul()

    def finalize(self):
        self._fuse(self._inputs)

    def forward(self, x):
        w = getattr(self, "_fused_w", None)
        if w is not None and w.device == x.device and w.dtype == x.dtype:
            return self.down(self.act(F.linear(x, w)))
        return self.down(self.act(torch.cat([self.gate(x), self.up(x)], dim=1)))


class BuvalixLayer(nn.Module):
    def __init__(self, lc: LayerConfig, cfg: BuvalixConfig, L, dtype, device):
        super().__init__()
        W, eps = cfg.hidden_size, cfg.norm_eps
        self.norm1, self.norm1b = L.LayerNorm(W, eps, device=device), L.LayerNorm(W, eps, device=device)
        if lc.mixer.kind == "channel_delta":
            self.mix = BuvalixChannelDelta(lc.mixer, W, eps, L, dtype, device)
        else:
            self.mix = BuvalixAttention(lc.mixer, W, L, dtype, device)
        self.mlp = None
        if lc.ff is not None:
            self.norm2, self.norm2b = L.LayerNorm(W, eps, device=device), L.LayerNorm(W, eps, device=device)
            self.mlp = BuvalixMLP(W, lc.ff, L, dtype, device)


class BuvalixForCausalLM(nn.Module):
    #: the in-tree library this model's layers need (`nanovllm_amd._lib.build(target)`)
    kernel_library = "mixers"
    #: a cached prompt prefix cannot be taken over: the recurrent layers' state at its end is not kept
    prefix_caching = False

    def __init__(self, cfg: BuvalixConfig, layers=None, dtype: torch.dtype = torch.bfloat16, device=None,
                 fused: bool = True):
        """fused: run each sublayer boundary (post-norm, stream update, next pre-norm) as one launch; False keeps
        them apart, and `forward(..., streams=[])` then collects the residual stream after every run."""
        super().__init__()
        L = layers if layers is not None else _default_layers()
        self.config, self.dtype, self.fused, self._L = cfg, dtype, fused, L
        self.embed = nn.Embedding(cfg.vocab_size, cfg.hidden_size, dtype=dtype, device=device)
        self.layers = nn.ModuleList(BuvalixLayer(lc, cfg, L, dtype, device) for lc in cfg.layers)
        self.final_norm = L.LayerNorm(cfg.hidden_size, cfg.norm_eps, device=device)
        self.head = _linear(cfg.hidden_size, cfg.vocab_size, False, dtype, device)
        self._runs = cfg.runs()
        self._caches: list | None = None

    # ---- weights ----------------------------------------------------------------------------------------
    def checkpoint_names(self) -> dict[str, str]:
        """checkpoint tensor name -> parameter name of this module tree."""
        names = {"embed": "embed.weight", "head": "head.weight", "final.norm": "final_norm.weight",
                 "final.norm.b": "final_norm.bias"}
        for i, layer in enumerate(self.layers):
            p, t = f"l{i}.", f"layers.{i}."
            norms = ["norm1", "norm1b"] + (["norm2", "norm2b"] if layer.mlp is not None else [])
            for n in norms:
                names[p + n] = t + n + ".weight"
                names[p + n + ".b"] = t + n + ".bias"
            kind = self.config.layers[i].mixer.kind
            if kind == "channel_delta":
                for n in ("q", "k", "v", "b", "a1", "a2", "g1", "g2", "o"):
                    names[p + "mix." + n] = t + f"mix.{n}.weight"
                names[p + "mix.A_log"] = t + "mix.rule.A_log"
                names[p + "mix.dt_bias"] = t + "mix.rule.dt_bias"
                names[p + "mix.norm"] = t + "mix.rule.norm_weight"
            else:
                for n in ("q", "k", "v", "o"):
                    names[p + "mix." + n] = t + f"mix.{n}.weight"
                if kind == "attention":
                    for n in ("q", "k", "v"):
                        names[p + f"mix.{n}.b"] = t + f"mix.{n}.bias"
                    names[p + "mix.sink"] = t + "mix.attn.sink"
                else:
                    names[p + "mix.rel"] = t + "mix.rel"
            if layer.mlp is not None:
                for n in ("gate", "up", "down"):
                    names[p + "mlp." + n] = t + f"mlp.{n}.weight"
        return names

    def load_tensors(self, tensors: dict[str, torch.Tensor]) -> None:
        """Copy checkpoint tensors (by checkpoint name) into the parameters.  Sizes that only the file knows (the
        low-rank widths, the rows of a distance table) shape their parameters; the q / k / v convolutions of a
        recurrent layer are stacked into its one convolution."""
        names = self.checkpoint_names()
        params = dict(self.named_parameters())
        seen = set()
        with torch.no_grad():
            for i, layer in enumerate(self.layers):
                if self.config.layers[i].mixer.kind == "channel_delta":
                    parts = [tensors[f"l{i}.mix.{n}.conv"] for n in ("q", "k", "v")]
                    w = torch.cat(parts, dim=0)
                    if w.shape != layer.mix.conv.weight.shape:
                        raise ValueError(f"l{i}: convolution weights {tuple(w.shape)} != {tuple(layer.mix.conv.weight.shape)}")
                    layer.mix.conv.weight.copy_(w)
                    seen.update(f"l{i}.mix.{n}.conv" for n in ("q", "k", "v"))
            for ck, pn in names.items():
                if ck not in tensors:
                    raise KeyError(f"checkpoint lacks {ck}")
                t, p = tensors[ck], params[pn]
                if t.shape != p.shape:
                    free = pn.endswith((".a1.weight", ".a2.weight", ".g1.weight", ".g2.weight", "mix.rel"))
                    if not free or t.dim() != p.dim():
                        raise ValueError(f"{ck}: checkpoint shape {tuple(t.shape)} != parameter {tuple(p.shape)}")
                    p.data = torch.empty(t.shape, dtype=p.dtype, device=p.device)
                p.copy_(t)
                seen.add(ck)
        extra = sorted(set(tensors) - seen)
        if extra:
            raise KeyError(f"checkpoint has tensors the model does not know, e.g. {extra[:3]}")
        self.finalize()

    def finalize(self) -> "BuvalixForCausalLM":
        """After the weights are in place: fuse the input projections, expand the distance tables."""
        for layer in self.layers:
            m = layer.mix
            if isinstance(m, BuvalixChannelDelta):
                if m.a2.weight.shape[1] != m.a1.weight.shape[0] or m.g2.weight.shape[1] != m.g1.weight.shape[0]:
                    raise ValueError("low-rank projections do not chain")
            m.finalize()
            if layer.mlp is not None:
                layer.mlp.finalize()
        return self

    # ---- caches -------------------------------------------------------------------------------------------
    def cache_specs(self) -> list:
        """One cache per run, in execution order."""
        return [self.layers[i].mix.cache_spec() for i, _ in self._runs]

    def bind_caches(self, caches: list) -> None:
        assert len(caches) == len(self._runs)
        self._caches = caches

    # ---- forward ------------------------------------------------------------------------------------------
    def forward(self, input_ids, positions, logits_rows=None, streams: list | None = None):
        """Returns float32 logits [T or len(logits_rows), vocab].  streams: a list that receives the residual stream
        after every run (needs fused=False)."""
        if self._caches is None:
            raise RuntimeError("caches are not bound: the model runs through the engine's cache and state manager")
        if streams is not None and self.fused:
            raise ValueError("collecting the streams needs fused=False")
        boundary, dt = self._L.residual_boundary, self.dtype
        x0 = self.embed(input_ids).float()
        x = x0.clone() if self.config.loop_times > 1 else x0
        ctx = get_context()
        pend_h, pend_norm = None, None            # sublayer output whose post-norm has not been applied yet
        for run, (i, reopen) in enumerate(self._runs):
            layer = self.layers[i]
            ctx.layer_idx = run
            extra = x0 if reopen else None
            if self.fused:
                y = boundary(x, pend_h, pend_norm, extra, layer.norm1, dt)
            else:
                if pend_h is not None:
                    boundary(x, pend_h, pend_norm)
                    if streams is not None:
                        streams.append(x.clone())
                if extra is not None:
                    boundary(x, extra=extra)
                y = boundary(x, pre=layer.norm1, out_dtype=dt)
            h = layer.mix(y, positions, self._caches[run])
            pend_h, pend_norm = h, layer.norm1b
            if layer.mlp is not None:
                if self.fused:
                    y = boundary(x, pend_h, pend_norm, None, layer.norm2, dt)
                else:
                    boundary(x, pend_h, pend_norm)
                    y = boundary(x, pre=layer.norm2, out_dtype=dt)
                pend_h, pend_norm = layer.mlp(y), layer.norm2b
        if logits_rows is not None and self.fused:
            x, pend_h = x[logits_rows], (pend_h[logits_rows] if pend_h is not None else None)
        if self.fused:
            y = boundary(x, pend_h, pend_norm, None, self.final_norm, dt)
        else:
            if pend_h is not None:
                boundary(x, pend_h, pend_norm)
                if streams is not None:
                    streams.append(x.clone())
            if logits_rows is not None:
                x = x[logits_rows]
            y = boundary(x, pre=self.final_norm, out_dtype=dt)
        return self.head(y).float()
