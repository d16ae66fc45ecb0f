"""Helpers of the Benarax tests: small configurations, random checkpoints in the design's tensor names, and engines on
the CPU stand-ins or on the HIP layers.  The replay driver and the error measure are the Buvalix tests'."""
import math

import torch

import nanovllm_amd  # noqa: F401
from buvalix_util import paged_context, rel_err, replay  # noqa: F401
from nanovllm_amd.engine.llm_engine import LLMEngine
from nanovllm_amd.model.benarax import BenaraxConfig, BenaraxForCausalLM
from oracle import ref_benarax, ref_benarax_modules


def moe(experts=5, top=2, ff=24, limit=1.5):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": limit}}


def delta_layer(heads=3, dim=12, mlp="default"):
    return {"type": "general_delta", "mixer": {"heads": heads, "dim": dim}, "mlp": moe() if mlp == "default" else mlp}


def latent_layer(kind="latent_attention", heads=3, dim=10, rot_dim=6, vdim=14, q_rank=20, kv_rank=18, base=300.0,
                 scaling="default", mlp="default"):
    rot = {"dims": rot_dim, "base": base}
    if scaling == "default":
        scaling = {"factor": 3.0, "fast": 8.0, "slow": 1.0, "original": 24} if kind == "latent_attention" else None
    if scaling:
        rot["scaling"] = scaling
    return {"type": kind, "mlp": moe() if mlp == "default" else mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "rot": rot, "scale": 1.1 / math.sqrt(dim + rot_dim)}}


def config(layers, loop=None, vocab=83, width=36, eps=1e-5, groups=3, taps=3, side=5, mult=0.8, embed_scale=3.0,
           logit_scale=0.5):
    cfg = {"architecture": "Benarax", "layers": layers, "loop": loop or {"start": 0, "stop": 0, "times": 1},
           "norm": {"eps": eps, "groups": groups}, "vocab": vocab, "width": width, "residual_mult": mult,
           "embedding": {"scale": embed_scale}, "logit_scale": logit_scale}
    if taps:
        cfg["canon"] = {"taps": taps}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


def random_checkpoint(cfg: dict, seed: int, rank: int = 4, dtype=torch.bfloat16) -> dict:
    """Tensors by checkpoint name, stored in bfloat16 like a file (so every dtype sees the same values)."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    rn = lambda *s, std=1.0, mean=0.0: (torch.randn(*s, generator=g) * std + mean).to(dtype)
    lin = lambda o, i, gain=1.0: rn(o, i, std=gain / math.sqrt(i))
    t = {"embed": rn(V, W, std=0.5), "head": lin(V, W), "final.norm": rn(W, std=0.1, mean=1.0)}
    side = (cfg.get("token_side") or {}).get("dim", 0)
    if side:
        t["side.embed"] = rn(V, side * len(cfg["layers"]))
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = rn(W, std=0.1, mean=1.0)
        if cfg.get("canon"):
            t[p + "canon1"] = rn(W, cfg["canon"]["taps"], std=0.4)
        if side:
            t[p + "side.gate"], t[p + "side.proj"] = lin(side, W, 2.0), lin(W, side)
            t[p + "side.norm"] = rn(W, std=0.1, mean=0.6)
        H, D = m["heads"], m["dim"]
        if L["type"] == "general_delta":
            for n in ("r", "k", "v", "a", "g"):
                t[p + "mix." + n] = lin(H * D, W, 1.5)
            t[p + "mix.w1"], t[p + "mix.w2"] = lin(rank, W, 2.0), lin(H * D, rank, 3.0)
            t[p + "mix.w0"], t[p + "mix.a.b"] = rn(H * D, std=1.5), rn(H * D, std=1.0)
            t[p + "mix.norm"] = rn(H * D, std=0.1, mean=1.0)
            t[p + "mix.o"] = lin(W, H * D)
        else:
            R, Dv, qr, kr = m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            t[p + "mix.dq"], t[p + "mix.dq.norm"] = lin(qr, W), rn(qr, std=0.1, mean=1.0)
            t[p + "mix.uq"] = lin(H * (D + R), qr)
            t[p + "mix.dkv"], t[p + "mix.dkv.norm"] = lin(kr + R, W, 1.5), rn(kr, std=0.1, mean=1.0)
            t[p + "mix.uk"], t[p + "mix.uv"] = lin(H * D, kr), lin(H * Dv, kr)
            t[p + "mix.o"] = lin(W, H * Dv)
        if L["mlp"] is not None:
            E, ff = L["mlp"]["router"]["experts"], L["mlp"]["expert"]["ff"]
            t[p + "mlp.router"] = lin(E, W, 3.0)
            for e in range(E):
                q = f"{p}mlp.e{e}."
                t[q + "gate"], t[q + "up"], t[q + "down"] = lin(ff, W, 2.0), lin(ff, W, 2.0), lin(W, ff)
    return t


def make_engine(cfg: dict, tensors: dict, device: str, dtype=torch.float32, block_size=4, num_blocks=64, max_seqs=4, **kw):
    layers = ref_benarax_modules if device == "cpu" else None
    model = BenaraxForCausalLM(BenaraxConfig.from_dict(cfg), layers=layers, dtype=dtype, device=device)
    model.load_tensors(tensors)
    return LLMEngine(model, model.config, block_size=block_size, num_kvcache_blocks=num_blocks, device=device,
                     max_num_seqs=max_seqs, dtype=dtype, **kw)


def oracle_logits(cfg: dict, tensors: dict, tokens, dtype=torch.float32):
    return ref_benarax.forward(cfg, tensors, tokens, dtype)[0]


def layer_namespace(device: str):
    """The layer classes the model would use on this device: eager stand-ins on the CPU, HIP-backed on the GPU."""
    if device == "cpu":
        return ref_benarax_modules
    from nanovllm_amd.model.benarax import _default_layers
    return _default_layers()


def steady_prefix(cfg: dict, tensors: dict, tokens, least=0.05) -> int:
    """Number of leading positions before the first close call of a router (the last chosen expert leads the next one
    by less than `least` of the logits' spread): up to there a bfloat16 run differs from float32 by rounding alone."""
    margins = []
    ref_benarax.forward(cfg, tensors, tokens, torch.float32, margins)
    if not margins:
        return len(tokens)
    close = torch.stack(margins).min(0).values < least
    return int(close.nonzero()[0]) if close.any() else len(tokens)
