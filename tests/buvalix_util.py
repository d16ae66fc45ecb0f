"""Helpers of the Buvalix tests: small configurations, random checkpoints in the design's tensor names, engines on
the CPU stand-ins or on the HIP layers, and a replay driver that feeds prompts in given portions."""
import math

import torch

import nanovllm_amd  # noqa: F401
from nanovllm_amd.engine.llm_engine import LLMEngine
from nanovllm_amd.model.buvalix import BuvalixConfig, BuvalixForCausalLM
from oracle import ref_buvalix, ref_mixer_modules


def attention_layer(heads=4, kv_heads=2, dim=24, vdim=40, rot_dims=12, base=500.0, softcap=15.0, ff=48):
    return {"type": "attention", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
                      "softcap": softcap, "rot": {"dims": rot_dims, "base": base}}}


def attention2_layer(heads=6, kv_heads=3, dim=16, vdim=8, coef=0.4, every=7, bias_max=40, softcap=30.0, ff=32):
    return {"type": "attention_2", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 1.3 * dim ** -0.5,
                      "softcap": softcap, "q_temp": {"coef": coef, "every": every}, "bias_max": bias_max}}


def delta_layer(heads=4, kv_heads=2, dim=20, vdim=12, conv=4, ff=None):
    return {"type": "channel_delta", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def config(layers, loop=None, vocab=97, width=56, eps=1e-5):
    return {"architecture": "Buvalix", "layers": layers, "loop": loop or {"start": 0, "stop": 0, "times": 1},
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_checkpoint(cfg: dict, seed: int, rank: int = 5, rel_rows: int = 12, dtype=torch.bfloat16) -> dict:
    """Tensors by checkpoint name, stored in bfloat16 like a file (so every dtype sees the same values)."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    rn = lambda *s, std=1.0, mean=0.0: (torch.randn(*s, generator=g) * std + mean).to(dtype)
    lin = lambda o, i: rn(o, i, std=1.0 / math.sqrt(i))
    t = {"embed": rn(V, W), "head": lin(V, W), "final.norm": rn(W, std=0.1, mean=1.0), "final.norm.b": rn(W, std=0.1)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        norms = ["norm1", "norm1b"] + (["norm2", "norm2b"] if L["mlp"] is not None else [])
        for n in norms:
            t[p + n] = rn(W, std=0.1, mean=1.0)
            t[p + n + ".b"] = rn(W, std=0.1)
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        if L["type"] == "channel_delta":
            for n, o in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                t[p + f"mix.{n}"] = lin(o, W)
                t[p + f"mix.{n}.conv"] = rn(o, m["conv"], std=0.6)
            t[p + "mix.b"] = lin(H, W)
            t[p + "mix.A_log"] = rn(H, std=0.5, mean=-1.0)
            t[p + "mix.norm"] = rn(Dv, std=0.1, mean=1.0)
            t[p + "mix.a1"], t[p + "mix.a2"] = lin(rank, W), lin(H * D, rank)
            t[p + "mix.dt_bias"] = rn(H * D)
            t[p + "mix.g1"], t[p + "mix.g2"] = lin(rank + 1, W), lin(H * Dv, rank + 1)
            t[p + "mix.o"] = lin(W, H * Dv)
        else:
            t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = lin(H * D, W) * 2, lin(G * D, W) * 2, lin(G * Dv, W)
            t[p + "mix.o"] = lin(W, H * Dv)
            if L["type"] == "attention":
                for n, o in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                    t[p + f"mix.{n}.b"] = rn(o, std=0.3)
                t[p + "mix.sink"] = rn(H, std=1.5)
            else:
                t[p + "mix.rel"] = rn(rel_rows, H, std=2.0)
        if L["mlp"] is not None:
            ff = L["mlp"]["ff"]
            t[p + "mlp.gate"], t[p + "mlp.up"], t[p + "mlp.down"] = lin(ff, W), lin(ff, W), lin(W, ff)
    return t


def make_engine(cfg: dict, tensors: dict, device: str, dtype=torch.float32, block_size=4, num_blocks=64, max_seqs=4,
                fused=True, **kw):
    layers = ref_mixer_modules if device == "cpu" else None
    model = BuvalixForCausalLM(BuvalixConfig.from_dict(cfg), layers=layers, dtype=dtype, device=device, fused=fused)
    model.load_tensors(tensors)
    return LLMEngine(model, model.config, block_size=block_size, num_kvcache_blocks=num_blocks, device=device,
                     max_num_seqs=max_seqs, dtype=dtype, **kw)


def oracle_logits(cfg: dict, tensors: dict, tokens, dtype=torch.float32):
    return ref_buvalix.forward(cfg, tensors, tokens, dtype)[0]


def replay(engine, prompts: dict, portions: dict, order=None):
    """Feed each request its prompt in the given portions (a list of sizes per request id), one portion of every
    live request per step (requests join at the step `order[id]`, default 0), asking for every position.
    Returns {id: logits [len, vocab]}."""
    order = order or {}
    at = {i: 0 for i in prompts}
    idx = {i: 0 for i in prompts}
    got = {i: [] for i in prompts}
    step = 0
    while any(at[i] < len(prompts[i]) for i in prompts):
        entries, end = [], []
        for i in prompts:
            if step < order.get(i, 0) or at[i] >= len(prompts[i]):
                continue
            sizes = portions[i]
            n = min(sizes[idx[i]] if idx[i] < len(sizes) else sizes[-1], len(prompts[i]) - at[i])
            entries.append((i, prompts[i][at[i]:at[i] + n], list(range(n))))
            at[i] += n
            idx[i] += 1
            if at[i] == len(prompts[i]):
                end.append(i)
        if entries:
            logits = engine.replay_step(entries, end).cpu()
            o = 0
            for i, toks, _ in entries:
                got[i].append(logits[o:o + len(toks)])
                o += len(toks)
        step += 1
    return {i: torch.cat(v) for i, v in got.items()}


def rel_err(got, want):
    """Per position: rms over the vocabulary of the difference with its mean removed, over the rms of the logits."""
    d = got.float() - want.float()
    d = d - d.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / want.float().pow(2).mean().sqrt()).max().item()


def layer_namespace(device: str):
    """The layer classes the model would use on this device: eager stand-ins on the CPU, HIP-backed on the GPU."""
    if device == "cpu":
        return ref_mixer_modules
    from nanovllm_amd.model.buvalix import _default_layers
    return _default_layers()


def paged_context(n_qs, n_ks, block_size, num_blocks, seed, device, slots=None):
    """A step's CacheContext with shuffled pages: sequence b has n_ks[b] tokens after the step, the last n_qs[b]
    are the step's rows.  Returns (context, positions of the rows)."""
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
    cu = lambda xs: torch.tensor([0] + torch.tensor(xs).cumsum(0).tolist(), dtype=torch.int32, device=device)
    ctx = nanovllm_amd.CacheContext(
        slot_mapping=torch.tensor(slot_map, dtype=torch.int32, device=device), cu_seqlens_q=cu(n_qs),
        cu_seqlens_k=cu(n_ks), max_seqlen_q=max(n_qs), max_seqlen_k=max(n_ks),
        block_tables=torch.tensor(tables, dtype=torch.int32, device=device), block_size=block_size,
        state_slots=None if slots is None else torch.tensor(slots, dtype=torch.int32, device=device))
    return ctx, torch.tensor(pos, dtype=torch.int64, device=device)
