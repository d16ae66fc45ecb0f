#!/usr/bin/env python3
"""Buvalix beside the Qwen3 path at equal sizes (random weights): every kernel of the second library next to the
like kernel of the first, with its HBM or MFMA rate, and prefill / decode throughput of whole models through the
engine.  `python bench.py --buvalix` prints the record as one JSON line."""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import nanovllm_amd as nv  # noqa: E402
from nanovllm_amd import ops  # noqa: E402
from nanovllm_amd.engine.llm_engine import LLMEngine  # noqa: E402
from nanovllm_amd.engine.sequence import SamplingParams  # noqa: E402
from nanovllm_amd.layers import attention, delta_rule  # noqa: E402
from nanovllm_amd.model.buvalix import BuvalixConfig, BuvalixForCausalLM  # noqa: E402
from nanovllm_amd.model.qwen3 import ModelConfig, Qwen3ForCausalLM  # noqa: E402

HBM_TBS, MFMA_PFS = 8.0, 2.5          # rooflines the rates are priced against


def timed(fn, iters=20, warm=3):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e-3 / iters


def rate(seconds, nbytes=None, flops=None):
    r = {"us": round(seconds * 1e6, 1)}
    if nbytes is not None:
        r["TB_s"] = round(nbytes / seconds / 1e12, 3)
        r["of_hbm"] = round(nbytes / seconds / 1e12 / HBM_TBS, 3)
    if flops is not None:
        r["TFLOP_s"] = round(flops / seconds / 1e12, 1)
        r["of_mfma"] = round(flops / seconds / 1e15 / MFMA_PFS, 3)
    return r


def paged(n_qs, n_ks, bs, dev, seed=0):
    g = torch.Generator().manual_seed(seed)
    need = [-(-n // bs) for n in n_ks]
    nb = sum(need) + 1
    perm = torch.randperm(nb, generator=g).tolist()
    width = max(need)
    tables, nxt, slots, pos = [], 0, [], []
    for nq, nk, n in zip(n_qs, n_ks, need):
        row = perm[nxt:nxt + n]
        nxt += n
        tables.append(row + [-1] * (width - n))
        p = torch.arange(nk - nq, nk)
        pos.append(p)
        slots.append(torch.tensor(row)[p // bs] * bs + p % bs)
    cu = lambda xs: torch.tensor([0] + torch.tensor(xs).cumsum(0).tolist(), dtype=torch.int32, device=dev)
    singles = sum(1 for n in n_qs if n == 1)
    ctx = nv.CacheContext(slot_mapping=torch.cat(slots).to(torch.int32).to(dev), cu_seqlens_q=cu(n_qs),
                          cu_seqlens_k=cu(n_ks), max_seqlen_q=max(n_qs), max_seqlen_k=max(n_ks),
                          block_tables=torch.tensor(tables, dtype=torch.int32, device=dev), block_size=bs,
                          num_decode_seqs=singles, num_leading_decode=singles if singles == len(n_qs) else None,
                          max_seqlen_k_decode=max(n_ks), max_seqlen_q_rest=max(n_qs), max_seqlen_k_rest=max(n_ks),
                          state_slots=torch.arange(len(n_qs), dtype=torch.int32, device=dev))
    return ctx, torch.cat(pos).to(dev), nb


def kernel_records(dev):
    out = {}
    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s, dtype=bf: torch.randn(*s, generator=g, device=dev).to(dtype)
    W, I = 2048, 8192
    for name, T in (("prefill_8192_tokens", 8192), ("decode_256_tokens", 256)):
        rec = {}
        resid, h = rn(T, W, dtype=torch.float32), rn(T, W)
        w, b = rn(W, dtype=torch.float32), rn(W, dtype=torch.float32)
        t = timed(lambda: ops.add_layernorm(resid, h, (w, b), None, (w, b), bf, 1e-5))
        rec["add_layernorm"] = rate(t, nbytes=T * W * (4 + 4 + 2 + 2))
        x, res, wr = rn(T, W), rn(T, W), rn(W)
        t = timed(lambda: ops.add_rmsnorm(x, res, wr, 1e-6))
        rec["like: add_rmsnorm"] = rate(t, nbytes=T * W * 8)
        gu = rn(T, 2 * I)
        rec["gelu_tanh_and_mul"] = rate(timed(lambda: ops.gelu_tanh_and_mul(gu)), nbytes=T * I * 6)
        rec["like: silu_and_mul"] = rate(timed(lambda: ops.silu_and_mul(gu)), nbytes=T * I * 6)
        out[name] = rec

    H, G, D, bs = 16, 8, 128, 256
    scale = D ** -0.5
    cases = {"prefill_4x2048": ([2048] * 4, [2048] * 4), "chunk_512_over_8192": ([512], [8192]),
             "decode_256_seqs_ctx_513_768": ([1] * 256, torch.randint(513, 769, (256,), generator=torch.Generator().manual_seed(1)).tolist()),
             "decode_8_seqs_ctx_8192": ([1] * 8, [8192] * 8)}
    for name, (n_qs, n_ks) in cases.items():
        ctx, pos, nb = paged(n_qs, n_ks, bs, dev)
        T = sum(n_qs)
        q, k, v = rn(T, H, D), rn(T, G, D), rn(T, G, D)
        kc, vc = rn(nb, bs, G, D), rn(nb, bs, G, D)
        attn = attention.ScoreModAttention(H, G, D, D, scale, softcap=30.0, rot_dims=64, rot_base=1e4, use_sink=True, device=dev)
        nv.set_context(ctx)
        pairs = sum(nq * (nk - nq) + nq * (nq + 1) // 2 for nq, nk in zip(n_qs, n_ks))
        flops = 4 * D * H * pairs
        kv_bytes = sum(n_ks) * G * D * 2 * 2 + T * H * D * 2 * 2
        rec = {}
        t = timed(lambda: ops.qk_prep_store(pos, q, k, v, ctx.slot_mapping, kc, vc, attn.inv_freq, 64))
        rec["qk_prep_store"] = rate(t, nbytes=T * (2 * H + 4 * G) * D * 2)
        cos_sin = torch.randn(max(n_ks) + 1, D, device=dev)
        qw = torch.ones(D, device=dev, dtype=bf)
        t = timed(lambda: ops.qknorm_rope_store(pos, q, k, v, qw, qw, cos_sin, 1e-6, ctx.slot_mapping, kc, vc, want_k=False))
        rec["like: qknorm_rope_store"] = rate(t, nbytes=T * (2 * H + 4 * G) * D * 2)
        singles = int(max(n_qs) == 1)
        t = timed(lambda: ops.attn_scoremod_paged(q, kc, vc, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.block_tables, scale,
                                                  30.0, attn.sink, None, max(n_qs), max(n_ks), singles))
        if singles:
            rec["attn_scoremod (single rows)"] = rate(t, nbytes=kv_bytes)
            t = timed(lambda: ops.attn_decode_paged(q, kc, vc, ctx.cu_seqlens_k, ctx.block_tables, max(n_ks), scale))
            rec["like: attn_decode_paged"] = rate(t, nbytes=kv_bytes)
        else:
            rec["attn_scoremod (MFMA tiles)"] = rate(t, flops=flops)
            t = timed(lambda: ops.attn_prefill_varlen(q, kc, vc, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.block_tables,
                                                      max(n_qs), max(n_ks), scale))
            rec["like: attn_prefill_varlen"] = rate(t, flops=flops)
        nv.set_context(None)
        out["attention " + name] = rec

    Hd, Gd, Dd, Dvd, taps = 16, 16, 128, 128, 4
    for name, n_qs in (("prefill_4x2048", [2048] * 4), ("decode_256_seqs", [1] * 256)):
        n_ks = [n + 100 for n in n_qs]
        ctx, pos, _ = paged(n_qs, n_ks, bs, dev)
        T, B = sum(n_qs), len(n_qs)
        C = 2 * Gd * Dd + Hd * Dvd
        x = rn(T, C)
        conv = delta_rule.ShortConvSilu(C, taps, device=dev)
        rule = delta_rule.GatedDeltaRule(Hd, Gd, Dd, Dvd, 1e-5, device=dev)
        cs = torch.zeros(B, taps - 1, C, device=dev, dtype=bf)
        st = torch.zeros(B, Hd, Dd, Dvd, device=dev)
        a_raw, b_raw, gate = rn(T, Hd * Dd), rn(T, Hd), rn(T, Hd * Dvd)
        nv.set_context(ctx)
        rec = {}
        rec["causal_conv_silu"] = rate(timed(lambda: conv(x, cs)), nbytes=T * C * 4)
        y = conv(x, cs)
        qk = Gd * Dd
        qq, kk, vv = (y[:, :qk].unflatten(1, (Gd, Dd)), y[:, qk:2 * qk].unflatten(1, (Gd, Dd)),
                      y[:, 2 * qk:].unflatten(1, (Hd, Dvd)))
        t = timed(lambda: rule(qq, kk, vv, a_raw, b_raw, gate, st), iters=5)
        io = T * (C + Hd * Dd + Hd + 2 * Hd * Dvd) * 2 + 2 * B * Hd * Dd * Dvd * 4
        rec["gated_delta_rule"] = dict(rate(t, nbytes=io), tokens_per_s=round(T / t))
        nv.set_context(None)
        out["recurrent " + name] = rec
    return out


def buvalix_config(width, ff, n_groups, vocab):
    att = {"heads": 16, "kv_heads": 8, "dim": 128, "vdim": 128, "scale": 128 ** -0.5, "softcap": 30.0}
    group = [
        {"type": "channel_delta", "mlp": {"kind": "dense", "ff": ff},
         "mixer": {"heads": 16, "kv_heads": 16, "dim": 128, "vdim": 128, "conv": 4}},
        {"type": "attention", "mlp": {"kind": "dense", "ff": ff}, "mixer": dict(att, rot={"dims": 64, "base": 1e4})},
        {"type": "channel_delta", "mlp": {"kind": "dense", "ff": ff},
         "mixer": {"heads": 16, "kv_heads": 16, "dim": 128, "vdim": 128, "conv": 4}},
        {"type": "attention_2", "mlp": {"kind": "dense", "ff": ff},
         "mixer": dict(att, q_temp={"coef": 0.1, "every": 1024}, bias_max=2048)},
    ]
    return {"architecture": "Buvalix", "layers": group * n_groups, "norm": {"eps": 1e-5}, "vocab": vocab, "width": width,
            "loop": {"start": 0, "stop": 0, "times": 1}}


def random_buvalix(cfg_dict, dev, dtype, rank=64, rel_rows=24):
    cfg = BuvalixConfig.from_dict(cfg_dict)
    model = BuvalixForCausalLM(cfg, dtype=dtype, device=dev)
    g = torch.Generator().manual_seed(0)
    W = cfg.hidden_size
    tensors = {}
    for ck, pn in model.checkpoint_names().items():
        p = dict(model.named_parameters())[pn]
        shape = list(p.shape)
        if pn.endswith(("a1.weight", "g1.weight")):
            shape = [rank, W]
        elif pn.endswith(("a2.weight", "g2.weight")):
            shape = [shape[0], rank]
        elif pn.endswith("mix.rel"):
            shape = [rel_rows, shape[1]]
        if ck.endswith((".norm1", ".norm2", ".norm1b", ".norm2b", "final.norm", "mix.norm")):
            t = torch.ones(shape)
        elif len(shape) == 2 and not pn.endswith("mix.rel"):
            t = torch.randn(shape, generator=g) * 0.02
        elif pn.endswith("A_log"):
            t = torch.full(shape, -1.0)
        else:
            t = torch.randn(shape, generator=g) * 0.1
        tensors[ck] = t.to(torch.bfloat16)
    for i, L in enumerate(cfg.layers):
        if L.mixer.kind == "channel_delta":
            m = L.mixer
            for n, o in (("q", m.kv_heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.heads * m.vdim)):
                tensors[f"l{i}.mix.{n}.conv"] = (torch.randn(o, m.conv, generator=g) * 0.5).to(torch.bfloat16)
    model.load_tensors(tensors)
    return model, cfg


def model_records(dev, width=2048, ff=6144, n_groups=2, vocab=32000, batch=32, prompt_len=1024, out_len=64):
    out = {"shape": dict(width=width, ff=ff, layers=4 * n_groups, heads="16/8 x 128", vocab=vocab, batch=batch,
                         prompt_len=prompt_len, out_len=out_len, block_size=256)}
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, vocab, (prompt_len,), generator=g).tolist() for _ in range(batch)]
    warm = [torch.randint(0, vocab, (prompt_len,), generator=g).tolist() for _ in range(2)]
    blocks = batch * (-(-(prompt_len + out_len) // 256)) + 8

    def measure(engine):
        engine.generate(warm, SamplingParams(0.0, 4))
        torch.cuda.synchronize()
        _, m = engine.generate(prompts, SamplingParams(0.0, out_len))
        s = m.summary()
        prefill = sum(t for t, _, only in m.step_times if not only)
        return {"prefill_tok_per_s": round(batch * prompt_len / prefill), "decode_tok_per_s": round(s["decode_only_tok_per_s"]),
                "mean_tpot_ms": round(s["mean_tpot_ms"], 3), "output_tok_per_s": round(s["output_tok_per_s"])}

    model, cfg = random_buvalix(buvalix_config(width, ff, n_groups, vocab), dev, torch.bfloat16)
    eng = LLMEngine(model, cfg, block_size=256, num_kvcache_blocks=blocks, max_num_batched_tokens=8192, device=dev,
                    eos=-1, max_num_seqs=batch, long_prefill_token_threshold=0)
    out["buvalix"] = measure(eng)
    del eng, model
    torch.cuda.empty_cache()
    qcfg = ModelConfig(vocab_size=vocab, hidden_size=width, intermediate_size=ff, num_hidden_layers=4 * n_groups,
                       num_attention_heads=16, num_key_value_heads=8, head_dim=128, tie_word_embeddings=False)
    torch.manual_seed(0)
    with torch.device(dev):
        qm = Qwen3ForCausalLM(qcfg)
    for name, p in qm.named_parameters():
        torch.nn.init.ones_(p) if "norm" in name else torch.nn.init.normal_(p, 0.0, 0.02)
    qm = qm.to(torch.bfloat16).fuse_weights()
    eng = LLMEngine(qm, qcfg, block_size=256, num_kvcache_blocks=blocks, max_num_batched_tokens=8192, device=dev,
                    eos=-1, long_prefill_token_threshold=0, use_graphs=False)
    out["like: qwen3 (same width, layers, heads; no graphs)"] = measure(eng)
    return out


def run(device="cuda:0", kernels=True, models=True):
    rec = {"metric": "buvalix_vs_like_model", "rooflines": {"hbm_TB_s": HBM_TBS, "mfma_bf16_PFLOP_s": MFMA_PFS},
           "data": "synthetic", "dtype": "bf16"}
    if kernels:
        rec["kernels"] = kernel_records(device)
    if models:
        rec["models"] = model_records(device)
    return rec


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--no-models", action="store_true")
    a = ap.parse_args()
    print(json.dumps(run(kernels=not a.no_kernels, models=not a.no_models)))
