#!/usr/bin/env python3
"""Benarax beside Buvalix (the closest existing model: fp32 stream, recurrent and attention mixers) at equal sizes,
random weights: every kernel of the design next to the like kernel, with its HBM or MFMA rate, and prefill / decode
throughput of whole models through the engine.  `python bench.py --benarax` prints the record as one JSON line."""
import argparse
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import nanovllm_amd as nv  # noqa: E402
from nanovllm_amd import ops  # noqa: E402
from nanovllm_amd.engine.llm_engine import LLMEngine  # noqa: E402
from nanovllm_amd.engine.sequence import SamplingParams  # noqa: E402
from nanovllm_amd.layers import delta_rule, general_delta, latent_attention, moe, stream  # noqa: E402
from nanovllm_amd.model.benarax import BenaraxConfig, BenaraxForCausalLM  # noqa: E402
from tools.buvalix_bench import buvalix_config, paged, random_buvalix, rate, timed  # noqa: E402


def kernel_records(dev):
    out = {}
    bf = torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s, dtype=bf: torch.randn(*s, generator=g, device=dev).to(dtype)
    W, bs = 2048, 256
    for name, T in (("prefill_8192_tokens", 8192), ("decode_256_tokens", 256)):
        rec = {}
        x, a, parts, y = rn(T, W, dtype=torch.float32), rn(T, W), rn(T, 4, W, dtype=torch.float32), rn(T, W)
        w = rn(W, dtype=torch.float32)
        t = timed(lambda: ops.stream_boundary(x, add=a, add_parts=parts, mult=0.5, copy_dtype=bf))
        rec["stream_boundary (mixer + 4 expert parts -> stream, bf16 copy)"] = rate(t, nbytes=T * W * (8 + 2 + 16 + 2))
        t = timed(lambda: ops.stream_boundary(x, normed=y, normed_weight=w, mult=0.5, norm=w, groups=4, eps=1e-5,
                                              out_dtype=bf, want_f32=True))
        rec["stream_boundary (normed side input -> stream -> grouped norm, fp32 + bf16)"] = rate(t, nbytes=T * W * (8 + 2 + 4 + 2))
        h = rn(T, W)
        b = rn(W, dtype=torch.float32)
        t = timed(lambda: ops.add_layernorm(x, h, (w, b), None, (w, b), bf, 1e-5))
        rec["like: add_layernorm"] = rate(t, nbytes=T * W * (4 + 4 + 2 + 2))
        rec["rms_norm_rows (1536 wide)"] = rate(timed(lambda: ops.rms_norm_rows(a[:, :1536], w[:1536], 1e-5)), nbytes=T * 1536 * 4)
        out[name] = rec

    H, D, taps = 16, 128, 4
    for name, n_qs in (("prefill_4x2048", [2048] * 4), ("decode_256_seqs", [1] * 256)):
        n_ks = [n + 100 for n in n_qs]
        ctx, pos, _ = paged(n_qs, n_ks, bs, dev)
        T, B = sum(n_qs), len(n_qs)
        nv.set_context(ctx)
        rec = {}
        x32 = rn(T, W, dtype=torch.float32)
        conv = stream.CausalConvAdd(W, taps, device=dev)
        cs = torch.zeros(B, taps - 1, W, device=dev)
        rec["causal_conv_add (fp32 in, bf16 out)"] = rate(timed(lambda: conv(x32, cs, bf)), nbytes=T * W * 6)
        xb = rn(T, 3 * H * D)
        conv2 = delta_rule.ShortConvSilu(3 * H * D, taps, device=dev)
        cs2 = torch.zeros(B, taps - 1, 3 * H * D, device=dev, dtype=bf)
        rec["like: causal_conv_silu"] = rate(timed(lambda: conv2(xb, cs2)), nbytes=T * 3 * H * D * 4)
        rule = general_delta.GeneralDeltaRule(H, D, 1e-5, device=dev)
        st = torch.zeros(B, H, D, D, device=dev)
        r, k, v = rn(T, H, D), rn(T, H, D), rn(T, H, D)
        wr, ar, gr = rn(T, H * D), rn(T, H * D), rn(T, H * D)
        t = timed(lambda: rule(r, k, v, wr, ar, gr, st), iters=5)
        io = T * 7 * H * D * 2 + 2 * B * H * D * D * 4
        rec["general_delta_rule"] = dict(rate(t, nbytes=io), tokens_per_s=round(T / t))
        old = delta_rule.GatedDeltaRule(H, H, D, D, 1e-5, device=dev)
        a_raw, b_raw = rn(T, H * D), rn(T, H)
        t = timed(lambda: old(r, k, v, a_raw, b_raw, gr, st), iters=5)
        rec["like: gated_delta_rule"] = dict(rate(t, nbytes=T * (6 * H * D + H) * 2 + 2 * B * H * D * D * 4), tokens_per_s=round(T / t))
        nv.set_context(None)
        out["recurrent " + name] = rec

    Hq = 16
    for rank, R, Dn in ((128, 32, 96), (192, 64, 128)):
        scale = (Dn + R) ** -0.5
        cases = {"prefill_4x2048": ([2048] * 4, [2048] * 4), "chunk_512_over_8192": ([512], [8192]),
                 "decode_256_seqs_ctx_513_768": ([1] * 256, torch.randint(513, 769, (256,), generator=torch.Generator().manual_seed(1)).tolist()),
                 "decode_8_seqs_ctx_8192": ([1] * 8, [8192] * 8)}
        for name, (n_qs, n_ks) in cases.items():
            ctx, pos, nb = paged(n_qs, n_ks, bs, dev)
            T = sum(n_qs)
            nv.set_context(ctx)
            lat = latent_attention.LatentAttention(Hq, rank, R, scale, 1e-5, 1e4, {"factor": 8.0, "fast": 16.0, "slow": 2.0, "original": 2048}, device=dev)
            q, q_lat, ckv = rn(T, Hq, Dn + R), rn(T, Hq, rank), rn(T, rank + R)
            kc = rn(nb, bs, 1, rank + R)
            vc = kc[..., :rank]                      # the values are the front of the key rows
            rec = {}
            t = timed(lambda: ops.latent_prep_store(q, q_lat, ckv, lat.latent_norm, lat.freq, lat.mag, True, pos,
                                                    ctx.slot_mapping, kc, vc, R, 1e-5))
            rec["latent_prep_store"] = rate(t, nbytes=T * (Hq * (rank + R) * 4 + (rank + R) * 2 * 2))
            qf = rn(T, Hq, rank + R)
            pairs = sum(nq * (nk - nq) + nq * (nq + 1) // 2 for nq, nk in zip(n_qs, n_ks))
            flops = 2 * (rank + R + rank) * Hq * pairs
            kv_bytes = sum(n_ks) * (rank + R) * 2 + T * Hq * (2 * rank + R) * 2
            singles = int(max(n_qs) == 1)
            t = timed(lambda: ops.attn_scoremod_paged(qf, kc, vc, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.block_tables, scale,
                                                      0.0, None, None, max(n_qs), max(n_ks), singles), iters=5)
            rec["latent attention (1 kv head, key %d, value %d)" % (rank + R, rank)] = rate(t, nbytes=kv_bytes if singles else None,
                                                                                         flops=None if singles else flops)
            G, Dh = 8, 128
            q2, kc2, vc2 = rn(T, Hq, Dh), rn(nb, bs, G, Dh), rn(nb, bs, G, Dh)
            pf = 4 * Dh * Hq * pairs
            kvb = sum(n_ks) * G * Dh * 4 + T * Hq * Dh * 4
            t = timed(lambda: ops.attn_scoremod_paged(q2, kc2, vc2, ctx.cu_seqlens_q, ctx.cu_seqlens_k, ctx.block_tables,
                                                      Dh ** -0.5, 30.0, None, None, max(n_qs), max(n_ks), singles), iters=5)
            rec["like: attn_scoremod (16/8 heads x 128)"] = rate(t, nbytes=kvb if singles else None, flops=None if singles else pf)
            nv.set_context(None)
            out["attention rank %d, %s" % (rank, name)] = rec

    E, top, ff = 32, 4, 1024
    gu, dn = rn(E, 2 * ff, W) * 0.02, rn(E, W, ff) * 0.02
    dense_gu, dense_dn = rn(2 * top * ff, W) * 0.02, rn(W, top * ff) * 0.02
    ex = moe.MoEExperts(top, 7.0)
    for name, T in (("prefill_8192_tokens", 8192), ("decode_256_tokens", 256), ("decode_16_tokens", 16)):
        h, lg = rn(T, W), rn(T, E, dtype=torch.float32)
        flops = 2 * T * top * 3 * ff * W
        used = min(E, T * top)
        wbytes = used * 3 * ff * W * 2
        t = timed(lambda: ex(h, lg, gu, dn), iters=5)
        rec = {"routed experts (32 experts, top 4, ff 1024)": rate(t, nbytes=wbytes + T * W * (2 + 4 * top), flops=flops)}

        def dense():
            y = ops.gelu_tanh_and_mul(torch.nn.functional.linear(h, dense_gu))
            return torch.nn.functional.linear(y, dense_dn)
        t = timed(dense, iters=5)
        rec["like: dense GLU of the same FLOPs (vendor matrix products, ff 4096)"] = rate(t, nbytes=3 * top * ff * W * 2 + T * W * 4, flops=flops)
        out["feed-forward " + name] = rec
    return out


def benarax_config(width, n_groups, vocab, experts=32, top=4, ff=1024):
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff, "limit": 7.0}}
    lat = {"heads": 16, "dim": 96, "rot_dim": 32, "vdim": 96, "q_rank": 768, "kv_rank": 128, "scale": 128 ** -0.5}
    group = [
        {"type": "general_delta", "mlp": mlp, "mixer": {"heads": 16, "dim": 128}},
        {"type": "latent_attention", "mlp": mlp,
         "mixer": dict(lat, rot={"dims": 32, "base": 1e4, "scaling": {"factor": 8.0, "fast": 16.0, "slow": 2.0, "original": 2048}})},
        {"type": "general_delta", "mlp": mlp, "mixer": {"heads": 16, "dim": 128}},
        {"type": "latent_attention_2", "mlp": mlp, "mixer": dict(lat, rot={"dims": 32, "base": 1e6})},
    ]
    return {"architecture": "Benarax", "layers": group * n_groups, "norm": {"eps": 1e-5, "groups": 4}, "vocab": vocab,
            "width": width, "loop": {"start": 0, "stop": 0, "times": 1}, "residual_mult": 0.5, "embedding": {"scale": 1.0},
            "logit_scale": 1.0, "canon": {"taps": 4}, "token_side": {"dim": 64}}


def random_benarax(cfg_dict, dev, dtype, rank=64):
    cfg = BenaraxConfig.from_dict(cfg_dict)
    model = BenaraxForCausalLM(cfg, dtype=dtype, device=dev)
    g = torch.Generator(device=dev).manual_seed(0)
    with torch.no_grad():
        for layer in model.layers:
            m = layer.mix
            if hasattr(m, "w1"):
                W = m.w1.weight.shape[1]
                m.w1.weight.data = torch.empty(rank, W, dtype=dtype, device=dev)
                m.w2.weight.data = torch.empty(m.w2.weight.shape[0], rank, dtype=dtype, device=dev)
        for name, p in model.named_parameters():
            if p.dim() >= 2:
                p.copy_((torch.randn(p.shape, generator=g, device=dev) * (0.5 if "canon" in name else 0.02)).to(p.dtype))
            elif "norm" in name:
                p.fill_(1.0)
            else:
                p.copy_((torch.randn(p.shape, generator=g, device=dev) * 0.1).to(p.dtype))
    model.finalize()
    return model, cfg


def model_records(dev, width=2048, n_groups=2, vocab=32000, batch=32, prompt_len=1024, out_len=64):
    out = {"shape": dict(width=width, layers=4 * n_groups, vocab=vocab, batch=batch, prompt_len=prompt_len, out_len=out_len,
                         block_size=256, benarax="16 heads; 32 experts, top 4, ff 1024 (active ff 4096); latent 128 + 32",
                         buvalix="16/8 heads x 128; dense ff 4096")}
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

    model, cfg = random_benarax(benarax_config(width, n_groups, vocab), dev, torch.bfloat16)
    eng = LLMEngine(model, cfg, block_size=256, num_kvcache_blocks=blocks, max_num_batched_tokens=8192, device=dev,
                    eos=-1, max_num_seqs=batch, long_prefill_token_threshold=0)
    out["benarax"] = measure(eng)
    del eng, model
    torch.cuda.empty_cache()
    model, cfg = random_buvalix(buvalix_config(width, 4096, n_groups, vocab), dev, torch.bfloat16)
    eng = LLMEngine(model, cfg, block_size=256, num_kvcache_blocks=blocks, max_num_batched_tokens=8192, device=dev,
                    eos=-1, max_num_seqs=batch, long_prefill_token_threshold=0)
    out["like: buvalix (same width, layers, head count; dense ff 4096)"] = measure(eng)
    return out


def run(device="cuda:0", kernels=True, models=True):
    rec = {"metric": "benarax_vs_like_model", "rooflines": {"hbm_TB_s": 8.0, "mfma_bf16_PFLOP_s": 2.5},
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
