"""Benarax with configurations drawn at random (sizes, head counts, layer order, repeated span, taps, norm groups,
experts, rotary constants, multipliers), through the engine against the plain oracle: what holds for the hand-made
configurations of the other tests must hold for any, in particular sizes that are no multiple of a vector or of a
matrix tile.  CPU: eager stand-ins; gpu: the HIP kernels in float32 (tight) and bfloat16 (rounding-sized)."""
import math
import os
import random

import pytest
import torch

from benarax_util import make_engine, oracle_logits, random_checkpoint, replay, steady_prefix

BACKENDS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
            pytest.param(("cuda", torch.float32), id="gpu-f32", marks=pytest.mark.gpu),
            pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=pytest.mark.gpu)]


def draw_config(seed: int) -> dict:
    rng = random.Random(seed)
    groups = rng.choice([1, 2, 3, 4, 6])
    width = groups * rng.choice([8, 10, 12, 16, 22, 32])
    n_layers = rng.randint(1, 4)

    def mlp():
        if rng.random() < 0.15:
            return None
        experts = rng.randint(1, 10)
        return {"kind": "moe", "router": {"experts": experts, "top": rng.randint(1, min(experts, 4))},
                "expert": {"ff": rng.choice([4, 8, 12, 20, 32, 40, 72]), "limit": rng.choice([0.5, 1.0, 3.0, 7.0])}}

    layers = []
    for _ in range(n_layers):
        kind = rng.choice(["general_delta", "latent_attention", "latent_attention_2"])
        if kind == "general_delta":
            mixer = {"heads": rng.randint(1, 5), "dim": rng.choice([4, 8, 12, 16, 20, 32, 36, 64, 72])}
        else:
            dim, rot = rng.choice([4, 8, 16, 24, 32, 48]), rng.choice([2, 4, 8, 12, 16, 32])
            r = {"dims": rot, "base": rng.choice([100.0, 1e4, 3e5])}
            if rng.random() < 0.5:
                r["scaling"] = {"factor": rng.choice([2.0, 4.0, 16.0]), "fast": rng.choice([4.0, 16.0, 32.0]),
                                "slow": rng.choice([0.5, 1.0, 2.0]), "original": rng.choice([8, 32, 256])}
            mixer = {"heads": rng.randint(1, 6), "dim": dim, "rot_dim": rot, "vdim": rng.choice([4, 8, 12, 16, 40]),
                     "q_rank": rng.choice([5, 8, 16, 24, 48]), "kv_rank": rng.choice([8, 12, 16, 24, 32, 48, 64, 96, 100]),
                     "rot": r, "scale": rng.choice([0.5, 1.0, 1.5]) / math.sqrt(dim + rot)}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp()})
    start = rng.randint(0, n_layers)
    stop = rng.randint(start, n_layers)
    cfg = {"architecture": "Benarax", "layers": layers, "loop": {"start": start, "stop": stop, "times": rng.randint(1, 3)},
           "norm": {"eps": rng.choice([1e-6, 1e-5, 1e-4]), "groups": groups}, "vocab": rng.randint(20, 120), "width": width,
           "residual_mult": rng.choice([0.3, 0.7, 1.0, 1.4]), "embedding": {"scale": rng.choice([0.5, 1.0, 4.0, 9.0])},
           "logit_scale": rng.choice([0.1, 0.5, 1.0, 2.0])}
    taps, side = rng.choice([0, 1, 2, 3, 4, 5]), rng.choice([0, 1, 3, 4, 8, 9])
    if taps:
        cfg["canon"] = {"taps": taps}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


def per_position(got, want):
    """Per position: rms over the vocabulary of the difference with its mean removed, over the rms of the logits."""
    d = got.float() - want.float()
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.float().pow(2).mean().sqrt()


@pytest.fixture(params=BACKENDS)
def backend(request):
    return request.param


@pytest.mark.parametrize("seed", range(int(os.environ.get("NV_RANDOM_CONFIGS", "12"))))      # more for a longer sweep
def test_random_configuration(seed, backend):
    dev, dtype = backend
    if True:      # (one indented body for every backend)
        cfg = draw_config(seed)
        ck = random_checkpoint(cfg, seed=100 + seed, rank=1 + seed % 5)
        g = torch.Generator().manual_seed(seed)
        V = cfg["vocab"]
        p = {"a": torch.randint(0, V, (29,), generator=g).tolist(), "b": torch.randint(0, V, (7,), generator=g).tolist(),
             "c": torch.randint(0, V, (40,), generator=g).tolist()}
        portions = {"a": [6, 1, 1, 14, 2, 1], "b": [1], "c": [2, 3, 30, 1]}
        got = replay(make_engine(cfg, ck, dev, dtype, block_size=4, num_blocks=40, max_seqs=3), p, portions, order={"b": 2, "c": 1})
        # Per position, against what the oracle's own bfloat16 evaluation loses there (deep random models have
        # ill-conditioned spots: a normalised vector that is almost zero, a softmax between two equal scores).
        # float32: every position within 1e-4, or within 2 % of that loss where it is large.  bfloat16: a fault moves
        # most positions, rounding moves a few by more than three times the oracle's loss.
        errs, noises = [], []
        for i in p:
            want = oracle_logits(cfg, ck, p[i])
            n = len(p[i]) if dtype == torch.float32 else steady_prefix(cfg, ck, p[i])
            if n:
                errs.append(per_position(got[i][:n], want[:n]))
                noises.append(per_position(oracle_logits(cfg, ck, p[i], torch.bfloat16)[:n], want[:n]))
        if not errs:
            return
        err, noise = torch.cat(errs), torch.cat(noises)
        if dtype == torch.float32:
            assert bool((err < torch.clamp(0.02 * noise, min=1e-4)).all()), (seed, dev, err.max().item())
        else:
            limit = 3 * torch.clamp(noise, min=noise.median().item()) + 1e-3
            assert int((err > limit).sum()) <= max(1, err.numel() // 10), (seed, (err / limit).topk(min(5, err.numel())).values.tolist())
            if err.numel() >= 20:
                assert err.median().item() <= 2 * noise.median().item() + 1e-3, (seed, err.median().item(), noise.median().item())
