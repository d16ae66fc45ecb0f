"""Benarax through the engine against the plain oracle (oracle/ref_benarax.py: whole sequences, no cache).

Every test runs on the CPU with the eager stand-in layers (host logic: scheduler, block and slot managers, runner,
model wiring) and, marked gpu, on the HIP kernels in float32 and bfloat16.  Float32 keeps the comparison tight (a key
that is off by one, a lost state, a stale slot or a wrong expert is far outside it); bfloat16 is bounded by three
times the error the oracle's own bfloat16 evaluation makes.  Small configurations of the tests' own: odd head counts,
key size != value size != rotated size, two and five taps, three norm groups, repeated passes with start > 0 and
stop < number of layers, a layer without feed-forward, top = 1 and top = experts."""
import pytest
import torch

from benarax_util import (config, delta_layer, latent_layer, make_engine, moe, oracle_logits, random_checkpoint, rel_err,
                          replay, steady_prefix)
from nanovllm_amd.engine.sequence import SamplingParams
from oracle import ref_benarax

BACKENDS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
            pytest.param(("cuda", torch.float32), id="gpu-f32", marks=pytest.mark.gpu),
            pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def backend(request):
    return request.param


def bound(dtype):
    return 5e-5 if dtype == torch.float32 else 6e-2


def assert_close_to_oracle(got, cfg, ck, prompt, dtype, what=""):
    """float32: a fixed tight bound.  bfloat16: at most three times the error that the oracle's own bfloat16
    evaluation makes (rounding alone), over the positions before the first close call of a router: where the last
    chosen expert leads the next one by less than a twentieth of the logits' spread, rounding may choose the other
    one, and everything after that token differs by more than rounding."""
    want = oracle_logits(cfg, ck, prompt, torch.float32)
    assert got.shape == want.shape
    if dtype == torch.float32:
        err = rel_err(got, want)
        assert err < bound(dtype), (what, err)
        return
    n = steady_prefix(cfg, ck, prompt)
    if n:
        noise = rel_err(oracle_logits(cfg, ck, prompt, torch.bfloat16)[:n], want[:n])
        err = rel_err(got[:n], want[:n])
        assert err < 3 * noise, (what, err, noise, n)


def tokens(n, seed, vocab=83):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


MIXED = config([delta_layer(), latent_layer(), latent_layer("latent_attention_2", heads=2, dim=8, rot_dim=4, vdim=6, kv_rank=12),
                delta_layer(heads=2, dim=20, mlp=None), latent_layer(mlp=moe(experts=3, top=3, ff=10))],
               loop={"start": 1, "stop": 4, "times": 2})
SINGLE = {"general_delta": config([delta_layer()]),
          "latent_attention": config([latent_layer()]),
          "latent_attention_2": config([latent_layer("latent_attention_2")], taps=5, groups=1),
          "plain_rotary_interleaved": config([latent_layer(scaling=None, mlp=moe(experts=4, top=1))], taps=2),
          "no_conv_no_side": config([latent_layer(), delta_layer()], taps=0, side=0, mult=1.0),
          "looped_from_0": config([latent_layer("latent_attention_2", heads=1), delta_layer(heads=1)],
                                  loop={"start": 0, "stop": 2, "times": 3}, groups=2)}


def check(engine, cfg, ck, prompts, portions, dtype, order=None):
    got = replay(engine, prompts, portions, order)
    for i, p in prompts.items():
        assert_close_to_oracle(got[i], cfg, ck, p, dtype, i)


@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mixer_alone_whole_prompt_and_token_by_token(backend, name):
    dev, dtype = backend
    cfg = SINGLE[name]
    ck = random_checkpoint(cfg, seed=len(name))
    p = {"a": tokens(41, 1)}
    check(make_engine(cfg, ck, dev, dtype), cfg, ck, p, {"a": [41]}, dtype)
    check(make_engine(cfg, ck, dev, dtype), cfg, ck, p, {"a": [1]}, dtype)


def test_whole_model_portions_of_many_sizes(backend):
    dev, dtype = backend
    ck = random_checkpoint(MIXED, seed=2)
    p = {"a": tokens(53, 3)}
    for sizes in ([53], [2], [3, 2, 7, 1, 1, 16, 2, 5], [1, 4, 4, 4], [17, 1]):
        check(make_engine(MIXED, ck, dev, dtype), MIXED, ck, p, {"a": sizes}, dtype)


def test_streams_after_every_run_match_the_oracle(backend):
    dev, dtype = backend
    if dtype != torch.float32:
        pytest.skip("streams are compared in float32")
    ck = random_checkpoint(MIXED, seed=4)
    toks = tokens(19, 5)
    eng = make_engine(MIXED, ck, dev, dtype)
    streams = []
    model = eng.runner.model
    orig = model.forward
    model.forward = lambda *a, **k: orig(*a, streams=streams, **k)
    got = eng.replay_step([("a", toks, [0, 18])], ["a"])
    want_logits, want = ref_benarax.forward(MIXED, ck, toks, dtype)
    assert len(streams) == want.shape[0] == 1 + 3 * 2 + 1
    for r, s in enumerate(streams):
        torch.testing.assert_close(s.cpu(), want[r], rtol=1e-4, atol=1e-4)
    assert rel_err(got.cpu(), want_logits[[0, 18]]) < bound(dtype)


def test_unequal_requests_in_one_batch_equal_each_alone(backend):
    dev, dtype = backend
    ck = random_checkpoint(MIXED, seed=6)
    p = {"a": tokens(37, 7), "b": tokens(9, 8), "c": tokens(1, 9), "d": tokens(23, 10)}
    portions = {"a": [5, 1, 1, 9, 1], "b": [1], "c": [1], "d": [2, 11, 1]}
    eng = make_engine(MIXED, ck, dev, dtype)
    check(eng, MIXED, ck, p, portions, dtype, order={"b": 1, "d": 2})
    if dtype != torch.float32:
        return
    together = replay(make_engine(MIXED, ck, dev, dtype), p, portions, order={"b": 1, "d": 2})
    for i in p:
        alone = replay(make_engine(MIXED, ck, dev, dtype), {i: p[i]}, {i: portions[i]})
        assert rel_err(together[i], alone[i]) < bound(dtype)


def test_pages_and_slots_are_used_again(backend):
    """A pool that holds two requests at a time, six requests in a row: every page and both slots are reused with
    what the previous owner left in them (latents, recurrent states, carried convolution inputs)."""
    dev, dtype = backend
    ck = random_checkpoint(MIXED, seed=11)
    eng = make_engine(MIXED, ck, dev, dtype, block_size=4, num_blocks=12, max_seqs=2)
    for r in range(3):
        p = {f"x{r}": tokens(22 - r, 20 + r), f"y{r}": tokens(13 + 3 * r, 30 + r)}
        got = replay(eng, p, {f"x{r}": [7, 2, 1], f"y{r}": [1, 5]})
        for i in p:
            assert_close_to_oracle(got[i], MIXED, ck, p[i], dtype, (r, i))
        assert eng.scheduler.block_manager.num_free_blocks == 12 and eng.scheduler.state_slots.num_free == 2
    assert not eng.scheduler.running and not eng.scheduler.waiting
    eng = make_engine(MIXED, ck, dev, dtype, block_size=4, num_blocks=3, max_seqs=1)
    eng.replay_step([("a", tokens(5, 1), [])])
    with pytest.raises(ValueError):
        eng.replay_step([("b", tokens(2, 2), [])])
    with pytest.raises(ValueError):
        eng.replay_step([("a", tokens(9, 3), [])])


def test_long_decoding_past_every_edge(backend):
    """A short prompt and 140 single tokens: they cross page borders (every 4), run far past the positions the blended
    rotary frequencies were made for (original 24), and leave the first tokens far behind."""
    dev, dtype = backend
    cfg = config([latent_layer(), delta_layer(), latent_layer("latent_attention_2")], loop={"start": 0, "stop": 3, "times": 2},
                 taps=4)
    ck = random_checkpoint(cfg, seed=12)
    p = {"a": tokens(143, 13)}
    check(make_engine(cfg, ck, dev, dtype, num_blocks=40), cfg, ck, p, {"a": [3, 1]}, dtype)


def test_greedy_generation_through_generate(backend):
    dev, dtype = backend
    if dtype != torch.float32:
        pytest.skip("token equality is asserted in float32")
    ck = random_checkpoint(MIXED, seed=14)
    prompts = [tokens(11, 15), tokens(3, 16), tokens(26, 17)]
    eng = make_engine(MIXED, ck, dev, dtype, block_size=4, num_blocks=40, max_seqs=2,       # the third waits for a slot
                      max_num_batched_tokens=16, long_prefill_token_threshold=6)
    outs, _ = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10))
    for p, o in zip(prompts, outs):
        seq = list(p)
        for _ in range(10):
            seq.append(int(oracle_logits(MIXED, ck, seq, dtype)[-1].argmax()))
        assert o["token_ids"] == seq[len(p):]
    assert eng.scheduler.state_slots.num_free == 2 and eng.scheduler.block_manager.num_free_blocks == 40


def test_preemption_recomputes_state_and_sampling_runs(backend):
    dev, dtype = backend
    if dtype != torch.float32:
        pytest.skip("token equality is asserted in float32")
    ck = random_checkpoint(MIXED, seed=18)
    prompts = [tokens(10, 19), tokens(9, 20)]
    eng = make_engine(MIXED, ck, dev, dtype, block_size=4, num_blocks=9, max_seqs=2)
    outs, _ = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12))
    assert sum(o["num_preemptions"] for o in outs) >= 1
    for p, o in zip(prompts, outs):
        seq = list(p)
        for _ in range(12):
            seq.append(int(oracle_logits(MIXED, ck, seq, dtype)[-1].argmax()))
        assert o["token_ids"] == seq[len(p):]
    outs, _ = make_engine(MIXED, ck, dev, dtype).generate(prompts, SamplingParams(temperature=0.8, max_tokens=5))
    assert all(len(o["token_ids"]) == 5 for o in outs)
