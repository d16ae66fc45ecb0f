"""Buvalix through the engine against the plain oracle (oracle/ref_buvalix.py: whole sequences, no cache).

Every test runs twice: on the CPU with the eager stand-in layers (host logic: scheduler, block and slot managers,
runner, model wiring) and, marked gpu, on the HIP kernels.  Float32 keeps the comparison tight (a key that is off
by one, a lost state or a stale slot is far outside it); the GPU also runs bfloat16 with a rounding-sized bound.
Small configurations of the tests' own: unequal head counts everywhere, key size != value size, several taps,
repeated passes with start > 0 and stop < number of layers."""
import pytest
import torch

from buvalix_util import (attention2_layer, attention_layer, config, delta_layer, make_engine, oracle_logits,
                          random_checkpoint, rel_err, replay)
from nanovllm_amd.engine.sequence import SamplingParams
from oracle import ref_buvalix

BACKENDS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
            pytest.param(("cuda", torch.float32), id="gpu-f32", marks=pytest.mark.gpu),
            pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def backend(request):
    return request.param


def bound(dtype):
    return 5e-5 if dtype == torch.float32 else 6e-2      # float32: rounding over a dozen layer runs stays below 3e-5


def assert_close_to_oracle(got, cfg, ck, prompt, dtype, what=""):
    """float32: a fixed tight bound.  bfloat16: against the float32 oracle, at most three times the error that the
    oracle's own bfloat16 evaluation makes on this prompt (rounding alone), so the bound follows the model's depth
    and width instead of being tuned."""
    want = oracle_logits(cfg, ck, prompt, torch.float32)
    assert got.shape == want.shape
    err = rel_err(got, want)
    if dtype == torch.float32:
        assert err < bound(dtype), (what, err)
    else:
        noise = rel_err(oracle_logits(cfg, ck, prompt, torch.bfloat16), want)
        assert err < 3 * noise, (what, err, noise)


def tokens(n, seed, vocab=97):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


MIXED = config([delta_layer(), attention_layer(), attention2_layer(), delta_layer(heads=2, kv_heads=1, conv=2, ff=40),
                attention_layer(heads=3, kv_heads=3, dim=10, vdim=10, rot_dims=10, ff=None)],
               loop={"start": 1, "stop": 4, "times": 3})
SINGLE = {"attention": config([attention_layer()]),
          "attention_2": config([attention2_layer()]),
          "channel_delta": config([delta_layer(ff=24)]),
          "delta_one_tap": config([delta_layer(conv=1, heads=3, kv_heads=3)]),
          "looped_from_0": config([attention2_layer(heads=2, kv_heads=1), delta_layer()],
                                  loop={"start": 0, "stop": 2, "times": 2})}


def check(engine, cfg, ck, prompts, portions, dtype, order=None):
    got = replay(engine, prompts, portions, order)
    for i, p in prompts.items():
        assert_close_to_oracle(got[i], cfg, ck, p, dtype, i)


@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mixer_alone_whole_prompt_and_token_by_token(backend, name):
    dev, dtype = backend
    cfg = SINGLE[name]
    ck = random_checkpoint(cfg, seed=len(name))
    p = {"a": tokens(45, 1)}
    check(make_engine(cfg, ck, dev, dtype), cfg, ck, p, {"a": [45]}, dtype)
    check(make_engine(cfg, ck, dev, dtype), cfg, ck, p, {"a": [1]}, dtype)


def test_whole_model_portions_of_many_sizes(backend):
    dev, dtype = backend
    ck = random_checkpoint(MIXED, seed=2)
    p = {"a": tokens(61, 3)}
    for sizes in ([61], [2], [3, 2, 7, 1, 1, 16, 2, 5], [1, 4, 4, 4], [17, 1]):
        check(make_engine(MIXED, ck, dev, dtype), MIXED, ck, p, {"a": sizes}, dtype)


def test_unfused_boundaries_and_streams_match_the_oracle(backend):
    dev, dtype = backend
    if dtype != torch.float32:
        pytest.skip("streams are compared in float32")
    ck = random_checkpoint(MIXED, seed=4)
    toks = tokens(19, 5)
    eng = make_engine(MIXED, ck, dev, dtype, fused=False)
    check(eng, MIXED, ck, {"a": toks}, {"a": [6, 13]}, dtype)
    # the residual stream after every run, one whole prompt
    eng = make_engine(MIXED, ck, dev, dtype, fused=False)
    streams = []
    model = eng.runner.model
    orig = model.forward
    model.forward = lambda *a, **k: orig(*a, streams=streams, **k)
    eng.replay_step([("a", toks, [0])], ["a"])
    want = ref_buvalix.forward(MIXED, ck, toks, dtype)[1]
    assert len(streams) == want.shape[0] == 1 + 3 * 3 + 1
    for r, s in enumerate(streams):
        torch.testing.assert_close(s.cpu(), want[r], rtol=1e-4, atol=1e-4)


def test_unequal_requests_in_one_batch_equal_each_alone(backend):
    dev, dtype = backend
    ck = random_checkpoint(MIXED, seed=6)
    p = {"a": tokens(37, 7), "b": tokens(9, 8), "c": tokens(1, 9), "d": tokens(23, 10)}
    portions = {"a": [5, 1, 1, 9, 1], "b": [1], "c": [1], "d": [2, 11, 1]}
    eng = make_engine(MIXED, ck, dev, dtype)
    check(eng, MIXED, ck, p, portions, dtype, order={"b": 1, "d": 2})
    if dtype != torch.float32:
        return            # bfloat16 matrix products round differently for other batch shapes; the oracle bound above holds
    # the same portions alone: same logits up to rounding
    together = replay(make_engine(MIXED, ck, dev, dtype), p, portions, order={"b": 1, "d": 2})
    for i in p:
        alone = replay(make_engine(MIXED, ck, dev, dtype), {i: p[i]}, {i: portions[i]})
        assert rel_err(together[i], alone[i]) < bound(dtype)


def test_pages_and_slots_are_used_again(backend):
    """A pool that holds two requests at a time, six requests in a row: every page and both slots are reused with
    what the previous owner left in them."""
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
    # a fifth live request has no slot; a step that outgrows the pool is refused
    eng = make_engine(MIXED, ck, dev, dtype, block_size=4, num_blocks=3, max_seqs=1)
    eng.replay_step([("a", tokens(5, 1), [])])
    with pytest.raises(ValueError):
        eng.replay_step([("b", tokens(2, 2), [])])
    with pytest.raises(ValueError):
        eng.replay_step([("a", tokens(9, 3), [])])


def test_long_decoding_past_every_edge(backend):
    """A short prompt and 150 single tokens: they cross page borders (every 4), the distance table's exact / shared
    / last rows (bias_max 40, far beyond it), the query temperature's steps (every 7) and the first tokens."""
    dev, dtype = backend
    cfg = config([attention2_layer(bias_max=40, every=7), delta_layer(conv=3), attention_layer()],
                 loop={"start": 0, "stop": 3, "times": 2})
    ck = random_checkpoint(cfg, seed=12, rel_rows=16)
    p = {"a": tokens(153, 13)}
    check(make_engine(cfg, ck, dev, dtype, num_blocks=40), cfg, ck, p, {"a": [3, 1]}, dtype)


def test_greedy_generation_through_generate(backend):
    dev, dtype = backend
    if dtype != torch.float32:
        pytest.skip("token equality is asserted in float32")
    ck = random_checkpoint(MIXED, seed=14)
    prompts = [tokens(11, 15), tokens(3, 16), tokens(26, 17)]
    eng = make_engine(MIXED, ck, dev, dtype, block_size=4, num_blocks=40, max_seqs=2,       # the third waits for a slot
                      max_num_batched_tokens=16, long_prefill_token_threshold=6)
    outs, _ = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12))
    for p, o in zip(prompts, outs):
        seq = list(p)
        for _ in range(12):
            seq.append(int(oracle_logits(MIXED, ck, seq, dtype)[-1].argmax()))
        assert o["token_ids"] == seq[len(p):]
    assert eng.scheduler.state_slots.num_free == 2 and eng.scheduler.block_manager.num_free_blocks == 40


def test_sampled_generation_runs_and_preemption_recomputes_state(backend):
    """A cache too small for both requests to finish: the younger one is preempted, loses its slot and its pages,
    and is recomputed from position 0 (greedy tokens still equal the oracle's)."""
    dev, dtype = backend
    if dtype != torch.float32:
        pytest.skip("token equality is asserted in float32")
    ck = random_checkpoint(MIXED, seed=18)
    prompts = [tokens(10, 19), tokens(9, 20)]
    eng = make_engine(MIXED, ck, dev, dtype, block_size=4, num_blocks=9, max_seqs=2)
    outs, _ = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=14))
    assert sum(o["num_preemptions"] for o in outs) >= 1
    for p, o in zip(prompts, outs):
        seq = list(p)
        for _ in range(14):
            seq.append(int(oracle_logits(MIXED, ck, seq, dtype)[-1].argmax()))
        assert o["token_ids"] == seq[len(p):]
    outs, _ = make_engine(MIXED, ck, dev, dtype).generate(prompts, SamplingParams(temperature=0.8, max_tokens=5))
    assert all(len(o["token_ids"]) == 5 for o in outs)
