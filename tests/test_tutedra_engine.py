"""Tutedra through the engine against the plain oracle (oracle/ref_tutedra.py: whole sequences, no cache).

Every test runs on the CPU with the eager stand-in layers (host logic: scheduler, block and slot managers, runner,
model wiring) and, marked gpu, on the HIP kernels in float32 and bfloat16.  Float32 keeps the comparison tight (a key
that is off by one, a lost state, a stale slot, a missing shift or a wrong expert is far outside it); bfloat16 is bounded
by three times the error the oracle's own bfloat16 evaluation makes.  Small configurations of the tests' own: odd head
counts, key size != value size, partial and full and no rotary, with and without frequency rescaling, one to five
taps and no convolution, every feed-forward kind on every mixer kind, a layer without feed-forward, groups of one
expert, one group, no shared expert, checkpoints without column scales, shift or selection bias, no bigram table."""
import pytest
import torch

from nanovllm_amd.engine.sequence import SamplingParams
from oracle import ref_tutedra
from tutedra_util import (attention_layer, config, dense, hgrn2_layer, make_engine, mlstm_layer, moe, oracle_logits,
                          random_checkpoint, rel_err, replay)

BACKENDS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
            pytest.param(("cuda", torch.float32), id="gpu-f32", marks=pytest.mark.gpu),
            pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def backend(request):
    return request.param


def bound(dtype):
    return 5e-5 if dtype == torch.float32 else 6e-2


def per_position(got, want):
    d = got.float() - want.float()
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.float().pow(2).mean().sqrt()


def assert_close_to_oracle(got, cfg, ck, prompt, dtype, what=""):
    """float32: every position.  bfloat16: against what the oracle's own bfloat16 evaluation loses per position; a fault
    moves most positions, while rounding can turn a close call of a router (two experts whose scores differ by less
    than the rounding) and move that position and the ones behind it that read it through a state: at most one
    position in ten may exceed three times the oracle's loss (not counting the trail behind the largest excess), and the
    median must not move."""
    want = oracle_logits(cfg, ck, prompt, torch.float32)
    assert got.shape == want.shape
    if dtype == torch.float32:
        err = rel_err(got, want)
        assert err < bound(dtype), (what, err)
    else:
        err = per_position(got, want)
        noise = per_position(oracle_logits(cfg, ck, prompt, torch.bfloat16), want)
        limit = 3 * torch.clamp(noise, min=noise.median().item()) + 1e-3
        over = (err > limit).nonzero().flatten().tolist()
        if len(over) > max(1, err.numel() // 10):          # the fading trail behind the largest excess does not count
            worst = int((err / limit).argmax())
            over = [at for at in over if at <= worst]
        assert len(over) <= max(1, err.numel() // 10), (what, (err / limit).topk(5).values.tolist())
        assert err.median().item() <= 2 * noise.median().item() + 1e-3, (what, err.median().item(), noise.median().item())


def tokens(n, seed, vocab=83):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


MIXED = config([mlstm_layer(), hgrn2_layer(), attention_layer(), mlstm_layer(heads=2, dim=6, vdim=11, mlp=moe(experts=4, top=1, groups=4, keep=2, shared=0)),
                attention_layer(heads=3, kv_heads=3, dim=10, conv=2, rot_dims=10, scaling=None, mlp=None),
                hgrn2_layer(heads=3, dim=5, vdim=5, mlp=dense(20))])
SINGLE = {"mlstm": config([mlstm_layer()]),
          "mlstm_moe_one_group": config([mlstm_layer(heads=1, dim=16, vdim=16, cap=4.0, mlp=moe(experts=5, top=3, groups=0))]),
          "hgrn2": config([hgrn2_layer()]),
          "hgrn2_no_ff": config([hgrn2_layer(heads=1, dim=7, vdim=20, mlp=None)]),
          "attention": config([attention_layer()]),
          "attention_no_conv_no_rotary": config([attention_layer(conv=0, rot_dims=0, kv_heads=1)]),
          "attention_one_tap_full_rotary": config([attention_layer(conv=1, rot_dims=12, scaling=None, mlp=moe(experts=8, top=2, groups=8, keep=3))]),
          "no_bigram": config([attention_layer(conv=5), mlstm_layer()], buckets=0)}


def check(engine, cfg, ck, prompts, portions, dtype, order=None):
    got = replay(engine, prompts, portions, order)
    for i, p in prompts.items():
        assert_close_to_oracle(got[i], cfg, ck, p, dtype, i)


@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_layer_kind_alone_whole_prompt_and_token_by_token(backend, name):
    dev, dtype = backend
    cfg = SINGLE[name]
    ck = random_checkpoint(cfg, seed=len(name))
    p = {"a": tokens(41, 1)}
    check(make_engine(cfg, ck, dev, dtype), cfg, ck, p, {"a": [41]}, dtype)
    check(make_engine(cfg, ck, dev, dtype), cfg, ck, p, {"a": [1]}, dtype)


@pytest.mark.parametrize("has", [dict(scales=False), dict(shift=False), dict(correction=False)], ids=lambda d: "no_" + next(iter(d)))
def test_checkpoints_without_the_optional_tensors(backend, has):
    dev, dtype = backend
    ck = random_checkpoint(MIXED, seed=31, **has)
    p = {"a": tokens(23, 32)}
    check(make_engine(MIXED, ck, dev, dtype), MIXED, ck, p, {"a": [5, 1, 2]}, dtype)


def test_whole_model_portions_of_many_sizes(backend):
    dev, dtype = backend
    ck = random_checkpoint(MIXED, seed=2)
    p = {"a": tokens(53, 3)}
    for sizes in ([53], [2], [3, 2, 7, 1, 1, 16, 2, 5], [1, 4, 4, 4], [17, 1], [6, 1, 7, 7]):
        check(make_engine(MIXED, ck, dev, dtype), MIXED, ck, p, {"a": sizes}, dtype)


def test_streams_after_every_layer_match_the_oracle(backend):
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
    want_logits, want = ref_tutedra.forward(MIXED, ck, toks, dtype)
    assert len(streams) == want.shape[0] == 6
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
    what the previous owner left in them (keys and values, memories with their normalisers and maxima, carried
    convolution inputs and shift rows, the previous token id)."""
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
    """A short prompt and 140 single tokens: they cross page borders (every 4), the rescaled rotary band, and leave the
    first tokens far behind, reachable through the attention's cache and the recurrent states."""
    dev, dtype = backend
    cfg = config([attention_layer(), mlstm_layer(), hgrn2_layer(mlp=dense())])
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


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_head_sizes_of_the_tile_kernels_through_the_engine(dtype):
    """Key sizes 64 and 128 with many query heads per key head, memories of 64 and 128 channels: prompt portions of the
    attention take its MFMA tile kernel, single rows its decode kernel; pages of 16."""
    cfg = config([attention_layer(heads=12, kv_heads=1, dim=64, conv=4, rot_dims=32, mlp=dense(64)),
                  mlstm_layer(heads=2, dim=64, vdim=128, mlp=moe(experts=9, top=2, ff=32, groups=3, keep=2, shared=48)),
                  hgrn2_layer(heads=2, dim=128, vdim=64, mlp=None),
                  attention_layer(heads=4, kv_heads=2, dim=128, conv=2, rot_dims=128, mlp=None)], width=64)
    ck = random_checkpoint(cfg, seed=21)
    p = {"a": tokens(333, 22), "b": tokens(70, 23), "c": tokens(150, 24)}
    eng = make_engine(cfg, ck, "cuda", dtype, block_size=16, num_blocks=64)
    check(eng, cfg, ck, p, {"a": [130, 1, 67, 64, 1, 70], "b": [1], "c": [65, 2, 83]}, dtype, order={"b": 1, "c": 2})


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_the_largest_head_sizes_through_the_engine(dtype):
    """Memories of up to 256 x 256 channels (64 key rows per lane, the 1024-thread instantiation, fewer tokens per LDS
    tile) and attention heads of 160 and 256 dimensions (the one-dimension-per-lane norm kernel, the wide attention
    tiles), eleven taps (beyond the register window)."""
    cfg = config([mlstm_layer(heads=1, dim=200, vdim=160, mlp=None), hgrn2_layer(heads=1, dim=256, vdim=256, mlp=dense(96)),
                  attention_layer(heads=2, kv_heads=1, dim=160, conv=11, rot_dims=64, mlp=None),
                  attention_layer(heads=2, kv_heads=2, dim=256, conv=2, rot_dims=256, scaling=None, mlp=moe(experts=4, top=2, ff=40, groups=2, keep=2, shared=33))],
                 width=48)
    ck = random_checkpoint(cfg, seed=41)
    p = {"a": tokens(150, 42), "b": tokens(40, 43)}
    eng = make_engine(cfg, ck, "cuda", dtype, block_size=16, num_blocks=24)
    check(eng, cfg, ck, p, {"a": [70, 1, 2, 66, 1], "b": [1]}, dtype, order={"b": 1})
