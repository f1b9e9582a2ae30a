"""Rugudra on the GPU against the plain restatement of the design (tests/rugudra_reference.py): every mechanism alone, prompts against
token-by-token decoding, portions down to two tokens, unequal batches, pages and state slots that are used again, keys far away and at
page / tile borders, the first tokens of a sequence, long decoding, odd sizes, and greedy generation through the engine's scheduler."""
import numpy as np
import pytest

import nvr_import
from rugudra_util import (Driver, TOL, attention_layer, expected_logits, make_config, make_weights, retention_layer, row_errors, bf16_round)

pytestmark = pytest.mark.gpu


def tokens_of(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


def check(got, want, dtype, what=""):
    e = row_errors(got, want)
    assert e.max() < TOL[dtype], f"{what}: row {int(e.argmax())} differs by {e.max():.3g} of the row's spread (limit {TOL[dtype]})"


# ------------------------------------------------------------------------------------------------ each mechanism alone
MECHANISMS = {
    "norm_and_convolution_taps_1": make_config([attention_layer(ff=None)], taps=1),
    "norm_and_convolution_taps_2": make_config([attention_layer(ff=None)], taps=2),
    "norm_and_convolution_taps_5": make_config([retention_layer(ff=None)], taps=5),
    "attention_grouped_heads": make_config([attention_layer(heads=6, kv_heads=2, dim=32, vdim=16, ff=None)]),
    "attention_one_kv_head_per_head": make_config([attention_layer(heads=3, kv_heads=3, dim=32, vdim=32, scale=0.3, ff=None)]),
    "attention_single_kv_head": make_config([attention_layer(heads=4, kv_heads=1, dim=64, vdim=48, ff=None)]),
    "attention_64_pairs_of_heads": make_config([attention_layer(heads=4, kv_heads=2, dim=64, vdim=64, ff=None)]),
    "attention_128_four_heads_per_kv_head": make_config([attention_layer(heads=4, kv_heads=1, dim=128, vdim=128, scale=0.05, ff=None)], width=128),
    "attention_128_one_head_per_kv_head": make_config([attention_layer(heads=2, kv_heads=2, dim=128, vdim=128, scale=0.07, ff=24)]),
    "retention_full_rotation": make_config([retention_layer(heads=3, dim=32, vdim=16, ff=None)]),
    "retention_partial_rotation": make_config([retention_layer(heads=2, dim=32, vdim=32, rot_dims=12, base=77.0, ff=None)]),
    "retention_no_rotation": make_config([retention_layer(heads=2, dim=16, vdim=40, rot_dims=0, ff=None)]),
    "feed_forward_clamped": make_config([attention_layer(ff=80, limit=0.4)]),
    "loop_of_two_layers_three_times": make_config([attention_layer(), retention_layer(), attention_layer(heads=2, kv_heads=2)], loop=(0, 2, 3)),
    "loop_once_and_scales_of_one": make_config([retention_layer(), attention_layer()], loop=(1, 2, 1), residual_mult=1.0, embedding_scale=1.0),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(name, dtype):
    cfg = MECHANISMS[name]
    w = make_weights(cfg, seed=len(name))
    toks = tokens_of(70, cfg["vocab"], 1)
    d = Driver(cfg, w, dtype)
    check(d.run_alone(toks), expected_logits(cfg, w, toks), dtype, name)


def test_sink_and_penalty_each_change_the_result():
    """A sink that is left out, or a penalty that is, must show: the same model with sink = -30 (no sink) and r1 = 0 (no penalty) differs from the full one by far
    more than the tolerance, and each variant agrees with the reference."""
    cfg = make_config([attention_layer(ff=None)], taps=1)
    w = make_weights(cfg, seed=3, gain=2.0)
    toks = tokens_of(50, cfg["vocab"], 2)
    full = expected_logits(cfg, w, toks)
    for key, val in (("l0.mix.sink", -30.0), ("l0.mix.r1", 0.0)):
        w2 = dict(w); w2[key] = np.full_like(w[key], val)
        want = expected_logits(cfg, w2, toks)
        assert row_errors(want, full).max() > 50 * TOL["float32"]
        check(Driver(cfg, w2, "float32").run_alone(toks), want, "float32", key)
    check(Driver(cfg, w, "float32").run_alone(toks), full, "float32", "full")


# ------------------------------------------------------------------------------------------------ a model with everything, in portions and batches
def hybrid(vocab=131, width=96):
    layers = [attention_layer(heads=4, kv_heads=2, dim=64, vdim=64, ff=64),
              retention_layer(heads=2, dim=32, vdim=16, rot_dims=16, ff=None),
              attention_layer(heads=2, kv_heads=1, dim=64, vdim=32, scale=0.11, ff=80, limit=0.9),
              retention_layer(heads=3, dim=16, vdim=32, ff=48)]
    return make_config(layers, vocab=vocab, width=width, taps=4, loop=(1, 3, 2))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_against_token_by_token_decoding(dtype):
    cfg = hybrid(); w = make_weights(cfg, seed=5)
    toks = tokens_of(90, cfg["vocab"], 3)
    want = expected_logits(cfg, w, toks)
    d = Driver(cfg, w, dtype)
    whole = d.run_alone(toks)
    single = d.run_alone(toks, cuts=[1])
    mostly = d.run_alone(toks, cuts=[57, 1])
    for got, what in ((whole, "whole"), (single, "token by token"), (mostly, "prompt then tokens")):
        check(got, want, dtype, what)
    if dtype == "float32":
        assert row_errors(single, whole).max() < 1e-4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cuts", [[2], [3, 2, 17, 2, 5, 1], [16, 16, 2, 30, 1], [15, 1, 16, 17], [64, 2, 63, 1]])
def test_portions_of_several_sizes(cuts, dtype):
    cfg = hybrid(); w = make_weights(cfg, seed=6)
    toks = tokens_of(150 if len(cuts) > 1 else 40, cfg["vocab"], 4)
    check(Driver(cfg, w, dtype).run_alone(toks, cuts=cuts), expected_logits(cfg, w, toks), dtype, str(cuts))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_against_each_alone_and_slots_and_pages_used_again(dtype):
    """Four live requests of unequal length, portions of some beside single tokens of others, a fifth and sixth request that take over the pages and the state
    slot of finished ones (a pool of 24 pages of 16 tokens for six requests of 330 tokens in all)."""
    cfg = hybrid(); w = make_weights(cfg, seed=7)
    lens = {"a": 75, "b": 1, "c": 33, "d": 100, "e": 61, "f": 60}
    toks = {k: tokens_of(n, cfg["vocab"], 10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: expected_logits(cfg, w, v) for k, v in toks.items()}
    d = Driver(cfg, w, dtype, page=16, pages=24, slots=4)
    got = {k: [] for k in toks}
    at = {k: 0 for k in toks}
    plan = [[("a", 3), ("b", 1)], [("a", 2), ("c", 20), ("d", 29)], [("a", 40), ("c", 1), ("d", 2), ("e", 17)], [("c", 1), ("d", 1), ("e", 2), ("a", 30)],
            [("c", 11), ("d", 68), ("e", 1), ("f", 2)], [("e", 41), ("f", 50)], [("f", 8)]]
    for step in plan:
        entries = [(k, toks[k][at[k]:at[k] + n]) for k, n in step]
        out = d.step(entries)
        for k, n in step:
            got[k].append(out[k]); at[k] += n
            if at[k] == lens[k]:
                d.end(k)
    assert at == lens and d.bm.free_state_slots() == 4 and d.bm.get_stats()["free_blocks"] == 24
    for k in toks:
        check(np.concatenate(got[k]), want[k], dtype, k)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(dtype):
    cfg = hybrid(); w = make_weights(cfg, seed=8)
    d = Driver(cfg, w, dtype)
    for n in (1, 2, 3, 4, 5):                                   # shorter than, as long as and longer than the convolution
        toks = tokens_of(n, cfg["vocab"], 20 + n)
        want = expected_logits(cfg, w, toks)
        check(d.run_alone(toks), want, dtype, f"{n} tokens at once")
        check(d.run_alone(toks, cuts=[1]), want, dtype, f"{n} tokens one by one")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_over_pages_and_key_tiles(dtype):
    cfg = hybrid(); w = make_weights(cfg, seed=9)
    toks = tokens_of(230, cfg["vocab"], 5)
    check(Driver(cfg, w, dtype, page=8, pages=40).run_alone(toks, cuts=[20, 1]), expected_logits(cfg, w, toks), dtype, "210 decoded tokens")


# ------------------------------------------------------------------------------------------------ one key that matters, wherever it lies
def probe_model(kind, vocab=61, width=64):
    """One layer whose query and key projections are the same matrix, scaled up, and read only the first half of the width; tokens 7 and 8 have embeddings with
    the same first half and opposite second halves (equal norms).  So the query of token 7 scores as high against a key of token 8 as against its own, while the
    two tokens' values differ.  No convolution (taps 1): a token's key does not depend on its neighbours.  Attention: a weak penalty and a low sink keep far
    keys alive; retention: decays close to 1."""
    if kind == "attention":
        cfg = make_config([attention_layer(heads=2, kv_heads=1, dim=64, vdim=64, scale=0.5, ff=None)], vocab=vocab, width=width, taps=1, residual_mult=4.0, embedding_scale=0.25)
    else:
        cfg = make_config([retention_layer(heads=2, dim=32, vdim=32, decay=[0.999, 0.9995], rot_dims=0, ff=None)], vocab=vocab, width=width, taps=1, residual_mult=4.0, embedding_scale=0.25)
    w = make_weights(cfg, seed=11)
    rng = np.random.default_rng(12)
    dk = cfg["layers"][0]["mixer"]["dim"]
    p = bf16_round(rng.standard_normal((dk, width)) * (4.0 / np.sqrt(width)))
    p[:, width // 2:] = 0.0
    w["embed"][:, :width // 2] = bf16_round(0.1 * w["embed"][:, :width // 2]); w["embed"][7, :width // 2] *= 16.0      # every other token's keys are short
    w["embed"][8, :width // 2] = w["embed"][7, :width // 2]
    w["embed"][8, width // 2:] = -w["embed"][7, width // 2:]
    H = cfg["layers"][0]["mixer"]["heads"]
    w["l0.mix.q"] = np.concatenate([p] * H, axis=0)
    w["l0.mix.k"] = np.concatenate([p] * (1 if kind == "attention" else H), axis=0)
    if kind == "attention":
        w["l0.mix.r1"] = np.full(H, 0.0625, np.float32); w["l0.mix.r2"] = np.full(H, 0.125, np.float32); w["l0.mix.sink"] = np.full(H, -2.0, np.float32)
    return cfg, w


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["attention", "retention"])
def test_one_matching_key_at_every_kind_of_place(kind, dtype):
    """The last token's query matches the key of exactly one earlier token, at a chosen distance; every other token differs from both.  With the probe model the answer at the
    last position is dominated by that one key, so a key that is lost, doubled or taken from a wrong page shows; it is checked in a prompt and decoded alone."""
    cfg, w = probe_model(kind)
    n, page = 300, 16
    probe, match = 7, 8
    others = [t for t in range(cfg["vocab"]) if t not in (probe, match)]
    rng = np.random.default_rng(13)
    d = Driver(cfg, w, dtype, page=page, pages=80)
    for back in (1, 2, 15, 16, 17, 63, 64, 65, 127, 128, 129, 250, 299):
        toks = [others[i] for i in rng.integers(0, len(others), n)]
        toks[n - 1] = probe; toks[n - 1 - back] = match
        want = expected_logits(cfg, w, toks)
        lost = list(toks); lost[n - 1 - back] = others[0]
        assert row_errors(expected_logits(cfg, w, lost)[-1:], want[-1:]).max() > 5 * TOL[dtype], "the probe does not matter enough to test anything"
        check(d.run_alone(toks)[-1:], want[-1:], dtype, f"{kind}: key {back} back, in a prompt")
        check(d.run_alone(toks, cuts=[n - 1, 1])[-1:], want[-1:], dtype, f"{kind}: key {back} back, decoded")
        check(d.run_alone(toks, cuts=[c for c in (n - 1 - back, back - 1, 2) if c > 0] if back > 1 else [n - 2, 2])[-1:], want[-1:], dtype, f"{kind}: key {back} back, at the end of a portion")


# ------------------------------------------------------------------------------------------------ sizes the matrix-core kernels do not take
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_odd_sizes(dtype):
    layers = [attention_layer(heads=3, kv_heads=1, dim=24, vdim=20, ff=36), retention_layer(heads=1, dim=40, vdim=24, rot_dims=10, ff=52),
              attention_layer(heads=5, kv_heads=5, dim=16, vdim=48, ff=None)]
    cfg = make_config(layers, vocab=67, width=72, taps=2)
    w = make_weights(cfg, seed=14)
    toks = tokens_of(80, cfg["vocab"], 6)
    want = expected_logits(cfg, w, toks)
    d = Driver(cfg, w, dtype, page=4, pages=64)
    check(d.run_alone(toks), want, dtype, "whole")
    check(d.run_alone(toks, cuts=[9, 2, 30, 1]), want, dtype, "portions")


def test_wide_heads_of_the_largest_size_class():
    cfg = make_config([attention_layer(heads=4, kv_heads=2, dim=160, vdim=256, ff=None), retention_layer(heads=2, dim=256, vdim=64, ff=None)], width=128)
    w = make_weights(cfg, seed=15)
    toks = tokens_of(140, cfg["vocab"], 7)
    want = expected_logits(cfg, w, toks)
    for dtype in ("float32", "bfloat16"):
        check(Driver(cfg, w, dtype).run_alone(toks, cuts=[100, 3, 1]), want, dtype, dtype)


# ------------------------------------------------------------------------------------------------ designs and schedules drawn at random
def random_design(rng):
    layers = []
    for _ in range(int(rng.integers(1, 5))):
        ff = None if rng.random() < 0.25 else int(rng.choice([24, 40, 64, 96]))
        if rng.random() < 0.55:
            heads = int(rng.choice([1, 2, 3, 4, 6, 8]))
            kv = int(rng.choice([d for d in range(1, heads + 1) if heads % d == 0]))
            dim = int(rng.choice([16, 32, 64, 128]))
            vdim = dim if rng.random() < 0.6 else int(rng.choice([16, 32, 48, 64]))
            layers.append(attention_layer(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=float(rng.uniform(0.5, 1.5)) * dim ** -0.5, ff=ff, limit=float(rng.uniform(0.5, 3.0))))
        else:
            heads = int(rng.choice([1, 2, 3, 4]))
            dim = int(rng.choice([16, 32, 64, 128]))
            layers.append(retention_layer(heads=heads, dim=dim, vdim=int(rng.choice([8, 16, 32, 64, 96])), decay=[float(x) for x in rng.uniform(0.9, 0.9995, heads)],
                                          rot_dims=int(rng.choice([0, dim // 2, dim])), base=float(rng.choice([100.0, 10000.0, 1e6])), ff=ff, limit=float(rng.uniform(0.5, 3.0))))
    n = len(layers)
    loop = None
    if rng.random() < 0.6:
        a = int(rng.integers(0, n)); b = int(rng.integers(a + 1, n + 1))
        loop = (a, b, int(rng.integers(1, 4)))
    return make_config(layers, vocab=int(rng.choice([50, 97, 128, 211])), width=int(rng.choice([64, 96, 128, 256])), taps=int(rng.integers(1, 6)), loop=loop,
                       residual_mult=float(rng.uniform(0.3, 1.0)), embedding_scale=float(rng.uniform(0.3, 1.5)), eps=float(rng.choice([1e-6, 1e-5, 1e-3])))


@pytest.mark.parametrize("seed", range(12))
def test_random_design_and_schedule(seed):
    """A design drawn at random (layer order, head counts, sizes, taps, loop, constants) under a schedule drawn at random: up to four live requests, portions of
    1 .. 70 tokens, requests that skip steps, pages of 8 or 16 or 64 tokens in a pool that only fits the live ones; float32 and bfloat16 against the restatement."""
    rng = np.random.default_rng(1000 + seed)
    cfg = random_design(rng)
    w = make_weights(cfg, seed=seed)
    lens = [int(x) for x in rng.integers(1, 160, 6)]
    toks = {i: tokens_of(n, cfg["vocab"], 50 + i) for i, n in enumerate(lens)}
    want = {i: expected_logits(cfg, w, t) for i, t in toks.items()}
    page = int(rng.choice([8, 16, 64]))
    plan, at, live, nxt = [], {}, [], 0
    prng = np.random.default_rng(2000 + seed)
    while nxt < len(lens) or live:
        while len(live) < 4 and nxt < len(lens) and (not live or prng.random() < 0.6):
            live.append(nxt); at[nxt] = 0; nxt += 1
        step = []
        for i in list(live):
            if len(live) > 1 and prng.random() < 0.25:
                continue                                                 # left out of this step
            n = min(int(prng.choice([1, 1, 2, 3, 7, 16, 33, 70])), lens[i] - at[i])
            step.append((i, at[i], n)); at[i] += n
            if at[i] == lens[i]:
                live.remove(i)
        if step:
            plan.append(step)
    pages = sum((n + page - 1) // page for n in sorted(lens)[-4:]) + 1
    for dtype in ("float32", "bfloat16"):
        d = Driver(cfg, w, dtype, page=page, pages=pages, slots=4, max_tokens=4 * 70 + 8, max_len=max(lens) + 1)
        got = {i: [] for i in toks}
        done = {i: 0 for i in toks}
        for step in plan:
            out = d.step([(str(i), toks[i][a:a + n]) for i, a, n in step])
            for i, a, n in step:
                got[i].append(out[str(i)]); done[i] += n
                if done[i] == lens[i]:
                    d.end(str(i))
        for i in toks:
            what = f"seed {seed}, request {i} ({dtype}): {cfg['layers']}"
            if dtype == "float32":
                check(np.concatenate(got[i]), want[i], dtype, what)
                continue
            # bfloat16: the first rows of a retention layer normalise a sum of one to four terms; where such a sum nearly cancels, rounding q and k to 16 bits
            # decides its sign (a numpy pipeline with the same roundings shows the same).  float32 above pins those rows; here they are left out of the bound
            e = row_errors(np.concatenate(got[i]), want[i])
            assert e[4:].max(initial=0.0) < 2 * TOL[dtype] and (e[4:] > TOL[dtype]).sum() <= 0.05 * len(e), f"{what}: row {int(e.argmax())} differs by {e.max():.3g}"


# ------------------------------------------------------------------------------------------------ the engine's own entry point
@pytest.mark.parametrize("chunked", [0, 1])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_scheduler(dtype, chunked):
    """Six requests through LLMEngine.add_request / step with three state slots and a token budget that cuts prompts (chunked) or batches them whole: every
    generated token is the arg-max of the reference's logits for the sequence so far (or as good as, where two logits are closer than the tolerance)."""
    nvr = nvr_import.load()
    cfg = hybrid(); w = make_weights(cfg, seed=16)
    eng = nvr.LLMEngine(nvr.Config(dtype=dtype, kvcache_block_size=16, skip_block_size_check=1, num_kvcache_blocks=40, max_num_seqs=3, max_num_batched_tokens=48,
                                   max_model_len=160, enable_chunked_prefill=chunked), nvr.ModelSpec(cfg))
    for k, v in w.items():
        eng.model_runner.load_tensor(k, np.asarray(v, dtype=np.float32))
    prompts = [tokens_of(n, cfg["vocab"], 30 + i) for i, n in enumerate([5, 40, 1, 23, 47, 12])]
    ids = [eng.add_request(p, nvr.SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True)) for p in prompts]
    steps = 0
    while not eng.is_finished():
        eng.step(); steps += 1
        assert steps < 400
    done = {s.seq_id: s for s in eng.take_finished()}
    assert sorted(done) == sorted(ids)
    for sid, p in zip(ids, prompts):
        full = done[sid].token_ids
        assert full[:len(p)] == p and len(full) == len(p) + 12
        lg = expected_logits(cfg, w, full[:-1])
        for k in range(len(p) - 1, len(full) - 1):
            row = lg[k]
            spread = np.sqrt(((row - row.mean()) ** 2).mean())
            assert row.max() - row[full[k + 1]] <= 3 * TOL[dtype] * spread, f"request {sid}: token {k + 1} is not the greedy choice"
