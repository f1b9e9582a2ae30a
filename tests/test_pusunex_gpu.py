"""Pusunex on the GPU against the plain restatement of the design (tests/pusunex_reference.py): every mechanism alone, prompts against token-by-token
decoding, portions down to two tokens, unequal batches, pages and state slots that are used again, one key that stands out far back and at page
borders, the first tokens of a sequence, long decoding, sizes that are 1 or equal to each other, and greedy generation through the engine's scheduler."""
import numpy as np
import pytest

import nvr_import
import pusunex_reference as ref
from pusunex_util import (dense, expected_logits, gla_layer, latent2_layer, latent_layer, make_config, make_key_stand_out, make_weights, moe, settled_tokens)
from rugudra_util import Driver, TOL, row_errors

pytestmark = pytest.mark.gpu


def tokens_of(n, vocab, seed, lo=0):
    return np.random.default_rng(seed).integers(lo, vocab, n).tolist()


def check(got, want, dtype, what=""):
    e = row_errors(got, want)
    assert e.max() < TOL[dtype], f"{what}: row {int(e.argmax())} differs by {e.max():.3g} of the row's spread (limit {TOL[dtype]})"


# ------------------------------------------------------------------------------------------------ each mechanism alone
MECHANISMS = {
    "norm_one_group": make_config([latent_layer()], groups=1, side=0),
    "norm_groups_of_four_numbers": make_config([latent_layer()], width=96, groups=24, side=0),
    "latent_attention": make_config([latent_layer(heads=3, dim=32, vdim=16, kv_rank=48)], side=0),
    "latent_attention_one_head_rank_below_dim": make_config([latent_layer(heads=1, dim=40, vdim=72, kv_rank=24, scale=0.2)], side=0),
    "latent_attention_shared_latent": make_config([latent_layer(heads=2, dim=16, vdim=16, kv_rank=32), gla_layer(), latent_layer(heads=4, dim=24, vdim=8, kv_rank=32, kv_from=0)], side=0),
    "latent_attention_2": make_config([latent2_layer(heads=2, dim=32, rot_dim=8, vdim=24, kv_rank=40, q_rank=56)], side=0),
    "latent_attention_2_two_rotated_small_base": make_config([latent2_layer(heads=3, dim=16, rot_dim=2, vdim=16, kv_rank=16, q_rank=16, base=3.0)], side=0),
    "latent_attention_2_mostly_rotated": make_config([latent2_layer(heads=2, dim=8, rot_dim=40, vdim=32, kv_rank=72, q_rank=24, base=500000.0)], side=0),
    "latent_attention_head_size_64_as_whole_prompt": make_config([latent_layer(heads=3, dim=64, vdim=64, kv_rank=96), gla_layer(), latent_layer(heads=2, dim=64, vdim=64, kv_rank=96, kv_from=0)], side=0),
    "latent_attention_2_head_size_64_as_whole_prompt": make_config([latent2_layer(heads=2, dim=48, rot_dim=16, vdim=64, kv_rank=48, q_rank=40)], side=0),
    "latent_attention_2_head_size_128_as_whole_prompt": make_config([latent2_layer(heads=2, dim=96, rot_dim=32, vdim=128, kv_rank=96, q_rank=64)], width=128, groups=4, side=0),
    "gla": make_config([gla_layer(heads=2, dim=24, vdim=32, tau=8.0)], side=0),
    "gla_tau_one_one_head": make_config([gla_layer(heads=1, dim=64, vdim=16, tau=1.0)], side=0),
    "gla_keys_of_256": make_config([gla_layer(heads=1, dim=256, vdim=24, tau=4.0)], side=0),
    "gla_wide_keys": make_config([gla_layer(heads=1, dim=272, vdim=40, tau=16.0)], side=0),
    "dense_feed_forward": make_config([latent_layer(mlp=dense(80))], side=0),
    "experts_top_two_with_shared": make_config([latent_layer(mlp=moe(6, 2, 24, 40))], side=0),
    "experts_top_one_no_shared": make_config([gla_layer(mlp=moe(5, 1, 32, 0))], side=0),
    "experts_all_chosen_and_a_single_expert": make_config([latent_layer(mlp=moe(3, 3, 16, 16)), latent_layer(mlp=moe(1, 1, 16, 0))], side=0),
    "many_experts": make_config([latent_layer(mlp=moe(70, 3, 8, 8))], side=0),
    "token_input": make_config([latent_layer(), gla_layer()], side=8),
    "token_input_of_one_number": make_config([latent_layer(mlp=dense(32)), latent_layer()], side=1),
    "depth_average_over_five_layers": make_config([latent_layer(), gla_layer(), latent2_layer(), gla_layer(mlp=dense(40)), latent_layer(kv_from=0)], side=4),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(name, dtype):
    if name == "token_input_of_one_number" and dtype == "bfloat16":
        pytest.skip("a token input of one number, divided by its own magnitude, is a sign: 16-bit arithmetic may decide it otherwise; the float32 case covers the size")
    cfg = MECHANISMS[name]
    w = make_weights(cfg, seed=len(name))
    toks = settled_tokens(cfg, w, 70, 1)
    d = Driver(cfg, w, dtype)
    check(d.run_alone(toks), expected_logits(cfg, w, toks), dtype, name)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_products_per_head_and_per_expert_with_many_rows(dtype):
    """A prompt long enough for the large tiles of the per-head and per-expert products (128 rows and more per head, about a hundred per expert), in one
    step and in two uneven ones."""
    cfg = make_config([latent_layer(heads=2, dim=32, vdim=24, kv_rank=40, mlp=moe(3, 2, 40, 24)), latent2_layer(mlp=moe(2, 1, 24, 0))], side=4)
    w = make_weights(cfg, seed=21)
    toks = settled_tokens(cfg, w, 300, 22)
    want = expected_logits(cfg, w, toks)
    check(Driver(cfg, w, dtype, page=16, pages=40, max_tokens=512).run_alone(toks), want, dtype, "one step")
    check(Driver(cfg, w, dtype, page=16, pages=40, max_tokens=512).run_alone(toks, cuts=[171, 129]), want, dtype, "two steps")


def test_experts_over_whole_row_blocks():
    """A step of more than two thousand expert rows at sizes the 256 x 256 product takes: the experts' rows are padded to whole blocks, gathered, and multiplied with
    one matrix per block.  The same prompt in portions below that size takes the small tiles; both must agree with the restatement."""
    cfg = make_config([latent_layer(heads=2, dim=32, vdim=32, kv_rank=64, mlp=moe(3, 2, 128, 128))], vocab=67, width=256, groups=4, side=0)
    w = make_weights(cfg, seed=23)
    toks = settled_tokens(cfg, w, 1100, 24)
    want = expected_logits(cfg, w, toks)
    check(Driver(cfg, w, "bfloat16", page=16, pages=80, max_tokens=1280, max_len=1280).run_alone(toks), want, "bfloat16", "one step")
    check(Driver(cfg, w, "bfloat16", page=16, pages=80, max_tokens=1280, max_len=1280).run_alone(toks, cuts=[400]), want, "bfloat16", "portions of 400")


def test_each_part_changes_the_result():
    """A part that is left out must show: with the output gate's, the decay's, the token input's or the depth average's weights changed the restatement's
    logits move by far more than the tolerance, and the engine follows each variant."""
    cfg = make_config([latent_layer(mlp=moe(4, 1, 16, 16)), gla_layer(mlp=dense(48))], side=4)
    w = make_weights(cfg, seed=11)
    toks = tokens_of(40, cfg["vocab"], 4)
    full = expected_logits(cfg, w, toks)
    check(Driver(cfg, w, "float32").run_alone(toks), full, "float32", "full")
    for key, val in (("l0.mix.g", 0.0), ("l1.mix.a2.b", -1.0), ("l1.side.norm", 0.0), ("l1.dwa", 0.5), ("l0.mlp.act" if False else "l1.mlp.act", 0.25), ("l0.mix.dkv.norm", 0.3)):
        w2 = dict(w); w2[key] = np.full_like(w[key], val)
        want = expected_logits(cfg, w2, toks)
        assert row_errors(want, full).max() > 50 * TOL["float32"], key
        check(Driver(cfg, w2, "float32").run_alone(toks), want, "float32", key)


# ------------------------------------------------------------------------------------------------ a model with everything, in portions and batches
def everything(vocab=113, width=96):
    layers = [latent_layer(heads=4, dim=32, vdim=32, kv_rank=64, mlp=dense(72)),
              latent_layer(heads=2, dim=48, vdim=16, kv_rank=64, kv_from=0, mlp=moe(6, 2, 24, 40)),
              gla_layer(heads=3, dim=16, vdim=32, tau=12.0, mlp=None),
              latent2_layer(heads=3, dim=16, rot_dim=16, vdim=40, kv_rank=48, q_rank=32, mlp=moe(4, 1, 32, 0))]
    return make_config(layers, vocab=vocab, width=width, groups=4, side=6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_against_token_by_token_decoding(dtype):
    cfg = everything(); w = make_weights(cfg, seed=5)
    toks = settled_tokens(cfg, w, 60, 3)
    want = expected_logits(cfg, w, toks)
    check(Driver(cfg, w, dtype).run_alone(toks), want, dtype, "whole prompt")
    check(Driver(cfg, w, dtype, page=8).run_alone(toks, cuts=[1]), want, dtype, "token by token")
    check(Driver(cfg, w, dtype, page=8).run_alone(toks, cuts=[37, 1]), want, dtype, "a prompt, then token by token")


@pytest.mark.parametrize("cuts", [[2], [3, 2, 17, 2, 5], [16], [15, 17], [33, 2, 1], [64, 7]])
def test_portions(cuts):
    cfg = everything(); w = make_weights(cfg, seed=6)
    toks = tokens_of(85, cfg["vocab"], 7)
    check(Driver(cfg, w, "float32", page=16).run_alone(toks, cuts=cuts), expected_logits(cfg, w, toks), "float32", f"portions {cuts}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_with_pages_and_slots_used_again(dtype):
    """Five requests of different lengths through three state slots and a pool of pages that cannot hold them all at once: portions of some beside single
    tokens of others; a finished request's pages and slot go to the next one.  Every request must come out as it does alone."""
    cfg = everything(); w = make_weights(cfg, seed=8)
    reqs = {n: settled_tokens(cfg, w, ln, 20 + k) for k, (n, ln) in enumerate([("a", 61), ("b", 9), ("c", 34), ("d", 47), ("e", 2)])}
    want = {n: expected_logits(cfg, w, t) for n, t in reqs.items()}
    d = Driver(cfg, w, dtype, page=8, pages=20, slots=3, max_tokens=256)
    at = {n: 0 for n in reqs}
    got = {n: [] for n in reqs}
    waiting, live = ["a", "b", "c", "d", "e"], []
    sizes, k = [5, 1, 2, 11, 1, 1, 3, 8, 1, 2], 0
    while waiting or live:
        while waiting and len(live) < 3 and sum((len(reqs[n]) + 7) // 8 for n in live + waiting[:1]) <= 20:
            live.append(waiting.pop(0))
        entries = []
        for n in live:
            c = min(sizes[k % len(sizes)], len(reqs[n]) - at[n]); k += 1
            entries.append((n, reqs[n][at[n]:at[n] + c]))
            at[n] += c
        out = d.step(entries)
        for n, _ in entries:
            got[n].append(out[n])
        for n in [n for n in live if at[n] == len(reqs[n])]:
            d.end(n); live.remove(n)
    for n in reqs:
        check(np.concatenate(got[n]), want[n], dtype, f"request {n}")


# ------------------------------------------------------------------------------------------------ one key that stands out
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["latent", "latent2", "latent_64", "latent2_64"])
@pytest.mark.parametrize("back", [0, 1, 7, 8, 9, 15, 16, 17, 63, 64, 65, 128, 331])
def test_one_key_stands_out(kind, back, dtype):
    """Token K occurs once, `back` positions before the last token Q, whose queries point at K's keys: the last row's logits are decided by that one key among
    hundreds (8-token pages: distances around page borders and far back).  The restatement without that key differs widely; the engine must agree with
    the restatement as a whole prompt, with the last token decoded alone, and with the last token ending a short portion."""
    first = {"latent": latent_layer(heads=2, dim=32, vdim=32, kv_rank=48), "latent2": latent2_layer(heads=2, dim=32, rot_dim=8, vdim=32, kv_rank=48, q_rank=40),
             "latent_64": latent_layer(heads=2, dim=64, vdim=64, kv_rank=64), "latent2_64": latent2_layer(heads=2, dim=48, rot_dim=16, vdim=64, kv_rank=48, q_rank=40)}[kind]
    if kind.endswith("_64") and back not in (0, 8, 63, 64, 65, 331):
        pytest.skip("the head size of 64 repeats the distances at the borders only")
    cfg = make_config([first, gla_layer()], vocab=61, side=4)
    Q, K, n = 0, 1, 340
    w = make_key_stand_out(cfg, make_weights(cfg, seed=9), Q, K)
    toks = tokens_of(n, cfg["vocab"], 10 + back, lo=2)
    toks[-1] = Q
    if back:
        toks[n - 1 - back] = K
    want = expected_logits(cfg, w, toks)
    if back:
        gone = list(toks); gone[n - 1 - back] = 2
        assert row_errors(expected_logits(cfg, w, gone)[-1:], want[-1:]).max() > 5 * TOL[dtype]
    for cuts, what in (([n], "whole"), ([n - 1, 1], "decoded"), ([n - 3, 3], "end of a portion")):
        got = Driver(cfg, w, dtype, page=8, pages=48, max_tokens=512).run_alone(toks, cuts=cuts)
        check(got[-4:], want[-4:], dtype, f"{what}, {back} back")


def test_state_reaches_far_back():
    """Gated linear attention with decays near one: the first eight tokens of 400 still move the last row; 16-token passes, state slots and single tokens agree."""
    cfg = make_config([gla_layer(heads=2, dim=16, vdim=16, tau=64.0)], vocab=41, side=0)
    w = make_weights(cfg, seed=12)
    w["l0.mix.a2.b"] = np.full_like(w["l0.mix.a2.b"], 6.0)
    toks = tokens_of(400, cfg["vocab"], 13)
    want = expected_logits(cfg, w, toks)
    other = [(t + 1) % cfg["vocab"] for t in toks[:8]] + toks[8:]
    assert row_errors(expected_logits(cfg, w, other)[-1:], want[-1:]).max() > 20 * TOL["float32"]
    for cuts in ([400], [399, 1], [17, 200, 2, 1]):
        check(Driver(cfg, w, "float32", page=16, pages=32, max_tokens=512).run_alone(toks, cuts=cuts), want, "float32", f"portions {cuts}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = everything(); w = make_weights(cfg, seed=14)
    toks = settled_tokens(cfg, w, 200, 15)
    got = Driver(cfg, w, dtype, page=8, pages=32).run_alone(toks, cuts=[10, 1])
    check(got, expected_logits(cfg, w, toks), dtype, "190 decoded tokens")


def test_decode_steps_replay_a_graph():
    """Decode-sized steps are captured the second time their shape is seen and replayed from then on; every replay is compared."""
    cfg = everything(); w = make_weights(cfg, seed=16)
    toks = tokens_of(48, cfg["vocab"], 17)
    d = Driver(cfg, w, "float32", page=8)
    got = d.run_alone(toks, cuts=[8, 1])
    check(got, expected_logits(cfg, w, toks), "float32", "replayed steps")


# ------------------------------------------------------------------------------------------------ through the engine's own entry point
@pytest.mark.parametrize("chunked", [0, 1])
def test_greedy_generation_through_the_scheduler(chunked):
    """Five requests through LLMEngine.add_request / step with three state slots and a token budget that cuts prompts (chunked) or batches them whole: every
    generated token is the arg-max of the restatement's logits for the sequence so far."""
    nvr = nvr_import.load()
    cfg = everything(); w = make_weights(cfg, seed=18)
    prompts = [settled_tokens(cfg, w, n, 30 + n) for n in (5, 23, 1, 40, 12)]
    new = 12
    eng = nvr.LLMEngine(nvr.Config(dtype="float32", kvcache_block_size=8, skip_block_size_check=1, num_kvcache_blocks=40, max_num_seqs=3, num_state_slots=3,
                                   max_num_batched_tokens=32 if chunked else 256, max_model_len=128, enable_chunked_prefill=chunked), nvr.ModelSpec(cfg))
    for k, v in w.items():
        eng.model_runner.load_tensor(k, np.asarray(v, dtype=np.float32))
    ids = [eng.add_request(p, nvr.SamplingParams(temperature=0.0, max_tokens=new, ignore_eos=True)) for p in prompts]
    steps = 0
    while not eng.is_finished():
        eng.step(); steps += 1
        assert steps < 400
    done = {s.seq_id: s for s in eng.take_finished()}
    assert sorted(done) == sorted(ids)
    for sid, p in zip(ids, prompts):
        full = done[sid].token_ids
        assert full[:len(p)] == p and len(full) == len(p) + new
        lg = expected_logits(cfg, w, full[:-1])
        for k in range(len(p) - 1, len(full) - 1):
            row = lg[k]
            spread = np.sqrt(((row - row.mean()) ** 2).mean())
            assert row.max() - row[full[k + 1]] <= 3 * TOL["float32"] * spread, f"request {sid}: token {k + 1} is not the greedy choice"


# ------------------------------------------------------------------------------------------------ designs and schedules drawn at random
def random_design(seed):
    rng = np.random.default_rng(seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    width = pick([48, 64, 96, 104, 128, 192, 256])
    groups = pick([g for g in (1, 2, 4, 8, 13) if width % g == 0])
    n_layers = int(rng.integers(1, 5))
    layers, owners = [], []

    def mlp():
        k = int(rng.integers(0, 3))
        if k == 0:
            return None
        if k == 1:
            return dense(pick([24, 40, 64, 100]))
        e = int(rng.integers(1, 10))
        return moe(e, int(rng.integers(1, min(e, 3) + 1)), pick([8, 16, 24, 40]), pick([0, 16, 24]))
    for i in range(n_layers):
        kind = pick(["latent", "latent", "latent2", "gla"])
        heads = int(rng.integers(1, 7))
        if kind == "latent":
            rank, src = pick([8, 16, 24, 32, 40, 64, 96]), None
            if owners and rng.random() < 0.5:                 # read an earlier layer's cached rows
                src = pick(owners); rank = layers[src]["mixer"]["kv_rank"]
            layers.append(latent_layer(heads=heads, dim=pick([8, 12, 16, 32, 40, 64]), vdim=pick([8, 16, 20, 32, 64]), kv_rank=rank, scale=float(rng.uniform(0.05, 0.4)),
                                       kv_from=src, mlp=mlp()))
            if src is None:
                owners.append(i)
        elif kind == "latent2":
            dim, rot = pick([(8, 8), (16, 16), (24, 8), (32, 32), (48, 16), (62, 2), (96, 32), (20, 4)])
            layers.append(latent2_layer(heads=heads, dim=dim, rot_dim=rot, vdim=pick([dim + rot, 16, 40]), kv_rank=pick([16, 24, 32, 48, 56, 96]), q_rank=pick([8, 24, 32, 72]),
                                        base=pick([10.0, 10000.0, 500000.0]), scale=float(rng.uniform(0.05, 0.3)), mlp=mlp()))
        else:
            layers.append(gla_layer(heads=heads, dim=pick([8, 16, 24, 40, 64, 128]), vdim=pick([8, 16, 32, 48]), tau=pick([1.0, 4.0, 16.0, 50.0]), mlp=mlp()))
    return make_config(layers, vocab=int(rng.integers(40, 200)), width=width, groups=groups, side=pick([0, 1, 8, 12, 16]) if width >= 64 else 0, eps=pick([1e-6, 1e-5]))


@pytest.mark.parametrize("seed", range(12))
def test_random_designs_and_schedules(seed):
    """A design drawn at random (layer order, sizes, shared latents, feed-forwards) runs a prompt whole, in random portions, and two requests of unequal length in one
    batch with their own portions, in both number formats.  (Token inputs of two to four numbers are left out: such a vector divided by its own magnitude is ill-conditioned for
    single tokens, and 16-bit products then differ from the float64 restatement by more than the bound, in every schedule alike; float32 agrees to 1e-5.)"""
    cfg = random_design(100 + seed)
    w = make_weights(cfg, seed=200 + seed, a_rank=int(np.random.default_rng(seed).integers(1, 20)))
    rng = np.random.default_rng(300 + seed)
    a, b = settled_tokens(cfg, w, int(rng.integers(20, 130)), 400 + seed), settled_tokens(cfg, w, int(rng.integers(2, 60)), 500 + seed)
    wa, wb = expected_logits(cfg, w, a), expected_logits(cfg, w, b)
    side_of_one = (cfg.get("token_side") or {}).get("dim") == 1
    for dtype in ("float32", "bfloat16"):
        if dtype == "bfloat16" and side_of_one:
            continue                                          # (a token input of one number is a sign: see test_mechanism_alone)
        check(Driver(cfg, w, dtype, page=8, pages=64).run_alone(a), wa, dtype, f"design {seed}, whole")
        cuts = [int(c) for c in rng.integers(1, 40, 12)] + [1]
        check(Driver(cfg, w, dtype, page=8, pages=64).run_alone(a, cuts=cuts), wa, dtype, f"design {seed}, portions {cuts}")
        d = Driver(cfg, w, dtype, page=8, pages=64, slots=2)
        at, got = {"a": 0, "b": 0}, {"a": [], "b": []}
        toks = {"a": a, "b": b}
        while at["a"] < len(a) or at["b"] < len(b):
            entries = []
            for n in ("a", "b"):
                if at[n] < len(toks[n]):
                    c = min(int(rng.integers(1, 24)), len(toks[n]) - at[n])
                    entries.append((n, toks[n][at[n]:at[n] + c])); at[n] += c
            out = d.step(entries)
            for n, _ in entries:
                got[n].append(out[n])
        check(np.concatenate(got["a"]), wa, dtype, f"design {seed}, batch, first request")
        check(np.concatenate(got["b"]), wb, dtype, f"design {seed}, batch, second request")
