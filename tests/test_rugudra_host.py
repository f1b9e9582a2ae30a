"""Host side of the layer-list model family, no GPU: the model registry's reading of a configuration, the block manager's state slots, and the
plain restatement's own consistency (its token-by-token forms against its whole-sequence forms)."""
import numpy as np
import pytest

import nvr_import
import rugudra_reference as ref
from rugudra_util import attention_layer, make_config, make_weights, retention_layer

nvr = nvr_import.load()


def test_registry_names_both_families():
    assert {"Qwen3ForCausalLM", "Rugudra"} <= set(nvr.registered_architectures())
    s = nvr.ModelSpec(make_config([attention_layer(), retention_layer(), attention_layer()], loop=(1, 3, 3)))
    assert (s.architecture, s.family, s.vocab_size, s.num_layer_runs) == ("Rugudra", 1, 97, 7)
    q = nvr.ModelSpec({"architectures": ["Qwen3ForCausalLM"], "vocab_size": 1000, "hidden_size": 64, "intermediate_size": 128, "num_hidden_layers": 2,
                       "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16, "rms_norm_eps": 1e-6, "rope_theta": 1e6})
    assert q.family == 0 and q.dense().c.num_key_value_heads == 2 and q.dense().c.head_dim == 16


@pytest.mark.parametrize("breakage, message", [
    (lambda c: c.pop("width"), "'width' is missing"),
    (lambda c: c["layers"][1]["mixer"].pop("decay"), "layers[1].mixer.decay"),
    (lambda c: c["layers"][0].update(type="convolution"), "layer type 'convolution'"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "heads over"),
    (lambda c: c.update(loop={"start": 2, "stop": 1, "times": 2}), "loop"),
    (lambda c: c.update(architecture="Nonesuch"), "not registered"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "even number"),
])
def test_registry_refuses_a_broken_configuration(breakage, message):
    cfg = make_config([attention_layer(), retention_layer()])
    breakage(cfg)
    with pytest.raises(nvr.NvrError, match=message.replace("[", r"\[").replace("]", r"\]")):
        nvr.ModelSpec(cfg)


def test_layer_order_with_and_without_a_loop():
    cfg = make_config([attention_layer()] * 5, loop=(1, 4, 2))
    assert ref.layer_runs(cfg) == [0, 1, 2, 3, 1, 2, 3, 4]
    assert nvr.ModelSpec(cfg).num_layer_runs == 8
    cfg.pop("loop")
    assert ref.layer_runs(cfg) == [0, 1, 2, 3, 4] and nvr.ModelSpec(cfg).num_layer_runs == 5


def test_state_slots_travel_with_the_blocks():
    bm = nvr.BlockManager(6, 4, state_slots=2)
    a, b, c = (nvr.Sequence(list(range(n)), block_size=4) for n in (5, 4, 3))
    bm.allocate(a); bm.allocate(b)
    assert (a.state_slot, b.state_slot) == (0, 1) and a.block_table == [0, 1] and b.block_table == [2]
    assert not bm.can_allocate(c)                                  # blocks are left, slots are not
    with pytest.raises(nvr.NvrError):
        bm.allocate(c)
    bm.deallocate(a)
    assert a.state_slot == -1 and bm.free_state_slots() == 1 and bm.can_allocate(c)
    bm.allocate(c)
    assert c.state_slot == 0 and c.num_cached_tokens == 0
    c.extend(list(range(10)))                                      # a portion of 10 more tokens: 13 tokens need 4 blocks
    assert bm.can_extend(c)
    bm.extend(c)
    assert len(c.block_table) == 4 and bm.get_stats()["free_blocks"] == 1
    b.extend(list(range(9)))
    assert not bm.can_extend(b)
    with pytest.raises(nvr.NvrError):
        bm.extend(b)
    bm.deallocate(b); bm.deallocate(c)
    assert bm.free_state_slots() == 2 and bm.get_stats()["free_blocks"] == 6 and bm.get_stats()["cached_blocks"] == 0


def test_equal_prompts_share_nothing_when_sequences_carry_state():
    bm = nvr.BlockManager(8, 4, state_slots=4)
    a, b = nvr.Sequence([1, 2, 3, 4, 5, 6, 7, 8], block_size=4), nvr.Sequence([1, 2, 3, 4, 5, 6, 7, 8], block_size=4)
    bm.allocate(a); bm.allocate(b)
    assert not set(a.block_table) & set(b.block_table) and b.num_cached_tokens == 0
    plain = nvr.BlockManager(8, 4)
    c, d = nvr.Sequence([1, 2, 3, 4, 5, 6, 7, 8], block_size=4), nvr.Sequence([1, 2, 3, 4, 5, 6, 7, 8], block_size=4)
    plain.allocate(c); plain.allocate(d)
    assert c.block_table == d.block_table and d.num_cached_tokens == 8 and d.state_slot == -1


def test_reference_recurrences_agree_with_their_whole_sequence_forms():
    rng = np.random.default_rng(0)
    cfg = make_config([retention_layer(heads=2, dim=16, vdim=8, rot_dims=8), attention_layer(heads=4, kv_heads=2, dim=8, vdim=8)])
    w = {k: np.asarray(v, np.float64) for k, v in make_weights(cfg).items()}
    h = rng.standard_normal((12, cfg["width"]))
    m = cfg["layers"][0]["mixer"]
    whole, _ = ref.retention_mixer(h, ref.sub(w, "l0.mix."), m, 1e-5)
    a, st = ref.retention_mixer(h[:5], ref.sub(w, "l0.mix."), m, 1e-5)
    b, _ = ref.retention_mixer(h[5:], ref.sub(w, "l0.mix."), m, 1e-5, pos0=5, state=st)
    assert np.allclose(np.concatenate([a, b]), whole, atol=1e-12)
    m = cfg["layers"][1]["mixer"]
    whole, _ = ref.sink_bias_attention_mixer(h, ref.sub(w, "l1.mix."), m)
    a, kv = ref.sink_bias_attention_mixer(h[:7], ref.sub(w, "l1.mix."), m)
    b, _ = ref.sink_bias_attention_mixer(h[7:], ref.sub(w, "l1.mix."), m, kv=kv)
    assert np.allclose(np.concatenate([a, b]), whole, atol=1e-12)
    x = rng.standard_normal((9, 5)); cw = rng.standard_normal((5, 3))
    out = ref.causal_conv_residual(x, cw)
    assert np.allclose(out[0], x[0] * (1 + cw[:, 2])) and np.allclose(out[4], x[4] + cw[:, 0] * x[2] + cw[:, 1] * x[3] + cw[:, 2] * x[4])
