"""Host side of the Pusunex design, no GPU: the model registry's reading of a configuration and its refusals, and the plain restatement's own
consistency — the forms the engine computes (keys folded into the queries, a carried recurrent state, rows grouped by expert) against the
restatement's direct forms."""
import copy

import numpy as np
import pytest

import nvr_import
import pusunex_reference as ref
from pusunex_util import dense, gla_layer, latent2_layer, latent_layer, make_config, make_weights, moe

nvr = nvr_import.load()


def small():
    return make_config([latent_layer(mlp=dense(40)), gla_layer(mlp=moe(4, 2, 16, 24)), latent_layer(kv_from=0), latent2_layer()], vocab=53, width=96, groups=4, side=5)


def test_registry_reads_the_design():
    assert "Pusunex" in nvr.registered_architectures()
    s = nvr.ModelSpec(small())
    assert (s.architecture, s.family, s.vocab_size, s.num_layer_runs) == ("Pusunex", 1, 53, 4)
    cfg = small(); cfg.pop("token_side")                           # no token input
    assert nvr.ModelSpec(cfg).num_layer_runs == 4


@pytest.mark.parametrize("breakage, message", [
    (lambda c: c.pop("width"), "'width' is missing"),
    (lambda c: c["norm"].update(groups=5), "norm.groups must divide"),
    (lambda c: c["layers"][0].update(type="attention"), "layer type 'attention'"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "must name an earlier layer"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "latent of its own"),
    (lambda c: c["layers"][2]["mixer"].update(kv_rank=32), "same kv_rank"),
    (lambda c: c["layers"][3]["mixer"]["rot"].update(dims=6), "rot.dims = rot_dim"),
    (lambda c: c["layers"][3]["mixer"].pop("q_rank"), "q_rank' is missing"),
    (lambda c: c["layers"][1]["mixer"].update(tau=0.0), "tau' must be positive"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "1 <= top <= experts"),
    (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "mlp.kind"),
    (lambda c: c["layers"][0]["mlp"].pop("ff"), "mlp.ff' is missing"),
])
def test_registry_refuses_a_broken_configuration(breakage, message):
    cfg = copy.deepcopy(small())
    breakage(cfg)
    with pytest.raises(nvr.NvrError, match=message.replace("[", r"\[").replace("]", r"\]")):
        nvr.ModelSpec(cfg)


def rand_inputs(T, W, seed):
    return np.random.default_rng(seed).standard_normal((T, W))


def test_keys_folded_into_the_queries_give_the_same_attention():
    """The engine caches the latent row only: scores are (Wuk_h^T q_h) . c (+ the rotated parts), values Wuv_h (sum_j p_j c_j)."""
    for layer in (latent_layer(heads=3, dim=16, vdim=8, kv_rank=24), latent2_layer(heads=2, dim=16, rot_dim=4, vdim=8, kv_rank=24, q_rank=20)):
        cfg = make_config([layer], width=48, groups=2, side=0)
        w = {k: np.asarray(v, np.float64) for k, v in make_weights(cfg, seed=1).items()}
        m, eps, p = layer["mixer"], cfg["norm"]["eps"], "l0.mix."
        H, D, Dv, rank, R = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m.get("rot_dim", 0)
        T = 19
        h = rand_inputs(T, 48, 2)
        pos = np.arange(T, dtype=np.float64)
        if layer["type"] == "latent_attention":
            want, _ = ref.latent_attention(h, m, w, p, eps, {})
            q = (h @ w[p + "q"].T).reshape(T, H, D)
            qr = np.zeros((T, H, 0))
            d = h @ w[p + "dkv"].T
        else:
            want = ref.latent_attention_2(h, m, w, p, eps)
            q = ((ref.rms(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]) @ w[p + "uq"].T).reshape(T, H, D + R)
            q, qr = q[..., :D], ref.rotate_pairs(q[..., D:], pos, R, m["rot"]["base"])
            d = h @ w[p + "dkv"].T
        row = np.concatenate([ref.rms(d[:, :rank], eps) * w[p + "dkv.norm"], ref.rotate_pairs(d[:, rank:], pos, R, m["rot"]["base"]) if R else d[:, rank:]], axis=1)   # the cached row
        out = np.zeros((T, H, Dv))
        for hd in range(H):
            qa = np.concatenate([q[:, hd] @ w[p + "uk"][hd * D:(hd + 1) * D], qr[:, hd]], axis=1)      # [T, rank + R]
            out[:, hd] = (ref.causal_softmax(qa @ row.T * m["scale"]) @ row[:, :rank]) @ w[p + "uv"][hd * Dv:(hd + 1) * Dv].T
        out = out.reshape(T, H * Dv)
        if layer["type"] == "latent_attention":
            out = out * ref.sigmoid(h @ w[p + "g"].T)
        assert np.allclose(out @ w[p + "o"].T, want, rtol=1e-10, atol=1e-12)


def test_recurrent_state_carries_over_a_cut():
    cfg = make_config([gla_layer(heads=2, dim=12, vdim=20, tau=5.0)], width=48, groups=2, side=0)
    w = {k: np.asarray(v, np.float64) for k, v in make_weights(cfg, seed=3).items()}
    m, eps = cfg["layers"][0]["mixer"], cfg["norm"]["eps"]
    h = rand_inputs(23, 48, 4)
    whole, S = ref.gla(h, m, w, "l0.mix.", eps)
    a, Sa = ref.gla(h[:9], m, w, "l0.mix.", eps)
    b, Sb = ref.gla(h[9:], m, w, "l0.mix.", eps, state=Sa)
    assert np.allclose(np.concatenate([a, b]), whole, rtol=1e-12, atol=1e-14) and np.allclose(S, Sb)
    # the decay is per key channel: a head's state rows shrink by different factors
    z = (h[:1] @ w["l0.mix.a1"].T) @ w["l0.mix.a2"].T + w["l0.mix.a2.b"]
    alpha = ref.sigmoid(z) ** (1.0 / m["tau"])
    assert alpha.std() > 1e-3 and (alpha > 0).all() and (alpha < 1).all()


def test_experts_grouped_by_rows_give_the_same_sum():
    """Rows sorted by expert, each expert's block multiplied at once, results added back per token: the engine's order of work."""
    mlp = moe(5, 2, 12, 16)
    cfg = make_config([latent_layer(mlp=mlp)], width=48, groups=2, side=0)
    w = {k: np.asarray(v, np.float64) for k, v in make_weights(cfg, seed=5).items()}
    h = rand_inputs(31, 48, 6)
    want = ref.moe_ff(h, mlp, w, "l0.mlp.")
    z = h @ w["l0.mlp.router"].T
    chosen = np.argsort(-z, axis=1, kind="stable")[:, :2]
    out = ref.gated_expert(h, w, "l0.mlp.shared.")
    for e in range(5):
        t, k = np.nonzero(chosen == e)
        if len(t):
            out[t] += ref.gated_expert(ref.sigmoid(z[t, e])[:, None] * h[t], w, "l0.mlp.e%d." % e)
    assert np.allclose(out, want, rtol=1e-10, atol=1e-12)
    # the weight is on the expert's INPUT: it does not factor out of a gated expert
    t = 0; e = chosen[0, 0]
    assert not np.allclose(ref.gated_expert(ref.sigmoid(z[t, e]) * h[:1], w, "l0.mlp.e%d." % e), ref.sigmoid(z[t, e]) * ref.gated_expert(h[:1], w, "l0.mlp.e%d." % e))


def test_norm_groups_and_depth_average():
    v = rand_inputs(4, 24, 7)
    w = np.linspace(0.5, 1.5, 24)
    one = ref.group_norm(v, w, 1, 1e-6)
    assert np.allclose(one, ref.rms(v, 1e-6) * w)
    three = ref.group_norm(v, w, 3, 1e-6)
    assert np.allclose(three[:, 8:16], ref.rms(v[:, 8:16], 1e-6) * w[8:16]) and not np.allclose(one, three)
    # with the depth weights (0, ..., 0, 1) every layer passes its own output on
    cfg = make_config([latent_layer(), gla_layer()], vocab=31, width=48, groups=2, side=3)
    wt = make_weights(cfg, seed=8)
    plain = dict(wt)
    for i in range(2):
        plain["l%d.dwa" % i] = np.array([0.0] * (i + 1) + [1.0])
    toks = list(range(12))
    assert not np.allclose(ref.forward(cfg, wt, toks), ref.forward(cfg, plain, toks))
    outs = []
    ref.forward(cfg, plain, toks, layer_outputs=outs)
    assert len(outs) == 2 and outs[0].shape == (12, 48)
