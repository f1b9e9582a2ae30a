"""Helpers of the Pusunex tests: small configurations and random weights by the checkpoint's tensor names, and a way to make ONE key stand out for
one query (so that a lost key, a wrong page or a stale row shows in the logits).  The expected values come from tests/pusunex_reference.py; the
engine is driven by rugudra_util.Driver (requests in arbitrary portions and batches, pages and state slots from the engine's block manager)."""
import numpy as np

import pusunex_reference as ref
from rugudra_util import bf16_round


def latent_layer(heads=3, dim=32, vdim=16, kv_rank=48, scale=None, kv_from=None, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale if scale is not None else dim ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def latent2_layer(heads=2, dim=32, rot_dim=8, vdim=24, kv_rank=40, q_rank=56, base=10000.0, scale=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "rot": {"dims": rot_dim, "base": base},
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    return {"type": "latent_attention_2", "mixer": m, "mlp": mlp}


def gla_layer(heads=2, dim=24, vdim=32, tau=8.0, mlp=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": mlp}


def dense(ff=80):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=24, shared=40):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def make_config(layers, vocab=89, width=96, groups=3, side=8, eps=1e-5):
    cfg = {"architecture": "Pusunex", "vocab": vocab, "width": width, "norm": {"eps": eps, "groups": groups}, "layers": layers}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


ROUTED = 8      # the routers read the first channels only, where the embeddings are large: see make_weights


def make_weights(cfg, seed=0, gain=1.0, a_rank=12):
    """Random tensors by the checkpoint's names (float32 values on the bfloat16 grid).  The first ROUTED channels of the embeddings are 16 times larger than
    the rest and the routers read only these channels: a router's decision is then (nearly) a property of the token, the noise of 16-bit arithmetic in
    the layers before it hardly reaches its logits, and tokens can be drawn so that no decision is a close call (settled_tokens)."""
    rng = np.random.default_rng(seed)
    W, V, nL = cfg["width"], cfg["vocab"], len(cfg["layers"])
    side = (cfg.get("token_side") or {}).get("dim", 0)

    def lin(o, i, g=1.0):
        return bf16_round(rng.standard_normal((o, i)) * (g / np.sqrt(i)))

    def gains(n):
        return bf16_round(1.0 + 0.2 * rng.standard_normal(n))
    emb = rng.standard_normal((V, W))
    emb[:, :ROUTED] *= 16.0
    w = {"embed": bf16_round(emb), "head": lin(V, W), "final.norm": gains(W)}
    if side:
        w["side.embed"] = bf16_round(rng.standard_normal((V, nL * side)))
    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], "l%d." % i
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        w[p + "norm1"], w[p + "norm1b"] = gains(W), gains(W)
        if L["type"] == "latent_attention":
            rank = m["kv_rank"]
            w[p + "mix.q"] = lin(H * D, W, gain)
            if m.get("kv_from") is None:
                w[p + "mix.dkv"], w[p + "mix.dkv.norm"] = lin(rank, W), gains(rank)
            w[p + "mix.uk"], w[p + "mix.uv"] = lin(H * D, rank, gain), lin(H * Dv, rank)
            w[p + "mix.g"] = lin(H * Dv, W)
        elif L["type"] == "latent_attention_2":
            rank, R, qr = m["kv_rank"], m["rot_dim"], m["q_rank"]
            w[p + "mix.dq"], w[p + "mix.dq.norm"], w[p + "mix.uq"] = lin(qr, W), gains(qr), lin(H * (D + R), qr, gain)
            w[p + "mix.dkv"], w[p + "mix.dkv.norm"] = lin(rank + R, W), gains(rank)
            w[p + "mix.uk"], w[p + "mix.uv"] = lin(H * D, rank, gain), lin(H * Dv, rank)
        else:
            w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"], w[p + "mix.g"] = lin(H * D, W), lin(H * D, W), lin(H * Dv, W), lin(H * Dv, W)
            w[p + "mix.norm"] = gains(Dv)
            w[p + "mix.a1"], w[p + "mix.a2"] = lin(a_rank, W), lin(H * D, a_rank, 2.0)
            w[p + "mix.a2.b"] = bf16_round(2.0 + rng.standard_normal(H * D))
        w[p + "mix.o"] = lin(W, H * Dv)
        mlp = L.get("mlp")
        if mlp:
            w[p + "norm2"], w[p + "norm2b"] = gains(W), gains(W)
            if mlp["kind"] == "dense":
                w[p + "mlp.up"], w[p + "mlp.down"] = lin(mlp["ff"], W), lin(W, mlp["ff"])
                w[p + "mlp.act"] = bf16_round(np.array([0.7, 0.4, -0.3, 0.1]) + 0.1 * rng.standard_normal(4))
            else:
                f = mlp["expert"]["ff"]
                rt = np.zeros((mlp["router"]["experts"], W))
                rt[:, :ROUTED] = rng.standard_normal((mlp["router"]["experts"], ROUTED)) * 1.5
                w[p + "mlp.router"] = bf16_round(rt)
                names = ["e%d" % e for e in range(mlp["router"]["experts"])] + (["shared"] if mlp.get("shared") else [])
                for n in names:
                    fe = mlp["shared"]["ff"] if n == "shared" else f
                    w[p + "mlp.%s.gate" % n], w[p + "mlp.%s.up" % n], w[p + "mlp.%s.down" % n] = lin(fe, W, 1.5), lin(fe, W, 1.5), lin(W, fe)
        if side:
            w[p + "side.gate"], w[p + "side.proj"], w[p + "side.norm"] = lin(side, W), lin(W, side), bf16_round(0.3 * gains(W))
        w[p + "dwa"] = bf16_round(np.concatenate([0.15 * rng.standard_normal(i + 1), [1.0]]))
    return w


def make_key_stand_out(cfg, w, qtok, ktok, amount=14.0):
    """Layer 0 (a latent-attention layer of either kind): the queries of token qtok are turned towards the unrotated keys of token ktok, so that this
    pair's score exceeds the others by about `amount` in every head.  Layer 0 sees the embeddings only, so the pair is a property of the two tokens."""
    L, m, eps, groups = cfg["layers"][0], cfg["layers"][0]["mixer"], cfg["norm"]["eps"], cfg["norm"]["groups"]
    H, D, rank = m["heads"], m["dim"], m["kv_rank"]
    w64 = {k: np.asarray(v, np.float64) for k, v in w.items()}
    h = ref.group_norm(w64["embed"][[qtok, ktok]], w64["l0.norm1"], groups, eps)
    c = ref.rms((h[1:] @ w64["l0.mix.dkv"].T)[:, :rank], eps) * w64["l0.mix.dkv.norm"]
    k = (c @ w64["l0.mix.uk"].T).reshape(H, D)
    if L["type"] == "latent_attention":
        src, name, rows = h[0], "l0.mix.q", lambda hd: slice(hd * D, (hd + 1) * D)
    else:
        R = m["rot_dim"]
        src, name, rows = (ref.rms(h[:1] @ w64["l0.mix.dq"].T, eps) * w64["l0.mix.dq.norm"])[0], "l0.mix.uq", lambda hd: slice(hd * (D + R), hd * (D + R) + D)
    wq = w64[name].copy()
    for hd in range(H):
        lam = amount / (m["scale"] * (k[hd] @ k[hd]))
        wq[rows(hd)] += lam * np.outer(k[hd], src) / (src @ src)
    out = dict(w)
    out[name] = bf16_round(wq)
    return out


def expected_logits(cfg, weights, tokens):
    return ref.forward(cfg, weights, list(tokens))


def settled_tokens(cfg, w, n, seed, gap=0.05):
    """n random tokens for which every router decision of the restatement has a gap of at least `gap` between the last chosen and the first rejected logit (a
    bfloat16 engine may otherwise choose another expert than the float64 restatement: no comparison should rest on such a call)."""
    V = cfg["vocab"]
    m = []
    ref.forward(cfg, w, list(range(V)), margins=m)
    ok = np.arange(V) if not m else np.flatnonzero(np.asarray(m).reshape(-1, V).min(axis=0) > 2 * gap)
    assert len(ok) >= V // 4, "too few tokens with settled router decisions"
    for k in range(100):
        toks, m = ok[np.random.default_rng(seed + 1000 * k).integers(0, len(ok), n)].tolist(), []
        ref.forward(cfg, w, toks, margins=m)
        if not m or min(m) > gap:
            return toks
    raise AssertionError("no token sequence with settled router decisions")
