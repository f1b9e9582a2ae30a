"""A plain restatement of the Pusunex design in numpy float64, one function per mechanism, written from the design's equations.  It shares no
code with the library: the GPU tests compare the engine against it.

Notation.  x [T, W] is the residual stream of ONE sequence (positions 0 .. T-1), `cfg` the configuration (the dict of config.json), `wt` a dict
name -> array with the checkpoint's tensor names.  Linear weights are [out, in].

  layer i:   x <- x + n1b(mixer(n1(x)));  x <- x + n2b(ff(n2(x)));  x <- x + side(x, token);  X_(i+1) = x;  x <- sum_j dwa[j] X_j
  n(v)   =   w * v / sqrt(mean_g(v^2) + eps) with the mean taken inside each of `groups` equal consecutive parts
"""
import math

import numpy as np


def rms(v, eps):
    return v / np.sqrt((v * v).mean(axis=-1, keepdims=True) + eps)


def group_norm(v, w, groups, eps):
    T, W = v.shape
    u = v.reshape(T, groups, W // groups)
    return (u / np.sqrt((u * u).mean(axis=-1, keepdims=True) + eps)).reshape(T, W) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def causal_softmax(s):
    """s [T, T] scores; row i sees columns j <= i."""
    T = s.shape[0]
    s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
    s = s - s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    return p / p.sum(axis=-1, keepdims=True)


def rotate_pairs(v, pos, dims, base):
    """v [T, ..., n]: coordinates (2i, 2i+1), i < dims/2, turn by the angle pos * base^(-2i/dims); the rest passes."""
    out = v.copy()
    for i in range(dims // 2):
        a = pos * base ** (-2.0 * i / dims)
        a = a.reshape((-1,) + (1,) * (v.ndim - 2))
        c, s = np.cos(a), np.sin(a)
        u, w = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = u * c - w * s
        out[..., 2 * i + 1] = w * c + u * s
    return out


def latent_attention(h, m, wt, p, eps, latents):
    """Keys and values are expanded from a normed latent c (kv_rank numbers per position); a layer with 'kv_from' reads another layer's latent.
    Output gate sigmoid(W_g h) on the concatenated heads.  No positions."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ wt[p + "q"].T).reshape(T, H, D)
    if m.get("kv_from") is not None:
        c = latents[m["kv_from"]]
    else:
        c = rms(h @ wt[p + "dkv"].T, eps) * wt[p + "dkv.norm"]
    k = (c @ wt[p + "uk"].T).reshape(T, H, D)
    v = (c @ wt[p + "uv"].T).reshape(T, H, Dv)
    o = np.zeros((T, H, Dv))
    for hd in range(H):
        o[:, hd] = causal_softmax(q[:, hd] @ k[:, hd].T * m["scale"]) @ v[:, hd]
    o = o.reshape(T, H * Dv) * sigmoid(h @ wt[p + "g"].T)
    return o @ wt[p + "o"].T, c


def latent_attention_2(h, m, wt, p, eps):
    """Queries through a normed latent; per head `dim` unrotated coordinates against keys expanded from the latent c plus `rot_dim` rotated ones
    against one rotated key part shared by the heads."""
    T = h.shape[0]
    H, D, R, Dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = np.arange(T, dtype=np.float64)
    cq = rms(h @ wt[p + "dq"].T, eps) * wt[p + "dq.norm"]
    q = (cq @ wt[p + "uq"].T).reshape(T, H, D + R)
    qn, qr = q[..., :D], rotate_pairs(q[..., D:], pos, m["rot"]["dims"], m["rot"]["base"])
    d = h @ wt[p + "dkv"].T
    c = rms(d[:, :rank], eps) * wt[p + "dkv.norm"]
    kr = rotate_pairs(d[:, rank:], pos, m["rot"]["dims"], m["rot"]["base"])
    k = (c @ wt[p + "uk"].T).reshape(T, H, D)
    v = (c @ wt[p + "uv"].T).reshape(T, H, Dv)
    o = np.zeros((T, H, Dv))
    for hd in range(H):
        s = (qn[:, hd] @ k[:, hd].T + qr[:, hd] @ kr.T) * m["scale"]
        o[:, hd] = causal_softmax(s) @ v[:, hd]
    return o.reshape(T, H * Dv) @ wt[p + "o"].T


def gla(h, m, wt, p, eps, state=None):
    """S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head, alpha = sigmoid(z)^(1/tau) per key channel."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ wt[p + "q"].T).reshape(T, H, D) * D ** -0.5
    k = (h @ wt[p + "k"].T).reshape(T, H, D)
    v = (h @ wt[p + "v"].T).reshape(T, H, Dv)
    z = (h @ wt[p + "a1"].T) @ wt[p + "a2"].T + wt[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).reshape(T, H, D)
    S = np.zeros((H, D, Dv)) if state is None else state
    o = np.zeros((T, H, Dv))
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    o = rms(o, eps) * wt[p + "norm"]
    return (o.reshape(T, H * Dv) * silu(h @ wt[p + "g"].T)) @ wt[p + "o"].T, S


def poly_ff(h, wt, p, eps):
    """W_down (a N(z) + b N(z^2) + c N(z^3) + e), z = W_up h, N = division by the root mean square over the ff values of a token."""
    z = h @ wt[p + "up"].T
    a, b, c, e = wt[p + "act"]
    return (a * rms(z, eps) + b * rms(z * z, eps) + c * rms(z ** 3, eps) + e) @ wt[p + "down"].T


def gated_expert(h, wt, p):
    return (silu(h @ wt[p + "gate"].T) * (h @ wt[p + "up"].T)) @ wt[p + "down"].T


def moe_ff(h, mlp, wt, p, margins=None):
    """Sigmoid scores, the `top` largest chosen, the score scales the expert's INPUT; a shared expert for every token.  margins (a list) receives, per
    token, the gap between the last chosen and the first rejected router logit."""
    top = mlp["router"]["top"]
    z = h @ wt[p + "router"].T
    s = sigmoid(z)
    out = np.zeros((h.shape[0], wt[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        if margins is not None and top < z.shape[1]:
            zs = np.sort(z[t])[::-1]
            margins.append(zs[top - 1] - zs[top])
        for e in np.argsort(-s[t], kind="stable")[:top]:
            out[t] += gated_expert(s[t, e] * h[t:t + 1], wt, p + "e%d." % e)[0]
    if mlp.get("shared") is not None:
        out += gated_expert(h, wt, p + "shared.")
    return out


def token_side(x, tokens, i, dim, wt, p, side_embed, eps):
    e = side_embed[tokens][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(x @ wt[p + "gate"].T) * e) @ wt[p + "proj"].T
    return rms(y, eps) * wt[p + "norm"]


def forward(cfg, wt, tokens, layer_outputs=None, margins=None):
    """Logits [T, vocab] of one sequence; layer_outputs (a list) receives the stream that leaves every layer, margins the routers' decision gaps."""
    wt = {k: np.asarray(v, dtype=np.float64) for k, v in wt.items()}
    tokens = np.asarray(tokens)
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = wt["embed"][tokens]
    X, latents = [x], {}
    for i, L in enumerate(cfg["layers"]):
        p, m = "l%d." % i, L["mixer"]
        h = group_norm(x, wt[p + "norm1"], groups, eps)
        if L["type"] == "latent_attention":
            y, latents[i] = latent_attention(h, m, wt, p + "mix.", eps, latents)
        elif L["type"] == "latent_attention_2":
            y = latent_attention_2(h, m, wt, p + "mix.", eps)
        elif L["type"] == "gla":
            y, _ = gla(h, m, wt, p + "mix.", eps)
        else:
            raise ValueError(L["type"])
        x = x + group_norm(y, wt[p + "norm1b"], groups, eps)
        mlp = L.get("mlp")
        if mlp is not None:
            h = group_norm(x, wt[p + "norm2"], groups, eps)
            y = poly_ff(h, wt, p + "mlp.", eps) if mlp["kind"] == "dense" else moe_ff(h, mlp, wt, p + "mlp.", margins)
            x = x + group_norm(y, wt[p + "norm2b"], groups, eps)
        if cfg.get("token_side") is not None:
            x = x + token_side(x, tokens, i, cfg["token_side"]["dim"], wt, p + "side.", wt["side.embed"], eps)
        X.append(x)
        if p + "dwa" in wt:
            x = sum(wt[p + "dwa"][j] * X[j] for j in range(i + 2))
        if layer_outputs is not None:
            layer_outputs.append(x)
    return group_norm(x, wt["final.norm"], groups, eps) @ wt["head"].T
