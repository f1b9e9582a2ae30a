"""Plain, slow restatement of the Rugudra design in numpy float64: one function per mechanism, written from the design's
equations and sharing no code with the library.  The tests compare the library with it.

A model is (cfg, weights): cfg is the dict that config.json holds, weights maps tensor names to float arrays.
Every function works on ONE sequence from position 0; token-by-token forms (`*_step`) carry explicit state so that tests can
check a recurrence against its whole-sequence form."""
import math

import numpy as np


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose gain is one number for all coordinates."""
    return rms_unit(x, eps) * float(g)


def causal_conv_residual(h, w):
    """h + conv(h): h [T, C], w [C, taps]; conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before the start."""
    T, C = h.shape
    taps = w.shape[1]
    pad = np.concatenate([np.zeros((taps - 1, C)), h], axis=0)
    out = h.copy()
    for j in range(taps):
        out += pad[j:j + T] * w[:, j][None, :]
    return out


def rotate_half_partial(x, pos, dims, base):
    """x [T, heads, dim]: the first `dims` coordinates of every head are rotated, coordinate i paired with i + dims/2."""
    if dims == 0:
        return x
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims)
    a = pos[:, None].astype(np.float64) * f[None, :]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def silu(z):
    return z / (1.0 + np.exp(-z))


def retention_mixer(h, w, m, eps, pos0=0, state=None):
    """Linear attention with a fixed decay per head, no softmax, no denominator.  h [T, width].  Returns (out [T, width], state);
    state [heads, dim, vdim] is what a continuation from position pos0 + T starts with."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).reshape(T, H, D)
    k = (h @ w["k"].T).reshape(T, H, D)
    v = (h @ w["v"].T).reshape(T, H, Dv)
    g = h @ w["g"].T
    pos = np.arange(pos0, pos0 + T)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = rotate_half_partial(q, pos, rot["dims"], rot["base"])
    k = rotate_half_partial(k, pos, rot["dims"], rot["base"]) * D ** -0.5
    S = np.zeros((H, D, Dv)) if state is None else state.copy()
    o = np.zeros((T, H, Dv))
    decay = np.asarray(m["decay"], dtype=np.float64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    o = rms_unit(o, eps).reshape(T, H * Dv) * silu(g)
    return o @ w["o"].T, S


def sink_bias_attention_mixer(h, w, m, kv=None):
    """Causal softmax attention over grouped key/value heads with a logarithmic distance penalty and a per-head sink in the
    denominator.  kv = (K, V) of earlier positions (a continuation); returns (out, (K, V))."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).reshape(T, H, D)
    k = (h @ w["k"].T).reshape(T, G, D)
    v = (h @ w["v"].T).reshape(T, G, Dv)
    if kv is not None:
        k = np.concatenate([kv[0], k], axis=0)
        v = np.concatenate([kv[1], v], axis=0)
    n0 = k.shape[0] - T
    out = np.zeros((T, H, Dv))
    for hd in range(H):
        kvh = hd // (H // G)
        for t in range(T):
            i = n0 + t
            dist = i - np.arange(i + 1)
            s = (k[:i + 1, kvh] @ q[t, hd]) * m["scale"] - w["r1"][hd] * np.log1p(w["r2"][hd] * dist)
            mx = max(s.max(), w["sink"][hd])
            e = np.exp(s - mx)
            out[t, hd] = (e @ v[:i + 1, kvh]) / (e.sum() + math.exp(w["sink"][hd] - mx))
    return out.reshape(T, H * Dv) @ w["o"].T, (k, v)


def clamped_gated_mlp(h, w, m):
    """g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); W_down (g * sigmoid(1.702 g) * (u + 1))."""
    lim = m["limit"]
    g = np.minimum(h @ w["gate"].T, lim)
    u = np.clip(h @ w["up"].T, -lim, lim)
    return (g / (1.0 + np.exp(-1.702 * g)) * (u + 1.0)) @ w["down"].T


def layer_runs(cfg):
    """The order in which layers run: indices start .. stop-1 are repeated `times` times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, t = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * t + list(range(b, n))


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence (float64), optionally also the residual stream after every layer run."""
    eps = cfg["norm"]["eps"]
    taps = cfg["canon"]["taps"]
    mult = cfg["residual_mult"]
    x = weights["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    trace = []
    for li in layer_runs(cfg):
        L = cfg["layers"][li]
        p = "l%d." % li
        h1 = causal_conv_residual(scalar_norm(x, weights[p + "norm1"], eps), weights[p + "canon1"]) if taps else scalar_norm(x, weights[p + "norm1"], eps)
        if L["type"] == "retention":
            y, _ = retention_mixer(h1, sub(weights, p + "mix."), L["mixer"], eps)
        elif L["type"] == "attention":
            y, _ = sink_bias_attention_mixer(h1, sub(weights, p + "mix."), L["mixer"])
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            h2 = causal_conv_residual(scalar_norm(x, weights[p + "norm2"], eps), weights[p + "canon2"])
            y = y + clamped_gated_mlp(h2, sub(weights, p + "mlp."), L["mlp"])
        x = x + mult * y
        trace.append(x.copy())
    logits = scalar_norm(x, weights["final.norm"], eps) @ weights["head"].T
    return (logits, np.stack(trace)) if return_layers else logits
