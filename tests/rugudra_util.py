"""Helpers of the Rugudra tests: small random models, a driver that feeds requests through the engine's runner in arbitrary portions and
batches (pages and state slots from the engine's block manager), and the error measure of the comparisons.  The expected values come from
tests/rugudra_reference.py."""
import numpy as np

import nvr_import
import rugudra_reference as ref


def bf16_round(a):
    """float32 values rounded to the nearest bfloat16 (so that a bfloat16 and a float32 engine hold the same weights)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def attention_layer(heads=4, kv_heads=2, dim=32, vdim=32, scale=None, ff=48, limit=1.25):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


def retention_layer(heads=2, dim=32, vdim=16, decay=None, rot_dims=None, base=500.0, ff=48, limit=1.25):
    decay = decay if decay is not None else [1.0 - 2.0 ** (-3 - j) for j in range(heads)]
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay, "rot": {"dims": dim if rot_dims is None else rot_dims, "base": base}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff, "limit": limit}}


def make_config(layers, vocab=97, width=64, taps=3, loop=None, residual_mult=0.6, embedding_scale=0.8, eps=1e-5):
    cfg = {"architecture": "Rugudra", "vocab": vocab, "width": width, "residual_mult": residual_mult, "embedding": {"scale": embedding_scale},
           "norm": {"eps": eps}, "canon": {"taps": taps}, "layers": layers}
    if loop is not None:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed=0, gain=1.0):
    """Random tensors by the checkpoint's names (float32 on the bfloat16 grid)."""
    rng = np.random.default_rng(seed)
    W, V, taps = cfg["width"], cfg["vocab"], cfg["canon"]["taps"]

    def lin(o, i, g=1.0):
        return bf16_round(rng.standard_normal((o, i)) * (g / np.sqrt(i)))
    w = {"embed": bf16_round(rng.standard_normal((V, W))), "head": lin(V, W), "final.norm": bf16_round(np.float32(1.1))}
    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], "l%d." % i
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        G = m.get("kv_heads", H)
        w[p + "norm1"] = bf16_round(np.float32(1.0 + 0.2 * rng.standard_normal()))
        w[p + "norm2"] = bf16_round(np.float32(1.0 + 0.2 * rng.standard_normal()))
        w[p + "canon1"] = bf16_round(0.3 * rng.standard_normal((W, taps)))
        w[p + "canon2"] = bf16_round(0.3 * rng.standard_normal((W, taps)))
        w[p + "mix.q"], w[p + "mix.k"] = lin(H * D, W, gain), lin(G * D, W, gain)
        w[p + "mix.v"], w[p + "mix.o"] = lin(G * Dv, W), lin(W, H * Dv)
        if L["type"] == "retention":
            w[p + "mix.g"] = lin(H * Dv, W)
        else:
            w[p + "mix.r1"] = bf16_round(rng.uniform(0.1, 1.0, H))
            w[p + "mix.r2"] = bf16_round(rng.uniform(0.05, 0.5, H))
            w[p + "mix.sink"] = bf16_round(rng.standard_normal(H))
        if L.get("mlp"):
            F = L["mlp"]["ff"]
            w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"] = lin(F, W, 2.0), lin(F, W, 2.0), lin(W, F)
    return w


def expected_logits(cfg, weights, tokens):
    w64 = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
    return ref.forward(cfg, w64, list(tokens))


def row_errors(got, want):
    """Per row: root mean square of the difference (mean taken off) over the root mean square of the expected row (mean taken off)."""
    d = np.asarray(got, np.float64) - want
    d = d - d.mean(axis=1, keepdims=True)
    s = want - want.mean(axis=1, keepdims=True)
    return np.sqrt((d * d).mean(axis=1)) / np.sqrt((s * s).mean(axis=1))


TOL = {"float32": 2e-4, "bfloat16": 4e-2}


class Driver:
    """An engine for (cfg, weights) and a way to feed it: step(entries) runs ONE model step over [(request name, new tokens)] — the batch is the
    caller's, pages / state slots are the engine's block manager's — and returns the logits at every new token of every entry."""

    def __init__(self, cfg, weights, dtype="float32", page=16, pages=64, slots=4, max_tokens=512, max_len=512):
        self.nvr = nvr = nvr_import.load()
        self.cfg, self.page = cfg, page
        self.engine = nvr.LLMEngine(nvr.Config(dtype=dtype, kvcache_block_size=page, skip_block_size_check=1, num_kvcache_blocks=pages, max_num_seqs=slots,
                                               num_state_slots=slots, max_num_batched_tokens=max_tokens, max_model_len=max_len, enable_chunked_prefill=1),
                                    nvr.ModelSpec(cfg))
        for k, v in weights.items():
            self.engine.model_runner.load_tensor(k, np.asarray(v, dtype=np.float32))
        self.runner, self.bm = self.engine.model_runner, self.engine.scheduler.block_manager
        self.live = {}

    def step(self, entries):
        nvr, batch, rows = self.nvr, [], 0
        for name, toks in entries:
            s = self.live.get(name)
            if s is None:
                s = self.live[name] = nvr.Sequence(list(toks), nvr.SamplingParams(temperature=0.0, max_tokens=1 << 20, ignore_eos=True), block_size=self.page)
                self.bm.allocate(s)
                start = 0
            else:
                start = len(s)
                s.extend(list(toks))
                self.bm.extend(s)
            s.set_chunk(start, len(toks))
            batch.append(s)
            rows += len(toks)
        self.runner.execute_step(batch, list(range(rows)))
        lg = self.runner.logits(rows, self.cfg["vocab"])
        out, r = {}, 0
        for name, toks in entries:
            out[name] = lg[r:r + len(toks)].copy()
            r += len(toks)
        return out

    def end(self, name):
        self.bm.deallocate(self.live.pop(name))

    def run_alone(self, tokens, cuts=None, name="r"):
        """One request in portions of the given sizes (None: whole; sizes are cycled, the rest token by token when the list ends with 1)."""
        tokens, out, at, k = list(tokens), [], 0, 0
        cuts = cuts or [len(tokens)]
        while at < len(tokens):
            n = min(cuts[min(k, len(cuts) - 1)], len(tokens) - at)
            out.append(self.step([(name, tokens[at:at + n])])[name])
            at += n
            k += 1
        self.end(name)
        return np.concatenate(out, axis=0)
