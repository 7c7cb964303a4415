"""CPU restatement of the reference's Qwen3 forward pass at batch 1, one token
at a time with a KV cache.  TEST INFRASTRUCTURE ONLY: tests, the smoke check
and the CPU leg of the benchmark may import this; the product never does.

Follows llvq-llm/src/model.rs:
  Rotary::new           :163-179   inverse frequencies, f32 angles, tables narrowed to the run dtype
  Block::forward_cached :766-835   ln1 -> q/k/v -> per-head q_norm/k_norm -> RoPE at the absolute
                                   position -> cache append -> grouped-query attention -> o_proj ->
                                   residual -> ln2 -> gate/up -> act(gate) * up -> down_proj -> residual
  Qwen3::hidden_cached  :968-982   embedding, blocks, final norm
  Head::project         :578-587   h E^T at the run dtype
  Qwen3::generate       :1041-1073 greedy loop; argmax of the logits widened to f32

The projections are dense matrices here (the oracle's decode_matrix output),
i.e. the reference's dense arm.  The run dtype is binary16: every tensor that
crosses an operator boundary in the reference is rounded to binary16 here too,
and each operator computes in f64 inside.

Pinned by the reference's own golden (llvq-llm/tests/kv_cache.rs:140-164): at run dtype
f32 this runner turns the tiny model's prompt [3,1,4,1,5,9,2,6] into the reference's tokens
[107,90,2,35,35,35,35,35], and exchanging k_proj and v_proj moves them
(tests/test_oracle_runner.py) — that fixes the structure: projection order, per-head norms,
the RoPE variant and its absolute positions, grouped-query attention over the cache,
residuals, the tied head and the argmax convention.

PARITY UNPINNED at run dtype binary16 in one respect: RMSNorm, rope, softmax and matmul are
candle-nn / candle-core 0.9 operators (Cargo.toml pins "0.9"; the crates are not vendored
in the reference tree), and which of their internal steps round to binary16 (e.g. the
score matrix before the softmax) is not fixed by anything the reference's own tests hold
for this path (its golden runs in f32).  This file rounds only at operator outputs that the
reference materialises as tensors of the run dtype, except inside attention, which is kept
in f64 from the scores to the context.
"""
import numpy as np


def r16(x):
    """Round to binary16 (nearest even) and widen again."""
    return np.asarray(x, dtype=np.float64).astype(np.float16).astype(np.float64)


def r32(x):
    """Round to binary32 and widen again (the run dtype of the reference's CPU tests)."""
    return np.asarray(x, dtype=np.float64).astype(np.float32).astype(np.float64)


def rope_tables(head_dim, theta, max_positions, rnd=r16):
    """model.rs:163-179: inv_i = 1f32 / (theta^(i/dim) as f32), i even; freqs = t * inv in f32;
    sin/cos in f32, then narrowed to the run dtype."""
    i = np.arange(0, head_dim, 2, dtype=np.float64)
    inv = (np.float32(1.0) / np.power(float(theta), i / float(head_dim)).astype(np.float32)).astype(np.float32)
    t = np.arange(max_positions, dtype=np.float32).reshape(-1, 1)
    freqs = (t * inv.reshape(1, -1)).astype(np.float32)
    return rnd(np.cos(freqs)), rnd(np.sin(freqs))


def rms_norm(x, w, eps, rnd=r16):
    """candle_nn::RmsNorm: x / sqrt(mean(x^2) + eps) * w, one rounding on the way out."""
    x = np.asarray(x, np.float64)
    return rnd(x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w)


KV_GROUP = 64  # kvq.rs:36


def kv_quantize(x):
    """llvq-llm/src/kvq.rs:110-165 up to the codes: per group of 64 along the last axis,
    s = f16((max - min) / 255), b = f16(min), q = clamp(round((x - b) / (s if s > 0 else 1)), 0, 255),
    every step an f32 operation as candle runs it.  Returns (q uint8, s, b) with s, b as f32 arrays
    holding binary16 values, shaped [..., groups, 1]."""
    x = np.asarray(x, np.float32)
    assert x.shape[-1] % KV_GROUP == 0, "head_dim is not a multiple of the group"
    xg = x.reshape(x.shape[:-1] + (x.shape[-1] // KV_GROUP, KV_GROUP))
    mn = xg.min(-1, keepdims=True)
    mx = xg.max(-1, keepdims=True)
    s = ((mx - mn) / np.float32(255.0)).astype(np.float16).astype(np.float32)
    b = mn.astype(np.float16).astype(np.float32)
    safe = np.where(s > 0, s, np.float32(1.0))
    t = (xg - b) / safe
    r = np.sign(t) * np.floor(np.abs(t) + np.float32(0.5))  # f32::round: half away from zero
    q = np.clip(r, 0, 255).astype(np.uint8)
    return q, s, b


def kv_dequantize(q, s, b, shape):
    """The value a reader gets back (kvq.rs:155-164): f16(q s + b); an ungraded group (s = 0) is its bias."""
    v = (q.astype(np.float32) * s).astype(np.float32) + b
    return v.astype(np.float16).astype(np.float64).reshape(shape)


def quantize_dequantize(x):
    """kvq.rs:110: what KvCache::append stores under KvMode::Q8."""
    q, s, b = kv_quantize(x)
    return kv_dequantize(q, s, b, np.shape(x))


def silu(x):
    return x / (1.0 + np.exp(-x))


class Qwen3Oracle:
    def __init__(self, cfg, dense_projections, weights, kv_mode="f16", run_dtype="f16"):
        """cfg: object with the Qwen3 Config field names; dense_projections[layer][j]: [d_out, d_in]
        arrays in the order q, k, v, o, gate, up, down; weights: arrays of the run dtype (input_norm,
        post_norm, q_norm, k_norm, final_norm, embed, lm_head or None).  run_dtype "f16" is how the
        reference serves; "f32" is how its CPU tests build the model (tests/kv_cache.rs:56-60)."""
        self.cfg = cfg
        assert kv_mode in ("f16", "q8") and run_dtype in ("f16", "f32")
        self.kv_mode = kv_mode
        self.rnd = rnd = r16 if run_dtype == "f16" else r32
        wide = np.float16 if run_dtype == "f16" else np.float32
        self.W = [[np.asarray(m, np.float64) for m in layer] for layer in dense_projections]
        f = lambda a: np.asarray(a, wide).astype(np.float64)
        self.ln1, self.ln2 = f(weights.input_norm), f(weights.post_norm)
        self.qn, self.kn, self.fn = f(weights.q_norm), f(weights.k_norm), f(weights.final_norm)
        # A table is a binary16 array, or (packed, scales, biases) of an int8 g64 tensor
        # (sealed.rs:64-78): rows f16(s q + b) on the way in (emb_q8.cu emb_q8_gather),
        # f32 weights s q + b on the way out (tv_q8_h).
        def table(t):
            if isinstance(t, tuple):
                from . import sealed_oracle
                W = sealed_oracle.q8_rows_f32(np.asarray(t[0], np.uint8), np.asarray(t[1], np.uint16),
                                              np.asarray(t[2], np.uint16), cfg.hidden_size)
                return W.astype(np.float16), W.astype(np.float64)
            a = np.asarray(t, wide)
            return a, a.astype(np.float64)

        self.embed, embed_w = table(weights.embed)
        self.head = embed_w if weights.lm_head is None else table(weights.lm_head)[1]
        self.cos, self.sin = rope_tables(cfg.head_dim, cfg.rope_theta, cfg.max_positions, rnd)
        self.reset()

    def reset(self):
        L = self.cfg.num_hidden_layers
        self.K = [[] for _ in range(L)]
        self.V = [[] for _ in range(L)]
        self.pos = 0

    def forward_token(self, token):
        """hidden_cached at l = 1, then the head: returns the logits (f32; binary16-valued at the f16 run dtype)."""
        c = self.cfg
        nh, nkv, hd = c.num_attention_heads, c.num_key_value_heads, c.head_dim
        eps = c.rms_norm_eps
        rnd = self.rnd
        h = self.embed[int(token)].astype(np.float64)
        cos, sin = self.cos[self.pos], self.sin[self.pos]
        for L in range(c.num_hidden_layers):
            Wq, Wk, Wv, Wo, Wg, Wu, Wd = self.W[L]
            x = rms_norm(h, self.ln1[L], eps, rnd)
            q = rnd(Wq @ x).reshape(nh, hd)
            k = rnd(Wk @ x).reshape(nkv, hd)
            v = rnd(Wv @ x).reshape(nkv, hd)
            q = rms_norm(q, self.qn[L], eps, rnd)
            k = rms_norm(k, self.kn[L], eps, rnd)

            def rope(t):  # rotate-half: candle_nn::rotary_emb::rope
                t1, t2 = t[:, : hd // 2], t[:, hd // 2:]
                return rnd(np.concatenate([t1 * cos - t2 * sin, t1 * sin + t2 * cos], axis=1))

            q, k = rope(q), rope(k)
            if self.kv_mode == "q8":  # KvCache::append, model.rs:231-237: quantized once, on the way in
                k, v = quantize_dequantize(k), quantize_dequantize(v)
            self.K[L].append(k)
            self.V[L].append(v)
            Kc = np.stack(self.K[L], axis=1)  # [nkv, T, hd]
            Vc = np.stack(self.V[L], axis=1)
            groups = nh // nkv
            ctx = np.empty((nh, hd))
            for head in range(nh):  # repeat_kv: query head -> cached head head // groups
                kv = head // groups
                s = (Kc[kv] @ q[head]) / np.sqrt(float(hd))
                p = np.exp(s - s.max())
                p /= p.sum()
                ctx[head] = p @ Vc[kv]
            ctx = rnd(ctx.reshape(-1))
            h = rnd(h + rnd(Wo @ ctx))
            x = rms_norm(h, self.ln2[L], eps, rnd)
            g, u = rnd(Wg @ x), rnd(Wu @ x)
            a = rnd(rnd(silu(g)) * u)
            h = rnd(h + rnd(Wd @ a))
        x = rms_norm(h, self.fn, eps, rnd)
        self.pos += 1
        return rnd(self.head @ x).astype(np.float32)

    def prefill_rows(self, tokens, progress=None):
        """The prompt's positions all at once, in matrix form (the reference's l > 1 path: every projection is
        applied to all rows, model.rs:521-529; the causal mask of model.rs:985-994), from an empty cache.  Same
        operators and the same roundings as forward_token — only the f64 summation order inside a product
        differs — so the cache it leaves and the logits of its last row are those of a token-by-token run
        (tests/test_oracle_runner.py compares the two).  Attention runs one query head at a time so that a long
        prompt's score matrix stays one head's.  Returns the last row's logits."""
        c = self.cfg
        nh, nkv, hd = c.num_attention_heads, c.num_key_value_heads, c.head_dim
        eps, rnd = c.rms_norm_eps, self.rnd
        assert self.pos == 0, "prefill_rows starts from an empty cache"
        T = len(tokens)
        h = self.embed[np.asarray(tokens, dtype=np.int64)].astype(np.float64)
        cos, sin = self.cos[:T, None, :], self.sin[:T, None, :]
        groups = nh // nkv
        rows = np.arange(T)

        def rope(t):
            t1, t2 = t[..., : hd // 2], t[..., hd // 2:]
            return rnd(np.concatenate([t1 * cos - t2 * sin, t1 * sin + t2 * cos], axis=-1))

        for L in range(c.num_hidden_layers):
            Wq, Wk, Wv, Wo, Wg, Wu, Wd = self.W[L]
            x = rms_norm(h, self.ln1[L], eps, rnd)
            q = rope(rms_norm(rnd(x @ Wq.T).reshape(T, nh, hd), self.qn[L], eps, rnd))
            k = rope(rms_norm(rnd(x @ Wk.T).reshape(T, nkv, hd), self.kn[L], eps, rnd))
            v = rnd(x @ Wv.T).reshape(T, nkv, hd)
            if self.kv_mode == "q8":
                k, v = quantize_dequantize(k), quantize_dequantize(v)
            self.K[L] = [k[t] for t in range(T)]
            self.V[L] = [v[t] for t in range(T)]
            ctx = np.empty((T, nh, hd))
            for head in range(nh):
                kv = head // groups
                s = (q[:, head, :] @ k[:, kv, :].T) / np.sqrt(float(hd))
                s[rows[None, :] > rows[:, None]] = -np.inf
                p = np.exp(s - s.max(-1, keepdims=True))
                p /= p.sum(-1, keepdims=True)
                ctx[:, head, :] = p @ v[:, kv, :]
            ctx = rnd(ctx.reshape(T, nh * hd))
            h = rnd(h + rnd(ctx @ Wo.T))
            x = rms_norm(h, self.ln2[L], eps, rnd)
            a = rnd(rnd(silu(rnd(x @ Wg.T))) * rnd(x @ Wu.T))
            h = rnd(h + rnd(a @ Wd.T))
            if progress:
                progress(L)
        self.pos = T
        x = rms_norm(h[-1], self.fn, eps, rnd)
        return rnd(self.head @ x).astype(np.float32)

    def generate(self, prompt, max_new):
        """model.rs:1041-1073; also returns the logits of every decoding step."""
        if max_new == 0:
            return np.zeros(0, np.uint32), []
        self.reset()
        logits = None
        for t in prompt:
            logits = self.forward_token(t)
        out, trace = [], []
        while True:
            trace.append(logits)
            nxt = int(np.argmax(logits))  # first index on ties
            out.append(nxt)
            if len(out) == max_new:
                return np.array(out, np.uint32), trace
            logits = self.forward_token(nxt)
