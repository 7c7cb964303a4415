"""Pins of the oracle's Qwen3 runner (oracle/qwen3_oracle.py) that do not retype
it: closed forms of the RoPE tables, special cases that collapse to one line,
and the reference's own strategy for its KV cache (llvq-llm/tests/kv_cache.rs:
the cached decode must reproduce a full causal re-run) against a full-sequence
forward written here in matrix form."""
from types import SimpleNamespace

import numpy as np

from oracle import qwen3_oracle as Q

CFG = SimpleNamespace(num_hidden_layers=2, hidden_size=48, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                      intermediate_size=80, vocab_size=61, rope_theta=1e4, rms_norm_eps=1e-6, max_positions=32)


def _model(seed=0, tied=True):
    rng = np.random.default_rng(seed)
    c = CFG
    qd, kvd = c.num_attention_heads * c.head_dim, c.num_key_value_heads * c.head_dim
    shapes = [(qd, c.hidden_size), (kvd, c.hidden_size), (kvd, c.hidden_size), (c.hidden_size, qd),
              (c.intermediate_size, c.hidden_size), (c.intermediate_size, c.hidden_size), (c.hidden_size, c.intermediate_size)]
    W = [[(rng.standard_normal(s) / np.sqrt(s[1])).astype(np.float32) for s in shapes] for _ in range(c.num_hidden_layers)]
    g = lambda *s: (1 + 0.1 * rng.standard_normal(s)).astype(np.float16)
    L = c.num_hidden_layers
    weights = SimpleNamespace(input_norm=g(L, c.hidden_size), post_norm=g(L, c.hidden_size), q_norm=g(L, c.head_dim),
                              k_norm=g(L, c.head_dim), final_norm=g(c.hidden_size),
                              embed=rng.standard_normal((c.vocab_size, c.hidden_size)).astype(np.float16),
                              lm_head=None if tied else rng.standard_normal((c.vocab_size, c.hidden_size)).astype(np.float16))
    return Q.Qwen3Oracle(c, W, weights), W, weights


def test_rope_tables_closed_form():
    cos, sin = Q.rope_tables(16, 1e4, 32)
    assert cos.shape == (32, 8)
    assert np.all(cos[0] == 1) and np.all(sin[0] == 0)  # position 0 is the identity
    # frequency 0 has inverse frequency 1: the angle is the position itself
    p = np.arange(32)
    assert np.allclose(cos[:, 0], np.cos(p), atol=1e-3) and np.allclose(sin[:, 0], np.sin(p), atol=1e-3)
    # last frequency: theta^(-(d-2)/d)
    assert np.allclose(sin[:, 7], np.sin(p * 1e4 ** (-14 / 16)), atol=1e-3)
    assert np.allclose(cos ** 2 + sin ** 2, 1, atol=2e-3)
    # values are binary16
    assert np.array_equal(cos, cos.astype(np.float16).astype(np.float64))


def test_rms_norm_scale_invariance_and_unit_rms():
    rng = np.random.default_rng(1)
    x = rng.standard_normal(64)
    y = Q.rms_norm(x, np.ones(64), 0.0)
    assert abs(np.sqrt(np.mean(y * y)) - 1) < 1e-3
    assert np.allclose(Q.rms_norm(4 * x, np.ones(64), 0.0), y, atol=2e-3)


def _full_sequence_logits(W, w, tokens):
    """Full causal forward in matrix form (the reference's uncached path, model.rs:985-994):
    every position at once, additive -inf mask above the diagonal."""
    c = CFG
    nh, nkv, hd = c.num_attention_heads, c.num_key_value_heads, c.head_dim
    f = lambda a: np.asarray(a, np.float16).astype(np.float64)
    T = len(tokens)
    cos, sin = Q.rope_tables(hd, c.rope_theta, c.max_positions)
    cos, sin = cos[:T, None, :], sin[:T, None, :]
    h = f(w.embed)[np.asarray(tokens)]
    mask = np.where(np.arange(T)[None, :] <= np.arange(T)[:, None], 0.0, -np.inf)
    for L in range(c.num_hidden_layers):
        Wq, Wk, Wv, Wo, Wg, Wu, Wd = [np.asarray(m, np.float64) for m in W[L]]
        x = Q.rms_norm(h, f(w.input_norm)[L], c.rms_norm_eps)
        q = Q.rms_norm(Q.r16(x @ Wq.T).reshape(T, nh, hd), f(w.q_norm)[L], c.rms_norm_eps)
        k = Q.rms_norm(Q.r16(x @ Wk.T).reshape(T, nkv, hd), f(w.k_norm)[L], c.rms_norm_eps)
        v = Q.r16(x @ Wv.T).reshape(T, nkv, hd)
        rot = lambda t: Q.r16(np.concatenate([t[..., : hd // 2] * cos - t[..., hd // 2:] * sin,
                                              t[..., : hd // 2] * sin + t[..., hd // 2:] * cos], axis=-1))
        q, k = rot(q), rot(k)
        k, v = np.repeat(k, nh // nkv, axis=1), np.repeat(v, nh // nkv, axis=1)
        s = np.einsum("qhd,khd->hqk", q, k) / np.sqrt(hd) + mask[None]
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        ctx = Q.r16(np.einsum("hqk,khd->qhd", p, v).reshape(T, nh * hd))
        h = Q.r16(h + Q.r16(ctx @ Wo.T))
        x = Q.rms_norm(h, f(w.post_norm)[L], c.rms_norm_eps)
        a = Q.r16(Q.r16(Q.silu(Q.r16(x @ Wg.T))) * Q.r16(x @ Wu.T))
        h = Q.r16(h + Q.r16(a @ Wd.T))
    x = Q.rms_norm(h, f(w.final_norm), c.rms_norm_eps)
    head = f(w.embed if w.lm_head is None else w.lm_head)
    return Q.r16(x @ head.T).astype(np.float32)


def test_cached_decode_reproduces_full_causal_rerun():
    for tied in (True, False):
        ref, W, w = _model(seed=3, tied=tied)
        tokens = np.random.default_rng(5).integers(0, CFG.vocab_size, size=11)
        full = _full_sequence_logits(W, w, tokens)
        for i, t in enumerate(tokens):
            step = ref.forward_token(int(t))
            # same roundings at the same places; summation order differs, so allow a binary16 step
            assert np.abs(step - full[i]).max() <= 2e-3 * np.abs(full[i]).max() + 1e-6


def test_single_position_attention_is_the_value():
    """With one cached position the softmax is 1: the context is v, repeated over the query groups."""
    ref, W, w = _model(seed=7)
    c = CFG
    f = lambda a: np.asarray(a, np.float16).astype(np.float64)
    tok = 9
    h = f(w.embed)[tok]
    x = Q.rms_norm(h, f(w.input_norm)[0], c.rms_norm_eps)
    v = Q.r16(np.asarray(W[0][2], np.float64) @ x).reshape(c.num_key_value_heads, c.head_dim)
    ctx = np.repeat(v, c.num_attention_heads // c.num_key_value_heads, axis=0).reshape(-1)
    h1 = Q.r16(h + Q.r16(np.asarray(W[0][3], np.float64) @ ctx))
    ref.forward_token(tok)
    # the oracle's cache holds exactly that v, and a second model truncated to the attention half agrees
    assert np.array_equal(ref.V[0][0], v)
    one_layer = SimpleNamespace(**{**CFG.__dict__, "num_hidden_layers": 1})
    r1 = Q.Qwen3Oracle(one_layer, [W[0]], SimpleNamespace(input_norm=w.input_norm[:1], post_norm=w.post_norm[:1],
                       q_norm=w.q_norm[:1], k_norm=w.k_norm[:1], final_norm=w.final_norm, embed=w.embed, lm_head=None))
    r1.W[0][4] = np.zeros_like(r1.W[0][4])  # gate = 0 -> MLP contributes nothing
    logits = r1.forward_token(tok)
    want = Q.r16(f(w.embed) @ Q.rms_norm(h1, f(w.final_norm), c.rms_norm_eps)).astype(np.float32)
    assert np.array_equal(logits, want)


def test_generate_edges():
    ref, _, _ = _model(seed=11)
    out, trace = ref.generate([1, 2, 3], 0)
    assert out.size == 0 and trace == []
    out, trace = ref.generate([1, 2, 3], 5)
    assert out.size == 5 and len(trace) == 5 and ref.pos == 3 + 4
    assert all(int(np.argmax(l)) == t for l, t in zip(trace, out))


# ---- KV-q8 (llvq-llm/src/kvq.rs tests :218-344) ---------------------------------------------
def _cache_like(t):
    """kvq.rs:223-237: 8 KV heads x t tokens x head_dim 128, spread growing with the head."""
    i = np.arange(8 * t * 128)
    head = (i // (t * 128)) % 8
    x = (i % 977).astype(np.float32) / np.float32(977.0) - np.float32(0.5)
    v = (1.0 + head).astype(np.float32) * x * np.sign(x) * np.float32(3.0)
    return v.reshape(1, 8, t, 128).astype(np.float16)


def test_kvq_prefill_and_decode_agree_bit_for_bit():  # kvq.rs:252-275
    full = _cache_like(16)
    both = Q.quantize_dequantize(full)
    for t in (0, 1, 7, 15):
        assert np.array_equal(Q.quantize_dequantize(full[:, :, t:t + 1]), both[:, :, t:t + 1])


def test_kvq_constant_group_reconstructs_exactly():  # kvq.rs:278-312
    v = np.where(np.arange(128) < 64, 0.375, np.arange(128) / 128.0).astype(np.float16).reshape(1, 1, 1, 128)
    out = Q.quantize_dequantize(v)
    assert np.array_equal(out[..., :64], v[..., :64].astype(np.float64))
    assert out[..., 64:].max() - out[..., 64:].min() > 0.4


def test_kvq_known_codes_and_half_step_bound():
    """Hand-computed: the ramp i/64, i = 0..63, has min 0 and max 63/64, so s = f16(63/64/255)
    and q_i = round((i/64)/s); the extremes land on 0 and 255 and the error is half a step."""
    x = (np.arange(64) / 64.0).astype(np.float16).reshape(1, 64)
    q, s, b = Q.kv_quantize(x)
    s16 = float(np.float16(np.float32(63 / 64) / np.float32(255)))
    assert float(s.reshape(())) == s16 and float(b.reshape(())) == 0.0
    want = np.floor(np.arange(64) / 64.0 / s16 + 0.5)
    assert np.array_equal(q.reshape(-1), np.clip(want, 0, 255).astype(np.uint8))
    assert q.reshape(-1)[0] == 0 and q.reshape(-1)[-1] == 255
    deq = Q.kv_dequantize(q, s, b, x.shape)
    assert np.abs(deq - x.astype(np.float64)).max() <= s16 / 2 + 2 ** -11  # half a step + the binary16 rounding
    # rounding, not truncation (kvq.rs:315-344): the mean error is centred
    big = _cache_like(4)
    err = Q.quantize_dequantize(big) - big.astype(np.float64)
    assert abs(err.mean()) < 0.1 * np.abs(err).mean()


def test_runner_q8_cache_holds_reconstructed_values():
    ref, W, w = _model(seed=13)
    c = SimpleNamespace(**{**CFG.__dict__, "head_dim": 64, "num_attention_heads": 2, "num_key_value_heads": 1,
                           "hidden_size": 48})
    qd, kvd = 128, 64
    rng = np.random.default_rng(2)
    shapes = [(qd, 48), (kvd, 48), (kvd, 48), (48, qd), (80, 48), (80, 48), (48, 80)]
    Wn = [[(rng.standard_normal(s) / np.sqrt(s[1])).astype(np.float32) for s in shapes] for _ in range(2)]
    g = lambda *s: (1 + 0.1 * rng.standard_normal(s)).astype(np.float16)
    wn = SimpleNamespace(input_norm=g(2, 48), post_norm=g(2, 48), q_norm=g(2, 64), k_norm=g(2, 64), final_norm=g(48),
                         embed=rng.standard_normal((61, 48)).astype(np.float16), lm_head=None)
    a = Q.Qwen3Oracle(c, Wn, wn, kv_mode="q8")
    b = Q.Qwen3Oracle(c, Wn, wn, kv_mode="f16")
    la, lb = a.forward_token(3), b.forward_token(3)
    # what the q8 cache holds is the quantize-dequantize of what the f16 cache holds (layer 0: same inputs)
    assert np.array_equal(a.K[0][0], Q.quantize_dequantize(b.K[0][0]))
    assert np.array_equal(a.V[0][0], Q.quantize_dequantize(b.V[0][0]))
    assert np.abs(la - lb).max() < 0.05 * np.abs(lb).max() and not np.array_equal(la, lb)


# ---- the reference's own golden for the runner (llvq-llm/tests/kv_cache.rs) -------------------
def _tiny_reference_model(swap_kv=False):
    """kv_cache.rs:31-52 (config) and :69-112 (weights): SplitMix64(0xA4_C0DE) Gaussians x 0.3 narrowed to
    f32, drawn in the order embed, then per layer q, k, v, o, gate, up, down; every norm weight is one;
    the head is tied; the model runs in f32 on the CPU."""
    from llvq_amd import synth

    cfg = SimpleNamespace(vocab_size=128, hidden_size=32, intermediate_size=64, num_hidden_layers=2,
                          num_attention_heads=4, num_key_value_heads=2, head_dim=8, rope_theta=10_000.0,
                          rms_norm_eps=1e-6, max_positions=64)
    rng = synth.SplitMix64(0xA4C0DE)

    def put(r, c):
        return (rng.gaussian(r * c) * 0.3).astype(np.float32).reshape(r, c)

    h, i, nh, nkv, hd = 32, 64, 4, 2, 8
    embed = put(cfg.vocab_size, h)
    layers = []
    for _ in range(cfg.num_hidden_layers):
        q = put(nh * hd, h)
        first, second = put(nkv * hd, h), put(nkv * hd, h)
        k, v = (second, first) if swap_kv else (first, second)
        layers.append([q, k, v, put(h, nh * hd), put(i, h), put(i, h), put(h, i)])
    ones = np.ones
    w = SimpleNamespace(input_norm=ones((2, h), np.float32), post_norm=ones((2, h), np.float32),
                        q_norm=ones((2, hd), np.float32), k_norm=ones((2, hd), np.float32),
                        final_norm=ones(h, np.float32), embed=embed, lm_head=None)
    return Q.Qwen3Oracle(cfg, layers, w, run_dtype="f32")


def test_reference_golden_tokens_of_the_tiny_model():
    """kv_cache.rs:140-153: prompt [3,1,4,1,5,9,2,6] -> [107,90,2,35,35,35,35,35], and exchanging
    k_proj and v_proj moves the sequence (:156-164).  Pins the runner's structure — projection
    order, per-head norms, the rotate-half RoPE at absolute positions, grouped-query attention over
    the cache, residuals, the tied head, first-index argmax — on values the reference holds.  The
    reference computes in f32 with candle's summation order and this runner in f64 between
    roundings, so a near-tie could legitimately differ; none does on this sequence."""
    golden = [107, 90, 2, 35, 35, 35, 35, 35]
    prompt = [3, 1, 4, 1, 5, 9, 2, 6]
    got, trace = _tiny_reference_model().generate(prompt, len(golden))
    assert got.tolist() == golden, (got.tolist(), [float(np.sort(t)[-1] - np.sort(t)[-2]) for t in trace])
    swapped, _ = _tiny_reference_model(swap_kv=True).generate(prompt, len(golden))
    assert swapped.tolist() != golden


def test_matrix_form_prompt_pass_leaves_the_cache_of_a_token_by_token_run():
    """prefill_rows (all prompt rows at once) against forward_token position by position: the cache
    entries and the last row's logits agree up to what a different f64 summation order can move across a
    binary16 rounding; the positions that follow, decoded over either cache, agree the same way."""
    global CFG
    saved = CFG
    try:
        for kv_mode, head_dim in (("f16", 16), ("q8", 64)):
            CFG = SimpleNamespace(**{**vars(saved), "head_dim": head_dim})
            _, W, w = _model(seed=7, tied=True)
            ref = Q.Qwen3Oracle(CFG, W, w, kv_mode=kv_mode)
            rows = Q.Qwen3Oracle(CFG, W, w, kv_mode=kv_mode)
            tokens = np.random.default_rng(8).integers(0, CFG.vocab_size, size=13)
            for t in tokens:
                step = ref.forward_token(int(t))
            last = rows.prefill_rows(tokens)
            assert rows.pos == ref.pos == 13
            assert np.abs(last - step).max() <= 2e-3 * np.abs(step).max() + 1e-6
            for L in range(CFG.num_hidden_layers):
                for a, b in ((ref.K[L], rows.K[L]), (ref.V[L], rows.V[L])):
                    a, b = np.asarray(a), np.asarray(b)
                    assert a.shape == b.shape and np.abs(a - b).max() <= 1e-2 * np.abs(a).max()
            for t in (5, 1, 4):
                x, y = ref.forward_token(t), rows.forward_token(t)
                assert np.abs(x - y).max() <= 2e-3 * np.abs(x).max() + 1e-6
    finally:
        CFG = saved
