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
