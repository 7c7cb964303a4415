"""A whole sealed artifact, end to end: matrices + raw tensors (norms as binary16,
the embedding as int8 g64, optionally an untied int8 head) + config.json /
tokenizer.json blobs are written with the file format, loaded back with
fused.load_bytes (fused::load, fused.rs:1147), turned into a decoder from the
file alone, and compared with the oracle runner fed the same tensors."""
import json
from types import SimpleNamespace

import numpy as np
import pytest

from llvq_amd import artifact, decoder, fused

pytestmark = pytest.mark.gpu


def _quantize_rows(w, group=64):
    """An int8 g64 encoding of a float table (what the reference's embedq tool emits: sealed.rs:64-78)."""
    rows, d = w.shape
    g = w.reshape(rows, d // group, group).astype(np.float32)
    mn, mx = g.min(-1, keepdims=True), g.max(-1, keepdims=True)
    s = ((mx - mn) / 255.0).astype(np.float16)
    b = mn.astype(np.float16)
    safe = np.where(s.astype(np.float32) > 0, s.astype(np.float32), 1.0)
    q = np.clip(np.rint((g - b.astype(np.float32)) / safe), 0, 255).astype(np.uint8)
    return q.reshape(rows, d), s.reshape(-1).view(np.uint16), b.reshape(-1).view(np.uint16)


def _sealed_file(cfg, seed, tied):
    rng = np.random.default_rng(seed)
    raws = decoder.synthetic_projections(cfg, seed)
    L, h, d = cfg.num_hidden_layers, cfg.hidden_size, cfg.head_dim
    gains = lambda n: (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float16).view(np.uint16)
    tensors = []
    for i in range(L):
        tensors += [artifact.RawTensor(f"model.layers.{i}.input_layernorm.weight", [h], data=gains(h)),
                    artifact.RawTensor(f"model.layers.{i}.post_attention_layernorm.weight", [h], data=gains(h)),
                    artifact.RawTensor(f"model.layers.{i}.self_attn.q_norm.weight", [d], data=gains(d)),
                    artifact.RawTensor(f"model.layers.{i}.self_attn.k_norm.weight", [d], data=gains(d))]
    tensors.append(artifact.RawTensor("model.norm.weight", [h], data=gains(h)))
    q, s, b = _quantize_rows(rng.standard_normal((cfg.vocab_size, h)))
    tensors.append(artifact.RawTensor("model.embed_tokens.weight", [cfg.vocab_size, h], bits=8, group=64, packed=q.reshape(-1),
                                      scales=s, biases=b))
    if not tied:
        q, s, b = _quantize_rows(0.1 * rng.standard_normal((cfg.vocab_size, h)))
        tensors.append(artifact.RawTensor("lm_head.weight", [cfg.vocab_size, h], bits=8, group=64, packed=q.reshape(-1),
                                          scales=s, biases=b))
    config = dict(hidden_size=h, num_hidden_layers=L, num_attention_heads=cfg.num_attention_heads,
                  num_key_value_heads=cfg.num_key_value_heads, head_dim=d, intermediate_size=cfg.intermediate_size,
                  vocab_size=cfg.vocab_size, rope_theta=cfg.rope_theta, rms_norm_eps=cfg.rms_norm_eps,
                  tie_word_embeddings=tied, max_position_embeddings=cfg.max_positions)
    blobs = [artifact.Blob("config.json", json.dumps(config).encode()), artifact.Blob("tokenizer.json", b"{}")]
    mats = [m for layer in raws for m in layer]
    rng.shuffle(mats)  # the loader finds projections by name, not by position
    return artifact.write_file(mats, version=4, raws=tensors, blobs=blobs), raws


@pytest.mark.parametrize("tied", [True, False])
def test_decoder_from_a_sealed_file(gpu_rt, orc, tied):
    from oracle import qwen3_oracle

    cfg = decoder.Qwen3Config(num_hidden_layers=2, hidden_size=192, num_attention_heads=4, num_key_value_heads=2,
                              head_dim=64, intermediate_size=320, vocab_size=264, rope_theta=1e6, rms_norm_eps=1e-6,
                              max_positions=32, tie_word_embeddings=tied)
    buf, raws = _sealed_file(cfg, 21, tied)
    model = fused.load_bytes(buf)
    assert len(model.matrices) == 14 and json.loads(model.config_json)["hidden_size"] == 192
    assert model.carried_weights == 2 * (2 * 192 + 2 * 64) + 192 + (1 if tied else 2) * 264 * 192
    dec = decoder.Decoder.from_model(gpu_rt, model, kv_mode="q8")
    assert dec.cfg.tie_word_embeddings == tied and dec.cfg.num_key_value_heads == 2

    def halves(name):
        return model.tensor(name).data.view(np.float16)

    def q8(name):
        t = model.tensor(name)
        return (t.packed, t.scales, t.biases)

    L = cfg.num_hidden_layers
    weights = SimpleNamespace(
        input_norm=np.stack([halves(f"model.layers.{i}.input_layernorm.weight") for i in range(L)]),
        post_norm=np.stack([halves(f"model.layers.{i}.post_attention_layernorm.weight") for i in range(L)]),
        q_norm=np.stack([halves(f"model.layers.{i}.self_attn.q_norm.weight") for i in range(L)]),
        k_norm=np.stack([halves(f"model.layers.{i}.self_attn.k_norm.weight") for i in range(L)]),
        final_norm=halves("model.norm.weight"), embed=q8("model.embed_tokens.weight"),
        lm_head=None if tied else q8("lm_head.weight"))
    dense = [[orc.read_matrix_raw(artifact.write_matrix_raw(m))[0].decode_matrix() for m in layer] for layer in raws]
    ref = qwen3_oracle.Qwen3Oracle(dec.cfg, dense, weights, kv_mode="q8")
    try:
        worst = 0.0
        for t in np.random.default_rng(4).integers(0, cfg.vocab_size, size=16):
            want = ref.forward_token(int(t))
            got, best = dec.forward_token(int(t))
            worst = max(worst, float(np.abs(got - want).max() / np.abs(want).max()))
            assert best == int(np.argmax(got))
        assert worst < 2e-2, f"max |dlogit| / max|logit| = {worst:.3e}"
    finally:
        dec.close()


def test_incomplete_files_are_refused_by_name(gpu_rt):
    cfg = decoder.Qwen3Config(num_hidden_layers=1, hidden_size=64, num_attention_heads=1, num_key_value_heads=1,
                              head_dim=64, intermediate_size=96, vocab_size=32, max_positions=8, tie_word_embeddings=True)
    buf, raws = _sealed_file(cfg, 3, True)
    version, mats, tensors, blobs = artifact.read_sealed(buf)
    with pytest.raises(ValueError, match="tokenizer.json"):  # fused.rs:1252-1254
        fused.load_bytes(artifact.write_file(mats, raws=tensors, blobs=blobs[:1]))
    with pytest.raises(ValueError, match="projections-only"):  # fused.rs:1151-1158
        fused.load_bytes(artifact.write_header(1, len(mats)) + b"".join(artifact.write_matrix_raw(m) for m in mats))
    model = fused.load_bytes(artifact.write_file(mats[:-1], raws=tensors, blobs=blobs))
    with pytest.raises(ValueError, match="carries no model.layers.0"):
        decoder.Decoder.from_model(gpu_rt, model)
    model = fused.load_bytes(artifact.write_file(mats, raws=tensors[:-1], blobs=blobs))
    with pytest.raises(KeyError, match="embed_tokens"):
        decoder.Decoder.from_model(gpu_rt, model)
