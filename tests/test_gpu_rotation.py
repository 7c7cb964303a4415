"""Rotated artifacts on the device: the activation rotation kernel against the
oracle's Rotation, and the product y = W'(Q x) against the oracle's dense arm
(decode_matrix un-rotates to the natural basis) — the identity of
llvq-artifact/tests/fused_path_matches_dense.rs."""
import numpy as np
import pytest

from llvq_amd import artifact, decoder, synth

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _x16(x):
    import torch

    return torch.from_numpy(x.view(np.int16).copy()).view(torch.float16).cuda()


def _rotated(name, d_out, d_in, seed, rot_seed):
    raw = synth.make_matrix(name, d_out, d_in, seed=seed)
    raw.rotation_seed = rot_seed
    return raw


# widths of fused.rs:1274 (k = 15, 5, 19, 1, 3) plus the 8B/14B hidden sizes (k = 1, 5)
@pytest.mark.parametrize("n,seed", [(240, 1), (2560, 2), (9728, 3), (4096, 4), (96, 5), (5120, 6), (24, 7)])
def test_rotate_kernel_matches_oracle(gpu_rt, orc, n, seed):
    raw = _rotated(f"model.layers.0.r{n}.weight", 8, n, 1, seed)
    x = synth.make_activation(n, seed=seed)[0]
    proj = gpu_rt.upload(raw)
    xr = gpu_rt.rotate(proj, _x16(x)).cpu().numpy().reshape(-1)
    gpu_rt.free(proj)
    want = orc.Rotation(n, seed).apply(x.astype(np.float64))
    dev = np.linalg.norm(xr - want) / np.linalg.norm(want)
    assert dev < 1e-5, f"relative deviation {dev:.3e}"   # f32 butterflies
    assert np.abs(xr - want).max() < 1e-4 * np.abs(want).max()


def test_natural_basis_rotate_only_widens(gpu_rt):
    raw = synth.make_matrix("model.layers.0.plain.weight", 8, 240, seed=1)
    x = synth.make_activation(240, seed=3)[0]
    proj = gpu_rt.upload(raw)
    xr = gpu_rt.rotate(proj, _x16(x)).cpu().numpy().reshape(-1)
    gpu_rt.free(proj)
    assert np.array_equal(xr, x.astype(np.float32))


@pytest.mark.parametrize("d_out,d_in", [(8, 240), (16, 2560), (8, 9728), (24, 4096), (8, 96), (5, 256), (7, 104)])
def test_rotated_gemv_matches_dense_arm(gpu_rt, orc, d_out, d_in):
    import torch

    raw = _rotated(f"model.layers.0.rot.{d_out}x{d_in}.weight", d_out, d_in, seed=d_in, rot_seed=0xA5 + d_in)
    x = synth.make_activation(d_in, seed=d_in + 1)[0]
    om, _ = orc.read_matrix_raw(artifact.write_matrix_raw(raw))
    y_ref, a_ref = om.fused_product(x.astype(np.float64))        # rotates the activation, f64
    W = om.decode_matrix().astype(np.float64)                      # un-rotated weights
    assert np.abs(W @ x.astype(np.float64) - y_ref).max() < 1e-6 * a_ref.max()
    proj = gpu_rt.upload(raw)
    try:
        y = gpu_rt.forward(proj, _x16(x), out_dtype=torch.float32).cpu().numpy().astype(np.float64)
        y2 = gpu_rt.forward_rotated(proj, gpu_rt.rotate(proj, _x16(x)), out_dtype=torch.float32).cpu().numpy().reshape(-1)
    finally:
        gpu_rt.free(proj)
    e = np.abs(y - y_ref) / np.maximum(a_ref, 1e-30)
    assert e.max() < 1e-5, f"max |dy|/sum|wx| = {e.max():.3e}"
    assert np.array_equal(y.astype(np.float32), y2)  # the two-call form is the same computation


def test_wide_odd_factor_is_refused_at_upload(gpu_rt):
    from llvq_amd import LlvqError

    raw = _rotated("model.layers.0.odd.weight", 8, 2568, 1, 5)  # 2568 = 8 * 321 (fused.rs:698-704)
    with pytest.raises(LlvqError) as e:
        gpu_rt.upload(raw)
    assert e.value.kind == "Unsupported" and "321" in str(e.value)


def test_group_with_mixed_bases(gpu_rt, orc):
    """q rotated with one seed, k with another, v in the natural basis: three bases, one call."""
    import torch

    mats = [_rotated("model.layers.1.self_attn.q_proj.weight", 32, 2560, 3, 11),
            _rotated("model.layers.1.self_attn.k_proj.weight", 16, 2560, 3, 12),
            synth.make_matrix("model.layers.1.self_attn.v_proj.weight", 16, 2560, seed=3),
            _rotated("model.layers.1.self_attn.x_proj.weight", 8, 2560, 4, 11)]
    x = synth.make_activation(2560, seed=8)[0]
    projs = [gpu_rt.upload(m) for m in mats]
    ys = gpu_rt.forward_group(projs, _x16(x), out_dtype=torch.float32)
    for p, raw, y in zip(projs, mats, ys):
        om, _ = orc.read_matrix_raw(artifact.write_matrix_raw(raw))
        y_ref, a_ref = om.fused_product(x.astype(np.float64))
        assert (np.abs(y.cpu().numpy() - y_ref) / a_ref).max() < 1e-5
        gpu_rt.free(p)


def test_rotated_batched_rows(gpu_rt, orc):
    import torch

    raw = _rotated("model.layers.2.mlp.up_proj.weight", 128, 2560, 4, 99)
    X = synth.make_activation(2560, seed=21, rows=24)
    om, _ = orc.read_matrix_raw(artifact.write_matrix_raw(raw))
    W = om.decode_matrix().astype(np.float64)
    Y_ref = X.astype(np.float64) @ W.T
    # the normaliser in the rotated basis, where the kernel sums
    rot = orc.Rotation(2560, 99)
    Wr = np.stack([rot.apply(r) for r in W])
    Xr = np.stack([rot.apply(r) for r in X.astype(np.float64)])
    A_ref = np.abs(Xr) @ np.abs(Wr).T
    proj = gpu_rt.upload(raw)
    Y = gpu_rt.forward_batched(proj, _x16(X), out_dtype=torch.float32).cpu().numpy()
    gpu_rt.free(proj)
    assert (np.abs(Y - Y_ref) / A_ref).max() < TOL


def test_decoder_with_rotated_projections(gpu_rt, orc):
    """The decode loop over an artifact whose projections are all stored rotated
    (one seed per activation site, as the reference's rotation keys are)."""
    from oracle import qwen3_oracle

    cfg = decoder.Qwen3Config(num_hidden_layers=2, hidden_size=192, num_attention_heads=4, num_key_value_heads=2,
                              head_dim=32, intermediate_size=320, vocab_size=300, rope_theta=1e4, rms_norm_eps=1e-6,
                              max_positions=32, tie_word_embeddings=True)
    raws = decoder.synthetic_projections(cfg, 5)
    for L, layer in enumerate(raws):
        for j, m in enumerate(layer):
            m.rotation_seed = 1000 + 10 * L + (0 if j < 3 else 1 if j == 3 else 2 if j < 6 else 3)
    weights = decoder.synthetic_weights(cfg, 5)
    dense = [[orc.read_matrix_raw(artifact.write_matrix_raw(m))[0].decode_matrix() for m in layer] for layer in raws]
    ref = qwen3_oracle.Qwen3Oracle(cfg, dense, weights)
    dec = decoder.Decoder(gpu_rt, cfg, raws, weights)
    try:
        worst = 0.0
        for t in np.random.default_rng(5).integers(0, cfg.vocab_size, size=12):
            want = ref.forward_token(int(t))
            got, _ = dec.forward_token(int(t))
            worst = max(worst, float(np.abs(got - want).max() / np.abs(want).max()))
        assert worst < 2e-2
    finally:
        dec.close()
