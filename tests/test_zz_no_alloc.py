"""llvq_hip_gemm_static — the batched product for callers that cannot allocate device
memory — against llvq_hip_gemm, through the C ABI.

Both entry points run the same kernels, so the outputs must be identical bit for bit; the
static one takes its partial sums, tiled activations and rotated rows from a static device
array that keeps the previous call's contents, which is why the second call here is the
smaller one.  Run last: a failure here must not hide the other tests.
"""
import numpy as np
import pytest

from llvq_amd import _ffi, synth

pytestmark = pytest.mark.gpu


def _x16(x):
    import torch

    return torch.from_numpy(x.view(np.int16).copy()).view(torch.float16).cuda()


def _both(rt, proj, X, dtype):
    import torch

    x = _x16(X)
    want = rt.forward_batched(proj, x, out_dtype=dtype)
    got = torch.full((X.shape[0], proj.d_out), float("nan"), dtype=dtype, device="cuda")
    rt.forward_batched_static_into(proj, x, got)
    rt.synchronize()
    return want.cpu().numpy(), got.cpu().numpy()


@pytest.mark.parametrize("rotated", [False, True])
def test_static_workspace_matches_the_allocating_entry_point(gpu_rt, rotated):
    import torch

    rot = 0x5EED if rotated else None
    big = synth.make_matrix("model.layers.0.static.big.weight", 1024, 4096, seed=11)
    small = synth.make_matrix("model.layers.0.static.small.weight", 72, 192 if rotated else 184, seed=12)
    big.rotation_seed = small.rotation_seed = rot  # stored as W Q^T: the call rotates the rows first
    p_big, p_small = gpu_rt.upload(big), gpu_rt.upload(small)
    try:
        # two calls in a row on the same GPU's array, the second with the smaller input
        for proj, M, seed in ((p_big, 130, 1), (p_small, 17, 2), (p_big, 2, 3)):
            X = synth.make_activation(proj.d_in, seed=seed, rows=M)
            for dtype in (torch.float32, torch.float16):
                want, got = _both(gpu_rt, proj, X, dtype)
                assert np.isfinite(want.astype(np.float64)).all()
                assert np.array_equal(want.view(np.uint8), got.view(np.uint8)), f"{proj.name} M={M} {dtype}"
        # the defining property: with inputs and outputs in place, the calls take no device memory
        x = _x16(synth.make_activation(p_big.d_in, seed=4, rows=130))
        y = torch.empty((130, p_big.d_out), dtype=torch.float16, device="cuda")
        gpu_rt.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        for M in (130, 64, 2):
            gpu_rt.forward_batched_static_into(p_big, x[:M], y[:M])
        gpu_rt.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
    finally:
        gpu_rt.free(p_big)
        gpu_rt.free(p_small)


def test_static_workspace_refuses_what_does_not_fit(gpu_rt):
    import torch

    # 12288 x 4096 at 512 rows needs several hundred MB of partial sums
    raw = synth.make_matrix("model.layers.0.static.wide.weight", 12288, 4096, seed=13)
    proj = gpu_rt.upload(raw)
    try:
        x = torch.zeros((512, 4096), dtype=torch.float16, device="cuda")
        y = torch.empty((512, 12288), dtype=torch.float16, device="cuda")
        with pytest.raises(_ffi.LlvqError) as err:
            gpu_rt.forward_batched_static_into(proj, x, y)
        assert err.value.kind == "Unsupported" and "static" in str(err.value)
        # and the refusal leaves the entry point usable
        y2 = torch.empty((16, 12288), dtype=torch.float16, device="cuda")
        gpu_rt.forward_batched_static_into(proj, x[:16].contiguous(), y2)
        gpu_rt.synchronize()
        assert torch.isfinite(y2).all()
    finally:
        gpu_rt.free(proj)


def test_static_workspace_refuses_the_whole_call(gpu_rt):
    """Rows beyond 512 go out as further launches, and a short last one can need more partial sums than a
    full one (its consumers split the K-steps): 17000 x 4096 at 576 rows fits its first 512 and not its last
    64.  The call is refused before anything is enqueued, so no row of y is written."""
    import torch

    raw = synth.make_matrix("model.layers.0.static.uneven.weight", 17000, 4096, seed=14)
    proj = gpu_rt.upload(raw)
    try:
        x = _x16(synth.make_activation(4096, seed=5, rows=576))
        y = torch.full((576, 17000), float("nan"), dtype=torch.float16, device="cuda")
        with pytest.raises(_ffi.LlvqError) as err:
            gpu_rt.forward_batched_static_into(proj, x, y)
        assert err.value.kind == "Unsupported" and "static" in str(err.value)
        gpu_rt.synchronize()
        assert bool(torch.isnan(y).all())
        gpu_rt.forward_batched_static_into(proj, x[:512], y[:512])  # the part that does fit, by itself
        gpu_rt.synchronize()
        assert bool(torch.isfinite(y[:512]).all()) and bool(torch.isnan(y[512:]).all())
    finally:
        gpu_rt.free(proj)
