"""llvq_hip_sequence_*: a list of group products as one persistent launch.  The bar is bit-identity with the
per-call entry points (llvq_hip_gemv_group), which tests/test_gpu_parity.py holds against the CPU oracle; one
case is also compared with the oracle directly."""
import numpy as np
import pytest

from llvq_amd import LlvqError, artifact, synth

from test_gpu_parity import _check_gemv, _class_ranges, _is_rare, _matrix_of_classes, _x16

pytestmark = pytest.mark.gpu


def _same_bits(a, b):
    import torch

    return a.dtype == b.dtype and a.shape == b.shape and bool(torch.equal(a.view(torch.int16 if a.dtype == torch.float16 else torch.int32),
                                                                         b.view(torch.int16 if b.dtype == torch.float16 else torch.int32)))


def _layer(gpu_rt, seed, shapes):
    raws = [synth.make_matrix(f"model.layers.{seed}.p{j}.weight", do, di, seed) for j, (do, di) in enumerate(shapes)]
    return raws, [gpu_rt.upload(m) for m in raws]


@pytest.mark.parametrize("out,widest", [("f16", 9728), ("f32", 9728), ("f16", 24 * 700 + 5)])
def test_independent_items_match_the_separate_calls(gpu_rt, orc, out, widest):
    """Eight items over six widths — tiles of many rows and of one, a width below one block (tail columns only),
    an item of three matrices, more tiles than workgroups and fewer — against llvq_hip_gemv_group item by item,
    bit for bit, on three runs of the same sequence; the first item also against the CPU oracle.  With rows
    of 700 blocks in the list the whole sequence runs the kernel variant that keeps two tables in L2."""
    import torch

    dt = torch.float16 if out == "f16" else torch.float32
    groups = [[(1024, 2560), (256, 2560), (256, 2560)], [(640, 4096)], [(2432, 2560), (2432, 2560)], [(320, 9728)],
              [(40, 17)], [(7, widest)], [(5000, 48)], [(64, 2560)]]
    uploaded, items, xs = [], [], {}
    try:
        for gi, shapes in enumerate(groups):
            raws, projs = _layer(gpu_rt, 100 + gi, shapes)
            uploaded.append((raws, projs))
            d_in = shapes[0][1]
            if d_in not in xs:
                xs[d_in] = synth.make_activation(d_in, seed=d_in)[0]
            items.append((projs, _x16(xs[d_in]), False))
        seq = gpu_rt.plan_sequence(items, out_dtype=dt)
        try:
            want = [gpu_rt.forward_group(projs, x, out_dtype=dt) for projs, x, _ in items]
            for run in range(3):
                for ys in seq.outputs:
                    for y in ys:
                        y.fill_(float("nan"))
                seq.run()
                seq.status()
                for gi, (ys, ws) in enumerate(zip(seq.outputs, want)):
                    for y, w in zip(ys, ws):
                        assert _same_bits(y, w), f"run {run}, item {gi}: outputs differ from the separate call"
            if out == "f32":
                raw0, x0 = uploaded[0][0][0], xs[2560]
                assert _check_gemv(orc, seq.outputs[0][0].cpu().numpy(), raw0, x0) < 1e-5
        finally:
            seq.close()
    finally:
        for _, projs in uploaded:
            for p in projs:
                gpu_rt.free(p)


def test_hostile_tiles_through_the_sequence(gpu_rt, orc):
    """Tiles full of generic-class blocks (the side queues overflow), of second-free-kind blocks (their queue
    overflows) and of origins, one item each, against the separate calls bit for bit."""
    import torch

    rare = _matrix_of_classes(_class_ranges(orc, _is_rare), 1280, 40, 11, "model.layers.0.rare.weight")
    second = _matrix_of_classes(_class_ranges(orc, lambda odd, w, vals: not odd and not _is_rare(odd, w, vals)
                                              and len([v for v in vals if v != 0 and abs(v) % 4 == 0]) > 1),
                                1280, 100, 21, "model.layers.0.second.weight")
    rng = synth.SplitMix64(7)
    idx = rng.take(600 * 30) % np.uint64(1 << 47)
    idx[rng.take(idx.size) % np.uint64(3) != 0] = 0  # two thirds origins
    origins = artifact.RawMatrix("model.layers.0.origins.weight", 600, 30 * 24 + 7, 12, [0.8, 1.25], np.exp(rng.gaussian(600)),
                                 rng.gaussian(600 * 7).astype(np.float32), artifact.pack_codes(idx, (rng.take(idx.size) & np.uint64(1)).astype(np.uint8)))
    raws = [rare, second, origins]
    projs = [gpu_rt.upload(m) for m in raws]
    try:
        items = [([p], _x16(synth.make_activation(m.d_in, seed=3)[0]), False) for p, m in zip(projs, raws)]
        seq = gpu_rt.plan_sequence(items, out_dtype=torch.float32)
        try:
            seq.run()
            seq.status()
            for (ps, x, _), ys, m in zip(items, seq.outputs, raws):
                want = gpu_rt.forward_group(ps, x, out_dtype=torch.float32)
                assert _same_bits(ys[0], want[0]), m.name
        finally:
            seq.close()
    finally:
        for p in projs:
            gpu_rt.free(p)


def _chain(gpu_rt, widths, seed):
    """Matrices W_k of shape widths[k+1] x widths[k]: item k's activation is item k-1's output."""
    raws = [synth.make_matrix(f"model.layers.{seed}.chain{k}.weight", widths[k + 1], widths[k], seed) for k in range(len(widths) - 1)]
    return raws, [gpu_rt.upload(m) for m in raws]


def _bind_chain(gpu_rt, projs, widths, x):
    import torch

    outs = [torch.empty(widths[k + 1], dtype=torch.float16, device="cuda") for k in range(len(projs))]
    items = [([projs[k]], x if k == 0 else outs[k - 1], k > 0, [outs[k]]) for k in range(len(projs))]
    return gpu_rt.plan_sequence(items), outs


def test_ordered_items_wait_for_the_item_before(gpu_rt):
    """A chain y1 = W1 x, y2 = W2 y1, y3 = W3 y2, y4 = W4 y3 in one launch: every item but the first reads what
    the item before it stores, so its workgroups wait on the device.  Five runs, each on a different activation
    written into the same buffer, against the four separate calls bit for bit."""
    import torch

    widths = [2560, 4096, 1200, 9728, 2560]
    raws, projs = _chain(gpu_rt, widths, 31)
    try:
        x = _x16(synth.make_activation(widths[0], seed=1)[0])
        seq, outs = _bind_chain(gpu_rt, projs, widths, x)
        try:
            for run in range(5):
                x.copy_(_x16(synth.make_activation(widths[0], seed=50 + run)[0]))
                for o in outs:
                    o.fill_(float("nan"))
                seq.run()
                seq.status()
                a = x
                for k in range(len(projs)):
                    a = gpu_rt.forward(projs[k], a, out_dtype=torch.float16)
                    assert _same_bits(outs[k], a), f"run {run}, item {k}"
        finally:
            seq.close()
    finally:
        for p in projs:
            gpu_rt.free(p)


def test_a_wait_that_cannot_end_gives_up_and_reports(gpu_rt):
    """The host withholds an item: the next run is told to treat item 0 as never complete, with a wait of 200
    polls.  The kernel must end by itself, the status call must report it, and the run after that must be
    right again."""
    widths = [2560, 1024, 512]
    raws, projs = _chain(gpu_rt, widths, 33)
    try:
        x = _x16(synth.make_activation(widths[0], seed=2)[0])
        seq, outs = _bind_chain(gpu_rt, projs, widths, x)
        try:
            seq.run()
            seq.status()
            good = outs[1].clone()
            seq.tune(spin_limit=200, hold_item=0)
            seq.run()
            with pytest.raises(LlvqError) as err:
                seq.status()
            assert err.value.kind == "Device" and "gave up" in str(err.value)
            seq.tune()
            outs[1].fill_(float("nan"))
            seq.run()
            seq.status()
            assert _same_bits(outs[1], good)
        finally:
            seq.close()
    finally:
        for p in projs:
            gpu_rt.free(p)


def test_sequence_refusals(gpu_rt):
    """Named refusals, nothing enqueued: a rotated matrix, an ordered first item, mixed widths in one item."""
    import torch

    raw = synth.make_matrix("model.layers.0.r.weight", 64, 512, 5)
    rot = artifact.RawMatrix(raw.name, raw.d_out, raw.d_in, 12, raw.centroids, raw.row_scales, raw.tail, raw.codes, rotation_seed=7)
    other = synth.make_matrix("model.layers.0.o.weight", 64, 768, 5)
    p, pr, po = gpu_rt.upload(raw), gpu_rt.upload(rot), gpu_rt.upload(other)
    try:
        x = torch.zeros(512, dtype=torch.float16, device="cuda")
        for items, kind in (([([pr], x, False)], "Unsupported"), ([([p], x, True)], "InvalidArgument"), ([([p, po], x, False)], "InvalidArgument")):
            with pytest.raises(LlvqError) as err:
                gpu_rt.plan_sequence(items)
            assert err.value.kind == kind
    finally:
        for q in (p, pr, po):
            gpu_rt.free(q)
