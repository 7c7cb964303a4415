#!/usr/bin/env python3
"""Where a launch's time goes, phase by phase, from timestamps the kernels store themselves.

Needs the tuning build of the library (the product library has no timestamps compiled in):
    make -C llvq_amd/csrc libllvq_hip_stamps.so        # -DLLVQ_PHASE_TIMING -DLLVQ_SEQ_STAMPS
    python3 llvq_amd/csrc/phase_stamps.py gemv|seq|gemm

  gemv  gemv_tiles_kernel on the four projection groups of a Qwen3-4B layer (one llvq_hip_gemv_group launch each):
        lane 0 of every workgroup stamps the phases of its first tile.
  seq   gemv_seq_kernel on six Qwen3-4B layers bound as one sequence of 24 independent items: the phases of every
        workgroup's first eight rounds (a round = one tile).
  gemm  gemm_tiles_kernel on a 4096 x 4096 matrix at 256 and 512 activation rows: lane 0 of every wavefront stamps
        the boundaries of its workgroup's third stage, so the spread between a stage's first and last producer —
        what the stage barrier waits for — can be read off.

Times are microseconds of the device's 100 MHz realtime counter, relative to the first workgroup's first stamp."""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from llvq_amd import _ffi  # noqa: E402

_ffi._LIB = os.path.join(HERE, "libllvq_hip_stamps.so")

import torch  # noqa: E402

import llvq_amd  # noqa: E402
from llvq_amd import synth  # noqa: E402

GROUPS_4B = [("q/k/v", [(4096, 2560), (1024, 2560), (1024, 2560)]), ("o_proj", [(2560, 4096)]),
             ("gate/up", [(9728, 2560), (9728, 2560)]), ("down_proj", [(2560, 9728)])]


def x16(d, seed=0, rows=None):
    a = synth.make_activation(d, seed, rows=rows) if rows else synth.make_activation(d, seed)[0]
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.float16).cuda()


def upload(rt, layer, shapes):
    return [rt.upload(synth.make_matrix(f"model.layers.{layer}.p{j}.weight", do, di, layer)) for j, (do, di) in enumerate(shapes)]


def gemv(rt, L):
    L.llvq_hip_debug_phase_stamps.argtypes = [C.c_void_p, C.c_size_t]
    names = ["enters", "activation staged", "first tile begins", "operands requested (barrier)", "P1: classified and queued (barrier)",
             "P2: unranked (this wavefront)", "P2: all wavefronts (barrier)", "P3: rows stored (barrier)"]
    order = [3, 7, 0, 1, 2, 4, 5, 6]
    for name, shapes in GROUPS_4B:
        projs = upload(rt, 0, shapes)
        x = x16(shapes[0][1])
        launch, _ = rt.plan_group(projs, x)
        rows = []
        for rep in range(12):
            launch()
            torch.cuda.synchronize()
            st = np.zeros(1024 * 8, np.uint64)
            L.llvq_hip_debug_phase_stamps(st.ctypes.data, st.size)
            st = st.reshape(1024, 8)[:256].astype(np.float64)
            st = st[st[:, 6] > 0]
            rows.append((st - st[:, 3].min()) / 100.0)
        med = np.median(np.stack([np.median(r, axis=0) for r in rows[2:]]), axis=0)
        hi = np.median(np.stack([np.max(r, axis=0) for r in rows[2:]]), axis=0)
        print(f"gemv_tiles_kernel, {name} ({sum(s[0] for s in shapes)} rows of {shapes[0][1] // 24} blocks): median over workgroups [latest workgroup], us")
        for k, n in zip(order, names):
            print(f"    {n:42s} {med[k]:7.2f} [{hi[k]:6.2f}]")
        for p in projs:
            rt.free(p)


def seq(rt, L):
    L.llvq_hip_sequence_debug.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_uint32)]
    items, keep = [], []
    xs = {d: x16(d) for d in (2560, 4096, 9728)}
    for layer in range(6):
        for _, shapes in GROUPS_4B:
            projs = upload(rt, layer, shapes)
            keep.append(projs)
            items.append((projs, xs[shapes[0][1]], False))
    s = rt.plan_sequence(items)
    stamps = torch.zeros(256 * 8 * 8, dtype=torch.int64, device="cuda")
    grid = C.c_uint32()
    res = []
    for rep in range(12):
        stamps.zero_()
        L.llvq_hip_sequence_debug(s.handle, stamps.data_ptr(), C.byref(grid))
        s.run()
        s.status()
        res.append(stamps.cpu().numpy().reshape(256, 8, 8).astype(np.float64))
    L.llvq_hip_sequence_debug(s.handle, None, None)
    a = np.stack(res[2:])
    us = (a - a[:, :, 0, 0].min(axis=1)[:, None, None, None]) / 100.0
    us[a == 0] = np.nan
    names = ["begins", "previous rows stored", "(signalled)", "(wait over)", "activation staged", "queues and planes ready (barrier)",
             "unranked, next tile classified (this wavefront)", "round ends (barrier)"]
    print(f"gemv_seq_kernel, 24 independent items (six Qwen3-4B layers), grid {grid.value}: median over workgroups and runs, us;")
    print("slots in brackets are only passed in a round that changes item")
    with np.errstate(all="ignore"):
        for r in range(8):
            med = np.nanmedian(us[:, :, r, :], axis=(0, 1))
            print(f"  round {r}: " + "; ".join(f"{n} {m:.1f}" for n, m in zip(names, med) if not np.isnan(m)))
        d = us[:, :, 1:8, :]
        print(f"  per round (rounds 1-7): begin -> ready {np.nanmedian(d[..., 5] - d[..., 0]):.2f}, ready -> unranked "
              f"{np.nanmedian(d[..., 6] - d[..., 5]):.2f}, unranked -> end {np.nanmedian(d[..., 7] - d[..., 6]):.2f}")
    s.close()
    for projs in keep:
        for p in projs:
            rt.free(p)


def gemm(rt, L):
    L.llvq_hip_debug_gemm_stamps.argtypes = [C.c_void_p, C.c_size_t]
    raw = synth.make_matrix("model.layers.0.probe.weight", 4096, 4096, seed=1)
    p = rt.upload(raw)
    for M in (256, 512):
        X = x16(4096, 0, rows=M)
        Y = torch.empty((M, 4096), dtype=torch.float16, device="cuda")
        pw = 12 if M <= 256 else 8
        out = []
        for rep in range(10):
            rt.forward_batched_into(p, X, Y)
            torch.cuda.synchronize()
            st = np.zeros(1024 * 16 * 4, np.uint64)
            L.llvq_hip_debug_gemm_stamps(st.ctypes.data, st.size)
            st = st.reshape(1024, 16, 4)[:256].astype(np.float64)
            ok = st[:, 0, 3] > 0
            out.append(((st - st[:, :1, :1]) / 100.0)[ok])  # relative to the workgroup's wavefront 0 at the stage's start
        a = np.concatenate(out[2:])
        prod, cons = a[:, :pw, :], a[:, pw:, :]
        print(f"gemm_tiles_kernel, 4096 x 4096, M = {M} ({pw} producer and {16 - pw} consumer wavefronts), stage 3 of every workgroup, us after the stage began:")
        print(f"    producers: share of the slice unranked   first {np.median(prod[:, :, 1].min(1)):5.2f}  median {np.median(prod[:, :, 1]):5.2f}  last {np.median(prod[:, :, 1].max(1)):5.2f}")
        print(f"               next slice classified         first {np.median(prod[:, :, 2].min(1)):5.2f}  median {np.median(prod[:, :, 2]):5.2f}  last {np.median(prod[:, :, 2].max(1)):5.2f}")
        print(f"    consumers: K-steps multiplied            first {np.median(cons[:, :, 1].min(1)):5.2f}  median {np.median(cons[:, :, 1]):5.2f}  last {np.median(cons[:, :, 1].max(1)):5.2f}")
        print(f"    stage ends (through the barrier)         {np.median(a[:, :, 3].max(1)):5.2f}")
        busy = (prod[:, :, 2].sum(1) + cons[:, :, 1].sum(1)) / (16 * a[:, :, 3].max(1))
        print(f"    wavefront-time spent before the barrier wait: {100 * np.median(busy):.0f} % of 16 wavefronts x stage")
    rt.free(p)


def main():
    which = sys.argv[1] if len(sys.argv) > 1 else ""
    if which not in ("gemv", "seq", "gemm"):
        raise SystemExit(__doc__)
    if not os.path.exists(_ffi._LIB):
        raise SystemExit(f"{_ffi._LIB} is missing: make -C {HERE} libllvq_hip_stamps.so")
    rt = llvq_amd.FusedRuntime(device=0)
    {"gemv": gemv, "seq": seq, "gemm": gemm}[which](rt, _ffi.lib())
    rt.close()


if __name__ == "__main__":
    main()
