"""The quantized-linear operator, host side.

Mirrors the reference's `FusedMatrix` / `fused::load` (llvq-llm/src/fused.rs:566-588,
:1147) and `FusedProj` / `FusedRuntime::{new, rotate, forward_rotated}`
(llvq-llm/src/fused_cuda.rs:119-134, :182, :362, :384) over the C ABI of
include/llvq_hip.h.  torch is used for device buffers and the stream only.
Refusals name the projection, as the reference's do; nothing here computes.
"""
import ctypes as C

import numpy as np

from . import _ffi
from .artifact import RawMatrix, read_header, read_matrix_raw, read_sealed


class FusedMatrix:
    """One projection ready to upload (fused.rs:566-588).  The payload is the
    file's own code stream; there is no load-time transcode on this path."""

    def __init__(self, raw: RawMatrix):
        # one gain bit is compiled into the kernels (fused.rs:1168-1177)
        if raw.centroids.size != 2:
            raise ValueError(f"{raw.name}: {raw.centroids.size} centroids, but the kernels hard-code 1 gain bit")
        self.raw = raw
        self.name = raw.name
        self.d_out, self.d_in = raw.d_out, raw.d_in
        self.nblocks, self.tail_w = raw.nblocks, raw.tail_w
        self.gscale = raw.centroids.astype(np.float32)
        self.rscale = raw.row_scales.astype(np.float32)
        self.tail = raw.tail
        self.rotation = None if raw.rotation_seed is None else (raw.d_in, raw.rotation_seed)
        self.bytes = raw.codes.size + 4 * raw.tail.size + 4 * raw.d_out + 8


EMBED_NAME = "model.embed_tokens.weight"  # fused.rs:204
HEAD_NAME = "lm_head.weight"              # fused.rs:209


class FusedModel:
    """Everything a runtime needs, still on the host (fused.rs:723-752): the
    projections, the carried raw tensors in the file's own encoding (f16 bits, or
    int8 g64 for an embedding), config.json and tokenizer.json."""

    def __init__(self, matrices, raw=(), config_json=b"", tokenizer_json=b""):
        self.matrices = list(matrices)
        self.raw = list(raw)
        self.config_json, self.tokenizer_json = bytes(config_json), bytes(tokenizer_json)
        self.runtime_bytes = sum(m.bytes for m in self.matrices)
        self.quantized_weights = sum(m.d_out * m.d_in for m in self.matrices)
        self.carried_weights = sum(len(t) for t in self.raw)

    def tensor(self, name):
        for t in self.raw:
            if t.name == name:
                return t
        raise KeyError(f"the file carries no {name}")


def load(path: str) -> FusedModel:
    """fused::load (fused.rs:1147): header, every matrix record, the raw tensors and
    the blobs; host only.  A projections-only file (format v1) is refused, as is a
    file without config.json or tokenizer.json (fused.rs:1151-1158, :1249-1254)."""
    with open(path, "rb") as f:
        buf = f.read()
    return load_bytes(buf, path)


def load_bytes(buf, path="<bytes>", projections_only=False) -> FusedModel:
    if projections_only:
        _version, n, pos = read_header(buf)
        mats = []
        for _ in range(n):
            raw, pos = read_matrix_raw(buf, pos)
            mats.append(FusedMatrix(raw))
        return FusedModel(mats)
    version, mats, raws, blobs = read_sealed(buf)
    if version < 2:
        raise ValueError(f"{path} is a projections-only artifact (format v{version}); it cannot run on its own")
    by_name = {b.name: b.data for b in blobs}
    for need in ("config.json", "tokenizer.json"):
        if need not in by_name:
            raise ValueError(f"{path} carries no {need}")
    return FusedModel([FusedMatrix(m) for m in mats], raws, by_name["config.json"], by_name["tokenizer.json"])


class FusedProj:
    """One projection's weights on the device (fused_cuda.rs:119-134)."""

    def __init__(self, rt, handle, fm: FusedMatrix):
        self._rt = rt
        self.handle = handle
        self.name = fm.name
        self.d_out, self.d_in = fm.d_out, fm.d_in
        self.nblocks, self.tail_w = fm.nblocks, fm.tail_w
        self._rotation = fm.rotation
        self.encoded_bytes = fm.raw.encoded_bytes()

    def rotation(self):
        return self._rotation


class FusedSequence:
    """A bound list of group products that runs as one persistent kernel (no counterpart in the reference,
    whose FusedOp launches per projection, fused_cuda.rs:758-900)."""

    def __init__(self, rt, handle, outputs, keep):
        self._rt, self.handle, self.outputs, self._keep = rt, handle, outputs, keep
        self._run = _ffi.lib().llvq_hip_sequence_run

    def run(self):
        """Enqueues the whole list on the runtime's stream."""
        rc = self._run(self._rt.handle, self.handle)
        if rc:
            _ffi.check(rc)

    def status(self):
        """Waits for the stream; raises LlvqError(Device) if a workgroup of an earlier run gave up waiting."""
        _ffi.check(_ffi.lib().llvq_hip_sequence_status(self._rt.handle, self.handle))

    def tune(self, spin_limit=0, hold_item=-1):
        _ffi.check(_ffi.lib().llvq_hip_sequence_tune(self.handle, spin_limit, hold_item))

    def close(self):
        if self.handle:
            _ffi.lib().llvq_hip_sequence_destroy(self._rt.handle, self.handle)
            self.handle = None


class FusedRuntime:
    """Tables and stream (fused_cuda.rs:145-180).  `FusedRuntime(model, device)`
    is `FusedRuntime::new`: it returns with every projection uploaded in `projs`."""

    def __init__(self, model: FusedModel = None, device: int = 0, stream=None):
        import torch

        self._torch = torch
        self.device = torch.device("cuda", device)
        L = _ffi.lib()
        if stream is None:
            stream = torch.cuda.current_stream(self.device)
        self._stream = stream
        h = C.c_void_p()
        _ffi.check(L.llvq_hip_runtime_create(device, C.c_void_p(stream.cuda_stream), C.byref(h)))
        self.handle = h
        self.projs = []
        if model is not None:
            for fm in model.matrices:
                self.projs.append(self.upload(fm))

    def upload(self, fm) -> FusedProj:
        if isinstance(fm, RawMatrix):
            fm = FusedMatrix(fm)
        raw = fm.raw
        d = _ffi.MatrixDesc()
        d.name = raw.name.encode()
        d.d_out, d.d_in, d.shell_cap, d.n_centroids = raw.d_out, raw.d_in, raw.shell_cap, raw.centroids.size
        d.centroids = raw.centroids.ctypes.data
        d.row_scales = raw.row_scales.ctypes.data
        d.tail = raw.tail.ctypes.data if raw.tail.size else None
        codes = np.ascontiguousarray(raw.codes)
        d.codes = codes.ctypes.data
        d.code_bytes = codes.size
        d.rotation_seed = raw.rotation_seed or 0
        d.has_rotation = 1 if raw.rotation_seed is not None else 0
        h = C.c_void_p()
        _ffi.check(_ffi.lib().llvq_hip_matrix_upload(self.handle, C.byref(d), C.byref(h)))
        return FusedProj(self, h, fm)

    def upload_record(self, buf, pos=0):
        """Parse one on-disk record with the library's own reader and upload it."""
        p = C.c_size_t(pos)
        h = C.c_void_p()
        _ffi.check(_ffi.lib().llvq_hip_matrix_from_record(self.handle, bytes(buf), len(buf), C.byref(p), C.byref(h)))
        raw, _ = read_matrix_raw(buf, pos)
        return FusedProj(self, h, FusedMatrix(raw)), p.value

    def free(self, proj: FusedProj):
        if proj.handle:
            _ffi.lib().llvq_hip_matrix_free(self.handle, proj.handle)
            proj.handle = None

    # -- the operator ---------------------------------------------------------------
    def _f16(self, x, proj):
        torch = self._torch
        if not x.is_cuda:
            raise ValueError("the fused LLVQ kernel has no CPU path")
        if x.shape[-1] != proj.d_in:
            raise ValueError(f"{proj.name} expects d_in={proj.d_in}, got {x.shape[-1]}")
        return x.to(torch.float16).contiguous()

    def _out_code(self, dtype):
        """The kernels store binary16 or f32 outputs and nothing else: any other dtype would be
        written with the wrong element size."""
        torch = self._torch
        if dtype == torch.float16:
            return _ffi.F16
        if dtype == torch.float32:
            return _ffi.F32
        raise ValueError(f"outputs are torch.float16 or torch.float32, not {dtype}")

    def rotate(self, proj: FusedProj, x):
        """FusedRuntime::rotate (fused_cuda.rs:362): one f16 activation [.., d_in] into the
        basis the projection was quantized in, as f32 [1, d_in].  Natural-basis matrices
        only widen it."""
        torch = self._torch
        x = self._f16(x, proj)
        rows = x.numel() // proj.d_in
        if rows != 1:
            raise ValueError(f"{proj.name}: rotation asked for {rows} vectors; the row loop belongs to the caller")
        xr = torch.empty((1, proj.d_in), dtype=torch.float32, device=x.device)
        _ffi.check(_ffi.lib().llvq_hip_rotate(self.handle, proj.handle, x.data_ptr(), xr.data_ptr()))
        return xr

    def forward_rotated(self, proj: FusedProj, xr, out_dims=None, out_dtype=None):
        """FusedRuntime::forward_rotated (fused_cuda.rs:384): y = W' xr for `rotate`'s f32
        output, shaped like the caller's tensor with the last dim replaced by d_out.
        f16 out by default."""
        torch = self._torch
        if not xr.is_cuda:
            raise ValueError("the fused LLVQ kernel has no CPU path")
        if not xr.is_contiguous():
            raise ValueError("activation is not contiguous")
        if xr.dtype != torch.float32:
            raise ValueError(f"{proj.name}: a rotated activation is f32, got {xr.dtype}")
        if xr.numel() != proj.d_in:
            raise ValueError(f"rotated activation of {xr.numel()} values for d_in={proj.d_in}")
        out_dtype = out_dtype or torch.float16
        dims = list(out_dims if out_dims is not None else xr.shape)
        dims[-1] = proj.d_out
        y = torch.empty(dims, dtype=out_dtype, device=xr.device)  # uninitialised: every row is stored
        code = self._out_code(out_dtype)
        _ffi.check(_ffi.lib().llvq_hip_gemv_rotated(self.handle, proj.handle, xr.data_ptr(), y.data_ptr(), code))
        return y

    def forward(self, proj: FusedProj, x, out_dtype=None):
        """Proj::forward (model.rs:337-345): rotate + forward_rotated in one call."""
        torch = self._torch
        x = self._f16(x, proj)
        if x.numel() != proj.d_in:
            raise ValueError(f"{proj.name}: one activation of {proj.d_in} values expected, got {x.numel()}")
        out_dtype = out_dtype or torch.float16
        dims = list(x.shape)
        dims[-1] = proj.d_out
        y = torch.empty(dims, dtype=out_dtype, device=x.device)
        code = self._out_code(out_dtype)
        _ffi.check(_ffi.lib().llvq_hip_gemv(self.handle, proj.handle, x.data_ptr(), y.data_ptr(), code))
        return y

    def forward_group(self, projs, x, out_dtype=None):
        """group_forward (llvq-llm/src/model.rs:497-536) for projections sharing one activation."""
        launch, ys = self.plan_group(projs, x, out_dtype)
        launch()
        return ys

    def plan_group(self, projs, x, out_dtype=None):
        """Pre-binds one group call: returns (launch, outputs).  `launch()` enqueues the
        group's GEMV on the runtime's stream with no Python-side allocation or
        argument marshalling — what a decode loop calls once per token."""
        torch = self._torch
        x = self._f16(x, projs[0])
        out_dtype = out_dtype or torch.float16
        ys = [torch.empty(list(x.shape[:-1]) + [p.d_out], dtype=out_dtype, device=x.device) for p in projs]
        mats = (C.c_void_p * len(projs))(*[p.handle for p in projs])
        outs = (C.c_void_p * len(projs))(*[y.data_ptr() for y in ys])
        code = self._out_code(out_dtype)
        fn = _ffi.lib().llvq_hip_gemv_group
        rt, n, xp = self.handle, len(projs), C.c_void_p(x.data_ptr())
        keep = (x, ys, mats, outs)

        def launch(_keep=keep):
            rc = fn(rt, mats, n, xp, outs, code)
            if rc:
                _ffi.check(rc)

        return launch, ys

    def plan_sequence(self, items, out_dtype=None):
        """Binds a list of group products as ONE launch (llvq_hip_sequence_create).  `items` is a list of
        (projections, activation, after_previous[, outputs]): `activation` is an f16 device tensor of d_in
        values; after_previous = True says the activation is (or depends on) an output of the item before it;
        `outputs`, when given, are the caller's own result tensors of `out_dtype` (so that a later item can be
        bound to them).  Returns a FusedSequence; its `outputs[i]` are item i's result tensors."""
        torch = self._torch
        out_dtype = out_dtype or torch.float16
        code = self._out_code(out_dtype)
        n = len(items)
        arr = (_ffi.SeqItem * n)()
        keep, outputs = [], []
        for i, item in enumerate(items):
            projs, x, after = item[0], item[1], item[2]
            x = self._f16(x, projs[0])
            ys = item[3] if len(item) > 3 and item[3] is not None else \
                [torch.empty(list(x.shape[:-1]) + [p.d_out], dtype=out_dtype, device=x.device) for p in projs]
            for y, p in zip(ys, projs):
                if y.dtype != out_dtype or y.numel() != p.d_out or not y.is_contiguous():
                    raise ValueError(f"{p.name}: output must be a contiguous {out_dtype} tensor of {p.d_out} values")
            mats = (C.c_void_p * len(projs))(*[p.handle for p in projs])
            outs = (C.c_void_p * len(projs))(*[y.data_ptr() for y in ys])
            arr[i].mats, arr[i].n_mats, arr[i].x_f16_dev = mats, len(projs), x.data_ptr()
            arr[i].y_dev, arr[i].y_dtype, arr[i].after_previous = outs, code, 1 if after else 0
            keep.append((x, ys, mats, outs))
            outputs.append(ys)
        handle = C.c_void_p()
        _ffi.check(_ffi.lib().llvq_hip_sequence_create(self.handle, arr, n, C.byref(handle)))
        return FusedSequence(self, handle, outputs, keep)

    def forward_batched(self, proj: FusedProj, x, out_dtype=None):
        """Rows of `x` [M, d_in] through one projection (the row loop of model.rs:521-529)."""
        torch = self._torch
        if x.dim() != 2 or x.shape[1] != proj.d_in:
            raise ValueError(f"{proj.name} expects [M, {proj.d_in}], got {list(x.shape)}")
        x = x.to(torch.float16).contiguous()
        out_dtype = out_dtype or torch.float16
        y = torch.empty((x.shape[0], proj.d_out), dtype=out_dtype, device=x.device)
        code = self._out_code(out_dtype)
        _ffi.check(_ffi.lib().llvq_hip_gemm(self.handle, proj.handle, x.data_ptr(), x.shape[0], y.data_ptr(), code))
        return y

    def forward_batched_into(self, proj: FusedProj, x, y):
        """`forward_batched` into a caller-owned [M, d_out] f16/f32 tensor (no allocation per call)."""
        torch = self._torch
        if x.dtype != torch.float16 or not x.is_contiguous() or x.shape[1] != proj.d_in:
            raise ValueError(f"{proj.name} expects a contiguous f16 [M, {proj.d_in}] activation")
        if tuple(y.shape) != (x.shape[0], proj.d_out) or not y.is_contiguous():
            raise ValueError(f"{proj.name}: output must be contiguous [M, {proj.d_out}]")
        code = self._out_code(y.dtype)
        _ffi.check(_ffi.lib().llvq_hip_gemm(self.handle, proj.handle, x.data_ptr(), x.shape[0], y.data_ptr(), code))
        return y

    def reserve_batched(self, projs, max_rows: int):
        """Sizes the runtime's batched-path workspaces for `forward_batched*` calls over this group with up
        to max_rows rows, so that those calls allocate nothing and return without synchronising."""
        mats = (C.c_void_p * len(projs))(*[p.handle for p in projs])
        _ffi.check(_ffi.lib().llvq_hip_reserve_batched(self.handle, mats, len(projs), int(max_rows)))

    def forward_batched_static_into(self, proj: FusedProj, x, y):
        """`forward_batched_into` through llvq_hip_gemm_static: the call allocates no device memory
        (its workspaces are a static device array); shapes beyond that array raise Unsupported."""
        torch = self._torch
        if x.dtype != torch.float16 or not x.is_contiguous() or x.dim() != 2 or x.shape[1] != proj.d_in:
            raise ValueError(f"{proj.name} expects a contiguous f16 [M, {proj.d_in}] activation")
        if tuple(y.shape) != (x.shape[0], proj.d_out) or not y.is_contiguous():
            raise ValueError(f"{proj.name}: output must be contiguous [M, {proj.d_out}]")
        code = self._out_code(y.dtype)
        _ffi.check(_ffi.lib().llvq_hip_gemm_static(self.handle, proj.handle, x.data_ptr(), x.shape[0], y.data_ptr(), code))
        return y

    def forward_batched_group_into(self, projs, x, ys):
        """Rows of `x` [M, d_in] through the projections of one group (q/k/v, gate/up) into caller-owned
        [M, d_out_i] tensors of one dtype: one batched launch per run of projections that share a basis
        (the row loop of group_forward, model.rs:497-536)."""
        torch = self._torch
        if len(projs) != len(ys) or not projs:
            raise ValueError("one output per projection")
        if x.dtype != torch.float16 or not x.is_contiguous() or x.dim() != 2:
            raise ValueError("the activation must be a contiguous f16 [M, d_in] tensor")
        for p, y in zip(projs, ys):
            if p.d_in != x.shape[1]:
                raise ValueError(f"{p.name} expects d_in {p.d_in}, got {x.shape[1]}")
            if tuple(y.shape) != (x.shape[0], p.d_out) or not y.is_contiguous() or y.dtype != ys[0].dtype:
                raise ValueError(f"{p.name}: output must be contiguous [M, {p.d_out}], one dtype for the group")
        mats = (C.c_void_p * len(projs))(*[p.handle for p in projs])
        outs = (C.c_void_p * len(projs))(*[y.data_ptr() for y in ys])
        code = self._out_code(ys[0].dtype)
        _ffi.check(_ffi.lib().llvq_hip_gemm_group(self.handle, mats, len(projs), x.data_ptr(), x.shape[0], outs, code))
        return ys

    def decode_blocks(self, codes):
        """Parity probe: packed 6-byte records (uint8 tensor on the device) →
        (points int8 [n,24], gains uint8 [n], shells uint8 [n])."""
        torch = self._torch
        n = codes.numel() // 6
        pts = torch.empty((n, 24), dtype=torch.int8, device=codes.device)
        gains = torch.empty(n, dtype=torch.uint8, device=codes.device)
        shells = torch.empty(n, dtype=torch.uint8, device=codes.device)
        _ffi.check(_ffi.lib().llvq_hip_decode_blocks(self.handle, codes.data_ptr(), n, pts.data_ptr(),
                                                      gains.data_ptr(), shells.data_ptr()))
        return pts, gains, shells

    def decode_stream(self, codes, nblocks: int, shell_cap: int):
        """`decode_blocks` for the code stream of any accepted shell cap (cap 13: 49 bits per block, dense)."""
        torch = self._torch
        n = int(nblocks)
        pts = torch.empty((n, 24), dtype=torch.int8, device=codes.device)
        gains = torch.empty(n, dtype=torch.uint8, device=codes.device)
        shells = torch.empty(n, dtype=torch.uint8, device=codes.device)
        _ffi.check(_ffi.lib().llvq_hip_decode_stream(self.handle, codes.data_ptr(), n, int(shell_cap), pts.data_ptr(),
                                                      gains.data_ptr(), shells.data_ptr()))
        return pts, gains, shells

    def synchronize(self):
        _ffi.check(_ffi.lib().llvq_hip_synchronize(self.handle))

    def close(self):
        if self.handle:
            for p in self.projs:
                self.free(p)
            _ffi.lib().llvq_hip_runtime_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
