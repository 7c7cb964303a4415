//! llvq-hip: the quantized-linear operator of `llvq-llm` on an MI355X.
//!
//! A thin layer over `include/llvq_hip.h` (libllvq_hip.so).  `HipRuntime` stands where
//! `FusedRuntime` stands (llvq-llm/src/fused_cuda.rs:145-180), `HipProj` where `FusedProj`
//! does (fused_cuda.rs:119-134); the model runner reaches them through one more arm of
//! `Proj` (llvq-llm/src/model.rs:265-272, see llvq-llm.patch).  Device pointers are raw
//! `*mut c_void`: the tensor runtime that owns the activations hands them over, as candle's
//! `CustomOp` does for the CUDA arm (fused_cuda.rs:758-900).
//!
//! Nothing here decodes, transcodes or copies weights on the host: the archive's 6-byte
//! records go to the device verbatim and are unranked by the kernels.
#![allow(clippy::missing_safety_doc)]

use std::ffi::{c_char, c_int, c_void, CStr, CString};
use std::sync::Arc;

#[repr(C)]
pub struct LlvqRt {
    _p: [u8; 0],
}
#[repr(C)]
pub struct LlvqMat {
    _p: [u8; 0],
}
#[repr(C)]
pub struct LlvqDecoder {
    _p: [u8; 0],
}
#[repr(C)]
pub struct LlvqSeq {
    _p: [u8; 0],
}

/// llvq_seq_item: one group product of a sequence (what one llvq_hip_gemv_group call would be)
#[repr(C)]
pub struct LlvqSeqItem {
    pub mats: *const *const LlvqMat,
    pub n_mats: c_int,
    pub x_f16_dev: *const c_void,
    pub y_dev: *const *mut c_void,
    pub y_dtype: c_int,
    pub after_previous: c_int,
}

/// llvq_matrix_desc
#[repr(C)]
pub struct LlvqMatrixDesc {
    pub name: *const c_char,
    pub d_out: u32,
    pub d_in: u32,
    pub shell_cap: u32,
    pub n_centroids: u32,
    pub centroids: *const f64,
    pub row_scales: *const f64,
    pub tail: *const f32,
    pub codes: *const u8,
    pub code_bytes: usize,
    pub rotation_seed: u64,
    pub has_rotation: u32,
}

/// llvq_record_info
#[repr(C)]
pub struct LlvqRecordInfo {
    pub name: [c_char; 256],
    pub d_out: u32,
    pub d_in: u32,
    pub shell_cap: u32,
    pub n_centroids: u32,
    pub rotation_seed: u64,
    pub has_rotation: u32,
    pub centroids_off: usize,
    pub row_scales_off: usize,
    pub tail_off: usize,
    pub codes_off: usize,
    pub code_bytes: usize,
}

/// llvq_raw_info
#[repr(C)]
pub struct LlvqRawInfo {
    pub name: [c_char; 256],
    pub rank: u32,
    pub dims: [u64; 8],
    pub tag: u32,
    pub bits: u32,
    pub group: u32,
    pub count: u64,
    pub data_off: usize,
    pub data_len: usize,
    pub scales_off: usize,
    pub biases_off: usize,
}

/// llvq_blob_info
#[repr(C)]
pub struct LlvqBlobInfo {
    pub name: [c_char; 256],
    pub data_off: usize,
    pub data_len: usize,
}

/// llvq_quant_rows
#[repr(C)]
#[derive(Clone, Copy)]
pub struct LlvqQuantRows {
    pub codes: *const u8,
    pub scales: *const u16,
    pub biases: *const u16,
    pub bits: u32,
    pub group: u32,
}

/// llvq_decoder_desc
#[repr(C)]
pub struct LlvqDecoderDesc {
    pub n_layers: u32,
    pub hidden: u32,
    pub n_heads: u32,
    pub n_kv_heads: u32,
    pub head_dim: u32,
    pub intermediate: u32,
    pub vocab: u32,
    pub max_positions: u32,
    pub rope_theta: f64,
    pub rms_eps: f64,
    pub projections: *const *const LlvqMat,
    pub input_norm: *const u16,
    pub post_norm: *const u16,
    pub q_norm: *const u16,
    pub k_norm: *const u16,
    pub final_norm: *const u16,
    pub embed: *const u16,
    pub lm_head: *const u16,
    pub kv_mode: u32,
    pub embed_q8: LlvqQuantRows,
    pub lm_head_q8: LlvqQuantRows,
    pub prefill_rows: u32,
    pub launch_mode: u32,
}

pub const LLVQ_F32: c_int = 0;
pub const LLVQ_F16: c_int = 1;
pub const LLVQ_KV_F16: u32 = 0;
pub const LLVQ_KV_Q8: u32 = 1;
/// LLVQ_STATIC_SCRATCH_BYTES
pub const STATIC_SCRATCH_BYTES: usize = 64 << 20;

extern "C" {
    pub fn llvq_hip_runtime_create(device: c_int, hip_stream: *mut c_void, out: *mut *mut LlvqRt) -> c_int;
    pub fn llvq_hip_runtime_destroy(rt: *mut LlvqRt);
    pub fn llvq_hip_codebook_fingerprint() -> u64;
    pub fn llvq_hip_host_decode(idx: u64, point: *mut i8, shell: *mut c_int) -> c_int;
    pub fn llvq_hip_matrix_upload(rt: *mut LlvqRt, desc: *const LlvqMatrixDesc, out: *mut *mut LlvqMat) -> c_int;
    pub fn llvq_hip_read_header(buf: *const u8, len: usize, pos: *mut usize, version: *mut u32, n_matrices: *mut u32) -> c_int;
    pub fn llvq_hip_parse_matrix_record(buf: *const u8, len: usize, pos: *mut usize, out: *mut LlvqRecordInfo) -> c_int;
    pub fn llvq_hip_matrix_from_record(rt: *mut LlvqRt, buf: *const u8, len: usize, pos: *mut usize, out: *mut *mut LlvqMat) -> c_int;
    pub fn llvq_hip_matrix_free(rt: *mut LlvqRt, m: *mut LlvqMat);
    pub fn llvq_hip_parse_raw_tensor(buf: *const u8, len: usize, pos: *mut usize, version: u32, out: *mut LlvqRawInfo) -> c_int;
    pub fn llvq_hip_parse_blob(buf: *const u8, len: usize, pos: *mut usize, out: *mut LlvqBlobInfo) -> c_int;
    pub fn llvq_hip_matrix_info(m: *const LlvqMat, d_out: *mut u32, d_in: *mut u32, nblocks: *mut u32, tail_w: *mut u32, device_bytes: *mut u64) -> c_int;
    pub fn llvq_hip_matrix_name(m: *const LlvqMat) -> *const c_char;
    pub fn llvq_hip_gemv(rt: *mut LlvqRt, m: *const LlvqMat, x_f16_dev: *const c_void, y_dev: *mut c_void, y_dtype: c_int) -> c_int;
    pub fn llvq_hip_rotate(rt: *mut LlvqRt, m: *const LlvqMat, x_f16_dev: *const c_void, xr_f32_dev: *mut f32) -> c_int;
    pub fn llvq_hip_gemv_rotated(rt: *mut LlvqRt, m: *const LlvqMat, xr_f32_dev: *const f32, y_dev: *mut c_void, y_dtype: c_int) -> c_int;
    pub fn llvq_hip_host_rotate(n: u32, seed: u64, v: *mut f64) -> c_int;
    pub fn llvq_hip_matrix_rotation(m: *const LlvqMat, has_rotation: *mut u32, seed: *mut u64) -> c_int;
    pub fn llvq_hip_gemv_group(rt: *mut LlvqRt, mats: *const *const LlvqMat, n: c_int, x_f16_dev: *const c_void, y_dev: *const *mut c_void, y_dtype: c_int) -> c_int;
    pub fn llvq_hip_sequence_create(rt: *mut LlvqRt, items: *const LlvqSeqItem, n_items: c_int, out: *mut *mut LlvqSeq) -> c_int;
    pub fn llvq_hip_sequence_run(rt: *mut LlvqRt, seq: *mut LlvqSeq) -> c_int;
    pub fn llvq_hip_sequence_status(rt: *mut LlvqRt, seq: *mut LlvqSeq) -> c_int;
    pub fn llvq_hip_sequence_destroy(rt: *mut LlvqRt, seq: *mut LlvqSeq);
    pub fn llvq_hip_sequence_tune(seq: *mut LlvqSeq, spin_limit: u32, hold_item: c_int) -> c_int;
    pub fn llvq_hip_gemm(rt: *mut LlvqRt, m: *const LlvqMat, x_f16_dev: *const c_void, rows: c_int, y_dev: *mut c_void, y_dtype: c_int) -> c_int;
    pub fn llvq_hip_gemm_group(rt: *mut LlvqRt, mats: *const *const LlvqMat, n: c_int, x_f16_dev: *const c_void, rows: c_int, y_dev: *const *mut c_void, y_dtype: c_int) -> c_int;
    pub fn llvq_hip_reserve_batched(rt: *mut LlvqRt, mats: *const *const LlvqMat, n: c_int, max_rows: c_int) -> c_int;
    pub fn llvq_hip_gemm_static(rt: *mut LlvqRt, m: *const LlvqMat, x_f16_dev: *const c_void, rows: c_int, y_dev: *mut c_void, y_dtype: c_int) -> c_int;
    pub fn llvq_hip_decode_blocks(rt: *mut LlvqRt, codes_dev: *const u8, nblocks: usize, points_dev: *mut i8, gains_dev: *mut u8, shells_dev: *mut u8) -> c_int;
    pub fn llvq_hip_decode_stream(rt: *mut LlvqRt, codes_dev: *const u8, nblocks: usize, shell_cap: u32, points_dev: *mut i8, gains_dev: *mut u8, shells_dev: *mut u8) -> c_int;
    pub fn llvq_hip_decoder_create(rt: *mut LlvqRt, desc: *const LlvqDecoderDesc, out: *mut *mut LlvqDecoder) -> c_int;
    pub fn llvq_hip_decoder_destroy(dec: *mut LlvqDecoder);
    pub fn llvq_hip_decoder_reset(dec: *mut LlvqDecoder) -> c_int;
    pub fn llvq_hip_decoder_position(dec: *const LlvqDecoder) -> c_int;
    pub fn llvq_hip_decoder_seek(dec: *mut LlvqDecoder, position: u32) -> c_int;
    pub fn llvq_hip_decoder_forward_token(dec: *mut LlvqDecoder, token: u32, logits_host: *mut f32, argmax_host: *mut u32) -> c_int;
    pub fn llvq_hip_decoder_generate(dec: *mut LlvqDecoder, prompt: *const u32, n_prompt: usize, max_new: usize, out: *mut u32) -> c_int;
    pub fn llvq_hip_decoder_prefill(dec: *mut LlvqDecoder, tokens: *const u32, n: usize, logits_host: *mut f32, argmax_host: *mut u32) -> c_int;
    pub fn llvq_hip_decoder_generate_prefilled(dec: *mut LlvqDecoder, prompt: *const u32, n_prompt: usize, max_new: usize, out: *mut u32) -> c_int;
    pub fn llvq_hip_decoder_generate_phased(dec: *mut LlvqDecoder, prompt: *const u32, n_prompt: usize, max_new: usize, out: *mut u32, phase_ms: *mut f64) -> c_int;
    pub fn llvq_hip_synchronize(rt: *mut LlvqRt) -> c_int;
    pub fn llvq_hip_last_error() -> *const c_char;
    pub fn llvq_hip_version() -> *const c_char;
}

fn check(rc: c_int) -> Result<(), String> {
    if rc == 0 {
        return Ok(());
    }
    // SAFETY: the library returns a NUL-terminated string owned by the calling thread
    Err(unsafe { CStr::from_ptr(llvq_hip_last_error()) }.to_string_lossy().into_owned())
}

/// The rotation a projection's weights were stored under: (d_in, seed) — `RotKey`
/// (llvq-llm/src/fused.rs:672-674).
pub type RotKey = (usize, u64);

/// Owns the device tables; every projection uploaded through it is freed with it.
pub struct HipRuntime {
    rt: *mut LlvqRt,
}

// The runtime and its matrices are immutable after construction and the library takes launches
// from one thread at a time — the contract `Arc<FusedRuntime>` is shared under (model.rs:268-271).
unsafe impl Send for HipRuntime {}
unsafe impl Sync for HipRuntime {}

/// One uploaded projection.  Keeps its runtime alive.
pub struct HipProj {
    pub name: String,
    pub d_out: usize,
    pub d_in: usize,
    pub rotation: Option<RotKey>,
    mat: *mut LlvqMat,
    rt: Arc<HipRuntime>,
}
unsafe impl Send for HipProj {}
unsafe impl Sync for HipProj {}

impl HipRuntime {
    /// FusedRuntime::new (fused_cuda.rs:182).  `stream` is the hipStream_t the tensor runtime
    /// orders its work on (null = the device's default stream).  Fails unless the library's
    /// index map reproduces the published codebook fingerprint.
    pub fn new(device: i32, stream: *mut c_void) -> Result<Arc<Self>, String> {
        let theirs = llvq_artifact::codebook_fingerprint();
        // SAFETY: no arguments, no device needed
        let ours = unsafe { llvq_hip_codebook_fingerprint() };
        if ours != theirs {
            return Err(format!("codebook fingerprint {ours:#018x}, llvq-artifact has {theirs:#018x}"));
        }
        let mut rt = std::ptr::null_mut();
        check(unsafe { llvq_hip_runtime_create(device, stream, &mut rt) })?;
        Ok(Arc::new(Self { rt }))
    }

    /// upload_matrix (fused_cuda.rs:1058): `m` as `llvq_artifact::read_matrix_raw` returned it,
    /// `codes` the record's packed stream exactly as the file holds it.
    pub fn upload(self: &Arc<Self>, m: &llvq_artifact::RawMatrix, codes: &[u8]) -> Result<HipProj, String> {
        let tail: Vec<f32> = m.tail.iter().map(|&t| t as f32).collect();
        let name = CString::new(m.name.clone()).map_err(|e| e.to_string())?;
        let d = LlvqMatrixDesc {
            name: name.as_ptr(),
            d_out: m.d_out as u32,
            d_in: m.d_in as u32,
            shell_cap: m.shell_cap,
            n_centroids: m.centroids.len() as u32,
            centroids: m.centroids.as_ptr(),
            row_scales: m.row_scales.as_ptr(),
            tail: tail.as_ptr(),
            codes: codes.as_ptr(),
            code_bytes: codes.len(),
            rotation_seed: m.rotation_seed.unwrap_or(0),
            has_rotation: m.rotation_seed.is_some() as u32,
        };
        let mut mat = std::ptr::null_mut();
        check(unsafe { llvq_hip_matrix_upload(self.rt, &d, &mut mat) })?;
        Ok(HipProj {
            name: m.name.clone(),
            d_out: m.d_out,
            d_in: m.d_in,
            rotation: m.rotation_seed.map(|s| (m.d_in, s)),
            mat,
            rt: Arc::clone(self),
        })
    }

    /// The same from the file's bytes: parses the record at `buf[*pos..]` (the refusals of
    /// format.rs:301-382) and uploads it without unpacking the stream on the host.
    pub fn upload_record(self: &Arc<Self>, buf: &[u8], pos: &mut usize) -> Result<HipProj, String> {
        let mut info = std::mem::MaybeUninit::<LlvqRecordInfo>::zeroed();
        let mut probe = *pos;
        check(unsafe { llvq_hip_parse_matrix_record(buf.as_ptr(), buf.len(), &mut probe, info.as_mut_ptr()) })?;
        // SAFETY: the call succeeded, so every field is written
        let info = unsafe { info.assume_init() };
        let mut mat = std::ptr::null_mut();
        check(unsafe { llvq_hip_matrix_from_record(self.rt, buf.as_ptr(), buf.len(), pos, &mut mat) })?;
        let name = unsafe { CStr::from_ptr(info.name.as_ptr()) }.to_string_lossy().into_owned();
        Ok(HipProj {
            name,
            d_out: info.d_out as usize,
            d_in: info.d_in as usize,
            rotation: (info.has_rotation != 0).then_some((info.d_in as usize, info.rotation_seed)),
            mat,
            rt: Arc::clone(self),
        })
    }

    /// FusedRuntime::rotate (fused_cuda.rs:362): x f16 [d_in] on the device -> xr f32 [d_in] in
    /// the projection's basis.
    pub unsafe fn rotate(&self, p: &HipProj, x_f16: *const c_void, xr_f32: *mut f32) -> Result<(), String> {
        check(llvq_hip_rotate(self.rt, p.mat, x_f16, xr_f32))
    }

    /// FusedRuntime::forward_rotated (fused_cuda.rs:384): xr f32 [d_in] -> y f16 [d_out].
    pub unsafe fn forward_rotated(&self, p: &HipProj, xr_f32: *const f32, y_f16: *mut c_void) -> Result<(), String> {
        check(llvq_hip_gemv_rotated(self.rt, p.mat, xr_f32, y_f16, LLVQ_F16))
    }

    /// Proj::forward (model.rs:337-345) in one call; the launch rotates its own activation.
    pub unsafe fn forward(&self, p: &HipProj, x_f16: *const c_void, y_f16: *mut c_void) -> Result<(), String> {
        check(llvq_hip_gemv(self.rt, p.mat, x_f16, y_f16, LLVQ_F16))
    }

    /// group_forward (model.rs:497-536) for projections that share an activation (q/k/v,
    /// gate/up): one launch per run of projections in the same basis.
    pub unsafe fn forward_group(&self, ps: &[&HipProj], x_f16: *const c_void, ys_f16: &[*mut c_void]) -> Result<(), String> {
        assert_eq!(ps.len(), ys_f16.len());
        let mats: Vec<*const LlvqMat> = ps.iter().map(|p| p.mat as *const LlvqMat).collect();
        check(llvq_hip_gemv_group(self.rt, mats.as_ptr(), mats.len() as c_int, x_f16, ys_f16.as_ptr(), LLVQ_F16))
    }

    /// The l > 1 row loop of group_forward (model.rs:521-529) as one batched product on the
    /// matrix cores: Y[rows, d_out_i] = X[rows, d_in] W_i^T.
    pub unsafe fn forward_rows(&self, ps: &[&HipProj], x_f16: *const c_void, rows: usize, ys_f16: &[*mut c_void]) -> Result<(), String> {
        assert_eq!(ps.len(), ys_f16.len());
        let mats: Vec<*const LlvqMat> = ps.iter().map(|p| p.mat as *const LlvqMat).collect();
        check(llvq_hip_gemm_group(self.rt, mats.as_ptr(), mats.len() as c_int, x_f16, rows as c_int, ys_f16.as_ptr(), LLVQ_F16))
    }

    /// Sizes the batched path's workspaces for `forward_rows` over this group with up to `max_rows`
    /// rows, so that those calls allocate nothing and only enqueue.
    pub fn reserve_rows(&self, ps: &[&HipProj], max_rows: usize) -> Result<(), String> {
        let mats: Vec<*const LlvqMat> = ps.iter().map(|p| p.mat as *const LlvqMat).collect();
        check(unsafe { llvq_hip_reserve_batched(self.rt, mats.as_ptr(), mats.len() as c_int, max_rows as c_int) })
    }

    /// `forward_rows` for one projection without any device allocation inside the call
    /// (workspaces in a static device array of STATIC_SCRATCH_BYTES; larger shapes are refused).
    pub unsafe fn forward_rows_static(&self, p: &HipProj, x_f16: *const c_void, rows: usize, y_f16: *mut c_void) -> Result<(), String> {
        check(llvq_hip_gemm_static(self.rt, p.mat, x_f16, rows as c_int, y_f16, LLVQ_F16))
    }

    pub fn synchronize(&self) -> Result<(), String> {
        check(unsafe { llvq_hip_synchronize(self.rt) })
    }

    pub fn raw(&self) -> *mut LlvqRt {
        self.rt
    }
}

impl HipProj {
    pub fn raw(&self) -> *const LlvqMat {
        self.mat
    }
}

impl Drop for HipProj {
    fn drop(&mut self) {
        // SAFETY: the matrix was created by this runtime, which the Arc keeps alive
        unsafe { llvq_hip_matrix_free(self.rt.rt, self.mat) }
    }
}

impl Drop for HipRuntime {
    fn drop(&mut self) {
        // SAFETY: every HipProj holds an Arc to the runtime, so none outlives it
        unsafe { llvq_hip_runtime_destroy(self.rt) }
    }
}

/// The library's own decoder on the host (the arithmetic the kernels run): what a
/// `cargo test` compares with `llvq_search::Indexer::decode` before any device exists.
pub fn host_decode(idx: u64) -> Option<([i8; 24], i32)> {
    let mut p = [0i8; 24];
    let mut shell: c_int = 0;
    // SAFETY: both outputs are sized as the header asks
    let ok = unsafe { llvq_hip_host_decode(idx, p.as_mut_ptr(), &mut shell) };
    (ok == 1).then_some((p, shell))
}

#[cfg(all(test, feature = "link"))]
mod tests {
    use super::*;

    #[test]
    fn fingerprint_is_the_published_one() {
        assert_eq!(unsafe { llvq_hip_codebook_fingerprint() }, 0x338f_420f_1186_6319);
    }

    #[test]
    fn host_decoder_knows_the_first_point() {
        let (p, shell) = host_decode(1).unwrap();
        assert_eq!(&p[..3], &[4, 4, 0]);
        assert_eq!(shell, 2);
        assert!(host_decode(280_974_212_784_721).is_none());
    }
}
