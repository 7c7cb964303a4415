"""ctypes binding of include/llvq_hip.h.  There is no fallback: if the HIP
library is missing every entry point raises."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "csrc", "libllvq_hip.so")

STATUS = {
    0: "Ok", 1: "NotAnArtifact", 2: "Truncated", 3: "BadName", 5: "Inconsistent", 7: "IndexTooWide",
    8: "IndexOutOfRange", 9: "BadRawEncoding", 10: "CodebookMismatch", 11: "UnknownVersion", 32: "InvalidArgument",
    33: "Unsupported", 34: "Device",
}
F32, F16 = 0, 1
LAUNCH_PER_GROUP, LAUNCH_SINGLE, LAUNCH_CHAINED = 0, 1, 2  # llvq_launch_mode
STATIC_SCRATCH_BYTES = 64 << 20  # LLVQ_STATIC_SCRATCH_BYTES of include/llvq_hip.h
FINGERPRINT = 0x338F420F11866319


class LlvqError(RuntimeError):
    def __init__(self, code, message):
        self.code = code
        self.kind = STATUS.get(code, str(code))
        super().__init__(f"{self.kind}: {message}")


class MatrixDesc(C.Structure):
    _fields_ = [
        ("name", C.c_char_p),
        ("d_out", C.c_uint32), ("d_in", C.c_uint32), ("shell_cap", C.c_uint32), ("n_centroids", C.c_uint32),
        ("centroids", C.c_void_p), ("row_scales", C.c_void_p), ("tail", C.c_void_p),
        ("codes", C.c_void_p), ("code_bytes", C.c_size_t),
        ("rotation_seed", C.c_uint64), ("has_rotation", C.c_uint32),
    ]


class RecordInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 256),
        ("d_out", C.c_uint32), ("d_in", C.c_uint32), ("shell_cap", C.c_uint32), ("n_centroids", C.c_uint32),
        ("rotation_seed", C.c_uint64), ("has_rotation", C.c_uint32),
        ("centroids_off", C.c_size_t), ("row_scales_off", C.c_size_t), ("tail_off", C.c_size_t),
        ("codes_off", C.c_size_t), ("code_bytes", C.c_size_t),
    ]


class RawInfo(C.Structure):
    _fields_ = [
        ("name", C.c_char * 256), ("rank", C.c_uint32), ("dims", C.c_uint64 * 8), ("tag", C.c_uint32),
        ("bits", C.c_uint32), ("group", C.c_uint32), ("count", C.c_uint64),
        ("data_off", C.c_size_t), ("data_len", C.c_size_t), ("scales_off", C.c_size_t), ("biases_off", C.c_size_t),
    ]


class BlobInfo(C.Structure):
    _fields_ = [("name", C.c_char * 256), ("data_off", C.c_size_t), ("data_len", C.c_size_t)]


class QuantRows(C.Structure):
    _fields_ = [("codes", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p), ("bits", C.c_uint32),
                ("group", C.c_uint32)]


class SeqItem(C.Structure):
    _fields_ = [("mats", C.POINTER(C.c_void_p)), ("n_mats", C.c_int), ("x_f16_dev", C.c_void_p),
                ("y_dev", C.POINTER(C.c_void_p)), ("y_dtype", C.c_int), ("after_previous", C.c_int)]


class DecoderDesc(C.Structure):
    _fields_ = [
        ("n_layers", C.c_uint32), ("hidden", C.c_uint32), ("n_heads", C.c_uint32), ("n_kv_heads", C.c_uint32),
        ("head_dim", C.c_uint32), ("intermediate", C.c_uint32), ("vocab", C.c_uint32), ("max_positions", C.c_uint32),
        ("rope_theta", C.c_double), ("rms_eps", C.c_double),
        ("projections", C.POINTER(C.c_void_p)),
        ("input_norm", C.c_void_p), ("post_norm", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p),
        ("final_norm", C.c_void_p), ("embed", C.c_void_p), ("lm_head", C.c_void_p),
        ("kv_mode", C.c_uint32), ("embed_q8", QuantRows), ("lm_head_q8", QuantRows),
        ("prefill_rows", C.c_uint32), ("launch_mode", C.c_uint32),
    ]


def lib_path():
    return _LIB


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB):
        raise RuntimeError(
            f"{_LIB} is missing: build it with `make -C {os.path.dirname(_LIB)}` "
            "(or __graft_entry__.build()); there is no CPU fallback")
    # torch ships its own HIP runtime; load it first so the process holds exactly
    # one (libllvq_hip.so's libamdhip64 dependency then resolves to that one, and
    # the two share devices, streams and allocations).
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(_LIB)
    vp, sz = C.c_void_p, C.c_size_t
    L.llvq_hip_runtime_create.argtypes = [C.c_int, vp, C.POINTER(vp)]
    L.llvq_hip_runtime_destroy.argtypes = [vp]
    L.llvq_hip_runtime_destroy.restype = None
    L.llvq_hip_codebook_fingerprint.restype = C.c_uint64
    L.llvq_hip_host_decode.argtypes = [C.c_uint64, vp, C.POINTER(C.c_int)]
    L.llvq_hip_matrix_upload.argtypes = [vp, C.POINTER(MatrixDesc), C.POINTER(vp)]
    L.llvq_hip_read_header.argtypes = [C.c_char_p, sz, C.POINTER(sz), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
    L.llvq_hip_parse_matrix_record.argtypes = [C.c_char_p, sz, C.POINTER(sz), C.POINTER(RecordInfo)]
    L.llvq_hip_parse_raw_tensor.argtypes = [C.c_char_p, sz, C.POINTER(sz), C.c_uint32, C.POINTER(RawInfo)]
    L.llvq_hip_parse_blob.argtypes = [C.c_char_p, sz, C.POINTER(sz), C.POINTER(BlobInfo)]
    L.llvq_hip_matrix_from_record.argtypes = [vp, C.c_char_p, sz, C.POINTER(sz), C.POINTER(vp)]
    L.llvq_hip_matrix_free.argtypes = [vp, vp]
    L.llvq_hip_matrix_free.restype = None
    L.llvq_hip_matrix_info.argtypes = [vp] + [C.POINTER(C.c_uint32)] * 4 + [C.POINTER(C.c_uint64)]
    L.llvq_hip_matrix_name.argtypes = [vp]
    L.llvq_hip_matrix_name.restype = C.c_char_p
    L.llvq_hip_gemv.argtypes = [vp, vp, vp, vp, C.c_int]
    L.llvq_hip_host_rotate.argtypes = [C.c_uint32, C.c_uint64, vp]
    L.llvq_hip_rotate.argtypes = [vp, vp, vp, vp]
    L.llvq_hip_gemv_rotated.argtypes = [vp, vp, vp, vp, C.c_int]
    L.llvq_hip_matrix_rotation.argtypes = [vp, C.POINTER(C.c_uint32), C.POINTER(C.c_uint64)]
    L.llvq_hip_gemv_group.argtypes = [vp, C.POINTER(vp), C.c_int, vp, C.POINTER(vp), C.c_int]
    L.llvq_hip_sequence_create.argtypes = [vp, C.POINTER(SeqItem), C.c_int, C.POINTER(vp)]
    L.llvq_hip_sequence_run.argtypes = [vp, vp]
    L.llvq_hip_sequence_status.argtypes = [vp, vp]
    L.llvq_hip_sequence_tune.argtypes = [vp, C.c_uint32, C.c_int]
    L.llvq_hip_sequence_destroy.argtypes = [vp, vp]
    L.llvq_hip_sequence_destroy.restype = None
    L.llvq_hip_gemm.argtypes = [vp, vp, vp, C.c_int, vp, C.c_int]
    L.llvq_hip_reserve_batched.argtypes = [vp, C.POINTER(vp), C.c_int, C.c_int]
    L.llvq_hip_decoder_generate_phased.argtypes = [vp, vp, sz, sz, vp, vp]
    L.llvq_hip_gemm_static.argtypes = [vp, vp, vp, C.c_int, vp, C.c_int]
    L.llvq_hip_gemm_group.argtypes = [vp, C.POINTER(vp), C.c_int, vp, C.c_int, C.POINTER(vp), C.c_int]
    L.llvq_hip_decode_blocks.argtypes = [vp, vp, sz, vp, vp, vp]
    L.llvq_hip_decode_stream.argtypes = [vp, vp, sz, C.c_uint32, vp, vp, vp]
    L.llvq_hip_synchronize.argtypes = [vp]
    L.llvq_hip_decoder_create.argtypes = [vp, C.POINTER(DecoderDesc), C.POINTER(vp)]
    L.llvq_hip_decoder_destroy.argtypes = [vp]
    L.llvq_hip_decoder_destroy.restype = None
    L.llvq_hip_decoder_reset.argtypes = [vp]
    L.llvq_hip_decoder_position.argtypes = [vp]
    L.llvq_hip_decoder_seek.argtypes = [vp, C.c_uint32]
    L.llvq_hip_decoder_forward_token.argtypes = [vp, C.c_uint32, vp, C.POINTER(C.c_uint32)]
    L.llvq_hip_decoder_generate.argtypes = [vp, vp, sz, sz, vp]
    L.llvq_hip_decoder_generate_prefilled.argtypes = [vp, vp, sz, sz, vp]
    L.llvq_hip_decoder_prefill.argtypes = [vp, vp, sz, vp, C.POINTER(C.c_uint32)]
    L.llvq_hip_last_error.restype = C.c_char_p
    L.llvq_hip_version.restype = C.c_char_p
    _lib = L
    return L


def check(rc):
    if rc != 0:
        raise LlvqError(rc, (lib().llvq_hip_last_error() or b"").decode("utf-8", "replace"))


EXPORTS = [
    "llvq_hip_runtime_create", "llvq_hip_runtime_destroy", "llvq_hip_codebook_fingerprint",
    "llvq_hip_host_decode", "llvq_hip_matrix_upload", "llvq_hip_read_header", "llvq_hip_parse_matrix_record",
    "llvq_hip_matrix_from_record", "llvq_hip_parse_raw_tensor", "llvq_hip_parse_blob",
    "llvq_hip_matrix_free", "llvq_hip_matrix_info", "llvq_hip_matrix_name", "llvq_hip_gemv",
    "llvq_hip_gemv_group", "llvq_hip_sequence_create", "llvq_hip_sequence_run", "llvq_hip_sequence_status", "llvq_hip_sequence_tune",
    "llvq_hip_sequence_destroy", "llvq_hip_gemm", "llvq_hip_gemm_static", "llvq_hip_reserve_batched", "llvq_hip_decoder_generate_phased", "llvq_hip_gemm_group", "llvq_hip_decode_blocks", "llvq_hip_decode_stream", "llvq_hip_synchronize",
    "llvq_hip_last_error", "llvq_hip_version",
    "llvq_hip_host_rotate", "llvq_hip_rotate", "llvq_hip_gemv_rotated", "llvq_hip_matrix_rotation",
    "llvq_hip_decoder_create", "llvq_hip_decoder_destroy", "llvq_hip_decoder_reset", "llvq_hip_decoder_position", "llvq_hip_decoder_seek",
    "llvq_hip_decoder_forward_token", "llvq_hip_decoder_generate", "llvq_hip_decoder_generate_prefilled",
    "llvq_hip_decoder_prefill",
]
