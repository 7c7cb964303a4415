"""Host mirror of the reference's model runner at batch 1
(llvq-llm/src/model.rs: Qwen3::new_with :869, hidden_cached :968, generate :1041)
over the HIP library's decode loop.  No computation happens here: the class
assembles the descriptor and calls the C ABI."""
import ctypes as C
import json
from dataclasses import dataclass

import numpy as np

from . import _ffi, artifact, synth
from .fused import FusedRuntime

SITES = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj",
         "mlp.gate_proj", "mlp.up_proj", "mlp.down_proj")


@dataclass
class Qwen3Config:
    """The fields of the reference's Config that the forward pass reads."""
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rope_theta: float = 1e6
    rms_norm_eps: float = 1e-6
    max_positions: int = 1024
    tie_word_embeddings: bool = True
    kv_mode: str = "f16"  # KvMode::parse (kvq.rs:38-49): "f16" or "q8"

    def shapes(self):
        """(site, d_out, d_in) of the seven projections of one layer."""
        qd, kvd = self.num_attention_heads * self.head_dim, self.num_key_value_heads * self.head_dim
        h, i = self.hidden_size, self.intermediate_size
        return [(SITES[0], qd, h), (SITES[1], kvd, h), (SITES[2], kvd, h), (SITES[3], h, qd),
                (SITES[4], i, h), (SITES[5], i, h), (SITES[6], h, i)]


QWEN3_14B = Qwen3Config(40, 5120, 40, 8, 128, 17408, 151936, max_positions=8192, tie_word_embeddings=False, kv_mode="q8")
QWEN3_4B = Qwen3Config(36, 2560, 32, 8, 128, 9728, 151936, max_positions=768, tie_word_embeddings=False)


@dataclass
class DecoderWeights:
    """Everything a decoder holds besides its LLVQ projections, as binary16 arrays."""
    input_norm: np.ndarray   # [n_layers, hidden]
    post_norm: np.ndarray    # [n_layers, hidden]
    q_norm: np.ndarray       # [n_layers, head_dim]
    k_norm: np.ndarray       # [n_layers, head_dim]
    final_norm: np.ndarray   # [hidden]
    embed: object            # [vocab, hidden] binary16 array, or an int8 g64 artifact.RawTensor
    lm_head: object = None   # the same, or None (tied to the embedding)


def synthetic_weights(cfg: Qwen3Config, seed: int = 0) -> DecoderWeights:
    """Random-init dense tensors: norm gains 1 + 0.1 N(0,1), embedding N(0,1), head 0.05 N(0,1)."""
    rng = np.random.default_rng(seed)
    L, h, d = cfg.num_hidden_layers, cfg.hidden_size, cfg.head_dim

    def gains(*shape):
        return (1.0 + 0.1 * rng.standard_normal(shape, dtype=np.float32)).astype(np.float16)

    embed = rng.standard_normal((cfg.vocab_size, h), dtype=np.float32).astype(np.float16)
    head = None
    if not cfg.tie_word_embeddings:
        head = (0.05 * rng.standard_normal((cfg.vocab_size, h), dtype=np.float32)).astype(np.float16)
    return DecoderWeights(gains(L, h), gains(L, h), gains(L, d), gains(L, d), gains(h), embed, head)


def quantize_rows_q8(name: str, table, group: int = 64) -> artifact.RawTensor:
    """A [rows, d] binary16 table as the int8 tensor of the sealed sections (llvq-artifact/src/sealed.rs:64-78), with the
    bytes the reference's embedq tool writes (llvq-llm/src/embedquant.rs:22-92, f32 arithmetic throughout): per group
    of `group` along a row, scale = f16((max - min) / 255), bias = f16(min), code = the quotient (w - bias) / scale
    against the rounded scale and bias, rounded half away from zero and clamped to [0, 255]; a group whose scale
    rounds to zero stores scale 1.0 and codes 0, the bias carrying the value."""
    w = np.asarray(table, dtype=np.float16).astype(np.float32)
    rows, d = w.shape
    if d % group:
        raise ValueError(f"{name}: row length {d} is not a multiple of the group {group}")
    g = w.reshape(rows, d // group, group)
    mn, mx = g.min(-1, keepdims=True), g.max(-1, keepdims=True)
    s = ((mx - mn) / np.float32(255.0)).astype(np.float16)
    b = mn.astype(np.float16)
    graded = s.astype(np.float32) > 0
    s = np.where(graded, s, np.float16(1.0)).astype(np.float16)
    t = ((g - b.astype(np.float32)) / s.astype(np.float32)).astype(np.float64)  # f32 quotient; the half is added exactly
    t = np.sign(t) * np.floor(np.abs(t) + 0.5)
    q = np.where(graded, np.clip(t, 0, 255), 0).astype(np.uint8)
    return artifact.RawTensor(name, [rows, d], bits=8, group=group, packed=q.reshape(-1), scales=s.reshape(-1).view(np.uint16),
                              biases=b.reshape(-1).view(np.uint16))


def synthetic_projections(cfg: Qwen3Config, seed: int = 0, shell_cap: int = 12):
    """Random LLVQ codes for every projection, drawn as the single-matrix benchmark draws them."""
    return [[synth.make_matrix(f"model.layers.{layer}.{site}.weight", do, di, seed, shell_cap=shell_cap)
             for site, do, di in cfg.shapes()] for layer in range(cfg.num_hidden_layers)]


class Decoder:
    """A Qwen3-architecture model on one GPU: projections uploaded through `rt`,
    the rest copied at construction."""

    def __init__(self, rt: FusedRuntime, cfg: Qwen3Config, projections, weights: DecoderWeights, prefill_rows: int = 0,
                 launch_mode: int = _ffi.LAUNCH_PER_GROUP):
        """prefill_rows > 0 also allocates the row buffers of the batched prompt path (`prefill`).
        launch_mode: llvq_launch_mode of include/llvq_hip.h (how a position's projection groups are launched)."""
        self.rt, self.cfg = rt, cfg
        self.handle = None
        self._owned = []
        projs = []
        for layer in projections:
            if len(layer) != 7:
                raise ValueError("a layer has seven projections: q, k, v, o, gate, up, down")
            for m in layer:
                if hasattr(m, "handle"):
                    projs.append(m)
                else:
                    p = rt.upload(m)
                    self._owned.append(p)
                    projs.append(p)
        self._projs = projs
        arr = (C.c_void_p * len(projs))(*[p.handle for p in projs])

        def f16(a, shape):
            a = np.ascontiguousarray(a, dtype=np.float16)
            if a.shape != tuple(shape):
                raise ValueError(f"expected shape {tuple(shape)}, got {a.shape}")
            return a

        L, h, d = cfg.num_hidden_layers, cfg.hidden_size, cfg.head_dim
        keep = [f16(weights.input_norm, (L, h)), f16(weights.post_norm, (L, h)), f16(weights.q_norm, (L, d)),
                f16(weights.k_norm, (L, d)), f16(weights.final_norm, (h,))]

        def table(t, what):
            """A [vocab, hidden] table: (binary16 pointer or None, QuantRows, arrays to keep alive)."""
            if t is None:
                return None, _ffi.QuantRows(), ()
            if isinstance(t, artifact.RawTensor) and t.kind == "quant":
                if t.dims != [cfg.vocab_size, h]:
                    raise ValueError(f"{what}: dims {t.dims}, expected [{cfg.vocab_size}, {h}]")
                alive = (np.ascontiguousarray(t.packed), np.ascontiguousarray(t.scales), np.ascontiguousarray(t.biases))
                return None, _ffi.QuantRows(alive[0].ctypes.data, alive[1].ctypes.data, alive[2].ctypes.data,
                                            int(t.bits), int(t.group)), alive
            if isinstance(t, artifact.RawTensor):
                t = t.data.view(np.float16).reshape(t.dims)
            a = f16(t, (cfg.vocab_size, h))
            return a.ctypes.data, _ffi.QuantRows(), (a,)

        e_ptr, e_q, e_alive = table(weights.embed, "embedding")
        h_ptr, h_q, h_alive = table(weights.lm_head, "lm_head")
        desc = _ffi.DecoderDesc(
            L, h, cfg.num_attention_heads, cfg.num_key_value_heads, d, cfg.intermediate_size, cfg.vocab_size,
            cfg.max_positions, float(cfg.rope_theta), float(cfg.rms_norm_eps),
            C.cast(arr, C.POINTER(C.c_void_p)),
            keep[0].ctypes.data, keep[1].ctypes.data, keep[2].ctypes.data, keep[3].ctypes.data, keep[4].ctypes.data,
            e_ptr, h_ptr, self._kv_mode(cfg.kv_mode), e_q, h_q, int(prefill_rows), int(launch_mode))
        self._alive = (keep, e_alive, h_alive)
        out = C.c_void_p()
        _ffi.check(_ffi.lib().llvq_hip_decoder_create(rt.handle, C.byref(desc), C.byref(out)))
        self.handle = out

    @classmethod
    def from_model(cls, rt: FusedRuntime, model, max_positions=None, kv_mode="f16", prefill_rows: int = 0):
        """Qwen3::new_with over a loaded sealed artifact (fused_cuda.rs:1226-1300 + model.rs:869):
        the architecture comes from the file's config.json, the projections from its matrix
        records (by `model.layers.{i}.{site}.weight`), norms and embedding from its raw tensors."""
        c = json.loads(model.config_json.decode("utf-8"))
        heads = c["num_attention_heads"]
        cfg = Qwen3Config(
            num_hidden_layers=c["num_hidden_layers"], hidden_size=c["hidden_size"], num_attention_heads=heads,
            num_key_value_heads=c.get("num_key_value_heads", heads), head_dim=c.get("head_dim", c["hidden_size"] // heads),
            intermediate_size=c["intermediate_size"], vocab_size=c["vocab_size"], rope_theta=c.get("rope_theta", 1e6),
            rms_norm_eps=c.get("rms_norm_eps", 1e-6),
            max_positions=int(max_positions or min(c.get("max_position_embeddings", 8192), 8192)),
            tie_word_embeddings=bool(c.get("tie_word_embeddings", False)), kv_mode=kv_mode)
        sites = {}
        for fm in model.matrices:
            layer, site = artifact.split_name(fm.name)
            sites[(layer, site)] = fm
        projections = []
        for layer in range(cfg.num_hidden_layers):
            row = []
            for site in SITES:
                if (layer, site) not in sites:
                    raise ValueError(f"the file carries no model.layers.{layer}.{site}.weight")
                row.append(sites[(layer, site)].raw)
            projections.append(row)

        def halves(name, shape):
            t = model.tensor(name)
            if t.kind != "f16":
                raise ValueError(f"{name}: stored quantized, a norm is carried as binary16")
            return t.data.view(np.float16).reshape(shape)

        L, h, d = cfg.num_hidden_layers, cfg.hidden_size, cfg.head_dim
        stack = lambda fmt, n: np.stack([halves(fmt.format(i), (n,)) for i in range(L)])
        head = None
        if not cfg.tie_word_embeddings:  # fused.rs:252-285: an untied model must carry its own head
            head = model.tensor("lm_head.weight")
        weights = DecoderWeights(
            stack("model.layers.{}.input_layernorm.weight", h), stack("model.layers.{}.post_attention_layernorm.weight", h),
            stack("model.layers.{}.self_attn.q_norm.weight", d), stack("model.layers.{}.self_attn.k_norm.weight", d),
            halves("model.norm.weight", (h,)), model.tensor("model.embed_tokens.weight"), head)
        return cls(rt, cfg, projections, weights, prefill_rows=prefill_rows)

    @staticmethod
    def _kv_mode(v):
        """KvMode::parse (kvq.rs:38-49): a typo is an error, never a silent default."""
        if v in (None, "", "f16"):
            return 0
        if v == "q8":
            return 1
        raise ValueError(f"kv_mode={v}: accepted values are 'f16' (default) and 'q8'")

    def reset(self):
        _ffi.check(_ffi.lib().llvq_hip_decoder_reset(self.handle))

    @property
    def position(self):
        return _ffi.lib().llvq_hip_decoder_position(self.handle)

    def seek(self, position: int):
        """Measurement aid: jump to `position` without feeding the tokens before it."""
        _ffi.check(_ffi.lib().llvq_hip_decoder_seek(self.handle, int(position)))

    def forward_token(self, token: int, want_logits: bool = True):
        """One position: (logits f32 [vocab] or None, argmax)."""
        logits = np.empty(self.cfg.vocab_size, np.float32) if want_logits else None
        best = C.c_uint32()
        _ffi.check(_ffi.lib().llvq_hip_decoder_forward_token(
            self.handle, int(token), logits.ctypes.data if want_logits else None, C.byref(best)))
        return logits, best.value

    def prefill(self, tokens, want_logits: bool = True):
        """The next len(tokens) positions through the batched product, `prefill_rows` at a time:
        (logits of the last one or None, its argmax).  The decoder must have been built with prefill_rows > 0."""
        tokens = np.ascontiguousarray(tokens, dtype=np.uint32)
        logits = np.empty(self.cfg.vocab_size, np.float32) if want_logits else None
        best = C.c_uint32()
        _ffi.check(_ffi.lib().llvq_hip_decoder_prefill(
            self.handle, tokens.ctypes.data, tokens.size, logits.ctypes.data if want_logits else None, C.byref(best)))
        return logits, best.value

    def generate(self, prompt, max_new: int, batched_prefill: bool = False) -> np.ndarray:
        """Greedy tokens after `prompt`.  batched_prefill takes the prompt through `prefill` (matrix cores,
        weights rounded to binary16 once) instead of position by position."""
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.zeros(max_new, np.uint32)
        fn = _ffi.lib().llvq_hip_decoder_generate_prefilled if batched_prefill else _ffi.lib().llvq_hip_decoder_generate
        _ffi.check(fn(self.handle, prompt.ctypes.data, prompt.size, max_new, out.ctypes.data))
        return out

    def generate_phased(self, prompt, max_new: int):
        """Qwen3::generate_phased (model.rs:1116-1163): the tokens of `generate` and, per decoded token,
        the device time of its phases in ms — columns head (final norm + head), rest (argmax), embed,
        blocks (the layers); the last token's embed and blocks are zero (it is not fed back)."""
        prompt = np.ascontiguousarray(prompt, dtype=np.uint32)
        out = np.zeros(max_new, np.uint32)
        phases = np.zeros((max_new, 4), np.float64)
        _ffi.check(_ffi.lib().llvq_hip_decoder_generate_phased(self.handle, prompt.ctypes.data, prompt.size, max_new,
                                                                out.ctypes.data, phases.ctypes.data))
        return out, phases

    def close(self):
        if self.handle is not None:
            _ffi.lib().llvq_hip_decoder_destroy(self.handle)
            self.handle = None
        for p in self._owned:
            self.rt.free(p)
        self._owned = []

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
