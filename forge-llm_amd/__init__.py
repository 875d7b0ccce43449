"""forge_llm_amd — MI355X (gfx950) backend for ForgeLLM's quantized-Llama hot path.

Python host side above the C ABI of libforge_hip.so (include/forge_hip.h).  The directory is
named `forge-llm_amd`; import it as `forge_llm_amd` through `load_package()` in the repo's
entry scripts, or put it on sys.path under that name.

There is no CPU fallback: every compute entry point goes to the HIP library and raises
`ForgeHipError` if the library is missing or reports an error.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libforge_hip.so")

Q4_0 = 2
Q8_0 = 8
Q4_K, Q6_K = 12, 14   # op level only: ops.QWeight + ops.matmul_vec_q
FLAG_EXACT = 1   # config.flags / op flags: order-faithful f32 arithmetic (bit-identical to the CPU path)
FLAG_QKV_BIAS = 2   # config.flags: q, k, v projections add a bias vector before RoPE (Qwen2); the blob carries the vectors

OK = 0
ERR_INVALID = -1
ERR_BLOB_SIZE = -2
ERR_POSITION = -3
ERR_NO_DEVICE = -4
ERR_HIP = -5

# every symbol include/forge_hip.h declares
EXPORTS = [
    "forge_hip_last_error", "forge_hip_device_count", "forge_hip_weights_nbytes", "forge_hip_model_create",
    "forge_hip_weights_nbytes_mixed", "forge_hip_model_create_mixed",
    "forge_hip_model_destroy", "forge_hip_forward", "forge_hip_forward_greedy", "forge_hip_prefill_batch",
    "forge_hip_forward_profile", "forge_hip_prefill_profile", "forge_hip_model_decode_launches", "forge_hip_reset", "forge_hip_model_pos", "forge_hip_model_set_poll_limit", "forge_hip_model_set_kv_pages", "forge_hip_model_read_kv", "forge_hip_f16_to_f32",
    "forge_hip_f32_to_f16", "forge_hip_quantize_f32", "forge_hip_expf_host", "forge_hip_dequant", "forge_hip_qweight_create",
    "forge_hip_qweight_destroy", "forge_hip_quantize_act", "forge_hip_gemv_q", "forge_hip_gemm_q", "forge_hip_gemm_silu_q",
    "forge_hip_block_isums", "forge_hip_gemv_q_f32act", "forge_hip_rms_norm", "forge_hip_silu_mul", "forge_hip_rope_kv_store",
    "forge_hip_attn_prefill_f16kv", "forge_hip_attn_decode_f16kv", "forge_hip_attn_decode_f16kv_noalloc", "forge_hip_attn_decode_f16kv_paged",
    "forge_hip_attn_prefill_sliding_f16kv", "forge_hip_attn_decode_sliding_f16kv", "forge_hip_argmax",
    "forge_hip_gguf_open", "forge_hip_gguf_parse", "forge_hip_gguf_close", "forge_hip_gguf_version", "forge_hip_gguf_alignment",
    "forge_hip_gguf_tensor_data_offset", "forge_hip_gguf_tensor_count", "forge_hip_gguf_metadata_count", "forge_hip_gguf_tensor",
    "forge_hip_gguf_find_tensor", "forge_hip_gguf_meta", "forge_hip_gguf_config", "forge_hip_gguf_export_weights",
    "forge_hip_gguf_config_mixed", "forge_hip_gguf_export_weights_mixed", "forge_hip_quantize_kquant",
    "forge_hip_model_create_from_gguf", "forge_hip_dequant_ggml", "forge_hip_model_set_repeat_penalty", "forge_hip_apply_repeat_penalty", "forge_hip_sample",
]


class ForgeHipError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"forge_hip error {code}: {msg}")
        self.code = code


class Config(C.Structure):
    """forge_hip_config (mirrors ModelConfig, crates/forgellm-frontend/src/ir.rs:484-519)."""
    _fields_ = [
        ("hidden", C.c_uint32), ("inter", C.c_uint32), ("layers", C.c_uint32), ("heads", C.c_uint32),
        ("kv_heads", C.c_uint32), ("head_dim", C.c_uint32), ("vocab", C.c_uint32), ("max_seq", C.c_uint32),
        ("rms_eps", C.c_float), ("rope_theta", C.c_float),
        ("wdtype", C.c_uint32), ("lm_head_dtype", C.c_uint32), ("flags", C.c_uint32),
        ("sliding_window", C.c_uint32),
    ]


_lib = None


def lib():
    """Load libforge_hip.so (built by build.py).  Raises if it is absent: there is no fallback."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ForgeHipError(ERR_NO_DEVICE, f"{LIB_PATH} not built; run `python forge-llm_amd/build.py`")
    # The Python host side uses PyTorch for device memory and streams, and PyTorch brings its own copy of the HIP
    # runtime: it has to be in the process first, so that the library binds to that same copy (loaded the other way
    # round, the two runtimes do not see each other's device).
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(LIB_PATH)
    vp, u32, u64, i32 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int32
    L.forge_hip_last_error.restype = C.c_char_p
    L.forge_hip_device_count.restype = i32
    L.forge_hip_weights_nbytes.restype = u64
    L.forge_hip_weights_nbytes.argtypes = [C.POINTER(Config)]
    L.forge_hip_model_create.restype = i32
    L.forge_hip_model_create.argtypes = [C.POINTER(Config), vp, u64, C.POINTER(vp)]
    L.forge_hip_model_destroy.argtypes = [vp]
    L.forge_hip_model_destroy.restype = None
    L.forge_hip_forward.restype = i32
    L.forge_hip_forward.argtypes = [vp, u32, vp]
    L.forge_hip_forward_greedy.restype = i32
    L.forge_hip_forward_greedy.argtypes = [vp, u32, C.POINTER(u32)]
    L.forge_hip_prefill_batch.restype = i32
    L.forge_hip_prefill_batch.argtypes = [vp, vp, u64, vp]
    L.forge_hip_forward_profile.restype = i32
    L.forge_hip_forward_profile.argtypes = [vp, u32, vp, vp]
    L.forge_hip_prefill_profile.restype = i32
    L.forge_hip_prefill_profile.argtypes = [vp, vp, u64, vp, vp]
    L.forge_hip_reset.restype = i32
    L.forge_hip_reset.argtypes = [vp]
    L.forge_hip_model_decode_launches.restype = C.c_int32
    L.forge_hip_model_decode_launches.argtypes = [vp]
    L.forge_hip_model_pos.restype = C.c_int64
    L.forge_hip_model_pos.argtypes = [vp]
    L.forge_hip_model_set_poll_limit.restype = i32
    L.forge_hip_model_set_poll_limit.argtypes = [vp, C.c_uint32]
    L.forge_hip_model_read_kv.restype = i32
    L.forge_hip_model_read_kv.argtypes = [vp, u32, u32, vp]
    L.forge_hip_weights_nbytes_mixed.restype = u64
    L.forge_hip_weights_nbytes_mixed.argtypes = [C.POINTER(Config), vp]
    L.forge_hip_model_create_mixed.restype = i32
    L.forge_hip_model_create_mixed.argtypes = [C.POINTER(Config), vp, vp, u64, C.POINTER(vp)]
    L.forge_hip_model_set_kv_pages.restype = i32
    L.forge_hip_model_set_kv_pages.argtypes = [vp, u32, vp, u32]
    L.forge_hip_f16_to_f32.restype = C.c_float
    L.forge_hip_f16_to_f32.argtypes = [C.c_uint16]
    L.forge_hip_f32_to_f16.restype = C.c_uint16
    L.forge_hip_f32_to_f16.argtypes = [C.c_float]
    L.forge_hip_quantize_f32.restype = i32
    L.forge_hip_quantize_f32.argtypes = [u32, vp, u64, vp]
    L.forge_hip_dequant.restype = i32
    L.forge_hip_dequant.argtypes = [u32, vp, u64, vp]
    L.forge_hip_qweight_create.restype = i32
    L.forge_hip_qweight_create.argtypes = [u32, vp, u32, u32, C.POINTER(vp)]
    L.forge_hip_qweight_destroy.argtypes = [vp]
    L.forge_hip_qweight_destroy.restype = None
    L.forge_hip_quantize_act.restype = i32
    L.forge_hip_quantize_act.argtypes = [vp, u32, u32, vp, vp, vp]
    L.forge_hip_gemv_q.restype = i32
    L.forge_hip_gemv_q.argtypes = [vp, vp, vp, vp]
    L.forge_hip_gemm_q.restype = i32
    L.forge_hip_gemm_q.argtypes = [vp, vp, u32, vp, u32, vp]
    L.forge_hip_gemm_silu_q.restype = i32
    L.forge_hip_gemm_silu_q.argtypes = [vp, vp, u32, vp, vp, vp]
    L.forge_hip_expf_host.restype = i32
    L.forge_hip_expf_host.argtypes = [vp, u64, vp]
    L.forge_hip_gemv_q_f32act.restype = i32
    L.forge_hip_gemv_q_f32act.argtypes = [vp, vp, vp, vp]
    L.forge_hip_block_isums.restype = i32
    L.forge_hip_block_isums.argtypes = [vp, vp, u32, vp, u32, vp]
    L.forge_hip_rms_norm.restype = i32
    L.forge_hip_rms_norm.argtypes = [vp, vp, C.c_float, u32, u32, vp, vp]
    L.forge_hip_silu_mul.restype = i32
    L.forge_hip_silu_mul.argtypes = [vp, vp, u64, vp, vp]
    L.forge_hip_rope_kv_store.restype = i32
    L.forge_hip_rope_kv_store.argtypes = [vp, vp, vp, vp, vp, u32, u32, u32, u32, u32, C.c_float, vp]
    L.forge_hip_attn_prefill_f16kv.restype = i32
    L.forge_hip_attn_prefill_f16kv.argtypes = [vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, vp]
    L.forge_hip_attn_decode_f16kv.restype = i32
    L.forge_hip_attn_decode_f16kv.argtypes = [vp, vp, vp, vp, u32, u32, u32, u32, u32, vp]
    L.forge_hip_attn_decode_f16kv_paged.restype = i32
    L.forge_hip_attn_decode_f16kv_paged.argtypes = [vp, vp, vp, vp, u32, vp, u32, u32, u32, u32, vp]
    L.forge_hip_attn_decode_f16kv_noalloc.restype = i32
    L.forge_hip_attn_decode_f16kv_noalloc.argtypes = [vp, vp, vp, vp, u32, u32, u32, u32, vp]
    L.forge_hip_attn_prefill_sliding_f16kv.restype = i32
    L.forge_hip_attn_prefill_sliding_f16kv.argtypes = [vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, u32, vp]
    L.forge_hip_attn_decode_sliding_f16kv.restype = i32
    L.forge_hip_attn_decode_sliding_f16kv.argtypes = [vp, vp, vp, vp, u32, u32, u32, u32, u32, u32, vp]
    L.forge_hip_argmax.restype = i32
    L.forge_hip_argmax.argtypes = [vp, u32, vp, vp]
    L.forge_hip_model_set_repeat_penalty.restype = i32
    L.forge_hip_model_set_repeat_penalty.argtypes = [vp, C.c_float]
    L.forge_hip_apply_repeat_penalty.restype = i32
    L.forge_hip_apply_repeat_penalty.argtypes = [vp, u64, vp, u64, C.c_float]
    L.forge_hip_sample.restype = i32
    L.forge_hip_sample.argtypes = [vp, u64, C.c_float, u64, C.c_float, C.POINTER(u64), C.POINTER(u32)]
    _lib = L
    return L


def check(rc):
    if rc != OK:
        raise ForgeHipError(rc, lib().forge_hip_last_error().decode("utf-8", "replace"))


def device_count():
    return int(lib().forge_hip_device_count())


def require_gpu():
    if device_count() < 1:
        raise ForgeHipError(ERR_NO_DEVICE, "no HIP device visible")


from .hip_model import HipModel  # noqa: E402
from . import gguf, ops, serve, synth  # noqa: E402

__all__ = ["HipModel", "ops", "serve", "synth", "Config", "ForgeHipError", "lib", "check", "device_count", "Q4_0", "Q8_0", "FLAG_EXACT"]
