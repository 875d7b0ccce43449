"""Op-level wrappers over the C ABI.  torch is used only to own device memory and streams;
every computation happens in libforge_hip.so.  Names follow the reference's kernels
(crates/forgellm-codegen-cpu/src/emit.rs): matmul_vec_q*, matmul_mat_q*, rms_norm, silu_mul,
rope, attention_flash, attention_flash_batch, argmax.
"""
import ctypes as C

import numpy as np


def _torch():
    import torch
    return torch


def _ptr(t):
    return C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(_torch().cuda.current_stream().cuda_stream)


def _dev(t, dtype):
    torch = _torch()
    if not (t.is_cuda and t.is_contiguous() and t.dtype == dtype):
        raise ValueError(f"expected a contiguous CUDA tensor of {dtype}")
    return t


# ---------------- host-side format helpers ----------------

def block_bytes(wdtype):
    return 34 if wdtype == 8 else 18


def quantize_weights(wdtype, x) -> np.ndarray:
    """quantize_f32_to_q8_0 / _q4_0 (weight_loader.rs:1454-1544): f32 array -> raw GGUF blocks."""
    from . import check, lib
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty((x.size + 31) // 32 * block_bytes(wdtype), np.uint8)
    check(lib().forge_hip_quantize_f32(wdtype, x.ctypes.data_as(C.c_void_p), x.size, out.ctypes.data_as(C.c_void_p)))
    return out


def dequant(wdtype, raw, n) -> np.ndarray:
    """dequant_q8_0 / dequant_q4_0 (weight_loader.rs:860-926)."""
    from . import check, lib
    raw = np.ascontiguousarray(raw, dtype=np.uint8)
    out = np.empty(n, np.float32)
    check(lib().forge_hip_dequant(wdtype, raw.ctypes.data_as(C.c_void_p), n, out.ctypes.data_as(C.c_void_p)))
    return out


def f16_to_f32(bits: int) -> float:
    from . import lib
    return float(lib().forge_hip_f16_to_f32(int(bits)))


def f32_to_f16(x: float) -> int:
    from . import lib
    return int(lib().forge_hip_f32_to_f16(float(x)))


def argmax_host(logits) -> int:
    """argmax of the generated main.rs (project.rs:501-503): the LAST index among equal maxima."""
    v = np.asarray(logits)
    return int(v.size - 1 - np.argmax(v[::-1]))


def apply_repeat_penalty(logits, recent_tokens, penalty: float) -> None:
    """apply_repeat_penalty (project.rs:505-513), in place on a float32 array."""
    from . import check, lib
    assert logits.dtype == np.float32 and logits.flags.c_contiguous
    r = np.ascontiguousarray(recent_tokens, dtype=np.uint32)
    check(lib().forge_hip_apply_repeat_penalty(logits.ctypes.data_as(C.c_void_p), logits.size, r.ctypes.data_as(C.c_void_p), r.size,
                                               float(penalty)))


def sample(logits, temperature: float, top_k: int, top_p: float, rng_state: int):
    """sample (project.rs:515-555): returns (token, new rng state).  `logits` (float32) is overwritten, as in the reference."""
    from . import check, lib
    assert logits.dtype == np.float32 and logits.flags.c_contiguous
    state, out = C.c_uint64(rng_state), C.c_uint32()
    check(lib().forge_hip_sample(logits.ctypes.data_as(C.c_void_p), logits.size, float(temperature), int(top_k), float(top_p),
                                 C.byref(state), C.byref(out)))
    return int(out.value), int(state.value)


# ---------------- device ops ----------------

class QWeight:
    """One weight matrix uploaded from raw GGUF blocks, row-major [N][K/32]."""

    def __init__(self, wdtype, raw, K, N):
        from . import check, lib, require_gpu
        require_gpu()
        raw = np.ascontiguousarray(raw, dtype=np.uint8)
        # Q8_0 / Q4_0: 34- / 18-byte blocks of 32; Q4_K (12) / Q6_K (14): 144- / 210-byte super-blocks of 256
        expect = N * (K // 256) * {12: 144, 14: 210}[wdtype] if wdtype in (12, 14) else N * (K // 32) * block_bytes(wdtype)
        if raw.size != expect:
            raise ValueError("raw weight bytes do not match N x K")
        self.wdtype, self.K, self.N = wdtype, K, N
        self._lib = lib()
        h = C.c_void_p()
        check(self._lib.forge_hip_qweight_create(wdtype, raw.ctypes.data_as(C.c_void_p), K, N, C.byref(h)))
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            self._lib.forge_hip_qweight_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def quantize_act(x):
    """quantize_to_q8_0_blocks_into (emit.rs:1410-1440): x f32 [M][K] -> (int8 [M][K], fp16-bit scales [M][K/32])."""
    from . import check, lib
    torch = _torch()
    x = _dev(x, torch.float32)
    M, K = (1, x.shape[0]) if x.dim() == 1 else x.shape
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    sc = torch.empty((M, K // 32), dtype=torch.int16, device=x.device)
    check(lib().forge_hip_quantize_act(_ptr(x), M, K, _ptr(q), _ptr(sc), _stream()))
    return q, sc


def matmul_vec_q(w: QWeight, x):
    """matmul_vec_q8_0_KxN / matmul_vec_q4_0_KxN: x f32 [K] -> f32 [N]."""
    from . import check, lib
    torch = _torch()
    x = _dev(x, torch.float32)
    if x.numel() != w.K:
        raise ValueError("input length must equal K")
    y = torch.empty(w.N, dtype=torch.float32, device=x.device)
    check(lib().forge_hip_gemv_q(w._h, _ptr(x), _ptr(y), _stream()))
    return y


def matmul_vec_q_portable(w: QWeight, x):
    """The same matmul through the reference's portable row dot (the x86 arithmetic: f32 activations, weights dequantised
    on the fly, one sequential sum per row; emit.rs:1359-1377, 2337-2359)."""
    from . import check, lib
    torch = _torch()
    x = _dev(x, torch.float32)
    if x.numel() != w.K:
        raise ValueError("input length must equal K")
    y = torch.empty(w.N, dtype=torch.float32, device=x.device)
    check(lib().forge_hip_gemv_q_f32act(w._h, _ptr(x), _ptr(y), _stream()))
    return y


def expf_host(x) -> np.ndarray:
    """exp as the GPU kernels evaluate it (host twin; bit-identical to the C library's expf)."""
    from . import check, lib
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    check(lib().forge_hip_expf_host(x.ctypes.data_as(C.c_void_p), x.size, out.ctypes.data_as(C.c_void_p)))
    return out


def gate_up_silu_q(w: QWeight, x):
    """The gate / up matmuls, silu_mul and the activation quantiser of the batched feed-forward block in one launch
    (crates/forgellm-codegen-cpu/src/emit.rs:5390-5420): w holds the gate rows then the up rows; x: f32 [M][K] on the GPU.
    Returns (codes int8 [M][N/2] with odd blocks negated, scales as fp16 bit patterns int16 [M][N/64])."""
    from . import check, lib
    torch = _torch()
    x = _dev(x, torch.float32)
    if x.dim() != 2 or x.shape[1] != w.K:
        raise ValueError("input must be [M][K]")
    M = x.shape[0]
    q = torch.empty((M, w.N // 2), dtype=torch.int8, device=x.device)
    sc = torch.empty((M, w.N // 64), dtype=torch.int16, device=x.device)
    check(lib().forge_hip_gemm_silu_q(w._h, _ptr(x), M, _ptr(q), _ptr(sc), _stream()))
    return q, sc


def matmul_mat_q(w: QWeight, x, flags=0):
    """matmul_mat_q8_0_KxN / matmul_mat_q4_0_KxN: x f32 [M][K] -> f32 [M][N]."""
    from . import check, lib
    torch = _torch()
    x = _dev(x, torch.float32)
    if x.dim() != 2 or x.shape[1] != w.K:
        raise ValueError("input must be [M][K]")
    M = x.shape[0]
    y = torch.empty((M, w.N), dtype=torch.float32, device=x.device)
    check(lib().forge_hip_gemm_q(w._h, _ptr(x), M, _ptr(y), flags, _stream()))
    return y


def block_isums(w: QWeight, x, path):
    """int32 block sums [M][N][K/32]; path 0 = GEMV kernel, 1 = MFMA GEMM kernel (exact mode), 2 = the same in fast mode."""
    from . import check, lib
    torch = _torch()
    x = _dev(x, torch.float32)
    x2 = x.reshape(-1, w.K)
    M = x2.shape[0]
    out = torch.empty((M, w.N, w.K // 32), dtype=torch.int32, device=x.device)
    check(lib().forge_hip_block_isums(w._h, _ptr(x2), M, _ptr(out), path, _stream()))
    return out


def rms_norm(x, weight, eps):
    from . import check, lib
    torch = _torch()
    x, weight = _dev(x, torch.float32), _dev(weight, torch.float32)
    x2 = x.reshape(-1, x.shape[-1])
    out = torch.empty_like(x2)
    check(lib().forge_hip_rms_norm(_ptr(x2), _ptr(weight), eps, x2.shape[0], x2.shape[1], _ptr(out), _stream()))
    return out.reshape(x.shape)


def silu_mul(gate, up):
    from . import check, lib
    torch = _torch()
    gate, up = _dev(gate, torch.float32), _dev(up, torch.float32)
    out = torch.empty_like(gate)
    check(lib().forge_hip_silu_mul(_ptr(gate), _ptr(up), gate.numel(), _ptr(out), _stream()))
    return out


def rope_kv_store(q, k, v, k_cache, v_cache, base_pos, heads, kv_heads, head_dim, theta):
    """rope on q,k in place (rows = tokens at base_pos..) and fp16 write of k,v into the caches."""
    from . import check, lib
    torch = _torch()
    q, k, v = _dev(q, torch.float32), _dev(k, torch.float32), _dev(v, torch.float32)
    k_cache, v_cache = _dev(k_cache, torch.int16), _dev(v_cache, torch.int16)
    M = q.shape[0]
    if base_pos + M > k_cache.shape[0]:
        raise ValueError("cache too small")
    check(lib().forge_hip_rope_kv_store(_ptr(q), _ptr(k), _ptr(v), _ptr(k_cache), _ptr(v_cache), M, base_pos, heads,
                                        kv_heads, head_dim, theta, _stream()))


def attention_flash_batch(q, k_cache, v_cache, base_pos, heads, kv_heads, head_dim, flags=0):
    """attention_flash_batch over an fp16 cache: q f32 [M][heads*hd] -> f32 [M][heads*hd]."""
    from . import check, lib
    torch = _torch()
    q = _dev(q, torch.float32)
    k_cache, v_cache = _dev(k_cache, torch.int16), _dev(v_cache, torch.int16)
    M = q.shape[0]
    if base_pos + M > k_cache.shape[0]:
        raise ValueError("cache holds fewer than base_pos + M rows")
    out = torch.empty_like(q)
    check(lib().forge_hip_attn_prefill_f16kv(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), M, base_pos, heads,
                                             kv_heads, head_dim, flags, _stream()))
    return out


def attention_flash(q, k_cache, v_cache, seq_len, heads, kv_heads, head_dim, flags=0):
    """attention_flash over an fp16 cache: one query f32 [heads*hd] against seq_len rows."""
    from . import check, lib
    torch = _torch()
    q = _dev(q, torch.float32)
    k_cache, v_cache = _dev(k_cache, torch.int16), _dev(v_cache, torch.int16)
    if seq_len > k_cache.shape[0]:
        raise ValueError("cache holds fewer than seq_len rows")
    out = torch.empty_like(q)
    check(lib().forge_hip_attn_decode_f16kv(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), seq_len, heads, kv_heads,
                                            head_dim, flags, _stream()))
    return out


def attention_flash_paged(q, k_pool, v_pool, page_table, page_rows, seq_len, heads, kv_heads, head_dim):
    """attention_flash over a paged fp16 cache: pools [pages][page_rows][kv_heads*head_dim] (int16 bit patterns),
    page_table int32/uint32 [ceil(seq_len / page_rows)] of pool page indices."""
    from . import check, lib
    torch = _torch()
    q = _dev(q, torch.float32)
    pt = page_table.to(torch.int32).contiguous()
    out = torch.empty(heads * head_dim, dtype=torch.float32, device=q.device)
    check(lib().forge_hip_attn_decode_f16kv_paged(_ptr(q), _ptr(k_pool), _ptr(v_pool), _ptr(pt), page_rows, _ptr(out), seq_len,
                                                  heads, kv_heads, head_dim, _stream()))
    return out


def attention_flash_noalloc(q, k_cache, v_cache, seq_len, heads, kv_heads, head_dim, out):
    """attention_flash (fast mode) through the entry point that allocates nothing: the caller brings `out` (f32 [heads*hd],
    on the device) as well as the inputs, all already of the right type and contiguous."""
    from . import check, lib
    torch = _torch()
    for t, dt in ((q, torch.float32), (out, torch.float32), (k_cache, torch.int16), (v_cache, torch.int16)):
        if not (t.is_cuda and t.dtype == dt and t.is_contiguous()):
            raise ValueError("attention_flash_noalloc takes contiguous device tensors (q, out f32; caches int16 bit patterns)")
    if seq_len > k_cache.shape[0] or out.numel() != q.numel() or q.numel() != heads * head_dim:
        raise ValueError("cache holds fewer than seq_len rows, or q / out do not hold heads * head_dim values")
    if k_cache.numel() < seq_len * kv_heads * head_dim or v_cache.numel() < seq_len * kv_heads * head_dim:
        raise ValueError("a cache holds fewer than seq_len rows of kv_heads * head_dim values")
    check(lib().forge_hip_attn_decode_f16kv_noalloc(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), seq_len, heads, kv_heads,
                                                    head_dim, _stream()))
    return out


def attention_sliding_batch(q, k_cache, v_cache, base_pos, window, heads, kv_heads, head_dim, flags=0):
    """attention_sliding_batch over an fp16 cache: row r (position base_pos + r) sees the last `window` positions up to its own."""
    from . import check, lib
    torch = _torch()
    q = _dev(q, torch.float32)
    k_cache, v_cache = _dev(k_cache, torch.int16), _dev(v_cache, torch.int16)
    M = q.shape[0]
    if base_pos + M > k_cache.shape[0]:
        raise ValueError("cache holds fewer than base_pos + M rows")
    out = torch.empty_like(q)
    check(lib().forge_hip_attn_prefill_sliding_f16kv(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), M, base_pos, window,
                                                     heads, kv_heads, head_dim, flags, _stream()))
    return out


def attention_sliding(q, k_cache, v_cache, seq_len, window, heads, kv_heads, head_dim, flags=0):
    """attention_sliding over an fp16 cache: one query f32 [heads*hd] against the last min(window, seq_len) of seq_len rows."""
    from . import check, lib
    torch = _torch()
    q = _dev(q, torch.float32)
    k_cache, v_cache = _dev(k_cache, torch.int16), _dev(v_cache, torch.int16)
    if seq_len > k_cache.shape[0]:
        raise ValueError("cache holds fewer than seq_len rows")
    out = torch.empty_like(q)
    check(lib().forge_hip_attn_decode_sliding_f16kv(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), seq_len, window, heads,
                                                    kv_heads, head_dim, flags, _stream()))
    return out


def argmax(x):
    from . import check, lib
    torch = _torch()
    x = _dev(x, torch.float32)
    out = torch.empty(1, dtype=torch.int32, device=x.device)
    check(lib().forge_hip_argmax(_ptr(x), x.numel(), _ptr(out), _stream()))
    return int(out.item())
