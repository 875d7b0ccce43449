"""ctypes binding of the CPU oracle (oracle/forge_oracle.cpp).

TEST INFRASTRUCTURE — only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg may import this module.  The HIP product never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libforge_oracle.so")


def build(force=False):
    """Compile the oracle with oracle/Makefile."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-C", _HERE, "-s"])


class Config(C.Structure):
    _fields_ = [
        ("hidden", C.c_uint32), ("inter", C.c_uint32), ("layers", C.c_uint32), ("heads", C.c_uint32),
        ("kv_heads", C.c_uint32), ("head_dim", C.c_uint32), ("vocab", C.c_uint32), ("max_seq", C.c_uint32),
        ("rms_eps", C.c_float), ("rope_theta", C.c_float),
        ("wdtype", C.c_uint32), ("lm_head_dtype", C.c_uint32), ("flags", C.c_uint32),
        ("sliding_window", C.c_uint32),
    ]


_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    L = C.CDLL(_LIB_PATH)
    vp, i64, i32, f32 = C.c_void_p, C.c_int64, C.c_int, C.c_float
    L.fo_weights_nbytes.restype = C.c_uint64
    L.fo_weights_nbytes.argtypes = [C.POINTER(Config)]
    L.fo_model_create.restype = vp
    L.fo_model_create.argtypes = [C.POINTER(Config), vp, C.c_uint64, i32, i32]
    L.fo_model_create_mixed.restype = vp
    L.fo_model_create_mixed.argtypes = [C.POINTER(Config), vp, vp, C.c_uint64, i32, i32]
    L.fo_weights_nbytes_mixed.restype = C.c_uint64
    L.fo_weights_nbytes_mixed.argtypes = [C.POINTER(Config), vp]
    L.fo_model_destroy.argtypes = [vp]
    L.fo_model_reset.argtypes = [vp]
    L.fo_model_pos.restype = i64
    L.fo_model_pos.argtypes = [vp]
    L.fo_forward.restype = i32
    L.fo_forward.argtypes = [vp, C.c_uint32, vp]
    L.fo_prefill_batched.restype = i32
    L.fo_prefill_batched.argtypes = [vp, vp, i64, vp]
    L.fo_model_read_kv.argtypes = [vp, i32, i32, vp]
    L.fo_model_write_kv.restype = i32
    L.fo_model_write_kv.argtypes = [vp, i32, i64, vp, vp]
    L.fo_f16_to_f32.restype = f32
    L.fo_f16_to_f32.argtypes = [C.c_uint16]
    L.fo_f32_to_f16.restype = C.c_uint16
    L.fo_f32_to_f16.argtypes = [f32]
    L.fo_f32_to_f16_array.argtypes = [vp, i64, vp]
    L.fo_f16_to_f32_array.argtypes = [vp, i64, vp]
    L.fo_dequant.argtypes = [i32, vp, i64, vp]
    L.fo_quantize_weights.argtypes = [i32, vp, i64, vp]
    L.fo_quantize_act.argtypes = [vp, i64, vp]
    L.fo_block_isums.argtypes = [i32, vp, vp, i64, i64, vp]
    L.fo_dot_a.restype = f32
    L.fo_dot_a.argtypes = [i32, vp, vp, i64, i32]
    L.fo_dot_b.restype = f32
    L.fo_dot_b.argtypes = [i32, vp, vp, i64]
    L.fo_matmul_vec.argtypes = [i32, i32, vp, vp, vp, i64, i64]
    L.fo_matmul_mat.argtypes = [i32, i32, vp, i64, vp, vp, i64, i64]
    L.fo_rms_norm.argtypes = [vp, vp, vp, i64, f32, i32]
    L.fo_silu_mul.argtypes = [vp, vp, vp, i64]
    L.fo_softmax.argtypes = [vp, i64]
    L.fo_rope.argtypes = [vp, i64, i32, i32, f32]
    L.fo_rope_table.argtypes = [i64, i32, f32, vp, vp]
    L.fo_quantize_kv.restype = f32
    L.fo_quantize_kv.argtypes = [vp, i64, vp]
    L.fo_expf_array.argtypes = [vp, i64, vp]
    L.fo_argmax.restype = C.c_uint32
    L.fo_argmax.argtypes = [vp, i64]
    L.fo_attention.argtypes = [i32, i32, vp, vp, vp, vp, vp, vp, i64, i64, i32, i32, i32, i64]
    L.fo_row_order.argtypes = [i32, i64, i64, i32, vp]
    L.fo_num_threads.restype = i32
    L.fo_set_num_threads.argtypes = [i32]
    _lib = L
    return L


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a):
    return np.ascontiguousarray(a, dtype=np.uint8)


VARIANT_A, VARIANT_B = 0, 1
KV_INT8, KV_F16 = 0, 1
Q8_0, Q4_0 = 8, 2


def block_bytes(wdtype):
    return 34 if wdtype == Q8_0 else 18


def f16_to_f32(bits):
    b = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(b.shape, np.float32)
    lib().fo_f16_to_f32_array(_p(b), b.size, _p(out))
    return out


def f32_to_f16(x):
    x = _f32(x)
    out = np.empty(x.shape, np.uint16)
    lib().fo_f32_to_f16_array(_p(x), x.size, _p(out))
    return out


def dequant(wdtype, data, n):
    data = _u8(data)
    out = np.empty(n, np.float32)
    lib().fo_dequant(wdtype, _p(data), n, _p(out))
    return out


def quantize_weights(wdtype, x):
    """Row-major weights [N][K] (or flat) -> raw GGUF block bytes."""
    x = _f32(x)
    n = x.size
    out = np.empty((n + 31) // 32 * block_bytes(wdtype), np.uint8)
    lib().fo_quantize_weights(wdtype, _p(x), n, _p(out))
    return out


def quantize_act(x):
    x = _f32(x)
    out = np.empty((x.size + 31) // 32 * 34, np.uint8)
    lib().fo_quantize_act(_p(x), x.size, _p(out))
    return out


def block_isums(wdtype, a_q8, w, k, n):
    a_q8, w = _u8(a_q8), _u8(w)
    out = np.empty((n, k // 32), np.int32)
    lib().fo_block_isums(wdtype, _p(a_q8), _p(w), k, n, _p(out))
    return out


def dot_a(wdtype, a_q8, w, k, seq=True):
    return float(lib().fo_dot_a(wdtype, _p(_u8(a_q8)), _p(_u8(w)), k, int(seq)))


def dot_b(wdtype, x, w, k):
    return float(lib().fo_dot_b(wdtype, _p(_f32(x)), _p(_u8(w)), k))


def matmul_vec(wdtype, variant, x, w, k, n):
    x, w = _f32(x), _u8(w)
    out = np.empty(n, np.float32)
    lib().fo_matmul_vec(wdtype, variant, _p(out), _p(x), _p(w), k, n)
    return out


def dot_kquant(ggml_type, a_q8, w, k):
    """dot_q4_k_q8_0 (ggml_type 12) / dot_q6_k_q8_0 (14) of a weight row with Q8_0-quantised activation blocks."""
    L = lib()
    L.fo_dot_kquant.restype = C.c_float
    L.fo_dot_kquant.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int64]
    return float(L.fo_dot_kquant(ggml_type, _p(_u8(a_q8)), _p(_u8(w)), k))


def matmul_vec_kquant(ggml_type, x, w, k, n):
    """matmul_vec_q4_k_KxN / matmul_vec_q6_k_KxN: quantise x to Q8_0 blocks, one dot per row."""
    L = lib()
    L.fo_matmul_vec_kquant.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64]
    x, w = _f32(x), _u8(w)
    out = np.empty(n, np.float32)
    L.fo_matmul_vec_kquant(ggml_type, _p(out), _p(x), _p(w), k, n)
    return out


def matmul_mat(wdtype, variant, x, w, m, k, n):
    x, w = _f32(x), _u8(w)
    out = np.empty((m, n), np.float32)
    lib().fo_matmul_mat(wdtype, variant, _p(out), m, _p(x), _p(w), k, n)
    return out


def rms_norm(x, w, eps, variant=VARIANT_A):
    x, w = _f32(x), _f32(w)
    out = np.empty_like(x)
    lib().fo_rms_norm(_p(out), _p(x), _p(w), x.size, eps, variant)
    return out


def silu_mul(g, u):
    g, u = _f32(g), _f32(u)
    out = np.empty_like(g)
    lib().fo_silu_mul(_p(out), _p(g), _p(u), g.size)
    return out


def softmax(v):
    v = _f32(v).copy()
    lib().fo_softmax(_p(v), v.size)
    return v


def rope(data, pos, head_dim, num_heads, theta):
    d = _f32(data).copy()
    lib().fo_rope(_p(d), pos, head_dim, num_heads, theta)
    return d


def rope_table(n_pos, head_dim, theta):
    c = np.empty((n_pos, head_dim // 2), np.float32)
    s = np.empty_like(c)
    lib().fo_rope_table(n_pos, head_dim, theta, _p(c), _p(s))
    return c, s


def quantize_kv(v):
    v = _f32(v)
    out = np.empty(v.size, np.int8)
    scale = lib().fo_quantize_kv(_p(v), v.size, _p(out))
    return out, float(scale)


def expf(x):
    """The C library's expf, element-wise."""
    x = _f32(x)
    out = np.empty_like(x)
    lib().fo_expf_array(_p(x), x.size, _p(out))
    return out


def argmax(v):
    v = _f32(v)
    return int(lib().fo_argmax(_p(v), v.size))


def row_order(wdtype, k, n, mode):
    """Output rows of a variant-A matmul that take the 4-accumulator order; mode: 'vec' | 'lm_forward' | 'lm_prefill' | 'mat'."""
    out = np.empty(n, np.uint8)
    lib().fo_row_order(wdtype, k, n, {"vec": 0, "lm_forward": 1, "lm_prefill": 2, "mat": 3}[mode], _p(out))
    return [int(i) for i in np.flatnonzero(out)]


def attention(kind, q, k, v, seq_or_m, nh, nkv, hd, base_pos=0, ks=None, vs=None, window=0):
    """kind: 'std' | 'flash' | 'flash_batch' | 'sliding' | 'sliding_batch' (the last two need `window` >= 1).
    k, v: int8 (with ks, vs) or uint16 fp16 bits."""
    kinds = {"std": 0, "flash": 1, "flash_batch": 2, "sliding": 3, "sliding_batch": 4}
    if kinds[kind] >= 3 and window < 1:
        raise ValueError("sliding attention needs a window of at least 1")
    q = _f32(q)
    if k.dtype == np.int8:
        kvmode, ks, vs = KV_INT8, _f32(ks), _f32(vs)
    else:
        assert k.dtype == np.uint16 and v.dtype == np.uint16
        kvmode = KV_F16
    k, v = np.ascontiguousarray(k), np.ascontiguousarray(v)
    out = np.empty_like(q)
    lib().fo_attention(kinds[kind], kvmode, _p(out), _p(q), _p(k), _p(v), _p(ks), _p(vs), seq_or_m, base_pos, nh, nkv, hd, window)
    return out


def num_threads():
    return int(lib().fo_num_threads())


def set_num_threads(n):
    lib().fo_set_num_threads(int(n))


class Model:
    """Oracle model: forward / forward_prefill_batched over a weights.bin blob."""

    def __init__(self, cfg: dict, blob, variant=VARIANT_A, kvmode=KV_F16, proj_dtypes=None):
        """proj_dtypes (optional): storage format of q, k, v, o, gate, up, down as GGML type ids (8, 2, 12, 14); the
        lm_head's is cfg["lm_head_dtype"].  Default: cfg["wdtype"] for all seven."""
        self.cfg = Config(**cfg)
        blob = _u8(blob)
        self.vocab = cfg["vocab"]
        if proj_dtypes is None:
            self._h = lib().fo_model_create(C.byref(self.cfg), _p(blob), blob.size, variant, kvmode)
        else:
            pd = np.ascontiguousarray(proj_dtypes, dtype=np.uint32)
            assert pd.size == 7
            self._h = lib().fo_model_create_mixed(C.byref(self.cfg), _p(pd), _p(blob), blob.size, variant, kvmode)
        if not self._h:
            raise ValueError("oracle: weights blob size does not match the config")

    def forward(self, token):
        out = np.empty(self.vocab, np.float32)
        rc = lib().fo_forward(self._h, int(token), _p(out))
        if rc != 0:
            raise RuntimeError(f"oracle forward failed: {rc}")
        return out

    def prefill_batched(self, tokens, want_logits=True):
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        out = np.empty(self.vocab, np.float32) if want_logits else None
        rc = lib().fo_prefill_batched(self._h, _p(t), t.size, _p(out))
        if rc != 0:
            raise RuntimeError(f"oracle prefill failed: {rc}")
        return out

    def read_kv(self, layer, which):
        n = self.pos
        kv = self.cfg.kv_heads * self.cfg.head_dim
        out = np.empty((n, kv), np.float32)
        lib().fo_model_read_kv(self._h, layer, which, _p(out))
        return out

    def adopt_context(self, other):
        """Take over the cached context of another oracle model of the same shape (its K/V rows pass through this
        model's own cache write); the position becomes the other model's."""
        for l in range(self.cfg.layers):
            k, v = other.read_kv(l, 0), other.read_kv(l, 1)
            rc = lib().fo_model_write_kv(self._h, l, k.shape[0], _p(k), _p(v))
            if rc != 0:
                raise RuntimeError(f"oracle write_kv failed: {rc}")

    @property
    def pos(self):
        return int(lib().fo_model_pos(self._h))

    def reset(self):
        lib().fo_model_reset(self._h)

    def close(self):
        if self._h:
            lib().fo_model_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def weights_nbytes_mixed(cfg: dict, proj_dtypes):
    pd = np.ascontiguousarray(proj_dtypes, dtype=np.uint32)
    return int(lib().fo_weights_nbytes_mixed(C.byref(Config(**cfg)), _p(pd)))


def weights_nbytes(cfg: dict):
    c = Config(**cfg)
    return int(lib().fo_weights_nbytes(C.byref(c)))
