"""GGUF on the input side: a writer for (synthetic) models and the host-side mirror of the library's reader.

The reference reads GGUF with `gguf::parse` (crates/forgellm-frontend/src/gguf.rs:484-551), takes the model
configuration from the metadata (crates/forgellm-cli/src/main.rs:700-830) and turns the tensors into `weights.bin`
with `forge export-weights` (main.rs:2585-2757).  `GgufFile` below is those three steps on libforge_hip.so;
`write_gguf` / `model_to_gguf` produce files in the layout `parse` reads (the same layout the reference's own
tests build, gguf.rs:559-604), so that a seeded synthetic model can travel as a GGUF file.
"""
import ctypes as C
import struct

import numpy as np

MAGIC = 0x46554747          # gguf.rs:18
F32, F16, Q4_0, Q8_0, BF16 = 0, 1, 2, 8, 30
Q4_1, Q4_K, Q5_K, Q6_K, Q8_K = 3, 12, 13, 14, 15

# GGUF metadata value type ids (gguf.rs:447-476)
U8, I8, U16, I16, U32, I32, FLOAT32, BOOL, STRING, ARRAY, U64, I64, FLOAT64 = range(13)
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", FLOAT32: "<f", BOOL: "<B", U64: "<Q", I64: "<q",
           FLOAT64: "<d"}


def _string(s) -> bytes:
    b = s if isinstance(s, bytes) else s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def encode_value(vtype: int, value) -> bytes:
    """The bytes of one metadata value.  An array is `(element_type, [values])`."""
    if vtype == STRING:
        return _string(value)
    if vtype == ARRAY:
        etype, items = value
        return struct.pack("<IQ", etype, len(items)) + b"".join(encode_value(etype, v) for v in items)
    return struct.pack(_SCALAR[vtype], value)


def write_gguf(metadata, tensors, version: int = 3, alignment: int = 32, path=None) -> bytes:
    """metadata: [(key, value_type, value)]; tensors: [(name, dims, ggml_type, data bytes or None)].
    Tensor data follows the descriptors, each tensor padded to `alignment` (a descriptor without data gets
    offset 0 and no bytes).  `general.alignment` is added when the alignment is not the default 32."""
    metadata = list(metadata)
    if alignment != 32 and not any(k == "general.alignment" for k, _, _ in metadata):
        metadata.append(("general.alignment", U32, alignment))
    head = struct.pack("<IIQQ", MAGIC, version, len(tensors), len(metadata))
    for key, vtype, value in metadata:
        head += _string(key) + struct.pack("<I", vtype) + encode_value(vtype, value)
    offsets, off = [], 0
    for _, _, _, data in tensors:
        offsets.append(off)
        if data is not None:
            n = len(data) if not isinstance(data, np.ndarray) else data.nbytes
            off = (off + n + alignment - 1) // alignment * alignment
    for (name, dims, gtype, _), o in zip(tensors, offsets):
        head += _string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        head += struct.pack("<IQ", gtype, o)
    parts = [head]
    if any(d is not None for _, _, _, d in tensors):
        parts.append(b"\0" * (-len(head) % alignment))
        for _, _, _, data in tensors:
            if data is None:
                continue
            raw = data.tobytes() if isinstance(data, np.ndarray) else bytes(data)
            parts.append(raw + b"\0" * (-len(raw) % alignment))
    out = b"".join(parts)
    if path is not None:
        with open(path, "wb") as f:
            f.write(out)
    return out


def split_blob(cfg: dict, blob: np.ndarray) -> dict:
    """The tensors of a weights blob (export-weights order, main.rs:2714-2757) by GGUF tensor name:
    {name: (dims, ggml_type, bytes)} with dims in GGUF order (row length first)."""
    from .ops import block_bytes
    H, I = cfg["hidden"], cfg["inter"]
    QKS, KV, V = cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"], cfg["vocab"]
    wt, lt = cfg["wdtype"], cfg["lm_head_dtype"]
    blob = np.ascontiguousarray(blob, np.uint8)
    pos = [0]
    out = {}

    def take(name, n_rows, k, gtype):
        nbytes = n_rows * k * 4 if gtype == F32 else n_rows * k // 32 * block_bytes(gtype)
        out[name] = ([k, n_rows] if n_rows > 1 else [k], gtype, blob[pos[0]:pos[0] + nbytes])
        pos[0] += nbytes

    take("token_embd.weight", V, H, F32)
    for l in range(cfg["layers"]):
        take(f"blk.{l}.attn_norm.weight", 1, H, F32)
        take(f"blk.{l}.attn_q.weight", QKS, H, wt)
        take(f"blk.{l}.attn_k.weight", KV, H, wt)
        take(f"blk.{l}.attn_v.weight", KV, H, wt)
        if cfg.get("flags", 0) & 2:
            take(f"blk.{l}.attn_q.bias", 1, QKS, F32)
            take(f"blk.{l}.attn_k.bias", 1, KV, F32)
            take(f"blk.{l}.attn_v.bias", 1, KV, F32)
        take(f"blk.{l}.attn_output.weight", H, QKS, wt)
        take(f"blk.{l}.ffn_norm.weight", 1, H, F32)
        take(f"blk.{l}.ffn_gate.weight", I, H, wt)
        take(f"blk.{l}.ffn_up.weight", I, H, wt)
        take(f"blk.{l}.ffn_down.weight", H, I, wt)
    take("output_norm.weight", 1, H, F32)
    take("output.weight", V, H, lt)
    assert pos[0] == blob.size, (pos[0], blob.size)
    return out


def model_to_gguf(cfg: dict, blob: np.ndarray, tied: bool = True, arch: str = None, path=None, tokens: bool = False,
                  fused: bool = False) -> bytes:
    """A weights blob as a GGUF v3 file with the metadata keys load_config reads (main.rs:700-830).
    tied=True stores the embedding once, as the quantised `token_embd.weight` (what llama.cpp does for models with tied
    embeddings; the blob's f32 table must then be the dequantised lm_head, as `synth.make_weights_blob` makes it);
    tied=False stores the f32 table and `output.weight`.  tokens=True also writes a `tokenizer.ggml.tokens` array of
    `vocab` one-character strings, the key the vocabulary size is read from first."""
    if arch is None:
        # the reference ties QKV bias to the architecture; a window is Mistral's
        arch = "qwen2" if cfg.get("flags", 0) & 2 else "mistral" if cfg.get("sliding_window", 0) else "phi3" if fused else "llama"
    t = split_blob(cfg, blob)
    if fused:
        # the Phi-3 file layout (weight_loader.rs:425-427, 531-534): q|k|v rows in `attn_qkv.weight`, gate|up rows in `ffn_up.weight`
        fused_t = {}
        for name, (dims, gtype, data) in t.items():
            if name.endswith("attn_q.weight"):
                b = name[:-len("attn_q.weight")]
                k, v = t[b + "attn_k.weight"], t[b + "attn_v.weight"]
                fused_t[b + "attn_qkv.weight"] = ([dims[0], dims[1] + k[0][1] + v[0][1]], gtype, np.concatenate([data, k[2], v[2]]))
            elif name.endswith("ffn_gate.weight"):
                b = name[:-len("ffn_gate.weight")]
                u = t[b + "ffn_up.weight"]
                fused_t[b + "ffn_up.weight"] = ([dims[0], dims[1] + u[0][1]], gtype, np.concatenate([data, u[2]]))
            elif not name.endswith(("attn_k.weight", "attn_v.weight", "ffn_up.weight")):
                fused_t[name] = (dims, gtype, data)
        t = fused_t
    if tied:
        dims, gtype, data = t.pop("output.weight")
        t["token_embd.weight"] = (dims, gtype, data)
    meta = [
        ("general.architecture", STRING, arch),
        (f"{arch}.embedding_length", U32, cfg["hidden"]),
        (f"{arch}.block_count", U32, cfg["layers"]),
        (f"{arch}.attention.head_count", U32, cfg["heads"]),
        (f"{arch}.attention.head_count_kv", U32, cfg["kv_heads"]),
        (f"{arch}.feed_forward_length", U32, cfg["inter"]),
        (f"{arch}.context_length", U32, cfg["max_seq"]),
        (f"{arch}.attention.layer_norm_rms_epsilon", FLOAT32, cfg["rms_eps"]),
        (f"{arch}.rope.freq_base", FLOAT32, cfg["rope_theta"]),
    ]
    if cfg.get("sliding_window", 0):
        meta.append((f"{arch}.attention.sliding_window", U32, cfg["sliding_window"]))
    if tokens:
        meta.append(("tokenizer.ggml.tokens", ARRAY, (STRING, [chr(33 + i % 90) for i in range(cfg["vocab"])])))
    else:
        meta.append((f"{arch}.vocab_size", U32, cfg["vocab"]))
    return write_gguf(meta, [(n, d, g, b) for n, (d, g, b) in t.items()], path=path)


def dequant_ggml(ggml_type: int, data, n: int) -> np.ndarray:
    """`dequantize` of the reference's loader (weight_loader.rs:809-825) for one tensor's bytes."""
    from . import check, lib
    L = lib()
    _declare(L)
    raw = np.ascontiguousarray(np.frombuffer(data, np.uint8) if not isinstance(data, np.ndarray) else data, np.uint8)
    out = np.empty(n, np.float32)
    check(L.forge_hip_dequant_ggml(ggml_type, raw.ctypes.data_as(C.c_void_p), n, out.ctypes.data_as(C.c_void_p)))
    return out


class GgufFile:
    """A parsed GGUF file: `GGUFFile` of the reference (gguf.rs:287-341) on the library's parser."""

    def __init__(self, source):
        """source: a path (the file is memory-mapped) or bytes / a uint8 array (kept alive by this object)."""
        from . import check, lib
        L = lib()
        _declare(L)
        self._lib, self._check = L, check
        h = C.c_void_p()
        if isinstance(source, (str,)):
            check(L.forge_hip_gguf_open(source.encode(), C.byref(h)))
            self._keep = None
        else:
            self._keep = np.frombuffer(source, np.uint8) if not isinstance(source, np.ndarray) else np.ascontiguousarray(source, np.uint8)
            check(L.forge_hip_gguf_parse(self._keep.ctypes.data_as(C.c_void_p), self._keep.size, C.byref(h)))
        self._h = h
        self.version = int(L.forge_hip_gguf_version(h))
        self.alignment = int(L.forge_hip_gguf_alignment(h))
        self.tensor_data_offset = int(L.forge_hip_gguf_tensor_data_offset(h))
        self.metadata_count = int(L.forge_hip_gguf_metadata_count(h))
        self.tensors = []
        for i in range(int(L.forge_hip_gguf_tensor_count(h))):
            name, nd, dims = C.c_char_p(), C.c_uint32(), (C.c_uint64 * 4)()
            gtype, off, size = C.c_uint32(), C.c_uint64(), C.c_uint64()
            check(L.forge_hip_gguf_tensor(h, i, C.byref(name), C.byref(nd), dims, C.byref(gtype), C.byref(off), C.byref(size)))
            self.tensors.append({"name": name.value.decode(), "dimensions": [int(dims[k]) for k in range(nd.value)],
                                 "ggml_type": int(gtype.value), "offset": int(off.value), "data_size": int(size.value)})

    def tensor(self, name):
        i = int(self._lib.forge_hip_gguf_find_tensor(self._h, name.encode()))
        return None if i < 0 else self.tensors[i]

    def meta(self, key):
        """The value of a metadata key: int / float / bool / str; an array gives (element_type, count).  None if absent."""
        vtype, bits, s, et, cnt = C.c_uint32(), C.c_uint64(), C.c_char_p(), C.c_uint32(), C.c_uint64()
        rc = self._lib.forge_hip_gguf_meta(self._h, key.encode(), C.byref(vtype), C.byref(bits), C.byref(s), C.byref(et), C.byref(cnt))
        if rc != 0:
            return None
        t, b = int(vtype.value), int(bits.value)
        if t == STRING:
            return s.value.decode()
        if t == ARRAY:
            return (int(et.value), int(cnt.value))
        if t == BOOL:
            return bool(b)
        raw = struct.pack("<Q", b)
        return struct.unpack_from(_SCALAR[t], raw)[0]

    def config(self, max_seq: int = 0, flags: int = 0) -> dict:
        from . import Config
        c = Config()
        self._check(self._lib.forge_hip_gguf_config(self._h, max_seq, flags, C.byref(c)))
        return {k: getattr(c, k) for k, _ in Config._fields_}

    def config_mixed(self, max_seq: int = 0, flags: int = 0):
        """detect_gguf_proj_dtypes on top of load_config (crates/forgellm-cli/src/main.rs:608-680, 782-793): the
        configuration, the storage formats of (q, k, v, o, gate, up, down) as GGML type ids, and the embedding table's
        (1 = dense).  config["lm_head_dtype"] is the lm_head category's format."""
        from . import Config
        c = Config()
        pd = np.zeros(7, np.uint32)
        embed = C.c_uint32()
        self._check(self._lib.forge_hip_gguf_config_mixed(self._h, max_seq, flags, C.byref(c), pd.ctypes.data_as(C.c_void_p), C.byref(embed)))
        return {name: getattr(c, name) for name, _ in Config._fields_}, [int(x) for x in pd], int(embed.value)

    def export_weights_mixed(self, cfg: dict, proj_dtypes) -> np.ndarray:
        """The weights.bin bytes with every projection in the format of its category (load_from_file_mixed_per_tensor,
        crates/forgellm-frontend/src/weight_loader.rs:152-238; blob order main.rs:2714-2757)."""
        from . import Config
        from .hip_model import weights_nbytes_mixed
        c = Config(**cfg)
        pd = np.ascontiguousarray(proj_dtypes, dtype=np.uint32)
        out = np.empty(weights_nbytes_mixed(cfg, pd), np.uint8)
        self._check(self._lib.forge_hip_gguf_export_weights_mixed(self._h, C.byref(c), pd.ctypes.data_as(C.c_void_p),
                                                            out.ctypes.data_as(C.c_void_p), out.size))
        return out

    def export_weights(self, cfg: dict) -> np.ndarray:
        from . import Config
        c = Config(**cfg)
        n = int(self._lib.forge_hip_weights_nbytes(C.byref(c)))
        out = np.empty(n, np.uint8)
        self._check(self._lib.forge_hip_gguf_export_weights(self._h, C.byref(c), out.ctypes.data_as(C.c_void_p), n))
        return out

    def close(self):
        if getattr(self, "_h", None):
            self._lib.forge_hip_gguf_close(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _declare(L):
    if getattr(L, "_gguf_declared", False):
        return
    vp, u32, u64, i32 = C.c_void_p, C.c_uint32, C.c_uint64, C.c_int32
    from . import Config
    L.forge_hip_gguf_open.restype = i32
    L.forge_hip_gguf_open.argtypes = [C.c_char_p, C.POINTER(vp)]
    L.forge_hip_gguf_parse.restype = i32
    L.forge_hip_gguf_parse.argtypes = [vp, u64, C.POINTER(vp)]
    L.forge_hip_gguf_close.restype = None
    L.forge_hip_gguf_close.argtypes = [vp]
    L.forge_hip_gguf_version.restype = u32
    L.forge_hip_gguf_version.argtypes = [vp]
    for f in ("alignment", "tensor_data_offset", "tensor_count", "metadata_count"):
        fn = getattr(L, "forge_hip_gguf_" + f)
        fn.restype = u64
        fn.argtypes = [vp]
    L.forge_hip_gguf_tensor.restype = i32
    L.forge_hip_gguf_tensor.argtypes = [vp, u64, C.POINTER(C.c_char_p), C.POINTER(u32), C.POINTER(u64), C.POINTER(u32), C.POINTER(u64),
                                        C.POINTER(u64)]
    L.forge_hip_gguf_find_tensor.restype = C.c_int64
    L.forge_hip_gguf_find_tensor.argtypes = [vp, C.c_char_p]
    L.forge_hip_gguf_meta.restype = i32
    L.forge_hip_gguf_meta.argtypes = [vp, C.c_char_p, C.POINTER(u32), C.POINTER(u64), C.POINTER(C.c_char_p), C.POINTER(u32), C.POINTER(u64)]
    L.forge_hip_gguf_config.restype = i32
    L.forge_hip_gguf_config.argtypes = [vp, u32, u32, C.POINTER(Config)]
    L.forge_hip_gguf_export_weights.restype = i32
    L.forge_hip_gguf_export_weights.argtypes = [vp, C.POINTER(Config), vp, u64]
    L.forge_hip_dequant_ggml.restype = i32
    L.forge_hip_dequant_ggml.argtypes = [u32, vp, u64, vp]
    L.forge_hip_model_create_from_gguf.restype = i32
    L.forge_hip_model_create_from_gguf.argtypes = [C.c_char_p, u32, u32, C.POINTER(vp)]
    L._gguf_declared = True


def quantize_kquant(ggml_type: int, x) -> np.ndarray:
    """quantize_f32_to_q4_k / quantize_f32_to_q6_k (crates/forgellm-frontend/src/weight_loader.rs:1773-1882, 2025-2140):
    f32 array -> ceil(n / 256) super-blocks of 144 (Q4_K, type 12) or 210 (Q6_K, type 14) bytes."""
    from . import check, lib
    L = lib()
    _declare(L)
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty((x.size + 255) // 256 * (144 if ggml_type == 12 else 210), np.uint8)
    check(L.forge_hip_quantize_kquant(ggml_type, x.ctypes.data_as(C.c_void_p), x.size, out.ctypes.data_as(C.c_void_p)))
    return out
