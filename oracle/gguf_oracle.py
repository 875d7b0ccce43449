"""TEST INFRASTRUCTURE ONLY — CPU restatement of the reference's GGUF input path, used by tests/ as the checker of
the library's reader.  Nothing the product ships imports this file.

Follows, step by step:
  parse            crates/forgellm-frontend/src/gguf.rs:484-551 (reader helpers :367-481)
  GGMLType sizes   gguf.rs:207-258;  GGUFTensorInfo::data_size gguf.rs:278-284
  load_config      crates/forgellm-cli/src/main.rs:700-830, dtype vote :479-555, lm_head dtype :567-581
  tensor names     crates/forgellm-frontend/src/weight_loader.rs:400-447
  export-weights   crates/forgellm-cli/src/main.rs:2585-2757 (blob order :2714-2757)
  dense dequant    weight_loader.rs:827-855; Q8_0 / Q4_0 dequant and the weight quantisers come from forge_oracle.cpp

Pinned by the reference's own unit tests for this path (gguf.rs:606-769: minimal v3 file, several tensors with
metadata, version 2, bad magic, unsupported version, data sizes, alignment; weight_loader.rs:3245-3259 and :3422-3656:
the Q4_1, Q4_K, Q5_K and Q6_K dequantiser fixtures), restated as byte strings in tests/test_gguf.py.  Q8_K has no
reference fixture: pinned by its closed form (scale * int8) only.  Where a GGUF tensor is stored in another format than the blob needs, the reference's exporter
writes bytes its own generated reader cannot consume (main.rs:2603-2626 handles only f32 -> Q4_0); this restatement
converts with the reference's dequantisers and quantisers instead, and says so here: that conversion is parity
unpinned (no reference test or fixture covers it).
"""
import struct

import numpy as np

MAGIC = 0x46554747
DEFAULT_ALIGNMENT = 32

# id: (elements per block, bytes per block), gguf.rs:207-258
TYPE_LAYOUT = {0: (1, 4), 1: (1, 2), 2: (32, 18), 3: (32, 20), 6: (32, 22), 7: (32, 24), 8: (32, 34), 9: (32, 40), 10: (256, 84),
               11: (256, 110), 12: (256, 144), 13: (256, 176), 14: (256, 210), 15: (256, 292), 16: (256, 66), 17: (256, 74),
               18: (256, 98), 19: (256, 50), 20: (32, 18), 21: (256, 110), 22: (256, 82), 23: (32, 36), 24: (1, 1), 25: (1, 2),
               26: (1, 4), 27: (1, 8), 28: (1, 8), 29: (256, 56), 30: (1, 2)}


class GgufError(ValueError):
    pass


class _Reader:
    def __init__(self, data):
        self.d, self.pos = bytes(data), 0

    def take(self, fmt):
        n = struct.calcsize(fmt)
        if self.pos + n > len(self.d):
            raise GgufError("unexpected end of file")
        v = struct.unpack_from(fmt, self.d, self.pos)[0]
        self.pos += n
        return v

    def string(self):
        n = self.take("<Q")
        if self.pos + n > len(self.d):
            raise GgufError("unexpected end of file")
        raw = self.d[self.pos:self.pos + n]
        self.pos += n
        try:
            return raw.decode("utf-8")
        except UnicodeDecodeError:
            raise GgufError("invalid UTF-8 in string")

    def value(self, t):
        fmts = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 10: "<Q", 11: "<q", 12: "<d"}
        if t in fmts:
            return (t, self.take(fmts[t]))
        if t == 7:
            return (t, self.take("<B") != 0)
        if t == 8:
            return (t, self.string())
        if t == 9:
            et = self.take("<I")
            n = self.take("<Q")
            return (t, (et, [self.value(et) for _ in range(n)]))
        raise GgufError(f"unsupported metadata value type: {t}")


def parse(data) -> dict:
    r = _Reader(data)
    magic = r.take("<I")
    if magic != MAGIC:
        raise GgufError(f"invalid GGUF magic number: got 0x{magic:08X}")
    version = r.take("<I")
    if version not in (2, 3):
        raise GgufError(f"unsupported GGUF version: {version} (supported: 2, 3)")
    n_tensors, n_meta = r.take("<Q"), r.take("<Q")
    meta = {}
    for _ in range(n_meta):
        key = r.string()
        meta[key] = r.value(r.take("<I"))
    tensors = []
    for _ in range(n_tensors):
        name = r.string()
        nd = r.take("<I")
        if nd > 4:
            raise GgufError(f"tensor dimension count {nd} exceeds maximum (4)")
        dims = [r.take("<Q") for _ in range(nd)]
        gtype = r.take("<I")
        if gtype not in TYPE_LAYOUT:
            raise GgufError(f"unsupported GGML type ID: {gtype}")
        tensors.append({"name": name, "dimensions": dims, "ggml_type": gtype, "offset": r.take("<Q")})
    al = meta.get("general.alignment")
    alignment = al[1] if al is not None and al[0] == 4 else DEFAULT_ALIGNMENT
    return {"version": version, "metadata": meta, "tensors": tensors, "alignment": alignment,
            "tensor_data_offset": (r.pos + alignment - 1) // alignment * alignment}


def numel(t) -> int:
    n = 1
    for d in t["dimensions"]:
        n *= d
    return n


def data_size(t) -> int:
    block, nbytes = TYPE_LAYOUT[t["ggml_type"]]
    return (numel(t) + block - 1) // block * nbytes


def _get(g, key, types):
    v = g["metadata"].get(key)
    return v[1] if v is not None and v[0] in types else None


def config(g, max_seq=0, flags=0) -> dict:
    arch = _get(g, "general.architecture", (8,)) or "unknown"
    if arch not in ("llama", "mistral", "qwen2", "phi3", "phi"):
        raise GgufError(f"unsupported GGUF architecture: {arch}")
    p = arch + "."
    hidden = _get(g, p + "embedding_length", (4,)) or 0
    layers = _get(g, p + "block_count", (4,)) or 0
    heads = _get(g, p + "attention.head_count", (4,)) or 0
    kv = _get(g, p + "attention.head_count_kv", (4,))
    kv = heads if kv is None else kv
    if hidden == 0 or layers == 0 or heads == 0:
        raise GgufError("could not extract model config from GGUF metadata")
    inter = _get(g, p + "feed_forward_length", (4,))
    inter = hidden * 4 if inter is None else inter
    tokens = g["metadata"].get("tokenizer.ggml.tokens")
    if tokens is not None and tokens[0] == 9:
        vocab = len(tokens[1][1])
    else:
        vocab = _get(g, p + "vocab_size", (10, 4))
        vocab = 32000 if vocab is None else vocab
    ctx = _get(g, p + "context_length", (10, 4))
    ctx = 2048 if ctx is None else ctx
    eps = _get(g, p + "attention.layer_norm_rms_epsilon", (6,))
    theta = _get(g, p + "rope.freq_base", (6,))
    q8 = q4 = q4k = f16 = f32 = 0
    as_q8 = {3, 20, 23, 6, 7, 9, 10, 11, 13, 14, 15, 16, 17, 22, 18, 21, 19, 29}
    for t in g["tensors"]:
        n = t["name"]
        if not (".weight" in n and "token_embd" not in n and "output.weight" not in n and "_norm" not in n):
            continue
        ty = t["ggml_type"]
        if ty == 8 or ty in as_q8:
            q8 += 1
        elif ty == 2:
            q4 += 1
        elif ty == 12:
            q4k += 1
        elif ty in (1, 30):
            f16 += 1
        elif ty == 0:
            f32 += 1
    total = q8 + q4 + q4k + f16 + f32
    if total == 0 or q4k > total // 2:
        raise GgufError("projection weights are neither mostly Q8_0 nor mostly Q4_0")
    if q8 > total // 2:
        wd = 8
    elif q4 > total // 2:
        wd = 2
    else:
        raise GgufError("projection weights are neither mostly Q8_0 nor mostly Q4_0")
    lm = wd
    ot = next((t for t in g["tensors"] if t["name"] in ("output.weight", "lm_head.weight")), None)
    if ot is not None:
        if ot["ggml_type"] in (2, 8):
            lm = ot["ggml_type"]
        elif ot["ggml_type"] in REQUANTISED_ON_LOAD:
            lm = 8
        elif ot["ggml_type"] not in (0, 1, 30):
            raise GgufError("output.weight has an unsupported GGML type")
    seq = max_seq or ctx
    window = _get(g, p + "attention.sliding_window", (4,))
    if window == 0:
        raise GgufError("a sliding window of 0 positions")
    f = np.float32
    return {"hidden": hidden, "inter": inter, "layers": layers, "heads": heads, "kv_heads": kv, "head_dim": hidden // heads,
            "vocab": vocab, "max_seq": seq, "rms_eps": float(f(1e-5) if eps is None else f(eps)),
            "rope_theta": float(f(10000.0) if theta is None else f(theta)), "wdtype": wd, "lm_head_dtype": lm,
            "flags": flags | (2 if arch == "qwen2" else 0),
            "sliding_window": window or 0}                  # qkv_bias goes with the architecture, main.rs:770


F = np.float32
REQUANTISED_ON_LOAD = (3, 12, 13, 14, 15)      # Q4_1, Q4_K, Q5_K, Q6_K, Q8_K become Q8_0 blocks when read, weight_loader.rs:219-229


def _half(oracle, blocks, off):
    return oracle.f16_to_f32(blocks[:, off:off + 2].copy().view("<u2")[:, 0]).astype(F)


def _scale_min_k4(sc):
    """get_scale_min_k4 (weight_loader.rs:977-987) for j = 0..7 of every block: two uint8 arrays [nblocks][8]."""
    s = np.empty((sc.shape[0], 8), np.uint8)
    m = np.empty((sc.shape[0], 8), np.uint8)
    s[:, :4] = sc[:, 0:4] & 63
    m[:, :4] = sc[:, 4:8] & 63
    s[:, 4:] = (sc[:, 8:12] & 0x0F) | ((sc[:, 0:4] >> 6) << 4)
    m[:, 4:] = (sc[:, 8:12] >> 4) | ((sc[:, 4:8] >> 6) << 4)
    return s, m


def dequant_ggml(oracle, ty, raw, n):
    """`dequantize` (weight_loader.rs:809-825), numpy float32 in the reference's order of operations."""
    raw = np.frombuffer(raw, np.uint8) if not isinstance(raw, np.ndarray) else raw
    if ty == 0:
        return raw[:4 * n].view("<f4").copy()
    if ty == 1:
        return oracle.f16_to_f32(raw[:2 * n].view("<u2"))
    if ty == 30:
        return (raw[:2 * n].view("<u2").astype(np.uint32) << 16).view(np.float32)
    if ty in (8, 2):
        return oracle.dequant(ty, raw, n)
    block, nbytes = TYPE_LAYOUT[ty]
    nb = (n + block - 1) // block
    b = raw[:nb * nbytes].reshape(nb, nbytes)
    out = np.empty((nb, block), F)
    if ty == 3:                                   # Q4_1, weight_loader.rs:931-965
        scale, mn = _half(oracle, b, 0)[:, None], _half(oracle, b, 2)[:, None]
        out[:, :16] = (b[:, 4:] & 0x0F).astype(F) * scale + mn
        out[:, 16:] = (b[:, 4:] >> 4).astype(F) * scale + mn
    elif ty in (12, 13):                          # Q4_K :1146-1201, Q5_K :1071-1135
        d, dmin = _half(oracle, b, 0), _half(oracle, b, 2)
        s, m = _scale_min_k4(b[:, 4:16])
        qs = b[:, (48 if ty == 13 else 16):].reshape(nb, 4, 32)
        lo, hi = (qs & 0x0F).astype(np.uint32), (qs >> 4).astype(np.uint32)
        if ty == 13:
            qh = b[:, 16:48]
            for c in range(4):
                lo[:, c] += np.where(qh & (1 << (2 * c)), 16, 0).astype(np.uint32)
                hi[:, c] += np.where(qh & (2 << (2 * c)), 16, 0).astype(np.uint32)
        o = out.reshape(nb, 4, 64)
        for c in range(4):
            d1, m1 = (d * s[:, 2 * c].astype(F))[:, None], (dmin * m[:, 2 * c].astype(F))[:, None]
            d2, m2 = (d * s[:, 2 * c + 1].astype(F))[:, None], (dmin * m[:, 2 * c + 1].astype(F))[:, None]
            o[:, c, :32] = d1 * lo[:, c].astype(F) - m1
            o[:, c, 32:] = d2 * hi[:, c].astype(F) - m2
    elif ty == 14:                                # Q6_K, weight_loader.rs:997-1057
        ql, qh = b[:, :128].reshape(nb, 2, 64), b[:, 128:192].reshape(nb, 2, 32)
        sc = b[:, 192:208].view(np.int8).reshape(nb, 2, 8).astype(F)
        d = _half(oracle, b, 208)[:, None, None]
        o = out.reshape(nb, 2, 4, 32)
        q = np.empty((nb, 2, 4, 32), np.int32)
        q[:, :, 0] = (ql[:, :, :32] & 0x0F) | ((qh & 3) << 4)
        q[:, :, 1] = (ql[:, :, 32:] & 0x0F) | (((qh >> 2) & 3) << 4)
        q[:, :, 2] = (ql[:, :, :32] >> 4) | (((qh >> 4) & 3) << 4)
        q[:, :, 3] = (ql[:, :, 32:] >> 4) | (((qh >> 6) & 3) << 4)
        q -= 32
        for k in range(4):
            scale = np.repeat(sc[:, :, 2 * k:2 * k + 2], 16, axis=2)          # is = l / 16 picks scale 2k or 2k + 1
            o[:, :, k] = d * scale * q[:, :, k].astype(F)
    elif ty == 15:                                # Q8_K, weight_loader.rs:1206-1229
        scale = b[:, :4].copy().view("<f4")
        out[:] = scale * b[:, 4:260].view(np.int8).astype(F)
    else:
        raise GgufError(f"unsupported GGML type {ty}")
    return out.reshape(-1)[:n].copy()


def _tensor_f32(oracle, g, data, t):
    """The tensor's values as the reference holds them after loading."""
    n = numel(t)
    raw = np.frombuffer(data, np.uint8, data_size(t), g["tensor_data_offset"] + t["offset"])
    ty = t["ggml_type"]
    if ty not in (0, 1, 30, 8, 2) + REQUANTISED_ON_LOAD:
        raise GgufError(f"tensor {t['name']}: unsupported GGML type {ty}")
    v = dequant_ggml(oracle, ty, raw, n)
    if ty in REQUANTISED_ON_LOAD:
        v = oracle.dequant(8, oracle.quantize_weights(8, v), n)
    return v


def export_weights(oracle, g, data, cfg) -> np.ndarray:
    """The weights.bin bytes for `cfg` (main.rs:2714-2757).  `oracle` is the oracle.oracle module."""
    data = bytes(data)
    by_name = {t["name"]: t for t in g["tensors"]}

    def find(name, n):
        t = by_name.get(name)
        if t is None:
            raise GgufError(f"weight not found: {name}")
        if numel(t) != n:
            raise GgufError(f"tensor {name} has the wrong number of elements")
        if g["tensor_data_offset"] + t["offset"] + data_size(t) > len(data):
            raise GgufError(f"tensor {name} extends past end of file")
        return t

    def f32(name, n):
        return _tensor_f32(oracle, g, data, find(name, n)).astype("<f4").view(np.uint8)

    def quant(name, n, wd):
        t = find(name, n)
        if t["ggml_type"] == wd:
            return np.frombuffer(data, np.uint8, data_size(t), g["tensor_data_offset"] + t["offset"])
        return oracle.quantize_weights(wd, _tensor_f32(oracle, g, data, t))

    def quant_parts(name, sizes, wd):
        """A fused Phi-3 tensor cut into parts (split_weight_three / split_weight_two, weight_loader.rs:543-583, 641-700):
        the loader converts the whole tensor first, the split cuts the result at element counts."""
        whole = np.ascontiguousarray(quant(name, sum(sizes), wd), np.uint8)
        bb = 34 if wd == 8 else 18
        out, at = [], 0
        for n in sizes:
            if n % 32:
                raise GgufError(f"fused tensor {name} cannot be split on block boundaries")
            out.append(whole[at // 32 * bb:(at + n) // 32 * bb])
            at += n
        return out

    H, I = cfg["hidden"], cfg["inter"]
    QKS, KV, V = cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"], cfg["vocab"]
    wd = cfg["wdtype"]
    parts = [f32("token_embd.weight", V * H)]
    for l in range(cfg["layers"]):
        b = f"blk.{l}."
        parts.append(f32(b + "attn_norm.weight", H))
        if b + "attn_q.weight" not in by_name and b + "attn_qkv.weight" in by_name:
            parts += quant_parts(b + "attn_qkv.weight", [QKS * H, KV * H, KV * H], wd)
        else:
            parts += [quant(b + "attn_q.weight", QKS * H, wd), quant(b + "attn_k.weight", KV * H, wd), quant(b + "attn_v.weight", KV * H, wd)]
        if cfg["flags"] & 2:
            parts += [f32(b + "attn_q.bias", QKS), f32(b + "attn_k.bias", KV), f32(b + "attn_v.bias", KV)]
        parts += [quant(b + "attn_output.weight", H * QKS, wd), f32(b + "ffn_norm.weight", H)]
        up = by_name.get(b + "ffn_up.weight")
        if b + "ffn_gate.weight" not in by_name and up is not None and numel(up) == 2 * I * H:
            parts += quant_parts(b + "ffn_up.weight", [I * H, I * H], wd)
        else:
            parts += [quant(b + "ffn_gate.weight", I * H, wd), quant(b + "ffn_up.weight", I * H, wd)]
        parts.append(quant(b + "ffn_down.weight", H * I, wd))
    parts.append(f32("output_norm.weight", H))
    lm_name = "output.weight" if "output.weight" in by_name else "lm_head.weight" if "lm_head.weight" in by_name else "token_embd.weight"
    parts.append(quant(lm_name, V * H, cfg["lm_head_dtype"]))
    return np.concatenate([np.ascontiguousarray(p, np.uint8) for p in parts])


# ---------------------------------------------------------------------------------------------------------------------
# A storage format per projection category: detect_gguf_proj_dtypes (main.rs:608-680), load_from_file_mixed_per_tensor
# (weight_loader.rs:152-238), and the K-quant weight quantisers that loader calls (weight_loader.rs:1666-1882, 1987-2140).
# The quantisers are written here in array form (all sub-blocks at once, f32 sums kept sequential), from the reference's text;
# the reference holds no input/output vectors for them, only quality bounds (weight_loader.rs:2735-2990), which
# tests/test_gguf.py applies to the reference tests' own inputs: beyond those bounds their parity is unpinned.

DENSE = 1
_CATS = ("embed", "q", "k", "v", "o", "gate", "up", "down", "lm_head")
_SUFFIX = {"attn_q.weight": "q", "attn_k.weight": "k", "attn_v.weight": "v", "attn_output.weight": "o", "ffn_gate.weight": "gate",
           "ffn_up.weight": "up", "ffn_down.weight": "down"}
_RANK = {DENSE: 5, 8: 4, 14: 3, 12: 2, 2: 1}


def _category(name):
    """ProjCategory::from_gguf_name, ir.rs:382-401."""
    if name == "token_embd.weight":
        return "embed"
    if name in ("output.weight", "lm_head.weight"):
        return "lm_head"
    if not name.startswith("blk."):
        return None
    rest = name[4:]
    if "." not in rest:
        return None
    return _SUFFIX.get(rest[rest.index(".") + 1:])


def _storage(ty):
    """ggml_type_storage_dtype, main.rs:586-599."""
    return ty if ty in (8, 2, 12, 14) else DENSE if ty in (0, 1, 30) else None


def _majority(g):
    """detect_gguf_dtype, main.rs:479-555: 8, 2, 12, or None for a dense majority."""
    q8 = q4 = q4k = f16 = f32 = 0
    as_q8 = {3, 20, 23, 6, 7, 9, 10, 11, 13, 14, 15, 16, 17, 22, 18, 21, 19, 29}
    for t in g["tensors"]:
        n = t["name"]
        if not (".weight" in n and "token_embd" not in n and "output.weight" not in n and "_norm" not in n):
            continue
        ty = t["ggml_type"]
        q8 += ty == 8 or ty in as_q8
        q4 += ty == 2
        q4k += ty == 12
        f16 += ty in (1, 30)
        f32 += ty == 0
    total = q8 + q4 + q4k + f16 + f32
    if total == 0:
        return None
    return 12 if q4k > total // 2 else 8 if q8 > total // 2 else 2 if q4 > total // 2 else None


def proj_dtypes(g, fallback):
    """The nine category formats {category: type id} (DENSE = 1 for F32 / F16 / BF16)."""
    out = {}
    for cat in _CATS:
        counts = {}
        for t in g["tensors"]:
            if _category(t["name"]) == cat and _storage(t["ggml_type"]) is not None:
                d = _storage(t["ggml_type"])
                counts[d] = counts.get(d, 0) + 1
        out[cat] = max(counts.items(), key=lambda kv: (kv[1], _RANK[kv[0]]))[0] if counts else fallback
    if not any(_category(t["name"]) == "lm_head" for t in g["tensors"]):
        out["lm_head"] = out["embed"]
    return out


def config_mixed(g, max_seq=0, flags=0):
    """(config, [q, k, v, o, gate, up, down], embed) as forge_hip_gguf_config_mixed reports them."""
    maj = _majority(g)
    if maj is None:
        raise GgufError("projection weights are neither mostly Q8_0, Q4_0 nor Q4_K")
    # the shape part of load_config does not depend on the formats: take it from config() of a file voted Q8_0
    shape_only = dict(g, tensors=[dict(t, ggml_type=8) for t in g["tensors"]])
    cfg = config(shape_only, max_seq, flags)
    cats = proj_dtypes(g, maj)
    dense_as = 8 if maj == 12 else maj
    fixed = {c: (dense_as if d == DENSE and c != "embed" else d) for c, d in cats.items()}
    cfg["wdtype"] = maj if maj in (8, 2) else 8
    cfg["lm_head_dtype"] = fixed["lm_head"]
    return cfg, [fixed[c] for c in _CATS[1:8]], cats["embed"]


def _round_away(x):
    """f32::round: halves away from zero (exact: the fraction of an f32 is itself an f32)."""
    a = np.abs(x)
    fl = np.floor(a)
    return np.copysign(fl + ((a - fl) >= F(0.5)), x).astype(F)


def _seq_sum(v):
    acc = np.zeros(v.shape[0], F)
    for i in range(v.shape[1]):
        acc = (acc + v[:, i]).astype(F)
    return acc


def _make_qkx2(x, nmax=15.0, rmin=-1.0, rdelta=0.1, nstep=20):
    """make_qkx2_quants (weight_loader.rs:1666-1768) for S sub-blocks at once: x [S][32] -> scale [S], the_min [S], L [S][32]."""
    x = np.ascontiguousarray(x, F)
    nmax, rmin, rdelta = F(nmax), F(rmin), F(rdelta)
    mn0, mx = x.min(axis=1), x.max(axis=1)
    flat = mx == mn0
    mn = np.minimum(mn0, F(0.0)).astype(F)
    span = np.where(flat, F(1.0), mx - mn).astype(F)
    iscale = (nmax / span).astype(F)
    scale = (F(1.0) / iscale).astype(F)
    L = np.clip(_round_away(((x - mn[:, None]) * iscale[:, None]).astype(F)), 0, nmax).astype(F)
    diff = ((scale[:, None] * L).astype(F) + mn[:, None]).astype(F) - x
    best_mad = _seq_sum((diff * diff).astype(F))
    best_scale, best_min, best_L = scale.copy(), mn.copy(), L.copy()
    nf = F(32.0)
    with np.errstate(all="ignore"):
        for step in range(nstep + 1):
            num = F(F(rmin + F(rdelta * F(step))) + nmax)
            itry = (num / span).astype(F)
            la = np.clip(_round_away(((x - mn[:, None]) * itry[:, None]).astype(F)), 0, nmax).astype(F)
            sum_l, sum_l2 = _seq_sum(la), _seq_sum((la * la).astype(F))
            sum_x, sum_xl = _seq_sum(x), _seq_sum((la * x).astype(F))
            det = ((nf * sum_l2).astype(F) - (sum_l * sum_l).astype(F)).astype(F)
            ok = det > 0
            sdet = np.where(ok, det, F(1.0))
            ts = ((((nf * sum_xl).astype(F) - (sum_x * sum_l).astype(F)).astype(F)) / sdet).astype(F)
            tm = ((((sum_l2 * sum_x).astype(F) - (sum_l * sum_xl).astype(F)).astype(F)) / sdet).astype(F)
            pos = tm > 0
            alt = (sum_xl / np.where(sum_l2 > 0, sum_l2, F(1.0))).astype(F)
            ts = np.where(pos & (sum_l2 > 0), alt, ts).astype(F)
            tm = np.where(pos, F(0.0), tm).astype(F)
            ok &= ts > 0
            d = ((ts[:, None] * la).astype(F) + tm[:, None]).astype(F) - x
            mad = _seq_sum((d * d).astype(F))
            better = ok & (mad < best_mad) & ~flat
            best_L[better], best_mad[better], best_scale[better], best_min[better] = la[better], mad[better], ts[better], tm[better]
    best_scale[flat], best_min[flat], best_L[flat] = 0.0, mn0[flat], 0.0
    return best_scale, (-best_min).astype(F), best_L.astype(np.uint8)


def quantize_q4_k(oracle, data):
    """quantize_f32_to_q4_k, weight_loader.rs:1773-1882."""
    data = np.ascontiguousarray(data, F).reshape(-1)
    nsb = (data.size + 255) // 256
    x = np.zeros(nsb * 256, F)
    x[:data.size] = data
    sc, mn, q = _make_qkx2(x.reshape(nsb * 8, 32))
    sc, mn, q = sc.reshape(nsb, 8), mn.reshape(nsb, 8), q.reshape(nsb, 8, 32)
    max_scale, max_min = np.maximum(sc.max(axis=1), F(0.0)), np.maximum(mn.max(axis=1), F(0.0))
    with np.errstate(all="ignore"):
        inv_scale = np.where(max_scale > 0, F(63.0) / max_scale, F(0.0)).astype(F)
        inv_min = np.where(max_min > 0, F(63.0) / max_min, F(0.0)).astype(F)
    d = np.where(max_scale > 0, max_scale / F(63.0), F(0.0)).astype(F)
    dmin = np.where(max_min > 0, max_min / F(63.0), F(0.0)).astype(F)
    sq = np.clip(_round_away((sc * inv_scale[:, None]).astype(F)), 0, 63).astype(np.uint8)
    mq = np.clip(_round_away((mn * inv_min[:, None]).astype(F)), 0, 63).astype(np.uint8)
    d_bits, dmin_bits = oracle.f32_to_f16(d), oracle.f32_to_f16(dmin)
    d_st, dmin_st = oracle.f16_to_f32(d_bits).astype(F), oracle.f16_to_f32(dmin_bits).astype(F)
    s_eff = (d_st[:, None] * sq.astype(F)).astype(F)
    dm_eff = (dmin_st[:, None] * mq.astype(F)).astype(F)
    with np.errstate(all="ignore"):
        inv = (F(1.0) / np.where(s_eff == 0, F(1.0), s_eff)).astype(F)
    xs = x.reshape(nsb, 8, 32)
    codes = np.clip(_round_away(((xs + dm_eff[:, :, None]).astype(F) * inv[:, :, None]).astype(F)), 0, 15).astype(np.uint8)
    codes[s_eff == 0] = 0
    out = np.zeros((nsb, 144), np.uint8)
    out[:, 0:2] = np.ascontiguousarray(d_bits, "<u2").view(np.uint8).reshape(nsb, 2)
    out[:, 2:4] = np.ascontiguousarray(dmin_bits, "<u2").view(np.uint8).reshape(nsb, 2)
    out[:, 4:8] = (sq[:, :4] & 63) | (((sq[:, 4:] >> 4) & 3) << 6)
    out[:, 8:12] = (mq[:, :4] & 63) | (((mq[:, 4:] >> 4) & 3) << 6)
    out[:, 12:16] = (sq[:, 4:] & 0x0F) | ((mq[:, 4:] & 0x0F) << 4)
    out[:, 16:] = ((codes[:, 0::2] & 0x0F) | (codes[:, 1::2] << 4)).reshape(nsb, 128)
    return out.reshape(-1)


def quantize_q6_k(oracle, data):
    """quantize_f32_to_q6_k, weight_loader.rs:2025-2140 (sub-block scale: make_q6k_quants :1987-2010)."""
    data = np.ascontiguousarray(data, F).reshape(-1)
    nsb = (data.size + 255) // 256
    x = np.zeros(nsb * 256, F)
    x[:data.size] = data
    xs = x.reshape(nsb, 16, 16)
    first = np.abs(xs).argmax(axis=2)                                  # the first element of largest magnitude
    mx = np.take_along_axis(xs, first[:, :, None], axis=2)[:, :, 0]
    zero = np.abs(mx) < F(1e-30)
    with np.errstate(all="ignore"):
        isc = (F(-32.0) / np.where(zero, F(1.0), mx)).astype(F)
        sub = np.where(zero, F(0.0), (F(1.0) / isc).astype(F)).astype(F)
    top = np.abs(sub).argmax(axis=1)
    max_scale = sub[np.arange(nsb), top]
    dead = np.abs(max_scale) < F(1e-30)
    with np.errstate(all="ignore"):
        sup_i = (F(-128.0) / np.where(dead, F(1.0), max_scale)).astype(F)
        sup_d = (F(1.0) / sup_i).astype(F)
    d_bits = oracle.f32_to_f16(sup_d)
    sq = np.clip(_round_away((sup_i[:, None] * sub).astype(F)), -128, 127).astype(np.int8)
    d_st = oracle.f16_to_f32(d_bits).astype(F)
    s_eff = (d_st[:, None] * sq.astype(F)).astype(F)
    with np.errstate(all="ignore"):
        inv = (F(1.0) / np.where(s_eff == 0, F(1.0), s_eff)).astype(F)
    L = np.clip(_round_away((inv[:, :, None] * xs).astype(F)), -32, 31).astype(np.int32)
    L[s_eff == 0] = 0
    q = (L.reshape(nsb, 2, 4, 32) + 32).astype(np.uint8)               # [block][half][quarter of 32][l]
    out = np.zeros((nsb, 210), np.uint8)
    ql = out[:, :128].reshape(nsb, 2, 64)
    qh = out[:, 128:192].reshape(nsb, 2, 32)
    ql[:, :, :32] = (q[:, :, 0] & 0x0F) | ((q[:, :, 2] & 0x0F) << 4)
    ql[:, :, 32:] = (q[:, :, 1] & 0x0F) | ((q[:, :, 3] & 0x0F) << 4)
    qh[:] = (q[:, :, 0] >> 4) | ((q[:, :, 1] >> 4) << 2) | ((q[:, :, 2] >> 4) << 4) | ((q[:, :, 3] >> 4) << 6)
    out[:, 192:208] = sq.view(np.uint8)
    out[:, 208:210] = np.ascontiguousarray(d_bits, "<u2").view(np.uint8).reshape(nsb, 2)
    out[dead] = 0
    return out.reshape(-1)


def export_weights_mixed(oracle, g, data, cfg, pd) -> np.ndarray:
    """The weights.bin bytes with each projection in its category's format."""
    data = bytes(data)
    by_name = {t["name"]: t for t in g["tensors"]}

    def find(name, n):
        t = by_name.get(name)
        if t is None:
            raise GgufError(f"weight not found: {name}")
        if numel(t) != n:
            raise GgufError(f"tensor {name} has the wrong number of elements")
        return t

    def raw(t):
        return np.frombuffer(data, np.uint8, data_size(t), g["tensor_data_offset"] + t["offset"])

    def f32(name, n):
        return _tensor_f32(oracle, g, data, find(name, n)).astype("<f4").view(np.uint8)

    def put(name, n, dt):
        t = find(name, n)
        if t["ggml_type"] == dt:
            return raw(t)
        if dt in (8, 2):
            return oracle.quantize_weights(dt, _tensor_f32(oracle, g, data, t))
        v = dequant_ggml(oracle, t["ggml_type"], raw(t), n)                  # directly: no Q8_0 stage for a K-quant target
        return quantize_q4_k(oracle, v) if dt == 12 else quantize_q6_k(oracle, v)

    H, I = cfg["hidden"], cfg["inter"]
    QKS, KV, V = cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"], cfg["vocab"]
    emb = find("token_embd.weight", V * H)
    if emb["ggml_type"] in (12, 14):
        parts = [dequant_ggml(oracle, emb["ggml_type"], raw(emb), V * H).astype("<f4").view(np.uint8)]
    else:
        parts = [f32("token_embd.weight", V * H)]
    for l in range(cfg["layers"]):
        b = f"blk.{l}."
        parts += [f32(b + "attn_norm.weight", H), put(b + "attn_q.weight", QKS * H, pd[0]), put(b + "attn_k.weight", KV * H, pd[1]),
                  put(b + "attn_v.weight", KV * H, pd[2])]
        if cfg.get("flags", 0) & 2:                                          # main.rs:2737-2742
            parts += [f32(b + "attn_q.bias", QKS), f32(b + "attn_k.bias", KV), f32(b + "attn_v.bias", KV)]
        parts += [put(b + "attn_output.weight", H * QKS, pd[3]), f32(b + "ffn_norm.weight", H),
                  put(b + "ffn_gate.weight", I * H, pd[4]), put(b + "ffn_up.weight", I * H, pd[5]), put(b + "ffn_down.weight", H * I, pd[6])]
    parts.append(f32("output_norm.weight", H))
    lm_name = "output.weight" if "output.weight" in by_name else "lm_head.weight" if "lm_head.weight" in by_name else "token_embd.weight"
    parts.append(put(lm_name, V * H, cfg["lm_head_dtype"]))
    return np.concatenate([np.ascontiguousarray(p, np.uint8) for p in parts])
