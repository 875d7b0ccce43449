"""Seeded synthetic tensors and models in the reference's on-disk formats.

There are no checkpoints offline, so every workload is random-init from a seed:
splitmix64 (counter based, so any slice can be generated independently) -> uniform ->
Box-Muller normals in f32.  Models are written as the headerless `weights.bin` that
`forge export-weights` produces (crates/forgellm-cli/src/main.rs:2714-2757; read back by
crates/forgellm-codegen-cpu/src/project.rs:342-407):

    embed_tokens f32 [vocab][hidden]
    per layer: attn_norm f32 | q | k | v | o raw blocks | ffn_norm f32 | gate | up | down raw blocks
    final_norm f32 | lm_head raw blocks

With tied embeddings the lm_head bytes are the quantised embedding and the f32 table is its
dequantisation (main.rs:2631-2693).
"""
from concurrent.futures import ThreadPoolExecutor

import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)
_CHUNK = 1 << 22


def splitmix64(seed: int, start: int, n: int) -> np.ndarray:
    """n outputs of splitmix64 seeded with `seed`, beginning at draw index `start`."""
    with np.errstate(over="ignore"):
        idx = np.arange(start + 1, start + n + 1, dtype=np.uint64)
        z = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + idx * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def _normal_chunk(seed, start_pair, npairs, std):
    z = splitmix64(seed, 2 * start_pair, 2 * npairs)
    u1 = ((z[0::2] >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / 9007199254740992.0)   # (0, 1]
    u2 = (z[1::2] >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)           # [0, 1)
    r = np.sqrt(-2.0 * np.log(u1)) * std
    ang = (2.0 * np.pi) * u2
    out = np.empty(2 * npairs, np.float32)
    out[0::2] = r * np.cos(ang)
    out[1::2] = r * np.sin(ang)
    return out


def normal(seed: int, n: int, std: float = 1.0, threads: int = 8) -> np.ndarray:
    """n f32 normals N(0, std^2), reproducible from (seed, n) alone."""
    npairs = (n + 1) // 2
    starts = list(range(0, npairs, _CHUNK))
    if len(starts) <= 1 or threads <= 1:
        parts = [_normal_chunk(seed, s, min(_CHUNK, npairs - s), std) for s in starts]
    else:
        with ThreadPoolExecutor(max_workers=threads) as ex:
            parts = list(ex.map(lambda s: _normal_chunk(seed, s, min(_CHUNK, npairs - s), std), starts))
    out = parts[0] if len(parts) == 1 else np.concatenate(parts)
    return out[:n]


def uniform_ids(seed: int, n: int, vocab: int) -> np.ndarray:
    """n token ids uniform in [0, vocab)."""
    return (splitmix64(seed, 0, n) % np.uint64(vocab)).astype(np.uint32)


# ---- model shapes named in the benchmark configurations ----
def _cfg(hidden, inter, layers, heads, kv_heads, head_dim, vocab, max_seq, theta, wdtype):
    return dict(hidden=hidden, inter=inter, layers=layers, heads=heads, kv_heads=kv_heads, head_dim=head_dim,
                vocab=vocab, max_seq=max_seq, rms_eps=1e-5, rope_theta=theta, wdtype=wdtype, lm_head_dtype=wdtype,
                flags=0)


def smollm2_135m(wdtype=8, max_seq=4096):
    return _cfg(576, 1536, 30, 9, 3, 64, 49152, max_seq, 100000.0, wdtype)


def llama32_1b(wdtype=8, max_seq=4096):
    return _cfg(2048, 8192, 16, 32, 8, 64, 128256, max_seq, 500000.0, wdtype)


def llama32_3b(wdtype=8, max_seq=4096):
    return _cfg(3072, 8192, 28, 24, 8, 128, 128256, max_seq, 500000.0, wdtype)


def llama31_8b(wdtype=8, max_seq=4096):
    return _cfg(4096, 14336, 32, 32, 8, 128, 128256, max_seq, 500000.0, wdtype)


def phi3_mini(wdtype=8, max_seq=4096):
    """Phi-3-mini-4k shape: 32 heads of 96 with a KV head each, vocabulary 32 064."""
    return _cfg(3072, 8192, 32, 32, 32, 96, 32064, max_seq, 10000.0, wdtype)


def qwen25_14b(wdtype=8, max_seq=4096):
    """Qwen2.5-14B shape: 48 layers (more than one launch of the resident decode kernel carries), QKV bias, 40 heads over
    8 KV heads, head_dim 128, vocabulary 152 064."""
    c = _cfg(5120, 13824, 48, 40, 8, 128, 152064, max_seq, 1000000.0, wdtype)
    c["flags"] = 2
    c["rms_eps"] = 1e-6
    return c


def mistral_7b(wdtype=8, max_seq=8192):
    """Mistral-7B-v0.1 shape: the Llama layer with a sliding window of 4096 positions, vocabulary 32 000."""
    c = _cfg(4096, 14336, 32, 32, 8, 128, 32000, max_seq, 10000.0, wdtype)
    c["sliding_window"] = 4096
    return c


def qwen25_1p5b(wdtype=8, max_seq=4096):
    """Qwen2.5-1.5B shape: QKV bias, 12 heads over 2 KV heads, head_dim 128, vocabulary 151 936."""
    c = _cfg(1536, 8960, 28, 12, 2, 128, 151936, max_seq, 1000000.0, wdtype)
    c["flags"] = 2
    c["rms_eps"] = 1e-6
    return c


def tiny(wdtype=8, max_seq=640, hidden=256, inter=512, layers=2, heads=4, kv_heads=2, head_dim=64, vocab=1000):
    return _cfg(hidden, inter, layers, heads, kv_heads, head_dim, vocab, max_seq, 10000.0, wdtype)


def make_weights_blob(cfg: dict, seed: int, std: float = 0.02, norm_jitter: float = 0.1, threads: int = 8) -> np.ndarray:
    """Random-init model as weights.bin bytes (tied embeddings).  Projection weights are f32
    N(0, std^2) quantised with the reference's quantisers; norm weights are 1 + norm_jitter*N(0,1)."""
    from .ops import block_bytes, dequant, quantize_weights
    H, I = cfg["hidden"], cfg["inter"]
    QKS, KV = cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"]
    wt, lt = cfg["wdtype"], cfg["lm_head_dtype"]
    counter = [0]

    def sub_seed():
        counter[0] += 1
        return (seed * 1000003 + counter[0] * 7919) & 0xFFFFFFFFFFFFFFFF

    def qmat(n, k, dtype):
        return quantize_weights(dtype, normal(sub_seed(), n * k, std, threads))

    def norm_vec():
        return (1.0 + norm_jitter * normal(sub_seed(), H, 1.0, 1)).astype(np.float32)

    parts = []
    lm_raw = qmat(cfg["vocab"], H, lt)
    embed = dequant(lt, lm_raw, cfg["vocab"] * H)
    parts.append(embed.view(np.uint8))
    has_bias = bool(cfg.get("flags", 0) & 2)
    for _ in range(cfg["layers"]):
        parts.append(norm_vec().view(np.uint8))
        parts.append(qmat(QKS, H, wt))
        parts.append(qmat(KV, H, wt))
        parts.append(qmat(KV, H, wt))
        if has_bias:                                        # q_bias | k_bias | v_bias, f32 (project.rs:286-292)
            parts.append(normal(sub_seed(), QKS + 2 * KV, 0.5, 1).astype(np.float32).view(np.uint8))
        parts.append(qmat(H, QKS, wt))
        parts.append(norm_vec().view(np.uint8))
        parts.append(qmat(I, H, wt))
        parts.append(qmat(I, H, wt))
        parts.append(qmat(H, I, wt))
    parts.append(norm_vec().view(np.uint8))
    parts.append(lm_raw)
    blob = np.concatenate(parts)
    expect = (cfg["vocab"] * H * 4 + cfg["layers"] * (2 * H * 4 + (QKS * H + 2 * KV * H + H * QKS + 3 * I * H) // 32 * block_bytes(wt)
                                                       + ((QKS + 2 * KV) * 4 if has_bias else 0))
              + H * 4 + cfg["vocab"] * H // 32 * block_bytes(lt))
    assert blob.size == expect, (blob.size, expect)
    return blob


def kquant_blocks(rng, ggml_type: int, n_blocks: int, std: float = 0.02) -> np.ndarray:
    """n_blocks random Q4_K (144-byte) or Q6_K (210-byte) super-blocks whose 256 weights each have zero mean and a standard
    deviation near `std`: every payload byte uniform, the fp16 super-block scales chosen for that spread.  (Not a
    quantisation of anything: the tests need valid blocks of sane magnitude, not a particular matrix.)"""
    if ggml_type == 12:
        raw = rng.integers(0, 256, (n_blocks, 144), dtype=np.uint8)
        # w = d * sc * q - dmin * m with sc, m uniform in 0..63 and q in 0..15: zero mean for dmin = 7.5 d, spread 258 d
        d = (std / 258.0) * rng.uniform(0.7, 1.3, n_blocks)
        raw[:, 0:2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
        raw[:, 2:4] = (7.5 * d).astype(np.float16).view(np.uint8).reshape(-1, 2)
    elif ggml_type == 14:
        raw = rng.integers(0, 256, (n_blocks, 210), dtype=np.uint8)
        # w = d * scale * (q - 32), scale an int8 kept within +-15 here, q in 0..63: spread about 165 d
        raw[:, 192:208] = rng.integers(-15, 16, (n_blocks, 16)).astype(np.int8).view(np.uint8)
        d = (std / 165.0) * rng.uniform(0.7, 1.3, n_blocks)
        raw[:, 208:210] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
    else:
        raise ValueError("kquant_blocks: Q4_K (12) or Q6_K (14)")
    return raw.reshape(-1)


def matrix_bytes(n: int, k: int, dtype: int) -> int:
    """Bytes of an [n][k] matrix in a storage format (GGML type id 8, 2, 12 or 14)."""
    if dtype in (12, 14):
        return n * (k // 256) * (144 if dtype == 12 else 210)
    return n * (k // 32) * (34 if dtype == 8 else 18)


def make_weights_blob_mixed(cfg: dict, proj_dtypes, seed: int, std: float = 0.02, norm_jitter: float = 0.1, threads: int = 8) -> np.ndarray:
    """Random-init model as weights.bin bytes with a storage format per projection: proj_dtypes = (q, k, v, o, gate, up,
    down) as GGML type ids, the lm_head in cfg["lm_head_dtype"]; Q8_0 / Q4_0 matrices are quantised normal weights, Q4_K /
    Q6_K matrices random super-blocks (kquant_blocks).  The f32 embedding table is drawn on its own (untied)."""
    from .ops import quantize_weights
    H, I = cfg["hidden"], cfg["inter"]
    QKS, KV = cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"]
    rng = np.random.default_rng(seed)
    counter = [0]

    def sub_seed():
        counter[0] += 1
        return (seed * 1000003 + counter[0] * 7919) & 0xFFFFFFFFFFFFFFFF

    def mat(n, k, dtype):
        if dtype in (12, 14):
            assert k % 256 == 0, "a K-quant matrix needs K to be a multiple of 256"
            return kquant_blocks(rng, dtype, n * (k // 256), std)
        return quantize_weights(dtype, normal(sub_seed(), n * k, std, threads))

    def norm_vec():
        return (1.0 + norm_jitter * normal(sub_seed(), H, 1.0, 1)).astype(np.float32)

    pq, pk, pv, po, pg, pu, pdn = [int(x) for x in proj_dtypes]
    parts = [normal(sub_seed(), cfg["vocab"] * H, std, threads).view(np.uint8)]
    has_bias = bool(cfg.get("flags", 0) & 2)
    for _ in range(cfg["layers"]):
        parts += [norm_vec().view(np.uint8), mat(QKS, H, pq), mat(KV, H, pk), mat(KV, H, pv)]
        if has_bias:                                        # q_bias | k_bias | v_bias, f32 (project.rs:286-292)
            parts.append(normal(sub_seed(), QKS + 2 * KV, 0.5, 1).astype(np.float32).view(np.uint8))
        parts += [mat(H, QKS, po), norm_vec().view(np.uint8), mat(I, H, pg), mat(I, H, pu), mat(H, I, pdn)]
    parts += [norm_vec().view(np.uint8), mat(cfg["vocab"], H, cfg["lm_head_dtype"])]
    return np.concatenate(parts)


def gemv_bytes(n: int, k: int, wdtype: int) -> int:
    """Algorithmic bytes of one quantised GEMV: the GGUF blocks of the matrix (34 or 18 bytes
    per 32 weights) plus the f32 input and output vectors."""
    from .ops import block_bytes
    return n * (k // 32) * block_bytes(wdtype) + 4 * k + 4 * n


def decode_weight_bytes(cfg: dict) -> int:
    """Bytes of quantised weights (34- or 18-byte GGUF blocks) one decode step streams."""
    from .ops import block_bytes
    H, I = cfg["hidden"], cfg["inter"]
    QKS, KV = cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"]

    def mat(n, k, dtype):
        return n * (k // 32) * block_bytes(dtype)

    wt = cfg["wdtype"]
    per_layer = mat(QKS, H, wt) + 2 * mat(KV, H, wt) + mat(H, QKS, wt) + 2 * mat(I, H, wt) + mat(H, I, wt)
    return cfg["layers"] * per_layer + mat(cfg["vocab"], H, cfg["lm_head_dtype"])
