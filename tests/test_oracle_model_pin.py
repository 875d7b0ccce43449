"""Pins the oracle's model-level functions (`forward`, `forward_prefill_batched`) and its row-grouping
rule with checks that share no code with the oracle.

The checker is a float64 numpy Llama layer stack written here from the reference's emitter text
(crates/forgellm-codegen-cpu/src/emit.rs:4029-4300 for the per-token step, :5118-5486 for the batched
prefill, :327-334 rms_norm, :380-386 silu_mul, :501-528 rope, :558-583 attention, :598-627 the window)
over tensors that this file cuts out of the blob itself by the offsets of the generated reader
(crates/forgellm-codegen-cpu/src/project.rs:342-407, bias vectors :286-292) and dequantises itself
(crates/forgellm-frontend/src/weight_loader.rs:860-926).  A wiring mistake in the oracle (a swapped
gate/up or k/v slice, RoPE on the wrong tensor or with the wrong pairing, a wrong GQA head map, a residual
taken from the wrong vector, the lm_head on another row than the last, a bias added after the rotation)
moves the logits by their own magnitude; rounding moves them by 1e-5.
"""
import numpy as np
import pytest

Q8, Q4 = 8, 2
A, B = 0, 1
KV_INT8, KV_F16 = 0, 1
FLAG_QKV_BIAS = 2


# ---------------------------------------------------------------- blob -> float64 tensors
def _dequant(raw, wd, n, k):
    """Q8_0: u16 LE f16 scale | 32 x i8.  Q4_0: f16 scale | 16 bytes, byte j = element j (low nibble) and
    element j + 16 (high nibble), both minus 8 (weight_loader.rs:860-926)."""
    bb = 34 if wd == Q8 else 18
    r = np.asarray(raw, np.uint8).reshape(-1, bb)
    scale = (r[:, 0].astype(np.uint16) | (r[:, 1].astype(np.uint16) << 8)).view(np.float16).astype(np.float64)
    if wd == Q8:
        codes = r[:, 2:].view(np.int8).astype(np.float64)
    else:
        codes = np.concatenate([(r[:, 2:] & 0x0F).astype(np.float64) - 8.0, (r[:, 2:] >> 4).astype(np.float64) - 8.0], axis=1)
    return (codes * scale[:, None]).reshape(n, k)


def _dequant_any(oracle, raw, dt, n, k):
    """Q8_0 / Q4_0 by the routine above; Q4_K (12) and Q6_K (14) super-blocks by the numpy restatement of
    weight_loader.rs:997-1201, which its own tests pin against the reference's fixtures."""
    if dt in (Q8, Q4):
        return _dequant(raw, dt, n, k)
    from oracle import gguf_oracle
    return gguf_oracle.dequant_ggml(oracle, dt, np.ascontiguousarray(raw), n * k).astype(np.float64).reshape(n, k)


def _nbytes(dt, n, k):
    return n * (k // 256) * (144 if dt == 12 else 210) if dt in (12, 14) else n * (k // 32) * (34 if dt == Q8 else 18)


def _cut(cfg, blob, pd=None, oracle=None):
    """Named tensors of a weights.bin, by the running byte offset of project.rs:342-407.  pd: the storage formats of
    (q, k, v, o, gate, up, down) when they differ (ProjectionDTypes, ir.rs:410-421)."""
    H, I, V = cfg["hidden"], cfg["inter"], cfg["vocab"]
    QK, KV = cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"]
    wd, lm = cfg["wdtype"], cfg["lm_head_dtype"]
    pq, pk, pv, po, pg, pu, pdn = pd if pd is not None else [wd] * 7
    boff = [0]

    def f32(n):
        v = blob[boff[0]:boff[0] + 4 * n].view(np.float32).astype(np.float64)
        boff[0] += 4 * n
        return v

    def mat(n, k, dt):
        nb = _nbytes(dt, n, k)
        w = _dequant_any(oracle, blob[boff[0]:boff[0] + nb], dt, n, k)
        boff[0] += nb
        return w

    t = {"embed": f32(V * H).reshape(V, H), "layers": []}
    for _ in range(cfg["layers"]):
        L = {"attn_norm": f32(H), "q": mat(QK, H, pq), "k": mat(KV, H, pk), "v": mat(KV, H, pv)}
        if cfg.get("flags", 0) & FLAG_QKV_BIAS:
            L["qb"], L["kb"], L["vb"] = f32(QK), f32(KV), f32(KV)
        L["o"] = mat(H, QK, po)
        L["ffn_norm"] = f32(H)
        L["gate"], L["up"], L["down"] = mat(I, H, pg), mat(I, H, pu), mat(H, I, pdn)
        t["layers"].append(L)
    t["final_norm"] = f32(H)
    t["lm_head"] = mat(V, H, lm)
    assert boff[0] == blob.size
    return t


# ---------------------------------------------------------------- the float64 model
def _rms(x, w, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def _rope(x, pos, heads, hd, theta):
    """Pairs (2i, 2i+1) of every head turn by pos * theta^(-2i/hd) (emit.rs:501-528)."""
    m = x.shape[0]
    ang = np.asarray(pos, np.float64)[:, None] * theta ** (-2.0 * np.arange(hd // 2) / hd)[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    v = x.reshape(m, heads, hd // 2, 2)
    out = np.empty_like(v)
    out[..., 0] = v[..., 0] * c - v[..., 1] * s
    out[..., 1] = v[..., 0] * s + v[..., 1] * c
    return out.reshape(m, heads * hd)


def _quant_act(x):
    """The variant-A activation quantiser (emit.rs:1410-1440) in float64 on f32-rounded inputs: per block of 32,
    scale = absmax / 127 (1 with codes 0 for a zero block), codes = round-half-away(x / scale) clamped to +-127;
    the scale that multiplies the block sum is the fp16 rounding of it."""
    xb = x.astype(np.float32).reshape(x.shape[0], -1, 32)
    amax = np.abs(xb).max(axis=2, keepdims=True)
    s = (amax / np.float32(127.0)).astype(np.float32)
    inv = np.where(amax > 0, np.float32(1.0) / np.where(amax > 0, s, np.float32(1.0)), np.float32(0.0)).astype(np.float32)
    y = (xb * inv).astype(np.float32).astype(np.float64)
    codes = np.clip(np.sign(y) * np.floor(np.abs(y) + 0.5), -127, 127)
    s16 = np.where(amax > 0, s, np.float32(1.0)).astype(np.float16).astype(np.float64)
    return (codes * s16).reshape(x.shape)


def _kv_round(x, mode):
    if mode == KV_F16:
        return x.astype(np.float32).astype(np.float16).astype(np.float64)
    # int8 with one scale per cached row over all KV heads (emit.rs:532-545)
    x32 = x.astype(np.float32)
    amax = np.abs(x32).max(axis=1, keepdims=True).astype(np.float64)
    scale = np.where(amax > 0, amax / 127.0, 1.0)
    y = x32.astype(np.float64) / scale
    return np.clip(np.sign(y) * np.floor(np.abs(y) + 0.5), -127, 127) * np.where(amax > 0, scale, 0.0)


def _forward64(cfg, blob, tokens, variant, kvmode, pd=None, oracle=None, win_from=0):
    """Logits of every prompt position [m][vocab] and the cached K/V per layer, all float64.  win_from: the first row the
    sliding window applies to (rows before it see every earlier position)."""
    t = _cut(cfg, blob, pd, oracle)
    H, hd, nh, nkv = cfg["hidden"], cfg["head_dim"], cfg["heads"], cfg["kv_heads"]
    eps, theta, win = cfg["rms_eps"], cfg["rope_theta"], cfg.get("sliding_window", 0)
    m = len(tokens)
    pos = np.arange(m)
    act = _quant_act if variant == A else (lambda v: v)
    # a K-quant projection quantises its input on every target (emit.rs:3388-3490), a Q8_0 / Q4_0 one under variant A only
    kq = (lambda dt: dt in (12, 14))
    pdl = list(pd) if pd is not None else [cfg["wdtype"]] * 7
    acts = [(_quant_act if kq(dt) else act) for dt in pdl] + [_quant_act if kq(cfg["lm_head_dtype"]) else act]
    x = t["embed"][np.asarray(tokens, np.int64)].copy()
    caches = []
    for L in t["layers"]:
        n = _rms(x, L["attn_norm"], eps)
        q, k, v = acts[0](n) @ L["q"].T, acts[1](n) @ L["k"].T, acts[2](n) @ L["v"].T
        if "qb" in L:
            q, k, v = q + L["qb"], k + L["kb"], v + L["vb"]
        q, k = _rope(q, pos, nh, hd, theta), _rope(k, pos, nkv, hd, theta)
        k, v = _kv_round(k, kvmode), _kv_round(v, kvmode)
        caches.append((k, v))
        out = np.empty((m, nh * hd))
        for h in range(nh):
            g = h // (nh // nkv)
            s = q[:, h * hd:(h + 1) * hd] @ k[:, g * hd:(g + 1) * hd].T / np.sqrt(hd)
            keep = pos[None, :] <= pos[:, None]
            if win:
                keep &= (pos[None, :] > pos[:, None] - win) | (pos[:, None] < win_from)
            s = np.where(keep, s, -np.inf)
            p = np.exp(s - s.max(axis=1, keepdims=True))
            out[:, h * hd:(h + 1) * hd] = (p / p.sum(axis=1, keepdims=True)) @ v[:, g * hd:(g + 1) * hd]
        x = x + acts[3](out) @ L["o"].T
        n = _rms(x, L["ffn_norm"], eps)
        gate, up = acts[4](n) @ L["gate"].T, acts[5](n) @ L["up"].T
        x = x + acts[6](gate / (1.0 + np.exp(-gate)) * up) @ L["down"].T
    return acts[7](_rms(x, t["final_norm"], eps)) @ t["lm_head"].T, caches


def _cfg(fh, wd, heads, kv_heads, hd, max_seq=640, layers=2, bias=False, window=0, vocab=301):
    c = fh.synth.tiny(wdtype=wd, max_seq=max_seq, hidden=heads * hd if heads * hd % 32 == 0 else 128, inter=256, layers=layers,
                      heads=heads, kv_heads=kv_heads, head_dim=hd, vocab=vocab)
    c["rope_theta"] = 10000.0
    if bias:
        c["flags"] = FLAG_QKV_BIAS
    if window:
        c["sliding_window"] = window
    return c


def _oracle_logits_per_position(oracle, cfg, blob, toks, variant, kvmode):
    m = oracle.Model(cfg, blob, variant, kvmode)
    rows = np.stack([m.forward(int(t)) for t in toks])
    return rows, m


SHAPES = [  # heads, kv_heads, head_dim
    (4, 2, 32),
    (9, 3, 32),     # SmolLM2's 9:3 grouping; hidden 288
]


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("heads,kv_heads,hd", SHAPES)
@pytest.mark.parametrize("ntok", [21, 70])
def test_variant_b_forward_and_prefill_match_float64_model(oracle, fh, wd, heads, kv_heads, hd, ntok):
    """Variant B (f32 activations x dequantised weights) with the fp16 cache is the float64 model up to f32 rounding:
    every position's logits from the token loop, the batched prefill's last-row logits, and the cached K and V."""
    cfg = _cfg(fh, wd, heads, kv_heads, hd)
    blob = fh.synth.make_weights_blob(cfg, seed=11 + ntok)
    toks = fh.synth.uniform_ids(3, ntok, cfg["vocab"])
    want, caches = _forward64(cfg, blob, toks, B, KV_F16)
    scale = float(np.abs(want).max())
    rows, m1 = _oracle_logits_per_position(oracle, cfg, blob, toks, B, KV_F16)
    assert np.abs(rows - want).max() < 1e-4 * scale
    m2 = oracle.Model(cfg, blob, B, KV_F16)
    batched = m2.prefill_batched(toks)
    assert np.abs(batched - want[-1]).max() < 1e-4 * scale
    for model in (m1, m2):
        for l, (k, v) in enumerate(caches):
            # fp16 rounding may land on the neighbouring value where f32 and f64 inputs straddle a tie
            assert np.abs(model.read_kv(l, 0) - k).max() <= 2.0 ** -10 * np.abs(k).max()
            assert np.abs(model.read_kv(l, 1) - v).max() <= 2.0 ** -10 * np.abs(v).max()
            assert np.mean(model.read_kv(l, 0) == k) > 0.8
    # the argmax rule on these logits: last maximum
    assert oracle.argmax(batched) == int(np.flatnonzero(want[-1] == want[-1].max())[-1])


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("heads,kv_heads,hd", SHAPES)
def test_variant_a_forward_and_prefill_match_float64_model(oracle, fh, wd, heads, kv_heads, hd):
    """Variant A (int8 activation blocks) against the float64 model with the same activation quantiser written in numpy,
    and within the quantisation noise of the unquantised model with the same greedy token."""
    cfg = _cfg(fh, wd, heads, kv_heads, hd)
    blob = fh.synth.make_weights_blob(cfg, seed=5)
    toks = fh.synth.uniform_ids(8, 70, cfg["vocab"])
    want_a, _ = _forward64(cfg, blob, toks, A, KV_F16)
    want_b, _ = _forward64(cfg, blob, toks, B, KV_F16)
    scale = float(np.abs(want_b).max())
    rows, _ = _oracle_logits_per_position(oracle, cfg, blob, toks, A, KV_F16)
    batched = oracle.Model(cfg, blob, A, KV_F16).prefill_batched(toks)
    # until the first activation code that rounds the other way (an f32 against an f64 input a hair from a tie) the two
    # agree to f32 rounding; from that position on the changed K/V row is in every later context and the difference is
    # the size of one quantisation step
    per_row = np.abs(rows - want_a).max(axis=1)
    assert (per_row < 1e-5 * scale).sum() >= 20 and per_row[0] < 1e-6 * scale
    assert per_row.max() < 1e-2 * scale
    assert np.abs(batched - want_a[-1]).max() < 1e-2 * scale
    assert np.abs(batched - want_b[-1]).max() < 0.05 * scale
    assert int(np.argmax(batched)) == int(np.argmax(want_b[-1]))


@pytest.mark.parametrize("variant", [A, B])
def test_int8_cache_forward_matches_float64_model(oracle, fh, variant):
    """The CPU reference's own cache (int8, one scale per row over all KV heads)."""
    cfg = _cfg(fh, Q8, 4, 2, 32)
    blob = fh.synth.make_weights_blob(cfg, seed=9)
    toks = fh.synth.uniform_ids(2, 40, cfg["vocab"])
    want, caches = _forward64(cfg, blob, toks, variant, KV_INT8)
    scale = float(np.abs(want).max())
    rows, m = _oracle_logits_per_position(oracle, cfg, blob, toks, variant, KV_INT8)
    tol = 1e-4 if variant == B else 2e-3
    # one int8 code of K or V that rounds the other way moves a logit by more than f32 rounding: hold the bulk tightly
    assert np.median(np.abs(rows - want)) < 2e-5 * scale
    assert np.abs(rows - want).max() < max(tol, 5e-3) * scale
    batched = oracle.Model(cfg, blob, variant, KV_INT8).prefill_batched(toks)
    assert np.abs(batched - want[-1]).max() < max(tol, 5e-3) * scale
    k0 = m.read_kv(0, 0)
    assert np.abs(k0 - caches[0][0]).max() <= np.abs(caches[0][0]).max() / 127.0 * 1.001


@pytest.mark.parametrize("wd", [Q8, Q4])
def test_qkv_bias_and_window_match_float64_model(oracle, fh, wd):
    """Qwen2's bias vectors (added before the rotation, emit.rs:4105-4120 / 5246-5260) and Mistral's window."""
    for kw in (dict(bias=True), dict(window=9), dict(bias=True, window=24)):
        cfg = _cfg(fh, wd, 4, 2, 32, **kw)
        blob = fh.synth.make_weights_blob(cfg, seed=21)
        toks = fh.synth.uniform_ids(4, 40, cfg["vocab"])
        want, _ = _forward64(cfg, blob, toks, B, KV_F16)
        scale = float(np.abs(want).max())
        rows, _ = _oracle_logits_per_position(oracle, cfg, blob, toks, B, KV_F16)
        assert np.abs(rows - want).max() < 1e-4 * scale, kw
        batched = oracle.Model(cfg, blob, B, KV_F16).prefill_batched(toks)
        assert np.abs(batched - want[-1]).max() < 1e-4 * scale, kw
        if "window" in kw:          # and the window matters at this length
            full, _ = _forward64(dict(cfg, sliding_window=0), blob, toks, B, KV_F16)
            assert np.abs(full[-1] - want[-1]).max() > 1e-3 * scale


def test_short_context_model_uses_plain_attention_and_matches(oracle, fh):
    """max_seq <= 512 selects `attention` instead of `attention_flash` (emit.rs:126-128); same function of the inputs."""
    cfg = _cfg(fh, Q8, 4, 2, 32, max_seq=256)
    blob = fh.synth.make_weights_blob(cfg, seed=2)
    toks = fh.synth.uniform_ids(6, 30, cfg["vocab"])
    want, _ = _forward64(cfg, blob, toks, B, KV_F16)
    rows, _ = _oracle_logits_per_position(oracle, cfg, blob, toks, B, KV_F16)
    assert np.abs(rows - want).max() < 1e-4 * float(np.abs(want).max())
    batched = oracle.Model(cfg, blob, B, KV_F16).prefill_batched(toks)
    assert np.abs(batched - want[-1]).max() < 1e-4 * float(np.abs(want).max())


def test_two_chunk_prefill_continues_the_cache(oracle, fh):
    """A second batched call starts at base_pos > 0 (emit.rs:5118-5140): same logits as one call over the whole prompt."""
    cfg = _cfg(fh, Q8, 4, 2, 32)
    blob = fh.synth.make_weights_blob(cfg, seed=4)
    toks = fh.synth.uniform_ids(9, 50, cfg["vocab"])
    want, _ = _forward64(cfg, blob, toks, B, KV_F16)
    m = oracle.Model(cfg, blob, B, KV_F16)
    m.prefill_batched(toks[:33])
    got = m.prefill_batched(toks[33:])
    assert np.abs(got - want[-1]).max() < 1e-4 * float(np.abs(want).max())


# ---------------------------------------------------------------- which rows take the 4-accumulator order
def _dot1_rows_by_hand(n, parallel, tail):
    """Rows that end up in the scalar `dot_q*_0_q8_0` call, walking the emitted loops literally:
    matmul_vec (emit.rs:1971-2046) and forward's lm_head (:4304-4330): [chunks of 256 when parallel] groups of 8,
    then groups of 4, then single rows; the batched prefill's lm_head (:5452-5470): chunks of 256, groups of 8, then
    single rows; matmul_mat (:2150-2268): groups of 8, one group of 4, single rows over the whole N."""
    rows = []
    chunks = [(b, min(256, n - b)) for b in range(0, n, 256)] if parallel else [(0, n)]
    for base, length in chunks:
        done = length // 8 * 8
        if tail == 4:
            done += (length - done) // 4 * 4
        rows += [base + i for i in range(done, length)]
    return rows


@pytest.mark.parametrize("wd", [Q8, Q4])
def test_row_grouping_rule_against_the_emitted_loops(oracle, wd):
    """`fo_row_order(wdtype, k, n, mode, out)` reports, per output row, whether the oracle adds its block products in
    the 4-accumulator order.  Cases: N with every remainder mod 8, below and above the one-megabyte switch to 256-row
    chunks (which the emitter computes with 34-byte blocks for Q4_0 as well, emit.rs:2837), and the three lm_head forms."""
    k = 64
    row34 = k // 32 * 34
    just_below = 1_000_000 // row34             # N * row34 < 1e6
    assert just_below * row34 < 1_000_000 <= (just_below + 1) * row34
    for n in list(range(1, 34)) + [255, 256, 257, 259, 263, 511, 517, just_below - 1, just_below, just_below + 1, just_below + 7]:
        par = n * row34 >= 1_000_000
        assert oracle.row_order(wd, k, n, "vec") == _dot1_rows_by_hand(n, par, 4), n
        assert oracle.row_order(wd, k, n, "mat") == _dot1_rows_by_hand(n, False, 4), n
        assert oracle.row_order(wd, k, n, "lm_forward") == _dot1_rows_by_hand(n, True, 4), n
        assert oracle.row_order(wd, k, n, "lm_prefill") == _dot1_rows_by_hand(n, True, 8), n
    # 256 is a multiple of 8, so chunking never moves the tail: only the last N % 4 (N % 8) rows are ever scalar
    assert _dot1_rows_by_hand(128256 + 5, True, 8) == [128256 + i for i in range(5)]
    assert _dot1_rows_by_hand(128256 + 5, True, 4) == [128256 + 4]


@pytest.mark.parametrize("wd", [Q8, Q4])
def test_tail_rows_really_use_the_other_order(oracle, wd):
    """matmul_vec output rows equal dot_a in the order the table says, bit for bit, for an N with tail rows; K = 7
    blocks so that the two orders differ in their roundings."""
    rng = np.random.default_rng(31)
    k, n = 7 * 32, 15
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    x = rng.standard_normal(k).astype(np.float32)
    wraw, araw = oracle.quantize_weights(wd, w), oracle.quantize_act(x)
    rb = k // 32 * (34 if wd == Q8 else 18)
    y = oracle.matmul_vec(wd, A, x, wraw, k, n)
    scalar_rows = set(oracle.row_order(wd, k, n, "vec"))
    assert scalar_rows == {12, 13, 14}
    differs = 0
    for r in range(n):
        seq = oracle.dot_a(wd, araw, wraw[r * rb:(r + 1) * rb], k, True)
        four = oracle.dot_a(wd, araw, wraw[r * rb:(r + 1) * rb], k, False)
        assert y[r] == np.float32(four if r in scalar_rows else seq)
        differs += seq != four
    assert differs > 0



# ---------------------------------------------------------------- a storage format per projection
Q4K, Q6K = 12, 14
MIXES = [  # (q, k, v, o, gate, up, down), lm_head
    ((Q4K, Q4K, Q6K, Q4K, Q4K, Q4K, Q6K), Q6K),     # what llama.cpp's Q4_K_M files hold
    ((Q8, Q4, Q4K, Q8, Q6K, Q4, Q4K), Q8),          # every format next to every other
    ((Q4, Q4, Q4, Q4, Q4, Q4, Q4), Q6K),            # uniform projections under a K-quant lm_head
]


def test_model_with_a_format_per_projection_and_qkv_bias_matches_float64_model(oracle, fh):
    """Qwen2's bias vectors (project.rs:286-292: after the v weights, whatever the formats) in a model with a format per
    projection: a bias read from the wrong offset, or left out, moves every logit."""
    pd, lm = MIXES[0]
    cfg = fh.synth.tiny(wdtype=Q8, max_seq=640, hidden=256, inter=512, layers=2, heads=4, kv_heads=2, head_dim=64, vocab=301)
    cfg["rope_theta"] = 10000.0
    cfg["lm_head_dtype"] = lm
    cfg["flags"] = FLAG_QKV_BIAS
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=17, std=0.05)
    assert blob.size == oracle.weights_nbytes_mixed(cfg, pd)
    toks = np.random.default_rng(6).integers(0, cfg["vocab"], 17).astype(np.uint32)
    want, _ = _forward64(cfg, blob, toks, A, KV_F16, pd, oracle)
    without, _ = _forward64(dict(cfg, flags=0), np.concatenate([blob[:0], _strip_bias(cfg, blob, pd)]), toks, A, KV_F16, pd, oracle)
    m = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    rows = np.stack([m.forward(int(t)) for t in toks])
    scale = np.abs(want).max()
    per_row = np.abs(rows - want).max(axis=1)
    assert per_row[0] < 1e-5 * scale and (per_row < 1e-4 * scale).sum() >= 3 and per_row.max() < 3e-2 * scale
    assert np.abs(without - want).max() > 0.2 * scale          # the bias matters at this size: leaving it out is not within the bound
    m2 = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    assert np.array_equal(m2.prefill_batched(toks), rows[-1])


def test_model_with_a_format_per_projection_and_a_window_walks_its_prompt_with_full_attention(oracle, fh):
    """forward_prefill's token-by-token walk calls `attention` (or attention_flash), never attention_sliding (emit.rs:4717-4720;
    use_flash_attention is false for a model with a window, emit.rs:126-128): the rows of a prompt see every earlier
    position, decode steps only the window (emit.rs:4156-4170).  The float64 model with exactly that mask rule; the rule
    that every row is windowed, and the rule that none is, both miss by far more than the bound."""
    pd, lm = MIXES[0]
    cfg = fh.synth.tiny(wdtype=Q8, max_seq=640, hidden=256, inter=512, layers=2, heads=4, kv_heads=2, head_dim=64, vocab=301)
    cfg["rope_theta"] = 10000.0
    cfg["lm_head_dtype"] = lm
    cfg["sliding_window"] = 6
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=23, std=0.05)
    toks = np.random.default_rng(8).integers(0, cfg["vocab"], 26).astype(np.uint32)
    n_prompt = 17
    want, _ = _forward64(cfg, blob, toks, A, KV_F16, pd, oracle, win_from=n_prompt)
    all_windowed, _ = _forward64(cfg, blob, toks, A, KV_F16, pd, oracle)
    none_windowed, _ = _forward64(dict(cfg, sliding_window=0), blob, toks, A, KV_F16, pd, oracle)
    m = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    rows = [m.prefill_batched(toks[:n_prompt])] + [m.forward(int(t)) for t in toks[n_prompt:]]
    got = np.stack(rows)
    ref = want[n_prompt - 1:]
    scale = np.abs(want).max()
    assert np.abs(got - ref).max() < 3e-2 * scale and np.abs(got[0] - ref[0]).max() < 2e-3 * scale
    assert np.abs(all_windowed[n_prompt - 1] - ref[0]).max() > 0.1 * scale       # the prompt's last row does see more than 6 positions
    assert np.abs(none_windowed[-1] - ref[-1]).max() > 0.1 * scale               # and the decode rows do not


def _strip_bias(cfg, blob, pd):
    """The same blob without its bias vectors."""
    H, I, V = cfg["hidden"], cfg["inter"], cfg["vocab"]
    QK, KV = cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"]
    parts, at = [blob[:V * H * 4]], V * H * 4
    for _ in range(cfg["layers"]):
        n = H * 4 + _nbytes(pd[0], QK, H) + 2 * _nbytes(pd[1], KV, H) if pd[1] == pd[2] else H * 4 + _nbytes(pd[0], QK, H) + _nbytes(pd[1], KV, H) + _nbytes(pd[2], KV, H)
        parts.append(blob[at:at + n])
        at += n + (QK + 2 * KV) * 4
        n = _nbytes(pd[3], H, QK) + H * 4 + _nbytes(pd[4], I, H) + _nbytes(pd[5], I, H) + _nbytes(pd[6], H, I)
        parts.append(blob[at:at + n])
        at += n
    parts.append(blob[at:])
    return np.concatenate(parts)


@pytest.mark.parametrize("variant", [A, B])
@pytest.mark.parametrize("pd,lm", MIXES)
def test_model_with_a_format_per_projection_matches_float64_model(oracle, fh, pd, lm, variant):
    """Each projection must reach the kernel of ITS format with ITS slice of the blob (matmul_call, emit.rs:3316-3334;
    reader offsets project.rs:342-407 with per-projection byte counts :195-213): a projection read with another's format
    or byte count turns the logits into noise.  The prompt goes through forward_prefill's per-token walk (emit.rs:4621-5040),
    which has to give forward's own numbers bit for bit."""
    cfg = fh.synth.tiny(wdtype=Q8, max_seq=640, hidden=256, inter=512, layers=2, heads=4, kv_heads=2, head_dim=64, vocab=301)
    cfg["rope_theta"] = 10000.0
    cfg["lm_head_dtype"] = lm
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=11 + variant, std=0.05)
    assert blob.size == oracle.weights_nbytes_mixed(cfg, pd)
    toks = np.random.default_rng(5).integers(0, cfg["vocab"], 19).astype(np.uint32)
    want, _ = _forward64(cfg, blob, toks, variant, KV_F16, pd, oracle)
    m = oracle.Model(cfg, blob, variant, KV_F16, proj_dtypes=pd)
    rows = np.stack([m.forward(int(t)) for t in toks])
    scale = np.abs(want).max()
    assert scale > 0.05
    # an activation code a hair from a rounding tie may fall the other way in f32 than in f64: from that position on the
    # difference is one quantisation step; before it (and for most rows) the two agree to f32 rounding
    per_row = np.abs(rows - want).max(axis=1)
    assert per_row[0] < 1e-5 * scale and (per_row < 1e-4 * scale).sum() >= 3
    assert per_row.max() < 3e-2 * scale          # a wiring mistake moves the logits by their own magnitude
    m2 = oracle.Model(cfg, blob, variant, KV_F16, proj_dtypes=pd)
    last = m2.prefill_batched(toks)
    assert np.array_equal(last, rows[-1])
    assert np.array_equal(m2.forward(7), m.forward(7))
