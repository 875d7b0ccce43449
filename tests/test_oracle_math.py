"""Pins the oracle's arithmetic: integer block dots by brute force, f32 combines against fp64
evaluations of the same quantised operands, the f32 kernels against the reference's known
answers and closed forms, the three attention kernels against each other on the reference's
own deterministic test inputs and against brute-force fp64 softmax attention."""
import numpy as np
import pytest

Q8, Q4 = 8, 2
A, B = 0, 1


def _split_blocks(raw, wd):
    bb = 34 if wd == Q8 else 18
    r = raw.reshape(-1, bb)
    scale_bits = r[:, 0].astype(np.uint16) | (r[:, 1].astype(np.uint16) << 8)
    scales = scale_bits.view(np.float16).astype(np.float64)
    if wd == Q8:
        codes = r[:, 2:].view(np.int8).astype(np.int64)
    else:
        lo = (r[:, 2:] & 0x0F).astype(np.int64) - 8
        hi = (r[:, 2:] >> 4).astype(np.int64) - 8
        codes = np.concatenate([lo, hi], axis=1)
    return scales, codes            # [nblk], [nblk][32]


@pytest.mark.parametrize("wd", [Q8, Q4])
def test_block_isums_brute_force(oracle, wd):
    rng = np.random.default_rng(11)
    K, N = 256, 24
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    x = rng.standard_normal(K).astype(np.float32)
    wraw = oracle.quantize_weights(wd, w)
    araw = oracle.quantize_act(x)
    got = oracle.block_isums(wd, araw, wraw, K, N)
    _, acodes = _split_blocks(araw, Q8)
    _, wcodes = _split_blocks(wraw, wd)
    want = np.einsum("bj,nbj->nb", acodes, wcodes.reshape(N, K // 32, 32))
    assert np.array_equal(got.astype(np.int64), want)


def test_block_isums_extremes(oracle):
    a = np.concatenate([np.array([0, 0x3C], np.uint8), np.full(32, 127, np.int8).view(np.uint8)])
    for wcode, want in ((127, 516128), (-127, -516128)):
        w = np.concatenate([np.array([0, 0x3C], np.uint8), np.full(32, wcode, np.int8).view(np.uint8)])
        assert oracle.block_isums(Q8, a, w, 32, 1)[0, 0] == want
    for byte, want in ((0x00, -8 * 32 * 127), (0xFF, 7 * 32 * 127)):
        w = np.concatenate([np.array([0, 0x3C], np.uint8), np.full(16, byte, np.uint8)])
        assert oracle.block_isums(Q4, a, w, 32, 1)[0, 0] == want


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("K", [576, 2048])
def test_dot_a_against_fp64(oracle, wd, K):
    """Both accumulation orders of variant A equal sum_b a_s*w_s*isum evaluated in fp64 to f32 rounding noise."""
    rng = np.random.default_rng(K + wd)
    w = (rng.standard_normal(K) * 0.02).astype(np.float32)
    x = rng.standard_normal(K).astype(np.float32)
    wraw, araw = oracle.quantize_weights(wd, w), oracle.quantize_act(x)
    a_s, a_c = _split_blocks(araw, Q8)
    w_s, w_c = _split_blocks(wraw, wd)
    want = float(np.sum(a_s * w_s * np.sum(a_c * w_c, axis=1)))
    for seq in (True, False):
        got = oracle.dot_a(wd, araw, wraw, K, seq)
        assert abs(got - want) <= 2e-6 * max(1.0, abs(want)) + 1e-6
    # and the quantised dot is close to the unquantised one (sanity of the whole scheme)
    exact = float(np.dot(x.astype(np.float64), w.astype(np.float64)))
    assert abs(want - exact) < (0.05 if wd == Q8 else 0.25)


@pytest.mark.parametrize("wd", [Q8, Q4])
def test_dot_b_against_fp64(oracle, wd):
    rng = np.random.default_rng(3)
    K = 2048
    w = (rng.standard_normal(K) * 0.02).astype(np.float32)
    x = rng.standard_normal(K).astype(np.float32)
    wraw = oracle.quantize_weights(wd, w)
    deq = oracle.dequant(wd, wraw, K)
    want = float(np.dot(x.astype(np.float64), deq.astype(np.float64)))
    assert abs(oracle.dot_b(wd, x, wraw, K) - want) < 2e-5


def test_dot1_order_differs_from_sequential_only_by_rounding(oracle):
    """N % 4 tail rows take the 4-accumulator order (emit.rs:1558-1571): with K = 7 blocks the tail rule
    fa0,fa1,fa2 applies; a dropped tail block would show as a large difference."""
    rng = np.random.default_rng(9)
    K = 7 * 32
    w = (rng.standard_normal(K) * 0.02).astype(np.float32)
    x = rng.standard_normal(K).astype(np.float32)
    wraw, araw = oracle.quantize_weights(Q8, w), oracle.quantize_act(x)
    assert abs(oracle.dot_a(Q8, araw, wraw, K, True) - oracle.dot_a(Q8, araw, wraw, K, False)) < 1e-6


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("variant", [A, B])
def test_matmul_vec_and_mat_agree_with_row_dots(oracle, wd, variant):
    rng = np.random.default_rng(21)
    K, N, M = 128, 13, 5          # N % 8 = 5: one dot4 group and one dot1 row in the tail
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    x = rng.standard_normal((M, K)).astype(np.float32)
    wraw = oracle.quantize_weights(wd, w)
    rb = K // 32 * (34 if wd == Q8 else 18)
    ymat = oracle.matmul_mat(wd, variant, x, wraw, M, K, N)
    for r in range(M):
        yvec = oracle.matmul_vec(wd, variant, x[r], wraw, K, N)
        assert np.array_equal(yvec, ymat[r])          # the reference claims byte-identical (CHANGELOG.md:955)
        araw = oracle.quantize_act(x[r])
        for n in range(N):
            row = wraw[n * rb:(n + 1) * rb]
            want = oracle.dot_a(wd, araw, row, K, n < N - N % 4) if variant == A else oracle.dot_b(wd, x[r], row, K)
            assert yvec[n] == np.float32(want)
    # variants A and B differ only by the activation quantisation error
    ya = oracle.matmul_mat(wd, A, x, wraw, M, K, N)
    yb = oracle.matmul_mat(wd, B, x, wraw, M, K, N)
    assert np.max(np.abs(ya - yb)) < 0.02


# ---- f32 kernels: reference known answers (runtime kernels.rs:396-413, interpreter.rs:245-303)
@pytest.mark.parametrize("variant", [A, B])
def test_rms_norm_known_answer(oracle, variant):
    x = np.array([1, 2, 3, 4], np.float32)
    out = oracle.rms_norm(x, np.ones(4, np.float32), 1e-5, variant)
    want = x / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-5)
    assert np.allclose(out, want, rtol=0, atol=1e-6)
    rng = np.random.default_rng(4)
    x = rng.standard_normal(576).astype(np.float32)
    w = rng.standard_normal(576).astype(np.float32)
    want = x.astype(np.float64) / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-5) * w
    assert np.allclose(oracle.rms_norm(x, w, 1e-5, variant), want, rtol=2e-6, atol=1e-6)


def test_silu_and_softmax_known_answers(oracle):
    out = oracle.silu_mul(np.array([1.0, -1.0, 0.0], np.float32), np.array([1.0, 1.0, 5.0], np.float32))
    assert out[0] == pytest.approx(0.7311, abs=1e-4) and out[1] == pytest.approx(-0.2689, abs=1e-4) and out[2] == 0.0
    out = oracle.silu_mul(np.array([2.0], np.float32), np.array([3.0], np.float32))
    assert out[0] == pytest.approx(3.0 * 2.0 / (1.0 + np.exp(-2.0)), rel=1e-6)
    p = oracle.softmax(np.array([1.0, 2.0, 3.0], np.float32))
    assert p.sum() == pytest.approx(1.0, abs=1e-6) and p[0] < p[1] < p[2]
    assert np.allclose(p, np.exp([1.0, 2.0, 3.0]) / np.exp([1.0, 2.0, 3.0]).sum(), atol=1e-7)


def test_rope_properties_and_closed_form(oracle):
    rng = np.random.default_rng(6)
    hd, nh, theta = 64, 3, 500000.0
    x = rng.standard_normal(nh * hd).astype(np.float32)
    assert np.array_equal(oracle.rope(x, 0, hd, nh, theta), x)                 # identity at position 0
    y = oracle.rope(x, 1234, hd, nh, theta)
    assert np.linalg.norm(y) == pytest.approx(np.linalg.norm(x), rel=1e-5)     # rotations preserve the norm
    # closed form in fp64 with the f32 frequency/angle the reference uses: pairs (2i, 2i+1)
    i = np.arange(hd // 2)
    expo = (np.float32(2.0) * i.astype(np.float32) / np.float32(hd)).astype(np.float32)
    powf = np.power(np.float64(np.float32(theta)), expo.astype(np.float64)).astype(np.float32)   # correctly rounded powf
    freq = (np.float32(1.0) / powf).astype(np.float32)
    ang = (np.float32(1234) * freq).astype(np.float32).astype(np.float64)
    xr = x.reshape(nh, hd // 2, 2).astype(np.float64)
    want = np.stack([xr[..., 0] * np.cos(ang) - xr[..., 1] * np.sin(ang),
                     xr[..., 0] * np.sin(ang) + xr[..., 1] * np.cos(ang)], axis=-1).reshape(-1)
    assert np.allclose(y, want, rtol=0, atol=2e-5)
    c, s = oracle.rope_table(1300, hd, theta)
    assert np.allclose(c[1234], np.cos(ang), atol=1e-5) and np.allclose(s[1234], np.sin(ang), atol=1e-5)


# ---- attention: the reference's deterministic inputs (emit.rs:6687-6741)
def _ref_attention_inputs(seq, hd=8, nh=3, nkv=1):
    q = ((np.arange(nh * hd) * 7 + 3).astype(np.float32) * np.float32(0.1) - np.float32(1.0)) * np.float32(0.5)
    k = ((np.arange(seq * nkv * hd) * 11 + 5).astype(np.float32) * np.float32(0.07) - np.float32(1.0)) * np.float32(0.3)
    v = ((np.arange(seq * nkv * hd) * 13 + 7).astype(np.float32) * np.float32(0.05) - np.float32(0.5)) * np.float32(0.4)
    return q.astype(np.float32), k.astype(np.float32), v.astype(np.float32)


def _attention_fp64(q, k, v, nh, nkv, hd, qpos=None):
    """Brute-force softmax attention in fp64.  q [m][nh*hd] (or one row), k/v [seq][nkv*hd] f64."""
    q2 = np.atleast_2d(q).astype(np.float64)
    seq = k.shape[0]
    out = np.zeros_like(q2)
    g = nh // nkv
    for r in range(q2.shape[0]):
        lim = seq if qpos is None else qpos[r] + 1
        for h in range(nh):
            kh = k[:lim, (h // g) * hd:(h // g + 1) * hd]
            vh = v[:lim, (h // g) * hd:(h // g + 1) * hd]
            s = kh @ q2[r, h * hd:(h + 1) * hd] / np.sqrt(hd)
            p = np.exp(s - s.max())
            out[r, h * hd:(h + 1) * hd] = (p / p.sum()) @ vh
    return out


@pytest.mark.parametrize("seq", [5, 64, 70, 128, 200])
def test_flash_equals_standard_on_reference_vectors(oracle, seq):
    """The reference requires flash == standard within 1e-4 on these inputs (HEAD_DIM 8, 3 heads, 1 kv head)."""
    hd, nh, nkv = 8, 3, 1
    q, k, v = _ref_attention_inputs(seq)
    # the reference test runs on f32 caches; a 1.0-scale int8 cache cannot hold them, so use the fp16 cache mode
    # (values are O(10), well inside fp16 range) and compare everything on the fp16-rounded K/V.
    k16, v16 = oracle.f32_to_f16(k), oracle.f32_to_f16(v)
    kf = oracle.f16_to_f32(k16).astype(np.float64).reshape(seq, nkv * hd)
    vf = oracle.f16_to_f32(v16).astype(np.float64).reshape(seq, nkv * hd)
    std = oracle.attention("std", q, k16, v16, seq, nh, nkv, hd)
    flash = oracle.attention("flash", q, k16, v16, seq, nh, nkv, hd)
    assert np.max(np.abs(std - flash)) < 1e-4
    want = _attention_fp64(q, kf, vf, nh, nkv, hd)[0]
    assert np.max(np.abs(flash - want)) < 1e-4
    assert np.max(np.abs(std - want)) < 1e-4


@pytest.mark.parametrize("kvmode", ["int8", "f16"])
def test_flash_batch_rows_equal_per_token_flash(oracle, kvmode):
    """attention_flash_batch row r == attention_flash at seq_len = base_pos + r + 1 (CHANGELOG.md:955),
    and both equal brute-force causal attention in fp64."""
    rng = np.random.default_rng(8)
    hd, nh, nkv, base, m = 16, 4, 2, 37, 83          # crosses 64-key blocks and 16-row query tiles
    seq = base + m
    q = rng.standard_normal((m, nh * hd)).astype(np.float32)
    kf32 = rng.standard_normal((seq, nkv * hd)).astype(np.float32)
    vf32 = rng.standard_normal((seq, nkv * hd)).astype(np.float32)
    if kvmode == "int8":
        kq = np.empty((seq, nkv * hd), np.int8); vq = np.empty_like(kq)
        ks = np.empty(seq, np.float32); vs = np.empty(seq, np.float32)
        for t in range(seq):
            kq[t], ks[t] = oracle.quantize_kv(kf32[t])
            vq[t], vs[t] = oracle.quantize_kv(vf32[t])
        kw = dict(ks=ks, vs=vs)
        kc, vc = kq, vq
        kd = kq.astype(np.float64) * ks[:, None].astype(np.float64)
        vd = vq.astype(np.float64) * vs[:, None].astype(np.float64)
    else:
        kc, vc = oracle.f32_to_f16(kf32), oracle.f32_to_f16(vf32)
        kw = {}
        kd, vd = oracle.f16_to_f32(kc).astype(np.float64), oracle.f16_to_f32(vc).astype(np.float64)
    batch = oracle.attention("flash_batch", q, kc, vc, m, nh, nkv, hd, base_pos=base, **kw)
    want = _attention_fp64(q, kd, vd, nh, nkv, hd, qpos=[base + r for r in range(m)])
    assert np.max(np.abs(batch - want)) < 2e-5
    for r in (0, 1, 15, 16, 26, 27, 82):
        one = oracle.attention("flash", q[r], kc[:base + r + 1], vc[:base + r + 1], base + r + 1, nh, nkv, hd,
                               **{k_: v_[:base + r + 1] for k_, v_ in kw.items()})
        assert np.max(np.abs(one - batch[r])) < 2e-6


# ---- sliding-window attention (emit.rs:598-627, 907-1046): no reference test executes these two, so they are pinned
# by what the definition fixes: an fp64 softmax over the window, window >= seq == attention, batch == per token
def _windowed_fp64(q, k, v, nh, nkv, hd, qpos, window):
    q2 = np.atleast_2d(q).astype(np.float64)
    out = np.zeros_like(q2)
    g = nh // nkv
    for r in range(q2.shape[0]):
        lo, hi = max(0, qpos[r] - window + 1), qpos[r] + 1
        for h in range(nh):
            kh = k[lo:hi, (h // g) * hd:(h // g + 1) * hd]
            vh = v[lo:hi, (h // g) * hd:(h // g + 1) * hd]
            s = kh @ q2[r, h * hd:(h + 1) * hd] / np.sqrt(hd)
            p = np.exp(s - s.max())
            out[r, h * hd:(h + 1) * hd] = (p / p.sum()) @ vh
    return out


@pytest.mark.parametrize("seq", [5, 64, 70, 200])
def test_sliding_with_a_wide_window_is_standard_attention(oracle, seq):
    """`When seq_len <= window, behaves identically to attention` (emit.rs:597): same bits, on the reference's inputs."""
    hd, nh, nkv = 8, 3, 1
    q, k, v = _ref_attention_inputs(seq)
    k16, v16 = oracle.f32_to_f16(k), oracle.f32_to_f16(v)
    std = oracle.attention("std", q, k16, v16, seq, nh, nkv, hd)
    for window in (seq, seq + 1, 4096):
        assert np.array_equal(oracle.attention("sliding", q, k16, v16, seq, nh, nkv, hd, window=window).view(np.uint32), std.view(np.uint32))
    # a shorter window is attention over the tail of the cache
    w = max(1, seq // 3)
    tail = oracle.attention("std", q, k16.reshape(seq, -1)[seq - w:], v16.reshape(seq, -1)[seq - w:], w, nh, nkv, hd)
    assert np.array_equal(oracle.attention("sliding", q, k16, v16, seq, nh, nkv, hd, window=w).view(np.uint32), tail.view(np.uint32))


@pytest.mark.parametrize("kvmode", ["int8", "f16"])
@pytest.mark.parametrize("window", [1, 7, 64, 65, 100, 1000])
def test_sliding_batch_against_fp64_and_per_token(oracle, kvmode, window):
    rng = np.random.default_rng(80 + window)
    hd, nh, nkv, base, m = 16, 4, 2, 37, 150         # crosses 64-key blocks and 16-row query tiles
    seq = base + m
    q = rng.standard_normal((m, nh * hd)).astype(np.float32)
    kf32 = rng.standard_normal((seq, nkv * hd)).astype(np.float32)
    vf32 = rng.standard_normal((seq, nkv * hd)).astype(np.float32)
    if kvmode == "int8":
        kq = np.empty((seq, nkv * hd), np.int8); vq = np.empty_like(kq)
        ks = np.empty(seq, np.float32); vs = np.empty(seq, np.float32)
        for t in range(seq):
            kq[t], ks[t] = oracle.quantize_kv(kf32[t])
            vq[t], vs[t] = oracle.quantize_kv(vf32[t])
        kw = dict(ks=ks, vs=vs)
        kc, vc = kq, vq
        kd = kq.astype(np.float64) * ks[:, None].astype(np.float64)
        vd = vq.astype(np.float64) * vs[:, None].astype(np.float64)
    else:
        kc, vc = oracle.f32_to_f16(kf32), oracle.f32_to_f16(vf32)
        kw = {}
        kd, vd = oracle.f16_to_f32(kc).astype(np.float64), oracle.f16_to_f32(vc).astype(np.float64)
    qpos = [base + r for r in range(m)]
    batch = oracle.attention("sliding_batch", q, kc, vc, m, nh, nkv, hd, base_pos=base, window=window, **kw)
    want = _windowed_fp64(q, kd, vd, nh, nkv, hd, qpos, window)
    assert np.max(np.abs(batch - want)) < 2e-5
    # a key one step outside the window must not count: moving it far away changes nothing
    if window < seq:
        r = m - 1
        kc2 = kc.copy()
        kc2[qpos[r] - window] = kc[qpos[r]]          # the row just before the last query's window
        again = oracle.attention("sliding_batch", q, kc2, vc, m, nh, nkv, hd, base_pos=base, window=window, **kw)
        assert np.array_equal(again[r], batch[r])
    for r in (0, 1, 15, 16, 27, 90, 149):
        n = base + r + 1
        one = oracle.attention("sliding", q[r], kc[:n], vc[:n], n, nh, nkv, hd, window=window, **{k_: v_[:n] for k_, v_ in kw.items()})
        assert np.max(np.abs(one - batch[r])) < 2e-6
        assert np.max(np.abs(one - want[r])) < 2e-5
    if window >= seq:                                 # then it is the causal flash attention, block for block
        flash = oracle.attention("flash_batch", q, kc, vc, m, nh, nkv, hd, base_pos=base, **kw)
        assert np.array_equal(flash.view(np.uint32), batch.view(np.uint32))


def test_sliding_model_prefill_batched_equals_token_loop(oracle, fh):
    """A model with a window: token loop (attention_sliding) and batched prefill (attention_sliding_batch) agree, and the
    window matters (the same weights without it give other logits once the prompt is longer than the window)."""
    cfg = fh.synth.tiny(wdtype=Q8, max_seq=640, hidden=128, inter=256, layers=2, heads=4, kv_heads=2, head_dim=32, vocab=300)
    cfg["sliding_window"] = 9
    blob = fh.synth.make_weights_blob(cfg, seed=3)
    toks = fh.synth.uniform_ids(5, 40, cfg["vocab"])
    m1 = oracle.Model(cfg, blob, A, 1)
    for t in toks:
        last = m1.forward(int(t))
    batched = oracle.Model(cfg, blob, A, 1).prefill_batched(toks)
    assert np.max(np.abs(last - batched)) < 1e-4 * max(1.0, float(np.max(np.abs(last))))
    full = oracle.Model(dict(cfg, sliding_window=0), blob, A, 1).prefill_batched(toks)
    assert np.max(np.abs(full - batched)) > 1e-3
    # a prompt that fits the window sees every key either way (the summation order differs: flash blocks against plain softmax)
    short = oracle.Model(dict(cfg, sliding_window=0), blob, A, 1).prefill_batched(toks[:9])
    assert np.max(np.abs(short - oracle.Model(cfg, blob, A, 1).prefill_batched(toks[:9]))) < 1e-4


# ---- whole model: per-token forward loop == batched prefill (the reference's own consistency claim)
@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("variant,kv", [(A, 1), (A, 0), (B, 0)])
def test_model_prefill_batched_equals_token_loop(oracle, fh, wd, variant, kv):
    cfg = fh.synth.tiny(wdtype=wd, max_seq=640, hidden=128, inter=256, layers=2, heads=4, kv_heads=2, head_dim=32, vocab=300)
    blob = fh.synth.make_weights_blob(cfg, seed=3)
    assert blob.size == oracle.weights_nbytes(cfg)
    toks = fh.synth.uniform_ids(5, 21, cfg["vocab"])
    m1 = oracle.Model(cfg, blob, variant, kv)
    for t in toks:
        last = m1.forward(int(t))
    m2 = oracle.Model(cfg, blob, variant, kv)
    batched = m2.prefill_batched(toks)
    assert m1.pos == m2.pos == 21
    assert np.max(np.abs(last - batched)) < 1e-5
    assert np.all(np.isfinite(batched))
    # a different prompt gives different logits; reset reproduces (interpreter.rs:305-651 style smoke checks)
    m2.reset()
    again = m2.prefill_batched(toks)
    assert np.array_equal(again, batched)
    m2.reset()
    other = m2.prefill_batched(toks[::-1].copy())
    assert not np.allclose(other, batched)
    with pytest.raises(ValueError):
        oracle.Model(cfg, blob[:-1], variant, kv)


# ---------------- K-quant row dots (emit.rs:3035-3306 Q4_K, 3553-3612 Q6_K) ----------------
def _superblocks(ty, n, seed):
    rng = np.random.default_rng(seed)
    b = rng.integers(0, 256, (n, {12: 144, 14: 210}[ty]), dtype=np.uint8)
    for off in {12: (0, 2), 14: (208,)}[ty]:
        b[:, off:off + 2] = rng.normal(0, 0.05, n).astype(np.float16).view(np.uint8).reshape(n, 2)
    return b.reshape(-1)


@pytest.mark.parametrize("ty", [12, 14])
@pytest.mark.parametrize("K", [256, 1024, 4096])
def test_kquant_dots_against_fp64_of_the_dequantised_operands(oracle, ty, K):
    """The reference has no test that runs dot_q4_k_q8_0 / dot_q6_k_q8_0.  What pins the restatement: the dot of a
    K-quant row with Q8_0 activation blocks is, up to f32 rounding, the float64 dot of the two DEQUANTISED vectors, and
    both dequantisers are held to the reference's own block fixtures (tests/test_gguf.py).  A wrong nibble or bit-pair
    field, scale index, minimum term or block order moves the result by its own magnitude."""
    from oracle import gguf_oracle as go
    w = _superblocks(ty, K // 256, seed=ty + K)
    x = np.random.default_rng(K).normal(0, 1, K).astype(np.float32)
    aq = oracle.quantize_act(x)
    got = oracle.dot_kquant(ty, aq, w, K)
    wd = go.dequant_ggml(oracle, ty, w, K).astype(np.float64)
    xd = oracle.dequant(Q8, aq, K).astype(np.float64)
    assert abs(got - float(np.dot(wd, xd))) <= 2e-6 * float(np.sum(np.abs(wd * xd)))


@pytest.mark.parametrize("ty", [12, 14])
def test_kquant_dot_special_cases(oracle, ty):
    """One super-block by hand.  Q4_K with every nibble c, sub-block scales sc and minima m:  x_s * (d sc c - dmin m) * sum(xq)
    per sub-block; Q6_K with every 6-bit value v and scales s:  d x_s s (v - 32) * sum(xq) per block.  Zero activations
    give exactly 0 whatever the weights."""
    K = 256
    x = np.tile(np.arange(1, 33, dtype=np.float32), 8)                 # every block the same codes, scale 32/127
    aq = oracle.quantize_act(x)
    codes = oracle.dequant(Q8, aq, K) / np.float32(oracle.f16_to_f32(np.frombuffer(aq[:2].tobytes(), np.uint16))[0])
    sumq = float(np.round(codes[:32]).sum())
    xs = float(oracle.f16_to_f32(np.frombuffer(aq[:2].tobytes(), np.uint16))[0])
    if ty == 12:
        blk = np.zeros(144, np.uint8)
        blk[0:2] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)   # d
        blk[2:4] = np.frombuffer(np.float16(0.25).tobytes(), np.uint8)  # dmin
        blk[4:8] = 3                                                    # scales of sub-blocks 0..3 (j < 4: low 6 bits)
        blk[8:12] = 2                                                   # minima of sub-blocks 0..3
        blk[12:16] = 3 | (2 << 4)                                       # sub-blocks 4..7: scale low nibble, minimum high nibble
        blk[16:144] = 0x55                                              # every nibble 5
        want = 8 * xs * (0.5 * 3 * 5 * sumq - 0.25 * 2 * sumq)
    else:
        blk = np.zeros(210, np.uint8)
        blk[0:128] = 0x99                                               # low nibbles 9
        blk[128:192] = 0xAA                                             # bit pairs 2: v = 9 | 2 << 4 = 41
        blk[192:208] = np.array([7], np.int8).view(np.uint8)[0]         # scales
        blk[208:210] = np.frombuffer(np.float16(0.125).tobytes(), np.uint8)
        want = 8 * 0.125 * xs * 7 * (41 - 32) * sumq
    got = oracle.dot_kquant(ty, aq, blk, K)
    assert abs(got - want) <= 1e-5 * abs(want)
    assert oracle.dot_kquant(ty, oracle.quantize_act(np.zeros(K, np.float32)), _superblocks(ty, 1, 3), K) == 0.0


@pytest.mark.parametrize("ty", [12, 14])
def test_matmul_vec_kquant_is_one_dot_per_row(oracle, ty):
    K, N = 512, 5
    w = _superblocks(ty, N * K // 256, seed=9)
    x = np.random.default_rng(4).normal(0, 1, K).astype(np.float32)
    rb = K // 256 * {12: 144, 14: 210}[ty]
    aq = oracle.quantize_act(x)
    want = np.array([oracle.dot_kquant(ty, aq, w[r * rb:(r + 1) * rb], K) for r in range(N)], np.float32)
    assert np.array_equal(oracle.matmul_vec_kquant(ty, x, w, K, N).view(np.uint32), want.view(np.uint32))
