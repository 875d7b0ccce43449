"""GPU parity of the op-level entry points, through the C ABI, against the CPU oracle.

Bit-exact: activation codes, int32 block sums (both kernels), argmax, and — because the
kernels follow the CPU path's own f32 operation order — rms_norm, silu_mul, rope, the GEMV, and
with FLAG_EXACT the GEMM and both attention kernels.  The fast GEMM (fused multiply-add) and
the MFMA / split-sequence attention kernels are held to rel 1e-3 / abs 1e-3."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q8, Q4 = 8, 2
EXACT = 1
RTOL, ATOL = 1e-3, 1e-3


def close(got, want, rtol=RTOL, atol=ATOL):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    bad = np.abs(got - want) > atol + rtol * np.abs(want)
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside tolerance; max abs err {np.max(np.abs(got - want)):.3e}"


def same_bits(got, want):
    got, want = np.ascontiguousarray(got, np.float32), np.ascontiguousarray(want, np.float32)
    diff = got.view(np.uint32) != want.view(np.uint32)
    assert not diff.any(), f"{diff.sum()} of {diff.size} differ in bits; max abs err {np.max(np.abs(got - want)):.3e}"


def act_planes(oracle, x2d):
    """Oracle activation quantisation of each row, split into (codes int8 [M][K], scale bits [M][K/32])."""
    M, K = x2d.shape
    raw = np.stack([oracle.quantize_act(x2d[r]) for r in range(M)]).reshape(M, K // 32, 34)
    codes = raw[:, :, 2:].reshape(M, K).view(np.int8)
    bits = raw[:, :, 0].astype(np.uint16) | (raw[:, :, 1].astype(np.uint16) << 8)
    return codes, bits


def make_weight(fh, wd, N, K, seed):
    w = fh.synth.normal(seed, N * K, 0.02).reshape(N, K)
    return fh.ops.quantize_weights(wd, w)


@pytest.mark.parametrize("M,K", [(1, 32), (1, 576), (3, 2048), (130, 8192)])
def test_quantize_act_bit_exact(fh, oracle, torch_gpu, M, K):
    torch = torch_gpu
    x = fh.synth.normal(100 + K, M * K, 1.0).reshape(M, K)
    x[0, :32] = 0.0                                        # an all-zero block: scale 1.0, codes 0
    if K >= 64:
        x[0, 32:64] = np.float32(1e-30)                    # scale below the fp16 range -> flushed to zero bits
    q, sc = fh.ops.quantize_act(torch.from_numpy(x).cuda())
    codes, bits = act_planes(oracle, x)
    assert np.array_equal(q.cpu().numpy(), codes)
    assert np.array_equal(sc.cpu().numpy().view(np.uint16), bits)


def test_quantize_act_rounding_ties(fh, torch_gpu):
    """Elements exactly half way between two codes go AWAY from zero (f32::round, emit.rs:1433).  Block 0 has its largest
    magnitude at 127 (scale and reciprocal exactly 1), block 1 at 254 (scale 2, reciprocal 0.5); expected codes by hand."""
    torch = torch_gpu
    ties = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 127.0, 0.25, -0.75, 3.0]
    want = [1, -1, 2, -2, 3, -3, 127, -127, 127, 0, -1, 3]
    x = np.zeros((2, 64), np.float32)
    x[0, :12] = ties
    x[0, 32:44] = [2.0 * t for t in ties]
    x[1, 32:44] = ties                                      # and in another row, second block
    q, sc = fh.ops.quantize_act(torch.from_numpy(x).cuda())
    q, sc = q.cpu().numpy(), sc.cpu().numpy().view(np.uint16)
    assert q[0, :12].tolist() == want and q[0, 32:44].tolist() == want and q[1, 32:44].tolist() == want
    assert sc[0].tolist() == [0x3C00, 0x4000] and sc[1].tolist() == [0x3C00, 0x3C00]    # row 1, block 0: all zero -> scale 1.0
    assert not q[0, 12:32].any() and not q[1, :32].any()


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("N,K", [(8, 32), (13, 576), (260, 2048), (64, 8192), (70, 3072)])
@pytest.mark.parametrize("path", [0, 1, 2])
def test_block_isums_bit_exact(fh, oracle, torch_gpu, wd, N, K, path):
    torch = torch_gpu
    M = 1 if path == 0 else 37
    wraw = make_weight(fh, wd, N, K, seed=N + K)
    x = fh.synth.normal(7 + K, M * K, 1.0).reshape(M, K)
    w = fh.ops.QWeight(wd, wraw, K, N)
    got = fh.ops.block_isums(w, torch.from_numpy(x).cuda(), path).cpu().numpy()
    for r in range(M):
        want = oracle.block_isums(wd, oracle.quantize_act(x[r]), wraw, K, N)
        assert np.array_equal(got[r], want), f"row {r}"


@pytest.mark.parametrize("path", [0, 1, 2])
def test_block_isums_extreme_codes(fh, oracle, torch_gpu, path):
    """All +-127 activations against all +-127 weights: |isum| = 516128, the int32 extreme of a block."""
    torch = torch_gpu
    K, N = 64, 4
    x = np.full((2, K), 3.0, np.float32); x[1] = -3.0                       # every code +-127
    wf = np.full((N, K), 0.5, np.float32); wf[1::2] = -0.5
    for wd, want_abs in ((Q8, 516128), (Q4, None)):
        wraw = fh.ops.quantize_weights(wd, wf)
        w = fh.ops.QWeight(wd, wraw, K, N)
        got = fh.ops.block_isums(w, torch.from_numpy(x).cuda(), path).cpu().numpy()
        for r in range(2):
            want = oracle.block_isums(wd, oracle.quantize_act(x[r]), wraw, K, N)
            assert np.array_equal(got[r], want)
            if want_abs:
                assert np.all(np.abs(got[r]) == want_abs)


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("K,N", [(2048, 2048), (2048, 512), (8192, 2048), (576, 1536), (3072, 1029), (32, 5),
                                 (2048, 1283), (96, 7), (1536, 301), (5120, 98), (4096, 130), (16384, 42), (8192, 4099),
                                 (2048, 18001)])
def test_matmul_vec_bit_exact(fh, oracle, torch_gpu, wd, K, N):
    """Sequential per-block combine, unfused, tail rows in the 4-accumulator order: identical bits.
    (2048, 1283) is over 1 MB, so the reference chunks rows by 256 and the tail rule applies per chunk.  The shapes from
    (1536, 301) on walk the ways K is dealt to the waves of a row group: a half-empty last chunk, six chunks over two
    waves, four and sixteen over four, a row count at which the split is narrowed to keep the launch within the CUs, and
    one (18001 rows) at which it is off and a workgroup walks several row groups."""
    torch = torch_gpu
    wraw = make_weight(fh, wd, N, K, seed=3 * N + K)
    x = fh.synth.normal(11 + K, K, 1.0)
    w = fh.ops.QWeight(wd, wraw, K, N)
    y = fh.ops.matmul_vec_q(w, torch.from_numpy(x).cuda()).cpu().numpy()
    same_bits(y, oracle.matmul_vec(wd, 0, x, wraw, K, N))


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("K,N", [(2048, 2048), (2048, 512), (8192, 2048), (576, 1536), (3072, 1029), (32, 5), (96, 7), (160, 64),
                                 (2048, 1283)])
def test_matmul_vec_portable_dot_bit_exact(fh, oracle, torch_gpu, wd, K, N):
    """The reference's x86 arithmetic (variant B: f32 activations against weights dequantised on the fly, one sequential
    sum per row, emit.rs:1359-1377 / 2337-2359): identical bits, row counts that are not multiples of 64, K that is not a
    multiple of the kernel's 128-element tile, and activations with large and tiny blocks side by side."""
    torch = torch_gpu
    wraw = make_weight(fh, wd, N, K, seed=7 * N + K)
    x = fh.synth.normal(17 + K, K, 1.0)
    x[:32] *= 1e4
    if K >= 64:
        x[32:64] *= 1e-6
    w = fh.ops.QWeight(wd, wraw, K, N)
    y = fh.ops.matmul_vec_q_portable(w, torch.from_numpy(x).cuda()).cpu().numpy()
    want = oracle.matmul_vec(wd, 1, x, wraw, K, N)
    same_bits(y, want)
    # and it is a different arithmetic from the int8 block-dot path: close, not equal
    ya = fh.ops.matmul_vec_q(w, torch.from_numpy(x).cuda()).cpu().numpy()
    assert np.abs(ya - want).max() <= 2e-2 * max(1.0, float(np.abs(want).max()))
    if K >= 2048:
        assert not np.array_equal(ya, want)


def random_superblocks(ty, n, seed, positive=False):
    """Random K-quant super-blocks with sane fp16 scale fields (every other bit pattern is a valid block).  `positive`:
    d and dmin >= 0, as every quantiser writes them."""
    rng = np.random.default_rng(seed)
    b = rng.integers(0, 256, (n, {12: 144, 14: 210}[ty]), dtype=np.uint8)
    for off in {12: (0, 2), 14: (208,)}[ty]:
        # (positive: small enough that d times a 6-bit / int8 sub-block scale stays below 2, the fast matmul's envelope)
        d = np.abs(rng.normal(0, 0.003, n)) if positive else rng.normal(0, 0.05, n)
        b[:, off:off + 2] = d.astype(np.float16).view(np.uint8).reshape(n, 2)
    return b.reshape(-1)


@pytest.mark.parametrize("ty", [12, 14])
@pytest.mark.parametrize("K,N", [(256, 3), (2048, 512), (2048, 2048), (8192, 300), (3072, 1029), (4096, 64)])
def test_matmul_vec_kquant_bit_exact(fh, oracle, torch_gpu, ty, K, N):
    """matmul_vec_q4_k / matmul_vec_q6_k (emit.rs:3388-3490, 3622-3655): exact sub-block integers and the reference's one
    f32 order per row, so the bits are the oracle's (whose dots are held to a float64 evaluation of the dequantised
    operands in tests/test_oracle_math.py)."""
    torch = torch_gpu
    wraw = random_superblocks(ty, N * K // 256, seed=ty * 1000 + K + N)
    x = fh.synth.normal(23 + K, K, 1.0)
    x[:32] = 0.0                                             # an all-zero activation block
    w = fh.ops.QWeight(ty, wraw, K, N)
    y = fh.ops.matmul_vec_q(w, torch.from_numpy(x).cuda()).cpu().numpy()
    same_bits(y, oracle.matmul_vec_kquant(ty, x, wraw, K, N))
    # M rows at once: the reference has no batched matmul for these formats, so every row is matmul_vec's, bit for bit,
    # whatever its place in the batch (1 row, a ragged 11, more than one workgroup's 8)
    rows = np.stack([x, -x, 0.5 * x] + [fh.synth.normal(31 + i, K, 1.0) for i in range(8)])
    want = np.stack([oracle.matmul_vec_kquant(ty, r, wraw, K, N) for r in rows])
    for M in (1, 11):
        same_bits(fh.ops.matmul_mat_q(w, torch.from_numpy(rows[:M]).cuda(), EXACT).cpu().numpy(), want[:M])
    w.close()
    with pytest.raises(fh.ForgeHipError):
        fh.ops.QWeight(ty, random_superblocks(ty, 1, 1), 288, 1)                # K must be a multiple of 256


@pytest.mark.parametrize("ty", [12, 14])
@pytest.mark.parametrize("M,K,N", [(1, 256, 32), (11, 2048, 512), (352, 2048, 2048), (130, 8192, 320), (700, 3072, 1029), (2502, 2048, 1024)])
def test_matmul_mat_kquant_on_the_matrix_unit(fh, oracle, torch_gpu, ty, M, K, N):
    """Fast mode for K-quant matrices: the matrix re-expressed once for the int8 MFMA GEMM (Q4_K: the nibbles as a Q4_0
    matrix under fp16(d * sc) plus the minimum term as a matmul over the activations' block sums; Q6_K: every 16-element half
    a block of a Q8_0 matrix of depth 2K under fp16(|d * sc|)).  Block sums stay exact; what differs from matmul_vec is the
    fp16 rounding of the block scales (2^-11 relative at most) and the order of the f32 additions.  Tolerance: 1e-3 of
    |value| + the row's root mean square (a sum of K signed products has no smaller natural unit).  With the order-faithful
    flag the same call gives matmul_vec's bits."""
    torch = torch_gpu
    wraw = random_superblocks(ty, N * K // 256, seed=ty * 77 + K + N + M, positive=True)
    x = fh.synth.normal(5 + K + M, M * K, 1.0).reshape(M, K)
    x[0, :32] = 0.0
    w = fh.ops.QWeight(ty, wraw, K, N)
    xd = torch.from_numpy(x).cuda()
    exact = fh.ops.matmul_mat_q(w, xd, EXACT).cpu().numpy()
    for m in {0, M // 2, M - 1}:
        same_bits(exact[m], oracle.matmul_vec_kquant(ty, x[m], wraw, K, N))
    fast = fh.ops.matmul_mat_q(w, xd, 0).cpu().numpy()
    again = fh.ops.matmul_mat_q(w, xd, 0).cpu().numpy()
    assert np.array_equal(fast, again)
    rms = np.sqrt(np.mean(exact.astype(np.float64) ** 2, axis=1, keepdims=True))
    err = np.abs(fast.astype(np.float64) - exact)
    assert np.all(err <= 1e-3 * (np.abs(exact) + rms)), f"max err / (|v| + rms) = {np.max(err / (np.abs(exact) + rms)):.3e}"
    assert np.sqrt(np.mean(err ** 2)) < 2e-4 * float(np.mean(rms))
    if M * N * K >= 2048 * 2048:
        assert not np.array_equal(fast, exact)                 # it IS the other arithmetic
    w.close()


def test_matmul_mat_kquant_scales_outside_the_fast_arithmetic_keep_the_exact_rows(fh, oracle, torch_gpu):
    """A Q4_K matrix with a negative d (no quantiser writes one, the format allows it) has no twin: the fast call then
    runs the order-faithful rows."""
    torch = torch_gpu
    K, N, M = 512, 64, 9
    wraw = random_superblocks(12, N * K // 256, seed=3)          # d of either sign
    x = fh.synth.normal(8, M * K, 1.0).reshape(M, K)
    w = fh.ops.QWeight(12, wraw, K, N)
    xd = torch.from_numpy(x).cuda()
    same_bits(fh.ops.matmul_mat_q(w, xd, 0).cpu().numpy(), fh.ops.matmul_mat_q(w, xd, EXACT).cpu().numpy())
    w.close()


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("M,K,N", [(1, 2048, 512), (37, 576, 960), (352, 2048, 2048), (130, 8192, 320), (129, 3072, 256)])
def test_matmul_mat_parity(fh, oracle, torch_gpu, wd, M, K, N):
    torch = torch_gpu
    wraw = make_weight(fh, wd, N, K, seed=5 * N + K + M)
    x = fh.synth.normal(13 + K, M * K, 1.0).reshape(M, K)
    x[M // 2, 32:64] = 0.0            # an all-zero activation block (reference scale 1.0: the fast kernel must not let it swamp its sums)
    w = fh.ops.QWeight(wd, wraw, K, N)
    want = oracle.matmul_mat(wd, 0, x, wraw, M, K, N)
    xd = torch.from_numpy(x).cuda()
    same_bits(fh.ops.matmul_mat_q(w, xd, EXACT).cpu().numpy(), want)      # N % 4 == 0: all rows sequential order
    close(fh.ops.matmul_mat_q(w, xd, 0).cpu().numpy(), want)


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("M,K,N", [(2502, 2048, 2048), (2502, 8192, 2048), (2100, 1152, 3072), (2502, 576, 2176)])
def test_matmul_mat_k_ranges_of_leftover_tiles(fh, torch_gpu, wd, M, K, N):
    """Fast mode, more 128 x 128 tiles than CUs but not a whole number of rounds: the left-over tiles are cut into K ranges
    that meet in a workspace.  Held to the fast mode's tolerance against EXACT mode (which is bit-identical to the CPU path,
    see the parity test above and never cuts K), twice in a row (the second call finds the counters the first one left),
    and the result must not depend on the run (ranges are added in K order, whoever finishes last)."""
    torch = torch_gpu
    wraw = make_weight(fh, wd, N, K, seed=3 * N + K + M)
    x = fh.synth.normal(17 + K, M * K, 1.0).reshape(M, K)
    w = fh.ops.QWeight(wd, wraw, K, N)
    xd = torch.from_numpy(x).cuda()
    want = fh.ops.matmul_mat_q(w, xd, EXACT).cpu().numpy()
    first = fh.ops.matmul_mat_q(w, xd, 0).cpu().numpy()
    close(first, want)
    for _ in range(3):
        same_bits(fh.ops.matmul_mat_q(w, xd, 0).cpu().numpy(), first)
    w.close()


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("M,K,I", [(2502, 2048, 8192), (37, 576, 1536), (300, 256, 64), (700, 3072, 1024), (65, 8192, 128)])
def test_gate_up_matmul_with_silu_and_quantiser_in_the_epilogue(fh, oracle, torch_gpu, wd, M, K, I):
    """forge_hip_gemm_silu_q: gate / up matmuls (fast arithmetic), silu(gate) * up and the activation quantiser in one kernel.
    Checked against the order-faithful matmul (bit-identical to the CPU path, see above) followed by silu_mul and the
    quantiser's definition in float64: every scale is absmax / 127 of its block to the fast mode's tolerance, every code is
    the nearest one (half a step, plus the tolerance on the value that was rounded), odd blocks come negated; rows past M
    stay untouched; the result does not depend on the run."""
    torch = torch_gpu
    wraw = make_weight(fh, wd, 2 * I, K, seed=7 * I + K + M)
    x = fh.synth.normal(19 + K, M * K, 1.0).reshape(M, K)
    w = fh.ops.QWeight(wd, wraw, K, 2 * I)
    xd = torch.from_numpy(x).cuda()
    y = fh.ops.matmul_mat_q(w, xd, EXACT).cpu().numpy().astype(np.float64)
    gate, up = y[:, :I], y[:, I:]
    o = gate / (1.0 + np.exp(-gate)) * up
    q, sc = fh.ops.gate_up_silu_q(w, xd)
    q2, sc2 = fh.ops.gate_up_silu_q(w, xd)
    assert torch.equal(q, q2) and torch.equal(sc, sc2)
    codes = q.cpu().numpy().astype(np.float64).reshape(M, I // 32, 32)
    scales = oracle.f16_to_f32(sc.cpu().numpy().view(np.uint16)).astype(np.float64).reshape(M, I // 32)
    ob = o.reshape(M, I // 32, 32)
    amax = np.abs(ob).max(axis=2)
    tol = 2e-3 * amax + 1e-6
    assert np.all(np.abs(scales - amax / 127.0) <= tol / 127.0 + amax / 127.0 * 2.0 ** -10)      # fp16 rounding of the scale
    sign = np.where(np.arange(I // 32) % 2 == 1, -1.0, 1.0)[None, :, None]
    recon = codes * sign * scales[:, :, None]
    assert np.all(np.abs(recon - ob) <= 0.5 * scales[:, :, None] * (1 + 2.0 ** -9) + tol[:, :, None])
    assert np.abs(codes).max() == 127                          # every block reaches its own maximum
    w.close()


def test_matmul_mat_ragged_n_within_tolerance(fh, oracle, torch_gpu):
    """N % 4 != 0: the reference's last rows use the 4-accumulator order; the GEMM kernel keeps one
    order for all rows, so those rows agree to tolerance only."""
    torch = torch_gpu
    M, K, N = 129, 3072, 257
    wraw = make_weight(fh, Q8, N, K, seed=99)
    x = fh.synth.normal(98, M * K, 1.0).reshape(M, K)
    w = fh.ops.QWeight(Q8, wraw, K, N)
    want = oracle.matmul_mat(Q8, 0, x, wraw, M, K, N)
    got = fh.ops.matmul_mat_q(w, torch.from_numpy(x).cuda(), EXACT).cpu().numpy()
    same_bits(got[:, :256], want[:, :256])
    close(got, want)


@pytest.mark.parametrize("M,H", [(1, 576), (5, 2048), (300, 3072), (2, 40)])
def test_rms_norm_bit_exact(fh, oracle, torch_gpu, M, H):
    torch = torch_gpu
    x = fh.synth.normal(1, M * H, 1.5).reshape(M, H)
    g = (1.0 + 0.1 * fh.synth.normal(2, H, 1.0)).astype(np.float32)
    out = fh.ops.rms_norm(torch.from_numpy(x).cuda(), torch.from_numpy(g).cuda(), 1e-5).cpu().numpy()
    want = np.stack([oracle.rms_norm(x[r], g, 1e-5, 0) for r in range(M)])
    same_bits(out, want)
    k = fh.ops.rms_norm(torch.tensor([1., 2., 3., 4.], device="cuda"), torch.ones(4, device="cuda"), 1e-5).cpu().numpy()
    close(k, np.array([1, 2, 3, 4]) / np.sqrt(7.5 + 1e-5), rtol=1e-6, atol=1e-6)      # kernels.rs:396-413


def test_silu_mul_bit_exact(fh, oracle, torch_gpu):
    torch = torch_gpu
    g = np.concatenate([fh.synth.normal(3, 8192 - 8, 2.0), np.array([0, -0.0, 30, -30, 88, -88, 100, -104], np.float32)])
    u = fh.synth.normal(4, 8192, 1.0)
    out = fh.ops.silu_mul(torch.from_numpy(g).cuda(), torch.from_numpy(u).cuda()).cpu().numpy()
    same_bits(out, oracle.silu_mul(g, u))


@pytest.mark.parametrize("heads,kv_heads,hd,theta", [(32, 8, 64, 500000.0), (9, 3, 64, 100000.0), (24, 8, 128, 500000.0)])
def test_rope_kv_store_bit_exact(fh, oracle, torch_gpu, heads, kv_heads, hd, theta):
    torch = torch_gpu
    M, base = 7, 2241
    q = fh.synth.normal(5, M * heads * hd, 1.0).reshape(M, heads * hd)
    k = fh.synth.normal(6, M * kv_heads * hd, 1.0).reshape(M, kv_heads * hd)
    v = fh.synth.normal(7, M * kv_heads * hd, 1.0).reshape(M, kv_heads * hd)
    qd, kd, vd = (torch.from_numpy(a.copy()).cuda() for a in (q, k, v))
    kc = torch.zeros((base + M, kv_heads * hd), dtype=torch.int16, device="cuda")
    vc = torch.zeros_like(kc)
    fh.ops.rope_kv_store(qd, kd, vd, kc, vc, base, heads, kv_heads, hd, theta)
    for r in range(M):
        wq = oracle.rope(q[r], base + r, hd, heads, theta)
        wk = oracle.rope(k[r], base + r, hd, kv_heads, theta)
        same_bits(qd[r].cpu().numpy(), wq)          # same C-library table, unfused multiply/subtract
        same_bits(kd[r].cpu().numpy(), wk)
        assert np.array_equal(kc[base + r].cpu().numpy().view(np.uint16), oracle.f32_to_f16(wk))
        assert np.array_equal(vc[base + r].cpu().numpy().view(np.uint16), oracle.f32_to_f16(v[r]))
    assert int(kc[:base].abs().max()) == 0        # rows before base_pos untouched


def _kv_cache(fh, oracle, seq, kv_heads, hd, seed):
    k16 = oracle.f32_to_f16(fh.synth.normal(seed, seq * kv_heads * hd, 1.0)).reshape(seq, kv_heads * hd)
    v16 = oracle.f32_to_f16(fh.synth.normal(seed + 1, seq * kv_heads * hd, 1.0)).reshape(seq, kv_heads * hd)
    return k16, v16


def _dev16(torch, a):
    return torch.from_numpy(a.view(np.int16)).cuda()


@pytest.mark.parametrize("heads,kv_heads,hd", [(32, 8, 64), (9, 3, 64), (32, 32, 96), (24, 8, 128), (8, 1, 64)])
@pytest.mark.parametrize("seq", [1, 5, 64, 70, 900])
def test_attention_decode_parity(fh, oracle, torch_gpu, heads, kv_heads, hd, seq):
    torch = torch_gpu
    k16, v16 = _kv_cache(fh, oracle, seq, kv_heads, hd, seed=seq + hd)
    q = fh.synth.normal(9, heads * hd, 1.0)
    want = oracle.attention("flash", q, k16, v16, seq, heads, kv_heads, hd)
    qd, kd, vd = torch.from_numpy(q).cuda(), _dev16(torch, k16), _dev16(torch, v16)
    same_bits(fh.ops.attention_flash(qd, kd, vd, seq, heads, kv_heads, hd, EXACT).cpu().numpy(), want)
    close(fh.ops.attention_flash(qd, kd, vd, seq, heads, kv_heads, hd, 0).cpu().numpy(), want)


@pytest.mark.parametrize("heads,kv_heads,hd", [(32, 8, 64), (9, 3, 64), (32, 32, 96), (24, 8, 128)])
@pytest.mark.parametrize("seq,page_rows", [(1, 16), (70, 16), (900, 64), (2250, 16), (2250, 256), (8192, 128), (777, 1)])
def test_attention_decode_paged_cache(fh, oracle, torch_gpu, heads, kv_heads, hd, seq, page_rows):
    """The sequence's rows scattered over a pool of pages in a random order (with pages of other sequences, poisoned, in
    between): the paged call must give the flat call's bits, and stays within the tolerance of the oracle."""
    torch = torch_gpu
    k16, v16 = _kv_cache(fh, oracle, seq, kv_heads, hd, seed=seq + hd + page_rows)
    q = fh.synth.normal(19, heads * hd, 1.0)
    n_pages = (seq + page_rows - 1) // page_rows
    rng = np.random.default_rng(seq * 31 + page_rows)
    pool_pages = 2 * n_pages + 3
    table = rng.permutation(pool_pages)[:n_pages].astype(np.int32)
    kvw = kv_heads * hd
    k_pool = np.full((pool_pages, page_rows, kvw), 0x7E00, np.uint16)       # NaN bit patterns wherever the sequence is not
    v_pool = np.full((pool_pages, page_rows, kvw), 0x7E00, np.uint16)
    for i, pg in enumerate(table):
        rows = slice(i * page_rows, min(seq, (i + 1) * page_rows))
        n = rows.stop - rows.start
        k_pool[pg, :n] = k16[rows]
        v_pool[pg, :n] = v16[rows]
    qd = torch.from_numpy(q).cuda()
    flat = fh.ops.attention_flash(qd, _dev16(torch, k16), _dev16(torch, v16), seq, heads, kv_heads, hd, 0).cpu().numpy()
    paged = fh.ops.attention_flash_paged(qd, _dev16(torch, k_pool), _dev16(torch, v_pool), torch.from_numpy(table).cuda(), page_rows,
                                         seq, heads, kv_heads, hd).cpu().numpy()
    same_bits(paged, flat)
    if seq <= 900:
        close(paged, oracle.attention("flash", q, k16, v16, seq, heads, kv_heads, hd))


def test_attention_decode_paged_cache_refusals(fh, torch_gpu):
    torch = torch_gpu
    q = torch.zeros(8 * 64, device="cuda")
    pool = torch.zeros((4, 24, 2 * 64), dtype=torch.int16, device="cuda")
    table = torch.zeros(4, dtype=torch.int32, device="cuda")
    with pytest.raises(fh.ForgeHipError):
        fh.ops.attention_flash_paged(q, pool, pool, table, 24, 50, 8, 2, 64)          # pages of 24 rows: not a power of two
    with pytest.raises(fh.ForgeHipError):
        fh.ops.attention_flash_paged(q, pool, pool, table, 16, 50, 8, 2, 80)          # head_dim


@pytest.mark.parametrize("heads,kv_heads,hd", [(8, 2, 64), (6, 6, 96), (6, 2, 128)])
@pytest.mark.parametrize("M,base", [(1, 0), (33, 0), (200, 0), (131, 77), (64, 64)])
def test_attention_prefill_parity(fh, oracle, torch_gpu, heads, kv_heads, hd, M, base):
    torch = torch_gpu
    seq = base + M
    k16, v16 = _kv_cache(fh, oracle, seq, kv_heads, hd, seed=M + hd + base)
    q = fh.synth.normal(10, M * heads * hd, 1.0).reshape(M, heads * hd)
    want = oracle.attention("flash_batch", q, k16, v16, M, heads, kv_heads, hd, base_pos=base)
    qd, kd, vd = torch.from_numpy(q).cuda(), _dev16(torch, k16), _dev16(torch, v16)
    same_bits(fh.ops.attention_flash_batch(qd, kd, vd, base, heads, kv_heads, hd, EXACT).cpu().numpy(), want)
    # MFMA path: q is rounded to fp16 for the matrix unit, so give it fp16-representable queries
    q16 = oracle.f16_to_f32(oracle.f32_to_f16(q))
    want16 = oracle.attention("flash_batch", q16, k16, v16, M, heads, kv_heads, hd, base_pos=base)
    close(fh.ops.attention_flash_batch(torch.from_numpy(q16).cuda(), kd, vd, base, heads, kv_heads, hd, 0).cpu().numpy(), want16)
    # and with full-precision queries it still holds the tolerance, a little more loosely
    close(fh.ops.attention_flash_batch(qd, kd, vd, base, heads, kv_heads, hd, 0).cpu().numpy(), want, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("heads,kv_heads,hd", [(32, 8, 64), (9, 3, 64), (6, 6, 96), (24, 8, 128)])
@pytest.mark.parametrize("seq,window", [(1, 1), (5, 3), (70, 1), (70, 64), (70, 70), (70, 4096), (900, 17), (900, 256), (900, 899)])
def test_attention_sliding_decode_parity(fh, oracle, torch_gpu, heads, kv_heads, hd, seq, window):
    """attention_sliding (emit.rs:598-627): one query against the last `window` cached rows."""
    torch = torch_gpu
    k16, v16 = _kv_cache(fh, oracle, seq, kv_heads, hd, seed=seq + hd + window)
    q = fh.synth.normal(9, heads * hd, 1.0)
    want = oracle.attention("sliding", q, k16, v16, seq, heads, kv_heads, hd, window=window)
    qd, kd, vd = torch.from_numpy(q).cuda(), _dev16(torch, k16), _dev16(torch, v16)
    got = fh.ops.attention_sliding(qd, kd, vd, seq, window, heads, kv_heads, hd).cpu().numpy()
    close(got, want)
    same_bits(fh.ops.attention_sliding(qd, kd, vd, seq, window, heads, kv_heads, hd, EXACT).cpu().numpy(), want)
    if window >= seq:       # then it is the plain decode attention, bit for bit
        same_bits(got, fh.ops.attention_flash(qd, kd, vd, seq, heads, kv_heads, hd, 0).cpu().numpy())
    else:                   # rows before the window do not count: poison them
        kd2, vd2 = kd.clone(), vd.clone()
        kd2[:seq - window] = 0x7BFF          # fp16 65504
        vd2[:seq - window] = 0x7BFF
        same_bits(fh.ops.attention_sliding(qd, kd2, vd2, seq, window, heads, kv_heads, hd).cpu().numpy(), got)


@pytest.mark.parametrize("heads,kv_heads,hd", [(8, 2, 64), (6, 6, 96), (6, 2, 128)])
@pytest.mark.parametrize("M,base,window", [(1, 0, 1), (33, 0, 5), (200, 0, 1), (200, 0, 31), (200, 0, 64), (200, 0, 100), (131, 77, 33),
                                           (131, 77, 128), (131, 77, 207), (131, 77, 208), (300, 500, 129), (64, 64, 1000)])
def test_attention_sliding_prefill_parity(fh, oracle, torch_gpu, heads, kv_heads, hd, M, base, window):
    """attention_sliding_batch (emit.rs:907-1046): row r sees the keys [max(0, base + r - window + 1), base + r]."""
    torch = torch_gpu
    seq = base + M
    k16, v16 = _kv_cache(fh, oracle, seq, kv_heads, hd, seed=M + hd + base + window)
    q = oracle.f16_to_f32(oracle.f32_to_f16(fh.synth.normal(10, M * heads * hd, 1.0))).reshape(M, heads * hd)
    want = oracle.attention("sliding_batch", q, k16, v16, M, heads, kv_heads, hd, base_pos=base, window=window)
    qd, kd, vd = torch.from_numpy(q).cuda(), _dev16(torch, k16), _dev16(torch, v16)
    got = fh.ops.attention_sliding_batch(qd, kd, vd, base, window, heads, kv_heads, hd).cpu().numpy()
    close(got, want)
    same_bits(fh.ops.attention_sliding_batch(qd, kd, vd, base, window, heads, kv_heads, hd, EXACT).cpu().numpy(), want)
    if window >= seq:       # every key of the call is inside every window: the causal kernel, bit for bit
        same_bits(got, fh.ops.attention_flash_batch(qd, kd, vd, base, heads, kv_heads, hd, 0).cpu().numpy())
    else:                   # rows before the first query's window are never read, and no query may see a row before its own
        first = max(0, base - window + 1)
        kd2, vd2 = kd.clone(), vd.clone()
        kd2[:first] = 0x7BFF
        vd2[:first] = 0x7BFF
        same_bits(fh.ops.attention_sliding_batch(qd, kd2, vd2, base, window, heads, kv_heads, hd).cpu().numpy(), got)
        r = M - 1                                  # the last query: poison everything before ITS window
        lo = max(0, base + r - window + 1)
        kd3, vd3 = kd.clone(), vd.clone()
        kd3[:lo] = 0x7BFF
        vd3[:lo] = 0x7BFF
        close(fh.ops.attention_sliding_batch(qd, kd3, vd3, base, window, heads, kv_heads, hd).cpu().numpy()[r], want[r])


def test_attention_sliding_refusals(fh, torch_gpu):
    torch = torch_gpu
    q = torch.zeros((4, 256), device="cuda")
    kc = torch.zeros((8, 64), dtype=torch.int16, device="cuda")
    with pytest.raises(fh.ForgeHipError, match="window"):
        fh.ops.attention_sliding_batch(q, kc, kc, 0, 0, 4, 1, 64)
    with pytest.raises(fh.ForgeHipError, match="window"):
        fh.ops.attention_sliding(q[0].contiguous(), kc, kc, 4, 0, 4, 1, 64)
    with pytest.raises(fh.ForgeHipError, match="head_dim"):
        fh.ops.attention_sliding(q[0].contiguous(), kc, kc, 4, 2, 4, 1, 48)


def test_attention_reference_vectors_shape_scaled(fh, oracle, torch_gpu):
    """The reference's deterministic attention inputs (emit.rs:6687-6741), widened to head_dim 64."""
    torch = torch_gpu
    hd, nh, nkv = 64, 3, 1
    for seq in (5, 64, 70, 128, 200):
        q = (((np.arange(nh * hd) * 7 + 3) % 41).astype(np.float32) * np.float32(0.1) - np.float32(1.0)) * np.float32(0.5)
        k = (((np.arange(seq * hd) * 11 + 5) % 43).astype(np.float32) * np.float32(0.07) - np.float32(1.0)) * np.float32(0.3)
        v = (((np.arange(seq * hd) * 13 + 7) % 47).astype(np.float32) * np.float32(0.05) - np.float32(0.5)) * np.float32(0.4)
        k16, v16 = oracle.f32_to_f16(k).reshape(seq, hd), oracle.f32_to_f16(v).reshape(seq, hd)
        want = oracle.attention("std", q, k16, v16, seq, nh, nkv, hd)
        for flags in (0, EXACT):
            got = fh.ops.attention_flash(torch.from_numpy(q).cuda(), _dev16(torch, k16), _dev16(torch, v16), seq, nh, nkv,
                                         hd, flags).cpu().numpy()
            assert np.max(np.abs(got - want)) < 1e-4          # the reference's own tolerance for this test


def test_argmax_last_maximum_on_device(fh, oracle, torch_gpu):
    torch = torch_gpu
    x = fh.synth.normal(12, 128256, 1.0)
    assert fh.ops.argmax(torch.from_numpy(x).cuda()) == oracle.argmax(x)
    x[[5, 70000, 128255]] = 99.0
    assert fh.ops.argmax(torch.from_numpy(x).cuda()) == 128255 == oracle.argmax(x)
    x[128255] = 0.0
    assert fh.ops.argmax(torch.from_numpy(x).cuda()) == 70000
    assert fh.ops.argmax(torch.tensor([3.0], device="cuda")) == 0
    assert fh.ops.argmax(torch.full((1000,), -7.0, device="cuda")) == 999


def test_bad_shapes_are_rejected(fh, torch_gpu):
    torch = torch_gpu
    q = torch.zeros((4, 4 * 48), device="cuda")
    kc = torch.zeros((4, 48), dtype=torch.int16, device="cuda")
    with pytest.raises(fh.ForgeHipError):
        fh.ops.attention_flash_batch(q, kc, kc, 0, 4, 1, 48)
    with pytest.raises(fh.ForgeHipError):
        fh.ops.attention_flash(q[0].contiguous(), kc, kc, 0, 4, 1, 64)
    with pytest.raises(fh.ForgeHipError):
        fh.ops.attention_flash(torch.zeros(256, device="cuda"), torch.zeros((4, 64), dtype=torch.int16, device="cuda"),
                               torch.zeros((4, 64), dtype=torch.int16, device="cuda"), 4, 4, 1, 64, flags=6)
