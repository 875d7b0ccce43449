"""Pins the oracle's format code (fp16 conversions, Q8_0/Q4_0 (de)quantisers, activation and
KV quantisers, argmax) against the reference's own unit-test vectors, IEEE via numpy, and
closed forms — none of these checks re-types the oracle's formula."""
import numpy as np
import pytest

Q8, Q4 = 8, 2


# ---- f16 -> f32: exhaustive vs IEEE, plus the reference's known answers (weight_loader.rs:2469-2491)
def test_f16_to_f32_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_reference_known_answers(oracle):
    f = lambda b: float(oracle.f16_to_f32(np.array([b], np.uint16))[0])
    assert f(0x0000) == 0.0
    assert f(0x3C00) == 1.0 and f(0xBC00) == -1.0 and f(0x3800) == 0.5 and f(0x4000) == 2.0
    assert np.isinf(f(0x7C00)) and np.isnan(f(0x7E00))
    assert f(0x8000) == 0.0 and np.signbit(np.float32(f(0x8000)))


# ---- f32 -> f16: RNE like numpy everywhere except the documented flush of |x| < 2^-24
def test_f32_to_f16_matches_ieee_rne(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-7, 5, 200000).astype(np.float32),
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32),          # every f16 value round-trips
        np.array([65504.0, 65519.9, 65520.0, 1e10, -1e10, 6.1e-5, 6.0e-5, 2.0 ** -14, 2.0 ** -24, 3 * 2.0 ** -25], np.float32),
    ])
    x = x[~np.isnan(x)]
    keep = np.abs(x) >= np.float32(2.0 ** -24)   # below that the reference flushes (tested next)
    x = x[keep | (x == 0)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = oracle.f32_to_f16(x)
    assert np.array_equal(got, want)
    # ties: halfway between two f16 values goes to even
    assert oracle.f32_to_f16(np.array([1.0 + 2.0 ** -11], np.float32))[0] == 0x3C00
    assert oracle.f32_to_f16(np.array([1.0 + 3 * 2.0 ** -11], np.float32))[0] == 0x3C02


def test_f32_to_f16_flush_rule(oracle):
    """emit.rs:1471-1474: f32 subnormals and unbiased exponent < -24 give signed zero — even
    1.5 * 2^-25, which IEEE would round up to the smallest subnormal."""
    f = lambda v: int(oracle.f32_to_f16(np.array([v], np.float32))[0])
    assert f(2.0 ** -24) == 0x0001
    assert f(2.0 ** -25) == 0x0000
    assert f(1.5 * 2.0 ** -25) == 0x0000          # IEEE RNE would give 0x0001
    assert np.float32(1.5 * 2.0 ** -25).astype(np.float16).view(np.uint16) == 0x0001
    assert f(-1.5 * 2.0 ** -25) == 0x8000
    assert f(1e-45) == 0x0000 and f(-1e-45) == 0x8000
    assert f(1.5 * 2.0 ** -24) == 0x0002          # tie at 1.5 ulp -> even


# ---- dequantisers: the reference's fixtures (weight_loader.rs:3209-3242, 3696-3759)
def _q8_block(scale_bits, codes):
    return np.concatenate([np.array([scale_bits & 0xFF, scale_bits >> 8], np.uint8), np.asarray(codes, np.int8).view(np.uint8)])


def test_dequant_q8_0_reference_fixtures(oracle):
    out = oracle.dequant(Q8, _q8_block(0x3C00, np.arange(32)), 32)
    assert np.array_equal(out, np.arange(32, dtype=np.float32))
    codes = [i if i % 2 == 0 else -i for i in range(32)]
    out = oracle.dequant(Q8, _q8_block(0x4000, codes), 32)
    assert np.array_equal(out, 2.0 * np.array(codes, np.float32))
    assert out[1] == -2.0 and out[2] == 4.0 and out[31] == -62.0
    out = oracle.dequant(Q8, _q8_block(0x0000, [127] * 32), 32)
    assert np.all(out == 0.0)


def test_dequant_q4_0_reference_fixture_and_nibble_order(oracle):
    blk = np.concatenate([np.array([0x00, 0x3C], np.uint8), np.full(16, 0x88, np.uint8)])
    assert np.all(oracle.dequant(Q4, blk, 32) == 0.0)
    # byte j: low nibble -> element j, high nibble -> element j+16, both minus 8
    packed = np.array([(j % 16) | (((15 - j) % 16) << 4) for j in range(16)], np.uint8)
    out = oracle.dequant(Q4, np.concatenate([np.array([0x00, 0x40], np.uint8), packed]), 32)
    want = np.concatenate([np.arange(16) - 8, (15 - np.arange(16)) - 8]).astype(np.float32) * 2.0
    assert np.array_equal(out, want)


def test_dequant_two_blocks_boundary(oracle):
    raw = np.concatenate([_q8_block(0x3C00, np.arange(32)), _q8_block(0x4000, np.arange(32) - 16)])
    out = oracle.dequant(Q8, raw, 64)
    assert np.array_equal(out[:32], np.arange(32, dtype=np.float32))
    assert np.array_equal(out[32:], 2.0 * (np.arange(32, dtype=np.float32) - 16))


# ---- weight quantisers: reference invariants (weight_loader.rs:3002-3028, 3340-3379, 3761-3796)
def test_quantize_q8_0_round_trip_reference_ramp(oracle):
    v = ((np.arange(64, dtype=np.float32) - 32.0) * np.float32(0.05)).astype(np.float32)
    raw = oracle.quantize_weights(Q8, v)
    assert raw.size == 2 * 34
    back = oracle.dequant(Q8, raw, 64)
    assert np.max(np.abs(back - v)) < 0.02
    assert np.all(oracle.dequant(Q8, oracle.quantize_weights(Q8, np.zeros(32, np.float32)), 32) == 0.0)


def test_quantize_q4_0_reference_invariants(oracle):
    v = ((np.arange(64, dtype=np.float32) - 32.0) * np.float32(0.1)).astype(np.float32)
    raw = oracle.quantize_weights(Q4, v)
    assert raw.size == 2 * 18
    back = oracle.dequant(Q4, raw, 64)
    for blk in range(2):
        seg = slice(32 * blk, 32 * blk + 32)
        step = np.max(np.abs(v[seg])) / 8.0
        assert np.all(np.abs(back[seg] - v[seg]) <= step + 0.01)
    z = oracle.quantize_weights(Q4, np.zeros(32, np.float32))
    assert z[0] == 0 and z[1] == 0 and np.all(oracle.dequant(Q4, z, 32) == 0.0)
    s = np.array([-(i + 1.0) if i < 16 else i - 15.0 for i in range(32)], np.float32)
    back = oracle.dequant(Q4, oracle.quantize_weights(Q4, s), 32)
    assert np.all(back[:16] <= 0) and np.all(back[16:] >= 0)


@pytest.mark.parametrize("wd", [Q8, Q4])
def test_weight_quantiser_brute_force(oracle, wd):
    """Independent restatement in float64 arithmetic + explicit rounding: scale = amax/127 (Q8) or
    unsigned amax/8 (Q4), codes = round-half-away(v * (1/scale)) clamped; scale stored as RNE f16."""
    rng = np.random.default_rng(5)
    v = (rng.standard_normal(32 * 200) * 0.02).astype(np.float32)
    v[32:64] = 0.0
    v[64] = 0.5                                   # an outlier block
    raw = oracle.quantize_weights(wd, v)
    bb = 34 if wd == Q8 else 18
    for b in range(200):
        blk = v[32 * b:32 * b + 32]
        amax = np.float32(np.max(np.abs(blk)))
        scale = np.float32(amax / np.float32(127.0 if wd == Q8 else 8.0))
        rb = raw[bb * b:bb * b + bb]
        with np.errstate(over="ignore"):
            want_bits = np.float32(scale).astype(np.float16).view(np.uint16)
        assert (int(rb[0]) | (int(rb[1]) << 8)) == int(want_bits)
        inv = np.float32(1.0) / scale if scale != 0 else np.float32(0.0)
        t = (blk * inv).astype(np.float32)
        r = np.sign(t) * np.floor(np.abs(t.astype(np.float64)) + 0.5)      # half away from zero
        if wd == Q8:
            want = np.clip(r, -127, 127).astype(np.int8)
            assert np.array_equal(rb[2:].view(np.int8), want)
        else:
            want = np.clip(r + 8, 0, 15).astype(np.uint8)
            assert np.array_equal(rb[2:] & 0x0F, want[:16]) and np.array_equal(rb[2:] >> 4, want[16:])


# ---- activation quantiser (emit.rs:1410-1440): invariants that fix its behaviour
def test_activation_quantiser_invariants(oracle):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(32 * 64).astype(np.float32)
    x[64:96] = 0.0
    raw = oracle.quantize_act(x).reshape(-1, 34)
    codes = raw[:, 2:].view(np.int8)
    scales = oracle.f16_to_f32(raw[:, 0].astype(np.uint16) | (raw[:, 1].astype(np.uint16) << 8))
    assert np.all(np.abs(codes.astype(np.int32)) <= 127)
    xb = x.reshape(-1, 32)
    for b in range(xb.shape[0]):
        if b == 2:
            assert raw[b, 0] == 0x00 and raw[b, 1] == 0x3C and np.all(codes[b] == 0)   # zero block: scale 1.0
            continue
        j = int(np.argmax(np.abs(xb[b])))
        assert abs(int(codes[b, j])) == 127                                              # absmax element saturates
        s = np.float32(np.max(np.abs(xb[b]))) / np.float32(127.0)
        assert scales[b] == np.float32(s).astype(np.float16).astype(np.float32)
        t = (xb[b] * (np.float32(1.0) / s)).astype(np.float32).astype(np.float64)
        want = np.clip(np.sign(t) * np.floor(np.abs(t) + 0.5), -127, 127)
        assert np.array_equal(codes[b].astype(np.float64), want)


# ---- rounding ties: f32::round is half AWAY from zero (weight_loader.rs:1482, 1534-1535; emit.rs:1433)
# A block whose largest magnitude is 127.0 (Q8_0, activations) or 8.0 (Q4_0) has scale 1.0 and reciprocal 1.0 exactly, so
# x * inv is x itself and the elements below sit exactly half way between two codes.  The expected codes are written out
# by hand; round-half-to-even (rintf, numpy.round) would give 0, 0, 2, 2, 2, 2, 126, -126 for the first eight.
TIE_INPUT = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 127.0, 0.25, -0.75, 3.0]
TIE_Q8_CODES = [1, -1, 2, -2, 3, -3, 127, -127, 127, 0, -1, 3]
TIE4_INPUT = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 6.5, -7.5, 8.0, -8.0, 7.5, 0.25]
TIE4_CODES = [9, 7, 10, 6, 11, 5, 15, 0, 15, 0, 15, 8]          # round(x) + 8, clamped to [0, 15]


def tie_block(values):
    v = np.zeros(32, np.float32)
    v[:len(values)] = values
    return v


def test_weight_quantiser_q8_0_rounding_ties(oracle):
    raw = oracle.quantize_weights(Q8, tie_block(TIE_INPUT))
    assert (int(raw[0]) | (int(raw[1]) << 8)) == 0x3C00                      # scale 127 / 127 = 1.0
    assert raw[2:2 + len(TIE_Q8_CODES)].view(np.int8).tolist() == TIE_Q8_CODES
    assert np.all(raw[2 + len(TIE_Q8_CODES):] == 0)


def test_weight_quantiser_q4_0_rounding_ties(oracle):
    raw = oracle.quantize_weights(Q4, tie_block(TIE4_INPUT))
    assert (int(raw[0]) | (int(raw[1]) << 8)) == 0x3C00                      # scale 8 / 8 = 1.0
    codes = np.concatenate([raw[2:] & 0x0F, raw[2:] >> 4])                   # elements 0..15, then 16..31
    assert codes[:len(TIE4_CODES)].tolist() == TIE4_CODES
    assert np.all(codes[len(TIE4_CODES):] == 8)                              # zeros sit at the offset


def test_activation_quantiser_rounding_ties(oracle):
    raw = oracle.quantize_act(tie_block(TIE_INPUT))
    assert (int(raw[0]) | (int(raw[1]) << 8)) == 0x3C00
    assert raw[2:2 + len(TIE_Q8_CODES)].view(np.int8).tolist() == TIE_Q8_CODES
    # the same ties at another power-of-two scale: absmax 254 -> s = 2, inv = 0.5, x * inv = 0.5 (k + 0.5)
    raw = oracle.quantize_act(tie_block([2.0 * t for t in TIE_INPUT]))
    assert (int(raw[0]) | (int(raw[1]) << 8)) == 0x4000
    assert raw[2:2 + len(TIE_Q8_CODES)].view(np.int8).tolist() == TIE_Q8_CODES


# ---- KV int8 quantiser: the reference's fixture (emit.rs:6813-6852)
def test_kv_quantiser_reference_fixture(oracle):
    v = (((np.arange(64) * 7 + 3).astype(np.float32) * np.float32(0.1) - np.float32(3.0)) * np.float32(0.5)).astype(np.float32)
    q, scale = oracle.quantize_kv(v)
    assert scale == pytest.approx(float(np.max(np.abs(v))) / 127.0, rel=1e-6)
    assert np.max(np.abs(q.astype(np.float32) * np.float32(scale) - v)) <= scale + 1e-6
    q0, s0 = oracle.quantize_kv(np.zeros(8, np.float32))
    assert s0 == 0.0 and np.all(q0 == 0)


# ---- argmax: Rust's Iterator::max_by keeps the LAST maximum (project.rs:501-503)
def test_argmax_last_maximum(oracle):
    assert oracle.argmax(np.array([1, 5, 3, 5, 2], np.float32)) == 3
    assert oracle.argmax(np.array([7, 7, 7], np.float32)) == 2
    assert oracle.argmax(np.array([-1, -3], np.float32)) == 0
    assert oracle.argmax(np.array([0.1, 0.9, 0.3], np.float32)) == 1     # sampling.rs:165-169 style, no ties
