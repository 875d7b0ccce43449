"""The reference's own unit-test vectors for the hot path (tests/golden/reference_vectors.json, written by
tests/golden/make_reference_vectors.py) against the oracle, against the host-side format code of the shipped
library (CPU tests) and against the GPU kernels (marked gpu)."""
import json
import os

import numpy as np
import pytest

Q8, Q4 = 8, 2
EXACT = 1
HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = json.load(open(os.path.join(HERE, "golden", "reference_vectors.json")))


def _value(text):
    """'2^-24', '1.5*2^-25', 'inf', '-0.0' ... -> float"""
    return float(eval(text.replace("^", "**"), {"__builtins__": {}}, {"inf": np.inf, "nan": np.nan}))


def _ramp(spec, n=None):
    i = np.arange(n if n is not None else spec["n"], dtype=np.float32)
    f = spec["formula"]
    terms = {"(i - 32) * 0.05": lambda: (i - np.float32(32.0)) * np.float32(0.05),
             "(i - 32) * 0.1": lambda: (i - np.float32(32.0)) * np.float32(0.1),
             "((i * 7 + 3) * 0.1 - 3.0) * 0.5": lambda: ((i * 7 + 3) * np.float32(0.1) - np.float32(3.0)) * np.float32(0.5),
             "((i * 7 + 3) * 0.1 - 1.0) * 0.5": lambda: ((i * 7 + 3) * np.float32(0.1) - np.float32(1.0)) * np.float32(0.5),
             "((i * 11 + 5) * 0.07 - 1.0) * 0.3": lambda: ((i * 11 + 5) * np.float32(0.07) - np.float32(1.0)) * np.float32(0.3),
             "((i * 13 + 7) * 0.05 - 0.5) * 0.4": lambda: ((i * 13 + 7) * np.float32(0.05) - np.float32(0.5)) * np.float32(0.4)}
    return terms[f]().astype(np.float32)


def _q8_block(scale_bits, codes):
    return np.concatenate([np.array([scale_bits & 0xFF, scale_bits >> 8], np.uint8), np.asarray(codes, np.int8).view(np.uint8)])


def _q4_block(scale_bits, packed):
    return np.concatenate([np.array([scale_bits & 0xFF, scale_bits >> 8], np.uint8), np.asarray(packed, np.uint8)])


def _impls(fh, oracle):
    """(name, f16->f32 of one pattern, f32->f16 of one value, dequant, weight quantiser) of the oracle and of the library."""
    return [("oracle", lambda b: float(oracle.f16_to_f32(np.array([b], np.uint16))[0]),
             lambda v: int(oracle.f32_to_f16(np.array([v], np.float32))[0]), oracle.dequant, oracle.quantize_weights),
            ("library", fh.ops.f16_to_f32, fh.ops.f32_to_f16, fh.ops.dequant, fh.ops.quantize_weights)]


def test_f16_known_answers(fh, oracle):
    for name, to32, to16, _, _ in _impls(fh, oracle):
        for bits, text in GOLD["f16_to_f32"]["cases"]:
            want, got = _value(text), to32(bits)
            if np.isnan(want):
                assert np.isnan(got), name
            else:
                assert got == want and np.signbit(np.float32(got)) == np.signbit(np.float32(want)), (name, hex(bits))
        for text, bits in GOLD["f32_to_f16_flush"]["cases"]:
            assert to16(_value(text)) == bits, (name, text)


def test_dequant_fixtures(fh, oracle):
    for name, _, _, dequant, _ in _impls(fh, oracle):
        for c in GOLD["dequant_q8_0"]["cases"]:
            assert np.array_equal(dequant(Q8, _q8_block(c["scale_bits"], c["codes"]), 32), np.array(c["expect"], np.float32)), name
        for c in GOLD["dequant_q4_0"]["cases"]:
            assert np.array_equal(dequant(Q4, _q4_block(c["scale_bits"], c["bytes"]), 32), np.array(c["expect"], np.float32)), name


def test_weight_quantiser_invariants(fh, oracle):
    for name, _, _, dequant, quant in _impls(fh, oracle):
        g = GOLD["quantize_q8_0_round_trip"]
        v = _ramp(g["input"])
        raw = quant(Q8, v)
        assert raw.size == g["bytes"], name
        assert np.max(np.abs(dequant(Q8, raw, v.size) - v)) < g["max_abs_error"], name
        assert np.all(dequant(Q8, quant(Q8, np.zeros(32, np.float32)), 32) == 0.0), name
        g = GOLD["quantize_q4_0_invariants"]
        v = _ramp(g["input"])
        raw = quant(Q4, v)
        assert raw.size == g["bytes"], name
        back = dequant(Q4, raw, v.size)
        for blk in range(v.size // 32):
            seg = slice(32 * blk, 32 * blk + 32)
            assert np.all(np.abs(back[seg] - v[seg]) <= np.max(np.abs(v[seg])) / 8.0 + 0.01), name


def test_kv_quantiser_fixture(oracle):
    g = GOLD["kv_int8_quantiser"]
    v = _ramp(g["input"])
    q, scale = oracle.quantize_kv(v)
    assert scale == pytest.approx(float(np.max(np.abs(v))) / 127.0, rel=1e-6)
    assert np.max(np.abs(q.astype(np.float32) * np.float32(scale) - v)) <= scale + 1e-6


def test_f32_kernel_known_answers(oracle):
    g = GOLD["rms_norm"]
    for variant in (0, 1):
        out = oracle.rms_norm(np.array(g["x"], np.float32), np.array(g["weight"], np.float32), g["eps"], variant)
        assert np.allclose(out, g["expect"], rtol=0, atol=g["atol"])
    g = GOLD["silu_mul"]
    assert np.allclose(oracle.silu_mul(np.array(g["gate"], np.float32), np.array(g["up"], np.float32)), g["expect"], rtol=0, atol=g["atol"])
    g = GOLD["softmax"]
    p = oracle.softmax(np.array(g["x"], np.float32))
    assert np.allclose(p, g["expect"], rtol=0, atol=g["atol"]) and p.sum() == pytest.approx(1.0, abs=1e-6)
    for xs, want in GOLD["argmax"]["cases"]:
        assert oracle.argmax(np.array(xs, np.float32)) == want


def _attention_inputs(oracle, seq):
    g = GOLD["attention"]
    hd, nh, nkv = g["head_dim"], g["heads"], g["kv_heads"]
    q = _ramp(g["q"], nh * hd)
    k16 = oracle.f32_to_f16(_ramp(g["k"], seq * nkv * hd)).reshape(seq, nkv * hd)
    v16 = oracle.f32_to_f16(_ramp(g["v"], seq * nkv * hd)).reshape(seq, nkv * hd)
    return q, k16, v16, hd, nh, nkv


def test_attention_flash_equals_standard(oracle):
    g = GOLD["attention"]
    for seq in g["seq_lens"]:
        q, k16, v16, hd, nh, nkv = _attention_inputs(oracle, seq)
        std = oracle.attention("std", q, k16, v16, seq, nh, nkv, hd)
        flash = oracle.attention("flash", q, k16, v16, seq, nh, nkv, hd)
        assert np.max(np.abs(std - flash)) < g["tolerance"]


# ---------------- the same vectors on the GPU, through the C ABI ----------------
@pytest.mark.gpu
def test_gpu_f32_kernels_on_reference_vectors(fh, oracle, torch_gpu):
    torch = torch_gpu
    g = GOLD["rms_norm"]
    x = np.tile(np.array(g["x"], np.float32), 8)                      # the kernel wants rows of at least 32 values
    out = fh.ops.rms_norm(torch.from_numpy(x.reshape(1, -1)).cuda(), torch.ones(x.size, device="cuda"), g["eps"]).cpu().numpy()[0]
    assert np.allclose(out[:4], g["expect"], rtol=0, atol=g["atol"])   # the mean square of the tiled row is the same
    g = GOLD["silu_mul"]
    gate = np.zeros(32, np.float32); up = np.zeros(32, np.float32)
    gate[:3], up[:3] = g["gate"], g["up"]
    out = fh.ops.silu_mul(torch.from_numpy(gate).cuda(), torch.from_numpy(up).cuda()).cpu().numpy()
    assert np.allclose(out[:3], g["expect"], rtol=0, atol=g["atol"])
    for xs, want in GOLD["argmax"]["cases"]:
        assert fh.ops.argmax(torch.tensor(xs, dtype=torch.float32, device="cuda")) == want


@pytest.mark.gpu
def test_gpu_dequant_block_dots_on_reference_blocks(fh, oracle, torch_gpu):
    """The reference's dequantiser fixtures as one-block weight rows: an all-ones activation block (every code 127, scale
    1/127) turns the GEMV into the sum of the dequantised block."""
    torch = torch_gpu
    x = torch.ones(32, device="cuda")
    for c in GOLD["dequant_q8_0"]["cases"]:
        w = fh.ops.QWeight(Q8, _q8_block(c["scale_bits"], c["codes"]), 32, 1)
        want = oracle.matmul_vec(Q8, 0, np.ones(32, np.float32), _q8_block(c["scale_bits"], c["codes"]), 32, 1)
        got = fh.ops.matmul_vec_q(w, x).cpu().numpy()
        assert got.view(np.uint32)[0] == want.view(np.uint32)[0]
        assert got[0] == pytest.approx(float(np.sum(c["expect"])), rel=1e-2, abs=1e-3)
    for c in GOLD["dequant_q4_0"]["cases"]:
        raw = _q4_block(c["scale_bits"], c["bytes"])
        w = fh.ops.QWeight(Q4, raw, 32, 1)
        want = oracle.matmul_vec(Q4, 0, np.ones(32, np.float32), raw, 32, 1)
        got = fh.ops.matmul_vec_q(w, x).cpu().numpy()
        assert got.view(np.uint32)[0] == want.view(np.uint32)[0]
        assert got[0] == pytest.approx(float(np.sum(c["expect"])), rel=1e-2, abs=1e-3)


@pytest.mark.gpu
def test_gpu_attention_on_reference_vectors(fh, oracle, torch_gpu):
    """The reference's inputs have head_dim 8; the kernels start at 64, so each head is padded with zero dimensions
    (which change neither scores nor outputs) and the query scaled by sqrt(64/8) to keep score = q.k / sqrt(8)."""
    torch = torch_gpu
    g = GOLD["attention"]
    for seq in g["seq_lens"]:
        q, k16, v16, hd, nh, nkv = _attention_inputs(oracle, seq)
        want = oracle.attention("std", q, k16, v16, seq, nh, nkv, hd)
        HD = 64
        qp = np.zeros((nh, HD), np.float32); qp[:, :hd] = q.reshape(nh, hd) * np.float32(np.sqrt(HD / hd))
        kp = np.zeros((seq, nkv, HD), np.uint16); kp[:, :, :hd] = k16.reshape(seq, nkv, hd)
        vp = np.zeros((seq, nkv, HD), np.uint16); vp[:, :, :hd] = v16.reshape(seq, nkv, hd)
        dev16 = lambda a: torch.from_numpy(a.reshape(seq, nkv * HD).view(np.int16)).cuda()
        for flags in (0, EXACT):
            got = fh.ops.attention_flash(torch.from_numpy(qp.reshape(-1)).cuda(), dev16(kp), dev16(vp), seq, nh, nkv, HD,
                                         flags).cpu().numpy().reshape(nh, HD)
            assert np.max(np.abs(got[:, :hd].reshape(-1) - want)) < g["tolerance"]
            assert np.all(got[:, hd:] == 0.0)
