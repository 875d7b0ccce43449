"""GGUF input: the library's parser / config reader / weights exporter against the reference's own unit-test vectors
(crates/forgellm-frontend/src/gguf.rs:606-769, restated as the byte strings those tests build), against the Python
restatement in oracle/gguf_oracle.py, and through round trips of seeded synthetic models.  Host code only, except
the last test, which loads a model from a GGUF file onto the GPU."""
import struct

import numpy as np
import pytest

Q8, Q4 = 8, 2


@pytest.fixture(scope="module")
def gg(fh):
    return fh.gguf


@pytest.fixture(scope="module")
def go():
    from oracle import gguf_oracle
    return gguf_oracle


def both(fh, go, data):
    """Parse with the library and with the oracle; check that they agree on everything a GGUFFile holds."""
    lib_file = fh.gguf.GgufFile(data)
    ora = go.parse(data)
    assert lib_file.version == ora["version"]
    assert lib_file.alignment == ora["alignment"]
    assert lib_file.tensor_data_offset == ora["tensor_data_offset"]
    assert lib_file.metadata_count == len(ora["metadata"])
    assert len(lib_file.tensors) == len(ora["tensors"])
    for a, b in zip(lib_file.tensors, ora["tensors"]):
        assert a["name"] == b["name"] and a["dimensions"] == b["dimensions"]
        assert a["ggml_type"] == b["ggml_type"] and a["offset"] == b["offset"]
        assert a["data_size"] == go.data_size(b)
    for key, (vtype, value) in ora["metadata"].items():
        got = lib_file.meta(key)
        if vtype == 9:
            assert got == (value[0], len(value[1])), key
        elif vtype in (6, 12):
            assert np.float64(got) == np.float64(value) or (np.isnan(got) and np.isnan(value)), key
        else:
            assert got == value, key
    return lib_file, ora


def err(fh, data):
    with pytest.raises(fh.ForgeHipError) as e:
        fh.gguf.GgufFile(data)
    assert e.value.code == fh.ERR_INVALID
    return str(e.value)


# ---------------- the reference's unit tests (gguf.rs:606-769) ----------------
def test_reference_parse_minimal_gguf_v3(fh, gg, go):
    data = gg.write_gguf([("general.architecture", gg.STRING, "llama")], [("token_embd.weight", [32000, 2048], gg.F16, None)])
    f, _ = both(fh, go, data)
    assert f.version == 3
    assert f.meta("general.architecture") == "llama"
    assert len(f.tensors) == 1
    assert f.tensors[0]["name"] == "token_embd.weight"
    assert f.tensors[0]["dimensions"] == [32000, 2048]
    assert f.tensors[0]["ggml_type"] == gg.F16


def test_reference_parse_with_multiple_tensors(fh, gg, go):
    # offsets as in the reference's test: 0, 4096, 8192 (descriptors only, no data section)
    meta = [("general.architecture", gg.STRING, "llama"), ("llama.embedding_length", gg.U32, 2048),
            ("llama.attention.layer_norm_rms_epsilon", gg.FLOAT32, 1e-5)]
    head = struct.pack("<IIQQ", gg.MAGIC, 3, 3, 3)
    for k, t, v in meta:
        head += struct.pack("<Q", len(k)) + k.encode() + struct.pack("<I", t) + gg.encode_value(t, v)
    for name, dims, ty, off in [("token_embd.weight", [32000, 2048], 1, 0), ("blk.0.attn_q.weight", [2048, 2048], 8, 4096),
                                ("blk.0.ffn_gate.weight", [5632, 2048], 2, 8192)]:
        head += struct.pack("<Q", len(name)) + name.encode() + struct.pack("<I", len(dims))
        head += b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<IQ", ty, off)
    f, _ = both(fh, go, head)
    assert len(f.tensors) == 3
    assert f.meta("llama.embedding_length") == 2048
    assert f.meta("llama.attention.layer_norm_rms_epsilon") == float(np.float32(1e-5))
    q = f.tensor("blk.0.attn_q.weight")
    assert q["ggml_type"] == Q8 and int(np.prod(q["dimensions"])) == 2048 * 2048 and q["offset"] == 4096
    assert f.tensor("blk.0.ffn_gate.weight")["offset"] == 8192
    assert f.tensor("nope") is None


def test_reference_parse_v2(fh, gg, go):
    f, _ = both(fh, go, gg.write_gguf([], [], version=2))
    assert f.version == 2 and f.tensors == []


def test_reference_reject_invalid_magic(fh, go):
    data = bytearray(32)
    data[0:4] = struct.pack("<I", 0xDEADBEEF)
    assert "invalid GGUF magic number: got 0xDEADBEEF" in err(fh, bytes(data))
    with pytest.raises(go.GgufError, match="0xDEADBEEF"):
        go.parse(bytes(data))


def test_reference_reject_unsupported_version(fh, gg, go):
    data = struct.pack("<IIQQ", gg.MAGIC, 99, 0, 0)
    assert "unsupported GGUF version: 99 (supported: 2, 3)" in err(fh, data)
    with pytest.raises(go.GgufError, match="99"):
        go.parse(data)


def test_reference_tensor_data_size(fh, gg, go):
    data = gg.write_gguf([], [("test", [32000, 2048], gg.F16, None), ("test2", [2048, 2048], gg.Q4_0, None)])
    f, _ = both(fh, go, data)
    assert f.tensors[0]["data_size"] == 32000 * 2048 * 2
    assert f.tensors[1]["data_size"] == (2048 * 2048 // 32) * 18


def test_reference_alignment_calculation(fh, gg, go):
    f, _ = both(fh, go, gg.write_gguf([], []))
    assert f.alignment == 32 and f.tensor_data_offset % 32 == 0
    # 24 header bytes round up to one alignment unit
    assert f.tensor_data_offset == 32


# ---------------- beyond the reference's tests ----------------
def test_every_metadata_type_and_nested_arrays(fh, gg, go):
    meta = [("a.u8", gg.U8, 200), ("a.i8", gg.I8, -100), ("a.u16", gg.U16, 60000), ("a.i16", gg.I16, -30000),
            ("a.u32", gg.U32, 4000000000), ("a.i32", gg.I32, -2000000000), ("a.f32", gg.FLOAT32, 0.1), ("a.true", gg.BOOL, 1),
            ("a.false", gg.BOOL, 0), ("a.str", gg.STRING, "héllo wörld ✓"), ("a.empty", gg.STRING, ""),
            ("a.u64", gg.U64, 2 ** 63 + 5), ("a.i64", gg.I64, -2 ** 62), ("a.f64", gg.FLOAT64, 1e300),
            ("arr.u32", gg.ARRAY, (gg.U32, [1, 2, 3])), ("arr.str", gg.ARRAY, (gg.STRING, ["a", "bc", ""])),
            ("arr.empty", gg.ARRAY, (gg.FLOAT64, [])),
            ("arr.nested", gg.ARRAY, (gg.ARRAY, [(gg.U8, [1, 2]), (gg.STRING, ["x"]), (gg.ARRAY, [(gg.I16, [-1])])])),
            ("general.alignment", gg.U32, 64)]
    data = gg.write_gguf(meta, [("t", [3], gg.F32, np.arange(3, dtype=np.float32))], alignment=64)
    f, o = both(fh, go, data)
    assert f.alignment == 64 and f.tensor_data_offset % 64 == 0
    assert f.meta("a.i8") == -100 and f.meta("a.i64") == -2 ** 62 and f.meta("a.u64") == 2 ** 63 + 5
    assert f.meta("a.true") is True and f.meta("a.false") is False
    assert f.meta("a.str") == "héllo wörld ✓"
    assert f.meta("arr.nested") == (gg.ARRAY, 3)
    assert f.meta("missing") is None
    # the data really sits at tensor_data_offset
    assert np.frombuffer(data, np.float32, 3, f.tensor_data_offset).tolist() == [0.0, 1.0, 2.0]


def test_a_repeated_key_keeps_the_last_value(fh, gg, go):
    f, _ = both(fh, go, gg.write_gguf([("k", gg.U32, 1), ("k", gg.U32, 2)], []))
    assert f.meta("k") == 2 and f.metadata_count == 1


def test_parse_errors(fh, gg, go):
    good = gg.write_gguf([("general.architecture", gg.STRING, "llama")], [("t", [4, 4], gg.F32, None)])
    assert "unsupported GGML type ID: 5" in err(fh, gg.write_gguf([], [("t", [4], 5, None)]))
    assert "unsupported GGML type ID: 31" in err(fh, gg.write_gguf([], [("t", [4], 31, None)]))
    assert "tensor dimension count 5 exceeds maximum (4)" in err(fh, gg.write_gguf([], [("t", [1, 1, 1, 1, 1], gg.F32, None)]))
    bad_type = struct.pack("<IIQQ", gg.MAGIC, 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<I", 13)
    assert "unsupported metadata value type: 13" in err(fh, bad_type)
    bad_utf8 = struct.pack("<IIQQ", gg.MAGIC, 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<I", 8) + struct.pack("<Q", 2) + b"\xff\xfe"
    assert "invalid UTF-8" in err(fh, bad_utf8)
    with pytest.raises(go.GgufError, match="UTF-8"):
        go.parse(bad_utf8)
    # every proper prefix of a good file is refused (never read past the end), the whole file is accepted
    for cut in range(len(good)):
        err(fh, good[:cut])
        with pytest.raises(go.GgufError):
            go.parse(good[:cut])
    both(fh, go, good)
    # a string length that points far past the end
    huge = struct.pack("<IIQQ", gg.MAGIC, 3, 0, 1) + struct.pack("<Q", 2 ** 62)
    err(fh, huge)
    # an array count that points far past the end
    huge_arr = struct.pack("<IIQQ", gg.MAGIC, 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<IIQ", 9, 4, 2 ** 61)
    err(fh, huge_arr)


@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("tied", [True, False])
@pytest.mark.parametrize("bias", [False, True])
def test_synthetic_model_round_trip(fh, gg, go, oracle, wd, tied, bias, tmp_path):
    """blob -> GGUF file -> (library) config + blob: identical bytes, identical configuration; same through the oracle.
    bias: a Qwen2-style model (architecture qwen2, bias vectors after the v weights)."""
    cfg = fh.synth.tiny(wd, max_seq=640)
    if bias:
        cfg["flags"] = fh.FLAG_QKV_BIAS
    blob = fh.synth.make_weights_blob(cfg, seed=11)
    path = str(tmp_path / "m.gguf")
    data = gg.model_to_gguf(cfg, blob, tied=tied, path=path, tokens=tied)
    for source in (path, data):
        f = gg.GgufFile(source)
        got = f.config()
        assert {k: got[k] for k in cfg if k not in ("rms_eps", "rope_theta")} == {k: cfg[k] for k in cfg if k not in ("rms_eps", "rope_theta")}
        assert np.float32(got["rms_eps"]) == np.float32(cfg["rms_eps"]) and np.float32(got["rope_theta"]) == np.float32(cfg["rope_theta"])
        out = f.export_weights(got)
        assert out.size == blob.size and np.array_equal(out, blob)
        assert f.config(max_seq=128, flags=1)["max_seq"] == 128 and f.config(max_seq=128, flags=1)["flags"] == 1 | cfg.get("flags", 0)
        f.close()
    o = go.parse(data)
    ocfg = go.config(o)
    assert ocfg == got
    assert np.array_equal(go.export_weights(oracle, o, data, ocfg), blob)


@pytest.mark.parametrize("wd", [Q8, Q4])
def test_phi3_fused_tensors_are_split(fh, gg, go, oracle, wd):
    """A Phi-3 file keeps Q|K|V rows in `attn_qkv.weight` and gate|up rows in `ffn_up.weight`; the reference's loader cuts them
    apart (split_fused_tensors, weight_loader.rs:543-583) before export-weights writes q, k, v, gate, up one by one.
    blob -> fused GGUF -> blob: identical bytes; library == oracle; the fused tensors vote like any projection."""
    cfg = fh.synth.tiny(wd, max_seq=640, heads=4, kv_heads=2, head_dim=96, hidden=384)     # Phi-3's head_dim, GQA so that q != k rows
    blob = fh.synth.make_weights_blob(cfg, seed=21)
    data = gg.model_to_gguf(cfg, blob, tied=False, fused=True)
    f = gg.GgufFile(data)
    names = {t["name"] for t in f.tensors}
    assert "blk.0.attn_qkv.weight" in names and "blk.0.attn_q.weight" not in names and "blk.0.ffn_gate.weight" not in names
    got = f.config()
    assert got["wdtype"] == wd and got["head_dim"] == 96 and got["flags"] == 0
    assert np.array_equal(f.export_weights(got), blob)
    o = go.parse(data)
    assert go.config(o) == got
    assert np.array_equal(go.export_weights(oracle, o, data, got), blob)
    f.close()
    # "phi" is the same architecture to the reference (main.rs:759)
    data_phi = gg.model_to_gguf(cfg, blob, tied=False, fused=True, arch="phi")
    assert np.array_equal(gg.GgufFile(data_phi).export_weights(got), blob)


def test_phi3_fused_tensors_in_other_formats(fh, gg, go, oracle):
    """Fused tensors that are not in the blob's format are converted whole and then cut, as the reference's loader does:
    an F16 `attn_qkv`, a Q6_K `ffn_up` (read as Q8_0) in a Q8_0 model; library == oracle, and each part equals what the same
    rows give as a tensor of their own."""
    cfg = fh.synth.tiny(Q8, max_seq=640, hidden=256, inter=512, heads=4, kv_heads=2, head_dim=64)
    blob = fh.synth.make_weights_blob(cfg, seed=22)
    t = gg.split_blob(cfg, blob)
    H, I, QKS, KV = cfg["hidden"], cfg["inter"], 256, 128
    qkv = np.concatenate([oracle.dequant(Q8, t[f"blk.0.attn_{n}.weight"][2], H * r) for n, r in (("q", QKS), ("k", KV), ("v", KV))])
    for n in ("q", "k", "v"):
        del t[f"blk.0.attn_{n}.weight"]
    t["blk.0.attn_qkv.weight"] = ([H, QKS + 2 * KV], gg.F16, oracle.f32_to_f16(qkv).astype("<u2").view(np.uint8))
    rng = np.random.default_rng(5)
    q6 = rng.integers(0, 256, 2 * I * H // 256 * 210, dtype=np.uint8)
    q6.reshape(-1, 210)[:, 208:] = np.frombuffer(np.float16(rng.uniform(0.001, 0.01, 2 * I * H // 256)).tobytes(), np.uint8).reshape(-1, 2)
    del t["blk.0.ffn_gate.weight"]
    t["blk.0.ffn_up.weight"] = ([H, 2 * I], gg.Q6_K, q6)
    meta = [("general.architecture", gg.STRING, "phi3"), ("phi3.embedding_length", gg.U32, H), ("phi3.block_count", gg.U32, cfg["layers"]),
            ("phi3.attention.head_count", gg.U32, cfg["heads"]), ("phi3.attention.head_count_kv", gg.U32, cfg["kv_heads"]),
            ("phi3.feed_forward_length", gg.U32, I), ("phi3.vocab_size", gg.U32, cfg["vocab"]), ("phi3.context_length", gg.U32, 640)]
    data = gg.write_gguf(meta, [(n, d, g, b) for n, (d, g, b) in t.items()])
    f = gg.GgufFile(data)
    got = f.config()
    o = go.parse(data)
    assert go.config(o) == got and got["wdtype"] == Q8
    out = f.export_weights(got)
    assert np.array_equal(out, go.export_weights(oracle, o, data, got))
    parts = gg.split_blob(got, out)
    # each part is what its own rows give when they are quantised as a tensor of their own
    qkv16 = oracle.f16_to_f32(oracle.f32_to_f16(qkv))
    for n, r, at in (("q", QKS, 0), ("k", KV, QKS), ("v", KV, QKS + KV)):
        assert np.array_equal(parts[f"blk.0.attn_{n}.weight"][2], oracle.quantize_weights(Q8, qkv16[at * H:(at + r) * H]))
    whole = oracle.quantize_weights(Q8, gg.dequant_ggml(gg.Q6_K, q6, 2 * I * H))
    assert np.array_equal(parts["blk.0.ffn_gate.weight"][2], whole[:I * H // 32 * 34])
    assert np.array_equal(parts["blk.0.ffn_up.weight"][2], whole[I * H // 32 * 34:])
    # a fused tensor of the wrong size is refused like any other
    t["blk.0.attn_qkv.weight"] = ([H, QKS + KV], gg.F16, oracle.f32_to_f16(qkv[:(QKS + KV) * H]).astype("<u2").view(np.uint8))
    bad = gg.write_gguf(meta, [(n, d, g, b) for n, (d, g, b) in t.items()])
    with pytest.raises(fh.ForgeHipError, match="elements"):
        gg.GgufFile(bad).export_weights(got)
    with pytest.raises(go.GgufError):
        go.export_weights(oracle, go.parse(bad), bad, got)


def test_tensors_in_other_formats_are_converted_like_the_oracle_does(fh, gg, go, oracle):
    """A Q8_0 model whose norms are F16, one projection F32, one BF16, one Q4_0, with an F16 embedding and a Q4_0 output
    matrix: the exporter dequantises / requantises with the reference's routines; library == oracle, byte for byte."""
    cfg = fh.synth.tiny(Q8, max_seq=640)
    blob = fh.synth.make_weights_blob(cfg, seed=12)
    t = gg.split_blob(cfg, blob)
    H, V = cfg["hidden"], cfg["vocab"]

    def f32_of(name):
        dims, ty, raw = t[name]
        n = int(np.prod(dims))
        return raw.view(np.float32).copy() if ty == gg.F32 else oracle.dequant(ty, raw, n)

    def as_f16(x):
        return oracle.f32_to_f16(x).astype("<u2").view(np.uint8)

    t["blk.0.attn_norm.weight"] = ([H], gg.F16, as_f16(f32_of("blk.0.attn_norm.weight")))
    t["blk.0.attn_q.weight"] = (t["blk.0.attn_q.weight"][0], gg.F32, f32_of("blk.0.attn_q.weight").view(np.uint8))
    bf = (f32_of("blk.1.ffn_up.weight").view(np.uint32) >> 16).astype("<u2").view(np.uint8)
    t["blk.1.ffn_up.weight"] = (t["blk.1.ffn_up.weight"][0], gg.BF16, bf)
    t["blk.1.attn_v.weight"] = (t["blk.1.attn_v.weight"][0], gg.Q4_0, oracle.quantize_weights(Q4, f32_of("blk.1.attn_v.weight")))
    t["token_embd.weight"] = ([H, V], gg.F16, as_f16(f32_of("token_embd.weight")))
    t["output.weight"] = ([H, V], gg.Q4_0, oracle.quantize_weights(Q4, f32_of("output.weight")))
    meta = [("general.architecture", gg.STRING, "llama"), ("llama.embedding_length", gg.U32, H), ("llama.block_count", gg.U32, cfg["layers"]),
            ("llama.attention.head_count", gg.U32, cfg["heads"]), ("llama.attention.head_count_kv", gg.U32, cfg["kv_heads"]),
            ("llama.feed_forward_length", gg.U32, cfg["inter"]), ("llama.vocab_size", gg.U64, V), ("llama.context_length", gg.U64, 640),
            ("llama.attention.layer_norm_rms_epsilon", gg.FLOAT32, cfg["rms_eps"]), ("llama.rope.freq_base", gg.FLOAT32, cfg["rope_theta"])]
    data = gg.write_gguf(meta, [(n, d, g, b) for n, (d, g, b) in t.items()])
    f = gg.GgufFile(data)
    got = f.config()
    assert got["wdtype"] == Q8 and got["lm_head_dtype"] == Q4 and got["vocab"] == V and got["max_seq"] == 640
    o = go.parse(data)
    assert go.config(o) == got
    out = f.export_weights(got)
    want = go.export_weights(oracle, o, data, got)
    assert out.size == want.size and np.array_equal(out, want)
    # untouched tensors came through verbatim
    same = gg.split_blob(got, out)
    for name in ("blk.0.attn_k.weight", "blk.1.ffn_down.weight", "output_norm.weight"):
        assert np.array_equal(same[name][2], t[name][2])
    # F32 -> Q8_0 of values that were Q8_0 to begin with reproduces the blocks' values
    assert np.array_equal(oracle.dequant(Q8, same["blk.0.attn_q.weight"][2], H * cfg["heads"] * cfg["head_dim"]), f32_of("blk.0.attn_q.weight"))


def test_config_defaults_and_refusals(fh, gg, go):
    def make(meta, tensors=(("blk.0.attn_q.weight", [64, 64], gg.Q8_0, None),)):
        return gg.write_gguf(meta, list(tensors))

    base = [("general.architecture", gg.STRING, "llama"), ("llama.embedding_length", gg.U32, 64), ("llama.block_count", gg.U32, 1),
            ("llama.attention.head_count", gg.U32, 1)]
    f = gg.GgufFile(make(base))
    c = f.config()
    o = go.config(go.parse(make(base)))
    assert c == o
    # defaults of main.rs:716-757
    assert (c["kv_heads"], c["inter"], c["vocab"], c["max_seq"], c["head_dim"]) == (1, 256, 32000, 2048, 64)
    assert np.float32(c["rms_eps"]) == np.float32(1e-5) and c["rope_theta"] == 10000.0
    assert c["wdtype"] == Q8 and c["lm_head_dtype"] == Q8

    def refused(meta, tensors=None, text=""):
        data = make(meta) if tensors is None else make(meta, tensors)
        g = gg.GgufFile(data)
        with pytest.raises(fh.ForgeHipError) as e:
            g.config()
        assert text in str(e.value)
        with pytest.raises(go.GgufError):
            go.config(go.parse(data))

    refused([("general.architecture", gg.STRING, "gemma")] + base[1:], text="unsupported GGUF architecture: gemma")
    # qwen2: the QKV bias goes with the architecture (main.rs:770)
    qmeta = [("general.architecture", gg.STRING, "qwen2")] + [(k.replace("llama.", "qwen2."), t, v) for k, t, v in base[1:]]
    cq = gg.GgufFile(make(qmeta)).config()
    assert cq["flags"] == fh.FLAG_QKV_BIAS and cq == go.config(go.parse(make(qmeta)))
    refused(base[1:], text="unsupported GGUF architecture: unknown")
    refused(base[:2], text="could not extract model config")
    # get_u32 takes a Uint32 value only (gguf.rs:306-308): the same key as u64 does not count
    refused([base[0], ("llama.embedding_length", gg.U64, 64)] + base[2:], text="could not extract model config")
    refused(base, tensors=(("blk.0.attn_q.weight", [64, 64], gg.F16, None),), text="neither mostly Q8_0 nor mostly Q4_0")
    refused(base, tensors=(("blk.0.attn_q.weight", [256, 64], 12, None),), text="neither mostly Q8_0 nor mostly Q4_0")
    refused(base, tensors=(("blk.0.attn_q.weight", [64, 64], gg.Q8_0, None), ("output.weight", [256, 64], 10, None)), text="output.weight")
    # a Q6_K output matrix is read as Q8_0 (GGMLType::to_dtype, gguf.rs:168-205); Q5_K projections vote as Q8_0 (main.rs:509-531)
    kq = (("blk.0.attn_q.weight", [256, 64], gg.Q5_K, None), ("output.weight", [256, 64], gg.Q6_K, None))
    ck = gg.GgufFile(make(base, kq)).config()
    assert (ck["wdtype"], ck["lm_head_dtype"]) == (Q8, Q8) and ck == go.config(go.parse(make(base, kq)))
    # the window travels into the config (main.rs:764-767)
    for w in (1024, 4096):
        blob_w = make(base + [("llama.attention.sliding_window", gg.U32, w)])
        win = gg.GgufFile(blob_w)
        cw = win.config()
        assert cw["sliding_window"] == w and cw["max_seq"] == 2048 and cw == go.config(go.parse(blob_w))
        assert win.config(flags=fh.FLAG_EXACT)["flags"] == fh.FLAG_EXACT
    assert c["sliding_window"] == 0
    refused(base + [("llama.attention.sliding_window", gg.U32, 0)], text="sliding window of 0")
    # the vote: 2 x Q4_0 against 1 x Q8_0
    vote = (("blk.0.attn_q.weight", [64, 64], gg.Q4_0, None), ("blk.0.attn_k.weight", [64, 64], gg.Q4_0, None),
            ("blk.0.ffn_up.weight", [64, 64], gg.Q8_0, None), ("blk.0.attn_norm.weight", [64], gg.F32, None),
            ("token_embd.weight", [64, 10], gg.F16, None))
    assert gg.GgufFile(make(base, vote)).config()["wdtype"] == Q4


def test_export_errors(fh, gg):
    cfg = fh.synth.tiny(Q8, max_seq=640)
    blob = fh.synth.make_weights_blob(cfg, seed=13)
    t = gg.split_blob(cfg, blob)
    meta = [("general.architecture", gg.STRING, "llama")]

    def export(tensors, c=cfg):
        f = gg.GgufFile(gg.write_gguf(meta, [(n, d, g, b) for n, (d, g, b) in tensors.items()]))
        with pytest.raises(fh.ForgeHipError) as e:
            f.export_weights(c)
        return str(e.value)

    missing = dict(t)
    del missing["blk.1.ffn_gate.weight"]
    assert "weight not found: blk.1.ffn_gate.weight" in export(missing)
    wrong = dict(t)
    wrong["blk.0.attn_k.weight"] = ([cfg["hidden"], 8], Q8, t["blk.0.attn_k.weight"][2][:8 * cfg["hidden"] // 32 * 34])
    assert "blk.0.attn_k.weight has" in export(wrong)
    kq = dict(t)
    d = kq["blk.0.ffn_down.weight"][0]
    kq["blk.0.ffn_down.weight"] = (d, 11, np.zeros(int(np.prod(d)) // 256 * 110, np.uint8))      # Q3_K
    assert "this library reads F32, F16, BF16, Q8_0, Q4_0, Q4_1, Q4_K, Q5_K, Q6_K and Q8_K tensors" in export(kq)
    # a data section cut short: the last tensor extends past the end of the file
    data = gg.write_gguf(meta, [(n, d, g, b) for n, (d, g, b) in t.items()])
    f = gg.GgufFile(data[:-4096])
    with pytest.raises(fh.ForgeHipError) as e:
        f.export_weights(cfg)
    assert "extends past end of file" in str(e.value)
    # wrong buffer size
    from ctypes import byref, c_void_p
    f = gg.GgufFile(data)
    c = fh.Config(**cfg)
    out = np.empty(16, np.uint8)
    assert fh.lib().forge_hip_gguf_export_weights(f._h, byref(c), out.ctypes.data_as(c_void_p), 16) == fh.ERR_BLOB_SIZE
    with pytest.raises(fh.ForgeHipError):
        gg.GgufFile("/nonexistent/dir/model.gguf")


def test_damaged_files_are_refused_or_read_but_never_crash(fh, gg):
    """Random byte damage to a small valid model file: parsing, configuration and export each either succeed or come
    back with an error code (the process survives; nothing is read outside the buffer)."""
    cfg = fh.synth.tiny(Q8, max_seq=640, hidden=64, inter=64, layers=1, heads=1, kv_heads=1, head_dim=64, vocab=64)
    blob = fh.synth.make_weights_blob(cfg, seed=17)
    good = bytearray(gg.model_to_gguf(cfg, blob, tied=False, tokens=True))
    head = gg.GgufFile(bytes(good)).tensor_data_offset
    rng = np.random.default_rng(5)
    outcomes = {"ok": 0, "refused": 0}
    for trial in range(600):
        data = bytearray(good)
        for _ in range(int(rng.integers(1, 4))):
            pos = int(rng.integers(0, head))                  # damage the header, metadata and descriptors
            data[pos] = int(rng.integers(0, 256))
        if trial % 5 == 0:
            data = data[:int(rng.integers(0, len(data)))]
        try:
            f = gg.GgufFile(bytes(data))
            c = f.config()
            if fh.hip_model.weights_nbytes(c) < (1 << 26):    # a damaged size field may ask for gigabytes: skip those
                f.export_weights(c)
            outcomes["ok"] += 1
        except fh.ForgeHipError:
            outcomes["refused"] += 1
    assert outcomes["refused"] > 50 and outcomes["ok"] > 5, outcomes


# ---------------- the other block formats the reference's loader reads ----------------
def test_hostile_sizes_are_refused_before_anything_is_computed_from_them(fh, gg, tmp_path):
    """Numbers a file controls (tensor dimensions, embedding length, vocabulary, layer count) are checked before any size
    is derived from them: products that wrap 64 bits, dimensions no kernel covers, a blob size beyond 64 bits, an
    allocation that cannot be had.  Every case comes back as an error code."""
    base = [("general.architecture", gg.STRING, "llama"), ("llama.embedding_length", gg.U32, 64), ("llama.block_count", gg.U32, 1),
            ("llama.attention.head_count", gg.U32, 1)]
    q = ("blk.0.attn_q.weight", [64, 64], gg.Q8_0, None)
    # tensor dimensions: a product that wraps to 0, one that wraps to a small number, one that is merely absurd
    for dims in ([1 << 32, 1 << 32], [(1 << 63) + 1, 2, 1, 1], [1 << 40, 1 << 20], [1 << 49]):
        assert "more than 2^48 elements" in err(fh, gg.write_gguf(base, [q, ("blk.0.attn_k.weight", dims, gg.F16, None)]))
    gg.GgufFile(gg.write_gguf(base, [q, ("blk.0.attn_k.weight", [1 << 24, 1 << 24], gg.F16, None)]))      # 2^48 itself parses

    def config_error(meta):
        with pytest.raises(fh.ForgeHipError) as e:
            gg.GgufFile(gg.write_gguf(meta, [q])).config()
        assert e.value.code == fh.ERR_INVALID
        return str(e.value)

    def with_(key, vtype, value):
        return [(k, t, value if k == key else v) for k, t, v in base] if any(k == key for k, _, _ in base) else base + [(key, vtype, value)]

    assert "embedding_length out of range" in config_error(with_("llama.embedding_length", gg.U32, 0xFFFFFFE0))   # 4 * hidden would wrap
    assert "hidden must be" in config_error(with_("llama.embedding_length", gg.U32, 1 << 20))
    assert "hidden must be" in config_error(with_("llama.embedding_length", gg.U32, 1 << 20) + [("llama.feed_forward_length", gg.U32, 64)])
    assert "head_dim must be" in config_error(with_("llama.attention.head_count", gg.U32, 0xFFFFFFFF))
    assert "inter must be" in config_error(with_("llama.feed_forward_length", gg.U32, 0xFFFFFFFF))
    assert "at most 16384" in config_error(with_("llama.feed_forward_length", gg.U32, 0xFFFFFFE0))
    assert "out of range" in config_error(with_("llama.vocab_size", gg.U64, 1 << 40))
    assert "out of range" in config_error(with_("llama.context_length", gg.U64, 1 << 33))
    # numbers that pass (a 32-bit vocabulary and layer count on a small hidden size): the sizes are real, just unobtainable
    big = gg.GgufFile(gg.write_gguf(base + [("llama.vocab_size", gg.U64, 0xFFFFFFFF)], [q]))
    c = big.config()
    assert c["vocab"] == 0xFFFFFFFF
    n = fh.hip_model.weights_nbytes(c)
    assert n > (1 << 40)
    from ctypes import byref, c_void_p
    small = np.empty(16, np.uint8)
    assert fh.lib().forge_hip_gguf_export_weights(big._h, byref(fh.Config(**c)), small.ctypes.data_as(c_void_p), 16) == fh.ERR_BLOB_SIZE
    path = str(tmp_path / "big.gguf")
    gg.write_gguf(base + [("llama.vocab_size", gg.U64, 0xFFFFFFFF)], [q], path=path)
    h = c_void_p()
    rc = fh.lib().forge_hip_model_create_from_gguf(path.encode(), 0, 0, byref(h))
    assert rc == fh.ERR_INVALID and not h.value               # no terabyte to be had, or no such tensors: an error either way
    # a configuration whose blob size does not fit 64 bits has size 0, and no model is made from it
    wild = dict(c, hidden=16352, inter=0xFFFFFFE0, layers=0xFFFFFFFF, vocab=0xFFFFFFFF, heads=128, kv_heads=128, head_dim=128)
    assert fh.hip_model.weights_nbytes(wild) == 0
    with pytest.raises(fh.ForgeHipError):
        fh.HipModel(wild, np.zeros(16, np.uint8))
    with pytest.raises(fh.ForgeHipError):
        big.export_weights(wild)


def f16le(bits):
    return struct.pack("<H", bits)


def dq(fh, go, oracle, ty, block, n):
    """Dequantise with the library and with the oracle; they must agree bit for bit."""
    a = fh.gguf.dequant_ggml(ty, np.frombuffer(bytes(block), np.uint8), n)
    b = go.dequant_ggml(oracle, ty, np.frombuffer(bytes(block), np.uint8), n)
    assert a.shape == (n,) and np.array_equal(a.view(np.uint32), np.asarray(b, np.float32).view(np.uint32))
    return a


def test_reference_dequant_q4_1_basic(fh, gg, go, oracle):
    """weight_loader.rs:3245-3259: scale 2.0, minimum 1.0, all nibbles 0 -> 1.0 everywhere."""
    block = f16le(0x4000) + f16le(0x3C00) + bytes(16)
    assert np.all(np.abs(dq(fh, go, oracle, gg.Q4_1, block, 32) - 1.0) < 1e-6)


def test_reference_dequant_q4_k(fh, gg, go, oracle):
    """weight_loader.rs:3422-3478."""
    block = bytearray(144)
    block[0:2] = f16le(0x3C00)
    for i in (4, 5, 6, 7, 12, 13, 14, 15):
        block[i] = 1
    assert np.all(np.abs(dq(fh, go, oracle, gg.Q4_K, block, 256)) < 1e-6)
    block = bytearray(144)
    block[0:2], block[2:4] = f16le(0x4000), f16le(0x3C00)
    block[4], block[8] = 3, 2
    for i in range(32):
        block[16 + i] = 0x05
    out = dq(fh, go, oracle, gg.Q4_K, block, 256)
    assert np.all(np.abs(out[:32] - 28.0) < 1e-4)


def test_reference_dequant_q5_k(fh, gg, go, oracle):
    """weight_loader.rs:3481-3560."""
    block = bytearray(176)
    block[0:2] = f16le(0x3C00)
    for i in (4, 5, 6, 7, 12, 13, 14, 15):
        block[i] = 1
    assert np.all(np.abs(dq(fh, go, oracle, gg.Q5_K, block, 256)) < 1e-6)
    block = bytearray(176)
    block[0:2] = f16le(0x3C00)
    block[4], block[16], block[48] = 1, 0x01, 0x03
    assert abs(dq(fh, go, oracle, gg.Q5_K, block, 256)[0] - 19.0) < 1e-4
    block = bytearray(176)
    block[0:2] = f16le(0x3C00)
    block[5], block[16], block[48] = 2, 0x02, 0x70
    assert abs(dq(fh, go, oracle, gg.Q5_K, block, 256)[32] - 46.0) < 1e-4


def test_reference_dequant_q6_k(fh, gg, go, oracle):
    """weight_loader.rs:3562-3656."""
    block = bytearray(210)
    block[208:210] = f16le(0x3C00)
    for i in range(192, 208):
        block[i] = 1
    assert np.all(np.abs(dq(fh, go, oracle, gg.Q6_K, block, 256) + 32.0) < 1e-4)
    block = bytearray(210)
    block[208:210] = f16le(0x3800)
    block[192], block[0], block[128] = 2, 0x0A, 0x02
    assert abs(dq(fh, go, oracle, gg.Q6_K, block, 256)[0] - 10.0) < 1e-4
    block = bytearray(210)
    block[208:210] = f16le(0x3C00)
    for i in range(192, 208):
        block[i] = 1
    block[0], block[32], block[128] = 0x31, 0x52, 0xE4
    out = dq(fh, go, oracle, gg.Q6_K, block, 256)
    assert [abs(out[i] - w) < 1e-4 for i, w in ((0, -31.0), (32, -14.0), (64, 3.0), (96, 21.0))] == [True] * 4


def random_blocks(ty, nblocks, seed):
    """Random bytes with sane scale fields (finite f16 / f32 in the positions that hold them)."""
    rng = np.random.default_rng(seed)
    nbytes = {3: 20, 12: 144, 13: 176, 14: 210, 15: 292}[ty]
    b = rng.integers(0, 256, (nblocks, nbytes), dtype=np.uint8)
    halves = {3: (0, 2), 12: (0, 2), 13: (0, 2), 14: (208,), 15: ()}[ty]
    for off in halves:
        b[:, off:off + 2] = (rng.normal(0, 0.05, nblocks).astype(np.float16)).view(np.uint8).reshape(nblocks, 2)
    if ty == 15:
        b[:, 0:4] = rng.normal(0, 0.05, nblocks).astype(np.float32).view(np.uint8).reshape(nblocks, 4)
    return b.reshape(-1)


@pytest.mark.parametrize("ty", [3, 12, 13, 14, 15])
def test_dequantisers_on_random_blocks_and_closed_forms(fh, gg, go, oracle, ty):
    per = 32 if ty == 3 else 256
    raw = random_blocks(ty, 37, 50 + ty)
    out = dq(fh, go, oracle, ty, raw, 37 * per)
    assert np.all(np.isfinite(out))
    # a ragged element count stops inside the last block
    assert np.array_equal(dq(fh, go, oracle, ty, raw, 36 * per + 5), out[:36 * per + 5])
    # an element-by-element float64 evaluation of the format's definition, independent of both implementations
    b = raw.reshape(37, -1)[3]
    h = lambda o: float(np.frombuffer(bytes(b[o:o + 2]), np.float16)[0])
    want = np.zeros(per)
    if ty == 3:
        for j in range(16):
            want[j] = (int(b[4 + j]) & 15) * h(0) + h(2)
            want[j + 16] = (int(b[4 + j]) >> 4) * h(0) + h(2)
    elif ty in (12, 13):
        sc = b[4:16]
        for j in range(8):
            sc = [int(x) for x in b[4:16]]
            s, m = (sc[j] & 63, sc[j + 4] & 63) if j < 4 else ((sc[j + 4] & 15) | ((sc[j - 4] >> 6) << 4), (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4))
            qs = b[(48 if ty == 13 else 16):]
            for l in range(32):
                q = int(qs[(j // 2) * 32 + l])
                v = (q >> 4) if j % 2 else (q & 15)
                if ty == 13 and (int(b[16 + l]) >> j) & 1:
                    v += 16
                want[j * 32 + l] = h(0) * s * v - h(2) * m
    elif ty == 14:
        ql, qh, sc, d = b[:128], b[128:192], b[192:208].view(np.int8), h(208)
        for e in range(256):
            half, r = divmod(e, 128)
            k, l = divmod(r, 32)
            lo = int(ql[64 * half + l + (32 if k in (1, 3) else 0)])
            nib = (lo >> 4) if k >= 2 else (lo & 15)
            hi2 = (int(qh[32 * half + l]) >> (2 * k)) & 3
            want[e] = d * int(sc[8 * half + 2 * k + l // 16]) * ((nib | (hi2 << 4)) - 32)
    else:
        scale = float(np.frombuffer(bytes(b[:4]), np.float32)[0])
        want = scale * b[4:260].view(np.int8).astype(np.float64)
    assert np.allclose(out[3 * per:4 * per], want, rtol=1e-5, atol=1e-6)


def test_unsupported_type_for_dequant(fh, gg):
    with pytest.raises(fh.ForgeHipError):
        gg.dequant_ggml(11, np.zeros(110, np.uint8), 256)


def test_k_quant_tensors_are_read_as_q8_0_like_the_reference_loader_does(fh, gg, go, oracle):
    """A Q8_0 model file in which the embedding is Q6_K (what llama.cpp writes into many files), one projection Q5_K, one
    Q4_K, one Q4_1 and the output matrix Q6_K: each becomes Q8_0 blocks on load (weight_loader.rs:219-229), the f32
    embedding table is the dequantised Q8_0 form (main.rs:2700-2705).  Library == oracle byte for byte; and the
    closed form: requantised tensor == quantize_q8_0(dequant(raw))."""
    cfg = fh.synth.tiny(Q8, max_seq=640, hidden=256, inter=512, vocab=1024)
    blob = fh.synth.make_weights_blob(cfg, seed=15)
    t = gg.split_blob(cfg, blob)
    H, V = cfg["hidden"], cfg["vocab"]
    swaps = {"token_embd.weight": gg.Q6_K, "output.weight": gg.Q6_K, "blk.0.ffn_up.weight": gg.Q5_K, "blk.1.attn_q.weight": gg.Q4_K,
             "blk.1.ffn_down.weight": gg.Q4_1, "blk.0.attn_k.weight": gg.Q8_K}
    raws = {}
    for i, (name, ty) in enumerate(swaps.items()):
        n = int(np.prod(t[name][0]))
        per = 32 if ty == 3 else 256
        raws[name] = random_blocks(ty, n // per, 70 + i)
        t[name] = (t[name][0], ty, raws[name])
    meta = [("general.architecture", gg.STRING, "llama"), ("llama.embedding_length", gg.U32, H), ("llama.block_count", gg.U32, cfg["layers"]),
            ("llama.attention.head_count", gg.U32, cfg["heads"]), ("llama.attention.head_count_kv", gg.U32, cfg["kv_heads"]),
            ("llama.feed_forward_length", gg.U32, cfg["inter"]), ("llama.vocab_size", gg.U32, V), ("llama.context_length", gg.U32, 640),
            ("llama.attention.layer_norm_rms_epsilon", gg.FLOAT32, cfg["rms_eps"]), ("llama.rope.freq_base", gg.FLOAT32, cfg["rope_theta"])]
    data = gg.write_gguf(meta, [(n, d, g, b) for n, (d, g, b) in t.items()])
    f = gg.GgufFile(data)
    got = f.config()
    assert (got["wdtype"], got["lm_head_dtype"]) == (Q8, Q8)
    o = go.parse(data)
    assert go.config(o) == got
    out = f.export_weights(got)
    assert np.array_equal(out, go.export_weights(oracle, o, data, got))
    parts = gg.split_blob(got, out)
    for name, ty in swaps.items():
        n = int(np.prod(t[name][0]))
        q8 = oracle.quantize_weights(Q8, gg.dequant_ggml(ty, raws[name], n))
        if name == "token_embd.weight":
            assert np.array_equal(parts[name][2].view(np.float32), oracle.dequant(Q8, q8, n))
        else:
            assert np.array_equal(parts[name][2], q8), name


@pytest.mark.gpu
def test_model_from_gguf_equals_model_from_blob(fh, gg, torch_gpu, tmp_path):
    """forge_hip_model_create_from_gguf: same logits, same greedy tokens, same cache as the model built from the blob."""
    for wd in (Q8, Q4):
        cfg = fh.synth.tiny(wd, max_seq=640)
        blob = fh.synth.make_weights_blob(cfg, seed=14)
        path = str(tmp_path / f"m{wd}.gguf")
        gg.model_to_gguf(cfg, blob, tied=True, path=path)
        a, b = fh.HipModel(cfg, blob), fh.HipModel.from_gguf(path)
        assert b.config == {"sliding_window": 0, **cfg, "rms_eps": b.config["rms_eps"], "rope_theta": b.config["rope_theta"]}
        prompt = fh.synth.uniform_ids(5, 40, cfg["vocab"])
        la, lb = a.forward_prefill(prompt), b.forward_prefill(prompt)
        assert np.array_equal(la.view(np.uint32), lb.view(np.uint32))
        tok = fh.ops.argmax_host(la)
        for _ in range(6):
            ta, tb = a.forward_greedy(tok), b.forward_greedy(tok)
            assert ta == tb
            tok = ta
        assert np.array_equal(a.read_kv(1, 0), b.read_kv(1, 0))
        a.close(); b.close()
        # a Qwen2-style file (QKV bias): same check
        cfgb = dict(cfg, flags=fh.FLAG_QKV_BIAS)
        blobb = fh.synth.make_weights_blob(cfgb, seed=16)
        pathb = str(tmp_path / f"b{wd}.gguf")
        gg.model_to_gguf(cfgb, blobb, tied=True, path=pathb)
        a, b = fh.HipModel(cfgb, blobb), fh.HipModel.from_gguf(pathb)
        assert b.config["flags"] == fh.FLAG_QKV_BIAS
        assert np.array_equal(a.forward_prefill(prompt).view(np.uint32), b.forward_prefill(prompt).view(np.uint32))
        a.close(); b.close()
        # a smaller cache than the file's context length, and the exact mode
        c = fh.HipModel.from_gguf(path, max_seq=600, flags=fh.FLAG_EXACT)
        assert c.config["max_seq"] == 600 and c.config["flags"] == fh.FLAG_EXACT
        c.forward_prefill(prompt)
        c.close()


@pytest.mark.gpu
def test_phi3_model_from_fused_gguf(fh, gg, oracle, torch_gpu, tmp_path):
    """A Phi-3-style file (fused tensors, head_dim 96, no GQA) read by forge_hip_model_create_from_gguf: same logits and greedy
    tokens as the model built from the blob, and the exact mode agrees with the CPU oracle bit for bit."""
    cfg = fh.synth.tiny(Q8, max_seq=640, hidden=384, inter=768, heads=4, kv_heads=4, head_dim=96)
    blob = fh.synth.make_weights_blob(cfg, seed=23)
    path = str(tmp_path / "phi3.gguf")
    gg.model_to_gguf(cfg, blob, tied=True, fused=True, path=path)
    a, b = fh.HipModel(cfg, blob), fh.HipModel.from_gguf(path)
    prompt = fh.synth.uniform_ids(6, 50, cfg["vocab"])
    la, lb = a.forward_prefill(prompt), b.forward_prefill(prompt)
    assert np.array_equal(la.view(np.uint32), lb.view(np.uint32))
    tok = fh.ops.argmax_host(la)
    for _ in range(6):
        ta, tb = a.forward_greedy(tok), b.forward_greedy(tok)
        assert ta == tb
        tok = ta
    a.close(); b.close()
    e = fh.HipModel.from_gguf(path, flags=fh.FLAG_EXACT)
    om = oracle.Model(dict(cfg, flags=fh.FLAG_EXACT), blob, 0, 1)
    assert np.array_equal(e.forward_prefill(prompt).view(np.uint32), om.prefill_batched(prompt).view(np.uint32))
    e.close(); om.close()


# ---------------------------------------------------------------- a storage format per projection category
def _xorshift(state):
    def nxt():
        s = nxt.s
        s ^= (s << 13) & 0xFFFFFFFF
        s ^= s >> 17
        s ^= (s << 5) & 0xFFFFFFFF
        nxt.s = s
        return s
    nxt.s = state
    return nxt


def _gauss_like_the_reference_tests(seed, n):
    """Box-Muller over a 32-bit xorshift, sigma 0.05 (the inputs of weight_loader.rs:2783-2840, 2924-2966; numpy's cos / ln need
    not round like Rust's: the bounds below hold for the distribution, not for particular bits)."""
    nxt = _xorshift(seed)
    out = []
    while len(out) < n:
        u1 = max(nxt() / 0xFFFFFFFF, 1e-7)
        u2 = nxt() / 0xFFFFFFFF
        r = np.sqrt(-2.0 * np.log(u1))
        out += [0.05 * r * np.cos(2 * np.pi * u2), 0.05 * r * np.sin(2 * np.pi * u2)]
    return np.asarray(out[:n], np.float32)


KQ_INPUTS = {
    "gauss": lambda: np.random.default_rng(1).normal(0, 0.05, 256 * 24).astype(np.float32),
    "heavy_tail": lambda: (np.random.default_rng(2).standard_t(3, 256 * 16) * 0.02).astype(np.float32),
    "ramp": lambda: ((np.arange(512) - 256.0) * 0.005).astype(np.float32),
    "zeros": lambda: np.zeros(512, np.float32),
    "flat_and_positive": lambda: np.concatenate([np.full(256, 0.25, np.float32), np.abs(np.random.default_rng(3).normal(0, 1, 256)).astype(np.float32),
                                                 np.full(128, -1.5, np.float32), np.zeros(128, np.float32)]),
    "ragged_tail": lambda: np.random.default_rng(4).normal(0, 1, 300).astype(np.float32),
    "one_outlier": lambda: np.concatenate([np.random.default_rng(5).normal(0, 0.01, 255).astype(np.float32), np.float32([3.0])]),
    "ties": lambda: np.tile(np.float32([-32, -31.5, -0.5, 0.5, 1.5, 2.5, 30.5, 31, 0, 0, 0, 0, 0, 0, 0, 0]), 16),
}


@pytest.mark.parametrize("ty", [12, 14])
@pytest.mark.parametrize("name", list(KQ_INPUTS))
def test_kquant_quantisers_library_equals_restatement(fh, gg, go, oracle, ty, name):
    """The library's quantize_f32_to_q4_k / _q6_k (C++ loops) against the array-form restatement, byte for byte, and what the
    format itself fixes: every code is the NEAREST one under the scales as stored (the refit step, weight_loader.rs:1826-1850,
    2085-2100), checked through the fixture-pinned dequantisers."""
    x = KQ_INPUTS[name]()
    got = gg.quantize_kquant(ty, x)
    want = (go.quantize_q4_k if ty == 12 else go.quantize_q6_k)(oracle, x)
    assert got.size == (x.size + 255) // 256 * (144 if ty == 12 else 210)
    assert np.array_equal(got, want)
    n = (x.size + 255) // 256 * 256
    xp = np.zeros(n, np.float32)
    xp[:x.size] = x
    back = gg.dequant_ggml(ty, got, n).astype(np.float64)
    if ty == 14:
        b = got.reshape(-1, 210)
        d = oracle.f16_to_f32(b[:, 208:210].copy().view("<u2")[:, 0]).astype(np.float64)
        step = np.abs(d[:, None] * b[:, 192:208].view(np.int8).astype(np.float64))           # [block][16 sub-blocks]
        step = np.repeat(step, 16, axis=1).reshape(-1)
        inside = (np.abs(xp) <= 31 * step)                       # codes -32 .. 31: beyond 31 steps a positive value is clamped
        assert np.all(np.abs(back - xp)[inside] <= 0.5 * step[inside] * (1 + 1e-5) + 1e-12)
    else:
        b = got.reshape(-1, 144)
        d = oracle.f16_to_f32(b[:, 0:2].copy().view("<u2")[:, 0]).astype(np.float64)
        dmin = oracle.f16_to_f32(b[:, 2:4].copy().view("<u2")[:, 0]).astype(np.float64)
        sc, mn = go._scale_min_k4(b[:, 4:16])                                                  # [block][8 sub-blocks]
        step = np.repeat(d[:, None] * sc, 32, axis=1).reshape(-1)
        low = -np.repeat(dmin[:, None] * mn, 32, axis=1).reshape(-1)                           # the value of code 0
        inside = (xp >= low) & (xp <= low + 15 * step)
        assert np.all(np.abs(back - xp)[inside] <= 0.5 * step[inside] * (1 + 1e-5) + 1e-12)
        assert inside.mean() > 0.9 or name not in ("gauss", "heavy_tail", "ramp")      # the check must bite where it can


def test_kquant_quantisers_meet_the_reference_tests_bounds(fh, gg, oracle):
    """The reference's own unit tests for the two quantisers (weight_loader.rs:2735-2990), on their inputs."""
    ramp = ((np.arange(512) - 256.0) * 0.005).astype(np.float32)
    q = gg.quantize_kquant(12, ramp)
    assert q.size == 2 * 144 and np.abs(gg.dequant_ggml(12, q, 512) - ramp).max() < 0.05                     # :2735-2755
    q = gg.quantize_kquant(14, ramp)
    assert q.size == 2 * 210 and np.abs(gg.dequant_ggml(14, q, 512) - ramp).max() < 0.02                     # :2906-2921
    state, vals = 0xDEADBEEF, []
    for _ in range(512):                                                                                      # :2758-2780
        state = (state * 1664525 + 1013904223) & 0xFFFFFFFF
        vals.append((np.float32(state >> 16) / np.float32(65535) - np.float32(0.5)) * np.float32(0.2))
    v = np.asarray(vals, np.float32)
    e = gg.dequant_ggml(12, gg.quantize_kquant(12, v), 512).astype(np.float64) - v
    assert np.sqrt(np.mean(e * e)) < 0.005
    for ty, seed in ((12, 0x13579BDF), (14, 0xFEEDBABE)):                                                     # :2783-2840, :2924-2966
        v = _gauss_like_the_reference_tests(seed, 4096)
        e = gg.dequant_ggml(ty, gg.quantize_kquant(ty, v), 4096).astype(np.float64) - v
        assert abs(e.mean()) < 5 * np.sqrt(np.mean(e * e)) / np.sqrt(4096)
    nxt = _xorshift(0xACEDF00D)                                                                               # :2844-2892
    vals = []
    for i in range(8192):
        u1 = max(nxt() / 0xFFFFFFFF * 0.99, 1e-6)
        u2 = max(nxt() / 0xFFFFFFFF, 1e-6)
        z = np.sqrt(-2 * np.log(u1)) * np.cos(2 * np.pi * u2)
        vals.append(0.3 * np.sign(z) if i % 200 == 0 else 0.05 * z)
    v = np.asarray(vals, np.float32)
    e = gg.dequant_ggml(12, gg.quantize_kquant(12, v), 8192).astype(np.float64) - v
    assert abs(e.mean()) < 5 * np.sqrt(np.mean(e * e)) / np.sqrt(8192)
    for ty in (12, 14):                                                                                       # :2895-2903, :2969-2976
        assert np.abs(gg.dequant_ggml(ty, gg.quantize_kquant(ty, np.zeros(256, np.float32)), 256)).max() < 1e-3
    with pytest.raises(fh.ForgeHipError):
        gg.quantize_kquant(13, np.zeros(256, np.float32))


def _kquant_file(fh, gg, recipe, seed=31, layers=4, tied=False, embed_ty=12, lm_ty=14, extra=None, arch="llama"):
    """A llama-architecture GGUF file of a small random model whose tensors are stored by `recipe(layer, suffix) -> type id`
    (12 = Q4_K, 14 = Q6_K, 8, 2); returns (bytes, {name: (type, raw bytes)}, shape dict)."""
    shape = dict(hidden=256, inter=512, layers=layers, heads=4, kv_heads=2, head_dim=64, vocab=512)
    H, I, V = shape["hidden"], shape["inter"], shape["vocab"]
    QKS, KV = 256, 128
    rng = np.random.default_rng(seed)

    def store(ty, n_rows, k):
        w = rng.normal(0, 0.05, n_rows * k).astype(np.float32)
        if ty in (12, 14):
            return gg.quantize_kquant(ty, w)
        if ty == 13:
            return random_blocks(13, n_rows * k // 256, int(rng.integers(1 << 30)))
        return fh.ops.quantize_weights(ty, w)

    t = {"token_embd.weight": ([H, V], embed_ty, store(embed_ty, V, H))}
    for l in range(layers):
        t[f"blk.{l}.attn_norm.weight"] = ([H], gg.F32, (1 + 0.1 * rng.normal(0, 1, H)).astype(np.float32).view(np.uint8))
        t[f"blk.{l}.ffn_norm.weight"] = ([H], gg.F32, (1 + 0.1 * rng.normal(0, 1, H)).astype(np.float32).view(np.uint8))
        for suffix, n_rows, k in (("attn_q", QKS, H), ("attn_k", KV, H), ("attn_v", KV, H), ("attn_output", H, QKS), ("ffn_gate", I, H),
                                  ("ffn_up", I, H), ("ffn_down", H, I)):
            ty = recipe(l, suffix)
            t[f"blk.{l}.{suffix}.weight"] = ([k, n_rows], ty, store(ty, n_rows, k))
        if arch == "qwen2":                                   # the bias vectors go with the architecture (main.rs:770)
            for suffix, n in (("attn_q", QKS), ("attn_k", KV), ("attn_v", KV)):
                t[f"blk.{l}.{suffix}.bias"] = ([n], gg.F32, rng.normal(0, 0.5, n).astype(np.float32).view(np.uint8))
    t["output_norm.weight"] = ([H], gg.F32, (1 + 0.1 * rng.normal(0, 1, H)).astype(np.float32).view(np.uint8))
    if not tied:
        t["output.weight"] = ([H, V], lm_ty, store(lm_ty, V, H))
    meta = [("general.architecture", gg.STRING, arch), (arch + ".embedding_length", gg.U32, H), (arch + ".block_count", gg.U32, layers),
            (arch + ".attention.head_count", gg.U32, 4), (arch + ".attention.head_count_kv", gg.U32, 2), (arch + ".feed_forward_length", gg.U32, I),
            (arch + ".vocab_size", gg.U32, V), (arch + ".context_length", gg.U32, 640), (arch + ".attention.layer_norm_rms_epsilon", gg.FLOAT32, 1e-5),
            (arch + ".rope.freq_base", gg.FLOAT32, 10000.0)] + list(extra or [])
    data = gg.write_gguf(meta, [(n, d, g, b) for n, (d, g, b) in t.items()])
    return data, {n: (g, np.ascontiguousarray(b, np.uint8).reshape(-1)) for n, (d, g, b) in t.items()}, shape


def _q4_k_m(l, suffix):
    """llama.cpp's Q4_K_M over four layers: attn_v and ffn_down are Q6_K in half of the layers, everything else Q4_K."""
    return 14 if suffix in ("attn_v", "ffn_down") and l in (0, 3) else 12


def test_q4_k_m_file_keeps_a_format_per_category(fh, gg, go, oracle):
    data, raw, shape = _kquant_file(fh, gg, _q4_k_m)
    f, o = gg.GgufFile(data), go.parse(data)
    with pytest.raises(fh.ForgeHipError):
        f.config()                                                     # no Q8_0 / Q4_0 majority: the uniform rules do not apply
    cfg, pd, embed = f.config_mixed()
    # v and down: two Q4_K against two Q6_K tensors, the tie goes to the more precise format (main.rs:626-640)
    assert pd == [12, 12, 14, 12, 12, 12, 14] and cfg["lm_head_dtype"] == 14 and embed == 12
    assert (cfg, pd, embed) == go.config_mixed(o)
    assert {k: cfg[k] for k in shape} == shape
    blob = f.export_weights_mixed(cfg, pd)
    assert np.array_equal(blob, go.export_weights_mixed(oracle, o, data, cfg, pd))
    H, V = 256, 512
    # the f32 table is the Q4_K table dequantised directly; tensors already in their category's format are the file's bytes
    assert np.array_equal(blob[:V * H * 4].view(np.float32), gg.dequant_ggml(12, raw["token_embd.weight"][1], V * H))
    at = V * H * 4 + H * 4
    assert np.array_equal(blob[at:at + raw["blk.0.attn_q.weight"][1].size], raw["blk.0.attn_q.weight"][1])
    assert np.array_equal(blob[-raw["output.weight"][1].size:], raw["output.weight"][1])
    # layer 1's attn_v is Q4_K in a Q6_K category: dequantised and quantised again (weight_loader.rs:208-218)
    per_layer = (blob.size - V * H * 4 - H * 4 - raw["output.weight"][1].size) // 4
    v_at = V * H * 4 + per_layer + H * 4 + 256 * 144 + 128 * 144
    want = gg.quantize_kquant(14, gg.dequant_ggml(12, raw["blk.1.attn_v.weight"][1], 128 * 256))
    assert np.array_equal(blob[v_at:v_at + want.size], want)


def test_category_rules_on_other_files(fh, gg, go, oracle):
    # a Q4_0 file whose output matrix is Q6_K (llama.cpp's default): Q4_0 projections under a Q6_K lm_head
    data, raw, _ = _kquant_file(fh, gg, lambda l, s: 2, embed_ty=2, lm_ty=14, layers=2)
    f, o = gg.GgufFile(data), go.parse(data)
    cfg, pd, embed = f.config_mixed()
    assert pd == [2] * 7 and (cfg["wdtype"], cfg["lm_head_dtype"], embed) == (2, 14, 2) and (cfg, pd, embed) == go.config_mixed(o)
    assert np.array_equal(f.export_weights_mixed(cfg, pd), go.export_weights_mixed(oracle, o, data, cfg, pd))
    # tied embeddings stored as Q6_K: the lm_head takes the embedding's format and bytes (main.rs:668-678, 2632-2676)
    data, raw, _ = _kquant_file(fh, gg, lambda l, s: 12, embed_ty=14, tied=True, layers=2)
    f, o = gg.GgufFile(data), go.parse(data)
    cfg, pd, embed = f.config_mixed()
    assert pd == [12] * 7 and (cfg["lm_head_dtype"], embed) == (14, 14) and (cfg, pd, embed) == go.config_mixed(o)
    blob = f.export_weights_mixed(cfg, pd)
    assert np.array_equal(blob, go.export_weights_mixed(oracle, o, data, cfg, pd))
    assert np.array_equal(blob[-raw["token_embd.weight"][1].size:], raw["token_embd.weight"][1])
    # a category whose tensors are all Q5_K has no vote and takes the file's majority format; its tensors are converted
    data, raw, _ = _kquant_file(fh, gg, lambda l, s: 13 if s == "ffn_up" else 12, layers=2)
    f, o = gg.GgufFile(data), go.parse(data)
    cfg, pd, embed = f.config_mixed()
    assert pd == [12] * 7 and (cfg, pd, embed) == go.config_mixed(o)
    blob = f.export_weights_mixed(cfg, pd)
    assert np.array_equal(blob, go.export_weights_mixed(oracle, o, data, cfg, pd))
    # a uniform Q8_0 file reports seven times Q8_0: forge_hip_model_create_from_gguf then takes the uniform rules
    cfg8 = fh.synth.tiny(Q8, max_seq=640)
    data = gg.model_to_gguf(cfg8, fh.synth.make_weights_blob(cfg8, seed=2), tied=True)
    cfg, pd, embed = gg.GgufFile(data).config_mixed()
    assert pd == [8] * 7 and cfg["lm_head_dtype"] == 8 and embed == 8
    # refusals: wrong buffer size, an unknown format
    f = gg.GgufFile(_kquant_file(fh, gg, _q4_k_m)[0])
    cfg, pd, _ = f.config_mixed()
    with pytest.raises(fh.ForgeHipError):
        f.export_weights_mixed(cfg, [13] + pd[1:])


def test_qwen2_q4_k_m_file_carries_its_bias_vectors(fh, gg, go, oracle):
    """A Qwen2 file in the Q4_K_M recipe: the bias flag comes with the architecture (main.rs:770) and the export writes
    q | k | v bias after the v weights of every layer (main.rs:2737-2742), whatever the weight formats."""
    data, raw, shape = _kquant_file(fh, gg, _q4_k_m, arch="qwen2", layers=2)
    f, o = gg.GgufFile(data), go.parse(data)
    cfg, pd, embed = f.config_mixed()
    assert cfg["flags"] & 2 and pd == [12, 12, 14, 12, 12, 12, 14] and (cfg, pd, embed) == go.config_mixed(o)
    blob = f.export_weights_mixed(cfg, pd)
    assert np.array_equal(blob, go.export_weights_mixed(oracle, o, data, cfg, pd))
    H, V = 256, 512
    at = V * H * 4 + H * 4 + 256 * 144 + 128 * 144 + 128 * 210          # embedding, layer 0: norm, q, k (Q4_K), v (Q6_K)
    want = np.concatenate([raw[f"blk.0.attn_{n}.bias"][1] for n in ("q", "k", "v")])
    assert np.array_equal(blob[at:at + want.size], want)


def test_mistral_q4_k_m_file_keeps_its_window(fh, gg, go, oracle):
    data, _, _ = _kquant_file(fh, gg, _q4_k_m, arch="mistral", layers=2, extra=[("mistral.attention.sliding_window", gg.U32, 32)])
    f, o = gg.GgufFile(data), go.parse(data)
    cfg, pd, embed = f.config_mixed()
    assert cfg["sliding_window"] == 32 and not cfg["flags"] & 2 and (cfg, pd, embed) == go.config_mixed(o)
    assert np.array_equal(f.export_weights_mixed(cfg, pd), go.export_weights_mixed(oracle, o, data, cfg, pd))


@pytest.mark.gpu
def test_mistral_q4_k_m_model_from_gguf_matches_the_oracle(fh, gg, go, oracle, torch_gpu, tmp_path):
    data, _, _ = _kquant_file(fh, gg, _q4_k_m, arch="mistral", layers=2, extra=[("mistral.attention.sliding_window", gg.U32, 16)])
    path = str(tmp_path / "mistral_q4km.gguf")
    with open(path, "wb") as fp:
        fp.write(data)
    o = go.parse(data)
    cfg, pd, _ = go.config_mixed(o, flags=fh.FLAG_EXACT)
    blob = go.export_weights_mixed(oracle, o, data, cfg, pd)
    gm = fh.HipModel.from_gguf(path, flags=fh.FLAG_EXACT)
    assert gm.config["sliding_window"] == 16
    om = oracle.Model(cfg, blob, 0, 1, proj_dtypes=pd)
    prompt = fh.synth.uniform_ids(10, 40, cfg["vocab"])
    gl, ol = gm.forward_prefill(prompt), om.prefill_batched(prompt)
    assert np.array_equal(gl.view(np.uint32), ol.view(np.uint32))
    tok = oracle.argmax(ol)
    for _ in range(8):
        g, w = gm.forward(tok), om.forward(tok)
        assert np.array_equal(g.view(np.uint32), w.view(np.uint32))
        tok = oracle.argmax(w)
    gm.close()


@pytest.mark.gpu
def test_qwen2_q4_k_m_model_from_gguf_matches_the_oracle(fh, gg, go, oracle, torch_gpu, tmp_path):
    data, _, _ = _kquant_file(fh, gg, _q4_k_m, arch="qwen2", layers=2)
    path = str(tmp_path / "qwen2_q4km.gguf")
    with open(path, "wb") as fp:
        fp.write(data)
    o = go.parse(data)
    cfg, pd, _ = go.config_mixed(o, flags=fh.FLAG_EXACT)
    blob = go.export_weights_mixed(oracle, o, data, cfg, pd)
    gm = fh.HipModel.from_gguf(path, flags=fh.FLAG_EXACT)
    assert gm.proj_dtypes == pd and gm.config["flags"] & 2
    om = oracle.Model(cfg, blob, 0, 1, proj_dtypes=pd)
    prompt = fh.synth.uniform_ids(9, 21, cfg["vocab"])
    gl, ol = gm.forward_prefill(prompt), om.prefill_batched(prompt)
    assert np.array_equal(gl.view(np.uint32), ol.view(np.uint32))
    tok = oracle.argmax(ol)
    for _ in range(8):
        g, w = gm.forward(tok), om.forward(tok)
        assert np.array_equal(g.view(np.uint32), w.view(np.uint32))
        tok = oracle.argmax(w)
    gm.close()


@pytest.mark.gpu
def test_q4_k_m_model_from_gguf_matches_the_oracle(fh, gg, go, oracle, torch_gpu, tmp_path):
    """forge_hip_model_create_from_gguf on a Q4_K_M-style file, order-faithful mode: prompt logits, cache rows and 12 greedy
    steps bit for bit those of the CPU oracle run on the oracle's own export of the same file."""
    data, _, _ = _kquant_file(fh, gg, _q4_k_m)
    path = str(tmp_path / "q4km.gguf")
    with open(path, "wb") as fp:
        fp.write(data)
    o = go.parse(data)
    cfg, pd, _ = go.config_mixed(o, flags=fh.FLAG_EXACT)
    blob = go.export_weights_mixed(oracle, o, data, cfg, pd)
    gm = fh.HipModel.from_gguf(path, flags=fh.FLAG_EXACT)
    assert gm.proj_dtypes == pd and gm.config["lm_head_dtype"] == 14 and gm.decode_launches == 1     # all K-quant: the resident kernel
    om = oracle.Model(cfg, blob, 0, 1, proj_dtypes=pd)
    prompt = fh.synth.uniform_ids(8, 24, cfg["vocab"])
    gl, ol = gm.forward_prefill(prompt), om.prefill_batched(prompt)
    assert np.array_equal(gl.view(np.uint32), ol.view(np.uint32))
    tok = oracle.argmax(ol)
    for _ in range(12):
        g, w = gm.forward(tok), om.forward(tok)
        assert np.array_equal(g.view(np.uint32), w.view(np.uint32))
        tok = oracle.argmax(w)
    assert np.array_equal(oracle.f16_to_f32(gm.read_kv(3, 1)), om.read_kv(3, 1))
    gm.close()
    # the same file in fast mode: one resident kernel per decode step, the model built from the oracle's export of the file
    # gives the same bits (same kernels on the same planes), and the logits stay near the order-faithful ones
    fm = fh.HipModel.from_gguf(path)
    assert fm.decode_launches == 1
    fcfg = dict(cfg, flags=0)
    bm = fh.HipModel(fcfg, blob, proj_dtypes=pd)
    fl = fm.forward_prefill(prompt)
    assert np.array_equal(fl, bm.forward_prefill(prompt))
    assert np.corrcoef(fl, ol)[0, 1] > 0.995
    t = int(np.argmax(fl))
    for _ in range(6):
        a, b = fm.forward(t), bm.forward(t)
        assert np.array_equal(a, b)
        t = int(np.argmax(a))
    fm.close(); bm.close()
