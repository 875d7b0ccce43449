"""CPU-side checks of the product: the C-ABI library loads and exports every symbol the header
declares, its host format code is bit-identical to the oracle, the synthetic generators are
deterministic, and argument errors come back as codes (no compute calls: there is no GPU here)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

Q8, Q4 = 8, 2
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(fh):
    header = open(os.path.join(ROOT, "include", "forge_hip.h")).read()
    declared = sorted(set(re.findall(r"\b(forge_hip_[a-z0-9_]+)\s*\(", header)))
    assert declared, "no declarations found in include/forge_hip.h"
    L = fh.lib()
    missing = [s for s in declared if not hasattr(L, s)]
    assert not missing, f"declared but not exported: {missing}"
    assert sorted(fh.EXPORTS) == declared


def test_host_f16_matches_oracle_exhaustively(fh, oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = oracle.f16_to_f32(bits)
    got = np.array([fh.ops.f16_to_f32(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
                        np.array([2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25, 1e-45, 65520.0, np.inf, -np.inf, 0.0, -0.0], np.float32)])
    want = oracle.f32_to_f16(x)
    got = np.array([fh.ops.f32_to_f16(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("wd", [Q8, Q4])
def test_host_quantisers_bit_identical_to_oracle(fh, oracle, wd):
    rng = np.random.default_rng(7)
    v = (rng.standard_normal(32 * 5000 + 17) * 0.02).astype(np.float32)     # ragged tail block
    v[320:352] = 0.0
    assert np.array_equal(fh.ops.quantize_weights(wd, v), oracle.quantize_weights(wd, v))
    raw = oracle.quantize_weights(wd, v)
    assert np.array_equal(fh.ops.dequant(wd, raw, v.size), oracle.dequant(wd, raw, v.size))
    assert fh.ops.quantize_weights(wd, np.zeros(0, np.float32)).size == 0


def test_host_quantisers_rounding_ties(fh):
    """Elements exactly half way between two codes (scale 1.0 exactly: largest magnitude 127 resp. 8) go AWAY from zero,
    as f32::round does (weight_loader.rs:1482, 1534-1535); expected codes written by hand."""
    v = np.zeros(32, np.float32)
    v[:12] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5, -126.5, 127.0, 0.25, -0.75, 3.0]
    raw = fh.ops.quantize_weights(Q8, v)
    assert (int(raw[0]) | (int(raw[1]) << 8)) == 0x3C00
    assert raw[2:14].view(np.int8).tolist() == [1, -1, 2, -2, 3, -3, 127, -127, 127, 0, -1, 3]
    v[:12] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 6.5, -7.5, 8.0, -8.0, 7.5, 0.25]
    raw = fh.ops.quantize_weights(Q4, v)
    assert (int(raw[0]) | (int(raw[1]) << 8)) == 0x3C00
    codes = np.concatenate([raw[2:] & 0x0F, raw[2:] >> 4])
    assert codes[:12].tolist() == [9, 7, 10, 6, 11, 5, 15, 0, 15, 0, 15, 8]


def test_expf_twin_matches_c_library(fh, oracle):
    """The kernels' exp (host twin) against the C library's expf, which the CPU path calls: dense
    sweep of the softmax/silu range plus the overflow/underflow edges.  (Over all 2.2e9 finite inputs
    with |x| <= 110 the two differ in two values, by one ulp.)"""
    rng = np.random.default_rng(3)
    x = np.concatenate([
        rng.uniform(-104.5, 89.5, 3_000_000).astype(np.float32),
        -np.abs(rng.standard_normal(1_000_000).astype(np.float32)) * 8,          # softmax arguments
        np.array([0.0, -0.0, 88.72, 88.73, -103.9, -104.0, -87.4, np.inf, -np.inf, 1e-10, -1e-10], np.float32),
    ])
    got, want = fh.ops.expf_host(x), oracle.expf(x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.isnan(fh.ops.expf_host(np.array([np.nan], np.float32))[0])


def test_argmax_host_last_maximum(fh):
    assert fh.ops.argmax_host(np.array([1, 5, 3, 5, 2], np.float32)) == 3
    assert fh.ops.argmax_host(np.array([7, 7, 7], np.float32)) == 2


def test_synth_is_deterministic_and_normal(fh):
    a = fh.synth.normal(42, 100001, 0.02)
    b = fh.synth.normal(42, 100001, 0.02)
    assert np.array_equal(a, b) and a.dtype == np.float32
    assert abs(float(a.mean())) < 3e-4 and float(a.std()) == pytest.approx(0.02, rel=0.02)
    # counter based: a later window equals the same window of a longer draw
    big = fh.synth.normal(42, (1 << 23) + 10, 1.0)
    assert np.array_equal(big[:1000], fh.synth.normal(42, 1000, 1.0))
    assert not np.array_equal(fh.synth.normal(43, 1000), fh.synth.normal(42, 1000))
    ids = fh.synth.uniform_ids(1, 5000, 49152)
    assert ids.max() < 49152 and len(set(ids.tolist())) > 4000
    # splitmix64 known answer for seed 0: first output
    assert int(fh.synth.splitmix64(0, 0, 1)[0]) == 0xE220A8397B1DCDAF


def test_weight_stream_bytes_match_published_figures(fh):
    """Algorithmic bytes per decode token (N*(K/32)*B + 4K + 4N per matmul)."""
    assert fh.synth.decode_weight_bytes(fh.synth.llama32_1b(Q8)) == 1312980992
    assert fh.synth.decode_weight_bytes(fh.synth.llama32_1b(Q4)) == 695107584
    assert fh.synth.decode_weight_bytes(fh.synth.smollm2_135m(Q8)) == 142884864
    assert fh.synth.decode_weight_bytes(fh.synth.llama32_3b(Q8)) == 3413360640


def test_blob_size_contract(fh, oracle):
    from forge_llm_amd.hip_model import weights_nbytes
    for cfg in (fh.synth.tiny(Q8), fh.synth.tiny(Q4), fh.synth.smollm2_135m(Q8), fh.synth.llama32_1b(Q8), fh.synth.llama32_3b(Q4)):
        assert weights_nbytes(cfg) == oracle.weights_nbytes(cfg)
    cfg = fh.synth.tiny(Q8)
    blob = fh.synth.make_weights_blob(cfg, seed=1)
    assert blob.size == weights_nbytes(cfg)
    # tied embeddings: the f32 table is the dequantised lm_head
    H, V = cfg["hidden"], cfg["vocab"]
    table = blob[:V * H * 4].view(np.float32)
    lm_raw = blob[-(V * H // 32 * 34):]
    assert np.array_equal(table, oracle.dequant(Q8, lm_raw, V * H))


def test_blob_size_contract_with_a_format_per_projection(fh, oracle):
    """project.rs:195-213 sizes every projection by its own format: 34 / 18 bytes per 32 weights, 144 / 210 per 256."""
    from forge_llm_amd.hip_model import weights_nbytes, weights_nbytes_mixed
    cfg = fh.synth.tiny(wdtype=Q8, max_seq=640, hidden=256, inter=512, layers=2, heads=4, kv_heads=2, head_dim=64, vocab=301)
    for pd, lm in (((12, 12, 14, 12, 12, 12, 14), 14), ((8, 2, 12, 8, 14, 2, 12), 8), ((2,) * 7, 2)):
        c = dict(cfg, lm_head_dtype=lm)
        n = weights_nbytes_mixed(c, pd)
        assert n == oracle.weights_nbytes_mixed(c, pd)
        assert fh.synth.make_weights_blob_mixed(c, pd, seed=1).size == n
    assert weights_nbytes_mixed(dict(cfg, wdtype=Q4, lm_head_dtype=Q4), (2,) * 7) == weights_nbytes(dict(cfg, wdtype=Q4, lm_head_dtype=Q4))
    # Qwen2's bias vectors (project.rs:286-292) add (QKS + 2 KV) floats per layer whatever the formats
    cb = dict(cfg, lm_head_dtype=14, flags=2)
    pdm = (12, 12, 14, 12, 12, 12, 14)
    assert weights_nbytes_mixed(cb, pdm) == weights_nbytes_mixed(dict(cb, flags=0), pdm) + 2 * (256 + 2 * 128) * 4 == oracle.weights_nbytes_mixed(cb, pdm)
    assert fh.synth.make_weights_blob_mixed(cb, pdm, seed=1).size == weights_nbytes_mixed(cb, pdm)
    # by hand for one matrix mix: H = 256, I = 512, QKS = 256, KV = 128, 2 layers, vocab 301
    c = dict(cfg, lm_head_dtype=14)
    per_layer = 2 * 256 * 4 + 256 * 144 + 128 * 144 + 128 * 210 + 256 * 144 + 2 * 512 * 144 + 256 * 2 * 210
    assert weights_nbytes_mixed(c, (12, 12, 14, 12, 12, 12, 14)) == 301 * 256 * 4 + 2 * per_layer + 256 * 4 + 301 * 210


def test_errors_are_codes_not_crashes(fh):
    L = fh.lib()
    cfg = fh.synth.tiny(Q8)
    blob = fh.synth.make_weights_blob(cfg, seed=1)
    h = C.c_void_p()
    bad = dict(cfg, head_dim=48)
    c = fh.Config(**bad)
    assert L.forge_hip_model_create(C.byref(c), blob.ctypes.data_as(C.c_void_p), blob.size, C.byref(h)) == fh.ERR_INVALID
    assert b"head_dim" in L.forge_hip_last_error()
    c = fh.Config(**dict(cfg, wdtype=12))
    assert L.forge_hip_model_create(C.byref(c), blob.ctypes.data_as(C.c_void_p), blob.size, C.byref(h)) == fh.ERR_INVALID
    c = fh.Config(**cfg)
    rc = L.forge_hip_model_create(C.byref(c), blob.ctypes.data_as(C.c_void_p), blob.size - 1, C.byref(h))
    assert rc == fh.ERR_BLOB_SIZE and not h.value        # the reference panics on a short blob (project.rs:342-406)
    with pytest.raises(fh.ForgeHipError):
        fh.HipModel(cfg, blob[:-5])
    assert L.forge_hip_quantize_f32(99, None, 0, None) == fh.ERR_INVALID
    w = C.c_void_p()
    assert L.forge_hip_qweight_create(Q8, blob.ctypes.data_as(C.c_void_p), 48, 4, C.byref(w)) == fh.ERR_INVALID
    if fh.device_count() == 0:
        rc = L.forge_hip_model_create(C.byref(c), blob.ctypes.data_as(C.c_void_p), blob.size, C.byref(h))
        assert rc == fh.ERR_NO_DEVICE                     # metal:4212 `expect("no Metal device found")`


def test_header_is_plain_c_and_the_library_links_from_c(fh, tmp_path):
    """include/forge_hip.h compiles as strict C99, and a C program linked against the library calls its host-side
    entry points (no GPU involved): f16 conversion, the GGUF parser on a buffer in memory, the sampler."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "forge_hip.h"
int main(void) {
    /* GGUF v3 header with no metadata and no tensors */
    unsigned char g[24];
    unsigned int magic = 0x46554747u, version = 3u;
    unsigned long long zero = 0;
    forge_hip_gguf* f = 0;
    forge_hip_config cfg;
    float logits[4] = {0.1f, 2.0f, 2.0f, -1.0f};
    uint64_t state = 1;
    uint32_t tok = 99;
    memcpy(g, &magic, 4); memcpy(g + 4, &version, 4); memcpy(g + 8, &zero, 8); memcpy(g + 16, &zero, 8);
    if (forge_hip_f32_to_f16(1.0f) != 0x3C00 || forge_hip_f16_to_f32(0xC000) != -2.0f) return 1;
    if (forge_hip_gguf_parse(g, sizeof g, &f) != FORGE_HIP_OK) return 2;
    if (forge_hip_gguf_version(f) != 3 || forge_hip_gguf_tensor_count(f) != 0 || forge_hip_gguf_tensor_data_offset(f) != 32) return 3;
    if (forge_hip_gguf_config(f, 0, 0, &cfg) != FORGE_HIP_ERR_INVALID) return 4;      /* no architecture key */
    if (strstr(forge_hip_last_error(), "unsupported GGUF architecture") == 0) return 5;
    forge_hip_gguf_close(f);
    g[0] = 0;
    if (forge_hip_gguf_parse(g, sizeof g, &f) != FORGE_HIP_ERR_INVALID || f != 0) return 6;
    if (forge_hip_sample(logits, 4, 0.0f, 0, 0.9f, &state, &tok) != FORGE_HIP_OK || tok != 2 || state != 1) return 7;
    if (forge_hip_model_create(0, 0, 0, 0) == FORGE_HIP_OK) return 8;
    printf("ok\n");
    return 0;
}
''')
    exe = tmp_path / "abi"
    inc = os.path.join(ROOT, "include")
    libdir = os.path.dirname(fh.LIB_PATH)
    r = subprocess.run([gcc, "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", inc, str(src), "-o", str(exe),
                        "-L", libdir, "-lforge_hip", "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    env = dict(os.environ, LD_LIBRARY_PATH=libdir + ":/opt/rocm/lib:" + os.environ.get("LD_LIBRARY_PATH", ""))
    r = subprocess.run([str(exe)], capture_output=True, text=True, env=env, timeout=120)
    assert r.returncode == 0 and r.stdout.strip() == "ok", (r.returncode, r.stdout, r.stderr)


def _c_declarations(header_text):
    """{name: [parameter declarations]} of every function the header declares."""
    import re
    text = re.sub(r"/\*.*?\*/", " ", header_text, flags=re.S)
    text = re.sub(r"^\s*#.*$", " ", text, flags=re.M)
    out = {}
    for m in re.finditer(r"\b(forge_hip_\w+)\s*\(([^;{}]*?)\)\s*;", text, flags=re.S):
        params = m.group(2).strip()
        out[m.group(1)] = [] if params in ("", "void") else [p.strip() for p in params.split(",")]
    return out, text


def test_rust_binding_matches_the_header():
    """The crate text that the reference's maintainers would add (forgellm-codegen-hip) cannot be compiled here, so its
    `extern "C"` block and its `#[repr(C)]` config are held to include/forge_hip.h: every function it names is declared
    there with the same number of parameters, in the same order by name, pointer for pointer; the struct has the header's
    fields in the header's order; placeholders and braces are balanced."""
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    rust = open(os.path.join(root, "forge-llm_amd", "bindings", "forgellm-codegen-hip", "src", "lib.rs")).read()
    decls, ctext = _c_declarations(open(os.path.join(root, "include", "forge_hip.h")).read())
    block = re.search(r'extern "C" \{(.*?)\n\}', rust, flags=re.S).group(1)
    fns = re.findall(r"fn (forge_hip_\w+)\((.*?)\)(?: -> ([\w\s\*]+))?;", block)
    assert len(fns) >= 14
    ctype = {"u32": "uint32_t", "u64": "uint64_t", "i32": "int32_t", "i64": "int64_t", "f32": "float", "u8": "uint8_t", "c_char": "char",
             "ForgeHipConfig": "forge_hip_config", "ForgeHipModel": "forge_hip_model"}
    for name, params, _ret in fns:
        assert name in decls, name
        rparams = [p.strip() for p in params.split(",")] if params.strip() else []
        assert len(rparams) == len(decls[name]), (name, rparams, decls[name])
        for rp, cp in zip(rparams, decls[name]):
            rname, rtype = [x.strip() for x in rp.split(":")]
            assert re.search(r"\b" + re.escape(rname) + r"$", cp), (name, rp, cp)          # same parameter name
            assert rtype.count("*") == cp.count("*"), (name, rp, cp)                         # same level of indirection
            assert ("*const" in rtype) == ("const" in cp) or "*" not in rtype, (name, rp, cp)
            base = rtype.replace("*const", "").replace("*mut", "").strip()
            assert ctype[base] in cp, (name, rp, cp)
    # the struct: same fields, same order, same types
    cstruct = re.search(r"typedef struct forge_hip_config \{(.*?)\} forge_hip_config;", ctext, flags=re.S).group(1)
    cfields = []
    for ty, names in re.findall(r"(uint32_t|float)\s+([^;]+);", cstruct):
        cfields += [(n.strip(), ty) for n in names.split(",")]
    rstruct = re.search(r"pub struct ForgeHipConfig \{(.*?)\}", rust, flags=re.S).group(1)
    rfields = [(n, ctype[t]) for n, t in re.findall(r"pub (\w+): (\w+),", rstruct)]
    assert rfields == cfields
    # every template placeholder is replaced by a .replace() of the generator
    for ph in set(re.findall(r"@[A-Z_]+@", rust)):
        assert f'.replace("{ph}"' in rust, ph
    for text in re.findall(r'r#"(.*?)"#', rust, flags=re.S) + [re.sub(r'r#".*?"#', '""', rust, flags=re.S)]:
        code = re.sub(r'"(?:[^"\\\n]|\\.)*"', '""', text)           # string literals may hold a lone bracket
        assert code.count("{") == code.count("}") and code.count("(") == code.count(")"), text[:60]
