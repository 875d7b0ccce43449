"""GPU parity at the sizes the benchmark configurations name (Llama-3.2-1B projection shapes, 2.5k-token
batches, 3k-token attention, 8k-token caches, the Llama-3.2-3B layer shape), through the C ABI.

The oracle would need minutes for whole outputs at these sizes, so each test runs the GPU on the full
problem and compares the parts the oracle can do in seconds, using what the operations guarantee:
  * a GEMM row depends only on its own activation row, an attention row only on its own query and the keys
    up to its position: sampled rows are checked against the oracle run on exactly those rows;
  * the same rows computed alone on the GPU must equal the rows of the full launch bit for bit
    (tiling, batching and chunking may not change a result) -- in EXACT mode and for attention; the fast GEMM
    promises it within its tolerance only."""
import hashlib
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q8, Q4 = 8, 2
A, KV_F16 = 0, 1
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


_weights = {}


def weight(fh, wd, K, N):
    """Seeded N(0, 0.02) weights quantised with the reference's quantiser; cached per shape."""
    key = (wd, K, N)
    if key not in _weights:
        w = fh.synth.normal(1000 + K + 3 * N, N * K, 0.02).reshape(N, K)
        raw = fh.ops.quantize_weights(wd, w)
        _weights[key] = (raw, fh.ops.QWeight(wd, raw, K, N))
    return _weights[key]


def sample_rows(M, seed):
    """First and last rows, the rows either side of every 128-row tile edge that exists, and a few random ones."""
    rows = {0, M - 1}
    for edge in (127, 128, 255, 256, 1023, 1024, 2047, 2048):
        if edge < M:
            rows.add(edge)
    rng = np.random.default_rng(seed)
    rows.update(int(r) for r in rng.integers(0, M, 6))
    return sorted(rows)


# ---------------- isolated GEMV, M = 1 ----------------
@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("K,N", [(2048, 2048), (2048, 512), (2048, 8192), (8192, 2048), (2048, 128256)])
def test_gemv_llama_1b_shapes_bit_exact(fh, oracle, torch_gpu, wd, K, N):
    """matmul_vec at every projection shape of Llama-3.2-1B, the LM head included: identical bits."""
    torch = torch_gpu
    raw, w = weight(fh, wd, K, N)
    x = fh.synth.normal(21 + K + N, K, 1.0)
    y = fh.ops.matmul_vec_q(w, torch.from_numpy(x).cuda()).cpu().numpy()
    same_bits(y, oracle.matmul_vec(wd, 0, x, raw, K, N))


# ---------------- batched-prefill GEMM ----------------
@pytest.mark.parametrize("wd", [Q8, Q4])
@pytest.mark.parametrize("K,N", [(2048, 2048), (2048, 512), (2048, 8192), (8192, 2048)])
@pytest.mark.parametrize("M", [352, 902, 1603, 2502])
def test_gemm_llama_1b_shapes(fh, oracle, torch_gpu, wd, K, N, M):
    torch = torch_gpu
    raw, w = weight(fh, wd, K, N)
    x = fh.synth.normal(31 + M + K, M * K, 1.0).reshape(M, K)
    rows = sample_rows(M, M + K + N)
    xd = torch.from_numpy(x).cuda()
    want = oracle.matmul_mat(wd, 0, x[rows], raw, len(rows), K, N)
    exact = fh.ops.matmul_mat_q(w, xd, EXACT).cpu().numpy()
    fast = fh.ops.matmul_mat_q(w, xd, 0).cpu().numpy()
    same_bits(exact[rows], want)
    close(fast[rows], want)
    # every row of the fast result against the exact one (same block sums, different f32 evaluation)
    close(fast, exact)
    # the sampled rows as a batch of their own: same bits as inside the full batch
    xs = torch.from_numpy(np.ascontiguousarray(x[rows])).cuda()
    same_bits(fh.ops.matmul_mat_q(w, xs, EXACT).cpu().numpy(), exact[rows])
    # fast mode: a large batch may have its left-over tiles cut along K (another f32 order for the rows in them), so
    # only the tolerance holds between batches; within one batch size the result is reproducible
    close(fh.ops.matmul_mat_q(w, xs, 0).cpu().numpy(), fast[rows], rtol=1e-4, atol=1e-4)
    same_bits(fh.ops.matmul_mat_q(w, xd, 0).cpu().numpy(), fast)


# ---------------- attention over an fp16 cache ----------------
def kv_cache(fh, oracle, seq, kv_heads, hd, seed):
    k = fh.synth.normal(seed, seq * kv_heads * hd, 1.0)
    v = fh.synth.normal(seed + 1, seq * kv_heads * hd, 1.0)
    return (oracle.f32_to_f16(k).reshape(seq, kv_heads * hd), oracle.f32_to_f16(v).reshape(seq, kv_heads * hd))


def dev16(torch, a):
    return torch.from_numpy(a.view(np.int16)).cuda()


@pytest.mark.parametrize("heads,kv_heads,hd", [(32, 8, 64), (32, 32, 96)])
@pytest.mark.parametrize("seq", [801, 1501, 3001])
def test_attention_prefill_long_sequences(fh, oracle, torch_gpu, heads, kv_heads, hd, seq):
    """attention_flash_batch over the whole sequence; sampled rows against the oracle's batch kernel run for
    that single row at its position (row r of a batch sees keys 0..r)."""
    torch = torch_gpu
    k16, v16 = kv_cache(fh, oracle, seq, kv_heads, hd, seed=seq + hd)
    q = fh.synth.normal(40 + seq, seq * heads * hd, 1.0).reshape(seq, heads * hd)
    q16 = oracle.f16_to_f32(oracle.f32_to_f16(q))            # the MFMA kernel rounds q to fp16: give it such queries
    kd, vd = dev16(torch, k16), dev16(torch, v16)
    exact = fh.ops.attention_flash_batch(torch.from_numpy(q).cuda(), kd, vd, 0, heads, kv_heads, hd, EXACT).cpu().numpy()
    fast = fh.ops.attention_flash_batch(torch.from_numpy(q16).cuda(), kd, vd, 0, heads, kv_heads, hd, 0).cpu().numpy()
    for r in sample_rows(seq, seq + hd):
        same_bits(exact[r], oracle.attention("flash_batch", q[r], k16, v16, 1, heads, kv_heads, hd, base_pos=r))
        close(fast[r], oracle.attention("flash_batch", q16[r], k16, v16, 1, heads, kv_heads, hd, base_pos=r))
    # a second chunk appended to an existing cache (base_pos > 0) reproduces the rows of the one-shot call
    cut = seq // 2 + 3
    tail_e = fh.ops.attention_flash_batch(torch.from_numpy(np.ascontiguousarray(q[cut:])).cuda(), kd, vd, cut, heads, kv_heads,
                                          hd, EXACT).cpu().numpy()
    same_bits(tail_e, exact[cut:])
    tail_f = fh.ops.attention_flash_batch(torch.from_numpy(np.ascontiguousarray(q16[cut:])).cuda(), kd, vd, cut, heads,
                                          kv_heads, hd, 0).cpu().numpy()
    close(tail_f, fast[cut:])


@pytest.mark.parametrize("heads,kv_heads,hd", [(32, 8, 64), (32, 32, 96)])
@pytest.mark.parametrize("seq", [900, 2250, 8192])
def test_attention_decode_long_caches(fh, oracle, torch_gpu, heads, kv_heads, hd, seq):
    torch = torch_gpu
    k16, v16 = kv_cache(fh, oracle, seq, kv_heads, hd, seed=seq + 7 * hd)
    q = fh.synth.normal(50 + seq, heads * hd, 1.0)
    want = oracle.attention("flash", q, k16, v16, seq, heads, kv_heads, hd)
    qd, kd, vd = torch.from_numpy(q).cuda(), dev16(torch, k16), dev16(torch, v16)
    same_bits(fh.ops.attention_flash(qd, kd, vd, seq, heads, kv_heads, hd, EXACT).cpu().numpy(), want)
    close(fh.ops.attention_flash(qd, kd, vd, seq, heads, kv_heads, hd, 0).cpu().numpy(), want)


# ---------------- Llama-3.2-3B layer shape end to end ----------------
def test_llama_3b_shape_two_layers_identical_tokens(fh, oracle, torch_gpu):
    """Llama-3.2-3B shape (hidden 3072, 24 heads over 8 KV heads, head_dim 128, intermediate 8192, vocabulary
    128256), Q8_0, cut to 2 of its 28 layers and a 300-token prompt so that the CPU oracle finishes in seconds:
    batched prefill, then greedy decode -- identical token ids and bit-identical logits in exact mode."""
    cfg = fh.synth.llama32_3b(Q8, max_seq=1024)
    cfg["layers"] = 2
    cfg["flags"] = EXACT
    blob = fh.synth.make_weights_blob(cfg, seed=3, threads=16)
    prompt = fh.synth.uniform_ids(4, 300, cfg["vocab"])
    gm = fh.HipModel(cfg, blob)
    om = oracle.Model(cfg, blob, A, KV_F16)
    glog = gm.forward_prefill(prompt)
    olog = om.prefill_batched(prompt)
    same_bits(glog, olog)
    tok = oracle.argmax(olog)
    for _ in range(8):
        gl, ol = gm.forward(tok), om.forward(tok)
        same_bits(gl, ol)
        tok = oracle.argmax(ol)
    for which in (0, 1):
        same_bits(oracle.f16_to_f32(gm.read_kv(1, which)), om.read_kv(1, which))
    gm.close(); om.close()


# ---------------- Llama-3.2-3B shape at full size: 28 layers, 2500-token prompt, 128 greedy tokens ----------------
_FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "config5_llama32_3b_q8.json")
_full_3b = {}


def full_3b(fh):
    """The model and prompt of tests/golden/config5_llama32_3b_q8.json, regenerated from its seeds (once per session)."""
    if not _full_3b:
        with open(_FIXTURE) as f:
            fx = json.load(f)
        cfg = fh.synth.llama32_3b(Q8, max_seq=4096)
        assert {k: cfg[k] for k in cfg} == {k: fx["config"][k] for k in cfg}
        blob = fh.synth.make_weights_blob(cfg, seed=fx["weight_seed"], threads=16)
        prompt = fh.synth.uniform_ids(fx["prompt_seed"], fx["prompt_tokens"], cfg["vocab"])
        assert [int(t) for t in prompt[:8]] == fx["prompt_head"]
        _full_3b.update(fx=fx, cfg=cfg, blob=blob, prompt=prompt)
    return _full_3b["fx"], _full_3b["cfg"], _full_3b["blob"], _full_3b["prompt"]


def _sha(a):
    return hashlib.sha256(np.ascontiguousarray(a, np.float32).tobytes()).hexdigest()


@pytest.mark.timeout(900)
def test_llama_3b_full_size_exact_mode_holds_the_oracle_fixture(fh, torch_gpu):
    """The whole workload -- 28 layers, batched prefill of 2500 tokens, 128 greedy tokens -- in exact mode against what the
    CPU oracle produced for it (a quarter of an hour on 8 cores, run once by tests/golden/make_config5_fixture.py): identical
    token ids, and the prefill logits and the logits behind the last token identical in every bit (SHA-256 of the f32 words)."""
    fx, cfg, blob, prompt = full_3b(fh)
    gm = fh.HipModel(dict(cfg, flags=EXACT), blob)
    logits = gm.forward_prefill(prompt)
    assert [int(i) for i in np.argsort(logits)[-5:][::-1]] == fx["prefill_top5"]
    assert _sha(logits) == fx["prefill_logits_sha256"]
    tokens = [fh.ops.argmax_host(logits)]
    for _ in range(len(fx["tokens"]) - 1):
        logits = gm.forward(tokens[-1])
        tokens.append(fh.ops.argmax_host(logits))
    first_bad = next((i for i, (a, b) in enumerate(zip(tokens, fx["tokens"])) if a != b), None)
    assert first_bad is None, f"token {first_bad} differs: {tokens[first_bad]} against the oracle's {fx['tokens'][first_bad]}"
    assert _sha(logits) == fx["last_logits_sha256"]
    gm.close()


@pytest.mark.timeout(900)
def test_llama_3b_full_size_resident_kernel_equals_kernel_sequence(fh, torch_gpu, monkeypatch):
    """Fast mode at full depth and context: after the same 2500-token prefill, 128 greedy steps of the one-kernel decode step
    (summing in the reference order) and of the kernel sequence give the same tokens, the same logits and the same cache,
    bit for bit; and the default summation of the one-kernel step stays close to the sequence over a single step from
    identical state."""
    fx, cfg, blob, prompt = full_3b(fh)
    monkeypatch.setenv("FORGE_HIP_PERSIST", "0")
    seq = fh.HipModel(cfg, blob)
    monkeypatch.setenv("FORGE_HIP_PERSIST", "1")
    monkeypatch.setenv("FORGE_HIP_PD_ORDERED", "1")
    one = fh.HipModel(cfg, blob)
    monkeypatch.setenv("FORGE_HIP_PD_ORDERED", "0")
    fast = fh.HipModel(cfg, blob)
    assert one.decode_launches == 1 and fast.decode_launches == 1 and seq.decode_launches > 1
    la = seq.forward_prefill(prompt)
    same_bits(one.forward_prefill(prompt), la)
    fast.forward_prefill_batch(prompt)
    a = b = fh.ops.argmax_host(la)
    lf, ls = fast.forward(a), seq.forward(a)                                   # one step, identical state
    # 28 layers of int8 activation quantisers amplify the first rounding difference to the quantisation-noise level
    assert np.corrcoef(lf, ls)[0, 1] > 0.99 and np.max(np.abs(lf - ls)) < 0.5 * max(1.0, float(np.std(ls)))
    same_bits(one.forward(a), ls)
    a = b = fh.ops.argmax_host(ls)
    for step in range(126):
        a2, b2 = one.forward_greedy(a), seq.forward_greedy(b)
        assert a2 == b2, f"step {step}: {a2} against {b2}"
        a, b = a2, b2
    same_bits(one.forward(a), seq.forward(b))
    for layer in (0, 13, 27):
        assert np.array_equal(one.read_kv(layer, 0), seq.read_kv(layer, 0))
        assert np.array_equal(one.read_kv(layer, 1), seq.read_kv(layer, 1))
    seq.close(); one.close(); fast.close()


@pytest.mark.timeout(600)
@pytest.mark.parametrize("name,pd,lm", [("q4_k_m", (12, 12, 14, 12, 12, 12, 14), 14), ("q4_0_under_q6_k", (2,) * 7, 14),
                                        ("q4_k_m_order_faithful", (12, 12, 14, 12, 12, 12, 14), 14)])
def test_llama_1b_shape_kquant_resident_kernel_equals_kernel_sequence(fh, torch_gpu, monkeypatch, name, pd, lm):
    """The Llama-3.2-1B shape with llama.cpp's Q4_K_M recipe (Q4_K q/k/o/gate/up, Q6_K v/down/lm_head: the v matrix shares the
    q;k;v phase on its own share of the 256 workgroups) and with seven Q4_0 projections under a Q6_K lm_head: after the same
    700-token prompt, 300 greedy steps of the one-kernel decode step (summing in the reference order) and of the kernel
    sequence give the same tokens, the same logits and the same cache, bit for bit.  Third case: the order-faithful mode of the
    Q4_K_M recipe, whose default is the kernel with the reference-order attention."""
    cfg = fh.synth.llama32_1b(Q4 if pd[0] == Q4 else Q8, max_seq=2048)
    cfg["lm_head_dtype"] = lm
    exact = name.endswith("order_faithful")
    if exact:
        cfg["flags"] = EXACT
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=5)
    monkeypatch.setenv("FORGE_HIP_PD_EXACT" if exact else "FORGE_HIP_PD_KQUANT", "0")
    seq = fh.HipModel(cfg, blob, proj_dtypes=pd)
    monkeypatch.delenv("FORGE_HIP_PD_EXACT" if exact else "FORGE_HIP_PD_KQUANT")
    monkeypatch.setenv("FORGE_HIP_PD_ORDERED", "1")
    one = fh.HipModel(cfg, blob, proj_dtypes=pd)
    monkeypatch.delenv("FORGE_HIP_PD_ORDERED")
    assert one.decode_launches == 1 and seq.decode_launches > 1
    prompt = fh.synth.uniform_ids(9, 700, cfg["vocab"])
    la = seq.forward_prefill(prompt)
    same_bits(one.forward_prefill(prompt), la)
    a = b = fh.ops.argmax_host(la)
    for step in range(300):
        a2, b2 = one.forward_greedy(a), seq.forward_greedy(b)
        assert a2 == b2, f"{name} step {step}: {a2} against {b2}"
        a, b = a2, b2
    same_bits(one.forward(a), seq.forward(b))
    for layer in (0, 7, 15):
        for which in (0, 1):
            assert np.array_equal(one.read_kv(layer, which), seq.read_kv(layer, which))
    seq.close(); one.close()
