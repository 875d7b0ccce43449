"""GPU parity of models that keep a storage format per projection (ProjectionDTypes,
crates/forgellm-frontend/src/ir.rs:410-421): Q8_0, Q4_0, Q4_K and Q6_K matrices side by side, as the reference builds
them from GGUF files whose tensor categories differ (detect_gguf_proj_dtypes, crates/forgellm-cli/src/main.rs:608-680).

The oracle is the CPU restatement of model::forward with matmul_call's per-projection dispatch (emit.rs:3316-3334) and of
forward_prefill's per-token walk (emit.rs:4621-5040); tests/test_oracle_model_pin.py holds it to a float64 model.  With
FLAG_EXACT every operation on the GPU is in the CPU path's order: logits, cache rows and greedy tokens are compared bit
for bit.  Without it the decode attention is the split-sequence kernel (within 1e-3 per call), held to the loose
end-to-end bound of the uniform models."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q8, Q4, Q4K, Q6K = 8, 2, 12, 14
A, KV_F16 = 0, 1
EXACT, QKV_BIAS = 1, 2

MIXES = {
    "q4_k_m": ((Q4K, Q4K, Q6K, Q4K, Q4K, Q4K, Q6K), Q6K),        # llama.cpp's Q4_K_M recipe
    "all_four": ((Q8, Q4, Q4K, Q8, Q6K, Q4, Q4K), Q8),
    "kquant_lm_head_only": ((Q4, Q4, Q4, Q4, Q4, Q4, Q4), Q6K),
    "q6_k": ((Q6K,) * 7, Q6K),
    "q8_0_under_q6_k": ((Q8,) * 7, Q6K),
}


def same_bits(got, want):
    got, want = np.ascontiguousarray(got, np.float32), np.ascontiguousarray(want, np.float32)
    diff = got.view(np.uint32) != want.view(np.uint32)
    assert not diff.any(), f"{diff.sum()} of {diff.size} differ in bits; max abs err {np.max(np.abs(got - want)):.3e}"


def rows_close(got, want, tol=2e-3):
    """Cache rows (fp16 values as f32) that went through different f32 arithmetic: within `tol` of |value| + the tensor's root
    mean square (half an fp16 step is 5e-4 of a value; the fast matmuls are held to 1e-3 of that unit at op level)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    unit = np.abs(want) + np.sqrt(np.mean(want ** 2))
    assert np.all(np.abs(got - want) <= tol * unit), f"max err / unit = {np.max(np.abs(got - want) / unit):.3e}"


def tiny(fh, lm, flags, **kw):
    shape = dict(hidden=256, inter=512, layers=2, heads=4, kv_heads=2, head_dim=64, vocab=1000)
    shape.update(kw)
    cfg = fh.synth.tiny(wdtype=Q8, max_seq=640, **shape)
    cfg["lm_head_dtype"] = lm
    cfg["flags"] = flags
    return cfg


@pytest.mark.parametrize("mix", list(MIXES))
def test_mixed_model_exact_mode_is_bit_identical(fh, oracle, torch_gpu, mix):
    pd, lm = MIXES[mix]
    cfg = tiny(fh, lm, EXACT)
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=21, std=0.05)
    toks = fh.synth.uniform_ids(12, 40, cfg["vocab"])
    gm = fh.HipModel(cfg, blob, proj_dtypes=pd)
    om = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    gl, ol = gm.forward_prefill(toks), om.prefill_batched(toks)
    assert gm.pos == om.pos == 40
    same_bits(gl, ol)
    for layer in range(cfg["layers"]):
        for which in (0, 1):
            same_bits(oracle.f16_to_f32(gm.read_kv(layer, which)), om.read_kv(layer, which))
    tok = oracle.argmax(ol)
    for _ in range(16):                                     # greedy decode, logits compared at every step
        g, o = gm.forward(tok), om.forward(tok)
        same_bits(g, o)
        tok = oracle.argmax(o)
    # a second prompt chunk continues the cache (a chat turn)
    more = fh.synth.uniform_ids(13, 9, cfg["vocab"])
    same_bits(gm.forward_prefill(more), om.prefill_batched(more))
    gm.reset()
    same_bits(gm.forward_prefill(toks), gl)
    gm.close()


@pytest.mark.parametrize("flags", [EXACT, 0])
def test_mixed_model_prompt_in_batches_equals_token_by_token(fh, oracle, torch_gpu, monkeypatch, flags):
    """A prompt through a K-quant model in batches of rows (every matrix read once per 8 rows) against the reference's
    token-by-token walk (FORGE_HIP_MIXED_BATCH=0).  Order-faithful mode: logits, cache rows and the tokens that follow, bit
    for bit (prompt lengths that end inside a batch of 8, at its end, and longer than one chunk would be).  Fast mode: the
    batches run on the int8 MFMA GEMM (K-quant matrices through their twins) and the MFMA attention: the first layer's cache
    rows to the fast matmul's bound, the logits to the fast mode's end-to-end bound."""
    pd, lm = MIXES["q4_k_m"]
    cfg = tiny(fh, lm, flags)
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=33, std=0.05)
    monkeypatch.setenv("FORGE_HIP_MIXED_BATCH", "0")
    walk = fh.HipModel(cfg, blob, proj_dtypes=pd)
    monkeypatch.delenv("FORGE_HIP_MIXED_BATCH")
    batch = fh.HipModel(cfg, blob, proj_dtypes=pd)
    for n in (1, 7, 8, 77):
        toks = fh.synth.uniform_ids(40 + n, n + 5, cfg["vocab"])
        walk.reset(); batch.reset()
        a, b = walk.forward_prefill(toks[:n]), batch.forward_prefill(toks[:n])
        for which in (0, 1):
            if flags & EXACT:
                assert np.array_equal(batch.read_kv(0, which), walk.read_kv(0, which))
            else:
                rows_close(oracle.f16_to_f32(batch.read_kv(0, which)), oracle.f16_to_f32(walk.read_kv(0, which)))
        if flags & EXACT:
            same_bits(b, a)
            more_a, more_b = walk.forward_prefill(toks[n:]), batch.forward_prefill(toks[n:])      # a second chunk continues the cache
            same_bits(more_b, more_a)
            assert np.array_equal(batch.read_kv(1, 1), walk.read_kv(1, 1))
        else:
            assert np.max(np.abs(a - b)) < 0.1 * max(1.0, float(np.std(a)) * 4) and (n < 8 or np.corrcoef(a, b)[0, 1] > 0.99)
    walk.close(); batch.close()


@pytest.mark.parametrize("mix", ["q4_k_m", "all_four"])
def test_mixed_model_with_qkv_bias(fh, oracle, torch_gpu, monkeypatch, mix):
    """Qwen2's q / k / v bias (emit.rs:4105-4120 in forward, :4663-4675 in the token-by-token prompt; blob project.rs:286-292)
    in a model with a format per projection.  Order-faithful mode: prompt (in batches for the all-K-quant mix, token by
    token for the other), cache rows and 12 greedy steps bit for bit the oracle's; the batched prompt equals the walk.  Fast
    mode (prompt on the MFMA GEMM): first-layer cache rows and logits to the fast mode's bounds."""
    pd, lm = MIXES[mix]
    cfg = tiny(fh, lm, EXACT | QKV_BIAS)
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=61, std=0.05)
    toks = fh.synth.uniform_ids(19, 45, cfg["vocab"])
    gm = fh.HipModel(cfg, blob, proj_dtypes=pd)
    om = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    gl, ol = gm.forward_prefill(toks), om.prefill_batched(toks)
    same_bits(gl, ol)
    for layer in range(cfg["layers"]):
        for which in (0, 1):
            same_bits(oracle.f16_to_f32(gm.read_kv(layer, which)), om.read_kv(layer, which))
    first_layer = [om.read_kv(0, which).copy() for which in (0, 1)]
    tok = oracle.argmax(ol)
    for _ in range(12):
        g, o = gm.forward(tok), om.forward(tok)
        same_bits(g, o)
        tok = oracle.argmax(o)
    monkeypatch.setenv("FORGE_HIP_MIXED_BATCH", "0")
    walk = fh.HipModel(cfg, blob, proj_dtypes=pd)
    monkeypatch.delenv("FORGE_HIP_MIXED_BATCH")
    same_bits(walk.forward_prefill(toks), gl)
    walk.close(); gm.close()
    fast = fh.HipModel(dict(cfg, flags=QKV_BIAS), blob, proj_dtypes=pd)
    fl = fast.forward_prefill(toks)
    for which in (0, 1):
        rows_close(oracle.f16_to_f32(fast.read_kv(0, which)), first_layer[which])
    assert np.max(np.abs(fl - ol)) < 0.1 * max(1.0, float(np.std(ol)) * 4) and np.corrcoef(fl, ol)[0, 1] > 0.995
    fast.close()


@pytest.mark.parametrize("mix", ["q4_k_m", "all_four"])
def test_mixed_model_with_a_sliding_window(fh, oracle, torch_gpu, monkeypatch, mix):
    """A model with a window and a format per projection (Mistral files in K-quant recipes).  The reference walks its prompt
    token by token through `attention` over ALL earlier rows (emit.rs:4717-4720; never attention_sliding) and applies the
    window in decode steps only (emit.rs:4156-4170).  Order-faithful mode: prompt longer than the window (in batches for the
    all-K-quant mix), a second chunk, cache rows and 14 greedy steps bit for bit the oracle's; fast mode to its bounds."""
    pd, lm = MIXES[mix]
    cfg = tiny(fh, lm, EXACT)
    cfg["sliding_window"] = 24
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=71, std=0.05)
    toks = fh.synth.uniform_ids(23, 70, cfg["vocab"])
    gm = fh.HipModel(cfg, blob, proj_dtypes=pd)
    om = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    gl, ol = gm.forward_prefill(toks[:50]), om.prefill_batched(toks[:50])
    same_bits(gl, ol)
    first_layer = [om.read_kv(0, which).copy() for which in (0, 1)]
    same_bits(gm.forward_prefill(toks[50:]), om.prefill_batched(toks[50:]))
    for which in (0, 1):
        same_bits(oracle.f16_to_f32(gm.read_kv(1, which)), om.read_kv(1, which))
    tok = 7
    for _ in range(14):
        g, o = gm.forward(tok), om.forward(tok)
        same_bits(g, o)
        tok = oracle.argmax(o)
    gm.close()
    fast = fh.HipModel(dict(cfg, flags=0), blob, proj_dtypes=pd)
    fl = fast.forward_prefill(toks[:50])
    for which in (0, 1):
        rows_close(oracle.f16_to_f32(fast.read_kv(0, which)), first_layer[which])
    assert np.max(np.abs(fl - ol)) < 0.1 * max(1.0, float(np.std(ol)) * 4) and np.corrcoef(fl, ol)[0, 1] > 0.995
    # decode steps with the window: against the oracle fed the same tokens (teacher forcing keeps the contexts equal)
    om2 = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    om2.prefill_batched(toks[:50])
    for t in (3, 99, 500, 41):
        a, b = fast.forward(t), om2.forward(t)
        assert np.max(np.abs(a - b)) < 0.1 * max(1.0, float(np.std(b)) * 4) and np.corrcoef(a, b)[0, 1] > 0.99
    fast.close()


def test_mixed_model_greedy_tokens_at_a_real_width(fh, oracle, torch_gpu):
    """Llama-3.2-1B's widths (hidden 2048 = 8 super-blocks per row, inter 8192, 32:8 heads of 64) in the Q4_K_M recipe:
    prompt + 24 greedy tokens, ids identical to the oracle's."""
    pd, lm = MIXES["q4_k_m"]
    cfg = tiny(fh, lm, EXACT, hidden=2048, inter=8192, heads=32, kv_heads=8, vocab=4096)
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=3, std=0.02)
    prompt = fh.synth.uniform_ids(5, 24, cfg["vocab"])
    gm = fh.HipModel(cfg, blob, proj_dtypes=pd)
    om = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    want = [oracle.argmax(om.prefill_batched(prompt))]
    for _ in range(23):
        want.append(oracle.argmax(om.forward(want[-1])))
    assert gm.generate_greedy(prompt, 24) == want
    gm.close()


@pytest.mark.parametrize("mix", ["q4_k_m", "all_four", "kquant_lm_head_only"])
def test_mixed_model_fast_mode(fh, oracle, torch_gpu, mix, monkeypatch):
    pd, lm = MIXES[mix]
    cfg = tiny(fh, lm, 0)
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=21, std=0.05)
    toks = fh.synth.uniform_ids(12, 40, cfg["vocab"])
    gm = fh.HipModel(cfg, blob, proj_dtypes=pd)
    # all matrices Q4_K / Q6_K, or seven plain projections of one format under a Q6_K lm_head: one resident kernel per step;
    # any other mix: the kernel sequence
    assert (gm.decode_launches == 1) == (mix != "all_four")
    om = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    gl, ol = gm.forward_prefill(toks), om.prefill_batched(toks)
    # layer 0's K/V rows depend on embedding -> rms_norm -> matmul -> rope only: the fast matmul's bound
    for which in (0, 1):
        rows_close(oracle.f16_to_f32(gm.read_kv(0, which)), om.read_kv(0, which))
    assert np.max(np.abs(gl - ol)) < 0.1 * max(1.0, float(np.std(ol)) * 4)
    assert np.corrcoef(gl, ol)[0, 1] > 0.995
    # the captured graph replays what the eager launches compute
    steps = [int(t) for t in fh.synth.uniform_ids(14, 6, cfg["vocab"])]
    graph = [gm.forward(t) for t in steps]
    gm.close()
    monkeypatch.setenv("FORGE_HIP_GRAPH", "0")
    ge = fh.HipModel(cfg, blob, proj_dtypes=pd)
    assert np.array_equal(ge.forward_prefill(toks), gl)
    for t, want in zip(steps, graph):
        assert np.array_equal(ge.forward(t), want)
    ge.close()


@pytest.mark.parametrize("mix", ["q4_k_m", "all_four", "q6_k"])
def test_mixed_model_prompt_on_the_matrix_unit(fh, oracle, torch_gpu, monkeypatch, mix):
    """Fast mode: a prompt's K-quant projections as int8 MFMA GEMMs over the matrices' twins, against the same model with
    FORGE_HIP_KQ_MFMA=0 (the multi-row GEMV, whose rows are matmul_vec's bit for bit) and against the oracle.  Cache rows of
    the first layer to the fast matmul's bound and NOT the same bits (the other arithmetic did run); logits to the fast
    mode's end-to-end bound; a prompt that ends inside a tile, a second chunk, and greedy tokens that follow."""
    pd, lm = MIXES[mix]
    cfg = tiny(fh, lm, 0)
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=44, std=0.05)
    toks = fh.synth.uniform_ids(17, 150, cfg["vocab"])
    monkeypatch.setenv("FORGE_HIP_KQ_MFMA", "0")
    rows = fh.HipModel(cfg, blob, proj_dtypes=pd)
    monkeypatch.delenv("FORGE_HIP_KQ_MFMA")
    mfma = fh.HipModel(cfg, blob, proj_dtypes=pd)
    om = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    a, b, o = rows.forward_prefill(toks[:131]), mfma.forward_prefill(toks[:131]), om.prefill_batched(toks[:131])
    differs = False
    for which in (0, 1):
        ra, rb = rows.read_kv(0, which), mfma.read_kv(0, which)
        rows_close(oracle.f16_to_f32(rb), oracle.f16_to_f32(ra))
        rows_close(oracle.f16_to_f32(rb), om.read_kv(0, which))
        differs = differs or not np.array_equal(ra, rb)
    assert differs
    bound = 0.1 * max(1.0, float(np.std(o)) * 4)
    assert np.max(np.abs(b - a)) < bound and np.max(np.abs(b - o)) < bound
    assert np.corrcoef(b, o)[0, 1] > 0.995
    b2, o2 = mfma.forward_prefill(toks[131:]), om.prefill_batched(toks[131:])
    assert np.max(np.abs(b2 - o2)) < bound and np.corrcoef(b2, o2)[0, 1] > 0.995
    again = fh.HipModel(cfg, blob, proj_dtypes=pd)                       # the same bits from a second model: nothing depends on the run
    assert np.array_equal(again.forward_prefill(toks[:131]), b)
    rows.close(); mfma.close(); again.close()


def test_mixed_model_grouped_launches_keep_the_bits(fh, torch_gpu, monkeypatch):
    """K-quant projections that read the same normed row (q, k, v; gate, up) go out as ONE launch that norms and quantises
    the row itself; FORGE_HIP_MIXED_FUSE=0 keeps the norm kernel in front.  Same logits and cache rows bit for bit, fewer
    launches per step.  A mix with a Q8_0 matrix in the group keeps the norm kernel for it."""
    monkeypatch.setenv("FORGE_HIP_PD_EXACT", "0")            # the kernel sequence (all-K-quant models default to the resident kernel)
    for mix, fewer in (("q4_k_m", True), ("all_four", False)):
        pd, lm = MIXES[mix]
        cfg = tiny(fh, lm, EXACT)
        blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=5, std=0.05)
        toks = fh.synth.uniform_ids(9, 19, cfg["vocab"])
        monkeypatch.setenv("FORGE_HIP_MIXED_FUSE", "0")
        plain = fh.HipModel(cfg, blob, proj_dtypes=pd)
        monkeypatch.delenv("FORGE_HIP_MIXED_FUSE")
        fused = fh.HipModel(cfg, blob, proj_dtypes=pd)
        assert (fused.decode_launches < plain.decode_launches) == fewer
        same_bits(fused.forward_prefill(toks), plain.forward_prefill(toks))
        for t in (3, 77, 500):
            same_bits(fused.forward(t), plain.forward(t))
        for layer in range(cfg["layers"]):
            assert np.array_equal(fused.read_kv(layer, 0), plain.read_kv(layer, 0))
        plain.close(); fused.close()


@pytest.mark.parametrize("mix,extra", [("q4_k_m", {}), ("q6_k", {}), ("q4_k_m", dict(flags=QKV_BIAS)), ("q4_k_m", dict(sliding_window=24)),
                                       ("q4_k_m", dict(hidden=512, inter=1024, heads=4, kv_heads=4, head_dim=128)),
                                       ("q4_k_m", dict(layers=36)), ("kquant_lm_head_only", dict(layers=35)),      # two launches per step
                                       ("kquant_lm_head_only", {}), ("q8_0_under_q6_k", dict(flags=QKV_BIAS)),
                                       ("kquant_lm_head_only", dict(sliding_window=24, hidden=512, inter=1024, heads=4, kv_heads=4, head_dim=96))])
def test_kquant_weight_units_in_the_resident_kernel(fh, torch_gpu, monkeypatch, mix, extra):
    """The decode step of a model whose matrices are all Q4_K / Q6_K is ONE resident kernel (FORGE_HIP_PD_KQUANT=0: the kernel
    sequence), the matrices re-laid out as its weight units (Q4_K: Q4_0-ordered nibbles + a word of d | dmin, scale and minimum
    per sub-block; Q6_K: 16 bytes per 16 weights with scale and d inside); a v matrix of another format than q and k shares
    the q;k;v phase with them, each side on its own share of the workgroups.  Seven Q4_0 or seven Q8_0 projections under a
    Q6_K lm_head (llama.cpp's Q4_0 / Q8_0 files with a K-quant output matrix) run the uniform model's kernel with the lm_head as
    K-quant weight units.  With
    the ordered row sums (FORGE_HIP_PD_ORDERED=1) every logit equals the kernel sequence's bit for bit, step after step, and
    the cache rows too; the default sums differ by the order of additions (and by the int8 activation codes that this moves)."""
    pd, lm = MIXES[mix]
    flags = extra.get("flags", 0)
    shape = {k: v for k, v in extra.items() if k not in ("flags", "sliding_window")}
    cfg = tiny(fh, lm, flags, **shape)
    cfg["sliding_window"] = extra.get("sliding_window", 0)
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=29, std=0.05)
    toks = fh.synth.uniform_ids(31, 45, cfg["vocab"])
    monkeypatch.setenv("FORGE_HIP_PD_KQUANT", "0")
    seq = fh.HipModel(cfg, blob, proj_dtypes=pd)
    assert seq.decode_launches > 1
    monkeypatch.delenv("FORGE_HIP_PD_KQUANT")
    fast = fh.HipModel(cfg, blob, proj_dtypes=pd)
    monkeypatch.setenv("FORGE_HIP_PD_ORDERED", "1")
    ordered = fh.HipModel(cfg, blob, proj_dtypes=pd)
    monkeypatch.delenv("FORGE_HIP_PD_ORDERED")
    assert fast.decode_launches == ordered.decode_launches == (cfg["layers"] + 33) // 34
    a = seq.forward_prefill(toks)
    assert np.array_equal(a, ordered.forward_prefill(toks)) and np.array_equal(a, fast.forward_prefill(toks))
    tok = int(np.argmax(a))
    for step in range(30):                                  # past the window where there is one
        x, y, z = seq.forward(tok), ordered.forward(tok), fast.forward(tok)
        same_bits(y, x)
        # a last-bit difference in a norm can move an int8 activation code by one: quantisation noise, not rounding noise, and
        # the caches of the two models drift apart by it from step to step
        assert np.corrcoef(z, x)[0, 1] > 0.999 and np.max(np.abs(z - x)) < (0.03 if step == 0 else 0.15) * max(1.0, float(np.std(x)))
        tok = int(np.argmax(x))
    for layer in range(cfg["layers"]):
        for which in (0, 1):
            assert np.array_equal(ordered.read_kv(layer, which), seq.read_kv(layer, which))
    # greedy decoding on the device, and a reset
    seq.reset(); ordered.reset()
    assert ordered.generate_greedy(toks[:9], 12) == seq.generate_greedy(toks[:9], 12)
    # the repeat penalty on the device (the lm_head phase's epilogue; the sequence's argmax kernel)
    seq.reset(); ordered.reset()
    seq.set_repeat_penalty(1.3); ordered.set_repeat_penalty(1.3)
    pa, pb = seq.generate_greedy(toks[:9], 16), ordered.generate_greedy(toks[:9], 16)
    assert pa == pb
    seq.close(); ordered.close(); fast.close()


def test_uniform_formats_through_the_mixed_entry_point_are_the_plain_model(fh, torch_gpu):
    cfg = tiny(fh, Q8, 0)
    cfg["wdtype"] = Q4
    blob = fh.synth.make_weights_blob(cfg, seed=4)
    toks = fh.synth.uniform_ids(2, 33, cfg["vocab"])
    a = fh.HipModel(cfg, blob)
    b = fh.HipModel(cfg, blob, proj_dtypes=[Q4] * 7)
    assert b.decode_launches == a.decode_launches == 1      # the resident kernel, as for forge_hip_model_create
    assert np.array_equal(a.forward_prefill(toks), b.forward_prefill(toks))
    assert a.generate_greedy([1, 2, 3], 8) == b.generate_greedy([1, 2, 3], 8)
    a.close()
    b.close()


def test_mixed_model_refusals(fh, torch_gpu):
    pd, lm = MIXES["q4_k_m"]
    cfg = tiny(fh, lm, 0)
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=1)
    with pytest.raises(fh.ForgeHipError) as e:                 # a format the kernels do not carry
        fh.HipModel(cfg, blob, proj_dtypes=[13] + list(pd[1:]))
    assert e.value.code == fh.ERR_INVALID
    with pytest.raises(fh.ForgeHipError) as e:                 # blob of another mix
        fh.HipModel(cfg, blob, proj_dtypes=MIXES["all_four"][0])
    assert e.value.code == fh.ERR_BLOB_SIZE
    with pytest.raises(fh.ForgeHipError) as e:                 # order-faithful mode keeps a prompt row's scores in LDS: max_seq <= 12288
        fh.HipModel(dict(cfg, sliding_window=64, max_seq=16384, flags=EXACT), blob, proj_dtypes=pd)
    assert e.value.code == fh.ERR_INVALID
    with pytest.raises(fh.ForgeHipError) as e:                 # the bias flag without bias vectors in the blob
        fh.HipModel(dict(cfg, flags=QKV_BIAS), blob, proj_dtypes=pd)
    assert e.value.code == fh.ERR_BLOB_SIZE
    # SmolLM2's hidden 576 is no multiple of a 256-weight super-block
    c = tiny(fh, Q8, 0, hidden=576, inter=1536, heads=9, kv_heads=3)
    with pytest.raises(fh.ForgeHipError) as e:
        fh.HipModel(c, np.zeros(16, np.uint8), proj_dtypes=pd)
    assert e.value.code == fh.ERR_INVALID
    # a K-quant lm_head needs the per-projection entry point
    with pytest.raises(fh.ForgeHipError) as e:
        fh.HipModel(cfg, blob)
    assert e.value.code == fh.ERR_INVALID


@pytest.mark.parametrize("mix", ["q4_k_m", "kquant_lm_head_only", "all_four"])
def test_mixed_model_on_a_paged_cache(fh, torch_gpu, mix):
    """A model with a format per projection over a PAGED cache (pages in a shuffled order): prompt in two chunks, logits of
    decode steps, greedy tokens and the cache rows equal the flat cache's bit for bit -- with the resident kernel (K-quant
    weight units; plain projections under a Q6_K lm_head) and with the kernel sequence (the mix of all four formats)."""
    pd, lm = MIXES[mix]
    cfg = tiny(fh, lm, 0)
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=61, std=0.05)
    toks = fh.synth.uniform_ids(62, 300, cfg["vocab"])
    flat, paged = fh.HipModel(cfg, blob, proj_dtypes=pd), fh.HipModel(cfg, blob, proj_dtypes=pd)
    page_rows = 64
    table = np.random.default_rng(9).permutation(cfg["max_seq"] // page_rows).astype(np.uint32)
    paged.set_kv_pages(page_rows, table)
    for m in (flat, paged):
        m.forward_prefill_batch(toks[:150])
    same_bits(paged.forward_prefill(toks[150:280]), flat.forward_prefill(toks[150:280]))
    for t in toks[280:290]:
        same_bits(paged.forward(int(t)), flat.forward(int(t)))
    a = b = int(toks[290])
    for _ in range(8):
        a, b = paged.forward_greedy(a), flat.forward_greedy(b)
        assert a == b
    for layer in range(cfg["layers"]):
        for which in (0, 1):
            assert np.array_equal(paged.read_kv(layer, which), flat.read_kv(layer, which))
    flat.close(); paged.close()


@pytest.mark.parametrize("mix", ["q4_k_m", "q6_k"])
def test_order_faithful_kquant_model_on_the_resident_kernel(fh, oracle, torch_gpu, monkeypatch, mix):
    """The order-faithful decode step of an all-K-quant model is ONE resident kernel (ordered row sums, the attention walked in
    the reference's 64-key blocks; FORGE_HIP_PD_EXACT=0: the kernel sequence): prompt, 16 greedy steps and the cache rows of
    both bit for bit the CPU oracle's."""
    pd, lm = MIXES[mix]
    cfg = tiny(fh, lm, EXACT)
    blob = fh.synth.make_weights_blob_mixed(cfg, pd, seed=77, std=0.05)
    toks = fh.synth.uniform_ids(78, 70, cfg["vocab"])
    monkeypatch.setenv("FORGE_HIP_PD_EXACT", "0")
    seq = fh.HipModel(cfg, blob, proj_dtypes=pd)
    assert seq.decode_launches > 1
    monkeypatch.delenv("FORGE_HIP_PD_EXACT")
    one = fh.HipModel(cfg, blob, proj_dtypes=pd)
    assert one.decode_launches == 1
    om = oracle.Model(cfg, blob, A, KV_F16, proj_dtypes=pd)
    ol = om.prefill_batched(toks)
    same_bits(one.forward_prefill(toks), ol)
    same_bits(seq.forward_prefill(toks), ol)
    tok = oracle.argmax(ol)
    for _ in range(16):
        w = om.forward(tok)
        same_bits(one.forward(tok), w)
        same_bits(seq.forward(tok), w)
        tok = oracle.argmax(w)
    for layer in range(cfg["layers"]):
        for which in (0, 1):
            assert np.array_equal(one.read_kv(layer, which), seq.read_kv(layer, which))
    seq.close(); one.close()
