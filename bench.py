"""Benchmark: Llama-3.2-1B-shape Q8_0 model (random-init from a seed) on ONE MI355X.

A "step" is one greedy decode token (forward + on-device argmax + 4-byte read-back).  The
script prefills a 2502-token prompt (timed: prefill tok/s), then runs W warm-up and K timed
decode steps at that context, and prints ONE JSON line.  Weights, KV cache and activations are
resident in HBM when the timed regions start.

roofline: the decode step's dominant kernel.  By default the whole step is ONE resident kernel
(decode_step_kernel): `achieved` = algorithmic bytes of one token (GGUF block bytes of every matrix + the
f32 input and output vectors of each GEMV + the fp16 K/V rows attention reads) / the kernel's duration,
measured live by the library's forward_profile from the kernel's own clock stamps (one per phase, summed).
With FORGE_HIP_PERSIST=0 the step is a sequence of kernels and the figure is that of the quantised GEMV
launches, each timed by a pair of HIP events attached to its dispatch.  The line also carries the other
path's figures under "kernel_sequence_path".  `peak` = 8 TB/s (MI355X HBM3E).

exact_mode: the same workload on a model created with FORGE_HIP_FLAG_EXACT (bit-identical to the reference's
generated kernels): its prefill and decode throughput, and the fast mode's distance from it (first greedy token
that differs, largest logit difference before that).

kquant_model: the same shape with a storage format per projection (llama.cpp's Q4_K_M recipe, random super-blocks):
prompt and decode throughput in fast mode (prompt on the MFMA GEMM through re-expressed matrices, decode as one resident
kernel with K-quant weight units, the kernel sequence beside it) and in the order-faithful mode (prompt through the
multi-row K-quant GEMV, decode as the resident kernel's ordered variant); and llama.cpp's Q4_0 recipe with a K-quant output matrix (seven Q4_0 projections under a Q6_K
lm_head) in fast mode.

cpu_baseline: the CPU restatement of the reference's generated kernels (oracle/) on this host's cores, on the same
model and prompt: in the aarch64 arithmetic (int8 activation blocks) the whole prompt as a batched prefill and
decode steps at that context; in the arithmetic the reference runs on an x86 host (f32 activations x dequantised
weights, int8 KV; `value`) decode steps at the same context and the batched prefill of a 64-token sample.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
from __graft_entry__ import load_package  # noqa: E402

HBM_PEAK_GBS = 8000.0
MFMA_I8_PEAK_TOPS = 5000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
PROMPT_TOKENS = 2502
DIVERGENCE_STEPS = 128         # greedy steps over which the fast mode's tokens are compared with the exact mode's
# HBM bytes per GEMV launch of this workload, averaged over the 65 GEMV launches of one decode step: FETCH_SIZE and
# WRITE_SIZE counters of two profiler runs of this script, each scaled by what the same counter reads for the 1 GiB
# copy of --calibrate-copy (FETCH_SIZE x2.000, WRITE_SIZE x1.000).  Summary: profiles/gemv_hbm_traffic_pmc.md.
GEMV_HBM_BYTES_PER_LAUNCH = 20.46e6 + 0.02e6      # fetched + written
# The same for one launch of the resident decode kernel (the whole step) at this context: 1 436.9 MB fetched + 13.8 MB
# written.  Summary: profiles/decode_step_kernel_hbm_traffic_pmc.md.
STEP_KERNEL_HBM_BYTES_PER_LAUNCH = 1450.7e6


def gemv_launch_bytes(fh, cfg):
    """Algorithmic bytes of the GEMV launches of one decode step, per stage."""
    H, I = cfg["hidden"], cfg["inter"]
    QKS, KV = cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"]
    wt, g = cfg["wdtype"], fh.synth.gemv_bytes
    L = cfg["layers"]
    return {
        "qkv_matmul": L * (g(QKS, H, wt) + 2 * g(KV, H, wt)),
        "o_matmul": L * g(H, QKS, wt),
        "gate_up_matmul": L * 2 * g(I, H, wt),
        "down_matmul": L * g(H, I, wt),
        "lm_head_matmul": g(cfg["vocab"], H, cfg["lm_head_dtype"]),
    }


def prefill_flops(cfg, m):
    H, I = cfg["hidden"], cfg["inter"]
    QKS, KV = cfg["heads"] * cfg["head_dim"], cfg["kv_heads"] * cfg["head_dim"]
    gemm = 2 * m * cfg["layers"] * (H * QKS + 2 * H * KV + QKS * H + 2 * H * I + I * H)
    w = cfg.get("sliding_window", 0)
    pairs = m * (m + 1) // 2 if not w or w >= m else w * (w + 1) // 2 + (m - w) * w      # sum over positions of min(p + 1, w)
    attn = cfg["layers"] * 4 * cfg["head_dim"] * cfg["heads"] * pairs
    return gemm, attn


def cpu_baseline(fh, cfg, blob, prompt, decode_steps=8, b_prefill_tokens=64):
    """The CPU restatement of the reference's generated kernels, timed on this host's cores on a bounded sample of the same
    workload.  Variant A (int8 activation blocks, fp16 KV: the arithmetic the GPU's exact mode reproduces bit for bit)
    runs the WHOLE prompt through forward_prefill_batched and then `decode_steps` greedy tokens at that context: the
    workload the GPU figures are measured on.  Variant B (f32 activations x dequantised weights, int8 KV: what an x86
    build of the reference executes, and `value`) prefills token by token inside matmul_mat, far too slowly for the whole
    prompt: its batched prefill is timed on the first `b_prefill_tokens` tokens, then the model takes over variant A's
    cached context (every K/V row through its own int8 cache write) and decodes `decode_steps` tokens at the full
    context."""
    from oracle import oracle
    threads = oracle.num_threads()
    n = len(prompt)
    a = oracle.Model(cfg, blob, oracle.VARIANT_A, oracle.KV_F16)
    t0 = time.perf_counter()
    tok_a = oracle.argmax(a.prefill_batched(prompt))
    a_prefill_s = time.perf_counter() - t0
    b = oracle.Model(cfg, blob, oracle.VARIANT_B, oracle.KV_INT8)
    t0 = time.perf_counter()
    b.prefill_batched(prompt[:b_prefill_tokens], want_logits=False)
    b_prefill_s = time.perf_counter() - t0
    b.adopt_context(a)
    rates = {}
    for name, om in (("A", a), ("B", b)):
        tok = tok_a
        t0 = time.perf_counter()
        for _ in range(decode_steps):
            tok = oracle.argmax(om.forward(tok))
        rates[name] = decode_steps / (time.perf_counter() - t0)
        om.close()
    return {"value": rates["B"], "unit": "tok/s", "cores": threads, "kind": "port",
            "decode_context": n, "prefill_tok_per_s": b_prefill_tokens / b_prefill_s, "prefill_tokens": b_prefill_tokens,
            "variant_a": {"decode_tok_per_s": rates["A"], "decode_context": n, "prefill_tok_per_s": n / a_prefill_s, "prefill_tokens": n,
                          "arithmetic": "int8 activation blocks x int8 weight blocks (the reference's aarch64 kernels), fp16 KV"},
            "sample": f"same model, weights and prompt.  Variant A: forward_prefill_batched over all {n} prompt tokens, then "
                      f"{decode_steps} greedy decode tokens at context {n}.  Variant B (value; f32 x dequantised-weight arithmetic "
                      f"of the reference's x86 build, int8 KV): forward_prefill_batched over the first {b_prefill_tokens} prompt "
                      f"tokens, then {decode_steps} decode tokens at context {n} over variant A's cached rows re-quantised to "
                      f"int8.  OpenMP over rows / heads with {threads} threads"}


def decode_profile(fh, model, cfg, tok, context, prof_steps=8):
    """Per-stage device time of the decode step and the roofline of its dominant kernel."""
    stage_ms, stage_n = {}, {}
    for _ in range(prof_steps):
        p = model.forward_profile(tok)
        for s, (ms, n) in p.items():
            stage_ms[s] = stage_ms.get(s, 0.0) + ms / prof_steps
            stage_n[s] = stage_n.get(s, 0) + n
    gbytes = gemv_launch_bytes(fh, cfg)
    gemv_bytes_total = sum(gbytes.values())
    per_stage = {s: {"GB/s": round(gbytes[s] / (stage_ms[s] * 1e-3) / 1e9, 1), "us_per_token": round(stage_ms[s] * 1e3, 1)} for s in gbytes}
    stage_us = {s: round(v * 1e3, 1) for s, v in stage_ms.items() if v > 0}
    n_launch = model.decode_launches
    if n_launch <= (cfg["layers"] + 33) // 34:
        # one resident kernel per token: its phases are the stages, timed by the kernel's own clock stamps
        rows = min(context, cfg.get("sliding_window", 0) or context)          # a sliding window bounds the rows a step reads
        kv_bytes = cfg["layers"] * 2 * rows * cfg["kv_heads"] * cfg["head_dim"] * 2
        total = gemv_bytes_total + kv_bytes
        kernel_ms = sum(stage_ms.values())
        achieved = total / (kernel_ms * 1e-3) / 1e9
        roof = {"kernel": "decode_step_kernel (the whole decode step: every quantised GEMV, decode attention, norms, argmax)",
                "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                "traffic": STEP_KERNEL_HBM_BYTES_PER_LAUNCH, "bytes_per_launch": total / n_launch, "us_per_launch": kernel_ms * 1e3 / n_launch,
                "launches_per_step": n_launch, "weights_and_vectors_bytes": gemv_bytes_total, "kv_cache_bytes": kv_bytes,
                "per_phase": per_stage}
    else:
        gemv_ms = sum(stage_ms[s] for s in gbytes)
        launches = sum(stage_n[s] for s in gbytes) // prof_steps
        achieved = gemv_bytes_total / (gemv_ms * 1e-3) / 1e9
        roof = {"kernel": "gemv_kernel (quantised GEMV, all launches of one decode step)", "bound": "hbm", "achieved": achieved,
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                "traffic": GEMV_HBM_BYTES_PER_LAUNCH if cfg["wdtype"] == fh.Q8_0 else None,
                "bytes_per_launch": gemv_bytes_total / launches, "us_per_launch": gemv_ms * 1e3 / launches,
                "launches_per_step": launches, "per_stage": per_stage}
    return roof, stage_us


def timed_decode(model, tok, warmup, steps):
    import torch
    for _ in range(warmup):
        tok = model.forward_greedy(tok)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        tok = model.forward_greedy(tok)
    torch.cuda.synchronize()
    return time.perf_counter() - t0, tok


def greedy_with_logits(fh, model, prompt, n):
    """Prefill, then n greedy picks, every step through `forward` so the logits come back: tokens [n] and logits
    [n][vocab] (logits[i] are the ones whose argmax is tokens[i])."""
    import numpy as np
    model.reset()
    logits = [model.forward_prefill(prompt)]
    toks = [fh.ops.argmax_host(logits[0])]
    for _ in range(n - 1):
        logits.append(model.forward(toks[-1]))
        toks.append(fh.ops.argmax_host(logits[-1]))
    return toks, np.stack(logits)


def exact_mode_figures(fh, cfg, blob, prompt, warmup, steps, fast_tokens, fast_logits):
    """The same workload with FORGE_HIP_FLAG_EXACT (the arithmetic that reproduces the reference's generated kernels bit
    for bit: ordered block sums, the reference's softmax and exponential): prefill and decode throughput, and how far the
    fast mode measured above is from it -- the first greedy token at which the two differ over `len(fast_tokens)` steps,
    the largest logit difference while both still had the same context, and the margin between the two largest exact
    logits at the step where they part (how close that choice was)."""
    import numpy as np
    import torch
    m = fh.HipModel(dict(cfg, flags=cfg.get("flags", 0) | fh.FLAG_EXACT), blob)
    m.forward_prefill_batch(prompt)
    m.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    logits = m.forward_prefill(prompt)
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    t_decode, _ = timed_decode(m, fh.ops.argmax_host(logits), warmup, steps)
    launches = m.decode_launches
    toks, lg = greedy_with_logits(fh, m, prompt, len(fast_tokens))
    m.close()
    same = [a == b for a, b in zip(toks, fast_tokens)]
    first = same.index(False) if False in same else None
    shared = len(toks) if first is None else first + 1            # logits[i] come from identical contexts for i <= first
    delta = np.abs(lg[:shared].astype(np.float64) - fast_logits[:shared]).max(axis=1)
    out = {"decode_tok_per_s": steps / t_decode, "ms_per_step": t_decode / steps * 1e3, "prefill_tok_per_s": len(prompt) / t_prefill,
           "prefill_ms": t_prefill * 1e3, "decode_path": f"{launches} kernels per token (graph replay), order-faithful kernels",
           "fast_vs_exact": {"greedy_steps_compared": len(toks), "first_divergent_token": first,
                             "max_logit_delta": float(delta.max()), "prefill_logit_delta": float(delta[0]),
                             "logit_absmax": float(np.abs(lg[:shared]).max())}}
    if first is not None:
        top2 = np.partition(lg[first], -2)[-2:]
        out["fast_vs_exact"]["exact_top2_margin_at_divergence"] = float(top2[1] - top2[0])
    # the same mode with the whole step as one resident kernel (ordered row sums, attention walked in the reference's
    # 64-key blocks): bit-identical to the kernel sequence, measured beside it; the library's default is the sequence
    if cfg.get("sliding_window", 0) == 0:
        import os
        os.environ["FORGE_HIP_PD_EXACT"] = "1"
        try:
            m = fh.HipModel(dict(cfg, flags=cfg.get("flags", 0) | fh.FLAG_EXACT), blob)
            if m.decode_launches < launches:
                m.forward_prefill_batch(prompt)
                t1, _ = timed_decode(m, fh.ops.argmax_host(logits), warmup, steps)
                one_toks, _ = greedy_with_logits(fh, m, prompt, min(16, len(toks)))
                out["one_resident_kernel"] = {"decode_tok_per_s": steps / t1, "ms_per_step": t1 / steps * 1e3, "launches_per_token": m.decode_launches,
                                              "tokens_identical_to_kernel_sequence": one_toks == toks[:len(one_toks)], "selected_by": "FORGE_HIP_PD_EXACT=1"}
            m.close()
        finally:
            del os.environ["FORGE_HIP_PD_EXACT"]
    return out


def kquant_model_figures(fh, cfg, prompt, warmup, steps, seed):
    """The same shape with llama.cpp's Q4_K_M recipe (Q4_K q/k/o/gate/up, Q6_K v/down/lm_head; random super-blocks): the model
    with a storage format per projection.  Fast mode: prompt on the int8 MFMA GEMM through the matrices' twins, decode as one
    resident kernel (the kernel sequence timed beside it); order-faithful mode: prompt through the multi-row K-quant GEMV (bit for bit the reference's
    token-by-token walk)."""
    kcfg = dict(cfg)
    kcfg["lm_head_dtype"] = 14
    pd = (12, 12, 14, 12, 12, 12, 14)
    blob = fh.synth.make_weights_blob_mixed(kcfg, pd, seed=seed)
    t0 = time.perf_counter()
    m = fh.HipModel(kcfg, blob, proj_dtypes=pd)
    t_create = time.perf_counter() - t0
    m.forward_prefill(prompt)                                # first pass: kernels loaded, workspaces touched
    m.reset()
    t0 = time.perf_counter()
    tok = fh.ops.argmax_host(m.forward_prefill(prompt))
    t_prefill = time.perf_counter() - t0
    t_decode, tok = timed_decode(m, tok, warmup, steps)
    out = {"formats": "Q4_K q/k/o/gate/up, Q6_K v/down/lm_head", "weights_bytes": int(blob.size),
           "prefill_tok_per_s": len(prompt) / t_prefill, "prefill_ms": t_prefill * 1e3,
           "decode_tok_per_s": steps / t_decode, "decode_launches_per_token": m.decode_launches,
           "create_s_incl_twins": round(t_create, 2)}
    m.close()
    import os
    os.environ["FORGE_HIP_PD_KQUANT"] = "0"                  # the same step as a sequence of kernels (grouped K-quant GEMVs)
    try:
        m = fh.HipModel(kcfg, blob, proj_dtypes=pd)
        tok = fh.ops.argmax_host(m.forward_prefill(prompt))
        t_seq, tok = timed_decode(m, tok, warmup, steps)
        out["kernel_sequence"] = {"decode_tok_per_s": steps / t_seq, "decode_launches_per_token": m.decode_launches}
        m.close()
    finally:
        del os.environ["FORGE_HIP_PD_KQUANT"]
    ecfg = dict(kcfg, flags=fh.FLAG_EXACT)
    e = fh.HipModel(ecfg, blob, proj_dtypes=pd)
    t0 = time.perf_counter()
    tok = fh.ops.argmax_host(e.forward_prefill(prompt))
    t_eprefill = time.perf_counter() - t0
    t_edecode, tok = timed_decode(e, tok, warmup, steps)
    out["order_faithful"] = {"prefill_tok_per_s": len(prompt) / t_eprefill, "decode_tok_per_s": steps / t_edecode}
    e.close()
    # llama.cpp's Q4_0 recipe with a K-quant output matrix: seven Q4_0 projections under a Q6_K lm_head (fast mode)
    qcfg = dict(cfg, wdtype=2, lm_head_dtype=14)
    qpd = (2,) * 7
    qblob = fh.synth.make_weights_blob_mixed(qcfg, qpd, seed=seed)
    q = fh.HipModel(qcfg, qblob, proj_dtypes=qpd)
    q.forward_prefill(prompt)
    q.reset()
    t0 = time.perf_counter()
    tok = fh.ops.argmax_host(q.forward_prefill(prompt))
    t_qprefill = time.perf_counter() - t0
    t_qdecode, tok = timed_decode(q, tok, warmup, steps)
    out["q4_0_under_q6_k_lm_head"] = {"prefill_tok_per_s": len(prompt) / t_qprefill, "decode_tok_per_s": steps / t_qdecode,
                                      "decode_launches_per_token": q.decode_launches, "weights_bytes": int(qblob.size)}
    q.close()
    return out


def ops_table(fh, reps=10):
    """The isolated kernels at the sizes of the benchmark configurations (GEMV and GEMM at Llama-3.2-1B projection
    shapes, prefill attention at 801/1501/3001 tokens, decode attention over 900/2250/8192-token caches), `reps` calls
    each in a fixed order, timed with events on the stream the ops launch on.  An op-level call quantises its f32
    activations first, so its wall time is that of two kernels; a kernel trace of this mode gives each kernel alone."""
    import numpy as np
    import torch
    ops = fh.ops
    rows = []

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / reps

    shapes = [(2048, 2048), (2048, 512), (2048, 8192), (8192, 2048), (2048, 128256)]
    for wd, name in ((fh.Q8_0, "Q8_0"), (fh.Q4_0, "Q4_0")):
        bpb = 34 if wd == fh.Q8_0 else 18
        for K, N in shapes:
            w = ops.QWeight(wd, ops.quantize_weights(wd, fh.synth.normal(K + N, N * K, 0.02)), K, N)
            x = torch.from_numpy(fh.synth.normal(7, K, 1.0)).cuda()
            us = timed(lambda: ops.matmul_vec_q(w, x))
            rows.append({"op": "gemv", "fmt": name, "K": K, "N": N, "us_per_call": round(us, 2),
                         "weight_bytes": N * (K // 32) * bpb})
            if (K, N) == (2048, 8192):      # the reference's x86 arithmetic (f32 activations, sequential row sums) on the same matrix
                us = timed(lambda: ops.matmul_vec_q_portable(w, x))
                rows.append({"op": "gemv_portable_dot", "fmt": name, "K": K, "N": N, "us_per_call": round(us, 2),
                             "weight_bytes": N * (K // 32) * bpb})
            if N <= 8192:
                for M in (352, 902, 1603, 2502):
                    xm = torch.from_numpy(fh.synth.normal(8, M * K, 1.0).reshape(M, K)).cuda()
                    us = timed(lambda: ops.matmul_mat_q(w, xm))
                    rows.append({"op": "gemm", "fmt": name, "M": M, "K": K, "N": N, "us_per_call": round(us, 2),
                                 "int8_ops": 2 * M * K * N})
            w.close()
    # K-quant GEMVs (matmul_vec_q4_k / matmul_vec_q6_k): random super-blocks with sane fp16 scales
    rng = np.random.default_rng(5)
    for ty, name, sbb in ((fh.Q4_K, "Q4_K", 144), (fh.Q6_K, "Q6_K", 210)):
        for K, N in ((2048, 8192), (8192, 2048), (2048, 128256)):
            raw = rng.integers(0, 256, (N * K // 256, sbb), dtype=np.uint8)
            for off in ((0, 2) if ty == fh.Q4_K else (208,)):
                raw[:, off:off + 2] = rng.normal(0, 0.05, raw.shape[0]).astype(np.float16).view(np.uint8).reshape(-1, 2)
            w = ops.QWeight(ty, raw.reshape(-1), K, N)
            x = torch.from_numpy(fh.synth.normal(7, K, 1.0)).cuda()
            us = timed(lambda: ops.matmul_vec_q(w, x))
            rows.append({"op": "gemv", "fmt": name, "K": K, "N": N, "us_per_call": round(us, 2), "weight_bytes": N * (K // 256) * sbb})
            w.close()
    for heads, kvh, hd in ((32, 8, 64), (32, 32, 96)):
        for seq in (801, 1501, 3001):
            q = torch.from_numpy(fh.synth.normal(9, seq * heads * hd, 1.0).reshape(seq, heads * hd)).cuda()
            k = torch.from_numpy(fh.synth.normal(10, seq * kvh * hd, 1.0).reshape(seq, kvh * hd)).cuda().half().view(torch.int16)
            v = torch.from_numpy(fh.synth.normal(11, seq * kvh * hd, 1.0).reshape(seq, kvh * hd)).cuda().half().view(torch.int16)
            us = timed(lambda: ops.attention_flash_batch(q, k, v, 0, heads, kvh, hd))
            rows.append({"op": "attention_prefill", "heads": heads, "kv_heads": kvh, "head_dim": hd, "seq": seq,
                         "us_per_call": round(us, 2), "flops": 4 * heads * hd * seq * (seq + 1) // 2})
        for seq in (900, 2250, 8192):
            q1 = torch.from_numpy(fh.synth.normal(12, heads * hd, 1.0)).cuda()
            k = torch.from_numpy(fh.synth.normal(13, seq * kvh * hd, 1.0).reshape(seq, kvh * hd)).cuda().half().view(torch.int16)
            v = torch.from_numpy(fh.synth.normal(14, seq * kvh * hd, 1.0).reshape(seq, kvh * hd)).cuda().half().view(torch.int16)
            us = timed(lambda: ops.attention_flash(q1, k, v, seq, heads, kvh, hd))
            rows.append({"op": "attention_decode", "heads": heads, "kv_heads": kvh, "head_dim": hd, "cache": seq,
                         "us_per_call": round(us, 2), "kv_bytes": 2 * seq * kvh * hd * 2})
    # sliding-window attention: the Llama-3.2-1B head shape with a 1024-position window and the Mistral-7B head shape
    # (32 / 8 heads of 128) with its 4096-position window
    for heads, kvh, hd, seq, window in ((32, 8, 64, 3001, 1024), (32, 8, 128, 8192, 4096)):
        q = torch.from_numpy(fh.synth.normal(15, seq * heads * hd, 1.0).reshape(seq, heads * hd)).cuda()
        k = torch.from_numpy(fh.synth.normal(16, seq * kvh * hd, 1.0).reshape(seq, kvh * hd)).cuda().half().view(torch.int16)
        v = torch.from_numpy(fh.synth.normal(17, seq * kvh * hd, 1.0).reshape(seq, kvh * hd)).cuda().half().view(torch.int16)
        pairs = sum(min(p + 1, window) for p in range(seq))
        for w, name in ((window, "attention_prefill_sliding"), (0, "attention_prefill")):
            us = timed((lambda: ops.attention_sliding_batch(q, k, v, 0, window, heads, kvh, hd)) if w else
                       (lambda: ops.attention_flash_batch(q, k, v, 0, heads, kvh, hd)))
            rows.append({"op": name, "heads": heads, "kv_heads": kvh, "head_dim": hd, "seq": seq, "window": w,
                         "us_per_call": round(us, 2), "flops": 4 * heads * hd * (pairs if w else seq * (seq + 1) // 2)})
        q1 = q[seq - 1].contiguous()
        for w, name in ((window, "attention_decode_sliding"), (0, "attention_decode")):
            us = timed((lambda: ops.attention_sliding(q1, k, v, seq, window, heads, kvh, hd)) if w else
                       (lambda: ops.attention_flash(q1, k, v, seq, heads, kvh, hd)))
            rows.append({"op": name, "heads": heads, "kv_heads": kvh, "head_dim": hd, "cache": seq, "window": w,
                         "us_per_call": round(us, 2), "kv_bytes": 2 * (min(seq, w) if w else seq) * kvh * hd * 2})
    print(json.dumps({"ops_table": rows, "reps": reps}))


def main():
    global PROMPT_TOKENS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gguf", action="store_true", help="create the model from the weights blob instead of from a GGUF file")
    ap.add_argument("--no-alt", action="store_true", help="skip the second model that measures the kernel-sequence decode step")
    ap.add_argument("--no-exact", action="store_true",
                    help="skip the third model that measures the exact mode and the fast mode's distance from it")
    ap.add_argument("--no-kquant", action="store_true", help="skip the Q4_K_M-recipe model of the same shape")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy kernel (known HBM traffic, for scaling counter readings)")
    ap.add_argument("--model", choices=("llama32_1b", "llama32_3b", "smollm2_135m", "llama31_8b", "qwen25_1p5b", "mistral_7b", "phi3_mini", "qwen25_14b"), default="llama32_1b",
                    help="shape of the synthetic model (default: the one the headline metric is quoted on)")
    ap.add_argument("--format", choices=("q8_0", "q4_0"), default="q8_0", help="weight format (default: the headline's)")
    ap.add_argument("--prompt-tokens", type=int, default=PROMPT_TOKENS,
                    help="length of the prompt (default: the 2502 tokens the metric is quoted on); the cache is sized to fit")
    ap.add_argument("--ops-table", action="store_true",
                    help="instead of the model benchmark, run the isolated kernels at the benchmark configurations' sizes")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU; --gpus must be 1 (no multi-GPU path exists to run)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    fh = load_package()
    fh.require_gpu()
    if args.ops_table:
        ops_table(fh)
        return
    wd = fh.Q8_0 if args.format == "q8_0" else fh.Q4_0
    PROMPT_TOKENS = args.prompt_tokens
    cfg = getattr(fh.synth, args.model)(wd, max_seq=max(4096, (PROMPT_TOKENS + max(2 * (args.warmup + args.steps), DIVERGENCE_STEPS) + 16 + 1023) // 1024 * 1024))
    headline = args.model == "llama32_1b" and args.format == "q8_0" and PROMPT_TOKENS == 2502
    model_name = {"llama32_1b": "Llama-3.2-1B", "llama32_3b": "Llama-3.2-3B", "smollm2_135m": "SmolLM2-135M", "llama31_8b": "Llama-3.1-8B",
                  "qwen25_1p5b": "Qwen2.5-1.5B", "mistral_7b": "Mistral-7B (sliding window 4096)", "phi3_mini": "Phi-3-mini", "qwen25_14b": "Qwen2.5-14B"}[args.model]
    t0 = time.perf_counter()
    blob = fh.synth.make_weights_blob(cfg, seed=args.seed, threads=16)
    t_gen = time.perf_counter() - t0
    # The model arrives the way a user's does: as a GGUF file that the library parses, converts and uploads
    # (--no-gguf: hand the weights blob over directly).
    gguf_info = None
    if args.no_gguf:
        t0 = time.perf_counter()
        model = fh.HipModel(cfg, blob)
        t_load = time.perf_counter() - t0
    else:
        import tempfile
        with tempfile.TemporaryDirectory() as tmp:
            path = os.path.join(tmp, "model.gguf")
            t0 = time.perf_counter()
            fh.gguf.model_to_gguf(cfg, blob, tied=True, path=path)
            t_write = time.perf_counter() - t0
            nbytes = os.path.getsize(path)
            t0 = time.perf_counter()
            model = fh.HipModel.from_gguf(path, max_seq=cfg["max_seq"])
            t_load = time.perf_counter() - t0
        assert {k: model.config[k] for k in cfg if k not in ("rms_eps", "rope_theta")} == {k: cfg[k] for k in cfg if k not in ("rms_eps", "rope_theta")}
        gguf_info = {"file_bytes": nbytes, "write_s": round(t_write, 2), "parse_convert_upload_s": round(t_load, 2),
                     "GB_per_s": round(nbytes / t_load / 1e9, 2)}
    prompt = fh.synth.uniform_ids(args.seed + 1, PROMPT_TOKENS, cfg["vocab"])

    # ---- prefill: one warm-up pass, then timed
    model.forward_prefill_batch(prompt)
    model.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    logits = model.forward_prefill(prompt)
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    tok = fh.ops.argmax_host(logits)

    # ---- decode at context ~2502: W warm-up steps, K timed steps
    t_decode, tok = timed_decode(model, tok, args.warmup, args.steps)
    roofline, stage_us = decode_profile(fh, model, cfg, tok, PROMPT_TOKENS + args.warmup + args.steps)
    if not headline:
        roofline["traffic"] = None        # the counter runs were made on the headline workload

    # ---- prefill kernels (GEMM / attention) from prefill_profile
    model.reset()
    pp = model.prefill_profile(prompt)
    gemm_flops, attn_flops = prefill_flops(cfg, PROMPT_TOKENS)
    gemm_ms = sum(pp[s][0] for s in ("qkv_matmul", "o_matmul", "gate_up_matmul", "down_matmul"))
    attn_ms = pp["attention"][0]

    # ---- short-context decode for reference (64-token style run of the reference's decode benchmark)
    model.reset()
    tok2 = fh.ops.argmax_host(model.forward_prefill(prompt[:32]))
    t_decode_short, _ = timed_decode(model, tok2, 4, args.steps)
    path = ("one resident kernel per token" if model.decode_launches == 1 else
            f"{model.decode_launches} launches of the resident kernel per token (34 layers each)"
            if model.decode_launches <= (cfg["layers"] + 33) // 34 else f"{model.decode_launches} kernels per token (graph replay)")

    # ---- the fast mode's greedy tokens and logits over DIVERGENCE_STEPS steps, for the comparison with the exact mode
    fast_tokens, fast_logits = (None, None) if args.no_exact else greedy_with_logits(fh, model, prompt, DIVERGENCE_STEPS)

    # ---- the reference's default loop: greedy with repeat penalty 1.1 over every token fed (project.rs:607-611, 742-744)
    model.reset()
    model.set_repeat_penalty(1.1)
    tok3 = fh.ops.argmax_host(model.forward_prefill(prompt))
    t_decode_pen, _ = timed_decode(model, tok3, args.warmup, args.steps)

    # ---- the same prompt and decode steps over a PAGED cache: pages of 64 rows in a shuffled order
    model.reset()
    model.set_repeat_penalty(1.0)
    n_pages = cfg["max_seq"] // 64
    model.set_kv_pages(64, np.random.default_rng(args.seed).permutation(n_pages).astype(np.uint32))
    model.forward_prefill_batch(prompt)
    model.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    logits_paged = model.forward_prefill(prompt)
    torch.cuda.synchronize()
    t_prefill_paged = time.perf_counter() - t0
    paged_same = bool(np.array_equal(logits_paged.view(np.uint32), logits.view(np.uint32)))
    t_decode_paged, _ = timed_decode(model, fh.ops.argmax_host(logits_paged), args.warmup, args.steps)
    model.close()

    # ---- the other decode path, for comparison: the step as a sequence of kernels
    alt = None
    if not args.no_alt and os.environ.get("FORGE_HIP_PERSIST", "1") != "0":
        os.environ["FORGE_HIP_PERSIST"] = "0"
        try:
            m2 = fh.HipModel(cfg, blob)
            tk = fh.ops.argmax_host(m2.forward_prefill(prompt))
            t2, tk = timed_decode(m2, tk, args.warmup, args.steps)
            roof2, stage2 = decode_profile(fh, m2, cfg, tk, PROMPT_TOKENS + args.warmup + args.steps)
            if not headline:
                roof2["traffic"] = None
            alt = {"path": f"{m2.decode_launches} kernels per token (graph replay)", "decode_tok_per_s": args.steps / t2,
                   "roofline": roof2, "decode_stage_us": stage2}
            m2.close()
        finally:
            os.environ["FORGE_HIP_PERSIST"] = "1"
    exact = None if args.no_exact else exact_mode_figures(fh, cfg, blob, prompt, args.warmup, args.steps, fast_tokens, fast_logits)
    kquant = None
    if not args.no_kquant and cfg["hidden"] % 256 == 0 and cfg["inter"] % 256 == 0 and not cfg.get("sliding_window") and not (cfg.get("flags", 0) & 2):
        kquant = kquant_model_figures(fh, cfg, prompt, args.warmup, args.steps, args.seed)
    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").fill_(1.0)     # 1 GiB
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)                                                                 # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    out = {
        "metric": f"decode tok/s ({model_name} {args.format.upper()}, 1 GPU)",
        "value": args.steps / t_decode,
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": t_decode / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 block dots (exact int32) + f32 combine; fp16 KV",
        "data": "synthetic",
        "config": {"workload": f"{model_name} shape, {args.format.upper()}, random-init seed {args.seed}: {PROMPT_TOKENS}-token prompt, "
                               f"then greedy decode at that context", "prompt_tokens": PROMPT_TOKENS,
                   "decode_context": PROMPT_TOKENS + args.warmup, "mode": "fast (MFMA prefill, split-seq decode attention)",
                   "decode_path": path},
        "prefill_tok_per_s": PROMPT_TOKENS / t_prefill,
        "prefill_ms": t_prefill * 1e3,
        "decode_tok_per_s_short_context": args.steps / t_decode_short,
        "decode_tok_per_s_repeat_penalty_1.1": args.steps / t_decode_pen,
        "paged_kv_cache": {"page_rows": 64, "page_order": "shuffled", "decode_tok_per_s": args.steps / t_decode_paged,
                           "prefill_tok_per_s": PROMPT_TOKENS / t_prefill_paged, "prefill_logits_bit_identical_to_flat_cache": paged_same},
        "decode_weight_stream_GBps_end_to_end": fh.synth.decode_weight_bytes(cfg) * args.steps / t_decode / 1e9,
        "exact_mode": exact,
        "roofline": roofline,
        "prefill_stage_ms": {k: round(v[0], 3) for k, v in pp.items() if v[1]},
        "prefill_rooflines": {
            "gemm": {"bound": "mfma", "achieved": gemm_flops / (gemm_ms * 1e-3) / 1e12, "peak": MFMA_I8_PEAK_TOPS,
                     "unit": "TOP/s (int8)", "frac": gemm_flops / (gemm_ms * 1e-3) / 1e12 / MFMA_I8_PEAK_TOPS, "ms": gemm_ms},
            "attention": {"bound": "mfma", "achieved": attn_flops / (attn_ms * 1e-3) / 1e12, "peak": MFMA_F16_PEAK_TFLOPS,
                          "unit": "TFLOP/s (fp16)", "frac": attn_flops / (attn_ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS,
                          "ms": attn_ms},
        },
        "decode_stage_us": stage_us,
        "kernel_sequence_path": alt,
        "kquant_model": kquant,
        "setup_s": {"generate_weights": round(t_gen, 1), "upload_and_repack": round(t_load, 1)},
        "gguf_load": gguf_info,
    }
    if exact:
        # the mode whose greedy tokens are identical to the reference's CPU path, beside the headline's
        out["config"]["token_identical_mode"] = {"flag": "FORGE_HIP_FLAG_EXACT", "decode_tok_per_s": exact["decode_tok_per_s"],
                                                 "prefill_tok_per_s": exact["prefill_tok_per_s"], "decode_path": exact["decode_path"]}
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(fh, cfg, blob, prompt)
        out["cpu_baseline"] = cpu
        # GPU over the CPU port on the same workload (vs_baseline stays null: no published figure exists for this metric)
        out["gpu_over_cpu_port"] = {"decode_vs_x86_arithmetic": out["value"] / cpu["value"],
                                    "decode_vs_aarch64_arithmetic": out["value"] / cpu["variant_a"]["decode_tok_per_s"],
                                    "prefill_vs_aarch64_arithmetic": out["prefill_tok_per_s"] / cpu["variant_a"]["prefill_tok_per_s"]}
        if exact:
            out["gpu_over_cpu_port"]["exact_mode_decode_vs_aarch64_arithmetic"] = exact["decode_tok_per_s"] / cpu["variant_a"]["decode_tok_per_s"]
    print(json.dumps(out))


if __name__ == "__main__":
    main()
