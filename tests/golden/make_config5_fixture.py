"""Writes tests/golden/config5_llama32_3b_q8.json: what the CPU oracle (oracle/forge_oracle.cpp, arithmetic variant A,
fp16 cache) produces for the Llama-3.2-3B-shape workload at full size -- 28 layers, a 2500-token random-id prompt through
`forward_prefill_batched`, then 128 greedy steps through `forward`.

The oracle needs about a quarter of an hour on 8 cores for this, too long for a test, so it is run once here and the GPU
test holds the library's exact mode to the numbers in the file: the 128 token ids, the SHA-256 of the raw f32 bits of the
prefill logits and of the logits behind the last token, and per step the margin between the two largest logits (how close
each greedy choice was).  Model and prompt are regenerated from the seeds in the file (forge-llm_amd/synth.py).

    python tests/golden/make_config5_fixture.py            # full size
    python tests/golden/make_config5_fixture.py --layers 2 --prompt 300 --steps 8 --out /tmp/small.json   # dry run
"""
import argparse
import hashlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

WEIGHT_SEED, PROMPT_SEED = 5, 55


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a, np.float32).tobytes()).hexdigest()


def top2_margin(logits):
    part = np.partition(logits, -2)[-2:]
    return float(part[1] - part[0])


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--layers", type=int, default=28)
    ap.add_argument("--prompt", type=int, default=2500)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--out", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "config5_llama32_3b_q8.json"))
    args = ap.parse_args()

    from conftest import load_package
    fh = load_package()
    from oracle import oracle

    cfg = fh.synth.llama32_3b(8, max_seq=4096)
    cfg["layers"] = args.layers
    t0 = time.time()
    blob = fh.synth.make_weights_blob(cfg, seed=WEIGHT_SEED, threads=os.cpu_count() or 8)
    prompt = fh.synth.uniform_ids(PROMPT_SEED, args.prompt, cfg["vocab"])
    print(f"weights: {blob.size / 1e9:.2f} GB in {time.time() - t0:.0f} s", flush=True)

    om = oracle.Model(cfg, blob, oracle.VARIANT_A, oracle.KV_F16)
    t0 = time.time()
    logits = om.prefill_batched(prompt)
    print(f"prefill of {args.prompt} tokens: {time.time() - t0:.0f} s", flush=True)
    prefill_sha, prefill_top = sha(logits), [int(i) for i in np.argsort(logits)[-5:][::-1]]
    tokens, margins = [], []
    t0 = time.time()
    for step in range(args.steps):
        tokens.append(oracle.argmax(logits))
        margins.append(top2_margin(logits))
        if step + 1 < args.steps:
            logits = om.forward(tokens[-1])
        if step % 16 == 0:
            print(f"step {step}: token {tokens[-1]} margin {margins[-1]:.4f} ({time.time() - t0:.0f} s)", flush=True)
    out = {
        "what": "CPU oracle, variant A (int8 activation blocks), fp16 KV cache: greedy tokens of the Llama-3.2-3B-shape workload",
        "made_by": "tests/golden/make_config5_fixture.py",
        "config": {k: (float(v) if isinstance(v, float) else int(v)) for k, v in cfg.items()},
        "weight_seed": WEIGHT_SEED, "prompt_seed": PROMPT_SEED, "prompt_tokens": args.prompt,
        "prompt_head": [int(t) for t in prompt[:8]],
        "prefill_logits_sha256": prefill_sha, "prefill_top5": prefill_top,
        "tokens": tokens, "top2_margin": [round(m, 6) for m in margins],
        "last_logits_sha256": sha(logits),           # the logits whose argmax is tokens[-1]
        "last_logits_absmax": float(np.abs(logits).max()),
    }
    with open(args.out, "w") as f:
        json.dump(out, f, indent=1)
        f.write("\n")
    print("wrote", args.out)


if __name__ == "__main__":
    main()
