"""Writes tests/golden/reference_vectors.json: the inputs and expected outputs that the reference's own unit tests hold
for the hot path, as data.  Nothing of the reference is imported or run; every entry was read from the test it cites
and is written down here as numbers (or, where the reference builds its input by a formula, as that formula's
parameters, which the loader expands).  Run from the repository root:  python tests/golden/make_reference_vectors.py"""
import json
import os

vectors = {
    "f16_to_f32": {   # forgellm-frontend/src/weight_loader.rs:2469-2491
        "cite": "weight_loader.rs:2469-2491",
        "cases": [[0x0000, "0.0"], [0x3C00, "1.0"], [0xBC00, "-1.0"], [0x3800, "0.5"], [0x4000, "2.0"],
                  [0x7C00, "inf"], [0x7E00, "nan"], [0x8000, "-0.0"]],
    },
    "f32_to_f16_flush": {   # forgellm-codegen-cpu/src/emit.rs:1471-1474: below 2^-24 the result is a signed zero
        "cite": "emit.rs:1460-1495",
        "cases": [["2^-24", 0x0001], ["2^-25", 0x0000], ["1.5*2^-25", 0x0000], ["-1.5*2^-25", 0x8000], ["1.5*2^-24", 0x0002]],
    },
    "dequant_q8_0": {   # weight_loader.rs:3209-3242
        "cite": "weight_loader.rs:3209-3242",
        "cases": [
            {"scale_bits": 0x3C00, "codes": list(range(32)), "expect": [float(i) for i in range(32)]},
            {"scale_bits": 0x4000, "codes": [i if i % 2 == 0 else -i for i in range(32)],
             "expect": [2.0 * (i if i % 2 == 0 else -i) for i in range(32)]},
            {"scale_bits": 0x0000, "codes": [127] * 32, "expect": [0.0] * 32},
        ],
    },
    "dequant_q4_0": {   # weight_loader.rs:3696-3759: byte j = element j (low nibble) and j+16 (high nibble), minus 8
        "cite": "weight_loader.rs:3696-3759",
        "cases": [
            {"scale_bits": 0x3C00, "bytes": [0x88] * 16, "expect": [0.0] * 32},
            {"scale_bits": 0x4000, "bytes": [(j % 16) | (((15 - j) % 16) << 4) for j in range(16)],
             "expect": [2.0 * (j - 8) for j in range(16)] + [2.0 * ((15 - j) - 8) for j in range(16)]},
        ],
    },
    "quantize_q8_0_round_trip": {   # weight_loader.rs:3002-3028: a ramp survives within 0.02, zeros stay zeros
        "cite": "weight_loader.rs:3002-3028",
        "input": {"formula": "(i - 32) * 0.05", "n": 64}, "max_abs_error": 0.02, "bytes": 68,
    },
    "quantize_q4_0_invariants": {   # weight_loader.rs:3340-3379, 3761-3796
        "cite": "weight_loader.rs:3340-3379, 3761-3796",
        "input": {"formula": "(i - 32) * 0.1", "n": 64}, "bytes": 36, "error_bound": "absmax/8 + 0.01 per block",
    },
    "kv_int8_quantiser": {   # emit.rs:6813-6852
        "cite": "emit.rs:6813-6852",
        "input": {"formula": "((i * 7 + 3) * 0.1 - 3.0) * 0.5", "n": 64}, "scale": "absmax/127", "error_bound": "scale",
    },
    "rms_norm": {   # forgellm-runtime/src/kernels.rs:396-413: x / sqrt(mean(x^2) + eps) with unit weights
        "cite": "kernels.rs:396-413", "x": [1.0, 2.0, 3.0, 4.0], "weight": [1.0, 1.0, 1.0, 1.0], "eps": 1e-5,
        "expect": [0.36514813, 0.73029625, 1.0954444, 1.4605925], "atol": 1e-5,   # the test's closed form, evaluated; its tolerance
    },
    "silu_mul": {   # interpreter.rs:245-303
        "cite": "interpreter.rs:245-303", "gate": [1.0, -1.0, 0.0], "up": [1.0, 1.0, 5.0],
        "expect": [0.7311, -0.2689, 0.0], "atol": 1e-4,
    },
    "softmax": {   # interpreter.rs:245-303: sums to one, increasing
        "cite": "interpreter.rs:245-303", "x": [1.0, 2.0, 3.0], "expect": [0.09003057, 0.24472848, 0.66524094], "atol": 1e-6,
    },
    "attention": {   # emit.rs:6687-6741: deterministic inputs, flash == standard within 1e-4
        "cite": "emit.rs:6687-6741", "head_dim": 8, "heads": 3, "kv_heads": 1, "seq_lens": [5, 64, 70, 128, 200],
        "q": {"formula": "((i * 7 + 3) * 0.1 - 1.0) * 0.5"}, "k": {"formula": "((i * 11 + 5) * 0.07 - 1.0) * 0.3"},
        "v": {"formula": "((i * 13 + 7) * 0.05 - 0.5) * 0.4"}, "tolerance": 1e-4,
    },
    "argmax": {   # forgellm-cli project.rs:501-503: Iterator::max_by keeps the LAST maximum
        "cite": "project.rs:501-503",
        "cases": [[[1, 5, 3, 5, 2], 3], [[7, 7, 7], 2], [[-1, -3], 0], [[0.1, 0.9, 0.3], 1]],
    },
}

if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")
    with open(path, "w") as f:
        json.dump(vectors, f, indent=1)
    print("wrote", path)
