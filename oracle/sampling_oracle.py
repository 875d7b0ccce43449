"""TEST INFRASTRUCTURE ONLY — CPU restatement of the sampler of the generated main.rs
(crates/forgellm-codegen-cpu/src/project.rs:501-555: argmax, apply_repeat_penalty, sample) and of its generation loop
(project.rs:714-751), in numpy float32.  Nothing the product ships imports this file.

Every step is an IEEE float32 operation in the reference's order: `np.cumsum` on float32 adds sequentially (it is the
running sum the Rust loops keep), divisions are elementwise, `exp` is the C library's expf through oracle.expf.

Pinned by: the xorshift64 recurrence against Python's unbounded integers; apply_repeat_penalty against the known
answers the reference's runtime crate holds for the same formula (crates/forgellm-runtime/src/sampling.rs:219-237);
properties the mathematics fixes (temperature -> argmax, top_k = 1, the chosen index brackets r in a float64 CDF,
empirical frequencies against softmax probabilities).  No reference test executes `sample` itself: beyond those
properties its parity is unpinned, and the order among exactly equal probabilities is open in the reference
(`sort_unstable_by`); here the lower index sorts first.
"""
import numpy as np

F = np.float32
MASK = (1 << 64) - 1


def argmax(logits) -> int:
    v = np.asarray(logits)
    return int(v.size - 1 - np.argmax(v[::-1]))          # max_by keeps the last maximum


def apply_repeat_penalty(logits, recent, penalty) -> None:
    p = F(penalty)
    if p <= F(1.0):
        return
    for t in recent:
        if t < logits.size:
            logits[t] = logits[t] / p if logits[t] > F(0.0) else logits[t] * p


def xorshift(state: int) -> int:
    state ^= (state << 13) & MASK
    state ^= state >> 7
    state ^= (state << 17) & MASK
    return state


def u64_to_f32(s: int):
    """`s as f32` for a u64: round to nearest, ties to even, done on integers (no detour through float64)."""
    nb = s.bit_length()
    if nb <= 24:
        return F(s)
    shift = nb - 24
    q, rem, half = s >> shift, s & ((1 << shift) - 1), 1 << (shift - 1)
    if rem > half or (rem == half and (q & 1)):
        q += 1
    return F(q) * F(2.0 ** shift)


def sample(oracle, logits, temperature, top_k, top_p, state):
    """Returns (token, new state); overwrites `logits` (float32) with the final probabilities."""
    l = logits
    n = l.size
    if F(temperature) <= F(0.0):
        return argmax(l), state
    l /= F(temperature)
    mx = l.max()
    l[:] = oracle.expf(l - mx)
    l /= np.cumsum(l, dtype=F)[-1]
    order = np.argsort(-l, kind="stable")
    if 0 < top_k < n:
        l[order[top_k:]] = F(0.0)
    if F(0.0) < F(top_p) < F(1.0):
        cs = np.cumsum(l[order], dtype=F)
        l[order[cs > F(top_p)]] = F(0.0)
    s = np.cumsum(l, dtype=F)[-1]
    if s > F(0.0):
        l /= s
    state = xorshift(state)
    r = u64_to_f32(state) / u64_to_f32(MASK)                # u64::MAX as f32 = 2^64
    cs = np.cumsum(l, dtype=F)
    hit = np.nonzero(cs >= r)[0]
    return (int(hit[0]) if hit.size else n - 1), state


def generate(oracle, model, prompt, max_tokens, temperature, top_k, top_p, repeat_penalty, seed, eos=()):
    """project.rs:714-751 over an oracle.Model."""
    logits = np.array(model.prefill_batched(prompt), dtype=F)
    nxt, rng = sample(oracle, logits, temperature, top_k, top_p, seed)
    recent = [int(t) for t in prompt]
    out = []
    for _ in range(max_tokens):
        if nxt in eos:
            break
        out.append(nxt)
        recent.append(nxt)
        logits = np.array(model.forward(nxt), dtype=F)
        apply_repeat_penalty(logits, recent, repeat_penalty)
        nxt, rng = sample(oracle, logits, temperature, top_k, top_p, rng)
    return out
