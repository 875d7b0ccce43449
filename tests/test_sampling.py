"""The sampler of the generated main.rs (project.rs:501-555) and its loop (project.rs:714-751): the library's host
functions against the numpy restatement in oracle/sampling_oracle.py, both against what the mathematics fixes, and the
device-side repeat penalty of forward_greedy against the host path."""
import numpy as np
import pytest

Q8, Q4 = 8, 2
EXACT = 1


@pytest.fixture(scope="module")
def so():
    from oracle import sampling_oracle
    return sampling_oracle


def logits_of(fh, seed, n, spread=3.0):
    return (fh.synth.normal(seed, n, 1.0) * spread).astype(np.float32)


# ---------------- pins of the oracle and of the library alike ----------------
def test_xorshift_recurrence_against_big_integers(fh, so):
    state = 0xdeadbeef12345678                      # the reference's default seed, project.rs:612
    lib_state = state
    for _ in range(50):
        x = state
        x ^= (x << 13) % (1 << 64)
        x ^= x >> 7
        x ^= (x << 17) % (1 << 64)
        state = so.xorshift(state)
        assert state == x
        _, lib_state = fh.ops.sample(np.array([0.0, 1.0], np.float32), 1.0, 0, 1.0, lib_state)
        assert lib_state == x
    # state 0 stays 0 (r = 0: the first index with cumsum >= 0 is index 0)
    assert fh.ops.sample(np.array([1.0, 2.0, 3.0], np.float32), 1.0, 0, 1.0, 0) == (0, 0)


def test_u64_to_f32_rounds_like_a_direct_conversion(so):
    for s in (0, 1, (1 << 24) - 1, 1 << 24, (1 << 24) + 1, (1 << 25) + 2, (1 << 25) + 6, (1 << 64) - 1, (1 << 63) + (1 << 39),
              (1 << 63) + (1 << 39) + 1, 0x8000008000000000, 0x8000018000000000, 0xdeadbeef12345678):
        # exact rational comparison: the result is the nearest float32, ties to even
        got = int(so.u64_to_f32(s))
        ulp = 1 << max(0, s.bit_length() - 24)
        assert abs(got - s) * 2 <= ulp
        if abs(got - s) * 2 == ulp:
            assert (got // ulp) % 2 == 0


def test_repeat_penalty_known_answers_of_the_reference(fh, so):
    """crates/forgellm-runtime/src/sampling.rs:219-237 holds these for the same formula."""
    for fn in (lambda l, r, p: fh.ops.apply_repeat_penalty(l, r, p), so.apply_repeat_penalty):
        l = np.array([0.5, 0.9, 0.3], np.float32)
        fn(l, [1], 2.0)
        assert abs(l[1] - 0.45) < 1e-6 and abs(l[0] - 0.5) < 1e-6 and abs(l[2] - 0.3) < 1e-6
        l = np.array([-0.5, 0.5, -0.3], np.float32)
        fn(l, [0, 2], 2.0)
        assert abs(l[0] - (-1.0)) < 1e-6 and abs(l[2] - (-0.6)) < 1e-6 and l[1] == np.float32(0.5)
        # once per occurrence, out-of-range ids ignored, penalty <= 1 is a no-op (project.rs:506)
        l = np.array([8.0, -1.0], np.float32)
        fn(l, [0, 0, 0, 7, 1, 1], 2.0)
        assert l.tolist() == [1.0, -4.0]
        l = np.array([8.0, -1.0], np.float32)
        fn(l, [0, 1], 1.0)
        fn(l, [0, 1], 0.5)
        assert l.tolist() == [8.0, -1.0]
        # zero is "not > 0": multiplied, stays zero
        l = np.array([0.0], np.float32)
        fn(l, [0], 1.5)
        assert l[0] == 0.0


def test_repeat_penalty_is_successive_divisions_not_a_power(fh, so):
    l0 = logits_of(fh, 3, 64)
    recent = [int(t) for t in fh.synth.uniform_ids(4, 500, 64)]
    a, b = l0.copy(), l0.copy()
    fh.ops.apply_repeat_penalty(a, recent, 1.1)
    so.apply_repeat_penalty(b, recent, 1.1)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    c = np.bincount(recent, minlength=64)
    p = l0.astype(np.float64) * np.where(l0 > 0, 1.1 ** -c.astype(np.float64), 1.1 ** c.astype(np.float64))
    assert np.allclose(a, p, rtol=1e-5)
    assert not np.array_equal(a, p.astype(np.float32))      # the f32 chain is its own sequence of roundings


@pytest.mark.parametrize("n", [1, 2, 33, 1000])
def test_greedy_and_degenerate_settings(fh, oracle, so, n):
    l = logits_of(fh, 10 + n, n)
    l[n // 2] = l.max()                                     # a tie: the last maximum wins
    want = so.argmax(l)
    assert want == int(np.flatnonzero(l == l.max())[-1])
    for temp in (0.0, -1.0):
        assert fh.ops.sample(l.copy(), temp, 0, 0.9, 123) == (want, 123)
        assert so.sample(oracle, l.copy(), temp, 0, 0.9, 123) == (want, 123)
    # top_k = 1 with top_p off: only the most probable entry survives (ties: the lower index sorts first)
    first = int(np.flatnonzero(l == l.max())[0])
    for seed in (1, 2, 3):
        tok, _ = fh.ops.sample(l.copy(), 0.7, 1, 1.0, seed)
        assert tok == (first if n > 1 else 0)


@pytest.mark.parametrize("temp,top_k,top_p", [(1.0, 0, 1.0), (0.7, 0, 1.0), (0.8, 40, 1.0), (1.0, 0, 0.9), (0.7, 40, 0.9), (1.3, 5, 0.5),
                                               (0.5, 0, 0.3), (2.0, 1000, 0.99)])
def test_sample_equals_oracle_and_brackets_r(fh, oracle, so, temp, top_k, top_p):
    n = 997
    state_l = state_o = 0xdeadbeef12345678
    for trial in range(40):
        l = logits_of(fh, 100 + trial, n)
        a, b = l.copy(), l.copy()
        tok_l, state_l = fh.ops.sample(a, temp, top_k, top_p, state_l)
        tok_o, state_o = so.sample(oracle, b, temp, top_k, top_p, state_o)
        assert (tok_l, state_l) == (tok_o, state_o)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))      # the final probabilities too
        # what is left is a distribution over the allowed set, and the choice brackets r in a float64 CDF
        p = a.astype(np.float64)
        kept = int((p > 0).sum())
        if kept:
            assert abs(p.sum() - 1.0) < 1e-4
            if top_k:
                assert kept <= top_k
            r = float(so.u64_to_f32(state_l) / so.u64_to_f32((1 << 64) - 1))
            cdf = np.cumsum(p)
            assert cdf[tok_l] >= r - 1e-4 and (tok_l == 0 or cdf[tok_l - 1] <= r + 1e-4)
            assert p[tok_l] > 0 or r <= 1e-4
        else:
            # top-p dropped everything (the most probable entry alone exceeds it): the reference returns the last index
            assert tok_l == n - 1


def test_top_p_drops_the_entry_that_crosses_the_threshold(fh, oracle, so):
    """project.rs:535-540 zeroes every entry from the first whose running sum exceeds top_p, that entry included."""
    l = np.log(np.array([0.5, 0.3, 0.15, 0.05], np.float32))
    a = l.copy()
    fh.ops.sample(a, 1.0, 0, 0.9, 77)
    assert a[3] == 0 and a[2] == 0 and a[0] > 0 and a[1] > 0        # 0.5, 0.8 stay; 0.95 > 0.9 goes
    assert abs(float(a[0]) - 0.625) < 1e-6
    b = l.copy()
    tok, _ = fh.ops.sample(b, 1.0, 0, 0.4, 77)                          # 0.5 > 0.4: nothing survives
    assert not b.any() and tok == 3
    assert so.sample(oracle, l.copy(), 1.0, 0, 0.4, 77)[0] == 3


def test_frequencies_follow_the_softmax(fh):
    l = np.array([2.0, 1.0, 0.0, -1.0, 0.5], np.float32)
    p = np.exp(l.astype(np.float64) / 0.8)
    p /= p.sum()
    state, hits, draws = 12345, np.zeros(5), 20000
    for _ in range(draws):
        tok, state = fh.ops.sample(l.copy(), 0.8, 0, 1.0, state)
        hits[tok] += 1
    # five standard deviations of a binomial count
    assert np.all(np.abs(hits - draws * p) < 5 * np.sqrt(draws * p * (1 - p)))


def test_sample_errors(fh):
    with pytest.raises(fh.ForgeHipError):
        fh.ops.sample(np.array([1.0, np.nan], np.float32), 1.0, 0, 1.0, 1)
    with pytest.raises(fh.ForgeHipError):
        fh.ops.sample(np.array([], np.float32), 1.0, 0, 1.0, 1)


# ---------------- device: the penalised greedy step ----------------
@pytest.mark.gpu
@pytest.mark.parametrize("wd,flags", [(Q8, 0), (Q4, 0), (Q8, EXACT)])
def test_greedy_with_repeat_penalty_on_the_device_equals_the_host_path(fh, so, torch_gpu, monkeypatch, wd, flags):
    """forward_greedy with a penalty set == forward + apply_repeat_penalty + argmax on the host, token for token, over a
    prompt with many repeats (each occurrence counts), across a reset, for the resident kernel and the kernel sequence."""
    cfg = fh.synth.tiny(wd, max_seq=640)
    cfg["flags"] = flags
    blob = fh.synth.make_weights_blob(cfg, seed=21)
    prompt = fh.synth.uniform_ids(6, 300, 40)               # 300 tokens out of 40 ids: every id repeats
    for persist in ("1", "0"):
        monkeypatch.setenv("FORGE_HIP_PERSIST", persist)
        dev, host = fh.HipModel(cfg, blob), fh.HipModel(cfg, blob)
        if not flags:
            assert dev.decode_launches == (1 if persist == "1" else dev.decode_launches)
        for penalty in (1.1, 1.7):
            dev.reset(); host.reset()
            dev.set_repeat_penalty(penalty)
            first = fh.ops.argmax_host(dev.forward_prefill(prompt))
            assert first == fh.ops.argmax_host(host.forward_prefill(prompt))
            recent = [int(t) for t in prompt]
            tok_d = tok_h = first
            for step in range(24):
                recent.append(tok_h)
                lg = host.forward(tok_h)
                so.apply_repeat_penalty(lg, recent, penalty)
                tok_h = so.argmax(lg)
                tok_d = dev.forward_greedy(tok_d)
                assert tok_d == tok_h, (persist, penalty, step)
        # the penalty changes the sequence (otherwise this test would prove nothing), and switching it off restores it
        dev.reset(); host.reset()
        dev.set_repeat_penalty(1.0)
        t0 = fh.ops.argmax_host(dev.forward_prefill(prompt))
        host.forward_prefill(prompt)
        plain = [dev.forward_greedy(t0)]
        unpen = [fh.ops.argmax_host(host.forward(t0))]
        for _ in range(23):
            plain.append(dev.forward_greedy(plain[-1]))
            unpen.append(fh.ops.argmax_host(host.forward(unpen[-1])))
        assert plain == unpen
        dev.close(); host.close()


@pytest.mark.gpu
def test_generate_loop_equals_the_oracle_loop(fh, oracle, so, torch_gpu):
    """HipModel.generate (project.rs:714-751 with its defaults: greedy, repeat penalty 1.1) in exact mode against the same
    loop over the CPU oracle: identical tokens; and with a temperature, host sampler on GPU logits against the oracle's."""
    cfg = fh.synth.tiny(Q8, max_seq=640)
    cfg["flags"] = EXACT
    blob = fh.synth.make_weights_blob(cfg, seed=22)
    prompt = fh.synth.uniform_ids(7, 120, 60)
    gm = fh.HipModel(cfg, blob)
    om = oracle.Model(cfg, blob, 0, 1)
    got = gm.generate(prompt, max_tokens=32)
    want = so.generate(oracle, om, prompt, 32, 0.0, 0, 0.9, 1.1, 0xdeadbeef12345678)
    assert got == want and len(got) == 32
    gm.reset(); om.reset()
    got = gm.generate(prompt, max_tokens=24, temperature=0.8, top_k=40, top_p=0.9, repeat_penalty=1.1, seed=42)
    want = so.generate(oracle, om, prompt, 24, 0.8, 40, 0.9, 1.1, 42)
    assert got == want
    # an EOS id stops the loop before it is emitted
    gm.reset()
    assert gm.generate(prompt, max_tokens=32, eos=(got[3],), temperature=0.8, top_k=40, top_p=0.9, seed=42) == got[:3]
    gm.close(); om.close()
