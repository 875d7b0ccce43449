"""GPU parity of the model API (create / forward / forward_prefill_batch / reset) against the
oracle model with variant-A arithmetic and an fp16 KV cache, on seeded synthetic models."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

Q8, Q4 = 8, 2
A, KV_F16 = 0, 1


def close(got, want, rtol=1e-3, atol=1e-3):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    bad = np.abs(got - want) > atol + rtol * np.abs(want)
    assert not bad.any(), f"{bad.sum()} of {bad.size} outside tolerance; max abs err {np.max(np.abs(got - want)):.3e}"


def greedy_oracle(oracle, om, prompt, n):
    logits = om.prefill_batched(prompt)
    out = [oracle.argmax(logits)]
    for _ in range(n - 1):
        out.append(oracle.argmax(om.forward(out[-1])))
    return out


@pytest.mark.parametrize("wd", [Q8, Q4])
def test_tiny_model_logits_and_cache(fh, oracle, torch_gpu, wd):
    cfg = fh.synth.tiny(wdtype=wd, max_seq=640, hidden=256, inter=512, layers=2, heads=4, kv_heads=2, head_dim=64, vocab=1000)
    blob = fh.synth.make_weights_blob(cfg, seed=11)
    toks = fh.synth.uniform_ids(12, 40, cfg["vocab"])
    gm = fh.HipModel(cfg, blob)
    om = oracle.Model(cfg, blob, A, KV_F16)
    # batched prefill: last-token logits and the fp16 cache contents
    gl = gm.forward_prefill(toks)
    ol = om.prefill_batched(toks)
    assert gm.pos == om.pos == 40
    close(gl, ol)
    for layer in range(cfg["layers"]):
        for which in (0, 1):
            got = oracle.f16_to_f32(gm.read_kv(layer, which))
            close(got, om.read_kv(layer, which), rtol=2e-3, atol=2e-3)
    # decode steps continue from the cache
    for t in (3, 999, 0):
        close(gm.forward(t), om.forward(t))
    assert gm.pos == om.pos == 43
    # per-token path from scratch equals the batched path (the reference's consistency claim)
    gm.reset()
    assert gm.pos == 0
    for t in toks:
        last = gm.forward(int(t))
    close(last, gl, rtol=1e-3, atol=1e-3)
    # reset reproduces
    gm.reset()
    again = gm.forward_prefill(toks)
    assert np.array_equal(again, gl)
    # Metal-style signature: fill the cache without logits, then forward(last)
    gm.reset()
    gm.forward_prefill_batch(toks[:-1])
    close(gm.forward(int(toks[-1])), gl)
    gm.close()


def test_forward_greedy_matches_forward_argmax(fh, oracle, torch_gpu):
    cfg = fh.synth.tiny(wdtype=Q8, max_seq=640)
    blob = fh.synth.make_weights_blob(cfg, seed=21)
    gm = fh.HipModel(cfg, blob)
    gm.forward_prefill_batch(fh.synth.uniform_ids(1, 9, cfg["vocab"]))
    logits = gm.forward(5)
    gm.reset()
    gm.forward_prefill_batch(fh.synth.uniform_ids(1, 9, cfg["vocab"]))
    assert gm.forward_greedy(5) == fh.ops.argmax_host(logits) == oracle.argmax(logits)
    gm.close()


def test_error_codes_on_device(fh, torch_gpu):
    cfg = fh.synth.tiny(wdtype=Q8, max_seq=16)
    blob = fh.synth.make_weights_blob(cfg, seed=2)
    gm = fh.HipModel(cfg, blob)
    with pytest.raises(fh.ForgeHipError) as e:
        gm.forward_prefill_batch(np.zeros(17, np.uint32))
    assert e.value.code == fh.ERR_POSITION
    gm.forward_prefill_batch(np.zeros(16, np.uint32))
    with pytest.raises(fh.ForgeHipError) as e:          # cache full (the reference would index out of bounds)
        gm.forward(1)
    assert e.value.code == fh.ERR_POSITION
    gm.reset()
    with pytest.raises(fh.ForgeHipError) as e:
        gm.forward(cfg["vocab"])
    assert e.value.code == fh.ERR_POSITION
    gm.close()


def test_prefill_in_chunks_equals_one_shot(fh, torch_gpu):
    """Prefilling 90 tokens as 50 + 40 (second call starts at base_pos 50) equals one call of 90."""
    cfg = fh.synth.tiny(wdtype=Q8, max_seq=640)
    blob = fh.synth.make_weights_blob(cfg, seed=5)
    toks = fh.synth.uniform_ids(6, 90, cfg["vocab"])
    gm = fh.HipModel(cfg, blob)
    one = gm.forward_prefill(toks)
    gm.reset()
    gm.forward_prefill_batch(toks[:50])
    two = gm.forward_prefill(toks[50:])
    close(two, one, rtol=1e-4, atol=1e-4)
    gm.close()


def test_smollm2_135m_greedy_64_tokens_identical(fh, oracle, torch_gpu):
    """SmolLM2-135M-shape Q8_0 model, random-init: 32-token prompt, 64 greedy tokens, identical ids."""
    cfg = fh.synth.smollm2_135m(Q8, max_seq=1024)
    blob = fh.synth.make_weights_blob(cfg, seed=135)
    prompt = fh.synth.uniform_ids(136, 32, cfg["vocab"])
    gm = fh.HipModel(cfg, blob)
    om = oracle.Model(cfg, blob, A, KV_F16)
    got = gm.generate_greedy(prompt, 64)
    want = greedy_oracle(oracle, om, prompt, 64)
    assert got == want
    gm.close()
