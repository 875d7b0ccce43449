"""The decode-attention entry point that allocates nothing (forge_hip_attn_decode_f16kv_noalloc) against the ordinary one
(forge_hip_attn_decode_f16kv, fast mode): the same kernels over a fixed array in the library's device image instead of an
allocation, so the results must be bit-identical -- and within rel/abs 1e-3 of the CPU oracle like the ordinary entry
point.  Two calls in a row share the array; the second is smaller, so stale records of the first lie behind it."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _case(fh, oracle, torch, heads, kv_heads, hd, seq, seed):
    k16 = oracle.f32_to_f16(fh.synth.normal(seed, seq * kv_heads * hd, 1.0)).reshape(seq, kv_heads * hd)
    v16 = oracle.f32_to_f16(fh.synth.normal(seed + 1, seq * kv_heads * hd, 1.0)).reshape(seq, kv_heads * hd)
    q = fh.synth.normal(seed + 2, heads * hd, 1.0)
    dev16 = lambda a: torch.from_numpy(a.view(np.int16)).cuda()
    return q, k16, v16, torch.from_numpy(q).cuda(), dev16(k16), dev16(v16)


def _same_bits(a, b):
    a, b = a.cpu().numpy(), b.cpu().numpy()
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"max abs difference {np.abs(a - b).max():.3e}"


def test_noalloc_decode_attention_equals_the_allocating_entry_point(fh, oracle, torch_gpu):
    torch = torch_gpu
    # first call: 32 query heads over 8 KV heads, head_dim 128, 900 rows; second call: fewer heads, shorter rows, 70 rows
    for heads, kv_heads, hd, seq, seed in ((32, 8, 128, 900, 40), (9, 3, 64, 70, 50)):
        q, k16, v16, qd, kd, vd = _case(fh, oracle, torch, heads, kv_heads, hd, seq, seed)
        out = torch.full((heads * hd,), float("nan"), device="cuda")
        got = fh.ops.attention_flash_noalloc(qd, kd, vd, seq, heads, kv_heads, hd, out)
        want = fh.ops.attention_flash(qd, kd, vd, seq, heads, kv_heads, hd, 0)
        _same_bits(got, want)
        ref = oracle.attention("flash", q, k16, v16, seq, heads, kv_heads, hd)
        err = np.abs(got.cpu().numpy().astype(np.float64) - ref)
        assert np.all(err <= 1e-3 + 1e-3 * np.abs(ref))
    # the same small case again after the large one, and the large one after the small one
    for heads, kv_heads, hd, seq, seed in ((32, 8, 128, 900, 40), (9, 3, 64, 70, 50), (32, 8, 128, 900, 40)):
        q, k16, v16, qd, kd, vd = _case(fh, oracle, torch, heads, kv_heads, hd, seq, seed)
        out = torch.empty(heads * hd, device="cuda")
        _same_bits(fh.ops.attention_flash_noalloc(qd, kd, vd, seq, heads, kv_heads, hd, out),
                   fh.ops.attention_flash(qd, kd, vd, seq, heads, kv_heads, hd, 0))


def test_noalloc_decode_attention_allocates_nothing_and_refuses_what_does_not_fit(fh, oracle, torch_gpu):
    torch = torch_gpu
    heads, kv_heads, hd, seq = 32, 8, 64, 300
    _, _, _, qd, kd, vd = _case(fh, oracle, torch, heads, kv_heads, hd, seq, 60)
    out = torch.empty(heads * hd, device="cuda")
    fh.ops.attention_flash_noalloc(qd, kd, vd, seq, heads, kv_heads, hd, out)       # the array's address is looked up here
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        fh.ops.attention_flash_noalloc(qd, kd, vd, seq, heads, kv_heads, hd, out)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before                                               # the device's free memory did not move
    # 160 query heads need more split records than the fixed array holds
    big_q = torch.zeros(160 * 64, device="cuda")
    big_out = torch.empty_like(big_q)
    kc = torch.zeros((4, 64), dtype=torch.int16, device="cuda")
    with pytest.raises(fh.ForgeHipError) as e:
        fh.ops.attention_flash_noalloc(big_q, kc, kc, 4, 160, 1, 64, big_out)
    assert e.value.code == fh.ERR_INVALID and "128" in str(e.value)
    with pytest.raises(fh.ForgeHipError):
        fh.ops.attention_flash_noalloc(qd, kd, vd, 0, heads, kv_heads, hd, out)      # no rows
