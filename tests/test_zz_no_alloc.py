"""The entry point that allocates nothing (mi355_fmha_fwd_noalloc): its split-KV partial results live in a static
device array instead of a workspace obtained with hipMalloc. Checked through the C ABI against mi355_fmha_fwd on the
same inputs, bit for bit (same kernels, same partials, different memory), on two calls in a row, the second smaller,
and against the fp32 oracle to the attention tolerance (max|dO| <= 2e-3, max|dLSE| <= 1e-3)."""
import pytest
import torch

import serving_oracle as so

pytestmark = pytest.mark.gpu


def both(lib, gpu, B, Hq, Hkv, Sq, Sk, causal, kvv, seed):
    q, k, v = so.fmha_inputs(B, Hq, Hkv, Sq, Sk, seed=seed)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    o_ref, l_ref = lib.fmha_fwd(qg, kg, vg, causal=causal, kv_valid_len=kvv)          # mi355_fmha_fwd
    o = torch.full_like(qg, float("nan"))
    l = torch.full((B, Hq, Sq), float("nan"), dtype=torch.float32, device=gpu)
    torch.cuda.synchronize()
    free_before, held_before = torch.cuda.mem_get_info(gpu)[0], torch.cuda.memory_reserved(gpu)
    lib.fmha_fwd_noalloc(qg, kg, vg, o, l, causal=causal, kv_valid_len=kvv)
    torch.cuda.synchronize()
    # nothing was taken from the device (hipMalloc of any kind lowers the free figure) nor from torch's allocator
    assert torch.cuda.mem_get_info(gpu)[0] == free_before and torch.cuda.memory_reserved(gpu) == held_before
    assert torch.equal(o, o_ref) and torch.equal(l, l_ref), (B, Hq, Hkv, Sq, Sk)
    oc, lc = so.attention_ref(q, k, v, causal=causal, kv_valid_len=kvv)
    ok, st = so.fmha_tolerance_ok(o.cpu(), l.cpu(), oc, lc)
    assert ok, st


def test_no_alloc_entry_point_matches_the_allocating_one_on_two_calls_in_a_row(lib, gpu):
    # Llama-3-8B generation step at batch 4 over 8192 keys (256 workgroups x 4 columns), then a smaller call that leaves
    # most of the previous call's partials in the array untouched
    both(lib, gpu, 4, 32, 8, 1, 8192, False, None, seed=71)
    both(lib, gpu, 1, 8, 2, 3, 1000, True, 990, seed=72)
    # and back to a larger one with 32 columns per unit
    both(lib, gpu, 2, 32, 1, 1, 3000, False, None, seed=73)


def test_no_alloc_entry_point_on_prefill_shapes_and_strided_operands(lib, gpu):
    # outside the split-KV path the array is not used; strided operands (a fused QKV projection) are read in place
    both(lib, gpu, 1, 4, 2, 300, 300, True, None, seed=74)
    B, S, Hq, Hkv = 2, 1500, 8, 2
    q, k, v = so.fmha_inputs(B, Hq, Hkv, 1, S, seed=75)
    fused = torch.zeros((B, S, (Hq + 2 * Hkv) * 128), dtype=torch.float16)
    fused[:, -1:, :Hq * 128] = q.transpose(1, 2).reshape(B, 1, Hq * 128)
    fused[:, :, Hq * 128:(Hq + Hkv) * 128] = k.transpose(1, 2).reshape(B, S, Hkv * 128)
    fused[:, :, (Hq + Hkv) * 128:] = v.transpose(1, 2).reshape(B, S, Hkv * 128)
    f = fused.to(gpu).view(B, S, Hq + 2 * Hkv, 128)
    qv, kv_, vv = f[:, -1:, :Hq].transpose(1, 2), f[:, :, Hq:Hq + Hkv].transpose(1, 2), f[:, :, Hq + Hkv:].transpose(1, 2)
    o_ref = lib.fmha_fwd(qv, kv_, vv, return_lse=False)
    o = torch.empty((B, 1, Hq, 128), dtype=torch.float16, device=gpu).transpose(1, 2)
    lib.fmha_fwd_noalloc(qv, kv_, vv, o)
    torch.cuda.synchronize()
    assert torch.equal(o, o_ref)


def test_no_alloc_entry_point_rejects_what_does_not_fit(lib, gpu):
    # 256 workgroups x 32 columns x 528 B = 4.3 MB of partials > the 4 MiB array: refused before anything is launched
    q, k, v = (t.to(gpu) for t in so.fmha_inputs(8, 32, 1, 1, 16384, seed=76))
    o = torch.empty_like(q)
    with pytest.raises(lib.Mi355Error, match="static scratch"):
        lib.fmha_fwd_noalloc(q, k, v, o)
    assert lib.load().mi355_last_error().decode().count("mi355_fmha_fwd_ws") == 1
