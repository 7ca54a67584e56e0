"""The allocation-free entry point lr_attn_decode_static against lr_attn_decode (same kernels, the
split-KV partial results in the library's own fixed device array instead of a caller buffer):
outputs must be bit-identical, on two calls in a row of which the second is smaller (it reuses a
prefix of the array that still holds the first call's partial results), and a shape that needs
more than the array holds is refused.  Collected last on purpose."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF = torch.bfloat16


def _case(hip, B, Hq, Hkv, hd, Smax, pos, seed):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    r = lambda *shape: torch.randn(*shape, generator=g, device=DEV).to(BF)
    q, kc, vc = r(B, Hq * hd), r(B, Hkv, Smax, hd), r(B, Hkv, Smax, hd)
    p = torch.tensor([pos], dtype=torch.int32, device=DEV)
    want = torch.empty(B, Hq * hd, dtype=BF, device=DEV)
    scratch = torch.empty(hip.attn_decode_scratch_bytes(B, Hq, hd, Smax) // 4, dtype=torch.float32, device=DEV)
    hip.attn_decode(q, kc, vc, p, want, scratch, B, Hq, Hkv, hd)
    got = torch.full_like(want, float("nan"))
    return (q, kc, vc, p, got, B, Hq, Hkv, hd), want


def test_static_scratch_decode_equals_the_workspace_variant_twice_in_a_row():
    from gpt_fast import _hip as hip

    hip.load()
    big, want_big = _case(hip, 8, 8, 1, 128, 2176, 2100, seed=31)       # 70B rank shard, batch 8: 4.3 MB of partials
    small, want_small = _case(hip, 2, 4, 2, 64, 264, 17, seed=32)       # a smaller problem, another layout
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    hip.attn_decode_static(*big)
    hip.attn_decode_static(*small)     # second call in a row, smaller: reads only what it wrote itself
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the calls must not allocate device memory"
    assert torch.equal(big[4], want_big)
    assert torch.equal(small[4], want_small)
    # and again in the other order, on a side stream
    big[4].fill_(float("nan"))
    small[4].fill_(float("nan"))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        hip.attn_decode_static(*small)
        hip.attn_decode_static(*big)
    side.synchronize()
    assert torch.equal(big[4], want_big) and torch.equal(small[4], want_small)


def test_static_scratch_decode_refuses_what_does_not_fit():
    from gpt_fast import _hip as hip

    lib = hip.load()
    B, Hq, Hkv, hd, Smax = 128, 8, 1, 128, 2176                         # 34 MB of partials > 32 MiB
    assert hip.attn_decode_scratch_bytes(B, Hq, hd, Smax) > hip.ATTN_DECODE_STATIC_MAX_BYTES
    q = torch.zeros(B, Hq * hd, dtype=BF, device=DEV)
    kc = torch.zeros(B, Hkv, Smax, hd, dtype=BF, device=DEV)
    p = torch.zeros(1, dtype=torch.int32, device=DEV)
    with pytest.raises(hip.LadderHipError, match="built-in buffer"):
        hip.attn_decode_static(q, kc, kc, p, torch.empty_like(q), B, Hq, Hkv, hd)
    assert lib.lr_attn_decode_static(None, 0, None, None, None, None, 0, 1, 8, 1, 128, 64, None) == -1   # LR_E_NULL
