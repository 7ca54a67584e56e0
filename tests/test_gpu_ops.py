"""Per-kernel parity on a real MI355X: every C-ABI entry point of libladder_hip.so against the
oracle's op (oracle/ladder_oracle.py, eager PyTorch on the same device, same seeded inputs).

Tolerances, all stated in bf16 units-in-the-last-place ("ulp") of the produced tensor:
  * pure data movement and element-wise work with one rounding (embed, add, RoPE, cache write,
    argmax, advance): bit-exact;
  * ops with an fp32 reduction inside (RMSNorm, linear, attention) or a transcendental (SwiGLU):
    the fp32 value before the final rounding differs from the oracle's by summation order /
    libm only, so results must agree within 1 ulp and on all but a small fraction of elements."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import ladder_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda"
BF = torch.bfloat16


@pytest.fixture(scope="module")
def hip():
    from gpt_fast import _hip

    _hip.load()
    return _hip


def rnd(*shape, seed=0, scale=1.0, dtype=BF):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    return (torch.randn(*shape, generator=g, device=DEV) * scale).to(dtype)


def ulp_diff(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in bf16 steps between two bf16 tensors (monotonic integer mapping of the bits)."""
    def key(t):
        i = t.contiguous().view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)
    return (key(a) - key(b)).abs()


def assert_close_ulp(got, want, max_ulp=1, max_frac=0.02, what=""):
    assert got.shape == want.shape and got.dtype == want.dtype == BF
    assert torch.isfinite(got.float()).all(), what
    d = ulp_diff(got, want)
    # values whose magnitude is far below the tensor's scale may differ by many ulps of their own
    # size while being equal to fp32 accuracy relative to the sum that produced them
    tiny = want.float().abs() < want.float().abs().max() * 2.0 ** -12
    bad = (d > max_ulp) & ~tiny
    frac = (d > 0).float().mean().item()
    assert not bad.any(), f"{what}: {int(bad.sum())} elements differ by more than {max_ulp} ulp (max {int(d.max())})"
    assert frac <= max_frac, f"{what}: {frac:.4f} of elements differ (limit {max_frac})"


# ------------------------------------------------------------------------------------ embed / add / advance

@pytest.mark.parametrize("idx_dtype", [torch.int64, torch.int32])
def test_embed_exact(hip, idx_dtype):
    table = rnd(1000, 512, seed=1)
    idx = torch.randint(0, 1000, (3, 17), device=DEV, dtype=idx_dtype)
    out = torch.empty(3 * 17, 512, dtype=BF, device=DEV)
    hip.embed(table, idx, out)
    assert torch.equal(out.view(3, 17, 512), F.embedding(idx.long(), table))


@pytest.mark.parametrize("n", [8, 2048, 8192 * 5 + 24, 1000003])
def test_add_exact(hip, n):
    a, b = rnd(n, seed=2), rnd(n, seed=3)
    out = torch.empty_like(a)
    hip.add(a, b, out)
    assert torch.equal(out, a + b)
    hip.add(a, b, out, b_div=8.0)
    assert torch.equal(out, a + b / 8)
    hip.add(a, b, out, b_div=3.0)
    assert torch.equal(out, a + b / 3)
    out2 = b.clone()
    hip.add(a, out2, out2)  # aliasing the second operand
    assert torch.equal(out2, a + b)


def test_advance_and_history(hip):
    B = 5
    cur = torch.zeros(B, 1, dtype=torch.int32, device=DEV)
    nxt = torch.arange(10, 10 + B, dtype=torch.int32, device=DEV).view(B, 1)
    pos = torch.tensor([7], dtype=torch.int32, device=DEV)
    hist = torch.full((B, 4), -1, dtype=torch.int32, device=DEV)
    hip.advance(cur, nxt, pos, B, hist, pos0=6)
    assert pos.item() == 8 and torch.equal(cur, nxt) and hist[:, 1].tolist() == list(range(10, 10 + B))
    assert (hist[:, [0, 2, 3]] == -1).all()
    hip.advance(None, None, pos, B)
    assert pos.item() == 9


# ------------------------------------------------------------------------------------ RMSNorm

@pytest.mark.parametrize("rows,dim", [(1, 8192), (3, 4096), (64, 8192), (2, 16384), (5, 256), (2048, 2048)])
def test_add_rmsnorm(hip, rows, dim):
    r, d1, d2 = rnd(rows, dim, seed=4), rnd(rows, dim, seed=5, scale=0.1), rnd(rows, dim, seed=6, scale=0.1)
    g = rnd(dim, seed=7, scale=0.02)
    ro, no = torch.empty_like(r), torch.empty_like(r)
    # plain norm
    hip.add_rmsnorm(r, None, None, g, None, no, 1e-5)
    # two roundings in a row (normalised value, then gain product): a 1-ulp flip of the first can
    # show as 2 ulp after the second, hence max_ulp=2 for this op only
    assert_close_ulp(no, O.rms_norm(r, g, 1e-5), max_ulp=2, max_frac=0.01, what="norm")
    # one pending partial (ladder add), residual written back
    hip.add_rmsnorm(r, d1, None, g, ro, no, 1e-5)
    assert torch.equal(ro, r + d1)
    assert_close_ulp(no, O.rms_norm(r + d1, g, 1e-5), max_ulp=2, max_frac=0.01, what="add+norm")
    # two pending partials (closing add of the ladder), in place
    r2 = r.clone()
    hip.add_rmsnorm(r2, d1, d2, g, r2, no, 1e-5)
    assert torch.equal(r2, r + d1 + d2)
    assert_close_ulp(no, O.rms_norm(r + d1 + d2, g, 1e-5), max_ulp=2, max_frac=0.01, what="add+add+norm")


# ------------------------------------------------------------------------------------ linear

def linear_ref(x, w):
    """fp64 product rounded once: what any fp32-accumulating bf16 linear must match within 1 ulp."""
    return (x.double() @ w.double().T).to(BF)


GEMV_SHAPES = [  # (N, K): the 70B rank shard, the 8B model, the 1B model, and ragged sizes
    (1280, 8192), (8192, 1024), (7168, 8192), (8192, 3584), (16032, 8192),
    (6144, 4096), (4096, 4096), (3072, 2048), (2048, 8192), (24, 64), (1001, 520),
]


@pytest.mark.parametrize("N,K", GEMV_SHAPES)
@pytest.mark.parametrize("M", [1, 2, 3, 5, 8])
def test_linear_gemv(hip, M, N, K):
    x = rnd(M, K, seed=8)
    w = rnd(N, K, seed=9, scale=0.02)
    y = torch.empty(M, N, dtype=BF, device=DEV)
    hip.linear(x, w, y)
    assert_close_ulp(y, linear_ref(x, w), what=f"gemv M={M} N={N} K={K}")
    # and against the library routine the reference uses
    assert_close_ulp(y, F.linear(x, w), max_frac=0.05, what="gemv vs F.linear")


@pytest.mark.parametrize("N,K", [(1280, 8192), (8192, 1024), (7168, 8192), (8192, 3584), (16032, 8192), (4096, 4096),
                                 (4096, 14336), (24, 64), (1001, 520), (130, 136), (33, 8)])
@pytest.mark.parametrize("M", [5, 8, 16, 17, 31, 33, 64])
def test_linear_decode_batches(hip, M, N, K):
    """Decode batches (4 < M <= 64) take the weight-streaming matrix-core kernel: ragged N (bands that end
    inside a 16-row unit), K not a multiple of the 128-element chunk or shorter than one, M on both sides
    of the 16-row column tiles, a strided output view."""
    x = rnd(M, K, seed=12)
    w = rnd(N, K, seed=13, scale=0.02)
    y = torch.empty(M, N, dtype=BF, device=DEV)
    hip.linear(x, w, y)
    assert_close_ulp(y, linear_ref(x, w), what=f"decode batch M={M} N={N} K={K}")
    if N % 8 == 0:
        wide = torch.zeros(M, N + 8, dtype=BF, device=DEV)
        hip.linear(x, w, wide[:, :N])
        assert torch.equal(wide[:, :N], y) and bool((wide[:, N:] == 0).all())


def swiglu_of_projection_ref(x, w1):
    """[up; gate] rows -> bf16(bf16(silu(g)) * u) with u, g the projections rounded to bf16 (utils.py:145-148)."""
    h = linear_ref(x, w1)
    inter = w1.shape[0] // 2
    return F.silu(h[:, inter:]) * h[:, :inter]   # feed_forward of the oracle: silu(g) * u on bf16 tensors


@pytest.mark.parametrize("M,D,NQ,I", [(8, 8192, 1280, 3584), (64, 8192, 1280, 3584), (16, 4096, 6144, 14336),
                                      (5, 264, 40, 50), (33, 136, 520, 17), (1, 512, 96, 200), (64, 72, 8, 1000)])
def test_linear_multi_two_projections_one_launch(hip, M, D, NQ, I):
    """q/k/v projection next to the up/gate projection with the SwiGLU epilogue, in one launch: each output
    against the oracle's op on its own input; bands of different heights in the two projections."""
    xa, xb = rnd(M, D, seed=30), rnd(M, D, seed=31)
    wq, w1 = rnd(NQ, D, seed=32, scale=0.03), rnd(2 * I, D, seed=33, scale=0.03)
    q = torch.empty(M, NQ, dtype=BF, device=DEV)
    act = torch.full((M, I), 3.0, dtype=BF, device=DEV)
    hip.linear_multi((xa, wq, q, hip.EPI_NONE), (xb, w1, act, hip.EPI_SWIGLU))
    assert_close_ulp(q, linear_ref(xa, wq), what="multi: plain projection")
    # u and g may each sit one ulp away from the fp64-rounded projections; the activation amplifies that
    want = swiglu_of_projection_ref(xb, w1)
    assert torch.isfinite(act.float()).all()
    err = (act.float() - want.float()).abs().max().item()
    assert err <= 2.0 ** -6 * want.float().abs().max().item(), err
    assert (ulp_diff(act, want) > 1).float().mean().item() < 0.05
    # the same projections one at a time give the same bits
    q1, act1 = torch.empty_like(q), torch.empty_like(act)
    hip.linear_multi((xa, wq, q1, hip.EPI_NONE))
    hip.linear_multi((xb, w1, act1, hip.EPI_SWIGLU))
    assert torch.equal(q1, q) and torch.equal(act1, act)


def test_linear_multi_swiglu_epilogue_equals_the_two_step_path(hip):
    """The fused epilogue rounds where the unfused path rounds: w1 -> h (bf16) -> lr_swiglu gives the same bits."""
    M, D, I = 8, 1024, 520
    x, w1 = rnd(M, D, seed=34), rnd(2 * I, D, seed=35, scale=0.03)
    act = torch.empty(M, I, dtype=BF, device=DEV)
    hip.linear_multi((x, w1, act, hip.EPI_SWIGLU))
    h = torch.empty(M, 2 * I, dtype=BF, device=DEV)
    hip.linear_multi((x, w1, h, hip.EPI_NONE))
    two_step = torch.empty(M, I, dtype=BF, device=DEV)
    hip.swiglu(h, two_step)
    assert torch.equal(act, two_step)


@pytest.mark.parametrize("B,Hq,Hkv,hd,D", [(8, 8, 1, 128, 1024), (64, 8, 1, 128, 512), (16, 32, 8, 128, 264),
                                            (5, 4, 2, 64, 136), (1, 2, 2, 64, 64)])
@pytest.mark.parametrize("pos_value", [0, 37])
def test_linear_multi_rope_kv_epilogue_equals_projection_then_rope_kv_write(hip, B, Hq, Hkv, hd, D, pos_value):
    """The q/k/v projection that rotates and caches on its way out leaves q, the K slot and the V slot exactly as
    the plain projection followed by lr_rope_kv_write does, and touches no other cache slot."""
    Smax, block = 48, 64
    N = (Hq + 2 * Hkv) * hd
    x, w = rnd(B, D, seed=40), rnd(N, D, seed=41, scale=0.05)
    table = O.rope_table(block, hd, 10000.0, BF).to(DEV)
    pos = torch.tensor([pos_value], dtype=torch.int32, device=DEV)
    kc = [rnd(B, Hkv, Smax, hd, seed=42) for _ in range(2)]
    vc = [rnd(B, Hkv, Smax, hd, seed=43) for _ in range(2)]
    # reference path
    q_ref = torch.empty(B, N, dtype=BF, device=DEV)
    hip.linear_multi((x, w, q_ref, hip.EPI_NONE))
    k_proj = q_ref[:, Hq * hd:].clone()
    hip.rope_kv_write(q_ref, table, False, pos, kc[0], vc[0], B, 1, Hq, Hkv, hd)
    # fused path
    q = torch.empty(B, N, dtype=BF, device=DEV)
    hip.linear_multi((x, w, q, hip.rope_kv_epilogue(table, pos, kc[1], vc[1], Hq, Hkv, hd)))
    assert torch.equal(q[:, :Hq * hd], q_ref[:, :Hq * hd])
    assert torch.equal(q[:, Hq * hd:], k_proj)          # k and v stay as projected in the row buffer
    assert torch.equal(kc[1], kc[0]) and torch.equal(vc[1], vc[0])
    assert not torch.equal(kc[1][:, :, pos_value], rnd(B, Hkv, Smax, hd, seed=42)[:, :, pos_value])


def test_linear_multi_rope_kv_epilogue_reports_a_position_outside_the_cache(hip):
    B, Hq, Hkv, hd, D, Smax = 8, 4, 1, 64, 128, 16
    N = (Hq + 2 * Hkv) * hd
    x, w = rnd(B, D, seed=44), rnd(N, D, seed=45, scale=0.05)
    table = O.rope_table(32, hd, 10000.0, BF).to(DEV)
    kc, vc = rnd(B, Hkv, Smax, hd, seed=46), rnd(B, Hkv, Smax, hd, seed=47)
    kc0, vc0 = kc.clone(), vc.clone()
    err = hip.device_error_word(DEV)
    err.zero_()
    plain, q = torch.empty(B, N, dtype=BF, device=DEV), torch.empty(B, N, dtype=BF, device=DEV)
    hip.linear_multi((x, w, plain, hip.EPI_NONE))
    hip.linear_multi((x, w, q, hip.rope_kv_epilogue(table, torch.tensor([Smax], dtype=torch.int32, device=DEV), kc, vc,
                                                    Hq, Hkv, hd)))
    torch.cuda.synchronize()
    assert int(err.item()) == hip.DEV_POS_RANGE
    err.zero_()
    assert torch.equal(q, plain) and torch.equal(kc, kc0) and torch.equal(vc, vc0)


@pytest.mark.parametrize("M,D,I", [(5, 264, 56), (64, 1024, 520), (100, 520, 136), (512, 4096, 14336 // 4), (700, 328, 1000),
                                   (2048, 1024, 3584), (2300, 520, 3000), (2300, 512, 3000)])
def test_linear_swiglu_out_equals_projection_then_swiglu(hip, M, D, I):
    """The first MLP projection with the activation in its epilogue -- the streaming kernel's row pairs (M <= 64), the
    256 x 256 tile GEMM on tiles of 128 pairs (M >= 512, ragged edges included), the two-step fallback in between --
    against the oracle's ops, and bit for bit against lr_linear followed by lr_swiglu."""
    x, w1 = rnd(M, D, seed=50), rnd(2 * I, D, seed=51, scale=0.03)
    act = torch.full((M, I), 3.0, dtype=BF, device=DEV)
    scratch = torch.empty(M, 2 * I, dtype=BF, device=DEV)
    hip.linear_swiglu_out(x, w1, act, scratch)
    h = torch.empty(M, 2 * I, dtype=BF, device=DEV)
    hip.linear(x, w1, h)
    two_step = torch.empty(M, I, dtype=BF, device=DEV)
    hip.swiglu(h, two_step)
    want = swiglu_of_projection_ref(x, w1)
    assert torch.isfinite(act.float()).all()
    assert (act.float() - want.float()).abs().max().item() <= 2.0 ** -6 * want.float().abs().max().item()
    assert (ulp_diff(act, want) > 1).float().mean().item() < 0.05
    # same kernel family on both sides (same summation order) wherever the fused form exists: identical bits
    assert torch.equal(act, two_step)


def test_linear_multi_is_deterministic(hip):
    x, w = rnd(64, 8192, seed=36), rnd(1280, 8192, seed=37, scale=0.02)
    ys = []
    for _ in range(4):
        y = torch.empty(64, 1280, dtype=BF, device=DEV)
        hip.linear_multi((x, w, y, hip.EPI_NONE))
        ys.append(y)
    assert all(torch.equal(ys[0], t) for t in ys[1:])


@pytest.mark.parametrize("cfg", [144, 212, 222, 242, 244, 412, 422, 442])
def test_linear_gemv_every_launch_configuration(hip, cfg):
    x = rnd(4, 3584, seed=10)
    w = rnd(1030, 3584, seed=11, scale=0.02)
    y = torch.empty(4, 1030, dtype=BF, device=DEV)
    hip.linear(x, w, y, gemv_cfg=cfg)   # lr_linear_tuned: the configuration is an argument of the call
    assert_close_ulp(y, linear_ref(x, w), what=f"gemv cfg {cfg}")


def test_linear_gemv_is_deterministic(hip):
    x = rnd(1, 8192, seed=12)
    w = rnd(1280, 8192, seed=13, scale=0.02)
    ys = []
    for _ in range(5):
        y = torch.empty(1, 1280, dtype=BF, device=DEV)
        hip.linear(x, w, y)
        ys.append(y)
    assert all(torch.equal(ys[0], t) for t in ys[1:])


@pytest.mark.parametrize("M,N,K", [(9, 256, 64), (128, 128, 64), (130, 1280, 8192), (2048, 1280, 1024),
                                   (333, 1001, 520), (64, 16032, 2048), (16, 8192, 3584), (257, 384, 8),
                                   # 256 x 256 tiles (M >= 512): whole tiles, ragged edges in M, N and K, the
                                   # XCD-aware tile order (M / 256 a multiple of 32) and the plain one
                                   (512, 256, 64), (700, 500, 328), (1024, 6144, 4096), (8192, 512, 136),
                                   (8192 + 3, 257, 72),
                                   # enough 256 x 256 tiles for the large-tile kernel (192 and more): whole tiles
                                   # in the plain and in the XCD-aware order, ragged edges in M and N with K a
                                   # multiple of the k-tile (scalar k offsets) and with a K tail (per-lane checks)
                                   (4096, 3072, 1024), (8192, 1536, 512), (5000, 3000, 512), (5000, 3000, 328),
                                   (6144, 2048, 64)])
def test_linear_gemm(hip, M, N, K):
    x = rnd(M, K, seed=14)
    w = rnd(N, K, seed=15, scale=0.02)
    y = torch.empty(M, N, dtype=BF, device=DEV)
    hip.linear(x, w, y)
    assert_close_ulp(y, linear_ref(x, w), what=f"gemm M={M} N={N} K={K}")


def test_linear_strided_rows(hip):
    big = rnd(6, 3 * 512, seed=16)
    x = big[:, 512:1024]                      # row stride 1536
    w = rnd(200, 512, seed=17, scale=0.05)
    out = torch.zeros(6, 2 * 200, dtype=BF, device=DEV)
    y = out[:, 200:]                          # row stride 400
    hip.linear(x, w, y)
    assert_close_ulp(y.contiguous(), linear_ref(x, w), what="strided")
    assert (out[:, :200] == 0).all()


@pytest.mark.parametrize("rows", [1, 4, 8, 40])
def test_swiglu_and_fused_w2(hip, rows):
    I, D = 3584, 1024
    h = rnd(rows, 2 * I, seed=18)
    w2 = rnd(D, I, seed=19, scale=0.02)
    u, g = h.chunk(2, dim=-1)
    act = F.silu(g) * u
    out = torch.empty(rows, I, dtype=BF, device=DEV)
    hip.swiglu(h, out)
    assert_close_ulp(out, act, max_frac=0.002, what="swiglu")
    y = torch.empty(rows, D, dtype=BF, device=DEV)
    hip.linear(h, w2, y, act_swiglu=True)
    assert_close_ulp(y, linear_ref(act, w2), max_frac=0.05, what="w2(silu(g)*u)")


# ------------------------------------------------------------------------------------ RoPE + cache

@pytest.mark.parametrize("hd,Hq,Hkv", [(128, 8, 1), (64, 32, 8), (128, 32, 8)])
@pytest.mark.parametrize("gathered", [False, True])
def test_rope_kv_write_exact(hip, hd, Hq, Hkv, gathered):
    B, S, Smax, block = 2, 9, 32, 64
    width = (Hq + 2 * Hkv) * hd
    qkv = rnd(B, S, width + 16, seed=20)[..., :width]          # padded rows: row stride != width
    pos = torch.tensor([3, 4, 5, 6, 7, 8, 9, 20, 31], dtype=torch.int32, device=DEV)
    table = O.rope_table(block, hd, 500000, BF).to(DEV)
    kc = torch.zeros(B + 1, Hkv, Smax, hd, dtype=BF, device=DEV)
    vc = torch.zeros_like(kc)
    q, k, v = qkv.clone().split([Hq * hd, Hkv * hd, Hkv * hd], dim=-1)
    fc = table[pos.long()]
    q_ref = O.apply_rope(q.reshape(B, S, Hq, hd), fc)
    k_ref = O.apply_rope(k.reshape(B, S, Hkv, hd), fc).transpose(1, 2)
    kc_ref, vc_ref = kc.clone(), vc.clone()
    O.kv_update(kc_ref, vc_ref, pos.long(), k_ref, v.reshape(B, S, Hkv, hd).transpose(1, 2))

    work = qkv  # rotated in place on the strided view
    hip.rope_kv_write(work, fc.contiguous() if gathered else table, gathered, pos, kc, vc, B, S, Hq, Hkv, hd)
    assert torch.equal(work[..., : Hq * hd].reshape(B, S, Hq, hd), q_ref)
    assert torch.equal(kc, kc_ref) and torch.equal(vc, vc_ref)
    assert torch.equal(work[..., Hq * hd:], torch.cat([k, v], -1))   # k and v columns are left as they were


@pytest.mark.parametrize("B,S,Hq,Hkv,hd,K,Smax,start", [
    # the 256 x 256-tile GEMM with the rotation and the cache writes in its output pass: whole tiles; ragged rows,
    # sequences that end inside a tile, K with a tail, positions that do not start at 0; then shapes below that
    # kernel's threshold (the two-call fallback) and a decode-sized one
    (4, 1024, 16, 4, 128, 1024, 1024, 0), (5, 1000, 32, 16, 64, 520, 1072, 37), (9, 300, 16, 4, 128, 256, 512, 100),
    (2, 100, 8, 1, 128, 512, 136, 0), (3, 1, 8, 2, 64, 264, 16, 5),
])
def test_linear_rope_kv_equals_the_two_calls(hip, B, S, Hq, Hkv, hd, K, Smax, start):
    """lr_linear_rope_kv against lr_linear followed by lr_rope_kv_write on the same buffers: the output rows and both
    caches bit for bit; and the separate calls against the oracle (apply_rope, kv_update) as everywhere."""
    N = (Hq + 2 * Hkv) * hd
    x = rnd(B * S, K, seed=80)
    w = rnd(N, K, seed=81, scale=0.05)
    pos = torch.arange(start, start + S, dtype=torch.int32, device=DEV)
    table = O.rope_table(start + S + 3, hd, 500000, BF).to(DEV)
    want = torch.empty(B * S, N, dtype=BF, device=DEV)
    hip.linear(x, w, want)
    proj = want.clone()
    kc_w = torch.zeros(B + 1, Hkv, Smax, hd, dtype=BF, device=DEV)
    vc_w = torch.zeros_like(kc_w)
    hip.rope_kv_write(want, table, False, pos, kc_w, vc_w, B, S, Hq, Hkv, hd)
    fc = table[pos.long()]
    q, k, v = proj.view(B, S, N).split([Hq * hd, Hkv * hd, Hkv * hd], dim=-1)
    assert torch.equal(want.view(B, S, N)[..., : Hq * hd].reshape(B, S, Hq, hd), O.apply_rope(q.reshape(B, S, Hq, hd), fc))
    kc_o, vc_o = torch.zeros_like(kc_w), torch.zeros_like(kc_w)
    O.kv_update(kc_o, vc_o, pos.long(), O.apply_rope(k.reshape(B, S, Hkv, hd), fc).transpose(1, 2),
                v.reshape(B, S, Hkv, hd).transpose(1, 2))
    assert torch.equal(kc_w, kc_o) and torch.equal(vc_w, vc_o)

    got = torch.full((B * S, N), 7.0, dtype=BF, device=DEV)
    kc, vc = torch.zeros_like(kc_w), torch.zeros_like(kc_w)
    hip.linear_rope_kv(x, w, got, table, pos, kc, vc, B, S, Hq, Hkv, hd)
    assert torch.equal(got, want)
    assert torch.equal(kc, kc_w) and torch.equal(vc, vc_w)
    hip.raise_on_device_error(got.device)


def test_linear_rope_kv_position_out_of_range(hip):
    """A position beyond the cache: that row stays as projected, nothing of it reaches the caches, the device error
    word is set (as lr_rope_kv_write does); the other rows are finished as usual."""
    B, S, Hq, Hkv, hd, K, Smax = 4, 1024, 16, 4, 128, 512, 1024
    N = (Hq + 2 * Hkv) * hd
    x, w = rnd(B * S, K, seed=82), rnd(N, K, seed=83, scale=0.05)
    pos = torch.arange(S, dtype=torch.int32, device=DEV)
    pos[700] = Smax + 5
    table = O.rope_table(2048, hd, 500000, BF).to(DEV)
    want = torch.empty(B * S, N, dtype=BF, device=DEV)
    hip.linear(x, w, want)
    kc_w = torch.zeros(B, Hkv, Smax, hd, dtype=BF, device=DEV)
    vc_w = torch.zeros_like(kc_w)
    hip.device_error_word(want.device).zero_()
    hip.rope_kv_write(want, table, False, pos, kc_w, vc_w, B, S, Hq, Hkv, hd)
    assert int(hip.device_error_word(want.device).item()) != 0
    hip.device_error_word(want.device).zero_()
    got = torch.empty_like(want)
    kc, vc = torch.zeros_like(kc_w), torch.zeros_like(kc_w)
    hip.linear_rope_kv(x, w, got, table, pos, kc, vc, B, S, Hq, Hkv, hd)
    torch.cuda.synchronize()
    assert int(hip.device_error_word(want.device).item()) != 0
    hip.device_error_word(want.device).zero_()
    assert torch.equal(got, want) and torch.equal(kc, kc_w) and torch.equal(vc, vc_w)


@pytest.mark.parametrize("hd,H", [(128, 1), (64, 8), (128, 8)])
@pytest.mark.parametrize("layout", ["bhsd", "bshd"])
def test_kv_cache_update_module_method(hd, H, layout):
    """KVCache.update (utils.py:50-59) through lr_kv_update: dense [B, H, S, D] values and the transposed view of a
    [B, S, H, D] tensor (what a caller holds right after splitting a projection), scattered positions, a batch
    smaller than the cache; bit-exact against the oracle's indexed assignment, rows not addressed stay zero."""
    from gpt_fast.utils import KVCache

    B, S, Smax = 2, 7, 40
    pos = torch.tensor([0, 5, 6, 7, 21, 38, 39], device=DEV)          # int64, as torch.arange gives
    if layout == "bhsd":
        k, v = rnd(B, H, S, hd, seed=70), rnd(B, H, S, hd, seed=71)
    else:
        k, v = rnd(B, S, H, hd, seed=70).transpose(1, 2), rnd(B, S, H, hd, seed=71).transpose(1, 2)
    cache = KVCache(B + 1, Smax, H, hd).to(DEV)
    kc_ref, vc_ref = cache.k_cache.clone(), cache.v_cache.clone()
    O.kv_update(kc_ref, vc_ref, pos, k, v)
    k_out, v_out = cache.update(pos, k, v)
    assert k_out is cache.k_cache and v_out is cache.v_cache
    assert torch.equal(k_out, kc_ref) and torch.equal(v_out, vc_ref)
    assert float(k_out[B].abs().max()) == 0.0 and float(k_out[:, :, 1].abs().max()) == 0.0


def test_kv_cache_update_reports_a_position_outside_the_cache(hip):
    from gpt_fast.utils import KVCache

    cache = KVCache(1, 16, 2, 64).to(DEV)
    k = rnd(1, 2, 2, 64, seed=72)
    hip.device_error_word(DEV).zero_()
    cache.update(torch.tensor([3, 16], device=DEV), k, k)
    torch.cuda.synchronize()
    assert int(hip.device_error_word(DEV).item()) == 2            # LR_DEV_POS_RANGE; slot 3 was still written
    assert torch.equal(cache.k_cache[0, :, 3], k[0, :, 0])
    hip.device_error_word(DEV).zero_()


@pytest.mark.parametrize("rows,dim", [(1, 8192), (8, 8192), (64, 4096), (3, 2048), (16, 16384), (5, 264)])
@pytest.mark.parametrize("first_block", [False, True])
def test_ladder_norms_equals_two_add_rmsnorm_calls(hip, rows, dim, first_block):
    """lr_ladder_norms (both residual updates + both norms of a block in one launch) must give, bit for bit, what
    two lr_add_rmsnorm calls give, and match the oracle's block prologue (gpt_ladder_TP.py:326-354)."""
    x, d1, d2 = rnd(rows, dim, seed=50), rnd(rows, dim, seed=51, scale=0.3), rnd(rows, dim, seed=52, scale=0.3)
    g1, g2 = rnd(dim, seed=53), rnd(dim, seed=54)
    if first_block:
        d1 = d2 = None
    r_ref, n1_ref, n2_ref = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    hip.add_rmsnorm(x, d1, None, g1, r_ref, n1_ref, 1e-5)
    hip.add_rmsnorm(r_ref, d2, None, g2, r_ref, n2_ref, 1e-5)
    r, n1, n2 = x.clone(), torch.empty_like(x), torch.empty_like(x)
    hip.ladder_norms(r, d1, d2, g1, g2, r, n1, n2, 1e-5)       # residual updated in place
    assert torch.equal(r, r_ref) and torch.equal(n1, n1_ref) and torch.equal(n2, n2_ref)
    r1 = x if first_block else x + d1
    r2 = r1 if first_block else r1 + d2
    assert torch.equal(r, r2)
    assert_close_ulp(n1, O.rms_norm(r1, g1, 1e-5), max_ulp=2, max_frac=0.05, what="ladder_norms n1")
    assert_close_ulp(n2, O.rms_norm(r2, g2, 1e-5), max_ulp=2, max_frac=0.05, what="ladder_norms n2")


# ------------------------------------------------------------------------------------ weight-only fp8 linear

def test_linear_fp8_decodes_every_e4m3_value_exactly(hip):
    """All 254 finite byte patterns of float8_e4m3fn (normals, denormals, both zeros) through the kernel's
    conversion: with one-hot inputs and unit scales the output IS the stored value."""
    codes = torch.arange(256, dtype=torch.uint8, device=DEV)
    codes[0x7F] = 0          # the two NaN patterns are replaced
    codes[0xFF] = 0x80
    w8 = codes.view(torch.float8_e4m3fn).view(16, 16).contiguous()
    scales = torch.ones(16, dtype=BF, device=DEV)
    want = w8.to(torch.float32).T.contiguous()      # y[m, n] = w8[n, m]
    for m0 in (0, 8):
        x = torch.eye(16, dtype=BF, device=DEV)[m0:m0 + 8].contiguous()
        y = torch.empty(8, 16, dtype=BF, device=DEV)
        hip.linear_fp8(x, w8, scales, y)
        assert torch.equal(y.float(), want[m0:m0 + 8])
    assert want.abs().max().item() == 448.0 and (want.abs()[want != 0].min().item() == 2.0 ** -9)


@pytest.mark.parametrize("N,K", [(1280, 8192), (8192, 1024), (7168, 8192), (8192, 3584), (16032, 8192), (3072, 2048),
                                 (1001, 528), (24, 64)])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 5, 8, 16, 17, 300])
def test_linear_fp8(hip, M, N, K):
    """Decode (one row: matrix-vector kernel; 2 to 16 rows: matrix-core bands; fp8 weights streamed once) and prefill
    (M > 16: expanded to bf16 in scratch + matrix-core GEMM + column scaling) against the oracle's
    F.linear(x, w8.to(bf16)) * scales."""
    if M == 300 and N * K > 30e6:
        M = 64
    x = rnd(M, K, seed=40)
    w8, scales = O.quantize_fp8_rowwise(rnd(N, K, seed=41, scale=0.02, dtype=torch.float32), BF)
    y = torch.empty(M, N, dtype=BF, device=DEV)
    hip.linear_fp8(x, w8, scales, y)
    want = O.linear_fp8(x, w8, scales)
    # two roundings (the sum, then the scaled sum): a one-step difference in the first can survive as one or,
    # through double rounding, two steps of the result
    assert_close_ulp(y, want, max_ulp=2, max_frac=0.06, what=f"fp8 linear M={M} N={N} K={K}")
    exact = ((x.double() @ w8.double().T) * scales.double()).to(BF)
    # (the single rounding of the exact product differs from the two roundings of the scheme at about a quarter of the elements, by one step)
    assert_close_ulp(y, exact, max_ulp=2, max_frac=0.4, what="fp8 linear vs fp64")


@pytest.mark.parametrize("M,D,Hq,Hkv,hd,I", [(1, 8192, 8, 1, 128, 3584), (8, 8192, 8, 1, 128, 3584), (3, 4096, 32, 8, 128, 1000),
                                             (5, 2048, 4, 2, 64, 72), (2, 1040, 2, 2, 64, 17), (4, 64, 1, 1, 8, 8),
                                             (16, 4096, 32, 8, 128, 14336), (13, 528, 4, 4, 64, 33)])
def test_linear_fp8_multi_equals_the_separate_calls(hip, M, D, Hq, Hkv, hd, I):
    """Two e4m3 projections per launch with their epilogues: q/k/v rotated and cached as lr_linear_fp8 followed by
    lr_rope_kv_write leaves them, up/gate as lr_linear_fp8 followed by lr_swiglu, plain projections as lr_linear_fp8
    -- bit for bit; rows (2p, 2p + 1) and (p, p + I) of one wave, K below and above the K-split thresholds."""
    Smax, block, pos_value = 40, 64, 23
    NQ = (Hq + 2 * Hkv) * hd
    xa, xb = rnd(M, D, seed=60), rnd(M, D, seed=61)
    wq, sq = O.quantize_fp8_rowwise(rnd(NQ, D, seed=62, scale=0.03, dtype=torch.float32), BF)
    w1, s1 = O.quantize_fp8_rowwise(rnd(2 * I, D, seed=63, scale=0.03, dtype=torch.float32), BF)
    table = O.rope_table(block, hd, 10000.0, BF).to(DEV)
    pos = torch.tensor([pos_value], dtype=torch.int32, device=DEV)
    kc = [rnd(M, Hkv, Smax, hd, seed=64) for _ in range(2)]
    vc = [rnd(M, Hkv, Smax, hd, seed=65) for _ in range(2)]
    # separate calls
    q_ref = torch.empty(M, NQ, dtype=BF, device=DEV)
    hip.linear_fp8(xa, wq, sq, q_ref)
    kv_proj = q_ref[:, Hq * hd:].clone()
    hip.rope_kv_write(q_ref, table, False, pos, kc[0], vc[0], M, 1, Hq, Hkv, hd)
    h = torch.empty(M, 2 * I, dtype=BF, device=DEV)
    hip.linear_fp8(xb, w1, s1, h)
    act_ref = F.silu(h[:, I:]) * h[:, :I]
    # one launch
    q = torch.empty(M, NQ, dtype=BF, device=DEV)
    act = torch.full((M, I), 3.0, dtype=BF, device=DEV)
    hip.linear_fp8_multi((xa, wq, sq, q, hip.rope_kv_epilogue(table, pos, kc[1], vc[1], Hq, Hkv, hd)),
                         (xb, w1, s1, act, hip.EPI_SWIGLU))
    if M == 1:   # the matrix-vector kernel: lr_linear_fp8's own sums
        assert torch.equal(q[:, :Hq * hd], q_ref[:, :Hq * hd]) and torch.equal(q[:, Hq * hd:], kv_proj)
        assert torch.equal(kc[1], kc[0]) and torch.equal(vc[1], vc[0])
        assert torch.equal(act, act_ref)
    else:        # from 2 rows on the matrix-core bands: another summation order, the same roundings
        assert_close_ulp(q, q_ref, max_ulp=2, max_frac=0.1, what="fp8 multi: q/k/v")
        keep = torch.ones(Smax, dtype=torch.bool, device=DEV)
        keep[pos_value] = False
        assert torch.equal(kc[1][:, :, keep], kc[0][:, :, keep]) and torch.equal(vc[1][:, :, keep], vc[0][:, :, keep])
        assert_close_ulp(kc[1][:, :, pos_value].contiguous(), kc[0][:, :, pos_value].contiguous(), max_ulp=2, max_frac=0.1,
                         what="fp8 multi: cached k")
        assert_close_ulp(vc[1][:, :, pos_value].contiguous(), vc[0][:, :, pos_value].contiguous(), max_ulp=2, max_frac=0.1,
                         what="fp8 multi: cached v")
        err = (act.float() - act_ref.float()).abs().max().item()
        assert err <= 2.0 ** -6 * act_ref.float().abs().max().item(), err
        assert (ulp_diff(act, act_ref) > 1).float().mean().item() < 0.05
    # plain projections, one of them with an odd number of rows
    wo, so = O.quantize_fp8_rowwise(rnd(D + 1, Hq * hd, seed=66, scale=0.03, dtype=torch.float32), BF) if (Hq * hd) % 16 == 0 \
        else (None, None)
    if wo is not None:
        y = rnd(M, Hq * hd, seed=67)
        a_ref, a = torch.empty(M, D + 1, dtype=BF, device=DEV), torch.zeros(M, D + 9, dtype=BF, device=DEV)
        hip.linear_fp8(y, wo, so, a_ref)
        m_ref, m = torch.empty(M, NQ, dtype=BF, device=DEV), torch.empty(M, NQ, dtype=BF, device=DEV)
        hip.linear_fp8(xa, wq, sq, m_ref)
        hip.linear_fp8_multi((y, wo, so, a[:, :D + 1], hip.EPI_NONE), (xa, wq, sq, m, hip.EPI_NONE))
        assert bool((a[:, D + 1:] == 0).all())
        if M == 1:
            assert torch.equal(a[:, :D + 1], a_ref) and torch.equal(m, m_ref)
        else:
            assert_close_ulp(a[:, :D + 1].contiguous(), a_ref, max_ulp=2, max_frac=0.1, what="fp8 multi: wo")
            assert_close_ulp(m, m_ref, max_ulp=2, max_frac=0.1, what="fp8 multi: second projection")


def test_rope_kv_write_position_out_of_range_sets_the_error_word(hip):
    """Positions beyond the cache or the RoPE table: the row is left alone, nothing lands in the cache and the
    per-device error word becomes LR_DEV_POS_RANGE (the reference raises an index error, utils.py:55)."""
    B, S, Smax, block, Hq, Hkv, hd = 1, 3, 16, 12, 2, 1, 64
    qkv = rnd(B, S, (Hq + 2 * Hkv) * hd, seed=29)
    before = qkv.clone()
    table = O.rope_table(block, hd, 10000, BF).to(DEV)
    kc = torch.zeros(B, Hkv, Smax, hd, dtype=BF, device=DEV)
    vc = torch.zeros_like(kc)
    word = hip.device_error_word(DEV)
    word.zero_()
    pos = torch.tensor([2, 16, 13], dtype=torch.int32, device=DEV)   # in range; beyond the cache; beyond the table
    hip.rope_kv_write(qkv, table, False, pos, kc, vc, B, S, Hq, Hkv, hd)
    torch.cuda.synchronize()
    assert word.item() == hip.DEV_POS_RANGE
    assert torch.equal(qkv[:, 1:], before[:, 1:]) and not torch.equal(qkv[:, 0], before[:, 0])
    assert bool((kc[:, :, 3:] == 0).all()) and bool((kc[:, :, 2] != 0).any())
    with pytest.raises(hip.LadderHipError):
        hip.raise_on_device_error(DEV)
    assert word.item() == 0      # reported once
    hip.raise_on_device_error(DEV)


# ------------------------------------------------------------------------------------ attention

@pytest.mark.parametrize("B,Hq,Hkv,hd,Smax,pos", [
    (1, 8, 1, 128, 2176, 2048), (1, 8, 1, 128, 2176, 0), (1, 8, 1, 128, 2176, 2175), (8, 8, 1, 128, 2176, 2100),
    (64, 8, 1, 128, 2176, 2111), (2, 32, 8, 128, 1280, 1033), (1, 32, 8, 64, 160, 131), (16, 16, 1, 128, 4160, 4100),
    (3, 4, 4, 64, 40, 17), (2, 8, 4, 128, 264, 200), (1, 16, 1, 128, 520, 519),
    # a cache long enough for more than 64 key chunks (merged by the general loop, not in one round trip), and
    # exactly 32 chunks
    (1, 8, 1, 128, 20000, 19000), (16, 8, 1, 128, 2048, 2047),
])
def test_attn_decode(hip, B, Hq, Hkv, hd, Smax, pos):
    q = rnd(B, Hq * hd, seed=21)
    kc = rnd(B, Hkv, Smax, hd, seed=22)
    vc = rnd(B, Hkv, Smax, hd, seed=23)
    kc[:, :, pos + 1:] = 7.0   # garbage beyond pos must not be read
    vc[:, :, pos + 1:] = -9.0
    p = torch.tensor([pos], dtype=torch.int32, device=DEV)
    y = torch.empty(B, Hq * hd, dtype=BF, device=DEV)
    scratch = torch.empty(hip.attn_decode_scratch_bytes(B, Hq, hd, Smax) // 4, dtype=torch.float32, device=DEV)
    hip.attn_decode(q, kc, vc, p, y, scratch, B, Hq, Hkv, hd)
    mask = (torch.arange(Smax, device=DEV) <= pos).view(1, Smax)
    want = O.sdpa_math(q.view(B, 1, Hq, hd).transpose(1, 2), kc, vc, mask).transpose(1, 2).reshape(B, Hq * hd)
    assert_close_ulp(y, want, max_frac=0.03, what="attn_decode")


@pytest.mark.parametrize("B,Hq,Hkv,hd,Smax,pos,D,I,epi_swiglu", [
    (8, 8, 1, 128, 2176, 2100, 1024, 456, True),     # the 70B rank shard's heads at batch 8
    (16, 32, 8, 128, 1100, 1024, 512, 1000, True),   # Ladder-8B's heads at batch 16
    (5, 4, 2, 64, 300, 0, 264, 72, True),            # first position: one key per sequence
    (16, 8, 8, 64, 520, 519, 136, 4100, False),      # one q head per kv head, a plain projection beside it
    (16, 16, 1, 128, 4224, 4100, 512, 456, True),    # the 405B rank shard's heads: 16 q heads as two groups of 8
    (3, 32, 2, 128, 200, 150, 264, 64, True),
    (1, 2, 1, 128, 64, 63, 64, 16, True),
])
def test_attn_decode_beside_equals_the_two_calls(hip, B, Hq, Hkv, hd, Smax, pos, D, I, epi_swiglu):
    """Attention items and projection bands in one grid: same bits as lr_attn_decode, then lr_linear_multi."""
    q = rnd(B, (Hq + 2 * Hkv) * hd, seed=50)         # q is the head of the fused q/k/v row, as in a decode step
    kc, vc = rnd(B, Hkv, Smax, hd, seed=51), rnd(B, Hkv, Smax, hd, seed=52)
    kc[:, :, pos + 1:] = 7.0
    vc[:, :, pos + 1:] = -9.0
    p = torch.tensor([pos], dtype=torch.int32, device=DEV)
    x = rnd(B, D, seed=53)
    w = rnd(2 * I if epi_swiglu else I, D, seed=54, scale=0.05)
    epi = hip.EPI_SWIGLU if epi_swiglu else hip.EPI_NONE
    nscr = hip.attn_decode_scratch_bytes(B, Hq, hd, Smax) // 4
    y, out = [torch.zeros(B, Hq * hd, dtype=BF, device=DEV) for _ in range(2)], \
        [torch.zeros(B, I, dtype=BF, device=DEV) for _ in range(2)]
    scratch = [torch.zeros(nscr, dtype=torch.float32, device=DEV) for _ in range(2)]
    hip.attn_decode(q, kc, vc, p, y[0], scratch[0], B, Hq, Hkv, hd)
    hip.linear_multi((x, w, out[0], epi))
    assert hip.attn_decode_beside(q, kc, vc, p, y[1], scratch[1], B, Hq, Hkv, hd, (x, w, out[1], epi))
    assert torch.equal(y[1], y[0]) and torch.equal(out[1], out[0])
    mask = (torch.arange(Smax, device=DEV) <= pos).view(1, Smax)
    want = O.sdpa_math(q[:, :Hq * hd].reshape(B, 1, Hq, hd).transpose(1, 2), kc, vc, mask).transpose(1, 2)
    assert_close_ulp(y[1], want.reshape(B, Hq * hd), max_frac=0.03, what="attn_decode_beside")


@pytest.mark.parametrize("B,Hq,Hkv,hd,Smax,pos,D,I", [(8, 8, 1, 128, 2176, 2100, 8192, 456), (2, 8, 1, 128, 600, 599, 1024, 200),
                                                    (16, 32, 8, 128, 300, 17, 512, 72), (5, 16, 1, 128, 520, 400, 2048, 40),
                                                    (4, 4, 2, 64, 100, 99, 272, 24)])
def test_attn_decode_beside_fp8_equals_the_two_calls(hip, B, Hq, Hkv, hd, Smax, pos, D, I):
    """Attention items and the bands of an e4m3 up/gate projection in one grid: same bits as lr_attn_decode, then
    lr_linear_fp8_multi; a single row is declined."""
    q = rnd(B, (Hq + 2 * Hkv) * hd, seed=70)
    kc, vc = rnd(B, Hkv, Smax, hd, seed=71), rnd(B, Hkv, Smax, hd, seed=72)
    p = torch.tensor([pos], dtype=torch.int32, device=DEV)
    x = rnd(B, D, seed=73)
    w8, sc = O.quantize_fp8_rowwise(rnd(2 * I, D, seed=74, scale=0.05, dtype=torch.float32), BF)
    nscr = hip.attn_decode_scratch_bytes(B, Hq, hd, Smax) // 4
    y = [torch.zeros(B, Hq * hd, dtype=BF, device=DEV) for _ in range(2)]
    out = [torch.zeros(B, I, dtype=BF, device=DEV) for _ in range(2)]
    scratch = [torch.zeros(nscr, dtype=torch.float32, device=DEV) for _ in range(2)]
    hip.attn_decode(q, kc, vc, p, y[0], scratch[0], B, Hq, Hkv, hd)
    hip.linear_fp8_multi((x, w8, sc, out[0], hip.EPI_SWIGLU))
    assert hip.attn_decode_beside_fp8(q, kc, vc, p, y[1], scratch[1], B, Hq, Hkv, hd, (x, w8, sc, out[1], hip.EPI_SWIGLU))
    assert torch.equal(y[1], y[0]) and torch.equal(out[1], out[0])
    assert out[1].float().abs().sum().item() > 0
    o1 = torch.full((1, I), 5.0, dtype=BF, device=DEV)
    y1 = torch.full((1, Hq * hd), 5.0, dtype=BF, device=DEV)
    assert not hip.attn_decode_beside_fp8(q[:1], kc[:1], vc[:1], p, y1, scratch[1], 1, Hq, Hkv, hd,
                                          (x[:1], w8, sc, o1, hip.EPI_SWIGLU))
    torch.cuda.synchronize()
    assert bool((o1 == 5.0).all()) and bool((y1 == 5.0).all())


def test_attn_decode_beside_declines_what_it_has_no_kernel_for(hip):
    """More than 16 rows, 32 q heads per kv head, or a projection that writes the cache: False, nothing launched."""
    def run(B, Hq, Hkv, epi=None):
        hd, Smax, D, I = 128, 64, 64, 16
        q = rnd(B, Hq * hd, seed=55)
        kc, vc = rnd(B, Hkv, Smax, hd, seed=56), rnd(B, Hkv, Smax, hd, seed=57)
        p = torch.tensor([3], dtype=torch.int32, device=DEV)
        y = torch.full((B, Hq * hd), 5.0, dtype=BF, device=DEV)
        N = (Hq + 2 * Hkv) * hd if epi is not None else I
        out = torch.full((B, N), 5.0, dtype=BF, device=DEV)
        scratch = torch.zeros(hip.attn_decode_scratch_bytes(B, Hq, hd, Smax) // 4, dtype=torch.float32, device=DEV)
        if epi is not None:
            epi = hip.rope_kv_epilogue(O.rope_table(64, hd, 10000.0, BF).to(DEV), p, kc, vc, Hq, Hkv, hd)
        ok = hip.attn_decode_beside(q, kc, vc, p, y, scratch, B, Hq, Hkv, hd,
                                    (rnd(B, D, seed=58), rnd(N, D, seed=59), out, hip.EPI_NONE if epi is None else epi))
        torch.cuda.synchronize()
        return ok, bool((y == 5.0).all()) and bool((out == 5.0).all())
    assert run(17, 8, 1) == (False, True)
    assert run(4, 32, 1) == (False, True)
    assert run(4, 8, 1, epi="rope") == (False, True)
    assert run(4, 8, 1)[0] is True


@pytest.mark.parametrize("B,S,Hq,Hkv,hd,Smax,start", [
    (1, 128, 8, 1, 128, 136, 0), (2, 100, 4, 2, 64, 160, 0), (1, 300, 8, 1, 128, 512, 100), (1, 2048, 8, 1, 128, 2176, 0),
    (3, 65, 32, 8, 64, 72, 0),
    # one q head per kv head (4 query tiles per workgroup), odd group sizes, 16 heads per kv head, S below the
    # matrix-core kernel's threshold, a single query tile with a long history
    (2, 130, 4, 4, 128, 136, 0), (1, 97, 6, 2, 64, 104, 3), (1, 64, 16, 1, 128, 64, 0), (2, 9, 8, 2, 64, 16, 0),
    (1, 17, 8, 1, 128, 1024, 1000),
])
def test_attn_prefill(hip, B, S, Hq, Hkv, hd, Smax, start):
    q = rnd(B, S, Hq * hd, seed=24)
    kc = rnd(B, Hkv, Smax, hd, seed=25)
    vc = rnd(B, Hkv, Smax, hd, seed=26)
    pos = torch.arange(start, start + S, dtype=torch.int32, device=DEV)
    y = torch.empty(B, S, Hq * hd, dtype=BF, device=DEV)
    hip.attn_prefill(q, kc, vc, pos, y, B, S, Hq, Hkv, hd)
    mask = torch.arange(Smax, device=DEV).view(1, Smax) <= pos.view(S, 1)
    want = O.sdpa_math(q.view(B, S, Hq, hd).transpose(1, 2), kc, vc, mask).transpose(1, 2).reshape(B, S, Hq * hd)
    assert_close_ulp(y, want, max_frac=0.03, what="attn_prefill")


@pytest.mark.parametrize("qscale", [4.0, 12.0])
def test_attn_prefill_large_scores(hip, qscale):
    """Scores with a standard deviation of 4 and 12: the running maximum of a query jumps by more than the kernel lets
    its reference point lag, on tiles late in the history too, so accumulators are rescaled in mid-stream; and the
    softmax is nearly one-hot at the larger scale."""
    B, S, Hq, Hkv, hd, Smax = 2, 700, 8, 2, 128, 704
    q = rnd(B, S, Hq * hd, seed=124, scale=qscale)
    kc = rnd(B, Hkv, Smax, hd, seed=125)
    vc = rnd(B, Hkv, Smax, hd, seed=126)
    pos = torch.arange(S, dtype=torch.int32, device=DEV)
    y = torch.empty(B, S, Hq * hd, dtype=BF, device=DEV)
    hip.attn_prefill(q, kc, vc, pos, y, B, S, Hq, Hkv, hd)
    mask = torch.arange(Smax, device=DEV).view(1, Smax) <= pos.view(S, 1)
    want = O.sdpa_math(q.view(B, S, Hq, hd).transpose(1, 2), kc, vc, mask).transpose(1, 2).reshape(B, S, Hq * hd)
    assert_close_ulp(y, want, max_frac=0.03, what="attn_prefill, large scores")


def test_attn_prefill_equal_sequences_give_equal_rows(hip):
    """Eight copies of one sequence: every copy's output is the same bit pattern, on repeated calls too (the kernel
    has no race and reads no register before its producer has finished)."""
    B, S, Hq, Hkv, hd, Smax = 8, 1024, 32, 8, 128, 1072
    q = rnd(1, S, Hq * hd, seed=224).repeat(B, 1, 1).contiguous()
    kc = rnd(1, Hkv, Smax, hd, seed=225).repeat(B, 1, 1, 1).contiguous()
    vc = rnd(1, Hkv, Smax, hd, seed=226).repeat(B, 1, 1, 1).contiguous()
    pos = torch.arange(S, dtype=torch.int32, device=DEV)
    first = None
    for _ in range(3):
        y = torch.empty(B, S, Hq * hd, dtype=BF, device=DEV)
        hip.attn_prefill(q, kc, vc, pos, y, B, S, Hq, Hkv, hd)
        assert all(torch.equal(y[0], y[b]) for b in range(1, B))
        first = y if first is None else first
        assert torch.equal(y, first)


# ------------------------------------------------------------------------------------ argmax

def test_argmax_lowest_index_on_ties(hip):
    B, V = 4, 128256
    lg = rnd(B, V, seed=27, scale=0.04)
    lg[0, [77, 100000]] = 5.0
    lg[1, [128255, 5]] = 5.0
    lg[2, 128255] = 9.0
    out = torch.empty(B, 1, dtype=torch.int32, device=DEV)
    hip.argmax(lg, out)
    want = torch.argmax(lg, dim=-1, keepdim=True).to(torch.int32)
    assert torch.equal(out, want) and out.flatten().tolist()[:3] == [77, 5, 128255]
    # last position of [B, S, V] logits: a strided [B, V] view; and a vocab that is not a multiple of 8
    lg3 = rnd(2, 3, 1008, seed=28)
    hip.argmax(lg3[:, -1, :1003], out[:2])
    assert torch.equal(out[:2], lg3[:, -1, :1003].argmax(-1, keepdim=True).to(torch.int32))


def test_torch_argmax_itself_returns_first_maximum_on_this_device():
    """The oracle's greedy() relies on it."""
    lg = torch.zeros(1, 16032, dtype=BF, device=DEV)
    lg[0, [15000, 40, 9000]] = 1.0
    assert torch.argmax(lg, -1).item() == 40


# ------------------------------------------------------------------------------------ stream read

def test_stream_read_runs_and_leaves_the_sink_alone(hip):
    """The measurement aid reads the buffer and writes nothing (the xor of the data is not the magic value)."""
    buf = torch.full((64 << 20,), 3, dtype=torch.uint8, device=DEV)
    sink = torch.full((1,), 1234, dtype=torch.int32, device=DEV)
    for _ in range(3):
        hip.stream_read(buf, sink)
    torch.cuda.synchronize()
    assert sink.item() == 1234
    with pytest.raises(hip.LadderHipError):
        hip.stream_read(buf[:1024], sink)
