"""ctypes binding of libladder_hip.so (declared in include/ladder_hip.h).

There is no fallback: if the shared library is missing or a call returns an error code the
caller gets an exception.  Tensors are passed as raw device pointers plus sizes; the stream is
torch's current HIP stream, so calls made under torch.cuda.graph() are captured."""
import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libladder_hip.so")
_lib = None

# name -> (restype, argtypes); mirrors include/ladder_hip.h
_PROTOS = {
    "lr_version": (c_int, []),
    "lr_error_string": (c_char_p, [c_int]),
    "lr_embed": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "lr_add": (c_int, [c_void_p, c_void_p, c_float, c_void_p, c_int64, c_void_p]),
    "lr_add_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float,
                               c_void_p]),
    "lr_ladder_norms": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                c_float, c_void_p]),
    "lr_linear": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    "lr_linear_tuned": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int,
                                c_void_p]),
    "lr_linear_multi": (c_int, [c_void_p, c_int, c_int, c_void_p]),
    "lr_linear_swiglu_out": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p,
                                     c_size_t, c_void_p]),
    "lr_linear_fp8_scratch_bytes": (c_size_t, [c_int, c_int, c_int]),
    "lr_linear_fp8_multi": (c_int, [c_void_p, c_int, c_int, c_void_p]),
    "lr_linear_fp8": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p,
                              c_size_t, c_void_p]),
    "lr_swiglu": (c_int, [c_void_p, c_int64, c_void_p, c_int, c_int, c_void_p]),
    "lr_rope_kv_write": (c_int, [c_void_p, c_int64, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                 c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "lr_kv_update": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int,
                             c_int, c_int, c_int, c_void_p, c_void_p]),
    "lr_linear_rope_kv": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p,
                                  c_void_p]),
    "lr_attn_decode_scratch_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "lr_attn_decode": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int,
                               c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "lr_attn_decode_beside": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int,
                                      c_int, c_int, c_int, c_void_p, c_size_t, c_void_p, c_int, c_void_p]),
    "lr_attn_decode_beside_fp8": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int,
                                          c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p, c_int, c_void_p]),
    "lr_attn_decode_static": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int,
                                      c_int, c_int, c_int, c_void_p]),
    "lr_attn_prefill": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int,
                                c_int, c_int, c_int, c_int, c_void_p]),
    "lr_argmax": (c_int, [c_void_p, c_int64, c_void_p, c_int, c_int, c_void_p]),
    "lr_stream_read": (c_int, [c_void_p, c_size_t, c_void_p, c_void_p]),
    "lr_sample_topk": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int, c_int, c_float, c_int, c_void_p, c_int64,
                               c_void_p, c_void_p]),
    "lr_advance": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "lr_ladder_step_workspace_bytes": (c_size_t, [c_void_p, c_int]),
    "lr_ladder_step_init": (c_int, [c_void_p, c_int, c_void_p, c_size_t, c_void_p]),
    "lr_ladder_decode_step": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int, c_void_p,
                                      c_void_p, c_int64, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "lr_ladder_decode_step_fp8": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int,
                                          c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "lr_ladder_step_fail_offset": (c_size_t, []),
    "lr_ladder_step_resident_workgroups": (c_int, [c_void_p, c_int]),
}


class LadderModelDesc(ctypes.Structure):
    """lr_ladder_model_t of include/ladder_hip.h (per-rank sizes)."""
    _fields_ = [(n, c_int32) for n in ("dim", "n_layer", "n_head", "n_kv_head", "head_dim", "ffn", "out_rows", "vocab",
                                       "smax", "block_size")] + [("eps", c_float), ("attention_workgroups", c_int32)] + \
               [(n, c_void_p) for n in ("tok_embeddings", "norm", "output", "freqs_cis", "layers_dev")]


E_UNSUPPORTED = -4   # LR_E_UNSUPPORTED of include/ladder_hip.h


class LadderHipError(RuntimeError):
    pass


def lib_path() -> str:
    return _LIB_PATH


def load():
    """Load the shared library once.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise LadderHipError(
                f"{_LIB_PATH} is missing: build it with `python {os.path.dirname(os.path.dirname(_LIB_PATH))}/build.py` "
                "(hipcc, gfx950).  This package has no CPU or PyTorch fallback.")
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (res, args) in _PROTOS.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def exported_names():
    return list(_PROTOS)


def _check(code: int, what: str):
    if code != 0:
        raise LadderHipError(f"{what} failed: {load().lr_error_string(code).decode()} ({code})")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, dtype=torch.bfloat16) -> int:
    assert t.is_cuda, "libladder_hip works on device tensors only"
    assert t.dtype == dtype, f"expected {dtype}, got {t.dtype}"
    return t.data_ptr()


def _rows_ld(t: torch.Tensor):
    """View a tensor as [rows, cols] with unit column stride; returns (rows, cols, row stride)."""
    assert t.stride(-1) == 1
    cols = t.shape[-1]
    if t.dim() == 1:
        return 1, cols, cols
    rows = t.numel() // cols
    ld = t.stride(-2)
    # every leading dimension must be a multiple walk of the row stride
    exp = ld
    for d in range(t.dim() - 2, -1, -1):
        assert t.shape[d] == 1 or t.stride(d) == exp, "tensor is not a regular [rows, cols] matrix"
        exp *= t.shape[d]
    return rows, cols, ld


# ------------------------------------------------------------------------------------------------
# thin typed wrappers
# ------------------------------------------------------------------------------------------------

def embed(table: torch.Tensor, idx: torch.Tensor, out: torch.Tensor):
    assert idx.dtype in (torch.int64, torch.int32) and idx.is_contiguous() and idx.is_cuda
    vocab, dim = table.shape
    _check(load().lr_embed(_dev(table), idx.data_ptr(), int(idx.dtype == torch.int64), _dev(out), idx.numel(), dim,
                           vocab, _stream()), "lr_embed")
    return out


def add(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor, b_div: float = 1.0):
    assert a.is_contiguous() and b.is_contiguous() and out.is_contiguous() and a.numel() == b.numel() == out.numel()
    _check(load().lr_add(_dev(a), _dev(b), float(b_div), _dev(out), a.numel(), _stream()), "lr_add")
    return out


def add_rmsnorm(resid_in, d1, d2, gain, resid_out, normed_out, eps: float):
    dim = resid_in.shape[-1]
    rows = resid_in.numel() // dim
    for t in (resid_in, d1, d2, resid_out, normed_out):
        assert t is None or (t.is_contiguous() and t.numel() == rows * dim)
    assert gain.numel() == dim
    p = lambda t: None if t is None else _dev(t)
    _check(load().lr_add_rmsnorm(_dev(resid_in), p(d1), p(d2), _dev(gain), p(resid_out), _dev(normed_out), rows, dim,
                                 float(eps), _stream()), "lr_add_rmsnorm")
    return normed_out


def ladder_norms(resid_in, d1, d2, gain1, gain2, resid_out, normed1, normed2, eps: float):
    """Both residual updates and both norms of a ladder block (lr_ladder_norms)."""
    dim = resid_in.shape[-1]
    rows = resid_in.numel() // dim
    for t in (resid_in, d1, d2, resid_out, normed1, normed2):
        assert t is None or (t.is_contiguous() and t.numel() == rows * dim)
    assert gain1.numel() == dim and gain2.numel() == dim
    p = lambda t: None if t is None else _dev(t)
    _check(load().lr_ladder_norms(_dev(resid_in), p(d1), p(d2), _dev(gain1), _dev(gain2), _dev(resid_out), _dev(normed1),
                                  _dev(normed2), rows, dim, float(eps), _stream()), "lr_ladder_norms")


def linear(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, act_swiglu: bool = False, gemv_cfg: int = 0):
    """out[M, N] = x[M, K] @ w[N, K]^T (x = [u | g] of width 2K when act_swiglu).  gemv_cfg != 0 goes
    through lr_linear_tuned (an explicit GEMV launch configuration for this one call)."""
    M, xc, ldx = _rows_ld(x)
    N, K = w.shape
    assert w.is_contiguous() and xc == (2 * K if act_swiglu else K), (x.shape, w.shape, act_swiglu)
    Mo, No, ldy = _rows_ld(out)
    assert (Mo, No) == (M, N), (out.shape, M, N)
    if gemv_cfg:
        _check(load().lr_linear_tuned(_dev(x), ldx, _dev(w), _dev(out), ldy, M, N, K, int(act_swiglu), int(gemv_cfg),
                                      _stream()), "lr_linear_tuned")
    else:
        _check(load().lr_linear(_dev(x), ldx, _dev(w), _dev(out), ldy, M, N, K, int(act_swiglu), _stream()),
               "lr_linear")
    return out


_FP8_SCRATCH = {}


class _RopeKv(ctypes.Structure):   # lr_rope_kv_t
    _fields_ = [("table", c_void_p), ("pos", c_void_p), ("k_cache", c_void_p), ("v_cache", c_void_p), ("err", c_void_p),
                ("n_head", c_int32), ("n_kv_head", c_int32), ("head_dim", c_int32), ("smax", c_int32),
                ("block_size", c_int32)]


class _Projection(ctypes.Structure):   # lr_projection_t
    _fields_ = [("x", c_void_p), ("ldx", c_int64), ("w", c_void_p), ("y", c_void_p), ("ldy", c_int64),
                ("N", c_int32), ("K", c_int32), ("epilogue", c_int32), ("rope", ctypes.POINTER(_RopeKv))]


EPI_NONE, EPI_SWIGLU, EPI_ROPE_KV = 0, 1, 2


def rope_kv_epilogue(table, pos, k_cache, v_cache, Hq, Hkv, hd, n_pos=1):
    """The descriptor an EPI_ROPE_KV projection of linear_multi carries (decode: one token per sequence), or
    linear_rope_kv (prefill: `n_pos` tokens per sequence)."""
    assert pos.dtype == torch.int32 and pos.is_cuda and pos.numel() == n_pos
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape == v_cache.shape
    _, hkv_c, Smax, hd_c = k_cache.shape
    assert hkv_c == Hkv and hd_c == hd and table.is_contiguous() and table.shape[-2:] == (hd // 2, 2)
    return _RopeKv(_dev(table), pos.data_ptr(), _dev(k_cache), _dev(v_cache),
                   device_error_word(k_cache.device).data_ptr(), Hq, Hkv, hd, Smax, table.shape[0])


def linear_rope_kv(x, w, out, table, pos, k_cache, v_cache, B, S, Hq, Hkv, hd):
    """The fused q/k/v projection of B * S rows, rotated and cached on its way out (lr_linear_rope_kv): what
    linear(x, w, out) followed by rope_kv_write(out, table, False, pos, ...) leaves."""
    M, K, ldx = _rows_ld(x)
    Mo, N, ldy = _rows_ld(out)
    assert M == Mo == B * S and w.is_contiguous() and tuple(w.shape) == ((Hq + 2 * Hkv) * hd, K) and N == w.shape[0]
    assert B <= k_cache.shape[0]
    rope = rope_kv_epilogue(table, pos, k_cache, v_cache, Hq, Hkv, hd, n_pos=S)
    _check(load().lr_linear_rope_kv(_dev(x), ldx, _dev(w), _dev(out), ldy, M, K, S, ctypes.byref(rope), _stream()),
           "lr_linear_rope_kv")
    return out


def linear_multi(*projections):
    """One launch of the weight-streaming kernel for one or two projections of the same M <= 64 rows.
    Each projection is (x [M, K], w [N, K], out, epilogue): EPI_NONE -> out [M, N] = x @ w^T;
    EPI_SWIGLU -> w holds [up; gate] rows and out [M, N / 2] = silu(gate) * up; or, for the fused q/k/v
    projection of a decode step, (x, w, out, rope_kv_epilogue(...)): q rotated in out, k and v into the cache
    (lr_linear_multi)."""
    arr, M, _keep = _projection_array(projections)
    _check(load().lr_linear_multi(ctypes.cast(arr, c_void_p), len(projections), M, _stream()), "lr_linear_multi")


def _projection_array(projections):
    arr = (_Projection * len(projections))()
    M = None
    keep = []
    for i, (x, w, out, epi) in enumerate(projections):
        rope = None
        if isinstance(epi, _RopeKv):
            rope, epi = epi, EPI_ROPE_KV
            keep.append(rope)
        m, K, ldx = _rows_ld(x)
        N, Kw = w.shape
        Mo, No, ldy = _rows_ld(out)
        assert w.is_contiguous() and Kw == K and Mo == m and No == (N // 2 if epi == EPI_SWIGLU else N), \
            (x.shape, w.shape, out.shape, epi)
        assert M is None or M == m
        M = m
        arr[i] = _Projection(_dev(x), ldx, _dev(w), _dev(out), ldy, N, K, epi,
                             ctypes.pointer(rope) if rope is not None else None)
    return arr, M, keep


class _ProjectionFp8(ctypes.Structure):
    """lr_projection_fp8_t of include/ladder_hip.h."""
    _fields_ = [("x", c_void_p), ("ldx", c_int64), ("w8", c_void_p), ("scales", c_void_p), ("y", c_void_p),
                ("ldy", c_int64), ("N", c_int32), ("K", c_int32), ("epilogue", c_int32), ("rope", ctypes.POINTER(_RopeKv))]


def linear_fp8_multi(*projections):
    """linear_multi for weight-only e4m3 projections of the same M <= 16 rows (lr_linear_fp8_multi).  Each projection
    is (x [M, K], w8 [N, K] float8_e4m3fn, scales [N], out, epilogue), epilogue as in linear_multi."""
    arr, M, _keep = _projection_fp8_array(projections)
    _check(load().lr_linear_fp8_multi(ctypes.cast(arr, c_void_p), len(projections), M, _stream()), "lr_linear_fp8_multi")


def attn_decode_beside_fp8(q, k_cache, v_cache, pos, y, scratch, B, Hq, Hkv, hd, projection) -> bool:
    """attn_decode and linear_fp8_multi(projection) in one launch (lr_attn_decode_beside_fp8); False, with nothing
    launched, when the library has no such kernel for the shape (a single row among them)."""
    _, _, ldq = _rows_ld(q)
    _, _, ldy = _rows_ld(y)
    Smax = k_cache.shape[2]
    assert pos.dtype == torch.int32 and pos.numel() == 1 and scratch.dtype == torch.float32
    arr, M, _keep = _projection_fp8_array((projection,))
    rc = load().lr_attn_decode_beside_fp8(_dev(q), ldq, _dev(k_cache), _dev(v_cache), pos.data_ptr(), _dev(y), ldy, B,
                                          Hq, Hkv, hd, Smax, scratch.data_ptr(), scratch.numel() * 4,
                                          ctypes.cast(arr, c_void_p), M, _stream())
    if rc == E_UNSUPPORTED:
        return False
    _check(rc, "lr_attn_decode_beside_fp8")
    return True


def _projection_fp8_array(projections):
    arr = (_ProjectionFp8 * len(projections))()
    M = None
    keep = []
    for i, (x, w8, scales, out, epi) in enumerate(projections):
        rope = None
        if isinstance(epi, _RopeKv):
            rope, epi = epi, EPI_ROPE_KV
            keep.append(rope)
        m, K, ldx = _rows_ld(x)
        N, Kw = w8.shape
        Mo, No, ldy = _rows_ld(out)
        assert w8.dtype == torch.float8_e4m3fn and w8.is_contiguous() and w8.is_cuda and Kw == K
        assert scales.dtype == torch.bfloat16 and scales.numel() == N and scales.is_contiguous()
        assert Mo == m and No == (N // 2 if epi == EPI_SWIGLU else N), (x.shape, w8.shape, out.shape, epi)
        assert M is None or M == m
        M = m
        arr[i] = _ProjectionFp8(_dev(x), ldx, w8.data_ptr(), _dev(scales), _dev(out), ldy, N, K, epi,
                                ctypes.pointer(rope) if rope is not None else None)
    return arr, M, keep


def linear_fp8(x: torch.Tensor, w8: torch.Tensor, scales: torch.Tensor, out: torch.Tensor):
    """out[M, N] = (x[M, K] @ w8[N, K]^T rounded to bf16) * scales[N]: weight-only e4m3 linear.  For M > 16 the
    expanded weights go through a per-device scratch buffer that grows to the largest matrix seen (allocated
    here, outside the library; allocate it before capturing a graph by running the shape once)."""
    M, K, ldx = _rows_ld(x)
    N, Kw = w8.shape
    assert w8.dtype == torch.float8_e4m3fn and w8.is_contiguous() and Kw == K and w8.is_cuda
    assert scales.dtype == torch.bfloat16 and scales.numel() == N and scales.is_contiguous()
    Mo, No, ldy = _rows_ld(out)
    assert (Mo, No) == (M, N), (out.shape, M, N)
    lib = load()
    need = int(lib.lr_linear_fp8_scratch_bytes(M, N, K))
    scratch = None
    if need:
        # one expansion buffer per (device, stream): calls on one stream are ordered and share it; calls on two
        # streams (a block's attention and MLP chains with overlap_modules) expand different matrices at once
        key = (x.device, _stream())
        scratch = _FP8_SCRATCH.get(key)
        if scratch is None or scratch.numel() < need:
            scratch = _FP8_SCRATCH[key] = torch.empty(need, dtype=torch.uint8, device=x.device)
    _check(lib.lr_linear_fp8(_dev(x), ldx, w8.data_ptr(), _dev(scales), _dev(out), ldy, M, N, K,
                             None if scratch is None else scratch.data_ptr(), need, _stream()), "lr_linear_fp8")
    return out


def linear_swiglu(h: torch.Tensor, w: torch.Tensor, out: torch.Tensor, act: torch.Tensor = None):
    """out = (silu(g) * u) @ w^T for h = [u | g].  Up to 4 rows the activation is fused into the
    weight-streaming GEMV; above that it is materialised once (in `act`, or a new tensor) and fed to
    the plain MFMA GEMM, whose operand loader is then a pure copy."""
    M, two_k, _ = _rows_ld(h)
    if M <= 4:
        return linear(h, w, out, act_swiglu=True)
    if act is None:
        act = h.new_empty(M, two_k // 2)
    swiglu(h, act)
    return linear(act, w, out)


def linear_swiglu_out(x: torch.Tensor, w1: torch.Tensor, act: torch.Tensor, scratch: torch.Tensor = None):
    """act[M, I] = silu(g) * u for [u | g] = x @ w1^T, w1 = [up; gate] rows: the activation is applied in the
    projection's epilogue where the shape allows (lr_linear_swiglu_out); `scratch` [M, 2 I] serves the rest."""
    M, K, ldx = _rows_ld(x)
    N, Kw = w1.shape
    Mo, Io, ldy = _rows_ld(act)
    assert w1.is_contiguous() and Kw == K and N % 2 == 0 and (Mo, Io) == (M, N // 2), (x.shape, w1.shape, act.shape)
    sp, sb = (None, 0) if scratch is None else (_dev(scratch), scratch.numel() * scratch.element_size())
    _check(load().lr_linear_swiglu_out(_dev(x), ldx, _dev(w1), _dev(act), ldy, M, N, K, sp, sb, _stream()),
           "lr_linear_swiglu_out")
    return act


def module_linear(x: torch.Tensor, mod, out: torch.Tensor):
    """mod(x) for an nn.Linear (bf16 weight) or a weight-only fp8 replacement (`weight` e4m3 + `scales`)."""
    scales = getattr(mod, "scales", None)
    if scales is not None:
        return linear_fp8(x, mod.weight, scales, out)
    return linear(x, mod.weight, out)


def module_linear_swiglu(h: torch.Tensor, mod, out: torch.Tensor, act: torch.Tensor = None):
    """mod(silu(g) * u) for h = [u | g]."""
    scales = getattr(mod, "scales", None)
    if scales is None:
        return linear_swiglu(h, mod.weight, out, act)
    M, two_k, _ = _rows_ld(h)
    if act is None:
        act = h.new_empty(M, two_k // 2)
    swiglu(h, act)
    return linear_fp8(act, mod.weight, scales, out)


def swiglu(h: torch.Tensor, out: torch.Tensor):
    rows, two_i, ldh = _rows_ld(h)
    assert out.is_contiguous() and out.numel() == rows * (two_i // 2)
    _check(load().lr_swiglu(_dev(h), ldh, _dev(out), rows, two_i // 2, _stream()), "lr_swiglu")
    return out


def device_error_word(device) -> torch.Tensor:
    """One int32 word per device that kernels set (never clear) when they meet a condition only the
    device can see -- a position outside the KV cache or the RoPE table.  Read by
    raise_on_device_error() at the caller's next synchronisation point."""
    key = torch.device(device)
    if key.index is None:
        key = torch.device("cuda", torch.cuda.current_device())
    w = _ERR_WORDS.get(key)
    if w is None:
        w = _ERR_WORDS[key] = torch.zeros(1, dtype=torch.int32, device=key)
    return w


_ERR_WORDS = {}
DEV_WAIT_EXPIRED, DEV_POS_RANGE = 1, 2
_DEV_ERR_TEXT = {DEV_WAIT_EXPIRED: "a bounded cross-workgroup wait of the decode-step kernel expired",
                 DEV_POS_RANGE: "a position outside the KV cache or the RoPE table was used"}


def raise_on_device_error(device=None, fused_steps=()):
    """Synchronising check of the device-side error words: the per-device word of the per-op kernels
    and the failure word of every FusedLadderStep given.  Raises LadderHipError and clears the
    per-device word (a failed step workspace must be reset by its owner)."""
    words = list(_ERR_WORDS.items()) if device is None else [(torch.device(device), device_error_word(device))]
    for dev, w in words:
        code = int(w.item())
        if code:
            w.zero_()
            raise LadderHipError(f"device-side error on {dev}: {_DEV_ERR_TEXT.get(code, code)}")
    for fs in fused_steps:
        code = fs.fail_code() if fs is not None else 0
        if code:
            raise LadderHipError(f"decode-step kernel failed: {_DEV_ERR_TEXT.get(code, code)}; "
                                 "its workspace has to be initialised again (FusedLadderStep.reset)")


def rope_kv_write(qkv, table, table_is_gathered, pos, k_cache, v_cache, B, S, Hq, Hkv, hd):
    rows, cols, ld = _rows_ld(qkv)
    assert rows == B * S and pos.dtype == torch.int32 and pos.is_cuda and pos.numel() == S
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape == v_cache.shape
    Bmax, hkv_c, Smax, hd_c = k_cache.shape
    assert B <= Bmax and hkv_c == Hkv and hd_c == hd and table.is_contiguous() and table.shape[-2:] == (hd // 2, 2)
    _check(load().lr_rope_kv_write(_dev(qkv), ld, _dev(table), int(bool(table_is_gathered)), pos.data_ptr(),
                                   _dev(k_cache), _dev(v_cache), B, S, Hq, Hkv, hd, Smax, table.shape[0],
                                   device_error_word(qkv.device).data_ptr(), _stream()),
           "lr_rope_kv_write")


def kv_update(k_val, v_val, pos, k_cache, v_cache):
    """KVCache.update: k_cache[:B, :, pos] = k_val ([B, H, S, hd], any strides with a dense last dimension)."""
    B, H, S, hd = k_val.shape
    assert v_val.shape == k_val.shape and v_val.stride() == k_val.stride() and k_val.stride(-1) == 1
    assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.shape == v_cache.shape
    Bmax, Hc, Smax, hdc = k_cache.shape
    assert B <= Bmax and Hc == H and hdc == hd and pos.dtype == torch.int32 and pos.is_cuda and pos.numel() == S
    sb, sh, ss, _ = k_val.stride()
    _check(load().lr_kv_update(_dev(k_val), _dev(v_val), sb, sh, ss, pos.data_ptr(), _dev(k_cache), _dev(v_cache), B, H,
                               S, hd, Smax, device_error_word(k_val.device).data_ptr(), _stream()), "lr_kv_update")


def attn_decode_scratch_bytes(B, Hq, hd, Smax) -> int:
    return int(load().lr_attn_decode_scratch_bytes(B, Hq, hd, Smax))


def attn_decode(q, k_cache, v_cache, pos, y, scratch, B, Hq, Hkv, hd):
    _, _, ldq = _rows_ld(q)
    _, _, ldy = _rows_ld(y)
    Smax = k_cache.shape[2]
    assert pos.dtype == torch.int32 and pos.numel() == 1 and scratch.dtype == torch.float32
    _check(load().lr_attn_decode(_dev(q), ldq, _dev(k_cache), _dev(v_cache), pos.data_ptr(), _dev(y), ldy, B, Hq, Hkv,
                                 hd, Smax, scratch.data_ptr(), scratch.numel() * 4, _stream()), "lr_attn_decode")
    return y


def attn_decode_beside(q, k_cache, v_cache, pos, y, scratch, B, Hq, Hkv, hd, projection) -> bool:
    """attn_decode and linear_multi(projection) in one launch (lr_attn_decode_beside); the two must not depend
    on each other.  False, with nothing launched, when the library has no such kernel for the shape."""
    _, _, ldq = _rows_ld(q)
    _, _, ldy = _rows_ld(y)
    Smax = k_cache.shape[2]
    assert pos.dtype == torch.int32 and pos.numel() == 1 and scratch.dtype == torch.float32
    arr, M, _keep = _projection_array((projection,))
    rc = load().lr_attn_decode_beside(_dev(q), ldq, _dev(k_cache), _dev(v_cache), pos.data_ptr(), _dev(y), ldy, B, Hq,
                                      Hkv, hd, Smax, scratch.data_ptr(), scratch.numel() * 4,
                                      ctypes.cast(arr, c_void_p), M, _stream())
    if rc == E_UNSUPPORTED:
        return False
    _check(rc, "lr_attn_decode_beside")
    return True


ATTN_DECODE_STATIC_MAX_BYTES = 32 << 20   # LR_ATTN_DECODE_STATIC_MAX_BYTES of include/ladder_hip.h


def attn_decode_static(q, k_cache, v_cache, pos, y, B, Hq, Hkv, hd):
    """lr_attn_decode with the partial results in the library's own fixed device array: nothing is allocated."""
    _, _, ldq = _rows_ld(q)
    _, _, ldy = _rows_ld(y)
    Smax = k_cache.shape[2]
    assert pos.dtype == torch.int32 and pos.numel() == 1
    _check(load().lr_attn_decode_static(_dev(q), ldq, _dev(k_cache), _dev(v_cache), pos.data_ptr(), _dev(y), ldy, B, Hq,
                                        Hkv, hd, Smax, _stream()), "lr_attn_decode_static")
    return y


def attn_prefill(q, k_cache, v_cache, pos, y, B, S, Hq, Hkv, hd):
    _, _, ldq = _rows_ld(q)
    _, _, ldy = _rows_ld(y)
    Smax = k_cache.shape[2]
    assert pos.dtype == torch.int32 and pos.numel() == S
    _check(load().lr_attn_prefill(_dev(q), ldq, _dev(k_cache), _dev(v_cache), pos.data_ptr(), _dev(y), ldy, B, S, Hq,
                                  Hkv, hd, Smax, _stream()), "lr_attn_prefill")
    return y


def stream_read(buf: torch.Tensor, sink: torch.Tensor):
    """One streaming read of `buf` by the whole GPU (measurement aid: the machine's read ceiling)."""
    assert buf.is_cuda and buf.is_contiguous() and sink.is_cuda and sink.dtype == torch.int32
    _check(load().lr_stream_read(buf.data_ptr(), buf.numel() * buf.element_size(), sink.data_ptr(), _stream()),
           "lr_stream_read")


def argmax(logits: torch.Tensor, out: torch.Tensor):
    B, V, ld = _rows_ld(logits)
    assert out.dtype == torch.int32 and out.numel() == B and out.is_cuda
    _check(load().lr_argmax(_dev(logits), ld, out.data_ptr(), B, V, _stream()), "lr_argmax")
    return out


def sample_topk(logits: torch.Tensor, noise: torch.Tensor, temperature: float, top_k, out: torch.Tensor,
                probs: torch.Tensor = None):
    """Temperature / top-k / softmax / exponential-race draw of benchmark.py:58-77 on bf16 rows [B, V];
    `noise` are the caller's Exp(1) draws (bf16 [B, V]); writes int32 tokens to `out` (and bf16 `probs`)."""
    B, V, ld = _rows_ld(logits)
    assert noise.dtype == torch.bfloat16 and noise.is_cuda and noise.shape == (B, V) and noise.stride(1) == 1
    assert out.dtype == torch.int32 and out.numel() == B and out.is_cuda
    if probs is not None:
        assert probs.dtype == torch.bfloat16 and probs.is_cuda and probs.shape == (B, V) and probs.stride(1) == 1
    _check(load().lr_sample_topk(_dev(logits), ld, noise.data_ptr(), noise.stride(0), B, V, float(temperature),
                                 int(top_k) if top_k is not None else 0,
                                 None if probs is None else probs.data_ptr(), 0 if probs is None else probs.stride(0),
                                 out.data_ptr(), _stream()), "lr_sample_topk")
    return out


def advance(cur_token, next_token, pos, B, history=None, pos0=0):
    """cur_token <- next_token, history[:, pos - pos0] <- next_token, pos += 1, all on the device."""
    p = lambda t: None if t is None else t.data_ptr()
    for t in (cur_token, next_token, pos, history):
        assert t is None or (t.dtype == torch.int32 and t.is_cuda)
    ld, n = (history.stride(0), history.shape[1]) if history is not None else (0, 0)
    _check(load().lr_advance(p(cur_token), p(next_token), p(pos), B, p(history), ld, n, int(pos0), _stream()),
           "lr_advance")


def _ladder_model_desc(model, attention_workgroups: int = 0):
    """lr_ladder_model_t for `model` (this rank's sizes), its device table of per-layer pointers, and the tensors
    whose addresses they hold."""
    cfg = model.config
    dev = model.output.weight.device
    fp8 = model.output.weight.dtype == torch.float8_e4m3fn
    rows, keep = [], []
    for blk in model.layers:
        lins = [blk.attention.wqkv, blk.attention.wo, blk.feed_forward.w1, blk.feed_forward.w2]
        if fp8:
            for lin in lins:
                pack_fp8_linear(lin)
        ts = [lin.weight for lin in lins] + [blk.attention_norm.weight, blk.ffn_norm.weight,
                                             blk.attention.kv_cache.k_cache, blk.attention.kv_cache.v_cache]
        for i, t in enumerate(ts):
            want = torch.float8_e4m3fn if fp8 and i < 4 else torch.bfloat16
            assert t.is_contiguous() and t.dtype == want and t.device == dev
        keep.append(ts + ([lin.scales for lin in lins] if fp8 else []))
        rows.append([t.data_ptr() for t in ts])
    if fp8:
        pack_fp8_linear(model.output)
        keep.append(model.output.scales)
    layer_table = torch.tensor(rows, dtype=torch.int64).to(dev)
    keep += [model.tok_embeddings.weight, model.norm.weight, model.output.weight, model.freqs_cis]
    desc = LadderModelDesc(
        dim=cfg.dim, n_layer=cfg.n_layer, n_head=cfg.n_head_local, n_kv_head=cfg.n_kv_local, head_dim=cfg.head_dim,
        ffn=cfg.ffn_local, out_rows=cfg.output_rows, vocab=cfg.vocab_size, smax=model.max_seq_length,
        block_size=cfg.block_size, eps=cfg.norm_eps, attention_workgroups=attention_workgroups,
        tok_embeddings=model.tok_embeddings.weight.data_ptr(),
        norm=model.norm.weight.data_ptr(), output=model.output.weight.data_ptr(),
        freqs_cis=model.freqs_cis.data_ptr(), layers_dev=layer_table.data_ptr())
    return desc, layer_table, keep


def pack_fp8_linear(lin):
    """The layout lr_ladder_decode_step_fp8 reads: the N bf16 scales of a weight-only e4m3 projection directly behind
    its N * K weight bytes.  Re-points the module's `weight` and `scales` buffers to views of one allocation (values
    unchanged) unless they already lie that way."""
    w, sc = lin.weight, lin.scales
    N, K = w.shape
    assert w.dtype == torch.float8_e4m3fn and sc.dtype == torch.bfloat16 and sc.numel() == N and (N * K) % 16 == 0
    if w.is_contiguous() and sc.is_contiguous() and sc.data_ptr() == w.data_ptr() + N * K and w.data_ptr() % 16 == 0:
        return
    buf = _aligned_bytes(N * K + 2 * N, w.device)
    buf[:N * K].view(torch.float8_e4m3fn).view(N, K).copy_(w)
    buf[N * K:].view(torch.bfloat16).copy_(sc)
    lin.weight = buf[:N * K].view(torch.float8_e4m3fn).view(N, K)
    lin.scales = buf[N * K:].view(torch.bfloat16)


def _aligned_bytes(n: int, dev):
    buf = torch.empty(n + 256, dtype=torch.uint8, device=dev)
    off = (-buf.data_ptr()) % 256
    return buf[off:off + n]


class FusedLadderStep:
    """Device-side state of lr_ladder_decode_step for one model and batch size: the layer pointer
    table, the model descriptor and the (initialised) workspace.  Keeps references to every tensor
    whose address it handed to the library."""

    def __init__(self, model, batch: int, attention_workgroups: int = 0):
        dev = model.output.weight.device
        self.fp8 = model.output.weight.dtype == torch.float8_e4m3fn
        self.desc, self.layer_table, self._keep = _ladder_model_desc(model, attention_workgroups)
        self.batch = batch
        lib = load()
        self.bytes = int(lib.lr_ladder_step_workspace_bytes(ctypes.byref(self.desc), batch))
        self.supported = self.bytes > 0
        if self.fp8:   # the additional conditions of lr_ladder_decode_step_fp8
            d = self.desc
            most = max((d.n_head + 2 * d.n_kv_head) * d.head_dim, 2 * d.ffn, d.out_rows) * d.dim
            self.supported = self.supported and d.dim % 16 == 0 and d.ffn % 16 == 0 and \
                (d.n_head * d.head_dim) % 16 == 0 and max(most, d.dim * d.ffn) < 0x7fffffff
        if self.supported:
            # one workgroup per compute unit, all resident at once: a device that cannot hold them leaves the model
            # to the per-op kernels (the launch itself would return LR_E_LAUNCH)
            with torch.cuda.device(dev):
                self.resident = int(lib.lr_ladder_step_resident_workgroups(ctypes.byref(self.desc), batch))
            self.supported = self.resident >= torch.cuda.get_device_properties(dev).multi_processor_count
        self.workspace = None
        if self.supported:
            self.workspace = _aligned_bytes(self.bytes, dev)
            self.reset()

    def reset(self):
        _check(load().lr_ladder_step_init(ctypes.byref(self.desc), self.batch, self.workspace.data_ptr(), self.bytes,
                                          _stream()), "lr_ladder_step_init")

    def fail_code(self) -> int:
        """Synchronises.  0, or the LR_DEV_* value an earlier step left in the workspace's failure word."""
        off = int(load().lr_ladder_step_fail_offset())
        return int(self.workspace[off:off + 4].view(torch.int32).item())

    def failed(self) -> bool:
        return self.fail_code() != 0

    def step(self, tokens, pos, logits, next_token=None, advance=False, cur_token=None, history=None, pos0=0):
        B = self.batch
        for t in (tokens, pos, next_token, cur_token, history):
            assert t is None or (t.dtype == torch.int32 and t.is_cuda)
        assert tokens.numel() == B and pos.numel() == 1 and logits.dtype == torch.bfloat16
        lrows, lcols, ldl = _rows_ld(logits)
        assert lrows == B and lcols == self.desc.out_rows
        p = lambda t: None if t is None else t.data_ptr()
        ld, n = (history.stride(0), history.shape[1]) if history is not None else (0, 0)
        entry = load().lr_ladder_decode_step_fp8 if self.fp8 else load().lr_ladder_decode_step
        _check(entry(ctypes.byref(self.desc), B, tokens.data_ptr(), pos.data_ptr(), logits.data_ptr(), ldl,
                     p(next_token), int(bool(advance)), p(cur_token), p(history), ld, n, int(pos0),
                     self.workspace.data_ptr(), self.bytes, _stream()),
               "lr_ladder_decode_step_fp8" if self.fp8 else "lr_ladder_decode_step")
