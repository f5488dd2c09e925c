"""ctypes binding of libmi355_serving.so (the C ABI declared in include/mi355_serving.h); the shared library is this
package's data file, so it is found the same way in the source tree and after `python setup.py install`.

This is the torch-free boundary: plain device pointers and sizes. Tensors are used here only as a convenient way
to own device memory and a stream; ``hgemm`` / ``fmha_fwd`` take anything with ``data_ptr()``.
There is no fallback: if the shared library has not been built, loading raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355_serving.so")

GEMM_NN, GEMM_NT, GEMM_TN = 0, 1, 2
LAYOUTS = {"NN": GEMM_NN, "NT": GEMM_NT, "TN": GEMM_TN}
ERR_BAD_ARGUMENT, ERR_UNSUPPORTED = 10001, 10002

EXPORTED_SYMBOLS = ("mi355_hgemm", "mi355_fmha_fwd", "mi355_fmha_fwd_strided", "mi355_fmha_fwd_bf16", "mi355_hgemm_silu_mul", "mi355_hgemm_add", "mi355_rmsnorm", "mi355_rope", "mi355_rope_qkv", "mi355_silu_mul",
                    "mi355_gemm_bf16", "mi355_gemm_silu_mul_bf16", "mi355_gemm_add_bf16", "mi355_rmsnorm_bf16", "mi355_rope_bf16", "mi355_rope_qkv_bf16", "mi355_silu_mul_bf16",
                    "mi355_fmha_fwd_workspace_bytes", "mi355_fmha_fwd_ws", "mi355_fmha_fwd_noalloc",
                    "mi355_last_error", "mi355_serving_version")
# exported for tests and tuning runs, declared in csrc/mi355_serving_internal.h and not in the public header
INTERNAL_SYMBOLS = ("mi355_internal_hgemm_variant", "mi355_internal_fmha_fwd_variant")

_lib = None


class Mi355Error(RuntimeError):
    def __init__(self, code, text):
        super().__init__("%s (code %d)" % (text, code))
        self.code = code


def load():
    """Load the shared library (once) and declare the argument types of its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            "%s is missing: build it with `python build.py` in %s (there is no CPU fallback)"
            % (LIB_PATH, os.path.dirname(_HERE)))
    import torch  # noqa: F401  loads the HIP runtime the library binds to
    lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    vp, i32, i64, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
    lib.mi355_hgemm.argtypes = [vp, vp, vp, i32, i32, i32, i64, i64, i64, i32, vp]
    lib.mi355_hgemm.restype = i32
    lib.mi355_fmha_fwd.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, i32, i32, vp]
    lib.mi355_fmha_fwd.restype = i32
    lib.mi355_fmha_fwd_strided.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, i32, i32,
                                           ctypes.POINTER(i64), vp]
    lib.mi355_fmha_fwd_strided.restype = i32
    lib.mi355_fmha_fwd_bf16.argtypes = lib.mi355_fmha_fwd_strided.argtypes
    lib.mi355_fmha_fwd_bf16.restype = i32
    lib.mi355_rmsnorm.argtypes = [vp, vp, vp, vp, vp, i64, i32, i64, i64, i64, i64, f32, vp]
    lib.mi355_rmsnorm.restype = i32
    lib.mi355_rope.argtypes = [vp, vp, i32, i32, i32, i32, i32, i64, i64, i64, i64, vp, vp, vp, i64, i32, vp]
    lib.mi355_rope.restype = i32
    lib.mi355_rope_qkv.argtypes = [vp, vp, i32, i32, i32, i32, i32, i64, i64, i64, i64, i64, vp, vp, vp, i64, i32, vp]
    lib.mi355_rope_qkv.restype = i32
    lib.mi355_silu_mul.argtypes = [vp, vp, i64, i32, i32, i64, i64, vp]
    lib.mi355_hgemm_silu_mul.argtypes = lib.mi355_hgemm.argtypes
    lib.mi355_hgemm_silu_mul.restype = i32
    lib.mi355_hgemm_add.argtypes = [vp, vp, vp, vp, i32, i32, i32, i64, i64, i64, i64, i32, vp]
    lib.mi355_hgemm_add.restype = i32
    lib.mi355_silu_mul.restype = i32
    for fp16_name, bf16_name in (("mi355_hgemm", "mi355_gemm_bf16"), ("mi355_hgemm_silu_mul", "mi355_gemm_silu_mul_bf16"),
                                 ("mi355_hgemm_add", "mi355_gemm_add_bf16"),
                                 ("mi355_rmsnorm", "mi355_rmsnorm_bf16"), ("mi355_rope", "mi355_rope_bf16"),
                                 ("mi355_rope_qkv", "mi355_rope_qkv_bf16"),
                                 ("mi355_silu_mul", "mi355_silu_mul_bf16")):
        getattr(lib, bf16_name).argtypes = getattr(lib, fp16_name).argtypes
        getattr(lib, bf16_name).restype = i32
    lib.mi355_last_error.argtypes = []
    lib.mi355_last_error.restype = ctypes.c_char_p
    lib.mi355_serving_version.argtypes = []
    lib.mi355_serving_version.restype = i32
    lib.mi355_fmha_fwd_workspace_bytes.argtypes = [i32] * 6
    lib.mi355_fmha_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.mi355_fmha_fwd_ws.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, i32, i32, ctypes.POINTER(i64), i32,
                                      vp, ctypes.c_size_t, vp]
    lib.mi355_fmha_fwd_ws.restype = i32
    lib.mi355_fmha_fwd_noalloc.argtypes = lib.mi355_fmha_fwd_strided.argtypes
    lib.mi355_fmha_fwd_noalloc.restype = i32
    lib.mi355_internal_hgemm_variant.argtypes = [vp, vp, vp, i32, i32, i32, i64, i64, i64, i32, i32, i32, vp]
    lib.mi355_internal_hgemm_variant.restype = i32
    lib.mi355_internal_fmha_fwd_variant.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, i32, i32,
                                                    ctypes.POINTER(i64), i32, i32, vp]
    lib.mi355_internal_fmha_fwd_variant.restype = i32
    _lib = lib
    return lib


DTYPE_FP16, DTYPE_BF16 = 0, 1


def _ptr(x):
    if x is None:
        return None
    return x.data_ptr() if hasattr(x, "data_ptr") else int(x)


def _check(rc):
    if rc != 0:
        raise Mi355Error(rc, load().mi355_last_error().decode())


def hgemm_raw(a_ptr, b_ptr, c_ptr, M, N, K, lda, ldb, ldc, layout, stream=0):
    """Direct call of mi355_hgemm with integer device addresses."""
    _check(load().mi355_hgemm(a_ptr, b_ptr, c_ptr, M, N, K, lda, ldb, ldc, layout, stream))


def fmha_fwd_raw(q_ptr, k_ptr, v_ptr, o_ptr, lse_ptr, B, Hq, Hkv, Sq, Sk, D, scale, causal, kv_valid_len, stream=0):
    """Direct call of mi355_fmha_fwd with integer device addresses."""
    _check(load().mi355_fmha_fwd(q_ptr, k_ptr, v_ptr, o_ptr, lse_ptr, B, Hq, Hkv, Sq, Sk, D, scale, causal,
                                 kv_valid_len, stream))


def hgemm(a, b, layout="NN", out=None, residual=None, variant=0):
    """C = op(a) op(b) (+ residual) through the C ABI on torch's current stream. a, b: contiguous fp16 or bf16 GPU
    tensors; `residual`: [M, N] rows with a contiguous last dimension, added in the GEMM's epilogue (mi355_hgemm_add);
    it may be `out` itself. `variant` != 0 pins a tile shape through the library's internal test hook (1 = 256x256,
    2 = 128x128, 3 = 64x128 or, for layout NT, 128x64, 4 = 64x64, 5 = 128x256, 6 = 256x128, 7 = 32x64 for layouts NN and NT) instead of the choice by shape."""
    import torch
    lay = LAYOUTS[layout] if isinstance(layout, str) else int(layout)
    assert a.dtype in (torch.float16, torch.bfloat16) and b.dtype == a.dtype and a.is_cuda and b.is_cuda
    assert a.is_contiguous() and b.is_contiguous()
    if lay == GEMM_TN:
        K, M = a.shape
    else:
        M, K = a.shape
    if lay == GEMM_NT:
        N, Kb = b.shape
    else:
        Kb, N = b.shape
    if K != Kb:
        raise ValueError("inner dimensions differ: %d vs %d" % (K, Kb))
    if out is None:
        out = torch.empty((M, N), dtype=a.dtype, device=a.device)
    stream = torch.cuda.current_stream(a.device).cuda_stream
    # leading dimensions of the contiguous operands (stride(0) of a size-1 dimension is arbitrary in torch)
    lda, ldb = a.shape[1], b.shape[1]
    if residual is not None:
        if tuple(residual.shape) != (M, N) or residual.dtype != a.dtype or residual.stride(1) != 1:
            raise ValueError("residual must be [%d, %d] %s with a contiguous last dimension" % (M, N, a.dtype))
        entry = load().mi355_gemm_add_bf16 if a.dtype == torch.bfloat16 else load().mi355_hgemm_add
        _check(entry(_ptr(a), _ptr(b), _ptr(residual), _ptr(out), M, N, K, lda, ldb, max(residual.stride(0), N),
                     max(out.stride(0), N), lay, stream))
        return out
    if variant:
        _check(load().mi355_internal_hgemm_variant(_ptr(a), _ptr(b), _ptr(out), M, N, K, lda, ldb, max(out.stride(0), N), lay,
                                                   DTYPE_BF16 if a.dtype == torch.bfloat16 else DTYPE_FP16, int(variant), stream))
        return out
    entry = load().mi355_gemm_bf16 if a.dtype == torch.bfloat16 else load().mi355_hgemm
    _check(entry(_ptr(a), _ptr(b), _ptr(out), M, N, K, lda, ldb, max(out.stride(0), N), lay, stream))
    return out


def fmha_fwd_strided_raw(q_ptr, k_ptr, v_ptr, o_ptr, lse_ptr, B, Hq, Hkv, Sq, Sk, D, scale, causal, kv_valid_len, strides,
                         stream=0):
    """Direct call of mi355_fmha_fwd_strided; `strides` = 12 element strides (q, k, v, o) x (batch, head, row)."""
    arr = (ctypes.c_int64 * 12)(*[int(x) for x in strides])
    _check(load().mi355_fmha_fwd_strided(q_ptr, k_ptr, v_ptr, o_ptr, lse_ptr, B, Hq, Hkv, Sq, Sk, D, scale, causal,
                                         kv_valid_len, arr, stream))


def _bhs_strides(t):
    return [t.stride(0), t.stride(1), t.stride(2)]


def fmha_workspace_bytes(B, Hq, Hkv, Sq, Sk, kv_valid_len=None):
    """Bytes of caller workspace mi355_fmha_fwd_ws uses for these sizes: the partial results of the split-KV path
    (generation steps; required) or of the key ranges of a chunk of queries against a long cache (optional: with less the
    call walks all keys in one kernel); 0 for every other shape."""
    return int(load().mi355_fmha_fwd_workspace_bytes(B, Hq, Hkv, Sq, Sk, Sk if kv_valid_len is None else kv_valid_len))


def fmha_fwd_noalloc(q, k, v, out, lse=None, causal=False, kv_valid_len=None, scale=None):
    """mi355_fmha_fwd_noalloc on torch's current stream: fp16 [B, H, S, D] tensors or views with a contiguous last
    dimension; `out` (and `lse`, if wanted) are the caller's. Neither this wrapper nor the library allocates."""
    import torch
    assert q.dtype == k.dtype == v.dtype == out.dtype == torch.float16, "mi355_fmha_fwd_noalloc is an fp16 entry point"
    assert q.is_cuda and q.dim() == 4 and k.dim() == 4 and v.shape == k.shape and out.shape == q.shape
    assert q.stride(3) == 1 and k.stride(3) == 1 and v.stride(3) == 1 and out.stride(3) == 1
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    assert lse is None or (lse.dtype == torch.float32 and tuple(lse.shape) == (B, Hq, Sq) and lse.is_contiguous())
    arr = (ctypes.c_int64 * 12)(*(_bhs_strides(q) + _bhs_strides(k) + _bhs_strides(v) + _bhs_strides(out)))
    _check(load().mi355_fmha_fwd_noalloc(_ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), B, Hq, Hkv, Sq, Sk, D,
                                         float(1.0 / (D ** 0.5) if scale is None else scale), int(bool(causal)),
                                         int(Sk if kv_valid_len is None else kv_valid_len), arr, _stream_of(q)))
    return out


def fmha_fwd(q, k, v, causal=False, kv_valid_len=None, scale=None, return_lse=True, out=None, variant=0, workspace=None):
    """Attention forward through the C ABI on torch's current stream. Returns (O, LSE) or O.

    q, k, v (and `out`, if given) are [B, H, S, D] fp16 GPU tensors or views with a contiguous last dimension, e.g.
    `x.view(B, S, H, D).transpose(1, 2)`; contiguous tensors take mi355_fmha_fwd, views mi355_fmha_fwd_strided.
    bfloat16 tensors take mi355_fmha_fwd_bf16. `workspace` (a uint8 GPU tensor): mi355_fmha_fwd_ws, which keeps the
    split-KV partial results there and never allocates. `variant` != 0 pins a kernel through the library's internal test
    hook (1 = 128-query workgroups, 2 = 256-query workgroups; both keep generation steps off the split-KV path; 3 = keys cut
    into ranges that a second kernel merges, an error where the choice by shape would not do that).
    """
    import torch
    assert q.dtype in (torch.float16, torch.bfloat16) and q.dtype == k.dtype == v.dtype and q.is_cuda
    B, Hq, Sq, D = q.shape
    _, Hkv, Sk, _ = k.shape
    if scale is None:
        scale = 1.0 / (D ** 0.5)
    if kv_valid_len is None:
        kv_valid_len = Sk
    o = torch.empty_like(q) if out is None else out
    lse = torch.empty((B, Hq, Sq), dtype=torch.float32, device=q.device) if return_lse else None
    stream = torch.cuda.current_stream(q.device).cuda_stream
    if variant or workspace is not None:
        assert all(t.stride(3) == 1 for t in (q, k, v, o)), "the last dimension must be contiguous"
        arr = (ctypes.c_int64 * 12)(*(_bhs_strides(q) + _bhs_strides(k) + _bhs_strides(v) + _bhs_strides(o)))
        dt = DTYPE_BF16 if q.dtype == torch.bfloat16 else DTYPE_FP16
        if variant:
            _check(load().mi355_internal_fmha_fwd_variant(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), B, Hq, Hkv, Sq, Sk, D,
                                                          float(scale), int(bool(causal)), int(kv_valid_len), arr, dt, int(variant),
                                                          stream))
        else:
            _check(load().mi355_fmha_fwd_ws(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), B, Hq, Hkv, Sq, Sk, D, float(scale),
                                            int(bool(causal)), int(kv_valid_len), arr, dt, _ptr(workspace),
                                            workspace.numel() * workspace.element_size(), stream))
    elif q.dtype == torch.bfloat16:
        assert all(t.stride(3) == 1 for t in (q, k, v, o)), "the last dimension must be contiguous"
        arr = (ctypes.c_int64 * 12)(*(_bhs_strides(q) + _bhs_strides(k) + _bhs_strides(v) + _bhs_strides(o)))
        _check(load().mi355_fmha_fwd_bf16(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), B, Hq, Hkv, Sq, Sk, D, float(scale),
                                          int(bool(causal)), int(kv_valid_len), arr, stream))
    elif all(t.is_contiguous() for t in (q, k, v, o)):
        fmha_fwd_raw(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), B, Hq, Hkv, Sq, Sk, D, float(scale), int(bool(causal)),
                     int(kv_valid_len), stream)
    else:
        assert all(t.stride(3) == 1 for t in (q, k, v, o)), "the last dimension must be contiguous"
        strides = _bhs_strides(q) + _bhs_strides(k) + _bhs_strides(v) + _bhs_strides(o)
        fmha_fwd_strided_raw(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), B, Hq, Hkv, Sq, Sk, D, float(scale),
                             int(bool(causal)), int(kv_valid_len), strides, stream)
    return (o, lse) if return_lse else o


def _stream_of(t):
    import torch
    return torch.cuda.current_stream(t.device).cuda_stream


def rmsnorm(x, weight, eps, residual=None, residual_out=None, out=None):
    """RMSNorm over the last dimension of a [rows, hidden] fp16 tensor (row stride free). With `residual`, normalises
    h = fp16(residual + x) and writes h to `residual_out` (default: a new tensor). Returns out or (out, h)."""
    import torch
    assert x.dim() == 2 and x.stride(1) == 1 and x.dtype in (torch.float16, torch.bfloat16) and weight.is_contiguous()
    assert weight.dtype == x.dtype
    rows, hidden = x.shape
    if out is None:
        out = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
    if residual is not None and residual_out is None:
        residual_out = torch.empty((rows, hidden), dtype=x.dtype, device=x.device)
    entry = load().mi355_rmsnorm_bf16 if x.dtype == torch.bfloat16 else load().mi355_rmsnorm
    _check(entry(_ptr(x), _ptr(residual), _ptr(residual_out), _ptr(weight), _ptr(out), rows, hidden,
                                x.stride(0), residual.stride(0) if residual is not None else 0,
                                residual_out.stride(0) if residual_out is not None else 0, out.stride(0), float(eps),
                                _stream_of(x)))
    return out if residual is None else (out, residual_out)


def rope(x, cos, sin, positions, out=None, copy_heads=0):
    """Rotary embedding of x [B, S, heads, 128] (any batch / token stride, heads contiguous), in place unless `out`
    (same shape, own strides) is given. The last `copy_heads` heads are copied unrotated. cos, sin: [n_positions, 64]
    fp32; positions: int32, [B, S] or [S] (shared by all batch rows)."""
    import torch
    B, S, heads, D = x.shape
    out = x if out is None else out
    assert x.dtype in (torch.float16, torch.bfloat16) and out.dtype == x.dtype
    assert x.stride(3) == 1 and x.stride(2) == D and out.stride(3) == 1 and out.stride(2) == D
    assert cos.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous() and cos.shape == sin.shape
    assert positions.dtype == torch.int32 and positions.is_contiguous() and positions.numel() in (S, B * S)
    pos_batch = S if (positions.numel() == B * S and B > 1) else 0
    entry = load().mi355_rope_bf16 if x.dtype == torch.bfloat16 else load().mi355_rope
    _check(entry(_ptr(x), _ptr(out), B, S, heads - copy_heads, copy_heads, D, x.stride(0), x.stride(1),
                             out.stride(0), out.stride(1), _ptr(cos), _ptr(sin), _ptr(positions), pos_batch, cos.shape[0],
                             _stream_of(x)))
    return out


def rope_qkv(qkv, kv_out, cos, sin, positions, q_heads, kv_heads):
    """One launch for a fused projection qkv [B, S, q_heads + 2 kv_heads, 128]: query heads rotated in place, rotated key heads
    and plain value heads written to kv_out [B, S, 2 kv_heads, 128] (own batch / token / head strides: the new rows of a KV
    cache, token-major or head-major)."""
    import torch
    B, S, heads, D = qkv.shape
    assert heads == q_heads + 2 * kv_heads and kv_out.shape == (B, S, 2 * kv_heads, D)
    assert qkv.dtype in (torch.float16, torch.bfloat16) and kv_out.dtype == qkv.dtype
    assert qkv.stride(3) == 1 and qkv.stride(2) == D and kv_out.stride(3) == 1
    assert cos.dtype == torch.float32 and cos.is_contiguous() and sin.is_contiguous() and cos.shape == sin.shape
    assert positions.dtype == torch.int32 and positions.is_contiguous() and positions.numel() in (S, B * S)
    pos_batch = S if (positions.numel() == B * S and B > 1) else 0
    entry = load().mi355_rope_qkv_bf16 if qkv.dtype == torch.bfloat16 else load().mi355_rope_qkv
    _check(entry(_ptr(qkv), _ptr(kv_out), B, S, q_heads, kv_heads, D, qkv.stride(0), qkv.stride(1), kv_out.stride(0),
                 kv_out.stride(1), kv_out.stride(2), _ptr(cos), _ptr(sin), _ptr(positions), pos_batch, cos.shape[0], _stream_of(qkv)))
    return kv_out


def silu_mul(gate_up, out=None, interleave=0):
    """silu(gate) * up for a [rows, 2F] fp16 tensor holding gate in its first F columns and up in the rest
    (interleave=0), or gate and up alternating in groups of `interleave` columns."""
    import torch
    assert gate_up.dim() == 2 and gate_up.stride(1) == 1 and gate_up.dtype in (torch.float16, torch.bfloat16)
    rows, two_f = gate_up.shape
    inter = two_f // 2
    if out is None:
        out = torch.empty((rows, inter), dtype=gate_up.dtype, device=gate_up.device)
    entry = load().mi355_silu_mul_bf16 if gate_up.dtype == torch.bfloat16 else load().mi355_silu_mul
    _check(entry(_ptr(gate_up), _ptr(out), rows, inter, int(interleave), gate_up.stride(0), out.stride(0),
                                 _stream_of(gate_up)))
    return out


GATE_UP_BLOCK = 32  # columns per gate / up group in the operand of mi355_hgemm_silu_mul


def interleave_gate_up(gate, up, dim=0):
    """Weight of mi355_hgemm_silu_mul from the two projection weights: groups of 32 gate outputs alternate with the
    32 up outputs of the same positions along `dim` (0 for nn.Linear-layout [out, in] weights, 1 for [in, out])."""
    import torch
    F = gate.shape[dim]
    assert gate.shape == up.shape and F % GATE_UP_BLOCK == 0
    if dim == 0:
        g = gate.reshape(F // GATE_UP_BLOCK, GATE_UP_BLOCK, -1)
        u = up.reshape(F // GATE_UP_BLOCK, GATE_UP_BLOCK, -1)
        return torch.stack((g, u), 1).reshape(2 * F, -1).contiguous()
    g = gate.reshape(-1, F // GATE_UP_BLOCK, GATE_UP_BLOCK)
    u = up.reshape(-1, F // GATE_UP_BLOCK, GATE_UP_BLOCK)
    return torch.stack((g, u), 2).reshape(-1, 2 * F).contiguous()


def hgemm_silu_mul(a, w, layout="NT", out=None):
    """silu(a @ gate) * (a @ up) for a weight built by interleave_gate_up: one launch where the tiled GEMM covers the
    shape (mi355_hgemm_silu_mul), otherwise the product followed by silu_mul on the interleaved columns."""
    import torch
    lay = LAYOUTS[layout] if isinstance(layout, str) else int(layout)
    assert lay in (GEMM_NN, GEMM_NT) and a.is_contiguous() and w.is_contiguous()
    assert a.dtype in (torch.float16, torch.bfloat16) and w.dtype == a.dtype
    M, K = a.shape
    N2 = w.shape[0] if lay == GEMM_NT else w.shape[1]
    N = N2 // 2
    if out is None:
        out = torch.empty((M, N), dtype=a.dtype, device=a.device)
    entry = load().mi355_gemm_silu_mul_bf16 if a.dtype == torch.bfloat16 else load().mi355_hgemm_silu_mul
    # leading dimensions of the logical layout: a contiguous tensor with a single row may carry any stride(0)
    rc = entry(_ptr(a), _ptr(w), _ptr(out), M, N, K, a.shape[1], w.shape[1], max(out.stride(0), N), lay, _stream_of(a))
    if rc == ERR_UNSUPPORTED:
        return silu_mul(hgemm(a, w, layout), out=out, interleave=GATE_UP_BLOCK)
    _check(rc)
    return out
