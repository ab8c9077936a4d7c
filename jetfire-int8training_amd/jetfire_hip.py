"""Host-side binding of libjetfire_hip.so (ctypes over the C ABI of include/jetfire_hip.h) for torch
tensors.  PyTorch is used for device memory and the current stream only; every computation below is a
hand-written gfx950 kernel.  There is no fallback: a missing library or a CPU tensor raises.

Each wrapper allocates its outputs (like the reference's launchers do with torch.empty, e.g.
JetfireGEMMKernel/BlockQuantize/cpp_extension/igemm/igemm_BlockSquare32OutputIntQuantizeBiasRowCol.cu:404-408,
Jetfire/Nonlinear/quantize.py:140-141) and takes/returns 2-D tensors; 3-D handling lives in the
Linear / Nonlinear packages.
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libjetfire_hip.so")
QB = 32

B_NK, B_KN = 0, 1
A_MK, A_KM = 0, 1
SCALE_F16, SCALE_F32 = 0, 1
SCALES_KMAJOR, SCALES_ROWMAJOR = 0, 1
FP_F16, FP_F32, FP_BF16 = 0, 1, 2
ROUND_NEAREST, ROUND_STOCHASTIC, ROUND_TRUNC, ROUND_STOCHASTIC_TRUNC = 0, 1, 2, 3
GELU_ERF, GELU_TANH = 0, 1

EXPORTS = [
    "jf_error_string", "jf_igemm_workspace_bytes", "jf_igemm_s32", "jf_igemm_block_acc", "jf_igemm_block_fp",
    "jf_igemm_splitk_plan", "jf_igemm_block_fp_workspace_bytes", "jf_igemm_block_q_gelu", "jf_igemm_block_fp_noalloc", "jf_igemm_block_q_gelu_bwd",
    "jf_igemm_block_q", "jf_quantize", "jf_dequantize", "jf_transpose_s8", "jf_rowstats", "jf_layernorm_fwd",
    "jf_layernorm_bwd_workspace_bytes", "jf_layernorm_bwd", "jf_layernorm_bwd_add", "jf_gelu_fwd", "jf_gelu_bwd", "jf_add", "jf_rowstats_finish",
    "jf_igemm_block_q_dequant", "jf_quantize_slabs", "jf_philox_rounds", "jf_block_colsum", "jf_block_colsum_workspace_bytes",
]

_lib = None
_p, _i, _u64, _f, _sz = C.c_void_p, C.c_int, C.c_uint64, C.c_float, C.c_size_t


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python {os.path.join(_HERE, 'build_ext.py')} hip`")
        L = C.CDLL(LIB_PATH)
        L.jf_error_string.argtypes = [_i]
        L.jf_error_string.restype = C.c_char_p
        L.jf_igemm_workspace_bytes.argtypes = [_i, _i, _i, _i]
        L.jf_igemm_workspace_bytes.restype = _sz
        L.jf_igemm_s32.argtypes = [_p, _p, _p, _i, _i, _i, _i, _p, _sz, _p]
        L.jf_igemm_block_acc.argtypes = [_p, _p, _p, _i, _i, _i, _i, _p, _sz, _p]
        L.jf_igemm_block_fp.argtypes = [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p, _sz, _p]
        L.jf_igemm_block_fp_noalloc.argtypes = [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _i, _p]
        L.jf_igemm_block_q_gelu_bwd.argtypes = [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _u64, _u64, _i, _u64, _u64, _p]
        L.jf_igemm_block_q_dequant.argtypes = [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _i, _u64, _u64, _p]
        L.jf_igemm_block_q_gelu.argtypes = [_p, _p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _f, _p]
        L.jf_igemm_splitk_plan.argtypes = [_i, _i, _i, _i, C.POINTER(C.c_int), C.POINTER(C.c_int)]
        L.jf_igemm_block_fp_workspace_bytes.argtypes = [_i, _i, _i, _i, _i]
        L.jf_igemm_block_fp_workspace_bytes.restype = _sz
        L.jf_rowstats_finish.argtypes = [_p, _p, _i, _i, _i, _p, _p, _p]
        L.jf_igemm_block_q.argtypes = [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _i, _u64, _u64, _p, _sz, _p]
        L.jf_quantize.argtypes = [_p, _i, _i, _i, _p, _p, _p, _i, _i, _u64, _u64, _f, _p]
        L.jf_quantize_slabs.argtypes = [_p, _p, _p, _i, _i, _i, _p, _p, _i, _i, _u64, _u64, _f, _p]
        L.jf_dequantize.argtypes = [_p, _p, _i, _i, _i, _p, _i, _p]
        L.jf_transpose_s8.argtypes = [_p, _i, _i, _p, _p]
        L.jf_rowstats.argtypes = [_p, _p, _i, _i, _i, _f, _p, _p, _p]
        L.jf_layernorm_fwd.argtypes = [_p, _p, _p, _p, _p, _p, _i, _i, _i, _p, _p, _p]
        L.jf_layernorm_bwd_workspace_bytes.argtypes = [_i, _i]
        L.jf_layernorm_bwd_workspace_bytes.restype = _sz
        L.jf_layernorm_bwd.argtypes = [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _u64, _u64, _p, _p, _p, _p, _p, _sz, _p]
        L.jf_gelu_fwd.argtypes = [_p, _p, _i, _i, _i, _i, _f, _p, _p, _p]
        L.jf_gelu_bwd.argtypes = [_p, _p, _p, _p, _i, _i, _i, _i, _i, _u64, _u64, _p, _p, _p]
        L.jf_layernorm_bwd_add.argtypes = [_p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _u64, _u64, _p, _i, _i, _u64, _u64,
                                           _p, _i, _p, _p, _p, _p, _p, _sz, _p]
        L.jf_add.argtypes = [_p, _i, _p, _p, _i, _i, _i, _i, _u64, _u64, _p, _i, _p, _p, _p, _p, _p]
        L.jf_block_colsum_workspace_bytes.argtypes = [_i, _i]
        L.jf_block_colsum_workspace_bytes.restype = _sz
        L.jf_block_colsum.argtypes = [_p, _p, _i, _i, _i, _p, _p, _sz, _p]
        missing = [name for name in EXPORTS if not hasattr(L, name)]
        if missing:
            raise RuntimeError(f"{LIB_PATH} does not export {missing}")
        _lib = L
    return _lib


PROF_LIB_PATH = os.path.join(_HERE, "libjetfire_prof.so")
PROF_EXPORTS = ["jf_prof_igemm_block_q", "jf_calibrate", "jf_wall_clock_khz"]
_prof = None


def prof_lib():
    """The measurement library (include/jetfire_prof.h); only the benchmark and its tests load it."""
    global _prof
    if _prof is None:
        if not os.path.exists(PROF_LIB_PATH):
            raise RuntimeError(f"{PROF_LIB_PATH} is missing: build it with `python {os.path.join(_HERE, 'build_ext.py')} hip`")
        L = C.CDLL(PROF_LIB_PATH)
        L.jf_prof_igemm_block_q.argtypes = [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _i, _u64, _u64, _p, _i, _p]
        L.jf_calibrate.argtypes = [_i, _i, _i, _i, _i, _i, _p, _p, _p]
        L.jf_wall_clock_khz.argtypes = []
        _prof = L
    return _prof


def check(rc):
    if rc != 0:
        raise RuntimeError(lib().jf_error_string(rc).decode())


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need(t, dtype, name, ndim=2):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError(f"{name}: expected a GPU tensor")
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError(f"{name}: expected dtype {dtype}, got {t.dtype}")
    if ndim is not None and t.dim() != ndim:
        raise RuntimeError(f"{name}: expected {ndim} dimensions, got {t.dim()}")
    if not t.is_contiguous():
        raise RuntimeError(f"{name}: expected a contiguous tensor")
    return t


def _scale_code(s, name):
    if s.dtype == torch.float16:
        return SCALE_F16
    if s.dtype == torch.float32:
        return SCALE_F32
    raise RuntimeError(f"{name}: scales must be float16 or float32, got {s.dtype}")


_SCALE_TORCH = {SCALE_F16: torch.float16, SCALE_F32: torch.float32}
_FP_CODE = {torch.float16: FP_F16, torch.float32: FP_F32, torch.bfloat16: FP_BF16}


def _mult32(*dims):
    for d in dims:
        if d <= 0 or d % QB:
            raise RuntimeError(f"dimension {d} is not a positive multiple of {QB}")


# ------------------------------------------------------------------------------------------------ RNG
class _Philox:
    """(seed, offset) for the stochastic-rounding kernels: reserved from the device's default torch generator (the one
    source of Philox counters for every stochastic op of this library, the GEMM extension included), one counter per 8
    output elements.  Consecutive ops therefore draw disjoint counter ranges and torch.manual_seed (also with an
    unchanged seed) rewinds them.  The generator refuses this during stream capture: captured code passes explicit
    seed / offset arguments."""

    @staticmethod
    def _gen(device):
        idx = device.index if device.index is not None else torch.cuda.current_device()
        return torch.cuda.default_generators[idx]

    def peek(self, device):
        g = self._gen(device)
        return g.initial_seed() & 0xFFFFFFFFFFFFFFFF, g.get_offset()

    def next(self, numel, device):
        g = self._gen(device)
        seed, off = g.initial_seed() & 0xFFFFFFFFFFFFFFFF, g.get_offset()
        g.set_offset(off + ((numel + 7) // 8 + 3) // 4 * 4)
        return seed, off


philox = _Philox()


def _rng(rounding, numel, seed, offset, device):
    if rounding in (ROUND_STOCHASTIC, ROUND_STOCHASTIC_TRUNC) and seed is None:
        return philox.next(numel, device)
    return (seed or 0), (offset or 0)


# ------------------------------------------------------------------------------------------------ GEMMs
def _gemm_operands(A, B, b_layout, a_layout=0):
    _need(A, torch.int8, "A")
    _need(B, torch.int8, "B")
    if a_layout == A_MK:
        M, K = A.shape
    elif a_layout == A_KM:
        K, M = A.shape
    else:
        raise RuntimeError("a_layout must be A_MK or A_KM")
    if b_layout == B_NK:
        N, K2 = B.shape
    elif b_layout == B_KN:
        K2, N = B.shape
    else:
        raise RuntimeError("b_layout must be B_NK or B_KN")
    if K2 != K:
        raise RuntimeError(f"inner dimensions differ: A is {tuple(A.shape)}, B is {tuple(B.shape)}")
    if B.device != A.device:
        raise RuntimeError("A and B are on different devices")
    _mult32(M, N, K)
    nbytes = lib().jf_igemm_workspace_bytes(M, N, K, b_layout)
    ws = torch.empty(nbytes, dtype=torch.int8, device=A.device) if nbytes else None
    return M, N, K, ws, nbytes


def _scale_layout(s, K, rows, name):
    """[K/32, rows/32] contiguous (K-major) or the .t() view of a contiguous [rows/32, K/32] tensor (row-major)."""
    if not isinstance(s, torch.Tensor) or not s.is_cuda or s.dim() != 2:
        raise RuntimeError(f"{name}: expected a 2-D GPU tensor")
    if tuple(s.shape) != (K // QB, rows // QB):
        raise RuntimeError(f"{name}: scale shape must be [K/32,rows/32]={K // QB, rows // QB}, got {tuple(s.shape)}")
    if s.is_contiguous():
        return SCALES_KMAJOR
    if s.stride() == (1, K // QB):
        return SCALES_ROWMAJOR
    raise RuntimeError(f"{name}: expected a contiguous tensor or the .t() view of one, got strides {s.stride()}")


def _gemm_scales(sa, sb, M, N, K):
    code = _scale_code(sa, "sa")
    if sb.dtype != sa.dtype:
        raise RuntimeError(f"sb: expected dtype {sa.dtype}, got {sb.dtype}")
    return code, _scale_layout(sa, K, M, "sa"), _scale_layout(sb, K, N, "sb")


def igemm_s32(A, B, b_layout=B_KN):
    M, N, K, ws, nb = _gemm_operands(A, B, b_layout)
    out = torch.empty((M, N), dtype=torch.int32, device=A.device)
    check(lib().jf_igemm_s32(_ptr(A), _ptr(B), _ptr(out), M, N, K, b_layout, _ptr(ws), nb, _stream()))
    return out


def igemm_block_acc(A, B, b_layout=B_KN):
    M, N, K, ws, nb = _gemm_operands(A, B, b_layout)
    out = torch.empty((K // QB, M, N), dtype=torch.int32, device=A.device)
    check(lib().jf_igemm_block_acc(_ptr(A), _ptr(B), _ptr(out), M, N, K, b_layout, _ptr(ws), nb, _stream()))
    return out


def splitk_plan(M, N, K, splitk):
    """(parts, K blocks per part) the library uses for this problem and splitk request."""
    parts, per = C.c_int(0), C.c_int(0)
    check(lib().jf_igemm_splitk_plan(M, N, K, splitk, C.byref(parts), C.byref(per)))
    return parts.value, per.value


def igemm_block_fp(A, B, sa, sb, b_layout=B_KN, out_dtype=torch.float16, a_layout=A_MK, splitk=1):
    """a_layout=A_KM: A is given as [K, M] (the un-transposed gradient of a weight-gradient GEMM).
    splitk: 1 = one accumulation chain over K (reference arithmetic); n > 1 = up to n ordered partial chains;
    0 = chosen by the library from the tile count."""
    M, N, K, ws, nb = _gemm_operands(A, B, b_layout, a_layout)
    nb = lib().jf_igemm_block_fp_workspace_bytes(M, N, K, b_layout, splitk)
    ws = torch.empty(nb, dtype=torch.int8, device=A.device) if nb else None
    code, la, lb = _gemm_scales(sa, sb, M, N, K)
    out = torch.empty((M, N), dtype=out_dtype, device=A.device)
    check(lib().jf_igemm_block_fp(_ptr(A), _ptr(B), _ptr(sa), _ptr(sb), _ptr(out), M, N, K, a_layout, b_layout, code, la,
                                  lb, _FP_CODE[out_dtype], splitk, _ptr(ws), nb, _stream()))
    return out


NOALLOC_SCRATCH_BYTES = 64 << 20


def igemm_block_fp_noalloc(A, B, sa, sb, out, b_layout=B_KN, a_layout=A_MK, splitk=1):
    """igemm_block_fp into a caller-supplied `out` ([M,N] float16 / float32 / bfloat16) through the entry point that
    neither takes nor allocates scratch (the K split uses the library's built-in buffer); this wrapper allocates
    nothing either.  Refuses K splits that need more than NOALLOC_SCRATCH_BYTES."""
    M, N, K, _, _ = _gemm_operands(A, B, b_layout, a_layout)
    code, la, lb = _gemm_scales(sa, sb, M, N, K)
    _need(out, None, "out")
    if tuple(out.shape) != (M, N) or out.dtype not in _FP_CODE or out.device != A.device:
        raise RuntimeError(f"out: expected a float [M,N]={M, N} tensor on {A.device}")
    check(lib().jf_igemm_block_fp_noalloc(_ptr(A), _ptr(B), _ptr(sa), _ptr(sb), _ptr(out), M, N, K, a_layout, b_layout,
                                          code, la, lb, _FP_CODE[out.dtype], splitk, _stream()))
    return out


def igemm_block_q_gelu(A, B, sa, sb, approx=GELU_ERF, amax_eps=5e-5, bias=None, biasmax=None):
    """Forward GEMM (B as [N,K], round to nearest) with the GELU forward fused into its epilogue.
    Returns (q, s, q_gelu, s_gelu): what igemm_block_q and then gelu_fwd would return."""
    M, N, K, _, _ = _gemm_operands(A, B, B_NK)
    code, la, lb = _gemm_scales(sa, sb, M, N, K)
    if bias is not None:
        _need(bias, torch.float32, "bias", 1)
        if bias.numel() != N:
            raise RuntimeError("bias must have N elements")
    if biasmax is not None:
        _need(biasmax, torch.float32, "biasmax", None)
    q = torch.empty((M, N), dtype=torch.int8, device=A.device)
    s = torch.empty((M // QB, N // QB), dtype=sa.dtype, device=A.device)
    qg, sg = torch.empty_like(q), torch.empty_like(s)
    check(lib().jf_igemm_block_q_gelu(_ptr(A), _ptr(B), _ptr(sa), _ptr(sb), _ptr(bias), _ptr(biasmax), _ptr(q), _ptr(s),
                                      _ptr(qg), _ptr(sg), M, N, K, code, la, lb, approx, amax_eps, _stream()))
    return q, s, qg, sg


def igemm_block_q_gelu_bwd(A, B, sa, sb, xq, xs, approx=GELU_ERF, gelu_rounding=ROUND_STOCHASTIC, seed=None, offset=None,
                           gelu_seed=None, gelu_offset=None):
    """Activation-gradient GEMM (B as [K,N], stochastic rounding) with the GELU backward fused into its epilogue:
    returns what gelu_bwd(xq, xs, *igemm_block_q(A, B, sa, sb, B_KN, rounding=ROUND_STOCHASTIC), approx, gelu_rounding)
    returns (the two draw their noise in that order)."""
    M, N, K, _, _ = _gemm_operands(A, B, B_KN)
    code, la, lb = _gemm_scales(sa, sb, M, N, K)
    R2, C2, code2 = _block_tensor(xq, xs, "x")
    if (R2, C2, code2) != (M, N, code):
        raise RuntimeError(f"x must be an [M,N]={M, N} block tensor with the scale dtype of sa / sb")
    if gelu_rounding not in (ROUND_NEAREST, ROUND_STOCHASTIC):
        raise RuntimeError("gelu_rounding must be ROUND_NEAREST or ROUND_STOCHASTIC")
    seed, offset = _rng(ROUND_STOCHASTIC, M * N, seed, offset, A.device)
    gelu_seed, gelu_offset = _rng(gelu_rounding, M * N, gelu_seed, gelu_offset, A.device)
    out = torch.empty((M, N), dtype=torch.int8, device=A.device)
    sc = torch.empty((M // QB, N // QB), dtype=sa.dtype, device=A.device)
    check(lib().jf_igemm_block_q_gelu_bwd(_ptr(A), _ptr(B), _ptr(sa), _ptr(sb), _ptr(xq), _ptr(xs), _ptr(out), _ptr(sc), M, N, K,
                                          code, la, lb, approx, seed, offset, gelu_rounding, gelu_seed, gelu_offset, _stream()))
    return out, sc


def igemm_block_q(A, B, sa, sb, b_layout=B_KN, bias=None, biasmax=None, rounding=ROUND_NEAREST, seed=None, offset=None):
    M, N, K, ws, nb = _gemm_operands(A, B, b_layout)
    code, la, lb = _gemm_scales(sa, sb, M, N, K)
    if bias is not None:
        _need(bias, torch.float32, "bias", 1)
        if bias.numel() != N:
            raise RuntimeError("bias must have N elements")
    if biasmax is not None:
        _need(biasmax, torch.float32, "biasmax", None)
    if rounding not in (ROUND_NEAREST, ROUND_STOCHASTIC):
        raise RuntimeError("rounding must be ROUND_NEAREST or ROUND_STOCHASTIC")
    seed, offset = _rng(rounding, M * N, seed, offset, A.device)
    out = torch.empty((M, N), dtype=torch.int8, device=A.device)
    sc = torch.empty((M // QB, N // QB), dtype=sa.dtype, device=A.device)
    check(lib().jf_igemm_block_q(_ptr(A), _ptr(B), _ptr(sa), _ptr(sb), _ptr(bias), _ptr(biasmax), _ptr(out), _ptr(sc),
                                 M, N, K, b_layout, code, la, lb, rounding, seed, offset, _ptr(ws), nb, _stream()))
    return out, sc


def igemm_block_q_dequant(A, B, sa, sb, b_layout=B_KN, out_dtype=None, bias=None, biasmax=None, rounding=ROUND_NEAREST,
                          seed=None, offset=None):
    """dequantize(*igemm_block_q(...), out_dtype) in one kernel: the requantised block tensor is formed in the GEMM's
    epilogue and leaves it as codes x scales (out_dtype: float16 / bfloat16 / float32, default the scales' dtype); same
    bits as the two calls, same noise counters."""
    M, N, K, _, _ = _gemm_operands(A, B, b_layout)
    code, la, lb = _gemm_scales(sa, sb, M, N, K)
    out_dtype = sa.dtype if out_dtype is None else out_dtype
    if out_dtype not in _FP_CODE:
        raise RuntimeError(f"out_dtype: unsupported {out_dtype}")
    if bias is not None:
        _need(bias, torch.float32, "bias", 1)
        if bias.numel() != N:
            raise RuntimeError("bias must have N elements")
    if biasmax is not None:
        _need(biasmax, torch.float32, "biasmax", None)
    if rounding not in (ROUND_NEAREST, ROUND_STOCHASTIC):
        raise RuntimeError("rounding must be ROUND_NEAREST or ROUND_STOCHASTIC")
    seed, offset = _rng(rounding, M * N, seed, offset, A.device)
    out = torch.empty((M, N), dtype=out_dtype, device=A.device)
    check(lib().jf_igemm_block_q_dequant(_ptr(A), _ptr(B), _ptr(sa), _ptr(sb), _ptr(bias), _ptr(biasmax), _ptr(out), M, N, K,
                                         b_layout, code, la, lb, _FP_CODE[out_dtype], rounding, seed, offset, _stream()))
    return out


# ------------------------------------------------------------------------------------------------ block ops
def quantize(x, rounding=ROUND_NEAREST, scale_dtype=torch.float16, transpose=False, amax_eps=0.0, seed=None, offset=None):
    _need(x, None, "x")
    if x.dtype not in _FP_CODE:
        raise RuntimeError(f"x: unsupported dtype {x.dtype}")
    R, Cc = x.shape
    _mult32(R, Cc)
    seed, offset = _rng(rounding, R * Cc, seed, offset, x.device)
    q = torch.empty((R, Cc), dtype=torch.int8, device=x.device)
    s = torch.empty((R // QB, Cc // QB), dtype=scale_dtype, device=x.device)
    qT = torch.empty((Cc, R), dtype=torch.int8, device=x.device) if transpose else None
    check(lib().jf_quantize(_ptr(x), _FP_CODE[x.dtype], R, Cc, _ptr(q), _ptr(s), _ptr(qT), _scale_code(s, "s"),
                            rounding, seed, offset, amax_eps, _stream()))
    return (q, s, qT) if transpose else (q, s)


def _block_tensor(q, s, name):
    _need(q, torch.int8, name)
    _need(s, None, name + " scale")
    R, Cc = q.shape
    _mult32(R, Cc)
    if tuple(s.shape) != (R // QB, Cc // QB):
        raise RuntimeError(f"{name}: scale shape {tuple(s.shape)} does not match codes {tuple(q.shape)}")
    if s.device != q.device:
        raise RuntimeError(f"{name}: codes and scales are on different devices")
    return R, Cc, _scale_code(s, name)


def quantize_slabs(slabs, rounding=ROUND_NEAREST, scale_dtype=torch.float16, amax_eps=0.0, seed=None, offset=None):
    """quantize(torch.cat(slabs, dim=1)) without making the concatenation: every slab ([R, C_i], unit column stride, any
    row stride) is quantised into its columns of one block tensor; same codes, scales and noise counters."""
    R = slabs[0].shape[0]
    widths = []
    for x in slabs:
        if not isinstance(x, torch.Tensor) or not x.is_cuda or x.dim() != 2 or x.shape[0] != R or x.stride(1) != 1:
            raise RuntimeError("slabs: expected 2-D GPU tensors with the same number of rows and unit column stride")
        if x.dtype not in _FP_CODE or x.dtype != slabs[0].dtype:
            raise RuntimeError("slabs: one floating dtype for all of them")
        widths.append(x.shape[1])
    Ct = sum(widths)
    _mult32(R, Ct, *widths)
    seed, offset = _rng(rounding, R * Ct, seed, offset, slabs[0].device)
    if len(slabs) > 4:
        raise RuntimeError("at most 4 slabs")
    q = torch.empty((R, Ct), dtype=torch.int8, device=slabs[0].device)
    s = torch.empty((R // QB, Ct // QB), dtype=scale_dtype, device=slabs[0].device)
    n = len(slabs)
    xs = (C.c_void_p * n)(*[x.data_ptr() for x in slabs])
    ld = (C.c_int * n)(*[x.stride(0) for x in slabs])
    wd = (C.c_int * n)(*widths)
    check(lib().jf_quantize_slabs(xs, ld, wd, n, _FP_CODE[slabs[0].dtype], R, _ptr(q), _ptr(s), _scale_code(s, "s"),
                                  rounding, seed, offset, amax_eps, _stream()))
    return q, s


def dequantize(q, s, out_dtype=torch.float32):
    """codes x scales as float32 (default), float16 or bfloat16 (the fp32 product rounded once)."""
    R, Cc, code = _block_tensor(q, s, "x")
    if out_dtype not in _FP_CODE:
        raise RuntimeError("dequantize: out_dtype must be float32, float16 or bfloat16")
    out = torch.empty((R, Cc), dtype=out_dtype, device=q.device)
    check(lib().jf_dequantize(_ptr(q), _ptr(s), R, Cc, code, _ptr(out), _FP_CODE[out_dtype], _stream()))
    return out


def transpose_s8(q):
    _need(q, torch.int8, "x")
    R, Cc = q.shape
    if R % 16 or Cc % 16:
        raise RuntimeError("transpose: dimensions must be multiples of 16")
    out = torch.empty((Cc, R), dtype=torch.int8, device=q.device)
    check(lib().jf_transpose_s8(_ptr(q), R, Cc, _ptr(out), _stream()))
    return out


def rowstats(q, s, eps=1e-5):
    R, Cc, code = _block_tensor(q, s, "x")
    mean = torch.empty(R, dtype=torch.float32, device=q.device)
    rstd = torch.empty(R, dtype=torch.float32, device=q.device)
    check(lib().jf_rowstats(_ptr(q), _ptr(s), R, Cc, code, eps, _ptr(mean), _ptr(rstd), _stream()))
    return mean, rstd


def _vec(t, n, name):
    _need(t, torch.float32, name, 1)
    if t.numel() != n:
        raise RuntimeError(f"{name}: expected {n} elements, got {t.numel()}")
    return t


def layernorm_fwd(q, s, gamma, beta, mean, rstd):
    R, Cc, code = _block_tensor(q, s, "x")
    _vec(gamma, Cc, "gamma")
    if beta is not None:
        _vec(beta, Cc, "beta")
    _vec(mean, R, "mean")
    _vec(rstd, R, "rstd")
    qy = torch.empty_like(q)
    sy = torch.empty_like(s)
    check(lib().jf_layernorm_fwd(_ptr(q), _ptr(s), _ptr(gamma), _ptr(beta), _ptr(mean), _ptr(rstd), R, Cc, code,
                                 _ptr(qy), _ptr(sy), _stream()))
    return qy, sy


def layernorm_bwd(qx, sx, qg, sg, gamma, mean, rstd, rounding=ROUND_NEAREST, want_dbeta=True, seed=None, offset=None):
    R, Cc, code = _block_tensor(qx, sx, "x")
    R2, C2, code2 = _block_tensor(qg, sg, "g")
    if (R2, C2, code2) != (R, Cc, code):
        raise RuntimeError("x and g must have the same shape and scale dtype")
    _vec(gamma, Cc, "gamma")
    _vec(mean, R, "mean")
    _vec(rstd, R, "rstd")
    seed, offset = _rng(rounding, R * Cc, seed, offset, qx.device)
    nbytes = lib().jf_layernorm_bwd_workspace_bytes(R, Cc)
    ws = torch.empty(nbytes, dtype=torch.int8, device=qx.device)
    qdx = torch.empty_like(qx)
    sdx = torch.empty_like(sx)
    dgamma = torch.empty(Cc, dtype=torch.float32, device=qx.device)
    dbeta = torch.empty(Cc, dtype=torch.float32, device=qx.device) if want_dbeta else None
    check(lib().jf_layernorm_bwd(_ptr(qx), _ptr(sx), _ptr(qg), _ptr(sg), _ptr(gamma), _ptr(mean), _ptr(rstd), R, Cc, code,
                                 rounding, seed, offset, _ptr(qdx), _ptr(sdx), _ptr(dgamma), _ptr(dbeta), _ptr(ws), nbytes,
                                 _stream()))
    return qdx, sdx, dgamma, dbeta


def layernorm_bwd_add(qx, sx, qg, sg, gamma, mean, rstd, x1, rounding=ROUND_NEAREST, add_rounding=ROUND_TRUNC,
                      want_dbeta=True, out_dtype=torch.float32, seed=None, offset=None, add_seed=None, add_offset=None):
    """layernorm_bwd followed by add(x1, dx codes, dx scales): (y1, q, s, dgamma, dbeta), the bits the two calls give
    (noise offsets are drawn in their order).  Rows of up to 2048 columns run as one kernel that never stores dx; wider
    rows make the two calls."""
    R, Cc, code = _block_tensor(qx, sx, "x")
    R2, C2, code2 = _block_tensor(qg, sg, "g")
    if (R2, C2, code2) != (R, Cc, code):
        raise RuntimeError("x and g must have the same shape and scale dtype")
    _vec(gamma, Cc, "gamma")
    _vec(mean, R, "mean")
    _vec(rstd, R, "rstd")
    _need(x1, None, "x1")
    if x1.dtype not in _FP_CODE or tuple(x1.shape) != (R, Cc):
        raise RuntimeError("x1 must be a float tensor of the same shape as x")
    if out_dtype not in _FP_CODE:
        raise RuntimeError("out_dtype must be float32, float16 or bfloat16")
    seed, offset = _rng(rounding, R * Cc, seed, offset, qx.device)
    add_seed, add_offset = _rng(add_rounding, R * Cc, add_seed, add_offset, qx.device)
    if Cc // QB > 64:
        qdx, sdx, dgamma, dbeta = layernorm_bwd(qx, sx, qg, sg, gamma, mean, rstd, rounding, want_dbeta, seed, offset)
        return add(x1, qdx, sdx, add_rounding, seed=add_seed, offset=add_offset, out_dtype=out_dtype) + (dgamma, dbeta)
    nbytes = lib().jf_layernorm_bwd_workspace_bytes(R, Cc)
    ws = torch.empty(nbytes, dtype=torch.int8, device=qx.device)
    y1 = torch.empty((R, Cc), dtype=out_dtype, device=qx.device)
    q = torch.empty_like(qx)
    s = torch.empty_like(sx)
    dgamma = torch.empty(Cc, dtype=torch.float32, device=qx.device)
    dbeta = torch.empty(Cc, dtype=torch.float32, device=qx.device) if want_dbeta else None
    check(lib().jf_layernorm_bwd_add(_ptr(qx), _ptr(sx), _ptr(qg), _ptr(sg), _ptr(gamma), _ptr(mean), _ptr(rstd), R, Cc,
                                     code, rounding, seed, offset, _ptr(x1), _FP_CODE[x1.dtype], add_rounding, add_seed,
                                     add_offset, _ptr(y1), _FP_CODE[out_dtype], _ptr(q), _ptr(s), _ptr(dgamma), _ptr(dbeta),
                                     _ptr(ws), nbytes, _stream()))
    return y1, q, s, dgamma, dbeta


def gelu_fwd(q, s, approx=GELU_ERF, amax_eps=5e-5):
    R, Cc, code = _block_tensor(q, s, "x")
    qy = torch.empty_like(q)
    sy = torch.empty_like(s)
    check(lib().jf_gelu_fwd(_ptr(q), _ptr(s), R, Cc, code, approx, amax_eps, _ptr(qy), _ptr(sy), _stream()))
    return qy, sy


def gelu_bwd(qx, sx, qg, sg, approx=GELU_ERF, rounding=ROUND_NEAREST, seed=None, offset=None):
    R, Cc, code = _block_tensor(qx, sx, "x")
    R2, C2, code2 = _block_tensor(qg, sg, "g")
    if (R2, C2, code2) != (R, Cc, code):
        raise RuntimeError("x and g must have the same shape and scale dtype")
    seed, offset = _rng(rounding, R * Cc, seed, offset, qx.device)
    qy = torch.empty_like(qx)
    sy = torch.empty_like(sx)
    check(lib().jf_gelu_bwd(_ptr(qx), _ptr(sx), _ptr(qg), _ptr(sg), R, Cc, code, approx, rounding, seed, offset,
                            _ptr(qy), _ptr(sy), _stream()))
    return qy, sy


def add(x1, q2, s2, rounding=ROUND_TRUNC, with_stats=False, seed=None, offset=None, out_dtype=torch.float32):
    """y = x1 + q2*s2 (fp32), returned in `out_dtype`, and its block quantisation; the quantisation and the row
    statistics are taken from the fp32 sum whatever `out_dtype` is."""
    R, Cc, code = _block_tensor(q2, s2, "x2")
    _need(x1, None, "x1")
    if x1.dtype not in _FP_CODE or tuple(x1.shape) != (R, Cc):
        raise RuntimeError("x1 must be a float tensor of the same shape as x2")
    if out_dtype not in _FP_CODE:
        raise RuntimeError("out_dtype must be float32, float16 or bfloat16")
    seed, offset = _rng(rounding, R * Cc, seed, offset, x1.device)
    y1 = torch.empty((R, Cc), dtype=out_dtype, device=x1.device)
    q = torch.empty_like(q2)
    s = torch.empty_like(s2)
    rs = torch.empty((Cc // QB, R), dtype=torch.float32, device=x1.device) if with_stats else None   # part-major
    rq = torch.empty((Cc // QB, R), dtype=torch.float32, device=x1.device) if with_stats else None
    check(lib().jf_add(_ptr(x1), _FP_CODE[x1.dtype], _ptr(q2), _ptr(s2), R, Cc, code, rounding, seed, offset,
                       _ptr(y1), _FP_CODE[out_dtype], _ptr(q), _ptr(s), _ptr(rs), _ptr(rq), _stream()))
    return (y1, q, s, rs, rq) if with_stats else (y1, q, s)


def block_colsum(q, s):
    """fp32 column sums of the block tensor (q, s) over all rows (the bias gradient of a linear layer)."""
    R, Cc, code = _block_tensor(q, s, "x")
    nbytes = lib().jf_block_colsum_workspace_bytes(R, Cc)
    ws = torch.empty(nbytes, dtype=torch.int8, device=q.device)
    out = torch.empty(Cc, dtype=torch.float32, device=q.device)
    check(lib().jf_block_colsum(_ptr(q), _ptr(s), R, Cc, code, _ptr(out), _ptr(ws), nbytes, _stream()))
    return out


def rowstats_finish(rowsum, rowsq, n_cols):
    """(mean, rstd) per row from add(..., with_stats=True)'s partial sums [parts, R]: partials added in ascending order,
    var = E[y^2] - mean^2, rstd = 1/sqrt(var), no epsilon."""
    _need(rowsum, torch.float32, "rowsum", 2)
    _need(rowsq, torch.float32, "rowsq", 2)
    if rowsum.shape != rowsq.shape:
        raise RuntimeError("rowsum and rowsq must have the same shape")
    parts, R = rowsum.shape
    mean = torch.empty(R, dtype=torch.float32, device=rowsum.device)
    rstd = torch.empty(R, dtype=torch.float32, device=rowsum.device)
    check(lib().jf_rowstats_finish(_ptr(rowsum), _ptr(rowsq), R, parts, int(n_cols), _ptr(mean), _ptr(rstd), _stream()))
    return mean, rstd


CAL_UNIFORM, CAL_SPLIT, CAL_STREAM, CAL_STREAM_DATA = 0, 1, 2, 3


def calibrate(with_mfma, valu_per_mfma, iters=2000, workgroups_per_cu=4, threads=256, mode=CAL_UNIFORM, launches=3):
    """Runs the register-only calibration kernel (jf_calibrate of the measurement library) and returns a dict: seconds per
    launch (events), the number of work items it ran (workgroups * waves * iters * 4; for CAL_SPLIT: items of the MFMA
    waves), the resident waves per SIMD, and the shader clock in MHz the kernel ran at (cycles / wall-clock time, from the
    per-workgroup readings of the last launch)."""
    props = torch.cuda.get_device_properties(0)
    cus = props.multi_processor_count
    wgs = cus * workgroups_per_cu
    waves = threads // 64
    scratch = torch.zeros(16, dtype=torch.float32, device="cuda")
    clocks = torch.zeros(2 * wgs, dtype=torch.int64, device="cuda")
    run = lambda: check(prof_lib().jf_calibrate(mode, with_mfma, valu_per_mfma, iters, wgs, threads, _ptr(scratch), _ptr(clocks),
                                                _stream()))
    run()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(launches):
        run()
    e1.record()
    torch.cuda.synchronize()
    c = clocks.view(wgs, 2).double().sum(0)
    wall_hz = _wall_clock_hz()
    items = wgs * (waves // 2 if mode == CAL_SPLIT else waves) * iters * 4
    return {"seconds": e0.elapsed_time(e1) * 1e-3 / launches, "items": items, "waves_per_simd": workgroups_per_cu * waves / 4,
            "shader_MHz": float(c[0] / c[1]) * wall_hz / 1e6, "simds": cus * 4}


def igemm_phases(A, B, sa, sb, b_layout=B_KN, rounding=ROUND_NEAREST, seed=0, offset=0):
    """igemm_block_q (fp32 scales) through the phase-recording build of its kernel (measurement library).  Returns
    (q, sc, phases): the same codes and scales, and per workgroup (one 128x128 output tile each) a dict of numpy arrays:
    'us' [workgroups, 6] (start, main loop begins, main loop ends, epilogue begins, blocks requantised, end; microseconds
    since the first workgroup started), 'cu' (an id of the CU it ran on), 'k_loop_MHz' (shader clock during its main
    loop) and 'k_loop_cycles'."""
    import numpy as np
    M, N, K, _, _ = _gemm_operands(A, B, b_layout)
    code, la, lb = _gemm_scales(sa, sb, M, N, K)
    if code != SCALE_F32:
        raise RuntimeError("igemm_phases: fp32 scales only")
    workgroups = ((M + 127) // 128) * ((N + 127) // 128)
    buf = torch.zeros(workgroups * 8, dtype=torch.int64, device=A.device)
    out = torch.empty((M, N), dtype=torch.int8, device=A.device)
    sc = torch.empty((M // QB, N // QB), dtype=torch.float32, device=A.device)
    check(prof_lib().jf_prof_igemm_block_q(_ptr(A), _ptr(B), _ptr(sa), _ptr(sb), None, None, _ptr(out), _ptr(sc), M, N, K,
                                           b_layout, la, lb, rounding, seed, offset, _ptr(buf), workgroups, _stream()))
    torch.cuda.synchronize()
    w = buf.view(workgroups, 8).cpu().numpy()
    hz = _wall_clock_hz()
    t = w[:, :6].astype(np.float64)
    us = (t - t[:, 0].min()) / hz * 1e6
    hw = w[:, 6]
    return out, sc, {"us": us, "cu": hw & 0xFF00 | ((hw >> 16) & 0xFF), "k_loop_cycles": w[:, 7].astype(np.float64),
                     "k_loop_MHz": w[:, 7] / np.maximum(t[:, 2] - t[:, 1], 1.0) * hz / 1e6}


def _wall_clock_hz():
    """Rate of the constant clock the kernel's wall-clock readings count in."""
    khz = prof_lib().jf_wall_clock_khz()
    if khz <= 0:
        raise RuntimeError("jf_wall_clock_khz: the device does not report a wall clock rate")
    return khz * 1e3
