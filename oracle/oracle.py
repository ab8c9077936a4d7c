"""numpy front-end of the CPU checker in jf_oracle.c (ctypes).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
cpu_baseline leg of the benchmark.  The shipped package never imports it.

All arrays are C-contiguous numpy arrays; block tensors are (q int8 [R,C],
s float32 [R/32,C/32]).  `scale_dtype="f16"` rounds produced scales to binary16
(returned as float16 arrays) the way the reference stores them
(Jetfire/Nonlinear/quantize.py:141); consumed scales are widened to float32,
which is exact.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libjf_oracle.so")
QB = 32


def build(force=False):
    """Compile jf_oracle.c with gcc (seconds)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE, "libjf_oracle.so"])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_p = C.c_void_p
_i = C.c_int
_u64 = C.c_uint64
_f = C.c_float


def _declare(L):
    L.jfo_philox4x32_10.argtypes = [_p, _p, _p]
    L.jfo_philox4x32.argtypes = [_p, _p, _i, _p]
    L.jfo_sr_noise.argtypes = [_u64, _u64, _u64]
    L.jfo_sr_noise.restype = _f
    L.jfo_f32_to_f16_bits.argtypes = [_f]
    L.jfo_f32_to_f16_bits.restype = C.c_uint16
    L.jfo_f16_bits_to_f32.argtypes = [C.c_uint16]
    L.jfo_f16_bits_to_f32.restype = _f
    L.jfo_quantize.argtypes = [_p, _i, _i, _p, _p, _i, _u64, _u64, _f, _i]
    L.jfo_dequantize.argtypes = [_p, _p, _i, _i, _p]
    L.jfo_transpose_s8.argtypes = [_p, _i, _i, _p]
    L.jfo_igemm_s32.argtypes = [_p, _p, _p, _i, _i, _i, _i]
    L.jfo_igemm_block_acc.argtypes = [_p, _p, _p, _i, _i, _i, _i]
    L.jfo_igemm_block_f32.argtypes = [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i]
    L.jfo_requant.argtypes = [_p, _i, _i, _p, _f, _i, _u64, _u64, _p, _p]
    for name in ("jfo_expf", "jfo_phi_neg", "jfo_norm_cdf", "jfo_tanhf"):
        getattr(L, name).argtypes = [_f]
        getattr(L, name).restype = _f
    for name in ("jfo_gelu", "jfo_dgelu"):
        getattr(L, name).argtypes = [_f, _i]
        getattr(L, name).restype = _f
    L.jfo_gelu_fwd.argtypes = [_p, _p, _i, _i, _i, _f, _p, _p]
    L.jfo_gelu_bwd.argtypes = [_p, _p, _p, _p, _i, _i, _i, _i, _u64, _u64, _p, _p]
    L.jfo_rowstats.argtypes = [_p, _p, _i, _i, _f, _p, _p]
    L.jfo_layernorm_fwd.argtypes = [_p, _p, _i, _i, _p, _p, _p, _p, _p, _p]
    L.jfo_layernorm_bwd.argtypes = [_p, _p, _p, _p, _i, _i, _p, _p, _p, _i, _u64, _u64, _p, _p, _p, _p]
    L.jfo_add.argtypes = [_p, _p, _p, _i, _i, _i, _u64, _u64, _i, _p, _p, _p, _p, _p]
    L.jfo_block_colsum.argtypes = [_p, _p, _i, _i, _p]


def _ptr(a):
    return None if a is None else a.ctypes.data_as(_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _scale_out(s, scale_dtype):
    if scale_dtype == "f16":
        return s.astype(np.float16)
    assert scale_dtype == "f32"
    return s


def _chk(R, C_):
    if R % QB or C_ % QB or R <= 0 or C_ <= 0:
        raise ValueError(f"shape ({R},{C_}) is not a positive multiple of {QB}")


def set_threads(n):
    """Limit the OpenMP team (the benchmark reports the count it used)."""
    C.CDLL("libgomp.so.1").omp_set_num_threads(int(n))


# --------------------------------------------------------------------------- RNG
def philox4x32_10(ctr, key):
    c = np.asarray(ctr, dtype=np.uint32).copy()
    k = np.asarray(key, dtype=np.uint32).copy()
    o = np.zeros(4, dtype=np.uint32)
    lib().jfo_philox4x32_10(_ptr(c), _ptr(k), _ptr(o))
    return o


NOISE_ROUNDS = 7            # rounds of the generator behind sr_noise (JFO_NOISE_ROUNDS); see set_noise_rounds


def set_noise_rounds(rounds):
    """Follow the round count the library under test was built with (jf_philox_rounds())."""
    global NOISE_ROUNDS
    lib().jfo_set_noise_rounds.argtypes = [_i]
    NOISE_ROUNDS = int(lib().jfo_set_noise_rounds(int(rounds)))
    return NOISE_ROUNDS


def philox4x32(ctr, key, rounds):
    c = np.asarray(ctr, dtype=np.uint32).copy()
    k = np.asarray(key, dtype=np.uint32).copy()
    o = np.zeros(4, dtype=np.uint32)
    lib().jfo_philox4x32(_ptr(c), _ptr(k), rounds, _ptr(o))
    return o


def sr_noise(seed, offset, e):
    return float(lib().jfo_sr_noise(seed, offset, e))


def f32_to_f16_bits(x):
    return int(lib().jfo_f32_to_f16_bits(float(x)))


# --------------------------------------------------------------------------- quantise family
def quantize(x, stochastic=False, seed=0, offset=0, amax_eps=0.0, truncate=False, scale_dtype="f32"):
    x = _c(x, np.float32)
    R, C_ = x.shape
    _chk(R, C_)
    q = np.empty((R, C_), np.int8)
    s = np.empty((R // QB, C_ // QB), np.float32)
    lib().jfo_quantize(_ptr(x), R, C_, _ptr(q), _ptr(s), int(stochastic), seed, offset, amax_eps, int(truncate))
    return q, _scale_out(s, scale_dtype)


def dequantize(q, s):
    q = _c(q, np.int8)
    s = _c(s, np.float32)
    R, C_ = q.shape
    _chk(R, C_)
    x = np.empty((R, C_), np.float32)
    lib().jfo_dequantize(_ptr(q), _ptr(s), R, C_, _ptr(x))
    return x


def transpose_s8(q):
    q = _c(q, np.int8)
    R, C_ = q.shape
    out = np.empty((C_, R), np.int8)
    lib().jfo_transpose_s8(_ptr(q), R, C_, _ptr(out))
    return out


# --------------------------------------------------------------------------- GEMMs
def _gemm_dims(A, B, b_layout):
    M, K = A.shape
    if b_layout == 0:
        N, K2 = B.shape
    else:
        K2, N = B.shape
    if K != K2:
        raise ValueError("inner dimensions differ")
    _chk(M, N)
    _chk(K, K)
    return M, N, K


def igemm_s32(A, B, b_layout):
    A = _c(A, np.int8)
    B = _c(B, np.int8)
    M, N, K = _gemm_dims(A, B, b_layout)
    out = np.empty((M, N), np.int32)
    lib().jfo_igemm_s32(_ptr(A), _ptr(B), _ptr(out), M, N, K, b_layout)
    return out


def igemm_block_acc(A, B, b_layout):
    """INT32 accumulators of every 32-deep K block: [K/32, M, N]."""
    A = _c(A, np.int8)
    B = _c(B, np.int8)
    M, N, K = _gemm_dims(A, B, b_layout)
    out = np.empty((K // QB, M, N), np.int32)
    lib().jfo_igemm_block_acc(_ptr(A), _ptr(B), _ptr(out), M, N, K, b_layout)
    return out


def igemm_block_f32(A, B, sa, sb, b_layout, fused=True):
    """fp32 dequantise-accumulate; sa [K/32, M/32], sb [K/32, N/32]."""
    A = _c(A, np.int8)
    B = _c(B, np.int8)
    sa = _c(sa, np.float32)
    sb = _c(sb, np.float32)
    M, N, K = _gemm_dims(A, B, b_layout)
    if sa.shape != (K // QB, M // QB) or sb.shape != (K // QB, N // QB):
        raise ValueError("scale shapes must be [K/32,M/32] and [K/32,N/32]")
    out = np.empty((M, N), np.float32)
    lib().jfo_igemm_block_f32(_ptr(A), _ptr(B), _ptr(sa), _ptr(sb), _ptr(out), M, N, K, b_layout, int(fused))
    return out


def igemm_block_f32_splitk(A, B, sa, sb, b_layout, parts, kb_per_part):
    """The K-split variant of the fp-output GEMM (an addition of this library's C ABI, no counterpart in the reference):
    part p accumulates K blocks [p*kb_per_part, (p+1)*kb_per_part) exactly as igemm_block_f32 does, and the partial
    results are added in ascending order in fp32.  Pinned by construction: igemm_block_f32 on K slices + IEEE adds."""
    A = _c(A, np.int8)
    B = _c(B, np.int8)
    sa = _c(sa, np.float32)
    sb = _c(sb, np.float32)
    M, N, K = _gemm_dims(A, B, b_layout)
    out = None
    for p in range(parts):
        kb0, kb1 = p * kb_per_part, min((p + 1) * kb_per_part, K // QB)
        ks = slice(kb0 * QB, kb1 * QB)
        Bp = B[ks, :] if b_layout == 1 else B[:, ks]
        part = igemm_block_f32(np.ascontiguousarray(A[:, ks]), np.ascontiguousarray(Bp), sa[kb0:kb1], sb[kb0:kb1], b_layout)
        out = part if out is None else (out + part).astype(np.float32)
    return out


def requant(acc, bias=None, biasmax=0.0, stochastic=False, seed=0, offset=0, scale_dtype="f32"):
    acc = _c(acc, np.float32)
    M, N = acc.shape
    _chk(M, N)
    b = None if bias is None else _c(bias, np.float32)
    q = np.empty((M, N), np.int8)
    sc = np.empty((M // QB, N // QB), np.float32)
    lib().jfo_requant(_ptr(acc), M, N, _ptr(b), float(biasmax), int(stochastic), seed, offset, _ptr(q), _ptr(sc))
    return q, _scale_out(sc, scale_dtype)


def igemm_block_q(A, B, sa, sb, b_layout, bias=None, biasmax=0.0, stochastic=False, seed=0, offset=0,
                  scale_dtype="f32"):
    """The fused kernels: accumulate, then requantise per 32x32 output block."""
    acc = igemm_block_f32(A, B, sa, sb, b_layout)
    return requant(acc, bias, biasmax, stochastic, seed, offset, scale_dtype)


def igemm_block_fp(A, B, sa, sb, b_layout, out_dtype="f16"):
    acc = igemm_block_f32(A, B, sa, sb, b_layout)
    return acc.astype(np.float16) if out_dtype == "f16" else acc


# --------------------------------------------------------------------------- elementary functions
def _vec(fn, x, *extra):
    x = np.asarray(x, dtype=np.float32)
    f = getattr(lib(), fn)
    return np.array([f(float(v), *extra) for v in x.ravel()], dtype=np.float32).reshape(x.shape)


def expf(x):
    return _vec("jfo_expf", x)


def phi_neg(x):
    return _vec("jfo_phi_neg", x)


def norm_cdf(x):
    return _vec("jfo_norm_cdf", x)


def tanhf(x):
    return _vec("jfo_tanhf", x)


def gelu(x, approx=0):
    return _vec("jfo_gelu", x, approx)


def dgelu(x, approx=0):
    return _vec("jfo_dgelu", x, approx)


# --------------------------------------------------------------------------- fused nonlinear ops
def gelu_fwd(q, s, approx=0, amax_eps=5e-5, scale_dtype="f32"):
    q = _c(q, np.int8)
    s = _c(s, np.float32)
    R, C_ = q.shape
    _chk(R, C_)
    qy = np.empty_like(q)
    sy = np.empty_like(s)
    lib().jfo_gelu_fwd(_ptr(q), _ptr(s), R, C_, approx, amax_eps, _ptr(qy), _ptr(sy))
    return qy, _scale_out(sy, scale_dtype)


def gelu_bwd(qx, sx, qg, sg, approx=0, stochastic=False, seed=0, offset=0, scale_dtype="f32"):
    qx = _c(qx, np.int8)
    sx = _c(sx, np.float32)
    qg = _c(qg, np.int8)
    sg = _c(sg, np.float32)
    R, C_ = qx.shape
    _chk(R, C_)
    qy = np.empty_like(qx)
    sy = np.empty_like(sx)
    lib().jfo_gelu_bwd(_ptr(qx), _ptr(sx), _ptr(qg), _ptr(sg), R, C_, approx, int(stochastic), seed, offset,
                       _ptr(qy), _ptr(sy))
    return qy, _scale_out(sy, scale_dtype)


def rowstats(q, s, eps=1e-5):
    q = _c(q, np.int8)
    s = _c(s, np.float32)
    R, C_ = q.shape
    _chk(R, C_)
    mean = np.empty(R, np.float32)
    rstd = np.empty(R, np.float32)
    lib().jfo_rowstats(_ptr(q), _ptr(s), R, C_, eps, _ptr(mean), _ptr(rstd))
    return mean, rstd


def layernorm_fwd(q, s, gamma, beta, mean, rstd, scale_dtype="f32"):
    q = _c(q, np.int8)
    s = _c(s, np.float32)
    gamma = _c(gamma, np.float32)
    beta = None if beta is None else _c(beta, np.float32)
    mean = _c(mean, np.float32)
    rstd = _c(rstd, np.float32)
    R, C_ = q.shape
    _chk(R, C_)
    qy = np.empty_like(q)
    sy = np.empty_like(s)
    lib().jfo_layernorm_fwd(_ptr(q), _ptr(s), R, C_, _ptr(gamma), _ptr(beta), _ptr(mean), _ptr(rstd),
                            _ptr(qy), _ptr(sy))
    return qy, _scale_out(sy, scale_dtype)


def layernorm_bwd(qx, sx, qg, sg, gamma, mean, rstd, stochastic=False, seed=0, offset=0, scale_dtype="f32"):
    qx = _c(qx, np.int8)
    sx = _c(sx, np.float32)
    qg = _c(qg, np.int8)
    sg = _c(sg, np.float32)
    gamma = _c(gamma, np.float32)
    mean = _c(mean, np.float32)
    rstd = _c(rstd, np.float32)
    R, C_ = qx.shape
    _chk(R, C_)
    qdx = np.empty_like(qx)
    sdx = np.empty_like(sx)
    dgamma = np.empty(C_, np.float32)
    dbeta = np.empty(C_, np.float32)
    lib().jfo_layernorm_bwd(_ptr(qx), _ptr(sx), _ptr(qg), _ptr(sg), R, C_, _ptr(gamma), _ptr(mean), _ptr(rstd),
                            int(stochastic), seed, offset, _ptr(qdx), _ptr(sdx), _ptr(dgamma), _ptr(dbeta))
    return qdx, _scale_out(sdx, scale_dtype), dgamma, dbeta


def add(x1, q2, s2, stochastic=False, seed=0, offset=0, truncate=True, with_stats=False, scale_dtype="f32"):
    x1 = _c(x1, np.float32)
    q2 = _c(q2, np.int8)
    s2 = _c(s2, np.float32)
    R, C_ = x1.shape
    _chk(R, C_)
    y1 = np.empty_like(x1)
    q = np.empty_like(q2)
    s = np.empty_like(s2)
    rs = np.empty((C_ // QB, R), np.float32) if with_stats else None       # part-major
    rq = np.empty((C_ // QB, R), np.float32) if with_stats else None
    lib().jfo_add(_ptr(x1), _ptr(q2), _ptr(s2), R, C_, int(stochastic), seed, offset, int(truncate),
                  _ptr(y1), _ptr(q), _ptr(s), _ptr(rs), _ptr(rq))
    if with_stats:
        return y1, q, _scale_out(s, scale_dtype), rs, rq
    return y1, q, _scale_out(s, scale_dtype)


def block_colsum(q, s):
    """Column sums of the block tensor (q, s) in fp32, in the library's fixed order (the bias gradient of a linear layer)."""
    q = _c(q, np.int8)
    s = _c(s, np.float32)
    R, C_ = q.shape
    _chk(R, C_)
    out = np.empty(C_, np.float32)
    lib().jfo_block_colsum(_ptr(q), _ptr(s), R, C_, _ptr(out))
    return out
