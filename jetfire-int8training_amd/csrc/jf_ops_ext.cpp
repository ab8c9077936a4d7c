// BlockQuantizeCUDA.jetfire -- the rest of the host side of the INT8 data-flow path as PyTorch C++ functions: the
// operators of Jetfire/Nonlinear (quantize, transpose, dequantize, LayerNorm, GELU, residual add; reference launchers:
// Jetfire/Nonlinear/*.py) and the GEMMs with fused epilogues that Jetfire/Linear uses besides the reference's eight
// (bindings.cpp:6-35 lives in bqc_ext.cpp).  The reference launches its Triton kernels from Python; here every operator
// is one C++ call that validates its tensors, allocates the outputs, reserves Philox counters under the generator's
// mutex, releases the GIL and enqueues the gfx950 kernel on the current stream through the C ABI.
//
// All tensors are 2-D ([R, C] codes / values, [R/32, C/32] scales, 1-D vectors); the Python packages fold 3-D operands.
// seed / offset arguments: None = reserve from the device's default generator (what the operator API does); integers =
// use exactly these (tests, captured graphs).
#include "bqc_common.h"

#include <vector>

namespace jfext {
namespace {

using torch::Tensor;
using OptU64 = c10::optional<uint64_t>;
using OptTensor = c10::optional<Tensor>;
using OptDtype = c10::optional<torch::ScalarType>;

int fp_code(torch::ScalarType t, const char *name)
{
    if (t == torch::kFloat16) return JF_FP_F16;
    if (t == torch::kFloat32) return JF_FP_F32;
    if (t == torch::kBFloat16) return JF_FP_BF16;
    TORCH_CHECK(false, name, ": expected float16, float32 or bfloat16, got ", t);
    return -1;
}

int scale_code_of(torch::ScalarType t)
{
    TORCH_CHECK(t == torch::kFloat16 || t == torch::kFloat32, "scale_dtype must be float16 or float32, got ", t);
    return t == torch::kFloat16 ? JF_SCALE_F16 : JF_SCALE_F32;
}

void check_rounding(int64_t r, bool trunc_ok)
{
    TORCH_CHECK(r == JF_ROUND_NEAREST || r == JF_ROUND_STOCHASTIC ||
                    (trunc_ok && (r == JF_ROUND_TRUNC || r == JF_ROUND_STOCHASTIC_TRUNC)),
                "unknown rounding code ", r);
}

bool is_stochastic(int64_t r) { return r == JF_ROUND_STOCHASTIC || r == JF_ROUND_STOCHASTIC_TRUNC; }

void need(const Tensor &t, const char *name, int64_t dim)
{
    TORCH_CHECK(t.is_cuda(), name, ": expected a GPU tensor");
    TORCH_CHECK(t.dim() == dim, name, ": expected ", dim, " dimensions, got ", t.dim());
    TORCH_CHECK(t.is_contiguous(), name, ": expected a contiguous tensor");
}

void mult32(int64_t d)
{
    TORCH_CHECK(d > 0 && d % QB == 0, "dimension ", d, " is not a positive multiple of 32");
}

// (codes [R,C] int8, scales [R/32,C/32]) -> scale code; R, C out
int block_tensor(const Tensor &q, const Tensor &s, const char *name, int64_t &R, int64_t &C)
{
    need(q, name, 2);
    TORCH_CHECK(q.scalar_type() == torch::kInt8, name, ": codes must be int8, got ", q.scalar_type());
    R = q.size(0); C = q.size(1);
    mult32(R); mult32(C);
    need(s, name, 2);
    TORCH_CHECK(s.size(0) == R / QB && s.size(1) == C / QB, name, ": scale shape ", s.sizes(), " does not match codes ", q.sizes());
    TORCH_CHECK(s.device() == q.device(), name, ": codes and scales are on different devices");
    return scale_code(s, name);
}

const float *vec(const Tensor &v, int64_t n, const Tensor &like, const char *name)
{
    need(v, name, 1);
    TORCH_CHECK(v.scalar_type() == torch::kFloat32 && v.numel() == n && v.device() == like.device(), name,
                ": expected a float32 vector of ", n, " elements on ", like.device());
    return v.data_ptr<float>();
}

// (seed, offset): the given pair, or counters reserved from the device's generator when the rounding draws noise
std::pair<uint64_t, uint64_t> rng(int64_t rounding, const Tensor &like, int64_t numel, const OptU64 &seed, const OptU64 &offset)
{
    if (is_stochastic(rounding) && !seed.has_value()) return next_philox(like, numel);
    return {seed.value_or(0), offset.value_or(0)};
}

Tensor scratch(const Tensor &like, size_t bytes)
{
    return torch::empty({(int64_t)(bytes ? bytes : 16)}, like.options().dtype(torch::kInt8));
}

// ---- quantize / dequantize / transpose -----------------------------------------------------------------------------

// quantize.py:128-164; with transpose: quantize_transpose.py:131-171
std::tuple<Tensor, Tensor, OptTensor> quantize(const Tensor &x, int64_t rounding, OptDtype scale_dtype_o, bool transpose,
                                               double amax_eps, OptU64 seed, OptU64 offset)
{
    need(x, "x", 2);
    const int xc = fp_code(x.scalar_type(), "x");
    const int64_t R = x.size(0), C = x.size(1);
    mult32(R); mult32(C);
    check_rounding(rounding, true);
    const torch::ScalarType scale_dtype = scale_dtype_o.value_or(torch::kFloat16);
    const int sc = scale_code_of(scale_dtype);
    c10::DeviceGuard guard(x.device());
    Tensor q = torch::empty({R, C}, x.options().dtype(torch::kInt8));
    Tensor s = torch::empty({R / QB, C / QB}, x.options().dtype(scale_dtype));
    OptTensor qT;
    if (transpose) qT = torch::empty({C, R}, x.options().dtype(torch::kInt8));
    const auto so = rng(rounding, x, R * C, seed, offset);
    {
        pybind11::gil_scoped_release nogil;
        check_rc(jf_quantize(x.data_ptr(), xc, (int)R, (int)C, (int8_t *)q.data_ptr(), s.data_ptr(),
                             transpose ? (int8_t *)qT->data_ptr() : nullptr, sc, (int)rounding, so.first, so.second,
                             (float)amax_eps, current_stream(x)),
                 "quantize");
    }
    return std::make_tuple(q, s, qT);
}

// the block tensor of torch.cat(slabs, dim=1) without the concatenation (jf_quantize_slabs)
std::tuple<Tensor, Tensor> quantize_slabs(const std::vector<Tensor> &slabs, int64_t rounding, OptDtype scale_dtype_o,
                                          double amax_eps, OptU64 seed, OptU64 offset)
{
    TORCH_CHECK(!slabs.empty() && slabs.size() <= 4, "between 1 and 4 slabs");
    const Tensor &x0 = slabs[0];
    const int64_t R = x0.dim() == 2 ? x0.size(0) : -1;
    int64_t Ct = 0;
    const void *xs[4];
    int ld[4], wd[4];
    for (size_t k = 0; k < slabs.size(); ++k) {
        const Tensor &x = slabs[k];
        TORCH_CHECK(x.is_cuda() && x.dim() == 2 && x.size(0) == R && x.stride(1) == 1 && x.device() == x0.device() &&
                        x.scalar_type() == x0.scalar_type(),
                    "slabs: expected 2-D GPU tensors of one dtype with the same number of rows and unit column stride");
        mult32(x.size(1));
        xs[k] = x.data_ptr(); ld[k] = (int)x.stride(0); wd[k] = (int)x.size(1);
        Ct += x.size(1);
    }
    mult32(R);
    const int xc = fp_code(x0.scalar_type(), "slabs");
    check_rounding(rounding, true);
    const torch::ScalarType scale_dtype = scale_dtype_o.value_or(torch::kFloat16);
    const int sc = scale_code_of(scale_dtype);
    c10::DeviceGuard guard(x0.device());
    Tensor q = torch::empty({R, Ct}, x0.options().dtype(torch::kInt8));
    Tensor s = torch::empty({R / QB, Ct / QB}, x0.options().dtype(scale_dtype));
    const auto so = rng(rounding, x0, R * Ct, seed, offset);
    {
        pybind11::gil_scoped_release nogil;
        check_rc(jf_quantize_slabs(xs, ld, wd, (int)slabs.size(), xc, (int)R, (int8_t *)q.data_ptr(), s.data_ptr(), sc,
                                   (int)rounding, so.first, so.second, (float)amax_eps, current_stream(x0)),
                 "quantize_slabs");
    }
    return std::make_tuple(q, s);
}

// dequantize.py:86-116
Tensor dequantize(const Tensor &q, const Tensor &s, OptDtype out_dtype_o)
{
    const torch::ScalarType out_dtype = out_dtype_o.value_or(torch::kFloat32);
    int64_t R, C;
    const int sc = block_tensor(q, s, "x", R, C);
    const int oc = fp_code(out_dtype, "out_dtype");
    c10::DeviceGuard guard(q.device());
    Tensor out = torch::empty({R, C}, q.options().dtype(out_dtype));
    pybind11::gil_scoped_release nogil;
    check_rc(jf_dequantize((const int8_t *)q.data_ptr(), s.data_ptr(), (int)R, (int)C, sc, out.data_ptr(), oc, current_stream(q)),
             "dequantize");
    return out;
}

// transpose.py:69-97
Tensor transpose_s8(const Tensor &q)
{
    need(q, "x", 2);
    TORCH_CHECK(q.scalar_type() == torch::kInt8, "x must be int8");
    const int64_t R = q.size(0), C = q.size(1);
    TORCH_CHECK(R > 0 && C > 0 && R % 16 == 0 && C % 16 == 0, "transpose: dimensions must be positive multiples of 16");
    c10::DeviceGuard guard(q.device());
    Tensor out = torch::empty({C, R}, q.options());
    pybind11::gil_scoped_release nogil;
    check_rc(jf_transpose_s8((const int8_t *)q.data_ptr(), (int)R, (int)C, (int8_t *)out.data_ptr(), current_stream(q)), "transpose");
    return out;
}

// ---- LayerNorm -----------------------------------------------------------------------------------------------------

std::tuple<Tensor, Tensor> rowstats(const Tensor &q, const Tensor &s, double eps)
{
    int64_t R, C;
    const int sc = block_tensor(q, s, "x", R, C);
    c10::DeviceGuard guard(q.device());
    Tensor mean = torch::empty({R}, q.options().dtype(torch::kFloat32)), rstd = torch::empty_like(mean);
    pybind11::gil_scoped_release nogil;
    check_rc(jf_rowstats((const int8_t *)q.data_ptr(), s.data_ptr(), (int)R, (int)C, sc, (float)eps, mean.data_ptr<float>(),
                         rstd.data_ptr<float>(), current_stream(q)),
             "rowstats");
    return std::make_tuple(mean, rstd);
}

// layernorm.py:430-465
std::tuple<Tensor, Tensor> layernorm_fwd(const Tensor &q, const Tensor &s, const Tensor &gamma, const OptTensor &beta,
                                         const Tensor &mean, const Tensor &rstd)
{
    int64_t R, C;
    const int sc = block_tensor(q, s, "x", R, C);
    const float *g = vec(gamma, C, q, "gamma"), *b = beta ? vec(*beta, C, q, "beta") : nullptr;
    const float *m = vec(mean, R, q, "mean"), *r = vec(rstd, R, q, "rstd");
    c10::DeviceGuard guard(q.device());
    Tensor qy = torch::empty_like(q), sy = torch::empty_like(s);
    pybind11::gil_scoped_release nogil;
    check_rc(jf_layernorm_fwd((const int8_t *)q.data_ptr(), s.data_ptr(), g, b, m, r, (int)R, (int)C, sc, (int8_t *)qy.data_ptr(),
                              sy.data_ptr(), current_stream(q)),
             "layernorm_fwd");
    return std::make_tuple(qy, sy);
}

// layernorm.py:467-526
std::tuple<Tensor, Tensor, Tensor, OptTensor> layernorm_bwd(const Tensor &qx, const Tensor &sx, const Tensor &qg, const Tensor &sg,
                                                            const Tensor &gamma, const Tensor &mean, const Tensor &rstd,
                                                            int64_t rounding, bool want_dbeta, OptU64 seed, OptU64 offset)
{
    int64_t R, C, R2, C2;
    const int sc = block_tensor(qx, sx, "x", R, C);
    TORCH_CHECK(block_tensor(qg, sg, "g", R2, C2) == sc && R2 == R && C2 == C && qg.device() == qx.device(),
                "x and g must have the same shape, scale dtype and device");
    const float *g = vec(gamma, C, qx, "gamma"), *m = vec(mean, R, qx, "mean"), *r = vec(rstd, R, qx, "rstd");
    check_rounding(rounding, true);
    c10::DeviceGuard guard(qx.device());
    const size_t nbytes = jf_layernorm_bwd_workspace_bytes((int)R, (int)C);
    Tensor ws = scratch(qx, nbytes);
    Tensor qdx = torch::empty_like(qx), sdx = torch::empty_like(sx);
    Tensor dgamma = torch::empty({C}, qx.options().dtype(torch::kFloat32));
    OptTensor dbeta;
    if (want_dbeta) dbeta = torch::empty_like(dgamma);
    const auto so = rng(rounding, qx, R * C, seed, offset);
    {
        pybind11::gil_scoped_release nogil;
        check_rc(jf_layernorm_bwd((const int8_t *)qx.data_ptr(), sx.data_ptr(), (const int8_t *)qg.data_ptr(), sg.data_ptr(), g, m, r,
                                  (int)R, (int)C, sc, (int)rounding, so.first, so.second, (int8_t *)qdx.data_ptr(), sdx.data_ptr(),
                                  dgamma.data_ptr<float>(), want_dbeta ? dbeta->data_ptr<float>() : nullptr, ws.data_ptr(), nbytes,
                                  current_stream(qx)),
                 "layernorm_bwd");
    }
    return std::make_tuple(qdx, sdx, dgamma, dbeta);
}

// add.py:164-211 / add_mean_var.py:179-230 (with_stats: the row statistics are finished here as well, :219-221)
std::tuple<Tensor, Tensor, Tensor, OptTensor, OptTensor> add(const Tensor &x1, const Tensor &q2, const Tensor &s2, int64_t rounding,
                                                             bool with_stats, OptDtype out_dtype_o, OptU64 seed, OptU64 offset)
{
    const torch::ScalarType out_dtype = out_dtype_o.value_or(torch::kFloat32);
    int64_t R, C;
    const int sc = block_tensor(q2, s2, "x2", R, C);
    need(x1, "x1", 2);
    const int xc = fp_code(x1.scalar_type(), "x1"), oc = fp_code(out_dtype, "out_dtype");
    TORCH_CHECK(x1.size(0) == R && x1.size(1) == C && x1.device() == q2.device(), "x1 must be a float tensor of the shape and device of x2");
    check_rounding(rounding, true);
    c10::DeviceGuard guard(x1.device());
    Tensor y1 = torch::empty({R, C}, x1.options().dtype(out_dtype));
    Tensor q = torch::empty_like(q2), s = torch::empty_like(s2);
    Tensor rs, rq;
    OptTensor mean, rstd;
    if (with_stats) {
        rs = torch::empty({C / QB, R}, x1.options().dtype(torch::kFloat32));          // part-major
        rq = torch::empty_like(rs);
        mean = torch::empty({R}, x1.options().dtype(torch::kFloat32));
        rstd = torch::empty_like(*mean);
    }
    const auto so = rng(rounding, x1, R * C, seed, offset);
    {
        pybind11::gil_scoped_release nogil;
        const jf_stream_t st = current_stream(x1);
        check_rc(jf_add(x1.data_ptr(), xc, (const int8_t *)q2.data_ptr(), s2.data_ptr(), (int)R, (int)C, sc, (int)rounding, so.first,
                        so.second, y1.data_ptr(), oc, (int8_t *)q.data_ptr(), s.data_ptr(), with_stats ? rs.data_ptr<float>() : nullptr,
                        with_stats ? rq.data_ptr<float>() : nullptr, st),
                 "add");
        if (with_stats)
            check_rc(jf_rowstats_finish(rs.data_ptr<float>(), rq.data_ptr<float>(), (int)R, (int)(C / QB), (int)C,
                                        mean->data_ptr<float>(), rstd->data_ptr<float>(), st),
                     "rowstats_finish");
    }
    return std::make_tuple(y1, q, s, mean, rstd);
}

// the pair layernorm.py:467-526 + add.py:164-211 (qmodel.py:125-128, 258-261): one kernel for rows of up to 2048 columns,
// the two calls (same noise counters, same bits) beyond
std::tuple<Tensor, Tensor, Tensor, Tensor, OptTensor> layernorm_bwd_add(const Tensor &qx, const Tensor &sx, const Tensor &qg,
                                                                        const Tensor &sg, const Tensor &gamma, const Tensor &mean,
                                                                        const Tensor &rstd, const Tensor &x1, int64_t rounding,
                                                                        int64_t add_rounding, bool want_dbeta,
                                                                        OptDtype out_dtype_o, OptU64 seed, OptU64 offset,
                                                                        OptU64 add_seed, OptU64 add_offset)
{
    const torch::ScalarType out_dtype = out_dtype_o.value_or(torch::kFloat32);
    int64_t R, C, R2, C2;
    const int sc = block_tensor(qx, sx, "x", R, C);
    TORCH_CHECK(block_tensor(qg, sg, "g", R2, C2) == sc && R2 == R && C2 == C && qg.device() == qx.device(),
                "x and g must have the same shape, scale dtype and device");
    const float *g = vec(gamma, C, qx, "gamma"), *m = vec(mean, R, qx, "mean"), *r = vec(rstd, R, qx, "rstd");
    need(x1, "x1", 2);
    const int xc = fp_code(x1.scalar_type(), "x1"), oc = fp_code(out_dtype, "out_dtype");
    TORCH_CHECK(x1.size(0) == R && x1.size(1) == C && x1.device() == qx.device(), "x1 must be a float tensor of the shape and device of x");
    check_rounding(rounding, true);
    check_rounding(add_rounding, true);
    const auto so = rng(rounding, qx, R * C, seed, offset);
    const auto ao = rng(add_rounding, qx, R * C, add_seed, add_offset);
    if (C / QB > 64) {
        auto [qdx, sdx, dgamma, dbeta] = layernorm_bwd(qx, sx, qg, sg, gamma, mean, rstd, rounding, want_dbeta, so.first, so.second);
        auto [y1, q, s, _m, _r] = add(x1, qdx, sdx, add_rounding, false, out_dtype, ao.first, ao.second);
        return std::make_tuple(y1, q, s, dgamma, dbeta);
    }
    c10::DeviceGuard guard(qx.device());
    const size_t nbytes = jf_layernorm_bwd_workspace_bytes((int)R, (int)C);
    Tensor ws = scratch(qx, nbytes);
    Tensor y1 = torch::empty({R, C}, x1.options().dtype(out_dtype));
    Tensor q = torch::empty_like(qx), s = torch::empty_like(sx);
    Tensor dgamma = torch::empty({C}, qx.options().dtype(torch::kFloat32));
    OptTensor dbeta;
    if (want_dbeta) dbeta = torch::empty_like(dgamma);
    {
        pybind11::gil_scoped_release nogil;
        check_rc(jf_layernorm_bwd_add((const int8_t *)qx.data_ptr(), sx.data_ptr(), (const int8_t *)qg.data_ptr(), sg.data_ptr(), g, m, r,
                                      (int)R, (int)C, sc, (int)rounding, so.first, so.second, x1.data_ptr(), xc, (int)add_rounding,
                                      ao.first, ao.second, y1.data_ptr(), oc, (int8_t *)q.data_ptr(), s.data_ptr(),
                                      dgamma.data_ptr<float>(), want_dbeta ? dbeta->data_ptr<float>() : nullptr, ws.data_ptr(), nbytes,
                                      current_stream(qx)),
                 "layernorm_bwd_add");
    }
    return std::make_tuple(y1, q, s, dgamma, dbeta);
}

// ---- GELU ----------------------------------------------------------------------------------------------------------

void check_approx(int64_t a) { TORCH_CHECK(a == JF_GELU_ERF || a == JF_GELU_TANH, "unknown GELU form ", a); }

// gelu_fwd.py:128-162
std::tuple<Tensor, Tensor> gelu_fwd(const Tensor &q, const Tensor &s, int64_t approx, double amax_eps)
{
    int64_t R, C;
    const int sc = block_tensor(q, s, "x", R, C);
    check_approx(approx);
    c10::DeviceGuard guard(q.device());
    Tensor qy = torch::empty_like(q), sy = torch::empty_like(s);
    pybind11::gil_scoped_release nogil;
    check_rc(jf_gelu_fwd((const int8_t *)q.data_ptr(), s.data_ptr(), (int)R, (int)C, sc, (int)approx, (float)amax_eps,
                         (int8_t *)qy.data_ptr(), sy.data_ptr(), current_stream(q)),
             "gelu_fwd");
    return std::make_tuple(qy, sy);
}

// gelu_bwd.py:173-215
std::tuple<Tensor, Tensor> gelu_bwd(const Tensor &qx, const Tensor &sx, const Tensor &qg, const Tensor &sg, int64_t approx,
                                    int64_t rounding, OptU64 seed, OptU64 offset)
{
    int64_t R, C, R2, C2;
    const int sc = block_tensor(qx, sx, "x", R, C);
    TORCH_CHECK(block_tensor(qg, sg, "g", R2, C2) == sc && R2 == R && C2 == C && qg.device() == qx.device(),
                "x and g must have the same shape, scale dtype and device");
    check_approx(approx);
    check_rounding(rounding, true);
    c10::DeviceGuard guard(qx.device());
    Tensor qy = torch::empty_like(qx), sy = torch::empty_like(sx);
    const auto so = rng(rounding, qx, R * C, seed, offset);
    pybind11::gil_scoped_release nogil;
    check_rc(jf_gelu_bwd((const int8_t *)qx.data_ptr(), sx.data_ptr(), (const int8_t *)qg.data_ptr(), sg.data_ptr(), (int)R, (int)C, sc,
                         (int)approx, (int)rounding, so.first, so.second, (int8_t *)qy.data_ptr(), sy.data_ptr(), current_stream(qx)),
             "gelu_bwd");
    return std::make_tuple(qy, sy);
}

// ---- column sums (bias gradient; QBlockLinear.py:63-66) -------------------------------------------------------------

Tensor block_colsum(const Tensor &q, const Tensor &s)
{
    int64_t R, C;
    const int sc = block_tensor(q, s, "x", R, C);
    c10::DeviceGuard guard(q.device());
    const size_t nbytes = jf_block_colsum_workspace_bytes((int)R, (int)C);
    Tensor ws = scratch(q, nbytes);
    Tensor out = torch::empty({C}, q.options().dtype(torch::kFloat32));
    pybind11::gil_scoped_release nogil;
    check_rc(jf_block_colsum((const int8_t *)q.data_ptr(), s.data_ptr(), (int)R, (int)C, sc, out.data_ptr<float>(), ws.data_ptr(), nbytes,
                             current_stream(q)),
             "block_colsum");
    return out;
}

// ---- GEMMs with fused epilogues ------------------------------------------------------------------------------------

struct GemmOperands {
    int M, N, K, code, la, lb;
    const float *bias = nullptr, *biasmax = nullptr;
};

// A [M,K] contiguous; B [N,K] (layout JF_B_NK) or [K,N] (JF_B_KN) contiguous; scale operands [K/32, rows/32], contiguous or
// the .t() view of the block tensor's own scales; bias [N] / biasmax [1] float32 or None
GemmOperands gemm_operands(const Tensor &A, const Tensor &B, const Tensor &sa, const Tensor &sb, int64_t layout, const OptTensor &bias,
                           const OptTensor &biasmax)
{
    TORCH_CHECK(layout == JF_B_NK || layout == JF_B_KN, "b_layout must be B_NK (0) or B_KN (1)");
    need(A, "A", 2); need(B, "B", 2);
    TORCH_CHECK(A.scalar_type() == torch::kInt8 && B.scalar_type() == torch::kInt8, "A and B must be int8");
    TORCH_CHECK(B.device() == A.device(), "A and B are on different devices");
    GemmOperands g;
    const int64_t M = A.size(0), K = A.size(1), N = layout == JF_B_NK ? B.size(0) : B.size(1);
    TORCH_CHECK((layout == JF_B_NK ? B.size(1) : B.size(0)) == K, "inner dimensions differ: A is ", A.sizes(), ", B is ", B.sizes());
    check_dims(M, N, K);
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.code = check_scales(sa, sb, A, M, N, K, g.la, g.lb);
    TORCH_CHECK(bias.has_value() == biasmax.has_value(), "bias and biasmax come together");
    if (bias) {
        TORCH_CHECK(bias->is_cuda() && bias->device() == A.device() && bias->scalar_type() == torch::kFloat32 && bias->is_contiguous() &&
                        bias->numel() == N, "bias must be a contiguous float32 GPU tensor of N elements");
        TORCH_CHECK(biasmax->is_cuda() && biasmax->device() == A.device() && biasmax->scalar_type() == torch::kFloat32 &&
                        biasmax->numel() >= 1, "biasmax must be a float32 GPU tensor with one element");
        g.bias = bias->data_ptr<float>();
        g.biasmax = biasmax->data_ptr<float>();
    }
    return g;
}

// linear_fwd.py:23 followed by gelu_fwd.py:128-162 (qmodel.py:210-214), one kernel
std::tuple<Tensor, Tensor, Tensor, Tensor> igemm_block_q_gelu(const Tensor &A, const Tensor &B, const Tensor &sa, const Tensor &sb,
                                                              int64_t approx, double amax_eps, const OptTensor &bias,
                                                              const OptTensor &biasmax)
{
    const GemmOperands g = gemm_operands(A, B, sa, sb, JF_B_NK, bias, biasmax);
    check_approx(approx);
    c10::DeviceGuard guard(A.device());
    Tensor q = torch::empty({g.M, g.N}, A.options());
    Tensor s = torch::empty({g.M / QB, g.N / QB}, sa.options().memory_format(c10::MemoryFormat::Contiguous));
    Tensor qg = torch::empty_like(q), sg = torch::empty_like(s);
    pybind11::gil_scoped_release nogil;
    check_rc(jf_igemm_block_q_gelu((const int8_t *)A.data_ptr(), (const int8_t *)B.data_ptr(), sa.data_ptr(), sb.data_ptr(), g.bias,
                                   g.biasmax, (int8_t *)q.data_ptr(), s.data_ptr(), (int8_t *)qg.data_ptr(), sg.data_ptr(), g.M, g.N, g.K,
                                   g.code, g.la, g.lb, (int)approx, (float)amax_eps, current_stream(A)),
             "igemm_block_q_gelu");
    return std::make_tuple(q, s, qg, sg);
}

// linear_bwd.py:17 followed by gelu_bwd.py:173-215 (qmodel.py:249-253), one kernel; the two draw their noise in that order
std::tuple<Tensor, Tensor> igemm_block_q_gelu_bwd(const Tensor &A, const Tensor &B, const Tensor &sa, const Tensor &sb, const Tensor &xq,
                                                  const Tensor &xs, int64_t approx, int64_t gelu_rounding, OptU64 seed, OptU64 offset,
                                                  OptU64 gelu_seed, OptU64 gelu_offset)
{
    const GemmOperands g = gemm_operands(A, B, sa, sb, JF_B_KN, c10::nullopt, c10::nullopt);
    int64_t R2, C2;
    TORCH_CHECK(block_tensor(xq, xs, "x", R2, C2) == g.code && R2 == g.M && C2 == g.N && xq.device() == A.device(),
                "x must be an [M,N] block tensor with the scale dtype of sa / sb");
    check_approx(approx);
    check_rounding(gelu_rounding, false);
    c10::DeviceGuard guard(A.device());
    const auto so = rng(JF_ROUND_STOCHASTIC, A, (int64_t)g.M * g.N, seed, offset);
    const auto go = rng(gelu_rounding, A, (int64_t)g.M * g.N, gelu_seed, gelu_offset);
    Tensor out = torch::empty({g.M, g.N}, A.options());
    Tensor sc = torch::empty({g.M / QB, g.N / QB}, sa.options().memory_format(c10::MemoryFormat::Contiguous));
    pybind11::gil_scoped_release nogil;
    check_rc(jf_igemm_block_q_gelu_bwd((const int8_t *)A.data_ptr(), (const int8_t *)B.data_ptr(), sa.data_ptr(), sb.data_ptr(),
                                       (const int8_t *)xq.data_ptr(), xs.data_ptr(), (int8_t *)out.data_ptr(), sc.data_ptr(), g.M, g.N, g.K,
                                       g.code, g.la, g.lb, (int)approx, so.first, so.second, (int)gelu_rounding, go.first, go.second,
                                       current_stream(A)),
             "igemm_block_q_gelu_bwd");
    return std::make_tuple(out, sc);
}

// linear_fwd.py:22-32 / linear_bwd.py:17-29 with output_quantized / dgrad_quantize = False, one kernel
Tensor igemm_block_q_dequant(const Tensor &A, const Tensor &B, const Tensor &sa, const Tensor &sb, int64_t layout,
                             c10::optional<torch::ScalarType> out_dtype, const OptTensor &bias, const OptTensor &biasmax, int64_t rounding,
                             OptU64 seed, OptU64 offset)
{
    const GemmOperands g = gemm_operands(A, B, sa, sb, layout, bias, biasmax);
    const torch::ScalarType odt = out_dtype.value_or(sa.scalar_type());
    const int oc = fp_code(odt, "out_dtype");
    check_rounding(rounding, false);
    c10::DeviceGuard guard(A.device());
    const auto so = rng(rounding, A, (int64_t)g.M * g.N, seed, offset);
    Tensor out = torch::empty({g.M, g.N}, A.options().dtype(odt));
    pybind11::gil_scoped_release nogil;
    check_rc(jf_igemm_block_q_dequant((const int8_t *)A.data_ptr(), (const int8_t *)B.data_ptr(), sa.data_ptr(), sb.data_ptr(), g.bias,
                                      g.biasmax, out.data_ptr(), g.M, g.N, g.K, (int)layout, g.code, g.la, g.lb, oc, (int)rounding,
                                      so.first, so.second, current_stream(A)),
             "igemm_block_q_dequant");
    return out;
}

// the requantising GEMM with every option of the C ABI (the reference's four variants fix them: bqc_ext.cpp)
std::tuple<Tensor, Tensor> igemm_block_q(const Tensor &A, const Tensor &B, const Tensor &sa, const Tensor &sb, int64_t layout,
                                         const OptTensor &bias, const OptTensor &biasmax, int64_t rounding, OptU64 seed, OptU64 offset)
{
    const GemmOperands g = gemm_operands(A, B, sa, sb, layout, bias, biasmax);
    check_rounding(rounding, false);
    c10::DeviceGuard guard(A.device());
    const auto so = rng(rounding, A, (int64_t)g.M * g.N, seed, offset);
    Tensor out = torch::empty({g.M, g.N}, A.options());
    Tensor sc = torch::empty({g.M / QB, g.N / QB}, sa.options().memory_format(c10::MemoryFormat::Contiguous));
    pybind11::gil_scoped_release nogil;
    check_rc(jf_igemm_block_q((const int8_t *)A.data_ptr(), (const int8_t *)B.data_ptr(), sa.data_ptr(), sb.data_ptr(), g.bias, g.biasmax,
                              (int8_t *)out.data_ptr(), sc.data_ptr(), g.M, g.N, g.K, (int)layout, g.code, g.la, g.lb, (int)rounding,
                              so.first, so.second, nullptr, 0, current_stream(A)),
             "igemm_block_q");
    return std::make_tuple(out, sc);
}

}  // namespace

void register_jetfire_ops(pybind11::module &m)
{
    namespace py = pybind11;
    const py::object none = py::none();
    m.attr("ROUND_NEAREST") = JF_ROUND_NEAREST;
    m.attr("ROUND_STOCHASTIC") = JF_ROUND_STOCHASTIC;
    m.attr("ROUND_TRUNC") = JF_ROUND_TRUNC;
    m.attr("ROUND_STOCHASTIC_TRUNC") = JF_ROUND_STOCHASTIC_TRUNC;
    m.attr("GELU_ERF") = JF_GELU_ERF;
    m.attr("GELU_TANH") = JF_GELU_TANH;
    m.attr("B_NK") = JF_B_NK;
    m.attr("B_KN") = JF_B_KN;
    m.def("quantize", &quantize, py::arg("x"), py::arg("rounding") = JF_ROUND_NEAREST, py::arg("scale_dtype") = none,
          py::arg("transpose") = false, py::arg("amax_eps") = 0.0, py::arg("seed") = none, py::arg("offset") = none,
          "(codes, scales, transposed codes or None) of a float [R,C] tensor");
    m.def("quantize_slabs", &quantize_slabs, py::arg("slabs"), py::arg("rounding") = JF_ROUND_NEAREST,
          py::arg("scale_dtype") = none, py::arg("amax_eps") = 0.0, py::arg("seed") = none, py::arg("offset") = none,
          "block tensor of the column-wise concatenation of up to 4 slabs, read where they lie");
    m.def("dequantize", &dequantize, py::arg("q"), py::arg("s"), py::arg("out_dtype") = none);
    m.def("transpose_s8", &transpose_s8, py::arg("q"));
    m.def("rowstats", &rowstats, py::arg("q"), py::arg("s"), py::arg("eps") = 1e-5);
    m.def("layernorm_fwd", &layernorm_fwd, py::arg("q"), py::arg("s"), py::arg("gamma"), py::arg("beta"), py::arg("mean"), py::arg("rstd"));
    m.def("layernorm_bwd", &layernorm_bwd, py::arg("qx"), py::arg("sx"), py::arg("qg"), py::arg("sg"), py::arg("gamma"), py::arg("mean"),
          py::arg("rstd"), py::arg("rounding") = JF_ROUND_NEAREST, py::arg("want_dbeta") = true, py::arg("seed") = none,
          py::arg("offset") = none);
    m.def("layernorm_bwd_add", &layernorm_bwd_add, py::arg("qx"), py::arg("sx"), py::arg("qg"), py::arg("sg"), py::arg("gamma"),
          py::arg("mean"), py::arg("rstd"), py::arg("x1"), py::arg("rounding") = JF_ROUND_NEAREST, py::arg("add_rounding") = JF_ROUND_TRUNC,
          py::arg("want_dbeta") = true, py::arg("out_dtype") = none, py::arg("seed") = none, py::arg("offset") = none,
          py::arg("add_seed") = none, py::arg("add_offset") = none);
    m.def("gelu_fwd", &gelu_fwd, py::arg("q"), py::arg("s"), py::arg("approx") = JF_GELU_ERF, py::arg("amax_eps") = 5e-5);
    m.def("gelu_bwd", &gelu_bwd, py::arg("qx"), py::arg("sx"), py::arg("qg"), py::arg("sg"), py::arg("approx") = JF_GELU_ERF,
          py::arg("rounding") = JF_ROUND_NEAREST, py::arg("seed") = none, py::arg("offset") = none);
    m.def("add", &add, py::arg("x1"), py::arg("q2"), py::arg("s2"), py::arg("rounding") = JF_ROUND_TRUNC, py::arg("with_stats") = false,
          py::arg("out_dtype") = none, py::arg("seed") = none, py::arg("offset") = none,
          "(y1, codes, scales, mean or None, rstd or None)");
    m.def("block_colsum", &block_colsum, py::arg("q"), py::arg("s"), "fp32 column sums of a block tensor (bias gradient)");
    m.def("igemm_block_q", &igemm_block_q, py::arg("A"), py::arg("B"), py::arg("sa"), py::arg("sb"), py::arg("b_layout") = JF_B_KN,
          py::arg("bias") = none, py::arg("biasmax") = none, py::arg("rounding") = JF_ROUND_NEAREST, py::arg("seed") = none,
          py::arg("offset") = none);
    m.def("igemm_block_q_gelu", &igemm_block_q_gelu, py::arg("A"), py::arg("B"), py::arg("sa"), py::arg("sb"),
          py::arg("approx") = JF_GELU_ERF, py::arg("amax_eps") = 5e-5, py::arg("bias") = none, py::arg("biasmax") = none);
    m.def("igemm_block_q_gelu_bwd", &igemm_block_q_gelu_bwd, py::arg("A"), py::arg("B"), py::arg("sa"), py::arg("sb"), py::arg("xq"),
          py::arg("xs"), py::arg("approx") = JF_GELU_ERF, py::arg("gelu_rounding") = JF_ROUND_STOCHASTIC, py::arg("seed") = none,
          py::arg("offset") = none, py::arg("gelu_seed") = none, py::arg("gelu_offset") = none);
    m.def("igemm_block_q_dequant", &igemm_block_q_dequant, py::arg("A"), py::arg("B"), py::arg("sa"), py::arg("sb"),
          py::arg("b_layout") = JF_B_KN, py::arg("out_dtype") = none, py::arg("bias") = none, py::arg("biasmax") = none,
          py::arg("rounding") = JF_ROUND_NEAREST, py::arg("seed") = none, py::arg("offset") = none);
}

}  // namespace jfext
