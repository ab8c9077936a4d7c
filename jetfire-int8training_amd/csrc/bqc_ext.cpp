// BlockQuantizeCUDA -- the PyTorch extension of the Jetfire per-block INT8 GEMMs for MI355X.
//
// Same module name and the same eight positional signatures as the reference extension
// (JetfireGEMMKernel/BlockQuantize/cpp_extension/bindings.cpp:6-35, include/igemm.h), so
// Jetfire/Linear/linear_fwd.py:23 and linear_bwd.py:17,19 call it unchanged.  This file is host C++
// only: it validates tensors (the reference checks nothing), allocates outputs, finds the current
// stream and the Philox (seed, offset), and calls the gfx950 kernels through the C ABI of
// include/jetfire_hip.h.
#include "bqc_common.h"

using namespace jfext;

namespace jfext { void register_jetfire_ops(pybind11::module &m); }     // jf_ops_ext.cpp

namespace {

std::tuple<torch::Tensor, torch::Tensor> block_q(const torch::Tensor &X, const torch::Tensor &W, const torch::Tensor *bias,
                                                 const torch::Tensor *biasmax, const torch::Tensor &SX,
                                                 const torch::Tensor &SW, int M, int N, int K, int layout, int rounding)
{
    check_dims(M, N, K);
    check_a(X, M, K);
    if (layout == JF_B_NK) check_b_nk(W, X, K, N); else check_b_kn(W, X, K, N);
    int sxl, swl;
    const int code = check_scales(SX, SW, X, M, N, K, sxl, swl);
    const float *bias_p = nullptr, *biasmax_p = nullptr;
    if (bias) {
        TORCH_CHECK(bias->is_cuda() && bias->device() == X.device() && bias->scalar_type() == torch::kFloat32 &&
                        bias->is_contiguous() && bias->numel() == N, "bias must be a contiguous float32 GPU tensor of N elements");
        TORCH_CHECK(biasmax && biasmax->is_cuda() && biasmax->device() == X.device() &&
                        biasmax->scalar_type() == torch::kFloat32 && biasmax->numel() >= 1,
                    "biasmax must be a float32 GPU tensor with one element");
        bias_p = bias->data_ptr<float>();
        biasmax_p = biasmax->data_ptr<float>();
    }
    c10::DeviceGuard guard(X.device());
    torch::Tensor O = torch::empty({M, N}, X.options().dtype(torch::kInt8));
    torch::Tensor SO = torch::empty({M / QB, N / QB}, SX.options().memory_format(c10::MemoryFormat::Contiguous));
    Workspace ws(X, M, N, K, layout);
    uint64_t seed = 0, offset = 0;
    if (rounding == JF_ROUND_STOCHASTIC) std::tie(seed, offset) = next_philox(X, (int64_t)M * N);
    {
        pybind11::gil_scoped_release nogil;
        check_rc(jf_igemm_block_q((const int8_t *)X.data_ptr(), (const int8_t *)W.data_ptr(), SX.data_ptr(), SW.data_ptr(),
                                  bias_p, biasmax_p, (int8_t *)O.data_ptr(), SO.data_ptr(), M, N, K, layout, code, sxl, swl, rounding,
                                  seed, offset, ws.ptr, ws.bytes, current_stream(X)),
                 "igemm_block_q");
    }
    return std::make_tuple(O, SO);
}

}  // namespace

// ---- the eight entry points of bindings.cpp ---------------------------------------------------------

// include/igemm.h:3-12
torch::Tensor igemm_basic_int8_gemm(torch::Tensor X, torch::Tensor W, const int M, const int N, const int K)
{
    check_dims(M, N, K);
    check_a(X, M, K);
    check_b_kn(W, X, K, N);
    c10::DeviceGuard guard(X.device());
    torch::Tensor O = torch::empty({M, N}, X.options().dtype(torch::kInt32));
    Workspace ws(X, M, N, K, JF_B_KN);
    pybind11::gil_scoped_release nogil;
    check_rc(jf_igemm_s32((const int8_t *)X.data_ptr(), (const int8_t *)W.data_ptr(), (int32_t *)O.data_ptr(), M, N, K,
                          JF_B_KN, ws.ptr, ws.bytes, current_stream(X)),
             "igemm_basic_int8_gemm");
    return O;
}

// include/igemm.h:14-25 : fp16 output, B [K,N]
// splitk (not in the reference's signature; default 1 = its arithmetic): see jf_igemm_block_fp.
// out_dtype (not in the reference's signature either; default float16 = its output): float32 or bfloat16 spare the caller a
// conversion kernel when the weight gradient is accumulated in another type.
torch::Tensor igemm_output_fp_no_quantize(torch::Tensor X, torch::Tensor W, torch::Tensor SX, torch::Tensor SW,
                                          const int M, const int N, const int K, const int splitk,
                                          c10::optional<torch::ScalarType> out_dtype)
{
    const torch::ScalarType odt = out_dtype.value_or(torch::kFloat16);
    TORCH_CHECK(odt == torch::kFloat16 || odt == torch::kFloat32 || odt == torch::kBFloat16,
                "out_dtype must be float16, float32 or bfloat16");
    const int ocode = odt == torch::kFloat16 ? JF_FP_F16 : odt == torch::kFloat32 ? JF_FP_F32 : JF_FP_BF16;
    check_dims(M, N, K);
    const int a_layout = check_a_any_layout(X, M, K);
    check_b_kn(W, X, K, N);
    int sxl, swl;
    const int code = check_scales(SX, SW, X, M, N, K, sxl, swl);
    c10::DeviceGuard guard(X.device());
    torch::Tensor O = torch::empty({M, N}, X.options().dtype(odt));
    TORCH_CHECK(splitk >= 0, "splitk must be >= 0");
    Workspace ws(X, jf_igemm_block_fp_workspace_bytes(M, N, K, JF_B_KN, splitk));
    pybind11::gil_scoped_release nogil;
    check_rc(jf_igemm_block_fp((const int8_t *)X.data_ptr(), (const int8_t *)W.data_ptr(), SX.data_ptr(), SW.data_ptr(),
                               O.data_ptr(), M, N, K, a_layout, JF_B_KN, code, sxl, swl, ocode, splitk, ws.ptr, ws.bytes,
                               current_stream(X)),
             "igemm_output_fp_no_quantize");
    return O;
}

// include/igemm.h:40-51 : deterministic requantised output, B [K,N]
std::tuple<torch::Tensor, torch::Tensor> igemm_output_int_quantize(torch::Tensor X, torch::Tensor W, torch::Tensor SX,
                                                                   torch::Tensor SW, const int M, const int N, const int K)
{
    return block_q(X, W, nullptr, nullptr, SX, SW, M, N, K, JF_B_KN, JF_ROUND_NEAREST);
}

// include/igemm.h:79-90 : stochastic-rounding requantised output, B [K,N]
std::tuple<torch::Tensor, torch::Tensor> igemm_output_int_quantize_stochastic(torch::Tensor X, torch::Tensor W,
                                                                              torch::Tensor SX, torch::Tensor SW,
                                                                              const int M, const int N, const int K)
{
    return block_q(X, W, nullptr, nullptr, SX, SW, M, N, K, JF_B_KN, JF_ROUND_STOCHASTIC);
}

// include/igemm.h:53-64 : bias variant, B [K,N]
std::tuple<torch::Tensor, torch::Tensor> igemm_output_int_quantize_bias_rowrow(torch::Tensor X, torch::Tensor W,
                                                                               torch::Tensor bias, torch::Tensor biasmax,
                                                                               torch::Tensor SX, torch::Tensor SW,
                                                                               const int M, const int N, const int K)
{
    return block_q(X, W, &bias, &biasmax, SX, SW, M, N, K, JF_B_KN, JF_ROUND_NEAREST);
}

// include/igemm.h:66-77 : the forward kernel, B given as the .t() view of [N,K]
std::tuple<torch::Tensor, torch::Tensor> igemm_output_int_quantize_bias_rowcol(torch::Tensor X, torch::Tensor W,
                                                                               torch::Tensor bias, torch::Tensor biasmax,
                                                                               torch::Tensor SX, torch::Tensor SW,
                                                                               const int M, const int N, const int K)
{
    return block_q(X, W, &bias, &biasmax, SX, SW, M, N, K, JF_B_NK, JF_ROUND_NEAREST);
}

// include/igemm.h:27-38 : the reference marks this one "useless" (bindings.cpp:23-26): older tiling, truncating
// quantiser, int32 codes and a different scale layout.  Not part of the data-flow path; exported so that the
// module surface is complete, and it says so when called.
std::tuple<torch::Tensor, torch::Tensor> igemm_output_int_quantize_fused(torch::Tensor, torch::Tensor, torch::Tensor,
                                                                         torch::Tensor, const int, const int, const int)
{
    TORCH_CHECK(false, "igemm_output_int_quantize_fused is not implemented: the reference declares it unused "
                       "(bindings.cpp:23-26); use igemm_output_int_quantize");
    return {};
}

// include/hgemm.h : fp16 comparison GEMM of the reference's benchmarks; a library GEMM here.
torch::Tensor hgemm_v1(torch::Tensor X, torch::Tensor W, const int M, const int N, const int K)
{
    TORCH_CHECK(X.is_cuda() && W.is_cuda() && X.scalar_type() == torch::kFloat16 && W.scalar_type() == torch::kFloat16,
                "hgemm_v1 expects float16 GPU tensors");
    TORCH_CHECK(X.dim() == 2 && W.dim() == 2 && X.size(0) == M && X.size(1) == K && W.size(0) == K && W.size(1) == N,
                "hgemm_v1: X must be [M,K] and W [K,N]");
    return torch::matmul(X, W);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.doc() = "Jetfire per-block INT8 GEMMs for MI355X (gfx950); drop-in for the reference's BlockQuantizeCUDA";
    m.def("igemm_output_int_quantize_stochastic", &igemm_output_int_quantize_stochastic,
          "dequantize + INT8 MFMA GEMM + stochastic-rounding requantize (fused); B is [K,N]; backward activation gradient");
    m.def("igemm_output_int_quantize_bias_rowcol", &igemm_output_int_quantize_bias_rowcol,
          "dequantize + INT8 MFMA GEMM + requantize (fused); B is the .t() view of [N,K]; forward");
    m.def("igemm_output_int_quantize_bias_rowrow", &igemm_output_int_quantize_bias_rowrow,
          "dequantize + INT8 MFMA GEMM + requantize (fused); B is [K,N]");
    m.def("igemm_output_int_quantize", &igemm_output_int_quantize,
          "dequantize + INT8 MFMA GEMM + round-to-nearest requantize (fused); B is [K,N]");
    m.def("igemm_output_int_quantize_fused", &igemm_output_int_quantize_fused, "not implemented (unused in the reference)");
    m.def("igemm_output_fp_no_quantize", &igemm_output_fp_no_quantize,
          "dequantize + INT8 MFMA GEMM, fp16 output; B is [K,N]; backward weight gradient", pybind11::arg("X"),
          pybind11::arg("W"), pybind11::arg("SX"), pybind11::arg("SW"), pybind11::arg("M"), pybind11::arg("N"),
          pybind11::arg("K"), pybind11::arg("splitk") = 1, pybind11::arg("out_dtype") = pybind11::none());
    m.def("igemm_basic_int8_gemm", &igemm_basic_int8_gemm, "INT8 MFMA GEMM, INT32 output; B is [K,N]");
    m.def("hgemm_v1", &hgemm_v1, "fp16 GEMM (library)");
    // not in the reference: makes the stochastic entry point reproducible from Python
    m.def("philox_peek", &philox_peek, "(seed, offset) the next stochastic call on this device index will use");
    m.def("philox_set_offset", &philox_set_offset, "set the Philox offset used by the next stochastic call");
    // every other operator of the path (Jetfire/Nonlinear, and the GEMMs with fused epilogues Jetfire/Linear uses)
    pybind11::module ops = m.def_submodule("jetfire", "Nonlinear operators and fused-epilogue GEMMs of the INT8 data flow (gfx950)");
    jfext::register_jetfire_ops(ops);
}
