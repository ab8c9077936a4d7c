// BlockQuantizeCUDA -- the PyTorch extension of the Jetfire per-block INT8 GEMMs for MI355X.
//
// Same module name and the same eight positional signatures as the reference extension
// (JetfireGEMMKernel/BlockQuantize/cpp_extension/bindings.cpp:6-35, include/igemm.h), so
// Jetfire/Linear/linear_fwd.py:23 and linear_bwd.py:17,19 call it unchanged.  This file is host C++
// only: it validates tensors (the reference checks nothing), allocates outputs, finds the current
// stream and the Philox (seed, offset), and calls the gfx950 kernels through the C ABI of
// include/jetfire_hip.h.
#include <torch/extension.h>

#include <ATen/detail/CUDAHooksInterface.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <mutex>
#include <tuple>

#include "../../include/jetfire_hip.h"

namespace {

constexpr int QB = 32;

void check_rc(int rc, const char *what)
{
    TORCH_CHECK(rc == 0, what, ": ", jf_error_string(rc));
}

int scale_code(const torch::Tensor &s, const char *name)
{
    if (s.scalar_type() == torch::kFloat16) return JF_SCALE_F16;
    if (s.scalar_type() == torch::kFloat32) return JF_SCALE_F32;
    TORCH_CHECK(false, name, ": scales must be float16 or float32, got ", s.scalar_type());
    return -1;
}

void check_dims(int64_t M, int64_t N, int64_t K)
{
    TORCH_CHECK(M > 0 && N > 0 && K > 0 && M % QB == 0 && N % QB == 0 && K % QB == 0,
                "M, N, K must be positive multiples of 32, got ", M, ", ", N, ", ", K);
}

void check_a(const torch::Tensor &X, int64_t M, int64_t K)
{
    TORCH_CHECK(X.is_cuda(), "X must be a GPU tensor");
    TORCH_CHECK(X.scalar_type() == torch::kInt8, "X must be int8, got ", X.scalar_type());
    TORCH_CHECK(X.dim() == 2 && X.size(0) == M && X.size(1) == K, "X must be [M,K] = [", M, ",", K, "], got ", X.sizes());
    TORCH_CHECK(X.is_contiguous(), "X must be contiguous");
}

// A of the weight-gradient GEMM: [M,K] contiguous (the reference's pre-transposed gradient G8T), or the .t() view
// of a contiguous [K,M] tensor (strides (1,M)), i.e. the gradient [tokens, C_out] as it lies in memory: JF_A_KM.
int check_a_any_layout(const torch::Tensor &X, int64_t M, int64_t K)
{
    TORCH_CHECK(X.is_cuda(), "X must be a GPU tensor");
    TORCH_CHECK(X.scalar_type() == torch::kInt8, "X must be int8, got ", X.scalar_type());
    TORCH_CHECK(X.dim() == 2 && X.size(0) == M && X.size(1) == K, "X must be [M,K] = [", M, ",", K, "], got ", X.sizes());
    if (X.is_contiguous()) return JF_A_MK;
    TORCH_CHECK(X.stride(0) == 1 && X.stride(1) == M,
                "X must be contiguous or the .t() view of a contiguous [K,M] tensor, got strides ", X.strides());
    return JF_A_KM;
}

// B as [K,N] row-major ("row x row" functions).
void check_b_kn(const torch::Tensor &W, const torch::Tensor &X, int64_t K, int64_t N)
{
    TORCH_CHECK(W.is_cuda() && W.device() == X.device(), "W must be on the same GPU as X");
    TORCH_CHECK(W.scalar_type() == torch::kInt8, "W must be int8, got ", W.scalar_type());
    TORCH_CHECK(W.dim() == 2 && W.size(0) == K && W.size(1) == N, "W must be [K,N] = [", K, ",", N, "], got ", W.sizes());
    TORCH_CHECK(W.is_contiguous(), "W must be contiguous");
}

// B for the "row x col" function: the caller passes W8.t(), a (K,N) view with strides (1,K) of a contiguous
// [N,K] tensor (Jetfire/Linear/linear_fwd.py:23); the kernel reads the underlying [N,K] storage.  A
// contiguous 2-D tensor of N*K elements is read as [N,K] as well (the reference ignores strides,
// …BiasRowCol.cu:422).
void check_b_nk(const torch::Tensor &W, const torch::Tensor &X, int64_t K, int64_t N)
{
    TORCH_CHECK(W.is_cuda() && W.device() == X.device(), "W must be on the same GPU as X");
    TORCH_CHECK(W.scalar_type() == torch::kInt8, "W must be int8, got ", W.scalar_type());
    TORCH_CHECK(W.dim() == 2 && W.numel() == K * N, "W must have K*N = ", K * N, " elements, got ", W.sizes());
    const bool t_view = W.size(0) == K && W.size(1) == N && W.stride(0) == 1 && W.stride(1) == K;
    TORCH_CHECK(t_view || W.is_contiguous(),
                "W must be the .t() view of a contiguous [N,K] tensor (strides (1,K)) or a contiguous [N,K] tensor; got sizes ",
                W.sizes(), " strides ", W.strides());
}

// A GEMM scale operand is [K/32, rows/32]: either contiguous (what the reference kernels need, JF_SCALES_KMAJOR) or the
// .t() view of a contiguous [rows/32, K/32] tensor, i.e. the block tensor's own scale array without the transposed
// copy (JF_SCALES_ROWMAJOR; strides (1, K/32)).
int scale_layout(const torch::Tensor &S, int64_t K, int64_t rows, const char *name)
{
    TORCH_CHECK(S.dim() == 2 && S.size(0) == K / QB && S.size(1) == rows / QB, name, " must be [K/32,rows/32] = [", K / QB,
                ",", rows / QB, "], got ", S.sizes());
    if (S.is_contiguous()) return JF_SCALES_KMAJOR;
    TORCH_CHECK(S.stride(0) == 1 && S.stride(1) == K / QB, name,
                " must be contiguous or the .t() view of a contiguous [rows/32,K/32] tensor, got strides ", S.strides());
    return JF_SCALES_ROWMAJOR;
}

int check_scales(const torch::Tensor &SX, const torch::Tensor &SW, const torch::Tensor &X, int64_t M, int64_t N, int64_t K,
                 int &sx_layout, int &sw_layout)
{
    const int code = scale_code(SX, "SX");
    TORCH_CHECK(SW.scalar_type() == SX.scalar_type(), "SX and SW must have the same dtype");
    TORCH_CHECK(SX.is_cuda() && SW.is_cuda() && SX.device() == X.device() && SW.device() == X.device(),
                "scales must be on the same GPU as X");
    sx_layout = scale_layout(SX, K, M, "SX");
    sw_layout = scale_layout(SW, K, N, "SW");
    return code;
}

jf_stream_t current_stream(const torch::Tensor &t)
{
    return (jf_stream_t)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

struct Workspace {
    torch::Tensor t;
    void *ptr = nullptr;
    size_t bytes = 0;
    Workspace(const torch::Tensor &like, int M, int N, int K, int layout) : Workspace(like, jf_igemm_workspace_bytes(M, N, K, layout)) {}
    Workspace(const torch::Tensor &like, size_t nbytes)
    {
        bytes = nbytes;
        if (bytes) {
            t = torch::empty({(int64_t)bytes}, like.options().dtype(torch::kInt8));
            ptr = t.data_ptr();
        }
    }
};

// (seed, offset) of the next stochastic kernel.  There is ONE source of Philox counters per device for everything in
// this library that rounds stochastically (these GEMMs and the Nonlinear operators, which reach it from Python): the
// device's default torch generator.  An op reserves the counters it may consume (one per 8 output elements) by advancing
// the generator's offset under the generator's mutex, so consecutive ops draw from disjoint ranges, torch.manual_seed
// (also with the seed it already has) rewinds everything, and torch's own random kernels never see a counter twice.
// The generator refuses this during stream capture: a captured graph would replay the same noise, so code that is
// captured passes explicit (seed, offset) through the C ABI instead.  (Reference: rand(), ...Stochastic.cu:416.)
at::Generator default_generator(int device_index)
{
    return at::detail::getCUDAHooks().getDefaultGenerator(device_index);
}

uint64_t reserve_calls(int64_t numel)
{
    const uint64_t calls = (uint64_t)(numel + 7) / 8;
    return (calls + 3) / 4 * 4;                                // the generator keeps its offset a multiple of 4
}

std::pair<uint64_t, uint64_t> next_philox(const torch::Tensor &t, int64_t numel)
{
    at::Generator gen = default_generator(t.device().index());
    std::lock_guard<std::mutex> g(gen.mutex());
    const uint64_t seed = gen.current_seed(), off = gen.get_offset();
    gen.set_offset(off + reserve_calls(numel));
    return {seed, off};
}

// For reproducible tests: the (seed, offset) the next stochastic call on `device_index` will use, and a way
// to place the offset (a multiple of 4).
std::tuple<uint64_t, uint64_t> philox_peek(int device_index)
{
    at::Generator gen = default_generator(device_index);
    std::lock_guard<std::mutex> g(gen.mutex());
    return std::make_tuple(gen.current_seed(), gen.get_offset());
}

void philox_set_offset(int device_index, uint64_t offset)
{
    TORCH_CHECK(offset % 4 == 0, "the Philox offset must be a multiple of 4, got ", offset);
    at::Generator gen = default_generator(device_index);
    std::lock_guard<std::mutex> g(gen.mutex());
    gen.set_offset(offset);
}

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
}
