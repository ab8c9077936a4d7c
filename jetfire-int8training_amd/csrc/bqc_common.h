// Helpers shared by the two halves of the BlockQuantizeCUDA extension (bqc_ext.cpp: the reference's eight GEMM entry
// points; jf_ops_ext.cpp: every other operator of the path): tensor checks, the current stream, and the one source of
// Philox (seed, offset) pairs for everything that rounds stochastically.  Host C++ only.
#pragma once

#include <torch/extension.h>

#include <ATen/detail/CUDAHooksInterface.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <mutex>
#include <tuple>

#include "../../include/jetfire_hip.h"

namespace jfext {


constexpr int QB = 32;

inline void check_rc(int rc, const char *what)
{
    TORCH_CHECK(rc == 0, what, ": ", jf_error_string(rc));
}

inline int scale_code(const torch::Tensor &s, const char *name)
{
    if (s.scalar_type() == torch::kFloat16) return JF_SCALE_F16;
    if (s.scalar_type() == torch::kFloat32) return JF_SCALE_F32;
    TORCH_CHECK(false, name, ": scales must be float16 or float32, got ", s.scalar_type());
    return -1;
}

inline void check_dims(int64_t M, int64_t N, int64_t K)
{
    TORCH_CHECK(M > 0 && N > 0 && K > 0 && M % QB == 0 && N % QB == 0 && K % QB == 0,
                "M, N, K must be positive multiples of 32, got ", M, ", ", N, ", ", K);
}

inline void check_a(const torch::Tensor &X, int64_t M, int64_t K)
{
    TORCH_CHECK(X.is_cuda(), "X must be a GPU tensor");
    TORCH_CHECK(X.scalar_type() == torch::kInt8, "X must be int8, got ", X.scalar_type());
    TORCH_CHECK(X.dim() == 2 && X.size(0) == M && X.size(1) == K, "X must be [M,K] = [", M, ",", K, "], got ", X.sizes());
    TORCH_CHECK(X.is_contiguous(), "X must be contiguous");
}

// A of the weight-gradient GEMM: [M,K] contiguous (the reference's pre-transposed gradient G8T), or the .t() view
// of a contiguous [K,M] tensor (strides (1,M)), i.e. the gradient [tokens, C_out] as it lies in memory: JF_A_KM.
inline int check_a_any_layout(const torch::Tensor &X, int64_t M, int64_t K)
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
inline void check_b_kn(const torch::Tensor &W, const torch::Tensor &X, int64_t K, int64_t N)
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
inline void check_b_nk(const torch::Tensor &W, const torch::Tensor &X, int64_t K, int64_t N)
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
inline int scale_layout(const torch::Tensor &S, int64_t K, int64_t rows, const char *name)
{
    TORCH_CHECK(S.dim() == 2 && S.size(0) == K / QB && S.size(1) == rows / QB, name, " must be [K/32,rows/32] = [", K / QB,
                ",", rows / QB, "], got ", S.sizes());
    if (S.is_contiguous()) return JF_SCALES_KMAJOR;
    TORCH_CHECK(S.stride(0) == 1 && S.stride(1) == K / QB, name,
                " must be contiguous or the .t() view of a contiguous [rows/32,K/32] tensor, got strides ", S.strides());
    return JF_SCALES_ROWMAJOR;
}

inline int check_scales(const torch::Tensor &SX, const torch::Tensor &SW, const torch::Tensor &X, int64_t M, int64_t N, int64_t K,
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

inline jf_stream_t current_stream(const torch::Tensor &t)
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
inline at::Generator default_generator(int device_index)
{
    return at::detail::getCUDAHooks().getDefaultGenerator(device_index);
}

inline uint64_t reserve_calls(int64_t numel)
{
    const uint64_t calls = (uint64_t)(numel + 7) / 8;
    return (calls + 3) / 4 * 4;                                // the generator keeps its offset a multiple of 4
}

inline std::pair<uint64_t, uint64_t> next_philox(const torch::Tensor &t, int64_t numel)
{
    at::Generator gen = default_generator(t.device().index());
    std::lock_guard<std::mutex> g(gen.mutex());
    const uint64_t seed = gen.current_seed(), off = gen.get_offset();
    gen.set_offset(off + reserve_calls(numel));
    return {seed, off};
}

// For reproducible tests: the (seed, offset) the next stochastic call on `device_index` will use, and a way
// to place the offset (a multiple of 4).
inline std::tuple<uint64_t, uint64_t> philox_peek(int device_index)
{
    at::Generator gen = default_generator(device_index);
    std::lock_guard<std::mutex> g(gen.mutex());
    return std::make_tuple(gen.current_seed(), gen.get_offset());
}

inline void philox_set_offset(int device_index, uint64_t offset)
{
    TORCH_CHECK(offset % 4 == 0, "the Philox offset must be a multiple of 4, got ", offset);
    at::Generator gen = default_generator(device_index);
    std::lock_guard<std::mutex> g(gen.mutex());
    gen.set_offset(offset);
}

}  // namespace jfext
