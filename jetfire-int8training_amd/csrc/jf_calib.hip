// Calibration kernels for the roofline discussion: what the matrix pipe and the vector ALU of this part deliver,
// alone and together, from registers (no memory traffic).  They have no counterpart in the reference; bench.py
// uses them to print the measured MFMA peak and the measured cost of the fp32 scale-accumulate next to it.
#include "jf_device.hpp"

namespace jf {

// Per iteration and wave: 4 x ( [one 32x32x32 INT8 MFMA on its own accumulator chain]  +  [NV independent v_fmac_f32] ).
//   WITH_MFMA / NV = (1, 0): matrix pipe alone; (0, 32): vector ALU alone; (1, 32): both, independent of each other.
template <int WITH_MFMA, int NV>
__global__ __launch_bounds__(256) void calib_kernel(int iters, float *out)
{
    v4i a = {(int)threadIdx.x, 1, 2, 3}, b = {4, 5, 6, (int)blockIdx.x};
    v16i c[4];
    for (int i = 0; i < 4; ++i)
        for (int v = 0; v < 16; ++v) c[i][v] = 0;
    float f[32];
    for (int i = 0; i < 32; ++i) f[i] = (float)i;
    const float s = 1.0f + 1e-6f * threadIdx.x, m = 0.5f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (WITH_MFMA) c[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c[i], 0, 0, 0);
#pragma unroll
            for (int v = 0; v < NV; ++v) f[v % 32] = __builtin_fmaf(s, m, f[v % 32]);
        }
    }
    float t = 0.0f;
    for (int i = 0; i < 32; ++i) t += f[i];
    int u = 0;
    for (int i = 0; i < 4; ++i)
        for (int v = 0; v < 16; ++v) u += c[i][v];
    if (t == 1.2345f || u == 123456789) out[0] = t + (float)u;      // never true: keeps the work alive
}

}  // namespace jf

using namespace jf;

extern "C" int jf_calibrate(int with_mfma, int valu_per_mfma, int iters, int workgroups, float *scratch, jf_stream_t stream)
{
    if (!scratch) return JF_ERR_NULL;
    if (iters <= 0 || workgroups <= 0) return JF_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
#define JF_CAL(M, NV)                                                                               \
    if (with_mfma == M && valu_per_mfma == NV) {                                                    \
        hipLaunchKernelGGL((calib_kernel<M, NV>), dim3(workgroups), dim3(256), 0, st, iters, scratch); \
        return (int)hipGetLastError();                                                              \
    }
    JF_CAL(1, 0) JF_CAL(0, 32) JF_CAL(1, 32) JF_CAL(0, 16) JF_CAL(1, 16)
#undef JF_CAL
    return JF_ERR_ENUM;
}
