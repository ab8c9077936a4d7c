// Per-block INT8 GEMMs for gfx950 (MI355X).
//
//   acc[m,n] = sum over 32-deep K blocks kb (ascending) of  (sa[kb,m/32]*sb[kb,n/32]) * d_kb[m,n]
//   d_kb     = exact INT32 dot product of the kb-th 32-wide slices of A[m,:] and B[n,:]
//
// One v_mfma_i32_32x32x32_i8 with a zero accumulator input produces d_kb for a whole 32x32 output
// block, i.e. exactly one Jetfire quantisation-block product; the fp32 scale-accumulate is one
// v_cvt_f32_i32 + one v_fma_f32 per value.  (Reference kernels: igemm_BlockSquare32OutputIntQuantize
// BiasRowCol.cu:134-225 and its siblings under JetfireGEMMKernel/BlockQuantize/cpp_extension/igemm/.)
//
// Work decomposition: workgroup = 256 threads = 4 waves (2x2), tile 128x128, each wave owns a
// 64x64 sub-tile = 2x2 quantisation blocks (64 fp32 accumulators per lane).  K is consumed in
// stages of KB_STAGE blocks, double-buffered in LDS.  The LDS image of a 32x32 int8 block is stored
// in MFMA operand order ([k-half][row][16 bytes]) so that every operand fetch is one linear
// ds_read_b128 (lane l reads bytes 16*l .. 16*l+15).  Both operands are K-contiguous ("NT"); a
// [K,N] B operand is transposed into a caller-provided workspace first.
#include "jf_device.hpp"

namespace jf {

constexpr int BM = 128, BN = 128;
constexpr int KB_STAGE = 4;                         // 32-deep K blocks per LDS stage (BK = 128 bytes)
constexpr int NTHREADS = 256;
constexpr int TILE_BYTES = (BM / QB) * KB_STAGE * 1024;          // one operand, one stage
constexpr int STAGE_BYTES = 2 * TILE_BYTES + 2 * KB_STAGE * 4 * (int)sizeof(float);
constexpr int EPI_LD = 36;                          // floats per staged row (32 + pad, keeps 16B alignment)
constexpr int EPI_BYTES = 4 * QB * EPI_LD * (int)sizeof(float);
constexpr int SMEM_BYTES = (2 * STAGE_BYTES > EPI_BYTES) ? 2 * STAGE_BYTES : EPI_BYTES;

enum Epilogue { EPI_S32 = 0, EPI_FP = 1, EPI_Q = 2 };

struct GemmArgs {
    const int8_t *A;      // [M, lda]
    const int8_t *B;      // [N, ldb]   (K-contiguous)
    const void *sa;       // [K/32, M/32]
    const void *sb;       // [K/32, N/32]
    void *C;              // s32 / fp / s8 [M, N]
    void *sc;             // [M/32, N/32]   (EPI_Q)
    const float *bias;    // [N] or null   (EPI_Q)
    const float *biasmax; // [1] or null   (EPI_Q)
    uint64_t seed, offset;
    int M, N, K, lda, ldb;
    int tiles_m, tiles_n;
    int out_dtype;        // JF_FP_*        (EPI_FP)
    int rounding;         // JF_ROUND_*     (EPI_Q)
};

// Logical tile of this workgroup.  Workgroups are dealt round-robin to the 8 XCDs, each with a
// private L2: give every XCD one contiguous run of tiles, and walk tiles in groups of 8 tile-rows so
// that concurrently resident workgroups of an XCD share A and B panels.
__device__ __forceinline__ void tile_of_workgroup(int tiles_m, int tiles_n, int &tm, int &tn)
{
    const int nwg = gridDim.x, wg = blockIdx.x;
    const int xcd = wg & 7, idx = wg >> 3;
    const int per = nwg >> 3, rem = nwg & 7;
    const int logical = xcd * per + (xcd < rem ? xcd : rem) + idx;
    constexpr int GROUP = 8;
    const int group_size = GROUP * tiles_n;
    const int g = logical / group_size;
    const int first_m = g * GROUP;
    const int gm = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    const int in_group = logical - g * group_size;
    tm = first_m + in_group % gm;
    tn = in_group / gm;
}

template <int EPI, typename ST>
__global__ __launch_bounds__(NTHREADS, 2) void igemm_nt_kernel(GemmArgs p)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;

    int tile_m, tile_n;
    tile_of_workgroup(p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int SM = p.M / QB, SN = p.N / QB;
    const int nkb = p.K / QB;
    const int nstages = (nkb + KB_STAGE - 1) / KB_STAGE;

    // ---- global -> register -> LDS staging -------------------------------------------------
    // One operand stage is 128 rows x 8 chunks of 16 bytes; thread t moves chunks t, t+256, ...
    // (8 consecutive lanes cover one 128-byte row segment).
    constexpr int CHUNKS = BM * KB_STAGE * 2 / NTHREADS;      // 4 per operand per thread
    v4i ra[CHUNKS], rb[CHUNKS];
    float rs = 0.0f;                                          // this thread's scale of the stage (tid < 32)

    auto load_stage = [&](int stage) {
        const int kb0 = stage * KB_STAGE;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int id = tid + c * NTHREADS;
            const int row = id >> 3, ch = id & 7;
            const int kb = kb0 + (ch >> 1);
            const int kbc = kb < nkb ? kb : nkb - 1;          // clamp: data of a missing block is never used
            const int koff = kbc * QB + (ch & 1) * 16;
            int ar = m0 + row; ar = ar < p.M ? ar : p.M - 1;  // clamp rows of partial tiles
            int br = n0 + row; br = br < p.N ? br : p.N - 1;
            ra[c] = *reinterpret_cast<const v4i *>(p.A + (size_t)ar * p.lda + koff);
            rb[c] = *reinterpret_cast<const v4i *>(p.B + (size_t)br * p.ldb + koff);
        }
        if (EPI != EPI_S32 && tid < 2 * KB_STAGE * 4) {
            // tid = which*16 + kb*4 + blk : scale of K block kb for tile block blk of A (which=0) / B (1)
            const int which = tid >> 4, kb = (tid >> 2) & 3, blk = tid & 3;
            int kbg = kb0 + kb; kbg = kbg < nkb ? kbg : nkb - 1;
            if (which == 0) {
                int mb = m0 / QB + blk; mb = mb < SM ? mb : SM - 1;
                rs = load_scale(reinterpret_cast<const ST *>(p.sa), kbg * SM + mb);
            } else {
                int nb = n0 / QB + blk; nb = nb < SN ? nb : SN - 1;
                rs = load_scale(reinterpret_cast<const ST *>(p.sb), kbg * SN + nb);
            }
        }
    };
    auto store_stage = [&](int buf) {
        unsigned char *base = smem + buf * STAGE_BYTES;
#pragma unroll
        for (int c = 0; c < CHUNKS; ++c) {
            const int id = tid + c * NTHREADS;
            const int row = id >> 3, ch = id & 7;
            const int off = (((row >> 5) * KB_STAGE + (ch >> 1)) * 2 + (ch & 1)) * 512 + (row & 31) * 16;
            *reinterpret_cast<v4i *>(base + off) = ra[c];
            *reinterpret_cast<v4i *>(base + TILE_BYTES + off) = rb[c];
        }
        if (EPI != EPI_S32 && tid < 2 * KB_STAGE * 4)
            reinterpret_cast<float *>(base + 2 * TILE_BYTES)[tid] = rs;
    };

    // ---- accumulators ------------------------------------------------------------------------
    float acc[2][2][16];
    v16i iacc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int v = 0; v < 16; ++v) { acc[i][j][v] = 0.0f; iacc[i][j][v] = 0; }
        }

    load_stage(0);
    store_stage(0);
    __syncthreads();

    for (int s = 0; s < nstages; ++s) {
        if (s + 1 < nstages) load_stage(s + 1);
        const unsigned char *base = smem + (s & 1) * STAGE_BYTES;
        const float *sc_lds = reinterpret_cast<const float *>(base + 2 * TILE_BYTES);
        const int kbs = (nkb - s * KB_STAGE) < KB_STAGE ? (nkb - s * KB_STAGE) : KB_STAGE;
        for (int kb = 0; kb < kbs; ++kb) {
            v4i a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                a[i] = *reinterpret_cast<const v4i *>(base + ((wm * 2 + i) * KB_STAGE + kb) * 1024 + lane * 16);
                b[i] = *reinterpret_cast<const v4i *>(base + TILE_BYTES + ((wn * 2 + i) * KB_STAGE + kb) * 1024 + lane * 16);
            }
            if (EPI == EPI_S32) {
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        iacc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], iacc[i][j], 0, 0, 0);
            } else {
                float fa[2], fb[2];
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    fa[i] = sc_lds[kb * 4 + wm * 2 + i];
                    fb[i] = sc_lds[16 + kb * 4 + wn * 2 + i];
                }
                const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                for (int i = 0; i < 2; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], zero, 0, 0, 0);
                        const float sab = fa[i] * fb[j];
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            acc[i][j][v] = __builtin_fmaf(sab, (float)d[v], acc[i][j][v]);
                    }
            }
        }
        if (s + 1 < nstages) store_stage((s + 1) & 1);
        __syncthreads();
    }

    // ---- epilogue: one 32x32 block at a time through a wave-private LDS patch ------------------
    // MFMA result layout: lane l, register v  <->  row 8*(v/4) + 4*(l/32) + v%4, column l%32.
    // Read-back layout: lane l  <->  row l/2, columns 16*(l%2) .. +15 (row-contiguous stores).
    float *patch = reinterpret_cast<float *>(smem) + wave * (QB * EPI_LD);
    const int rrow = lane >> 1, rcol = (lane & 1) * 16;
    const float biasmax = (EPI == EPI_Q && p.biasmax) ? p.biasmax[0] : 0.0f;

#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int bm = m0 + (wm * 2 + i) * QB, bn = n0 + (wn * 2 + j) * QB;
            const bool valid = bm < p.M && bn < p.N;          // wave-uniform
            float amax = 0.0f;
            if (EPI == EPI_Q) {
                float m = 0.0f;
#pragma unroll
                for (int v = 0; v < 16; ++v) m = fmaxf(m, fabsf(acc[i][j][v]));
                amax = wave_max(m) + biasmax;
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (EPI == EPI_S32) patch[r * EPI_LD + (lane & 31)] = __int_as_float(iacc[i][j][v]);
                else patch[r * EPI_LD + (lane & 31)] = acc[i][j][v];
            }
            __syncthreads();
            float x[16];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const v4f t = *reinterpret_cast<const v4f *>(patch + rrow * EPI_LD + rcol + 4 * k);
                x[4 * k] = t.x; x[4 * k + 1] = t.y; x[4 * k + 2] = t.z; x[4 * k + 3] = t.w;
            }
            __syncthreads();
            if (!valid) continue;
            const size_t e0 = (size_t)(bm + rrow) * p.N + bn + rcol;
            if (EPI == EPI_S32) {
                v4i *dst = reinterpret_cast<v4i *>(reinterpret_cast<int32_t *>(p.C) + e0);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    v4i t = {__float_as_int(x[4 * k]), __float_as_int(x[4 * k + 1]),
                             __float_as_int(x[4 * k + 2]), __float_as_int(x[4 * k + 3])};
                    dst[k] = t;
                }
            } else if (EPI == EPI_FP) {
                if (p.out_dtype == JF_FP_F32) {
                    v4f *dst = reinterpret_cast<v4f *>(reinterpret_cast<float *>(p.C) + e0);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        v4f t = {x[4 * k], x[4 * k + 1], x[4 * k + 2], x[4 * k + 3]};
                        dst[k] = t;
                    }
                } else if (p.out_dtype == JF_FP_F16) {
                    half_t h[16];
#pragma unroll
                    for (int k = 0; k < 16; ++k) h[k] = (half_t)x[k];
                    v4i *dst = reinterpret_cast<v4i *>(reinterpret_cast<half_t *>(p.C) + e0);
                    dst[0] = *reinterpret_cast<v4i *>(&h[0]);
                    dst[1] = *reinterpret_cast<v4i *>(&h[8]);
                } else {
                    __bf16 h[16];
#pragma unroll
                    for (int k = 0; k < 16; ++k) h[k] = (__bf16)x[k];
                    v4i *dst = reinterpret_cast<v4i *>(reinterpret_cast<__bf16 *>(p.C) + e0);
                    dst[0] = *reinterpret_cast<v4i *>(&h[0]);
                    dst[1] = *reinterpret_cast<v4i *>(&h[8]);
                }
            } else {
                v4i codes = {0, 0, 0, 0};
                float scale = 0.0f;
                if (amax > 0.0f) {
                    scale = amax / 127.0f;
                    BlockDivisor d(amax);
                    float t[16];
                    if (p.bias) {
#pragma unroll
                        for (int k = 0; k < 16; ++k) x[k] = x[k] + p.bias[bn + rcol + k];
                    }
#pragma unroll
                    for (int k = 0; k < 16; ++k) t[k] = d.div(127.0f * x[k]);
                    if (p.rounding == JF_ROUND_STOCHASTIC) {
                        float n[16];
                        sr_noise16(p.seed, p.offset, (uint64_t)e0, n);
#pragma unroll
                        for (int k = 0; k < 16; ++k) t[k] = t[k] + n[k];
                    }
                    int c[16];
#pragma unroll
                    for (int k = 0; k < 16; ++k) c[k] = clamp127(__builtin_rintf(t[k]));
                    codes.x = (int)pack4(c[0], c[1], c[2], c[3]);
                    codes.y = (int)pack4(c[4], c[5], c[6], c[7]);
                    codes.z = (int)pack4(c[8], c[9], c[10], c[11]);
                    codes.w = (int)pack4(c[12], c[13], c[14], c[15]);
                }
                *reinterpret_cast<v4i *>(reinterpret_cast<int8_t *>(p.C) + e0) = codes;
                if (lane == 0) store_scale(reinterpret_cast<ST *>(p.sc), (bm / QB) * SN + bn / QB, scale);
            }
        }
}

// -------------------------------------------------------------------------------------------------
// int8 transpose: out[C,R] = in[R,C].  64x64 tiles through LDS; 16-byte loads and stores.
__global__ __launch_bounds__(256) void transpose_s8_kernel(const int8_t *in, int8_t *out, int R, int C)
{
    __shared__ __attribute__((aligned(16))) unsigned char tile[64][64 + 16];
    const int tiles_c = (C + 63) / 64;
    const int tr = blockIdx.x / tiles_c, tc = blockIdx.x % tiles_c;
    const int r0 = tr * 64, c0 = tc * 64;
    const int tid = threadIdx.x;
    {
        const int row = tid >> 2, ch = tid & 3;                 // 64 rows x 4 chunks of 16 bytes
        v4i v = {0, 0, 0, 0};
        if (r0 + row < R && c0 + ch * 16 < C)
            v = *reinterpret_cast<const v4i *>(in + (size_t)(r0 + row) * C + c0 + ch * 16);
        *reinterpret_cast<v4i *>(&tile[row][ch * 16]) = v;
    }
    __syncthreads();
    {
        const int orow = tid >> 2, och = tid & 3;               // output row = input column
        unsigned char b[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) b[k] = tile[och * 16 + k][orow];
        if (c0 + orow < C && r0 + och * 16 < R)
            *reinterpret_cast<v4i *>(out + (size_t)(c0 + orow) * R + r0 + och * 16) = *reinterpret_cast<v4i *>(b);
    }
}

static int launch_transpose(const int8_t *in, int R, int C, int8_t *out, hipStream_t st)
{
    const int tiles = ((R + 63) / 64) * ((C + 63) / 64);
    hipLaunchKernelGGL(transpose_s8_kernel, dim3(tiles), dim3(256), 0, st, in, out, R, C);
    return (int)hipGetLastError();
}

template <int EPI, typename ST> static int launch_gemm(const GemmArgs &a, hipStream_t st)
{
    GemmArgs p = a;
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    auto kern = igemm_nt_kernel<EPI, ST>;
    // more than 64 KiB of dynamic LDS has to be opted into, per function
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       SMEM_BYTES);
    if (e != hipSuccess) return (int)e;
    hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n), dim3(NTHREADS), SMEM_BYTES, st, p);
    return (int)hipGetLastError();
}

static int check_gemm_common(const void *A, const void *B, const void *C, int M, int N, int K, int b_layout,
                             const void *ws, size_t ws_bytes)
{
    if (!A || !B || !C) return JF_ERR_NULL;
    if (!mult32(M) || !mult32(N) || !mult32(K)) return JF_ERR_SHAPE;
    if (b_layout != JF_B_NK && b_layout != JF_B_KN) return JF_ERR_ENUM;
    if (!aligned16(A) || !aligned16(B) || !aligned16(C)) return JF_ERR_ALIGN;
    if (b_layout == JF_B_KN) {
        if (!ws || ws_bytes < (size_t)N * (size_t)K) return JF_ERR_WORKSPACE;
        if (!aligned16(ws)) return JF_ERR_ALIGN;
    }
    return JF_OK;
}

// B as [N,K]: either the caller's buffer or its transpose in the workspace.
static int b_as_nk(const int8_t *&B, int N, int K, int b_layout, void *ws, hipStream_t st)
{
    if (b_layout == JF_B_NK) return JF_OK;
    int rc = launch_transpose(B, K, N, reinterpret_cast<int8_t *>(ws), st);
    B = reinterpret_cast<const int8_t *>(ws);
    return rc;
}

}  // namespace jf

using namespace jf;

extern "C" {

const char *jf_error_string(int code)
{
    switch (code) {
    case JF_OK: return "ok";
    case JF_ERR_NULL: return "jetfire_hip: required pointer is NULL";
    case JF_ERR_SHAPE: return "jetfire_hip: dimension is not a positive multiple of 32";
    case JF_ERR_ENUM: return "jetfire_hip: unknown layout/dtype/rounding code";
    case JF_ERR_ALIGN: return "jetfire_hip: pointer not 16-byte aligned";
    case JF_ERR_WORKSPACE: return "jetfire_hip: workspace missing or too small";
    case JF_ERR_DEVICE: return "jetfire_hip: device is not gfx950";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "jetfire_hip: unknown error";
    }
}

size_t jf_igemm_workspace_bytes(int M, int N, int K, int b_layout)
{
    (void)M;
    return b_layout == JF_B_KN ? (size_t)N * (size_t)K : 0;
}

int jf_igemm_s32(const int8_t *A, const int8_t *B, int32_t *C, int M, int N, int K, int b_layout,
                 void *workspace, size_t workspace_bytes, jf_stream_t stream)
{
    int rc = check_gemm_common(A, B, C, M, N, K, b_layout, workspace, workspace_bytes);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    if ((rc = b_as_nk(B, N, K, b_layout, workspace, st))) return rc;
    GemmArgs a = {};
    a.A = A; a.B = B; a.C = C; a.M = M; a.N = N; a.K = K; a.lda = K; a.ldb = K;
    return launch_gemm<EPI_S32, float>(a, st);
}

int jf_igemm_block_acc(const int8_t *A, const int8_t *B, int32_t *acc, int M, int N, int K, int b_layout,
                       void *workspace, size_t workspace_bytes, jf_stream_t stream)
{
    int rc = check_gemm_common(A, B, acc, M, N, K, b_layout, workspace, workspace_bytes);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    if ((rc = b_as_nk(B, N, K, b_layout, workspace, st))) return rc;
    for (int kb = 0; kb < K / QB; ++kb) {
        GemmArgs a = {};
        a.A = A + kb * QB; a.B = B + kb * QB; a.C = acc + (size_t)kb * M * N;
        a.M = M; a.N = N; a.K = QB; a.lda = K; a.ldb = K;
        if ((rc = launch_gemm<EPI_S32, float>(a, st))) return rc;
    }
    return JF_OK;
}

int jf_igemm_block_fp(const int8_t *A, const int8_t *B, const void *sa, const void *sb, void *C,
                      int M, int N, int K, int b_layout, int scale_dtype, int out_dtype,
                      void *workspace, size_t workspace_bytes, jf_stream_t stream)
{
    int rc = check_gemm_common(A, B, C, M, N, K, b_layout, workspace, workspace_bytes);
    if (rc) return rc;
    if (!sa || !sb) return JF_ERR_NULL;
    if ((scale_dtype != JF_SCALE_F16 && scale_dtype != JF_SCALE_F32) ||
        (out_dtype != JF_FP_F16 && out_dtype != JF_FP_F32 && out_dtype != JF_FP_BF16)) return JF_ERR_ENUM;
    hipStream_t st = (hipStream_t)stream;
    if ((rc = b_as_nk(B, N, K, b_layout, workspace, st))) return rc;
    GemmArgs a = {};
    a.A = A; a.B = B; a.sa = sa; a.sb = sb; a.C = C; a.M = M; a.N = N; a.K = K; a.lda = K; a.ldb = K;
    a.out_dtype = out_dtype;
    return scale_dtype == JF_SCALE_F16 ? launch_gemm<EPI_FP, half_t>(a, st) : launch_gemm<EPI_FP, float>(a, st);
}

int jf_igemm_block_q(const int8_t *A, const int8_t *B, const void *sa, const void *sb,
                     const float *bias, const float *biasmax, int8_t *C, void *sc,
                     int M, int N, int K, int b_layout, int scale_dtype, int rounding,
                     uint64_t seed, uint64_t offset,
                     void *workspace, size_t workspace_bytes, jf_stream_t stream)
{
    int rc = check_gemm_common(A, B, C, M, N, K, b_layout, workspace, workspace_bytes);
    if (rc) return rc;
    if (!sa || !sb || !sc) return JF_ERR_NULL;
    if ((scale_dtype != JF_SCALE_F16 && scale_dtype != JF_SCALE_F32) ||
        (rounding != JF_ROUND_NEAREST && rounding != JF_ROUND_STOCHASTIC)) return JF_ERR_ENUM;
    hipStream_t st = (hipStream_t)stream;
    if ((rc = b_as_nk(B, N, K, b_layout, workspace, st))) return rc;
    GemmArgs a = {};
    a.A = A; a.B = B; a.sa = sa; a.sb = sb; a.C = C; a.sc = sc; a.bias = bias; a.biasmax = biasmax;
    a.M = M; a.N = N; a.K = K; a.lda = K; a.ldb = K; a.rounding = rounding; a.seed = seed; a.offset = offset;
    return scale_dtype == JF_SCALE_F16 ? launch_gemm<EPI_Q, half_t>(a, st) : launch_gemm<EPI_Q, float>(a, st);
}

int jf_transpose_s8(const int8_t *in, int R, int C, int8_t *out, jf_stream_t stream)
{
    if (!in || !out) return JF_ERR_NULL;
    if (R <= 0 || C <= 0 || (R % 16) || (C % 16)) return JF_ERR_SHAPE;
    if (!aligned16(in) || !aligned16(out)) return JF_ERR_ALIGN;
    return launch_transpose(in, R, C, out, (hipStream_t)stream);
}

}  // extern "C"
