// Memory-bound kernels of the INT8 data flow for gfx950: block quantise (+transpose), dequantise,
// fused dequant->LayerNorm->requant, dequant->GELU->requant (forward and backward), residual add.
//
// Common shape: ONE WAVEFRONT OWNS ONE 32x32 QUANTISATION BLOCK.  Lane l holds row l/2, columns
// 16*(l%2) .. +15 of the block: one 16-byte load/store of INT8 codes per lane (two lanes cover a
// 32-byte row segment), four 16-byte accesses for fp32 data.  The block absmax is a pure 64-lane
// reduction, so no LDS and no workgroup barrier is needed on the block-local kernels.  Workgroups
// have 4 waves and walk the block grid with a grid stride.
//
// Reference kernels being replaced: the Triton kernels of Jetfire/Nonlinear/*.py (cited per kernel).
#include "jf_device.hpp"

#include <atomic>

namespace jf {

constexpr int NT = 256;                 // threads per workgroup
constexpr int WPB = NT / WAVE;          // waves (= blocks in flight) per workgroup

template <typename T> struct Load16;
template <> struct Load16<float> {
    static __device__ __forceinline__ void run(const float *p, float x[16])
    {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            v4f t = reinterpret_cast<const v4f *>(p)[k];
            x[4 * k] = t.x; x[4 * k + 1] = t.y; x[4 * k + 2] = t.z; x[4 * k + 3] = t.w;
        }
    }
};
template <> struct Load16<half_t> {
    static __device__ __forceinline__ void run(const half_t *p, float x[16])
    {
        half_t h[16];
        *reinterpret_cast<v4i *>(&h[0]) = reinterpret_cast<const v4i *>(p)[0];
        *reinterpret_cast<v4i *>(&h[8]) = reinterpret_cast<const v4i *>(p)[1];
#pragma unroll
        for (int k = 0; k < 16; ++k) x[k] = (float)h[k];
    }
};
template <> struct Load16<__bf16> {
    static __device__ __forceinline__ void run(const __bf16 *p, float x[16])
    {
        uint16_t h[16];
        *reinterpret_cast<v4i *>(&h[0]) = reinterpret_cast<const v4i *>(p)[0];
        *reinterpret_cast<v4i *>(&h[8]) = reinterpret_cast<const v4i *>(p)[1];
#pragma unroll
        for (int k = 0; k < 16; ++k) x[k] = __uint_as_float((uint32_t)h[k] << 16);
    }
};

__device__ __forceinline__ void store16_f32(float *p, const float x[16])
{
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        v4f t = {x[4 * k], x[4 * k + 1], x[4 * k + 2], x[4 * k + 3]};
        reinterpret_cast<v4f *>(p)[k] = t;
    }
}

// 16 consecutive values, rounded to nearest even, as two 16-byte stores
template <typename OT> __device__ __forceinline__ void store16_as(OT *p, const float x[16])
{
    OT h[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) h[k] = (OT)x[k];
    reinterpret_cast<v4i *>(p)[0] = *reinterpret_cast<v4i *>(&h[0]);
    reinterpret_cast<v4i *>(p)[1] = *reinterpret_cast<v4i *>(&h[8]);
}
template <> __device__ __forceinline__ void store16_as<float>(float *p, const float x[16]) { store16_f32(p, x); }

// Position of this wave's block / this lane's 16 elements.
struct BlockPos {
    int rb, cb, row, col;     // block coordinates; absolute row / first column of the lane
    size_t e0;                // flat index of the lane's first element
    __device__ __forceinline__ BlockPos(int blk, int SC, int C, int lane)
    {
        rb = blk / SC; cb = blk - rb * SC;
        row = rb * QB + (lane >> 1);
        col = cb * QB + (lane & 1) * 16;
        e0 = (size_t)row * C + col;
    }
};

#define JF_FOR_EACH_BLOCK(R, C)                                                            \
    const int lane = threadIdx.x & 63;                                                     \
    const int SC = (C) / QB;                                                               \
    const int nblk = ((R) / QB) * SC;                                                      \
    for (int blk = blockIdx.x * WPB + (threadIdx.x >> 6); blk < nblk; blk += gridDim.x * WPB)

// Codes leave in whole 128-byte lines.  In the row layout of a block (lane l: row l/2, 16 bytes) a store instruction
// writes 32 rows x 32 bytes, a quarter of each line; out of the caches those quarter-line writes cost a third of the
// bandwidth, also when the four waves of a workgroup write the four quarters at the same moment (copies of 8192 x 6400
// bytes: 32 us that way, 23 us with the same reads and whole-line writes).  Kernels whose workgroup works on four adjacent
// column blocks of one row block (a group; wave w: block 4*cg + w, idle beyond the end of the row) therefore exchange
// the codes through a 32 x 128-byte patch in LDS (144 bytes per row) and wave w stores rows 8w .. 8w+7 of the group.
// Two patches take turns, so one barrier per group is enough: a patch is rewritten two groups later, behind the
// barrier of the group in between.  Every wave of the workgroup must make the call (it contains the barrier).
constexpr int LINE_PITCH = 4 * QB + 16;
struct GroupLineStore {
    unsigned char *patches;       // [2][QB * LINE_PITCH], shared by the workgroup
    int turn, lane, wave;
    __device__ __forceinline__ GroupLineStore(unsigned char *p, int lane_, int wave_) : patches(p), turn(0), lane(lane_), wave(wave_) {}
    __device__ __forceinline__ void store(v4i codes, int8_t *out, int rb, int cg, int C)
    {
        unsigned char *patch = patches + turn * (QB * LINE_PITCH);
        turn ^= 1;
        *reinterpret_cast<v4i *>(patch + (lane >> 1) * LINE_PITCH + QB * wave + 16 * (lane & 1)) = codes;
        __syncthreads();
        const int row = 8 * wave + (lane >> 3), lcol = 16 * (lane & 7);
        if (cg * 4 * QB + lcol < C)
            *reinterpret_cast<v4i *>(out + (size_t)(rb * QB + row) * C + cg * 4 * QB + lcol) =
                *reinterpret_cast<const v4i *>(patch + row * LINE_PITCH + lcol);
    }
};

// ------------------------------------------------------------------------------------------------
// quantize.py:33-117 (and quantize_transpose.py:33-129 when qT != nullptr)
// The input is up to QSRC_MAX column slabs lying side by side in the result: slab k is [R, end[k] - end[k-1]] with rows
// ldx[k] elements apart (plain case: one slab, ldx = C).  The rounding noise of an element depends on its position in
// the result, so quantising slabs where they lie gives the codes of quantising their concatenation.
// workgroups of the quantize kernel (4 waves = 4 adjacent column blocks of one row block); with a transposed copy: 32 per
// 8 (quad of row blocks, group of 4 column blocks) pairs, see the kernel
__host__ __device__ static inline int quantize_groups(int R, int C, bool transposed)
{
    const int RB = R / QB, SC = C / QB, G4 = (SC + WPB - 1) / WPB;
    if (!transposed) return RB * G4;
    const int pairs = ((RB + 3) / 4) * G4;
    return 32 * ((pairs + 7) / 8);
}
constexpr int QSRC_MAX = 4;
struct QuantSrc {
    const void *x[QSRC_MAX];
    int ldx[QSRC_MAX];
    int end[QSRC_MAX];       // first column behind slab k (cumulative widths)
    int n;
};
template <typename T, typename ST>
__global__ __launch_bounds__(NT) void quantize_kernel(QuantSrc src, int R, int C, int8_t *q, ST *s, int8_t *qT,
                                                      int rounding, uint64_t seed, uint64_t offset, float amax_eps)
{
    __shared__ __attribute__((aligned(16))) unsigned char tpatch[WPB][QB][QB + 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int SC = C / QB, RB = R / QB, G4 = (SC + WPB - 1) / WPB;
    // Which blocks a workgroup takes: four adjacent column blocks of one row block (whole 128-byte lines of q).  Without
    // a transposed copy workgroups walk the tensor row block by row block.  With one, the 128-byte lines of qT are
    // written 32 bytes at a time by the workgroups of four consecutive row blocks: those four are made the workgroups
    // b, b+8, b+16, b+24, which the dispatcher deals to the same XCD one after the other, so that the four pieces of a
    // line meet in that XCD's L2 before the line leaves for memory (see quantize_groups() for the count).
    const int nwg = quantize_groups(R, C, qT != nullptr);
    __shared__ __attribute__((aligned(16))) unsigned char line_patches[2 * QB * LINE_PITCH];
    GroupLineStore lines(line_patches, lane, wave);
    for (int wg = blockIdx.x; wg < nwg; wg += gridDim.x)
    {
        int rbq, cg;
        if (qT) {
            const int idx = (wg >> 5) * 8 + (wg & 7), j = (wg >> 3) & 3;     // (row-block quad, column group) and the row block of the quad
            rbq = (idx / G4) * 4 + j; cg = idx % G4;
        } else {
            rbq = wg / G4; cg = wg - rbq * G4;
        }
        const int cbq = cg * WPB + wave;
        const bool valid = rbq < RB && cbq < SC;                            // wave-uniform
        if (!valid) {
            if (!qT && rbq < RB) lines.store(v4i{0, 0, 0, 0}, q, rbq, cg, C);   // (the barrier; its bytes lie beyond the row's end)
            continue;
        }
        const int blk = rbq * SC + cbq;
        BlockPos pos(blk, SC, C, lane);
        // the slab of this block (uniform over the wave; slabs are whole blocks wide)
        const T *x = reinterpret_cast<const T *>(src.x[0]);
        int ldx = src.ldx[0], begin = 0;
#pragma unroll
        for (int k = 1; k < QSRC_MAX; ++k)
            if (k < src.n && pos.cb * QB >= src.end[k - 1]) { x = reinterpret_cast<const T *>(src.x[k]); ldx = src.ldx[k]; begin = src.end[k - 1]; }
        float v[16];
        Load16<T>::run(x + (size_t)pos.row * ldx + (pos.col - begin), v);
        float scale;
        v4i codes = quantize16(v, amax_eps, rounding, seed, offset, pos.e0, &scale);
        if (qT) *reinterpret_cast<v4i *>(q + pos.e0) = codes;
        else lines.store(codes, q, rbq, cg, C);
        if (lane == 0) store_scale(s, pos.rb * SC + pos.cb, scale);
        if (qT) {
            unsigned char(*tp)[QB + 16] = tpatch[threadIdx.x >> 6];
            *reinterpret_cast<v4i *>(&tp[lane >> 1][(lane & 1) * 16]) = codes;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // The transposing LDS read of gfx950 (groups of 16 lanes; lanes 2k, 2k+1 address the two 8-byte pieces of
            // patch row k, lane i receives byte i%8 of the pieces addressed by lanes i/8, i/8+2, ..: one column, 8 rows).
            // Lane group g takes the 16-column window g%2 and the 16-row half g/2 of the block; two reads (rows +0..7,
            // +8..15) leave a lane with 16 consecutive bytes of one output row.
            typedef __attribute__((address_space(3))) unsigned char lds_u8;
            const int g = lane >> 4, i = lane & 15, cw = g & 1, rh = g >> 1;
            const unsigned addr = (unsigned)(uintptr_t)(lds_u8 *)&tp[16 * rh + (i >> 1)][16 * cw + 8 * (i & 1)];
            v2i lo, hi;
            asm volatile("ds_read_b64_tr_b8 %0, %1" : "=v"(lo) : "v"(addr));
            asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "n"(8 * (QB + 16)));
            asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo), "+v"(hi));
            const int ocol = 16 * cw + (i & 7) + 8 * (i >> 3);           // output row = input column
            *reinterpret_cast<v4i *>(qT + (size_t)(pos.cb * QB + ocol) * R + pos.rb * QB + 16 * rh) = v4i{lo.x, lo.y, hi.x, hi.y};
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// dequantize.py:28-84
template <typename ST, typename OT>
__global__ __launch_bounds__(NT) void dequantize_kernel(const int8_t *q, const ST *s, int R, int C, OT *out)
{
    JF_FOR_EACH_BLOCK(R, C)
    {
        BlockPos pos(blk, SC, C, lane);
        float x[16];
        unpack16(*reinterpret_cast<const v4i *>(q + pos.e0), load_scale(s, pos.rb * SC + pos.cb), x);
        store16_as<OT>(out + pos.e0, x);
    }
}

// Code tensors leave the GELU kernels in whole 128-byte row pieces.  A wave works on one 32x32 block in the row layout
// (lane l: row l/2, 16 bytes), in which a store instruction touches 32 rows with 32 bytes each: a quarter of each
// 128-byte line.  Out of the caches that costs a third of the bandwidth (a copy of 8192x6400 bytes: 30 us when written
// in that shape, 23 us read in that shape but written in whole lines, 21 us with both in whole lines).  So a wave
// works through four adjacent blocks (a group; the last group of a row may be partial), leaves each block's codes in
// a wave-private 32 x 128-byte patch in LDS (padded to 144 bytes per row) and then stores the group's 32 rows, 128
// bytes each (lane l: rows l/8, l/8 + 8, .., bytes 16*(l%8) ..).  All blocks of a group are requested at once, so the
// later ones arrive while the first is worked on; one group per wave and many workgroups beat fewer, longer-lived ones
// with requests further ahead here (the dispatcher evens them out).
__device__ __forceinline__ void group_put(unsigned char *patch, int lane, int j, v4i codes)
{
    *reinterpret_cast<v4i *>(patch + (lane >> 1) * LINE_PITCH + QB * j + 16 * (lane & 1)) = codes;
}
__device__ __forceinline__ void group_store_lines(unsigned char *patch, int lane, int8_t *out, int rb, int cg, int C)
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int lcol = 16 * (lane & 7);
    if (cg * 4 * QB + lcol < C) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int row = 8 * k + (lane >> 3);
            *reinterpret_cast<v4i *>(out + (size_t)(rb * QB + row) * C + cg * 4 * QB + lcol) =
                *reinterpret_cast<const v4i *>(patch + row * LINE_PITCH + lcol);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();                               // the patch may be rewritten
}
// The (up to) four blocks of group (rb, cg) of a block tensor, in the row layout, and their scales.
template <typename ST>
__device__ __forceinline__ void group_request(const int8_t *q, const ST *s, int C, int rb, int cg, int lane, v4i (&c)[4], float (&sc)[4])
{
    const int SC = C / QB;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        // beyond the end of a row the last block is read again (and not used): four loads in a straight line, whose
        // arrivals the compiler can then count one by one
        const int cb = (cg * 4 + j < SC) ? cg * 4 + j : SC - 1;
        c[j] = *reinterpret_cast<const v4i *>(q + (size_t)(rb * QB + (lane >> 1)) * C + cb * QB + (lane & 1) * 16);
        sc[j] = load_scale(s, rb * SC + cb);
    }
}
static inline int grid_for_groups(int R, int C)
{
    const long groups = (long)(R / QB) * ((C / QB + 3) / 4), g = (groups + WPB - 1) / WPB;
    return (int)(g < 256L * 16 ? g : 256L * 16);
}

// gelu_fwd.py:34-126
template <int APPROX, typename ST>
__global__ __launch_bounds__(NT) void gelu_fwd_kernel(const int8_t *q, const ST *s, int R, int C, float amax_eps,
                                                      int8_t *qy, ST *sy)
{
    __shared__ __attribute__((aligned(16))) float table[WPB][256];
    __shared__ __attribute__((aligned(16))) int qtable[WPB][64];      // 256 one-byte entries per wave
    __shared__ __attribute__((aligned(16))) unsigned char patches[WPB][QB * LINE_PITCH];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float *tab = table[wave];
    int *qtab = qtable[wave];
    unsigned char *patch = patches[wave];
    const int SC = C / QB, SG = (SC + 3) / 4, ngrp = (R / QB) * SG, stride = gridDim.x * WPB;
    int g = blockIdx.x * WPB + wave;
    if (g >= ngrp) return;
    float zero = 0.0f;
    asm volatile("" : "+v"(zero));                                 // evaluated on the device, like every other entry
    const float f0 = gelu<APPROX>(zero);
    for (; g < ngrp; g += stride) {
        const int rb = g / SG, cg = g - rb * SG;
        v4i cur[4];
        float csc[4];
        group_request(q, s, C, rb, cg, lane, cur, csc);            // the later blocks arrive while the first is worked on
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int cb = cg * 4 + j;
            if (cb < SC) {                                         // uniform
                float scale;
                group_put(patch, lane, j, gelu_fwd_block<APPROX>(cur[j], csc[j], f0, amax_eps, tab, qtab, lane, &scale));
                if (lane == 0) store_scale(sy, rb * SC + cb, scale);
            }
        }
        group_store_lines(patch, lane, qy, rb, cg, C);
    }
}

// gelu_bwd.py:28-171
// (Held to five waves per SIMD: with the codes of four blocks of both inputs in flight the kernel wants 97 registers, one
// more than five waves allow, and runs 1 us faster at 8192x6400 with five waves than with four.)
template <int APPROX, typename ST>
__global__ __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(5, 5)))
void gelu_bwd_kernel(const int8_t *qx, const ST *sx, const int8_t *qg, const ST *sg,
                                                      int R, int C, int rounding, uint64_t seed, uint64_t offset,
                                                      int8_t *qy, ST *sy)
{
    __shared__ __attribute__((aligned(16))) float table[WPB][256];
    __shared__ __attribute__((aligned(16))) unsigned char patches[WPB][QB * LINE_PITCH];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float *tab = table[wave];
    unsigned char *patch = patches[wave];
    const int SC = C / QB, SG = (SC + 3) / 4, ngrp = (R / QB) * SG, stride = gridDim.x * WPB;
    int g = blockIdx.x * WPB + wave;
    if (g >= ngrp) return;
    float zero = 0.0f;
    asm volatile("" : "+v"(zero));
    const float f0 = dgelu<APPROX>(zero);
    for (; g < ngrp; g += stride) {
        const int rb = g / SG, cg = g - rb * SG;
        v4i cx[4], cgr[4];
        float scx[4], scg[4];
        group_request(qx, sx, C, rb, cg, lane, cx, scx);
        group_request(qg, sg, C, rb, cg, lane, cgr, scg);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int cb = cg * 4 + j;
            if (cb < SC) {                                         // uniform
                const size_t e0 = (size_t)(rb * QB + (lane >> 1)) * C + cb * QB + (lane & 1) * 16;
                float scale;
                group_put(patch, lane, j, gelu_bwd_block<APPROX>(cx[j], scx[j], cgr[j], scg[j], f0, tab, lane, rounding, seed, offset, e0, &scale));
                if (lane == 0) store_scale(sy, rb * SC + cb, scale);
            }
        }
        group_store_lines(patch, lane, qy, rb, cg, C);
    }
}

// layernorm.py:74-190, with a real beta.  Arithmetic (this library's definition; the reference dequantises in binary16):
//   a = s * rstd[r],  b = -(mean[r] * rstd[r]),  xhat = fma(float(q), a, b),  y = fma(xhat, gamma[c], beta[c])
// i.e. dequantisation and normalisation are one fma per element with two per-row, per-block constants.
// One wave: one column block x CW_ROWS consecutive row blocks (gamma and beta are loaded once per wave); the four waves
// of a workgroup take four adjacent column blocks, i.e. whole 128-byte lines per row.  The source asks for everything a
// wave reads before it computes anything and stores at the end.  Measured at 8192x1600: storing each block as soon as it
// is done, or pinning the requests above the arithmetic (the compiler moves those of the later blocks behind the first
// block's), changes nothing; what counts is how evenly the waves fill the SIMDs: 9.1 us with 2 row blocks per wave (6.5
// waves per SIMD), 10.0 us with 4 (3.25: a quarter of the SIMDs get a fourth wave), 11.6 us with 8.
constexpr int CW_ROWS = 2;
template <typename ST>
__global__ __launch_bounds__(NT) void layernorm_fwd_kernel(const int8_t *q, const ST *s, const float *gamma,
                                                           const float *beta, const float *mean, const float *rstd,
                                                           int R, int C, int8_t *qy, ST *sy)
{
    __shared__ __attribute__((aligned(16))) unsigned char line_patches[2 * QB * LINE_PITCH];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int SC = C / QB, RB = R / QB, S4 = (SC + WPB - 1) / WPB;
    const int cg = blockIdx.x % S4, grp = blockIdx.x / S4;
    GroupLineStore lines(line_patches, lane, wave);
    // a wave of the last, partial group of column blocks computes its neighbour's block again (and keeps none of it):
    // it is needed for the whole-line stores of the group's rows
    const bool mine = cg * WPB + wave < SC;
    const int cb = mine ? cg * WPB + wave : SC - 1;
    const int col = cb * QB + (lane & 1) * 16;
    const int nrb = (RB - grp * CW_ROWS) < CW_ROWS ? (RB - grp * CW_ROWS) : CW_ROWS;      // uniform
    float g[16], bt[16];
    Load16<float>::run(gamma + col, g);
    if (beta) Load16<float>::run(beta + col, bt);
    else {
#pragma unroll
        for (int k = 0; k < 16; ++k) bt[k] = 0.0f;
    }
    v4i c[CW_ROWS];
    float sc[CW_ROWS], mu[CW_ROWS], rs[CW_ROWS];
#pragma unroll
    for (int k = 0; k < CW_ROWS; ++k) {
        const int rb = grp * CW_ROWS + (k < nrb ? k : 0);
        const int row = rb * QB + (lane >> 1);
        c[k] = *reinterpret_cast<const v4i *>(q + (size_t)row * C + col);
        sc[k] = load_scale(s, rb * SC + cb);
        mu[k] = mean[row];
        rs[k] = rstd[row];
    }
    v4i out[CW_ROWS];
    float so[CW_ROWS];
#pragma unroll
    for (int k = 0; k < CW_ROWS; ++k) {
        const size_t e0 = (size_t)((grp * CW_ROWS + k) * QB + (lane >> 1)) * C + col;
        const float a = sc[k] * rs[k], b = -(mu[k] * rs[k]);
        float x[16];
        codes_to_float16(c[k], x);
#pragma unroll
        for (int j = 0; j < 16; ++j) x[j] = __builtin_fmaf(__builtin_fmaf(x[j], a, b), g[j], bt[j]);
        out[k] = quantize16(x, 0.0f, JF_ROUND_NEAREST, 0, 0, e0, &so[k]);
    }
#pragma unroll
    for (int k = 0; k < CW_ROWS; ++k) {
        if (k < nrb) {                                             // (uniform over the workgroup)
            const int rb = grp * CW_ROWS + k;
            lines.store(out[k], qy, rb, cg, C);
            if (mine && lane == 0) store_scale(sy, rb * SC + cb, so[k]);
        }
    }
}

// Row statistics of a block tensor.  One workgroup per 32-row strip; the 4 waves take the column
// blocks round-robin and leave the exact integer sums (sum q, sum q^2 per row and block) in LDS;
// then one lane per row combines them in ascending block order with fmaf.
template <typename ST>
__global__ __launch_bounds__(NT) void rowstats_kernel(const int8_t *q, const ST *s, int R, int C, float eps,
                                                      float *mean, float *rstd)
{
    extern __shared__ int isum[];                 // [2][32][SC]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int SC = C / QB, rb = blockIdx.x;
    int *i1 = isum, *i2 = isum + QB * SC;
    for (int cb = wave; cb < SC; cb += WPB) {
        const size_t e0 = (size_t)(rb * QB + (lane >> 1)) * C + cb * QB + (lane & 1) * 16;
        const v4i p = *reinterpret_cast<const v4i *>(q + e0);
        const int w[4] = {p.x, p.y, p.z, p.w};
        int a = 0, b = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int v0 = (w[k] << 24) >> 24, v1 = (w[k] << 16) >> 24, v2 = (w[k] << 8) >> 24, v3 = w[k] >> 24;
            a += v0 + v1 + v2 + v3;
            b += v0 * v0 + v1 * v1 + v2 * v2 + v3 * v3;
        }
        a += __shfl_xor(a, 1, WAVE);
        b += __shfl_xor(b, 1, WAVE);
        if ((lane & 1) == 0) { i1[(lane >> 1) * SC + cb] = a; i2[(lane >> 1) * SC + cb] = b; }
    }
    __syncthreads();
    if (threadIdx.x < QB) {
        const int r = threadIdx.x;
        float s1 = 0.0f, s2 = 0.0f;
        for (int cb = 0; cb < SC; ++cb) {
            const float sc = load_scale(s, rb * SC + cb);
            s1 = __builtin_fmaf(sc, (float)i1[r * SC + cb], s1);
            s2 = __builtin_fmaf(sc * sc, (float)i2[r * SC + cb], s2);
        }
        const float mu = s1 / (float)C;
        float var = __builtin_fmaf(-mu, mu, s2 / (float)C);
        var = var < 0.0f ? 0.0f : var;
        mean[rb * QB + r] = mu;
        rstd[rb * QB + r] = 1.0f / __builtin_sqrtf(var + eps);
    }
}

// Column sums over the 32 rows of a block: lane l holds row l/2 and 16 values (index k) of column set l%2.  The values
// go through a wave-private LDS patch, value k of lane l at word 66*k + l; lane j then adds rows 16*(j%2) .. +15 of
// output j/2 = (value index k = j/4, column set (j/2)%2) and the two halves are combined with one lane swap.  The pitch
// of 66 words puts the 64 lanes of every read (and of every write) on 64 different banks.  Plain adds in a fixed order
// (reproducible); moving data through LDS costs this kernel's bottleneck, the vector ALU, 17 instructions where a
// cross-lane butterfly costs 3 per value.  On return lanes with j%2 == 0 hold the total of output j/2.
constexpr int COLSUM_PITCH = 66, COLSUM_PATCH = 16 * COLSUM_PITCH;   // floats per wave
__device__ __forceinline__ float colsum16_over_rows(const float (&v)[16], int lane, float *patch)
{
#pragma unroll
    for (int k = 0; k < 16; ++k) patch[k * COLSUM_PITCH + lane] = v[k];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const float *src = patch + (lane >> 2) * COLSUM_PITCH + ((lane >> 1) & 1) + 32 * (lane & 1);
    float t = src[0];
#pragma unroll
    for (int i = 1; i < 16; ++i) t = t + src[2 * i];
    const int o = __builtin_amdgcn_update_dpp(0, __float_as_int(t), 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
    t = t + __int_as_float(o);                                     // both lanes of the pair: same two operands
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();                               // the patch may be rewritten
    return t;
}

// A block's fp32 values leave through a wave-private LDS patch: in the layout the arithmetic uses (lane l: row l/2, 16
// columns) a store instruction would write 64 separate 16-byte pieces; read back as "lane l: row 8i + l/8, columns
// 4*(l%8) .. +3" each of the four store instructions writes 8 whole 128-byte rows of the block (measured on an fp32 copy
// of 8192x1600: 17.0 against 22.9 us; the mapping of the loads makes no difference).  16-bit outputs (rounded to nearest
// even): a row of the block is 64 bytes and a store instruction writes 16 whole rows (lane l: row 16i + l/4, columns
// 8*(l%4) .. +7).  `out` points at the block's first element, ld = elements per row.
constexpr int ADD_PITCH = QB + 4;                  // floats per patch row (16-byte aligned rows, rotated over the banks)
template <typename OT>
__device__ __forceinline__ void store_block_rows(float *ypatch, const float (&a)[16], OT *out, int ld, int lane)
{
    float *w = ypatch + (lane >> 1) * ADD_PITCH + (lane & 1) * 16;
#pragma unroll
    for (int k = 0; k < 4; ++k) *reinterpret_cast<v4f *>(w + 4 * k) = v4f{a[4 * k], a[4 * k + 1], a[4 * k + 2], a[4 * k + 3]};
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (sizeof(OT) == 4) {
        float *dst = reinterpret_cast<float *>(out) + (size_t)(lane >> 3) * ld + (lane & 7) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<v4f *>(dst + (size_t)(8 * i) * ld) =
                *reinterpret_cast<const v4f *>(ypatch + (8 * i + (lane >> 3)) * ADD_PITCH + (lane & 7) * 4);
    } else {
        OT *dst = out + (size_t)(lane >> 2) * ld + (lane & 3) * 8;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float *r = ypatch + (16 * i + (lane >> 2)) * ADD_PITCH + (lane & 3) * 8;
            const v4f lo = *reinterpret_cast<const v4f *>(r), hi = *reinterpret_cast<const v4f *>(r + 4);
            OT h[8] = {(OT)lo.x, (OT)lo.y, (OT)lo.z, (OT)lo.w, (OT)hi.x, (OT)hi.y, (OT)hi.z, (OT)hi.w};
            *reinterpret_cast<v4i *>(dst + (size_t)(16 * i) * ld) = *reinterpret_cast<v4i *>(h);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();                               // the patch may be rewritten
}

// The residual add that follows a LayerNorm backward in the recipe, for the kernel that does both (ADD instantiations of
// layernorm_bwd_strip_kernel): y = x1 + dx as a reader of the stored dx would form it, and y's block quantisation.
struct LnAddArgs {
    const void *x1;       // [R, C] x1_dtype
    void *y1;             // [R, C] y1_dtype
    int8_t *q;            // [R, C]
    void *s;              // [R/32, C/32] ST
    int x1_dtype, y1_dtype, rounding;
    uint64_t seed, offset;
};

// ------------------------------------------------------------------------------------------------
// LayerNorm backward over full rows (layernorm.py:197-428; the reference reduces over its 128-column tile only).
// Arithmetic (this library's definition, restated by the CPU checker):
//   xhat = fma(float(qx), sx * rstd[r], -(mean[r] * rstd[r]))     g = float(qg) * sg     wdy = gamma[c] * g
//   per row and 16-column half block: p1 = fma chain of xhat * wdy, p2 = add chain of wdy, ascending columns;
//   per block b = p(columns 0..15) + p(columns 16..31);  per row T_j = sum of b over the blocks j, j+8, ... (ascending),
//   S = ((T0+T1)+(T2+T3)) + ((T4+T5)+(T6+T7));  c1 = S1 / C, c2 = S2 / C;   dx = (wdy - fma(xhat, c1, c2)) * rstd[r]
//   dgamma[c] = sum over rows of g * xhat, dbeta[c] = sum over rows of g  (fp32, order fixed by the kernels below).
//
// Rows of up to 2048 columns take one pass over the inputs (layernorm_bwd_strip_kernel, further down).  Wider rows take
// two launches.  layernorm_bwd_stats_kernel: one wave per (column block, group of LNB_RPW row blocks) walks down its
// column block (the four waves of a workgroup take four adjacent column blocks, i.e. whole 128-byte lines); the lane
// keeps gamma and its dgamma / dbeta accumulators in registers (the cross-lane reduction over the 32 rows of a block
// happens once per wave, not once per block) and stores the per-row block partials b1, b2.
// layernorm_bwd_dx_kernel: one workgroup per 32-row strip first adds its rows' partials (c1, c2), then computes and
// requantises dx block by block; at its end the launch also adds the row groups' dgamma / dbeta partials.
constexpr int LNB_RPW = 4;                 // row blocks per wave of the statistics kernel
constexpr int LNB_DX_WAVES = 16;           // waves per strip of the dx kernel

// Workgroup = 4 waves = 4 adjacent column blocks (whole 128-byte lines per row) x LNB_RPW row blocks.
// part1 / part2: [C/32][R] (a wave stores 32 consecutive rows); pdg / pdb: [C][groups].
template <typename ST>
__global__ __launch_bounds__(NT) void layernorm_bwd_stats_kernel(const int8_t *qx, const ST *sx, const int8_t *qg,
                                                                 const ST *sg, const float *gamma, const float *mean,
                                                                 const float *rstd, int R, int C, int groups, float *part1,
                                                                 float *part2, float *pdg, float *pdb)
{
    __shared__ float cpatch_all[WPB][COLSUM_PATCH];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, SC = C / QB, RB = R / QB, S4 = (SC + WPB - 1) / WPB;
    const int cb = (blockIdx.x % S4) * WPB + wave, grp = blockIdx.x / S4;
    if (cb >= SC) return;                                          // a wave of the last, partial group of column blocks
    float *cpatch = cpatch_all[wave];
    const int col = cb * QB + (lane & 1) * 16;
    const int nrb = (RB - grp * LNB_RPW) < LNB_RPW ? (RB - grp * LNB_RPW) : LNB_RPW;      // uniform
    // everything the wave reads is requested up front, what it needs first (gamma) first
    float w[16];
    Load16<float>::run(gamma + col, w);
    v4i cx[LNB_RPW], cg[LNB_RPW];
    float scx[LNB_RPW], scg[LNB_RPW], mu[LNB_RPW], rs[LNB_RPW];
#pragma unroll
    for (int k = 0; k < LNB_RPW; ++k) {
        const int rb = grp * LNB_RPW + (k < nrb ? k : 0);
        const int row = rb * QB + (lane >> 1);
        const size_t e0 = (size_t)row * C + col;
        cx[k] = *reinterpret_cast<const v4i *>(qx + e0);
        cg[k] = *reinterpret_cast<const v4i *>(qg + e0);
        scx[k] = load_scale(sx, rb * SC + cb);
        scg[k] = load_scale(sg, rb * SC + cb);
        mu[k] = mean[row];
        rs[k] = rstd[row];
    }
    float accg[16], accb[16], o1[LNB_RPW], o2[LNB_RPW];
#pragma unroll
    for (int j = 0; j < 16; ++j) { accg[j] = 0.0f; accb[j] = 0.0f; }
#pragma unroll
    for (int k = 0; k < LNB_RPW; ++k) {
        if (k < nrb) {
            const float a = scx[k] * rs[k], b = -(mu[k] * rs[k]);
            float x[16], g[16];
            codes_to_float16(cx[k], x);
            codes_to_float16(cg[k], g);
            float p1 = 0.0f, p2 = 0.0f;
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const float xh = __builtin_fmaf(x[j], a, b);
                const float gj = g[j] * scg[k];
                const float wdy = w[j] * gj;
                p1 = __builtin_fmaf(xh, wdy, p1);
                p2 = p2 + wdy;
                accg[j] = __builtin_fmaf(gj, xh, accg[j]);
                accb[j] = accb[j] + gj;
            }
            // the two half blocks of a row: the same two operands in both lanes of the pair
            p1 = p1 + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(p1), 0xB1, 0xF, 0xF, false));
            p2 = p2 + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(p2), 0xB1, 0xF, 0xF, false));
            o1[k] = p1; o2[k] = p2;
        }
    }
#pragma unroll
    for (int k = 0; k < LNB_RPW; ++k) {                            // all stores after all loads have been consumed
        if (k < nrb && (lane & 1) == 0) {
            const int row = (grp * LNB_RPW + k) * QB + (lane >> 1);
            part1[(size_t)cb * R + row] = o1[k];
            part2[(size_t)cb * R + row] = o2[k];
        }
    }
    if (pdg) {
        // output of lane j (j even): value index j/4 of column set (j/2)%2
        const size_t dst = ((size_t)cb * QB + ((lane >> 1) & 1) * 16 + (lane >> 2)) * groups + grp;
        const float tg = colsum16_over_rows(accg, lane, cpatch);
        if ((lane & 1) == 0) pdg[dst] = tg;
        const float tb = colsum16_over_rows(accb, lane, cpatch);
        if ((lane & 1) == 0) pdb[dst] = tb;
    }
}

// 64-lane sum, every lane returns it (data-parallel-primitive forms of v_add_f32; a fixed tree: pairs, quads, eights,
// rows of 16, then row 1 += row 0 and row 3 += row 2, then rows 2-3 += rows 0-1; asm for the reason given at wave_max)
__device__ __forceinline__ float wave_sum(float v)
{
    asm volatile("s_nop 1\n\t"
                 "v_add_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1\n\t"
                 "v_add_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1\n\t"
                 "v_add_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1\n\t"
                 "v_add_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1\n\t"
                 "v_add_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
                 "s_nop 1\n\t"
                 "v_add_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
                 : "+v"(v));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

template <typename ST>
__global__ __launch_bounds__(WAVE * LNB_DX_WAVES) void layernorm_bwd_dx_kernel(
    const int8_t *qx, const ST *sx, const int8_t *qg, const ST *sg, const float *gamma, const float *mean,
    const float *rstd, int R, int C, int rounding, uint64_t seed, uint64_t offset, const float *part1, const float *part2,
    int8_t *qdx, ST *sdx, const float *pdg, const float *pdb, int groups, float *dgamma, float *dbeta)
{
    extern __shared__ __attribute__((aligned(16))) float lds_f[];  // gamma[C], c1[32], c2[32], T[2][8][32]
    float *gl = lds_f, *cs = lds_f + C, *tj = cs + 2 * QB;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int SC = C / QB, rb = blockIdx.x;
    const int row = rb * QB + (lane >> 1);
    // A wave's blocks are cb = wave, wave + 16, ...: up to DXB of them are requested at once, before anything else; they
    // are computed in arrival order and their results stored together at the end (no wait follows a store, except
    // between the batches of rows wider than 16 * DXB blocks).
    constexpr int DXB = 4;
    v4i cx[DXB], cg[DXB];
    float scx[DXB], scg[DXB];
    auto request_batch = [&](int cb0) {
        static_for<0, DXB>([&](auto i_c) {
            constexpr int I = decltype(i_c)::value;
            const int cb = cb0 + I * LNB_DX_WAVES;
            if (cb < SC) {
                const size_t e0 = (size_t)row * C + cb * QB + (lane & 1) * 16;
                cx[I] = *reinterpret_cast<const v4i *>(qx + e0);
                cg[I] = *reinterpret_cast<const v4i *>(qg + e0);
                scx[I] = load_scale(sx, rb * SC + cb);
                scg[I] = load_scale(sg, rb * SC + cb);
            }
        });
    };
    request_batch(wave);
    const float mu = mean[row], rs = rstd[row];
    for (int c = threadIdx.x * 4; c < C; c += WAVE * LNB_DX_WAVES * 4)
        *reinterpret_cast<v4f *>(gl + c) = *reinterpret_cast<const v4f *>(gamma + c);
    if (threadIdx.x < 512) {
        // Row sums of the block partials.  Threads 0..255: S1, 256..511: S2; thread (j, r) adds the blocks j, j+8, ... of
        // row r in ascending order (absent blocks contribute +0, which changes no bit; 8 independent loads at a time).
        const int t = threadIdx.x & 255, j = t >> 5, r = t & 31, which = threadIdx.x >> 8;
        const float *part = (which ? part2 : part1) + rb * QB + r;
        float acc = 0.0f;
        for (int cb0 = 0; cb0 < SC; cb0 += 64) {
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) { const int cb = cb0 + j + 8 * i; v[i] = cb < SC ? part[(size_t)cb * R] : 0.0f; }
#pragma unroll
            for (int i = 0; i < 8; ++i) acc = acc + v[i];
        }
        tj[(which * 8 + j) * QB + r] = acc;
    }
    // dgamma / dbeta: one column per wave of the whole launch: the row groups' partials, one per lane, then a wave sum
    if (pdg) {
        for (int c = blockIdx.x * LNB_DX_WAVES + wave; c < C; c += gridDim.x * LNB_DX_WAVES) {
            float tg = 0.0f, tb = 0.0f;
            for (int gi = lane; gi < groups; gi += WAVE) { tg = tg + pdg[(size_t)c * groups + gi]; tb = tb + pdb[(size_t)c * groups + gi]; }
            tg = wave_sum(tg);
            tb = wave_sum(tb);
            if (lane == 0) {
                if (dgamma) dgamma[c] = tg;
                if (dbeta) dbeta[c] = tb;
            }
        }
    }
    __syncthreads();
    if (threadIdx.x < 2 * QB) {
        // S = ((T0+T1)+(T2+T3)) + ((T4+T5)+(T6+T7)),  c = S / C
        const float *T = tj + (threadIdx.x >> 5) * 8 * QB + (threadIdx.x & 31);
        const float S = ((T[0] + T[QB]) + (T[2 * QB] + T[3 * QB])) + ((T[4 * QB] + T[5 * QB]) + (T[6 * QB] + T[7 * QB]));
        cs[threadIdx.x] = S / (float)C;
    }
    __syncthreads();
    const float k1 = cs[lane >> 1], k2 = cs[QB + (lane >> 1)];
    const float b = -(mu * rs);
    for (int cb0 = wave; cb0 < SC; cb0 += DXB * LNB_DX_WAVES) {
        if (cb0 != wave) request_batch(cb0);                       // rows of more than 64 blocks only
        v4i out[DXB];
        float so[DXB];
        static_for<0, DXB>([&](auto i_c) {
            constexpr int I = decltype(i_c)::value;
            const int cb = cb0 + I * LNB_DX_WAVES;
            if (cb >= SC) return;                                  // uniform
            const int col = cb * QB + (lane & 1) * 16;
            const size_t e0 = (size_t)row * C + col;
            const float a = scx[I] * rs, sgk = scg[I];
            float x[16], g[16], w[16];
            Load16<float>::run(gl + col, w);
            codes_to_float16(cx[I], x);
            codes_to_float16(cg[I], g);
#pragma unroll
            for (int jj = 0; jj < 16; ++jj) {
                const float xh = __builtin_fmaf(x[jj], a, b);
                const float wdy = w[jj] * (g[jj] * sgk);
                x[jj] = (wdy - __builtin_fmaf(xh, k1, k2)) * rs;
            }
            out[I] = quantize16(x, 0.0f, rounding, seed, offset, e0, &so[I]);
        });
        static_for<0, DXB>([&](auto i_c) {
            constexpr int I = decltype(i_c)::value;
            const int cb = cb0 + I * LNB_DX_WAVES;
            if (cb >= SC) return;
            *reinterpret_cast<v4i *>(qdx + (size_t)row * C + cb * QB + (lane & 1) * 16) = out[I];
            if (lane == 0) store_scale(sdx, rb * SC + cb, so[I]);
        });
    }
}

// LayerNorm backward of rows of up to LNS_WAVES * LNS_BPW column blocks (2048 columns) in ONE pass over the inputs: a
// workgroup owns a 32-row strip and keeps the strip's codes in registers (wave w: column blocks w, w + 16, ...) from the
// first read to the store of dx.  Phase 1 forms the per-row block partials of sum(xhat * wdy) and sum(wdy) (into LDS)
// and, when dgamma / dbeta are wanted, the strip's column sums of g * xhat and g (to pdg / pdb [R/32][C], finished by
// layernorm_bwd_colsum_finish_kernel); the row sums are then added in the order given above (T_j over the blocks j,
// j + 8, ..., the tree over T_0..T_7), and phase 2 converts the codes again (cheaper than keeping 32 floats per block
// alive), forms dx and requantises it.  Same arithmetic, bit for bit, as the two-launch form above, which stays for
// wider rows.
// ADD: the residual add that follows in the recipe (add.py:164-211) happens here as well: dx is requantised exactly as
// without ADD, but instead of being stored it is dequantised again as a reader of the stored tensor would (codes x the
// scale rounded to ST), added to x1, and the sum and its own block quantisation are what leaves -- the same bits as this
// kernel without ADD followed by add_kernel, without dx's round trip through memory and the second launch.
constexpr int LNS_WAVES = 16, LNS_BPW = 4;
constexpr int LNS_PATCH_ADD = QB * ADD_PITCH;      // floats per wave: the sum's patch, also used for the column sums
static_assert(LNS_PATCH_ADD >= COLSUM_PATCH, "one patch per wave serves both");
template <typename ST, bool WANT_DW, bool ADD>
__global__ __launch_bounds__(WAVE * LNS_WAVES) void layernorm_bwd_strip_kernel(
    const int8_t *qx, const ST *sx, const int8_t *qg, const ST *sg, const float *gamma, const float *mean,
    const float *rstd, int R, int C, int rounding, uint64_t seed, uint64_t offset, int8_t *qdx, ST *sdx, float *pdg,
    float *pdb, LnAddArgs ad)
{
    extern __shared__ __attribute__((aligned(16))) float lds_f[];  // gamma[C], part[2][C/32][32], T[2][8][32], c[2][32], patches
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int SC = C / QB, rb = blockIdx.x;
    float *gl = lds_f, *part = gl + C, *tj = part + 2 * SC * QB, *cs = tj + 2 * 8 * QB;
    float *cpatch = cs + 2 * QB + wave * (ADD ? LNS_PATCH_ADD : COLSUM_PATCH);   // (only with WANT_DW or ADD)
    const int row = rb * QB + (lane >> 1);
    v4i cx[LNS_BPW], cg[LNS_BPW];
    float scx[LNS_BPW], scg[LNS_BPW];
    static_for<0, LNS_BPW>([&](auto i_c) {
        constexpr int I = decltype(i_c)::value;
        const int cb = wave + I * LNS_WAVES;
        if (cb < SC) {
            const size_t e0 = (size_t)row * C + cb * QB + (lane & 1) * 16;
            cx[I] = *reinterpret_cast<const v4i *>(qx + e0);
            cg[I] = *reinterpret_cast<const v4i *>(qg + e0);
            scx[I] = load_scale(sx, rb * SC + cb);
            scg[I] = load_scale(sg, rb * SC + cb);
        }
    });
    const float mu = mean[row], rs = rstd[row];
    for (int c = threadIdx.x * 4; c < C; c += WAVE * LNS_WAVES * 4)
        *reinterpret_cast<v4f *>(gl + c) = *reinterpret_cast<const v4f *>(gamma + c);
    __syncthreads();
    const float b = -(mu * rs);
    // phase 1: block partials of the two row sums; column sums of the strip
    static_for<0, LNS_BPW>([&](auto i_c) {
        constexpr int I = decltype(i_c)::value;
        const int cb = wave + I * LNS_WAVES;
        if (cb >= SC) return;                                      // uniform
        const int col = cb * QB + (lane & 1) * 16;
        const float a = scx[I] * rs, sgk = scg[I];
        float x[16], g[16], w[16];
        Load16<float>::run(gl + col, w);
        codes_to_float16(cx[I], x);
        codes_to_float16(cg[I], g);
        float p1 = 0.0f, p2 = 0.0f;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const float xh = __builtin_fmaf(x[j], a, b);
            const float gj = g[j] * sgk;
            const float wdy = w[j] * gj;
            p1 = __builtin_fmaf(xh, wdy, p1);
            p2 = p2 + wdy;
            if (WANT_DW) { x[j] = gj * xh; g[j] = gj; }            // this strip's terms of dgamma / dbeta
        }
        // the two half blocks of a row: the same two operands in both lanes of the pair
        p1 = p1 + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(p1), 0xB1, 0xF, 0xF, false));
        p2 = p2 + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(p2), 0xB1, 0xF, 0xF, false));
        if ((lane & 1) == 0) {
            part[cb * QB + (lane >> 1)] = p1;
            part[(SC + cb) * QB + (lane >> 1)] = p2;
        }
        if (WANT_DW) {
            // output of lane j (j even): value index j/4 of column set (j/2)%2
            const size_t dst = (size_t)rb * C + cb * QB + ((lane >> 1) & 1) * 16 + (lane >> 2);
            const float tg = colsum16_over_rows(x, lane, cpatch);
            if ((lane & 1) == 0) pdg[dst] = tg;
            const float tb = colsum16_over_rows(g, lane, cpatch);
            if ((lane & 1) == 0) pdb[dst] = tb;
        }
        __builtin_amdgcn_sched_barrier(0);                         // block by block: interleaved, their temporaries do not fit
    });
    __syncthreads();
    if (threadIdx.x < 512) {
        // threads 0..255: first sum, 256..511: second; thread (j, r) adds the blocks j, j+8, ... of row r in ascending order
        const int t = threadIdx.x & 255, j = t >> 5, r = t & 31, which = threadIdx.x >> 8;
        const float *src = part + (size_t)which * SC * QB + r;
        float acc = 0.0f;
        for (int cb = j; cb < SC; cb += 8) acc = acc + src[cb * QB];
        tj[(which * 8 + j) * QB + r] = acc;
    }
    __syncthreads();
    if (threadIdx.x < 2 * QB) {
        // S = ((T0+T1)+(T2+T3)) + ((T4+T5)+(T6+T7)),  c = S / C
        const float *T = tj + (threadIdx.x >> 5) * 8 * QB + (threadIdx.x & 31);
        const float S = ((T[0] + T[QB]) + (T[2 * QB] + T[3 * QB])) + ((T[4 * QB] + T[5 * QB]) + (T[6 * QB] + T[7 * QB]));
        cs[threadIdx.x] = S / (float)C;
    }
    __syncthreads();
    const float k1 = cs[lane >> 1], k2 = cs[QB + (lane >> 1)];
    // phase 2: dx of the blocks still held as codes
    static_for<0, LNS_BPW>([&](auto i_c) {
        constexpr int I = decltype(i_c)::value;
        const int cb = wave + I * LNS_WAVES;
        if (cb >= SC) return;                                      // uniform
        const int col = cb * QB + (lane & 1) * 16;
        const size_t e0 = (size_t)row * C + col;
        const float a = scx[I] * rs, sgk = scg[I];
        float x[16], g[16], w[16];
        v4i raw[4];                                                // (ADD) the lane's 16 values of x1 as they lie in memory
        if (ADD) {
            if (ad.x1_dtype == JF_FP_F32) {
#pragma unroll
                for (int k = 0; k < 4; ++k) raw[k] = reinterpret_cast<const v4i *>(reinterpret_cast<const float *>(ad.x1) + e0)[k];
            } else {
#pragma unroll
                for (int k = 0; k < 2; ++k) raw[k] = reinterpret_cast<const v4i *>(reinterpret_cast<const uint16_t *>(ad.x1) + e0)[k];
            }
        }
        Load16<float>::run(gl + col, w);
        // (opaque copies: otherwise the optimiser keeps phase 1's 32 converted values per block alive across the barriers,
        // in registers this kernel does not have)
        v4i kx = cx[I], kg = cg[I];
        asm volatile("" : "+v"(kx), "+v"(kg));
        codes_to_float16(kx, x);
        codes_to_float16(kg, g);
#pragma unroll
        for (int jj = 0; jj < 16; ++jj) {
            const float xh = __builtin_fmaf(x[jj], a, b);
            const float wdy = w[jj] * (g[jj] * sgk);
            x[jj] = (wdy - __builtin_fmaf(xh, k1, k2)) * rs;
        }
        float so;
        const v4i out = quantize16(x, 0.0f, rounding, seed, offset, e0, &so);
        if (!ADD) {
            *reinterpret_cast<v4i *>(qdx + e0) = out;
            if (lane == 0) store_scale(sdx, rb * SC + cb, so);
        } else {
            float y[16];
            unpack16(out, (float)(ST)so, x);                       // dx as stored
            if (ad.x1_dtype == JF_FP_F32) {
#pragma unroll
                for (int k = 0; k < 16; ++k) y[k] = __int_as_float(raw[k >> 2][k & 3]);
            } else if (ad.x1_dtype == JF_FP_F16) {
#pragma unroll
                for (int k = 0; k < 16; ++k)
                    y[k] = (float)__builtin_bit_cast(half_t, (uint16_t)((uint32_t)raw[k >> 3][(k >> 1) & 3] >> (16 * (k & 1))));
            } else {
#pragma unroll
                for (int k = 0; k < 16; ++k)
                    y[k] = __uint_as_float(((uint32_t)raw[k >> 3][(k >> 1) & 3] >> (16 * (k & 1))) << 16);
            }
#pragma unroll
            for (int k = 0; k < 16; ++k) y[k] = y[k] + x[k];
            const size_t b0 = (size_t)rb * QB * C + cb * QB;       // the block's first element
            if (ad.y1_dtype == JF_FP_F32) store_block_rows(cpatch, y, reinterpret_cast<float *>(ad.y1) + b0, C, lane);
            else if (ad.y1_dtype == JF_FP_F16) store_block_rows(cpatch, y, reinterpret_cast<half_t *>(ad.y1) + b0, C, lane);
            else store_block_rows(cpatch, y, reinterpret_cast<__bf16 *>(ad.y1) + b0, C, lane);
            float s2;
            const v4i c2 = quantize16(y, 0.0f, ad.rounding, ad.seed, ad.offset, e0, &s2);
            *reinterpret_cast<v4i *>(ad.q + e0) = c2;
            if (lane == 0) store_scale(reinterpret_cast<ST *>(ad.s), rb * SC + cb, s2);
        }
        __builtin_amdgcn_sched_barrier(0);
    });
}

// dgamma / dbeta from the per-strip column sums (pdg, pdb: [strips][C]).  Workgroup (32 columns, which array) of 1024
// threads; thread (g, column) adds the strips g, g+32, ... in ascending order (8 independent loads at a time: one round
// trip for 256 strips), then thread (0, column) adds the 32 partial sums in ascending order.
__global__ __launch_bounds__(1024) void layernorm_bwd_colsum_finish_kernel(const float *pdg, const float *pdb, int strips,
                                                                           int C, float *dgamma, float *dbeta)
{
    __shared__ float red[32][QB + 1];
    const float *src = blockIdx.y ? pdb : pdg;
    float *dst = blockIdx.y ? dbeta : dgamma;
    if (!dst) return;                                              // uniform
    const int k = threadIdx.x & 31, c = blockIdx.x * QB + k, g = threadIdx.x >> 5;
    float acc = 0.0f;
    for (int s0 = g; s0 < strips; s0 += 256) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) { const int s = s0 + 32 * i; v[i] = s < strips ? src[(size_t)s * C + c] : 0.0f; }
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = acc + v[i];
    }
    red[g][k] = acc;
    __syncthreads();
    if (g == 0) {
        float t = red[0][k];
#pragma unroll
        for (int i = 1; i < 32; ++i) t = t + red[i][k];
        dst[c] = t;
    }
}

// Column sums of a block tensor's 32-row strips (the bias gradient of a linear layer is the column sum of its output
// gradient; the reference sketches it as G8.sum(0), JetfireGEMMKernel/BlockQuantize/QBlockLinear.py:63-66).
// strip term t[rb][c] = float(sum of the 32 codes of column c in row block rb) * s[rb][c/32]: the integer sum is exact,
// the product rounds once.  One wave: 256 columns (4 per lane, whole 256-byte row segments) of one strip, all 32 row
// loads in flight at once.  The strips' terms are then added by layernorm_bwd_colsum_finish_kernel in its fixed order.
template <typename ST>
__global__ __launch_bounds__(NT) void colsum_strip_kernel(const int8_t *q, const ST *s, int R, int C, float *terms)
{
    const int lane = threadIdx.x & 63, SC = C / QB, CG = (C + 255) / 256;
    const int item = blockIdx.x * WPB + (threadIdx.x >> 6);        // (strip, 256-column group)
    if (item >= (R / QB) * CG) return;
    const int rb = item / CG, c0 = (item - rb * CG) * 256 + lane * 4;
    if (c0 >= C) return;
    const int8_t *src = q + (size_t)rb * QB * C + c0;
    int w[QB];
#pragma unroll
    for (int i = 0; i < QB; ++i) w[i] = *reinterpret_cast<const int *>(src + (size_t)i * C);
    int a0 = 0, a1 = 0, a2 = 0, a3 = 0;
#pragma unroll
    for (int i = 0; i < QB; ++i) { a0 += (w[i] << 24) >> 24; a1 += (w[i] << 16) >> 24; a2 += (w[i] << 8) >> 24; a3 += w[i] >> 24; }
    const float sc = load_scale(s, rb * SC + c0 / QB);
    *reinterpret_cast<v4f *>(terms + (size_t)rb * C + c0) = v4f{(float)a0 * sc, (float)a1 * sc, (float)a2 * sc, (float)a3 * sc};
}

// add.py:29-162 / add_mean_var.py:28-177
// The sum leaves through a wave-private LDS patch in whole rows (store_block_rows).
// rowsum / rowsq: [C/32][R] (a wave stores the 32 consecutive rows of its block).
template <typename T, typename ST, typename OT>
__global__ __launch_bounds__(NT) void add_kernel(const T *x1, const int8_t *q2, const ST *s2, int R, int C,
                                                 int rounding, uint64_t seed, uint64_t offset, OT *y1, int8_t *q,
                                                 ST *s, float *rowsum, float *rowsq)
{
    __shared__ __attribute__((aligned(16))) float ypatch_all[WPB][QB * ADD_PITCH];
    __shared__ __attribute__((aligned(16))) unsigned char line_patches[2 * QB * LINE_PITCH];
    float *ypatch = ypatch_all[threadIdx.x >> 6];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int SC = C / QB, SG = (SC + WPB - 1) / WPB, ngrp = (R / QB) * SG;
    GroupLineStore lines(line_patches, lane, wave);
    // a workgroup: four adjacent column blocks of one row block (a group), so that the codes leave in whole lines
    for (int grp = blockIdx.x; grp < ngrp; grp += gridDim.x)
    {
        const int rbg = grp / SG, cg = grp - rbg * SG, cbg = cg * WPB + wave;
        if (cbg >= SC) {                                           // (wave-uniform) beyond the row's end: the barrier only
            lines.store(v4i{0, 0, 0, 0}, q, rbg, cg, C);
            continue;
        }
        BlockPos pos(rbg * SC + cbg, SC, C, lane);
        float a[16], b[16];
        Load16<T>::run(x1 + pos.e0, a);
        unpack16(*reinterpret_cast<const v4i *>(q2 + pos.e0), load_scale(s2, pos.rb * SC + pos.cb), b);
#pragma unroll
        for (int k = 0; k < 16; ++k) a[k] = a[k] + b[k];
        store_block_rows(ypatch, a, y1 + (size_t)pos.rb * QB * C + pos.cb * QB, C, lane);
        if (rowsum) {
            float t1 = 0.0f, t2 = 0.0f;
#pragma unroll
            for (int k = 0; k < 16; ++k) { t1 = t1 + a[k]; t2 = __builtin_fmaf(a[k], a[k], t2); }
            const float o1 = __shfl_xor(t1, 1, WAVE), o2 = __shfl_xor(t2, 1, WAVE);
            if ((lane & 1) == 0) {
                rowsum[(size_t)pos.cb * R + pos.row] = t1 + o1;     // columns 0..15 partial + 16..31 partial
                rowsq[(size_t)pos.cb * R + pos.row] = t2 + o2;
            }
        }
        float scale;
        v4i codes = quantize16(a, 0.0f, rounding, seed, offset, pos.e0, &scale);
        lines.store(codes, q, rbg, cg, C);
        if (lane == 0) store_scale(s, pos.rb * SC + pos.cb, scale);
    }
}

// ------------------------------------------------------------------------------------------------
static inline int grid_for_blocks(int R, int C)
{
    const long nblk = (long)(R / QB) * (C / QB);
    long g = (nblk + WPB - 1) / WPB;
    const long cap = 256L * 32;                    // 32 workgroups per CU is plenty of waves in flight
    return (int)(g < cap ? g : cap);
}

// kernels whose workgroup takes a group of four adjacent column blocks of one row block per step
static inline int grid_for_workgroup_groups(int R, int C)
{
    const long g = (long)(R / QB) * ((C / QB + WPB - 1) / WPB), cap = 256L * 32;
    return (int)(g < cap ? g : cap);
}

static int check_block_tensor(const void *q, const void *s, int R, int C, int scale_dtype)
{
    if (!q || !s) return JF_ERR_NULL;
    if (!mult32(R) || !mult32(C)) return JF_ERR_SHAPE;
    if (scale_dtype != JF_SCALE_F16 && scale_dtype != JF_SCALE_F32) return JF_ERR_ENUM;
    if (!aligned16(q)) return JF_ERR_ALIGN;
    return JF_OK;
}

// per-column fp32 vectors (gamma, beta) are kept in LDS by the LayerNorm kernels: up to 64 KiB of them, i.e. rows of up
// to 8192 columns forward and 16320 backward
constexpr size_t LDS_VECTOR_LIMIT = 64 * 1024;

static inline bool rounding_ok(int r) { return r >= JF_ROUND_NEAREST && r <= JF_ROUND_STOCHASTIC_TRUNC; }

}  // namespace jf

using namespace jf;

// mean and 1/sqrt(variance) of every row from its per-32-column partial sums (rowsum, rowsq: [parts][R], what add_kernel
// leaves): the partials are added in ascending order, var = E[y^2] - mean^2, no epsilon (add_mean_var.py:219-221).
constexpr int RSF_ROWS = 32;                       // rows per workgroup
__global__ __launch_bounds__(256) void rowstats_finish_kernel(const float *rowsum, const float *rowsq, int R, int parts,
                                                              float n, float *mean, float *rstd)
{
    // the partial sums of RSF_ROWS consecutive rows are fetched by all threads (128 contiguous bytes per part and array),
    // then one thread per row (and array) adds its row's partials in ascending order from LDS
    extern __shared__ float rsf_lds[];                                // [2][parts][RSF_ROWS]
    const int r0 = blockIdx.x * RSF_ROWS;
    const int rows = (R - r0) < RSF_ROWS ? (R - r0) : RSF_ROWS;
    const int count = parts * RSF_ROWS;
    for (int i = threadIdx.x; i < count; i += 256) {
        const int j = i / RSF_ROWS, r = i % RSF_ROWS;
        if (r < rows) {
            rsf_lds[i] = rowsum[(size_t)j * R + r0 + r];
            rsf_lds[count + i] = rowsq[(size_t)j * R + r0 + r];
        }
    }
    __syncthreads();
    const int row = threadIdx.x & (RSF_ROWS - 1), which = threadIdx.x / RSF_ROWS;     // which: 0 = sums, 1 = squares
    float acc = 0.0f;
    if (which < 2 && row < rows) {
        const float *p = rsf_lds + which * count + row;
        for (int j = 0; j < parts; ++j) acc = acc + p[j * RSF_ROWS];
    }
    __syncthreads();
    if (which == 1 && row < rows) rsf_lds[row] = acc;                 // hand the sum of squares to the row's other thread
    __syncthreads();
    if (which == 0 && row < rows) {
        const float m = acc / n;
        const float var = rsf_lds[row] / n - m * m;
        mean[r0 + row] = m;
        rstd[r0 + row] = 1.0f / __builtin_sqrtf(var);
    }
}

#define JF_LAUNCH(kern, grid, smem, st, ...)                         \
    do {                                                             \
        if (!device_is_gfx950()) return JF_ERR_DEVICE;               \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(NT), smem, st, __VA_ARGS__); \
        return (int)hipGetLastError();                               \
    } while (0)

extern "C" {

int jf_quantize(const void *x, int x_dtype, int R, int C, int8_t *q, void *s, int8_t *qT,
                int scale_dtype, int rounding, uint64_t seed, uint64_t offset, float amax_eps, jf_stream_t stream)
{
    int rc = check_block_tensor(q, s, R, C, scale_dtype);
    if (rc) return rc;
    if (!x) return JF_ERR_NULL;
    if (!rounding_ok(rounding) || x_dtype < JF_FP_F16 || x_dtype > JF_FP_BF16) return JF_ERR_ENUM;
    if (!aligned16(x) || (qT && !aligned16(qT))) return JF_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const int groups = quantize_groups(R, C, qT != nullptr);
    const int grid = groups < 256 * 32 ? groups : 256 * 32;       // (a multiple of 32, which the transposed walk needs)
    QuantSrc src = {};
    src.x[0] = x; src.ldx[0] = C; src.end[0] = C; src.n = 1;
#define JF_Q(T, ST)                                                                                          \
    JF_LAUNCH((quantize_kernel<T, ST>), grid, 0, st, src, R, C, q, (ST *)s, qT, rounding, seed, offset, amax_eps)
    if (scale_dtype == JF_SCALE_F16) {
        if (x_dtype == JF_FP_F32) JF_Q(float, half_t);
        if (x_dtype == JF_FP_F16) JF_Q(half_t, half_t);
        JF_Q(__bf16, half_t);
    } else {
        if (x_dtype == JF_FP_F32) JF_Q(float, float);
        if (x_dtype == JF_FP_F16) JF_Q(half_t, float);
        JF_Q(__bf16, float);
    }
#undef JF_Q
}

int jf_quantize_slabs(const void *const *x, const int *ldx, const int *widths, int nslabs, int x_dtype, int R,
                      int8_t *q, void *s, int scale_dtype, int rounding, uint64_t seed, uint64_t offset, float amax_eps,
                      jf_stream_t stream)
{
    if (!x || !ldx || !widths) return JF_ERR_NULL;
    if (nslabs < 1 || nslabs > QSRC_MAX) return JF_ERR_SHAPE;
    if (!rounding_ok(rounding) || x_dtype < JF_FP_F16 || x_dtype > JF_FP_BF16) return JF_ERR_ENUM;
    const size_t xbytes = x_dtype == JF_FP_F32 ? 4 : 2;
    QuantSrc src = {};
    int C = 0;
    for (int k = 0; k < nslabs; ++k) {
        if (!x[k]) return JF_ERR_NULL;
        if (!mult32(widths[k]) || ldx[k] < widths[k]) return JF_ERR_SHAPE;
        if (!aligned16(x[k]) || ((size_t)ldx[k] * xbytes) % 16) return JF_ERR_ALIGN;
        C += widths[k];
        src.x[k] = x[k]; src.ldx[k] = ldx[k]; src.end[k] = C;
    }
    src.n = nslabs;
    int rc = check_block_tensor(q, s, R, C, scale_dtype);
    if (rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    const int grid = grid_for_blocks(R, C);
#define JF_Q(T, ST)                                                                                          \
    JF_LAUNCH((quantize_kernel<T, ST>), grid, 0, st, src, R, C, q, (ST *)s, (int8_t *)nullptr, rounding, seed, offset, amax_eps)
    if (scale_dtype == JF_SCALE_F16) {
        if (x_dtype == JF_FP_F32) JF_Q(float, half_t);
        if (x_dtype == JF_FP_F16) JF_Q(half_t, half_t);
        JF_Q(__bf16, half_t);
    } else {
        if (x_dtype == JF_FP_F32) JF_Q(float, float);
        if (x_dtype == JF_FP_F16) JF_Q(half_t, float);
        JF_Q(__bf16, float);
    }
#undef JF_Q
}

int jf_dequantize(const int8_t *q, const void *s, int R, int C, int scale_dtype, void *out, int out_dtype, jf_stream_t stream)
{
    int rc = check_block_tensor(q, s, R, C, scale_dtype);
    if (rc) return rc;
    if (!out) return JF_ERR_NULL;
    if (out_dtype != JF_FP_F32 && out_dtype != JF_FP_F16 && out_dtype != JF_FP_BF16) return JF_ERR_ENUM;
    if (!aligned16(out)) return JF_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const int grid = grid_for_blocks(R, C);
#define JF_DQ(ST, OT) JF_LAUNCH((dequantize_kernel<ST, OT>), grid, 0, st, q, (const ST *)s, R, C, (OT *)out)
    if (scale_dtype == JF_SCALE_F16) {
        if (out_dtype == JF_FP_F32) JF_DQ(half_t, float);
        if (out_dtype == JF_FP_F16) JF_DQ(half_t, half_t);
        JF_DQ(half_t, __bf16);
    }
    if (out_dtype == JF_FP_F32) JF_DQ(float, float);
    if (out_dtype == JF_FP_F16) JF_DQ(float, half_t);
    JF_DQ(float, __bf16);
#undef JF_DQ
}

int jf_rowstats(const int8_t *q, const void *s, int R, int C, int scale_dtype, float eps, float *mean, float *rstd,
                jf_stream_t stream)
{
    int rc = check_block_tensor(q, s, R, C, scale_dtype);
    if (rc) return rc;
    if (!mean || !rstd) return JF_ERR_NULL;
    const size_t smem = (size_t)2 * QB * (C / QB) * sizeof(int);
    if (smem > 64 * 1024) return JF_ERR_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    if (scale_dtype == JF_SCALE_F16)
        JF_LAUNCH(rowstats_kernel<half_t>, R / QB, smem, st, q, (const half_t *)s, R, C, eps, mean, rstd);
    JF_LAUNCH(rowstats_kernel<float>, R / QB, smem, st, q, (const float *)s, R, C, eps, mean, rstd);
}

int jf_layernorm_fwd(const int8_t *q, const void *s, const float *gamma, const float *beta, const float *mean,
                     const float *rstd, int R, int C, int scale_dtype, int8_t *qy, void *sy, jf_stream_t stream)
{
    int rc = check_block_tensor(q, s, R, C, scale_dtype);
    if (rc) return rc;
    if (!gamma || !mean || !rstd || !qy || !sy) return JF_ERR_NULL;
    if (!aligned16(qy) || !aligned16(gamma) || (beta && !aligned16(beta))) return JF_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const int grid = ((C / QB + WPB - 1) / WPB) * ((R / QB + CW_ROWS - 1) / CW_ROWS);
    const size_t smem = 0;
    if (scale_dtype == JF_SCALE_F16)
        JF_LAUNCH(layernorm_fwd_kernel<half_t>, grid, smem, st, q, (const half_t *)s, gamma, beta, mean, rstd, R, C, qy,
                  (half_t *)sy);
    JF_LAUNCH(layernorm_fwd_kernel<float>, grid, smem, st, q, (const float *)s, gamma, beta, mean, rstd, R, C, qy,
              (float *)sy);
}

// workspace: per-row block partials [2][C/32][R] and per-row-group column partials [2][C][groups]
static inline int lnb_groups(int R) { return (R / QB + LNB_RPW - 1) / LNB_RPW; }

size_t jf_layernorm_bwd_workspace_bytes(int R, int C)
{
    if (R <= 0 || C <= 0) return 0;
    return ((size_t)2 * R * (C / QB) + (size_t)2 * lnb_groups(R) * C) * sizeof(float);
}

}  // extern "C"

// rows of up to 2048 columns: one pass over the inputs, the strip's codes held in registers.  add != nullptr: the residual
// add that follows happens in the same kernel (qdx / sdx are not written).
static int launch_layernorm_bwd_strip(const int8_t *qx, const void *sx, const int8_t *qg, const void *sg, const float *gamma,
                                      const float *mean, const float *rstd, int R, int C, int scale_dtype, int rounding,
                                      uint64_t seed, uint64_t offset, int8_t *qdx, void *sdx, float *dgamma, float *dbeta,
                                      void *workspace, const LnAddArgs *add, hipStream_t st)
{
    const bool want_dw = dgamma || dbeta;
    const int SC = C / QB;
    float *sdg = (float *)workspace, *sdb = sdg + (size_t)(R / QB) * C;      // [R/32][C] each: fits the workspace size
    const size_t patch = add ? LNS_PATCH_ADD : want_dw ? COLSUM_PATCH : 0;
    const size_t lds = ((size_t)C + 2 * SC * QB + 2 * 8 * QB + 2 * QB + LNS_WAVES * patch) * sizeof(float);
    const LnAddArgs ad = add ? *add : LnAddArgs{};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return JF_ERR_DEVICE;
#define JF_LNS(ST, DW, ADD)                                                                                            \
    do {                                                                                                               \
        auto kern = layernorm_bwd_strip_kernel<ST, DW, ADD>;                                                           \
        static std::atomic<bool> opted_in[MAX_DEVICES] = {};      /* more than 64 KiB of LDS: once per device */        \
        if (lds > 64 * 1024 && !opted_in[dev].load(std::memory_order_acquire)) {                                       \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                                   \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);                \
            if (e != hipSuccess) return (int)e;                                                                        \
            opted_in[dev].store(true, std::memory_order_release);                                                      \
        }                                                                                                              \
        hipLaunchKernelGGL(kern, dim3(R / QB), dim3(WAVE * LNS_WAVES), lds, st, qx, (const ST *)sx, qg,                \
                           (const ST *)sg, gamma, mean, rstd, R, C, rounding, seed, offset, qdx, (ST *)sdx,            \
                           DW ? sdg : nullptr, DW ? sdb : nullptr, ad);                                                \
    } while (0)
#define JF_LNS_DW(ST, ADD) do { if (want_dw) JF_LNS(ST, true, ADD); else JF_LNS(ST, false, ADD); } while (0)
    if (scale_dtype == JF_SCALE_F16) { if (add) JF_LNS_DW(half_t, true); else JF_LNS_DW(half_t, false); }
    else { if (add) JF_LNS_DW(float, true); else JF_LNS_DW(float, false); }
#undef JF_LNS_DW
#undef JF_LNS
    if (want_dw)
        hipLaunchKernelGGL(layernorm_bwd_colsum_finish_kernel, dim3(SC, 2), dim3(1024), 0, st, sdg, sdb, R / QB, C, dgamma, dbeta);
    return (int)hipGetLastError();
}

extern "C" {

int jf_layernorm_bwd_add(const int8_t *qx, const void *sx, const int8_t *qg, const void *sg, const float *gamma,
                         const float *mean, const float *rstd, int R, int C, int scale_dtype, int rounding, uint64_t seed,
                         uint64_t offset, const void *x1, int x1_dtype, int add_rounding, uint64_t add_seed,
                         uint64_t add_offset, void *y1, int y1_dtype, int8_t *q, void *s, float *dgamma, float *dbeta,
                         void *workspace, size_t workspace_bytes, jf_stream_t stream)
{
    int rc = check_block_tensor(qx, sx, R, C, scale_dtype);
    if (rc) return rc;
    if ((rc = check_block_tensor(qg, sg, R, C, scale_dtype))) return rc;
    if (!gamma || !mean || !rstd || !x1 || !y1 || !q || !s) return JF_ERR_NULL;
    if (!rounding_ok(rounding) || !rounding_ok(add_rounding)) return JF_ERR_ENUM;
    if (x1_dtype < JF_FP_F16 || x1_dtype > JF_FP_BF16 || y1_dtype < JF_FP_F16 || y1_dtype > JF_FP_BF16) return JF_ERR_ENUM;
    if (!aligned16(gamma) || !aligned16(x1) || !aligned16(y1) || !aligned16(q)) return JF_ERR_ALIGN;
    if (C / QB > LNS_WAVES * LNS_BPW) return JF_ERR_SHAPE;         // wider rows: jf_layernorm_bwd, then jf_add
    if (!workspace || workspace_bytes < jf_layernorm_bwd_workspace_bytes(R, C)) return JF_ERR_WORKSPACE;
    if (!aligned16(workspace)) return JF_ERR_ALIGN;
    if (!device_is_gfx950()) return JF_ERR_DEVICE;
    LnAddArgs ad;
    ad.x1 = x1; ad.y1 = y1; ad.q = q; ad.s = s;
    ad.x1_dtype = x1_dtype; ad.y1_dtype = y1_dtype; ad.rounding = add_rounding;
    ad.seed = add_seed; ad.offset = add_offset;
    return launch_layernorm_bwd_strip(qx, sx, qg, sg, gamma, mean, rstd, R, C, scale_dtype, rounding, seed, offset, nullptr,
                                      nullptr, dgamma, dbeta, workspace, &ad, (hipStream_t)stream);
}

int jf_layernorm_bwd(const int8_t *qx, const void *sx, const int8_t *qg, const void *sg, const float *gamma,
                     const float *mean, const float *rstd, int R, int C, int scale_dtype, int rounding, uint64_t seed,
                     uint64_t offset, int8_t *qdx, void *sdx, float *dgamma, float *dbeta, void *workspace,
                     size_t workspace_bytes, jf_stream_t stream)
{
    int rc = check_block_tensor(qx, sx, R, C, scale_dtype);
    if (rc) return rc;
    if ((rc = check_block_tensor(qg, sg, R, C, scale_dtype))) return rc;
    if (!gamma || !mean || !rstd || !qdx || !sdx) return JF_ERR_NULL;
    if (!rounding_ok(rounding)) return JF_ERR_ENUM;
    if (!aligned16(qdx) || !aligned16(gamma)) return JF_ERR_ALIGN;
    if (!workspace || workspace_bytes < jf_layernorm_bwd_workspace_bytes(R, C)) return JF_ERR_WORKSPACE;
    if (!aligned16(workspace)) return JF_ERR_ALIGN;
    if (!device_is_gfx950()) return JF_ERR_DEVICE;
    hipStream_t st = (hipStream_t)stream;
    const bool want_dw = dgamma || dbeta;
    const int SC = C / QB, groups = lnb_groups(R);
    if (SC <= LNS_WAVES * LNS_BPW)
        return launch_layernorm_bwd_strip(qx, sx, qg, sg, gamma, mean, rstd, R, C, scale_dtype, rounding, seed, offset, qdx,
                                          sdx, dgamma, dbeta, workspace, nullptr, st);
    const size_t smem = ((size_t)C + 2 * QB + 16 * QB) * sizeof(float);   // gamma, c1, c2 and the row-sum partials in LDS
    if (smem > LDS_VECTOR_LIMIT) return JF_ERR_SHAPE;
    float *part1 = (float *)workspace, *part2 = part1 + (size_t)R * SC;
    float *pdg = want_dw ? part2 + (size_t)R * SC : nullptr, *pdb = want_dw ? pdg + (size_t)groups * C : nullptr;
#define JF_LNB(ST)                                                                                                     \
    do {                                                                                                               \
        hipLaunchKernelGGL(layernorm_bwd_stats_kernel<ST>, dim3((SC + WPB - 1) / WPB * groups), dim3(NT), 0, st, qx,   \
                           (const ST *)sx, qg, (const ST *)sg, gamma, mean, rstd, R, C, groups, part1, part2, pdg, pdb); \
        hipLaunchKernelGGL(layernorm_bwd_dx_kernel<ST>, dim3(R / QB), dim3(WAVE * LNB_DX_WAVES), smem, st, qx,         \
                           (const ST *)sx, qg, (const ST *)sg, gamma, mean, rstd, R, C, rounding, seed, offset, part1, \
                           part2, qdx, (ST *)sdx, pdg, pdb, groups, dgamma, dbeta);                                    \
    } while (0)
    if (scale_dtype == JF_SCALE_F16) JF_LNB(half_t);
    else JF_LNB(float);
#undef JF_LNB
    return (int)hipGetLastError();
}

int jf_gelu_fwd(const int8_t *q, const void *s, int R, int C, int scale_dtype, int approx, float amax_eps, int8_t *qy,
                void *sy, jf_stream_t stream)
{
    int rc = check_block_tensor(q, s, R, C, scale_dtype);
    if (rc) return rc;
    if (!qy || !sy) return JF_ERR_NULL;
    if (approx != JF_GELU_ERF && approx != JF_GELU_TANH) return JF_ERR_ENUM;
    if (!aligned16(qy)) return JF_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const int grid = grid_for_groups(R, C);
#define JF_GF(A, ST) JF_LAUNCH((gelu_fwd_kernel<A, ST>), grid, 0, st, q, (const ST *)s, R, C, amax_eps, qy, (ST *)sy)
    if (scale_dtype == JF_SCALE_F16) {
        if (approx == JF_GELU_ERF) JF_GF(JF_GELU_ERF, half_t);
        JF_GF(JF_GELU_TANH, half_t);
    } else {
        if (approx == JF_GELU_ERF) JF_GF(JF_GELU_ERF, float);
        JF_GF(JF_GELU_TANH, float);
    }
#undef JF_GF
}

int jf_gelu_bwd(const int8_t *qx, const void *sx, const int8_t *qg, const void *sg, int R, int C, int scale_dtype,
                int approx, int rounding, uint64_t seed, uint64_t offset, int8_t *qy, void *sy, jf_stream_t stream)
{
    int rc = check_block_tensor(qx, sx, R, C, scale_dtype);
    if (rc) return rc;
    if ((rc = check_block_tensor(qg, sg, R, C, scale_dtype))) return rc;
    if (!qy || !sy) return JF_ERR_NULL;
    if ((approx != JF_GELU_ERF && approx != JF_GELU_TANH) || !rounding_ok(rounding)) return JF_ERR_ENUM;
    if (!aligned16(qy)) return JF_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const int grid = grid_for_groups(R, C);
#define JF_GB(A, ST)                                                                                              \
    JF_LAUNCH((gelu_bwd_kernel<A, ST>), grid, 0, st, qx, (const ST *)sx, qg, (const ST *)sg, R, C, rounding, seed, \
              offset, qy, (ST *)sy)
    if (scale_dtype == JF_SCALE_F16) {
        if (approx == JF_GELU_ERF) JF_GB(JF_GELU_ERF, half_t);
        JF_GB(JF_GELU_TANH, half_t);
    } else {
        if (approx == JF_GELU_ERF) JF_GB(JF_GELU_ERF, float);
        JF_GB(JF_GELU_TANH, float);
    }
#undef JF_GB
}

int jf_add(const void *x1, int x1_dtype, const int8_t *q2, const void *s2, int R, int C, int scale_dtype, int rounding,
           uint64_t seed, uint64_t offset, void *y1, int y1_dtype, int8_t *q, void *s, float *rowsum, float *rowsq,
           jf_stream_t stream)
{
    int rc = check_block_tensor(q2, s2, R, C, scale_dtype);
    if (rc) return rc;
    if (!x1 || !y1 || !q || !s) return JF_ERR_NULL;
    if ((rowsum == nullptr) != (rowsq == nullptr)) return JF_ERR_NULL;
    if (!rounding_ok(rounding) || x1_dtype < JF_FP_F16 || x1_dtype > JF_FP_BF16) return JF_ERR_ENUM;
    if (y1_dtype < JF_FP_F16 || y1_dtype > JF_FP_BF16) return JF_ERR_ENUM;
    if (!aligned16(x1) || !aligned16(y1) || !aligned16(q)) return JF_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const int grid = grid_for_workgroup_groups(R, C);
#define JF_ADD(T, ST, OT)                                                                                         \
    JF_LAUNCH((add_kernel<T, ST, OT>), grid, 0, st, (const T *)x1, q2, (const ST *)s2, R, C, rounding, seed, offset, \
              (OT *)y1, q, (ST *)s, rowsum, rowsq)
#define JF_ADD_OUT(T, ST)                                                                                         \
    do {                                                                                                          \
        if (y1_dtype == JF_FP_F32) JF_ADD(T, ST, float);                                                          \
        if (y1_dtype == JF_FP_F16) JF_ADD(T, ST, half_t);                                                         \
        JF_ADD(T, ST, __bf16);                                                                                    \
    } while (0)
    if (scale_dtype == JF_SCALE_F16) {
        if (x1_dtype == JF_FP_F32) JF_ADD_OUT(float, half_t);
        if (x1_dtype == JF_FP_F16) JF_ADD_OUT(half_t, half_t);
        JF_ADD_OUT(__bf16, half_t);
    } else {
        if (x1_dtype == JF_FP_F32) JF_ADD_OUT(float, float);
        if (x1_dtype == JF_FP_F16) JF_ADD_OUT(half_t, float);
        JF_ADD_OUT(__bf16, float);
    }
#undef JF_ADD_OUT
#undef JF_ADD
}

int jf_rowstats_finish(const float *rowsum, const float *rowsq, int R, int parts, int C, float *mean, float *rstd,
                       jf_stream_t stream)
{
    if (!rowsum || !rowsq || !mean || !rstd) return JF_ERR_NULL;
    if (R <= 0 || parts <= 0 || C <= 0) return JF_ERR_SHAPE;
    if (!device_is_gfx950()) return JF_ERR_DEVICE;
    if ((size_t)parts * RSF_ROWS * 2 * sizeof(float) > LDS_VECTOR_LIMIT) return JF_ERR_SHAPE;
    hipLaunchKernelGGL(rowstats_finish_kernel, dim3((R + RSF_ROWS - 1) / RSF_ROWS), dim3(256),
                       (size_t)parts * RSF_ROWS * 2 * sizeof(float), (hipStream_t)stream, rowsum, rowsq, R, parts, (float)C,
                       mean, rstd);
    return (int)hipGetLastError();
}

size_t jf_block_colsum_workspace_bytes(int R, int C)
{
    if (R <= 0 || C <= 0) return 0;
    return (size_t)(R / QB) * (size_t)C * sizeof(float);
}

int jf_block_colsum(const int8_t *q, const void *s, int R, int C, int scale_dtype, float *out, void *workspace,
                    size_t workspace_bytes, jf_stream_t stream)
{
    int rc = check_block_tensor(q, s, R, C, scale_dtype);
    if (rc) return rc;
    if (!out) return JF_ERR_NULL;
    if (!workspace || workspace_bytes < jf_block_colsum_workspace_bytes(R, C)) return JF_ERR_WORKSPACE;
    if (!aligned16(workspace)) return JF_ERR_ALIGN;
    if (!device_is_gfx950()) return JF_ERR_DEVICE;
    hipStream_t st = (hipStream_t)stream;
    float *terms = (float *)workspace;
    const int items = (R / QB) * ((C + 255) / 256);
    if (scale_dtype == JF_SCALE_F16)
        hipLaunchKernelGGL(colsum_strip_kernel<half_t>, dim3((items + WPB - 1) / WPB), dim3(NT), 0, st, q, (const half_t *)s, R, C, terms);
    else
        hipLaunchKernelGGL(colsum_strip_kernel<float>, dim3((items + WPB - 1) / WPB), dim3(NT), 0, st, q, (const float *)s, R, C, terms);
    hipLaunchKernelGGL(layernorm_bwd_colsum_finish_kernel, dim3(C / QB, 1), dim3(1024), 0, st, terms, (const float *)nullptr, R / QB, C,
                       out, (float *)nullptr);
    return (int)hipGetLastError();
}

}  // extern "C"
