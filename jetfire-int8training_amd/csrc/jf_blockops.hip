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

// ------------------------------------------------------------------------------------------------
// quantize.py:33-117 (and quantize_transpose.py:33-129 when qT != nullptr)
template <typename T, typename ST>
__global__ __launch_bounds__(NT) void quantize_kernel(const T *x, int R, int C, int8_t *q, ST *s, int8_t *qT,
                                                      int rounding, uint64_t seed, uint64_t offset, float amax_eps)
{
    __shared__ __attribute__((aligned(16))) unsigned char tpatch[WPB][QB][QB + 16];
    JF_FOR_EACH_BLOCK(R, C)
    {
        BlockPos pos(blk, SC, C, lane);
        float v[16];
        Load16<T>::run(x + pos.e0, v);
        float scale;
        v4i codes = quantize16(v, amax_eps, rounding, seed, offset, pos.e0, &scale);
        *reinterpret_cast<v4i *>(q + pos.e0) = codes;
        if (lane == 0) store_scale(s, pos.rb * SC + pos.cb, scale);
        if (qT) {
            unsigned char(*tp)[QB + 16] = tpatch[threadIdx.x >> 6];
            *reinterpret_cast<v4i *>(&tp[lane >> 1][(lane & 1) * 16]) = codes;
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            unsigned char b[16];
            const int ocol = lane >> 1, orow0 = (lane & 1) * 16;     // output row = input column
#pragma unroll
            for (int k = 0; k < 16; ++k) b[k] = tp[orow0 + k][ocol];
            *reinterpret_cast<v4i *>(qT + (size_t)(pos.cb * QB + ocol) * R + pos.rb * QB + orow0) =
                *reinterpret_cast<v4i *>(b);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// dequantize.py:28-84
template <typename ST>
__global__ __launch_bounds__(NT) void dequantize_kernel(const int8_t *q, const ST *s, int R, int C, float *out)
{
    JF_FOR_EACH_BLOCK(R, C)
    {
        BlockPos pos(blk, SC, C, lane);
        float x[16];
        unpack16(*reinterpret_cast<const v4i *>(q + pos.e0), load_scale(s, pos.rb * SC + pos.cb), x);
        store16_f32(out + pos.e0, x);
    }
}

// A wave that loads one block (1 KiB of codes), waits, computes and stores keeps far too few bytes in flight to
// cover the memory latency, so the GELU kernels run the block loop with the codes and scales of the next PF blocks
// already requested.
constexpr int PF = 3;
// Walks the blocks blk0, blk0 + stride, ... of a wave without a division per block: (row block, column block) advance
// by (stride / SC, stride % SC) with a carry.
struct BlockWalk {
    int rb, cb, drb, dcb, SC;
    __device__ __forceinline__ BlockWalk(int blk0, int stride, int SC_) : SC(SC_)
    {
        rb = blk0 / SC; cb = blk0 - rb * SC;
        drb = stride / SC; dcb = stride - drb * SC;
    }
    __device__ __forceinline__ void step()
    {
        rb += drb; cb += dcb;
        if (cb >= SC) { cb -= SC; ++rb; }
    }
};
template <typename ST> struct CodeStream {
    const int8_t *q;
    const ST *s;
    int C, RB, lane;
    BlockWalk at;                 // the next block to request
    v4i codes[PF];
    float scale[PF];
    __device__ __forceinline__ void request(int slot)
    {
        if (at.rb < RB) {
            codes[slot] = *reinterpret_cast<const v4i *>(q + (size_t)(at.rb * QB + (lane >> 1)) * C + at.cb * QB + (lane & 1) * 16);
            scale[slot] = load_scale(s, at.rb * at.SC + at.cb);
        }
        at.step();
    }
    __device__ __forceinline__ CodeStream(const int8_t *q_, const ST *s_, int R, int C_, int stride, int lane_, int blk0)
        : q(q_), s(s_), C(C_), RB(R / QB), lane(lane_), at(blk0, stride, C_ / QB)
    {
#pragma unroll
        for (int i = 0; i < PF; ++i) request(i);
    }
    // hands out the oldest block and requests the one PF strides ahead
    __device__ __forceinline__ void next(v4i &c, float &sc)
    {
        c = codes[0]; sc = scale[0];
#pragma unroll
        for (int i = 0; i + 1 < PF; ++i) { codes[i] = codes[i + 1]; scale[i] = scale[i + 1]; }
        request(PF - 1);
    }
};

// gelu_fwd.py:34-126
template <int APPROX, typename ST>
__global__ __launch_bounds__(NT) void gelu_fwd_kernel(const int8_t *q, const ST *s, int R, int C, float amax_eps,
                                                      int8_t *qy, ST *sy)
{
    __shared__ __attribute__((aligned(16))) float table[WPB][256];
    __shared__ __attribute__((aligned(16))) int qtable[WPB][256];
    float *tab = table[threadIdx.x >> 6];
    int *qtab = qtable[threadIdx.x >> 6];
    const int lane = threadIdx.x & 63, SC = C / QB, RB = R / QB, stride = gridDim.x * WPB;
    const int blk0 = __builtin_amdgcn_readfirstlane(blockIdx.x * WPB + (threadIdx.x >> 6));
    CodeStream<ST> in(q, s, R, C, stride, lane, blk0);
    float zero = 0.0f;
    asm volatile("" : "+v"(zero));                                 // evaluated on the device, like every other entry
    const float f0 = gelu<APPROX>(zero);
    for (BlockWalk w(blk0, stride, SC); w.rb < RB; w.step()) {
        const size_t e0 = (size_t)(w.rb * QB + (lane >> 1)) * C + w.cb * QB + (lane & 1) * 16;
        v4i c; float sc;
        in.next(c, sc);
        float scale;
        const v4i codes = gelu_fwd_block<APPROX>(c, sc, f0, amax_eps, tab, qtab, lane, &scale);
        *reinterpret_cast<v4i *>(qy + e0) = codes;
        if (lane == 0) store_scale(sy, w.rb * SC + w.cb, scale);
    }
}

// gelu_bwd.py:28-171
template <int APPROX, typename ST>
__global__ __launch_bounds__(NT) void gelu_bwd_kernel(const int8_t *qx, const ST *sx, const int8_t *qg, const ST *sg,
                                                      int R, int C, int rounding, uint64_t seed, uint64_t offset,
                                                      int8_t *qy, ST *sy)
{
    __shared__ __attribute__((aligned(16))) float table[WPB][256];
    float *tab = table[threadIdx.x >> 6];
    const int lane = threadIdx.x & 63, SC = C / QB, RB = R / QB, stride = gridDim.x * WPB;
    const int blk0 = __builtin_amdgcn_readfirstlane(blockIdx.x * WPB + (threadIdx.x >> 6));
    CodeStream<ST> inx(qx, sx, R, C, stride, lane, blk0), ing(qg, sg, R, C, stride, lane, blk0);
    float zero = 0.0f;
    asm volatile("" : "+v"(zero));
    const float f0 = dgelu<APPROX>(zero);
    for (BlockWalk w(blk0, stride, SC); w.rb < RB; w.step()) {
        const size_t e0 = (size_t)(w.rb * QB + (lane >> 1)) * C + w.cb * QB + (lane & 1) * 16;
        v4i cx, cg; float scx, scg;
        inx.next(cx, scx);
        ing.next(cg, scg);
        float x[16], g[16];
        unpack16(cg, scg, g);
        fill_code_table(tab, lane, scx, f0, [](float v, float &a, float &b) { dgelu_pair<APPROX>(v, a, b); });
        gather16(tab, cx, x);
        table_done();
#pragma unroll
        for (int k = 0; k < 16; ++k) x[k] = x[k] * g[k];
        float scale;
        v4i codes = quantize16(x, 0.0f, rounding, seed, offset, e0, &scale);
        *reinterpret_cast<v4i *>(qy + e0) = codes;
        if (lane == 0) store_scale(sy, w.rb * SC + w.cb, scale);
    }
}

// layernorm.py:74-190, with a real beta
template <typename ST>
__global__ __launch_bounds__(NT) void layernorm_fwd_kernel(const int8_t *q, const ST *s, const float *gamma,
                                                           const float *beta, const float *mean, const float *rstd,
                                                           int R, int C, int8_t *qy, ST *sy)
{
    JF_FOR_EACH_BLOCK(R, C)
    {
        BlockPos pos(blk, SC, C, lane);
        float x[16], w[16], b[16];
        unpack16(*reinterpret_cast<const v4i *>(q + pos.e0), load_scale(s, pos.rb * SC + pos.cb), x);
        Load16<float>::run(gamma + pos.col, w);
        if (beta) Load16<float>::run(beta + pos.col, b);
        else {
#pragma unroll
            for (int k = 0; k < 16; ++k) b[k] = 0.0f;
        }
        const float mu = mean[pos.row], rs = rstd[pos.row];
#pragma unroll
        for (int k = 0; k < 16; ++k) x[k] = __builtin_fmaf((x[k] - mu) * rs, w[k], b[k]);
        float scale;
        v4i codes = quantize16(x, 0.0f, JF_ROUND_NEAREST, 0, 0, pos.e0, &scale);
        *reinterpret_cast<v4i *>(qy + pos.e0) = codes;
        if (lane == 0) store_scale(sy, pos.rb * SC + pos.cb, scale);
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

constexpr int LNB_THREADS = 1024;
// LayerNorm backward in one launch (layernorm.py:197-402): one workgroup (16 waves) per 32-row strip; the waves take
// the column blocks round-robin.  Row reductions in a defined order (per row: 16-column partial sums of xhat*wdy as an
// fmaf chain and of wdy as an add chain go to LDS, then one lane per row adds all C/16 partials in ascending order ->
// c1, c2, so the requantised dx is bit-reproducible); then dx is computed and requantised.  The strip (2 x 32 x C bytes) is read a second time for that, from the L2 it was just fetched
// into (keeping it in registers instead does not fit next to the column-sum butterfly).  Also the strip's column sums
// for dgamma / dbeta.
template <typename ST>
__global__ __launch_bounds__(LNB_THREADS) void layernorm_bwd_fused_kernel(const int8_t *qx, const ST *sx, const int8_t *qg,
                                                                          const ST *sg, const float *gamma, const float *mean,
                                                                          const float *rstd, int R, int C, int rounding,
                                                                          uint64_t seed, uint64_t offset, int8_t *qdx, ST *sdx,
                                                                          float *pdg, float *pdb)
{
    extern __shared__ float fsm[];                // part1[32][C/16], part2[32][C/16], c1[32], c2[32], column-sum patches
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int SC = C / QB, H = C / 16, rb = blockIdx.x;
    float *part1 = fsm, *part2 = fsm + QB * H, *c1s = part2 + QB * H, *c2s = c1s + QB;
    float *cpatch = c2s + QB + wave * COLSUM_PATCH;
    const int r = lane >> 1;
    const float mu = mean[rb * QB + r], rs = rstd[rb * QB + r];
    for (int cb = wave; cb < SC; cb += LNB_THREADS / WAVE) {
        const int col = cb * QB + (lane & 1) * 16;
        const size_t e0 = (size_t)(rb * QB + r) * C + col;
        float x[16], g[16], w[16], v[16];
        unpack16(*reinterpret_cast<const v4i *>(qx + e0), load_scale(sx, rb * SC + cb), x);
        unpack16(*reinterpret_cast<const v4i *>(qg + e0), load_scale(sg, rb * SC + cb), g);
        Load16<float>::run(gamma + col, w);
        float p1 = 0.0f, p2 = 0.0f;
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const float xh = (x[k] - mu) * rs;
            const float wdy = w[k] * g[k];
            p1 = __builtin_fmaf(xh, wdy, p1);
            p2 = p2 + wdy;
            v[k] = g[k] * xh;
        }
        part1[r * H + cb * 2 + (lane & 1)] = p1;
        part2[r * H + cb * 2 + (lane & 1)] = p2;
        if (pdg) {
            // output of lane j (j even): value index j/4 of column set (j/2)%2
            const size_t dst = (size_t)rb * C + cb * QB + ((lane >> 1) & 1) * 16 + (lane >> 2);
            const float tg = colsum16_over_rows(v, lane, cpatch);  // sum of dy*xhat
            if ((lane & 1) == 0) pdg[dst] = tg;
            const float tb = colsum16_over_rows(g, lane, cpatch);  // sum of dy
            if ((lane & 1) == 0) pdb[dst] = tb;
        }
    }
    __syncthreads();
    if (threadIdx.x < QB) {
        const int rr = threadIdx.x;
        float t1 = 0.0f, t2 = 0.0f;
        for (int h = 0; h < H; ++h) { t1 = t1 + part1[rr * H + h]; t2 = t2 + part2[rr * H + h]; }
        c1s[rr] = t1 / (float)C;
        c2s[rr] = t2 / (float)C;
    }
    __syncthreads();
    const float k1 = c1s[r], k2 = c2s[r];
    for (int cb = wave; cb < SC; cb += LNB_THREADS / WAVE) {
        const int col = cb * QB + (lane & 1) * 16;
        const size_t e0 = (size_t)(rb * QB + r) * C + col;
        float x[16], g[16], w[16];
        unpack16(*reinterpret_cast<const v4i *>(qx + e0), load_scale(sx, rb * SC + cb), x);
        unpack16(*reinterpret_cast<const v4i *>(qg + e0), load_scale(sg, rb * SC + cb), g);
        Load16<float>::run(gamma + col, w);
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const float xh = (x[k] - mu) * rs;
            const float wdy = w[k] * g[k];
            x[k] = (wdy - __builtin_fmaf(xh, k1, k2)) * rs;
        }
        float scale;
        v4i codes = quantize16(x, 0.0f, rounding, seed, offset, e0, &scale);
        *reinterpret_cast<v4i *>(qdx + e0) = codes;
        if (lane == 0) store_scale(sdx, rb * SC + cb, scale);
    }
}

// out[c] = sum over strips of part[strip][c]   (layernorm.py:405-428).  64 columns per workgroup, 16 strip lanes
// per column (fixed partition and a fixed tree, so the result is reproducible).
__global__ __launch_bounds__(1024) void colsum_kernel(const float *part0, float *out0, const float *part1, float *out1,
                                                      int strips, int C)
{
    __shared__ float red[16][65];
    const float *part = blockIdx.y ? part1 : part0;
    float *out = blockIdx.y ? out1 : out0;
    if (!out) return;                                              // uniform
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + tx;
    float a = 0.0f;
    if (c < C)
        for (int i = ty; i < strips; i += 16) a += part[(size_t)i * C + c];
    red[ty][tx] = a;
    __syncthreads();
    if (ty == 0 && c < C) {
        float t = 0.0f;
#pragma unroll
        for (int k = 0; k < 16; ++k) t += red[k][tx];
        out[c] = t;
    }
}

// add.py:29-162 / add_mean_var.py:28-177
template <typename T, typename ST>
__global__ __launch_bounds__(NT) void add_kernel(const T *x1, const int8_t *q2, const ST *s2, int R, int C,
                                                 int rounding, uint64_t seed, uint64_t offset, float *y1, int8_t *q,
                                                 ST *s, float *rowsum, float *rowsq)
{
    JF_FOR_EACH_BLOCK(R, C)
    {
        BlockPos pos(blk, SC, C, lane);
        float a[16], b[16];
        Load16<T>::run(x1 + pos.e0, a);
        unpack16(*reinterpret_cast<const v4i *>(q2 + pos.e0), load_scale(s2, pos.rb * SC + pos.cb), b);
#pragma unroll
        for (int k = 0; k < 16; ++k) a[k] = a[k] + b[k];
        store16_f32(y1 + pos.e0, a);
        if (rowsum) {
            float t1 = 0.0f, t2 = 0.0f;
#pragma unroll
            for (int k = 0; k < 16; ++k) { t1 = t1 + a[k]; t2 = __builtin_fmaf(a[k], a[k], t2); }
            const float o1 = __shfl_xor(t1, 1, WAVE), o2 = __shfl_xor(t2, 1, WAVE);
            if ((lane & 1) == 0) {
                rowsum[(size_t)pos.row * SC + pos.cb] = t1 + o1;     // columns 0..15 partial + 16..31 partial
                rowsq[(size_t)pos.row * SC + pos.cb] = t2 + o2;
            }
        }
        float scale;
        v4i codes = quantize16(a, 0.0f, rounding, seed, offset, pos.e0, &scale);
        *reinterpret_cast<v4i *>(q + pos.e0) = codes;
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

// kernels that keep several blocks in flight per wave and have per-kernel setup: no more workgroups than are resident
static inline int grid_for_resident(int R, int C)
{
    const long nblk = (long)(R / QB) * (C / QB);
    long g = (nblk + WPB - 1) / WPB;
    const long cap = 256L * 8;
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

static inline bool rounding_ok(int r) { return r >= JF_ROUND_NEAREST && r <= JF_ROUND_STOCHASTIC_TRUNC; }

}  // namespace jf

using namespace jf;

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
    const int grid = grid_for_blocks(R, C);
#define JF_Q(T, ST)                                                                                          \
    JF_LAUNCH((quantize_kernel<T, ST>), grid, 0, st, (const T *)x, R, C, q, (ST *)s, qT, rounding, seed, offset, amax_eps)
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

int jf_dequantize(const int8_t *q, const void *s, int R, int C, int scale_dtype, float *out, jf_stream_t stream)
{
    int rc = check_block_tensor(q, s, R, C, scale_dtype);
    if (rc) return rc;
    if (!out) return JF_ERR_NULL;
    if (!aligned16(out)) return JF_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const int grid = grid_for_blocks(R, C);
    if (scale_dtype == JF_SCALE_F16) JF_LAUNCH(dequantize_kernel<half_t>, grid, 0, st, q, (const half_t *)s, R, C, out);
    JF_LAUNCH(dequantize_kernel<float>, grid, 0, st, q, (const float *)s, R, C, out);
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
    const int grid = grid_for_blocks(R, C);
    if (scale_dtype == JF_SCALE_F16)
        JF_LAUNCH(layernorm_fwd_kernel<half_t>, grid, 0, st, q, (const half_t *)s, gamma, beta, mean, rstd, R, C, qy,
                  (half_t *)sy);
    JF_LAUNCH(layernorm_fwd_kernel<float>, grid, 0, st, q, (const float *)s, gamma, beta, mean, rstd, R, C, qy,
              (float *)sy);
}

size_t jf_layernorm_bwd_workspace_bytes(int R, int C)
{
    if (R <= 0 || C <= 0) return 0;
    return ((size_t)2 * R + (size_t)2 * (R / QB) * C) * sizeof(float);
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
    // LDS: two [32][C/16] partial-sum arrays, c1/c2, one column-sum patch per wave
    const size_t smem = ((size_t)2 * QB * (C / 16) + 2 * QB + (LNB_THREADS / WAVE) * COLSUM_PATCH) * sizeof(float);
    if (smem > 160 * 1024 - 512) return JF_ERR_SHAPE;          // rows of up to ~5700 columns
    if (!device_is_gfx950()) return JF_ERR_DEVICE;
    hipStream_t st = (hipStream_t)stream;
    const bool want_dw = dgamma || dbeta;
    // workspace: [2R floats, unused by this implementation][strips x C partial dgamma][strips x C partial dbeta]
    float *pdg = want_dw ? (float *)workspace + (size_t)2 * R : nullptr, *pdb = want_dw ? pdg + (size_t)(R / QB) * C : nullptr;
#define JF_LNF(ST)                                                                                                    \
    do {                                                                                                              \
        auto kern = layernorm_bwd_fused_kernel<ST>;                                                                   \
        if (smem > 64 * 1024) {                                                                                       \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                                  \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);                \
            if (e != hipSuccess) return (int)e;                                                                       \
        }                                                                                                             \
        hipLaunchKernelGGL(kern, dim3(R / QB), dim3(LNB_THREADS), smem, st, qx, (const ST *)sx, qg, (const ST *)sg,   \
                           gamma, mean, rstd, R, C, rounding, seed, offset, qdx, (ST *)sdx, pdg, pdb);                \
    } while (0)
    if (scale_dtype == JF_SCALE_F16) JF_LNF(half_t);
    else JF_LNF(float);
#undef JF_LNF
    if (want_dw)
        hipLaunchKernelGGL(colsum_kernel, dim3((C + 63) / 64, 2), dim3(1024), 0, st, pdg, dgamma, pdb, dbeta, R / QB, C);
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
    const int grid = grid_for_resident(R, C);
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
    const int grid = grid_for_resident(R, C);
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
           uint64_t seed, uint64_t offset, float *y1, int8_t *q, void *s, float *rowsum, float *rowsq,
           jf_stream_t stream)
{
    int rc = check_block_tensor(q2, s2, R, C, scale_dtype);
    if (rc) return rc;
    if (!x1 || !y1 || !q || !s) return JF_ERR_NULL;
    if ((rowsum == nullptr) != (rowsq == nullptr)) return JF_ERR_NULL;
    if (!rounding_ok(rounding) || x1_dtype < JF_FP_F16 || x1_dtype > JF_FP_BF16) return JF_ERR_ENUM;
    if (!aligned16(x1) || !aligned16(y1) || !aligned16(q)) return JF_ERR_ALIGN;
    hipStream_t st = (hipStream_t)stream;
    const int grid = grid_for_blocks(R, C);
#define JF_ADD(T, ST)                                                                                             \
    JF_LAUNCH((add_kernel<T, ST>), grid, 0, st, (const T *)x1, q2, (const ST *)s2, R, C, rounding, seed, offset, y1, q, \
              (ST *)s, rowsum, rowsq)
    if (scale_dtype == JF_SCALE_F16) {
        if (x1_dtype == JF_FP_F32) JF_ADD(float, half_t);
        if (x1_dtype == JF_FP_F16) JF_ADD(half_t, half_t);
        JF_ADD(__bf16, half_t);
    } else {
        if (x1_dtype == JF_FP_F32) JF_ADD(float, float);
        if (x1_dtype == JF_FP_F16) JF_ADD(half_t, float);
        JF_ADD(__bf16, float);
    }
#undef JF_ADD
}

}  // extern "C"
