// Device-side building blocks shared by the gfx950 kernels: wave reductions, Philox noise,
// the exact block-constant division, packing of INT8 codes, and the elementary functions.
//
// Everything that feeds an INT8 code is written with IEEE +,*,/ and explicit fmaf only
// (the translation unit is compiled with -ffp-contract=off), so a host evaluation of the same
// sequence gives the same bits.
#pragma once

#include <hip/hip_runtime.h>
#include <type_traits>
#include <stdint.h>

#include "../../include/jetfire_hip.h"

namespace jf {

constexpr int QB = 32;        // quantisation block edge
constexpr int WAVE = 64;

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 half_t;

// f(integral_constant<int, I>) for I = 0 .. N-1, unrolled at compile time
template <int I, int N, typename F> __device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// ---------------------------------------------------------------------------------------------
// scale element access: binary16 or binary32 behind one template parameter
template <typename ST> __device__ __forceinline__ float load_scale(const ST *p, int i) { return (float)p[i]; }
template <typename ST> __device__ __forceinline__ void store_scale(ST *p, int i, float v) { p[i] = (ST)v; }

// ---------------------------------------------------------------------------------------------
// 64-lane max reduction of NON-NEGATIVE values; every lane returns the maximum (it comes back through a scalar
// register, so the compiler knows it is wave-uniform).  Data-parallel-primitive forms of v_max_f32 inside the vector
// ALU: a shuffle through the LDS crossbar would cost six dependent LDS round trips.  Written as asm: from the
// update_dpp builtin the compiler makes a copy, a v_mov_b32_dpp and two v_max_f32 per step (36 instructions where 6 do;
// every block-wise kernel runs this once per block and lane).  A DPP operand read needs two wait states behind the
// vector instruction that wrote the register: the s_nop between the dependent steps.
__device__ __forceinline__ float wave_max(float v)
{
    asm volatile("s_nop 1\n\t"
                 "v_max_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1\n\t"
                 "v_max_f32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
                 "s_nop 1\n\t"
                 "v_max_f32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"     // max of 8
                 "s_nop 1\n\t"
                 "v_max_f32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"          // max of the 16-lane row, in all its lanes
                 "s_nop 1\n\t"
                 "v_max_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"        // rows 1, 3: with the row before
                 "s_nop 1\n\t"
                 "v_max_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"        // rows 2, 3: with rows 0-1; lane 63 has all
                 : "+v"(v));
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// ---------------------------------------------------------------------------------------------
// Philox4x32-R.  (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11.)  The rounding noise uses
// R = 7, the smallest round count the authors report as passing BigCrush (10 is their default with a safety margin):
// the generator is the largest single cost of every stochastic-rounding kernel here (its 64-bit multiplies take twice
// the issue time of a plain fp32 instruction).
// Build-time switch: -DJF_PHILOX_ROUNDS=10 gives the reference generator's round count (curandStatePhilox4_32_10,
// tl.rand); jf_philox_rounds() reports what a library was built with, and the CPU checker follows it.
#ifndef JF_PHILOX_ROUNDS
#define JF_PHILOX_ROUNDS 7
#endif
constexpr int PHILOX_ROUNDS = JF_PHILOX_ROUNDS;
static_assert(PHILOX_ROUNDS >= 7 && PHILOX_ROUNDS <= 10, "Philox4x32: 7 to 10 rounds");
template <int ROUNDS>
__device__ __forceinline__ void philox4x32(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                           uint32_t k0, uint32_t k1, uint32_t out[4])
{
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// Rounding noise for the 16 consecutive output elements e0 .. e0+15 (e0 a multiple of 16):
// two Philox calls at counters offset + e0/8 and +1, 16 bits per element, low half first;
// noise = (h + 0.5) * 2^-16 - 0.5 in (-0.5, 0.5).
__device__ __forceinline__ void sr_noise16(uint64_t seed, uint64_t offset, uint64_t e0, float n[16])
{
    uint64_t c = offset + (e0 >> 3);
#pragma unroll
    for (int call = 0; call < 2; ++call) {
        uint32_t o[4];
        uint64_t cc = c + (uint64_t)call;
        philox4x32<PHILOX_ROUNDS>((uint32_t)cc, (uint32_t)(cc >> 32), 0u, 0u, (uint32_t)seed, (uint32_t)(seed >> 32), o);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            // (h + 0.5) * 2^-16 - 0.5 = h * 2^-16 + (2^-17 - 0.5): every step of either form is exact (17 significant
            // bits at most), so the single fma gives the same value
            n[call * 8 + 2 * w]     = __builtin_fmaf((float)(o[w] & 0xFFFFu), 1.52587890625e-05f, -0.49999237060546875f);
            n[call * 8 + 2 * w + 1] = __builtin_fmaf((float)(o[w] >> 16), 1.52587890625e-05f, -0.49999237060546875f);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// a / 127, correctly rounded, for a in [2^-80, 2^100]: q0 = a * rn(1/127), e = fma(-q0, 127, a) (exact),
// q = fma(e, rn(1/127), q0) equals the IEEE quotient for every binary32 mantissa (checked exhaustively on the host;
// powers of two do not matter while nothing underflows).  3 plain instructions where the IEEE sequence takes 11, five of
// them at half or quarter rate.
__device__ __forceinline__ float div_by_127_in_range(float a)
{
    constexpr float R127 = 1.0f / 127.0f;
    const float q0 = a * R127;
    const float e = __builtin_fmaf(-q0, 127.0f, a);
    return __builtin_fmaf(e, R127, q0);
}

// ---------------------------------------------------------------------------------------------
// x / s for a divisor shared by many elements.  With r = 1/s (IEEE), q0 = x*r, e = x - q0*s (exact
// in one fma), q0 + e*r is the correctly rounded quotient as long as nothing under/overflows; the
// caller takes this path only for s in [2^-60, 2^60] and falls back to the IEEE division otherwise.
struct BlockDivisor {
    float s, r;
    bool fast;                  // the same in all lanes (s is a block constant): kept in a scalar register
    __device__ __forceinline__ explicit BlockDivisor(float s_) : s(s_)
    {
        fast = __builtin_amdgcn_readfirstlane((s_ > 8.67361738e-19f) && (s_ < 1.15292150e+18f)) != 0;
        r = 1.0f / s_;
    }
    // The divisor amax / 127 of a block quantisation, from the block maximum: one range test serves both this
    // division and the quotients (amax in (2^-53, 2^66) puts s inside (2^-60, 2^60)).
    struct FromAmax {};
    __device__ __forceinline__ BlockDivisor(float amax, FromAmax)
    {
        // (as an unsigned comparison of the bit patterns: amax comes out of a wave reduction in a scalar register, and
        // the scalar unit compares integers, not floats; negative values and NaNs fall outside as they should)
        fast = (__float_as_uint(amax) - 0x25000001u) < (0x60800000u - 0x25000001u);
        s = fast ? div_by_127_in_range(amax) : amax / 127.0f;
        r = 1.0f / s;
    }
    // y[i] = x[i] / s for N values; ONE uniform branch around the whole batch
    template <int N> __device__ __forceinline__ void divn(const float *x, float *y) const
    {
        if (fast) {
#pragma unroll
            for (int i = 0; i < N; ++i) {
                float q0 = x[i] * r;
                float e = __builtin_fmaf(-q0, s, x[i]);
                y[i] = __builtin_fmaf(e, r, q0);
            }
        } else {
#pragma unroll
            for (int i = 0; i < N; ++i) y[i] = x[i] / s;
        }
    }
    __device__ __forceinline__ void div16(const float x[16], float y[16]) const { divn<16>(x, y); }
};

__device__ __forceinline__ int clamp127(float y_rounded)
{
    float c = fminf(fmaxf(y_rounded, -127.0f), 127.0f);
    return (int)c;
}

__device__ __forceinline__ uint32_t pack4(int a, int b, int c, int d)
{
    return (uint32_t)(a & 0xFF) | ((uint32_t)(b & 0xFF) << 8) | ((uint32_t)(c & 0xFF) << 16) | ((uint32_t)d << 24);
}

// Round-to-nearest-even codes of 4 values, clamped to +-127, packed into one word.  Clamping first and rounding
// second gives the same integers as rounding first (the bounds are integers).  Adding 1.5*2^23 rounds to an
// integer in the addition itself and leaves its two's-complement low byte in the low byte of the bit pattern.
// CLAMP = false: for values the caller knows to round into [-127, 127] (|y| < 127.5).
template <bool CLAMP = true>
__device__ __forceinline__ uint32_t round_clamp_pack4(float a, float b, float c, float d)
{
    auto code_bits = [](float y) {
        const float yc = CLAMP ? __builtin_amdgcn_fmed3f(y, -127.0f, 127.0f) : y;
        return __float_as_uint(yc + 12582912.0f);
    };
    const uint32_t ab = __builtin_amdgcn_perm(code_bits(b), code_bits(a), 0x0c0c0400u);   // bytes: a, b, 0, 0
    const uint32_t cd = __builtin_amdgcn_perm(code_bits(d), code_bits(c), 0x0c0c0400u);
    return __builtin_amdgcn_perm(cd, ab, 0x05040100u);                                    // bytes: a, b, c, d
}

// ---------------------------------------------------------------------------------------------
// Block quantisation of 16 values per lane, one wave = one 32x32 block (lane l: row l/2,
// columns 16*(l%2) .. +15).  Returns the packed codes; *scale_out = amax/127 (all lanes).
//   y = v / s;  nearest: rn(y);  stochastic: rn(copysign(min(|y|+noise, 127), y));
//   trunc variants: trunc instead of rn.  All-zero block: s = 0, codes = 0.
__device__ __forceinline__ v4i quantize16(const float v[16], float amax_eps, int rounding,
                                          uint64_t seed, uint64_t offset, uint64_t e0, float *scale_out)
{
    float m = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) m = fmaxf(m, fabsf(v[i]));
    float amax = wave_max(m) + amax_eps;
    v4i out = {0, 0, 0, 0};
    if (!(amax > 0.0f)) { *scale_out = 0.0f; return out; }
    const BlockDivisor d(amax, BlockDivisor::FromAmax{});
    const float s = d.s;
    *scale_out = s;
    float y[16];
    d.div16(v, y);
    if (!d.fast) {                                             // uniform, rare: a scale near the ends of the exponent range
#pragma unroll                                                 // (a denormal s can be off by far more than an ulp)
        for (int i = 0; i < 16; ++i) y[i] = __builtin_amdgcn_fmed3f(y[i], -127.0f, 127.0f);
    }
    if (rounding == JF_ROUND_STOCHASTIC || rounding == JF_ROUND_STOCHASTIC_TRUNC) {
        float n[16];
        sr_noise16(seed, offset, e0, n);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float a = fminf(fabsf(y[i]) + n[i], 127.0f);
            y[i] = __builtin_copysignf(a, y[i]);
        }
    }
    if (rounding == JF_ROUND_TRUNC || rounding == JF_ROUND_STOCHASTIC_TRUNC) {
        int c[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) c[i] = clamp127(__builtin_truncf(y[i]));
        out.x = (int)pack4(c[0], c[1], c[2], c[3]);
        out.y = (int)pack4(c[4], c[5], c[6], c[7]);
        out.z = (int)pack4(c[8], c[9], c[10], c[11]);
        out.w = (int)pack4(c[12], c[13], c[14], c[15]);
    } else {
        // no clamp here: |v| <= amax and s = amax/127 correctly rounded give |v/s| <= 127 * (1 + 2^-23) < 127.5 (scales
        // outside the normal range were clamped above), and the stochastic path has limited |y| + noise to 127
        out.x = (int)round_clamp_pack4<false>(y[0], y[1], y[2], y[3]);
        out.y = (int)round_clamp_pack4<false>(y[4], y[5], y[6], y[7]);
        out.z = (int)round_clamp_pack4<false>(y[8], y[9], y[10], y[11]);
        out.w = (int)round_clamp_pack4<false>(y[12], y[13], y[14], y[15]);
    }
    return out;
}

// the 16 codes of a lane as floats (no scale applied)
__device__ __forceinline__ void codes_to_float16(v4i p, float x[16])
{
    const int w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        x[4 * i + 0] = (float)((w[i] << 24) >> 24);
        x[4 * i + 1] = (float)((w[i] << 16) >> 24);
        x[4 * i + 2] = (float)((w[i] << 8) >> 24);
        x[4 * i + 3] = (float)(w[i] >> 24);
    }
}

__device__ __forceinline__ void unpack16(v4i p, float scale, float x[16])
{
    const int w[4] = {p.x, p.y, p.z, p.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        x[4 * i + 0] = (float)((w[i] << 24) >> 24) * scale;
        x[4 * i + 1] = (float)((w[i] << 16) >> 24) * scale;
        x[4 * i + 2] = (float)((w[i] << 8) >> 24) * scale;
        x[4 * i + 3] = (float)(w[i] >> 24) * scale;
    }
}

// ---------------------------------------------------------------------------------------------
// Elementary functions (same sequences as the host checker uses).
__device__ __forceinline__ float expf_det(float x)
{
    const bool tiny = x < -87.0f;                    // result 0; selected at the end so that the code stays branch-free
    x = fmaxf(fminf(x, 88.0f), -87.0f);
    float n = __builtin_rintf(x * 1.44269504f);
    float r = __builtin_fmaf(n, -0.693145752f, x);
    r = __builtin_fmaf(n, -1.42860677e-06f, r);
    float p = 1.98412698e-04f;
    p = __builtin_fmaf(p, r, 1.38888889e-03f);
    p = __builtin_fmaf(p, r, 8.33333333e-03f);
    p = __builtin_fmaf(p, r, 4.16666667e-02f);
    p = __builtin_fmaf(p, r, 1.66666667e-01f);
    p = __builtin_fmaf(p, r, 0.5f);
    p = __builtin_fmaf(p, r, 1.0f);
    p = __builtin_fmaf(p, r, 1.0f);
    const float r2 = __int_as_float(__float_as_int(p) + (((int)n) << 23));
    return tiny ? 0.0f : r2;
}

// Phi(-x) = erfc(x / sqrt 2) / 2 for x >= 0, as 0.5 / (1 + b1 x + ... + b6 x^6)^16: Abramowitz & Stegun 7.1.28 with the
// coefficients rescaled to x / sqrt 2; absolute error below 1e-6 including the float rounding of the sixteenth power.
// No exponential and no IEEE division: the reciprocal is three Newton steps from an integer-subtraction seed, every
// step an fma, so the host evaluates the same bits (an approximate v_rcp_f32 would not be reproducible there).  The GELU
// tables are the largest piece of the GELU kernels' vector work; this form takes about half the instructions of an erfc
// fit with its division and exponential.
__device__ __forceinline__ float phi_neg(float x)
{
    float p = 5.38297490e-06f;
    p = __builtin_fmaf(p, x, 4.88906371e-05f);
    p = __builtin_fmaf(p, x, 3.80035744e-05f);
    p = __builtin_fmaf(p, x, 3.27762635e-03f);
    p = __builtin_fmaf(p, x, 2.11410057e-02f);
    p = __builtin_fmaf(p, x, 4.98673469e-02f);
    float u = __builtin_fmaf(p, x, 1.0f);
    u = u * u; u = u * u; u = u * u; u = u * u;
    u = fminf(u, 1.2676506e30f);                      // 2^100 (x > 12.4): keeps the seed below in range; the result is 0 there
    float r = __int_as_float(0x7EF311C7 - __float_as_int(u));     // 1/u to 12 %; each step squares the error
#pragma unroll
    for (int i = 0; i < 3; ++i) {
        const float e = __builtin_fmaf(-u, r, 1.0f);
        r = __builtin_fmaf(r, e, r);
    }
    // beyond the clamp Phi(-x) < 4e-31 is returned as 0, so that x * Phi(-x) vanishes for huge x as the function does
    return u < 1.2676506e30f ? 0.5f * r : 0.0f;
}

__device__ __forceinline__ float norm_cdf(float x)
{
    const float h = phi_neg(fabsf(x));
    return x > 0.0f ? 1.0f - h : h;
}

__device__ __forceinline__ float tanhf_det(float u)
{
    float a = fminf(fabsf(u), 15.0f);
    float e = expf_det(a + a);
    float t = 1.0f - 2.0f / (e + 1.0f);
    return __builtin_copysignf(t, u);
}

template <int APPROX> __device__ __forceinline__ float gelu(float x)
{
    if (APPROX == JF_GELU_ERF) return x * norm_cdf(x);
    float x2 = x * x;
    float inner = 0.797884561f * (x * __builtin_fmaf(0.044715f, x2, 1.0f));
    return (0.5f * x) * (1.0f + tanhf_det(inner));
}

template <int APPROX> __device__ __forceinline__ float dgelu(float x)
{
    if (APPROX == JF_GELU_ERF) {
        float pdf = 0.398942280f * expf_det(-0.5f * (x * x));
        return __builtin_fmaf(x, pdf, norm_cdf(x));
    }
    float x2 = fminf(x * x, 1e30f);                        // (keeps dinner finite: sech2 is exactly 0 long before, and 0 * inf is not)
    float inner = 0.797884561f * (x * __builtin_fmaf(0.044715f, x2, 1.0f));
    float t = tanhf_det(inner);
    float dinner = 0.797884561f * __builtin_fmaf(0.134145f, x2, 1.0f);
    float sech2 = __builtin_fmaf(-t, t, 1.0f);
    return __builtin_fmaf((0.5f * x) * sech2, dinner, 0.5f * (1.0f + t));
}

// gelu / dgelu at +x and -x (x >= 0) from one evaluation of the expensive part.  Every operation below is the one
// gelu<>/dgelu<> performs at that argument, or differs from it by exact sign symmetries only (x*x, |x|, a product with one
// factor negated, 1 + (-t)), so the pair is bit-identical to two separate evaluations.
template <int APPROX> __device__ __forceinline__ void gelu_pair(float x, float &pos, float &neg)
{
    if (APPROX == JF_GELU_ERF) {
        const float h = phi_neg(x);
        pos = x * (x > 0.0f ? 1.0f - h : h);
        neg = (-x) * h;
        return;
    }
    const float x2 = x * x;
    const float inner = 0.797884561f * (x * __builtin_fmaf(0.044715f, x2, 1.0f));
    const float t = tanhf_det(inner);                      // inner >= 0, so t >= 0 and tanh(-inner) = -t
    const float hx = 0.5f * x;
    pos = hx * (1.0f + t);
    neg = (-hx) * (1.0f - t);
}

template <int APPROX> __device__ __forceinline__ void dgelu_pair(float x, float &pos, float &neg)
{
    if (APPROX == JF_GELU_ERF) {
        const float pdf = 0.398942280f * expf_det(-0.5f * (x * x));
        const float h = phi_neg(x);
        pos = __builtin_fmaf(x, pdf, x > 0.0f ? 1.0f - h : h);
        neg = __builtin_fmaf(-x, pdf, h);
        return;
    }
    const float x2 = fminf(x * x, 1e30f);
    const float inner = 0.797884561f * (x * __builtin_fmaf(0.044715f, x2, 1.0f));
    const float t = tanhf_det(inner);
    const float dinner = 0.797884561f * __builtin_fmaf(0.134145f, x2, 1.0f);
    const float sech2 = __builtin_fmaf(-t, t, 1.0f);
    const float a = (0.5f * x) * sech2;
    pos = __builtin_fmaf(a, dinner, 0.5f * (1.0f + t));
    neg = __builtin_fmaf(-a, dinner, 0.5f * (1.0f - t));
}

// ---------------------------------------------------------------------------------------------
// GELU on a block tensor.  A block has ONE scale, so its 1024 inputs take at most 256 distinct values code*scale:
// the wave evaluates the function once per code (4 codes per lane) into a 1 KiB LDS table and every element then
// costs one LDS gather instead of ~40 vector instructions.  The table entry is computed from (float)code * scale,
// the very expression a per-element evaluation would use, so the results are bit-identical to it.
// PAIR(x, pos, neg) evaluates the function at +x and -x (x >= 0).  Lane l covers the magnitudes 2l+1 and 2l+2
// (1 .. 128); entry index = the code's byte value, so -m sits at 256-m and index 128 is the code -128.  Entry 0
// (the function at +0, the same for every block) is passed in.
template <typename PAIR>
__device__ __forceinline__ void fill_code_table(float *table, int lane, float scale, float f0, PAIR pair)
{
    const int m = 2 * lane + 1;
    float p0, n0, p1, n1;
    pair((float)m * scale, p0, n0);
    pair((float)(m + 1) * scale, p1, n1);
    table[m] = p0;
    if (lane < 63) table[m + 1] = p1;                              // +128 is not a code
    table[256 - m] = n0;
    table[255 - m] = n1;
    if (lane == 0) table[0] = f0;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}
__device__ __forceinline__ void gather16(const float *table, v4i p, float x[16])
{
    const uint32_t w[4] = {(uint32_t)p.x, (uint32_t)p.y, (uint32_t)p.z, (uint32_t)p.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        x[4 * i + 0] = table[w[i] & 0xFF];
        x[4 * i + 1] = table[(w[i] >> 8) & 0xFF];
        x[4 * i + 2] = table[(w[i] >> 16) & 0xFF];
        x[4 * i + 3] = table[w[i] >> 24];
    }
}
// The largest of a lane's 16 codes (signed bytes): one SDWA instruction per code (the operand's byte, sign-extended).
__device__ __forceinline__ int max_code16(v4i p)
{
    int m = -128;
#define JF_MAXB(W, B) asm("v_max_i32_sdwa %0, sext(%1), %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_" #B " src1_sel:DWORD" \
                          : "=v"(m) : "v"(W), "v"(m))
#define JF_MAXW(W) JF_MAXB(W, 0); JF_MAXB(W, 1); JF_MAXB(W, 2); JF_MAXB(W, 3)
    JF_MAXW(p.x); JF_MAXW(p.y); JF_MAXW(p.z); JF_MAXW(p.w);
#undef JF_MAXW
#undef JF_MAXB
    return m;
}
// max |gelu(x)| over x <= 0 is 0.169972 (erf form, at x = -0.7516) and 0.170041 (tanh form, at x = -0.7525) in this
// library's arithmetic (checked over the whole negative axis on the host); the bound leaves 6e-5 above both.
constexpr float GELU_NEG_BOUND = 0.1701f;
__device__ __forceinline__ void table_done()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();                               // all gathers done before the next block's fill
}

// GELU forward of one block: 16 codes per lane (lane l: row l/2, columns 16*(l%2) .. +15) with scale sc -> packed codes
// of the requantised result, *scale_out = its scale (all lanes).  tab / qtab: 256 floats / 64 ints (256 bytes) of LDS private to the
// wave.  f0 = gelu(+0), evaluated by the caller once (the same for every block).  (gelu_fwd.py:34-126)
template <int APPROX>
__device__ __forceinline__ v4i gelu_fwd_block(v4i c, float sc, float f0, float amax_eps, float *tab, int *qtab, int lane,
                                              float *scale_out)
{
    fill_code_table(tab, lane, sc, f0, [](float v, float &a, float &b) { gelu_pair<APPROX>(v, a, b); });
    // The outputs take at most 256 distinct values too, so the requantisation (exact division, rounding, clamp) is
    // done on the table, 4 entries per lane, once the block's absmax is known; an element costs two gathers.
    // The block's absmax.  x * Phi(x) rises with x > 0 (from one code to the next by at least 1/127 of itself, five
    // orders of magnitude above the table's rounding errors), so among the positive codes present the largest code has
    // the largest table entry, and no entry of a code <= 0 exceeds GELU_NEG_BOUND in magnitude at any scale.  A lane
    // therefore looks up the entry of its own largest code only; if the wave's maximum of those reaches the bound it
    // is the block's absmax.  Otherwise (no positive code, all of them tiny, a scale that overflows) every element's
    // entry is looked at.
    const int cl = max_code16(c);
    const float tl = tab[cl & 0xFF];
    float amax0 = wave_max(cl > 0 ? tl : 0.0f);
    if (!(amax0 >= GELU_NEG_BOUND && amax0 < __builtin_inff())) {   // uniform
        float x[16];
        gather16(tab, c, x);
        float m = 0.0f;
#pragma unroll
        for (int k = 0; k < 16; ++k) m = fmaxf(m, fabsf(x[k]));
        amax0 = wave_max(m);
    }
    const float amax = amax0 + amax_eps;
    float scale = 0.0f;
    v4i codes = {0, 0, 0, 0};
    if (amax > 0.0f) {                                         // uniform
        const BlockDivisor d(amax, BlockDivisor::FromAmax{});
        scale = d.s;
        const v4f t4 = *reinterpret_cast<const v4f *>(tab + 4 * lane);
        const float t[4] = {t4.x, t4.y, t4.z, t4.w};
        float y[4];
        d.divn<4>(t, y);
        // the requantised table is a BYTE table (entry e at byte e: lane l writes the word of its four entries): 64 words
        // instead of 256, so twice as many of a gather's lanes meet in the same word (a broadcast, not a bank conflict)
        qtab[lane] = (int)pack4(clamp127(__builtin_rintf(y[0])), clamp127(__builtin_rintf(y[1])),
                                clamp127(__builtin_rintf(y[2])), clamp127(__builtin_rintf(y[3])));
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // entry address = table + the code's byte: one SDWA add per element (the operand's byte, zero-extended)
        typedef __attribute__((address_space(3))) unsigned char lds_u8;
        const uint32_t q8 = (uint32_t)(uintptr_t)(lds_u8 *)qtab;
        const int wd[4] = {c.x, c.y, c.z, c.w};
        int o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t a0, a1, a2, a3;
#define JF_ADDB(DST, B) asm("v_add_u32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:BYTE_" #B " src1_sel:DWORD" \
                            : "=v"(DST) : "v"(wd[i]), "v"(q8))
            JF_ADDB(a0, 0); JF_ADDB(a1, 1); JF_ADDB(a2, 2); JF_ADDB(a3, 3);
#undef JF_ADDB
            const uint32_t b0 = *(const lds_u8 *)(uintptr_t)a0, b1 = *(const lds_u8 *)(uintptr_t)a1;
            const uint32_t b2 = *(const lds_u8 *)(uintptr_t)a2, b3 = *(const lds_u8 *)(uintptr_t)a3;
            // four zero-extended bytes into one word with three byte permutes
            o[i] = (int)__builtin_amdgcn_perm(__builtin_amdgcn_perm(b3, b2, 0x0c0c0400u), __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u),
                                              0x05040100u);
        }
        codes = v4i{o[0], o[1], o[2], o[3]};
    }
    table_done();
    *scale_out = scale;
    return codes;
}

// GELU backward of one block: codes / scale of the forward input (cx, scx) and of the incoming gradient (cg, scg), 16
// per lane in the row layout -> packed codes of gelu'(x) * g requantised with `rounding`, *scale_out = its scale.
// tab: 256 floats of LDS private to the wave; f0 = gelu'(+0), evaluated by the caller once.  (gelu_bwd.py:28-171)
template <int APPROX>
__device__ __forceinline__ v4i gelu_bwd_block(v4i cx, float scx, v4i cg, float scg, float f0, float *tab, int lane,
                                              int rounding, uint64_t seed, uint64_t offset, uint64_t e0, float *scale_out)
{
    float x[16], g[16];
    unpack16(cg, scg, g);
    fill_code_table(tab, lane, scx, f0, [](float v, float &a, float &b) { dgelu_pair<APPROX>(v, a, b); });
    gather16(tab, cx, x);
    table_done();
#pragma unroll
    for (int k = 0; k < 16; ++k) x[k] = x[k] * g[k];
    return quantize16(x, 0.0f, rounding, seed, offset, e0, scale_out);
}

// ---------------------------------------------------------------------------------------------
// host-side argument checks shared by the entry points
// The kernels exist as gfx950 code objects only: say so instead of failing at launch with "no binary for GPU".
// (One property query per device and process; afterwards a table look-up.)
constexpr int MAX_DEVICES = 64;                     // devices a process may use (per-device host state)
static inline bool device_is_gfx950()
{
    static signed char known[MAX_DEVICES] = {};           // 0: not asked yet, 1: gfx950, -1: something else
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return false;
    if (known[dev] == 0) {
        hipDeviceProp_t prop;
        bool ok = hipGetDeviceProperties(&prop, dev) == hipSuccess;
        if (ok) {
            const char *a = prop.gcnArchName;
            ok = a[0] == 'g' && a[1] == 'f' && a[2] == 'x' && a[3] == '9' && a[4] == '5' && a[5] == '0' && (a[6] == 0 || a[6] == ':');
        }
        known[dev] = ok ? 1 : -1;
    }
    return known[dev] == 1;
}
static inline bool mult32(int v) { return v > 0 && (v % QB) == 0; }
static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace jf
