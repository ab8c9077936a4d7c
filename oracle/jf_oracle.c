/*
 * jf_oracle.c -- CPU restatement of the Jetfire per-block INT8 data-flow path.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker that the HIP kernels are
 * compared against (tests/, the smoke check, and the cpu_baseline leg of the
 * benchmark). Nothing in the shipped library links, loads or calls it.
 *
 * Every function restates, in scalar C with IEEE binary32 arithmetic (no
 * contraction: build with -ffp-contract=off; fused operations are written as
 * explicit fmaf), the algorithm of one reference kernel.  Paths are relative
 * to the reference tree.
 *
 * Conventions (reference: JetfireGEMMKernel/tests/test_int8igemmoutputIntQuantizeStochastic.py:24-45):
 *   - a block tensor is (q: int8 [R,C] row-major, s: float [R/32, C/32]); x ~= q*s
 *   - all R, C, M, N, K are multiples of 32
 *   - GEMM scale operands are K-major:  sa[kb*(M/32)+mb], sb[kb*(N/32)+nb]
 *     (JetfireGEMMKernel/BlockQuantize/cpp_extension/igemm/igemm_BlockSquare32OutputIntQuantizeBiasRowCol.cu:110-111,187-188)
 *   - scales are carried as float here; the fp16-scale API variant is the same
 *     arithmetic on values that happen to be representable in binary16
 *     (round with jfo_round_to_f16 before/after as the caller needs).
 *
 * Deliberate definitions where the reference is undefined or not reproducible:
 *   - all-zero block: scale 0, codes 0 (reference: 0/0 -> NaN)
 *   - divisions are IEEE (reference is built with -use_fast_math, setup.py:28)
 *   - stochastic rounding noise comes from Philox4x32-7 keyed by (seed, element
 *     index) instead of curand keyed by threadIdx (…Stochastic.cu:311-312,416)
 *     or a materialised torch noise tensor (Jetfire/Nonlinear/quantize.py:143-146)
 *   - stochastic GEMM epilogue clamps to +-127 (reference wraps 128 -> -128)
 *
 * Parity status of each function (what pins it) is listed in oracle/README.md.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QB 32

/* ------------------------------------------------------------------------- */
/* Philox4x32-R (Salmon et al., "Parallel random numbers: as easy as 1,2,3",   */
/* SC'11; with R = 10 the generator behind curandStatePhilox4_32_10_t used at */
/* …Stochastic.cu:311).  Pinned by the Random123 known-answer vectors (R=10). */
/* ------------------------------------------------------------------------- */
void jfo_philox4x32(const uint32_t ctr[4], const uint32_t key[2], int rounds, uint32_t out[4])
{
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int r = 0; r < rounds; ++r) {
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

void jfo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4])
{
    jfo_philox4x32(ctr, key, 10, out);
}

/* Rounds of the generator behind the rounding noise: 7, the smallest count Salmon et al. report as passing BigCrush
 * (the kernels pay for every round with two quarter-rate multiplies per 8 elements).  The round function and key
 * schedule are the ones the 10-round known answers pin. */
static int jfo_noise_rounds_now = 7;
#define JFO_NOISE_ROUNDS jfo_noise_rounds_now

/* The product library has a build-time round count (7 by default, 10 = the reference generator's); a test run sets the
 * checker to what the library under test reports.  Returns the count in force afterwards. */
int jfo_set_noise_rounds(int rounds)
{
    if (rounds >= 1 && rounds <= 10) jfo_noise_rounds_now = rounds;
    return jfo_noise_rounds_now;
}

/*
 * Rounding noise for element `e` (flat row-major index r*C+c of the OUTPUT
 * tensor).  One Philox4x32-7 call serves 8 consecutive elements, 16 bits each:
 *   counter = (offset + e/8) as 64-bit in words 0,1; words 2,3 = 0; key = seed
 *   h = 16-bit field (e%8): word (e%8)/2, low half for even e, high half for odd
 *   noise = (h + 0.5) * 2^-16 - 0.5      in (-0.5, 0.5), symmetric, exact in f32
 * Replaces curand_uniform4 - 0.5 (…Stochastic.cu:351-355) and
 * uniform_(-0.5, 0.5) (quantize.py:144).
 */
float jfo_sr_noise(uint64_t seed, uint64_t offset, uint64_t e)
{
    uint64_t c = offset + (e >> 3);
    uint32_t ctr[4] = { (uint32_t)c, (uint32_t)(c >> 32), 0u, 0u };
    uint32_t key[2] = { (uint32_t)seed, (uint32_t)(seed >> 32) };
    uint32_t o[4];
    jfo_philox4x32(ctr, key, JFO_NOISE_ROUNDS, o);
    unsigned lane = (unsigned)(e & 7u);
    uint32_t w = o[lane >> 1];
    uint32_t h = (lane & 1u) ? (w >> 16) : (w & 0xFFFFu);
    return ((float)h + 0.5f) * 1.52587890625e-05f - 0.5f;
}

/* binary32 -> binary16 bits, round-to-nearest-even (what __float2half does at
 * …BiasRowCol.cu:367 and what Triton's .to(tl.float16) does at quantize.py:95). */
uint16_t jfo_f32_to_f16_bits(float f)
{
    uint32_t x; memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t em = x & 0x7FFFFFFFu;
    if (em >= 0x7F800000u) return (uint16_t)(sign | (em > 0x7F800000u ? 0x7E00u : 0x7C00u));
    if (em >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);          /* >= 65520 -> inf */
    if (em < 0x33000001u) return (uint16_t)sign;                        /* <= 2^-25 -> 0   */
    int exp = (int)(em >> 23) - 127;
    uint32_t man = (em & 0x7FFFFFu) | 0x800000u;
    int shift;
    uint32_t base;
    if (exp < -14) { shift = 13 + (-14 - exp); base = 0; }             /* subnormal half  */
    else           { shift = 13; base = (uint32_t)(exp + 15) << 10; man &= 0x7FFFFFu; }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return (uint16_t)(sign | (base + q));
}

float jfo_f16_bits_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu, x;
    if (e == 0) {
        if (m == 0) x = sign;
        else { int s = 0; while (!(m & 0x400u)) { m <<= 1; s++; } m &= 0x3FFu; x = sign | ((uint32_t)(113 - s) << 23) | (m << 13); }
    } else if (e == 31) x = sign | 0x7F800000u | (m << 13);
    else x = sign | ((e + 112u) << 23) | (m << 13);
    float f; memcpy(&f, &x, 4); return f;
}

float jfo_round_to_f16(float f) { return jfo_f16_bits_to_f32(jfo_f32_to_f16_bits(f)); }

static inline int8_t rn_s8_clamp127(float y)
{
    float r = rintf(y);                       /* ties-to-even: __float2int_rn / llrint */
    if (r > 127.0f) r = 127.0f;
    if (r < -127.0f) r = -127.0f;
    return (int8_t)(int)r;
}

/* ------------------------------------------------------------------------- */
/* A.1  Block quantise.  Jetfire/Nonlinear/quantize.py:60-96                   */
/*   xf = float(x); amax = max|xf| over the 32x32 block (+ amax_eps: the       */
/*   SCALE_MIN_THRES of gelu_fwd.py:90); s = amax/127; y = xf/s (div_rn);      */
/*   nearest: q = rn(y).  stochastic (quantize.py:119-126 then :92):            */
/*   q = rn( sign(y) * clamp(|y| + noise, -128, 127) ).                          */
/*   mode 2 = truncate toward zero instead of rn: the `.to(int8)` without      */
/*   llrint of add.py:139 / add_mean_var.py:138.                                */
/* ------------------------------------------------------------------------- */
static void quantize_block(const float *xf /*[32][ld]*/, int ld, int8_t *q, int ldq,
                           float *s_out, int stochastic, uint64_t seed, uint64_t offset,
                           uint64_t e00 /*flat index of element (0,0)*/, uint64_t C,
                           float amax_eps, int truncate)
{
    float amax = 0.0f;
    for (int i = 0; i < QB; ++i)
        for (int j = 0; j < QB; ++j) {
            float a = fabsf(xf[i * ld + j]);
            if (a > amax) amax = a;           /* NaN never wins: same as v_max_f32 */
        }
    amax = amax + amax_eps;
    if (!(amax > 0.0f)) {
        *s_out = 0.0f;
        for (int i = 0; i < QB; ++i) for (int j = 0; j < QB; ++j) q[i * ldq + j] = 0;
        return;
    }
    float s = amax / 127.0f;
    *s_out = s;
    for (int i = 0; i < QB; ++i)
        for (int j = 0; j < QB; ++j) {
            float y = xf[i * ld + j] / s;
            if (stochastic) {
                float n = jfo_sr_noise(seed, offset, e00 + (uint64_t)i * C + (uint64_t)j);
                float a = fabsf(y) + n;
                if (a > 127.0f) a = 127.0f;
                if (a < -128.0f) a = -128.0f;
                y = copysignf(a, y);
            }
            float r = truncate ? truncf(y) : rintf(y);
            if (r > 127.0f) r = 127.0f;
            if (r < -127.0f) r = -127.0f;
            q[i * ldq + j] = (int8_t)(int)r;
        }
}

void jfo_quantize(const float *x, int R, int C, int8_t *q, float *s,
                  int stochastic, uint64_t seed, uint64_t offset, float amax_eps, int truncate)
{
    int SC = C / QB;
    #pragma omp parallel for collapse(2) schedule(static)
    for (int rb = 0; rb < R / QB; ++rb)
        for (int cb = 0; cb < SC; ++cb) {
            size_t o = (size_t)rb * QB * C + (size_t)cb * QB;
            quantize_block(x + o, C, q + o, C, &s[rb * SC + cb], stochastic, seed, offset,
                           (uint64_t)o, (uint64_t)C, amax_eps, truncate);
        }
}

/* Jetfire/Nonlinear/dequantize.py:70-72 (we multiply in fp32, reference in fp16). */
void jfo_dequantize(const int8_t *q, const float *s, int R, int C, float *x)
{
    int SC = C / QB;
    #pragma omp parallel for schedule(static)
    for (int r = 0; r < R; ++r)
        for (int c = 0; c < C; ++c)
            x[(size_t)r * C + c] = (float)q[(size_t)r * C + c] * s[(r / QB) * SC + c / QB];
}

/* Jetfire/Nonlinear/transpose.py:29-67 */
void jfo_transpose_s8(const int8_t *in, int R, int C, int8_t *out)
{
    #pragma omp parallel for schedule(static)
    for (int r = 0; r < R; ++r)
        for (int c = 0; c < C; ++c)
            out[(size_t)c * R + r] = in[(size_t)r * C + c];
}

/* ------------------------------------------------------------------------- */
/* GEMMs.  b_layout 0: B is [N,K] row-major (forward, …BiasRowCol.cu:104);     */
/*         b_layout 1: B is [K,N] row-major (…Stochastic.cu:102,142).          */
/* ------------------------------------------------------------------------- */
static int8_t *b_as_nk(const int8_t *B, int N, int K, int b_layout)
{
    if (b_layout == 0) return (int8_t *)B;
    int8_t *t = (int8_t *)malloc((size_t)N * K);
    jfo_transpose_s8(B, K, N, t);
    return t;
}

__attribute__((target_clones("arch=skylake-avx512", "avx2", "default")))
static int32_t dot32(const int8_t *a, const int8_t *b)
{
    int32_t d = 0;
    for (int k = 0; k < QB; ++k) d += (int32_t)a[k] * (int32_t)b[k];
    return d;
}

/* igemm_BasicInt8Gemm.cu:14-110: C_s32 = A * B (exact). */
void jfo_igemm_s32(const int8_t *A, const int8_t *B, int32_t *Cout, int M, int N, int K, int b_layout)
{
    int8_t *Bt = b_as_nk(B, N, K, b_layout);
    #pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            int32_t d = 0;
            for (int kb = 0; kb < K / QB; ++kb)
                d += dot32(A + (size_t)m * K + kb * QB, Bt + (size_t)n * K + kb * QB);
            Cout[(size_t)m * N + n] = d;
        }
    if (Bt != B) free(Bt);
}

/* The per-K-block INT32 accumulators frag_intc of …BiasRowCol.cu:209-211: acc[kb][m][n]. */
void jfo_igemm_block_acc(const int8_t *A, const int8_t *B, int32_t *acc, int M, int N, int K, int b_layout)
{
    int8_t *Bt = b_as_nk(B, N, K, b_layout);
    #pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n)
            for (int kb = 0; kb < K / QB; ++kb)
                acc[((size_t)kb * M + m) * N + n] =
                    dot32(A + (size_t)m * K + kb * QB, Bt + (size_t)n * K + kb * QB);
    if (Bt != B) free(Bt);
}

/*
 * A.2  Dequantise-accumulate.  …BiasRowCol.cu:173-217:
 *   acc = 0; for kb ascending: acc += (sa[kb,mb]*sb[kb,nb]) * (float)d_kb
 * nvcc contracts the += into one FFMA, hence fused=1 (fmaf) is canonical.
 * fused=0 gives the two-rounding form of a naive torch emulation.
 */
void jfo_igemm_block_f32(const int8_t *A, const int8_t *B, const float *sa, const float *sb,
                         float *out, int M, int N, int K, int b_layout, int fused)
{
    int8_t *Bt = b_as_nk(B, N, K, b_layout);
    int SM = M / QB, SN = N / QB;
    #pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            float acc = 0.0f;
            for (int kb = 0; kb < K / QB; ++kb) {
                int32_t d = dot32(A + (size_t)m * K + kb * QB, Bt + (size_t)n * K + kb * QB);
                float sab = sa[kb * SM + m / QB] * sb[kb * SN + n / QB];
                if (fused) acc = fmaf(sab, (float)d, acc);
                else { float p = sab * (float)d; acc = acc + p; }
            }
            out[(size_t)m * N + n] = acc;
        }
    if (Bt != B) free(Bt);
}

/*
 * A.3 / A.4  Requantising epilogues on an fp32 accumulator matrix.
 *  deterministic (…BiasRowCol.cu:313-367; …IntQuantize.cu:346):
 *     amax = max_block|acc| + biasmax
 *     q = clamp( rn( (127*(acc+bias[n])) / amax ), -127, 127 );  sc = amax/127
 *     (bias may be NULL = the bias-free …IntQuantize.cu form)
 *  stochastic (…Stochastic.cu:342-365):
 *     q = clamp( rn( (127*acc)/amax + noise ), -127, 127 )
 */
void jfo_requant(const float *acc, int M, int N, const float *bias, float biasmax,
                 int stochastic, uint64_t seed, uint64_t offset, int8_t *q, float *sc)
{
    int SN = N / QB;
    #pragma omp parallel for collapse(2) schedule(static)
    for (int mb = 0; mb < M / QB; ++mb)
        for (int nb = 0; nb < SN; ++nb) {
            const float *a = acc + (size_t)mb * QB * N + nb * QB;
            int8_t *qo = q + (size_t)mb * QB * N + nb * QB;
            float amax = 0.0f;
            for (int i = 0; i < QB; ++i)
                for (int j = 0; j < QB; ++j) {
                    float v = fabsf(a[(size_t)i * N + j]);
                    if (v > amax) amax = v;
                }
            amax = amax + biasmax;
            if (!(amax > 0.0f)) {
                sc[mb * SN + nb] = 0.0f;
                for (int i = 0; i < QB; ++i) for (int j = 0; j < QB; ++j) qo[(size_t)i * N + j] = 0;
                continue;
            }
            sc[mb * SN + nb] = amax / 127.0f;
            for (int i = 0; i < QB; ++i)
                for (int j = 0; j < QB; ++j) {
                    float v = a[(size_t)i * N + j];
                    if (bias) v = v + bias[nb * QB + j];
                    float t = (127.0f * v) / amax;
                    if (stochastic)
                        t = t + jfo_sr_noise(seed, offset,
                                             (uint64_t)(mb * QB + i) * (uint64_t)N + (uint64_t)(nb * QB + j));
                    qo[(size_t)i * N + j] = rn_s8_clamp127(t);
                }
        }
}

/* ------------------------------------------------------------------------- */
/* Elementary functions written with IEEE +,*,/,fmaf only, so that the device  */
/* evaluates the very same sequence and the INT8 codes can be compared         */
/* bit-for-bit.  (Reference uses NVIDIA libdevice erf/exp: gelu_fwd.py:81,      */
/* gelu_bwd.py:104-105 -- not reproducible off NVIDIA.)                         */
/* ------------------------------------------------------------------------- */
float jfo_expf(float x)
{
    if (x < -87.0f) return 0.0f;
    if (x > 88.0f) x = 88.0f;
    float n = rintf(x * 1.44269504f);
    float r = fmaf(n, -0.693145752f, x);
    r = fmaf(n, -1.42860677e-06f, r);
    float p = 1.98412698e-04f;            /* 1/5040 */
    p = fmaf(p, r, 1.38888889e-03f);      /* 1/720  */
    p = fmaf(p, r, 8.33333333e-03f);      /* 1/120  */
    p = fmaf(p, r, 4.16666667e-02f);      /* 1/24   */
    p = fmaf(p, r, 1.66666667e-01f);      /* 1/6    */
    p = fmaf(p, r, 0.5f);
    p = fmaf(p, r, 1.0f);
    p = fmaf(p, r, 1.0f);
    int32_t bits; memcpy(&bits, &p, 4);
    bits += ((int32_t)n) << 23;
    memcpy(&p, &bits, 4);
    return p;
}

/* Phi(-x) = erfc(x/sqrt2)/2 for x >= 0: 0.5 / (1 + b1 x + ... + b6 x^6)^16, Abramowitz & Stegun 7.1.28 (|error| <= 3e-7
 * on erf) with the coefficients rescaled to x/sqrt2; with float rounding (the sixteenth power amplifies the rounding of
 * its base sixteen times) the absolute error stays below 1e-6.  The reciprocal is three Newton steps from an
 * integer-subtraction seed, so that host and device evaluate the same bits without an IEEE division or an exponential. */
float jfo_phi_neg(float x)
{
    float p = 5.38297490e-06f;
    p = fmaf(p, x, 4.88906371e-05f);
    p = fmaf(p, x, 3.80035744e-05f);
    p = fmaf(p, x, 3.27762635e-03f);
    p = fmaf(p, x, 2.11410057e-02f);
    p = fmaf(p, x, 4.98673469e-02f);
    float u = fmaf(p, x, 1.0f);
    u = u * u; u = u * u; u = u * u; u = u * u;
    u = fminf(u, 1.2676506e30f);                      /* 2^100 */
    int32_t bits; memcpy(&bits, &u, 4);
    bits = 0x7EF311C7 - bits;
    float r; memcpy(&r, &bits, 4);
    for (int i = 0; i < 3; ++i) {
        float e = fmaf(-u, r, 1.0f);
        r = fmaf(r, e, r);
    }
    /* beyond the clamp (x > 12.4, Phi(-x) < 4e-31) the result is 0, so that x * Phi(-x) vanishes for huge x */
    return u < 1.2676506e30f ? 0.5f * r : 0.0f;
}

/* Phi(x) = (1+erf(x/sqrt2))/2  (gelu_fwd.py:81) */
float jfo_norm_cdf(float x)
{
    float h = jfo_phi_neg(fabsf(x));
    return x > 0.0f ? 1.0f - h : h;
}

/* tanh(u) = 1 - 2/(exp(2u)+1), |u| clamped to 15 */
float jfo_tanhf(float u)
{
    float a = fabsf(u);
    if (a > 15.0f) a = 15.0f;
    float e = jfo_expf(a + a);
    float t = 1.0f - 2.0f / (e + 1.0f);
    return copysignf(t, u);
}

/* approx 0: x*Phi(x)  (gelu_fwd.py:81-82);  approx 1: tanh form (torch approximate='tanh') */
float jfo_gelu(float x, int approx)
{
    if (approx == 0) return x * jfo_norm_cdf(x);
    float x2 = x * x;
    float inner = 0.797884561f * (x * fmaf(0.044715f, x2, 1.0f));
    return (0.5f * x) * (1.0f + jfo_tanhf(inner));
}

/* approx 0: Phi(x) + x*phi(x)  (gelu_bwd.py:104-107) */
float jfo_dgelu(float x, int approx)
{
    if (approx == 0) {
        float pdf = 0.398942280f * jfo_expf(-0.5f * (x * x));
        return fmaf(x, pdf, jfo_norm_cdf(x));
    }
    float x2 = fminf(x * x, 1e30f);      /* keeps dinner finite: sech2 is exactly 0 long before, and 0 * inf is not */
    float inner = 0.797884561f * (x * fmaf(0.044715f, x2, 1.0f));
    float t = jfo_tanhf(inner);
    float dinner = 0.797884561f * fmaf(0.134145f, x2, 1.0f);
    float sech2 = fmaf(-t, t, 1.0f);
    return fmaf((0.5f * x) * sech2, dinner, 0.5f * (1.0f + t));
}

/* ------------------------------------------------------------------------- */
/* Block-local fused ops: dequant -> f -> requant (A.1 on the result)          */
/* ------------------------------------------------------------------------- */
#define FOR_BLOCKS(R, C)                                         \
    _Pragma("omp parallel for collapse(2) schedule(static)")    \
    for (int rb = 0; rb < (R) / QB; ++rb)                        \
        for (int cb = 0; cb < (C) / QB; ++cb)

/* gelu_fwd.py:34-126 (amax_eps = 5e-5 reproduces :90) */
void jfo_gelu_fwd(const int8_t *q, const float *s, int R, int C, int approx, float amax_eps,
                  int8_t *qy, float *sy)
{
    int SC = C / QB;
    FOR_BLOCKS(R, C) {
        float tmp[QB * QB];
        size_t o = (size_t)rb * QB * C + (size_t)cb * QB;
        float sc = s[rb * SC + cb];
        for (int i = 0; i < QB; ++i)
            for (int j = 0; j < QB; ++j)
                tmp[i * QB + j] = jfo_gelu((float)q[o + (size_t)i * C + j] * sc, approx);
        quantize_block(tmp, QB, qy + o, C, &sy[rb * SC + cb], 0, 0, 0, (uint64_t)o, (uint64_t)C, amax_eps, 0);
    }
}

/* gelu_bwd.py:28-171 */
void jfo_gelu_bwd(const int8_t *qx, const float *sx, const int8_t *qg, const float *sg, int R, int C,
                  int approx, int stochastic, uint64_t seed, uint64_t offset, int8_t *qy, float *sy)
{
    int SC = C / QB;
    FOR_BLOCKS(R, C) {
        float tmp[QB * QB];
        size_t o = (size_t)rb * QB * C + (size_t)cb * QB;
        float scx = sx[rb * SC + cb], scg = sg[rb * SC + cb];
        for (int i = 0; i < QB; ++i)
            for (int j = 0; j < QB; ++j) {
                float x = (float)qx[o + (size_t)i * C + j] * scx;
                float g = (float)qg[o + (size_t)i * C + j] * scg;
                tmp[i * QB + j] = jfo_dgelu(x, approx) * g;
            }
        quantize_block(tmp, QB, qy + o, C, &sy[rb * SC + cb], stochastic, seed, offset, (uint64_t)o, (uint64_t)C, 0.0f, 0);
    }
}

/*
 * Row statistics of a block tensor (what add_mean_var.py:111-118,219-221 hands
 * to LayerNorm, restated on the quantised values so the sums are exact):
 *   S1 = sum_b s_b * (sum_{j in b} q_j),  S2 = sum_b s_b^2 * (sum q_j^2)   (integer inner sums)
 *   combined over column blocks b ascending with fmaf;
 *   mean = S1/C; var = max(S2/C - mean^2, 0); rstd = 1/sqrt(var + eps)
 */
void jfo_rowstats(const int8_t *q, const float *s, int R, int C, float eps, float *mean, float *rstd)
{
    int SC = C / QB;
    #pragma omp parallel for schedule(static)
    for (int r = 0; r < R; ++r) {
        float s1 = 0.0f, s2 = 0.0f;
        for (int cb = 0; cb < SC; ++cb) {
            int32_t i1 = 0, i2 = 0;
            for (int j = 0; j < QB; ++j) {
                int32_t v = q[(size_t)r * C + cb * QB + j];
                i1 += v; i2 += v * v;
            }
            float sc = s[(r / QB) * SC + cb];
            s1 = fmaf(sc, (float)i1, s1);
            s2 = fmaf(sc * sc, (float)i2, s2);
        }
        float mu = s1 / (float)C;
        float var = fmaf(-mu, mu, s2 / (float)C);
        if (var < 0.0f) var = 0.0f;
        mean[r] = mu;
        rstd[r] = 1.0f / sqrtf(var + eps);
    }
}

/* layernorm.py:74-190 with a real beta.  Dequantisation and normalisation are ONE fma per element with two constants
 * per (row, block): a = s*rstd, b = -(mean*rstd), xhat = fmaf(q, a, b), y = fmaf(xhat, gamma, beta)   (this library's
 * definition: the reference dequantises in binary16 first, layernorm.py:131; pinned to torch's layer_norm by tolerance) */
void jfo_layernorm_fwd(const int8_t *q, const float *s, int R, int C, const float *gamma, const float *beta,
                       const float *mean, const float *rstd, int8_t *qy, float *sy)
{
    int SC = C / QB;
    FOR_BLOCKS(R, C) {
        float tmp[QB * QB];
        size_t o = (size_t)rb * QB * C + (size_t)cb * QB;
        float sc = s[rb * SC + cb];
        for (int i = 0; i < QB; ++i)
            for (int j = 0; j < QB; ++j) {
                float a = sc * rstd[rb * QB + i], b = -(mean[rb * QB + i] * rstd[rb * QB + i]);
                float xh = fmaf((float)q[o + (size_t)i * C + j], a, b);
                tmp[i * QB + j] = fmaf(xh, gamma[cb * QB + j], beta ? beta[cb * QB + j] : 0.0f);
            }
        quantize_block(tmp, QB, qy + o, C, &sy[rb * SC + cb], 0, 0, 0, (uint64_t)o, (uint64_t)C, 0.0f, 0);
    }
}

/*
 * LayerNorm backward, full-row (textbook) form of layernorm.py:197-402:
 *   wdy = gamma*dy; c1 = mean_row(xhat*wdy); c2 = mean_row(wdy)
 *   dx = (wdy - fmaf(xhat, c1, c2)) * rstd ;  dgamma = sum_rows dy*xhat ; dbeta = sum_rows dy
 * with xhat = fmaf(q_x, s_x*rstd, -(mean*rstd)) as in the forward and dy = q_g*s_g.
 * Row sums are defined as: 16-column partials (ascending, fmaf / add chain from 0), the two partials of a
 * block added; T_j = sum of the blocks j, j+8, ... ascending; S = ((T0+T1)+(T2+T3)) + ((T4+T5)+(T6+T7)).  c1 = S/C.
 * (The reference reduces c1,c2 over its 128-column tile only, :331-332 -- wrong for C>128.)
 */
void jfo_layernorm_bwd(const int8_t *qx, const float *sx, const int8_t *qg, const float *sg, int R, int C,
                       const float *gamma, const float *mean, const float *rstd,
                       int stochastic, uint64_t seed, uint64_t offset,
                       int8_t *qdx, float *sdx, float *dgamma, float *dbeta)
{
    int SC = C / QB;
    float *c1 = (float *)malloc(sizeof(float) * R), *c2 = (float *)malloc(sizeof(float) * R);
    #pragma omp parallel for schedule(static)
    for (int r = 0; r < R; ++r) {
        /* per block: fma / add chains over columns 0..15 and 16..31, added; per row: T_j = blocks j, j+8, ... ascending,
         * then ((T0+T1)+(T2+T3)) + ((T4+T5)+(T6+T7))  (the order the kernels reduce in) */
        float t1[8] = { 0 }, t2[8] = { 0 };
        float bx = -(mean[r] * rstd[r]);
        for (int cb = 0; cb < SC; ++cb) {
            float ax = sx[(r / QB) * SC + cb] * rstd[r], scg = sg[(r / QB) * SC + cb];
            float h1[2], h2[2];
            for (int h = 0; h < 2; ++h) {
                float p1 = 0.0f, p2 = 0.0f;
                for (int j = 0; j < 16; ++j) {
                    int c = cb * QB + h * 16 + j;
                    float xh = fmaf((float)qx[(size_t)r * C + c], ax, bx);
                    float wdy = gamma[c] * ((float)qg[(size_t)r * C + c] * scg);
                    p1 = fmaf(xh, wdy, p1);
                    p2 = p2 + wdy;
                }
                h1[h] = p1; h2[h] = p2;
            }
            t1[cb & 7] = t1[cb & 7] + (h1[0] + h1[1]);
            t2[cb & 7] = t2[cb & 7] + (h2[0] + h2[1]);
        }
        c1[r] = (((t1[0] + t1[1]) + (t1[2] + t1[3])) + ((t1[4] + t1[5]) + (t1[6] + t1[7]))) / (float)C;
        c2[r] = (((t2[0] + t2[1]) + (t2[2] + t2[3])) + ((t2[4] + t2[5]) + (t2[6] + t2[7]))) / (float)C;
    }
    FOR_BLOCKS(R, C) {
        float tmp[QB * QB];
        size_t o = (size_t)rb * QB * C + (size_t)cb * QB;
        float scx = sx[rb * SC + cb], scg = sg[rb * SC + cb];
        for (int i = 0; i < QB; ++i)
            for (int j = 0; j < QB; ++j) {
                int r = rb * QB + i, c = cb * QB + j;
                float xh = fmaf((float)qx[o + (size_t)i * C + j], scx * rstd[r], -(mean[r] * rstd[r]));
                float wdy = gamma[c] * ((float)qg[o + (size_t)i * C + j] * scg);
                tmp[i * QB + j] = (wdy - fmaf(xh, c1[r], c2[r])) * rstd[r];
            }
        quantize_block(tmp, QB, qdx + o, C, &sdx[rb * SC + cb], stochastic, seed, offset, (uint64_t)o, (uint64_t)C, 0.0f, 0);
    }
    if (dgamma || dbeta) {
        #pragma omp parallel for schedule(static)
        for (int c = 0; c < C; ++c) {
            double a = 0.0, b = 0.0;       /* fp output: tolerance-compared, so a careful sum */
            for (int r = 0; r < R; ++r) {
                float g = (float)qg[(size_t)r * C + c] * sg[(r / QB) * SC + c / QB];
                float xh = fmaf((float)qx[(size_t)r * C + c], sx[(r / QB) * SC + c / QB] * rstd[r], -(mean[r] * rstd[r]));
                a += (double)g * (double)xh; b += (double)g;
            }
            if (dgamma) dgamma[c] = (float)a;
            if (dbeta) dbeta[c] = (float)b;
        }
    }
    free(c1); free(c2);
}

/*
 * Residual add: y1 = x1 + q2*s2 (fp32 out) and its block quantisation.
 * add.py:29-162 (stochastic allowed) / add_mean_var.py:28-177 (+ per-row partial
 * sums of y1 and y1^2 per 32-column block, stored [C/32][R]: two 16-column add / fmaf chains, added).
 * truncate=1 reproduces the reference's `.to(int8)` without llrint (add.py:139).
 */
void jfo_add(const float *x1, const int8_t *q2, const float *s2, int R, int C,
             int stochastic, uint64_t seed, uint64_t offset, int truncate,
             float *y1, int8_t *q, float *s, float *rowsum, float *rowsq)
{
    int SC = C / QB;
    FOR_BLOCKS(R, C) {
        float tmp[QB * QB];
        size_t o = (size_t)rb * QB * C + (size_t)cb * QB;
        float sc = s2[rb * SC + cb];
        for (int i = 0; i < QB; ++i) {
            float a[2] = {0.0f, 0.0f}, b[2] = {0.0f, 0.0f};   /* two 16-column chains, then added */
            for (int j = 0; j < QB; ++j) {
                float v = x1[o + (size_t)i * C + j] + (float)q2[o + (size_t)i * C + j] * sc;
                tmp[i * QB + j] = v;
                y1[o + (size_t)i * C + j] = v;
                a[j / 16] = a[j / 16] + v; b[j / 16] = fmaf(v, v, b[j / 16]);
            }
            if (rowsum) rowsum[(size_t)cb * R + rb * QB + i] = a[0] + a[1];      /* [C/32][R] */
            if (rowsq) rowsq[(size_t)cb * R + rb * QB + i] = b[0] + b[1];
        }
        quantize_block(tmp, QB, q + o, C, &s[rb * SC + cb], stochastic, seed, offset, (uint64_t)o, (uint64_t)C, 0.0f, truncate);
    }
}

/*
 * Column sums of a block tensor: out[c] = sum over all rows of q[r][c] * s[r/32][c/32] -- the bias gradient of a
 * linear layer from its quantised output gradient (the reference only sketches it: grad_bias = G8.sum(0),
 * JetfireGEMMKernel/BlockQuantize/QBlockLinear.py:63-66, which forgets the scales).  The order is this library's
 * definition (an fp32 sum has to have one): per 32-row strip the exact integer sum of the column's codes times the
 * strip's scale (one rounding); partial sum g of 32 adds the strips g, g+32, ... ascending from +0; the 32 partial
 * sums are added ascending.
 */
void jfo_block_colsum(const int8_t *q, const float *s, int R, int C, float *out)
{
    int SC = C / QB, strips = R / QB;
    #pragma omp parallel for schedule(static)
    for (int c = 0; c < C; ++c) {
        float part[32];
        for (int g = 0; g < 32; ++g) {
            float acc = 0.0f;
            for (int rb = g; rb < strips; rb += 32) {
                int isum = 0;
                for (int i = 0; i < QB; ++i) isum += q[(size_t)(rb * QB + i) * C + c];
                acc = acc + (float)isum * s[rb * SC + c / QB];
            }
            part[g] = acc;
        }
        float t = part[0];
        for (int g = 1; g < 32; ++g) t = t + part[g];
        out[c] = t;
    }
}

/* ------------------------------------------------------------------------- */
/* Model of the division shortcut the device kernels use for x/s with a        */
/* block-constant s:  r = 1/s (IEEE), q0 = x*r, e = fmaf(-q0, s, x),            */
/* q1 = fmaf(e, r, q0).  The tests count where q1 differs from the IEEE x/s     */
/* that the functions above use (it must be nowhere on the ranges the kernels   */
/* take this path for).                                                         */
/* ------------------------------------------------------------------------- */
float jfo_model_fast_div(float x, float s)
{
    float r = 1.0f / s;
    float q0 = x * r;
    float e = fmaf(-q0, s, x);
    return fmaf(e, r, q0);
}

/* Model of the device's division of a block maximum by 127 (q0 = a * rn(1/127), e = fmaf(-q0, 127, a),            */
/* q = fmaf(e, rn(1/127), q0)): counts the mantissas, over the binades 2^lo .. 2^hi, for which it differs from the   */
/* IEEE a / 127.0f that the functions above use.                                                                     */
long jfo_model_div127_mismatches(int lo, int hi)
{
    const float r = 1.0f / 127.0f;
    long bad = 0;
    for (int ex = lo; ex <= hi; ++ex)
        for (uint32_t m = 0; m < (1u << 23); ++m) {
            uint32_t bits = ((uint32_t)(127 + ex) << 23) | m;
            float a; memcpy(&a, &bits, 4);
            float q0 = a * r, e = fmaf(-q0, 127.0f, a), q = fmaf(e, r, q0), w = a / 127.0f;
            if (memcmp(&q, &w, 4) != 0) bad++;
        }
    return bad;
}

long jfo_model_fast_div_mismatches(const float *x, const float *s, long n)
{
    long bad = 0;
    for (long i = 0; i < n; ++i) {
        float a = x[i] / s[i], b = jfo_model_fast_div(x[i], s[i]);
        if (memcmp(&a, &b, 4) != 0) bad++;
    }
    return bad;
}
