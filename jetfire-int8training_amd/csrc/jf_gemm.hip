// Per-block INT8 GEMMs for gfx950 (MI355X).
//
//   acc[m,n] = sum over 32-deep K blocks kb (ascending) of  (sa[kb,m/32]*sb[kb,n/32]) * d_kb[m,n]
//   d_kb     = exact INT32 dot product of the kb-th 32-wide slices of A[m,:] and B[n,:]
//
// One v_mfma_i32_32x32x32_i8 produces d_kb for a whole 32x32 output block, i.e. exactly one Jetfire
// quantisation-block product.  (Reference kernels: igemm_BlockSquare32OutputIntQuantizeBiasRowCol.cu:134-225 and
// its siblings under JetfireGEMMKernel/BlockQuantize/cpp_extension/igemm/.)
//
// Scale-accumulate.  The vector ALU is the bottleneck of this kernel, and on this part it runs plain fp32
// add/mul/fma at twice the rate of conversions (v_cvt_f32_i32 included).  So the product is not converted:
// the MFMA's accumulator input is the inline constant 0x3e22f983 (the bit pattern of 1/(2 pi)) in every
// element.  |d| <= 32*127^2 < 2^21 keeps 0x3e22f983 + d inside the binade [1/8, 1/4), whose unit in the last
// place is 2^-26, so  as_float(0x3e22f983 + d) - as_float(0x3e22f983) = d * 2^-26  exactly (one v_sub_f32),
// and  fma(sa*sb*2^26, d*2^-26, acc)  has the same exact product, hence the same rounding, as
// fma(sa*sb, float(d), acc).  The only way the two differ is an overflow of sa*sb*2^26; that is detected
// after the K loop and the wave then recomputes its blocks with the plain sequence (see there).
//
// Work decomposition: workgroup = 8 waves (2 x 4), tile 128x128, each wave owns 64x32 = 2 quantisation
// blocks (32 fp32 accumulators per lane); two workgroups per CU.  K is consumed in stages of 4 blocks (128
// bytes per row) through an LDS ring filled by LDS-direct loads (global_load_lds_dwordx4: no register
// staging).  LDS rows are 128 bytes with an XOR chunk swizzle, so the 16-byte MFMA operand reads are
// conflict-free.  A is K-contiguous; B is either K-contiguous ([N,K]) or [K,N], which is staged as it lies
// in memory and read with the transposing LDS read.  Scales are wave-uniform and are fetched by each wave
// into a private LDS patch.
#include "jf_device.hpp"

#include <atomic>
#include <mutex>
#include <type_traits>

#pragma clang diagnostic ignored "-Winline-asm"     // M0 appears in clobber lists on purpose

namespace jf {

constexpr int KB_STAGE = 4;                         // 32-deep K blocks per LDS stage (128 bytes of K per row)
constexpr int ROW_BYTES = KB_STAGE * QB;            // 128: one LDS row = one 128-byte global segment
constexpr int EPI_LD = 36;                          // floats per staged row (32 + pad, keeps 16B alignment)

// EPI_QG: EPI_Q (deterministic) followed by the GELU forward of the block just requantised: two block tensors leave
// EPI_QB: EPI_Q (stochastic: an activation gradient) followed by the GELU backward of the block just requantised against
//         the saved forward input of the GELU: only the result of the GELU backward leaves
// EPI_QD: EPI_Q followed by the dequantisation of the block just requantised (codes x stored scale), written as float /
//         binary16 / bfloat16: the requantised tensor itself is never written.
enum Epilogue { EPI_S32 = 0, EPI_FP = 1, EPI_Q = 2, EPI_QG = 3, EPI_QB = 4, EPI_QD = 5 };
// Wave-priority schemes of the main loop (launch_gemm_cfg picks one per launch)
enum Pace { PACE_HARDWARE = 0, PACE_EVEN = 1, PACE_ORDERED = 2 };

struct GemmArgs {
    const int8_t *A;      // [M, lda] (K-contiguous) or, for the AKM kernels, [K, lda] (M-contiguous rows)
    const int8_t *B;      // [N, ldb] (K-contiguous) or, for the BKN kernels, [K, ldb] (N-contiguous)
    const void *sa;       // scale of A block (mb, kb) at sa[kb * sa_ks + mb * sa_is]
    const void *sb;       // scale of B block (nb, kb) at sb[kb * sb_ks + nb * sb_is]
    int sa_ks, sa_is, sb_ks, sb_is;
    void *C;              // s32 / fp / s8 [M, N]
    void *sc;             // [M/32, N/32]   (EPI_Q)
    const float *bias;    // [N] or null   (EPI_Q)
    const float *biasmax; // [1] or null   (EPI_Q)
    uint64_t seed, offset;
    int M, N, K, lda, ldb;
    int tiles_m, tiles_n;
    int splits, kb_per_split;   // split-K (EPI_FP only): workgroup w works on K blocks [s*kb_per_split, ...) of tile w % tiles,
                                // s = w / tiles, and stores fp32 partial sums at C + s*M*N
    int out_dtype;        // JF_FP_*        (EPI_FP)
    int rounding;         // JF_ROUND_*     (EPI_Q)
    void *C2, *sc2;       // s8 [M, N], [M/32, N/32]: GELU of the requantised result   (EPI_QG)
    int gelu_approx;      // JF_GELU_*
    float gelu_eps;       // added to the GELU output's block absmax (the reference: 5e-5, gelu_fwd.py:93)
    const int8_t *Xq;     // s8 [M, N]: forward input of the GELU   (EPI_QB)
    const void *Xs;       // [M/32, N/32]
    uint64_t seed2, offset2;   // noise of the GELU backward's own requantisation   (EPI_QB)
    int rounding2;        // JF_ROUND_NEAREST / JF_ROUND_STOCHASTIC   (EPI_QB)
    int pace;             // PACE_*: wave priorities that order the resident workgroups of a CU (set by the launcher, see there)
    unsigned long long *phases;   // PROF kernels: 8 words per workgroup (jf_prof_igemm_block_q), first phase_capacity workgroups
    int phase_capacity;
};

// Logical tile (and K split) of this workgroup.  Workgroups are dealt round-robin to the 8 XCDs, each with a
// private L2: give every XCD one contiguous run of the launch's work, and walk tiles in groups of 8 tile-rows so
// that concurrently resident workgroups of an XCD share A and B panels.  With K splits the order is split-major.
__device__ __forceinline__ void tile_of_workgroup(int tiles_m, int tiles_n, bool has_splits, int &tm, int &tn, int &split)
{
    const int nwg = gridDim.x, wg = blockIdx.x;
    const int xcd = wg & 7, idx = wg >> 3;
    const int per = nwg >> 3, rem = nwg & 7;
    int logical = xcd * per + (xcd < rem ? xcd : rem) + idx;
    split = has_splits ? logical / (tiles_m * tiles_n) : 0;
    logical -= split * (tiles_m * tiles_n);
    constexpr int GROUP = 8;
    const int group_size = GROUP * tiles_n;
    const int g = logical / group_size;
    const int first_m = g * GROUP;
    const int gm = (tiles_m - first_m) < GROUP ? (tiles_m - first_m) : GROUP;
    const int in_group = logical - g * group_size;
    tm = first_m + in_group % gm;
    tn = in_group / gm;
}

// vmcnt(n), no wait on the other counters (gfx9 encoding: vmcnt = bits 3:0 and 15:14)
#define JF_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | 0x0F70)

// WGM x WGN waves, each owning WBM x WBN quantisation blocks (64x32 elements).
constexpr int WBM = 2, WBN = 1;
// NSTAGE = depth of the LDS ring (one stage being computed, NSTAGE-1 in flight); WGPC = workgroups per CU
// (the second launch bound counts waves per SIMD: WGPC workgroups of WGM*WGN waves over 4 SIMDs).
// AKM = 1: A is [K, lda] (M-contiguous rows), staged and read like a [K,N] B operand (below).
// BKN = 0: B is [N, ldb] (K-contiguous rows, like A).  BKN = 1: B is [K, ldb] (N-contiguous rows); its tile is staged
// as it lies in memory and the K-contiguous MFMA operand is produced by the transposing LDS read of gfx950.
static int cu_count();

// PROF = 1: the first wave of every workgroup also records when the workgroup's phases began and ended (wall clock) and
// how many shader cycles its main loop took: a profiling build of the same code, instantiated only in the measurement
// library (jf_prof_igemm_block_q).
template <int EPI, typename ST, int WGM, int WGN, int NSTAGE, int WGPC, int BKN, int AKM = 0, int PROF = 0>
__global__ __launch_bounds__(64 * WGM * WGN, WGPC * WGM * WGN / 4) void igemm_nt_kernel(GemmArgs p_in)
{
    GemmArgs p = p_in;                                        // K-split launches narrow it to the split's K range below
    unsigned long long *const prof_buf = p_in.phases;
    const int prof_cap = p_in.phase_capacity;
    // (a macro, so that the clock is read by the one storing thread only)
#define phase(k, v) do { if (PROF && threadIdx.x == 0 && (int)blockIdx.x < prof_cap) prof_buf[(size_t)blockIdx.x * 8 + (k)] = (v); } while (0)
    if (PROF) {
        phase(0, (unsigned long long)wall_clock64());
        phase(6, (unsigned long long)__builtin_amdgcn_s_getreg((31 << 11) | 4));      // HW_ID: which CU it ran on
    }
    constexpr int NW = WGM * WGN;
    constexpr int BM = QB * WBM * WGM, BN = QB * WBN * WGN;
    constexpr int A_BYTES = BM * ROW_BYTES;                  // one stage of A
    constexpr int STAGE_BYTES = (BM + BN) * ROW_BYTES;
    constexpr int GROUPS = (BM + BN) / 8;                    // 8-row groups (1 KiB each) per stage
    constexpr int LPW = GROUPS / NW;                         // LDS-direct loads per wave per stage
    static_assert(GROUPS % NW == 0, "stage must split evenly over the waves");
    static_assert(NSTAGE >= 2 && NSTAGE <= 5, "ring depth");
    static_assert(!BKN || (BN == ROW_BYTES && WBN == 1), "a staged [K,N] row is one 128-byte LDS row");
    static_assert(!AKM || BM == ROW_BYTES, "a staged [K,M] row is one 128-byte LDS row");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    typedef __attribute__((address_space(3))) unsigned char lds_u8;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave % WGM, wn = wave / WGM;

    int tile_m, tile_n, split;
    tile_of_workgroup(p.tiles_m, p.tiles_n, EPI == EPI_FP && p.splits > 1, tile_m, tile_n, split);
    int kb_base = 0;                                          // first K block of this workgroup (scale indices count from 0)
    if (EPI == EPI_FP && p.splits > 1) {                      // uniform: the same problem on a K range, fp32 partial output
        kb_base = split * p.kb_per_split;
        const int kbn = (p.K / QB - kb_base) < p.kb_per_split ? (p.K / QB - kb_base) : p.kb_per_split;
        p.A += AKM ? (size_t)kb_base * QB * (size_t)p.lda : (size_t)kb_base * QB;
        p.B += BKN ? (size_t)kb_base * QB * (size_t)p.ldb : (size_t)kb_base * QB;
        p.K = kbn * QB;
        p.C = reinterpret_cast<float *>(p.C) + (size_t)split * (size_t)p.M * (size_t)p.N;
        p.out_dtype = JF_FP_F32;
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int SM = p.M / QB, SN = p.N / QB;
    const int nkb = p.K / QB;
    const int nstages = (nkb + KB_STAGE - 1) / KB_STAGE;

    // ---- global -> LDS, without passing through registers ------------------------------------
    // A stage in LDS is (BM+BN) rows of 128 bytes (A rows first).  One load instruction of one wave
    // moves 8 rows: lane l supplies the address of one 16-byte chunk and the hardware writes it to
    // LDS at (base + 16*l), i.e. row l/8, slot l%8.  To keep the later 16-byte operand reads free of
    // bank conflicts, slot c' of row r holds global chunk c' ^ ((r>>1)&7); the permutation stays
    // inside the row's 128-byte segment, so every instruction still reads 8 full 128-byte lines.
    // Address split: the 8-row group of load j is wave-uniform (scalar base pointer, advanced by 128 bytes per
    // stage on the scalar ALU); the lane contributes a fixed offset (its row of the group, its swizzled chunk).
    // The vector ALU is the bottleneck of this kernel, so the loads must not cost vector instructions.
    static_assert(NW % 2 == 0, "the chunk swizzle of a lane must not depend on the load index");
    const int lrow = lane >> 3;
    const int gchunk = (lane & 7) ^ (((wave & 1) * 4 + (lane >> 4)) & 7);     // global chunk this lane fetches
    // A as [K,M]: as for B as [K,N] below (8 K rows x 128 M bytes per load, slot c' of row r holds chunk c' ^ r)
    const int km_chunk = (m0 + (((lane & 7) ^ lrow) << 4)) < p.M ? ((lane & 7) ^ lrow) : 0;
    const unsigned loff_a = AKM ? (unsigned)lrow * (unsigned)p.lda + km_chunk * 16
                                : (unsigned)lrow * (unsigned)p.lda + gchunk * 16;
    // B as [K,N]: a load moves 8 K rows x 128 N bytes (group g of a stage = K rows 8g .. 8g+7 of the stage).  Slot c'
    // of row r holds global chunk c' ^ r, which makes the transposing reads below conflict-free.  Chunks beyond N (partial
    // tile) fetch the tile's first chunk instead (never used).
    const int kn_chunk = (n0 + (((lane & 7) ^ lrow) << 4)) < p.N ? ((lane & 7) ^ lrow) : 0;
    const unsigned loff_b = BKN ? (unsigned)lrow * (unsigned)p.ldb + kn_chunk * 16
                                : (unsigned)lrow * (unsigned)p.ldb + gchunk * 16;
    const int8_t *gbase[LPW];      // wave-uniform: first byte of the group's first row (stage 0)
    bool is_a[LPW];
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
        const int grp = wave + j * NW;
        is_a[j] = grp < BM / 8;
        if (BKN && !is_a[j]) {
            const int k0 = (grp - BM / 8) * 8;                     // K row of the stage (redirected at issue time if beyond K)
            gbase[j] = p.B + (size_t)k0 * (size_t)p.ldb + n0;
        } else if (AKM && is_a[j]) {
            gbase[j] = p.A + (size_t)(grp * 8) * (size_t)p.lda + m0;
        } else {
            int r0 = (is_a[j] ? m0 : n0) + (is_a[j] ? grp : grp - BM / 8) * 8;
            if (r0 >= (is_a[j] ? p.M : p.N)) r0 = is_a[j] ? m0 : n0;   // groups of a partial tile: any valid group
            gbase[j] = (is_a[j] ? p.A : p.B) + (size_t)r0 * (size_t)(is_a[j] ? p.lda : p.ldb);
        }
    }
    // Scales of a stage: every wave fetches, again LDS-direct, the scales it needs itself into a private 256-byte
    // patch (lane l: K block l/16; word l%16 = the wave's WBM A-side scales, then its WBN B-side scales, the rest
    // padding), so that scale reads need no cross-wave synchronisation, every wave has the same number of loads in
    // flight, and one LDS read per K block fetches all of them.  The lane keeps a running pointer.
    constexpr int SCALE_WORDS = 64;
    constexpr int NSC = WBM + WBN;                            // scales per wave and K block
    static_assert(NSC <= 4, "one 16-byte LDS read per K block");
    unsigned char *const scale_ring = smem + NSTAGE * STAGE_BYTES + wave * (NSTAGE * SCALE_WORDS * 4);
    const int s_blk = lane & 15;
    const bool s_is_a = !(s_blk >= WBM && s_blk < NSC);       // padding lanes repeat the first A-side scale
    int s_idx = s_is_a ? m0 / QB + wm * WBM + (s_blk < WBM ? s_blk : 0) : n0 / QB + wn * WBN + s_blk - WBM;
    { const int lim = s_is_a ? SM : SN; s_idx = s_idx < lim ? s_idx : lim - 1; }
    const int s_ks = s_is_a ? p.sa_ks : p.sb_ks, s_is = s_is_a ? p.sa_is : p.sb_is;   // element strides: K block, tile block
    const unsigned char *const s_base = reinterpret_cast<const unsigned char *>(s_is_a ? p.sa : p.sb);
    auto scale_addr = [&](int kbg) {
        const unsigned e = (unsigned)((kbg + kb_base) * s_ks + s_idx * s_is);
        return s_base + e * (unsigned)sizeof(ST);
    };
    const unsigned char *s_ptr = scale_addr((lane >> 4) < nkb ? (lane >> 4) : nkb - 1);
    const unsigned s_step = (unsigned)(KB_STAGE * s_ks) * (unsigned)sizeof(ST);

    constexpr int A_LOADS = (BM / 8) / NW;                    // loads 0 .. A_LOADS-1 of a wave fetch A rows, the rest B rows
    static_assert((BM / 8) % NW == 0, "a load instruction fetches rows of one operand");
    // FULL: the stage has all KB_STAGE K blocks (every stage but a short last one)
    auto issue_stage_as = [&](int stage, auto full_c) {
        constexpr bool FULL = decltype(full_c)::value;
        const unsigned slot_lds = (unsigned)(uintptr_t)(lds_u8 *)smem + (unsigned)(stage % NSTAGE) * STAGE_BYTES;
        const unsigned scale_lds = (unsigned)(uintptr_t)(lds_u8 *)scale_ring + (unsigned)(stage % NSTAGE) * (SCALE_WORDS * 4);
        const int kb0 = stage * KB_STAGE;
        // asm: scalar base + 32-bit lane offset is the addressing mode that costs no vector instruction, and the
        // compiler does not choose it by itself here.  M0 holds the LDS destination of an LDS-direct load.
        if (EPI != EPI_S32) {
            const unsigned char *src = s_ptr;
            if (!FULL) {                                      // missing K blocks: fetch the last one again (never used)
                int kbg = kb0 + (lane >> 4);
                src = scale_addr(kbg < nkb ? kbg : nkb - 1);
            }
            // a binary16 scale is fetched with the 16-bit form (zero-extended into the lane's LDS word): exactly the
            // element's two bytes are read, whatever the parity of its index or the length of the array
            if (sizeof(ST) == 4)
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(src), "s"(scale_lds) : "memory", "m0");
            else
                asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_ushort %0, off" ::"v"(src), "s"(scale_lds) : "memory", "m0");
            s_ptr += s_step;
        }
        unsigned la = loff_a, lb = loff_b;
        if (!FULL && kb0 + (gchunk >> 1) >= nkb) {            // chunks of missing K blocks: the stage's first block again
            if (!AKM) la -= (unsigned)(gchunk >> 1) * QB;
            if (!BKN) lb -= (unsigned)(gchunk >> 1) * QB;
        }
#pragma unroll
        for (int j = 0; j < LPW; ++j) {
            const int grp = wave + j * NW;
            const int8_t *base;                                // wave-uniform
            if (BKN && j >= A_LOADS) {
                base = gbase[j] + (size_t)kb0 * QB * (size_t)p.ldb;
                // K rows of a missing K block: the stage's first group again
                if (!FULL && kb0 * QB + (grp - BM / 8) * 8 >= p.K) base -= (size_t)((grp - BM / 8) * 8) * (size_t)p.ldb;
            } else if (AKM && j < A_LOADS) {
                base = gbase[j] + (size_t)kb0 * QB * (size_t)p.lda;
                if (!FULL && kb0 * QB + grp * 8 >= p.K) base -= (size_t)(grp * 8) * (size_t)p.lda;
            } else {
                base = gbase[j] + (size_t)kb0 * QB;
            }
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         ::"v"(j < A_LOADS ? la : lb), "s"(base), "s"(slot_lds + (unsigned)grp * 1024u) : "memory", "m0");
        }
    };
    auto issue_stage = [&](int stage) {                       // stage < nstages
        if (stage < nkb / KB_STAGE) issue_stage_as(stage, std::true_type{});
        else issue_stage_as(stage, std::false_type{});
    };

    // ---- operand fetch addresses ----------------------------------------------------------------
    // MFMA operand layout: lane l holds row l%32 of the block and K bytes 16*(l/32) .. +15, i.e. chunk
    // 2*kb + l/32 of the stage row.  Both operands use the same mapping, so one offset per K block.
    // (Ring slot, block index and the A/B split are compile-time offsets folded into the instruction.)
    lds_u8 *const lds = (lds_u8 *)smem;
    unsigned fa_u[KB_STAGE], fb_u[KB_STAGE];          // per-lane LDS addresses (ring slot 0), fixed for the whole kernel
#pragma unroll
    for (int kb = 0; kb < KB_STAGE; ++kb) {
        const unsigned fo = (lane & 31) * ROW_BYTES + (((2 * kb + (lane >> 5)) ^ ((lane >> 1) & 7)) << 4);
        fa_u[kb] = (unsigned)(uintptr_t)lds + fo + (wm * WBM * QB) * ROW_BYTES;
        fb_u[kb] = (unsigned)(uintptr_t)lds + A_BYTES + fo + (wn * WBN * QB) * ROW_BYTES;
    }
    // B staged as [K,N]: ds_read_b64_tr_b8 works on groups of 16 lanes; lane i of a group receives byte (i & 7) of the
    // 8-byte rows addressed by lanes (i>>3), (i>>3)+2, ... (i>>3)+14 of the group.  Lanes 2q and 2q+1 address K row q
    // of an 8-row group at N bytes 0..7 and 8..15 of a 16-column strip, so lane i gets 8 consecutive K values of
    // column i: the MFMA operand (lane l: column l%32, K bytes 16*(l/32) .. +15) is two such reads (K rows +0..7, +8..15).
    // The K block and the half are immediates, so one address register serves all of a stage.
    unsigned fb_kn = 0;
    if (BKN) {
        const int g = lane >> 4, r = lane & 15, rho = r >> 1;
        const int c = 2 * wn * WBN + (g & 1);                                    // 16-byte chunk of the N strip
        fb_kn = (unsigned)(uintptr_t)lds + A_BYTES + (g >> 1) * 2048 + ((rho * 8 + (c ^ rho)) << 4) + 8 * (r & 1);
    }
    unsigned fa_km[WBM];                                                             // A staged as [K,M]: the same, per block
#pragma unroll
    for (int i = 0; i < WBM; ++i) {
        const int g = lane >> 4, r = lane & 15, rho = r >> 1;
        const int c = 2 * (wm * WBM + i) + (g & 1);
        fa_km[i] = AKM ? (unsigned)(uintptr_t)lds + (g >> 1) * 2048 + ((rho * 8 + (c ^ rho)) << 4) + 8 * (r & 1) : 0u;
    }
    // scale patch of this wave: a uniform address, parked in a vector register once (LDS reads take a VGPR address)
    unsigned sc_v;
    {
        const unsigned sc_u = (unsigned)(uintptr_t)(lds_u8 *)scale_ring;
        asm volatile("v_mov_b32 %0, %1" : "=v"(sc_v) : "s"(sc_u));
    }

    // ---- accumulators ------------------------------------------------------------------------
    float acc[WBM][WBN][16];
    v16i iacc[WBM][WBN];
#pragma unroll
    for (int i = 0; i < WBM; ++i)
#pragma unroll
        for (int j = 0; j < WBN; ++j) {
#pragma unroll
            for (int v = 0; v < 16; ++v) { acc[i][j][v] = 0.0f; iacc[i][j][v] = 0; }
        }
    // block indices of this wave's scales (clamped for partial tiles: those blocks are never stored)
    int mb[WBM], nb[WBN];
#pragma unroll
    for (int i = 0; i < WBM; ++i) { mb[i] = m0 / QB + wm * WBM + i; mb[i] = mb[i] < SM ? mb[i] : SM - 1; }
#pragma unroll
    for (int j = 0; j < WBN; ++j) { nb[j] = n0 / QB + wn * WBN + j; nb[j] = nb[j] < SN ? nb[j] : SN - 1; }

    // ---- main loop ----------------------------------------------------------------------------
    // The whole ring is filled up front; afterwards the loads of stage s+NSTAGE are issued when the last K block
    // of stage s has been read.  Operand fragments and scales of K block k+1 are read from LDS into a second set
    // of registers BEFORE the products of K block k are issued, so the LDS pipe works while the wave multiplies
    // and accumulates; without this all waves of a SIMD queue at the LDS together and then compute together.
    constexpr int LOADS = LPW + (EPI != EPI_S32 ? 1 : 0);     // LDS-direct loads per wave and stage
    const int nfull = nkb / KB_STAGE;                         // stages with all KB_STAGE blocks
    const int ktail = nkb - nfull * KB_STAGE;                 // K blocks of the short last stage (0: none)
#pragma unroll
    for (int s = 0; s < NSTAGE; ++s)
        if (s < nstages) issue_stage(s);

    // The fragment reads are written as asm so that they stay where they are and so that the wait for them can
    // name a count: the compiler, tracking them itself, waits for ALL outstanding LDS reads (the prefetch included)
    // on every other K block.  LDS reads of a wave return in order, so "at most FETCH_OPS outstanding" after issuing
    // the next K block's reads means that the current K block's have arrived.
    typedef float scale_vec __attribute__((ext_vector_type(NSC == 3 ? 3 : NSC <= 2 ? 2 : 4)));
    v4i fa_reg[2][WBM], fb_reg[2][WBN];
    scale_vec sc_raw[2];
    constexpr int FETCH_OPS = (AKM ? 2 : 1) * WBM + (BKN ? 2 : 1) * WBN + (EPI != EPI_S32 ? 1 : 0);
    static_assert(2 * FETCH_OPS <= 15, "lgkmcnt is a 4-bit counter");
    // pa/pb: this lane's fragment addresses for the K block (ring slot 0); psc: the wave's scale patch;
    // slot_bytes / slot_words: compile-time offset of the ring slot in the tile ring and of the K block in the patch
    // kn_base: runtime offset of the ring slot for the transposing reads (0 where the slot is in the immediates)
    auto fetch = [&](const unsigned pa, const unsigned pb, const unsigned kn_base, const unsigned psc, auto slot_bytes_c,
                     auto kn_off_c, auto slot_words_c, auto buf_c) {
        constexpr int BUF = decltype(buf_c)::value;
        constexpr int SB = decltype(slot_bytes_c)::value, SW = decltype(slot_words_c)::value;
        // the instruction's offset field has 16 bits: slots beyond that are reached through the address register
        constexpr int HI = (SB + (WBM > WBN ? WBM : WBN) * QB * ROW_BYTES) > 65535 ? SB : 0;
        const unsigned pa2 = pa + HI, pb2 = pb + HI;
        constexpr int KO = decltype(kn_off_c)::value;         // slot + K block offset of a [K,N] / [K,M] staging
        if (AKM) {
#pragma unroll
            for (int i = 0; i < WBM; ++i) {
                const unsigned pakm = fa_km[i] + kn_base;
                v2i lo, hi;
                asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(lo) : "v"(pakm), "n"(KO));
                asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(hi) : "v"(pakm), "n"(KO + 1024));
                fa_reg[BUF][i] = v4i{lo.x, lo.y, hi.x, hi.y};
            }
        } else {
#pragma unroll
            for (int i = 0; i < WBM; ++i)
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fa_reg[BUF][i]) : "v"(pa2), "n"(SB - HI + i * (QB * ROW_BYTES)));
        }
        if (BKN) {
            const unsigned pbkn = fb_kn + kn_base;
            v2i lo, hi;
            asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(lo) : "v"(pbkn), "n"(KO));
            asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(hi) : "v"(pbkn), "n"(KO + 1024));
            fb_reg[BUF][0] = v4i{lo.x, lo.y, hi.x, hi.y};
        } else {
#pragma unroll
            for (int j = 0; j < WBN; ++j)
                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(fb_reg[BUF][j]) : "v"(pb2), "n"(SB - HI + j * (QB * ROW_BYTES)));
        }
        if (EPI != EPI_S32) {
            scale_vec &dst = sc_raw[BUF];
            if (NSC == 3) asm volatile("ds_read_b96 %0, %1 offset:%2" : "=v"(dst) : "v"(psc), "n"(SW * 4));
            else if (NSC <= 2) asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(dst) : "v"(psc), "n"(SW * 4));
            else asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(psc), "n"(SW * 4));
        }
    };
    // wait until at most `n` LDS reads are outstanding, and tie register set BUF to that point in program order
    auto fetched = [&](auto n_c, auto buf_c) {
        constexpr int BUF = decltype(buf_c)::value, N = decltype(n_c)::value;
        __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8));        // lgkmcnt(N) only
#pragma unroll
        for (int i = 0; i < WBM; ++i) asm volatile("" : "+v"(fa_reg[BUF][i]));
#pragma unroll
        for (int j = 0; j < WBN; ++j) asm volatile("" : "+v"(fb_reg[BUF][j]));
        if (EPI != EPI_S32) { scale_vec &r = sc_raw[BUF]; asm volatile("" : "+v"(r)); }
    };
    // Products and scale-accumulate of one K block (global index kbg) from register set CUR.
    // The matrix pipe and the vector ALU do not run concurrently on this part, and a product needs about 40 cycles
    // before the vector ALU can read it.  So the accumulation lags the products by one: product n is issued, THEN
    // product n-1 (long finished) is converted and accumulated.  (d_pend, sab_pend) carry the lagging product across
    // K blocks and stages; the first accumulation adds 0*0 and the last product is accumulated after the loop.
    constexpr int NBLK = WBM * WBN;
    constexpr int C_MAGIC = 0x3e22f983;                        // accumulator input of the MFMAs (file header)
    v16i d_pend = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    float sab_pend = 0.0f;
    auto accumulate = [&](auto blk_c) {
        constexpr int i = decltype(blk_c)::value / WBN, j = decltype(blk_c)::value % WBN;
        float t[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) t[v] = __int_as_float(d_pend[v]) - __int_as_float(C_MAGIC);   // = d * 2^-26, exactly
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = __builtin_fmaf(sab_pend, t[v], acc[i][j][v]);
        // pin the accumulation here: the optimiser would otherwise postpone it past the next K blocks and keep their
        // products alive in registers it does not have
#pragma unroll
        for (int v = 0; v < 16; ++v) asm volatile("" : "+v"(acc[i][j][v]));
    };
    auto compute = [&](auto cur_c, const int kbg) {
        constexpr int CUR = decltype(cur_c)::value;
        if (EPI == EPI_S32) {
#pragma unroll
            for (int i = 0; i < WBM; ++i)
#pragma unroll
                for (int j = 0; j < WBN; ++j)
                    iacc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa_reg[CUR][i], fb_reg[CUR][j], iacc[i][j], 0, 0, 0);
        } else {
            float fa[WBM], fb[WBN];
            // a binary16 scale sits in the low half of its word
            auto scale_of = [&](float raw) -> float {
                if (sizeof(ST) == 4) return raw;
                return (float)__builtin_bit_cast(half_t, (uint16_t)__float_as_uint(raw));
            };
#pragma unroll
            for (int i = 0; i < WBM; ++i) fa[i] = scale_of(sc_raw[CUR][i]);
#pragma unroll
            for (int j = 0; j < WBN; ++j) fb[j] = scale_of(sc_raw[CUR][WBM + j]);
            static_for<0, NBLK>([&](auto n_c) {
                constexpr int n = decltype(n_c)::value, i = n / WBN, j = n % WBN;
                // asm: as a builtin operand the constant is hoisted into 16 registers instead of being encoded inline.
                // The compiler therefore does not know this is an MFMA; its result is first read by the accumulate()
                // AFTER the one below (32 vector instructions and another MFMA later), far beyond the wait states
                // a vector read of an MFMA result needs.
                v16i d_new;
                asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, 0x3e22f983" : "=&v"(d_new) : "v"(fa_reg[CUR][i]), "v"(fb_reg[CUR][j]));
                const float sab_new = (fa[i] * fb[j]) * 67108864.0f;       // * 2^26, see accumulate()
                __builtin_amdgcn_sched_barrier(0);
                accumulate(std::integral_constant<int, (n + NBLK - 1) % NBLK>{});
                __builtin_amdgcn_sched_barrier(0);
                d_pend = d_new;
                sab_pend = sab_new;
            });
        }
    };
    // Loads retire in order: stage t has landed once only the loads of the stages issued after it are outstanding.
    auto wait_stage = [&](int t, int last_issued) {
        int younger = (last_issued < nstages - 1 ? last_issued : nstages - 1) - t;
        if (younger >= 4) JF_WAIT_VMCNT(4 * LOADS);
        else if (younger == 3) JF_WAIT_VMCNT(3 * LOADS);
        else if (younger == 2) JF_WAIT_VMCNT(2 * LOADS);
        else if (younger == 1) JF_WAIT_VMCNT(LOADS);
        else JF_WAIT_VMCNT(0);
    };
    using c0 = std::integral_constant<int, 0>;
    wait_stage(0, NSTAGE - 1);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();                              // bare: __syncthreads() would drain every load
    asm volatile("" ::: "memory");
    // A wave whose blocks all lie beyond M or N (the ragged edge of the tile grid: GPT-2 XL's 1600 columns are 12.5
    // tiles) keeps its part in the loads and barriers of the workgroup but neither reads operands nor multiplies: the
    // SIMD it sits on is left to the waves of the other resident workgroup.  ACTIVE = false is that walk.
    const bool wave_active = m0 + wm * (WBM * QB) < p.M && n0 + wn * (WBN * QB) < p.N;        // wave-uniform
    // which of the CU's two workgroup slots this is: the base of its LDS allocation (the low field of the LDS_ALLOC
    // register; its size field starts at bit 12)
    const bool second_slot = (__builtin_amdgcn_s_getreg((31 << 11) | 6) & 0xFFF) != 0;
    long long prof_c0 = 0;
    if (PROF) { phase(1, (unsigned long long)wall_clock64()); prof_c0 = clock64(); }
    auto main_loop = [&](auto active_c, auto pace_c) {
    constexpr bool ACTIVE = decltype(active_c)::value;
    constexpr int PACE = decltype(pace_c)::value;
    if constexpr (ACTIVE) fetch(fa_u[0], fb_u[0], 0u, sc_v, c0{}, c0{}, c0{}, c0{});

    for (int s0 = 0; s0 < nfull; s0 += NSTAGE) static_for<0, NSTAGE>([&](auto slot_c) {
        constexpr int SLOT = decltype(slot_c)::value;         // ring slot of this stage, a compile-time constant
        constexpr int NEXT_SLOT = (SLOT + 1) % NSTAGE;
        const int s = s0 + SLOT;
        if (s >= nfull) return;
        static_for<0, KB_STAGE>([&](auto kb_c) {
            constexpr int kb = decltype(kb_c)::value;
            constexpr int CUR = kb & 1, NXT = CUR ^ 1;
            if constexpr (kb == KB_STAGE - 1) {
                if (s + 1 < nstages) {
                    // Stage hand-over.  This wave's LDS reads of stage s are complete (lgkmcnt 0) and stage s+1 has
                    // landed; after the barrier that holds for every wave, so (a) stage s+1 may be read and (b) the
                    // ring slot of stage s may be overwritten by the loads of stage s+NSTAGE.
                    __builtin_amdgcn_s_waitcnt(0xC07F);       // lgkmcnt(0) only
                    wait_stage(s + 1, s + NSTAGE - 1);
                    asm volatile("" ::: "memory");
                    __builtin_amdgcn_s_barrier();
                    asm volatile("" ::: "memory");
                    if (s + NSTAGE < nstages) issue_stage(s + NSTAGE);
                }
                // unconditional: past the last stage it reads bytes of the ring that nobody uses
                if constexpr (ACTIVE)
                    fetch(fa_u[0], fb_u[0], 0u, sc_v, std::integral_constant<int, NEXT_SLOT * STAGE_BYTES>{},
                          std::integral_constant<int, NEXT_SLOT * STAGE_BYTES>{},
                          std::integral_constant<int, NEXT_SLOT * 64>{}, std::integral_constant<int, NXT>{});
            } else {
                if constexpr (ACTIVE)
                    fetch(fa_u[kb + 1], fb_u[kb + 1], 0u, sc_v, std::integral_constant<int, SLOT * STAGE_BYTES>{},
                          std::integral_constant<int, SLOT * STAGE_BYTES + (kb + 1) * 4096>{},
                          std::integral_constant<int, SLOT * 64 + (kb + 1) * 16>{}, std::integral_constant<int, NXT>{});
            }
            // The arbiter of a SIMD serves its oldest wave first, so the older of two resident workgroups runs about 1.4
            // times as fast as the younger one and the second wave of a workgroup on a SIMD trails the first by a quarter
            // of a stage.  PACE_EVEN: priority rises with the K block of the stage (and falls back at the next stage):
            // all four waves of a SIMD advance together.  PACE_ORDERED: the workgroup in the CU's second LDS slot always
            // goes before the one in the first, and inside a workgroup the wave that is behind goes first.
            if constexpr (PACE == PACE_EVEN) __builtin_amdgcn_s_setprio(kb);
            if constexpr (PACE == PACE_ORDERED && kb == 0) { if (second_slot) __builtin_amdgcn_s_setprio(3); else __builtin_amdgcn_s_setprio(1); }
            if constexpr (PACE == PACE_ORDERED && kb == 2) { if (second_slot) __builtin_amdgcn_s_setprio(2); else __builtin_amdgcn_s_setprio(0); }
            if constexpr (ACTIVE) {
                fetched(std::integral_constant<int, FETCH_OPS>{}, std::integral_constant<int, CUR>{});
                __builtin_amdgcn_sched_barrier(0);            // the reads above stay above the products below,
                compute(std::integral_constant<int, CUR>{}, s * KB_STAGE + kb);
                __builtin_amdgcn_sched_barrier(0);            // and K blocks are scheduled one by one (register pressure)
            }
        });
    });
    if (ACTIVE && ktail) {
        // short last stage (K not a multiple of 128): its first K block is already on its way to register set 0
        const unsigned slot = (unsigned)(nfull % NSTAGE);
        static_for<0, KB_STAGE - 1>([&](auto kb_c) {
            constexpr int kb = decltype(kb_c)::value;
            constexpr int CUR = kb & 1;
            if (kb < ktail) {
                if (kb > 0)
                    fetch(fa_u[kb] + slot * STAGE_BYTES, fb_u[kb] + slot * STAGE_BYTES, slot * STAGE_BYTES, sc_v + slot * 256,
                          c0{}, std::integral_constant<int, kb * 4096>{}, std::integral_constant<int, kb * 16>{},
                          std::integral_constant<int, CUR>{});
                fetched(c0{}, std::integral_constant<int, CUR>{});
                compute(std::integral_constant<int, CUR>{}, nfull * KB_STAGE + kb);
            }
        });
    }
    };
    if (!wave_active) main_loop(std::false_type{}, std::integral_constant<int, PACE_HARDWARE>{});
    else if (p.pace == PACE_EVEN) main_loop(std::true_type{}, std::integral_constant<int, PACE_EVEN>{});
    else if (p.pace == PACE_ORDERED) main_loop(std::true_type{}, std::integral_constant<int, PACE_ORDERED>{});
    else main_loop(std::true_type{}, std::integral_constant<int, PACE_HARDWARE>{});
    __builtin_amdgcn_s_waitcnt(0xC07F);                        // the last, unused prefetch must land before its registers are reused
    if (EPI != EPI_S32 && wave_active) {
        accumulate(std::integral_constant<int, NBLK - 1>{});
        // The scaled factor sa*sb*2^26 overflows when sa*sb >= 2^102.  An infinite factor leaves every accumulator
        // it touches infinite or NaN (inf*0 included), so "some accumulator of the wave is not finite" catches all such
        // cases; the wave then recomputes its blocks the plain way (operands straight from memory, zero accumulator
        // input, v_cvt_f32_i32, unscaled factor), which also reproduces results that really are infinite.
        float chk = 0.0f;
#pragma unroll
        for (int i = 0; i < WBM; ++i)
#pragma unroll
            for (int j = 0; j < WBN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) chk = __builtin_fmaf(acc[i][j][v], 0.0f, chk);
        if (__builtin_expect(__ballot(chk != chk) != 0, 0)) {
            const ST *const sa_t = reinterpret_cast<const ST *>(p.sa), *const sb_t = reinterpret_cast<const ST *>(p.sb);
            static_for<0, NBLK>([&](auto blk_c) {              // compile-time block index: no indexed register arrays
                constexpr int blk = decltype(blk_c)::value, i = blk / WBN, j = blk % WBN;
                const size_t arow = (size_t)(mb[i] * QB + (lane & 31)), bcol = (size_t)(nb[j] * QB + (lane & 31));
                float r[16];
#pragma unroll
                for (int v = 0; v < 16; ++v) r[v] = 0.0f;
#pragma unroll 1
                for (int kb = 0; kb < nkb; ++kb) {
                    const int k0 = kb * QB + 16 * (lane >> 5);
                    v4i fa;
                    if (AKM) {
                        const int8_t *src = p.A + (size_t)k0 * (size_t)p.lda + arow;
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            unsigned w = 0;
#pragma unroll 1
                            for (int q = 0; q < 4; ++q, src += p.lda) w |= (unsigned)(uint8_t)*src << (8 * q);
                            fa[c] = (int)w;
                        }
                    } else {
                        fa = *reinterpret_cast<const v4i *>(p.A + arow * (size_t)p.lda + k0);
                    }
                    v4i fb;
                    if (BKN) {
                        const int8_t *src = p.B + (size_t)k0 * (size_t)p.ldb + bcol;
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            unsigned w = 0;
#pragma unroll 1
                            for (int q = 0; q < 4; ++q, src += p.ldb) w |= (unsigned)(uint8_t)*src << (8 * q);
                            fb[c] = (int)w;
                        }
                    } else {
                        fb = *reinterpret_cast<const v4i *>(p.B + bcol * (size_t)p.ldb + k0);
                    }
                    const v16i z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                    const v16i d = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa, fb, z, 0, 0, 0);
                    const float sab = (float)sa_t[(kb + kb_base) * p.sa_ks + mb[i] * p.sa_is] * (float)sb_t[(kb + kb_base) * p.sb_ks + nb[j] * p.sb_is];
#pragma unroll
                    for (int v = 0; v < 16; ++v) r[v] = __builtin_fmaf(sab, (float)d[v], r[v]);
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = r[v];
            });
        }
    }
    if (PROF) { phase(2, (unsigned long long)wall_clock64()); phase(7, (unsigned long long)(clock64() - prof_c0)); }
    if (p.pace != PACE_HARDWARE) __builtin_amdgcn_s_setprio(0);
    __syncthreads();           // the epilogue reuses the ring as scratch
    if (PROF) phase(3, (unsigned long long)wall_clock64());

    // ---- epilogue ------------------------------------------------------------------------------------------
    // One 32x32 block at a time goes through a wave-private LDS patch that turns the MFMA result layout
    //   (lane l, register v  <->  row 8*(v/4) + 4*(l/32) + v%4, column l%32)
    // into a row layout (lane l <-> row l/2, columns 16*(l%2) .. +15): 16 consecutive columns per lane are what the
    // Philox noise (8 elements per call) and 16-byte packing want.  Results are stored straight from the row layout: 16,
    // 32 or 64 contiguous bytes per lane, two lanes per row of the block (measured 1 % faster than collecting one- and
    // two-byte outputs in a workgroup-wide LDS image of the tile and writing that out in whole rows behind a barrier).
    auto wave_sync = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    float *patch = reinterpret_cast<float *>(smem) + wave * (QB * EPI_LD);
    const int rrow = lane >> 1, rcol = (lane & 1) * 16;
    constexpr bool QUANT = EPI == EPI_Q || EPI == EPI_QG || EPI == EPI_QB || EPI == EPI_QD;
    const float biasmax = (QUANT && p.biasmax) ? p.biasmax[0] : 0.0f;
    float gelu_f0 = 0.0f;                                     // gelu(+0), evaluated on the device like every table entry
    if (EPI == EPI_QG) {
        float zero = 0.0f;
        asm volatile("" : "+v"(zero));
        gelu_f0 = p.gelu_approx == JF_GELU_TANH ? gelu<JF_GELU_TANH>(zero) : gelu<JF_GELU_ERF>(zero);
    }
    // EPI_QB: the saved forward input of this wave's blocks is requested now, so that it has arrived when the
    // requantisation of the first block is done
    v4i xq_codes[WBM][WBN];
    float xq_scale[WBM][WBN];
    if (EPI == EPI_QB) {
        float zero = 0.0f;
        asm volatile("" : "+v"(zero));
        gelu_f0 = p.gelu_approx == JF_GELU_TANH ? dgelu<JF_GELU_TANH>(zero) : dgelu<JF_GELU_ERF>(zero);
#pragma unroll
        for (int i = 0; i < WBM; ++i)
#pragma unroll
            for (int j = 0; j < WBN; ++j) {
                const int bm = m0 + (wm * WBM + i) * QB, bn = n0 + (wn * WBN + j) * QB;
                if (bm < p.M && bn < p.N) {
                    xq_codes[i][j] = *reinterpret_cast<const v4i *>(p.Xq + (size_t)(bm + rrow) * p.N + bn + rcol);
                    xq_scale[i][j] = load_scale(reinterpret_cast<const ST *>(p.Xs), (bm / QB) * SN + bn / QB);
                }
            }
    }

    // 16 consecutive results of a row as float / binary16 / bfloat16 (rounded to nearest even): 64 or 32 contiguous bytes
    auto store_fp = [&](const float (&x)[16], const size_t e0) {
        if (p.out_dtype == JF_FP_F32) {
            v4f *dst = reinterpret_cast<v4f *>(reinterpret_cast<float *>(p.C) + e0);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                v4f t = {x[4 * k], x[4 * k + 1], x[4 * k + 2], x[4 * k + 3]};
                dst[k] = t;
            }
        } else {
            v4i lo, hi;
            if (p.out_dtype == JF_FP_F16) {
                half_t h[16];
#pragma unroll
                for (int k = 0; k < 16; ++k) h[k] = (half_t)x[k];
                lo = *reinterpret_cast<v4i *>(&h[0]); hi = *reinterpret_cast<v4i *>(&h[8]);
            } else {
                __bf16 h[16];
#pragma unroll
                for (int k = 0; k < 16; ++k) h[k] = (__bf16)x[k];
                lo = *reinterpret_cast<v4i *>(&h[0]); hi = *reinterpret_cast<v4i *>(&h[8]);
            }
            v4i *dst = reinterpret_cast<v4i *>(reinterpret_cast<unsigned char *>(p.C) + e0 * 2);   // 32 of a row's 64 bytes
            dst[0] = lo; dst[1] = hi;
        }
    };
#pragma unroll
    for (int i = 0; i < WBM; ++i)
#pragma unroll
        for (int j = 0; j < WBN; ++j) {
            const int bm = m0 + (wm * WBM + i) * QB, bn = n0 + (wn * WBN + j) * QB;
            const bool valid = bm < p.M && bn < p.N;          // wave-uniform
            if (!valid) continue;
            float amax = 0.0f;
            if (QUANT) {
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
            wave_sync();
            if (EPI == EPI_FP && p.out_dtype == JF_FP_F32) {
                // No arithmetic follows, so the patch is read back in the shape that stores best: every store instruction
                // writes 8 whole 128-byte rows of the block instead of 64 separate 16-byte pieces (3-6 us off the weight
                // gradients of GPT-2 XL; the same for 16-bit outputs, 16 rows x 64 bytes per instruction, measured slower
                // than the two 16-byte pieces per lane of the row layout below)
#pragma unroll
                for (int h = 0; h < 4; ++h) {
                    const int row = 8 * h + (lane >> 3), c4 = (lane & 7) * 4;
                    const v4f t = *reinterpret_cast<const v4f *>(patch + row * EPI_LD + c4);
                    *reinterpret_cast<v4f *>(reinterpret_cast<float *>(p.C) + (size_t)(bm + row) * p.N + bn + c4) = t;
                }
                wave_sync();
                continue;
            }
            float x[16];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const v4f t = *reinterpret_cast<const v4f *>(patch + rrow * EPI_LD + rcol + 4 * k);
                x[4 * k] = t.x; x[4 * k + 1] = t.y; x[4 * k + 2] = t.z; x[4 * k + 3] = t.w;
            }
            wave_sync();
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
                store_fp(x, e0);
            } else {
                v4i codes = {0, 0, 0, 0};
                float scale = 0.0f;
                if (amax > 0.0f) {
                    BlockDivisor d(amax);
                    scale = d.fast ? div_by_127_in_range(amax) : amax / 127.0f;      // (uniform)
                    float t[16];
                    if (p.bias) {
#pragma unroll
                        for (int k = 0; k < 16; ++k) x[k] = x[k] + p.bias[bn + rcol + k];
                    }
#pragma unroll
                    for (int k = 0; k < 16; ++k) x[k] = 127.0f * x[k];
                    d.div16(x, t);
                    if (p.rounding == JF_ROUND_STOCHASTIC) {
                        float n[16];
                        sr_noise16(p.seed, p.offset, (uint64_t)e0, n);
#pragma unroll
                        for (int k = 0; k < 16; ++k) t[k] = t[k] + n[k];
                    }
                    codes.x = (int)round_clamp_pack4(t[0], t[1], t[2], t[3]);
                    codes.y = (int)round_clamp_pack4(t[4], t[5], t[6], t[7]);
                    codes.z = (int)round_clamp_pack4(t[8], t[9], t[10], t[11]);
                    codes.w = (int)round_clamp_pack4(t[12], t[13], t[14], t[15]);
                }
                if (EPI == EPI_QB) {
                    // GELU backward of the gradient block as a reader of the stored tensor would see it (codes x the scale
                    // rounded to ST) against the saved forward input, with the wave's patch (free again) as the code table
                    const float stored = (float)(ST)scale;
                    float scale2;
                    codes = p.gelu_approx == JF_GELU_TANH
                        ? gelu_bwd_block<JF_GELU_TANH>(xq_codes[i][j], xq_scale[i][j], codes, stored, gelu_f0, patch, lane,
                                                       p.rounding2, p.seed2, p.offset2, (uint64_t)e0, &scale2)
                        : gelu_bwd_block<JF_GELU_ERF>(xq_codes[i][j], xq_scale[i][j], codes, stored, gelu_f0, patch, lane,
                                                      p.rounding2, p.seed2, p.offset2, (uint64_t)e0, &scale2);
                    scale = scale2;
                    wave_sync();                              // the table is the next block's patch
                }
                if (EPI == EPI_QD) {
                    // the block as a reader of the stored tensor would dequantise it: codes x the scale rounded to ST
                    float y[16];
                    unpack16(codes, (float)(ST)scale, y);
                    store_fp(y, e0);
                } else {
                    *reinterpret_cast<v4i *>(reinterpret_cast<int8_t *>(p.C) + e0) = codes;     // 16 of a row's 32 bytes
                    if (lane == 0) store_scale(reinterpret_cast<ST *>(p.sc), (bm / QB) * SN + bn / QB, scale);
                }
                if (EPI == EPI_QG) {
                    // GELU of the block as a reader of the stored tensor would see it (codes x the scale rounded to ST),
                    // with the wave's patch (free again) as the code tables
                    const float stored = (float)(ST)scale;
                    float *tab = patch;
                    int *qtab = reinterpret_cast<int *>(patch + 256);
                    float scale2;
                    const v4i codes2 = p.gelu_approx == JF_GELU_TANH
                        ? gelu_fwd_block<JF_GELU_TANH>(codes, stored, gelu_f0, p.gelu_eps, tab, qtab, lane, &scale2)
                        : gelu_fwd_block<JF_GELU_ERF>(codes, stored, gelu_f0, p.gelu_eps, tab, qtab, lane, &scale2);
                    *reinterpret_cast<v4i *>(reinterpret_cast<int8_t *>(p.C2) + e0) = codes2;
                    if (lane == 0) store_scale(reinterpret_cast<ST *>(p.sc2), (bm / QB) * SN + bn / QB, scale2);
                    wave_sync();                              // the tables are the next block's patch
                }
            }
        }

    if (PROF) phase(4, (unsigned long long)wall_clock64());
    if (PROF) phase(5, (unsigned long long)wall_clock64());
#undef phase
}

// -------------------------------------------------------------------------------------------------
// int8 transpose: out[C,R] = in[R,C].  TR_ROWS x 64 tiles through LDS: 16-byte loads, the transposing LDS read of gfx950
// (ds_read_b64_tr_b8, as for the GEMM's [K,N] operands) and 16-byte stores.  The instruction works on groups of 16 lanes:
// lanes 2k and 2k+1 of a group address the 8-byte pieces [8 columns] x 2 of tile row k (k = 0..7), and lane i receives
// byte i%8 of the pieces addressed by lanes i/8, i/8 + 2, ..., i/8 + 14: column i of the 16, rows 0..7.  Two reads (rows
// +0..7, +8..15) give a lane 16 consecutive bytes of one output row.  Wave w of the workgroup takes tile columns 16w ..
// 16w+15 (16 output rows); its four lane groups take 16 tile rows each, so a store instruction writes 64 contiguous bytes
// of each of its 16 output rows, and the passes of a tall tile continue those runs.
constexpr int TR_ROWS = 64;                        // tile rows (input rows = bytes per output-row run)
__global__ __launch_bounds__(256) void transpose_s8_kernel(const int8_t *in, int8_t *out, int R, int C)
{
    __shared__ __attribute__((aligned(16))) unsigned char tile[TR_ROWS][64 + 16];
    typedef __attribute__((address_space(3))) unsigned char lds_u8;
    const int tiles_c = (C + 63) / 64;
    // Workgroups are dealt round-robin to the 8 XCDs: with 8 consecutive workgroups on 8 consecutive row tiles of one
    // column tile, every XCD walks along the columns of its own rows, so the two 64-byte halves of a 128-byte line meet
    // in one L2 (measured at 8192x6400: 17.8 us against 24.4 us with the column tile running fastest).
    const int tiles_r = (R + TR_ROWS - 1) / TR_ROWS;
    const int per = 8 * tiles_c, grp = blockIdx.x / per, rem = blockIdx.x % per;
    const int nr = (tiles_r - grp * 8) < 8 ? (tiles_r - grp * 8) : 8;
    const int tr = grp * 8 + rem % nr, tc = rem / nr;
    const int r0 = tr * TR_ROWS, c0 = tc * 64;
    const int tid = threadIdx.x;
#pragma unroll
    for (int pass = 0; pass < TR_ROWS / 64; ++pass) {
        const int row = pass * 64 + (tid >> 2), ch = tid & 3;   // 64 rows x 4 chunks of 16 bytes per pass
        v4i v = {0, 0, 0, 0};
        if (r0 + row < R && c0 + ch * 16 < C)
            v = *reinterpret_cast<const v4i *>(in + (size_t)(r0 + row) * C + c0 + ch * 16);
        *reinterpret_cast<v4i *>(&tile[row][ch * 16]) = v;
    }
    __syncthreads();
    const int lane = tid & 63, wave = tid >> 6;
    const int g = lane >> 4, i = lane & 15;
    const int ocol = 16 * wave + (i & 7) + 8 * (i >> 3);        // tile column this lane receives = output row
#pragma unroll
    for (int pass = 0; pass < TR_ROWS / 64; ++pass) {
        const int trow = pass * 64 + 16 * g;                    // first of the 16 tile rows of this lane group
        const unsigned addr = (unsigned)(uintptr_t)(lds_u8 *)&tile[trow + (i >> 1)][16 * wave + 8 * (i & 1)];
        v2i lo, hi;
        asm volatile("ds_read_b64_tr_b8 %0, %1" : "=v"(lo) : "v"(addr));
        asm volatile("ds_read_b64_tr_b8 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "n"(8 * (64 + 16)));
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo), "+v"(hi));
        if (c0 + ocol < C && r0 + trow < R)
            *reinterpret_cast<v4i *>(out + (size_t)(c0 + ocol) * R + r0 + trow) = v4i{lo.x, lo.y, hi.x, hi.y};
    }
}

static int launch_transpose(const int8_t *in, int R, int C, int8_t *out, hipStream_t st)
{
    const int tiles = ((R + TR_ROWS - 1) / TR_ROWS) * ((C + 63) / 64);
    hipLaunchKernelGGL(transpose_s8_kernel, dim3(tiles), dim3(256), 0, st, in, out, R, C);
    return (int)hipGetLastError();
}

template <int EPI, typename ST, int WGM, int WGN, int NSTAGE, int WGPC, int BKN, int AKM = 0, int PROF = 0>
static int launch_gemm_cfg(const GemmArgs &a, hipStream_t st)
{
    constexpr int BM = QB * WBM * WGM, BN = QB * WBN * WGN, NT = 64 * WGM * WGN;
    constexpr int RING = NSTAGE * (BM + BN) * ROW_BYTES + WGM * WGN * NSTAGE * 256;   // operand ring + per-wave scale patches
    constexpr int PATCH = WGM * WGN * QB * EPI_LD * (int)sizeof(float);     // the epilogue's per-wave transposition patches
    constexpr int SMEM = RING > PATCH ? RING : PATCH;
    if (!device_is_gfx950()) return JF_ERR_DEVICE;
    GemmArgs p = a;
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BN - 1) / BN;
    auto kern = igemm_nt_kernel<EPI, ST, WGM, WGN, NSTAGE, WGPC, BKN, AKM, PROF>;
    // more than 64 KiB of dynamic LDS has to be opted into, per function and device: once, not on every launch
    // (the reference sets its attribute on every call, igemm_BlockSquare32OutputIntQuantizeBiasRowCol.cu:418)
    static std::atomic<bool> opted_in[MAX_DEVICES] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return JF_ERR_DEVICE;
    if (!opted_in[dev].load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
        if (e != hipSuccess) return (int)e;
        opted_in[dev].store(true, std::memory_order_release);
    }
    if (EPI != EPI_FP || p.splits < 1) p.splits = 1;
    // Pace of the workgroups that share a CU.  Left to the hardware, the older one runs ahead: a launch ends with every CU
    // half empty while the younger workgroups finish alone, at two thirds of the shared throughput (two waves per SIMD
    // meeting at a barrier).  Kept in step by wave priorities (PACE_EVEN) they finish together: 5-16 % faster for launches
    // of up to two rounds of workgroups.  The exception is a launch of between 1 and 1.5 rounds: there the early finishers
    // are what starts the short second round early, and an even pace is 5-9 % slower than the hardware's order.  A strict
    // order with fairness inside each workgroup (PACE_ORDERED) does that job 4-6 % better than the hardware when tiles are
    // long (K >= 4096) and 5-16 % worse when they are short.  Beyond two rounds the schemes are within 3 % of each other,
    // either way depending on shape and data: left to the hardware.  (All measured; results do not depend on the scheme.)
    const long wgs = (long)p.tiles_m * p.tiles_n * p.splits, slots = (long)WGPC * cu_count();
    const bool short_second_round = wgs > slots && 2 * wgs < 3 * slots;
    const int k_per_wg = p.splits > 1 ? p.kb_per_split * QB : p.K;
    p.pace = short_second_round ? (k_per_wg >= 4096 ? PACE_ORDERED : PACE_HARDWARE)
                                : (wgs <= 2 * slots ? PACE_EVEN : PACE_HARDWARE);
    hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n * p.splits), dim3(NT), SMEM, st, p);
    return (int)hipGetLastError();
}

// out[i] = convert(part[0][i] + part[1][i] + ... + part[S-1][i]), added in ascending split order.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *part, size_t n, int splits, void *out, int out_dtype)
{
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= n) return;                                        // n is a multiple of 1024
    v4f t = *reinterpret_cast<const v4f *>(part + i);
    for (int s = 1; s < splits; ++s) {
        const v4f u = *reinterpret_cast<const v4f *>(part + (size_t)s * n + i);
        t.x = t.x + u.x; t.y = t.y + u.y; t.z = t.z + u.z; t.w = t.w + u.w;
    }
    if (out_dtype == JF_FP_F32) {
        *reinterpret_cast<v4f *>(reinterpret_cast<float *>(out) + i) = t;
    } else if (out_dtype == JF_FP_F16) {
        half_t h[4] = {(half_t)t.x, (half_t)t.y, (half_t)t.z, (half_t)t.w};
        *reinterpret_cast<v2i *>(reinterpret_cast<half_t *>(out) + i) = *reinterpret_cast<v2i *>(h);
    } else {
        __bf16 h[4] = {(__bf16)t.x, (__bf16)t.y, (__bf16)t.z, (__bf16)t.w};
        *reinterpret_cast<v2i *>(reinterpret_cast<__bf16 *>(out) + i) = *reinterpret_cast<v2i *>(h);
    }
}

// compute units of the current device (asked once per device; 256 if the query fails)
static int cu_count()
{
    static std::atomic<int> known[MAX_DEVICES] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return 256;
    int cus = known[dev].load(std::memory_order_relaxed);
    if (cus == 0) {
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        known[dev].store(cus, std::memory_order_relaxed);
    }
    return cus;
}

// K split of the fp-output GEMM.  request 1: none; request > 1: that many parts (fewer if K is short); request 0: as
// many parts as it takes to give every CU two workgroups, when the tiles alone fill less than half of them.  Parts are
// whole multiples of 4 K blocks (one LDS stage), at least 16 K blocks long.
static void splitk_plan(int M, int N, int K, int request, int &splits, int &kb_per_split)
{
    const int nkb = K / QB;
    int want = request;
    if (request == 0) {
        const int tiles = ((M + 127) / 128) * ((N + 127) / 128), slots = 2 * cu_count();
        want = 2 * tiles <= slots ? slots / tiles : 1;
        if (want > 16) want = 16;
    }
    if (want > nkb / 16) want = nkb / 16;
    if (want < 1) want = 1;
    kb_per_split = ((nkb + want - 1) / want + 3) / 4 * 4;
    splits = (nkb + kb_per_split - 1) / kb_per_split;
}

// Tile configuration: 128x128 tiles, 8 waves, a 2-deep ring and two workgroups per CU (the epilogue of one overlaps
// the main loop of the other).  A [K,N] B operand (and, for the weight gradient, a [K,M] A operand) is read in place.
// a_km (A given as [K,M]) exists for the weight-gradient form only: fp output, B as [K,N].
template <int EPI, typename ST> static int launch_gemm(const GemmArgs &a, hipStream_t st, bool b_kn, bool a_km = false)
{
    if constexpr (EPI == EPI_QG) {                            // the forward form only: A [M,K], B [N,K]
        if (a_km || b_kn) return JF_ERR_UNSUPPORTED;
        return launch_gemm_cfg<EPI, ST, 2, 4, 2, 2, 0>(a, st);
    } else if constexpr (EPI == EPI_QB) {                     // the activation-gradient form only: A [M,K], B [K,N]
        if (a_km || !b_kn) return JF_ERR_UNSUPPORTED;
        return launch_gemm_cfg<EPI, ST, 2, 4, 2, 2, 1>(a, st);
    } else {
        if (a_km) {
            if constexpr (EPI == EPI_FP) {
                if (b_kn) return launch_gemm_cfg<EPI, ST, 2, 4, 2, 2, 1, 1>(a, st);
            }
            return JF_ERR_UNSUPPORTED;
        }
#ifdef JF_PROF_LIB
        if constexpr (EPI == EPI_Q && std::is_same<ST, float>::value) {
            if (a.phases)                                     // the profiling library: the PROF build of the same kernel
                return b_kn ? launch_gemm_cfg<EPI, ST, 2, 4, 2, 2, 1, 0, 1>(a, st) : launch_gemm_cfg<EPI, ST, 2, 4, 2, 2, 0, 0, 1>(a, st);
        }
#endif
        return b_kn ? launch_gemm_cfg<EPI, ST, 2, 4, 2, 2, 1>(a, st) : launch_gemm_cfg<EPI, ST, 2, 4, 2, 2, 0>(a, st);
    }
}

static int check_gemm_common(const void *A, const void *B, const void *C, int M, int N, int K, int b_layout)
{
    if (!A || !B || !C) return JF_ERR_NULL;
    if (!mult32(M) || !mult32(N) || !mult32(K)) return JF_ERR_SHAPE;
    if (b_layout != JF_B_NK && b_layout != JF_B_KN) return JF_ERR_ENUM;
    if (!aligned16(A) || !aligned16(B) || !aligned16(C)) return JF_ERR_ALIGN;
    return JF_OK;
}

}  // namespace jf

using namespace jf;

// element strides (K block, tile block) of a scale operand with `blocks` tile blocks
static bool scale_strides(int layout, int K, int blocks, int &ks, int &is)
{
    if (layout == JF_SCALES_KMAJOR) { ks = blocks; is = 1; return true; }
    if (layout == JF_SCALES_ROWMAJOR) { ks = 1; is = K / QB; return true; }
    return false;
}

// scale arrays need the natural alignment of their element type (binary16 scales are fetched one element at a time)
static bool scale_ptr_ok(const void *p, int scale_dtype)
{
    return (reinterpret_cast<uintptr_t>(p) & (scale_dtype == JF_SCALE_F32 ? 3u : 1u)) == 0;
}

#ifndef JF_PROF_LIB
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
    case JF_ERR_UNSUPPORTED: return "jetfire_hip: this combination of operand layouts is not implemented";
    case JF_ERR_SCRATCH_LIMIT: return "jetfire_hip: the K split of this problem needs more than the built-in scratch buffer (JF_NOALLOC_SCRATCH_BYTES); use jf_igemm_block_fp with a workspace, or splitk = 1";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "jetfire_hip: unknown error";
    }
}

int jf_philox_rounds(void) { return PHILOX_ROUNDS; }

size_t jf_igemm_workspace_bytes(int M, int N, int K, int b_layout)
{
    (void)M; (void)N; (void)K; (void)b_layout;                // both B layouts are read in place
    return 0;
}

int jf_igemm_s32(const int8_t *A, const int8_t *B, int32_t *C, int M, int N, int K, int b_layout,
                 void *workspace, size_t workspace_bytes, jf_stream_t stream)
{
    (void)workspace; (void)workspace_bytes;
    int rc = check_gemm_common(A, B, C, M, N, K, b_layout);
    if (rc) return rc;
    const bool kn = b_layout == JF_B_KN;
    GemmArgs a = {};
    a.A = A; a.B = B; a.C = C; a.M = M; a.N = N; a.K = K; a.lda = K; a.ldb = kn ? N : K;
    return launch_gemm<EPI_S32, float>(a, (hipStream_t)stream, kn);
}

int jf_igemm_block_acc(const int8_t *A, const int8_t *B, int32_t *acc, int M, int N, int K, int b_layout,
                       void *workspace, size_t workspace_bytes, jf_stream_t stream)
{
    (void)workspace; (void)workspace_bytes;
    int rc = check_gemm_common(A, B, acc, M, N, K, b_layout);
    if (rc) return rc;
    const bool kn = b_layout == JF_B_KN;
    for (int kb = 0; kb < K / QB; ++kb) {
        GemmArgs a = {};
        a.A = A + kb * QB; a.B = kn ? B + (size_t)kb * QB * N : B + kb * QB; a.C = acc + (size_t)kb * M * N;
        a.M = M; a.N = N; a.K = QB; a.lda = K; a.ldb = kn ? N : K;
        if ((rc = launch_gemm<EPI_S32, float>(a, (hipStream_t)stream, kn))) return rc;
    }
    return JF_OK;
}

int jf_igemm_splitk_plan(int M, int N, int K, int splitk, int *splits, int *kb_per_split)
{
    if (!mult32(M) || !mult32(N) || !mult32(K)) return JF_ERR_SHAPE;
    if (splitk < 0 || !splits || !kb_per_split) return splitk < 0 ? JF_ERR_ENUM : JF_ERR_NULL;
    splitk_plan(M, N, K, splitk, *splits, *kb_per_split);
    return JF_OK;
}

size_t jf_igemm_block_fp_workspace_bytes(int M, int N, int K, int b_layout, int splitk)
{
    (void)b_layout;
    int splits = 1, kb_per = 0;
    if (jf_igemm_splitk_plan(M, N, K, splitk, &splits, &kb_per) != JF_OK) return 0;
    return splits > 1 ? (size_t)splits * (size_t)M * (size_t)N * sizeof(float) : 0;
}

// The fp-output GEMM behind both of its entry points.  partials: fp32 [splits][M][N] scratch for the K split (only
// touched when the plan has more than one part; every element of it that is read has been written by this call).
static int block_fp_run(const int8_t *A, const int8_t *B, const void *sa, const void *sb, void *C, int M, int N, int K,
                        int a_layout, int b_layout, int scale_dtype, int sa_layout, int sb_layout, int out_dtype,
                        int splits, int kb_per, void *partials, hipStream_t st)
{
    GemmArgs a = {};
    const bool a_km = a_layout == JF_A_KM, kn = b_layout == JF_B_KN;
    a.A = A; a.B = B; a.sa = sa; a.sb = sb; a.C = C; a.M = M; a.N = N; a.K = K; a.lda = a_km ? M : K; a.ldb = kn ? N : K;
    if (!scale_strides(sa_layout, K, M / QB, a.sa_ks, a.sa_is) || !scale_strides(sb_layout, K, N / QB, a.sb_ks, a.sb_is))
        return JF_ERR_ENUM;
    a.out_dtype = out_dtype;
    a.splits = splits; a.kb_per_split = kb_per;
    if (splits > 1) a.C = partials;
    int rc = scale_dtype == JF_SCALE_F16 ? launch_gemm<EPI_FP, half_t>(a, st, kn, a_km) : launch_gemm<EPI_FP, float>(a, st, kn, a_km);
    if (rc || splits == 1) return rc;
    const size_t n = (size_t)M * (size_t)N;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)(n / 1024)), dim3(256), 0, st, (const float *)partials, n, splits, C, out_dtype);
    return (int)hipGetLastError();
}

static int block_fp_check(const int8_t *A, const int8_t *B, const void *sa, const void *sb, void *C, int M, int N, int K,
                          int a_layout, int b_layout, int scale_dtype, int out_dtype)
{
    int rc = check_gemm_common(A, B, C, M, N, K, b_layout);
    if (rc) return rc;
    if (a_layout != JF_A_MK && a_layout != JF_A_KM) return JF_ERR_ENUM;
    if (!sa || !sb) return JF_ERR_NULL;
    if ((scale_dtype != JF_SCALE_F16 && scale_dtype != JF_SCALE_F32) ||
        (out_dtype != JF_FP_F16 && out_dtype != JF_FP_F32 && out_dtype != JF_FP_BF16)) return JF_ERR_ENUM;
    if (!scale_ptr_ok(sa, scale_dtype) || !scale_ptr_ok(sb, scale_dtype)) return JF_ERR_ALIGN;
    return JF_OK;
}

int jf_igemm_block_fp(const int8_t *A, const int8_t *B, const void *sa, const void *sb, void *C,
                      int M, int N, int K, int a_layout, int b_layout, int scale_dtype, int sa_layout, int sb_layout,
                      int out_dtype, int splitk, void *workspace, size_t workspace_bytes, jf_stream_t stream)
{
    int rc = block_fp_check(A, B, sa, sb, C, M, N, K, a_layout, b_layout, scale_dtype, out_dtype);
    if (rc) return rc;
    int splits = 1, kb_per = 0;
    if ((rc = jf_igemm_splitk_plan(M, N, K, splitk, &splits, &kb_per))) return rc;
    if (splits > 1 && (!workspace || !aligned16(workspace) || workspace_bytes < jf_igemm_block_fp_workspace_bytes(M, N, K, b_layout, splitk)))
        return JF_ERR_WORKSPACE;
    return block_fp_run(A, B, sa, sb, C, M, N, K, a_layout, b_layout, scale_dtype, sa_layout, sb_layout, out_dtype, splits,
                        kb_per, workspace, (hipStream_t)stream);
}

// ---- the allocation-free weight-gradient entry point ---------------------------------------------------------------
// Scratch of the K split, for callers that cannot hand over a workspace: one array per device, resident until the
// process ends.  In host code `noalloc_scratch` is only a handle; the device address is looked up once per device.
}  // extern "C"
static __device__ __align__(256) unsigned char noalloc_scratch[JF_NOALLOC_SCRATCH_BYTES];
namespace {
std::mutex noalloc_mu;
void *noalloc_ptr[jf::MAX_DEVICES] = {};                       // device address of noalloc_scratch, per device
// rc = 0 and *out = this device's copy of the array (looked up on the first call on the device, with it current)
int noalloc_scratch_of_current_device(void **out)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= jf::MAX_DEVICES) return JF_ERR_DEVICE;
    std::lock_guard<std::mutex> g(noalloc_mu);
    if (!noalloc_ptr[dev]) {
        void *ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(noalloc_scratch));
        if (e != hipSuccess) return (int)e;
        if (!ptr) return JF_ERR_DEVICE;
        noalloc_ptr[dev] = ptr;
    }
    *out = noalloc_ptr[dev];
    return JF_OK;
}
}  // namespace
extern "C" {

int jf_igemm_block_fp_noalloc(const int8_t *A, const int8_t *B, const void *sa, const void *sb, void *C,
                              int M, int N, int K, int a_layout, int b_layout, int scale_dtype, int sa_layout,
                              int sb_layout, int out_dtype, int splitk, jf_stream_t stream)
{
    int rc = block_fp_check(A, B, sa, sb, C, M, N, K, a_layout, b_layout, scale_dtype, out_dtype);
    if (rc) return rc;
    int splits = 1, kb_per = 0;
    if ((rc = jf_igemm_splitk_plan(M, N, K, splitk, &splits, &kb_per))) return rc;
    void *partials = nullptr;
    if (splits > 1) {
        if ((size_t)splits * (size_t)M * (size_t)N * sizeof(float) > (size_t)JF_NOALLOC_SCRATCH_BYTES) return JF_ERR_SCRATCH_LIMIT;
        if ((rc = noalloc_scratch_of_current_device(&partials))) return rc;
    }
    // nothing in the scratch has to start at zero: every part stores its whole [M][N] partial result before the
    // reduction reads it, so what an earlier (larger) call left behind is never read
    return block_fp_run(A, B, sa, sb, C, M, N, K, a_layout, b_layout, scale_dtype, sa_layout, sb_layout, out_dtype, splits,
                        kb_per, partials, (hipStream_t)stream);
}

int jf_igemm_block_q(const int8_t *A, const int8_t *B, const void *sa, const void *sb,
                     const float *bias, const float *biasmax, int8_t *C, void *sc,
                     int M, int N, int K, int b_layout, int scale_dtype, int sa_layout, int sb_layout, int rounding,
                     uint64_t seed, uint64_t offset,
                     void *workspace, size_t workspace_bytes, jf_stream_t stream)
{
    (void)workspace; (void)workspace_bytes;
    int rc = check_gemm_common(A, B, C, M, N, K, b_layout);
    if (rc) return rc;
    if (!sa || !sb || !sc) return JF_ERR_NULL;
    if ((scale_dtype != JF_SCALE_F16 && scale_dtype != JF_SCALE_F32) ||
        (rounding != JF_ROUND_NEAREST && rounding != JF_ROUND_STOCHASTIC)) return JF_ERR_ENUM;
    if (!scale_ptr_ok(sa, scale_dtype) || !scale_ptr_ok(sb, scale_dtype)) return JF_ERR_ALIGN;
    const bool kn = b_layout == JF_B_KN;
    GemmArgs a = {};
    a.A = A; a.B = B; a.sa = sa; a.sb = sb; a.C = C; a.sc = sc; a.bias = bias; a.biasmax = biasmax;
    a.M = M; a.N = N; a.K = K; a.lda = K; a.ldb = kn ? N : K; a.rounding = rounding; a.seed = seed; a.offset = offset;
    if (!scale_strides(sa_layout, K, M / QB, a.sa_ks, a.sa_is) || !scale_strides(sb_layout, K, N / QB, a.sb_ks, a.sb_is))
        return JF_ERR_ENUM;
    hipStream_t st = (hipStream_t)stream;
    return scale_dtype == JF_SCALE_F16 ? launch_gemm<EPI_Q, half_t>(a, st, kn) : launch_gemm<EPI_Q, float>(a, st, kn);
}

int jf_igemm_block_q_dequant(const int8_t *A, const int8_t *B, const void *sa, const void *sb, const float *bias,
                             const float *biasmax, void *out, int M, int N, int K, int b_layout, int scale_dtype,
                             int sa_layout, int sb_layout, int out_dtype, int rounding, uint64_t seed, uint64_t offset,
                             jf_stream_t stream)
{
    int rc = check_gemm_common(A, B, out, M, N, K, b_layout);
    if (rc) return rc;
    if (!sa || !sb) return JF_ERR_NULL;
    if ((scale_dtype != JF_SCALE_F16 && scale_dtype != JF_SCALE_F32) ||
        (rounding != JF_ROUND_NEAREST && rounding != JF_ROUND_STOCHASTIC) ||
        (out_dtype != JF_FP_F16 && out_dtype != JF_FP_F32 && out_dtype != JF_FP_BF16)) return JF_ERR_ENUM;
    if (!scale_ptr_ok(sa, scale_dtype) || !scale_ptr_ok(sb, scale_dtype)) return JF_ERR_ALIGN;
    const bool kn = b_layout == JF_B_KN;
    GemmArgs a = {};
    a.A = A; a.B = B; a.sa = sa; a.sb = sb; a.C = out; a.bias = bias; a.biasmax = biasmax; a.out_dtype = out_dtype;
    a.M = M; a.N = N; a.K = K; a.lda = K; a.ldb = kn ? N : K; a.rounding = rounding; a.seed = seed; a.offset = offset;
    if (!scale_strides(sa_layout, K, M / QB, a.sa_ks, a.sa_is) || !scale_strides(sb_layout, K, N / QB, a.sb_ks, a.sb_is))
        return JF_ERR_ENUM;
    hipStream_t st = (hipStream_t)stream;
    return scale_dtype == JF_SCALE_F16 ? launch_gemm<EPI_QD, half_t>(a, st, kn) : launch_gemm<EPI_QD, float>(a, st, kn);
}

int jf_igemm_block_q_gelu(const int8_t *A, const int8_t *B, const void *sa, const void *sb, const float *bias,
                          const float *biasmax, int8_t *C, void *sc, int8_t *C_gelu, void *sc_gelu, int M, int N, int K,
                          int scale_dtype, int sa_layout, int sb_layout, int gelu_approx, float gelu_amax_eps,
                          jf_stream_t stream)
{
    int rc = check_gemm_common(A, B, C, M, N, K, JF_B_NK);
    if (rc) return rc;
    if (!sa || !sb || !sc || !C_gelu || !sc_gelu) return JF_ERR_NULL;
    if ((scale_dtype != JF_SCALE_F16 && scale_dtype != JF_SCALE_F32) ||
        (gelu_approx != JF_GELU_ERF && gelu_approx != JF_GELU_TANH)) return JF_ERR_ENUM;
    if (!aligned16(C_gelu) || !scale_ptr_ok(sa, scale_dtype) || !scale_ptr_ok(sb, scale_dtype)) return JF_ERR_ALIGN;
    GemmArgs a = {};
    a.A = A; a.B = B; a.sa = sa; a.sb = sb; a.C = C; a.sc = sc; a.bias = bias; a.biasmax = biasmax;
    a.C2 = C_gelu; a.sc2 = sc_gelu; a.gelu_approx = gelu_approx; a.gelu_eps = gelu_amax_eps;
    a.M = M; a.N = N; a.K = K; a.lda = K; a.ldb = K; a.rounding = JF_ROUND_NEAREST;
    if (!scale_strides(sa_layout, K, M / QB, a.sa_ks, a.sa_is) || !scale_strides(sb_layout, K, N / QB, a.sb_ks, a.sb_is))
        return JF_ERR_ENUM;
    hipStream_t st = (hipStream_t)stream;
    return scale_dtype == JF_SCALE_F16 ? launch_gemm<EPI_QG, half_t>(a, st, false) : launch_gemm<EPI_QG, float>(a, st, false);
}

int jf_igemm_block_q_gelu_bwd(const int8_t *A, const int8_t *B, const void *sa, const void *sb, const int8_t *Xq,
                              const void *Xs, int8_t *C, void *sc, int M, int N, int K, int scale_dtype, int sa_layout,
                              int sb_layout, int gelu_approx, uint64_t seed, uint64_t offset, int gelu_rounding,
                              uint64_t gelu_seed, uint64_t gelu_offset, jf_stream_t stream)
{
    int rc = check_gemm_common(A, B, C, M, N, K, JF_B_KN);
    if (rc) return rc;
    if (!sa || !sb || !sc || !Xq || !Xs) return JF_ERR_NULL;
    if ((scale_dtype != JF_SCALE_F16 && scale_dtype != JF_SCALE_F32) ||
        (gelu_approx != JF_GELU_ERF && gelu_approx != JF_GELU_TANH) ||
        (gelu_rounding != JF_ROUND_NEAREST && gelu_rounding != JF_ROUND_STOCHASTIC)) return JF_ERR_ENUM;
    if (!aligned16(Xq) || !scale_ptr_ok(sa, scale_dtype) || !scale_ptr_ok(sb, scale_dtype) || !scale_ptr_ok(Xs, scale_dtype))
        return JF_ERR_ALIGN;
    GemmArgs a = {};
    a.A = A; a.B = B; a.sa = sa; a.sb = sb; a.C = C; a.sc = sc; a.Xq = Xq; a.Xs = Xs;
    a.M = M; a.N = N; a.K = K; a.lda = K; a.ldb = N;
    a.rounding = JF_ROUND_STOCHASTIC; a.seed = seed; a.offset = offset;
    a.gelu_approx = gelu_approx; a.rounding2 = gelu_rounding; a.seed2 = gelu_seed; a.offset2 = gelu_offset;
    if (!scale_strides(sa_layout, K, M / QB, a.sa_ks, a.sa_is) || !scale_strides(sb_layout, K, N / QB, a.sb_ks, a.sb_is))
        return JF_ERR_ENUM;
    hipStream_t st = (hipStream_t)stream;
    return scale_dtype == JF_SCALE_F16 ? launch_gemm<EPI_QB, half_t>(a, st, true) : launch_gemm<EPI_QB, float>(a, st, true);
}

int jf_transpose_s8(const int8_t *in, int R, int C, int8_t *out, jf_stream_t stream)
{
    if (!in || !out) return JF_ERR_NULL;
    if (R <= 0 || C <= 0 || (R % 16) || (C % 16)) return JF_ERR_SHAPE;
    if (!aligned16(in) || !aligned16(out)) return JF_ERR_ALIGN;
    if (!device_is_gfx950()) return JF_ERR_DEVICE;
    return launch_transpose(in, R, C, out, (hipStream_t)stream);
}

}  // extern "C"
#else   // JF_PROF_LIB: libjetfire_prof.so

#include "../../include/jetfire_prof.h"

// jf_igemm_block_q with fp32 scales through the PROF instantiation of the kernel: same arithmetic, same bits, plus the
// per-workgroup phase record (include/jetfire_prof.h).
extern "C" int jf_prof_igemm_block_q(const int8_t *A, const int8_t *B, const float *sa, const float *sb, const float *bias,
                                     const float *biasmax, int8_t *C, float *sc, int M, int N, int K, int b_layout,
                                     int sa_layout, int sb_layout, int rounding, uint64_t seed, uint64_t offset,
                                     unsigned long long *phases, int capacity_workgroups, jf_stream_t stream)
{
    int rc = check_gemm_common(A, B, C, M, N, K, b_layout);
    if (rc) return rc;
    if (!sa || !sb || !sc || !phases) return JF_ERR_NULL;
    if (capacity_workgroups <= 0) return JF_ERR_SHAPE;
    if (rounding != JF_ROUND_NEAREST && rounding != JF_ROUND_STOCHASTIC) return JF_ERR_ENUM;
    const bool kn = b_layout == JF_B_KN;
    GemmArgs a = {};
    a.A = A; a.B = B; a.sa = sa; a.sb = sb; a.C = C; a.sc = sc; a.bias = bias; a.biasmax = biasmax;
    a.M = M; a.N = N; a.K = K; a.lda = K; a.ldb = kn ? N : K; a.rounding = rounding; a.seed = seed; a.offset = offset;
    if (!scale_strides(sa_layout, K, M / QB, a.sa_ks, a.sa_is) || !scale_strides(sb_layout, K, N / QB, a.sb_ks, a.sb_is))
        return JF_ERR_ENUM;
    a.phases = phases;
    a.phase_capacity = capacity_workgroups;
    return launch_gemm<EPI_Q, float>(a, (hipStream_t)stream, kn);
}

#endif  // JF_PROF_LIB
