/*
 * jetfire_prof.h -- C ABI of libjetfire_prof.so: measurement aids for the gfx950 kernels of libjetfire_hip.so.
 *
 * Nothing here has a counterpart in the reference and nothing here is part of the drop-in boundary: the benchmark uses
 * these entry points to say where the GEMM's time goes and what the hardware allows.  The library is built from the
 * same kernel source as the product library (the PROF instantiation of igemm_nt_kernel) plus register-only
 * calibration loops.  Conventions (device pointers, streams, return codes) as in jetfire_hip.h.
 */
#ifndef JETFIRE_PROF_H
#define JETFIRE_PROF_H

#include "jetfire_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* jf_igemm_block_q (fp32 scales) through a build of its kernel that also records, per workgroup w < capacity_workgroups
 * (a workgroup computes one 128x128 output tile), 8 64-bit words at phases[8*w]:
 *   [0] start  [1] main loop begins  [2] main loop ends  [3] epilogue begins  [4] blocks requantised  [5] end
 *       (ticks of the constant-rate wall clock, jf_wall_clock_khz)
 *   [6] the hardware id register of its first wave (which CU it ran on)
 *   [7] shader-clock cycles its main loop took ([7] / ([2]-[1]) = the clock the shader ran at under this load).
 * `phases`: device memory of 8 * capacity_workgroups words.  The results (C, sc) are the same bits as jf_igemm_block_q's. */
int jf_prof_igemm_block_q(const int8_t *A, const int8_t *B, const float *sa, const float *sb, const float *bias,
                          const float *biasmax, int8_t *C, float *sc, int M, int N, int K, int b_layout,
                          int sa_layout, int sb_layout, int rounding, uint64_t seed, uint64_t offset,
                          unsigned long long *phases, int capacity_workgroups, jf_stream_t stream);

/* Calibration: launches `workgroups` x `threads` (128, 256, 384 or 512) threads; per iteration every wave runs 4 work
 * items from registers, an item being
 *   JF_CAL_UNIFORM: [one 32x32x32 INT8 MFMA if with_mfma] + [valu_per_mfma independent v_fmac_f32]
 *                   supported (with_mfma, valu_per_mfma): (1,0) (0,32) (1,32) (0,16) (1,16);
 *   JF_CAL_SPLIT:   the MFMA in the first half of a workgroup's waves, 32 v_fmac_f32 in the second half (1, 32): with
 *                   512 threads the two kinds of wave share each SIMD;
 *   JF_CAL_STREAM:  the GEMM's K-block instruction stream (1, 32): MFMA with the constant accumulator input, then 16
 *                   subtractions and 16 v_fmac_f32 on the previous product;
 *   JF_CAL_STREAM_DATA: the same stream (1, 32) on operands that change with every MFMA and use all 8 bits, and a
 *                   scale with a full mantissa: the clock rate the stream sustains when the datapaths toggle as on
 *                   real tensors (launch it long enough, tens of milliseconds, for the clock to settle).
 * `scratch`: a device buffer of at least 4 bytes (never written in practice).  `clocks` (may be NULL): 2 x workgroups
 * 64-bit words; workgroup w's first wave stores the shader-clock cycles and the wall-clock ticks (constant rate,
 * hipDeviceAttributeWallClockRate) it ran for, which gives the clock the shader ran at under this load. */
#define JF_CAL_UNIFORM 0
#define JF_CAL_SPLIT   1
#define JF_CAL_STREAM  2
#define JF_CAL_STREAM_DATA 3
int jf_calibrate(int mode, int with_mfma, int valu_per_mfma, int iters, int workgroups, int threads, float *scratch,
                 unsigned long long *clocks, jf_stream_t stream);

/* Rate of the constant clock the kernels' wall-clock readings count in, kHz (0 if the device does not report one). */
int jf_wall_clock_khz(void);

#ifdef __cplusplus
}
#endif
#endif /* JETFIRE_PROF_H */
