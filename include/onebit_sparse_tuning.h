/*
 * Tuning hooks, test hooks and diagnostics of libonebitmul. None of them has a counterpart in the reference; a
 * program that only replaces the reference's library needs include/onebit_sparse_tensor.h alone. They are exported by
 * the same shared library and are what the tests and the benchmark of this build use to reach every kernel variant.
 */
#ifndef ONEBIT_SPARSE_TUNING_H_
#define ONEBIT_SPARSE_TUNING_H_

#include "onebit_sparse_tensor.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Tuning / test hooks: force a tile configuration of the main kernel (-1 = automatic) and choose whether
 * shapes with n <= 32 (n <= 64 when m <= 40960) use the split-K kernel (1, default) or the main kernel (0).
 * Tile codes 0-15 are the TileConfig values of csrc/onebit_launch.h (the linear-layer form has 4, 6, 9-15).
 * These five hooks act on the calling thread only: the calls that thread makes afterwards. A hook set on one thread
 * does not change what another thread launches (worker threads of a data-parallel wrapper, autograd threads). */
void onebit_sparse_set_tile_config(int tile_config);
void onebit_sparse_set_skinny_enabled(int enabled);
/* Weight rows one workgroup of the split-K kernel covers: 32, 64 or 128; <= 0 = automatic. */
void onebit_sparse_set_skinny_rows(int rows);
/* K splits over workgroups, of the main kernel and of the split-K kernel (which also splits K among the wavefronts
 * of a workgroup): 1 = never split, N > 1 = N splits (at most one per 256 of K), <= 0 = automatic (few tiles or row
 * groups and a long K). A split call writes fp32 partial sums to a library-owned buffer kept per
 * device and stream (grown with hipMalloc on first use: warm up before capturing the call in a HIP graph) and adds
 * them in split order, so results do not depend on timing. */
void onebit_sparse_set_split_k(int splits);
/* B whose rows are not 16-byte aligned (n % 8 != 0 or an unaligned base) and n beyond the split-K kernel's range:
 * 1 (default) = the main kernel reads a copy of B with rows padded to a multiple of 8 columns, made by one extra
 * pass into a library-owned buffer kept per device and stream (same rules as the K-split buffer); 0 = the main
 * kernel's element-copy variant reads B in place (much slower; always used when k * n < 65536). */
void onebit_sparse_set_pad_b(int enabled);

/* Diagnostic: what a prepared call of this shape would launch under the calling thread's hooks. The plan is made for
 * the compute-unit count of the current device, as the calls themselves do; without a usable device (a host without a
 * GPU) for 256 compute units, the MI355X figure. plan[0] = 1 for the split-K kernel (n <= 64), 0 for the main kernel;
 * plan[1] = weight rows per workgroup (split-K kernel) or the tile code (main kernel); plan[2] = K splits over
 * workgroups (1 = none); plan[3] = 1 if B is read through a padded copy. onebit_sparse_describe_launch_for does the
 * same for an explicit compute-unit count and never touches a device. */
int onebit_sparse_describe_launch(int m, int n, int k, int b_16_byte_aligned, int *plan);
int onebit_sparse_describe_launch_for(int m, int n, int k, int b_16_byte_aligned, int compute_units, int *plan);

/* Diagnostic: sustained rate of one SMFMAC instruction in a register-only loop on the current device (one wavefront
 * per SIMD, `iterations` x 16 instructions each on 16 independent accumulator tiles, no LDS or global memory inside
 * the loop), in dense-equivalent TFLOP/s. shape: ONEBIT_SMFMAC_32X32X32 = v_smfmac_f32_32x32x32_f16 (the
 * eight-wavefront tiles), ONEBIT_SMFMAC_16X16X64 = v_smfmac_f32_16x16x64_f16 (the default large tile and the
 * sixteen-column split-K kernel). random_operands = 1 uses +-1 values, N(0,1) fp16 B values and random 2:4 indices
 * (the benchmark's distribution), 0 uses constants. The clock the GPU sustains under matrix load depends on the
 * operand values and on the instruction, so this is the practical ceiling next to the nominal peak. Allocates and
 * frees its own device buffers; synchronous. onebit_sparse_measure_smfmac_rate is the 32x32x32 shape. */
#define ONEBIT_SMFMAC_32X32X32 0
#define ONEBIT_SMFMAC_16X16X64 1
int onebit_sparse_measure_smfmac_rate_shape(int shape, int random_operands, int iterations, double *dense_equiv_tflops);
int onebit_sparse_measure_smfmac_rate(int random_operands, int iterations, double *dense_equiv_tflops);

/* Diagnostic: compute units and peak engine clock (kHz) of the current device, the two figures the SMFMAC peak is
 * computed from (units x clock x 4096 dense fp16 FLOP per clock per unit x 2). */
int onebit_sparse_device_info(int *compute_units, int *clock_khz);

#ifdef __cplusplus
}
#endif

#endif /* ONEBIT_SPARSE_TUNING_H_ */
