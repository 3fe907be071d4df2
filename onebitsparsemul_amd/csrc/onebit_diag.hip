// Diagnostic of libonebitmul: the sustained SMFMAC rate of this GPU in a register-only loop (no LDS, no global
// memory inside the timed loop). The chip lowers its clock under matrix load, and by how much depends on the
// operand values, so this is the practical ceiling the main kernel can be compared with next to the nominal peak.
// No counterpart in the reference.
#include "onebit_sparse_tuning.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cmath>
#include <vector>

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half16_t __attribute__((ext_vector_type(16)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4v_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void smfmac_rate_kernel(float* out, const half8_t* pa, const half16_t* pb,
                                                          const int* pidx, int iters) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  half8_t a[4];
  half16_t b[4];
  int idx[4];
  for (int i = 0; i < 4; ++i) {
    a[i] = pa[t * 4 + i];
    b[i] = pb[t * 4 + i];
    idx[i] = pidx[t * 4 + i];
  }
  float16_t acc[16];
  for (int j = 0; j < 16; ++j)
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j)
      acc[j] = __builtin_amdgcn_smfmac_f32_32x32x32_f16(a[j & 3], b[(j >> 2) & 3], acc[j], idx[j & 3], 0, 0);
  }
  float s = 0.f;
  for (int j = 0; j < 16; ++j)
    for (int i = 0; i < 16; ++i) s += acc[j][i];
  out[t] = s;
}

// The same loop on v_smfmac_f32_16x16x64_f16, the instruction of the default large tile and of the sixteen-column
// split-K kernel: 16 independent 16 x 16 accumulator tiles per wavefront, 32768 dense-equivalent FLOPs per instruction.
__global__ __launch_bounds__(256) void smfmac_rate_kernel_16x16x64(float* out, const half8_t* pa, const half16_t* pb,
                                                                   const int* pidx, int iters) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  half8_t a[4];
  half16_t b[4];
  int idx[4];
  for (int i = 0; i < 4; ++i) {
    a[i] = pa[t * 4 + i];
    b[i] = pb[t * 4 + i];
    idx[i] = pidx[t * 4 + i];
  }
  float4v_t acc[16];
  for (int j = 0; j < 16; ++j) acc[j] = float4v_t{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 16; ++j)
      acc[j] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a[j & 3], b[(j >> 2) & 3], acc[j], idx[j & 3], 0, 0);
  }
  float s = 0.f;
  for (int j = 0; j < 16; ++j)
    for (int i = 0; i < 4; ++i) s += acc[j][i];
  out[t] = s;
}

uint32_t lcg(uint32_t& state) {
  state = state * 1664525u + 1013904223u;
  return state >> 8;
}

}  // namespace

extern "C" int onebit_sparse_measure_smfmac_rate_shape(int shape, int random_operands, int iterations,
                                                       double* dense_equiv_tflops) {
  if (!dense_equiv_tflops || iterations <= 0) return ONEBIT_ERR_ARGUMENT;
  if (shape != ONEBIT_SMFMAC_32X32X32 && shape != ONEBIT_SMFMAC_16X16X64) return ONEBIT_ERR_ARGUMENT;
  auto kernel = shape == ONEBIT_SMFMAC_16X16X64 ? smfmac_rate_kernel_16x16x64 : smfmac_rate_kernel;
  const double flops_per_instruction = shape == ONEBIT_SMFMAC_16X16X64 ? 2.0 * 16 * 16 * 64 : 2.0 * 32 * 32 * 32;
  int device = 0, cus = 0;
  if (hipGetDevice(&device) != hipSuccess) return ONEBIT_ERR_HIP;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return ONEBIT_ERR_HIP;
  const int blocks = cus;  // one workgroup of four wavefronts per CU = one wavefront per SIMD
  const size_t threads = (size_t)blocks * 256;
  std::vector<_Float16> ha(threads * 32), hb(threads * 64);
  std::vector<int> hi(threads * 4);
  const int legal[6] = {0x4, 0x8, 0x9, 0xC, 0xD, 0xE};
  uint32_t st = 12345u;
  for (auto& v : ha) v = (_Float16)(random_operands ? ((lcg(st) & 1) ? 1.0f : -1.0f) : 1.0f);
  for (auto& v : hb) {
    const float u1 = (lcg(st) + 1.0f) / 16777217.0f, u2 = (lcg(st) + 1.0f) / 16777217.0f;
    v = (_Float16)(random_operands ? std::sqrt(-2.0f * std::log(u1)) * std::cos(6.2831853f * u2) : 0.5f);
  }
  for (auto& v : hi) {
    int w = 0;
    for (int g = 0; g < 8; ++g) w |= (random_operands ? legal[lcg(st) % 6] : 0x4) << (4 * g);
    v = w;
  }
  float* out = nullptr;
  half8_t* pa = nullptr;
  half16_t* pb = nullptr;
  int* pidx = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  int rc = ONEBIT_ERR_HIP;
  float ms = 0.f;
  if (hipMalloc(&out, threads * 4) != hipSuccess) goto done;
  if (hipMalloc(&pa, ha.size() * 2) != hipSuccess) goto done;
  if (hipMalloc(&pb, hb.size() * 2) != hipSuccess) goto done;
  if (hipMalloc(&pidx, hi.size() * 4) != hipSuccess) goto done;
  if (hipMemcpy(pa, ha.data(), ha.size() * 2, hipMemcpyHostToDevice) != hipSuccess) goto done;
  if (hipMemcpy(pb, hb.data(), hb.size() * 2, hipMemcpyHostToDevice) != hipSuccess) goto done;
  if (hipMemcpy(pidx, hi.data(), hi.size() * 4, hipMemcpyHostToDevice) != hipSuccess) goto done;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) goto done;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), 0, nullptr, out, pa, pb, pidx, 200);
  if (hipDeviceSynchronize() != hipSuccess) goto done;
  if (hipEventRecord(e0, nullptr) != hipSuccess) goto done;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), 0, nullptr, out, pa, pb, pidx, iterations);
  if (hipEventRecord(e1, nullptr) != hipSuccess) goto done;
  if (hipDeviceSynchronize() != hipSuccess) goto done;
  if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) goto done;
  *dense_equiv_tflops = (double)blocks * 4 * iterations * 16 * flops_per_instruction / (ms * 1e-3) / 1e12;
  rc = ONEBIT_OK;
done:
  // clean-up failures leave nothing to undo and do not change the measurement's outcome
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  (void)hipFree(out);
  (void)hipFree(pa);
  (void)hipFree(pb);
  (void)hipFree(pidx);
  return rc;
}

extern "C" int onebit_sparse_measure_smfmac_rate(int random_operands, int iterations, double* dense_equiv_tflops) {
  return onebit_sparse_measure_smfmac_rate_shape(ONEBIT_SMFMAC_32X32X32, random_operands, iterations, dense_equiv_tflops);
}

extern "C" int onebit_sparse_device_info(int* compute_units, int* clock_khz) {
  if (!compute_units || !clock_khz) return ONEBIT_ERR_ARGUMENT;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return ONEBIT_ERR_HIP;
  if (hipDeviceGetAttribute(compute_units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return ONEBIT_ERR_HIP;
  if (hipDeviceGetAttribute(clock_khz, hipDeviceAttributeClockRate, device) != hipSuccess) return ONEBIT_ERR_HIP;
  return ONEBIT_OK;
}
