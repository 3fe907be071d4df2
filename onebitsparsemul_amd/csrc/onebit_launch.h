// Host-visible launch interface of the gfx950 kernels (internal to libonebitmul).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace onebit {

struct GemmArgs {
  const uint8_t* prep;   // prepared A operand
  const _Float16* b;     // K x N row-major fp16
  const void* c;         // M x N row-major source (read only when beta != 0)
  void* d;               // M x N row-major destination
  int m, n, k;
  int kc_total;          // 256-wide K chunks in the prepared operand
  float alpha, beta;
  int c_f16, d_f16;      // 1: fp16, 0: fp32
  int tiles_m, tiles_n;  // filled by the launcher
};

struct SkinnyArgs {
  const uint8_t* prep;
  const _Float16* b;
  const void* c;
  void* d;
  float* partials;  // splits x m x n fp32 (unused when splits == 1)
  int* counters;    // one arrival counter per row group, zero between calls
  int m, n, k;
  int kc_total;
  int splits;       // ceil(kc_total / SK)
  float alpha, beta;
  int c_f16, d_f16;
};

enum TileConfig { kTile512x128 = 0, kTile256x128 = 1, kTile128x128 = 2, kTile256x256 = 3, kTileAuto = -1 };

hipError_t launch_prepare(const void* a, const void* e, void* prep, int m, int k, int layout, hipStream_t stream);
hipError_t launch_gemm(GemmArgs args, int tile_config, hipStream_t stream);

// Split-K kernel for n <= 32. sk = K chunks (of 256) per workgroup, one of 1, 2, 4, 8.
int skinny_rows_per_group();
int skinny_pick_sk(int m, int k);
hipError_t launch_skinny(SkinnyArgs args, int sk, hipStream_t stream);

}  // namespace onebit
