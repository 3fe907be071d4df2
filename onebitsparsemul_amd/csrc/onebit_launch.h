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
  int xcds;              // filled by the launcher: XCDs the workgroups are dealt over (workgroup b runs on XCD b % xcds)
  int vector_epilogue;   // filled by the launcher: C and D allow 16-byte accesses
  // K split over workgroups (grid.y = splits): split s multiplies the K chunks [s * chunks_per_split, +chunks_per_split)
  // and writes raw fp32 sums to split_ws + s * m * n; a second kernel adds the splits in order and applies the
  // epilogue. splits <= 1: one pass straight into d. split_ws: at least splits * m * n floats, 16-byte aligned.
  int splits;
  int chunks_per_split;
  float* split_ws;
  // B whose rows are not 16-byte aligned (n % 8 != 0, or a base address that is not) cannot feed the asynchronous
  // 16-byte copies. If b_pad is set (at least k * round_up(n, 8) halves, 16-byte aligned), the launcher first copies
  // B into it with rows padded to a multiple of 8 columns and the main kernel reads that; otherwise such operands
  // take the slower element-copy variant. ldb (elements between B rows) is filled by the launcher.
  _Float16* b_pad;
  int ldb;
  // linear-layer form (launch_gemm_tokens) only: m values added to every token's row of y, may be null
  const void* bias;
  int bias_f16;
};

struct SkinnyArgs {
  const uint8_t* prep;
  const _Float16* b;
  const void* c;
  void* d;
  int m, n, k;
  int kc_total;
  float alpha, beta;
  int c_f16, d_f16;
  // token-major form (launch_skinny_tokens) only: b is x (n tokens x k), d is y (n tokens x m), alpha, beta and c are
  // not used, bias (m values, may be null) is added to every token's row
  const void* bias;
  int bias_f16;
  // K split over workgroups (grid.y = splits), for few row groups over a long K: split s multiplies the K chunks
  // [s * chunks_per_split, +chunks_per_split) and writes raw fp32 sums to split_ws + s * m * n (laid out like the
  // result); a second kernel adds the splits in order and applies the epilogue. splits <= 1: one pass straight into d.
  int splits;
  int chunks_per_split;
  float* split_ws;
};

// Several token-major products with the same token count in one launch of the split-K kernel (no K split over
// workgroups); first_block is filled by the launcher.
constexpr int kSkinnyMaxGroup = 16;
struct SkinnyGroupArgs {
  SkinnyArgs problem[kSkinnyMaxGroup];
  int first_block[kSkinnyMaxGroup + 1];
  int count;
};

enum TileConfig { kTile512x128 = 0, kTile256x128 = 1, kTile128x128 = 2, kTile256x256 = 3, kTile256x128w = 4, kTile512x128t = 5, kTile128x128s = 6, kTile256x64 = 7, kTile256x256w8 = 8, kTile512x128w8 = 9, kTile256x128w8 = 10, kTile128x128w8 = 11, kTile64x128 = 12, kTile128x128k2 = 13, kTile64x128k2 = 14, kTile512x128m16 = 15, kTileAuto = -1 };

hipError_t launch_prepare(const void* a, const void* e, void* prep, int m, int k, int layout, hipStream_t stream);
hipError_t launch_gemm(GemmArgs args, int tile_config, hipStream_t stream);
// The linear layer's form of the main kernel: b is x (n tokens x k, token-major, 16-byte aligned), d is y (n tokens x
// m), y = x W^T + bias; c, alpha, beta and the padded copy of B are not used, splits / chunks_per_split / split_ws as in
// launch_gemm. Tiles 4, 6, 9, 10, 11, 12, 13, 14, 15.
hipError_t launch_gemm_tokens(GemmArgs args, int tile_config, hipStream_t stream);
// dense fp16 (m x k) -> one-bit values `a` and metadata `e`; prune != 0 applies the 2:4 magnitude mask first
hipError_t launch_pack(const void* w, void* a, void* e, int m, int k, int prune, int layout, hipStream_t stream);

// Split-K kernel for n <= 64; rows_per_group (32, 64 or 128) = weight rows one workgroup covers (n > 32: at most 64).
constexpr int kSkinnyMaxN = 64;
hipError_t launch_skinny(SkinnyArgs args, int rows_per_group, hipStream_t stream);
// The linear layer's form of the same kernel: y[t][r] = sum_k W[r][k] x[t][k] + bias[r] for n <= 64 tokens, x and y
// token-major (x 16-byte aligned).
hipError_t launch_skinny_tokens(SkinnyArgs args, int rows_per_group, hipStream_t stream);
// count <= kSkinnyMaxGroup problems of the same form, each with its own weight, x, bias, y, m and k, in one launch.
hipError_t launch_skinny_group(SkinnyGroupArgs group, int rows_per_group, hipStream_t stream);

}  // namespace onebit
