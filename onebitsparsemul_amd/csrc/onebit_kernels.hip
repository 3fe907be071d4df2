// gfx950 kernels of the one-bit 2:4 sparse GEMM  D = alpha * A * B + beta * C.
//   prepare_kernel  : reference operands (1-bit values, reordered 2-bit-index metadata) -> prepared operand
//   pack_kernel     : dense fp16 weight -> the reference operands (2:4 magnitude mask, compression, one-bit values)
//   gemm_kernel     : main SMFMAC kernel (B staged through LDS, A expanded in registers)
//   skinny_kernel   : split-K kernel for N <= 64 (decode shapes)
//   pad_b_kernel, splitk_reduce_kernel : helpers of the main kernel (unaligned B rows; K split over workgroups)
// The two GEMM kernels also come in a token-major form for the linear layer, y = x W^T + bias with x and y stored
// token by token (the transposes of B and D).
// Replaces the CUTLASS specialisations of the reference (csrc/kernel.h:13-72, csrc/threadblock.h:62-233,
// csrc/warp.h:18-690) with code written for 64-wide wavefronts; nothing is translated from them.
#include "onebit_device.h"
#include "onebit_launch.h"
#include <atomic>
#include <type_traits>

namespace onebit {

// =====================================================================================================
// prepare_kernel: one wavefront per prepared block (rb, kc).
// Reads  a : bit (r, j) of the (m x k/2) column-major one-bit matrix = bit (r + j m) % 8 of byte (r + j m) / 8
//            (csrc/kernel_lib.cu:28,37; produced by onebit_sparse_mul/__init__.py:139-143), 1 = +1, 0 = -1
//        e : int16 metadata (m x k/16) in the reference's reordered layout or the CUTLASS one
//            (_semi_structured_conversions.py:21-48,173-177)
// Writes the block described in onebit_device.h. K is padded up to a multiple of 256 with +1 values on
// positions 0,1 of each group; the GEMM kernels multiply that padding by zero rows of B.
// =====================================================================================================
__global__ __launch_bounds__(64) void prepare_kernel(const uint8_t* __restrict__ a, const uint16_t* __restrict__ e,
                                                     uint8_t* __restrict__ prep, int m, int k, int kc_total,
                                                     int layout) {
  const int kc = blockIdx.x, rb = blockIdx.y, lane = threadIdx.x;
  const int i = lane & 31, ga = lane >> 5;
  const int64_t r = (int64_t)rb * kRowBlock + i;  // m % 32 == 0: every row of the block exists
  const int ncols = k / 16;
  // The value bits of the block's 32 rows for one compressed column are one aligned dword of `a` (bit position
  // 32 rb + j m, m % 32 == 0). The block spans 128 compressed columns: two dwords per lane, shared through LDS.
  __shared__ __attribute__((aligned(16))) uint32_t column_bits[128];
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int local = lane + 64 * half;
    const int64_t j = (int64_t)kc * 128 + local;     // compressed column
    uint32_t word = 0xFFFFFFFFu;                      // padding past K: +1
    if (j < k / 2) {
      const uint8_t* src = a + (((int64_t)rb * kRowBlock + j * m) >> 3);
      if ((reinterpret_cast<uintptr_t>(a) & 3) == 0)
        word = *reinterpret_cast<const uint32_t*>(src);
      else
        word = (uint32_t)src[0] | ((uint32_t)src[1] << 8) | ((uint32_t)src[2] << 16) | ((uint32_t)src[3] << 24);
    }
    column_bits[local] = ~word;  // stored inverted: a set bit now means -1, which is what the sign words hold
  }
  __syncthreads();
  uint32_t meta[4] = {0, 0, 0, 0};
  uint32_t sign[2] = {0, 0};
  // metadata column of step s: c = 16 kc + 2 s + ga. In all three layouts the element of column c + 2 lies a fixed
  // distance after that of column c (one column pair = 2 m elements in the reordered layouts), so one offset is
  // computed and then advanced.
  const int c0 = kc * 16 + ga;
  int64_t off = layout == 0 ? meta_offset_reference(r, c0, m) : layout == 1 ? meta_offset_cutlass(r, c0, m) : r * ncols + c0;
  const int64_t off_step = layout == 2 ? 2 : 2 * (int64_t)m;
#pragma unroll
  for (int s = 0; s < kStepsPerChunk; ++s) {
    const int c = c0 + 2 * s;
    uint32_t mv = 0x4444u;
    if (c < ncols) mv = e[off];
    off += off_step;
    meta[s >> 1] |= mv << (16 * (s & 1));
    // kept value t of this step = compressed column 8 c + t = entry 8 (2 s + ga) + t of the block's 128; it goes to
    // bit 15 - j (t even) or 31 - j (t odd) of the step group's sign word, j = 4 (s % 4) + t / 2: one bit-field
    // extract and one shift-or per value
    const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(&column_bits[8 * (2 * s + ga)]);
    const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(&column_bits[8 * (2 * s + ga) + 4]);
    const uint32_t w8[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const int j = 4 * (s & 3) + (t >> 1);
      const int position = ((t & 1) ? 31 : 15) - j;
      sign[s >> 2] |= ((w8[t] >> i) & 1u) << position;
    }
  }
  uint8_t* block = prep + ((size_t)rb * kc_total + kc) * kBlockBytes;
  u32x4_t mvec = {meta[0], meta[1], meta[2], meta[3]};
  u32x2_t svec = {sign[0], sign[1]};
  *reinterpret_cast<u32x4_t*>(block + lane * 16) = mvec;
  *reinterpret_cast<u32x2_t*>(block + kSignOffset + lane * 8) = svec;
}

// =====================================================================================================
// pack_kernel: dense fp16 weight (m x k, row-major) -> the reference's stored operands (a bits, e metadata).
// Fuses the steps of BinaryLinear_2_4.pack (onebit_sparse_mul/__init__.py:130-145): optional 2:4 magnitude
// pruning (mask_creator, _semi_structured_conversions.py:286-314; among equal magnitudes the lower index is
// pruned first), compression to kept values + nibbles (:126-159, including the fixed encodings of groups
// with fewer or more than two non-zeros), sign quantisation (value > 0 -> 1, __init__.py:22-23), transposed
// bit packing (__init__.py:25-34,142-143) and the metadata reorder (:21-48).
// One wavefront = 64 consecutive rows x four metadata columns (64 dense K, one 128-byte line per row); the eight
// sign bits of a row and column are gathered across the wavefront with ballots, so every store of `a` is 8 bytes
// of 64 consecutive rows.
// =====================================================================================================
__device__ __constant__ uint8_t kNibbleOfPattern[16] = {0xE, 0x8, 0x9, 0x4, 0xE, 0x8, 0x9, 0x4,
                                                        0xE, 0xC, 0xD, 0x4, 0xE, 0xC, 0xD, 0x4};

__global__ __launch_bounds__(64) void pack_kernel(const _Float16* __restrict__ w, uint8_t* __restrict__ a,
                                                  uint16_t* __restrict__ e, int m, int k, int prune, int layout) {
  const int64_t r = (int64_t)blockIdx.y * 64 + threadIdx.x;  // m % 64 == 0: always a valid row
  const int ncols = k / 16;
  // four metadata columns (64 weights = 128 consecutive bytes of the lane's row) per wavefront: requests of whole
  // 128-byte lines; the last group of a row may hold two columns only (k % 32 == 0)
  const int c_first = blockIdx.x * 4;
  const int c_count = ncols - c_first < 4 ? ncols - c_first : 4;
  u32x4_t line[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
    if (i < 2 * c_count) line[i] = reinterpret_cast<const u32x4_t*>(w + r * k + 16 * c_first)[i];
#pragma unroll
  for (int ci = 0; ci < 4; ++ci) {
    if (ci >= c_count) break;  // wave-uniform
    const int c = c_first + ci;                       // metadata column
    u32x4_t raw[2] = {line[2 * ci], line[2 * ci + 1]};
    _Float16 v[16];
    __builtin_memcpy(v, raw, 32);
    uint32_t word = 0, bits = 0;  // bits: bit t = kept value t of this metadata element is > 0
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      float x[4], mag[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        x[i] = (float)v[4 * g + i];
        mag[i] = x[i] < 0.f ? -x[i] : x[i];
      }
      int pattern = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        bool keep = true;
        if (prune) {
          int beaten = 0;  // elements that outrank i: larger magnitude, or equal magnitude and higher index
#pragma unroll
          for (int j = 0; j < 4; ++j) beaten += (j != i) && (mag[j] > mag[i] || (mag[j] == mag[i] && j > i));
          keep = beaten < 2;
        }
        if (!keep) x[i] = 0.f;
        pattern |= (x[i] != 0.f) << i;
      }
      const int nib = kNibbleOfPattern[pattern];
      const int i0 = nib & 3, i1 = nib >> 2;
      word |= (uint32_t)nib << (4 * g);
      float k0 = x[0], k1 = x[0];
#pragma unroll
      for (int i = 1; i < 4; ++i) {
        if (i0 == i) k0 = x[i];
        if (i1 == i) k1 = x[i];
      }
      bits |= (uint32_t)(k0 > 0.f) << (2 * g);
      bits |= (uint32_t)(k1 > 0.f) << (2 * g + 1);
    }
    int64_t off;
    if (layout == 0) off = meta_offset_reference(r, c, m);
    else if (layout == 1) off = meta_offset_cutlass(r, c, m);
    else off = r * ncols + c;
    e[off] = (uint16_t)word;
    const int64_t row0 = (int64_t)blockIdx.y * 64;
#pragma unroll
    for (int t = 0; t < 8; ++t) {
      const uint64_t mask = __ballot((bits >> t) & 1u);  // bit l = row row0 + l, compressed column 8c + t
      if (threadIdx.x == 0) {
        const int64_t pos = row0 + (int64_t)(8 * c + t) * m;  // multiple of 64
        *reinterpret_cast<uint64_t*>(a + (pos >> 3)) = mask;
      }
    }
  }
}

// =====================================================================================================
// Main kernel.
// Workgroup = 4 or 8 wavefronts arranged WM x WN; each wavefront owns FM x FN accumulator tiles of 32 x 32.
// B is staged through LDS in stages of 64 K rows; the LDS image of a stage is row-major (N contiguous)
// with the 16-byte column chunks of row r XOR-swizzled so that the four rows a 16-lane group touches in
// one transpose read fall into different bank groups.
// =====================================================================================================
constexpr int kStageK = 64;
constexpr int kStages = 4;  // LDS ring; one prepared-operand chunk (256 K) = one trip around the ring

template <int BN>
__device__ __forceinline__ int chunk_swizzle(int row) {
  // 16-byte chunk index XOR; rows r..r+3 must land in four different 64-byte bank groups. Bit 3 of the row swaps the
  // 32-byte halves of a group: the 16x16x64 form's lanes 0-15 and 16-31 read 32 bytes each of rows r..r+3 and
  // r+8..r+11 in one pass (the 32x32x32 form reads whole 64-byte groups and does not notice).
  return (BN >= 128) ? (((row & 3) << 2) | (((row >> 3) & 1) << 1)) : (((row >> 1) & 1) << 2);
}

// KG = 2: two groups of WM x WN wavefronts cover the same tile; group g multiplies K step g of every 64-row stage,
// and the two partial tiles are added through LDS at the end (twice the wavefronts per SIMD for the same tile).
template <int WM, int WN, int FM, int FN, int KG = 1>
struct TileShape {
  static constexpr int BM = WM * FM * 32;
  static constexpr int BN = WN * FN * 32;
  static constexpr int CH = BN / 8;                       // 16-byte chunks per LDS row
  static constexpr int NW = WM * WN * KG;                 // wavefronts per workgroup
  static constexpr int NL = kStageK * CH / (64 * NW);     // chunk copies per thread per stage
  static constexpr int STAGE_BYTES = kStageK * BN * 2;
  static constexpr int LDS_B_BYTES = kStages * STAGE_BYTES;
  static constexpr int NA = ((BM / 32) * 1536 + 1024 * NW - 1) / (1024 * NW);  // 1 KiB A copies per wavefront per chunk
  static constexpr int LDS_BYTES = LDS_B_BYTES + NA * 1024 * NW;
  static_assert(NW == 4 || NW == 8, "four or eight wavefronts per workgroup");
  static_assert(kStageK * CH % (64 * NW) == 0, "the stage must divide into whole wavefront copies");
  static_assert(NL >= 1, "tile too narrow for the copy pattern");
  static_assert(KG == 1 || (KG == 2 && WM * FM <= 4), "the second group's partial tile must fit the stage ring");
};

// XCD-aware tile order. Workgroup b runs on XCD b % xcds (xcds = 8 on a whole MI355X; the launcher derives it from the
// device's compute-unit count, so a partitioned GPU keeps the property), so XCD x is given a contiguous range of a tile list
// that is ordered in blocks of GROUP_M row tiles x 4 column tiles (row tile fastest), blocks running down M inside
// a strip of 4 column tiles, strips running along N. GROUP_M x 4 = the workgroups resident on one XCD (64 for the
// four-wavefront tiles with two workgroups per CU; 32 for the tiles with one per CU), which then form one block: every B column
// panel it streams is shared by GROUP_M workgroups and every A row panel by 4 in that XCD's L2, and the whole
// range of one XCD covers few column strips, so B is fetched into few L2s.
template <int GROUP_M>
__device__ __forceinline__ void tile_of_block(int b, int tiles_m, int tiles_n, int xcds, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  int per, rem, x, local;
  if (xcds == 8) {  // the usual case with constant divisors
    per = total / 8, rem = total % 8, x = b % 8, local = b / 8;
  } else {
    per = total / xcds, rem = total % xcds, x = b % xcds, local = b / xcds;
  }
  const int v = x * per + (x < rem ? x : rem) + local;
  constexpr int STRIP_N = 4;
  const int strip = v / (tiles_m * STRIP_N);
  const int strip_w = (tiles_n - strip * STRIP_N) < STRIP_N ? (tiles_n - strip * STRIP_N) : STRIP_N;
  const int w = v - strip * STRIP_N * tiles_m;
  const int group = w / (GROUP_M * strip_w);
  const int group_h = (tiles_m - group * GROUP_M) < GROUP_M ? (tiles_m - group * GROUP_M) : GROUP_M;
  const int u = w - group * GROUP_M * strip_w;
  tm = group * GROUP_M + u % group_h;
  tn = strip * STRIP_N + u / group_h;
}

// One stage (64 K = two SMFMAC K steps) of a wavefront's FM x FN tile.
template <int FM, int FN, int BN, int STAGE_IN_CHUNK>
__device__ __forceinline__ void compute_stage(const char* stage_lds, const AChunk (&a)[FM], float16_t (&acc)[FM][FN],
                                              const int (&frag_off)[FN], int lane_row_off, uint32_t one) {
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    half16_t bv[FN];
#pragma unroll
    for (int fn = 0; fn < FN; ++fn) {
      u32x8_t raw;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row_const = ks * 32 + 4 * (q & 1) + 16 * (q >> 1);
        const u32x2_t t = lds_read_tr16(stage_lds + lane_row_off + row_const * (BN * 2) + frag_off[fn]);
        raw[2 * q] = t.x;
        raw[2 * q + 1] = t.y;
      }
      bv[fn] = __builtin_bit_cast(half16_t, raw);
    }
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) {
      half8_t av;
      if (ks == 0) av = expand_signs<2 * STAGE_IN_CHUNK>(a[fm], one);
      else av = expand_signs<2 * STAGE_IN_CHUNK + 1>(a[fm], one);
#pragma unroll
      for (int fn = 0; fn < FN; ++fn) {
        if (ks == 0) acc[fm][fn] = smfmac_step<2 * STAGE_IN_CHUNK, false>(a[fm], av, bv[fn], acc[fm][fn]);
        else acc[fm][fn] = smfmac_step<2 * STAGE_IN_CHUNK + 1, false>(a[fm], av, bv[fn], acc[fm][fn]);
      }
    }
  }
}

// ---- building blocks of the asynchronous-copy main loop ----------------------------------------------
// Token-major stage image (linear-layer form): row t = the stage's 64 K values of token t (128 bytes, eight 16-byte
// pieces, piece p stored at position p ^ token_swizzle(t)). The operand of K step ks is pieces 4 ks + gb and 4 ks + 2 + gb of
// the lane's token: two plain 16-byte reads at the precomputed lane offsets piece_off[2 ks + h].
// Position XOR of the 16-byte pieces of token row t in the token-major images: sixteen consecutive tokens that read the
// same piece touch sixteen different 16-byte columns of the 256 bytes the LDS banks span (rows of 128 bytes: two rows
// fill the span, so the XOR changes every second token; rows of 256 bytes or more: every token).
template <int ROW_BYTES = 128>
__device__ __forceinline__ constexpr int token_swizzle(int token) {
  return ROW_BYTES >= 256 ? (token & 15) : ((token >> 1) & 7);
}

// One packed register (kept values 2p, 2p+1 of K step STEP) of expand_signs. The empty volatile statement keeps the two
// instructions where they are written: the optimizer otherwise sinks them past the stage's barrier to the block of their
// first use.
template <int STEP>
__device__ __forceinline__ uint32_t expand_sign_register(const AChunk& a, uint32_t packed_one, int p) {
  const uint32_t w = STEP < 4 ? a.sign.x : a.sign.y;
  uint32_t v = ((w << (4 * (STEP % 4) + p)) & 0x80008000u) | packed_one;
  asm volatile("" : "+v"(v));
  return v;
}

// One piece of the B fragments of a K step: piece r of the row-major image is transpose read q = r % 4 of fragment
// r / 4, piece r of the token-major image is 16-byte read h = r % 2 of fragment r / 2.
template <int BN>
__device__ __forceinline__ void load_b_piece(const char* stage_lds, int ks, int r, u32x8_t* bv, const int* frag_off,
                                             int lane_row_off) {
  const int fn = r >> 2, q = r & 3;
  const int row_const = ks * 32 + 4 * (q & 1) + 16 * (q >> 1);
  const u32x2_t t = lds_read_tr16(stage_lds + lane_row_off + row_const * (BN * 2) + frag_off[fn]);
  bv[fn][2 * q] = t.x;
  bv[fn][2 * q + 1] = t.y;
}

__device__ __forceinline__ void load_b_piece_tokens(const char* wave_lds, int ks, int r, u32x8_t* bv,
                                                    const int* piece_off) {
  const int fn = r >> 1, h = r & 1;
  const u32x4_t t = *reinterpret_cast<const u32x4_t*>(wave_lds + piece_off[2 * ks + h] + fn * (32 * kStageK * 2));
  bv[fn][4 * h] = t.x; bv[fn][4 * h + 1] = t.y; bv[fn][4 * h + 2] = t.z; bv[fn][4 * h + 3] = t.w;
}

// The SMFMACs of one K step with the fetch work for the next step placed between them by hand: fetch(slot) runs right
// behind SMFMAC number `slot`, and scheduling fences keep it there (the compiler would otherwise keep the
// inline-assembly SMFMACs of the one-wavefront-per-SIMD tiles in one block, and order the rest as it likes).
template <int STEP, bool PINNED, int FM, int FN, class Fetch>
__device__ __forceinline__ void mfma_frags_fused(const AChunk (&a)[FM], const u32x4_t (&av)[FM], const u32x8_t (&bv)[FN],
                                                 float16_t (&acc)[FM][FN], Fetch&& fetch) {
#pragma unroll
  for (int fm = 0; fm < FM; ++fm)
#pragma unroll
    for (int fn = 0; fn < FN; ++fn) {
      __builtin_amdgcn_s_setprio(1);  // the wavefront that is about to issue an SMFMAC wins the arbitration on its SIMD
      acc[fm][fn] = smfmac_step<STEP, PINNED>(a[fm], __builtin_bit_cast(half8_t, av[fm]),
                                              __builtin_bit_cast(half16_t, bv[fn]), acc[fm][fn]);
      __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
      fetch(fm * FN + fn);
      __builtin_amdgcn_sched_barrier(0);
    }
}

// Source of zeros for the asynchronous copies of B rows at or past K.
__device__ __attribute__((aligned(16))) uint32_t g_zero16[4] = {0, 0, 0, 0};

// TOKENS (with DMA only): the linear-layer form. p.b is x (p.n tokens x p.k, token-major), p.d is y (p.n tokens x
// p.m), the epilogue is y = acc + bias; a tile column is a token.
template <int WM, int WN, int FM, int FN, bool DMA, bool TOKENS = false, int KG = 1, bool M16 = false>
__global__ __launch_bounds__(64 * WM * WN * KG, (FM * FN <= 8 ? 2 : 1)) void gemm_kernel(GemmArgs p) {
  static_assert(!M16 || (DMA && KG == 1 && WN == 1 && FM == 4 && FN == 4), "the 16x16x64 form exists for the 512x128 four-wavefront tile");
  static_assert(DMA || !TOKENS, "the token-major form uses the asynchronous copies");
  static_assert(DMA || KG == 1, "the two-group form uses the asynchronous copies");
  using TS = TileShape<WM, WN, FM, FN, KG>;
  constexpr int BM = TS::BM, BN = TS::BN, CH = TS::CH, NL = TS::NL, NW = TS::NW;
  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in a scalar register
  const int kg = KG == 2 ? wave / (WM * WN) : 0;   // K group of this wavefront
  const int wave_in_group = KG == 2 ? wave % (WM * WN) : wave;
  const int wm = wave_in_group / WN, wn = wave_in_group % WN;
  int tile_m, tile_n;
  // one workgroup per compute unit (eight wavefronts, or four that use all the registers): 32 resident on an XCD
  tile_of_block<(NW == 8 || FM * FN > 8 ? 8 : 16)>(blockIdx.x, p.tiles_m, p.tiles_n, p.xcds, tile_m, tile_n);
  const int row0 = tile_m * BM + wm * FM * 32;  // first row of this wavefront
  const int n0 = tile_n * BN;                   // first column of the workgroup
  const int col0 = n0 + wn * FN * 32;           // first column of this wavefront

  // ---- A operand addressing (prepared blocks) ----
  const int rb_total = p.m / kRowBlock;
  const uint8_t* a_block[FM];
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) {
    int rb = row0 / kRowBlock + fm;
    if (rb >= rb_total) rb = rb_total - 1;  // rows past M: compute on valid data, never stored
    a_block[fm] = p.prep + (size_t)rb * p.kc_total * kBlockBytes;
  }

  // ---- B fragment addressing inside a stage ----
  const int i16 = lane & 15;
  const int gb = lane >> 5;
  const int c8 = ((lane & 31) >> 4) * 4 + (i16 & 3);  // 8-byte chunk inside the 32-column fragment
  const int lane_row = 8 * gb + (i16 >> 2);           // + compile-time row constants
  const int lane_row_off = lane_row * (BN * 2);
  int frag_off[FN];
#pragma unroll
  for (int fn = 0; fn < FN; ++fn) {
    const int lc = 4 * (wn * FN + fn) + (c8 >> 1);
    frag_off[fn] = ((lc ^ chunk_swizzle<BN>(lane_row)) << 4) + (c8 & 1) * 8;
  }

  int piece_off[4];  // token-major image: byte offsets of the lane's four pieces of a stage (see load_b_frags_tokens)
  {
    const int token = lane & 31;
    const int base = token * (kStageK * 2) + ((gb ^ token_swizzle(token)) << 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) piece_off[j] = base ^ ((4 * (j >> 1) + 2 * (j & 1)) << 4);
  }
  const char* const wave_image = smem + wn * FN * (32 * kStageK * 2);  // first token row of this wavefront in stage 0

  const uint32_t one = packed_one_in_vgpr();
  // 32x32x32 form: FM x FN tiles of 32 x 32; 16x16x64 form: 2 FM x 2 FN tiles of 16 x 16 (the other array has one element)
  float16_t acc[M16 ? 1 : FM][M16 ? 1 : FN];
  float4v_t acc16[M16 ? 2 * FM : 1][M16 ? 2 * FN : 1];
#pragma unroll
  for (int fm = 0; fm < (M16 ? 1 : FM); ++fm)
#pragma unroll
    for (int fn = 0; fn < (M16 ? 1 : FN); ++fn)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[fm][fn][v] = 0.f;
#pragma unroll
  for (int rt = 0; rt < (M16 ? 2 * FM : 1); ++rt)
#pragma unroll
    for (int ct = 0; ct < (M16 ? 2 * FN : 1); ++ct) acc16[rt][ct] = float4v_t{0.f, 0.f, 0.f, 0.f};

  const int stages_total = (p.k + kStageK - 1) / kStageK;
  const int chunks = (stages_total + kStages - 1) / kStages;
  // K split over workgroups: this one multiplies chunks [chunk_begin, chunk_end) and writes to its own slice of d
  const int chunk_begin = blockIdx.y * p.chunks_per_split;  // the launcher makes every split non-empty
  const int chunk_end = chunk_begin + p.chunks_per_split < chunks ? chunk_begin + p.chunks_per_split : chunks;
  char* const d_out = reinterpret_cast<char*>(p.d) + (size_t)blockIdx.y * p.m * p.n * (p.d_f16 ? 2 : 4);
  // Two K groups: with an even number of row fragments each group finishes half of them (it hands the other half of
  // its sums to the other group); otherwise the second group hands everything to the first and stores nothing.
  constexpr bool kSplitEpilogue = KG == 2 && FM % 2 == 0;
  const int row_limit = (kg == 0 || kSplitEpilogue) ? p.m : 0;
  auto finishes = [&](int fm) __attribute__((always_inline)) { return !kSplitEpilogue || (fm >= FM / 2) == (kg == 1); };

  if constexpr (DMA) {
    // ---- asynchronous copy pattern for B: NL 16-byte copies per thread per stage ----
    // copy i of wavefront w fills LDS slots [(NW i + w) * 64, +64) of the stage; slot = (row, physical chunk).
    // Global address = wave-uniform base of the stage + per-lane byte offset.
    uint32_t b_off[NL];
    int copy_row[NL];  // first K row of the stage that copy i carries
    uint32_t lds_dst[NL];
    const uint32_t smem_base = lds_offset_of(smem);
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int slot = (NW * i + wave) * 64 + lane;
      if constexpr (TOKENS) {
        // slot = (token of the tile, physical piece): fetches K values [8 lc, 8 lc + 8) of the stage for that token
        int token = slot / 8;
        const int lc = (slot % 8) ^ token_swizzle(token);
        if (n0 + token >= p.n) token = 0;  // tokens past the end: any valid address will do, the results are not stored
        b_off[i] = (uint32_t)(token * p.k + 8 * lc) * 2u;  // the launcher checks that BN * k * 2 fits 32 bits
        copy_row[i] = 8 * lc;
      } else {
        const int row = slot / CH, pc = slot % CH;
        const int lc = pc ^ chunk_swizzle<BN>(row);
        int col = 8 * lc;
        if (n0 + col >= p.ldb) col = 0;  // columns past the row: any valid address will do, the results are not stored
        b_off[i] = (uint32_t)(row * p.ldb + col) * 2u;
        copy_row[i] = row;
      }
      lds_dst[i] = smem_base + (NW * i + wave) * 1024;
    }
    const size_t stage_stride = TOKENS ? (size_t)kStageK * 2 : (size_t)kStageK * p.ldb * 2;
    const char* b_stage = reinterpret_cast<const char*>(p.b) + (TOKENS ? (size_t)n0 * p.k * 2 : (size_t)n0 * 2) +
                          (size_t)chunk_begin * kStages * stage_stride;  // advances one stage per copy
    const char* zeros = reinterpret_cast<const char*>(g_zero16);
    int next_k0 = chunk_begin * kChunkK;  // first K row of the next stage to copy
    // Rows at or past K are copied from a block of zeros, so stages past the end of K (the ring always runs
    // whole chunks of four stages) and the padding of the prepared operand contribute nothing, and the
    // number of copies in flight, which the vmcnt waits rely on, is the same in every iteration.
    auto issue_b = [&](int ring) {
      if (next_k0 + kStageK <= p.k) {  // wave-uniform: a full stage
#pragma unroll
        for (int i = 0; i < NL; ++i) lds_dma16_base(b_stage, b_off[i], lds_dst[i] + ring * TS::STAGE_BYTES);
      } else {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
          const char* src = (next_k0 + copy_row[i] < p.k) ? b_stage + b_off[i] : zeros;
          lds_dma16(src, lds_dst[i] + ring * TS::STAGE_BYTES);
        }
      }
      b_stage += stage_stride;
      next_k0 += kStageK;
    };
    // the same for a stage that the caller knows to lie inside K: no branch, so that the K loop's body stays one block
    auto issue_b_full = [&](int ring) {
#pragma unroll
      for (int i = 0; i < NL; ++i) lds_dma16_base(b_stage, b_off[i], lds_dst[i] + ring * TS::STAGE_BYTES);
      b_stage += stage_stride;
      next_k0 += kStageK;
    };

    // ---- asynchronous copy pattern for A: the workgroup's BM/32 prepared blocks of one K chunk ----
    // LDS image = the blocks back to back; NA copies of 1 KiB per wavefront (the tail past the last block
    // re-copies the first block into padding so that every wavefront issues the same number of requests).
    constexpr int NA = TS::NA;
    char* a_lds = smem + TS::LDS_B_BYTES;
    uint32_t a_off[NA];
    uint32_t a_dst[NA];
    {
      const int rb0 = tile_m * (BM / kRowBlock);
#pragma unroll
      for (int j = 0; j < NA; ++j) {
        const int byte = (NW * j + wave) * 1024 + lane * 16;
        int blk = byte / kBlockBytes, off = byte % kBlockBytes;
        if (blk >= BM / kRowBlock) blk = 0;
        int rb = rb0 + blk;
        if (rb >= rb_total) rb = rb_total - 1;
        a_off[j] = (uint32_t)((size_t)rb * p.kc_total * kBlockBytes + off);  // the launcher checks it fits 32 bits
        a_dst[j] = smem_base + TS::LDS_B_BYTES + (NW * j + wave) * 1024;
      }
    }
    const char* a_chunk = reinterpret_cast<const char*>(p.prep) + (size_t)chunk_begin * kBlockBytes;  // advances one K chunk per copy
    int next_chunk = chunk_begin;
    auto advance_a = [&]() {
      if (next_chunk + 1 < chunks) a_chunk += kBlockBytes;  // past the last chunk the last one is copied again
      ++next_chunk;
    };
    auto issue_a = [&]() {
#pragma unroll
      for (int j = 0; j < NA; ++j) lds_dma16_base(a_chunk, a_off[j], a_dst[j]);
      advance_a();
    };
    const char* a_frag_lds[FM];
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) a_frag_lds[fm] = a_lds + (wm * FM + fm) * kBlockBytes;

    // ---- the K loop ------------------------------------------------------------------------------------
    // Software pipeline over a ring of four 64-row stages of B (and one K chunk of A) in LDS. The SMFMACs of one K step
    // run while the B fragments and the expanded signs of the next step this wavefront multiplies are fetched; one
    // workgroup barrier per stage publishes the next stage and frees the ring slot of the one whose reads have all been
    // issued, into which the stage four ahead is then copied.
    // Request order: A(0) B(0) B(1) B(2) B(3) | chunk c: stage 0: A(c+1) B(4c+4)  stage 1: B(4c+5)
    //                                                     stage 2: B(4c+6)        stage 3: B(4c+7)
    // The order of the instructions inside each K-step region is written out and fenced: behind SMFMAC number `slot` of
    // the step comes that slot's share of the fetch work (fragment reads in the first half of the slots, the two
    // instructions per sign register spread evenly, the copies one by one), so that the two wavefronts of a SIMD, which
    // leave every barrier in lock-step, alternate on the matrix pipe instead of both fetching first; left to itself the
    // optimizer sinks the sign expansion past the barrier to the block of its first use.
    constexpr bool PINNED = FM * FN > 8;
    constexpr int SLOTS = FM * FN;
    constexpr int PIECES = TOKENS ? 2 * FN : 4 * FN;
    constexpr int PPS = (2 * PIECES + SLOTS - 1) / SLOTS > 1 ? (2 * PIECES + SLOTS - 1) / SLOTS : 1;  // pieces per slot
    auto read_piece = [&](int ring_slot, int ks, int r, u32x8_t* bv) __attribute__((always_inline)) {
      if constexpr (TOKENS) load_b_piece_tokens(wave_image + ring_slot * TS::STAGE_BYTES, ks, r, bv, piece_off);
      else load_b_piece<BN>(smem + ring_slot * TS::STAGE_BYTES, ks, r, bv, frag_off, lane_row_off);
    };
// the fetch work behind SMFMAC `slot`: pieces of the fragments of (RING, KS) into BV, registers of step FILL_STEP of A_SRC into AV
#define ONEBIT_FETCH_SLOT(RING, KS, BV, FILL_STEP, A_SRC, AV)                                                      \
          _Pragma("unroll") for (int r = 0; r < PIECES; ++r)                                                        \
            if (r / PPS == slot) read_piece((RING), (KS), r, BV);                                                   \
          _Pragma("unroll") for (int g = 0; g < 4 * FM; ++g)                                                        \
            if (g * FN / 4 == slot) AV[g / 4][g % 4] = expand_sign_register<(FILL_STEP)>(A_SRC[g / 4], one, g % 4);
// the copies of stage S + 4 (and of the next chunk of A) behind SMFMAC `slot`: one by one when the stage is known to lie
// inside K (A first, same request order), else all behind the first SMFMAC through the general, branching form.
// The copies are spread evenly over the region's slots: the wavefronts of a workgroup leave the barrier together, a
// compute unit's address path takes one 16-byte-per-lane copy instruction per 16 clocks, and copies issued back to back
// by every wavefront at once queue up there and hold the issuing wavefronts.
#define ONEBIT_COPY_SLOT(S, ISSUE_A)                                                                               \
          if constexpr (FULL) {                                                                                    \
            constexpr int COPIES = ((ISSUE_A) ? NA : 0) + NL, CPS = (COPIES + SLOTS - 1) / SLOTS;                  \
            constexpr int SPREAD = COPIES <= SLOTS ? SLOTS / COPIES : 1;  /* slots from one copy to the next */    \
            _Pragma("unroll") for (int c = 0; c < COPIES; ++c)                                                     \
              if ((c / CPS) * SPREAD == slot) {                                                                    \
                const int i = c - ((ISSUE_A) ? NA : 0);                                                            \
                if (i < 0) lds_dma16_base(a_chunk, a_off[c], a_dst[c]);                                            \
                else lds_dma16_base(b_stage, b_off[i], lds_dst[i] + (S) * TS::STAGE_BYTES);                        \
              }                                                                                                    \
            if (slot == ((COPIES - 1) / CPS) * SPREAD) {                                                           \
              if (ISSUE_A) advance_a();                                                                            \
              b_stage += stage_stride;                                                                             \
              next_k0 += kStageK;                                                                                  \
            }                                                                                                      \
            __builtin_amdgcn_sched_barrier(0);                                                                     \
          } else if (slot == 0) {                                                                                  \
            if (ISSUE_A) issue_a();                                                                                \
            issue_b(S);                                                                                            \
            __builtin_amdgcn_sched_barrier(0);                                                                     \
          }
    // chunk kc copies the stages of chunk kc + 1: they are whole while (kc + 2) * 256 <= K
    const int full_end = p.k / kChunkK - 1 < chunk_end ? p.k / kChunkK - 1 : chunk_end;

    if constexpr (M16) {
      // ---- 16x16x64 form of the K loop (one wavefront per SIMD, wave tile 128 x 128 = 8 x 8 tiles of 16 x 16) ----
      // One SMFMAC covers a whole 64-row stage. A-operand lane (row l % 16, group l / 16) holds the kept values of K
      // positions [16 g, 16 g + 16) of the stage, i.e. what lane row + 32 (g % 2) of the prepared block holds for K step
      // 2 S + g / 2; B-operand lane (column l % 16, group g) holds K rows 8 g ... 8 g + 7 of both 32-row halves.
      // First half of a stage (before the barrier): row tiles 0-3 against all column tiles, the signs of the next row
      // tile and of row tiles 4-7 expanded between the SMFMACs. Second half: column tile by column tile against row
      // tiles 4-7; a column tile's fragment registers are free after its four SMFMACs and take the next stage's
      // fragment, which the barrier has just published.
      constexpr int RT = 2 * FM, CT = 2 * FN;
      const int g16 = lane >> 4, c16 = lane & 15;
      const int brow = 8 * g16 + (c16 >> 2);  // + 0, 4, 32, 36
      const int brow_off = brow * (BN * 2);
      int ct_off[CT];
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
        ct_off[ct] = (((2 * (wn * CT + ct) + ((c16 & 3) >> 1)) ^ chunk_swizzle<BN>(brow)) << 4) + (c16 & 1) * 8;
      // Token-major image (linear-layer form): the operand of token 16 ct + c16 is pieces g16 and 4 + g16 of its row, two plain
      // 16-byte reads (q = 0, 1); the swizzle of a token row depends on c16 alone, so the column tile is an immediate offset.
      const int token_piece = c16 * (kStageK * 2) + ((g16 ^ token_swizzle(c16)) << 4);
      auto read_b16 = [&](int ring_slot, int ct, int q, u32x8_t* bv) __attribute__((always_inline)) {
        if constexpr (TOKENS) {
          if (q < 2) {
            const u32x4_t t = *reinterpret_cast<const u32x4_t*>(smem + ring_slot * TS::STAGE_BYTES + ct * (16 * kStageK * 2) +
                                                                 (token_piece ^ (q << 6)));
            bv[ct][4 * q] = t.x; bv[ct][4 * q + 1] = t.y; bv[ct][4 * q + 2] = t.z; bv[ct][4 * q + 3] = t.w;
          }
          return;
        }
        const int row_const = 4 * (q & 1) + 32 * (q >> 1);
        const u32x2_t t = lds_read_tr16(smem + ring_slot * TS::STAGE_BYTES + brow_off + row_const * (BN * 2) + ct_off[ct]);
        bv[ct][2 * q] = t.x;
        bv[ct][2 * q + 1] = t.y;
      };
      // per row tile: metadata of stages 0,1 and 2,3 (16 bits each, chosen by ABID), sign words of stages 0,1 and 2,3
      struct ATile { uint32_t idx01, idx23, w01, w23; };
      const uint32_t half_select = (g16 >> 1) ? 0x07060302u : 0x05040100u;
      const int sign_shift = 4 * (g16 >> 1);
      // A row tile's operands of one chunk in two steps, so that the LDS latency of the first lies under SMFMACs: the
      // holder lane's 24 bytes as they are, then the selection of this lane's 16 index bits per stage and the shift
      // of its sign words.
      struct ARaw { u32x4_t meta; u32x2_t sign; };
      auto load_a_raw = [&](int rt) __attribute__((always_inline)) {
        const char* block = a_frag_lds[rt >> 1];
        const int holder = c16 + 16 * (rt & 1) + 32 * (g16 & 1);
        ARaw r;
        r.meta = *reinterpret_cast<const u32x4_t*>(block + holder * 16);
        r.sign = *reinterpret_cast<const u32x2_t*>(block + kSignOffset + holder * 8);
        return r;
      };
      auto finish_a = [&](const ARaw& r) __attribute__((always_inline)) {
        ATile t;
        t.idx01 = __builtin_amdgcn_perm(r.meta.y, r.meta.x, half_select);
        t.idx23 = __builtin_amdgcn_perm(r.meta.w, r.meta.z, half_select);
        t.w01 = r.sign.x << sign_shift;
        t.w23 = r.sign.y << sign_shift;
        return t;
      };
      auto gather_a = [&](int rt) __attribute__((always_inline)) { return finish_a(load_a_raw(rt)); };
      // register p (kept values 2p, 2p+1) of the expanded signs of stage S
      auto expand16 = [&](const ATile& t, int S, int p_) __attribute__((always_inline)) {
        const uint32_t w = S < 2 ? t.w01 : t.w23;
        uint32_t v = ((w << (8 * (S & 1) + p_)) & 0x80008000u) | one;
        asm volatile("" : "+v"(v));
        return v;
      };
      auto mma16 = [&](float4v_t& c, const u32x4_t& av, const u32x8_t& bv, const ATile& t, int S) __attribute__((always_inline)) {
        const uint32_t idx = S < 2 ? t.idx01 : t.idx23;
        const half8_t a8 = __builtin_bit_cast(half8_t, av);
        const half16_t b16 = __builtin_bit_cast(half16_t, bv);
        // accumulators tied to accumulation registers, as in smfmac_step
        if ((S & 1) == 0) asm("v_smfmac_f32_16x16x64_f16 %0, %1, %2, %3" : "+a"(c) : "v"(a8), "v"(b16), "v"(idx));
        else asm("v_smfmac_f32_16x16x64_f16 %0, %1, %2, %3 abid:1" : "+a"(c) : "v"(a8), "v"(b16), "v"(idx));
      };

      issue_a();
#pragma unroll
      for (int s = 0; s < kStages; ++s) issue_b(s);
      ATile a_cur[RT];
      u32x8_t bv[CT];
      u32x4_t av_roll[2], av_hi[RT / 2];
      wait_vmcnt<3 * NL>();  // A(0) and B(0) have landed
      __builtin_amdgcn_s_barrier();
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) a_cur[rt] = gather_a(rt);
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int q = 0; q < 4; ++q) read_b16(0, ct, q, bv);
#pragma unroll
      for (int p_ = 0; p_ < 4; ++p_) av_roll[0][p_] = expand16(a_cur[0], 0, p_);

      auto chunk_body = [&](auto full_tag) __attribute__((always_inline)) {
        constexpr bool FULL = decltype(full_tag)::value;
        constexpr int SLOTS = RT / 2 * CT;  // SMFMACs per half stage (shadows the 32x32x32 form's count for the copy macro)
        auto stage = [&](auto s_tag, auto wait_tag, auto issue_a_tag) __attribute__((always_inline)) {
          constexpr int S = decltype(s_tag)::value;
          constexpr int WAITCNT = decltype(wait_tag)::value;
          constexpr bool ISSUE_A = decltype(issue_a_tag)::value;
          // first half: row tiles 0-3
#pragma unroll
          for (int rt = 0; rt < RT / 2; ++rt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
              mma16(acc16[rt][ct], av_roll[rt & 1], bv[ct], a_cur[rt], S);
              __builtin_amdgcn_sched_barrier(0);
              // this slot's share of the eight registers to expand: the next row tile's four, then row tile 4 + rt's four
#pragma unroll
              for (int e = ct * 8 / CT; e < (ct + 1) * 8 / CT; ++e) {
                if (e < 4) {
                  if (rt + 1 < RT / 2) av_roll[(rt + 1) & 1][e] = expand16(a_cur[rt + 1], S, e);
                } else {
                  av_hi[rt][e - 4] = expand16(a_cur[RT / 2 + rt], S, e - 4);
                }
              }
              __builtin_amdgcn_sched_barrier(0);
            }
          wait_vmcnt_lgkm0<WAITCNT>();  // copies of stage S+1 landed
          __builtin_amdgcn_s_barrier();
          // Last stage of a chunk: the next chunk of A is readable after this stage's barrier. Row tiles 0-3 are done
          // with this chunk: their holder lanes' bytes are requested right here and turned into operands behind the
          // SMFMACs of column tile 1, by when they have arrived; row tiles 4-7 are multiplied to the end of the stage:
          // requested behind column tile 5, turned into operands after the last SMFMAC.
          constexpr bool LAST = S == kStages - 1;
          ARaw a_raw[RT / 2];
          if constexpr (LAST) {
#pragma unroll
            for (int rt = 0; rt < RT / 2; ++rt) a_raw[rt] = load_a_raw(rt);
            __builtin_amdgcn_sched_barrier(0);
          }
          // second half: column tile by column tile against row tiles 4-7
#pragma unroll
          for (int ct = 0; ct < CT; ++ct)
#pragma unroll
            for (int rl = 0; rl < RT / 2; ++rl) {
              const int slot = ct * (RT / 2) + rl;
              mma16(acc16[RT / 2 + rl][ct], av_hi[rl], bv[ct], a_cur[RT / 2 + rl], S);
              __builtin_amdgcn_sched_barrier(0);
              ONEBIT_COPY_SLOT(S, ISSUE_A)
              // the fragment of column tile ct - 1 for the next stage, one read behind each of this tile's SMFMACs
              if (ct >= 1) read_b16((S + 1) % kStages, ct - 1, rl, bv);
              if constexpr (LAST) {
                if (ct == 1) a_cur[rl] = finish_a(a_raw[rl]);
                if (ct == CT - 3) a_raw[rl] = load_a_raw(RT / 2 + rl);
              }
              // signs of row tile 0 of the next stage
              if (ct == CT - 1) av_roll[0][rl] = expand16(a_cur[0], (S + 1) % kStages, rl);
              __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
          for (int q = 0; q < 4; ++q) read_b16((S + 1) % kStages, CT - 1, q, bv);
          if constexpr (LAST) {
#pragma unroll
            for (int rl = 0; rl < RT / 2; ++rl) a_cur[RT / 2 + rl] = finish_a(a_raw[rl]);
          }
        };
        using std::integral_constant;
        stage(integral_constant<int, 0>{}, integral_constant<int, 2 * NL>{}, std::true_type{});        // waits for B(4c+1)
        stage(integral_constant<int, 1>{}, integral_constant<int, 2 * NL + NA>{}, std::false_type{});  // B(4c+2)
        stage(integral_constant<int, 2>{}, integral_constant<int, 2 * NL + NA>{}, std::false_type{});  // B(4c+3)
        stage(integral_constant<int, 3>{}, integral_constant<int, 2 * NL>{}, std::false_type{});       // B(4c+4)
      };
      int kc = chunk_begin;
      for (; kc < full_end; ++kc) chunk_body(std::true_type{});
      for (; kc < chunk_end; ++kc) chunk_body(std::false_type{});
      wait_vmcnt<0>();  // drain the copies issued past the end before the LDS is released
    } else if constexpr (KG == 1) {
      // The barrier sits in the middle of each stage s: it publishes stage s+1 (read right after it) and frees the ring
      // slot of stage s (all of its reads were issued in the first half).
      issue_a();
#pragma unroll
      for (int s = 0; s < kStages; ++s) issue_b(s);

      AChunk a_cur[FM], a_next[FM];
      u32x8_t bv0[FN], bv1[FN];
      u32x4_t av0[FM], av1[FM];
      wait_vmcnt<3 * NL>();  // A(0) and B(0) have landed
      __builtin_amdgcn_s_barrier();
#pragma unroll
      for (int fm = 0; fm < FM; ++fm) a_cur[fm] = load_a_chunk_lds(a_frag_lds[fm], lane);
#pragma unroll
      for (int r = 0; r < PIECES; ++r) read_piece(0, 0, r, bv0);
#pragma unroll
      for (int g = 0; g < 4 * FM; ++g) av0[g / 4][g % 4] = expand_sign_register<0>(a_cur[g / 4], one, g % 4);

#define ONEBIT_FUSED_STAGE(S, WAITCNT, ISSUE_A)                                                                  \
      {                                                                                                            \
        mfma_frags_fused<2 * (S), PINNED>(a_cur, av0, bv0, acc, [&](int slot) __attribute__((always_inline)) {     \
          ONEBIT_FETCH_SLOT((S), 1, bv1, 2 * (S) + 1, a_cur, av1)                                                  \
        });                                                                                                        \
        wait_vmcnt_lgkm0<(WAITCNT)>(); /* copies of stage S+1 landed; this wavefront's reads of stage S returned */ \
        __builtin_amdgcn_s_barrier();                                                                              \
        if constexpr ((S) == kStages - 1) {                                                                        \
          /* the next chunk of A is readable after this stage's barrier */                                         \
          _Pragma("unroll") for (int fm = 0; fm < FM; ++fm) a_next[fm] = load_a_chunk_lds(a_frag_lds[fm], lane);   \
          __builtin_amdgcn_sched_barrier(0);                                                                       \
        }                                                                                                          \
        mfma_frags_fused<2 * (S) + 1, PINNED>(a_cur, av1, bv1, acc, [&](int slot) __attribute__((always_inline)) { \
          ONEBIT_COPY_SLOT(S, ISSUE_A)                                                                             \
          if constexpr ((S) < kStages - 1) {                                                                       \
            ONEBIT_FETCH_SLOT((S) + 1, 0, bv0, 2 * (S) + 2, a_cur, av0)                                            \
          } else {                                                                                                 \
            ONEBIT_FETCH_SLOT(0, 0, bv0, 0, a_next, av0)                                                           \
          }                                                                                                        \
        });                                                                                                        \
        if constexpr ((S) == kStages - 1) {                                                                        \
          _Pragma("unroll") for (int fm = 0; fm < FM; ++fm) a_cur[fm] = a_next[fm];                                \
        }                                                                                                          \
      }

      auto chunk_body = [&](auto full_tag) __attribute__((always_inline)) {
        constexpr bool FULL = decltype(full_tag)::value;  // the four stages copied during this chunk lie inside K
        ONEBIT_FUSED_STAGE(0, 2 * NL, true)        // waits for B(4c+1); newer requests: B(4c+2), B(4c+3)
        ONEBIT_FUSED_STAGE(1, 2 * NL + NA, false)  // waits for B(4c+2); newer: B(4c+3), A(c+1), B(4c+4)
        ONEBIT_FUSED_STAGE(2, 2 * NL + NA, false)  // waits for B(4c+3); newer: A(c+1), B(4c+4), B(4c+5)
        ONEBIT_FUSED_STAGE(3, 2 * NL, false)       // waits for B(4c+4), which is newer than A(c+1)
      };
      int kc = chunk_begin;
      for (; kc < full_end; ++kc) chunk_body(std::true_type{});
      for (; kc < chunk_end; ++kc) chunk_body(std::false_type{});
#undef ONEBIT_FUSED_STAGE
      wait_vmcnt<0>();  // drain the copies issued past the end before the LDS is released
    } else {
      // Two K groups: this wavefront multiplies K step KGV of every stage. One barrier per stage: before it the
      // wavefront waits for its fragments of stage S (read during stage S - 1) and for the copies of stage S + 1; after
      // it the ring slot of stage S is free for stage S + 4 and stage S + 1 is readable. Same request order and wait
      // counts as the one-group pipeline.
      auto run = [&](auto group_tag) __attribute__((always_inline)) {
        constexpr int KGV = decltype(group_tag)::value;
        issue_a();
#pragma unroll
        for (int s = 0; s < kStages; ++s) issue_b(s);
        AChunk a_cur[FM], a_next[FM];
        u32x8_t bv_even[FN], bv_odd[FN];
        u32x4_t av_even[FM], av_odd[FM];
        wait_vmcnt<3 * NL>();  // A(0) and B(0) have landed
        __builtin_amdgcn_s_barrier();
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) a_cur[fm] = load_a_chunk_lds(a_frag_lds[fm], lane);
#pragma unroll
        for (int r = 0; r < PIECES; ++r) read_piece(0, KGV, r, bv_even);
#pragma unroll
        for (int g = 0; g < 4 * FM; ++g) av_even[g / 4][g % 4] = expand_sign_register<KGV>(a_cur[g / 4], one, g % 4);
#define ONEBIT_GROUP_STAGE(S, WAITCNT, ISSUE_A, BV, AV, BV_NEXT, AV_NEXT)                                         \
        {                                                                                                        \
          wait_vmcnt_lgkm0<(WAITCNT)>();                                                                         \
          __builtin_amdgcn_s_barrier();                                                                          \
          if constexpr ((S) == kStages - 1) {                                                                    \
            _Pragma("unroll") for (int fm = 0; fm < FM; ++fm) a_next[fm] = load_a_chunk_lds(a_frag_lds[fm], lane); \
            __builtin_amdgcn_sched_barrier(0);                                                                   \
          }                                                                                                      \
          mfma_frags_fused<2 * (S) + KGV, false>(a_cur, AV, BV, acc, [&](int slot) __attribute__((always_inline)) { \
            ONEBIT_COPY_SLOT(S, ISSUE_A)                                                                         \
            if constexpr ((S) < kStages - 1) {                                                                   \
              ONEBIT_FETCH_SLOT((S) + 1, KGV, BV_NEXT, 2 * ((S) + 1) + KGV, a_cur, AV_NEXT)                      \
            } else {                                                                                             \
              ONEBIT_FETCH_SLOT(0, KGV, BV_NEXT, KGV, a_next, AV_NEXT)                                           \
            }                                                                                                    \
          });                                                                                                    \
          if constexpr ((S) == kStages - 1) {                                                                    \
            _Pragma("unroll") for (int fm = 0; fm < FM; ++fm) a_cur[fm] = a_next[fm];                            \
          }                                                                                                      \
        }
        auto chunk_body = [&](auto full_tag) __attribute__((always_inline)) {
          constexpr bool FULL = decltype(full_tag)::value;
          ONEBIT_GROUP_STAGE(0, 2 * NL, true, bv_even, av_even, bv_odd, av_odd)
          ONEBIT_GROUP_STAGE(1, 2 * NL + NA, false, bv_odd, av_odd, bv_even, av_even)
          ONEBIT_GROUP_STAGE(2, 2 * NL + NA, false, bv_even, av_even, bv_odd, av_odd)
          ONEBIT_GROUP_STAGE(3, 2 * NL, false, bv_odd, av_odd, bv_even, av_even)
        };
        int kc = chunk_begin;
        for (; kc < full_end; ++kc) chunk_body(std::true_type{});
        for (; kc < chunk_end; ++kc) chunk_body(std::false_type{});
#undef ONEBIT_GROUP_STAGE
        wait_vmcnt<0>();  // drain the copies issued past the end before the LDS is released
      };
      if (kg == 0) run(std::integral_constant<int, 0>{});
      else run(std::integral_constant<int, 1>{});
#undef ONEBIT_FETCH_SLOT
#undef ONEBIT_COPY_SLOT
      smfmac_drain();
      __syncthreads();  // the stage ring is free
      if constexpr (kSplitEpilogue) {
        // each group keeps half of the row fragments and passes its sums for the other half through the ring, lane for
        // lane: group 0 finishes fragments [0, FM / 2), group 1 the rest
        constexpr int HALF = FM / 2, PER_WAVE = HALF * FN * 16 * 64;
        float* const given = reinterpret_cast<float*>(smem) + (size_t)wave * PER_WAVE + lane;
        const float* const taken =
            reinterpret_cast<const float*>(smem) + (size_t)(wave_in_group + (1 - kg) * WM * WN) * PER_WAVE + lane;
#pragma unroll
        for (int fm = 0; fm < HALF; ++fm)
#pragma unroll
          for (int fn = 0; fn < FN; ++fn)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              if (kg == 0) given[((fm * FN + fn) * 16 + v) * 64] = acc[HALF + fm][fn][v];
              else given[((fm * FN + fn) * 16 + v) * 64] = acc[fm][fn][v];
            }
        __syncthreads();
#pragma unroll
        for (int fm = 0; fm < HALF; ++fm)
#pragma unroll
          for (int fn = 0; fn < FN; ++fn)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              if (kg == 0) acc[fm][fn][v] += taken[((fm * FN + fn) * 16 + v) * 64];
              else acc[HALF + fm][fn][v] += taken[((fm * FN + fn) * 16 + v) * 64];
            }
      } else {
        // the second group's partial tile goes to the first, lane for lane
        float* const handover = reinterpret_cast<float*>(smem) + (size_t)wave_in_group * (FM * FN * 16 * 64) + lane;
        if (kg == 1) {
#pragma unroll
          for (int fm = 0; fm < FM; ++fm)
#pragma unroll
            for (int fn = 0; fn < FN; ++fn)
#pragma unroll
              for (int v = 0; v < 16; ++v) handover[((fm * FN + fn) * 16 + v) * 64] = acc[fm][fn][v];
        }
        __syncthreads();
        if (kg == 0) {
#pragma unroll
          for (int fm = 0; fm < FM; ++fm)
#pragma unroll
            for (int fn = 0; fn < FN; ++fn)
#pragma unroll
              for (int v = 0; v < 16; ++v) acc[fm][fn][v] += handover[((fm * FN + fn) * 16 + v) * 64];
        }
      }
      __syncthreads();  // the epilogue's scratch overlaps the handover area
    }
  } else {
    // ---- generic path: any N, any K % 32 == 0, any alignment. One stage at a time, element copies. ----
    for (int kc = chunk_begin; kc < chunk_end; ++kc) {
      AChunk a_cur[FM];
#pragma unroll
      for (int fm = 0; fm < FM; ++fm) a_cur[fm] = load_a_chunk(a_block[fm] + (size_t)kc * kBlockBytes, lane);
      auto fill = [&](int stage) {
        const int k0 = (kc * kStages + stage) * kStageK;
        __syncthreads();
        for (int idx = tid; idx < kStageK * BN; idx += 64 * NW) {
          const int row = idx / BN, col = idx % BN;
          _Float16 v = (_Float16)0.f;
          if (k0 + row < p.k && n0 + col < p.n) v = p.b[(size_t)(k0 + row) * p.n + n0 + col];
          const int lc = (col >> 3) ^ chunk_swizzle<BN>(row);
          *reinterpret_cast<_Float16*>(smem + row * (BN * 2) + (lc << 4) + (col & 7) * 2) = v;
        }
        __syncthreads();
      };
      if (kc * kStages + 0 < stages_total) { fill(0); compute_stage<FM, FN, BN, 0>(smem, a_cur, acc, frag_off, lane_row_off, one); }
      if (kc * kStages + 1 < stages_total) { fill(1); compute_stage<FM, FN, BN, 1>(smem, a_cur, acc, frag_off, lane_row_off, one); }
      if (kc * kStages + 2 < stages_total) { fill(2); compute_stage<FM, FN, BN, 2>(smem, a_cur, acc, frag_off, lane_row_off, one); }
      if (kc * kStages + 3 < stages_total) { fill(3); compute_stage<FM, FN, BN, 3>(smem, a_cur, acc, frag_off, lane_row_off, one); }
    }
  }

  smfmac_drain();
  if constexpr (TOKENS) {
    // ---- epilogue of the linear-layer form: y[token][row] = acc + bias[row], fp16 (RNE) or fp32 ----
    const int token_lane = lane & 31;
    auto bias_of = [&](int row) __attribute__((always_inline)) {
      if (!p.bias) return 0.f;
      return p.bias_f16 ? (float)reinterpret_cast<const _Float16*>(p.bias)[row] : reinterpret_cast<const float*>(p.bias)[row];
    };
    // COUNT (4 or 8) consecutive bias values starting at a row that is a multiple of COUNT, by 16-byte loads
    auto bias_vector = [&](int row, float* out, auto count_tag) __attribute__((always_inline)) {
      constexpr int COUNT = decltype(count_tag)::value;
#pragma unroll
      for (int e = 0; e < COUNT; ++e) out[e] = 0.f;
      if (!p.bias) return;
      if (p.bias_f16) {
        if constexpr (COUNT == 8) {
          const half8_t v = *reinterpret_cast<const half8_t*>(reinterpret_cast<const _Float16*>(p.bias) + row);
#pragma unroll
          for (int e = 0; e < 8; ++e) out[e] = (float)v[e];
        } else {
          const half4_t v = *reinterpret_cast<const half4_t*>(reinterpret_cast<const _Float16*>(p.bias) + row);
#pragma unroll
          for (int e = 0; e < 4; ++e) out[e] = (float)v[e];
        }
      } else {
#pragma unroll
        for (int e = 0; e < COUNT; e += 4) {
          const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p.bias) + row + e);
          out[e] = v.x; out[e + 1] = v.y; out[e + 2] = v.z; out[e + 3] = v.w;
        }
      }
    };
    if (p.vector_epilogue) {
      // Each wavefront turns one 32-row block of its tile at a time through a private LDS scratch laid out
      // [token][32 rows] fp32: a lane's four accumulator registers of one group are four consecutive rows of its token,
      // one 16-byte slot (slot s = rows 4 s ... 4 s + 3, stored at position s ^ (token % 8) against bank conflicts);
      // then every lane handles 16 bytes of one token's row of y.
      __syncthreads();  // every wavefront is done with the stage ring, which becomes the scratch
      constexpr int WCOLS = FN * 32;
      char* scratch = smem + wave * (WCOLS * 128);
      if constexpr (!M16) if (p.d_f16) {
        // (measured: 1-5 % off the launch for the 32x32x32 tiles, e.g. 4096 x 4096 with 2048 tokens 37.5 -> 36.7 us; the
        // 16x16x64 tile, whose single wavefront per SIMD has nothing to hide the conversions behind, is 0.5 % slower
        // with it and keeps the fp32 form)
        // fp16 result: the bias is added and the sum rounded in the accumulator layout, where a lane's four registers of
        // one group are four consecutive rows of its token, i.e. 8 bytes of y. The scratch line of a token then holds its
        // 32 rows as halves (64 bytes, four 16-byte pieces; piece j of token t stored at position j ^ ((t / 4) % 4), so
        // that the sixteen lanes that write one slot of sixteen consecutive tokens meet in no bank): half the LDS
        // traffic of the fp32 form below, same bits (one rounding of sum + bias).
        typedef float float2v __attribute__((ext_vector_type(2)));
        typedef _Float16 half2v __attribute__((ext_vector_type(2)));
        auto packed_rows = [&](const float* x, const float* b4) __attribute__((always_inline)) {
          const float2v lo = {x[0] + b4[0], x[1] + b4[1]}, hi = {x[2] + b4[2], x[3] + b4[3]};
          return u32x2_t{__builtin_bit_cast(uint32_t, __builtin_convertvector(lo, half2v)),
                         __builtin_bit_cast(uint32_t, __builtin_convertvector(hi, half2v))};
        };
        // bias of the four rows starting at `row` (a multiple of 4); rows at or past the end are never stored
        auto bias_rows = [&](int row, float* b4) __attribute__((always_inline)) {
          if (row < row_limit) bias_vector(row, b4, std::integral_constant<int, 4>{});
          else b4[0] = b4[1] = b4[2] = b4[3] = 0.f;
        };
        auto slot_at = [&](int t, int slot) __attribute__((always_inline)) {  // byte offset of 8-byte slot `slot` of token t
          return t * 64 + ((((slot >> 1) ^ ((t >> 2) & 3)) << 4) | ((slot & 1) << 3));
        };
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
          if (!finishes(fm)) continue;  // the other K group stores this fragment
          const int row_base = row0 + fm * 32;
          {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              float b4[4];
              bias_rows(row_base + 8 * q + 4 * gb, b4);
#pragma unroll
              for (int fn = 0; fn < FN; ++fn) {
                const float x[4] = {acc[fm][fn][4 * q], acc[fm][fn][4 * q + 1], acc[fm][fn][4 * q + 2], acc[fm][fn][4 * q + 3]};
                *reinterpret_cast<u32x2_t*>(scratch + slot_at(fn * 32 + token_lane, 2 * q + gb)) = packed_rows(x, b4);
              }
            }
          }
#pragma unroll
          for (int it = 0; it < WCOLS * 4 / 64; ++it) {
            const int piece = it * 64 + lane;
            const int t = piece / 4, j = piece % 4;
            const int token = col0 + t, row = row_base + 8 * j;
            const u32x4_t v = *reinterpret_cast<const u32x4_t*>(scratch + slot_at(t, 2 * j));
            if (token < p.n && row < row_limit)
              *reinterpret_cast<u32x4_t*>(reinterpret_cast<_Float16*>(d_out) + (size_t)token * p.m + row) = v;
          }
        }
        return;
      }
#pragma unroll
      for (int fm = 0; fm < FM; ++fm) {
        if (!finishes(fm)) continue;  // the other K group stores this fragment
        if constexpr (M16) {
          // 16x16x64 form: the four registers of tile (2 fm + rh, ct) are rows 16 rh + 4 (lane / 16) ... + 3 of token
          // 16 ct + lane % 16: slot 4 rh + lane / 16 of that token's line
          const int g16 = lane >> 4, c16 = lane & 15;
#pragma unroll
          for (int rh = 0; rh < 2; ++rh)
#pragma unroll
            for (int ct = 0; ct < 2 * FN; ++ct) {
              const float4v_t v4 = acc16[2 * fm + rh][ct];
              *reinterpret_cast<float4*>(scratch + (ct * 16 + c16) * 128 + (((4 * rh + g16) ^ token_swizzle(c16)) << 4)) =
                  float4{v4[0], v4[1], v4[2], v4[3]};
            }
        } else {
#pragma unroll
        for (int fn = 0; fn < FN; ++fn)
#pragma unroll
          for (int q = 0; q < 4; ++q)
            *reinterpret_cast<float4*>(scratch + (fn * 32 + token_lane) * 128 + (((2 * q + gb) ^ token_swizzle(token_lane)) << 4)) =
                float4{acc[fm][fn][4 * q], acc[fm][fn][4 * q + 1], acc[fm][fn][4 * q + 2], acc[fm][fn][4 * q + 3]};
        }
        const int row_base = row0 + fm * 32;
        if (p.d_f16) {
#pragma unroll
          for (int it = 0; it < WCOLS * 4 / 64; ++it) {
            const int piece = it * 64 + lane;
            const int t = piece / 4, j = piece % 4;
            const int token = col0 + t, row = row_base + 8 * j;
            const float4 lo = *reinterpret_cast<const float4*>(scratch + t * 128 + (((2 * j) ^ token_swizzle(t)) << 4));
            const float4 hi = *reinterpret_cast<const float4*>(scratch + t * 128 + (((2 * j + 1) ^ token_swizzle(t)) << 4));
            const float x[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            if (token < p.n && row < row_limit) {
              float bias8[8];
              bias_vector(row, bias8, std::integral_constant<int, 8>{});
              half8_t out;
#pragma unroll
              for (int e = 0; e < 8; ++e) out[e] = (_Float16)(x[e] + bias8[e]);
              *reinterpret_cast<half8_t*>(reinterpret_cast<_Float16*>(d_out) + (size_t)token * p.m + row) = out;
            }
          }
        } else {
#pragma unroll
          for (int it = 0; it < WCOLS * 8 / 64; ++it) {
            const int piece = it * 64 + lane;
            const int t = piece / 8, j = piece % 8;
            const int token = col0 + t, row = row_base + 4 * j;
            const float4 v4 = *reinterpret_cast<const float4*>(scratch + t * 128 + ((j ^ token_swizzle(t)) << 4));
            if (token < p.n && row < row_limit) {
              float bias4[4];
              bias_vector(row, bias4, std::integral_constant<int, 4>{});
              *reinterpret_cast<float4*>(reinterpret_cast<float*>(d_out) + (size_t)token * p.m + row) =
                  float4{v4.x + bias4[0], v4.y + bias4[1], v4.z + bias4[2], v4.w + bias4[3]};
            }
          }
        }
      }
      return;
    }
    // y not 16-byte aligned: one element per accumulator register
    if constexpr (M16) {
#pragma unroll
      for (int rt = 0; rt < 2 * FM; ++rt)
#pragma unroll
        for (int ct = 0; ct < 2 * FN; ++ct)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int token = col0 + ct * 16 + (lane & 15), row = row0 + rt * 16 + 4 * (lane >> 4) + v;
            if (token < p.n && row < row_limit) {
              const float x = acc16[rt][ct][v] + bias_of(row);
              const size_t o = (size_t)token * p.m + row;
              if (p.d_f16) reinterpret_cast<_Float16*>(d_out)[o] = (_Float16)x;
              else reinterpret_cast<float*>(d_out)[o] = x;
            }
          }
      return;
    }
#pragma unroll
    for (int fm = 0; fm < FM; ++fm) {
      if (!finishes(fm)) continue;  // the other K group stores this fragment
#pragma unroll
      for (int fn = 0; fn < FN; ++fn) {
        const int token = col0 + fn * 32 + token_lane;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int row = row0 + fm * 32 + 8 * (v / 4) + 4 * gb + (v % 4);
          if (token < p.n && row < row_limit) {
            const float x = acc[fm][fn][v] + bias_of(row);
            const size_t o = (size_t)token * p.m + row;
            if (p.d_f16) reinterpret_cast<_Float16*>(d_out)[o] = (_Float16)x;
            else reinterpret_cast<float*>(d_out)[o] = x;
          }
        }
      }
    }
    return;
  }
  // ---- epilogue: D = alpha * acc + beta * C (csrc/kernel.h:27-31), fp16 (RNE) or fp32 output ----
  if constexpr (DMA) {
    if (p.vector_epilogue) {
      // Coalesced form: each wavefront turns one 32-row block of its tile at a time through a private LDS
      // scratch (fp32, row-major) so that every lane then handles 16 bytes of one output row: C is read and D
      // written in full 128-byte segments instead of 64-byte (fp16) pieces per accumulator register.
      __syncthreads();  // every wavefront is done with the stage ring, which becomes the scratch
      constexpr int WCOLS = FN * 32;                   // columns of the wavefront's tile
      float* scratch = reinterpret_cast<float*>(smem) + wave * (32 * WCOLS);
      const int col_lane = lane & 31, row_lane = 4 * (lane >> 5);
      // Column swizzle of the scratch against bank conflicts, the same for rows of floats and for row pairs of packed
      // halves: line L keeps its 16-byte slots swapped in pairs when L is odd (two consecutive lines are read by one
      // group of sixteen lanes: they then touch different banks), and, with lines of 256 bytes or more, its two halves of
      // 128 bytes swapped when bit 2 (rows) or bit 1 (row pairs) of L is set (the upper half-wavefront writes the line
      // that many below the lower half's).
      constexpr int kHalfSwap = WCOLS >= 64 ? 32 : 0;
      // The accumulators of 32-row block fm into the scratch. 32x32x32 form: register v of fragment fn is row
      // 8 (v / 4) + 4 (lane / 32) + v % 4, column 32 fn + lane % 32; 16x16x64 form: register v of tile (2 fm + rh, ct) is
      // row 16 rh + 4 (lane / 16) + v, column 16 ct + lane % 16. In both, bit 2 of the row is one bit of the lane
      // (the writer's own half swap) and bit 0 of the row is bit 0 of v.
      const int g16 = lane >> 4, c16 = lane & 15;
      const int half_write = (M16 ? (g16 & 1) : (lane >> 5)) * kHalfSwap;
      auto store_rows = [&](int fm) __attribute__((always_inline)) {
        if constexpr (M16) {
#pragma unroll
          for (int rh = 0; rh < 2; ++rh)
#pragma unroll
            for (int ct = 0; ct < 2 * FN; ++ct)
#pragma unroll
              for (int v = 0; v < 4; ++v)
                scratch[(16 * rh + 4 * g16 + v) * WCOLS + ((ct * 16 + c16) ^ half_write ^ ((v & 1) << 2))] =
                    acc16[2 * fm + rh][ct][v];
        } else {
#pragma unroll
          for (int fn = 0; fn < FN; ++fn)
#pragma unroll
            for (int v = 0; v < 16; ++v)
              scratch[(8 * (v / 4) + row_lane + (v % 4)) * WCOLS + ((fn * 32 + col_lane) ^ half_write ^ ((v & 1) << 2))] =
                  acc[fm][fn][v];
        }
      };
      auto read_swizzle = [&](int line, int half_bit) __attribute__((always_inline)) {
        return ((line & 1) << 2) ^ (((line >> half_bit) & 1) * kHalfSwap);
      };
      // The pieces of C that a lane will need for one 32-row block are requested together, before the block's sums
      // travel through the scratch, so that one memory latency per block is paid instead of one per piece.
      const bool use_c = p.beta != 0.f;
      if (p.d_f16 && !use_c && WCOLS >= 8) {
        // fp16 result without C: alpha * sum is rounded in the accumulator layout, where registers v and v + 1 (v even)
        // of a lane are rows r and r + 1 of one column; the two halves go through the scratch as one word (a quarter of
        // the LDS traffic of the fp32 form). A lane then reads eight such words (columns c .. c + 7 of a row pair),
        // separates low and high halves and stores 16 bytes of row r and 16 bytes of row r + 1.
        uint32_t* const words = reinterpret_cast<uint32_t*>(scratch);  // [16 row pairs][WCOLS]
        typedef float float2v __attribute__((ext_vector_type(2)));
        typedef _Float16 half2v __attribute__((ext_vector_type(2)));
        constexpr int PER_PAIR = WCOLS / 8;            // 8-column pieces per row pair
        constexpr int TASKS = 16 * PER_PAIR;           // (row pair, piece) per 32-row block
        constexpr int ITERS = (TASKS + 63) / 64;
        // alpha == 1 is tested once per wavefront, not per value: two copies of the loop
        auto packed_turn = [&](auto scale_tag) __attribute__((always_inline)) {
        constexpr bool SCALE = decltype(scale_tag)::value;
#pragma unroll
        for (int fm = 0; fm < FM; ++fm) {
          if (!finishes(fm)) continue;  // the other K group stores this fragment
          const int row_base = row0 + fm * 32;
          auto pack = [&](float x0, float x1) __attribute__((always_inline)) {  // one packed conversion per register pair
            float2v x = {x0, x1};
            if constexpr (SCALE) x = float2v{p.alpha * x.x, p.alpha * x.y};
            return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, half2v));
          };
          if constexpr (M16) {
            // registers (0, 1) and (2, 3) of a tile: rows 16 rh + 4 (lane / 16) + 2 h and the next, row pair
            // 8 rh + 2 (lane / 16) + h
#pragma unroll
            for (int rh = 0; rh < 2; ++rh)
#pragma unroll
              for (int ct = 0; ct < 2 * FN; ++ct)
#pragma unroll
                for (int h = 0; h < 2; ++h)
                  words[(8 * rh + 2 * g16 + h) * WCOLS + ((ct * 16 + c16) ^ half_write ^ (h << 2))] =
                      pack(acc16[2 * fm + rh][ct][2 * h], acc16[2 * fm + rh][ct][2 * h + 1]);
          } else {
#pragma unroll
            for (int fn = 0; fn < FN; ++fn)
#pragma unroll
              for (int q = 0; q < 8; ++q)
                // rows 8 (q / 2) + 4 (lane / 32) + 2 (q % 2) and the next: row pair 4 (q / 2) + 2 (lane / 32) + q % 2
                words[(4 * (q / 2) + (row_lane >> 1) + (q & 1)) * WCOLS + ((fn * 32 + col_lane) ^ half_write ^ ((q & 1) << 2))] =
                    pack(acc[fm][fn][2 * q], acc[fm][fn][2 * q + 1]);
          }
#pragma unroll
          for (int it = 0; it < ITERS; ++it) {
            const int task = it * 64 + lane;
            if (TASKS % 64 != 0 && task >= TASKS) break;
            const int pair = task / PER_PAIR, c8 = (task % PER_PAIR) * 8;
            const int sw = read_swizzle(pair, 1);
            const u32x4_t lo = *reinterpret_cast<const u32x4_t*>(words + pair * WCOLS + (c8 ^ sw));
            const u32x4_t hi = *reinterpret_cast<const u32x4_t*>(words + pair * WCOLS + ((c8 + 4) ^ sw));
            const uint32_t d[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            u32x4_t even_row, odd_row;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              even_row[j] = __builtin_amdgcn_perm(d[2 * j + 1], d[2 * j], 0x05040100u);  // low halves
              odd_row[j] = __builtin_amdgcn_perm(d[2 * j + 1], d[2 * j], 0x07060302u);   // high halves
            }
            const int row = row_base + 2 * pair, col = col0 + c8;
            if (col < p.n) {
              _Float16* const out = reinterpret_cast<_Float16*>(d_out) + (size_t)row * p.n + col;
              if (row < row_limit) *reinterpret_cast<u32x4_t*>(out) = even_row;
              if (row + 1 < row_limit) *reinterpret_cast<u32x4_t*>(out + p.n) = odd_row;
            }
          }
        }
        };
        if (p.alpha != 1.f) packed_turn(std::true_type{});
        else packed_turn(std::false_type{});
        return;
      }
#pragma unroll
      for (int fm = 0; fm < FM; ++fm) {
        if (!finishes(fm)) continue;  // the other K group stores this fragment
        const int row_base = row0 + fm * 32;
        if (p.d_f16) {
          constexpr int PER_ROW = WCOLS / 8;           // 16-byte pieces (8 halves) per row
          constexpr int ITERS = 32 * PER_ROW / 64;
          uint32_t c_raw[ITERS][8];                    // fp16 C: one 16-byte load per piece (words 0-3); fp32 C: two
#pragma unroll
          for (int it = 0; it < ITERS; ++it) {
            const int piece = it * 64 + lane;
            const int row = row_base + piece / PER_ROW, col = col0 + (piece % PER_ROW) * 8;
            u32x4_t lo = u32x4_t{0, 0, 0, 0}, hi = u32x4_t{0, 0, 0, 0};
            if (use_c && row < row_limit && col < p.n) {
              const size_t o = (size_t)row * p.n + col;
              if (p.c_f16) {
                lo = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const _Float16*>(p.c) + o);
              } else {
                lo = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const float*>(p.c) + o);
                hi = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const float*>(p.c) + o + 4);
              }
            }
            c_raw[it][0] = lo.x; c_raw[it][1] = lo.y; c_raw[it][2] = lo.z; c_raw[it][3] = lo.w;
            c_raw[it][4] = hi.x; c_raw[it][5] = hi.y; c_raw[it][6] = hi.z; c_raw[it][7] = hi.w;
          }
          store_rows(fm);
#pragma unroll
          for (int it = 0; it < ITERS; ++it) {
            const int piece = it * 64 + lane;
            const int r = piece / PER_ROW, c8 = (piece % PER_ROW) * 8;
            const int row = row_base + r, col = col0 + c8;
            const int sw = read_swizzle(r, 2);
            const float4 lo = *reinterpret_cast<const float4*>(scratch + r * WCOLS + (c8 ^ sw));
            const float4 hi = *reinterpret_cast<const float4*>(scratch + r * WCOLS + ((c8 + 4) ^ sw));
            float x[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            if (row < row_limit && col < p.n) {
              const size_t o = (size_t)row * p.n + col;
#pragma unroll
              for (int j = 0; j < 8; ++j) x[j] = p.alpha * x[j];
              if (use_c) {
                if (p.c_f16) {
                  const half8_t cv =
                      __builtin_bit_cast(half8_t, u32x4_t{c_raw[it][0], c_raw[it][1], c_raw[it][2], c_raw[it][3]});
#pragma unroll
                  for (int j = 0; j < 8; ++j) x[j] = x[j] + p.beta * (float)cv[j];
                } else {
#pragma unroll
                  for (int j = 0; j < 8; ++j) x[j] = x[j] + p.beta * __builtin_bit_cast(float, c_raw[it][j]);
                }
              }
              half8_t out;
#pragma unroll
              for (int j = 0; j < 8; ++j) out[j] = (_Float16)x[j];
              *reinterpret_cast<half8_t*>(reinterpret_cast<_Float16*>(d_out) + o) = out;
            }
          }
        } else {
          constexpr int PER_ROW = WCOLS / 4;           // 16-byte pieces (4 floats) per row
          constexpr int ITERS = 32 * PER_ROW / 64;
          uint32_t c_raw[ITERS][4];                    // fp32 C: one 16-byte load per piece; fp16 C: one 8-byte load
#pragma unroll
          for (int it = 0; it < ITERS; ++it) {
            const int piece = it * 64 + lane;
            const int row = row_base + piece / PER_ROW, col = col0 + (piece % PER_ROW) * 4;
            u32x4_t lo = u32x4_t{0, 0, 0, 0};
            if (use_c && row < row_limit && col < p.n) {
              const size_t o = (size_t)row * p.n + col;
              if (p.c_f16) {
                const u32x2_t t = *reinterpret_cast<const u32x2_t*>(reinterpret_cast<const _Float16*>(p.c) + o);
                lo.x = t.x; lo.y = t.y;
              } else {
                lo = *reinterpret_cast<const u32x4_t*>(reinterpret_cast<const float*>(p.c) + o);
              }
            }
            c_raw[it][0] = lo.x; c_raw[it][1] = lo.y; c_raw[it][2] = lo.z; c_raw[it][3] = lo.w;
          }
          store_rows(fm);
#pragma unroll
          for (int it = 0; it < ITERS; ++it) {
            const int piece = it * 64 + lane;
            const int r = piece / PER_ROW, c4 = (piece % PER_ROW) * 4;
            const int row = row_base + r, col = col0 + c4;
            const float4 a4 = *reinterpret_cast<const float4*>(scratch + r * WCOLS + (c4 ^ read_swizzle(r, 2)));
            float x[4] = {a4.x, a4.y, a4.z, a4.w};
            if (row < row_limit && col < p.n) {
              const size_t o = (size_t)row * p.n + col;
#pragma unroll
              for (int j = 0; j < 4; ++j) x[j] = p.alpha * x[j];
              if (use_c) {
                if (p.c_f16) {
                  const half4_t cv = __builtin_bit_cast(half4_t, u32x2_t{c_raw[it][0], c_raw[it][1]});
#pragma unroll
                  for (int j = 0; j < 4; ++j) x[j] = x[j] + p.beta * (float)cv[j];
                } else {
#pragma unroll
                  for (int j = 0; j < 4; ++j) x[j] = x[j] + p.beta * __builtin_bit_cast(float, c_raw[it][j]);
                }
              }
              *reinterpret_cast<float4*>(reinterpret_cast<float*>(d_out) + o) = float4{x[0], x[1], x[2], x[3]};
            }
          }
        }
      }
      return;
    }
  }
  // Direct form (generic variant, or C / D not 16-byte aligned): one element per accumulator register.
  auto finish_element = [&](int row, int col, float sum) __attribute__((always_inline)) {
    if (row < row_limit && col < p.n) {
      const size_t o = (size_t)row * p.n + col;
      float x = p.alpha * sum;
      if (p.beta != 0.f) {
        const float cv = p.c_f16 ? (float)reinterpret_cast<const _Float16*>(p.c)[o]
                                 : reinterpret_cast<const float*>(p.c)[o];
        x = x + p.beta * cv;
      }
      if (p.d_f16) reinterpret_cast<_Float16*>(d_out)[o] = (_Float16)x;
      else reinterpret_cast<float*>(d_out)[o] = x;
    }
  };
  if constexpr (M16) {
#pragma unroll
    for (int rt = 0; rt < 2 * FM; ++rt)
#pragma unroll
      for (int ct = 0; ct < 2 * FN; ++ct)
#pragma unroll
        for (int v = 0; v < 4; ++v)
          finish_element(row0 + rt * 16 + 4 * (lane >> 4) + v, col0 + ct * 16 + (lane & 15), acc16[rt][ct][v]);
    return;
  }
  const int col_lane = lane & 31;
  const int row_lane = 4 * (lane >> 5);
#pragma unroll
  for (int fm = 0; fm < FM; ++fm) {
    if (!finishes(fm)) continue;  // the other K group stores this fragment
#pragma unroll
    for (int fn = 0; fn < FN; ++fn) {
      const int col = col0 + fn * 32 + col_lane;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        finish_element(row0 + fm * 32 + 8 * (v / 4) + row_lane + (v % 4), col, acc[fm][fn][v]);
      }
    }
  }
}

// =====================================================================================================
// skinny_kernel: N <= 64 (decode shapes). HBM-bound: every byte of the prepared operand is read once.
// Workgroup = NW wavefronts that share R row blocks (32 rows each) and split K among themselves: wavefront w
// takes the K chunks (of 256) w, w + NW, w + 2 NW, ... Each wavefront stages B rows in a private 8 KiB LDS region
// as a zero-padded fp16 image of NC columns (NC = 16: the 256 rows of a chunk; NC = 32: 128 rows, two images per
// chunk; NC = 64: 64 rows, four images, two column fragments), feeds them to SMFMAC through transpose reads (one fragment serves the R row blocks) and keeps a 32x32
// fp32 partial tile per row block (NC = 16: two 16x16 tiles, multiplied with v_smfmac_f32_16x16x64_f16, which has no
// idle columns at sixteen). The prepared operand and the next image are loaded into registers while the
// current one is multiplied. Wavefronts never wait for one another inside the K loop (LDS operations of one
// wavefront execute in order). The NW partial tiles of a row block are added through LDS in wavefront order
// (deterministic; the tiles take the place of the images, as many row blocks per round as fit the 8 KiB) and the
// epilogue is applied. grid = M / (32 R) workgroups; no global workspace, no atomics.
// =====================================================================================================
constexpr int kSkinnyRegion = 8192;  // bytes of one B image

// how B rows reach the image: whole rows are the image rows (n == NC), rows of n % 8 == 0 elements in 16-byte
// pieces padded to the image row, 8-byte rows (n == 4, NC == 16), or element by element (any n <= NC, any alignment)
// kSkinnyBTokens: the token-major form of the linear layer. B is x, n rows (tokens) of k consecutive values, and
// the result is written as y[token][weight row] (+ bias[weight row]). The image is then token-major too: row t holds
// the image's K range of token t in 16-byte pieces, piece p stored at position p ^ token_swizzle(t) so that lanes
// which read the same piece of consecutive tokens fall into different banks; a lane's SMFMAC operand is two plain
// 16-byte reads (K consecutive inside a piece), no transpose.
// kSkinnyBRun: n = 2 or 4 with B 16-byte aligned. The 256 rows of a chunk are one run of 512 n consecutive bytes,
// loaded in 16-byte pieces (32 n of them: at most two load instructions per wavefront and chunk, where the row-wise
// modes issue eight; the split-K kernel's time is set by the number of load instructions it issues) and spread over the image rows
// by LDS stores of 2 n bytes.
enum SkinnyBMode { kSkinnyBFull = 0, kSkinnyB8 = 1, kSkinnyB4 = 2, kSkinnyBScalar = 3, kSkinnyBTokens = 4, kSkinnyBRun = 5 };

// 16-byte piece q of the image whose first row is B row k_base: image row q / (NC / 8), columns 8 (q % (NC / 8))
// ... + 7; zero outside B. Vector modes only.
template <int NC>
__device__ __forceinline__ u32x4_t skinny_load_piece(const _Float16* __restrict__ b, int n, int mode, int k_base,
                                                      int rows_valid, int q) {
  constexpr int PPR = NC / 8;  // pieces per image row
  const int row = q / PPR, h = q % PPR;
  const bool ok = row < rows_valid;
  const char* base = reinterpret_cast<const char*>(b);
  u32x4_t v = u32x4_t{0, 0, 0, 0};
  if (mode == kSkinnyBFull) {
    const char* src = ok ? base + ((size_t)k_base * NC + (size_t)q * 8) * 2 : base;
    v = *reinterpret_cast<const u32x4_t*>(src);
    if (!ok) v = u32x4_t{0, 0, 0, 0};
  } else if (mode == kSkinnyB8) {
    const bool use = ok && 8 * h < n;
    const char* src = use ? base + ((size_t)(k_base + row) * n + 8 * h) * 2 : base;
    v = *reinterpret_cast<const u32x4_t*>(src);
    if (!use) v = u32x4_t{0, 0, 0, 0};
  } else {  // kSkinnyB4
    const bool use = ok && h == 0;
    const char* src = use ? base + (size_t)(k_base + row) * 8 : base;
    const u32x2_t t = *reinterpret_cast<const u32x2_t*>(src);
    if (use) v = u32x4_t{t.x, t.y, 0, 0};
  }
  return v;
}

// The body of the split-K kernel for workgroup (block_x, block_y) of problem p: block_x = row group, block_y = K split.
template <int NW, int R, int MODE, int NC>
__device__ __forceinline__ void skinny_body(const SkinnyArgs& p, const int block_x, const int block_y) {
  constexpr int NT = 64 * NW;
  constexpr int IMG_ROWS = kSkinnyRegion / (NC * 2);   // B rows per image: 256, 128 or 64
  constexpr int SUB = kChunkK / IMG_ROWS;              // images per chunk: 1, 2 or 4
  constexpr int IMG_STEPS = kStepsPerChunk / SUB;      // 32-wide K steps per image: 8, 4 or 2
  constexpr int ROW_BYTES = NC * 2;
  constexpr int NF = NC <= 32 ? 1 : NC / 32;           // 32-column fragments per image row
  constexpr int TILE_BYTES = kRowBlock * NC * 4;       // one fp32 partial tile
  static_assert(NC == 16 || NC == 32 || NC == 64, "image width");
  static_assert(MODE != kSkinnyB4 || NC == 16, "the 8-byte-row mode is for 16 columns");
  static_assert(MODE != kSkinnyBRun || NC == 16, "the run mode is for 16 columns");
  // the partial tiles reuse the wavefront's image memory, RT row blocks per round of the final reduction
  constexpr int RT = R * TILE_BYTES <= kSkinnyRegion ? R : kSkinnyRegion / TILE_BYTES;
  static_assert(RT >= 1 && R % RT == 0, "the row blocks must divide into whole reduction rounds");
  constexpr bool TOKENS = MODE == kSkinnyBTokens;
  // Sixteen columns fill half of the 32x32x32 SMFMAC's result tile; v_smfmac_f32_16x16x64_f16 has no idle half and
  // multiplies a row block's chunk in half the matrix-pipe time (eight instructions of four passes).
  constexpr bool M16 = NC == 16;
  constexpr int PPT = IMG_ROWS / 8;                    // token-major image: 16-byte pieces per token row
  constexpr int TPI = 64 / PPT;                        // ... and tokens covered by the 64 pieces of one wavefront load
  constexpr int TOKEN_ROW_BYTES = IMG_ROWS * 2;
  __shared__ __attribute__((aligned(16))) char bs[NW * kSkinnyRegion];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rb_total = p.m / kRowBlock;
  const int rb_first = block_x * R;
  char* region = bs + wave * kSkinnyRegion;
  // kernel arguments the lambdas use, as values (capturing the argument struct would move it to scratch memory)
  const _Float16* __restrict__ b_ptr = p.b;
  const uint8_t* __restrict__ prep = p.prep;
  const int n_cols = p.n, k_rows = p.k, kc_total = p.kc_total;

  // The streaming loads go through buffer descriptors: wave-uniform base and offset in scalar registers, lane
  // offsets in one vector register, no vector address arithmetic inside the K loop. One descriptor per row block
  // (its kc_total blocks are consecutive, under 4 GiB for any K the argument checks admit) and one for B.
  const uint32_t meta_off = (uint32_t)lane * 16u, sign_off = (uint32_t)kSignOffset + (uint32_t)lane * 8u;
  buffer_t a_buffer[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    int rb = rb_first + r;
    if (rb >= rb_total) rb = rb_total - 1;  // never stored
    a_buffer[r] = make_buffer(prep + (size_t)rb * kc_total * kBlockBytes, (uint32_t)kc_total * kBlockBytes);
  }
  auto load_a = [&](int kc, AChunk (&a)[R]) __attribute__((always_inline)) {
    if (kc >= kc_total) kc = kc_total - 1;  // never multiplied
    const uint32_t block = (uint32_t)kc * kBlockBytes;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      a[r].meta = buffer_load16(a_buffer[r], meta_off, block);
      a[r].sign = buffer_load8(a_buffer[r], sign_off, block);
    }
  };
  // K split over workgroups (grid.y > 1): this workgroup multiplies the chunks [kc_begin, kc_end) and writes raw fp32
  // sums to its slice of the partial-sum buffer; a second kernel adds the slices in order and applies the epilogue.
  const int kc_begin = block_y * p.chunks_per_split;
  const int kc_end = kc_begin + p.chunks_per_split < kc_total ? kc_begin + p.chunks_per_split : kc_total;
  const int first = kc_begin + wave;  // this wavefront's first chunk
  // Short K (at most two chunks per wavefront, e.g. 11008 x 4096): everything the wavefront will read is requested
  // at once, so the kernel pays one memory latency instead of one per chunk.
  constexpr bool kShortPath = NW <= 8 && SUB == 1 && MODE != kSkinnyBScalar;
  const bool short_k = kShortPath && kc_end - kc_begin <= 2 * NW;
  // The prepared operand comes from HBM and is what the first SMFMAC waits for longest: the loop form issues its first
  // loads here, before the rest of the set-up (B descriptor, image offsets, fragment addresses), which then runs under
  // their latency (4096 x 4096 x 16: 4.87 -> 4.70 us). The short form keeps B first: loads return in order, and a B image
  // requested behind the weights would reach LDS only after them (11008 x 4096 x 1: 5.6 -> 6.3 us when tried).
  AChunk a_cur[R], a_next[R];
  if (!short_k) {
    load_a(first, a_cur);
    __builtin_amdgcn_sched_barrier(0);
  }
  const size_t b_bytes = (size_t)k_rows * n_cols * 2;
  const bool b_fits = b_bytes < (size_t(1) << 32);  // else every image takes the general path
  const buffer_t b_buffer = make_buffer(b_ptr, b_fits ? (uint32_t)b_bytes : 0u);
  auto rows_valid_of = [&](int k_base) __attribute__((always_inline)) {
    const int rows = k_rows - k_base;
    return rows < 0 ? 0 : (rows > IMG_ROWS ? IMG_ROWS : rows);
  };
  // element mode: image position of element `lane` of an image's run of IMG_ROWS * n elements, and the step of 64
  const int elem_col0 = lane % n_cols;
  const int elem_offset0 = (lane / n_cols) * ROW_BYTES + elem_col0 * 2;
  const int step_cols = 64 % n_cols;
  const int step_bytes = (64 / n_cols) * ROW_BYTES + step_cols * 2;
  // Image t of this wavefront = B rows [k_base, k_base + IMG_ROWS) with k_base = (wave + NW (t / SUB)) * 256 +
  // (t % SUB) * IMG_ROWS. Vector modes: the image travels through registers, loaded while the previous image is
  // multiplied; element mode: loaded and stored in one go when the image is due.
  // token-major image: piece lane + 64 i = K values [8 p, 8 p + 8) of the image for token token_lane + TPI i
  const int piece_lane = lane % PPT, token_lane = lane / PPT;
  const uint32_t token_load_base = ((uint32_t)token_lane * (uint32_t)k_rows + 8u * piece_lane) * 2u;
  const uint32_t token_load_step = (uint32_t)TPI * (uint32_t)k_rows * 2u;
  const uint32_t token_store_base =
      (uint32_t)token_lane * TOKEN_ROW_BYTES + (uint32_t)((piece_lane ^ token_swizzle<TOKEN_ROW_BYTES>(token_lane)) << 4);
  // run mode: piece q = lane + 64 i of the image's run; pieces at or past 32 n are sent outside the descriptor (zero)
  const uint32_t run_pieces = 32u * (uint32_t)n_cols;
  auto load_b = [&](int k_base, u32x4_t (&v)[8]) __attribute__((always_inline)) {
    if (MODE == kSkinnyBScalar) return;
    if (MODE == kSkinnyBRun) {
      const uint32_t run_base = (uint32_t)k_base * (uint32_t)n_cols * 2u;  // the launcher checks k n 2 < 2^32
      if (k_base + IMG_ROWS <= k_rows) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
          if (64u * i < run_pieces)
            v[i] = buffer_load16(b_buffer, lane + 64u * i < run_pieces ? meta_off + 1024u * i : 0xFFFFFF00u, run_base);
        return;
      }
      // last image of a K that is no multiple of 256 (or an image past the end that is loaded but never multiplied):
      // pieces inside B as they are, zeros past its end. K is a multiple of 32, so the valid bytes are a multiple of 16 n
      // and no piece straddles the end.
      const uint32_t valid_bytes = (uint32_t)rows_valid_of(k_base) * (uint32_t)n_cols * 2u;
#pragma unroll
      for (int i = 0; i < 2; ++i)
        if (64u * i < run_pieces)
          v[i] = buffer_load16(b_buffer, meta_off + 1024u * i + 16u <= valid_bytes ? run_base + meta_off + 1024u * i : 0xFFFFFF00u, 0);
      return;
    }
    if (TOKENS) {
      // offsets at or past n * k * 2 (tokens >= n) fall outside the descriptor and read as zero; K positions at or
      // past k are sent there too (the launcher checks that 64 * k * 2 stays well below 2^32)
      if (k_base + IMG_ROWS <= k_rows) {
        // the image's whole K range exists (wave-uniform test): lane offsets that do not change from image to image
        // plus a scalar offset; the range check looks at the lane offset alone, which is what sends tokens >= n to zero
        // (load i covers tokens TPI i ... TPI i + TPI - 1: nothing to fetch past the last token)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (TPI * i < n_cols) v[i] = buffer_load16(b_buffer, token_load_base + i * token_load_step, (uint32_t)k_base * 2u);
          else v[i] = u32x4_t{0, 0, 0, 0};
        }
        return;
      }
      const bool inside = k_base + 8 * piece_lane < k_rows;
      const uint32_t first = token_load_base + (uint32_t)k_base * 2u;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (TPI * i < n_cols) v[i] = buffer_load16(b_buffer, inside ? first + i * token_load_step : 0xFFFFFF00u, 0);
        else v[i] = u32x4_t{0, 0, 0, 0};
      }
      return;
    }
    if (MODE == kSkinnyBFull && b_fits && k_base + IMG_ROWS <= k_rows) {
      // the whole image lies inside B (wave-uniform test): 8 KiB of consecutive memory, no per-piece checks
      const uint32_t image = (uint32_t)k_base * (NC * 2);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = buffer_load16(b_buffer, meta_off + 1024u * i, image);
      return;
    }
    const int rows_valid = rows_valid_of(k_base);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = skinny_load_piece<NC>(b_ptr, n_cols, MODE, k_base, rows_valid, lane + i * 64);
  };
  auto store_b = [&](int k_base, const u32x4_t (&v)[8]) __attribute__((always_inline)) {
    if (MODE == kSkinnyBScalar) {
      // the image's rows are one run of IMG_ROWS n elements; rows at or past K are written as zeros, the padding
      // columns n ... NC - 1 keep the zeros the image was cleared to
      const int valid = rows_valid_of(k_base) * n_cols, total = IMG_ROWS * n_cols;
      const _Float16* src = b_ptr + (size_t)k_base * n_cols;
      constexpr int BATCH = NC >= 32 ? 16 : 4;  // loads in flight per lane
      int offset = elem_offset0;  // byte offset in the image of element e = lane + 64 i, kept without divisions
      int col = elem_col0;
      for (int e0 = lane; e0 < total; e0 += 64 * BATCH) {
        uint16_t bits[BATCH];
#pragma unroll
        for (int i = 0; i < BATCH; ++i) {
          const int e = e0 + i * 64;
          bits[i] = __builtin_bit_cast(uint16_t, e < valid ? src[e] : b_ptr[0]);
          if (e >= valid) bits[i] = 0;
        }
#pragma unroll
        for (int i = 0; i < BATCH; ++i) {
          const int e = e0 + i * 64;
          if (e < total) *reinterpret_cast<uint16_t*>(region + offset) = bits[i];
          // e += 64: 64 / n rows further and 64 % n columns, with one carry at most
          col += step_cols;
          offset += step_bytes;
          if (col >= n_cols) {
            col -= n_cols;
            offset += ROW_BYTES - n_cols * 2;
          }
        }
      }
      return;
    }
    if (MODE == kSkinnyBRun) {
      // piece q holds the n columns of rows 8 q / n ... : 2 n bytes to each row's start; columns n ... 15 keep the zeros the
      // image was cleared to
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint32_t q = lane + 64u * i;
        if (q >= run_pieces) continue;
        if (n_cols == 4) {
          *reinterpret_cast<u32x2_t*>(region + (2 * q) * ROW_BYTES) = u32x2_t{v[i].x, v[i].y};
          *reinterpret_cast<u32x2_t*>(region + (2 * q + 1) * ROW_BYTES) = u32x2_t{v[i].z, v[i].w};
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) *reinterpret_cast<uint32_t*>(region + (4 * q + j) * ROW_BYTES) = v[i][j];
        }
      }
      return;
    }
    if (TOKENS) {
      // token = token_lane + TPI i with token_lane < TPI (a power of two): the two terms share no bits, so the swizzle of
      // piece i differs from that of piece 0 by a compile-time XOR
#pragma unroll
      for (int i = 0; i < 8; ++i)
        *reinterpret_cast<u32x4_t*>(region + (token_store_base ^ (uint32_t)(token_swizzle<TOKEN_ROW_BYTES>(TPI * i) << 4)) + i * 1024) = v[i];
      return;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4_t*>(region + (lane + i * 64) * 16) = v[i];
  };

  float16_t acc[R][NF];
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[r][f][v] = 0.f;
  float4v_t acc16[R][2];  // M16: rows 0-15 and 16-31 of the row block; register v of lane l = row 4 (l / 16) + v, column l % 16
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int h = 0; h < 2; ++h) acc16[r][h] = float4v_t{0.f, 0.f, 0.f, 0.f};
  const uint32_t one = packed_one_in_vgpr();
  const int i16 = lane & 15, gb = lane >> 5, g16 = lane >> 4;
  // (32x32x32 form, NC >= 32; sixteen-column images use the 16x16x64 form further down)
  const int chunk8 = (NC >= 32 ? ((lane & 31) >> 4) * 4 : 0) + (i16 & 3);  // 8-byte piece of the 32-column fragment
  const char* lane_ptr = region + (8 * gb + (i16 >> 2)) * ROW_BYTES + chunk8 * 8;

  // token-major image: this lane's token row and swizzle; K step s of the image needs pieces 4 s + gb and 4 s + 2 + gb
  const int token_col = NC >= 32 ? (lane & 31) : i16;
  const uint32_t token_read_base = (uint32_t)token_col * TOKEN_ROW_BYTES + (uint32_t)((gb ^ token_swizzle<TOKEN_ROW_BYTES>(token_col)) << 4);
  // ---- 16x16x64 form (M16). The instruction's A lane (row l % 16, group g = l / 16) holds eight kept values and their
  // 16 index bits for 16 consecutive K positions, as a lane of the prepared block does for one K step: lane
  // (row, half ga) of the block, step s. Which K positions group g stands for is free as long as B agrees, so the
  // operands are built with one v_permlane16_swap per register pair instead of a gather: swapping the odd 16-lane
  // rows of metadata register 2 P with the even rows of register 2 P + 1 leaves in the first register, for
  // block rows 0-15, the groups (ga 0, steps 4 P + {0, 1}), (ga 0, steps 4 P + {2, 3}), (ga 1, steps 4 P + {0, 1}),
  // (ga 1, steps 4 P + {2, 3}) and in the second register the same for block rows 16-31; ABID picks the even or the
  // odd step of each pair. Instruction (P, abid) therefore covers K positions 128 P + 32 abid + [0, 32) and
  // 128 P + 32 abid + 64 + [0, 32) of the chunk: group g positions 128 P + 32 abid + 64 (g % 2) + 16 (g / 2) + [0, 16).
  // The sign words travel the same way (a register swapped with its own copy) and are shifted by 8 (g % 2) once, after
  // which the expansion uses compile-time shifts. B lane (column l % 16, group gb) holds instruction K rows
  // 8 gb + [0, 8) and 32 + 8 gb + [0, 8), i.e. chunk rows base + [0, 8) and base + 16 + [0, 8) with
  // base = 128 P + 32 abid + 64 (gb / 2) + 8 (gb % 2).
  struct A16 {
    uint32_t idx[2][2];   // [row half][P]
    uint32_t sign[2][2];
  };
  const uint32_t sign_shift16 = 8u * (g16 & 1);
  auto gather16 = [&](const AChunk& a) __attribute__((always_inline)) {
    A16 t;
#pragma unroll
    for (int P = 0; P < 2; ++P) {
      const auto m = __builtin_amdgcn_permlane16_swap(a.meta[2 * P], a.meta[2 * P + 1], false, false);
      const uint32_t w = P == 0 ? a.sign.x : a.sign.y;
      const auto sg = __builtin_amdgcn_permlane16_swap(w, w, false, false);
      t.idx[0][P] = m[0];
      t.idx[1][P] = m[1];
      t.sign[0][P] = sg[0] << sign_shift16;
      t.sign[1][P] = sg[1] << sign_shift16;
    }
    return t;
  };
  const char* lane_ptr16 = region + (64 * (g16 >> 1) + 8 * (g16 & 1) + (i16 >> 2)) * ROW_BYTES + (i16 & 3) * 8;
  const uint32_t token_read_base16 =
      (uint32_t)i16 * TOKEN_ROW_BYTES + (uint32_t)(((8 * (g16 >> 1) + (g16 & 1)) ^ token_swizzle<TOKEN_ROW_BYTES>(i16)) << 4);
  // B operand of instruction F = 2 P + abid
  auto frag16 = [&](int F) __attribute__((always_inline)) {
    u32x8_t raw;
    if (TOKENS) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const u32x4_t t = *reinterpret_cast<const u32x4_t*>(
            region + (token_read_base16 ^ (uint32_t)((16 * (F >> 1) + 4 * (F & 1) + 2 * h) << 4)));
        raw[4 * h] = t.x; raw[4 * h + 1] = t.y; raw[4 * h + 2] = t.z; raw[4 * h + 3] = t.w;
      }
      return __builtin_bit_cast(half16_t, raw);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int row_const = 128 * (F >> 1) + 32 * (F & 1) + 4 * (q & 1) + 16 * (q >> 1);
      const u32x2_t t = lds_read_tr16(lane_ptr16 + row_const * ROW_BYTES);
      raw[2 * q] = t.x;
      raw[2 * q + 1] = t.y;
    }
    return __builtin_bit_cast(half16_t, raw);
  };
  auto compute16 = [&](const AChunk (&a)[R]) __attribute__((always_inline)) {
    half16_t bf[4];
#pragma unroll
    for (int F = 0; F < 4; ++F) bf[F] = frag16(F);
    A16 t[R];
#pragma unroll
    for (int r = 0; r < R; ++r) t[r] = gather16(a[r]);
#pragma unroll
    for (int F = 0; F < 4; ++F)
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          u32x4_t av;
#pragma unroll
          for (int q = 0; q < 4; ++q) av[q] = ((t[r].sign[h][F >> 1] << (4 * (F & 1) + q)) & 0x80008000u) | one;
          const half8_t a8 = __builtin_bit_cast(half8_t, av);
          if ((F & 1) == 0)
            acc16[r][h] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a8, bf[F], acc16[r][h], (int)t[r].idx[h][F >> 1], 0, 0);
          else
            acc16[r][h] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a8, bf[F], acc16[r][h], (int)t[r].idx[h][F >> 1], 0, 1);
        }
  };

  auto frag = [&](int image_step, int f) __attribute__((always_inline)) {
    u32x8_t raw;
    if (TOKENS) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const u32x4_t t = *reinterpret_cast<const u32x4_t*>(
            region + (token_read_base ^ (uint32_t)((4 * image_step + 2 * h) << 4)) + f * 32 * TOKEN_ROW_BYTES);
        raw[4 * h] = t.x; raw[4 * h + 1] = t.y; raw[4 * h + 2] = t.z; raw[4 * h + 3] = t.w;
      }
      return __builtin_bit_cast(half16_t, raw);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int row_const = image_step * 32 + 4 * (q & 1) + 16 * (q >> 1);
      const u32x2_t t = lds_read_tr16(lane_ptr + row_const * ROW_BYTES + f * 64);
      raw[2 * q] = t.x;
      raw[2 * q + 1] = t.y;
    }
    return __builtin_bit_cast(half16_t, raw);
  };
  // the SMFMACs of image SUB_INDEX of a chunk: steps SUB_INDEX * IMG_STEPS ... + IMG_STEPS - 1
  auto compute = [&](const AChunk (&a)[R], auto sub_tag) __attribute__((always_inline)) {
    if constexpr (M16) {
      compute16(a);
      return;
    }
    constexpr int FIRST_STEP = decltype(sub_tag)::value * IMG_STEPS;
    // Fragments are read in groups of FG K steps (4 FG transpose reads per column fragment) into one of two register
    // sets: while the SMFMACs of a group run, the reads of the next group are already in flight, so only the first
    // group of an image waits for LDS. The scheduling barriers keep later groups' reads from being hoisted as well
    // (8 registers per fragment). Sixteen-wavefront workgroups have 128 registers per wavefront and no room for the
    // second set: they read each group when it is due.
    constexpr bool kAhead = NW <= 8;
    constexpr int FG = (R >= 4 || NF > 1) ? 2 : 4;
    constexpr int GROUPS = IMG_STEPS / FG;
    static_assert(IMG_STEPS % FG == 0 && GROUPS >= 1 && GROUPS <= 4, "whole groups of K steps per image");
    half16_t bfrag[kAhead ? 2 : 1][FG][NF];
    auto read_group = [&](int first_in_image, half16_t (&dst)[FG][NF]) __attribute__((always_inline)) {
#pragma unroll
      for (int st = 0; st < FG; ++st)
#pragma unroll
        for (int f = 0; f < NF; ++f) dst[st][f] = frag(first_in_image + st, f);
    };
    auto group = [&](auto index_tag) __attribute__((always_inline)) {
      constexpr int G = decltype(index_tag)::value;
      if constexpr (G < GROUPS) {
        constexpr int FIRST = FIRST_STEP + G * FG;  // step within the chunk
        constexpr int SET = kAhead ? (G & 1) : 0;
        if constexpr (!kAhead) read_group(G * FG, bfrag[0]);
        else if constexpr (G + 1 < GROUPS) read_group((G + 1) * FG, bfrag[SET ^ 1]);
        auto step = [&](auto offset_tag) __attribute__((always_inline)) {
          constexpr int OFFSET = decltype(offset_tag)::value;
          if constexpr (OFFSET < FG) {
            constexpr int STEP = FIRST + OFFSET;
#pragma unroll
            for (int r = 0; r < R; ++r) {
              const half8_t av = expand_signs<STEP>(a[r], one);
#pragma unroll
              for (int f = 0; f < NF; ++f)
                acc[r][f] = smfmac_step<STEP, false>(a[r], av, bfrag[SET][OFFSET][f], acc[r][f]);
            }
          }
        };
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
        step(std::integral_constant<int, 2>{});
        step(std::integral_constant<int, 3>{});
        if constexpr (G + 1 < GROUPS) __builtin_amdgcn_sched_barrier(0);
      }
    };
    if constexpr (kAhead) read_group(0, bfrag[0]);
    group(std::integral_constant<int, 0>{});
    group(std::integral_constant<int, 1>{});
    group(std::integral_constant<int, 2>{});
    group(std::integral_constant<int, 3>{});
  };

  // sixteen wavefronts leave 128 registers each: no room to hold the next image (32 registers) during the SMFMACs
  constexpr bool kPrefetchB = NW <= 8 && MODE != kSkinnyBScalar;
  if (MODE == kSkinnyBScalar || MODE == kSkinnyBRun) {
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4_t*>(region + (lane + i * 64) * 16) = u32x4_t{0, 0, 0, 0};
  }
  u32x4_t breg[8];
  char* const d_out = reinterpret_cast<char*>(p.d) + (size_t)block_y * p.m * p.n * (p.d_f16 ? 2 : 4);
  if (short_k) {
    u32x4_t breg2[8];
    load_b(first * kChunkK, breg);
    load_a(first, a_cur);
    load_b((first + NW) * kChunkK, breg2);
    load_a(first + NW, a_next);
    if (first < kc_end) {
      store_b(first * kChunkK, breg);
      compute(a_cur, std::integral_constant<int, 0>{});
    }
    if (first + NW < kc_end) {
      store_b((first + NW) * kChunkK, breg2);
      compute(a_next, std::integral_constant<int, 0>{});
    }
  }
  if (kPrefetchB && !short_k) load_b(first * kChunkK, breg);
  for (int kc = short_k ? kc_end : first; kc < kc_end; kc += NW) {
    const int k_base = kc * kChunkK;
    // this wavefront has another chunk after this one (wave-uniform): only then is the next chunk requested; a load
    // past the last chunk would be one more instruction for the memory pipeline, a third of them when a wavefront
    // has two or three chunks
    const bool more = kc + NW < kc_end;
    if (!kPrefetchB) load_b(k_base, breg);
    store_b(k_base, breg);  // after the previous image's fragment reads: LDS operations of a wavefront execute in order
    if (kPrefetchB && (SUB > 1 || more)) load_b(SUB > 1 ? k_base + IMG_ROWS : k_base + NW * kChunkK, breg);
    if (more) load_a(kc + NW, a_next);
    compute(a_cur, std::integral_constant<int, 0>{});
    // the chunk's further images (SUB - 1 of them)
    auto further = [&](auto sub_tag) __attribute__((always_inline)) {
      constexpr int S = decltype(sub_tag)::value;
      if constexpr (S < SUB) {
        const int image_base = k_base + S * IMG_ROWS;
        if (!kPrefetchB) {
          __builtin_amdgcn_sched_barrier(0);  // this image's loads stay behind the previous image's SMFMACs
          load_b(image_base, breg);
        }
        store_b(image_base, breg);
        if (kPrefetchB && (S + 1 < SUB || more)) load_b(S + 1 < SUB ? image_base + IMG_ROWS : k_base + NW * kChunkK, breg);
        compute(a_cur, sub_tag);
      }
    };
    further(std::integral_constant<int, 1>{});
    further(std::integral_constant<int, 2>{});
    further(std::integral_constant<int, 3>{});
#pragma unroll
    for (int r = 0; r < R; ++r) a_cur[r] = a_next[r];
  }

  smfmac_drain();
  // ---- add the NW partial tiles through LDS: region of wavefront w := its R tiles as [r][32 rows][NC cols] fp32
  constexpr int ROUND_ROWS = RT * kRowBlock;
#pragma unroll
  for (int round = 0; round < R / RT; ++round) {
    if (round > 0) __syncthreads();  // the previous round's tiles have been read
    {
      float* tile = reinterpret_cast<float*>(region);
      const int col = lane & 31;
      if (M16) {
#pragma unroll
        for (int rr = 0; rr < RT; ++rr)
#pragma unroll
          for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              const int row = 16 * h + 4 * g16 + v;
              const float value = acc16[round * RT + rr][h][v];
              if (TOKENS) tile[i16 * ROUND_ROWS + ((rr * 32 + row) ^ i16)] = value;
              else tile[(rr * 32 + row) * NC + i16] = value;
            }
      } else if (col < NC) {
#pragma unroll
        for (int rr = 0; rr < RT; ++rr)
#pragma unroll
          for (int f = 0; f < NF; ++f)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
              const int row = 8 * (v / 4) + 4 * (lane >> 5) + (v % 4);
              const float value = acc[round * RT + rr][f][v];
              // token-major: [token][weight row of the round], the row index XOR-swizzled by the token so that neither
              // these stores (32 tokens, one row) nor the reads below (one token, consecutive rows) collide in a bank
              if (TOKENS) tile[(f * 32 + col) * ROUND_ROWS + ((rr * 32 + row) ^ col)] = value;
              else tile[(rr * 32 + row) * NC + f * 32 + col] = value;
            }
      }
    }
    __syncthreads();
    const int round_row0 = rb_first * kRowBlock + round * ROUND_ROWS;
    if (TOKENS) {
      for (int idx = tid; idx < ROUND_ROWS * NC; idx += NT) {
        const int local = idx % ROUND_ROWS, token = idx / ROUND_ROWS;
        const int pos = token * ROUND_ROWS + (local ^ (token & 31));
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += reinterpret_cast<const float*>(bs + w * kSkinnyRegion)[pos];
        const int row = round_row0 + local;
        if (token < p.n && row < p.m) {
          if (p.bias) sum += p.bias_f16 ? (float)reinterpret_cast<const _Float16*>(p.bias)[row]
                                        : reinterpret_cast<const float*>(p.bias)[row];
          const size_t o = (size_t)token * p.m + row;
          // a B of one column is a token-major x of one token and its result column is y: the launcher sends such calls
          // here with their alpha, beta and C (element o of C in both layouts); the linear layer passes 1, 0, null
          sum = p.alpha * sum;
          if (p.beta != 0.f)
            sum = sum + p.beta * (p.c_f16 ? (float)reinterpret_cast<const _Float16*>(p.c)[o] : reinterpret_cast<const float*>(p.c)[o]);
          if (p.d_f16) reinterpret_cast<_Float16*>(d_out)[o] = (_Float16)sum;
          else reinterpret_cast<float*>(d_out)[o] = sum;
        }
      }
    } else {
      for (int idx = tid; idx < ROUND_ROWS * NC; idx += NT) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) sum += reinterpret_cast<const float*>(bs + w * kSkinnyRegion)[idx];
        const int col = idx % NC;
        const int row = round_row0 + idx / NC;
        if (col < p.n && row < p.m) {
          const size_t o = (size_t)row * p.n + col;
          float x = p.alpha * sum;
          if (p.beta != 0.f) {
            const float cv = p.c_f16 ? (float)reinterpret_cast<const _Float16*>(p.c)[o] : reinterpret_cast<const float*>(p.c)[o];
            x = x + p.beta * cv;
          }
          if (p.d_f16) reinterpret_cast<_Float16*>(d_out)[o] = (_Float16)x;
          else reinterpret_cast<float*>(d_out)[o] = x;
        }
      }
    }
  }
}

template <int NW, int R, int MODE, int NC>
__global__ __launch_bounds__(64 * NW, NW == 16 ? 4 : 2) void skinny_kernel(SkinnyArgs p) {
  skinny_body<NW, R, MODE, NC>(p, blockIdx.x, blockIdx.y);
}

// Grouped form: several independent products y_i = x_i W_i^T + bias_i that share the token count, in one launch. The
// workgroups are numbered over the concatenated row groups of the problems; a workgroup finds its problem by
// comparing its number with the problems' first workgroups (wave-uniform, a handful of scalar compares) and then runs
// the token-major body on that problem's arguments. Decode-sized products take a few microseconds each, of which the
// launch itself and the ramp of the memory pipeline are a large part: one launch for the q / k / v or gate / up
// projections of a layer pays them once.
template <int NW, int R, int NC>
__global__ __launch_bounds__(64 * NW, NW == 16 ? 4 : 2) void skinny_group_kernel(SkinnyGroupArgs g) {
  int which = 0;
  for (int i = 1; i < g.count; ++i)
    if ((int)blockIdx.x >= g.first_block[i]) which = i;
  skinny_body<NW, R, kSkinnyBTokens, NC>(g.problem[which], (int)blockIdx.x - g.first_block[which], 0);
}

// =====================================================================================================
// pad_b_kernel: copies B (k x n, row stride n, any alignment) into rows of ldb = round_up(n, 8) halves, zeros in the
// padding columns, so that every row starts 16-byte aligned for the asynchronous copies of the main kernel.
// One thread per 16-byte piece of the destination.
// =====================================================================================================
__global__ __launch_bounds__(256) void pad_b_kernel(const _Float16* __restrict__ b, _Float16* __restrict__ dst, int k,
                                                    int n, int ldb) {
  const int pieces_per_row = ldb / 8;
  const size_t piece = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (piece >= (size_t)k * pieces_per_row) return;
  const size_t row = piece / pieces_per_row;
  const int col0 = (int)(piece % pieces_per_row) * 8;
  half8_t v;
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = col0 + j < n ? b[row * n + col0 + j] : (_Float16)0.f;
  *reinterpret_cast<half8_t*>(dst + row * ldb + col0) = v;
}

// =====================================================================================================
// splitk_reduce_kernel: d = alpha * (sum over splits, in split order, of the fp32 partial sums) + beta * c.
// Elementwise over the m * n results; VEC = 4 when the element count and the alignment of c and d allow it.
// Linear-layer form: bias (row_length values, may be null) is added instead, element i taking bias[i % row_length].
// =====================================================================================================
template <int VEC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ ws, int splits, size_t stride,
                                                            const void* __restrict__ c, void* __restrict__ d,
                                                            size_t total, float alpha, float beta, int c_f16,
                                                            int d_f16, const void* __restrict__ bias, int bias_f16,
                                                            int row_length) {
  const size_t first = ((size_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (first >= total) return;
  float x[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) x[j] = 0.f;
  for (int s = 0; s < splits; ++s) {
    const float* src = ws + (size_t)s * stride + first;
    if (VEC == 4) {
      const float4 v = *reinterpret_cast<const float4*>(src);
      x[0] += v.x; x[1 % VEC] += v.y; x[2 % VEC] += v.z; x[3 % VEC] += v.w;
    } else {
      x[0] += src[0];
    }
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    x[j] = alpha * x[j];
    if (beta != 0.f) {
      const float cv = c_f16 ? (float)reinterpret_cast<const _Float16*>(c)[first + j]
                             : reinterpret_cast<const float*>(c)[first + j];
      x[j] = x[j] + beta * cv;
    }
  }
  if (bias) {
    const size_t at = first % (size_t)row_length;  // row_length is a multiple of 4: a vector never wraps
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      x[j] += bias_f16 ? (float)reinterpret_cast<const _Float16*>(bias)[at + j] : reinterpret_cast<const float*>(bias)[at + j];
  }
  if (VEC == 4) {
    if (d_f16) {
      *reinterpret_cast<half4_t*>(reinterpret_cast<_Float16*>(d) + first) =
          half4_t{(_Float16)x[0], (_Float16)x[1 % VEC], (_Float16)x[2 % VEC], (_Float16)x[3 % VEC]};
    } else {
      *reinterpret_cast<float4*>(reinterpret_cast<float*>(d) + first) = float4{x[0], x[1 % VEC], x[2 % VEC], x[3 % VEC]};
    }
  } else {
    if (d_f16) reinterpret_cast<_Float16*>(d)[first] = (_Float16)x[0];
    else reinterpret_cast<float*>(d)[first] = x[0];
  }
}

// Second pass of a K split: ordered sum of the partial results and the epilogue (bias and row_length for the
// token-major form, where element i of y takes bias[i % m]).
static hipError_t launch_split_reduce(const float* ws, int splits, size_t total, const void* c, void* d, float alpha,
                                      float beta, int c_f16, int d_f16, const void* bias, int bias_f16, int row_length,
                                      hipStream_t stream) {
  const bool vec = total % 4 == 0 && (reinterpret_cast<uintptr_t>(d) & 15) == 0 &&
                   (beta == 0.f || (reinterpret_cast<uintptr_t>(c) & 15) == 0) && (!bias || row_length % 4 == 0);
  if (vec)
    hipLaunchKernelGGL(splitk_reduce_kernel<4>, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0, stream, ws,
                       splits, total, c, d, total, alpha, beta, c_f16, d_f16, bias, bias_f16, row_length);
  else
    hipLaunchKernelGGL(splitk_reduce_kernel<1>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, ws,
                       splits, total, c, d, total, alpha, beta, c_f16, d_f16, bias, bias_f16, row_length);
  return hipGetLastError();
}

// =====================================================================================================
// Host-side launchers
// =====================================================================================================
hipError_t launch_prepare(const void* a, const void* e, void* prep, int m, int k, int layout, hipStream_t stream) {
  const int kc_total = (k + kChunkK - 1) / kChunkK;
  const int rb_total = (m + kRowBlock - 1) / kRowBlock;
  dim3 grid(kc_total, rb_total);
  hipLaunchKernelGGL(prepare_kernel, grid, dim3(64), 0, stream, (const uint8_t*)a, (const uint16_t*)e, (uint8_t*)prep,
                     m, k, kc_total, layout);
  return hipGetLastError();
}

hipError_t launch_pack(const void* w, void* a, void* e, int m, int k, int prune, int layout, hipStream_t stream) {
  hipLaunchKernelGGL(pack_kernel, dim3((k / 16 + 3) / 4, m / 64), dim3(64), 0, stream, (const _Float16*)w, (uint8_t*)a,
                     (uint16_t*)e, m, k, prune, layout);
  return hipGetLastError();
}

template <int WM, int WN, int FM, int FN, bool DMA, bool TOKENS = false, int KG = 1, bool M16 = false>
static hipError_t launch_gemm_cfg(GemmArgs args, hipStream_t stream) {
  using TS = TileShape<WM, WN, FM, FN, KG>;
  args.tiles_m = (args.m + TS::BM - 1) / TS::BM;
  args.tiles_n = (args.n + TS::BN - 1) / TS::BN;
  const int lds = DMA ? TS::LDS_BYTES : TS::STAGE_BYTES;
  auto kern = gemm_kernel<WM, WN, FM, FN, DMA, TOKENS, KG, M16>;
  // the dynamic-LDS limit is a per-device attribute of the kernel; threads that race here set the same value
  static std::atomic<bool> attr_done[64] = {};
  int device = 0;
  if (hipError_t st = hipGetDevice(&device); st != hipSuccess) return st;
  if (device < 0 || device >= 64) return hipErrorInvalidDevice;
  if (!attr_done[device].load(std::memory_order_acquire)) {
    hipError_t st = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                        hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (st != hipSuccess) return st;
    attr_done[device].store(true, std::memory_order_release);
  }
  // XCDs of the device as the tile order sees them: gfx950 has 32 compute units per XCD, a whole MI355X eight of them;
  // a partition of the GPU shows fewer compute units and is served by as many XCDs
  static std::atomic<int> xcds_of[64] = {};
  int xcds = xcds_of[device].load(std::memory_order_relaxed);
  if (xcds <= 0) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) cus = 256;
    xcds = cus / 32 < 1 ? 1 : (cus / 32 > 8 ? 8 : cus / 32);
    xcds_of[device].store(xcds, std::memory_order_relaxed);
  }
  args.xcds = xcds;
  hipLaunchKernelGGL(kern, dim3(args.tiles_m * args.tiles_n, args.splits), dim3(64 * TS::NW), lds, stream, args);
  return hipGetLastError();
}

static hipError_t launch_gemm_pass(GemmArgs args, int tile_config, hipStream_t stream) {
  const bool aligned = (args.ldb % 8 == 0) && ((reinterpret_cast<uintptr_t>(args.b) & 15) == 0);
  // the coalesced epilogue moves 16 bytes per lane: n % 8 == 0 keeps every row start aligned when the bases are
  args.vector_epilogue = args.n % 8 == 0 && (reinterpret_cast<uintptr_t>(args.d) & 15) == 0 &&
                         (args.beta == 0.f || (reinterpret_cast<uintptr_t>(args.c) & 15) == 0);
  if (!aligned) return launch_gemm_cfg<4, 1, 1, 4, false>(args, stream);
  switch (tile_config) {
    case kTile512x128: return launch_gemm_cfg<4, 1, 4, 4, true>(args, stream);
    case kTile256x128: return launch_gemm_cfg<4, 1, 2, 4, true>(args, stream);
    case kTile128x128: return launch_gemm_cfg<4, 1, 1, 4, true>(args, stream);
    case kTile256x256: return launch_gemm_cfg<2, 2, 4, 4, true>(args, stream);
    case kTile256x128w: return launch_gemm_cfg<2, 2, 4, 2, true>(args, stream);
    case kTile512x128t: return launch_gemm_cfg<2, 2, 8, 2, true>(args, stream);
    case kTile128x128s: return launch_gemm_cfg<2, 2, 2, 2, true>(args, stream);
    case kTile256x64: return launch_gemm_cfg<2, 2, 4, 1, true>(args, stream);
    case kTile256x256w8: return launch_gemm_cfg<2, 4, 4, 2, true>(args, stream);
    case kTile512x128w8: return launch_gemm_cfg<4, 2, 4, 2, true>(args, stream);
    case kTile256x128w8: return launch_gemm_cfg<4, 2, 2, 2, true>(args, stream);
    case kTile128x128w8: return launch_gemm_cfg<2, 4, 2, 1, true>(args, stream);
    case kTile64x128: return launch_gemm_cfg<2, 2, 1, 2, true>(args, stream);
    case kTile128x128k2: return launch_gemm_cfg<2, 2, 2, 2, true, false, 2>(args, stream);
    case kTile64x128k2: return launch_gemm_cfg<2, 2, 1, 2, true, false, 2>(args, stream);
    case kTile512x128m16: return launch_gemm_cfg<4, 1, 4, 4, true, false, 1, true>(args, stream);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_gemm_tokens(GemmArgs args, int tile_config, hipStream_t stream) {
  if (prepared_bytes(args.m, args.k) >= (size_t(1) << 32)) return hipErrorInvalidValue;  // 32-bit copy offsets
  if ((reinterpret_cast<uintptr_t>(args.b) & 15) != 0 || (size_t)args.k * 256 * 2 >= (size_t(1) << 32))
    return hipErrorInvalidValue;  // 16-byte copies of x; 32-bit offsets inside a tile's token rows
  const int chunks = (args.k + kChunkK - 1) / kChunkK;
  args.ldb = args.k;
  args.alpha = 1.f;
  args.beta = 0.f;
  args.c = nullptr;
  auto pass = [&](GemmArgs a) {
    a.vector_epilogue = (reinterpret_cast<uintptr_t>(a.d) & 15) == 0 && a.m % 8 == 0 &&
                        (reinterpret_cast<uintptr_t>(a.bias) & 15) == 0;
    switch (tile_config) {
      case kTile256x128w: return launch_gemm_cfg<2, 2, 4, 2, true, true>(a, stream);
      case kTile128x128s: return launch_gemm_cfg<2, 2, 2, 2, true, true>(a, stream);
      case kTile512x128w8: return launch_gemm_cfg<4, 2, 4, 2, true, true>(a, stream);
      case kTile256x128w8: return launch_gemm_cfg<4, 2, 2, 2, true, true>(a, stream);
      case kTile128x128w8: return launch_gemm_cfg<2, 4, 2, 1, true, true>(a, stream);
      case kTile64x128: return launch_gemm_cfg<2, 2, 1, 2, true, true>(a, stream);
      case kTile128x128k2: return launch_gemm_cfg<2, 2, 2, 2, true, true, 2>(a, stream);
      case kTile64x128k2: return launch_gemm_cfg<2, 2, 1, 2, true, true, 2>(a, stream);
      case kTile512x128m16: return launch_gemm_cfg<4, 1, 4, 4, true, true, 1, true>(a, stream);
      default: return hipErrorInvalidValue;  // the tiles the automatic choice uses
    }
  };
  if (args.splits <= 1) {
    args.splits = 1;
    args.chunks_per_split = chunks;
    return pass(args);
  }
  if (args.chunks_per_split < 1 || (long)(args.splits - 1) * args.chunks_per_split >= chunks || !args.split_ws)
    return hipErrorInvalidValue;  // an empty split would address past the prepared operand
  // pass 1: raw fp32 partial sums per split, token-major like y; pass 2: ordered sum and bias
  GemmArgs first = args;
  first.d = args.split_ws;
  first.d_f16 = 0;
  first.bias = nullptr;
  if (hipError_t st = pass(first); st != hipSuccess) return st;
  return launch_split_reduce(args.split_ws, args.splits, (size_t)args.m * args.n, nullptr, args.d, 1.f, 0.f, 0, args.d_f16,
                             args.bias, args.bias_f16, args.m, stream);
}

hipError_t launch_gemm(GemmArgs args, int tile_config, hipStream_t stream) {
  if (prepared_bytes(args.m, args.k) >= (size_t(1) << 32)) return hipErrorInvalidValue;  // 32-bit copy offsets
  args.ldb = args.n;
  const bool aligned = (args.n % 8 == 0) && ((reinterpret_cast<uintptr_t>(args.b) & 15) == 0);
  if (!aligned && args.b_pad) {
    const int ldb = (args.n + 7) / 8 * 8;
    const size_t pieces = (size_t)args.k * (ldb / 8);
    hipLaunchKernelGGL(pad_b_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, stream, args.b, args.b_pad,
                       args.k, args.n, ldb);
    if (hipError_t st = hipGetLastError(); st != hipSuccess) return st;
    args.b = args.b_pad;
    args.ldb = ldb;
  }
  const int chunks = (args.k + kChunkK - 1) / kChunkK;
  if (args.splits <= 1) {
    args.splits = 1;
    args.chunks_per_split = chunks;
    return launch_gemm_pass(args, tile_config, stream);
  }
  if (args.chunks_per_split < 1 || (long)(args.splits - 1) * args.chunks_per_split >= chunks || !args.split_ws)
    return hipErrorInvalidValue;  // an empty split would address past the prepared operand
  // pass 1: raw fp32 partial sums per split; pass 2: ordered sum and epilogue
  GemmArgs pass = args;
  pass.alpha = 1.f;
  pass.beta = 0.f;
  pass.c = nullptr;
  pass.d = args.split_ws;
  pass.d_f16 = 0;
  if (hipError_t st = launch_gemm_pass(pass, tile_config, stream); st != hipSuccess) return st;
  return launch_split_reduce(args.split_ws, args.splits, (size_t)args.m * args.n, args.c, args.d, args.alpha, args.beta,
                             args.c_f16, args.d_f16, nullptr, 0, 1, stream);
}

template <int NW, int R, int MODE, int NC>
static hipError_t launch_skinny_mode(const SkinnyArgs& args, hipStream_t stream) {
  const int row_blocks = args.m / kRowBlock;
  hipLaunchKernelGGL((skinny_kernel<NW, R, MODE, NC>), dim3((row_blocks + R - 1) / R, args.splits), dim3(64 * NW), 0,
                     stream, args);
  return hipGetLastError();
}

template <int NW, int R>
static hipError_t launch_skinny_cfg(const SkinnyArgs& args, hipStream_t stream) {
  const uintptr_t address = reinterpret_cast<uintptr_t>(args.b);
  if (args.n > 32) {  // 64-column images, two column fragments: at most two row blocks fit the registers
    constexpr int R64 = R > 2 ? 2 : R;
    if (args.n == 64 && (address & 15) == 0) return launch_skinny_mode<NW, R64, kSkinnyBFull, 64>(args, stream);
    if (args.n % 8 == 0 && (address & 15) == 0) return launch_skinny_mode<NW, R64, kSkinnyB8, 64>(args, stream);
    return launch_skinny_mode<NW, R64, kSkinnyBScalar, 64>(args, stream);
  }
  if (args.n > 16) {  // 32-column images
    constexpr int R32 = R;
    if (args.n == 32 && (address & 15) == 0) return launch_skinny_mode<NW, R32, kSkinnyBFull, 32>(args, stream);
    if (args.n % 8 == 0 && (address & 15) == 0) return launch_skinny_mode<NW, R32, kSkinnyB8, 32>(args, stream);
    return launch_skinny_mode<NW, R32, kSkinnyBScalar, 32>(args, stream);
  }
  if (args.n == 16 && (address & 15) == 0) return launch_skinny_mode<NW, R, kSkinnyBFull, 16>(args, stream);
  if (args.n == 8 && (address & 15) == 0) return launch_skinny_mode<NW, R, kSkinnyB8, 16>(args, stream);
  // one column: B is a token-major x of one token and D is its y (same memory in both layouts)
  if (args.n == 1 && (address & 15) == 0 && (size_t)args.k * 64 * 2 < 0xFFFFFF00u)
    return launch_skinny_mode<NW, R, kSkinnyBTokens, 16>(args, stream);
  if ((args.n == 2 || args.n == 4) && (address & 15) == 0 && (size_t)args.k * args.n * 2 < 0xFFFFFF00u)
    return launch_skinny_mode<NW, R, kSkinnyBRun, 16>(args, stream);
  if (args.n == 4 && (address & 7) == 0) return launch_skinny_mode<NW, R, kSkinnyB4, 16>(args, stream);
  return launch_skinny_mode<NW, R, kSkinnyBScalar, 16>(args, stream);
}

template <int NW, int R>
static hipError_t launch_skinny_tokens_cfg(const SkinnyArgs& args, hipStream_t stream) {
  if (args.n > 32) return launch_skinny_mode<NW, (R > 2 ? 2 : R), kSkinnyBTokens, 64>(args, stream);
  if (args.n > 16) return launch_skinny_mode<NW, R, kSkinnyBTokens, 32>(args, stream);
  return launch_skinny_mode<NW, R, kSkinnyBTokens, 16>(args, stream);
}

// Fills in the K split of a split-K kernel launch: splits <= 1 = one pass straight into d.
static hipError_t skinny_split_setup(SkinnyArgs& args, SkinnyArgs& first_pass) {
  if (args.splits <= 1) {
    args.splits = 1;
    args.chunks_per_split = args.kc_total;
    first_pass = args;
    return hipSuccess;
  }
  if (args.chunks_per_split < 1 || (long)(args.splits - 1) * args.chunks_per_split >= args.kc_total || !args.split_ws)
    return hipErrorInvalidValue;  // an empty split would only add zeros, but it is a planning error
  first_pass = args;  // raw fp32 partial sums per split, laid out like the result
  first_pass.alpha = 1.f;
  first_pass.beta = 0.f;
  first_pass.c = nullptr;
  first_pass.bias = nullptr;
  first_pass.d = args.split_ws;
  first_pass.d_f16 = 0;
  return hipSuccess;
}

hipError_t launch_skinny_tokens(SkinnyArgs args, int rows_per_group, hipStream_t stream) {
  if (args.n < 1 || args.n > kSkinnyMaxN) return hipErrorInvalidValue;
  // 16-byte loads of x; lane offsets of up to 64 token rows must stay below the "outside" offset of the kernel
  if ((reinterpret_cast<uintptr_t>(args.b) & 15) != 0 || (size_t)args.k * 64 * 2 >= 0xFFFFFF00u) return hipErrorInvalidValue;
  SkinnyArgs pass;
  if (hipError_t st = skinny_split_setup(args, pass); st != hipSuccess) return st;
  hipError_t st;
  switch (rows_per_group) {
    case 32: st = launch_skinny_tokens_cfg<16, 1>(pass, stream); break;
    case 64: st = launch_skinny_tokens_cfg<8, 2>(pass, stream); break;
    case 128: st = launch_skinny_tokens_cfg<8, 4>(pass, stream); break;
    default: return hipErrorInvalidValue;
  }
  if (st != hipSuccess || args.splits <= 1) return st;
  return launch_split_reduce(args.split_ws, args.splits, (size_t)args.m * args.n, nullptr, args.d, 1.f, 0.f, 0, args.d_f16,
                             args.bias, args.bias_f16, args.m, stream);
}

template <int NW, int R>
static hipError_t launch_skinny_group_cfg(const SkinnyGroupArgs& g, int blocks, int tokens, hipStream_t stream) {
  if (tokens > 32) hipLaunchKernelGGL((skinny_group_kernel<NW, (R > 2 ? 2 : R), 64>), dim3(blocks), dim3(64 * NW), 0, stream, g);
  else if (tokens > 16) hipLaunchKernelGGL((skinny_group_kernel<NW, R, 32>), dim3(blocks), dim3(64 * NW), 0, stream, g);
  else hipLaunchKernelGGL((skinny_group_kernel<NW, R, 16>), dim3(blocks), dim3(64 * NW), 0, stream, g);
  return hipGetLastError();
}

hipError_t launch_skinny_group(SkinnyGroupArgs g, int rows_per_group, hipStream_t stream) {
  if (g.count < 1 || g.count > kSkinnyMaxGroup) return hipErrorInvalidValue;
  const int tokens = g.problem[0].n;
  if (tokens < 1 || tokens > kSkinnyMaxN) return hipErrorInvalidValue;
  if (rows_per_group != 32 && rows_per_group != 64 && rows_per_group != 128) return hipErrorInvalidValue;
  const int rows = (rows_per_group == 128 && tokens > 32) ? 64 : rows_per_group;  // as launch_skinny_tokens_cfg does
  int blocks = 0;
  for (int i = 0; i < g.count; ++i) {
    SkinnyArgs& p = g.problem[i];
    if (p.n != tokens || p.m <= 0 || p.k <= 0 || !p.prep || !p.b || !p.d) return hipErrorInvalidValue;
    // 16-byte loads of x; lane offsets of up to 64 token rows must stay below the "outside" offset of the kernel
    if ((reinterpret_cast<uintptr_t>(p.b) & 15) != 0 || (size_t)p.k * 64 * 2 >= 0xFFFFFF00u) return hipErrorInvalidValue;
    p.splits = 1;
    p.chunks_per_split = p.kc_total;
    p.split_ws = nullptr;
    g.first_block[i] = blocks;
    blocks += (p.m + rows - 1) / rows;
  }
  g.first_block[g.count] = blocks;
  switch (rows_per_group) {
    case 32: return launch_skinny_group_cfg<16, 1>(g, blocks, tokens, stream);
    case 64: return launch_skinny_group_cfg<8, 2>(g, blocks, tokens, stream);
    default: return launch_skinny_group_cfg<8, 4>(g, blocks, tokens, stream);
  }
}

hipError_t launch_skinny(SkinnyArgs args, int rows_per_group, hipStream_t stream) {
  if (args.n < 1 || args.n > kSkinnyMaxN) return hipErrorInvalidValue;
  SkinnyArgs pass;
  if (hipError_t st = skinny_split_setup(args, pass); st != hipSuccess) return st;
  hipError_t st;
  switch (rows_per_group) {
    case 32: st = launch_skinny_cfg<16, 1>(pass, stream); break;  // sixteen wavefronts split K: small M
    case 64: st = launch_skinny_cfg<8, 2>(pass, stream); break;
    case 128: st = launch_skinny_cfg<8, 4>(pass, stream); break;  // n > 32: 64-row groups
    default: return hipErrorInvalidValue;
  }
  if (st != hipSuccess || args.splits <= 1) return st;
  return launch_split_reduce(args.split_ws, args.splits, (size_t)args.m * args.n, args.c, args.d, args.alpha, args.beta,
                             args.c_f16, args.d_f16, nullptr, 0, 1, stream);
}

}  // namespace onebit
