// Device-side building blocks shared by the gfx950 kernels of the one-bit 2:4 sparse GEMM.
//
// Operand layouts of v_smfmac_f32_32x32x32_f16 as measured on MI355X with one-hot operands
// (lane l of a 64-wide wavefront):
//   A (sparse, 32 rows x 32 dense K, 8 kept values per lane): row = l % 32, ga = l / 32.
//     Kept value s (0..7) of the lane belongs to the aligned group of four dense K
//       kB = 16 * (s / 4) + 8 * ga + 4 * ((s / 2) % 2)      (in the K numbering of the B operand)
//     and its 2-bit position inside that group sits at bits [2s+1 : 2s] of the 16-bit index half that
//     ABID selects (ABID 0 = bits 15:0, ABID 1 = bits 31:16). The encoding of a pair is therefore the
//     reference's metadata nibble  idx0 | idx1 << 2  (_semi_structured_conversions.py:99-108,150).
//   B (dense, 32 K x 32 columns, 16 values per lane): column = l % 32, gb = l / 32, slot t (0..15)
//     holds K index kB = 16 * gb + t.
//   C/D (32 x 32 fp32, 16 values per lane): column = l % 32, row = 8 * (v / 4) + 4 * (l / 32) + v % 4.
//
// This code numbers the dense K of one 32-wide step so that A lane group ga owns the sixteen consecutive
// K values [16 ga, 16 ga + 16) - exactly one metadata element of the reference format - which makes B lane
// group gb own K in [8 gb, 8 gb + 8) and [16 + 8 gb, 16 + 8 gb + 8).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace onebit {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half16_t __attribute__((ext_vector_type(16)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4v_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x8_t __attribute__((ext_vector_type(8)));
typedef __fp16 fp16x4_t __attribute__((__vector_size__(8)));

// ---- prepared A operand ---------------------------------------------------------------------------
// The weight operand is consumed from a "prepared" buffer written by prepare_kernel: one 1536-byte block
// per (32-row block rb, 256-wide K chunk kc), blocks ordered rb-major. Inside a block, lane l of the
// consuming wavefront owns
//   bytes [16 l, 16 l + 16):        eight int16 metadata elements, one per 32-wide K step s of the chunk:
//                                    logical meta (row 32 rb + l % 32, column 16 kc + 2 s + l / 32),
//   bytes [1024 + 8 l, 1024 + 8 l + 8): two 32-bit sign words (steps 0-3, steps 4-7). In a sign word, the
//                                    pair p (kept values 2p, 2p+1) of step s is stored at bit 15 - j
//                                    (value 2p) and bit 31 - j (value 2p+1) with j = 4 (s % 4) + p, and a
//                                    set bit means -1. Shifting the word left by j therefore puts both
//                                    signs on the fp16 sign positions of one packed register.
constexpr int kRowBlock = 32;
constexpr int kChunkK = 256;
constexpr int kStepsPerChunk = 8;
constexpr int kBlockBytes = 1536;
constexpr int kSignOffset = 1024;

__host__ __device__ inline size_t prepared_bytes(int m, int k) {
  size_t rb = (size_t)(m + kRowBlock - 1) / kRowBlock;
  size_t kc = (size_t)(k + kChunkK - 1) / kChunkK;
  return rb * kc * kBlockBytes;
}

struct AChunk {      // per lane, per row block: one K chunk of the prepared operand
  u32x4_t meta;      // meta[q]: steps 2q (low half, ABID 0) and 2q+1 (high half, ABID 1)
  u32x2_t sign;
};

__device__ __forceinline__ AChunk load_a_chunk(const uint8_t* __restrict__ block, int lane) {
  AChunk r;
  r.meta = *reinterpret_cast<const u32x4_t*>(block + lane * 16);
  r.sign = *reinterpret_cast<const u32x2_t*>(block + kSignOffset + lane * 8);
  return r;
}

__device__ __forceinline__ AChunk load_a_chunk_lds(const char* block, int lane) {
  AChunk r;
  r.meta = *reinterpret_cast<const u32x4_t*>(block + lane * 16);
  r.sign = *reinterpret_cast<const u32x2_t*>(block + kSignOffset + lane * 8);
  return r;
}

// fp16 1.0 in both halves, held in a vector register: v_and_or_b32 can then take the sign mask as its only
// literal operand (two literals in one instruction are not encodable, and cost a third instruction).
__device__ __forceinline__ uint32_t packed_one_in_vgpr() {
  uint32_t one = 0x3C003C00u;
  asm volatile("" : "+v"(one));
  return one;
}

// Expand the eight +-1 values of K step `STEP` (0..7, compile time) into four packed fp16 registers:
// two instructions per register (shift, and-or).
template <int STEP>
__device__ __forceinline__ half8_t expand_signs(const AChunk& a, uint32_t packed_one) {
  const uint32_t w = STEP < 4 ? a.sign.x : a.sign.y;
  u32x4_t v;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const int j = 4 * (STEP % 4) + p;
    v[p] = ((w << j) & 0x80008000u) | packed_one;  // fp16 1.0 with the stored sign
  }
  return __builtin_bit_cast(half8_t, v);
}

// One SMFMAC of K step STEP. Written as inline assembly with the accumulator tied to an accumulation-register
// tuple ("+a") and the operands to vector registers: with 256 accumulator registers in flight the compiler's own
// allocation mixes the two register files and then copies whole accumulator tiles between them behind the SMFMAC
// that produced them, which serialises the matrix pipe. Consecutive SMFMACs never share an accumulator, so no
// wait states are needed between them.
template <int STEP, bool PINNED = true>
__device__ __forceinline__ float16_t smfmac_step(const AChunk& a, half8_t av, half16_t bv, float16_t acc) {
  const int idx = (int)a.meta[STEP / 2];
  // Kernels whose consecutive SMFMACs update the same accumulator use the builtin, so that the compiler inserts
  // the wait states that dependency needs.
  if (!PINNED) return __builtin_amdgcn_smfmac_f32_32x32x32_f16(av, bv, acc, idx, 0, STEP % 2);
  if (STEP % 2 == 0) asm("v_smfmac_f32_32x32x32_f16 %0, %1, %2, %3" : "+a"(acc) : "v"(av), "v"(bv), "v"(idx));
  else asm("v_smfmac_f32_32x32x32_f16 %0, %1, %2, %3 abid:1" : "+a"(acc) : "v"(av), "v"(bv), "v"(idx));
  return acc;
}

// Wait states between the last SMFMAC and the first read of its result by a vector instruction.
__device__ __forceinline__ void smfmac_drain() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

// ---- LDS transpose read ---------------------------------------------------------------------------
// ds_read_b64_tr_b16 (measured): result element v of lane l is element l % 4 of the 8-byte chunk whose
// address was supplied by lane 16 (l / 16) + 4 v + (l % 16) / 4. With B rows (K) stored N-contiguous in
// LDS, lane 4 v + c of a 16-lane group points at row v, columns 4c..4c+3, and lane i receives the four
// K-consecutive values of column i.
__device__ __forceinline__ u32x2_t lds_read_tr16(const void* lds_ptr) {
  fp16x4_t r = __builtin_amdgcn_ds_read_tr16_b64_v4f16(
      (fp16x4_t __attribute__((address_space(3)))*)(lds_ptr));
  return __builtin_bit_cast(u32x2_t, r);
}

// ---- asynchronous global -> LDS copy --------------------------------------------------------------
// global_load_lds_dwordx4: each lane fetches 16 bytes from its own global address; the wavefront's 1 KiB
// lands at LDS offset M0 + 16 * lane. Issued through inline assembly so that the compiler does not
// serialise later LDS reads behind it; completion is tracked by hand with s_waitcnt vmcnt.
__device__ __forceinline__ void lds_dma16(const void* gptr, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_wave_base), "v"(gptr) : "memory");
}

// Same copy with the address split into a wave-uniform 64-bit base (scalar registers) and a per-lane 32-bit
// byte offset: one vector register per copy instead of two, and the base advances with scalar arithmetic.
__device__ __forceinline__ void lds_dma16_base(const void* base, uint32_t lane_offset, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_wave_base), "v"(lane_offset), "s"(base)
               : "memory");
}

// Raw buffer loads: address = descriptor base (wave-uniform) + vector offset + scalar offset, so a loop that walks
// memory needs scalar additions only and one vector register of lane offsets. The descriptor covers `bytes` bytes
// (untyped 32-bit data format); the scalar offset takes no part in its range check, so callers keep every access
// inside [base, base + bytes) themselves.
typedef __amdgpu_buffer_rsrc_t buffer_t;
__device__ __forceinline__ buffer_t make_buffer(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, bytes, 0x00020000);
}
__device__ __forceinline__ u32x4_t buffer_load16(buffer_t buffer, uint32_t lane_offset, uint32_t uniform_offset) {
  return __builtin_amdgcn_raw_buffer_load_b128(buffer, lane_offset, uniform_offset, 0);
}
__device__ __forceinline__ u32x2_t buffer_load8(buffer_t buffer, uint32_t lane_offset, uint32_t uniform_offset) {
  return __builtin_amdgcn_raw_buffer_load_b64(buffer, lane_offset, uniform_offset, 0);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter on gfx9");
  // simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14]; other counters left open.
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0xF << 8) | ((N >> 4) << 14));
}

// Same, and additionally waits for every outstanding LDS operation of the wavefront (lgkmcnt = 0).
template <int N>
__device__ __forceinline__ void wait_vmcnt_lgkm0() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter on gfx9");
  __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0x0 << 8) | ((N >> 4) << 14));
}

__device__ __forceinline__ uint32_t lds_offset_of(const void* p) {
  return (uint32_t)(size_t)(const __attribute__((address_space(3))) char*)p;
}

// Reference metadata layout: int16 offset of logical element (r, c) of an (m x ncols) metadata matrix.
// Closed form of onebit_sparse_mul/_semi_structured_conversions.py:21-48 (row permutation inside 64 rows,
// 2x2 swizzle, 2-interleaved column-major): each (64 rows x 2 columns) block is 128 consecutive elements.
__host__ __device__ inline int64_t meta_offset_reference(int64_t r, int64_t c, int64_t m) {
  const int64_t b0 = r & 1, b1 = (r >> 1) & 1, b2 = (r >> 2) & 1, b345 = (r >> 3) & 7;
  return (c >> 1) * 2 * m + (r >> 6) * 128 + ((b1 << 6) | (b345 << 3) | (b0 << 2) | ((c & 1) << 1) | b2);
}

// CUTLASS reorder_meta layout (row permutation inside 32 rows, same swizzle and interleave).
__host__ __device__ inline int64_t meta_offset_cutlass(int64_t r, int64_t c, int64_t m) {
  int64_t dr = (r / 32) * 32 + (r % 8) * 4 + (r % 32) / 8;
  int64_t dc = c;
  const int64_t tr = (dr % 2 == 0) && (dc % 2 == 1), bl = (dr % 2 == 1) && (dc % 2 == 0);
  dr += tr - bl;
  dc -= tr - bl;
  return (dc / 2) * m * 2 + dr * 2 + dc % 2;
}

}  // namespace onebit
