/*
 * TEST INFRASTRUCTURE — CPU oracle for the one-bit 2:4 sparse GEMM path.
 *
 * This file restates, in plain C, the algorithm of the reference (Adeshen/OneBitSparseMul) for
 *   D = alpha * A * B + beta * C,  A = +-1 values, 2:4 sparse, one bit per kept value + 2-bit positions.
 * It is a checker only: nothing in the shipped library links, loads or calls it. Only the test-suite,
 * the smoke check and the benchmark's cpu_baseline leg may use it.
 *
 * Every function names the reference lines it follows (paths relative to the reference tree).
 * Pinning of each function (what, besides this file, fixes its results) is listed in oracle/README.md.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

#define OB_LAYOUT_REFERENCE 0 /* onebit_sparse_mul/_semi_structured_conversions.py:21-48 */
#define OB_LAYOUT_CUTLASS   1 /* CUTLASS reorder_meta as restated by torch/sparse/_semi_structured_conversions.py */
#define OB_LAYOUT_LOGICAL   2 /* plain row-major (m, k/16): no reordering */

/* ------------------------------------------------------------------------------------------------
 * fp16 <-> fp32, IEEE binary16, round-to-nearest-even (cutlass::half_t / torch.float16 semantics).
 * ---------------------------------------------------------------------------------------------- */
float ob_half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; e++; } while (!(man & 0x400u));
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t ob_float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t absx = x & 0x7fffffffu;
  if (absx >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((absx > 0x7f800000u) ? (0x200u | ((absx >> 13) & 0x3ffu)) : 0u));
  }
  if (absx >= 0x477ff000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (absx < 0x33000001u) { /* < 2^-25 (or exactly 2^-25, which ties to even = 0) */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(absx >> 23) - 127;
  uint32_t man = (absx & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift;
  uint32_t base;
  if (e < -14) { /* subnormal half: value = man * 2^(e-23); unit = 2^-24 */
    shift = -e - 1; /* man >> shift gives units of 2^-24 : shift = 23 - (e + 24) */
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    man &= 0x7fffffu;
  }
  uint32_t q = man >> shift;
  uint32_t rem = man & ((1u << shift) - 1u);
  uint32_t halfway = 1u << (shift - 1);
  uint32_t h = base + q;
  if (rem > halfway || (rem == halfway && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}

/* ------------------------------------------------------------------------------------------------
 * F1 — one-bit value format.
 * ---------------------------------------------------------------------------------------------- */

/* binary_quant: value > 0 -> 1 else 0 (zero and negatives -> 0).  onebit_sparse_mul/__init__.py:22-23 */
void ob_binary_quant(const float *x, int64_t n, uint8_t *bits) {
  for (int64_t i = 0; i < n; i++) bits[i] = x[i] > 0.0f ? 1 : 0;
}

/* pack_binary: 2-D (rows, cols) of 0/1 -> (rows, cols/8) bytes, element 8c+i of a row goes to bit i of
 * byte c.  onebit_sparse_mul/__init__.py:25-34 (tensor[:, i::8] << i). */
int ob_pack_binary(const uint8_t *bits, int rows, int cols, uint8_t *packed) {
  if (cols % 8) return -1;
  int pc = cols / 8;
  for (int r = 0; r < rows; r++)
    for (int c = 0; c < pc; c++) {
      uint8_t b = 0;
      for (int i = 0; i < 8; i++) b |= (uint8_t)((bits[(int64_t)r * cols + 8 * c + i] & 1u) << i);
      packed[(int64_t)r * pc + c] = b;
    }
  return 0;
}

/* unpack_binary: inverse of pack_binary.  onebit_sparse_mul/__init__.py:36-45 */
void ob_unpack_binary(const uint8_t *packed, int rows, int pcols, uint8_t *bits) {
  int cols = pcols * 8;
  for (int r = 0; r < rows; r++)
    for (int j = 0; j < cols; j++)
      bits[(int64_t)r * cols + j] = (packed[(int64_t)r * pcols + j / 8] >> (j % 8)) & 1u;
}

/* ------------------------------------------------------------------------------------------------
 * F2 — metadata format.
 * ---------------------------------------------------------------------------------------------- */

/* Offset (in int16 elements) of logical meta element (r, c) inside the reordered buffer.
 * Reference layout: _semi_structured_conversions.py:21-48, statement by statement, for int16 metadata
 * (group_x = 64, group_y = 32). */
int64_t ob_meta_offset_reference(int64_t r, int64_t c, int64_t m) {
  const int64_t group_x = 64, group_y = 32;
  int64_t dr = r / group_x * group_x + (r % 2) * 2 + (r % 8) / 4 + ((r % group_y) % 4) / 2 * 32 +
               ((r % group_x) / 8) * 4;                                     /* :29-35 */
  int64_t dc = c;
  int64_t topright = (dr % 2 == 0) && (dc % 2 == 1);                         /* :37 */
  int64_t bottomleft = (dr % 2 == 1) && (dc % 2 == 0);                       /* :38 */
  dr += topright - bottomleft;                                              /* :39 */
  dc -= topright - bottomleft;                                              /* :40 */
  const int64_t interleave = 2;                                             /* :45 */
  return (dc / interleave) * m * interleave + dr * interleave + dc % interleave; /* :46-48 */
}

/* CUTLASS reorder_meta variant (what tests/unit/warp_test.h:377-379 calls); the source is absent from the
 * reference tree (un-vendored submodule NVIDIA/cutlass, version not pinned); restated from the published
 * algorithm: row permutation within 32 rows, then the same 2x2 swizzle and 2-interleaved column-major. */
int64_t ob_meta_offset_cutlass(int64_t r, int64_t c, int64_t m) {
  int64_t dr = r / 32 * 32 + (r % 8) * 4 + (r % 32) / 8;
  int64_t dc = c;
  int64_t topright = (dr % 2 == 0) && (dc % 2 == 1);
  int64_t bottomleft = (dr % 2 == 1) && (dc % 2 == 0);
  dr += topright - bottomleft;
  dc -= topright - bottomleft;
  return (dc / 2) * m * 2 + dr * 2 + dc % 2;
}

int64_t ob_meta_offset(int64_t r, int64_t c, int64_t m, int64_t ncols, int layout) {
  if (layout == OB_LAYOUT_REFERENCE) return ob_meta_offset_reference(r, c, m);
  if (layout == OB_LAYOUT_CUTLASS) return ob_meta_offset_cutlass(r, c, m);
  return r * ncols + c;
}

/* Nibble for one group of four non-zero flags.  _semi_structured_conversions.py:126-150
 * (expr0..2, bit0..3, idxs0 | idxs1 << 2); also returns the two selected positions. */
static inline int ob_encode_group(int m0, int m1, int m2, int m3, int *i0, int *i1) {
  (void)m2;
  int expr0 = m0 && m1;
  int expr1 = !m0 && m1;
  int expr2 = !m0 && !m1;
  int bit0 = expr1, bit1 = expr2;
  int bit2 = expr0 || expr2 || m3;
  int bit3 = expr1 || !m1;
  *i0 = bit0 | (bit1 << 1);
  *i1 = bit2 | (bit3 << 1);
  return *i0 | (*i1 << 2);
}

/* sparse_semi_structured_from_dense_cutlass for the 16-bit-metadata, ksparse = 4 path (dense dtype half /
 * bfloat16 / int32 in the reference: _semi_structured_conversions.py:54-179; the torch.float path with
 * ksparse = 2 is not used by the one-bit pipeline and is not restated).
 * dense: (m, k) row-major; sparse: (m, k/2); meta_reordered: (m, k/16) in `layout`.
 * Returns 0, or -1 when the shape is rejected by the reference's own checks (:79-87). Note that the
 * reference layout is only a bijection when m % 64 == 0 and k % 32 == 0; -2 is returned otherwise. */
int ob_sparse_from_dense(const float *dense, int m, int k, float *sparse, int16_t *meta_reordered, int layout) {
  if (m % 32 != 0 || k % 16 != 0) return -1;
  if (layout == OB_LAYOUT_REFERENCE && (m % 64 != 0 || k % 32 != 0)) return -2;
  if (layout == OB_LAYOUT_CUTLASS && (k % 32 != 0)) return -2;
  int ncols = k / 16;
  for (int r = 0; r < m; r++) {
    for (int c = 0; c < ncols; c++) {
      uint16_t word = 0;
      for (int g = 0; g < 4; g++) {
        const float *q = dense + (int64_t)r * k + 16 * c + 4 * g;
        int i0, i1;
        int nib = ob_encode_group(q[0] != 0.0f, q[1] != 0.0f, q[2] != 0.0f, q[3] != 0.0f, &i0, &i1);
        sparse[(int64_t)r * (k / 2) + 8 * c + 2 * g + 0] = q[i0]; /* :143-146 gather */
        sparse[(int64_t)r * (k / 2) + 8 * c + 2 * g + 1] = q[i1];
        word |= (uint16_t)(nib << (4 * g));                       /* :153-159 */
      }
      meta_reordered[ob_meta_offset(r, c, m, ncols, layout)] = (int16_t)word; /* :173-177 scatter */
    }
  }
  return 0;
}

/* sparse_semi_structured_to_dense_cutlass (ksparse = 4, int16 meta).  _semi_structured_conversions.py:186-283
 * sparse: (m, ks) with ks = k/2; dense: (m, 2*ks). */
int ob_sparse_to_dense(const float *sparse, const int16_t *meta_reordered, int m, int ks, float *dense, int layout) {
  int k = 2 * ks;
  if (k % 16) return -1;
  int ncols = k / 16;
  memset(dense, 0, sizeof(float) * (size_t)m * k);                    /* :274 */
  for (int r = 0; r < m; r++)
    for (int c = 0; c < ncols; c++) {
      uint16_t word = (uint16_t)meta_reordered[ob_meta_offset(r, c, m, ncols, layout)]; /* :226-229 gather */
      for (int j = 0; j < 8; j++) {                                   /* :243-251: eight 2-bit fields */
        int idx = (word >> (2 * j)) & 3;
        /* :266-277: value j of this meta element lands at 4*(group) + idx, group = (8c + j) / 2 */
        dense[(int64_t)r * k + 4 * ((8 * c + j) / 2) + idx] = sparse[(int64_t)r * ks + 8 * c + j];
      }
    }
  return 0;
}

/* mask_creator: keep the 2 largest |w| of every group of 4 (flattened order).
 * _semi_structured_conversions.py:286-314. The reference prunes the first two entries of an ascending
 * argsort whose order among equal keys is unspecified; this restatement uses the stable order (lower
 * index pruned first), which reproduces the only tie case the reference documents (all-ones weights ->
 * mask 0,0,1,1: tests/python/test_sparse.py:23-24) and is what PyTorch's CPU argsort returns for all 256 rank
 * patterns of four magnitudes (tests/test_oracle_format.py checks that against PyTorch's own routine). */
void ob_mask_creator(const float *w, int64_t numel, float *mask) {
  for (int64_t g = 0; g < numel / 4; g++) {
    int order[4] = {0, 1, 2, 3};
    float a[4];
    for (int i = 0; i < 4; i++) a[i] = fabsf(w[4 * g + i]);
    for (int i = 1; i < 4; i++) { /* stable insertion sort, ascending */
      int o = order[i], j = i - 1;
      while (j >= 0 && a[order[j]] > a[o]) { order[j + 1] = order[j]; j--; }
      order[j + 1] = o;
    }
    for (int i = 0; i < 4; i++) mask[4 * g + i] = 1.0f;
    mask[4 * g + order[0]] = 0.0f;
    mask[4 * g + order[1]] = 0.0f;
  }
}

/* ------------------------------------------------------------------------------------------------
 * The C entry point's operands -> dense A.
 *   a: one bit per kept value, column-major (m x k/2), packed stride m, LSB first
 *      (csrc/kernel_lib.cu:28,37; csrc/kernel.h:13-14; produced by __init__.py:139-143: quantise, transpose, pack)
 *   e: int16 (m x k/16) metadata in `layout` (csrc/kernel_lib.cu:41)
 *   bit 1 -> +1, bit 0 -> -1 (csrc/warp.h:41-50; tests/kernel_test.cu:81-117)
 * dense: int8 (m, k) row-major with values in {-1, 0, +1}.
 * ---------------------------------------------------------------------------------------------- */
int ob_decompress_operands(const uint8_t *a, const int16_t *e, int m, int k, int layout, int8_t *dense) {
  if (m % 8 || k % 16) return -1;
  int ncols = k / 16;
  int64_t ks = k / 2;
  memset(dense, 0, (size_t)m * k);
  for (int64_t r = 0; r < m; r++)
    for (int64_t c = 0; c < ncols; c++) {
      uint16_t word = (uint16_t)e[ob_meta_offset(r, c, m, ncols, layout)];
      for (int j = 0; j < 8; j++) {
        int idx = (word >> (2 * j)) & 3;
        int64_t col = 8 * c + j;            /* compressed column */
        int64_t bitpos = r + col * m;       /* column-major, stride m */
        int bit = (a[bitpos >> 3] >> (bitpos & 7)) & 1;
        (void)ks;
        dense[r * k + 4 * (col / 2) + idx] = bit ? 1 : -1;
      }
    }
  return 0;
}

/* ------------------------------------------------------------------------------------------------
 * Host GEMM + epilogue.  tests/kernel_test.cu:441-456 (cutlass::reference::host::Gemm with
 * ElementCompute = ElementAccumulator = float: one fp32 accumulator per output, k ascending,
 * acc = a*b + acc; then D = alpha*acc + beta*C in fp32, converted to the output type with RNE),
 * epilogue definition csrc/kernel.h:27-31.
 * dtype codes: 0 = fp32, 1 = fp16.  acc_mode: 0 = fp32 sequential, 1 = fp64 sequential (tight oracle).
 * C is not read when beta == 0.
 * ---------------------------------------------------------------------------------------------- */
int ob_host_gemm(const int8_t *a_dense, const uint16_t *b_half, const void *c, void *d, int m, int n, int k,
                 float alpha, float beta, int c_dtype, int d_dtype, int acc_mode) {
  float *bf = (float *)malloc(sizeof(float) * (size_t)k * n);
  if (!bf) return -1;
  for (int64_t i = 0; i < (int64_t)k * n; i++) bf[i] = ob_half_to_float(b_half[i]);
  float *accf = (float *)malloc(sizeof(float) * (size_t)n);
  double *accd = (double *)malloc(sizeof(double) * (size_t)n);
  for (int64_t i = 0; i < m; i++) {
    if (acc_mode == 0) {
      for (int j = 0; j < n; j++) accf[j] = 0.0f;
      for (int64_t t = 0; t < k; t++) {
        int8_t av = a_dense[i * k + t];
        if (av == 0) continue; /* 0*b + acc == acc exactly for finite b */
        const float *brow = bf + t * n;
        if (av > 0) for (int j = 0; j < n; j++) accf[j] = brow[j] + accf[j];
        else        for (int j = 0; j < n; j++) accf[j] = -brow[j] + accf[j];
      }
    } else {
      for (int j = 0; j < n; j++) accd[j] = 0.0;
      for (int64_t t = 0; t < k; t++) {
        int8_t av = a_dense[i * k + t];
        if (av == 0) continue;
        const float *brow = bf + t * n;
        if (av > 0) for (int j = 0; j < n; j++) accd[j] += (double)brow[j];
        else        for (int j = 0; j < n; j++) accd[j] -= (double)brow[j];
      }
    }
    for (int j = 0; j < n; j++) {
      float out;
      if (acc_mode == 0) {
        out = alpha * accf[j];
        if (beta != 0.0f) {
          float cv = c_dtype == 0 ? ((const float *)c)[i * n + j] : ob_half_to_float(((const uint16_t *)c)[i * n + j]);
          out = out + beta * cv;
        }
      } else {
        double o = (double)alpha * accd[j];
        if (beta != 0.0f) {
          float cv = c_dtype == 0 ? ((const float *)c)[i * n + j] : ob_half_to_float(((const uint16_t *)c)[i * n + j]);
          o += (double)beta * (double)cv;
        }
        out = (float)o;
      }
      if (d_dtype == 0) ((float *)d)[i * n + j] = out;
      else ((uint16_t *)d)[i * n + j] = ob_float_to_half(out);
    }
  }
  free(bf); free(accf); free(accd);
  return 0;
}

/* Whole path as the C entry point defines it: operands in the device formats -> D. */
int ob_reference_matmul(const uint8_t *a, const uint16_t *b, const void *c, void *d, const int16_t *e, int m, int n,
                        int k, float alpha, float beta, int c_dtype, int d_dtype, int layout, int acc_mode) {
  int8_t *dense = (int8_t *)malloc((size_t)m * k);
  if (!dense) return -1;
  int rc = ob_decompress_operands(a, e, m, k, layout, dense);
  if (rc == 0) rc = ob_host_gemm(dense, b, c, d, m, n, k, alpha, beta, c_dtype, d_dtype, acc_mode);
  free(dense);
  return rc;
}
