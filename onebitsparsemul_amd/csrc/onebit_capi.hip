// C ABI of libonebitmul (declared in include/onebit_sparse_tensor.h): argument validation, per-device
// workspaces, kernel selection. Host code only; the kernels live in onebit_kernels.hip.
// Counterpart of the reference's host launcher csrc/kernel_lib.cu:23-97.
#include "onebit_sparse_tuning.h"
#include "onebit_device.h"
#include "onebit_launch.h"

#include <algorithm>
#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace {

thread_local std::string g_last_error;
// Tuning / test hooks: per calling thread, so that a test or a tuning run never changes what other threads of the
// process launch.
thread_local int g_tile_config = -1;
thread_local int g_skinny_enabled = 1;
thread_local int g_skinny_rows = -1;
thread_local int g_split_k = -1;
thread_local int g_pad_b = 1;
std::atomic<int> g_weight_cache_entries{0};

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

#define ONEBIT_HIP(expr)                                                                         \
  do {                                                                                           \
    hipError_t st_ = (expr);                                                                     \
    if (st_ != hipSuccess)                                                                       \
      return fail(ONEBIT_ERR_HIP, "HIP error '%s' from %s", hipGetErrorString(st_), #expr);      \
  } while (0)

constexpr int kMaxDevices = 64;

// Workspace of onebit_sparse_matmul_prepared_static: device memory that exists from the moment the code object is
// loaded, so that entry point never allocates. Every GPU the library runs on holds its own copy at its own address
// until the process ends. In host code the name is only a handle for hipGetSymbolAddress; kernels and copies use the
// per-device address kept in DeviceState::static_scratch.
constexpr size_t kStaticScratchBytes = ONEBIT_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];

// Library-owned device memory. Grow-only, one buffer per device and stream (calls on one stream are ordered, calls
// on different streams must not share a buffer), freed at process exit by the runtime.
struct Buffer {
  void* ptr = nullptr;
  size_t bytes = 0;
};
struct DeviceState {
  // recursive: the one-call entry points keep it while they launch, and the launch takes it again for its own buffers
  std::recursive_mutex mu;
  // the reordered operand of the one-call entry points (when the weight cache is off)
  std::map<hipStream_t, Buffer> prep;
  // fp32 partial sums of the K-split passes: one buffer per stream, so that calls on different streams do not
  // share one (calls on the same stream are ordered)
  std::map<hipStream_t, Buffer> split_ws;
  // B with rows padded to a multiple of 8 columns (operands the asynchronous copies cannot read in place), per stream
  std::map<hipStream_t, Buffer> b_pad;
  // opt-in cache of prepared operands of the one-call entry points, keyed by the caller's weight pointers
  struct CachedWeight {
    const void* a;
    const void* e;
    int m, k, layout;
    void* prep;
    hipStream_t stream;  // the stream its reorder kernel was enqueued on
    hipEvent_t ready;    // recorded after that kernel
    unsigned long last_use;
  };
  std::vector<CachedWeight> weight_cache;
  unsigned long use_counter = 0;
  // compute units of the device (0 until first asked): the launch plans scale with it
  std::atomic<int> compute_units{0};
  // this device's address of g_static_scratch (null until the first non-allocating call on the device)
  unsigned char* static_scratch = nullptr;
};
DeviceState g_dev[kMaxDevices];

// Grows a library-owned buffer. Growing frees the old memory after a device synchronization: a HIP graph captured
// earlier on this stream still holds the old address and must be captured again after a larger call. Inside a stream
// capture neither the synchronization nor the allocation is possible, so a call that would have to grow there is
// refused instead of invalidating the capture.
int grow(void** ptr, size_t* have, size_t need, hipStream_t stream) {
  if (need <= *have) return ONEBIT_OK;
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  ONEBIT_HIP(hipStreamIsCapturing(stream, &capture));
  if (capture != hipStreamCaptureStatusNone)
    return fail(ONEBIT_ERR_ARGUMENT,
                "a library-owned buffer would have to grow to %zu bytes while the stream is being captured: run the "
                "call once outside the capture first, or use the non-allocating entry point", need);
  if (*ptr) {
    // earlier work on any stream may still read the old buffer
    ONEBIT_HIP(hipDeviceSynchronize());
    ONEBIT_HIP(hipFree(*ptr));
    *ptr = nullptr;
    *have = 0;
  }
  const size_t bytes = (need + 4095) & ~size_t(4095);
  ONEBIT_HIP(hipMalloc(ptr, bytes));
  *have = bytes;
  return ONEBIT_OK;
}

// Compute units of the current device, asked once per device. A failure leaves the MI355X figure the plans were
// measured on.
int current_compute_units() {
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return 256;
  int cus = g_dev[device].compute_units.load(std::memory_order_relaxed);
  if (cus > 0) return cus;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) cus = 256;
  g_dev[device].compute_units.store(cus, std::memory_order_relaxed);
  return cus;
}

int check_shape(int m, int n, int k) {
  if (m <= 0 || n <= 0 || k <= 0) return fail(ONEBIT_ERR_ARGUMENT, "m, n, k must be positive (got %d, %d, %d)", m, n, k);
  if (m % 64 != 0) return fail(ONEBIT_ERR_ARGUMENT, "m = %d must be a multiple of 64 (metadata layout)", m);
  if (k % 32 != 0) return fail(ONEBIT_ERR_ARGUMENT, "k = %d must be a multiple of 32 (metadata layout)", k);
  return ONEBIT_OK;
}

int check_dtype(int c_dtype, int d_dtype) {
  if ((c_dtype != ONEBIT_DTYPE_F32 && c_dtype != ONEBIT_DTYPE_F16) ||
      (d_dtype != ONEBIT_DTYPE_F32 && d_dtype != ONEBIT_DTYPE_F16))
    return fail(ONEBIT_ERR_ARGUMENT, "dtype codes must be 0 (fp32) or 1 (fp16), got c=%d d=%d", c_dtype, d_dtype);
  return ONEBIT_OK;
}

// Tile and number of K splits of the main kernel. The time is rounds of resident workgroups times one workgroup's K
// loop; the choice among the tiles, and among splits of K that fill idle compute units at the price of a second launch
// and of writing and re-reading fp32 partial sums, comes from a cost model fitted to measurements on MI355X
// (microseconds):
//   K loop of one workgroup per 256-wide chunk with every slot of the GPU taken: 512 x 128: 3.8, 256 x 128 on eight
//   wavefronts: 2.3, on four (two workgroups per CU): 3.9, 128 x 128 on four (two per CU): 2.4, as two K groups:
//   1.2, as 64 x 32 wavefronts: 1.5, 64 x 128: 1.0, as two K groups: 0.88;
//   a round that fills only a fraction f of the slots is shorter: with one workgroup per CU 0.85 of a full round
//   below f = 0.9; with two per CU 0.6 up to f = 0.5 (every workgroup has its CU to itself) and a full round above
//   (some CUs hold two again); the two-K-group tiles pay 1.5 and 1.0 per round for exchanging the groups' sums;
//   4 for launch, prologue and epilogue; a split adds 5 and moves (S + 1) partial results at about 5 TB/s.
// Examples the model was checked against (measured, us): 4096 x 3072 x 4096: 512 x 128 57.0, 256 x 128 68.3;
// 4096 x 1536 x 4096: 256 x 128 35.0, 128 x 128 38.9; 4096 x 384 x 11008: 64 x 128 40.2, 256 x 128 with four splits
// 32.5; 11008 x 768 x 4096: 512 x 128 51.2, 256 x 128 65.5; 4096 x 128 x 4096: 64 x 128 with four splits 13.9,
// unsplit 17.3.
struct GemmPlan {
  int tile;
  int splits;
};

struct TileCost {
  int tile, bm, bn;
  int slots;        // workgroups resident at once on the 256 compute units the timings were taken on
  double chunk_us;  // K loop of one workgroup per 256-wide chunk with every slot taken
  double round_us;  // per round on top of the K loop
  bool may_split;
};
const TileCost kTileCosts[] = {
    {onebit::kTile512x128w8, 512, 128, 256, 3.8, 0.0, false}, {onebit::kTile256x128w8, 256, 128, 256, 2.3, 0.0, true},
    {onebit::kTile256x128w, 256, 128, 512, 3.9, 0.0, false},  {onebit::kTile128x128s, 128, 128, 512, 2.4, 0.0, false},
    {onebit::kTile128x128k2, 128, 128, 256, 1.2, 1.5, true}, {onebit::kTile128x128w8, 128, 128, 256, 1.5, 0.0, true},
    {onebit::kTile64x128, 64, 128, 256, 1.0, 0.0, true},      {onebit::kTile64x128k2, 64, 128, 256, 0.88, 1.0, true},
};

// compute_units: of the device the call runs on. The per-chunk times are per workgroup and do not depend on it; the
// number of resident workgroups scales with it (a partitioned or smaller GPU runs more rounds of the same tiles).
double model_us(const TileCost& t, int m, int n, int chunks, int s, int compute_units) {
  const long tiles = (long)((m + t.bm - 1) / t.bm) * ((n + t.bn - 1) / t.bn) * s;
  const int per_split = (chunks + s - 1) / s;
  const long slots = std::max(1L, (long)t.slots * compute_units / 256);
  const long full_rounds = tiles / slots;
  const double f = (double)(tiles % slots) / slots;
  double rounds = (double)full_rounds;
  if (f > 0.0) rounds += t.slots == 256 ? (f > 0.9 ? 1.0 : 0.85) : (f <= 0.5 ? 0.6 : 1.0);
  double us = 4.0 + (t.chunk_us * per_split + t.round_us) * rounds;
  if (s > 1) us += 5.0 + (s + 1) * 4.0 * m * n / 5.0e6;
  return us;
}

GemmPlan plan_gemm(int m, int n, int k, int compute_units) {
  const int chunks = (k + onebit::kChunkK - 1) / onebit::kChunkK;
  const int forced_tile = g_tile_config;
  const int forced_splits = g_split_k;
  if (forced_tile >= 0) {
    // a forced tile of the table may still be split by the model
    int splits = forced_splits >= 1 ? forced_splits : 1;
    if (forced_splits < 1)
      for (const TileCost& t : kTileCosts)
        if (t.tile == forced_tile && t.may_split) {
          double best_us = 1e30;
          for (int s : {1, 2, 3, 4, 6, 8, 12, 16}) {
            if (s > chunks) break;
            const double us = model_us(t, m, n, chunks, s, compute_units);
            if (us < best_us) best_us = us, splits = s;
          }
        }
    if (splits > chunks) splits = chunks;
    return GemmPlan{forced_tile, splits};
  }
  const int fixed_splits = forced_splits >= 1 ? (forced_splits > chunks ? chunks : forced_splits) : 0;
  GemmPlan best{onebit::kTile128x128s, fixed_splits ? fixed_splits : 1};
  double best_us = 1e30;
  auto consider = [&](const TileCost& t, int s) {
    const double us = model_us(t, m, n, chunks, s, compute_units);
    if (us < best_us) {
      best_us = us;
      best = GemmPlan{t.tile, s};
    }
  };
  for (const TileCost& t : kTileCosts) {
    if (fixed_splits) {
      consider(t, fixed_splits);
      continue;
    }
    for (int s : {1, 2, 3, 4, 6, 8, 12, 16}) {
      if (s > chunks || (s > 1 && !t.may_split)) break;
      consider(t, s);
    }
  }
  // With every compute unit busy the 512 x 128 tile is bound by power, and the same tile built on the 16x16x64 SMFMAC
  // (four wavefronts, one per SIMD) draws less of it per product: 3-5 % faster from about one full round of tiles on
  // (8192^3, 4096^3, 25600^3; 28672 x 512 x 8192 with 224 tiles: 102.9 against 107.0 us), slower when part of the chip
  // idles and the schedule decides (4096 x 3072 x 4096 with 192 tiles: 51.2 against 50.6; 11008 x 768 x 4096: 49 against 41).
  if (best.tile == onebit::kTile512x128w8 && best.splits == 1) {
    const long tiles = (long)((m + 511) / 512) * ((n + 127) / 128);
    if (tiles * 20 >= 17L * compute_units) best.tile = onebit::kTile512x128m16;  // from 85 % of a round on
  }
  return best;
}

// Everything the C ABI decides about one prepared call, from the shape and the alignment of B alone (no GPU needed).
struct LaunchPlan {
  int split_k_kernel;  // 1: skinny_kernel, 0: gemm_kernel
  int rows_or_tile;    // skinny_kernel: weight rows per workgroup; gemm_kernel: TileConfig
  int splits;          // gemm_kernel: K splits over workgroups (1 = none)
  int pad_b;           // gemm_kernel: B is read through a padded copy
};

// Row group and K splits over workgroups of the split-K kernel. Every workgroup of that kernel reads all of B's rows
// of its K range, so with few row groups over a long K (4096 x 28672 x 16: 128 workgroups that each read 900 KB of B
// for 170 KB of weights) the compute units spend their time re-reading B and half of them have no workgroup at all.
// Splitting K over S workgroups per row group divides both; the price is a second launch that adds the S partial
// results (about 3 us in all). Rule fitted to a sweep of m = 2048 ... 11008, k = 4096 ... 28672, n = 16, 32, 64 over
// every row group and S = 1 ... 8 (us, unsplit -> split): 2048 x 28672 x 16 18.5 -> 9.2, 4096 x 16384 x 16 12.0 -> 9.1,
// 4096 x 28672 x 32 28.0 -> 15.6, 8192 x 28672 x 16 21.4 -> 18.4, 8192 x 16384 x 64 30.2 -> 23.0, 11008 x 28672 x 32
// 34.2 -> 28.9; the best split always has at most one workgroup per compute unit and 64-row groups (128 rows when 64
// rows leave no room for two splits); below the threshold on B's bytes per workgroup the second launch costs more
// than the split saves (4096 x 11008 x 16: 8.9 against 8.5).
struct SkinnyPlan {
  int rows, splits;
};
SkinnyPlan plan_skinny(int m, int n, int k, int compute_units) {
  const int chunks = (k + onebit::kChunkK - 1) / onebit::kChunkK;
  const int forced_rows = g_skinny_rows, forced_splits = g_split_k;
  // the largest row group that still gives about two workgroups per three compute units (measured: larger groups
  // re-read B less often, but idle compute units cost more)
  // (n > 32: two column fragments per row block, at most two row blocks per wavefront)
  const int enough = std::max(1, 160 * compute_units / 256);
  int rows = forced_rows > 0 ? forced_rows : (m / 128 >= enough && n <= 32) ? 128 : (m / 64 >= enough) ? 64 : 32;
  if (forced_splits >= 1) return SkinnyPlan{rows, forced_splits > chunks ? chunks : forced_splits};
  const double image_row_bytes = n <= 16 ? 32.0 : n <= 32 ? 64.0 : 128.0;
  const double threshold = 400e3 * std::max(1.0, m / 4096.0);
  if (chunks < 32 || k * image_row_bytes < threshold) return SkinnyPlan{rows, 1};
  auto splits_for = [&](int r) {
    const int groups = (m + r - 1) / r;
    return std::min(compute_units / groups, chunks / 8);  // one workgroup per compute unit, eight chunks per workgroup
  };
  if (forced_rows > 0) {
    const int s = splits_for(rows);
    return SkinnyPlan{rows, s >= 2 ? s : 1};
  }
  if (const int s = splits_for(64); s >= 2) return SkinnyPlan{64, s};
  if (n <= 32)
    if (const int s = splits_for(128); s >= 2) return SkinnyPlan{128, s};
  return SkinnyPlan{rows, 1};
}

LaunchPlan choose_launch(int m, int n, int k, bool b_16_byte_aligned, int compute_units = 256) {
  LaunchPlan plan{};
  // 32 < n <= 64: every 64-row workgroup of the split-K kernel stages all of B, which the main kernel's tiles overtake
  // from about 48k rows on (n = 64: 28672 x 8192 32 us against 42; 32768 x 4096 20 against 26; 49152 x 4096 32.5
  // against 34.4; 65536 x 8192 66 against 68, at n = 40 77 against 66; 131072 x 2048 51 against 35)
  const bool skinny_shape = n <= 32 || (n <= onebit::kSkinnyMaxN && m <= 40960);
  if (skinny_shape && g_skinny_enabled) {
    const SkinnyPlan sk = plan_skinny(m, n, k, compute_units);
    plan.split_k_kernel = 1;
    plan.rows_or_tile = sk.rows;
    plan.splits = sk.splits;
    return plan;
  }
  const GemmPlan gemm = plan_gemm(m, n, k, compute_units);
  plan.rows_or_tile = gemm.tile;
  plan.splits = gemm.splits;
  // B rows that are not 16-byte aligned: pad a copy (one extra pass over B) unless the problem is too small for that
  // to pay against the element-copy variant of the kernel
  const bool b_in_place = n % 8 == 0 && b_16_byte_aligned;
  plan.pad_b = !b_in_place && (size_t)k * n >= 65536 && g_pad_b;
  return plan;
}

// Workspace of one call that the caller cannot let allocate: `base` is this device's copy of the file-scope array
// g_static_scratch (see onebit_sparse_matmul_prepared_static), `bytes` its size.
struct FixedScratch {
  unsigned char* base;
  size_t bytes;
};

// K split of a split-K kernel launch: the split geometry and the partial-sum buffer (the caller's fixed workspace, or
// the library-owned buffer of this device and stream).
int setup_skinny_split(onebit::SkinnyArgs& args, int splits, hipStream_t stream, const FixedScratch* fixed) {
  args.splits = 1;
  if (splits <= 1) return ONEBIT_OK;
  const int cps = (args.kc_total + splits - 1) / splits;
  args.chunks_per_split = cps;
  args.splits = (args.kc_total + cps - 1) / cps;  // every split non-empty
  if (args.splits <= 1) return ONEBIT_OK;
  const size_t bytes = (size_t)args.splits * args.m * args.n * sizeof(float);
  if (fixed) {
    if (bytes > fixed->bytes)
      return fail(ONEBIT_ERR_ARGUMENT,
                  "this shape needs %zu bytes of scratch (%d K splits of %d x %d fp32 partial sums); the static "
                  "workspace of the non-allocating entry point holds %zu", bytes, args.splits, args.m, args.n, fixed->bytes);
    args.split_ws = reinterpret_cast<float*>(fixed->base);
    return ONEBIT_OK;
  }
  int device = 0;
  ONEBIT_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) return fail(ONEBIT_ERR_ARGUMENT, "device ordinal %d not supported", device);
  DeviceState& st = g_dev[device];
  std::lock_guard<std::recursive_mutex> lock(st.mu);
  Buffer& ws = st.split_ws[stream];
  if (int rc = grow(&ws.ptr, &ws.bytes, bytes, stream); rc != ONEBIT_OK) return rc;
  args.split_ws = static_cast<float*>(ws.ptr);
  return ONEBIT_OK;
}

int matmul_prepared_impl(const void* prepared, const void* b, const void* c, void* d, int m, int n, int k, float alpha,
                         float beta, int c_dtype, int d_dtype, hipStream_t stream, const FixedScratch* fixed = nullptr) {
  if (!prepared || !b || !d) return fail(ONEBIT_ERR_ARGUMENT, "null operand pointer");
  if (beta != 0.f && !c) return fail(ONEBIT_ERR_ARGUMENT, "c must not be null when beta != 0");
  const int kc_total = (k + onebit::kChunkK - 1) / onebit::kChunkK;

  const LaunchPlan plan = choose_launch(m, n, k, (reinterpret_cast<uintptr_t>(b) & 15) == 0, current_compute_units());
  if (plan.split_k_kernel) {
    onebit::SkinnyArgs args{};
    args.prep = static_cast<const uint8_t*>(prepared);
    args.b = static_cast<const _Float16*>(b);
    args.c = c;
    args.d = d;
    args.m = m; args.n = n; args.k = k;
    args.kc_total = kc_total;
    args.alpha = alpha; args.beta = beta;
    args.c_f16 = c_dtype == ONEBIT_DTYPE_F16;
    args.d_f16 = d_dtype == ONEBIT_DTYPE_F16;
    if (int rc = setup_skinny_split(args, plan.splits, stream, fixed); rc != ONEBIT_OK) return rc;
    ONEBIT_HIP(onebit::launch_skinny(args, plan.rows_or_tile, stream));
    return ONEBIT_OK;
  }

  if (onebit::prepared_bytes(m, k) >= (size_t(1) << 32))
    return fail(ONEBIT_ERR_ARGUMENT,
                "the main kernel addresses the prepared operand with 32-bit offsets: m x k = %d x %d needs %zu bytes, "
                "the limit is 4 GiB (about 22.9e9 weights); split the weight by rows", m, k, onebit::prepared_bytes(m, k));
  onebit::GemmArgs args{};
  args.prep = static_cast<const uint8_t*>(prepared);
  args.b = static_cast<const _Float16*>(b);
  args.c = c;
  args.d = d;
  args.m = m; args.n = n; args.k = k;
  args.kc_total = kc_total;
  args.alpha = alpha; args.beta = beta;
  args.c_f16 = c_dtype == ONEBIT_DTYPE_F16;
  args.d_f16 = d_dtype == ONEBIT_DTYPE_F16;
  const int tile = plan.rows_or_tile;
  const int splits = plan.splits;
  const bool pad_b = plan.pad_b != 0;
  if (splits > 1 || pad_b) {
    size_t split_bytes = 0, pad_bytes = 0;
    if (splits > 1) {
      const int cps = (kc_total + splits - 1) / splits;
      args.chunks_per_split = cps;
      args.splits = (kc_total + cps - 1) / cps;  // every split non-empty
      split_bytes = (size_t)args.splits * m * n * sizeof(float);
    }
    if (pad_b) pad_bytes = (size_t)k * ((size_t)(n + 7) / 8 * 8) * sizeof(_Float16);
    if (fixed) {
      // partial sums first, the padded copy of B behind them on the next 256-byte boundary; both are written in
      // full by this call's own kernels before they are read, so nothing has to start at zero
      const size_t pad_at = (split_bytes + 255) & ~size_t(255);
      if (pad_at + pad_bytes > fixed->bytes)
        return fail(ONEBIT_ERR_ARGUMENT,
                    "this shape needs %zu bytes of scratch (%d K splits of %d x %d fp32 partial sums, %zu bytes of "
                    "padded B); the static workspace of the non-allocating entry point holds %zu",
                    pad_at + pad_bytes, splits > 1 ? args.splits : 0, m, n, pad_bytes, fixed->bytes);
      if (splits > 1) args.split_ws = reinterpret_cast<float*>(fixed->base);
      if (pad_b) args.b_pad = reinterpret_cast<_Float16*>(fixed->base + pad_at);
      ONEBIT_HIP(onebit::launch_gemm(args, tile, stream));
      return ONEBIT_OK;
    }
    int device = 0;
    ONEBIT_HIP(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return fail(ONEBIT_ERR_ARGUMENT, "device ordinal %d not supported", device);
    DeviceState& st = g_dev[device];
    std::lock_guard<std::recursive_mutex> lock(st.mu);
    if (splits > 1) {
      Buffer& ws = st.split_ws[stream];
      if (int rc = grow(&ws.ptr, &ws.bytes, split_bytes, stream); rc != ONEBIT_OK) return rc;
      args.split_ws = static_cast<float*>(ws.ptr);
    }
    if (pad_b) {
      Buffer& pb = st.b_pad[stream];
      if (int rc = grow(&pb.ptr, &pb.bytes, pad_bytes, stream); rc != ONEBIT_OK) return rc;
      args.b_pad = static_cast<_Float16*>(pb.ptr);
    }
    ONEBIT_HIP(onebit::launch_gemm(args, tile, stream));
    return ONEBIT_OK;
  }
  ONEBIT_HIP(onebit::launch_gemm(args, tile, stream));
  return ONEBIT_OK;
}

}  // namespace

extern "C" {

const char* onebit_sparse_last_error(void) { return g_last_error.c_str(); }

void onebit_sparse_set_tile_config(int tile_config) { g_tile_config = tile_config; }
void onebit_sparse_set_skinny_enabled(int enabled) { g_skinny_enabled = enabled ? 1 : 0; }
void onebit_sparse_set_skinny_rows(int rows) { g_skinny_rows = rows; }
void onebit_sparse_set_split_k(int splits) { g_split_k = splits; }
void onebit_sparse_set_pad_b(int enabled) { g_pad_b = enabled ? 1 : 0; }

int onebit_sparse_describe_launch_for(int m, int n, int k, int b_16_byte_aligned, int compute_units, int* plan) {
  g_last_error.clear();
  if (!plan) return fail(ONEBIT_ERR_ARGUMENT, "plan must not be null");
  if (compute_units <= 0) return fail(ONEBIT_ERR_ARGUMENT, "compute_units must be positive (got %d)", compute_units);
  if (int rc = check_shape(m, n, k)) return rc;
  const LaunchPlan p = choose_launch(m, n, k, b_16_byte_aligned != 0, compute_units);
  plan[0] = p.split_k_kernel;
  plan[1] = p.rows_or_tile;
  plan[2] = p.splits;
  plan[3] = p.pad_b;
  return ONEBIT_OK;
}

int onebit_sparse_describe_launch(int m, int n, int k, int b_16_byte_aligned, int* plan) {
  // the compute units of the current device, as the calls themselves plan; 256 when there is no usable device
  return onebit_sparse_describe_launch_for(m, n, k, b_16_byte_aligned, current_compute_units(), plan);
}

size_t onebit_sparse_prepared_bytes(int m, int k) {
  if (m <= 0 || k <= 0) return 0;
  return onebit::prepared_bytes(m, k);
}

int onebit_sparse_prepare(const void* a, const void* e, int m, int k, int meta_layout, void* prepared, void* stream) {
  g_last_error.clear();
  if (int rc = check_shape(m, 1, k)) return rc;
  if (!a || !e || !prepared) return fail(ONEBIT_ERR_ARGUMENT, "null operand pointer");
  if (meta_layout < ONEBIT_META_REFERENCE || meta_layout > ONEBIT_META_LOGICAL)
    return fail(ONEBIT_ERR_ARGUMENT, "unknown metadata layout %d", meta_layout);
  ONEBIT_HIP(onebit::launch_prepare(a, e, prepared, m, k, meta_layout, static_cast<hipStream_t>(stream)));
  return ONEBIT_OK;
}

int onebit_sparse_pack(const void* weight, int m, int k, int prune, void* a, void* e, int meta_layout, void* stream) {
  g_last_error.clear();
  if (int rc = check_shape(m, 1, k)) return rc;
  if (!weight || !a || !e) return fail(ONEBIT_ERR_ARGUMENT, "null operand pointer");
  if ((reinterpret_cast<uintptr_t>(weight) & 15) != 0)
    return fail(ONEBIT_ERR_ARGUMENT, "the dense weight must be 16-byte aligned");
  if ((reinterpret_cast<uintptr_t>(a) & 7) != 0 || (reinterpret_cast<uintptr_t>(e) & 1) != 0)
    return fail(ONEBIT_ERR_ARGUMENT, "a must be 8-byte aligned and e 2-byte aligned");
  if (meta_layout < ONEBIT_META_REFERENCE || meta_layout > ONEBIT_META_LOGICAL)
    return fail(ONEBIT_ERR_ARGUMENT, "unknown metadata layout %d", meta_layout);
  ONEBIT_HIP(onebit::launch_pack(weight, a, e, m, k, prune, meta_layout, static_cast<hipStream_t>(stream)));
  return ONEBIT_OK;
}

int onebit_sparse_matmul_prepared(const void* prepared, const void* b, const void* c, void* d, int m, int n, int k,
                                  float alpha, float beta, int c_dtype, int d_dtype, void* stream) {
  g_last_error.clear();
  if (int rc = check_shape(m, n, k)) return rc;
  if (int rc = check_dtype(c_dtype, d_dtype)) return rc;
  return matmul_prepared_impl(prepared, b, c, d, m, n, k, alpha, beta, c_dtype, d_dtype, static_cast<hipStream_t>(stream));
}

int onebit_sparse_matmul_prepared_static(const void* prepared, const void* b, const void* c, void* d, int m, int n, int k,
                                         float alpha, float beta, int c_dtype, int d_dtype, void* stream) {
  g_last_error.clear();
  if (int rc = check_shape(m, n, k)) return rc;
  if (int rc = check_dtype(c_dtype, d_dtype)) return rc;
  int device = 0;
  ONEBIT_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) return fail(ONEBIT_ERR_ARGUMENT, "device ordinal %d not supported", device);
  DeviceState& st = g_dev[device];
  FixedScratch fixed{nullptr, kStaticScratchBytes};
  {
    std::lock_guard<std::recursive_mutex> lock(st.mu);
    if (!st.static_scratch) {
      // once per device, with that device current: the address of this device's copy of the array
      void* address = nullptr;
      ONEBIT_HIP(hipGetSymbolAddress(&address, HIP_SYMBOL(g_static_scratch)));
      if (!address) return fail(ONEBIT_ERR_HIP, "hipGetSymbolAddress returned a null address for the static workspace");
      st.static_scratch = static_cast<unsigned char*>(address);
    }
    fixed.base = st.static_scratch;
  }
  return matmul_prepared_impl(prepared, b, c, d, m, n, k, alpha, beta, c_dtype, d_dtype,
                              static_cast<hipStream_t>(stream), &fixed);
}

int onebit_sparse_linear_prepared(const void* prepared, const void* x, const void* bias, void* y, int tokens, int m,
                                  int k, int bias_dtype, int y_dtype, void* stream) {
  g_last_error.clear();
  if (int rc = check_shape(m, tokens, k)) return rc;
  if (int rc = check_dtype(bias_dtype, y_dtype)) return rc;
  if (!prepared || !x || !y) return fail(ONEBIT_ERR_ARGUMENT, "null operand pointer");
  if ((reinterpret_cast<uintptr_t>(x) & 15) != 0) return fail(ONEBIT_ERR_ARGUMENT, "x must be 16-byte aligned");
  const int kc_total = (k + onebit::kChunkK - 1) / onebit::kChunkK;
  LaunchPlan plan = choose_launch(m, tokens, k, true, current_compute_units());
  if ((size_t)k * 256 * 2 >= (size_t(1) << 32))
    return fail(ONEBIT_ERR_ARGUMENT, "the token-major form addresses x with 32-bit offsets inside a tile of 256 tokens: "
                                     "k = %d is beyond its limit of 8388607", k);
  if (plan.split_k_kernel) {
    onebit::SkinnyArgs args{};
    args.prep = static_cast<const uint8_t*>(prepared);
    args.b = static_cast<const _Float16*>(x);
    args.d = y;
    args.m = m; args.n = tokens; args.k = k;
    args.kc_total = kc_total;
    args.alpha = 1.f; args.beta = 0.f;
    args.d_f16 = y_dtype == ONEBIT_DTYPE_F16;
    args.bias = bias;
    args.bias_f16 = bias_dtype == ONEBIT_DTYPE_F16;
    if (int rc = setup_skinny_split(args, plan.splits, static_cast<hipStream_t>(stream), nullptr); rc != ONEBIT_OK) return rc;
    ONEBIT_HIP(onebit::launch_skinny_tokens(args, plan.rows_or_tile, static_cast<hipStream_t>(stream)));
    return ONEBIT_OK;
  }
  switch (plan.rows_or_tile) {
    case onebit::kTile256x128w: case onebit::kTile128x128s: case onebit::kTile512x128w8: case onebit::kTile256x128w8:
    case onebit::kTile128x128w8: case onebit::kTile64x128: case onebit::kTile128x128k2: case onebit::kTile64x128k2:
    case onebit::kTile512x128m16: break;
    default:
      return fail(ONEBIT_ERR_ARGUMENT, "tile configuration %d has no token-major variant (4, 6, 9 ... 15 have)",
                  plan.rows_or_tile);
  }
  if (onebit::prepared_bytes(m, k) >= (size_t(1) << 32))
    return fail(ONEBIT_ERR_ARGUMENT,
                "the main kernel addresses the prepared operand with 32-bit offsets: m x k = %d x %d needs %zu bytes, "
                "the limit is 4 GiB (about 22.9e9 weights); split the weight by rows", m, k, onebit::prepared_bytes(m, k));
  onebit::GemmArgs args{};
  args.prep = static_cast<const uint8_t*>(prepared);
  args.b = static_cast<const _Float16*>(x);
  args.d = y;
  args.m = m; args.n = tokens; args.k = k;
  args.kc_total = kc_total;
  args.d_f16 = y_dtype == ONEBIT_DTYPE_F16;
  args.bias = bias;
  args.bias_f16 = bias_dtype == ONEBIT_DTYPE_F16;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (plan.splits > 1) {
    int device = 0;
    ONEBIT_HIP(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return fail(ONEBIT_ERR_ARGUMENT, "device ordinal %d not supported", device);
    DeviceState& st = g_dev[device];
    std::lock_guard<std::recursive_mutex> lock(st.mu);
    const int cps = (kc_total + plan.splits - 1) / plan.splits;
    args.chunks_per_split = cps;
    args.splits = (kc_total + cps - 1) / cps;  // every split non-empty
    Buffer& ws = st.split_ws[s];
    if (int rc = grow(&ws.ptr, &ws.bytes, (size_t)args.splits * m * tokens * sizeof(float), s); rc != ONEBIT_OK) return rc;
    args.split_ws = static_cast<float*>(ws.ptr);
    ONEBIT_HIP(onebit::launch_gemm_tokens(args, plan.rows_or_tile, s));
    return ONEBIT_OK;
  }
  ONEBIT_HIP(onebit::launch_gemm_tokens(args, plan.rows_or_tile, s));
  return ONEBIT_OK;
}

int onebit_sparse_linear_prepared_grouped(const onebit_linear_problem* problems, int count, int tokens, int bias_dtype,
                                          int y_dtype, void* stream) {
  g_last_error.clear();
  if (!problems || count < 1) return fail(ONEBIT_ERR_ARGUMENT, "problems must point to at least one problem (count = %d)", count);
  if (int rc = check_dtype(bias_dtype, y_dtype)) return rc;
  for (int i = 0; i < count; ++i) {
    const onebit_linear_problem& q = problems[i];
    if (int rc = check_shape(q.m, tokens, q.k)) return rc;
    if (!q.prepared || !q.x || !q.y) return fail(ONEBIT_ERR_ARGUMENT, "null operand pointer in problem %d", i);
    if ((reinterpret_cast<uintptr_t>(q.x) & 15) != 0) return fail(ONEBIT_ERR_ARGUMENT, "x of problem %d must be 16-byte aligned", i);
    if ((size_t)q.k * 256 * 2 >= (size_t(1) << 32))
      return fail(ONEBIT_ERR_ARGUMENT, "the token-major form addresses x with 32-bit offsets inside a tile of 256 tokens: "
                                       "k = %d of problem %d is beyond its limit of 8388607", q.k, i);
  }
  // Beyond the split-K kernel's range of token counts, or with that kernel switched off, there is nothing to share:
  // one call of the single form per problem.
  if (tokens > onebit::kSkinnyMaxN || !g_skinny_enabled) {
    for (int i = 0; i < count; ++i) {
      const onebit_linear_problem& q = problems[i];
      if (int rc = onebit_sparse_linear_prepared(q.prepared, q.x, q.bias, q.y, tokens, q.m, q.k, bias_dtype, y_dtype, stream))
        return rc;
    }
    return ONEBIT_OK;
  }
  // Row group of the launch: as for one product with all the weight rows, the largest that still gives about two
  // workgroups per three compute units.
  const int compute_units = current_compute_units();
  for (int first = 0; first < count; first += onebit::kSkinnyMaxGroup) {
    const int in_launch = std::min(count - first, onebit::kSkinnyMaxGroup);
    long rows_total = 0;
    for (int i = 0; i < in_launch; ++i) rows_total += problems[first + i].m;
    const int enough = std::max(1, 160 * compute_units / 256);
    const int rows = g_skinny_rows > 0 ? g_skinny_rows
                     : (rows_total / 128 >= enough && tokens <= 32) ? 128 : (rows_total / 64 >= enough) ? 64 : 32;
    if (rows != 32 && rows != 64 && rows != 128) return fail(ONEBIT_ERR_ARGUMENT, "row group %d: must be 32, 64 or 128", rows);
    onebit::SkinnyGroupArgs group{};
    group.count = in_launch;
    for (int i = 0; i < in_launch; ++i) {
      const onebit_linear_problem& q = problems[first + i];
      onebit::SkinnyArgs& args = group.problem[i];
      args.prep = static_cast<const uint8_t*>(q.prepared);
      args.b = static_cast<const _Float16*>(q.x);
      args.d = q.y;
      args.m = q.m; args.n = tokens; args.k = q.k;
      args.kc_total = (q.k + onebit::kChunkK - 1) / onebit::kChunkK;
      args.alpha = 1.f; args.beta = 0.f;
      args.d_f16 = y_dtype == ONEBIT_DTYPE_F16;
      args.bias = q.bias;
      args.bias_f16 = bias_dtype == ONEBIT_DTYPE_F16;
    }
    ONEBIT_HIP(onebit::launch_skinny_group(group, rows, static_cast<hipStream_t>(stream)));
  }
  return ONEBIT_OK;
}

int onebit_sparse_matmul_ex(const void* a, const void* b, const void* c, void* d, const void* e, int m, int n, int k,
                            float alpha, float beta, int c_dtype, int d_dtype, int meta_layout, void* stream) {
  g_last_error.clear();
  if (int rc = check_shape(m, n, k)) return rc;
  if (int rc = check_dtype(c_dtype, d_dtype)) return rc;
  if (!a || !b || !d || !e) return fail(ONEBIT_ERR_ARGUMENT, "null operand pointer");
  if (beta != 0.f && !c) return fail(ONEBIT_ERR_ARGUMENT, "c must not be null when beta != 0");
  if (meta_layout < ONEBIT_META_REFERENCE || meta_layout > ONEBIT_META_LOGICAL)
    return fail(ONEBIT_ERR_ARGUMENT, "unknown metadata layout %d", meta_layout);
  hipStream_t s = static_cast<hipStream_t>(stream);
  int device = 0;
  ONEBIT_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) return fail(ONEBIT_ERR_HIP, "device index %d out of range", device);
  DeviceState& ds = g_dev[device];
  void* prep = nullptr;
  const int cache_entries = g_weight_cache_entries.load();
  if (cache_entries > 0) {
    {  // the lock ends before the multiplication is launched, which may take it again for its own buffers
      std::lock_guard<std::recursive_mutex> lock(ds.mu);
      for (auto& w : ds.weight_cache)
        if (w.a == a && w.e == e && w.m == m && w.k == k && w.layout == meta_layout) {
          w.last_use = ++ds.use_counter;
          if (w.stream != s) ONEBIT_HIP(hipStreamWaitEvent(s, w.ready, 0));  // its reorder kernel ran on another stream
          prep = w.prep;
          break;
        }
      if (!prep) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        ONEBIT_HIP(hipStreamIsCapturing(s, &capture));
        if (capture != hipStreamCaptureStatusNone)
          return fail(ONEBIT_ERR_ARGUMENT, "a weight that is not in the cache yet cannot be added while the stream is "
                                           "being captured: run the call once outside the capture first");
        if ((int)ds.weight_cache.size() >= cache_entries) {  // evict the least recently used entry
          size_t victim = 0;
          for (size_t i = 1; i < ds.weight_cache.size(); ++i)
            if (ds.weight_cache[i].last_use < ds.weight_cache[victim].last_use) victim = i;
          ONEBIT_HIP(hipDeviceSynchronize());  // earlier work on any stream may still read it
          ONEBIT_HIP(hipFree(ds.weight_cache[victim].prep));
          ONEBIT_HIP(hipEventDestroy(ds.weight_cache[victim].ready));
          ds.weight_cache.erase(ds.weight_cache.begin() + victim);
        }
        DeviceState::CachedWeight w{a, e, m, k, meta_layout, nullptr, s, nullptr, ++ds.use_counter};
        ONEBIT_HIP(hipMalloc(&w.prep, onebit::prepared_bytes(m, k)));
        if (hipError_t st = hipEventCreateWithFlags(&w.ready, hipEventDisableTiming); st != hipSuccess) {
          (void)hipFree(w.prep);
          return fail(ONEBIT_ERR_HIP, "HIP error '%s' from hipEventCreateWithFlags", hipGetErrorString(st));
        }
        hipError_t st = onebit::launch_prepare(a, e, w.prep, m, k, meta_layout, s);
        if (st == hipSuccess) st = hipEventRecord(w.ready, s);
        if (st != hipSuccess) {
          (void)hipFree(w.prep);
          (void)hipEventDestroy(w.ready);
          return fail(ONEBIT_ERR_HIP, "HIP error '%s' while reordering a cached weight", hipGetErrorString(st));
        }
        ds.weight_cache.push_back(w);
        prep = w.prep;
      }
    }
    return matmul_prepared_impl(prep, b, c, d, m, n, k, alpha, beta, c_dtype, d_dtype, s);
  }
  // the lock is kept until both kernels are enqueued: a call from another thread that has to grow this stream's
  // buffer (which frees the old one) then waits, and its device synchronization covers the work enqueued here
  std::lock_guard<std::recursive_mutex> lock(ds.mu);
  Buffer& own = ds.prep[s];
  if (int rc = grow(&own.ptr, &own.bytes, onebit::prepared_bytes(m, k), s)) return rc;
  prep = own.ptr;
  ONEBIT_HIP(onebit::launch_prepare(a, e, prep, m, k, meta_layout, s));
  return matmul_prepared_impl(prep, b, c, d, m, n, k, alpha, beta, c_dtype, d_dtype, s);
}

int onebit_sparse_clear_weight_cache(void) {
  g_last_error.clear();
  int previous = 0;
  const bool have_device = hipGetDevice(&previous) == hipSuccess;
  int rc = ONEBIT_OK;
  for (int device = 0; device < kMaxDevices; ++device) {
    DeviceState& ds = g_dev[device];
    std::lock_guard<std::recursive_mutex> lock(ds.mu);
    if (ds.weight_cache.empty()) continue;
    if (hipSetDevice(device) != hipSuccess || hipDeviceSynchronize() != hipSuccess) {
      rc = fail(ONEBIT_ERR_HIP, "cannot synchronize device %d to clear its weight cache", device);
      continue;
    }
    for (auto& w : ds.weight_cache) {
      (void)hipFree(w.prep);
      (void)hipEventDestroy(w.ready);
    }
    ds.weight_cache.clear();
  }
  if (have_device) (void)hipSetDevice(previous);
  return rc;
}

int onebit_sparse_release_buffers(void) {
  g_last_error.clear();
  int previous = 0;
  const bool have_device = hipGetDevice(&previous) == hipSuccess;
  int rc = ONEBIT_OK;
  for (int device = 0; device < kMaxDevices; ++device) {
    DeviceState& ds = g_dev[device];
    std::lock_guard<std::recursive_mutex> lock(ds.mu);
    if (ds.prep.empty() && ds.split_ws.empty() && ds.b_pad.empty()) continue;
    if (hipSetDevice(device) != hipSuccess || hipDeviceSynchronize() != hipSuccess) {
      rc = fail(ONEBIT_ERR_HIP, "cannot synchronize device %d to release its buffers", device);
      continue;
    }
    for (auto* buffers : {&ds.prep, &ds.split_ws, &ds.b_pad}) {
      for (auto& entry : *buffers)
        if (entry.second.ptr) (void)hipFree(entry.second.ptr);
      buffers->clear();
    }
  }
  if (have_device) (void)hipSetDevice(previous);
  return rc;
}

int onebit_sparse_set_weight_cache(int entries) {
  g_weight_cache_entries.store(entries > 0 ? entries : 0);
  return entries > 0 ? ONEBIT_OK : onebit_sparse_clear_weight_cache();
}

void onebit_sparse_matmul(void* a, void* b, void* c, void* d, void* e, int m, int n, int k) {
  const int rc = onebit_sparse_matmul_ex(a, b, c, d, e, m, n, k, 1.0f, 0.0f, ONEBIT_DTYPE_F32, ONEBIT_DTYPE_F32,
                                         ONEBIT_META_REFERENCE, nullptr);
  if (rc != ONEBIT_OK) {
    fprintf(stderr, "Got onebit_sparse_matmul error: %s\n", g_last_error.c_str());
    exit(EXIT_FAILURE);
  }
}

}  // extern "C"

// The reference header declares the entry point without extern "C" (include/onebit_sparse_tensor.h:5), so
// objects compiled against it reference the C++-mangled name; export that name as well.
void onebit_sparse_matmul_cxx_name(void* a, void* b, void* c, void* d, void* e, int m, int n, int k)
    __asm__("_Z20onebit_sparse_matmulPvS_S_S_S_iii");
__attribute__((visibility("default"))) void onebit_sparse_matmul_cxx_name(void* a, void* b, void* c, void* d, void* e,
                                                                          int m, int n, int k) {
  onebit_sparse_matmul(a, b, c, d, e, m, n, k);
}
