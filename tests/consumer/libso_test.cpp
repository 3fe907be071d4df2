// A C++ program that consumes libonebitmul the way a program built against the reference does: it declares the entry
// point exactly as the reference's header does (include/onebit_sparse_tensor.h:5 of the reference: C++ linkage, no
// extern "C"), so the linker must resolve the C++-mangled name _Z20onebit_sparse_matmulPvS_S_S_S_iii, and links with
// -lonebitmul as the reference's makefile does (makefile:22-23, tests/libso_test.cu:3-22). Unlike the reference's
// link test, which passes uninitialised pointers, this one multiplies real operands:
//
//   libso_test <m> <n> <k> <a.bin> <b.bin> <e.bin> <d.bin>
//
// reads the stored operands (a: m*k/16 bytes of sign bits, b: k*n fp16, e: m*k/16 int16 of metadata in the reference
// layout), calls onebit_sparse_matmul on device copies (fp32 c = d, alpha 1, beta 0, default stream, as the reference's
// torch binding does, onebit_sparse_mul/torch_kernel_cuda.cpp:20-29), writes the m*n fp32 results to d.bin and prints
// their sum.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

void onebit_sparse_matmul(void *a, void *b, void *c, void *d, void *e, int m, int n, int k);

static std::vector<char> read_file(const char *path, size_t bytes) {
  std::vector<char> data(bytes);
  FILE *f = std::fopen(path, "rb");
  if (!f || std::fread(data.data(), 1, bytes, f) != bytes) {
    std::fprintf(stderr, "cannot read %zu bytes from %s\n", bytes, path);
    std::exit(2);
  }
  std::fclose(f);
  return data;
}

#define CHECK(expr)                                                                     \
  do {                                                                                  \
    hipError_t st_ = (expr);                                                            \
    if (st_ != hipSuccess) {                                                            \
      std::fprintf(stderr, "%s failed: %s\n", #expr, hipGetErrorString(st_));           \
      return 3;                                                                         \
    }                                                                                   \
  } while (0)

int main(int argc, char **argv) {
  if (argc != 8) {
    std::fprintf(stderr, "usage: %s m n k a.bin b.bin e.bin d.bin\n", argv[0]);
    return 2;
  }
  const int m = std::atoi(argv[1]), n = std::atoi(argv[2]), k = std::atoi(argv[3]);
  const size_t a_bytes = (size_t)m * k / 16, b_bytes = (size_t)k * n * 2, e_bytes = (size_t)m * k / 8;
  const size_t d_bytes = (size_t)m * n * 4;
  const std::vector<char> a = read_file(argv[4], a_bytes), b = read_file(argv[5], b_bytes), e = read_file(argv[6], e_bytes);
  void *da = nullptr, *db = nullptr, *de = nullptr, *dd = nullptr;
  CHECK(hipMalloc(&da, a_bytes));
  CHECK(hipMalloc(&db, b_bytes));
  CHECK(hipMalloc(&de, e_bytes));
  CHECK(hipMalloc(&dd, d_bytes));
  CHECK(hipMemcpy(da, a.data(), a_bytes, hipMemcpyHostToDevice));
  CHECK(hipMemcpy(db, b.data(), b_bytes, hipMemcpyHostToDevice));
  CHECK(hipMemcpy(de, e.data(), e_bytes, hipMemcpyHostToDevice));
  CHECK(hipMemset(dd, 0xFF, d_bytes));
  onebit_sparse_matmul(da, db, dd, dd, de, m, n, k);
  CHECK(hipDeviceSynchronize());
  std::vector<float> d((size_t)m * n);
  CHECK(hipMemcpy(d.data(), dd, d_bytes, hipMemcpyDeviceToHost));
  FILE *f = std::fopen(argv[7], "wb");
  if (!f || std::fwrite(d.data(), 1, d_bytes, f) != d_bytes) {
    std::fprintf(stderr, "cannot write %s\n", argv[7]);
    return 2;
  }
  std::fclose(f);
  double sum = 0.0;
  for (float v : d) sum += v;
  std::printf("sum %.1f\n", sum);
  (void)hipFree(da);
  (void)hipFree(db);
  (void)hipFree(de);
  (void)hipFree(dd);
  return 0;
}
