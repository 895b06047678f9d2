// Records what the gfx950 matrix instruction v_mfma_f32_32x32x64_f8f6f4 returns for given operands: the source of the
// hardware vectors in mfma_f8f6f4_vectors.npz (see make_mfma_vectors.py, which builds and runs this file).
//
//   mfma_probe IN OUT
// IN : int32 n, int32 fmt (0 = e4m3, 1 = e5m2); A[n][32][64] fp8 codes (row, k); B[n][32][64] fp8 codes (column, k);
//      C[n][32][32] float (row, column).     OUT: D[n][32][32] float, D = A B^T + C, one instruction per n.
// Register layouts of the instruction: lane l holds row (column) l % 32 and k = 32 * (l / 32) ... + 31 of A (B);
// accumulator register i of lane l is row 8 * (i / 4) + 4 * (l / 32) + i % 4, column l % 32.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <vector>

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

template <int FMT>
__global__ void one_mfma_per_block(const uint8_t* A, const uint8_t* B, const float* C, float* D) {
  const int n = blockIdx.x, l = threadIdx.x;
  const int* a = (const int*)(A + (size_t)n * 2048 + (l % 32) * 64 + 32 * (l / 32));
  const int* b = (const int*)(B + (size_t)n * 2048 + (l % 32) * 64 + 32 * (l / 32));
  v8i av, bv;
  for (int i = 0; i < 8; ++i) {
    av[i] = a[i];
    bv[i] = b[i];
  }
  v16f c;
  for (int i = 0; i < 16; ++i) c[i] = C[(size_t)n * 1024 + (8 * (i / 4) + 4 * (l / 32) + i % 4) * 32 + l % 32];
  c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, FMT, FMT, 0, 0, 0, 0);
  for (int i = 0; i < 16; ++i) D[(size_t)n * 1024 + (8 * (i / 4) + 4 * (l / 32) + i % 4) * 32 + l % 32] = c[i];
}

#define CHECK(x)                                                                  \
  do {                                                                            \
    hipError_t e_ = (x);                                                          \
    if (e_ != hipSuccess) {                                                       \
      fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));              \
      return 1;                                                                   \
    }                                                                             \
  } while (0)

int main(int argc, char** argv) {
  if (argc != 3) {
    fprintf(stderr, "usage: mfma_probe IN OUT\n");
    return 2;
  }
  FILE* f = fopen(argv[1], "rb");
  int hdr[2];
  if (!f || fread(hdr, 4, 2, f) != 2 || hdr[0] < 1 || hdr[0] > (1 << 20) || (hdr[1] != 0 && hdr[1] != 1)) {
    fprintf(stderr, "cannot read the header of %s\n", argv[1]);
    return 2;
  }
  const size_t n = (size_t)hdr[0];
  std::vector<uint8_t> a(n * 2048), b(n * 2048);
  std::vector<float> c(n * 1024), d(n * 1024);
  if (fread(a.data(), 1, a.size(), f) != a.size() || fread(b.data(), 1, b.size(), f) != b.size() ||
      fread(c.data(), 4, c.size(), f) != c.size()) {
    fprintf(stderr, "%s is shorter than its header says\n", argv[1]);
    return 2;
  }
  fclose(f);
  uint8_t *da, *db;
  float *dc, *dd;
  CHECK(hipMalloc(&da, a.size()));
  CHECK(hipMalloc(&db, b.size()));
  CHECK(hipMalloc(&dc, c.size() * 4));
  CHECK(hipMalloc(&dd, d.size() * 4));
  CHECK(hipMemcpy(da, a.data(), a.size(), hipMemcpyHostToDevice));
  CHECK(hipMemcpy(db, b.data(), b.size(), hipMemcpyHostToDevice));
  CHECK(hipMemcpy(dc, c.data(), c.size() * 4, hipMemcpyHostToDevice));
  if (hdr[1] == 0)
    hipLaunchKernelGGL(one_mfma_per_block<0>, dim3((unsigned)n), dim3(64), 0, 0, da, db, dc, dd);
  else
    hipLaunchKernelGGL(one_mfma_per_block<1>, dim3((unsigned)n), dim3(64), 0, 0, da, db, dc, dd);
  CHECK(hipGetLastError());
  CHECK(hipDeviceSynchronize());
  CHECK(hipMemcpy(d.data(), dd, d.size() * 4, hipMemcpyDeviceToHost));
  f = fopen(argv[2], "wb");
  if (!f || fwrite(d.data(), 4, d.size(), f) != d.size()) {
    fprintf(stderr, "cannot write %s\n", argv[2]);
    return 2;
  }
  fclose(f);
  return 0;
}
