// A plain C++ host of libfa8.so: no Python, no PyTorch.  Reads fp8 q, k, v (contiguous [B,H,N,d] bytes) from files, runs
// fa8_fwd on a stream of its own and writes the fp16 output bytes.  tests/test_cabi_host_gpu.py builds it with hipcc,
// runs it on the golden inputs and compares the bytes with what the same call gives through ctypes.
//
//   cabi_host B H N d causal scale q.bin k.bin v.bin o.bin
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "fa8_api.h"

#define HIP_OK(x)                                                            \
  do {                                                                       \
    hipError_t e_ = (x);                                                     \
    if (e_ != hipSuccess) {                                                  \
      std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));           \
      return 1;                                                              \
    }                                                                        \
  } while (0)

static bool read_file(const char* path, std::vector<unsigned char>& buf) {
  FILE* f = std::fopen(path, "rb");
  if (!f) return false;
  const bool ok = std::fread(buf.data(), 1, buf.size(), f) == buf.size();
  std::fclose(f);
  return ok;
}

int main(int argc, char** argv) {
  if (argc != 11) {
    std::fprintf(stderr, "usage: cabi_host B H N d causal scale q.bin k.bin v.bin o.bin\n");
    return 2;
  }
  const int B = std::atoi(argv[1]), H = std::atoi(argv[2]), N = std::atoi(argv[3]), d = std::atoi(argv[4]);
  const size_t n = (size_t)B * H * N * d;
  std::vector<unsigned char> q(n), k(n), v(n), o(2 * n);
  if (!read_file(argv[7], q) || !read_file(argv[8], k) || !read_file(argv[9], v)) {
    std::fprintf(stderr, "cannot read the inputs\n");
    return 2;
  }
  if (fa8_query(FA8_QUERY_PARAMS_SIZE) != (int)sizeof(Fa8FwdParams)) {
    std::fprintf(stderr, "libfa8.so was built against another Fa8FwdParams layout\n");
    return 2;
  }
  void *dq, *dk, *dv, *dout;
  hipStream_t stream;
  HIP_OK(hipSetDevice(0));
  HIP_OK(hipStreamCreate(&stream));
  HIP_OK(hipMalloc(&dq, n));
  HIP_OK(hipMalloc(&dk, n));
  HIP_OK(hipMalloc(&dv, n));
  HIP_OK(hipMalloc(&dout, 2 * n));
  HIP_OK(hipMemcpyAsync(dq, q.data(), n, hipMemcpyHostToDevice, stream));
  HIP_OK(hipMemcpyAsync(dk, k.data(), n, hipMemcpyHostToDevice, stream));
  HIP_OK(hipMemcpyAsync(dv, v.data(), n, hipMemcpyHostToDevice, stream));

  Fa8FwdParams p = {};
  p.q = dq;
  p.k = dk;
  p.v = dv;
  p.o = dout;
  p.batch = B;
  p.heads = H;
  p.seqlen_q = p.seqlen_k = N;
  p.head_dim = d;
  p.is_causal = std::atoi(argv[5]) ? 1 : 0;
  p.in_dtype = FA8_DTYPE_E4M3;
  p.out_dtype = FA8_OUT_FP16;
  p.v_layout = FA8_V_ROWS;
  p.softmax_scale = (float)std::atof(argv[6]);
  p.q_row_stride = p.k_row_stride = p.v_row_stride = p.o_row_stride = d;
  p.q_head_stride = p.k_head_stride = p.v_head_stride = p.o_head_stride = (int64_t)N * d;
  p.q_batch_stride = p.k_batch_stride = p.v_batch_stride = p.o_batch_stride = (int64_t)H * N * d;
  int rc = fa8_fwd_validate(&p);
  if (rc == FA8_OK) rc = fa8_fwd(&p, stream);
  if (rc != FA8_OK) {
    std::fprintf(stderr, "fa8_fwd: %s (code %d)\n", fa8_error_string(rc), rc);
    return 1;
  }
  // a rejected call launches nothing and says why
  Fa8FwdParams bad = p;
  bad.head_dim = 80;
  if (fa8_fwd(&bad, stream) != FA8_ERR_HEAD_DIM) {
    std::fprintf(stderr, "head_dim 80 was not rejected\n");
    return 1;
  }
  HIP_OK(hipMemcpyAsync(o.data(), dout, 2 * n, hipMemcpyDeviceToHost, stream));
  HIP_OK(hipStreamSynchronize(stream));
  FILE* f = std::fopen(argv[10], "wb");
  if (!f || std::fwrite(o.data(), 1, o.size(), f) != o.size()) {
    std::fprintf(stderr, "cannot write %s\n", argv[10]);
    return 2;
  }
  std::fclose(f);
  HIP_OK(hipFree(dq));
  HIP_OK(hipFree(dk));
  HIP_OK(hipFree(dv));
  HIP_OK(hipFree(dout));
  HIP_OK(hipStreamDestroy(stream));
  std::printf("cabi_host ok: B=%d H=%d N=%d d=%d\n", B, H, N, d);
  return 0;
}
