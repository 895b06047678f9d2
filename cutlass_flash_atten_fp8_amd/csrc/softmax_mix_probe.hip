// Measurement tool (not part of libfa8.so): what one SIMD of gfx950 needs for the instruction mix of one KV block of the
// attention loop -- 32 logits per lane: 16 v_max3, 32 v_fma, 33 v_exp, 32 v_add, 16 v_cvt_pk_fp8, the 64 v_mul of the O
// rescale in a given share of the blocks, and the 8 v_mfma_f32_32x32x64_f8f6f4 (4 for S^T, 4 for P V) -- with no LDS, no
// HBM traffic and no barrier.  It bounds what fa8_fwd_kernel<128, ...> can reach and shows how far the vector and the matrix
// work of a SIMD overlap.  `bench.py --instruction-mix` runs it; profiles/ holds the output of one run.
//
//   softmax_mix_probe            prints one JSON line per measurement
#include <hip/hip_runtime.h>

#include <cstdio>

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

#define CHECK(x)                                                             \
  do {                                                                       \
    hipError_t e_ = (x);                                                     \
    if (e_ != hipSuccess) {                                                  \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                \
      return 1;                                                              \
    }                                                                        \
  } while (0)

// VALU: the softmax arithmetic of a block; MFMA: the eight matrix instructions; RESCALE_OF_5: in how many of five blocks
// the 64 accumulators are multiplied (the kernel does it when some row's max moved: about 4 of 5 blocks on the headline data)
template <bool VALU, bool MFMA, int RESCALE_OF_5>
__global__ __launch_bounds__(768) void block_mix(float* out, const v8i* operands, int iters, float c) {
  v16f s[2], o[4];
  const v8i kv = operands[threadIdx.x & 63], q0 = operands[64 + (threadIdx.x & 63)], q1 = operands[128 + (threadIdx.x & 63)];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) s[t][i] = 0.01f * (float)((threadIdx.x + 5 * i + 3 * t) & 63);
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[t][i] = 0.f;
  float m_run = 0.f, l_run = 0.f;
  v8i p8 = kv;
  for (int it = 0; it < iters; ++it) {
    if constexpr (VALU) {
      float mx[4];
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) mx[ch] = __builtin_fmaxf(__builtin_fmaxf(s[0][4 * ch], s[0][4 * ch + 1]), s[0][4 * ch + 2]);
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) mx[ch] = __builtin_fmaxf(__builtin_fmaxf(mx[ch], s[0][4 * ch + 3]), s[1][4 * ch]);
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) mx[ch] = __builtin_fmaxf(__builtin_fmaxf(mx[ch], s[1][4 * ch + 1]), s[1][4 * ch + 2]);
      float m_new = __builtin_fmaxf(__builtin_fmaxf(__builtin_fmaxf(__builtin_fmaxf(mx[0], s[1][3]), s[1][7]),
                                                    __builtin_fmaxf(__builtin_fmaxf(mx[1], s[1][11]), s[1][15])),
                                    __builtin_fmaxf(__builtin_fmaxf(mx[2], mx[3]), m_run));
      const unsigned both = __builtin_amdgcn_permlane32_swap(__float_as_uint(m_new), __float_as_uint(m_new), false, false)[0];
      m_new = __builtin_fmaxf(m_new, __uint_as_float(both));
      if (it % 5 < RESCALE_OF_5) {  // wave-uniform, like the kernel's "some row's max moved"
        const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c);
        l_run *= alpha;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[t][i] *= alpha;
      }
      m_run = m_new;
      const float mc = m_new * c;
      float sum0 = 0.f, sum1 = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int i = 0; i < 16; ++i) s[t][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][i], c, -mc));
#pragma unroll
        for (int i = 0; i < 16; i += 2) {
          sum0 += s[t][i];
          sum1 += s[t][i + 1];
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          int r = p8[4 * t + w];
          r = __builtin_amdgcn_cvt_pk_fp8_f32(s[t][4 * w], s[t][4 * w + 1], r, false);
          r = __builtin_amdgcn_cvt_pk_fp8_f32(s[t][4 * w + 2], s[t][4 * w + 3], r, true);
          p8[4 * t + w] = r;
        }
      }
      l_run += sum0 + sum1;
      asm volatile("" : "+v"(l_run));
    }
    if constexpr (MFMA) {
#pragma unroll
      for (int t = 0; t < 4; ++t) o[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kv, p8, o[t], 0, 0, 0, 0, 0, 0);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        v16f z;
#pragma unroll
        for (int i = 0; i < 16; ++i) z[i] = VALU ? 0.f : s[t][i] * 1e-30f;  // MFMA-only run: keep the chain alive
        s[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kv, q0, z, 0, 0, 0, 0, 0, 0);
        s[t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(p8, q1, s[t], 0, 0, 0, 0, 0, 0);
      }
    } else {
      // vector-only run: new "logits" for the next block from two cheap instructions per value (reported separately)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) s[t][i] = __builtin_fmaf(s[t][i], 3.0f, (float)(i & 3));
    }
  }
  float r = l_run + m_run + __int_as_float(p8[0] & 0x3f000000);
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) r += s[t][i];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) r += o[t][i];
  if (r == 1.2345f) out[0] = r;  // never true: keeps the work alive
}

template <bool VALU, bool MFMA, int R>
static int measure(const char* what, int waves_per_simd, float* dout, const v8i* dops, int n_cus) {
  const int iters = 4000;
  float best = 1e30f;
  for (int rep = 0; rep < 3; ++rep) {
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    CHECK(hipEventRecord(e0));
    hipLaunchKernelGGL((block_mix<VALU, MFMA, R>), dim3(n_cus), dim3(256 * waves_per_simd), 0, 0, dout, dops, iters, 0.1275f);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    if (rep > 0 && ms < best) best = ms;
  }
  const double ns = best * 1e6 / iters / waves_per_simd;  // per block and wavefront slot of a SIMD
  printf("{\"mix\": \"%s\", \"waves_per_simd\": %d, \"rescale_blocks_of_5\": %d, \"ns_per_block_per_wavefront\": %.1f, "
         "\"headline_kernel_floor_us\": %.1f}\n", what, waves_per_simd, R, ns, ns * 512 / 1e3);
  return 0;
}

int main() {
  hipDeviceProp_t prop;
  CHECK(hipGetDeviceProperties(&prop, 0));
  const int n_cus = prop.multiProcessorCount;
  float* dout;
  v8i* dops;
  CHECK(hipMalloc(&dout, 64));
  CHECK(hipMalloc(&dops, 192 * sizeof(v8i)));
  v8i hops[192];
  unsigned x = 12345u;
  for (int i = 0; i < 192; ++i)
    for (int j = 0; j < 8; ++j) {
      x = x * 1664525u + 1013904223u;
      hops[i][j] = (int)(x & 0x3f3f3f3fu) | 0x20202020;  // fp8 codes of moderate positive values
    }
  CHECK(hipMemcpy(dops, hops, sizeof(hops), hipMemcpyHostToDevice));
  // the headline kernel runs 3 wavefronts per SIMD, each for 512/3 ... in total 512 (wavefront, block) pairs per SIMD
  for (int w : {2, 3}) {
    if (measure<false, true, 0>("8 mfma", w, dout, dops, n_cus)) return 1;
    if (measure<true, false, 0>("softmax vector work + 32 fma, no rescale", w, dout, dops, n_cus)) return 1;
    if (measure<true, false, 4>("softmax vector work + 32 fma, rescale in 4 of 5 blocks", w, dout, dops, n_cus)) return 1;
    if (measure<true, true, 0>("softmax vector work + 8 mfma, no rescale", w, dout, dops, n_cus)) return 1;
    if (measure<true, true, 4>("softmax vector work + 8 mfma, rescale in 4 of 5 blocks", w, dout, dops, n_cus)) return 1;
    if (measure<true, true, 5>("softmax vector work + 8 mfma, rescale in every block", w, dout, dops, n_cus)) return 1;
  }
  return 0;
}
