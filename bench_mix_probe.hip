// Measurement tool of `bench.py --instruction-mix` (not part of the library): what one SIMD of an MI355X needs for the
// instructions of one KV block of the FP8 attention loop, added up one kind at a time.
//
// One "group" is one matrix instruction (v_mfma_f32_32x32x64_f8f6f4) followed by one eighth of the vector work the kernel
// does per KV block and wavefront of 32 query rows: 4 v_exp_f32, 4 v_fma_f32, 4 v_add_f32, 6 v_mul_f32 (the rescale of O in
// 3 of 4 blocks), 2 v_max3_f32, 2 v_cvt_pk_fp8_f32.  Eight groups are one KV block.  Every instruction is independent of its
// neighbours, so the figures are what the issue ports allow, not what a dependency chain costs.  To that the probe adds what
// the loop needs besides: the 24 LDS operand reads of a block (8 ds_read_b128 for K, 16 ds_read_b64_tr_b8 for V^T) feeding the
// matrix instructions, the 4 HBM -> LDS tile-copy loads of a wavefront (buffer_load_dwordx4 ... lds from an L2-resident
// buffer), one workgroup barrier per block.  768 workgroups of 4 wavefronts with 48 KB of LDS each: three per CU, three
// wavefronts per SIMD, the occupancy of the kernel.  The "wide" rows are the same work laid out as 64 query rows per
// wavefront (16 groups share the LDS reads, copies and barrier of one block; 512 workgroups, two wavefronts per SIMD).
// Operands are constants: the shader clock stays near 2.4 GHz here, the attention kernel itself runs power-limited near
// 2.05 GHz on random data, so compare cycles, not nanoseconds.
// Output: one JSON line per row: nanoseconds per KV block and wavefront slot of 32 query rows (HIP events over the launch),
// shader clock (s_memtime against the 100 MHz s_memrealtime inside the kernel) and the cycles that follow.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#define CK(x)                                                                  \
  do {                                                                         \
    hipError_t e = (x);                                                        \
    if (e != hipSuccess) {                                                     \
      printf("HIP error %s at line %d\n", hipGetErrorString(e), __LINE__);     \
      return 1;                                                                \
    }                                                                          \
  } while (0)
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))
#define VALU_CHUNK                                                                                                                          \
  asm volatile("v_exp_f32 %0, %0\n v_exp_f32 %1, %1\n v_exp_f32 %2, %2\n v_exp_f32 %3, %3" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3])); \
  asm volatile("v_fma_f32 %0, %0, %4, %4\n v_fma_f32 %1, %1, %4, %4\n v_fma_f32 %2, %2, %4, %4\n v_fma_f32 %3, %3, %4, %4"                   \
               : "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]) : "v"(q[0]));                                                              \
  asm volatile("v_add_f32 %0, %0, %4\n v_add_f32 %1, %1, %4\n v_add_f32 %2, %2, %4\n v_add_f32 %3, %3, %4"                                   \
               : "+v"(r[8]), "+v"(r[9]), "+v"(r[10]), "+v"(r[11]) : "v"(q[1]));                                                            \
  asm volatile("v_mul_f32 %0, %0, %4\n v_mul_f32 %1, %1, %4\n v_mul_f32 %2, %2, %4\n v_mul_f32 %3, %3, %4"                                   \
               : "+v"(r[12]), "+v"(r[13]), "+v"(r[14]), "+v"(r[15]) : "v"(q[2]));                                                          \
  asm volatile("v_mul_f32 %0, %0, %2\n v_mul_f32 %1, %1, %2" : "+v"(r[16]), "+v"(r[17]) : "v"(q[2]));                                       \
  asm volatile("v_max3_f32 %0, %0, %2, %3\n v_max3_f32 %1, %1, %2, %3" : "+v"(r[18]), "+v"(r[19]) : "v"(q[3]), "v"(q[4]));                  \
  asm volatile("v_cvt_pk_fp8_f32 %0, %2, %3\n v_cvt_pk_fp8_f32 %1, %3, %2" : "+v"(p[0]), "+v"(p[1]) : "v"(q[5]), "v"(q[6]));

enum { kValu = 1, kMfma = 2, kLdsReads = 4, kCopies = 8, kBarrier = 16 };

// WIDE 0: 32 query rows per wavefront (8 groups per block).  1: 64 rows, the V^T fragments shared by the two halves, the K
// fragments read per half (32 LDS reads per 16 groups).  2: 64 rows, no fragment shared (48 reads).
template <int FLAGS, int WIDE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WIDE ? 2 : 3))) void mix_kernel(float* out, const uint8_t* src,
                                                                                                      int iters, long long* clk) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[(WIDE ? 72 : 48) * 1024];
  float r[20], q[8];
  int p[2] = {0, 0};
  for (int i = 0; i < 20; ++i) r[i] = 0.001f * (threadIdx.x + i);
  for (int i = 0; i < 8; ++i) q[i] = 1.0f + 0.01f * i;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  for (int i = threadIdx.x; i < 48 * 1024 / 4; i += 256) ((int*)lds)[i] = i;
  __syncthreads();
  v8i a = {1, 2, 3, 4, 5, 6, 7, (int)threadIdx.x}, b = {7, 6, 5, 4, 3, 2, 1, (int)threadIdx.x};
  v16f acc[4];
  for (int t = 0; t < 4; ++t)
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
  // conflict-free addresses: lane l reads the 16 bytes at 16 l; the transposing read takes row (l % 16) / 2 of 128-byte rows
  const int off128 = lane * 16;
  const int tr_j = (lane & 15) >> 1, tr_e = lane & 1, tr_g = lane >> 4;
  const int offtr = tr_j * 128 + (((tr_g * 2) ^ tr_j) << 4) + 8 * tr_e;
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, 1 << 20, 0x00020000);
  const unsigned voff = (wave * 64 + lane) * 16;
  const long long t0 = clock64();
  const long long w0 = wall_clock64();
  v8i fr[2] = {a, a};
  for (int it = 0; it < iters; ++it) {
    if (FLAGS & kCopies) {
      const int soff = (it & 63) * 8192;  // 512 KB of source, shared by all workgroups: L2 hits
#pragma unroll
      for (int pz = 0; pz < 4; ++pz)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, LDS_PTR(void, lds + 32768 + pz * 4096 + wave * 1024), 16, voff, soff + pz * 4096, 0, 0);
    }
#pragma unroll
    for (int gg = 0; gg < (WIDE ? 16 : 8); ++gg) {
      const int g = WIDE ? gg >> 1 : gg;
      v8i nxt = a;
      if ((FLAGS & kLdsReads) && (!WIDE || WIDE == 2 || (gg & 1) == 0 || g >= 4)) {
        const uint8_t* base = lds + (g & 3) * 8192;
        if (g < 4) {
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            const v2i d = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, base + offtr + x * 1024));
            nxt[2 * x] = d[0];
            nxt[2 * x + 1] = d[1];
          }
        } else {
          const v4i lo = *LDS_PTR(const v4i, base + off128);
          const v4i hi = *LDS_PTR(const v4i, base + off128 + 1024);
          nxt = v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
      }
      if (FLAGS & kMfma)
        acc[gg & 3] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4((FLAGS & kLdsReads) ? fr[gg & 1] : a, b, acc[gg & 3], 0, 0, 0, 0, 0, 0);
      if (FLAGS & kLdsReads) fr[gg & 1] = nxt;  // consumed two groups later
      __builtin_amdgcn_sched_barrier(0);
      if (FLAGS & kValu) { VALU_CHUNK }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (FLAGS & kCopies) __builtin_amdgcn_s_waitcnt(0x0F70 | 4);  // the copies of the previous iteration have landed
    if (FLAGS & kBarrier) __builtin_amdgcn_s_barrier();
  }
  const long long t1 = clock64();
  const long long w1 = wall_clock64();
  __builtin_amdgcn_s_waitcnt(0x0F70);
  float s = 0;
  for (int i = 0; i < 20; ++i) s += r[i];
  s += p[0] + p[1];
  for (int t = 0; t < 4; ++t)
    for (int i = 0; i < 16; ++i) s += acc[t][i];
  for (int i = 0; i < 8; ++i) s += fr[0][i] + fr[1][i];
  if (s == 1.2345f) out[0] = s;
  if (blockIdx.x == 100 && threadIdx.x == 0) {
    clk[0] = t1 - t0;
    clk[1] = w1 - w0;
  }
}


// The matrix pipe alone: every wavefront issues v_mfma_f32_32x32x64_f8f6f4 back to back (four accumulators, four A and four B
// fragments in registers, three wavefronts per SIMD), once on constant operands and once on operands that differ from lane to lane
// and from instruction to instruction (e4m3 codes of random sign and mantissa with exponents spread over five binades, the spread
// of N(0,1) draws): what the board delivers under its power limit when nothing but the matrix pipe works.
template <int RANDOM>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3))) void mfma_alone_kernel(float* out, int iters, long long* clk) {
  v8i a[4], b[4];
  unsigned x = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
  for (int f = 0; f < 4; ++f)
    for (int i = 0; i < 8; ++i) {
      unsigned wa = 0, wb = 0;
      for (int byte = 0; byte < 4; ++byte) {
        x ^= x << 13, x ^= x >> 17, x ^= x << 5;
        const unsigned ca = RANDOM ? ((x & 0x80u) | ((4u + (x >> 8) % 5u) << 3) | ((x >> 16) & 7u)) : 0x38u;   // 0x38 = 1.0
        const unsigned cb = RANDOM ? (((x >> 1) & 0x80u) | ((4u + (x >> 12) % 5u) << 3) | ((x >> 20) & 7u)) : 0x38u;
        wa |= ca << (8 * byte);
        wb |= cb << (8 * byte);
      }
      a[f][i] = (int)wa;
      b[f][i] = (int)wb;
    }
  v16f acc[4];
  for (int t = 0; t < 4; ++t)
    for (int i = 0; i < 16; ++i) acc[t][i] = 0.f;
  const long long t0 = clock64();
  const long long w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int g = 0; g < 8; ++g)
      acc[g & 3] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[g & 3], b[(g + (g >> 2)) & 3], acc[g & 3], 0, 0, 0, 0, 0, 0);
  }
  const long long t1 = clock64();
  const long long w1 = wall_clock64();
  float s = 0;
  for (int t = 0; t < 4; ++t)
    for (int i = 0; i < 16; ++i) s += acc[t][i];
  if (s == 1.2345f) out[0] = s;
  if (blockIdx.x == 100 && threadIdx.x == 0) {
    clk[0] = t1 - t0;
    clk[1] = w1 - w0;
  }
}

template <int RANDOM>
int run_mfma_alone(const char* name, float* dout, long long* dclk) {
  const int iters = 40000, grid = 768;
  float ms = 0;
  long long hclk[2] = {0, 1};
  for (int rep = 0; rep < 3; ++rep) {  // the last of three launches: the clock has settled under the load by then
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL((mfma_alone_kernel<RANDOM>), dim3(grid), dim3(256), 0, 0, dout, iters, dclk);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    CK(hipEventElapsedTime(&ms, e0, e1));
    CK(hipMemcpy(hclk, dclk, 16, hipMemcpyDeviceToHost));
  }
  const double flop = (double)grid * 4 * iters * 8 * 2.0 * 32 * 32 * 64;
  const double ghz = (double)hclk[0] / ((double)hclk[1] * 10.0);
  printf("{\"mix\": \"%s\", \"wavefronts_per_simd\": 3, \"launch_ms\": %.2f, \"tflops\": %.0f, \"sclk_ghz\": %.2f, "
         "\"pct_of_5_pflops\": %.1f}\n", name, ms, flop / (ms * 1e-3) / 1e12, ghz, flop / (ms * 1e-3) / 5.0e15 * 100);
  fflush(stdout);
  return 0;
}

template <int FLAGS, int WIDE>
int run(const char* name, float* dout, const uint8_t* src, long long* dclk) {
  const int iters = 3000;
  const int grid = WIDE ? 512 : 768, waves = WIDE ? 2 : 3, blocks_per_iter = WIDE ? 2 : 1;
  float best = 1e9;
  long long hclk[2] = {0, 1};
  for (int rep = 0; rep < 3; ++rep) {
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL((mix_kernel<FLAGS, WIDE>), dim3(grid), dim3(256), 0, 0, dout, src, iters, dclk);
    CK(hipEventRecord(e1));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    if (rep && ms < best) {
      best = ms;
      CK(hipMemcpy(hclk, dclk, 16, hipMemcpyDeviceToHost));
    }
  }
  const double ns = best * 1e6 / iters / (waves * blocks_per_iter);
  const double ghz = (double)hclk[0] / ((double)hclk[1] * 10.0);
  printf("{\"mix\": \"%s\", \"query_rows_per_wavefront\": %d, \"wavefronts_per_simd\": %d, \"ns_per_block_and_32_rows\": %.1f, "
         "\"sclk_ghz\": %.2f, \"cycles_per_block_and_32_rows\": %.0f, \"headline_launch_us\": %.1f}\n",
         name, WIDE ? 64 : 32, waves, ns, ghz, ns * ghz, ns * 512 / 1e3);
  fflush(stdout);
  return 0;
}

int main() {
  float* dout;
  CK(hipMalloc(&dout, 64));
  uint8_t* src;
  CK(hipMalloc(&src, 1 << 20));
  CK(hipMemset(src, 1, 1 << 20));
  long long* dclk;
  CK(hipMalloc(&dclk, 16));
  run<kValu, 0>("vector work", dout, src, dclk);
  run<kMfma, 0>("8 matrix instructions", dout, src, dclk);
  run<kValu | kMfma, 0>("vector + matrix", dout, src, dclk);
  run<kValu | kMfma | kLdsReads, 0>("vector + matrix + LDS operand reads", dout, src, dclk);
  run<kValu | kMfma | kCopies, 0>("vector + matrix + tile copies", dout, src, dclk);
  run<kValu | kMfma | kBarrier, 0>("vector + matrix + barrier", dout, src, dclk);
  run<kValu | kMfma | kLdsReads | kCopies | kBarrier, 0>("everything", dout, src, dclk);
  run<kValu | kMfma, 1>("wide: vector + matrix", dout, src, dclk);
  run<kValu | kMfma | kLdsReads | kCopies | kBarrier, 1>("wide: everything, V^T fragments shared", dout, src, dclk);
  run<kValu | kMfma | kLdsReads | kCopies | kBarrier, 2>("wide: everything, no fragment shared", dout, src, dclk);
  run_mfma_alone<0>("matrix pipe alone, constant operands", dout, dclk);
  run_mfma_alone<1>("matrix pipe alone, random operands", dout, dclk);
  return 0;
}
