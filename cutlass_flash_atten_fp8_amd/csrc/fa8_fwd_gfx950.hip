// FP8 flash-attention forward for gfx950 (MI355X): kernels and the C-ABI launcher (libfa8.so).
//
// One workgroup = 4 wavefronts = 128 query rows of one (batch, head); every wavefront owns 32 query
// rows and the whole head dimension (a multiple of 32 up to 256: the bucket sizes of the reference's
// dispatch, csrc/static_switch.h:50-77).  KV is walked in ascending blocks of 64 rows, the block size
// the reference instantiates (kBlockM = kBlockN = 64, reference csrc/flash_attention.cu:624), so the
// running max that P is quantised against evolves exactly as in the reference loop
// (csrc/flash_attention.cu:468-534).
//
// Formulation (different from the reference, which computes S = Q K^T with m16n8k32 atoms,
// csrc/mma_sm89.hpp:10-35):
//   * S^T = K Q^T with v_mfma_f32_32x32x64_f8f6f4 (A = K tile from LDS, B = Q held in registers).
//     In the 32x32 accumulator layout a lane owns ONE query column and 16 kv rows, so the online
//     softmax row max / row sum (reference csrc/utils.h:22-98 quad butterflies) are in-register
//     reductions plus one v_permlane32_swap.
//   * O^T = V^T P^T with the same instruction (A = V^T, B = P^T).  The fp32 -> fp8 P registers of a
//     lane already are a valid B operand when the K tile rows are stored in LDS in a permuted order
//     (kv_of_lds_row below); this replaces the reference's accumulator-to-A-operand reshuffle
//     (csrc/reg2reg.h:31-96).  V^T fragments come from the row-major V tile in LDS through the
//     transposing LDS read ds_read_b64_tr_b8, so V is consumed as [B,H,N,d] with no extra pass.
//   * K and V tiles go HBM -> LDS with buffer_load_dwordx4 ... lds (no register staging), two or three
//     stages, one barrier per KV block; 16-byte chunks are XOR-swizzled against bank conflicts,
//     the swizzle being applied on the global-address side of the copy.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <type_traits>

#include "fa8_api.h"

// wavefronts per SIMD the kernels are compiled for: 3 (at most 168 VGPRs per lane) up to head dim 128, 2 (256 VGPRs:
// the output accumulators alone take 128) for head dim 256; the pipelined loop 2; the dense loop 3 (head dim 64: 4)
#define FA8_WAVES_PER_EU(D, LOOP) ((LOOP) == 1 ? 2 : ((LOOP) == 2 ? ((D) == 64 ? 4 : 3) : ((D) > 128 ? 2 : 3)))

namespace {

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))
#define GLOBAL_PTR(T, p) ((__attribute__((address_space(1))) T*)(p))

constexpr int kQBlock = 128;   // query rows per workgroup
constexpr int kQWave = 32;     // query rows per wavefront
constexpr int kKvBlock = 64;   // kv rows per online-softmax step
constexpr int kThreads = 256;  // 4 wavefronts
constexpr int kVersion = 4;
// main loops (template parameter LOOP of the kernel)
constexpr int kLoopRolling = 0, kLoopPipelined = 1, kLoopDense = 2;

struct KernelArgs {
  const uint8_t* q;
  const uint8_t* k;
  const uint8_t* v;
  void* o;
  float* lse;  // optional
  int heads, seqlen_q, seqlen_k, n_qblocks, bh_total;
  int kv_group;      // q heads per k/v head
  int interleave;    // causal: how many heads deal their q blocks alternately (see decode_block)
  int causal_shift;  // key j is visible to query i when j <= i + causal_shift
  float scale_log2;  // softmax_scale * log2(e)
  long long q_bs, q_hs, q_rs;
  long long k_bs, k_hs, k_rs;
  long long v_bs, v_hs, v_rs;
  long long o_bs, o_hs, o_rs;
  long long lse_bs, lse_hs;
};

// LDS row r (0..63) of a K tile holds kv row kv_of_lds_row(r) of the block.  With this order the 16
// accumulator registers a lane gets from S^T sub-tile t (rows 8a+4h+b of the 32x32 result, h = lane/32)
// are kv rows 32h+16t+(4a+b): exactly the bytes 16t..16t+15 of the lane's B operand in the PV MFMA.
__device__ __forceinline__ int kv_of_lds_row(int r) {
  const int t = r >> 5, a = (r >> 3) & 3, h = (r >> 2) & 1, b = r & 3;
  return 32 * h + 16 * t + 4 * a + b;
}

// Swizzle: a tile is an array of 128-byte lines of eight 16-byte chunks.  A row of D bytes is two lines (D = 256),
// one line (128), half a line (64) or a quarter (32).  The chunk position inside its line is XORed with a key
// taken from the row (line) number, chosen so that the eight lanes the LDS serves together (eight consecutive
// rows, same chunk) fall on eight different positions, for the K reads and for the transposing V reads alike.
template <int D, bool IS_V>
__device__ __forceinline__ int tile_offset(int row, int chunk) {
  if constexpr (D == 256) {
    const int key = IS_V ? (row & 7) : ((row & 7) ^ ((row >> 3) & 1));
    return row * 256 + ((chunk >> 3) << 7) + (((chunk & 7) ^ key) << 4);
  } else if constexpr (D == 128) {
    const int key = IS_V ? (row & 7) : ((row & 7) ^ ((row >> 3) & 1));
    return row * 128 + ((chunk ^ key) << 4);
  } else if constexpr (D == 64) {
    const int line = row >> 1;
    const int key = IS_V ? (line & 3) : ((line & 3) ^ ((line >> 2) & 1));
    return line * 128 + ((((row & 1) << 2) | (chunk ^ key)) << 4);
  } else {
    static_assert(D == 32, "head dims: 32, 64, 128, 256");
    const int line = row >> 2;
    return line * 128 + ((((row & 3) << 1) | (chunk ^ (line & 1))) << 4);
  }
}

// Inverse of tile_offset for the copy engine: which (row, chunk) lives at 16-byte slot `slot`.
template <int D, bool IS_V>
__device__ __forceinline__ void tile_slot_decode(int slot, int& row, int& chunk) {
  if constexpr (D == 256) {
    row = slot >> 4;
    const int key = IS_V ? (row & 7) : ((row & 7) ^ ((row >> 3) & 1));
    chunk = (slot & 8) | ((slot & 7) ^ key);
  } else if constexpr (D == 128) {
    row = slot >> 3;
    const int key = IS_V ? (row & 7) : ((row & 7) ^ ((row >> 3) & 1));
    chunk = (slot & 7) ^ key;
  } else if constexpr (D == 64) {
    const int line = slot >> 3, w = slot & 7;
    const int key = IS_V ? (line & 3) : ((line & 3) ^ ((line >> 2) & 1));
    row = line * 2 + (w >> 2);
    chunk = (w & 3) ^ key;
  } else {
    const int line = slot >> 3, w = slot & 7;
    row = line * 4 + (w >> 1);
    chunk = (w & 1) ^ (line & 1);
  }
}

// v_permlane32_swap exchanges lanes 32-63 of its first operand with lanes 0-31 of its second.  Fed the same
// value x twice it returns {x of the low half-lane, x of the high half-lane} in every lane of a query.
typedef unsigned v2u __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float lane32_max(float x) {
  const v2u r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  // median(a, b, +inf) = max(a, b) in one instruction (fmaxf would first quiet both operands); the +inf is made opaque to
  // the optimiser, which would otherwise turn the median back into that max
  float inf = INFINITY;
  asm("" : "+v"(inf));
  return __builtin_amdgcn_fmed3f(__uint_as_float(r[0]), __uint_as_float(r[1]), inf);
}
__device__ __forceinline__ float lane32_sum(float x) {
  const v2u r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// max of three floats; the compiler fuses the pair into one v_max3_f32.
__device__ __forceinline__ float max3(float a, float b, float c) { return __builtin_fmaxf(__builtin_fmaxf(a, b), c); }

template <bool E5M2>
__device__ __forceinline__ v16f mfma_fp8(const v8i& a, const v8i& b, const v16f& c) {
  if constexpr (E5M2)
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 1, 1, 0, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, 0, 0, 0, 0, 0, 0);
}

template <bool E5M2>
__device__ __forceinline__ int pack4_fp8(float a, float b, float c, float d) {
  int r;
  asm volatile("" : "=v"(r));  // any value will do (both 16-bit halves are overwritten below): defines r, emits nothing
  if constexpr (E5M2) {
    r = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, r, false);
    r = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, r, true);
  } else {
    r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, r, false);
    r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
  }
  return r;
}

// Workgroup id -> (batch*head, q block).  Workgroups are dealt to the 8 XCDs round-robin by id; when
// batch*heads is a multiple of 8 all q blocks of one head are kept on one XCD so its K/V stay in that
// XCD's L2.  Workgroups start in id order.  Full attention: head after head.  Causal: workgroups differ in length
// (q block i walks i+1 of the n q blocks' worth of keys), so the longest come first and `interleave` heads of the XCD
// take turns at every q block: the workgroups that run side by side then have about the same length and the
// short ones fill the end of the launch (head after head, a late head's longest workgroup would start when the
// rest of the chip is already draining).
template <bool CAUSAL>
__device__ __forceinline__ void decode_block(const KernelArgs& a, int id, int& bh, int& qb) {
  int qi;
  if ((a.bh_total & 7) == 0) {
    const int xcd = id & 7, s = id >> 3;
    int hl;  // head index inside this XCD's share of bh_total / 8 heads
    if (CAUSAL) {
      // groups of `interleave` heads (the last group takes what is left)
      const int per_group = a.interleave * a.n_qblocks;
      const int grp = s / per_group, r = s - grp * per_group;
      const int g = min(a.interleave, (a.bh_total >> 3) - grp * a.interleave);
      qi = r / g;
      hl = grp * a.interleave + (r - qi * g);
    } else {
      hl = s / a.n_qblocks;
      qi = s - hl * a.n_qblocks;
    }
    // grouped-query attention: an XCD takes a contiguous range of q heads, so the heads that share a k/v head follow
    // each other on one XCD
    bh = a.kv_group > 1 ? xcd * (a.bh_total >> 3) + hl : hl * 8 + xcd;
  } else if (CAUSAL) {
    qi = id / a.bh_total;  // no head stays on one XCD anyway: all heads take turns
    bh = id - qi * a.bh_total;
  } else {
    bh = id / a.n_qblocks;
    qi = id - bh * a.n_qblocks;
  }
  qb = CAUSAL ? (a.n_qblocks - 1 - qi) : qi;
}

// LOOP selects the main loop; all three perform the same arithmetic in the same order, their results are bitwise equal.
// kLoopRolling: one KV block after the other (S^T, softmax, PV), three wavefronts per SIMD hide each other's latencies.
// kLoopPipelined: software-pipelined for launches that leave a SIMD with two wavefronts or fewer (short sequences, few
// heads): the matrix instructions of the neighbouring blocks (PV of block j-1, S^T of block j+1) are issued between the
// chunks of the softmax of block j, so that one wavefront alone keeps the matrix and the vector pipe busy; about 180
// VGPRs (two wavefronts per SIMD), four LDS stages; every block may be masked.
// kLoopDense: the same pipeline squeezed into 168 VGPRs (three wavefronts per SIMD, three LDS stages) for launches
// in which no block needs a mask (full attention over a whole number of KV blocks): one logits buffer, whose halves are
// refilled by the S^T products of block j+1 as soon as the softmax of block j has turned them into weights.
template <int D, bool CAUSAL, bool E5M2, int OUT, bool VT, int LOOP>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(FA8_WAVES_PER_EU(D, LOOP)))) void fa8_fwd_kernel(
    const KernelArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses device-only types (buffer resources); the host pass only needs the stub
  static_assert(D % 32 == 0 && D >= 32 && D <= 256, "head dims: multiples of 32 up to 256");
  constexpr bool PIPE = LOOP == kLoopPipelined, DENSE = LOOP == kLoopDense;
  static_assert(LOOP == kLoopRolling || D == 64 || D == 128, "the pipelined loops are built for head dims 64 and 128");
  static_assert(!DENSE || !CAUSAL, "the dense loop has no masks");
  // LDS tiles are laid out for the next power of two: rows of DP bytes, of which the first D are used
  constexpr int DP = D <= 32 ? 32 : (D <= 64 ? 64 : (D <= 128 ? 128 : 256));
  constexpr int kTileBytes = kKvBlock * DP;  // one K or V tile
  // copy passes per tile: one pass is 256 lanes x 16 bytes.  A 32-wide tile is half a pass: there wavefronts 0-1 copy
  // K and wavefronts 2-3 copy V in one common pass.
  constexpr bool kSplitPass = kTileBytes < kThreads * 16;
  constexpr int kPasses = kSplitPass ? 1 : kTileBytes / (kThreads * 16);
  constexpr int kKSteps = (D + 63) / 64;  // MFMA k-steps over the head dim for S^T (D % 64 == 32: the last one is half zeros)
  constexpr int kMTiles = D / 32;         // 32-row tiles of O^T
  // LDS stages per operand: three (copies issued two KV blocks ahead) where three workgroups then still fit in the
  // 160 KB of a CU, two for head dims above 128 (2 x 32 KB per workgroup, two workgroups per CU)
  // (the pipelined loop: four, copies issued up to four blocks ahead; the dense loop: three)
  constexpr int kStages = PIPE ? 4 : (D > 128 ? 2 : 3);
  // One LDS object per (stage, operand): the compiler then knows that the asynchronous HBM -> LDS copy into one
  // stage cannot alias the reads of the other stage and does not wait for the copy before those reads.
  __shared__ __attribute__((aligned(1024))) uint8_t k_lds0[kTileBytes];
  __shared__ __attribute__((aligned(1024))) uint8_t k_lds1[kTileBytes];
  __shared__ __attribute__((aligned(1024))) uint8_t k_lds2[kStages >= 3 ? kTileBytes : 16];
  __shared__ __attribute__((aligned(1024))) uint8_t k_lds3[kStages >= 4 ? kTileBytes : 16];
  __shared__ __attribute__((aligned(1024))) uint8_t v_lds0[kTileBytes];
  __shared__ __attribute__((aligned(1024))) uint8_t v_lds1[kTileBytes];
  __shared__ __attribute__((aligned(1024))) uint8_t v_lds2[kStages >= 3 ? kTileBytes : 16];
  __shared__ __attribute__((aligned(1024))) uint8_t v_lds3[kStages >= 4 ? kTileBytes : 16];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keep it (and all it feeds) in scalar registers
  const int qn = lane & 31, h = lane >> 5;

  int bh, qb;
  decode_block<CAUSAL>(a, blockIdx.x, bh, qb);
  const int b = bh / a.heads, hd = bh - b * a.heads;
  const int q0 = qb * kQBlock;
  const int q_wave0 = q0 + wave * kQWave;
  const int q_row = q_wave0 + qn;  // this lane's query row
  const uint8_t* qp = a.q + b * a.q_bs + hd * a.q_hs;
  const int hd_kv = a.kv_group == 1 ? hd : hd / a.kv_group;  // grouped-query attention: several q heads per k/v head
  const uint8_t* kp = a.k + b * a.k_bs + hd_kv * a.k_hs;
  const uint8_t* vp = a.v + b * a.v_bs + hd_kv * a.v_hs;
  const float c = a.scale_log2;

  // ---- Q fragment (B operand of S^T = K Q^T): row q_row, bytes [64ks + 32h, +32) ----
  // (D % 64 == 32: the upper half of the last k-step does not exist; those lanes hold zeros and load nothing)
  v8i qf[kKSteps];
  {
    const int qr = min(q_row, a.seqlen_q - 1);
    const uint8_t* src = qp + (long long)qr * a.q_rs;
#pragma unroll
    for (int ks = 0; ks < kKSteps; ++ks) {
      const bool upper_exists = 64 * ks + 32 < D;
      const uint8_t* s8 = src + 64 * ks + (upper_exists ? 32 * h : 0);
      const v4i lo = *(const v4i*)(s8);
      const v4i hi = *(const v4i*)(s8 + 16);
      qf[ks] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      if (!upper_exists && h) qf[ks] = v8i{0, 0, 0, 0, 0, 0, 0, 0};
    }
  }

  // ---- HBM -> LDS copy: buffer_load_dwordx4 ... lds ----
  // In pass p wavefront w fills LDS bytes [(4p+w)*1024, +1024) of the tile, lane l the 16 bytes at +16l; which
  // (kv row, 16-byte chunk) belongs there follows from the swizzle.  (A 32-wide tile is 2 KB: wavefronts 0-1 fill the K
  // tile, wavefronts 2-3 the V tile.)  The source address is the head's base (buffer resource) + a per-lane byte
  // offset that never changes (VGPR) + the block's byte offset (SGPR): no vector ALU work per block.  The resource
  // ends with the last kv row, so rows past the end of a ragged last block read 0.  LDS chunks that lie past the
  // head dim (D < DP) get an offset beyond any resource and read 0 as well: the K fragments of a half k-step rely on it.
  constexpr unsigned kNoSource = 0x80000000u;
  auto copy_segment = [&](int p) __attribute__((always_inline)) { return kSplitPass ? (wave & 1) : (p * 4 + wave); };
  unsigned k_src[kPasses], v_src[kPasses];
#pragma unroll
  for (int p = 0; p < kPasses; ++p) {
    const int slot = copy_segment(p) * 64 + lane;
    int r, ch;
    tile_slot_decode<DP, false>(slot, r, ch);
    k_src[p] = ch * 16 < D ? (unsigned)(kv_of_lds_row(r) * (int)a.k_rs + ch * 16) : kNoSource;
    if constexpr (VT) {
      // v is [d, Nk]: the tile is D rows of 64 kv bytes (4 chunks), laid out like a 64-byte-row K tile
      tile_slot_decode<64, false>(slot, r, ch);
      v_src[p] = r < D ? (unsigned)(r * (int)a.v_rs + ch * 16) : kNoSource;
    } else {
      tile_slot_decode<DP, true>(slot, r, ch);
      v_src[p] = ch * 16 < D ? (unsigned)(r * (int)a.v_rs + ch * 16) : kNoSource;
    }
  }
  const int kv_last = a.seqlen_k - 1;
  constexpr int kRsrcFlags = 0x00020000;  // raw buffer, 32-bit data format
  // Start the asynchronous copy of the K rows / the V rows of KV block j into the LDS buffer kb / vb.  The pipelined loops
  // start two tile copies in every step, also when the block no longer exists (so that one s_waitcnt constant fits every
  // step): such a copy (exists = false, wave-uniform) goes through a resource of length 0, every lane of it is out of range,
  // zeros land in LDS and no memory is touched.
  // (Dense loop: the second pass of a copy differs from the first by a whole number of rows, 16 kv rows of K and 32 (64) rows
  // of V (V^T): the difference sits in the scalar offset and both passes share one vector register.)
  const int k_bytes = (int)(kv_last * a.k_rs + D);
  const int v_bytes = VT ? (int)((D - 1) * a.v_rs + a.seqlen_k) : (int)(kv_last * a.v_rs + D);
  auto issue_k = [&](int j, uint8_t* kb, bool exists) __attribute__((always_inline)) {
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)kp, 0, exists ? k_bytes : 0, kRsrcFlags);
    const int k_base = (int)((unsigned)j * kKvBlock * (unsigned)a.k_rs);  // below 2^32 (fa8_fwd_validate)
#pragma unroll
    for (int p = 0; p < kPasses; ++p)
      if (!kSplitPass || wave < 2)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, LDS_PTR(void, kb + copy_segment(p) * 1024), 16, DENSE ? k_src[0] : k_src[p],
                                                 DENSE ? k_base + p * 16 * (int)a.k_rs : k_base, 0, 0);
  };
  auto issue_v = [&](int j, uint8_t* vb, bool exists) __attribute__((always_inline)) {
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)vp, 0, exists ? v_bytes : 0, kRsrcFlags);
    const int v_base = VT ? j * kKvBlock : (int)((unsigned)j * kKvBlock * (unsigned)a.v_rs);
    // transposed v, ragged last block: the 16-byte chunks past the last kv column would read the start of the next
    // head-dim row (or run off the tensor); they are pulled back onto the last chunk instead (and masked later)
    const bool v_clamp = VT && (j + 1) * kKvBlock > a.seqlen_k;
#pragma unroll
    for (int p = 0; p < kPasses; ++p) {
      const int seg = copy_segment(p) * 1024;
      if (!kSplitPass || wave >= 2) {
        if (v_clamp) {
          int r, ch;
          tile_slot_decode<64, false>(copy_segment(p) * 64 + lane, r, ch);
          const unsigned off = r < D ? (unsigned)(r * (int)a.v_rs + min(v_base + ch * 16, a.seqlen_k - 16)) : kNoSource;
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, LDS_PTR(void, vb + seg), 16, off, 0, 0, 0);
        } else {
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, LDS_PTR(void, vb + seg), 16, DENSE ? v_src[0] : v_src[p],
                                                   DENSE ? v_base + p * (VT ? 64 : 32) * (int)a.v_rs : v_base, 0, 0);
        }
      }
    }
  };
  auto issue_tile = [&](int j, uint8_t* kb, uint8_t* vb) __attribute__((always_inline)) {
    issue_k(j, kb, true);
    issue_v(j, vb, true);
  };

  // ---- per-lane LDS read offsets ----
  // K fragment (A operand of S^T): the lane's row inside the 32-row MFMA tile is lane % 32 and its k-group
  // lane / 32: chunks 4ks+2h and 4ks+2h+1 of LDS row 32t + lane % 32.  (Head dim 32: both k-groups read chunks 0
  // and 1; the upper group meets the zeros of the Q fragment.  Head dims 96, 160, 224: the upper group of the last
  // k-step reads zero-filled chunks.)
  int k_off[kKSteps][2];
#pragma unroll
  for (int ks = 0; ks < kKSteps; ++ks)
#pragma unroll
    for (int e = 0; e < 2; ++e) k_off[ks][e] = tile_offset<DP, false>(qn, DP >= 64 ? 4 * ks + 2 * h + e : e);
  constexpr int kSubTileStride = 32 * DP;  // LDS bytes between S^T sub-tiles (32 rows)
  // V^T fragment (A operand of O^T = V^T P^T) through ds_read_b64_tr_b8: inside a group of 16 lanes, lanes
  // 2j and 2j+1 address the two 8-byte halves of kv row j of an 8 x 16 byte block, and lane i receives
  // byte i of each of the 8 rows: 8 consecutive kv for one head-dim column.
  const int tr_j = (lane & 15) >> 1, tr_e = lane & 1, tr_g1 = (lane >> 4) & 1;
  // (transposed v: the tile already is V^T, [d][64 kv]: plain 16-byte reads of row 32mt + lane % 32, chunks 2h, 2h+1)
  int v_off[kMTiles], vt_off[2];
#pragma unroll
  for (int mt = 0; mt < kMTiles; ++mt) v_off[mt] = tile_offset<DP, true>(32 * h + tr_j, 2 * mt + tr_g1) + 8 * tr_e;
#pragma unroll
  for (int e = 0; e < 2; ++e) vt_off[e] = tile_offset<64, false>(qn, 2 * h + e);
  constexpr int kVtTileStride = 32 * 64;  // LDS bytes between 32-row groups of the [d][64] tile
  constexpr int kTrStride = 8 * DP;  // LDS bytes between successive groups of 8 kv rows

  // Causal: key j is visible to query i when j <= i + shift (shift 0: the reference's rule, csrc/flash_attention.cu:62-64;
  // shift = Nk - Nq aligns the diagonal with the bottom right corner).  At least block 0 is always walked (fully
  // masked if need be), so a query that sees no key ends with l = 0 and an all-zero output row.
  const int shift = CAUSAL ? a.causal_shift : 0;
  const int n_tiles = CAUSAL ? max(1, (min(a.seqlen_k, q0 + kQBlock + shift) + kKvBlock - 1) / kKvBlock)
                             : (a.seqlen_k + kKvBlock - 1) / kKvBlock;
  // Leading blocks that need no mask for any row of the workgroup: they end at or before the first query row's
  // last visible key (causal) and inside the kv range.  They are processed by the mask-free copy of the loop body.
  const int n_plain = (CAUSAL ? max(0, min(q0 + shift, a.seqlen_k)) : a.seqlen_k) / kKvBlock;

  v16f o_acc[kMTiles];
#pragma unroll
  for (int mt = 0; mt < kMTiles; ++mt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o_acc[mt][i] = 0.f;
  // running row max of raw S (both half-lanes of a query hold the same value).  The pipelined loop starts it at a finite value
  // below every possible logit (|s| <= 57344^2 * 256 < 1e12) instead of -inf: a row that has not seen a key yet then needs no
  // special case (its rescale factor exp2((m_run - m_new) * c) is 0 or multiplies zeros, m_new * c stays finite, and a masked
  // logit -inf still gives exp2(-inf) = 0 for the positive scales this loop runs with); the results are the same bit for bit.
  float m_run = PIPE ? -1.0e30f : -INFINITY;
  float l_run = 0.f;        // this lane's share of the running row sum

  // K fragment of S^T sub-tile t, k-step ks, and V^T fragment of O^T tile mt, from the tiles in kb / vb
  auto load_kf = [&](const uint8_t* kb, int t, int ks) __attribute__((always_inline)) {
    const v4i lo = *LDS_PTR(const v4i, kb + t * kSubTileStride + k_off[ks][0]);
    const v4i hi = *LDS_PTR(const v4i, kb + t * kSubTileStride + k_off[ks][1]);
    return v8i{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  };
  auto load_vf = [&](const uint8_t* vb, int mt) __attribute__((always_inline)) {
    v8i vf;
    if constexpr (VT) {
      const v4i lo = *LDS_PTR(const v4i, vb + mt * kVtTileStride + vt_off[0]);
      const v4i hi = *LDS_PTR(const v4i, vb + mt * kVtTileStride + vt_off[1]);
      vf = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    } else {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const v2i r = __builtin_amdgcn_ds_read_tr8_b64_v2i32(LDS_PTR(v2i, vb + v_off[mt] + g * kTrStride));
        vf[2 * g] = r[0];
        vf[2 * g + 1] = r[1];
      }
    }
    return vf;
  };

  // S^T, online softmax and PV for KV block j held in kb / vb.
  auto compute_tile = [&](int j, const uint8_t* kb, const uint8_t* vb, auto masked_c) __attribute__((always_inline)) {
    // kMasked also marks the general path (first block, diagonal, tail): only there can the running max still be -inf
    constexpr bool kMasked = decltype(masked_c)::value;
    const int kv0 = j * kKvBlock;
    // ---- S^T = K Q^T : two 32(kv) x 32(q) sub-tiles ----
    v16f s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[t][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) {
        s[t] = mfma_fp8<E5M2>(load_kf(kb, t, ks), qf[ks], s[t]);
      }
    }
    // ---- causal / tail mask: register i of sub-tile t is kv row kv0 + 32h + 16t + i ----
    const int kv_limit = CAUSAL ? min(q_row + shift, kv_last) : kv_last;  // last kv this query attends to
    if constexpr (kMasked) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (kv0 + 32 * h + 16 * t + i > kv_limit) s[t][i] = -INFINITY;
    }
    // ---- online softmax (reference softmax_rescale_o, csrc/flash_attention.cu:233-273) ----
    // 33 values (32 logits and the running max) in 16 three-input maxima: four independent chains over sub-tile 0
    // (it is ready first), then sub-tile 1
    float mx[4];
#pragma unroll
    for (int ch = 0; ch < 4; ++ch) mx[ch] = max3(s[0][4 * ch], s[0][4 * ch + 1], s[0][4 * ch + 2]);
#pragma unroll
    for (int ch = 0; ch < 4; ++ch) mx[ch] = max3(mx[ch], s[0][4 * ch + 3], s[1][4 * ch]);
#pragma unroll
    for (int ch = 0; ch < 4; ++ch) mx[ch] = max3(mx[ch], s[1][4 * ch + 1], s[1][4 * ch + 2]);
    const float m_new = lane32_max(max3(max3(mx[0], s[1][3], s[1][7]), max3(mx[1], s[1][11], s[1][15]), max3(mx[2], mx[3], m_run)));
    if (__any(m_new != m_run)) {
      float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c);
      if constexpr (kMasked) alpha = (m_run == -INFINITY) ? 0.f : alpha;
      l_run *= alpha;
      // only the lanes of the queries whose max moved multiply (the others would multiply by exactly 1): the instructions are
      // issued either way, but idle lanes draw no power, and this kernel runs at the board's power limit
      if (alpha != 1.f) {
#pragma unroll
        for (int mt = 0; mt < kMTiles; ++mt)
#pragma unroll
          for (int i = 0; i < 16; ++i) o_acc[mt][i] *= alpha;
      }
      m_run = m_new;
    }
    float mc = m_new * c;
    if constexpr (kMasked) mc = (m_new == -INFINITY) ? 0.f : mc;
    float sum0, sum1;  // row sum of this block in two chains, started from the first two weights
    v8i p8;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[t][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][i], c, -mc));
      if constexpr (kMasked) {
        // a masked logit is -inf; force its weight to 0 even when scale <= 0 would give NaN or 1
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (kv0 + 32 * h + 16 * t + i > kv_limit) s[t][i] = 0.f;
      }
#pragma unroll
      for (int i = 0; i < 16; i += 2) {
        sum0 = (t == 0 && i == 0) ? s[t][i] : sum0 + s[t][i];
        sum1 = (t == 0 && i == 0) ? s[t][i + 1] : sum1 + s[t][i + 1];
      }
#pragma unroll
      for (int w = 0; w < 4; ++w)
        p8[4 * t + w] = pack4_fp8<E5M2>(s[t][4 * w], s[t][4 * w + 1], s[t][4 * w + 2], s[t][4 * w + 3]);
    }
    l_run += sum0 + sum1;
    // ---- O^T += V^T P^T : the V^T fragment of tile mt+1 is fetched while the MFMA of tile mt runs ----
    v8i vf_cur = load_vf(vb, 0);
#pragma unroll
    for (int mt = 0; mt < kMTiles; ++mt) {
      v8i vf_next;
      if (mt + 1 < kMTiles) vf_next = load_vf(vb, mt + 1);
      o_acc[mt] = mfma_fp8<E5M2>(vf_cur, p8, o_acc[mt]);
      if (mt + 1 < kMTiles) vf_cur = vf_next;
    }
  };
  // Three LDS stages: copies issued two KV blocks ahead.  At the end of the step for block j the copy of block
  // j+1 (issued one step earlier) must have landed while the copy of block j+2 (issued in this step: kLoadsPerTile
  // loads per lane) may stay in flight; vmcnt counts this lane's loads in issue order.  The barrier then tells every
  // wavefront that all shares of block j+1 are in LDS and that block j's stage may be overwritten.  It is a bare
  // s_barrier: __syncthreads() would also wait for the copy that is meant to stay in flight.
  constexpr int kLoadsPerTile = kSplitPass ? 1 : 2 * kPasses;
  auto stage_sync = [&](bool next_in_flight) __attribute__((always_inline)) {
    // s_waitcnt immediate (gfx9 layout): vmcnt[3:0], expcnt[6:4] = 7 and lgkmcnt[11:8] = 15 (no wait on those)
    if (next_in_flight)
      __builtin_amdgcn_s_waitcnt(0x0F70 | kLoadsPerTile);
    else
      __builtin_amdgcn_s_waitcnt(0x0F70);
    __builtin_amdgcn_s_barrier();
  };
  static_assert(kLoadsPerTile < 16, "vmcnt immediate above");

  if constexpr (DENSE) {
    // ---- dense loop: the software pipeline in 168 VGPRs ----
    // Iteration j is the softmax of block j in 8 chunks of 4 weights.  In front of chunks 0-3 go the PV products of block j-1
    // (head dim 64: chunks 0 and 2), in front of chunks 4-5 the S^T products of sub-tile 0 of block j+1, written over sub-tile 0
    // of block j, which is all weights by then; the S^T products of sub-tile 1 follow the last chunk and run under the rescale
    // of O.  LDS operands are fetched one matrix instruction ahead.  K(t) and V(t) live in stage t % 3.  Step j starts the
    // copies of K(j+3) (its stage held K(j), last read in step j-1) and V(j+1) (its stage held V(j-2), last read in step j-1)
    // in front of chunks 1 and 2, reads K(j+1) and V(j-1), and ends when K(j+2) and V(j), started in step j-1, have landed.
    v16f s[2];
    v8i p8;
    constexpr int kPvEvery = 4 / kMTiles;  // the PV product of tile mt goes in front of chunk mt * kPvEvery
    constexpr int kSEvery = 2 / kKSteps;   // the S^T product (sub-tile 0, k-step ks) in front of chunk 4 + ks * kSEvery
    auto iteration = [&](auto first_c, int j, const uint8_t* kb_next, const uint8_t* vb_prev, uint8_t* k_dst, uint8_t* v_dst)
                         __attribute__((always_inline)) {
      constexpr bool kFirst = decltype(first_c)::value;
      v8i vfrag[kMTiles];
      v8i kfrag[2][kKSteps];
      if constexpr (!kFirst) vfrag[0] = load_vf(vb_prev, 0);
      float mx[4];
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) mx[ch] = max3(s[0][4 * ch], s[0][4 * ch + 1], s[0][4 * ch + 2]);
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) mx[ch] = max3(mx[ch], s[0][4 * ch + 3], s[1][4 * ch]);
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) mx[ch] = max3(mx[ch], s[1][4 * ch + 1], s[1][4 * ch + 2]);
      const float m_new = lane32_max(max3(max3(mx[0], s[1][3], s[1][7]), max3(mx[1], s[1][11], s[1][15]), max3(mx[2], mx[3], m_run)));
      bool changed = false;
      float alpha = 1.f;
      const float mc = m_new * c;
      if constexpr (kFirst) {
        m_run = m_new;  // O and l are still zero
      } else {
        changed = __any(m_new != m_run);
        if (changed) {
          alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c);
          l_run *= alpha;
          m_run = m_new;
        }
      }
      float sum0, sum1;
      v8i p8_cur;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (u == 1) issue_k(min(j + 3, n_tiles), k_dst, j + 3 < n_tiles);
        if (u == 2) issue_v(min(j + 1, n_tiles), v_dst, j + 1 < n_tiles);
        // LDS operands of the matrix instructions in front of the next chunk
        if constexpr (!kFirst) {
#pragma unroll
          for (int mt = 1; mt < kMTiles; ++mt)
            if (mt * kPvEvery - 1 == u) vfrag[mt] = load_vf(vb_prev, mt);
        }
#pragma unroll
        for (int ks = 0; ks < kKSteps; ++ks)
          if (4 + ks * kSEvery - 1 == u) kfrag[0][ks] = load_kf(kb_next, 0, ks);
        if (u >= 8 - kKSteps) kfrag[1][u - (8 - kKSteps)] = load_kf(kb_next, 1, u - (8 - kKSteps));
        // one matrix instruction in front of the chunk
        if (u < 4 && u % kPvEvery == 0) {
          if constexpr (!kFirst) o_acc[u / kPvEvery] = mfma_fp8<E5M2>(vfrag[u / kPvEvery], p8, o_acc[u / kPvEvery]);
        }
        if (u >= 4 && (u - 4) % kSEvery == 0 && (u - 4) / kSEvery < kKSteps) {
          // (after the last block this is the product of a stale tile: never used)
          const int ks = (u - 4) / kSEvery;
          if (ks == 0) {
            v16f z;
#pragma unroll
            for (int i = 0; i < 16; ++i) z[i] = 0.f;
            s[0] = mfma_fp8<E5M2>(kfrag[0][ks], qf[ks], z);
          } else {
            s[0] = mfma_fp8<E5M2>(kfrag[0][ks], qf[ks], s[0]);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        // chunk u of the softmax: weights 4w .. 4w+3 of sub-tile t
        const int t = u >> 2, w = u & 3;
        float x[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) x[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][4 * w + i], c, -mc));
        sum0 = (u == 0) ? x[0] : sum0 + x[0];
        sum1 = (u == 0) ? x[1] : sum1 + x[1];
        sum0 += x[2];
        sum1 += x[3];
        int packed = pack4_fp8<E5M2>(x[0], x[1], x[2], x[3]);
        // the weights are only read in the next iteration; without this pin the compiler sinks the conversions there
        asm volatile("" : "+v"(packed));
        p8_cur[u] = packed;
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) {
        if (ks == 0) {
          v16f z;
#pragma unroll
          for (int i = 0; i < 16; ++i) z[i] = 0.f;
          s[1] = mfma_fp8<E5M2>(kfrag[1][ks], qf[ks], z);
        } else {
          s[1] = mfma_fp8<E5M2>(kfrag[1][ks], qf[ks], s[1]);
        }
      }
      l_run += sum0 + sum1;
      asm volatile("" : "+v"(l_run));  // keeps the additions above where they are written
      // O now holds the PV product of block j-1: bring it to the new row max (in the lanes whose max moved, see compute_tile)
      if (changed) {
        if (alpha != 1.f) {
#pragma unroll
          for (int mt = 0; mt < kMTiles; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o_acc[mt][i] *= alpha;
        }
      }
      p8 = p8_cur;
    };
    // Waits until at most `tiles` tile copies (kPasses loads each) are in flight, then the barrier: it publishes the landed
    // tiles and frees the stages read before it.  vmcnt counts this lane's loads in issue order.
    auto wait_in_flight = [&](auto tiles_c) __attribute__((always_inline)) {
      constexpr int n = decltype(tiles_c)::value * kPasses;
      static_assert(n < 16, "vmcnt immediate");
      __builtin_amdgcn_s_waitcnt(0x0F70 | n);
      __builtin_amdgcn_s_barrier();
    };
    using T = std::true_type;
    using F = std::false_type;
    issue_k(0, k_lds0, true);
    issue_k(min(1, n_tiles), k_lds1, 1 < n_tiles);
    issue_k(min(2, n_tiles), k_lds2, 2 < n_tiles);
    issue_v(0, v_lds0, true);
    wait_in_flight(std::integral_constant<int, 2>());  // K(0) and K(1) landed
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[t][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) s[t] = mfma_fp8<E5M2>(load_kf(k_lds0, t, ks), qf[ks], s[t]);
    }
    __builtin_amdgcn_s_barrier();  // every wavefront has read K(0): step 0 may overwrite its stage
    // One step with compile-time LDS stages (PH = j % 3).
    auto step = [&](auto first_c, auto ph_c, int j) __attribute__((always_inline)) {
      constexpr int PH = decltype(ph_c)::value;
      uint8_t* const kst[3] = {k_lds0, k_lds1, k_lds2};
      uint8_t* const vst[3] = {v_lds0, v_lds1, v_lds2};
      iteration(first_c, j, kst[(PH + 1) % 3], vst[(PH + 2) % 3], kst[PH], vst[(PH + 1) % 3]);
      wait_in_flight(std::integral_constant<int, 2>());  // the two copies of this step may stay in flight
    };
    constexpr std::integral_constant<int, 0> ph0{};
    constexpr std::integral_constant<int, 1> ph1{};
    constexpr std::integral_constant<int, 2> ph2{};
    step(T(), ph0, 0);
    int j = 1;
    for (; j + 2 < n_tiles; j += 3) {
      step(F(), ph1, j);
      step(F(), ph2, j + 1);
      step(F(), ph0, j + 2);
    }
    if (j < n_tiles) {
      step(F(), ph1, j);
      if (j + 1 < n_tiles) step(F(), ph2, j + 1);
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // the last copies (of nothing) must not outlive the workgroup's LDS
    // the PV product of the last block
    {
      const int st = (n_tiles - 1) % 3;
      const uint8_t* vb = st == 0 ? v_lds0 : (st == 1 ? v_lds1 : v_lds2);
#pragma unroll
      for (int mt = 0; mt < kMTiles; ++mt) o_acc[mt] = mfma_fp8<E5M2>(load_vf(vb, mt), p8, o_acc[mt]);
    }
  } else if constexpr (PIPE) {
    // ---- software-pipelined loop ----
    // Iteration j is the softmax of block j in 8 chunks of 4 weights with a matrix instruction in front of the chunks: first
    // the PV products of block j-1, then the S^T products of block j+1 (head dim 128: one per chunk, 64: every second
    // chunk), their LDS operands fetched two instructions ahead.  K(t) lives in K stage t % 4, V(t) in V stage t % 4.  Step j
    // starts the copies of K(j+4) and V(j+2) (their stages held K(j) and V(j-2), last read in iteration j-1), reads K(j+1)
    // and V(j-1), and ends when K(j+2) and V(j) have landed.  Every block takes this path, masked blocks included (their
    // weights become exact zeros), so the loop needs no second form.
    constexpr int kSlots = kMTiles + 2 * kKSteps;  // matrix instructions per iteration
    constexpr int kChunksPerSlot = 8 / kSlots;     // 1 (head dim 128) or 2 (64)
    v16f sbuf[2][2];
    v8i p8buf[2];
    const int kv_limit = CAUSAL ? min(q_row + shift, kv_last) : kv_last;  // last kv this query attends to
    auto iteration = [&](auto first_c, int j, const uint8_t* kb_next, const uint8_t* vb_prev, v16f(&s)[2], v16f(&sn)[2],
                         const v8i& p8_prev, v8i& p8_cur) __attribute__((always_inline)) {
      constexpr bool kFirst = decltype(first_c)::value;
      const bool masked = j >= n_plain;  // wave-uniform
      v8i frag[kSlots];
      if constexpr (!kFirst) {
        frag[0] = load_vf(vb_prev, 0);
        frag[1] = load_vf(vb_prev, 1);
      }
      if (masked) {
        // a masked logit becomes -inf and its weight exp2(-inf) = 0 (the launcher takes this loop only for scale > 0)
        const int kv0 = j * kKvBlock;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (kv0 + 32 * h + 16 * t + i > kv_limit) s[t][i] = -INFINITY;
      }
      float mx[4];
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) mx[ch] = max3(s[0][4 * ch], s[0][4 * ch + 1], s[0][4 * ch + 2]);
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) mx[ch] = max3(mx[ch], s[0][4 * ch + 3], s[1][4 * ch]);
#pragma unroll
      for (int ch = 0; ch < 4; ++ch) mx[ch] = max3(mx[ch], s[1][4 * ch + 1], s[1][4 * ch + 2]);
      const float m_new = lane32_max(max3(max3(mx[0], s[1][3], s[1][7]), max3(mx[1], s[1][11], s[1][15]), max3(mx[2], mx[3], m_run)));
      bool changed = false;
      float alpha = 1.f;
      float mc = m_new * c;
      if constexpr (kFirst) {
        m_run = m_new;  // O and l are still zero
      } else {
        changed = __any(m_new != m_run);
        if (changed) {
          alpha = __builtin_amdgcn_exp2f((m_run - m_new) * c);
          l_run *= alpha;
          m_run = m_new;
        }
      }
      float sum0, sum1;
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (u % kChunksPerSlot == 0) {
          const int slot = u / kChunksPerSlot;
          // operands of the matrix instruction two slots ahead
          if (slot + 2 < kSlots) {
            const int sl = slot + 2;
            if (sl < kMTiles) {
              if constexpr (!kFirst) frag[sl] = load_vf(vb_prev, sl);
            } else {
              frag[sl] = load_kf(kb_next, (sl - kMTiles) / kKSteps, (sl - kMTiles) % kKSteps);
            }
          }
          if (slot < kMTiles) {
            if constexpr (!kFirst) o_acc[slot] = mfma_fp8<E5M2>(frag[slot], p8_prev, o_acc[slot]);
          } else {
            // (after the last block this is the product of a stale tile: never used)
            const int t = (slot - kMTiles) / kKSteps, ks = (slot - kMTiles) % kKSteps;
            if (ks == 0) {
              v16f z;
#pragma unroll
              for (int i = 0; i < 16; ++i) z[i] = 0.f;
              sn[t] = mfma_fp8<E5M2>(frag[slot], qf[ks], z);
            } else {
              sn[t] = mfma_fp8<E5M2>(frag[slot], qf[ks], sn[t]);
            }
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        // chunk u of the softmax: weights 4w .. 4w+3 of sub-tile t
        const int t = u >> 2, w = u & 3;
#pragma unroll
        for (int i = 4 * w; i < 4 * w + 4; ++i) s[t][i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][i], c, -mc));
        sum0 = (u == 0) ? s[t][4 * w] : sum0 + s[t][4 * w];
        sum1 = (u == 0) ? s[t][4 * w + 1] : sum1 + s[t][4 * w + 1];
        sum0 += s[t][4 * w + 2];
        sum1 += s[t][4 * w + 3];
        int packed = pack4_fp8<E5M2>(s[t][4 * w], s[t][4 * w + 1], s[t][4 * w + 2], s[t][4 * w + 3]);
        // the weights are only read in the next iteration; without this pin the compiler sinks the conversions there, in
        // one clump in front of the PV products that wait for them
        asm volatile("" : "+v"(packed));
        p8_cur[u] = packed;
        __builtin_amdgcn_sched_barrier(0);
      }
      l_run += sum0 + sum1;
      asm volatile("" : "+v"(l_run));  // keeps the additions above where they are written (sunk to the end they cost registers)
      // O now holds the PV product of block j-1 (issued four or more chunks ago): bring it to the new row max (in the lanes
      // whose max moved, see compute_tile)
      if (changed) {
        if (alpha != 1.f) {
#pragma unroll
          for (int mt = 0; mt < kMTiles; ++mt)
#pragma unroll
            for (int i = 0; i < 16; ++i) o_acc[mt][i] *= alpha;
        }
      }
    };
    // Every step starts two tile copies, also past the last block this workgroup walks (those copy nothing, see issue_k), so the
    // number of loads in flight is the same at every step.  vmcnt counts this lane's loads in issue order.
    // Waits until at most `tiles` tile copies (kPasses loads each) are in flight, then the barrier: it publishes the landed
    // tiles and frees the stages read before it.
    auto wait_in_flight = [&](auto tiles_c) __attribute__((always_inline)) {
      constexpr int n = decltype(tiles_c)::value * kPasses;
      static_assert(n < 16, "vmcnt immediate");
      __builtin_amdgcn_s_waitcnt(0x0F70 | n);
      __builtin_amdgcn_s_barrier();
    };
    // Ends step j: K(j+2) and V(j) must have landed; the copies of steps j-1 and j (K(j+3), V(j+1), K(j+4), V(j+2)) may stay
    // in flight.
    auto end_step = [&]() __attribute__((always_inline)) { wait_in_flight(std::integral_constant<int, 4>()); };
    // The PV product of the last block (its weights are in p8), V in stage vb.
    auto finish = [&](const uint8_t* vb, const v8i& p8) __attribute__((always_inline)) {
#pragma unroll
      for (int mt = 0; mt < kMTiles; ++mt) o_acc[mt] = mfma_fp8<E5M2>(load_vf(vb, mt), p8, o_acc[mt]);
    };
    using T = std::true_type;
    using F = std::false_type;
    // the copies of steps -4 .. -1
    issue_k(0, k_lds0, true);
    issue_k(min(1, n_tiles), k_lds1, 1 < n_tiles);
    issue_k(min(2, n_tiles), k_lds2, 2 < n_tiles);
    issue_v(0, v_lds0, true);
    issue_k(min(3, n_tiles), k_lds3, 3 < n_tiles);
    issue_v(min(1, n_tiles), v_lds1, 1 < n_tiles);
    wait_in_flight(std::integral_constant<int, 5>());  // K(0) landed
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int i = 0; i < 16; ++i) sbuf[0][t][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < kKSteps; ++ks) sbuf[0][t] = mfma_fp8<E5M2>(load_kf(k_lds0, t, ks), qf[ks], sbuf[0][t]);
    }
    end_step();  // K(1) landed, and every wavefront has read K(0): step 0 may overwrite its stage
    // One step with compile-time LDS stages (PH = j % 4) and buffers (j % 2); the mask-free form for the leading blocks.
    auto step = [&](auto first_c, auto ph_c, int j) __attribute__((always_inline)) {
      constexpr int PH = decltype(ph_c)::value;
      constexpr bool kFirst = decltype(first_c)::value;
      uint8_t* const kst[4] = {k_lds0, k_lds1, k_lds2, k_lds3};
      uint8_t* const vst[4] = {v_lds0, v_lds1, v_lds2, v_lds3};
      issue_k(min(j + 4, n_tiles), kst[PH], j + 4 < n_tiles);
      issue_v(min(j + 2, n_tiles), vst[(PH + 2) % 4], j + 2 < n_tiles);
      iteration(first_c, j, kst[(PH + 1) % 4], vst[(PH + 3) % 4], sbuf[PH % 2], sbuf[(PH + 1) % 2], p8buf[(PH + 1) % 2],
                p8buf[PH % 2]);
      end_step();
      (void)kFirst;
    };
    constexpr std::integral_constant<int, 0> ph0{};
    constexpr std::integral_constant<int, 1> ph1{};
    constexpr std::integral_constant<int, 2> ph2{};
    constexpr std::integral_constant<int, 3> ph3{};
    step(T(), ph0, 0);
    int j = 1;
    for (; j + 3 < n_tiles; j += 4) {
      step(F(), ph1, j);
      step(F(), ph2, j + 1);
      step(F(), ph3, j + 2);
      step(F(), ph0, j + 3);
    }
    // up to three more blocks; the weights of the last block end in p8buf[0]
    if (j < n_tiles) {
      step(F(), ph1, j);
      if (j + 1 < n_tiles) {
        step(F(), ph2, j + 1);
        if (j + 2 < n_tiles) {
          step(F(), ph3, j + 2);
          p8buf[0] = p8buf[1];
        }
      } else {
        p8buf[0] = p8buf[1];
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // the copies past the last block must not outlive the workgroup's LDS
    {
      const int st = (n_tiles - 1) & 3;
      finish(st == 0 ? v_lds0 : (st == 1 ? v_lds1 : (st == 2 ? v_lds2 : v_lds3)), p8buf[0]);
    }
  } else if constexpr (kStages == 3) {
    issue_tile(0, k_lds0, v_lds0);
    if (n_tiles > 1) issue_tile(1, k_lds1, v_lds1);
    stage_sync(n_tiles > 1);
    // Block 0 takes the general path: it is the only block that can meet a running max of -inf.
    if (n_tiles > 2) issue_tile(2, k_lds2, v_lds2);
    compute_tile(0, k_lds0, v_lds0, std::true_type());
    stage_sync(n_tiles > 2);
    int j = 1;
    // Mask-free blocks, three per trip so that every third reads one fixed LDS stage (the compiler can then tell
    // that the copies in flight go to other stages and need not be waited for before the reads).
    // Inside this loop every copy is issued unconditionally (block j+4 exists), which lets the compiler see that each
    // s_waitcnt below always leaves exactly one block in flight.
    for (; j + 2 < n_plain && j + 4 < n_tiles; j += 3) {
      issue_tile(j + 2, k_lds0, v_lds0);
      compute_tile(j, k_lds1, v_lds1, std::false_type());
      stage_sync(true);
      issue_tile(j + 3, k_lds1, v_lds1);
      compute_tile(j + 1, k_lds2, v_lds2, std::false_type());
      stage_sync(true);
      issue_tile(j + 4, k_lds2, v_lds2);
      compute_tile(j + 2, k_lds0, v_lds0, std::false_type());
      stage_sync(true);
    }
    // The last few mask-free blocks: same arithmetic, LDS stage chosen at run time, copies issued while blocks remain.
    for (; j < n_plain; ++j) {
      const int st = j % 3, st2 = (j + 2) % 3;
      if (j + 2 < n_tiles)
        issue_tile(j + 2, st2 == 0 ? k_lds0 : (st2 == 1 ? k_lds1 : k_lds2), st2 == 0 ? v_lds0 : (st2 == 1 ? v_lds1 : v_lds2));
      compute_tile(j, st == 0 ? k_lds0 : (st == 1 ? k_lds1 : k_lds2), st == 0 ? v_lds0 : (st == 1 ? v_lds1 : v_lds2),
                   std::false_type());
      stage_sync(j + 2 < n_tiles);
    }
    // The remaining blocks (the blocks on the diagonal, the kv tail) take the masking copy.
    for (; j < n_tiles; ++j) {
      const int st = j % 3, st2 = (j + 2) % 3;
      if (j + 2 < n_tiles)
        issue_tile(j + 2, st2 == 0 ? k_lds0 : (st2 == 1 ? k_lds1 : k_lds2), st2 == 0 ? v_lds0 : (st2 == 1 ? v_lds1 : v_lds2));
      // a wavefront whose 32 query rows all lie before this kv block has nothing to add (causal)
      if (!CAUSAL || j * kKvBlock <= q_wave0 + kQWave - 1 + shift)
        compute_tile(j, st == 0 ? k_lds0 : (st == 1 ? k_lds1 : k_lds2), st == 0 ? v_lds0 : (st == 1 ? v_lds1 : v_lds2),
                     std::true_type());
      stage_sync(j + 2 < n_tiles);
    }
  } else {
    // Two stages: the copy of block j+1 is issued at the start of the step for block j and must have landed at its end.
    issue_tile(0, k_lds0, v_lds0);
    stage_sync(false);
    if (n_tiles > 1) issue_tile(1, k_lds1, v_lds1);
    compute_tile(0, k_lds0, v_lds0, std::true_type());
    stage_sync(false);
    int j = 1;
    for (; j + 1 < n_plain && j + 2 < n_tiles; j += 2) {
      issue_tile(j + 1, k_lds0, v_lds0);
      compute_tile(j, k_lds1, v_lds1, std::false_type());
      stage_sync(false);
      issue_tile(j + 2, k_lds1, v_lds1);
      compute_tile(j + 1, k_lds0, v_lds0, std::false_type());
      stage_sync(false);
    }
    for (; j < n_plain; ++j) {  // the last mask-free blocks
      const bool odd = j & 1;
      if (j + 1 < n_tiles) issue_tile(j + 1, odd ? k_lds0 : k_lds1, odd ? v_lds0 : v_lds1);
      compute_tile(j, odd ? k_lds1 : k_lds0, odd ? v_lds1 : v_lds0, std::false_type());
      stage_sync(false);
    }
    for (; j < n_tiles; ++j) {
      const bool odd = j & 1;
      if (j + 1 < n_tiles) issue_tile(j + 1, odd ? k_lds0 : k_lds1, odd ? v_lds0 : v_lds1);
      if (!CAUSAL || j * kKvBlock <= q_wave0 + kQWave - 1 + shift)
        compute_tile(j, odd ? k_lds1 : k_lds0, odd ? v_lds1 : v_lds0, std::true_type());
      stage_sync(false);
    }
  }

  // ---- epilogue: O / l, convert, store (reference csrc/flash_attention.cu:542-582) ----
  const float l_tot = lane32_sum(l_run);
  const float inv = (l_tot == 0.f || l_tot != l_tot) ? 1.f : 1.f / l_tot;
  // log-sum-exp of the scaled logits of the row (natural log), -inf for a row that saw no key; the reference reserves
  // the output but never writes it (csrc/flash.h:56, csrc/flash_attention.cu:658-659)
  if (a.lse != nullptr && h == 0 && q_row < a.seqlen_q) {
    const float lse = l_tot > 0.f ? (m_run * c + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f : (l_tot == 0.f ? -INFINITY : l_tot);
    a.lse[b * a.lse_bs + hd * a.lse_hs + q_row] = lse;
  }
  if (q_row < a.seqlen_q) {
    // register i = 4a2 + b2 of tile mt is head-dim column 32mt + 8a2 + 4h + b2
    if constexpr (OUT == FA8_OUT_FP16) {
      _Float16* op = (_Float16*)a.o + b * a.o_bs + hd * a.o_hs + (long long)q_row * a.o_rs + 4 * h;
#pragma unroll
      for (int mt = 0; mt < kMTiles; ++mt)
#pragma unroll
        for (int a2 = 0; a2 < 4; ++a2) {
          v4h w;
#pragma unroll
          for (int b2 = 0; b2 < 4; ++b2) w[b2] = (_Float16)(o_acc[mt][4 * a2 + b2] * inv);
          *(v4h*)(op + 32 * mt + 8 * a2) = w;
        }
    } else {
      uint8_t* op = (uint8_t*)a.o + b * a.o_bs + hd * a.o_hs + (long long)q_row * a.o_rs + 4 * h;
#pragma unroll
      for (int mt = 0; mt < kMTiles; ++mt)
#pragma unroll
        for (int a2 = 0; a2 < 4; ++a2) {
          float x[4];
          constexpr float kMaxFinite = OUT == FA8_OUT_E5M2 ? 57344.f : 448.f;
#pragma unroll
          for (int b2 = 0; b2 < 4; ++b2) {
            const float y = o_acc[mt][4 * a2 + b2] * inv;
            x[b2] = (y != y) ? y : fminf(fmaxf(y, -kMaxFinite), kMaxFinite);  // saturate to finite, keep NaN
          }
          *(int*)(op + 32 * mt + 8 * a2) = pack4_fp8<OUT == FA8_OUT_E5M2>(x[0], x[1], x[2], x[3]);
        }
    }
  }
#endif  // __HIP_DEVICE_COMPILE__
}

template <int D, bool CAUSAL, bool E5M2, int OUT>
int launch(const KernelArgs& a, bool v_transposed, int loop, hipStream_t stream) {
  const dim3 grid((unsigned)(a.bh_total * a.n_qblocks));
  // hipLaunchKernel returns the status of this launch itself; the thread's sticky "last error" (which an earlier,
  // unrelated call may have left behind) is neither read nor cleared.
  KernelArgs args = a;
  void* argv[] = {&args};
  const void* fn = v_transposed ? (const void*)&fa8_fwd_kernel<D, CAUSAL, E5M2, OUT, true, kLoopRolling>
                                : (const void*)&fa8_fwd_kernel<D, CAUSAL, E5M2, OUT, false, kLoopRolling>;
  if constexpr (D == 64 || D == 128) {
    if (loop == FA8_SCHEDULE_PIPELINED)
      fn = v_transposed ? (const void*)&fa8_fwd_kernel<D, CAUSAL, E5M2, OUT, true, kLoopPipelined>
                        : (const void*)&fa8_fwd_kernel<D, CAUSAL, E5M2, OUT, false, kLoopPipelined>;
    if constexpr (!CAUSAL) {
      if (loop == FA8_SCHEDULE_DENSE)
        fn = v_transposed ? (const void*)&fa8_fwd_kernel<D, false, E5M2, OUT, true, kLoopDense>
                          : (const void*)&fa8_fwd_kernel<D, false, E5M2, OUT, false, kLoopDense>;
    }
  }
  return (int)hipLaunchKernel(fn, grid, dim3(kThreads), argv, 0, stream);
}

template <int D, bool CAUSAL>
int launch_types(const Fa8FwdParams* p, const KernelArgs& a, int loop, hipStream_t stream) {
  const bool e5m2 = p->in_dtype == FA8_DTYPE_E5M2, vt = p->v_layout == FA8_V_TRANSPOSED;
  if (p->out_dtype == FA8_OUT_FP16)
    return e5m2 ? launch<D, CAUSAL, true, FA8_OUT_FP16>(a, vt, loop, stream)
                : launch<D, CAUSAL, false, FA8_OUT_FP16>(a, vt, loop, stream);
  // fp8 output: the reference stores O in the input element type (csrc/flash_attention.cu:557, :655-656); the two
  // mixed combinations are not built
  if (e5m2)
    return p->out_dtype == FA8_OUT_E5M2 ? launch<D, CAUSAL, true, FA8_OUT_E5M2>(a, vt, loop, stream) : FA8_ERR_UNSUPPORTED;
  return p->out_dtype == FA8_OUT_E4M3 ? launch<D, CAUSAL, false, FA8_OUT_E4M3>(a, vt, loop, stream) : FA8_ERR_UNSUPPORTED;
}

// KV blocks walked by all workgroups of a launch together.
long long launch_kv_blocks(const Fa8FwdParams* p) {
  const long long bh = (long long)p->batch * p->heads, nq = (p->seqlen_q + kQBlock - 1) / kQBlock;
  const long long tk = (p->seqlen_k + kKvBlock - 1) / kKvBlock;
  if (!p->is_causal) return bh * nq * tk;
  // q block i walks clamp(base + 2 i, 1, tk) blocks: one block up to i = n1 - 1, all tk blocks from i = first
  const long long s64 = p->causal_align == FA8_CAUSAL_BOTTOM_RIGHT ? (long long)p->seqlen_k - p->seqlen_q : 0;
  const long long base = 2 + (s64 >= 0 ? (s64 + kKvBlock - 1) / kKvBlock : -((-s64) / kKvBlock));
  long long n1 = base <= 1 ? (1 - base) / 2 + 1 : 0;
  if (n1 > nq) n1 = nq;
  long long first = tk > base ? (tk - base + 1) / 2 : 0;
  if (first < n1) first = n1;
  if (first > nq) first = nq;
  const long long cnt = first - n1;
  return bh * (n1 + cnt * base + (n1 + first - 1) * cnt + (nq - first) * tk);
}

// Compute units of the current device (0 if the runtime cannot tell), asked once per device.  The current device must be the
// one that owns the stream and the tensors of the call (the PyTorch binding and the ctypes mirror see to it).
int compute_units() {
  static std::atomic<int> cached[64];  // zero-initialised; racing first calls store the same value
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n < 1) return 0;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Which main loop a valid call runs (see fa8_fwd_kernel): FA8_SCHEDULE_ROLLING, _PIPELINED or _DENSE.
// The pipelined loops exist for head dims 64 and 128 and for a softmax scale in (0, 1e6) (the pipelined loop relies on
// exp2(-inf * scale) = 0 for masked logits and on its finite stand-in for a row max of -inf times the scale staying finite);
// elsewhere every hint is ignored and the rolling loop runs.
// Dense: full (non-causal) attention over a whole number of KV blocks, where no logit is ever masked; measured 1 - 2 % faster
// than the rolling loop on launches that fill the chip and 3 - 5 % faster than the pipelined loop on small ones, so it is
// the choice wherever it applies.  A hint for it that does not apply falls back to the automatic choice.
// Pipelined: launches that cannot keep three wavefronts on every SIMD for most of their run: at most four workgroups per
// compute unit (two resident at a time), or little work per compute unit (then filling and draining the chip, and for
// causal launches the thinning out of the workgroups, is a large share of the run).  Measured 5 - 15 % faster than the
// rolling loop there; the rolling loop is equal or up to 5 % faster elsewhere.
int choose_loop(const Fa8FwdParams* p) {
  if ((p->head_dim != 64 && p->head_dim != 128) || !(p->softmax_scale > 0.f && p->softmax_scale < 1.0e6f)) return FA8_SCHEDULE_ROLLING;
  const bool dense_ok = !p->is_causal && p->seqlen_k % kKvBlock == 0;
  if (p->schedule == FA8_SCHEDULE_ROLLING || p->schedule == FA8_SCHEDULE_PIPELINED) return p->schedule;
  if (dense_ok) return FA8_SCHEDULE_DENSE;
  const long long cus = compute_units();
  const long long wgs = (long long)p->batch * p->heads * ((p->seqlen_q + kQBlock - 1) / kQBlock);
  // KV blocks per compute unit below which the pipelined loop was measured to win (head dim 64 has half the matrix work
  // per block)
  const long long few_blocks = p->head_dim == 64 ? 264 : 144;
  const bool small = cus > 0 && (wgs <= 4 * cus || (wgs <= few_blocks * cus && launch_kv_blocks(p) <= few_blocks * cus));
  return small ? FA8_SCHEDULE_PIPELINED : FA8_SCHEDULE_ROLLING;
}

// Tuning aid for measurements only: FA8_CAUSAL_INTERLEAVE=n in the environment (read once) replaces the number of heads of an
// XCD that take turns at every q block of a causal launch (see decode_block; the results do not depend on it).  0: unset.
int env_causal_interleave() {
  static std::atomic<int> cached{-1};
  int v = cached.load(std::memory_order_relaxed);
  if (v < 0) {
    const char* e = std::getenv("FA8_CAUSAL_INTERLEAVE");
    v = e ? std::atoi(e) : 0;
    if (v < 0 || v > 64) v = 0;
    cached.store(v, std::memory_order_relaxed);
  }
  return v;
}

bool span_ok(long long outer_stride, long long inner_extent) { return outer_stride >= inner_extent; }

}  // namespace

extern "C" int fa8_fwd_validate(const Fa8FwdParams* p) {
  if (p == nullptr || p->q == nullptr || p->k == nullptr || p->v == nullptr || p->o == nullptr) return FA8_ERR_NULL;
  if (p->batch < 1 || p->heads < 1 || p->seqlen_q < 1 || p->seqlen_k < 1 || p->head_dim < 1) return FA8_ERR_SHAPE;
  if (p->is_causal != 0 && p->is_causal != 1) return FA8_ERR_SHAPE;
  if (p->heads_k < 0 || (p->heads_k > 0 && p->heads % p->heads_k != 0)) return FA8_ERR_SHAPE;
  if (p->causal_align != FA8_CAUSAL_TOP_LEFT && p->causal_align != FA8_CAUSAL_BOTTOM_RIGHT) return FA8_ERR_DTYPE;
  if (p->schedule < FA8_SCHEDULE_AUTO || p->schedule > FA8_SCHEDULE_DENSE) return FA8_ERR_DTYPE;
  if (p->reserved0 != 0) return FA8_ERR_UNSUPPORTED;  // a field of a later version of the parameter block
  if ((long long)p->batch * p->heads > 0x7fffffffLL / ((p->seqlen_q + kQBlock - 1) / kQBlock)) return FA8_ERR_SHAPE;
  if (p->in_dtype != FA8_DTYPE_E4M3 && p->in_dtype != FA8_DTYPE_E5M2) return FA8_ERR_DTYPE;
  if (p->out_dtype != FA8_OUT_FP16 && p->out_dtype != FA8_OUT_E4M3 && p->out_dtype != FA8_OUT_E5M2) return FA8_ERR_DTYPE;
  if (p->v_layout != FA8_V_ROWS && p->v_layout != FA8_V_TRANSPOSED) return FA8_ERR_DTYPE;
  if (p->head_dim % 32 != 0 || p->head_dim > 256) return FA8_ERR_HEAD_DIM;
  if (!(p->softmax_scale == p->softmax_scale) || std::isinf(p->softmax_scale)) return FA8_ERR_SCALE;
  const long long d = p->head_dim;
  const long long v_rows = p->v_layout == FA8_V_ROWS ? p->seqlen_k : d;
  const long long v_cols = p->v_layout == FA8_V_ROWS ? d : p->seqlen_k;
  if (!span_ok(p->q_row_stride, d) || !span_ok(p->q_head_stride, 1) || !span_ok(p->q_batch_stride, 1)) return FA8_ERR_STRIDE;
  if (!span_ok(p->k_row_stride, d) || !span_ok(p->k_head_stride, 1) || !span_ok(p->k_batch_stride, 1)) return FA8_ERR_STRIDE;
  if (!span_ok(p->v_row_stride, v_cols) || !span_ok(p->v_head_stride, 1) || !span_ok(p->v_batch_stride, 1)) return FA8_ERR_STRIDE;
  if (!span_ok(p->o_row_stride, d) || !span_ok(p->o_head_stride, 1) || !span_ok(p->o_batch_stride, 1)) return FA8_ERR_STRIDE;
  // 16-byte vector loads of q/k/v rows, 8-byte (fp16) or 4-byte (fp8) vector stores of o
  const long long in_strides[] = {p->q_batch_stride, p->q_head_stride, p->q_row_stride, p->k_batch_stride, p->k_head_stride,
                                  p->k_row_stride,   p->v_batch_stride, p->v_head_stride, p->v_row_stride};
  for (long long s : in_strides)
    if (s % 16 != 0) return FA8_ERR_ALIGN;
  if (((uintptr_t)p->q | (uintptr_t)p->k | (uintptr_t)p->v) % 16 != 0) return FA8_ERR_ALIGN;
  const long long o_elem = p->out_dtype == FA8_OUT_FP16 ? 2 : 1;
  const long long o_strides[] = {p->o_batch_stride, p->o_head_stride, p->o_row_stride};
  for (long long s : o_strides)
    if ((s * o_elem) % 8 != 0) return FA8_ERR_ALIGN;
  if ((uintptr_t)p->o % 8 != 0) return FA8_ERR_ALIGN;
  if (p->lse != nullptr) {
    if (!span_ok(p->lse_head_stride, p->seqlen_q) || !span_ok(p->lse_batch_stride, 1)) return FA8_ERR_STRIDE;
    if ((uintptr_t)p->lse % 4 != 0) return FA8_ERR_ALIGN;
  }
  // the kernels address k and v of one head with 32-bit byte offsets; a tile copy forms offsets for all 64 rows of a
  // block (rows past the end are not read, but their offsets are computed), hence at least 64 rows here
  const long long k_rows_addr = p->seqlen_k > kKvBlock ? p->seqlen_k : kKvBlock;
  const long long v_rows_addr = v_rows > kKvBlock ? v_rows : kKvBlock;
  if (k_rows_addr * p->k_row_stride > 0x7fffffffLL || v_rows_addr * p->v_row_stride > 0x7fffffffLL) return FA8_ERR_SHAPE;
  // ... and the offsets of a whole block just past the last row (block offset + row offset of its 64th row) must not wrap
  // around 32 bits, or the buffer's range check would take them for rows of the tensor (matters only for a few rows with a
  // row stride of tens of megabytes)
  if ((p->seqlen_k + 126LL) * p->k_row_stride + 256 > 0xffffffffLL || (v_rows + 126LL) * p->v_row_stride + 256 > 0xffffffffLL)
    return FA8_ERR_SHAPE;
  // transposed v is read in 16-byte chunks along kv
  if (p->v_layout == FA8_V_TRANSPOSED && p->seqlen_k % 16 != 0) return FA8_ERR_ALIGN;
  // an fp8 output has the element type of the inputs
  if ((p->out_dtype == FA8_OUT_E4M3 && p->in_dtype != FA8_DTYPE_E4M3) || (p->out_dtype == FA8_OUT_E5M2 && p->in_dtype != FA8_DTYPE_E5M2))
    return FA8_ERR_UNSUPPORTED;
  return FA8_OK;
}

extern "C" int fa8_fwd(const Fa8FwdParams* p, void* hip_stream) {
  const int rc = fa8_fwd_validate(p);
  if (rc != FA8_OK) return rc;
  KernelArgs a;
  a.q = (const uint8_t*)p->q;
  a.k = (const uint8_t*)p->k;
  a.v = (const uint8_t*)p->v;
  a.o = p->o;
  a.lse = (float*)p->lse;
  a.lse_bs = p->lse_batch_stride; a.lse_hs = p->lse_head_stride;
  a.kv_group = p->heads_k > 0 ? p->heads / p->heads_k : 1;
  a.causal_shift = p->causal_align == FA8_CAUSAL_BOTTOM_RIGHT ? p->seqlen_k - p->seqlen_q : 0;
  a.heads = p->heads;
  a.seqlen_q = p->seqlen_q;
  a.seqlen_k = p->seqlen_k;
  a.n_qblocks = (p->seqlen_q + kQBlock - 1) / kQBlock;
  a.bh_total = p->batch * p->heads;
  a.interleave = a.bh_total / 8 < 8 ? (a.bh_total / 8 > 0 ? a.bh_total / 8 : 1) : 8;  // causal launches, see decode_block
  if (env_causal_interleave() > 0) a.interleave = env_causal_interleave();
  a.scale_log2 = p->softmax_scale * 1.4426950408889634f;
  a.q_bs = p->q_batch_stride; a.q_hs = p->q_head_stride; a.q_rs = p->q_row_stride;
  a.k_bs = p->k_batch_stride; a.k_hs = p->k_head_stride; a.k_rs = p->k_row_stride;
  a.v_bs = p->v_batch_stride; a.v_hs = p->v_head_stride; a.v_rs = p->v_row_stride;
  a.o_bs = p->o_batch_stride; a.o_hs = p->o_head_stride; a.o_rs = p->o_row_stride;
  hipStream_t stream = (hipStream_t)hip_stream;
  const int loop = choose_loop(p);
  switch (p->head_dim) {
#define FA8_HEAD_DIM_CASE(D_) \
  case D_: return p->is_causal ? launch_types<D_, true>(p, a, loop, stream) : launch_types<D_, false>(p, a, loop, stream)
    FA8_HEAD_DIM_CASE(32);  // the head-dim buckets of the reference (csrc/static_switch.h:50-77)
    FA8_HEAD_DIM_CASE(64);
    FA8_HEAD_DIM_CASE(96);
    FA8_HEAD_DIM_CASE(128);
    FA8_HEAD_DIM_CASE(160);
    FA8_HEAD_DIM_CASE(192);
    FA8_HEAD_DIM_CASE(224);
    FA8_HEAD_DIM_CASE(256);
#undef FA8_HEAD_DIM_CASE
    default: return FA8_ERR_HEAD_DIM;
  }
}

extern "C" int fa8_fwd_schedule(const Fa8FwdParams* p) {
  const int rc = fa8_fwd_validate(p);
  if (rc != FA8_OK) return rc;
  return choose_loop(p);
}

extern "C" int fa8_query(int what) {
  switch (what) {
    case FA8_QUERY_VERSION: return kVersion;
    case FA8_QUERY_KV_BLOCK: return kKvBlock;
    case FA8_QUERY_Q_BLOCK: return kQBlock;
    case FA8_QUERY_KV_ASCENDING: return 1;
    case FA8_QUERY_THREADS: return kThreads;
    case FA8_QUERY_PARAMS_SIZE: return (int)sizeof(Fa8FwdParams);
    default: return -1;
  }
}

extern "C" const char* fa8_error_string(int code) {
  switch (code) {
    case FA8_OK: return "ok";
    case FA8_ERR_NULL: return "a required pointer is NULL";
    case FA8_ERR_SHAPE: return "bad shape (a size < 1, too many workgroups, heads not a multiple of heads_k, or k/v of one head spanning 2 GiB or more)";
    case FA8_ERR_HEAD_DIM: return "head_dim must be a multiple of 32, at most 256";
    case FA8_ERR_STRIDE: return "a stride is smaller than the extent it spans";
    case FA8_ERR_ALIGN: return "q/k/v rows must be 16-byte aligned and o rows 8-byte aligned";
    case FA8_ERR_DTYPE: return "unknown in_dtype / out_dtype / v_layout / causal_align code";
    case FA8_ERR_UNSUPPORTED: return "this build has no kernel for the requested combination";
    case FA8_ERR_SCALE: return "softmax_scale must be finite";
    default: return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown fa8 error code";
  }
}
