/*
 * fa8_api.h -- C ABI of the MI355X (gfx950) FP8 flash-attention forward library (libfa8.so).
 *
 * This is the drop-in boundary for the one hot path of weishengying/cutlass_flash_atten_fp8:
 * the host entry `flash_attention_v2_cutlass(q, k, v, is_causal, softmax_scale)`
 * (reference csrc/flash_attention.cu:639-668, declared include/attention_api.h:10-11,
 * bound to Python at csrc/attention_api.cpp:6-10).  The PyTorch binding of this repository
 * (module `attention_cutlass_fp8`) and any other host (ctypes, plain C++) call the kernels only
 * through the functions below: plain pointers and sizes, no torch types.
 *
 * Error convention: 0 = success; negative = rejected arguments (FA8_ERR_*), nothing was launched;
 * positive = a hipError_t reported by the HIP runtime.  The library never exits the process
 * (the reference printf+exit()s on CUDA errors, include/attention_api.cuh:20-29).
 */
#ifndef FA8_API_H_
#define FA8_API_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of q/k/v */
#define FA8_DTYPE_E4M3 0 /* OCP float8 e4m3fn (torch.float8_e4m3fn) */
#define FA8_DTYPE_E5M2 1 /* OCP float8 e5m2   (torch.float8_e5m2); reference FP8_SWITCH, csrc/static_switch.h:39-48 */

/* element types of o */
#define FA8_OUT_FP16 0 /* IEEE half, round-to-nearest-even */
#define FA8_OUT_E4M3 1 /* e4m3fn, RNE, saturate-to-finite: what the reference stores (csrc/flash_attention.cu:557,656); e4m3 inputs only */
#define FA8_OUT_E5M2 2 /* e5m2, RNE, saturate-to-finite: the reference's output for e5m2 inputs (same lines); e5m2 inputs only */

/* layouts of v */
#define FA8_V_ROWS 0       /* v is [B,H,Nk,d]: same as k */
#define FA8_V_TRANSPOSED 1 /* v is [B,H,d,Nk]: what the reference requires of its caller (test.py:71) */

/* which keys a query sees when is_causal (matters only when seqlen_q != seqlen_k) */
#define FA8_CAUSAL_TOP_LEFT 0     /* key j <= query i: the reference's rule (csrc/flash_attention.cu:62-64, loop bound :458) */
#define FA8_CAUSAL_BOTTOM_RIGHT 1 /* key j <= i + seqlen_k - seqlen_q: the last query sees every key (decode, chunked prefill) */

/* which main loop the kernel runs: a performance hint, the results are bitwise the same
 *   AUTO      the library chooses from the shape of the launch
 *   ROLLING   one KV block after the other, three wavefronts per SIMD: for masked launches that fill the chip
 *   PIPELINED software-pipelined over neighbouring KV blocks, two wavefronts per SIMD: for small masked launches
 *   DENSE     the same pipeline in three wavefronts per SIMD, for launches without any masked logit: full (non-causal)
 *             attention with seqlen_k a multiple of 64; asked for elsewhere, the library chooses as for AUTO
 *   (PIPELINED and DENSE are built for head dims 64 and 128 and a softmax scale in (0, 1e6); ignored elsewhere) */
#define FA8_SCHEDULE_AUTO 0
#define FA8_SCHEDULE_ROLLING 1
#define FA8_SCHEDULE_PIPELINED 2
#define FA8_SCHEDULE_DENSE 3

/* error codes (all negative) */
#define FA8_OK 0
#define FA8_ERR_NULL (-1)        /* a required pointer is NULL */
#define FA8_ERR_SHAPE (-2)       /* a size is < 1, the grid would overflow, or heads is not a multiple of heads_k */
#define FA8_ERR_HEAD_DIM (-3)    /* head_dim is not a multiple of 32 in 32..256 */
#define FA8_ERR_STRIDE (-4)      /* a stride is smaller than the extent it must span, or rows overlap */
#define FA8_ERR_ALIGN (-5)       /* a base pointer or stride breaks the 16-byte row alignment the kernels load with (FA8_V_TRANSPOSED: also seqlen_k % 16 != 0) */
#define FA8_ERR_DTYPE (-6)       /* unknown in_dtype/out_dtype/v_layout/causal_align/schedule code */
#define FA8_ERR_UNSUPPORTED (-7) /* a valid combination that this build has no kernel for */
#define FA8_ERR_SCALE (-8)       /* softmax_scale is NaN or infinite */

/*
 * Parameter block.  Replaces the reference's by-value kernel argument
 * Flash_fwd_params / Qkv_params (csrc/flash.h:6-61) as filled by set_params_fprop
 * (csrc/flash_attention.cu:277-318).  Strides are in ELEMENTS and 64-bit (the reference
 * uses one shared 32-bit head offset for q, k, v and o, csrc/flash_attention.cu:364).
 * The last dimension of every tensor must be contiguous (stride 1).
 */
typedef struct Fa8FwdParams {
  const void* q; /* [B,H,Nq,d] fp8 */
  const void* k; /* [B,Hk,Nk,d] fp8; Hk = heads_k (or heads) */
  const void* v; /* [B,Hk,Nk,d] fp8 (FA8_V_ROWS) or [B,Hk,d,Nk] (FA8_V_TRANSPOSED) */
  void* o;       /* [B,H,Nq,d] fp16, or fp8 of the input element type */
  int32_t batch;
  int32_t heads;
  int32_t seqlen_q;
  int32_t seqlen_k;
  int32_t head_dim;
  int32_t is_causal; /* 0/1 */
  int32_t in_dtype;  /* FA8_DTYPE_* */
  int32_t out_dtype; /* FA8_OUT_* */
  int32_t v_layout;  /* FA8_V_* */
  float softmax_scale; /* natural-log domain: P = exp(scale*S - scale*rowmax), csrc/flash_attention.cu:197-216 */
  int64_t q_batch_stride, q_head_stride, q_row_stride;
  int64_t k_batch_stride, k_head_stride, k_row_stride;
  int64_t v_batch_stride, v_head_stride, v_row_stride; /* row = kv row (FA8_V_ROWS) or d row (FA8_V_TRANSPOSED) */
  int64_t o_batch_stride, o_head_stride, o_row_stride;
  /* ---- library version 2 (fa8_query(FA8_QUERY_VERSION) >= 2); all-zero = the behaviour of version 1 ---- */
  /* Optional output (NULL: not wanted): lse[b,h,i] = log(sum_j exp(softmax_scale * S[i,j])) over the keys query i sees,
   * fp32 [B,H,Nq], rows contiguous; -inf for a query that sees no key.  It is what merges partial results of a kv-split
   * (context-parallel) run.  The reference reserves softmax_lse_ptr but always passes nullptr
   * (csrc/flash.h:56, csrc/flash_attention.cu:658-659). */
  void* lse;
  int64_t lse_batch_stride, lse_head_stride;
  /* Grouped-query / multi-query attention: number of k/v heads; 0 (or == heads) = one per q head.  heads must be a
   * multiple; q head h reads k/v head h / (heads / heads_k).  (Reference fields k_head, h_h_k_ratio, csrc/flash.h:36-45:
   * declared, never used by its kernel.) */
  int32_t heads_k;
  int32_t causal_align; /* FA8_CAUSAL_* */
  /* ---- library version 3; all-zero = the library chooses ---- */
  int32_t schedule;  /* FA8_SCHEDULE_*: a performance hint, never changes the result */
  int32_t reserved0; /* must be 0 (anything else: FA8_ERR_UNSUPPORTED) */
} Fa8FwdParams;

/*
 * Host-only argument check: the same validation fa8_fwd performs before it touches the GPU.
 * Never calls into HIP.  Replaces CHECK_INPUT (reference include/attention_api.cuh:12-18) and adds
 * the shape/head-dim checks the reference lacks (csrc/flash_attention.cu:140,152-154 TODOs).
 */
int fa8_fwd_validate(const Fa8FwdParams* p);

/*
 * Enqueue the forward pass on `hip_stream` (a hipStream_t; NULL = the null stream) of the current
 * device and return without synchronising.  Replaces run_flash_attn_cutlass + the <<<>>> launch
 * (reference csrc/flash_attention.cu:586-637), which uses stream 0 and cudaDeviceSynchronize().
 * The caller keeps q/k/v/o alive until the stream has passed the work.  Stateless and re-entrant.
 * The current HIP device must be the one that owns the stream and the tensors (the library asks it for its number of
 * compute units when it chooses the main loop).  The parameter block has grown from version to version and carries no
 * size field: a caller compares fa8_query(FA8_QUERY_PARAMS_SIZE) with its own sizeof(Fa8FwdParams) once, before the first
 * call, and zero-initialises the whole block.
 */
int fa8_fwd(const Fa8FwdParams* p, void* hip_stream);

/*
 * Which main loop fa8_fwd would run for these arguments on the current device: FA8_SCHEDULE_ROLLING,
 * FA8_SCHEDULE_PIPELINED or FA8_SCHEDULE_DENSE (all > 0), or the FA8_ERR_* code fa8_fwd_validate gives.  Launches nothing.  No counterpart in
 * the reference (one kernel, one loop: csrc/flash_attention.cu:468-534); it makes the library's choice visible to
 * benchmarks and tests.
 */
int fa8_fwd_schedule(const Fa8FwdParams* p);

/* What fa8_query can report. */
#define FA8_QUERY_VERSION 0       /* integer library version */
#define FA8_QUERY_KV_BLOCK 1      /* kv columns per online-softmax step (reference kBlockN = 64, csrc/flash_attention.cu:624) */
#define FA8_QUERY_Q_BLOCK 2       /* q rows per workgroup */
#define FA8_QUERY_KV_ASCENDING 3  /* 1: kv blocks are visited in ascending order (as the reference loop :468) */
#define FA8_QUERY_THREADS 4       /* threads per workgroup */
#define FA8_QUERY_PARAMS_SIZE 5   /* sizeof(Fa8FwdParams) of the library: a caller built against another layout can tell */
int fa8_query(int what);

/* Static, human-readable text for a return code of this library (never NULL). */
const char* fa8_error_string(int code);

#ifdef __cplusplus
}
#endif
#endif /* FA8_API_H_ */
