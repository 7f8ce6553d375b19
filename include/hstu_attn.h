/*
 * hstu_attn.h -- C ABI of the MI355X (gfx950) HSTU pointwise-SiLU attention:
 * the forward (below) and its backward (hstu_attn_bwd).
 *
 *   S[b,h,i,j] = alpha * sum_c q[b,i,h,c] k[b,j,h,c]
 *                (+ pos_tab[h|0][(L-1)+j-i]) (+ ts_tab[h|0][bucket(dt)])
 *                (+ dense_bias[b|0][i][j])
 *   P          = S * sigmoid(S) * inv_n
 *   out[b,i,h,:] = sum_j (M[b,i,j] ? P : 0) * v[b,j,h,:]
 *
 * Every entry point is enqueue-only on the caller's HIP stream, allocates no
 * device memory and never synchronises.  The caller owns every buffer.
 *
 * Reference interfaces this library stands in for (paths relative to the
 * RecML checkout):
 *   hstu_attn_fwd            recml/core/ops/hstu_ops.py:829-851
 *                            (pointwise_splash_attention) and
 *                            recml/layers/keras/hstu.py:356-390
 *                            (HSTUBlock._pointwise_attention)
 *   mask fields              recml/core/ops/hstu_ops.py:926-979 (mask type,
 *                            sliding window, segment ids) and
 *                            recml/layers/keras/utils.py:29-41 (length mask)
 *   pos_tab                  recml/layers/keras/hstu.py:58-128
 *   ts / ts_tab              recml/layers/keras/hstu.py:33-55, 131-237
 */
#ifndef HSTU_ATTN_H_
#define HSTU_ATTN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HSTU_ATTN_ABI_VERSION 3

/* Tensor layouts of q, k, v, out. */
enum HstuLayout {
  HSTU_LAYOUT_PADDED = 0, /* [B, L, H, d]; strides given per tensor          */
  HSTU_LAYOUT_JAGGED = 1  /* [T, H, d] with seq_offsets[B+1]                  */
};

enum HstuDtype {
  HSTU_DTYPE_FP32 = 0,
  HSTU_DTYPE_BF16 = 1,
  HSTU_DTYPE_FP8_E4M3FN = 2 /* q and k only (v, out bf16); per-head scales in
                               q_scale / k_scale multiply the logits; not in
                               the reference (its README lists fp8 as roadmap) */
};

/* Which positions take part, on top of causal / window / explicit mask. */
enum HstuMaskMode {
  HSTU_MASK_NONE = 0,    /* all L x Lkv positions                             */
  HSTU_MASK_LENGTH = 1,  /* i < n_b and j < n_b; rows >= n_b are written as 0 */
  HSTU_MASK_SEGMENT = 2  /* q_segment_ids[b,i] == kv_segment_ids[b,j]         */
};

/* Bits of HstuAttnFwdArgs.flags. */
enum HstuFwdFlags {
  /* The workspace still holds what an earlier call prepared from the same
   * shapes, lengths / offsets, timestamps, bias tables and dense mask (for
   * example the same call repeated, or a benchmark timing the main kernel
   * alone): skip the preparation kernel.  Undefined results if that does not
   * hold. */
  HSTU_FWD_WORKSPACE_PREPARED = 1,
  /* Only prepare the workspace (the kernel that builds the work list, the scaled
   * tables, the int32 timestamps and the timestamp descriptors) and return: a model whose layers share
   * lengths, timestamps and bias tables prepares once per batch and then calls
   * every layer with HSTU_FWD_WORKSPACE_PREPARED and the same workspace. */
  HSTU_FWD_PREPARE_ONLY = 2,
  /* How the matrix-core kernel takes the entries of its work list (bf16,
   * d = 128, no dense operands, no segment ids; ignored elsewhere): one
   * workgroup per entry, or two resident workgroups per compute unit that
   * draw entry after entry and start the next one's loads under the last steps
   * of the one at hand.  By default the library picks the second when the
   * batch has at least 8 entries per resident workgroup.  These bits force one
   * or the other (the first wins); the results are the same bit for bit. */
  HSTU_FWD_ONE_ITEM_PER_WORKGROUP = 4,
  HSTU_FWD_RESIDENT_WORKGROUPS = 8,
  /* The matrix-core kernel at d = 128 in bf16 runs the steps that no mask touches
   * as one hand-scheduled instruction stream (software-pipelined across steps).
   * This bit sends those steps through the compiler-scheduled code that handles
   * every other step instead: a comparison switch; same arithmetic in the same
   * order, the same bits out.  In the `fwd` member of hstu_attn_bwd's arguments
   * it does the same to the backward's dK/dV kernel, which runs its unmasked
   * blocks without bias as such a stream at d = 128. */
  HSTU_FWD_COMPILER_SCHEDULED_BLOCKS = 16
};

/* Return codes (0 = launched). */
enum HstuStatus {
  HSTU_OK = 0,
  HSTU_ERR_NULL = -1,         /* a required pointer is null                   */
  HSTU_ERR_VERSION = -2,      /* struct_size / version mismatch               */
  HSTU_ERR_DTYPE = -3,        /* unsupported dtype combination                */
  HSTU_ERR_SHAPE = -4,        /* bad B/L/H/d, strides or option combination   */
  HSTU_ERR_WORKSPACE = -5,    /* workspace missing or too small               */
  HSTU_ERR_LAUNCH = -6        /* HIP reported an error at launch              */
};

typedef struct HstuAttnFwdArgs {
  uint32_t struct_size;   /* sizeof(HstuAttnFwdArgs)                          */
  uint32_t version;       /* HSTU_ATTN_ABI_VERSION                            */

  int32_t layout;         /* HstuLayout                                       */
  int32_t qk_dtype;       /* HstuDtype of q and k                             */
  int32_t v_dtype;        /* HstuDtype of v                                   */
  int32_t out_dtype;      /* HstuDtype of out (fp32 or bf16)                  */

  int32_t B;              /* sequences                                        */
  int32_t L;              /* max query length (padded length; bias geometry)  */
  int32_t Lkv;            /* max key length; == L except padded cross-length  */
  int32_t H;              /* heads                                            */
  int32_t d_qk;           /* head dim of q and k                              */
  int32_t d_v;            /* head dim of v and out                            */
  int64_t total_tokens;   /* T for the jagged layout, else ignored            */

  const void* q;
  const void* k;
  const void* v;
  void* out;
  /* Strides in ELEMENTS; the innermost (d) stride is 1.  *_stride_b is only
   * read for the padded layout. */
  int64_t q_stride_b, q_stride_t, q_stride_h;
  int64_t k_stride_b, k_stride_t, k_stride_h;
  int64_t v_stride_b, v_stride_t, v_stride_h;
  int64_t o_stride_b, o_stride_t, o_stride_h;

  float alpha;            /* logit scale: 1 or 1/sqrt(d)                      */
  float inv_n;            /* 1/N normaliser applied after SiLU                */

  int32_t causal;         /* 1: keep j <= i                                   */
  int32_t mask_mode;      /* HstuMaskMode                                     */
  int32_t window;         /* keep |i-j| <= window; < 0 disables               */
  int32_t flags;          /* HstuFwdFlags, 0 by default                       */

  const int32_t* seq_lens;     /* [B], LENGTH mode with the padded layout     */
  const int32_t* seq_offsets;  /* [B+1], jagged layout                        */
  const int32_t* q_segment_ids;  /* [B, L],   SEGMENT mode                    */
  const int32_t* kv_segment_ids; /* [B, Lkv], SEGMENT mode                    */

  /* Dense operands (the layer-side call of recml/layers/keras/hstu.py:356-390).  bf16 calls take
   * them on the matrix cores when Lkv is a multiple of 16 (mask) / 4 (bias), the arrays are
   * 16-byte aligned and no table bias or segment ids come with them; any other call on the
   * general kernel.  Key steps in which the mask keeps no pair of a query tile cost nothing
   * (a causal mask given as a matrix costs what the causal flag costs, plus reading it). */
  const uint8_t* mask;    /* explicit keep-mask (non-zero = keep) or null     */
  int32_t mask_batched;   /* 0: [L, Lkv] shared; 1: [B, L, Lkv]               */
  int32_t dense_bias_batched; /* 0: [L, Lkv] shared; 1: [B, L, Lkv]           */
  const float* dense_bias; /* additive logit bias shared by heads, or null    */

  const float* pos_tab;   /* [pos_heads, 2L-1] relative-position table / null */
  int32_t pos_heads;      /* 1 or H                                           */
  int32_t ts_heads;       /* 1 or H                                           */
  const float* ts_tab;    /* [ts_heads, ts_num_buckets+1] or null             */
  const int64_t* ts;      /* timestamps; padded [B, ts_stride_b] or jagged [T]*/
  int64_t ts_stride_b;    /* elements between sequences; 0 = jagged by
                             seq_offsets                                      */
  int32_t ts_num_buckets; /* clip bound; table has ts_num_buckets+1 entries   */
  float ts_bucket_size;   /* 0.301 in the reference                           */

  const float* q_scale;   /* [H] dequantisation scales (fp8 q); null = 1      */
  const float* k_scale;   /* [H] dequantisation scales (fp8 k); null = 1      */

  void* workspace;        /* device scratch of hstu_attn_fwd_workspace_bytes  */
  size_t workspace_bytes;

  /* Dropout on the attention weights (the training-mode step of
   * recml/layers/keras/hstu.py:386-387): each kept pair (b, h, i, j) is dropped
   * with probability dropout_p and the others are scaled by 1 / (1 - dropout_p).
   * Which pairs go is a function of (dropout_seed, b, h, i, j) alone -- a
   * counter-based hash, hstu_attn_dropout_keep below -- so the backward, given
   * the same two values, drops the same pairs, and a caller can reproduce the
   * mask.  0 (the default) switches it off.  With dropout the matrix-core
   * kernel runs every step through its compiler-scheduled block code.
   * Both values travel as kernel arguments: a HIP graph that recorded a call
   * replays that call's pattern until its kernel nodes are given new ones. */
  float dropout_p;        /* in [0, 1)                                        */
  uint32_t reserved0;     /* 0                                                */
  uint64_t dropout_seed;
} HstuAttnFwdArgs;

/* Whether dropout keeps pair (query i, key j) of sequence b and head h (of H
 * heads): the rule every kernel follows, as a host function for callers and
 * checkers.  i and j count from the start of the sequence.  Always 1 for
 * dropout_p = 0. */
int hstu_attn_dropout_keep(uint64_t dropout_seed, float dropout_p, int32_t b, int32_t h, int32_t H, int32_t i, int32_t j);

/* ABI version of the loaded library (HSTU_ATTN_ABI_VERSION at build time). */
int hstu_attn_abi_version(void);

/* Bytes of device scratch the call needs for these arguments; pass a buffer of
 * at least that size, 256-byte aligned, in args->workspace.  0 for calls the
 * general kernel serves.  For the matrix-core kernel it holds what a small
 * preparation kernel builds (on every call, or once per batch, see
 * HSTU_FWD_PREPARE_ONLY): the work list of (sequence, query tile, key chunk)
 * items, the scaled position table, the timestamp bucket tables, int32
 * timestamps with their per-tile ranges, for a timestamp bias at d = 128 in
 * bf16 under the causal mask one 16-bit descriptor per (query row, step of 32
 * keys) -- the bucket of the step's nearest key and how many of its keys lie one
 * bucket further, or a flag that says the step needs the per-pair lookup --
 * written by extra workgroups of the same preparation launch, for the steps below each 128-row tile (2 bytes x rows x ceil(L/32); left out, and
 * the per-pair lookup used throughout, for L above 16384, above 256 MiB, or
 * when the buffer is too small for them), for a dense mask the range of key
 * steps in which it keeps anything per tile of 128 query rows (the mask is
 * read once for that); and what the main kernel itself
 * uses: the counters it draws work from and, for query tiles whose keys are
 * split between workgroups (decided on the device from the lengths, when few
 * long tiles would otherwise finish long after the rest), the arrival counters
 * and up to 32 fp32 partial outputs of 128 rows x H heads x d_v, summed in a
 * fixed order by whichever workgroup of the tile arrives last: the result does
 * not depend on the order of arrival.  A larger buffer than asked for is fine;
 * a smaller one that still holds everything but the partial outputs makes the
 * library split fewer tiles (none below two) instead of failing.  The size
 * depends on shapes, options and total_tokens only, never on device data.
 * Counters are left at zero by every call; the rest means nothing between
 * calls unless HSTU_FWD_WORKSPACE_PREPARED says so; two calls that overlap on
 * one GPU need two buffers.  No reference counterpart: the reference's op is a
 * pure function under jax.jit. */
size_t hstu_attn_fwd_workspace_bytes(const HstuAttnFwdArgs* args);

/* Validate `args` and enqueue the forward on `stream` (a hipStream_t passed
 * as void* so that C callers need no HIP headers).  Returns an HstuStatus.
 * (Calls that the general kernel serves -- fp32 storage, head dims other than
 * 32 / 64 / 128, unaligned rows -- take at most 65535 sequences.)
 * Replaces recml/core/ops/hstu_ops.py:829-1046 and the dense path of
 * recml/layers/keras/hstu.py:356-390. */
int hstu_attn_fwd(const HstuAttnFwdArgs* args, void* stream);

/* Bytes of the scratch array built into the library that hstu_attn_fwd_noalloc
 * uses in place of a caller workspace (one copy per GPU the library runs on,
 * held until the process ends). */
#define HSTU_ATTN_NOALLOC_SCRATCH_BYTES (4u << 20)

/* hstu_attn_fwd for callers that cannot allocate device memory at all: code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  No counterpart in the reference (its op is a pure function under
 * jax.jit and XLA owns every buffer).  Same arguments, kernels and results as
 * hstu_attn_fwd, except that args->workspace / workspace_bytes are ignored:
 * the scratch that call would need (hstu_attn_fwd_workspace_bytes) lives in
 * a fixed array of HSTU_ATTN_NOALLOC_SCRATCH_BYTES inside the library.  The
 * call allocates and frees nothing, on the device or through any library.
 * Calls whose scratch need exceeds the array even with no tile split return
 * HSTU_ERR_WORKSPACE (use hstu_attn_fwd with a caller buffer then); between
 * that and the full need, fewer tiles are split, as with any small workspace.  Every call on a GPU shares that
 * GPU's array: calls that overlap on one GPU (two streams, two threads) race;
 * HSTU_FWD_WORKSPACE_PREPARED refers to what the previous call of this entry
 * point on the same GPU prepared. */
int hstu_attn_fwd_noalloc(const HstuAttnFwdArgs* args, void* stream);

/* Backward of the same op: gradients of sum(out * dout) with respect to q, k, v
 * and the two bias tables.  `fwd` describes the forward call (its `out` is
 * not used; its `workspace`, sized by hstu_attn_fwd_workspace_bytes, is
 * overwritten when the matrix-core kernels run, see below).  dout has the
 * layout, dtype and strides of out;
 * dq, dk, dv those of q, k, v and are fully written (rows past a sequence's
 * length as zeros).  dpos_tab / dts_tab are fp32 tables shaped like pos_tab /
 * ts_tab that are ACCUMULATED into by atomic adds: the caller zero-fills them
 * (or passes null when the table gradient is not wanted).  Those float atomic
 * adds arrive in no fixed order, so the table gradients may differ in their
 * last bits from run to run; out, dq, dk and dv are the same bits every run.  (Outside
 * the bf16 matrix-core pair: at most 65535 sequences per call, and a dts_tab of
 * at most 4096 entries.)  fp32 or bf16
 * storage, every option of the forward, fp32 arithmetic; fp8 q/k is not
 * supported.  bf16 calls that meet the conditions of the
 * matrix-core forward (without a dense mask or bias, and with keys and
 * queries of one length), pass 16-byte aligned gradient buffers and bring
 * the workspace run on the matrix cores instead (bf16 products, fp32
 * accumulation, table gradients included); every other bf16 call whose head
 * dims are multiples of 16 up to 128 and whose q, k, v, dout rows lie on
 * 16-byte boundaries keeps the general kernels but forms its products on the
 * bf16 matrix cores too (P and dS rounded to bf16 for the last products, as the
 * forward rounds P); hstu_attn_bwd_variant tells
 * which.  Math of recml/core/ops/hstu_ops.py:417-548 (dq, dk, dv), which
 * the reference reaches through jax.custom_vjp (hstu_ops.py:551-826), extended
 * by the table gradients that jax derives for recml/layers/keras/hstu.py:91-113,
 * 190-221. */
typedef struct HstuAttnBwdArgs {
  uint32_t struct_size;   /* sizeof(HstuAttnBwdArgs)                          */
  uint32_t version;       /* HSTU_ATTN_ABI_VERSION                            */
  HstuAttnFwdArgs fwd;
  const void* dout;
  void* dq;
  void* dk;
  void* dv;
  float* dpos_tab;
  float* dts_tab;
  /* Gradient of fwd.dense_bias, fp32, shaped like it ([L, Lkv] or [B, L, Lkv] by
   * fwd.dense_bias_batched): dS summed over the heads (and over the batch for a
   * shared bias), ACCUMULATED into by atomic adds like the table gradients (the
   * caller zero-fills; null = not wanted; needs fwd.dense_bias).  jax's derivative
   * of recml/layers/keras/hstu.py:373-374. */
  float* ddense_bias;
} HstuAttnBwdArgs;

int hstu_attn_bwd(const HstuAttnBwdArgs* args, void* stream);

/* Name of the kernel pair hstu_attn_bwd would launch for `args` (diagnostics;
 * static storage): "hstu_bwd_mfma_bf16", "hstu_bwd_general<float>", "hstu_bwd_general<bf16>",
 * "hstu_bwd_general<bf16, bf16 products>" or "invalid". */
const char* hstu_attn_bwd_variant(const HstuAttnBwdArgs* args);

/* Message for the last non-zero status on this thread ("" if none). */
const char* hstu_attn_last_error(void);

/* The timestamp bucket law every kernel here follows, as integer thresholds:
 *   bucket(dt) = min(floor(ln(fl32(clip(|dt|, 1, 1e9))) / bucket_size), ts_num_buckets)
 * -- recml/layers/keras/hstu.py:48-55 (float log and divide of the clipped
 * difference, truncated) with the logarithm and the quotient taken in double,
 * bucket_size being the float the caller passes.  thresholds[b], b < count,
 * receives the smallest clipped |dt| whose bucket (before the clip to
 * ts_num_buckets) is >= b, INT32_MAX where 1e9 does not reach b; thresholds[0]
 * is 1.  Host-only (no GPU work).  Returns the number of buckets 1e9 reaches
 * (its own bucket + 1), or a negative HstuStatus.  The reference evaluates
 * the same expression in float inside XLA; within a few hundred of a
 * threshold at the top of the range its rounding may differ, which no test
 * of the reference pins. */
int hstu_attn_bucket_thresholds(float bucket_size, int32_t* thresholds, int count);

/* Name of the kernel variant hstu_attn_fwd would launch for `args`
 * (diagnostics for profiles and benchmarks; static storage). */
const char* hstu_attn_fwd_variant(const HstuAttnFwdArgs* args);

#ifdef __cplusplus
}
#endif
#endif /* HSTU_ATTN_H_ */
