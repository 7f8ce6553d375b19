/* C ABI of libhstu_block.so: the fused steps of the HSTU block that sit on
 * either side of the attention kernel (recml/layers/keras/hstu.py:444-474) and
 * of the model's front end (hstu.py:593-601), for gfx950.  bf16 tensors, row-major, on the current device; fp32 arithmetic
 * inside.  Plain pointers and sizes: no framework types.
 *
 *   hstu_gemm_silu_fwd    out = silu(x W + bias): the U, Q, K, V projections of
 *                         the normalised input with their activation
 *                         (hstu.py:444-449, the EinsumDense layers of :281-330
 *                         with activation="silu"), as ONE matrix product with
 *                         the activation applied by the product's epilogue
 *                         (hipBLASLt) instead of a pass of its own.
 *   hstu_norm_gate_fwd    out = u * layer_norm(attn): the layer norm over
 *                         (heads, head_dim) of the attention output and the U
 *                         gate (hstu.py:471-472) in one pass over memory.
 *   hstu_norm_gate_bwd    the gradients of that step for training: of the
 *                         attention output, of U, of the norm's scale and
 *                         offset (what the framework's autodiff derives from
 *                         hstu.py:471-472); without a gate, the gradients of a
 *                         plain layer norm (the block's input norm,
 *                         hstu.py:442, and the model's final_norm).
 *   hstu_embed_norm_fwd   out = layer_norm(scale * table[ids] + pos_table[positions]):
 *                         the model's front end (hstu.py:593-601: item
 *                         embedding, optional sqrt(D) scale, position
 *                         embedding, final_norm) as one gather pass.
 *
 * Every function returns 0 or a negative HstuBlockStatus; the message of the
 * last failure on the calling thread is at hstu_block_last_error().
 */
#ifndef HSTU_BLOCK_H_
#define HSTU_BLOCK_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HSTU_BLOCK_ABI_VERSION 3

typedef enum HstuBlockStatus {
  HSTU_BLOCK_OK = 0,
  HSTU_BLOCK_ERR_NULL = -1,
  HSTU_BLOCK_ERR_VERSION = -2,
  HSTU_BLOCK_ERR_SHAPE = -4,
  HSTU_BLOCK_ERR_WORKSPACE = -5,
  HSTU_BLOCK_ERR_LAUNCH = -6,
  HSTU_BLOCK_ERR_BLAS = -7      /* hipBLASLt has no kernel for the request, or failed */
} HstuBlockStatus;

/* out[t, :] = u[t, :] * (gamma * (a[t, :] - mean_t) * rstd_t + beta), mean and
 * (biased) variance of a[t, :] over its `width` entries, rstd = 1/sqrt(var + eps)
 * (keras LayerNormalization over the last two axes of [.., H, hd] flattened,
 * hstu.py:340-346 and :471-472).  a, u, out: bf16 [rows, width] with the given
 * row strides in elements (u is usually a slice of the fused projection);
 * gamma, beta: bf16 [width].  width a multiple of 8 up to 8192; pointers and
 * row strides multiples of 8 elements (16 bytes).  u may be null: then
 * out = layer_norm(a), the plain norm (u_stride is ignored). */
typedef struct HstuNormGateArgs {
  uint32_t struct_size;   /* sizeof(HstuNormGateArgs)  */
  uint32_t version;       /* HSTU_BLOCK_ABI_VERSION    */
  int64_t rows;
  int32_t width;
  float eps;
  const void* a;
  const void* u;
  void* out;
  int64_t a_stride, u_stride, out_stride;
  const void* gamma;
  const void* beta;
} HstuNormGateArgs;

int hstu_norm_gate_fwd(const HstuNormGateArgs* args, void* stream);

/* Gradients of hstu_norm_gate_fwd for the gradient `dout` of its result (the
 * reference leaves these to autodiff of hstu.py:471-472 and of keras
 * LayerNormalization):
 *   da     bf16 [rows, width]  gradient of a
 *   du     bf16 [rows, width]  gradient of u (usually a slice of the gradient
 *                              of the fused projection: du_stride)
 *   dgamma, dbeta  fp32 [width], overwritten: sums over the rows, added in a
 *                              fixed order (the same bits on every run)
 * a, u, gamma, beta, eps as in the forward call; u and du null together: the
 * gradients of a plain layer norm.  width a multiple of 8 up to 2048; pointers
 * and row strides multiples of 8 elements.  `workspace`: device memory of
 * hstu_norm_gate_bwd_workspace_bytes(rows, width) bytes (one partial row of
 * column sums per workgroup), owned by the caller; the library allocates
 * nothing.  rows = 0 writes zeros to dgamma and dbeta. */
typedef struct HstuNormGateBwdArgs {
  uint32_t struct_size;   /* sizeof(HstuNormGateBwdArgs) */
  uint32_t version;       /* HSTU_BLOCK_ABI_VERSION      */
  int64_t rows;
  int32_t width;
  float eps;
  const void* a;
  const void* u;
  const void* dout;
  void* da;
  void* du;
  int64_t a_stride, u_stride, dout_stride, da_stride, du_stride;
  const void* gamma;
  const void* beta;
  float* dgamma;
  float* dbeta;
  void* workspace;
  size_t workspace_bytes;
} HstuNormGateBwdArgs;

size_t hstu_norm_gate_bwd_workspace_bytes(int64_t rows, int32_t width);
int hstu_norm_gate_bwd(const HstuNormGateBwdArgs* args, void* stream);

/* out[m, n] = silu(sum_k x[m, k] w[k, n] + bias[n]); x: bf16 [M, K] (row stride
 * x_stride), w: bf16 [K, N] contiguous, bias: bf16 [N] or null, out: bf16
 * [M, N] contiguous; with `c` (bf16 [M, N], row stride c_stride, 16-byte aligned,
 * c_stride a multiple of 8) out = act(x w + c + bias).  fp32 accumulation.  `workspace` (device memory, may be
 * null) is handed to hipBLASLt; hstu_gemm_silu_workspace_bytes() says how much
 * it would like.  The descriptor and the chosen algorithm of a shape are kept
 * by the library after the first call with it: every call must therefore offer
 * what the first did, so x, w, bias, out and workspace must be 16-byte aligned
 * and x_stride a multiple of 8 elements (HSTU_BLOCK_ERR_SHAPE otherwise). */
typedef struct HstuGemmSiluArgs {
  uint32_t struct_size;   /* sizeof(HstuGemmSiluArgs)  */
  uint32_t version;       /* HSTU_BLOCK_ABI_VERSION    */
  int64_t M;
  int32_t N, K;
  int32_t activation;     /* 1: silu (the projections); 0: none */
  int32_t reserved0;
  const void* x;
  int64_t x_stride;
  const void* w;
  const void* bias;
  void* out;
  void* workspace;
  size_t workspace_bytes;
  const void* c;          /* bf16 [M, N] added to the product before bias and activation, or null: the block's */
  int64_t c_stride;       /* residual as the product's C operand (hstu.py:474), no pass of its own; row stride */
} HstuGemmSiluArgs;

size_t hstu_gemm_silu_workspace_bytes(void);
int hstu_gemm_silu_fwd(const HstuGemmSiluArgs* args, void* stream);

/* out[t, :] = gamma * (x_t - mean) * rstd + beta with x_t = scale * table[ids[t], :]
 * (+ pos_table[positions[t], :] when pos_table is given), statistics over the
 * `width` entries of x_t as in hstu_norm_gate_fwd.  table: bf16 [vocab, width]
 * (row stride table_stride), pos_table: bf16 [n_positions, width] contiguous or
 * null, ids / positions: int64 [rows] (positions null with pos_table null),
 * out: bf16 [rows, width] contiguous.  Indices outside their table are clamped
 * into it (the reference's gather on an accelerator does the same).  width a
 * multiple of 8 up to 8192; pointers and table_stride multiples of 8 elements. */
typedef struct HstuEmbedNormArgs {
  uint32_t struct_size;   /* sizeof(HstuEmbedNormArgs) */
  uint32_t version;       /* HSTU_BLOCK_ABI_VERSION    */
  int64_t rows;
  int32_t width;
  float eps;
  float scale;            /* 1, or sqrt(model_dim) (scale_by_sqrt_dim) */
  int32_t reserved0;
  const int64_t* ids;
  const void* table;
  int64_t vocab, table_stride;
  const int64_t* positions;
  const void* pos_table;
  int64_t n_positions;
  const void* gamma;
  const void* beta;
  void* out;
} HstuEmbedNormArgs;

int hstu_embed_norm_fwd(const HstuEmbedNormArgs* args, void* stream);

int hstu_block_abi_version(void);
const char* hstu_block_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* HSTU_BLOCK_H_ */
