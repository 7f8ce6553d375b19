// Fused steps of the HSTU block around the attention kernel and of the model's front end, for
// gfx950 (MI355X): see include/hstu_block.h.
//
//   hstu_norm_gate   out = u * layer_norm(attn)   (recml/layers/keras/hstu.py:471-472)
//                    one wavefront per token row, 16 bytes per lane and trip: the row is read once,
//                    kept in registers for the two reductions (mean, then centred sum of squares) and
//                    written once: 3 x width x 2 bytes of HBM traffic per row, which is the bound.
//   hstu_norm_gate_bwd  the gradients of that step (and, without a gate, of a plain layer norm): one
//                    pass over the row, its gradient and the gate; column sums for dgamma / dbeta in
//                    registers, one partial row per workgroup, added in a fixed order by hstu_colsum.
//   gemm + silu      out = silu(x W + bias)       (hstu.py:444-449)
//                    hipBLASLt matrix product with the activation in its epilogue.
//   hstu_embed_norm  out = layer_norm(scale * table[ids] + pos_table[positions])   (hstu.py:593-601)
//                    the same one-wave-per-row scheme with a gathered row: one read of the table row
//                    (and of the small position table, which stays in cache), one write.

#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <map>
#include <mutex>
#include <tuple>

#include "hstu_block.h"

namespace {

typedef __bf16 bf16_t;
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

__device__ __forceinline__ void unpack8(const uint4& v, float (&f)[8]) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    f[2 * i] = __builtin_bit_cast(float, w[i] << 16);
    f[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
  }
}

__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  floatx2 f = {lo, hi};
  bf16x2 r = __builtin_convertvector(f, bf16x2);
  return __builtin_bit_cast(uint32_t, r);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, 64);
  return v;
}

struct NormGateParams {
  const bf16_t* a;
  const bf16_t* u;
  bf16_t* out;
  const bf16_t* gamma;
  const bf16_t* beta;
  int64_t rows, a_stride, u_stride, out_stride;
  int32_t width;
  float eps;
};

// One wavefront per row; lane l owns the 8-element pieces l, l + 64, ... of the row (CH of them at most).
template <int CH>
__global__ __launch_bounds__(256) void hstu_norm_gate(const NormGateParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= p.rows) return;
  const bf16_t* ar = p.a + row * p.a_stride;
  const bf16_t* ur = p.u ? p.u + row * p.u_stride : nullptr;   // no gate: the plain layer norm
  bf16_t* orow = p.out + row * p.out_stride;
  float x[CH][8];
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int e = (c * 64 + lane) * 8;
    if (e < p.width) {
      unpack8(*(const uint4*)(ar + e), x[c]);
#pragma unroll
      for (int i = 0; i < 8; ++i) sum += x[c][i];
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) x[c][i] = 0.f;
    }
  }
  const float mean = wave_sum(sum) / (float)p.width;
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int e = (c * 64 + lane) * 8;
    if (e < p.width) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float d = x[c][i] - mean;
        ss += d * d;
      }
    }
  }
  const float rstd = __builtin_amdgcn_rsqf(wave_sum(ss) / (float)p.width + p.eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int e = (c * 64 + lane) * 8;
    if (e < p.width) {
      float g[8], b[8], uu[8];
      unpack8(*(const uint4*)(p.gamma + e), g);
      unpack8(*(const uint4*)(p.beta + e), b);
      if (ur) {
        unpack8(*(const uint4*)(ur + e), uu);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) uu[i] = 1.f;
      }
      float y[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = uu[i] * __builtin_fmaf((x[c][i] - mean) * rstd, g[i], b[i]);
      uint4 o;
      o.x = pack2(y[0], y[1]);
      o.y = pack2(y[2], y[3]);
      o.z = pack2(y[4], y[5]);
      o.w = pack2(y[6], y[7]);
      *(uint4*)(orow + e) = o;
    }
  }
}

struct NormGateBwdParams {
  const bf16_t* a;
  const bf16_t* u;
  const bf16_t* dout;
  const bf16_t* gamma;
  const bf16_t* beta;
  bf16_t* da;
  bf16_t* du;
  float* partial;          // [gridDim.x][2 * width]: each workgroup's sums for dgamma, then for dbeta
  int64_t rows, a_stride, u_stride, dout_stride, da_stride, du_stride;
  int32_t width;
  float eps;
};

// Backward of out = u * (gamma * xhat + beta), xhat = (a - mean) * rstd, for the gradient g of out:
//   du = g * (gamma * xhat + beta),  gn = g * u  (the gradient at the normalised row; gn = g without a gate)
//   dgamma += gn * xhat,  dbeta += gn           (summed over the rows)
//   da = rstd * (gn gamma - mean_w(gn gamma) - xhat * mean_w(gn gamma xhat))
// One wavefront per row as in the forward, a workgroup walking over rows with the grid's stride: the row,
// its gradient and the gate are read once, da and du written once (5 x width x 2 bytes per row, the
// bound).  The two column sums stay in registers over a wave's rows, are added across the workgroup's
// four waves through LDS and leave as one partial row per workgroup; hstu_colsum adds those in a fixed
// order, so the result does not depend on the timing of the run.
template <int CH>
__global__ __launch_bounds__(256) void hstu_norm_gate_bwd(const NormGateBwdParams p) {
  __shared__ float red[4][CH * 512];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const float inv_w = 1.f / (float)p.width;
  float dg[CH][8], db[CH][8];
#pragma unroll
  for (int c = 0; c < CH; ++c)
#pragma unroll
    for (int i = 0; i < 8; ++i) dg[c][i] = db[c][i] = 0.f;
  for (int64_t row = (int64_t)blockIdx.x * 4 + w; row < p.rows; row += (int64_t)gridDim.x * 4) {
    const bf16_t* ar = p.a + row * p.a_stride;
    const bf16_t* gr = p.dout + row * p.dout_stride;
    float x[CH][8], g[CH][8];
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int e = (c * 64 + lane) * 8;
      if (e < p.width) {
        unpack8(*(const uint4*)(ar + e), x[c]);
        unpack8(*(const uint4*)(gr + e), g[c]);
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += x[c][i];
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) x[c][i] = g[c][i] = 0.f;
      }
    }
    const float mean = wave_sum(sum) * inv_w;
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int e = (c * 64 + lane) * 8;
      if (e < p.width) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float d = x[c][i] - mean;
          ss += d * d;
        }
      }
    }
    const float rstd = __builtin_amdgcn_rsqf(wave_sum(ss) * inv_w + p.eps);
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int e = (c * 64 + lane) * 8;
      if (e < p.width) {
        float gm[8];
        unpack8(*(const uint4*)(p.gamma + e), gm);
        if (p.u) {
          float bt[8], uu[8], y[8];
          unpack8(*(const uint4*)(p.beta + e), bt);
          unpack8(*(const uint4*)(p.u + row * p.u_stride + e), uu);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            y[i] = g[c][i] * __builtin_fmaf((x[c][i] - mean) * rstd, gm[i], bt[i]);
            g[c][i] *= uu[i];
          }
          uint4 o;
          o.x = pack2(y[0], y[1]);
          o.y = pack2(y[2], y[3]);
          o.z = pack2(y[4], y[5]);
          o.w = pack2(y[6], y[7]);
          *(uint4*)(p.du + row * p.du_stride + e) = o;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float xh = (x[c][i] - mean) * rstd;
          const float gn = g[c][i];
          x[c][i] = xh;
          dg[c][i] = __builtin_fmaf(gn, xh, dg[c][i]);
          db[c][i] += gn;
          const float gx = gn * gm[i];
          g[c][i] = gx;
          s1 += gx;
          s2 = __builtin_fmaf(gx, xh, s2);
        }
      }
    }
    const float c1 = wave_sum(s1) * inv_w, c2 = wave_sum(s2) * inv_w;
    bf16_t* dr = p.da + row * p.da_stride;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int e = (c * 64 + lane) * 8;
      if (e < p.width) {
        float y[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = rstd * (g[c][i] - c1 - x[c][i] * c2);
        uint4 o;
        o.x = pack2(y[0], y[1]);
        o.y = pack2(y[2], y[3]);
        o.z = pack2(y[4], y[5]);
        o.w = pack2(y[6], y[7]);
        *(uint4*)(dr + e) = o;
      }
    }
  }
  // the workgroup's column sums: every wave gets here, whatever rows it had
  float* part = p.partial + (int64_t)blockIdx.x * (2 * p.width);
#pragma unroll
  for (int half = 0; half < 2; ++half) {
#pragma unroll
    for (int c = 0; c < CH; ++c)
#pragma unroll
      for (int i = 0; i < 8; ++i) red[w][(c * 64 + lane) * 8 + i] = half == 0 ? dg[c][i] : db[c][i];
    __syncthreads();
    for (int col = threadIdx.x; col < p.width; col += 256)
      part[half * p.width + col] = (red[0][col] + red[1][col]) + (red[2][col] + red[3][col]);
    __syncthreads();
  }
}

// out[col] = sum over the nb partial rows of part[.][col], rows added in a fixed order; columns
// [0, width) go to dgamma, [width, 2 width) to dbeta.  nb = 0 writes zeros.  A workgroup of 1024
// threads takes 32 columns: 32 groups of threads each add every 32nd row (four sums in flight per
// thread: the loop is nothing but dependent loads otherwise), then the groups' sums are added through LDS.
__global__ __launch_bounds__(1024) void hstu_colsum(const float* __restrict__ part, int nb, int width, float* __restrict__ dgamma,
                                                    float* __restrict__ dbeta) {
  __shared__ float red[32][33];
  const int cl = threadIdx.x & 31, rg = threadIdx.x >> 5;
  const int col = blockIdx.x * 32 + cl, n2 = 2 * width;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (col < n2) {
    const float* pc = part + col;
    int r = rg;
    for (; r + 96 < nb; r += 128) {
      s0 += pc[(int64_t)r * n2];
      s1 += pc[(int64_t)(r + 32) * n2];
      s2 += pc[(int64_t)(r + 64) * n2];
      s3 += pc[(int64_t)(r + 96) * n2];
    }
    for (; r < nb; r += 32) s0 += pc[(int64_t)r * n2];
  }
  red[rg][cl] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (rg == 0 && col < n2) {
    float s = 0.f;
#pragma unroll
    for (int g = 0; g < 32; ++g) s += red[g][cl];
    if (col < width) dgamma[col] = s; else dbeta[col - width] = s;
  }
}

// workgroups of the backward kernel for this many rows (each walks over rows with the grid's stride)
int norm_gate_bwd_blocks(int64_t rows) {
  const int64_t nb = (rows + 3) / 4;
  return (int)(nb < 1 ? 1 : (nb > 1024 ? 1024 : nb));
}

struct EmbedNormParams {
  const int64_t* ids;
  const int64_t* positions;
  const bf16_t* table;
  const bf16_t* pos_table;
  const bf16_t* gamma;
  const bf16_t* beta;
  bf16_t* out;
  int64_t rows, vocab, table_stride, n_positions;
  int32_t width;
  float eps, scale;
};

// One wavefront per token: its table row (and position row) is gathered into registers, normalised
// there and written once.
template <int CH>
__global__ __launch_bounds__(256) void hstu_embed_norm(const EmbedNormParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= p.rows) return;
  int64_t id = p.ids[row];
  id = id < 0 ? 0 : (id >= p.vocab ? p.vocab - 1 : id);
  const bf16_t* er = p.table + id * p.table_stride;
  const bf16_t* pr = nullptr;
  if (p.pos_table) {
    int64_t ps = p.positions[row];
    ps = ps < 0 ? 0 : (ps >= p.n_positions ? p.n_positions - 1 : ps);
    pr = p.pos_table + ps * (int64_t)p.width;
  }
  float x[CH][8];
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int e = (c * 64 + lane) * 8;
    if (e < p.width) {
      unpack8(*(const uint4*)(er + e), x[c]);
      if (pr) {
        float pe[8];
        unpack8(*(const uint4*)(pr + e), pe);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[c][i] = __builtin_fmaf(x[c][i], p.scale, pe[i]);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) x[c][i] *= p.scale;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) sum += x[c][i];
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) x[c][i] = 0.f;
    }
  }
  const float mean = wave_sum(sum) / (float)p.width;
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int e = (c * 64 + lane) * 8;
    if (e < p.width) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float d = x[c][i] - mean;
        ss += d * d;
      }
    }
  }
  const float rstd = __builtin_amdgcn_rsqf(wave_sum(ss) / (float)p.width + p.eps);
  bf16_t* orow = p.out + row * (int64_t)p.width;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int e = (c * 64 + lane) * 8;
    if (e < p.width) {
      float g[8], b[8], y[8];
      unpack8(*(const uint4*)(p.gamma + e), g);
      unpack8(*(const uint4*)(p.beta + e), b);
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = __builtin_fmaf((x[c][i] - mean) * rstd, g[i], b[i]);
      uint4 o;
      o.x = pack2(y[0], y[1]);
      o.y = pack2(y[2], y[3]);
      o.z = pack2(y[4], y[5]);
      o.w = pack2(y[6], y[7]);
      *(uint4*)(orow + e) = o;
    }
  }
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// ---- hipBLASLt side -------------------------------------------------------

constexpr size_t kBlasWorkspace = 32u << 20;

struct GemmPlan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t la = nullptr, lb = nullptr, lc = nullptr, lres = nullptr;   // lres: the C operand when it is not the output
  hipblasLtMatmulAlgo_t algo;
  size_t workspace = 0;
};

struct BlasState {
  std::mutex mu;
  hipblasLtHandle_t handle[64] = {};
  // (device, M, N, K, x_stride, bias?, activation, workspace offered, row stride of c or 0) -> plan
  std::map<std::tuple<int, int64_t, int, int, int64_t, int, int, size_t, int64_t>, GemmPlan> plans;
};

BlasState& blas() {
  static BlasState s;
  return s;
}

const char* blas_str(hipblasStatus_t st) {
  switch (st) {
    case HIPBLAS_STATUS_SUCCESS: return "success";
    case HIPBLAS_STATUS_NOT_INITIALIZED: return "not initialized";
    case HIPBLAS_STATUS_ALLOC_FAILED: return "allocation failed";
    case HIPBLAS_STATUS_INVALID_VALUE: return "invalid value";
    case HIPBLAS_STATUS_NOT_SUPPORTED: return "not supported";
    case HIPBLAS_STATUS_EXECUTION_FAILED: return "execution failed";
    default: return "error";
  }
}

}  // namespace

extern "C" {

int hstu_block_abi_version(void) { return HSTU_BLOCK_ABI_VERSION; }

const char* hstu_block_last_error(void) { return g_err; }

int hstu_norm_gate_fwd(const HstuNormGateArgs* a, void* stream) {
  if (!a) return fail(HSTU_BLOCK_ERR_NULL, "args is null");
  if (a->struct_size != sizeof(HstuNormGateArgs) || a->version != HSTU_BLOCK_ABI_VERSION)
    return fail(HSTU_BLOCK_ERR_VERSION, "norm-gate args struct_size/version (%u/%u) do not match this library (%zu/%d)",
                a->struct_size, a->version, sizeof(HstuNormGateArgs), HSTU_BLOCK_ABI_VERSION);
  if (a->rows < 0 || a->width < 8 || a->width > 8192 || (a->width & 7))
    return fail(HSTU_BLOCK_ERR_SHAPE, "rows >= 0 and width a multiple of 8 in [8, 8192] expected, got rows=%lld width=%d",
                (long long)a->rows, a->width);
  g_err[0] = 0;
  if (a->rows == 0) return HSTU_BLOCK_OK;
  if (!a->a || !a->out || !a->gamma || !a->beta) return fail(HSTU_BLOCK_ERR_NULL, "a, out, gamma and beta must be non-null");
  if (!aligned16(a->a) || !aligned16(a->u) || !aligned16(a->out) || !aligned16(a->gamma) || !aligned16(a->beta) ||
      (a->a_stride & 7) || (a->out_stride & 7) || a->a_stride < a->width || a->out_stride < a->width ||
      (a->u && ((a->u_stride & 7) || a->u_stride < a->width)))
    return fail(HSTU_BLOCK_ERR_SHAPE, "pointers must be 16-byte aligned, row strides multiples of 8 elements and >= width");
  if ((a->rows + 3) / 4 > 0x7fffffffLL) return fail(HSTU_BLOCK_ERR_SHAPE, "too many rows");
  NormGateParams p;
  p.a = (const bf16_t*)a->a; p.u = (const bf16_t*)a->u; p.out = (bf16_t*)a->out;
  p.gamma = (const bf16_t*)a->gamma; p.beta = (const bf16_t*)a->beta;
  p.rows = a->rows; p.a_stride = a->a_stride; p.u_stride = a->u_stride; p.out_stride = a->out_stride;
  p.width = a->width; p.eps = a->eps;
  const dim3 grid((unsigned)((a->rows + 3) / 4)), block(256);
  hipStream_t st = (hipStream_t)stream;
  const int ch = (a->width + 511) / 512;
  if (ch <= 1) hipLaunchKernelGGL(hstu_norm_gate<1>, grid, block, 0, st, p);
  else if (ch <= 2) hipLaunchKernelGGL(hstu_norm_gate<2>, grid, block, 0, st, p);
  else if (ch <= 4) hipLaunchKernelGGL(hstu_norm_gate<4>, grid, block, 0, st, p);
  else hipLaunchKernelGGL(hstu_norm_gate<16>, grid, block, 0, st, p);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(HSTU_BLOCK_ERR_LAUNCH, "norm-gate kernel launch: %s", hipGetErrorString(e));
  return HSTU_BLOCK_OK;
}

size_t hstu_norm_gate_bwd_workspace_bytes(int64_t rows, int32_t width) {
  if (rows < 0 || width < 8) return 0;
  return (size_t)norm_gate_bwd_blocks(rows) * 2u * (size_t)width * sizeof(float);
}

int hstu_norm_gate_bwd(const HstuNormGateBwdArgs* a, void* stream) {
  if (!a) return fail(HSTU_BLOCK_ERR_NULL, "args is null");
  if (a->struct_size != sizeof(HstuNormGateBwdArgs) || a->version != HSTU_BLOCK_ABI_VERSION)
    return fail(HSTU_BLOCK_ERR_VERSION, "norm-gate backward args struct_size/version (%u/%u) do not match this library (%zu/%d)",
                a->struct_size, a->version, sizeof(HstuNormGateBwdArgs), HSTU_BLOCK_ABI_VERSION);
  if (a->rows < 0 || a->width < 8 || a->width > 2048 || (a->width & 7))
    return fail(HSTU_BLOCK_ERR_SHAPE, "rows >= 0 and width a multiple of 8 in [8, 2048] expected, got rows=%lld width=%d",
                (long long)a->rows, a->width);
  g_err[0] = 0;
  if (!a->dgamma || !a->dbeta) return fail(HSTU_BLOCK_ERR_NULL, "dgamma and dbeta must be non-null");
  hipStream_t st = (hipStream_t)stream;
  const int nb = a->rows == 0 ? 0 : norm_gate_bwd_blocks(a->rows);
  if (nb > 0) {
    if (!a->a || !a->dout || !a->da || !a->gamma || !a->beta) return fail(HSTU_BLOCK_ERR_NULL, "a, dout, da, gamma and beta must be non-null");
    if ((a->u == nullptr) != (a->du == nullptr)) return fail(HSTU_BLOCK_ERR_NULL, "u and du go together (both null: the plain layer norm)");
    if (!aligned16(a->a) || !aligned16(a->u) || !aligned16(a->dout) || !aligned16(a->da) || !aligned16(a->du) ||
        !aligned16(a->gamma) || !aligned16(a->beta) ||
        (a->a_stride & 7) || (a->dout_stride & 7) || (a->da_stride & 7) ||
        a->a_stride < a->width || a->dout_stride < a->width || a->da_stride < a->width ||
        (a->u && ((a->u_stride & 7) || (a->du_stride & 7) || a->u_stride < a->width || a->du_stride < a->width)))
      return fail(HSTU_BLOCK_ERR_SHAPE, "pointers must be 16-byte aligned, row strides multiples of 8 elements and >= width");
    const size_t need = hstu_norm_gate_bwd_workspace_bytes(a->rows, a->width);
    if (!a->workspace || a->workspace_bytes < need || ((uintptr_t)a->workspace & 3u))
      return fail(HSTU_BLOCK_ERR_WORKSPACE, "workspace of %zu bytes needed (hstu_norm_gate_bwd_workspace_bytes), got %zu", need,
                  a->workspace ? a->workspace_bytes : (size_t)0);
    NormGateBwdParams p;
    p.a = (const bf16_t*)a->a; p.u = (const bf16_t*)a->u; p.dout = (const bf16_t*)a->dout;
    p.gamma = (const bf16_t*)a->gamma; p.beta = (const bf16_t*)a->beta;
    p.da = (bf16_t*)a->da; p.du = (bf16_t*)a->du; p.partial = (float*)a->workspace;
    p.rows = a->rows; p.a_stride = a->a_stride; p.u_stride = a->u_stride; p.dout_stride = a->dout_stride;
    p.da_stride = a->da_stride; p.du_stride = a->du_stride; p.width = a->width; p.eps = a->eps;
    const dim3 grid((unsigned)nb), block(256);
    const int ch = (a->width + 511) / 512;
    if (ch <= 1) hipLaunchKernelGGL(hstu_norm_gate_bwd<1>, grid, block, 0, st, p);
    else if (ch <= 2) hipLaunchKernelGGL(hstu_norm_gate_bwd<2>, grid, block, 0, st, p);
    else hipLaunchKernelGGL(hstu_norm_gate_bwd<4>, grid, block, 0, st, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_BLOCK_ERR_LAUNCH, "norm-gate backward kernel launch: %s", hipGetErrorString(e));
  }
  hipLaunchKernelGGL(hstu_colsum, dim3((unsigned)((2 * a->width + 31) / 32)), dim3(1024), 0, st, (const float*)a->workspace, nb, a->width,
                     a->dgamma, a->dbeta);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(HSTU_BLOCK_ERR_LAUNCH, "column-sum kernel launch: %s", hipGetErrorString(e));
  return HSTU_BLOCK_OK;
}

int hstu_embed_norm_fwd(const HstuEmbedNormArgs* a, void* stream) {
  if (!a) return fail(HSTU_BLOCK_ERR_NULL, "args is null");
  if (a->struct_size != sizeof(HstuEmbedNormArgs) || a->version != HSTU_BLOCK_ABI_VERSION)
    return fail(HSTU_BLOCK_ERR_VERSION, "embed-norm args struct_size/version (%u/%u) do not match this library (%zu/%d)",
                a->struct_size, a->version, sizeof(HstuEmbedNormArgs), HSTU_BLOCK_ABI_VERSION);
  if (a->rows < 0 || a->width < 8 || a->width > 8192 || (a->width & 7) || a->vocab < 1)
    return fail(HSTU_BLOCK_ERR_SHAPE, "rows >= 0, vocab >= 1 and width a multiple of 8 in [8, 8192] expected, got rows=%lld vocab=%lld width=%d",
                (long long)a->rows, (long long)a->vocab, a->width);
  g_err[0] = 0;
  if (a->rows == 0) return HSTU_BLOCK_OK;
  if (!a->ids || !a->table || !a->out || !a->gamma || !a->beta) return fail(HSTU_BLOCK_ERR_NULL, "ids, table, out, gamma and beta must be non-null");
  if ((a->pos_table != nullptr) != (a->positions != nullptr) || (a->pos_table && a->n_positions < 1))
    return fail(HSTU_BLOCK_ERR_NULL, "pos_table and positions go together (with n_positions >= 1)");
  if (!aligned16(a->table) || !aligned16(a->pos_table) || !aligned16(a->out) || !aligned16(a->gamma) || !aligned16(a->beta) ||
      (a->table_stride & 7) || a->table_stride < a->width)
    return fail(HSTU_BLOCK_ERR_SHAPE, "pointers must be 16-byte aligned, table_stride a multiple of 8 elements and >= width");
  if ((a->rows + 3) / 4 > 0x7fffffffLL) return fail(HSTU_BLOCK_ERR_SHAPE, "too many rows");
  EmbedNormParams p;
  p.ids = a->ids; p.positions = a->positions;
  p.table = (const bf16_t*)a->table; p.pos_table = (const bf16_t*)a->pos_table;
  p.gamma = (const bf16_t*)a->gamma; p.beta = (const bf16_t*)a->beta; p.out = (bf16_t*)a->out;
  p.rows = a->rows; p.vocab = a->vocab; p.table_stride = a->table_stride; p.n_positions = a->n_positions;
  p.width = a->width; p.eps = a->eps; p.scale = a->scale;
  const dim3 grid((unsigned)((a->rows + 3) / 4)), block(256);
  hipStream_t st = (hipStream_t)stream;
  const int ch = (a->width + 511) / 512;
  if (ch <= 1) hipLaunchKernelGGL(hstu_embed_norm<1>, grid, block, 0, st, p);
  else if (ch <= 2) hipLaunchKernelGGL(hstu_embed_norm<2>, grid, block, 0, st, p);
  else if (ch <= 4) hipLaunchKernelGGL(hstu_embed_norm<4>, grid, block, 0, st, p);
  else hipLaunchKernelGGL(hstu_embed_norm<16>, grid, block, 0, st, p);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(HSTU_BLOCK_ERR_LAUNCH, "embed-norm kernel launch: %s", hipGetErrorString(e));
  return HSTU_BLOCK_OK;
}

size_t hstu_gemm_silu_workspace_bytes(void) { return kBlasWorkspace; }

int hstu_gemm_silu_fwd(const HstuGemmSiluArgs* a, void* stream) {
  if (!a) return fail(HSTU_BLOCK_ERR_NULL, "args is null");
  if (a->struct_size != sizeof(HstuGemmSiluArgs) || a->version != HSTU_BLOCK_ABI_VERSION)
    return fail(HSTU_BLOCK_ERR_VERSION, "gemm args struct_size/version (%u/%u) do not match this library (%zu/%d)",
                a->struct_size, a->version, sizeof(HstuGemmSiluArgs), HSTU_BLOCK_ABI_VERSION);
  if (a->M < 0 || a->N < 1 || a->K < 1 || a->M > 0x7fffffffLL || a->x_stride < a->K)
    return fail(HSTU_BLOCK_ERR_SHAPE, "bad shape M=%lld N=%d K=%d x_stride=%lld", (long long)a->M, a->N, a->K, (long long)a->x_stride);
  if (a->activation != 0 && a->activation != 1) return fail(HSTU_BLOCK_ERR_SHAPE, "activation must be 0 (none) or 1 (silu)");
  g_err[0] = 0;
  if (a->M == 0) return HSTU_BLOCK_OK;
  if (!a->x || !a->w || !a->out) return fail(HSTU_BLOCK_ERR_NULL, "x, w and out must be non-null");
  // the kernel picked for a shape is kept and reused for every later call of that shape: it may assume what
  // the first call's pointers offered, so every call has to offer it
  if (!aligned16(a->x) || !aligned16(a->w) || !aligned16(a->out) || !aligned16(a->bias) || !aligned16(a->workspace) || (a->x_stride & 7))
    return fail(HSTU_BLOCK_ERR_SHAPE, "x, w, out, bias and workspace must be 16-byte aligned and x_stride a multiple of 8 elements");
  if (a->c && (!aligned16(a->c) || (a->c_stride & 7) || a->c_stride < a->N))
    return fail(HSTU_BLOCK_ERR_SHAPE, "c must be 16-byte aligned with a row stride that is a multiple of 8 elements and >= N");
  if (a->workspace_bytes && !a->workspace) return fail(HSTU_BLOCK_ERR_WORKSPACE, "workspace_bytes without a workspace");
  int dev = 0;
  hipError_t he = hipGetDevice(&dev);
  if (he != hipSuccess) return fail(HSTU_BLOCK_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(he));
  if (dev < 0 || dev >= 64) return fail(HSTU_BLOCK_ERR_LAUNCH, "device index %d out of range", dev);

  BlasState& bs = blas();
  GemmPlan plan;
  hipblasLtHandle_t handle;
  {
    std::lock_guard<std::mutex> lock(bs.mu);
    if (!bs.handle[dev]) {
      const hipblasStatus_t st = hipblasLtCreate(&bs.handle[dev]);
      if (st != HIPBLAS_STATUS_SUCCESS) return fail(HSTU_BLOCK_ERR_BLAS, "hipblasLtCreate: %s", blas_str(st));
    }
    handle = bs.handle[dev];
    const auto key = std::make_tuple(dev, a->M, a->N, a->K, a->x_stride, a->bias ? 1 : 0, a->activation, a->workspace_bytes,
                                     a->c ? a->c_stride : (int64_t)0);
    auto it = bs.plans.find(key);
    if (it == bs.plans.end()) {
      // row-major out[M, N] = x[M, K] w[K, N] is, in the column-major terms of the library,
      // out^T [N x M] = w^T [N x K] x^T [K x M] with leading dimensions N, x_stride and N
      // (built in a holder that frees whatever exists of the plan on every early return)
      struct Partial {
        GemmPlan p{};
        hipblasLtMatmulPreference_t pref = nullptr;
        bool keep = false;
        ~Partial() {
          if (pref) hipblasLtMatmulPreferenceDestroy(pref);
          if (keep) return;
          if (p.la) hipblasLtMatrixLayoutDestroy(p.la);
          if (p.lb) hipblasLtMatrixLayoutDestroy(p.lb);
          if (p.lc) hipblasLtMatrixLayoutDestroy(p.lc);
          if (p.lres) hipblasLtMatrixLayoutDestroy(p.lres);
          if (p.desc) hipblasLtMatmulDescDestroy(p.desc);
        }
      } part;
      GemmPlan& np = part.p;
      hipblasStatus_t st = hipblasLtMatmulDescCreate(&np.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F);
      if (st != HIPBLAS_STATUS_SUCCESS) return fail(HSTU_BLOCK_ERR_BLAS, "hipblasLtMatmulDescCreate: %s", blas_str(st));
      // every attribute is checked: a rejected epilogue or bias type would otherwise come back as "no kernel",
      // or as a product without its epilogue
      auto set_desc = [&](hipblasLtMatmulDescAttributes_t attr, const void* val, size_t bytes) {
        return hipblasLtMatmulDescSetAttribute(np.desc, attr, val, bytes);
      };
      const hipblasOperation_t op_n = HIPBLAS_OP_N;
      st = set_desc(HIPBLASLT_MATMUL_DESC_TRANSA, &op_n, sizeof(op_n));
      if (st == HIPBLAS_STATUS_SUCCESS) st = set_desc(HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n));
      hipblasLtEpilogue_t epi = HIPBLASLT_EPILOGUE_DEFAULT;
      if (a->activation == 1) epi = a->bias ? HIPBLASLT_EPILOGUE_SWISH_BIAS_EXT : HIPBLASLT_EPILOGUE_SWISH_EXT;
      else if (a->bias) epi = HIPBLASLT_EPILOGUE_BIAS;
      if (st == HIPBLAS_STATUS_SUCCESS) st = set_desc(HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi));
      if (st == HIPBLAS_STATUS_SUCCESS && a->bias) {
        const hipDataType bt = HIP_R_16BF;
        st = set_desc(HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt));
        // the heuristic looks at the pointer's presence; the real one is set on every call below
        if (st == HIPBLAS_STATUS_SUCCESS) st = set_desc(HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &a->bias, sizeof(void*));
      }
      if (st != HIPBLAS_STATUS_SUCCESS)
        return fail(HSTU_BLOCK_ERR_BLAS, "hipblasLtMatmulDescSetAttribute (epilogue %d, bias %d): %s", (int)epi, a->bias ? 1 : 0, blas_str(st));
      st = hipblasLtMatrixLayoutCreate(&np.la, HIP_R_16BF, (uint64_t)a->N, (uint64_t)a->K, (int64_t)a->N);
      if (st == HIPBLAS_STATUS_SUCCESS) st = hipblasLtMatrixLayoutCreate(&np.lb, HIP_R_16BF, (uint64_t)a->K, (uint64_t)a->M, a->x_stride);
      if (st == HIPBLAS_STATUS_SUCCESS) st = hipblasLtMatrixLayoutCreate(&np.lc, HIP_R_16BF, (uint64_t)a->N, (uint64_t)a->M, (int64_t)a->N);
      if (st == HIPBLAS_STATUS_SUCCESS && a->c)
        st = hipblasLtMatrixLayoutCreate(&np.lres, HIP_R_16BF, (uint64_t)a->N, (uint64_t)a->M, a->c_stride);
      if (st != HIPBLAS_STATUS_SUCCESS) return fail(HSTU_BLOCK_ERR_BLAS, "hipblasLtMatrixLayoutCreate: %s", blas_str(st));
      st = hipblasLtMatmulPreferenceCreate(&part.pref);
      if (st != HIPBLAS_STATUS_SUCCESS) return fail(HSTU_BLOCK_ERR_BLAS, "hipblasLtMatmulPreferenceCreate: %s", blas_str(st));
      const uint64_t ws = a->workspace_bytes;
      st = hipblasLtMatmulPreferenceSetAttribute(part.pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws));
      if (st != HIPBLAS_STATUS_SUCCESS) return fail(HSTU_BLOCK_ERR_BLAS, "hipblasLtMatmulPreferenceSetAttribute: %s", blas_str(st));
      hipblasLtMatmulHeuristicResult_t res[1];
      int found = 0;
      st = hipblasLtMatmulAlgoGetHeuristic(handle, np.desc, np.la, np.lb, a->c ? np.lres : np.lc, np.lc, part.pref, 1, res, &found);
      if (st != HIPBLAS_STATUS_SUCCESS || found < 1)
        return fail(HSTU_BLOCK_ERR_BLAS, "hipBLASLt has no kernel for M=%lld N=%d K=%d with this epilogue (%s)",
                    (long long)a->M, a->N, a->K, blas_str(st));
      np.algo = res[0].algo;
      np.workspace = res[0].workspaceSize;
      if (bs.plans.size() >= 256) {
        for (auto& kv : bs.plans) {
          hipblasLtMatrixLayoutDestroy(kv.second.la);
          hipblasLtMatrixLayoutDestroy(kv.second.lb);
          hipblasLtMatrixLayoutDestroy(kv.second.lc);
          if (kv.second.lres) hipblasLtMatrixLayoutDestroy(kv.second.lres);
          hipblasLtMatmulDescDestroy(kv.second.desc);
        }
        bs.plans.clear();
      }
      it = bs.plans.emplace(key, np).first;
      part.keep = true;
    }
    plan = it->second;
    // the descriptor is shared by every call of this shape: the bias pointer is set under the lock
    // and the product is enqueued before it is released
    if (a->bias) {
      const hipblasStatus_t sb = hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &a->bias, sizeof(void*));
      if (sb != HIPBLAS_STATUS_SUCCESS) return fail(HSTU_BLOCK_ERR_BLAS, "hipblasLtMatmulDescSetAttribute (bias pointer): %s", blas_str(sb));
    }
    // (with c: D = alpha A B + beta C with C = c and beta = 1, the output written elsewhere)
    const float alpha = 1.0f, beta = a->c ? 1.0f : 0.0f;
    const hipblasStatus_t st = hipblasLtMatmul(handle, plan.desc, &alpha, a->w, plan.la, a->x, plan.lb, &beta, a->c ? a->c : a->out,
                                               a->c ? plan.lres : plan.lc, a->out, plan.lc, &plan.algo, a->workspace, a->workspace_bytes,
                                               (hipStream_t)stream);
    if (st != HIPBLAS_STATUS_SUCCESS) return fail(HSTU_BLOCK_ERR_BLAS, "hipblasLtMatmul: %s", blas_str(st));
  }
  return HSTU_BLOCK_OK;
}

}  // extern "C"
