// Microbenchmark of the forward kernel's 32 x 32 block on its own: the issue time of a wave-block
// with the K / V tiles already in LDS (no global loads, no workgroup barrier), two waves per SIMD
// on every CU, for
//   * the block as the compiler schedules it from C++ (logits, pointwise part, P V one after another),
//   * the hand-scheduled stream of gen_fwd_stream.py (hstu_fwd_stream_d128.inc),
// each checked against a host computation of the same sums.  The LDS layout (unpadded 32 x 128 bf16
// tiles with XOR-swizzled 16-byte chunks, four shifted copies of the position window) and the
// fragment addressing are those of hstu_fwd_mfma_bf16<128, ...> in hstu_attn.hip.
//
// Build: hipcc -O3 -std=c++17 --offload-arch=gfx950 -Xclang -target-feature -Xclang -packed-fp32-ops
//        -o micro_fwd_stream micro_fwd_stream.hip
// Run:   ./micro_fwd_stream [rounds [zero_operands [probes]]]        (one JSON line per variant)
//        zero_operands: bit 0 K, bit 1 V, bit 2 Q all zero (the same instructions on data that toggles no bits);
//        probes 0: the blocks only, not the instruction-rate probes
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

#define CK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__); exit(1); } } while (0)

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v* lds_short4_ptr;

constexpr int D = 128, BN = 32, BM = 128, NSTAGE = 4;
constexpr int K_BYTES = BN * D * 2, STAGE = 2 * K_BYTES;
constexpr int POS_LANES = (BM + BN - 1 + 3 + 3) / 4, POS_COPY = POS_LANES * 16, POS_BYTES = 4 * POS_COPY;
constexpr int WIN = BM + BN - 1 + 3;                 // window entries a copy must hold
constexpr int BIAS_OFF = NSTAGE * STAGE;
constexpr int LDS_BYTES = BIAS_OFF + NSTAGE * POS_BYTES;
constexpr float LOG2E = 1.4426950408889634f;

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  floatx2 f = {lo, hi};
  bf16x2 r = __builtin_convertvector(f, bf16x2);
  return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ uint2 lds_read_tr(const unsigned char* p) {
  short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)p);
  return __builtin_bit_cast(uint2, v);
}

// K tile: 16-byte chunk c of row r at chunk c ^ (r % 16); V tile: at chunk c ^ 4 (r % 4).
__device__ __forceinline__ void fill_lds(unsigned char* smem, const bf16_t* kg, const bf16_t* vg, const float* wing) {
  for (int i = threadIdx.x; i < NSTAGE * BN * 16; i += blockDim.x) {
    const int st = i / (BN * 16), r = (i / 16) % BN, c = i % 16;
    const uint4 kv = *(const uint4*)(kg + ((size_t)st * BN + r) * D + c * 8);
    const uint4 vv = *(const uint4*)(vg + ((size_t)st * BN + r) * D + c * 8);
    *(uint4*)(smem + st * STAGE + r * 256 + ((c ^ (r % 16)) * 16)) = kv;
    *(uint4*)(smem + st * STAGE + K_BYTES + r * 256 + ((c ^ (4 * (r & 3))) * 16)) = vv;
  }
  for (int i = threadIdx.x; i < NSTAGE * 4 * (POS_COPY / 4); i += blockDim.x) {
    const int st = i / (4 * (POS_COPY / 4)), c = (i / (POS_COPY / 4)) % 4, x = i % (POS_COPY / 4);
    const int xi = x + c;
    ((float*)(smem + BIAS_OFF + st * POS_BYTES + c * POS_COPY))[x] = xi < WIN ? wing[st * WIN + xi] : 0.f;
  }
}

struct LaneAddr { uint32_t ka[8], va[4], pa; };
__device__ __forceinline__ LaneAddr lane_addresses(uint32_t smem_lds) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, m = lane & 31, hh = lane >> 5;
  LaneAddr a;
  const int gk = m % 16;
  for (int ks = 0; ks < 8; ++ks) a.ka[ks] = smem_lds + m * 256 + (((2 * ks + hh) ^ gk) * 16);
  const int gi = lane & 15, vrow = 4 * hh + (gi >> 2), gq = vrow & 3, vc2 = 2 * ((lane >> 4) & 1) + ((gi & 3) >> 1);
  for (int d = 0; d < 4; ++d) a.va[d] = smem_lds + K_BYTES + vrow * 256 + 8 * (gi & 1) + vc2 * 16 + ((d ^ gq) & 3) * 64;
  const int xb = 4 * hh + (BM - 1) - 32 * w - m, sft = xb & 3;
  a.pa = smem_lds + BIAS_OFF + sft * POS_COPY + (xb - sft) * 4;
  return a;
}

__device__ __forceinline__ void load_q(uintx4 (&qf)[8], const bf16_t* qg) {
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, m = lane & 31, hh = lane >> 5;
  const bf16_t* row = qg + (size_t)(32 * w + m) * D + 8 * hh;
  for (int ks = 0; ks < 8; ++ks) qf[ks] = *(const uintx4*)(row + 16 * ks);
}
__device__ __forceinline__ void store_o(const floatx16 (&o)[4], float* og) {
  // O^T[dv = 32 dvb + 8g + 4hh + t][q]; written as og[wg][q row of the workgroup][dv]
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, m = lane & 31, hh = lane >> 5;
  float* row = og + ((size_t)blockIdx.x * BM + 32 * w + m) * D;
  for (int d = 0; d < 4; ++d)
    for (int r = 0; r < 16; ++r) row[32 * d + 8 * (r >> 2) + 4 * hh + (r & 3)] = o[d][r];
}

// ---- the block as the compiler schedules it (the C++ of hstu_fwd_mfma_bf16's `block`, no masks)
template <bool POS>
__global__ __launch_bounds__(256, 2) void k_cpp(const bf16_t* qg, const bf16_t* kg, const bf16_t* vg, const float* wing, float alpha2,
                                              int rounds, float* og, long long* cyc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  fill_lds(smem, kg, vg, wing);
  uintx4 qf[8];
  load_q(qf, qg);
  __syncthreads();
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, m = lane & 31, hh = lane >> 5;
  const int gk = m % 16, gi = lane & 15, vrow = 4 * hh + (gi >> 2), gq = vrow & 3, vc2 = 2 * ((lane >> 4) & 1) + ((gi & 3) >> 1);
  floatx16 o[4];
  for (int d = 0; d < 4; ++d) for (int r = 0; r < 16; ++r) o[d][r] = 0.f;
  const long long rt0 = wall_clock64();
  const long long t0 = clock64();
  for (int rd = 0; rd < rounds; ++rd) {
#pragma unroll
    for (int st = 0; st < NSTAGE; ++st) {
      floatx16 sacc;
      {
        uint4 kf[8];
        const unsigned char* kr = smem + st * STAGE + m * 256;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) kf[ks] = *(const uint4*)(kr + (((2 * ks + hh) ^ gk) * 16));
        const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
          sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[ks]), __builtin_bit_cast(bf16x8, qf[ks]), ks == 0 ? zero : sacc, 0, 0, 0);
      }
      uint4 vf[2][4];
      {
        const unsigned char* vr = smem + st * STAGE + K_BYTES + vrow * 256 + 8 * (gi & 1);
#pragma unroll
        for (int cc = 0; cc < 2; ++cc)
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            const int pch = (4 * ((d ^ gq) & 3) + vc2) * 16;
            uint2 lo = lds_read_tr(vr + (16 * cc) * 256 + pch);
            uint2 hi = lds_read_tr(vr + (16 * cc + 8) * 256 + pch);
            vf[cc][d] = uint4{lo.x, lo.y, hi.x, hi.y};
          }
      }
      float u[16];
      if (POS) {
        const int xb = 4 * hh + (BM - 1) - 32 * w - m, sft = xb & 3;
        const float* wrow = (const float*)(smem + BIAS_OFF + st * POS_BYTES + sft * POS_COPY) + (xb - sft);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float4 bv = *(const float4*)(wrow + 8 * g);
          u[4 * g + 0] = __builtin_fmaf(sacc[4 * g + 0], alpha2, bv.x);
          u[4 * g + 1] = __builtin_fmaf(sacc[4 * g + 1], alpha2, bv.y);
          u[4 * g + 2] = __builtin_fmaf(sacc[4 * g + 2], alpha2, bv.z);
          u[4 * g + 3] = __builtin_fmaf(sacc[4 * g + 3], alpha2, bv.w);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) u[r] = sacc[r] * alpha2;
      }
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        float e[8];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < 8; ++r) e[r] = __builtin_amdgcn_exp2f(-u[8 * cc + r]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < 8; ++r) e[r] = 1.0f + e[r];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < 8; ++r) e[r] = __builtin_amdgcn_rcpf(e[r]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int r = 0; r < 8; ++r) e[r] = u[8 * cc + r] * e[r];
        uint4 pk = {pack_bf16(e[0], e[1]), pack_bf16(e[2], e[3]), pack_bf16(e[4], e[5]), pack_bf16(e[6], e[7])};
        const bf16x8 pb = __builtin_bit_cast(bf16x8, pk);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int d = 0; d < 4; ++d) o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf[cc][d]), pb, o[d], 0, 0, 0);
      }
    }
  }
  const long long t1 = clock64();
  const long long rt1 = wall_clock64();
  store_o(o, og);
  if (lane == 0) { cyc[blockIdx.x * 4 + w] = t1 - t0; if (blockIdx.x == 0 && w == 0) cyc[gridDim.x * 4] = rt1 - rt0; }
}

// ---- the hand-scheduled stream
#include "hstu_fwd_stream_d128.inc"
template <bool POS>
__global__ __launch_bounds__(256, 2) void k_stream(const bf16_t* qg, const bf16_t* kg, const bf16_t* vg, const float* wing, float alpha2,
                                                 int rounds, float* og, long long* cyc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  fill_lds(smem, kg, vg, wing);
  uintx4 hs_q[8];
  load_q(hs_q, qg);
  __syncthreads();
  const LaneAddr a = lane_addresses(__builtin_amdgcn_groupstaticsize());
  uint32_t hs_ka[8], hs_va[4], hs_pa = a.pa;
  for (int i = 0; i < 8; ++i) hs_ka[i] = a.ka[i];
  for (int i = 0; i < 4; ++i) hs_va[i] = a.va[i];
  floatx16 hs_o[4];
  for (int d = 0; d < 4; ++d) for (int r = 0; r < 16; ++r) hs_o[d][r] = 0.f;
  float hs_alpha = alpha2;
  int hs_n = rounds;
  const long long rt0 = wall_clock64();
  const long long t0 = clock64();
  if constexpr (POS) {
#define HSTU_STREAM_VARIANT HSTU_STREAM_COMPUTE_ONLY_POS
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
  } else {
#define HSTU_STREAM_VARIANT HSTU_STREAM_COMPUTE_ONLY
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
    (void)hs_pa;
  }
  const long long t1 = clock64();
  const long long rt1 = wall_clock64();
  store_o(hs_o, og);
  if ((threadIdx.x & 63) == 0) cyc[blockIdx.x * 4 + (threadIdx.x >> 6)] = t1 - t0;
  if (threadIdx.x == 0 && blockIdx.x == 0) cyc[gridDim.x * 4] = rt1 - rt0;
}

// ---- the stream as the kernel runs it: tiles streamed from global memory by direct loads, one barrier per pair of steps
__device__ __forceinline__ void lds_dma16(const void* gbase_uniform, uint32_t byte_off, uint32_t lds_addr_wave_uniform) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(lds_addr_wave_uniform);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(base), "v"(byte_off), "s"(gbase_uniform) : "memory", "m0");
}
template <bool POS>
__global__ __launch_bounds__(256, 2) void k_stream_dma(const bf16_t* qg, const bf16_t* kg, const bf16_t* vg, const float* ptab, float alpha2,
                                                     int rounds, int reps, float* og, long long* cyc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uintx4 hs_q[8];
  load_q(hs_q, qg);
  const uint32_t smem_lds = __builtin_amdgcn_groupstaticsize();
  const LaneAddr a = lane_addresses(smem_lds);
  uint32_t hs_ka[8], hs_va[4], hs_pa = a.pa;
  for (int i = 0; i < 8; ++i) hs_ka[i] = a.ka[i];
  for (int i = 0; i < 4; ++i) hs_va[i] = a.va[i];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // wave w brings 1 KB pieces 2w, 2w+1 of a K and of a V tile; lane l of piece j lands at 16-byte chunk 64 j + l
  uint32_t hs_koff[2], hs_voff[2];
  for (int r = 0; r < 2; ++r) {
    const int c = 64 * (2 * w + r) + lane, row = c / 16, pc = c % 16;
    hs_koff[r] = (uint32_t)row * 256u + (uint32_t)((pc ^ (row % 16)) * 16);
    hs_voff[r] = (uint32_t)row * 256u + (uint32_t)((pc ^ (4 * (row & 3))) * 16);
  }
  const uint32_t hs_kdst = smem_lds + 2 * w * 1024, hs_vdst = smem_lds + K_BYTES + 2 * w * 1024;
  const uint32_t hs_kstep = BN * 256, hs_vstep = BN * 256;
  const uint32_t hs_bdst = smem_lds + BIAS_OFF + w * POS_COPY;
  const uint32_t hs_boff = (uint32_t)(w + 4 * lane) * 4u;
  const uint64_t hs_bexec = (1ull << POS_LANES) - 1ull;
  floatx16 hs_o[4];
  for (int d = 0; d < 4; ++d) for (int r = 0; r < 16; ++r) hs_o[d][r] = 0.f;
  float hs_alpha = alpha2;
  const long long rt0 = wall_clock64();
  const long long t0 = clock64();
  for (int rep = 0; rep < reps; ++rep) {
    // steps 0 and 1: K and V tiles, position windows
    for (int t = 0; t < 2; ++t) {
      for (int r = 0; r < 2; ++r) lds_dma16((const char*)kg + (size_t)t * hs_kstep, hs_koff[r], hs_kdst + t * STAGE + r * 1024);
      if (POS && lane < POS_LANES) lds_dma16((const char*)ptab + (size_t)t * 128, hs_boff, hs_bdst + t * POS_BYTES);
      for (int r = 0; r < 2; ++r) lds_dma16((const char*)vg + (size_t)t * hs_vstep, hs_voff[r], hs_vdst + t * STAGE + r * 1024);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const char* hs_kp = (const char*)kg + (size_t)2 * hs_kstep;
    const char* hs_vp = (const char*)vg + (size_t)2 * hs_vstep;
    const char* hs_bp = (const char*)ptab + (size_t)2 * 128;
    int hs_n = rounds;
    if constexpr (POS) {
#define HSTU_STREAM_VARIANT HSTU_STREAM_FULL_POS
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
    } else {
#define HSTU_STREAM_VARIANT HSTU_STREAM_FULL
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
      (void)hs_pa; (void)hs_bp; (void)hs_bdst; (void)hs_boff; (void)hs_bexec;
    }
  }
  const long long t1 = clock64();
  const long long rt1 = wall_clock64();
  store_o(hs_o, og);
  if (lane == 0) cyc[blockIdx.x * 4 + w] = t1 - t0;
  if (threadIdx.x == 0 && blockIdx.x == 0) cyc[gridDim.x * 4] = rt1 - rt0;
}

__device__ __forceinline__ void lds_dma16(const void* gbase_uniform, uint32_t byte_off, uint32_t lds_addr_wave_uniform);
// ---- the generator's sweep (gen_fwd_stream.py --experiments FILE; build with -DHSTU_STREAM_EXPERIMENTS='"FILE"')
#ifdef HSTU_STREAM_EXPERIMENTS
#define HS_PARAMS floatx16 (&hs_o)[4], const uintx4 (&hs_q)[8], const uint32_t (&hs_ka)[8], const uint32_t (&hs_va)[4], uint32_t hs_pa, \
    float hs_alpha, int& hs_n, uint32_t hs_kdst, uint32_t hs_vdst, uint32_t hs_kstep, uint32_t hs_vstep, const uint32_t (&hs_koff)[2], \
    const uint32_t (&hs_voff)[2], const char* hs_kp, const char* hs_vp, uint32_t hs_bdst, uint32_t hs_boff, uint64_t hs_bexec, const char* hs_bp
template <int V> __device__ __forceinline__ void hs_exp(HS_PARAMS);
#include HSTU_STREAM_EXPERIMENTS
template <int V, bool FULL>
__global__ __launch_bounds__(256, 2) void k_exp(const bf16_t* qg, const bf16_t* kg, const bf16_t* vg, const float* ptab, float alpha2,
                                              int rounds, int reps, float* og, long long* cyc) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  if (!FULL) fill_lds(smem, kg, vg, ptab);
  uintx4 hs_q[8];
  load_q(hs_q, qg);
  __syncthreads();
  const uint32_t smem_lds = __builtin_amdgcn_groupstaticsize();
  const LaneAddr a = lane_addresses(smem_lds);
  uint32_t hs_ka[8], hs_va[4], hs_pa = a.pa;
  for (int i = 0; i < 8; ++i) hs_ka[i] = a.ka[i];
  for (int i = 0; i < 4; ++i) hs_va[i] = a.va[i];
  const int lane = threadIdx.x & 63;
  const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  uint32_t hs_koff[2], hs_voff[2];
  for (int r = 0; r < 2; ++r) {
    const int c = 64 * (2 * w + r) + lane, row = c / 16, pc = c % 16;
    hs_koff[r] = (uint32_t)row * 256u + (uint32_t)((pc ^ (row % 16)) * 16);
    hs_voff[r] = (uint32_t)row * 256u + (uint32_t)((pc ^ (4 * (row & 3))) * 16);
  }
  const uint32_t hs_kdst = smem_lds + 2 * w * 1024, hs_vdst = smem_lds + K_BYTES + 2 * w * 1024;
  const uint32_t hs_kstep = BN * 256, hs_vstep = BN * 256;
  const uint32_t hs_bdst = smem_lds + BIAS_OFF + w * POS_COPY;
  const uint32_t hs_boff = (uint32_t)(w + 4 * lane) * 4u;
  const uint64_t hs_bexec = (1ull << POS_LANES) - 1ull;
  floatx16 hs_o[4];
  for (int d = 0; d < 4; ++d) for (int r = 0; r < 16; ++r) hs_o[d][r] = 0.f;
  const long long t0 = clock64();
  for (int rep = 0; rep < reps; ++rep) {
    if (FULL) {
      for (int t = 0; t < 2; ++t) {
        for (int r = 0; r < 2; ++r) lds_dma16((const char*)kg + (size_t)t * hs_kstep, hs_koff[r], hs_kdst + t * STAGE + r * 1024);
        if (lane < POS_LANES) lds_dma16((const char*)ptab + (size_t)t * 128, hs_boff, hs_bdst + t * POS_BYTES);
        for (int r = 0; r < 2; ++r) lds_dma16((const char*)vg + (size_t)t * hs_vstep, hs_voff[r], hs_vdst + t * STAGE + r * 1024);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
    int hs_n = rounds;
    hs_exp<V>(hs_o, hs_q, hs_ka, hs_va, hs_pa, alpha2, hs_n, hs_kdst, hs_vdst, hs_kstep, hs_vstep, hs_koff, hs_voff,
              (const char*)kg + (size_t)2 * hs_kstep, (const char*)vg + (size_t)2 * hs_vstep, hs_bdst, hs_boff, hs_bexec, (const char*)ptab + (size_t)2 * 128);
  }
  const long long t1 = clock64();
  store_o(hs_o, og);
  if (lane == 0) cyc[blockIdx.x * 4 + w] = t1 - t0;
}
#endif

// ---- what the clock does under load: a wave of nothing but matrix instructions (MODE 0), nothing but exp2 (MODE 1)
template <int MODE>
__global__ __launch_bounds__(256, 2) void k_clock(int iters, float* out, long long* cyc, long long* rt) {
  floatx16 acc[4];
  for (int d = 0; d < 4; ++d) for (int r = 0; r < 16; ++r) acc[d][r] = 0.f;
  uintx4 a = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u}, b = a;
  float x[8];
  for (int i = 0; i < 8; ++i) x[i] = threadIdx.x * 1e-3f + i;
  __shared__ __attribute__((aligned(16))) unsigned char lbuf[36864];
  for (int i = threadIdx.x; i < 36864 / 4; i += 256) ((uint32_t*)lbuf)[i] = 0x3f803f80u;
  __syncthreads();
  // the K fragment read's pattern: one 256-byte row per lane, 16-byte chunk swizzled by the row
  const uint32_t laddr = (threadIdx.x & 31) * 256 + ((((threadIdx.x >> 5) & 1) ^ (threadIdx.x & 15)) * 16);
  uintx4 lv[4] = {a, a, a, a};
  typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
  uintx2 lt[4] = {{0u, 0u}, {0u, 0u}, {0u, 0u}, {0u, 0u}};
  // operands of modes 19 and 20: a hash of (lane, register, word) as two bf16 values each, exponents 126..127
  uintx4 ra[4], rb[4];
  for (int i = 0; i < 4; ++i)
    for (int c = 0; c < 4; ++c) {
      uint32_t h = (threadIdx.x * 16u + i * 4u + c) * 2654435761u;
      h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
      const uint32_t g = h * 3266489917u ^ (h >> 16);
      ra[i][c] = (h & 0x80ff80ffu) | 0x3f003f00u;
      rb[i][c] = (g & 0x80ff80ffu) | 0x3f003f00u;
    }
  const long long r0 = wall_clock64(), t0 = clock64();
  for (int it = 0; it < iters; ++it) {
    if (MODE == 0) {
#pragma unroll
      for (int j = 0; j < 16; ++j) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
    } else if (MODE == 2) {       // a matrix instruction, then four exp2 of the same wave
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
#pragma unroll
        for (int i = 0; i < 4; ++i) asm volatile("v_exp_f32 %0, %0" : "+v"(x[(4 * j + i) & 7]));
      }
    } else if (MODE == 3) {       // a matrix instruction, then two exp2 and four multiplications (the block's mix)
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[0]));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[1]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[2]) : "v"(1.0001f));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[3]));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[4]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[5]) : "v"(1.0001f));
      }
    } else if (MODE == 4) {       // the same vector mix without the matrix instruction
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[0]));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[1]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[2]) : "v"(1.0001f));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[3]));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[4]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[5]) : "v"(1.0001f));
      }
    } else if (MODE == 6) {       // 16-byte LDS reads only
#pragma unroll
      for (int j = 0; j < 32; ++j) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(lv[j & 3]) : "v"(laddr), "n"((j & 7) * 4096));
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    } else if (MODE == 7) {       // transpose reads only
#pragma unroll
      for (int j = 0; j < 32; ++j) asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lt[j & 3]) : "v"(laddr), "n"((j & 7) * 4096));
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    } else if (MODE == 8) {       // the block's matrix and LDS instructions without the vector part: 16 x (mfma, 0.5 b128, 1 tr_b64)
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
        if (j & 1) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(lv[(j >> 1) & 3]) : "v"(laddr), "n"((j & 7) * 4096));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lt[j & 3]) : "v"(laddr), "n"((j & 7) * 4096 + 2048));
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    } else if (MODE == 9) {       // the block's whole mix, nothing depending on anything near: 16 x (mfma, 2 exp2, 4 mul, 0.5 b128 (+ 0.25 for a window), 1 tr_b64)
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[0]));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[1]) : "v"(1.0001f));
        if (j & 1) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(lv[(j >> 1) & 3]) : "v"(laddr), "n"((j & 7) * 4096));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[2]) : "v"(1.0001f));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[3]));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lt[j & 3]) : "v"(laddr), "n"((j & 7) * 4096 + 2048));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[4]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[5]) : "v"(1.0001f));
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    } else if (MODE == 12) {      // a wave of 64 rows: per 32 keys twice the matrix and vector work for the same fragment reads
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[0]));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[1]) : "v"(1.0001f));
        if ((j & 3) == 1) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(lv[(j >> 2) & 3]) : "v"(laddr), "n"((j & 7) * 4096));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[2]) : "v"(1.0001f));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[3]));
        if (j & 1) asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lt[j & 3]) : "v"(laddr), "n"((j & 7) * 4096 + 2048));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[4]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[5]) : "v"(1.0001f));
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    } else if (MODE == 13) {      // matrix instruction + 2 exp2
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[0]));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[3]));
      }
    } else if (MODE == 14) {      // matrix instruction + 4 mul
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[1]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[2]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[4]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[5]) : "v"(1.0001f));
      }
    } else if (MODE == 15) {      // matrix instruction + 6 packed f16 fma
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
#pragma unroll
        for (int i = 0; i < 6; ++i) asm volatile("v_pk_fma_f16 %0, %0, %1, %0" : "+v"(x[i]) : "v"(1.0001f));
      }
    } else if (MODE == 16) {      // packed f16 fma only
#pragma unroll
      for (int j = 0; j < 64; ++j) asm volatile("v_pk_fma_f16 %0, %0, %1, %0" : "+v"(x[j & 7]) : "v"(1.0001f));
    } else if (MODE == 17) {      // matrix instruction + 8 mul
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[i]) : "v"(1.0001f));
      }
    } else if (MODE == 18) {      // matrix instruction + 12 mul
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(a), "v"(b));
#pragma unroll
        for (int i = 0; i < 12; ++i) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[i & 7]) : "v"(1.0001f));
      }
    } else if (MODE == 19 || MODE == 20) {
      // matrix instructions alone (19) or with the block's vector mix (20), on operands whose bits differ from lane
      // to lane and from one instruction to the next (bf16 values of either sign between 0.5 and 2): the same
      // instructions as modes 0 and 3, which multiply ones, with the data paths toggling as they do on real tiles
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[j & 3]) : "v"(ra[j & 3]), "v"(rb[(j >> 2) & 3]));
        if (MODE == 20) {
          asm volatile("v_exp_f32 %0, %0" : "+v"(x[0]));
          asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[1]) : "v"(1.0001f));
          asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[2]) : "v"(1.0001f));
          asm volatile("v_exp_f32 %0, %0" : "+v"(x[3]));
          asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[4]) : "v"(1.0001f));
          asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[5]) : "v"(1.0001f));
        }
      }
    } else if (MODE == 10) {      // one chain of dependent matrix instructions
#pragma unroll
      for (int j = 0; j < 16; ++j) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[0]) : "v"(a), "v"(b));
    } else if (MODE == 11) {      // chains of 8 dependent ones, the first of a chain starting from zero (the logits' pattern), + the vector mix
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        if ((j & 7) == 0) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=v"(acc[0]) : "v"(a), "v"(b));
        else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[0]) : "v"(a), "v"(b));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[0]));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[1]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[2]) : "v"(1.0001f));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[3]));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[4]) : "v"(1.0001f));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[5]) : "v"(1.0001f));
      }
    } else if (MODE == 5) {       // multiplications only
#pragma unroll
      for (int j = 0; j < 64; ++j) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[j & 7]) : "v"(1.0001f));
    } else {
#pragma unroll
      for (int j = 0; j < 64; ++j) asm volatile("v_exp_f32 %0, %0" : "+v"(x[j & 7]));
    }
  }
  const long long t1 = clock64(), r1 = wall_clock64();
  float sum = 0.f;
  for (int d = 0; d < 4; ++d) for (int r = 0; r < 16; ++r) sum += acc[d][r];
  for (int i = 0; i < 8; ++i) sum += x[i];
  for (int i = 0; i < 4; ++i) sum += (float)(lv[i].x + lv[i].w + lt[i].x + lt[i].y);
  out[blockIdx.x * 256 + threadIdx.x] = sum;
  if ((threadIdx.x & 63) == 0) { cyc[blockIdx.x * 4 + (threadIdx.x >> 6)] = t1 - t0; rt[blockIdx.x * 4 + (threadIdx.x >> 6)] = r1 - r0; }
}
template <int MODE>
static void run_clock(const char* name, int iters, int n_wg, int groups_per_iter) {
  float* out; long long *cyc, *rt;
  CK(hipMalloc(&out, (size_t)n_wg * 256 * 4)); CK(hipMalloc(&cyc, (size_t)n_wg * 32)); CK(hipMalloc(&rt, (size_t)n_wg * 32));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  float ms = 0.f;
  for (int rep = 0; rep < 4; ++rep) {
    CK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(k_clock<MODE>, dim3(n_wg), dim3(256), 0, 0, iters, out, cyc, rt);
    CK(hipEventRecord(e1, 0));
    CK(hipDeviceSynchronize());
    CK(hipEventElapsedTime(&ms, e0, e1));
  }
  std::vector<long long> c((size_t)n_wg * 4), r((size_t)n_wg * 4);
  CK(hipMemcpy(c.data(), cyc, c.size() * 8, hipMemcpyDeviceToHost));
  CK(hipMemcpy(r.data(), rt, r.size() * 8, hipMemcpyDeviceToHost));
  double cs = 0, rs = 0;
  for (size_t i = 0; i < c.size(); ++i) { cs += (double)c[i]; rs += (double)r[i]; }
  // wall_clock64 ticks at 100 MHz
  // two waves per SIMD: a SIMD issues 2 x iters x groups_per_iter groups during the kernel
  printf("{\"variant\": \"%s\", \"workgroups\": %d, \"iters\": %d, \"kernel_ms\": %.3f, \"ns_per_group_per_simd\": %.2f, \"s_memtime_ticks_per_wave\": %.0f, "
         "\"s_memrealtime_ticks_per_wave\": %.0f}\n",
         name, n_wg, iters, ms, ms * 1e6 / (2.0 * n_wg / (2.0 * 256) * iters * groups_per_iter), cs / c.size(), rs / r.size());
  fflush(stdout);
  CK(hipFree(out)); CK(hipFree(cyc)); CK(hipFree(rt));
}

// ---- host
static float bf16_round(float x) {
  uint32_t b; memcpy(&b, &x, 4);
  b += 0x7fffu + ((b >> 16) & 1u);
  b &= 0xffff0000u;
  float y; memcpy(&y, &b, 4);
  return y;
}
static uint16_t bf16_bits(float x) { float y = bf16_round(x); uint32_t b; memcpy(&b, &y, 4); return (uint16_t)(b >> 16); }
static float frand(uint32_t& s) { s = s * 1664525u + 1013904223u; return ((s >> 8) & 0xffff) / 32768.0f - 1.0f; }

// What the operands' values cost (second argument of the program): bit 0 makes K all zero, bit 1 V, bit 2 Q.
// The instruction stream and its timing rules are the same; what changes is how many bits toggle in the matrix
// cores' and the register file's data paths, i.e. the power the chip draws, and with it the clock it sustains.
static int g_zero_data = 0;

template <typename KernelT>
static void run(const char* name, KernelT kern, bool pos, int rounds, int n_wg) {
  std::vector<float> q(BM * D), k(NSTAGE * BN * D), v(NSTAGE * BN * D), win(NSTAGE * WIN);
  uint32_t seed = 12345u;
  for (auto& x : q) x = bf16_round(0.3f * frand(seed));
  for (auto& x : k) x = bf16_round(0.3f * frand(seed));
  for (auto& x : v) x = bf16_round(0.3f * frand(seed));
  for (auto& x : win) x = 0.05f * frand(seed) * LOG2E;
  if (g_zero_data & 1) for (auto& x : k) x = 0.f;
  if (g_zero_data & 2) for (auto& x : v) x = 0.f;
  if (g_zero_data & 4) for (auto& x : q) x = 0.f;
  const float alpha2 = LOG2E;
  std::vector<uint16_t> qb(q.size()), kb(k.size()), vb(v.size());
  for (size_t i = 0; i < q.size(); ++i) qb[i] = bf16_bits(q[i]);
  for (size_t i = 0; i < k.size(); ++i) kb[i] = bf16_bits(k[i]);
  for (size_t i = 0; i < v.size(); ++i) vb[i] = bf16_bits(v[i]);
  // reference: one pass over the four stages, times the rounds
  std::vector<double> ref(BM * D, 0.0);
  for (int st = 0; st < NSTAGE; ++st)
    for (int r = 0; r < BM; ++r)
      for (int j = 0; j < BN; ++j) {
        double s = 0;
        for (int c = 0; c < D; ++c) s += (double)q[r * D + c] * k[(st * BN + j) * D + c];
        double u = s * alpha2;
        if (pos) u += win[st * WIN + (BM - 1) - r + j];
        const float p = bf16_round((float)(u / (1.0 + exp2(-u))));
        for (int c = 0; c < D; ++c) ref[r * D + c] += (double)p * v[(st * BN + j) * D + c];
      }
  bf16_t *dq, *dk, *dv; float *dwin, *dout; long long* dcyc;
  CK(hipMalloc(&dq, qb.size() * 2)); CK(hipMalloc(&dk, kb.size() * 2)); CK(hipMalloc(&dv, vb.size() * 2));
  CK(hipMalloc(&dwin, win.size() * 4)); CK(hipMalloc(&dout, (size_t)n_wg * BM * D * 4)); CK(hipMalloc(&dcyc, ((size_t)n_wg * 4 + 1) * 8));
  CK(hipMemcpy(dq, qb.data(), qb.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dk, kb.data(), kb.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dv, vb.data(), vb.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dwin, win.data(), win.size() * 4, hipMemcpyHostToDevice));
  CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  float ms = 0.f;
  for (int rep = 0; rep < 3; ++rep) {
    CK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(kern, dim3(n_wg), dim3(256), LDS_BYTES, 0, dq, dk, dv, dwin, alpha2, rounds, dout, dcyc);
    CK(hipEventRecord(e1, 0));
    CK(hipDeviceSynchronize());
    CK(hipEventElapsedTime(&ms, e0, e1));
  }
  std::vector<float> out((size_t)n_wg * BM * D);
  std::vector<long long> cyc((size_t)n_wg * 4);
  CK(hipMemcpy(out.data(), dout, out.size() * 4, hipMemcpyDeviceToHost));
  CK(hipMemcpy(cyc.data(), dcyc, cyc.size() * 8, hipMemcpyDeviceToHost));
  long long rt_ticks = 0;
  CK(hipMemcpy(&rt_ticks, dcyc + (size_t)n_wg * 4, 8, hipMemcpyDeviceToHost));
  const double mhz = (double)cyc[0] / ((double)rt_ticks / 100.0);
  double max_ref = 0, max_err = 0;
  for (size_t i = 0; i < ref.size(); ++i) max_ref = fmax(max_ref, fabs(ref[i] * rounds));
  for (int g = 0; g < n_wg; g += (n_wg > 8 ? n_wg / 8 : 1))
    for (size_t i = 0; i < ref.size(); ++i) max_err = fmax(max_err, fabs(out[(size_t)g * BM * D + i] - ref[i] * rounds));
  double cyc_sum = 0; long long cyc_max = 0;
  for (auto c : cyc) { cyc_sum += (double)c; cyc_max = c > cyc_max ? c : cyc_max; }
  const double blocks = 4.0 * rounds;           // blocks per wave
  // two waves per SIMD when the grid holds two workgroups per CU: a SIMD's time per wave-block is half a wave's
  printf("{\"variant\": \"%s\", \"zero_operands\": %d, \"pos_bias\": %s, \"workgroups\": %d, \"rounds\": %d, \"kernel_ms\": %.4f, "
         "\"wave_cycles_per_block_avg\": %.1f, \"wave_cycles_per_block_max\": %.1f, \"simd_cycles_per_wave_block\": %.1f, "
         "\"mfma_cycles_per_block\": 512, \"clock_mhz\": %.0f, \"tflops\": %.0f, \"max_abs_err_over_max_ref\": %.3e}\n",
         name, g_zero_data, pos ? "true" : "false", n_wg, rounds, ms, cyc_sum / cyc.size() / blocks, (double)cyc_max / blocks,
         cyc_sum / cyc.size() / blocks / 2.0, mhz, 4.0 * n_wg * blocks * 16 * 32768 / (ms * 1e-3) * 1e-12, max_ref > 0 ? max_err / max_ref : max_err);
  fflush(stdout);
  CK(hipFree(dq)); CK(hipFree(dk)); CK(hipFree(dv)); CK(hipFree(dwin)); CK(hipFree(dout)); CK(hipFree(dcyc));
}

template <typename KernelT>
static void run_dma(const char* name, KernelT kern, bool pos, int rounds, int reps, int n_wg) {
  const int T = 4 * rounds, TP = T + 8;       // steps computed, steps allocated (the stream loads up to four steps ahead)
  std::vector<float> q(BM * D), k((size_t)TP * BN * D), v((size_t)TP * BN * D), ptab((size_t)TP * BN + WIN + 8);
  uint32_t seed = 777u;
  for (auto& x : q) x = bf16_round(0.3f * frand(seed));
  for (auto& x : k) x = bf16_round(0.3f * frand(seed));
  for (auto& x : v) x = bf16_round(0.3f * frand(seed));
  for (auto& x : ptab) x = 0.05f * frand(seed) * LOG2E;
  if (g_zero_data & 1) for (auto& x : k) x = 0.f;
  if (g_zero_data & 2) for (auto& x : v) x = 0.f;
  if (g_zero_data & 4) for (auto& x : q) x = 0.f;
  const float alpha2 = LOG2E;
  std::vector<uint16_t> qb(q.size()), kb(k.size()), vb(v.size());
  for (size_t i = 0; i < q.size(); ++i) qb[i] = bf16_bits(q[i]);
  for (size_t i = 0; i < k.size(); ++i) kb[i] = bf16_bits(k[i]);
  for (size_t i = 0; i < v.size(); ++i) vb[i] = bf16_bits(v[i]);
  std::vector<double> ref(BM * D, 0.0);
  for (int t = 0; t < T; ++t)
    for (int r = 0; r < BM; ++r)
      for (int j = 0; j < BN; ++j) {
        double s = 0;
        for (int c = 0; c < D; ++c) s += (double)q[r * D + c] * k[((size_t)t * BN + j) * D + c];
        double u = s * alpha2;
        if (pos) u += ptab[(size_t)t * BN + (BM - 1) - r + j];
        const float p = bf16_round((float)(u / (1.0 + exp2(-u))));
        for (int c = 0; c < D; ++c) ref[r * D + c] += (double)p * v[((size_t)t * BN + j) * D + c];
      }
  bf16_t *dq, *dk, *dv; float *dtab, *dout; long long* dcyc;
  CK(hipMalloc(&dq, qb.size() * 2)); CK(hipMalloc(&dk, kb.size() * 2)); CK(hipMalloc(&dv, vb.size() * 2));
  CK(hipMalloc(&dtab, ptab.size() * 4)); CK(hipMalloc(&dout, (size_t)n_wg * BM * D * 4)); CK(hipMalloc(&dcyc, ((size_t)n_wg * 4 + 1) * 8));
  CK(hipMemcpy(dq, qb.data(), qb.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dk, kb.data(), kb.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dv, vb.data(), vb.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dtab, ptab.data(), ptab.size() * 4, hipMemcpyHostToDevice));
  CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  float ms = 0.f;
  for (int rep = 0; rep < 3; ++rep) {
    CK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(kern, dim3(n_wg), dim3(256), LDS_BYTES, 0, dq, dk, dv, dtab, alpha2, rounds, reps, dout, dcyc);
    CK(hipEventRecord(e1, 0));
    CK(hipDeviceSynchronize());
    CK(hipEventElapsedTime(&ms, e0, e1));
  }
  std::vector<float> out((size_t)n_wg * BM * D);
  std::vector<long long> cyc((size_t)n_wg * 4);
  CK(hipMemcpy(out.data(), dout, out.size() * 4, hipMemcpyDeviceToHost));
  CK(hipMemcpy(cyc.data(), dcyc, cyc.size() * 8, hipMemcpyDeviceToHost));
  long long rt_ticks = 0;
  CK(hipMemcpy(&rt_ticks, dcyc + (size_t)n_wg * 4, 8, hipMemcpyDeviceToHost));
  const double mhz = (double)cyc[0] / ((double)rt_ticks / 100.0);
  double max_ref = 0, max_err = 0;
  for (size_t i = 0; i < ref.size(); ++i) max_ref = fmax(max_ref, fabs(ref[i] * reps));
  for (int g = 0; g < n_wg; g += (n_wg > 8 ? n_wg / 8 : 1))
    for (size_t i = 0; i < ref.size(); ++i) max_err = fmax(max_err, fabs(out[(size_t)g * BM * D + i] - ref[i] * reps));
  double cyc_sum = 0; long long cyc_max = 0;
  for (auto c : cyc) { cyc_sum += (double)c; cyc_max = c > cyc_max ? c : cyc_max; }
  const double blocks = (double)T * reps;
  printf("{\"variant\": \"%s\", \"zero_operands\": %d, \"pos_bias\": %s, \"workgroups\": %d, \"steps_per_item\": %d, \"items\": %d, \"kernel_ms\": %.4f, "
         "\"wave_cycles_per_block_avg\": %.1f, \"wave_cycles_per_block_max\": %.1f, \"simd_cycles_per_wave_block\": %.1f, "
         "\"mfma_cycles_per_block\": 512, \"clock_mhz\": %.0f, \"tflops\": %.0f, \"max_abs_err_over_max_ref\": %.3e}\n",
         name, g_zero_data, pos ? "true" : "false", n_wg, T, reps, ms, cyc_sum / cyc.size() / blocks, (double)cyc_max / blocks,
         cyc_sum / cyc.size() / blocks / 2.0, mhz, 4.0 * n_wg * blocks * 16 * 32768 / (ms * 1e-3) * 1e-12, max_ref > 0 ? max_err / max_ref : max_err);
  fflush(stdout);
  CK(hipFree(dq)); CK(hipFree(dk)); CK(hipFree(dv)); CK(hipFree(dtab)); CK(hipFree(dout)); CK(hipFree(dcyc));
}

#ifdef HSTU_STREAM_EXPERIMENTS
// One variant of the sweep.  Compute-only variants go round the four ring stages (filled once) `rounds` times;
// variants with loads stream 64 steps from global memory per item, `items` items.  ns per wave-block is the
// kernel's time over the blocks a SIMD's two waves go through; 16 matrix instructions alone take 217 ns.
template <int V, bool FULL>
static void run_exp(const char* name, bool pos, bool wrong, int rounds, int n_wg) {
  const int reps = FULL ? rounds / 4 : 1, rnd = FULL ? 16 : rounds;
  const int T = FULL ? 4 * rnd : NSTAGE, TP = T + 8;
  std::vector<float> q(BM * D), k((size_t)TP * BN * D), v((size_t)TP * BN * D), ptab((size_t)TP * WIN + WIN + 8);
  uint32_t seed = 4242u;
  for (auto& x : q) x = bf16_round(0.3f * frand(seed));
  for (auto& x : k) x = bf16_round(0.3f * frand(seed));
  for (auto& x : v) x = bf16_round(0.3f * frand(seed));
  for (auto& x : ptab) x = 0.05f * frand(seed) * LOG2E;
  if (g_zero_data & 1) for (auto& x : k) x = 0.f;
  if (g_zero_data & 2) for (auto& x : v) x = 0.f;
  if (g_zero_data & 4) for (auto& x : q) x = 0.f;
  // compute-only variants read window st of the table at float st * WIN (fill_lds), streamed ones at 32 t
  const float alpha2 = LOG2E;
  std::vector<uint16_t> qb(q.size()), kb(k.size()), vb(v.size());
  for (size_t i = 0; i < q.size(); ++i) qb[i] = bf16_bits(q[i]);
  for (size_t i = 0; i < k.size(); ++i) kb[i] = bf16_bits(k[i]);
  for (size_t i = 0; i < v.size(); ++i) vb[i] = bf16_bits(v[i]);
  std::vector<double> ref(BM * D, 0.0);
  for (int t = 0; t < T; ++t)
    for (int r = 0; r < BM; ++r)
      for (int j = 0; j < BN; ++j) {
        double s = 0;
        for (int c = 0; c < D; ++c) s += (double)q[r * D + c] * k[((size_t)t * BN + j) * D + c];
        double u = s * alpha2;
        if (pos) u += ptab[(size_t)t * (FULL ? BN : WIN) + (BM - 1) - r + j];
        const float p = bf16_round((float)(u / (1.0 + exp2(-u))));
        for (int c = 0; c < D; ++c) ref[r * D + c] += (double)p * v[((size_t)t * BN + j) * D + c];
      }
  const double mult = FULL ? reps : rounds;
  bf16_t *dq, *dk, *dv; float *dtab, *dout; long long* dcyc;
  CK(hipMalloc(&dq, qb.size() * 2)); CK(hipMalloc(&dk, kb.size() * 2)); CK(hipMalloc(&dv, vb.size() * 2));
  CK(hipMalloc(&dtab, ptab.size() * 4)); CK(hipMalloc(&dout, (size_t)n_wg * BM * D * 4)); CK(hipMalloc(&dcyc, ((size_t)n_wg * 4 + 1) * 8));
  CK(hipMemcpy(dq, qb.data(), qb.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dk, kb.data(), kb.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dv, vb.data(), vb.size() * 2, hipMemcpyHostToDevice));
  CK(hipMemcpy(dtab, ptab.data(), ptab.size() * 4, hipMemcpyHostToDevice));
  auto kern = k_exp<V, FULL>;
  CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES));
  hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
  float ms = 0.f, best = 1e30f;
  for (int rep = 0; rep < 4; ++rep) {
    CK(hipEventRecord(e0, 0));
    hipLaunchKernelGGL(kern, dim3(n_wg), dim3(256), LDS_BYTES, 0, dq, dk, dv, dtab, alpha2, rnd, reps, dout, dcyc);
    CK(hipEventRecord(e1, 0));
    CK(hipDeviceSynchronize());
    CK(hipEventElapsedTime(&ms, e0, e1));
    if (rep > 0 && ms < best) best = ms;
  }
  std::vector<float> out((size_t)n_wg * BM * D);
  CK(hipMemcpy(out.data(), dout, out.size() * 4, hipMemcpyDeviceToHost));
  double max_ref = 0, max_err = 0;
  for (size_t i = 0; i < ref.size(); ++i) max_ref = fmax(max_ref, fabs(ref[i] * mult));
  for (int g = 0; g < n_wg; g += (n_wg > 8 ? n_wg / 8 : 1))
    for (size_t i = 0; i < ref.size(); ++i) max_err = fmax(max_err, fabs(out[(size_t)g * BM * D + i] - ref[i] * mult));
  const double blocks = (double)T * mult;        // per wave
  const double waves_per_simd = n_wg * 4.0 / (4.0 * 256);
  printf("{\"variant\": \"%s\", \"window\": %s, \"loads\": %s, \"kernel_ms\": %.3f, \"ns_per_wave_block_per_simd\": %.1f, \"tflops\": %.0f, "
         "\"max_abs_err_over_max_ref\": %.2e, \"results\": \"%s\"}\n",
         name, pos ? "true" : "false", FULL ? "true" : "false", best, best * 1e6 / (blocks * waves_per_simd),
         4.0 * n_wg * blocks * 16 * 32768 / (best * 1e-3) * 1e-12, max_err / max_ref, wrong ? "wrong on purpose (ablation)" : (max_err / max_ref < 2e-3 ? "ok" : "WRONG"));
  fflush(stdout);
  CK(hipFree(dq)); CK(hipFree(dk)); CK(hipFree(dv)); CK(hipFree(dtab)); CK(hipFree(dout)); CK(hipFree(dcyc));
}
#endif

int main(int argc, char** argv) {
  const int rounds = argc > 1 ? atoi(argv[1]) : 500;
  g_zero_data = argc > 2 ? atoi(argv[2]) : 0;
  hipDeviceProp_t prop; CK(hipGetDeviceProperties(&prop, 0));
  const int n_wg = 2 * prop.multiProcessorCount;       // two workgroups per CU, eight waves: two per SIMD
#if defined(HSTU_STREAM_EXPERIMENTS) && !defined(HSTU_PROBES_TOO)
#define HSTU_EXP_TABLE
#define HSTU_EXP_ENTRY(i, name, pos, wrong, full) run_exp<i, full>(name, pos, wrong, rounds, n_wg);
#include HSTU_STREAM_EXPERIMENTS
  return 0;
#endif
  int wall_khz = 0, clk_khz = 0;
  CK(hipDeviceGetAttribute(&wall_khz, hipDeviceAttributeWallClockRate, 0));
  CK(hipDeviceGetAttribute(&clk_khz, hipDeviceAttributeClockRate, 0));
  printf("{\"device\": \"%s\", \"cus\": %d, \"wall_clock_khz\": %d, \"clock_khz\": %d}\n", prop.name, prop.multiProcessorCount, wall_khz, clk_khz);
  const bool probes = !(argc > 3 && atoi(argv[3]) == 0);     // third argument 0: the blocks only, not the instruction-rate probes
  if (probes) {
  run_clock<1>("exp2_only (64 per iter)", 10000, n_wg, 64);
  run_clock<1>("exp2_only (64 per iter)", 40000, n_wg, 64);
  run_clock<5>("mul_only (64 per iter)", 40000, n_wg, 64);
  run_clock<0>("mfma_only (16 per iter)", 10000, n_wg, 16);
  run_clock<0>("mfma_only (16 per iter)", 40000, n_wg, 16);
  run_clock<0>("mfma_only, one workgroup per CU", 40000, n_wg / 2, 16);
  run_clock<19>("mfma_only, operands of random bits (16 per iter)", 40000, n_wg, 16);
  run_clock<20>("mfma + 2 exp2 + 4 mul, operands of random bits (16 groups per iter)", 40000, n_wg, 16);
  run_clock<2>("mfma + 4 exp2 (16 groups per iter)", 40000, n_wg, 16);
  run_clock<3>("mfma + 2 exp2 + 4 mul (16 groups per iter)", 40000, n_wg, 16);
  run_clock<4>("2 exp2 + 4 mul (16 groups per iter)", 40000, n_wg, 16);
  run_clock<10>("mfma, one dependent chain (16 per iter)", 40000, n_wg, 16);
  run_clock<11>("mfma in chains of 8 + 2 exp2 + 4 mul (16 groups per iter)", 40000, n_wg, 16);
  run_clock<6>("ds_read_b128 only (32 per iter)", 40000, n_wg, 32);
  run_clock<7>("ds_read_b64_tr_b16 only (32 per iter)", 40000, n_wg, 32);
  run_clock<8>("mfma + 0.5 b128 + 1 tr_b64 (16 groups per iter)", 40000, n_wg, 16);
  run_clock<9>("mfma + 2 exp2 + 4 mul + 0.5 b128 + 1 tr_b64 (16 groups per iter)", 40000, n_wg, 16);
  run_clock<12>("one workgroup per CU: mfma + 2 exp2 + 4 mul + 0.25 b128 + 0.5 tr_b64 (16 groups per iter)", 40000, n_wg / 2, 16);
  run_clock<9>("one workgroup per CU: mfma + 2 exp2 + 4 mul + 0.5 b128 + 1 tr_b64 (16 groups per iter)", 40000, n_wg / 2, 16);
  run_clock<12>("mfma + 2 exp2 + 4 mul + 0.25 b128 + 0.5 tr_b64 (16 groups per iter)", 40000, n_wg, 16);
  run_clock<13>("mfma + 2 exp2 (16 groups per iter)", 40000, n_wg, 16);
  run_clock<14>("mfma + 4 mul (16 groups per iter)", 40000, n_wg, 16);
  run_clock<17>("mfma + 8 mul (16 groups per iter)", 40000, n_wg, 16);
  run_clock<18>("mfma + 12 mul (16 groups per iter)", 40000, n_wg, 16);
  run_clock<18>("one workgroup per CU: mfma + 12 mul (16 groups per iter)", 40000, n_wg / 2, 16);
  run_clock<15>("mfma + 6 pk_fma_f16 (16 groups per iter)", 40000, n_wg, 16);
  run_clock<16>("pk_fma_f16 only (64 per iter)", 40000, n_wg, 64);
  run_clock<16>("one workgroup per CU: pk_fma_f16 only (64 per iter)", 40000, n_wg / 2, 64);
  run_clock<5>("one workgroup per CU: mul only (64 per iter)", 40000, n_wg / 2, 64);
  run_clock<3>("mfma + 2 exp2 + 4 mul, one workgroup per CU", 40000, n_wg / 2, 16);
  run_clock<3>("mfma + 2 exp2 + 4 mul, one workgroup in all", 40000, 1, 16);
  run_clock<0>("mfma_only, one workgroup in all", 40000, 1, 16);
  }
  run("cpp_block", k_cpp<false>, false, rounds, n_wg);
  run("cpp_block", k_cpp<true>, true, rounds, n_wg);
  run("hand_stream", k_stream<false>, false, rounds, n_wg);
  run("hand_stream", k_stream<true>, true, rounds, n_wg);
  // 64 steps per item (the longest tile of a 2048-token sequence), every workgroup streaming the same rows
  run_dma("hand_stream_with_loads", k_stream_dma<false>, false, 16, rounds / 4, n_wg);
  run_dma("hand_stream_with_loads", k_stream_dma<true>, true, 16, rounds / 4, n_wg);
  return 0;
}
