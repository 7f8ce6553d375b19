// HSTU pointwise-SiLU attention, forward and backward, for gfx950 (MI355X, CDNA4).
//
//   out[b,i,h,:] = sum_j M[b,i,j] * silu(alpha*q_i.k_j + bias(b,h,i,j)) * inv_n * v[b,j,h,:]
//
// Kernels behind the C entry points (see include/hstu_attn.h).  Forward:
//
//   hstu_fwd_mfma_bf16   the hot path.  bf16 (or fp8 e4m3fn) Q/K, bf16 V, fp32
//                        accumulation on the 32x32x16 MFMA; 128 query rows per
//                        workgroup, keys streamed 32 at a time through a
//                        4-stage (d <= 64: 3-stage) LDS ring filled by direct global->LDS loads;
//                        relative-position and timestamp bias + SiLU + mask
//                        fused on the accumulator registers; causal / length /
//                        sliding-window tile skipping, segment ids; or, in
//                        their place, tiles of a dense [L, Lkv] keep-mask and
//                        fp32 bias streamed through the same ring.  Computes
//                        S^T = K Q^T so that the
//                        accumulator layout of S^T is already the B-operand
//                        layout of O^T = V^T P^T: P never touches LDS.  Its
//                        work list is taken one workgroup per item or by
//                        resident workgroups that draw item after item; query
//                        tiles that alone would outlast the rest are split by
//                        key range between workgroups, and the one that
//                        arrives last at the tile's counter sums the parts.
//   hstu_prepare         runs before it, once per batch: work list of
//                        (sequence, tile, key chunk) items, longest sequences
//                        first; scaled bias tables; the timestamp bucket
//                        tables; int32 timestamps and their per-tile ranges.
//   hstu_fwd_general     every option of the op (segment ids, explicit mask,
//                        sliding window, dense bias, cross lengths, any head
//                        dim <= 256, fp32 or bf16 storage, any strides) in
//                        fp32 arithmetic on the fp32 matrix cores.  The path of
//                        fp32 callers (the reference's default dtype) and of
//                        the options the bf16 kernel does not cover.
//
// Backward (dq, dk, dv and the gradients of the two bias tables):
//
//   hstu_bwd_dq_mfma     bf16 on the matrix cores under the conditions of the
//   hstu_bwd_dkv_mfma    MFMA forward: one kernel per 128 query rows streaming
//                        K and V, one per 128 keys streaming Q and dO; both
//                        recompute the logits; the first also sums the table
//                        gradients.
//   hstu_bwd_dq_mm,      every option and storage form in fp32 arithmetic on the
//   hstu_bwd_dkv_mm      fp32 matrix cores, head dims up to 128.
//   hstu_bwd_dq,         the same by fp32 FMA loops for head dims up to 256.
//   hstu_bwd_dkv
//
// The math follows recml/layers/keras/hstu.py:356-390 (dense formulation),
// recml/core/ops/hstu_ops.py:230-264 (order: scale, SiLU, 1/N, mask, PV in
// fp32), hstu.py:91-113 (relative position bias = w[(L-1)+j-i]) and
// hstu.py:33-55, 190-221 (timestamp buckets).

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <type_traits>

#include "hstu_attn.h"

namespace {

typedef __bf16 bf16_t;
typedef bf16_t bf16x8 __attribute__((ext_vector_type(8)));
typedef bf16_t bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

struct Params {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  int64_t q_sb, q_st, q_sh;
  int64_t k_sb, k_st, k_sh;
  int64_t v_sb, v_st, v_sh;
  int64_t o_sb, o_st, o_sh;
  const int32_t* seq_lens;
  const int32_t* seq_offsets;
  const int32_t* q_seg;
  const int32_t* kv_seg;
  const uint8_t* mask;
  const float* dense_bias;
  const float* pos_tab;
  const float* ts_tab;
  const int64_t* ts;
  const float* pos_scaled;   // workspace: log2(e) * pos_tab, zero-padded (MFMA kernel)
  // workspace of the MFMA kernel's timestamp path: per sequence, 1 when max - min timestamp fits
  // 31 bits; then timestamps minus the sequence minimum as int32, and their (min, max) per 32-key tile
  const int32_t* ts_ok;
  const int32_t* ts_rel;
  const int32_t* ts_range;
  const int4* ts_keyed;      // workspace: the bucket tables [heads][3 KB], see TsKeys
  const void* ws_base;       // start of the workspace (all of the above lie within 4 GB of it)
  const float* q_scale;      // [H] or null: dequantisation scales of fp8 q / k
  const float* k_scale;
  int64_t ts_sb;
  int32_t B, L, Lkv, H, d_qk, d_v;
  int32_t jagged, causal, mask_mode, window;
  int32_t mask_batched, dense_bias_batched, pos_heads, ts_heads;
  int32_t ts_nb;
  float ts_bucket_size;
  float alpha, inv_n;
  int32_t n_qtiles;
  // Key-range splitting (MFMA forward; off when split_cap == 0): hstu_prepare, which sees the lengths,
  // shares a query tile with more steps than twice a slot's average load between up to MAX_CHUNKS workgroups,
  // each covering a contiguous part of the keys and leaving its fp32 partial O^T in `partial`; the
  // workgroup that arrives last at the tile's counter sums them and writes the rows.
  int32_t split_cap;         // chunk slots of the partial buffer (per head)
  int32_t n_slots;           // workgroups that run at once per XCD (what the split decision balances for)
  const int32_t* mask_range; // workspace: per (mask batch, query tile) the first 32-key step with a kept pair and one past the last
  int32_t persist;           // forward: resident workgroups that loop over the work list
  int32_t no_stream;         // forward: interior steps through the compiler-scheduled block code too (a comparison switch)
  int32_t mask_pres;         // the preparation also fills the dense mask's presence table (the backward asks for it)
  // Dropout on the attention weights: pair (b, h, i, j) is kept when drop_hash(...) >= drop_thr (0: no dropout).
  // The survivors' scale 1 / (1 - p) is folded into inv_n by the host.
  uint32_t drop_thr, drop_key;
  // Timestamp descriptors (matrix-core forward at d = 128; null = none): one 16-bit word per (32-key step, query
  // row), [step][row] with `ts_desc_pitch` rows per step, built by hstu_prepare (ts_desc_block) for every head and layer of
  // a batch; and per (128-row tile, chunk of TS_DESC_CHUNK steps) the first step in which some row needs the per-pair
  // lookup (INT32_MAX: none).
  const uint16_t* ts_desc;
  const int32_t* ts_tquads;
  int32_t ts_desc_pitch;
  int32_t ts_desc_tiles;     // tile slots of ts_tquads
  int32_t ts_desc_chunks;    // entries per tile slot: chunks of TS_DESC_CHUNK steps
  float* partial;            // [chunk slot][head][BM x d_v floats in register order]
  uint32_t* ctr;             // workspace: [0, 8) draw counters of the XCDs, [8] workgroups done, then from
                             // CTR_RESERVED on one arrival counter per (chunk slot, head); all zero between launches
  // Work list built on the device by hstu_prepare (MFMA kernel; null = workgroups enumerate every
  // possible (sequence, tile) and most exit): sched[0] = number of items, then from
  // sched[4] on one int4 per (sequence, query tile, chunk) that has work:
  // {b | first chunk slot << 14, qt | chunk << 16 | chunks << 24, first token, stored length}.
  const int32_t* sched;
  // backward pass: gradient of out in, gradients of q, k, v out (layouts of out, q, k, v), and
  // fp32 table gradients that are accumulated into (null = not wanted)
  const void* dout;
  void* dq;
  void* dk;
  void* dv;
  float* dpos;
  float* dts;
  float* dbias;              // gradient of the dense bias (general backward), or null
  int64_t items_max;         // capacity of the list (sizes the grid)
};

// Per-sequence geometry shared by both kernels.
struct Seq {
  int n_q;        // query rows that produce output
  int n_kv;       // keys that may be attended
  int rows;       // rows of the output tile space (L, or n_b when jagged)
  int64_t tok0;   // first token of the sequence in the token axis
  int64_t bq, bk, bv, bo;  // element offsets of (token 0, head h)
  int64_t ts0;    // element offset of timestamp 0
  int n_ts;       // timestamps addressable for this sequence
};

// o0: first token (jagged layout); nraw: the sequence's length as stored (offset difference or
// seq_lens entry; ignored for the padded layout without a length mask).
__device__ __forceinline__ Seq seq_from(const Params& p, int b, int h, int o0, int nraw) {
  Seq s;
  if (p.jagged) {
    int n = nraw;
    n = n < 0 ? 0 : (n > p.L ? p.L : n);
    s.n_q = n; s.n_kv = n; s.rows = n; s.tok0 = o0;
    s.bq = (int64_t)o0 * p.q_st + (int64_t)h * p.q_sh;
    s.bk = (int64_t)o0 * p.k_st + (int64_t)h * p.k_sh;
    s.bv = (int64_t)o0 * p.v_st + (int64_t)h * p.v_sh;
    s.bo = (int64_t)o0 * p.o_st + (int64_t)h * p.o_sh;
  } else {
    int nq = p.L, nk = p.Lkv;
    if (p.mask_mode == HSTU_MASK_LENGTH) {
      int n = nraw;
      n = n < 0 ? 0 : n;
      nq = n < p.L ? n : p.L;
      nk = n < p.Lkv ? n : p.Lkv;
    }
    s.n_q = nq; s.n_kv = nk; s.rows = p.L; s.tok0 = 0;
    s.bq = (int64_t)b * p.q_sb + (int64_t)h * p.q_sh;
    s.bk = (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
    s.bv = (int64_t)b * p.v_sb + (int64_t)h * p.v_sh;
    s.bo = (int64_t)b * p.o_sb + (int64_t)h * p.o_sh;
  }
  if (p.ts_sb != 0) { s.ts0 = (int64_t)b * p.ts_sb; s.n_ts = p.L; }
  else              { s.ts0 = s.tok0;               s.n_ts = s.n_kv; }
  return s;
}

__device__ __forceinline__ void seq_raw(const Params& p, int b, int& o0, int& nraw) {
  o0 = 0;
  nraw = p.L;
  if (p.jagged) {
    o0 = p.seq_offsets[b];
    nraw = p.seq_offsets[b + 1] - o0;
  } else if (p.mask_mode == HSTU_MASK_LENGTH) {
    nraw = p.seq_lens[b];
  }
}

__device__ __forceinline__ Seq seq_info(const Params& p, int b, int h) {
  int o0, nraw;
  seq_raw(p, b, o0, nraw);
  return seq_from(p, b, h, o0, nraw);
}

__device__ __forceinline__ float ldf(const float* p) { return *p; }
__device__ __forceinline__ float ldf(const bf16_t* p) { return (float)*p; }
__device__ __forceinline__ void stf(float* p, float x) { *p = x; }
__device__ __forceinline__ void stf(bf16_t* p, float x) { *p = (bf16_t)x; }

// ---------------------------------------------------------------------------
// General kernel: fp32 FMA arithmetic, every option.
// ---------------------------------------------------------------------------

constexpr float LOG2E = 1.4426950408889634f;
constexpr int GT = 32;       // query rows and keys per tile
constexpr int GMAXX = 32;    // d_v / 8 accumulators per thread, d_v <= 256
// floats of the general backward's timestamp-bucket histogram in LDS: one per table entry, a multiple of four
__host__ __device__ inline int general_hist_len(int ts_nb) { return ts_nb < 0 ? 4 : ((ts_nb + 4) & ~3); }

// the table biases of pair (i, j): position and timestamp
__device__ __forceinline__ float general_table_bias(const Params& p, const Seq& s,
                                                    int b, int h, int i, int j, int* bucket = nullptr) {
  float bias = 0.f;
  if (p.pos_tab) {
    int hh = p.pos_heads > 1 ? h : 0;
    bias += p.pos_tab[(int64_t)hh * (2 * p.L - 1) + (p.L - 1) + j - i];
  }
  if (p.ts_tab) {
    int iq = i + 1 < s.n_ts ? i + 1 : s.n_ts - 1;
    int jk = j < s.n_ts ? j : s.n_ts - 1;
    int64_t dt = p.ts[s.ts0 + iq] - p.ts[s.ts0 + jk];
    if (dt < 0) dt = -dt;
    if (dt < 1) dt = 1;
    if (dt > 1000000000LL) dt = 1000000000LL;
    // the bucket law: floor(ln(fl32(|dt|)) / size), evaluated in double so that every |dt| falls on the
    // side of a bucket boundary that the law's integer thresholds (bucket_law below) put it on
    const double lg = log((double)(float)dt) / (double)p.ts_bucket_size;
    int bk = (int)lg;
    bk = bk < 0 ? 0 : (bk > p.ts_nb ? p.ts_nb : bk);
    if (bucket) *bucket = bk;
    int hh = p.ts_heads > 1 ? h : 0;
    bias += p.ts_tab[(int64_t)hh * (p.ts_nb + 1) + bk];
  }
  return bias;
}
// every bias of pair (i, j)
__device__ __forceinline__ float general_bias(const Params& p, const Seq& s,
                                              int b, int h, int i, int j, int* bucket = nullptr) {
  float bias = general_table_bias(p, s, b, h, i, j, bucket);
  if (p.dense_bias) {
    int64_t o = p.dense_bias_batched ? (int64_t)b * p.L * p.Lkv : 0;
    bias += p.dense_bias[o + (int64_t)i * p.Lkv + j];
  }
  return bias;
}

// The explicit mask's bytes for the 16 pairs (row i, keys j0 + 8g + 4hh .. +3, g < 4) a lane holds after a
// product with the query row fixed: one 32-bit word per g (byte tt = key j0 + 8g + 4hh + tt).  Row and keys are
// clamped into the matrix: bytes of pairs outside it are never looked at (their indices drop them).
// (WORDS_ONLY: the caller has checked that whole words can be fetched; the byte-wise form is then left out)
template <bool WORDS_ONLY = false>
__device__ __forceinline__ void general_mask_words(const Params& p, int b, int i, int j0, int hh, uint32_t (&w)[4]) {
  const uint8_t* mrow = p.mask + (p.mask_batched ? (int64_t)b * p.L * p.Lkv : 0) + (int64_t)(i < p.L - 1 ? i : p.L - 1) * p.Lkv;
  if (WORDS_ONLY || ((p.Lkv & 3) == 0 && ((uintptr_t)p.mask & 3) == 0)) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      int j = j0 + 8 * g + 4 * hh;
      j = j < p.Lkv - 4 ? j : p.Lkv - 4;
      w[g] = *(const uint32_t*)(mrow + j);
    }
  } else {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      uint32_t v = 0u;
#pragma unroll
      for (int tt = 0; tt < 4; ++tt) {
        int j = j0 + 8 * g + 4 * hh + tt;
        j = j < p.Lkv - 1 ? j : p.Lkv - 1;
        v |= (uint32_t)mrow[j] << (8 * tt);
      }
      w[g] = v;
    }
  }
}
// The same for a product with the key fixed: pairs (rows i0 + 8g + 4hh + tt, key j), bytes a row apart.
__device__ __forceinline__ void general_mask_words_col(const Params& p, int b, int i0, int j, int hh, uint32_t (&w)[4]) {
  const uint8_t* mcol = p.mask + (p.mask_batched ? (int64_t)b * p.L * p.Lkv : 0) + (j < p.Lkv - 1 ? j : p.Lkv - 1);
  uint8_t v[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    int i = i0 + 8 * (r >> 2) + 4 * hh + (r & 3);
    i = i < p.L - 1 ? i : p.L - 1;
    v[r] = mcol[(int64_t)i * p.Lkv];
  }
#pragma unroll
  for (int g = 0; g < 4; ++g)
    w[g] = (uint32_t)v[4 * g] | ((uint32_t)v[4 * g + 1] << 8) | ((uint32_t)v[4 * g + 2] << 16) | ((uint32_t)v[4 * g + 3] << 24);
}
// The explicit mask's live steps for one workgroup's tile, found by one pass of its 256 threads over the tile's
// bytes before the step loop (an L x Lkv mask is mostly zeros when it carries the causal rule, and a step the mask
// empties still costs its tile loads and barriers):
//   ROWS:  rows [t0, t0 + 128) -> the 32-key steps [lo, hi) outside of which every byte of those rows is zero;
//   !ROWS: keys [t0, t0 + 128) -> the 32-row steps likewise.
// Reads 16 bytes per lane: where Lkv or the pointer does not allow that, the full range comes back.  Every
// thread of the workgroup must call it (one barrier inside).
template <bool ROWS>
__device__ __forceinline__ void general_mask_live_steps(const Params& p, int b, int t0, int tid, int& lo, int& hi) {
  // (lo, hi come in as the range of steps the other rules leave: only that part of the mask is looked at)
  __shared__ int ends[4][2];
  const int s_lo = lo, s_hi = hi;
  if ((p.Lkv & 15) != 0 || ((uintptr_t)p.mask & 15) != 0 || s_lo >= s_hi) return;
  const uint8_t* mb = p.mask + (p.mask_batched ? (int64_t)b * p.L * p.Lkv : 0);
  const int lane = tid & 63, w = tid >> 6;
  int mn = 0x7fffffff, mx = -1;
  if (ROWS) {
    // wave w: rows t0 + 32 w .. + 31 (clamped into the matrix); lane: 16-byte chunks lane, lane + 64, ... of a row
    const int n_chunks = (p.Lkv >> 4) < 2 * s_hi ? (p.Lkv >> 4) : 2 * s_hi;
    for (int c = 2 * s_lo + lane; c < n_chunks; c += 64) {
      uint32_t any = 0u;
#pragma unroll 8
      for (int rr = 0; rr < 32; ++rr) {
        int r = t0 + 32 * w + rr;
        r = r < p.L - 1 ? r : p.L - 1;
        const uint4 v = *(const uint4*)(mb + (int64_t)r * p.Lkv + 16 * c);
        any |= v.x | v.y | v.z | v.w;
      }
      if (any != 0u) {
        mn = mn < (c >> 1) ? mn : (c >> 1);
        mx = mx > (c >> 1) ? mx : (c >> 1);
      }
    }
  } else {
    // 8 chunks per row cover the 128 keys; a wave's instruction reads 8 rows: wave w takes rows 32 i + 8 w + lane / 8
    const int ch = lane & 7;
    const bool col_ok = t0 + 16 * ch < p.Lkv;
#pragma unroll 4
    for (int i = s_lo; i < s_hi; ++i) {
      const int r = 32 * i + 8 * w + (lane >> 3);
      if (col_ok && r < p.L) {
        const uint4 v = *(const uint4*)(mb + (int64_t)r * p.Lkv + t0 + 16 * ch);
        if ((v.x | v.y | v.z | v.w) != 0u) {
          mn = mn < i ? mn : i;
          mx = mx > i ? mx : i;
        }
      }
    }
  }
#pragma unroll
  for (int dl = 32; dl >= 1; dl >>= 1) {
    const int on = __shfl_xor(mn, dl, 64), ox = __shfl_xor(mx, dl, 64);
    mn = mn < on ? mn : on;
    mx = mx > ox ? mx : ox;
  }
  if (lane == 0) {
    ends[w][0] = mn;
    ends[w][1] = mx;
  }
  __syncthreads();
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    mn = mn < ends[x][0] ? mn : ends[x][0];
    mx = mx > ends[x][1] ? mx : ends[x][1];
  }
  // (the same in every lane, and said so: loop bounds derived from these must stay scalar)
  lo = __builtin_amdgcn_readfirstlane(mx < 0 ? s_lo : mn);
  hi = __builtin_amdgcn_readfirstlane(mx < 0 ? s_lo : mx + 1);             // nothing kept at all: an empty range
}

// The dense bias of the same 16 pairs (query row fixed / key fixed), fetched together ahead of their use: four
// 16-byte loads where the rows allow, else one load per pair; indices clamped into the matrix like the mask's.
template <bool WORDS_ONLY = false>
__device__ __forceinline__ void general_dense_row(const Params& p, int b, int i, int j0, int hh, float (&v)[16]) {
  const float* row = p.dense_bias + (p.dense_bias_batched ? (int64_t)b * p.L * p.Lkv : 0) + (int64_t)(i < p.L - 1 ? i : p.L - 1) * p.Lkv;
  if (WORDS_ONLY || ((p.Lkv & 3) == 0 && ((uintptr_t)p.dense_bias & 15) == 0)) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      int j = j0 + 8 * g + 4 * hh;
      j = j < p.Lkv - 4 ? j : p.Lkv - 4;
      const float4 t4 = *(const float4*)(row + j);
      v[4 * g] = t4.x; v[4 * g + 1] = t4.y; v[4 * g + 2] = t4.z; v[4 * g + 3] = t4.w;
    }
  } else {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      int j = j0 + 8 * (r >> 2) + 4 * hh + (r & 3);
      v[r] = row[j < p.Lkv - 1 ? j : p.Lkv - 1];
    }
  }
}
__device__ __forceinline__ void general_dense_col(const Params& p, int b, int i0, int j, int hh, float (&v)[16]) {
  const float* col = p.dense_bias + (p.dense_bias_batched ? (int64_t)b * p.L * p.Lkv : 0) + (j < p.Lkv - 1 ? j : p.Lkv - 1);
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    int i = i0 + 8 * (r >> 2) + 4 * hh + (r & 3);
    v[r] = col[(int64_t)(i < p.L - 1 ? i : p.L - 1) * p.Lkv];
  }
}
// Dropout's keep rule: a counter-based hash of (seed, b, h, i, j), the same on the host, in every kernel and in
// the CPU oracle.  drop_seed_key folds the 64-bit seed (host, once per call), drop_bh_key the sequence and the
// head (once per work item), drop_keep the pair: two multiply-add steps on the indices, of which a kernel hoists
// the one that is fixed for its lane, then drop_keep_mixed.
__host__ __device__ inline uint32_t drop_seed_key(uint64_t seed) {
  uint32_t z = (uint32_t)seed ^ 0x9E3779B9u;
  z = (z ^ (z >> 16)) * 0x85EBCA6Bu;
  z ^= (uint32_t)(seed >> 32);
  z = (z ^ (z >> 13)) * 0xC2B2AE35u;
  return z ^ (z >> 16);
}
__host__ __device__ inline uint32_t drop_bh_key(uint32_t key, uint32_t bh) {
  uint32_t z = key + bh * 0x9E3779B1u;
  z = (z ^ (z >> 15)) * 0x2C1B3C6Du;
  return z ^ (z >> 13);
}
constexpr uint32_t DROP_CI = 0x85EBCA77u, DROP_CJ = 0xC2B2AE3Du;
// ij = kbh + i * DROP_CI + j * DROP_CJ (wrapping)
// (two multiplications with one fold of the high half onto the low half between them: the comparison reads the product
// from its top bits down, which depend on every bit of ij; seven instructions per pair with the index step and the select)
__host__ __device__ inline bool drop_keep_mixed(uint32_t ij, uint32_t thr) {
  uint32_t z = ij * 0x2C1B3C6Du;
  z = (z ^ (z >> 16)) * 0x297A2D39u;
  return z >= thr;
}
__host__ __device__ inline bool drop_keep(uint32_t kbh, uint32_t i, uint32_t j, uint32_t thr) {
  return drop_keep_mixed(kbh + i * DROP_CI + j * DROP_CJ, thr);
}
// The 16 values a lane holds in a 32 x 32 block sit at offsets c(r) = 8 (r / 4) + r % 4 along the axis that is not the
// lane's own: ij0 carries everything else, `step` is that axis's multiplier.  One value after the other on purpose (the
// scheduling barrier): sixteen hashes in flight at once would cost the kernels around this forty registers on a path
// that inference and most training never take.
__device__ __forceinline__ void drop_apply16(float (&x)[16], uint32_t ij0, uint32_t step, uint32_t thr) {
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    x[r] = drop_keep_mixed(ij0 + (uint32_t)(8 * (r >> 2) + (r & 3)) * step, thr) ? x[r] : 0.f;
    __builtin_amdgcn_sched_barrier(0);
  }
}
__device__ __forceinline__ void drop_apply16(float (&x)[16], float (&y)[16], uint32_t ij0, uint32_t step, uint32_t thr) {
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const bool keep = drop_keep_mixed(ij0 + (uint32_t)(8 * (r >> 2) + (r & 3)) * step, thr);
    x[r] = keep ? x[r] : 0.f;
    y[r] = keep ? y[r] : 0.f;
    __builtin_amdgcn_sched_barrier(0);
  }
}
// p in [0, 1) -> the threshold on the 32-bit hash: a pair is dropped with probability thr / 2^32
__host__ inline uint32_t drop_threshold(float p) {
  const double t = (double)p * 4294967296.0;
  return t <= 0.0 ? 0u : (t >= 4294967295.0 ? 0xffffffffu : (uint32_t)(t + 0.5));
}

// pair (i, j) under the segment ids alone (SEGMENT mode)
__device__ __forceinline__ bool general_same_segment(const Params& p, int b, int i, int j) {
  return p.q_seg[(int64_t)b * p.L + i] == p.kv_seg[(int64_t)b * p.Lkv + j];
}

__device__ __forceinline__ bool general_keep(const Params& p, const Seq& s,
                                             int b, int i, int j) {
  bool keep = (i < s.n_q) && (j < s.n_kv);
  if (p.causal) keep = keep && (j <= i);
  if (p.window >= 0) {
    int dd = i - j; dd = dd < 0 ? -dd : dd;
    keep = keep && (dd <= p.window);
  }
  if (!keep) return false;
  if (p.mask_mode == HSTU_MASK_SEGMENT)
    keep = p.q_seg[(int64_t)b * p.L + i] == p.kv_seg[(int64_t)b * p.Lkv + j];
  if (keep && p.mask) {
    int64_t o = p.mask_batched ? (int64_t)b * p.L * p.Lkv : 0;
    keep = p.mask[o + (int64_t)i * p.Lkv + j] != 0;
  }
  return keep;
}

// The general forward: fp32 arithmetic on the matrix cores (v_mfma_f32_32x32x2_f32: fp32 products, fp32
// sums), every option, any head dims up to 256, fp32 or bf16 storage, any strides.  A workgroup takes up
// to 128 query rows of one (sequence, head), 32 per wave, and streams the keys 32 at a time through LDS:
//   S^T = K Q^T        A = K rows, B = Q rows, both read from LDS two floats per lane and pair of steps;
//   pointwise          on the accumulators, one (query, key) pair per value, through general_keep / general_bias;
//   O^T += V^T P^T     A = V rows from LDS, B = the accumulators of S^T as they are (fp32: no packing).
// The order of the terms of a dot product is free, so slot l / 32 of step s of a pair takes channel
// 4 (s / 2) + 2 (l / 32) + s % 2: the two channels of a lane are neighbours in memory.  Row pitches keep the
// reads free of bank conflicts: twice an odd number of floats for Q and K (rows 0 .. 31 then start on the 32
// even banks), 8 more than a multiple of 32 for V (rows k and k + 4, read by the two halves of a wave, then
// lie 32 banks apart).
__host__ __device__ inline int general_pitch_qk(int d) { const int d4 = (d + 3) & ~3; return ((d4 >> 1) & 1) ? d4 : d4 + 2; }
__host__ __device__ inline int general_pitch_v(int d) { return ((d + 31) & ~31) + 8; }

// Four consecutive elements of a row as floats, zeros where the row or the column is out of range; one
// 16-byte (fp32) or 8-byte (bf16) load when the caller says the address is aligned for it.
__device__ __forceinline__ float4 general_load4(const float* row, int c, int d, bool row_ok, bool vec) {
  float4 r = {0.f, 0.f, 0.f, 0.f};
  if (!row_ok || c >= d) return r;
  if (vec && c + 4 <= d) return *(const float4*)(row + c);
  r.x = row[c];
  if (c + 1 < d) r.y = row[c + 1];
  if (c + 2 < d) r.z = row[c + 2];
  if (c + 3 < d) r.w = row[c + 3];
  return r;
}
__device__ __forceinline__ float4 general_load4(const bf16_t* row, int c, int d, bool row_ok, bool vec) {
  float4 r = {0.f, 0.f, 0.f, 0.f};
  if (!row_ok || c >= d) return r;
  if (vec && c + 4 <= d) {
    const uint2 u = *(const uint2*)(row + c);
    r.x = __builtin_bit_cast(float, u.x << 16);
    r.y = __builtin_bit_cast(float, u.x & 0xffff0000u);
    r.z = __builtin_bit_cast(float, u.y << 16);
    r.w = __builtin_bit_cast(float, u.y & 0xffff0000u);
    return r;
  }
  r.x = (float)row[c];
  if (c + 1 < d) r.y = (float)row[c + 1];
  if (c + 2 < d) r.z = (float)row[c + 2];
  if (c + 3 < d) r.w = (float)row[c + 3];
  return r;
}

// acc += A B^T over the channels: A rows from LDS (`arow` = the lane's row + 2 hh, pitch twice an odd number),
// B = a register fragment; sixteen channels at a time, their reads ahead of their products, then what is left
// four at a time (nothing past d4 is read).
__device__ __forceinline__ void general_dot_rows(floatx16& acc, const float* arow, const float2 (&bf)[32], int d4) {
#pragma unroll
  for (int u0 = 0; u0 < 32; u0 += 4) {
    if (4 * (u0 + 4) <= d4) {
      float2 a[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) a[u] = *(const float2*)(arow + 4 * (u0 + u));
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].x, bf[u0 + u].x, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u].y, bf[u0 + u].y, acc, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (4 * (u0 + u) < d4) {
          const float2 a = *(const float2*)(arow + 4 * (u0 + u));
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, bf[u0 + u].x, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, bf[u0 + u].y, acc, 0, 0, 0);
        }
      }
    }
  }
}

// DMAX (128 or 256): the head dims the instance holds.  The wave's Q row shares live in DMAX / 2 registers and
// its output in DMAX / 2 accumulators: up to 128, 255 registers in all and two waves per SIMD, so that one
// workgroup's loads, barriers and pointwise work run under another's products; up to 256, one wave per SIMD.
// TAB = false: an instance for calls without bias tables whose rows, mask and dense bias can be fetched whole (the
// launch checks): none of the tables' code and none of the element-wise fetches in it.
template <typename T, int DMAX, bool TAB = true>
__global__ __launch_bounds__(256, DMAX <= 128 ? 2 : 1) void hstu_fwd_general(const Params p) {
  extern __shared__ __attribute__((aligned(16))) float gsm[];
  constexpr int NB = DMAX / 32;            // 32-channel blocks of the output
  constexpr int NU = DMAX / 4;             // pairs of steps of a product over the channels
  constexpr int GQ = 128;                  // query rows of a workgroup
  const int dq = p.d_qk, dv = p.d_v;
  const int dq4 = (dq + 3) & ~3;
  const int qp_ = general_pitch_qk(dq), vp_ = general_pitch_v(dv);
  const int nblk = (dv + 31) >> 5;
  float* Ks = gsm;                         // [32][qp_]
  float* Vs = Ks + GT * qp_;               // [32][vp_]

  // Workgroups are handed to the eight XCDs in turn by their linear index: with the head fastest and the query
  // tile slowest every XCD sees every tile position (under the causal mask the last tiles have many times the
  // work of the first), a sequence's tiles of one head meet its K and V rows in one L2, and the longest
  // tiles start first.
  const int h = blockIdx.x, b = blockIdx.y, qt = gridDim.z - 1 - blockIdx.z;
  const Seq s = seq_info(p, b, h);
  const int q0 = qt * GQ;
  if (q0 >= s.rows) return;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, m = lane & 31, hh = lane >> 5;
  const T* __restrict__ qp = (const T*)p.q;
  const T* __restrict__ kp_ = (const T*)p.k;
  const T* __restrict__ vp = (const T*)p.v;
  T* __restrict__ op = (T*)p.out;
  const int r0 = q0 + 32 * w;
  const int qi = r0 + m;                   // this lane's query row
  // whole groups of four elements can be fetched by one load when bases and row strides allow
  constexpr uintptr_t VMASK = sizeof(T) * 4 - 1;
  const bool kvec = !TAB || ((((uintptr_t)(kp_ + s.bk) & VMASK) == 0) && (p.k_st & 3) == 0);
  const bool vvec = !TAB || ((((uintptr_t)(vp + s.bv) & VMASK) == 0) && (p.v_st & 3) == 0);

  // the key steps of this tile (found first, while nothing else is held in registers)
  int kv_end = s.n_kv;
  if (p.causal && q0 + GQ < kv_end) kv_end = q0 + GQ;
  if (p.window >= 0 && q0 + GQ + p.window < kv_end) kv_end = q0 + GQ + p.window;
  int kv_begin = 0;
  if (p.window >= 0 && q0 - p.window > 0) kv_begin = ((q0 - p.window) / GT) * GT;
  if (p.mask && q0 < s.n_q) {
    // the steps before the first and after the last key the mask keeps for these rows are left out
    int t_lo = kv_begin / GT, t_hi = (kv_end + GT - 1) / GT;
    general_mask_live_steps<true>(p, b, q0, tid, t_lo, t_hi);
    kv_begin = t_lo * GT > kv_begin ? t_lo * GT : kv_begin;
    kv_end = t_hi * GT < kv_end ? t_hi * GT : kv_end;
  }

  floatx16 o[NB];
#pragma unroll
  for (int x = 0; x < NB; ++x)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[x][r] = 0.f;

  if (q0 < s.n_q) {
    // tiles are brought by eight threads per row, four channels per thread and turn
    const int lr = tid >> 3, lc = (tid & 7) * 4;
    // the lane's share of its query row: channels 4u + 2hh and 4u + 2hh + 1 for the pair of steps u
    float2 qf[NU];
    {
      const T* qrow_g = qp + s.bq + (int64_t)qi * p.q_st;
#pragma unroll
      for (int u = 0; u < NU; ++u) {
        qf[u] = float2{0.f, 0.f};
        if (4 * u < dq4 && qi < s.n_q) {
          const int c = 4 * u + 2 * hh;
          if (c < dq) qf[u].x = ldf(qrow_g + c);
          if (c + 1 < dq) qf[u].y = ldf(qrow_g + c + 1);
        }
      }
    }
    const int vcols = nblk * 32;
    // The next tile travels in registers while this one is computed on.  When bases and strides allow whole
    // groups and the head dims are multiples of four, the loads are unconditional (rows past the sequence
    // re-read its last key, columns past the head dim the last group) and what must be zero is zeroed on the way
    // into LDS: nothing then uses a loaded value before the tile is staged, and the loads stay in flight behind
    // the products.  Otherwise element by element (bf16 elements packed again: nothing is lost).
    constexpr int NG = DMAX / 32;
    typedef typename std::conditional<sizeof(T) == 4, float4, uint2>::type Raw;
    const bool fast = !TAB || (kvec && vvec && (dq & 3) == 0 && (dv & 3) == 0);
    const int ngk = (dq4 + 31) >> 5, ngv = (vcols + 31) >> 5;
    Raw kraw[NG], vraw[NG];
    auto widen = [](const Raw& u) -> float4 {
      if constexpr (sizeof(T) == 4) {
        return u;
      } else {
        return float4{__builtin_bit_cast(float, u.x << 16), __builtin_bit_cast(float, u.x & 0xffff0000u),
                      __builtin_bit_cast(float, u.y << 16), __builtin_bit_cast(float, u.y & 0xffff0000u)};
      }
    };
    auto narrow = [](const float4& f) -> Raw {
      if constexpr (sizeof(T) == 4) {
        return f;
      } else {
        return uint2{(__builtin_bit_cast(uint32_t, f.x) >> 16) | (__builtin_bit_cast(uint32_t, f.y) & 0xffff0000u),
                     (__builtin_bit_cast(uint32_t, f.z) >> 16) | (__builtin_bit_cast(uint32_t, f.w) & 0xffff0000u)};
      }
    };
    auto fetch_k = [&](int kv0) {
      const int j = kv0 + lr;
      const int jc = fast && j >= s.n_kv ? s.n_kv - 1 : j;
      const T* krow = kp_ + s.bk + (int64_t)jc * p.k_st;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int c = lc + 32 * g;
        if (g < ngk) {
          if (fast) kraw[g] = *(const Raw*)(krow + (c < dq ? c : dq - 4));
          else kraw[g] = narrow(general_load4(krow, c, dq, j < s.n_kv, false));
        }
      }
    };
    auto fetch_v = [&](int kv0) {
      const int j = kv0 + lr;
      const int jc = fast && j >= s.n_kv ? s.n_kv - 1 : j;
      const T* vrow = vp + s.bv + (int64_t)jc * p.v_st;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int c = lc + 32 * g;
        if (g < ngv) {
          if (fast) vraw[g] = *(const Raw*)(vrow + (c < dv ? c : dv - 4));
          else vraw[g] = narrow(general_load4(vrow, c, dv, j < s.n_kv, false));
        }
      }
    };
    auto stage = [&](int kv0) {
      const bool row_ok = kv0 + lr < s.n_kv;
      const float4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int c = lc + 32 * g;
        if (g < ngk && c < dq4) {
          const float4 t4 = (!fast || (row_ok && c < dq)) ? widen(kraw[g]) : zero4;
          // (rows of K start on 8-byte, not 16-byte boundaries: two stores)
          *(float2*)(Ks + lr * qp_ + c) = float2{t4.x, t4.y};
          *(float2*)(Ks + lr * qp_ + c + 2) = float2{t4.z, t4.w};
        }
        if (g < ngv && c < vcols) *(float4*)(Vs + lr * vp_ + c) = (!fast || (row_ok && c < dv)) ? widen(vraw[g]) : zero4;
      }
    };
    // the slack behind a row's channels is read by the logit loop when the head dim is no multiple of 16
    // (what lies behind the slack is tile data: finite)
    for (int e = tid; e < GT * (qp_ - dq4); e += 256) Ks[(e / (qp_ - dq4)) * qp_ + dq4 + e % (qp_ - dq4)] = 0.f;
    if (kv_begin < kv_end) {
      fetch_k(kv_begin);
      fetch_v(kv_begin);
    }

    for (int kv0 = kv_begin; kv0 < kv_end; kv0 += GT) {
      // nothing for a wave whose rows all lie before these keys (causal) or outside the window
      bool live = r0 < s.n_q;
      if (p.causal && kv0 > r0 + 31) live = false;
      if (p.window >= 0 && (kv0 > r0 + 31 + p.window || kv0 + 31 + p.window < r0)) live = false;
      // an explicit mask: the bytes of the lane's 16 pairs, asked for ahead of the barriers below; a block they
      // all drop is left out altogether
      uint32_t mw[4] = {~0u, ~0u, ~0u, ~0u};
      if (live && p.mask) general_mask_words<!TAB>(p, b, qi, kv0, hh, mw);
      // (the block's dense-bias values likewise, where there are registers for them: one wave per SIMD)
      constexpr bool DENSE_AHEAD = DMAX > 128;
      float db[DENSE_AHEAD ? 16 : 1];
      if constexpr (DENSE_AHEAD) {
        if (live && p.dense_bias) general_dense_row<!TAB>(p, b, qi, kv0, hh, db);
      }
      __syncthreads();                     // everyone is done with the tile before
      stage(kv0);
      __syncthreads();
      // the next tile: its K rows are asked for now, its V rows once the pointwise part is done (fewer
      // registers held across it)
      const bool more = kv0 + GT < kv_end;
      if (more) fetch_k(kv0 + GT);
      if (live && p.mask && __builtin_amdgcn_ballot_w64((mw[0] | mw[1] | mw[2] | mw[3]) != 0u) == 0) live = false;
      if (!live) {
        if (more) fetch_v(kv0 + GT);
        continue;
      }
      floatx16 sacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[r] = 0.f;
      const float* krow = Ks + m * qp_ + 2 * hh;
#pragma unroll
      for (int u0 = 0; u0 < NU; u0 += 4) {
        if (4 * u0 < dq4) {       // (sixteen channels at a time; head dims that are no multiple of 16 read up to 12 floats
          float2 kk[4];           // of the pitch's slack or of the rows behind, and multiply them by zeros of Q)
#pragma unroll
          for (int u = 0; u < 4; ++u) kk[u] = *(const float2*)(krow + 4 * (u0 + u));
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kk[u].x, qf[u0 + u].x, sacc, 0, 0, 0);
            sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kk[u].y, qf[u0 + u].y, sacc, 0, 0, 0);
          }
        }
      }
      // lane holds S^T[key kv0 + 8g + 4hh + tt][query qi], r = 4g + tt.  The index masks are two bounds per
      // lane; segment ids and the biases go through the per-pair helpers only when present.
      int hi = s.n_kv - 1, lo = 0;
      if (p.causal) hi = qi < hi ? qi : hi;
      if (p.window >= 0) {
        hi = qi + p.window < hi ? qi + p.window : hi;
        lo = qi - p.window;
      }
      if (qi >= s.n_q) hi = -1;
      const bool by_seg = p.mask_mode == HSTU_MASK_SEGMENT;
      const bool tabled = TAB && (p.pos_tab != nullptr || p.ts_tab != nullptr);
      // (dropout: the part of the pair's hash that this lane's row fixes)
      const uint32_t drop_row = drop_bh_key(p.drop_key, (uint32_t)b * (uint32_t)p.H + (uint32_t)h) + (uint32_t)qi * DROP_CI;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = kv0 + 8 * (r >> 2) + 4 * hh + (r & 3);
        bool keep = j >= lo && j <= hi && ((mw[r >> 2] >> (8 * (r & 3))) & 0xffu) != 0u;
        if (by_seg) keep = keep && general_same_segment(p, b, qi, j);
        if (p.drop_thr) keep = keep && drop_keep_mixed(drop_row + (uint32_t)j * DROP_CJ, p.drop_thr);
        float x = p.alpha * sacc[r];
        if (tabled && keep) x += general_table_bias(p, s, b, h, qi, j);
        if constexpr (DENSE_AHEAD) {
          if (p.dense_bias) x += db[r];
        } else {
          if (p.dense_bias && keep)
            x += p.dense_bias[(p.dense_bias_batched ? (int64_t)b * p.L * p.Lkv : 0) + (int64_t)qi * p.Lkv + j];
        }
        // silu(x) = x / (1 + e^-x), by the hardware's exp2 and reciprocal (1 ulp each)
        const float val = x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-x * LOG2E));
        sacc[r] = keep ? val : 0.f;      // P^T in place of S^T
      }
      if (more) fetch_v(kv0 + GT);
      const float* vcol = Vs + (4 * hh) * vp_ + m;
#pragma unroll
      for (int x = 0; x < NB; ++x) {
        if (x < nblk) {
#pragma unroll
          for (int r = 0; r < 16; ++r)
            o[x] = __builtin_amdgcn_mfma_f32_32x32x2f32(vcol[(8 * (r >> 2) + (r & 3)) * vp_ + 32 * x], sacc[r], o[x], 0, 0, 0);
        }
      }
    }
  }
  // O^T[channel 32x + 8g + 4hh + tt][query qi]; rows past the sequence are written as exact zeros (padded layout)
  if (qi < s.rows) {
    const bool live_row = qi < s.n_q;
#pragma unroll
    for (int x = 0; x < NB; ++x) {
      if (x < nblk) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int c = 32 * x + 8 * (r >> 2) + 4 * hh + (r & 3);
          if (c < dv) stf(op + s.bo + (int64_t)qi * p.o_st + c, live_row ? o[x][r] * p.inv_n : 0.f);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Backward, general form (fp32 FMA arithmetic, every option of the forward):
//   P = silu(S)/N masked, dV = P^T dO, dP = dO V^T,
//   dS = dP sigma(S) (1 + S (1 - sigma(S))) / N masked, dQ = alpha dS K, dK = alpha dS^T Q,
// and every (i, j) adds dS to the table entries its logit read
// (recml/core/ops/hstu_ops.py:461-517 for q, k, v).  S is recomputed in both kernels.
// ---------------------------------------------------------------------------

// logit x, keep flag and timestamp bucket of pair (i, j); returns dS given dP, and P through *pout
__device__ __forceinline__ float bwd_pair(const Params& p, const Seq& s, int b, int h, int i, int j,
                                          float qk, float dp, float* pout, int* bucket) {
  *pout = 0.f;
  if (!general_keep(p, s, b, i, j)) return 0.f;
  if (p.drop_thr && !drop_keep(drop_bh_key(p.drop_key, (uint32_t)b * (uint32_t)p.H + (uint32_t)h), (uint32_t)i, (uint32_t)j, p.drop_thr)) return 0.f;
  const float x = p.alpha * qk + general_bias(p, s, b, h, i, j, bucket);
  const float sg = 1.0f / (1.0f + expf(-x));
  *pout = x * sg * p.inv_n;
  return dp * sg * (1.0f + x * (1.0f - sg)) * p.inv_n;
}

// dQ and the table gradients: one workgroup per 32 query rows of one (sequence, head), keys streamed
template <typename T>
__global__ __launch_bounds__(256) void hstu_bwd_dq(const Params p) {
  extern __shared__ float gsm[];
  const int dq = p.d_qk, dv = p.d_v;
  const int kp = dq + 1, vp_ = dv + 1;     // odd pitches: one row per lane reads
  float* Qs = gsm;                         // [GT][dq]
  float* Os = Qs + GT * dq;                // [GT][dv]   dO rows
  float* Ks = Os + GT * dv;                // [GT][kp]
  float* Vs = Ks + GT * kp;                // [GT][vp_]
  float* Ds = Vs + GT * vp_;               // [GT][GT+1] dS
  float* Hist = Ds + GT * (GT + 1);        // [ts_nb + 1] timestamp-bucket sums of this tile
  int* Bk = (int*)(Hist + general_hist_len(p.ts_nb));   // [GT][GT] bucket of each pair

  // (head fastest, tile slowest and longest first: see hstu_fwd_general)
  const int h = blockIdx.x, b = blockIdx.y, qt = gridDim.z - 1 - blockIdx.z;
  const Seq s = seq_info(p, b, h);
  const int q0 = qt * GT;
  if (q0 >= s.rows) return;
  const int tid = threadIdx.x;
  const T* __restrict__ qp = (const T*)p.q;
  const T* __restrict__ kp_ = (const T*)p.k;
  const T* __restrict__ vp = (const T*)p.v;
  const T* __restrict__ dop = (const T*)p.dout;
  T* __restrict__ dqp = (T*)p.dq;
  const bool want_ts = p.dts != nullptr && p.ts_tab != nullptr;
  const bool want_pos = p.dpos != nullptr && p.pos_tab != nullptr;

  const int oi = tid >> 3, ocg = tid & 7;
  const int nx = (dq + 7) >> 3;
  float acc[GMAXX];
#pragma unroll
  for (int x = 0; x < GMAXX; ++x) acc[x] = 0.f;

  if (q0 < s.n_q) {
    for (int e = tid; e < GT * dq; e += 256) {
      int r = e / dq, c = e - r * dq, i = q0 + r;
      Qs[e] = (i < s.n_q) ? ldf(qp + s.bq + (int64_t)i * p.q_st + c) : 0.f;
    }
    for (int e = tid; e < GT * dv; e += 256) {
      int r = e / dv, c = e - r * dv, i = q0 + r;
      Os[e] = (i < s.n_q) ? ldf(dop + s.bo + (int64_t)i * p.o_st + c) : 0.f;
    }
    if (want_ts) for (int e = tid; e <= p.ts_nb; e += 256) Hist[e] = 0.f;
    int kv_end = s.n_kv;
    if (p.causal && q0 + GT < kv_end) kv_end = q0 + GT;
    if (p.window >= 0 && q0 + GT + p.window < kv_end) kv_end = q0 + GT + p.window;
    int kv_begin = 0;
    if (p.window >= 0 && q0 - p.window > 0) kv_begin = ((q0 - p.window) / GT) * GT;

    for (int kv0 = kv_begin; kv0 < kv_end; kv0 += GT) {
      __syncthreads();
      for (int e = tid; e < GT * dq; e += 256) {
        int r = e / dq, c = e - r * dq, j = kv0 + r;
        Ks[r * kp + c] = (j < s.n_kv) ? ldf(kp_ + s.bk + (int64_t)j * p.k_st + c) : 0.f;
      }
      for (int e = tid; e < GT * dv; e += 256) {
        int r = e / dv, c = e - r * dv, j = kv0 + r;
        Vs[r * vp_ + c] = (j < s.n_kv) ? ldf(vp + s.bv + (int64_t)j * p.v_st + c) : 0.f;
      }
      __syncthreads();
      {
        const int tx = tid & 31, ty = tid >> 5;
        float sacc[4] = {0.f, 0.f, 0.f, 0.f}, pacc[4] = {0.f, 0.f, 0.f, 0.f};
        const float* krow = Ks + tx * kp;
        for (int c = 0; c < dq; ++c) {
          const float kvv = krow[c];
#pragma unroll
          for (int r = 0; r < 4; ++r) sacc[r] = fmaf(Qs[(ty + 8 * r) * dq + c], kvv, sacc[r]);
        }
        const float* vrow = Vs + tx * vp_;
        for (int c = 0; c < dv; ++c) {
          const float vv = vrow[c];
#pragma unroll
          for (int r = 0; r < 4; ++r) pacc[r] = fmaf(Os[(ty + 8 * r) * dv + c], vv, pacc[r]);
        }
        const int j = kv0 + tx;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = q0 + ty + 8 * r;
          float pval;
          int bk = 0;
          const float ds = bwd_pair(p, s, b, h, i, j, sacc[r], pacc[r], &pval, &bk);
          Ds[(ty + 8 * r) * (GT + 1) + tx] = ds;
          if (want_ts) Bk[(ty + 8 * r) * GT + tx] = bk;
        }
      }
      __syncthreads();
      if (p.dbias) {
        float* db = p.dbias + (p.dense_bias_batched ? (int64_t)b * p.L * p.Lkv : 0);
        for (int e = tid; e < GT * GT; e += 256) {
          const float ds = Ds[(e >> 5) * (GT + 1) + (e & 31)];
          if (ds != 0.f) atomicAdd(db + (int64_t)(q0 + (e >> 5)) * p.Lkv + kv0 + (e & 31), ds);
        }
      }
      // table gradients of this tile: one sum per diagonal (position), one LDS histogram (time)
      if (want_pos && tid < 2 * GT - 1) {
        const int dd = tid - (GT - 1);           // j - i inside the tile
        float sum = 0.f;
        for (int r = 0; r < GT; ++r) {
          const int c = r + dd;
          if (c >= 0 && c < GT) sum += Ds[r * (GT + 1) + c];
        }
        const int idx = (p.L - 1) + (kv0 - q0) + dd;
        if (sum != 0.f && idx >= 0 && idx < 2 * p.L - 1)
          atomicAdd(p.dpos + (int64_t)(p.pos_heads > 1 ? h : 0) * (2 * p.L - 1) + idx, sum);
      }
      if (want_ts) {
        for (int e = tid; e < GT * GT; e += 256) {
          const float ds = Ds[(e >> 5) * (GT + 1) + (e & 31)];
          if (ds != 0.f) atomicAdd(Hist + Bk[e], ds);
        }
      }
      for (int jj = 0; jj < GT; ++jj) {
        const float ds = Ds[oi * (GT + 1) + jj];
        const float* krow = Ks + jj * kp;
#pragma unroll
        for (int x = 0; x < GMAXX; ++x) {
          if (x < nx) {
            const int c = ocg + 8 * x;
            if (c < dq) acc[x] = fmaf(ds, krow[c], acc[x]);
          }
        }
      }
    }
    if (want_ts) {
      __syncthreads();
      for (int e = tid; e <= p.ts_nb; e += 256)
        if (Hist[e] != 0.f) atomicAdd(p.dts + (int64_t)(p.ts_heads > 1 ? h : 0) * (p.ts_nb + 1) + e, Hist[e]);
    }
  }
  const int i = q0 + oi;
  if (i < s.rows) {
    const bool live = i < s.n_q;
#pragma unroll
    for (int x = 0; x < GMAXX; ++x) {
      if (x < nx) {
        const int c = ocg + 8 * x;
        if (c < dq) stf(dqp + s.bq + (int64_t)i * p.q_st + c, live ? acc[x] * p.alpha : 0.f);
      }
    }
  }
}

// dK and dV: one workgroup per 32 keys of one (sequence, head), query rows streamed
template <typename T>
__global__ __launch_bounds__(256) void hstu_bwd_dkv(const Params p) {
  extern __shared__ float gsm[];
  const int dq = p.d_qk, dv = p.d_v;
  const int kp = dq + 1, vp_ = dv + 1;
  float* Ks = gsm;                         // [GT][kp]
  float* Vs = Ks + GT * kp;                // [GT][vp_]
  float* Qs = Vs + GT * vp_;               // [GT][dq]
  float* Os = Qs + GT * dq;                // [GT][dv]
  float* Ds = Os + GT * dv;                // [GT][GT+1] dS   [row][key]
  float* Ps = Ds + GT * (GT + 1);          // [GT][GT+1] P

  // (head fastest, tile slowest; under the causal mask the first key tile has the most rows behind it)
  const int h = blockIdx.x, b = blockIdx.y, kt = blockIdx.z;
  const Seq s = seq_info(p, b, h);
  const int kv0 = kt * GT;
  const int krows = p.jagged ? s.n_kv : p.Lkv;      // rows of dk / dv that exist
  if (kv0 >= krows) return;
  const int tid = threadIdx.x;
  const T* __restrict__ qp = (const T*)p.q;
  const T* __restrict__ kp_ = (const T*)p.k;
  const T* __restrict__ vp = (const T*)p.v;
  const T* __restrict__ dop = (const T*)p.dout;
  T* __restrict__ dkp = (T*)p.dk;
  T* __restrict__ dvp = (T*)p.dv;

  const int oj = tid >> 3, ocg = tid & 7;
  const int nxk = (dq + 7) >> 3, nxv = (dv + 7) >> 3;
  float acck[GMAXX], accv[GMAXX];
#pragma unroll
  for (int x = 0; x < GMAXX; ++x) { acck[x] = 0.f; accv[x] = 0.f; }

  if (kv0 < s.n_kv) {
    for (int e = tid; e < GT * dq; e += 256) {
      int r = e / dq, c = e - r * dq, j = kv0 + r;
      Ks[r * kp + c] = (j < s.n_kv) ? ldf(kp_ + s.bk + (int64_t)j * p.k_st + c) : 0.f;
    }
    for (int e = tid; e < GT * dv; e += 256) {
      int r = e / dv, c = e - r * dv, j = kv0 + r;
      Vs[r * vp_ + c] = (j < s.n_kv) ? ldf(vp + s.bv + (int64_t)j * p.v_st + c) : 0.f;
    }
    // query rows that can see these keys
    int q_begin = 0, q_end = s.n_q;
    if (p.causal) q_begin = kv0;
    if (p.window >= 0 && kv0 - p.window > q_begin) q_begin = kv0 - p.window;
    if (p.window >= 0 && kv0 + GT + p.window < q_end) q_end = kv0 + GT + p.window;
    q_begin = (q_begin / GT) * GT;
    for (int q0 = q_begin; q0 < q_end; q0 += GT) {
      __syncthreads();
      for (int e = tid; e < GT * dq; e += 256) {
        int r = e / dq, c = e - r * dq, i = q0 + r;
        Qs[e] = (i < s.n_q) ? ldf(qp + s.bq + (int64_t)i * p.q_st + c) : 0.f;
      }
      for (int e = tid; e < GT * dv; e += 256) {
        int r = e / dv, c = e - r * dv, i = q0 + r;
        Os[e] = (i < s.n_q) ? ldf(dop + s.bo + (int64_t)i * p.o_st + c) : 0.f;
      }
      __syncthreads();
      {
        const int tx = tid & 31, ty = tid >> 5;
        float sacc[4] = {0.f, 0.f, 0.f, 0.f}, pacc[4] = {0.f, 0.f, 0.f, 0.f};
        const float* krow = Ks + tx * kp;
        for (int c = 0; c < dq; ++c) {
          const float kvv = krow[c];
#pragma unroll
          for (int r = 0; r < 4; ++r) sacc[r] = fmaf(Qs[(ty + 8 * r) * dq + c], kvv, sacc[r]);
        }
        const float* vrow = Vs + tx * vp_;
        for (int c = 0; c < dv; ++c) {
          const float vv = vrow[c];
#pragma unroll
          for (int r = 0; r < 4; ++r) pacc[r] = fmaf(Os[(ty + 8 * r) * dv + c], vv, pacc[r]);
        }
        const int j = kv0 + tx;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = q0 + ty + 8 * r;
          float pval;
          const float ds = bwd_pair(p, s, b, h, i, j, sacc[r], pacc[r], &pval, nullptr);
          Ds[(ty + 8 * r) * (GT + 1) + tx] = ds;
          Ps[(ty + 8 * r) * (GT + 1) + tx] = pval;
        }
      }
      __syncthreads();
      for (int ii = 0; ii < GT; ++ii) {
        const float ds = Ds[ii * (GT + 1) + oj], pv = Ps[ii * (GT + 1) + oj];
        const float* qrow = Qs + ii * dq;
        const float* orow = Os + ii * dv;
#pragma unroll
        for (int x = 0; x < GMAXX; ++x) {
          const int c = ocg + 8 * x;
          if (x < nxk && c < dq) acck[x] = fmaf(ds, qrow[c], acck[x]);
          if (x < nxv && c < dv) accv[x] = fmaf(pv, orow[c], accv[x]);
        }
      }
    }
  }
  const int j = kv0 + oj;
  if (j < krows) {
    const bool live = j < s.n_kv;
#pragma unroll
    for (int x = 0; x < GMAXX; ++x) {
      const int c = ocg + 8 * x;
      if (x < nxk && c < dq) stf(dkp + s.bk + (int64_t)j * p.k_st + c, live ? acck[x] * p.alpha : 0.f);
      if (x < nxv && c < dv) stf(dvp + s.bv + (int64_t)j * p.v_st + c, live ? accv[x] : 0.f);
    }
  }
}

// ---------------------------------------------------------------------------
// The general backward on the fp32 matrix cores (head dims up to 128; beyond that the two kernels above).
// Same products, masks and biases as above; tiles of 32 rows travel through registers into LDS as in
// hstu_fwd_general, each in up to two layouts: pitch twice an odd number where its rows are the A operand of
// a product over the channels (two floats per lane and pair of steps), pitch 8 more than a multiple of 32
// where its rows are read across the channels (A operand of a product over the tile's 32 rows).
// ---------------------------------------------------------------------------

typedef __attribute__((address_space(3))) float* general_lds_float_ptr;   // (a float atomic on LDS named as such)

// A tile of 32 rows x d channels of a [row][channel] array, rows `row0 ..` of at most `nrows`: eight threads per
// row, four channels per thread and turn, held in registers between fetch and stage.
template <typename T, int NG>
struct GeneralTile {
  typedef typename std::conditional<sizeof(T) == 4, float4, uint2>::type Raw;
  Raw raw[NG];
  static __device__ __forceinline__ float4 widen(const Raw& u) {
    if constexpr (sizeof(T) == 4) {
      return u;
    } else {
      return float4{__builtin_bit_cast(float, u.x << 16), __builtin_bit_cast(float, u.x & 0xffff0000u),
                    __builtin_bit_cast(float, u.y << 16), __builtin_bit_cast(float, u.y & 0xffff0000u)};
    }
  }
  static __device__ __forceinline__ Raw narrow(const float4& f) {
    if constexpr (sizeof(T) == 4) {
      return f;
    } else {
      return uint2{(__builtin_bit_cast(uint32_t, f.x) >> 16) | (__builtin_bit_cast(uint32_t, f.y) & 0xffff0000u),
                   (__builtin_bit_cast(uint32_t, f.z) >> 16) | (__builtin_bit_cast(uint32_t, f.w) & 0xffff0000u)};
    }
  }
  // fast: whole groups of four can be loaded (aligned base and row stride, d a multiple of four); then the loads
  // are unconditional (rows past the end re-read the last row) and stage() writes the zeros
  __device__ __forceinline__ void fetch(const T* base, int64_t row_stride, int row0, int nrows, int d, bool fast, int tid) {
    const int lr = tid >> 3, lc = (tid & 7) * 4;
    const int d4 = (d + 3) & ~3;
    const int ng = (d4 + 31) >> 5;
    const int j = row0 + lr;
    const int jc = fast && j >= nrows ? nrows - 1 : j;
    const T* row = base + (int64_t)jc * row_stride;
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const int c = lc + 32 * g;
      if (g < ng) {
        if (fast) raw[g] = *(const Raw*)(row + (c < d ? c : d - 4));
        else raw[g] = narrow(general_load4(row, c, d, j < nrows, false));
      }
    }
  }
  // into LDS: `by_row` (pitch twice an odd number: 8-byte stores) and / or `by_col` (pitch a multiple of four)
  __device__ __forceinline__ void stage(int row0, int nrows, int d, bool fast, int tid, float* by_row, int pitch_row, float* by_col,
                                        int pitch_col) const {
    const int lr = tid >> 3, lc = (tid & 7) * 4;
    const int d4 = (d + 3) & ~3;
    const int ng = (d4 + 31) >> 5;
    const bool row_ok = row0 + lr < nrows;
    const float4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < NG; ++g) {
      const int c = lc + 32 * g;
      if (g < ng && c < d4) {
        const float4 t4 = (!fast || (row_ok && c < d)) ? widen(raw[g]) : zero4;
        if (by_row) {
          *(float2*)(by_row + lr * pitch_row + c) = float2{t4.x, t4.y};
          *(float2*)(by_row + lr * pitch_row + c + 2) = float2{t4.z, t4.w};
        }
        if (by_col) *(float4*)(by_col + lr * pitch_col + c) = t4;
      }
    }
  }
  // bf16 storage, kept as bf16 in LDS (the instances with bf16 products; `fast` loads only): rows at `by_row`
  // (pitch in bytes, a multiple of 16) and / or transposed at `by_chan`: [channel][row of the tile], pitch in bytes
  __device__ __forceinline__ void stage_bf16(int row0, int nrows, int d, int tid, unsigned char* by_row, int pitch_row,
                                             unsigned char* by_chan, int pitch_chan) const {
    static_assert(sizeof(T) == 2 || sizeof(T) == 4, "");
    if constexpr (sizeof(T) == 2) {
      const int lr = tid >> 3, lc = (tid & 7) * 4;
      const int ng = (d + 31) >> 5;
      const bool row_ok = row0 + lr < nrows;
#pragma unroll
      for (int g = 0; g < NG; ++g) {
        const int c = lc + 32 * g;
        if (g < ng && c < d) {
          const uint2 v = row_ok ? raw[g] : uint2{0u, 0u};
          if (by_row) *(uint2*)(by_row + lr * pitch_row + 2 * c) = v;
          if (by_chan) {
            unsigned short* col = (unsigned short*)(by_chan + c * pitch_chan) + lr;
            const int ps = pitch_chan >> 1;
            col[0] = (unsigned short)(v.x & 0xffffu);
            col[ps] = (unsigned short)(v.x >> 16);
            col[2 * ps] = (unsigned short)(v.y & 0xffffu);
            col[3 * ps] = (unsigned short)(v.y >> 16);
          }
        }
      }
    }
  }
};

// The lane's share of row `row` as the B operand of a product over the channels: channels 4u + 2hh and
// 4u + 2hh + 1 for the pair of steps u; zeros past d or when the row does not exist.
template <typename T>
__device__ __forceinline__ void general_row_frag(float2 (&f)[32], const T* row, int d, bool row_ok, int hh) {
  const int d4 = (d + 3) & ~3;
#pragma unroll
  for (int u = 0; u < 32; ++u) {
    f[u] = float2{0.f, 0.f};
    if (4 * u < d4 && row_ok) {
      const int c = 4 * u + 2 * hh;
      if (c < d) f[u].x = ldf(row + c);
      if (c + 1 < d) f[u].y = ldf(row + c + 1);
    }
  }
}

// out[x]^T += A^T B over the tile's 32 rows: A = LDS tile read across the channels (`acol` = tile + 4 hh rows + m,
// pitch 8 more than a multiple of 32), B = the 16 values of an accumulator (row 8g + 4hh + tt, r = 4g + tt).
template <int NB>
__device__ __forceinline__ void general_dot_cols(floatx16 (&out)[NB], const float* acol, int pitch, const floatx16& bv, int nblk) {
#pragma unroll
  for (int x = 0; x < NB; ++x) {
    if (x < nblk) {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        out[x] = __builtin_amdgcn_mfma_f32_32x32x2f32(acol[(8 * (r >> 2) + (r & 3)) * pitch + 32 * x], bv[r], out[x], 0, 0, 0);
    }
  }
}

// ---- the same products on the bf16 matrix cores, for tensors stored in bf16 (BP instances of the two kernels) ----
// Every operand of the first two products is then a bf16 value, so v_mfma_f32_32x32x16_bf16 forms the same
// products and fp32 sums in one instruction per 16 channels instead of eight per 16; P and dS are rounded to
// bf16 for the last products, as the forward rounds P.  The instruction leaves its result in the same lanes and
// registers as the fp32 one, so everything between the products is shared.  The tiles are kept in LDS as bf16:
// by rows for the products over the channels (16-byte reads), transposed for the products over the tile's rows
// (a lane's eight rows of a product are two 8-byte reads).
__device__ __forceinline__ uint32_t general_pack_bf16(float lo, float hi) {
  floatx2 f = {lo, hi};
  typedef bf16_t bf16x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}
// The lane's share of a bf16 row as the B operand: channels 16 ks + 8 hh .. + 7 (16-byte reads: d a multiple
// of 16, rows on 16-byte boundaries); zeros when the row does not exist.
__device__ __forceinline__ void general_row_frag_bf16(bf16x8 (&f)[8], const bf16_t* row, int d, bool row_ok, int hh) {
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    uint4 v = {0u, 0u, 0u, 0u};
    if (16 * ks < d && row_ok) v = *(const uint4*)(row + 16 * ks + 8 * hh);
    f[ks] = __builtin_bit_cast(bf16x8, v);
  }
}
// acc += A B^T over the channels: `arow` = the lane's row of the bf16 tile + 16 hh bytes (16-byte reads)
__device__ __forceinline__ void general_dot_rows_bf16(floatx16& acc, const unsigned char* arow, const bf16x8 (&bf)[8], int d) {
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) {
    if (16 * ks < d) {
      const uint4 pa = *(const uint4*)(arow + 32 * ks);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, pa), bf[ks], acc, 0, 0, 0);
    }
  }
}
// out[x]^T += A^T B over the tile's 32 rows, 16 at a time: B = the accumulator's values 8 cc .. 8 cc + 7 (rows
// 16 cc + 4 hh + tt and 16 cc + 8 + 4 hh + tt), A = channel 32 x + m of the same rows: two 8-byte reads of the
// transposed tile (`acol` = its channel m + 8 hh bytes, `pitch` bytes per channel)
template <int NB>
__device__ __forceinline__ void general_dot_cols_bf16(floatx16 (&out)[NB], const unsigned char* acol, int pitch, const floatx16& bv, int nblk) {
#pragma unroll
  for (int cc = 0; cc < 2; ++cc) {
    const uint4 pb = {general_pack_bf16(bv[8 * cc + 0], bv[8 * cc + 1]), general_pack_bf16(bv[8 * cc + 2], bv[8 * cc + 3]),
                      general_pack_bf16(bv[8 * cc + 4], bv[8 * cc + 5]), general_pack_bf16(bv[8 * cc + 6], bv[8 * cc + 7])};
#pragma unroll
    for (int x = 0; x < NB; ++x) {
      if (x < nblk) {
        const unsigned char* ap = acol + 32 * x * pitch + 32 * cc;
        const uint2 lo = *(const uint2*)ap, hi = *(const uint2*)(ap + 16);
        const uint4 pa = {lo.x, lo.y, hi.x, hi.y};
        out[x] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, pa), __builtin_bit_cast(bf16x8, pb), out[x], 0, 0, 0);
      }
    }
  }
}
// Pitches of the bf16 tiles in bytes: rows of d channels + 16 bytes (16 consecutive rows then sweep the banks once
// under 16-byte reads); a channel's 32 keys + 8 bytes (72: consecutive channels 18 banks apart, 8-byte reads).
__host__ __device__ inline int general_bf16_row_pitch(int d) { return 2 * d + 16; }
constexpr int GENERAL_BF16_CHAN_PITCH = 72;
__host__ __device__ inline int general_bwd_dq_lds_bf16(int dq, int dv, bool want_ds, int ts_nb) {   // bytes
  return GT * general_bf16_row_pitch(dq) + dq * GENERAL_BF16_CHAN_PITCH + GT * general_bf16_row_pitch(dv) +
         4 * ((want_ds ? 4 * GT * (GT + 1) : 0) + general_hist_len(ts_nb));
}
__host__ __device__ inline int general_bwd_dkv_lds_bf16(int dq, int dv) {                            // bytes
  return GT * general_bf16_row_pitch(dq) + dq * GENERAL_BF16_CHAN_PITCH + GT * general_bf16_row_pitch(dv) + dv * GENERAL_BF16_CHAN_PITCH;
}

// LDS floats of the two kernels (host and device agree through these)
__host__ __device__ inline int general_bwd_dq_lds(int dq, int dv, bool want_pos, int ts_nb) {
  return GT * (general_pitch_qk(dq) + general_pitch_v(dq) + general_pitch_qk(dv)) + (want_pos ? 4 * GT * (GT + 1) : 0) + general_hist_len(ts_nb);
}
__host__ __device__ inline int general_bwd_dkv_lds(int dq, int dv) {
  return GT * (general_pitch_qk(dq) + general_pitch_v(dq) + general_pitch_qk(dv) + general_pitch_v(dv));
}

// dQ and the table gradients: one workgroup per 128 query rows of one (sequence, head), 32 per wave, keys streamed.
//   S^T = K Q^T, dP^T = V dO^T (A = K / V rows, B = the wave's Q / dO rows in registers), dS^T pointwise,
//   dQ^T += K^T dS^T (A = K read across the channels, B = dS^T as it leaves the pointwise part).
template <typename T, bool BP = false, bool TAB = true>
__global__ __launch_bounds__(256, (BP && !TAB) ? 2 : 1) void hstu_bwd_dq_mm(const Params p) {
  extern __shared__ __attribute__((aligned(16))) float gsm[];
  const int dq = p.d_qk, dv = p.d_v;
  const int dq4 = (dq + 3) & ~3, dv4 = (dv + 3) & ~3;
  const int pk = general_pitch_qk(dq), pc = general_pitch_v(dq), pv = general_pitch_qk(dv);
  // (TAB = false: an instance for calls without bias tables, which then carries none of their code)
  const bool want_ts = TAB && p.dts != nullptr && p.ts_tab != nullptr;
  const bool want_pos = TAB && p.dpos != nullptr && p.pos_tab != nullptr;
  float* Kr = gsm;                         // [32][pk]  K rows for S^T
  float* Kc = Kr + GT * pk;                // [32][pc]  K read across the channels for dQ^T
  float* Vr = Kc + GT * pc;                // [32][pv]  V rows for dP^T
  // (bf16 products: [32][prk bytes] K rows | [dq][72 bytes] K transposed | [32][prv bytes] V rows)
  unsigned char* const smb = (unsigned char*)gsm;
  const int prk = general_bf16_row_pitch(dq), prv = general_bf16_row_pitch(dv);
  unsigned char* const Krb = smb;
  unsigned char* const Ktb = Krb + GT * prk;
  unsigned char* const Vrb = Ktb + dq * GENERAL_BF16_CHAN_PITCH;
  float* Hist = BP ? (float*)(Vrb + GT * prv) : Vr + GT * pv;   // [buckets] timestamp-bucket sums of this workgroup
  float* Ds = Hist + general_hist_len(p.ts_nb);   // [4][32][33] dS of each wave's block, [query][key] (position and dense-bias gradients only)

  const int h = blockIdx.x, b = blockIdx.y, qt = gridDim.z - 1 - blockIdx.z;
  const Seq s = seq_info(p, b, h);
  const int q0 = qt * 128;
  if (q0 >= s.rows) return;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, m = lane & 31, hh = lane >> 5;
  const T* __restrict__ qp = (const T*)p.q + s.bq;
  const T* __restrict__ kp_ = (const T*)p.k + s.bk;
  const T* __restrict__ vp = (const T*)p.v + s.bv;
  const T* __restrict__ dop = (const T*)p.dout + s.bo;
  T* __restrict__ dqp = (T*)p.dq + s.bq;
  const int r0 = q0 + 32 * w, qi = r0 + m;
  constexpr uintptr_t VMASK = sizeof(T) * 4 - 1;
  // (bf16 products are only taken with rows on 16-byte boundaries and head dims in multiples of 16)
  // (and the instances without tables, fp32 ones included, are only launched where whole groups of four can be fetched)
  const bool kfast = BP || !TAB || ((((uintptr_t)kp_ & VMASK) == 0) && (p.k_st & 3) == 0 && (dq & 3) == 0);
  const bool vfast = BP || !TAB || ((((uintptr_t)vp & VMASK) == 0) && (p.v_st & 3) == 0 && (dv & 3) == 0);
  constexpr bool LEAN = !TAB;            // also: mask and dense bias fetched by whole words (checked at the launch)

  constexpr int NB = 4;
  const int nblk = (dq + 31) >> 5;
  floatx16 o[NB];
#pragma unroll
  for (int x = 0; x < NB; ++x)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[x][r] = 0.f;

  if (q0 < s.n_q) {
    float2 qf[BP ? 1 : 32], dof[BP ? 1 : 32];
    bf16x8 qb[BP ? 8 : 1], dob[BP ? 8 : 1];
    if constexpr (BP) {
      general_row_frag_bf16(qb, (const bf16_t*)(qp + (int64_t)qi * p.q_st), dq, qi < s.n_q, hh);
      general_row_frag_bf16(dob, (const bf16_t*)(dop + (int64_t)qi * p.o_st), dv, qi < s.n_q, hh);
    } else {
      general_row_frag(qf, qp + (int64_t)qi * p.q_st, dq, qi < s.n_q, hh);
      general_row_frag(dof, dop + (int64_t)qi * p.o_st, dv, qi < s.n_q, hh);
    }
    if (want_ts) for (int e = tid; e <= p.ts_nb; e += 256) Hist[e] = 0.f;
    int kv_end = s.n_kv;
    if (p.causal && q0 + 128 < kv_end) kv_end = q0 + 128;
    if (p.window >= 0 && q0 + 128 + p.window < kv_end) kv_end = q0 + 128 + p.window;
    int kv_begin = 0;
    if (p.window >= 0 && q0 - p.window > 0) kv_begin = ((q0 - p.window) / GT) * GT;
    if (p.mask) {
      // the steps before the first and after the last key the mask keeps for these rows are left out
      int t_lo = kv_begin / GT, t_hi = (kv_end + GT - 1) / GT;
      general_mask_live_steps<true>(p, b, q0, tid, t_lo, t_hi);
      kv_begin = t_lo * GT > kv_begin ? t_lo * GT : kv_begin;
      kv_end = t_hi * GT < kv_end ? t_hi * GT : kv_end;
    }
    GeneralTile<T, 4> kt_, vt_;
    if (kv_begin < kv_end) {
      kt_.fetch(kp_, p.k_st, kv_begin, s.n_kv, dq, kfast, tid);
      vt_.fetch(vp, p.v_st, kv_begin, s.n_kv, dv, vfast, tid);
    }
    int hi = s.n_kv - 1, lo = 0;
    if (p.causal) hi = qi < hi ? qi : hi;
    if (p.window >= 0) {
      hi = qi + p.window < hi ? qi + p.window : hi;
      lo = qi - p.window;
    }
    if (qi >= s.n_q) hi = -1;
    const bool by_seg = p.mask_mode == HSTU_MASK_SEGMENT;
    const bool tabled = TAB && (p.pos_tab != nullptr || p.ts_tab != nullptr);
    float* dsw = Ds + w * (GT * (GT + 1));

    for (int kv0 = kv_begin; kv0 < kv_end; kv0 += GT) {
      bool live = r0 < s.n_q;
      if (p.causal && kv0 > r0 + 31) live = false;
      if (p.window >= 0 && (kv0 > r0 + 31 + p.window || kv0 + 31 + p.window < r0)) live = false;
      // an explicit mask: the bytes of the lane's 16 pairs, asked for ahead of the barriers; a block they all
      // drop is left out
      uint32_t mw[4] = {~0u, ~0u, ~0u, ~0u};
      if (live && p.mask) general_mask_words<LEAN>(p, b, qi, kv0, hh, mw);
      float db[16];
      if (live && p.dense_bias) general_dense_row<LEAN>(p, b, qi, kv0, hh, db);
      __syncthreads();
      if constexpr (BP) {
        kt_.stage_bf16(kv0, s.n_kv, dq, tid, Krb, prk, Ktb, GENERAL_BF16_CHAN_PITCH);
        vt_.stage_bf16(kv0, s.n_kv, dv, tid, Vrb, prv, nullptr, 0);
      } else {
        kt_.stage(kv0, s.n_kv, dq, kfast, tid, Kr, pk, Kc, pc);
        vt_.stage(kv0, s.n_kv, dv, vfast, tid, Vr, pv, nullptr, 0);
      }
      __syncthreads();
      if (kv0 + GT < kv_end) {
        kt_.fetch(kp_, p.k_st, kv0 + GT, s.n_kv, dq, kfast, tid);
        vt_.fetch(vp, p.v_st, kv0 + GT, s.n_kv, dv, vfast, tid);
      }
      if (live && p.mask && __builtin_amdgcn_ballot_w64((mw[0] | mw[1] | mw[2] | mw[3]) != 0u) == 0) live = false;
      if (!live) continue;
      floatx16 sacc, dpacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) { sacc[r] = 0.f; dpacc[r] = 0.f; }
      if constexpr (BP) {
        general_dot_rows_bf16(sacc, Krb + m * prk + 16 * hh, qb, dq);
        general_dot_rows_bf16(dpacc, Vrb + m * prv + 16 * hh, dob, dv);
      } else {
        general_dot_rows(sacc, Kr + m * pk + 2 * hh, qf, dq4);
        general_dot_rows(dpacc, Vr + m * pv + 2 * hh, dof, dv4);
      }
      // lane holds pair (query qi, key kv0 + 8g + 4hh + tt), r = 4g + tt
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = kv0 + 8 * (r >> 2) + 4 * hh + (r & 3);
        bool keep = j >= lo && j <= hi && ((mw[r >> 2] >> (8 * (r & 3))) & 0xffu) != 0u;
        if (by_seg) keep = keep && general_same_segment(p, b, qi, j);
        if (p.drop_thr) keep = keep && drop_keep(drop_bh_key(p.drop_key, (uint32_t)b * (uint32_t)p.H + (uint32_t)h), (uint32_t)qi, (uint32_t)j, p.drop_thr);
        float x = p.alpha * sacc[r];
        int bk = 0;
        if (tabled && keep) x += general_table_bias(p, s, b, h, qi, j, &bk);
        if (p.dense_bias) x += db[r];
        const float sg = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-x * LOG2E));
        const float ds = keep ? dpacc[r] * sg * (1.0f + x * (1.0f - sg)) * p.inv_n : 0.f;
        sacc[r] = ds;                      // dS^T in place of S^T
        if (want_ts && ds != 0.f) __hip_atomic_fetch_add((general_lds_float_ptr)(Hist + bk), ds, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (want_pos || p.dbias) dsw[m * (GT + 1) + 8 * (r >> 2) + 4 * hh + (r & 3)] = ds;
      }
      if (p.dbias) {
        // Dense-bias gradient: the heads' workgroups, and the sequences' for a shared bias, add into one matrix.
        // A lane's own 16 pairs lie in one row of it, so added from the accumulators one instruction would touch
        // 32 rows; read back from the wave's LDS by rows (its operations run in order), an instruction adds two
        // whole rows of the block: two cache lines instead of 32.
        float* dbp = p.dbias + (p.dense_bias_batched ? (int64_t)b * p.L * p.Lkv : 0) + (int64_t)r0 * p.Lkv + kv0;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int row = 2 * i + (lane >> 5), col = lane & 31;
          const float v = dsw[row * (GT + 1) + col];
          if (v != 0.f) atomicAdd(dbp + (int64_t)row * p.Lkv + col, v);      // zero wherever the pair is masked or outside
        }
      }
      if (want_pos) {
        // one sum per diagonal of the wave's 32 x 32 block (the wave's own LDS: its operations run in order)
        const int dd = lane - (GT - 1);          // key - query inside the block; lane 63 has none
        if (lane < 2 * GT - 1) {
          float sum = 0.f;
          for (int r = 0; r < GT; ++r) {
            const int c = r + dd;
            if (c >= 0 && c < GT) sum += dsw[r * (GT + 1) + c];
          }
          const int idx = (p.L - 1) + (kv0 - r0) + dd;
          if (sum != 0.f && idx >= 0 && idx < 2 * p.L - 1)
            atomicAdd(p.dpos + (int64_t)(p.pos_heads > 1 ? h : 0) * (2 * p.L - 1) + idx, sum);
        }
      }
      if constexpr (BP) general_dot_cols_bf16<NB>(o, Ktb + m * GENERAL_BF16_CHAN_PITCH + 8 * hh, GENERAL_BF16_CHAN_PITCH, sacc, nblk);
      else general_dot_cols<NB>(o, Kc + (4 * hh) * pc + m, pc, sacc, nblk);
    }
    if (want_ts) {
      __syncthreads();
      for (int e = tid; e <= p.ts_nb; e += 256)
        if (Hist[e] != 0.f) atomicAdd(p.dts + (int64_t)(p.ts_heads > 1 ? h : 0) * (p.ts_nb + 1) + e, Hist[e]);
    }
  }
  // dQ^T[channel 32x + 8g + 4hh + tt][query qi]; rows past the sequence are written as zeros
  if (qi < s.rows) {
    const bool live_row = qi < s.n_q;
#pragma unroll
    for (int x = 0; x < NB; ++x) {
      if (x < nblk) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int c = 32 * x + 8 * (r >> 2) + 4 * hh + (r & 3);
          if (c < dq) stf(dqp + (int64_t)qi * p.q_st + c, live_row ? o[x][r] * p.alpha : 0.f);
        }
      }
    }
  }
}

// dK and dV: one workgroup per 128 keys of one (sequence, head), 32 per wave, query rows streamed 32 at a time.
//   S = Q K^T, dP = dO V^T (A = Q / dO rows, B = the wave's K / V rows in registers), P and dS pointwise,
//   dV^T += dO^T P, dK^T += Q^T dS (A = dO / Q read across the channels, B = P / dS as they leave the pointwise part).
template <typename T, bool BP = false, bool TAB = true>
__global__ __launch_bounds__(256, 1) void hstu_bwd_dkv_mm(const Params p) {
  extern __shared__ __attribute__((aligned(16))) float gsm[];
  const int dq = p.d_qk, dv = p.d_v;
  const int dq4 = (dq + 3) & ~3, dv4 = (dv + 3) & ~3;
  const int pqr = general_pitch_qk(dq), pqc = general_pitch_v(dq), por = general_pitch_qk(dv), poc = general_pitch_v(dv);
  float* Qr = gsm;                         // [32][pqr] Q rows for S
  float* Qc = Qr + GT * pqr;               // [32][pqc] Q read across the channels for dK^T
  float* Or = Qc + GT * pqc;               // [32][por] dO rows for dP
  float* Oc = Or + GT * por;               // [32][poc] dO read across the channels for dV^T
  // (bf16 products: Q rows | Q transposed | dO rows | dO transposed, pitches in bytes)
  unsigned char* const smb = (unsigned char*)gsm;
  const int prq = general_bf16_row_pitch(dq), pro = general_bf16_row_pitch(dv);
  unsigned char* const Qrb = smb;
  unsigned char* const Qtb = Qrb + GT * prq;
  unsigned char* const Orb = Qtb + dq * GENERAL_BF16_CHAN_PITCH;
  unsigned char* const Otb = Orb + GT * pro;

  const int h = blockIdx.x, b = blockIdx.y, kt = blockIdx.z;
  const Seq s = seq_info(p, b, h);
  const int k0 = kt * 128;
  const int krows = p.jagged ? s.n_kv : p.Lkv;      // rows of dk / dv that exist
  if (k0 >= krows) return;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, m = lane & 31, hh = lane >> 5;
  const T* __restrict__ qp = (const T*)p.q + s.bq;
  const T* __restrict__ kp_ = (const T*)p.k + s.bk;
  const T* __restrict__ vp = (const T*)p.v + s.bv;
  const T* __restrict__ dop = (const T*)p.dout + s.bo;
  T* __restrict__ dkp = (T*)p.dk + s.bk;
  T* __restrict__ dvp = (T*)p.dv + s.bv;
  const int c0 = k0 + 32 * w, kj = c0 + m;          // the wave's first key, this lane's key
  constexpr uintptr_t VMASK = sizeof(T) * 4 - 1;
  const bool qfast = BP || !TAB || ((((uintptr_t)qp & VMASK) == 0) && (p.q_st & 3) == 0 && (dq & 3) == 0);
  const bool ofast = BP || !TAB || ((((uintptr_t)dop & VMASK) == 0) && (p.o_st & 3) == 0 && (dv & 3) == 0);

  constexpr int NB = 4;
  const int nbk = (dq + 31) >> 5, nbv = (dv + 31) >> 5;
  floatx16 ak[NB], av[NB];
#pragma unroll
  for (int x = 0; x < NB; ++x)
#pragma unroll
    for (int r = 0; r < 16; ++r) { ak[x][r] = 0.f; av[x][r] = 0.f; }

  if (k0 < s.n_kv) {
    float2 kf[BP ? 1 : 32], vf[BP ? 1 : 32];
    bf16x8 kb[BP ? 8 : 1], vb[BP ? 8 : 1];
    if constexpr (BP) {
      general_row_frag_bf16(kb, (const bf16_t*)(kp_ + (int64_t)kj * p.k_st), dq, kj < s.n_kv, hh);
      general_row_frag_bf16(vb, (const bf16_t*)(vp + (int64_t)kj * p.v_st), dv, kj < s.n_kv, hh);
    } else {
      general_row_frag(kf, kp_ + (int64_t)kj * p.k_st, dq, kj < s.n_kv, hh);
      general_row_frag(vf, vp + (int64_t)kj * p.v_st, dv, kj < s.n_kv, hh);
    }
    // query rows that can see these keys
    int q_begin = 0, q_end = s.n_q;
    if (p.causal) q_begin = k0;
    if (p.window >= 0 && k0 - p.window > q_begin) q_begin = k0 - p.window;
    if (p.window >= 0 && k0 + 128 + p.window < q_end) q_end = k0 + 128 + p.window;
    q_begin = (q_begin / GT) * GT;
    if (p.mask) {
      // the steps before the first and after the last row for which the mask keeps one of these keys are left out
      int t_lo = q_begin / GT, t_hi = (q_end + GT - 1) / GT;
      general_mask_live_steps<false>(p, b, k0, tid, t_lo, t_hi);
      q_begin = t_lo * GT > q_begin ? t_lo * GT : q_begin;
      q_end = t_hi * GT < q_end ? t_hi * GT : q_end;
    }
    GeneralTile<T, 4> qt_, ot_;
    if (q_begin < q_end) {
      qt_.fetch(qp, p.q_st, q_begin, s.n_q, dq, qfast, tid);
      ot_.fetch(dop, p.o_st, q_begin, s.n_q, dv, ofast, tid);
    }
    // the query rows this lane's key keeps: lo <= i <= hi
    int lo = p.causal ? kj : 0, hi = s.n_q - 1;
    if (p.window >= 0) {
      lo = kj - p.window > lo ? kj - p.window : lo;
      hi = kj + p.window < hi ? kj + p.window : hi;
    }
    if (kj >= s.n_kv) hi = -1;
    const bool by_seg = p.mask_mode == HSTU_MASK_SEGMENT;
    const bool tabled = TAB && (p.pos_tab != nullptr || p.ts_tab != nullptr);

    for (int i0 = q_begin; i0 < q_end; i0 += GT) {
      // nothing for a wave whose keys all lie behind these rows (causal) or outside the window
      bool live = c0 < s.n_kv;
      if (p.causal && c0 > i0 + 31) live = false;
      if (p.window >= 0 && (c0 > i0 + 31 + p.window || c0 + 31 + p.window < i0)) live = false;
      // an explicit mask: the bytes of the lane's 16 pairs, asked for ahead of the barriers
      uint32_t mw[4] = {~0u, ~0u, ~0u, ~0u};
      if (live && p.mask) general_mask_words_col(p, b, i0, kj, hh, mw);
      float db[16];
      if (live && p.dense_bias) general_dense_col(p, b, i0, kj, hh, db);
      __syncthreads();
      if constexpr (BP) {
        qt_.stage_bf16(i0, s.n_q, dq, tid, Qrb, prq, Qtb, GENERAL_BF16_CHAN_PITCH);
        ot_.stage_bf16(i0, s.n_q, dv, tid, Orb, pro, Otb, GENERAL_BF16_CHAN_PITCH);
      } else {
        qt_.stage(i0, s.n_q, dq, qfast, tid, Qr, pqr, Qc, pqc);
        ot_.stage(i0, s.n_q, dv, ofast, tid, Or, por, Oc, poc);
      }
      __syncthreads();
      if (i0 + GT < q_end) {
        qt_.fetch(qp, p.q_st, i0 + GT, s.n_q, dq, qfast, tid);
        ot_.fetch(dop, p.o_st, i0 + GT, s.n_q, dv, ofast, tid);
      }
      if (live && p.mask && __builtin_amdgcn_ballot_w64((mw[0] | mw[1] | mw[2] | mw[3]) != 0u) == 0) live = false;
      if (!live) continue;
      floatx16 sacc, dpacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) { sacc[r] = 0.f; dpacc[r] = 0.f; }
      if constexpr (BP) {
        general_dot_rows_bf16(sacc, Qrb + m * prq + 16 * hh, kb, dq);
        general_dot_rows_bf16(dpacc, Orb + m * pro + 16 * hh, vb, dv);
      } else {
        general_dot_rows(sacc, Qr + m * pqr + 2 * hh, kf, dq4);
        general_dot_rows(dpacc, Or + m * por + 2 * hh, vf, dv4);
      }
      // MFMA rows are the A operand's rows: lane holds pair (query i0 + 8g + 4hh + tt, key ... ) -- see below
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = i0 + 8 * (r >> 2) + 4 * hh + (r & 3);
        bool keep = i >= lo && i <= hi && ((mw[r >> 2] >> (8 * (r & 3))) & 0xffu) != 0u;
        if (by_seg) keep = keep && general_same_segment(p, b, i, kj);
        if (p.drop_thr) keep = keep && drop_keep(drop_bh_key(p.drop_key, (uint32_t)b * (uint32_t)p.H + (uint32_t)h), (uint32_t)i, (uint32_t)kj, p.drop_thr);
        float x = p.alpha * sacc[r];
        if (tabled && keep) x += general_table_bias(p, s, b, h, i, kj);
        if (p.dense_bias) x += db[r];
        const float sg = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-x * LOG2E));
        const float ds = keep ? dpacc[r] * sg * (1.0f + x * (1.0f - sg)) * p.inv_n : 0.f;
        sacc[r] = keep ? x * sg * p.inv_n : 0.f;    // P in place of S
        dpacc[r] = ds;                              // dS in place of dP
      }
      if constexpr (BP) {
        general_dot_cols_bf16<NB>(av, Otb + m * GENERAL_BF16_CHAN_PITCH + 8 * hh, GENERAL_BF16_CHAN_PITCH, sacc, nbv);
        general_dot_cols_bf16<NB>(ak, Qtb + m * GENERAL_BF16_CHAN_PITCH + 8 * hh, GENERAL_BF16_CHAN_PITCH, dpacc, nbk);
      } else {
        general_dot_cols<NB>(av, Oc + (4 * hh) * poc + m, poc, sacc, nbv);
        general_dot_cols<NB>(ak, Qc + (4 * hh) * pqc + m, pqc, dpacc, nbk);
      }
    }
  }
  if (kj < krows) {
    const bool live_row = kj < s.n_kv;
#pragma unroll
    for (int x = 0; x < NB; ++x) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 32 * x + 8 * (r >> 2) + 4 * hh + (r & 3);
        if (x < nbk && c < dq) stf(dkp + (int64_t)kj * p.k_st + c, live_row ? ak[x][r] * p.alpha : 0.f);
        if (x < nbv && c < dv) stf(dvp + (int64_t)kj * p.v_st + c, live_row ? av[x][r] : 0.f);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// MFMA kernel: bf16, causal/full + length masking, fused pos / timestamp bias.
//
// One workgroup = 4 wavefronts = 128 query rows (32 per wavefront); two
// workgroups per CU, i.e. two wavefronts per SIMD, so that one wavefront's
// MFMAs can run while the other's SiLU arithmetic does.  Keys are streamed 32
// at a time through a 4-stage LDS ring filled by direct global->LDS loads (no
// staging registers): at d = 128 two steps at a time, one pair ahead, with one
// barrier per pair (32-48 KB in flight per workgroup); with dense operands
// three steps ahead, one barrier per step; at d <= 64 a 3-stage ring, two ahead.
//
//   S^T[kv, q] = K Q^T   A = K fragment (LDS, 16-byte reads), B = Q (registers)
//   O^T[dv, q] = V^T P^T A = V fragment (LDS transpose reads), B = P (registers)
//
// The 32x32 fp32 accumulator of S^T leaves lane (q = lane%32, half = lane/32)
// holding keys 8g + 4*half + t (g, t in 0..3).  Read as the B operand of the
// second product, those 16 values are two 16-key chunks whose k-slot e of
// half h is key 16c + 8(e/4) + 4h + e%4 -- exactly what two 4-key transpose
// reads of row-major V deliver.  P therefore never leaves registers.
// ---------------------------------------------------------------------------

constexpr int BM = 128;       // query rows per workgroup (4 waves x 32)
constexpr int BN = 32;        // keys per step
constexpr int NSTAGE = 4;     // LDS ring depth
constexpr int MFMA_THREADS = 256;
constexpr int NWAVES = MFMA_THREADS / 64;
constexpr int POS_PAD = 256;  // zero margin on both sides of the scaled position table
constexpr int TS_TAB_LEN = 128;  // most timestamp buckets the matrix-core kernels index (the backward's histogram)
// Timestamp buckets without a logarithm.  The bucket law is floor(ln(f) / size) of f = fl32(clip(|dt|, 1, 1e9));
// it depends on dt only through the float f.  The key of f is its exponent and the top two bits of its
// mantissa (four keys per octave, 120 keys up to 1e9).  When size > ln(1.25) a key's range of floats holds
// at most one bucket boundary, so one entry per key {table value of the bucket the range starts in, first
// float of the next bucket} decides the value with a single comparison; the value from the threshold on
// is the next key's first field, so one 12-byte read brings all three -- exactly, boundaries included:
// the thresholds are computed on the host in double.  The general kernels evaluate the law in double and
// the CPU oracle is the same law, so all of them agree on every dt.
// One head's table (TS_LDS_BYTES, copied to LDS by every workgroup):
//   [(TS_KEYS + 2) x {float log2(e) * value, float threshold}]  by key (the per-pair path)
//   [TS_KEYS x float: log2(e) * value of bucket b]  by bucket (the backward's table-gradient path)
//   [TS_KEYS x int: smallest clipped |dt| of bucket b, INT32_MAX for buckets nothing reaches]  by bucket (the
//   per-tile shortcuts)
//   [TS_KEYS x byte: bucket the key's range starts in]  by key (the per-tile shortcuts, table gradients)
constexpr int TS_KEYS = 128;               // keys, and the most buckets the matrix-core kernels index
constexpr int TS_KEY0 = 127 << 2;          // key of f = 1.0 before the offset is taken off
constexpr int TS_DT_MAX = 1000000000;
constexpr int TS_VAL_OFF = (TS_KEYS + 2) * 8, TS_INT_OFF = TS_VAL_OFF + TS_KEYS * 4, TS_BKT_OFF = TS_INT_OFF + TS_KEYS * 4;
constexpr int TS_LDS_BYTES = TS_BKT_OFF + TS_KEYS;
static_assert(TS_LDS_BYTES % 16 == 0 && TS_LDS_BYTES <= 3 * 1024, "table layout: at most three direct loads");
struct TsKeys {                            // host-built part of the table, a kernel argument of hstu_prepare
  float thr_f[TS_KEYS];                    // by key: first float of the bucket behind the one the key's range starts in
  int32_t thr_b[TS_KEYS];                  // by bucket: smallest clipped |dt| in bucket b or a later one
  uint8_t bkt[TS_KEYS];                    // by key: bucket the key's range starts in
};


template <int D, int KB>   // KB: bytes per q / k element (2 = bf16, 1 = fp8)
struct MfmaSmem {
  // K and V tiles are stored unpadded ([32 keys][D]) because they arrive by direct
  // global->LDS loads, which write 64 lanes x 16 bytes contiguously.  Bank conflicts
  // are avoided by XOR-swizzling the 16-byte chunk index of a row instead (different
  // functions for K and V, matched to how each is read).
  static constexpr int CPR = D / 8;                       // 16-byte chunks per V row
  static constexpr int RPB = CPR >= 16 ? 1 : 16 / CPR;    // V rows per 256 bytes (one sweep of the banks)
  static constexpr int KCPR = D * KB / 16;                // the same for K
  static constexpr int KRPB = KCPR >= 16 ? 1 : 16 / KCPR;
  static constexpr int K_BYTES = BN * D * KB;
  static constexpr int V_BYTES = BN * D * 2;
  static constexpr int STAGE = K_BYTES + V_BYTES;
  static constexpr int POS_LANES = (BM + BN - 1 + 3 + 3) / 4;   // 16-byte pieces of one window copy
  static constexpr int POS_COPY = POS_LANES * 16;   // one shifted copy of the window
  static constexpr int POS_BYTES = 4 * POS_COPY;    // 4 copies shifted by 0..3 floats
  static constexpr int TK_LANES = BN / 4 + 1;       // 16-byte pieces: 32 int32 key timestamps, then (min, max, -, -)
  static constexpr int TK_BYTES = TK_LANES * 16;
  static constexpr int TAB_BYTES = TS_LDS_BYTES;         // the bucket table of the workgroup's head
  static constexpr int SEG_BYTES = BN * 4;           // the step's 32 int32 key segment ids
  static constexpr int bias_stage(bool pos, bool ts, bool seg = false) {
    return (pos ? POS_BYTES : 0) + (ts ? TK_BYTES : 0) + (seg ? SEG_BYTES : 0);
  }
  // dense operands of a step: the fp32 bias tile (128 rows x 32 keys) and the keep-mask tile (bytes)
  static constexpr int DB_BYTES = BM * BN * 4;
  static constexpr int DM_BYTES = BM * BN;
  static constexpr int dense_stage(int dense) { return ((dense & 1) ? DB_BYTES : 0) + ((dense & 2) ? DM_BYTES : 0); }
  // (the dense operands have one stage: each wave owns the rows of its 32 queries and refills them itself)
  static constexpr int total(bool pos, bool ts, bool seg = false, int dense = 0, int nst = NSTAGE) {
    return nst * (STAGE + bias_stage(pos, ts, seg)) + dense_stage(dense) + (ts ? TAB_BYTES : 0);
  }
  // K is read one row per lane, 16 bytes at a time: 16 consecutive rows must hit 16 different chunks
  __device__ static constexpr int swz_k(int row) { return (row / KRPB) % KCPR; }
  // V is read 4 rows x 64 bytes per half-wave: the 4 rows must land in 4 different 64-byte groups
  __device__ static constexpr int swz_v(int row) { return (4 * ((row / RPB) & 3)) % CPR; }
};

typedef __attribute__((address_space(3))) unsigned char* lds_byte_ptr;
// A pointer that is the same for every lane, taken from the first lane into scalar registers.
__device__ __forceinline__ const void* scalar_ptr(const void* p_) {
  const uint64_t v = (uint64_t)(uintptr_t)p_;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const void*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

// Direct global -> LDS loads, 64 lanes x 16 (or 4) bytes: lane l of the wave
// writes LDS bytes [lds_base + size*l, +size) with the bytes at gbase +
// byte_off(l).  Issued as inline assembly on purpose: the compiler then does
// not know that LDS is written (it would otherwise put a wait for ALL
// outstanding loads in front of every LDS read) nor that a load is in flight
// (so it never waits for these itself).  The kernel counts them by hand:
// every wave issues the same number per step and waits with s_waitcnt vmcnt(n)
// before the barrier that publishes a stage.
__device__ __forceinline__ void lds_dma16(const void* gbase_uniform, uint32_t byte_off, const void* lds_dst_wave_uniform) {
  // the low half of a flat pointer into LDS is the LDS address (no address-space cast: its null check
  // trips the compiler in some instantiations)
  const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds_dst_wave_uniform);
  // (the base pointer through scalar_ptr: a pointer the compiler does not see to be uniform would be handed over in
  // vector registers, which the instruction does not take)
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(base), "v"(byte_off), "s"(scalar_ptr(gbase_uniform))
               : "memory", "m0");
}
// The same with the destination given as an LDS byte address: the dynamic LDS array of a kernel
// starts where its static LDS ends (these kernels have none of the latter).
__device__ __forceinline__ void lds_dma16_at(const void* gbase_uniform, uint32_t byte_off, uint32_t lds_addr_wave_uniform) {
  const uint32_t base = __builtin_amdgcn_readfirstlane(lds_addr_wave_uniform);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(base), "v"(byte_off), "s"(scalar_ptr(gbase_uniform))
               : "memory", "m0");
}
__device__ __forceinline__ void lds_dma4(const void* gbase_uniform, uint32_t byte_off, const void* lds_dst_wave_uniform) {
  // the low half of a flat pointer into LDS is the LDS address (no address-space cast: its null check
  // trips the compiler in some instantiations)
  const uint32_t base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds_dst_wave_uniform);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :
               : "s"(base), "v"(byte_off), "s"(gbase_uniform)
               : "memory", "m0");
}

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  floatx2 f = {lo, hi};
  bf16x2 r = __builtin_convertvector(f, bf16x2);
  return __builtin_bit_cast(uint32_t, r);
}

// u = x * log2(e);  returns u * sigmoid(x) = u / (1 + 2^-u).  The caller folds
// the missing 1/log2(e) into the output scale.
__device__ __forceinline__ float silu_log2(float u) {
  float e = __builtin_amdgcn_exp2f(-u);
  return u * __builtin_amdgcn_rcpf(1.0f + e);
}

typedef short short4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v* lds_short4_ptr;

// 4 keys x 16 channels per 16-lane group, transposed on the way out of LDS:
// lane i of a group receives channel i of 4 consecutive keys.
__device__ __forceinline__ uint2 lds_read_tr(const bf16_t* p) {
  short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)p);
  return __builtin_bit_cast(uint2, v);
}

// vmcnt(n) with expcnt / lgkmcnt left alone (gfx9 encoding: vmcnt = bits 3:0 and 15:14)
#define HSTU_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt((((n) & 15) | ((((n) >> 4) & 3) << 14)) | 0x0F70)

constexpr int MAX_CHUNKS = 4;
constexpr int CTR_RESERVED = 16;     // counters in front of the arrival counters

// The dense keep-mask's presence table, behind the ranges in the workspace: for mask batch mb, query tile qt and key
// tile kt (128 keys) one byte whose bit i says that rows 32 i .. 32 i + 31 of the query tile keep a pair among the
// key tile's keys.  Written by hstu_prepare with the ranges; read by the dK/dV kernel, which walks query steps.
constexpr int MASK_PRES_MAX_KT = 256;      // key tiles the preparation's LDS has room for (beyond: the kernel looks itself)
__device__ __forceinline__ const uint8_t* mask_presence(const Params& p) {
  return (const uint8_t*)(p.mask_range + 2 * (int64_t)(p.mask_batched ? p.B : 1) * p.n_qtiles);
}

// Steps of a tile: keys [0, kv_end) in 32-key steps
__device__ __forceinline__ int tile_steps(const Params& p, const Seq& s, int q0) {
  int kv_end = s.n_kv;
  const int row_end = q0 + BM < s.n_q ? q0 + BM : s.n_q;
  if (p.causal) kv_end = row_end < kv_end ? row_end : kv_end;
  if (p.window >= 0 && row_end - 1 + p.window + 1 < kv_end) kv_end = row_end + p.window;   // |i - j| <= window
  return (kv_end + BN - 1) / BN;
}

// Which (sequence, head, query tile, chunk) a workgroup of the main kernels has.
// Workgroups are dealt round-robin to the 8 XCDs (blockIdx % 8), each with its own L2: every
// tile of one (sequence, head) goes to the same XCD, and tiles of a sequence are adjacent in
// launch order, the one with most keys first, so that the tiles running together stream the
// same K/V rows and share them through that L2.  (Calls with a dense mask or bias are dealt
// differently, see below.)  Returns false when there is nothing to do.
struct Work { int b, h, qt, chunk, n_chunks, pslot; Seq s; };
__device__ __forceinline__ void work_from_item(const Params& p, const int4& item, int h, Work& wk) {
  wk.b = item.x & 0x3fff; wk.pslot = (int)((uint32_t)item.x >> 14); wk.h = h;
  wk.qt = item.y & 0xffff; wk.chunk = (item.y >> 16) & 0xff; wk.n_chunks = (int)((uint32_t)item.y >> 24);
  wk.s = seq_from(p, wk.b, h, item.z, item.w);
}
__device__ __forceinline__ bool work_of_block(const Params& p, unsigned block, Work& wk) {
  const int xcd = block & 7, j = block >> 3;
  if (p.sched) {
    // from the work list: with H >= 8 head h runs on XCD h % 8, else 8 / H items share a round
    int it, h;
    if (p.mask || p.dense_bias) {
      // Dense operands are shared by the heads, not by the query tiles: the H workgroups of an item
      // are neighbours on one XCD (they start together and fetch the same mask / bias tiles, so all
      // but the first find them in that L2), and runs of n_qtiles items -- the tiles of one full
      // sequence, which share K and V -- stay on one XCD too, dealt round-robin over the eight.
      const int li = j / p.H, nq = p.n_qtiles;
      h = j - li * p.H;
      const int grp = li / nq;
      it = (grp * 8 + xcd) * nq + (li - grp * nq);
    }
    else if (p.H >= 8) { const int hx = p.H >> 3; it = j / hx; h = (j - it * hx) * 8 + xcd; }
    else          { const int r = 8 / p.H;   it = j * r + xcd / p.H; h = xcd % p.H; }
    // the item is read before the count is checked (the grid never reaches past the list's capacity):
    // both loads miss the cache, and one after the other they cost a workgroup twice the latency
    // (the dense mapping rounds its grid up to whole rounds of eight runs: indices past the capacity read item 0)
    const int it_ld = it < p.items_max ? it : 0;
    const int4 item = ((const int4*)(p.sched + 4))[it_ld];
    if (it >= p.sched[0]) return false;
    work_from_item(p, item, h, wk);
    return true;
  }
  // without a list: one entry per (sequence, head, query tile), tiles from the last one down, never split
  const int bhk = j / p.n_qtiles;
  const int qt = p.n_qtiles - 1 - (j - bhk * p.n_qtiles);
  const int bh = bhk * 8 + xcd;
  if (bh >= p.B * p.H) return false;
  wk.b = bh / p.H; wk.h = bh - wk.b * p.H; wk.qt = qt; wk.chunk = 0; wk.n_chunks = 1; wk.pslot = 0;
  wk.s = seq_info(p, wk.b, wk.h);
  return true;
}

// A 64-bit time difference clipped to [1, 1e9].
__device__ __forceinline__ int ts_clip64(int64_t d) {
  d = d < 0 ? -d : d;      // |INT64_MIN| stays negative and is clipped to 1; differences of real timestamps never get there
  d = d < 1 ? 1 : d;
  return (int)(d < TS_DT_MAX ? d : TS_DT_MAX);
}
// Lookup of a time difference in the head's table (in LDS): f = fl32(clip(|d|, 1, 1e9)), its key, and the
// key's {value below the threshold, threshold, value from the threshold on}.
struct TsLook { float f, lo, thr, hi; uint32_t key; };
__device__ __forceinline__ TsLook ts_look(const unsigned char* tab, int d) {
  TsLook l;
  l.f = __builtin_amdgcn_fmed3f(__builtin_fabsf((float)d), 1.0f, (float)TS_DT_MAX);
  l.key = (__builtin_bit_cast(uint32_t, l.f) >> 21) - (uint32_t)TS_KEY0;
  const float* e = (const float*)(tab + (l.key << 3));
  const float2 a = *(const float2*)e;
  l.lo = a.x;
  l.thr = a.y;
  l.hi = e[2];
  return l;
}
__device__ __forceinline__ float ts_value(const TsLook& l) { return l.f >= l.thr ? l.hi : l.lo; }
__device__ __forceinline__ int ts_bucket(const unsigned char* tab, const TsLook& l) { return (int)tab[TS_BKT_OFF + l.key] + (l.f >= l.thr ? 1 : 0); }
// The bucket alone (its value is then one more read, ts_bucket_value): fewer registers than ts_look,
// for the kernel that also needs the bucket's index.
__device__ __forceinline__ int ts_bucket_of(const unsigned char* tab, int d) {
  const float f = __builtin_amdgcn_fmed3f(__builtin_fabsf((float)d), 1.0f, (float)TS_DT_MAX);
  const uint32_t key = (__builtin_bit_cast(uint32_t, f) >> 21) - (uint32_t)TS_KEY0;
  return (int)tab[TS_BKT_OFF + key] + (f >= *(const float*)(tab + (key << 3) + 4) ? 1 : 0);
}
// A range of time differences [d_near, d_far], d_near <= d_far: the near end's bucket b and its table value
// by one lookup, then the integer thresholds of the next two buckets tell where the far end lies: `same`
// when it is still in b and d_near >= 0 (then so is every difference between them); `two` when it is in
// b or b + 1: differences >= thr are then in b + 1 (value v_far), the others in b.
struct TsEnds { int b_near, b_far, thr; float v_near, v_far; bool same, two; };
__device__ __forceinline__ TsEnds ts_ends(const unsigned char* tab, int d_near, int d_far) {
  const TsLook n = ts_look(tab, d_near);
  TsEnds r;
  r.b_near = ts_bucket(tab, n);
  r.v_near = ts_value(n);
  const int* next = (const int*)(tab + TS_INT_OFF) + r.b_near;
  const int t1 = next[1], t2 = next[2];          // first differences of buckets b + 1 and b + 2
  int far = d_far < 0 ? -d_far : d_far;
  far = far < 1 ? 1 : (far > TS_DT_MAX ? TS_DT_MAX : far);
  const bool sorted = d_near >= 0;
  r.same = sorted && far < t1;
  r.two = sorted && far < t2;
  r.b_far = far < t1 ? r.b_near : r.b_near + 1;
  r.thr = t1;
  r.v_far = *(const float*)(tab + TS_VAL_OFF + ((r.b_near + 1) << 2));
  return r;
}
__device__ __forceinline__ float ts_bucket_value(const unsigned char* tab, int b) { return *(const float*)(tab + TS_VAL_OFF + (b << 2)); }

// Where sequence b starts in the int32 timestamp copy and in the per-tile range table.
// Timestamps that follow the token axis are packed like it (tiles by an upper bound of
// the tiles before them); timestamps with a batch stride are [B][L].
__device__ __forceinline__ int64_t ts_rel_base(const Params& p, int b, int64_t tok0) {
  return p.ts_sb != 0 ? (int64_t)b * p.L : tok0;
}
__device__ __forceinline__ int64_t ts_range_slot0(const Params& p, int b, int64_t tok0) {
  return p.ts_sb != 0 ? (int64_t)b * ((p.L + BN - 1) / BN) : (tok0 >> 5) + b;
}

// ---------------------------------------------------------------------------
// Timestamp descriptors.  The bucket of a pair depends on the sequence's timestamps alone: not on the head, not
// on the layer.  With sorted timestamps the buckets of one row fall from key to key, and away from the diagonal
// a step of 32 keys holds one bucket or two for a row.  This kernel works that out once per batch: for every
// query row and every 32-key step below its 128-row tile's first row one 16-bit word
//   bits 0..6   bucket b of the step's last key the row keeps (the nearest in time)
//   bits 7..12  c: the step's first c keys are one bucket further (b + 1), the others in b (0: one bucket)
//   bit 15      neither holds (three buckets or more, timestamps out of order in the step, a key later than the
//               row's own time, buckets past the table): the kernel looks every pair of the block up
// laid out [step][row] (ts_desc_pitch rows per step; a sequence's rows start at ts_desc_row0), so that the 32
// rows of a wave are 64 contiguous bytes per step.  Rows past the sequence get 0.  The main kernel's blocks then
// read one word per lane instead of testing the tile's time range against the bucket thresholds, and the steps
// before a tile's first flagged one can run as the hand-scheduled stream (ts_tquads: per tile and chunk of
// TS_DESC_CHUNK steps the first flagged step of the chunk, or INT32_MAX).
// The work of extra workgroups of hstu_prepare's launch, one per (128-row tile slot, chunk of steps): it depends
// on nothing else that launch writes, and so hides behind the work list, which one workgroup builds.
// ---------------------------------------------------------------------------
constexpr int TS_DESC_MAX_L = 16384;      // longest sequence descriptors are built for (table size)
constexpr uint32_t TS_DESC_GENERAL = 0x8000u;
__device__ __host__ __forceinline__ int64_t ts_desc_row0(int jagged, int L, int b, int64_t tok0) {
  return jagged ? 8 * ((tok0 >> 3) + b) : (int64_t)b * ((L + 7) & ~7);
}
__device__ __host__ __forceinline__ int64_t ts_desc_tile0(int jagged, int n_qtiles, int b, int64_t tok0) {
  return jagged ? (tok0 >> 7) + b : (int64_t)b * n_qtiles;
}

constexpr int TS_DESC_CHUNK = 8;          // steps per workgroup of the descriptor build
__device__ __host__ __forceinline__ int ts_desc_chunks(int L) { return ((L + BN - 1) / BN + TS_DESC_CHUNK - 1) / TS_DESC_CHUNK; }
__device__ __forceinline__ void ts_desc_block(const Params& p, uint16_t* __restrict__ desc, int32_t* __restrict__ tgen,
                                              const int block, const int n_chunks, const TsKeys& keys) {
  // The rows' own times and the chunk's 256 key timestamps in LDS.
  __shared__ int64_t tq_l[BM], k_l[TS_DESC_CHUNK * BN];
  __shared__ float thr_f[TS_KEYS];
  __shared__ int32_t thr_b[TS_KEYS];
  __shared__ unsigned char bkt[TS_KEYS];
  __shared__ int sorted_to[TS_DESC_CHUNK];
  __shared__ int found_b, found_o0, found_o1, first_general;
  const int tid = threadIdx.x;
  const int64_t slot = block / n_chunks;
  const int chunk = block - (int)slot * n_chunks;
  int b, qt, o0 = 0, nraw = 0;
  if (p.jagged) {
    // the sequence whose tile slots hold this one: every thread tries the sequences tid, tid + 256, ...; the
    // slots of sequence b start at (its first token >> 7) + b, so exactly one sequence has
    // tile0(b) <= slot < tile0(b + 1), or none (a slot past the last sequence's).  The thread that finds it
    // hands its offsets on with it: one trip to memory for both.
    if (tid == 0) { found_b = -1; first_general = 0x7fffffff; }
    __syncthreads();
    for (int c = tid; c < p.B; c += 256) {
      const int f0 = p.seq_offsets[c], f1 = p.seq_offsets[c + 1];
      if (ts_desc_tile0(1, 0, c, f0) <= slot && slot < ts_desc_tile0(1, 0, c + 1, f1)) { found_b = c; found_o0 = f0; found_o1 = f1; }
    }
    __syncthreads();
    b = found_b;
    if (b < 0) return;
    o0 = found_o0;
    nraw = found_o1 - o0;
    qt = (int)(slot - ts_desc_tile0(1, 0, b, o0));
  } else {
    if (tid == 0) first_general = 0x7fffffff;
    b = (int)(slot / p.n_qtiles);
    qt = (int)(slot - (int64_t)b * p.n_qtiles);
    if (b >= p.B) return;
    seq_raw(p, b, o0, nraw);
  }
  const Seq s = seq_from(p, b, 0, o0, nraw);
  const int q0 = qt * BM;
  if (q0 >= s.rows) return;
  // The steps the stream can take: those whose 32 keys every row of the tile keeps (below the tile's first row and
  // whole inside the sequence).  The tile's diagonal steps go through the block code, which does not read these words.
  const int n_steps_tile = (q0 < s.n_kv ? q0 : s.n_kv) / BN;
  const int t0 = chunk * TS_DESC_CHUNK;
  if (t0 >= n_steps_tile) return;
  const int t1 = t0 + TS_DESC_CHUNK < n_steps_tile ? t0 + TS_DESC_CHUNK : n_steps_tile;
  const int64_t row0 = ts_desc_row0(p.jagged, p.L, b, s.tok0);
  // (the next sequence's first token: this one's plus its stored rows)
  const int64_t row_end = b + 1 < p.B ? ts_desc_row0(p.jagged, p.L, b + 1, p.jagged ? s.tok0 + s.rows : 0) : (int64_t)p.ts_desc_pitch;
  const int n_ts = s.n_ts;
  const int64_t* tsg = p.ts + s.ts0;
  if (tid < BM) {
    // the time a row takes: that of the next row (its own for the last)
    int iq = q0 + tid + 1;
    iq = iq < n_ts ? iq : n_ts - 1;
    tq_l[tid] = tsg[iq < 0 ? 0 : iq];
  }
#pragma unroll
  for (int e = 0; e < TS_DESC_CHUNK * BN / 256; ++e) {
    int j = t0 * BN + e * 256 + tid;
    j = j < n_ts ? j : n_ts - 1;
    k_l[e * 256 + tid] = (t0 * BN + e * 256 < (t1 * BN)) ? tsg[j < 0 ? 0 : j] : 0;
  }
  if (tid < TS_KEYS) {
    thr_f[tid] = keys.thr_f[tid];
    thr_b[tid] = tid <= p.ts_nb ? keys.thr_b[tid] : 0x7fffffff;
    bkt[tid] = keys.bkt[tid];
  }
  __syncthreads();
  {
    // up to which key of a step the timestamps are in order: every thread compares one neighbouring pair, a
    // wave's ballot covers two steps
    static_assert(TS_DESC_CHUNK * BN == 256, "one key per thread");
    const int l32 = tid & 31;
    const int j_last = (n_ts - 1) - t0 * BN;                 // the last timestamp there is, as an index into k_l
    const bool breaks = l32 < BN - 1 && tid + 1 <= j_last && k_l[tid + 1] < k_l[tid];
    const uint64_t mask = __builtin_amdgcn_ballot_w64(breaks);
    if (l32 == 0) {
      const uint32_t mine = (uint32_t)(mask >> (tid & 32));
      int e = mine ? __builtin_ctz(mine) : BN - 1;           // the step is in order up to its key e
      e = tid + e < j_last ? tid + e : j_last;
      sorted_to[tid >> 5] = e;
    }
  }
  __syncthreads();
  auto bucket = [&](int64_t d) {       // the bucket law on a difference >= 0, clipped to the table
    const int dc = d < 1 ? 1 : (d < TS_DT_MAX ? (int)d : TS_DT_MAX);
    const float f = (float)dc;
    const uint32_t key = (__builtin_bit_cast(uint32_t, f) >> 21) - (uint32_t)TS_KEY0;
    const int bk = (int)bkt[key] + (f >= thr_f[key] ? 1 : 0);
    return bk < p.ts_nb ? bk : p.ts_nb;
  };
  int my_general = 0x7fffffff;
  // A thread's four (row, step) pairs side by side and without branches: each is a chain of dependent LDS reads
  // (two bucket lookups, five steps of bisection), and one after the other they cost the workgroup four times
  // the chain's latency.  Indices of pairs that do not exist are clamped and their words are not written.
  constexpr int NIT = BM * TS_DESC_CHUNK / 256;
  const int n_idx = BM * (t1 - t0);
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    const int idx = tid + 256 * it;
    const bool on = idx < n_idx;
    const int r = idx & (BM - 1), tl = on ? idx >> 7 : 0, t = t0 + tl;
    const int i = q0 + r;
    const int j0 = t * BN;
    int j1 = j0 + BN - 1;
    j1 = j1 < s.n_kv - 1 ? j1 : s.n_kv - 1;
    j1 = j1 < i ? j1 : i;                // (the causal mask: later keys are masked whatever their bucket)
    const bool pair = on && i < s.n_q && j1 >= j0;
    const int l0 = tl * BN, l1 = pair ? j1 - t0 * BN : l0;     // the step's first key and the row's last, as indices into k_l
    const int64_t tq = tq_l[r];
    const int64_t k_first = k_l[l0], k_last = k_l[l1];
    const bool in_order = sorted_to[tl] >= l1 && tq >= k_last;
    const int bn = bucket(in_order ? tq - k_last : 0), bf = bucket(in_order ? tq - k_first : 0);
    const bool one = in_order && bf == bn && bn < TS_KEYS, two = in_order && bf == bn + 1 && bf < TS_KEYS;
    // keys in order: those with tq - ts >= thr, i.e. ts <= tq - thr, are the first c of the step
    const int64_t cut = tq - (int64_t)thr_b[bf < TS_KEYS ? bf : TS_KEYS - 1];
    int lo = l0, hi = l1;                // (when `two`) k[lo] <= cut < k[hi]: the first and last key are on different sides
#pragma unroll
    for (int step = 0; step < 5; ++step) {         // l1 - l0 <= 31
      const int mid = (lo + hi) >> 1;
      const bool more = hi - lo > 1, left = k_l[mid] <= cut;
      lo = more && left ? mid : lo;
      hi = more && !left ? mid : hi;
    }
    uint32_t word = one ? (uint32_t)bn : ((uint32_t)bn | ((uint32_t)(lo + 1 - l0) << 7));
    if (pair && !one && !two) {
      word = TS_DESC_GENERAL;
      my_general = t < my_general ? t : my_general;
    }
    word = pair ? word : 0u;
    // (a tile's last rows may lie past the sequence: those up to the next sequence's first row are this
    // workgroup's to clear, the rest are that sequence's own)
    if (on && row0 + i < row_end) desc[(int64_t)t * p.ts_desc_pitch + row0 + i] = (uint16_t)word;
  }
  // the chunk's first flagged step, INT32_MAX when it has none: a slot of its own per (tile, chunk), written every time
  if (my_general != 0x7fffffff) atomicMin(&first_general, my_general);
  __syncthreads();
  if (tid == 0) tgen[(ts_desc_tile0(p.jagged, p.n_qtiles, b, s.tok0) + qt) * n_chunks + chunk] = first_general;
}


// What the main kernel reads from the workspace, rebuilt by every call:
//  * the relative-position table scaled by log2(e) and zero-padded,
//    [heads][POS_PAD + 2L-1 + POS_PAD]; the margins make every window read in-bounds;
//  * the timestamp bucket tables (TsKeys above), [heads][TS_LDS_BYTES];
//  * per sequence whose timestamps span less than 2^31: the timestamps minus their minimum
//    as int32 (differences of two of them are then exact in 32 bits), and the (min, max)
//    of those in each 32-key tile.  One workgroup per sequence;
//  * with a dense keep-mask: per query tile the range of 32-key steps that hold a kept pair.
__global__ __launch_bounds__(256) void hstu_prepare(const Params p, float* __restrict__ pos_out, int4* __restrict__ tab_out,
                                                    int32_t* __restrict__ ok_out, int32_t* __restrict__ rel_out,
                                                    int32_t* __restrict__ range_out, int32_t* __restrict__ sched_out,
                                                    int32_t* __restrict__ mrange_out, uint16_t* __restrict__ desc_out,
                                                    int32_t* __restrict__ tgen_out, const int n_prep, const int desc_chunks,
                                                    const TsKeys keys) {
  // workgroups [0, n_prep): what this comment lists; those behind them: the timestamp descriptors
  if ((int)blockIdx.x >= n_prep) {
    ts_desc_block(p, desc_out, tgen_out, (int)blockIdx.x - n_prep, desc_chunks, keys);
    return;
  }
  const int tid = threadIdx.x;
  const int gtid = blockIdx.x * blockDim.x + tid, gsz = n_prep * blockDim.x;
  if (sched_out && (int)blockIdx.x == n_prep - 1) {
    // The work list, by the last of these workgroups (the host launches one more than the rest needs).
    // Sequences are taken longest first (batches of up to SEG sequences; larger ones in batch order,
    // SEG at a time): the tiles with most keys start first and short ones fill in behind them.  Within
    // a sequence the last query tile (most keys) comes first.  The tiles of the sequences at hand are
    // numbered in that order and dealt to the threads 256 at a time (a thread finds its tile's
    // sequence by bisection over the prefix sums of the tiles per sequence); prefix sums over the
    // threads tell each tile where its chunk slots and its items start.  Two passes: the steps of all
    // tiles (what decides which tiles are split), then the items.
    constexpr int SEG = 1024;
    __shared__ int wave_sums[4];
    __shared__ int keys[SEG], firsts[SEG], order[SEG], tbase[SEG + 1];
    const bool sorted = p.B <= SEG;
    int4* items = (int4*)(sched_out + 4);
    int walk_first = -1, walk_r = 0;      // memo of `walk` below: the first tile of the thread's run and its sequence
    // sum over the workgroup and exclusive prefix of this thread's value (all 256 threads take part)
    auto block_scan = [&](int v, int& total) {
      int inc = v;
#pragma unroll
      for (int d = 1; d < 64; d <<= 1) {
        const int a = __shfl_up(inc, d, 64);
        if ((tid & 63) >= d) inc += a;
      }
      __syncthreads();            // the previous scan's readers are done with wave_sums
      if ((tid & 63) == 63) wave_sums[tid >> 6] = inc;
      __syncthreads();
      int base = inc - v;
      total = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        base += i < (tid >> 6) ? wave_sums[i] : 0;
        total += wave_sums[i];
      }
      return base;
    };
    // rows with output, keys and rows of the tile space of a sequence of stored length nraw (as seq_from)
    auto dims = [&](int nraw, int& nq, int& nk, int& rows) {
      if (p.jagged) {
        const int n = nraw < 0 ? 0 : (nraw > p.L ? p.L : nraw);
        nq = n; nk = n; rows = n;
      } else {
        nq = p.L; nk = p.Lkv; rows = p.L;
        if (p.mask_mode == HSTU_MASK_LENGTH) {
          const int n = nraw < 0 ? 0 : nraw;
          nq = n < p.L ? n : p.L;
          nk = n < p.Lkv ? n : p.Lkv;
        }
      }
    };
    auto steps_of = [&](int nq, int nk, int q0) {       // as tile_steps
      if (q0 >= nq) return 0;
      int kv_end = nk;
      const int row_end = q0 + BM < nq ? q0 + BM : nq;
      if (p.causal) kv_end = row_end < kv_end ? row_end : kv_end;
      if (p.window >= 0 && row_end - 1 + p.window + 1 < kv_end) kv_end = row_end + p.window;
      return (kv_end + BN - 1) / BN;
    };
    // Sequences [s0, s0 + cnt) into LDS: stored lengths and first tokens, their order, the prefix sums of
    // their tiles.  Returns the number of tiles.
    auto load_segment = [&](int s0, int cnt) {
      __syncthreads();            // the readers of the segment before are done
      for (int i = tid; i < cnt; i += 256) {
        int o0, nraw;
        seq_raw(p, s0 + i, o0, nraw);
        keys[i] = nraw;
        firsts[i] = o0;
      }
      __syncthreads();
      // (the rank of a sequence: how many are longer, or as long and earlier.  A wave takes the lengths 64 at a
      // time, one per lane, and every lane compares its own with each of them from the lanes' registers: one
      // LDS read per 64 comparisons)
      for (int i0 = 0; i0 < cnt; i0 += 256) {
        const int i = i0 + tid;
        int rank = i;
        if (sorted) {
          const int kb = i < cnt ? keys[i] : 0;
          rank = 0;
          for (int c0 = 0; c0 < cnt; c0 += 64) {
            const int mine = c0 + (tid & 63) < cnt ? keys[c0 + (tid & 63)] : (int)0x80000000;   // (past the end: shorter than any)
#pragma unroll
            for (int j = 0; j < 64; ++j) {
              const int kc = __builtin_amdgcn_readlane(mine, j);
              rank += (kc > kb || (kc == kb && c0 + j < i)) ? 1 : 0;
            }
          }
        }
        if (i < cnt) order[rank] = i;
      }
      walk_first = -1;            // (the walks' memo of where a thread's run starts belongs to the segment before)
      __syncthreads();
      int c[SEG / 256], sum = 0;
#pragma unroll
      for (int k = 0; k < SEG / 256; ++k) {
        const int r = tid * (SEG / 256) + k;
        c[k] = 0;
        if (r < cnt) {
          int nq, nk, rows;
          dims(keys[order[r]], nq, nk, rows);
          c[k] = (rows + BM - 1) / BM;
        }
        sum += c[k];
      }
      int total;
      int base = block_scan(sum, total);
#pragma unroll
      for (int k = 0; k < SEG / 256; ++k) {
        const int r = tid * (SEG / 256) + k;
        if (r < cnt) tbase[r] = base;
        base += c[k];
      }
      if (tid == 0) tbase[cnt] = total;
      __syncthreads();
      return total;
    };
    // chunks of a tile of nt steps once the threshold is known: balanced parts of at most split_steps
    auto chunks_of = [&](int nt, int split_steps) {
      if (split_steps <= 0 || nt <= split_steps) return 1;
      const int c = (nt + split_steps - 1) / split_steps;
      return c < MAX_CHUNKS ? c : MAX_CHUNKS;
    };
    // A thread's run of the segment's tiles, [f_lo, f_hi): one bisection finds the first tile's sequence, the
    // rest follow in order.  fn(i, qt, nq, nk): index of the sequence within the segment, query tile, dimensions.
    auto walk = [&](int cnt, int f_lo, int f_hi, auto&& fn) {
      if (f_lo >= f_hi) return;
      // (a thread walks the same run several times over a segment: the bisection, a chain of dependent LDS reads,
      // is done for the first walk only)
      if (walk_first != f_lo) {
        int lo = 0, hi = cnt;     // the last r with tbase[r] <= f_lo (those before it with the same value have no tiles)
        while (hi - lo > 1) {
          const int mid = (lo + hi) >> 1;
          if (tbase[mid] <= f_lo) lo = mid; else hi = mid;
        }
        walk_first = f_lo;
        walk_r = lo;
      }
      int r = walk_r;
      for (int f = f_lo; f < f_hi;) {
        while (f >= tbase[r + 1]) ++r;
        const int i = order[r], t0 = tbase[r], t1 = tbase[r + 1];
        int nq, nk, rows;
        dims(keys[i], nq, nk, rows);
        const int last = f_hi < t1 ? f_hi : t1;
        for (; f < last; ++f) fn(i, (t1 - t0) - 1 - (f - t0), nq, nk);
      }
    };
    const int nseg = (p.B + SEG - 1) / SEG;
    int split_steps = 0, tiles = -1;
    if (p.split_cap > 0) {
      int steps = 0;
      for (int sg = 0; sg < nseg; ++sg) {
        const int cnt = p.B - sg * SEG < SEG ? p.B - sg * SEG : SEG;
        tiles = load_segment(sg * SEG, cnt);
        const int per = (tiles + 255) / 256;
        walk(cnt, tid * per < tiles ? tid * per : tiles, (tid + 1) * per < tiles ? (tid + 1) * per : tiles,
             [&](int, int qt, int nq, int nk) { steps += steps_of(nq, nk, qt * BM); });
      }
      int total;
      block_scan(steps, total);
      // steps one slot of an XCD gets on average: with H >= 8 an XCD runs H / 8 heads of every item,
      // else 8 / H XCDs share the items of one head
      const long long per_xcd = p.H >= 8 ? (long long)total * (p.H >> 3) : (long long)total / (8 / p.H);
      const long long avg = (per_xcd + p.n_slots - 1) / p.n_slots;
      // A tile is split when it alone is more than twice that average: its chunks cost a round trip of
      // fp32 partial sums through memory, so tiles near the average are left whole.  (Measured, kernel
      // time with the threshold at 1x / 1.5x / 2x the average / never: one sequence of 2048 tokens
      // 40 / 37 / 34 / 55 us; two 65 / 60 / 46 / 56; two long among 60 short 62 / 46 / 48 / 57; the
      // headline shape of 64 jagged sequences 72 / 68 / 69 / 69.)
      const long long thr = 2 * avg;
      split_steps = thr < 8 ? 8 : (thr > 0x3fffffff ? 0x3fffffff : (int)thr);
    }
    int item_base = 0, slot_base = 0;
    for (int sg = 0; sg < nseg; ++sg) {
      const int cnt = p.B - sg * SEG < SEG ? p.B - sg * SEG : SEG;
      if (nseg > 1 || tiles < 0) tiles = load_segment(sg * SEG, cnt);     // (a single segment is still there from the first pass)
      const int per = (tiles + 255) / 256;
      const int f_lo = tid * per < tiles ? tid * per : tiles, f_hi = (tid + 1) * per < tiles ? (tid + 1) * per : tiles;
      // the chunk slots this thread's tiles ask for, and where they start: a tile is split only while slots last
      int want = 0, asked = 0;
      if (split_steps > 0)
        walk(cnt, f_lo, f_hi, [&](int, int qt, int nq, int nk) {
          const int c = chunks_of(steps_of(nq, nk, qt * BM), split_steps);
          want += c > 1 ? c : 0;
        });
      const int slot0 = split_steps > 0 ? slot_base + block_scan(want, asked) : 0;
      // one walk shared by the count and the write
      auto emit = [&](int base, bool write) {
        int n = 0, slot = slot0;
        walk(cnt, f_lo, f_hi, [&](int i, int qt, int nq, int nk) {
          int c = chunks_of(steps_of(nq, nk, qt * BM), split_steps), ps = 0;
          if (c > 1) {
            ps = slot;
            slot += c;
            if (ps + c > p.split_cap) { c = 1; ps = 0; }      // the partial buffer is full: this tile stays whole
          }
          for (int k = 0; k < c; ++k, ++n)
            if (write && base + n < p.items_max)
              items[base + n] = int4{(sg * SEG + i) | (ps << 14), qt | (k << 16) | (c << 24), firsts[i], keys[i]};
        });
        return n;
      };
      int made;
      const int at = item_base + block_scan(emit(0, false), made);
      emit(at, true);
      slot_base += asked;
      item_base += made;
    }
    if (tid == 0) {
      sched_out[0] = item_base < p.items_max ? item_base : (int)p.items_max;
      sched_out[1] = split_steps;
    }
    // the arrival counters of the split tiles start at zero (their last arriver leaves them so again)
    if (p.ctr)
      for (int i = tid; i < CTR_RESERVED + p.split_cap * p.H; i += 256) p.ctr[i] = 0u;
  }
  if (tab_out) {
    // every head's bucket table: thresholds and buckets from the host, the table values times log2(e) with
    // bucket indices clipped to the table's last entry (the clip of the bucket law)
    for (int i = gtid; i < p.ts_heads * (TS_KEYS + 2); i += gsz) {
      const int hd = i / (TS_KEYS + 2), e = i - hd * (TS_KEYS + 2);
      unsigned char* out = (unsigned char*)tab_out + (int64_t)hd * (3 * 1024);
      const float* tab = p.ts_tab + (int64_t)hd * (p.ts_nb + 1);
      const int ek = e < TS_KEYS ? e : TS_KEYS - 1;      // the entries behind the last key repeat it
      const int bk = keys.bkt[ek];
      ((float2*)out)[e] = float2{tab[bk < p.ts_nb ? bk : p.ts_nb] * LOG2E, keys.thr_f[ek]};
      if (e < TS_KEYS) {
        ((float*)(out + TS_VAL_OFF))[e] = tab[e < p.ts_nb ? e : p.ts_nb] * LOG2E;
        ((int*)(out + TS_INT_OFF))[e] = e <= p.ts_nb ? keys.thr_b[e] : 0x7fffffff;    // buckets are clipped to ts_nb
        out[TS_BKT_OFF + e] = (unsigned char)bk;
      }
    }
  }
  if (pos_out) {
    const int len = 2 * p.L - 1;
    const int stride = len + 2 * POS_PAD;
    const int total = p.pos_heads * stride;
    for (int i = gtid; i < total; i += gsz) {
      const int hd = i / stride, j = i - hd * stride - POS_PAD;
      pos_out[i] = (j >= 0 && j < len) ? p.pos_tab[(int64_t)hd * len + j] * LOG2E : 0.f;
    }
  }
  if (mrange_out) {
    // The dense keep-mask, per query tile of 128 rows: the range of 32-key steps outside of which no pair
    // of the tile is kept (a causal or length mask handed over as a matrix keeps a prefix of the keys: the
    // main kernel then leaves the other steps out altogether, loads included).  One workgroup per tile, 16
    // bytes per lane and load, eight loads in flight; rows are whole 16-byte pieces (Lkv is a multiple of 16).
    __shared__ int mr_lo[4], mr_hi[4];
    __shared__ unsigned int kbits[MASK_PRES_MAX_KT];      // per key tile: which of the tile's four 32-row steps keep a pair there
    const int nb = p.mask_batched ? p.B : 1;
    const int ppr = p.Lkv / 16;
    const int n_kt = (p.Lkv + BM - 1) / BM;
    const bool pres_on = p.mask_pres && n_kt <= MASK_PRES_MAX_KT;
    uint8_t* pres = (uint8_t*)(mrange_out + 2 * (int64_t)nb * p.n_qtiles);
    for (int tile = blockIdx.x; tile < nb * p.n_qtiles; tile += n_prep) {
      const int b = tile / p.n_qtiles, qt = tile - b * p.n_qtiles;
      const int r0 = qt * BM;
      const int rows = p.L - r0 < BM ? p.L - r0 : BM;
      const uint4* mg = (const uint4*)(p.mask + ((int64_t)b * p.L + r0) * p.Lkv);
      const int n = rows * ppr;
      int lo = 0x7fffffff, hi = 0;
      if (pres_on) {
        for (int i = tid; i < n_kt; i += 256) kbits[i] = 0u;      // (a thread clears what it wrote out for the tile before)
        __syncthreads();
      }
      for (int i0 = 0; i0 < n; i0 += 8 * 256) {
        uint4 v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          const int i = i0 + 256 * k + tid;
          v[k] = i < n ? mg[i] : uint4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          if ((v[k].x | v[k].y | v[k].z | v[k].w) != 0u) {
            const int i = i0 + 256 * k + tid;
            const int row = i / ppr, piece = i - row * ppr;
            const int step = piece >> 1;
            lo = step < lo ? step : lo;
            hi = step + 1 > hi ? step + 1 : hi;
            if (pres_on) {
              // (looked at before it is set: once the tile's bits are up, which is soon for a mask with any density,
              // the atomics stop)
              const unsigned int bit = 1u << (row >> 5);
              if (!(kbits[piece >> 3] & bit)) atomicOr(&kbits[piece >> 3], bit);
            }
          }
        }
      }
#pragma unroll
      for (int d = 32; d >= 1; d >>= 1) {
        const int a = __shfl_xor(lo, d, 64), c = __shfl_xor(hi, d, 64);
        lo = a < lo ? a : lo;
        hi = c > hi ? c : hi;
      }
      __syncthreads();            // the readers of the tile before are done
      if ((tid & 63) == 0) { mr_lo[tid >> 6] = lo; mr_hi[tid >> 6] = hi; }
      __syncthreads();
      if (tid == 0) {
#pragma unroll
        for (int i = 1; i < 4; ++i) {
          lo = mr_lo[i] < lo ? mr_lo[i] : lo;
          hi = mr_hi[i] > hi ? mr_hi[i] : hi;
        }
        mrange_out[2 * tile] = hi > 0 ? lo : 0;
        mrange_out[2 * tile + 1] = hi;
      }
      // (every thread's atomics on kbits lie before the barriers above)
      if (pres_on)
        for (int i = tid; i < n_kt; i += 256) pres[(int64_t)tile * n_kt + i] = (uint8_t)kbits[i];
    }
  }
  if (!ok_out) return;
  static_assert(BN == 32, "one lane per key of a tile");
  __shared__ int64_t red_lo[4], red_hi[4];
  const int lane = tid & 63, wv = tid >> 6, l32 = tid & 31;
  for (int b = blockIdx.x; b < p.B; b += n_prep) {
    const Seq s = seq_info(p, b, 0);
    const int n = s.n_ts;
    if (n <= 0) {
      if (tid == 0) ok_out[b] = 0;
      continue;
    }
    const int64_t* ts = p.ts + s.ts0;
    // (eight loads in flight per thread: one memory round trip per 2048 timestamps instead of eight)
    int64_t lo_v = ts[0], hi_v = lo_v;
    for (int j0 = 0; j0 < n; j0 += 2048) {
      int64_t x[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int j = j0 + i * 256 + tid;
        x[i] = ts[j < n ? j : n - 1];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        lo_v = x[i] < lo_v ? x[i] : lo_v;
        hi_v = x[i] > hi_v ? x[i] : hi_v;
      }
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
      const int64_t a = __shfl_xor(lo_v, d, 64), c = __shfl_xor(hi_v, d, 64);
      lo_v = a < lo_v ? a : lo_v;
      hi_v = c > hi_v ? c : hi_v;
    }
    __syncthreads();   // the previous sequence's readers are done with red_*
    if (lane == 0) { red_lo[wv] = lo_v; red_hi[wv] = hi_v; }
    __syncthreads();
    for (int i = 0; i < 4; ++i) {
      lo_v = red_lo[i] < lo_v ? red_lo[i] : lo_v;
      hi_v = red_hi[i] > hi_v ? red_hi[i] : hi_v;
    }
    const bool ok = ((uint64_t)hi_v - (uint64_t)lo_v) < 0x7fffffffull;
    if (tid == 0) ok_out[b] = ok ? 1 : 0;
    if (!ok) continue;
    int32_t* rel = rel_out + ts_rel_base(p, b, s.tok0);
    int32_t* rng = range_out + 2 * ts_range_slot0(p, b, s.tok0);
    const int tiles = (n + BN - 1) / BN;
    for (int t0 = 0; t0 < tiles; t0 += 64) {      // one half-wave per tile, eight tiles in flight per half-wave
      int64_t x[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int j = (t0 + 8 * i + (tid >> 5)) * BN + l32;
        x[i] = ts[j < n ? j : n - 1];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int t = t0 + 8 * i + (tid >> 5);
        const int j = t * BN + l32;
        const int32_t r = (int32_t)(x[i] - lo_v);
        if (j < n) rel[j] = r;
        int32_t mn = r, mx = r;
#pragma unroll
        for (int d = 16; d >= 1; d >>= 1) {
          const int32_t a = __shfl_xor(mn, d, 32), c = __shfl_xor(mx, d, 32);
          mn = a < mn ? a : mn;
          mx = c > mx ? c : mx;
        }
        if (l32 == 0 && t < tiles) { rng[2 * t] = mn; rng[2 * t + 1] = mx; }
      }
    }
  }
}

// SEG: segment ids (padded layout, L a multiple of 4): a pair is kept when its row's and its key's
// ids are equal.  The step's 32 key ids arrive by one more direct load per wave and every block
// compares them with the lane's row id.
//
// DENSE (bit 0: additive bias, bit 1: keep-mask; the layer-side call of
// recml/layers/keras/hstu.py:356-390): the step's 128 x 32 tile of the [L, Lkv] fp32 bias and / or
// of the byte mask comes by direct loads like K and V (four per wave for the bias, one for the mask),
// but into a single 16 KB + 4 KB buffer instead of a ring: a wave reads only the 32 rows of its own
// queries, and the loads that bring those rows are its own, so each wave takes its part of step t into
// registers at the start of the step and at once asks for step t + 1 into the same bytes -- no other
// wave is involved, and the loads have the whole block and the barrier to land.  With a three-stage K / V
// ring that is 68 KB at d = 128: two workgroups per CU.  A block whose mask tile is all zero is skipped.
// Ring depth of the forward kernel.  Up to d = 64 a wave needs at most 128 registers, so four
// workgroups fit a CU once their LDS does: three stages (two steps in flight behind the one being
// computed) instead of four take the d = 64 kernel with a position table from 43 KB to 32 KB, three
// workgroups per CU to four (measured: 148 -> 139 us on the d = 64 benchmark shape).  At d = 128
// registers allow two workgroups whatever the ring, and the depth makes no measurable difference.
constexpr int fwd_stages(int d, int dense) { return (d <= 64 || dense != 0) ? 3 : 4; }
constexpr int FWD_XCH_BYTES = 16;     // behind everything else in the forward kernel's LDS
// which instances of the forward kernel are laid out for timestamp descriptors (64 bytes per wave and ring stage)
constexpr bool fwd_takes_ts_desc(int d, bool ts, bool f8, bool seg, int dense) { return ts && d == 128 && !f8 && !seg && dense == 0; }

#include "hstu_fwd_stream_d128.inc"   // (the variants' names; the statements are expanded inside the kernel)
#include "hstu_bwd_stream_d128.inc"

template <int D, bool POS, bool TS, bool F8, bool SEG = false, int DENSE = 0, bool PERSIST = false>
__global__ __launch_bounds__(MFMA_THREADS, 2) void hstu_fwd_mfma_bf16(const Params p) {
  constexpr int KB = F8 ? 1 : 2;       // bytes per q / k element
  using SM = MfmaSmem<D, KB>;
  constexpr int CPR = SM::CPR;
  constexpr int KCPR = SM::KCPR;
  constexpr int KSTEPS = D / 16;       // MFMA k-steps over the head dim
  constexpr int QCH = D * KB / 32;     // 16-byte chunks of a q (or k) row per lane: chunk 2j + hh, j < QCH
  constexpr int DVB = D / 32;          // 32-row blocks of O^T
  // 1 KB pieces (one wave-wide direct load each) in a K and in a V tile, and direct loads per wave per tile
  constexpr int NPIECE_K = SM::K_BYTES / 1024, NPIECE = SM::V_BYTES / 1024;
  constexpr int LDK = NPIECE_K >= NWAVES ? NPIECE_K / NWAVES : 1;
  constexpr int LD = NPIECE >= NWAVES ? NPIECE / NWAVES : 1;
  static_assert(SM::K_BYTES % 1024 == 0 && SM::V_BYTES % 1024 == 0, "tile must be a whole number of 1 KB pieces");
  constexpr int NSTAGE = fwd_stages(D, DENSE);   // the ring depth of this kernel (shadows the backward kernels' constant)
  static_assert(BM * BN * 4 / 1024 == 4 * NWAVES && BM * BN / 1024 == NWAVES, "dense tiles: 4 + 1 pieces per wave");
  // direct loads per wave per step
  constexpr int NDMA = LDK + LD + ((POS || TS) ? 1 : 0) + (SEG ? 1 : 0);
  constexpr int NDENSE = ((DENSE & 1) ? 4 : 0) + ((DENSE & 2) ? 1 : 0);     // the dense operands' loads, counted apart
  static_assert((NSTAGE - 1) * NDMA + NDENSE <= 63, "vmcnt range");
  static_assert(DENSE == 0 || (!POS && !TS && !SEG && !F8), "dense operands come without table biases, segment ids and fp8");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const uint32_t smem_lds = __builtin_amdgcn_groupstaticsize();   // LDS byte address of smem
  // LDS map: [ring: NSTAGE x (K | V)][bias operands x NSTAGE: 4 pos windows | key timestamps][ts table]
  // [dense operands: bias tile | mask tile].
  // The key timestamps sit right behind the last position window so that one direct load of the
  // last wave can fill both.
  auto Ks = [&](int st) { return (bf16_t*)(smem + st * SM::STAGE); };
  auto Vs = [&](int st) { return (bf16_t*)(smem + st * SM::STAGE + SM::K_BYTES); };
  constexpr int BIAS_OFF = NSTAGE * SM::STAGE;
  // TSD: the kernel can take timestamp descriptors (ts_desc_block in hstu_prepare).  The bias operands of a stage are then
  // [4 x (window copy w | the 32 descriptors of wave w's rows)][key timestamps]: each wave's one bias load brings
  // its window copy and, in the four lanes behind it, its own rows' descriptors.
  constexpr bool TSD = fwd_takes_ts_desc(D, TS, F8, SEG, DENSE);
  constexpr int DESC_WAVE = 64;                                      // 32 descriptors of 2 bytes
  constexpr int CS = TSD ? (POS ? SM::POS_COPY : 0) + DESC_WAVE : SM::POS_COPY;   // from one wave's copy to the next
  constexpr int BIAS_STAGE = SM::bias_stage(POS, TS, SEG) + (TSD ? NWAVES * DESC_WAVE : 0);
  auto Wc = [&](int st) { return (float*)(smem + BIAS_OFF + st * BIAS_STAGE); };
  auto Tk = [&](int st) { return (int32_t*)(smem + BIAS_OFF + st * BIAS_STAGE + (TSD ? NWAVES * CS : (POS ? SM::POS_BYTES : 0))); };
  auto Sg = [&](int st) { return (int32_t*)(smem + BIAS_OFF + st * BIAS_STAGE + SM::bias_stage(POS, TS)); };
  const unsigned char* TsKey = smem + BIAS_OFF + NSTAGE * BIAS_STAGE;   // the keyed bucket table of this head
  constexpr int DENSE_OFF = BIAS_OFF + NSTAGE * BIAS_STAGE + (TS ? SM::TAB_BYTES : 0);
  constexpr int DENSE_STAGE = SM::dense_stage(DENSE);
  constexpr int XCH_OFF = DENSE_OFF + DENSE_STAGE;   // 16 bytes for values one lane hands to the workgroup
  auto Db = [&]() { return smem + DENSE_OFF; };
  auto Dm = [&]() { return smem + DENSE_OFF + ((DENSE & 1) ? SM::DB_BYTES : 0); };

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave index, kept scalar
  const int m = lane & 31, hh = lane >> 5;
  constexpr bool PAIRS = NSTAGE == 4 && DENSE == 0;
  static_assert(!PERSIST || (PAIRS && !SEG && !F8), "the loop over items is built on the paired step loop");
  const int win = p.window;
  const uint32_t kst_bytes = (uint32_t)p.k_st * (uint32_t)KB, vst_bytes = (uint32_t)p.v_st * 2u;
  const char* wsb = (const char*)p.ws_base;
  uint32_t* xch = (uint32_t*)(smem + XCH_OFF);

  // What the direct loads of an item's steps need (everything here is the same for the whole workgroup).
  // What an item's set-up needs of the arguments.  A workgroup that stays reads them again from the kernel
  // argument segment at each item (scalar loads through a pointer the compiler cannot see through):
  // kept in scalar registers across the step loop they would not fit beside what the loop itself holds.
  auto fresh = [&]() -> Params {
    if constexpr (PERSIST) {
      typedef const __attribute__((address_space(4))) Params* KernArg;
      KernArg ka = (KernArg)__builtin_amdgcn_kernarg_segment_ptr();
      asm volatile("" : "+s"(ka));
      return *(const Params*)ka;
    } else {
      return p;
    }
  };
  struct DmaCtx { const char* kg; const bf16_t* vg; int n_kv, n_ts, q0, b; uint32_t pos_off, rel_off, rng_off, desc_off; };
  // Bias operands are fetched with 32-bit byte offsets from the start of the workspace.
  // pos_off: the head's padded table; entry x of the unpadded table sits at float POS_PAD + x.
  auto ctx_of = [&](const Work& k) {
    const Params pf = fresh();
    DmaCtx c;
    c.kg = (const char*)pf.k + k.s.bk * KB;
    c.vg = (const bf16_t*)pf.v + k.s.bv;
    c.n_kv = k.s.n_kv; c.n_ts = k.s.n_ts; c.q0 = k.qt * BM; c.b = k.b;
    c.pos_off = POS ? (uint32_t)((const char*)(pf.pos_scaled + (int64_t)(pf.pos_heads > 1 ? k.h : 0) * (2 * pf.L - 1 + 2 * POS_PAD)) - wsb) : 0u;
    c.rel_off = TS ? (uint32_t)((const char*)(pf.ts_rel + ts_rel_base(pf, k.b, k.s.tok0)) - wsb) : 0u;
    c.rng_off = TS ? (uint32_t)((const char*)(pf.ts_range + 2 * ts_range_slot0(pf, k.b, k.s.tok0)) - wsb) : 0u;
    // (descriptor of row i at step t: entry t * pitch + i from here; 0 = no descriptors)
    c.desc_off = (TSD && pf.ts_desc) ? (uint32_t)((const char*)(pf.ts_desc + ts_desc_row0(pf.jagged, pf.L, k.b, k.s.tok0)) - wsb) : 0u;
    if constexpr (PERSIST) {
      // (the same for every lane, and the direct loads want them in scalar registers: said outright, the
      // compiler otherwise moves the arithmetic of an item drawn at run time to the vector unit)
      c.kg = (const char*)scalar_ptr(c.kg);
      c.vg = (const bf16_t*)scalar_ptr(c.vg);
    }
    return c;
  };
  // The steps [t_lo, nt) an item covers: the whole tile, or balanced part `chunk` of n_chunks (a part can be
  // empty only if the list were inconsistent; such a workgroup still arrives at the tile's counter);
  // nothing for a tile of padding rows.  A sliding window (never combined with key-range splitting) also
  // drops the steps before the tile's first key.
  auto range_of = [&](const Work& k, int& t_lo_, int& nt_) {
    const Params pf = fresh();
    const int q0_ = k.qt * BM;
    t_lo_ = 0;
    nt_ = q0_ < k.s.n_q ? tile_steps(pf, k.s, q0_) : 0;
    if (k.n_chunks > 1) {
      const int per = (nt_ + k.n_chunks - 1) / k.n_chunks;
      t_lo_ = k.chunk * per;
      t_lo_ = t_lo_ < nt_ ? t_lo_ : nt_;
      nt_ = t_lo_ + per < nt_ ? t_lo_ + per : nt_;
    }
    if (win >= 0 && q0_ - win > 0 && nt_ > 0) t_lo_ = (q0_ - win) / BN;
    if constexpr ((DENSE & 2) != 0) {
      // the steps in which the keep-mask keeps a pair of this tile at all (found by the preparation kernel)
      const int2 mr = ((const int2*)pf.mask_range)[(pf.mask_batched ? k.b : 0) * pf.n_qtiles + k.qt];
      t_lo_ = t_lo_ > mr.x ? t_lo_ : mr.x;
      nt_ = nt_ < mr.y ? nt_ : mr.y;
      nt_ = nt_ > t_lo_ ? nt_ : t_lo_;
    }
  };

  // Direct loads of step t into ring stage t % NSTAGE.  Wave w fills 1 KB
  // pieces w*LD .. w*LD+LD-1 of K and of V; lane l of piece j lands at chunk
  // 64j + l, i.e. row (64j+l)/CPR, physical chunk (64j+l)%CPR, and fetches the
  // logical chunk that the swizzle maps there.  Rows past the sequence re-read
  // the last valid row (finite data; their logits are masked).  Every wave
  // issues the same number of loads per step: the vmcnt arithmetic relies on it.
  // The ring stage is a compile-time constant everywhere (the step loop is unrolled over the ring):
  // LDS addresses are then a per-lane register plus an immediate, with no address arithmetic per step.
  // What a lane of the step's one bias load per wave fetches: byte offset from the workspace base, and whether the
  // lane takes part.  Wave c writes position-window copy c: window[x + c], window[x] = pos[(L-1) + kv0 - (q0+127) + x];
  // the table index is >= POS_PAD - 127 > 0 and inside the padded table (the offset register is unsigned: a negative
  // index would address 4 GB past the base).  With descriptors the four lanes behind the window bring the wave's own
  // 32 rows of the step's descriptors.  The lanes behind those on the last wave (or the first lanes of every wave
  // when there is neither window nor descriptors) bring 32 int32 key timestamps, 4 per lane, and the tile's (min, max).
  // Keys past the sequence read whatever follows in the workspace: their logits are masked.
  auto bias_lane = [&](const DmaCtx& c_, int t, bool& on, int lane) -> uint32_t {
    constexpr int DESC_LANE0 = POS ? SM::POS_LANES : 0;
    constexpr int TS_LANE0 = DESC_LANE0 + (TSD ? DESC_WAVE / 16 : 0);
    const int kv0 = t * BN;
    const bool ts_wave = TS && ((!POS && !TSD) || w == NWAVES - 1);
    const int tl = lane - TS_LANE0;
    uint32_t off = 0;
    on = false;
    if (POS && lane < SM::POS_LANES) {
      off = c_.pos_off + (uint32_t)(POS_PAD + (p.L - 1) + kv0 - (c_.q0 + BM - 1) + w + 4 * lane) * 4u;
      on = true;
    }
    if (TSD && c_.desc_off != 0u && lane >= DESC_LANE0 && lane < TS_LANE0) {
      // the wave's own 32 rows of the step's descriptors: 8 rows per lane
      off = c_.desc_off + ((uint32_t)t * (uint32_t)p.ts_desc_pitch + (uint32_t)(c_.q0 + 32 * w + 8 * (lane - DESC_LANE0))) * 2u;
      on = true;
    }
    if (ts_wave && tl >= 0 && tl < SM::TK_LANES) {
      int tr = t;                                  // tiles past the last timestamp repeat the last tile's range
      const int tr_last = (c_.n_ts - 1) >> 5;
      tr = tr < tr_last ? tr : tr_last;
      off = tl < BN / 4 ? c_.rel_off + (uint32_t)(kv0 + 4 * tl) * 4u : c_.rng_off + (uint32_t)tr * 8u;
      on = true;
    }
    return off;
  };
  // `part_`: 3 = the whole step, 1 = its K tile and bias operands only, 2 = its V tile only (the hand-scheduled
  // stream of the interior steps keeps the K side of the ring one step ahead of the V side).
  auto dma_part = [&](const DmaCtx& c_, int t, auto st_, auto part_) {
    constexpr int st = decltype(st_)::value;
    constexpr int part = decltype(part_)::value;
    const int kv0 = t * BN;
    const int last = c_.n_kv - 1;
    if constexpr ((part & 1) != 0) {
#pragma unroll
    for (int r = 0; r < LDK; ++r) {
      const int j = (w * LDK + r) % NPIECE_K;   // small tiles: several waves repeat the same piece
      const int c = 64 * j + lane;
      const int row = c / KCPR, pc = c - row * KCPR;
      int grow = kv0 + row;
      grow = grow < last ? grow : last;
      const uint32_t koff = (uint32_t)grow * kst_bytes + (uint32_t)((pc ^ SM::swz_k(row)) * 16);
      lds_dma16(c_.kg, koff, (const unsigned char*)Ks(st) + j * 1024);
    }
    }
    if constexpr ((part & 2) != 0) {
#pragma unroll
    for (int r = 0; r < LD; ++r) {
      const int j = (w * LD + r) % NPIECE;
      const int c = 64 * j + lane;
      const int row = c / CPR, pc = c - row * CPR;
      int grow = kv0 + row;
      grow = grow < last ? grow : last;
      const uint32_t voff = (uint32_t)grow * vst_bytes + (uint32_t)((pc ^ SM::swz_v(row)) * 16);
      lds_dma16(c_.vg, voff, Vs(st) + j * 512);
    }
    }
    if ((POS || TS) && (part & 1) != 0) {
      // one more load per wave brings the bias operands (bias_lane)
      bool on;
      const uint32_t off = bias_lane(c_, t, on, lane);
      if (on) lds_dma16(wsb, off, (const unsigned char*)Wc(st) + ((POS || TSD) ? w * CS : 0));
    }
    if (SEG && (part & 1) != 0) {
      // every wave brings the same 32 ids (each wave must issue the same number of loads); groups of 4
      // past the row repeat the last group (L is a multiple of 4; those keys are masked by their index)
      if (lane < BN / 4) {
        int g4 = kv0 + 4 * lane;
        g4 = g4 < p.Lkv - 4 ? g4 : p.Lkv - 4;
        lds_dma16_at(p.kv_seg + (int64_t)c_.b * p.Lkv, (uint32_t)g4 * 4u, smem_lds + (uint32_t)((const unsigned char*)Sg(st) - smem));
      }
    }
  };
  auto dma_step = [&](const DmaCtx& c_, int t, auto st_) { dma_part(c_, t, st_, std::integral_constant<int, 3>{}); };
  // The dense operands of step t, each wave its own rows (the same number of loads whatever the step).
  auto dense_refill = [&](const DmaCtx& c_, int t) {
    const int kv0 = t * BN;
    if (DENSE & 1) {
      // Bias tile: row r of the tile at LDS byte 128 r, its 16-byte chunks XOR-swizzled by r & 7
      // (the wave reads one chunk per lane from 16 consecutive rows).  Wave w brings 1 KB pieces
      // 4w .. 4w+3 (8 rows each, the rows of its own queries); lane l of a piece lands at row l / 8,
      // physical chunk l % 8.  Rows past L and keys past Lkv re-read the last row / the last four keys:
      // finite data for logits that are masked by their index.
      const float* dbg = p.dense_bias + (p.dense_bias_batched ? (int64_t)c_.b * p.L * p.Lkv : 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int j = 4 * w + r;
        const int row = 8 * j + (lane >> 3), pc = lane & 7;
        int gr = c_.q0 + row;
        gr = gr < p.L - 1 ? gr : p.L - 1;
        int col = kv0 + 4 * (pc ^ (row & 7));
        col = col < p.Lkv - 4 ? col : p.Lkv - 4;
        lds_dma16(dbg, ((uint32_t)gr * (uint32_t)p.Lkv + (uint32_t)col) * 4u, Db() + j * 1024);
      }
    }
    if (DENSE & 2) {
      // Mask tile: row r at LDS byte 32 r; wave w brings its own 32 rows, two lanes per row.
      const uint8_t* mg = p.mask + (p.mask_batched ? (int64_t)c_.b * p.L * p.Lkv : 0);
      const int row = 32 * w + (lane >> 1);
      int gr = c_.q0 + row;
      gr = gr < p.L - 1 ? gr : p.L - 1;
      int col = kv0 + 16 * (lane & 1);
      col = col < p.Lkv - 16 ? col : p.Lkv - 16;
      lds_dma16(mg, (uint32_t)gr * (uint32_t)p.Lkv + (uint32_t)col, Dm() + w * 1024);
    }
  };
  // The lane's share of the dense operands that have landed: 16 bias values (keys 8g + 4hh .. +3 of its
  // row) and their 16 mask bytes.  The empty statement at the end makes the compiler wait for the values
  // here: once it is passed, the buffer may be refilled.
  float4 dbv[4];
  uint32_t mbits[4] = {0u, 0u, 0u, 0u};
  auto dense_take = [&]() {
    if (DENSE & 2) {
      const unsigned char* mrow = Dm() + (32 * w + m) * 32 + 4 * hh;
#pragma unroll
      for (int g = 0; g < 4; ++g) mbits[g] = *(const uint32_t*)(mrow + 8 * g);
      asm volatile("" : "+v"(mbits[0]), "+v"(mbits[1]), "+v"(mbits[2]), "+v"(mbits[3]));
    }
    if (DENSE & 1) {
      const int row = 32 * w + m;
      const unsigned char* brow = Db() + row * 128;
#pragma unroll
      for (int g = 0; g < 4; ++g) dbv[g] = *(const float4*)(brow + (((2 * g + hh) ^ (row & 7)) * 16));
#pragma unroll
      for (int g = 0; g < 4; ++g) asm volatile("" : "+v"(dbv[g].x), "+v"(dbv[g].y), "+v"(dbv[g].z), "+v"(dbv[g].w));
    }
  };


  // ---- the item at hand: the same for the whole workgroup except where a lane's row enters
  DmaCtx cx;
  struct { int n_q, n_kv, rows, n_ts; } s;       // of the item's sequence
  int h = 0, q0 = 0, r0 = 0, qrow = 0, wave_last = -1, nt = 0, t_lo = 0, n_chunks = 1, chunk = 0, pslot = 0, ts32 = 0;
  int has_desc = 0, desc_first = 0x7fffffff;   // descriptors at hand; per lane, a chunk's first step with a flagged row
  uint32_t drop_thr = 0u, drop_kbh = 0u;       // dropout: the threshold (0: off) and the item's (sequence, head) key
  float alpha2 = 0.f;
  const int64_t* tsg = nullptr;
  bf16_t* og = nullptr;
  auto begin_item = [&](const Work& k) {
    const Params pf = fresh();
    s.n_q = k.s.n_q; s.n_kv = k.s.n_kv; s.rows = k.s.rows; s.n_ts = k.s.n_ts;
    h = k.h; q0 = k.qt * BM; chunk = k.chunk; n_chunks = k.n_chunks; pslot = k.pslot;
    cx = ctx_of(k);
    range_of(k, t_lo, nt);
    r0 = q0 + 32 * w;                    // first query row of this wave
    qrow = r0 + m;                       // this lane's query row
    // last key this wave needs (under a window without the causal mask: the last key its last row sees)
    wave_last = pf.causal ? r0 + 31 : (win >= 0 ? r0 + 31 + win : s.n_kv - 1);
    wave_last = wave_last < s.n_kv - 1 ? wave_last : s.n_kv - 1;
    if (r0 >= s.n_q) wave_last = -1;
    // fp8 q and k carry per-head dequantisation scales: they multiply the logits
    alpha2 = pf.alpha * LOG2E * (F8 && pf.q_scale ? pf.q_scale[h] : 1.0f) * (F8 && pf.k_scale ? pf.k_scale[h] : 1.0f);
    tsg = TS ? pf.ts + k.s.ts0 : nullptr;
    // whether the sequence's int32 timestamps are valid (its time span allows them)
    ts32 = TS ? pf.ts_ok[k.b] : 0;
    if constexpr (TSD) {
      // (each lane takes one chunk's first flagged step, of the chunks that hold interior steps; the first lane
      // that has one holds the tile's: stream_quads reads it, behind the loads that go out in between)
      has_desc = pf.ts_desc != nullptr;
      const int interior = (q0 < s.n_kv ? q0 : s.n_kv) / BN;
      desc_first = 0x7fffffff;
      if (has_desc && lane * TS_DESC_CHUNK < interior)
        desc_first = pf.ts_tquads[(ts_desc_tile0(pf.jagged, pf.n_qtiles, k.b, k.s.tok0) + k.qt) * pf.ts_desc_chunks + lane];
    }
    og = (bf16_t*)pf.out + k.s.bo;
    drop_thr = pf.drop_thr;
    drop_kbh = drop_thr ? drop_bh_key(pf.drop_key, (uint32_t)k.b * (uint32_t)pf.H + (uint32_t)k.h) : 0u;
  };
  // the head's bucket table: three direct loads of up to 1 KB, one each by waves 0 to 2 (the last wave repeats the first)
  auto load_ts_table = [&](int head) {
    const Params pf = fresh();
    const int c = w < 3 ? w : 0;
    if (1024 * c + 16 * lane < TS_LDS_BYTES)
      lds_dma16((const unsigned char*)pf.ts_keyed + (int64_t)(pf.ts_heads > 1 ? head : 0) * (3 * 1024) + 1024 * c, (uint32_t)lane * 16u, TsKey + 1024 * c);
  };

  // Q fragments (B operand of S^T = K Q^T).  bf16: k-step ks of lane (row, hh) holds
  // q[qrow][16ks+8hh .. +7], i.e. 16-byte chunk 2ks+hh of the row.  fp8: the lane holds chunks
  // 2j+hh of the row, each feeding two k-steps (its low and its high 8 bytes); K is read the
  // same way, and the order of the terms of a dot product is free.  With them the lane's segment id
  // and the timestamp its row takes (that of the next row).
  uint4 qf[QCH];
  int32_t qseg = 0;
  int64_t tq = 0;
  int32_t tq32 = 0;
  auto load_q = [&](const Work& k) {
    const Params pf = fresh();
    // (the lane's index enters through a register the compiler cannot see through: it would otherwise
    // work the lane's share of every address out once, ahead of the loop over items, and keep it all in
    // registers that loop does not have; the same in finish_item)
    int m_ = m, hh_ = hh;
    if (PERSIST) asm volatile("" : "+v"(m_), "+v"(hh_));
    const int qr = k.qt * BM + 32 * w + m_;
    const char* qg = (const char*)pf.q + (k.s.bq + (int64_t)qr * pf.q_st) * KB + 16 * hh_;
#pragma unroll
    for (int ks = 0; ks < QCH; ++ks) {
      uint4 t4 = {0u, 0u, 0u, 0u};
      if (qr < k.s.n_q) t4 = *(const uint4*)(qg + 32 * ks);
      qf[ks] = t4;
    }
    if (SEG) qseg = pf.q_seg[(int64_t)k.b * pf.L + (qr < pf.L ? qr : pf.L - 1)];
    if (TS) {
      int iq = qr + 1 < k.s.n_ts ? qr + 1 : k.s.n_ts - 1;
      iq = iq < 0 ? 0 : iq;
      tq32 = (pf.ts_rel + ts_rel_base(pf, k.b, k.s.tok0))[iq];     // meaningless when the sequence has no int32 timestamps, and then unused
      tq = (pf.ts + k.s.ts0)[iq];
    }
  };
  // Use what load_q fetched so that the compiler's wait for those loads sits here.  Left to the first
  // use inside the loop it would be a vmcnt(0) on every step, which also waits for every direct
  // load in flight and serialises the whole ring.
  auto settle_q = [&]() {
#pragma unroll
    for (int ks = 0; ks < QCH; ++ks) asm volatile("" ::"v"(qf[ks].x), "v"(qf[ks].y), "v"(qf[ks].z), "v"(qf[ks].w));
    if (SEG) asm volatile("" ::"v"(qseg));
    if (TS) asm volatile("" ::"v"(tq), "v"(tq32));
  };

  floatx16 o[DVB];

  // K: lane (row m, half hh) reads logical chunk 2ks+hh of row m
  const int gk = SM::swz_k(m);
  // V: lane i of 16-lane group G addresses 8 bytes of row 4hh + i/4 (+ 8x + 16cc):
  // logical chunk 4dvb + 2(G&1) + (i&3)/2, byte half (i&3)&1
  const int gi = lane & 15;
  const int vrow = 4 * hh + (gi >> 2);
  const int gq = SM::swz_v(vrow) >> 2;          // the swizzle acts on the chunk's upper bits only
  const int vc2 = 2 * ((lane >> 4) & 1) + ((gi & 3) >> 1);

  // One 32-key block for this wave: logits, bias, SiLU, P.V.  Blocks that touch
  // the causal diagonal or the end of the sequence get their logits zeroed where
  // masked: silu(0) = 0 exactly, so nothing is needed after the activation and
  // interior blocks pay nothing.
  auto block = [&](int t, auto st_) {
    constexpr int st = decltype(st_)::value;
    const int kbs = t * BN;
    if (DENSE & 2) {
      // nothing to do when the wave's whole mask tile is 0
      if (__builtin_amdgcn_ballot_w64((mbits[0] | mbits[1] | mbits[2] | mbits[3]) != 0u) == 0) return;
    }
    floatx16 sacc;
    {
      uint4 kf[QCH];
      const unsigned char* kr = (const unsigned char*)Ks(st) + m * (D * KB);
#pragma unroll
      for (int ks = 0; ks < QCH; ++ks) kf[ks] = *(const uint4*)(kr + (((2 * ks + hh) ^ gk) * 16));
      const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (F8) {
#pragma unroll
        for (int ks = 0; ks < QCH; ++ks) {
          const long ka = (long)(((uint64_t)kf[ks].y << 32) | kf[ks].x), kb = (long)(((uint64_t)kf[ks].w << 32) | kf[ks].z);
          const long qa = (long)(((uint64_t)qf[ks].y << 32) | qf[ks].x), qb = (long)(((uint64_t)qf[ks].w << 32) | qf[ks].z);
          sacc = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(ka, qa, ks == 0 ? zero : sacc, 0, 0, 0);
          sacc = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(kb, qb, sacc, 0, 0, 0);
        }
      } else {
#pragma unroll
        for (int ks = 0; ks < QCH; ++ks)
          sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[ks]), __builtin_bit_cast(bf16x8, qf[ks]),
                                                         ks == 0 ? zero : sacc, 0, 0, 0);
      }
    }
    // V fragments, requested now so that they arrive while the SiLU runs
    uint4 vf[2][DVB];
    {
      const bf16_t* vr = Vs(st) + vrow * D + 4 * (gi & 1);
#pragma unroll
      for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int dvb = 0; dvb < DVB; ++dvb) {
          const int pch = (4 * ((dvb ^ gq) % (CPR / 4 > 0 ? CPR / 4 : 1)) + vc2) * 8;
          uint2 lo = lds_read_tr(vr + (16 * cc) * D + pch);
          uint2 hi = lds_read_tr(vr + (16 * cc + 8) * D + pch);
          vf[cc][dvb] = uint4{lo.x, lo.y, hi.x, hi.y};
        }
    }
    // lane holds S^T[kv = kbs + 8g + 4hh + tt][q = qrow], r = 4g + tt
    float u[16];
    if (POS) {
      const int xb = 4 * hh + (BM - 1) - 32 * w - m;
      const int sft = xb & 3;
      const float* wrow = (const float*)((const unsigned char*)Wc(st) + sft * CS) + (xb - sft);
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
      if constexpr (TSD) {
        // (the product rounded by itself, as the hand-scheduled stream has it: the compiler would otherwise fuse it
        // with the timestamp bias's addition below, and the two paths would differ in the last bit)
#pragma unroll
        for (int r = 0; r < 16; ++r) asm volatile("" : "+v"(u[r]));
      }
    }
    if (TS) {
      if (ts32) {
        const int32_t* tk = Tk(st);
        const int2 rg = *(const int2*)(tk + BN);
        // |tq - tk| grows as tk falls: when no key of the tile is later than tq and both ends of
        // the tile fall in the same bucket, so does everything between
        const TsEnds en = ts_ends(TsKey, tq32 - rg.y, tq32 - rg.x);
        if (__builtin_amdgcn_ballot_w64(!en.same) == 0) {
          const float add = en.v_near;
#pragma unroll
          for (int r = 0; r < 16; ++r) u[r] += add;
        } else if (__builtin_amdgcn_ballot_w64(!en.two) == 0) {
          // at most one bucket boundary inside the tile for every lane: a key is in the farther bucket
          // exactly when tq - tk >= thr, i.e. tk <= tq - thr (lanes whose ends share a bucket: add_far == add_near)
          const float add_near = en.v_near, add_far = en.v_far;
          const int cut = tq32 - en.thr;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int4 kk = *(const int4*)(tk + 8 * g + 4 * hh);
            u[4 * g + 0] += kk.x <= cut ? add_far : add_near;
            u[4 * g + 1] += kk.y <= cut ? add_far : add_near;
            u[4 * g + 2] += kk.z <= cut ? add_far : add_near;
            u[4 * g + 3] += kk.w <= cut ? add_far : add_near;
          }
        } else {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int4 kk = *(const int4*)(tk + 8 * g + 4 * hh);
            u[4 * g + 0] += ts_value(ts_look(TsKey, tq32 - kk.x));
            u[4 * g + 1] += ts_value(ts_look(TsKey, tq32 - kk.y));
            u[4 * g + 2] += ts_value(ts_look(TsKey, tq32 - kk.z));
            u[4 * g + 3] += ts_value(ts_look(TsKey, tq32 - kk.w));
          }
        }
      } else {
        // time span of the sequence beyond 31 bits: 64-bit differences of timestamps read
        // straight from memory (rare; correctness over speed)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
#pragma unroll
          for (int tt = 0; tt < 4; ++tt) {
            int j = kbs + 8 * g + 4 * hh + tt;
            j = j < s.n_ts ? j : s.n_ts - 1;
            u[4 * g + tt] += ts_value(ts_look(TsKey, ts_clip64(tq - tsg[j])));
          }
        }
      }
    }
    if (DENSE & 1) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float4 bv = dbv[g];
        u[4 * g + 0] = __builtin_fmaf(bv.x, LOG2E, u[4 * g + 0]);
        u[4 * g + 1] = __builtin_fmaf(bv.y, LOG2E, u[4 * g + 1]);
        u[4 * g + 2] = __builtin_fmaf(bv.z, LOG2E, u[4 * g + 2]);
        u[4 * g + 3] = __builtin_fmaf(bv.w, LOG2E, u[4 * g + 3]);
      }
    }
    if ((p.causal && kbs + 31 > r0) || (kbs + 32 > s.n_kv) || (win >= 0 && (r0 + 31 - kbs > win || kbs + 31 - r0 > win))) {
      // keys the lane's row keeps: lo <= kv <= hi; register r holds key kbs + 4hh + c(r), c(r) = 8 (r / 4) + r % 4,
      // so one comparison of a constant with a per-lane bound decides each logit
      int hi = p.causal ? qrow : (win >= 0 ? qrow + win : s.n_kv - 1);
      hi = hi < s.n_kv - 1 ? hi : s.n_kv - 1;
      const int hi_rel = hi - kbs - 4 * hh;
      if (win < 0) {
#pragma unroll
        for (int r = 0; r < 16; ++r) u[r] = (8 * (r >> 2) + (r & 3)) <= hi_rel ? u[r] : 0.f;
      } else {
        const int lo_rel = qrow - win - kbs - 4 * hh;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int c = 8 * (r >> 2) + (r & 3);
          u[r] = (c <= hi_rel && c >= lo_rel) ? u[r] : 0.f;
        }
      }
    }
    if (SEG) {
      const int32_t* sg = Sg(st);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int4 ks4 = *(const int4*)(sg + 8 * g + 4 * hh);
        u[4 * g + 0] = ks4.x == qseg ? u[4 * g + 0] : 0.f;
        u[4 * g + 1] = ks4.y == qseg ? u[4 * g + 1] : 0.f;
        u[4 * g + 2] = ks4.z == qseg ? u[4 * g + 2] : 0.f;
        u[4 * g + 3] = ks4.w == qseg ? u[4 * g + 3] : 0.f;
      }
    }
    if (DENSE & 2) {
#pragma unroll
      for (int r = 0; r < 16; ++r) u[r] = ((mbits[r >> 2] >> (8 * (r & 3))) & 0xffu) ? u[r] : 0.f;
    }
    if (drop_thr) {
      // dropout: a dropped pair is one more masked logit (the survivors' scale is in the output scale)
      drop_apply16(u, drop_kbh + (uint32_t)qrow * DROP_CI + (uint32_t)(kbs + 4 * hh) * DROP_CJ, DROP_CJ, drop_thr);
    }
    // SiLU and P V in two halves of 8 keys, each in four phases of 8 independent operations with the order
    // fixed by scheduling barriers: left to itself under register pressure, the compiler has run the 16
    // exp -> add -> rcp -> mul chains one after another through one register, each link waiting for the last
    // (the transcendental unit's latency 32 times per step).  The first half's matrix products run while the
    // second half's vector work is issued.
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
      uint4 pk;
      pk.x = pack_bf16(e[0], e[1]);
      pk.y = pack_bf16(e[2], e[3]);
      pk.z = pack_bf16(e[4], e[5]);
      pk.w = pack_bf16(e[6], e[7]);
      const bf16x8 pb = __builtin_bit_cast(bf16x8, pk);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int dvb = 0; dvb < DVB; ++dvb)
        o[dvb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf[cc][dvb]), pb, o[dvb], 0, 0, 0);
    }
  };

  // wait until this wave's loads of step `t` have landed, leaving younger steps in flight
  auto wait_step = [&](int t) {
    int younger = nt - 1 - t;                  // steps issued after t
    younger = younger > NSTAGE - 2 ? NSTAGE - 2 : younger;
    if (younger >= 2) HSTU_WAIT_VMCNT(2 * NDMA);
    else if (younger == 1) HSTU_WAIT_VMCNT(NDMA);
    else HSTU_WAIT_VMCNT(0);
  };
  const auto live = [&](int t) { return t * BN <= wave_last && (win < 0 || t * BN + 31 + win >= r0); };

  auto zero_o = [&]() {
#pragma unroll
    for (int i = 0; i < DVB; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[i][r] = 0.f;
  };

  // The end of an item: its rows (or its partial sums) leave the workgroup.  `ot_base`: LDS bytes free
  // for the waves' 32 x D staging tiles.
  auto finish_item = [&](int ot_base) {
    const Params pf = fresh();
    int tid_ = tid;
    if (PERSIST) asm volatile("" : "+v"(tid_));
    const int tid = tid_, lane = tid_ & 63, m = lane & 31, hh = lane >> 5;     // shadow the kernel's: see load_q
    const int qrow = r0 + m;
    if (q0 >= s.n_q) {
      // padded rows of the padded layout: exact zeros
      const int rows = (s.rows - q0) < BM ? (s.rows - q0) : BM;
      const uint4 z = {0u, 0u, 0u, 0u};
      for (int e = tid; e < rows * (D / 8); e += MFMA_THREADS) {
        int r = e / (D / 8), c = e - r * (D / 8);
        *(uint4*)(og + (int64_t)(q0 + r) * pf.o_st + c * 8) = z;
      }
      return;
    }
    // O^T[dv = 32 dvb + 8g + 4hh + t][q = qrow]; rows past the sequence are 0.
    // The 1/log2(e) left out of the SiLU is folded into the output scale.
    if (n_chunks > 1) {
      // This workgroup covered part of the tile's keys.  It leaves its fp32 partial O^T (register order:
      // 8-byte piece (16 w + i) * 128 + 2 lane + j of the chunk's slot) in the workspace and counts itself
      // in at the tile's arrival counter; the workgroup that arrives last adds the others' partials to
      // its own, always in the order of the chunks, and writes the rows.  Partials and counter go by
      // device-scope atomic stores, loads and adds (which bypass the caches that are not coherent across
      // the chip).  The order is the memory model's: every wave's stores, then the workgroup barrier, then
      // thread 0's count as a release-acquire add at device scope (the barrier makes the other waves' stores
      // part of what it releases); the last arriver's count reads the others' releases, its barrier hands
      // that on to its other waves, and each of them takes an acquire fence before it loads.  (The wait for
      // the stores' acknowledgement stays: it costs nothing once the release is there.)  Nothing depends on
      // which workgroup runs where, and the result does not depend on the order of arrival.
      constexpr int NPC = BM * D / 2;      // 8-byte pieces of a chunk's partial
      uint64_t* slot0 = (uint64_t*)pf.partial + ((int64_t)pslot * pf.H + h) * NPC;
      uint64_t* mine = slot0 + (int64_t)chunk * pf.H * NPC + (w * (DVB * 4)) * 128 + 2 * lane;
#pragma unroll
      for (int i = 0; i < DVB * 4; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          // (through named floats: a bit cast applied to a vector element directly reads element 0)
          const float f0 = o[i >> 2][4 * (i & 3) + 2 * j], f1 = o[i >> 2][4 * (i & 3) + 2 * j + 1];
          const uint64_t bits = (uint64_t)__builtin_bit_cast(uint32_t, f0) | ((uint64_t)__builtin_bit_cast(uint32_t, f1) << 32);
          __hip_atomic_store(mine + i * 128 + j, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
      HSTU_WAIT_VMCNT(0);                  // every store of this wave has been acknowledged
      __syncthreads();
      uint32_t* arrive = pf.ctr + CTR_RESERVED + pslot * pf.H + h;
      if (tid == 0) xch[0] = __hip_atomic_fetch_add(arrive, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
      __syncthreads();
      const uint32_t before = xch[0];
      if (before != (uint32_t)(n_chunks - 1)) return;
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
      if (tid == 0) __hip_atomic_store(arrive, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next call
      // (a chunk's pieces are asked for 16 at a time per lane and added once they are there: two round trips
      // per chunk instead of one per piece)
      auto add_chunk = [&](int c, floatx16 (&dst)[DVB]) {
        const uint64_t* src = slot0 + (int64_t)c * pf.H * NPC + (w * (DVB * 4)) * 128 + 2 * lane;
#pragma unroll
        for (int i0 = 0; i0 < DVB * 4; i0 += 8) {       // 16 pieces at a time
          uint64_t bits[16];
#pragma unroll
          for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
              bits[2 * i + j] = __hip_atomic_load(src + (i0 + i) * 128 + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
          for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const int ii = i0 + i;
              dst[ii >> 2][4 * (ii & 3) + 2 * j] += __builtin_bit_cast(float, (uint32_t)bits[2 * i + j]);
              dst[ii >> 2][4 * (ii & 3) + 2 * j + 1] += __builtin_bit_cast(float, (uint32_t)(bits[2 * i + j] >> 32));
            }
        }
      };
      // (its own partial comes back from the workspace like the others: one code path, no second accumulator)
      zero_o();
      for (int c = 0; c < n_chunks; ++c) add_chunk(c, o);
    }
    // Each wave turns its O^T fragment into whole output rows through LDS (those stages of the ring are
    // free: the loop ended on a barrier and no load into them is in flight), so that global memory sees
    // 16-byte stores that cover full rows instead of 8-byte pieces: lane (row m, half hh) writes 8 bytes
    // of row m at a time, 16-byte chunks XOR-swizzled by row against bank conflicts, then reads 16 bytes
    // per lane, 64 / (D/8) rows per instruction.  Only lanes of the same wave exchange data here and
    // LDS executes a wave's operations in order: no barrier is needed.
    const float oscale = pf.inv_n * (1.0f / LOG2E);
    unsigned char* ot = smem + ot_base + w * (32 * D * 2);
    auto oswz = [](int row) { return (row / SM::RPB) % CPR; };
    {
      const bool live_row = qrow < s.n_q;
      unsigned char* orow = ot + m * (D * 2) + 8 * hh;
#pragma unroll
      for (int dvb = 0; dvb < DVB; ++dvb) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          uint2 pko = {0u, 0u};
          if (live_row) {
            pko.x = pack_bf16(o[dvb][4 * g + 0] * oscale, o[dvb][4 * g + 1] * oscale);
            pko.y = pack_bf16(o[dvb][4 * g + 2] * oscale, o[dvb][4 * g + 3] * oscale);
          }
          *(uint2*)(orow + (((4 * dvb + g) ^ oswz(m)) * 16)) = pko;
        }
      }
    }
    constexpr int ROWS_PER_STORE = 64 / CPR;
    const int rr = lane / CPR, cc = lane - rr * CPR;
#pragma unroll
    for (int r0s = 0; r0s < 32; r0s += ROWS_PER_STORE) {
      const int row = r0s + rr;
      const uint4 val = *(const uint4*)(ot + row * (D * 2) + ((cc ^ oswz(row)) * 16));
      const int grow = r0 + row;
      if (grow < s.rows) {
        // streaming store: the output is not read again by this kernel, and K / V rows that other tiles of the
        // sequence still need are worth more of the L2 than it is (d = 64 benchmark shape: 134 -> 122 us)
        typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
        const uintx4 vv = {val.x, val.y, val.z, val.w};
        __builtin_nontemporal_store(vv, (uintx4*)(og + (int64_t)grow * pf.o_st + cc * 8));
      }
    }
  };
  // ---- The interior steps as one hand-scheduled instruction stream (d = 128 in bf16, no segment ids or dense
  // operands; hstu_fwd_stream_d128.inc, written by gen_fwd_stream.py).  With timestamps it takes each (row, step)'s
  // bias from the descriptors that hstu_prepare wrote (the bucket of the step's nearest key and how many of
  // its keys are one bucket further), and only the leading steps in which no row of the tile is flagged.  A step is interior when every key
  // of it is kept for every row of the tile: under the causal mask the steps below the tile's first row, without
  // it those that lie whole inside the sequence.  The stream takes them four at a time from the item's first step
  // on (ring stage 0), software-pipelined across steps, with the K side of the ring one step ahead of the V side.
  // It starts where a pair of the loops below would start (the first two steps' tiles in the ring and published,
  // nothing else in flight) and sends for the K side of the third step itself; on exit, n quads later, the tiles of
  // the next two steps are in the ring and published (and the K side of the one after), so the paired loop takes
  // over where the stream stops.  The stream's last pair asks for K tiles up to two steps past its end and for V
  // tiles up to one: those steps must exist and lie whole inside the sequence (no row to clamp).  The arithmetic
  // and its order are those of `block`: the same bits either way.
  // (Not in the resident-workgroup instances with timestamps: what those keep across their loop over items and
  // what the stream clobbers do not fit the register file together, and the compiler's spills cost the block code
  // more than the stream gains.  Calls with timestamp descriptors take one workgroup per item instead.)
  constexpr bool STREAM = D == 128 && !F8 && !SEG && DENSE == 0 && PAIRS && !(TS && PERSIST);
  auto stream_quads = [&]() -> int {
    if constexpr (!STREAM) return 0;
    const Params pf = fresh();
    if (pf.no_stream || win >= 0) return 0;
    int keys = s.n_kv;
    if (pf.causal) keys = q0 < keys ? q0 : keys;
    const int t_int = keys / BN;                 // steps [0, t_int) are interior for all four waves
    int n = (t_int - t_lo) >> 2;
    if constexpr (TS) {
      // with timestamps: only on descriptors, and only the leading steps in which no row of the tile is flagged
      if (!ts32 || !has_desc) return 0;
      const uint64_t flagged = __builtin_amdgcn_ballot_w64(desc_first != 0x7fffffff);
      const int first = flagged ? __builtin_amdgcn_readlane(desc_first, (int)__builtin_ctzll(flagged)) : 0x7fffffff;
      const int nd = (first >> 2) - (t_lo >> 2);
      n = (t_lo & 3) != 0 ? 0 : (n < nd ? n : nd);
    }
    // lookahead: steps up to t_lo + 4n + 2 exist and are whole
    const int whole = s.n_kv / BN;
    while (n > 0 && !(t_lo + 4 * n + 2 < nt && t_lo + 4 * n + 3 <= whole)) --n;
    return n > 0 ? n : 0;
  };
  auto run_stream = [&](int n_quads) {
    if constexpr (STREAM) {
      // (the lane's index enters through a register the compiler cannot see through: it would otherwise work the
      // lane's share of the stream's two dozen addresses out once, ahead of the loop over items, and keep them in
      // registers the block code needs)
      int tid_ = tid;
      asm volatile("" : "+v"(tid_));
      const int lane = tid_ & 63, m = lane & 31, hh = lane >> 5;
      const int gk = SM::swz_k(m), gi = lane & 15, vrow = 4 * hh + (gi >> 2), gq = SM::swz_v(vrow) >> 2;
      const int vc2 = 2 * ((lane >> 4) & 1) + ((gi & 3) >> 1);
      typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
      uintx4 hs_q[8];
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) hs_q[ks] = uintx4{qf[ks].x, qf[ks].y, qf[ks].z, qf[ks].w};
      uint32_t hs_ka[8], hs_va[4];
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) hs_ka[ks] = smem_lds + (uint32_t)(m * 256 + (((2 * ks + hh) ^ gk) * 16));
#pragma unroll
      for (int d = 0; d < 4; ++d) hs_va[d] = smem_lds + (uint32_t)(SM::K_BYTES + vrow * 256 + 8 * (gi & 1) + vc2 * 16 + ((d ^ gq) & 3) * 64);
      const int xb = 4 * hh + (BM - 1) - 32 * w - m, sft = xb & 3;
      const uint32_t hs_pa = smem_lds + (uint32_t)(BIAS_OFF + sft * CS + (xb - sft) * 4);
      uint32_t hs_koff[2], hs_voff[2];
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int c = 64 * (2 * w + r) + lane, row = c / 16, pc = c - row * 16;
        hs_koff[r] = (uint32_t)row * kst_bytes + (uint32_t)((pc ^ SM::swz_k(row)) * 16);
        hs_voff[r] = (uint32_t)row * vst_bytes + (uint32_t)((pc ^ SM::swz_v(row)) * 16);
      }
      const uint32_t hs_kdst = __builtin_amdgcn_readfirstlane(smem_lds + (uint32_t)(2 * w * 1024));
      const uint32_t hs_vdst = __builtin_amdgcn_readfirstlane(smem_lds + (uint32_t)(SM::K_BYTES + 2 * w * 1024));
      const uint32_t hs_kstep = (uint32_t)BN * kst_bytes, hs_vstep = (uint32_t)BN * vst_bytes;
      const char* hs_kp = cx.kg + (size_t)(t_lo + 2) * hs_kstep;
      const char* hs_vp = (const char*)cx.vg + (size_t)(t_lo + 2) * hs_vstep;
      const uint32_t hs_bdst = __builtin_amdgcn_readfirstlane(smem_lds + (uint32_t)(BIAS_OFF + w * CS));
      // the bias load: without timestamps one scalar pointer walks along the table, 128 bytes a step; with them
      // window, descriptors and key timestamps move on by different strides, so each lane's offset from the
      // workspace base takes a per-lane step (the differences of two steps' offsets)
      uint32_t hs_boff = (uint32_t)(w + 4 * lane) * 4u, hs_binc = 0u;
      uint64_t hs_bexec = (1ull << SM::POS_LANES) - 1ull;
      // the window of step t starts at table entry POS_PAD + (L - 1) + 32 t - (q0 + 127) of the head's padded table
      const char* hs_bp = wsb + cx.pos_off + (int64_t)(POS_PAD + (fresh().L - 1) + BN * (t_lo + 2) - (q0 + BM - 1)) * 4;
      uint32_t hs_dsa = 0u, hs_hh4 = 0u, hs_tva = 0u;
      if constexpr (TS) {
        bool on2, on3;
        const uint32_t o2 = bias_lane(cx, t_lo + 2, on2, lane), o3 = bias_lane(cx, t_lo + 3, on3, lane);
        hs_boff = o2;
        hs_binc = o3 - o2;
        hs_bexec = __builtin_amdgcn_ballot_w64(on2);
        hs_bp = wsb;
        hs_dsa = smem_lds + (uint32_t)(BIAS_OFF + w * CS + (POS ? SM::POS_COPY : 0) + 2 * m);
        hs_hh4 = (uint32_t)(4 * hh);
        hs_tva = __builtin_amdgcn_readfirstlane(smem_lds + (uint32_t)(BIAS_OFF + NSTAGE * BIAS_STAGE + TS_VAL_OFF));
      }
      const float hs_alpha = alpha2;
      int hs_n = n_quads;
      floatx16 (&hs_o)[DVB] = o;
      if (wave_last < 0) {
        // a wave whose 32 rows lie past the sequence's end: its share of the loads and every barrier, nothing else
        if constexpr (POS && TS) {
#define HSTU_STREAM_VARIANT HSTU_STREAM_LOADS_ONLY_POS_TS
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
        } else if constexpr (TS) {
#define HSTU_STREAM_VARIANT HSTU_STREAM_LOADS_ONLY_TS
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
        } else if constexpr (POS) {
#define HSTU_STREAM_VARIANT HSTU_STREAM_LOADS_ONLY_POS
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
        } else {
#define HSTU_STREAM_VARIANT HSTU_STREAM_LOADS_ONLY
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
        }
      } else if constexpr (POS && TS) {
#define HSTU_STREAM_VARIANT HSTU_STREAM_FULL_POS_TS
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
      } else if constexpr (TS) {
#define HSTU_STREAM_VARIANT HSTU_STREAM_FULL_TS
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
      } else if constexpr (POS) {
#define HSTU_STREAM_VARIANT HSTU_STREAM_FULL_POS
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
      } else {
#define HSTU_STREAM_VARIANT HSTU_STREAM_FULL
#include "hstu_fwd_stream_d128.inc"
#undef HSTU_STREAM_VARIANT
      }
      (void)hs_pa; (void)hs_bdst; (void)hs_boff; (void)hs_binc; (void)hs_bexec; (void)hs_bp; (void)hs_dsa; (void)hs_hh4; (void)hs_tva;
    }
  };
  if constexpr (!PERSIST) {
    // ---- one item per workgroup
    Work first;
    if (!work_of_block(p, blockIdx.x, first)) return;
    if (first.qt * BM >= first.s.rows) return;
    begin_item(first);
    if (q0 >= s.n_q) {
      if (chunk == 0) finish_item(0);
      return;
    }
    // prologue: the bucket table, then the first steps in flight before the first block (two when the
    // loop runs in pairs, else NSTAGE - 1).  The first step's tiles go out alone; the rest of the
    // prologue follows behind the Q fragments, whose wait covers every load issued before it: behind
    // all of the prologue it held up the first block until everything had landed.
    if (TS) load_ts_table(h);
    if (t_lo < nt) dma_step(cx, t_lo, std::integral_constant<int, 0>{});
    if (DENSE != 0 && t_lo < nt) dense_refill(cx, t_lo);
    load_q(first);
    settle_q();
    if (t_lo + 1 < nt) dma_step(cx, t_lo + 1, std::integral_constant<int, 1>{});
    if constexpr (NSTAGE > 3 && !PAIRS) {
      if (t_lo + 2 < nt) dma_step(cx, t_lo + 2, std::integral_constant<int, 2>{});
    }
    const int n_quads = stream_quads();
    zero_o();
    if constexpr (PAIRS) {
      // Steps in pairs, one barrier per pair.  The barrier that ended the pair (t-2, t-1) freed that
      // pair's two ring stages, which now receive steps t+2 and t+3; the blocks of steps t and t+1
      // are computed; then every wave makes sure that its share of the next pair has landed.  Between
      // two barriers the waves of a workgroup drift apart by up to two blocks, which the diagonal
      // tiles (where wave i has i+1 blocks to do) and the direct loads' issue stalls both use.
      // (With a four-stage ring and no dense operands only: d = 128 68.8 -> 64.9 us on the headline
      // shape; dense operands bring five to ten more loads per step and lose by pairs, 490 -> 556 us,
      // and so does a fourth stage bought for them at d <= 64, 110 -> 116 us.)
      HSTU_WAIT_VMCNT(0);
      __syncthreads();
      if (n_quads > 0) run_stream(n_quads);
      auto pair = [&](int t, auto st_) {
        constexpr int st = decltype(st_)::value;
        if (t + 2 < nt) dma_step(cx, t + 2, std::integral_constant<int, (st + 2) % NSTAGE>{});
        if (t + 3 < nt) dma_step(cx, t + 3, std::integral_constant<int, (st + 3) % NSTAGE>{});
        if (live(t)) block(t, st_);
        if (t + 1 < nt && live(t + 1)) block(t + 1, std::integral_constant<int, (st + 1) % NSTAGE>{});
        HSTU_WAIT_VMCNT(0);
        __syncthreads();
      };
      for (int t = t_lo + 4 * n_quads; t < nt; t += NSTAGE) {
        pair(t, std::integral_constant<int, 0>{});
        if (t + 2 >= nt) break;
        pair(t + 2, std::integral_constant<int, 2>{});
      }
    } else if constexpr (DENSE != 0) {
      // Step t with dense operands: the wave takes its rows of the step's bias and mask tiles into registers,
      // asks for the next step's into the same bytes, then for the K / V tiles of step t + 2 (into the ring
      // stage that the barrier before freed), and computes its block.  Before the barrier, everything of
      // step t + 1 has landed: the loads are counted in the order of their issue, so only the K / V tiles of
      // step t + 2, the youngest, stay in flight.
      static_assert(NSTAGE == 3, "two steps of K / V tiles in flight");
      if (t_lo + 1 < nt) HSTU_WAIT_VMCNT(NDMA); else HSTU_WAIT_VMCNT(0);      // all of step t_lo
      __syncthreads();
      auto step = [&](int t, auto st_) {
        constexpr int st = decltype(st_)::value;
        const bool lv = live(t);
        if (lv) dense_take();
        if (t + 1 < nt) dense_refill(cx, t + 1);
        if (t + 2 < nt) dma_step(cx, t + 2, std::integral_constant<int, (st + 2) % NSTAGE>{});
        if (lv) block(t, st_);
        if (t + 2 < nt) HSTU_WAIT_VMCNT(NDMA); else HSTU_WAIT_VMCNT(0);
        __syncthreads();
      };
      for (int t = t_lo; t < nt; t += NSTAGE) {
        step(t, std::integral_constant<int, 0>{});
        if (t + 1 >= nt) break;
        step(t + 1, std::integral_constant<int, 1>{});
        if (t + 2 >= nt) break;
        step(t + 2, std::integral_constant<int, 2>{});
      }
    } else {
      wait_step(t_lo);
      __syncthreads();
      // Step t: the barrier that ended step t-1 freed the ring stage of step t-1,
      // which now receives step t+NSTAGE-1; the block of step t is computed; then every
      // wave makes sure its share of step t+1 has landed before the next barrier.
      auto step = [&](int t, auto st_) {
        constexpr int st = decltype(st_)::value;
        if (t + NSTAGE - 1 < nt) dma_step(cx, t + NSTAGE - 1, std::integral_constant<int, (st + NSTAGE - 1) % NSTAGE>{});
        if (live(t)) block(t, st_);
        if (t + 1 < nt) wait_step(t + 1);
        __syncthreads();
      };
      for (int t = t_lo; t < nt; t += NSTAGE) {
        step(t, std::integral_constant<int, 0>{});
        if (t + 1 >= nt) break;
        step(t + 1, std::integral_constant<int, 1>{});
        if (t + 2 >= nt) break;
        step(t + 2, std::integral_constant<int, 2>{});
        if constexpr (NSTAGE > 3) {
          if (t + 3 >= nt) break;
          step(t + 3, std::integral_constant<int, 3>{});
        }
      }
    }
    finish_item(0);
  } else {
    // ---- a workgroup that stays: it takes item after item of its XCD's part of the work list.  Job j of
    // an XCD is (item, head) as in work_of_block; a workgroup's first job is j = slot, every later one is
    // drawn from the XCD's counter (the list is in order of falling work, so whoever is free takes the
    // longest job left).  The draw is made late, when at most two pairs of steps of the item at hand are
    // left: a job drawn early would wait for a workgroup that may still be busy for long while others
    // run dry.  While an item's last pair of steps is computed, the next item's first pair of tiles is
    // already on its way into the two ring stages that pair does not use, and its Q rows follow as soon
    // as the last logits are done: the latencies of an item's start hide behind the item before it.
    const int xcd = blockIdx.x & 7, slots = gridDim.x >> 3;
    const int n_items = p.sched[0];
    const int4* items = (const int4*)(p.sched + 4);
    auto job_item = [&](int job, int& head) {
      const int H = fresh().H;
      int it;
      if (H >= 8) { const int hx = H >> 3; it = job / hx; head = (job - it * hx) * 8 + xcd; }
      else        { const int r = 8 / H;   it = job * r + xcd / H; head = xcd % H; }
      return it;
    };
    int head_now = 0;
    int it_now = job_item(blockIdx.x >> 3, head_now);
    bool have = it_now < n_items;
    if (have) {
      Work first;
      work_from_item(p, items[it_now], head_now, first);
      begin_item(first);
      if (TS) load_ts_table(h);
      if (t_lo < nt) dma_step(cx, t_lo, std::integral_constant<int, 0>{});
      load_q(first);
      settle_q();
      if (t_lo + 1 < nt) dma_step(cx, t_lo + 1, std::integral_constant<int, 1>{});
    }
    while (have) {
      zero_o();
      HSTU_WAIT_VMCNT(0);                  // the item's first pair of tiles, its Q rows, the stores of the item before
      __syncthreads();
      // the item's interior steps, four at a time, as the hand-scheduled stream; the loop below takes the rest
      const int n_quads = stream_quads();
      if (n_quads > 0) run_stream(n_quads);
      const int t_first = t_lo + 4 * n_quads;
      // the next item: known from the draw on
      bool have_next = false, drew = false;
      int head_next = 0;
      int4 entry = {0, 0, 0, 0};
      // The next item's scalars are worked out from its list entry each time they are needed (its first
      // tiles, its Q rows, its turn): kept across the last pair they would not fit the scalar registers.
      auto prefetch_next = [&]() {
        Work k;
        work_from_item(fresh(), entry, head_next, k);
        const DmaCtx ncx = ctx_of(k);
        int n_tlo, n_nt;
        range_of(k, n_tlo, n_nt);
        if (n_tlo < n_nt) dma_step(ncx, n_tlo, std::integral_constant<int, 0>{});
        if (n_tlo + 1 < n_nt) dma_step(ncx, n_tlo + 1, std::integral_constant<int, 1>{});
      };
      // Every item starts at ring stage 0 (the stage is a compile-time constant everywhere; a stage picked at
      // run time costs the block code 60 registers).  Its steps go in pairs through stages (0, 1) and (2, 3) in
      // turn, an even number of pairs: with an odd number of real ones the last pair at (2, 3) has no steps.
      // That last pair is where the next item's first tiles are sent for (into stages (0, 1), free since the
      // barrier before it) and, once the last logits are done, its Q rows; it ends without waiting for
      // them: the item's rows are written while they arrive.
      for (int t = t_first;; t += 4) {
        // stages (0, 1)
        const bool draw = !drew && t + 8 >= nt;
        if (t + 2 < nt) dma_step(cx, t + 2, std::integral_constant<int, 2>{});
        if (t + 3 < nt) dma_step(cx, t + 3, std::integral_constant<int, 3>{});
        uint32_t drawn = 0u;
        if (draw && tid == 0) drawn = __hip_atomic_fetch_add(p.ctr + xcd, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (t < nt && live(t)) block(t, std::integral_constant<int, 0>{});
        if (t + 1 < nt && live(t + 1)) block(t + 1, std::integral_constant<int, 1>{});
        HSTU_WAIT_VMCNT(0);
        if (draw && tid == 0) xch[1] = drawn;
        __syncthreads();
        // stages (2, 3)
        if (draw) {
          drew = true;
          const int job_next = slots + __builtin_amdgcn_readfirstlane((int)xch[1]);
          const int it_next = job_item(job_next, head_next);
          have_next = it_next < n_items;
          if (have_next) {
            // (a scalar load by hand: this kernel also writes memory, so the compiler would fetch the entry
            // once per lane into vector registers)
            typedef int intx4 __attribute__((ext_vector_type(4)));
            intx4 e4;
            asm volatile("s_load_dwordx4 %0, %1, 0x0\n\ts_waitcnt lgkmcnt(0)" : "=s"(e4) : "s"(items + it_next));
            entry.x = e4.x; entry.y = e4.y; entry.z = e4.z; entry.w = e4.w;
          }
        }
        const bool last = t + 4 >= nt;
        if (!last) {
          dma_step(cx, t + 4, std::integral_constant<int, 0>{});
          if (t + 5 < nt) dma_step(cx, t + 5, std::integral_constant<int, 1>{});
        } else if (have_next) {
          prefetch_next();
        }
        if (t + 2 < nt && live(t + 2)) block(t + 2, std::integral_constant<int, 2>{});
        if (t + 3 < nt && live(t + 3)) block(t + 3, std::integral_constant<int, 3>{});
        if (last && have_next) {             // the Q registers are free: this item's last logits are done
          Work k;
          work_from_item(fresh(), entry, head_next, k);
          load_q(k);
        }
        if (!last) HSTU_WAIT_VMCNT(0);
        __syncthreads();
        if (last) break;
      }
      // stages (2, 3) are free now (the next item's tiles are landing in (0, 1)): they take the waves' staging tiles
      finish_item(2 * SM::STAGE);
      have = have_next;
      if (have) {
        const int head_before = h;
        Work k;
        work_from_item(fresh(), entry, head_next, k);
        begin_item(k);
        settle_q();
        if (TS && h != head_before) load_ts_table(h);
      }
    }
    // the last workgroup out leaves the draw counters at zero for the next launch
    if (tid == 0) {
      const uint32_t done = __hip_atomic_fetch_add(p.ctr + 8, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (done == gridDim.x - 1) {
        for (int i = 0; i < 9; ++i) __hip_atomic_store(p.ctr + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Backward on the matrix cores: bf16, d in {32, 64, 128}, the options of the MFMA forward.
//
// Two kernels, each recomputing the logits (recml/core/ops/hstu_ops.py:461-517):
//
//   hstu_bwd_dq_mfma   one workgroup per 128 query rows, keys streamed as in the forward:
//     S^T = K Q^T, dP^T = V dO^T, dS^T = dP^T f'(S^T), dQ^T += K^T dS^T
//   hstu_bwd_dkv_mfma  one workgroup per 128 keys, query rows streamed 32 at a time:
//     S = Q K^T, dP = dO V^T, dV^T += dO^T P, dK^T += Q^T dS
//
// with f'(x) = sigma(x) (1 + x (1 - sigma(x))); the factors alpha and 1/N are applied to the
// accumulators at the end.  In both, the operand that stays (Q and dO rows of the wave; K and V
// rows of the wave) is held in registers as the B operand, the streamed tiles are the A operand:
// read by rows for the first two products and through transpose reads for the last.  A streamed
// tile is therefore read both ways, and one swizzle serves both: 16-byte chunk c of row r sits at
// chunk c ^ swz_rt<D>(r), which spreads 16 consecutive rows over the 16 chunk slots of a 256-byte
// sweep of the banks (row reads) and 4 consecutive rows over 4 different 64-byte groups (transpose
// reads).  P and dS are rounded to bf16 for the last products like P in the forward.  Neither
// kernel splits its streamed range.  The table gradients, when wanted, come from the dQ kernel,
// which sees every pair once.  Sliding window and segment ids as in the forward.
// ---------------------------------------------------------------------------

constexpr float LN2 = 0.6931471805599453f;

template <int D>
__device__ __forceinline__ constexpr int swz_rt(int row) {
  // rows of 256 / 128 / 64 bytes: 16 / 8 / 4 chunks, 1 / 2 / 4 rows per sweep of the banks
  return D == 128 ? (((row & 3) << 2) | ((row >> 2) & 3)) : D == 64 ? ((((row >> 1) & 1) << 2) | ((row >> 2) & 3)) : ((row >> 2) & 3);
}
// The upper part of swz_rt for the rows a lane addresses in transpose reads (row = 4hh + gi/4 + 8x + 16cc,
// gi = lane % 16), in units of 4 chunks; its lower part is (hh + 2x) & 3 for every D.
template <int D>
__device__ __forceinline__ constexpr int swz_rt_group(int gi) { return D == 128 ? (gi >> 2) : D == 64 ? ((gi >> 3) & 1) : 0; }

// sigma and f' from u = x log2(e): returns sigma(x), stores f'(x)
__device__ __forceinline__ float silu_grad_log2(float u, float* fprime) {
  const float e = __builtin_amdgcn_exp2f(-u);
  const float sg = __builtin_amdgcn_rcpf(1.0f + e);
  *fprime = sg * __builtin_fmaf(u * LN2, 1.0f - sg, 1.0f);
  return sg;
}

// Turns a wave's 32 x D accumulator (lane (col m, half hh) holds channels 32 dvb + 8g + 4hh + t of
// row m) into whole bf16 rows through the wave's own 32 x D x 2 bytes of LDS and stores rows
// [row0, row0 + 32) that are below `rows`, rows at or past `n_live` as zeros.
template <int D>
__device__ __forceinline__ void store_rows(const floatx16 (&acc)[D / 32], float scale, unsigned char* ot, bf16_t* __restrict__ dst,
                                           int64_t row_stride, int row0, int n_live, int rows, int lane) {
  constexpr int CPR = D / 8, RPB = CPR >= 16 ? 1 : 16 / CPR;
  auto oswz = [](int row) { return (row / RPB) % CPR; };
  const int m = lane & 31, hh = lane >> 5;
  const bool live = row0 + m < n_live;
  unsigned char* orow = ot + m * (D * 2) + 8 * hh;
#pragma unroll
  for (int dvb = 0; dvb < D / 32; ++dvb) {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      uint2 pko = {0u, 0u};
      if (live) {
        pko.x = pack_bf16(acc[dvb][4 * g + 0] * scale, acc[dvb][4 * g + 1] * scale);
        pko.y = pack_bf16(acc[dvb][4 * g + 2] * scale, acc[dvb][4 * g + 3] * scale);
      }
      *(uint2*)(orow + (((4 * dvb + g) ^ oswz(m)) * 16)) = pko;
    }
  }
  constexpr int ROWS_PER_STORE = 64 / CPR;
  const int rr = lane / CPR, cc = lane - rr * CPR;
#pragma unroll
  for (int r0s = 0; r0s < 32; r0s += ROWS_PER_STORE) {
    const int row = r0s + rr;
    const uint4 val = *(const uint4*)(ot + row * (D * 2) + ((cc ^ oswz(row)) * 16));
    const int grow = row0 + row;
    if (grow < rows) *(uint4*)(dst + (int64_t)grow * row_stride + cc * 8) = val;
  }
}

// Extra LDS of the dQ kernel when it also sums table gradients: a ring of TG_RING diagonal sums per
// wave, then one sum per bucket for the workgroup.  Kept this small on purpose: with both biases at
// d = 128 the kernel's LDS is 78 KB, and two workgroups must still fit a CU's 160 KB.
constexpr int TG_RING = 128;
constexpr int TG_WG_RING = 256;      // the workgroup's ring of diagonal sums (within the NWAVES * TG_RING floats set aside)
constexpr int BWD_TG_BYTES = (NWAVES * TG_RING + TS_TAB_LEN) * 4;

// v of the lane `CTRL` names (data-parallel-primitive controls of the vector ALU: 0x110 + n = n lanes
// down within a row of 16, 0x142 / 0x143 = lane 15 of the previous row / lane 31 to the rows that
// ROW_MASK selects); 0 where there is no such lane or row
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, true));
}
// sum of v over the 64 lanes, the same value in every lane (all lanes must be active)
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp_f<0x111>(v);
  v += dpp_f<0x112>(v);
  v += dpp_f<0x114>(v);
  v += dpp_f<0x118>(v);
  v += dpp_f<0x142, 0xa>(v);
  v += dpp_f<0x143, 0xc>(v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// float atomic add on an LDS location given by an ordinary pointer (named as LDS for the compiler: on
// a pointer of unknown address space it builds a run-time dispatch that some instantiations miscompile)
typedef __attribute__((address_space(3))) float* lds_float_ptr;
__device__ __forceinline__ void lds_atomic_add(float* lds_location, float v) {
  __hip_atomic_fetch_add((lds_float_ptr)lds_location, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// TG: also accumulate the table gradients.  Every pair adds its dS to the entry of each table its
// logit read; LDS float atomics with many lanes on one address turned out to cost about 4 cycles per
// lane, so the sums are formed in registers first and reach LDS one lane per address.
// Position table: pair (q, key) of a workgroup lies on diagonal X = key - q + (q0 + 127) >= 0.  A block's
// 32 x 32 pairs are brought onto their 63 diagonals by lane permutes (see the block), one value per
// lane, and added to the workgroup's ring of sums.  The blocks of a pair of steps (t, t + 1) only touch
// X in [32 t, 32 t + 192), so everything below 32 (t + 2) is final after the pair's barrier: at the start
// of the next pair one wave adds those 64 diagonals to the table in memory and clears them.
// Bucket table: where each lane has one bucket for the whole block (or two neighbours), lanes with
// the same bucket are summed across the wave and one lane adds the sum to the workgroup's
// histogram (an LDS atomic, but of one lane); only blocks with more buckets per lane use one
// atomic per lane and run of equal buckets.
// MSK: a dense keep-mask [L, Lkv] or [B, L, Lkv] (the layer-side calling convention, without the dense bias): each
// step's tile of it -- this workgroup's 128 rows x 32 keys, 4 KB -- rides in the ring like the segment ids, every
// wave fetching its own 32 rows, and the steps outside the range the preparation found for the tile are left out.
// DB: the dense additive bias of that calling convention ([L, Lkv] or [B, L, Lkv] fp32, shared by the heads), the
// same way: a step's tile of 128 rows x 32 keys (16 KB) in the ring, each wave fetching its own 32 rows, 16-byte
// chunks XOR-swizzled by the row as in the forward.  Its gradient (p.dbias, when asked for) is dS: the wave writes
// its block of dS over its rows of the tile, which it has just read, and adds it to the matrix in memory by rows.
template <int D, bool POS, bool TS, bool TG, bool SEG = false, bool MSK = false, bool DB = false>
__global__ __launch_bounds__(MFMA_THREADS, DB ? 1 : 2) void hstu_bwd_dq_mfma(const Params p) {
  using SM = MfmaSmem<D, 2>;
  constexpr int CPR = SM::CPR;
  constexpr int QCH = D / 16;
  constexpr int DVB = D / 32;
  constexpr int NPIECE = SM::V_BYTES / 1024;            // 1 KB pieces of a tile; small tiles: several waves repeat a piece
  constexpr int LD = NPIECE >= NWAVES ? NPIECE / NWAVES : 1;
  constexpr int NDMA = 2 * LD + ((POS || TS) ? 1 : 0) + (SEG ? 1 : 0) + (MSK ? 1 : 0) + (DB ? 4 : 0);
  static_assert((NSTAGE - 1) * NDMA <= 63, "vmcnt range");
  static_assert(!(MSK || DB) || (!POS && !TS && !TG && !SEG), "dense operands come without the table biases and the segment ids");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const uint32_t smem_lds = __builtin_amdgcn_groupstaticsize();   // LDS byte address of smem
  auto Ks = [&](int st) { return (bf16_t*)(smem + st * SM::STAGE); };
  auto Vs = [&](int st) { return (bf16_t*)(smem + st * SM::STAGE + SM::K_BYTES); };
  constexpr int BIAS_OFF = NSTAGE * SM::STAGE;
  constexpr int BIAS_STAGE = SM::bias_stage(POS, TS, SEG) + (MSK ? SM::DM_BYTES : 0) + (DB ? SM::DB_BYTES : 0);
  auto Wc = [&](int st) { return (float*)(smem + BIAS_OFF + st * BIAS_STAGE); };
  auto Tk = [&](int st) { return (int32_t*)(smem + BIAS_OFF + st * BIAS_STAGE + (POS ? SM::POS_BYTES : 0)); };
  auto Sg = [&](int st) { return (int32_t*)(smem + BIAS_OFF + st * BIAS_STAGE + SM::bias_stage(POS, TS)); };
  auto Mk = [&](int st) { return smem + BIAS_OFF + st * BIAS_STAGE + SM::bias_stage(POS, TS, SEG); };   // MSK: [128 rows][32 bytes]
  auto Bk = [&](int st) { return smem + BIAS_OFF + st * BIAS_STAGE + SM::bias_stage(POS, TS, SEG) + (MSK ? SM::DM_BYTES : 0); };   // DB: [128 rows][128 bytes]
  const unsigned char* TsKey = smem + BIAS_OFF + NSTAGE * BIAS_STAGE;   // the keyed bucket table of this head
  float* TgBase = (float*)(smem + BIAS_OFF + NSTAGE * BIAS_STAGE + (TS ? SM::TAB_BYTES : 0));   // TG only
  const bool want_dpos = TG && POS && p.dpos != nullptr, want_dts = TG && TS && p.dts != nullptr;

  Work wk;
  if (!work_of_block(p, blockIdx.x, wk)) return;
  const int b = wk.b, h = wk.h, qt = wk.qt;
  const Seq& s = wk.s;
  const int q0 = qt * BM;
  if (q0 >= s.rows || wk.chunk > 0) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = lane & 31, hh = lane >> 5;
  const char* __restrict__ kg = (const char*)p.k + s.bk * 2;
  const char* __restrict__ vg = (const char*)p.v + s.bv * 2;
  bf16_t* __restrict__ dqg = (bf16_t*)p.dq + s.bq;

  if (q0 >= s.n_q) {
    const int rows = (s.rows - q0) < BM ? (s.rows - q0) : BM;
    const uint4 z = {0u, 0u, 0u, 0u};
    for (int e = tid; e < rows * (D / 8); e += MFMA_THREADS) {
      int r = e / (D / 8), c = e - r * (D / 8);
      *(uint4*)(dqg + (int64_t)(q0 + r) * p.q_st + c * 8) = z;
    }
    return;
  }

  const int r0 = q0 + 32 * w;
  const int qrow = r0 + m;
  const bool wave_live = r0 < s.n_q;
  int nt = tile_steps(p, s, q0);
  // a sliding window drops the steps before the tile's first key, and for each wave the blocks outside its band
  const int win = p.window;
  int t_lo = (win >= 0 && q0 - win > 0) ? (q0 - win) / BN : 0;
  if (MSK) {
    // the steps in which the keep-mask keeps a pair of this tile at all (found by the preparation kernel)
    const int2 mr = ((const int2*)p.mask_range)[(p.mask_batched ? b : 0) * p.n_qtiles + qt];
    t_lo = t_lo > mr.x ? t_lo : mr.x;
    nt = nt < mr.y ? nt : mr.y;
    nt = nt > t_lo ? nt : t_lo;
  }
  int wave_last = p.causal ? r0 + 31 : (win >= 0 ? r0 + 31 + win : s.n_kv - 1);
  wave_last = wave_last < s.n_kv - 1 ? wave_last : s.n_kv - 1;
  if (!wave_live) wave_last = -1;

  const float alpha2 = p.alpha * LOG2E;
  const uint32_t kst_bytes = (uint32_t)p.k_st * 2u, vst_bytes = (uint32_t)p.v_st * 2u;
  const char* wsb = (const char*)p.ws_base;
  const uint32_t pos_off = POS ? (uint32_t)((const char*)(p.pos_scaled + (int64_t)(p.pos_heads > 1 ? h : 0) * (2 * p.L - 1 + 2 * POS_PAD)) - wsb) : 0u;
  const int64_t* tsg = TS ? p.ts + s.ts0 : nullptr;
  const int32_t* trel = TS ? p.ts_rel + ts_rel_base(p, b, s.tok0) : nullptr;
  const int ts32 = TS ? p.ts_ok[b] : 0;
  const uint32_t rel_off = TS ? (uint32_t)((const char*)trel - wsb) : 0u;
  const uint32_t rng_off = TS ? (uint32_t)((const char*)(p.ts_range + 2 * ts_range_slot0(p, b, s.tok0)) - wsb) : 0u;

  // direct loads of step t, as in the forward, both tiles with the two-way swizzle
  auto dma_step = [&](int t) {
    const int st = t % NSTAGE;
    const int kv0 = t * BN;
    const int last = s.n_kv - 1;
#pragma unroll
    for (int r = 0; r < LD; ++r) {
      const int j = (w * LD + r) % NPIECE;
      const int c = 64 * j + lane;
      const int row = c / CPR, pc = c - row * CPR;
      int grow = kv0 + row;
      grow = grow < last ? grow : last;
      const uint32_t sw = (uint32_t)((pc ^ swz_rt<D>(row)) * 16);
      lds_dma16(kg, (uint32_t)grow * kst_bytes + sw, (const unsigned char*)Ks(st) + j * 1024);
      lds_dma16(vg, (uint32_t)grow * vst_bytes + sw, (const unsigned char*)Vs(st) + j * 1024);
    }
    if (POS || TS) {
      constexpr int TS_LANE0 = POS ? SM::POS_LANES : 0;
      const bool ts_wave = TS && (!POS || w == NWAVES - 1);
      const int tl = lane - TS_LANE0;
      uint32_t off = 0;
      bool on = false;
      if (POS && lane < SM::POS_LANES) {
        off = pos_off + (uint32_t)(POS_PAD + (p.L - 1) + kv0 - (q0 + BM - 1) + w + 4 * lane) * 4u;
        on = true;
      }
      if (ts_wave && tl >= 0 && tl < SM::TK_LANES) {
        int tr = t;
        const int tr_last = (s.n_ts - 1) >> 5;
        tr = tr < tr_last ? tr : tr_last;
        off = tl < BN / 4 ? rel_off + (uint32_t)(kv0 + 4 * tl) * 4u : rng_off + (uint32_t)tr * 8u;
        on = true;
      }
      if (on) lds_dma16(wsb, off, (const unsigned char*)Wc(st) + (POS ? w * SM::POS_COPY : 0));
    }
    if (SEG) {
      // the step's 32 key segment ids, as in the forward
      if (lane < BN / 4) {
        int g4 = kv0 + 4 * lane;
        g4 = g4 < p.Lkv - 4 ? g4 : p.Lkv - 4;
        lds_dma16_at(p.kv_seg + (int64_t)b * p.Lkv, (uint32_t)g4 * 4u, smem_lds + (uint32_t)((const unsigned char*)Sg(st) - smem));
      }
    }
    if (MSK) {
      // the wave's own 32 rows of the step's mask tile, two lanes per row; rows past L and the second half of a last
      // step of 16 keys re-read bytes inside the matrix (those pairs are masked by their index)
      const uint8_t* mg = p.mask + (p.mask_batched ? (int64_t)b * p.L * p.Lkv : 0);
      int gr = r0 + (lane >> 1);
      gr = gr < p.L - 1 ? gr : p.L - 1;
      int col = kv0 + 16 * (lane & 1);
      col = col < p.Lkv - 16 ? col : p.Lkv - 16;
      lds_dma16(mg, (uint32_t)gr * (uint32_t)p.Lkv + (uint32_t)col, Mk(st) + w * 1024);
    }
    if (DB) {
      // the wave's own 32 rows of the step's bias tile in four pieces of 8 rows: row r at byte 128 r, lane l of a piece
      // lands at row l / 8, physical chunk l % 8, and fetches the logical chunk the swizzle maps there.  Rows past L
      // and keys past Lkv re-read the last row / the last four keys (those pairs are masked by their index).
      const float* bg = p.dense_bias + (p.dense_bias_batched ? (int64_t)b * p.L * p.Lkv : 0);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = 32 * w + 8 * r + (lane >> 3), pc = lane & 7;
        int gr = q0 + row;
        gr = gr < p.L - 1 ? gr : p.L - 1;
        int col = kv0 + 4 * (pc ^ (row & 7));
        col = col < p.Lkv - 4 ? col : p.Lkv - 4;
        lds_dma16(bg, ((uint32_t)gr * (uint32_t)p.Lkv + (uint32_t)col) * 4u, Bk(st) + (4 * w + r) * 1024);
      }
    }
  };

  if (TS) {
    // three direct loads of up to 1 KB, one each by waves 0 to 2 (the last wave repeats the first)
    const int c = w < 3 ? w : 0;
    if (1024 * c + 16 * lane < TS_LDS_BYTES)
      lds_dma16((const unsigned char*)p.ts_keyed + (int64_t)(p.ts_heads > 1 ? h : 0) * (3 * 1024) + 1024 * c, (uint32_t)lane * 16u, TsKey + 1024 * c);
  }
  // the first pair of steps in flight (the step loop runs in pairs, see there)
  if (t_lo < nt) dma_step(t_lo);
  if (t_lo + 1 < nt) dma_step(t_lo + 1);
  if (TG) {
    for (int i = tid; i < NWAVES * TG_RING + TS_TAB_LEN; i += MFMA_THREADS) TgBase[i] = 0.f;
  }

  // Q and dO fragments of this lane's row (B operands): 16-byte chunk 2ks + hh of the row
  uint4 qf[QCH], dof[QCH];
  {
    const char* qg = (const char*)p.q + (s.bq + (int64_t)qrow * p.q_st) * 2 + 16 * hh;
    const char* dg = (const char*)p.dout + (s.bo + (int64_t)qrow * p.o_st) * 2 + 16 * hh;
#pragma unroll
    for (int ks = 0; ks < QCH; ++ks) {
      uint4 a = {0u, 0u, 0u, 0u}, c = {0u, 0u, 0u, 0u};
      if (qrow < s.n_q) { a = *(const uint4*)(qg + 32 * ks); c = *(const uint4*)(dg + 32 * ks); }
      qf[ks] = a;
      dof[ks] = c;
    }
    // consumed here so that the wait for these loads stays out of the loop (it would be a wait for
    // every direct load in flight as well)
#pragma unroll
    for (int ks = 0; ks < QCH; ++ks) {
      asm volatile("" ::"v"(qf[ks].x), "v"(qf[ks].y), "v"(qf[ks].z), "v"(qf[ks].w));
      asm volatile("" ::"v"(dof[ks].x), "v"(dof[ks].y), "v"(dof[ks].z), "v"(dof[ks].w));
    }
  }
  int32_t qseg = 0;
  if (SEG) {
    qseg = p.q_seg[(int64_t)b * p.L + (qrow < p.L ? qrow : p.L - 1)];
    asm volatile("" ::"v"(qseg));
  }
  int32_t tq32 = 0;
  int iq_lane = 0;       // index of the timestamp this lane's row takes (the 64-bit path reads it from memory again)
  if (TS) {
    int iq = qrow + 1 < s.n_ts ? qrow + 1 : s.n_ts - 1;
    iq_lane = iq < 0 ? 0 : iq;
    tq32 = trel[iq_lane];     // meaningless when !ts32, and then unused
    asm volatile("" ::"v"(tq32));
  }

  floatx16 acc[DVB];
#pragma unroll
  for (int i = 0; i < DVB; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;

  const int gk = swz_rt<D>(m);
  // transpose reads of K: lane i of 16-lane group G addresses 8 bytes of row 4hh + i/4 (+ 8x + 16cc),
  // logical chunk 4 dvb + 2 (G & 1) + (i & 3) / 2.  For those rows swz_rt = 4 (i/4) + ((hh + 2x) & 3).
  const int gi = lane & 15;
  const int vrow = 4 * hh + (gi >> 2);
  const int vc2 = 2 * ((lane >> 4) & 1) + ((gi & 3) >> 1);
  const int c_lo = vc2 ^ hh, c_hi = vc2 ^ (hh + 2);

  auto block = [&](int t) {
    const int st = t % NSTAGE;
    const int kbs = t * BN;
    const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    floatx16 sacc, dpacc;
    {
      uint4 kf[QCH];
      const unsigned char* kr = (const unsigned char*)Ks(st) + m * (D * 2);
#pragma unroll
      for (int ks = 0; ks < QCH; ++ks) kf[ks] = *(const uint4*)(kr + (((2 * ks + hh) ^ gk) * 16));
#pragma unroll
      for (int ks = 0; ks < QCH; ++ks)
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[ks]), __builtin_bit_cast(bf16x8, qf[ks]),
                                                       ks == 0 ? zero : sacc, 0, 0, 0);
    }
    {
      uint4 vf[QCH];
      const unsigned char* vr = (const unsigned char*)Vs(st) + m * (D * 2);
#pragma unroll
      for (int ks = 0; ks < QCH; ++ks) vf[ks] = *(const uint4*)(vr + (((2 * ks + hh) ^ gk) * 16));
#pragma unroll
      for (int ks = 0; ks < QCH; ++ks)
        dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf[ks]), __builtin_bit_cast(bf16x8, dof[ks]),
                                                        ks == 0 ? zero : dpacc, 0, 0, 0);
    }
    // lane holds S^T[kv = kbs + 8g + 4hh + tt][q = qrow], r = 4g + tt
    float u[16];
    // for the table gradients: either this lane's 16 pairs are in bucket bk_lane >= 0, those with a bit
    // in far_bits in the next one (then every lane of the wave has such a pair of buckets), or bkp holds
    // the 16 buckets, one byte each (bucket < TS_TAB_LEN <= 255)
    uint32_t bkp[4] = {0u, 0u, 0u, 0u};
    uint32_t far_bits = 0u;
    int bk_lane = -1;
    if (POS) {
      const int xb = 4 * hh + (BM - 1) - 32 * w - m;
      const int sft = xb & 3;
      const float* wrow = (const float*)((const unsigned char*)Wc(st) + sft * SM::POS_COPY) + (xb - sft);
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
    if (DB) {
      // the lane's row of the bias tile: keys 8g + 4hh .. + 3 are logical chunk 2g + hh
      const int row = 32 * w + m;
      const unsigned char* brow = Bk(st) + row * 128;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float4 bv = *(const float4*)(brow + (((2 * g + hh) ^ (row & 7)) * 16));
        u[4 * g + 0] = __builtin_fmaf(bv.x, LOG2E, u[4 * g + 0]);
        u[4 * g + 1] = __builtin_fmaf(bv.y, LOG2E, u[4 * g + 1]);
        u[4 * g + 2] = __builtin_fmaf(bv.z, LOG2E, u[4 * g + 2]);
        u[4 * g + 3] = __builtin_fmaf(bv.w, LOG2E, u[4 * g + 3]);
      }
    }
    if (TS) {
      if (ts32) {
        const int32_t* tk = Tk(st);
        const int2 rg = *(const int2*)(tk + BN);
        const TsEnds en = ts_ends(TsKey, tq32 - rg.y, tq32 - rg.x);
        if (__builtin_amdgcn_ballot_w64(!en.same) == 0) {
          const float add = en.v_near;
#pragma unroll
          for (int r = 0; r < 16; ++r) u[r] += add;
          bk_lane = en.b_near;
        } else if (__builtin_amdgcn_ballot_w64(!en.two) == 0) {
          // at most one bucket boundary inside the tile for every lane: a key is in the farther
          // bucket exactly when tq - tk >= thr, i.e. tk <= tq - thr (a lane whose ends share a bucket
          // must not flag any key: the next bucket's sum would take its dS)
          const float add_near = en.v_near, add_far = en.v_far;
          const int cut = en.b_far != en.b_near ? tq32 - en.thr : (int)0x80000000;
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int4 kk = *(const int4*)(tk + 8 * g + 4 * hh);
            const bool f0 = kk.x <= cut, f1 = kk.y <= cut, f2 = kk.z <= cut, f3 = kk.w <= cut;
            u[4 * g + 0] += f0 ? add_far : add_near;
            u[4 * g + 1] += f1 ? add_far : add_near;
            u[4 * g + 2] += f2 ? add_far : add_near;
            u[4 * g + 3] += f3 ? add_far : add_near;
            if (TG) far_bits |= ((uint32_t)f0 | ((uint32_t)f1 << 1) | ((uint32_t)f2 << 2) | ((uint32_t)f3 << 3)) << (4 * g);
          }
          bk_lane = en.b_near;
        } else {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int4 kk = *(const int4*)(tk + 8 * g + 4 * hh);
            if (TG) {
              const int b0 = ts_bucket_of(TsKey, tq32 - kk.x), b1 = ts_bucket_of(TsKey, tq32 - kk.y);
              const int b2 = ts_bucket_of(TsKey, tq32 - kk.z), b3 = ts_bucket_of(TsKey, tq32 - kk.w);
              u[4 * g + 0] += ts_bucket_value(TsKey, b0);
              u[4 * g + 1] += ts_bucket_value(TsKey, b1);
              u[4 * g + 2] += ts_bucket_value(TsKey, b2);
              u[4 * g + 3] += ts_bucket_value(TsKey, b3);
              bkp[g] = (uint32_t)b0 | ((uint32_t)b1 << 8) | ((uint32_t)b2 << 16) | ((uint32_t)b3 << 24);
            } else {
              u[4 * g + 0] += ts_value(ts_look(TsKey, tq32 - kk.x));
              u[4 * g + 1] += ts_value(ts_look(TsKey, tq32 - kk.y));
              u[4 * g + 2] += ts_value(ts_look(TsKey, tq32 - kk.z));
              u[4 * g + 3] += ts_value(ts_look(TsKey, tq32 - kk.w));
            }
          }
        }
      } else {
        // time span of the sequence beyond 31 bits: 64-bit differences of timestamps read straight
        // from memory (rare; correctness over speed)
        const int64_t tq = tsg[iq_lane];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
#pragma unroll
          for (int tt = 0; tt < 4; ++tt) {
            int j = kbs + 8 * g + 4 * hh + tt;
            j = j < s.n_ts ? j : s.n_ts - 1;
            const int bb = ts_bucket_of(TsKey, ts_clip64(tq - tsg[j]));
            u[4 * g + tt] += ts_bucket_value(TsKey, bb);
            if (TG) bkp[g] = tt == 0 ? (uint32_t)bb : bkp[g] | ((uint32_t)bb << (8 * tt));
          }
        }
      }
    }
    float ds[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float fp;
      silu_grad_log2(u[r], &fp);
      ds[r] = dpacc[r] * fp;
    }
    // f'(0) is not 0: masked pairs are cleared after the activation's derivative
    if ((p.causal && kbs + 31 > r0) || (kbs + 32 > s.n_kv) || (win >= 0 && (r0 + 31 - kbs > win || kbs + 31 - r0 > win))) {
      // lo <= kv <= hi for the lane's row; register r holds key kbs + 4hh + c(r), c(r) = 8 (r / 4) + r % 4
      int hi = p.causal ? qrow : (win >= 0 ? qrow + win : s.n_kv - 1);
      hi = hi < s.n_kv - 1 ? hi : s.n_kv - 1;
      const int hi_rel = hi - kbs - 4 * hh;
      const int lo_rel = win >= 0 ? qrow - win - kbs - 4 * hh : -1;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 8 * (r >> 2) + (r & 3);
        ds[r] = (c <= hi_rel && c >= lo_rel) ? ds[r] : 0.f;
      }
    }
    if (SEG) {
      const int32_t* sg = Sg(st);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int4 ks4 = *(const int4*)(sg + 8 * g + 4 * hh);
        ds[4 * g + 0] = ks4.x == qseg ? ds[4 * g + 0] : 0.f;
        ds[4 * g + 1] = ks4.y == qseg ? ds[4 * g + 1] : 0.f;
        ds[4 * g + 2] = ks4.z == qseg ? ds[4 * g + 2] : 0.f;
        ds[4 * g + 3] = ks4.w == qseg ? ds[4 * g + 3] : 0.f;
      }
    }
    if (MSK) {
      // the lane's row of the mask tile: bytes of keys 8g + 4hh .. + 3
      const unsigned char* mrow = Mk(st) + (32 * w + m) * 32 + 4 * hh;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const uint32_t mb = *(const uint32_t*)(mrow + 8 * g);
        ds[4 * g + 0] = (mb & 0xffu) ? ds[4 * g + 0] : 0.f;
        ds[4 * g + 1] = (mb & 0xff00u) ? ds[4 * g + 1] : 0.f;
        ds[4 * g + 2] = (mb & 0xff0000u) ? ds[4 * g + 2] : 0.f;
        ds[4 * g + 3] = (mb & 0xff000000u) ? ds[4 * g + 3] : 0.f;
      }
    }
    if (p.drop_thr) {
      // dropout: the pairs the forward dropped carry no gradient
      drop_apply16(ds, drop_bh_key(p.drop_key, (uint32_t)b * (uint32_t)p.H + (uint32_t)h) + (uint32_t)qrow * DROP_CI +
                           (uint32_t)(kbs + 4 * hh) * DROP_CJ, DROP_CJ, p.drop_thr);
    }
    if (DB && p.dbias != nullptr) {
      // Dense-bias gradient: the heads' workgroups, and the sequences' for a shared bias, add dS / N into one matrix.
      // A lane's 16 pairs lie in one row of it; written over the wave's rows of the bias tile (read above; the wave's
      // LDS operations run in order, and nobody else touches these rows before the next barrier but one) and read
      // back by rows, an instruction adds two whole rows of the block: two cache lines instead of 32.  Masked pairs
      // and pairs outside the matrix are 0 and are skipped.
      const int row = 32 * w + m;
      unsigned char* brow = Bk(st) + row * 128;
#pragma unroll
      for (int g = 0; g < 4; ++g)
        *(float4*)(brow + (((2 * g + hh) ^ (row & 7)) * 16)) =
            float4{ds[4 * g + 0] * p.inv_n, ds[4 * g + 1] * p.inv_n, ds[4 * g + 2] * p.inv_n, ds[4 * g + 3] * p.inv_n};
      float* dbp = p.dbias + (p.dense_bias_batched ? (int64_t)b * p.L * p.Lkv : 0) + (int64_t)r0 * p.Lkv + kbs;
      const int col = lane & 31;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int rr = 2 * i + (lane >> 5), rw = 32 * w + rr;
        const float val = *(const float*)(Bk(st) + rw * 128 + (((col >> 2) ^ (rw & 7)) * 16) + (col & 3) * 4);
        if (val != 0.f) atomicAdd(dbp + (int64_t)rr * p.Lkv + col, val);
      }
    }
    if (want_dpos) {
      // Pair (row m, key offset c = 8g + 4hh + tt) lies on diagonal c - m.  Lane j takes, for each of
      // its 16 offsets, the value of row (j + c) mod 32 of its half: all 16 are then on diagonal -j or,
      // where j + c wrapped, 32 - j.  The two sums are completed with the other half's and added to
      // the wave's ring: lanes of the lower half own -j, lanes of the upper half 32 - j.
      // (the lane's index enters through a register the compiler cannot see through: it would otherwise
      // keep the 16 permute addresses of the loop below in registers across the whole key loop, which
      // this kernel does not have)
      int jj = m + 4 * hh;
      if (D == 128) asm volatile("" : "+v"(jj));        // (smaller head dims have the 16 registers)
      const int half4 = (lane & 32) << 2;
      float s_all = 0.f, s_low = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c0 = 8 * (r >> 2) + (r & 3);
        const int addr = (((jj + c0) & 31) << 2) | half4;
        const float rv = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(addr, __builtin_bit_cast(int, ds[r])));
        s_all += rv;
        s_low += (jj + c0 < 32) ? rv : 0.f;
      }
      const float s_high = s_all - s_low;
      const float mine = hh ? s_high : s_low, theirs = hh ? s_low : s_high;
      const float got = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, __builtin_bit_cast(int, theirs)));
      // the workgroup's ring of diagonal sums: this wave's diagonal X is the workgroup's X + 96 - 32 w (a lane per
      // slot within the instruction; other waves may add to the same slots, hence the atomic form)
      lds_atomic_add(TgBase + ((kbs + 127 - m + 32 * hh - 32 * w) & (TG_WG_RING - 1)), mine + got);
    }
    if (want_dts) {
      float* hist = TgBase + NWAVES * TG_RING;
      if (bk_lane >= 0) {
        float s_near = 0.f, s_far = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const bool far = (far_bits >> r) & 1u;
          s_near += far ? 0.f : ds[r];
          s_far += far ? ds[r] : 0.f;
        }
        // lanes with the same bucket are summed together, one bucket value per round
        const bool any_far = __builtin_amdgcn_ballot_w64(far_bits != 0u) != 0;
        bool done = false;
        for (;;) {
          const uint64_t act = __builtin_amdgcn_ballot_w64(!done);
          if (act == 0) break;
          const int leader = __builtin_ctzll(act);
          const int b0 = __builtin_amdgcn_readlane(bk_lane, leader);
          const bool mine = !done && bk_lane == b0;
          const float a = wave_sum(mine ? s_near : 0.f);
          const float c = any_far ? wave_sum(mine ? s_far : 0.f) : 0.f;
          if (lane == 0) {
            lds_atomic_add(&hist[b0], a);
            if (any_far) lds_atomic_add(&hist[b0 + 1], c);
          }
          done = done || mine;
        }
      } else {
        // LDS atomics cost by the lane: neighbouring keys mostly share a bucket, so each run of equal
        // buckets is summed first, and runs that add nothing (masked pairs) are skipped
        float carry = 0.f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const uint32_t bcur = (bkp[r >> 2] >> (8 * (r & 3))) & 255u;
          const uint32_t bnext = r < 15 ? (bkp[(r + 1) >> 2] >> (8 * ((r + 1) & 3))) & 255u : 256u;
          carry += ds[r];
          if (bcur != bnext) {
            if (carry != 0.f) lds_atomic_add(&hist[bcur], carry);
            carry = 0.f;
          }
        }
      }
    }
    // K^T fragments for the last product
    uint4 ktf[2][DVB];
    {
      const bf16_t* kr = Ks(st) + vrow * D + 4 * (gi & 1);
#pragma unroll
      for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int dvb = 0; dvb < DVB; ++dvb) {
          const int cb = 4 * (dvb ^ swz_rt_group<D>(gi));
          uint2 lo = lds_read_tr(kr + (16 * cc) * D + (cb + c_lo) * 8);
          uint2 hi = lds_read_tr(kr + (16 * cc + 8) * D + (cb + c_hi) * 8);
          ktf[cc][dvb] = uint4{lo.x, lo.y, hi.x, hi.y};
        }
    }
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      uint4 pk;
      pk.x = pack_bf16(ds[8 * cc + 0], ds[8 * cc + 1]);
      pk.y = pack_bf16(ds[8 * cc + 2], ds[8 * cc + 3]);
      pk.z = pack_bf16(ds[8 * cc + 4], ds[8 * cc + 5]);
      pk.w = pack_bf16(ds[8 * cc + 6], ds[8 * cc + 7]);
      const bf16x8 pb = __builtin_bit_cast(bf16x8, pk);
#pragma unroll
      for (int dvb = 0; dvb < DVB; ++dvb)
        acc[dvb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ktf[cc][dvb]), pb, acc[dvb], 0, 0, 0);
    }
  };

  // adds diagonals [x0, x0 + 64) of the workgroup's ring to the table in memory and clears them (one wave's job)
  auto flush_diag = [&](int x0) {
    float* slot = TgBase + ((x0 + lane) & (TG_WG_RING - 1));
    const float val = *slot;
    *slot = 0.f;
    const int idx = (p.L - 1) + (x0 + lane) - (BM - 1) - q0;
    if (val != 0.f && idx >= 0 && idx < 2 * p.L - 1)
      atomicAdd(p.dpos + (int64_t)(p.pos_heads > 1 ? h : 0) * (2 * p.L - 1) + idx, val * p.inv_n);
  };

  // Steps in pairs with one barrier per pair, as in the forward: the barrier that ended the pair
  // (t-2, t-1) freed its two ring stages for steps t+2 and t+3 (full-length batch 4.90 -> 4.67 ms,
  // the headline shape 0.356 -> 0.347 ms with both backward kernels changed).
  static_assert(NSTAGE == 4, "two pairs of stages");
  HSTU_WAIT_VMCNT(0);
  __syncthreads();
  // Position-table gradient: the four waves add their blocks' diagonal sums into ONE ring of the workgroup
  // (diagonal X = key - row + q0 + 127; the blocks of step pair (t, t + 1) touch [32 t, 32 t + 192)), and what a
  // pair has completed -- [32 t, 32 t + 64), final once every wave is past the pair's barrier -- goes to memory
  // at the start of the next pair, by one wave in turn.  Every workgroup of the launch adds into the one table:
  // with a ring per wave, each flushing its own 64 diagonals per pair, those adds (four times as many) cost a
  // config-4 layer 0.19 of the 0.31 ms the table gradient took.
  for (int t = t_lo; t < nt; t += 2) {
    if (want_dpos && t > t_lo && w == ((t >> 1) & 3)) flush_diag(32 * (t - 2));
    if (t + 2 < nt) dma_step(t + 2);
    if (t + 3 < nt) dma_step(t + 3);
#pragma unroll
    for (int u = t; u < t + 2; ++u) {
      if (u < nt && u * BN <= wave_last && (win < 0 || u * BN + 31 + win >= r0)) block(u);
    }
    HSTU_WAIT_VMCNT(0);
    __syncthreads();
  }
  if (want_dpos && t_lo < nt && w < 3) {
    // what the last pair left in the ring (every wave is past the loop's last barrier)
    const int t_last = t_lo + ((nt - 1 - t_lo) & ~1);
    flush_diag(32 * t_last + 64 * w);
  }
  if (want_dts) {
    // every wave is past the loop's last barrier: the histogram is complete
    const float* hist = TgBase + NWAVES * TG_RING;
    for (int e = tid; e < TS_TAB_LEN; e += MFMA_THREADS) {
      const float val = hist[e];
      if (val != 0.f) atomicAdd(p.dts + (int64_t)(p.ts_heads > 1 ? h : 0) * (p.ts_nb + 1) + (e < p.ts_nb ? e : p.ts_nb), val * p.inv_n);
    }
  }
  // dQ^T[d][q] -> rows of dq (the ring is free: the loop ended on a barrier, no load is in flight)
  store_rows<D>(acc, p.alpha * p.inv_n, smem + w * (32 * D * 2), dqg, p.q_st, r0, s.n_q, s.rows, lane);
}

// At d = 128 two 32 x 128 accumulators plus the K and V fragments are 192 registers before any
// temporary: one workgroup per CU, the accumulators in the accumulation registers (ACC_ASM below).
// DSPLIT = 2 would share the work of 32 keys between two waves, each accumulating dK and dV for
// half of the channels (8 waves per workgroup): measured, no gain -- both waves repeat S, dP and
// the pointwise math -- and left at 1.
// acc = 0 and acc += A B with the accumulator named as accumulation registers (ACC_ASM).  Left to the
// compiler, the loop-carried accumulators of the d = 128 kernel live in ordinary registers and all
// 128 are copied to the accumulation file and back around the products of every block.  Written
// this way every definition of them is an accumulation register, so they stay there.  They are
// only ever read as the C operand of the same instruction (chained by the hardware without wait
// states) and by the final stores, which wait out the last product first.
// VREG: the accumulator in ordinary vector registers instead (the instances whose interior blocks run as the
// hand-scheduled stream, which keeps them there: as the C / D operand of this instruction an accumulation
// register costs about 140 cycles an instruction against 32, measured; every statement that names an
// accumulator must use the same kind, or the compiler copies all of them across).
template <bool VREG>
__device__ __forceinline__ void mfma_acc_zero(floatx16& acc) {
  const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
  if constexpr (VREG) asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %1, 0" : "=v"(acc) : "v"(z));
  else asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %1, 0" : "=a"(acc) : "v"(z));
}
template <bool VREG>
__device__ __forceinline__ void mfma_acc(floatx16& acc, bf16x8 a, bf16x8 b) {
  // The wait states cover an operand written by the vector ALU just before: the compiler pads such a
  // pair to two wait states for its own matrix instructions but does not look into this statement
  // (without them results were wrong); four leave a margin.
  if constexpr (VREG) asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
  else asm volatile("s_nop 3\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}

// Ring depth of the dK/dV kernel (see there).
constexpr int dkv_stages(int d, bool dense_bias) { return (d == 128 && !dense_bias) ? 6 : NSTAGE; }

template <int D>
struct DkvShape {
  static constexpr bool ACC_ASM = D == 128;
  static constexpr int DSPLIT = 1;                       // waves per 32 keys
  static constexpr int NW = NWAVES * DSPLIT;             // waves per workgroup
  static constexpr int THREADS = 64 * NW;
  static constexpr int DW = D / DSPLIT;                  // channels of dK / dV per wave
};

// MSK: the dense keep-mask as in the other backward kernel; here a step's tile is 32 query rows x this workgroup's
// 128 keys (wave w fetches rows 8w .. 8w + 7 of it, 128 bytes each), a lane reads the 16 bytes of its key's column,
// and the workgroup finds the query steps in which the mask keeps one of its keys by one pass over its columns.
// DB: the dense bias likewise, a step's tile of 32 rows x 128 keys (16 KB): wave w fetches rows 8w .. 8w + 7, a lane
// reads the 16 values of its key's column (consecutive lanes, consecutive words: no swizzle needed).  The bias's
// gradient is the other kernel's business.
template <int D, bool POS, bool TS, bool SEG = false, bool MSK = false, bool DB = false>
__global__ __launch_bounds__(DkvShape<D>::THREADS, (D == 128 || DB) ? 1 : 2) void hstu_bwd_dkv_mfma(const Params p) {
  using SH = DkvShape<D>;
  constexpr int NW = SH::NW, THREADS = SH::THREADS, DW = SH::DW;
  constexpr bool ACC_ASM = SH::ACC_ASM;
  // A pair of blocks that needs no mask runs as one hand-scheduled instruction stream (hstu_bwd_stream_d128.inc,
  // written by gen_bwd_stream.py): the vector part of one block behind the matrix instructions of the other.
  constexpr bool STREAM = D == 128 && !POS && !TS && !SEG && !MSK && !DB && SH::DSPLIT == 1;
  constexpr int DVBW = DW / 32;          // 32-channel blocks of dK / dV per wave
  using SM = MfmaSmem<D, 2>;
  constexpr int CPR = SM::CPR;
  constexpr int QCH = D / 16;
  constexpr int DVB = D / 32;
  constexpr int NPIECE = SM::V_BYTES / 1024;
  constexpr int LD = NPIECE >= NW ? NPIECE / NW : 1;
  constexpr int NDMA = 2 * LD + ((POS || TS) ? 1 : 0) + (SEG ? 1 : 0) + (MSK ? 1 : 0) + (DB ? 4 : 0);
  // Ring depth: 4 stages (two pairs of steps: one at work, one on its way), or 6 where the workgroup has the CU's
  // LDS to itself anyway (d = 128) and the stages are small enough: the loads of a pair then have the time of two
  // pairs to arrive, which the hand-scheduled pairs need (one pair's time is less than a trip to memory).
  constexpr int NST = dkv_stages(D, DB);
  constexpr int AHEAD = NST - 2;           // steps between a load and its use
  static_assert((NST - 1) * NDMA <= 63, "vmcnt range");
  static_assert(!(MSK || DB) || (!POS && !TS && !SEG && SH::DSPLIT == 1), "dense operands come without the table biases and the segment ids");
  // timestamp operands of a step: 36 int32 query-side timestamps (rows qbs .. qbs + 35), then the
  // (min, max) of timestamp tiles t and t + 1
  constexpr int TQ_LANES = BN / 4 + 2;
  constexpr int TQ_BYTES = TQ_LANES * 16;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const uint32_t smem_lds = __builtin_amdgcn_groupstaticsize();   // LDS byte address of smem
  // ring stage: [Q tile | dO tile], 32 rows each
  auto Qs = [&](int st) { return (bf16_t*)(smem + st * SM::STAGE); };
  auto Os = [&](int st) { return (bf16_t*)(smem + st * SM::STAGE + SM::K_BYTES); };
  constexpr int BIAS_OFF = NST * SM::STAGE;
  constexpr int BIAS_STAGE = (POS ? SM::POS_BYTES : 0) + (TS ? TQ_BYTES : 0) + (SEG ? SM::SEG_BYTES : 0) + (MSK ? SM::DM_BYTES : 0) +
                             (DB ? SM::DB_BYTES : 0);
  auto Sg = [&](int st) { return (int32_t*)(smem + BIAS_OFF + st * BIAS_STAGE + (POS ? SM::POS_BYTES : 0) + (TS ? TQ_BYTES : 0)); };
  auto Mk = [&](int st) { return smem + BIAS_OFF + st * BIAS_STAGE; };      // MSK (first in the stage): [32 rows][128 bytes]
  auto Bk = [&](int st) { return smem + BIAS_OFF + st * BIAS_STAGE + (MSK ? SM::DM_BYTES : 0); };   // DB: [32 rows][128 floats]
  auto Wc = [&](int st) { return (float*)(smem + BIAS_OFF + st * BIAS_STAGE); };
  auto Tq = [&](int st) { return (int32_t*)(smem + BIAS_OFF + st * BIAS_STAGE + (POS ? SM::POS_BYTES : 0)); };
  const unsigned char* TsKey = smem + BIAS_OFF + NST * BIAS_STAGE;   // the keyed bucket table of this head

  Work wk;
  if (!work_of_block(p, blockIdx.x, wk)) return;
  const int b = wk.b, h = wk.h;
  const Seq& s = wk.s;
  if (wk.chunk > 0) return;
  // The list names query tiles, the one with most keys first; here the key tile with most query
  // rows behind it goes first: under the causal mask that is the reverse order.
  const int n_live = (s.n_kv + BM - 1) / BM;
  const int kt = (p.causal && wk.qt < n_live) ? n_live - 1 - wk.qt : wk.qt;
  const int kv0 = kt * BM;
  if (kv0 >= s.rows) return;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int w8 = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int w = w8 % NWAVES;            // which 32 keys of the tile
  const int dh = w8 / NWAVES;           // which part of the channels
  const int m = lane & 31, hh = lane >> 5;
  const char* __restrict__ qg = (const char*)scalar_ptr((const char*)p.q + s.bq * 2);
  const char* __restrict__ dog = (const char*)scalar_ptr((const char*)p.dout + s.bo * 2);
  bf16_t* __restrict__ dkg = (bf16_t*)p.dk + s.bk;
  bf16_t* __restrict__ dvg = (bf16_t*)p.dv + s.bv;

  if (kv0 >= s.n_kv) {
    const int rows = (s.rows - kv0) < BM ? (s.rows - kv0) : BM;
    const uint4 z = {0u, 0u, 0u, 0u};
    for (int e = tid; e < rows * (D / 8); e += THREADS) {
      int r = e / (D / 8), c = e - r * (D / 8);
      *(uint4*)(dkg + (int64_t)(kv0 + r) * p.k_st + c * 8) = z;
      *(uint4*)(dvg + (int64_t)(kv0 + r) * p.v_st + c * 8) = z;
    }
    return;
  }

  const int r0 = kv0 + 32 * w;          // first key of this wave
  const int kcol = r0 + m;              // this lane's key
  const bool wave_live = r0 < s.n_kv;
  // steps: 32 query rows each; under the causal mask only rows from the tile's first key on
  // and, under a sliding window, only rows up to the window past the tile's (the wave's) last key
  const int win = p.window;
  int nt = (s.n_q + BN - 1) / BN;
  if (win >= 0 && (kv0 + BM - 1 + win) / BN + 1 < nt) nt = (kv0 + BM - 1 + win) / BN + 1;
  int t_lo = p.causal ? kv0 / BN : ((win >= 0 && kv0 - win > 0) ? (kv0 - win) / BN : 0);
  if (MSK) {
    // the query steps in which the mask keeps one of this tile's keys (a mask that carries the causal rule is
    // empty above the diagonal: without this every key tile would walk all the rows)
    int lo = t_lo < nt ? t_lo : nt, hi = nt;
    const int n_kt = (p.Lkv + BM - 1) / BM;
    if (p.mask_pres && n_kt <= MASK_PRES_MAX_KT) {
      // from the preparation's presence table: the first and the last 32-row step with a kept pair among this tile's
      // keys (every wave works the same two numbers out for itself)
      const uint8_t* pres = mask_presence(p) + (int64_t)(p.mask_batched ? b : 0) * p.n_qtiles * n_kt + kt;
      int first = 0x7fffffff, last = 0;
      for (int qt_ = lane; qt_ < p.n_qtiles; qt_ += 64) {
        const uint32_t by = pres[(int64_t)qt_ * n_kt];
        if (by) {
          const int a = 4 * qt_ + __builtin_ctz(by), c = 4 * qt_ + 32 - __builtin_clz(by);
          first = a < first ? a : first;
          last = c > last ? c : last;
        }
      }
#pragma unroll
      for (int dl = 32; dl >= 1; dl >>= 1) {
        const int a = __shfl_xor(first, dl, 64), c = __shfl_xor(last, dl, 64);
        first = a < first ? a : first;
        last = c > last ? c : last;
      }
      first = __builtin_amdgcn_readfirstlane(first);
      last = __builtin_amdgcn_readfirstlane(last);
      if (last == 0) {
        hi = lo;                      // nothing kept among these keys
      } else {
        lo = first > lo ? first : lo;
        hi = last < hi ? last : hi;
        hi = hi > lo ? hi : lo;
      }
    } else {
      general_mask_live_steps<false>(p, b, kv0, tid, lo, hi);
    }
    t_lo = lo;
    nt = hi > lo ? hi : lo;
  }
  const int t_wave = p.causal ? r0 / BN : ((win >= 0 && r0 - win > 0) ? (r0 - win) / BN : 0);   // first step with a row that sees a key of this wave
  const int t_wave_end = win >= 0 ? (r0 + 31 + win) / BN : 0x7fffffff / BN;                     // last such step

  const float alpha2 = p.alpha * LOG2E;
  const uint32_t qst_bytes = (uint32_t)p.q_st * 2u, ost_bytes = (uint32_t)p.o_st * 2u;
  const char* wsb = (const char*)p.ws_base;
  const uint32_t pos_off = POS ? (uint32_t)((const char*)(p.pos_scaled + (int64_t)(p.pos_heads > 1 ? h : 0) * (2 * p.L - 1 + 2 * POS_PAD)) - wsb) : 0u;
  const int64_t* tsg = TS ? p.ts + s.ts0 : nullptr;
  const int32_t* trel = TS ? p.ts_rel + ts_rel_base(p, b, s.tok0) : nullptr;
  const int ts32 = TS ? p.ts_ok[b] : 0;
  const uint32_t rel_off = TS ? (uint32_t)((const char*)trel - wsb) : 0u;
  const uint32_t rng_off = TS ? (uint32_t)((const char*)(p.ts_range + 2 * ts_range_slot0(p, b, s.tok0)) - wsb) : 0u;

  auto dma_step = [&](int t) __attribute__((always_inline)) {
    const int st = (t - t_lo) % NST;      // (a pair of steps starts at an even stage)
    const int qbs = t * BN;
    const int last = s.n_q - 1;
#pragma unroll
    for (int r = 0; r < LD; ++r) {
      const int j = (w8 * LD + r) % NPIECE;
      const int c = 64 * j + lane;
      const int row = c / CPR, pc = c - row * CPR;
      int grow = qbs + row;
      grow = grow < last ? grow : last;
      const uint32_t sw = (uint32_t)((pc ^ swz_rt<D>(row)) * 16);
      lds_dma16(qg, (uint32_t)grow * qst_bytes + sw, (const unsigned char*)Qs(st) + j * 1024);
      lds_dma16(dog, (uint32_t)grow * ost_bytes + sw, (const unsigned char*)Os(st) + j * 1024);
    }
    if (POS || TS) {
      // wave c writes position-window copy c: window[x + c], window[x] = pos[(L-1) + kv0 - (qbs+31) + x]
      // (table index >= POS_PAD - 31 > 0); behind the last wave's copy, 36 int32 timestamps from row qbs on
      constexpr int TS_LANE0 = POS ? SM::POS_LANES : 0;
      const bool ts_wave = TS && (!POS || w == NWAVES - 1);
      const int tl = lane - TS_LANE0;
      uint32_t off = 0;
      bool on = false;
      if (POS && lane < SM::POS_LANES) {
        off = pos_off + (uint32_t)(POS_PAD + (p.L - 1) + kv0 - (qbs + BN - 1) + w + 4 * lane) * 4u;
        on = true;
      }
      if (ts_wave && tl >= 0 && tl < TQ_LANES) {
        // the ranges of tiles (tr, tr + 1) cover rows qbs + 1 .. qbs + 32; at the end of the sequence
        // the pair before does (what lies past the last tile only widens the range)
        int tr = t;
        const int tr_last = (s.n_ts - 1) >> 5;
        tr = tr < tr_last ? tr : (tr_last > 0 ? tr_last - 1 : 0);
        off = tl < TQ_LANES - 1 ? rel_off + (uint32_t)(qbs + 4 * tl) * 4u : rng_off + (uint32_t)tr * 8u;
        on = true;
      }
      if (on) lds_dma16(wsb, off, (const unsigned char*)Wc(st) + (POS ? w * SM::POS_COPY : 0));
    }
    if (SEG) {
      // the step's 32 row segment ids (every wave the same load; groups of 4 past the row repeat the last)
      if (lane < BN / 4) {
        int g4 = qbs + 4 * lane;
        g4 = g4 < p.L - 4 ? g4 : p.L - 4;
        lds_dma16_at(p.q_seg + (int64_t)b * p.L, (uint32_t)g4 * 4u, smem_lds + (uint32_t)((const unsigned char*)Sg(st) - smem));
      }
    }
    if (MSK) {
      // rows 8w .. 8w + 7 of the step's mask tile, eight lanes per row (16 bytes each = this tile's 128 keys); rows past
      // L and pieces past Lkv re-read bytes inside the matrix (those pairs are masked by their index)
      const uint8_t* mg = (const uint8_t*)scalar_ptr(p.mask + (p.mask_batched ? (int64_t)b * p.L * p.Lkv : 0));
      int gr = qbs + 8 * w + (lane >> 3);
      gr = gr < p.L - 1 ? gr : p.L - 1;
      int col = kv0 + 16 * (lane & 7);
      col = col < p.Lkv - 16 ? col : p.Lkv - 16;
      lds_dma16(mg, (uint32_t)gr * (uint32_t)p.Lkv + (uint32_t)col, Mk(st) + w * 1024);
    }
    if (DB) {
      // rows 8w .. 8w + 7 of the step's bias tile in four pieces of two rows (512 bytes a row = this tile's 128 keys);
      // rows past L and pieces past Lkv re-read values inside the matrix (those pairs are masked by their index)
      const float* bg = (const float*)scalar_ptr(p.dense_bias + (p.dense_bias_batched ? (int64_t)b * p.L * p.Lkv : 0));
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        int gr = qbs + 8 * w + 2 * r + (lane >> 5);
        gr = gr < p.L - 1 ? gr : p.L - 1;
        int col = kv0 + 4 * (lane & 31);
        col = col < p.Lkv - 4 ? col : p.Lkv - 4;
        lds_dma16(bg, ((uint32_t)gr * (uint32_t)p.Lkv + (uint32_t)col) * 4u, Bk(st) + (4 * w + r) * 1024);
      }
    }
  };

  if (TS) {
    // three direct loads of up to 1 KB, one each by waves 0 to 2 (the last wave repeats the first)
    const int c = w < 3 ? w : 0;
    if (1024 * c + 16 * lane < TS_LDS_BYTES)
      lds_dma16((const unsigned char*)p.ts_keyed + (int64_t)(p.ts_heads > 1 ? h : 0) * (3 * 1024) + 1024 * c, (uint32_t)lane * 16u, TsKey + 1024 * c);
  }
  // the first pairs of steps in flight (the step loop runs in pairs, see there)
#pragma unroll
  for (int i = 0; i < AHEAD; ++i)
    if (t_lo + i < nt) dma_step(t_lo + i);

  // K and V fragments of this lane's key (B operands)
  typedef unsigned uintx4 __attribute__((ext_vector_type(4)));
  uintx4 hs_k[QCH], hs_v[QCH];
  {
    uint4 kfr[QCH], vfr[QCH];
    const char* kp = (const char*)p.k + (s.bk + (int64_t)kcol * p.k_st) * 2 + 16 * hh;
    const char* vp = (const char*)p.v + (s.bv + (int64_t)kcol * p.v_st) * 2 + 16 * hh;
#pragma unroll
    for (int ks = 0; ks < QCH; ++ks) {
      uint4 a = {0u, 0u, 0u, 0u}, c = {0u, 0u, 0u, 0u};
      if (kcol < s.n_kv) { a = *(const uint4*)(kp + 32 * ks); c = *(const uint4*)(vp + 32 * ks); }
      kfr[ks] = a;
      vfr[ks] = c;
    }
#pragma unroll
    for (int ks = 0; ks < QCH; ++ks) {
      asm volatile("" ::"v"(kfr[ks].x), "v"(kfr[ks].y), "v"(kfr[ks].z), "v"(kfr[ks].w));
      asm volatile("" ::"v"(vfr[ks].x), "v"(vfr[ks].y), "v"(vfr[ks].z), "v"(vfr[ks].w));
      hs_k[ks] = uintx4{kfr[ks].x, kfr[ks].y, kfr[ks].z, kfr[ks].w};
      hs_v[ks] = uintx4{vfr[ks].x, vfr[ks].y, vfr[ks].z, vfr[ks].w};
    }
  }
  int32_t kseg = 0;
  if (SEG) {
    kseg = p.kv_seg[(int64_t)b * p.Lkv + (kcol < p.Lkv ? kcol : p.Lkv - 1)];
    asm volatile("" ::"v"(kseg));
  }
  int64_t tk = 0;
  int32_t tk32 = 0;
  if (TS) {
    int ik = kcol < s.n_ts ? kcol : s.n_ts - 1;
    ik = ik < 0 ? 0 : ik;
    tk32 = trel[ik];     // meaningless when !ts32, and then unused
    tk = tsg[ik];
    asm volatile("" ::"v"(tk), "v"(tk32));
  }

  floatx16 dka[DVBW], dva[DVBW];
#pragma unroll
  for (int i = 0; i < DVBW; ++i) {
    if (ACC_ASM) {
      mfma_acc_zero<STREAM>(dka[i]);
      mfma_acc_zero<STREAM>(dva[i]);
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) { dka[i][r] = 0.f; dva[i][r] = 0.f; }
    }
  }

  const int gk = swz_rt<D>(m);
  const int gi = lane & 15;
  const int vrow = 4 * hh + (gi >> 2);
  const int vc2 = 2 * ((lane >> 4) & 1) + ((gi & 3) >> 1);
  const int c_lo = vc2 ^ hh, c_hi = vc2 ^ (hh + 2);

  // One block: 32 query rows against this wave's 32 keys.  Lane (key m, half hh) holds
  // S[q = qbs + 8g + 4hh + tt][kcol], r = 4g + tt.
  auto block = [&](int t) __attribute__((always_inline)) {
    const int st = (t - t_lo) % NST;      // (a pair of steps starts at an even stage)
    const int qbs = t * BN;
    const floatx16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    floatx16 sacc, dpacc;
    {
      uint4 af[QCH];
      const unsigned char* ar = (const unsigned char*)Qs(st) + m * (D * 2);
#pragma unroll
      for (int ks = 0; ks < QCH; ++ks) af[ks] = *(const uint4*)(ar + (((2 * ks + hh) ^ gk) * 16));
#pragma unroll
      for (int ks = 0; ks < QCH; ++ks)
        sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af[ks]), __builtin_bit_cast(bf16x8, hs_k[ks]),
                                                       ks == 0 ? zero : sacc, 0, 0, 0);
    }
    {
      uint4 af[QCH];
      const unsigned char* ar = (const unsigned char*)Os(st) + m * (D * 2);
#pragma unroll
      for (int ks = 0; ks < QCH; ++ks) af[ks] = *(const uint4*)(ar + (((2 * ks + hh) ^ gk) * 16));
#pragma unroll
      for (int ks = 0; ks < QCH; ++ks)
        dpacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af[ks]), __builtin_bit_cast(bf16x8, hs_v[ks]),
                                                        ks == 0 ? zero : dpacc, 0, 0, 0);
    }
    float u[16];
    if (POS) {
      // pair (q = qbs + 8g + 4hh + tt, key): window index 32w + m + 31 - 8g - 4hh - tt; the four tt of a
      // group are four consecutive entries, read as one float4 from the copy that aligns them
      const int a0 = 32 * w + m + 28 - 4 * hh;
      const int sft = a0 & 3;
      const float* wrow = (const float*)((const unsigned char*)Wc(st) + sft * SM::POS_COPY) + (a0 - sft);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float4 bv = *(const float4*)(wrow - 8 * g);
        u[4 * g + 0] = __builtin_fmaf(sacc[4 * g + 0], alpha2, bv.w);
        u[4 * g + 1] = __builtin_fmaf(sacc[4 * g + 1], alpha2, bv.z);
        u[4 * g + 2] = __builtin_fmaf(sacc[4 * g + 2], alpha2, bv.y);
        u[4 * g + 3] = __builtin_fmaf(sacc[4 * g + 3], alpha2, bv.x);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) u[r] = sacc[r] * alpha2;
    }
    if (DB) {
      // the lane's column of the bias tile: row 8g + 4hh + tt at key 32w + m
      const float* bcol = (const float*)Bk(st) + 32 * w + m + (4 * hh) * 128;
#pragma unroll
      for (int r = 0; r < 16; ++r) u[r] = __builtin_fmaf(bcol[(8 * (r >> 2) + (r & 3)) * 128], LOG2E, u[r]);
    }
    if (TS) {
      const int32_t* tqs = Tq(st);
      // row i's logit takes the timestamp of row min(i + 1, last); index into this step's 36
      auto tq_at = [&](int r) {
        int iq = qbs + 8 * (r >> 2) + 4 * hh + (r & 3) + 1;
        iq = iq < s.n_ts - 1 ? iq : s.n_ts - 1;
        return iq < qbs ? qbs : iq;                 // only for rows past the sequence (masked below)
      };
      if (ts32) {
        // the time differences of this lane's key to the step's rows lie between those to the
        // smallest and to the largest timestamp of the two tiles the rows come from
        const int4 rg = *(const int4*)(tqs + 4 * (TQ_LANES - 1));
        const int t_min = rg.x < rg.z ? rg.x : rg.z, t_max = rg.y > rg.w ? rg.y : rg.w;
        const TsEnds en = ts_ends(TsKey, t_min - tk32, t_max - tk32);
        if (__builtin_amdgcn_ballot_w64(!en.same) == 0) {
          const float add = en.v_near;
#pragma unroll
          for (int r = 0; r < 16; ++r) u[r] += add;
        } else if (__builtin_amdgcn_ballot_w64(!en.two) == 0) {
          // one bucket boundary at most: the farther bucket exactly when tq - tk >= thr
          const float add_near = en.v_near, add_far = en.v_far;
#pragma unroll
          for (int r = 0; r < 16; ++r) u[r] += tqs[tq_at(r) - qbs] - tk32 >= en.thr ? add_far : add_near;
        } else {
#pragma unroll
          for (int r = 0; r < 16; ++r) u[r] += ts_value(ts_look(TsKey, tqs[tq_at(r) - qbs] - tk32));
        }
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) u[r] += ts_value(ts_look(TsKey, ts_clip64(tsg[tq_at(r)] - tk)));
      }
    }
    // transposed fragments of dO (for dV) and of Q (for dK)
    uint4 otf[2][DVBW], qtf[2][DVBW];
    {
      const bf16_t* orr = Os(st) + vrow * D + 4 * (gi & 1);
      const bf16_t* qrr = Qs(st) + vrow * D + 4 * (gi & 1);
#pragma unroll
      for (int cc = 0; cc < 2; ++cc)
#pragma unroll
        for (int dvb = 0; dvb < DVBW; ++dvb) {
          const int cb = 4 * ((dh * DVBW + dvb) ^ swz_rt_group<D>(gi));
          uint2 lo = lds_read_tr(orr + (16 * cc) * D + (cb + c_lo) * 8);
          uint2 hi = lds_read_tr(orr + (16 * cc + 8) * D + (cb + c_hi) * 8);
          otf[cc][dvb] = uint4{lo.x, lo.y, hi.x, hi.y};
          lo = lds_read_tr(qrr + (16 * cc) * D + (cb + c_lo) * 8);
          hi = lds_read_tr(qrr + (16 * cc + 8) * D + (cb + c_hi) * 8);
          qtf[cc][dvb] = uint4{lo.x, lo.y, hi.x, hi.y};
        }
    }
    float pv[16], ds[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float fp;
      const float sg = silu_grad_log2(u[r], &fp);
      pv[r] = u[r] * sg;
      ds[r] = dpacc[r] * fp;
    }
    // rows past the sequence hold a repeat of the last row: they are masked like the rest
    if ((p.causal && qbs < r0 + 31) || (qbs + 32 > s.n_q) || (r0 + 32 > s.n_kv) ||
        (win >= 0 && (qbs + 31 - r0 > win || r0 + 31 - qbs > win))) {
      // lo <= qi <= hi for the lane's key; register r holds row qbs + 4hh + c(r), c(r) = 8 (r / 4) + r % 4
      int lo = p.causal ? kcol : (win >= 0 ? kcol - win : 0);
      lo = kcol < s.n_kv ? lo : 0x3fffffff;          // a key past the sequence keeps nothing
      int hi = win >= 0 ? kcol + win : s.n_q - 1;
      hi = hi < s.n_q - 1 ? hi : s.n_q - 1;
      const int lo_rel = lo - qbs - 4 * hh, hi_rel = hi - qbs - 4 * hh;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c = 8 * (r >> 2) + (r & 3);
        const bool keep = c >= lo_rel && c <= hi_rel;
        pv[r] = keep ? pv[r] : 0.f;
        ds[r] = keep ? ds[r] : 0.f;
      }
    }
    if (SEG) {
      const int32_t* sg = Sg(st);
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int4 qs4 = *(const int4*)(sg + 8 * g + 4 * hh);
        const bool k0 = qs4.x == kseg, k1 = qs4.y == kseg, k2 = qs4.z == kseg, k3 = qs4.w == kseg;
        pv[4 * g + 0] = k0 ? pv[4 * g + 0] : 0.f;  ds[4 * g + 0] = k0 ? ds[4 * g + 0] : 0.f;
        pv[4 * g + 1] = k1 ? pv[4 * g + 1] : 0.f;  ds[4 * g + 1] = k1 ? ds[4 * g + 1] : 0.f;
        pv[4 * g + 2] = k2 ? pv[4 * g + 2] : 0.f;  ds[4 * g + 2] = k2 ? ds[4 * g + 2] : 0.f;
        pv[4 * g + 3] = k3 ? pv[4 * g + 3] : 0.f;  ds[4 * g + 3] = k3 ? ds[4 * g + 3] : 0.f;
      }
    }
    if (MSK) {
      // the lane's column of the mask tile: byte of row 8g + 4hh + tt at key 32w + m
      const unsigned char* mcol = Mk(st) + 32 * w + m + (4 * hh) * 128;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const bool keep = mcol[(8 * (r >> 2) + (r & 3)) * 128] != 0;
        pv[r] = keep ? pv[r] : 0.f;
        ds[r] = keep ? ds[r] : 0.f;
      }
    }
    if (p.drop_thr) {
      // dropout: register r holds row qbs + 4hh + c(r) of this lane's key
      drop_apply16(pv, ds, drop_bh_key(p.drop_key, (uint32_t)b * (uint32_t)p.H + (uint32_t)h) + (uint32_t)kcol * DROP_CJ +
                               (uint32_t)(qbs + 4 * hh) * DROP_CI, DROP_CI, p.drop_thr);
    }
#pragma unroll
    for (int cc = 0; cc < 2; ++cc) {
      uint4 pk, dk4;
      pk.x = pack_bf16(pv[8 * cc + 0], pv[8 * cc + 1]);
      pk.y = pack_bf16(pv[8 * cc + 2], pv[8 * cc + 3]);
      pk.z = pack_bf16(pv[8 * cc + 4], pv[8 * cc + 5]);
      pk.w = pack_bf16(pv[8 * cc + 6], pv[8 * cc + 7]);
      dk4.x = pack_bf16(ds[8 * cc + 0], ds[8 * cc + 1]);
      dk4.y = pack_bf16(ds[8 * cc + 2], ds[8 * cc + 3]);
      dk4.z = pack_bf16(ds[8 * cc + 4], ds[8 * cc + 5]);
      dk4.w = pack_bf16(ds[8 * cc + 6], ds[8 * cc + 7]);
      const bf16x8 pb = __builtin_bit_cast(bf16x8, pk), db = __builtin_bit_cast(bf16x8, dk4);
#pragma unroll
      for (int dvb = 0; dvb < DVBW; ++dvb) {
        if (ACC_ASM) {
          mfma_acc<STREAM>(dva[dvb], __builtin_bit_cast(bf16x8, otf[cc][dvb]), pb);
          mfma_acc<STREAM>(dka[dvb], __builtin_bit_cast(bf16x8, qtf[cc][dvb]), db);
        } else {
          dva[dvb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, otf[cc][dvb]), pb, dva[dvb], 0, 0, 0);
          dka[dvb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, qtf[cc][dvb]), db, dka[dvb], 0, 0, 0);
        }
      }
    }
    // The compiler does not know of the matrix instructions above: whatever it puts behind them (a copy of an
    // accumulator at a join of two paths, say) must find the last product's result in place.
    if (ACC_ASM) asm volatile("s_nop 15");
  };

  // (the stream's operands)
  const bool stream_on = STREAM && !p.no_stream && !p.drop_thr && win < 0 && wave_live && r0 + 32 <= s.n_kv;
  const uint32_t hs_a0 = (uint32_t)(m * (D * 2) + ((hh ^ gk) * 16));
  const uint32_t hs_t0 = (uint32_t)(vrow * (D * 2) + 8 * (gi & 1) + 64 * swz_rt_group<D>(gi) + 16 * c_lo);
  const float hs_alpha = alpha2;

  // steps in pairs, one barrier per pair (see the other backward kernel).  Three loops, so that the stream's loop
  // holds nothing of the block code: pairs ahead of the stream's (the diagonal), the stream's, the rest (the
  // sequence's end).  Every wave passes one barrier per pair whichever loop the pair falls into.
  static_assert(NST % 2 == 0 && NST >= 4, "pairs of stages");
  int t_s0 = nt, t_s1 = nt;           // the stream's pairs: [t_s0, t_s1), in steps of 2 from t_lo
  if constexpr (STREAM) {
    if (stream_on) {
      // both blocks whole: every row at or past the wave's last key (causal), inside the sequence
      int first = p.causal ? (r0 + 31 + BN - 1) / BN : 0;
      first = first > t_lo ? first : t_lo;
      first += (first - t_lo) & 1;
      int end = s.n_q / BN;                              // steps [first, end) are whole
      end = end < nt ? end : nt;
      end -= (end - t_lo) & 1;
      if (end > first) { t_s0 = first; t_s1 = end; }
    }
  }
  // a pair's loads go out AHEAD steps before it; at its end the next pair's must have landed, the ones just sent need not
  auto send_ahead = [&](int t) __attribute__((always_inline)) {
    int n = 0;
    if (t + AHEAD < nt) { dma_step(t + AHEAD); ++n; }
    if (t + AHEAD + 1 < nt) { dma_step(t + AHEAD + 1); ++n; }
    return n;
  };
  auto end_of_pair = [&](int n_sent) __attribute__((always_inline)) {
    if (AHEAD == 2 || n_sent == 0) HSTU_WAIT_VMCNT(0);
    else if (n_sent == 1) HSTU_WAIT_VMCNT(NDMA);
    else HSTU_WAIT_VMCNT(2 * NDMA);
    __syncthreads();
  };
  auto block_pair = [&](int t) __attribute__((always_inline)) {
    const int n_sent = send_ahead(t);
    if (wave_live && t >= t_wave && t <= t_wave_end) block(t);
    if (t + 1 < nt && wave_live && t + 1 >= t_wave && t + 1 <= t_wave_end) block(t + 1);
    end_of_pair(n_sent);
  };
  HSTU_WAIT_VMCNT(0);
  __syncthreads();
  int t = t_lo;
  for (; t < nt && t < t_s0; t += 2) block_pair(t);
  if constexpr (STREAM) {
    for (; t < t_s1; t += 2) {
      const int n_sent = send_ahead(t);
      const uint32_t hs_sb = __builtin_amdgcn_readfirstlane(smem_lds + (uint32_t)(((t - t_lo) % NST) * SM::STAGE));
#define HSTU_BWD_STREAM_VARIANT HSTU_BWD_STREAM_PAIR
#include "hstu_bwd_stream_d128.inc"
#undef HSTU_BWD_STREAM_VARIANT
      end_of_pair(n_sent);
    }
  }
  for (; t < nt; t += 2) block_pair(t);

  if (ACC_ASM) asm volatile("s_nop 15\n\ts_nop 15");   // the last product has left the pipeline before its result is read
  unsigned char* ot = smem + w8 * (32 * DW * 2);
  store_rows<DW>(dka, p.alpha * p.inv_n, ot, dkg + dh * DW, p.k_st, r0, s.n_kv, s.rows, lane);
  store_rows<DW>(dva, p.inv_n * (1.0f / LOG2E), ot, dvg + dh * DW, p.v_st, r0, s.n_kv, s.rows, lane);
}

// ---------------------------------------------------------------------------
// Host side: validation, dispatch, C ABI.
// ---------------------------------------------------------------------------

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

enum Variant { V_INVALID = 0, V_GENERAL_F32, V_GENERAL_BF16, V_MFMA_BF16, V_MFMA_FP8 };

// The timestamp bucket law on the host: bucket(dt) = floor(ln(fl32(clip(|dt|, 1, 1e9))) / size), the float
// log and divide of recml/layers/keras/hstu.py:48-55 taken in double.  thr[b] is the smallest clipped
// |dt| whose bucket is >= b (INT32_MAX when 1e9 does not reach b): the integer thresholds that the
// kernels and the CPU oracle share.  `keys` is the part of the matrix-core kernels' keyed table that does
// not depend on the bias values, `keyed_ok` whether that table can represent this bucket size (at most
// one boundary per key range, bucket indices within the backward's histogram).
constexpr int LAW_THR_LEN = 256;
struct BucketLaw {
  float size;
  bool valid, keyed_ok;
  int reach;                       // bucket of 1e9
  int32_t thr[LAW_THR_LEN];
  TsKeys keys;
};
int law_bucket(float f, double size) { return (int)floor(log((double)f) / size); }

const BucketLaw& bucket_law(float size_f) {
  thread_local BucketLaw law = {0.f, false, false, 0, {0}, {{0}, {0}, {0}}};
  if (law.valid && law.size == size_f) return law;
  const double size = (double)size_f;
  law.size = size_f;
  law.reach = law_bucket((float)TS_DT_MAX, size);
  for (int b = 0; b < LAW_THR_LEN; ++b) {
    if (b > law.reach) { law.thr[b] = 0x7fffffff; continue; }
    int64_t lo = 1, hi = TS_DT_MAX;              // bucket(hi) >= b
    while (lo < hi) {
      const int64_t mid = lo + (hi - lo) / 2;
      if (law_bucket((float)mid, size) >= b) hi = mid; else lo = mid + 1;
    }
    law.thr[b] = (int32_t)lo;
  }
  law.keyed_ok = law.reach + 2 < TS_KEYS && law.reach + 2 < LAW_THR_LEN;     // the kernels read thresholds up to bucket reach + 2
  for (int b = 0; b < TS_KEYS; ++b) law.keys.thr_b[b] = b < LAW_THR_LEN ? law.thr[b] : 0x7fffffff;
  for (int key = 0; key < TS_KEYS && law.keyed_ok; ++key) {
    // floats of this key: [f_lo, f_next); the time differences behind them are integers
    uint32_t bits_lo = (uint32_t)(TS_KEY0 + key) << 21, bits_next = (uint32_t)(TS_KEY0 + key + 1) << 21;
    float f_lo, f_next;
    memcpy(&f_lo, &bits_lo, 4);
    memcpy(&f_next, &bits_next, 4);
    float f_first = ceilf(f_lo);                 // first integer-valued float of the range
    if (f_first > (float)TS_DT_MAX) f_first = (float)TS_DT_MAX;
    float f_last = nextafterf(f_next, 0.f);
    if (f_last > (float)TS_DT_MAX) f_last = (float)TS_DT_MAX;
    const int b_lo = law_bucket(f_first, size);
    law.keys.bkt[key] = (uint8_t)b_lo;
    law.keys.thr_f[key] = (float)law.thr[b_lo + 1];      // INT32_MAX becomes 2^31: beyond every clipped difference
    if (f_first < f_next) {
      // at most one boundary inside the key's range; and when there is one, the next key must start in
      // the bucket behind it (the kernels take the value from the threshold on from the next key's entry)
      const int b_last = law_bucket(f_last, size);
      float f_after = ceilf(f_next);
      if (f_after > (float)TS_DT_MAX) f_after = (float)TS_DT_MAX;
      if (b_last > b_lo + 1 || (b_last == b_lo + 1 && key + 1 < TS_KEYS && law_bucket(f_after, size) != b_last)) law.keyed_ok = false;
    }
  }
  law.valid = true;
  return law;
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// The sliding window as the kernels take it: a window that reaches across the whole sequence restricts
// nothing and is passed on as "no window" (the kernels add it to row indices in 32 bits).
int effective_window(const HstuAttnFwdArgs* a) {
  const int longest = a->L > a->Lkv ? a->L : a->Lkv;
  return (a->window >= 0 && a->window < longest) ? a->window : -1;
}

// Whether the matrix-core kernel covers these arguments (dtype aside: bf16, or fp8 q/k).
bool mfma_eligible(const HstuAttnFwdArgs* a) {
  const int kb = a->qk_dtype == HSTU_DTYPE_FP8_E4M3FN ? 1 : 2;   // bytes per q / k element
  const bool d_ok = a->d_qk == a->d_v && (a->d_qk == 32 || a->d_qk == 64 || a->d_qk == 128);
  // segment ids: bf16 only, rows of a multiple of 4 ids (the kernel fetches them four at a time)
  const bool seg_ok = a->mask_mode != HSTU_MASK_SEGMENT ||
                      (kb == 2 && a->L % 4 == 0 && a->Lkv % 4 == 0 && aligned16(a->q_segment_ids) && aligned16(a->kv_segment_ids));
  // a dense bias or mask: bf16, in place of the table biases and the segment ids; whole 16-byte pieces of
  // a row (4 floats, 16 mask bytes) must not straddle its end, and a [L, Lkv] matrix is addressed with 32 bits
  const bool dense = a->mask || a->dense_bias;
  const bool dense_ok = !dense ||
      (kb == 2 && !a->pos_tab && !a->ts_tab && a->mask_mode != HSTU_MASK_SEGMENT &&
       (!a->dense_bias || (a->Lkv % 4 == 0 && aligned16(a->dense_bias))) &&
       (!a->mask || (a->Lkv % 16 == 0 && aligned16(a->mask))) &&
       (int64_t)a->L * a->Lkv * 4 < (1LL << 32));
  // keys and queries of different lengths: the padded layout without the table biases (whose geometry needs one length)
  const bool len_ok = a->L == a->Lkv || (a->layout == HSTU_LAYOUT_PADDED && !a->pos_tab && !a->ts_tab);
  const bool opts_ok = seg_ok && dense_ok && len_ok &&
                       // the keyed bucket table must be able to hold this bucket size (sizes above ln 1.25 = 0.2232)
                       (!a->ts_tab || (a->ts_num_buckets <= 128 && bucket_law(a->ts_bucket_size).keyed_ok));
  auto s8 = [](int64_t x) { return (x & 7) == 0; };
  auto sq = [kb](int64_t x) { return (x * kb & 15) == 0; };
  const bool align_ok = aligned16(a->q) && aligned16(a->k) && aligned16(a->v) && aligned16(a->out) &&
                        sq(a->q_stride_t) && sq(a->q_stride_h) && sq(a->k_stride_t) && sq(a->k_stride_h) &&
                        s8(a->v_stride_t) && s8(a->v_stride_h) && s8(a->o_stride_t) && s8(a->o_stride_h) &&
                        (a->layout == HSTU_LAYOUT_JAGGED ||
                         (sq(a->q_stride_b) && sq(a->k_stride_b) && s8(a->v_stride_b) && s8(a->o_stride_b)));
  // the kernel addresses K and V rows with 32-bit byte offsets from the (sequence, head) base
  const bool off_ok = (int64_t)a->Lkv * a->k_stride_t * kb < (1LL << 31) && (int64_t)a->Lkv * a->v_stride_t * 2 < (1LL << 31) &&
                      a->k_stride_t > 0 && a->v_stride_t > 0;
  return d_ok && opts_ok && align_ok && off_ok;
}

int validate(const HstuAttnFwdArgs* a) {
  if (!a) return fail(HSTU_ERR_NULL, "args is null");
  if (a->struct_size != sizeof(HstuAttnFwdArgs) || a->version != HSTU_ATTN_ABI_VERSION)
    return fail(HSTU_ERR_VERSION, "args struct_size/version (%u/%u) do not match this library (%zu/%d)",
                a->struct_size, a->version, sizeof(HstuAttnFwdArgs), HSTU_ATTN_ABI_VERSION);
  constexpr uint32_t known_flags = HSTU_FWD_WORKSPACE_PREPARED | HSTU_FWD_PREPARE_ONLY | HSTU_FWD_ONE_ITEM_PER_WORKGROUP |
                                   HSTU_FWD_RESIDENT_WORKGROUPS | HSTU_FWD_COMPILER_SCHEDULED_BLOCKS;
  if ((uint32_t)a->flags & ~known_flags) return fail(HSTU_ERR_SHAPE, "unknown bits in flags: 0x%x", (unsigned)a->flags);
  if (!(a->dropout_p >= 0.0f && a->dropout_p < 1.0f)) return fail(HSTU_ERR_SHAPE, "dropout_p must be in [0, 1), got %g", (double)a->dropout_p);
  if (a->reserved0 != 0u) return fail(HSTU_ERR_SHAPE, "reserved0 must be 0");
  const bool empty = a->B == 0 || (a->layout == HSTU_LAYOUT_JAGGED && a->total_tokens == 0);
  if (!empty && (!a->q || !a->k || !a->v || !a->out))
    return fail(HSTU_ERR_NULL, "q, k, v and out must be non-null");
  if (a->B < 0 || a->L < 1 || a->Lkv < 1 || a->H < 1)
    return fail(HSTU_ERR_SHAPE, "bad shape B=%d L=%d Lkv=%d H=%d", a->B, a->L, a->Lkv, a->H);
  if (a->d_qk < 1 || a->d_qk > 256 || a->d_v < 1 || a->d_v > 256)
    return fail(HSTU_ERR_SHAPE, "head dims must be in [1,256], got d_qk=%d d_v=%d", a->d_qk, a->d_v);
  if (a->layout != HSTU_LAYOUT_PADDED && a->layout != HSTU_LAYOUT_JAGGED)
    return fail(HSTU_ERR_SHAPE, "unknown layout %d", a->layout);
  if (a->mask_mode < HSTU_MASK_NONE || a->mask_mode > HSTU_MASK_SEGMENT)
    return fail(HSTU_ERR_SHAPE, "unknown mask_mode %d", a->mask_mode);
  const bool f32 = a->qk_dtype == HSTU_DTYPE_FP32 && a->v_dtype == HSTU_DTYPE_FP32 && a->out_dtype == HSTU_DTYPE_FP32;
  const bool b16 = a->qk_dtype == HSTU_DTYPE_BF16 && a->v_dtype == HSTU_DTYPE_BF16 && a->out_dtype == HSTU_DTYPE_BF16;
  const bool f8 = a->qk_dtype == HSTU_DTYPE_FP8_E4M3FN && a->v_dtype == HSTU_DTYPE_BF16 && a->out_dtype == HSTU_DTYPE_BF16;
  if (!f32 && !b16 && !f8)
    return fail(HSTU_ERR_DTYPE, "unsupported dtype combination qk=%d v=%d out=%d (all fp32, all bf16, or fp8 q/k with bf16 v/out)",
                a->qk_dtype, a->v_dtype, a->out_dtype);
  if (a->layout == HSTU_LAYOUT_JAGGED) {
    if (!a->seq_offsets) return fail(HSTU_ERR_NULL, "jagged layout needs seq_offsets");
    if (a->mask_mode == HSTU_MASK_SEGMENT) return fail(HSTU_ERR_SHAPE, "segment ids need the padded layout");
    if (a->L != a->Lkv) return fail(HSTU_ERR_SHAPE, "jagged layout needs L == Lkv");
    if (a->total_tokens < 0) return fail(HSTU_ERR_SHAPE, "total_tokens < 0");
  } else if (a->mask_mode == HSTU_MASK_LENGTH && !a->seq_lens) {
    return fail(HSTU_ERR_NULL, "LENGTH mask mode needs seq_lens");
  }
  if (a->mask_mode == HSTU_MASK_SEGMENT && (!a->q_segment_ids || !a->kv_segment_ids))
    return fail(HSTU_ERR_NULL, "both or neither of q_segment_ids and kv_segment_ids must be provided");
  if (a->pos_tab) {
    if (a->L != a->Lkv) return fail(HSTU_ERR_SHAPE, "relative-position bias needs L == Lkv");
    if (a->pos_heads != 1 && a->pos_heads != a->H) return fail(HSTU_ERR_SHAPE, "pos_heads must be 1 or H");
  }
  if (a->ts_tab || a->ts) {
    if (!a->ts_tab || !a->ts) return fail(HSTU_ERR_NULL, "timestamp bias needs both ts and ts_tab");
    if (a->L != a->Lkv) return fail(HSTU_ERR_SHAPE, "timestamp bias needs L == Lkv");
    if (a->ts_heads != 1 && a->ts_heads != a->H) return fail(HSTU_ERR_SHAPE, "ts_heads must be 1 or H");
    if (a->ts_num_buckets < 0 || !(a->ts_bucket_size > 0.f))
      return fail(HSTU_ERR_SHAPE, "bad timestamp bucket parameters");
    if (a->ts_stride_b == 0 && a->layout != HSTU_LAYOUT_JAGGED)
      return fail(HSTU_ERR_SHAPE, "jagged timestamps need the jagged layout");
  }
  if (f8 && !mfma_eligible(a))
    return fail(HSTU_ERR_DTYPE, "fp8 q/k runs on the matrix-core kernel only: d_qk == d_v in {32, 64, 128}, q_len == kv_len, "
                "16-byte aligned pointers and row strides, no segment ids, explicit mask or dense bias");
  return HSTU_OK;
}

Variant pick_variant(const HstuAttnFwdArgs* a) {
  if (a->qk_dtype == HSTU_DTYPE_FP32) return V_GENERAL_F32;
  if (mfma_eligible(a)) return a->qk_dtype == HSTU_DTYPE_FP8_E4M3FN ? V_MFMA_FP8 : V_MFMA_BF16;
  return V_GENERAL_BF16;
}

// Workspace of the MFMA kernel: [scaled, padded position table][per-sequence int32-timestamp flag]
// [int32 timestamps][their (min, max) per key tile], each part a multiple of 256 bytes.
struct WorkspacePlan {
  size_t pos_bytes, tab_bytes, ok_bytes, rel_bytes, range_bytes, mrange_bytes, sched_bytes, ctr_bytes, partial_bytes;
  int split_cap;          // chunk slots of the partial buffer (0: no tile is split)
  long long items_max;    // capacity of the work list (0 = no list)
  size_t desc_bytes, tquad_bytes;   // timestamp descriptors and the tiles' stream quads (forward, d = 128; 0 = none)
  long long desc_pitch, desc_tiles; // rows per step of the descriptor table, tile slots
  size_t bias_total() const { return pos_bytes + tab_bytes + ok_bytes + rel_bytes + range_bytes + mrange_bytes + desc_bytes + tquad_bytes; }
  size_t total() const { return bias_total() + sched_bytes + ctr_bytes + partial_bytes; }
};

// Chunk slots the partial buffer is sized for.  A tile is only split when it has more steps than a
// slot's average load, so at most (slots per XCD) tiles per head ask for it, and few do in practice
// (the headline batch: 14 tiles, 28 chunks); tiles beyond the capacity simply stay whole.
constexpr int SPLIT_CAP_DEFAULT = 32;

// max_bytes: a workspace this small must do (the split capacity is cut down to fit it).
WorkspacePlan plan_workspace(const HstuAttnFwdArgs* a, bool allow_split = true, size_t max_bytes = ~(size_t)0, bool want_desc = true) {
  WorkspacePlan w = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const Variant var = pick_variant(a);
  if (var != V_MFMA_BF16 && var != V_MFMA_FP8) return w;
  auto up = [](size_t x) { return (x + 255) / 256 * 256; };
  const int n_qtiles = (a->L + BM - 1) / BM;
  const bool jag = a->layout == HSTU_LAYOUT_JAGGED;
  // A work list built on the device spares the launch of workgroups that would find nothing to do
  // (a jagged batch with a long maximum length and mostly short sequences is mostly such).  Its
  // head mapping needs H to divide 8 or 8 to divide H; its builder is one workgroup.
  // A batch so small that one workgroup per (sequence, head, query tile) fits the chip at once, with tiles of at
  // most 16 steps, goes without: nothing is left to order or to balance, no tile is long enough for a split to pay
  // for its partial sums, and building the list would cost the call more than the kernel gains by it (measured:
  // 32 sequences of up to 512 tokens, 4 heads, d = 64: the call 28.7 -> 20.3 us, the kernel alone 19.6 -> 17.8).
  const bool small = (long long)a->B * n_qtiles * a->H <= (a->d_qk > 64 ? 512 : 1024) && a->Lkv <= 16 * BN;
  const bool list = (a->H % 8 == 0 || 8 % a->H == 0) && a->B <= 8192 && !small;
  // Key-range splitting (decided per tile by the preparation kernel, which sees the lengths) needs the list.
  // (no tile of at most 8 steps is ever split; a tile takes at most MAX_CHUNKS slots)
  const long long t128_all = jag ? a->total_tokens / BM + a->B : (long long)a->B * n_qtiles;
  if (list && allow_split && effective_window(a) < 0 && (a->Lkv + BN - 1) / BN > 8)
    w.split_cap = (int)(t128_all * MAX_CHUNKS < SPLIT_CAP_DEFAULT ? t128_all * MAX_CHUNKS : SPLIT_CAP_DEFAULT);
  if (a->pos_tab) w.pos_bytes = up((size_t)a->pos_heads * (size_t)(2 * a->L - 1 + 2 * POS_PAD) * sizeof(float));
  if (a->ts_tab) {
    const size_t tiles_per_seq = (size_t)((a->L + BN - 1) / BN);
    const bool by_token = a->ts_stride_b == 0;
    const size_t n_ts = by_token ? (size_t)a->total_tokens : (size_t)a->B * (size_t)a->L;
    const size_t tiles = by_token ? (size_t)(a->total_tokens >> 5) + (size_t)a->B + tiles_per_seq : (size_t)a->B * tiles_per_seq;
    w.tab_bytes = up((size_t)a->ts_heads * 3 * 1024);   // the bucket tables (three direct loads of 1 KB per head)
    w.ok_bytes = up((size_t)a->B * sizeof(int32_t));
    // the kernels fetch whole 16-byte pieces: up to 35 timestamps and one range past the end
    w.rel_bytes = up(n_ts * sizeof(int32_t) + 160);
    w.range_bytes = up(tiles * 2 * sizeof(int32_t) + 16);
  }
  // (behind the ranges: per (mask batch, query tile, key tile of 128) one byte, see mask_presence)
  if (a->mask) w.mrange_bytes = up((size_t)(a->mask_batched ? a->B : 1) * (size_t)n_qtiles * (2 * sizeof(int32_t) + (size_t)((a->Lkv + BM - 1) / BM)));
  // Timestamp descriptors: the forward at d = 128 in bf16 under the causal mask with lengths (what the descriptor
  // kernel's LDS holds; tables small enough to be worth their memory), when the caller's workspace has the room.
  if (want_desc && a->ts_tab && var == V_MFMA_BF16 && a->d_qk == 128 && a->causal && effective_window(a) < 0 && a->L == a->Lkv &&
      a->L <= TS_DESC_MAX_L && !a->mask && !a->dense_bias && (jag || a->mask_mode != HSTU_MASK_SEGMENT)) {
    const long long rows = jag ? 8 * ((a->total_tokens >> 3) + a->B) + BM : (long long)a->B * ((a->L + 7) & ~7) + BM;
    const long long steps = (a->L + BN - 1) / BN;
    const size_t bytes = up((size_t)rows * (size_t)steps * sizeof(uint16_t));
    if (bytes <= ((size_t)256 << 20)) {
      w.desc_pitch = rows;
      w.desc_tiles = jag ? (a->total_tokens >> 7) + a->B + 1 : (long long)a->B * n_qtiles;
      w.desc_bytes = bytes;
      w.tquad_bytes = up((size_t)w.desc_tiles * (size_t)ts_desc_chunks(a->L) * sizeof(int32_t));
    }
  }
  const long long t128 = jag ? a->total_tokens / BM + a->B : (long long)a->B * n_qtiles;
  const size_t chunk_bytes = (size_t)a->H * (size_t)BM * (size_t)a->d_v * sizeof(float);
  for (;;) {
    if (list) {
      w.items_max = t128 + w.split_cap;     // every tile one item, and one more per chunk slot at most
      w.sched_bytes = up((size_t)(4 + 4 * w.items_max) * sizeof(int32_t));
    }
    w.ctr_bytes = list ? up((size_t)(CTR_RESERVED + (size_t)w.split_cap * a->H) * sizeof(uint32_t)) : 0;
    w.partial_bytes = up((size_t)w.split_cap * chunk_bytes);
    if (w.total() <= max_bytes) break;
    if (w.split_cap == 0) {
      // still too large without any chunk slot: the descriptors go (every block then looks its pairs up)
      if (!w.desc_bytes) break;
      w.desc_bytes = w.tquad_bytes = 0; w.desc_pitch = w.desc_tiles = 0;
      continue;
    }
    const size_t over = w.total() - max_bytes;
    const int fewer = (int)((over + chunk_bytes - 1) / chunk_bytes);
    w.split_cap = w.split_cap - fewer >= 2 ? w.split_cap - fewer : 0;
  }
  return w;
}

Params make_params(const HstuAttnFwdArgs* a) {
  Params p;
  memset(&p, 0, sizeof(p));
  p.q = a->q; p.k = a->k; p.v = a->v; p.out = a->out;
  p.q_sb = a->q_stride_b; p.q_st = a->q_stride_t; p.q_sh = a->q_stride_h;
  p.k_sb = a->k_stride_b; p.k_st = a->k_stride_t; p.k_sh = a->k_stride_h;
  p.v_sb = a->v_stride_b; p.v_st = a->v_stride_t; p.v_sh = a->v_stride_h;
  p.o_sb = a->o_stride_b; p.o_st = a->o_stride_t; p.o_sh = a->o_stride_h;
  p.seq_lens = a->seq_lens; p.seq_offsets = a->seq_offsets;
  p.q_seg = a->q_segment_ids; p.kv_seg = a->kv_segment_ids;
  p.mask = a->mask; p.dense_bias = a->dense_bias;
  p.pos_tab = a->pos_tab; p.ts_tab = a->ts_tab; p.ts = a->ts; p.ts_sb = a->ts_stride_b;
  p.B = a->B; p.L = a->L; p.Lkv = a->Lkv; p.H = a->H; p.d_qk = a->d_qk; p.d_v = a->d_v;
  p.jagged = a->layout == HSTU_LAYOUT_JAGGED;
  p.causal = a->causal != 0;
  p.mask_mode = p.jagged ? HSTU_MASK_LENGTH : a->mask_mode;
  p.window = effective_window(a);
  p.mask_batched = a->mask_batched; p.dense_bias_batched = a->dense_bias_batched;
  p.pos_heads = a->pos_heads; p.ts_heads = a->ts_heads;
  p.ts_nb = a->ts_num_buckets;
  p.ts_bucket_size = a->ts_bucket_size;
  p.alpha = a->alpha; p.inv_n = a->inv_n;
  p.drop_thr = drop_threshold(a->dropout_p);
  p.drop_key = drop_seed_key(a->dropout_seed);
  if (p.drop_thr) p.inv_n = a->inv_n / (1.0f - a->dropout_p);     // the survivors' scale rides on 1 / N
  p.q_scale = a->q_scale; p.k_scale = a->k_scale;
  p.n_qtiles = (a->L + BM - 1) / BM;
  return p;
}

// Raises the dynamic-LDS limit of a kernel once per device (the attribute is
// sticky; asking again on every launch would only cost host time).
int allow_lds(const void* fn, int bytes, int* granted /* [kMaxDev] */) {
  constexpr int kMaxDev = 64;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev >= 0 && dev < kMaxDev && __atomic_load_n(&granted[dev], __ATOMIC_ACQUIRE) >= bytes) return HSTU_OK;
  e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "hipFuncSetAttribute(%d bytes of LDS): %s", bytes, hipGetErrorString(e));
  if (dev >= 0 && dev < kMaxDev) __atomic_store_n(&granted[dev], bytes, __ATOMIC_RELEASE);
  return HSTU_OK;
}

template <typename T>
int launch_general(const Params& p, hipStream_t st) {
  const bool small = p.d_qk <= 128 && p.d_v <= 128;
  if (p.B > 65535 || (p.L + 127) / 128 > 65535)
    return fail(HSTU_ERR_SHAPE, "the general kernel takes at most 65535 sequences and 65535 tiles of 128 rows per call (B = %d, L = %d)", p.B, p.L);
  const size_t smem = sizeof(float) * ((size_t)GT * general_pitch_qk(p.d_qk) + (size_t)GT * general_pitch_v(p.d_v));
  static int granted_small[64], granted_large[64];
  if (int rc = small ? allow_lds((const void*)hstu_fwd_general<T, 128>, (int)smem, granted_small)
                     : allow_lds((const void*)hstu_fwd_general<T, 256>, (int)smem, granted_large)) return rc;
  hipError_t e;
  dim3 grid(p.H, p.B, (p.L + 127) / 128);
  {
    auto whole = [&](const void* base, int64_t row, int64_t head, int64_t batch) {
      return ((uintptr_t)base & (4 * sizeof(T) - 1)) == 0 && ((row | head | batch) & 3) == 0;
    };
    const bool words = (!p.mask || ((p.Lkv & 3) == 0 && ((uintptr_t)p.mask & 3) == 0)) &&
                       (!p.dense_bias || ((p.Lkv & 3) == 0 && ((uintptr_t)p.dense_bias & 15) == 0));
    if (small && p.pos_tab == nullptr && p.ts_tab == nullptr && words && (p.d_qk & 3) == 0 && (p.d_v & 3) == 0 &&
        whole(p.k, p.k_st, p.k_sh, p.k_sb) && whole(p.v, p.v_st, p.v_sh, p.v_sb)) {
      static int granted_lean[64];
      if (int rc = allow_lds((const void*)hstu_fwd_general<T, 128, false>, (int)smem, granted_lean)) return rc;
      hipLaunchKernelGGL((hstu_fwd_general<T, 128, false>), grid, dim3(256), smem, st, p);
      e = hipGetLastError();
      if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "general kernel launch: %s", hipGetErrorString(e));
      return HSTU_OK;
    }
  }
  if (small) hipLaunchKernelGGL((hstu_fwd_general<T, 128>), grid, dim3(256), smem, st, p);
  else hipLaunchKernelGGL((hstu_fwd_general<T, 256>), grid, dim3(256), smem, st, p);
  e = hipGetLastError();
  if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "general kernel launch: %s", hipGetErrorString(e));
  return HSTU_OK;
}

// Workgroups of the main kernel.
long long mfma_grid(const Params& p) {
  if (p.sched) {
    const long long n = p.items_max;
    if (p.mask || p.dense_bias) {
      const long long groups = (n + p.n_qtiles - 1) / p.n_qtiles;     // runs of n_qtiles items, eight runs a round
      return 8LL * ((groups + 7) / 8) * p.n_qtiles * p.H;
    }
    const long long rounds = p.H >= 8 ? n * (p.H / 8) : (n + 8 / p.H - 1) / (8 / p.H);
    return 8LL * rounds;
  }
  return 8LL * p.n_qtiles * (((long long)p.B * p.H + 7) / 8);
}

// Whether a bf16 call of the general backward takes its products to the bf16 matrix cores: head dims up to 128
// in multiples of 16, every row of q, k, v and dout on a 16-byte boundary.
bool general_bwd_bf16_products(const Params& p) {
  auto rows16 = [](const void* base, int64_t row, int64_t head, int64_t batch) {
    return ((uintptr_t)base & 15u) == 0 && ((row | head | batch) & 7) == 0;
  };
  return p.d_qk <= 128 && p.d_v <= 128 && (p.d_qk & 15) == 0 && (p.d_v & 15) == 0 && rows16(p.q, p.q_st, p.q_sh, p.q_sb) &&
         rows16(p.k, p.k_st, p.k_sh, p.k_sb) && rows16(p.v, p.v_st, p.v_sh, p.v_sb) && rows16(p.dout, p.o_st, p.o_sh, p.o_sb);
}

// The general backward: head dims up to 128 on the matrix cores (fp32 products; bf16 products for bf16 storage
// where the rows allow), larger ones by the FMA kernels.
template <typename T>
int launch_bwd(const Params& p, hipStream_t st) {
  if (p.B > 65535) return fail(HSTU_ERR_SHAPE, "the general backward takes at most 65535 sequences per call, got %d", p.B);
  if (p.d_qk <= 128 && p.d_v <= 128) {
    // (each wave's block of dS goes through LDS for the position table's diagonal sums and for the dense bias's row-wise adds)
    const bool want_pos = (p.dpos != nullptr && p.pos_tab != nullptr) || p.dbias != nullptr;
    const int smem_q = 4 * general_bwd_dq_lds(p.d_qk, p.d_v, want_pos, p.ts_nb), smem_kv = 4 * general_bwd_dkv_lds(p.d_qk, p.d_v);
    if constexpr (sizeof(T) == 2) {
      // bf16 storage whose rows can be fetched 16 bytes at a time: the products on the bf16 matrix cores
      if (general_bwd_bf16_products(p)) {
        const int smem_qb = general_bwd_dq_lds_bf16(p.d_qk, p.d_v, want_pos, p.ts_nb), smem_kvb = general_bwd_dkv_lds_bf16(p.d_qk, p.d_v);
        static int granted_qb[64], granted_kvb[64], granted_qn[64], granted_kvn[64];
        const bool tables = p.pos_tab != nullptr || p.ts_tab != nullptr;
        const dim3 grid_q(p.H, p.B, (p.L + 127) / 128), grid_kv(p.H, p.B, (p.Lkv + 127) / 128);
        const bool words = (!p.mask || ((p.Lkv & 3) == 0 && ((uintptr_t)p.mask & 3) == 0)) &&
                           (!p.dense_bias || ((p.Lkv & 3) == 0 && ((uintptr_t)p.dense_bias & 15) == 0));
        if (!tables && words) {
          // no bias tables (the layer's dense operands, or no bias at all): instances without the tables' code,
          // which fit two workgroups per CU
          if (int rc = allow_lds((const void*)hstu_bwd_dq_mm<T, true, false>, smem_qb, granted_qn)) return rc;
          if (int rc = allow_lds((const void*)hstu_bwd_dkv_mm<T, true, false>, smem_kvb, granted_kvn)) return rc;
          hipLaunchKernelGGL((hstu_bwd_dq_mm<T, true, false>), grid_q, dim3(256), smem_qb, st, p);
          hipError_t e = hipGetLastError();
          if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dq kernel launch: %s", hipGetErrorString(e));
          hipLaunchKernelGGL((hstu_bwd_dkv_mm<T, true, false>), grid_kv, dim3(256), smem_kvb, st, p);
          e = hipGetLastError();
          if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dk/dv kernel launch: %s", hipGetErrorString(e));
          return HSTU_OK;
        }
        if (int rc = allow_lds((const void*)hstu_bwd_dq_mm<T, true>, smem_qb, granted_qb)) return rc;
        if (int rc = allow_lds((const void*)hstu_bwd_dkv_mm<T, true>, smem_kvb, granted_kvb)) return rc;
        hipLaunchKernelGGL((hstu_bwd_dq_mm<T, true>), grid_q, dim3(256), smem_qb, st, p);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dq kernel launch: %s", hipGetErrorString(e));
        hipLaunchKernelGGL((hstu_bwd_dkv_mm<T, true>), grid_kv, dim3(256), smem_kvb, st, p);
        e = hipGetLastError();
        if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dk/dv kernel launch: %s", hipGetErrorString(e));
        return HSTU_OK;
      }
    }
    if constexpr (sizeof(T) == 4) {
      // fp32 calls without bias tables whose rows, mask and dense bias can be fetched whole: instances with those
      // fetches fixed at compile time (none of the tables' code, none of the element-wise fallbacks)
      auto whole = [&](const void* base, int64_t row, int64_t head, int64_t batch) {
        return ((uintptr_t)base & 15u) == 0 && ((row | head | batch) & 3) == 0;
      };
      const bool words = (!p.mask || ((p.Lkv & 3) == 0 && ((uintptr_t)p.mask & 3) == 0)) &&
                         (!p.dense_bias || ((p.Lkv & 3) == 0 && ((uintptr_t)p.dense_bias & 15) == 0));
      if (p.pos_tab == nullptr && p.ts_tab == nullptr && words && (p.d_qk & 3) == 0 && (p.d_v & 3) == 0 &&
          whole(p.q, p.q_st, p.q_sh, p.q_sb) && whole(p.k, p.k_st, p.k_sh, p.k_sb) && whole(p.v, p.v_st, p.v_sh, p.v_sb) &&
          whole(p.dout, p.o_st, p.o_sh, p.o_sb)) {
        static int granted_ql[64], granted_kvl[64];
        if (int rc = allow_lds((const void*)hstu_bwd_dq_mm<T, false, false>, smem_q, granted_ql)) return rc;
        if (int rc = allow_lds((const void*)hstu_bwd_dkv_mm<T, false, false>, smem_kv, granted_kvl)) return rc;
        hipLaunchKernelGGL((hstu_bwd_dq_mm<T, false, false>), dim3(p.H, p.B, (p.L + 127) / 128), dim3(256), smem_q, st, p);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dq kernel launch: %s", hipGetErrorString(e));
        hipLaunchKernelGGL((hstu_bwd_dkv_mm<T, false, false>), dim3(p.H, p.B, (p.Lkv + 127) / 128), dim3(256), smem_kv, st, p);
        e = hipGetLastError();
        if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dk/dv kernel launch: %s", hipGetErrorString(e));
        return HSTU_OK;
      }
    }
    static int granted_q[64], granted_kv[64];
    if (int rc = allow_lds((const void*)hstu_bwd_dq_mm<T>, smem_q, granted_q)) return rc;
    if (int rc = allow_lds((const void*)hstu_bwd_dkv_mm<T>, smem_kv, granted_kv)) return rc;
    hipLaunchKernelGGL(hstu_bwd_dq_mm<T>, dim3(p.H, p.B, (p.L + 127) / 128), dim3(256), smem_q, st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dq kernel launch: %s", hipGetErrorString(e));
    hipLaunchKernelGGL(hstu_bwd_dkv_mm<T>, dim3(p.H, p.B, (p.Lkv + 127) / 128), dim3(256), smem_kv, st, p);
    e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dk/dv kernel launch: %s", hipGetErrorString(e));
    return HSTU_OK;
  }
  const size_t tile = (size_t)GT * p.d_qk + (size_t)GT * p.d_v + (size_t)GT * (p.d_qk + 1) + (size_t)GT * (p.d_v + 1);
  const size_t smem_q = sizeof(float) * (tile + GT * (GT + 1) + general_hist_len(p.ts_nb) + GT * GT);
  const size_t smem_kv = sizeof(float) * (tile + 2 * GT * (GT + 1));
  static int granted_q[64], granted_kv[64];
  if (int rc = allow_lds((const void*)hstu_bwd_dq<T>, (int)smem_q, granted_q)) return rc;
  if (int rc = allow_lds((const void*)hstu_bwd_dkv<T>, (int)smem_kv, granted_kv)) return rc;
  if (p.B > 65535 || (p.L + GT - 1) / GT > 65535 || (p.Lkv + GT - 1) / GT > 65535)
    return fail(HSTU_ERR_SHAPE, "the general backward takes at most 65535 sequences and 65535 tiles of 32 rows per call");
  hipLaunchKernelGGL(hstu_bwd_dq<T>, dim3(p.H, p.B, (p.L + GT - 1) / GT), dim3(256), smem_q, st, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dq kernel launch: %s", hipGetErrorString(e));
  hipLaunchKernelGGL(hstu_bwd_dkv<T>, dim3(p.H, p.B, (p.Lkv + GT - 1) / GT), dim3(256), smem_kv, st, p);
  e = hipGetLastError();
  if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dk/dv kernel launch: %s", hipGetErrorString(e));
  return HSTU_OK;
}

template <int D, bool POS, bool TS, bool F8, bool SEG = false, int DENSE = 0, bool PERSIST = false>
int launch_mfma_inst(const Params& p, hipStream_t st) {
  const int smem = MfmaSmem<D, F8 ? 1 : 2>::total(POS, TS, SEG, DENSE, fwd_stages(D, DENSE)) + FWD_XCH_BYTES +
                   (fwd_takes_ts_desc(D, TS, F8, SEG, DENSE) ? fwd_stages(D, DENSE) * NWAVES * 64 : 0);
  static int granted[64];
  if (int rc = allow_lds((const void*)hstu_fwd_mfma_bf16<D, POS, TS, F8, SEG, DENSE, PERSIST>, smem, granted)) return rc;
  hipError_t e;
  long long blocks = mfma_grid(p);
  // resident workgroups: as many as run at once, fewer when the list cannot be longer than that
  if (PERSIST && blocks > 8LL * p.n_slots) blocks = 8LL * p.n_slots;
  if (blocks > 0x7fffffffLL) return fail(HSTU_ERR_SHAPE, "grid too large");
  hipLaunchKernelGGL((hstu_fwd_mfma_bf16<D, POS, TS, F8, SEG, DENSE, PERSIST>), dim3((unsigned)blocks), dim3(MFMA_THREADS), smem, st, p);
  e = hipGetLastError();
  if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "mfma kernel launch: %s", hipGetErrorString(e));
  return HSTU_OK;
}

template <int D, bool F8>
int launch_mfma_d(const Params& p, hipStream_t st) {
  const bool pos = p.pos_tab != nullptr, ts = p.ts_tab != nullptr;
  if (!F8 && (p.mask || p.dense_bias)) {
    if (p.mask && p.dense_bias) return launch_mfma_inst<D, false, false, false, false, 3>(p, st);
    if (p.mask) return launch_mfma_inst<D, false, false, false, false, 2>(p, st);
    return launch_mfma_inst<D, false, false, false, false, 1>(p, st);
  }
  if (!F8 && p.mask_mode == HSTU_MASK_SEGMENT) {
    if (pos && ts) return launch_mfma_inst<D, true, true, false, true>(p, st);
    if (pos) return launch_mfma_inst<D, true, false, false, true>(p, st);
    if (ts) return launch_mfma_inst<D, false, true, false, true>(p, st);
    return launch_mfma_inst<D, false, false, false, true>(p, st);
  }
  if constexpr (D == 128 && !F8) {
    if (p.persist) {
      if (pos && ts) return launch_mfma_inst<D, true, true, false, false, 0, true>(p, st);
      if (pos) return launch_mfma_inst<D, true, false, false, false, 0, true>(p, st);
      if (ts) return launch_mfma_inst<D, false, true, false, false, 0, true>(p, st);
      return launch_mfma_inst<D, false, false, false, false, 0, true>(p, st);
    }
  }
  if (pos && ts) return launch_mfma_inst<D, true, true, F8>(p, st);
  if (pos) return launch_mfma_inst<D, true, false, F8>(p, st);
  if (ts) return launch_mfma_inst<D, false, true, F8>(p, st);
  return launch_mfma_inst<D, false, false, F8>(p, st);
}

// HSTU_ONLY_D128: a development build that compiles the d = 128 instances only (a quarter of the
// compile time); other head dims then report an error instead of running.
template <bool F8>
int launch_mfma(const Params& p, hipStream_t st) {
  if (p.d_qk == 128) return launch_mfma_d<128, F8>(p, st);
#ifndef HSTU_ONLY_D128
  if (p.d_qk == 64) return launch_mfma_d<64, F8>(p, st);
  return launch_mfma_d<32, F8>(p, st);
#else
  return fail(HSTU_ERR_SHAPE, "development build: d = 128 only");
#endif
}


// Workgroups of the forward kernel that run at once on one XCD (an eighth of the chip): what the
// preparation kernel balances the split of long tiles for.  Two workgroups per compute unit at
// d = 128, four below, one with dense operands; the count of compute units is read once per device.
int slots_per_xcd(const Params& p, int32_t* out) {
  constexpr int kMaxDev = 64;
  static int cus[kMaxDev];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  int n = (dev >= 0 && dev < kMaxDev) ? __atomic_load_n(&cus[dev], __ATOMIC_ACQUIRE) : 0;
  if (n <= 0) {
    e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess || n <= 0) return fail(HSTU_ERR_LAUNCH, "hipDeviceGetAttribute(multiprocessor count): %s", hipGetErrorString(e));
    if (dev >= 0 && dev < kMaxDev) __atomic_store_n(&cus[dev], n, __ATOMIC_RELEASE);
  }
  // (by registers and LDS: with dense operands the d = 64 kernel takes 153 registers, three waves per SIMD)
  const bool dense = p.mask || p.dense_bias;
  const int per_cu = p.d_qk > 64 ? 2 : (dense && p.d_qk > 32 ? 3 : 4);
  const int slots = n * per_cu / 8;
  *out = slots > 0 ? slots : 1;
  return HSTU_OK;
}

// Points the workspace fields of `q` into the caller's buffer as `ws` lays it out and enqueues the
// kernel that fills it (unless the caller says it is filled already).
int setup_workspace(const HstuAttnFwdArgs* args, const WorkspacePlan& ws, Params& q, hipStream_t st) {
  q.split_cap = ws.split_cap;
  if (!ws.total()) return HSTU_OK;
  if (!args->workspace || args->workspace_bytes < ws.total())
    return fail(HSTU_ERR_WORKSPACE, "workspace of %zu bytes needed (see hstu_attn_fwd_workspace_bytes), got %zu",
                ws.total(), args->workspace ? args->workspace_bytes : (size_t)0);
  if (((uintptr_t)args->workspace & 255u) != 0) return fail(HSTU_ERR_WORKSPACE, "workspace must be 256-byte aligned");
  char* base = (char*)args->workspace;
  if (ws.bias_total() >= (1ull << 32)) return fail(HSTU_ERR_WORKSPACE, "workspace of %zu bytes is beyond what the kernel addresses", ws.bias_total());
  float* pos_out = ws.pos_bytes ? (float*)base : nullptr;
  int4* tab_out = ws.tab_bytes ? (int4*)(base + ws.pos_bytes) : nullptr;
  int32_t* ok_out = ws.ok_bytes ? (int32_t*)(base + ws.pos_bytes + ws.tab_bytes) : nullptr;
  int32_t* rel_out = (int32_t*)(base + ws.pos_bytes + ws.tab_bytes + ws.ok_bytes);
  int32_t* range_out = (int32_t*)(base + ws.pos_bytes + ws.tab_bytes + ws.ok_bytes + ws.rel_bytes);
  int32_t* mrange_out = ws.mrange_bytes ? (int32_t*)(base + ws.pos_bytes + ws.tab_bytes + ws.ok_bytes + ws.rel_bytes + ws.range_bytes) : nullptr;
  q.mask_range = mrange_out;
  q.ws_base = base;
  uint16_t* desc_out = ws.desc_bytes ? (uint16_t*)(base + ws.pos_bytes + ws.tab_bytes + ws.ok_bytes + ws.rel_bytes + ws.range_bytes + ws.mrange_bytes) : nullptr;
  int32_t* tquad_out = ws.desc_bytes ? (int32_t*)((char*)desc_out + ws.desc_bytes) : nullptr;
  q.ts_desc = desc_out;
  q.ts_tquads = tquad_out;
  q.ts_desc_pitch = (int32_t)ws.desc_pitch;
  q.ts_desc_tiles = (int32_t)ws.desc_tiles;
  q.ts_desc_chunks = ts_desc_chunks(q.L);
  int32_t* sched_out = ws.sched_bytes ? (int32_t*)(base + ws.bias_total()) : nullptr;
  q.sched = sched_out;
  q.items_max = ws.items_max;
  q.ctr = ws.ctr_bytes ? (uint32_t*)(base + ws.bias_total() + ws.sched_bytes) : nullptr;
  q.partial = ws.partial_bytes ? (float*)(base + ws.bias_total() + ws.sched_bytes + ws.ctr_bytes) : nullptr;
  if (int rc = slots_per_xcd(q, &q.n_slots)) return rc;
  q.ts_keyed = tab_out;
  q.pos_scaled = pos_out;
  q.ts_ok = ok_out;
  q.ts_rel = rel_out;
  q.ts_range = range_out;
  const long long blocks_pos = ws.pos_bytes ? ((long long)q.pos_heads * (2 * q.L - 1 + 2 * POS_PAD) + 255) / 256 : 0;
  const long long blocks_ts = ws.ok_bytes ? q.B : 0;
  long long blocks = blocks_pos > blocks_ts ? blocks_pos : blocks_ts;
  const long long blocks_mask = ws.mrange_bytes ? (long long)(q.mask_batched ? q.B : 1) * q.n_qtiles : 0;
  blocks = blocks > blocks_mask ? blocks : blocks_mask;
  blocks = blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks);
  if (ws.sched_bytes) ++blocks;   // the last workgroup builds the work lists
  if ((ws.bias_total() || ws.sched_bytes) && (!(args->flags & HSTU_FWD_WORKSPACE_PREPARED) || (args->flags & HSTU_FWD_PREPARE_ONLY))) {
    static const TsKeys no_keys = {{0}, {0}, {0}};
    const TsKeys& keys = tab_out ? bucket_law(q.ts_bucket_size).keys : no_keys;
    // (the descriptors: one more workgroup per tile slot and chunk of steps, behind the others)
    const int n_chunks = ts_desc_chunks(q.L);
    const long long desc_blocks = desc_out ? (long long)ws.desc_tiles * n_chunks : 0;
    hipLaunchKernelGGL(hstu_prepare, dim3((unsigned)(blocks + desc_blocks)), dim3(256), 0, st, q, pos_out, tab_out, ok_out, rel_out, range_out,
                       sched_out, mrange_out, desc_out, tquad_out, (int)blocks, n_chunks, keys);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "prepare kernel launch: %s", hipGetErrorString(e));
  }
  return HSTU_OK;
}

// The matrix-core backward: bf16 under the conditions of the matrix-core forward, 16-byte aligned
// gradient buffers, and the forward's workspace at hand.
bool bwd_mfma_eligible(const HstuAttnBwdArgs* b) {
  HstuAttnFwdArgs f = b->fwd;
  f.out = (void*)b->dout;
  if (f.qk_dtype != HSTU_DTYPE_BF16 || !mfma_eligible(&f)) return false;
  // keys and queries of different lengths: the general pair.  A dense keep-mask and a dense bias are taken
  // (mfma_eligible has checked their rows: whole 16-byte pieces, aligned, no table bias, no segment ids).
  if (f.L != f.Lkv) return false;
  if (!aligned16(b->dq) || !aligned16(b->dk) || !aligned16(b->dv)) return false;
  // q rows are addressed with 32-bit byte offsets here, like k and v rows in the forward
  if ((int64_t)f.L * f.q_stride_t * 2 >= (1LL << 31) || (int64_t)f.L * f.o_stride_t * 2 >= (1LL << 31) ||
      f.q_stride_t <= 0 || f.o_stride_t <= 0) return false;
  const WorkspacePlan ws = plan_workspace(&f, false, ~(size_t)0, false);
  return ws.total() == 0 || (f.workspace && f.workspace_bytes >= ws.total() && ((uintptr_t)f.workspace & 255u) == 0);
}

template <int D, bool POS, bool TS, bool TG, bool SEG = false, bool MSK = false, bool DB = false>
int launch_bwd_mfma_inst(const Params& p, hipStream_t st) {
  const int smem = MfmaSmem<D, 2>::total(POS, TS, SEG) + (MSK ? NSTAGE * MfmaSmem<D, 2>::DM_BYTES : 0) +
                   (DB ? NSTAGE * MfmaSmem<D, 2>::DB_BYTES : 0);
  const int smem_q = smem + (TG ? BWD_TG_BYTES : 0);
  constexpr int nst_kv = dkv_stages(D, DB);
  const int smem_kv = MfmaSmem<D, 2>::total(POS, TS, SEG, 0, nst_kv) + (MSK ? nst_kv * MfmaSmem<D, 2>::DM_BYTES : 0) +
                      (DB ? nst_kv * MfmaSmem<D, 2>::DB_BYTES : 0) +
                      (TS ? nst_kv * 16 : 0);     // one more 16-byte piece of timestamp operands per stage
  static int granted_q[64], granted_kv[64];
  if (int rc = allow_lds((const void*)hstu_bwd_dq_mfma<D, POS, TS, TG, SEG, MSK, DB>, smem_q, granted_q)) return rc;
  if (int rc = allow_lds((const void*)hstu_bwd_dkv_mfma<D, POS, TS, SEG, MSK, DB>, smem_kv, granted_kv)) return rc;
  const long long blocks = mfma_grid(p);
  if (blocks > 0x7fffffffLL) return fail(HSTU_ERR_SHAPE, "grid too large");
  hipLaunchKernelGGL((hstu_bwd_dq_mfma<D, POS, TS, TG, SEG, MSK, DB>), dim3((unsigned)blocks), dim3(MFMA_THREADS), smem_q, st, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dq kernel launch: %s", hipGetErrorString(e));
  hipLaunchKernelGGL((hstu_bwd_dkv_mfma<D, POS, TS, SEG, MSK, DB>), dim3((unsigned)blocks), dim3(DkvShape<D>::THREADS), smem_kv, st, p);
  e = hipGetLastError();
  if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "backward dk/dv kernel launch: %s", hipGetErrorString(e));
  return HSTU_OK;
}

template <int D, bool SEG>
int launch_bwd_mfma_ds(const Params& q, hipStream_t st) {
  const bool pos = q.pos_tab != nullptr, ts = q.ts_tab != nullptr;
  const bool tg = (pos && q.dpos) || (ts && q.dts);
  if (pos && ts) return tg ? launch_bwd_mfma_inst<D, true, true, true, SEG>(q, st) : launch_bwd_mfma_inst<D, true, true, false, SEG>(q, st);
  if (pos) return tg ? launch_bwd_mfma_inst<D, true, false, true, SEG>(q, st) : launch_bwd_mfma_inst<D, true, false, false, SEG>(q, st);
  if (ts) return tg ? launch_bwd_mfma_inst<D, false, true, true, SEG>(q, st) : launch_bwd_mfma_inst<D, false, true, false, SEG>(q, st);
  return launch_bwd_mfma_inst<D, false, false, false, SEG>(q, st);
}

template <int D>
int launch_bwd_mfma_d(const Params& q, hipStream_t st) {
  if (q.mask && q.dense_bias) return launch_bwd_mfma_inst<D, false, false, false, false, true, true>(q, st);
  if (q.dense_bias) return launch_bwd_mfma_inst<D, false, false, false, false, false, true>(q, st);
  if (q.mask) return launch_bwd_mfma_inst<D, false, false, false, false, true>(q, st);
  return q.mask_mode == HSTU_MASK_SEGMENT ? launch_bwd_mfma_ds<D, true>(q, st) : launch_bwd_mfma_ds<D, false>(q, st);
}

int launch_bwd_mfma(const HstuAttnBwdArgs* b, const Params& p, hipStream_t st) {
  HstuAttnFwdArgs f = b->fwd;
  f.out = (void*)b->dout;
  f.flags &= ~HSTU_FWD_WORKSPACE_PREPARED;   // the backward lays the work list out without key-range splits
  const WorkspacePlan ws = plan_workspace(&f, false, ~(size_t)0, false);
  Params q = p;
  q.mask_pres = 1;
  q.no_stream = (b->fwd.flags & HSTU_FWD_COMPILER_SCHEDULED_BLOCKS) ? 1 : 0;
  if (int rc = setup_workspace(&f, ws, q, st)) return rc;
  if (q.d_qk == 128) return launch_bwd_mfma_d<128>(q, st);
#ifndef HSTU_ONLY_D128
  if (q.d_qk == 64) return launch_bwd_mfma_d<64>(q, st);
  return launch_bwd_mfma_d<32>(q, st);
#else
  return fail(HSTU_ERR_SHAPE, "development build: d = 128 only");
#endif
}

}  // namespace

// Scratch of hstu_attn_fwd_noalloc: the workspace of a forward call, built into the library so that
// the call needs no allocation.  In host code this name is only a handle for hipGetSymbolAddress;
// each GPU holds its own copy at its own address.
static __device__ __align__(256) unsigned char scratch[HSTU_ATTN_NOALLOC_SCRATCH_BYTES];

namespace {

// Device address of `scratch` on the current GPU, looked up once per device.
int scratch_of_current_device(void** out) {
  constexpr int kMaxDev = 64;
  static void* ptrs[kMaxDev];
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(HSTU_ERR_LAUNCH, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDev) return fail(HSTU_ERR_LAUNCH, "device index %d beyond the %d this library keeps scratch for", dev, kMaxDev);
  void* ptr = __atomic_load_n(&ptrs[dev], __ATOMIC_ACQUIRE);
  if (!ptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) return fail(HSTU_ERR_LAUNCH, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    __atomic_store_n(&ptrs[dev], ptr, __ATOMIC_RELEASE);   // two threads racing here store the same address
  }
  *out = ptr;
  return HSTU_OK;
}

}  // namespace

extern "C" {

int hstu_attn_abi_version(void) { return HSTU_ATTN_ABI_VERSION; }

int hstu_attn_dropout_keep(uint64_t dropout_seed, float dropout_p, int32_t b, int32_t h, int32_t H, int32_t i, int32_t j) {
  const uint32_t thr = drop_threshold(dropout_p);
  if (!thr) return 1;
  const uint32_t kbh = drop_bh_key(drop_seed_key(dropout_seed), (uint32_t)b * (uint32_t)H + (uint32_t)h);
  return drop_keep(kbh, (uint32_t)i, (uint32_t)j, thr) ? 1 : 0;
}

const char* hstu_attn_last_error(void) { return g_err; }

size_t hstu_attn_fwd_workspace_bytes(const HstuAttnFwdArgs* args) {
  if (validate(args) != HSTU_OK) return 0;
  return plan_workspace(args).total();
}

int hstu_attn_bucket_thresholds(float bucket_size, int32_t* thresholds, int count) {
  if (!(bucket_size > 0.f) || (count > 0 && !thresholds)) return fail(HSTU_ERR_SHAPE, "bad bucket size or null output");
  const BucketLaw& law = bucket_law(bucket_size);
  for (int b = 0; b < count; ++b) thresholds[b] = b < LAW_THR_LEN ? law.thr[b] : 0x7fffffff;
  return law.reach + 1;
}

const char* hstu_attn_fwd_variant(const HstuAttnFwdArgs* args) {
  if (validate(args) != HSTU_OK) return "invalid";
  switch (pick_variant(args)) {
    case V_GENERAL_F32: return "hstu_fwd_general<float>";
    case V_GENERAL_BF16: return "hstu_fwd_general<bf16>";
    case V_MFMA_BF16: return "hstu_fwd_mfma_bf16";
    case V_MFMA_FP8: return "hstu_fwd_mfma_fp8";
    default: return "invalid";
  }
}

const char* hstu_attn_bwd_variant(const HstuAttnBwdArgs* args) {
  if (!args || args->struct_size != sizeof(HstuAttnBwdArgs) || args->version != HSTU_ATTN_ABI_VERSION) return "invalid";
  HstuAttnFwdArgs probe = args->fwd;
  if (!probe.out) probe.out = (void*)args->dout;
  if (validate(&probe) != HSTU_OK || probe.qk_dtype == HSTU_DTYPE_FP8_E4M3FN) return "invalid";
  if (bwd_mfma_eligible(args)) return "hstu_bwd_mfma_bf16";
  if (probe.qk_dtype == HSTU_DTYPE_FP32) return "hstu_bwd_general<float>";
  Params p = make_params(&probe);
  p.dout = args->dout;
  return general_bwd_bf16_products(p) ? "hstu_bwd_general<bf16, bf16 products>" : "hstu_bwd_general<bf16>";
}

int hstu_attn_bwd(const HstuAttnBwdArgs* args, void* stream) {
  if (!args) return fail(HSTU_ERR_NULL, "args is null");
  if (args->struct_size != sizeof(HstuAttnBwdArgs) || args->version != HSTU_ATTN_ABI_VERSION)
    return fail(HSTU_ERR_VERSION, "backward args struct_size/version (%u/%u) do not match this library (%zu/%d)",
                args->struct_size, args->version, sizeof(HstuAttnBwdArgs), HSTU_ATTN_ABI_VERSION);
  const HstuAttnFwdArgs* f = &args->fwd;
  // the forward's own checks apply, except that its `out` is not needed
  HstuAttnFwdArgs probe = *f;
  if (!probe.out) probe.out = (void*)args->dout;
  int rc = validate(&probe);
  if (rc != HSTU_OK) return rc;
  g_err[0] = 0;
  if (f->qk_dtype == HSTU_DTYPE_FP8_E4M3FN) return fail(HSTU_ERR_DTYPE, "the backward takes fp32 or bf16 storage, not fp8 q/k");
  if (f->B == 0 || (f->layout == HSTU_LAYOUT_JAGGED && f->total_tokens == 0)) return HSTU_OK;
  if (!args->dout || !args->dq || !args->dk || !args->dv) return fail(HSTU_ERR_NULL, "dout, dq, dk and dv must be non-null");
  Params p = make_params(f);
  p.dout = args->dout; p.dq = args->dq; p.dk = args->dk; p.dv = args->dv;
  p.dpos = args->dpos_tab; p.dts = args->dts_tab;
  p.dbias = args->ddense_bias;
  if (p.dbias && !p.dense_bias) return fail(HSTU_ERR_NULL, "ddense_bias needs the forward's dense_bias");
  hipStream_t st = (hipStream_t)stream;
  if (bwd_mfma_eligible(args)) return launch_bwd_mfma(args, p, st);
  // (the general kernels sum the bucket table's gradient in LDS first, one float per entry)
  if (p.dts && p.ts_tab && p.ts_nb > 4095)
    return fail(HSTU_ERR_SHAPE, "the gradient of a timestamp table of more than 4096 entries is not supported, got %d", p.ts_nb + 1);
  return f->qk_dtype == HSTU_DTYPE_FP32 ? launch_bwd<float>(p, st) : launch_bwd<bf16_t>(p, st);
}

int hstu_attn_fwd_noalloc(const HstuAttnFwdArgs* args, void* stream) {
  int rc = validate(args);
  if (rc != HSTU_OK) return rc;
  HstuAttnFwdArgs a = *args;
  a.workspace = nullptr;
  a.workspace_bytes = 0;
  const size_t need = plan_workspace(&a, true, (size_t)HSTU_ATTN_NOALLOC_SCRATCH_BYTES).total();
  if (need > (size_t)HSTU_ATTN_NOALLOC_SCRATCH_BYTES)
    return fail(HSTU_ERR_WORKSPACE, "this call needs %zu bytes of scratch, the array built into the library holds %zu: "
                "use hstu_attn_fwd with a caller workspace", need, (size_t)HSTU_ATTN_NOALLOC_SCRATCH_BYTES);
  if (need) {
    void* ptr = nullptr;
    if ((rc = scratch_of_current_device(&ptr)) != HSTU_OK) return rc;
    a.workspace = ptr;
    a.workspace_bytes = HSTU_ATTN_NOALLOC_SCRATCH_BYTES;
  }
  return hstu_attn_fwd(&a, stream);
}

int hstu_attn_fwd(const HstuAttnFwdArgs* args, void* stream) {
  int rc = validate(args);
  if (rc != HSTU_OK) return rc;
  g_err[0] = 0;
  if (args->B == 0 || (args->layout == HSTU_LAYOUT_JAGGED && args->total_tokens == 0)) return HSTU_OK;
  const Params p = make_params(args);
  hipStream_t st = (hipStream_t)stream;
  switch (pick_variant(args)) {
    // (the general kernel has nothing to prepare)
    case V_GENERAL_F32: return (args->flags & HSTU_FWD_PREPARE_ONLY) ? HSTU_OK : launch_general<float>(p, st);
    case V_GENERAL_BF16: return (args->flags & HSTU_FWD_PREPARE_ONLY) ? HSTU_OK : launch_general<bf16_t>(p, st);
    case V_MFMA_BF16:
    case V_MFMA_FP8: {
      const bool f8 = args->qk_dtype == HSTU_DTYPE_FP8_E4M3FN;
      // the split capacity adapts to the workspace the caller brought (never below what the call needs)
      const WorkspacePlan ws = plan_workspace(args, true, args->workspace ? args->workspace_bytes : 0);
      Params q = p;
      if (int rc2 = setup_workspace(args, ws, q, st)) return rc2;
      if (args->flags & HSTU_FWD_PREPARE_ONLY) return HSTU_OK;
      // Resident workgroups over the work list, where that loop is built (d = 128 in bf16, lengths or no mask)
      // and where it pays: with many items per resident workgroup.  (B = 64, L = 2048, H = 8, every sequence
      // full, 17 items each: 0.962 -> 0.924 ms.  The jagged headline shape has under 3 items each; there the
      // end of the launch, where each workgroup finishes whatever it drew last, costs more than the items'
      // starts save: 69 -> 77 us.)  The padded layout with lengths leaves the host guessing the number of
      // items: one workgroup per item there.
      const bool can_stay = q.sched && q.ctr && q.d_qk == 128 && !f8 && !q.mask && !q.dense_bias && q.mask_mode != HSTU_MASK_SEGMENT;
      const bool count_known = q.jagged || !q.seq_lens;
      const long long tiles = q.jagged ? args->total_tokens / BM + args->B : (long long)args->B * q.n_qtiles;
      const long long jobs_per_xcd = q.H >= 8 ? tiles * (q.H >> 3) : tiles / (8 / q.H);
      q.no_stream = ((args->flags & HSTU_FWD_COMPILER_SCHEDULED_BLOCKS) || q.drop_thr) ? 1 : 0;   // (the stream has no dropout)
      // (with timestamp descriptors the interior steps run as the hand-scheduled stream, which the resident instances
      // with timestamps do not have: one workgroup per item there)
      q.persist = can_stay && !(args->flags & HSTU_FWD_ONE_ITEM_PER_WORKGROUP) &&
                  ((args->flags & HSTU_FWD_RESIDENT_WORKGROUPS) || (count_known && jobs_per_xcd >= 8LL * q.n_slots && !q.ts_desc));
      if (int rc2 = f8 ? launch_mfma<true>(q, st) : launch_mfma<false>(q, st)) return rc2;
      return HSTU_OK;
    }
    default: return fail(HSTU_ERR_SHAPE, "no kernel for these arguments");
  }
}

}  // extern "C"

