/*
 * Plain-C restatement of the HSTU pointwise-SiLU attention forward.
 *
 * TEST INFRASTRUCTURE ONLY: a second, independent CPU statement of the op
 * (next to oracle/hstu_oracle.py) used by tests as a checker and by the
 * benchmark as the CPU baseline.  Nothing in the shipped package links it.
 *
 * Follows, per output row i of sequence b and head h:
 *   s_j  = alpha * <q_i, k_j>                      recml/layers/keras/hstu.py:365-371
 *        + pos_tab[(L-1) + j - i]                  hstu.py:91-113 (closed form)
 *        + ts_tab[clip(floor(log(fl32(clip(|ts[i+1]-ts[j]|,1,1e9))) / size), 0, nb)]   (log, divide in double)
 *                                                  hstu.py:33-55, 190-221
 *   p_j  = s_j * sigmoid(s_j) * inv_n              hstu.py:376-378
 *   keep j <= i (causal), j < n_b, i < n_b         recml/layers/keras/utils.py:29-41
 *   out_i = sum_j p_j v_j                          hstu.py:389
 * Rows i >= n_b of the padded layout are written as zeros.
 *
 * Inputs are fp32 (bf16 storage is rounded by the caller).  Two variants:
 * hstu_oracle_fwd_f64 accumulates in double (the checker), hstu_oracle_fwd_f32
 * in float (the timed CPU baseline).  Parallel over (sequence, head) with
 * OpenMP; `nthreads` <= 0 keeps the OpenMP default.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef struct {
  const float *q, *k, *v;
  float* out;
  int B, L, H, d_qk, d_v;
  const int32_t* seq_offsets; /* [B+1] jagged, or NULL for padded [B,L,H,d] */
  const int32_t* seq_lens;    /* [B] padded lengths, or NULL (= all L)       */
  float alpha, inv_n;
  int causal;
  const float* pos_tab; int pos_heads;       /* [pos_heads, 2L-1] or NULL     */
  const int64_t* ts; int64_t ts_stride_b;    /* padded stride, 0 = jagged     */
  const float* ts_tab; int ts_heads; int ts_nb; float ts_bucket_size;
} OracleArgs;

static int bucket_of(int64_t dt, float size, int nb) {
  if (dt < 0) dt = -dt;
  if (dt < 1) dt = 1;
  if (dt > 1000000000LL) dt = 1000000000LL;
  /* the bucket law: the reference's float log and divide (hstu.py:48-55) taken in double on the
   * float-rounded difference and the float bucket size; the kernels follow it exactly */
  double lg = log((double)(float)dt) / (double)size;
  int b = (int)lg;
  return b < 0 ? 0 : (b > nb ? nb : b);
}

#define DEFINE_FWD(NAME, ACC)                                                        \
  int NAME(const OracleArgs* a, int nthreads) {                                      \
    const int H = a->H, dq = a->d_qk, dv = a->d_v, L = a->L;                          \
    const int64_t tok_stride_q = (int64_t)H * dq, tok_stride_v = (int64_t)H * dv;    \
    if (nthreads > 0) {                                                              \
      _Pragma("omp parallel for schedule(dynamic, 1) num_threads(nthreads)")         \
      for (int bh = 0; bh < a->B * H; ++bh) NAME##_one(a, bh / H, bh % H);           \
    } else {                                                                         \
      _Pragma("omp parallel for schedule(dynamic, 1)")                               \
      for (int bh = 0; bh < a->B * H; ++bh) NAME##_one(a, bh / H, bh % H);           \
    }                                                                                \
    (void)tok_stride_q; (void)tok_stride_v; (void)dq; (void)dv; (void)L;             \
    return 0;                                                                        \
  }

#define DEFINE_ONE(NAME, ACC)                                                        \
  static void NAME##_one(const OracleArgs* a, int b, int h) {                        \
    const int H = a->H, dq = a->d_qk, dv = a->d_v, L = a->L;                          \
    int64_t tok0; int n, rows;                                                       \
    if (a->seq_offsets) {                                                            \
      tok0 = a->seq_offsets[b]; n = a->seq_offsets[b + 1] - a->seq_offsets[b];       \
      if (n > L) n = L;                                                              \
      rows = n;                                                                      \
    } else {                                                                         \
      tok0 = (int64_t)b * L; n = a->seq_lens ? a->seq_lens[b] : L;                   \
      if (n > L) n = L;                                                              \
      if (n < 0) n = 0;                                                              \
      rows = L;                                                                      \
    }                                                                                \
    const int64_t ts0 = a->ts_stride_b ? (int64_t)b * a->ts_stride_b : tok0;         \
    const int n_ts = a->ts_stride_b ? L : n;                                         \
    const float* pos = a->pos_tab ? a->pos_tab + (int64_t)(a->pos_heads > 1 ? h : 0) * (2 * L - 1) : NULL; \
    const float* tab = a->ts_tab ? a->ts_tab + (int64_t)(a->ts_heads > 1 ? h : 0) * (a->ts_nb + 1) : NULL; \
    ACC* acc = (ACC*)malloc(sizeof(ACC) * dv);                                       \
    for (int i = 0; i < rows; ++i) {                                                 \
      float* o = a->out + ((tok0 + i) * H + h) * dv;                                 \
      if (i >= n) { memset(o, 0, sizeof(float) * dv); continue; }                    \
      const float* qi = a->q + ((tok0 + i) * H + h) * dq;                            \
      for (int c = 0; c < dv; ++c) acc[c] = 0;                                       \
      const int jend = a->causal ? i + 1 : n;                                        \
      int64_t tq = 0;                                                                \
      if (tab) { int iq = i + 1 < n_ts ? i + 1 : n_ts - 1; tq = a->ts[ts0 + iq]; }   \
      for (int j = 0; j < jend; ++j) {                                               \
        const float* kj = a->k + ((tok0 + j) * H + h) * dq;                          \
        ACC s = 0;                                                                   \
        for (int c = 0; c < dq; ++c) s += (ACC)qi[c] * (ACC)kj[c];                   \
        s *= (ACC)a->alpha;                                                          \
        if (pos) s += (ACC)pos[(L - 1) + j - i];                                     \
        if (tab) s += (ACC)tab[bucket_of(tq - a->ts[ts0 + j], a->ts_bucket_size, a->ts_nb)]; \
        ACC p = s / ((ACC)1 + (ACC)exp(-(double)s)) * (ACC)a->inv_n;                 \
        const float* vj = a->v + ((tok0 + j) * H + h) * dv;                          \
        for (int c = 0; c < dv; ++c) acc[c] += p * (ACC)vj[c];                       \
      }                                                                              \
      for (int c = 0; c < dv; ++c) o[c] = (float)acc[c];                             \
    }                                                                                \
    free(acc);                                                                       \
  }

DEFINE_ONE(hstu_oracle_fwd_f64, double)
DEFINE_FWD(hstu_oracle_fwd_f64, double)

/* float variant: expf instead of exp so that the loop stays in single precision */
#undef DEFINE_ONE
static void hstu_oracle_fwd_f32_one(const OracleArgs* a, int b, int h) {
  const int H = a->H, dq = a->d_qk, dv = a->d_v, L = a->L;
  int64_t tok0; int n, rows;
  if (a->seq_offsets) {
    tok0 = a->seq_offsets[b]; n = a->seq_offsets[b + 1] - a->seq_offsets[b];
    if (n > L) n = L;
    rows = n;
  } else {
    tok0 = (int64_t)b * L; n = a->seq_lens ? a->seq_lens[b] : L;
    if (n > L) n = L;
    if (n < 0) n = 0;
    rows = L;
  }
  const int64_t ts0 = a->ts_stride_b ? (int64_t)b * a->ts_stride_b : tok0;
  const int n_ts = a->ts_stride_b ? L : n;
  const float* pos = a->pos_tab ? a->pos_tab + (int64_t)(a->pos_heads > 1 ? h : 0) * (2 * L - 1) : NULL;
  const float* tab = a->ts_tab ? a->ts_tab + (int64_t)(a->ts_heads > 1 ? h : 0) * (a->ts_nb + 1) : NULL;
  float* acc = (float*)malloc(sizeof(float) * dv);
  float* p = (float*)malloc(sizeof(float) * (L > 0 ? L : 1));
  for (int i = 0; i < rows; ++i) {
    float* o = a->out + ((tok0 + i) * H + h) * dv;
    if (i >= n) { memset(o, 0, sizeof(float) * dv); continue; }
    const float* qi = a->q + ((tok0 + i) * H + h) * dq;
    const int jend = a->causal ? i + 1 : n;
    int64_t tq = 0;
    if (tab) { int iq = i + 1 < n_ts ? i + 1 : n_ts - 1; tq = a->ts[ts0 + iq]; }
    for (int j = 0; j < jend; ++j) {
      const float* kj = a->k + ((tok0 + j) * H + h) * dq;
      float s = 0.f;
      _Pragma("omp simd reduction(+:s)")
      for (int c = 0; c < dq; ++c) s += qi[c] * kj[c];
      s *= a->alpha;
      if (pos) s += pos[(L - 1) + j - i];
      if (tab) s += tab[bucket_of(tq - a->ts[ts0 + j], a->ts_bucket_size, a->ts_nb)];
      p[j] = s;
    }
    for (int j = 0; j < jend; ++j) p[j] = p[j] / (1.0f + expf(-p[j])) * a->inv_n;
    for (int c = 0; c < dv; ++c) acc[c] = 0.f;
    for (int j = 0; j < jend; ++j) {
      const float* vj = a->v + ((tok0 + j) * H + h) * dv;
      const float pj = p[j];
      for (int c = 0; c < dv; ++c) acc[c] += pj * vj[c];
    }
    for (int c = 0; c < dv; ++c) o[c] = acc[c];
  }
  free(acc);
  free(p);
}
DEFINE_FWD(hstu_oracle_fwd_f32, float)

int hstu_oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
