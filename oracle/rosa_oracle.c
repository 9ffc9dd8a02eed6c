/*
 * Row-streamed float64 restatement of the reference RosaSoft operator.
 * TEST ORACLE: linked or loaded only by tests/, __graft_entry__.smoke() and the
 * cpu_baseline leg of bench.py.  The shipped operator never calls into it.
 *
 * It follows the reference's row algorithm, which keeps no O(T^2) state
 * (all file:line below are in /root/reference/rosa_soft/csrc/cuda/
 * rosa_soft_kernels.cu unless another file is named):
 *   - sign packing: bit i of a word is x[..., i] > 0            (:202-241)
 *   - exact suffix length with the min(W, t+1, a) step bound    (:311-348)
 *   - latest-longest merge, length 0 never wins                 (:351-363, :509-510)
 *   - value gather of sign(v[a*]) or exact zero for null        (:511-530)
 *   - local gate exp(-ms * popcount(q ^ k) / D)                 (:534-547)
 *   - counter-hash dropout multiplier                           (:549-586)
 *   - raw suffix score as a sum of prefix products              (:589-641)
 *   - U(S) = (sqrt2+1)(sqrt(1+S)-1) and its derivative          (:650-656)
 *   - row pass 1: logits scale*U - log t, null 0.5*scale, row max,
 *     denominator, expected dropped utility                     (:1190-1351)
 *   - row pass 2: probability, value credit d*p*go, route adjoint
 *     scale*p*(d*u - E)*U'(S), gate adjoints A*tail_j with
 *     tail_0 = S, tail_{j+1} = tail_j - P_{j+1}, scattered as
 *     0.5*(ms/D)*A*tail_j*sign to query t-j and key a-1-j       (:1353-1597, :960-1019)
 *   - softsign Jacobian 1/(1+|x|)^2 applied once at the end     (:1685-1731)
 * The equations are the ones of rosa_soft/soft_reference.py:116-359.
 *
 * All arithmetic is float64 except the two places where the reference fixes
 * float32 semantics: the keep test `uniform >= dropout_p` compares float32
 * values, and the keep multiplier is 1.0f / (1.0f - p).  Inputs are float32
 * images of the tensors (half types convert exactly).
 *
 * The score loop stops early once a prefix product can no longer change the
 * float64 partial sum (gates are <= 1, so later products are not larger);
 * this leaves every score bit-identical to the full loop.  The gradient
 * scatter loop stops once the remaining tail is below 2^-80 of the route's
 * own score, i.e. it drops only weights more than 24 decimal orders below
 * the route's leading weight.
 */

#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ROSA_NULL_SCORE 0.5
#define ROSA_SQRT_SCALE 2.414213562373095048801688724209698

static inline uint32_t pack_bits(const float* x, int width) {
  uint32_t word = 0u;
  for (int bit = 0; bit < width; ++bit) {
    if (x[bit] > 0.0f) word |= (1u << bit);
  }
  return word;
}

static inline uint32_t avalanche(uint32_t s) {
  s ^= s >> 16;
  s *= 0x7feb352du;
  s ^= s >> 15;
  s *= 0x846ca68bu;
  s ^= s >> 16;
  return s;
}

/* float32 uniform in [0,1) for one (batch, head, row, route) coordinate */
float rosa_oracle_dropout_uniform(uint64_t seed, uint32_t batch, uint32_t head,
                                  uint32_t row, uint32_t route) {
  uint32_t s = avalanche(route ^ 0x68e31da4u);
  s = avalanche(s ^ row ^ 0xb5297a4du);
  s = avalanche(s ^ head ^ 0x63d83595u);
  s = avalanche(s ^ batch ^ 0xa511e9b3u);
  s = avalanche(s ^ (uint32_t)seed);
  s = avalanche(s ^ (uint32_t)(seed >> 32) ^ 0x9e3779b9u);
  return (float)(s >> 8) * 0x1.0p-24f;
}

static inline double dropout_multiplier(int enabled, float p, float inverse_keep,
                                        uint64_t seed, int batch, int head,
                                        int row, int route) {
  if (!enabled) return 1.0;
  const float u = rosa_oracle_dropout_uniform(seed, (uint32_t)batch, (uint32_t)head,
                                              (uint32_t)row, (uint32_t)route);
  return u >= p ? (double)inverse_keep : 0.0;
}

int rosa_oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

void rosa_oracle_set_threads(int n) {
#ifdef _OPENMP
  if (n > 0) omp_set_num_threads(n);
#else
  (void)n;
#endif
}

/* Pack q and k into head-major words [B, H, T]. */
void rosa_oracle_pack(const float* q, const float* k, int B, int T, int H, int D,
                      int32_t* packed_q, int32_t* packed_k) {
  for (int b = 0; b < B; ++b)
    for (int t = 0; t < T; ++t)
      for (int h = 0; h < H; ++h) {
        const int64_t src = (((int64_t)b * T + t) * H + h) * D;
        const int64_t dst = ((int64_t)b * H + h) * T + t;
        packed_q[dst] = (int32_t)pack_bits(q + src, D);
        packed_k[dst] = (int32_t)pack_bits(k + src, D);
      }
}

/*
 * Exact hard forward.  out [B,T,H,Dv] (values in {-1,0,+1}), routes [B,H,T]
 * (0 = null), best_len [B,H,T].  W must already be clamped to T.
 */
int rosa_oracle_hard_forward(const float* q, const float* k, const float* v,
                             int B, int T, int H, int D, int Hv, int Dv, int W,
                             float* out, int32_t* routes, int32_t* best_len) {
  if (H % Hv != 0 || D < 1 || D > 32 || W < 1) return 1;
  int32_t* pq = (int32_t*)malloc(sizeof(int32_t) * (size_t)B * H * T);
  int32_t* pk = (int32_t*)malloc(sizeof(int32_t) * (size_t)B * H * T);
  if (!pq || !pk) { free(pq); free(pk); return 2; }
  rosa_oracle_pack(q, k, B, T, H, D, pq, pk);
  const int group = H / Hv;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int bh = 0; bh < B * H; ++bh) {
    for (int t = 0; t < T; ++t) {
      const int b = bh / H, h = bh % H;
      const uint32_t* qw = (const uint32_t*)pq + (int64_t)bh * T;
      const uint32_t* kw = (const uint32_t*)pk + (int64_t)bh * T;
      int best = 0, best_a = 0;
      for (int a = 1; a <= t; ++a) {
        int steps = W < a ? W : a;
        if (t + 1 < steps) steps = t + 1;
        int len = 0;
        while (len < steps && qw[t - len] == kw[a - 1 - len]) ++len;
        if (len > best || (len > 0 && len == best && a > best_a)) {
          best = len;
          best_a = a;
        }
      }
      const int chosen = best > 0 ? best_a : 0;
      routes[(int64_t)bh * T + t] = chosen;
      best_len[(int64_t)bh * T + t] = best;
      float* o = out + (((int64_t)b * T + t) * H + h) * Dv;
      if (chosen > 0) {
        const float* vv = v + (((int64_t)b * T + chosen) * Hv + h / group) * Dv;
        for (int d = 0; d < Dv; ++d) o[d] = vv[d] > 0.0f ? 1.0f : -1.0f;
      } else {
        for (int d = 0; d < Dv; ++d) o[d] = 0.0f;
      }
    }
  }
  free(pq);
  free(pk);
  return 0;
}

static inline double gate_of(uint32_t qw, uint32_t kw, const double* gate_table) {
  return gate_table[__builtin_popcount(qw ^ kw)];
}

/* raw suffix score with early exit once products stop mattering in float64 */
static inline double raw_score(const uint32_t* qw, const uint32_t* kw, int t, int a,
                               int W, const double* gate_table) {
  int steps = W < a ? W : a;
  if (t + 1 < steps) steps = t + 1;
  double product = 1.0, score = 0.0;
  for (int j = 0; j < steps; ++j) {
    product *= gate_of(qw[t - j], kw[a - 1 - j], gate_table);
    score += product;
    if (product < score * 0x1.0p-60) break;
  }
  return score;
}

/*
 * Surrogate VJP.  grad_q/grad_k [B,T,H,D] and grad_v [B,T,Hv,Dv] are float64
 * outputs (overwritten; pass NULL to skip one).  batch_ids[B] and head_offset
 * give the dropout coordinates, so a slice of a larger problem reproduces the
 * masks of the full call.  W must already be clamped.
 */
int rosa_oracle_surrogate_vjp(const float* q, const float* k, const float* v,
                              const float* go, int B, int T, int H, int D, int Hv,
                              int Dv, int W, double scale, double dropout_p,
                              double mismatch_scale, int has_seed, uint64_t seed,
                              const int32_t* batch_ids, int head_offset,
                              double* grad_q, double* grad_k, double* grad_v) {
  if (H % Hv != 0 || D < 1 || D > 32 || W < 1) return 1;
  const int group = H / Hv;
  const int dropout_on = dropout_p > 0.0;
  if (dropout_on && !has_seed) return 3;
  const float p_f = (float)dropout_p;
  const float inverse_keep_f = 1.0f / (1.0f - p_f);
  double gate_table[33];
  for (int c = 0; c <= 32; ++c)
    gate_table[c] = exp(-mismatch_scale * (double)c / (double)D);
  const uint32_t width_mask = D == 32 ? 0xffffffffu : ((1u << D) - 1u);
  (void)width_mask; /* packed words never carry bits above D */

  int32_t* pq = (int32_t*)malloc(sizeof(int32_t) * (size_t)B * H * T);
  int32_t* pk = (int32_t*)malloc(sizeof(int32_t) * (size_t)B * H * T);
  if (!pq || !pk) { free(pq); free(pk); return 2; }
  rosa_oracle_pack(q, k, B, T, H, D, pq, pk);

  const size_t nq = (size_t)B * T * H * D, nv = (size_t)B * T * Hv * Dv;
  if (grad_q) memset(grad_q, 0, sizeof(double) * nq);
  if (grad_k) memset(grad_k, 0, sizeof(double) * nq);
  if (grad_v) memset(grad_v, 0, sizeof(double) * nv);
  const double symbol_scale = 0.5 * mismatch_scale / (double)D;
  const double null_logit = ROSA_NULL_SCORE * scale;
  int failed = 0;

  const size_t row_q = (size_t)T * D, row_v = (size_t)T * Dv;
  for (int bh = 0; bh < B * H && !failed; ++bh) {
    const int b = bh / H, h = bh % H;
    const int hv = h / group;
    const uint32_t* qw = (const uint32_t*)pq + (int64_t)bh * T;
    const uint32_t* kw = (const uint32_t*)pk + (int64_t)bh * T;
#pragma omp parallel
    {
      /* per-thread scratch rows and private gradient slabs for this (b, h) */
      double* scores = (double*)malloc(sizeof(double) * (size_t)(T + 1));
      double* utils = (double*)malloc(sizeof(double) * (size_t)(T + 1));
      double* drops = (double*)malloc(sizeof(double) * (size_t)(T + 1));
      double* local_q = grad_q ? (double*)calloc(row_q, sizeof(double)) : NULL;
      double* local_k = grad_k ? (double*)calloc(row_q, sizeof(double)) : NULL;
      double* local_v = grad_v ? (double*)calloc(row_v, sizeof(double)) : NULL;
      const int ok = scores && utils && drops && (!grad_q || local_q) &&
                     (!grad_k || local_k) && (!grad_v || local_v);
      if (!ok) {
#pragma omp atomic write
        failed = 1;
      }
#pragma omp for schedule(dynamic, 8)
      for (int t = 1; t < T; ++t) {
        if (!ok) continue;
        const float* go_row = go + (((int64_t)b * T + t) * H + h) * Dv;
        const double log_count = log((double)t);
        /* pass 1: scores, utilities, dropout, softmax statistics */
        double row_max = null_logit;
        for (int a = 1; a <= t; ++a) {
          const double s = raw_score(qw, kw, t, a, W, gate_table);
          scores[a] = s;
          const float* vv = v + (((int64_t)b * T + a) * Hv + hv) * Dv;
          double u = 0.0;
          for (int d = 0; d < Dv; ++d)
            u += (double)go_row[d] * (vv[d] > 0.0f ? 1.0 : -1.0);
          utils[a] = u;
          drops[a] = dropout_multiplier(dropout_on, p_f, inverse_keep_f, seed,
                                        batch_ids[b], h + head_offset, t, a);
          const double logit =
              scale * ROSA_SQRT_SCALE * (sqrt(1.0 + s) - 1.0) - log_count;
          if (logit > row_max) row_max = logit;
        }
        double denom = exp(null_logit - row_max);
        double numer = 0.0;
        for (int a = 1; a <= t; ++a) {
          const double logit =
              scale * ROSA_SQRT_SCALE * (sqrt(1.0 + scores[a]) - 1.0) - log_count;
          const double e = exp(logit - row_max);
          denom += e;
          numer += e * drops[a] * utils[a];
        }
        const double expected = numer / denom;
        /* pass 2: gradients */
        for (int a = 1; a <= t; ++a) {
          const double s = scores[a];
          const double root = sqrt(1.0 + s);
          const double logit = scale * ROSA_SQRT_SCALE * (root - 1.0) - log_count;
          const double prob = exp(logit - row_max) / denom;
          const double dropped = prob * drops[a];
          if (local_v && dropped != 0.0) {
            double* gv = local_v + (size_t)a * Dv;
            for (int d = 0; d < Dv; ++d) gv[d] += dropped * (double)go_row[d];
          }
          if (!local_q && !local_k) continue;
          const double adjoint = scale * prob * (drops[a] * utils[a] - expected) *
                                 (0.5 * ROSA_SQRT_SCALE / root);
          if (adjoint == 0.0) continue;
          int steps = W < a ? W : a;
          if (t + 1 < steps) steps = t + 1;
          double product = 1.0, tail = s;
          for (int j = 0; j < steps; ++j) {
            const uint32_t qword = qw[t - j], kword = kw[a - 1 - j];
            product *= gate_of(qword, kword, gate_table);
            const double weight = symbol_scale * adjoint * (tail > 0.0 ? tail : 0.0);
            if (weight != 0.0) {
              double* gq = local_q ? local_q + (size_t)(t - j) * D : NULL;
              double* gk = local_k ? local_k + (size_t)(a - 1 - j) * D : NULL;
              for (int bit = 0; bit < D; ++bit) {
                if (gq) gq[bit] += ((kword >> bit) & 1u) ? weight : -weight;
                if (gk) gk[bit] += ((qword >> bit) & 1u) ? weight : -weight;
              }
            }
            tail -= product;
            if (product < s * 0x1.0p-80) break;
          }
        }
      }
      /* fold the private slabs into the outputs (query/key are owned by this
       * (b, h); value rows are shared by the heads of a group, visited serially) */
#pragma omp critical
      {
        if (ok) {
          for (int t = 0; t < T; ++t) {
            if (local_q) {
              double* dst = grad_q + (((int64_t)b * T + t) * H + h) * D;
              for (int bit = 0; bit < D; ++bit) dst[bit] += local_q[(size_t)t * D + bit];
            }
            if (local_k) {
              double* dst = grad_k + (((int64_t)b * T + t) * H + h) * D;
              for (int bit = 0; bit < D; ++bit) dst[bit] += local_k[(size_t)t * D + bit];
            }
            if (local_v) {
              double* dst = grad_v + (((int64_t)b * T + t) * Hv + hv) * Dv;
              for (int d = 0; d < Dv; ++d) dst[d] += local_v[(size_t)t * Dv + d];
            }
          }
        }
      }
      free(scores);
      free(utils);
      free(drops);
      free(local_q);
      free(local_k);
      free(local_v);
    }
  }
  free(pq);
  free(pk);
  if (failed) return 2;

  /* softsign Jacobian */
  for (size_t i = 0; i < nq; ++i) {
    if (grad_q) { const double den = 1.0 + fabs((double)q[i]); grad_q[i] *= 1.0 / (den * den); }
    if (grad_k) { const double den = 1.0 + fabs((double)k[i]); grad_k[i] *= 1.0 / (den * den); }
  }
  if (grad_v)
    for (size_t i = 0; i < nv; ++i) {
      const double den = 1.0 + fabs((double)v[i]);
      grad_v[i] *= 1.0 / (den * den);
    }
  return 0;
}
