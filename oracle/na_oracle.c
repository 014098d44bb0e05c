/*
 * CPU oracle (plain C) for neighborhood attention forward and backward, evaluated query by query.
 *
 * TEST INFRASTRUCTURE ONLY: this file is the checker for the HIP path (tests, smoke, the bench's
 * CPU-baseline leg).  Nothing shipped links or calls it.
 *
 * It restates the naive reference kernel of SHI-Labs/NATTEN
 *   csrc/include/natten/cuda/reference/fna_reference_forward.hpp:63-211  (one query at a time,
 *       scaled dot products, mask, softmax, LSE = log(sum) + max of the scaled logits)
 *   csrc/include/natten/cuda/reference/mask.hpp:59-91, 220-225, 295-346  (window, dilation groups)
 * but walks only the keys inside the window instead of testing every key, which is the same
 * set by construction (is_neighbor is an interval test per dimension, mask.hpp:172-194).
 * It shares no code with the numpy oracle (na_oracle.py), which builds the dense N x N mask;
 * the tests require the two to agree.
 *
 * Layout: q [B, X0, X1, X2, H, D], k/v [B, X0, X1, X2, Hkv, D] (unused leading dims = 1),
 * float32 in, float64 arithmetic, float64 out.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

static int imin(int a, int b) { return a < b ? a : b; }
static int imax(int a, int b) { return a > b ? a : b; }

/* mask.hpp:59-82 */
static int win_start(int i, int k, int s, int L, int causal) {
  int wl = k / 2, wr = k / 2 + (k % 2 - 1);
  if (causal) {
    int leader = imin((i / s) * s + s - 1, L - 1);
    return imax(leader - wl - wr, 0);
  }
  int leader = imin((i / s) * s + s / 2, L - 1);
  return imax(leader - wl, 0) + ((leader + wr >= L) ? (L - wr - leader - 1) : 0);
}

/* mask.hpp:84-91 */
static int win_end(int i, int start, int k, int L, int causal) {
  return causal ? imin(i + 1, L) : start + k;
}

/* mask.hpp:220-225 */
static int fix_extent(int X, int d, int g) { return X / d + 1 - ((g + (d - X % d)) / d); }

int na_oracle_window(int i, int k, int s, int L, int causal, int* start, int* end) {
  *start = win_start(i, k, s, L, causal);
  *end = win_end(i, *start, k, L, causal);
  return 0;
}

/*
 * Evaluate `nq` queries given by (batch index, row-major token index) for all heads.
 * out [nq, H, D] and lse [nq, H] are float64.  Returns the number of (query, head, key) triples
 * visited so callers can turn a timing into FLOP/s.
 */
int64_t na_oracle_rows(const float* q, const float* k, const float* v, int B, const int* X /*3*/,
                       int H, int Hkv, int D, const int* ksz, const int* stride, const int* dil,
                       const int* causal, double scale, int nq, const int* q_batch,
                       const int64_t* q_token, double* out, double* lse) {
  (void)B;
  const int64_t N = (int64_t)X[0] * X[1] * X[2];
  const int rep = H / Hkv;
  int64_t visited = 0;
  int maxw = 1;
  for (int a = 0; a < 3; ++a) maxw *= (X[a] < 1 ? 1 : X[a]);
  double* logits = (double*)malloc(sizeof(double) * (size_t)maxw);
  int64_t* keyidx = (int64_t*)malloc(sizeof(int64_t) * (size_t)maxw);
  if (!logits || !keyidx) return -1;
  for (int n = 0; n < nq; ++n) {
    const int b = q_batch[n];
    const int64_t t = q_token[n];
    int c[3] = {(int)(t / ((int64_t)X[1] * X[2])), (int)((t / X[2]) % X[1]), (int)(t % X[2])};
    int st[3], en[3], g[3];
    for (int a = 0; a < 3; ++a) {
      g[a] = c[a] % dil[a];
      int L = fix_extent(X[a], dil[a], g[a]);
      int i = c[a] / dil[a];
      st[a] = win_start(i, ksz[a], stride[a], L, causal[a]);
      en[a] = win_end(i, st[a], ksz[a], L, causal[a]);
    }
    /* enumerate the window once: global key indices */
    int w = 0;
    for (int j0 = st[0]; j0 < en[0]; ++j0)
      for (int j1 = st[1]; j1 < en[1]; ++j1)
        for (int j2 = st[2]; j2 < en[2]; ++j2) {
          int64_t x0 = (int64_t)j0 * dil[0] + g[0], x1 = (int64_t)j1 * dil[1] + g[1],
                  x2 = (int64_t)j2 * dil[2] + g[2];
          keyidx[w++] = (x0 * X[1] + x1) * X[2] + x2;
        }
    for (int h = 0; h < H; ++h) {
      const int hk = h / rep;
      const float* qrow = q + (((int64_t)b * N + t) * H + h) * D;
      double m = -INFINITY;
      for (int j = 0; j < w; ++j) {
        const float* krow = k + (((int64_t)b * N + keyidx[j]) * Hkv + hk) * D;
        double acc = 0.0;
        for (int e = 0; e < D; ++e) acc += (double)qrow[e] * (double)krow[e];
        acc *= scale;
        logits[j] = acc;
        if (acc > m) m = acc;
      }
      double sum = 0.0;
      double* orow = out + ((int64_t)n * H + h) * D;
      for (int e = 0; e < D; ++e) orow[e] = 0.0;
      for (int j = 0; j < w; ++j) {
        double p = exp(logits[j] - m);
        sum += p;
        const float* vrow = v + (((int64_t)b * N + keyidx[j]) * Hkv + hk) * D;
        for (int e = 0; e < D; ++e) orow[e] += p * (double)vrow[e];
      }
      for (int e = 0; e < D; ++e) orow[e] /= sum;
      lse[(int64_t)n * H + h] = log(sum) + m;
      visited += w;
    }
  }
  free(logits);
  free(keyidx);
  return visited;
}

/*
 * Backward: gradients of sum(out * d_out) with respect to q, k, v, for the q heads of the KV
 * heads hk_lo .. hk_hi-1 of batch entry b (callers split the work over disjoint ranges, so
 * no two calls write the same gradient rows).  Restates the naive backward kernels of
 *   csrc/include/natten/cuda/reference/fna_reference_backward.hpp:60-150 (dQ), :165-265 (dK),
 *   :282-380 (dV):   P = exp(scale * q.k - LSE),  dS = P * scale * (dO.v - dO.o),
 *   dQ = sum_j dS k_j,  dK_j = sum_i dS q_i,  dV_j = sum_i P dO_i
 * one query at a time over its window.  LSE is recomputed here and dO.o is evaluated as
 * sum_j P_j (dO.v_j), the same number, so the forward output is not an input.  The gradient of
 * the returned LSE is not propagated, as in the reference.
 * d_out [B, X0, X1, X2, H, D] float32; dq like q, dk / dv like k (float64, zero-initialised by
 * the caller).
 */
int64_t na_oracle_backward(const float* q, const float* k, const float* v, const float* d_out, int b,
                           const int* X /*3*/, int H, int Hkv, int D, const int* ksz, const int* stride,
                           const int* dil, const int* causal, double scale, int hk_lo, int hk_hi,
                           double* dq, double* dk, double* dv) {
  const int64_t N = (int64_t)X[0] * X[1] * X[2];
  const int rep = H / Hkv;
  int64_t visited = 0;
  int maxw = 1;
  for (int a = 0; a < 3; ++a) maxw *= (X[a] < 1 ? 1 : X[a]);
  double* prob = (double*)malloc(sizeof(double) * (size_t)maxw);
  double* dprob = (double*)malloc(sizeof(double) * (size_t)maxw);
  int64_t* keyidx = (int64_t*)malloc(sizeof(int64_t) * (size_t)maxw);
  if (!prob || !dprob || !keyidx) return -1;
  for (int64_t t = 0; t < N; ++t) {
    int c[3] = {(int)(t / ((int64_t)X[1] * X[2])), (int)((t / X[2]) % X[1]), (int)(t % X[2])};
    int st[3], en[3], g[3];
    for (int a = 0; a < 3; ++a) {
      g[a] = c[a] % dil[a];
      int L = fix_extent(X[a], dil[a], g[a]);
      int i = c[a] / dil[a];
      st[a] = win_start(i, ksz[a], stride[a], L, causal[a]);
      en[a] = win_end(i, st[a], ksz[a], L, causal[a]);
    }
    int w = 0;
    for (int j0 = st[0]; j0 < en[0]; ++j0)
      for (int j1 = st[1]; j1 < en[1]; ++j1)
        for (int j2 = st[2]; j2 < en[2]; ++j2) {
          int64_t x0 = (int64_t)j0 * dil[0] + g[0], x1 = (int64_t)j1 * dil[1] + g[1],
                  x2 = (int64_t)j2 * dil[2] + g[2];
          keyidx[w++] = (x0 * X[1] + x1) * X[2] + x2;
        }
    for (int h = hk_lo * rep; h < hk_hi * rep; ++h) {
      const int hk = h / rep;
      const int64_t qoff = (((int64_t)b * N + t) * H + h) * D;
      const float* qrow = q + qoff;
      const float* dorow = d_out + qoff;
      double m = -INFINITY;
      for (int j = 0; j < w; ++j) {
        const float* krow = k + (((int64_t)b * N + keyidx[j]) * Hkv + hk) * D;
        double acc = 0.0;
        for (int e = 0; e < D; ++e) acc += (double)qrow[e] * (double)krow[e];
        prob[j] = acc * scale;
        if (prob[j] > m) m = prob[j];
      }
      double sum = 0.0;
      for (int j = 0; j < w; ++j) {
        prob[j] = exp(prob[j] - m);
        sum += prob[j];
      }
      double delta = 0.0;
      for (int j = 0; j < w; ++j) {
        prob[j] /= sum;
        const float* vrow = v + (((int64_t)b * N + keyidx[j]) * Hkv + hk) * D;
        double acc = 0.0;
        for (int e = 0; e < D; ++e) acc += (double)dorow[e] * (double)vrow[e];
        dprob[j] = acc;
        delta += prob[j] * acc;
      }
      double* dqrow = dq + qoff;
      for (int j = 0; j < w; ++j) {
        const int64_t koff = (((int64_t)b * N + keyidx[j]) * Hkv + hk) * D;
        const double ds = prob[j] * (dprob[j] - delta) * scale;
        const float* krow = k + koff;
        double* dkrow = dk + koff;
        double* dvrow = dv + koff;
        for (int e = 0; e < D; ++e) {
          dqrow[e] += ds * (double)krow[e];
          dkrow[e] += ds * (double)qrow[e];
          dvrow[e] += prob[j] * (double)dorow[e];
        }
      }
      visited += w;
    }
  }
  free(prob);
  free(dprob);
  free(keyidx);
  return visited;
}
