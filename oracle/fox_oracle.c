/*
 * fox_oracle.c -- TEST INFRASTRUCTURE ONLY, not part of the shipped operator.
 *
 * A scalar C restatement (double precision, no tiling, no tricks) of the
 * arithmetic of the reference's Forgetting Attention kernels, used next to the
 * PyTorch restatement in fox_oracle.py so that two independently written
 * checkers have to agree.  Only tests, the smoke check and the CPU-baseline leg
 * of the benchmark may load it.
 *
 * Reference lines followed (src/forgetting_transformer/ops/forgetting_attention.py):
 *   fox_oracle_cumsum            :117-127   zero gates left of seq_start, cumulative sum (fp32 running sum)
 *   fox_oracle_fwd               :505-693   _fwd_kernel: s = q.k*scale + c[i+P] - c[j], causal + seq_start mask,
 *                                           softmax, o = p v, L = log normaliser, empty rows -> o = 0, L = -inf
 *   fox_oracle_bwd               :902-943   delta = rowsum(o*do)
 *                                :956-1143  dv = p^T do, dk = scale ds^T q, dc[n] -= sum_i ds[i,n]
 *                                :1156-1344 dq = scale ds k, dc[i+P] += sum_j ds[i,j]
 *                                :390-392   dg = reverse inclusive cumulative sum of dc
 *   fox_oracle_find_start_index  :695-745   two-pointer scan, first key block each query block must visit
 *   fox_oracle_find_end_index    :747-795   two-pointer scan, first query row from which a key block is prunable
 *
 * and (src/forgetting_transformer/model/forgetting_transformer/token_shift.py):
 *   fox_oracle_token_shift_fwd   :21-71     out[t] = x[t]*curr[t] + x[t-1]*prev[t], x[-1] = 0
 *   fox_oracle_token_shift_bwd   :83-156    dx[t] = dout[t]*curr[t] + dout[t+1]*prev[t+1]; dcurr = <dout[t], x[t]>;
 *                                           dprev = <dout[t], x[t-1]>
 *
 * and (src/forgetting_transformer/model/forgetting_transformer/fuse_norm_gate.py):
 *   fox_oracle_norm_gate_fwd/bwd :132-206, :309-417  per-group RMS norm * weight * sigmoid(g) (swish = 1: g*sigmoid(g);
 *                                                     swish = 2: no gate, g and dg untouched = layernorm.py:183-254, :328-435),
 *                                           dx, dg, dweight as in the backward kernel
 *
 * Layouts: q,out,dout,dq are (B,H,M,D); k,v,dk,dv are (B,H,N,D); c,dc,dg are (B,H,N);
 * lse is (B,H,M); all contiguous.  Build: make -C oracle
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define IDX4(b, h, t, d, H, T, D) ((((int64_t)(b) * (H) + (h)) * (T) + (t)) * (D) + (d))
#define IDX3(b, h, t, H, T) (((int64_t)(b) * (H) + (h)) * (T) + (t))

void fox_oracle_cumsum(const float* g, const int64_t* seq_start, float* c, int B, int H, int N) {
  for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h) {
      const int64_t s = seq_start ? seq_start[b] : 0;
      float run = 0.f;
      for (int n = 0; n < N; ++n) {
        const float x = (n < s) ? 0.f : g[IDX3(b, h, n, H, N)];
        run += x; /* fp32 running sum, as torch.cumsum on a float32 tensor */
        c[IDX3(b, h, n, H, N)] = run;
      }
    }
}

/* scores of one query row; returns the number of valid columns */
static int row_scores(const double* q, const double* k, const float* c, int64_t seq, double sm_scale, int b, int h, int i,
                      int H, int M, int N, int D, double* s, int* j_lo, int* j_hi) {
  const int P = N - M, a = i + P;
  int lo = (int)(seq < 0 ? 0 : seq), hi = a; /* valid: lo <= j <= hi */
  if (hi > N - 1) hi = N - 1;
  *j_lo = lo;
  *j_hi = hi;
  if (lo > hi) return 0;
  const double* qi = q + IDX4(b, h, i, 0, H, M, D);
  const double ca = (double)c[IDX3(b, h, a, H, N)];
  for (int j = lo; j <= hi; ++j) {
    const double* kj = k + IDX4(b, h, j, 0, H, N, D);
    double dot = 0.0;
    for (int d = 0; d < D; ++d) dot += qi[d] * kj[d];
    s[j] = dot * sm_scale + (ca - (double)c[IDX3(b, h, j, H, N)]);
  }
  return hi - lo + 1;
}

int fox_oracle_fwd(const double* q, const double* k, const double* v, const float* c, const int64_t* seq_start,
                   double sm_scale, int B, int H, int M, int N, int D, double* out, double* lse) {
  double* s = (double*)malloc(sizeof(double) * (size_t)N);
  if (!s) return -1;
  for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h)
      for (int i = 0; i < M; ++i) {
        int lo, hi;
        double* oi = out + IDX4(b, h, i, 0, H, M, D);
        for (int d = 0; d < D; ++d) oi[d] = 0.0;
        if (!row_scores(q, k, c, seq_start ? seq_start[b] : 0, sm_scale, b, h, i, H, M, N, D, s, &lo, &hi)) {
          lse[IDX3(b, h, i, H, M)] = -INFINITY;
          continue;
        }
        double mx = -INFINITY, l = 0.0;
        for (int j = lo; j <= hi; ++j) mx = s[j] > mx ? s[j] : mx;
        for (int j = lo; j <= hi; ++j) l += exp(s[j] - mx);
        for (int j = lo; j <= hi; ++j) {
          const double p = exp(s[j] - mx) / l;
          const double* vj = v + IDX4(b, h, j, 0, H, N, D);
          for (int d = 0; d < D; ++d) oi[d] += p * vj[d];
        }
        lse[IDX3(b, h, i, H, M)] = mx + log(l);
      }
  free(s);
  return 0;
}

/* out and lse are the forward results (out possibly rounded the way the operator stores it). */
int fox_oracle_bwd(const double* q, const double* k, const double* v, const float* c, const int64_t* seq_start,
                   double sm_scale, int B, int H, int M, int N, int D, const double* out, const double* lse,
                   const double* dout, double* dq, double* dk, double* dv, double* dc, double* dg) {
  const int P = N - M;
  double* s = (double*)malloc(sizeof(double) * (size_t)N);
  if (!s) return -1;
  memset(dq, 0, sizeof(double) * (size_t)B * H * M * D);
  memset(dk, 0, sizeof(double) * (size_t)B * H * N * D);
  memset(dv, 0, sizeof(double) * (size_t)B * H * N * D);
  memset(dc, 0, sizeof(double) * (size_t)B * H * N);
  for (int b = 0; b < B; ++b)
    for (int h = 0; h < H; ++h) {
      for (int i = 0; i < M; ++i) {
        int lo, hi;
        if (!row_scores(q, k, c, seq_start ? seq_start[b] : 0, sm_scale, b, h, i, H, M, N, D, s, &lo, &hi)) continue;
        const double* qi = q + IDX4(b, h, i, 0, H, M, D);
        const double* oi = out + IDX4(b, h, i, 0, H, M, D);
        const double* doi = dout + IDX4(b, h, i, 0, H, M, D);
        double* dqi = dq + IDX4(b, h, i, 0, H, M, D);
        const double L = lse[IDX3(b, h, i, H, M)];
        double delta = 0.0;
        for (int d = 0; d < D; ++d) delta += oi[d] * doi[d];
        double row = 0.0;
        for (int j = lo; j <= hi; ++j) {
          const double p = exp(s[j] - L);
          const double* kj = k + IDX4(b, h, j, 0, H, N, D);
          const double* vj = v + IDX4(b, h, j, 0, H, N, D);
          double* dkj = dk + IDX4(b, h, j, 0, H, N, D);
          double* dvj = dv + IDX4(b, h, j, 0, H, N, D);
          double dp = 0.0;
          for (int d = 0; d < D; ++d) dp += doi[d] * vj[d];
          const double ds = p * (dp - delta);
          for (int d = 0; d < D; ++d) {
            dvj[d] += p * doi[d];
            dkj[d] += sm_scale * ds * qi[d];
            dqi[d] += sm_scale * ds * kj[d];
          }
          dc[IDX3(b, h, j, H, N)] -= ds;
          row += ds;
        }
        dc[IDX3(b, h, i + P, H, N)] += row;
      }
      double run = 0.0;
      for (int n = N - 1; n >= 0; --n) {
        run += dc[IDX3(b, h, n, H, N)];
        dg[IDX3(b, h, n, H, N)] = run;
      }
    }
  free(s);
  return 0;
}

/* One (b,h) row of c.  out has ceil(M / block_m) entries. */
void fox_oracle_find_start_index(const float* c, float threshold, int M, int N, int block_m, int block_n, int64_t* out) {
  const int P = N - M;
  int64_t start = 0;
  int o = 0;
  for (int m0 = 0; m0 < M; m0 += block_m) {
    const float c_out = c[P + m0];
    for (;;) {
      int64_t col = start + block_n - 1;
      if (col > N - 1) col = N - 1;
      const float decay = c_out - c[col];
      if (decay < threshold && start + block_n <= P + m0) /* the block holding the row itself is never skipped */
        start += block_n;
      else
        break;
    }
    out[o++] = start;
  }
}

/* tight != 0 reads c[row + P] (the reference reads c[row], :783,789, which can only prune less). */
void fox_oracle_find_end_index(const float* c, float threshold, int M, int N, int block_m, int block_n, int tight,
                               int64_t* out) {
  const int P = tight ? N - M : 0;
  int64_t end = 0;
  int o = 0;
  for (int n0 = 0; n0 < N; n0 += block_n) {
    int col = n0 + block_n - 1;
    if (col > N - 1) col = N - 1;
    while (end < M) {
      int64_t row = end < M - 1 ? end : M - 1;
      const float decay = c[row + P] - c[col];
      if (decay >= threshold)
        end = end + block_m < M ? end + block_m : M;
      else
        break;
    }
    out[o++] = end;
  }
}


/* Token shift: x, out, dout, dx are (B,T,H,D) contiguous doubles; weights and their gradients (B,T,H). */
void fox_oracle_token_shift_fwd(const double* x, const double* prev_w, const double* curr_w, double* out, int B, int T, int H,
                                int D) {
  for (int b = 0; b < B; ++b)
    for (int t = 0; t < T; ++t)
      for (int h = 0; h < H; ++h) {
        const int64_t w = ((int64_t)b * T + t) * H + h;
        for (int d = 0; d < D; ++d) {
          const double cur = x[w * D + d];
          const double before = t > 0 ? x[(w - H) * D + d] : 0.0;
          out[w * D + d] = cur * curr_w[w] + before * prev_w[w];
        }
      }
}

void fox_oracle_token_shift_bwd(const double* x, const double* prev_w, const double* curr_w, const double* dout, double* dx,
                                double* dprev_w, double* dcurr_w, int B, int T, int H, int D) {
  for (int b = 0; b < B; ++b)
    for (int t = 0; t < T; ++t)
      for (int h = 0; h < H; ++h) {
        const int64_t w = ((int64_t)b * T + t) * H + h;
        double sc = 0.0, sp = 0.0;
        for (int d = 0; d < D; ++d) {
          const double g = dout[w * D + d];
          const double g_after = t + 1 < T ? dout[(w + H) * D + d] : 0.0;
          const double p_after = t + 1 < T ? prev_w[w + H] : 0.0;
          dx[w * D + d] = g * curr_w[w] + g_after * p_after;
          sc += g * x[w * D + d];
          sp += g * (t > 0 ? x[(w - H) * D + d] : 0.0);
        }
        dcurr_w[w] = sc;
        dprev_w[w] = sp;
      }
}


/* Gated per-group RMS norm: x, g, y, dy, dx, dg are (R, G, D) contiguous doubles; w, dw are (G, D).
 * swish: 0 = sigmoid gate, 1 = swish gate, 2 = no gate (g is not read, dg is not written). */
static double gate_act(const double* g, int64_t i, int mode) {
  if (mode == 2) return 1.0;
  const double s = 1.0 / (1.0 + exp(-g[i]));
  return mode ? g[i] * s : s;
}
static double gate_dact(const double* g, int64_t i, int mode) {
  if (mode == 2) return 0.0;
  const double s = 1.0 / (1.0 + exp(-g[i]));
  return mode ? s + g[i] * s * (1.0 - s) : s * (1.0 - s);
}
void fox_oracle_norm_gate_fwd(const double* x, const double* g, const double* w, double* y, int64_t R, int G, int D, double eps,
                              int swish) {
  for (int64_t r = 0; r < R; ++r)
    for (int h = 0; h < G; ++h) {
      const int64_t o = (r * G + h) * D;
      double ss = 0.0;
      for (int d = 0; d < D; ++d) ss += x[o + d] * x[o + d];
      const double rstd = 1.0 / sqrt(ss / D + eps);
      for (int d = 0; d < D; ++d) y[o + d] = x[o + d] * rstd * w[h * D + d] * gate_act(g, o + d, swish);
    }
}

void fox_oracle_norm_gate_bwd(const double* x, const double* g, const double* w, const double* dy, double* dx, double* dg,
                              double* dw, int64_t R, int G, int D, double eps, int swish) {
  for (int j = 0; j < G * D; ++j) dw[j] = 0.0;
  for (int64_t r = 0; r < R; ++r)
    for (int h = 0; h < G; ++h) {
      const int64_t o = (r * G + h) * D;
      double ss = 0.0;
      for (int d = 0; d < D; ++d) ss += x[o + d] * x[o + d];
      const double rstd = 1.0 / sqrt(ss / D + eps);
      double c1 = 0.0;
      for (int d = 0; d < D; ++d) {
        const double xhat = x[o + d] * rstd;
        if (swish != 2) dg[o + d] = dy[o + d] * xhat * w[h * D + d] * gate_dact(g, o + d, swish);
        const double dyn = dy[o + d] * gate_act(g, o + d, swish);
        dw[h * D + d] += dyn * xhat;
        c1 += xhat * dyn * w[h * D + d];
      }
      c1 /= D;
      for (int d = 0; d < D; ++d) {
        const double xhat = x[o + d] * rstd;
        dx[o + d] = (dy[o + d] * gate_act(g, o + d, swish) * w[h * D + d] - xhat * c1) * rstd;
      }
    }
}
