// Backward kernels of Forgetting Attention for gfx950.
//
//   delta_kernel : delta_i = sum_d o_id * do_id
//   dkdv_kernel  : one workgroup keeps 128 key rows (K, V in registers as MFMA B
//                  operands; dK^T, dV^T accumulators) and walks the query tiles
//                  below its diagonal; writes dk, dv and dc[n] = -sum_i dS[i,n].
//   dq_kernel    : one workgroup keeps 128 query rows (Q, dO in registers) and
//                  walks the key tiles like the forward; writes dq and adds
//                  sum_j dS[i,j] into dc[i + N - M].
//
// Probabilities are rebuilt from the stored log-normaliser:
//   P = exp2( (q.k)*sm_scale*log2e + rowc_i - colc_j ),
//   rowc_i = (c_i - c_ref - lse_i)*log2e   (-inf for rows past M or empty rows),
//   colc_j = (c_j - c_ref)*log2e           (+inf left of seq_start or past N),
// so row/column validity costs nothing in the loop; only tiles that cross the
// diagonal run the causal compare.  In every kernel the first MFMA leaves each
// lane with one index of the dimension that stays free in the second MFMA, so the
// recomputed P / dS feed the second MFMA straight from registers.
#include "fox_common.hpp"
#include "fox_kernels.hpp"

namespace fox {

// ---------------------------------------------------------------------------
template <typename Tr, int D>
__global__ __launch_bounds__(256) void delta_kernel(const BwdK a) {
  constexpr int LPR = D / 8;          // lanes per row
  constexpr int RPP = 256 / LPR;      // rows per pass
  constexpr int ROWS = 128;           // rows per workgroup
  const int tid = threadIdx.x;
  const int bh = blockIdx.y, b = bh / a.H, h = bh % a.H;
  const uint16_t* op = a.o.ptr + b * a.o.sb + h * a.o.sh;
  const uint16_t* dop = a.d_o.ptr + b * a.d_o.sb + h * a.d_o.sh;
  const int ch = tid % LPR;
#pragma unroll
  for (int pass = 0; pass < ROWS / RPP; ++pass) {
    const int m = blockIdx.x * ROWS + pass * RPP + tid / LPR;
    float acc = 0.f;
    if (m < a.M) {
      const u32x4 x = *reinterpret_cast<const u32x4*>(op + (int64_t)m * a.o.st + ch * 8);
      const u32x4 y = *reinterpret_cast<const u32x4*>(dop + (int64_t)m * a.d_o.st + ch * 8);
#pragma unroll
      for (int e = 0; e < 4; ++e) acc += Tr::lo(x[e]) * Tr::lo(y[e]) + Tr::hi(x[e]) * Tr::hi(y[e]);
    }
#pragma unroll
    for (int off = LPR / 2; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (m < a.M && ch == 0) a.delta[(int64_t)bh * a.M + m] = acc;
  }
}

// ---------------------------------------------------------------------------
template <typename Tr, int D>
__global__ __launch_bounds__(256) void dkdv_kernel(const BwdK a) {
  constexpr int BN = kKvBN, BMQ = kKvBM, NT = 256;
  constexpr int KK = D / 16, DB = (D + 31) / 32, MB = BMQ / 32;
  static_assert(BN == 128, "four waves of 32 key rows");
  __shared__ __align__(16) char q_tile[BMQ * D * 2];
  __shared__ __align__(16) char do_tile[BMQ * D * 2];
  __shared__ __align__(16) float rc_s[BMQ];
  __shared__ __align__(16) float dl_s[BMQ];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, i = lane & 31;
  int bh, nt;
  decode_block(blockIdx.x, a.n_tiles, a.B * a.H, bh, nt);
  const int b = bh / a.H, h = bh % a.H;
  const int M = a.M, N = a.N, p_seq = N - M;
  const int n0 = nt * BN;
  const float* c_row = a.c + (int64_t)bh * N;
  const float* lse_row = a.lse + (int64_t)bh * M;
  const float* delta_row = a.delta + (int64_t)bh * M;
  const uint16_t* qp = a.q.ptr + b * a.q.sb + h * a.q.sh;
  const uint16_t* kp = a.k.ptr + b * a.k.sb + h * a.k.sh;
  const uint16_t* vp = a.v.ptr + b * a.v.sb + h * a.v.sh;
  const uint16_t* dop = a.d_o.ptr + b * a.d_o.sb + h * a.d_o.sh;
  uint16_t* dkp = const_cast<uint16_t*>(a.dk.ptr) + b * a.dk.sb + h * a.dk.sh;
  uint16_t* dvp = const_cast<uint16_t*>(a.dv.ptr) + b * a.dv.sb + h * a.dv.sh;

  int seq = 0;
  if (a.seq_start) {
    const int64_t s64 = a.seq_start[b];
    seq = (int)(s64 < 0 ? 0 : (s64 > N ? N : s64));
  }
  // query range: rows whose key position reaches this tile, up to the pruning bound
  int m_lo = max(n0 - p_seq, 0);
  m_lo = (m_lo / BMQ) * BMQ;
  int m_hi = M;
  if (a.thr) {
    const int last = min(N - 1, n0 + BN - 1);
    const int U = (M + BMQ - 1) / BMQ;
    const int u = acp_first_pruned_qblock(c_row, c_row[last], a.thr[bh], p_seq, BMQ, m_lo / BMQ, U, lane);
    m_hi = min(M, u * BMQ);
  }
  if (n0 + BN <= seq) m_hi = m_lo;  // every key of the tile is left padding

  const int n_w0 = n0 + 32 * wave;
  const int n = n_w0 + i;  // this lane's key row
  u32x4 kreg[KK], vreg[KK];
  load_row_operand_regs<D>(kreg, kp, a.k.st, n, N, g);
  load_row_operand_regs<D>(vreg, vp, a.v.st, n, N, g);
  const float c_ref = c_row[n0];
  const float colc = (n < N && n >= seq) ? (c_row[n] - c_ref) * kLog2e : INFINITY;
  const float qk_scale = a.sm_scale * kLog2e;

  f32x16 dkacc[DB], dvacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) { dkacc[db][r] = 0.f; dvacc[db][r] = 0.f; }
  float csum = 0.f;

  TileLoader<D, BMQ, NT> ql, dol;
  float rc_pref = 0.f, dl_pref = 0.f;
  auto prefetch = [&](int ms) {
    ql.load(qp, a.q.st, ms, M, tid);
    dol.load(dop, a.d_o.st, ms, M, tid);
    if (tid < BMQ) {
      const int mm = ms + tid;
      rc_pref = -INFINITY;
      dl_pref = 0.f;
      if (mm < M) {
        const float l = lse_row[mm];
        if (l > -INFINITY) rc_pref = (c_row[p_seq + mm] - c_ref - l) * kLog2e;
        dl_pref = delta_row[mm];
      }
    }
  };
  if (m_lo < m_hi) prefetch(m_lo);

  for (int ms = m_lo; ms < m_hi; ms += BMQ) {
    __syncthreads();
    ql.store(q_tile, tid);
    dol.store(do_tile, tid);
    if (tid < BMQ) { rc_s[tid] = rc_pref; dl_s[tid] = dl_pref; }
    __syncthreads();
    if (ms + BMQ < m_hi) prefetch(ms + BMQ);

#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int a_b0 = p_seq + ms + 32 * mb;  // key position of the block's first query row
      if (a_b0 + 31 < n_w0) continue;         // block entirely above the diagonal for this wave
      const bool diag = a_b0 < n_w0 + 31;
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) s = Tr::mfma32(lds_row_operand<D>(q_tile, 32 * mb + i, 2 * kk + g), kreg[kk], s);
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) dp = Tr::mfma32(lds_row_operand<D>(do_tile, 32 * mb + i, 2 * kk + g), vreg[kk], dp);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const f32x4 rc = *reinterpret_cast<const f32x4*>(&rc_s[32 * mb + 8 * q4 + 4 * g]);
        const f32x4 dl = *reinterpret_cast<const f32x4*>(&dl_s[32 * mb + 8 * q4 + 4 * g]);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int r = 4 * q4 + t;
          float p = __builtin_amdgcn_exp2f(fmaf(s[r], qk_scale, rc[t]) - colc);
          if (diag) {
            const int am = a_b0 + 8 * q4 + 4 * g + t;
            p = (n > am) ? 0.f : p;
          }
          const float ds = p * (dp[r] - dl[t]);
          s[r] = p;
          dp[r] = ds;
          csum += ds;
        }
      }
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const u32x4 pb = pack8<Tr>(s, 8 * hh);
        const u32x4 dsb = pack8<Tr>(dp, 8 * hh);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          dvacc[db] = Tr::mfma32(lds_col_operand<D>(do_tile, 32 * mb + 16 * hh, db, lane), pb, dvacc[db]);
          dkacc[db] = Tr::mfma32(lds_col_operand<D>(q_tile, 32 * mb + 16 * hh, db, lane), dsb, dkacc[db]);
        }
      }
    }
  }

  const float ctot = half_sum(csum);
  if (n < N) {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d = 32 * db + 8 * q4 + 4 * g;
        if (d < D) {
          u32x2 w;
          w[0] = Tr::pack2(dkacc[db][4 * q4 + 0] * a.sm_scale, dkacc[db][4 * q4 + 1] * a.sm_scale);
          w[1] = Tr::pack2(dkacc[db][4 * q4 + 2] * a.sm_scale, dkacc[db][4 * q4 + 3] * a.sm_scale);
          *reinterpret_cast<u32x2*>(dkp + (int64_t)n * a.dk.st + d) = w;
          w[0] = Tr::pack2(dvacc[db][4 * q4 + 0], dvacc[db][4 * q4 + 1]);
          w[1] = Tr::pack2(dvacc[db][4 * q4 + 2], dvacc[db][4 * q4 + 3]);
          *reinterpret_cast<u32x2*>(dvp + (int64_t)n * a.dv.st + d) = w;
        }
      }
    if (g == 0) a.dc[(int64_t)bh * N + n] = -ctot;
  }
}

// ---------------------------------------------------------------------------
template <typename Tr, int D>
__global__ __launch_bounds__(256) void dq_kernel(const BwdK a) {
  constexpr int BM = kFwdBM, BN = kFwdBN, NT = 256;
  constexpr int KK = D / 16, DB = (D + 31) / 32, NB = BN / 32;
  __shared__ __align__(16) char k_tile[BN * D * 2];
  __shared__ __align__(16) char v_tile[BN * D * 2];
  __shared__ __align__(16) float cn_s[BN];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, i = lane & 31;
  int bh, mt;
  decode_block(blockIdx.x, a.n_tiles, a.B * a.H, bh, mt);
  const int b = bh / a.H, h = bh % a.H;
  const int M = a.M, N = a.N, p_seq = N - M;
  const int m0 = mt * BM;
  const float* c_row = a.c + (int64_t)bh * N;
  const uint16_t* qp = a.q.ptr + b * a.q.sb + h * a.q.sh;
  const uint16_t* kp = a.k.ptr + b * a.k.sb + h * a.k.sh;
  const uint16_t* vp = a.v.ptr + b * a.v.sb + h * a.v.sh;
  const uint16_t* dop = a.d_o.ptr + b * a.d_o.sb + h * a.d_o.sh;
  uint16_t* dqp = const_cast<uint16_t*>(a.dq.ptr) + b * a.dq.sb + h * a.dq.sh;

  const int a0 = p_seq + m0;
  const int hi = min(N, a0 + BM);
  int seq = 0;
  if (a.seq_start) {
    const int64_t s64 = a.seq_start[b];
    seq = (int)(s64 < 0 ? 0 : (s64 > N ? N : s64));
  }
  int lo = min(seq, hi);
  if (a.thr) {
    const int t = acp_first_kept_block(c_row, c_row[a0], a.thr[bh], N, BN, a0 / BN, lane);
    lo = max(lo, t * BN);
  }
  lo = (lo / BN) * BN;

  const int m = m0 + 32 * wave + i;
  const int a_m = p_seq + m;
  const int a_w0 = a0 + 32 * wave;
  u32x4 qreg[KK], doreg[KK];
  load_row_operand_regs<D>(qreg, qp, a.q.st, m, M, g);
  load_row_operand_regs<D>(doreg, dop, a.d_o.st, m, M, g);
  const float c_ref = c_row[a0];
  float rowc = -INFINITY, delta = 0.f;
  if (m < M) {
    const float l = a.lse[(int64_t)bh * M + m];
    if (l > -INFINITY) rowc = (c_row[a_m] - c_ref - l) * kLog2e;
    delta = a.delta[(int64_t)bh * M + m];
  }
  const float qk_scale = a.sm_scale * kLog2e;

  f32x16 dqacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) dqacc[db][r] = 0.f;
  float rsum = 0.f;

  TileLoader<D, BN, NT> kl, vl;
  float cn_pref = 0.f;
  auto prefetch = [&](int nn0) {
    kl.load(kp, a.k.st, nn0, N, tid);
    vl.load(vp, a.v.st, nn0, N, tid);
    if (tid < BN) {
      const int nn = nn0 + tid;
      cn_pref = (nn < N && nn >= seq) ? (c_row[nn] - c_ref) * kLog2e : INFINITY;
    }
  };
  if (lo < hi) prefetch(lo);

  for (int n0 = lo; n0 < hi; n0 += BN) {
    __syncthreads();
    kl.store(k_tile, tid);
    vl.store(v_tile, tid);
    if (tid < BN) cn_s[tid] = cn_pref;
    __syncthreads();
    if (n0 + BN < hi) prefetch(n0 + BN);

#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const int nb0 = n0 + 32 * nb;
      if (nb0 > a_w0 + 31) continue;  // block entirely above this wave's rows
      const bool diag = nb0 + 31 > a_w0;
      f32x16 s, dp;
#pragma unroll
      for (int r = 0; r < 16; ++r) { s[r] = 0.f; dp[r] = 0.f; }
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) s = Tr::mfma32(lds_row_operand<D>(k_tile, 32 * nb + i, 2 * kk + g), qreg[kk], s);
#pragma unroll
      for (int kk = 0; kk < KK; ++kk) dp = Tr::mfma32(lds_row_operand<D>(v_tile, 32 * nb + i, 2 * kk + g), doreg[kk], dp);
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const f32x4 cn = *reinterpret_cast<const f32x4*>(&cn_s[32 * nb + 8 * q4 + 4 * g]);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int r = 4 * q4 + t;
          float p = __builtin_amdgcn_exp2f(fmaf(s[r], qk_scale, rowc) - cn[t]);
          if (diag) {
            const int nn = nb0 + 8 * q4 + 4 * g + t;
            p = (nn > a_m) ? 0.f : p;
          }
          const float ds = p * (dp[r] - delta);
          dp[r] = ds;
          rsum += ds;
        }
      }
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const u32x4 dsb = pack8<Tr>(dp, 8 * hh);
#pragma unroll
        for (int db = 0; db < DB; ++db)
          dqacc[db] = Tr::mfma32(lds_col_operand<D>(k_tile, 32 * nb + 16 * hh, db, lane), dsb, dqacc[db]);
      }
    }
  }

  const float rtot = half_sum(rsum);
  if (m < M) {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d = 32 * db + 8 * q4 + 4 * g;
        if (d < D) {
          u32x2 w;
          w[0] = Tr::pack2(dqacc[db][4 * q4 + 0] * a.sm_scale, dqacc[db][4 * q4 + 1] * a.sm_scale);
          w[1] = Tr::pack2(dqacc[db][4 * q4 + 2] * a.sm_scale, dqacc[db][4 * q4 + 3] * a.sm_scale);
          *reinterpret_cast<u32x2*>(dqp + (int64_t)m * a.dq.st + d) = w;
        }
      }
    if (g == 0) a.dc[(int64_t)bh * N + a_m] += rtot;  // the dK/dV kernel wrote the column part earlier on this stream
  }
}

// ---------------------------------------------------------------------------
#define FOX_DISPATCH_D(KERNEL, GRID, SMEM)                                                        \
  switch (D) {                                                                                    \
    case 16: hipLaunchKernelGGL((KERNEL<Tr, 16>), GRID, dim3(256), SMEM, s, a); break;            \
    case 32: hipLaunchKernelGGL((KERNEL<Tr, 32>), GRID, dim3(256), SMEM, s, a); break;            \
    case 64: hipLaunchKernelGGL((KERNEL<Tr, 64>), GRID, dim3(256), SMEM, s, a); break;            \
    case 128: hipLaunchKernelGGL((KERNEL<Tr, 128>), GRID, dim3(256), SMEM, s, a); break;          \
    default: return hipErrorInvalidValue;                                                         \
  }

template <typename Tr>
static hipError_t delta_t(const BwdK& a, int D, hipStream_t s) {
  const dim3 grid((unsigned)((a.M + 127) / 128), (unsigned)(a.B * a.H));
  FOX_DISPATCH_D(delta_kernel, grid, 0)
  return hipGetLastError();
}
template <typename Tr>
static hipError_t dkdv_t(const BwdK& a0, int D, hipStream_t s) {
  BwdK a = a0;
  a.n_tiles = (a.N + kKvBN - 1) / kKvBN;
  const dim3 grid((unsigned)(a.n_tiles * a.B * a.H));
  FOX_DISPATCH_D(dkdv_kernel, grid, 0)
  return hipGetLastError();
}
template <typename Tr>
static hipError_t dq_t(const BwdK& a0, int D, hipStream_t s) {
  BwdK a = a0;
  a.n_tiles = (a.M + kFwdBM - 1) / kFwdBM;
  const dim3 grid((unsigned)(a.n_tiles * a.B * a.H));
  FOX_DISPATCH_D(dq_kernel, grid, 0)
  return hipGetLastError();
}

hipError_t launch_bwd_delta(const BwdK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? delta_t<Bf16>(a, D, s) : delta_t<Fp16>(a, D, s);
}
hipError_t launch_bwd_dkdv(const BwdK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? dkdv_t<Bf16>(a, D, s) : dkdv_t<Fp16>(a, D, s);
}
hipError_t launch_bwd_dq(const BwdK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? dq_t<Bf16>(a, D, s) : dq_t<Fp16>(a, D, s);
}

}  // namespace fox
