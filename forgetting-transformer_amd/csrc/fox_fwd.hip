// Forward kernel of Forgetting Attention for gfx950.
//
// One workgroup (4 waves) owns 128 query rows of one (batch, head); wave w owns
// rows 32w..32w+31 and keeps them in registers as the B operand of
// S^T = K Q^T (32x32x16 MFMA).  With the scores transposed, lane (g, i) holds one
// query row i and 16 key columns per 32-column block, so the online-softmax row
// statistics are lane-local plus one exchange between the two 32-lane halves, and
// the probabilities are already laid out as the B operand of O^T = V^T P^T.  K and
// V tiles are staged through LDS; V^T is read with the transposing LDS load.
//
// The decay bias enters relative to c_ref = c[first query row of the tile]:
//   x = (q.k) * sm_scale*log2e - (c_n - c_ref)*log2e          (per score)
// and the row term (c_m - c_ref)*log2e, constant along a row, is only added to the
// stored log-normaliser.  Columns left of seq_start (and beyond N) get
// (c_n - c_ref) = +inf, which makes x = -inf without a compare in the loop; only
// tiles crossing the diagonal run the causal compare.
#include "fox_common.hpp"
#include "fox_kernels.hpp"

namespace fox {

template <typename Tr, int D>
__global__ __launch_bounds__(256, 2) void fwd_kernel(const FwdK a) {
  constexpr int BM = kFwdBM, BN = kFwdBN, NT = 256;
  constexpr int KK = D / 16, DB = (D + 31) / 32, NB = BN / 32;
  static_assert(BM == 128, "four waves of 32 rows");
  __shared__ __align__(16) char k_tile[BN * D * 2];
  __shared__ __align__(16) char v_tile[BN * D * 2];
  __shared__ __align__(16) float cn_s[BN];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 5, i = lane & 31;
  int bh, mt;
  decode_block(blockIdx.x, a.n_mtiles, a.B * a.H, bh, mt);
  const int b = bh / a.H, h = bh % a.H;
  const int M = a.M, N = a.N, p_seq = N - M;
  const int m0 = mt * BM;
  const float* c_row = a.c + (int64_t)bh * N;
  const uint16_t* qp = a.q.ptr + b * a.q.sb + h * a.q.sh;
  const uint16_t* kp = a.k.ptr + b * a.k.sb + h * a.k.sh;
  const uint16_t* vp = a.v.ptr + b * a.v.sb + h * a.v.sh;
  uint16_t* op = const_cast<uint16_t*>(a.o.ptr) + b * a.o.sb + h * a.o.sh;

  const int a0 = p_seq + m0;  // key position of the tile's first query row
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
  if (a.first_block && tid == 0) a.first_block[(int64_t)bh * a.n_mtiles + mt] = lo / BN;

  const int m = m0 + 32 * wave + i;  // this lane's query row
  const int a_m = p_seq + m;
  const int a_w0 = a0 + 32 * wave;   // key position of the wave's first row
  u32x4 qreg[KK];
  load_row_operand_regs<D>(qreg, qp, a.q.st, m, M, g);
  const float c_ref = c_row[a0];
  const float cm2 = (m < M) ? (c_row[a_m] - c_ref) * kLog2e : 0.f;
  const float qk_scale = a.sm_scale * kLog2e;

  f32x16 oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  float m_i = -INFINITY, l_i = 0.f;

  TileLoader<D, BN, NT> kl, vl;
  float cn_pref = 0.f;
  auto prefetch = [&](int n0) {
    kl.load(kp, a.k.st, n0, N, tid);
    vl.load(vp, a.v.st, n0, N, tid);
    if (tid < BN) {
      const int n = n0 + tid;
      cn_pref = (n < N && n >= seq) ? (c_row[n] - c_ref) * kLog2e : INFINITY;
    }
  };
  if (lo < hi) prefetch(lo);

  for (int n0 = lo; n0 < hi; n0 += BN) {
    __syncthreads();  // every wave is done with the previous tile
    kl.store(k_tile, tid);
    vl.store(v_tile, tid);
    if (tid < BN) cn_s[tid] = cn_pref;
    __syncthreads();
    if (n0 + BN < hi) prefetch(n0 + BN);
    if (n0 > a_w0 + 31) continue;  // tile entirely above this wave's rows
    const bool diag = n0 + BN - 1 > a_w0;

    // S^T = K Q^T
    f32x16 s[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[nb][r] = 0.f;
#pragma unroll
      for (int kk = 0; kk < KK; ++kk)
        s[nb] = Tr::mfma32(lds_row_operand<D>(k_tile, 32 * nb + i, 2 * kk + g), qreg[kk], s[nb]);
    }

    // scores in the log2 domain, running max
    float mloc = -INFINITY;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const f32x4 cn = *reinterpret_cast<const f32x4*>(&cn_s[32 * nb + 8 * q4 + 4 * g]);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int r = 4 * q4 + t;
          float x = fmaf(s[nb][r], qk_scale, -cn[t]);
          if (diag) {
            const int n = n0 + 32 * nb + 8 * q4 + 4 * g + t;
            x = (n > a_m) ? -INFINITY : x;
          }
          s[nb][r] = x;
          mloc = fmaxf(mloc, x);
        }
      }
    }
    mloc = half_max(mloc);
    const float m_use = fmaxf(fmaxf(m_i, mloc), -3.0e38f);  // finite even when the row is still empty
    const float alpha = __builtin_amdgcn_exp2f(m_i - m_use);
    float rsum = 0.f;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = __builtin_amdgcn_exp2f(s[nb][r] - m_use);
        s[nb][r] = p;
        rsum += p;
      }
    l_i = l_i * alpha + rsum;  // per-lane partial sum; the two halves are added in the epilogue
    m_i = m_use;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;

    // O^T += V^T P^T
#pragma unroll
    for (int sl = 0; sl < BN / 16; ++sl) {
      const u32x4 pb = pack8<Tr>(s[sl >> 1], 8 * (sl & 1));
#pragma unroll
      for (int db = 0; db < DB; ++db) oacc[db] = Tr::mfma32(lds_col_operand<D>(v_tile, 16 * sl, db, lane), pb, oacc[db]);
    }
  }

  // epilogue
  const float l_tot = half_sum(l_i);
  const bool empty = a_m < seq;
  const float inv = empty ? 0.f : 1.0f / l_tot;
  if (m < M) {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int d = 32 * db + 8 * q4 + 4 * g;
        if (d < D) {
          u32x2 w;
          w[0] = Tr::pack2(oacc[db][4 * q4 + 0] * inv, oacc[db][4 * q4 + 1] * inv);
          w[1] = Tr::pack2(oacc[db][4 * q4 + 2] * inv, oacc[db][4 * q4 + 3] * inv);
          *reinterpret_cast<u32x2*>(op + (int64_t)m * a.o.st + d) = w;
        }
      }
    if (g == 0) a.lse[(int64_t)bh * M + m] = empty ? -INFINITY : (m_i + cm2) * kLn2 + __logf(l_tot);
  }
}

template <typename Tr>
static hipError_t launch_fwd_t(const FwdK& a, int D, hipStream_t s) {
  const dim3 grid((unsigned)(a.n_mtiles * a.B * a.H)), block(256);
  switch (D) {
    case 16: hipLaunchKernelGGL((fwd_kernel<Tr, 16>), grid, block, 0, s, a); break;
    case 32: hipLaunchKernelGGL((fwd_kernel<Tr, 32>), grid, block, 0, s, a); break;
    case 64: hipLaunchKernelGGL((fwd_kernel<Tr, 64>), grid, block, 0, s, a); break;
    case 128: hipLaunchKernelGGL((fwd_kernel<Tr, 128>), grid, block, 0, s, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

hipError_t launch_fwd(const FwdK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? launch_fwd_t<Bf16>(a, D, s) : launch_fwd_t<Fp16>(a, D, s);
}

}  // namespace fox
