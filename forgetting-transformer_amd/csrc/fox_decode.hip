// Single-query forward (decode step, M == 1) of Forgetting Attention for gfx950.
//
// With one query row per (batch, head) there is nothing for the matrix cores to do: the step is one
// pass over the K and V cache, 4*D flops per 4*D bytes.  Like the reference, which switches to an
// element-wise multiply-and-sum for this case (ops/forgetting_attention.py:148-153, :637-641,
// :665-668), this kernel is dot-free.  It keeps nothing in LDS while it streams: a key row of D
// elements is spread over D/8 lanes (16 bytes each), a wave instruction covers 64/(D/8) consecutive
// keys, and every lane holds eight such loads of K and of V in flight, so that a CU has hundreds of
// KiB outstanding instead of the two 64-key tiles of the tiled kernel.  The lanes of a key row reduce
// the partial dot products with four DPP adds; each row group runs its own online softmax
// (running maximum m, sum l, eight accumulator elements per lane), and the groups of a workgroup are
// merged once at the end.
//
// The key range [lo, N) -- lo = max(seq_start, first block the pruning bound keeps) -- is dealt out
// over `splits` workgroups per (batch, head); with more than one split the partial (m, l, acc) go to
// the same workspace layout as the tiled kernel's key splits and fox::combine_kernel merges them.
#include "fox_common.hpp"
#include "fox_kernels.hpp"

namespace fox {

namespace {

// x + (x of the lane selected by a DPP control), as one v_add_f32 with a DPP operand
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  const int y = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true);
  return x + __int_as_float(y);
}

// Sum over the LPR (2, 4, 8 or 16) consecutive lanes that hold one key row; every lane gets the total.
template <int LPR>
__device__ __forceinline__ float row_sum(float x) {
  x = dpp_add<0xB1>(x);                            // quad_perm [1,0,3,2]
  if constexpr (LPR >= 4) x = dpp_add<0x4E>(x);    // quad_perm [2,3,0,1]
  if constexpr (LPR >= 8) x = dpp_add<0x141>(x);   // row_half_mirror: lane i <-> 7 - i of its eight
  if constexpr (LPR >= 16) x = dpp_add<0x140>(x);  // row_mirror: lane i <-> 15 - i of its sixteen
  return x;
}

template <typename Tr>
__device__ __forceinline__ void unpack8f(const u32x4& v, float (&f)[8]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    f[2 * e] = Tr::lo(v[e]);
    f[2 * e + 1] = Tr::hi(v[e]);
  }
}

// merge the online-softmax state (m2, l2, acc2) into (m, l, acc)
__device__ __forceinline__ void merge_state(float& m, float& l, float (&acc)[8], float m2, float l2, const float (&acc2)[8]) {
  const float mx = fmaxf(m, m2);
  const float w1 = __builtin_amdgcn_exp2f(m - mx), w2 = __builtin_amdgcn_exp2f(m2 - mx);
  l = l * w1 + l2 * w2;
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = acc[e] * w1 + acc2[e] * w2;
  m = mx;
}

}  // namespace

template <typename Tr, int D>
__global__ __launch_bounds__(256) void decode_kernel(const FwdK a) {
  constexpr int LPR = D / 8;      // lanes per key row
  constexpr int KPL = 64 / LPR;   // keys per wave load instruction
  constexpr int U = 8;            // loads of K and of V in flight per lane
  constexpr int KPB = KPL * U;    // keys per wave and batch
  __shared__ float part_m[4], part_l[4];
  __shared__ __align__(16) float part_acc[4][D];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ch = lane % LPR, r = lane / LPR;
  const int sp = blockIdx.x % a.splits, bh = blockIdx.x / a.splits;
  const int b = bh / a.H, h = bh % a.H;
  const int N = a.N;
  const float* c_row = a.c + (int64_t)bh * N;
  const uint16_t* qp = a.q.ptr + b * a.q.sb + h * a.q.sh;
  const uint16_t* kp = a.k.ptr + b * a.k.sb + h * a.k.sh + ch * 8;
  const uint16_t* vp = a.v.ptr + b * a.v.sb + h * a.v.sh + ch * 8;

  int seq = 0;
  if (a.seq_start) {
    const int64_t s64 = a.seq_start[b];
    seq = (int)(s64 < 0 ? 0 : (s64 > N ? N : s64));
  }
  const int a0 = N - 1;  // key position of the query row
  const float c_ref = c_row[a0];
  int lo = seq;
  if (a.thr) {
    const int t = acp_first_kept_block(c_row, c_ref, a.thr[bh], N, kFwdBN, a0 / kFwdBN, lane);
    lo = max(lo, t * kFwdBN);
  }
  if (a.first_block && tid == 0 && sp == 0) a.first_block[bh] = lo / kFwdBN;

  // this workgroup's share of [lo, N): whole rounds of 4 waves x KPB keys
  const int n_keys = N - lo;
  int per = (n_keys + a.splits - 1) / a.splits;
  per = (per + 4 * KPB - 1) / (4 * KPB) * (4 * KPB);
  const int k0 = min(N, lo + sp * per), k1 = min(N, k0 + per);

  float qf[8];
  {
    const float qk_scale = a.sm_scale * kLog2e;
    unpack8f<Tr>(*reinterpret_cast<const u32x4*>(qp + ch * 8), qf);
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[e] *= qk_scale;
  }
  float m = -3.0e38f, l = 0.f;  // finite floor: a group that has seen no key yet yields exp2(-inf) = 0
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;

  for (int base = k0 + wave * KPB; base < k1; base += 4 * KPB) {
    u32x4 kx[U], vx[U];
    float cn[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int n = min(base + u * KPL + r, N - 1);  // keys past the range read a valid row and are masked below
      kx[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kp + (int64_t)n * a.k.st));
      cn[u] = c_row[n];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int n = min(base + u * KPL + r, N - 1);
      vx[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vp + (int64_t)n * a.v.st));
    }
    float s[U];
    float bmax = -INFINITY;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float kf[8];
      unpack8f<Tr>(kx[u], kf);
      float dot = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) dot = fmaf(qf[e], kf[e], dot);
      dot = row_sum<LPR>(dot);
      // log2-domain score: sm_scale*log2e*(q.k) + (c_ref - c_n)*log2e.  The two cumulative sums are subtracted
      // first (they are of similar, possibly large, magnitude; their difference is small and exact to an ulp of
      // itself), then scaled: the order of the reference (:642-643).
      const float x = fmaf(c_ref - cn[u], kLog2e, dot);
      s[u] = (base + u * KPL + r < k1) ? x : -INFINITY;
      bmax = fmaxf(bmax, s[u]);
    }
    const float m_new = fmaxf(m, bmax);
    const float alpha = __builtin_amdgcn_exp2f(m - m_new);
    m = m_new;
    l *= alpha;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= alpha;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const float p = __builtin_amdgcn_exp2f(s[u] - m);
      l += p;
      float vf[8];
      unpack8f<Tr>(vx[u], vf);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = fmaf(p, vf[e], acc[e]);
    }
  }

  // merge the KPL row groups of the wave, then the four waves
#pragma unroll
  for (int off = LPR; off < 64; off <<= 1) {
    const float m2 = __shfl_xor(m, off), l2 = __shfl_xor(l, off);
    float acc2[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc2[e] = __shfl_xor(acc[e], off);
    merge_state(m, l, acc, m2, l2, acc2);
  }
  if (r == 0) {
    if (ch == 0) { part_m[wave] = m; part_l[wave] = l; }
#pragma unroll
    for (int e = 0; e < 8; ++e) part_acc[wave][ch * 8 + e] = acc[e];
  }
  __syncthreads();
  if (tid >= LPR) return;
  m = part_m[0];
  l = part_l[0];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = part_acc[0][ch * 8 + e];
#pragma unroll
  for (int w = 1; w < 4; ++w) {
    float acc2[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc2[e] = part_acc[w][ch * 8 + e];
    merge_state(m, l, acc, part_m[w], part_l[w], acc2);
  }

  if (a.splits > 1) {  // partial result of this key split, in the layout fox::combine_kernel reads (M == 1)
    const int64_t row = (int64_t)sp * a.B * a.H + bh;
    float* wo = a.ws_o + row * D + ch * 8;
    const f32x4 w0 = {acc[0], acc[1], acc[2], acc[3]}, w1 = {acc[4], acc[5], acc[6], acc[7]};
    *reinterpret_cast<f32x4*>(wo) = w0;
    *reinterpret_cast<f32x4*>(wo + 4) = w1;
    if (ch == 0) {
      a.ws_ml[2 * row] = m;
      a.ws_ml[2 * row + 1] = l;
    }
    return;
  }
  const bool empty = a0 < seq;  // every key is left padding: o = 0, lse = -inf (:679-685)
  const float inv = empty ? 0.f : 1.0f / l;
  uint16_t* op = const_cast<uint16_t*>(a.o.ptr) + b * a.o.sb + h * a.o.sh + ch * 8;
  u32x4 w;
#pragma unroll
  for (int e = 0; e < 4; ++e) w[e] = Tr::pack2(acc[2 * e] * inv, acc[2 * e + 1] * inv);
  *reinterpret_cast<u32x4*>(op) = w;
  if (ch == 0) a.lse[bh] = empty ? -INFINITY : m * kLn2 + __logf(l);
}

#define FOX_INSTANTIATE_DECODE(TR)                               \
  template __global__ void decode_kernel<TR, 16>(const FwdK);   \
  template __global__ void decode_kernel<TR, 32>(const FwdK);   \
  template __global__ void decode_kernel<TR, 64>(const FwdK);   \
  template __global__ void decode_kernel<TR, 128>(const FwdK);
FOX_INSTANTIATE_DECODE(Bf16)
FOX_INSTANTIATE_DECODE(Fp16)

template <typename Tr>
static hipError_t launch_decode_t(const FwdK& a, int D, hipStream_t s) {
  const dim3 grid((unsigned)(a.splits * a.B * a.H));
  switch (D) {
    case 16: hipLaunchKernelGGL((decode_kernel<Tr, 16>), grid, dim3(256), 0, s, a); break;
    case 32: hipLaunchKernelGGL((decode_kernel<Tr, 32>), grid, dim3(256), 0, s, a); break;
    case 64: hipLaunchKernelGGL((decode_kernel<Tr, 64>), grid, dim3(256), 0, s, a); break;
    case 128: hipLaunchKernelGGL((decode_kernel<Tr, 128>), grid, dim3(256), 0, s, a); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

// The streaming part of a single-query forward; the caller merges the splits (fox::combine_kernel).
hipError_t launch_fwd_decode(const FwdK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? launch_decode_t<Bf16>(a, D, s) : launch_decode_t<Fp16>(a, D, s);
}

}  // namespace fox
