// Token shift for gfx950: the data-dependent mix of each key / value row with its
// predecessor that the FoX layer applies before attention,
//   out[b,t,h,:] = x[b,t,h,:] * curr[b,t,h] + x[b,t-1,h,:] * prev[b,t,h]      (x[b,-1] := 0)
// and its backward
//   dx[b,t,h,:]  = dout[b,t,h,:] * curr[b,t,h] + dout[b,t+1,h,:] * prev[b,t+1,h]
//   dcurr[b,t,h] = sum_d dout[b,t,h,d] * x[b,t,h,d]
//   dprev[b,t,h] = sum_d dout[b,t,h,d] * x[b,t-1,h,d].
// (reference: model/forgetting_transformer/token_shift.py:21-71 forward, :83-156 backward)
//
// Both are pure streams over HBM.  A thread owns 8 consecutive head-dim elements
// (one 16-byte vector) of one (batch, head) column and walks a strip of kStrip time
// steps with the neighbouring row carried in registers, so every element is fetched
// once (plus one halo row per strip) and consecutive lanes cover consecutive memory
// of the (H*D)-element token row.  (strip, head, chunk) triples are flattened over
// the grid so that small H still fills every lane.
#include "fox_common.hpp"
#include "fox_kernels.hpp"

namespace fox {

constexpr int kStrip = 32;  // time steps per thread

template <typename Tr>
__device__ __forceinline__ void unpack8(const u32x4& v, float (&f)[8]) {
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    f[2 * e] = Tr::lo(v[e]);
    f[2 * e + 1] = Tr::hi(v[e]);
  }
}

template <typename Tr, int D>
__global__ __launch_bounds__(256) void shift_fwd_kernel(const ShiftK a) {
  constexpr int CH = D / 8;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int chunk = (int)(gid % CH);
  const int64_t col = gid / CH;
  const int h = (int)(col % a.H);
  const int strip = (int)(col / a.H);
  const int b = blockIdx.y;
  const int t0 = strip * kStrip;
  if (t0 >= a.T) return;
  const int t1 = min(a.T, t0 + kStrip);
  const uint16_t* xp = a.x + b * a.x_sb + h * a.x_sh + chunk * 8;
  uint16_t* op = a.out + b * a.x_sb + h * a.x_sh + chunk * 8;
  const float* pw = a.prev_w + b * a.w_sb + h * a.w_sh;
  const float* cw = a.curr_w + b * a.w_sb + h * a.w_sh;

  u32x4 before = {0u, 0u, 0u, 0u};
  if (t0 > 0) before = *reinterpret_cast<const u32x4*>(xp + (int64_t)(t0 - 1) * a.x_st);
  constexpr int U = 4;  // rows in flight per thread
  for (int tb = t0; tb < t1; tb += U) {
    u32x4 cur[U];
    float wp[U], wc[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = min(tb + u, t1 - 1);
      cur[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xp + (int64_t)t * a.x_st));
      wp[u] = pw[(int64_t)t * a.w_st];
      wc[u] = cw[(int64_t)t * a.w_st];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (tb + u < t1) {
        float xc[8], xb[8];
        unpack8<Tr>(cur[u], xc);
        unpack8<Tr>(before, xb);
        u32x4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          r[e] = Tr::pack2(xc[2 * e] * wc[u] + xb[2 * e] * wp[u], xc[2 * e + 1] * wc[u] + xb[2 * e + 1] * wp[u]);
        *reinterpret_cast<u32x4*>(op + (int64_t)(tb + u) * a.x_st) = r;
        before = cur[u];
      }
    }
  }
}

template <typename Tr, int D>
__global__ __launch_bounds__(256) void shift_bwd_kernel(const ShiftK a) {
  constexpr int CH = D / 8;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int chunk = (int)(gid % CH);
  const int64_t col = gid / CH;
  const int h = (int)(col % a.H);
  const int strip = (int)(col / a.H);
  const int b = blockIdx.y;
  const int t0 = strip * kStrip;
  // no early return: the lanes of one (head, strip) reduce together, and whole groups leave together
  const bool live = t0 < a.T;
  const int t1 = live ? min(a.T, t0 + kStrip) : t0;
  const int hh = live ? h : 0;
  const uint16_t* xp = a.x + b * a.x_sb + hh * a.x_sh + chunk * 8;
  const uint16_t* gp = a.dout + b * a.x_sb + hh * a.x_sh + chunk * 8;
  uint16_t* dxp = a.dx + b * a.x_sb + hh * a.x_sh + chunk * 8;
  const float* pw = a.prev_w + b * a.w_sb + hh * a.w_sh;
  const float* cw = a.curr_w + b * a.w_sb + hh * a.w_sh;
  float* dpw = a.dprev_w + b * a.w_sb + hh * a.w_sh;
  float* dcw = a.dcurr_w + b * a.w_sb + hh * a.w_sh;

  // walk the strip from its last row to its first, carrying dout[t+1], prev[t+1] and x[t]
  u32x4 g_after = {0u, 0u, 0u, 0u};
  float wp_after = 0.f;
  u32x4 x_cur = {0u, 0u, 0u, 0u};
  if (live) {
    if (t1 < a.T) {
      g_after = *reinterpret_cast<const u32x4*>(gp + (int64_t)t1 * a.x_st);
      wp_after = pw[(int64_t)t1 * a.w_st];
    }
    x_cur = *reinterpret_cast<const u32x4*>(xp + (int64_t)(t1 - 1) * a.x_st);
  }
  constexpr int U = 4;
  for (int tb = t1 - 1; tb >= t0; tb -= U) {
    u32x4 g[U], xb[U];
    float wp[U], wc[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = max(tb - u, t0);
      g[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(gp + (int64_t)t * a.x_st));
      const u32x4 z = {0u, 0u, 0u, 0u};
      xb[u] = z;
      if (t > 0) xb[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xp + (int64_t)(t - 1) * a.x_st));
      wp[u] = pw[(int64_t)t * a.w_st];
      wc[u] = cw[(int64_t)t * a.w_st];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int t = tb - u;
      if (t >= t0) {  // uniform over the lanes of a (head, strip) group
        float gc[8], ga[8], xc[8], xp8[8];
        unpack8<Tr>(g[u], gc);
        unpack8<Tr>(g_after, ga);
        unpack8<Tr>(x_cur, xc);
        unpack8<Tr>(xb[u], xp8);
        u32x4 r;
        float sc = 0.f, sp = 0.f;
#pragma unroll
        for (int e = 0; e < 4; ++e)
          r[e] = Tr::pack2(gc[2 * e] * wc[u] + ga[2 * e] * wp_after, gc[2 * e + 1] * wc[u] + ga[2 * e + 1] * wp_after);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          sc += gc[e] * xc[e];
          sp += gc[e] * xp8[e];
        }
        *reinterpret_cast<u32x4*>(dxp + (int64_t)t * a.x_st) = r;
#pragma unroll
        for (int off = CH / 2; off > 0; off >>= 1) {
          sc += __shfl_xor(sc, off);
          sp += __shfl_xor(sp, off);
        }
        if (chunk == 0) {
          dcw[(int64_t)t * a.w_st] = sc;
          dpw[(int64_t)t * a.w_st] = sp;
        }
        g_after = g[u];
        wp_after = wp[u];
        x_cur = xb[u];
      }
    }
  }
}

#define FOX_INSTANTIATE_SHIFT(TR)                                    \
  template __global__ void shift_fwd_kernel<TR, 16>(const ShiftK);  \
  template __global__ void shift_fwd_kernel<TR, 32>(const ShiftK);  \
  template __global__ void shift_fwd_kernel<TR, 64>(const ShiftK);  \
  template __global__ void shift_fwd_kernel<TR, 128>(const ShiftK); \
  template __global__ void shift_bwd_kernel<TR, 16>(const ShiftK);  \
  template __global__ void shift_bwd_kernel<TR, 32>(const ShiftK);  \
  template __global__ void shift_bwd_kernel<TR, 64>(const ShiftK);  \
  template __global__ void shift_bwd_kernel<TR, 128>(const ShiftK);
FOX_INSTANTIATE_SHIFT(Bf16)
FOX_INSTANTIATE_SHIFT(Fp16)

template <typename Tr, bool BWD>
static hipError_t shift_t(const ShiftK& a, int D, hipStream_t s) {
  const int64_t strips = (a.T + kStrip - 1) / kStrip;
  const int64_t threads = strips * a.H * (D / 8);
  const dim3 grid((unsigned)((threads + 255) / 256), (unsigned)a.B);
#define FOX_SHIFT_CASE(DD)                                                                   \
  case DD:                                                                                    \
    if (BWD) hipLaunchKernelGGL((shift_bwd_kernel<Tr, DD>), grid, dim3(256), 0, s, a);        \
    else hipLaunchKernelGGL((shift_fwd_kernel<Tr, DD>), grid, dim3(256), 0, s, a);            \
    break;
  switch (D) {
    FOX_SHIFT_CASE(16)
    FOX_SHIFT_CASE(32)
    FOX_SHIFT_CASE(64)
    FOX_SHIFT_CASE(128)
    default: return hipErrorInvalidValue;
  }
#undef FOX_SHIFT_CASE
  return hipGetLastError();
}

hipError_t launch_shift_fwd(const ShiftK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? shift_t<Bf16, false>(a, D, s) : shift_t<Fp16, false>(a, D, s);
}
hipError_t launch_shift_bwd(const ShiftK& a, int D, int dtype, hipStream_t s) {
  return dtype == 0 ? shift_t<Bf16, true>(a, D, s) : shift_t<Fp16, true>(a, D, s);
}

}  // namespace fox
