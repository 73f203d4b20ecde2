// The gated delta rule with a decay per head and key channel and a per-request fp32 state, gfx950.  Compiled without
// fast-math: everything that enters the recurrence is 32-bit by definition of such a model.
//
//   delta_rule_prep   per row: q and k of every query / key head made unit vectors (q times dim^-0.5), the decays
//                     g = exp(-exp(a_log[h]) * softplus(dt + dt_bias)) per head and key channel, b = sigmoid(beta);
//                     all fp32, computed once per row instead of once per lane of the recurrence
//   gated_delta_rule  per (sequence, head, tile of value columns) one wave walks the sequence's rows:
//                       S <- g * S (by rows) ; u = b (v - S^T k) ; S <- S + k u^T ; o = S^T q
//                     as ONE read of the decayed state per row - r = (gS)^T k and p = (gS)^T q together, then
//                     u = b (v - r), o = p + (k.q) u, S = gS + k u^T.  The wave's 64 lanes are CT columns x RP row parts;
//                     a lane keeps R = ceil(dim / RP) rows of one column in registers, the row parts are summed with
//                     xor-shuffles (no LDS, no barrier), and the next row's q / k / g are loaded while the current one
//                     is computed.  A prompt portion and a single decoded row are the same kernel.
#include "common.h"
#include <math.h>
#include <type_traits>

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)(*p); }

template <typename F> int by_dtype(int dt, F&& f) {
  switch (dt) {
    case DT_BF16: f((bf16_t*)nullptr); return 0;
    case DT_F16: f((f16_t*)nullptr); return 0;
    case DT_F32: f((float*)nullptr); return 0;
  }
  return 1;
}

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// grid (rows): waves of the block take the units in turn - G query heads, G key heads (a wave each: sum of squares
// over dim), then the H * dim decays and H betas element by element.
template <typename T>
__global__ __launch_bounds__(256) void delta_rule_prep_kernel(float* __restrict__ qn, float* __restrict__ kn,
                                                              float* __restrict__ decay, float* __restrict__ bsig,
                                                              const T* __restrict__ x, long x_stride,
                                                              const T* __restrict__ beta, long beta_stride,
                                                              const T* __restrict__ dt, long dt_stride,
                                                              const float* __restrict__ dt_bias,
                                                              const float* __restrict__ a_log, int H, int G, int dim,
                                                              float norm_eps) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const T* xr = x + t * x_stride;
  const float qscale = 1.0f / sqrtf((float)dim);
  for (int u = wave; u < 2 * G; u += nwaves) {
    const bool is_k = u >= G;
    const int g = is_k ? u - G : u;
    const T* src = xr + (long)u * dim;               // [q heads | k heads], each dim wide
    float ss = 0.f;
    for (int i = lane; i < dim; i += 64) { const float v = ldf(src + i); ss += v * v; }
    const float inv = 1.0f / sqrtf(wave_sum(ss) + norm_eps) * (is_k ? 1.0f : qscale);
    float* dst = (is_k ? kn : qn) + (t * G + g) * (long)dim;
    for (int i = lane; i < dim; i += 64) dst[i] = ldf(src + i) * inv;
  }
  const T* dr = dt + t * dt_stride;
  for (int i = threadIdx.x; i < H * dim; i += blockDim.x) {
    const int h = i / dim;
    decay[t * (long)H * dim + i] = expf(-expf(a_log[h]) * softplus_f(ldf(dr + i) + dt_bias[i]));
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x) bsig[t * H + h] = 1.0f / (1.0f + expf(-ldf(beta + t * beta_stride + h)));
}

template <int RP> __device__ __forceinline__ float parts_sum(float v) {
  // lanes are (row part) * CT + column: sum over the row parts
#pragma unroll
  for (int o = 64 / RP; o < 64; o <<= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// grid (column tiles, H, sequences), one wave.  x rows hold [.. | v (H * vdim)] at column v_off; qn / kn [T, G, dim],
// decay [T, H, dim], bsig [T, H] fp32; out [T, H * vdim] fp32; state [slots, H, dim, vdim] fp32.
template <typename T, int R, int RP>
__global__ __launch_bounds__(64) void gated_delta_rule_kernel(float* __restrict__ out, const T* __restrict__ x,
                                                              long x_stride, int v_off, const float* __restrict__ qn,
                                                              const float* __restrict__ kn,
                                                              const float* __restrict__ decay,
                                                              const float* __restrict__ bsig, float* __restrict__ state,
                                                              const int* __restrict__ slots, const int* __restrict__ qsl,
                                                              const int* __restrict__ seq_lens, int H, int G, int dim,
                                                              int vdim) {
  constexpr int CT = 64 / RP;
  const int lane = threadIdx.x;
  const int col = blockIdx.x * CT + (lane & (CT - 1));
  const int part = lane / CT;
  const int h = blockIdx.y, s = blockIdx.z;
  const int g = h / (H / G);
  const int q0 = qsl[s], n = qsl[s + 1] - q0;
  if (n <= 0) return;
  const bool col_ok = col < vdim;
  const int ccol = col_ok ? col : vdim - 1;
  const int r0 = part * R;
  float* st = state + (((long)slots[s] * H + h) * dim) * vdim + ccol;
  float S[R];
  const bool fresh = seq_lens[s] - n <= 0;          // the rows start the sequence: whatever the slot holds is not ours
#pragma unroll
  for (int i = 0; i < R; ++i) S[i] = (!fresh && r0 + i < dim) ? st[(long)(r0 + i) * vdim] : 0.f;
  float qc[R], kc[R], gc[R], qx[R], kx[R], gx[R];
  float vc, bc, vx = 0.f, bx = 0.f;
  auto load = [&](long t, float* q, float* k, float* gg, float& v, float& b) {
    const float* qp = qn + (t * G + g) * (long)dim + r0;
    const float* kp = kn + (t * G + g) * (long)dim + r0;
    const float* gp = decay + (t * H + h) * (long)dim + r0;
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const bool ok = r0 + i < dim;
      q[i] = ok ? qp[i] : 0.f;
      k[i] = ok ? kp[i] : 0.f;
      gg[i] = ok ? gp[i] : 0.f;
    }
    v = ldf(x + t * x_stride + v_off + (long)h * vdim + ccol);
    b = bsig[t * H + h];
  };
  load(q0, qc, kc, gc, vc, bc);
  for (int i = 0; i < n; ++i) {
    const long t = q0 + i;
    if (i + 1 < n) load(t + 1, qx, kx, gx, vx, bx);
    float r = 0.f, p = 0.f, kq = 0.f;
#pragma unroll
    for (int j = 0; j < R; ++j) {
      S[j] *= gc[j];
      r += S[j] * kc[j];
      p += S[j] * qc[j];
      kq += kc[j] * qc[j];
    }
    r = parts_sum<RP>(r);
    p = parts_sum<RP>(p);
    kq = parts_sum<RP>(kq);
    const float u = bc * (vc - r);
#pragma unroll
    for (int j = 0; j < R; ++j) S[j] += kc[j] * u;
    if (part == 0 && col_ok) out[t * (long)H * vdim + (long)h * vdim + col] = p + kq * u;
#pragma unroll
    for (int j = 0; j < R; ++j) { qc[j] = qx[j]; kc[j] = kx[j]; gc[j] = gx[j]; }
    vc = vx; bc = bx;
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (r0 + i < dim) st[(long)(r0 + i) * vdim] = S[i];
  }
}

}  // namespace

VDAMD_API int vdamd_delta_rule_prep(float* qn, float* kn, float* decay, float* bsig, const void* x, long x_stride,
                                    const void* beta, long beta_stride, const void* dt, long dt_stride,
                                    const float* dt_bias, const float* a_log, int T, int H, int G, int dim,
                                    float norm_eps, int dtype, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || dim <= 0) return 1;
  const int rc = by_dtype(dtype, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    hipLaunchKernelGGL((delta_rule_prep_kernel<TT>), dim3(T), dim3(256), 0, stream, qn, kn, decay, bsig, (const TT*)x,
                       x_stride, (const TT*)beta, beta_stride, (const TT*)dt, dt_stride, dt_bias, a_log, H, G, dim,
                       norm_eps);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

// x [T, x_stride] of type dtype with v at column v_off; dim <= 256
VDAMD_API int vdamd_gated_delta_rule(float* out, const void* x, long x_stride, int v_off, const float* qn,
                                     const float* kn, const float* decay, const float* bsig, float* state,
                                     const int* slots, const int* qsl, const int* seq_lens, int B, int H, int G, int dim,
                                     int vdim, int dtype, hipStream_t stream) {
  if (B <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || dim <= 0 || dim > 256 || vdim <= 0) return 1;
  // row parts so that a lane keeps at most 16 rows; fewer parts (more columns per wave) for small heads
  const int rp = dim <= 64 ? 4 : (dim <= 128 ? 8 : 16);
  const int ct = 64 / rp;
  const int r = (dim + rp - 1) / rp;
  const dim3 grid((vdim + ct - 1) / ct, H, B);
  const int rc = by_dtype(dtype, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
#define GDR(R_, RP_)                                                                                                 \
  hipLaunchKernelGGL((gated_delta_rule_kernel<TT, R_, RP_>), grid, dim3(64), 0, stream, out, (const TT*)x, x_stride,   \
                     v_off, qn, kn, decay, bsig, state, slots, qsl, seq_lens, H, G, dim, vdim)
    if (rp == 4) { if (r <= 4) GDR(4, 4); else if (r <= 8) GDR(8, 4); else GDR(16, 4); }
    else if (rp == 8) { if (r <= 12) GDR(12, 8); else GDR(16, 8); }
    else { if (r <= 12) GDR(12, 16); else GDR(16, 16); }
#undef GDR
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}
