// The gated delta rule with a decay per head and key channel and a per-request fp32 state, gfx950.  Compiled without
// fast-math: everything that enters the recurrence is 32-bit by definition of such a model.
//
//   delta_rule_prep   per row: q and k of every query / key head made unit vectors (q times dim^-0.5), the decays
//                     g = exp(-exp(a_log[h]) * softplus(dt + dt_bias)) per head and key channel, b = sigmoid(beta);
//                     all fp32, computed once per row instead of once per lane of the recurrence
//   gated_delta_rule  per (sequence, head, tile of 64 value columns) a workgroup walks the sequence's rows:
//                       S <- g * S (by rows) ; u = b (v - S^T k) ; S <- S + k u^T ; o = S^T q
//                     as ONE read of the decayed state per row - r = (gS)^T k and p = (gS)^T q together, then
//                     u = b (v - r), o = p + (k.q) u, S = gS + k u^T.  A lane keeps a quarter of one column of S in
//                     registers; the quarters are summed with two xor-shuffles; q / k / g / v / b of a chunk of rows
//                     are staged in LDS with the next chunk's loads in flight (one barrier per chunk).  A prompt
//                     portion and a single decoded row are the same kernel.
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

// sum over the four row parts of a wave (lanes are part * 16 + column)
__device__ __forceinline__ float parts_sum(float v) {
  v += __shfl_xor(v, 16, 64);
  v += __shfl_xor(v, 32, 64);
  return v;
}

// grid (tiles of 64 value columns, H, sequences), 4 waves: wave w owns columns 16 w .. 16 w + 15 of the tile, a lane
// (part = lane / 16, column = lane % 16) keeps rows part * R .. part * R + R - 1 of its column of S in registers
// (4 R >= dim).  The sequence's rows are walked in chunks of C: q, k, g (all of the head, fp32), v (the tile's columns)
// and b of a chunk are staged in LDS by the whole workgroup - the next chunk's loads are in flight while the current
// one is computed, one barrier per chunk - and read back as broadcasts (16-byte reads: a lane's rows are neighbours).
// x rows hold v (H * vdim) at column v_off; qn / kn [T, G, dim], decay [T, H, dim], bsig [T, H] fp32; out
// [T, H * vdim] fp32; state [slots, H, dim, vdim] fp32.
template <typename T, int R, int C>
__global__ __launch_bounds__(256) void gated_delta_rule_kernel(float* __restrict__ out, const T* __restrict__ x,
                                                               long x_stride, int v_off, const float* __restrict__ qn,
                                                               const float* __restrict__ kn,
                                                               const float* __restrict__ decay,
                                                               const float* __restrict__ bsig, float* __restrict__ state,
                                                               const int* __restrict__ slots, const int* __restrict__ qsl,
                                                               const int* __restrict__ seq_lens, int H, int G, int dim,
                                                               int vdim) {
  constexpr int DP = 4 * R;                         // rows, padded (rows past dim stay zero)
  constexpr int ROW = 3 * DP + 64 + 4;              // floats staged per sequence row: q | k | g | v (64) | b, pad
  constexpr int NST = (C * ROW + 255) / 256;        // staged values per thread and chunk
  __shared__ __attribute__((aligned(16))) float lds[2][C * ROW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cl = lane & 15, part = lane >> 4;
  const int col0 = blockIdx.x * 64;
  const int col = col0 + wave * 16 + cl;
  const int h = blockIdx.y, s = blockIdx.z;
  const int g = h / (H / G);
  const int q0 = qsl[s], n = qsl[s + 1] - q0;
  if (n <= 0) return;                               // (the whole workgroup)
  const bool col_ok = col < vdim;
  const int ccol = col_ok ? col : vdim - 1;
  const int r0 = part * R;
  float* st = state + (((long)slots[s] * H + h) * dim) * vdim + ccol;
  float S[R];
  const bool fresh = seq_lens[s] - n <= 0;          // the rows start the sequence: whatever the slot holds is not ours
#pragma unroll
  for (int i = 0; i < R; ++i) S[i] = (!fresh && r0 + i < dim) ? st[(long)(r0 + i) * vdim] : 0.f;

  float stage[NST];
  auto fetch = [&](int chunk) {                     // this thread's share of a chunk, global -> registers
    const int rows = min(C, n - chunk * C);
#pragma unroll
    for (int e = 0; e < NST; ++e) {
      const int idx = tid + e * 256;
      const int j = idx / ROW, f = idx - j * ROW;
      float val = 0.f;
      if (j < rows) {
        const long t = q0 + chunk * C + j;
        if (f < DP) { if (f < dim) val = qn[(t * G + g) * (long)dim + f]; }
        else if (f < 2 * DP) { if (f - DP < dim) val = kn[(t * G + g) * (long)dim + f - DP]; }
        else if (f < 3 * DP) { if (f - 2 * DP < dim) val = decay[(t * H + h) * (long)dim + f - 2 * DP]; }
        else if (f < 3 * DP + 64) { if (col0 + f - 3 * DP < vdim) val = ldf(x + t * x_stride + v_off + (long)h * vdim + col0 + f - 3 * DP); }
        else if (f == 3 * DP + 64) val = bsig[t * H + h];
      }
      stage[e] = val;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int e = 0; e < NST; ++e) {
      const int idx = tid + e * 256;
      if (idx < C * ROW) lds[buf][idx] = stage[e];
    }
  };
  const int chunks = (n + C - 1) / C;
  fetch(0);
  stash(0);
  __syncthreads();
  for (int c = 0; c < chunks; ++c) {
    if (c + 1 < chunks) fetch(c + 1);
    const float* base = lds[c & 1];
    const int rows = min(C, n - c * C);
    for (int j = 0; j < rows; ++j) {
      const float* L = base + j * ROW;
      float r = 0.f, p = 0.f, kq = 0.f;
      float kr[R];
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const f32x4 qv = *reinterpret_cast<const f32x4*>(L + r0 + i);
        const f32x4 kv = *reinterpret_cast<const f32x4*>(L + DP + r0 + i);
        const f32x4 gv = *reinterpret_cast<const f32x4*>(L + 2 * DP + r0 + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[i + e] *= gv[e];
          r += S[i + e] * kv[e];
          p += S[i + e] * qv[e];
          kq += kv[e] * qv[e];
          kr[i + e] = kv[e];
        }
      }
      r = parts_sum(r);
      p = parts_sum(p);
      kq = parts_sum(kq);
      const float u = L[3 * DP + 64] * (L[3 * DP + wave * 16 + cl] - r);
#pragma unroll
      for (int i = 0; i < R; ++i) S[i] += kr[i] * u;
      if (part == 0 && col_ok) out[(long)(q0 + c * C + j) * H * vdim + (long)h * vdim + col] = p + kq * u;
    }
    if (c + 1 < chunks) stash((c + 1) & 1);
    __syncthreads();
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
  const int r = (dim + 3) / 4;                      // rows per lane
  const dim3 grid((vdim + 63) / 64, H, B);
  const int rc = by_dtype(dtype, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
#define GDR(R_, C_)                                                                                                  \
  hipLaunchKernelGGL((gated_delta_rule_kernel<TT, R_, C_>), grid, dim3(256), 0, stream, out, (const TT*)x, x_stride,   \
                     v_off, qn, kn, decay, bsig, state, slots, qsl, seq_lens, H, G, dim, vdim)
    if (r <= 8) GDR(8, 8);
    else if (r <= 16) GDR(16, 8);
    else if (r <= 32) GDR(32, 8);
    else GDR(64, 4);
#undef GDR
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}
