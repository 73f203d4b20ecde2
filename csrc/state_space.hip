// Kernels for layers with a state-space recurrence and for attention whose values are its keys and whose heads mix
// their softmax weights, gfx950.  Compiled without fast-math: step sizes, decays, the recurrence, norms and the mixing
// of head weights are 32-bit by definition of such a model.
//
//   selective_scan        S <- exp(-exp(a_log[h]) * d) S + d B u^T ; y = S^T C + D[h] u per head, with the step size
//                         d = softplus(dt + dt_bias[h]) taken from the token; rows hold [u (H * vdim) | B (G * N) |
//                         C (G * N)]; S (N x vdim, fp32) kept per request slot.  A workgroup owns 64 columns of one
//                         head's S for one sequence, in registers, and walks the sequence's rows in chunks staged
//                         through LDS (d * B and the decay of a row are formed once, while staging): prompt portions
//                         and single decoded rows are the same kernel
//   act_gate_group_norm   z = y * silu(gate) ; z / sqrt(mean(z^2) + eps) * w over runs of `group` columns
//   joint_norm_cache      per token: RMS norm of q over ALL heads and of k over all key heads, q times the position
//                         factor 1 + coef * ln(floor((p + 1) / every) + 1), normed k into the key rows, the projected
//                         k into the values (eight keys side by side per channel)
//   mix_heads             out[t, h] = sum_g talk[h, g] * o[t, g, kv(h)] over fp32 [T, H, G, Dv]
// The 16-bit forms of the two norm kernels give a lane 8 neighbouring columns (16-byte accesses).
#include "common.h"
#include <math.h>
#include <type_traits>

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

template <typename F> int by_dtype(int dt, F&& f) {
  switch (dt) {
    case DT_BF16: f((bf16_t*)nullptr); return 0;
    case DT_F16: f((f16_t*)nullptr); return 0;
    case DT_F32: f((float*)nullptr); return 0;
  }
  return 1;
}

__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }
__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

// ------------------------------------------------------------------------------------------------ state-space scan
// grid (sequences, heads, column tiles of 64), G waves: thread (g = tid / 64, c = tid % 64) owns rows g * R .. g * R +
// R - 1 of column c of the head's state, in registers (G * R >= N).  Per chunk of C rows: d * B and C vectors of the
// head's group, the tile's u columns and the row's decay go to LDS, the next chunk's loads are in flight while the
// current one is computed, and the G row groups' partial outputs are summed after one barrier: two barriers per chunk.
template <typename T, int R, int G, int C>
__global__ __launch_bounds__(64 * G) __attribute__((amdgpu_waves_per_eu(G >= 16 ? 8 : 1, 8))) void selective_scan_kernel(
    float* __restrict__ out, const T* __restrict__ x, long x_stride, const T* __restrict__ dt, long dt_stride,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, const float* __restrict__ d_skip,
    float* __restrict__ state, const int* __restrict__ slots, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, int H, int groups, int N, int vdim) {
  constexpr int W = G * R, TH = 64 * G;                   // W: the state size padded to the G row groups
  constexpr int NQ = C * W / TH;                          // B (and C) values a thread stages per chunk
  constexpr int NV = (C * 64 + TH - 1) / TH;
  static_assert(R % 4 == 0 && (C * W) % TH == 0 && C <= 64, "chunk does not divide over the threads");
  __shared__ __attribute__((aligned(16))) float bs[C][W];
  __shared__ __attribute__((aligned(16))) float cs[C][W];
  __shared__ float us[C][64];
  __shared__ float ds[C];
  __shared__ float part[G][C][64];
  const int b = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, g = tid >> 6, lane = tid & 63;
  const int col0 = blockIdx.z * 64;
  const bool col = col0 + lane < vdim;
  const int s = qsl[b], e = qsl[b + 1];
  if (e <= s) return;                                            // (uniform over the workgroup)
  const int start = seq_lens[b] - (e - s);
  float* st = state + ((long)slots[b] * H + h) * (long)N * vdim;
  const float a_rate = expf(a_log[h]), bias = dt_bias[h], skip = d_skip ? d_skip[h] : 0.f;
  const int grp = h / (H / groups);
  float S[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int r = g * R + i;
    S[i] = (start > 0 && col && r < N) ? st[(long)r * vdim + col0 + lane] : 0.f;
  }
  const long uoff = (long)h * vdim + col0, boff = (long)H * vdim + (long)grp * N, coff = boff + (long)groups * N;
  float pb[NQ], pc[NQ], pu[NV], pd = 1.f;
  auto step = [&](int row) { return softplus_f(ldf(dt + (long)row * dt_stride + h) + bias); };
  auto fetch = [&](int r0) {                       // rows r0 .. of the sequence into registers (zero beyond its end)
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      const int idx = tid + TH * u, t = idx / W, j = idx - t * W;
      const bool ok = r0 + t < e && j < N;
      const T* xr = x + (long)(r0 + t) * x_stride;
      pb[u] = ok ? step(r0 + t) * ldf(xr + boff + j) : 0.f;      // d * B, once per row and state channel
      pc[u] = ok ? ldf(xr + coff + j) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + TH * u, t = idx >> 6, c = idx & 63;
      const bool ok = idx < C * 64 && r0 + t < e && col0 + c < vdim;
      pu[u] = ok ? ldf(x + (long)(r0 + t) * x_stride + uoff + c) : 0.f;
    }
    if (tid < C) pd = r0 + tid < e ? expf(-a_rate * step(r0 + tid)) : 1.f;      // the row's decay
  };
  fetch(s);
  for (int r0 = s; r0 < e; r0 += C) {
    const int n = min(C, e - r0);
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      const int idx = tid + TH * u, t = idx / W, j = idx - t * W;
      bs[t][j] = pb[u];
      cs[t][j] = pc[u];
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + TH * u;
      if (idx < C * 64) us[idx >> 6][idx & 63] = pu[u];
    }
    if (tid < C) ds[tid] = pd;
    if (r0 + C < e) fetch(r0 + C);
    __syncthreads();
#pragma unroll 2
    for (int t = 0; t < n; ++t) {
      const float v = us[t][lane];
      const float d = ds[t];
      const float4* k4 = reinterpret_cast<const float4*>(&bs[t][g * R]);
      const float4* q4 = reinterpret_cast<const float4*>(&cs[t][g * R]);
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;              // (four chains: the sums do not wait for each other)
#pragma unroll
      for (int i = 0; i < R / 4; ++i) {
        const float4 kk = k4[i], qq = q4[i];
        S[4 * i] = d * S[4 * i] + kk.x * v;         a0 += S[4 * i] * qq.x;
        S[4 * i + 1] = d * S[4 * i + 1] + kk.y * v; a1 += S[4 * i + 1] * qq.y;
        S[4 * i + 2] = d * S[4 * i + 2] + kk.z * v; a2 += S[4 * i + 2] * qq.z;
        S[4 * i + 3] = d * S[4 * i + 3] + kk.w * v; a3 += S[4 * i + 3] * qq.w;
      }
      part[g][t][lane] = (a0 + a1) + (a2 + a3) + (g == 0 ? skip * v : 0.f);      // (+ D[h] u, once)
    }
    __syncthreads();
    for (int idx = tid; idx < n * 64; idx += TH) {
      const int t = idx >> 6, c = idx & 63;
      if (col0 + c < vdim) {
        float sum = 0.f;
#pragma unroll
        for (int gg = 0; gg < G; ++gg) sum += part[gg][t][c];
        out[(long)(r0 + t) * H * vdim + (long)h * vdim + col0 + c] = sum;
      }
    }
  }
  if (col) {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int r = g * R + i;
      if (r < N) st[(long)r * vdim + col0 + lane] = S[i];
    }
  }
}

// ------------------------------------------------------------------------------------------------ gate, then norm
// grid (rows, groups): z = y * silu(gate) over the group's columns, then z / sqrt(mean(z^2) + eps) * w.
template <typename T>
__global__ __launch_bounds__(256) void act_gate_group_norm_kernel(T* __restrict__ out, const float* __restrict__ y,
                                                                  const T* __restrict__ gate, long gate_stride,
                                                                  const float* __restrict__ w, float eps, int N,
                                                                  int group) {
  __shared__ float red[17];
  const long t = blockIdx.x;
  const int c0 = blockIdx.y * group;
  const float* yr = y + t * N + c0;
  const T* gr = gate + t * gate_stride + c0;
  float sq = 0.f;
  for (int i = threadIdx.x; i < group; i += blockDim.x) {
    const float gv = ldf(gr + i);
    const float z = yr[i] * (gv * sigmoid_f(gv));
    sq += z * z;
  }
  const float inv = 1.0f / sqrtf(block_sum(sq, red) / (float)group + eps);
  T* o = out + t * N + c0;
  for (int i = threadIdx.x; i < group; i += blockDim.x) {
    const float gv = ldf(gr + i);
    stf(o + i, yr[i] * (gv * sigmoid_f(gv)) * inv * w[c0 + i]);
  }
}

// the same for 16-bit gates and results with 8 columns per lane (16-byte accesses); a lane keeps up to P portions of
// 8 gated values in registers between the sum of squares and the result, so a group of up to 8 * P * blockDim columns
// is read once
template <typename T, int P>
__global__ __launch_bounds__(256) void act_gate_group_norm_vec_kernel(T* __restrict__ out, const float* __restrict__ y,
                                                                      const T* __restrict__ gate, long gate_stride,
                                                                      const float* __restrict__ w, float eps, int N,
                                                                      int group) {
  using V8 = typename Vec8<T>::type;
  __shared__ float red[17];
  const long t = blockIdx.x;
  const int c0 = blockIdx.y * group;
  const float* yr = y + t * N + c0;
  const T* gr = gate + t * gate_stride + c0;
  float z[P][8];
  float sq = 0.f;
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int i = (p * blockDim.x + threadIdx.x) * 8;
    if (i < group) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(yr + i), b = *reinterpret_cast<const f32x4*>(yr + i + 4);
      const V8 gv = ld8<T>(gr + i);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float gf = (float)gv[e];
        z[p][e] = (e < 4 ? a[e & 3] : b[e & 3]) * (gf * sigmoid_f(gf));
        sq += z[p][e] * z[p][e];
      }
    }
  }
  const float inv = 1.0f / sqrtf(block_sum(sq, red) / (float)group + eps);
  T* o = out + t * N + c0;
#pragma unroll
  for (int p = 0; p < P; ++p) {
    const int i = (p * blockDim.x + threadIdx.x) * 8;
    if (i < group) {
      const f32x4 wa = *reinterpret_cast<const f32x4*>(w + c0 + i), wb = *reinterpret_cast<const f32x4*>(w + c0 + i + 4);
      V8 r;
#pragma unroll
      for (int e = 0; e < 8; ++e) r[e] = (T)(z[p][e] * inv * (e < 4 ? wa[e & 3] : wb[e & 3]));
      st8<T>(o + i, r);
    }
  }
}

// ------------------------------------------------------------------------------------------------ q / k over all heads
// grid (rows): x row = [q (H * D) | k (G * D)].
template <typename T>
__global__ __launch_bounds__(256) void joint_norm_cache_kernel(T* __restrict__ q_out, const T* __restrict__ x,
                                                               long x_stride, const float* __restrict__ q_w,
                                                               const float* __restrict__ k_w, float eps,
                                                               const int* __restrict__ positions, float coef, int every,
                                                               T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                               const int* __restrict__ slot_mapping, int H, int G, int D,
                                                               int bs) {
  __shared__ float red[17];
  const long t = blockIdx.x;
  const T* xr = x + t * x_stride;
  const int qs = H * D, ks = G * D;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < qs; i += blockDim.x) { const float v = ldf(xr + i); sq += v * v; }
  for (int i = threadIdx.x; i < ks; i += blockDim.x) { const float v = ldf(xr + qs + i); sk += v * v; }
  sq = block_sum(sq, red);
  sk = block_sum(sk, red);
  float iq = 1.0f / sqrtf(sq / (float)qs + eps);
  const float ik = 1.0f / sqrtf(sk / (float)ks + eps);
  float temp = 1.0f;
  if (every > 0) temp = 1.0f + coef * logf((float)((positions[t] + 1) / every) + 1.0f);
  T* qo = q_out + t * qs;
  for (int i = threadIdx.x; i < qs; i += blockDim.x) stf(qo + i, ldf(xr + i) * iq * q_w[i] * temp);
  if (k_cache == nullptr) return;
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const long blk = slot / bs;
  const int off = slot % bs;
  for (int i = threadIdx.x; i < ks; i += blockDim.x) {
    const int g = i / D, d = i - g * D;
    const float v = ldf(xr + qs + i);
    stf(k_cache + ((blk * G + g) * bs + off) * (long)D + d, v * ik * k_w[i]);
    v_cache[(((blk * G + g) * (bs >> 3) + (off >> 3)) * (long)D + d) * 8 + (off & 7)] = xr[qs + i];
  }
}

// the same for 16-bit types with 8 channels per lane (16-byte loads of the row, 16-byte stores of q and of the key
// row; the values go eight 2-byte stores per lane, one per channel, into the key-grouped layout)
template <typename T>
__global__ __launch_bounds__(256) void joint_norm_cache_vec_kernel(T* __restrict__ q_out, const T* __restrict__ x,
                                                                   long x_stride, const float* __restrict__ q_w,
                                                                   const float* __restrict__ k_w, float eps,
                                                                   const int* __restrict__ positions, float coef,
                                                                   int every, T* __restrict__ k_cache,
                                                                   T* __restrict__ v_cache,
                                                                   const int* __restrict__ slot_mapping, int H, int G,
                                                                   int D, int bs) {
  using V8 = typename Vec8<T>::type;
  __shared__ float red[17];
  const long t = blockIdx.x;
  const T* xr = x + t * x_stride;
  const int qs = H * D, ks = G * D;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x * 8; i < qs + ks; i += blockDim.x * 8) {
    const V8 v = ld8<T>(xr + i);
    float a = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) a += (float)v[e] * (float)v[e];
    if (i < qs) sq += a; else sk += a;
  }
  sq = block_sum(sq, red);
  sk = block_sum(sk, red);
  float iq = 1.0f / sqrtf(sq / (float)qs + eps);
  const float ik = 1.0f / sqrtf(sk / (float)ks + eps);
  if (every > 0) iq *= 1.0f + coef * logf((float)((positions[t] + 1) / every) + 1.0f);
  const int slot = k_cache != nullptr ? slot_mapping[t] : -1;
  const long blk = slot >= 0 ? slot / bs : 0;
  const int off = slot >= 0 ? slot % bs : 0;
  T* qo = q_out + t * qs;
  for (int i = threadIdx.x * 8; i < qs + ks; i += blockDim.x * 8) {
    const V8 v = ld8<T>(xr + i);                                   // (the row is still in the cache)
    const bool is_q = i < qs;
    const float* wp = is_q ? q_w + i : k_w + (i - qs);
    const f32x4 wa = *reinterpret_cast<const f32x4*>(wp), wb = *reinterpret_cast<const f32x4*>(wp + 4);
    const float mul = is_q ? iq : ik;
    V8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (T)((float)v[e] * mul * (e < 4 ? wa[e & 3] : wb[e & 3]));
    if (is_q) {
      st8<T>(qo + i, r);
    } else if (slot >= 0) {
      const int j = i - qs, g = j / D, d = j - g * D;              // (D % 8 == 0: the 8 channels share a head)
      st8<T>(k_cache + ((blk * G + g) * bs + off) * (long)D + d, r);
      T* vd = v_cache + (((blk * G + g) * (bs >> 3) + (off >> 3)) * (long)D + d) * 8 + (off & 7);
#pragma unroll
      for (int e = 0; e < 8; ++e) vd[e * 8] = v[e];
    }
  }
}

// ------------------------------------------------------------------------------------------------ mixed head weights
// grid (rows, key / value heads): o fp32 [T, H, G, Dv]; the heads h of key / value head c each sum
// talk[h, g] * o[t, g, c] over g.  A lane owns a column d and four of those heads at a time, so every value of o is
// read once per four heads.
template <typename T>
__global__ __launch_bounds__(256) void mix_heads_kernel(T* __restrict__ out, const float* __restrict__ o,
                                                        const float* __restrict__ talk, int H, int G, int Dv) {
  const long t = blockIdx.x;
  const int c = blockIdx.y;
  const int qpg = H / G;
  const float* src = o + (t * H * G + c) * (long)Dv;               // + g * G * Dv + d
  for (int d = threadIdx.x; d < Dv; d += blockDim.x) {
    for (int h0 = 0; h0 < qpg; h0 += 4) {
      const float* tw = talk + (long)(c * qpg + h0) * H;
      const int nh = min(4, qpg - h0);
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
      for (int g = 0; g < H; ++g) {
        const float v = src[(long)g * G * Dv + d];
        a0 += tw[g] * v;
        if (nh > 1) a1 += tw[H + g] * v;
        if (nh > 2) a2 += tw[2 * H + g] * v;
        if (nh > 3) a3 += tw[3 * H + g] * v;
      }
      T* dst = out + (t * H + c * qpg + h0) * (long)Dv + d;
      stf(dst, a0);
      if (nh > 1) stf(dst + Dv, a1);
      if (nh > 2) stf(dst + 2 * (long)Dv, a2);
      if (nh > 3) stf(dst + 3 * (long)Dv, a3);
    }
  }
}

}  // namespace

// x [T, x_stride] = [u | B | C] of type dt, step sizes [T, dt_stride] (H used), out fp32 [T, H * vdim], state fp32
// [slots, H, N, vdim]; N <= 256.  max_rows: the most rows any sequence brings (0 = unknown)
VDAMD_API int vdamd_selective_scan(float* out, const void* x, long x_stride, const void* dt, long dt_stride,
                                   const float* a_log, const float* dt_bias, const float* d_skip, float* state,
                                   const int* slots, const int* qsl, const int* seq_lens, int num_seqs, int H, int groups,
                                   int N, int vdim, int max_rows, int dtype, hipStream_t stream) {
  if (num_seqs <= 0) return 0;
  if (H <= 0 || groups <= 0 || H % groups || N <= 0 || vdim <= 0 || N > 256) return 1;
  const dim3 grid(num_seqs, H, (vdim + 63) / 64);
  const int rc = by_dtype(dtype, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
#define SSM(R_, G_, C_)                                                                                            \
  hipLaunchKernelGGL((selective_scan_kernel<TT, R_, G_, C_>), grid, dim3(64 * G_), 0, stream, out, (const TT*)x,   \
                     x_stride, (const TT*)dt, dt_stride, a_log, dt_bias, d_skip, state, slots, qsl, seq_lens, H,    \
                     groups, N, vdim)
    if (max_rows > 0 && max_rows <= 2) {
      // decoded rows only: bound by reading and writing the states, so small workgroups that overlap each other
      if (N <= 32) SSM(8, 4, 8);
      else if (N <= 64) SSM(16, 4, 4);
      else if (N <= 128) SSM(32, 4, 4);
      else SSM(64, 4, 4);
    } else {
      // prompt portions: the walk over the rows is sequential, so as many waves per workgroup as the rows allow
      if (N <= 32) SSM(8, 4, 8);
      else if (N <= 64) SSM(8, 8, 8);
      else if (N <= 128) SSM(8, 16, 8);
      else SSM(16, 16, 8);
    }
#undef SSM
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

// y fp32 [T, N] contiguous, gate [T, gate_stride] and out [T, N] of type dtype, w fp32 [N]; N % group == 0
VDAMD_API int vdamd_act_gate_group_norm(void* out, const float* y, const void* gate, long gate_stride, const float* w,
                                        float eps, int T, int N, int group, int dtype, hipStream_t stream) {
  if (T <= 0) return 0;
  if (N <= 0 || group <= 0 || N % group) return 1;
  const int th = group >= 1024 ? 256 : (group >= 256 ? 128 : 64);
  const bool vec = dtype != DT_F32 && group % 8 == 0 && gate_stride % 8 == 0 && ((uintptr_t)gate & 15) == 0 &&
                   ((uintptr_t)out & 15) == 0 && ((uintptr_t)y & 15) == 0 && ((uintptr_t)w & 15) == 0 &&
                   group <= 8 * 4 * 256;
  const int rc = by_dtype(dtype, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    if constexpr (!std::is_same_v<TT, float>) {
      if (vec) {
        const int lanes = group / 8;                // a lane per 8 columns, up to 4 portions per lane
        const int tv = lanes >= 256 ? 256 : (lanes >= 128 ? 128 : 64);
        const dim3 grid(T, N / group);
        if (lanes <= tv)
          hipLaunchKernelGGL((act_gate_group_norm_vec_kernel<TT, 1>), grid, dim3(tv), 0, stream, (TT*)out, y,
                             (const TT*)gate, gate_stride, w, eps, N, group);
        else if (lanes <= 2 * tv)
          hipLaunchKernelGGL((act_gate_group_norm_vec_kernel<TT, 2>), grid, dim3(tv), 0, stream, (TT*)out, y,
                             (const TT*)gate, gate_stride, w, eps, N, group);
        else
          hipLaunchKernelGGL((act_gate_group_norm_vec_kernel<TT, 4>), grid, dim3(tv), 0, stream, (TT*)out, y,
                             (const TT*)gate, gate_stride, w, eps, N, group);
        return;
      }
    }
    hipLaunchKernelGGL((act_gate_group_norm_kernel<TT>), dim3(T, N / group), dim3(th), 0, stream, (TT*)out, y,
                       (const TT*)gate, gate_stride, w, eps, N, group);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

// x [T, x_stride] = [q (H * D) | k (G * D)], q_out [T, H * D]; caches may be null (nothing is written then):
// k_cache [blocks, G, bs, D], v_cache [blocks, G, bs / 8, D, 8]
VDAMD_API int vdamd_joint_norm_cache(void* q_out, const void* x, long x_stride, const float* q_w, const float* k_w,
                                     float eps, const int* positions, float coef, int every, void* k_cache,
                                     void* v_cache, const int* slot_mapping, int T, int H, int G, int D, int bs,
                                     int dtype, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || D <= 0 || every < 0) return 1;
  if (k_cache != nullptr && (v_cache == nullptr || slot_mapping == nullptr || bs <= 0 || bs % 8)) return 1;
  const bool vec = dtype != DT_F32 && D % 8 == 0 && x_stride % 8 == 0 && ((uintptr_t)x & 15) == 0 &&
                   ((uintptr_t)q_out & 15) == 0 && ((uintptr_t)k_cache & 15) == 0 && ((uintptr_t)q_w & 15) == 0 &&
                   ((uintptr_t)k_w & 15) == 0;
  const int rc = by_dtype(dtype, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    if constexpr (!std::is_same_v<TT, float>) {
      if (vec) {
        const int lanes = (H + G) * D / 8;
        hipLaunchKernelGGL((joint_norm_cache_vec_kernel<TT>), dim3(T), dim3(lanes >= 256 ? 256 : (lanes >= 128 ? 128 : 64)),
                           0, stream, (TT*)q_out, (const TT*)x, x_stride, q_w, k_w, eps, positions, coef, every,
                           (TT*)k_cache, (TT*)v_cache, slot_mapping, H, G, D, bs);
        return;
      }
    }
    hipLaunchKernelGGL((joint_norm_cache_kernel<TT>), dim3(T), dim3(256), 0, stream, (TT*)q_out, (const TT*)x, x_stride,
                       q_w, k_w, eps, positions, coef, every, (TT*)k_cache, (TT*)v_cache, slot_mapping, H, G, D, bs);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

// o fp32 [T, H, G, Dv], talk fp32 [H, H], out [T, H * Dv] of type dtype
VDAMD_API int vdamd_mix_heads(void* out, const float* o, const float* talk, int T, int H, int G, int Dv, int dtype,
                              hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || Dv <= 0) return 1;
  const int th = Dv >= 256 ? 256 : (Dv >= 128 ? 128 : 64);
  const int rc = by_dtype(dtype, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    hipLaunchKernelGGL((mix_heads_kernel<TT>), dim3(T, G), dim3(th), 0, stream, (TT*)out, o, talk, H, G, Dv);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}
