// Kernels of layers that mix a sequence through a short convolution and windowed attention, with fp32 arithmetic
// wherever a norm, a score, a softmax weight or the residual stream is formed:
//
//   scalar_norm            x / sqrt(mean(x^2) + eps) * g with ONE gain for the row
//   scalar_norm_residual   residual(fp32) += norm(y) * g_post ; out = norm(residual) * g_next     (one launch)
//   poly_norm              c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3,  N(u) = u / sqrt(mean(u^2) + eps)
//   conv_norm_cache        causal per-channel convolution over time of a fused [q | k | v | ..] projection (history
//                          from the chunk itself or from a per-request state slot), per-head RMS norm of q and k,
//                          value mixing, k / v into row caches, q out
//                          (the head norms are optional; with frequencies given, q and k heads are then rotated by
//                          their position, value i paired with value i + half)
//   short_conv_act         the convolution alone over the leading columns of a fused projection, through SiLU when
//                          asked, result in the activation type
//   conv_state_update      the last taps-1 projected rows of every sequence into its state slot
//   window_bias_attention  attention over the caches K [blocks, Hkv, block, D] (key rows) and V [blocks, Hkv,
//                          block / 8, Dv, 8] (8 keys side by side per channel: the V^T operand of the matrix cores
//                          is one 16-byte load): causal window that keeps the first keys (or blocks of `chunk`
//                          positions counted from the sequence's start), score cap, logarithmic
//                          distance bias, sink in the denominator, sigmoid gate on the output, online softmax in
//                          fp32.  Two kernels: a matrix-core one for bf16 (16 query rows x 32 keys per wave and
//                          step, softmax weights fed to the matrix cores as a high and a low bf16 part so that they
//                          keep fp32 precision), and a plain one (any head size, fp16 / fp32) with one wave per
//                          (token, query head)
//
// Element types: bf16 / fp16 / fp32 for activations and caches (fp32: the model runs entirely in 32-bit).
#include "common.h"
#include <math.h>
#include <type_traits>

namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p) { return (float)(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

// residual stream at its start: token row + position row, summed in fp32
template <typename T>
__global__ void embed_positions_kernel(float* __restrict__ out, const int* __restrict__ ids,
                                       const int* __restrict__ positions, const T* __restrict__ embed,
                                       const T* __restrict__ pos, int H, int vocab_rows, int pos_rows) {
  const long t = blockIdx.x;
  const int id = min(max(ids[t], 0), vocab_rows - 1), p = min(max(positions[t], 0), pos_rows - 1);
  const T* e = embed + (long)id * H;
  const T* q = pos + (long)p * H;
  float* o = out + t * (long)H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = ldf(e + i) + ldf(q + i);
}

// ------------------------------------------------------------------------------------------------ norms
template <typename TI, typename TO>
__global__ void scalar_norm_kernel(TO* __restrict__ out, const TI* __restrict__ x, const float* __restrict__ gain,
                                   float eps, int H, long x_stride) {
  __shared__ float red[17];
  const long row = blockIdx.x;
  const TI* xr = x + row * x_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) { const float f = ldf(xr + i); ss += f * f; }
  ss = block_sum(ss, red);
  const float inv = (1.0f / sqrtf(ss / (float)H + eps)) * gain[0];
  TO* orow = out + row * (long)H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) stf(orow + i, ldf(xr + i) * inv);
}

// residual += y / rms(y) * g_post ; out = residual / rms(residual) * g_next (skipped when out == nullptr)
template <typename TY, typename TO>
__global__ void scalar_norm_residual_kernel(TO* __restrict__ out, const TY* __restrict__ y, float* __restrict__ residual,
                                            const float* __restrict__ g_post, const float* __restrict__ g_next,
                                            float eps, int H, long y_stride) {
  __shared__ float red[17];
  const long row = blockIdx.x;
  const TY* yr = y + row * y_stride;
  float* rr = residual + row * (long)H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) { const float f = ldf(yr + i); ss += f * f; }
  ss = block_sum(ss, red);
  const float inv = (1.0f / sqrtf(ss / (float)H + eps)) * g_post[0];
  float s2 = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float r = rr[i] + ldf(yr + i) * inv;
    rr[i] = r;
    s2 += r * r;
  }
  if (out == nullptr) return;
  s2 = block_sum(s2, red);
  const float inv2 = (1.0f / sqrtf(s2 / (float)H + eps)) * g_next[0];
  TO* orow = out + row * (long)H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) stf(orow + i, rr[i] * inv2);      // (each thread rereads its own stores)
}

template <typename T>
__global__ void poly_norm_kernel(T* __restrict__ out, const T* __restrict__ z, const float* __restrict__ coef,
                                 float eps, int F, long z_stride) {
  __shared__ float red[17];
  const long row = blockIdx.x;
  const T* zr = z + row * z_stride;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < F; i += blockDim.x) {
    const float f = ldf(zr + i), f2 = f * f, f3 = f2 * f;
    s2 += f2; s4 += f2 * f2; s6 += f3 * f3;
  }
  s2 = block_sum(s2, red);
  s4 = block_sum(s4, red);
  s6 = block_sum(s6, red);
  const float n = (float)F;
  const float a = coef[0] / sqrtf(s2 / n + eps), b = coef[1] / sqrtf(s4 / n + eps), c = coef[2] / sqrtf(s6 / n + eps);
  const float e = coef[3];
  T* orow = out + row * (long)F;
  for (int i = threadIdx.x; i < F; i += blockDim.x) {
    const float f = ldf(zr + i), f2 = f * f;
    stf(orow + i, a * f + b * f2 + c * f2 * f + e);
  }
}


// 16-bit rows whose length and stride are multiples of 8: the same two kernels with 16-byte accesses
template <typename T>
__global__ void poly_norm_vec_kernel(T* __restrict__ out, const T* __restrict__ z, const float* __restrict__ coef,
                                     float eps, int F, long z_stride) {
  using V8 = typename Vec8<T>::type;
  __shared__ float red[17];
  const long row = blockIdx.x;
  const T* zr = z + row * z_stride;
  const int nv = F >> 3;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const V8 v = ld8<T>(zr + 8 * i);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float f = (float)v[e], f2 = f * f, f3 = f2 * f;
      s2 += f2; s4 += f2 * f2; s6 += f3 * f3;
    }
  }
  s2 = block_sum(s2, red);
  s4 = block_sum(s4, red);
  s6 = block_sum(s6, red);
  const float n = (float)F;
  const float a = coef[0] / sqrtf(s2 / n + eps), b = coef[1] / sqrtf(s4 / n + eps), c = coef[2] / sqrtf(s6 / n + eps);
  const float e0 = coef[3];
  T* orow = out + row * (long)F;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const V8 v = ld8<T>(zr + 8 * i);
    V8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float f = (float)v[e], f2 = f * f;
      o[e] = (T)(a * f + b * f2 + c * f2 * f + e0);
    }
    st8<T>(orow + 8 * i, o);
  }
}

template <typename T>
__global__ void scalar_norm_residual_vec_kernel(T* __restrict__ out, const T* __restrict__ y, float* __restrict__ residual,
                                                const float* __restrict__ g_post, const float* __restrict__ g_next,
                                                float eps, int H, long y_stride) {
  using V8 = typename Vec8<T>::type;
  __shared__ float red[17];
  const long row = blockIdx.x;
  const T* yr = y + row * y_stride;
  float* rr = residual + row * (long)H;
  const int nv = H >> 3;
  float ss = 0.f;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const V8 v = ld8<T>(yr + 8 * i);
#pragma unroll
    for (int e = 0; e < 8; ++e) { const float f = (float)v[e]; ss += f * f; }
  }
  ss = block_sum(ss, red);
  const float inv = (1.0f / sqrtf(ss / (float)H + eps)) * g_post[0];
  float s2 = 0.f;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const V8 v = ld8<T>(yr + 8 * i);
    f32x4 r0 = *reinterpret_cast<const f32x4*>(rr + 8 * i), r1 = *reinterpret_cast<const f32x4*>(rr + 8 * i + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      r0[e] += (float)v[e] * inv;
      r1[e] += (float)v[e + 4] * inv;
      s2 += r0[e] * r0[e] + r1[e] * r1[e];
    }
    *reinterpret_cast<f32x4*>(rr + 8 * i) = r0;
    *reinterpret_cast<f32x4*>(rr + 8 * i + 4) = r1;
  }
  if (out == nullptr) return;
  s2 = block_sum(s2, red);
  const float inv2 = (1.0f / sqrtf(s2 / (float)H + eps)) * g_next[0];
  T* orow = out + row * (long)H;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {                 // (each thread rereads its own stores)
    const f32x4 r0 = *reinterpret_cast<const f32x4*>(rr + 8 * i), r1 = *reinterpret_cast<const f32x4*>(rr + 8 * i + 4);
    V8 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) { o[e] = (T)(r0[e] * inv2); o[e + 4] = (T)(r1[e] * inv2); }
    st8<T>(orow + 8 * i, o);
  }
}

// ---------------------------------------------------------------------------- convolution + norm + cache write
constexpr int CONV_MAX_TAPS = 16;
constexpr int UNIT_MAX_PER_LANE = 8;        // a head is at most 64 * 8 = 512 channels wide

struct ConvArgs {
  const void* x; long x_stride;             // [T, x_stride]: [q | k | v | ...]
  const void* conv_w;                       // [taps, C] (tap-major: the taps of neighbouring channels side by side)
  void* state;                              // [slots, R, C], R = max(taps - 1, 1)
  const int* slots;                         // [B]
  const int* qsl;                           // [B + 1]
  const int* seq_lens;                      // [B]
  const int* token_seq;                     // [T] or null (token t is sequence t)
  const int* positions;                     // [T]
  const float* q_norm; const float* k_norm; // [D]
  const float* v_first;                     // [T, G * Dv] fp32 or null
  const float* v_lambda;                    // [1] or null
  float* v_keep;                            // [T, G * Dv] fp32 or null
  void* q_out;                              // [T, H, D]
  void* k_cache; void* v_cache;             // [blocks, G, bs, D | Dv] or null
  const int* slot_mapping;                  // [T]
  int T, H, G, D, Dv, taps, block_size;
  float eps;
  const float* inv_freq; int rot_half;      // [rot_half] fp32 or null: q and k heads rotated, pairs rot_half apart
};

__device__ __forceinline__ void conv_rotate(float u, float v, int pos, float freq, float& ou, float& ov) {
  const float ang = (float)pos * freq;
  const float cs = cosf(ang), sn = sinf(ang);
  ou = u * cs - v * sn;
  ov = v * cs + u * sn;
}

template <typename T>
__global__ void conv_norm_cache_kernel(ConvArgs a) {
  __shared__ float rot_lds[4][64 * UNIT_MAX_PER_LANE];
  const int t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const int s = a.token_seq ? a.token_seq[t] : t;
  const int n = a.qsl[s + 1] - a.qsl[s];
  const int pos = a.positions[t];
  const int chunk_start = a.seq_lens[s] - n;
  const int R = a.taps - 1;
  const int C = a.H * a.D + a.G * (a.D + a.Dv);
  const T* x = (const T*)a.x;
  const T* w = (const T*)a.conv_w;
  T* st = (T*)a.state + (long)a.slots[s] * (R > 0 ? R : 1) * C;
  const bool own_state = (n == 1) && R > 0;       // the only row of its sequence: this block also moves the state on
  const int slot = a.slot_mapping[t];
  const int units = a.H + 2 * a.G;
  for (int u = wave; u < units; u += nwaves) {
    int c0, width, kind, head;                    // kind 0 q, 1 k, 2 v
    if (u < a.H) { kind = 0; head = u; width = a.D; c0 = u * a.D; }
    else if (u < a.H + a.G) { kind = 1; head = u - a.H; width = a.D; c0 = a.H * a.D + head * a.D; }
    else { kind = 2; head = u - a.H - a.G; width = a.Dv; c0 = (a.H + a.G) * a.D + head * a.Dv; }
    float acc[UNIT_MAX_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < UNIT_MAX_PER_LANE; ++it) {
      const int cl = lane + it * 64;
      acc[it] = 0.f;
      if (cl < width) {
        const int c = c0 + cl;
        float hist[CONV_MAX_TAPS];                // hist[j] = input at position pos - (taps - 1 - j)
        float v = 0.f;
        for (int j = 0; j < a.taps; ++j) {
          const int back = a.taps - 1 - j;
          const int p = pos - back;
          float uv = 0.f;
          if (p >= chunk_start && p >= 0) uv = ldf(x + (long)(t - back) * a.x_stride + c);
          else if (p >= 0) uv = ldf(st + (long)(R - (chunk_start - p)) * C + c);
          hist[j] = uv;
          v += ldf(w + (long)j * C + c) * uv;
        }
        if (own_state) {
          for (int k = 0; k < R; ++k) stf(st + (long)k * C + c, hist[k + 1]);
        }
        acc[it] = v;
        ss += v * v;
      }
    }
    if (kind < 2 && a.q_norm != nullptr) {
      ss = wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)width + a.eps);
      const float* nw = kind == 0 ? a.q_norm : a.k_norm;
#pragma unroll
      for (int it = 0; it < UNIT_MAX_PER_LANE; ++it) {
        const int cl = lane + it * 64;
        if (cl < width) acc[it] = acc[it] * inv * nw[cl];
      }
    }
    if (kind < 2 && a.rot_half > 0) {             // (uniform over the wave) partners meet through the wave's LDS row
      float* rl = rot_lds[wave];
#pragma unroll
      for (int it = 0; it < UNIT_MAX_PER_LANE; ++it) {
        const int cl = lane + it * 64;
        if (cl < width) rl[cl] = acc[it];
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int it = 0; it < UNIT_MAX_PER_LANE; ++it) {
        const int cl = lane + it * 64;
        if (cl < 2 * a.rot_half) {
          const int pi = cl < a.rot_half ? cl : cl - a.rot_half;
          float ou, ov;
          conv_rotate(rl[pi], rl[pi + a.rot_half], pos, a.inv_freq[pi], ou, ov);
          acc[it] = cl < a.rot_half ? ou : ov;
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
    if (kind == 0) {
      T* q = (T*)a.q_out + ((long)t * a.H + head) * a.D;
#pragma unroll
      for (int it = 0; it < UNIT_MAX_PER_LANE; ++it) {
        const int cl = lane + it * 64;
        if (cl < width) stf(q + cl, acc[it]);
      }
      continue;
    }
    if (kind == 2) {
      const long vrow = (long)t * a.G * a.Dv + (long)head * a.Dv;
      const float lam = a.v_first ? a.v_lambda[0] : 0.f;
#pragma unroll
      for (int it = 0; it < UNIT_MAX_PER_LANE; ++it) {
        const int cl = lane + it * 64;
        if (cl < width) {
          if (a.v_keep) a.v_keep[vrow + cl] = acc[it];
          if (a.v_first) acc[it] = (1.0f - lam) * acc[it] + lam * a.v_first[vrow + cl];
        }
      }
    }
    if (slot < 0 || a.k_cache == nullptr) continue;
    const long blk = slot / a.block_size, off = slot % a.block_size;
    if (kind == 1) {
      T* dst = (T*)a.k_cache + ((blk * a.G + head) * a.block_size + off) * (long)width;
#pragma unroll
      for (int it = 0; it < UNIT_MAX_PER_LANE; ++it) {
        const int cl = lane + it * 64;
        if (cl < width) stf(dst + cl, acc[it]);
      }
    } else {                                      // [blocks, G, bs / 8, Dv, 8]
      T* dst = (T*)a.v_cache + (((blk * a.G + head) * (a.block_size >> 3) + (off >> 3)) * (long)width) * 8 + (off & 7);
#pragma unroll
      for (int it = 0; it < UNIT_MAX_PER_LANE; ++it) {
        const int cl = lane + it * 64;
        if (cl < width) stf(dst + (long)cl * 8, acc[it]);
      }
    }
  }
}


// The same for 16-bit types with head sizes that are multiples of 8: a lane owns 8 consecutive channels (16-byte
// loads and stores), a unit (one head of q, k or v) takes width / 8 lanes, and a wave carries as many units as fit
// when that is a power of two (the per-head sum of squares is then a few xor-shuffles inside the lane group).
// Wave tasks are numbered (token, task) across the grid: q and k units first, then v units.
template <typename T>
__device__ __forceinline__ void conv_vec_token(const ConvArgs& a, int t, int task, int gs_d, int upw_d, int gs_v,
                                               int upw_v, int tasks_d) {
  using V8 = typename Vec8<T>::type;
  const int lane = threadIdx.x & 63;
  const bool is_v = task >= tasks_d;
  const int gs = is_v ? gs_v : gs_d, upw = is_v ? upw_v : upw_d;
  // unit within the wave, lane within the unit (several units per wave only when gs is a power of two)
  const int sub = upw > 1 ? lane >> __builtin_ctz(gs) : lane / gs;
  const int li = upw > 1 ? lane & (gs - 1) : lane - sub * gs;
  const int unit = (is_v ? task - tasks_d : task) * upw + sub;
  const int n_units = is_v ? a.G : a.H + a.G;
  const bool live = sub < upw && unit < n_units;
  int kind, head, width, c0;
  if (is_v) { kind = 2; head = unit; width = a.Dv; c0 = (a.H + a.G) * a.D + head * a.Dv; }
  else if (unit < a.H) { kind = 0; head = unit; width = a.D; c0 = unit * a.D; }
  else { kind = 1; head = unit - a.H; width = a.D; c0 = a.H * a.D + head * a.D; }
  const int s = a.token_seq ? a.token_seq[t] : t;
  const int n = a.qsl[s + 1] - a.qsl[s];
  const int pos = a.positions[t];
  const int chunk_start = a.seq_lens[s] - n;
  const int R = a.taps - 1;
  const int C = a.H * a.D + a.G * (a.D + a.Dv);
  const T* x = (const T*)a.x;
  const T* w = (const T*)a.conv_w;
  T* st = (T*)a.state + (long)a.slots[s] * (R > 0 ? R : 1) * C;
  const bool own_state = (n == 1) && R > 0;
  const int c = c0 + 8 * li;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  if (live) {
    for (int j = 0; j < a.taps; ++j) {
      const V8 wv = ld8<T>(w + (long)j * C + c);
      const int back = a.taps - 1 - j;
      const int p = pos - back;
      V8 u;
      if (p >= chunk_start && p >= 0) u = ld8<T>(x + (long)(t - back) * a.x_stride + c);
      else if (p >= 0) u = ld8<T>(st + (long)(R - (chunk_start - p)) * C + c);
      else {
#pragma unroll
        for (int e = 0; e < 8; ++e) u[e] = (T)0.f;
      }
      if (own_state && j >= 1) st8<T>(st + (long)(j - 1) * C + c, u);     // (row j - 1 was read one turn earlier)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += (float)wv[e] * (float)u[e];
    }
  }
  if (kind < 2 && a.q_norm != nullptr) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += acc[e] * acc[e];
    if (upw == 1) ss = wave_sum(ss);
    else for (int o = gs >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
    const float inv = 1.0f / sqrtf(ss / (float)width + a.eps);
    if (live) {
      const float* nw = (kind == 0 ? a.q_norm : a.k_norm) + 8 * li;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = acc[e] * inv * nw[e];
    }
  }
  if (a.rot_half > 0 && !is_v) {                   // (uniform over the wave; rot_half is a multiple of 8 here)
    // a lane's 8 values lie wholly in the first half, the second half or the unrotated rest; the partner's 8 values
    // are rot_half / 8 lanes up or down, inside the same unit
    const int shift = a.rot_half >> 3;
    const int region = 8 * li < a.rot_half ? 0 : (8 * li < 2 * a.rot_half ? 1 : 2);
    const int src = region == 0 ? lane + shift : (region == 1 ? lane - shift : lane);
    float other[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) other[e] = __shfl(acc[e], src & 63, 64);
    if (region < 2) {
      const int p0 = 8 * li - (region == 1 ? a.rot_half : 0);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float ou, ov;
        if (region == 0) conv_rotate(acc[e], other[e], pos, a.inv_freq[p0 + e], ou, ov);
        else conv_rotate(other[e], acc[e], pos, a.inv_freq[p0 + e], ou, ov);
        acc[e] = region == 0 ? ou : ov;
      }
    }
  }
  if (!live) return;
  if (kind == 0) {
    V8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (T)acc[e];
    st8<T>((T*)a.q_out + ((long)t * a.H + head) * a.D + 8 * li, o);
    return;
  }
  if (kind == 2) {
    const long vrow = (long)t * a.G * a.Dv + (long)head * a.Dv + 8 * li;
    if (a.v_keep) {
      *reinterpret_cast<f32x4*>(a.v_keep + vrow) = f32x4{acc[0], acc[1], acc[2], acc[3]};
      *reinterpret_cast<f32x4*>(a.v_keep + vrow + 4) = f32x4{acc[4], acc[5], acc[6], acc[7]};
    }
    if (a.v_first) {
      const float lam = a.v_lambda[0];
      const f32x4 f0 = *reinterpret_cast<const f32x4*>(a.v_first + vrow);
      const f32x4 f1 = *reinterpret_cast<const f32x4*>(a.v_first + vrow + 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = (1.0f - lam) * acc[e] + lam * (e < 4 ? f0[e & 3] : f1[e & 3]);
    }
  }
  const int slot = a.slot_mapping[t];
  if (slot < 0 || a.k_cache == nullptr) return;
  long blk, off;
  if ((a.block_size & (a.block_size - 1)) == 0) { blk = slot >> __builtin_ctz(a.block_size); off = slot & (a.block_size - 1); }
  else { blk = slot / a.block_size; off = slot % a.block_size; }
  if (kind == 1) {
    V8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (T)acc[e];
    st8<T>((T*)a.k_cache + ((blk * a.G + head) * a.block_size + off) * (long)width + 8 * li, o);
  } else {                                        // [blocks, G, bs / 8, Dv, 8]: one key's column of 8 channels
    T* dst = (T*)a.v_cache + (((blk * a.G + head) * (a.block_size >> 3) + (off >> 3)) * (long)width + 8 * li) * 8 + (off & 7);
#pragma unroll
    for (int e = 0; e < 8; ++e) dst[e * 8] = (T)acc[e];
  }
}

// A wave takes one task (a group of heads) of `tok_per_wave` consecutive rows: the index loads of the next row
// overlap the arithmetic of the current one, and its taps are still in the cache.
template <typename T>
__global__ __launch_bounds__(256) void conv_norm_cache_vec_kernel(ConvArgs a, int gs_d, int upw_d, int gs_v, int upw_v,
                                                                  int tasks_d, int tasks_v, int tok_per_wave) {
  // grid (row groups / 4, tasks): no division to find the wave's place
  const long t0 = ((long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * tok_per_wave;
  const int task = blockIdx.y;
  for (int i = 0; i < tok_per_wave; ++i) {
    if (t0 + i >= a.T) return;                    // (the same for every lane of the wave)
    conv_vec_token<T>(a, (int)(t0 + i), task, gs_d, upw_d, gs_v, upw_v, tasks_d);
  }
}

// Sequences that ran two or more rows: their slot takes the last R inputs of (old state ++ this step's rows).
// One thread per (sequence, channel) reads all R before it writes any.
template <typename T>
__global__ void conv_state_update_kernel(const T* __restrict__ x, long x_stride, T* __restrict__ state,
                                         const int* __restrict__ slots, const int* __restrict__ qsl, int C, int R) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int q0 = qsl[s], n = qsl[s + 1] - q0;
  if (c >= C || n < 2) return;
  T* st = state + (long)slots[s] * R * C;
  float keep[CONV_MAX_TAPS];
  for (int k = 0; k < R; ++k) {
    const int i = n - R + k;
    keep[k] = i >= 0 ? ldf(x + (long)(q0 + i) * x_stride + c) : ldf(st + (long)(k + n) * C + c);
  }
  for (int k = 0; k < R; ++k) stf(st + (long)k * C + c, keep[k]);
}

// The convolution alone (no head structure): out[t, c] = act(bias[c] + sum_j w[j, c] * u[t - taps + 1 + j, c]) for the
// first C columns of x (plus u[t, c] itself with `residual`), history from the step's own rows or the state slot as above.  One thread per (row, channel); the 16-bit
// variant gives a thread 8 neighbouring channels (16-byte accesses).  A sequence's only row moves its state on here.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void short_conv_act_kernel(T* __restrict__ out, long out_stride, const T* __restrict__ x,
                                                             long x_stride, const T* __restrict__ w, T* __restrict__ state,
                                                             const int* __restrict__ slots, const int* __restrict__ qsl,
                                                             const int* __restrict__ seq_lens,
                                                             const int* __restrict__ token_seq,
                                                             const int* __restrict__ positions, int C, int taps, int silu,
                                                             const float* __restrict__ bias, int residual) {
  constexpr int W = VEC ? 8 : 1;
  const int t = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * W;
  if (c >= C) return;
  const int s = token_seq ? token_seq[t] : t;
  const int n = qsl[s + 1] - qsl[s];
  const int pos = positions[t];
  const int chunk_start = seq_lens[s] - n;
  const int R = taps - 1;
  T* st = state + (long)slots[s] * (R > 0 ? R : 1) * C;
  const bool own_state = (n == 1) && R > 0;
  float acc[W], cur[W];
#pragma unroll
  for (int e = 0; e < W; ++e) { acc[e] = bias ? bias[c + e] : 0.f; cur[e] = 0.f; }
  for (int j = 0; j < taps; ++j) {
    const int back = taps - 1 - j;
    const int p = pos - back;
    if constexpr (VEC) {
      using V8 = typename Vec8<T>::type;
      const V8 wv = ld8<T>(w + (long)j * C + c);
      V8 u;
      if (p >= chunk_start && p >= 0) u = ld8<T>(x + (long)(t - back) * x_stride + c);
      else if (p >= 0) u = ld8<T>(st + (long)(R - (chunk_start - p)) * C + c);
      else {
#pragma unroll
        for (int e = 0; e < 8; ++e) u[e] = (T)0.f;
      }
      if (own_state && j >= 1) st8<T>(st + (long)(j - 1) * C + c, u);       // (row j - 1 was read one turn earlier)
#pragma unroll
      for (int e = 0; e < 8; ++e) { acc[e] += (float)wv[e] * (float)u[e]; cur[e] = (float)u[e]; }
    } else {
      float u = 0.f;
      if (p >= chunk_start && p >= 0) u = ldf(x + (long)(t - back) * x_stride + c);
      else if (p >= 0) u = ldf(st + (long)(R - (chunk_start - p)) * C + c);
      if (own_state && j >= 1) stf(st + (long)(j - 1) * C + c, u);
      acc[0] += ldf(w + (long)j * C + c) * u;
      cur[0] = u;
    }
  }
  if (silu) {
#pragma unroll
    for (int e = 0; e < W; ++e) acc[e] = acc[e] / (1.0f + expf(-acc[e]));
  }
  if (residual) {                               // (the last tap's input is the row itself)
#pragma unroll
    for (int e = 0; e < W; ++e) acc[e] += cur[e];
  }
  if constexpr (VEC) {
    typename Vec8<T>::type o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (T)acc[e];
    st8<T>(out + (long)t * out_stride + c, o);
  } else {
    stf(out + (long)t * out_stride + c, acc[0]);
  }
}

// ------------------------------------------------------------------------------------------- attention
struct AttnArgs {
  const void* q;                    // [T, H, D]
  const void* k_cache; const void* v_cache;
  const int* block_table; long bt_stride;
  const int* token_seq;             // [T] or null
  const int* positions;             // [T]
  const float* bias_scale; const float* bias_rate; const float* sinks;    // [H] or null
  const void* gate; long gate_stride;                                      // [T, gate_stride] raw, or null
  void* out;                        // [T, H, Dv]
  int T, H, G, D, Dv, block_size, window, keep_first;
  float scale, softcap;
  int chunk;                        // > 0: a query sees only the keys of its own block of `chunk` positions
  int cross;                        // > 0: every query head's weights are applied to the values of EVERY key / value head,
                                    // out is fp32 [T, H, G, Dv] (blockIdx.y then counts (key head, value head(s)) pairs)
  int xcd_seqs;                     // > 0 (= sequences; grid.x == 1, grid.z padded to a multiple of 8): the workgroups of
                                    // one sequence are dealt to ONE of the chip's 8 dies (workgroups go to the dies in
                                    // turn by their linear number), so that what they all read is shared in its L2
  int key_heads;                    // > 0 (crossed, decoded rows): a workgroup's wave sets take this many KEY heads, one
                                    // each, for the same value heads, whose fragments they then share in the CU's cache
};

template <typename T, bool VEC> struct RowDot;
template <bool VEC> struct RowDot<float, VEC> {
  static __device__ __forceinline__ float run(const float* k, const float* q, int D) {
    float s = 0.f;
    if (VEC) {
      for (int d = 0; d < D; d += 4) {
        const f32x4 kv = *reinterpret_cast<const f32x4*>(k + d);
        s += kv[0] * q[d] + kv[1] * q[d + 1] + kv[2] * q[d + 2] + kv[3] * q[d + 3];
      }
    } else {
      for (int d = 0; d < D; ++d) s += k[d] * q[d];
    }
    return s;
  }
};
template <typename T, bool VEC> struct RowDot {
  static __device__ __forceinline__ float run(const T* k, const float* q, int D) {
    float s = 0.f;
    if (VEC) {
      for (int d = 0; d < D; d += 8) {
        const typename Vec8<T>::type kv = ld8<T>(k + d);
#pragma unroll
        for (int j = 0; j < 8; ++j) s += (float)kv[j] * q[d + j];
      }
    } else {
      for (int d = 0; d < D; ++d) s += (float)k[d] * q[d];
    }
    return s;
  }
};

constexpr int ATTN_MAX_WAVES = 16;
constexpr int ATTN_V_PER_LANE = 8;          // Dv <= 512

// grid (T, G, head chunks); block = waves x 64: wave w of chunk z is query head g * (H / G) + z * waves + w.
// LDS: per wave D floats of q, 64 weights, 64 value-row offsets.
template <typename T, bool VEC>
__global__ void window_bias_attention_kernel(AttnArgs a) {
  extern __shared__ float lds[];
  const int t = blockIdx.x;
  const int g = a.cross ? blockIdx.y / a.G : blockIdx.y;          // key head
  const int gv = a.cross ? blockIdx.y % a.G : g;                  // value head
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const int qpg = a.H / a.G;
  const int hl = blockIdx.z * nwaves + wave;
  if (hl >= qpg) return;                      // (no block-wide barrier below: a wave may leave)
  const int h = g * qpg + hl;
  float* sq = lds + (long)wave * (a.D + 128);
  float* sp = sq + a.D;
  long* srow = reinterpret_cast<long*>(lds + (((long)nwaves * (a.D + 128) + 1) & ~1L)) + wave * 64;
  const int s = a.token_seq ? a.token_seq[t] : t;
  const int pos = a.positions[t];
  const T* q = (const T*)a.q + ((long)t * a.H + h) * a.D;
  for (int d = lane; d < a.D; d += 64) sq[d] = ldf(q + d);
  int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
  if (a.chunk > 0) lo = max(lo, pos - pos % a.chunk);
  const int nkeep = a.window > 0 && a.chunk == 0 ? min(a.keep_first, lo) : 0;
  const int total = nkeep + (pos - lo + 1);
  const float r1 = a.bias_scale ? a.bias_scale[h] : 0.f, r2 = a.bias_rate ? a.bias_rate[h] : 0.f;
  const int* bt = a.block_table + (long)s * a.bt_stride;
  const T* kc = (const T*)a.k_cache;
  const T* vc = (const T*)a.v_cache;
  // value channels: with Dv <= 32 the lanes split the keys of a tile 2 or 4 ways as well
  const int kparts = a.Dv <= 16 ? 4 : (a.Dv <= 32 ? 2 : 1);
  const int cw = 64 / kparts;
  const int kp = lane / cw, cl0 = lane % cw;
  float acc[ATTN_V_PER_LANE];
#pragma unroll
  for (int i = 0; i < ATTN_V_PER_LANE; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  __builtin_amdgcn_wave_barrier();
  for (int f0 = 0; f0 < total; f0 += 64) {
    const int f = f0 + lane;
    float sc = -INFINITY;
    long vrow = 0;
    if (f < total) {
      const int j = f < nkeep ? f : lo + (f - nkeep);
      const long blk = bt[j / a.block_size];
      const long row = (blk * a.G + g) * a.block_size + (j % a.block_size);
      sc = RowDot<T, VEC>::run(kc + row * a.D, sq, a.D) * a.scale;
      if (a.softcap > 0.f) sc = a.softcap * tanhf(sc / a.softcap);
      if (a.bias_scale) sc -= r1 * log1pf(r2 * (float)(pos - j));
      vrow = (((blk * a.G + gv) * (a.block_size >> 3) + ((j % a.block_size) >> 3)) * (long)a.Dv) * 8 + (j & 7);
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float p = f < total ? expf(sc - m_new) : 0.f;
    const float corr = expf(m - m_new);          // (m = -inf on the first tile: exp(-inf) = 0)
    l = l * corr + wave_sum(p);
    m = m_new;
    sp[lane] = p;
    srow[lane] = vrow;
    __builtin_amdgcn_wave_barrier();
    const int cnt = min(64, total - f0);
#pragma unroll
    for (int i = 0; i < ATTN_V_PER_LANE; ++i) acc[i] *= corr;
    for (int jj = kp; jj < cnt; jj += kparts) {
      const float pj = sp[jj];
      const T* vr = vc + srow[jj];
#pragma unroll
      for (int i = 0; i < ATTN_V_PER_LANE; ++i) {
        const int c = cl0 + i * cw;
        if (c < a.Dv) acc[i] += pj * ldf(vr + (long)c * 8);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (kparts > 1) {
#pragma unroll
    for (int i = 0; i < ATTN_V_PER_LANE; ++i) {
      float v = acc[i];
      for (int o = cw; o < 64; o <<= 1) v += __shfl_xor(v, o, 64);
      acc[i] = v;
    }
  }
  if (a.sinks) {                                // exp(sink) joins the denominator, once, with no value
    const float sk = a.sinks[h];
    const float m_f = fmaxf(m, sk);
    const float corr = expf(m - m_f);
    l = l * corr + expf(sk - m_f);
#pragma unroll
    for (int i = 0; i < ATTN_V_PER_LANE; ++i) acc[i] *= corr;
  }
  float mul = 1.0f / l;
  if (a.gate) {
    const float gv = ldf((const T*)a.gate + (long)t * a.gate_stride + h);
    mul *= 1.0f / (1.0f + expf(-gv));
  }
  if (a.cross) {
    float* o = (float*)a.out + (((long)t * a.H + h) * a.G + gv) * a.Dv;
    if (kp == 0) {
#pragma unroll
      for (int i = 0; i < ATTN_V_PER_LANE; ++i) {
        const int c = cl0 + i * cw;
        if (c < a.Dv) o[c] = acc[i] * mul;
      }
    }
    return;
  }
  T* o = (T*)a.out + ((long)t * a.H + h) * a.Dv;
  if (kp == 0) {
#pragma unroll
    for (int i = 0; i < ATTN_V_PER_LANE; ++i) {
      const int c = cl0 + i * cw;
      if (c < a.Dv) stf(o + c, acc[i] * mul);
    }
  }
}


// ------------------------------------------------------------------- attention on the matrix cores (bf16)
// A wave owns 16 query rows = `tpw` consecutive tokens of one sequence x `hp` heads of one GQA group (row r: token
// r / hp, head r % hp) and walks the visible keys 32 at a time.  Per step: S^T = K Q^T (two 16-key tiles whose rows
// interleave so that a lane ends up with 8 consecutive keys of ITS query row), cap / bias / mask / online softmax in
// fp32 per lane, O^T += V^T P^T with P split into bf16 high and low parts.  Everything a query row needs (max, sum,
// rescale factor, its O^T column) lives in the lanes with l % 16 == row.  With `kw` > 1 the block's waves take the
// key steps in turn for the same rows and are merged through LDS (decode: few rows, many keys).  CG > 1 (crossed
// value heads only): the step's weights are applied to CG value heads in turn, each with accumulators of its own, so
// the scores and the softmax are computed once for all of them.
template <int DT, int VT, int CG>
__global__ __launch_bounds__(CG > 1 ? 512 : 256) void window_bias_attention_mfma_kernel(AttnArgs a, const int* __restrict__ qsl,
                                                                         const int* __restrict__ seq_lens, int hp,
                                                                         int tpw, int kw) {
  using T = bf16_t;
  using V8 = bf16x8;
  extern __shared__ float lds[];
  constexpr int D = 32 * DT, DV = 16 * VT;
  constexpr float LOG2E = 1.4426950408889634f;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const int r16 = lane & 15, g4 = lane >> 4;
  int s = blockIdx.z, by = blockIdx.y;
  if (a.xcd_seqs > 0) {
    const int linear = blockIdx.y + gridDim.y * blockIdx.z;
    const int die = linear & 7, slot = linear >> 3;
    s = die + 8 * (slot / (int)gridDim.y);
    by = slot % (int)gridDim.y;
    if (s >= a.xcd_seqs) return;                  // (the whole workgroup)
  }
  const int qpg = a.H / a.G;
  const int hchunks = (qpg + hp - 1) / hp;
  const int gy = by / hchunks, hc = by % hchunks;
  const int vchunks = a.cross ? (a.G + CG - 1) / CG : 1;
  const int tw = nwaves / kw;                     // wave sets: over tokens, or (key_heads) over key heads
  const int wt = wave / kw, wk = wave % kw;
  const int g = a.cross ? (a.key_heads > 0 ? (gy / vchunks) * a.key_heads + wt : gy / vchunks) : gy;       // key head
  const int gv0 = a.cross ? (gy % vchunks) * CG : g;          // first value head (the only one unless crossed)
  const int q0 = qsl[s], n_tok = qsl[s + 1] - q0;
  // first token (within the step's rows of the sequence) of this wave
  const int tok0 = a.key_heads > 0 ? 0 : (blockIdx.x * tw + wt) * tpw;
  if (tok0 >= n_tok && kw == 1) return;
  const bool wave_live = tok0 < n_tok;
  const int start = seq_lens[s] - n_tok;          // position of the sequence's first row in this step
  // ---- this lane's query row
  const int tl = r16 / hp, hh = r16 % hp;
  const int tok = tok0 + tl;
  const bool row_ok = wave_live && tl < tpw && tok < n_tok && hc * hp + hh < qpg;
  const int h = g * qpg + min(hc * hp + hh, qpg - 1);
  const long trow = q0 + min(tok, max(n_tok - 1, 0));
  const int pos = start + min(tok, max(n_tok - 1, 0));
  V8 qf[DT];
  {
    const T* qp = (const T*)a.q + (trow * a.H + h) * (long)D + 8 * g4;
#pragma unroll
    for (int k = 0; k < DT; ++k) {
      if (row_ok) qf[k] = ld8<T>(qp + 32 * k);
      else {
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[k][j] = (T)0.f;
      }
    }
  }
  const float r1 = a.bias_scale ? a.bias_scale[h] : 0.f;      // (r1 ln(x) on the log2 scale is r1 log2(x))
  const float r2 = a.bias_rate ? a.bias_rate[h] : 0.f;
  const float scale2 = a.scale * LOG2E;
  // ---- key steps of the wave: [0, kept) and [window start of its first row, position of its last row]
  const int p_first = start + min(tok0, max(n_tok - 1, 0));
  const int p_last = start + min(tok0 + tpw - 1, max(n_tok - 1, 0));
  int lo_min = a.window > 0 ? max(0, p_first - a.window + 1) : 0;
  if (a.chunk > 0) lo_min = max(lo_min, p_first - p_first % a.chunk);
  const int keep_first = a.chunk > 0 ? 0 : a.keep_first;
  const int nkeep = a.window > 0 ? min(keep_first, lo_min) : 0;
  int start_b = lo_min & ~31;
  int n_a = (nkeep + 31) >> 5;
  if (start_b < (n_a << 5)) { start_b = 0; n_a = 0; }
  const int n_steps = wave_live ? n_a + ((p_last - start_b) >> 5) + 1 : 0;
  const int* bt = a.block_table + (long)s * a.bt_stride;
  const T* kc = (const T*)a.k_cache;
  const T* vc = (const T*)a.v_cache;
  const int bs = a.block_size, bs8 = a.block_size >> 3;
  // block sizes are powers of two in practice: key -> (block, offset) by shift and mask instead of two divisions
  const int bs_shift = (bs & (bs - 1)) == 0 ? __builtin_ctz(bs) : -1;
  auto split = [&](int key, int& bi, int& off) {
    if (bs_shift >= 0) { bi = key >> bs_shift; off = key & (bs - 1); }
    else { bi = key / bs; off = key - bi * bs; }
  };
  f32x4 acc[CG][VT];
#pragma unroll
  for (int cc = 0; cc < CG; ++cc)
#pragma unroll
    for (int c = 0; c < VT; ++c) acc[cc][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  int lo_row = a.window > 0 ? pos - a.window + 1 : 0;
  if (a.chunk > 0) lo_row = max(lo_row, pos - pos % a.chunk);
  // a step all of whose 32 keys every row of the wave sees needs no mask: inside [window start of the wave's
  // last row, position of its first row], or inside the kept first keys
  int full_lo = a.window > 0 ? p_last - a.window + 1 : 0;
  if (a.chunk > 0) full_lo = max(full_lo, p_last - p_last % a.chunk);
  const float posf = (float)pos;
  const float cap_in = a.softcap > 0.f ? 2.f / a.softcap : 0.f, cap_out = a.softcap * LOG2E;
  // newest keys first: with a distance bias they carry the largest scores, so the running maximum settles in the
  // first steps and the accumulators are rarely rescaled afterwards
  for (int it = wk; it < n_steps; it += kw) {
    const int si = n_steps - 1 - it;
    const int base = si < n_a ? (si << 5) : start_b + ((si - n_a) << 5);
    const bool interior = base + 31 <= p_first && (base >= full_lo || base + 31 < keep_first);
    // K rows of the two interleaved tiles
    const int key0 = base + 8 * (r16 >> 2) + (r16 & 3);
    const int ka = min(key0, p_last), kb = min(key0 + 4, p_last);
    int bi_a, off_a, bi_b, off_b, bi_v, off_v;
    split(ka, bi_a, off_a);
    split(kb, bi_b, off_b);
    const long blk_a = bt[bi_a], blk_b = bt[bi_b];
    const T* kpa = kc + ((blk_a * a.G + g) * bs + off_a) * (long)D + 8 * g4;
    const T* kpb = kc + ((blk_b * a.G + g) * bs + off_b) * (long)D + 8 * g4;
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < DT; ++k) {
      s0 = mfma16(ld8<T>(kpa + 32 * k), qf[k], s0);
      s1 = mfma16(ld8<T>(kpb + 32 * k), qf[k], s1);
    }
    // V^T rows: this lane's 8 keys are base + 8 * g4 .. + 7, channel 16 * c + r16
    const int vkey = min(base + 8 * g4, p_last) & ~7;
    split(vkey, bi_v, off_v);
    const long blk_v = bt[bi_v];
    const long vhead = (long)bs8 * DV * 8;         // from a value head's fragments to the next head's
    const T* vp = vc + (((blk_v * a.G + gv0) * bs8 + (off_v >> 3)) * (long)DV + r16) * 8;
    V8 vf[VT];
#pragma unroll
    for (int c = 0; c < VT; ++c) vf[c] = ld8<T>(vp + (long)c * 128);
    const int kidx0 = base + 8 * g4;
    const float d0 = posf - (float)kidx0;          // distance of this lane's key j: d0 - j
    float p[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float sv = (j < 4 ? s0[j & 3] : s1[j & 3]) * scale2;
      if (a.softcap > 0.f) {                       // cap * tanh(s / cap) = cap * (1 - 2 / (1 + e^(2 s / cap)))
        const float e = fast_exp2(sv * cap_in);
        sv = fmaf(-2.f * cap_out, __builtin_amdgcn_rcpf(1.f + e), cap_out);
      }
      // r1 * ln(1 + r2 * dist) on the log2 scale is r1 * log2(1 + r2 * dist); v_log_f32 is log2
      if (a.bias_scale) sv = fmaf(-r1, __builtin_amdgcn_logf(fmaf(r2, d0 - (float)j, 1.f)), sv);
      p[j] = sv;
    }
    if (!interior) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int key = kidx0 + j;
        const bool seen = row_ok && key <= pos && (key >= lo_row || key < keep_first);
        p[j] = seen ? p[j] : -INFINITY;            // (also drops the NaN a negative distance gives the logarithm)
      }
    }
    float tmax = fmaxf(fmaxf(fmaxf(p[0], p[1]), fmaxf(p[2], p[3])), fmaxf(fmaxf(p[4], p[5]), fmaxf(p[6], p[7])));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m, tmax);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;       // a row with nothing visible yet: every weight 0
    const float alpha = fast_exp2(m - m_use);                    // (m = -inf: 0)
    float psum = 0.f;
    V8 ph, pl;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float e = fast_exp2(p[j] - m_use);                   // (masked: 2^-inf = 0)
      psum += e;
      const T hi = (T)e;
      ph[j] = hi;
      pl[j] = (T)(e - (float)hi);
    }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l = l * alpha + psum;
    m = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int cc = 0; cc < CG; ++cc)
#pragma unroll
        for (int c = 0; c < VT; ++c) acc[cc][c] *= alpha;
    }
#pragma unroll
    for (int cc = 0; cc < CG; ++cc) {
      V8 vn[VT];
      if (cc + 1 < CG) {                           // the next value head's fragments, in flight during this head's MFMAs
        const T* vq = vp + (long)min(cc + 1, a.G - 1 - gv0) * vhead;
#pragma unroll
        for (int c = 0; c < VT; ++c) vn[c] = ld8<T>(vq + (long)c * 128);
      }
#pragma unroll
      for (int c = 0; c < VT; ++c) {
        acc[cc][c] = mfma16(vf[c], ph, acc[cc][c]);
        acc[cc][c] = mfma16(vf[c], pl, acc[cc][c]);
      }
      if (cc + 1 < CG) {
#pragma unroll
        for (int c = 0; c < VT; ++c) vf[c] = vn[c];
      }
    }
  }
  // ---- merge the key-split waves of a row set (wave wk == 0 of each set ends up with the result): every wave
  // brings its sums to the common maximum, then wave 0 adds them up, one value head at a time
  if (kw > 1) {
    float* ml = lds;                                                    // [tw * kw * 64][2]
    float* buf = lds + (long)tw * kw * 64 * 2;                          // [tw * (kw - 1) * 64][4 * VT]: waves wk > 0
    float* mine = ml + ((long)(wt * kw + wk) * 64 + lane) * 2;
    mine[0] = m; mine[1] = l;
    __syncthreads();
    float m_all = m;
    for (int o = 0; o < kw; ++o) m_all = fmaxf(m_all, ml[((long)(wt * kw + o) * 64 + lane) * 2]);
    const float m_use = m_all == -INFINITY ? 0.f : m_all;
    float l_all = 0.f;
    for (int o = 0; o < kw; ++o) {
      const float* th = ml + ((long)(wt * kw + o) * 64 + lane) * 2;
      l_all += th[1] * fast_exp2(th[0] - m_use);
    }
    const float fs = fast_exp2(m - m_use);
    m = m_all; l = l_all;
#pragma unroll
    for (int cc = 0; cc < CG; ++cc) {
      if (wk > 0) {
        float* pa = buf + ((long)(wt * (kw - 1) + wk - 1) * 64 + lane) * (4 * VT);
#pragma unroll
        for (int c = 0; c < VT; ++c) {
          pa[4 * c] = acc[cc][c][0] * fs; pa[4 * c + 1] = acc[cc][c][1] * fs;
          pa[4 * c + 2] = acc[cc][c][2] * fs; pa[4 * c + 3] = acc[cc][c][3] * fs;
        }
      }
      __syncthreads();
      if (wk == 0) {
#pragma unroll
        for (int c = 0; c < VT; ++c) acc[cc][c] *= fs;
        for (int o = 1; o < kw; ++o) {
          const float* th = buf + ((long)(wt * (kw - 1) + o - 1) * 64 + lane) * (4 * VT);
#pragma unroll
          for (int c = 0; c < VT; ++c) {
            acc[cc][c][0] += th[4 * c]; acc[cc][c][1] += th[4 * c + 1];
            acc[cc][c][2] += th[4 * c + 2]; acc[cc][c][3] += th[4 * c + 3];
          }
        }
      }
      if (cc + 1 < CG) __syncthreads();
    }
    if (wk > 0) return;
  }
  if (!row_ok) return;
  if (a.sinks) {
    const float sk = a.sinks[h] * LOG2E;
    const float m_f = fmaxf(m, sk);
    const float fa = fast_exp2(m - m_f);
    l = l * fa + fast_exp2(sk - m_f);
#pragma unroll
    for (int c = 0; c < VT; ++c) acc[0][c] *= fa;
  }
  float mul = 1.0f / l;
  if (a.gate) {
    const float gate_v = (float)((const T*)a.gate)[trow * a.gate_stride + h];
    mul *= 1.0f / (1.0f + expf(-gate_v));
  }
  if (a.cross) {
#pragma unroll
    for (int cc = 0; cc < CG; ++cc) {
      if (gv0 + cc >= a.G) break;
      float* o = (float*)a.out + ((trow * a.H + h) * a.G + gv0 + cc) * (long)DV + 4 * g4;
#pragma unroll
      for (int c = 0; c < VT; ++c) *reinterpret_cast<f32x4*>(o + 16 * c) = acc[cc][c] * mul;
    }
    return;
  }
  T* o = (T*)a.out + (trow * a.H + h) * (long)DV + 4 * g4;
#pragma unroll
  for (int c = 0; c < VT; ++c) {
    bf16x4 ov;
#pragma unroll
    for (int i = 0; i < 4; ++i) ov[i] = (T)(acc[0][c][i] * mul);
    *reinterpret_cast<bf16x4*>(o + 16 * c) = ov;
  }
}

template <typename F> int by_dtype(int dt, F&& f) {
  switch (dt) {
    case DT_BF16: f((bf16_t*)nullptr); return 0;
    case DT_F16: f((f16_t*)nullptr); return 0;
    case DT_F32: f((float*)nullptr); return 0;
  }
  return 1;
}

int norm_threads(int h) { return h >= 2048 ? 512 : (h >= 512 ? 256 : 128); }

}  // namespace

VDAMD_API int vdamd_embed_positions(float* out, const int* ids, const int* positions, const void* embed, const void* pos,
                                    int T, int H, int vocab_rows, int pos_rows, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || vocab_rows <= 0 || pos_rows <= 0) return 1;
  return by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    hipLaunchKernelGGL((embed_positions_kernel<TT>), dim3(T), dim3(norm_threads(H)), 0, stream, out, ids, positions,
                       (const TT*)embed, (const TT*)pos, H, vocab_rows, pos_rows);
  });
}

// out[rows, H] (dtype out_dt) = x[rows, x_stride..] (dtype in_dt) normalised with one gain
VDAMD_API int vdamd_scalar_norm(void* out, const void* x, const float* gain, float eps, int rows, int H, long x_stride,
                                int in_dt, int out_dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H <= 0) return 1;
  const int th = norm_threads(H);
  int inner = 0;
  const int rc = by_dtype(in_dt, [&](auto* ti) {
    using TI = std::remove_pointer_t<decltype(ti)>;
    inner = by_dtype(out_dt, [&](auto* to) {
      using TO = std::remove_pointer_t<decltype(to)>;
      hipLaunchKernelGGL((scalar_norm_kernel<TI, TO>), dim3(rows), dim3(th), 0, stream, (TO*)out, (const TI*)x, gain,
                         eps, H, x_stride);
    });
  });
  return rc | inner;
}

VDAMD_API int vdamd_scalar_norm_residual(void* out, const void* y, float* residual, const float* g_post,
                                         const float* g_next, float eps, int rows, int H, long y_stride, int y_dt,
                                         int out_dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || (out != nullptr && g_next == nullptr)) return 1;
  const int th = norm_threads(H);
  int inner = 0;
  if (y_dt != DT_F32 && y_dt == out_dt && H % 8 == 0 && y_stride % 8 == 0) {
    return by_dtype(y_dt, [&](auto* ty) {
      using TY = std::remove_pointer_t<decltype(ty)>;
      if constexpr (!std::is_same_v<TY, float>)
        hipLaunchKernelGGL((scalar_norm_residual_vec_kernel<TY>), dim3(rows), dim3(H >= 2048 ? 256 : 128), 0, stream,
                           (TY*)out, (const TY*)y, residual, g_post, g_next, eps, H, y_stride);
    });
  }
  const int rc = by_dtype(y_dt, [&](auto* ty) {
    using TY = std::remove_pointer_t<decltype(ty)>;
    inner = by_dtype(out_dt, [&](auto* to) {
      using TO = std::remove_pointer_t<decltype(to)>;
      hipLaunchKernelGGL((scalar_norm_residual_kernel<TY, TO>), dim3(rows), dim3(th), 0, stream, (TO*)out,
                         (const TY*)y, residual, g_post, g_next, eps, H, y_stride);
    });
  });
  return rc | inner;
}

VDAMD_API int vdamd_poly_norm(void* out, const void* z, const float* coef, float eps, int rows, int F, long z_stride,
                              int dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (F <= 0) return 1;
  const int th = norm_threads(F);
  const bool vec = dt != DT_F32 && F % 8 == 0 && z_stride % 8 == 0;
  return by_dtype(dt, [&](auto* tp) {
    using T = std::remove_pointer_t<decltype(tp)>;
    if constexpr (!std::is_same_v<T, float>) {
      if (vec) {
        hipLaunchKernelGGL((poly_norm_vec_kernel<T>), dim3(rows), dim3(F >= 4096 ? 512 : 256), 0, stream, (T*)out,
                           (const T*)z, coef, eps, F, z_stride);
        return;
      }
    }
    hipLaunchKernelGGL((poly_norm_kernel<T>), dim3(rows), dim3(th), 0, stream, (T*)out, (const T*)z, coef, eps, F,
                       z_stride);
  });
}

VDAMD_API int vdamd_conv_norm_cache(const void* x, long x_stride, const void* conv_w, void* state, const int* slots,
                                    const int* qsl, const int* seq_lens, const int* token_seq, const int* positions,
                                    const float* q_norm, const float* k_norm, const float* v_first,
                                    const float* v_lambda, float* v_keep, void* q_out, void* k_cache, void* v_cache,
                                    const int* slot_mapping, int T, int B, int H, int G, int D, int Dv, int taps,
                                    int block_size, float eps, int update_multi, const float* inv_freq, int rot_half,
                                    int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (taps < 1 || taps > CONV_MAX_TAPS || D > 64 * UNIT_MAX_PER_LANE || Dv > 64 * UNIT_MAX_PER_LANE || H % G ||
      block_size <= 0 || (v_first != nullptr && v_lambda == nullptr) || (q_norm == nullptr) != (k_norm == nullptr) ||
      rot_half < 0 || 2 * rot_half > D || (rot_half > 0 && inv_freq == nullptr))
    return 1;
  ConvArgs a{x, x_stride, conv_w, state, slots, qsl, seq_lens, token_seq, positions, q_norm, k_norm, v_first, v_lambda,
             v_keep, q_out, k_cache, v_cache, slot_mapping, T, H, G, D, Dv, taps, block_size, eps, inv_freq, rot_half};
  const int units = H + 2 * G;
  const int waves = units >= 4 ? 4 : units;
  const int C = H * D + G * (D + Dv), R = taps - 1;
  const bool vec = dt != DT_F32 && D % 8 == 0 && Dv % 8 == 0 && D <= 512 && Dv <= 512 && x_stride % 8 == 0 &&
                   rot_half % 8 == 0;
  auto pack = [](int width, int& gs, int& upw) {        // lanes per unit, units per wave
    gs = width / 8;
    upw = (gs & (gs - 1)) == 0 ? 64 / gs : 1;
  };
  return by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    if constexpr (!std::is_same_v<TT, float>) {
      if (vec) {
        int gs_d, upw_d, gs_v, upw_v;
        pack(D, gs_d, upw_d);
        pack(Dv, gs_v, upw_v);
        const int tasks_d = (H + G + upw_d - 1) / upw_d, tasks_v = (G + upw_v - 1) / upw_v;
        const int tok_per_wave = T >= 4096 ? 4 : (T >= 1024 ? 2 : 1);
        const int groups = (T + tok_per_wave - 1) / tok_per_wave;
        hipLaunchKernelGGL((conv_norm_cache_vec_kernel<TT>), dim3((groups + 3) / 4, tasks_d + tasks_v), dim3(256), 0,
                           stream, a, gs_d, upw_d, gs_v, upw_v, tasks_d, tasks_v, tok_per_wave);
      }
    }
    if (!vec || std::is_same_v<TT, float>)
      hipLaunchKernelGGL((conv_norm_cache_kernel<TT>), dim3(T), dim3(64 * waves), 0, stream, a);
    if (update_multi && R > 0)
      hipLaunchKernelGGL((conv_state_update_kernel<TT>), dim3((C + 255) / 256, B), dim3(256), 0, stream,
                         (const TT*)x, x_stride, (TT*)state, slots, qsl, C, R);
  });
}

// out [T, out_stride] = act(conv over time of x[:, :C]); state [slots, max(taps - 1, 1), C] moves on.  update_multi: 0
// when every sequence of the step has one row
VDAMD_API int vdamd_short_conv_act(void* out, long out_stride, const void* x, long x_stride, const void* conv_w,
                                   void* state, const int* slots, const int* qsl, const int* seq_lens,
                                   const int* token_seq, const int* positions, int T, int B, int C, int taps, int silu,
                                   int update_multi, const float* bias, int residual, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (taps < 1 || taps > CONV_MAX_TAPS || C <= 0) return 1;
  const int R = taps - 1;
  const bool vec = dt != DT_F32 && C % 8 == 0 && x_stride % 8 == 0 && out_stride % 8 == 0 &&
                   ((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0;
  return by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    bool done = false;
    if constexpr (!std::is_same_v<TT, float>) {
      if (vec) {
        hipLaunchKernelGGL((short_conv_act_kernel<TT, true>), dim3(T, (C / 8 + 255) / 256), dim3(256), 0, stream,
                           (TT*)out, out_stride, (const TT*)x, x_stride, (const TT*)conv_w, (TT*)state, slots, qsl,
                           seq_lens, token_seq, positions, C, taps, silu, bias, residual);
        done = true;
      }
    }
    if (!done)
      hipLaunchKernelGGL((short_conv_act_kernel<TT, false>), dim3(T, (C + 255) / 256), dim3(256), 0, stream, (TT*)out,
                         out_stride, (const TT*)x, x_stride, (const TT*)conv_w, (TT*)state, slots, qsl, seq_lens,
                         token_seq, positions, C, taps, silu, bias, residual);
    if (update_multi && R > 0)
      hipLaunchKernelGGL((conv_state_update_kernel<TT>), dim3((C + 255) / 256, B), dim3(256), 0, stream,
                         (const TT*)x, x_stride, (TT*)state, slots, qsl, C, R);
  });
}

namespace {

template <int DT, int CG> int launch_mfma(int vt, dim3 grid, dim3 block, size_t lds, hipStream_t stream,
                                          const AttnArgs& a, const int* qsl, const int* seq_lens, int hp, int tpw,
                                          int kw) {
  switch (vt) {
#define VDAMD_CASE(VT_)                                                                                              \
  case VT_:                                                                                                          \
    if constexpr (CG * VT_ <= 32) {                                                                                  \
      hipLaunchKernelGGL((window_bias_attention_mfma_kernel<DT, VT_, CG>), grid, block, lds, stream, a, qsl,         \
                         seq_lens, hp, tpw, kw);                                                                     \
      return 0;                                                                                                      \
    }                                                                                                                \
    return 1;
    VDAMD_CASE(1) VDAMD_CASE(2) VDAMD_CASE(4) VDAMD_CASE(8)
#undef VDAMD_CASE
  }
  return 1;
}

int compute_units() {
  static int n = 0;
  if (n == 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0)
      v = 256;
    n = v;
  }
  return n;
}

// value heads a workgroup of the crossed form takes: as many as share one computation of the scores without the
// accumulators (CG * Dv / 16 vectors of four) outgrowing the register file
int cross_group(int G, int vtiles) {
  int cg = G >= 3 ? 4 : (G == 2 ? 2 : 1);
  while (cg > 1 && cg * vtiles > 32) cg >>= 1;
  return cg;
}

}  // namespace

// q [T, H, D]; sequence b owns rows qsl[b] .. qsl[b + 1], the last positions of its seq_lens[b] tokens
// (token_seq / positions say the same per row, for the kernel that walks rows).  use_mfma: 0 never, 1 when the
// shape allows (bf16, D a multiple of 32 up to 256, Dv in {16, 32, 64, 128}).  cross: 0, or the most value heads
// (1, 2 or 4) that may share one computation of the scores in the crossed form.
VDAMD_API int vdamd_window_bias_attention(const void* q, const void* k_cache, const void* v_cache,
                                          const int* block_table, long bt_stride, const int* token_seq,
                                          const int* positions, const int* qsl, const int* seq_lens,
                                          const float* bias_scale, const float* bias_rate, const float* sinks,
                                          const void* gate, long gate_stride, void* out, int T, int B, int H, int G,
                                          int D, int Dv, int block_size, int window, int keep_first,
                                          int max_query_len, float scale, float softcap, int use_mfma, int chunk,
                                          int cross, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H % G || D <= 0 || Dv <= 0 || Dv > 64 * ATTN_V_PER_LANE || block_size <= 0 || block_size % 8 ||
      (bias_scale && !bias_rate) || chunk < 0 || (cross && (gate || sinks)))
    return 1;
  AttnArgs a{q, k_cache, v_cache, block_table, bt_stride, token_seq, positions, bias_scale, bias_rate, sinks, gate,
             gate_stride, out, T, H, G, D, Dv, block_size, window, keep_first, scale, softcap, chunk, cross ? 1 : 0, 0, 0};
  const int gy = cross ? G * G : G;               // key heads, or (key head, value head) pairs
  const int qpg = H / G;
  const int dtiles = D / 32, vtiles = Dv / 16;
  if (use_mfma && dt == DT_BF16 && qsl && seq_lens && B > 0 && max_query_len > 0 && D % 32 == 0 && Dv % 16 == 0 &&
      (dtiles == 1 || dtiles == 2 || dtiles == 4 || dtiles == 8) &&
      (vtiles == 1 || vtiles == 2 || vtiles == 4 || vtiles == 8)) {
    const int hp = qpg < 16 ? qpg : 16;
    const int tpw = 16 / hp;
    const int hchunks = (qpg + hp - 1) / hp;
    int tw = 4, kw = 1;
    if (max_query_len <= tpw) { tw = 1; kw = 4; }          // few rows, many keys: the waves share the keys
    const int cg = cross ? (cross_group(G, vtiles) < cross ? cross_group(G, vtiles) : cross) : 1;
    // crossed, decoded rows: the wave sets of a workgroup take 4 key heads for the same value heads and split each
    // head's keys in two, so a value head is fetched once per workgroup instead of once per key head - where that
    // still leaves a workgroup for every CU (fewer, longer walks over the keys lose more than the fetches save)
    int key_heads = (cross && cg > 1 && max_query_len <= tpw && G % 4 == 0) ? 4 : 0;
    if (key_heads > 0 && (long)B * (G / key_heads) * ((G + cg - 1) / cg) * hchunks < compute_units()) key_heads = 0;
    if (key_heads > 0) { tw = key_heads; kw = 2; }
    const int gx = key_heads > 0 ? 1 : (max_query_len + tw * tpw - 1) / (tw * tpw);
    const size_t lds = kw > 1 ? (size_t)tw * 64 * (2 * kw + 4 * vtiles * (kw - 1)) * sizeof(float) : 0;
    a.key_heads = key_heads;
    // (key head(s), group of value heads)
    const int pairs = cross ? (key_heads > 0 ? G / key_heads : G) * ((G + cg - 1) / cg) : G;
    dim3 grid(gx, pairs * hchunks, B), block(64 * tw * kw);
    if (cross && gx == 1 && pairs * hchunks > 1) {          // decoded rows: a sequence's workgroups on one die
      a.xcd_seqs = B;
      grid.z = (B + 7) / 8 * 8;
    }
#define VDAMD_DT(DT_)                                                                                          \
  case DT_:                                                                                                    \
    if (cg == 4) return launch_mfma<DT_, 4>(vtiles, grid, block, lds, stream, a, qsl, seq_lens, hp, tpw, kw);  \
    if (cg == 2) return launch_mfma<DT_, 2>(vtiles, grid, block, lds, stream, a, qsl, seq_lens, hp, tpw, kw);  \
    return launch_mfma<DT_, 1>(vtiles, grid, block, lds, stream, a, qsl, seq_lens, hp, tpw, kw);
    switch (dtiles) { VDAMD_DT(1) VDAMD_DT(2) VDAMD_DT(4) VDAMD_DT(8) }
#undef VDAMD_DT
  }
  const int waves = qpg < ATTN_MAX_WAVES ? qpg : ATTN_MAX_WAVES;
  const int chunks = (qpg + waves - 1) / waves;
  const size_t lds = (((size_t)waves * (D + 128) + 1) & ~(size_t)1) * sizeof(float) + (size_t)waves * 64 * sizeof(long);
  if (lds > 64 * 1024) return 2;
  const bool vec = dt == DT_F32 ? (D % 4 == 0) : (D % 8 == 0);
  return by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    if (vec)
      hipLaunchKernelGGL((window_bias_attention_kernel<TT, true>), dim3(T, gy, chunks), dim3(64 * waves), lds, stream, a);
    else
      hipLaunchKernelGGL((window_bias_attention_kernel<TT, false>), dim3(T, gy, chunks), dim3(64 * waves), lds, stream, a);
  });
}
