// Kernels for models that keep an fp32 residual stream between layer norms with weight and bias and mix sequences
// with decayed linear attention and with latent attention over one row cache, gfx950.  Compiled without fast-math:
// norms, rotations, scores, softmax weights and the recurrence are 32-bit by definition of such a model.
//
//   embed_scaled             token row * scale -> fp32 residual stream
//   layer_norm_to            (x - mean) / sqrt(var + eps) * w + b of rows of any float type, result in any
//   add_layer_norm           residual(fp32) += y ; out = layer norm of the sum                         (one launch)
//   decay_linear_attention   S <- decay[h] S + k v^T ; o = S^T q per head, q / k / v read (through SiLU) from a fused
//                            projection, S (dim x vdim, fp32) kept per request slot.  A workgroup owns 64 columns of
//                            one head's S for one sequence, in registers (up to 16 waves x dim/16 rows each), and walks
//                            the sequence's rows in chunks staged through LDS: prompt portions and single decoded rows
//                            are the same kernel (launches of decoded rows only take small workgroups)
//   gated_rms_norm           o / sqrt(mean(o^2) + eps) * w * sigmoid(g) * scale, over whole rows or over runs of `group`
//                            values (heads) that share w
//   clamped_glu              min(g, L) sigmoid(alpha min(g, L)) (clamp(u, -L, L) + 1) over [g | u]
//   relu_squared             max(x, 0)^2
//   expert_epilogue          routed + x * (weights of the chosen identity experts) + shared * sigmoid(gate)
//   latent_prep              per token: RMS norm of the latent and rotation of the shared key part into the row cache;
//                            the query [q_lat | rotated q_rope] assembled; angles = position * frequency in fp32
//   latent_row_attention     causal softmax attention of every head over the shared rows (value = a row's first
//                            `rank` values): one wave per (token, head), a lane per key for the scores, lanes over
//                            the value's columns for the weighted sum, online softmax; any sizes, any float type;
//                            optionally a sliding window, a sink per head in the denominator, a sigmoid gate per head
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

int row_threads(int h) { return h >= 2048 ? 512 : (h >= 512 ? 256 : 128); }

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

template <typename T>
__global__ void embed_scaled_kernel(float* __restrict__ out, const int* __restrict__ ids, const T* __restrict__ embed,
                                    float scale, int H, int vocab_rows) {
  const long t = blockIdx.x;
  const int id = min(max(ids[t], 0), vocab_rows - 1);
  const T* e = embed + (long)id * H;
  float* o = out + t * (long)H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = ldf(e + i) * scale;
}

// ------------------------------------------------------------------------------------------------ layer norms
// y == nullptr: plain norm of x (type TX, row stride x_stride).  Otherwise x is the fp32 residual stream, updated in
// place to x + y before it is normed.
template <typename TX, typename TY, typename TO>
__global__ void layer_norm_kernel(TO* __restrict__ out, TX* __restrict__ x, long x_stride, const TY* __restrict__ y,
                                  long y_stride, const float* __restrict__ w, const float* __restrict__ b, float eps,
                                  int H) {
  __shared__ float red[17];
  const long row = blockIdx.x;
  TX* xr = x + row * x_stride;
  float sum = 0.f;
  if (y != nullptr) {
    if constexpr (std::is_same_v<TX, float>) {
      const TY* yr = y + row * y_stride;
      for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float r = xr[i] + ldf(yr + i);
        xr[i] = r;                                         // (each thread rereads only its own stores below)
        sum += r;
      }
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) sum += ldf(xr + i);
  }
  const float mean = block_sum(sum, red) / (float)H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) { const float d = ldf(xr + i) - mean; ss += d * d; }
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)H + eps);
  TO* orow = out + row * (long)H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    stf(orow + i, (ldf(xr + i) - mean) * inv * w[i] + (b != nullptr ? b[i] : 0.f));
}

template <typename TG, typename TO>
__global__ void gated_rms_norm_kernel(TO* __restrict__ out, long out_stride, const float* __restrict__ o,
                                      const float* __restrict__ w, const TG* __restrict__ gate, long gate_stride,
                                      float eps, int N, float scale) {
  __shared__ float red[17];
  const long row = blockIdx.x;
  const float* orow = o + row * (long)N;
  const TG* g = gate + row * gate_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < N; i += blockDim.x) { const float f = orow[i]; ss += f * f; }
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)N + eps);
  TO* dst = out + row * out_stride;
  for (int i = threadIdx.x; i < N; i += blockDim.x) stf(dst + i, orow[i] * inv * w[i] * sigmoid_f(ldf(g + i)) * scale);
}

// the norm over runs of `group` values (one head each) that share w[group]: a wave per run, rows x runs of work
template <typename TG, typename TO>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(TO* __restrict__ out, long out_stride,
                                                               const float* __restrict__ o, const float* __restrict__ w,
                                                               const TG* __restrict__ gate, long gate_stride, float eps,
                                                               int rows, int N, int group, float scale) {
  const int lane = threadIdx.x & 63;
  const int per_row = N / group;
  const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= (long)rows * per_row) return;
  const long row = unit / per_row;
  const int c0 = (int)(unit - row * per_row) * group;
  const float* orow = o + row * (long)N + c0;
  float ss = 0.f;
  for (int i = lane; i < group; i += 64) { const float f = orow[i]; ss += f * f; }
  const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)group + eps);
  const TG* g = gate + row * gate_stride + c0;
  TO* dst = out + row * out_stride + c0;
  for (int i = lane; i < group; i += 64) stf(dst + i, orow[i] * inv * w[i] * sigmoid_f(ldf(g + i)) * scale);
}

// the same for 16-bit gate and result and runs of 8 L values, L a power of two up to 64: L neighbouring lanes per run, 8
// values per lane in 16-byte accesses, the sum of squares over the L lanes by xor-shuffles (every lane takes part: the
// lanes past the last run repeat it and store nothing)
template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_vec_kernel(T* __restrict__ out, long out_stride,
                                                                   const float* __restrict__ o,
                                                                   const float* __restrict__ w,
                                                                   const T* __restrict__ gate, long gate_stride,
                                                                   float eps, long units, int N, int group, int L,
                                                                   float scale) {
  using V8 = typename Vec8<T>::type;
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  const long unit = idx / L;
  const int l = (int)(idx - unit * L);
  const bool ok = unit < units;
  const long u = ok ? unit : units - 1;
  const int per_row = N / group;
  const long row = u / per_row;
  const int c0 = (int)(u - row * per_row) * group + 8 * l;
  const float4* o4 = reinterpret_cast<const float4*>(o + row * (long)N + c0);
  const float4 a = o4[0], b = o4[1];
  float ss = a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w + b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
  for (int off = 1; off < L; off <<= 1) ss += __shfl_xor(ss, off, 64);
  const float inv = 1.0f / sqrtf(ss / (float)group + eps) * scale;
  const float4* w4 = reinterpret_cast<const float4*>(w + 8 * l);
  const float4 wa = w4[0], wb = w4[1];
  const V8 gv = ld8<T>(gate + row * gate_stride + c0);
  const float of[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
  const float wf[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
  V8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (T)(of[e] * inv * wf[e] * sigmoid_f((float)gv[e]));
  if (ok) st8<T>(out + row * out_stride + c0, r);
}

// 16-bit gate and result, rows whose length and gate stride are multiples of 8: 16-byte accesses
template <typename T>
__global__ void gated_rms_norm_vec_kernel(T* __restrict__ out, const float* __restrict__ o, const float* __restrict__ w,
                                          const T* __restrict__ gate, long gate_stride, float eps, int N) {
  using V8 = typename Vec8<T>::type;
  __shared__ float red[17];
  const long row = blockIdx.x;
  const float4* o4 = reinterpret_cast<const float4*>(o + row * (long)N);
  const float4* w4 = reinterpret_cast<const float4*>(w);
  const T* g = gate + row * gate_stride;
  const int nv = N >> 3;
  float ss = 0.f;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const float4 a = o4[2 * i], b = o4[2 * i + 1];
    ss += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w + b.x * b.x + b.y * b.y + b.z * b.z + b.w * b.w;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)N + eps);
  T* dst = out + row * (long)N;
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const float4 a = o4[2 * i], b = o4[2 * i + 1], wa = w4[2 * i], wb = w4[2 * i + 1];
    const V8 gv = ld8<T>(g + 8 * i);
    const float of[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    const float wf[8] = {wa.x, wa.y, wa.z, wa.w, wb.x, wb.y, wb.z, wb.w};
    V8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (T)(of[e] * inv * wf[e] * sigmoid_f((float)gv[e]));
    st8<T>(dst + 8 * i, r);
  }
}

// ------------------------------------------------------------------------------------------------ activations
template <typename T>
__global__ void clamped_glu_kernel(T* __restrict__ out, const T* __restrict__ h, long h_stride, int F, float limit,
                                   float alpha) {
  const long row = blockIdx.x;
  const T* hr = h + row * h_stride;
  T* o = out + row * (long)F;
  for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < F; i += gridDim.y * blockDim.x) {
    const float g = fminf(ldf(hr + i), limit);
    const float u = fminf(fmaxf(ldf(hr + F + i), -limit), limit);
    stf(o + i, g * sigmoid_f(alpha * g) * (u + 1.0f));
  }
}

// 16-bit rows whose length and stride are multiples of 8: 16-byte accesses
template <typename T>
__global__ void clamped_glu_vec_kernel(T* __restrict__ out, const T* __restrict__ h, long h_stride, int F, float limit,
                                       float alpha) {
  using V8 = typename Vec8<T>::type;
  const long row = blockIdx.x;
  const T* hr = h + row * h_stride;
  T* o = out + row * (long)F;
  for (int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8; i < F; i += gridDim.y * blockDim.x * 8) {
    const V8 gv = ld8<T>(hr + i), uv = ld8<T>(hr + F + i);
    V8 r;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float g = fminf((float)gv[e], limit);
      const float u = fminf(fmaxf((float)uv[e], -limit), limit);
      r[e] = (T)(g * sigmoid_f(alpha * g) * (u + 1.0f));
    }
    st8<T>(o + i, r);
  }
}

// out = routed + x * (sum of the weights of the chosen outputs that are identity experts) + shared * sigmoid(gate):
// what follows the routed experts of a block with identity experts and a gated shared expert, in one pass
template <typename T>
__global__ void expert_epilogue_kernel(T* __restrict__ out, const T* __restrict__ routed, const T* __restrict__ x,
                                       long x_stride, const float* __restrict__ topw, const int* __restrict__ topi,
                                       int k, int real_experts, const T* __restrict__ shared,
                                       const T* __restrict__ gate, long gate_stride, int H, bool vec) {
  const long row = blockIdx.x;
  float share = 0.f;
  if (topw != nullptr)
    for (int j = 0; j < k; ++j)
      if (topi[row * k + j] >= real_experts) share += topw[row * k + j];
  const float g = gate != nullptr ? sigmoid_f(ldf(gate + row * gate_stride)) : 0.f;
  const T* rr = routed + row * (long)H;
  const T* xr = x + row * x_stride;
  const T* sr = shared != nullptr ? shared + row * (long)H : nullptr;
  T* o = out + row * (long)H;
  if constexpr (!std::is_same_v<T, float>) {
    if (vec) {
      using V8 = typename Vec8<T>::type;
      for (int i = threadIdx.x * 8; i < H; i += blockDim.x * 8) {
        const V8 rv = ld8<T>(rr + i), xv = ld8<T>(xr + i);
        V8 sv = rv, res;
        if (sr != nullptr) sv = ld8<T>(sr + i);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          res[e] = (T)((float)rv[e] + (float)xv[e] * share + (sr != nullptr ? (float)sv[e] * g : 0.f));
        st8<T>(o + i, res);
      }
      return;
    }
  }
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    stf(o + i, ldf(rr + i) + ldf(xr + i) * share + (sr != nullptr ? ldf(sr + i) * g : 0.f));
}

template <typename T>
__global__ void relu_squared_kernel(T* __restrict__ out, const T* __restrict__ x, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    const float f = fmaxf(ldf(x + i), 0.f);
    stf(out + i, f * f);
  }
}

// ------------------------------------------------------------------------------------------------ linear attention
// grid (sequences, heads, column tiles of 64), G waves: thread (g = tid / 64, c = tid % 64) owns rows
// g * R .. g * R + R - 1 of column c of the head's state, in registers (G * R >= dim).  x rows hold [q (H * dim) | k (H * dim) |
// v (H * vdim) | ..].  The sequence's rows are walked in chunks of C: q / k (all of the head) and v (this
// tile's columns) of a chunk are staged in LDS through SiLU, the next chunk's loads are in flight while the current
// one is computed, and the G row groups' partial outputs of a chunk are summed after one barrier - two barriers
// per chunk whatever its length, so a single decoded row and a long prompt portion are the same launch.
template <typename T, int R, int G, int C>
__global__ __launch_bounds__(64 * G) __attribute__((amdgpu_waves_per_eu(G >= 16 ? 8 : 1, 8))) void decay_linear_attention_kernel(
    float* __restrict__ out, const T* __restrict__ x, long x_stride, const float* __restrict__ decay,
    float* __restrict__ state, const int* __restrict__ slots, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, int H, int dim, int vdim, int silu) {
  constexpr int W = G * R, TH = 64 * G;                   // W: the key size padded to the G row groups
  constexpr int NQ = C * W / TH;                          // q (and k) values a thread stages per chunk
  constexpr int NV = (C * 64 + TH - 1) / TH;              // (with more threads than v values, the first ones stage)
  static_assert(R % 4 == 0 && (C * W) % TH == 0, "chunk does not divide over the threads");
  __shared__ __attribute__((aligned(16))) float qs[C][W];
  __shared__ __attribute__((aligned(16))) float ks[C][W];
  __shared__ float vs[C][64];
  __shared__ float part[G][C][64];
  const int b = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, g = tid >> 6, lane = tid & 63;
  const int col0 = blockIdx.z * 64;
  const bool col = col0 + lane < vdim;
  const int s = qsl[b], e = qsl[b + 1];
  if (e <= s) return;                                            // (uniform over the workgroup)
  const int start = seq_lens[b] - (e - s);
  float* st = state + ((long)slots[b] * H + h) * (long)dim * vdim;
  const float d = decay[h];
  float S[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int r = g * R + i;
    S[i] = (start > 0 && col && r < dim) ? st[(long)r * vdim + col0 + lane] : 0.f;
  }
  const long qoff = (long)h * dim, koff = (long)(H + h) * dim, voff = 2L * H * dim + (long)h * vdim + col0;
  auto act = [&](float f) { return silu ? f * sigmoid_f(f) : f; };
  float pq[NQ], pk[NQ], pv[NV];
  auto fetch = [&](int r0) {                       // rows r0 .. of the sequence into registers (zero beyond its end)
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      const int idx = tid + TH * u, t = idx / W, j = idx - t * W;
      const bool ok = r0 + t < e && j < dim;
      const T* xr = x + (long)(r0 + t) * x_stride;
      pq[u] = ok ? act(ldf(xr + qoff + j)) : 0.f;
      pk[u] = ok ? act(ldf(xr + koff + j)) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + TH * u, t = idx >> 6, c = idx & 63;
      const bool ok = idx < C * 64 && r0 + t < e && col0 + c < vdim;
      pv[u] = ok ? act(ldf(x + (long)(r0 + t) * x_stride + voff + c)) : 0.f;
    }
  };
  fetch(s);
  for (int r0 = s; r0 < e; r0 += C) {
    const int n = min(C, e - r0);
#pragma unroll
    for (int u = 0; u < NQ; ++u) {
      const int idx = tid + TH * u, t = idx / W, j = idx - t * W;
      qs[t][j] = pq[u];
      ks[t][j] = pk[u];
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int idx = tid + TH * u;
      if (idx < C * 64) vs[idx >> 6][idx & 63] = pv[u];
    }
    if (r0 + C < e) fetch(r0 + C);
    __syncthreads();
#pragma unroll 2
    for (int t = 0; t < n; ++t) {
      const float v = vs[t][lane];
      const float4* k4 = reinterpret_cast<const float4*>(&ks[t][g * R]);
      const float4* q4 = reinterpret_cast<const float4*>(&qs[t][g * R]);
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;              // (four chains: the sums do not wait for each other)
#pragma unroll
      for (int i = 0; i < R / 4; ++i) {
        const float4 kk = k4[i], qq = q4[i];
        S[4 * i] = d * S[4 * i] + kk.x * v;         a0 += S[4 * i] * qq.x;
        S[4 * i + 1] = d * S[4 * i + 1] + kk.y * v; a1 += S[4 * i + 1] * qq.y;
        S[4 * i + 2] = d * S[4 * i + 2] + kk.z * v; a2 += S[4 * i + 2] * qq.z;
        S[4 * i + 3] = d * S[4 * i + 3] + kk.w * v; a3 += S[4 * i + 3] * qq.w;
      }
      part[g][t][lane] = (a0 + a1) + (a2 + a3);
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
      if (r < dim) st[(long)r * vdim + col0 + lane] = S[i];
    }
  }
}

// ------------------------------------------------------------------------------------------------ latent attention
__device__ __forceinline__ void rotate_pair(float u, float v, int pos, float freq, float rs, float& ou, float& ov) {
  const float a = (float)pos * freq;
  const float cs = cosf(a) * rs, sn = sinf(a) * rs;
  ou = u * cs - v * sn;
  ov = v * cs + u * sn;
}

// one workgroup per token.  q [T, H, nope + rope] (strides q_st, q_sh), q_lat [H, T, rank] (strides l_sh, l_st),
// latent [T, rank + rope] (stride lat_st) or nullptr, out [T, H, rank + rope] contiguous, cache rows of rank + rope.
template <typename T>
__global__ void latent_prep_kernel(T* __restrict__ out, const T* __restrict__ q, long q_st, long q_sh, int nope,
                                   const T* __restrict__ q_lat, long l_sh, long l_st, const T* __restrict__ latent,
                                   long lat_st, const float* __restrict__ norm_w, float eps,
                                   const float* __restrict__ inv_freq, int half, float rs,
                                   const int* __restrict__ positions, T* __restrict__ cache, T* __restrict__ vfrag,
                                   const int* __restrict__ slot_mapping, int H, int rank, int rope, int bs,
                                   int interleaved) {
  __shared__ float red[17];
  const long t = blockIdx.x;
  const int pos = positions[t];
  const int dk = rank + rope;
  T* o = out + t * (long)H * dk;
  for (int i = threadIdx.x; i < H * rank; i += blockDim.x) {
    const int h = i / rank, j = i - h * rank;
    o[(long)h * dk + j] = q_lat[h * l_sh + t * l_st + j];
  }
  for (int i = threadIdx.x; i < H * rope; i += blockDim.x) {
    const int h = i / rope, j = i - h * rope;
    const T* src = q + t * q_st + h * q_sh + nope;
    float val;
    if (j < 2 * half) {
      // pair p: values (p, p + half), or neighbours (2p, 2p + 1)
      const int p = interleaved ? j >> 1 : (j < half ? j : j - half);
      const bool first = interleaved ? (j & 1) == 0 : j < half;
      float a, bb;
      rotate_pair(ldf(src + (interleaved ? 2 * p : p)), ldf(src + (interleaved ? 2 * p + 1 : p + half)), pos,
                  inv_freq[p], rs, a, bb);
      val = first ? a : bb;
    } else {
      val = ldf(src + j);
    }
    stf(o + (long)h * dk + rank + j, val);
  }
  if (latent == nullptr) return;                            // (uniform)
  const T* lr = latent + t * lat_st;
  float ss = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) { const float f = ldf(lr + i); ss += f * f; }
  const float inv = 1.0f / sqrtf(block_sum(ss, red) / (float)rank + eps);
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  T* row = cache + (long)slot * dk;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) stf(row + i, ldf(lr + i) * inv * norm_w[i]);
  if (vfrag != nullptr) {
    // the same values as V^T fragments [blocks][rank / 16][bs / 8][16][8] (what the matrix-core kernel reads)
    const long blk = slot / bs;
    const int off = slot % bs;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) {
      const long at = (((blk * (rank >> 4) + (i >> 4)) * (bs >> 3) + (off >> 3)) * 16 + (i & 15)) * 8 + (off & 7);
      stf(vfrag + at, ldf(lr + i) * inv * norm_w[i]);
    }
  }
  for (int j = threadIdx.x; j < rope; j += blockDim.x) {
    float val;
    if (j < 2 * half) {
      const int p = interleaved ? j >> 1 : (j < half ? j : j - half);
      const bool first = interleaved ? (j & 1) == 0 : j < half;
      float a, bb;
      rotate_pair(ldf(lr + rank + (interleaved ? 2 * p : p)), ldf(lr + rank + (interleaved ? 2 * p + 1 : p + half)), pos,
                  inv_freq[p], rs, a, bb);
      val = first ? a : bb;
    } else {
      val = ldf(lr + rank + j);
    }
    stf(row + rank + j, val);
  }
}

template <typename T> __device__ __forceinline__ float dot_row(const float* __restrict__ qs, const T* __restrict__ k, int dk) {
  float acc = 0.f;
  if constexpr (std::is_same_v<T, float>) {
    if ((dk & 3) == 0) {
      for (int d = 0; d < dk; d += 4) {
        const float4 kv = *reinterpret_cast<const float4*>(k + d);
        acc += qs[d] * kv.x; acc += qs[d + 1] * kv.y; acc += qs[d + 2] * kv.z; acc += qs[d + 3] * kv.w;
      }
      return acc;
    }
  } else {
    if ((dk & 7) == 0) {
      for (int d = 0; d < dk; d += 8) {
        const typename Vec8<T>::type kv = ld8<T>(k + d);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += qs[d + e] * (float)kv[e];
      }
      return acc;
    }
  }
  for (int d = 0; d < dk; ++d) acc += qs[d] * ldf(k + d);
  return acc;
}

// grid (tokens, ceil(H / 4)), 256 threads: wave w serves head blockIdx.y * 4 + w.  Waves share nothing but the
// workgroup's LDS allocation (each its own query copy): no workgroup barrier.
template <typename T, int NV>
__global__ __launch_bounds__(256) void latent_row_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ cache, const int* __restrict__ block_table,
    long bt_stride, const int* __restrict__ token_seq, const int* __restrict__ seq_lens, float scale, int H, int dk,
    int rank, int bs, int window, const float* __restrict__ sinks, const T* __restrict__ gate, long gate_stride) {
  extern __shared__ float q_lds[];
  const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long t = blockIdx.x;
  const int h = blockIdx.y * 4 + w;
  if (h >= H) return;
  float* qs = q_lds + (long)w * dk;
  const T* qr = q + (t * H + h) * (long)dk;
  for (int d = lane; d < dk; d += 64) qs[d] = ldf(qr + d);
  __builtin_amdgcn_wave_barrier();
  const int n = seq_lens[t];
  const int* bt = block_table + (token_seq != nullptr ? (long)token_seq[t] : t) * bt_stride;
  float m = -1.0e30f, l = 0.f;
  float o[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) o[i] = 0.f;
  // with a window only the last `window` keys are read (the pages before them may have gone back to the pool)
  const int first = window > 0 ? max(n - window, 0) : 0;
  for (int j0 = first; j0 < n; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j < n;
    long row = 0;
    float sc = -1.0e30f;
    if (valid) {
      row = ((long)bt[j / bs] * bs + (j % bs)) * dk;
      sc = dot_row<T>(qs, cache + row, dk) * scale;
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float p = valid ? expf(sc - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < NV; ++i) o[i] *= alpha;
    const int cnt = min(64, n - j0);
    const int row_lo = (int)(row & 0xffffffffL), row_hi = (int)(row >> 32);
    for (int jj = 0; jj < cnt; ++jj) {
      const float pj = __shfl(p, jj, 64);
      const long ro = ((long)__shfl(row_hi, jj, 64) << 32) | (unsigned int)__shfl(row_lo, jj, 64);
      const T* vr = cache + ro;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int dcol = lane + 64 * i;
        if (dcol < rank) o[i] += pj * ldf(vr + dcol);
      }
    }
  }
  if (sinks != nullptr) {                        // exp(sink) joins the denominator, once, with no value
    const float sk = sinks[h];
    const float m_f = fmaxf(m, sk);
    const float corr = expf(m - m_f);
    l = l * corr + expf(sk - m_f);
#pragma unroll
    for (int i = 0; i < NV; ++i) o[i] *= corr;
  }
  T* orow = out + (t * H + h) * (long)rank;
  float inv = l > 0.f ? 1.0f / l : 0.f;
  if (gate != nullptr) inv *= sigmoid_f(ldf(gate + t * gate_stride + h));
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int dcol = lane + 64 * i;
    if (dcol < rank) stf(orow + dcol, o[i] * inv);
  }
}

}  // namespace

VDAMD_API int vdamd_embed_scaled(float* out, const int* ids, const void* embed, float scale, int T, int H,
                                 int vocab_rows, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || vocab_rows <= 0) return 1;
  return by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    hipLaunchKernelGGL((embed_scaled_kernel<TT>), dim3(T), dim3(row_threads(H)), 0, stream, out, ids, (const TT*)embed,
                       scale, H, vocab_rows);
  });
}

// y == nullptr: out = LN(x) with x of type x_dt.  Otherwise x is the fp32 residual (x_dt must be DT_F32, x_stride H).
VDAMD_API int vdamd_layer_norm_to(void* out, void* x, long x_stride, const void* y, long y_stride, const float* w,
                                  const float* b, float eps, int rows, int H, int x_dt, int y_dt, int out_dt,
                                  hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || w == nullptr || (y != nullptr && x_dt != DT_F32)) return 1;
  const int th = row_threads(H);
  int i1 = 0, i2 = 0;
  const int rc = by_dtype(x_dt, [&](auto* tx) {
    using TX = std::remove_pointer_t<decltype(tx)>;
    i1 = by_dtype(y_dt, [&](auto* ty) {
      using TY = std::remove_pointer_t<decltype(ty)>;
      i2 = by_dtype(out_dt, [&](auto* to) {
        using TO = std::remove_pointer_t<decltype(to)>;
        hipLaunchKernelGGL((layer_norm_kernel<TX, TY, TO>), dim3(rows), dim3(th), 0, stream, (TO*)out, (TX*)x, x_stride,
                           (const TY*)y, y_stride, w, b, eps, H);
      });
    });
  });
  if (rc | i1 | i2) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

VDAMD_API int vdamd_gated_rms_norm(void* out, long out_stride, const float* o, const float* w, const void* gate,
                                   long gate_stride, float eps, int rows, int N, int group, float scale, int gate_dt,
                                   int out_dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (N <= 0 || group < 0 || (group > 0 && N % group) || out_stride < N) return 1;
  int inner = 0;
  if (group > 0) {
    const long units = (long)rows * (N / group);
    const int L = group / 8;
    if (gate_dt != DT_F32 && gate_dt == out_dt && group % 8 == 0 && L <= 64 && (L & (L - 1)) == 0 && out_stride % 8 == 0 &&
        gate_stride % 8 == 0 && aligned16(gate) && aligned16(o) && aligned16(w) && aligned16(out)) {
      const int rv = by_dtype(gate_dt, [&](auto* tg) {
        using TG = std::remove_pointer_t<decltype(tg)>;
        if constexpr (!std::is_same_v<TG, float>)
          hipLaunchKernelGGL((gated_group_norm_vec_kernel<TG>), dim3((unsigned)((units * L + 255) / 256)), dim3(256), 0,
                             stream, (TG*)out, out_stride, o, w, (const TG*)gate, gate_stride, eps, units, N, group, L,
                             scale);
      });
      if (rv) return 1;
      HIP_LAUNCH_CHECK();
      return 0;
    }
    const int rc = by_dtype(gate_dt, [&](auto* tg) {
      using TG = std::remove_pointer_t<decltype(tg)>;
      inner = by_dtype(out_dt, [&](auto* to) {
        using TO = std::remove_pointer_t<decltype(to)>;
        hipLaunchKernelGGL((gated_group_norm_kernel<TG, TO>), dim3((unsigned)((units + 3) / 4)), dim3(256), 0, stream,
                           (TO*)out, out_stride, o, w, (const TG*)gate, gate_stride, eps, rows, N, group, scale);
      });
    });
    if (rc | inner) return 1;
    HIP_LAUNCH_CHECK();
    return 0;
  }
  if (scale == 1.0f && out_stride == N && gate_dt != DT_F32 && gate_dt == out_dt && N % 8 == 0 && gate_stride % 8 == 0 && aligned16(gate) && aligned16(o) &&
      aligned16(w) && aligned16(out)) {
    const int rv = by_dtype(gate_dt, [&](auto* tg) {
      using TG = std::remove_pointer_t<decltype(tg)>;
      if constexpr (!std::is_same_v<TG, float>)
        hipLaunchKernelGGL((gated_rms_norm_vec_kernel<TG>), dim3(rows), dim3(N >= 2048 ? 256 : 128), 0, stream, (TG*)out,
                           o, w, (const TG*)gate, gate_stride, eps, N);
    });
    if (rv) return 1;
    HIP_LAUNCH_CHECK();
    return 0;
  }
  const int rc = by_dtype(gate_dt, [&](auto* tg) {
    using TG = std::remove_pointer_t<decltype(tg)>;
    inner = by_dtype(out_dt, [&](auto* to) {
      using TO = std::remove_pointer_t<decltype(to)>;
      hipLaunchKernelGGL((gated_rms_norm_kernel<TG, TO>), dim3(rows), dim3(row_threads(N)), 0, stream, (TO*)out,
                         out_stride, o, w, (const TG*)gate, gate_stride, eps, N, scale);
    });
  });
  if (rc | inner) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

VDAMD_API int vdamd_clamped_glu(void* out, const void* h, long h_stride, int rows, int F, float limit, float alpha,
                                int dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (F <= 0) return 1;
  const int rc = by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    if constexpr (!std::is_same_v<TT, float>) {
      if (F % 8 == 0 && h_stride % 8 == 0 && aligned16(h) && aligned16(out)) {
        hipLaunchKernelGGL((clamped_glu_vec_kernel<TT>), dim3(rows, (F + 2047) / 2048), dim3(256), 0, stream, (TT*)out,
                           (const TT*)h, h_stride, F, limit, alpha);
        return;
      }
    }
    hipLaunchKernelGGL((clamped_glu_kernel<TT>), dim3(rows, (F + 1023) / 1024), dim3(256), 0, stream, (TT*)out,
                       (const TT*)h, h_stride, F, limit, alpha);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

// routed, shared (may be null), out: [rows, H] contiguous; x rows x_stride apart; topw / topi [rows, k] (may be null:
// no identity share); gate (may be null with shared) one value per row, gate_stride apart
VDAMD_API int vdamd_expert_epilogue(void* out, const void* routed, const void* x, long x_stride, const float* topw,
                                    const int* topi, int k, int real_experts, const void* shared, const void* gate,
                                    long gate_stride, int rows, int H, int dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || (topw != nullptr && (topi == nullptr || k < 1)) || (shared != nullptr && gate == nullptr)) return 1;
  // 16-byte accesses where every row of every operand starts on a 16-byte border
  const bool vec = H % 8 == 0 && x_stride % 8 == 0 && aligned16(out) && aligned16(routed) && aligned16(x) &&
                   (shared == nullptr || aligned16(shared));
  const int rc = by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    hipLaunchKernelGGL((expert_epilogue_kernel<TT>), dim3(rows), dim3(H >= 2048 ? 256 : 128), 0, stream, (TT*)out,
                       (const TT*)routed, (const TT*)x, x_stride, topw, topi, k, real_experts, (const TT*)shared,
                       (const TT*)gate, gate_stride, H, vec);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

VDAMD_API int vdamd_relu_squared(void* out, const void* x, long n, int dt, hipStream_t stream) {
  if (n <= 0) return 0;
  const unsigned blocks = (unsigned)((n + 1023) / 1024 > 65535 ? 65535 : (n + 1023) / 1024);
  const int rc = by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    hipLaunchKernelGGL((relu_squared_kernel<TT>), dim3(blocks), dim3(256), 0, stream, (TT*)out, (const TT*)x, n);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

// x [T, x_stride] of type dt, out fp32 [T, H * vdim], state fp32 [slots, H, dim, vdim]; dim <= 256.  max_rows: the most
// rows any sequence brings (0 = unknown)
VDAMD_API int vdamd_decay_linear_attention(float* out, const void* x, long x_stride, const float* decay, float* state,
                                           const int* slots, const int* qsl, const int* seq_lens, int num_seqs, int H,
                                           int dim, int vdim, int silu, int max_rows, int dt, hipStream_t stream) {
  if (num_seqs <= 0) return 0;
  if (H <= 0 || dim <= 0 || vdim <= 0 || dim > 256) return 1;
  const dim3 grid(num_seqs, H, (vdim + 63) / 64);
  const int rc = by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
#define DLA(R_, G_, C_)                                                                                          \
  hipLaunchKernelGGL((decay_linear_attention_kernel<TT, R_, G_, C_>), grid, dim3(64 * G_), 0, stream, out,          \
                     (const TT*)x, x_stride, decay, state, slots, qsl, seq_lens, H, dim, vdim, silu)
    if (max_rows > 0 && max_rows <= 2) {
      // decoded rows only: the launch is bound by reading and writing the states, so small workgroups, several of
      // which fit a CU and overlap each other's loads
      if (dim <= 32) DLA(8, 4, 8);
      else if (dim <= 64) DLA(16, 4, 4);
      else if (dim <= 128) DLA(32, 4, 4);
      else DLA(64, 4, 4);
    } else {
      // prompt portions: the walk over the rows is sequential, so as many waves per workgroup as the rows allow
      if (dim <= 32) DLA(8, 4, 8);
      else if (dim <= 64) DLA(8, 8, 8);
      else if (dim <= 128) DLA(8, 16, 8);
      else DLA(16, 16, 8);
    }
#undef DLA
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

VDAMD_API int vdamd_latent_prep(void* out, const void* q, long q_st, long q_sh, int nope, const void* q_lat, long l_sh,
                                long l_st, const void* latent, long lat_st, const float* norm_w, float eps,
                                const float* inv_freq, int half, float rs, const int* positions, void* cache,
                                void* vfrag, const int* slot_mapping, int T, int H, int rank, int rope, int bs,
                                int interleaved, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || rank <= 0 || rope < 0 || 2 * half > rope) return 1;
  if (vfrag != nullptr && (latent == nullptr || rank % 16 || bs <= 0 || bs % 8)) return 1;
  if (latent != nullptr && (cache == nullptr || slot_mapping == nullptr || norm_w == nullptr)) return 1;
  const int rc = by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    hipLaunchKernelGGL((latent_prep_kernel<TT>), dim3(T), dim3(256), 0, stream, (TT*)out, (const TT*)q, q_st, q_sh, nope,
                       (const TT*)q_lat, l_sh, l_st, (const TT*)latent, lat_st, norm_w, eps, inv_freq, half, rs,
                       positions, (TT*)cache, (TT*)vfrag, slot_mapping, H, rank, rope, bs, interleaved);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

VDAMD_API int vdamd_latent_row_attention(void* out, const void* q, const void* cache, const int* block_table,
                                         long bt_stride, const int* token_seq, const int* seq_lens, float scale, int T,
                                         int H, int dk, int rank, int bs, int window, const float* sinks,
                                         const void* gate, long gate_stride, int dt, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || rank <= 0 || rank > dk || dk > 4096 || rank > 1024 || bs <= 0 || window < 0) return 1;
  const dim3 grid(T, (H + 3) / 4);
  const size_t lds = (size_t)4 * dk * sizeof(float);
  const int rc = by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
#define LRA(NV_)                                                                                                      \
  hipLaunchKernelGGL((latent_row_attention_kernel<TT, NV_>), grid, dim3(256), lds, stream, (TT*)out, (const TT*)q,     \
                     (const TT*)cache, block_table, bt_stride, token_seq, seq_lens, scale, H, dk, rank, bs, window,     \
                     sinks, (const TT*)gate, gate_stride)
    if (rank <= 64) LRA(1);
    else if (rank <= 128) LRA(2);
    else if (rank <= 256) LRA(4);
    else if (rank <= 512) LRA(8);
    else LRA(16);
#undef LRA
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}
