// The gated delta rule with a decay per head and key channel and a per-request fp32 state, gfx950.  Compiled without
// fast-math: everything that enters the recurrence is 32-bit by definition of such a model.
//
//   delta_rule_prep   per row: q and k of every query / key head made unit vectors (q times dim^-0.5), the decays
//                     g = exp(-exp(a_log[h]) * softplus(dt + dt_bias)) per head and key channel, b = sigmoid(beta),
//                     k.q of the unit vectors;
//                     all fp32, computed once per row instead of once per lane of the recurrence
//   gated_delta_rule  per (sequence, head, tile of 16 to 64 value columns) a workgroup walks the sequence's rows:
//                       S <- g * S (by rows) ; u = b (v - S^T k) ; S <- S + k u^T ; o = S^T q
//                     as ONE read of the decayed state per row - r = (gS)^T k and p = (gS)^T q together, then
//                     u = b (v - r), o = p + (k.q) u, S = gS + k u^T.  A lane keeps a part (a 4th, 8th or 16th) of one
//                     column of S in registers; the parts are summed across lanes; q / k / g / v / b / k.q of a
//                     chunk of rows are staged in LDS with the next chunk's loads in flight (one barrier per chunk).
//                     A prompt portion and a single decoded row are the same kernel in two lane layouts.
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
  for (int g = wave; g < G; g += nwaves) {          // [q heads | k heads], each dim wide
    const T* qs = xr + (long)g * dim;
    const T* ks = xr + (long)(G + g) * dim;
    float sq = 0.f, sk = 0.f;
    for (int i = lane; i < dim; i += 64) { const float a = ldf(qs + i), b = ldf(ks + i); sq += a * a; sk += b * b; }
    const float iq = 1.0f / sqrtf(wave_sum(sq) + norm_eps) * qscale, ik = 1.0f / sqrtf(wave_sum(sk) + norm_eps);
    float* qd = qn + (t * G + g) * (long)dim;
    float* kd = kn + (t * G + g) * (long)dim;
    float dot = 0.f;
    for (int i = lane; i < dim; i += 64) {
      const float a = ldf(qs + i) * iq, b = ldf(ks + i) * ik;
      qd[i] = a;
      kd[i] = b;
      dot += a * b;
    }
    dot = wave_sum(dot);
    const int per = H / G;
    for (int j = lane; j < per; j += 64) bsig[t * 2 * H + H + g * per + j] = dot;
  }
  const T* dr = dt + t * dt_stride;
  for (int i = threadIdx.x; i < H * dim; i += blockDim.x) {
    const int h = i / dim;
    decay[t * (long)H * dim + i] = expf(-expf(a_log[h]) * softplus_f(ldf(dr + i) + dt_bias[i]));
  }
  for (int h = threadIdx.x; h < H; h += blockDim.x) bsig[t * 2 * H + h] = 1.0f / (1.0f + expf(-ldf(beta + t * beta_stride + h)));
}

// one step of a sum over neighbouring lanes as a data-parallel-primitive add (no trip through LDS)
template <int CTRL> __device__ __forceinline__ float dpp_add(float v) {
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}

// sum over the P row parts of a wave, every lane gets it.  NEAR: the parts of a column are P neighbouring lanes
// (lane = column * P + part): swaps inside quads, then mirrors of 8 and 16 lanes.  Otherwise the parts are 64 / P
// lanes apart (lane = part * (64 / P) + column): xor-shuffles.
template <int P, bool NEAR> __device__ __forceinline__ float parts_sum(float v) {
  if constexpr (NEAR) {
    v = dpp_add<0xB1>(v);                           // quad_perm [1, 0, 3, 2]
    v = dpp_add<0x4E>(v);                           // quad_perm [2, 3, 0, 1]
    if constexpr (P >= 8) v = dpp_add<0x141>(v);    // row_half_mirror
    if constexpr (P >= 16) v = dpp_add<0x140>(v);   // row_mirror
  } else {
#pragma unroll
    for (int o = 64 / P; o < 64; o <<= 1) v += __shfl_xor(v, o, 64);
  }
  return v;
}

// grid (tiles of CB = 4 * 64 / P value columns, H, sequences), 4 waves: wave w owns columns w * 64 / P .. of the tile,
// a lane keeps R rows of one column of S in registers (P R >= dim; groups of four rows, dealt to the parts in turn).
// Two lane layouts.
// Launches of decoded rows are bound by reading and writing the states: P = 4, parts 16 lanes apart, so that a wave
// reads 64 bytes of a state row at a time.  Prompt portions are bound by the chain of dependent steps per row (the
// state cannot be written before r = (gS)^T k is summed over the parts): P = 8 or 16 neighbouring lanes per column,
// short chains, and the sums stay in the vector unit.  The sequence's rows are walked in chunks of C: q, k, g (all of
// the head, fp32), v (the tile's columns), b and k.q of a chunk are staged in LDS by the whole workgroup - the next
// chunk's loads are in flight while the current one is computed, one barrier per chunk - and read back as broadcasts
// (16-byte reads: a group of four rows).
// x rows hold v (H * vdim) at column v_off; qn / kn [T, G, dim], decay [T, H, dim], bsig [T, 2, H] (sigmoid(beta), then
// k.q of the head's group) fp32; out [T, H * vdim] fp32; state [slots, H, dim, vdim] fp32.
template <typename T, int R, int C, int P, bool NEAR>
__global__ __launch_bounds__(256) void gated_delta_rule_kernel(float* __restrict__ out, const T* __restrict__ x,
                                                               long x_stride, int v_off, const float* __restrict__ qn,
                                                               const float* __restrict__ kn,
                                                               const float* __restrict__ decay,
                                                               const float* __restrict__ bsig, float* __restrict__ state,
                                                               const int* __restrict__ slots, const int* __restrict__ qsl,
                                                               const int* __restrict__ seq_lens, int H, int G, int dim,
                                                               int vdim) {
  constexpr int CT = 64 / P, CB = 4 * CT;           // columns per wave, per workgroup
  constexpr int DP = P * R;                         // rows, padded (rows past dim stay zero)
  constexpr int ROW = 3 * DP + CB + 4;              // floats staged per sequence row: q | k | g | v (CB) | b, k.q, pad
  __shared__ __attribute__((aligned(16))) float lds[2][C * ROW];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int cl = NEAR ? lane / P : lane & (CT - 1), part = NEAR ? lane & (P - 1) : lane / CT;
  const int col0 = blockIdx.x * CB;
  const int col = col0 + wave * CT + cl;
  const int h = blockIdx.y, s = blockIdx.z;
  const int g = h / (H / G);
  const int q0 = qsl[s], n = qsl[s + 1] - q0;
  if (n <= 0) return;                               // (the whole workgroup)
  const bool col_ok = col < vdim;
  const int ccol = col_ok ? col : vdim - 1;
  // the lane's rows: groups of four, the groups of neighbouring parts side by side (the 16 parts of a column read 256
  // consecutive bytes of q, k or g at a time: no LDS bank is asked twice)
  auto row_of = [&](int i) { return ((i >> 2) * P + part) * 4 + (i & 3); };
  float* st = state + (((long)slots[s] * H + h) * dim) * vdim + ccol;
  float S[R];
  const bool fresh = seq_lens[s] - n <= 0;          // the rows start the sequence: whatever the slot holds is not ours
#pragma unroll
  for (int i = 0; i < R; ++i) S[i] = (!fresh && row_of(i) < dim) ? st[(long)row_of(i) * vdim] : 0.f;

  // staging: a thread brings 16 bytes of q, of k and of g per pass (all of one row), v and b / k.q element by element
  constexpr int F4 = DP / 4;                        // 16-byte pieces per row and array (a power of two)
  constexpr int NQ = (C * F4 + 255) / 256, NV = (C * CB + 255) / 256;
  static_assert(2 * C <= 256, "b and k.q of a chunk are one pass");
  const bool vec = (dim & 3) == 0;                  // (rows of qn / kn / decay start on 16-byte borders)
  const float* qsrc = qn + ((long)q0 * G + g) * dim;
  const float* ksrc = kn + ((long)q0 * G + g) * dim;
  const float* gsrc = decay + ((long)q0 * H + h) * dim;
  const T* vsrc = x + (long)q0 * x_stride + v_off + (long)h * vdim + col0;
  const float* bsrc = bsig + (long)q0 * 2 * H + h;
  const long qstep = (long)G * dim, gstep = (long)H * dim;
  f32x4 sq[NQ], sk[NQ], sg[NQ];
  float sv[NV], sb = 0.f;
  auto piece = [&](const float* row, int f) {       // row[f .. f + 3], zeros past dim
    f32x4 o = {0.f, 0.f, 0.f, 0.f};
    if (vec) { if (f < dim) o = *reinterpret_cast<const f32x4*>(row + f); }
    else {
#pragma unroll
      for (int e = 0; e < 4; ++e) if (f + e < dim) o[e] = row[f + e];
    }
    return o;
  };
  auto fetch = [&](int chunk) {                     // this thread's share of a chunk, global -> registers
    const int first = chunk * C, rows = min(C, n - first);
#pragma unroll
    for (int e = 0; e < NQ; ++e) {
      const int idx = tid + e * 256, j = idx / F4, f = (idx & (F4 - 1)) * 4;
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
      sq[e] = sk[e] = sg[e] = z;
      if (j < rows) {
        sq[e] = piece(qsrc + (first + j) * qstep, f);
        sk[e] = piece(ksrc + (first + j) * qstep, f);
        sg[e] = piece(gsrc + (first + j) * gstep, f);
      }
    }
#pragma unroll
    for (int e = 0; e < NV; ++e) {
      const int idx = tid + e * 256, j = idx / CB, cc = idx & (CB - 1);
      sv[e] = (j < rows && col0 + cc < vdim) ? ldf(vsrc + (first + j) * x_stride + cc) : 0.f;
    }
    sb = (tid < 2 * C && (tid >> 1) < rows) ? bsrc[(long)(first + (tid >> 1)) * 2 * H + (tid & 1) * H] : 0.f;
  };
  auto stash = [&](int buf) {
    float* dst = lds[buf];
#pragma unroll
    for (int e = 0; e < NQ; ++e) {
      const int idx = tid + e * 256, j = idx / F4, f = (idx & (F4 - 1)) * 4;
      if (j < C) {
        *reinterpret_cast<f32x4*>(dst + j * ROW + f) = sq[e];
        *reinterpret_cast<f32x4*>(dst + j * ROW + DP + f) = sk[e];
        *reinterpret_cast<f32x4*>(dst + j * ROW + 2 * DP + f) = sg[e];
      }
    }
#pragma unroll
    for (int e = 0; e < NV; ++e) {
      const int idx = tid + e * 256, j = idx / CB, cc = idx & (CB - 1);
      if (j < C) dst[j * ROW + 3 * DP + cc] = sv[e];
    }
    if (tid < 2 * C) dst[(tid >> 1) * ROW + 3 * DP + CB + (tid & 1)] = sb;
  };
  const int chunks = (n + C - 1) / C;
  fetch(0);
  stash(0);
  __syncthreads();
  for (int c = 0; c < chunks; ++c) {
    if (c + 1 < chunks) fetch(c + 1);
    const float* base = lds[c & 1];
    const int rows = min(C, n - c * C);
#pragma unroll 2
    for (int j = 0; j < rows; ++j) {
      const float* L = base + j * ROW;
      float ra = 0.f, rb = 0.f, pa = 0.f, pb = 0.f; // (two chains each: the sums do not wait for each other)
      float kr[R];
#pragma unroll
      for (int i = 0; i < R; i += 4) {
        const int off = ((i >> 2) * P + part) * 4;
        const f32x4 qv = *reinterpret_cast<const f32x4*>(L + off);
        const f32x4 kv = *reinterpret_cast<const f32x4*>(L + DP + off);
        const f32x4 gv = *reinterpret_cast<const f32x4*>(L + 2 * DP + off);
#pragma unroll
        for (int e = 0; e < 4; e += 2) {
          S[i + e] *= gv[e];
          S[i + e + 1] *= gv[e + 1];
          ra += S[i + e] * kv[e];
          rb += S[i + e + 1] * kv[e + 1];
          pa += S[i + e] * qv[e];
          pb += S[i + e + 1] * qv[e + 1];
          kr[i + e] = kv[e];
          kr[i + e + 1] = kv[e + 1];
        }
      }
      const float r = parts_sum<P, NEAR>(ra + rb);
      const float p = parts_sum<P, NEAR>(pa + pb);
      const float u = L[3 * DP + CB] * (L[3 * DP + wave * CT + cl] - r);
#pragma unroll
      for (int i = 0; i < R; ++i) S[i] += kr[i] * u;
      if (part == 0 && col_ok) out[(long)(q0 + c * C + j) * H * vdim + (long)h * vdim + col] = p + L[3 * DP + CB + 1] * u;
    }
    if (c + 1 < chunks) stash((c + 1) & 1);
    __syncthreads();
  }
  if (col_ok) {
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (row_of(i) < dim) st[(long)row_of(i) * vdim] = S[i];
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

// x [T, x_stride] of type dtype with v at column v_off; dim <= 256.  max_rows: the most rows any sequence brings (0 =
// unknown).  parts: row parts per wave (4, 8 or 16; 0 = chosen here)
VDAMD_API int vdamd_gated_delta_rule(float* out, const void* x, long x_stride, int v_off, const float* qn,
                                     const float* kn, const float* decay, const float* bsig, float* state,
                                     const int* slots, const int* qsl, const int* seq_lens, int B, int H, int G, int dim,
                                     int vdim, int max_rows, int parts, int dtype, hipStream_t stream) {
  if (B <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G || dim <= 0 || dim > 256 || vdim <= 0) return 1;
  if (parts == 0) {
    // decoded rows: 4.  Prompt portions: as many parts as still leave every compute unit no more than four workgroups
    // (the chain per row gets shorter with more parts, but the workgroups of a head then read q / k / g more often)
    parts = 4;
    if (max_rows != 1)
      for (int p = 16; p > 4; p >>= 1)
        if (4 * p <= (dim < 16 ? 16 : 2 * dim) && (long)B * H * ((vdim + 256 / p - 1) / (256 / p)) <= 1024) { parts = p; break; }
    if (max_rows != 1 && parts == 4 && dim > 32) parts = 8;
  }
  if (parts != 4 && parts != 8 && parts != 16) return 1;
  if (parts == 4 && dim > 128) parts = 8;           // (a lane keeps at most 32 rows)
  const int r = (dim + parts - 1) / parts;          // rows per lane
  const dim3 grid((vdim + 256 / parts - 1) / (256 / parts), H, B);
  const int rc = by_dtype(dtype, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
#define GDR(R_, P_)                                                                                                    \
  hipLaunchKernelGGL((gated_delta_rule_kernel<TT, R_, 8, P_, (P_ >= 8)>), grid, dim3(256), 0, stream, out,             \
                     (const TT*)x, x_stride, v_off, qn, kn, decay, bsig, state, slots, qsl, seq_lens, H, G, dim, vdim)
#define GDR_P(P_)                                                        \
  do {                                                                   \
    if (r <= 4) GDR(4, P_); else if (r <= 8) GDR(8, P_);                 \
    else if (r <= 16) GDR(16, P_); else GDR(32, P_);                     \
  } while (0)
    if (parts == 4) GDR_P(4);
    else if (parts == 8) GDR_P(8);
    else GDR_P(16);
#undef GDR_P
#undef GDR
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}
