// Kernels around an fp32 residual stream with RMS norms, gfx950.  Compiled without fast-math: norms and the residual
// sum are 32-bit by definition of such a model.
//
//   residual_rms     one launch per sublayer boundary.  With x the fp32 residual stream (updated in place):
//                      x += a + b                      (outputs of two sublayers that read the same input; either absent)
//                      x += y / rms(y) * post_w        (an output that is RMS-normed before it joins the stream; absent)
//                      out = x / rms(x) * (offset + w) (the next sublayer's input) or out = x, in any float type
//                    and, with nothing to add, the plain RMS norm of rows of any float type (fp32 gains)
//   gelu_mul_rows    gelu_tanh(g[t, :]) * table[ids[t], col : col + n]
//   sigmoid_mul      o * sigmoid(gate) * scale into a destination with strided rows
//   gelu             the tanh form or the exact one, element-wise
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

int row_threads(int h) { return h >= 4096 ? 512 : (h >= 1024 ? 256 : 128); }

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

__device__ __forceinline__ float sigmoid_f(float x) { return 1.0f / (1.0f + expf(-x)); }

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

__device__ __forceinline__ float gelu_erf_f(float z) { return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f)); }

// four consecutive values of a row of type T as floats (16-byte load for fp32, 8-byte for the 16-bit types)
template <typename T> __device__ __forceinline__ f32x4 ld4(const T* p) {
  if constexpr (std::is_same_v<T, float>) {
    return *reinterpret_cast<const f32x4*>(p);
  } else {
    const typename Vec4<T>::type v = *reinterpret_cast<const typename Vec4<T>::type*>(p);
    return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
  }
}
template <typename T> __device__ __forceinline__ void st4(T* p, f32x4 v) {
  if constexpr (std::is_same_v<T, float>) {
    *reinterpret_cast<f32x4*>(p) = v;
  } else {
    typename Vec4<T>::type o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (T)v[e];
    *reinterpret_cast<typename Vec4<T>::type*>(p) = o;
  }
}

struct ResidualArgs {
  void* out; long out_stride;        // [rows, H] of the output type
  void* x; long x_stride;            // [rows, H]: the fp32 residual stream when anything is added, else any type
  const void* a; long a_stride;      // [rows, H] or null
  const void* b; long b_stride;      // [rows, H] or null
  const void* y; long y_stride;      // [rows, H] or null
  const float* post_w;               // [H] (with y)
  const float* w;                    // [H] or null: no gain
  float offset, eps;
  int H, normed;
};

// W values per thread and turn (4: rows whose length, strides and addresses allow 16 / 8-byte accesses).  A row is
// walked up to three times by the same threads (each rereads only what it wrote itself).
template <typename TX, typename TA, typename TO, int W>
__global__ void residual_rms_kernel(ResidualArgs p) {
  __shared__ float red[17];
  const long row = blockIdx.x;
  TX* xr = (TX*)p.x + row * p.x_stride;
  const TA* ar = p.a ? (const TA*)p.a + row * p.a_stride : nullptr;
  const TA* br = p.b ? (const TA*)p.b + row * p.b_stride : nullptr;
  const TA* yr = p.y ? (const TA*)p.y + row * p.y_stride : nullptr;
  const int n = p.H / W;
  float inv_y = 0.f;
  if (yr != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      if constexpr (W == 4) { const f32x4 v = ld4<TA>(yr + 4 * i); ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3]; }
      else { const float v = ldf(yr + i); ss += v * v; }
    }
    inv_y = 1.0f / sqrtf(block_sum(ss, red) / (float)p.H + p.eps);
  }
  const bool adds = ar != nullptr || yr != nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    if constexpr (W == 4) {
      f32x4 r = ld4<TX>(xr + 4 * i);
      if constexpr (std::is_same_v<TX, float>) {
        if (adds) {
          if (ar != nullptr) {
            const f32x4 av = ld4<TA>(ar + 4 * i);
            if (br != nullptr) { const f32x4 bv = ld4<TA>(br + 4 * i); r += av + bv; }
            else r += av;
          }
          if (yr != nullptr) {
            const f32x4 yv = ld4<TA>(yr + 4 * i), pw = *reinterpret_cast<const f32x4*>(p.post_w + 4 * i);
            r += yv * inv_y * pw;
          }
          *reinterpret_cast<f32x4*>(xr + 4 * i) = r;
        }
      }
      ss += r[0] * r[0] + r[1] * r[1] + r[2] * r[2] + r[3] * r[3];
    } else {
      float r = ldf(xr + i);
      if constexpr (std::is_same_v<TX, float>) {
        if (adds) {
          if (ar != nullptr) r += br != nullptr ? ldf(ar + i) + ldf(br + i) : ldf(ar + i);
          if (yr != nullptr) r += ldf(yr + i) * inv_y * p.post_w[i];
          xr[i] = r;
        }
      }
      ss += r * r;
    }
  }
  TO* orow = (TO*)p.out + row * p.out_stride;
  float inv = 1.f;
  if (p.normed) inv = 1.0f / sqrtf(block_sum(ss, red) / (float)p.H + p.eps);
  const bool gain = p.normed && p.w != nullptr;
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    if constexpr (W == 4) {
      f32x4 r = ld4<TX>(xr + 4 * i);
      if (p.normed) r *= inv;
      if (gain) { const f32x4 wv = *reinterpret_cast<const f32x4*>(p.w + 4 * i); r *= (wv + p.offset); }
      st4<TO>(orow + 4 * i, r);
    } else {
      float r = ldf(xr + i);
      if (p.normed) r *= inv;
      if (gain) r *= (p.w[i] + p.offset);
      stf(orow + i, r);
    }
  }
}

template <typename T>
__global__ void gelu_mul_rows_kernel(T* __restrict__ out, const T* __restrict__ g, long g_stride,
                                     const T* __restrict__ table, long table_stride, const int* __restrict__ ids,
                                     int col, int n, int rows, int table_rows) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (long)rows * n) return;
  const long t = i / n;
  const int j = (int)(i - t * n);
  const int id = min(max(ids[t], 0), table_rows - 1);
  stf(out + i, gelu_tanh_f(ldf(g + t * g_stride + j)) * ldf(table + (long)id * table_stride + col + j));
}

template <typename T, int W>
__global__ void sigmoid_mul_kernel(T* __restrict__ out, long out_stride, const T* __restrict__ o, long o_stride,
                                   const T* __restrict__ gate, long gate_stride, float scale, int n, int rows) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int per = n / W;
  if (i >= (long)rows * per) return;
  const long t = i / per;
  const int j = (int)(i - t * per) * W;
  if constexpr (W == 8) {
    const typename Vec8<T>::type ov = ld8<T>(o + t * o_stride + j), gv = ld8<T>(gate + t * gate_stride + j);
    typename Vec8<T>::type r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (T)((float)ov[e] * sigmoid_f((float)gv[e]) * scale);
    st8<T>(out + t * out_stride + j, r);
  } else {
    stf(out + t * out_stride + j, ldf(o + t * o_stride + j) * sigmoid_f(ldf(gate + t * gate_stride + j)) * scale);
  }
}

template <typename T, int W>
__global__ void gelu_kernel(T* __restrict__ out, const T* __restrict__ x, long n, int tanh_form) {
  const long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * W;
  if (i >= n) return;
  if constexpr (W == 8) {
    const typename Vec8<T>::type v = ld8<T>(x + i);
    typename Vec8<T>::type r;
#pragma unroll
    for (int e = 0; e < 8; ++e) r[e] = (T)(tanh_form ? gelu_tanh_f((float)v[e]) : gelu_erf_f((float)v[e]));
    st8<T>(out + i, r);
  } else {
    const float v = ldf(x + i);
    stf(out + i, tanh_form ? gelu_tanh_f(v) : gelu_erf_f(v));
  }
}

}  // namespace

// x_dt: the type of x (DT_F32 whenever a / b / y is given: x is then the residual stream, updated in place);
// in_dt: the type of a, b and y; out_dt: the type of out.  normed 0: out = x (after the adds).
VDAMD_API int vdamd_residual_rms(void* out, long out_stride, void* x, long x_stride, const void* a, long a_stride,
                                 const void* b, long b_stride, const void* y, long y_stride, const float* post_w,
                                 const float* w, float offset, float eps, int rows, int H, int normed, int x_dt,
                                 int in_dt, int out_dt, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || (b != nullptr && a == nullptr) || (y != nullptr && post_w == nullptr)) return 1;
  if ((a != nullptr || y != nullptr) && x_dt != DT_F32) return 1;
  ResidualArgs p{out, out_stride, x, x_stride, a, a_stride, b, b_stride, y, y_stride, post_w, w, offset, eps, H, normed};
  const bool vec = H % 4 == 0 && x_stride % 4 == 0 && out_stride % 4 == 0 && a_stride % 4 == 0 && b_stride % 4 == 0 &&
                   y_stride % 4 == 0 && aligned16(x) && aligned16(out) && aligned16(a) && aligned16(b) &&
                   aligned16(y) && aligned16(w) && aligned16(post_w);
  const dim3 grid(rows), block(row_threads(vec ? H : 4 * H));
  int r1 = 0, r2 = 0;
  const int rc = by_dtype(x_dt, [&](auto* tx) {
    using TX = std::remove_pointer_t<decltype(tx)>;
    r1 = by_dtype(in_dt, [&](auto* ta) {
      using TA = std::remove_pointer_t<decltype(ta)>;
      r2 = by_dtype(out_dt, [&](auto* to) {
        using TO = std::remove_pointer_t<decltype(to)>;
        if (vec) hipLaunchKernelGGL((residual_rms_kernel<TX, TA, TO, 4>), grid, block, 0, stream, p);
        else hipLaunchKernelGGL((residual_rms_kernel<TX, TA, TO, 1>), grid, block, 0, stream, p);
      });
    });
  });
  if (rc | r1 | r2) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

VDAMD_API int vdamd_gelu_mul_rows(void* out, const void* g, long g_stride, const void* table, long table_stride,
                                  const int* ids, int col, int n, int rows, int table_rows, int dt,
                                  hipStream_t stream) {
  if (rows <= 0 || n <= 0) return 0;
  if (col < 0 || col + n > table_stride || table_rows <= 0) return 1;
  const long total = (long)rows * n;
  const int rc = by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    hipLaunchKernelGGL((gelu_mul_rows_kernel<TT>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, (TT*)out,
                       (const TT*)g, g_stride, (const TT*)table, table_stride, ids, col, n, rows, table_rows);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

VDAMD_API int vdamd_sigmoid_mul(void* out, long out_stride, const void* o, long o_stride, const void* gate,
                                long gate_stride, float scale, int rows, int n, int dt, hipStream_t stream) {
  if (rows <= 0 || n <= 0) return 0;
  const bool vec = dt != DT_F32 && n % 8 == 0 && out_stride % 8 == 0 && o_stride % 8 == 0 && gate_stride % 8 == 0 &&
                   aligned16(out) && aligned16(o) && aligned16(gate);
  const long total = (long)rows * (vec ? n / 8 : n);
  const dim3 grid((unsigned)((total + 255) / 256));
  const int rc = by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    bool done = false;
    if constexpr (!std::is_same_v<TT, float>) {
      if (vec) {
        hipLaunchKernelGGL((sigmoid_mul_kernel<TT, 8>), grid, dim3(256), 0, stream, (TT*)out, out_stride, (const TT*)o,
                           o_stride, (const TT*)gate, gate_stride, scale, n, rows);
        done = true;
      }
    }
    if (!done)
      hipLaunchKernelGGL((sigmoid_mul_kernel<TT, 1>), grid, dim3(256), 0, stream, (TT*)out, out_stride, (const TT*)o,
                         o_stride, (const TT*)gate, gate_stride, scale, n, rows);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}

VDAMD_API int vdamd_gelu(void* out, const void* x, long n, int tanh_form, int dt, hipStream_t stream) {
  if (n <= 0) return 0;
  const bool vec = dt != DT_F32 && n % 8 == 0 && aligned16(out) && aligned16(x);
  const long total = vec ? n / 8 : n;
  const dim3 grid((unsigned)((total + 255) / 256));
  const int rc = by_dtype(dt, [&](auto* tp) {
    using TT = std::remove_pointer_t<decltype(tp)>;
    bool done = false;
    if constexpr (!std::is_same_v<TT, float>) {
      if (vec) {
        hipLaunchKernelGGL((gelu_kernel<TT, 8>), grid, dim3(256), 0, stream, (TT*)out, (const TT*)x, n, tanh_form);
        done = true;
      }
    }
    if (!done) hipLaunchKernelGGL((gelu_kernel<TT, 1>), grid, dim3(256), 0, stream, (TT*)out, (const TT*)x, n, tanh_form);
  });
  if (rc) return 1;
  HIP_LAUNCH_CHECK();
  return 0;
}
