// K5 / K5b: RMSNorm (+fused residual add) and LayerNorm (+fused residual add).
// One workgroup per row; the row lives in registers (VPT bf16x8 vectors per
// thread) so x is read once and written once: HBM-bound, 16-B vector access
// (guide §6 G13).  Decode rows (H=4096..16384) are 8-32 KiB.
#include "eia_common.h"

template <int VPT, bool ADD, bool HAS_RES_OUT>
__global__ void __launch_bounds__(256)
rms_norm_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ x,
                bf16_t* __restrict__ residual, const bf16_t* __restrict__ w,
                float eps, int H, long x_stride, long out_stride) {
  __shared__ float scratch[4];
  const long row = blockIdx.x;
  const int nvec = H >> 3;
  const bf16x8* xr = reinterpret_cast<const bf16x8*>(x + row * x_stride);
  bf16x8* rr = reinterpret_cast<bf16x8*>(residual + row * (long)H);
  float v[VPT][8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * blockDim.x;
    if (idx < nvec) {
      bf16x8 a = xr[idx];
      if constexpr (ADD) {
        bf16x8 r = rr[idx];
        bf16x8 s;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          float t = bf2f(a[j]) + bf2f(r[j]);
          s[j] = f2bf(t);
          v[i][j] = bf2f(s[j]);      // round like the stored residual
        }
        if constexpr (HAS_RES_OUT) rr[idx] = s;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = bf2f(a[j]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += v[i][j] * v[i][j];
    }
  }
  const float tot = block_sum(ss, scratch);
  const float inv = rsqrtf(tot / (float)H + eps);
  const bf16x8* wv = reinterpret_cast<const bf16x8*>(w);
  bf16x8* orow = reinterpret_cast<bf16x8*>(out + row * out_stride);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * blockDim.x;
    if (idx < nvec) {
      bf16x8 ww = wv[idx];
      bf16x8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = f2bf(v[i][j] * inv * bf2f(ww[j]));
      orow[idx] = o;
    }
  }
}

template <int VPT, bool ADD>
__global__ void __launch_bounds__(256)
layer_norm_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ x,
                  bf16_t* __restrict__ residual, const bf16_t* __restrict__ w,
                  const bf16_t* __restrict__ b, float eps, int H) {
  __shared__ float scratch[4];
  const long row = blockIdx.x;
  const int nvec = H >> 3;
  const bf16x8* xr = reinterpret_cast<const bf16x8*>(x + row * (long)H);
  bf16x8* rr = reinterpret_cast<bf16x8*>(residual + row * (long)H);
  float v[VPT][8];
  float s1 = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * blockDim.x;
    if (idx < nvec) {
      bf16x8 a = xr[idx];
      if constexpr (ADD) {
        bf16x8 r = rr[idx];
        bf16x8 s;
#pragma unroll
        for (int j = 0; j < 8; ++j) { s[j] = f2bf(bf2f(a[j]) + bf2f(r[j])); v[i][j] = bf2f(s[j]); }
        rr[idx] = s;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[i][j] = bf2f(a[j]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) s1 += v[i][j];
    }
  }
  const float mean = block_sum(s1, scratch) / (float)H;
  float s2 = 0.f;
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * blockDim.x;
    if (idx < nvec) {
#pragma unroll
      for (int j = 0; j < 8; ++j) { float d = v[i][j] - mean; s2 += d * d; }
    }
  }
  const float inv = rsqrtf(block_sum(s2, scratch) / (float)H + eps);
  const bf16x8* wv = reinterpret_cast<const bf16x8*>(w);
  const bf16x8* bv = reinterpret_cast<const bf16x8*>(b);
  bf16x8* orow = reinterpret_cast<bf16x8*>(out + row * (long)H);
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int idx = threadIdx.x + i * blockDim.x;
    if (idx < nvec) {
      bf16x8 ww = wv[idx];
      bf16x8 bb;
      if (b) bb = bv[idx];
      bf16x8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float y = (v[i][j] - mean) * inv * bf2f(ww[j]);
        if (b) y += bf2f(bb[j]);
        o[j] = f2bf(y);
      }
      orow[idx] = o;
    }
  }
}

static inline int pick_threads(int nvec) {
  if (nvec >= 256 * 2) return 256;
  int t = ((nvec + 63) / 64) * 64;
  return t < 64 ? 64 : (t > 256 ? 256 : t);
}

#define RMS_DISPATCH(ADD, RES)                                                        \
  switch (vpt) {                                                                      \
    case 1: hipLaunchKernelGGL((rms_norm_kernel<1, ADD, RES>), grid, block, 0, st,    \
                               (bf16_t*)out, (const bf16_t*)x, (bf16_t*)residual,     \
                               (const bf16_t*)w, eps, H, x_stride, out_stride); break; \
    case 2: hipLaunchKernelGGL((rms_norm_kernel<2, ADD, RES>), grid, block, 0, st,    \
                               (bf16_t*)out, (const bf16_t*)x, (bf16_t*)residual,     \
                               (const bf16_t*)w, eps, H, x_stride, out_stride); break; \
    case 4: hipLaunchKernelGGL((rms_norm_kernel<4, ADD, RES>), grid, block, 0, st,    \
                               (bf16_t*)out, (const bf16_t*)x, (bf16_t*)residual,     \
                               (const bf16_t*)w, eps, H, x_stride, out_stride); break; \
    case 8: hipLaunchKernelGGL((rms_norm_kernel<8, ADD, RES>), grid, block, 0, st,    \
                               (bf16_t*)out, (const bf16_t*)x, (bf16_t*)residual,     \
                               (const bf16_t*)w, eps, H, x_stride, out_stride); break; \
    default: return EIA_UNSUPPORTED;                                                  \
  }

static inline int vpt_for(int nvec, int threads) {
  int v = (nvec + threads - 1) / threads;
  if (v <= 1) return 1;
  if (v <= 2) return 2;
  if (v <= 4) return 4;
  if (v <= 8) return 8;
  return -1;
}

// out[T,H] = rmsnorm(x) * w            (residual == nullptr)
// residual = x + residual; out = rmsnorm(residual) * w   (residual != nullptr)
EIA_API int eia_rms_norm(void* out, const void* x, void* residual, const void* w, float eps,
                         int T, int H, long x_stride, long out_stride, hipStream_t st) {
  if (H % 8 != 0 || T < 0) return EIA_BAD_SHAPE;
  if (T == 0) return EIA_OK;
  const int nvec = H / 8;
  const int threads = pick_threads(nvec);
  const int vpt = vpt_for(nvec, threads);
  dim3 grid(T), block(threads);
  if (residual) {
    RMS_DISPATCH(true, true)
  } else {
    RMS_DISPATCH(false, false)
  }
  EIA_LAUNCH_CHECK();
}

EIA_API int eia_layer_norm(void* out, const void* x, void* residual, const void* w, const void* b,
                           float eps, int T, int H, hipStream_t st) {
  if (H % 8 != 0 || T < 0) return EIA_BAD_SHAPE;
  if (T == 0) return EIA_OK;
  const int nvec = H / 8;
  const int threads = pick_threads(nvec);
  const int vpt = vpt_for(nvec, threads);
  dim3 grid(T), block(threads);
#define LN_CASE(V)                                                                          \
  case V:                                                                                   \
    if (residual)                                                                           \
      hipLaunchKernelGGL((layer_norm_kernel<V, true>), grid, block, 0, st, (bf16_t*)out,    \
                         (const bf16_t*)x, (bf16_t*)residual, (const bf16_t*)w,             \
                         (const bf16_t*)b, eps, H);                                         \
    else                                                                                    \
      hipLaunchKernelGGL((layer_norm_kernel<V, false>), grid, block, 0, st, (bf16_t*)out,   \
                         (const bf16_t*)x, (bf16_t*)residual, (const bf16_t*)w,             \
                         (const bf16_t*)b, eps, H);                                         \
    break;
  switch (vpt) {
    LN_CASE(1) LN_CASE(2) LN_CASE(4) LN_CASE(8)
    default: return EIA_UNSUPPORTED;
  }
#undef LN_CASE
  EIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------
// Post-norm residual with an fp32 residual stream (sublayer-output norm):
//   x[row] += layernorm(y[row]) * w          (no bias; variance = mean of squared deviations)
//   xb[row] = (T) x[row]                      (optional copy in the activation type for the GEMMs)
// and the plain form on an fp32 input:  out[row] = (T)(layernorm(x[row]) * w).
// One workgroup per row, three passes over a row that stays in L1/L2 (mean, variance, write):
// the two-pass variance keeps fp32 exact enough for widths of several thousand.
template <typename TIn, typename T, bool RESID>
__global__ void __launch_bounds__(256)
ln_nobias_kernel(const TIn* __restrict__ y, long ldy, const T* __restrict__ w,
                 float* __restrict__ x, T* __restrict__ out, long ldo, float eps, int W) {
  __shared__ float scratch[4];
  const long row = blockIdx.x;
  const TIn* yr = y + row * ldy;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) s += ld_f32<TIn>(yr, c);
  const float mean = block_sum(s, scratch) / (float)W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float d = ld_f32<TIn>(yr, c) - mean;
    q += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum(q, scratch) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = (ld_f32<TIn>(yr, c) - mean) * inv * ld_f32<T>(w, c);
    if constexpr (RESID) {
      v += x[row * (long)W + c];
      x[row * (long)W + c] = v;
    }
    if (out) st_f32<T>(out + row * ldo, c, v);
  }
}

// y [rows, W] (bf16 when is_bf16 else fp32, row stride ldy); x fp32 [rows, W] contiguous, updated
// in place; xb nullable copy of the new x in y's type.
EIA_API int eia_ln_residual(const void* y, long ldy, const void* w, float* x, void* xb, long ldxb,
                            float eps, int rows, int W, int is_bf16, hipStream_t st) {
  if (rows < 0 || W < 1) return EIA_BAD_SHAPE;
  if (rows == 0) return EIA_OK;
  if (is_bf16)
    hipLaunchKernelGGL((ln_nobias_kernel<bf16_t, bf16_t, true>), dim3(rows), dim3(256), 0, st,
                       (const bf16_t*)y, ldy, (const bf16_t*)w, x, (bf16_t*)xb, ldxb, eps, W);
  else
    hipLaunchKernelGGL((ln_nobias_kernel<float, float, true>), dim3(rows), dim3(256), 0, st,
                       (const float*)y, ldy, (const float*)w, x, (float*)xb, ldxb, eps, W);
  EIA_LAUNCH_CHECK();
}

// out [rows, W] (bf16 when is_bf16 else fp32) = layernorm(x fp32 [rows, W], row stride ldx) * w.
EIA_API int eia_ln_f32in(const float* x, long ldx, const void* w, void* out, long ldo, float eps,
                         int rows, int W, int is_bf16, hipStream_t st) {
  if (rows < 0 || W < 1 || !out) return EIA_BAD_SHAPE;
  if (rows == 0) return EIA_OK;
  if (is_bf16)
    hipLaunchKernelGGL((ln_nobias_kernel<float, bf16_t, false>), dim3(rows), dim3(256), 0, st, x,
                       ldx, (const bf16_t*)w, nullptr, (bf16_t*)out, ldo, eps, W);
  else
    hipLaunchKernelGGL((ln_nobias_kernel<float, float, false>), dim3(rows), dim3(256), 0, st, x,
                       ldx, (const float*)w, nullptr, (float*)out, ldo, eps, W);
  EIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------
// RMS norm in groups with an fp32 residual stream.  A row of width W is NG equal consecutive
// parts; each part is divided by its own sqrt(mean(part^2) + eps) and the row is multiplied by a
// weight.  One launch does, per row,
//   x += gnorm(y) * w_post          (y != nullptr: a sublayer's output joins the stream)
//   x += add                        (add != nullptr: fp32 rows added before the next norm)
//   h  = gnorm(x) * w_next          (h != nullptr: the next sublayer's input, activation type)
// so a sublayer boundary (output norm, residual add, next input norm) is one pass over the row.
// A wave owns whole groups and walks them with the same lane-to-column map in both phases, so a
// lane re-reads only what it wrote and the row needs no barrier.
template <typename T> struct Vec4;
template <> struct Vec4<bf16_t> { typedef bf16x4 type; };
template <> struct Vec4<float> { typedef f32x4 type; };
template <typename T> EIA_DEV f32x4 ld4_f32(const T* p) {
  const typename Vec4<T>::type v = *reinterpret_cast<const typename Vec4<T>::type*>(p);
  return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}
template <typename T> EIA_DEV void st4_f32(T* p, f32x4 v) {
  typename Vec4<T>::type o;
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = (T)v[i];
  *reinterpret_cast<typename Vec4<T>::type*>(p) = o;
}
EIA_DEV float sumsq4(f32x4 v) { return v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3]; }

// VEC: group size and row strides are multiples of 4, so a lane handles four consecutive columns
// per step with 8- / 16-byte accesses; otherwise one column per step.
template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
gnorm_kernel(const T* __restrict__ y, long ldy, const float* __restrict__ ypart, int sk,
             long pstride, const T* __restrict__ ybias, const T* __restrict__ w_post,
             float* __restrict__ x, const float* __restrict__ add, const T* __restrict__ w_next,
             T* __restrict__ h, long ldh, float eps, int W, int NG) {
  const long row = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int gs = W / NG;
  float* xr = x + row * (long)W;
  extern __shared__ float ysum[];                   // [W] when the output arrives as partials
  if (ypart) {
    // the whole workgroup sums the GEMM's split-K partials of this row once, into LDS
    // (16-byte loads, eight partials in flight per thread; W % 4 == 0)
    for (int c = 4 * threadIdx.x; c < W; c += 4 * blockDim.x) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (ybias) v = f32x4{ld_f32<T>(ybias, c), ld_f32<T>(ybias, c + 1), ld_f32<T>(ybias, c + 2),
                           ld_f32<T>(ybias, c + 3)};
      const float* p = ypart + row * (long)W + c;
#pragma unroll 8
      for (int z = 0; z < sk; ++z) v += *reinterpret_cast<const f32x4*>(p + z * pstride);
      *reinterpret_cast<f32x4*>(ysum + c) = v;
    }
    __syncthreads();
  }
  const T* yr = y ? y + row * ldy : nullptr;
  for (int g = wave; g < NG; g += nw) {
    const int c0 = g * gs;
    if constexpr (VEC) {
      if (y || ypart) {
        float ss = 0.f;
        for (int c = c0 + 4 * lane; c < c0 + gs; c += 256)
          ss += sumsq4(y ? ld4_f32<T>(yr + c) : *reinterpret_cast<const f32x4*>(ysum + c));
        const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)gs + eps);
        for (int c = c0 + 4 * lane; c < c0 + gs; c += 256) {
          const f32x4 v = y ? ld4_f32<T>(yr + c) : *reinterpret_cast<const f32x4*>(ysum + c);
          f32x4 xv = *reinterpret_cast<f32x4*>(xr + c) + v * inv * ld4_f32<T>(w_post + c);
          if (add) xv += *reinterpret_cast<const f32x4*>(add + row * (long)W + c);
          *reinterpret_cast<f32x4*>(xr + c) = xv;
        }
      } else if (add) {
        for (int c = c0 + 4 * lane; c < c0 + gs; c += 256)
          *reinterpret_cast<f32x4*>(xr + c) += *reinterpret_cast<const f32x4*>(add + row * (long)W + c);
      }
      if (h) {
        float ss = 0.f;
        for (int c = c0 + 4 * lane; c < c0 + gs; c += 256)
          ss += sumsq4(*reinterpret_cast<const f32x4*>(xr + c));
        const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)gs + eps);
        for (int c = c0 + 4 * lane; c < c0 + gs; c += 256)
          st4_f32<T>(h + row * ldh + c,
                     *reinterpret_cast<const f32x4*>(xr + c) * inv * ld4_f32<T>(w_next + c));
      }
    } else {
      // the sublayer output at column c: a stored row, or the summed partials
      auto yval = [&](int c) -> float { return y ? ld_f32<T>(yr, c) : ysum[c]; };
      if (y || ypart) {
        float ss = 0.f;
        for (int c = lane; c < gs; c += 64) {
          const float v = yval(c0 + c);
          ss += v * v;
        }
        const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)gs + eps);
        for (int c = lane; c < gs; c += 64)
          xr[c0 + c] += yval(c0 + c) * inv * ld_f32<T>(w_post, c0 + c);
      }
      if (add) {
        const float* ar = add + row * (long)W + c0;
        for (int c = lane; c < gs; c += 64) xr[c0 + c] += ar[c];
      }
      if (h) {
        float ss = 0.f;
        for (int c = lane; c < gs; c += 64) {
          const float v = xr[c0 + c];
          ss += v * v;
        }
        const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)gs + eps);
        T* hr = h + row * ldh + c0;
        for (int c = lane; c < gs; c += 64)
          st_f32<T>(hr, c, xr[c0 + c] * inv * ld_f32<T>(w_next, c0 + c));
      }
    }
  }
}

// x fp32 [rows, W] contiguous, updated in place when y / ypart or add is given; y, ybias, w_post,
// w_next, h are bf16 when is_bf16 else fp32.  The sublayer output is either y [rows, W] (row
// stride ldy) or the fp32 split-K partials ypart [sk, rows, W] of the GEMM that produced it
// (+ ybias), summed here.
EIA_API int eia_gnorm(const void* y, long ldy, const float* ypart, int sk, const void* ybias,
                      const void* w_post, float* x, const float* add, const void* w_next, void* h,
                      long ldh, float eps, int rows, int W, int NG, int is_bf16, hipStream_t st) {
  if (rows < 0 || W < 1 || NG < 1 || W % NG || !x || ((y || ypart) && !w_post) || (h && !w_next) ||
      (y && ypart) || (ypart && (sk < 1 || W % 4)))
    return EIA_BAD_SHAPE;
  if (rows == 0) return EIA_OK;
  const int threads = (NG >= 4 || ypart) ? 256 : 64 * NG;
  const long ps = (long)rows * W;
  const size_t lds = ypart ? sizeof(float) * W : 0;
  if (lds > 64 * 1024) return EIA_UNSUPPORTED;
  const bool vec = (W / NG) % 4 == 0 && ldy % 4 == 0 && ldh % 4 == 0;
#define GNORM_LAUNCH(TT, VV)                                                                     \
  hipLaunchKernelGGL((gnorm_kernel<TT, VV>), dim3(rows), dim3(threads), lds, st, (const TT*)y, ldy, \
                     ypart, sk, ps, (const TT*)ybias, (const TT*)w_post, x, add, (const TT*)w_next, \
                     (TT*)h, ldh, eps, W, NG)
  if (is_bf16) {
    if (vec) GNORM_LAUNCH(bf16_t, true); else GNORM_LAUNCH(bf16_t, false);
  } else {
    if (vec) GNORM_LAUNCH(float, true); else GNORM_LAUNCH(float, false);
  }
#undef GNORM_LAUNCH
  EIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------
// Boundary of a layer whose sublayers run side by side on one normed input, around an fp32
// residual stream.  One launch does, per row,
//   x += y1 + y2                              (each given or not: sublayer outputs, un-normed)
//   h  = x / sqrt(mean(x^2) + eps) * w_next   (h != nullptr: the next layer's input)
// Each y is a stored row (type T, row stride ld) or the fp32 split-K partials [sk, rows, W] of the
// GEMM that produced it (+ bias), summed here.  A thread re-reads only the columns it wrote, so
// the row needs no barrier besides the one inside the sum of squares.
template <typename T> struct AddRmsSrc {
  const T* y; long ld; const float* part; int sk; const T* bias;
};
template <typename T>
EIA_DEV f32x4 add_rms_load(const AddRmsSrc<T>& s, long row, int c, long pstride, int W) {
  f32x4 v = {0.f, 0.f, 0.f, 0.f};
  if (s.y) {
    v = ld4_f32<T>(s.y + row * s.ld + c);
  } else if (s.part) {
    if (s.bias) v = ld4_f32<T>(s.bias + c);
    const float* p = s.part + row * (long)W + c;
#pragma unroll 4
    for (int z = 0; z < s.sk; ++z) v += *reinterpret_cast<const f32x4*>(p + z * pstride);
  }
  return v;
}

template <typename T, bool VEC>
__global__ void __launch_bounds__(256)
add_rms_kernel(AddRmsSrc<T> s1, AddRmsSrc<T> s2, float* __restrict__ x,
               const T* __restrict__ w_next, T* __restrict__ h, long ldh, float eps, int W,
               long pstride) {
  __shared__ float scratch[4];
  const long row = blockIdx.x;
  float* xr = x + row * (long)W;
  const bool any = s1.y || s1.part || s2.y || s2.part;
  float ss = 0.f;
  if constexpr (VEC) {
    for (int c = 4 * threadIdx.x; c < W; c += 4 * blockDim.x) {
      f32x4 xv = *reinterpret_cast<f32x4*>(xr + c);
      if (any) {
        xv += add_rms_load<T>(s1, row, c, pstride, W) + add_rms_load<T>(s2, row, c, pstride, W);
        *reinterpret_cast<f32x4*>(xr + c) = xv;
      }
      ss += sumsq4(xv);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
      float xv = xr[c];
      if (s1.y) xv += ld_f32<T>(s1.y + row * s1.ld, c);
      if (s2.y) xv += ld_f32<T>(s2.y + row * s2.ld, c);
      if (any) xr[c] = xv;
      ss += xv * xv;
    }
  }
  if (!h) return;
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)W + eps);
  if constexpr (VEC) {
    for (int c = 4 * threadIdx.x; c < W; c += 4 * blockDim.x)
      st4_f32<T>(h + row * ldh + c,
                 *reinterpret_cast<const f32x4*>(xr + c) * inv * ld4_f32<T>(w_next + c));
  } else {
    for (int c = threadIdx.x; c < W; c += blockDim.x)
      st_f32<T>(h + row * ldh, c, xr[c] * inv * ld_f32<T>(w_next, c));
  }
}

// x fp32 [rows, W] contiguous; y1 / y2, their biases, w_next and h are bf16 when is_bf16 else
// fp32.  Partials need W % 4 == 0.
EIA_API int eia_add_rms(const void* y1, long ld1, const float* p1, int sk1, const void* b1,
                        const void* y2, long ld2, const float* p2, int sk2, const void* b2,
                        float* x, const void* w_next, void* h, long ldh, float eps, int rows, int W,
                        int is_bf16, hipStream_t st) {
  if (rows < 0 || W < 1 || !x || (h && !w_next) || (y1 && p1) || (y2 && p2) ||
      (p1 && (sk1 < 1 || W % 4)) || (p2 && (sk2 < 1 || W % 4)))
    return EIA_BAD_SHAPE;
  if (rows == 0) return EIA_OK;
  const bool vec = W % 4 == 0 && ld1 % 4 == 0 && ld2 % 4 == 0 && ldh % 4 == 0;
  if (!vec && (p1 || p2)) return EIA_BAD_SHAPE;
  const int threads = W >= 1024 ? 256 : (W >= 512 ? 128 : 64);
  const long ps = (long)rows * W;
#define ADD_RMS_LAUNCH(TT, VV)                                                                  \
  do {                                                                                          \
    AddRmsSrc<TT> a{(const TT*)y1, ld1, p1, sk1, (const TT*)b1};                                \
    AddRmsSrc<TT> b{(const TT*)y2, ld2, p2, sk2, (const TT*)b2};                                \
    hipLaunchKernelGGL((add_rms_kernel<TT, VV>), dim3(rows), dim3(threads), 0, st, a, b, x,     \
                       (const TT*)w_next, (TT*)h, ldh, eps, W, ps);                             \
  } while (0)
  if (is_bf16) {
    if (vec) ADD_RMS_LAUNCH(bf16_t, true); else ADD_RMS_LAUNCH(bf16_t, false);
  } else {
    if (vec) ADD_RMS_LAUNCH(float, true); else ADD_RMS_LAUNCH(float, false);
  }
#undef ADD_RMS_LAUNCH
  EIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------
// Boundary of a sublayer whose residual is kept as NS streams joined by hyper-connections, one
// launch and one workgroup per token row.  X fp32 [rows, NS, W], updated in place:
//
//   X_j <- sum_s mix[s, j] X_s + ymult * outw[j] * y            (y given; all streams at once)
//   u    = sum_j in_next[j] X_j;   h = u / sqrt(mean(u^2) + eps) * (w_off + w_next)   (h given)
//
// y is a stored row (type T) or the fp32 split-K partials [sk, rows, W] (+ bias) of the GEMM that
// produced it, summed here.  mix [NS, NS] (from, to), outw [NS] and in_next [NS] are fp32 device
// arrays.  NS = 1 with mix = outw = in_next = 1 is the plain residual sum.  All arithmetic fp32.
constexpr int HC_MAX = 8;

// V: columns per thread and step (4: 16-byte accesses; needs W, ldy and ldh multiples of 4)
template <typename T, int V>
__global__ void __launch_bounds__(256)
hyper_step_kernel(float* __restrict__ X, int NS, int W, const T* __restrict__ y, long ldy,
                  const float* __restrict__ part, int sk, long pstride,
                  const T* __restrict__ ybias, const float* __restrict__ mix,
                  const float* __restrict__ outw, float ymult, const float* __restrict__ in_next,
                  const T* __restrict__ w_next, float w_off, T* __restrict__ h, long ldh,
                  float eps) {
  __shared__ float scratch[4];
  extern __shared__ float u_s[];                    // [W] when h is given
  const long row = blockIdx.x;
  float* xr = X + row * (long)NS * W;
  const bool upd = y || part;
  float mx[HC_MAX][HC_MAX], ow[HC_MAX], iw[HC_MAX];
#pragma unroll
  for (int s = 0; s < HC_MAX; ++s) {
    ow[s] = (upd && s < NS) ? ymult * outw[s] : 0.f;
    iw[s] = (h && s < NS) ? in_next[s] : 0.f;
#pragma unroll
    for (int j = 0; j < HC_MAX; ++j) mx[s][j] = (upd && s < NS && j < NS) ? mix[s * NS + j] : 0.f;
  }
  float ss = 0.f;
  for (int c = V * threadIdx.x; c < W; c += V * blockDim.x) {
    float xs[HC_MAX][V];
#pragma unroll
    for (int s = 0; s < HC_MAX; ++s) {
      if (s < NS) {
        if constexpr (V == 4) {
          const f32x4 v = *reinterpret_cast<const f32x4*>(xr + (long)s * W + c);
#pragma unroll
          for (int e = 0; e < V; ++e) xs[s][e] = v[e];
        } else {
          xs[s][0] = xr[(long)s * W + c];
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) xs[s][e] = 0.f;
      }
    }
    if (upd) {
      float yv[V];
      if (y) {
        if constexpr (V == 4) {
          const f32x4 v = ld4_f32<T>(y + row * ldy + c);
#pragma unroll
          for (int e = 0; e < V; ++e) yv[e] = v[e];
        } else {
          yv[0] = ld_f32<T>(y + row * ldy, c);
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) yv[e] = ybias ? ld_f32<T>(ybias, c + e) : 0.f;
        const float* p = part + row * (long)W + c;
        for (int z = 0; z < sk; ++z) {
          if constexpr (V == 4) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(p + z * pstride);
#pragma unroll
            for (int e = 0; e < V; ++e) yv[e] += v[e];
          } else {
            yv[0] += p[z * pstride];
          }
        }
      }
      float nx[HC_MAX][V];
#pragma unroll
      for (int j = 0; j < HC_MAX; ++j)
#pragma unroll
        for (int e = 0; e < V; ++e) {
          float v = ow[j] * yv[e];
#pragma unroll
          for (int s = 0; s < HC_MAX; ++s) v += mx[s][j] * xs[s][e];
          nx[j][e] = v;
        }
#pragma unroll
      for (int j = 0; j < HC_MAX; ++j) {
        if (j < NS) {
          if constexpr (V == 4)
            *reinterpret_cast<f32x4*>(xr + (long)j * W + c) =
                f32x4{nx[j][0], nx[j][1], nx[j][2], nx[j][3]};
          else
            xr[(long)j * W + c] = nx[j][0];
        }
#pragma unroll
        for (int e = 0; e < V; ++e) xs[j][e] = nx[j][e];
      }
    }
    if (h) {
#pragma unroll
      for (int e = 0; e < V; ++e) {
        float u = 0.f;
#pragma unroll
        for (int j = 0; j < HC_MAX; ++j) u += iw[j] * xs[j][e];
        u_s[c + e] = u;
        ss += u * u;
      }
    }
  }
  if (!h) return;
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)W + eps);
  for (int c = V * threadIdx.x; c < W; c += V * blockDim.x) {
    if constexpr (V == 4) {
      const f32x4 wv = ld4_f32<T>(w_next + c);
      const f32x4 u = *reinterpret_cast<const f32x4*>(u_s + c);
      st4_f32<T>(h + row * ldh + c, u * inv * (wv + w_off));
    } else {
      st_f32<T>(h + row * ldh, c, u_s[c] * inv * (w_off + ld_f32<T>(w_next, c)));
    }
  }
}

// X fp32 [rows, NS, W] contiguous; y, ybias, w_next and h are bf16 when is_bf16 else fp32.
EIA_API int eia_hyper_step(float* X, int NS, int W, const void* y, long ldy, const float* part,
                           int sk, const void* ybias, const float* mix, const float* outw,
                           float ymult, const float* in_next, const void* w_next, float w_off,
                           void* h, long ldh, float eps, int rows, int is_bf16, hipStream_t st) {
  if (rows < 0 || W < 1 || NS < 1 || NS > HC_MAX || !X || (y && part) || (part && sk < 1) ||
      ((y || part) && (!mix || !outw)) || (h && (!w_next || !in_next)))
    return EIA_BAD_SHAPE;
  if ((size_t)W * sizeof(float) > 64 * 1024) return EIA_UNSUPPORTED;
  if (rows == 0) return EIA_OK;
  const bool vec = W % 4 == 0 && ldy % 4 == 0 && ldh % 4 == 0;
  const int threads = W >= 1024 ? 256 : (W >= 512 ? 128 : 64);
  const size_t lds = h ? sizeof(float) * W : 0;
  const long ps = (long)rows * W;
#define HC_LAUNCH(TT, VV)                                                                        \
  hipLaunchKernelGGL((hyper_step_kernel<TT, VV>), dim3(rows), dim3(threads), lds, st, X, NS, W,  \
                     (const TT*)y, ldy, part, sk, ps, (const TT*)ybias, mix, outw, ymult,        \
                     in_next, (const TT*)w_next, w_off, (TT*)h, ldh, eps)
  if (is_bf16) {
    if (vec) HC_LAUNCH(bf16_t, 4); else HC_LAUNCH(bf16_t, 1);
  } else {
    if (vec) HC_LAUNCH(float, 4); else HC_LAUNCH(float, 1);
  }
#undef HC_LAUNCH
  EIA_LAUNCH_CHECK();
}
