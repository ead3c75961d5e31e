// Gated activations (SwiGLU / GeGLU) and GELU: out[T, F] = act(x[:, :F]) * x[:, F:].
// Memory-bound: 16-B vector loads/stores, grid-stride over (row, vector).
#include "eia_common.h"

enum ActKind { ACT_SILU = 0, ACT_GELU_TANH = 1, ACT_GELU_ERF = 2 };

template <int KIND>
EIA_DEV float act_f(float x) {
  if constexpr (KIND == ACT_SILU) return x / (1.f + __expf(-x));
  else if constexpr (KIND == ACT_GELU_TANH) {
    const float k0 = 0.7978845608028654f, k1 = 0.044715f;
    return 0.5f * x * (1.f + tanhf(k0 * (x + k1 * x * x * x)));
  } else return 0.5f * x * (1.f + erff(x * 0.7071067811865476f));
}

template <int KIND>
__global__ void __launch_bounds__(256)
act_and_mul_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ x, int F, long nvec_total,
                   long in_stride, long out_stride) {
  const int nvec_row = F >> 3;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < nvec_total;
       i += (long)gridDim.x * blockDim.x) {
    const long r = i / nvec_row;
    const int v = (int)(i % nvec_row);
    const bf16_t* xr = x + r * in_stride;
    bf16x8 a = *reinterpret_cast<const bf16x8*>(xr + 8 * v);
    bf16x8 b = *reinterpret_cast<const bf16x8*>(xr + F + 8 * v);
    bf16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      o[j] = f2bf(act_f<KIND>(bf2f(a[j])) * bf2f(b[j]));
    }
    *reinterpret_cast<bf16x8*>(out + r * out_stride + 8 * v) = o;
  }
}

template <int KIND>
__global__ void __launch_bounds__(256)
act_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ x, long nvec) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < nvec;
       i += (long)gridDim.x * blockDim.x) {
    bf16x8 a = reinterpret_cast<const bf16x8*>(x)[i];
    bf16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = f2bf(act_f<KIND>(bf2f(a[j])));
    reinterpret_cast<bf16x8*>(out)[i] = o;
  }
}

static inline int grid_for(long nvec) {
  long g = (nvec + 255) / 256;
  if (g > 4096) g = 4096;
  if (g < 1) g = 1;
  return (int)g;
}

EIA_API int eia_act_and_mul(void* out, const void* x, int T, int F, long in_stride,
                            long out_stride, int kind, hipStream_t st) {
  if (F % 8 != 0 || T < 0) return EIA_BAD_SHAPE;
  if (T == 0) return EIA_OK;
  const long nv = (long)T * (F / 8);
  dim3 grid(grid_for(nv)), block(256);
  switch (kind) {
    case ACT_SILU:
      hipLaunchKernelGGL(act_and_mul_kernel<ACT_SILU>, grid, block, 0, st, (bf16_t*)out,
                         (const bf16_t*)x, F, nv, in_stride, out_stride); break;
    case ACT_GELU_TANH:
      hipLaunchKernelGGL(act_and_mul_kernel<ACT_GELU_TANH>, grid, block, 0, st, (bf16_t*)out,
                         (const bf16_t*)x, F, nv, in_stride, out_stride); break;
    case ACT_GELU_ERF:
      hipLaunchKernelGGL(act_and_mul_kernel<ACT_GELU_ERF>, grid, block, 0, st, (bf16_t*)out,
                         (const bf16_t*)x, F, nv, in_stride, out_stride); break;
    default: return EIA_UNSUPPORTED;
  }
  EIA_LAUNCH_CHECK();
}

EIA_API int eia_act(void* out, const void* x, long numel, int kind, hipStream_t st) {
  if (numel % 8 != 0) return EIA_BAD_SHAPE;
  if (numel == 0) return EIA_OK;
  const long nv = numel / 8;
  dim3 grid(grid_for(nv)), block(256);
  switch (kind) {
    case ACT_SILU: hipLaunchKernelGGL(act_kernel<ACT_SILU>, grid, block, 0, st, (bf16_t*)out, (const bf16_t*)x, nv); break;
    case ACT_GELU_TANH: hipLaunchKernelGGL(act_kernel<ACT_GELU_TANH>, grid, block, 0, st, (bf16_t*)out, (const bf16_t*)x, nv); break;
    case ACT_GELU_ERF: hipLaunchKernelGGL(act_kernel<ACT_GELU_ERF>, grid, block, 0, st, (bf16_t*)out, (const bf16_t*)x, nv); break;
    default: return EIA_UNSUPPORTED;
  }
  EIA_LAUNCH_CHECK();
}

// Squared ReLU, out = max(x, 0)^2, for bf16 or fp32 activations (ungated expert MLPs).
template <typename T>
__global__ void __launch_bounds__(256)
relu2_kernel(T* __restrict__ out, const T* __restrict__ x, long n) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
    const float v = fmaxf(ld_f32<T>(x, i), 0.f);
    st_f32<T>(out, i, v * v);
  }
}

EIA_API int eia_relu2(void* out, const void* x, long numel, int is_bf16, hipStream_t st) {
  if (numel < 0) return EIA_BAD_SHAPE;
  if (numel == 0) return EIA_OK;
  dim3 grid(grid_for((numel + 3) / 4)), block(256);
  if (is_bf16)
    hipLaunchKernelGGL(relu2_kernel<bf16_t>, grid, block, 0, st, (bf16_t*)out, (const bf16_t*)x, numel);
  else
    hipLaunchKernelGGL(relu2_kernel<float>, grid, block, 0, st, (float*)out, (const float*)x, numel);
  EIA_LAUNCH_CHECK();
}

// Gated activation straight from the fp32 split-K partials [sk, T, 2F] of a [gate; up] GEMM:
// out[T, F] = act(sum_z gate_z) * (sum_z up_z), four columns per thread.
template <int KIND>
__global__ void __launch_bounds__(256)
splitk_act_and_mul_kernel(const float* __restrict__ part, int sk, int T, int F,
                          bf16_t* __restrict__ out, long ldo) {
  const long idx = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (idx >= (long)T * F) return;
  const int row = idx / F, col = idx % F;
  const long slab = (long)T * 2 * F;
  const float* p = part + (long)row * 2 * F + col;
  f32x4 gs = *reinterpret_cast<const f32x4*>(p), us = *reinterpret_cast<const f32x4*>(p + F);
  for (int z = 1; z < sk; ++z) {
    gs += *reinterpret_cast<const f32x4*>(p + z * slab);
    us += *reinterpret_cast<const f32x4*>(p + z * slab + F);
  }
  bf16x4 o;
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = f2bf(act_f<KIND>(gs[i]) * us[i]);
  *reinterpret_cast<bf16x4*>(out + (long)row * ldo + col) = o;
}

EIA_API int eia_splitk_act_and_mul(const float* part, int sk, int T, int F, void* out, long ldo,
                                   int kind, hipStream_t st) {
  if (F % 4 != 0 || T < 0 || sk < 1 || ldo % 4 != 0) return EIA_BAD_SHAPE;
  if (T == 0) return EIA_OK;
  dim3 grid((int)(((long)T * F / 4 + 255) / 256)), block(256);
  switch (kind) {
    case ACT_SILU: hipLaunchKernelGGL(splitk_act_and_mul_kernel<ACT_SILU>, grid, block, 0, st, part, sk, T, F, (bf16_t*)out, ldo); break;
    case ACT_GELU_TANH: hipLaunchKernelGGL(splitk_act_and_mul_kernel<ACT_GELU_TANH>, grid, block, 0, st, part, sk, T, F, (bf16_t*)out, ldo); break;
    case ACT_GELU_ERF: hipLaunchKernelGGL(splitk_act_and_mul_kernel<ACT_GELU_ERF>, grid, block, 0, st, part, sk, T, F, (bf16_t*)out, ldo); break;
    default: return EIA_UNSUPPORTED;
  }
  EIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------
// xIELU with two learned numbers (p, q) read from device memory (a weight reload needs no new
// launch arguments):  z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z)
// + z/2.  fp32 inside.  The input is a stored row [T, F] (type T, row stride ldx) or the fp32
// split-K partials [sk, T, ldp] of the GEMM that produced it (the F columns from the pointer on;
// a fused projection's row is wider than F), summed here (F, ldp % 4 == 0 then).
EIA_DEV float softplus_f(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
EIA_DEV float xielu_f(float z, float ap, float aq) {
  return z > 0.f ? ap * z * z + 0.5f * z : aq * (expm1f(z) - z) + 0.5f * z;
}

// four consecutive elements of a bf16 or fp32 row (8- / 16-byte accesses)
template <typename T> EIA_DEV f32x4 act_ld4(const T* p);
template <> EIA_DEV f32x4 act_ld4<bf16_t>(const bf16_t* p) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
  return f32x4{(float)v[0], (float)v[1], (float)v[2], (float)v[3]};
}
template <> EIA_DEV f32x4 act_ld4<float>(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
template <typename T> EIA_DEV void act_st4(T* p, f32x4 v);
template <> EIA_DEV void act_st4<bf16_t>(bf16_t* p, f32x4 v) {
  *reinterpret_cast<bf16x4*>(p) = bf16x4{f2bf(v[0]), f2bf(v[1]), f2bf(v[2]), f2bf(v[3])};
}
template <> EIA_DEV void act_st4<float>(float* p, f32x4 v) { *reinterpret_cast<f32x4*>(p) = v; }

template <typename T>
__global__ void __launch_bounds__(256)
xielu_kernel(const T* __restrict__ x, long ldx, const float* __restrict__ part, int sk, long ldp,
             const T* __restrict__ pq, T* __restrict__ out, long ldo, int rows, int F, int vec) {
  const float ap = softplus_f(ld_f32<T>(pq, 0)), aq = 0.5f + softplus_f(ld_f32<T>(pq, 1));
  if (part) {
    const long idx = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (idx >= (long)rows * F) return;
    const int row = idx / F, col = idx % F;
    const long slab = (long)rows * ldp;              // rows of the partials are ldp wide
    const float* p = part + (long)row * ldp + col;
    f32x4 v = *reinterpret_cast<const f32x4*>(p);
    for (int z = 1; z < sk; ++z) v += *reinterpret_cast<const f32x4*>(p + z * slab);
    if (vec) {
      act_st4<T>(out + (long)row * ldo + col, f32x4{xielu_f(v[0], ap, aq), xielu_f(v[1], ap, aq),
                                                    xielu_f(v[2], ap, aq), xielu_f(v[3], ap, aq)});
      return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) st_f32<T>(out + (long)row * ldo, col + i, xielu_f(v[i], ap, aq));
    return;
  }
  if (vec) {                                         // F, ldx, ldo multiples of 4
    const long idx = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (idx >= (long)rows * F) return;
    const int row = idx / F, col = idx % F;
    const f32x4 v = act_ld4<T>(x + (long)row * ldx + col);
    act_st4<T>(out + (long)row * ldo + col, f32x4{xielu_f(v[0], ap, aq), xielu_f(v[1], ap, aq),
                                                  xielu_f(v[2], ap, aq), xielu_f(v[3], ap, aq)});
    return;
  }
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)rows * F) return;
  const int row = idx / F, col = idx % F;
  st_f32<T>(out + (long)row * ldo, col, xielu_f(ld_f32<T>(x + (long)row * ldx, col), ap, aq));
}

EIA_API int eia_xielu(const void* x, long ldx, const float* part, int sk, long ldp, const void* pq,
                      void* out, long ldo, int rows, int F, int is_bf16, hipStream_t st) {
  if (rows < 0 || F < 1 || !pq || !out || (x == nullptr) == (part == nullptr) ||
      (part && (sk < 1 || F % 4 || ldp % 4 || ldp < F || reinterpret_cast<uintptr_t>(part) % 16)))
    return EIA_BAD_SHAPE;
  if (rows == 0) return EIA_OK;
  const int esz = is_bf16 ? 2 : 4;
  const int vec = F % 4 == 0 && ldx % 4 == 0 && ldo % 4 == 0 &&
                  ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) % (4 * esz)) == 0;
  const long n = (part || vec) ? (long)rows * F / 4 : (long)rows * F;
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (is_bf16)
    hipLaunchKernelGGL(xielu_kernel<bf16_t>, grid, block, 0, st, (const bf16_t*)x, ldx, part, sk,
                       ldp, (const bf16_t*)pq, (bf16_t*)out, ldo, rows, F, vec);
  else
    hipLaunchKernelGGL(xielu_kernel<float>, grid, block, 0, st, (const float*)x, ldx, part, sk,
                       ldp, (const float*)pq, (float*)out, ldo, rows, F, vec);
  EIA_LAUNCH_CHECK();
}

// out[t, c] = a(t, c) * sigmoid(g[t, c]), fp32 inside.  g and out are rows with their own strides
// (g may be a column slice of a wider row); a is either such a row too (V == N) or laid out head
// by head, a(t, h * V + v) = a[h * a_sh + t * lda + v] (the output of a batched product over
// heads), so the heads are concatenated here without a transposing copy.  vec: four columns per
// thread (V, the strides and the pointers allow 8- / 16-byte accesses).
template <typename T>
__global__ void __launch_bounds__(256)
sigmoid_gate_kernel(const T* __restrict__ a, long lda, long a_sh, int V, const T* __restrict__ g,
                    long ldg, T* __restrict__ out, long ldo, int rows, int N, int vec) {
  if (vec) {
    const long idx = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
    if (idx >= (long)rows * N) return;
    const int row = idx / N, col = idx % N;
    const int h = col / V;
    const f32x4 av = act_ld4<T>(a + h * a_sh + (long)row * lda + (col - h * V));
    const f32x4 gv = act_ld4<T>(g + (long)row * ldg + col);
    f32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = av[i] / (1.0f + expf(-gv[i]));
    act_st4<T>(out + (long)row * ldo + col, o);
    return;
  }
  const long idx = (long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (long)rows * N) return;
  const int row = idx / N, col = idx % N;
  const int h = col / V;
  const float gv = ld_f32<T>(g + (long)row * ldg, col);
  st_f32<T>(out + (long)row * ldo, col,
            ld_f32<T>(a + h * a_sh + (long)row * lda, col - h * V) / (1.0f + expf(-gv)));
}

EIA_API int eia_sigmoid_gate(const void* a, long lda, long a_sh, int V, const void* g, long ldg,
                             void* out, long ldo, int rows, int N, int is_bf16, hipStream_t st) {
  if (rows < 0 || N < 1 || V < 1 || N % V || !a || !g || !out) return EIA_BAD_SHAPE;
  if (rows == 0) return EIA_OK;
  const int esz = is_bf16 ? 2 : 4;
  const int vec = V % 4 == 0 && lda % 4 == 0 && a_sh % 4 == 0 && ldg % 4 == 0 && ldo % 4 == 0 &&
                  ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(g) |
                    reinterpret_cast<uintptr_t>(out)) % (4 * esz)) == 0;
  const long n = vec ? (long)rows * N / 4 : (long)rows * N;
  dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (is_bf16)
    hipLaunchKernelGGL(sigmoid_gate_kernel<bf16_t>, grid, block, 0, st, (const bf16_t*)a, lda, a_sh,
                       V, (const bf16_t*)g, ldg, (bf16_t*)out, ldo, rows, N, vec);
  else
    hipLaunchKernelGGL(sigmoid_gate_kernel<float>, grid, block, 0, st, (const float*)a, lda, a_sh,
                       V, (const float*)g, ldg, (float*)out, ldo, rows, N, vec);
  EIA_LAUNCH_CHECK();
}
