// Windowed multi-map softmax attention over a paged cache: key rows are token-major
// [blocks, block, G * P * D]; values are stored transposed inside a page, [blocks, G * Dv, block],
// so that eight consecutive keys of one value column are one 16-byte load.
//
// A query row carries M = H * P score maps (H heads, P maps per head: 1 for ordinary heads, 2 for
// a differential pair), each D wide and already RMS-normed.  Map m = h * P + c of head h reads
// key map (h / (H / G)) * P + c of the token's key row ([G * P, D], normed at write time) and
// value head h / (H / G) of its value columns ([G, Dv]).  For the pair (query position i, key j):
//
//   raw_m  = (q_m . k) * mult[m] - slope[m] * (i - j)            (slope == nullptr: no distance term)
//   s_h    = sum_g talk[h, g] * raw_g                             (talk == nullptr: s = raw)
//   visible: j <= i and (i - j < window or j < keep)              (window <= 0: every j <= i)
//   p      = softmax over the visible keys, per map;  a_m = sum_j p_mj v_j
//   wmode 1: p = sigmoid(s_m + bias[m]) for every visible key, not normalised over the keys
//            (bias == nullptr: 0; no head mixing, P == 1)
//   sink (wmode 0, nullable): exp(sink[m]) joins map m's softmax denominator -- a term without a
//            key or a value, not scaled, counted once.  The running (max, sum) of a row simply
//            starts at (sink, 1) instead of (-inf, 0); with key partitions, in partition 0.
//
// Epilogue 0: out[h] = a_h * sigmoid(gate[h]) * post   (gate == nullptr: no gate; P must be 1)
// Epilogue 1: o = a_{2h} - lam * a_{2h+1};  out[h] = o / sqrt(mean(o^2) + eps) * post   (P == 2;
//             lam is read from device memory, so a captured launch follows a weight reload)
//
// Scores, softmax weights, accumulators, norms and gates are fp32 whatever the storage type.
// Rows are [decode rows (one per sequence) | prefill chunks]; both read the cache after
// qk_norm_cache wrote this step's tokens, so chunked prompts and mixed batches need no
// special path: a row is (position, block-table row) and nothing else.
#include "eia_common.h"

// ---------------------------------------------------------------------------------------------
// Cache write.  One workgroup per token of a fused projection row:
//   q maps  -> RMS norm (weight qw[D]) -> q_out[t, MQ * D]
//   k maps  -> RMS norm (weight kw[D]) -> key row of the token's slot
//   values  -> copied as projected     -> value columns of the token's slot (page-transposed)
//   gate    -> copied as projected     -> gate_out[t, GW]          (GW == 0: no gate columns)
// (values may alias the un-normed key columns: v_off == k_off).  Slots < 0 write no cache rows.
// The row is either stored (fused, type T) or still the fp32 split-K partials [sk, T, N] of the
// projection GEMM (+ bias), summed here; then the gate columns leave in type T for the
// attention kernel.
template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_cache_kernel(const T* __restrict__ fused, long ld, const float* __restrict__ part, int sk,
                     long pstride, const T* __restrict__ bias, int q_off, int k_off, int v_off,
                     int g_off, int MQ, int MK, int D, int VW, int GW, const T* __restrict__ qw,
                     const T* __restrict__ kw, T* __restrict__ q_out, long ldq,
                     T* __restrict__ kc, T* __restrict__ vc, T* __restrict__ gate_out, long ldg,
                     const int* __restrict__ slots, int bs, float eps) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const long slot = slots ? (long)slots[t] : -1;
  extern __shared__ float rsum[];                   // [ld] when the row arrives as partials
  if (part) {
    // the whole workgroup sums the GEMM's split-K partials of this row once, into LDS
    // (16-byte loads, eight partials in flight per thread; ld % 4 == 0)
    for (int c = 4 * threadIdx.x; c < (int)ld; c += 4 * blockDim.x) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (bias) v = f32x4{ld_f32<T>(bias, c), ld_f32<T>(bias, c + 1), ld_f32<T>(bias, c + 2),
                          ld_f32<T>(bias, c + 3)};
      const float* p = part + t * ld + c;
#pragma unroll 8
      for (int z = 0; z < sk; ++z) v += *reinterpret_cast<const f32x4*>(p + z * pstride);
      *reinterpret_cast<f32x4*>(rsum + c) = v;
    }
    __syncthreads();
  }
  auto val = [&](int c) -> float { return fused ? ld_f32<T>(fused + t * ld, c) : rsum[c]; };
  for (int u = wave; u < MQ + MK; u += nw) {
    const bool isq = u < MQ;
    const int m = isq ? u : u - MQ;
    if (!isq && slot < 0) continue;
    const int c0 = (isq ? q_off : k_off) + m * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float v = val(c0 + d);
      ss += v * v;
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
    T* dst = isq ? q_out + t * ldq + m * D : kc + slot * ((long)MK * D) + m * D;
    const T* w = isq ? qw : kw;
    for (int d = lane; d < D; d += 64) st_f32<T>(dst, d, val(c0 + d) * inv * ld_f32<T>(w, d));
  }
  if (slot >= 0) {
    T* dst = vc + (slot / bs) * (long)VW * bs + slot % bs;
    for (int c = threadIdx.x; c < VW; c += blockDim.x) st_f32<T>(dst, (long)c * bs, val(v_off + c));
  }
  if (gate_out)
    for (int c = threadIdx.x; c < GW; c += blockDim.x)
      st_f32<T>(gate_out + t * ldg, c, val(g_off + c));
}

EIA_API int eia_qk_norm_cache(const void* fused, long ld, const float* part, int sk,
                              const void* bias, int q_off, int k_off, int v_off, int g_off, int MQ,
                              int MK, int D, int VW, int GW, const void* qw, const void* kw,
                              void* q_out, long ldq, void* kc, void* vc, void* gate_out, long ldg,
                              const int* slots, int bs, float eps, int T, int is_bf16,
                              hipStream_t st) {
  if (T < 0 || MQ < 1 || MK < 1 || D < 1 || VW < 1 || bs < 1 || !q_out || !kc || !vc ||
      (fused == nullptr) == (part == nullptr) || (part && (sk < 1 || ld % 4)))
    return EIA_BAD_SHAPE;
  if (T == 0) return EIA_OK;
  const long ps = (long)T * ld;
  const size_t lds = part ? sizeof(float) * ld : 0;
  if (lds > 64 * 1024) return EIA_UNSUPPORTED;
  if (is_bf16)
    hipLaunchKernelGGL((qk_norm_cache_kernel<bf16_t>), dim3(T), dim3(256), lds, st,
                       (const bf16_t*)fused, ld, part, sk, ps, (const bf16_t*)bias, q_off, k_off,
                       v_off, g_off, MQ, MK, D, VW, GW, (const bf16_t*)qw, (const bf16_t*)kw,
                       (bf16_t*)q_out, ldq, (bf16_t*)kc, (bf16_t*)vc, (bf16_t*)gate_out, ldg, slots,
                       bs, eps);
  else
    hipLaunchKernelGGL((qk_norm_cache_kernel<float>), dim3(T), dim3(256), lds, st,
                       (const float*)fused, ld, part, sk, ps, (const float*)bias, q_off, k_off,
                       v_off, g_off, MQ, MK, D, VW, GW, (const float*)qw, (const float*)kw,
                       (float*)q_out, ldq, (float*)kc, (float*)vc, (float*)gate_out, ldg, slots, bs,
                       eps);
  EIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------
// Cache write for heads that are normed as ONE vector and then rotated.  One workgroup per token:
//   q columns [MQ * D] -> divided by their common root mean square, times qw[MQ * D] (qw == null:
//                         no norm) -> rotation of the first rot_dims entries of every head
//                         -> q_out[t, MQ * D]
//   k columns [MK * D] -> the same with kw -> key row of the token's slot
//   values             -> copied as projected -> value columns of the slot (page-transposed)
// Rotation of head entry d < rot_dims at position p: pairs (2i, 2i+1), or (i, i + rot_dims/2) when
// half; angle p * inv_freq[i] in fp32; cos and sin times amp.  Slots < 0 write no cache rows.
// The row is stored (fused) or still the fp32 split-K partials of the projection GEMM (+ bias).
template <typename T>
__global__ void __launch_bounds__(256)
qk_rope_cache_kernel(const T* __restrict__ fused, long ld, const float* __restrict__ part, int sk,
                     long pstride, const T* __restrict__ bias, int q_off, int k_off, int v_off,
                     int MQ, int MK, int D, int VW, const T* __restrict__ qw,
                     const T* __restrict__ kw, const float* __restrict__ inv_freq, int rot_dims,
                     int half, float amp, const int* __restrict__ positions, T* __restrict__ q_out,
                     long ldq, T* __restrict__ kc, T* __restrict__ vc,
                     const int* __restrict__ slots, int bs, float eps, int nsum) {
  __shared__ float scratch[4];
  const long t = blockIdx.x;
  const long slot = slots ? (long)slots[t] : -1;
  extern __shared__ float rsum[];                   // [ld] when the row arrives as partials
  const int hd = rot_dims >> 1;
  // the token's cos / sin (times amp), once per pair index, behind the summed row
  // (nsum: the row's first columns that hold q, k and v, a multiple of 4; a fused projection's
  // row may go on with other consumers' columns)
  float* cs_t = rsum + (part ? nsum : 0);           // [hd] cos, then [hd] sin
  for (int i = threadIdx.x; i < hd; i += blockDim.x) {
    float sn, cs;
    sincosf((float)positions[t] * inv_freq[i], &sn, &cs);
    cs_t[i] = cs * amp;
    cs_t[hd + i] = sn * amp;
  }
  if (part) {
    for (int c = 4 * threadIdx.x; c < nsum; c += 4 * blockDim.x) {
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (bias) v = f32x4{ld_f32<T>(bias, c), ld_f32<T>(bias, c + 1), ld_f32<T>(bias, c + 2),
                          ld_f32<T>(bias, c + 3)};
      const float* p = part + t * ld + c;
#pragma unroll 8
      for (int z = 0; z < sk; ++z) v += *reinterpret_cast<const f32x4*>(p + z * pstride);
      *reinterpret_cast<f32x4*>(rsum + c) = v;
    }
  }
  __syncthreads();
  auto val = [&](int c) -> float { return fused ? ld_f32<T>(fused + t * ld, c) : rsum[c]; };
  for (int side = 0; side < 2; ++side) {
    if (side == 1 && slot < 0) break;               // (uniform per workgroup)
    const int n = (side ? MK : MQ) * D, off = side ? k_off : q_off;
    const T* w = side ? kw : qw;
    float inv = 1.f;
    if (w) {
      float ss = 0.f;
      for (int c = threadIdx.x; c < n; c += blockDim.x) {
        const float v = val(off + c);
        ss += v * v;
      }
      inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
    }
    T* dst = side ? kc + slot * (long)n : q_out + t * ldq;
    auto normed = [&](int c) -> float {
      return val(off + c) * inv * (w ? ld_f32<T>(w, c) : 1.f);
    };
    for (int c = threadIdx.x; c < n; c += blockDim.x) {
      const int d = c % D, c0 = c - d;
      float v = normed(c);
      if (d < rot_dims) {
        const int i = half ? (d < hd ? d : d - hd) : (d >> 1);
        const bool second = half ? d >= hd : (d & 1);
        const float cs = cs_t[i], sn = cs_t[hd + i];
        const int da = half ? i : 2 * i, db = half ? i + hd : 2 * i + 1;
        const float o = normed(c0 + (second ? da : db));    // the pair's other entry
        v = second ? (v * cs + o * sn) : (v * cs - o * sn);
      }
      st_f32<T>(dst, c, v);
    }
  }
  if (slot >= 0) {
    T* dst = vc + (slot / bs) * (long)VW * bs + slot % bs;
    for (int c = threadIdx.x; c < VW; c += blockDim.x) st_f32<T>(dst, (long)c * bs, val(v_off + c));
  }
}

EIA_API int eia_qk_rope_cache(const void* fused, long ld, const float* part, int sk,
                              const void* bias, int q_off, int k_off, int v_off, int MQ, int MK,
                              int D, int VW, const void* qw, const void* kw, const float* inv_freq,
                              int rot_dims, int half, float amp, const int* positions, void* q_out,
                              long ldq, void* kc, void* vc, const int* slots, int bs, float eps,
                              int T, int is_bf16, hipStream_t st) {
  if (T < 0 || MQ < 1 || MK < 1 || D < 1 || VW < 1 || bs < 1 || !q_out || !kc || !vc || !positions ||
      rot_dims < 0 || rot_dims > D || (rot_dims & 1) || (rot_dims && !inv_freq) ||
      (fused == nullptr) == (part == nullptr) || (part && (sk < 1 || ld % 4)))
    return EIA_BAD_SHAPE;
  if (T == 0) return EIA_OK;
  const long ps = (long)T * ld;
  int nsum = q_off + MQ * D;
  if (k_off + MK * D > nsum) nsum = k_off + MK * D;
  if (v_off + VW > nsum) nsum = v_off + VW;
  nsum = (nsum + 3) & ~3;                           // (<= ld: ld % 4 == 0)
  if (part && nsum > ld) return EIA_BAD_SHAPE;
  const size_t lds = (part ? sizeof(float) * nsum : 0) + sizeof(float) * rot_dims;
  if (lds > 64 * 1024) return EIA_UNSUPPORTED;
  if (is_bf16)
    hipLaunchKernelGGL((qk_rope_cache_kernel<bf16_t>), dim3(T), dim3(256), lds, st,
                       (const bf16_t*)fused, ld, part, sk, ps, (const bf16_t*)bias, q_off, k_off,
                       v_off, MQ, MK, D, VW, (const bf16_t*)qw, (const bf16_t*)kw, inv_freq,
                       rot_dims, half, amp, positions, (bf16_t*)q_out, ldq, (bf16_t*)kc,
                       (bf16_t*)vc, slots, bs, eps, nsum);
  else
    hipLaunchKernelGGL((qk_rope_cache_kernel<float>), dim3(T), dim3(256), lds, st,
                       (const float*)fused, ld, part, sk, ps, (const float*)bias, q_off, k_off,
                       v_off, MQ, MK, D, VW, (const float*)qw, (const float*)kw, inv_freq, rot_dims,
                       half, amp, positions, (float*)q_out, ldq, (float*)kc, (float*)vc, slots, bs,
                       eps, nsum);
  EIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------
struct WinAttnArgs {
  const void* q; long ldq;          // [rows, M * D]
  const void* kc; const void* vc;   // [blocks, bs, G * P * D], [blocks, G * Dv, bs]
  const int* bt; int ldbt;          // block tables [seqs, ldbt]
  const int* positions;             // [rows]
  const int* cu;                    // prefill: first row of each sequence's chunk; decode: null
  const int* work;                  // prefill: (sequence, first query of the chunk) pairs
  const int* lens;                  // decode: sequence lengths (0: padding row)
  const float* mult;                // [M]
  const float* slope;               // [M] or null
  const float* talk;                // [M, M] or null
  const void* gate; long ldg;       // [rows, H * Dv] before the sigmoid, or null
  void* out; long ldo;              // [rows, H * Dv]
  int H, G, P, D, Dv, bs, window, keep, qb, epilogue;
  const float* lam;                 // [1], epilogue 1
  float eps, post;
  int nparts;                       // MFMA form: key partitions over grid.z (1: none)
  int raw_bufs;                     // MFMA form with head mixing: raw-score buffers in LDS (1, 2)
  float* part_acc; float* part_ml;  // [rows, M, nparts, Dv] and [rows, M, nparts, 2] partials
  int wmode;                        // 0: softmax; 1: sigmoid(score + bias), un-normalised
  const float* bias;                // [M] or null (wmode 1)
  const float* sink;                // [M] or null (wmode 0)
};

// The visible keys of a 16-query tile as absolute 32-key blocks: the blocks of the kept first
// tokens that lie before the window (nsink of them, from block 0), then blocks wb0 .. wb1.
struct WaBlocks { int wb0, nsink, nblocks; };
EIA_DEV WaBlocks wa_blocks(int pos_first, int pos_last, int window, int keep) {
  const int lo_min = window > 0 ? max(0, pos_first - window + 1) : 0;
  const int wb0 = lo_min >> 5;
  const int nsink = min((min(keep, lo_min) + 31) >> 5, wb0);
  return WaBlocks{wb0, nsink, nsink + (pos_last >> 5) - wb0 + 1};
}
// Key partitions a row really uses: at least two blocks each (a block's dependent chain of
// loads, products and the exchange is microseconds long, so a lone workgroup should walk few),
// so short contexts use few partitions whatever the launch's grid.z (the same on both sides of
// the merge).
EIA_DEV int wa_parts(int nparts, int nblocks) { return min(nparts, max(1, nblocks >> 1)); }

constexpr int WA_KT = 64;           // keys per tile = lanes of a wave
constexpr int WA_PAGES = 256;       // MFMA form: block -> page entries kept in LDS
constexpr int WA_ACC = 16;          // (map, value column) accumulators per thread

// Scalar-FMA form (fp32 models; bf16 shapes the MFMA form does not take).  One workgroup of four
// waves per work item; its queries run one after the other.  Per 64-key tile: (1) lane = key,
// the waves split the maps: raw scores into LDS; (2) the waves split the mixed maps: head mixing,
// mask, running max / sum with wave reductions, weights into LDS; (3) threads split the (map,
// value column) outputs and sweep the tile.
template <typename T>
__global__ void __launch_bounds__(256)
window_attn_kernel(const WinAttnArgs a) {
  extern __shared__ float lds[];
  const int H = a.H, P = a.P, D = a.D, Dv = a.Dv, M = H * P, rep = H / a.G;
  float* qs = lds;                        // [M, D]
  float* sraw = qs + M * D;               // [M, 64]
  float* pw = sraw + M * WA_KT;           // [M, 64]
  float* fin = pw + M * WA_KT;            // [M, Dv]
  float* mrun = fin + M * Dv;             // [M]
  float* lrun = mrun + M;                 // [M]
  float* alpha = lrun + M;                // [M]
  long* vbase = reinterpret_cast<long*>(alpha + M + (M & 1));   // [64], 8-byte aligned
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* q = (const T*)a.q;
  const T* kc = (const T*)a.kc;
  const T* vc = (const T*)a.vc;
  const T* gate = (const T*)a.gate;
  T* out = (T*)a.out;
  const long krow = (long)a.G * P * D, vrow = (long)a.G * Dv;

  int seq, row0, nq;
  if (a.cu) {
    seq = a.work[2 * blockIdx.x];
    const int q0 = a.work[2 * blockIdx.x + 1];
    const int n = a.cu[seq + 1] - a.cu[seq];
    row0 = a.cu[seq] + q0;
    nq = min(a.qb, n - q0);
  } else {
    seq = blockIdx.x;
    row0 = seq;
    nq = 1;
  }
  const int* bt = a.bt + (long)seq * a.ldbt;
  const int outw = H * Dv;

  for (int qi = 0; qi < nq; ++qi) {
    const long row = row0 + qi;
    if (a.lens && a.lens[seq] <= 0) {                  // padding row of a fixed-size batch
      for (int c = tid; c < outw; c += 256) st_f32<T>(out + row * a.ldo, c, 0.f);
      continue;
    }
    const int pos = a.positions[row];
    const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    const int nsink = min(a.keep, lo);
    const int nkeys = nsink + pos - lo + 1;
    __syncthreads();                                   // previous query's LDS reads are over
    for (int c = tid; c < M * D; c += 256) qs[c] = ld_f32<T>(q + row * a.ldq, c);
    for (int m = tid; m < M; m += 256) {
      mrun[m] = a.sink ? a.sink[m] : -INFINITY;
      lrun[m] = a.sink ? 1.f : 0.f;
    }
    float acc[WA_ACC];
#pragma unroll
    for (int i = 0; i < WA_ACC; ++i) acc[i] = 0.f;

    for (int k0 = 0; k0 < nkeys; k0 += WA_KT) {
      const int kk = k0 + lane;
      const bool valid = kk < nkeys;
      const int j = valid ? (kk < nsink ? kk : lo + kk - nsink) : pos;
      const long slot = (long)bt[j / a.bs] * a.bs + j % a.bs;
      __syncthreads();                                 // qs / mrun ready; last tile's reads over
      if (wave == 0) vbase[lane] = (long)bt[j / a.bs] * vrow * a.bs + j % a.bs;
      // (1) raw scores of this lane's key
      for (int m = wave; m < M; m += 4) {
        const int h = m / P, c = m - h * P;
        const T* kp = kc + slot * krow + ((h / rep) * P + c) * D;
        const float* qp = qs + m * D;
        float s = 0.f;
        for (int d = 0; d < D; ++d) s += qp[d] * ld_f32<T>(kp, d);
        s *= a.mult[m];
        if (a.slope) s -= a.slope[m] * (float)(pos - j);
        sraw[m * WA_KT + lane] = s;
      }
      __syncthreads();
      // (2) head mixing, mask, online softmax
      for (int m = wave; m < M; m += 4) {
        float s;
        if (a.talk) {
          s = 0.f;
          for (int g = 0; g < M; ++g) s += a.talk[m * M + g] * sraw[g * WA_KT + lane];
        } else {
          s = sraw[m * WA_KT + lane];
        }
        if (a.wmode == 1) {                            // plain sigmoid weights: nothing to rescale
          const float z = s + (a.bias ? a.bias[m] : 0.f);
          pw[m * WA_KT + lane] = valid ? 1.0f / (1.0f + expf(-z)) : 0.f;
          if (lane == 0) { alpha[m] = 1.f; lrun[m] = 1.f; }
          continue;
        }
        if (!valid) s = -INFINITY;
        const float mo = mrun[m];
        const float mn = fmaxf(mo, wave_max(s));
        const float p = valid ? expf(s - mn) : 0.f;
        const float ps = wave_sum(p);
        pw[m * WA_KT + lane] = p;
        if (lane == 0) {
          const float al = expf(mo - mn);              // exp(-inf) = 0 at the first tile
          alpha[m] = al;
          lrun[m] = lrun[m] * al + ps;
          mrun[m] = mn;
        }
      }
      __syncthreads();
      // (3) weighted values
      const int nk = min(WA_KT, nkeys - k0);
#pragma unroll
      for (int i = 0; i < WA_ACC; ++i) {
        const int idx = tid + i * 256;
        if (idx < M * Dv) {
          const int m = idx / Dv, d = idx - m * Dv;
          const T* vp = vc + (long)(((m / P) / rep) * Dv + d) * a.bs;
          const float* pm = pw + m * WA_KT;
          float s = acc[i] * alpha[m];
          for (int k = 0; k < nk; ++k) s += pm[k] * ld_f32<T>(vp, vbase[k]);
          acc[i] = s;
        }
      }
    }
    __syncthreads();
    if (a.epilogue == 0) {
#pragma unroll
      for (int i = 0; i < WA_ACC; ++i) {
        const int idx = tid + i * 256;
        if (idx < M * Dv) {
          float v = acc[i] / lrun[idx / Dv] * a.post;
          if (gate) v *= 1.0f / (1.0f + expf(-ld_f32<T>(gate + row * a.ldg, idx)));
          st_f32<T>(out + row * a.ldo, idx, v);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < WA_ACC; ++i) {
        const int idx = tid + i * 256;
        if (idx < M * Dv) fin[idx] = acc[i] / lrun[idx / Dv];
      }
      __syncthreads();
      const float lam = a.lam[0];
      for (int h = wave; h < H; h += 4) {
        const float* a1 = fin + (2 * h) * Dv;
        const float* a2 = a1 + Dv;
        float ss = 0.f;
        for (int d = lane; d < Dv; d += 64) {
          const float o = a1[d] - lam * a2[d];
          ss += o * o;
        }
        const float inv = a.post / sqrtf(wave_sum(ss) / (float)Dv + a.eps);
        for (int d = lane; d < Dv; d += 64)
          st_f32<T>(out + row * a.ldo, h * Dv + d, (a1[d] - lam * a2[d]) * inv);
      }
    }
  }
}

static size_t wa_lds_bytes(int M, int D, int Dv) {
  return sizeof(float) * ((size_t)M * D + 2 * (size_t)M * WA_KT + (size_t)M * Dv + 3 * M + (M & 1))
         + sizeof(long) * WA_KT;
}

// n_items: decode rows (cu == nullptr) or prefill work items.
EIA_API int eia_window_attn(const void* q, long ldq, const void* kc, const void* vc, const int* bt,
                            int ldbt, const int* positions, const int* cu, const int* work,
                            const int* lens, int n_items, const float* mult, const float* slope,
                            const float* talk, const void* gate, long ldg, void* out, long ldo,
                            int H, int G, int P, int D, int Dv, int bs, int window, int keep,
                            int qb, int epilogue, const float* lam, float eps, float post,
                            int wmode, const float* bias, const float* sink, int is_bf16,
                            hipStream_t st) {
  if (n_items < 0 || H < 1 || G < 1 || H % G || (P != 1 && P != 2) || D < 1 || Dv < 1 || bs < 1 ||
      keep < 0 || qb < 1 || !q || !kc || !vc || !bt || !positions || !mult || !out)
    return EIA_BAD_SHAPE;
  if ((cu == nullptr) != (work == nullptr)) return EIA_BAD_SHAPE;
  if ((epilogue == 1) != (P == 2) || (epilogue == 1 && (gate || !lam)))
    return EIA_BAD_SHAPE;
  if ((wmode != 0 && wmode != 1) || (wmode == 1 && (talk || P != 1 || sink))) return EIA_BAD_SHAPE;
  const int M = H * P;
  const size_t lds = wa_lds_bytes(M, D, Dv);
  if (M * Dv > 256 * WA_ACC || lds > 64 * 1024) return EIA_UNSUPPORTED;
  if (n_items == 0) return EIA_OK;
  WinAttnArgs a{q, ldq, kc, vc, bt, ldbt, positions, cu, work, lens, mult, slope, talk, gate, ldg,
                out, ldo, H, G, P, D, Dv, bs, window, keep, qb, epilogue, lam, eps, post, 1, 2,
                nullptr, nullptr, wmode, bias, sink};
  if (is_bf16)
    hipLaunchKernelGGL((window_attn_kernel<bf16_t>), dim3(n_items), dim3(256), lds, st, a);
  else
    hipLaunchKernelGGL((window_attn_kernel<float>), dim3(n_items), dim3(256), lds, st, a);
  EIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------
// MFMA form (bf16): v_mfma_f32_16x16x32_bf16, operands straight from the cache into registers.
//
// A workgroup of NWV <= 8 waves owns a tile of 16 queries of one sequence and NWV * HW heads (at
// most 256 registers per wave, so two waves share a SIMD and one's loads hide behind the other's
// arithmetic); a wave owns HW heads (HW * P maps) and walks the visible keys in absolute 32-key blocks (a block
// never straddles a page: block size % 32 == 0), first the blocks of the kept first tokens that
// lie before the window, then the window's.  Per block and map it forms S^T (keys x queries)
// as two 16-key tiles whose rows are ordered so that the accumulator registers of a lane --
// query lane % 16, keys 8 (lane / 16) + e -- are the B operand of the second product,
// O^T (value columns x queries) += V^T P^T, with V^T read as eight consecutive keys of a value
// column (the page-transposed value layout).  Nothing passes through LDS except, with head
// mixing, the raw scores: every wave writes its maps' tiles, one barrier, every wave reads all
// maps and mixes the rows of its own heads (buffers alternate between blocks).
// Softmax weights stay fp32: P enters the second product as a bf16 high part plus a bf16
// remainder, and the normaliser sums the fp32 weights.
// SIG: sigmoid weights (wmode 1) instead of the running softmax.
template <int HW, int P, bool TALK, bool SHARE, int ND, int NDV, bool SIG = false>
__global__ void __launch_bounds__(512)
window_attn_mfma_kernel(const WinAttnArgs a) {
  constexpr int MW = HW * P;
  constexpr int NKV = SHARE ? 1 : HW;          // distinct kv heads among this wave's heads
  constexpr int HPK = HW / NKV;                // heads per kv head
  constexpr float LOG2E = 1.4426950408889634f;
  extern __shared__ float lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int H = a.H, D = a.D, Dv = a.Dv, M = H * P, rep = H / a.G, bs = a.bs;
  const int nd = (D + 31) >> 5, ndv = Dv >> 4;
  const bf16_t* q = (const bf16_t*)a.q;
  const bf16_t* kc = (const bf16_t*)a.kc;
  const bf16_t* vc = (const bf16_t*)a.vc;
  const long krow = (long)a.G * P * D, vpage = (long)a.G * Dv * bs;

  int seq, row0, nq;
  if (a.cu) {
    seq = a.work[2 * blockIdx.x];
    const int q0 = a.work[2 * blockIdx.x + 1];
    row0 = a.cu[seq] + q0;
    nq = min(16, a.cu[seq + 1] - a.cu[seq] - q0);
  } else {
    seq = blockIdx.x;
    row0 = seq;
    nq = (a.lens && a.lens[seq] <= 0) ? 0 : 1;
  }
  const int h0 = (blockIdx.y * (blockDim.x >> 6) + wave) * HW;      // this wave's first head
  const bool wave_on = h0 < H;                                      // (H % HW == 0)
  const int* bt = a.bt + (long)seq * a.ldbt;
  bf16_t* out = (bf16_t*)a.out;
  if (nq == 0) {                                                    // padding row: zeros
    if (wave_on)
      for (int i = lane; i < HW * Dv; i += 64) out[(long)row0 * a.ldo + h0 * Dv + i] = f2bf(0.f);
    return;
  }
  float* talk_s = lds;                                              // [M, M] (TALK)
  f32x4* raw_s = reinterpret_cast<f32x4*>(lds + ((M * M + 3) & ~3));  // [2][M][2][64]
  if constexpr (TALK) {
    for (int i = threadIdx.x; i < M * M; i += blockDim.x) talk_s[i] = a.talk[i];
  }
  const int hs = wave_on ? h0 : 0;                                  // idle waves read head 0
  const bool row_ok = c < nq;
  const long row = row0 + (row_ok ? c : 0);
  const int qpos = a.positions[row];
  const int pos_first = a.positions[row0], pos_last = a.positions[row0 + nq - 1];
  const WaBlocks kbs = wa_blocks(pos_first, pos_last, a.window, a.keep);
  const int wb0 = kbs.wb0, nsink = kbs.nsink, nblocks = kbs.nblocks;
  const int np = wa_parts(a.nparts, nblocks);
  if ((int)blockIdx.z >= np) return;                                // (whole workgroup)

  // Q^T operands of this wave's maps: column = query c, rows = d 32 s + 8 g .. + 8
  bf16x8 qf[MW][ND];
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int m = 0; m < MW; ++m)
#pragma unroll
    for (int s = 0; s < ND; ++s) {
      const int d = 32 * s + 8 * g;
      const bf16x8 v = *reinterpret_cast<const bf16x8*>(q + row * a.ldq + (hs * P + m) * D +
                                                        (d < D ? d : 0));
      qf[m][s] = d < D ? v : zero8;
    }
  float mult[MW], slope[MW], sbias[MW];
#pragma unroll
  for (int m = 0; m < MW; ++m) {
    mult[m] = a.mult[hs * P + m];
    slope[m] = a.slope ? a.slope[hs * P + m] : 0.f;
    sbias[m] = (SIG && a.bias) ? a.bias[hs * P + m] : 0.f;
  }
  f32x4 acc[MW][NDV];
  float mrun[MW], lrun[MW];
#pragma unroll
  for (int m = 0; m < MW; ++m) {
    const bool snk = !SIG && a.sink && blockIdx.z == 0;
    mrun[m] = snk ? a.sink[hs * P + m] : -1e30f;
    lrun[m] = snk ? 1.f : 0.f;
#pragma unroll
    for (int t = 0; t < NDV; ++t) acc[m][t] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // S^T tiles: tile t, row 4 g' + i  <->  key 8 g' + 4 t + i; this lane's A rows are c
  const int r0 = 8 * (c >> 2) + (c & 3);                            // key of row c in tile 0
  const int dq = 8 * g;

  // with key partitions (decode rows of small batches) this workgroup takes a slice of the blocks
  const int per = (nblocks + np - 1) / np;
  const int b_lo = blockIdx.z * per, b_hi = min(nblocks, b_lo + per);
  // the pages of this workgroup's blocks, looked up once (the block loop then has no dependent
  // global load in front of its operand addresses); blocks past the table's size look up directly
  __shared__ int page_s[WA_PAGES];
  for (int i = threadIdx.x; i < min(b_hi - b_lo, WA_PAGES); i += blockDim.x) {
    const int bb = b_lo + i;
    page_s[i] = bt[((bb < nsink ? bb : wb0 + bb - nsink) << 5) / bs];
  }
  __syncthreads();
  auto page_of = [&](int b, int key0) -> long {
    return b - b_lo < WA_PAGES ? page_s[b - b_lo] : bt[key0 / bs];
  };
  // K operands of one block: every load issued together (addresses clamped, not branched)
  auto load_k = [&](int b, bf16x8 (&kf)[NKV][P][2][ND]) {
    const int kb = b < nsink ? b : wb0 + b - nsink;
    const int key0 = kb << 5;
    const bf16_t* k0p = kc + (page_of(b, key0) * bs + key0 % bs + r0) * krow;
#pragma unroll
    for (int j = 0; j < NKV; ++j) {
      const int kvh = (hs + j * HPK) / rep;
#pragma unroll
      for (int pm = 0; pm < P; ++pm)
#pragma unroll
        for (int s = 0; s < ND; ++s) {
          const int d = 32 * s + dq;
          const bf16_t* kp = k0p + (kvh * P + pm) * D + (d < D ? d : 0);
          const bf16x8 ka = *reinterpret_cast<const bf16x8*>(kp);
          const bf16x8 kb2 = *reinterpret_cast<const bf16x8*>(kp + 4 * krow);
          kf[j][pm][0][s] = d < D ? ka : zero8;
          kf[j][pm][1][s] = d < D ? kb2 : zero8;
        }
    }
  };
  // software pipeline (where the second operand set fits the register budget): block b + 1's
  // page lookup and K loads are in flight during block b's softmax and second product
  constexpr bool PIPE = NKV * P * ND <= 4;
  // a wave with a single map and no head mixing has registers left to keep the next block's V^T
  // operands in flight too, so no global load latency is exposed inside a block
  constexpr bool VPIPE = PIPE && MW == 1 && !TALK;
  bf16x8 kf[NKV][P][2][ND], kn[PIPE ? NKV : 1][PIPE ? P : 1][2][PIPE ? ND : 1];
  bf16x8 vn[VPIPE ? NKV : 1][VPIPE ? NDV : 1];
  auto load_v = [&](int b, bf16x8 (&vv)[VPIPE ? NKV : 1][VPIPE ? NDV : 1]) {
    const int key0 = (b < nsink ? b : wb0 + b - nsink) << 5;
    const bf16_t* vp = vc + page_of(b, key0) * vpage + ((long)(hs / rep) * Dv + c) * bs +
                       key0 % bs + dq;
#pragma unroll
    for (int t = 0; t < (VPIPE ? NDV : 1); ++t)
      vv[0][t] = *reinterpret_cast<const bf16x8*>(vp + (long)(t < ndv ? t : 0) * 16 * bs);
  };
  if constexpr (PIPE) {
    if (b_lo < b_hi) load_k(b_lo, kn);
  }
  if constexpr (VPIPE) {
    if (b_lo < b_hi) load_v(b_lo, vn);
  }
  for (int b = b_lo; b < b_hi; ++b) {
    const int kb = b < nsink ? b : wb0 + b - nsink;                 // absolute 32-key block
    const int key0 = kb << 5;
    const long page = page_of(b, key0);
    const int off = key0 % bs;
    if constexpr (PIPE) {
#pragma unroll
      for (int j = 0; j < NKV; ++j)
#pragma unroll
        for (int pm = 0; pm < P; ++pm)
#pragma unroll
          for (int s = 0; s < ND; ++s) {
            kf[j][pm][0][s] = kn[j][pm][0][s];
            kf[j][pm][1][s] = kn[j][pm][1][s];
          }
    } else {
      load_k(b, kf);
    }
    f32x4 sc[MW][2];
#pragma unroll
    for (int j = 0; j < NKV; ++j) {
#pragma unroll
      for (int hh = 0; hh < HPK; ++hh)
#pragma unroll
        for (int pm = 0; pm < P; ++pm) {
          const int m = (j * HPK + hh) * P + pm;
          f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < ND; ++s) {
            if (s < nd) {
              s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[j][pm][0][s], qf[m][s], s0, 0, 0, 0);
              s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[j][pm][1][s], qf[m][s], s1, 0, 0, 0);
            }
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int ka = key0 + 8 * g + i;
            s0[i] = s0[i] * mult[m] - slope[m] * (float)(qpos - ka);
            s1[i] = s1[i] * mult[m] - slope[m] * (float)(qpos - ka - 4);
          }
          sc[m][0] = s0;
          sc[m][1] = s1;
        }
    }
    if constexpr (PIPE) {
      if (b + 1 < b_hi) load_k(b + 1, kn);
    }
    // the block's V^T operands are requested before the softmax arithmetic needs them (or were
    // requested a block ago)
    bf16x8 vf[NKV][NDV];
    if constexpr (VPIPE) {
#pragma unroll
      for (int t = 0; t < NDV; ++t) vf[0][t] = vn[0][t];
      if (b + 1 < b_hi) load_v(b + 1, vn);
    } else {
#pragma unroll
      for (int j = 0; j < NKV; ++j) {
        const bf16_t* vp = vc + page * vpage + ((long)((hs + j * HPK) / rep) * Dv + c) * bs + off + dq;
#pragma unroll
        for (int t = 0; t < NDV; ++t)
          vf[j][t] = *reinterpret_cast<const bf16x8*>(vp + (long)(t < ndv ? t : 0) * 16 * bs);
      }
    }
    if constexpr (TALK) {
      // raw scores of every map through LDS: [buffer][map][tile][lane] f32x4
      f32x4* buf = raw_s + (size_t)(a.raw_bufs == 2 ? (b & 1) : 0) * M * 128;
      if (wave_on) {
#pragma unroll
        for (int m = 0; m < MW; ++m) {
          buf[((h0 + m) * 2 + 0) * 64 + lane] = sc[m][0];
          buf[((h0 + m) * 2 + 1) * 64 + lane] = sc[m][1];
        }
      }
      __syncthreads();
#pragma unroll
      for (int m = 0; m < MW; ++m) {
        sc[m][0] = f32x4{0.f, 0.f, 0.f, 0.f};
        sc[m][1] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll 4
      for (int gm = 0; gm < M; ++gm) {
        const f32x4 r0v = buf[(gm * 2 + 0) * 64 + lane], r1v = buf[(gm * 2 + 1) * 64 + lane];
#pragma unroll
        for (int m = 0; m < MW; ++m) {
          const float tw = talk_s[(hs + m) * M + gm];
          sc[m][0] += tw * r0v;
          sc[m][1] += tw * r1v;
        }
      }
      if (a.raw_bufs != 2) __syncthreads();           // one buffer: reads end before it is rewritten
    }
    // mask, running max / sum, P^T operands
    bf16x8 ph[MW], pl[MW];
    float alpha[MW];
    bool vis[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int key = key0 + 8 * g + e;
      vis[e] = row_ok && key <= qpos && (a.window <= 0 || qpos - key < a.window || key < a.keep);
    }
#pragma unroll
    for (int m = 0; m < MW; ++m) {
      float v[8];
      if constexpr (SIG) {
        // un-normalised sigmoid weights: no running maximum, nothing to rescale
        alpha[m] = 1.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float z = (e < 4 ? sc[m][0][e] : sc[m][1][e - 4]) + sbias[m];
          const float p = vis[e] ? __builtin_amdgcn_rcpf(1.0f + exp2f(-z * LOG2E)) : 0.f;
          const bf16_t hi = f2bf(p);
          ph[m][e] = hi;
          pl[m][e] = f2bf(p - bf2f(hi));
        }
        lrun[m] = 1.f;
      } else {
      float mloc = -1e30f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        v[e] = e < 4 ? sc[m][0][e] : sc[m][1][e - 4];
        if (vis[e]) mloc = fmaxf(mloc, v[e]);
      }
      mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
      mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
      const float mnew = fmaxf(mrun[m], mloc);
      alpha[m] = exp2f((mrun[m] - mnew) * LOG2E);
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float p = vis[e] ? exp2f((v[e] - mnew) * LOG2E) : 0.f;
        const bf16_t hi = f2bf(p);
        ph[m][e] = hi;
        pl[m][e] = f2bf(p - bf2f(hi));
        psum += p;
      }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      lrun[m] = lrun[m] * alpha[m] + psum;
      mrun[m] = mnew;
      }
    }
    // O^T += V^T P^T: A rows = value columns 16 t + c, k = keys 8 g .. + 8 of the block
#pragma unroll
    for (int m = 0; m < MW; ++m) {
      const int j = (m / P) / HPK;
#pragma unroll
      for (int t = 0; t < NDV; ++t) {
        if (t < ndv) {
          f32x4 o = SIG ? acc[m][t] : acc[m][t] * alpha[m];
          o = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[j][t], ph[m], o, 0, 0, 0);
          acc[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[j][t], pl[m], o, 0, 0, 0);
        }
      }
    }
  }
  if (!wave_on || !row_ok) return;
  // this lane holds, per map and tile t, value columns 16 t + 4 g + i of query c
  if (np > 1) {                                     // partials; window_attn_merge finishes the row
#pragma unroll
    for (int m = 0; m < MW; ++m) {
      const long pr = ((row * M + h0 * P + m) * a.nparts + blockIdx.z);
      if (g == 0) {
        a.part_ml[pr * 2] = mrun[m];
        a.part_ml[pr * 2 + 1] = lrun[m];
      }
#pragma unroll
      for (int t = 0; t < NDV; ++t)
        if (t < ndv) *reinterpret_cast<f32x4*>(a.part_acc + pr * Dv + 16 * t + 4 * g) = acc[m][t];
    }
    return;
  }
  if (a.epilogue == 0) {
    const bf16_t* gate = (const bf16_t*)a.gate;
#pragma unroll
    for (int m = 0; m < MW; ++m) {
      const float inv = a.post / lrun[m];
#pragma unroll
      for (int t = 0; t < NDV; ++t) {
        if (t < ndv) {
          const int col = (h0 + m) * Dv + 16 * t + 4 * g;
          bf16x4 o;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float v = acc[m][t][i] * inv;
            if (gate) v *= 1.0f / (1.0f + __expf(-bf2f(gate[row * a.ldg + col + i])));
            o[i] = f2bf(v);
          }
          *reinterpret_cast<bf16x4*>(out + row * a.ldo + col) = o;
        }
      }
    }
  } else {
    const float lam = a.lam[0];
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) {
      const float i1 = 1.0f / lrun[2 * hh], i2 = lam / lrun[2 * hh + 1];
      float ss = 0.f;
#pragma unroll
      for (int t = 0; t < NDV; ++t) {
        if (t < ndv) {
          const f32x4 o = acc[2 * hh][t] * i1 - acc[2 * hh + 1][t] * i2;
          acc[2 * hh][t] = o;
          ss += o[0] * o[0] + o[1] * o[1] + o[2] * o[2] + o[3] * o[3];
        }
      }
      ss += __shfl_xor(ss, 16, 64);
      ss += __shfl_xor(ss, 32, 64);
      const float inv = a.post / sqrtf(ss / (float)Dv + a.eps);
#pragma unroll
      for (int t = 0; t < NDV; ++t) {
        if (t < ndv) {
          bf16x4 o;
#pragma unroll
          for (int i = 0; i < 4; ++i) o[i] = f2bf(acc[2 * hh][t][i] * inv);
          *reinterpret_cast<bf16x4*>(out + row * a.ldo + (h0 + hh) * Dv + 16 * t + 4 * g) = o;
        }
      }
    }
  }
}

// Merge of key partitions and the row's epilogue: one wave per (row, head).  Lane z first turns
// partition z's (max, sum) into its weight; the value columns are then summed over the partitions
// with independent loads (nparts <= 64).
__global__ void __launch_bounds__(64)
window_attn_merge_kernel(const WinAttnArgs a) {
  const int H = a.H, P = a.P, Dv = a.Dv, M = H * P, NP = a.nparts;
  const long row = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  bf16_t* out = (bf16_t*)a.out + row * a.ldo + h * Dv;
  if (a.lens && a.lens[row] <= 0) return;           // padding row: the partition kernel wrote zeros
  const int pos = a.positions[row];
  const int np = wa_parts(NP, wa_blocks(pos, pos, a.window, a.keep).nblocks);
  if (np == 1) return;                              // a whole row: already finished and written
  float o[2][2];                                    // [map][column lane, lane + 64]
  for (int pm = 0; pm < P; ++pm) {
    const long pr = (row * M + h * P + pm) * NP;
    const float mz = lane < np ? a.part_ml[(pr + lane) * 2] : -1e30f;
    const float lz = lane < np ? a.part_ml[(pr + lane) * 2 + 1] : 0.f;
    // sigmoid weights: the partitions' sums simply add up
    const float wz = a.wmode == 1 ? (lane < np ? 1.f : 0.f) : __expf(mz - wave_max(mz));
    const float inv = a.wmode == 1 ? 1.f : 1.0f / wave_sum(wz * lz);
    float v0 = 0.f, v1 = 0.f;
#pragma unroll 4
    for (int z = 0; z < np; ++z) {
      const float w = __shfl(wz, z, 64);
      if (lane < Dv) v0 += w * a.part_acc[(pr + z) * Dv + lane];
      if (lane + 64 < Dv) v1 += w * a.part_acc[(pr + z) * Dv + lane + 64];
    }
    o[pm][0] = v0 * inv;
    o[pm][1] = v1 * inv;
  }
  float r0, r1;
  if (a.epilogue == 0) {
    const bf16_t* gate = (const bf16_t*)a.gate;
    r0 = o[0][0] * a.post;
    r1 = o[0][1] * a.post;
    if (gate) {
      if (lane < Dv) r0 *= 1.0f / (1.0f + __expf(-bf2f(gate[row * a.ldg + h * Dv + lane])));
      if (lane + 64 < Dv) r1 *= 1.0f / (1.0f + __expf(-bf2f(gate[row * a.ldg + h * Dv + lane + 64])));
    }
  } else {
    const float lam = a.lam[0];
    r0 = lane < Dv ? o[0][0] - lam * o[1][0] : 0.f;
    r1 = lane + 64 < Dv ? o[0][1] - lam * o[1][1] : 0.f;
    const float inv = a.post / sqrtf(wave_sum(r0 * r0 + r1 * r1) / (float)Dv + a.eps);
    r0 *= inv;
    r1 *= inv;
  }
  if (lane < Dv) out[lane] = f2bf(r0);
  if (lane + 64 < Dv) out[lane + 64] = f2bf(r1);
}

// Heads per wave of the MFMA form for (H, P), 0 when the shape runs the scalar form: with head
// mixing one workgroup must hold every head (H / HW <= 8 waves of one or two heads); without it
// the heads are spread over grid.y in workgroups of up to four single-head waves.
static int wa_mfma_hw(int H, int P, int talk) {
  if (!talk) return 1;
  if (P != 1) return 0;
  if (H <= 4 || (H <= 8 && H % 2)) return 1;
  if (H <= 16 && H % 2 == 0) return 2;
  return 0;
}

EIA_API int eia_window_attn_mfma_ok(int H, int G, int P, int D, int Dv, int bs, int talk) {
  const int hw = wa_mfma_hw(H, P, talk);
  if (hw == 0 || G < 1 || H % G || D % 8 || D > 128 || Dv % 16 || Dv > 128 || bs % 32) return 0;
  return 1;
}

EIA_API int eia_window_attn_mfma(const void* q, long ldq, const void* kc, const void* vc,
                                 const int* bt, int ldbt, const int* positions, const int* cu,
                                 const int* work, const int* lens, int n_items, const float* mult,
                                 const float* slope, const float* talk, const void* gate, long ldg,
                                 void* out, long ldo, int H, int G, int P, int D, int Dv, int bs,
                                 int window, int keep, int epilogue, const float* lam, float eps,
                                 float post, int wmode, const float* bias, int nparts,
                                 float* part_acc, float* part_ml, const float* sink,
                                 hipStream_t st) {
  if (n_items < 0 || H < 1 || G < 1 || H % G || (P != 1 && P != 2) || bs < 1 || keep < 0 || !q ||
      !kc || !vc || !bt || !positions || !mult || !out)
    return EIA_BAD_SHAPE;
  if ((cu == nullptr) != (work == nullptr)) return EIA_BAD_SHAPE;
  if ((epilogue == 1) != (P == 2) || (epilogue == 1 && (gate || !lam))) return EIA_BAD_SHAPE;
  if ((wmode != 0 && wmode != 1) || (wmode == 1 && (talk || P != 1 || sink))) return EIA_BAD_SHAPE;
  if (!eia_window_attn_mfma_ok(H, G, P, D, Dv, bs, talk != nullptr)) return EIA_UNSUPPORTED;
  if (ldq % 8 || ldo % 4) return EIA_BAD_SHAPE;
  // key partitions: decode rows only (a row is its own work item), partials in the workspace
  if (nparts < 1 || nparts > 64 || (nparts > 1 && (cu || !part_acc || !part_ml)))
    return EIA_BAD_SHAPE;
  if (n_items == 0) return EIA_OK;
  WinAttnArgs a{q, ldq, kc, vc, bt, ldbt, positions, cu, work, lens, mult, slope, talk, gate, ldg,
                out, ldo, H, G, P, D, Dv, bs, window, keep, 16, epilogue, lam, eps, post, nparts,
                2, part_acc, part_ml, wmode, bias, sink};
  // raw-score buffers of the head-mixing form: two (one barrier per block) while they fit 48 KiB
  if (talk) a.raw_bufs = (size_t)2 * H * P * 128 * sizeof(f32x4) > 48 * 1024 ? 1 : 2;
  // sigmoid weights: a wave takes two heads of one kv head where the grouping allows it, so the
  // block's K / V^T operands are loaded once for both (the kernel is bound by those loads)
  const int hw = (wmode == 1 && (H / G) % 2 == 0) ? 2 : wa_mfma_hw(H, P, talk != nullptr);
  const int waves_needed = H / hw;
  const int nwv = talk ? waves_needed : (waves_needed < 4 ? waves_needed : 4);
  const int gy = talk ? 1 : (waves_needed + nwv - 1) / nwv;
  const size_t lds = talk ? (size_t)a.raw_bufs * H * P * 128 * sizeof(f32x4) +
                                sizeof(float) * ((H * H + 3) & ~3) : 0;
  if (lds > 128 * 1024) return EIA_UNSUPPORTED;
  const bool share = (H / G) % hw == 0;          // the heads of a wave read one kv head
  const bool big = D > 64 || Dv > 64;
  dim3 grid(n_items, gy, nparts), block(64 * nwv);
#define WA_LAUNCH1(HWV, PV, TK, SH, NDX, NDVX)                                                  \
  do {                                                                                          \
    if (lds > 48 * 1024)                                                                        \
      (void)hipFuncSetAttribute(                                                                \
          reinterpret_cast<const void*>(&window_attn_mfma_kernel<HWV, PV, TK, SH, NDX, NDVX>),  \
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                                \
    hipLaunchKernelGGL((window_attn_mfma_kernel<HWV, PV, TK, SH, NDX, NDVX>), grid, block, lds, \
                       st, a);                                                                  \
  } while (0)
#define WA_LAUNCH(HWV, PV, TK, SH)                                                              \
  do {                                                                                          \
    if (big) WA_LAUNCH1(HWV, PV, TK, SH, 4, 8);                                                 \
    else WA_LAUNCH1(HWV, PV, TK, SH, 2, 4);                                                     \
  } while (0)
#define WA_LAUNCH_SIG(NDX, NDVX)                                                                \
  do {                                                                                          \
    if (hw == 2)                                                                                \
      hipLaunchKernelGGL((window_attn_mfma_kernel<2, 1, false, true, NDX, NDVX, true>), grid,   \
                         block, lds, st, a);                                                    \
    else                                                                                        \
      hipLaunchKernelGGL((window_attn_mfma_kernel<1, 1, false, true, NDX, NDVX, true>), grid,   \
                         block, lds, st, a);                                                    \
  } while (0)
  // without head mixing the key width may be half the value width (a differential pair)
  const bool narrow_k = !talk && D <= 64 && Dv > 64;
  if (talk) {
    if (hw == 1) WA_LAUNCH(1, 1, true, true);
    else if (share) WA_LAUNCH(2, 1, true, true);
    else WA_LAUNCH(2, 1, true, false);
  } else if (P == 2) {
    if (narrow_k) WA_LAUNCH1(1, 2, false, true, 2, 8);
    else WA_LAUNCH(1, 2, false, true);
  } else if (wmode == 1) {
    if (narrow_k) WA_LAUNCH_SIG(2, 8);
    else if (big) WA_LAUNCH_SIG(4, 8);
    else WA_LAUNCH_SIG(2, 4);
  } else {
    if (narrow_k) WA_LAUNCH1(1, 1, false, true, 2, 8);
    else WA_LAUNCH(1, 1, false, true);
  }
#undef WA_LAUNCH_SIG
#undef WA_LAUNCH
#undef WA_LAUNCH1
  if (nparts > 1)
    hipLaunchKernelGGL(window_attn_merge_kernel, dim3(n_items, H), dim3(64), 0, st, a);
  EIA_LAUNCH_CHECK();
}
