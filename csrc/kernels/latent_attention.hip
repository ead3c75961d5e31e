// Latent (low-rank KV) attention over a paged latent cache.
//
// Cache row of one token: [ c (kv_rank, RMS-normed latent) | k_rot (rot_dim, rotated key part
// shared by all heads) ].  With the key up-projection absorbed into the query,
//   q_abs[h] = W_uk[h]^T q_nope[h]                       (a batched GEMM, done by the caller)
//   score[h][j] = (q_abs[h] . c_j + rot(q_rot[h]) . k_rot_j) * scale
//   lat[h] = sum_j softmax(score[h])_j c_j                (value up-projection by the caller)
// every head reads the SAME cache rows, so a workgroup stages a key tile in LDS once and uses it
// for all (query, head) rows it owns.  Options: a sliding window (position i sees j with
// 0 <= i - j < window), a per-head sink (the softmax denominator also holds exp(sink[h]), which
// has no key and no value and is not scaled), and the pair layout of the rotation ((2i, 2i+1) or
// (i, i + rot_dims/2)) with a common factor on cos and sin.  Scores, softmax weights and the
// accumulators are fp32; activations are bf16 or fp32 (template T).
//
//   eia_latent_prep : RMS-norm of the query latent, RMS-norm of c, rotation of k_rot, cache write
//   eia_latent_attn : rotation of q_rot, tiled online-softmax attention, sigmoid head gate
#include "eia_common.h"

// Entry d (< rot_dims) of a vector after the rotation by position pos: src holds the unrotated
// vector; pairs are (2i, 2i+1), or (i, i + rot_dims/2) when half; cos and sin are times amp.
template <typename T>
EIA_DEV float lat_rotated(const T* src, int d, int rot_dims, bool half, float amp, float pos,
                          const float* __restrict__ inv_freq) {
  const int hd = rot_dims >> 1;
  const int i = half ? (d < hd ? d : d - hd) : (d >> 1);
  const bool second = half ? d >= hd : (d & 1);
  float sn, cs;
  sincosf(pos * inv_freq[i], &sn, &cs);
  sn *= amp;
  cs *= amp;
  const float u = ld_f32<T>(src, half ? i : 2 * i), w = ld_f32<T>(src, half ? i + hd : 2 * i + 1);
  return second ? (w * cs + u * sn) : (u * cs - w * sn);
}

// ------------------------------------------------------------------------------------------ prep
// fused [T, ld]: columns [q_off, q_off+q_rank) query latent, [c_off, c_off+R) KV latent,
// [kr_off, kr_off+rd) shared rotary key part.  q_rank == 0: no query latent; cache == nullptr:
// no KV part (a layer that reads another layer's cache).
template <typename T>
__global__ void __launch_bounds__(128)
latent_prep_kernel(const T* __restrict__ fused, long ld, int q_off, int q_rank,
                   const T* __restrict__ wq, T* __restrict__ cq, long ldcq, int c_off, int R,
                   const T* __restrict__ wc, int kr_off, int rd, int rot_dims,
                   const float* __restrict__ inv_freq, const int* __restrict__ positions,
                   const int* __restrict__ slot_mapping, T* __restrict__ cache, long cache_row,
                   float eps, int rot_half, float rot_amp) {
  __shared__ float scratch[2];
  const long t = blockIdx.x;
  const T* row = fused + t * ld;
  if (q_rank > 0) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < q_rank; c += blockDim.x) {
      const float v = ld_f32<T>(row, q_off + c);
      ss += v * v;
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
    for (int c = threadIdx.x; c < q_rank; c += blockDim.x)
      st_f32<T>(cq + t * ldcq, c, ld_f32<T>(row, q_off + c) * inv * ld_f32<T>(wq, c));
  }
  if (cache == nullptr) return;
  const int slot = slot_mapping[t];
  if (slot < 0) return;                       // uniform per workgroup
  T* dst = cache + (long)slot * cache_row;
  float ss = 0.f;
  for (int c = threadIdx.x; c < R; c += blockDim.x) {
    const float v = ld_f32<T>(row, c_off + c);
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)R + eps);
  for (int c = threadIdx.x; c < R; c += blockDim.x)
    st_f32<T>(dst, c, ld_f32<T>(row, c_off + c) * inv * ld_f32<T>(wc, c));
  const float pos = (float)positions[t];
  for (int d = threadIdx.x; d < rd; d += blockDim.x) {
    const float v = d < rot_dims
        ? lat_rotated<T>(row + kr_off, d, rot_dims, rot_half != 0, rot_amp, pos, inv_freq)
        : ld_f32<T>(row, kr_off + d);
    st_f32<T>(dst, R + d, v);
  }
}

EIA_API int eia_latent_prep(const void* fused, long ld, int q_off, int q_rank, const void* wq,
                            void* cq, long ldcq, int c_off, int R, const void* wc, int kr_off,
                            int rd, int rot_dims, const float* inv_freq, const int* positions,
                            const int* slot_mapping, void* cache, long cache_row, float eps,
                            int rot_half, float rot_amp, int T_, int is_bf16, hipStream_t st) {
  if (T_ < 0 || q_rank < 0 || (cache && (R < 1 || rd < 0 || rot_dims > rd || (rot_dims & 1))))
    return EIA_BAD_SHAPE;
  if (T_ == 0) return EIA_OK;
  if (is_bf16)
    hipLaunchKernelGGL((latent_prep_kernel<bf16_t>), dim3(T_), dim3(128), 0, st,
                       (const bf16_t*)fused, ld, q_off, q_rank, (const bf16_t*)wq, (bf16_t*)cq,
                       ldcq, c_off, R, (const bf16_t*)wc, kr_off, rd, rot_dims, inv_freq, positions,
                       slot_mapping, (bf16_t*)cache, cache_row, eps, rot_half, rot_amp);
  else
    hipLaunchKernelGGL((latent_prep_kernel<float>), dim3(T_), dim3(128), 0, st,
                       (const float*)fused, ld, q_off, q_rank, (const float*)wq, (float*)cq, ldcq,
                       c_off, R, (const float*)wc, kr_off, rd, rot_dims, inv_freq, positions,
                       slot_mapping, (float*)cache, cache_row, eps, rot_half, rot_amp);
  EIA_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------- attention
// Key partitions a decode row uses out of the launch's grid.z: at least two 32-key units each.
EIA_DEV int lat_parts(int nparts, int kmin, int kmax) {
  return min(nparts, max(1, ((kmax - kmin + 31) >> 5) >> 1));
}

#define LAT_ACC_MAX 32     // fp32 accumulators per thread: QB * HB * R <= 256 * LAT_ACC_MAX

struct LatentAttnArgs {
  const void* qa; long qa_st, qa_sh;        // absorbed queries (t, h, r)
  const void* qr; long qr_st, qr_sh;        // rotary query part, not yet rotated (t, h, d)
  const float* inv_freq; int rot_dims;
  const void* cache; long cache_row;        // rows of R + rd
  const int* block_table; int bt_stride;
  const int* seq_lens;                      // nullable: rows with 0 are padding
  const int* cu_q;                          // nullable: one query per sequence (decode)
  const int* work; int n_work;              // nullable with cu_q == nullptr: item = sequence
  const int* positions;                     // per query row
  const void* gate; long gate_st;           // nullable: sigmoid(gate[t][h]) scales head h
  void* out; long out_st, out_sh;           // (t, h, r)
  float scale; int H, R, rd, bs, QB, HB, KC, ldk;
  int window;                               // > 0: position i sees j with 0 <= i - j < window
  const float* sink;                        // nullable [H]: exp(sink[h]) joins the denominator
  int rot_half; float rot_amp;              // pair layout and cos / sin factor of the rotation
  // MFMA decode only: the keys of a row split over grid.z partitions; each writes its
  // unnormalised accumulators and (running max in log2 units, sum) for the merge kernel
  int nparts; float* part_acc; float* part_ml;
};

template <typename T>
__global__ void __launch_bounds__(256)
latent_attn_kernel(LatentAttnArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int Dk = a.R + a.rd, M = a.QB * a.HB, KC = a.KC, ldk = a.ldk;
  float* qs = reinterpret_cast<float*>(smem);            // [M][Dk]
  float* ps = qs + (long)M * Dk;                         // [M][KC]
  float* mrow = ps + (long)M * KC;                       // [M]
  float* lrow = mrow + M;                                // [M]
  float* arow = lrow + M;                                // [M]
  T* kt = reinterpret_cast<T*>(arow + M);                // [KC][ldk]

  int seq, row0, ntok;
  if (a.cu_q) {
    seq = a.work[2 * blockIdx.x];
    const int q0 = a.work[2 * blockIdx.x + 1];
    const int lo = a.cu_q[seq], hi = a.cu_q[seq + 1];
    row0 = lo + q0;
    ntok = min(a.QB, hi - row0);
  } else {
    seq = blockIdx.x;
    row0 = seq;
    ntok = 1;
  }
  if (ntok <= 0 || (a.seq_lens && a.seq_lens[seq] <= 0)) return;
  const int h0 = blockIdx.y * a.HB;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* qa = static_cast<const T*>(a.qa);
  const T* qr = static_cast<const T*>(a.qr);
  const T* cache = static_cast<const T*>(a.cache);
  const int* bt = a.block_table + (long)seq * a.bt_stride;

  // queries -> LDS (rotated, pre-scaled); rows of absent tokens / heads are zero
  for (int e = tid; e < M * Dk; e += 256) {
    const int m = e / Dk, d = e - m * Dk;
    const int t = m / a.HB, h = h0 + (m - t * a.HB);
    float v = 0.f;
    if (t < ntok && h < a.H) {
      const long row = row0 + t;
      if (d < a.R) {
        v = ld_f32<T>(qa, row * a.qa_st + h * a.qa_sh + d);
      } else {
        const int dd = d - a.R;
        const T* src = qr + row * a.qr_st + h * a.qr_sh;
        v = dd < a.rot_dims
            ? lat_rotated<T>(src, dd, a.rot_dims, a.rot_half != 0, a.rot_amp,
                             (float)a.positions[row], a.inv_freq)
            : ld_f32<T>(src, dd);
      }
      v *= a.scale;
    }
    qs[e] = v;
  }
  for (int m = tid; m < M; m += 256) {
    mrow[m] = -INFINITY;
    lrow[m] = 0.f;
    arow[m] = 1.f;
  }
  float acc[LAT_ACC_MAX];
#pragma unroll
  for (int i = 0; i < LAT_ACC_MAX; ++i) acc[i] = 0.f;
  const int nacc = (M * a.R + 255) >> 8;
  const int kmax = a.positions[row0 + ntok - 1] + 1;     // keys kmin..kmax-1 are visible to the tile
  const int kmin = a.window > 0 ? max(0, a.positions[row0] - a.window + 1) : 0;
  __syncthreads();

  for (int k0 = kmin; k0 < kmax; k0 += KC) {
    // key tile -> LDS
    for (int e = tid; e < KC * Dk; e += 256) {
      const int j = e / Dk, d = e - j * Dk;
      const int kp = k0 + j;
      T v = (T)0.f;
      if (kp < kmax) {
        const long slot = (long)bt[kp / a.bs] * a.bs + (kp % a.bs);
        v = cache[slot * a.cache_row + d];
      }
      kt[j * ldk + d] = v;
    }
    __syncthreads();
    // scores: consecutive lanes take consecutive keys of one query row
    for (int e = tid; e < M * KC; e += 256) {
      const int m = e / KC, j = e - m * KC;
      const int t = m / a.HB;
      const int kp = k0 + j;
      float s = -INFINITY;
      if (t < ntok && kp <= a.positions[row0 + t] &&
          (a.window <= 0 || a.positions[row0 + t] - kp < a.window)) {
        const float* q = qs + (long)m * Dk;
        const T* k = kt + (long)j * ldk;
        s = 0.f;
        for (int d = 0; d < Dk; ++d) s += q[d] * ld_f32<T>(k, d);
      }
      ps[e] = s;
    }
    __syncthreads();
    // online softmax per row: one wave per row, lanes over the tile's keys
    for (int m = wave; m < M; m += 4) {
      float tmax = -INFINITY;
      for (int j = lane; j < KC; j += 64) tmax = fmaxf(tmax, ps[m * KC + j]);
      tmax = wave_max(tmax);
      const float mold = mrow[m];
      const float mnew = fmaxf(mold, tmax);
      float psum = 0.f;
      for (int j = lane; j < KC; j += 64) {
        const float s = ps[m * KC + j];
        const float p = (s == -INFINITY) ? 0.f : expf(s - mnew);
        ps[m * KC + j] = p;
        psum += p;
      }
      psum = wave_sum(psum);
      if (lane == 0) {
        const float al = (mold == -INFINITY) ? ((mnew == -INFINITY) ? 1.f : 0.f) : expf(mold - mnew);
        arow[m] = al;
        lrow[m] = lrow[m] * al + psum;
        mrow[m] = mnew;
      }
    }
    __syncthreads();
    // accumulate the latent part of the keys
#pragma unroll
    for (int i = 0; i < LAT_ACC_MAX; ++i) {
      if (i < nacc) {
        const int e = tid + (i << 8);
        const int m = e / a.R, r = e - m * a.R;
        if (m < M) {
          float v = acc[i] * arow[m];
          const float* p = ps + (long)m * KC;
          for (int j = 0; j < KC; ++j) v += p[j] * ld_f32<T>(kt, (long)j * ldk + r);
          acc[i] = v;
        }
      }
    }
    __syncthreads();
  }

  T* out = static_cast<T*>(a.out);
  const T* gate = static_cast<const T*>(a.gate);
#pragma unroll
  for (int i = 0; i < LAT_ACC_MAX; ++i) {
    if (i < nacc) {
      const int e = tid + (i << 8);
      const int m = e / a.R, r = e - m * a.R;
      if (m < M) {
        const int t = m / a.HB, h = h0 + (m - t * a.HB);
        if (t < ntok && h < a.H) {
          const long row = row0 + t;
          float l = lrow[m];
          if (a.sink) l += expf(a.sink[h] - mrow[m]);
          float v = acc[i] / l;
          if (gate) v *= 1.0f / (1.0f + expf(-ld_f32<T>(gate, row * a.gate_st + h)));
          st_f32<T>(out, row * a.out_st + h * a.out_sh + r, v);
        }
      }
    }
  }
}

// n_items: sequences (cu_q == nullptr, one query row per sequence) or work items (seq, first
// query) of QB queries each.  Heads are processed HB at a time (grid.y).
EIA_API int eia_latent_attn(const void* qa, long qa_st, long qa_sh, const void* qr, long qr_st,
                            long qr_sh, const float* inv_freq, int rot_dims, const void* cache,
                            long cache_row, const int* block_table, int bt_stride,
                            const int* seq_lens, const int* cu_q, const int* work, int n_items,
                            const int* positions, const void* gate, long gate_st, void* out,
                            long out_st, long out_sh, float scale, int H, int R, int rd, int bs,
                            int QB, int window, const float* sink, int rot_half, float rot_amp,
                            int is_bf16, hipStream_t st) {
  if (H < 1 || R < 1 || rd < 0 || bs < 1 || QB < 1 || rot_dims > rd || (rot_dims & 1) ||
      cache_row < R + rd || (cu_q && !work))
    return EIA_BAD_SHAPE;
  if (n_items <= 0) return EIA_OK;
  int HB = H < 16 ? H : 16;
  while (HB > 1 && (long)QB * HB * R > 256L * LAT_ACC_MAX) HB = (HB + 1) / 2;
  if ((long)QB * HB * R > 256L * LAT_ACC_MAX) return EIA_UNSUPPORTED;
  const int Dk = R + rd, M = QB * HB;
  const int esz = is_bf16 ? 2 : 4;
  // key-tile row stride: an odd number of 32-bit words, so lanes reading one column of
  // consecutive rows hit distinct LDS banks
  int ldk = Dk;
  if (is_bf16) { ldk += ldk & 1; if (((ldk / 2) & 1) == 0) ldk += 2; }
  else if ((ldk & 1) == 0) ldk += 1;
  int KC = 64;
  size_t lds = 0;
  for (;; KC >>= 1) {
    lds = ((size_t)M * Dk + (size_t)M * KC + 3 * (size_t)M) * 4 + (size_t)KC * ldk * esz;
    if (lds <= 96 * 1024 || KC == 8) break;
  }
  if (lds > 150 * 1024) return EIA_UNSUPPORTED;
  LatentAttnArgs a{qa, qa_st, qa_sh, qr, qr_st, qr_sh, inv_freq, rot_dims, cache, cache_row,
                   block_table, bt_stride, seq_lens, cu_q, work, n_items, positions, gate, gate_st,
                   out, out_st, out_sh, scale, H, R, rd, bs, QB, HB, KC, ldk, window, sink, rot_half,
                   rot_amp, 1, nullptr, nullptr};
  dim3 grid(n_items, (H + HB - 1) / HB);
  if (is_bf16) {
    if (lds > 48 * 1024)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attn_kernel<bf16_t>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL((latent_attn_kernel<bf16_t>), grid, dim3(256), lds, st, a);
  } else {
    if (lds > 48 * 1024)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attn_kernel<float>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL((latent_attn_kernel<float>), grid, dim3(256), lds, st, a);
  }
  EIA_LAUNCH_CHECK();
}

// --------------------------------------------------------------------------- MFMA form (bf16)
// Flash-style kernel on v_mfma_f32_16x16x32_bf16.  A workgroup of NW waves owns NW x 16 rows
// (row = (query, head) pair; every row reads the same keys) and walks the keys in units of 32.
// Per unit the workgroup stages the 32 cache rows in LDS twice: row-major ("K tile", the A
// operand of S^T = K Q^T) and transposed ("V^T tile", latent columns only, the A operand of
// O^T = V^T P^T).  The K tile rows are stored in the order the two S^T tiles read them, so that
// their accumulators hold, per lane, one row's scores of keys 8g..8g+7 -- exactly the B operand
// of the second product (no shuffle, no LDS round trip for P).  Softmax weights stay fp32: P
// is fed as a bf16 high part plus a bf16 remainder (two MFMAs), and the normaliser sums the
// fp32 weights.  The next unit's cache rows are prefetched into registers during the products.
// SPLITV (decode, one query): all NW waves own the SAME 16 rows (the heads of one query) and
// each takes every NW-th latent column tile of the second product; the first product is
// repeated per wave (decode is bound by the cache stream, not by MFMA issue), which buys NW
// times the loading threads (so the prefetch fits) and a quarter of the accumulators.
template <int NKMAX, int NCMAX, int NW, bool SPLITV>
__global__ void __launch_bounds__(NW * 64)
latent_attn_mfma_kernel(LatentAttnArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int NT = NW * 64;
  constexpr int PRE = (32 * NKMAX * 4 + NT - 1) / NT;      // 16-byte chunks per thread per unit
  constexpr bool PREFETCH = PRE <= 12;                     // else the registers go to Q and O
  const int Dk = a.R + a.rd;
  const int nk = (Dk + 31) >> 5, Dkp = nk << 5;            // k-steps of 32
  const int nc = (a.R + 15) >> 4;                          // latent column tiles of 16
  const int ldk = a.ldk;                                   // K tile row stride (elements)
  constexpr int LDV = 40;                                  // V^T tile row stride (elements)
  bf16_t* kt = reinterpret_cast<bf16_t*>(smem);            // [32][ldk]
  bf16_t* vt = kt + 32 * ldk;                              // [nc * 16][LDV]

  int seq, row0, ntok;
  if (a.cu_q) {
    seq = a.work[2 * blockIdx.x];
    const int q0 = a.work[2 * blockIdx.x + 1];
    row0 = a.cu_q[seq] + q0;
    ntok = min(a.QB, a.cu_q[seq + 1] - row0);
  } else {
    seq = blockIdx.x;
    row0 = seq;
    ntok = 1;
  }
  if (ntok <= 0 || (a.seq_lens && a.seq_lens[seq] <= 0)) return;
  {   // a partition beyond the ones this row's context uses has nothing to do (whole workgroup)
    const int kmax0 = a.positions[row0 + ntok - 1] + 1;
    const int kmin0 = a.window > 0 ? (max(0, a.positions[row0] - a.window + 1) & ~31) : 0;
    if ((int)blockIdx.z >= lat_parts(a.nparts, kmin0, kmax0)) return;
  }
  const int h0 = blockIdx.y * a.HB;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int c = lane & 15, g = lane >> 4;
  const bf16_t* cache = static_cast<const bf16_t*>(a.cache);
  const int* bt = a.block_table + (long)seq * a.bt_stride;

  // this lane's row (B operand column / accumulator column)
  const int m = SPLITV ? c : wave * 16 + c;
  const int t = m / a.HB, h = h0 + (m - t * a.HB);
  const bool row_ok = t < ntok && h < a.H && m < a.QB * a.HB;
  const long row = row0 + (row_ok ? t : 0);
  const int qpos = row_ok ? a.positions[row] : -1;
  // the rotary query parts of the workgroup's rows, rotated once into LDS: a thread takes whole
  // pairs (one sine / cosine each, independent loads), not the entries of its own operand
  bf16_t* qrs = vt + nc * 16 * LDV;                        // [rows][rd]
  {
    constexpr int NROWS = SPLITV ? 16 : NW * 16;
    const bf16_t* qrb = static_cast<const bf16_t*>(a.qr);
    const int hp = a.rot_dims >> 1, npass = a.rd - a.rot_dims;
    for (int e = tid; e < NROWS * hp; e += NT) {
      const int mm = e / hp, i = e - mm * hp;
      const int tt = mm / a.HB, hh = h0 + (mm - tt * a.HB);
      if (tt < ntok && hh < a.H && mm < a.QB * a.HB) {
        const bf16_t* src = qrb + (long)(row0 + tt) * a.qr_st + (long)hh * a.qr_sh;
        const int ia = a.rot_half ? i : 2 * i, ib = a.rot_half ? i + hp : 2 * i + 1;
        const float u = bf2f(src[ia]), w = bf2f(src[ib]);
        float sn, cs;
        sincosf((float)a.positions[row0 + tt] * a.inv_freq[i], &sn, &cs);
        sn *= a.rot_amp;
        cs *= a.rot_amp;
        qrs[mm * a.rd + ia] = f2bf(u * cs - w * sn);
        qrs[mm * a.rd + ib] = f2bf(w * cs + u * sn);
      }
    }
    for (int e = tid; e < NROWS * npass; e += NT) {        // entries past rot_dims pass unchanged
      const int mm = e / npass, d = a.rot_dims + (e - mm * npass);
      const int tt = mm / a.HB, hh = h0 + (mm - tt * a.HB);
      if (tt < ntok && hh < a.H && mm < a.QB * a.HB)
        qrs[mm * a.rd + d] = qrb[(long)(row0 + tt) * a.qr_st + (long)hh * a.qr_sh + d];
    }
    __syncthreads();
  }
  bf16x8 qf[NKMAX];
  {
    const bf16_t* qa = static_cast<const bf16_t*>(a.qa) + row * a.qa_st + (long)h * a.qa_sh;
    // R % 8 == 0 and rd % 8 == 0: a lane's 8-entry chunk lies wholly in the absorbed part (one
    // 16-byte load when the rows are aligned) or wholly in the rotary part (one LDS read)
    const bool qvec = ((reinterpret_cast<uintptr_t>(a.qa) | (uintptr_t)(a.qa_st * 2) |
                        (uintptr_t)(a.qa_sh * 2)) & 15) == 0;
#pragma unroll
    for (int s = 0; s < NKMAX; ++s) {
      const int d0 = s * 32 + 8 * g;
      bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (row_ok && s < nk && d0 < Dk) {
        if (d0 >= a.R) {
          v = *reinterpret_cast<const bf16x8*>(qrs + m * a.rd + (d0 - a.R));
        } else if (qvec) {
          v = *reinterpret_cast<const bf16x8*>(qa + d0);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = qa[d0 + e];
        }
      }
      qf[s] = v;
    }
  }
  constexpr int NACC = SPLITV ? (NCMAX + NW - 1) / NW : NCMAX;   // column tiles of this wave
  const int ct0 = SPLITV ? wave : 0, ctstep = SPLITV ? NW : 1;   // tile i -> ct0 + i * ctstep
  f32x4 acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; ++i) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float mrun = -INFINITY, lrun = 0.f;
  const float scale_log2 = a.scale * 1.4426950408889634f;
  const int kmax = a.positions[row0 + ntok - 1] + 1;
  // first 32-key unit that holds a key some row of the tile sees
  const int kmin = a.window > 0 ? (max(0, a.positions[row0] - a.window + 1) & ~31) : 0;
  int k_begin = kmin, k_end = kmax;
  // partitions this row really uses: at least two 32-key units each (decided here and, the same
  // way, in the merge kernel), so short contexts do not pay for idle partitions
  const int np = lat_parts(a.nparts, kmin, kmax);
  if (np > 1) {                                            // this partition's run of 32-key units
    const int units = (kmax - kmin + 31) >> 5;
    const int per = (units + np - 1) / np;
    k_begin = kmin + (min((int)blockIdx.z * per, units) << 5);
    k_end = min(kmax, kmin + (((int)blockIdx.z + 1) * per << 5));
  }
  const int wlo = a.window > 0 ? qpos - a.window + 1 : 0;   // first key this lane's row sees
  const int cpr = Dkp >> 3;                                // 16-byte chunks per (padded) key row
  const int nchunk = 32 * cpr;

  auto load_chunk = [&](int k0, int ch) {
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    const int j = ch / cpr, d = (ch - j * cpr) << 3;
    const int kp = k0 + j;
    if (kp < k_end && d < Dk) {                            // Dk % 8 == 0: whole chunk inside
      const long slot = (long)bt[kp / a.bs] * a.bs + (kp % a.bs);
      v = *reinterpret_cast<const bf16x8*>(cache + slot * a.cache_row + d);
    }
    return v;
  };
  // key j = 8G + i lands in K tile row 4G + i (i < 4) or 16 + 4G + i - 4
  auto store_chunk = [&](int ch, bf16x8 v) {
    const int j = ch / cpr, d = (ch - j * cpr) << 3;
    const int r = ((j & 4) ? 16 : 0) + 4 * (j >> 3) + (j & 3);
    *reinterpret_cast<bf16x8*>(kt + r * ldk + d) = v;
  };
  bf16x8 pre[PREFETCH ? PRE : 1];
  auto fetch = [&](int k0) {
    if constexpr (PREFETCH) {
#pragma unroll
      for (int i = 0; i < PRE; ++i) {
        const int ch = tid + i * NT;
        if (ch < nchunk) pre[i] = load_chunk(k0, ch);
      }
    }
  };
  fetch(k_begin);
  for (int k0 = k_begin; k0 < k_end; k0 += 32) {
    if constexpr (PREFETCH) {
#pragma unroll
      for (int i = 0; i < PRE; ++i) {
        const int ch = tid + i * NT;
        if (ch < nchunk) store_chunk(ch, pre[i]);
      }
    } else {
      for (int ch = tid; ch < nchunk; ch += NT) store_chunk(ch, load_chunk(k0, ch));
    }
    __syncthreads();
    // K tile -> V^T tile (latent columns; rows past R are zero from the padded chunks)
    for (int ch = tid; ch < 32 * nc * 2; ch += NT) {
      const int j = ch & 31, d = (ch >> 5) << 3;
      const int r = ((j & 4) ? 16 : 0) + 4 * (j >> 3) + (j & 3);
      bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (d < a.R) v = *reinterpret_cast<const bf16x8*>(kt + r * ldk + d);   // R % 8 == 0
#pragma unroll
      for (int e = 0; e < 8; ++e) vt[(d + e) * LDV + j] = v[e];
    }
    __syncthreads();
    if (k0 + 32 < k_end) fetch(k0 + 32);
    // S^T tiles: keys (rows) x this wave's 16 rows (columns)
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NKMAX; ++s) {
      if (s < nk) {
        const bf16x8 ka = *reinterpret_cast<const bf16x8*>(kt + c * ldk + s * 32 + 8 * g);
        const bf16x8 kb = *reinterpret_cast<const bf16x8*>(kt + (16 + c) * ldk + s * 32 + 8 * g);
        s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qf[s], s0, 0, 0, 0);
        s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kb, qf[s], s1, 0, 0, 0);
      }
    }
    float v[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ka = k0 + 8 * g + i, kb = ka + 4;
      v[i] = (ka <= qpos && ka >= wlo) ? s0[i] * scale_log2 : -INFINITY;
      v[4 + i] = (kb <= qpos && kb >= wlo) ? s1[i] * scale_log2 : -INFINITY;
    }
    float mloc = v[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) mloc = fmaxf(mloc, v[i]);
    mloc = fmaxf(mloc, __shfl_xor(mloc, 16, 64));
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
    const float mnew = fmaxf(mrun, mloc);
    const float muse = (mnew == -INFINITY) ? 0.f : mnew;
    const float alpha = exp2f(mrun - muse);                // mrun = -inf: 0 (nothing summed yet)
    bf16x8 ph, pl;
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float p = exp2f(v[i] - muse);
      const bf16_t hi = f2bf(p);
      ph[i] = hi;
      pl[i] = f2bf(p - bf2f(hi));
      psum += p;
    }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    lrun = lrun * alpha + psum;
    mrun = mnew;
    const bool rescale = !__all(alpha == 1.f);
#pragma unroll
    for (int ai = 0; ai < NACC; ++ai) {
      const int ct = ct0 + ai * ctstep;
      if (ct < nc) {
        const bf16x8 vf = *reinterpret_cast<const bf16x8*>(vt + (ct * 16 + c) * LDV + 8 * g);
        f32x4 o = acc[ai];
        if (rescale) o *= alpha;
        o = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, ph, o, 0, 0, 0);
        acc[ai] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pl, o, 0, 0, 0);
      }
    }
    __syncthreads();
  }
  if (!row_ok) return;
  if (np > 1) {
    const long pr = ((long)row * a.H + h) * a.nparts + blockIdx.z;
    float* pa = a.part_acc + pr * a.R;
#pragma unroll
    for (int ai = 0; ai < NACC; ++ai) {
      const int ct = ct0 + ai * ctstep;
      if (ct < nc) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int col = ct * 16 + 4 * g + i;
          if (col < a.R) pa[col] = acc[ai][i];
        }
      }
    }
    if (g == 0 && (!SPLITV || wave == 0)) {
      a.part_ml[2 * pr] = mrun;
      a.part_ml[2 * pr + 1] = lrun;
    }
    return;
  }
  if (a.sink) lrun += exp2f(a.sink[h] * 1.4426950408889634f - mrun);
  float f = 1.0f / lrun;
  if (a.gate) {
    const bf16_t* gate = static_cast<const bf16_t*>(a.gate);
    f *= 1.0f / (1.0f + expf(-bf2f(gate[row * a.gate_st + h])));
  }
  bf16_t* out = static_cast<bf16_t*>(a.out) + row * a.out_st + (long)h * a.out_sh;
#pragma unroll
  for (int ai = 0; ai < NACC; ++ai) {
    const int ct = ct0 + ai * ctstep;
    if (ct < nc) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int col = ct * 16 + 4 * g + i;
        if (col < a.R) out[col] = f2bf(acc[ai][i] * f);
      }
    }
  }
}

// Merge of the decode partitions: out = sum_p acc_p 2^(m_p - M) / sum_p l_p 2^(m_p - M), times
// the head gate.  One workgroup per (row, head); lane p first turns partition p's (max, sum) into
// its weight, then the threads sum the latent columns over the partitions with independent loads
// (nparts <= 64).  Rows whose context is too short for two partitions were finished by the
// attention kernel itself.
__global__ void __launch_bounds__(128)
latent_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml,
                    int nparts, const int* __restrict__ seq_lens, const int* __restrict__ positions,
                    int window, const bf16_t* __restrict__ gate, long gate_st,
                    const float* __restrict__ sink, bf16_t* __restrict__ out, long out_st,
                    long out_sh, int H, int R) {
  const int row = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63;
  if (seq_lens && seq_lens[row] <= 0) return;
  const int kmax = positions[row] + 1;
  const int kmin = window > 0 ? (max(0, kmax - window) & ~31) : 0;
  const int np = lat_parts(nparts, kmin, kmax);
  if (np == 1) return;
  const long pr = ((long)row * H + h) * nparts;
  const float mp = lane < np ? part_ml[2 * (pr + lane)] : -INFINITY;
  const float lp = lane < np ? part_ml[2 * (pr + lane) + 1] : 0.f;
  const float M = wave_max(mp);
  const float wp = (mp == -INFINITY) ? 0.f : exp2f(mp - M);
  float L = wave_sum(lp * wp);
  if (sink && M != -INFINITY) L += exp2f(sink[h] * 1.4426950408889634f - M);
  float f = L > 0.f ? 1.0f / L : 0.f;
  if (gate) f *= 1.0f / (1.0f + expf(-bf2f(gate[row * gate_st + h])));
  for (int c0 = 0; c0 < R; c0 += blockDim.x) {
    const int c = c0 + threadIdx.x;
    float v = 0.f;
#pragma unroll 4
    for (int p = 0; p < np; ++p) {
      const float w = __shfl(wp, p, 64);
      if (c < R) v += part_acc[(pr + p) * R + c] * w;
    }
    if (c < R) out[row * out_st + h * out_sh + c] = f2bf(v * f);
  }
}

// Rows per work item of the MFMA form: NW waves x 16; HB = min(H, 16) heads, QB = rows / HB
// queries.  Returns QB for (H, prefill) so the host builds its work list with the same number.
EIA_API int eia_latent_attn_mfma_qb(int H, int decode) {
  const int HB = H < 16 ? H : 16;
  return decode ? 1 : (64 / HB);
}

EIA_API int eia_latent_attn_mfma(const void* qa, long qa_st, long qa_sh, const void* qr,
                                 long qr_st, long qr_sh, const float* inv_freq, int rot_dims,
                                 const void* cache, long cache_row, const int* block_table,
                                 int bt_stride, const int* seq_lens, const int* cu_q,
                                 const int* work, int n_items, const int* positions,
                                 const void* gate, long gate_st, void* out, long out_st,
                                 long out_sh, float scale, int H, int R, int rd, int bs, int QB,
                                 int window, const float* sink, int rot_half, float rot_amp,
                                 int nparts, float* part_acc, float* part_ml, hipStream_t st) {
  if (H < 1 || R < 1 || rd < 0 || bs < 1 || QB < 1 || rot_dims > rd || (rot_dims & 1) ||
      cache_row < R + rd || (cu_q && !work))
    return EIA_BAD_SHAPE;
  const int Dk = R + rd;
  // 16-byte chunks must not straddle the latent / rotary boundary or the row end
  if ((R & 7) || (Dk & 7) || (cache_row & 7) || Dk > 640 || R > 512) return EIA_UNSUPPORTED;
  if (n_items <= 0) return EIA_OK;
  const int HB = H < 16 ? H : 16;
  const bool decode = cu_q == nullptr;
  if (QB != eia_latent_attn_mfma_qb(H, decode ? 1 : 0)) return EIA_BAD_SHAPE;
  if (nparts < 1 || nparts > 64 || (nparts > 1 && (!decode || !part_acc || !part_ml)))
    return EIA_BAD_SHAPE;
  const int nk = (Dk + 31) / 32, Dkp = nk * 32, nc = (R + 15) / 16;
  const int ldk = ((Dkp / 8) & 1) ? Dkp : Dkp + 8;       // odd number of 16-byte units per row
  // K tile, V^T tile, and the rotated rotary query parts of up to 64 rows
  const size_t lds = ((size_t)32 * ldk + (size_t)nc * 16 * 40 + (size_t)64 * rd) * 2;
  LatentAttnArgs a{qa, qa_st, qa_sh, qr, qr_st, qr_sh, inv_freq, rot_dims, cache, cache_row,
                   block_table, bt_stride, seq_lens, cu_q, work, n_items, positions, gate, gate_st,
                   out, out_st, out_sh, scale, H, R, rd, bs, QB, HB, 32, ldk, window, sink, rot_half,
                   rot_amp, nparts, part_acc, part_ml};
  dim3 grid(n_items, (H + HB - 1) / HB, nparts);
#define LAT_MFMA(NK, NC, SV)                                                                \
  do {                                                                                      \
    if (lds > 48 * 1024)                                                                    \
      (void)hipFuncSetAttribute(                                                            \
          reinterpret_cast<const void*>(&latent_attn_mfma_kernel<NK, NC, 4, SV>),           \
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                            \
    hipLaunchKernelGGL((latent_attn_mfma_kernel<NK, NC, 4, SV>), grid, dim3(256), lds, st, a); \
  } while (0)
  if (decode) {
    if (nk <= 6 && nc <= 8) LAT_MFMA(6, 8, true);
    else if (nk <= 12 && nc <= 16) LAT_MFMA(12, 16, true);
    else LAT_MFMA(20, 32, true);
  } else {
    if (nk <= 6 && nc <= 8) LAT_MFMA(6, 8, false);
    else if (nk <= 12 && nc <= 16) LAT_MFMA(12, 16, false);
    else LAT_MFMA(20, 32, false);
  }
#undef LAT_MFMA
  if (nparts > 1)
    hipLaunchKernelGGL(latent_merge_kernel, dim3(n_items, H), dim3(128), 0, st, part_acc, part_ml,
                       nparts, seq_lens, positions, window, static_cast<const bf16_t*>(gate),
                       gate_st, sink, static_cast<bf16_t*>(out), out_st, out_sh, H, R);
  EIA_LAUNCH_CHECK();
}
