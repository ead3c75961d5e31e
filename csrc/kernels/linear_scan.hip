// Linear-attention recurrences with ONE decay number per head and token on per-sequence state
// slots: a matrix state S [dk, dv] per head that every token scales and adds an outer product to,
//
//   S_t = a_t S_(t-1) + b_t k_t v_t^T,      o_t = S_t^T q_t        (the token sees itself)
//
// mode 0 (fixed decay, "retention"):  a_t = decay[h], b_t = 1.
// mode 1 (exponential gates with a running maximum, "matrix memory"): per head two gate
//   pre-activations x_i, x_f ride in the token's row;
//     i = cap tanh(x_i / cap),  f = logsigmoid(cap tanh(x_f / cap))   (cap 0: no cap),
//     m_t = max(f + m_(t-1), i),
//     a_t = exp(f + m_(t-1) - m_t),  b_t = exp(i - m_t),  n_t = a_t n_(t-1) + b_t k_t,
//     o_t <- o_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6);       m starts at 0, S and n at zero.
// Both: q and k may be rotated by the token's position on their first rot_dims entries (pairs
// (i, i + rot_dims/2) or (2i, 2i+1)), then scaled (qscale, kscale); each head's o is divided by
// its root mean square, multiplied by an optional weight and by silu or sigmoid of the gate
// columns, and by out_scale.
//
// q, k, v, the gate and the gate pre-activations are column ranges of one fused projection row
// per token (type T: bf16 or float).  Decays, gates, exponentials, the state, the normaliser and
// the head norm are fp32.  A sequence whose first row of the step is position 0 starts from the
// initial state whatever its slot held, so slots are reused without clearing.
// Batch layout: sequence s owns rows [cu[s], cu[s+1]) (cu == nullptr: row s).
#include "eia_common.h"

struct ScanArgs {
  const void* x; long ld;                   // fused rows [rows, *]
  int q_off, k_off, v_off, g_off, i_off, f_off;
  const float* decay;                       // [H] (mode 0)
  const float* inv_freq; int rot_dims, rot_half;
  float qscale, kscale, cap, out_scale;
  const void* norm_w;                       // [H * Dv] or null
  float* S; float* N; float* M;             // [slots, H, D, Dv], [slots, H, D], [slots, H]
  const int* slots; const int* cu; const int* positions; const int* seq_lens;
  void* y; long ldy;                        // [rows, >= H * Dv]
  float eps;
  int H, D, Dv, mode, gate_act;
};

EIA_DEV float ls_logsigmoid(float z) { return -(log1pf(expf(-fabsf(z))) + fmaxf(-z, 0.f)); }

// One workgroup per (sequence, head), 4 x max(64, DMAX) threads: thread (qt, j) owns rows
// [qt DMAX/4, (qt+1) DMAX/4) of column j of S in registers and walks the sequence's tokens in
// order.  Tokens are staged TC at a time: q, k (rotated, scaled), v and the gate of TC tokens go
// to LDS, the gate recurrence of the chunk runs (its transcendentals in parallel over the
// tokens, the running maximum serially in one thread), then the state recurrence runs TC steps on
// LDS broadcasts leaving four partial outputs per token and column, which are summed, divided,
// normed and gated.  NRM: the normaliser n rides along (every thread of a quarter keeps the
// quarter's rows of n; column 0 reports n . q).
template <typename T, int DMAX, bool NRM>
__global__ void __launch_bounds__(4 * (DMAX < 64 ? 64 : DMAX))
linear_scan_kernel(ScanArgs a) {
  constexpr int DP = DMAX < 64 ? 64 : DMAX;          // threads per quarter
  constexpr int DQ = DMAX / 4;                       // dk rows per thread
  constexpr int TC = DMAX <= 64 ? 16 : DMAX <= 128 ? 8 : 4;
  constexpr int NWV = DP / 64;
  __shared__ __align__(16) float sq[TC][DMAX], sk[TC][DMAX];
  __shared__ float sv[TC][DMAX], sg[TC][DMAX], po[TC][4][DP];
  __shared__ float sa[TC], sb[TC], se[TC], gi[TC], gf[TC], pn[TC][4];
  __shared__ float red[4][NWV];
  __shared__ float m_run;
  const int s = blockIdx.x, h = blockIdx.y, D = a.D, Dv = a.Dv;
  const int qt = threadIdx.x / DP, j = threadIdx.x % DP;
  const int slot = a.slots[s];
  if (slot < 0 || (a.seq_lens && a.seq_lens[s] <= 0)) return;
  const int lo = a.cu ? a.cu[s] : s, hi = a.cu ? a.cu[s + 1] : s + 1;
  if (hi <= lo) return;
  const bool fresh = a.positions[lo] == 0;
  const bool col = j < Dv;                           // this thread owns a state column
  const bool chan = j < D;                           // ... and stages a q / k channel
  float* Sg = a.S + ((long)slot * a.H + h) * D * Dv;
  float* Ng = NRM ? a.N + ((long)slot * a.H + h) * D : nullptr;
  const int i0 = qt * DQ;
  float S[DQ], Nn[NRM ? DQ : 1];
#pragma unroll
  for (int i = 0; i < DQ; ++i) {
    S[i] = (!fresh && i0 + i < D && col) ? Sg[(long)(i0 + i) * Dv + j] : 0.f;
    if constexpr (NRM) Nn[i] = (!fresh && i0 + i < D) ? Ng[i0 + i] : 0.f;
  }
  if (threadIdx.x == 0) m_run = (NRM && !fresh) ? a.M[(long)slot * a.H + h] : 0.f;
  const float dec = a.mode == 0 ? a.decay[h] : 1.f;
  const T* X = static_cast<const T*>(a.x);
  const T* NW = static_cast<const T*>(a.norm_w);
  T* Y = static_cast<T*>(a.y);
  const float nw = (NW && col) ? ld_f32<T>(NW, (long)h * Dv + j) : 1.f;
  const float inv_dv = 1.0f / (float)Dv;
  // rotation of channel j: partner channel, the pair's frequency and the sign of the cross term
  const int hd = a.rot_dims >> 1;
  const bool rot = chan && j < a.rot_dims;
  int jp = j;
  float freq = 0.f, sgn = 0.f;
  if (rot) {
    const bool second = a.rot_half ? j >= hd : (j & 1);
    const int pi = a.rot_half ? (second ? j - hd : j) : (j >> 1);
    jp = a.rot_half ? (second ? j - hd : j + hd) : (j ^ 1);
    freq = a.inv_freq[pi];
    sgn = second ? 1.f : -1.f;
  }
  const long qc = a.q_off + (long)h * D, kc = a.k_off + (long)h * D;
  const long vc = a.v_off + (long)h * Dv, gc = a.g_off + (long)h * Dv;
  for (int base = lo; base < hi; base += TC) {
    const int nt = min(TC, hi - base);
    __syncthreads();                       // the previous chunk's LDS reads are done
    if (j < DMAX) {
#pragma unroll
      for (int tt = 0; tt < TC / 4; ++tt) {            // quarter qt stages tokens qt, qt + 4, ...
        const int t = tt * 4 + qt;
        if (t < nt) {
          const T* xr = X + (long)(base + t) * a.ld;
          float q = 0.f, k = 0.f, v = 0.f, g = 0.f;
          if (chan) {
            q = ld_f32<T>(xr, qc + j);
            k = ld_f32<T>(xr, kc + j);
            if (rot) {
              float sn, cs;
              sincosf((float)a.positions[base + t] * freq, &sn, &cs);
              q = q * cs + sgn * ld_f32<T>(xr, qc + jp) * sn;
              k = k * cs + sgn * ld_f32<T>(xr, kc + jp) * sn;
            }
            q *= a.qscale;
            k *= a.kscale;
          }
          if (col) {
            v = ld_f32<T>(xr, vc + j);
            g = ld_f32<T>(xr, gc + j);
          }
          sq[t][j] = q;
          sk[t][j] = k;
          sv[t][j] = v;
          sg[t][j] = g;
        }
      }
    }
    if constexpr (NRM) {
      if (threadIdx.x < nt) {                          // log gates of the chunk's tokens
        const T* xr = X + (long)(base + threadIdx.x) * a.ld;
        const float xi = ld_f32<T>(xr, a.i_off + h), xf = ld_f32<T>(xr, a.f_off + h);
        gi[threadIdx.x] = a.cap > 0.f ? a.cap * tanhf(xi / a.cap) : xi;
        gf[threadIdx.x] = ls_logsigmoid(a.cap > 0.f ? a.cap * tanhf(xf / a.cap) : xf);
      }
      __syncthreads();
      if (threadIdx.x == 0) {                          // the running maximum, token by token
        float m = m_run;
        for (int t = 0; t < nt; ++t) {
          const float fm = gf[t] + m;
          m = fmaxf(fm, gi[t]);
          sa[t] = fm;                                  // f + m_(t-1)
          se[t] = m;
        }
        m_run = m;
      }
      __syncthreads();
      if (threadIdx.x < nt) {
        const float m = se[threadIdx.x];
        sa[threadIdx.x] = expf(sa[threadIdx.x] - m);
        sb[threadIdx.x] = expf(gi[threadIdx.x] - m);
        se[threadIdx.x] = expf(-m);
      }
    }
    __syncthreads();
    for (int t = 0; t < nt; ++t) {
      const float v = sv[t][j < DMAX ? j : 0];
      const float at = NRM ? sa[t] : dec, bt = NRM ? sb[t] : 1.f;
      float o = 0.f, nq = 0.f;
#pragma unroll
      for (int i = 0; i < DQ; ++i) {
        const float bk = bt * sk[t][i0 + i];
        S[i] = at * S[i] + bk * v;
        o += sq[t][i0 + i] * S[i];
        if constexpr (NRM) {
          Nn[i] = at * Nn[i] + bk;
          nq += sq[t][i0 + i] * Nn[i];
        }
      }
      po[t][qt][j] = o;
      if (NRM && j == 0) pn[t][qt] = nq;
    }
    __syncthreads();
    // quarter qt finishes tokens qt, qt + 4, ...: sum of the partials, normaliser, head RMS norm,
    // weight, gate
#pragma unroll
    for (int tt = 0; tt < TC / 4; ++tt) {
      const int t = tt * 4 + qt;
      const bool ok = t < nt && col;
      float o = ok ? po[t][0][j] + po[t][1][j] + po[t][2][j] + po[t][3][j] : 0.f;
      if constexpr (NRM) {
        if (t < nt) {
          const float nq = pn[t][0] + pn[t][1] + pn[t][2] + pn[t][3];
          o = o / (fmaxf(fabsf(nq), se[t]) + 1e-6f);
        }
      }
      float ss = wave_sum(o * o);
      if (NWV > 1) {
        __syncthreads();
        if ((j & 63) == 0) red[qt][j >> 6] = ss;
        __syncthreads();
        ss = 0.f;
#pragma unroll
        for (int x = 0; x < NWV; ++x) ss += red[qt][x];
      }
      if (ok) {
        const float g = sg[t][j];
        const float sig = 1.0f / (1.0f + expf(-g));
        const float gate = a.gate_act == 0 ? g * sig : sig;
        st_f32<T>(Y, (long)(base + t) * a.ldy + (long)h * Dv + j,
                  o / sqrtf(ss * inv_dv + a.eps) * nw * gate * a.out_scale);
      }
    }
  }
  if (col) {
#pragma unroll
    for (int i = 0; i < DQ; ++i)
      if (i0 + i < D) Sg[(long)(i0 + i) * Dv + j] = S[i];
  }
  if constexpr (NRM) {
    if (j == 0) {
#pragma unroll
      for (int i = 0; i < DQ; ++i)
        if (i0 + i < D) Ng[i0 + i] = Nn[i];
    }
    __syncthreads();
    if (threadIdx.x == 0) a.M[(long)slot * a.H + h] = m_run;
  }
}

// x: fused rows (bf16 when is_bf16, else fp32) holding the q [H*D], k [H*D], v [H*Dv] and gate
// [H*Dv] columns at the given offsets (mode 1: also the H input-gate and H forget-gate
// pre-activations at i_off / f_off); y [rows, >= H*Dv] of the same type.
EIA_API int eia_linear_scan(const void* x, long ld, int q_off, int k_off, int v_off, int g_off,
                            int i_off, int f_off, const float* decay, const float* inv_freq,
                            int rot_dims, int rot_half, float qscale, float kscale, float cap,
                            float out_scale, const void* norm_w, float* S, float* N, float* M,
                            const int* slots, const int* cu, const int* positions,
                            const int* seq_lens, void* y, long ldy, float eps, int nseq, int H,
                            int D, int Dv, int mode, int gate_act, int is_bf16, hipStream_t st) {
  if (nseq < 0 || H < 1 || D < 1 || Dv < 1 || !x || !y || !S || !slots || !positions ||
      (mode != 0 && mode != 1) || (mode == 0 && !decay) || (mode == 1 && (!N || !M || cap < 0.f)) ||
      rot_dims < 0 || rot_dims > D || (rot_dims & 1) || (rot_dims && !inv_freq) ||
      (gate_act != 0 && gate_act != 1))
    return EIA_BAD_SHAPE;
  const int dm = D > Dv ? D : Dv;
  if (dm > 256) return EIA_UNSUPPORTED;
  if (nseq == 0) return EIA_OK;
  ScanArgs a{x, ld, q_off, k_off, v_off, g_off, i_off, f_off, decay, inv_freq, rot_dims, rot_half,
             qscale, kscale, cap, out_scale, norm_w, S, N, M, slots, cu, positions, seq_lens, y,
             ldy, eps, H, D, Dv, mode, gate_act};
  dim3 grid(nseq, H);
#define LS_LAUNCH(TT, DM, NR)                                                                  \
  hipLaunchKernelGGL((linear_scan_kernel<TT, DM, NR>), grid, dim3(4 * (DM < 64 ? 64 : DM)), 0, \
                     st, a)
#define LS_SIZES(TT, NR)                      \
  do {                                        \
    if (dm <= 32) LS_LAUNCH(TT, 32, NR);      \
    else if (dm <= 64) LS_LAUNCH(TT, 64, NR); \
    else if (dm <= 128) LS_LAUNCH(TT, 128, NR); \
    else LS_LAUNCH(TT, 256, NR);              \
  } while (0)
  if (is_bf16) {
    if (mode == 1) LS_SIZES(bf16_t, true); else LS_SIZES(bf16_t, false);
  } else {
    if (mode == 1) LS_SIZES(float, true); else LS_SIZES(float, false);
  }
#undef LS_SIZES
#undef LS_LAUNCH
  EIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------
// Chunk-parallel form for prompt portions (dk, dv <= 128).  The token-by-token kernel above walks
// a sequence with one workgroup per head; here a step's rows are cut into chunks of LC tokens
// (never across sequences) and, with A_t the running sum of log a inside a chunk,
//
//   U_c   = sum_s exp(A_end - A_s) b_s k_s v_s^T            (1) per chunk, in parallel
//   S_c+1 = exp(A_end) S_c + U_c                            (2) a short scan over a sequence's chunks
//   o_t   = exp(A_t) S_c^T q_t + sum_(s<=t) exp(A_t - A_s) b_s (q_t . k_s) v_s     (3) per chunk
//
// (the normaliser n likewise; n_t . q_t is the row sum of the same weights).  Every exponent is
// <= 0.  The log gates of the gated mode come from a pre-pass that carries the running maximum
// through the sequence.  All of it fp32 FMA: the 32-bit mode needs it, and the work is small
// beside the projections.
constexpr int LC = 32;                      // tokens per chunk
constexpr int LD = 128;                     // largest dk / dv of this form
constexpr int LP = LD + 4;                  // LDS row pitch: 16-byte rows that rotate the banks

struct ChunkArgs {
  const int* chunks;                        // [nchunk, 4]: sequence, first row, tokens, unused
  const int* seq_first;                     // [nseq + 1]: first chunk of every sequence
  float* wsS; float* wsN; float* wsG;       // [nchunk, H, D, Dv], [nchunk, H, D], [nchunk, H]
  float* la; float* lb; float* nm;          // [rows, H] log a, log b, -m  (mode 1)
};

// (A) log gates of the gated mode: one workgroup per (sequence, head); the transcendentals of 256
// tokens in parallel, the running maximum serially in one thread.
template <typename T>
__global__ void __launch_bounds__(256)
ls_gates_kernel(ScanArgs a, ChunkArgs c) {
  __shared__ float gi[256], gf[256], o1[256], o2[256], o3[256];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int slot = a.slots[s];
  if (slot < 0) return;
  const int lo = a.cu ? a.cu[s] : s, hi = a.cu ? a.cu[s + 1] : s + 1;
  if (hi <= lo) return;
  float m = a.positions[lo] == 0 ? 0.f : a.M[(long)slot * a.H + h];
  const T* X = static_cast<const T*>(a.x);
  for (int base = lo; base < hi; base += 256) {
    const int n = min(256, hi - base);
    if (tid < n) {
      const T* xr = X + (long)(base + tid) * a.ld;
      const float xi = ld_f32<T>(xr, a.i_off + h), xf = ld_f32<T>(xr, a.f_off + h);
      gi[tid] = a.cap > 0.f ? a.cap * tanhf(xi / a.cap) : xi;
      gf[tid] = ls_logsigmoid(a.cap > 0.f ? a.cap * tanhf(xf / a.cap) : xf);
    }
    __syncthreads();
    if (tid == 0) {
      for (int t = 0; t < n; ++t) {
        const float fm = gf[t] + m;
        const float mn = fmaxf(fm, gi[t]);
        o1[t] = fm - mn;
        o2[t] = gi[t] - mn;
        o3[t] = -mn;
        m = mn;
      }
    }
    __syncthreads();
    if (tid < n) {
      const long o = (long)(base + tid) * a.H + h;
      c.la[o] = o1[tid];
      c.lb[o] = o2[tid];
      c.nm[o] = o3[tid];
    }
    __syncthreads();
  }
  if (tid == 0) a.M[(long)slot * a.H + h] = m;
}

// Stages rotated, scaled q or k rows ([LC][LD], zero beyond n tokens / D channels).
template <typename T>
EIA_DEV void ls_stage_rot(const ScanArgs& a, const T* X, int row0, int n, long off, float scale,
                          float (*dst)[LP]) {
  const int hd = a.rot_dims >> 1;
  for (int idx = threadIdx.x; idx < LC * LD; idx += blockDim.x) {
    const int t = idx / LD, j = idx % LD;
    float v = 0.f;
    if (t < n && j < a.D) {
      const T* xr = X + (long)(row0 + t) * a.ld;
      v = ld_f32<T>(xr, off + j);
      if (j < a.rot_dims) {
        const bool second = a.rot_half ? j >= hd : (j & 1);
        const int pi = a.rot_half ? (second ? j - hd : j) : (j >> 1);
        const int jp = a.rot_half ? (second ? j - hd : j + hd) : (j ^ 1);
        float sn, cs;
        sincosf((float)a.positions[row0 + t] * a.inv_freq[pi], &sn, &cs);
        v = v * cs + (second ? 1.f : -1.f) * ld_f32<T>(xr, off + jp) * sn;
      }
      v *= scale;
    }
    dst[t][j] = v;
  }
}

// Running sums of log a inside the chunk (sA) and log b (sB) into LDS, by the first wave.
EIA_DEV void ls_chunk_decay(const ScanArgs& a, const ChunkArgs& c, int row0, int n, int h,
                            float* sA, float* sB) {
  if (threadIdx.x < 64) {
    const int t = threadIdx.x;
    float la = 0.f, lb = 0.f;
    if (t < n) {
      if (a.mode == 0) {
        la = logf(a.decay[h]);
      } else {
        la = c.la[(long)(row0 + t) * a.H + h];
        lb = c.lb[(long)(row0 + t) * a.H + h];
      }
    }
#pragma unroll
    for (int o = 1; o < LC; o <<= 1) {                 // inclusive prefix sum over the lanes
      const float up = __shfl_up(la, o, 64);
      if (t >= o) la += up;
    }
    if (t < LC) { sA[t] = la; sB[t] = lb; }
  }
}

// (1) a chunk's own contribution to the state: U = sum_s w_s k_s v_s^T, u_n = sum_s w_s k_s,
// w_s = exp(A_end - A_s + log b_s), and the chunk's total log decay.  Thread (r, j): rows
// [64 r, 64 r + 64) of column j.
template <typename T>
__global__ void __launch_bounds__(256)
ls_chunk_state_kernel(ScanArgs a, ChunkArgs c) {
  __shared__ __align__(16) float sk[LC][LP], sv[LC][LD];
  __shared__ float sA[LC], sB[LC];
  const int ch = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int s = c.chunks[4 * ch], row0 = c.chunks[4 * ch + 1], n = c.chunks[4 * ch + 2];
  if (a.slots[s] < 0) return;
  const int D = a.D, Dv = a.Dv;
  const T* X = static_cast<const T*>(a.x);
  ls_stage_rot<T>(a, X, row0, n, a.k_off + (long)h * D, a.kscale, sk);
  for (int idx = tid; idx < LC * LD; idx += 256) {
    const int t = idx / LD, j = idx % LD;
    sv[t][j] = (t < n && j < Dv) ? ld_f32<T>(X + (long)(row0 + t) * a.ld, a.v_off + (long)h * Dv + j)
                                 : 0.f;
  }
  ls_chunk_decay(a, c, row0, n, h, sA, sB);
  __syncthreads();
  const float Aend = sA[n - 1];
  for (int idx = tid; idx < LC * LD; idx += 256) {     // k_s <- w_s k_s
    const int t = idx / LD, j = idx % LD;
    if (t < n) sk[t][j] *= expf(Aend - sA[t] + sB[t]);
  }
  __syncthreads();
  const int r = tid >> 7, j = tid & 127;
  float acc[64];
#pragma unroll
  for (int i = 0; i < 64; ++i) acc[i] = 0.f;
  for (int t = 0; t < n; ++t) {
    const float v = sv[t][j];
#pragma unroll
    for (int i = 0; i < 64; ++i) acc[i] += sk[t][64 * r + i] * v;
  }
  float* U = c.wsS + ((long)ch * a.H + h) * D * Dv;
  if (j < Dv) {
#pragma unroll
    for (int i = 0; i < 64; ++i)
      if (64 * r + i < D) U[(long)(64 * r + i) * Dv + j] = acc[i];
  }
  if (a.mode == 1 && tid < D) {
    float un = 0.f;
    for (int t = 0; t < n; ++t) un += sk[t][tid];
    c.wsN[((long)ch * a.H + h) * D + tid] = un;
  }
  if (tid == 0) c.wsG[(long)ch * a.H + h] = Aend;
}

// (2) the scan over a sequence's chunks, element by element: the workspace entry of a chunk turns
// from its own contribution into the state BEFORE the chunk; the slot receives the final state.
__global__ void __launch_bounds__(256)
ls_chunk_scan_kernel(ScanArgs a, ChunkArgs c) {
  const int s = blockIdx.x, h = blockIdx.y;
  const int slot = a.slots[s];
  if (slot < 0) return;
  const int c0 = c.seq_first[s], c1 = c.seq_first[s + 1];
  if (c1 <= c0) return;
  const int lo = a.cu ? a.cu[s] : s;
  const bool fresh = a.positions[lo] == 0;
  const long n_el = (long)a.D * a.Dv;
  const long e = (long)blockIdx.z * 256 + threadIdx.x;
  if (e < n_el) {
    float* Sg = a.S + ((long)slot * a.H + h) * n_el;
    float S = fresh ? 0.f : Sg[e];
    for (int ch = c0; ch < c1; ++ch) {
      float* w = c.wsS + ((long)ch * a.H + h) * n_el + e;
      const float U = *w;
      *w = S;
      S = expf(c.wsG[(long)ch * a.H + h]) * S + U;
    }
    Sg[e] = S;
  }
  if (a.mode == 1 && blockIdx.z == 0 && threadIdx.x < a.D) {
    float* Ng = a.N + ((long)slot * a.H + h) * a.D;
    float nn = fresh ? 0.f : Ng[threadIdx.x];
    for (int ch = c0; ch < c1; ++ch) {
      float* w = c.wsN + ((long)ch * a.H + h) * a.D + threadIdx.x;
      const float U = *w;
      *w = nn;
      nn = expf(c.wsG[(long)ch * a.H + h]) * nn + U;
    }
    Ng[threadIdx.x] = nn;
  }
}

// (3) a chunk's outputs from the state before it and its own tokens.  Thread (r, j): tokens
// r, r + 2, ... of column j.
template <typename T>
__global__ void __launch_bounds__(256)
ls_chunk_out_kernel(ScanArgs a, ChunkArgs c) {
  __shared__ __align__(16) float sq[LC][LP], sk[LC][LP], sv[LC][LD];
  __shared__ float P[LC][LC + 1];
  __shared__ float sA[LC], sB[LC], snq[LC], red[LC][2];
  const int ch = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int s = c.chunks[4 * ch], row0 = c.chunks[4 * ch + 1], n = c.chunks[4 * ch + 2];
  if (a.slots[s] < 0) return;
  const int D = a.D, Dv = a.Dv;
  const T* X = static_cast<const T*>(a.x);
  ls_stage_rot<T>(a, X, row0, n, a.q_off + (long)h * D, a.qscale, sq);
  ls_stage_rot<T>(a, X, row0, n, a.k_off + (long)h * D, a.kscale, sk);
  for (int idx = tid; idx < LC * LD; idx += 256) {
    const int t = idx / LD, j = idx % LD;
    sv[t][j] = (t < n && j < Dv) ? ld_f32<T>(X + (long)(row0 + t) * a.ld, a.v_off + (long)h * Dv + j)
                                 : 0.f;
  }
  ls_chunk_decay(a, c, row0, n, h, sA, sB);
  __syncthreads();
  // weights of the chunk's own pairs: P[t][u] = (q_t . k_u) exp(A_t - A_u + log b_u), u <= t
  for (int idx = tid; idx < LC * LC; idx += 256) {
    const int t = idx / LC, u = idx % LC;
    float p = 0.f;
    if (u <= t && t < n) {
      const f32x4* qa = reinterpret_cast<const f32x4*>(sq[t]);
      const f32x4* ka = reinterpret_cast<const f32x4*>(sk[u]);
#pragma unroll 8
      for (int i = 0; i < LD / 4; ++i) {
        const f32x4 x = qa[i], y = ka[i];
        p += x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
      }
      p *= expf(sA[t] - sA[u] + sB[u]);
    }
    P[t][u] = p;
  }
  // n_before . q_t of the gated mode
  if (a.mode == 1 && tid < n) {
    const float* nb = c.wsN + ((long)ch * a.H + h) * D;
    float d = 0.f;
    for (int i = 0; i < D; ++i) d += nb[i] * sq[tid][i];
    snq[tid] = d;
  }
  __syncthreads();
  const int r = tid >> 7, j = tid & 127;
  const float* Sb = c.wsS + ((long)ch * a.H + h) * D * Dv;      // the state before the chunk
  float own[LC / 2], carry[LC / 2];
#pragma unroll
  for (int tt = 0; tt < LC / 2; ++tt) { own[tt] = 0.f; carry[tt] = 0.f; }
  if (j < Dv) {
    for (int i = 0; i < D; ++i) {
      const float sv_ = Sb[(long)i * Dv + j];
#pragma unroll
      for (int tt = 0; tt < LC / 2; ++tt) carry[tt] += sq[2 * tt + r][i] * sv_;
    }
    for (int u = 0; u < n; ++u) {
      const float v = sv[u][j];
#pragma unroll
      for (int tt = 0; tt < LC / 2; ++tt) own[tt] += P[2 * tt + r][u] * v;
    }
  }
  const T* NW = static_cast<const T*>(a.norm_w);
  const float nw = (NW && j < Dv) ? ld_f32<T>(NW, (long)h * Dv + j) : 1.f;
  T* Y = static_cast<T*>(a.y);
  const float inv_dv = 1.0f / (float)Dv;
#pragma unroll
  for (int tt = 0; tt < LC / 2; ++tt) {
    const int t = 2 * tt + r;
    const float eA = expf(sA[t < n ? t : 0]);
    float o = (j < Dv && t < n) ? own[tt] + eA * carry[tt] : 0.f;
    if (a.mode == 1 && t < n) {
      float nq = eA * snq[t];
      for (int u = 0; u <= t; ++u) nq += P[t][u];
      o = o / (fmaxf(fabsf(nq), expf(c.nm[(long)(row0 + t) * a.H + h])) + 1e-6f);
    }
    const float ss = wave_sum(o * o);
    if ((tid & 63) == 0) red[t][(tid >> 6) & 1] = ss;
    own[tt] = o;
  }
  __syncthreads();
#pragma unroll
  for (int tt = 0; tt < LC / 2; ++tt) {
    const int t = 2 * tt + r;
    if (t < n && j < Dv) {
      const float g = ld_f32<T>(X + (long)(row0 + t) * a.ld, a.g_off + (long)h * Dv + j);
      const float sig = 1.0f / (1.0f + expf(-g));
      const float gate = a.gate_act == 0 ? g * sig : sig;
      st_f32<T>(Y, (long)(row0 + t) * a.ldy + (long)h * Dv + j,
                own[tt] / sqrtf((red[t][0] + red[t][1]) * inv_dv + a.eps) * nw * gate * a.out_scale);
    }
  }
}

// The same arguments as eia_linear_scan plus the step's chunk list (chunks int32 [nchunk, 4]:
// sequence, first row, tokens (1 .. 32), 0; seq_first int32 [nseq + 1]) and fp32 workspaces
// wsS [nchunk, H, D, Dv], wsN [nchunk, H, D], wsG [nchunk, H], la / lb / nm [rows, H].
EIA_API int eia_linear_scan_chunked(const void* x, long ld, int q_off, int k_off, int v_off,
                                    int g_off, int i_off, int f_off, const float* decay,
                                    const float* inv_freq, int rot_dims, int rot_half,
                                    float qscale, float kscale, float cap, float out_scale,
                                    const void* norm_w, float* S, float* N, float* M,
                                    const int* slots, const int* cu, const int* positions,
                                    void* y, long ldy, float eps, int nseq, int H, int D, int Dv,
                                    int mode, int gate_act, int is_bf16, const int* chunks,
                                    const int* seq_first, int nchunk, float* wsS, float* wsN,
                                    float* wsG, float* la, float* lb, float* nm, hipStream_t st) {
  if (nseq < 0 || nchunk < 0 || H < 1 || D < 1 || Dv < 1 || !x || !y || !S || !slots || !positions ||
      !chunks || !seq_first || !wsS || !wsG || (mode != 0 && mode != 1) || (mode == 0 && !decay) ||
      (mode == 1 && (!N || !M || cap < 0.f || !wsN || !la || !lb || !nm)) || rot_dims < 0 ||
      rot_dims > D || (rot_dims & 1) || (rot_dims && !inv_freq) ||
      (gate_act != 0 && gate_act != 1))
    return EIA_BAD_SHAPE;
  if (D > LD || Dv > LD) return EIA_UNSUPPORTED;
  if (nseq == 0 || nchunk == 0) return EIA_OK;
  ScanArgs a{x, ld, q_off, k_off, v_off, g_off, i_off, f_off, decay, inv_freq, rot_dims, rot_half,
             qscale, kscale, cap, out_scale, norm_w, S, N, M, slots, cu, positions, nullptr, y,
             ldy, eps, H, D, Dv, mode, gate_act};
  ChunkArgs c{chunks, seq_first, wsS, wsN, wsG, la, lb, nm};
  const dim3 gs(nseq, H), gc(nchunk, H), gz(nseq, H, (D * Dv + 255) / 256);
  if (is_bf16) {
    if (mode == 1) hipLaunchKernelGGL((ls_gates_kernel<bf16_t>), gs, dim3(256), 0, st, a, c);
    hipLaunchKernelGGL((ls_chunk_state_kernel<bf16_t>), gc, dim3(256), 0, st, a, c);
    hipLaunchKernelGGL(ls_chunk_scan_kernel, gz, dim3(256), 0, st, a, c);
    hipLaunchKernelGGL((ls_chunk_out_kernel<bf16_t>), gc, dim3(256), 0, st, a, c);
  } else {
    if (mode == 1) hipLaunchKernelGGL((ls_gates_kernel<float>), gs, dim3(256), 0, st, a, c);
    hipLaunchKernelGGL((ls_chunk_state_kernel<float>), gc, dim3(256), 0, st, a, c);
    hipLaunchKernelGGL(ls_chunk_scan_kernel, gz, dim3(256), 0, st, a, c);
    hipLaunchKernelGGL((ls_chunk_out_kernel<float>), gc, dim3(256), 0, st, a, c);
  }
  EIA_LAUNCH_CHECK();
}
