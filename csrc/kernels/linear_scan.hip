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
