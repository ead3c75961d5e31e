// Token embedding with a hashed bigram term, written as the NS equal fp32 residual streams of a
// hyper-connected decoder:
//
//   x = embed[tok] * scale + bigram[(prev * mul_prev + tok * mul_cur) mod buckets]
//
// and row `buckets` of the bigram table for a sequence's first token.  The previous token of a
// step's first row lives in the sequence's state slot (last_tok [slots], int32); the workgroup of
// that row reads it and then stores the step's last token there, so no other workgroup touches
// the slot.  Batch layout: sequence s owns rows [cu[s], cu[s+1]) (cu == nullptr: row s);
// slots[s] < 0 is a padding row (no previous token, nothing stored).
#include "eia_common.h"

template <typename T>
__global__ void __launch_bounds__(256)
bigram_embed_kernel(const int* __restrict__ ids, const T* __restrict__ embed, float scale,
                    const T* __restrict__ bigram, int buckets, long mul_prev, long mul_cur,
                    int* __restrict__ last_tok, const int* __restrict__ slots,
                    const int* __restrict__ cu, int nseq, const int* __restrict__ positions,
                    float* __restrict__ X, int NS, int W, int vocab) {
  const int row = blockIdx.x;
  int s = row;
  if (cu) {                                  // largest s with cu[s] <= row
    int lo = 0, hi = nseq - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (cu[mid] <= row) lo = mid; else hi = mid - 1;
    }
    s = lo;
  }
  const int first = cu ? cu[s] : row, last = cu ? cu[s + 1] - 1 : row;
  const int slot = slots ? slots[s] : -1;
  int tok = ids[row];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  long prev = -1;
  if (row > first) prev = ids[row - 1];
  else if (positions[row] > 0 && slot >= 0 && last_tok) prev = last_tok[slot];
  __syncthreads();                           // every thread has read the slot
  if (row == first && slot >= 0 && last_tok && threadIdx.x == 0) last_tok[slot] = ids[last];
  const T* er = embed + (long)tok * W;
  const T* br = nullptr;
  if (bigram) {
    const long r = prev < 0 ? (long)buckets : (prev * mul_prev + (long)tok * mul_cur) % buckets;
    br = bigram + r * W;
  }
  float* xr = X + (long)row * NS * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = ld_f32<T>(er, c) * scale;
    if (br) v += ld_f32<T>(br, c);
    for (int j = 0; j < NS; ++j) xr[(long)j * W + c] = v;
  }
}

// ids int32 [rows]; embed [vocab, W] and bigram [buckets + 1, W] (nullable) bf16 when is_bf16
// else fp32; X fp32 [rows, NS, W].
EIA_API int eia_bigram_embed(const int* ids, const void* embed, float scale, const void* bigram,
                             int buckets, long mul_prev, long mul_cur, int* last_tok,
                             const int* slots, const int* cu, int nseq, const int* positions,
                             float* X, int NS, int W, int vocab, int rows, int is_bf16,
                             hipStream_t st) {
  if (rows < 0 || W < 1 || NS < 1 || vocab < 1 || !ids || !embed || !X || !positions ||
      (bigram && buckets < 1) || (cu && nseq < 1))
    return EIA_BAD_SHAPE;
  if (rows == 0) return EIA_OK;
  const int threads = W >= 1024 ? 256 : (W >= 512 ? 128 : 64);
  if (is_bf16)
    hipLaunchKernelGGL((bigram_embed_kernel<bf16_t>), dim3(rows), dim3(threads), 0, st, ids,
                       (const bf16_t*)embed, scale, (const bf16_t*)bigram, buckets, mul_prev,
                       mul_cur, last_tok, slots, cu, nseq, positions, X, NS, W, vocab);
  else
    hipLaunchKernelGGL((bigram_embed_kernel<float>), dim3(rows), dim3(threads), 0, st, ids,
                       (const float*)embed, scale, (const float*)bigram, buckets, mul_prev, mul_cur,
                       last_tok, slots, cu, nseq, positions, X, NS, W, vocab);
  EIA_LAUNCH_CHECK();
}
