// Paged attention with head-mixed ("talking") scores, aligned-chunk and
// trailing-window visibility, and an optional denominator sink.
//
// One launch covers a ragged batch: every token carries (its sequence's
// block-table row, its position); keys and values come from the paged
// cache, which already holds the token's own key. Because the score mix
//     s'_h = sum_g talk[h, g] * s_g
// couples all heads of one (query, key) pair before the softmax, a
// workgroup owns one query token with ALL its heads: per key tile it
// computes the raw scores of every head, mixes them, runs an online
// softmax per mixed head (the sink enters as an initial maximum of 0 with
// denominator 1 and no value) and accumulates P.V per head. Scores,
// weights and accumulators are fp32 in LDS.
#include "mix_common.h"

#define TA_KT 32

template <typename T>
__global__ __launch_bounds__(256) void talk_attn_kernel(
    T* __restrict__ out, int ldout, const T* __restrict__ q, int ldq,
    const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ block_tables, int max_blocks,
    const int* __restrict__ token_seq, const int* __restrict__ token_pos,
    const float* __restrict__ talk, int H, int G, int D, int DV, int BS,
    float scale, int chunk, int window, int sink) {
  extern __shared__ float lds[];
  float* sq = lds;                 // [H*D]
  float* ss = sq + H * D;          // [H][KT] raw scores
  float* sp = ss + H * TA_KT;      // [H][KT] mixed scores -> weights
  float* sacc = sp + H * TA_KT;    // [H*DV]
  float* sm = sacc + H * DV;       // [H] running max
  float* sl = sm + H;              // [H] running denominator
  float* sal = sl + H;             // [H] rescale of this tile
  float* stk = sal + H;            // [H*H]

  const int t = blockIdx.x;
  const int pos = token_pos[t];
  const int* table = block_tables + (size_t)token_seq[t] * max_blocks;
  int lo = 0;
  if (chunk > 0) lo = (pos / chunk) * chunk;
  if (window > 0) lo = max(lo, pos - window + 1);
  const int rep = H / G;

  for (int c = threadIdx.x; c < H * D; c += blockDim.x)
    sq[c] = MxElem<T>::ld(q + (size_t)t * ldq + c);
  for (int c = threadIdx.x; c < H * DV; c += blockDim.x) sacc[c] = 0.f;
  if (talk != nullptr)
    for (int c = threadIdx.x; c < H * H; c += blockDim.x) stk[c] = talk[c];
  for (int h = threadIdx.x; h < H; h += blockDim.x) {
    sm[h] = sink ? 0.f : PS_NEG_INF;
    sl[h] = sink ? 1.f : 0.f;
  }
  __syncthreads();

  for (int j0 = lo; j0 <= pos; j0 += TA_KT) {
    const int nk = min(TA_KT, pos + 1 - j0);
    // raw scores of every (head, key) pair of the tile
    for (int it = threadIdx.x; it < H * nk; it += blockDim.x) {
      const int jj = it / H, h = it % H;
      const int j = j0 + jj;
      const int64_t blk = table[j / BS];
      const T* kr = kc + ((blk * G + h / rep) * BS + (j % BS)) * (int64_t)D;
      const float* qh = sq + h * D;
      float acc = 0.f;
      for (int d = 0; d < D; ++d) acc += qh[d] * MxElem<T>::ld(kr + d);
      ss[h * TA_KT + jj] = acc * scale;
    }
    __syncthreads();
    // mix across heads
    for (int it = threadIdx.x; it < H * nk; it += blockDim.x) {
      const int jj = it / H, h = it % H;
      float m;
      if (talk != nullptr) {
        m = 0.f;
        for (int g2 = 0; g2 < H; ++g2)
          m += stk[h * H + g2] * ss[g2 * TA_KT + jj];
      } else {
        m = ss[h * TA_KT + jj];
      }
      sp[h * TA_KT + jj] = m;
    }
    __syncthreads();
    // online softmax bookkeeping: one thread per head
    for (int h = threadIdx.x; h < H; h += blockDim.x) {
      float mx = sm[h];
      for (int jj = 0; jj < nk; ++jj) mx = fmaxf(mx, sp[h * TA_KT + jj]);
      const float alpha = expf(sm[h] - mx);
      float l = sl[h] * alpha;
      for (int jj = 0; jj < nk; ++jj) {
        const float p = expf(sp[h * TA_KT + jj] - mx);
        sp[h * TA_KT + jj] = p;
        l += p;
      }
      sm[h] = mx;
      sl[h] = l;
      sal[h] = alpha;
    }
    __syncthreads();
    // P.V
    for (int it = threadIdx.x; it < H * DV; it += blockDim.x) {
      const int h = it / DV, d = it % DV;
      const int gk = h / rep;
      float acc = sacc[it] * sal[h];
      for (int jj = 0; jj < nk; ++jj) {
        const int j = j0 + jj;
        const int64_t blk = table[j / BS];
        acc += sp[h * TA_KT + jj] *
               MxElem<T>::ld(vc + ((blk * G + gk) * BS + (j % BS)) *
                                      (int64_t)DV + d);
      }
      sacc[it] = acc;
    }
    __syncthreads();
  }
  for (int it = threadIdx.x; it < H * DV; it += blockDim.x)
    MxElem<T>::st(out + (size_t)t * ldout + it, sacc[it] / sl[it / DV]);
}

extern "C" int mx_talk_attention(void* out, int ldout, const void* q,
                                 int ldq, const void* kc, const void* vc,
                                 const void* block_tables, int max_blocks,
                                 const void* token_seq,
                                 const void* token_pos, const void* talk,
                                 int T_, int H, int G, int D, int DV, int BS,
                                 float scale, int chunk, int window,
                                 int sink, int dtype, void* stream) {
  if (T_ <= 0) return 0;
  const size_t lds =
      (size_t)(H * D + 2 * H * TA_KT + H * DV + 3 * H + H * H) *
      sizeof(float);
  if (lds > 64 * 1024) return 1;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((talk_attn_kernel<T>), dim3(T_), dim3(256), lds,
                       (hipStream_t)stream, (T*)out, ldout, (const T*)q, ldq,
                       (const T*)kc, (const T*)vc, (const int*)block_tables,
                       max_blocks, (const int*)token_seq,
                       (const int*)token_pos, (const float*)talk, H, G, D, DV,
                       BS, scale, chunk, window, sink);
  })
  return 0;
}
