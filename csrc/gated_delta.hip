// Gated delta rule with one decay per head and key channel (prefill portions
// and single decode tokens in one launch).
//
// Per head the state S is a D x DV fp32 matrix (rows = key channels, columns
// = value channels). For every token, with q and k the head's (group's)
// convolved projections,
//     k^ = k / sqrt(sum k^2 + 1e-6),  q^ = q / sqrt(sum q^2 + 1e-6) * qscale
//     g  = exp(-exp(a_log) * softplus(zdec + dt_bias))     per key channel
//     b  = sigmoid(beta)                                   per head
//     S <- diag(g) S;  u = b (v - S^T k^);  S <- S + k^ u^T;  o = S^T q^
// and the head's o is divided by its root mean square over DV, scaled by a
// weight shared by the heads and by sigmoid(zgate).
//
// Since S^T k^ after the decay is (g * k^)^T S_old, one pass over a column
// does it all: sa = sum_i (g k^)_i S_i, then S_i <- g_i S_i + k^_i b (v - sa)
// and the read-out sum in the same sweep.
//
// Mapping: one workgroup per (sequence segment, head). Column j of S lives
// in the registers of P adjacent lanes, lane p holding rows p, p+P, ...
// (DKP / P rows, D padded up to DKP), so both sums are short thread-local
// dot products finished by a P-lane butterfly. Tokens go through in tiles:
// the per-row vectors (g k^, g, k^, q^) of a whole tile are prepared
// cooperatively into LDS (each lane's rows contiguous, segments padded
// against bank conflicts), then each thread walks the tile's tokens with
// broadcast LDS reads and no barrier.
#include "mix_common.h"

PS_DEV float mx_softplus(float z) {
  return z > 20.f ? z : log1pf(expf(z));
}

template <typename T, int DKP, int TILE, int P, int MAXT>
__global__ __launch_bounds__(MAXT) void gated_delta_kernel(
    T* __restrict__ out, int ldo, const T* __restrict__ q, int ldq,
    const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    const T* __restrict__ beta, int ldb, const T* __restrict__ zdec, int ldzd,
    const T* __restrict__ zgate, int ldzg, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, const float* __restrict__ normw,
    float* __restrict__ state, const int* __restrict__ seq_rows, int H, int G,
    int D, int DV, float eps, float qscale) {
  extern __shared__ __align__(16) float lds[];
  constexpr int R = DKP / P;        // rows per lane
  constexpr int RP = P > 1 ? R + 4 : R;
  constexpr int TP = RP * P;        // words per token and array
  float* sgk = lds;                 // [TILE][TP] decay * unit key
  float* sg = sgk + TILE * TP;      // decay
  float* sk = sg + TILE * TP;       // unit key
  float* sq = sk + TILE * TP;       // unit query * qscale
  float* red = sq + TILE * TP;      // [16][TILE] cross-wave partials
  float* sbeta = red + 16 * TILE;   // [TILE] write strength

  const int seg = blockIdx.x / H, hd = blockIdx.x % H;
  const int t0 = seq_rows[4 * seg + 0], n = seq_rows[4 * seg + 1];
  const int p0 = seq_rows[4 * seg + 2], slot = seq_rows[4 * seg + 3];
  const int j = threadIdx.x / P, p = threadIdx.x % P;
  const bool col = j < DV;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int hk = (hd / (H / G)) * D;  // channel offset of the q/k group
  const int hz = hd * D;              // channel offset in zdec / dt_bias
  const int hv = hd * DV;             // channel offset in v / zgate / out
  const float rate = expf(a_log[hd]);

  float* Sg = state + ((size_t)slot * H + hd) * (size_t)D * DV;
  float S[R];  // S[r] = row p + P * r of column j
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int i = p + P * r;
    S[r] = (col && i < D && p0 != 0) ? Sg[(size_t)i * DV + j] : 0.f;
  }

  // The inputs of tile t+1 are fetched into registers before tile t is
  // swept, so their global-memory latency hides behind the sweep. A thread
  // prepares elements tid + e * blockDim of a tile (token-major, DKP per
  // token); the first NE of them go through the registers, any beyond that
  // (few columns on a tall state) are loaded when the tile is committed.
  // (a 1024-thread launch has 128 registers a lane: no room for them).
  // Fetching ahead pays for launches of up to 256 threads; wider ones
  // (measured: 512 threads on 128 x 128 states) are bound by the sweep's
  // LDS reads and run faster when a tile's inputs are fetched at its start.
  constexpr bool AHEAD = MAXT <= 256;
  constexpr int NE = AHEAD ? 8 : 0;
  constexpr int NEA = NE > 0 ? NE : 1;
  float pk[NEA], pq[NEA], pz[NEA], pdt[NEA];
  constexpr int TA = AHEAD ? TILE : 1;
  float vnext[TA], gnext[TA];
  float bnext = 0.f;
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    const int i = (threadIdx.x + e * blockDim.x) % DKP;
    pdt[e] = i < D ? dt_bias[hz + i] : 0.f;
  }
  auto prefetch = [&](int tb) {
    const int nt = min(TILE, n - tb);
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      const int idx = threadIdx.x + e * blockDim.x;
      const int tt = idx / DKP, i = idx % DKP;
      pk[e] = pq[e] = pz[e] = 0.f;
      if (idx < nt * DKP && i < D) {
        const size_t row = (size_t)(t0 + tb + tt);
        pk[e] = MxElem<T>::ld(k + row * ldk + hk + i);
        pq[e] = MxElem<T>::ld(q + row * ldq + hk + i);
        pz[e] = MxElem<T>::ld(zdec + row * ldzd + hz + i);
      }
    }
#pragma unroll
    for (int tt = 0; tt < TA; ++tt) {
      const size_t row = (size_t)(t0 + tb + min(tt, nt - 1));
      vnext[tt] = col ? MxElem<T>::ld(v + row * ldv + hv + j) : 0.f;
      gnext[tt] = col ? MxElem<T>::ld(zgate + row * ldzg + hv + j) : 0.f;
    }
    if (threadIdx.x < nt)
      bnext = MxElem<T>::ld(beta + (size_t)(t0 + tb + threadIdx.x) * ldb + hd);
  };
  if (AHEAD) prefetch(0);

  for (int tb = 0; tb < n; tb += TILE) {
    const int nt = min(TILE, n - tb);
    __syncthreads();  // previous tile's LDS reads are done
    float vreg[TILE], greg[TILE];
    if constexpr (AHEAD) {
#pragma unroll
      for (int tt = 0; tt < TILE; ++tt) {
        vreg[tt] = vnext[tt];
        greg[tt] = gnext[tt];
      }
      if (threadIdx.x < nt) sbeta[threadIdx.x] = mx_sigmoid(bnext);
    } else {
      // this tile's value and gate entries of column j: issued together,
      // up front, so their latency hides behind the preparation
#pragma unroll
      for (int tt = 0; tt < TILE; ++tt) {
        const size_t row = (size_t)(t0 + tb + min(tt, nt - 1));
        vreg[tt] = col ? MxElem<T>::ld(v + row * ldv + hv + j) : 0.f;
        greg[tt] = col ? MxElem<T>::ld(zgate + row * ldzg + hv + j) : 0.f;
      }
      if (threadIdx.x < nt)
        sbeta[threadIdx.x] = mx_sigmoid(MxElem<T>::ld(
            beta + (size_t)(t0 + tb + threadIdx.x) * ldb + hd));
    }
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      const int idx = threadIdx.x + e * blockDim.x;
      if (idx < nt * DKP) {
        const int tt = idx / DKP, i = idx % DKP;
        // row i is kept at (i % P) * RP + i / P: a lane's rows are
        // contiguous
        const int at = tt * TP + (i % P) * RP + i / P;
        sk[at] = pk[e];
        sq[at] = pq[e];
        sg[at] = i < D ? expf(-rate * mx_softplus(pz[e] + pdt[e])) : 0.f;
      }
    }
    for (int idx = threadIdx.x + NE * blockDim.x; idx < nt * DKP;
         idx += blockDim.x) {
      const int tt = idx / DKP, i = idx % DKP;
      const int at = tt * TP + (i % P) * RP + i / P;
      float kv = 0.f, qv = 0.f, gv = 0.f;
      if (i < D) {
        const size_t row = (size_t)(t0 + tb + tt);
        kv = MxElem<T>::ld(k + row * ldk + hk + i);
        qv = MxElem<T>::ld(q + row * ldq + hk + i);
        const float z = MxElem<T>::ld(zdec + row * ldzd + hz + i);
        gv = expf(-rate * mx_softplus(z + dt_bias[hz + i]));
      }
      sk[at] = kv;
      sq[at] = qv;
      sg[at] = gv;
    }
    if (AHEAD && tb + TILE < n) prefetch(tb + TILE);
    __syncthreads();
    for (int tt = wave; tt < nt; tt += nw) {
      float sk2 = 0.f, sq2 = 0.f;
      for (int i = lane; i < DKP; i += 64) {
        const int at = tt * TP + (i % P) * RP + i / P;
        sk2 += sk[at] * sk[at];
        sq2 += sq[at] * sq[at];
      }
      sk2 = mx_wave_sum(sk2);
      sq2 = mx_wave_sum(sq2);
      const float ik = 1.0f / sqrtf(sk2 + 1e-6f);
      const float iq = qscale / sqrtf(sq2 + 1e-6f);
      for (int i = lane; i < DKP; i += 64) {
        const int at = tt * TP + (i % P) * RP + i / P;
        const float ku = sk[at] * ik;
        sk[at] = ku;
        sgk[at] = sg[at] * ku;
        sq[at] *= iq;
      }
    }
    __syncthreads();

    float o[TILE];
#pragma unroll
    for (int tt = 0; tt < TILE; ++tt) {
      o[tt] = 0.f;
      if (tt < nt) {
        const float4* pgk = (const float4*)(sgk + tt * TP + p * RP);
        const float4* pg = (const float4*)(sg + tt * TP + p * RP);
        const float4* pk = (const float4*)(sk + tt * TP + p * RP);
        const float4* pq = (const float4*)(sq + tt * TP + p * RP);
        float sa = 0.f;
#pragma unroll
        for (int i = 0; i < R / 4; ++i) {
          const float4 a4 = pgk[i];
          sa += a4.x * S[4 * i] + a4.y * S[4 * i + 1] + a4.z * S[4 * i + 2] +
                a4.w * S[4 * i + 3];
        }
#pragma unroll
        for (int off = 1; off < P; off <<= 1) sa += __shfl_xor(sa, off, 64);
        const float u = sbeta[tt] * (vreg[tt] - sa);
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < R / 4; ++i) {
          const float4 g4 = pg[i], k4 = pk[i], q4 = pq[i];
          const float gv[4] = {g4.x, g4.y, g4.z, g4.w};
          const float kv[4] = {k4.x, k4.y, k4.z, k4.w};
          const float qv[4] = {q4.x, q4.y, q4.z, q4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float s = gv[e] * S[4 * i + e] + kv[e] * u;
            S[4 * i + e] = s;
            acc += s * qv[e];
          }
        }
#pragma unroll
        for (int off = 1; off < P; off <<= 1) acc += __shfl_xor(acc, off, 64);
        o[tt] = acc;
      }
    }

    // per-token sum over the head's columns of o^2
#pragma unroll
    for (int tt = 0; tt < TILE; ++tt) {
      const float s2 = mx_wave_sum((col && p == 0) ? o[tt] * o[tt] : 0.f);
      if (lane == 0) red[wave * TILE + tt] = s2;
    }
    __syncthreads();
    if (col && p == 0) {
#pragma unroll
      for (int tt = 0; tt < TILE; ++tt) {
        if (tt < nt) {
          float ss = 0.f;
          for (int w = 0; w < nw; ++w) ss += red[w * TILE + tt];
          const size_t row = (size_t)(t0 + tb + tt);
          const float inv = 1.0f / sqrtf(ss / (float)DV + eps);
          MxElem<T>::st(out + row * ldo + hv + j,
                        o[tt] * inv * normw[j] * mx_sigmoid(greg[tt]));
        }
      }
    }
  }
  if (col) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int i = p + P * r;
      if (i < D) Sg[(size_t)i * DV + j] = S[r];
    }
  }
}

#define GD_ARGS                                                              \
  void *out, int ldo, const void *q, int ldq, const void *k, int ldk,        \
      const void *v, int ldv, const void *beta, int ldb, const void *zdec,   \
      int ldzd, const void *zgate, int ldzg, const void *a_log,              \
      const void *dt_bias, const void *normw, void *state,                   \
      const void *seq_rows, int S_, int H, int G, int D, int DV, float eps,  \
      float qscale, void *stream
#define GD_PASS                                                              \
  out, ldo, q, ldq, k, ldk, v, ldv, beta, ldb, zdec, ldzd, zgate, ldzg,      \
      a_log, dt_bias, normw, state, seq_rows, S_, H, G, D, DV, eps, qscale,  \
      stream

template <typename T, int DKP>
static int launch_gated_delta(GD_ARGS) {
  constexpr int TILE = DKP <= 128 ? 16 : 8;
  // lanes per column: enough to keep a lane's rows within 32 registers
  // where the column count allows it
  constexpr int P = DKP >= 64 ? 4 : (DKP >= 32 ? 2 : 1);
  const int threads = ((DV * P + 63) / 64) * 64;
  if (threads > 1024) return 1;
  const size_t lds =
      (size_t)(4 * TILE * (DKP + (P > 1 ? 4 * P : 0)) + 16 * TILE + TILE) *
      sizeof(float);
#define GD_LAUNCH(MAXT)                                                      \
  hipLaunchKernelGGL((gated_delta_kernel<T, DKP, TILE, P, MAXT>),            \
                     dim3(S_ * H), dim3(threads), lds, (hipStream_t)stream,  \
                     (T*)out, ldo, (const T*)q, ldq, (const T*)k, ldk,       \
                     (const T*)v, ldv, (const T*)beta, ldb, (const T*)zdec,  \
                     ldzd, (const T*)zgate, ldzg, (const float*)a_log,       \
                     (const float*)dt_bias, (const float*)normw,             \
                     (float*)state, (const int*)seq_rows, H, G, D, DV, eps,  \
                     qscale)
  // the launch bound follows the thread count, so small launches get the
  // registers for the prefetched tile and a lane's rows stay out of scratch
  if (threads <= 256) {
    GD_LAUNCH(256);
  } else if (threads <= 512) {
    GD_LAUNCH(512);
  } else {
    GD_LAUNCH(1024);
  }
#undef GD_LAUNCH
  return 0;
}

#define GD_CASE(PAD) \
  if (D <= PAD) return launch_gated_delta<T, PAD>(GD_PASS);

template <typename T>
static int dispatch_gated_delta(GD_ARGS) {
  GD_CASE(16)
  GD_CASE(32)
  GD_CASE(48)
  GD_CASE(64)
  GD_CASE(96)
  GD_CASE(128)
  GD_CASE(192)
  GD_CASE(256)
  return 1;  // key dim above 256: not built
}

// The file may be compiled once per element type (MX_ONLY_DTYPE = 0 bf16,
// 1 float) so the two sets of head-size instantiations build in parallel;
// the float unit also carries the entry point.
extern "C" int mx_gated_delta_bf16(GD_ARGS);
extern "C" int mx_gated_delta_f32(GD_ARGS);

#if !defined(MX_ONLY_DTYPE) || MX_ONLY_DTYPE == 0
extern "C" int mx_gated_delta_bf16(GD_ARGS) {
  return dispatch_gated_delta<mx_bf16>(GD_PASS);
}
#endif
#if !defined(MX_ONLY_DTYPE) || MX_ONLY_DTYPE == 1
extern "C" int mx_gated_delta_f32(GD_ARGS) {
  return dispatch_gated_delta<float>(GD_PASS);
}

extern "C" int mx_gated_delta(
    void* out, int ldo, const void* q, int ldq, const void* k, int ldk,
    const void* v, int ldv, const void* beta, int ldb, const void* zdec,
    int ldzd, const void* zgate, int ldzg, const void* a_log,
    const void* dt_bias, const void* normw, void* state,
    const void* seq_rows, int S_, int H, int G, int D, int DV, float eps,
    float qscale, int dtype, void* stream) {
  if (S_ <= 0) return 0;
  if (dtype == MX_BF16) return mx_gated_delta_bf16(GD_PASS);
  return mx_gated_delta_f32(GD_PASS);
}
#endif
