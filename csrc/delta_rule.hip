// Gated delta-rule recurrence (prefill portions and single decode tokens in
// one launch).
//
// Per head the state S is a D x D fp32 matrix (rows = key channels, columns
// = value channels). For every token
//     w = exp(-decay_scale * sigmoid(zw + w0))        per key channel
//     a = sigmoid(za + ab)                            per key channel
//     u = k / sqrt(sum(k^2) + 1e-6)
//     S <- diag(w) S - (a*u)(u^T S) + k v^T           (both read the old S)
//     o = S^T r
// and the head's o is divided by its root mean square, scaled by a channel
// weight and by sigmoid(g).
//
// Mapping: one workgroup per (sequence segment, head). Column j of S lives
// in the registers of P adjacent lanes, lane p holding rows p, p+P, ...
// (DKP / P rows, D padded up to DKP), so u^T S and S^T r are short
// thread-local dot products finished by a P-lane butterfly; the only other
// cross-lane traffic is the two norms. Tokens go through in tiles: the
// per-row vectors (u, a*u, w, k, r) of a whole tile are prepared
// cooperatively into LDS (stored so that each lane's rows are contiguous),
// then each thread walks the tile's tokens with broadcast LDS reads and no
// barrier.
#include "mix_common.h"

template <typename T, int DKP, int TILE, int P>
__global__ __launch_bounds__(DKP * P <= 256 ? 256 : DKP * P)
void delta_rule_kernel(
    T* __restrict__ out, int ldo, const T* __restrict__ r, int ldr,
    const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    const T* __restrict__ zw, int ldzw, const T* __restrict__ za, int ldza,
    const T* __restrict__ g, int ldg, const float* __restrict__ w0,
    const float* __restrict__ ab, const float* __restrict__ normw,
    float* __restrict__ state, const int* __restrict__ seq_rows, int H, int D,
    float eps, float decay_scale) {
  extern __shared__ __align__(16) float lds[];
  constexpr int R = DKP / P;        // rows per lane
  // a lane's R rows are contiguous; the P segments of a token are RP words
  // apart so that the P addresses of one broadcast read fall into
  // different banks
  constexpr int RP = P > 1 ? R + 4 : R;
  constexpr int TP = RP * P;        // words per token and array
  float* su = lds;                  // [TILE][TP] unit key
  float* sau = su + TILE * TP;      // a * u
  float* sw = sau + TILE * TP;      // decay
  float* sk = sw + TILE * TP;       // key
  float* sr = sk + TILE * TP;       // receptance
  float* red = sr + TILE * TP;      // [16][TILE] cross-wave partials

  const int seg = blockIdx.x / H, hd = blockIdx.x % H;
  const int t0 = seq_rows[4 * seg + 0], n = seq_rows[4 * seg + 1];
  const int p0 = seq_rows[4 * seg + 2], slot = seq_rows[4 * seg + 3];
  const int j = threadIdx.x / P, p = threadIdx.x % P;
  const bool col = j < D;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int hc = hd * D;  // channel offset of this head

  float* Sg = state + ((size_t)slot * H + hd) * (size_t)D * D;
  float S[R];  // S[k] = row p + P * k of column j
#pragma unroll
  for (int k2 = 0; k2 < R; ++k2) {
    const int i = p + P * k2;
    S[k2] = (col && i < D && p0 != 0) ? Sg[(size_t)i * D + j] : 0.f;
  }

  for (int tb = 0; tb < n; tb += TILE) {
    const int nt = min(TILE, n - tb);
    __syncthreads();  // previous tile's LDS reads are done
    // this tile's value and gate entries of column j: issued together, up
    // front, so their latency hides behind the cooperative preparation
    float vreg[TILE], greg[TILE];
#pragma unroll
    for (int tt = 0; tt < TILE; ++tt) {
      const size_t row = (size_t)(t0 + tb + min(tt, nt - 1));
      vreg[tt] = col ? MxElem<T>::ld(v + row * ldv + hc + j) : 0.f;
      greg[tt] = col ? MxElem<T>::ld(g + row * ldg + hc + j) : 0.f;
    }
    // four elements per thread and pass, all their loads before any use
    for (int base = 0; base < nt * DKP; base += blockDim.x * 4) {
      float kv[4], rv[4], zv[4], av[4];
      int at[4], ch[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int idx = base + u * blockDim.x + threadIdx.x;
        at[u] = -1;
        ch[u] = -1;
        kv[u] = rv[u] = zv[u] = av[u] = 0.f;
        if (idx < nt * DKP) {
          const int tt = idx / DKP, i = idx % DKP;
          // row i is kept at (i % P) * R + i / P: a lane's rows are
          // contiguous
          at[u] = tt * TP + (i % P) * RP + i / P;
          if (i < D) {
            const size_t row = (size_t)(t0 + tb + tt);
            const int c = hc + i;
            ch[u] = c;
            kv[u] = MxElem<T>::ld(k + row * ldk + c);
            rv[u] = MxElem<T>::ld(r + row * ldr + c);
            zv[u] = MxElem<T>::ld(zw + row * ldzw + c);
            av[u] = MxElem<T>::ld(za + row * ldza + c);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        if (at[u] >= 0) {
          float wv = 0.f, aa = 0.f;
          if (ch[u] >= 0) {
            wv = expf(-decay_scale * mx_sigmoid(zv[u] + w0[ch[u]]));
            aa = mx_sigmoid(av[u] + ab[ch[u]]);
          }
          sk[at[u]] = kv[u];
          sr[at[u]] = rv[u];
          sw[at[u]] = wv;
          sau[at[u]] = aa;
        }
      }
    }
    __syncthreads();
    for (int tt = wave; tt < nt; tt += nw) {
      float ss = 0.f;
      for (int i = lane; i < DKP; i += 64) {
        const float kv = sk[tt * TP + (i % P) * RP + i / P];
        ss += kv * kv;
      }
      ss = mx_wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss + 1e-6f);
      for (int i = lane; i < DKP; i += 64) {
        const int at = tt * TP + (i % P) * RP + i / P;
        const float u = sk[at] * inv;
        su[at] = u;
        sau[at] *= u;
      }
    }
    __syncthreads();

    float o[TILE];
#pragma unroll
    for (int tt = 0; tt < TILE; ++tt) {
      o[tt] = 0.f;
      if (tt < nt) {
        const float vj = vreg[tt];
        const float4* pu = (const float4*)(su + tt * TP + p * RP);
        const float4* pau = (const float4*)(sau + tt * TP + p * RP);
        const float4* pw = (const float4*)(sw + tt * TP + p * RP);
        const float4* pk = (const float4*)(sk + tt * TP + p * RP);
        const float4* pr = (const float4*)(sr + tt * TP + p * RP);
        float sa = 0.f;
#pragma unroll
        for (int i = 0; i < R / 4; ++i) {
          const float4 u4 = pu[i];
          sa += u4.x * S[4 * i] + u4.y * S[4 * i + 1] + u4.z * S[4 * i + 2] +
                u4.w * S[4 * i + 3];
        }
#pragma unroll
        for (int off = 1; off < P; off <<= 1) sa += __shfl_xor(sa, off, 64);
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < R / 4; ++i) {
          const float4 w4 = pw[i], a4 = pau[i], k4 = pk[i], r4 = pr[i];
          const float wv[4] = {w4.x, w4.y, w4.z, w4.w};
          const float av[4] = {a4.x, a4.y, a4.z, a4.w};
          const float kv[4] = {k4.x, k4.y, k4.z, k4.w};
          const float rv[4] = {r4.x, r4.y, r4.z, r4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float s = wv[e] * S[4 * i + e] - av[e] * sa + kv[e] * vj;
            S[4 * i + e] = s;
            acc += s * rv[e];
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
      const float q = mx_wave_sum((col && p == 0) ? o[tt] * o[tt] : 0.f);
      if (lane == 0) red[wave * TILE + tt] = q;
    }
    __syncthreads();
    if (col && p == 0) {
#pragma unroll
      for (int tt = 0; tt < TILE; ++tt) {
        if (tt < nt) {
          float ss = 0.f;
          for (int w = 0; w < nw; ++w) ss += red[w * TILE + tt];
          const size_t row = (size_t)(t0 + tb + tt);
          const float inv = 1.0f / sqrtf(ss / (float)D + eps);
          const float gate = mx_sigmoid(greg[tt]);
          MxElem<T>::st(out + row * ldo + hc + j,
                        o[tt] * inv * normw[hc + j] * gate);
        }
      }
    }
  }
  if (col) {
#pragma unroll
    for (int k2 = 0; k2 < R; ++k2) {
      const int i = p + P * k2;
      if (i < D) Sg[(size_t)i * D + j] = S[k2];
    }
  }
}

template <typename T, int DKP>
static void launch_delta(void* out, int ldo, const void* r, int ldr,
                         const void* k, int ldk, const void* v, int ldv,
                         const void* zw, int ldzw, const void* za, int ldza,
                         const void* g, int ldg, const void* w0,
                         const void* ab, const void* normw, void* state,
                         const void* seq_rows, int S_, int H, int D,
                         float eps, float decay_scale, hipStream_t stream) {
  constexpr int TILE = DKP <= 128 ? 16 : 8;
  constexpr int P = DKP >= 64 ? 4 : (DKP >= 32 ? 2 : 1);
  const int threads = ((D * P + 63) / 64) * 64;
  const size_t lds =
      (size_t)(5 * TILE * (DKP + (P > 1 ? 4 * P : 0)) + 16 * TILE) *
      sizeof(float);
  hipLaunchKernelGGL((delta_rule_kernel<T, DKP, TILE, P>), dim3(S_ * H),
                     dim3(threads), lds, stream, (T*)out, ldo, (const T*)r,
                     ldr, (const T*)k, ldk, (const T*)v, ldv, (const T*)zw,
                     ldzw, (const T*)za, ldza, (const T*)g, ldg,
                     (const float*)w0, (const float*)ab,
                     (const float*)normw, (float*)state,
                     (const int*)seq_rows, H, D, eps, decay_scale);
}

#define DR_CASE(P)                                                          \
  if (D <= P) {                                                             \
    launch_delta<T, P>(out, ldo, r, ldr, k, ldk, v, ldv, zw, ldzw, za,      \
                       ldza, g, ldg, w0, ab, normw, state, seq_rows, S_, H, \
                       D, eps, decay_scale, (hipStream_t)stream);           \
    return 0;                                                               \
  }

template <typename T>
static int dispatch_delta(void* out, int ldo, const void* r, int ldr,
                          const void* k, int ldk, const void* v, int ldv,
                          const void* zw, int ldzw, const void* za, int ldza,
                          const void* g, int ldg, const void* w0,
                          const void* ab, const void* normw, void* state,
                          const void* seq_rows, int S_, int H, int D,
                          float eps, float decay_scale, void* stream) {
  DR_CASE(16)
  DR_CASE(32)
  DR_CASE(48)
  DR_CASE(64)
  DR_CASE(80)
  DR_CASE(96)
  DR_CASE(112)
  DR_CASE(128)
  DR_CASE(192)
  DR_CASE(256)
  return 1;  // head dim above 256: not built
}

// The file may be compiled once per element type (MX_ONLY_DTYPE = 0 bf16,
// 1 float) so the two sets of head-size instantiations build in parallel;
// the float unit also carries the entry point.
#define DR_ARGS                                                              \
  void *out, int ldo, const void *r, int ldr, const void *k, int ldk,        \
      const void *v, int ldv, const void *zw, int ldzw, const void *za,      \
      int ldza, const void *g, int ldg, const void *w0, const void *ab,      \
      const void *normw, void *state, const void *seq_rows, int S_, int H,   \
      int D, float eps, float decay_scale, void *stream
#define DR_PASS                                                              \
  out, ldo, r, ldr, k, ldk, v, ldv, zw, ldzw, za, ldza, g, ldg, w0, ab,      \
      normw, state, seq_rows, S_, H, D, eps, decay_scale, stream

extern "C" int mx_delta_rule_bf16(DR_ARGS);
extern "C" int mx_delta_rule_f32(DR_ARGS);

#if !defined(MX_ONLY_DTYPE) || MX_ONLY_DTYPE == 0
extern "C" int mx_delta_rule_bf16(DR_ARGS) {
  return dispatch_delta<mx_bf16>(DR_PASS);
}
#endif
#if !defined(MX_ONLY_DTYPE) || MX_ONLY_DTYPE == 1
extern "C" int mx_delta_rule_f32(DR_ARGS) {
  return dispatch_delta<float>(DR_PASS);
}

extern "C" int mx_delta_rule(void* out, int ldo, const void* r, int ldr,
                             const void* k, int ldk, const void* v, int ldv,
                             const void* zw, int ldzw, const void* za,
                             int ldza, const void* g, int ldg,
                             const void* w0, const void* ab,
                             const void* normw, void* state,
                             const void* seq_rows, int S_, int H, int D,
                             float eps, float decay_scale, int dtype,
                             void* stream) {
  if (S_ <= 0) return 0;
  if (dtype == MX_BF16)
    return mx_delta_rule_bf16(out, ldo, r, ldr, k, ldk, v, ldv, zw, ldzw, za,
                              ldza, g, ldg, w0, ab, normw, state, seq_rows,
                              S_, H, D, eps, decay_scale, stream);
  return mx_delta_rule_f32(out, ldo, r, ldr, k, ldk, v, ldv, zw, ldzw, za,
                           ldza, g, ldg, w0, ab, normw, state, seq_rows, S_,
                           H, D, eps, decay_scale, stream);
}
#endif
