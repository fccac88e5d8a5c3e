// fp32 residual-stream kernels: scaled embedding gather, fused
// (residual += deltas) + RMSNorm, gated-MLP inner activations, paged KV
// append with independent key/value widths.
#include "mix_common.h"

template <typename T>
__global__ __launch_bounds__(256) void embed_scale_kernel(
    float* __restrict__ x, const int64_t* __restrict__ tokens,
    const T* __restrict__ embed, float scale, int W) {
  const int t = blockIdx.x;
  const T* row = embed + (size_t)tokens[t] * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    x[(size_t)t * W + c] = MxElem<T>::ld(row + c) * scale;
}

// x[t] += d0[t] + d1[t] (each optional), h[t] = x[t] / rms(x[t]) * w.
template <typename T>
__global__ __launch_bounds__(256) void add_rms_norm32_kernel(
    T* __restrict__ h, float* __restrict__ x, const T* __restrict__ d0,
    int ld0, const T* __restrict__ d1, int ld1, const float* __restrict__ w,
    float eps, int W) {
  __shared__ float red[17];
  const int t = blockIdx.x;
  float* xr = x + (size_t)t * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    float v = xr[c];
    if (d0 != nullptr) {
      float d = MxElem<T>::ld(d0 + (size_t)t * ld0 + c);
      if (d1 != nullptr) d += MxElem<T>::ld(d1 + (size_t)t * ld1 + c);
      v += d;
      xr[c] = v;
    }
    ss += v * v;
  }
  ss = mx_block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += blockDim.x)
    MxElem<T>::st(h + (size_t)t * W + c, xr[c] * inv * w[c]);
}

#define MX_ACT_SILU 0
#define MX_ACT_GELU_TANH 1
#define MX_ACT_CLAMPED_SWISH 2

template <typename T, int KIND>
__global__ __launch_bounds__(256) void gated_act_kernel(
    T* __restrict__ out, int ldo, const T* __restrict__ gate, int ldg,
    const T* __restrict__ up, int ldu, int F, float limit) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= F) return;
  float g = MxElem<T>::ld(gate + (size_t)t * ldg + c);
  float u = MxElem<T>::ld(up + (size_t)t * ldu + c);
  float y;
  if (KIND == MX_ACT_SILU) {
    y = g * mx_sigmoid(g) * u;
  } else if (KIND == MX_ACT_GELU_TANH) {
    const float z = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    y = 0.5f * g * (1.0f + tanhf(z)) * u;
  } else {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    y = g * mx_sigmoid(1.702f * g) * (u + 1.0f);
  }
  MxElem<T>::st(out + (size_t)t * ldo + c, y);
}

// k [T, G*D] (row stride ldk), v [T, G*DV] -> caches [NB, G, BS, D|DV]
template <typename T>
__global__ __launch_bounds__(256) void kv_append_kernel(
    const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    T* __restrict__ kc, T* __restrict__ vc,
    const int64_t* __restrict__ slots, int G, int D, int DV, int BS) {
  const int t = blockIdx.x;
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const int64_t blk = slot / BS;
  const int off = (int)(slot % BS);
  for (int c = threadIdx.x; c < G * D; c += blockDim.x) {
    const int g = c / D, d = c % D;
    kc[((blk * G + g) * BS + off) * (int64_t)D + d] = k[(size_t)t * ldk + c];
  }
  for (int c = threadIdx.x; c < G * DV; c += blockDim.x) {
    const int g = c / DV, d = c % DV;
    vc[((blk * G + g) * BS + off) * (int64_t)DV + d] = v[(size_t)t * ldv + c];
  }
}

extern "C" {

void mx_embed_scale(void* x, const void* tokens, const void* embed,
                    float scale, int T_, int W, int dtype, void* stream) {
  if (T_ <= 0) return;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((embed_scale_kernel<T>), dim3(T_), dim3(256), 0,
                       (hipStream_t)stream, (float*)x,
                       (const int64_t*)tokens, (const T*)embed, scale, W);
  })
}

void mx_add_rms_norm32(void* h, void* x, const void* d0, int ld0,
                       const void* d1, int ld1, const void* w, float eps,
                       int T_, int W, int dtype, void* stream) {
  if (T_ <= 0) return;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((add_rms_norm32_kernel<T>), dim3(T_), dim3(256), 0,
                       (hipStream_t)stream, (T*)h, (float*)x, (const T*)d0,
                       ld0, (const T*)d1, ld1, (const float*)w, eps, W);
  })
}

void mx_gated_act(void* out, int ldo, const void* gate, int ldg,
                  const void* up, int ldu, int T_, int F, int kind,
                  float limit, int dtype, void* stream) {
  if (T_ <= 0 || F <= 0) return;
  dim3 grid((F + 255) / 256, T_);
  MX_DISPATCH_DTYPE(dtype, {
    if (kind == MX_ACT_SILU) {
      hipLaunchKernelGGL((gated_act_kernel<T, MX_ACT_SILU>), grid, dim3(256),
                         0, (hipStream_t)stream, (T*)out, ldo,
                         (const T*)gate, ldg, (const T*)up, ldu, F, limit);
    } else if (kind == MX_ACT_GELU_TANH) {
      hipLaunchKernelGGL((gated_act_kernel<T, MX_ACT_GELU_TANH>), grid,
                         dim3(256), 0, (hipStream_t)stream, (T*)out, ldo,
                         (const T*)gate, ldg, (const T*)up, ldu, F, limit);
    } else {
      hipLaunchKernelGGL((gated_act_kernel<T, MX_ACT_CLAMPED_SWISH>), grid,
                         dim3(256), 0, (hipStream_t)stream, (T*)out, ldo,
                         (const T*)gate, ldg, (const T*)up, ldu, F, limit);
    }
  })
}

void mx_kv_append(const void* k, int ldk, const void* v, int ldv, void* kc,
                  void* vc, const void* slots, int T_, int G, int D, int DV,
                  int BS, int dtype, void* stream) {
  if (T_ <= 0) return;
  MX_DISPATCH_DTYPE(dtype, {
    hipLaunchKernelGGL((kv_append_kernel<T>), dim3(T_), dim3(256), 0,
                       (hipStream_t)stream, (const T*)k, ldk, (const T*)v,
                       ldv, (T*)kc, (T*)vc, (const int64_t*)slots, G, D, DV,
                       BS);
  })
}

}  // extern "C"
