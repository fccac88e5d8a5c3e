// Shared helpers for the fp32-residual mixer kernels (gfx950, wave64).
//
// Every kernel here is templated on the activation element type (bf16 or
// float) and keeps its arithmetic in fp32; the element type only decides
// how values are loaded and how results are rounded when stored. The
// launchers use a plain C ABI (pointers, sizes, stream) so the library
// builds with hipcc alone and is loaded through ctypes.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ps_common.h"

struct mx_bf16 {
  unsigned short x;
};

template <typename T>
struct MxElem;

template <>
struct MxElem<float> {
  static PS_DEV float ld(const float* p) { return *p; }
  static PS_DEV void st(float* p, float v) { *p = v; }
};

template <>
struct MxElem<mx_bf16> {
  static PS_DEV float ld(const mx_bf16* p) { return ps_bf16_to_f32(p->x); }
  static PS_DEV void st(mx_bf16* p, float v) { p->x = ps_f32_to_bf16(v); }
};

PS_DEV float mx_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

PS_DEV float mx_wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Sum over the whole block (blockDim.x a multiple of 64, at most 1024);
// `red` is 17 floats of LDS. Every thread gets the total.
PS_DEV float mx_block_sum(float v, float* red) {
  v = mx_wave_sum(v);
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();  // red may still be read from a previous call
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
  for (int w = 0; w < nw; ++w) s += red[w];
  return s;
}

// dtype codes of the C ABI
#define MX_BF16 0
#define MX_F32 1

#define MX_DISPATCH_DTYPE(code, ...)  \
  if ((code) == MX_BF16) {            \
    typedef mx_bf16 T;                \
    __VA_ARGS__                       \
  } else {                            \
    typedef float T;                  \
    __VA_ARGS__                       \
  }
