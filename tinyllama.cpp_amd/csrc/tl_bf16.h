// tl_bf16.h — device helpers shared by the bf16-weight kernels (tl_dense.hip, tl_moe.hip): exact widening of bf16 pairs and
// the dot product of bf16 weight rows with an FP32 vector over the lanes of a wave.
#pragma once
#include <hip/hip_runtime.h>

__device__ __forceinline__ float tl_bf2f(unsigned short h) { return __uint_as_float((unsigned)h << 16); }

// 8 bf16 weights (one 16-byte load) against 8 FP32 values
__device__ __forceinline__ float tl_dot8(const uint4 w, const float4 x0, const float4 x1, float s) {
  s += __uint_as_float(w.x << 16) * x0.x;
  s += __uint_as_float(w.x & 0xffff0000u) * x0.y;
  s += __uint_as_float(w.y << 16) * x0.z;
  s += __uint_as_float(w.y & 0xffff0000u) * x0.w;
  s += __uint_as_float(w.z << 16) * x1.x;
  s += __uint_as_float(w.z & 0xffff0000u) * x1.y;
  s += __uint_as_float(w.w << 16) * x1.z;
  s += __uint_as_float(w.w & 0xffff0000u) * x1.w;
  return s;
}

__device__ __forceinline__ uint4 tl_ldw(const unsigned short* p) {  // weights are read once: keep them out of the caches' way
  typedef unsigned tl_u32x4 __attribute__((ext_vector_type(4)));
  const tl_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const tl_u32x4*>(p));
  return make_uint4(v[0], v[1], v[2], v[3]);
}

__device__ __forceinline__ float tl_wave_sum(float s) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) s += __shfl_xor(s, o);
  return s;
}

// R rows of a bf16 matrix (row r at w + r * stride; rows >= nrows read row 0 and are to be ignored by the caller) against
// x[n]: R x 2 sixteen-byte weight loads are in flight per lane before the first product needs them. vec: n % 8 == 0 and
// 16-byte aligned pointers / strides; otherwise a plain strided loop. Results valid in every lane.
template <int R>
__device__ __forceinline__ void tl_wave_dot_rows(const unsigned short* __restrict__ w, size_t stride, int nrows,
                                                 const float* __restrict__ x, int n, bool vec, int lane, float* out) {
  float acc[R];
  const unsigned short* wr[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    acc[r] = 0.0f;
    wr[r] = w + (r < nrows ? r : 0) * stride;
  }
  if (vec) {
    int k = lane * 8;
    for (; k + 512 < n; k += 1024) {
      uint4 wa[R], wb[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        wa[r] = tl_ldw(wr[r] + k);
        wb[r] = tl_ldw(wr[r] + k + 512);
      }
      const float4 x0 = *reinterpret_cast<const float4*>(x + k), x1 = *reinterpret_cast<const float4*>(x + k + 4);
      const float4 x2 = *reinterpret_cast<const float4*>(x + k + 512), x3 = *reinterpret_cast<const float4*>(x + k + 516);
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] = tl_dot8(wb[r], x2, x3, tl_dot8(wa[r], x0, x1, acc[r]));
    }
    if (k < n) {
      uint4 wa[R];
#pragma unroll
      for (int r = 0; r < R; ++r) wa[r] = tl_ldw(wr[r] + k);
      const float4 x0 = *reinterpret_cast<const float4*>(x + k), x1 = *reinterpret_cast<const float4*>(x + k + 4);
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] = tl_dot8(wa[r], x0, x1, acc[r]);
    }
  } else {
    for (int k = lane; k < n; k += 64) {
      const float xv = x[k];
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] += tl_bf2f(wr[r][k]) * xv;
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) out[r] = tl_wave_sum(acc[r]);
}
