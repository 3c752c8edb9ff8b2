// tl_route.h — the selection step of a mixture's router, shared by the stand-alone router launch (tl_moe.hip) and the
// residual-norm launch that carries the router of the feed-forward behind it (tl_norm.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <math.h>

// One wave (all 64 lanes) picks the `top` largest of z[experts] (LDS; overwritten), the lower index among equals, and writes
// ids[top] (largest first) and wts[top] = the softmax over the chosen logits.
__device__ __forceinline__ void tl_route_select(float* z, int experts, int top, int* ids, float* wts, int lane) {
    // `top` rounds: the lanes scan the experts not yet chosen for the largest logit (lower index wins among equals)
    float mx = 0.0f, denom = 0.0f, mine = 0.0f;
    int my_id = -1;
    for (int j = 0; j < top; ++j) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int e = lane; e < experts; e += 64) {
        const float v = z[e];
        if (v > bv || (v == bv && e < bi)) {
          bv = v;
          bi = e;
        }
      }
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) {
        const float ov = __shfl_xor(bv, o);
        const int oi = __shfl_xor(bi, o);
        if (ov > bv || (ov == bv && oi < bi)) {
          bv = ov;
          bi = oi;
        }
      }
      if (bi == 0x7fffffff) bi = 0;  // only when every logit is NaN
      if (j == 0) mx = bv;
      const float p = expf(bv - mx);
      denom += p;
      if (lane == j % 64 && j < 64) {
        mine = p;
        my_id = bi;
      }
      if (j >= 64 && lane == 0) {  // more than 64 choices: written unnormalised, fixed up below
        ids[j] = bi;
        wts[j] = p;
      }
      if (lane == 0) z[bi] = -INFINITY;  // chosen: out of the next rounds
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    if (lane < top && lane < 64) {
      ids[lane] = my_id;
      wts[lane] = mine / denom;
    }
    if (top > 64 && lane == 0)
      for (int j = 64; j < top; ++j) wts[j] /= denom;
}
