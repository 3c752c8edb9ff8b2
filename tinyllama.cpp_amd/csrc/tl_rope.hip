// tl_rope.hip — rotary positions for the heads of a layer-list mixer, with what follows them in the same pass.
//
//   rotation   on the first rot_dims dimensions of each head, dimension 2i paired with 2i + 1 (the interleaved layout):
//              (u, v) at position p -> (u cos a - v sin a, v cos a + u sin a), a = p * f_i, f_i = base^(-2i / rot_dims).
//              The angle is formed in double (an integer position times a double frequency) and brought into [-pi, pi]
//              there; cos and sin of that remainder are FP32. An FP32 product p * f_i alone is off by up to p * 2^-24
//              radians, which at a few thousand positions is what decides the error of the logits.
//   extension  (factor > 0) the frequencies of slowly turning pairs are divided by `factor`, fast ones stay, with a linear
//              ramp between the pair that makes `fast` turns and the one that makes `slow` turns over the original context:
//              d(t) = rot_dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(d(fast)), 0),
//              hi = min(ceil(d(slow)), rot_dims - 1), r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1),
//              f_i <- f_i / factor * r_i + f_i * (1 - r_i); cos and sin are multiplied by 0.1 ln(factor) + 1.
//              The table of rot_dims / 2 frequencies is computed once on the host in double precision.
//   unit norm  after the rotation each head is divided by its root mean square over dim (eps inside the root; no weights).
//   caches     the finished keys go to row `pos` of the key cache; a design whose values are its keys as projected gets the
//              untouched key row in the value cache in the same pass.
// A wave per (token, head), four heads a workgroup; a lane holds up to 4 pairs of a head (dim <= 512).
#include <math.h>

#include <vector>

#include "tl_stack.h"

void tl_rotary_frequencies(int rot_dims, double base, double factor, double original, double fast, double slow, double* f,
                           float* mscale) {
  const int half = rot_dims / 2;
  const double pi = 3.14159265358979323846;
  double lo = 0.0, hi = 0.0;
  if (factor > 0.0) {
    auto turn_dim = [&](double t) { return rot_dims * log(original / (2.0 * pi * t)) / (2.0 * log(base)); };
    lo = floor(turn_dim(fast));
    lo = lo < 0.0 ? 0.0 : lo;
    hi = ceil(turn_dim(slow));
    hi = hi > rot_dims - 1 ? rot_dims - 1 : hi;
  }
  for (int i = 0; i < half; ++i) {
    double fi = pow(base, -2.0 * i / rot_dims);
    if (factor > 0.0) {
      const double span = hi - lo > 0.001 ? hi - lo : 0.001;
      double r = (i - lo) / span;
      r = r < 0.0 ? 0.0 : r > 1.0 ? 1.0 : r;
      fi = fi / factor * r + fi * (1.0 - r);
    }
    f[i] = fi;
  }
  *mscale = factor > 0.0 ? (float)(0.1 * log(factor) + 1.0) : 1.0f;
}

namespace {

constexpr int kMaxPairs = 4;  // per lane: dim <= 512

__global__ __launch_bounds__(256) void rotary_kernel(const RotaryArgs a) {
  const int t = blockIdx.x, lane = threadIdx.x & 63;
  const int pos = (a.pos_dev ? *a.pos_dev : a.start_pos) + t;
  const double dpos = (double)pos;
  const int kd = a.kv_heads * a.dim;
  // a wave per head: workgroup y of a token takes heads 4 y .. 4 y + 3 (one token of a decode step still fills several CUs)
  for (int hh = blockIdx.y * 4 + (threadIdx.x >> 6); hh < a.heads + a.kv_heads; hh += 4 * gridDim.y) {
    float* x = a.qk + (size_t)t * a.ld + (size_t)hh * a.dim;
    const bool is_k = hh >= a.heads;
    const int kcol = (hh - a.heads) * a.dim;
    float u[kMaxPairs], v[kMaxPairs];
    float ss = 0.0f;
#pragma unroll
    for (int r = 0; r < kMaxPairs; ++r) {
      const int i = lane + 64 * r, d0 = 2 * i, d1 = d0 + 1;
      u[r] = d0 < a.dim ? x[d0] : 0.0f;
      v[r] = d1 < a.dim ? x[d1] : 0.0f;
      if (is_k && a.vc) {  // the values are the keys as projected
        float* vr = a.vc + (size_t)pos * kd + kcol;
        if (d0 < a.dim) vr[d0] = u[r];
        if (d1 < a.dim) vr[d1] = v[r];
      }
      if (d1 < a.rot_dims) {
        const double full = dpos * a.freq[i];
        const float ang = (float)(full - 6.283185307179586476925 * rint(full * 0.159154943091895335769));
        float sn, cs;
        sincosf(ang, &sn, &cs);
        sn *= a.mscale;
        cs *= a.mscale;
        const float nu = u[r] * cs - v[r] * sn, nv = v[r] * cs + u[r] * sn;
        u[r] = nu;
        v[r] = nv;
      }
      ss += u[r] * u[r] + v[r] * v[r];
    }
    float inv = 1.0f;
    if (a.unit_norm) {
#pragma unroll
      for (int o = 32; o >= 1; o >>= 1) ss += __shfl_xor(ss, o);
      inv = 1.0f / sqrtf(ss / (float)a.dim + a.eps);
    }
    float* kr = (is_k && a.kc) ? a.kc + (size_t)pos * kd + kcol : nullptr;
#pragma unroll
    for (int r = 0; r < kMaxPairs; ++r) {
      const int d0 = 2 * (lane + 64 * r), d1 = d0 + 1;
      if (d0 < a.dim) {
        x[d0] = u[r] * inv;
        if (kr) kr[d0] = u[r] * inv;
      }
      if (d1 < a.dim) {
        x[d1] = v[r] * inv;
        if (kr) kr[d1] = v[r] * inv;
      }
    }
  }
  if (a.v_src)
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < a.vd; c += blockDim.x * gridDim.y)
      a.v_dst[(size_t)pos * a.vd + c] = a.v_src[(size_t)t * a.ld + c];
}

}  // namespace

int tl_launch_rotary(const RotaryArgs& a, hipStream_t s) {
  TL_REQUIRE(a.qk && a.T > 0 && a.heads >= 0 && a.kv_heads >= 0 && a.heads + a.kv_heads > 0 && a.dim > 0, "rotary: bad arguments");
  TL_REQUIRE(a.dim <= 128 * kMaxPairs, "rotary: head size %d above %d", a.dim, 128 * kMaxPairs);
  TL_REQUIRE(a.rot_dims >= 0 && a.rot_dims <= a.dim && (a.rot_dims & 1) == 0, "rotary: %d rotating dimensions of %d", a.rot_dims,
             a.dim);
  TL_REQUIRE(a.rot_dims == 0 || a.freq, "rotary: no frequency table");
  TL_REQUIRE(a.ld >= (a.heads + a.kv_heads) * a.dim, "rotary: row stride %d too short", a.ld);
  TL_REQUIRE(a.pos_dev || a.start_pos >= 0, "rotary: negative start position");
  TL_REQUIRE(!a.v_src || (a.v_dst && a.vd > 0), "rotary: a value row without its cache");
  const int per_token = (a.heads + a.kv_heads + 3) / 4;
  rotary_kernel<<<dim3(a.T, per_token < 65535 ? per_token : 65535), 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

extern "C" int tl_rotary_heads(float* x_dev, int num_tokens, int start_pos, int heads, int dim, int rot_dims, float rot_base,
                               float rot_factor, float rot_original, float rot_fast, float rot_slow, int unit_norm, float eps,
                               void* stream) {
  TL_REQUIRE(rot_dims >= 0 && rot_dims <= dim && (rot_dims & 1) == 0, "tl_rotary_heads: %d rotating dimensions of %d", rot_dims, dim);
  hipStream_t s = static_cast<hipStream_t>(stream);
  std::vector<double> f(rot_dims / 2 + 1);
  float mscale = 1.0f;
  double* fdev = nullptr;
  if (rot_dims > 0) {
    tl_rotary_frequencies(rot_dims, rot_base, rot_factor, rot_original, rot_fast, rot_slow, f.data(), &mscale);
    void* ws = nullptr;
    TL_TRY(tl_scratch(TL_SCRATCH_ROTARY, sizeof(double) * (rot_dims / 2), &ws));
    fdev = static_cast<double*>(ws);
    TL_HIP(hipMemcpyAsync(fdev, f.data(), sizeof(double) * (rot_dims / 2), hipMemcpyHostToDevice, s));
    TL_HIP(hipStreamSynchronize(s));
  }
  RotaryArgs a = {};
  a.qk = x_dev;
  a.ld = heads * dim;
  a.heads = heads;
  a.kv_heads = 0;
  a.dim = dim;
  a.rot_dims = rot_dims;
  a.freq = fdev;
  a.mscale = mscale;
  a.unit_norm = unit_norm;
  a.eps = eps;
  a.T = num_tokens;
  a.start_pos = start_pos;
  return tl_launch_rotary(a, s);
}
