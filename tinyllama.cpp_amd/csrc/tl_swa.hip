// tl_swa.hip — sliding-window attention over a flat FP32 cache, without rotation: scores are (q . k) * scale, position i sees
// the keys j with 0 <= i - j < window, ordinary softmax, everything in FP32. Key size (dim) and value size (vdim) are
// independent; query head h reads key/value head h / (heads / kv_heads).
//
// One workgroup of 4 waves per (token, head), for the tokens of a prompt chunk and for the single token of a decode step
// alike. The visible keys are cut into pieces of 64; piece c belongs to wave c % 4. Within a piece a lane owns one key
// (score = its dot product with the query held in LDS), the wave keeps a running maximum and sum, and the weighted values
// are accumulated with the lanes spread over the value columns (coalesced rows of V; a key's weight is read from its lane). The four waves' partial
// (max, sum, output) are merged through LDS at the end.
#include <math.h>

#include "tl_stack.h"

namespace {

constexpr int SWA_WAVES = 4;
constexpr int SWA_MAX_VR = 4;  // value columns per lane: vdim <= 256

__global__ __launch_bounds__(256) void swa_kernel(const SwaArgs a) {
  extern __shared__ float lds[];
  float* qs = lds;                                  // [dim]
  float* ow = qs + ((a.dim + 3) & ~3);              // [waves][vdim]
  float* ml = ow + SWA_WAVES * a.vdim;              // [waves][2]
  const int t = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int i = (a.pos_dev ? *a.pos_dev : a.start_pos) + t;
  const int g = h / (a.heads / a.kv_heads);
  const int jlo = (a.window > 0 && i - a.window + 1 > 0) ? i - a.window + 1 : 0;
  const int n = i - jlo + 1;
  const int kld = a.kv_heads * a.dim, vld = a.kv_heads * a.vdim;
  const float* qp = a.q + (size_t)t * a.ldq + (size_t)h * a.dim;
  for (int d = tid; d < a.dim; d += 256) qs[d] = qp[d];
  __syncthreads();
  const bool v4 = (a.dim & 3) == 0 && (kld & 3) == 0 && ((size_t)a.kc & 15) == 0;
  float m = -INFINITY, l = 0.0f;
  float o[SWA_MAX_VR];
#pragma unroll
  for (int r = 0; r < SWA_MAX_VR; ++r) o[r] = 0.0f;
  const int pieces = (n + 63) >> 6;
  for (int c = wave; c < pieces; c += SWA_WAVES) {
    const int j0 = jlo + c * 64;
    const int j = j0 + lane;
    const bool valid = j <= i;
    float sc = -INFINITY;
    if (valid) {
      const float* kp = a.kc + (size_t)j * kld + (size_t)g * a.dim;
      float acc = 0.0f;
      if (v4) {
        for (int d = 0; d < a.dim; d += 4) {
          const float4 kv = *reinterpret_cast<const float4*>(kp + d);
          const float4 qv = *reinterpret_cast<const float4*>(qs + d);
          acc += qv.x * kv.x + qv.y * kv.y + qv.z * kv.z + qv.w * kv.w;
        }
      } else {
        for (int d = 0; d < a.dim; ++d) acc += qs[d] * kp[d];
      }
      sc = acc * a.scale;
    }
    float cm = sc;
#pragma unroll
    for (int w = 32; w >= 1; w >>= 1) cm = fmaxf(cm, __shfl_xor(cm, w));
    const float mn = fmaxf(m, cm);  // finite: lane 0 of a piece is always a visible key
    const float p = valid ? expf(sc - mn) : 0.0f;
    const float corr = expf(m - mn);  // m = -inf at the first piece: 0
    float ps = p;
#pragma unroll
    for (int w = 32; w >= 1; w >>= 1) ps += __shfl_xor(ps, w);
    l = l * corr + ps;
    m = mn;
    const int cnt = (i - j0 + 1) < 64 ? (i - j0 + 1) : 64;
#pragma unroll
    for (int r = 0; r < SWA_MAX_VR; ++r) o[r] *= corr;
    const float* vp = a.vc + (size_t)j0 * vld + (size_t)g * a.vdim;
    for (int jj = 0; jj < cnt; ++jj) {  // jj is wave-uniform: the weight of key jj comes straight from its lane's register
      const float pj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(p), jj));
      const float* vr = vp + (size_t)jj * vld;
#pragma unroll
      for (int r = 0; r < SWA_MAX_VR; ++r) {
        const int d = lane + 64 * r;
        if (d < a.vdim) o[r] += pj * vr[d];
      }
    }
  }
  if (lane == 0) {
    ml[wave * 2] = m;
    ml[wave * 2 + 1] = l;
  }
#pragma unroll
  for (int r = 0; r < SWA_MAX_VR; ++r) {
    const int d = lane + 64 * r;
    if (d < a.vdim) ow[wave * a.vdim + d] = o[r];
  }
  __syncthreads();
  float M = -INFINITY;
#pragma unroll
  for (int w = 0; w < SWA_WAVES; ++w) M = fmaxf(M, ml[w * 2]);
  float f[SWA_WAVES], L = 0.0f;
#pragma unroll
  for (int w = 0; w < SWA_WAVES; ++w) {
    f[w] = expf(ml[w * 2] - M);  // a wave without a piece: exp(-inf) = 0
    L += ml[w * 2 + 1] * f[w];
  }
  float* op = a.out + (size_t)t * a.heads * a.vdim + (size_t)h * a.vdim;
  for (int d = tid; d < a.vdim; d += 256) {
    float acc = 0.0f;
#pragma unroll
    for (int w = 0; w < SWA_WAVES; ++w) acc += ow[w * a.vdim + d] * f[w];
    op[d] = acc / L;
  }
}

}  // namespace

int tl_launch_swa(const SwaArgs& a, hipStream_t s) {
  TL_REQUIRE(a.q && a.kc && a.vc && a.out && a.T > 0, "swa: bad arguments");
  TL_REQUIRE(a.heads > 0 && a.kv_heads > 0 && a.heads % a.kv_heads == 0, "swa: %d heads over %d key/value heads", a.heads,
             a.kv_heads);
  TL_REQUIRE(a.dim > 0 && a.vdim > 0 && a.vdim <= 64 * SWA_MAX_VR, "swa: value size %d outside (0, %d]", a.vdim,
             64 * SWA_MAX_VR);
  TL_REQUIRE(a.pos_dev || a.start_pos >= 0, "swa: negative start position");
  const size_t lds = sizeof(float) * (((a.dim + 3) & ~3) + SWA_WAVES * a.vdim + SWA_WAVES * 2);
  TL_REQUIRE(lds <= 64 * 1024, "swa: key size %d too large", a.dim);
  TL_REQUIRE(a.heads <= 65535, "swa: too many heads");
  swa_kernel<<<dim3(a.T, a.heads), 256, lds, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

extern "C" int tl_swa_attention(const float* q_dev, const float* k_cache_dev, const float* v_cache_dev, float* out_dev,
                                int num_tokens, int start_pos, int heads, int kv_heads, int dim, int vdim, int window,
                                float scale, void* stream) {
  SwaArgs a = {};
  a.q = q_dev;
  a.ldq = heads * dim;
  a.kc = k_cache_dev;
  a.vc = v_cache_dev;
  a.out = out_dev;
  a.T = num_tokens;
  a.heads = heads;
  a.kv_heads = kv_heads;
  a.dim = dim;
  a.vdim = vdim;
  a.window = window;
  a.scale = scale;
  a.start_pos = start_pos;
  return tl_launch_swa(a, static_cast<hipStream_t>(stream));
}
