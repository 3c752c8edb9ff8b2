// tl_dense.hip — products with bf16 weight matrices [rows][cols] (row-major, y = W x), FP32 activations and accumulation.
//
//   GEMV (one token): a wave per output row, 16 B of weights per lane per step, widened exactly to FP32: FP32 arithmetic
//   throughout, bound by the bytes of the matrix.
//   GEMM (a chunk of tokens) on the matrix cores: v_mfma_f32_32x32x8_bf16 with the WEIGHTS as the A operand (M = output
//   features) and the tokens as B (N = tokens), so that a lane ends up holding 4 x 4 consecutive features of ONE token and
//   stores them as 16-byte pieces of that token's output row. The FP32 activations are split while they are staged into
//   LDS: terms = 1 keeps their bf16 rounding, terms = 3 keeps hi + mid + lo (3 x 8 mantissa bits = all 24 of an FP32
//   value); the weights are bf16 to begin with, so three MFMAs per product reproduce the FP32 product exactly and only the
//   order of the FP32 accumulation differs from a scalar loop.
//   A workgroup of 4 waves owns a 64-feature x 64-token tile, BK = 32. Items may be gathered (x_rows), scattered (y_rows) and
//   grouped (group_off: blockIdx.z = matrix of the group; tiles beyond a group's items leave at once), which is what the
//   experts of a mixture need: the plan lives on the device, the grid is sized for the worst case.
#include "tl_bf16.h"
#include "tl_stack.h"

namespace {

typedef __attribute__((ext_vector_type(4))) short bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __forceinline__ unsigned short f2bf(float f) {  // round to nearest even
  unsigned u = __float_as_uint(f);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (unsigned short)(u >> 16);
}
__device__ __forceinline__ float bf2f(unsigned short h) { return tl_bf2f(h); }

constexpr int BM = 64, BN = 64, BK = 32, LDK = 40;  // LDK: padded row of a tile in LDS (80 B, keeps 16 B / 8 B alignment)

template <int TERMS>
__global__ __launch_bounds__(256) void dense_gemm_kernel(const DenseArgs a) {
  __shared__ __attribute__((aligned(16))) unsigned short Ws[BM][LDK];
  __shared__ __attribute__((aligned(16))) unsigned short Xs[TERMS][BN][LDK];
  __shared__ int xrow[BN];
  const int tid = threadIdx.x, g = blockIdx.z;
  int lo = 0, hi = a.T;
  if (a.group_off) {
    lo = a.group_off[g];
    hi = a.group_off[g + 1];
  }
  const int t0 = lo + blockIdx.y * BN;
  if (t0 >= hi) return;
  const int f0 = blockIdx.x * BM;
  const unsigned short* W = a.w + (size_t)g * a.rows * a.cols;
  if (tid < BN) {
    const int it = t0 + tid;
    int r = -1;
    if (it < hi) r = a.x_rows ? a.x_rows[it] / a.x_div : it;
    xrow[tid] = r;
  }
  __syncthreads();
  const int wave = tid >> 6, lane = tid & 63, wm = wave & 1, wn = wave >> 1;
  const int lr = tid >> 2, lk = (tid & 3) * 8;  // this thread stages 8 consecutive k of row lr of both tiles
  const int K = a.cols;
  const bool vec = (K & 7) == 0 && (a.ldx & 3) == 0 && ((size_t)a.x & 15) == 0 && ((size_t)W & 15) == 0;
  const int frow = f0 + lr;
  const int xr = xrow[lr];
  const unsigned short* wp = W + (size_t)(frow < a.rows ? frow : 0) * K;
  const float* xp = a.x + (size_t)(xr >= 0 ? xr : 0) * a.ldx;
  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  for (int k0 = 0; k0 < K; k0 += BK) {
    const int k = k0 + lk;
    unsigned short wv[8];
    float xv[8];
    if (vec && k + 8 <= K) {
      const uint4 w4 = frow < a.rows ? *reinterpret_cast<const uint4*>(wp + k) : make_uint4(0, 0, 0, 0);
      wv[0] = w4.x & 0xffff; wv[1] = w4.x >> 16; wv[2] = w4.y & 0xffff; wv[3] = w4.y >> 16;
      wv[4] = w4.z & 0xffff; wv[5] = w4.z >> 16; wv[6] = w4.w & 0xffff; wv[7] = w4.w >> 16;
      float4 x0 = make_float4(0, 0, 0, 0), x1 = x0;
      if (xr >= 0) {
        x0 = *reinterpret_cast<const float4*>(xp + k);
        x1 = *reinterpret_cast<const float4*>(xp + k + 4);
      }
      xv[0] = x0.x; xv[1] = x0.y; xv[2] = x0.z; xv[3] = x0.w;
      xv[4] = x1.x; xv[5] = x1.y; xv[6] = x1.z; xv[7] = x1.w;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const bool in = k + i < K;
        wv[i] = (in && frow < a.rows) ? wp[k + i] : (unsigned short)0;
        xv[i] = (in && xr >= 0) ? xp[k + i] : 0.0f;
      }
    }
    {
      uint4 p;
      p.x = wv[0] | ((unsigned)wv[1] << 16); p.y = wv[2] | ((unsigned)wv[3] << 16);
      p.z = wv[4] | ((unsigned)wv[5] << 16); p.w = wv[6] | ((unsigned)wv[7] << 16);
      *reinterpret_cast<uint4*>(&Ws[lr][lk]) = p;
    }
#pragma unroll
    for (int t = 0; t < TERMS; ++t) {
      unsigned short h[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        h[i] = f2bf(xv[i]);
        xv[i] -= bf2f(h[i]);  // exact: the remainder of an FP32 value after its leading 8 bits
      }
      uint4 p;
      p.x = h[0] | ((unsigned)h[1] << 16); p.y = h[2] | ((unsigned)h[3] << 16);
      p.z = h[4] | ((unsigned)h[5] << 16); p.w = h[6] | ((unsigned)h[7] << 16);
      *reinterpret_cast<uint4*>(&Xs[t][lr][lk]) = p;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < BK / 8; ++ks) {
      const int kk = ks * 8 + (lane >> 5) * 4;
      const bf16x4 af = *reinterpret_cast<const bf16x4*>(&Ws[wm * 32 + (lane & 31)][kk]);
#pragma unroll
      for (int t = TERMS - 1; t >= 0; --t) {  // small terms first
        const bf16x4 bfr = *reinterpret_cast<const bf16x4*>(&Xs[t][wn * 32 + (lane & 31)][kk]);
        acc = __builtin_amdgcn_mfma_f32_32x32x8bf16_1k(af, bfr, acc, 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // C layout: lane holds token (lane & 31) of its wave's 32, features (i / 4) * 8 + (lane >> 5) * 4 + (i & 3)
  const int it = t0 + wn * 32 + (lane & 31);
  if (it < hi) {
    const int orow = a.y_rows ? a.y_rows[it] : it;
    float* yr = a.y + (size_t)orow * a.ldy;
    const bool v4 = (a.ldy & 3) == 0 && ((size_t)a.y & 15) == 0;
#pragma unroll
    for (int gq = 0; gq < 4; ++gq) {
      const int f = f0 + wm * 32 + gq * 8 + (lane >> 5) * 4;
      if (v4 && f + 4 <= a.rows) {
        *reinterpret_cast<float4*>(yr + f) = make_float4(acc[gq * 4], acc[gq * 4 + 1], acc[gq * 4 + 2], acc[gq * 4 + 3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (f + i < a.rows) yr[f + i] = acc[gq * 4 + i];
      }
    }
  }
}

// RW rows per wave, 4 waves per workgroup: 2 x RW sixteen-byte weight loads in flight per lane (tl_bf16.h)
template <int RW>
__global__ __launch_bounds__(256) void dense_gemv_kernel(const unsigned short* __restrict__ W, int rows, int cols,
                                                         const float* __restrict__ x, float* __restrict__ y, int vec) {
  const int lane = threadIdx.x & 63;
  const int row0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * RW;
  if (row0 >= rows) return;
  float out[RW];
  tl_wave_dot_rows<RW>(W + (size_t)row0 * cols, (size_t)cols, rows - row0, x, cols, vec != 0, lane, out);
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < RW; ++r)
      if (row0 + r < rows) y[row0 + r] = out[r];
  }
}

}  // namespace

int tl_launch_dense_gemm(const DenseArgs& a, hipStream_t s) {
  TL_REQUIRE(a.w && a.x && a.y && a.rows > 0 && a.cols > 0 && a.T > 0, "dense gemm: bad arguments");
  TL_REQUIRE(a.terms == 1 || a.terms == 3, "dense gemm: terms must be 1 or 3 (got %d)", a.terms);
  TL_REQUIRE(!a.x_rows || a.x_div >= 1, "dense gemm: x_div must be >= 1");
  const int groups = a.groups > 0 ? a.groups : 1;
  TL_REQUIRE(groups == 1 || a.group_off, "dense gemm: groups without group_off");
  dim3 grid((a.rows + BM - 1) / BM, (a.T + BN - 1) / BN, groups);
  TL_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "dense gemm: launch too large");
  if (a.terms == 1) dense_gemm_kernel<1><<<grid, 256, 0, s>>>(a);
  else dense_gemm_kernel<3><<<grid, 256, 0, s>>>(a);
  TL_HIP(hipGetLastError());
  return 0;
}

int tl_launch_dense_gemv(const uint16_t* w, int rows, int cols, const float* x, float* y, hipStream_t s) {
  TL_REQUIRE(w && x && y && rows > 0 && cols > 0, "dense gemv: bad arguments");
  const int vec = (cols & 7) == 0 && ((size_t)x & 15) == 0 && ((size_t)w & 15) == 0;
  // rows per wave: as many as still leave every CU a few workgroups
  const int cus = tl_num_cus();
  if (rows >= 16 * 4 * cus) dense_gemv_kernel<4><<<(rows + 15) / 16, 256, 0, s>>>(w, rows, cols, x, y, vec);
  else if (rows >= 8 * 4 * cus) dense_gemv_kernel<2><<<(rows + 7) / 8, 256, 0, s>>>(w, rows, cols, x, y, vec);
  else dense_gemv_kernel<1><<<(rows + 3) / 4, 256, 0, s>>>(w, rows, cols, x, y, vec);
  TL_HIP(hipGetLastError());
  return 0;
}

extern "C" int tl_dense_matmul(const void* w_bf16_dev, int rows, int cols, const float* x_dev, float* y_dev, int num_tokens,
                               int terms, void* stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (terms == 0) {
    TL_REQUIRE(num_tokens == 1, "tl_dense_matmul: terms 0 (FP32 GEMV) takes one token, not %d", num_tokens);
    return tl_launch_dense_gemv(static_cast<const uint16_t*>(w_bf16_dev), rows, cols, x_dev, y_dev, s);
  }
  DenseArgs a = {};
  a.w = static_cast<const uint16_t*>(w_bf16_dev);
  a.rows = rows;
  a.cols = cols;
  a.x = x_dev;
  a.ldx = cols;
  a.y = y_dev;
  a.ldy = rows;
  a.T = num_tokens;
  a.terms = terms;
  return tl_launch_dense_gemm(a, s);
}
