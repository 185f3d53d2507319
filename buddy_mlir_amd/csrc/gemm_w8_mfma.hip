// gemm_w8_mfma.hip -- prefill matmul: C[M,N] (+)= A[M,K] . (int8 W[K,N] * scale)
// on the bf16 matrix cores.
//
// Replaces the BLIS-style kernel with dequantisation fused into B packing that
// midend/lib/Conversion/MatMulOptimization/MatMulBlisVectorization.cpp:351-360,
// 398-986 generates for M > 1.
//
// Shape of the kernel:
//  * the weights are read from the same wave-tile packed copy the decode GEMV
//    streams (one resident copy serves prefill and decode);
//  * a workgroup owns a 128 x 128 tile of C; per 64-wide k slab it converts the
//    int8 tile to bf16 while storing it to LDS (|q| <= 128 is exact in bf16; the
//    per-channel scale is applied once to the f32 accumulators, where the
//    reference multiplies every element before the FMA) and the f32 activations
//    to bf16 (one, two or three bf16 terms: one term is "activations cast to
//    bf16", three terms carry all 24 significand bits of the f32 input);
//  * four wavefronts each hold a 64 x 64 block of C as 2 x 2 MFMA 32x32x16 bf16
//    accumulators (f32), fragments come from LDS with 16-byte reads;
//  * the next slab's global loads are in flight while the current slab is
//    multiplied.
#include "gemm.h"

namespace bh {
namespace {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDSK = BK + 8; // bf16 elements per LDS row, padded against conflicts

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned short u16;

__device__ __forceinline__ u16 bf16_rne(float x) {
  unsigned u = __float_as_uint(x);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (u16)(u >> 16);
}
__device__ __forceinline__ float bf16_to_f32(u16 b) {
  return __uint_as_float((unsigned)b << 16);
}
__device__ __forceinline__ unsigned pack2(u16 lo, u16 hi) {
  return (unsigned)lo | ((unsigned)hi << 16);
}
// two int8 (bytes j, j+1 of v) -> two exact bf16
__device__ __forceinline__ unsigned q2_to_bf16x2(int v, int j) {
  const float a = (float)(signed char)(v >> (8 * j));
  const float b = (float)(signed char)(v >> (8 * j + 8));
  return (__float_as_uint(a) >> 16) | (__float_as_uint(b) & 0xffff0000u);
}

struct GemmArgs {
  const float *A;
  const int4 *W;
  const float *scale;
  const float *bias;
  float *C;
  int64_t lda, ldc;
  int M, K, N, groups, chunks;
  int accumulate;
};

template <int TERMS>
__global__ void __launch_bounds__(256) gemm_w8_bf16_kernel(GemmArgs a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  u16(*As)[BM][LDSK] = reinterpret_cast<u16(*)[BM][LDSK]>(smem);
  u16(*Bs)[LDSK] = reinterpret_cast<u16(*)[LDSK]>(smem + sizeof(u16) * TERMS * BM * LDSK);

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int wm = wave >> 1, wn = wave & 1;

  // global -> register staging assignments
  const int arow = tid >> 1, ahalf = tid & 1;   // A: 32 consecutive k of a row
  const int btile = tid >> 6;                   // B: tiles btile and btile + 4
  const int bch = lane & 15, bkg = lane >> 4;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e)
        acc[i][j][e] = 0.f;

  float4 areg[8];
  int4 breg[2];
  auto load_global = [&](int c) {
    const int k0 = c * BK + ahalf * 32;
    const int m = m0 + arow;
    const float *src = a.A + (int64_t)m * a.lda + k0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int k = k0 + i * 4;
      if (m < a.M && k + 3 < a.K && ((reinterpret_cast<uintptr_t>(src + i * 4) & 15) == 0))
        areg[i] = *reinterpret_cast<const float4 *>(src + i * 4);
      else if (m < a.M)
        areg[i] = make_float4(k < a.K ? src[i * 4] : 0.f,
                              k + 1 < a.K ? src[i * 4 + 1] : 0.f,
                              k + 2 < a.K ? src[i * 4 + 2] : 0.f,
                              k + 3 < a.K ? src[i * 4 + 3] : 0.f);
      else
        areg[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int g = n0 / 16 + btile + 4 * t;
      breg[t] = g < a.groups ? a.W[((size_t)g * a.chunks + c) * 64 + lane]
                             : make_int4(0, 0, 0, 0);
    }
  };
  auto store_lds = [&]() {
    // A: f32 -> TERMS bf16 terms
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      const float v[8] = {areg[i].x, areg[i].y, areg[i].z, areg[i].w,
                          areg[i + 1].x, areg[i + 1].y, areg[i + 1].z, areg[i + 1].w};
      float r[8];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        r[e] = v[e];
#pragma unroll
      for (int t = 0; t < TERMS; ++t) {
        u16 h[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          h[e] = bf16_rne(r[e]);
          r[e] = r[e] - bf16_to_f32(h[e]);
        }
        *reinterpret_cast<uint4 *>(&As[t][arow][ahalf * 32 + i * 4]) =
            make_uint4(pack2(h[0], h[1]), pack2(h[2], h[3]), pack2(h[4], h[5]),
                       pack2(h[6], h[7]));
      }
    }
    // B: int8 -> bf16, row = channel, 16 consecutive k
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int ch = (btile + 4 * t) * 16 + bch;
      const int4 w = breg[t];
      uint4 lo = make_uint4(q2_to_bf16x2(w.x, 0), q2_to_bf16x2(w.x, 2),
                            q2_to_bf16x2(w.y, 0), q2_to_bf16x2(w.y, 2));
      uint4 hi = make_uint4(q2_to_bf16x2(w.z, 0), q2_to_bf16x2(w.z, 2),
                            q2_to_bf16x2(w.w, 0), q2_to_bf16x2(w.w, 2));
      *reinterpret_cast<uint4 *>(&Bs[ch][bkg * 16]) = lo;
      *reinterpret_cast<uint4 *>(&Bs[ch][bkg * 16 + 8]) = hi;
    }
  };

  load_global(0);
  for (int c = 0; c < a.chunks; ++c) {
    __syncthreads(); // previous slab fully consumed
    store_lds();
    __syncthreads();
    if (c + 1 < a.chunks)
      load_global(c + 1);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      const int kk = ks * 16 + (lane >> 5) * 8;
      bf16x8 bf[2];
#pragma unroll
      for (int j = 0; j < 2; ++j)
        bf[j] = *reinterpret_cast<const bf16x8 *>(&Bs[wn * 64 + j * 32 + (lane & 31)][kk]);
#pragma unroll
      for (int t = 0; t < TERMS; ++t) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const bf16x8 af =
              *reinterpret_cast<const bf16x8 *>(&As[t][wm * 64 + i * 32 + (lane & 31)][kk]);
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bf[j], acc[i][j], 0, 0, 0);
        }
      }
    }
  }

  // epilogue: scale per channel, optional bias / accumulate
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int n = n0 + wn * 64 + j * 32 + (lane & 31);
    if (n >= a.N)
      continue;
    const float s = a.scale[n];
    const float b = a.bias ? a.bias[n] : 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m0 + wm * 64 + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (m < a.M) {
          float *c = a.C + (int64_t)m * a.ldc + n;
          const float v = acc[i][j][e] * s;
          *c = a.accumulate ? *c + v : b + v;
        }
      }
    }
  }
}

template <int TERMS>
int launch_terms(const GemmArgs &a, dim3 grid, hipStream_t stream) {
  constexpr size_t lds = sizeof(u16) * LDSK * (size_t)(TERMS * BM + BN);
  auto kernel = gemm_w8_bf16_kernel<TERMS>;
  static bool attr_set = false;
  if (!attr_set) {
    BH_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize,
                                     (int)lds));
    attr_set = true;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(256), lds, stream, a);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
}

} // namespace

int launch_gemm_w8(const GemmW8Args &in, hipStream_t stream) {
  BH_REQUIRE(in.A && in.W && in.scale && in.C, "gemm_w8: null pointer");
  BH_REQUIRE(in.M > 0 && in.K > 0 && in.N > 0 && in.M < (1 << 30) &&
                 in.K < (1 << 30) && in.N < (1 << 30),
             "gemm_w8: bad shape M=%lld K=%lld N=%lld", (long long)in.M,
             (long long)in.K, (long long)in.N);
  BH_REQUIRE(in.lda >= in.K && in.ldc >= in.N, "gemm_w8: row stride below row length");
  BH_REQUIRE(in.terms >= 1 && in.terms <= 3, "gemm_w8: terms=%d outside 1..3", in.terms);
  BH_REQUIRE(!(in.bias && in.accumulate), "gemm_w8: bias with accumulate");
  BH_REQUIRE((reinterpret_cast<uintptr_t>(in.W) & 15) == 0,
             "gemm_w8: packed weights must be 16-byte aligned");
  GemmArgs a;
  a.A = in.A;
  a.W = reinterpret_cast<const int4 *>(in.W);
  a.scale = in.scale;
  a.bias = in.bias;
  a.C = in.C;
  a.lda = in.lda;
  a.ldc = in.ldc;
  a.M = (int)in.M;
  a.K = (int)in.K;
  a.N = (int)in.N;
  a.groups = (int)ceil_div(in.N, kTileN);
  a.chunks = (int)ceil_div(in.K, kTileK);
  a.accumulate = in.accumulate ? 1 : 0;
  const dim3 grid((unsigned)ceil_div(in.N, BN), (unsigned)ceil_div(in.M, BM));
  switch (in.terms) {
  case 1: return launch_terms<1>(a, grid, stream);
  case 2: return launch_terms<2>(a, grid, stream);
  default: return launch_terms<3>(a, grid, stream);
  }
}

} // namespace bh

extern "C" {

int buddy_hip_gemm_w8a32(const float *A, const int8_t *packed, const float *scale,
                         float *C, int64_t M, int64_t K, int64_t N,
                         unsigned flags, buddy_hip_stream stream) {
  bh::GemmW8Args a;
  a.A = A;
  a.lda = K;
  a.W = packed;
  a.scale = scale;
  a.C = C;
  a.ldc = N;
  a.M = M;
  a.K = K;
  a.N = N;
  a.accumulate = (flags & BUDDY_HIP_GEMV_ACCUMULATE) != 0;
  a.terms = (flags & BUDDY_HIP_GEMM_A_F32_EXACT) ? 3 : 1;
  return bh::launch_gemm_w8(a, bh::as_stream(stream));
}
}
