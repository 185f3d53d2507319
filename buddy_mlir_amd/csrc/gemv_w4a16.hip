// gemv_w4a16.hip -- the reference's int4 weight-only decode GEMV (W4A16).
//
// Replaces the kernel that
// midend/lib/Conversion/MatMulOptimization/Int4DequantMatMulVectorizationDecode.cpp
// :385-468 generates: C[n] = C[n] + (sum_k a[k] * w[k][n]) * scale[n] with f16
// activations, scales, accumulator and output, int4 weights packed two per
// byte along n ([K, N/2] bytes: low nibble = even channel, high = odd;
// tools/buddy-codegen/import_model.py:810-815), and the nibble packing itself.
//
// The reference accumulates in f16, k in order: every step rounds to 11
// significand bits, so a kernel that sums in another order (or in f32) does not
// reproduce its results to 1e-3.  The kernels here therefore keep the reference's
// order: one thread walks k for a channel, rounding the f32 fused multiply-add
// to f16 after every step, which is exactly what f16 arithmetic is on the
// reference's x86 target.  The result equals the reference's bit for bit; the
// price is a chain of K dependent roundings per channel, so the launch time is
// K times the time of one step, not the bytes it reads.
#include "common.h"

namespace bh {
namespace {

typedef unsigned short u16;

__device__ __forceinline__ float f16_bits_to_f32(u16 h) {
  union {
    u16 u;
    _Float16 f;
  } x;
  x.u = h;
  return (float)x.f;
}
__device__ __forceinline__ float round_to_f16(float v) { return (float)(_Float16)v; }
__device__ __forceinline__ u16 f32_to_f16_bits(float v) {
  union {
    u16 u;
    _Float16 f;
  } x;
  x.f = (_Float16)v;
  return x.u;
}

constexpr int kThreads = 64;
constexpr int kStage = 2048; // activations staged per round

__global__ void __launch_bounds__(kThreads)
w4a16_gemv_kernel(const u16 *__restrict__ a, const int8_t *__restrict__ packed,
                  const u16 *__restrict__ scale, u16 *__restrict__ c, int K, int N,
                  int first_col) {
#pragma clang fp contract(off)
  __shared__ float a_s[kStage];
  const int cols = N / 2;
  const int j = first_col + blockIdx.x * kThreads + threadIdx.x;
  const bool live = j < cols;
  const int8_t *col = packed + (live ? j : 0);
  float acc0 = 0.f, acc1 = 0.f; // always exactly representable in f16
  for (int k0 = 0; k0 < K; k0 += kStage) {
    const int kn = min(kStage, K - k0);
    __syncthreads();
    for (int i = threadIdx.x; i < kn; i += kThreads)
      a_s[i] = f16_bits_to_f32(a[k0 + i]);
    __syncthreads();
    constexpr int U = 8;
    for (int kk = 0; kk < kn; kk += U) {
      int b[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        b[u] = col[(size_t)(k0 + min(kk + u, kn - 1)) * cols];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (kk + u < kn) {
          // low = ((b & 0x0F) << 4) >> 4, high = b >> 4 (arithmetic, 8 bits)
          const float lo = (float)((int)((unsigned)b[u] << 28) >> 28);
          const float hi = (float)((int)((unsigned)b[u] << 24) >> 28);
          const float x = a_s[kk + u];
          acc0 = round_to_f16(fmaf(x, lo, acc0));
          acc1 = round_to_f16(fmaf(x, hi, acc1));
        }
      }
    }
  }
  if (!live)
    return;
  const int n = 2 * j;
  const float s0 = round_to_f16(acc0 * f16_bits_to_f32(scale[n]));
  const float s1 = round_to_f16(acc1 * f16_bits_to_f32(scale[n + 1]));
  c[n] = f32_to_f16_bits(f16_bits_to_f32(c[n]) + s0);
  c[n + 1] = f32_to_f16_bits(f16_bits_to_f32(c[n + 1]) + s1);
}

// The same arithmetic with the chain of dependent roundings as (nearly) the only
// thing its wavefront does.  A workgroup owns 64 channels (32 byte columns).
// Wavefront 0 walks k for them, one channel per lane.  A step is one
// v_fma_mixlo_f16: f16 operands taken from either half of a register, f32
// multiply-add, one rounding to f16 -- the reference's step as one instruction.
// Its operands: the activations of a whole block of 256 rows sit in registers
// (read from LDS once per block, the same for every lane), and one LDS read
// brings the lane's weights of two consecutive rows, already widened to f16;
// the reads for the next 16 steps are issued before the chain of these 16.
// Wavefronts 1..3 prepare the block of rows after the one being consumed: a lane
// reads four packed bytes of each of two consecutive rows (a wavefront: 16 whole
// rows of the block per pair of loads), widens the 16 nibbles to f16 and stores
// them as 32 contiguous bytes of the block, laid out [row pair][channel][2].  The
// bytes are requested a whole block ahead of their decoding.  One barrier per
// block of rows.
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
constexpr int kChainRows = 256; // rows per block
constexpr int kChainChannels = 64;

__global__ void __launch_bounds__(256)
w4a16_gemv_chain_kernel(const u16 *__restrict__ a, const int8_t *__restrict__ packed,
                        const u16 *__restrict__ scale, u16 *__restrict__ c, int K, int N) {
#pragma clang fp contract(off)
  // [row pair][channel] of (even row, odd row)
  __shared__ __attribute__((aligned(16))) half2v w_s[2][kChainRows / 2 * kChainChannels];
  __shared__ __attribute__((aligned(16))) _Float16 x_s[2][kChainRows];
  const int cols = N / 2;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col0 = blockIdx.x * (kChainChannels / 2);
  const int nblocks = (K + kChainRows - 1) / kChainRows;

  // producer lane: row pair (lane / 8) of a group of 16 rows, bytes 4 (lane % 8) ..
  // + 3 of the block's 32 byte columns = channels 8 (lane % 8) .. + 7.  Groups
  // g = wave - 1, wave + 2, ... of the block's 16: at most 6 per wavefront.
  constexpr int kGroups = kChainRows / 16;
  constexpr int kTasks = (kGroups + 2) / 3;
  struct Raw {
    int b[kTasks][2];
    u16 x[kChainRows / 64];
  };
  const int ppair = lane >> 3, pcol = lane & 7;
  // four bytes at once where rows are 4-byte aligned, byte by byte otherwise
  const bool aligned4 =
      ((reinterpret_cast<uintptr_t>(packed) | (unsigned)cols | (unsigned)col0) & 3) == 0;
  auto request = [&](int blk, Raw &raw) {
    const int k0 = blk * kChainRows;
#pragma unroll
    for (int t = 0; t < kTasks; ++t) {
      const int g = min(wave - 1 + 3 * t, kGroups - 1);
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int8_t *p =
            packed + (size_t)min(k0 + g * 16 + ppair * 2 + e, K - 1) * cols + col0 + pcol * 4;
        if (aligned4) {
          raw.b[t][e] = *reinterpret_cast<const int *>(p);
        } else {
          raw.b[t][e] =
              (int)((unsigned)(unsigned char)p[0] | ((unsigned)(unsigned char)p[1] << 8) |
                    ((unsigned)(unsigned char)p[2] << 16) | ((unsigned)(unsigned char)p[3] << 24));
        }
      }
    }
    if (wave == 1) {
#pragma unroll
      for (int i = 0; i < kChainRows / 64; ++i)
        raw.x[i] = a[min(k0 + i * 64 + lane, K - 1)];
    }
  };
  auto decode = [&](const Raw &raw, int buf) {
#pragma unroll
    for (int t = 0; t < kTasks; ++t) {
      const int g = wave - 1 + 3 * t;
      if (g < kGroups) {
        half8 h[2]; // channels 8 pcol .. + 3 and + 4 .. + 7, (even row, odd row) each
#pragma unroll
        for (int j = 0; j < 8; ++j) { // nibble j: low nibble of a byte = the even channel
          h[j / 4][2 * (j % 4)] =
              (_Float16)(short)((int)((unsigned)raw.b[t][0] << (28 - 4 * j)) >> 28);
          h[j / 4][2 * (j % 4) + 1] =
              (_Float16)(short)((int)((unsigned)raw.b[t][1] << (28 - 4 * j)) >> 28);
        }
        half8 *dst = reinterpret_cast<half8 *>(
            &w_s[buf][(g * 8 + ppair) * kChainChannels + pcol * 8]);
        dst[0] = h[0];
        dst[1] = h[1];
      }
    }
    if (wave == 1) {
#pragma unroll
      for (int i = 0; i < kChainRows / 64; ++i) {
        union {
          u16 u;
          _Float16 f;
        } v;
        v.u = raw.x[i];
        x_s[buf][i * 64 + lane] = v.f;
      }
    }
  };

  _Float16 acc = (_Float16)0.0f;
  Raw raw0, raw1; // block blk + 1 being decoded, block blk + 2 in flight (they swap)
  if (wave != 0) {
    request(0, raw0);
    decode(raw0, 0);
    request(1, raw0);
  }
  __syncthreads();
  for (int blk = 0; blk < nblocks; ++blk) {
    const int buf = blk & 1;
    if (wave != 0) {
      // (a request past the last block rereads clamped rows: always the same
      // number of loads, so that waiting for the older set leaves the newer in flight)
      if (buf == 0) {
        request(blk + 2, raw1);
        if (blk + 1 < nblocks)
          decode(raw0, 1);
      } else {
        request(blk + 2, raw0);
        if (blk + 1 < nblocks)
          decode(raw1, 0);
      }
    } else {
      const int kn = min(kChainRows, K - blk * kChainRows);
      const half2v *wcol = &w_s[buf][lane];
      // the block's activations: 32 reads, the same address in every lane
      half8 x[kChainRows / 8];
#pragma unroll
      for (int q = 0; q < kChainRows / 8; ++q)
        x[q] = *reinterpret_cast<const half8 *>(&x_s[buf][q * 8]);
      // keep them in registers: left alone, the compiler reads each one again
      // from LDS right before its use and the chain waits for that read
#pragma unroll
      for (int q = 0; q < kChainRows / 8; ++q)
        asm volatile("" : "+v"(x[q]));
      if (kn == kChainRows) {
        half2v w[8];
#pragma unroll
        for (int r = 0; r < 8; ++r)
          w[r] = wcol[r * kChainChannels];
#pragma unroll
        for (int q = 0; q < kChainRows / 16; ++q) { // 16 steps
          half2v v[8];
          const int nq = q + 1 < kChainRows / 16 ? q + 1 : q; // after the last: reread it
#pragma unroll
          for (int r = 0; r < 8; ++r)
            v[r] = wcol[(nq * 8 + r) * kChainChannels];
#pragma unroll
          for (int r = 0; r < 8; ++r) {
            acc = (_Float16)fmaf((float)x[2 * q + r / 4][2 * (r % 4)], (float)w[r][0], (float)acc);
            acc = (_Float16)fmaf((float)x[2 * q + r / 4][2 * (r % 4) + 1], (float)w[r][1],
                                 (float)acc);
          }
#pragma unroll
          for (int r = 0; r < 8; ++r)
            w[r] = v[r];
        }
      } else { // the ragged last block
        for (int kk = 0; kk < kn; ++kk) {
          const half2v w = wcol[(kk >> 1) * kChainChannels];
          acc = (_Float16)fmaf((float)x_s[buf][kk], (float)w[kk & 1], (float)acc);
        }
      }
    }
    __syncthreads();
  }
  if (wave != 0)
    return;
  const int n = 2 * col0 + lane;
  const float s = round_to_f16((float)acc * f16_bits_to_f32(scale[n]));
  c[n] = f32_to_f16_bits(f16_bits_to_f32(c[n]) + s);
}

// two int4 (stored as int8 in [-8, 7]) per byte, element 2i low, 2i+1 high
__global__ void __launch_bounds__(256)
pack_int4_kernel(const int8_t *__restrict__ q, int64_t pairs, int8_t *__restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= pairs)
    return;
  const unsigned lo = (unsigned)q[2 * i] & 0x0Fu, hi = ((unsigned)q[2 * i + 1] & 0x0Fu) << 4;
  out[i] = (int8_t)(lo | hi);
}

} // namespace
} // namespace bh

extern "C" {

int buddy_hip_pack_int4(const int8_t *q, int64_t count, int8_t *packed,
                        buddy_hip_stream stream) try {
  BH_REQUIRE(q && packed && count > 0, "pack_int4: bad argument");
  BH_REQUIRE(count % 2 == 0, "pack_int4: odd element count %lld", (long long)count);
  hipLaunchKernelGGL(bh::pack_int4_kernel, dim3((unsigned)bh::ceil_div(count / 2, 256)),
                     dim3(256), 0, bh::as_stream(stream), q, count / 2, packed);
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_pack_int4")

int buddy_hip_gemv_w4a16(const uint16_t *A, const int8_t *packed, const uint16_t *scale,
                         uint16_t *C, int64_t K, int64_t N, buddy_hip_stream stream) try {
  BH_REQUIRE(A && packed && scale && C, "gemv_w4a16: null pointer");
  BH_REQUIRE(K > 0 && N > 0 && K < (1 << 30) && N < (1 << 30),
             "gemv_w4a16: bad shape K=%lld N=%lld", (long long)K, (long long)N);
  BH_REQUIRE(N % 2 == 0, "gemv_w4a16: N=%lld is odd (two channels per byte)",
             (long long)N);
  // full blocks of 64 byte columns with 16-byte readable rows take the blocked
  // kernel, the ragged rest (or everything, if rows are not aligned) the plain one
  const int64_t cols = N / 2;
  // whole blocks of 32 byte columns take the kernel whose chain wavefront does
  // nothing but the chain; the ragged rest the plain one
  const int64_t blocked = cols / 32 * 32;
  if (blocked) {
    hipLaunchKernelGGL(bh::w4a16_gemv_chain_kernel, dim3((unsigned)(blocked / 32)), dim3(256), 0,
                       bh::as_stream(stream), A, packed, scale, C, (int)K, (int)N);
  }
  if (blocked < cols) {
    hipLaunchKernelGGL(bh::w4a16_gemv_kernel,
                       dim3((unsigned)bh::ceil_div(cols - blocked, bh::kThreads)),
                       dim3(bh::kThreads), 0, bh::as_stream(stream), A, packed, scale, C,
                       (int)K, (int)N, (int)blocked);
  }
  BH_CHECK_HIP(hipGetLastError());
  return BUDDY_HIP_OK;
} BH_CATCH_INT("buddy_hip_gemv_w4a16")
}
