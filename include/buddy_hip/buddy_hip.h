/*
 * buddy_hip.h -- C ABI of libbuddy_hip.so: buddy-mlir's int8 weight-only
 * (w8a32) LLM decode / prefill arithmetic as hand-written HIP kernels for
 * gfx950 (MI355X).
 *
 * Two layers are exported.
 *
 *  (1) `_mlir_ciface_*` entry points that take pointers to memref descriptors,
 *      the convention of buddy-mlir's external kernels
 *      (runtime/include/buddy/runtime/Matmul.h:35-36,
 *      runtime/external_kernels/matmul/MatmulTorq.cpp:116-166) and of the
 *      compiled model library (tools/buddy-codegen/gen_session.py:974-1007).
 *      Data pointers may be host or device memory.
 *
 *  (2) `buddy_hip_*` entry points that take plain device pointers and sizes
 *      and launch on a caller-supplied HIP stream.  They are what layer (1)
 *      is built from and what a resident-weights caller uses directly.
 *
 * Every function returns 0 on success and a non-zero code on failure unless it
 * is `void` by the reference's convention; failures also print one
 * `[buddy_hip] ...` line to stderr and are queryable with
 * buddy_hip_last_error().  Nothing unwinds through this boundary.
 * Calls on one stream are ordered.
 */
#ifndef BUDDY_HIP_H
#define BUDDY_HIP_H

#include "buddy_hip/memref.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef void *buddy_hip_stream; /* a hipStream_t; NULL = the default stream */

enum {
  BUDDY_HIP_OK = 0,
  BUDDY_HIP_ERR_ARG = 1,     /* shape / pointer / size check failed */
  BUDDY_HIP_ERR_HIP = 2,     /* a HIP runtime call failed */
  BUDDY_HIP_ERR_NO_DEVICE = 3
};

/* ---- library ---------------------------------------------------------- */
const char *buddy_hip_version(void);
const char *buddy_hip_last_error(void);
int buddy_hip_device_count(void);

/* ---- packed int8 weight layout ("wave tiles") --------------------------
 * Replaces frontend/Python/graph/transform/pack_decode_weights.py:102-108
 * (panels [N/V][K][V], refused for int8 by tools/buddy-codegen/gen_config.py:
 * 366-370) with a layout cut for 64-lane wavefronts issuing 128-bit loads:
 * the matrix W[K,N] is padded to Kp = ceil64(K), Np = ceil16(N) and stored as
 * tiles of 16 output channels x 64 k (1 KiB).  Tile (g = n/16, c = k/64) is at
 * byte ((g * Kp/64) + c) * 1024; inside it lane L (0..63) owns 16 consecutive
 * bytes holding k = c*64 + (L/16)*16 + 0..15 of channel n = g*16 + L%16.
 * A wavefront's one load instruction therefore reads one contiguous KiB and a
 * channel group's whole K extent is one contiguous run.  Padding is zero. */
size_t buddy_hip_w8_packed_bytes(int64_t K, int64_t N);
/* W: device int8 [K,N] row-major (the reference layout).  packed: device. */
int buddy_hip_pack_w8(const int8_t *W, int64_t K, int64_t N, int8_t *packed,
                      buddy_hip_stream stream);
int buddy_hip_unpack_w8(const int8_t *packed, int64_t K, int64_t N, int8_t *W,
                        buddy_hip_stream stream);

/* ---- per-output-channel symmetric quantizer ----------------------------
 * tools/buddy-codegen/import_model.py:837-848,874-880 on device: W f32 [K,N],
 * q int8 [K,N], scale f32 [N].  Bit-exact with the reference recipe. */
int buddy_hip_quantize_w8(const float *W, int64_t K, int64_t N, int8_t *q,
                          float *scale, buddy_hip_stream stream);

/* ---- int8 dequant decode GEMV / small-batch matmul ---------------------
 * Replaces the kernel that
 * midend/lib/Conversion/MatMulOptimization/DequantMatMulVectorizationDecode.cpp
 * :250-321 generates:  C[m,n] (+)= (sum_k A[m,k] * W[k,n]) * scale[n].
 * M is 1..16 (the reference pattern is m == 1 only; M > 1 streams the weights
 * once for all rows).  A: f32 [M,K] row-major (lda = K), C: f32 [M,N]. */
enum {
  BUDDY_HIP_GEMV_ACCUMULATE = 1 /* C += ...  (linalg.matmul semantics);
                                   without it C = ... and C need not be
                                   initialised */
};
int buddy_hip_gemv_w8a32(const float *A, const int8_t *packed,
                         const float *scale, float *C, int64_t M, int64_t K,
                         int64_t N, unsigned flags, buddy_hip_stream stream);

/* ---- plain f32 matmul ---------------------------------------------------
 * C (+)= A[M,K] * B[K,N], all dense row-major device pointers.  The f32
 * sibling of the kernel above (MatMulVectorizationDecode.cpp:142-175); the
 * reference's shipped w8a32 build keeps q/k/v projections in f32. */
int buddy_hip_matmul_f32(const float *A, const float *B, float *C, int64_t M,
                         int64_t N, int64_t K, unsigned flags,
                         buddy_hip_stream stream);

/* ---- operator-level memref entry points --------------------------------
 * result = A * B, f32.  Same symbol and contract as
 * runtime/external_kernels/matmul/MatmulTorq.cpp:116-166: `result` is an
 * uninitialised descriptor; the callee malloc()s M*N floats and fills it;
 * strided inputs are honoured. */
void _mlir_ciface_buddy_matmul_f32(buddy_memref_f32_2d *result,
                                   buddy_memref_f32_2d *A,
                                   buddy_memref_f32_2d *B);
/* result = A * (sitofp(W) (.) scale), W int8 [K,N], scale f32 [1,N] or [N,1]
 * viewed as N values.  New symbol in the same convention (the reference has no
 * int8 external kernel: runtime/external_kernels/CMakeLists.txt:5-9); it
 * stands for the sitofp -> mulf -> linalg.matmul chain that
 * DequantMatMulVectorizationDecode.cpp:93-189 matches.  The packed device copy
 * of W is cached by (W pointer, K, N) because weights are immutable after
 * loadWeights (tools/buddy-codegen/gen_session.py:1301-1331). */
void _mlir_ciface_buddy_dequant_matmul_i8_f32(buddy_memref_f32_2d *result,
                                              buddy_memref_f32_2d *A,
                                              buddy_memref_i8_2d *W,
                                              buddy_memref_f32_2d *scale);
/* C += A * (sitofp(W) (.) scale) in place: linalg.matmul's accumulate-into-
 * outs semantics (DequantMatMulVectorizationDecode.cpp:313-320). */
void _mlir_ciface_buddy_dequant_matmul_i8_f32_acc(buddy_memref_f32_2d *C,
                                                  buddy_memref_f32_2d *A,
                                                  buddy_memref_i8_2d *W,
                                                  buddy_memref_f32_2d *scale);
/* Drops every cached device copy made by the entry points above. */
void buddy_hip_clear_weight_cache(void);

#ifdef __cplusplus
}
#endif
#endif /* BUDDY_HIP_H */
