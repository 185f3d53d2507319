/*
 * memref.h -- the strided memref descriptor that crosses the C ABI.
 *
 * Layout-identical to buddy-mlir's MemRef<T,N>
 * (frontend/Interfaces/buddy/Core/Container.h:126-137: allocated, aligned,
 * offset, sizes[N], strides[N]; no virtual members) and therefore to the
 * struct MLIR's `llvm.emit_c_interface` wrappers pass by pointer
 * (runtime/include/buddy/runtime/Matmul.h:17-22).  Strides are in elements.
 * The element address of index (i0..iN-1) is aligned + offset + sum(i*stride).
 * sizeof == 24 + 16*N bytes.
 */
#ifndef BUDDY_HIP_MEMREF_H
#define BUDDY_HIP_MEMREF_H

#include <stddef.h>
#include <stdint.h>

#define BUDDY_HIP_DECLARE_MEMREF(NAME, T, RANK)                                \
  typedef struct NAME {                                                        \
    T *allocated;                                                              \
    T *aligned;                                                                \
    intptr_t offset;                                                           \
    intptr_t sizes[RANK];                                                      \
    intptr_t strides[RANK];                                                    \
  } NAME

BUDDY_HIP_DECLARE_MEMREF(buddy_memref_f32_1d, float, 1);
BUDDY_HIP_DECLARE_MEMREF(buddy_memref_f32_2d, float, 2);
BUDDY_HIP_DECLARE_MEMREF(buddy_memref_f32_3d, float, 3);
BUDDY_HIP_DECLARE_MEMREF(buddy_memref_f32_4d, float, 4);
BUDDY_HIP_DECLARE_MEMREF(buddy_memref_i8_1d, int8_t, 1);
BUDDY_HIP_DECLARE_MEMREF(buddy_memref_i8_2d, int8_t, 2);
BUDDY_HIP_DECLARE_MEMREF(buddy_memref_i64_1d, long long, 1);
BUDDY_HIP_DECLARE_MEMREF(buddy_memref_i64_2d, long long, 2);

#ifdef __cplusplus
static_assert(sizeof(buddy_memref_f32_1d) == 24 + 16 * 1, "memref<1> layout");
static_assert(sizeof(buddy_memref_f32_2d) == 24 + 16 * 2, "memref<2> layout");
static_assert(sizeof(buddy_memref_f32_3d) == 24 + 16 * 3, "memref<3> layout");
static_assert(sizeof(buddy_memref_f32_4d) == 24 + 16 * 4, "memref<4> layout");
static_assert(offsetof(buddy_memref_f32_2d, sizes) == 24, "memref sizes at 24");
#endif

#endif /* BUDDY_HIP_MEMREF_H */
