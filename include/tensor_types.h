/*
 * Scalar and handle types shared by the host side and the gfx950 device library.
 *
 * Replaces the reference's src/cuda/tensor_types.h:1-100 and the StreamContext /
 * PaddedPtr declarations of src/cuda/kernel_header.h:10-17 for the HIP build:
 *   - len_t stays `unsigned long` (tensor_types.h:5);
 *   - r16/r32/r64 keep their storage size (tensor_types.h:20-33); on the C side
 *     r16 is an opaque 2-byte struct, on the device side it is _Float16;
 *   - StreamContext keeps its 16-byte, two-pointer, pass-by-value layout; slot 0 now
 *     carries a hipStream_t, slot 1 the BLAS state of the stream (see below), NULL for a
 *     stream that has none.
 *   - WAVE_SIZE is 64 (the reference's WARP_SIZE = 32, tensor_types.h:6).
 */
#ifndef MP_TENSOR_TYPES_H
#define MP_TENSOR_TYPES_H

#include <stdint.h>

#define MAX_DIMS 6
typedef unsigned long len_t;

#define MP_WAVE_SIZE 64

/* dtype keys in the order of the reference's scalar.Tag (src/core/scalar.zig:35-40),
 * which is also the order of every generated dispatch array. */
#define MP_R16 0
#define MP_R32 1
#define MP_R64 2

#if defined(__HIPCC__)
typedef _Float16 r16;
#else
typedef struct { unsigned short x_; } r16;
#endif
typedef float  r32;
typedef double r64;

typedef struct { void* ptr; } PaddedPtr;

typedef struct {
  PaddedPtr hip_stream;   /* hipStream_t */
  PaddedPtr blas_handle;  /* BLAS state (handle + workspace) made by mpInitStream / mpAdoptStream; NULL for a borrowed stream */
} StreamContext;

/* SELU constants of the fused-chain workload (self-normalising networks' alpha and
 * scale, truncated as the workload definition states them). */
#define MP_SELU_ALPHA 1.6732632
#define MP_SELU_SCALE 1.0507010

#endif
