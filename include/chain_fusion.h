/*
 * Elementwise expressions fused at run time (lib/libmp_fusion.so).
 *
 * No counterpart in the reference: there every elementwise op is one launch through one temporary
 * (src/ops/addition.zig:37-47, src/ops/hadamard.zig:35-45, src/ops/relu.zig:13-52) and the kernel
 * generator only replicates fixed sources at build time (file_gen.zig:200-328). These entry
 * points are for a host side that defers elementwise ops and wants whatever expression it ends
 * up with as one kernel per direction, also when nobody listed that expression at build time.
 *
 * An expression is text over the ops add, sub, mul (hadamard), neg, relu, selu and, with a literal
 * constant as second argument, scale (the reference's dilate: x * c) and shift (its translate:
 * x + c), with its leaves written as 0, 1, ... (or x0, x1, ...) and numbered in order of first
 * appearance; a leaf may appear more than once. Examples: "selu(mul(add(0,1),add(2,3)))",
 * "relu(scale(mul(0,1),0.125))". Up to four results over the same leaves are written one after the
 * other with ';' between them, leaves numbered across all of them
 * ("selu(mul(add(0,1),2));relu(sub(add(0,1),3))"): one kernel computes them all and reads every
 * leaf once (mpChainForwardMany / mpChainReverseMany). At most 8 leaves, 8 constants, 64 nodes. The constants are
 * arguments of the kernels, read from the text at every call: an expression is compiled once,
 * whatever the values (a learning rate that changes every step costs nothing).
 * dtype is MP_R16, MP_R32 or MP_R64 (tensor_types.h).
 *
 * The first use of an (expression, dtype) in a process compiles it (about half a second, with
 * hiprtc, no compiler driver needed on the machine); the result is kept until the process ends.
 * Every function is safe to call from several threads. Under HIP graph capture a call is one
 * kernel node, provided the (expression, dtype) has been used on that device before the capture
 * began: compiling and loading cannot be captured.
 *
 * Errors: these functions return 0 on success and non-zero when nothing was enqueued (text that
 * does not parse, too many leaves, a compile or launch failure); mpChainError() then describes
 * the reason for the calling thread. They do not exit, unlike the launchers, because the caller
 * has a fallback: one launch per op.
 */
#ifndef MP_CHAIN_FUSION_H
#define MP_CHAIN_FUSION_H

#include "tensor_types.h"

#if defined(__cplusplus)
  #define EXTERN_C extern "C"
#else
  #define EXTERN_C extern
#endif

/* out[i] = expression(x[0][i], ..., x[k-1][i]) for i < n: one read of each leaf, one write.
 * x: k device pointers (k = the expression's leaf count), any element alignment; out may alias
 * any x[j] exactly. Leaves that are 16-byte aligned and together no larger than 256 MiB are read so
 * that they stay in the GPU's memory-side cache, where mpChainReverse, which reads them all again,
 * finds them. */
EXTERN_C int mpChainForward(const char* expression, int dtype, const void* const* x, void* out, len_t n, StreamContext);

/* Every leaf gradient in one pass: g[j][i] = d expression / d x[j] * out_grads[i] + alpha * g[j][i].
 * alpha == 0 never reads g (k + 1 reads and k writes per element), any other alpha blends
 * (2k + 1 reads). g: k device pointers, distinct from each other. */
EXTERN_C int mpChainReverse(const char* expression, int dtype, const void* const* x, const void* out_grads,
                            void* const* g, double alpha, len_t n, StreamContext);

/* The same for an expression with R results: outs holds R device pointers, out_grads R upstream
 * gradients; g[j] receives the sum over all results of d result_r / d x[j] * out_grads[r]. A leaf
 * that no result depends on gets 0 (+ alpha * g). mpChainForward / mpChainReverse refuse an
 * expression with more than one result. */
EXTERN_C int mpChainForwardMany(const char* expressions, int dtype, const void* const* x, void* const* outs, len_t n, StreamContext);
EXTERN_C int mpChainReverseMany(const char* expressions, int dtype, const void* const* x, const void* const* out_grads,
                                void* const* g, double alpha, len_t n, StreamContext);
/* How many results an expression has, -1 when it does not parse. */
EXTERN_C int mpChainRoots(const char* expressions);

/* Compile now rather than at the first launch. Needs no GPU. */
EXTERN_C int mpChainCompile(const char* expression, int dtype);
/* The leaf count of an expression, -1 when it does not parse. */
EXTERN_C int mpChainLeaves(const char* expression);
/* The HIP source generated for (expression, dtype); NULL on error. Valid until the process ends. */
EXTERN_C const char* mpChainSource(const char* expression, int dtype);
/* The gfx950 code object compiled for (expression, dtype) and its size; NULL on error. Its kernels are
 * chain_forward_<l>, chain_reverse_overwrite_<l>, chain_reverse_blend_<l> with l = 0 (all operands
 * 16-byte aligned), 1 (operands that share a place in a 128-byte line) or 2 (any alignment). */
EXTERN_C const void* mpChainCodeObject(const char* expression, int dtype, len_t* bytes);
/* How many (expression, dtype) pairs this process has compiled (expressions that differ in their
 * constants only are one). */
EXTERN_C len_t mpChainCacheSize(void);
/* How many compilations this process has started, failed ones included. A compilation that failed is
 * not tried again: later calls for that (expression, dtype) fail at once with the same reason. */
EXTERN_C len_t mpChainCompilations(void);
/* Why the calling thread's last failing call failed. Valid until that thread's next failure. */
EXTERN_C const char* mpChainError(void);

#endif
