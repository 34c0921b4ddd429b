// The one entry point of this library that allocates nothing.
//
// It has no counterpart in the reference (ROCm/ATOM), whose matrix products come from a library
// that allocates its own workspaces.  It is for callers that cannot allocate device memory:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
//   y[m, n] = x[m, k] * w[n, k]^T (+ bias)     bfloat16 x and w, float32 bias, y bfloat16 or float32
//
// It is atom_gemm_skinny followed, where that kernel cuts K, by atom_splitk_reduce: the same
// kernels, the same order of the sum, the same result to the bit.  The float32 slices that lie
// between the two kernels go to a buffer that is part of the loaded library
// (kLinearStaticFloats floats = 16 MiB on every GPU the library runs on, held until the process
// ends) instead of a workspace that the caller allocates and passes in.
//
// Returns 0 when both kernels are queued on `stream`, else an AtomStatus:
//   ATOM_UNSUPPORTED (3)  the skinny kernels do not take this product (atom_gemm_skinny_supports)
//   ATOM_TOO_LARGE (5)    splits * m * n floats (atom_gemm_skinny_splits) exceed kLinearStaticFloats;
//                         atom_linear_skinny_static_limit() returns that number
//   ATOM_BAD_SHAPE (2)    a null or misaligned operand, or a size below 1
//   ATOM_LAUNCH_FAILED (4) the buffer's address could not be taken, or a launch failed
//
// Every call on a GPU uses that GPU's one buffer, which keeps the last call's slices: two calls
// that overlap in time on one GPU (different streams, different threads) race, and the caller has to
// order them.  Nothing in the buffer needs to start at zero: the product writes every slice
// element that the reduction reads.  The buffer's device address is looked up once per device, at
// the first call on it (or by atom_linear_skinny_static_init, which a caller that captures
// graphs calls beforehand, with that device current); the current device must be the stream's.
#pragma once

#include "common.h"

constexpr long kLinearStaticFloats = 4L * 1024 * 1024;

ATOM_EXPORT int atom_linear_skinny_static_init(void);
ATOM_EXPORT long atom_linear_skinny_static_limit(void);
ATOM_EXPORT int atom_linear_skinny_static(const void* x, const void* w, const float* bias, void* y, int m, int n,
                                          int k, int out_f32, hipStream_t stream);
