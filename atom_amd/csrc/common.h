// Shared device helpers for the gfx950 kernels: element types, wave and block
// reductions.  A wavefront has 64 lanes on CDNA; every reduction below assumes it.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define ATOM_EXPORT extern "C" __attribute__((visibility("default")))

// Element type codes of the C interface.
enum AtomDtype : int { ATOM_F32 = 0, ATOM_BF16 = 1 };

// Return codes of the C interface (0 = launched).
enum AtomStatus : int {
  ATOM_OK = 0,
  ATOM_BAD_DTYPE = 1,
  ATOM_BAD_SHAPE = 2,
  ATOM_UNSUPPORTED = 3,
  ATOM_LAUNCH_FAILED = 4,
  ATOM_TOO_LARGE = 5,
};

typedef __bf16 bf16_t;

constexpr int kWave = 64;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return static_cast<float>(v); }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return static_cast<bf16_t>(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// The maximum (the sum) of v over the four lanes r, r + 16, r + 32 and r + 48, in each of them.  The rows of 16
// lanes change places through the row-swap instructions of gfx950, without a trip through LDS: the first leaves
// rows (0, 0, 2, 2) of v in one register and rows (1, 1, 3, 3) in the other, the second the lower half of its
// operand twice in one and the upper half twice in the other.
__device__ __forceinline__ float rows_max(float v) {
  const unsigned bits = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
  const unsigned pair = __float_as_uint(fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1])));
  const auto b = __builtin_amdgcn_permlane32_swap(pair, pair, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

__device__ __forceinline__ float rows_sum(float v) {
  const unsigned bits = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
  const unsigned pair = __float_as_uint(__uint_as_float(a[0]) + __uint_as_float(a[1]));
  const auto b = __builtin_amdgcn_permlane32_swap(pair, pair, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Sum over a block of up to 1024 threads; `scratch` holds one float per wave
// (16 at most).  Every thread receives the total.  The order of the partial sums
// is fixed, so the result does not depend on what else runs.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();  // scratch may still be read from a previous call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < waves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

// The CUs of the current device, asked for once per device: what the launch plans count blocks against (256 on
// the MI355X that their other figures were measured on; also the answer where no device can be asked).
static inline int device_cus() {
  static int known[16] = {0};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 16) return 256;
  if (!known[device]) {
    int cus = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0) cus = 256;
    known[device] = cus;
  }
  return known[device];
}

static inline int launch_status() {
  return hipGetLastError() == hipSuccess ? ATOM_OK : ATOM_LAUNCH_FAILED;
}

// Calls `fn.template operator()<T>()` with the element type that `dtype` names.
#define ATOM_DISPATCH_DTYPE(dtype, ...)                 \
  do {                                                  \
    if ((dtype) == ATOM_F32) {                          \
      using T = float;                                  \
      __VA_ARGS__;                                      \
    } else if ((dtype) == ATOM_BF16) {                  \
      using T = bf16_t;                                 \
      __VA_ARGS__;                                      \
    } else {                                            \
      return ATOM_BAD_DTYPE;                            \
    }                                                   \
  } while (0)
