// Kernels of the toy parts in test_gpu_parts.py: a part outside the framework brings HIP code of its own,
// compiled with the framework's flags and bound through ctypes.  Plain element-wise loops, float32 arithmetic.
#include <hip/hip_runtime.h>

typedef __bf16 bf16_t;

template <typename T>
__global__ void toy_scale_kernel(T* x, long n, float factor) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = static_cast<T>(static_cast<float>(x[i]) * factor);
}

__global__ void toy_softcap_kernel(float* x, long n, float cap) {
  const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

// x[i] *= factor in place; bf16 = 1 for bfloat16 elements, 0 for float32.  Returns 0 when launched.
extern "C" __attribute__((visibility("default"))) int toy_scale(void* x, long n, float factor, int bf16,
                                                                hipStream_t stream) {
  if (n < 0 || !x) return 2;
  if (n == 0) return 0;
  const unsigned blocks = (unsigned)((n + 255) / 256);
  if (bf16) hipLaunchKernelGGL(toy_scale_kernel<bf16_t>, dim3(blocks), dim3(256), 0, stream, (bf16_t*)x, n, factor);
  else hipLaunchKernelGGL(toy_scale_kernel<float>, dim3(blocks), dim3(256), 0, stream, (float*)x, n, factor);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}

// x[i] = cap * tanh(x[i] / cap) in place, float32.
extern "C" __attribute__((visibility("default"))) int toy_softcap(float* x, long n, float cap, hipStream_t stream) {
  if (n < 0 || !x || !(cap > 0.f)) return 2;
  if (n == 0) return 0;
  hipLaunchKernelGGL(toy_softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, x, n, cap);
  return hipGetLastError() == hipSuccess ? 0 : 4;
}
