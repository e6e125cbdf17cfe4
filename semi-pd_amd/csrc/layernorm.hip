// LayerNorm of post-norm residual blocks and the squared-ReLU activation (gfx950, wave64).
//
//  * layernorm_kernel: y = (x + in_bias - mean) / sqrt(var + eps) * w + b per row, var = mean of the squared deviations,
//    all in fp32.  With a residual stream (fp32, updated in place) the result is ADDED to it and the sum is what comes
//    out in the activation type: the block "x <- x + norm(sublayer(x))" between two GEMMs in one launch, the residual
//    never leaving fp32.  Input rows are of the activation type or fp32 (the final norm reads the stream itself).
//  * bias_relu_square_kernel: u <- max(u + b, 0)^2 in place.
#include "common.h"

namespace semipd {

template <typename T, typename TIn>
__global__ void __launch_bounds__(256) layernorm_kernel(const TIn* __restrict__ in, int64_t in_ld, const T* __restrict__ in_bias,
                                                        const T* __restrict__ w, const T* __restrict__ b, float eps,
                                                        float* __restrict__ residual, int64_t res_ld, T* __restrict__ out,
                                                        int64_t out_ld, int64_t width) {
  __shared__ float red[16];
  const int64_t r = blockIdx.x;
  const TIn* x = in + r * in_ld;
  auto at = [&](int64_t i) -> float {
    float v = Elem<TIn>::to_f(x[i]);
    if (in_bias) v += Elem<T>::to_f(in_bias[i]);
    return v;
  };
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += 256) s += at(i);
  const float mean = block_sum(s, red) / (float)width;
  float q = 0.f;
  for (int64_t i = threadIdx.x; i < width; i += 256) {
    const float d = at(i) - mean;
    q += d * d;
  }
  __syncthreads();
  const float var = block_sum(q, red) / (float)width;
  const float rs = 1.0f / sqrtf(var + eps);
  for (int64_t i = threadIdx.x; i < width; i += 256) {
    float v = (at(i) - mean) * rs * Elem<T>::to_f(w[i]) + Elem<T>::to_f(b[i]);
    if (residual) {
      v += residual[r * res_ld + i];
      residual[r * res_ld + i] = v;
    }
    if (out) out[r * out_ld + i] = Elem<T>::from_f(v);
  }
}

template <typename T>
__global__ void __launch_bounds__(256) bias_relu_square_kernel(T* __restrict__ u, int64_t ld, const T* __restrict__ bias,
                                                               int64_t rows, int64_t width) {
  const int64_t n = rows * width;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / width, c = i - r * width;
    float v = Elem<T>::to_f(u[r * ld + c]);
    if (bias) v += Elem<T>::to_f(bias[c]);
    v = v > 0.f ? v * v : 0.f;
    u[r * ld + c] = Elem<T>::from_f(v);
  }
}

}  // namespace semipd

using namespace semipd;

extern "C" int semipd_layernorm(const void* in, int64_t in_ld, int in_is_f32, const void* in_bias, const void* weight,
                                const void* bias, float eps, float* residual, int64_t residual_ld, void* out, int64_t out_ld,
                                int64_t rows, int64_t width, int dtype, void* stream) {
  SEMIPD_CHECK_ARG(rows >= 0 && width > 0, SEMIPD_EINVAL, "layernorm: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG(in && weight && bias && (residual || out), SEMIPD_EINVAL, "layernorm: null pointer");
  SEMIPD_DISPATCH_DTYPE(dtype, T, {
    if (in_is_f32)
      hipLaunchKernelGGL((layernorm_kernel<T, float>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream), (const float*)in,
                         in_ld, (const T*)in_bias, (const T*)weight, (const T*)bias, eps, residual, residual_ld, (T*)out, out_ld,
                         width);
    else
      hipLaunchKernelGGL((layernorm_kernel<T, T>), dim3((unsigned)rows), dim3(256), 0, as_stream(stream), (const T*)in, in_ld,
                         (const T*)in_bias, (const T*)weight, (const T*)bias, eps, residual, residual_ld, (T*)out, out_ld, width);
  });
  return launch_status("layernorm");
}

extern "C" int semipd_bias_relu_square(void* u, int64_t ld, const void* bias, int64_t rows, int64_t width, int dtype,
                                       void* stream) {
  SEMIPD_CHECK_ARG(rows >= 0 && width > 0 && ld >= width, SEMIPD_EINVAL, "bias_relu_square: bad sizes");
  if (rows == 0) return 0;
  SEMIPD_CHECK_ARG(u, SEMIPD_EINVAL, "bias_relu_square: null pointer");
  const int64_t n = rows * width;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  SEMIPD_DISPATCH_DTYPE(dtype, T,
                        hipLaunchKernelGGL((bias_relu_square_kernel<T>), dim3(blocks), dim3(256), 0, as_stream(stream), (T*)u, ld,
                                           (const T*)bias, rows, width));
  return launch_status("bias_relu_square");
}
