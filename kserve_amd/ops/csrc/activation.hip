// SwiGLU activation: out = silu(gate) * up, input layout [rows, 2*d] = [gate|up].
// Memory-bound elementwise; vectorized short8 (CDNA guide Appendix B).
//
// clamped_swiglu: out = g * sigmoid(alpha * g) * (u + 1) with g = min(gate,
// limit) and u = clamp(up, -limit, limit); same [gate|up] layout, either
// activation dtype, fp32 arithmetic.
//
// glu_silu_scale: out = silu(gate) * up * scale[row] (scale optional), same
// [gate|up] layout, either dtype, exact exp: a mixture of experts folds each
// (token, expert) routing weight into the activation this way.
// bias_gelu_tanh: out = gelu_tanh(x + bias[col]),
// gelu_tanh(z) = 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).
// relu2_scale: out = max(x, 0)^2 * scale[row] (scale optional), same dtype.
// scale_softcap: fp32 out = cap * tanh(x * scale / cap) (cap 0: x * scale).
#include "dtype_io.h"

namespace {

template <typename T>
__global__ void glu_silu_scale_kernel(T* __restrict__ out,
                                      const T* __restrict__ input,
                                      const float* __restrict__ scales,
                                      const long rows, const int d) {
  const long total = rows * d;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / d;
    const long col = idx % d;
    const float sc = scales ? scales[row] : 1.0f;
    float y = 0.f;
    if (!scales || sc != 0.0f) {
      const float g = ld_f32(input, row * 2 * d + col);
      const float u = ld_f32(input, row * 2 * d + d + col);
      y = g / (1.0f + expf(-g)) * u * sc;
    }
    st_f32(out, idx, y);
  }
}

__global__ void glu_silu_scale_bf16x8_kernel(short* __restrict__ out,
                                             const short* __restrict__ input,
                                             const float* __restrict__ scales,
                                             const long rows, const int d) {
  const int nvec = d >> 3;
  const short8_t* in_vec = reinterpret_cast<const short8_t*>(input);
  short8_t* out_vec = reinterpret_cast<short8_t*>(out);
  const long total = rows * nvec;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / nvec;
    const long col = idx % nvec;
    const float sc = scales ? scales[row] : 1.0f;
    short8_t o;
    if (scales && sc == 0.0f) {
      // an expert the token did not choose: nothing to read
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = 0;
    } else {
      const short8_t g8 = in_vec[row * (2 * nvec) + col];
      const short8_t u8 = in_vec[row * (2 * nvec) + nvec + col];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float g = bf16_bits_to_float(g8[j]);
        const float u = bf16_bits_to_float(u8[j]);
        o[j] = float_to_bf16_bits(g / (1.0f + expf(-g)) * u * sc);
      }
    }
    out_vec[idx] = o;
  }
}

template <typename T>
__global__ void relu2_scale_kernel(T* __restrict__ out,
                                   const T* __restrict__ input,
                                   const float* __restrict__ scales,
                                   const long rows, const int d) {
  const long total = rows * d;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const float sc = scales ? scales[idx / d] : 1.0f;
    float y = 0.f;
    if (!scales || sc != 0.0f) {
      const float x = fmaxf(ld_f32(input, idx), 0.f);
      y = x * x * sc;
    }
    st_f32(out, idx, y);
  }
}

__global__ void relu2_scale_bf16x8_kernel(short* __restrict__ out,
                                          const short* __restrict__ input,
                                          const float* __restrict__ scales,
                                          const long rows, const int d) {
  const int nvec = d >> 3;
  const short8_t* in_vec = reinterpret_cast<const short8_t*>(input);
  short8_t* out_vec = reinterpret_cast<short8_t*>(out);
  const long total = rows * nvec;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const float sc = scales ? scales[idx / nvec] : 1.0f;
    short8_t o;
    if (scales && sc == 0.0f) {
      // an expert the token did not choose: nothing to read
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = 0;
    } else {
      const short8_t x8 = in_vec[idx];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float x = fmaxf(bf16_bits_to_float(x8[j]), 0.f);
        o[j] = float_to_bf16_bits(x * x * sc);
      }
    }
    out_vec[idx] = o;
  }
}

template <typename T>
__global__ void scale_softcap_kernel(float* __restrict__ out,
                                     const T* __restrict__ input, float scale,
                                     float cap, const long total) {
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const float x = ld_f32(input, idx) * scale;
    out[idx] = cap > 0.f ? cap * tanhf(x / cap) : x;
  }
}

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z *
         (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void bias_gelu_tanh_kernel(T* __restrict__ out,
                                      const T* __restrict__ input,
                                      const float* __restrict__ bias,
                                      const long rows, const int d) {
  const long total = rows * d;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x)
    st_f32(out, idx, gelu_tanh_f(ld_f32(input, idx) + bias[idx % d]));
}

__global__ void bias_gelu_tanh_bf16x8_kernel(short* __restrict__ out,
                                             const short* __restrict__ input,
                                             const float* __restrict__ bias,
                                             const long rows, const int d) {
  const int nvec = d >> 3;
  const short8_t* in_vec = reinterpret_cast<const short8_t*>(input);
  short8_t* out_vec = reinterpret_cast<short8_t*>(out);
  const long total = rows * nvec;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const int col = (int)(idx % nvec) * 8;
    const short8_t x8 = in_vec[idx];
    const float4_t b0 = *reinterpret_cast<const float4_t*>(bias + col);
    const float4_t b1 = *reinterpret_cast<const float4_t*>(bias + col + 4);
    short8_t o;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      o[j] = float_to_bf16_bits(gelu_tanh_f(
          bf16_bits_to_float(x8[j]) + (j < 4 ? b0[j] : b1[j - 4])));
    out_vec[idx] = o;
  }
}

template <typename T>
__global__ void clamped_swiglu_kernel(T* __restrict__ out,
                                      const T* __restrict__ input,
                                      const long rows, const int d,
                                      const float alpha, const float limit) {
  const long total = rows * d;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / d;
    const long col = idx % d;
    const float g = fminf(ld_f32(input, row * 2 * d + col), limit);
    const float u =
        fminf(fmaxf(ld_f32(input, row * 2 * d + d + col), -limit), limit);
    st_f32(out, idx, g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
  }
}

// 8 bf16 per lane when rows are 8-element aligned
__global__ void clamped_swiglu_bf16x8_kernel(short* __restrict__ out,
                                             const short* __restrict__ input,
                                             const long rows, const int d,
                                             const float alpha,
                                             const float limit) {
  const int nvec = d >> 3;
  const short8_t* in_vec = reinterpret_cast<const short8_t*>(input);
  short8_t* out_vec = reinterpret_cast<short8_t*>(out);
  const long total = rows * nvec;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / nvec;
    const long col = idx % nvec;
    const short8_t g8 = in_vec[row * (2 * nvec) + col];
    const short8_t u8 = in_vec[row * (2 * nvec) + nvec + col];
    short8_t o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float g = fminf(bf16_bits_to_float(g8[j]), limit);
      const float u = fminf(fmaxf(bf16_bits_to_float(u8[j]), -limit), limit);
      o[j] = float_to_bf16_bits(g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
    }
    out_vec[idx] = o;
  }
}

__global__ void silu_and_mul_kernel(short* __restrict__ out,
                                    const short* __restrict__ input,
                                    const int rows, const int d) {
  const int nvec = d >> 3;
  const short8_t* in_vec = reinterpret_cast<const short8_t*>(input);
  short8_t* out_vec = reinterpret_cast<short8_t*>(out);
  const long total = (long)rows * nvec;
  for (long idx = blockIdx.x * (long)blockDim.x + threadIdx.x; idx < total;
       idx += (long)gridDim.x * blockDim.x) {
    const long row = idx / nvec;
    const long col = idx % nvec;
    short8_t g = in_vec[row * (2 * nvec) + col];
    short8_t u = in_vec[row * (2 * nvec) + nvec + col];
    short8_t o;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float gf = bf16_bits_to_float(g[j]);
      float uf = bf16_bits_to_float(u[j]);
      float s = gf / (1.f + __expf(-gf));
      o[j] = float_to_bf16_bits(s * uf);
    }
    out_vec[idx] = o;
  }
}

}  // namespace

extern "C" hipError_t ks_silu_and_mul(void* out, const void* input, int rows,
                                      int d, hipStream_t stream) {
  if (d % 8 != 0) return hipErrorInvalidValue;
  long total = (long)rows * (d >> 3);
  if (total == 0) return hipSuccess;
  int grid = (int)((total + 255) / 256);
  if (grid > 2048) grid = 2048;  // grid-stride (G11)
  hipLaunchKernelGGL(silu_and_mul_kernel, dim3(grid), dim3(256), 0, stream,
                     (short*)out, (const short*)input, rows, d);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_clamped_swiglu(void* out, const void* input, int rows,
                                        int d, float alpha, float limit,
                                        int is_f32, hipStream_t stream) {
  long total = (long)rows * d;
  if (total == 0) return hipSuccess;
  int grid = (int)((total + 255) / 256);
  if (grid > 4096) grid = 4096;
  if (is_f32)
    hipLaunchKernelGGL(clamped_swiglu_kernel<float>, dim3(grid), dim3(256), 0,
                       stream, (float*)out, (const float*)input, (long)rows, d,
                       alpha, limit);
  else if (d % 8 == 0 && ((uintptr_t)input % 16) == 0 &&
           ((uintptr_t)out % 16) == 0) {
    long tv = (long)rows * (d >> 3);
    int gv = (int)((tv + 255) / 256);
    if (gv > 8192) gv = 8192;
    hipLaunchKernelGGL(clamped_swiglu_bf16x8_kernel, dim3(gv), dim3(256), 0,
                       stream, (short*)out, (const short*)input, (long)rows, d,
                       alpha, limit);
  } else
    hipLaunchKernelGGL(clamped_swiglu_kernel<short>, dim3(grid), dim3(256), 0,
                       stream, (short*)out, (const short*)input, (long)rows, d,
                       alpha, limit);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_glu_silu_scale(void* out, const void* input,
                                        const void* scales, int rows, int d,
                                        int is_f32, hipStream_t stream) {
  const long total = (long)rows * d;
  if (total == 0) return hipSuccess;
  int grid = (int)((total + 255) / 256);
  if (grid > 4096) grid = 4096;
  if (is_f32)
    hipLaunchKernelGGL(glu_silu_scale_kernel<float>, dim3(grid), dim3(256), 0,
                       stream, (float*)out, (const float*)input,
                       (const float*)scales, (long)rows, d);
  else if (d % 8 == 0 && ((uintptr_t)input % 16) == 0 &&
           ((uintptr_t)out % 16) == 0) {
    const long tv = (long)rows * (d >> 3);
    int gv = (int)((tv + 255) / 256);
    if (gv > 8192) gv = 8192;
    hipLaunchKernelGGL(glu_silu_scale_bf16x8_kernel, dim3(gv), dim3(256), 0,
                       stream, (short*)out, (const short*)input,
                       (const float*)scales, (long)rows, d);
  } else
    hipLaunchKernelGGL(glu_silu_scale_kernel<short>, dim3(grid), dim3(256), 0,
                       stream, (short*)out, (const short*)input,
                       (const float*)scales, (long)rows, d);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_bias_gelu_tanh(void* out, const void* input,
                                        const void* bias, int rows, int d,
                                        int is_f32, hipStream_t stream) {
  const long total = (long)rows * d;
  if (total == 0) return hipSuccess;
  int grid = (int)((total + 255) / 256);
  if (grid > 4096) grid = 4096;
  if (is_f32)
    hipLaunchKernelGGL(bias_gelu_tanh_kernel<float>, dim3(grid), dim3(256), 0,
                       stream, (float*)out, (const float*)input,
                       (const float*)bias, (long)rows, d);
  else if (d % 8 == 0 && ((uintptr_t)input % 16) == 0 &&
           ((uintptr_t)out % 16) == 0 && ((uintptr_t)bias % 16) == 0) {
    const long tv = (long)rows * (d >> 3);
    int gv = (int)((tv + 255) / 256);
    if (gv > 8192) gv = 8192;
    hipLaunchKernelGGL(bias_gelu_tanh_bf16x8_kernel, dim3(gv), dim3(256), 0,
                       stream, (short*)out, (const short*)input,
                       (const float*)bias, (long)rows, d);
  } else
    hipLaunchKernelGGL(bias_gelu_tanh_kernel<short>, dim3(grid), dim3(256), 0,
                       stream, (short*)out, (const short*)input,
                       (const float*)bias, (long)rows, d);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_relu2_scale(void* out, const void* input,
                                     const void* scales, int rows, int d,
                                     int is_f32, hipStream_t stream) {
  const long total = (long)rows * d;
  if (total == 0) return hipSuccess;
  int grid = (int)((total + 255) / 256);
  if (grid > 4096) grid = 4096;
  if (is_f32)
    hipLaunchKernelGGL(relu2_scale_kernel<float>, dim3(grid), dim3(256), 0,
                       stream, (float*)out, (const float*)input,
                       (const float*)scales, (long)rows, d);
  else if (d % 8 == 0 && ((uintptr_t)input % 16) == 0 &&
           ((uintptr_t)out % 16) == 0) {
    const long tv = (long)rows * (d >> 3);
    int gv = (int)((tv + 255) / 256);
    if (gv > 8192) gv = 8192;
    hipLaunchKernelGGL(relu2_scale_bf16x8_kernel, dim3(gv), dim3(256), 0,
                       stream, (short*)out, (const short*)input,
                       (const float*)scales, (long)rows, d);
  } else
    hipLaunchKernelGGL(relu2_scale_kernel<short>, dim3(grid), dim3(256), 0,
                       stream, (short*)out, (const short*)input,
                       (const float*)scales, (long)rows, d);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_scale_softcap(void* out, const void* input,
                                       float scale, float cap, long total,
                                       int is_f32, hipStream_t stream) {
  if (total == 0) return hipSuccess;
  int grid = (int)((total + 255) / 256);
  if (grid > 4096) grid = 4096;
  if (is_f32)
    hipLaunchKernelGGL(scale_softcap_kernel<float>, dim3(grid), dim3(256), 0,
                       stream, (float*)out, (const float*)input, scale, cap,
                       total);
  else
    hipLaunchKernelGGL(scale_softcap_kernel<short>, dim3(grid), dim3(256), 0,
                       stream, (float*)out, (const short*)input, scale, cap,
                       total);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}
