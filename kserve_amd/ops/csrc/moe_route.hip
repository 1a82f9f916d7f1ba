// Routing of a mixture of experts and the row movements around its GEMMs.
//
//  * router_topk: one wave per token. Scores of fp32 logits [T, E] (sigmoid,
//    or softmax over the experts), the `top` largest chosen one at a time
//    (ties go to the lower expert), optionally renormalised to sum 1
//    (divided by their sum + renorm_eps) and multiplied by weight_scale. With a correction vector the
//    choice goes by score + correction[e] while the weights stay the scores.
//    Outputs expert ids and weights [T, top] and, if asked, the same weights
//    as a dense [T, E] matrix that is zero for experts not chosen.
//  * route_tokens: the router's matrix product fused in front of the same
//    choice: a block per token, the input row in LDS as fp32, fp32 router
//    rows, fp32 sums; the logits never travel through memory.
//  * gather_scale_rows: out[r] = x[rows[r]] * scales[r], product in fp32,
//    rounded to the activation dtype (an expert's input is the token's input
//    times its routing weight); without scales a plain row gather.
//  * combine_rows: out[t] = sum_k weights[t*top + k] * y[index[t*top + k]]
//    (+ extra[t]) (+ scaled_w[t] * scaled[t]) in fp32, k in ascending order,
//    then extra, then the scaled row: no atomics, the same sum every run.
//    Weights default to 1; the scaled row is how experts that return their
//    input join the sum.
#include "dtype_io.h"

namespace {

constexpr int NT = 256;
constexpr int NW = NT / WAVE_SIZE;
constexpr int MAX_PER_LANE = 16;  // experts <= 64 * MAX_PER_LANE

// One wave picks the `top` largest scores of one token. `z` points at the
// token's E logits (global or LDS).
__device__ __forceinline__ void wave_topk(int* __restrict__ idx_out,
                                          float* __restrict__ w_out,
                                          float* __restrict__ dense_out,
                                          const float* z, long t, int E,
                                          int top, int softmax, int renorm,
                                          const float* __restrict__ correction,
                                          float renorm_eps, float weight_scale) {
  const int lane = threadIdx.x & 63;
  float sc[MAX_PER_LANE];  // scores of experts lane + 64 j
  float mx = -INFINITY;
#pragma unroll
  for (int j = 0; j < MAX_PER_LANE; ++j) {
    const int e = lane + 64 * j;
    sc[j] = e < E ? z[e] : -INFINITY;
    mx = fmaxf(mx, sc[j]);
  }
  if (softmax) {
    mx = wave_reduce_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < MAX_PER_LANE; ++j) {
      const int e = lane + 64 * j;
      sc[j] = e < E ? expf(sc[j] - mx) : 0.f;
      sum += sc[j];
    }
    sum = wave_reduce_sum(sum);
#pragma unroll
    for (int j = 0; j < MAX_PER_LANE; ++j) sc[j] = sc[j] / sum;
  } else {
#pragma unroll
    for (int j = 0; j < MAX_PER_LANE; ++j) sc[j] = 1.0f / (1.0f + expf(-sc[j]));
  }
  unsigned chosen = 0;  // bit j: expert lane + 64 j was chosen
  float my_w = 0.f;     // lane k keeps the k-th pick
  int my_e = 0;
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;  // choice value (score + correction)
    float bs = 0.f;        // the score itself
    int be = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < MAX_PER_LANE; ++j) {
      const int e = lane + 64 * j;
      if (e < E && !(chosen >> j & 1u)) {
        const float cv = correction ? sc[j] + correction[e] : sc[j];
        if (cv > bv) {
          bv = cv;
          bs = sc[j];
          be = e;
        }
      }
    }
    // a lane whose candidates are all taken (or NaN) offers nothing
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, WAVE_SIZE);
      const float os = __shfl_xor(bs, off, WAVE_SIZE);
      const int oe = __shfl_xor(be, off, WAVE_SIZE);
      if (ov > bv || (ov == bv && oe < be)) {
        bv = ov;
        bs = os;
        be = oe;
      }
    }
    if (be == 0x7fffffff) be = 0;  // nothing comparable left (NaN scores)
    if ((be & 63) == lane) chosen |= 1u << (be >> 6);
    total += bs;
    if (lane == k) {
      my_w = bs;
      my_e = be;
    }
  }
  const float norm =
      (renorm ? 1.0f / (total + renorm_eps) : 1.0f) * weight_scale;
  if (lane < top) {
    idx_out[t * top + lane] = my_e;
    w_out[t * top + lane] = my_w * norm;
  }
  if (dense_out) {
#pragma unroll
    for (int j = 0; j < MAX_PER_LANE; ++j) {
      const int e = lane + 64 * j;
      if (e < E) dense_out[t * E + e] = (chosen >> j & 1u) ? sc[j] * norm : 0.f;
    }
  }
}

__global__ void router_topk_kernel(int* __restrict__ idx_out,
                                   float* __restrict__ w_out,
                                   float* __restrict__ dense_out,
                                   const float* __restrict__ logits, int tokens,
                                   int E, int top, int softmax, int renorm,
                                   const float* __restrict__ correction,
                                   float renorm_eps, float weight_scale) {
  const long t = (long)blockIdx.x * NW + (threadIdx.x >> 6);
  if (t >= tokens) return;  // whole waves leave together
  wave_topk(idx_out, w_out, dense_out, logits + t * E, t, E, top, softmax,
            renorm, correction, renorm_eps, weight_scale);
}

// Router logits and the choice in one kernel: a block per token keeps the
// token's input row in LDS as fp32, its waves share out the experts (fp32
// dot products against fp32 router rows), then the first wave chooses.
template <typename T>
__global__ void __launch_bounds__(NT) route_tokens_kernel(
    int* __restrict__ idx_out, float* __restrict__ w_out,
    float* __restrict__ dense_out, float* __restrict__ logits_out,
    const T* __restrict__ h, long h_stride, const float* __restrict__ router,
    int W, int E, int top, int softmax, int renorm,
    const float* __restrict__ correction, float renorm_eps, float weight_scale) {
  extern __shared__ float lds[];
  float* row = lds;      // [W]
  float* z = lds + ((W + 3) & ~3);  // [E]
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* hr = h + t * h_stride;
  // 4-wide path: rows, strides and pointers are 4-element aligned
  const bool vec = (W % 4) == 0 && (h_stride % 4) == 0 &&
                   ((uintptr_t)h % (4 * sizeof(T))) == 0 &&
                   ((uintptr_t)router % 16) == 0;
  if (vec) {
    for (int i = threadIdx.x * 4; i < W; i += NT * 4) {
      float x[4];
      if (sizeof(T) == 2) {
        const short4_t u = *reinterpret_cast<const short4_t*>(
            reinterpret_cast<const short*>(hr) + i);
#pragma unroll
        for (int c = 0; c < 4; ++c) x[c] = bf16_bits_to_float(u[c]);
      } else {
        const float4_t u = *reinterpret_cast<const float4_t*>(
            reinterpret_cast<const float*>(hr) + i);
#pragma unroll
        for (int c = 0; c < 4; ++c) x[c] = u[c];
      }
      *reinterpret_cast<float4_t*>(row + i) = float4_t{x[0], x[1], x[2], x[3]};
    }
  } else {
    for (int i = threadIdx.x; i < W; i += NT) row[i] = ld_f32(hr, i);
  }
  __syncthreads();
  for (int e = wave; e < E; e += NW) {
    const float* wr = router + (long)e * W;
    float acc = 0.f;
    if (vec) {
      for (int i = lane * 4; i < W; i += WAVE_SIZE * 4) {
        const float4_t a = *reinterpret_cast<const float4_t*>(row + i);
        const float4_t b = *reinterpret_cast<const float4_t*>(wr + i);
        acc += a[0] * b[0] + a[1] * b[1] + a[2] * b[2] + a[3] * b[3];
      }
    } else {
      for (int i = lane; i < W; i += WAVE_SIZE) acc += row[i] * wr[i];
    }
    acc = wave_reduce_sum(acc);
    if (lane == 0) {
      z[e] = acc;
      if (logits_out) logits_out[t * E + e] = acc;
    }
  }
  __syncthreads();
  if (wave == 0)
    wave_topk(idx_out, w_out, dense_out, z, t, E, top, softmax, renorm,
              correction, renorm_eps, weight_scale);
}

__device__ __forceinline__ void ld4_any(const short* p, float* v) {
  const short4_t x = *reinterpret_cast<const short4_t*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = bf16_bits_to_float(x[i]);
}
__device__ __forceinline__ void ld4_any(const float* p, float* v) {
  const float4_t x = *reinterpret_cast<const float4_t*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = x[i];
}

template <typename T>
__global__ void gather_scale_rows_kernel(T* __restrict__ out,
                                         const T* __restrict__ x, long x_stride,
                                         const int* __restrict__ rows,
                                         const float* __restrict__ scales,
                                         int width) {
  const long r = blockIdx.x;
  const T* src = x + (long)rows[r] * x_stride;
  if (!scales) {
    for (int i = threadIdx.x; i < width; i += NT) out[r * width + i] = src[i];
    return;
  }
  const float s = scales[r];
  for (int i = threadIdx.x; i < width; i += NT)
    st_f32(out, r * width + i, ld_f32(src, i) * s);
}

template <typename T>
__global__ void combine_rows_kernel(float* __restrict__ out,
                                    const T* __restrict__ y,
                                    const int* __restrict__ index, int top,
                                    const T* __restrict__ extra,
                                    long extra_stride, int width,
                                    const float* __restrict__ weights,
                                    const T* __restrict__ scaled,
                                    long scaled_stride,
                                    const float* __restrict__ scaled_w) {
  const long t = blockIdx.x;
  const bool vec = (width % 4) == 0 && (extra_stride % 4) == 0 &&
                   (scaled_stride % 4) == 0 &&
                   ((uintptr_t)y % (4 * sizeof(T))) == 0 &&
                   ((uintptr_t)extra % (4 * sizeof(T))) == 0 &&
                   ((uintptr_t)scaled % (4 * sizeof(T))) == 0 &&
                   ((uintptr_t)out % 16) == 0;
  if (vec) {
    for (int i = threadIdx.x * 4; i < width; i += NT * 4) {
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
      for (int k = 0; k < top; ++k) {
        float x[4];
        ld4_any(y + (long)index[t * top + k] * width + i, x);
        const float wk = weights ? weights[t * top + k] : 1.0f;
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] += wk * x[c];
      }
      if (extra) {
        float x[4];
        ld4_any(extra + t * extra_stride + i, x);
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] += x[c];
      }
      if (scaled) {
        float x[4];
        ld4_any(scaled + t * scaled_stride + i, x);
        const float ws = scaled_w[t];
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] += ws * x[c];
      }
      *reinterpret_cast<float4_t*>(out + t * width + i) =
          float4_t{acc[0], acc[1], acc[2], acc[3]};
    }
    return;
  }
  for (int i = threadIdx.x; i < width; i += NT) {
    float acc = 0.f;
    for (int k = 0; k < top; ++k)
      acc += (weights ? weights[t * top + k] : 1.0f) *
             ld_f32(y, (long)index[t * top + k] * width + i);
    if (extra) acc += ld_f32(extra, t * extra_stride + i);
    if (scaled) acc += scaled_w[t] * ld_f32(scaled, t * scaled_stride + i);
    out[t * width + i] = acc;
  }
}

}  // namespace

extern "C" hipError_t ks_router_topk(void* idx_out, void* w_out,
                                     void* dense_out, const void* logits,
                                     int tokens, int E, int top, int softmax,
                                     int renorm, const void* correction,
                                     float renorm_eps, float weight_scale,
                                     hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (E < 1 || E > 64 * MAX_PER_LANE || top < 1 || top > E || top > 64)
    return hipErrorInvalidValue;
  hipLaunchKernelGGL(router_topk_kernel, dim3(cdiv(tokens, NW)), dim3(NT), 0,
                     stream, (int*)idx_out, (float*)w_out, (float*)dense_out,
                     (const float*)logits, tokens, E, top, softmax, renorm,
                     (const float*)correction, renorm_eps, weight_scale);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_route_tokens(void* idx_out, void* w_out,
                                      void* dense_out, void* logits_out,
                                      const void* h, long h_stride,
                                      const void* router, int tokens, int W,
                                      int E, int top, int softmax, int renorm,
                                      const void* correction, float renorm_eps, float weight_scale,
                                      int is_f32, hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (E < 1 || E > 64 * MAX_PER_LANE || top < 1 || top > E || top > 64 ||
      W < 1 || W + E > 15 * 1024)
    return hipErrorInvalidValue;
  const size_t smem = sizeof(float) * (size_t)(((W + 3) & ~3) + E);
  if (is_f32) {
    if (smem > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(
          (const void*)route_tokens_kernel<float>,
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(route_tokens_kernel<float>, dim3(tokens), dim3(NT), smem,
                       stream, (int*)idx_out, (float*)w_out, (float*)dense_out,
                       (float*)logits_out, (const float*)h, h_stride,
                       (const float*)router, W, E, top, softmax, renorm,
                       (const float*)correction, renorm_eps, weight_scale);
  } else {
    if (smem > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(
          (const void*)route_tokens_kernel<short>,
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(route_tokens_kernel<short>, dim3(tokens), dim3(NT), smem,
                       stream, (int*)idx_out, (float*)w_out, (float*)dense_out,
                       (float*)logits_out, (const short*)h, h_stride,
                       (const float*)router, W, E, top, softmax, renorm,
                       (const float*)correction, renorm_eps, weight_scale);
  }
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_gather_scale_rows(void* out, const void* x,
                                           long x_stride, const void* rows,
                                           const void* scales, int n_rows,
                                           int width, int is_f32,
                                           hipStream_t stream) {
  if (n_rows == 0) return hipSuccess;
  if (is_f32)
    hipLaunchKernelGGL(gather_scale_rows_kernel<float>, dim3(n_rows), dim3(NT),
                       0, stream, (float*)out, (const float*)x, x_stride,
                       (const int*)rows, (const float*)scales, width);
  else
    hipLaunchKernelGGL(gather_scale_rows_kernel<short>, dim3(n_rows), dim3(NT),
                       0, stream, (short*)out, (const short*)x, x_stride,
                       (const int*)rows, (const float*)scales, width);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_combine_rows(void* out, const void* y,
                                      const void* index, int top,
                                      const void* extra, long extra_stride,
                                      int tokens, int width, int is_f32,
                                      const void* weights, const void* scaled,
                                      long scaled_stride, const void* scaled_w,
                                      hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (scaled && !scaled_w) return hipErrorInvalidValue;
  if (is_f32)
    hipLaunchKernelGGL(combine_rows_kernel<float>, dim3(tokens), dim3(NT), 0,
                       stream, (float*)out, (const float*)y, (const int*)index,
                       top, (const float*)extra, extra_stride, width,
                       (const float*)weights, (const float*)scaled,
                       scaled_stride, (const float*)scaled_w);
  else
    hipLaunchKernelGGL(combine_rows_kernel<short>, dim3(tokens), dim3(NT), 0,
                       stream, (float*)out, (const short*)y, (const int*)index,
                       top, (const short*)extra, extra_stride, width,
                       (const float*)weights, (const short*)scaled,
                       scaled_stride, (const float*)scaled_w);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}
