// Norms over an fp32 residual stream, plus the embedding that starts it.
//
//  * embed_scale_sinpos: row = table[token] * scale + interleaved sinusoid
//    (even entry sin, odd entry cos of position * inv_freq[i]); fp32 out.
//  * add_rms_norm_f32res: residual += s0*d0 + s1*d1 (fp32, in place), then
//    out = residual / sqrt(mean(residual^2) + eps) * (w_offset + w).
//    The deltas are sublayer outputs in the activation dtype; either may be
//    absent. One kernel covers "add the previous sublayer, norm for the next".
//  * post_norm_add_rms_norm: closes a sandwich-normed sublayer and opens the
//    next one: residual += layer_scale * (delta / rms(delta) * post_gain),
//    += an optional per-token row and an optional shared row, then
//    out = residual / rms(residual) * next_gain. Both norms have ONE gain for
//    all channels (host scalars).
//  * post_layer_norm_add: residual += mult * LayerNorm(delta) * weight (mean
//    removed, biased variance, no bias term: the norm sits on the sublayer's
//    OUTPUT), then either out = residual in the activation dtype (the next
//    sublayer reads the stream itself) or out = LayerNorm(residual) *
//    next_weight (the model's final norm). Variances are two-pass.
//  * gated_group_rms_norm (gate_after set: the norm of y first, the gate on
//    the normed value; a weight shorter than the row repeats; no weight = 1)
//    otherwise: v = y * silu(z), normalised separately in equal
//    contiguous groups of the row, times a weight (gate before the norm).
//
// Everything is accumulated in fp32 with exact (non-approximate) sqrt and
// division: these ops sit on the 32-bit path of the models that use them.
#include "dtype_io.h"

namespace {

constexpr int NT = 256;
constexpr int NW = NT / WAVE_SIZE;

template <typename T>
__global__ void embed_scale_sinpos_kernel(float* __restrict__ out,
                                          const T* __restrict__ table,
                                          const long* __restrict__ tokens,
                                          const long* __restrict__ positions,
                                          const float* __restrict__ inv_freq,
                                          float scale, int width) {
  const long t = blockIdx.x;
  const long tok = tokens[t];
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < width; i += NT) {
    float pe = 0.f;  // no table of frequencies: no positional term
    if (inv_freq) {
      const float ang = pos * inv_freq[i >> 1];
      pe = (i & 1) ? cosf(ang) : sinf(ang);
    }
    out[t * width + i] = ld_f32(table, tok * width + i) * scale + pe;
  }
}

template <typename TD, typename TO>
__global__ void add_rms_norm_f32res_kernel(
    float* __restrict__ residual, const TD* __restrict__ d0, long d0_stride,
    float s0, const TD* __restrict__ d1, long d1_stride, float s1,
    const float* __restrict__ weight, float w_offset, float eps,
    TO* __restrict__ out, int width) {
  __shared__ float scratch[NW];
  const long row = blockIdx.x;
  float* r = residual + row * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) {
    float v = r[i];
    if (d0) v += s0 * ld_f32(d0, row * d0_stride + i);
    if (d1) v += s1 * ld_f32(d1, row * d1_stride + i);
    if (d0 || d1) r[i] = v;
    ss += v * v;
  }
  ss = block_sum_sync<NW>(ss, scratch);
  if (!out) return;
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += NT) {
    // each thread re-reads only what it wrote itself
    st_f32(out, row * width + i, r[i] * inv * (w_offset + weight[i]));
  }
}

// 4 elements per lane and step, the row kept in registers between the two
// passes (rows up to 256 * 4 * VEC_STEPS wide); picked by the launcher when
// widths, strides and pointers are 4-element aligned
constexpr int VEC_STEPS = 8;

template <typename T>
__device__ __forceinline__ void ld4(const T* p, float* v);
template <>
__device__ __forceinline__ void ld4<float>(const float* p, float* v) {
  const float4_t x = *reinterpret_cast<const float4_t*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = x[i];
}
template <>
__device__ __forceinline__ void ld4<short>(const short* p, float* v) {
  const short4_t x = *reinterpret_cast<const short4_t*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = bf16_bits_to_float(x[i]);
}
template <typename T>
__device__ __forceinline__ void st4(T* p, const float* v);
template <>
__device__ __forceinline__ void st4<float>(float* p, const float* v) {
  *reinterpret_cast<float4_t*>(p) = float4_t{v[0], v[1], v[2], v[3]};
}
template <>
__device__ __forceinline__ void st4<short>(short* p, const float* v) {
  short4_t o;
#pragma unroll
  for (int i = 0; i < 4; ++i) o[i] = float_to_bf16_bits(v[i]);
  *reinterpret_cast<short4_t*>(p) = o;
}

template <typename TD, typename TO>
__global__ void add_rms_norm_f32res_vec4_kernel(
    float* __restrict__ residual, const TD* __restrict__ d0, long d0_stride,
    float s0, const TD* __restrict__ d1, long d1_stride, float s1,
    const float* __restrict__ weight, float w_offset, float eps,
    TO* __restrict__ out, int width) {
  __shared__ float scratch[NW];
  const long row = blockIdx.x;
  float* r = residual + row * width;
  float keep[VEC_STEPS][4];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VEC_STEPS; ++k) {
    const int i = (threadIdx.x + NT * k) * 4;
    if (i < width) {
      float v[4], d[4];
      ld4<float>(r + i, v);
      if (d0) {
        ld4<TD>(d0 + row * d0_stride + i, d);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] += s0 * d[j];
      }
      if (d1) {
        ld4<TD>(d1 + row * d1_stride + i, d);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] += s1 * d[j];
      }
      if (d0 || d1) st4<float>(r + i, v);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        keep[k][j] = v[j];
        ss += v[j] * v[j];
      }
    }
  }
  ss = block_sum_sync<NW>(ss, scratch);
  if (!out) return;
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int k = 0; k < VEC_STEPS; ++k) {
    const int i = (threadIdx.x + NT * k) * 4;
    if (i < width) {
      float w[4], o[4];
      ld4<float>(weight + i, w);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = keep[k][j] * inv * (w_offset + w[j]);
      st4<TO>(out + row * width + i, o);
    }
  }
}

template <typename TD, typename TO>
__global__ void post_layer_norm_add_kernel(
    float* __restrict__ residual, const TD* __restrict__ delta,
    long delta_stride, const float* __restrict__ weight, float mult, float eps,
    TO* __restrict__ out, const float* __restrict__ next_weight, int width) {
  __shared__ float scratch[NW];
  const long row = blockIdx.x;
  float* r = residual + row * width;
  const float inv_w = 1.0f / (float)width;
  if (delta) {
    const TD* d = delta + row * delta_stride;
    float sm = 0.f;
    for (int i = threadIdx.x; i < width; i += NT) sm += ld_f32(d, i);
    const float mean = block_sum_sync<NW>(sm, scratch) * inv_w;
    float sv = 0.f;
    for (int i = threadIdx.x; i < width; i += NT) {
      const float c = ld_f32(d, i) - mean;
      sv += c * c;
    }
    sv = block_sum_sync<NW>(sv, scratch);
    const float inv = 1.0f / sqrtf(sv * inv_w + eps);
    for (int i = threadIdx.x; i < width; i += NT)
      r[i] += mult * ((ld_f32(d, i) - mean) * inv * weight[i]);
  }
  if (!out) return;
  // each thread re-reads only what it wrote itself
  if (!next_weight) {
    for (int i = threadIdx.x; i < width; i += NT)
      st_f32(out, row * width + i, r[i]);
    return;
  }
  float sm = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) sm += r[i];
  const float mean = block_sum_sync<NW>(sm, scratch) * inv_w;
  float sv = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) {
    const float c = r[i] - mean;
    sv += c * c;
  }
  sv = block_sum_sync<NW>(sv, scratch);
  const float inv = 1.0f / sqrtf(sv * inv_w + eps);
  for (int i = threadIdx.x; i < width; i += NT)
    st_f32(out, row * width + i, (r[i] - mean) * inv * next_weight[i]);
}

// the row stays in registers between the passes
template <typename TD, typename TO>
__global__ void post_layer_norm_add_vec4_kernel(
    float* __restrict__ residual, const TD* __restrict__ delta,
    long delta_stride, const float* __restrict__ weight, float mult, float eps,
    TO* __restrict__ out, const float* __restrict__ next_weight, int width) {
  __shared__ float scratch[NW];
  const long row = blockIdx.x;
  float* r = residual + row * width;
  const float inv_w = 1.0f / (float)width;
  float keep[VEC_STEPS][4];
  if (delta) {
    float sm = 0.f;
#pragma unroll
    for (int k = 0; k < VEC_STEPS; ++k) {
      const int i = (threadIdx.x + NT * k) * 4;
      if (i < width) {
        ld4<TD>(delta + row * delta_stride + i, keep[k]);
#pragma unroll
        for (int j = 0; j < 4; ++j) sm += keep[k][j];
      }
    }
    const float mean = block_sum_sync<NW>(sm, scratch) * inv_w;
    float sv = 0.f;
#pragma unroll
    for (int k = 0; k < VEC_STEPS; ++k) {
      const int i = (threadIdx.x + NT * k) * 4;
      if (i < width) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          keep[k][j] -= mean;
          sv += keep[k][j] * keep[k][j];
        }
      }
    }
    sv = block_sum_sync<NW>(sv, scratch);
    const float inv = 1.0f / sqrtf(sv * inv_w + eps);
#pragma unroll
    for (int k = 0; k < VEC_STEPS; ++k) {
      const int i = (threadIdx.x + NT * k) * 4;
      if (i < width) {
        float v[4], w[4];
        ld4<float>(r + i, v);
        ld4<float>(weight + i, w);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v[j] += mult * (keep[k][j] * inv * w[j]);
          keep[k][j] = v[j];
        }
        st4<float>(r + i, v);
      }
    }
  } else if (out) {
#pragma unroll
    for (int k = 0; k < VEC_STEPS; ++k) {
      const int i = (threadIdx.x + NT * k) * 4;
      if (i < width) ld4<float>(r + i, keep[k]);
    }
  }
  if (!out) return;
  if (!next_weight) {
#pragma unroll
    for (int k = 0; k < VEC_STEPS; ++k) {
      const int i = (threadIdx.x + NT * k) * 4;
      if (i < width) st4<TO>(out + row * width + i, keep[k]);
    }
    return;
  }
  float sm = 0.f;
#pragma unroll
  for (int k = 0; k < VEC_STEPS; ++k) {
    const int i = (threadIdx.x + NT * k) * 4;
    if (i < width) {
#pragma unroll
      for (int j = 0; j < 4; ++j) sm += keep[k][j];
    }
  }
  const float mean = block_sum_sync<NW>(sm, scratch) * inv_w;
  float sv = 0.f;
#pragma unroll
  for (int k = 0; k < VEC_STEPS; ++k) {
    const int i = (threadIdx.x + NT * k) * 4;
    if (i < width) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        keep[k][j] -= mean;
        sv += keep[k][j] * keep[k][j];
      }
    }
  }
  sv = block_sum_sync<NW>(sv, scratch);
  const float inv = 1.0f / sqrtf(sv * inv_w + eps);
#pragma unroll
  for (int k = 0; k < VEC_STEPS; ++k) {
    const int i = (threadIdx.x + NT * k) * 4;
    if (i < width) {
      float w[4], o[4];
      ld4<float>(next_weight + i, w);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = keep[k][j] * inv * w[j];
      st4<TO>(out + row * width + i, o);
    }
  }
}

template <typename TD, typename TO>
__global__ void post_norm_add_rms_norm_kernel(
    float* __restrict__ residual, const TD* __restrict__ delta,
    long delta_stride, float post_gain, const float* __restrict__ layer_scale,
    const float* __restrict__ add_rows, const float* __restrict__ add_vec,
    float eps, float next_gain, TO* __restrict__ out, int width) {
  __shared__ float scratch[NW];
  const long row = blockIdx.x;
  float* r = residual + row * width;
  float dinv = 0.f;
  if (delta) {
    float sd = 0.f;
    for (int i = threadIdx.x; i < width; i += NT) {
      const float d = ld_f32(delta, row * delta_stride + i);
      sd += d * d;
    }
    sd = block_sum_sync<NW>(sd, scratch);
    dinv = 1.0f / sqrtf(sd / (float)width + eps);
  }
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += NT) {
    float v = r[i];
    if (delta)
      v += ld_f32(delta, row * delta_stride + i) * dinv * post_gain * layer_scale[i];
    if (add_rows) v += add_rows[row * width + i];
    if (add_vec) v += add_vec[i];
    if (delta || add_rows || add_vec) r[i] = v;
    ss += v * v;
  }
  if (!out) return;
  ss = block_sum_sync<NW>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += NT)
    // each thread re-reads only what it wrote itself
    st_f32(out, row * width + i, r[i] * inv * next_gain);
}

template <typename TD, typename TO>
__global__ void post_norm_add_rms_norm_vec4_kernel(
    float* __restrict__ residual, const TD* __restrict__ delta,
    long delta_stride, float post_gain, const float* __restrict__ layer_scale,
    const float* __restrict__ add_rows, const float* __restrict__ add_vec,
    float eps, float next_gain, TO* __restrict__ out, int width) {
  __shared__ float scratch[NW];
  const long row = blockIdx.x;
  float* r = residual + row * width;
  float keep[VEC_STEPS][4];
  float dinv = 0.f;
  if (delta) {
    float sd = 0.f;
#pragma unroll
    for (int k = 0; k < VEC_STEPS; ++k) {
      const int i = (threadIdx.x + NT * k) * 4;
      if (i < width) {
        ld4<TD>(delta + row * delta_stride + i, keep[k]);
#pragma unroll
        for (int j = 0; j < 4; ++j) sd += keep[k][j] * keep[k][j];
      }
    }
    sd = block_sum_sync<NW>(sd, scratch);
    dinv = 1.0f / sqrtf(sd / (float)width + eps);
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VEC_STEPS; ++k) {
    const int i = (threadIdx.x + NT * k) * 4;
    if (i < width) {
      float v[4], a[4];
      ld4<float>(r + i, v);
      if (delta) {
        ld4<float>(layer_scale + i, a);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] += keep[k][j] * dinv * post_gain * a[j];
      }
      if (add_rows) {
        ld4<float>(add_rows + row * width + i, a);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] += a[j];
      }
      if (add_vec) {
        ld4<float>(add_vec + i, a);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] += a[j];
      }
      if (delta || add_rows || add_vec) st4<float>(r + i, v);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        keep[k][j] = v[j];
        ss += v[j] * v[j];
      }
    }
  }
  if (!out) return;
  ss = block_sum_sync<NW>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int k = 0; k < VEC_STEPS; ++k) {
    const int i = (threadIdx.x + NT * k) * 4;
    if (i < width) {
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = keep[k][j] * inv * next_gain;
      st4<TO>(out + row * width + i, o);
    }
  }
}

template <typename TZ, typename TO>
__global__ void gated_group_rms_norm_kernel(TO* __restrict__ out,
                                            const float* __restrict__ y,
                                            const TZ* __restrict__ z,
                                            long z_stride,
                                            const float* __restrict__ weight,
                                            int weight_n, float eps, int inner,
                                            int group_size, int gate_after) {
  __shared__ float scratch[NW];
  const long row = blockIdx.x;
  const int g0 = blockIdx.y * group_size;
  float ss = 0.f;
  for (int i = threadIdx.x; i < group_size; i += NT) {
    const float zf = ld_f32(z, row * z_stride + g0 + i);
    const float yv = y[row * inner + g0 + i];
    const float v = gate_after ? yv : yv * (zf / (1.0f + expf(-zf)));
    ss += v * v;
  }
  ss = block_sum_sync<NW>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)group_size + eps);
  for (int i = threadIdx.x; i < group_size; i += NT) {
    const float zf = ld_f32(z, row * z_stride + g0 + i);
    const float gate = zf / (1.0f + expf(-zf));
    const float yv = y[row * inner + g0 + i];
    const float w = weight ? weight[(g0 + i) % weight_n] : 1.0f;
    st_f32(out, row * inner + g0 + i,
           gate_after ? yv * inv * w * gate : yv * gate * inv * w);
  }
}

template <typename TZ, typename TO>
__global__ void gated_group_rms_norm_vec4_kernel(
    TO* __restrict__ out, const float* __restrict__ y, const TZ* __restrict__ z,
    long z_stride, const float* __restrict__ weight, int weight_n, float eps,
    int inner, int group_size, int gate_after) {
  __shared__ float scratch[NW];
  const long row = blockIdx.x;
  const int g0 = blockIdx.y * group_size;
  float keep[VEC_STEPS][4], gate[VEC_STEPS][4];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VEC_STEPS; ++k) {
    const int i = (threadIdx.x + NT * k) * 4;
    if (i < group_size) {
      float yv[4], zv[4];
      ld4<float>(y + row * inner + g0 + i, yv);
      ld4<TZ>(z + row * z_stride + g0 + i, zv);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float sg = zv[j] / (1.0f + expf(-zv[j]));
        const float v = gate_after ? yv[j] : yv[j] * sg;
        gate[k][j] = gate_after ? sg : 1.0f;
        keep[k][j] = v;
        ss += v * v;
      }
    }
  }
  ss = block_sum_sync<NW>(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)group_size + eps);
#pragma unroll
  for (int k = 0; k < VEC_STEPS; ++k) {
    const int i = (threadIdx.x + NT * k) * 4;
    if (i < group_size) {
      float w[4] = {1.f, 1.f, 1.f, 1.f}, o[4];
      if (weight) ld4<float>(weight + (g0 + i) % weight_n, w);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = keep[k][j] * inv * w[j] * gate[k][j];
      st4<TO>(out + row * inner + g0 + i, o);
    }
  }
}

// Groups of at most 256 elements (heads of a recurrent read-out): a block
// takes a whole row and each of its waves a group at a time, 4 elements per
// lane, so a row costs one block instead of one block per group.
template <typename TZ, typename TO>
__global__ void __launch_bounds__(NT) gated_group_rms_norm_wave_kernel(
    TO* __restrict__ out, const float* __restrict__ y, const TZ* __restrict__ z,
    long z_stride, const float* __restrict__ weight, int weight_n, float eps,
    int inner, int group_size, int groups, int gate_after) {
  const long row = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int i = lane * 4;
  const bool on = i < group_size;
  for (int g = threadIdx.x >> 6; g < groups; g += NW) {
    const int g0 = g * group_size;
    float v[4] = {0.f, 0.f, 0.f, 0.f}, gate[4] = {1.f, 1.f, 1.f, 1.f};
    float ss = 0.f;
    if (on) {
      float zv[4];
      ld4<float>(y + row * inner + g0 + i, v);
      ld4<TZ>(z + row * z_stride + g0 + i, zv);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float sg = zv[j] / (1.0f + expf(-zv[j]));
        if (gate_after) gate[j] = sg;
        else v[j] *= sg;
        ss += v[j] * v[j];
      }
    }
    ss = wave_reduce_sum(ss);
    if (on) {
      const float inv = 1.0f / sqrtf(ss / (float)group_size + eps);
      float w[4] = {1.f, 1.f, 1.f, 1.f}, o[4];
      if (weight) ld4<float>(weight + (g0 + i) % weight_n, w);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = v[j] * inv * w[j] * gate[j];
      st4<TO>(out + row * inner + g0 + i, o);
    }
  }
}

}  // namespace

extern "C" hipError_t ks_embed_scale_sinpos(void* out, const void* table,
                                            const void* tokens,
                                            const void* positions,
                                            const void* inv_freq, float scale,
                                            int rows, int width, int is_f32,
                                            hipStream_t stream) {
  if (rows == 0) return hipSuccess;
  if (is_f32)
    hipLaunchKernelGGL(embed_scale_sinpos_kernel<float>, dim3(rows), dim3(NT),
                       0, stream, (float*)out, (const float*)table,
                       (const long*)tokens, (const long*)positions,
                       (const float*)inv_freq, scale, width);
  else
    hipLaunchKernelGGL(embed_scale_sinpos_kernel<short>, dim3(rows), dim3(NT),
                       0, stream, (float*)out, (const short*)table,
                       (const long*)tokens, (const long*)positions,
                       (const float*)inv_freq, scale, width);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_add_rms_norm_f32res(
    void* residual, const void* d0, long d0_stride, float s0, const void* d1,
    long d1_stride, float s1, const void* weight, float w_offset, float eps,
    void* out, int rows, int width, int is_f32, int d_is_f32,
    hipStream_t stream) {
  if (rows == 0) return hipSuccess;
  const int esz = is_f32 ? 4 : 2;
  const int dsz = d_is_f32 ? 4 : 2;
  auto al = [](const void* p, int bytes) { return ((uintptr_t)p % bytes) == 0; };
  const bool vec = width % 4 == 0 && width <= NT * 4 * VEC_STEPS &&
                   d0_stride % 4 == 0 && d1_stride % 4 == 0 &&
                   al(residual, 16) && al(weight, 16) && al(d0, 4 * dsz) &&
                   al(d1, 4 * dsz) && al(out, 4 * esz);
#define NORM_ARGS(TT)                                                         \
  (float*)residual, (const TT*)d0, d0_stride, s0, (const TT*)d1, d1_stride,   \
      s1, (const float*)weight, w_offset, eps, (TT*)out, width
#define NORM_ARGS_MIXED                                                       \
  (float*)residual, (const float*)d0, d0_stride, s0, (const float*)d1,        \
      d1_stride, s1, (const float*)weight, w_offset, eps, (short*)out, width
  if (!is_f32 && d_is_f32) {
    // fp32 deltas (an fp32 sum of sublayer outputs) beside a bf16 output
    if (vec)
      hipLaunchKernelGGL((add_rms_norm_f32res_vec4_kernel<float, short>),
                         dim3(rows), dim3(NT), 0, stream, NORM_ARGS_MIXED);
    else
      hipLaunchKernelGGL((add_rms_norm_f32res_kernel<float, short>), dim3(rows),
                         dim3(NT), 0, stream, NORM_ARGS_MIXED);
  } else if (is_f32) {
    if (vec)
      hipLaunchKernelGGL((add_rms_norm_f32res_vec4_kernel<float, float>),
                         dim3(rows), dim3(NT), 0, stream, NORM_ARGS(float));
    else
      hipLaunchKernelGGL((add_rms_norm_f32res_kernel<float, float>), dim3(rows),
                         dim3(NT), 0, stream, NORM_ARGS(float));
  } else {
    if (vec)
      hipLaunchKernelGGL((add_rms_norm_f32res_vec4_kernel<short, short>),
                         dim3(rows), dim3(NT), 0, stream, NORM_ARGS(short));
    else
      hipLaunchKernelGGL((add_rms_norm_f32res_kernel<short, short>), dim3(rows),
                         dim3(NT), 0, stream, NORM_ARGS(short));
  }
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

template <typename TD, typename TO>
static void launch_post_norm(bool vec, void* residual, const void* delta,
                             long delta_stride, float post_gain,
                             const void* layer_scale, const void* add_rows,
                             const void* add_vec, float eps, float next_gain,
                             void* out, int rows, int width,
                             hipStream_t stream) {
  auto fn = vec ? post_norm_add_rms_norm_vec4_kernel<TD, TO>
                : post_norm_add_rms_norm_kernel<TD, TO>;
  hipLaunchKernelGGL(fn, dim3(rows), dim3(NT), 0, stream, (float*)residual,
                     (const TD*)delta, delta_stride, post_gain,
                     (const float*)layer_scale, (const float*)add_rows,
                     (const float*)add_vec, eps, next_gain, (TO*)out, width);
}

extern "C" hipError_t ks_post_norm_add_rms_norm(
    void* residual, const void* delta, long delta_stride, int delta_is_f32,
    float post_gain, const void* layer_scale, const void* add_rows,
    const void* add_vec, float eps, float next_gain, void* out, int out_is_f32,
    int rows, int width, hipStream_t stream) {
  if (rows == 0) return hipSuccess;
  if (delta && !layer_scale) return hipErrorInvalidValue;
  auto al = [](const void* p, int bytes) { return ((uintptr_t)p % bytes) == 0; };
  const bool vec = width % 4 == 0 && width <= NT * 4 * VEC_STEPS &&
                   delta_stride % 4 == 0 && al(residual, 16) &&
                   al(layer_scale, 16) && al(add_rows, 16) && al(add_vec, 16) &&
                   al(delta, delta_is_f32 ? 16 : 8) &&
                   al(out, out_is_f32 ? 16 : 8);
#define PN_ARGS                                                                vec, residual, delta, delta_stride, post_gain, layer_scale, add_rows,            add_vec, eps, next_gain, out, rows, width, stream
  if (delta_is_f32) {
    if (out_is_f32) launch_post_norm<float, float>(PN_ARGS);
    else launch_post_norm<float, short>(PN_ARGS);
  } else {
    if (out_is_f32) launch_post_norm<short, float>(PN_ARGS);
    else launch_post_norm<short, short>(PN_ARGS);
  }
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

template <typename TD, typename TO>
void launch_post_ln(bool vec, void* residual, const void* delta,
                    long delta_stride, const void* weight, float mult,
                    float eps, void* out, const void* next_weight, int rows,
                    int width, hipStream_t stream) {
  auto fn = vec ? post_layer_norm_add_vec4_kernel<TD, TO>
                : post_layer_norm_add_kernel<TD, TO>;
  hipLaunchKernelGGL(fn, dim3(rows), dim3(NT), 0, stream, (float*)residual,
                     (const TD*)delta, delta_stride, (const float*)weight, mult,
                     eps, (TO*)out, (const float*)next_weight, width);
}

extern "C" hipError_t ks_post_layer_norm_add(
    void* residual, const void* delta, long delta_stride, int delta_is_f32,
    const void* weight, float mult, float eps, void* out, int out_is_f32,
    const void* next_weight, int rows, int width, hipStream_t stream) {
  if (rows == 0) return hipSuccess;
  if (delta && !weight) return hipErrorInvalidValue;
  if (!delta && !out) return hipSuccess;
  auto al = [](const void* p, int bytes) { return ((uintptr_t)p % bytes) == 0; };
  const bool vec = width % 4 == 0 && width <= NT * 4 * VEC_STEPS &&
                   delta_stride % 4 == 0 && al(residual, 16) && al(weight, 16) &&
                   al(next_weight, 16) && al(delta, delta_is_f32 ? 16 : 8) &&
                   al(out, out_is_f32 ? 16 : 8);
#define PLN_ARGS                                                             \
  vec, residual, delta, delta_stride, weight, mult, eps, out, next_weight,   \
      rows, width, stream
  if (delta_is_f32) {
    if (out_is_f32) launch_post_ln<float, float>(PLN_ARGS);
    else launch_post_ln<float, short>(PLN_ARGS);
  } else {
    if (out_is_f32) launch_post_ln<short, float>(PLN_ARGS);
    else launch_post_ln<short, short>(PLN_ARGS);
  }
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_gated_group_rms_norm(void* out, const void* y,
                                              const void* z, long z_stride,
                                              const void* weight, int weight_n,
                                              float eps, int rows, int inner,
                                              int groups, int gate_after,
                                              int is_f32,
                                              hipStream_t stream) {
  if (rows == 0) return hipSuccess;
  if (groups <= 0 || inner % groups != 0) return hipErrorInvalidValue;
  const int gs = inner / groups;
  // a weight shorter than the row repeats (one weight vector per group)
  if (weight && (weight_n <= 0 || inner % weight_n != 0 ||
                 (weight_n != inner && weight_n % gs != 0 && gs % weight_n != 0)))
    return hipErrorInvalidValue;
  const int esz = is_f32 ? 4 : 2;
  const bool vec = gs % 4 == 0 && gs <= NT * 4 * VEC_STEPS && z_stride % 4 == 0 &&
                   (!weight || weight_n % 4 == 0) &&
                   ((uintptr_t)y % 16) == 0 && ((uintptr_t)weight % 16) == 0 &&
                   ((uintptr_t)z % (4 * esz)) == 0 &&
                   ((uintptr_t)out % (4 * esz)) == 0;
#define GNORM_ARGS(TT)                                                        \
  (TT*)out, (const float*)y, (const TT*)z, z_stride, (const float*)weight,    \
      weight_n, eps, inner, gs
  if (vec && gs <= 4 * WAVE_SIZE && groups > 1) {
    if (is_f32)
      hipLaunchKernelGGL((gated_group_rms_norm_wave_kernel<float, float>),
                         dim3(rows), dim3(NT), 0, stream, GNORM_ARGS(float),
                         groups, gate_after);
    else
      hipLaunchKernelGGL((gated_group_rms_norm_wave_kernel<short, short>),
                         dim3(rows), dim3(NT), 0, stream, GNORM_ARGS(short),
                         groups, gate_after);
    HIP_CHECK_KERNEL();
    return hipSuccess;
  }
  if (is_f32) {
    if (vec)
      hipLaunchKernelGGL((gated_group_rms_norm_vec4_kernel<float, float>),
                         dim3(rows, groups), dim3(NT), 0, stream,
                         GNORM_ARGS(float), gate_after);
    else
      hipLaunchKernelGGL((gated_group_rms_norm_kernel<float, float>),
                         dim3(rows, groups), dim3(NT), 0, stream,
                         GNORM_ARGS(float), gate_after);
  } else {
    if (vec)
      hipLaunchKernelGGL((gated_group_rms_norm_vec4_kernel<short, short>),
                         dim3(rows, groups), dim3(NT), 0, stream,
                         GNORM_ARGS(short), gate_after);
    else
      hipLaunchKernelGGL((gated_group_rms_norm_kernel<short, short>),
                         dim3(rows, groups), dim3(NT), 0, stream,
                         GNORM_ARGS(short), gate_after);
  }
  HIP_CHECK_KERNEL();
  return hipSuccess;
}
