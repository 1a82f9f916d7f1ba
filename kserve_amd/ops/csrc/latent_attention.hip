// The steps around attention over one cached latent row per token.
//
//  * latent_norm_rope_cache: a block per token. The token's projection row is
//    [query latent | kv latent | key part | ...]. The query latent is
//    RMS-normed (x / sqrt(mean(x^2) + eps) * w) and written out in the
//    activation dtype. With a cache, the kv latent is RMS-normed the same way
//    and the key part is rotated in pairs (2i, 2i+1) by pos * inv_freq[i]
//    (fp32 angle, exact sin/cos; pairs past the frequency table and an odd
//    last coordinate are copied); [normed latent | rotated key part] is the
//    token's row of the paged cache [blocks, 1, block, kv_rank + rot_dim].
//  * head_matmul_rope: per head h, out[t, h, :n] = x[t, h, :k] W[h] with
//    W [heads, k, n] (fp32 sums), and the `tail` coordinates after the first
//    k copied behind the product after the same pair rotation. It folds the
//    queries into latent coordinates (q_h^T U_k[h], tail = the query's
//    rotated part, fp32 out) and takes the weighted latent sums through
//    U_v[h] (tail 0, activation dtype out).
//    A block takes TT tokens of one head and 256 output columns: the x tile
//    sits in LDS as fp32 (read as broadcasts), a wave owns TT/4 tokens, a lane
//    up to 4 columns 64 apart, so W rows are read in 256-byte runs and every
//    W element loaded feeds TT/4 FMAs.
#include "dtype_io.h"

namespace {

constexpr int NT = 256;
constexpr int NW = NT / WAVE_SIZE;

template <typename T>
__global__ void __launch_bounds__(NT) latent_norm_rope_cache_kernel(
    T* __restrict__ cq_out, const T* __restrict__ proj, long row_stride,
    int q_rank, int kv_rank, int rot_dim, const float* __restrict__ qw,
    const float* __restrict__ kw, const long* __restrict__ positions,
    const int* __restrict__ slot_mapping, T* __restrict__ cache, float eps,
    const float* __restrict__ inv_freq, int half) {
  __shared__ float scratch[NW];
  const long t = blockIdx.x;
  const T* row = proj + t * row_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += NT) {
    const float x = ld_f32(row, i);
    ss += x * x;
  }
  ss = block_sum_sync<NW>(ss, scratch);
  const float qinv = 1.0f / sqrtf(ss / (float)q_rank + eps);
  for (int i = threadIdx.x; i < q_rank; i += NT)
    st_f32(cq_out, t * q_rank + i, ld_f32(row, i) * qinv * qw[i]);
  if (!cache) return;
  const long slot = slot_mapping[t];
  if (slot < 0) return;  // the whole block leaves together
  const T* c = row + q_rank;
  ss = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += NT) {
    const float x = ld_f32(c, i);
    ss += x * x;
  }
  ss = block_sum_sync<NW>(ss, scratch);
  const float cinv = 1.0f / sqrtf(ss / (float)kv_rank + eps);
  T* dst = cache + slot * (long)(kv_rank + rot_dim);
  for (int i = threadIdx.x; i < kv_rank; i += NT)
    st_f32(dst, i, ld_f32(c, i) * cinv * kw[i]);
  const T* kr = c + kv_rank;
  const float pos = (float)positions[t];
  for (int p = threadIdx.x; 2 * p < rot_dim; p += NT) {
    const float u = ld_f32(kr, 2 * p);
    if (2 * p + 1 >= rot_dim) {
      st_f32(dst, kv_rank + 2 * p, u);
    } else {
      const float v = ld_f32(kr, 2 * p + 1);
      float sn = 0.f, cs = 1.f;
      if (p < half) sincosf(pos * inv_freq[p], &sn, &cs);
      st_f32(dst, kv_rank + 2 * p, u * cs - v * sn);
      st_f32(dst, kv_rank + 2 * p + 1, v * cs + u * sn);
    }
  }
}

constexpr int TT = 32;         // tokens per block
constexpr int TPW = TT / NW;   // tokens per wave
constexpr int CPL = 4;         // columns per lane (64 apart)

template <typename T, typename TO>
__global__ void __launch_bounds__(NT) head_matmul_rope_kernel(
    TO* __restrict__ out, const T* __restrict__ x, long x_stride,
    const T* __restrict__ w, int tokens, int heads, int K, int N, int tail,
    const long* __restrict__ positions, const float* __restrict__ inv_freq,
    int half) {
  extern __shared__ float xs[];  // [TT][K]
  const int t0 = blockIdx.x * TT;
  const int h = blockIdx.y;
  const int n0 = blockIdx.z * (64 * CPL);
  const int nt = min(TT, tokens - t0);
  const int in_w = K + tail, out_w = N + tail;
  for (int e = threadIdx.x; e < TT * K; e += NT) {
    const int tt = e / K, k = e % K;
    xs[e] = tt < nt ? ld_f32(x, (long)(t0 + tt) * x_stride + (long)h * in_w + k)
                    : 0.f;
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float acc[TPW][CPL];
#pragma unroll
  for (int a = 0; a < TPW; ++a)
#pragma unroll
    for (int c = 0; c < CPL; ++c) acc[a][c] = 0.f;
  const T* wh = w + (long)h * K * N;
  const float* xw = xs + wave * TPW * K;
  for (int k = 0; k < K; ++k) {
    float wv[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const int n = n0 + lane + 64 * c;
      wv[c] = n < N ? ld_f32(wh, (long)k * N + n) : 0.f;
    }
#pragma unroll
    for (int a = 0; a < TPW; ++a) {
      const float xv = xw[a * K + k];
#pragma unroll
      for (int c = 0; c < CPL; ++c) acc[a][c] += xv * wv[c];
    }
  }
#pragma unroll
  for (int a = 0; a < TPW; ++a) {
    const int tt = wave * TPW + a;
    if (tt < nt) {
      const long o = ((long)(t0 + tt) * heads + h) * out_w;
#pragma unroll
      for (int c = 0; c < CPL; ++c) {
        const int n = n0 + lane + 64 * c;
        if (n < N) st_f32(out, o + n, acc[a][c]);
      }
    }
  }
  if (tail == 0 || blockIdx.z != 0) return;
  const int pairs = (tail + 1) / 2;
  for (int e = threadIdx.x; e < nt * pairs; e += NT) {
    const int tt = e / pairs, p = e % pairs;
    const long src = (long)(t0 + tt) * x_stride + (long)h * in_w + K;
    const long o = ((long)(t0 + tt) * heads + h) * out_w + N;
    const float u = ld_f32(x, src + 2 * p);
    if (2 * p + 1 >= tail) {
      st_f32(out, o + 2 * p, u);
    } else {
      const float v = ld_f32(x, src + 2 * p + 1);
      float sn = 0.f, cs = 1.f;
      if (p < half) sincosf((float)positions[t0 + tt] * inv_freq[p], &sn, &cs);
      st_f32(out, o + 2 * p, u * cs - v * sn);
      st_f32(out, o + 2 * p + 1, v * cs + u * sn);
    }
  }
}

}  // namespace

extern "C" hipError_t ks_latent_norm_rope_cache(
    void* cq_out, const void* proj, long row_stride, int tokens, int q_rank,
    int kv_rank, int rot_dim, const void* qw, const void* kw,
    const void* positions, const void* slot_mapping, void* cache, float eps,
    const void* inv_freq, int half, int is_f32, hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (q_rank < 1 || (cache && (kv_rank < 1 || !kw)) || 2 * half > rot_dim ||
      (half > 0 && !inv_freq))
    return hipErrorInvalidValue;
  if (is_f32)
    hipLaunchKernelGGL(latent_norm_rope_cache_kernel<float>, dim3(tokens),
                       dim3(NT), 0, stream, (float*)cq_out, (const float*)proj,
                       row_stride, q_rank, kv_rank, rot_dim, (const float*)qw,
                       (const float*)kw, (const long*)positions,
                       (const int*)slot_mapping, (float*)cache, eps,
                       (const float*)inv_freq, half);
  else
    hipLaunchKernelGGL(latent_norm_rope_cache_kernel<short>, dim3(tokens),
                       dim3(NT), 0, stream, (short*)cq_out, (const short*)proj,
                       row_stride, q_rank, kv_rank, rot_dim, (const float*)qw,
                       (const float*)kw, (const long*)positions,
                       (const int*)slot_mapping, (short*)cache, eps,
                       (const float*)inv_freq, half);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

template <typename T, typename TO>
static hipError_t launch_head_matmul(void* out, const void* x, long x_stride,
                                     const void* w, int tokens, int heads,
                                     int K, int N, int tail,
                                     const void* positions,
                                     const void* inv_freq, int half,
                                     hipStream_t stream) {
  const size_t smem = sizeof(float) * (size_t)TT * K;
  auto fn = head_matmul_rope_kernel<T, TO>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(
        (const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
  }
  dim3 grid(cdiv(tokens, TT), heads, cdiv(N, 64 * CPL));
  hipLaunchKernelGGL(fn, grid, dim3(NT), smem, stream, (TO*)out, (const T*)x,
                     x_stride, (const T*)w, tokens, heads, K, N, tail,
                     (const long*)positions, (const float*)inv_freq, half);
  return hipGetLastError();
}

// in_f32: dtype of x and w; out_f32: dtype of out (fp32 out with bf16 inputs
// keeps the folded queries unrounded)
extern "C" hipError_t ks_head_matmul_rope(void* out, const void* x,
                                          long x_stride, const void* w,
                                          int tokens, int heads, int K, int N,
                                          int tail, const void* positions,
                                          const void* inv_freq, int half,
                                          int in_f32, int out_f32,
                                          hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (heads < 1 || K < 1 || N < 1 || tail < 0 || 2 * half > tail ||
      (half > 0 && (!inv_freq || !positions)) || K > 1024 ||
      (in_f32 && !out_f32))
    return hipErrorInvalidValue;
#define HM_ARGS                                                              \
  out, x, x_stride, w, tokens, heads, K, N, tail, positions, inv_freq, half, \
      stream
  if (in_f32) return launch_head_matmul<float, float>(HM_ARGS);
  if (out_f32) return launch_head_matmul<short, float>(HM_ARGS);
  return launch_head_matmul<short, short>(HM_ARGS);
}
