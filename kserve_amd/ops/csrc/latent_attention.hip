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
//  * head_matmul_rope: per head h, out[t, h, :n] = W[h] x[t, h, :k] with
//    W [heads, n, k] (fp32 sums), and the `tail` coordinates after the first
//    k copied behind the product after the same pair rotation. It folds the
//    queries into latent coordinates (U_k[h]^T q_h, tail = the query's
//    rotated part, fp32 out) and takes the weighted latent sums through
//    U_v[h] (tail 0, activation dtype out). Aligned operands run on the
//    matrix cores straight from global memory; anything else takes a plain
//    LDS-tiled form.
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

// Pair rotation of the tail coordinates behind the product, for the tokens
// [t0, t0 + nt) of head h (all threads of the block take part).
template <typename T, typename TO>
__device__ __forceinline__ void rotate_tail(
    TO* __restrict__ out, const T* __restrict__ x, long x_stride, int t0,
    int nt, int h, int heads, int K, int N, int tail,
    const long* __restrict__ positions, const float* __restrict__ inv_freq,
    int half) {
  const int in_w = K + tail, out_w = N + tail;
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

// Any sizes and alignments: the x tile in LDS as fp32 (read as broadcasts),
// a wave owns TT/4 tokens, a lane up to 4 columns 64 apart.
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
  const T* wh = w + (long)h * N * K;  // [N][K]
  const float* xw = xs + wave * TPW * K;
  for (int k = 0; k < K; ++k) {
    float wv[CPL];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
      const int n = n0 + lane + 64 * c;
      wv[c] = n < N ? ld_f32(wh, (long)n * K + k) : 0.f;
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
  rotate_tail(out, x, x_stride, t0, nt, h, heads, K, N, tail, positions,
              inv_freq, half);
}

// Matrix-core form for 16-byte aligned operands (K, the head widths and the
// row stride multiples of 8 bf16 / 4 fp32). Both operands have the
// contraction index contiguous in memory, so every fragment is one 16-byte
// global load and nothing is staged in LDS. The weights are the A operand
// and the tokens the B operand: C^T[n][token], so a lane ends up with 4
// consecutive output columns of one token (one vector store).
//   bf16: v_mfma_f32_16x16x32_bf16, a lane's 8 values are k = 8 lg + j.
//   fp32: 4 x v_mfma_f32_16x16x4_f32 per 16 k; k-step s of lane group lg
//         stands for k = 4 lg + s in both operands, which leaves the sum
//         unchanged and makes a lane's 4 values contiguous.
// A wave takes 16 MT tokens x 64 columns; a block 4 waves = 64 MT tokens.
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template <typename T>
struct Frag;
template <>
struct Frag<short> {
  static constexpr int KB = 32;  // k per step
  bf16x8 v;
  __device__ __forceinline__ void load(const short* p, bool ok) {
    if (ok) {
      v = *reinterpret_cast<const bf16x8*>(p);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = (__bf16)0.0f;
    }
  }
  static __device__ __forceinline__ f32x4 mma(const Frag& a, const Frag& b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, c, 0, 0, 0);
  }
};
template <>
struct Frag<float> {
  static constexpr int KB = 16;
  f32x4 v;
  __device__ __forceinline__ void load(const float* p, bool ok) {
    v = ok ? *reinterpret_cast<const f32x4*>(p) : f32x4{0.f, 0.f, 0.f, 0.f};
  }
  static __device__ __forceinline__ f32x4 mma(const Frag& a, const Frag& b, f32x4 c) {
#pragma unroll
    for (int s = 0; s < 4; ++s)
      c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[s], b.v[s], c, 0, 0, 0);
    return c;
  }
};

template <typename T, typename TO, int MT>
__global__ void __launch_bounds__(NT) head_matmul_rope_mfma_kernel(
    TO* __restrict__ out, const T* __restrict__ x, long x_stride,
    const T* __restrict__ w, int tokens, int heads, int K, int N, int tail,
    const long* __restrict__ positions, const float* __restrict__ inv_freq,
    int half) {
  constexpr int KB = Frag<T>::KB;
  constexpr int CH = KB / 4;  // elements per lane and step
  constexpr int NTILE = 4;    // 16-column tiles per wave
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, lg = lane >> 4;
  const int h = blockIdx.y;
  const int t0 = blockIdx.x * (64 * MT);
  const int n0 = blockIdx.z * (16 * NTILE);
  const int in_w = K + tail, out_w = N + tail;
  const T* wh = w + (long)h * N * K;
  // rows past the end are clamped for the loads and never stored
  const T* wrow[NTILE];
#pragma unroll
  for (int c = 0; c < NTILE; ++c)
    wrow[c] = wh + (long)min(n0 + 16 * c + li, N - 1) * K + lg * CH;
  const T* xrow[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int t = min(t0 + (wave * MT + m) * 16 + li, tokens - 1);
    xrow[m] = x + (long)t * x_stride + (long)h * in_w + lg * CH;
  }
  f32x4 acc[MT][NTILE];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int c = 0; c < NTILE; ++c) acc[m][c] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < K; k0 += KB) {
    const bool ok = k0 + lg * CH < K;  // K is a multiple of CH
    Frag<T> a[NTILE], b[MT];
#pragma unroll
    for (int c = 0; c < NTILE; ++c) a[c].load(wrow[c] + k0, ok);
#pragma unroll
    for (int m = 0; m < MT; ++m) b[m].load(xrow[m] + k0, ok);
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
      for (int c = 0; c < NTILE; ++c)
        acc[m][c] = Frag<T>::mma(a[c], b[m], acc[m][c]);
  }
  // acc[m][c][r] = out[token (wave MT + m) 16 + li][n0 + 16 c + 4 lg + r]
  const bool vec_out = (out_w % 4) == 0 && (N % 4) == 0;
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int t = t0 + (wave * MT + m) * 16 + li;
    if (t >= tokens) continue;
    TO* orow = out + ((long)t * heads + h) * out_w;
#pragma unroll
    for (int c = 0; c < NTILE; ++c) {
      const int n = n0 + 16 * c + 4 * lg;
      if (vec_out && n + 3 < N) {
        if (sizeof(TO) == 4) {
          *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(orow) + n) = acc[m][c];
        } else {
          short4_t o;
#pragma unroll
          for (int r = 0; r < 4; ++r) o[r] = float_to_bf16_bits(acc[m][c][r]);
          *reinterpret_cast<short4_t*>(reinterpret_cast<short*>(orow) + n) = o;
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < N) st_f32(orow, n + r, acc[m][c][r]);
      }
    }
  }
  if (tail == 0 || blockIdx.z != 0) return;
  rotate_tail(out, x, x_stride, t0, min(64 * MT, tokens - t0), h, heads, K, N,
              tail, positions, inv_freq, half);
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
  constexpr int CH = 16 / sizeof(T);
  const bool aligned = K % CH == 0 && (K + tail) % CH == 0 &&
                       x_stride % CH == 0 && ((uintptr_t)x % 16) == 0 &&
                       ((uintptr_t)w % 16) == 0 &&
                       ((uintptr_t)out % 16) == 0;
  if (aligned) {
    // large batches: 128 tokens per block (a weight fragment feeds two
    // token tiles); small ones: 64, for more blocks
    const bool big = tokens >= 2048;
    const int per_block = big ? 128 : 64;
    dim3 grid(cdiv(tokens, per_block), heads, cdiv(N, 64));
    auto fn = big ? head_matmul_rope_mfma_kernel<T, TO, 2>
                  : head_matmul_rope_mfma_kernel<T, TO, 1>;
    hipLaunchKernelGGL(fn, grid, dim3(NT), 0, stream, (TO*)out, (const T*)x,
                       x_stride, (const T*)w, tokens, heads, K, N, tail,
                       (const long*)positions, (const float*)inv_freq, half);
    return hipGetLastError();
  }
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
