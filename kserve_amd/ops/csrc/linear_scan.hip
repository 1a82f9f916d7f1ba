// Linear-attention recurrences with a matrix state per head, over a flat,
// variable-length token batch with per-sequence state slots (the layout of
// ssm_scan.hip: `positions[t]`, `cu_seqlens[s]`, `slots[s]`; a portion that
// starts at position 0 ignores what its slot held).
//
// The state of head h is S (K x V, fp32), stored per slot as [H, V, K] so
// that the contraction index is contiguous. Per token, with query q and key k
// of the head's q/k group and value v:
//
//   decay form (retention):   S <- d S + k v^T                 o = S^T q
//   delta form (gated delta): S <- g S;  u = b (v - S^T k);
//                             S <- S + k u^T                   o = S^T q
//
// d is a constant per head; g = exp(-exp(A_log) softplus(a + dt_bias)) and
// b = sigmoid(beta_raw) are computed here in fp32 from raw per-token, per-head
// projection columns. Both forms are evaluated from the OLD state with two
// independent contractions, p1 = S^T k and p2 = S^T q:
//   u = b (v - g p1)   (decay form: u = v)
//   o = g p2 + u (k . q)
//   S <- g S + k u^T
// so a token costs one pass over the registers that hold the state.
//
// Lane (ns, pl) of a 256-thread block owns rows n = ns + 16 r of columns
// pl + 16 c of one head's tile; a 16-lane DPP tree sums the contractions.
// Tokens go through LDS a chunk at a time with the next chunk's loads in
// flight. Grid = column tiles x heads x sequences: prefill portions and
// single-token decode batches run the same kernel.
//
// Helpers for what precedes the recurrence:
//  * rope_scale_heads: rotary positions on the first 2*half coordinates of
//    every head (coordinate i pairs with i + half), times a constant, fp32
//    out; two runs of heads with a constant each (queries, keys), columns
//    after them are only widened to fp32 (values).
//  * unit_norm_heads: x / sqrt(sum(x^2) + eps) * scale per head, in place on
//    fp32 rows; two runs of heads with a scale each (queries, keys).
#include "dtype_io.h"

#include <type_traits>

namespace {

constexpr int NT = 256;
constexpr int NW = NT / WAVE_SIZE;

__device__ __forceinline__ float row16_sum(float v) {
  auto swz = [](float x, auto ctrl) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x),
                                           decltype(ctrl)::value, 0xF, 0xF, true));
  };
  v += swz(v, std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
  v += swz(v, std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
  v += swz(v, std::integral_constant<int, 0x141>{});  // row_half_mirror
  v += swz(v, std::integral_constant<int, 0x140>{});  // row_mirror
  return v;
}

template <typename T>
__global__ void rope_scale_heads_kernel(
    float* __restrict__ out, const T* __restrict__ in, long in_stride,
    const long* __restrict__ positions, const float* __restrict__ inv_freq,
    int half, int heads_a, float scale_a, int heads_b, float scale_b, int dim,
    int width) {
  extern __shared__ float cs[];  // [half][2] = (cos, sin)
  const long t = blockIdx.x;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < half; i += NT) {
    float sn, co;
    sincosf(pos * inv_freq[i], &sn, &co);
    cs[2 * i] = co;
    cs[2 * i + 1] = sn;
  }
  __syncthreads();
  const int na = heads_a * dim, n = (heads_a + heads_b) * dim;
  const T* row = in + t * in_stride;
  for (int e = threadIdx.x; e < width; e += NT) {
    float r = ld_f32(row, e);
    if (e < n) {
      const int i = e % dim;
      if (i < 2 * half) {
        const bool lo = i < half;
        const int fi = lo ? i : i - half;
        const float y = ld_f32(row, lo ? e + half : e - half);
        const float co = cs[2 * fi], sn = cs[2 * fi + 1];
        r = lo ? r * co - y * sn : r * co + y * sn;
      }
      r *= e < na ? scale_a : scale_b;
    }
    out[t * width + e] = r;
  }
}

__global__ void unit_norm_heads_kernel(float* __restrict__ x, long stride,
                                       int heads_a, float scale_a, int heads_b,
                                       float scale_b, int dim, float eps) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  for (int job = wave; job < heads_a + heads_b; job += NW) {
    float* p = x + t * stride + (long)job * dim;
    float ss = 0.f;
    for (int i = lane; i < dim; i += WAVE_SIZE) ss += p[i] * p[i];
    ss = wave_reduce_sum(ss);
    const float m = (job < heads_a ? scale_a : scale_b) / sqrtf(ss + eps);
    for (int i = lane; i < dim; i += WAVE_SIZE) p[i] *= m;
  }
}

constexpr int SCAN_TC = 16;  // tokens per chunk

// R = state rows per lane (K <= 16 R), PC = columns per lane (a block covers
// 16 PC value columns of one head).
template <int R, int PC, bool DELTA>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4)))
linear_scan_kernel(
    float* __restrict__ o, const float* __restrict__ q, long q_stride,
    const float* __restrict__ k, long k_stride, const float* __restrict__ v,
    long v_stride, const float* __restrict__ decay,
    const float* __restrict__ a_f32, const short* __restrict__ a_bf16,
    const float* __restrict__ b_f32, const short* __restrict__ b_bf16,
    long ab_stride, const float* __restrict__ a_log,
    const float* __restrict__ dt_bias, float* __restrict__ state,
    const long* __restrict__ positions, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, int heads, int qk_heads, int V, int K) {
  extern __shared__ float lds[];
  constexpr int tc = SCAN_TC;
  constexpr int XS = 16 * PC;
  const int s = blockIdx.z;
  const int h = blockIdx.y;
  const int ns = threadIdx.x & 15;
  const int pl = threadIdx.x >> 4;
  const int p0 = blockIdx.x * XS;
  const int pt = min(XS, V - p0);  // columns of this tile
  const int first = cu_seqlens[s];
  const int len = cu_seqlens[s + 1] - first;
  if (len <= 0) return;
  const int hq = h / (heads / qk_heads);
  const int inner = heads * V;
  const long slot = slots[s];
  const bool fresh = positions[first] == 0;
  const float fixed = DELTA ? 1.f : decay[h];
  const float A = DELTA ? -expf(a_log[h]) : 0.f;
  const float bias = DELTA ? dt_bias[h] : 0.f;

  // LDS: k[tc][K] | q[tc][K] | v[tc][XS] | g[tc] | beta[tc] | k.q[tc] | o[tc][XS]
  float* Ks = lds;
  float* Qs = Ks + tc * K;
  float* Vs = Qs + tc * K;
  float* Gs = Vs + tc * XS;
  float* Bs = Gs + tc;
  float* Ds = Bs + tc;
  float* Os = Ds + tc;
  float S[R][PC];
  float* sp = state + ((slot * heads + h) * (long)V) * K;
#pragma unroll
  for (int c = 0; c < PC; ++c) {
    const int p = p0 + pl + 16 * c;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = ns + 16 * r;
      S[r][c] = (!fresh && p < V && n < K) ? sp[(long)p * K + n] : 0.f;
    }
  }

  // staging: 16 threads per token of the chunk, each takes every 16th
  // element of the token's k, q and v rows
  const int stk = threadIdx.x >> 4;
  const int sl = threadIdx.x & 15;
  float sK[R], sQ[R], sV[PC], sa = 0.f, sb = 0.f;
  auto prefetch = [&](int t0, int cnt) {
    const bool on = stk < cnt;
    const long t = first + t0 + (on ? stk : 0);
    const float* krow = k + t * k_stride + (long)hq * K;
    const float* qrow = q + t * q_stride + (long)hq * K;
    const float* vrow = v + t * v_stride + (long)h * V + p0;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = sl + 16 * r;
      const bool ok = on && n < K;
      sK[r] = ok ? krow[n] : 0.f;
      sQ[r] = ok ? qrow[n] : 0.f;
    }
#pragma unroll
    for (int c = 0; c < PC; ++c) {
      const int col = sl + 16 * c;
      sV[c] = (on && col < pt) ? vrow[col] : 0.f;
    }
    if (DELTA && on && sl == 0) {
      const long i = t * ab_stride + h;
      sa = (a_f32 ? a_f32[i] : bf16_bits_to_float(a_bf16[i])) + bias;
      sb = b_f32 ? b_f32[i] : bf16_bits_to_float(b_bf16[i]);
    }
  };
  auto commit = [&](int cnt) {
    float kq = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) kq += sK[r] * sQ[r];
    kq = row16_sum(kq);  // every lane takes part, staged or not
    if (stk < cnt) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = sl + 16 * r;
        if (n < K) {
          Ks[stk * K + n] = sK[r];
          Qs[stk * K + n] = sQ[r];
        }
      }
#pragma unroll
      for (int c = 0; c < PC; ++c) Vs[stk * XS + sl + 16 * c] = sV[c];
      if (sl == 0) {
        Ds[stk] = kq;
        if (DELTA) {
          // softplus without a clamp; log1p(exp(x)) is x itself past x ~ 30
          const float sp_ = sa > 30.f ? sa : log1pf(expf(sa));
          Gs[stk] = expf(A * sp_);
          Bs[stk] = 1.0f / (1.0f + expf(-sb));
        } else {
          Gs[stk] = fixed;
          Bs[stk] = 1.f;
        }
      }
    }
  };

  prefetch(0, min(tc, len));
  for (int t0 = 0; t0 < len; t0 += tc) {
    const int cnt = min(tc, len - t0);
    __syncthreads();  // previous chunk's LDS fully consumed
    commit(cnt);
    __syncthreads();
    if (t0 + tc < len) prefetch(t0 + tc, min(tc, len - t0 - tc));
    for (int tk = 0; tk < cnt; ++tk) {
      const float g = Gs[tk], bt = Bs[tk], kq = Ds[tk];
      float kk[R], qq[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = ns + 16 * r;
        const bool ok = n < K;
        kk[r] = ok ? Ks[tk * K + n] : 0.f;
        qq[r] = ok ? Qs[tk * K + n] : 0.f;
      }
#pragma unroll
      for (int c = 0; c < PC; ++c) {
        const int col = pl + 16 * c;
        const float vv = col < pt ? Vs[tk * XS + col] : 0.f;
        float p1 = 0.f, p2 = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          if (DELTA) p1 += S[r][c] * kk[r];
          p2 += S[r][c] * qq[r];
        }
        p2 = row16_sum(p2);
        float u = vv;
        if (DELTA) {
          p1 = row16_sum(p1);
          u = bt * (vv - g * p1);
        }
#pragma unroll
        for (int r = 0; r < R; ++r) S[r][c] = g * S[r][c] + kk[r] * u;
        if (ns == 0) Os[tk * XS + col] = g * p2 + u * kq;
      }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < cnt * pt; e += 256) {
      const int tk = e / pt, col = e % pt;
      o[(long)(first + t0 + tk) * inner + h * V + p0 + col] = Os[tk * XS + col];
    }
  }
#pragma unroll
  for (int c = 0; c < PC; ++c) {
    const int p = p0 + pl + 16 * c;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = ns + 16 * r;
      if (p < V && n < K) sp[(long)p * K + n] = S[r][c];
    }
  }
}

}  // namespace

extern "C" hipError_t ks_rope_scale_heads(void* out, const void* in,
                                          long in_stride, const void* positions,
                                          const void* inv_freq, int half,
                                          int tokens, int heads_a,
                                          float scale_a, int heads_b,
                                          float scale_b, int dim, int width,
                                          int is_f32, hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (!inv_freq) half = 0;
  if (2 * half > dim || (long)(heads_a + heads_b) * dim > width)
    return hipErrorInvalidValue;
  const size_t smem = sizeof(float) * 2 * (size_t)half;
  if (is_f32)
    hipLaunchKernelGGL(rope_scale_heads_kernel<float>, dim3(tokens), dim3(NT),
                       smem, stream, (float*)out, (const float*)in, in_stride,
                       (const long*)positions, (const float*)inv_freq, half,
                       heads_a, scale_a, heads_b, scale_b, dim, width);
  else
    hipLaunchKernelGGL(rope_scale_heads_kernel<short>, dim3(tokens), dim3(NT),
                       smem, stream, (float*)out, (const short*)in, in_stride,
                       (const long*)positions, (const float*)inv_freq, half,
                       heads_a, scale_a, heads_b, scale_b, dim, width);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_unit_norm_heads(void* x, long stride, int tokens,
                                         int heads_a, float scale_a,
                                         int heads_b, float scale_b, int dim,
                                         float eps, hipStream_t stream) {
  if (tokens == 0 || heads_a + heads_b == 0) return hipSuccess;
  hipLaunchKernelGGL(unit_norm_heads_kernel, dim3(tokens), dim3(NT), 0, stream,
                     (float*)x, stride, heads_a, scale_a, heads_b, scale_b, dim,
                     eps);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

#define LSCAN_LAUNCH(RR, PCC, DD)                                             \
  hipLaunchKernelGGL((linear_scan_kernel<RR, PCC, DD>), grid, dim3(256), smem, \
                     stream, (float*)o, (const float*)q, q_stride,            \
                     (const float*)k, k_stride, (const float*)v, v_stride,    \
                     (const float*)decay,                                     \
                     ab_is_f32 ? (const float*)a_raw : nullptr,               \
                     ab_is_f32 ? nullptr : (const short*)a_raw,               \
                     ab_is_f32 ? (const float*)b_raw : nullptr,               \
                     ab_is_f32 ? nullptr : (const short*)b_raw, ab_stride,    \
                     (const float*)a_log, (const float*)dt_bias,              \
                     (float*)state, (const long*)positions,                   \
                     (const int*)cu_seqlens, (const int*)slots, heads,        \
                     qk_heads, V, K)

#define LSCAN_LAUNCH_PC(RR, DD)                                               \
  do {                                                                        \
    if (pc == 1) LSCAN_LAUNCH(RR, 1, DD);                                     \
    else if (pc == 2) LSCAN_LAUNCH(RR, 2, DD);                                \
    else LSCAN_LAUNCH(RR, 4, DD);                                             \
  } while (0)

#define LSCAN_LAUNCH_R(DD)                                                    \
  do {                                                                        \
    if (R <= 1) LSCAN_LAUNCH_PC(1, DD);                                       \
    else if (R <= 2) LSCAN_LAUNCH_PC(2, DD);                                  \
    else if (R <= 4) LSCAN_LAUNCH_PC(4, DD);                                  \
    else if (R <= 8) LSCAN_LAUNCH_PC(8, DD);                                  \
    else if (pc == 1) LSCAN_LAUNCH(16, 1, DD);                                \
    else LSCAN_LAUNCH(16, 2, DD);                                             \
  } while (0)

// decay != null: decay form; otherwise the delta form, which reads a_raw /
// b_raw [T, heads] (two column ranges of rows with one stride), a_log and
// dt_bias.
extern "C" hipError_t ks_linear_scan(
    void* o, const void* q, long q_stride, const void* k, long k_stride,
    const void* v, long v_stride, const void* decay, const void* a_raw,
    const void* b_raw, long ab_stride, int ab_is_f32, const void* a_log,
    const void* dt_bias, void* state, const void* positions,
    const void* cu_seqlens, const void* slots, int num_seqs, int heads,
    int qk_heads, int V, int K, hipStream_t stream) {
  if (num_seqs == 0) return hipSuccess;
  if (qk_heads <= 0 || heads % qk_heads != 0 || K < 1 || K > 256 || V < 1)
    return hipErrorInvalidValue;
  if (!decay && (!a_raw || !b_raw || !a_log || !dt_bias))
    return hipErrorInvalidValue;
  const int R = cdiv(K, 16);
  int pc = V > 32 ? 4 : (V > 16 ? 2 : 1);
  if (R > 8 && pc > 2) pc = 2;
  // a block walks its tokens one after the other, so a launch with few
  // (sequence, head) pairs takes narrower tiles to put more blocks on the chip
  while (pc > 1 && (long)cdiv(V, 16 * pc) * heads * num_seqs < 1024) pc >>= 1;
  const int xs = 16 * pc;
  const size_t smem = sizeof(float) * ((size_t)SCAN_TC * (2 * K + 2 * xs + 3));
  dim3 grid(cdiv(V, xs), heads, num_seqs);
  if (decay) LSCAN_LAUNCH_R(false);
  else LSCAN_LAUNCH_R(true);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}
