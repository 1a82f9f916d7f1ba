// State-space (Mamba-2 / SSD form) sequence mixer kernels over a flat,
// variable-length token batch with per-sequence state slots.
//
// A sequence's portion may start anywhere: `positions[t]` is the absolute
// position of token t, `seq_of_token[t]` its sequence in the batch,
// `cu_seqlens[s]` the first flat token of sequence s and `slots[s]` the row
// of the state pools that carries it between steps. A portion that starts at
// position 0 ignores whatever its slot held (slots are reused, never cleared).
//
//  * causal_conv_silu: depthwise causal convolution over `taps` inputs per
//    channel + bias (optional) + silu. Inputs before the portion come from the conv
//    state (the last taps-1 raw inputs of the sequence), zeros before
//    position 0.
//  * conv_state_update: runs after the above, shifts the new raw inputs in.
//  * ssd_scan: per head h with group g(h):
//        a_t = exp(-exp(A_log_h) * dt_t),  dt_t = softplus(dt_raw + dt_bias_h)
//        S_t = a_t S_{t-1} + dt_t B_t x_t^T        (S: N x P, fp32)
//        y_t = S_t^T C_t + D_h x_t
//    The state lives in registers: lane (ns, pl) owns rows n = ns + 16 r of
//    a few columns of one head, a 16-lane shuffle tree sums the C-contraction.
//    Tokens of a sequence are walked in order, a chunk at a time through LDS.
//    Serves prefill portions and single-token decode alike (grid = column
//    tiles x heads x sequences, so decode batches fill the chip).
#include "dtype_io.h"

#include <type_traits>

namespace {

constexpr int MAX_TAPS = 16;

// sum over each row of 16 lanes with DPP lane swaps (VALU rate, no LDS
// traffic): swap within pairs, within quads, mirror the 8-lane half, mirror
// the row; every lane of the row ends with the row's sum
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

__device__ __forceinline__ float silu_f(float v) {
  return v / (1.0f + expf(-v));
}

template <typename T>
__global__ void causal_conv_silu_kernel(
    float* __restrict__ out, const T* __restrict__ in, long in_stride,
    const float* __restrict__ w, const float* __restrict__ bias,
    const T* __restrict__ conv_state, const long* __restrict__ positions,
    const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, int channels, int taps) {
  const int t = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int s = seq_of_token[t];
  const int first = cu_seqlens[s];
  const long pos = positions[t];
  const long slot = slots[s];
  const int hist = taps - 1;
  float acc = bias ? bias[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int back = hist - j;  // 0 = the current token
    if (pos - back < 0) continue;
    float v;
    if (t - back >= first) {
      v = ld_f32(in, (long)(t - back) * in_stride + c);
    } else {
      // state row i holds the input at position (portion start - hist + i)
      const int i = hist - back + (t - first);
      v = ld_f32(conv_state, (slot * hist + i) * channels + c);
    }
    acc += w[(long)c * taps + j] * v;
  }
  out[(long)t * channels + c] = silu_f(acc);
}

// 4 consecutive channels per lane (8- or 16-byte loads, 16-byte stores); the
// launcher picks it when pointers, strides and the channel count allow
template <typename T>
__device__ __forceinline__ void load4(const T* p, float* v);
template <>
__device__ __forceinline__ void load4<short>(const short* p, float* v) {
  const short4_t x = *reinterpret_cast<const short4_t*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = bf16_bits_to_float(x[i]);
}
template <>
__device__ __forceinline__ void load4<float>(const float* p, float* v) {
  const float4_t x = *reinterpret_cast<const float4_t*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = x[i];
}

constexpr int CONV_TT = 8;  // tokens per block of the vector kernel

template <typename T, int TAPS>
__global__ void causal_conv_silu_vec4_kernel(
    float* __restrict__ out, const T* __restrict__ in, long in_stride,
    const float* __restrict__ w, const float* __restrict__ bias,
    const T* __restrict__ conv_state, const long* __restrict__ positions,
    const int* __restrict__ seq_of_token, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, int tokens, int channels) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (c >= channels) return;
  constexpr int hist = TAPS - 1;
  // taps and bias of this lane's 4 channels, reused for every token
  float wt[4][TAPS], b4[4];
  if (bias) load4<float>(bias + c, b4);
  else b4[0] = b4[1] = b4[2] = b4[3] = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < TAPS; ++j) wt[i][j] = w[(long)(c + i) * TAPS + j];
  const int t_end = min(tokens, (int)(blockIdx.y + 1) * CONV_TT);
  for (int t = blockIdx.y * CONV_TT; t < t_end; ++t) {
    const int s = seq_of_token[t];
    const int first = cu_seqlens[s];
    const long pos = positions[t];
    const long slot = slots[s];
    float acc[4] = {b4[0], b4[1], b4[2], b4[3]};
#pragma unroll
    for (int j = 0; j < TAPS; ++j) {
      const int back = hist - j;
      if (pos - back < 0) continue;
      float v[4];
      if (t - back >= first)
        load4<T>(in + (long)(t - back) * in_stride + c, v);
      else
        load4<T>(conv_state + (slot * hist + (hist - back + (t - first))) * channels + c, v);
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] += wt[i][j] * v[i];
    }
    float4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = silu_f(acc[i]);
    *reinterpret_cast<float4_t*>(out + (long)t * channels + c) = o;
  }
}

template <typename T>
__global__ void conv_state_update_kernel(
    T* __restrict__ conv_state, const T* __restrict__ in, long in_stride,
    const long* __restrict__ positions, const int* __restrict__ cu_seqlens,
    const int* __restrict__ slots, int channels, int taps) {
  const int s = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int first = cu_seqlens[s];
  const int len = cu_seqlens[s + 1] - first;
  if (len <= 0) return;
  const long start = positions[first];
  const long slot = slots[s];
  const int hist = taps - 1;
  T keep[MAX_TAPS];
  // new row i holds position (start + len - hist + i)
  for (int i = 0; i < hist; ++i) {
    const long rel = (long)len - hist + i;  // offset into the portion
    T v;
    if (rel >= 0) {
      v = in[(first + rel) * in_stride + c];
    } else if (start + rel < 0) {
      st_f32(&v, 0, 0.f);
    } else {
      v = conv_state[(slot * hist + (hist + rel)) * channels + c];
    }
    keep[i] = v;
  }
  for (int i = 0; i < hist; ++i)
    conv_state[(slot * hist + i) * channels + c] = keep[i];
}

// R = state rows per lane (N <= 16 R), PC = columns per lane (tile of 16 PC
// columns of one head per block). blockDim = 256 = 16 row-lanes x 16 col-lanes.
// Tokens are taken in chunks of `tc`: the chunk's B, C, x rows and step sizes
// are staged in LDS with coalesced loads (the next chunk's loads are in
// flight while this one is computed), softplus/exp run once per (token, head)
// instead of once per lane, and y leaves through LDS as whole rows.
constexpr int SCAN_TC = 16;  // tokens per chunk

template <int R, int PC>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4)))
ssd_scan_kernel(
    float* __restrict__ y, const float* __restrict__ xbc,
    const float* __restrict__ dt_raw_f32, const short* __restrict__ dt_raw_bf16,
    long dt_stride, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ d_skip,
    float* __restrict__ state, const long* __restrict__ positions,
    const int* __restrict__ cu_seqlens, const int* __restrict__ slots,
    int heads, int groups, int P, int N) {
  extern __shared__ float lds[];
  constexpr int tc = SCAN_TC;
  const int s = blockIdx.z;
  const int h = blockIdx.y;
  const int ns = threadIdx.x & 15;
  const int pl = threadIdx.x >> 4;
  const int p0 = blockIdx.x * (16 * PC);
  const int pt = min(16 * PC, P - p0);  // columns of this tile
  const int first = cu_seqlens[s];
  const int len = cu_seqlens[s + 1] - first;
  if (len <= 0) return;
  const int g = h / (heads / groups);
  const int inner = heads * P;
  const int channels = inner + 2 * groups * N;
  const long slot = slots[s];
  const bool fresh = positions[first] == 0;
  const float A = -expf(a_log[h]);
  const float bias = dt_bias[h];
  const float Dh = d_skip[h];

  // LDS: B[tc][N] | C[tc][N] | x[tc][16 PC] | dt[tc] | decay[tc] | y[tc][16 PC]
  const int XS = 16 * PC;
  float* Bs = lds;
  float* Cs = Bs + tc * N;
  float* Xs = Cs + tc * N;
  float* Ds = Xs + tc * XS;
  float* As = Ds + tc;
  float* Ys = As + tc;
  float S[R][PC];
  float* sp = state + ((slot * heads + h) * (long)P) * N;
#pragma unroll
  for (int c = 0; c < PC; ++c) {
    const int p = p0 + pl + 16 * c;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = ns + 16 * r;
      S[r][c] = (!fresh && p < P && n < N) ? sp[(long)p * N + n] : 0.f;
    }
  }

  // staging: 16 threads per token of the chunk, each takes every 16th
  // element of the token's B, C and x rows (no index arithmetic beyond adds)
  const int stk = threadIdx.x >> 4;   // token of the chunk this thread stages
  const int sl = threadIdx.x & 15;
  float sB[R], sC[R], sX[PC], sdt = 0.f;
  auto prefetch = [&](int t0, int cnt) {
    if (stk < cnt) {
      const long t = first + t0 + stk;
      const float* row = xbc + t * channels;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = sl + 16 * r;
        sB[r] = n < N ? row[inner + g * N + n] : 0.f;
        sC[r] = n < N ? row[inner + groups * N + g * N + n] : 0.f;
      }
#pragma unroll
      for (int c = 0; c < PC; ++c) {
        const int col = sl + 16 * c;
        sX[c] = col < pt ? row[h * P + p0 + col] : 0.f;
      }
      if (sl == 0) {
        const long i = t * dt_stride + h;
        sdt = (dt_raw_f32 ? dt_raw_f32[i] : bf16_bits_to_float(dt_raw_bf16[i])) + bias;
      }
    }
  };
  auto commit = [&](int cnt) {
    if (stk < cnt) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = sl + 16 * r;
        if (n < N) {
          Bs[stk * N + n] = sB[r];
          Cs[stk * N + n] = sC[r];
        }
      }
#pragma unroll
      for (int c = 0; c < PC; ++c) Xs[stk * XS + sl + 16 * c] = sX[c];
      if (sl == 0) {
        // softplus without a clamp; log1p(exp(v)) is v itself past v ~ 30
        const float dt = sdt > 30.f ? sdt : log1pf(expf(sdt));
        Ds[stk] = dt;
        As[stk] = expf(A * dt);
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
      const float a = As[tk], dt = Ds[tk];
      float B[R], C[R];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int n = ns + 16 * r;
        const bool ok = n < N;
        B[r] = ok ? Bs[tk * N + n] : 0.f;
        C[r] = ok ? Cs[tk * N + n] : 0.f;
      }
#pragma unroll
      for (int c = 0; c < PC; ++c) {
        const int col = pl + 16 * c;
        const float x = col < pt ? Xs[tk * XS + col] : 0.f;
        const float dtx = dt * x;
        float acc = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
          S[r][c] = a * S[r][c] + B[r] * dtx;
          acc += S[r][c] * C[r];
        }
        acc = row16_sum(acc);
        if (ns == 0) Ys[tk * XS + col] = acc + Dh * x;
      }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < cnt * pt; e += 256) {
      const int tk = e / pt, col = e % pt;
      y[(long)(first + t0 + tk) * inner + h * P + p0 + col] = Ys[tk * XS + col];
    }
  }
#pragma unroll
  for (int c = 0; c < PC; ++c) {
    const int p = p0 + pl + 16 * c;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int n = ns + 16 * r;
      if (p < P && n < N) sp[(long)p * N + n] = S[r][c];
    }
  }
}

}  // namespace

extern "C" hipError_t ks_causal_conv_silu(
    void* out, const void* in, long in_stride, const void* w, const void* bias,
    void* conv_state, const void* positions, const void* seq_of_token,
    const void* cu_seqlens, const void* slots, int tokens, int num_seqs,
    int channels, int taps, int is_f32, hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (taps < 1 || taps > MAX_TAPS) return hipErrorInvalidValue;
  dim3 grid(cdiv(channels, 256), tokens);
  dim3 grid_u(cdiv(channels, 256), num_seqs);
  const int esz = is_f32 ? 4 : 2;
  // 4-channel vectors need every row start on a 4-element boundary
  const bool vec = channels % 4 == 0 && in_stride % 4 == 0 &&
                   ((uintptr_t)in % (4 * esz)) == 0 &&
                   ((uintptr_t)conv_state % (4 * esz)) == 0 &&
                   ((uintptr_t)out % 16) == 0 && ((uintptr_t)bias % 16) == 0 &&
                   taps >= 2 && taps <= 4;
  dim3 grid_v(cdiv(channels / 4, 256), cdiv(tokens, CONV_TT));
#define CONV_ARGS(TT)                                                         \
  (float*)out, (const TT*)in, in_stride, (const float*)w, (const float*)bias, \
      (const TT*)conv_state, (const long*)positions,                          \
      (const int*)seq_of_token, (const int*)cu_seqlens, (const int*)slots
#define CONV_VEC_K(TT, K)                                                     \
  hipLaunchKernelGGL((causal_conv_silu_vec4_kernel<TT, K>), grid_v,           \
                     dim3(256), 0, stream, CONV_ARGS(TT), tokens, channels)
#define CONV_VEC(TT)                                                          \
  do {                                                                        \
    if (taps == 2) CONV_VEC_K(TT, 2);                                         \
    else if (taps == 3) CONV_VEC_K(TT, 3);                                    \
    else CONV_VEC_K(TT, 4);                                                   \
  } while (0)
  if (is_f32) {
    if (vec) CONV_VEC(float);
    else
      hipLaunchKernelGGL(causal_conv_silu_kernel<float>, grid, dim3(256), 0,
                         stream, CONV_ARGS(float), channels, taps);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<float>, grid_u, dim3(256), 0,
                         stream, (float*)conv_state, (const float*)in,
                         in_stride, (const long*)positions,
                         (const int*)cu_seqlens, (const int*)slots, channels,
                         taps);
  } else {
    if (vec) CONV_VEC(short);
    else
      hipLaunchKernelGGL(causal_conv_silu_kernel<short>, grid, dim3(256), 0,
                         stream, CONV_ARGS(short), channels, taps);
    if (taps > 1)
      hipLaunchKernelGGL(conv_state_update_kernel<short>, grid_u, dim3(256), 0,
                         stream, (short*)conv_state, (const short*)in,
                         in_stride, (const long*)positions,
                         (const int*)cu_seqlens, (const int*)slots, channels,
                         taps);
  }
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

#define SSD_LAUNCH(RR, PCC)                                                   \
  hipLaunchKernelGGL((ssd_scan_kernel<RR, PCC>), grid, dim3(256), smem,       \
                     stream, (float*)y, (const float*)xbc,                    \
                     dt_is_f32 ? (const float*)dt_raw : nullptr,              \
                     dt_is_f32 ? nullptr : (const short*)dt_raw, dt_stride,   \
                     (const float*)dt_bias, (const float*)a_log,              \
                     (const float*)d_skip, (float*)state,                     \
                     (const long*)positions, (const int*)cu_seqlens,          \
                     (const int*)slots, heads, groups, P, N)

#define SSD_LAUNCH_R(RR)                                                      \
  do {                                                                        \
    if (pc == 1) SSD_LAUNCH(RR, 1);                                           \
    else if (pc == 2) SSD_LAUNCH(RR, 2);                                      \
    else SSD_LAUNCH(RR, 4);                                                   \
  } while (0)

extern "C" hipError_t ks_ssd_scan(void* y, const void* xbc, const void* dt_raw,
                                  long dt_stride, int dt_is_f32,
                                  const void* dt_bias, const void* a_log,
                                  const void* d_skip, void* state,
                                  const void* positions,
                                  const void* cu_seqlens, const void* slots,
                                  int num_seqs, int heads, int groups, int P,
                                  int N, hipStream_t stream) {
  if (num_seqs == 0) return hipSuccess;
  if (groups <= 0 || heads % groups != 0 || N < 1 || N > 256)
    return hipErrorInvalidValue;
  // columns per lane: a block covers up to 64 columns of one head; wide
  // state rows (R = 16) keep two columns so the state stays in registers
  const int R = cdiv(N, 16);
  int pc = P > 32 ? 4 : (P > 16 ? 2 : 1);
  if (R > 8 && pc > 2) pc = 2;
  const int xs = 16 * pc;
  const size_t smem = sizeof(float) * ((size_t)SCAN_TC * (2 * N + 2 * xs + 2));
  dim3 grid(cdiv(P, xs), heads, num_seqs);
  if (R <= 1) SSD_LAUNCH_R(1);
  else if (R <= 2) SSD_LAUNCH_R(2);
  else if (R <= 3) SSD_LAUNCH_R(3);
  else if (R <= 4) SSD_LAUNCH_R(4);
  else if (R <= 6) SSD_LAUNCH_R(6);
  else if (R <= 8) SSD_LAUNCH_R(8);
  else SSD_LAUNCH_R(16);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}
