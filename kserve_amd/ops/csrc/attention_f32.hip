// Softmax attention against the paged KV cache with scores and weights kept
// in fp32 end to end, for any (query/key dim, value dim, group size).
//
//  * qk_norm_temp_cache: per token, RMS-normalise the WHOLE query projection
//    (all heads at once) and the whole key projection with plain weights,
//    scale the query by a position-dependent temperature
//        1 + coef * ln(floor((pos + 1) / every) + 1),
//    write q (fp32) out and scatter k / v into the paged cache.
//  * qk_headnorm_rope_cache: per token and per HEAD, RMS-normalise q and k
//    with a weight of the head size shared by the heads, rotate the first
//    2*half coordinates (coordinate i pairs with i + half, angle
//    pos * inv_freq[i] in fp32), optionally divide each value head by its
//    RMS and rotate it by the token's position over its whole width, write
//    q (fp32) out and scatter k / v into the paged cache.
//  * ctx_attention_f32: causal attention of a flat variable-length query
//    batch against each sequence's pages (the portion's own keys are already
//    in the cache). Both products run on the fp32 matrix cores
//    (v_mfma_f32_16x16x4_f32), so q.k, the softmax weights and weights x V
//    are all true fp32 whatever the cache dtype; K/V tiles of 64 keys are
//    converted to fp32 while they are staged in LDS.
//    The kernel works on transposed tiles: S^T = K Q^T puts one query per
//    lane column, so the running max / sum / rescale are per-lane scalars,
//    and the S^T accumulator registers are already the B operand of
//    O^T += V^T P^T (the contraction runs over keys in the accumulator's own
//    order; V is read from LDS in that order), so the weights never leave
//    registers. The head-dimension contraction and the value columns are
//    likewise assigned to lanes so that every LDS operand read is 16 bytes.
//    Optional parts: a chunk-local mask (a query sees only keys of its own
//    block of `chunk` positions, so the key loop starts at the chunk of the
//    block's first query), a per-head sink (one more term exp(sink) in the
//    softmax denominator, with no key and no value), and turning every
//    head output back by its query's position (pairs m, m + DV/2; the
//    normalised rows pass through LDS so a pair meets in one lane).
//    Prefill: a block takes 64 consecutive tokens of one query head, 16 per
//    wave, all waves sharing the staged K/V tile. Decode (one token per
//    sequence): a block takes the query heads of one KV group as its 16
//    columns and the four waves split every tile's keys, merging their
//    partial (max, sum, O) through LDS at the end, so the group's K/V is read
//    once. Head sizes are padded up to 64/128/256 with zeros. An optional
//    per-(token, head) gate multiplies the result by sigmoid(gate).
#include <type_traits>

#include "dtype_io.h"

namespace {

constexpr int NT = 256;
constexpr int NW = NT / WAVE_SIZE;
constexpr int BK = 64;  // keys per staged tile

typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename T>
__global__ void qk_norm_temp_cache_kernel(
    float* __restrict__ q_out, const T* __restrict__ q, const T* __restrict__ k,
    const T* __restrict__ v, long row_stride, const float* __restrict__ qw,
    const float* __restrict__ kw, const long* __restrict__ positions,
    const int* __restrict__ slot_mapping, T* __restrict__ k_cache,
    T* __restrict__ v_cache, float eps, float temp_coef, int temp_every,
    int q_width, int kv_heads, int D, int DV, int block_size) {
  __shared__ float scratch[NW];
  const long t = blockIdx.x;
  const T* qr = q + t * row_stride;
  const T* kr = k + t * row_stride;
  const T* vr = v + t * row_stride;
  const int k_width = kv_heads * D;
  float ss = 0.f;
  for (int i = threadIdx.x; i < q_width; i += NT) {
    const float x = ld_f32(qr, i);
    ss += x * x;
  }
  ss = block_sum_sync<NW>(ss, scratch);
  float qinv = 1.0f / sqrtf(ss / (float)q_width + eps);
  const long pos = positions[t];
  if (temp_every > 0)
    qinv *= 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
  for (int i = threadIdx.x; i < q_width; i += NT)
    q_out[t * q_width + i] = ld_f32(qr, i) * qw[i] * qinv;

  ss = 0.f;
  for (int i = threadIdx.x; i < k_width; i += NT) {
    const float x = ld_f32(kr, i);
    ss += x * x;
  }
  ss = block_sum_sync<NW>(ss, scratch);
  const float kinv = 1.0f / sqrtf(ss / (float)k_width + eps);
  const long slot = slot_mapping[t];
  if (slot < 0) return;
  const long blk = slot / block_size, off = slot % block_size;
  for (int i = threadIdx.x; i < k_width; i += NT) {
    const int g = i / D, d = i % D;
    st_f32(k_cache, ((blk * kv_heads + g) * block_size + off) * D + d,
           ld_f32(kr, i) * kw[i] * kinv);
  }
  for (int i = threadIdx.x; i < kv_heads * DV; i += NT) {
    const int g = i / DV, d = i % DV;
    v_cache[((blk * kv_heads + g) * block_size + off) * DV + d] = vr[i];
  }
}

// A block per token. The angles depend on the token's position only, so
// their sines and cosines are computed once per block into LDS ([qk_half]
// then [v_half] pairs) and shared by every head. Then one wave per head
// job: jobs 0..heads-1 are q heads, then kv_heads k heads, then kv_heads v
// heads. x_n[j] = x[j] * inv_rms * w[j]; coordinate i < half pairs with
// i + half. VEC = 2: a lane owns two neighbouring coordinates (4- and 8-byte
// accesses); needs even head sizes, halves and row stride.
template <int VEC>
__device__ __forceinline__ void ld_vec(const short* p, float* v) {
  if (VEC == 2) {
    const unsigned u = *reinterpret_cast<const unsigned*>(p);
    v[0] = bf16_bits_to_float((short)(u & 0xffffu));
    v[1] = bf16_bits_to_float((short)(u >> 16));
  } else {
    v[0] = bf16_bits_to_float(p[0]);
  }
}
template <int VEC>
__device__ __forceinline__ void ld_vec(const float* p, float* v) {
  if (VEC == 2) {
    const float2_t u = *reinterpret_cast<const float2_t*>(p);
    v[0] = u[0];
    v[1] = u[1];
  } else {
    v[0] = p[0];
  }
}
template <int VEC>
__device__ __forceinline__ void st_vec(short* p, const float* v) {
  if (VEC == 2) {
    const unsigned lo = (unsigned short)float_to_bf16_bits(v[0]);
    const unsigned hi = (unsigned short)float_to_bf16_bits(v[1]);
    *reinterpret_cast<unsigned*>(p) = lo | (hi << 16);
  } else {
    p[0] = float_to_bf16_bits(v[0]);
  }
}
template <int VEC>
__device__ __forceinline__ void st_vec(float* p, const float* v) {
  if (VEC == 2)
    *reinterpret_cast<float2_t*>(p) = float2_t{v[0], v[1]};
  else
    p[0] = v[0];
}

template <typename T, int VEC>
__global__ void qk_headnorm_rope_cache_kernel(
    float* __restrict__ q_out, const T* __restrict__ q, const T* __restrict__ k,
    const T* __restrict__ v, long row_stride, const float* __restrict__ qw,
    const float* __restrict__ kw, const long* __restrict__ positions,
    const int* __restrict__ slot_mapping, T* __restrict__ k_cache,
    T* __restrict__ v_cache, float eps, int heads, int kv_heads, int D, int DV,
    int block_size, const float* __restrict__ qk_inv_freq, int qk_half,
    int v_unit_norm, const float* __restrict__ v_inv_freq, int v_half) {
  extern __shared__ float lds[];
  if (!qk_inv_freq) qk_half = 0;
  if (!v_inv_freq) v_half = 0;
  float* cs_qk = lds;               // [qk_half][2] = (cos, sin)
  float* cs_v = lds + 2 * qk_half;  // [v_half][2]
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < qk_half + v_half; i += NT) {
    const float f = i < qk_half ? qk_inv_freq[i] : v_inv_freq[i - qk_half];
    float sn, cs;
    sincosf(pos * f, &sn, &cs);
    lds[2 * i] = cs;
    lds[2 * i + 1] = sn;
  }
  __syncthreads();
  const long slot = slot_mapping[t];
  const long blk = slot >= 0 ? slot / block_size : 0;
  const long off = slot >= 0 ? slot % block_size : 0;
  const int jobs = heads + 2 * kv_heads;
  for (int job = wave; job < jobs; job += NW) {
    const T* src;
    const float* w = nullptr;
    const float* cs;
    int width, half;
    bool norm = true;
    float* dst_f = nullptr;
    T* dst_c = nullptr;
    if (job < heads) {
      src = q + t * row_stride + (long)job * D;
      w = qw;
      width = D;
      cs = cs_qk;
      half = qk_half;
      dst_f = q_out + (t * heads + job) * D;
    } else if (job < heads + kv_heads) {
      const int g = job - heads;
      src = k + t * row_stride + (long)g * D;
      w = kw;
      width = D;
      cs = cs_qk;
      half = qk_half;
      if (slot < 0) continue;
      dst_c = k_cache + ((blk * kv_heads + g) * block_size + off) * D;
    } else {
      const int g = job - heads - kv_heads;
      src = v + t * row_stride + (long)g * DV;
      width = DV;
      cs = cs_v;
      half = v_half;
      norm = v_unit_norm != 0;
      if (slot < 0) continue;
      dst_c = v_cache + ((blk * kv_heads + g) * block_size + off) * DV;
    }
    float inv = 1.0f;
    if (norm) {
      float ss = 0.f;
      for (int i = lane * VEC; i < width; i += WAVE_SIZE * VEC) {
        float x[VEC];
        ld_vec<VEC>(src + i, x);
#pragma unroll
        for (int c = 0; c < VEC; ++c) ss += x[c] * x[c];
      }
      ss = wave_reduce_sum(ss);
      inv = 1.0f / sqrtf(ss / (float)width + eps);
    }
    for (int i = lane * VEC; i < width; i += WAVE_SIZE * VEC) {
      float x[VEC], r[VEC];
      ld_vec<VEC>(src + i, x);
#pragma unroll
      for (int c = 0; c < VEC; ++c) {
        if (norm) x[c] = w ? x[c] * inv * w[i + c] : x[c] * inv;
        r[c] = x[c];
      }
      if (i < 2 * half) {  // i and i + VEC - 1 lie in the same half
        const int pi = i < half ? i + half : i - half;  // partner
        const int fi = i < half ? i : i - half;
        float y[VEC];
        ld_vec<VEC>(src + pi, y);
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
          if (norm) y[c] = w ? y[c] * inv * w[pi + c] : y[c] * inv;
          const float co = cs[2 * (fi + c)], sn = cs[2 * (fi + c) + 1];
          r[c] = i < half ? x[c] * co - y[c] * sn : x[c] * co + y[c] * sn;
        }
      }
      if (dst_f) st_vec<VEC>(dst_f + i, r);
      else st_vec<VEC>(dst_c + i, r);
    }
  }
}

// 8 consecutive elements of a cache row, kept in the cache dtype while the
// load is in flight (a bf16 chunk costs 4 registers) and widened on the way
// into LDS
template <typename T>
struct Chunk8;
template <>
struct Chunk8<short> {
  short8_t x;
  __device__ __forceinline__ void load(const short* p, bool vec, int valid) {
    if (vec && valid >= 8) {
      x = *reinterpret_cast<const short8_t*>(p);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = i < valid ? p[i] : (short)0;
    }
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = 0;
  }
  __device__ __forceinline__ float get(int i) const { return bf16_bits_to_float(x[i]); }
};
template <>
struct Chunk8<float> {
  f32x4 a, b;
  __device__ __forceinline__ void load(const float* p, bool vec, int valid) {
    if (vec && valid >= 8) {
      a = *reinterpret_cast<const f32x4*>(p);
      b = *reinterpret_cast<const f32x4*>(p + 4);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        a[i] = i < valid ? p[i] : 0.f;
        b[i] = 4 + i < valid ? p[4 + i] : 0.f;
      }
    }
  }
  __device__ __forceinline__ void zero() {
    a = f32x4{0.f, 0.f, 0.f, 0.f};
    b = a;
  }
  __device__ __forceinline__ float get(int i) const { return i < 4 ? a[i] : b[i - 4]; }
};

// rows [k0, k0 + nk) of one kv head, WP (padded width) columns: each thread
// owns WP / 32 chunks of 8; fetch() issues the global loads, store() writes
// them to LDS in the cache dtype as [BK][WP + 4], zero past the head size and
// past nk. A bf16 tile is widened when the matrix-core operands are read
// (lds4): half the LDS of an fp32 tile, so twice the blocks per compute unit.
template <typename T, int WP>
struct TileStage {
  static constexpr int CPR = WP / 8;          // chunks per row
  static constexpr int NCH = BK * CPR / NT;   // chunks per thread
  static constexpr int LS = WP + 4;
  Chunk8<T> ch[NCH];

  __device__ __forceinline__ void fetch(const T* cache, const int* bt, int k0,
                                        int nk, int g, int kv_heads, int W,
                                        long row_stride, int block_size,
                                        int bs_shift, bool vec) {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + NT * i;
      const int j = c / CPR, d0 = (c % CPR) * 8;
      const int valid = j < nk ? W - d0 : 0;
      if (valid > 0) {
        const int kp = k0 + j;
        // bs_shift >= 0: pages of 2^bs_shift tokens (no integer division)
        const int pb = bs_shift >= 0 ? kp >> bs_shift : kp / block_size;
        const int po = bs_shift >= 0 ? kp & (block_size - 1) : kp % block_size;
        const long blk = bt[pb];
        ch[i].load(cache + ((blk * kv_heads + g) * block_size + po) * row_stride + d0,
                   vec, valid);
      } else {
        ch[i].zero();
      }
    }
  }
  __device__ __forceinline__ void store(float* dst) const {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + NT * i;
      const int j = c / CPR, d0 = (c % CPR) * 8;
      f32x4* o = reinterpret_cast<f32x4*>(dst + j * LS + d0);
      o[0] = f32x4{ch[i].get(0), ch[i].get(1), ch[i].get(2), ch[i].get(3)};
      o[1] = f32x4{ch[i].get(4), ch[i].get(5), ch[i].get(6), ch[i].get(7)};
    }
  }
  // rows are 8-byte aligned only (LS = WP + 4 elements): two 8-byte stores
  __device__ __forceinline__ void store(short* dst) const {
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
      const int c = threadIdx.x + NT * i;
      const int j = c / CPR, d0 = (c % CPR) * 8;
      short4_t* o = reinterpret_cast<short4_t*>(dst + j * LS + d0);
      o[0] = short4_t{ch[i].x[0], ch[i].x[1], ch[i].x[2], ch[i].x[3]};
      o[1] = short4_t{ch[i].x[4], ch[i].x[5], ch[i].x[6], ch[i].x[7]};
    }
  }
};

// four consecutive tile elements as fp32
__device__ __forceinline__ f32x4 lds4(const float* p) {
  return *reinterpret_cast<const f32x4*>(p);
}
__device__ __forceinline__ f32x4 lds4(const short* p) {
  const short4_t x = *reinterpret_cast<const short4_t*>(p);
  return f32x4{bf16_bits_to_float(x[0]), bf16_bits_to_float(x[1]),
               bf16_bits_to_float(x[2]), bf16_bits_to_float(x[3])};
}

template <typename T, int DP, int DVP, bool SPLITK, bool VK>
__global__ void __launch_bounds__(NT) ctx_attention_f32_kernel(
    T* __restrict__ out, const float* __restrict__ q,
    const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens,
    const T* __restrict__ gate, long gate_stride, float scale, int heads,
    int kv_heads, int D, int DV, int block_size, int hpb,
    const float* __restrict__ sink, int chunk,
    const float* __restrict__ out_inv_freq, int window, long v_row_stride,
    float* __restrict__ ws) {
  extern __shared__ float lds[];
  constexpr int KS = DP + 4;   // K row stride: lanes of one MFMA read hit 64 banks
  // V row stride: likewise for the 4-key-apart rows. VK: the values are the
  // leading columns of the key rows, so the staged K tile serves as V too
  constexpr int VS = VK ? KS : DVP + 4;
  constexpr int ROWS = SPLITK ? 16 : 64;  // query rows per block
  // Staged tiles: fp32 in prefill (widened once when stored; every wave
  // reads the whole tile), the cache dtype in decode (widened when the
  // operands are read; each wave reads a quarter of the tile, and half the
  // LDS means twice the blocks per compute unit, which is what a decode block
  // waiting on its tile loads needs).
  using TL = typename std::conditional<SPLITK, T, float>::type;
  TL* Ks = reinterpret_cast<TL*>(lds);   // [BK][KS]
  TL* Vs = VK ? Ks : Ks + BK * KS;       // [BK][VS]

  const int s = blockIdx.y;
  const int q0 = cu_q[s];
  const int q_len = cu_q[s + 1] - q0;
  const int tpb = ROWS / hpb;  // tokens per block
  // decode: blockIdx.x numbers the key splits of the one token, and block
  // x takes the tiles x, x + nsplit, ... of the visible keys
  const int nsplit = SPLITK ? gridDim.x : 1;
  const int split = SPLITK ? blockIdx.x : 0;
  const int kstep = nsplit * BK;
  const int tok0 = SPLITK ? 0 : blockIdx.x * tpb;
  if (tok0 >= q_len) return;
  const int head0 = blockIdx.z * hpb;
  const int g = head0 / (heads / kv_heads);
  const int ctx = ctx_lens[s];
  const int ntok = min(tpb, q_len - tok0);
  const int nrows = ntok * hpb;
  const int base_pos = ctx - q_len + tok0;  // position of the block's first token
  const int last_pos = base_pos + ntok - 1;

  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int li = lane & 15;  // query column of this lane
  const int lg = lane >> 4;

  // this lane's query
  const int r = (SPLITK ? 0 : wave * 16) + li;
  const bool row_ok = r < nrows;
  const int tok = q0 + tok0 + r / hpb;
  const int hd = head0 + r % hpb;
  const int qpos = row_ok ? base_pos + r / hpb : -1;
  // first visible key of this lane's query, of the block and of this wave
  // (chunk and window exclude each other: the host checks)
  const int qstart = !row_ok      ? 0
                     : chunk > 0  ? qpos / chunk * chunk
                     : window > 0 ? max(qpos - window + 1, 0)
                                  : 0;
  const int kbeg = chunk > 0    ? base_pos / chunk * chunk
                   : window > 0 ? max(base_pos - window + 1, 0)
                                : 0;
  // keys this wave needs: from its first row's chunk up to its own last
  // row's position
  const int wave_last =
      SPLITK ? last_pos : base_pos + min(wave * 16 + 15, nrows - 1) / hpb;
  const int wave_first_pos = base_pos + min(wave * 16, nrows - 1) / hpb;
  const int wave_first =
      SPLITK       ? kbeg
      : chunk > 0  ? wave_first_pos / chunk * chunk
      : window > 0 ? max(wave_first_pos - window + 1, 0)
                   : kbeg;

  // Q^T fragments (B operand). The contraction over the head dimension may
  // run in any order as long as both operands agree: k-step ks of lane group
  // lg stands for d = lg * DP/4 + ks, so a lane's K values are contiguous in
  // LDS (16-byte reads) and so are its q values here. Pre-multiplied by the
  // softmax scale and log2(e): the softmax runs on exp2.
  // Q^T fragments, pre-multiplied by the softmax scale and log2(e) (the
  // softmax runs on exp2). The block's query rows go through LDS first (rows
  // of D contiguous floats, read by consecutive lanes; zero past D and past
  // the last row), where the K tile is staged afterwards: a lane's own
  // values are 64 floats apart from its neighbour's, which global memory
  // serves badly.
  const float qscale = scale * 1.44269504088896340736f;
  float qf[DP / 4];
  {
    float* Qs = lds;  // [ROWS][KS] floats
    for (int e = threadIdx.x; e < ROWS * (DP / 4); e += NT) {
      const int rr = e / (DP / 4), d = (e % (DP / 4)) * 4;
      f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
      if (rr < nrows) {
        const float* src =
            q + ((long)(q0 + tok0 + rr / hpb) * heads + head0 + rr % hpb) * D;
        if ((D % 4) == 0 && d + 3 < D) {
          v = *reinterpret_cast<const f32x4*>(src + d);
        } else {
#pragma unroll
          for (int c = 0; c < 4; ++c)
            if (d + c < D) v[c] = src[d + c];
        }
      }
      *reinterpret_cast<f32x4*>(Qs + rr * KS + d) = v * qscale;
    }
    __syncthreads();
#pragma unroll
    for (int k4 = 0; k4 < DP / 16; ++k4) {
      const f32x4 v =
          *reinterpret_cast<const f32x4*>(Qs + r * KS + lg * (DP / 4) + 4 * k4);
#pragma unroll
      for (int c = 0; c < 4; ++c) qf[4 * k4 + c] = v[c];
    }
    // the first K tile is stored behind the loop's own barrier
  }
  f32x4 o[DVP / 16];
#pragma unroll
  for (int i = 0; i < DVP / 16; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  const int* bt = block_tables + (long)s * bt_stride;
  const bool kvec = (D % 8) == 0;
  const bool vvec = (DV % 8) == 0 && (v_row_stride % 8) == 0 &&
                    ((uintptr_t)v_cache % 32) == 0;
  const int bs_shift =
      (block_size & (block_size - 1)) == 0 ? __builtin_ctz(block_size) : -1;
  constexpr int KT = SPLITK ? 1 : 4;  // 16-key sub-tiles per wave and tile

  // the next tile's global loads are in flight while this one is computed
  TileStage<T, DP> kst;
  TileStage<T, DVP> vst;
  const int kfirst = kbeg + split * BK;
  kst.fetch(k_cache, bt, kfirst, min(BK, last_pos + 1 - kfirst), g, kv_heads, D, D, block_size, bs_shift, kvec);
  if (!VK)
    vst.fetch(v_cache, bt, kfirst, min(BK, last_pos + 1 - kfirst), g, kv_heads, DV, v_row_stride, block_size, bs_shift, vvec);
  for (int k0 = kfirst; k0 <= last_pos; k0 += kstep) {
    __syncthreads();  // previous tile fully consumed
    kst.store(Ks);
    if (!VK) vst.store(Vs);
    __syncthreads();
    if (k0 + kstep <= last_pos) {
      const int nn = min(BK, last_pos + 1 - (k0 + kstep));
      kst.fetch(k_cache, bt, k0 + kstep, nn, g, kv_heads, D, D, block_size, bs_shift, kvec);
      if (!VK)
        vst.fetch(v_cache, bt, k0 + kstep, nn, g, kv_heads, DV, v_row_stride, block_size, bs_shift, vvec);
    }
    if (k0 > wave_last || k0 + BK <= wave_first) continue;

    // S^T sub-tiles: acc[kt][v] = score(key k0 + 16 kt' + 4 lg + v, query li)
    // k-steps outermost, two accumulators per sub-tile: 2 KT independent
    // MFMA chains are in flight instead of one long dependent one
    f32x4 sc[KT], sc2[KT];
#pragma unroll
    for (int t = 0; t < KT; ++t) {
      sc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      sc2[t] = sc[t];
    }
#pragma unroll
    for (int k4 = 0; k4 < DP / 16; ++k4) {
#pragma unroll
      for (int t = 0; t < KT; ++t) {
        const int kt = SPLITK ? wave : t;
        const f32x4 kv = lds4(Ks + (16 * kt + li) * KS + lg * (DP / 4) + 4 * k4);
        sc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[0], qf[4 * k4 + 0], sc[t], 0, 0, 0);
        sc2[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[1], qf[4 * k4 + 1], sc2[t], 0, 0, 0);
        sc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[2], qf[4 * k4 + 2], sc[t], 0, 0, 0);
        sc2[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[3], qf[4 * k4 + 3], sc2[t], 0, 0, 0);
      }
    }
#pragma unroll
    for (int t = 0; t < KT; ++t) sc[t] += sc2[t];
    float mt = -INFINITY;
#pragma unroll
    for (int t = 0; t < KT; ++t) {
      const int kt = SPLITK ? wave : t;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const int kp = k0 + 16 * kt + 4 * lg + v;
        sc[t][v] = (kp <= qpos && kp >= qstart) ? sc[t][v] : -INFINITY;
        mt = fmaxf(mt, sc[t][v]);
      }
    }
    mt = fmaxf(mt, __shfl_xor(mt, 16, WAVE_SIZE));
    mt = fmaxf(mt, __shfl_xor(mt, 32, WAVE_SIZE));
    const float mn = fmaxf(m, mt);
    // a column that has seen no visible key yet keeps mn = -inf
    const float corr = (mn == -INFINITY) ? 1.f : exp2f(m - mn);
    float ps = 0.f;
#pragma unroll
    for (int t = 0; t < KT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        const float pv = sc[t][v] == -INFINITY ? 0.f : exp2f(sc[t][v] - mn);
        sc[t][v] = pv;
        ps += pv;
      }
    ps += __shfl_xor(ps, 16, WAVE_SIZE);
    ps += __shfl_xor(ps, 32, WAVE_SIZE);
    l = l * corr + ps;
    m = mn;
#pragma unroll
    for (int i = 0; i < DVP / 16; ++i) o[i] *= corr;
    // O^T += V^T P^T, contraction index of k-step v = key 4 lg + v
#pragma unroll
    for (int t = 0; t < KT; ++t) {
      const int kt = SPLITK ? wave : t;
#pragma unroll
      for (int v = 0; v < 4; ++v) {
        // row li of output tile i is value column 64 (i/4) + 4 li + i%4: the
        // four tiles of a 64-column block come from one 16-byte read
        const TL* va = Vs + (16 * kt + 4 * lg + v) * VS + 4 * li;
        const float pb = sc[t][v];
#pragma unroll
        for (int j = 0; j < DVP / 64; ++j) {
          const f32x4 vv = lds4(va + 64 * j);
#pragma unroll
          for (int c = 0; c < 4; ++c)
            o[4 * j + c] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv[c], pb, o[4 * j + c], 0, 0, 0);
        }
      }
    }
  }

  if (SPLITK) {
    // merge the four waves' partial results: Ms/Ls [NW][16], Os [NW][16][pw].
    // Value columns go through LDS in passes of pw columns (two passes of
    // 128 for wider values, which bounds the block's LDS; one pass when the
    // output is turned back, since a pair spans both halves of the row).
    const int np = (DVP <= 128 || out_inv_freq) ? 1 : 2;
    const int pw = np == 1 ? DVP : 128;
    __syncthreads();
    float* Ms = lds;
    float* Ls = Ms + NW * 16;
    float* Os = Ls + NW * 16;
    if (lg == 0) {
      Ms[wave * 16 + li] = m;
      Ls[wave * 16 + li] = l;
    }
    for (int p = 0; p < np; ++p) {
      const int c0 = p * pw, c1 = min(DV, c0 + pw);
      if (p) __syncthreads();  // the previous pass has been read
#pragma unroll
      for (int i = 0; i < DVP / 16; ++i)
        if (64 * (i / 4) / pw == p) {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            Os[(wave * 16 + li) * pw + 64 * (i / 4) - c0 + 4 * (4 * lg + v) + i % 4] = o[i][v];
        }
      __syncthreads();
      if (nsplit > 1) {
        // partial (max, sum, weighted values) of this split, merged over the
        // waves; ctx_attention_merge_kernel finishes. ws: per (seq, head,
        // split) DV values, then max and sum.
        const int cw = c1 - c0;
        for (int e = threadIdx.x; e < nrows * cw; e += NT) {
          const int row = e / cw, dv = c0 + e % cw;
          const int h2 = head0 + row % hpb;
          float M = -INFINITY;
#pragma unroll
          for (int w = 0; w < NW; ++w) M = fmaxf(M, Ms[w * 16 + row]);
          float L = 0.f, O = 0.f;
#pragma unroll
          for (int w = 0; w < NW; ++w) {
            const float mw = Ms[w * 16 + row];
            const float f = mw == -INFINITY ? 0.f : exp2f(mw - M);
            L += Ls[w * 16 + row] * f;
            O += Os[(w * 16 + row) * pw + dv - c0] * f;
          }
          float* wr = ws + (((long)s * heads + h2) * nsplit + split) * (DV + 2);
          wr[dv] = O;
          if (dv == 0) {
            wr[DV] = M;
            wr[DV + 1] = L;
          }
        }
        continue;
      }
      // an element pair (dv, dv + DV/2) per thread when the output is turned
      // back (one pass), else one element
      const int ohalf = out_inv_freq ? DV / 2 : 0;
      const int per_row = out_inv_freq ? ohalf : c1 - c0;
      for (int e = threadIdx.x; e < nrows * per_row; e += NT) {
        const int row = e / per_row, dv = c0 + e % per_row;
        const int tk = q0 + tok0 + row / hpb, h2 = head0 + row % hpb;
        float M = -INFINITY;
#pragma unroll
        for (int w = 0; w < NW; ++w) M = fmaxf(M, Ms[w * 16 + row]);
        float L = 0.f;
        if (sink) {
          const float sl = sink[h2] * 1.44269504088896340736f;
          M = fmaxf(M, sl);
          L = exp2f(sl - M);
        }
        float O = 0.f, O2 = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
          const float mw = Ms[w * 16 + row];
          const float f = mw == -INFINITY ? 0.f : exp2f(mw - M);
          L += Ls[w * 16 + row] * f;
          O += Os[(w * 16 + row) * pw + dv - c0] * f;
          if (out_inv_freq) O2 += Os[(w * 16 + row) * pw + dv + ohalf] * f;
        }
        float f = 1.0f / L;
        if (gate) {
          const float gv = ld_f32(gate, (long)tk * gate_stride + h2);
          f *= 1.0f / (1.0f + expf(-gv));
        }
        O *= f;
        if (out_inv_freq) {
          O2 *= f;
          float sn, cs;
          sincosf((float)(base_pos + row / hpb) * out_inv_freq[dv], &sn, &cs);
          st_f32(out, ((long)tk * heads + h2) * DV + dv, O * cs + O2 * sn);
          st_f32(out, ((long)tk * heads + h2) * DV + dv + ohalf, O2 * cs - O * sn);
        } else {
          st_f32(out, ((long)tk * heads + h2) * DV + dv, O);
        }
      }
    }
    return;
  }

  if (row_ok && sink) {
    const float sl = sink[hd] * 1.44269504088896340736f;
    const float mn = fmaxf(m, sl);
    const float corr = m == -INFINITY ? 0.f : exp2f(m - mn);
    l = l * corr + exp2f(sl - mn);
#pragma unroll
    for (int i = 0; i < DVP / 16; ++i) o[i] *= corr;
  }
  float f = row_ok ? 1.0f / l : 0.f;
  if (row_ok && gate) {
    const float gv = ld_f32(gate, (long)tok * gate_stride + hd);
    f *= 1.0f / (1.0f + expf(-gv));
  }
  if (out_inv_freq) {
    // rows through LDS [64][DVP + 1] so that a lane holds both halves of a pair
    constexpr int OS = DVP + 1;
    __syncthreads();  // every wave is done with the K/V tiles
    float* Os = lds;
    if (row_ok) {
#pragma unroll
      for (int i = 0; i < DVP / 16; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v)
          Os[r * OS + 64 * (i / 4) + 4 * (4 * lg + v) + i % 4] = o[i][v] * f;
    }
    __syncthreads();
    const int ohalf = DV / 2;
    for (int e = threadIdx.x; e < nrows * ohalf; e += NT) {
      const int row = e / ohalf, dv = e % ohalf;
      const int tk = q0 + tok0 + row / hpb, h2 = head0 + row % hpb;
      const float a = Os[row * OS + dv], b = Os[row * OS + dv + ohalf];
      float sn, cs;
      sincosf((float)(base_pos + row / hpb) * out_inv_freq[dv], &sn, &cs);
      st_f32(out, ((long)tk * heads + h2) * DV + dv, a * cs + b * sn);
      st_f32(out, ((long)tk * heads + h2) * DV + dv + ohalf, b * cs - a * sn);
    }
    return;
  }
  if (!row_ok) return;
#pragma unroll
  for (int i = 0; i < DVP / 16; ++i)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int dv = 64 * (i / 4) + 4 * (4 * lg + v) + i % 4;
      if (dv < DV) st_f32(out, ((long)tok * heads + hd) * DV + dv, o[i][v] * f);
    }
}

// Second pass of a split decode: one block per (sequence, head) combines the
// splits' partials, adds the sink term, normalises and applies the gate.
template <typename T>
__global__ void ctx_attention_merge_kernel(
    T* __restrict__ out, const float* __restrict__ ws,
    const int* __restrict__ cu_q, const T* __restrict__ gate, long gate_stride,
    const float* __restrict__ sink, int heads, int DV, int nsplit) {
  const int s = blockIdx.x / heads, h = blockIdx.x % heads;
  const int tok = cu_q[s];
  if (cu_q[s + 1] - tok < 1) return;
  const float* wr = ws + ((long)s * heads + h) * nsplit * (DV + 2);
  float M = -INFINITY;
  for (int i = 0; i < nsplit; ++i) M = fmaxf(M, wr[i * (DV + 2) + DV]);
  float L = 0.f;
  if (sink) {
    const float sl = sink[h] * 1.44269504088896340736f;
    M = fmaxf(M, sl);
    L = exp2f(sl - M);
  }
  for (int i = 0; i < nsplit; ++i) {
    const float mi = wr[i * (DV + 2) + DV];
    if (mi != -INFINITY) L += wr[i * (DV + 2) + DV + 1] * exp2f(mi - M);
  }
  float f = 1.0f / L;
  if (gate) {
    const float gv = ld_f32(gate, (long)tok * gate_stride + h);
    f *= 1.0f / (1.0f + expf(-gv));
  }
  for (int dv = threadIdx.x; dv < DV; dv += blockDim.x) {
    float O = 0.f;
    for (int i = 0; i < nsplit; ++i) {
      const float mi = wr[i * (DV + 2) + DV];
      if (mi != -INFINITY) O += wr[i * (DV + 2) + dv] * exp2f(mi - M);
    }
    st_f32(out, ((long)tok * heads + h) * DV + dv, O * f);
  }
}

}  // namespace

extern "C" hipError_t ks_qk_norm_temp_cache(
    void* q_out, const void* q, const void* k, const void* v, long row_stride,
    const void* qw, const void* kw, const void* positions,
    const void* slot_mapping, void* k_cache, void* v_cache, float eps,
    float temp_coef, int temp_every, int tokens, int heads, int kv_heads,
    int D, int DV, int block_size, int is_f32, hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (is_f32)
    hipLaunchKernelGGL(qk_norm_temp_cache_kernel<float>, dim3(tokens), dim3(NT),
                       0, stream, (float*)q_out, (const float*)q,
                       (const float*)k, (const float*)v, row_stride,
                       (const float*)qw, (const float*)kw,
                       (const long*)positions, (const int*)slot_mapping,
                       (float*)k_cache, (float*)v_cache, eps, temp_coef,
                       temp_every, heads * D, kv_heads, D, DV, block_size);
  else
    hipLaunchKernelGGL(qk_norm_temp_cache_kernel<short>, dim3(tokens), dim3(NT),
                       0, stream, (float*)q_out, (const short*)q,
                       (const short*)k, (const short*)v, row_stride,
                       (const float*)qw, (const float*)kw,
                       (const long*)positions, (const int*)slot_mapping,
                       (short*)k_cache, (short*)v_cache, eps, temp_coef,
                       temp_every, heads * D, kv_heads, D, DV, block_size);
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

extern "C" hipError_t ks_qk_headnorm_rope_cache(
    void* q_out, const void* q, const void* k, const void* v, long row_stride,
    const void* qw, const void* kw, const void* positions,
    const void* slot_mapping, void* k_cache, void* v_cache, float eps,
    int tokens, int heads, int kv_heads, int D, int DV, int block_size,
    const void* qk_inv_freq, int qk_half, int v_unit_norm,
    const void* v_inv_freq, int v_half, int is_f32, hipStream_t stream) {
  if (tokens == 0) return hipSuccess;
  if (2 * qk_half > D || 2 * v_half > DV) return hipErrorInvalidValue;
#define HN_ARGS(TT)                                                          \
  (float*)q_out, (const TT*)q, (const TT*)k, (const TT*)v, row_stride,       \
      (const float*)qw, (const float*)kw, (const long*)positions,            \
      (const int*)slot_mapping, (TT*)k_cache, (TT*)v_cache, eps, heads,      \
      kv_heads, D, DV, block_size, (const float*)qk_inv_freq, qk_half,       \
      v_unit_norm, (const float*)v_inv_freq, v_half
  const size_t smem = sizeof(float) * 2 * (size_t)(qk_half + v_half);
  const int esz = is_f32 ? 4 : 2;
  auto al = [&](const void* p) { return ((uintptr_t)p % (2 * esz)) == 0; };
  const bool vec = D % 2 == 0 && DV % 2 == 0 && qk_half % 2 == 0 &&
                   v_half % 2 == 0 && row_stride % 2 == 0 && al(q) && al(k) &&
                   al(v) && al(k_cache) && al(v_cache) &&
                   ((uintptr_t)q_out % 8) == 0;
  if (is_f32) {
    if (vec)
      hipLaunchKernelGGL((qk_headnorm_rope_cache_kernel<float, 2>), dim3(tokens),
                         dim3(NT), smem, stream, HN_ARGS(float));
    else
      hipLaunchKernelGGL((qk_headnorm_rope_cache_kernel<float, 1>), dim3(tokens),
                         dim3(NT), smem, stream, HN_ARGS(float));
  } else {
    if (vec)
      hipLaunchKernelGGL((qk_headnorm_rope_cache_kernel<short, 2>), dim3(tokens),
                         dim3(NT), smem, stream, HN_ARGS(short));
    else
      hipLaunchKernelGGL((qk_headnorm_rope_cache_kernel<short, 1>), dim3(tokens),
                         dim3(NT), smem, stream, HN_ARGS(short));
  }
  HIP_CHECK_KERNEL();
  return hipSuccess;
}

// decode: one token per sequence, a block takes up to 16 heads of one group
static int decode_heads_per_block(int heads, int kv_heads) {
  const int gs = heads / kv_heads;
  int hpb = 1;
  for (int c = 1; c <= 16 && c <= gs; ++c)
    if (gs % c == 0) hpb = c;
  return hpb;
}

// Key splits of a decode launch: enough blocks to put several on every
// compute unit (a block runs few waves and waits on its tile loads), no more
// than 8, and with a window no more than the window has tiles. It cannot
// depend on the context lengths, which only the device knows: a split
// without keys writes an empty partial.
extern "C" int ks_ctx_attention_decode_splits(int num_seqs, int heads,
                                              int kv_heads, int window,
                                              int has_out_rotation) {
  if (has_out_rotation) return 1;
  const int blocks = num_seqs * (heads / decode_heads_per_block(heads, kv_heads));
  int n = cdiv(1024, blocks > 0 ? blocks : 1);
  if (n > 8) n = 8;
  if (window > 0 && n > cdiv(window, BK)) n = cdiv(window, BK);
  return n < 1 ? 1 : n;
}

struct CtxArgs {
  void* out;
  const void *q, *k_cache, *v_cache, *block_tables;
  int bt_stride;
  const void *cu_q, *ctx_lens, *gate;
  long gate_stride;
  float scale;
  int num_seqs, max_q_len, heads, kv_heads, D, DV, block_size;
  const void* sink;
  int chunk;
  const void* out_inv_freq;
  int window;
  long v_row_stride;
  void* ws;
  int nsplit;
  hipStream_t stream;
};

template <typename T, int DP, int DVP, bool VK>
hipError_t launch_ctx_attention(const CtxArgs& a) {
  // the staged tiles are fp32 in prefill and in the cache dtype in decode;
  // the other uses of the same LDS (query rows; decode: cross-wave merge;
  // prefill: rows to turn back) are fp32
  const bool decode = a.max_q_len == 1;
  size_t smem = (decode ? sizeof(T) : sizeof(float)) * (size_t)BK *
                (DP + 4 + (VK ? 0 : DVP + 4));
  int hpb = 1;
  if (decode) {
    hpb = decode_heads_per_block(a.heads, a.kv_heads);
    const int pw = (DVP <= 128 || a.out_inv_freq) ? DVP : 128;
    const size_t merge = sizeof(float) * (size_t)NW * 16 * (pw + 2);
    const size_t qrows = sizeof(float) * (size_t)16 * (DP + 4);
    if (merge > smem) smem = merge;
    if (qrows > smem) smem = qrows;
  } else if (a.out_inv_freq) {
    const size_t rows = sizeof(float) * (size_t)64 * (DVP + 1);
    if (rows > smem) smem = rows;
  }
  const int rows = decode ? 16 : 64;
  const int nsplit = decode ? a.nsplit : 1;
  dim3 grid(decode ? nsplit : cdiv(a.max_q_len, rows / hpb), a.num_seqs,
            a.heads / hpb);
  auto fn = decode ? ctx_attention_f32_kernel<T, DP, DVP, true, VK>
                   : ctx_attention_f32_kernel<T, DP, DVP, false, VK>;
  if (smem > 48 * 1024) {
    hipError_t e = hipFuncSetAttribute(
        (const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
  }
  hipLaunchKernelGGL(fn, grid, dim3(NT), smem, a.stream, (T*)a.out,
                     (const float*)a.q, (const T*)a.k_cache,
                     (const T*)a.v_cache, (const int*)a.block_tables,
                     a.bt_stride, (const int*)a.cu_q, (const int*)a.ctx_lens,
                     (const T*)a.gate, a.gate_stride, a.scale, a.heads,
                     a.kv_heads, a.D, a.DV, a.block_size, hpb,
                     (const float*)a.sink, a.chunk,
                     (const float*)a.out_inv_freq, a.window, a.v_row_stride,
                     (float*)a.ws);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess || nsplit <= 1) return e;
  hipLaunchKernelGGL(ctx_attention_merge_kernel<T>,
                     dim3(a.num_seqs * a.heads), dim3(64), 0, a.stream,
                     (T*)a.out, (const float*)a.ws, (const int*)a.cu_q,
                     (const T*)a.gate, a.gate_stride, (const float*)a.sink,
                     a.heads, a.DV, nsplit);
  return hipGetLastError();
}

template <typename T, int DP, int DVP>
hipError_t dispatch_vk(const CtxArgs& a) {
  // the values are the leading columns of the key rows themselves
  const bool vk = a.v_cache == a.k_cache && a.v_row_stride == a.D && DVP <= DP;
  if constexpr (DVP <= DP) {
    if (vk) return launch_ctx_attention<T, DP, DVP, true>(a);
  }
  return launch_ctx_attention<T, DP, DVP, false>(a);
}

template <typename T, int DP>
hipError_t dispatch_dv(const CtxArgs& a) {
  if (a.DV <= 64) return dispatch_vk<T, DP, 64>(a);
  if (a.DV <= 128) return dispatch_vk<T, DP, 128>(a);
  if (a.DV <= 192) return dispatch_vk<T, DP, 192>(a);
  return dispatch_vk<T, DP, 256>(a);
}

template <typename T>
hipError_t dispatch_d(const CtxArgs& a) {
  if (a.D <= 64) return dispatch_dv<T, 64>(a);
  if (a.D <= 128) return dispatch_dv<T, 128>(a);
  return dispatch_dv<T, 256>(a);
}

extern "C" hipError_t ks_ctx_attention_f32(
    void* out, const void* q, const void* k_cache, const void* v_cache,
    const void* block_tables, int bt_stride, const void* cu_q,
    const void* ctx_lens, const void* gate, long gate_stride, float scale,
    int num_seqs, int max_q_len, int heads, int kv_heads, int D, int DV,
    int block_size, int is_f32, const void* sink, int chunk,
    const void* out_inv_freq, int window, long v_row_stride, void* ws,
    int nsplit, hipStream_t stream) {
  if (num_seqs == 0 || max_q_len == 0) return hipSuccess;
  if (D < 1 || D > 256 || DV < 1 || DV > 256 || kv_heads < 1 ||
      heads % kv_heads != 0 || chunk < 0 || window < 0 ||
      (chunk > 0 && window > 0) || v_row_stride < DV ||
      (out_inv_freq && DV % 2 != 0) || nsplit < 1 || (nsplit > 1 && !ws) ||
      (nsplit > 1 && out_inv_freq))
    return hipErrorInvalidValue;
  const CtxArgs a{out, q, k_cache, v_cache, block_tables, bt_stride, cu_q,
                  ctx_lens, gate, gate_stride, scale, num_seqs, max_q_len,
                  heads, kv_heads, D, DV, block_size, sink, chunk,
                  out_inv_freq, window, v_row_stride, ws, nsplit, stream};
  return is_f32 ? dispatch_d<float>(a) : dispatch_d<short>(a);
}
