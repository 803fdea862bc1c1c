// Kernels for decoder stacks with an fp32 residual stream, scalar-gain
// RMS norms on sublayer outputs, token shift, and sliding-window
// attention whose far context is mean-pooled blocks (gfx950 / CDNA4).
//
//   scalar_rms_norm        x / sqrt(mean(x^2)+eps) * g        (one g)
//   add_scaled_scalar_norm res += m * norm(y)  [+ cast copy of res]
//   token_shift            h + (h_prev - h) * mu, carry in state rows
//   norm_qk_cache_write    per-head RMS norm of q and k fused with the
//                          paged K/V write (K and V widths may differ)
//   pool_update            finalize the pooled blocks a step completed
//   pooled_window_attention  one workgroup per (token, head): online
//                          softmax over [pooled blocks | window tokens],
//                          sigmoid output gate in the epilogue. Serves
//                          decode rows at any dtype and every row in
//                          fp32; 16-bit prefill rows run on the MFMA
//                          tile kernel in pooled_attention_prefill.hip.
//
// Scores, softmax, norms and the residual are fp32 in every dtype.
// Cache layout: k [blocks, G, 64, D], v [blocks, G, 64, Dv], pooled
// areas fp32 [blocks, G, slots, D|Dv]; pooled block b (positions
// b*P .. b*P+P-1) sits in the page of its last position, slot
// b - (page*64)/P.

#include <torch/all.h>
#include <c10/hip/HIPStream.h>

#include "common.h"
#include "pooled_attention.h"

namespace vllm_amd {

namespace {

constexpr int EW_BLOCK = 256;

DEVINL float block_sum_256(float v, float* scratch) {
  v = wave_reduce_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  return scratch[0] + scratch[1] + scratch[2] + scratch[3];
}

DEVINL float block_max_256(float v, float* scratch) {
  v = wave_reduce_max(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  return fmaxf(fmaxf(scratch[0], scratch[1]),
               fmaxf(scratch[2], scratch[3]));
}

// ---------------------------------------------------------------------
template <typename TI, typename TO>
__global__ __launch_bounds__(EW_BLOCK) void scalar_rms_norm_kernel(
    typename ET<TO>::t* __restrict__ out,
    const typename ET<TI>::t* __restrict__ x, const float* __restrict__ gain,
    const float eps, const int width) {
  __shared__ float scratch[4];
  const int64_t row = blockIdx.x;
  const typename ET<TI>::t* xr = x + row * width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += EW_BLOCK) {
    const float v = ET<TI>::ld(xr[c]);
    ss += v * v;
  }
  ss = block_sum_256(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  const float g = gain[0];
  for (int c = threadIdx.x; c < width; c += EW_BLOCK)
    out[row * width + c] = ET<TO>::st(ET<TI>::ld(xr[c]) * inv * g);
}

template <typename TY, typename TO>
__global__ __launch_bounds__(EW_BLOCK) void add_scaled_scalar_norm_kernel(
    float* __restrict__ residual, const typename ET<TY>::t* __restrict__ y,
    const float* __restrict__ gain, const float eps, const float mult,
    const int width, typename ET<TO>::t* __restrict__ out_copy) {
  __shared__ float scratch[4];
  const int64_t row = blockIdx.x;
  const typename ET<TY>::t* yr = y + row * width;
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += EW_BLOCK) {
    const float v = ET<TY>::ld(yr[c]);
    ss += v * v;
  }
  ss = block_sum_256(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  const float g = gain[0];
  for (int c = threadIdx.x; c < width; c += EW_BLOCK) {
    const float r =
        residual[row * width + c] + mult * (ET<TY>::ld(yr[c]) * inv * g);
    residual[row * width + c] = r;
    if (out_copy != nullptr) out_copy[row * width + c] = ET<TO>::st(r);
  }
}

// 4-wide variants (width % 4 == 0, width <= 4 * EW_BLOCK * EW_VCH): 16 B
// fp32 accesses, and the sublayer output stays in registers between the
// sum of squares and the add.
constexpr int EW_VCH = 4;

template <typename T>
DEVINL f32x4 ld4(const typename ET<T>::t* __restrict__ p) {
  if constexpr (sizeof(typename ET<T>::t) == 4) {
    return *reinterpret_cast<const f32x4*>(p);
  } else {
    const s16x4 v = *reinterpret_cast<const s16x4*>(p);
    return f32x4{ET<T>::ld(v[0]), ET<T>::ld(v[1]), ET<T>::ld(v[2]),
                 ET<T>::ld(v[3])};
  }
}

template <typename T>
DEVINL void st4(typename ET<T>::t* __restrict__ p, const f32x4 v) {
  if constexpr (sizeof(typename ET<T>::t) == 4) {
    *reinterpret_cast<f32x4*>(p) = v;
  } else {
    *reinterpret_cast<s16x4*>(p) =
        s16x4{ET<T>::st(v[0]), ET<T>::st(v[1]), ET<T>::st(v[2]),
              ET<T>::st(v[3])};
  }
}

template <typename TI, typename TO>
__global__ __launch_bounds__(EW_BLOCK) void scalar_rms_norm_vec_kernel(
    typename ET<TO>::t* __restrict__ out,
    const typename ET<TI>::t* __restrict__ x, const float* __restrict__ gain,
    const float eps, const int width) {
  __shared__ float scratch[4];
  const int64_t row = blockIdx.x;
  const typename ET<TI>::t* xr = x + row * width;
  f32x4 xv[EW_VCH];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < EW_VCH; ++k) {
    const int c = (k * EW_BLOCK + threadIdx.x) * 4;
    xv[k] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (c < width) xv[k] = ld4<TI>(xr + c);
    ss += xv[k][0] * xv[k][0] + xv[k][1] * xv[k][1] + xv[k][2] * xv[k][2] +
          xv[k][3] * xv[k][3];
  }
  ss = block_sum_256(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  const float g = gain[0];
#pragma unroll
  for (int k = 0; k < EW_VCH; ++k) {
    const int c = (k * EW_BLOCK + threadIdx.x) * 4;
    if (c >= width) continue;
    f32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = xv[k][e] * inv * g;
    st4<TO>(out + row * width + c, o);
  }
}

template <typename TY, typename TO>
__global__ __launch_bounds__(EW_BLOCK) void add_scaled_scalar_norm_vec_kernel(
    float* __restrict__ residual, const typename ET<TY>::t* __restrict__ y,
    const float* __restrict__ gain, const float eps, const float mult,
    const int width, typename ET<TO>::t* __restrict__ out_copy) {
  __shared__ float scratch[4];
  const int64_t row = blockIdx.x;
  const typename ET<TY>::t* yr = y + row * width;
  f32x4 yv[EW_VCH];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < EW_VCH; ++k) {
    const int c = (k * EW_BLOCK + threadIdx.x) * 4;
    yv[k] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (c < width) yv[k] = ld4<TY>(yr + c);
    ss += yv[k][0] * yv[k][0] + yv[k][1] * yv[k][1] + yv[k][2] * yv[k][2] +
          yv[k][3] * yv[k][3];
  }
  ss = block_sum_256(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)width + eps);
  const float g = gain[0];
#pragma unroll
  for (int k = 0; k < EW_VCH; ++k) {
    const int c = (k * EW_BLOCK + threadIdx.x) * 4;
    if (c >= width) continue;
    f32x4 r = *reinterpret_cast<const f32x4*>(residual + row * width + c);
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = r[e] + mult * (yv[k][e] * inv * g);
    *reinterpret_cast<f32x4*>(residual + row * width + c) = r;
    if (out_copy != nullptr) st4<TO>(out_copy + row * width + c, r);
  }
}

// Request that owns flat token t: largest r with qsl[r] <= t.
DEVINL int find_req(const int* __restrict__ qsl, int num_reqs, int t) {
  int lo = 0, hi = num_reqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

template <typename TO>
__global__ __launch_bounds__(EW_BLOCK) void token_shift_kernel(
    typename ET<TO>::t* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ mu, const float* __restrict__ state,
    const int64_t* __restrict__ state_rows, const int* __restrict__ qsl,
    const int num_reqs, const int width) {
  const int t = blockIdx.x;
  const int r = find_req(qsl, num_reqs, t);
  const bool first = (t == qsl[r]);
  const float* prev = nullptr;
  if (!first) prev = x + (int64_t)(t - 1) * width;
  else if (state != nullptr) prev = state + state_rows[r] * width;
  const float* xr = x + (int64_t)t * width;
  for (int c = threadIdx.x; c < width; c += EW_BLOCK) {
    const float h = xr[c];
    const float p = prev != nullptr ? prev[c] : 0.f;
    out[(int64_t)t * width + c] = ET<TO>::st(h + (p - h) * mu[c]);
  }
}

template <typename TO>
__global__ __launch_bounds__(EW_BLOCK) void token_shift_vec_kernel(
    typename ET<TO>::t* __restrict__ out, const float* __restrict__ x,
    const float* __restrict__ mu, const float* __restrict__ state,
    const int64_t* __restrict__ state_rows, const int* __restrict__ qsl,
    const int num_reqs, const int width) {
  const int t = blockIdx.x;
  const int r = find_req(qsl, num_reqs, t);
  const bool first = (t == qsl[r]);
  const float* prev = nullptr;
  if (!first) prev = x + (int64_t)(t - 1) * width;
  else if (state != nullptr) prev = state + state_rows[r] * width;
  const float* xr = x + (int64_t)t * width;
  for (int c = threadIdx.x * 4; c < width; c += EW_BLOCK * 4) {
    const f32x4 h = *reinterpret_cast<const f32x4*>(xr + c);
    const f32x4 m = *reinterpret_cast<const f32x4*>(mu + c);
    f32x4 p = f32x4{0.f, 0.f, 0.f, 0.f};
    if (prev != nullptr) p = *reinterpret_cast<const f32x4*>(prev + c);
    f32x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = h[e] + (p[e] - h[e]) * m[e];
    st4<TO>(out + (int64_t)t * width + c, o);
  }
}

__global__ __launch_bounds__(EW_BLOCK) void shift_state_save_kernel(
    float* __restrict__ state, const float* __restrict__ x,
    const int64_t* __restrict__ state_rows, const int* __restrict__ qsl,
    const int width) {
  const int r = blockIdx.x;
  const int s = qsl[r], e = qsl[r + 1];
  if (e <= s) return;
  const float* xr = x + (int64_t)(e - 1) * width;
  float* dst = state + state_rows[r] * width;
  for (int c = threadIdx.x; c < width; c += EW_BLOCK) dst[c] = xr[c];
}

template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void silu_and_mul_any_kernel(
    typename ET<T>::t* __restrict__ out,
    const typename ET<T>::t* __restrict__ x, const int d) {
  const int64_t row = blockIdx.x;
  for (int c = threadIdx.x; c < d; c += EW_BLOCK) {
    const float a = ET<T>::ld(x[row * 2 * d + c]);
    const float b = ET<T>::ld(x[row * 2 * d + d + c]);
    out[row * d + c] = ET<T>::st(a / (1.f + expf(-a)) * b);
  }
}

// ---------------------------------------------------------------------
// One wave per (token, head slot): slots [0,H) = q heads (normed to
// q_out), [H,H+G) = k heads (normed into the cache), [H+G,H+2G) = v.
template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void norm_qk_cache_write_kernel(
    typename ET<T>::t* __restrict__ q_out,        // [T, H, D]
    const typename ET<T>::t* __restrict__ q_in, const int64_t q_stride,
    const typename ET<T>::t* __restrict__ k_in, const int64_t k_stride,
    const typename ET<T>::t* __restrict__ v_in, const int64_t v_stride,
    const typename ET<T>::t* __restrict__ q_w,    // [D] or null
    const typename ET<T>::t* __restrict__ k_w,    // [D] or null
    const float eps, typename ET<T>::t* __restrict__ k_cache,
    typename ET<T>::t* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, const int H, const int G,
    const int D, const int Dv, const int block_size) {
  const int t = blockIdx.x;
  const int slot_id = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (slot_id >= H + 2 * G) return;
  const int64_t slot = slot_mapping[t];
  if (slot_id < H + G) {
    const bool is_q = slot_id < H;
    const int head = is_q ? slot_id : slot_id - H;
    if (!is_q && slot < 0) return;
    const typename ET<T>::t* src =
        is_q ? q_in + t * q_stride + (int64_t)head * D
             : k_in + t * k_stride + (int64_t)head * D;
    const typename ET<T>::t* w = is_q ? q_w : k_w;
    typename ET<T>::t* dst;
    if (is_q) {
      dst = q_out + ((int64_t)t * H + head) * D;
    } else {
      const int64_t blk = slot / block_size, off = slot % block_size;
      dst = k_cache + ((blk * G + head) * block_size + off) * D;
    }
    float inv = 1.f;
    if (w != nullptr) {
      float ss = 0.f;
      for (int c = lane; c < D; c += 64) {
        const float v = ET<T>::ld(src[c]);
        ss += v * v;
      }
      ss = wave_reduce_sum(ss);
      inv = 1.f / sqrtf(ss / (float)D + eps);
    }
    for (int c = lane; c < D; c += 64) {
      float v = ET<T>::ld(src[c]);
      if (w != nullptr) v = v * inv * ET<T>::ld(w[c]);
      dst[c] = ET<T>::st(v);
    }
  } else {
    if (slot < 0) return;
    const int head = slot_id - H - G;
    const typename ET<T>::t* src = v_in + t * v_stride + (int64_t)head * Dv;
    const int64_t blk = slot / block_size, off = slot % block_size;
    typename ET<T>::t* dst =
        v_cache + ((blk * G + head) * block_size + off) * Dv;
    for (int c = lane; c < Dv; c += 64) dst[c] = src[c];
  }
}

// 16-bit, 8-aligned variant: 16 lanes per (token, head slot), 8 channels
// = one 16 B access per lane and 128-channel stride; a 256-thread block
// covers 16 head slots. Head widths up to 256 stay in registers.
template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void norm_qk_cache_write_vec_kernel(
    short* __restrict__ q_out, const short* __restrict__ q_in,
    const int64_t q_stride, const short* __restrict__ k_in,
    const int64_t k_stride, const short* __restrict__ v_in,
    const int64_t v_stride, const short* __restrict__ q_w,
    const short* __restrict__ k_w, const float eps,
    short* __restrict__ k_cache, short* __restrict__ v_cache,
    const int64_t* __restrict__ slot_mapping, const int H, const int G,
    const int D, const int Dv, const int block_size) {
  const int t = blockIdx.x;
  const int slot_id = blockIdx.y * 16 + (threadIdx.x >> 4);
  const int l16 = threadIdx.x & 15;
  if (slot_id >= H + 2 * G) return;
  const int64_t slot = slot_mapping[t];
  const bool is_q = slot_id < H;
  const bool is_v = slot_id >= H + G;
  if (!is_q && slot < 0) return;
  const int head = is_q ? slot_id : (is_v ? slot_id - H - G : slot_id - H);
  const int W = is_v ? Dv : D;
  const short* src = is_q ? q_in + t * q_stride + (int64_t)head * D
                   : is_v ? v_in + t * v_stride + (int64_t)head * Dv
                          : k_in + t * k_stride + (int64_t)head * D;
  short* dst;
  if (is_q) {
    dst = q_out + ((int64_t)t * H + head) * D;
  } else {
    const int64_t blk = slot / block_size, off = slot % block_size;
    dst = (is_v ? v_cache : k_cache) +
          ((blk * G + head) * block_size + off) * W;
  }
  const short* w = is_q ? q_w : (is_v ? nullptr : k_w);
  s16x8 raw[2];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const int c = k * 128 + l16 * 8;
    if (c < W) {
      raw[k] = *reinterpret_cast<const s16x8*>(src + c);
      if (w != nullptr) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float f = ET<T>::ld(raw[k][e]);
          ss += f * f;
        }
      }
    }
  }
  if (w != nullptr) {
    ss = group16_reduce_sum(ss);
    const float inv = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int c = k * 128 + l16 * 8;
      if (c < W) {
        const s16x8 wv = *reinterpret_cast<const s16x8*>(w + c);
#pragma unroll
        for (int e = 0; e < 8; ++e)
          raw[k][e] = ET<T>::st(ET<T>::ld(raw[k][e]) * inv *
                                ET<T>::ld(wv[e]));
      }
    }
  }
#pragma unroll
  for (int k = 0; k < 2; ++k) {
    const int c = k * 128 + l16 * 8;
    if (c < W) *reinterpret_cast<s16x8*>(dst + c) = raw[k];
  }
}

// Pooled blocks whose last position was written this step:
// b in [start / P, end / P) with start = seq_len - query_len.
template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void pool_update_kernel(
    float* __restrict__ pool_k, float* __restrict__ pool_v,
    const typename ET<T>::t* __restrict__ k_cache,
    const typename ET<T>::t* __restrict__ v_cache,
    const int* __restrict__ block_table, const int max_blocks,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int G, const int D, const int Dv, const int block_size,
    const int P, const int slots) {
  const int r = blockIdx.x;
  const int g = blockIdx.z;
  const int end = seq_lens[r];
  const int start = end - (qsl[r + 1] - qsl[r]);
  const int* bt = block_table + (int64_t)r * max_blocks;
  const float inv = 1.f / (float)P;
  for (int b = start / P + blockIdx.y; b < end / P; b += gridDim.y) {
    const int last = b * P + P - 1;
    const int page = last / block_size;
    const int slot = b - (page * block_size) / P;
    const int64_t pb = bt[page];
    for (int c = threadIdx.x; c < D + Dv; c += EW_BLOCK) {
      const bool is_k = c < D;
      const int cc = is_k ? c : c - D;
      const int W = is_k ? D : Dv;
      const typename ET<T>::t* cache = is_k ? k_cache : v_cache;
      float s = 0.f;
#pragma unroll 4
      for (int p = b * P; p <= last; ++p) {
        const int64_t blk = bt[p / block_size];
        s += ET<T>::ld(
            cache[((blk * G + g) * block_size + p % block_size) * W + cc]);
      }
      float* dst = is_k ? pool_k : pool_v;
      dst[((pb * G + g) * slots + slot) * W + cc] = s * inv;
    }
  }
}

// 16-bit, 8-aligned variant: (D + Dv) / 8 lanes cover one position with
// 16 B loads and the remaining threads take other positions of the
// block, so a block of P positions costs P * (D + Dv) / 2048 dependent
// loads per thread instead of P. Position slices merge through LDS in a
// fixed order (the mean of a block never depends on the step that
// finished it).
template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void pool_update_vec_kernel(
    float* __restrict__ pool_k, float* __restrict__ pool_v,
    const short* __restrict__ k_cache, const short* __restrict__ v_cache,
    const int* __restrict__ block_table, const int max_blocks,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const int G, const int D, const int Dv, const int block_size,
    const int P, const int slots) {
  __shared__ float red[EW_BLOCK][9];     // padded: no bank conflicts
  const int r = blockIdx.x;
  const int g = blockIdx.z;
  const int end = seq_lens[r];
  const int start = end - (qsl[r + 1] - qsl[r]);
  const int* bt = block_table + (int64_t)r * max_blocks;
  const float inv = 1.f / (float)P;
  const int LP = (D + Dv) / 8;           // lanes per position
  const int NS = EW_BLOCK / LP;          // position slices
  const int lane = threadIdx.x % LP;
  const int slice = threadIdx.x / LP;
  const bool is_k = lane * 8 < D;
  const int cc = is_k ? lane * 8 : lane * 8 - D;
  const int W = is_k ? D : Dv;
  const short* cache = is_k ? k_cache : v_cache;
  for (int b = start / P + blockIdx.y; b < end / P; b += gridDim.y) {
    const int last = b * P + P - 1;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    if (slice < NS) {
#pragma unroll 4
      for (int p = b * P + slice; p <= last; p += NS) {
        const int64_t blk = bt[p / block_size];
        const s16x8 v = *reinterpret_cast<const s16x8*>(
            cache + ((blk * G + g) * block_size + p % block_size) * W + cc);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += ET<T>::ld(v[e]);
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) red[threadIdx.x][e] = acc[e];
    __syncthreads();
    if (slice == 0) {
      const int page = last / block_size;
      const int slot = b - (page * block_size) / P;
      const int64_t pb = bt[page];
      float* dst = (is_k ? pool_k : pool_v) +
                   ((pb * G + g) * slots + slot) * W + cc;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float t = 0.f;
        for (int sl = 0; sl < NS; ++sl) t += red[sl * LP + lane][e];
        dst[e] = t * inv;
      }
    }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------
// One workgroup per (token, head). Keys are enumerated as
// [pooled 0..nb) | window tokens lo..i], 256 per tile: thread-per-key
// scores, block softmax statistics, then (channel, key-slice) threads
// accumulate p*V.
constexpr int PWA_MAXD = 256;

template <typename T>
__global__ __launch_bounds__(EW_BLOCK) void pwa_rowwise_kernel(
    typename ET<T>::t* __restrict__ out,        // [T, H, Dv]
    const typename ET<T>::t* __restrict__ q,    // [T, H, D]
    const typename ET<T>::t* __restrict__ k_cache,
    const typename ET<T>::t* __restrict__ v_cache,
    const float* __restrict__ pool_k, const float* __restrict__ pool_v,
    const int* __restrict__ block_table, const int max_blocks,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const typename ET<T>::t* __restrict__ gate, const int64_t gate_stride,
    const float scale, const int num_reqs, const int row0, const int H,
    const int G, const int D, const int Dv, const int block_size,
    const int window, const int P, const int slots, const int dvc) {
  __shared__ float q_s[PWA_MAXD];
  __shared__ float p_s[EW_BLOCK];
  __shared__ int64_t voff_s[EW_BLOCK];
  __shared__ float red_s[EW_BLOCK];
  __shared__ float scratch[4];

  const int t = row0 + blockIdx.x;
  const int h = blockIdx.y;
  const int g = h / (H / G);
  const int r = find_req(qsl, num_reqs, t);
  const int L = seq_lens[r];
  const int i = L - (qsl[r + 1] - t);          // sequence position
  const int lo = max(0, i - window + 1);
  const int nb = max(0, (i - window + 1) / P);
  const int n_keys = nb + (i - lo + 1);
  const int* bt = block_table + (int64_t)r * max_blocks;
  const int tid = threadIdx.x;

  for (int c = tid; c < D; c += EW_BLOCK)
    q_s[c] = ET<T>::ld(q[((int64_t)t * H + h) * D + c]) * scale;
  __syncthreads();

  const int c_out = tid % dvc;
  const int sl = tid / dvc;
  const int ns = EW_BLOCK / dvc;
  float m_run = -3.0e38f, l_run = 0.f, acc = 0.f;

  for (int j0 = 0; j0 < n_keys; j0 += EW_BLOCK) {
    const int j = j0 + tid;
    float s = -3.0e38f;
    if (j < n_keys) {
      float dot = 0.f;
      if (j < nb) {
        const int last = j * P + P - 1;
        const int page = last / block_size;
        const int slot = j - (page * block_size) / P;
        const int64_t base = ((int64_t)bt[page] * G + g) * slots + slot;
        const float* kp = pool_k + base * D;
        for (int c = 0; c < D; ++c) dot += q_s[c] * kp[c];
        voff_s[tid] = -(base * Dv) - 1;          // negative: pooled area
      } else {
        const int pos = lo + (j - nb);
        const int64_t base =
            ((int64_t)bt[pos / block_size] * G + g) * block_size +
            pos % block_size;
        const typename ET<T>::t* kp = k_cache + base * D;
        for (int c = 0; c < D; ++c) dot += q_s[c] * ET<T>::ld(kp[c]);
        voff_s[tid] = base * Dv;
      }
      s = dot;
    }
    const float m_new = fmaxf(m_run, block_max_256(s, scratch));
    const float p = (j < n_keys) ? expf(s - m_new) : 0.f;
    p_s[tid] = p;
    const float tile_sum = block_sum_256(p, scratch);  // syncs: p_s visible
    const float f = expf(m_run - m_new);
    l_run = l_run * f + tile_sum;
    acc *= f;
    m_run = m_new;
    if (c_out < Dv) {
      const int lim = min(EW_BLOCK, n_keys - j0);
      for (int kk = sl; kk < lim; kk += ns) {
        const int64_t vo = voff_s[kk];
        const float v = vo < 0 ? pool_v[-(vo + 1) + c_out]
                               : ET<T>::ld(v_cache[vo + c_out]);
        acc += p_s[kk] * v;
      }
    }
    __syncthreads();   // p_s / voff_s reused by the next tile
  }

  red_s[tid] = acc;
  __syncthreads();
  if (sl == 0 && c_out < Dv) {
    float o = 0.f;
    for (int k = 0; k < ns; ++k) o += red_s[k * dvc + c_out];
    o /= l_run;
    if (gate != nullptr) {
      const float z = ET<T>::ld(gate[(int64_t)t * gate_stride + h]);
      o *= 1.f / (1.f + expf(-z));
    }
    out[((int64_t)t * H + h) * Dv + c_out] = ET<T>::st(o);
  }
}

}  // namespace

// ---------------------------------------------------------------------
// Host side.

#define DISPATCH_ANY(DTYPE, FN)                                   \
  if ((DTYPE) == torch::kBFloat16) { FN(BF16Tag); }               \
  else if ((DTYPE) == torch::kHalf) { FN(FP16Tag); }              \
  else if ((DTYPE) == torch::kFloat32) { FN(F32Tag); }            \
  else { TORCH_CHECK(false, "unsupported dtype"); }

torch::Tensor scalar_rms_norm(torch::Tensor x, torch::Tensor gain,
                              double eps, torch::ScalarType out_dtype) {
  TORCH_CHECK(x.is_contiguous() && x.dim() == 2);
  TORCH_CHECK(gain.scalar_type() == torch::kFloat32 && gain.numel() == 1);
  auto out = torch::empty(x.sizes(), x.options().dtype(out_dtype));
  const int rows = x.size(0), width = x.size(1);
  if (rows == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = width % 4 == 0 && width <= 4 * EW_BLOCK * EW_VCH;
#define L2(TI, TO)                                                         \
  if (vec)                                                                 \
    hipLaunchKernelGGL((scalar_rms_norm_vec_kernel<TI, TO>), dim3(rows),   \
                       dim3(EW_BLOCK), 0, stream,                          \
                       (ET<TO>::t*)out.data_ptr(),                         \
                       (const ET<TI>::t*)x.data_ptr(),                     \
                       gain.data_ptr<float>(), (float)eps, width);         \
  else                                                                     \
  hipLaunchKernelGGL((scalar_rms_norm_kernel<TI, TO>), dim3(rows),         \
                     dim3(EW_BLOCK), 0, stream,                            \
                     (ET<TO>::t*)out.data_ptr(),                           \
                     (const ET<TI>::t*)x.data_ptr(),                       \
                     gain.data_ptr<float>(), (float)eps, width)
#define L1(TI)                                                             \
  if (out_dtype == torch::kFloat32) { L2(TI, F32Tag); }                    \
  else if (out_dtype == torch::kBFloat16) { L2(TI, BF16Tag); }             \
  else if (out_dtype == torch::kHalf) { L2(TI, FP16Tag); }                 \
  else { TORCH_CHECK(false, "unsupported out dtype"); }
  DISPATCH_ANY(x.scalar_type(), L1);
#undef L1
#undef L2
  HIP_CHECK_KERNEL();
  return out;
}

torch::Tensor add_scaled_scalar_norm(torch::Tensor residual, torch::Tensor y,
                                     torch::Tensor gain, double eps,
                                     double mult,
                                     c10::optional<torch::ScalarType> out_dtype) {
  TORCH_CHECK(residual.scalar_type() == torch::kFloat32 &&
              residual.is_contiguous() && y.is_contiguous());
  TORCH_CHECK(residual.sizes() == y.sizes() && residual.dim() == 2);
  TORCH_CHECK(gain.scalar_type() == torch::kFloat32 && gain.numel() == 1);
  const int rows = residual.size(0), width = residual.size(1);
  const bool copy = out_dtype.has_value() && *out_dtype != torch::kFloat32;
  torch::Tensor out = residual;
  if (copy) out = torch::empty(residual.sizes(),
                               residual.options().dtype(*out_dtype));
  if (rows == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = width % 4 == 0 && width <= 4 * EW_BLOCK * EW_VCH;
#define L2(TY, TO)                                                         \
  if (vec)                                                                 \
    hipLaunchKernelGGL((add_scaled_scalar_norm_vec_kernel<TY, TO>),        \
                       dim3(rows), dim3(EW_BLOCK), 0, stream,              \
                       residual.data_ptr<float>(),                         \
                       (const ET<TY>::t*)y.data_ptr(),                     \
                       gain.data_ptr<float>(), (float)eps, (float)mult,    \
                       width, copy ? (ET<TO>::t*)out.data_ptr() : nullptr);\
  else                                                                     \
  hipLaunchKernelGGL((add_scaled_scalar_norm_kernel<TY, TO>), dim3(rows),  \
                     dim3(EW_BLOCK), 0, stream, residual.data_ptr<float>(),\
                     (const ET<TY>::t*)y.data_ptr(), gain.data_ptr<float>(),\
                     (float)eps, (float)mult, width,                       \
                     copy ? (ET<TO>::t*)out.data_ptr() : nullptr)
#define L1(TY)                                                             \
  if (!copy) { L2(TY, F32Tag); }                                           \
  else if (*out_dtype == torch::kBFloat16) { L2(TY, BF16Tag); }            \
  else if (*out_dtype == torch::kHalf) { L2(TY, FP16Tag); }                \
  else { TORCH_CHECK(false, "unsupported out dtype"); }
  DISPATCH_ANY(y.scalar_type(), L1);
#undef L1
#undef L2
  HIP_CHECK_KERNEL();
  return out;
}

torch::Tensor token_shift(torch::Tensor x, torch::Tensor mu,
                          c10::optional<torch::Tensor> state,
                          c10::optional<torch::Tensor> state_rows,
                          torch::Tensor query_start_loc,
                          torch::ScalarType out_dtype) {
  TORCH_CHECK(x.scalar_type() == torch::kFloat32 && x.is_contiguous() &&
              x.dim() == 2);
  TORCH_CHECK(mu.scalar_type() == torch::kFloat32 &&
              mu.numel() == x.size(1));
  TORCH_CHECK(query_start_loc.scalar_type() == torch::kInt32);
  const int T = x.size(0), width = x.size(1);
  const int num_reqs = query_start_loc.size(0) - 1;
  auto out = torch::empty(x.sizes(), x.options().dtype(out_dtype));
  if (T == 0 || num_reqs <= 0) return out;
  const bool has_state = state.has_value();
  if (has_state) {
    TORCH_CHECK(state->scalar_type() == torch::kFloat32 &&
                state->is_contiguous() && state->size(1) == width);
    TORCH_CHECK(state_rows.has_value() &&
                state_rows->scalar_type() == torch::kInt64 &&
                state_rows->numel() >= num_reqs);
  }
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = width % 4 == 0;
#define L(TO)                                                              \
  if (vec)                                                                 \
    hipLaunchKernelGGL((token_shift_vec_kernel<TO>), dim3(T),              \
                       dim3(EW_BLOCK), 0, stream,                          \
                       (ET<TO>::t*)out.data_ptr(), x.data_ptr<float>(),    \
                       mu.data_ptr<float>(),                               \
                       has_state ? state->data_ptr<float>() : nullptr,     \
                       has_state ? state_rows->data_ptr<int64_t>()         \
                                 : nullptr,                                \
                       query_start_loc.data_ptr<int>(), num_reqs, width);  \
  else                                                                     \
  hipLaunchKernelGGL((token_shift_kernel<TO>), dim3(T), dim3(EW_BLOCK), 0, \
                     stream, (ET<TO>::t*)out.data_ptr(),                   \
                     x.data_ptr<float>(), mu.data_ptr<float>(),            \
                     has_state ? state->data_ptr<float>() : nullptr,       \
                     has_state ? state_rows->data_ptr<int64_t>() : nullptr,\
                     query_start_loc.data_ptr<int>(), num_reqs, width)
  DISPATCH_ANY(out_dtype, L);
#undef L
  if (has_state)
    hipLaunchKernelGGL(shift_state_save_kernel, dim3(num_reqs),
                       dim3(EW_BLOCK), 0, stream, state->data_ptr<float>(),
                       x.data_ptr<float>(), state_rows->data_ptr<int64_t>(),
                       query_start_loc.data_ptr<int>(), width);
  HIP_CHECK_KERNEL();
  return out;
}

torch::Tensor silu_and_mul_any(torch::Tensor x) {
  TORCH_CHECK(x.is_contiguous() && x.dim() == 2 && x.size(1) % 2 == 0);
  const int rows = x.size(0), d = x.size(1) / 2;
  auto out = torch::empty({rows, d}, x.options());
  if (rows == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
#define L(TT)                                                              \
  hipLaunchKernelGGL((silu_and_mul_any_kernel<TT>), dim3(rows),            \
                     dim3(EW_BLOCK), 0, stream, (ET<TT>::t*)out.data_ptr(),\
                     (const ET<TT>::t*)x.data_ptr(), d)
  DISPATCH_ANY(x.scalar_type(), L);
#undef L
  HIP_CHECK_KERNEL();
  return out;
}

static void check_caches(const torch::Tensor& k_cache,
                         const torch::Tensor& v_cache) {
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 4 &&
              k_cache.is_contiguous() && v_cache.is_contiguous());
  TORCH_CHECK(k_cache.size(0) == v_cache.size(0) &&
              k_cache.size(1) == v_cache.size(1) &&
              k_cache.size(2) == v_cache.size(2));
  TORCH_CHECK(k_cache.scalar_type() == v_cache.scalar_type());
}

torch::Tensor norm_qk_cache_write(torch::Tensor q, torch::Tensor k,
                                  torch::Tensor v,
                                  c10::optional<torch::Tensor> q_w,
                                  c10::optional<torch::Tensor> k_w, double eps,
                                  torch::Tensor k_cache, torch::Tensor v_cache,
                                  torch::Tensor slot_mapping) {
  check_caches(k_cache, v_cache);
  TORCH_CHECK(q.dim() == 3 && k.dim() == 3 && v.dim() == 3);
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k.size(1), Dv = v.size(2);
  TORCH_CHECK(k.size(0) == T && v.size(0) == T && k.size(2) == D &&
              v.size(1) == G);
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D &&
              v_cache.size(3) == Dv);
  TORCH_CHECK(q.stride(2) == 1 && q.stride(1) == D && k.stride(2) == 1 &&
              k.stride(1) == D && v.stride(2) == 1 && v.stride(1) == Dv,
              "q/k/v must be head-contiguous");
  TORCH_CHECK(q.scalar_type() == k_cache.scalar_type() &&
              k.scalar_type() == q.scalar_type() &&
              v.scalar_type() == q.scalar_type(),
              "cache dtype must equal the compute dtype");
  TORCH_CHECK(slot_mapping.scalar_type() == torch::kInt64 &&
              slot_mapping.numel() >= T);
  TORCH_CHECK(q_w.has_value() == k_w.has_value());
  if (q_w.has_value())
    TORCH_CHECK(q_w->numel() == D && k_w->numel() == D &&
                q_w->scalar_type() == q.scalar_type() &&
                k_w->scalar_type() == q.scalar_type());
  auto q_out = torch::empty({T, H, D}, q.options());
  if (T == 0) return q_out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  auto al16 = [](const torch::Tensor& x) {
    return reinterpret_cast<uintptr_t>(x.data_ptr()) % 16 == 0;
  };
  const bool vec =
      q.scalar_type() != torch::kFloat32 && D % 8 == 0 && Dv % 8 == 0 &&
      D <= 256 && Dv <= 256 && q.stride(0) % 8 == 0 && k.stride(0) % 8 == 0 &&
      v.stride(0) % 8 == 0 && al16(q) && al16(k) && al16(v) &&
      (!q_w.has_value() || (al16(*q_w) && al16(*k_w)));
  if (vec) {
    dim3 vgrid(T, (H + 2 * G + 15) / 16);
#define LV(TT)                                                             \
  hipLaunchKernelGGL(                                                      \
      (norm_qk_cache_write_vec_kernel<TT>), vgrid, dim3(EW_BLOCK), 0,      \
      stream, (short*)q_out.data_ptr(), (const short*)q.data_ptr(),        \
      q.stride(0), (const short*)k.data_ptr(), k.stride(0),                \
      (const short*)v.data_ptr(), v.stride(0),                             \
      q_w.has_value() ? (const short*)q_w->data_ptr() : nullptr,           \
      k_w.has_value() ? (const short*)k_w->data_ptr() : nullptr,           \
      (float)eps, (short*)k_cache.data_ptr(), (short*)v_cache.data_ptr(),  \
      slot_mapping.data_ptr<int64_t>(), H, G, D, Dv, (int)k_cache.size(2))
    if (q.scalar_type() == torch::kBFloat16) { LV(BF16Tag); }
    else { LV(FP16Tag); }
#undef LV
    HIP_CHECK_KERNEL();
    return q_out;
  }
  dim3 grid(T, (H + 2 * G + 3) / 4);
#define L(TT)                                                              \
  hipLaunchKernelGGL(                                                      \
      (norm_qk_cache_write_kernel<TT>), grid, dim3(EW_BLOCK), 0, stream,   \
      (ET<TT>::t*)q_out.data_ptr(), (const ET<TT>::t*)q.data_ptr(),        \
      q.stride(0), (const ET<TT>::t*)k.data_ptr(), k.stride(0),            \
      (const ET<TT>::t*)v.data_ptr(), v.stride(0),                         \
      q_w.has_value() ? (const ET<TT>::t*)q_w->data_ptr() : nullptr,       \
      k_w.has_value() ? (const ET<TT>::t*)k_w->data_ptr() : nullptr,       \
      (float)eps, (ET<TT>::t*)k_cache.data_ptr(),                          \
      (ET<TT>::t*)v_cache.data_ptr(), slot_mapping.data_ptr<int64_t>(), H, \
      G, D, Dv, (int)k_cache.size(2))
  DISPATCH_ANY(q.scalar_type(), L);
#undef L
  HIP_CHECK_KERNEL();
  return q_out;
}

void pool_update(torch::Tensor k_cache, torch::Tensor v_cache,
                 torch::Tensor pool_k, torch::Tensor pool_v,
                 torch::Tensor block_table, torch::Tensor query_start_loc,
                 torch::Tensor seq_lens, int64_t pool,
                 int64_t max_query_len) {
  check_caches(k_cache, v_cache);
  const int G = k_cache.size(1), bs = k_cache.size(2);
  const int D = k_cache.size(3), Dv = v_cache.size(3);
  const int slots = pool_k.size(2);
  TORCH_CHECK(pool >= 1 && slots == (bs + pool - 1) / pool);
  TORCH_CHECK(pool_k.scalar_type() == torch::kFloat32 &&
              pool_v.scalar_type() == torch::kFloat32 &&
              pool_k.is_contiguous() && pool_v.is_contiguous());
  TORCH_CHECK(pool_k.size(0) == k_cache.size(0) && pool_k.size(1) == G &&
              pool_k.size(3) == D && pool_v.size(0) == k_cache.size(0) &&
              pool_v.size(1) == G && pool_v.size(2) == slots &&
              pool_v.size(3) == Dv);
  TORCH_CHECK(block_table.scalar_type() == torch::kInt32 &&
              block_table.is_contiguous() &&
              seq_lens.scalar_type() == torch::kInt32 &&
              query_start_loc.scalar_type() == torch::kInt32);
  const int num_reqs = seq_lens.size(0);
  TORCH_CHECK(block_table.size(0) >= num_reqs &&
              query_start_loc.size(0) >= num_reqs + 1);
  if (num_reqs == 0 || max_query_len <= 0) return;
  // A step of n tokens completes at most n / P + 1 pooled blocks.
  // Workgroups stride over them, so a wide batch with one long chunk
  // does not launch a grid of mostly idle workgroups.
  const int per_req = (int)(max_query_len / pool) + 1;
  const int wide = std::max(1, 8192 / (num_reqs * G));
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid(num_reqs, std::min(per_req, wide), G);
  if (k_cache.scalar_type() != torch::kFloat32 && D % 8 == 0 &&
      Dv % 8 == 0 && (D + Dv) / 8 <= EW_BLOCK) {
#define LV(TT)                                                             \
  hipLaunchKernelGGL((pool_update_vec_kernel<TT>), grid, dim3(EW_BLOCK), 0,\
                     stream, pool_k.data_ptr<float>(),                     \
                     pool_v.data_ptr<float>(),                             \
                     (const short*)k_cache.data_ptr(),                     \
                     (const short*)v_cache.data_ptr(),                     \
                     block_table.data_ptr<int>(), (int)block_table.size(1),\
                     query_start_loc.data_ptr<int>(),                      \
                     seq_lens.data_ptr<int>(), G, D, Dv, bs, (int)pool,    \
                     slots)
    if (k_cache.scalar_type() == torch::kBFloat16) { LV(BF16Tag); }
    else { LV(FP16Tag); }
#undef LV
    HIP_CHECK_KERNEL();
    return;
  }
#define L(TT)                                                              \
  hipLaunchKernelGGL((pool_update_kernel<TT>), grid, dim3(EW_BLOCK), 0,    \
                     stream, pool_k.data_ptr<float>(),                     \
                     pool_v.data_ptr<float>(),                             \
                     (const ET<TT>::t*)k_cache.data_ptr(),                 \
                     (const ET<TT>::t*)v_cache.data_ptr(),                 \
                     block_table.data_ptr<int>(), (int)block_table.size(1),\
                     query_start_loc.data_ptr<int>(),                      \
                     seq_lens.data_ptr<int>(), G, D, Dv, bs, (int)pool,    \
                     slots)
  DISPATCH_ANY(k_cache.scalar_type(), L);
#undef L
  HIP_CHECK_KERNEL();
}

void pwa_check_args(const torch::Tensor& out, const torch::Tensor& q,
                    const torch::Tensor& k_cache,
                    const torch::Tensor& v_cache,
                    const torch::Tensor& pool_k, const torch::Tensor& pool_v,
                    const torch::Tensor& block_table,
                    const torch::Tensor& query_start_loc,
                    const torch::Tensor& seq_lens,
                    const c10::optional<torch::Tensor>& gate, int64_t window,
                    int64_t pool) {
  check_caches(k_cache, v_cache);
  TORCH_CHECK(q.dim() == 3 && q.is_contiguous() && out.is_contiguous());
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k_cache.size(1), bs = k_cache.size(2);
  const int Dv = v_cache.size(3);
  TORCH_CHECK(out.size(0) == T && out.size(1) == H && out.size(2) == Dv);
  TORCH_CHECK(k_cache.size(3) == D && H % G == 0);
  TORCH_CHECK(D <= PWA_MAXD && Dv <= PWA_MAXD,
              "head widths above 256 are not supported");
  TORCH_CHECK(q.scalar_type() == k_cache.scalar_type() &&
              out.scalar_type() == q.scalar_type());
  TORCH_CHECK(window >= 1 && pool >= 1);
  TORCH_CHECK(pool_k.scalar_type() == torch::kFloat32 &&
              pool_v.scalar_type() == torch::kFloat32 &&
              pool_k.is_contiguous() && pool_v.is_contiguous());
  TORCH_CHECK(pool_k.size(0) == k_cache.size(0) && pool_k.size(1) == G &&
              pool_k.size(2) == (bs + pool - 1) / pool &&
              pool_k.size(3) == D && pool_v.size(0) == k_cache.size(0) &&
              pool_v.size(1) == G && pool_v.size(2) == pool_k.size(2) &&
              pool_v.size(3) == Dv);
  TORCH_CHECK(block_table.scalar_type() == torch::kInt32 &&
              block_table.is_contiguous() &&
              seq_lens.scalar_type() == torch::kInt32 &&
              query_start_loc.scalar_type() == torch::kInt32);
  const int num_reqs = seq_lens.size(0);
  TORCH_CHECK(block_table.size(0) >= num_reqs &&
              query_start_loc.size(0) >= num_reqs + 1);
  if (gate.has_value())
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == T &&
                gate->size(1) == H && gate->stride(1) == 1 &&
                gate->scalar_type() == q.scalar_type());
}

// Rows [row0, row0 + num_rows) of the flat batch on the row-wise kernel.
void pooled_window_attention_rows(
    torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
    torch::Tensor v_cache, torch::Tensor pool_k, torch::Tensor pool_v,
    torch::Tensor block_table, torch::Tensor query_start_loc,
    torch::Tensor seq_lens, c10::optional<torch::Tensor> gate, double scale,
    int64_t window, int64_t pool, int64_t row0, int64_t num_rows) {
  pwa_check_args(out, q, k_cache, v_cache, pool_k, pool_v, block_table,
                 query_start_loc, seq_lens, gate, window, pool);
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  TORCH_CHECK(row0 >= 0 && num_rows >= 0 && row0 + num_rows <= T);
  if (num_rows == 0) return;
  const int G = k_cache.size(1), bs = k_cache.size(2);
  const int Dv = v_cache.size(3);
  int dvc = 16;
  while (dvc < Dv) dvc *= 2;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid((int)num_rows, H);
#define L(TT)                                                              \
  hipLaunchKernelGGL(                                                      \
      (pwa_rowwise_kernel<TT>), grid, dim3(EW_BLOCK), 0, stream,           \
      (ET<TT>::t*)out.data_ptr(), (const ET<TT>::t*)q.data_ptr(),          \
      (const ET<TT>::t*)k_cache.data_ptr(),                                \
      (const ET<TT>::t*)v_cache.data_ptr(), pool_k.data_ptr<float>(),      \
      pool_v.data_ptr<float>(), block_table.data_ptr<int>(),               \
      (int)block_table.size(1), query_start_loc.data_ptr<int>(),           \
      seq_lens.data_ptr<int>(),                                            \
      gate.has_value() ? (const ET<TT>::t*)gate->data_ptr() : nullptr,     \
      gate.has_value() ? gate->stride(0) : 0, (float)scale,                \
      (int)seq_lens.size(0), (int)row0, H, G, D, Dv, bs, (int)window,      \
      (int)pool, (int)pool_k.size(2), dvc)
  DISPATCH_ANY(q.scalar_type(), L);
#undef L
  HIP_CHECK_KERNEL();
}

}  // namespace vllm_amd
