// State-space-duality (Mamba-2) mixer kernels for gfx950.
//
//   causal_conv_silu   per-channel causal convolution + bias + silu over
//       a varlen batch. Taps that reach before a chunk's first token
//       read the request's conv tail (its last K-1 inputs, kept in a
//       state row); conv_state_update then advances the tails. Output
//       is fp32 or the input dtype.
//   ssd_scan           the recurrence, one workgroup per (request, head,
//       slab of 16*PA value columns), sequential over the request's
//       tokens with the state in registers:
//           dt' = softplus(dt + dt_bias)
//           S   = exp(-exp(A_log) dt') S + dt' B x^T
//           y   = S^T C + D x
//       Tokens are staged through LDS sixteen at a time, so the inner
//       loop has no workgroup barrier: a thread owns PA columns x NK
//       state rows (n = lane%16 + 16k) and the sum over n is a 16-lane
//       shuffle. The state row layout is [heads, P, N] (n fastest), so
//       state loads and stores are 64 B per 16 lanes. Decode steps are
//       the one-token case of the same kernel.
//   gated_group_rms_norm  (y * silu(z)) normed per group of columns,
//       times a weight; fp32 statistics.
//
// Everything inside the recurrence is fp32.

#include <torch/all.h>
#include <c10/hip/HIPStream.h>

#include "common.h"
#include "pooled_attention.h"

namespace vllm_amd {

namespace {

constexpr int SB = 256;
constexpr int SSD_TT = 16;     // tokens staged per LDS tile
constexpr int SSD_MAX_N = 256;

DEVINL int sfind_req(const int* __restrict__ qsl, int num_reqs, int t) {
  int lo = 0, hi = num_reqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// Sum over the 16 lanes of a DPP row (rotations by 8, 4, 2, 1); every
// lane ends with the total.
DEVINL float row16_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));
  return v;
}

// Four taps, 16-bit input, eight channels per thread with 16 B loads;
// output fp32 (TO = F32Tag) or the input type.
template <typename T, typename TO>
__global__ __launch_bounds__(SB) void causal_conv4_silu_vec_kernel(
    typename ET<TO>::t* __restrict__ out,              // [T, C]
    const short* __restrict__ x, const int64_t x_st,
    const short* __restrict__ w,                       // [C, 4]
    const short* __restrict__ bias,                    // [C]
    const short* __restrict__ conv_state,              // [rows, C, 3]
    const int64_t* __restrict__ state_rows, const int* __restrict__ qsl,
    const int num_reqs, const int C) {
  constexpr int K = 4;
  const int ch0 = (blockIdx.y * SB + threadIdx.x) * 8;
  const int t = blockIdx.x;
  if (ch0 >= C) return;
  const int r = sfind_req(qsl, num_reqs, t);
  const int s = qsl[r];
  const short* hist =
      conv_state == nullptr
          ? nullptr
          : conv_state + (state_rows[r] * C + ch0) * (int64_t)(K - 1);
  // w for channel e, tap j sits at wv[(e * 4 + j) / 8][(e * 4 + j) % 8].
  s16x8 wv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    wv[i] = *reinterpret_cast<const s16x8*>(w + (int64_t)ch0 * K + i * 8);
  const s16x8 bv = *reinterpret_cast<const s16x8*>(bias + ch0);
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = ET<T>::ld(bv[e]);
#pragma unroll
  for (int j = 0; j < K; ++j) {
    const int src = t - (K - 1) + j;
    if (src >= s) {
      const s16x8 xv =
          *reinterpret_cast<const s16x8*>(x + (int64_t)src * x_st + ch0);
#pragma unroll
      for (int e = 0; e < 8; ++e)
        acc[e] += ET<T>::ld(wv[(e * 4 + j) / 8][(e * 4 + j) % 8]) *
                  ET<T>::ld(xv[e]);
    } else if (hist != nullptr) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        acc[e] += ET<T>::ld(wv[(e * 4 + j) / 8][(e * 4 + j) % 8]) *
                  ET<T>::ld(hist[e * (K - 1) + (K - 1) + (src - s)]);
    }
  }
  typename ET<TO>::t* o = out + (int64_t)t * C + ch0;
#pragma unroll
  for (int e = 0; e < 8; ++e)
    o[e] = ET<TO>::st(acc[e] / (1.f + expf(-acc[e])));
}

template <typename T, typename TO>
__global__ __launch_bounds__(SB) void causal_conv_silu_kernel(
    typename ET<TO>::t* __restrict__ out,              // [T, C]
    const typename ET<T>::t* __restrict__ x, const int64_t x_st,
    const typename ET<T>::t* __restrict__ w,           // [C, K]
    const typename ET<T>::t* __restrict__ bias,        // [C]
    const typename ET<T>::t* __restrict__ conv_state,  // [rows, C, K-1]
    const int64_t* __restrict__ state_rows, const int* __restrict__ qsl,
    const int num_reqs, const int C, const int K) {
  const int ch = blockIdx.y * SB + threadIdx.x;
  const int t = blockIdx.x;
  if (ch >= C) return;
  const int r = sfind_req(qsl, num_reqs, t);
  const int s = qsl[r];
  const typename ET<T>::t* hist =
      conv_state == nullptr
          ? nullptr
          : conv_state + (state_rows[r] * C + ch) * (int64_t)(K - 1);
  float acc = ET<T>::ld(bias[ch]);
  for (int j = 0; j < K; ++j) {
    const int src = t - (K - 1) + j;
    float v = 0.f;
    if (src >= s)
      v = ET<T>::ld(x[(int64_t)src * x_st + ch]);
    else if (hist != nullptr)
      v = ET<T>::ld(hist[(K - 1) + (src - s)]);
    acc += ET<T>::ld(w[ch * K + j]) * v;
  }
  out[(int64_t)t * C + ch] = ET<TO>::st(acc / (1.f + expf(-acc)));
}

// New tail[j] = input at chunk offset n-(K-1)+j, which for a negative
// offset is old tail[n+j]; n >= 1, so ascending j never reads a slot it
// has already overwritten.
template <typename T>
__global__ __launch_bounds__(SB) void conv_state_update_kernel(
    typename ET<T>::t* __restrict__ conv_state,
    const typename ET<T>::t* __restrict__ x, const int64_t x_st,
    const int64_t* __restrict__ state_rows, const int* __restrict__ qsl,
    const int C, const int K) {
  const int ch = blockIdx.x * SB + threadIdx.x;
  const int r = blockIdx.y;
  if (ch >= C) return;
  const int s = qsl[r], n = qsl[r + 1] - s;
  if (n <= 0) return;
  typename ET<T>::t* tail =
      conv_state + (state_rows[r] * C + ch) * (int64_t)(K - 1);
  for (int j = 0; j < K - 1; ++j) {
    const int rel = n - (K - 1) + j;
    tail[j] = rel >= 0 ? x[(int64_t)(s + rel) * x_st + ch] : tail[n + j];
  }
}

// A long prompt portion is cut into segments of SSD_SEG tokens that run
// side by side: pass 1 runs every segment from a zero state and keeps
// its end state and the product of its decays, ssd_seg_carry_kernel
// chains those per request (S_in of segment j+1 = decay_j S_in_j + end_j)
// and leaves each segment's true start state in the same buffer, pass 3
// reruns the segments from there and writes y.
constexpr int SSD_SEG = 256;
constexpr int MODE_WHOLE = 0, MODE_LOCAL = 1, MODE_FINAL = 3;

struct Seg {
  int req, t0, t1;
};

DEVINL Seg find_seg(int g, const int* __restrict__ qsl, int num_reqs) {
  for (int r = 0; r < num_reqs; ++r) {
    const int n = qsl[r + 1] - qsl[r];
    const int segs = (n + SSD_SEG - 1) / SSD_SEG;
    if (g < segs) {
      const int t0 = qsl[r] + g * SSD_SEG;
      return Seg{r, t0, min(t0 + SSD_SEG, qsl[r + 1])};
    }
    g -= segs;
  }
  return Seg{-1, 0, 0};
}

__global__ __launch_bounds__(SB) void ssd_seg_carry_kernel(
    float* __restrict__ seg_state,         // [segs, Hm, P*N]
    const float* __restrict__ seg_decay,   // [segs, Hm]
    float* __restrict__ ssm_state,         // [rows, Hm, P*N] or null
    const int64_t* __restrict__ state_rows, const int* __restrict__ qsl,
    const int Hm, const int PN) {
  const int r = blockIdx.x, h = blockIdx.y;
  const int i = blockIdx.z * SB + threadIdx.x;
  if (i >= PN) return;
  int g0 = 0;
  for (int q = 0; q < r; ++q)
    g0 += (qsl[q + 1] - qsl[q] + SSD_SEG - 1) / SSD_SEG;
  const int nseg = (qsl[r + 1] - qsl[r] + SSD_SEG - 1) / SSD_SEG;
  if (nseg == 0) return;
  float* st = ssm_state == nullptr
                  ? nullptr
                  : ssm_state + (state_rows[r] * Hm + h) * (int64_t)PN + i;
  float carry = st != nullptr ? *st : 0.f;
  for (int j = 0; j < nseg; ++j) {
    float* slot = seg_state + ((int64_t)(g0 + j) * Hm + h) * PN + i;
    const float end = *slot;
    *slot = carry;
    carry = seg_decay[(int64_t)(g0 + j) * Hm + h] * carry + end;
  }
  if (st != nullptr) *st = carry;
}

template <int PA, int NK>
__global__ __launch_bounds__(SB) void ssd_scan_kernel(
    float* __restrict__ y,                 // [T, Hm, P]
    const float* __restrict__ xbc,         // [T, Cc]: x | B | C
    const int Cc, const int inner, const int G, const int N,
    const float* __restrict__ dt, const int64_t dt_st,   // [T, Hm] raw
    const float* __restrict__ dt_bias, const float* __restrict__ a_log,
    const float* __restrict__ d_skip,
    float* __restrict__ ssm_state,         // [rows, Hm, P, N] or null
    const int64_t* __restrict__ state_rows, const int* __restrict__ qsl,
    const int Hm, const int P, const int mode, const int num_reqs,
    float* __restrict__ seg_state, float* __restrict__ seg_decay) {
  __shared__ float Bs[SSD_TT][SSD_MAX_N];
  __shared__ float Cs[SSD_TT][SSD_MAX_N];
  __shared__ float xs[SSD_TT][16 * PA];
  __shared__ float ys[SSD_TT][16 * PA];
  __shared__ float dts[SSD_TT], dec[SSD_TT];

  const int h = blockIdx.y;
  const int p0 = blockIdx.z * 16 * PA;
  int r = blockIdx.x, s, e;
  if (mode == MODE_WHOLE) {
    s = qsl[r];
    e = qsl[r + 1];
  } else {
    const Seg sg = find_seg(blockIdx.x, qsl, num_reqs);
    r = sg.req;
    s = sg.t0;
    e = sg.t1;
  }
  if (r < 0 || s >= e) return;
  const int g = h / (Hm / G);
  const int tid = threadIdx.x;
  const int sl = tid & 15, pl = tid >> 4;
  const float A = expf(a_log[h]);
  const float bias = dt_bias[h], dsk = d_skip[h];

  float S[PA][NK];
  float* st;
  if (mode == MODE_WHOLE)
    st = ssm_state == nullptr
             ? nullptr
             : ssm_state + (state_rows[r] * Hm + h) * (int64_t)P * N;
  else
    st = seg_state + ((int64_t)blockIdx.x * Hm + h) * (int64_t)P * N;
  const bool load_state = st != nullptr && mode != MODE_LOCAL;
#pragma unroll
  for (int a = 0; a < PA; ++a) {
    const int p = p0 + pl + 16 * a;
#pragma unroll
    for (int k = 0; k < NK; ++k) {
      const int n = sl + 16 * k;
      S[a][k] = (load_state && p < P && n < N) ? st[(int64_t)p * N + n]
                                               : 0.f;
    }
  }
  float dprod = 1.f;

  const float* Bg = xbc + inner + g * N;
  const float* Cg = xbc + inner + G * N + g * N;
  const float* xh = xbc + h * P + p0;
  for (int t0 = s; t0 < e; t0 += SSD_TT) {
    const int nt = min(SSD_TT, e - t0);
    __syncthreads();          // previous tile's ys / inputs consumed
    for (int i = tid; i < nt * N; i += SB) {
      const int tt = i / N, n = i - tt * N;
      Bs[tt][n] = Bg[(int64_t)(t0 + tt) * Cc + n];
      Cs[tt][n] = Cg[(int64_t)(t0 + tt) * Cc + n];
    }
    for (int i = tid; i < nt * 16 * PA; i += SB) {
      const int tt = i / (16 * PA), pp = i - tt * (16 * PA);
      xs[tt][pp] = (p0 + pp < P) ? xh[(int64_t)(t0 + tt) * Cc + pp] : 0.f;
    }
    if (tid < nt) {
      const float z = dt[(int64_t)(t0 + tid) * dt_st + h] + bias;
      // softplus without a clamp; log1p(exp(z)) overflows past ~88.
      const float sp = z > 20.f ? z : log1pf(expf(z));
      dts[tid] = sp;
      dec[tid] = expf(-A * sp);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float dtp = dts[tt], dc = dec[tt];
      dprod *= dc;
      float xp[PA], yacc[PA];
#pragma unroll
      for (int a = 0; a < PA; ++a) {
        xp[a] = xs[tt][pl + 16 * a] * dtp;
        yacc[a] = 0.f;
      }
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        const int n = sl + 16 * k;
        const float b = n < N ? Bs[tt][n] : 0.f;
        const float c = n < N ? Cs[tt][n] : 0.f;
#pragma unroll
        for (int a = 0; a < PA; ++a) {
          S[a][k] = dc * S[a][k] + b * xp[a];
          yacc[a] += S[a][k] * c;
        }
      }
#pragma unroll
      for (int a = 0; a < PA; ++a) {
        const float v = row16_sum(yacc[a]);
        if (sl == 0) ys[tt][pl + 16 * a] = v;
      }
    }
    __syncthreads();
    if (mode != MODE_LOCAL) {
      for (int i = tid; i < nt * 16 * PA; i += SB) {
        const int tt = i / (16 * PA), pp = i - tt * (16 * PA);
        if (p0 + pp < P)
          y[((int64_t)(t0 + tt) * Hm + h) * P + p0 + pp] =
              ys[tt][pp] + dsk * xs[tt][pp];
      }
    }
  }
  if (mode == MODE_LOCAL && blockIdx.z == 0 && tid == 0)
    seg_decay[(int64_t)blockIdx.x * Hm + h] = dprod;
  if (st != nullptr && mode != MODE_FINAL) {
#pragma unroll
    for (int a = 0; a < PA; ++a) {
      const int p = p0 + pl + 16 * a;
#pragma unroll
      for (int k = 0; k < NK; ++k) {
        const int n = sl + 16 * k;
        if (p < P && n < N) st[(int64_t)p * N + n] = S[a][k];
      }
    }
  }
}

// Up to GN_REG gated values per thread stay in registers between the
// statistics and the output pass; wider groups recompute them.
constexpr int GN_REG = 4;

template <typename TZ, typename TO>
__global__ __launch_bounds__(SB) void gated_group_rms_norm_kernel(
    typename ET<TO>::t* __restrict__ out,       // [T, W]
    const float* __restrict__ y,                // [T, W]
    const typename ET<TZ>::t* __restrict__ z, const int64_t z_st,
    const float* __restrict__ w, const float eps, const int W,
    const int Wg) {
  __shared__ float scratch[4];
  const int64_t t = blockIdx.x;
  const int c0 = blockIdx.y * Wg;
  const bool keep = Wg <= SB * GN_REG;
  float g[GN_REG];
  float ss = 0.f;
  if (keep) {
#pragma unroll
    for (int k = 0; k < GN_REG; ++k) {
      const int c = threadIdx.x + k * SB;
      g[k] = 0.f;
      if (c < Wg) {
        const float zz = ET<TZ>::ld(z[t * z_st + c0 + c]);
        g[k] = y[t * W + c0 + c] * (zz / (1.f + expf(-zz)));
      }
      ss += g[k] * g[k];
    }
  } else {
    for (int c = threadIdx.x; c < Wg; c += SB) {
      const float zz = ET<TZ>::ld(z[t * z_st + c0 + c]);
      const float v = y[t * W + c0 + c] * (zz / (1.f + expf(-zz)));
      ss += v * v;
    }
  }
  ss = wave_reduce_sum(ss);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) scratch[wave] = ss;
  __syncthreads();
  ss = scratch[0] + scratch[1] + scratch[2] + scratch[3];
  const float inv = 1.f / sqrtf(ss / (float)Wg + eps);
  if (keep) {
#pragma unroll
    for (int k = 0; k < GN_REG; ++k) {
      const int c = threadIdx.x + k * SB;
      if (c < Wg) out[t * W + c0 + c] = ET<TO>::st(g[k] * inv * w[c0 + c]);
    }
  } else {
    for (int c = threadIdx.x; c < Wg; c += SB) {
      const float zz = ET<TZ>::ld(z[t * z_st + c0 + c]);
      const float v = y[t * W + c0 + c] * (zz / (1.f + expf(-zz)));
      out[t * W + c0 + c] = ET<TO>::st(v * inv * w[c0 + c]);
    }
  }
}

}  // namespace

#define SDISPATCH(DTYPE, FN)                                      \
  if ((DTYPE) == torch::kBFloat16) { FN(BF16Tag); }               \
  else if ((DTYPE) == torch::kHalf) { FN(FP16Tag); }              \
  else if ((DTYPE) == torch::kFloat32) { FN(F32Tag); }            \
  else { TORCH_CHECK(false, "unsupported dtype"); }

torch::Tensor causal_conv_silu(torch::Tensor x, torch::Tensor weight,
                               torch::Tensor bias,
                               c10::optional<torch::Tensor> conv_state,
                               c10::optional<torch::Tensor> state_rows,
                               torch::Tensor query_start_loc,
                               torch::ScalarType out_dtype) {
  TORCH_CHECK(x.dim() == 2 && x.stride(1) == 1);
  const int T = x.size(0), C = x.size(1);
  TORCH_CHECK(weight.dim() == 2 && weight.is_contiguous() &&
              weight.size(0) == C && bias.is_contiguous() &&
              bias.numel() == C);
  const int K = weight.size(1);
  TORCH_CHECK(K >= 1);
  TORCH_CHECK(weight.scalar_type() == x.scalar_type() &&
              bias.scalar_type() == x.scalar_type());
  TORCH_CHECK(out_dtype == torch::kFloat32 || out_dtype == x.scalar_type());
  TORCH_CHECK(query_start_loc.scalar_type() == torch::kInt32 &&
              query_start_loc.is_contiguous());
  const int num_reqs = query_start_loc.numel() - 1;
  const bool has_state = conv_state.has_value() && K > 1;
  if (has_state) {
    TORCH_CHECK(state_rows.has_value() &&
                state_rows->scalar_type() == torch::kInt64 &&
                state_rows->is_contiguous() &&
                state_rows->numel() >= num_reqs);
    TORCH_CHECK(conv_state->is_contiguous() && conv_state->dim() == 3 &&
                conv_state->size(1) == C && conv_state->size(2) == K - 1 &&
                conv_state->scalar_type() == x.scalar_type());
  }
  auto out = torch::empty({T, C}, x.options().dtype(out_dtype));
  if (T == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec4 = K == 4 && C % 8 == 0 && x.stride(0) % 8 == 0 &&
                    x.storage_offset() % 8 == 0 &&
                    x.scalar_type() != torch::kFloat32;
  if (vec4) {
    const dim3 gv(T, (C / 8 + SB - 1) / SB);
#define LV2(TT, TO)                                                        \
  hipLaunchKernelGGL(                                                      \
      (causal_conv4_silu_vec_kernel<TT, TO>), gv, dim3(SB), 0, stream,     \
      (ET<TO>::t*)out.data_ptr(), (const short*)x.data_ptr(), x.stride(0), \
      (const short*)weight.data_ptr(), (const short*)bias.data_ptr(),      \
      has_state ? (const short*)conv_state->data_ptr() : nullptr,          \
      has_state ? state_rows->data_ptr<int64_t>() : nullptr,               \
      query_start_loc.data_ptr<int>(), num_reqs, C)
    if (x.scalar_type() == torch::kBFloat16) {
      if (out_dtype == torch::kFloat32) { LV2(BF16Tag, F32Tag); }
      else { LV2(BF16Tag, BF16Tag); }
    } else {
      if (out_dtype == torch::kFloat32) { LV2(FP16Tag, F32Tag); }
      else { LV2(FP16Tag, FP16Tag); }
    }
#undef LV2
    HIP_CHECK_KERNEL();
  }
  const dim3 grid(T, (C + SB - 1) / SB);
#define L2(TT, TO)                                                         \
  hipLaunchKernelGGL(                                                      \
      (causal_conv_silu_kernel<TT, TO>), grid, dim3(SB), 0, stream,        \
      (ET<TO>::t*)out.data_ptr(), (const ET<TT>::t*)x.data_ptr(),          \
      x.stride(0), (const ET<TT>::t*)weight.data_ptr(),                    \
      (const ET<TT>::t*)bias.data_ptr(),                                   \
      has_state ? (const ET<TT>::t*)conv_state->data_ptr() : nullptr,      \
      has_state ? state_rows->data_ptr<int64_t>() : nullptr,               \
      query_start_loc.data_ptr<int>(), num_reqs, C, K)
#define L1(TT)                                                             \
  if (out_dtype == torch::kFloat32) { L2(TT, F32Tag); } else { L2(TT, TT); }
  if (!vec4) { SDISPATCH(x.scalar_type(), L1); }
#undef L1
#undef L2
  HIP_CHECK_KERNEL();
  if (has_state) {
    const dim3 g2((C + SB - 1) / SB, num_reqs);
#define L1(TT)                                                             \
  hipLaunchKernelGGL((conv_state_update_kernel<TT>), g2, dim3(SB), 0,      \
                     stream, (ET<TT>::t*)conv_state->data_ptr(),           \
                     (const ET<TT>::t*)x.data_ptr(), x.stride(0),          \
                     state_rows->data_ptr<int64_t>(),                      \
                     query_start_loc.data_ptr<int>(), C, K)
    SDISPATCH(x.scalar_type(), L1);
#undef L1
    HIP_CHECK_KERNEL();
  }
  return out;
}

torch::Tensor ssd_scan(torch::Tensor xbc, int64_t heads, int64_t head_dim,
                       int64_t groups, int64_t state, torch::Tensor dt,
                       torch::Tensor dt_bias, torch::Tensor a_log,
                       torch::Tensor d_skip,
                       c10::optional<torch::Tensor> ssm_state,
                       c10::optional<torch::Tensor> state_rows,
                       torch::Tensor query_start_loc,
                       int64_t max_query_len) {
  const int Hm = heads, P = head_dim, G = groups, N = state;
  TORCH_CHECK(xbc.dim() == 2 && xbc.is_contiguous() &&
              xbc.scalar_type() == torch::kFloat32);
  const int T = xbc.size(0), Cc = xbc.size(1);
  TORCH_CHECK(Cc == Hm * P + 2 * G * N && Hm % G == 0);
  TORCH_CHECK(N <= SSD_MAX_N, "ssd_scan: state size <= 256");
  TORCH_CHECK(dt.dim() == 2 && dt.stride(1) == 1 && dt.size(0) == T &&
              dt.size(1) == Hm && dt.scalar_type() == torch::kFloat32);
  for (const auto& v : {dt_bias, a_log, d_skip})
    TORCH_CHECK(v.scalar_type() == torch::kFloat32 && v.is_contiguous() &&
                v.numel() == Hm);
  TORCH_CHECK(query_start_loc.scalar_type() == torch::kInt32 &&
              query_start_loc.is_contiguous());
  const int num_reqs = query_start_loc.numel() - 1;
  if (ssm_state.has_value()) {
    TORCH_CHECK(state_rows.has_value() &&
                state_rows->scalar_type() == torch::kInt64 &&
                state_rows->is_contiguous() &&
                state_rows->numel() >= num_reqs);
    TORCH_CHECK(ssm_state->is_contiguous() && ssm_state->dim() == 4 &&
                ssm_state->size(1) == Hm && ssm_state->size(2) == P &&
                ssm_state->size(3) == N &&
                ssm_state->scalar_type() == torch::kFloat32);
  }
  auto y = torch::empty({T, Hm, P}, xbc.options());
  if (T == 0 || num_reqs == 0) return y;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  // Columns per workgroup 16*PA with PA in {1,2,4}; wider heads take
  // several slabs (columns are independent). NK covers N in 16s.
  // Fewer columns per workgroup when the batch alone cannot fill the
  // chip (a few long prompts): the recurrence is sequential in time, so
  // width is the only parallelism there is.
  const bool segmented = max_query_len > SSD_SEG;
  const int nseg = segmented ? (T + SSD_SEG - 1) / SSD_SEG + num_reqs : 0;
  const int gx = segmented ? nseg : num_reqs;
  torch::Tensor seg_state, seg_decay;
  if (segmented) {
    seg_state = torch::empty({(int64_t)nseg * Hm * P * N}, xbc.options());
    seg_decay = torch::empty({(int64_t)nseg * Hm}, xbc.options());
  }
  int pa = P <= 16 ? 1 : (P <= 32 ? 2 : 4);
  while (pa > 1 &&
         (int64_t)gx * Hm * ((P + 16 * pa - 1) / (16 * pa)) < 1024)
    pa /= 2;
  const int nk_need = (N + 15) / 16;
  const int nk = nk_need <= 2 ? 2 : (nk_need <= 4 ? 4 : (nk_need <= 8 ? 8
                                                                      : 16));
  const dim3 grid(gx, Hm, (P + 16 * pa - 1) / (16 * pa));
  float* st_ptr =
      ssm_state.has_value() ? ssm_state->data_ptr<float>() : nullptr;
  const int64_t* rows_ptr =
      ssm_state.has_value() ? state_rows->data_ptr<int64_t>() : nullptr;
#define L2(PA_, NK_, MODE_)                                                \
  hipLaunchKernelGGL(                                                      \
      (ssd_scan_kernel<PA_, NK_>), grid, dim3(SB), 0, stream,              \
      y.data_ptr<float>(), xbc.data_ptr<float>(), Cc, Hm * P, G, N,        \
      dt.data_ptr<float>(), dt.stride(0), dt_bias.data_ptr<float>(),       \
      a_log.data_ptr<float>(), d_skip.data_ptr<float>(), st_ptr, rows_ptr, \
      query_start_loc.data_ptr<int>(), Hm, P, MODE_, num_reqs,             \
      segmented ? seg_state.data_ptr<float>() : nullptr,                   \
      segmented ? seg_decay.data_ptr<float>() : nullptr)
#define L1(PA_, MODE_)                                                     \
  if (nk == 2) { L2(PA_, 2, MODE_); } else if (nk == 4) { L2(PA_, 4, MODE_); } \
  else if (nk == 8) { L2(PA_, 8, MODE_); } else { L2(PA_, 16, MODE_); }
#define L0(MODE_)                                                          \
  if (pa == 1) { L1(1, MODE_); } else if (pa == 2) { L1(2, MODE_); }       \
  else { L1(4, MODE_); }
  if (!segmented) {
    L0(MODE_WHOLE);
  } else {
    L0(MODE_LOCAL);
    const int PN = P * N;
    hipLaunchKernelGGL(ssd_seg_carry_kernel,
                       dim3(num_reqs, Hm, (PN + SB - 1) / SB), dim3(SB), 0,
                       stream, seg_state.data_ptr<float>(),
                       seg_decay.data_ptr<float>(), st_ptr, rows_ptr,
                       query_start_loc.data_ptr<int>(), Hm, PN);
    L0(MODE_FINAL);
  }
#undef L0
#undef L1
#undef L2
  HIP_CHECK_KERNEL();
  return y;
}

torch::Tensor gated_group_rms_norm(torch::Tensor y, torch::Tensor z,
                                   torch::Tensor weight, double eps,
                                   int64_t groups,
                                   torch::ScalarType out_dtype) {
  TORCH_CHECK(y.dim() == 2 && y.is_contiguous() &&
              y.scalar_type() == torch::kFloat32);
  const int T = y.size(0), W = y.size(1);
  TORCH_CHECK(z.dim() == 2 && z.stride(1) == 1 && z.size(0) == T &&
              z.size(1) == W);
  TORCH_CHECK(weight.scalar_type() == torch::kFloat32 &&
              weight.is_contiguous() && weight.numel() == W);
  TORCH_CHECK(groups >= 1 && W % groups == 0);
  auto out = torch::empty({T, W}, y.options().dtype(out_dtype));
  if (T == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const dim3 grid(T, groups);
#define L2(TZ, TO)                                                         \
  hipLaunchKernelGGL((gated_group_rms_norm_kernel<TZ, TO>), grid, dim3(SB),\
                     0, stream, (ET<TO>::t*)out.data_ptr(),                \
                     y.data_ptr<float>(), (const ET<TZ>::t*)z.data_ptr(),  \
                     z.stride(0), weight.data_ptr<float>(), (float)eps, W, \
                     (int)(W / groups))
#define L1(TZ)                                                             \
  if (out_dtype == torch::kFloat32) { L2(TZ, F32Tag); }                    \
  else if (out_dtype == torch::kBFloat16) { L2(TZ, BF16Tag); }             \
  else if (out_dtype == torch::kHalf) { L2(TZ, FP16Tag); }                 \
  else { TORCH_CHECK(false, "unsupported out dtype"); }
  SDISPATCH(z.scalar_type(), L1);
#undef L1
#undef L2
  HIP_CHECK_KERNEL();
  return out;
}

}  // namespace vllm_amd
