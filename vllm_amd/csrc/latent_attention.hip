// Latent attention over a paged cache of ONE row per token shared by
// all heads (gfx950): row = [c (L values) | kr (R values)].
//
//   latent_rope_cache_write  per token: rotate the last R coordinates of
//       every query head in place; RMS-norm the first L coordinates of
//       the key projection (weight, eps), rotate its last R, and store
//       the row at the token's slot. Rotation turns coordinate pairs
//       (2i, 2i+1), i < n_pairs, by position * inv_freq[i]; angles,
//       sines and the norm are fp32.
//   latent_attention_rows    one workgroup per (token, head): scores
//       (q_abs . c_j + q_rot . kr_j) * scale over j <= position, online
//       softmax in fp32 whose running state starts at (m = sink_h,
//       l = 1): the sink adds exp(sink_h) to the denominator and nothing
//       to the numerator. Output = sum_j p_j c_j  [T, H, L]. Serves every
//       dtype; bf16 batches with 16 B-stepped widths take the MFMA tile
//       kernel instead
//       (latent_attention_tiles.hip).

#include <torch/all.h>
#include <c10/hip/HIPStream.h>

#include "common.h"
#include "pooled_attention.h"

namespace vllm_amd {

namespace {

constexpr int LB = 256;
constexpr int LAT_MAX_L = 1024;
constexpr int LAT_MAX_R = 256;

DEVINL float lblock_sum(float v, float* scratch) {
  v = wave_reduce_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  return scratch[0] + scratch[1] + scratch[2] + scratch[3];
}

DEVINL float lblock_max(float v, float* scratch) {
  v = wave_reduce_max(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  return fmaxf(fmaxf(scratch[0], scratch[1]),
               fmaxf(scratch[2], scratch[3]));
}

DEVINL int lfind_req(const int* __restrict__ qsl, int num_reqs, int t) {
  int lo = 0, hi = num_reqs - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
  }
  return lo;
}

template <typename T>
__global__ __launch_bounds__(LB) void latent_rope_cache_write_kernel(
    typename ET<T>::t* __restrict__ q, const int64_t q_st, const int H,
    const int nope, const int R,
    const typename ET<T>::t* __restrict__ dkv, const int64_t dkv_st,
    const float* __restrict__ norm_w, const float eps, const int L,
    const int64_t* __restrict__ positions,
    const float* __restrict__ inv_freq, const int n_pairs,
    typename ET<T>::t* __restrict__ cache,
    const int64_t* __restrict__ slot_mapping) {
  __shared__ float scratch[4];
  // One sine / cosine per pair index, shared by every head and the key.
  __shared__ float sn_s[LAT_MAX_R / 2], cs_s[LAT_MAX_R / 2];
  const int64_t t = blockIdx.x;
  const float pos = (float)positions[t];
  const int tid = threadIdx.x;
  const int hd = nope + R;
  for (int i = tid; i < n_pairs; i += LB)
    sincosf(pos * inv_freq[i], &sn_s[i], &cs_s[i]);
  __syncthreads();
  for (int idx = tid; idx < H * n_pairs; idx += LB) {
    const int h = idx / n_pairs, i = idx - h * n_pairs;
    const float sn = sn_s[i], cs = cs_s[i];
    typename ET<T>::t* p = q + t * q_st + h * hd + nope + 2 * i;
    const float u = ET<T>::ld(p[0]), v = ET<T>::ld(p[1]);
    p[0] = ET<T>::st(u * cs - v * sn);
    p[1] = ET<T>::st(v * cs + u * sn);
  }
  if (dkv == nullptr) return;
  const int64_t slot = slot_mapping[t];
  const typename ET<T>::t* d = dkv + t * dkv_st;
  float ss = 0.f;
  for (int c = tid; c < L; c += LB) {
    const float v = ET<T>::ld(d[c]);
    ss += v * v;
  }
  ss = lblock_sum(ss, scratch);
  if (slot < 0) return;
  const float inv = 1.f / sqrtf(ss / (float)L + eps);
  typename ET<T>::t* row = cache + slot * (int64_t)(L + R);
  for (int c = tid; c < L; c += LB)
    row[c] = ET<T>::st(ET<T>::ld(d[c]) * inv * norm_w[c]);
  for (int i = tid; i < n_pairs; i += LB) {
    const float sn = sn_s[i], cs = cs_s[i];
    const float u = ET<T>::ld(d[L + 2 * i]), v = ET<T>::ld(d[L + 2 * i + 1]);
    row[L + 2 * i] = ET<T>::st(u * cs - v * sn);
    row[L + 2 * i + 1] = ET<T>::st(v * cs + u * sn);
  }
  for (int c = 2 * n_pairs + tid; c < R; c += LB) row[L + c] = d[L + c];
}

// NACC output coordinates per thread: c = c_out + a * dvc.
template <typename T, int NACC>
__global__ __launch_bounds__(LB) void latent_attention_rows_kernel(
    typename ET<T>::t* __restrict__ out,            // [T, H, L]
    const typename ET<T>::t* __restrict__ q_abs,    // [T, H, L]
    const int64_t qa_st, const int64_t qa_sh,
    const typename ET<T>::t* __restrict__ q_rot,    // [T, H, R] strided
    const int64_t qr_st, const int64_t qr_sh,
    const typename ET<T>::t* __restrict__ cache,    // [blocks, page, L+R]
    const int* __restrict__ block_table, const int max_blocks,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const float* __restrict__ sink, const float scale, const int num_reqs,
    const int H, const int L, const int R, const int page, const int dvc) {
  __shared__ float q_s[LAT_MAX_L + LAT_MAX_R];
  __shared__ float p_s[LB];
  __shared__ int64_t off_s[LB];
  __shared__ float red_s[LB * NACC];
  __shared__ float scratch[4];

  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int r = lfind_req(qsl, num_reqs, t);
  const int ctx = seq_lens[r];
  const int i = ctx - (qsl[r + 1] - t);          // sequence position
  const int n_keys = i + 1;
  const int* bt = block_table + (int64_t)r * max_blocks;
  const int tid = threadIdx.x;
  const int DK = L + R;

  for (int c = tid; c < L; c += LB)
    q_s[c] = ET<T>::ld(q_abs[t * qa_st + h * qa_sh + c]) * scale;
  for (int c = tid; c < R; c += LB)
    q_s[L + c] = ET<T>::ld(q_rot[t * qr_st + h * qr_sh + c]) * scale;
  __syncthreads();

  const int c_out = tid % dvc;
  const int sl = tid / dvc;
  const int ns = LB / dvc;
  float m_run = -3.0e38f, l_run = 0.f;
  if (sink != nullptr) {
    m_run = sink[h];
    l_run = 1.f;
  }
  float acc[NACC];
#pragma unroll
  for (int a = 0; a < NACC; ++a) acc[a] = 0.f;

  for (int j0 = 0; j0 < n_keys; j0 += LB) {
    const int j = j0 + tid;
    float s = -3.0e38f;
    if (j < n_keys) {
      const int64_t base =
          ((int64_t)bt[j / page] * page + j % page) * DK;
      const typename ET<T>::t* kp = cache + base;
      float dot = 0.f;
      for (int c = 0; c < DK; ++c) dot += q_s[c] * ET<T>::ld(kp[c]);
      off_s[tid] = base;
      s = dot;
    }
    const float m_new = fmaxf(m_run, lblock_max(s, scratch));
    const float p = (j < n_keys) ? expf(s - m_new) : 0.f;
    p_s[tid] = p;
    const float tile_sum = lblock_sum(p, scratch);   // syncs: p_s visible
    const float f = expf(m_run - m_new);
    l_run = l_run * f + tile_sum;
    m_run = m_new;
    const int lim = min(LB, n_keys - j0);
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
      acc[a] *= f;
      const int c = c_out + a * dvc;
      if (c < L) {
        for (int kk = sl; kk < lim; kk += ns)
          acc[a] += p_s[kk] * ET<T>::ld(cache[off_s[kk] + c]);
      }
    }
    __syncthreads();   // p_s / off_s reused by the next tile
  }

#pragma unroll
  for (int a = 0; a < NACC; ++a) red_s[a * LB + tid] = acc[a];
  __syncthreads();
  if (sl == 0) {
#pragma unroll
    for (int a = 0; a < NACC; ++a) {
      const int c = c_out + a * dvc;
      if (c >= L) continue;
      float o = 0.f;
      for (int k = 0; k < ns; ++k) o += red_s[a * LB + k * dvc + c_out];
      out[((int64_t)t * H + h) * L + c] = ET<T>::st(o / l_run);
    }
  }
}

}  // namespace

#define LDISPATCH(DTYPE, FN)                                      \
  if ((DTYPE) == torch::kBFloat16) { FN(BF16Tag); }               \
  else if ((DTYPE) == torch::kHalf) { FN(FP16Tag); }              \
  else if ((DTYPE) == torch::kFloat32) { FN(F32Tag); }            \
  else { TORCH_CHECK(false, "unsupported dtype"); }

void latent_rope_cache_write(torch::Tensor q,
                             c10::optional<torch::Tensor> dkv,
                             c10::optional<torch::Tensor> norm_w, double eps,
                             torch::Tensor positions, torch::Tensor inv_freq,
                             int64_t nope_dim, int64_t kv_rank,
                             c10::optional<torch::Tensor> cache,
                             c10::optional<torch::Tensor> slot_mapping) {
  TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1 &&
              q.stride(1) == q.size(2));
  const int T = q.size(0), H = q.size(1);
  const int R = (int)q.size(2) - (int)nope_dim;
  const int n_pairs = inv_freq.numel();
  TORCH_CHECK(R >= 0 && 2 * n_pairs <= R && R <= LAT_MAX_R,
              "rotation: dims <= rot_dim <= 256");
  TORCH_CHECK(positions.scalar_type() == torch::kInt64 &&
              positions.is_contiguous() && positions.numel() == T);
  TORCH_CHECK(inv_freq.scalar_type() == torch::kFloat32 &&
              inv_freq.is_contiguous());
  const bool write = dkv.has_value();
  if (write) {
    TORCH_CHECK(cache.has_value() && slot_mapping.has_value() &&
                norm_w.has_value());
    TORCH_CHECK(dkv->dim() == 2 && dkv->stride(1) == 1 &&
                dkv->size(0) == T && dkv->size(1) == kv_rank + R);
    TORCH_CHECK(dkv->scalar_type() == q.scalar_type() &&
                cache->scalar_type() == q.scalar_type());
    TORCH_CHECK(cache->is_contiguous() && cache->dim() == 3 &&
                cache->size(2) == kv_rank + R);
    TORCH_CHECK(norm_w->scalar_type() == torch::kFloat32 &&
                norm_w->is_contiguous() && norm_w->numel() == kv_rank);
    TORCH_CHECK(slot_mapping->scalar_type() == torch::kInt64 &&
                slot_mapping->is_contiguous() &&
                slot_mapping->numel() == T);
  }
  if (T == 0) return;
  auto stream = c10::hip::getCurrentHIPStream().stream();
#define L1(TT)                                                             \
  hipLaunchKernelGGL(                                                      \
      (latent_rope_cache_write_kernel<TT>), dim3(T), dim3(LB), 0, stream,  \
      (ET<TT>::t*)q.data_ptr(), q.stride(0), H, (int)nope_dim, R,          \
      write ? (const ET<TT>::t*)dkv->data_ptr() : nullptr,                 \
      write ? dkv->stride(0) : 0,                                          \
      write ? norm_w->data_ptr<float>() : nullptr, (float)eps,             \
      (int)kv_rank, positions.data_ptr<int64_t>(),                         \
      inv_freq.data_ptr<float>(), n_pairs,                                 \
      write ? (ET<TT>::t*)cache->data_ptr() : nullptr,                     \
      write ? slot_mapping->data_ptr<int64_t>() : nullptr)
  LDISPATCH(q.scalar_type(), L1);
#undef L1
  HIP_CHECK_KERNEL();
}

void latent_check_args(const torch::Tensor& out, const torch::Tensor& q_abs,
                       const torch::Tensor& q_rot,
                       const torch::Tensor& cache,
                       const torch::Tensor& block_table,
                       const torch::Tensor& query_start_loc,
                       const torch::Tensor& seq_lens,
                       const c10::optional<torch::Tensor>& sink) {
  TORCH_CHECK(q_abs.dim() == 3 && q_rot.dim() == 3 && cache.dim() == 3);
  const int64_t T = q_abs.size(0), H = q_abs.size(1), L = q_abs.size(2);
  const int64_t R = q_rot.size(2);
  TORCH_CHECK(q_rot.size(0) == T && q_rot.size(1) == H);
  TORCH_CHECK(q_abs.stride(2) == 1 && (R == 0 || q_rot.stride(2) == 1));
  TORCH_CHECK(cache.is_contiguous() && cache.size(2) == L + R);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 3 && out.size(0) == T &&
              out.size(1) == H && out.size(2) == L);
  TORCH_CHECK(q_abs.scalar_type() == q_rot.scalar_type() &&
              q_abs.scalar_type() == cache.scalar_type() &&
              q_abs.scalar_type() == out.scalar_type());
  TORCH_CHECK(block_table.scalar_type() == torch::kInt32 &&
              block_table.dim() == 2 && block_table.stride(1) == 1);
  TORCH_CHECK(query_start_loc.scalar_type() == torch::kInt32 &&
              seq_lens.scalar_type() == torch::kInt32 &&
              query_start_loc.is_contiguous() && seq_lens.is_contiguous());
  TORCH_CHECK(query_start_loc.numel() == seq_lens.numel() + 1);
  TORCH_CHECK(block_table.size(0) >= seq_lens.numel());
  if (sink.has_value())
    TORCH_CHECK(sink->scalar_type() == torch::kFloat32 &&
                sink->is_contiguous() && sink->numel() == H);
}

void latent_attention_rows(torch::Tensor out, torch::Tensor q_abs,
                           torch::Tensor q_rot, torch::Tensor cache,
                           torch::Tensor block_table,
                           torch::Tensor query_start_loc,
                           torch::Tensor seq_lens,
                           c10::optional<torch::Tensor> sink, double scale) {
  latent_check_args(out, q_abs, q_rot, cache, block_table, query_start_loc,
                    seq_lens, sink);
  const int T = q_abs.size(0), H = q_abs.size(1), L = q_abs.size(2);
  const int R = q_rot.size(2);
  TORCH_CHECK(L <= LAT_MAX_L && R <= LAT_MAX_R,
              "latent attention: kv_rank <= 1024 and rot_dim <= 256");
  if (T == 0) return;
  int dvc = 1;
  while (dvc < L && dvc < LB) dvc *= 2;
  const int nacc = (L + dvc - 1) / dvc;
  const int num_reqs = seq_lens.numel();
  auto stream = c10::hip::getCurrentHIPStream().stream();
#define L2(TT, NA)                                                         \
  hipLaunchKernelGGL(                                                      \
      (latent_attention_rows_kernel<TT, NA>), dim3(T, H), dim3(LB), 0,     \
      stream, (ET<TT>::t*)out.data_ptr(),                                  \
      (const ET<TT>::t*)q_abs.data_ptr(), q_abs.stride(0), q_abs.stride(1),\
      (const ET<TT>::t*)q_rot.data_ptr(), q_rot.stride(0), q_rot.stride(1),\
      (const ET<TT>::t*)cache.data_ptr(), block_table.data_ptr<int>(),     \
      (int)block_table.stride(0), query_start_loc.data_ptr<int>(),         \
      seq_lens.data_ptr<int>(),                                            \
      sink.has_value() ? sink->data_ptr<float>() : nullptr, (float)scale,  \
      num_reqs, H, L, R, (int)cache.size(1), dvc)
#define L1(TT)                                                             \
  if (nacc == 1) { L2(TT, 1); }                                            \
  else if (nacc == 2) { L2(TT, 2); }                                       \
  else { L2(TT, 4); }
  LDISPATCH(q_abs.scalar_type(), L1);
#undef L1
#undef L2
  HIP_CHECK_KERNEL();
}

}  // namespace vllm_amd
