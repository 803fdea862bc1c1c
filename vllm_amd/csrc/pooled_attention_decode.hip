// Decode kernel for sliding-window attention with mean-pooled far
// blocks (gfx950, bf16/fp16). Companion of pooled_attention.hip (row-wise
// kernel: fp32 and fallback) and pooled_attention_prefill.hip (MFMA
// tiles for prompt chunks).
//
// A decode row reads min(L, window) cached keys plus one fp32 mean per
// finished far block and does a handful of flops per byte, so this is a
// streaming VALU kernel shaped like the paged decode kernel of the
// other families:
//   - one workgroup = (decode row, kv head [x chunk of its query
//     heads], partition of PD_PART keys); the keys of a row are
//     enumerated as [pooled 0..nb) | window tokens lo..i];
//   - HD/8 lanes cover one key (8 channels = one 16 B load per lane),
//     so 256 threads stream 256*8/HD keys per iteration, and every K/V
//     byte is read once for all query heads of the group;
//   - each key slot keeps its own online-softmax state (m, l, acc) and
//     the slots merge through LDS at the end; partitions merge in a
//     small second kernel (LSE merge) which also applies the sigmoid
//     output gate. A row whose keys fit one partition skips the merge.
// Scores, softmax statistics and accumulators are fp32.

#include <torch/all.h>
#include <c10/hip/HIPStream.h>

#include "common.h"
#include "pooled_attention.h"

namespace vllm_amd {

void pwa_check_args(const torch::Tensor& out, const torch::Tensor& q,
                    const torch::Tensor& k_cache,
                    const torch::Tensor& v_cache,
                    const torch::Tensor& pool_k, const torch::Tensor& pool_v,
                    const torch::Tensor& block_table,
                    const torch::Tensor& query_start_loc,
                    const torch::Tensor& seq_lens,
                    const c10::optional<torch::Tensor>& gate, int64_t window,
                    int64_t pool);

namespace {

constexpr int PD_BLOCK = 256;
constexpr int PD_PART = 256;          // keys per partition
constexpr float PD_NEG = -3.0e38f;

// 8 consecutive channels [d0, d0+8) of a 16-bit row of width W.
template <typename Tag>
DEVINL void load8_16(float (&dst)[8], const short* __restrict__ row,
                     const int d0, const int W, const bool vec) {
  if (vec) {
    if (d0 < W) {
      const s16x8 v = *reinterpret_cast<const s16x8*>(row + d0);
#pragma unroll
      for (int e = 0; e < 8; ++e) dst[e] = to_f32<Tag>(v[e]);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) dst[e] = 0.f;
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      dst[e] = (d0 + e < W) ? to_f32<Tag>(row[d0 + e]) : 0.f;
  }
}

DEVINL void load8_f32(float (&dst)[8], const float* __restrict__ row,
                      const int d0, const int W, const bool vec) {
  if (vec) {
    if (d0 < W) {
      const f32x4 a = *reinterpret_cast<const f32x4*>(row + d0);
      const f32x4 b = *reinterpret_cast<const f32x4*>(row + d0 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) { dst[e] = a[e]; dst[4 + e] = b[e]; }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) dst[e] = 0.f;
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) dst[e] = (d0 + e < W) ? row[d0 + e] : 0.f;
  }
}

// Keys visible to the decode row at position i.
DEVINL void pd_key_range(const int i, const int window, const int P,
                         int& lo, int& nb, int& n_keys) {
  lo = max(0, i - window + 1);
  nb = max(0, (i - window + 1) / P);
  n_keys = nb + (i - lo + 1);
}

// HD: head width rounded up to 64/128/256. GC: query heads per
// workgroup (the GQA group, or a chunk of it when the group is wider).
template <typename Tag, int HD, int GC>
__global__ __launch_bounds__(PD_BLOCK) void pwa_decode_kernel(
    short* __restrict__ out,               // [T, H, Dv]
    float* __restrict__ tmp_out,           // [rows, H, parts, Dv]
    float* __restrict__ tmp_ml,            // [rows, H, parts, 2]
    const short* __restrict__ q,           // [T, H, D]
    const short* __restrict__ k_cache,     // [blocks, G, bs, D]
    const short* __restrict__ v_cache,     // [blocks, G, bs, Dv]
    const float* __restrict__ pool_k,      // [blocks, G, slots, D]
    const float* __restrict__ pool_v,      // [blocks, G, slots, Dv]
    const int* __restrict__ block_table, const int max_blocks,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const short* __restrict__ gate, const int64_t gate_stride,
    const float scale, const int H, const int G, const int D, const int Dv,
    const int block_size, const int window, const int P, const int slots,
    const int n_parts, const int chunks) {
  constexpr int LPT = HD / 8;              // lanes per key
  constexpr int SLOTS = PD_BLOCK / LPT;    // keys in flight
  __shared__ float m_s[SLOTS][GC];
  __shared__ float l_s[SLOTS][GC];
  __shared__ float acc_s[SLOTS][GC][HD];

  const int r = blockIdx.x;
  const int g = blockIdx.y / chunks;
  const int chunk = blockIdx.y % chunks;
  const int part = blockIdx.z;
  const int group = H / G;
  const int h0 = g * group + chunk * GC;
  const int nh = min(GC, group - chunk * GC);   // heads of this workgroup
  const int t = qsl[r];
  const int i = seq_lens[r] - 1;
  int lo, nb, n_keys;
  pd_key_range(i, window, P, lo, nb, n_keys);
  const int j_begin = part * PD_PART;
  const int j_end = min(n_keys, j_begin + PD_PART);
  if (n_keys <= 0) {
    // Inert row (a padded entry of a captured batch): defined output.
    if (part == 0)
      for (int idx = threadIdx.x; idx < nh * Dv; idx += PD_BLOCK)
        out[((int64_t)t * H + h0 + idx / Dv) * Dv + idx % Dv] = 0;
    return;
  }
  if (j_begin >= j_end) return;

  const int slot = threadIdx.x / LPT;
  const int d0 = (threadIdx.x % LPT) * 8;
  const bool kvec = (D % 8) == 0, vvec = (Dv % 8) == 0;
  const int* bt = block_table + (int64_t)r * max_blocks;

  float qf[GC][8];
#pragma unroll
  for (int c = 0; c < GC; ++c) {
    if (c < nh) {
      load8_16<Tag>(qf[c], q + ((int64_t)t * H + h0 + c) * D, d0, D, kvec);
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[c][e] *= scale;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[c][e] = 0.f;
    }
  }

  float m_run[GC], l_run[GC], acc[GC][8];
#pragma unroll
  for (int c = 0; c < GC; ++c) {
    m_run[c] = PD_NEG;
    l_run[c] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[c][e] = 0.f;
  }

  auto absorb = [&](const float (&kf)[8], const float (&vf)[8]) {
#pragma unroll
    for (int c = 0; c < GC; ++c) {
      float s = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) s += qf[c][e] * kf[e];
#pragma unroll
      for (int off = LPT / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
      const float m_new = fmaxf(m_run[c], s);
      const float f = __expf(m_run[c] - m_new);
      const float p = __expf(s - m_new);
      l_run[c] = l_run[c] * f + p;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[c][e] = acc[c][e] * f + p * vf[e];
      m_run[c] = m_new;
    }
  };

  // Pooled far blocks of this partition.
  const int pooled_end = min(j_end, nb);
  for (int j = j_begin + slot; j < pooled_end; j += SLOTS) {
    const int last = j * P + P - 1;
    const int page = last / block_size;
    const int sl = j - (page * block_size) / P;
    const int64_t base = ((int64_t)bt[page] * G + g) * slots + sl;
    float kf[8], vf[8];
    load8_f32(kf, pool_k + base * D, d0, D, kvec);
    load8_f32(vf, pool_v + base * Dv, d0, Dv, vvec);
    absorb(kf, vf);
  }
  // Window tokens of this partition.
#pragma unroll 2
  for (int j = max(j_begin, nb) + slot; j < j_end; j += SLOTS) {
    const int pos = lo + (j - nb);
    const int64_t base =
        ((int64_t)bt[pos / block_size] * G + g) * block_size +
        pos % block_size;
    float kf[8], vf[8];
    load8_16<Tag>(kf, k_cache + base * D, d0, D, kvec);
    load8_16<Tag>(vf, v_cache + base * Dv, d0, Dv, vvec);
    absorb(kf, vf);
  }

  // Merge the key slots.
#pragma unroll
  for (int c = 0; c < GC; ++c) {
    if (d0 == 0) { m_s[slot][c] = m_run[c]; l_s[slot][c] = l_run[c]; }
#pragma unroll
    for (int e = 0; e < 8; ++e) acc_s[slot][c][d0 + e] = acc[c][e];
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < nh * HD; idx += PD_BLOCK) {
    const int c = idx / HD, d = idx % HD;
    if (d >= Dv) continue;
    float M = PD_NEG;
#pragma unroll 4
    for (int s = 0; s < SLOTS; ++s) M = fmaxf(M, m_s[s][c]);
    float L = 0.f, O = 0.f;
#pragma unroll 4
    for (int s = 0; s < SLOTS; ++s) {
      const float w = __expf(m_s[s][c] - M);
      L += l_s[s][c] * w;
      O += acc_s[s][c][d] * w;
    }
    const int h = h0 + c;
    if (n_parts == 1) {
      float o = O / L;
      if (gate != nullptr) {
        const float z = to_f32<Tag>(gate[(int64_t)t * gate_stride + h]);
        o *= 1.f / (1.f + __expf(-z));
      }
      out[((int64_t)t * H + h) * Dv + d] = from_f32<Tag>(o);
    } else {
      const int64_t pi = ((int64_t)r * H + h) * n_parts + part;
      tmp_out[pi * Dv + d] = O;
      if (d == 0) { tmp_ml[pi * 2] = M; tmp_ml[pi * 2 + 1] = L; }
    }
  }
}

// out = sum_p O_p e^(m_p - M) / sum_p l_p e^(m_p - M), then the gate.
template <typename Tag>
__global__ __launch_bounds__(PD_BLOCK) void pwa_decode_merge_kernel(
    short* __restrict__ out, const float* __restrict__ tmp_out,
    const float* __restrict__ tmp_ml, const int* __restrict__ qsl,
    const int* __restrict__ seq_lens, const short* __restrict__ gate,
    const int64_t gate_stride, const int H, const int Dv, const int window,
    const int P, const int n_parts) {
  const int r = blockIdx.x, h = blockIdx.y;
  const int t = qsl[r];
  int lo, nb, n_keys;
  pd_key_range(seq_lens[r] - 1, window, P, lo, nb, n_keys);
  const int used = min(n_parts, (n_keys + PD_PART - 1) / PD_PART);
  if (used <= 0) return;                 // inert row: zeros already written
  const int64_t p0 = ((int64_t)r * H + h) * n_parts;
  float M = PD_NEG;
  for (int p = 0; p < used; ++p) M = fmaxf(M, tmp_ml[(p0 + p) * 2]);
  float L = 0.f;
  for (int p = 0; p < used; ++p)
    L += tmp_ml[(p0 + p) * 2 + 1] * __expf(tmp_ml[(p0 + p) * 2] - M);
  float gmul = 1.f / L;
  if (gate != nullptr) {
    const float z = to_f32<Tag>(gate[(int64_t)t * gate_stride + h]);
    gmul *= 1.f / (1.f + __expf(-z));
  }
  for (int d = threadIdx.x; d < Dv; d += PD_BLOCK) {
    float O = 0.f;
    for (int p = 0; p < used; ++p)
      O += tmp_out[(p0 + p) * Dv + d] * __expf(tmp_ml[(p0 + p) * 2] - M);
    out[((int64_t)t * H + h) * Dv + d] = from_f32<Tag>(O * gmul);
  }
}

}  // namespace

// Decode rows = the first num_decodes requests of the flat batch, one
// token each. max_seq_len bounds their context lengths (it sizes the
// partition grid; rows with fewer keys leave partitions idle).
void pooled_window_attention_decode(
    torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
    torch::Tensor v_cache, torch::Tensor pool_k, torch::Tensor pool_v,
    torch::Tensor block_table, torch::Tensor query_start_loc,
    torch::Tensor seq_lens, c10::optional<torch::Tensor> gate, double scale,
    int64_t window, int64_t pool, int64_t num_decodes, int64_t max_seq_len) {
  pwa_check_args(out, q, k_cache, v_cache, pool_k, pool_v, block_table,
                 query_start_loc, seq_lens, gate, window, pool);
  TORCH_CHECK(q.scalar_type() == torch::kBFloat16 ||
              q.scalar_type() == torch::kHalf,
              "the decode kernel serves 16-bit dtypes");
  TORCH_CHECK(num_decodes >= 0 && num_decodes <= seq_lens.size(0) &&
              num_decodes <= q.size(0));
  if (num_decodes == 0) return;
  TORCH_CHECK(max_seq_len >= 1);
  const int H = q.size(1), D = q.size(2);
  const int G = k_cache.size(1), bs = k_cache.size(2);
  const int Dv = v_cache.size(3);
  const int group = H / G;
  const int dmax = D > Dv ? D : Dv;
  const int64_t far = max_seq_len - window;
  const int64_t max_keys = std::min<int64_t>(max_seq_len, window) +
                           (far > 0 ? far / pool : 0);
  const int n_parts = (int)((max_keys + PD_PART - 1) / PD_PART);
  const int gc = group >= 4 ? 4 : (group >= 2 ? 2 : 1);
  const int chunks = (group + gc - 1) / gc;
  const int rows = (int)num_decodes;
  torch::Tensor tmp_out, tmp_ml;
  if (n_parts > 1) {
    auto fopt = q.options().dtype(torch::kFloat32);
    tmp_out = torch::empty({rows, H, n_parts, Dv}, fopt);
    tmp_ml = torch::empty({rows, H, n_parts, 2}, fopt);
  }
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid(rows, G * chunks, n_parts);
#define LAUNCH(TAG, HDV, GCV)                                              \
  hipLaunchKernelGGL(                                                      \
      (pwa_decode_kernel<TAG, HDV, GCV>), grid, dim3(PD_BLOCK), 0, stream, \
      (short*)out.data_ptr(),                                              \
      n_parts > 1 ? tmp_out.data_ptr<float>() : nullptr,                   \
      n_parts > 1 ? tmp_ml.data_ptr<float>() : nullptr,                    \
      (const short*)q.data_ptr(), (const short*)k_cache.data_ptr(),        \
      (const short*)v_cache.data_ptr(), pool_k.data_ptr<float>(),          \
      pool_v.data_ptr<float>(), block_table.data_ptr<int>(),               \
      (int)block_table.size(1), query_start_loc.data_ptr<int>(),           \
      seq_lens.data_ptr<int>(),                                            \
      gate.has_value() ? (const short*)gate->data_ptr() : nullptr,         \
      gate.has_value() ? gate->stride(0) : 0, (float)scale, H, G, D, Dv,   \
      bs, (int)window, (int)pool, (int)pool_k.size(2), n_parts, chunks)
#define BY_GC(TAG, HDV)                                                    \
  if (gc == 4) { LAUNCH(TAG, HDV, 4); }                                    \
  else if (gc == 2) { LAUNCH(TAG, HDV, 2); }                               \
  else { LAUNCH(TAG, HDV, 1); }
#define BY_HD(TAG)                                                         \
  if (dmax <= 64) { BY_GC(TAG, 64); }                                      \
  else if (dmax <= 128) { BY_GC(TAG, 128); }                               \
  else { BY_GC(TAG, 256); }
  const bool is_bf16 = q.scalar_type() == torch::kBFloat16;
  if (is_bf16) { BY_HD(BF16Tag); } else { BY_HD(FP16Tag); }
#undef BY_HD
#undef BY_GC
#undef LAUNCH
  HIP_CHECK_KERNEL();
  if (n_parts > 1) {
    dim3 mgrid(rows, H);
#define MERGE(TAG)                                                         \
  hipLaunchKernelGGL(                                                      \
      (pwa_decode_merge_kernel<TAG>), mgrid, dim3(PD_BLOCK), 0, stream,    \
      (short*)out.data_ptr(), tmp_out.data_ptr<float>(),                   \
      tmp_ml.data_ptr<float>(), query_start_loc.data_ptr<int>(),           \
      seq_lens.data_ptr<int>(),                                            \
      gate.has_value() ? (const short*)gate->data_ptr() : nullptr,         \
      gate.has_value() ? gate->stride(0) : 0, H, Dv, (int)window,          \
      (int)pool, n_parts)
    if (is_bf16) { MERGE(BF16Tag); } else { MERGE(FP16Tag); }
#undef MERGE
    HIP_CHECK_KERNEL();
  }
}

}  // namespace vllm_amd
