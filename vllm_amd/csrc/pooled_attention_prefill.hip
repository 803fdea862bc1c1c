// MFMA prefill kernel for sliding-window attention with mean-pooled far
// blocks (gfx950, bf16). Companion of pooled_attention.hip, which holds
// the row-wise kernel used for decode rows, fp16 and fp32.
//
// One workgroup = 64 consecutive query rows of one (request, head); 4
// waves x 16 rows. Key tiles of 64 are walked in two phases that share
// ONE online softmax:
//   1. pooled tiles: entries b = 64*t .. of the request's pooled blocks
//      (fp32 means, gathered through the block table, rounded to bf16
//      for the matrix product); entry b is visible to position i iff
//      b < (i - window + 1) / pool.
//   2. token tiles: cache pages from the first page the tile's window
//      touches to the page of its last row; key j visible iff
//      i - window < j <= i.
// K is staged row-major [64][DP] and V transposed [DP][64] in LDS, both
// zero-padded from the real head widths (any D, Dv <= DP) and
// XOR-swizzled as in attention_prefill.hip. S = Q K^T and O^T = V^T P^T
// run on 16x16x32 bf16 MFMA with fp32 accumulation; scores, softmax
// statistics and the sigmoid output gate are fp32.

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

constexpr int PP_BLOCK = 256;
constexpr int PP_QTILE = 64;
constexpr int PP_KTILE = 64;
constexpr float PP_LOG2E = 1.4426950408889634f;

DEVINL int pp_swz(int row, int col_byte) {
  return col_byte ^ ((row & 7) << 4);
}

template <int DP>
__global__ __launch_bounds__(PP_BLOCK) void pwa_prefill_kernel(
    short* __restrict__ out,               // [T, H, Dv]
    const short* __restrict__ q,           // [T, H, D]
    const short* __restrict__ k_cache,     // [blocks, G, 64, D]
    const short* __restrict__ v_cache,     // [blocks, G, 64, Dv]
    const float* __restrict__ pool_k,      // [blocks, G, slots, D]
    const float* __restrict__ pool_v,      // [blocks, G, slots, Dv]
    const int* __restrict__ block_table, const int max_blocks,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const short* __restrict__ gate, const int64_t gate_stride,
    const float scale, const int num_decodes, const int H, const int G,
    const int D, const int Dv, const int window, const int P,
    const int slots) {
  const int req = num_decodes + blockIdx.z;
  const int h = blockIdx.y;
  const int g = h / (H / G);
  const int q_start = qsl[req];
  const int ql = qsl[req + 1] - q_start;
  const int qtile0 = blockIdx.x * PP_QTILE;
  if (qtile0 >= ql) return;
  const int ctx = seq_lens[req];
  const int* bt = block_table + (int64_t)req * max_blocks;

  const int wave = threadIdx.x / WAVE_SIZE;
  const int lane = threadIdx.x % WAVE_SIZE;
  const int l16 = lane & 15;
  const int l4 = lane >> 4;

  __shared__ short k_lds[PP_KTILE * DP];     // [key][d], swizzled
  __shared__ short vt_lds[DP * PP_KTILE];    // [d][key], swizzled
  __shared__ short p_lds[4][16 * 80];
  __shared__ float f_lds[4][16];

  // Q A-fragments, zero beyond D.
  const int q_row_safe = min(qtile0 + wave * 16 + l16, ql - 1);
  s16x8 qfrag[DP / 32];
  {
    const short* qbase = q + ((int64_t)(q_start + q_row_safe) * H + h) * D;
#pragma unroll
    for (int kk = 0; kk < DP / 32; ++kk) {
      const int d0 = kk * 32 + l4 * 8;
      s16x8 f;
#pragma unroll
      for (int j = 0; j < 8; ++j) f[j] = (d0 + j < D) ? qbase[d0 + j] : 0;
      qfrag[kk] = f;
    }
  }

  float m_st[4], l_st[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) { m_st[r] = -3.0e38f; l_st[r] = 0.f; }
  f32x4 o_acc[DP / 16];
#pragma unroll
  for (int i = 0; i < DP / 16; ++i) o_acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};

  const float scale_log2e = scale * PP_LOG2E;
  const int pos0 = ctx - ql;                       // position of q row 0
  const int rows_here = min(PP_QTILE, ql - qtile0);
  const int pos_first = pos0 + qtile0;
  const int pos_last = pos_first + rows_here - 1;
  const int nb_max = max(0, (pos_last - window + 1) / P);
  const int pooled_tiles = (nb_max + PP_KTILE - 1) / PP_KTILE;
  const int page_first = max(0, pos_first - window + 1) / PP_KTILE;
  const int page_last = pos_last / PP_KTILE;
  const int n_tiles = pooled_tiles + (page_last - page_first + 1);

  for (int it = 0; it < n_tiles; ++it) {
    const bool pooled = it < pooled_tiles;
    const int page = page_first + (it - pooled_tiles);
    // ---- stage K [64][DP] and V^T [DP][64], zero-padded --------------
    if (pooled) {
      for (int idx = threadIdx.x; idx < PP_KTILE * (DP / 8);
           idx += PP_BLOCK) {
        const int row = idx / (DP / 8);
        const int d0 = (idx % (DP / 8)) * 8;
        const int b = it * PP_KTILE + row;
        s16x8 kv8, vv8;
#pragma unroll
        for (int j = 0; j < 8; ++j) { kv8[j] = 0; vv8[j] = 0; }
        if (b < nb_max) {
          const int last = b * P + P - 1;
          const int pg = last / PP_KTILE;
          const int slot = b - (pg * PP_KTILE) / P;
          const int64_t base = ((int64_t)bt[pg] * G + g) * slots + slot;
          const float* kp = pool_k + base * D;
          const float* vp = pool_v + base * Dv;
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            if (d0 + j < D) kv8[j] = f32_to_bf16(kp[d0 + j]);
            if (d0 + j < Dv) vv8[j] = f32_to_bf16(vp[d0 + j]);
          }
        }
        *reinterpret_cast<s16x8*>(reinterpret_cast<char*>(k_lds) +
                                  row * (DP * 2) + pp_swz(row, d0 * 2)) = kv8;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int d = d0 + j;
          *reinterpret_cast<short*>(reinterpret_cast<char*>(vt_lds) +
                                    d * 128 + pp_swz(d, row * 2)) = vv8[j];
        }
      }
    } else {
      const int64_t pb = ((int64_t)bt[page] * G + g) * PP_KTILE;
      const short* ksrc = k_cache + pb * D;
      const short* vsrc = v_cache + pb * Dv;
      const bool kvec = (D % 8) == 0, vvec = (Dv % 8) == 0;
      for (int idx = threadIdx.x; idx < PP_KTILE * (DP / 8);
           idx += PP_BLOCK) {
        const int row = idx / (DP / 8);
        const int d0 = (idx % (DP / 8)) * 8;
        s16x8 kv8, vv8;
#pragma unroll
        for (int j = 0; j < 8; ++j) { kv8[j] = 0; vv8[j] = 0; }
        if (d0 < D) {
          if (kvec) {
            kv8 = *reinterpret_cast<const s16x8*>(ksrc + row * D + d0);
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (d0 + j < D) kv8[j] = ksrc[row * D + d0 + j];
          }
        }
        if (d0 < Dv) {
          if (vvec) {
            vv8 = *reinterpret_cast<const s16x8*>(vsrc + row * Dv + d0);
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (d0 + j < Dv) vv8[j] = vsrc[row * Dv + d0 + j];
          }
        }
        *reinterpret_cast<s16x8*>(reinterpret_cast<char*>(k_lds) +
                                  row * (DP * 2) + pp_swz(row, d0 * 2)) = kv8;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int d = d0 + j;
          *reinterpret_cast<short*>(reinterpret_cast<char*>(vt_lds) +
                                    d * 128 + pp_swz(d, row * 2)) = vv8[j];
        }
      }
    }
    __syncthreads();

    // ---- S = Q K^T ----------------------------------------------------
    f32x4 s_frag[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) s_frag[n] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const int key = n * 16 + l16;
#pragma unroll
      for (int kk = 0; kk < DP / 32; ++kk) {
        const int cb = (kk * 32 + l4 * 8) * 2;
        s16x8 bfrag = *reinterpret_cast<const s16x8*>(
            reinterpret_cast<const char*>(k_lds) + key * (DP * 2) +
            pp_swz(key, cb));
        s_frag[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            qfrag[kk], bfrag, s_frag[n], 0, 0, 0);
      }
    }

    // ---- mask + online softmax (exp2 domain) --------------------------
    float p[4][4];
    float rmax[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) rmax[r] = -3.0e38f;
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      const int kidx = n * 16 + l16;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int qrow = qtile0 + wave * 16 + l4 * 4 + r;
        const int qpos = pos0 + qrow;
        bool visible;
        if (pooled) {
          const int b = it * PP_KTILE + kidx;
          visible = b < (qpos - window + 1) / P && qpos - window + 1 > 0;
        } else {
          const int kpos = page * PP_KTILE + kidx;
          visible = kpos <= qpos && kpos > qpos - window;
        }
        visible = visible && qrow < ql;
        p[n][r] = visible ? s_frag[n][r] * scale_log2e : -3.0e38f;
        rmax[r] = fmaxf(rmax[r], p[n][r]);
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      rmax[r] = group16_reduce_max(rmax[r]);
      const float m_new = fmaxf(m_st[r], rmax[r]);
      const float factor = exp2f(m_st[r] - m_new);
      l_st[r] *= factor;
      m_st[r] = m_new;
      if (l16 == 0) f_lds[wave][l4 * 4 + r] = factor;
    }
    float rsum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        // A row that has seen no visible key yet keeps m = -3e38 and
        // would turn masked entries into exp2(0); give them weight 0.
        const float pv =
            p[n][r] <= -1.0e38f ? 0.f : exp2f(p[n][r] - m_st[r]);
        rsum[r] += pv;
        p_lds[wave][(l4 * 4 + r) * 80 + n * 16 + l16] = f32_to_bf16(pv);
      }
#pragma unroll
    for (int r = 0; r < 4; ++r) l_st[r] += group16_reduce_sum(rsum[r]);

    __syncthreads();

    // ---- O^T += V^T P^T -------------------------------------------------
    const float fac = f_lds[wave][l16];
#pragma unroll
    for (int i = 0; i < DP / 16; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) o_acc[i][r] *= fac;
#pragma unroll
    for (int kc = 0; kc < 2; ++kc) {
      const int tb = (kc * 32 + l4 * 8) * 2;
      s16x8 pfrag = *reinterpret_cast<const s16x8*>(
          &p_lds[wave][l16 * 80] + (kc * 32 + l4 * 8));
#pragma unroll
      for (int msub = 0; msub < DP / 16; ++msub) {
        const int d = msub * 16 + l16;
        s16x8 afrag = *reinterpret_cast<const s16x8*>(
            reinterpret_cast<const char*>(vt_lds) + d * 128 +
            pp_swz(d, tb));
        o_acc[msub] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            afrag, pfrag, o_acc[msub], 0, 0, 0);
      }
    }
    __syncthreads();
  }

  // ---- epilogue ---------------------------------------------------------
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (l16 == 0) f_lds[wave][l4 * 4 + r] = l_st[r];
  __syncthreads();
  const int qrow_o = qtile0 + wave * 16 + l16;
  if (qrow_o < ql) {
    const float l = f_lds[wave][l16];
    float w = l > 0.f ? 1.f / l : 0.f;
    const int64_t t = q_start + qrow_o;
    if (gate != nullptr) {
      const float z = bf16_to_f32(gate[t * gate_stride + h]);
      w *= 1.f / (1.f + expf(-z));
    }
    short* obase = out + (t * H + h) * Dv;
#pragma unroll
    for (int msub = 0; msub < DP / 16; ++msub)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int d = msub * 16 + l4 * 4 + r;
        if (d < Dv) obase[d] = f32_to_bf16(o_acc[msub][r] * w);
      }
  }
}

}  // namespace

// Prefill requests (those after the first num_decodes) of the flat
// batch; bf16 only, head widths up to 256.
void pooled_window_attention_prefill(
    torch::Tensor out, torch::Tensor q, torch::Tensor k_cache,
    torch::Tensor v_cache, torch::Tensor pool_k, torch::Tensor pool_v,
    torch::Tensor block_table, torch::Tensor query_start_loc,
    torch::Tensor seq_lens, c10::optional<torch::Tensor> gate, double scale,
    int64_t window, int64_t pool, int64_t num_decodes,
    int64_t max_query_len) {
  pwa_check_args(out, q, k_cache, v_cache, pool_k, pool_v, block_table,
                 query_start_loc, seq_lens, gate, window, pool);
  TORCH_CHECK(q.scalar_type() == torch::kBFloat16,
              "the MFMA prefill kernel is bf16 only");
  TORCH_CHECK(k_cache.size(2) == PP_KTILE, "cache block_size must be 64");
  const int num_reqs = seq_lens.size(0);
  const int num_prefills = num_reqs - (int)num_decodes;
  TORCH_CHECK(num_decodes >= 0 && num_prefills >= 0);
  if (num_prefills == 0 || max_query_len <= 0) return;
  const int H = q.size(1), D = q.size(2);
  const int G = k_cache.size(1), Dv = v_cache.size(3);
  const int dmax = D > Dv ? D : Dv;
  const int tiles = (int)((max_query_len + PP_QTILE - 1) / PP_QTILE);
  auto stream = c10::hip::getCurrentHIPStream().stream();
  dim3 grid(tiles, H, num_prefills);
#define LAUNCH(DPV)                                                        \
  hipLaunchKernelGGL(                                                      \
      (pwa_prefill_kernel<DPV>), grid, dim3(PP_BLOCK), 0, stream,          \
      (short*)out.data_ptr(), (const short*)q.data_ptr(),                  \
      (const short*)k_cache.data_ptr(), (const short*)v_cache.data_ptr(),  \
      pool_k.data_ptr<float>(), pool_v.data_ptr<float>(),                  \
      block_table.data_ptr<int>(), (int)block_table.size(1),               \
      query_start_loc.data_ptr<int>(), seq_lens.data_ptr<int>(),           \
      gate.has_value() ? (const short*)gate->data_ptr() : nullptr,         \
      gate.has_value() ? gate->stride(0) : 0, (float)scale,                \
      (int)num_decodes, H, G, D, Dv, (int)window, (int)pool,               \
      (int)pool_k.size(2))
  if (dmax <= 64) { LAUNCH(64); }
  else if (dmax <= 128) { LAUNCH(128); }
  else { LAUNCH(256); }
#undef LAUNCH
  HIP_CHECK_KERNEL();
}

}  // namespace vllm_amd
