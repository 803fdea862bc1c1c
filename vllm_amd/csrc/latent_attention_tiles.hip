// MFMA tile kernel for latent attention (gfx950, bf16): every head
// attends ONE shared stream of cached rows [c (LORA) | kr (ROPE)], so a
// tile of 32 (token, head) rows against 32 cached tokens is a pair of
// small GEMMs — S[32 x 32] = Q[32 x DK] K^T and O[32 x LORA] += P V with
// V = the first LORA columns of the same rows — on 16x16x32 bf16 MFMA.
//
// A workgroup (4 waves) owns 32 rows of one request: all heads of
// 32/H consecutive tokens (H <= 32) or 32 heads of one token, and
// walks the keys 0 .. last visible in 32-token subtiles. Each row is
// masked to its own position (causal), so prefill chunks and decode
// rows run the same code; decode batches additionally split the keys
// into 1024-token partitions merged by latent_tile_reduce_kernel.
//   QK : wave (mtile = w&1, ntile = w>>1) computes a 16 x 16 score tile.
//   softmax: online, fp32, log2 domain; per-row max/sum shared through
//            LDS. The running state of partition 0 starts at
//            (m = sink_h, l = 1) when the layer has a sink.
// LORA and ROPE are tile widths; the cached row may be narrower (any
// kv_rank <= LORA and rot_dim <= ROPE in steps of 8), the missing columns
// are zero in LDS and in the query fragments.
//   PV : wave w owns value columns [w*LORA/4, (w+1)*LORA/4).
// The subtile is staged once: [tok][DK] (padded rows, QK reads rows) plus a
// transposed copy of the first LORA columns [col][token pair] (PV reads
// rows), written without LDS bank conflicts.

#include <torch/all.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime.h>

#include "common.h"

namespace vllm_amd {

namespace lat {

constexpr int HG = 32;           // rows per workgroup
constexpr int SUB = 32;          // cached tokens per subtile
constexpr int PART = 1024;       // tokens per decode partition
constexpr int THREADS = 256;
constexpr float NEG_INF = -1e30f;
constexpr float LOG2E = 1.4426950408889634f;
constexpr int VS = 18;           // dwords per column of the transposed V

struct Group {
  int req, t0, nt, h0;   // request, first token, tokens, first head
};

// Which rows this workgroup owns; nt == 0: none.
DEVINL Group find_group(int g, const int* __restrict__ qsl, int req0,
                        int num_reqs, int H, int tpg, int gpt) {
  Group out{0, 0, 0, 0};
  if (gpt > 1) {
    const int t = qsl[req0] + g / gpt;
    if (t >= qsl[req0 + num_reqs]) return out;
    int lo = req0, hi = req0 + num_reqs - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (qsl[mid] <= t) lo = mid; else hi = mid - 1;
    }
    out = Group{lo, t, 1, (g % gpt) * HG};
    return out;
  }
  for (int r = req0; r < req0 + num_reqs; ++r) {
    const int n = qsl[r + 1] - qsl[r];
    const int groups = (n + tpg - 1) / tpg;
    if (g < groups) {
      const int t0 = qsl[r] + g * tpg;
      out = Group{r, t0, min(tpg, qsl[r + 1] - t0), 0};
      return out;
    }
    g -= groups;
  }
  return out;
}

// Reductions over the 16 lanes of a DPP row (rotations by 8, 4, 2, 1):
// every lane ends with the result, no LDS crossbar involved.
template <int CTRL>
DEVINL float dpp_rot(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(
      0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
DEVINL float row16_max(float v) {
  v = fmaxf(v, dpp_rot<0x128>(v));
  v = fmaxf(v, dpp_rot<0x124>(v));
  v = fmaxf(v, dpp_rot<0x122>(v));
  v = fmaxf(v, dpp_rot<0x121>(v));
  return v;
}
DEVINL float row16_add(float v) {
  v += dpp_rot<0x128>(v);
  v += dpp_rot<0x124>(v);
  v += dpp_rot<0x122>(v);
  v += dpp_rot<0x121>(v);
  return v;
}

// MINW = 2 asks for two workgroups per CU (one wave of each per SIMD, at
// most 256 registers per lane): prompt portions launch thousands of
// workgroups and gain from the overlap; decode launches about one per CU
// and is better off with all the registers.
template <int LORA, int ROPE, int MINW>
__launch_bounds__(THREADS, MINW) __global__ void latent_tile_kernel(
    short* __restrict__ out,                          // [T, H, LORA]
    const short* __restrict__ q_abs, const long qa_st, const long qa_sh,
    const short* __restrict__ q_rot, const long qr_st, const long qr_sh,
    const short* __restrict__ kv,                     // [NB, BS, DK]
    const int* __restrict__ block_table, const int bt_stride,
    const int* __restrict__ qsl, const int* __restrict__ seq_lens,
    const float* __restrict__ sink, const float scale, const int H,
    const int block_size, const int req0, const int num_reqs, const int tpg,
    const int gpt,
    const int L, const int R,      // actual widths, multiples of 8
    float* __restrict__ tmp_out,   // [T, H, parts, L]
    float* __restrict__ tmp_lse,   // [T, H, parts, 2]
    const int max_parts) {
  constexpr int DK = LORA + ROPE;
  constexpr int KF = DK / 32;          // MFMA k-steps of the score GEMM
  constexpr int WC = LORA / 4;         // value columns per wave
  constexpr int NF = WC / 16;          // 16-column fragments per wave
  // Rows of the staged tile are padded by 16 B: with a row stride of
  // 36 dwords (mod 64 banks) both the token-pair-major stores of the
  // staging loop and the QK reads (16 rows x 16 B per quarter wave) touch
  // every bank group equally often, the best a 1 KB access can do.
  constexpr int KROW = DK * 2 + 16;   // bytes
  auto kaddr = [](int tok, int byte_off) { return tok * KROW + byte_off; };

  const Group grp = find_group(blockIdx.x, qsl, req0, num_reqs, H, tpg, gpt);
  if (grp.nt == 0) return;
  const int part = blockIdx.y;
  const int ctx = seq_lens[grp.req];
  const int q_end = qsl[grp.req + 1];
  // Keys visible to the group's last token.
  const int vis_end = ctx - (q_end - (grp.t0 + grp.nt - 1)) + 1;
  const int t_begin = part * PART;
  if (t_begin >= vis_end) return;
  // A launch without partitions (prompt portions) walks all its keys.
  const bool single = gridDim.y == 1;
  const int t_end = single ? vis_end : min(t_begin + PART, vis_end);

  __shared__ short k_lds[SUB * KROW / 2];  // [tok][DK], 16 B slots
  __shared__ uint32_t vt_lds[LORA * VS];  // [col][token pair]
  __shared__ short p_lds[HG * SUB];       // [row][tok] bf16
  __shared__ float m_st[HG], l_st[HG], f_st[HG];
  __shared__ float wmax[2][HG], wsum[2][HG];
  __shared__ int row_tok[HG], row_head[HG], row_lim[HG];

  const int tid = threadIdx.x;
  const int wave = tid / WAVE_SIZE;
  const int lane = tid % WAVE_SIZE;
  const int l16 = lane & 15;
  const int l4 = lane >> 4;
  const int mtile = wave & 1;
  const int ntile = wave >> 1;

  if (tid < HG) {
    int tok, head;
    bool ok;
    if (gpt > 1) {
      tok = grp.t0;
      head = grp.h0 + tid;
      ok = head < H;
    } else {
      tok = grp.t0 + tid / H;
      head = tid % H;
      ok = tid / H < grp.nt;
    }
    row_tok[tid] = ok ? tok : -1;
    row_head[tid] = ok ? head : 0;
    // Visible keys of this row: its position + 1 (0 = padding row).
    row_lim[tid] = ok ? ctx - (q_end - tok) + 1 : 0;
    const bool sk = ok && sink != nullptr && part == 0;
    m_st[tid] = sk ? sink[head] * LOG2E : NEG_INF;
    l_st[tid] = sk ? 1.f : 0.f;
  }
  __syncthreads();

  // Running max per owned row, kept redundantly in registers by the
  // two waves that share an mtile (identical updates from LDS).
  float m_reg[4];
  int lim[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    m_reg[r] = m_st[mtile * 16 + l4 * 4 + r];
    lim[r] = row_lim[mtile * 16 + l4 * 4 + r];
  }

  // Q fragments: this wave's A rows are rows mtile*16 + l16.
  s16x8 qfrag[KF];
  {
    const int qr = mtile * 16 + l16;
    const int qt = row_tok[qr], qh = row_head[qr];
#pragma unroll
    for (int kf = 0; kf < KF; ++kf) {
      const int f = kf * 32 + l4 * 8;
      s16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      // Columns [L, LORA) and [LORA + R, DK) of the tile are zero.
      if (qt >= 0 && f < L)
        v = *reinterpret_cast<const s16x8*>(q_abs + qt * qa_st +
                                            qh * qa_sh + f);
      else if (qt >= 0 && f >= LORA && f - LORA < R)
        v = *reinterpret_cast<const s16x8*>(q_rot + qt * qr_st +
                                            qh * qr_sh + (f - LORA));
      qfrag[kf] = v;
    }
  }

  f32x4 o_acc[2][NF];
#pragma unroll
  for (int mt = 0; mt < 2; ++mt)
#pragma unroll
    for (int nf = 0; nf < NF; ++nf) o_acc[mt][nf] = f32x4{0.f, 0.f, 0.f, 0.f};

  const float sc2 = scale * LOG2E;
  const int* bt = block_table + (long)grp.req * bt_stride;

  // Staging: a thread takes one 16 B column chunk of a PAIR of adjacent
  // tokens. The pair's values go into the transposed copy as one dword
  // per column; with token pairs fastest across lanes and a column
  // stride of VS = 18 dwords a wave's 64 stores fall on 64 different
  // banks. The global loads of the NEXT subtile are issued before the
  // current one is computed, so their latency hides behind the MFMAs.
  constexpr int ITEMS = (SUB / 2) * (DK / 8);
  constexpr int NIT = (ITEMS + THREADS - 1) / THREADS;
  s16x8 pre0[NIT], pre1[NIT];
  const bool bs_pow2 = (block_size & (block_size - 1)) == 0;
  const int bs_shift = 31 - __builtin_clz(block_size);
  auto row_of = [&](int t) -> long {
    const int page = bs_pow2 ? (t >> bs_shift) : t / block_size;
    const int off = bs_pow2 ? (t & (block_size - 1)) : t % block_size;
    return ((long)bt[page] * block_size + off) * (L + R);
  };
  // Tile column chunk f8 -> offset in a cached row, or -1 (zero fill).
  auto src_col = [&](int f8) -> int {
    const int col = f8 * 8;
    if (col < LORA) return col < L ? col : -1;
    return col - LORA < R ? L + (col - LORA) : -1;
  };
  auto fetch = [&](int sub0) {
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = tid + it * THREADS;
      const int tp = c % (SUB / 2);
      const int f8 = c / (SUB / 2);
      const int t_glob = sub0 + 2 * tp;
      pre0[it] = s16x8{0, 0, 0, 0, 0, 0, 0, 0};
      pre1[it] = s16x8{0, 0, 0, 0, 0, 0, 0, 0};
      const int sc = c < ITEMS ? src_col(f8) : -1;
      if (sc >= 0 && t_glob < t_end)
        pre0[it] = *reinterpret_cast<const s16x8*>(kv + row_of(t_glob) +
                                                   sc);
      if (sc >= 0 && t_glob + 1 < t_end)
        pre1[it] = *reinterpret_cast<const s16x8*>(
            kv + row_of(t_glob + 1) + sc);
    }
  };
  fetch(t_begin);

  for (int sub0 = t_begin; sub0 < t_end; sub0 += SUB) {
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const int c = tid + it * THREADS;
      if (c >= ITEMS) continue;
      const int tp = c % (SUB / 2);
      const int f8 = c / (SUB / 2);
      *reinterpret_cast<s16x8*>(reinterpret_cast<char*>(k_lds) +
                                kaddr(2 * tp, f8 * 16)) = pre0[it];
      *reinterpret_cast<s16x8*>(reinterpret_cast<char*>(k_lds) +
                                kaddr(2 * tp + 1, f8 * 16)) = pre1[it];
      if (f8 * 8 < LORA) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          vt_lds[(f8 * 8 + j) * VS + tp] =
              (uint32_t)(uint16_t)pre0[it][j] |
              ((uint32_t)(uint16_t)pre1[it][j] << 16);
      }
    }
    __syncthreads();
    if (sub0 + SUB < t_end) fetch(sub0 + SUB);

    // ---- QK: S[16 rows x 16 tokens] for (mtile, ntile).
    f32x4 s_frag = {0.f, 0.f, 0.f, 0.f};
    {
      const int tok = ntile * 16 + l16;
#pragma unroll
      for (int kf = 0; kf < KF; ++kf) {
        s16x8 bfrag = *reinterpret_cast<const s16x8*>(
            reinterpret_cast<const char*>(k_lds) +
            kaddr(tok, kf * 64 + l4 * 16));
        s_frag = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qfrag[kf], bfrag,
                                                         s_frag, 0, 0, 0);
      }
    }
    // C fragment: column = lane&15 = token, row = l4*4 + r.
    const int tok_g = sub0 + ntile * 16 + l16;
    float s_val[4], rowmax[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s_val[r] = tok_g < min(t_end, lim[r]) ? s_frag[r] * sc2 : NEG_INF;
      rowmax[r] = row16_max(s_val[r]);
    }
    if (l16 == 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        wmax[ntile][mtile * 16 + l4 * 4 + r] = rowmax[r];
    }
    __syncthreads();

    // ---- softmax update.
    float factor[4], m_new[4], rowsum[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = mtile * 16 + l4 * 4 + r;
      const float mo = m_reg[r];
      m_new[r] = fmaxf(mo, fmaxf(wmax[0][row], wmax[1][row]));
      factor[r] = exp2f(mo - m_new[r]);
      m_reg[r] = m_new[r];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float p =
          tok_g < min(t_end, lim[r]) ? exp2f(s_val[r] - m_new[r]) : 0.f;
      p_lds[(mtile * 16 + l4 * 4 + r) * SUB + ntile * 16 + l16] =
          f32_to_bf16(p);
      rowsum[r] = row16_add(p);
    }
    if (l16 == 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int row = mtile * 16 + l4 * 4 + r;
        wsum[ntile][row] = rowsum[r];
        if (ntile == 0) {
          m_st[row] = m_new[r];
          f_st[row] = factor[r];
        }
      }
    }
    __syncthreads();

    // ---- PV.
#pragma unroll
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int nf = 0; nf < NF; ++nf) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          o_acc[mt][nf][r] *= f_st[mt * 16 + l4 * 4 + r];
      }
      const int arow = mt * 16 + l16;
      s16x8 afrag =
          *reinterpret_cast<const s16x8*>(p_lds + arow * SUB + l4 * 8);
#pragma unroll
      for (int nf = 0; nf < NF; ++nf) {
        const int col = wave * WC + nf * 16 + l16;
        // 8 tokens = 4 dwords; columns are 8 B aligned (VS is even).
        const uint32_t* vp = vt_lds + col * VS + l4 * 4;
        const uint2 lo = *reinterpret_cast<const uint2*>(vp);
        const uint2 hi = *reinterpret_cast<const uint2*>(vp + 2);
        union { uint32_t u[4]; s16x8 v; } pk;
        pk.u[0] = lo.x; pk.u[1] = lo.y; pk.u[2] = hi.x; pk.u[3] = hi.y;
        s16x8 bfrag = pk.v;
        o_acc[mt][nf] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
            afrag, bfrag, o_acc[mt][nf], 0, 0, 0);
      }
    }
    if (wave == 0 && tid < HG)
      l_st[tid] = l_st[tid] * f_st[tid] + wsum[0][tid] + wsum[1][tid];
    __syncthreads();
  }

  // ---- write out: rows mt*16 + l4*4 + r, columns wave*WC + nf*16 + l16.
#pragma unroll
  for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int row = mt * 16 + l4 * 4 + r;
      const int t = row_tok[row];
      if (t < 0) continue;
      const long oh = (long)t * H + row_head[row];
      const float l = l_st[row];
#pragma unroll
      for (int nf = 0; nf < NF; ++nf) {
        const int col = wave * WC + nf * 16 + l16;
        if (col >= L) continue;
        if (single)
          out[oh * L + col] = f32_to_bf16(o_acc[mt][nf][r] / l);
        else
          tmp_out[(oh * max_parts + part) * L + col] = o_acc[mt][nf][r];
      }
    }
  }
  if (!single && tid < HG && row_tok[tid] >= 0) {
    const long base =
        (((long)row_tok[tid] * H + row_head[tid]) * max_parts + part) * 2;
    tmp_lse[base] = m_st[tid];       // log2-domain max
    tmp_lse[base + 1] = l_st[tid];   // sum (with the sink in partition 0)
  }
}

// out[t,h,:] = sum_p w_p tmp[t,h,p,:] / sum_p w_p l_p, w_p = 2^(m_p - max).
// Decode rows only (token index == request index). Grid (T, H).
__global__ void latent_tile_reduce_kernel(
    short* __restrict__ out, const float* __restrict__ tmp_out,
    const float* __restrict__ tmp_lse, const int* __restrict__ seq_lens,
    const int H, const int max_parts, const int LORA) {
  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int parts = min((seq_lens[t] + PART - 1) / PART, max_parts);
  const long lse_base = (((long)t * H + h) * max_parts) * 2;
  float m = NEG_INF;
  for (int p = 0; p < parts; ++p) m = fmaxf(m, tmp_lse[lse_base + p * 2]);
  float l = 0.f;
  for (int p = 0; p < parts; ++p)
    l += exp2f(tmp_lse[lse_base + p * 2] - m) * tmp_lse[lse_base + p * 2 + 1];
  const float inv_l = 1.f / l;
  const long o_base = ((long)t * H + h) * (long)max_parts * LORA;
  for (int c = threadIdx.x; c < LORA; c += blockDim.x) {
    float acc = 0.f;
    for (int p = 0; p < parts; ++p)
      acc += exp2f(tmp_lse[lse_base + p * 2] - m) *
             tmp_out[o_base + (long)p * LORA + c];
    out[((long)t * H + h) * LORA + c] = f32_to_bf16(acc * inv_l);
  }
}

}  // namespace lat

void latent_check_args(const torch::Tensor& out, const torch::Tensor& q_abs,
                       const torch::Tensor& q_rot,
                       const torch::Tensor& cache,
                       const torch::Tensor& block_table,
                       const torch::Tensor& query_start_loc,
                       const torch::Tensor& seq_lens,
                       const c10::optional<torch::Tensor>& sink);

// Any widths in 16 B steps up to the largest tile: the kernel is built
// for tile widths {64, 128, 256, 512} x {32, 64} and zero-fills the
// columns a narrower row does not have.
bool latent_attention_tiles_supported(int64_t kv_rank, int64_t rot_dim) {
  return kv_rank >= 8 && kv_rank <= 512 && kv_rank % 8 == 0 &&
         rot_dim >= 0 && rot_dim <= 64 && rot_dim % 8 == 0;
}

void latent_attention_tiles(torch::Tensor out, torch::Tensor q_abs,
                            torch::Tensor q_rot, torch::Tensor cache,
                            torch::Tensor block_table,
                            torch::Tensor query_start_loc,
                            torch::Tensor seq_lens,
                            c10::optional<torch::Tensor> sink, double scale,
                            int64_t num_decodes, int64_t max_seq_len) {
  using namespace lat;
  latent_check_args(out, q_abs, q_rot, cache, block_table, query_start_loc,
                    seq_lens, sink);
  TORCH_CHECK(q_abs.scalar_type() == torch::kBFloat16,
              "latent_attention_tiles: bf16 only");
  const int T = q_abs.size(0), H = q_abs.size(1), L = q_abs.size(2);
  const int R = q_rot.size(2);
  TORCH_CHECK(latent_attention_tiles_supported(L, R),
              "latent_attention_tiles: unsupported (kv_rank, rot_dim)");
  // 16 B fragment loads.
  TORCH_CHECK(q_abs.stride(0) % 8 == 0 && q_abs.stride(1) % 8 == 0 &&
              q_abs.storage_offset() % 8 == 0 &&
              (R == 0 || (q_rot.stride(0) % 8 == 0 &&
                          q_rot.stride(1) % 8 == 0 &&
                          q_rot.storage_offset() % 8 == 0)),
              "latent_attention_tiles: queries must be 16 B aligned");
  const int num_reqs = seq_lens.numel();
  TORCH_CHECK(num_decodes >= 0 && num_decodes <= num_reqs &&
              num_decodes <= T);
  if (T == 0) return;
  const int tpg = H <= HG ? HG / H : 1;
  const int gpt = H <= HG ? 1 : (H + HG - 1) / HG;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const int n_dec = (int)num_decodes;
  int parts = 1;
  torch::Tensor tmp_out, tmp_lse;
  if (n_dec > 0) {
    parts = std::max<int>(1, (int)((max_seq_len + PART - 1) / PART));
    if (parts > 1) {
      auto f32 = q_abs.options().dtype(torch::kFloat32);
      tmp_out = torch::empty({(int64_t)n_dec * H * parts * L}, f32);
      tmp_lse = torch::empty({(int64_t)n_dec * H * parts * 2}, f32);
    }
  }
  auto launch = [&](auto lora, auto rope) {
    constexpr int LO = decltype(lora)::value;
    constexpr int RO = decltype(rope)::value;
    auto run = [&](int req0, int nreq, int tokens, int nparts, auto minw) {
      constexpr int MW = decltype(minw)::value;
      const int gx = gpt > 1 ? tokens * gpt
                             : (tokens + tpg - 1) / tpg + nreq;
      hipLaunchKernelGGL(
          (latent_tile_kernel<LO, RO, MW>), dim3(gx, nparts), dim3(THREADS), 0,
          stream, (short*)out.data_ptr(), (const short*)q_abs.data_ptr(),
          (long)q_abs.stride(0), (long)q_abs.stride(1),
          (const short*)q_rot.data_ptr(), (long)q_rot.stride(0),
          (long)q_rot.stride(1), (const short*)cache.data_ptr(),
          block_table.data_ptr<int>(), (int)block_table.stride(0),
          query_start_loc.data_ptr<int>(), seq_lens.data_ptr<int>(),
          sink.has_value() ? sink->data_ptr<float>() : nullptr,
          (float)scale, H, (int)cache.size(1), req0, nreq, tpg, gpt, L, R,
          nparts > 1 ? tmp_out.data_ptr<float>() : nullptr,
          nparts > 1 ? tmp_lse.data_ptr<float>() : nullptr, nparts);
    };
    if (n_dec > 0) {
      run(0, n_dec, n_dec, parts, std::integral_constant<int, 1>{});
      if (parts > 1)
        hipLaunchKernelGGL(latent_tile_reduce_kernel, dim3(n_dec, H),
                           dim3(256), 0, stream, (short*)out.data_ptr(),
                           tmp_out.data_ptr<float>(),
                           tmp_lse.data_ptr<float>(),
                           seq_lens.data_ptr<int>(), H, parts, L);
    }
    if (num_reqs > n_dec && T > n_dec)
      run(n_dec, num_reqs - n_dec, T - n_dec, 1,
          std::integral_constant<int, 2>{});
  };
  using std::integral_constant;
  auto with_rope = [&](auto lora) {
    if (R <= 32)
      launch(lora, integral_constant<int, 32>{});
    else
      launch(lora, integral_constant<int, 64>{});
  };
  if (L <= 64)
    with_rope(integral_constant<int, 64>{});
  else if (L <= 128)
    with_rope(integral_constant<int, 128>{});
  else if (L <= 256)
    with_rope(integral_constant<int, 256>{});
  else
    with_rope(integral_constant<int, 512>{});
  HIP_CHECK_KERNEL();
}

}  // namespace vllm_amd
