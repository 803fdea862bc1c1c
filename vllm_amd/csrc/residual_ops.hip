// Elementwise kernels for decoder stacks that keep an fp32 residual
// stream and put WEIGHTED RMS norms on sublayer outputs (gfx950).
//
//   scaled_embedding   out[t] = table[id[t]] * scale            (fp32)
//   rms_norm_cast      x / sqrt(mean(x^2)+eps) * w, any in/out dtype
//   add_rms_norm       res += norm(y) * w   [+ cast copy of res]
//   relu2              max(x, 0)^2
//   logit_softcap      cap * tanh(x / cap)                      (fp32)
//   sigmoid_gate_mul   out[t, h*D+d] = x[t, h, d] * sigmoid(gate[t, .])
//                      with x given by strides (a transposed batched
//                      GEMM result is read in place)
//
// Norm statistics, the residual sum and the gates are fp32 whatever the
// tensors' dtype.

#include <torch/all.h>
#include <c10/hip/HIPStream.h>

#include "common.h"
#include "pooled_attention.h"

namespace vllm_amd {

namespace {

constexpr int RB = 256;
constexpr int RV = 4;   // 16 B chunks per thread in the vector kernels

DEVINL float rblock_sum(float v, float* scratch) {
  v = wave_reduce_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  return scratch[0] + scratch[1] + scratch[2] + scratch[3];
}

template <typename T>
DEVINL f32x4 rld4(const typename ET<T>::t* __restrict__ p) {
  if constexpr (sizeof(typename ET<T>::t) == 4) {
    return *reinterpret_cast<const f32x4*>(p);
  } else {
    const s16x4 v = *reinterpret_cast<const s16x4*>(p);
    return f32x4{ET<T>::ld(v[0]), ET<T>::ld(v[1]), ET<T>::ld(v[2]),
                 ET<T>::ld(v[3])};
  }
}

template <typename T>
DEVINL void rst4(typename ET<T>::t* __restrict__ p, const f32x4 v) {
  if constexpr (sizeof(typename ET<T>::t) == 4) {
    *reinterpret_cast<f32x4*>(p) = v;
  } else {
    *reinterpret_cast<s16x4*>(p) =
        s16x4{ET<T>::st(v[0]), ET<T>::st(v[1]), ET<T>::st(v[2]),
              ET<T>::st(v[3])};
  }
}

template <typename T>
__global__ __launch_bounds__(RB) void scaled_embedding_kernel(
    float* __restrict__ out, const int64_t* __restrict__ ids,
    const typename ET<T>::t* __restrict__ table, const float scale,
    const int width) {
  const int64_t t = blockIdx.x;
  const typename ET<T>::t* row = table + ids[t] * (int64_t)width;
  for (int c = threadIdx.x; c < width; c += RB)
    out[t * width + c] = ET<T>::ld(row[c]) * scale;
}

// VEC: width % 4 == 0 and width <= 4 * RB * RV; rows stay in registers
// between the sum of squares and the output pass.
template <typename TI, typename TO, bool VEC>
__global__ __launch_bounds__(RB) void rms_norm_cast_kernel(
    typename ET<TO>::t* __restrict__ out,
    const typename ET<TI>::t* __restrict__ x, const float* __restrict__ w,
    const float eps, const int width) {
  __shared__ float scratch[4];
  const int64_t row = blockIdx.x;
  const typename ET<TI>::t* xr = x + row * width;
  if constexpr (VEC) {
    f32x4 xv[RV];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < RV; ++k) {
      const int c = (k * RB + threadIdx.x) * 4;
      xv[k] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (c < width) xv[k] = rld4<TI>(xr + c);
      ss += xv[k][0] * xv[k][0] + xv[k][1] * xv[k][1] +
            xv[k][2] * xv[k][2] + xv[k][3] * xv[k][3];
    }
    ss = rblock_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)width + eps);
#pragma unroll
    for (int k = 0; k < RV; ++k) {
      const int c = (k * RB + threadIdx.x) * 4;
      if (c >= width) continue;
      const f32x4 wv = *reinterpret_cast<const f32x4*>(w + c);
      f32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = xv[k][e] * inv * wv[e];
      rst4<TO>(out + row * width + c, o);
    }
  } else {
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += RB) {
      const float v = ET<TI>::ld(xr[c]);
      ss += v * v;
    }
    ss = rblock_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += RB)
      out[row * width + c] = ET<TO>::st(ET<TI>::ld(xr[c]) * inv * w[c]);
  }
}

template <typename TY, typename TO, bool VEC>
__global__ __launch_bounds__(RB) void add_rms_norm_kernel(
    float* __restrict__ residual, const typename ET<TY>::t* __restrict__ y,
    const float* __restrict__ w, const float eps, const int width,
    typename ET<TO>::t* __restrict__ out_copy) {
  __shared__ float scratch[4];
  const int64_t row = blockIdx.x;
  const typename ET<TY>::t* yr = y + row * width;
  if constexpr (VEC) {
    f32x4 yv[RV];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < RV; ++k) {
      const int c = (k * RB + threadIdx.x) * 4;
      yv[k] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (c < width) yv[k] = rld4<TY>(yr + c);
      ss += yv[k][0] * yv[k][0] + yv[k][1] * yv[k][1] +
            yv[k][2] * yv[k][2] + yv[k][3] * yv[k][3];
    }
    ss = rblock_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)width + eps);
#pragma unroll
    for (int k = 0; k < RV; ++k) {
      const int c = (k * RB + threadIdx.x) * 4;
      if (c >= width) continue;
      const f32x4 wv = *reinterpret_cast<const f32x4*>(w + c);
      f32x4 r = *reinterpret_cast<const f32x4*>(residual + row * width + c);
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = r[e] + yv[k][e] * inv * wv[e];
      *reinterpret_cast<f32x4*>(residual + row * width + c) = r;
      if (out_copy != nullptr) rst4<TO>(out_copy + row * width + c, r);
    }
  } else {
    float ss = 0.f;
    for (int c = threadIdx.x; c < width; c += RB) {
      const float v = ET<TY>::ld(yr[c]);
      ss += v * v;
    }
    ss = rblock_sum(ss, scratch);
    const float inv = 1.f / sqrtf(ss / (float)width + eps);
    for (int c = threadIdx.x; c < width; c += RB) {
      const float r =
          residual[row * width + c] + ET<TY>::ld(yr[c]) * inv * w[c];
      residual[row * width + c] = r;
      if (out_copy != nullptr) out_copy[row * width + c] = ET<TO>::st(r);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(RB) void relu2_kernel(
    typename ET<T>::t* __restrict__ out,
    const typename ET<T>::t* __restrict__ x, const int64_t n) {
  const int64_t i0 = ((int64_t)blockIdx.x * RB + threadIdx.x) * 4;
  if (i0 + 4 <= n) {
    f32x4 v = rld4<T>(x + i0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float r = fmaxf(v[e], 0.f);
      v[e] = r * r;
    }
    rst4<T>(out + i0, v);
  } else {
    for (int64_t i = i0; i < n; ++i) {
      const float r = fmaxf(ET<T>::ld(x[i]), 0.f);
      out[i] = ET<T>::st(r * r);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(RB) void logit_softcap_kernel(
    float* __restrict__ out, const typename ET<T>::t* __restrict__ x,
    const float cap, const int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * RB + threadIdx.x;
  if (i < n) out[i] = cap * tanhf(ET<T>::ld(x[i]) / cap);
}

template <typename T>
__global__ __launch_bounds__(RB) void sigmoid_gate_mul_kernel(
    typename ET<T>::t* __restrict__ out,
    const typename ET<T>::t* __restrict__ x, const int64_t x_st,
    const int64_t x_sh, const typename ET<T>::t* __restrict__ gate,
    const int64_t g_st, const int H, const int D) {
  const int64_t t = blockIdx.x;
  const int W = H * D;
  for (int c = threadIdx.x; c < W; c += RB) {
    const int h = c / D, d = c - h * D;
    const float v = ET<T>::ld(x[t * x_st + h * x_sh + d]);
    const float z = ET<T>::ld(gate[t * g_st + c]);
    out[t * W + c] = ET<T>::st(v / (1.f + expf(-z)));
  }
}

}  // namespace

#define RDISPATCH(DTYPE, FN)                                      \
  if ((DTYPE) == torch::kBFloat16) { FN(BF16Tag); }               \
  else if ((DTYPE) == torch::kHalf) { FN(FP16Tag); }              \
  else if ((DTYPE) == torch::kFloat32) { FN(F32Tag); }            \
  else { TORCH_CHECK(false, "unsupported dtype"); }

torch::Tensor scaled_embedding(torch::Tensor ids, torch::Tensor table,
                               double scale) {
  TORCH_CHECK(ids.scalar_type() == torch::kInt64 && ids.is_contiguous());
  TORCH_CHECK(table.dim() == 2 && table.is_contiguous());
  const int T = ids.numel(), width = table.size(1);
  auto out = torch::empty({T, width},
                          table.options().dtype(torch::kFloat32));
  if (T == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
#define L1(TT)                                                             \
  hipLaunchKernelGGL((scaled_embedding_kernel<TT>), dim3(T), dim3(RB), 0,  \
                     stream, out.data_ptr<float>(),                        \
                     ids.data_ptr<int64_t>(),                              \
                     (const ET<TT>::t*)table.data_ptr(), (float)scale,     \
                     width)
  RDISPATCH(table.scalar_type(), L1);
#undef L1
  HIP_CHECK_KERNEL();
  return out;
}

torch::Tensor rms_norm_cast(torch::Tensor x, torch::Tensor weight,
                            double eps, torch::ScalarType out_dtype) {
  TORCH_CHECK(x.is_contiguous() && x.dim() == 2);
  TORCH_CHECK(weight.scalar_type() == torch::kFloat32 &&
              weight.is_contiguous() && weight.numel() == x.size(1));
  auto out = torch::empty(x.sizes(), x.options().dtype(out_dtype));
  const int rows = x.size(0), width = x.size(1);
  if (rows == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = width % 4 == 0 && width <= 4 * RB * RV;
#define L3(TI, TO, V)                                                      \
  hipLaunchKernelGGL((rms_norm_cast_kernel<TI, TO, V>), dim3(rows),        \
                     dim3(RB), 0, stream, (ET<TO>::t*)out.data_ptr(),      \
                     (const ET<TI>::t*)x.data_ptr(),                       \
                     weight.data_ptr<float>(), (float)eps, width)
#define L2(TI, TO) if (vec) { L3(TI, TO, true); } else { L3(TI, TO, false); }
#define L1(TI)                                                             \
  if (out_dtype == torch::kFloat32) { L2(TI, F32Tag); }                    \
  else if (out_dtype == torch::kBFloat16) { L2(TI, BF16Tag); }             \
  else if (out_dtype == torch::kHalf) { L2(TI, FP16Tag); }                 \
  else { TORCH_CHECK(false, "unsupported out dtype"); }
  RDISPATCH(x.scalar_type(), L1);
#undef L1
#undef L2
#undef L3
  HIP_CHECK_KERNEL();
  return out;
}

torch::Tensor add_rms_norm(torch::Tensor residual, torch::Tensor y,
                           torch::Tensor weight, double eps,
                           c10::optional<torch::ScalarType> out_dtype) {
  TORCH_CHECK(residual.scalar_type() == torch::kFloat32 &&
              residual.is_contiguous() && y.is_contiguous());
  TORCH_CHECK(residual.sizes() == y.sizes() && residual.dim() == 2);
  TORCH_CHECK(weight.scalar_type() == torch::kFloat32 &&
              weight.is_contiguous() && weight.numel() == y.size(1));
  const int rows = residual.size(0), width = residual.size(1);
  const bool copy = out_dtype.has_value() && *out_dtype != torch::kFloat32;
  torch::Tensor out = residual;
  if (copy) out = torch::empty(residual.sizes(),
                               residual.options().dtype(*out_dtype));
  if (rows == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const bool vec = width % 4 == 0 && width <= 4 * RB * RV;
#define L3(TY, TO, V)                                                      \
  hipLaunchKernelGGL((add_rms_norm_kernel<TY, TO, V>), dim3(rows),         \
                     dim3(RB), 0, stream, residual.data_ptr<float>(),      \
                     (const ET<TY>::t*)y.data_ptr(),                       \
                     weight.data_ptr<float>(), (float)eps, width,          \
                     copy ? (ET<TO>::t*)out.data_ptr() : nullptr)
#define L2(TY, TO) if (vec) { L3(TY, TO, true); } else { L3(TY, TO, false); }
#define L1(TY)                                                             \
  if (!copy) { L2(TY, F32Tag); }                                           \
  else if (*out_dtype == torch::kBFloat16) { L2(TY, BF16Tag); }            \
  else if (*out_dtype == torch::kHalf) { L2(TY, FP16Tag); }                \
  else { TORCH_CHECK(false, "unsupported out dtype"); }
  RDISPATCH(y.scalar_type(), L1);
#undef L1
#undef L2
#undef L3
  HIP_CHECK_KERNEL();
  return out;
}

torch::Tensor relu2(torch::Tensor x) {
  TORCH_CHECK(x.is_contiguous());
  auto out = torch::empty_like(x);
  const int64_t n = x.numel();
  if (n == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const int blocks = (int)((n + RB * 4 - 1) / (RB * 4));
#define L1(TT)                                                             \
  hipLaunchKernelGGL((relu2_kernel<TT>), dim3(blocks), dim3(RB), 0, stream,\
                     (ET<TT>::t*)out.data_ptr(),                           \
                     (const ET<TT>::t*)x.data_ptr(), n)
  RDISPATCH(x.scalar_type(), L1);
#undef L1
  HIP_CHECK_KERNEL();
  return out;
}

torch::Tensor logit_softcap(torch::Tensor logits, double cap) {
  TORCH_CHECK(logits.is_contiguous() && cap > 0);
  auto out = torch::empty(logits.sizes(),
                          logits.options().dtype(torch::kFloat32));
  const int64_t n = logits.numel();
  if (n == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
  const int blocks = (int)((n + RB - 1) / RB);
#define L1(TT)                                                             \
  hipLaunchKernelGGL((logit_softcap_kernel<TT>), dim3(blocks), dim3(RB),   \
                     0, stream, out.data_ptr<float>(),                     \
                     (const ET<TT>::t*)logits.data_ptr(), (float)cap, n)
  RDISPATCH(logits.scalar_type(), L1);
#undef L1
  HIP_CHECK_KERNEL();
  return out;
}

torch::Tensor sigmoid_gate_mul(torch::Tensor x, torch::Tensor gate) {
  TORCH_CHECK(x.dim() == 3 && gate.dim() == 2);
  TORCH_CHECK(x.stride(2) == 1 && gate.stride(1) == 1);
  TORCH_CHECK(x.scalar_type() == gate.scalar_type());
  const int T = x.size(0), H = x.size(1), D = x.size(2);
  TORCH_CHECK(gate.size(0) == T && gate.size(1) == (int64_t)H * D);
  auto out = torch::empty({T, (int64_t)H * D}, x.options());
  if (T == 0) return out;
  auto stream = c10::hip::getCurrentHIPStream().stream();
#define L1(TT)                                                             \
  hipLaunchKernelGGL((sigmoid_gate_mul_kernel<TT>), dim3(T), dim3(RB), 0,  \
                     stream, (ET<TT>::t*)out.data_ptr(),                   \
                     (const ET<TT>::t*)x.data_ptr(), x.stride(0),          \
                     x.stride(1), (const ET<TT>::t*)gate.data_ptr(),       \
                     gate.stride(0), H, D)
  RDISPATCH(x.scalar_type(), L1);
#undef L1
  HIP_CHECK_KERNEL();
  return out;
}

}  // namespace vllm_amd
