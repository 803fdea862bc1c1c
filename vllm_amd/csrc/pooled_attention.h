// Element traits shared by the pooled-window attention kernels: the
// same templates serve bf16, fp16 and fp32 tensors.
#pragma once

#include "common.h"

namespace vllm_amd {

struct F32Tag {};

template <typename Tag> struct ET;
template <> struct ET<BF16Tag> {
  using t = short;
  static DEVINL float ld(short v) { return bf16_to_f32(v); }
  static DEVINL short st(float f) { return f32_to_bf16(f); }
};
template <> struct ET<FP16Tag> {
  using t = short;
  static DEVINL float ld(short v) { return f16_to_f32(v); }
  static DEVINL short st(float f) { return f16_from_f32(f); }
};
template <> struct ET<F32Tag> {
  using t = float;
  static DEVINL float ld(float v) { return v; }
  static DEVINL float st(float f) { return f; }
};

}  // namespace vllm_amd
