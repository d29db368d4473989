// Shared helpers for the hybrid-mixer kernels (gfx950 / CDNA4).
//
// Every kernel here is templated on the activation storage type: bf16 (held
// as unsigned short, as in the rest of the kernels) or float. All arithmetic
// is fp32; only loads/stores convert.
#pragma once

#include "../ops/common.h"

namespace xllm {
namespace hyb {

template <typename T> struct IO;
template <> struct IO<float> {
  static XLLM_DEV float ld(const float* p) { return *p; }
  static XLLM_DEV void st(float* p, float v) { *p = v; }
  static XLLM_DEV float rnd(float v) { return v; }
};
template <> struct IO<unsigned short> {
  static XLLM_DEV float ld(const unsigned short* p) { return bf16_to_f32(*p); }
  static XLLM_DEV void st(unsigned short* p, float v) { *p = f32_to_bf16(v); }
  static XLLM_DEV float rnd(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};

XLLM_DEV float sigmoidf_(float x) { return 1.0f / (1.0f + __expf(-x)); }
XLLM_DEV float siluf_(float x) { return x / (1.0f + __expf(-x)); }

}  // namespace hyb
}  // namespace xllm
