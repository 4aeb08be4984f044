#pragma once
#include "hipserve/common.h"

namespace hipserve {

template <typename T> HS_DEVICE float ldf(const T* p, long i);
template <> HS_DEVICE float ldf<unsigned short>(const unsigned short* p, long i) { return bf16_to_f32(p[i]); }
template <> HS_DEVICE float ldf<float>(const float* p, long i) { return p[i]; }
template <typename T> HS_DEVICE void stf(T* p, long i, float v);
template <> HS_DEVICE void stf<unsigned short>(unsigned short* p, long i, float v) { p[i] = f32_to_bf16(v); }
template <> HS_DEVICE void stf<float>(float* p, long i, float v) { p[i] = v; }

HS_DEVICE float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }

}  // namespace hipserve
