// Residual update + grouped RMSNorm of the layer-list decoders, one workgroup per token row:
//   r = residual + ls1 * mix (ls1 null: 1) + ls2 * (1/top) * sum_j y[pair_slot[t*top + j]] + extra     (fp32, written back)
//   out = r / sqrt(mean over the element's group of r^2 + eps) * w
// The row is split into `groups` equal consecutive parts with their own mean square. The MoE
// combine (rows of the expert-sorted y picked through pair_slot) and the embedding re-added at
// the start of a loop pass (`extra`) ride along, so one launch sits between two layers.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

constexpr int kNT = 256;

template <typename T>
__global__ __launch_bounds__(kNT) void scaled_add_group_rmsnorm_kernel(
    T* __restrict__ out, float* __restrict__ residual, const float* __restrict__ w, int H, int groups, float eps,
    const T* __restrict__ mix, const float* __restrict__ ls1, const T* __restrict__ y,
    const int* __restrict__ pair_slot, int top, const float* __restrict__ ls2, const T* __restrict__ extra) {
  extern __shared__ float sm[];  // [H] squares, then [groups] inverse rms
  float* sq = sm;
  float* ginv = sm + H;
  const long t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float* r = residual + t * H;
  const float wtop = top > 0 ? 1.f / (float)top : 0.f;
  for (int e = tid; e < H; e += kNT) {
    float v = r[e];
    if (mix != nullptr) v += ls1 != nullptr ? ldf<T>(mix, t * H + e) * ls1[e] : ldf<T>(mix, t * H + e);
    if (y != nullptr) {
      float f = 0.f;
      for (int j = 0; j < top; ++j) f += ldf<T>(y, (long)pair_slot[t * top + j] * H + e);
      v += f * wtop * ls2[e];
    }
    if (extra != nullptr) v += ldf<T>(extra, t * H + e);
    r[e] = v;
    sq[e] = v * v;
  }
  __syncthreads();
  const int gs = H / groups;
  for (int g = wave; g < groups; g += kNT / 64) {  // one wave sums a group, in a fixed order
    float a = 0.f;
    for (int e = lane; e < gs; e += 64) a += sq[g * gs + e];
    a = wave_sum(a);
    if (lane == 0) ginv[g] = 1.f / sqrtf(a / (float)gs + eps);
  }
  __syncthreads();
  for (int e = tid; e < H; e += kNT) stf<T>(out, t * H + e, r[e] * ginv[e / gs] * w[e]);
}

}  // namespace

void launch_scaled_add_group_rmsnorm(void* out, float* residual, const float* w, int T, int H, int groups, float eps,
                                     const void* mix, const float* ls1, const void* y, const int* pair_slot, int top,
                                     const float* ls2, const void* extra, bool f32, hipStream_t s) {
  if (T <= 0) return;
  const size_t smem = (size_t)(H + groups) * sizeof(float);
  if (f32)
    scaled_add_group_rmsnorm_kernel<float><<<T, kNT, smem, s>>>(
        (float*)out, residual, w, H, groups, eps, (const float*)mix, ls1, (const float*)y, pair_slot, top, ls2,
        (const float*)extra);
  else
    scaled_add_group_rmsnorm_kernel<unsigned short><<<T, kNT, smem, s>>>(
        (unsigned short*)out, residual, w, H, groups, eps, (const unsigned short*)mix, ls1, (const unsigned short*)y,
        pair_slot, top, ls2, (const unsigned short*)extra);
}

}  // namespace hipserve
