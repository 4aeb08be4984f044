// Expert GEMMs of the table-routed MoE over moe_align tiles: out[slot, :] = act(W[e] . x[row(slot)])
// where a tile is `tile` consecutive expert-sorted slots of one expert (tile_expert[t], -1 = unused),
// row(slot) = slots[slot] / gather_k (the token row of the pair; first GEMM) or the slot itself
// (second GEMM) and act = squared ReLU or none. Any N and K: edges are bounds-checked. A workgroup
// computes a [32 slots x 64 columns] block, x and W staged through LDS in K-chunks of 32, fp32
// accumulation; bf16 and fp32 element types.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

constexpr int kTM = 32, kTN = 64, kTK = 32;

template <typename T>
__global__ __launch_bounds__(256) void expert_gemm_kernel(T* __restrict__ out, const T* __restrict__ x, long x_ld,
                                                          const T* __restrict__ w, const int* __restrict__ slots,
                                                          const int* __restrict__ tile_expert, int tile, int gather_k,
                                                          int N, int K, int relu2) {
  __shared__ float xs[kTM][kTK + 1], ws[kTN][kTK + 1];
  __shared__ long xrow[kTM];
  const int e = tile_expert[(blockIdx.y * kTM) / tile];
  if (e < 0) return;
  const int tid = threadIdx.x;
  const int slot0 = blockIdx.y * kTM, n0 = blockIdx.x * kTN;
  if (tid < kTM) {
    const int p = slots[slot0 + tid];
    xrow[tid] = p < 0 ? -1 : (gather_k > 0 ? (long)(p / gather_k) : (long)(slot0 + tid)) * x_ld;
  }
  const T* we = w + (long)e * N * K;
  const int tx = tid & 15, ty = tid >> 4;  // 4 columns x 2 slots per thread
  float acc[2][4] = {};
  for (int k0 = 0; k0 < K; k0 += kTK) {
    __syncthreads();
    for (int idx = tid; idx < kTM * kTK; idx += 256) {
      const int r = idx / kTK, k = idx % kTK;
      const long xr = xrow[r];
      xs[r][k] = (xr >= 0 && k0 + k < K) ? ldf<T>(x, xr + k0 + k) : 0.f;
    }
    for (int idx = tid; idx < kTN * kTK; idx += 256) {
      const int c = idx / kTK, k = idx % kTK;
      ws[c][k] = (n0 + c < N && k0 + k < K) ? ldf<T>(we, (long)(n0 + c) * K + k0 + k) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int k = 0; k < kTK; ++k) {
      const float a0 = xs[ty * 2][k], a1 = xs[ty * 2 + 1][k];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float b = ws[tx + 16 * j][k];
        acc[0][j] = __builtin_fmaf(a0, b, acc[0][j]);
        acc[1][j] = __builtin_fmaf(a1, b, acc[1][j]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = ty * 2 + i;
    if (xrow[r] < 0) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = n0 + tx + 16 * j;
      if (c >= N) continue;
      float v = acc[i][j];
      if (relu2) { v = fmaxf(v, 0.f); v *= v; }
      stf<T>(out, (long)(slot0 + r) * N + c, v);
    }
  }
}

}  // namespace

void launch_expert_gemm(void* out, const void* x, long x_ld, const void* w, const int* slots, const int* tile_expert,
                        int ntiles_cap, int tile, int gather_k, int N, int K, bool relu2, bool f32, hipStream_t s) {
  if (ntiles_cap <= 0) return;
  dim3 grid((N + kTN - 1) / kTN, (long)ntiles_cap * tile / kTM);
  if (f32)
    expert_gemm_kernel<float><<<grid, 256, 0, s>>>((float*)out, (const float*)x, x_ld, (const float*)w, slots,
                                                   tile_expert, tile, gather_k, N, K, relu2);
  else
    expert_gemm_kernel<unsigned short><<<grid, 256, 0, s>>>((unsigned short*)out, (const unsigned short*)x, x_ld,
                                                            (const unsigned short*)w, slots, tile_expert, tile,
                                                            gather_k, N, K, relu2);
}

}  // namespace hipserve
