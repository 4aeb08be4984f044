// minGRU scan. proj rows = [z | x | g] pre-activations (width each). Per sequence and channel,
//   z = sigmoid(zp + b_z), u = xp + b_x, c = u + 0.5 (u >= 0) or sigmoid(u),
//   S_t = (1 - z_t) S_{t-1} + z_t c_t,   y_t = S_t * silu(g_t),
// all in fp32, from the sequence's state slot (zero when the step starts at position 0) and back
// into it. A workgroup owns 64 channels of one sequence; its waves split the step's rows into
// consecutive segments: each wave first folds its segment into (A, B) with S_out = A S_in + B, the
// segment states are chained through LDS, and the segment is then replayed from its true S_in.
#include "seq_common.h"
#include "hipserve/seq_kernels.h"

namespace hipserve {
namespace {

constexpr int kMaxWaves = 16;

template <typename T>
__global__ __launch_bounds__(64 * kMaxWaves) void mingru_scan_kernel(
    T* __restrict__ y, float* __restrict__ state, const T* __restrict__ proj, const float* __restrict__ b_z,
    const float* __restrict__ b_x, const int* __restrict__ seq_cu, const int* __restrict__ seq_ctx,
    const int* __restrict__ seq_state, int width) {
  __shared__ float sa[kMaxWaves][64], sb[kMaxWaves][64];
  const int s = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int c = blockIdx.y * 64 + lane;
  const int r0 = seq_cu[s], n = seq_cu[s + 1] - r0;
  if (n <= 0) return;
  const bool live = c < width;
  const int cc = live ? c : 0;
  const float bz = b_z[cc], bx = b_x[cc];
  const int per = (n + nw - 1) / nw;
  const int a = min(wave * per, n), b = min(a + per, n);
  // rows go through in blocks of kB: the block's loads are issued together, then the serial update
  constexpr int kB = 8;
  const long ld = 3L * width;
  float A = 1.f, B = 0.f;
  for (int t0 = a; t0 < b; t0 += kB) {
    float zp[kB], xp[kB];
#pragma unroll
    for (int i = 0; i < kB; ++i) {
      const long base = (long)(r0 + min(t0 + i, b - 1)) * ld;
      zp[i] = ldf<T>(proj, base + cc);
      xp[i] = ldf<T>(proj, base + width + cc);
    }
#pragma unroll
    for (int i = 0; i < kB; ++i) {
      if (t0 + i < b) {
        const float z = sigmoid_f(zp[i] + bz);
        const float u = xp[i] + bx;
        const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
        A *= 1.f - z;
        B = (1.f - z) * B + z * cand;
      }
    }
  }
  sa[wave][lane] = A;
  sb[wave][lane] = B;
  // every wave reads the carried state before the barrier; the slot is rewritten only after it
  const long slot = (long)seq_state[s] * width + cc;
  float S = (seq_ctx[s] - n > 0) ? state[slot] : 0.f;
  __syncthreads();
  for (int k = 0; k < wave; ++k) S = sa[k][lane] * S + sb[k][lane];
  for (int t0 = a; t0 < b; t0 += kB) {
    float zp[kB], xp[kB], gp[kB];
#pragma unroll
    for (int i = 0; i < kB; ++i) {
      const long base = (long)(r0 + min(t0 + i, b - 1)) * ld;
      zp[i] = ldf<T>(proj, base + cc);
      xp[i] = ldf<T>(proj, base + width + cc);
      gp[i] = ldf<T>(proj, base + 2 * width + cc);
    }
#pragma unroll
    for (int i = 0; i < kB; ++i) {
      if (t0 + i < b) {
        const float z = sigmoid_f(zp[i] + bz);
        const float u = xp[i] + bx;
        const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
        S = (1.f - z) * S + z * cand;
        if (live) stf<T>(y, (long)(r0 + t0 + i) * width + c, S * (gp[i] * sigmoid_f(gp[i])));
      }
    }
  }
  // the wave that holds the last row leaves the state (empty trailing segments keep S = chained value)
  if (live && wave == nw - 1) state[slot] = S;
}

}  // namespace

void launch_mingru_scan(void* y, float* state, const void* proj, const float* b_z, const float* b_x,
                        const int* seq_cu, const int* seq_ctx, const int* seq_state, int nseq, int width, int max_q,
                        bool f32, hipStream_t s) {
  if (nseq <= 0 || max_q <= 0) return;
  const int nw = max_q <= 8 ? 1 : (max_q <= 64 ? 4 : kMaxWaves);
  dim3 grid(nseq, (width + 63) / 64), block(64 * nw);
  if (f32)
    mingru_scan_kernel<float><<<grid, block, 0, s>>>((float*)y, state, (const float*)proj, b_z, b_x, seq_cu, seq_ctx,
                                                     seq_state, width);
  else
    mingru_scan_kernel<unsigned short><<<grid, block, 0, s>>>((unsigned short*)y, state, (const unsigned short*)proj,
                                                              b_z, b_x, seq_cu, seq_ctx, seq_state, width);
}

}  // namespace hipserve
