// Column sums of a [rows, S] matrix: out[s] = sum over r of x[r, s].
//
// This is the bias gradient of a linear layer, d loss / d bias = sum over rows of the output's gradient, which
// the SSM layer needs twice per step (A_proj and out_proj carry a bias, quick_ssm/layers.py:50-58).  Two small
// launches, fp32 accumulation in a fixed order, so results repeat bit for bit: the first spreads the rows over
// `P` row chunks and writes one fp32 partial row per chunk, the second adds the partial rows in order.
#include "scan_common.h"

namespace qssm {

// Workgroup (bx, by): 64 lanes x VEC columns starting at bx * 64 * VEC, rows of chunk by; its four wavefronts take
// every fourth row of the chunk and meet in LDS.
template <typename T, int VEC>
__global__ void __launch_bounds__(256) colsum_partial_kernel(const T* __restrict__ x, int64_t ld, int64_t rows, int S,
                                                            int64_t rows_per_chunk, float* __restrict__ partial) {
  __shared__ float part[4][64 * VEC];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int col = (blockIdx.x * 64 + lane) * VEC;
  const int64_t lo = (int64_t)blockIdx.y * rows_per_chunk;
  const int64_t hi = lo + rows_per_chunk < rows ? lo + rows_per_chunk : rows;
  float acc[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) acc[v] = 0.0f;
  if (col < S) {
    const T* p = x + col;
    int64_t r = lo + w;
    // four rows of a wavefront in flight at a time
    for (; r + 12 < hi; r += 16) {
      Words<T, VEC> q[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) q[k] = load_stream<T, VEC>((const char*)(p + (r + 4 * k) * ld), 0u);
#pragma unroll
      for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int v = 0; v < VEC; ++v) acc[v] += elem(q[k], v);
    }
    for (; r < hi; r += 4) {
      const Words<T, VEC> q = load_stream<T, VEC>((const char*)(p + r * ld), 0u);
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[v] += elem(q, v);
    }
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) part[w][lane * VEC + v] = acc[v];
  __syncthreads();
  if (w == 0 && col < S) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const int c = lane * VEC + v;
      partial[(int64_t)blockIdx.y * S + col + v] = (part[0][c] + part[1][c]) + (part[2][c] + part[3][c]);
    }
  }
}

// out[col] = partial[0][col] + partial[1][col] + ... in that order: 64 columns x 4 row groups per workgroup.
template <typename T>
__global__ void __launch_bounds__(256) colsum_final_kernel(const float* __restrict__ partial, int n, int S, T* __restrict__ out) {
  __shared__ float part[4][64];
  const int cl = threadIdx.x & 63, grp = threadIdx.x >> 6;
  const int col = blockIdx.x * 64 + cl;
  const int per = (n + 3) / 4;
  float sum = 0.0f;
  if (col < S) {
    const int lo = grp * per, hi = n < lo + per ? n : lo + per;
    for (int i = lo; i < hi; ++i) sum += partial[(int64_t)i * S + col];
  }
  part[grp][cl] = sum;
  __syncthreads();
  if (grp == 0 && col < S) out[col] = (T)((part[0][cl] + part[1][cl]) + (part[2][cl] + part[3][cl]));
}

template <typename T>
static bool launch_colsum(const void* x, int64_t ld, int64_t rows, int S, int vec, float* partial, int chunks, void* out,
                          hipStream_t stream) {
  const int64_t per = (rows + chunks - 1) / chunks;
  const dim3 grid((unsigned)((S + 64 * vec - 1) / (64 * vec)), (unsigned)chunks);
  const T* xp = reinterpret_cast<const T*>(x);
  if (vec == 4) hipLaunchKernelGGL((colsum_partial_kernel<T, 4>), grid, dim3(256), 0, stream, xp, ld, rows, S, per, partial);
  else if (vec == 2) hipLaunchKernelGGL((colsum_partial_kernel<T, 2>), grid, dim3(256), 0, stream, xp, ld, rows, S, per, partial);
  else hipLaunchKernelGGL((colsum_partial_kernel<T, 1>), grid, dim3(256), 0, stream, xp, ld, rows, S, per, partial);
  hipLaunchKernelGGL((colsum_final_kernel<T>), dim3((unsigned)((S + 63) / 64)), dim3(256), 0, stream, partial, chunks, S,
                     reinterpret_cast<T*>(out));
  return true;
}

bool launch_colsum_any(int dtype, const void* x, int64_t ld, int64_t rows, int S, int vec, float* partial, int chunks,
                       void* out, hipStream_t stream) {
  if (dtype == QSSM_F32) return launch_colsum<float>(x, ld, rows, S, vec, partial, chunks, out, stream);
  if (dtype == QSSM_F16) return launch_colsum<f16_t>(x, ld, rows, S, vec, partial, chunks, out, stream);
  if (dtype == QSSM_BF16) return launch_colsum<bf16_t>(x, ld, rows, S, vec, partial, chunks, out, stream);
  return false;
}

}  // namespace qssm
