// RMSNorm of the SSM layer for gfx950: y = x * weight / sqrt(mean(x^2) + eps) over the last axis,
// and its backward (dx, dweight).
//
// It takes the place of the reference's RMSNorm.forward (quick_ssm/layers.py:14-17: pow, mean, add,
// sqrt, divide, multiply - six passes over [rows, H] and as many again recorded for autograd).
// One to eight wavefronts own a row at a time (so that a lane keeps at most 16 elements of it): the
// row is read once, kept in registers, reduced with cross-lane moves (and through LDS when wavefronts
// share it) and written once.  Arithmetic is fp32 whatever the storage; each result is rounded once.
// Rows wider than that take a variant that reads the row again from cache instead of keeping it.
//
//   r = 1 / sqrt(mean(x^2) + eps)         y = x * w * r
//   g = dy * w     s = sum(g * x)          dx = r * g - x * r^3 * s / H       dw = sum over rows dy * x * r
//
// dw is summed in a fixed order (per workgroup in registers, across the wavefronts of a workgroup
// through LDS, across workgroups by a second small launch), so results do not change from run to run.
#include "scan_common.h"

namespace qssm {

constexpr int kNormWaves = 8;                 // wavefronts (rows in flight) per workgroup
constexpr int kNormThreads = 64 * kNormWaves;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

template <typename T, int V>
__device__ __forceinline__ Words<T, V> load_cached(const char* base, uint32_t byte_off) {
  typedef typename RawOf<sizeof(T) * V>::type raw_t;
  const raw_t r = *reinterpret_cast<const raw_t*>(base + byte_off);
  Words<T, V> out;
  if constexpr (sizeof(T) * V <= 4) {
    out.w[0] = (uint32_t)r;
  } else {
#pragma unroll
    for (int k = 0; k < Words<T, V>::N; ++k) out.w[k] = r[k];
  }
  return out;
}

// Sum of `v` over the W wavefronts that share a row (every lane gets the total).  `red` holds one float
// per wavefront of the workgroup; every wavefront of the workgroup must call this the same number of times.
template <int W>
__device__ __forceinline__ float row_sum(float v, float* red, int wave) {
  v = wave_sum(v);
  if constexpr (W > 1) {
    __syncthreads();  // the previous round's readers are done with `red`
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    const int first = wave & ~(W - 1);
    v = 0.0f;
#pragma unroll
    for (int k = 0; k < W; ++k) v += red[first + k];
  }
  return v;
}

// ---- rows that fit in registers: W wavefronts share a row, NCH chunks of V elements per lane --------

template <typename T, int V, int NCH, int W>
__global__ void __launch_bounds__(kNormThreads) rmsnorm_fwd_kernel(const NormFwdArgs p) {
  __shared__ float red[kNormWaves];
  constexpr int RPW = kNormWaves / W;  // rows a workgroup works on at a time
  const int wave = threadIdx.x >> 6;
  const int group = threadIdx.x / (64 * W), gl = threadIdx.x % (64 * W);
  const float inv_h = 1.0f / (float)p.H;
  Words<T, V> w[NCH];
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int col = (k * 64 * W + gl) * V;
    w[k] = fill_words<T, V>(false);
    if (col < p.H) w[k] = load_cached<T, V>((const char*)p.w, (uint32_t)(col * (int)sizeof(T)));
  }
  for (int64_t base = (int64_t)blockIdx.x * RPW; base < p.rows; base += (int64_t)gridDim.x * RPW) {
    const int64_t row = base + group;
    const bool live = row < p.rows;
    const char* xr = (const char*)p.x + row * p.ld_x * (int64_t)sizeof(T);
    char* yr = (char*)p.y + row * (int64_t)p.H * (int64_t)sizeof(T);
    Words<T, V> x[NCH];
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
      const int col = (k * 64 * W + gl) * V;
      x[k] = fill_words<T, V>(false);
      if (live && col < p.H) x[k] = load_stream<T, V>(xr, (uint32_t)(col * (int)sizeof(T)));
    }
    float ss = 0.0f;
#pragma unroll
    for (int k = 0; k < NCH; ++k)
#pragma unroll
      for (int v = 0; v < V; ++v) ss += elem(x[k], v) * elem(x[k], v);
    ss = row_sum<W>(ss, red, wave);
    const float r = 1.0f / sqrtf(ss * inv_h + p.eps);
    if (live && gl == 0 && p.rstd != nullptr) p.rstd[row] = r;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
      const int col = (k * 64 * W + gl) * V;
      float out[V];
#pragma unroll
      for (int v = 0; v < V; ++v) out[v] = elem(x[k], v) * (elem(w[k], v) * r);
      if (live && col < p.H) store_stream<T, V>(yr, (uint32_t)(col * (int)sizeof(T)), out);
    }
  }
}

template <typename T, int V, int NCH, int W>
__global__ void __launch_bounds__(kNormThreads) rmsnorm_bwd_kernel(const NormBwdArgs p) {
  extern __shared__ __align__(16) float lds[];  // [H] this workgroup's dw
  __shared__ float red[kNormWaves];
  constexpr int RPW = kNormWaves / W;
  const int wave = threadIdx.x >> 6;
  const int group = threadIdx.x / (64 * W), gl = threadIdx.x % (64 * W);
  const float inv_h = 1.0f / (float)p.H;
  Words<T, V> w[NCH];
  float acc[NCH][V];
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int col = (k * 64 * W + gl) * V;
    w[k] = fill_words<T, V>(false);
    if (col < p.H) w[k] = load_cached<T, V>((const char*)p.w, (uint32_t)(col * (int)sizeof(T)));
#pragma unroll
    for (int v = 0; v < V; ++v) acc[k][v] = 0.0f;
  }
  for (int64_t base = (int64_t)blockIdx.x * RPW; base < p.rows; base += (int64_t)gridDim.x * RPW) {
    const int64_t row = base + group;
    const bool live = row < p.rows;
    const char* xr = (const char*)p.x + row * p.ld_x * (int64_t)sizeof(T);
    const char* gr = (const char*)p.dy + row * p.ld_dy * (int64_t)sizeof(T);
    char* dr = (char*)p.dx + row * (int64_t)p.H * (int64_t)sizeof(T);
    Words<T, V> x[NCH], dy[NCH];
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
      const int col = (k * 64 * W + gl) * V;
      x[k] = fill_words<T, V>(false);
      dy[k] = fill_words<T, V>(false);
      if (live && col < p.H) {
        x[k] = load_stream<T, V>(xr, (uint32_t)(col * (int)sizeof(T)));
        dy[k] = load_stream<T, V>(gr, (uint32_t)(col * (int)sizeof(T)));
      }
    }
    float r;
    if (p.rstd != nullptr) {  // uniform over the launch
      r = live ? p.rstd[row] : 0.0f;
    } else {
      float ss = 0.0f;
#pragma unroll
      for (int k = 0; k < NCH; ++k)
#pragma unroll
        for (int v = 0; v < V; ++v) ss += elem(x[k], v) * elem(x[k], v);
      r = 1.0f / sqrtf(row_sum<W>(ss, red, wave) * inv_h + p.eps);
      if (!live) r = 0.0f;
    }
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < NCH; ++k)
#pragma unroll
      for (int v = 0; v < V; ++v) s += elem(dy[k], v) * elem(w[k], v) * elem(x[k], v);
    s = row_sum<W>(s, red, wave);
    const float q = r * r * r * s * inv_h;
#pragma unroll
    for (int k = 0; k < NCH; ++k) {
      const int col = (k * 64 * W + gl) * V;
      float out[V];
#pragma unroll
      for (int v = 0; v < V; ++v) {
        const float xv = elem(x[k], v), gv = elem(dy[k], v);
        out[v] = r * (gv * elem(w[k], v)) - xv * q;
        acc[k][v] += gv * xv * r;   // rows past the end were filled with zeros
      }
      if (live && col < p.H) store_stream<T, V>(dr, (uint32_t)(col * (int)sizeof(T)), out);
    }
  }
  // dw of this workgroup: the row groups add their sums one after the other, always in the same order.
  for (int turn = 0; turn < RPW; ++turn) {
    if (group == turn) {
#pragma unroll
      for (int k = 0; k < NCH; ++k) {
        const int col = (k * 64 * W + gl) * V;
        if (col < p.H) {
#pragma unroll
          for (int v = 0; v < V; ++v) lds[col + v] = (turn == 0 ? 0.0f : lds[col + v]) + acc[k][v];
        }
      }
    }
    __syncthreads();
  }
  float* out = p.partial + (int64_t)blockIdx.x * p.H;
  for (int col = threadIdx.x; col < p.H; col += kNormThreads) out[col] = lds[col];
}

// ---- rows of any width: the whole workgroup shares a row and reads it again from cache ---------------

template <typename T, int V>
__global__ void __launch_bounds__(kNormThreads) rmsnorm_fwd_wide_kernel(const NormFwdArgs p) {
  __shared__ float red[kNormWaves];
  const int wave = threadIdx.x >> 6;
  const float inv_h = 1.0f / (float)p.H;
  for (int64_t row = blockIdx.x; row < p.rows; row += gridDim.x) {
    const char* xr = (const char*)p.x + row * p.ld_x * (int64_t)sizeof(T);
    char* yr = (char*)p.y + row * (int64_t)p.H * (int64_t)sizeof(T);
    float ss = 0.0f;
    for (int col = threadIdx.x * V; col < p.H; col += kNormThreads * V) {
      const Words<T, V> xv = load_cached<T, V>(xr, (uint32_t)(col * (int)sizeof(T)));
#pragma unroll
      for (int v = 0; v < V; ++v) ss += elem(xv, v) * elem(xv, v);
    }
    const float r = 1.0f / sqrtf(row_sum<kNormWaves>(ss, red, wave) * inv_h + p.eps);
    if (threadIdx.x == 0 && p.rstd != nullptr) p.rstd[row] = r;
    for (int col = threadIdx.x * V; col < p.H; col += kNormThreads * V) {
      const Words<T, V> xv = load_cached<T, V>(xr, (uint32_t)(col * (int)sizeof(T)));
      const Words<T, V> wv = load_cached<T, V>((const char*)p.w, (uint32_t)(col * (int)sizeof(T)));
      float out[V];
#pragma unroll
      for (int v = 0; v < V; ++v) out[v] = elem(xv, v) * (elem(wv, v) * r);
      store_stream<T, V>(yr, (uint32_t)(col * (int)sizeof(T)), out);
    }
  }
}

// The workgroup keeps its dw row in `partial` itself (read-modify-write from cache; a column is always
// touched by the same lane), one row of `partial` per workgroup.
template <typename T, int V>
__global__ void __launch_bounds__(kNormThreads) rmsnorm_bwd_wide_kernel(const NormBwdArgs p) {
  __shared__ float red[kNormWaves];
  const int wave = threadIdx.x >> 6;
  const float inv_h = 1.0f / (float)p.H;
  float* mine = p.partial + (int64_t)blockIdx.x * p.H;
  for (int col = threadIdx.x * V; col < p.H; col += kNormThreads * V)
#pragma unroll
    for (int v = 0; v < V; ++v) mine[col + v] = 0.0f;
  for (int64_t row = blockIdx.x; row < p.rows; row += gridDim.x) {
    const char* xr = (const char*)p.x + row * p.ld_x * (int64_t)sizeof(T);
    const char* gr = (const char*)p.dy + row * p.ld_dy * (int64_t)sizeof(T);
    char* dr = (char*)p.dx + row * (int64_t)p.H * (int64_t)sizeof(T);
    float ss = 0.0f, s = 0.0f;
    for (int col = threadIdx.x * V; col < p.H; col += kNormThreads * V) {
      const uint32_t off = (uint32_t)(col * (int)sizeof(T));
      const Words<T, V> xv = load_cached<T, V>(xr, off), gv = load_cached<T, V>(gr, off);
      const Words<T, V> wv = load_cached<T, V>((const char*)p.w, off);
#pragma unroll
      for (int v = 0; v < V; ++v) {
        ss += elem(xv, v) * elem(xv, v);
        s += elem(gv, v) * elem(wv, v) * elem(xv, v);
      }
    }
    ss = row_sum<kNormWaves>(ss, red, wave);
    s = row_sum<kNormWaves>(s, red, wave);
    const float r = p.rstd != nullptr ? p.rstd[row] : 1.0f / sqrtf(ss * inv_h + p.eps);
    const float q = r * r * r * s * inv_h;
    for (int col = threadIdx.x * V; col < p.H; col += kNormThreads * V) {
      const uint32_t off = (uint32_t)(col * (int)sizeof(T));
      const Words<T, V> xv = load_cached<T, V>(xr, off), gv = load_cached<T, V>(gr, off);
      const Words<T, V> wv = load_cached<T, V>((const char*)p.w, off);
      float out[V];
#pragma unroll
      for (int v = 0; v < V; ++v) {
        out[v] = r * (elem(gv, v) * elem(wv, v)) - elem(xv, v) * q;
        mine[col + v] += elem(gv, v) * elem(xv, v) * r;
      }
      store_stream<T, V>(dr, off, out);
    }
  }
}

// dw[col] = sum over the first n rows of `partial`, rows in order: 64 columns x 16 row groups per workgroup.
template <typename T>
__global__ void __launch_bounds__(1024) rmsnorm_dw_kernel(const float* partial, int n, int H, T* dw) {
  __shared__ float part[16][64];
  const int cl = threadIdx.x & 63, grp = threadIdx.x >> 6;
  const int col = blockIdx.x * 64 + cl;
  const int per = (n + 15) / 16;
  float sum = 0.0f;
  if (col < H) {
    const int lo = grp * per, hi = min(n, lo + per);
    for (int i = lo; i < hi; ++i) sum += partial[(int64_t)i * H + col];
  }
  part[grp][cl] = sum;
  __syncthreads();
  if (grp == 0 && col < H) {
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < 16; ++k) total += part[k][cl];
    dw[col] = (T)total;
  }
}

template <typename T>
static bool launch_norm(const NormFwdArgs* f, const NormBwdArgs* b, int vec, int max_partial_rows, void* dw,
                        hipStream_t stream) {
  const int64_t rows = f ? f->rows : b->rows;
  const int H = f ? f->H : b->H;
  // Chunks of 64 lanes x vec elements in a row; W wavefronts share a row so that a lane keeps 4 chunks at most.
  const int chunks = (H + 64 * vec - 1) / (64 * vec);
  int W = 1;
  while (W < kNormWaves && (chunks + W - 1) / W > 4) W <<= 1;
  const int per_lane = (chunks + W - 1) / W;
  const bool wide = per_lane > 4;
  const int nch = per_lane <= 1 ? 1 : per_lane <= 2 ? 2 : 4;
  const int rows_per_wg = wide ? 1 : kNormWaves / W;
  int64_t blocks = (rows + rows_per_wg - 1) / rows_per_wg;
  if (blocks < 1) blocks = 1;
  // Forward: one short workgroup per pass over rows_per_wg rows, started in index order.  Backward: at most
  // 512 workgroups that stay (each sums its own dweight) and stride through the rows together.
  int grid = (int)(blocks < 512 ? blocks : 512);
  if (f) grid = (int)(blocks < (1 << 30) ? blocks : (1 << 30));
  if (b && grid > max_partial_rows) grid = max_partial_rows;
  if (grid < 1) return false;
  bool done = false;
#define QSSM_NORM_CASE(V, NCH, WW)                                                                                \
  if (!done && !wide && vec == V && nch == NCH && W == WW) {                                                      \
    if (f) hipLaunchKernelGGL((rmsnorm_fwd_kernel<T, V, NCH, WW>), dim3(grid), dim3(kNormThreads), 0, stream, *f); \
    else hipLaunchKernelGGL((rmsnorm_bwd_kernel<T, V, NCH, WW>), dim3(grid), dim3(kNormThreads),                   \
                            (size_t)H * sizeof(float), stream, *b);                                               \
    done = true;                                                                                                  \
  }
#define QSSM_NORM_VEC(V)                                                                                          \
  QSSM_NORM_CASE(V, 1, 1)                                                                                         \
  QSSM_NORM_CASE(V, 2, 1)                                                                                         \
  QSSM_NORM_CASE(V, 4, 1)                                                                                         \
  QSSM_NORM_CASE(V, 4, 2)                                                                                         \
  QSSM_NORM_CASE(V, 4, 4)                                                                                         \
  QSSM_NORM_CASE(V, 4, 8)                                                                                         \
  if (!done && wide && vec == V) {                                                                                \
    if (f) hipLaunchKernelGGL((rmsnorm_fwd_wide_kernel<T, V>), dim3(grid), dim3(kNormThreads), 0, stream, *f);     \
    else hipLaunchKernelGGL((rmsnorm_bwd_wide_kernel<T, V>), dim3(grid), dim3(kNormThreads), 0, stream, *b);       \
    done = true;                                                                                                  \
  }
  QSSM_NORM_VEC(4)
  QSSM_NORM_VEC(2)
  QSSM_NORM_VEC(1)
#undef QSSM_NORM_VEC
#undef QSSM_NORM_CASE
  if (!done) return false;
  if (b)
    hipLaunchKernelGGL((rmsnorm_dw_kernel<T>), dim3((H + 63) / 64), dim3(1024), 0, stream, b->partial, grid, H,
                       reinterpret_cast<T*>(dw));
  return true;
}

// Exactly one of f, b is non-null; dw and max_partial_rows belong to the backward.  False if the
// storage type or vec is not built, or `partial` is too small for one launch.
bool launch_norm_any(int dtype, const NormFwdArgs* f, const NormBwdArgs* b, int vec, int max_partial_rows, void* dw,
                     hipStream_t stream) {
  if (dtype == QSSM_F32) return launch_norm<float>(f, b, vec, max_partial_rows, dw, stream);
  if (dtype == QSSM_F16) return launch_norm<f16_t>(f, b, vec, max_partial_rows, dw, stream);
  if (dtype == QSSM_BF16) return launch_norm<bf16_t>(f, b, vec, max_partial_rows, dw, stream);
  return false;
}

}  // namespace qssm
