// Forward gated linear scan for gfx950: h(t) = a(t) h(t-1) + b(t) x(t), y(t) = c(t) h(t).
//
// One launch, one pass: x, a, b, c are read once and y is written once.  It takes the place
// of the reference's three forward launches and their N-sized fp32 scratch
// (ssm_local_forward_kernel / ssm_forward_carry_scan_kernel / ssm_fwd_apply_kernel,
// quick_ssm/triton_forwards.py:33-131) and of the y = c*h multiply and cast that follow them
// (quick_ssm/scan_interface.py:104-107).  The affine-map composition is the reference's
// combine_fn (quick_ssm/triton_forwards.py:26-30): (aL,xL) then (aR,xR) = (aR*aL, aR*xL+xR).
#include "scan_common.h"

namespace qssm {

template <typename Tin, typename Tout, int VEC, int T, int NTH>
__global__ void __launch_bounds__(NTH) scan_fwd_kernel(const FwdArgs p) {
  extern __shared__ float lds[];
  const Geometry& g = p.g;
  const int G = 1 << g.g_log2;
  const int NG = NTH >> g.g_log2;
  const int cols = G * VEC;
  const int R = g.cluster;
  float* sA = lds;                       // [NTH * VEC] per-lane map, multiplier
  float* sX = sA + NTH * VEC;            // [NTH * VEC] per-lane map, offset
  float* sPA = sX + NTH * VEC;           // [(R-1) * cols] maps of the earlier tiles of the cluster
  float* sPX = sPA + (R - 1) * cols;
  float* sH = sPX + (R - 1) * cols;      // [cols] state entering the tile
  int* sSeg = reinterpret_cast<int*>(sH + cols);

  const int tid = threadIdx.x;
  const int chain = blockIdx.x % g.n_chains;

  // ---- claim a tile of this chain, in time order -------------------------------------------
  int seg = 0;
  if (g.n_seg > 1) {
    if (tid == 0) *sSeg = (int)claim_ticket(g.tickets, chain, g.epoch);
    __syncthreads();
    seg = __builtin_amdgcn_readfirstlane(*sSeg);
    if ((unsigned)seg >= (unsigned)g.n_seg) {  // more claims than tiles: the epoch was reused
      if (tid == 0) raise_status(g.status, 2);
      return;
    }
  }

  const int bi = chain / g.n_strips;
  const int strip = chain - bi * g.n_strips;
  const int j = tid >> g.g_log2;         // lane group = time sub-segment
  const int dl = (tid & (G - 1)) * VEC;  // first column of this lane inside the strip
  const int d = strip * cols + dl;
  const bool dok = d < g.D;
  const int t_tile = seg * g.seg_len;
  const int t0 = t_tile + j * T;

  // Workgroup-uniform base of the tile in every operand, plus a 32-bit per-lane byte offset.
  const int64_t col0 = (int64_t)strip * cols;
  const char* xb = (const char*)p.x + ((int64_t)bi * p.x_sb + (int64_t)t_tile * p.x_sl + col0) * (int64_t)sizeof(Tin);
  const char* ab = (const char*)p.a + ((int64_t)bi * p.a_sb + (int64_t)t_tile * p.a_sl + col0) * (int64_t)sizeof(Tin);
  const char* bb = (const char*)p.b + ((int64_t)bi * p.b_sb + (int64_t)t_tile * p.b_sl + col0) * (int64_t)sizeof(Tin);
  const char* cb = (const char*)p.c + ((int64_t)bi * p.c_sb + (int64_t)t_tile * p.c_sl + col0) * (int64_t)sizeof(Tin);
  const uint32_t xo = (uint32_t)((j * T * (int)p.x_sl + dl) * (int)sizeof(Tin)), xs = (uint32_t)p.x_sl * sizeof(Tin);
  const uint32_t ao = (uint32_t)((j * T * (int)p.a_sl + dl) * (int)sizeof(Tin)), as = (uint32_t)p.a_sl * sizeof(Tin);
  const uint32_t bo = (uint32_t)((j * T * (int)p.b_sl + dl) * (int)sizeof(Tin)), bs = (uint32_t)p.b_sl * sizeof(Tin);
  const uint32_t co = (uint32_t)((j * T * (int)p.c_sl + dl) * (int)sizeof(Tin)), cs = (uint32_t)p.c_sl * sizeof(Tin);
  const bool want_y = p.y != nullptr;
  const bool has_c = want_y && p.c != nullptr;

  // ---- issue every load of the tile before touching any of them ------------------------------
  Words<Tin, VEC> rx[T], ra[T], rb[T], rc[T];
  const bool tile_full = (t_tile + g.seg_len <= g.L) && ((strip + 1) * cols <= g.D);
  if (tile_full) {
#pragma unroll
    for (int i = 0; i < T; ++i) {
      ra[i] = load_stream<Tin, VEC>(ab, ao + i * as);
      rb[i] = load_stream<Tin, VEC>(bb, bo + i * bs);
      rx[i] = load_stream<Tin, VEC>(xb, xo + i * xs);
    }
    if (has_c) {
#pragma unroll
      for (int i = 0; i < T; ++i) rc[i] = load_stream<Tin, VEC>(cb, co + i * cs);
    }
  } else {
    // Steps past L and columns past D act as the identity map (a = 1, b*x = 0).
#pragma unroll
    for (int i = 0; i < T; ++i) {
      ra[i] = fill_words<Tin, VEC>(true);
      rb[i] = fill_words<Tin, VEC>(false);
      rx[i] = fill_words<Tin, VEC>(false);
      rc[i] = fill_words<Tin, VEC>(false);
    }
#pragma unroll
    for (int i = 0; i < T; ++i) {
      if (dok && t0 + i < g.L) {
        ra[i] = load_stream<Tin, VEC>(ab, ao + i * as);
        rb[i] = load_stream<Tin, VEC>(bb, bo + i * bs);
        rx[i] = load_stream<Tin, VEC>(xb, xo + i * xs);
        if (has_c) rc[i] = load_stream<Tin, VEC>(cb, co + i * cs);
      }
    }
  }

  // ---- sweep 1: fold this lane's T steps into one affine map ---------------------------------
  float A[VEC], X[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) { A[v] = 1.0f; X[v] = 0.0f; }
#pragma unroll
  for (int i = 0; i < T; ++i) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float av = elem(ra[i], v);
      X[v] = av * X[v] + elem(rb[i], v) * elem(rx[i], v);
      A[v] = av * A[v];
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    sA[tid * VEC + v] = A[v];
    sX[tid * VEC + v] = X[v];
  }
#pragma unroll
  for (int i = 0; i < T; ++i) { forget(ra[i]); forget(rb[i]); forget(rx[i]); }
  __syncthreads();

  // ---- compose the maps of the lane groups before this one ------------------------------------
  float Ap[VEC], Xp[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) { Ap[v] = 1.0f; Xp[v] = 0.0f; }
  for (int k = 0; k < j; ++k) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float ak = sA[k * cols + dl + v];
      Xp[v] = ak * Xp[v] + sX[k * cols + dl + v];
      Ap[v] = ak * Ap[v];
    }
  }

  // ---- state entering the tile ------------------------------------------------------------------
  float hin[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) hin[v] = 0.0f;
  if (g.n_seg > 1) {
    const int s = seg / R;       // cluster of this tile
    const int m = seg - s * R;   // tiles of the cluster before this one
    const bool edge = (j == NG - 1);  // the last lane group holds the tile's total map
    float At[VEC], Xt[VEC];
    if (edge) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) { At[v] = A[v] * Ap[v]; Xt[v] = A[v] * Xp[v] + X[v]; }
      // Later tiles of the cluster need this tile's map; it depends on nothing, so it goes out first.
      if (dok && m + 1 < R && seg + 1 < g.n_seg) {
        unsigned long long* mw = g.maps + (((int64_t)chain * g.n_seg + seg) * cols + dl) * 2;
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          word_publish(mw + 2 * v, g.epoch, At[v]);
          word_publish(mw + 2 * v + 1, g.epoch, Xt[v]);
        }
      }
    }
    if (m > 0) {
      // Lane group j fetches the maps of the earlier tiles j, j+NG, ... of the cluster.
      for (int i = j; i < m; i += NG) {
        if (dok) {
          float w[2 * VEC];
          const unsigned long long* mw = g.maps + (((int64_t)chain * g.n_seg + (seg - m + i)) * cols + dl) * 2;
          if (!words_wait<2 * VEC>(mw, g.epoch, w)) raise_status(g.status, 1);
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            sPA[i * cols + dl + v] = w[2 * v];
            sPX[i * cols + dl + v] = w[2 * v + 1];
          }
        }
      }
      __syncthreads();
    }
    if (edge) {
      // The one serial hop: the state the previous cluster ended with.
      if (dok && s > 0) {
        const unsigned long long* sw = g.states + ((int64_t)chain * g.n_super + (s - 1)) * cols + dl;
        if (!words_wait<VEC>(sw, g.epoch, hin)) raise_status(g.status, 1);
      }
      for (int i = 0; i < m; ++i) {
#pragma unroll
        for (int v = 0; v < VEC; ++v) hin[v] = sPA[i * cols + dl + v] * hin[v] + sPX[i * cols + dl + v];
      }
      if (dok && m == R - 1 && s + 1 < g.n_super) {
        unsigned long long* sw = g.states + ((int64_t)chain * g.n_super + s) * cols + dl;
#pragma unroll
        for (int v = 0; v < VEC; ++v) word_publish(sw + v, g.epoch, At[v] * hin[v] + Xt[v]);
      }
#pragma unroll
      for (int v = 0; v < VEC; ++v) sH[dl + v] = hin[v];
    }
    __syncthreads();
#pragma unroll
    for (int v = 0; v < VEC; ++v) hin[v] = sH[dl + v];
  }

  float h[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) h[v] = Ap[v] * hin[v] + Xp[v];

  // ---- keep h(t0-1) where the backward will want it ---------------------------------------------
  if (p.ckpt != nullptr && dok && t0 < g.L && (t0 % g.ckpt_stride) == 0) {
    Pack<float, VEC> hv;
#pragma unroll
    for (int v = 0; v < VEC; ++v) hv.v[v] = h[v];
    store_pack<float, VEC>(p.ckpt + ((int64_t)bi * g.n_ckpt + t0 / g.ckpt_stride) * g.D + d, hv);
  }
  if (!want_y && p.h_out == nullptr) return;

  // ---- sweep 2: the recurrence proper, from the true carry-in -----------------------------------
  char* yb = (char*)p.y + ((int64_t)bi * p.y_sb + (int64_t)t_tile * p.y_sl + col0) * (int64_t)sizeof(Tout);
  char* hb = (char*)p.h_out + ((int64_t)bi * p.h_sb + (int64_t)t_tile * p.h_sl + col0) * (int64_t)sizeof(float);
  const uint32_t yo = (uint32_t)((j * T * (int)p.y_sl + dl) * (int)sizeof(Tout)), ys = (uint32_t)p.y_sl * sizeof(Tout);
  const uint32_t ho = (uint32_t)((j * T * (int)p.h_sl + dl) * (int)sizeof(float)), hs = (uint32_t)p.h_sl * sizeof(float);
#pragma unroll
  for (int i = 0; i < T; ++i) {
    float yv[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      h[v] = elem(ra[i], v) * h[v] + elem(rb[i], v) * elem(rx[i], v);
      yv[v] = has_c ? elem(rc[i], v) * h[v] : h[v];
    }
    if (tile_full || (dok && t0 + i < g.L)) {
      if (want_y) store_stream<Tout, VEC>(yb, yo + i * ys, yv);
      if (p.h_out != nullptr) store_stream<float, VEC>(hb, ho + i * hs, h);
    }
    // Keep each step's conversions next to their use: hoisting them all above the recurrence
    // would hold an fp32 copy of the whole tile in registers.
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <typename Tin, typename Tout>
static bool launch_fwd(const FwdArgs& args, int vec, int steps, int threads, dim3 grid, size_t lds,
                       hipStream_t stream) {
#define QSSM_FWD_CASE(V, S, N)                                                                        \
  if (vec == V && steps == S && threads == N) {                                                       \
    hipLaunchKernelGGL((scan_fwd_kernel<Tin, Tout, V, S, N>), grid, dim3(N), lds, stream, args);       \
    return true;                                                                                      \
  }
  QSSM_FWD_CASE(1, 4, 256)
  QSSM_FWD_CASE(1, 8, 256)
  QSSM_FWD_CASE(2, 4, 256)
  QSSM_FWD_CASE(2, 8, 256)
  QSSM_FWD_CASE(4, 4, 256)
  QSSM_FWD_CASE(4, 8, 256)
  QSSM_FWD_CASE(2, 4, 512)
  QSSM_FWD_CASE(2, 8, 512)
  QSSM_FWD_CASE(4, 4, 512)
  QSSM_FWD_CASE(4, 8, 512)
  QSSM_FWD_CASE(2, 4, 1024)
  QSSM_FWD_CASE(2, 8, 1024)
  QSSM_FWD_CASE(4, 4, 1024)
  QSSM_FWD_CASE(4, 8, 1024)
#undef QSSM_FWD_CASE
  return false;
}

fwd_launch_fn find_fwd_launcher(int in_dtype, int out_dtype) {
  if (in_dtype == QSSM_F32 && out_dtype == QSSM_F32) return launch_fwd<float, float>;
  if (in_dtype == QSSM_F16 && out_dtype == QSSM_F16) return launch_fwd<f16_t, f16_t>;
  if (in_dtype == QSSM_BF16 && out_dtype == QSSM_BF16) return launch_fwd<bf16_t, bf16_t>;
  if (in_dtype == QSSM_F16 && out_dtype == QSSM_F32) return launch_fwd<f16_t, float>;
  if (in_dtype == QSSM_BF16 && out_dtype == QSSM_F32) return launch_fwd<bf16_t, float>;
  return nullptr;
}

}  // namespace qssm
