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

template <typename Tin, typename Tout, int VEC, int T>
__global__ void __launch_bounds__(kThreads) scan_fwd_kernel(const FwdArgs p) {
  __shared__ float sA[kThreads * VEC];
  __shared__ float sX[kThreads * VEC];
  __shared__ float sHin[kThreads * VEC];
  __shared__ int sSeg;

  const Geometry& g = p.g;
  const int tid = threadIdx.x;
  const int chain = blockIdx.x % g.n_chains;

  // ---- claim a tile of this chain, in time order -------------------------------------------
  int seg = 0;
  if (g.n_seg > 1) {
    if (tid == 0) sSeg = (int)claim_ticket(g.tickets, chain, g.n_seg);
    __syncthreads();
    seg = sSeg;
    if (seg >= g.n_seg) {  // workspace was not zero on entry
      if (tid == 0) raise_status(g.status, 2);
      return;
    }
  }

  const int bi = chain / g.n_strips;
  const int strip = chain - bi * g.n_strips;
  const int G = 1 << g.g_log2;
  const int NG = kThreads >> g.g_log2;
  const int j = tid >> g.g_log2;        // lane group = time sub-segment
  const int dl = (tid & (G - 1)) * VEC;  // first column of this lane inside the strip
  const int cols = G * VEC;
  const int d = strip * cols + dl;
  const bool dok = d < g.D;
  const int t_tile = seg * g.seg_len;
  const int t0 = t_tile + j * T;

  const Tin* xp = (const Tin*)p.x + (int64_t)bi * p.x_sb + (int64_t)t0 * p.x_sl + d;
  const Tin* ap = (const Tin*)p.a + (int64_t)bi * p.a_sb + (int64_t)t0 * p.a_sl + d;
  const Tin* bp = (const Tin*)p.b + (int64_t)bi * p.b_sb + (int64_t)t0 * p.b_sl + d;
  const Tin* cp = (const Tin*)p.c + (int64_t)bi * p.c_sb + (int64_t)t0 * p.c_sl + d;
  const bool want_y = p.y != nullptr;
  const bool has_c = want_y && p.c != nullptr;

  // ---- issue every load of the tile before touching any of them ------------------------------
  Pack<Tin, VEC> rx[T], ra[T], rb[T], rc[T];
  const bool tile_full = (t_tile + g.seg_len <= g.L) && ((strip + 1) * cols <= g.D);
  if (tile_full) {
#pragma unroll
    for (int i = 0; i < T; ++i) {
      ra[i] = load_pack<Tin, VEC>(ap + (int64_t)i * p.a_sl);
      rb[i] = load_pack<Tin, VEC>(bp + (int64_t)i * p.b_sl);
      rx[i] = load_pack<Tin, VEC>(xp + (int64_t)i * p.x_sl);
    }
    if (has_c) {
#pragma unroll
      for (int i = 0; i < T; ++i) rc[i] = load_pack<Tin, VEC>(cp + (int64_t)i * p.c_sl);
    }
  } else {
    // Steps past L and columns past D act as the identity map (a = 1, b*x = 0).
#pragma unroll
    for (int i = 0; i < T; ++i) {
      ra[i] = fill_pack<Tin, VEC>(1.0f);
      rb[i] = fill_pack<Tin, VEC>(0.0f);
      rx[i] = fill_pack<Tin, VEC>(0.0f);
      rc[i] = fill_pack<Tin, VEC>(0.0f);
    }
#pragma unroll
    for (int i = 0; i < T; ++i) {
      if (dok && t0 + i < g.L) {
        ra[i] = load_pack<Tin, VEC>(ap + (int64_t)i * p.a_sl);
        rb[i] = load_pack<Tin, VEC>(bp + (int64_t)i * p.b_sl);
        rx[i] = load_pack<Tin, VEC>(xp + (int64_t)i * p.x_sl);
        if (has_c) rc[i] = load_pack<Tin, VEC>(cp + (int64_t)i * p.c_sl);
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
      const float av = to_f32(ra[i].v[v]);
      X[v] = av * X[v] + to_f32(rb[i].v[v]) * to_f32(rx[i].v[v]);
      A[v] = av * A[v];
    }
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    sA[tid * VEC + v] = A[v];
    sX[tid * VEC + v] = X[v];
  }
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

  // ---- chain: the last lane group owns the tile's total map and talks to the neighbours -------
  if (j == NG - 1) {
    unsigned long long* cw = g.carry + ((int64_t)chain * g.n_seg + seg) * cols + dl;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      float hin = 0.0f;
      if (dok) {
        if (seg > 0 && !carry_consume(cw - cols + v, &hin)) raise_status(g.status, 1);
        if (seg + 1 < g.n_seg) {
          const float atot = A[v] * Ap[v];
          const float xtot = A[v] * Xp[v] + X[v];
          carry_publish(cw + v, atot * hin + xtot);
        }
      }
      sHin[dl + v] = hin;
    }
  }
  __syncthreads();

  float h[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) h[v] = Ap[v] * sHin[dl + v] + Xp[v];

  // ---- keep h(t0-1) where the backward will want it ---------------------------------------------
  if (p.ckpt != nullptr && dok && t0 < g.L && (t0 % g.ckpt_stride) == 0) {
    Pack<float, VEC> hv;
#pragma unroll
    for (int v = 0; v < VEC; ++v) hv.v[v] = h[v];
    store_pack<float, VEC>(p.ckpt + ((int64_t)bi * g.n_ckpt + t0 / g.ckpt_stride) * g.D + d, hv);
  }
  if (!want_y && p.h_out == nullptr) return;

  // ---- sweep 2: the recurrence proper, from the true carry-in -----------------------------------
  Tout* yp = (Tout*)p.y + (int64_t)bi * p.y_sb + (int64_t)t0 * p.y_sl + d;
  float* hp = p.h_out + (int64_t)bi * p.h_sb + (int64_t)t0 * p.h_sl + d;
#pragma unroll
  for (int i = 0; i < T; ++i) {
    Pack<Tout, VEC> yv;
    Pack<float, VEC> hv;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      h[v] = to_f32(ra[i].v[v]) * h[v] + to_f32(rb[i].v[v]) * to_f32(rx[i].v[v]);
      hv.v[v] = h[v];
      yv.v[v] = (Tout)(has_c ? to_f32(rc[i].v[v]) * h[v] : h[v]);
    }
    if (tile_full || (dok && t0 + i < g.L)) {
      if (want_y) store_pack<Tout, VEC>(yp + (int64_t)i * p.y_sl, yv);
      if (p.h_out != nullptr) store_pack<float, VEC>(hp + (int64_t)i * p.h_sl, hv);
    }
  }
}

template <typename Tin, typename Tout>
static void launch_fwd(const FwdArgs& args, int vec, int steps, dim3 grid, hipStream_t stream) {
#define QSSM_FWD_CASE(V, S)                                                              \
  if (vec == V && steps == S) {                                                          \
    hipLaunchKernelGGL((scan_fwd_kernel<Tin, Tout, V, S>), grid, dim3(kThreads), 0, stream, args); \
    return;                                                                              \
  }
  QSSM_FWD_CASE(1, 4)
  QSSM_FWD_CASE(1, 8)
  QSSM_FWD_CASE(2, 4)
  QSSM_FWD_CASE(2, 8)
  QSSM_FWD_CASE(4, 4)
  QSSM_FWD_CASE(4, 8)
#undef QSSM_FWD_CASE
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
