// Backward gated linear scan for gfx950.
//
//   dH(t) = c(t) dy(t) + a(t+1) dH(t+1),  dH(L) = 0
//   dx = b dH,  db = x dH,  da(t) = h(t-1) dH(t),  dc = dy h
//
// One launch, one reverse-time pass: x, a, b, c, dy are read once, dx, da, db, dc are written
// once, and h is rebuilt inside each tile from the fp32 state saved every `ckpt_stride` steps
// by the forward (or read from a full fp32 h when the caller kept one).  It takes the place of
// the reference's forward re-run plus its three backward launches and their scratch
// (quick_ssm/scan_interface.py:133-140; ssm_local_backward_kernel /
// ssm_backward_carry_scan_kernel / ssm_bwd_apply_kernel, quick_ssm/triton_backwards.py:32-165).
//
// The reverse recurrence is carried as E(t) = a(t) * dH(t) (what naive_backward_3d calls
// dh_next, quick_ssm/naive_baseline.py:135), so that dH(t) = c(t) dy(t) + E(t+1) and
// E(t) = a(t) * (c(t) dy(t) + E(t+1)): each step's multiplier is its own a(t), and no a(t+1)
// has to be fetched across a tile edge (the reference kernel loads the shifted a,
// triton_backwards.py:62-66).  Over a run of steps the map E_in -> E_out is affine with the same
// multiplier prod a(t) as the forward map, so one product serves both directions.
#include "scan_common.h"

namespace qssm {

template <typename Tin, typename Tout, int VEC, int T>
__global__ void __launch_bounds__(kThreads) scan_bwd_kernel(const BwdArgs p) {
  __shared__ float sA[kThreads * VEC];
  __shared__ float sXf[kThreads * VEC];
  __shared__ float sXe[kThreads * VEC];
  __shared__ float sEin[kThreads * VEC];
  __shared__ int sSeg;

  const Geometry& g = p.g;
  const int tid = threadIdx.x;
  const int chain = blockIdx.x % g.n_chains;

  // ---- claim a tile of this chain, last tile in time first -----------------------------------
  int seg = 0;
  if (g.n_seg > 1) {
    if (tid == 0) sSeg = (int)claim_ticket(g.tickets, chain, g.n_seg);
    __syncthreads();
    const int tk = sSeg;
    if (tk >= g.n_seg) {  // workspace was not zero on entry
      if (tid == 0) raise_status(g.status, 2);
      return;
    }
    seg = g.n_seg - 1 - tk;
  }

  const int bi = chain / g.n_strips;
  const int strip = chain - bi * g.n_strips;
  const int G = 1 << g.g_log2;
  const int NG = kThreads >> g.g_log2;
  const int j = tid >> g.g_log2;
  const int dl = (tid & (G - 1)) * VEC;
  const int cols = G * VEC;
  const int d = strip * cols + dl;
  const bool dok = d < g.D;
  const int t_tile = seg * g.seg_len;
  const int t0 = t_tile + j * T;
  const bool have_h = p.h != nullptr;

  const Tin* xp = (const Tin*)p.x + (int64_t)bi * p.x_sb + (int64_t)t0 * p.x_sl + d;
  const Tin* ap = (const Tin*)p.a + (int64_t)bi * p.a_sb + (int64_t)t0 * p.a_sl + d;
  const Tin* bp = (const Tin*)p.b + (int64_t)bi * p.b_sb + (int64_t)t0 * p.b_sl + d;
  const Tin* cp = (const Tin*)p.c + (int64_t)bi * p.c_sb + (int64_t)t0 * p.c_sl + d;
  const Tout* gp = (const Tout*)p.dy + (int64_t)bi * p.dy_sb + (int64_t)t0 * p.dy_sl + d;
  const float* hp = p.h + (int64_t)bi * p.h_sb + (int64_t)t0 * p.h_sl + d;

  // ---- issue every load of the tile before touching any of them ------------------------------
  Pack<Tin, VEC> rx[T], ra[T], rb[T], rc[T];
  Pack<Tout, VEC> rg[T];
  float hs[T][VEC];   // h(t0 + i)
  float hprev[VEC];   // h(t0 - 1), then the tile-level state for the rebuild
  const bool tile_full = (t_tile + g.seg_len <= g.L) && ((strip + 1) * cols <= g.D);
  if (tile_full) {
#pragma unroll
    for (int i = 0; i < T; ++i) {
      ra[i] = load_pack<Tin, VEC>(ap + (int64_t)i * p.a_sl);
      rc[i] = load_pack<Tin, VEC>(cp + (int64_t)i * p.c_sl);
      rg[i] = load_pack<Tout, VEC>(gp + (int64_t)i * p.dy_sl);
    }
#pragma unroll
    for (int i = 0; i < T; ++i) {
      rb[i] = load_pack<Tin, VEC>(bp + (int64_t)i * p.b_sl);
      rx[i] = load_pack<Tin, VEC>(xp + (int64_t)i * p.x_sl);
    }
  } else {
    // Steps past L and columns past D act as the identity map (a = 1, everything else 0).
#pragma unroll
    for (int i = 0; i < T; ++i) {
      ra[i] = fill_pack<Tin, VEC>(1.0f);
      rb[i] = fill_pack<Tin, VEC>(0.0f);
      rx[i] = fill_pack<Tin, VEC>(0.0f);
      rc[i] = fill_pack<Tin, VEC>(0.0f);
      rg[i] = fill_pack<Tout, VEC>(0.0f);
    }
#pragma unroll
    for (int i = 0; i < T; ++i) {
      if (dok && t0 + i < g.L) {
        ra[i] = load_pack<Tin, VEC>(ap + (int64_t)i * p.a_sl);
        rc[i] = load_pack<Tin, VEC>(cp + (int64_t)i * p.c_sl);
        rg[i] = load_pack<Tout, VEC>(gp + (int64_t)i * p.dy_sl);
        rb[i] = load_pack<Tin, VEC>(bp + (int64_t)i * p.b_sl);
        rx[i] = load_pack<Tin, VEC>(xp + (int64_t)i * p.x_sl);
      }
    }
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) hprev[v] = 0.0f;
  if (have_h) {
#pragma unroll
    for (int i = 0; i < T; ++i) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) hs[i][v] = 0.0f;
      if (dok && t0 + i < g.L) {
        const Pack<float, VEC> hv = load_pack<float, VEC>(hp + (int64_t)i * p.h_sl);
#pragma unroll
        for (int v = 0; v < VEC; ++v) hs[i][v] = hv.v[v];
      }
    }
    if (dok && t0 > 0 && t0 < g.L) {
      const Pack<float, VEC> hv = load_pack<float, VEC>(hp - p.h_sl);
#pragma unroll
      for (int v = 0; v < VEC; ++v) hprev[v] = hv.v[v];
    }
  } else if (dok && t_tile > 0) {
    // state at the tile's first step, saved by the forward
    const Pack<float, VEC> hv = load_pack<float, VEC>(
        p.ckpt + ((int64_t)bi * g.n_ckpt + t_tile / g.ckpt_stride) * g.D + d);
#pragma unroll
    for (int v = 0; v < VEC; ++v) hprev[v] = hv.v[v];
  }

  // ---- sweep 1: fold this lane's T steps into the forward and the reverse affine map ----------
  float A[VEC], Xf[VEC], Xe[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) { A[v] = 1.0f; Xf[v] = 0.0f; Xe[v] = 0.0f; }
#pragma unroll
  for (int i = 0; i < T; ++i) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float av = to_f32(ra[i].v[v]);
      Xf[v] = av * Xf[v] + to_f32(rb[i].v[v]) * to_f32(rx[i].v[v]);
      A[v] = av * A[v];
    }
  }
#pragma unroll
  for (int i = T - 1; i >= 0; --i) {
#pragma unroll
    for (int v = 0; v < VEC; ++v)
      Xe[v] = to_f32(ra[i].v[v]) * (to_f32(rc[i].v[v]) * to_f32(rg[i].v[v]) + Xe[v]);
  }
#pragma unroll
  for (int v = 0; v < VEC; ++v) {
    sA[tid * VEC + v] = A[v];
    sXf[tid * VEC + v] = Xf[v];
    sXe[tid * VEC + v] = Xe[v];
  }
  __syncthreads();

  // ---- compose: groups before this one (forward state), groups after it (reverse carry) --------
  float Ap[VEC], Xp[VEC], As[VEC], Xs[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) { Ap[v] = 1.0f; Xp[v] = 0.0f; As[v] = 1.0f; Xs[v] = 0.0f; }
  if (!have_h) {
    for (int k = 0; k < j; ++k) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float ak = sA[k * cols + dl + v];
        Xp[v] = ak * Xp[v] + sXf[k * cols + dl + v];
        Ap[v] = ak * Ap[v];
      }
    }
  }
  for (int k = NG - 1; k > j; --k) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float ak = sA[k * cols + dl + v];
      Xs[v] = ak * Xs[v] + sXe[k * cols + dl + v];
      As[v] = ak * As[v];
    }
  }

  // ---- chain: the first lane group owns the tile's total reverse map ---------------------------
  if (j == 0) {
    unsigned long long* cw = g.carry + ((int64_t)chain * g.n_seg + seg) * cols + dl;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      float ein = 0.0f;
      if (dok) {
        if (seg + 1 < g.n_seg && !carry_consume(cw + cols + v, &ein)) raise_status(g.status, 1);
        if (seg > 0) {
          const float atot = A[v] * As[v];
          const float xtot = A[v] * Xs[v] + Xe[v];
          carry_publish(cw + v, atot * ein + xtot);
        }
      }
      sEin[dl + v] = ein;
    }
  }
  __syncthreads();

  float E[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) E[v] = As[v] * sEin[dl + v] + Xs[v];

  // ---- sweep 2: rebuild h over this lane's steps -------------------------------------------------
  if (!have_h) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) hprev[v] = Ap[v] * hprev[v] + Xp[v];
#pragma unroll
    for (int i = 0; i < T; ++i) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float hm = (i == 0) ? hprev[v] : hs[i - 1][v];
        hs[i][v] = to_f32(ra[i].v[v]) * hm + to_f32(rb[i].v[v]) * to_f32(rx[i].v[v]);
      }
    }
  }

  // ---- sweep 3: reverse recurrence and the four gradients ---------------------------------------
  Tin* dxp = (Tin*)p.dx + (int64_t)bi * p.dx_sb + (int64_t)t0 * p.dx_sl + d;
  Tin* dap = (Tin*)p.da + (int64_t)bi * p.da_sb + (int64_t)t0 * p.da_sl + d;
  Tin* dbp = (Tin*)p.db + (int64_t)bi * p.db_sb + (int64_t)t0 * p.db_sl + d;
  Tin* dcp = (Tin*)p.dc + (int64_t)bi * p.dc_sb + (int64_t)t0 * p.dc_sl + d;
#pragma unroll
  for (int i = T - 1; i >= 0; --i) {
    Pack<Tin, VEC> vdx, vda, vdb, vdc;
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float gy = to_f32(rg[i].v[v]);
      const float dH = to_f32(rc[i].v[v]) * gy + E[v];
      const float hm = (i == 0) ? hprev[v] : hs[i - 1][v];
      vdc.v[v] = (Tin)(gy * hs[i][v]);
      vdx.v[v] = (Tin)(to_f32(rb[i].v[v]) * dH);
      vdb.v[v] = (Tin)(to_f32(rx[i].v[v]) * dH);
      vda.v[v] = (Tin)(hm * dH);
      E[v] = to_f32(ra[i].v[v]) * dH;
    }
    if (tile_full || (dok && t0 + i < g.L)) {
      if (p.dx != nullptr) store_pack<Tin, VEC>(dxp + (int64_t)i * p.dx_sl, vdx);
      if (p.da != nullptr) store_pack<Tin, VEC>(dap + (int64_t)i * p.da_sl, vda);
      if (p.db != nullptr) store_pack<Tin, VEC>(dbp + (int64_t)i * p.db_sl, vdb);
      if (p.dc != nullptr) store_pack<Tin, VEC>(dcp + (int64_t)i * p.dc_sl, vdc);
    }
  }
}

template <typename Tin, typename Tout>
static void launch_bwd(const BwdArgs& args, int vec, int steps, dim3 grid, hipStream_t stream) {
#define QSSM_BWD_CASE(V, S)                                                              \
  if (vec == V && steps == S) {                                                          \
    hipLaunchKernelGGL((scan_bwd_kernel<Tin, Tout, V, S>), grid, dim3(kThreads), 0, stream, args); \
    return;                                                                              \
  }
  QSSM_BWD_CASE(1, 4)
  QSSM_BWD_CASE(1, 8)
  QSSM_BWD_CASE(2, 4)
  QSSM_BWD_CASE(2, 8)
  QSSM_BWD_CASE(4, 4)
  QSSM_BWD_CASE(4, 8)
#undef QSSM_BWD_CASE
}

bwd_launch_fn find_bwd_launcher(int in_dtype, int out_dtype) {
  if (in_dtype == QSSM_F32 && out_dtype == QSSM_F32) return launch_bwd<float, float>;
  if (in_dtype == QSSM_F16 && out_dtype == QSSM_F16) return launch_bwd<f16_t, f16_t>;
  if (in_dtype == QSSM_BF16 && out_dtype == QSSM_BF16) return launch_bwd<bf16_t, bf16_t>;
  if (in_dtype == QSSM_F16 && out_dtype == QSSM_F32) return launch_bwd<f16_t, float>;
  if (in_dtype == QSSM_BF16 && out_dtype == QSSM_F32) return launch_bwd<bf16_t, float>;
  return nullptr;
}

}  // namespace qssm
