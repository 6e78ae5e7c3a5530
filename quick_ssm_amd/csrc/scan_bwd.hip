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
#include <type_traits>

#include "scan_common.h"

namespace qssm {

typedef __attribute__((address_space(1))) const void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// CLDS: c and dy are loaded straight into LDS (no destination registers) and read from there in the
// sweeps that use them: 32 VGPRs fewer across the tile's whole life, which is one more resident
// workgroup per SIMD.  Needs 64 lanes per row and 8 bytes per lane in both tensors, so that one
// wavefront-wide 16-byte-per-lane load covers two rows of the strip.  With 16-bit operands and fp32 dy (16 bytes
// per lane) only dy goes through LDS, every lane fetching its own piece, and c stays in registers: LDS has room
// for one 16-byte or two 8-byte operands at three workgroups per compute unit, and dy is the larger one.
//
// GATED: the operands are the SSM layer's projection outputs (quick_ssm/layers.py:76-88) and both the gate
// activations and their derivatives happen here: a = sigmoid(A_pre), b = sigmoid(D_pre) replace their
// pre-activations in registers, c = silu(Ca) * Cb is formed from two LDS-resident operands where it is used, and
// the last sweep turns the scan's gradients (rounded to the storage type, as the scan stores them) into the
// projections' gradients dA_pre = da a (1 - a), dB_in = dx, dD_pre = db b (1 - b),
// dCa = dc Cb s (1 + Ca (1 - s)), dCb = dc Ca s with s = sigmoid(Ca): no gradient of a, x, b, c ever exists in HBM.
//
// XLANE: rows of 16 lanes or fewer (a few columns of D), where a tile has 16 to 256 lane groups: their maps are
// combined, in both directions, by exchanges between the lanes of a wavefront instead of two walks through LDS.
//
// Tc is the type the layer rounds the gates' outputs and the scan's gradients to (its compute dtype): the projections'
// storage type, or a 16-bit type that only exists in registers when the projections are fp32.
template <typename Tin, typename Tout, int VEC, int T, int NTH, bool CLDS, bool GATED, bool XLANE, typename Tc = Tin>
__global__ void __launch_bounds__(NTH) scan_bwd_kernel(const BwdArgs p) {
  static_assert(!GATED || CLDS, "gated scan: Ca, Cb and dy through LDS");
  static_assert(GATED || std::is_same<Tc, Tin>::value, "a compute dtype of its own only means something to the gated scan");
  constexpr bool ROUND = !std::is_same<Tc, Tin>::value;   // gate outputs and scan gradients are rounded to a type narrower than their storage
  static_assert(!XLANE || (!CLDS && !GATED), "cross-lane fold: register-only operands");
  static_assert(!CLDS || (sizeof(Tin) * VEC == 8 && (sizeof(Tout) * VEC == 8 || sizeof(Tout) * VEC == 16) && T % 2 == 0),
                "LDS-resident c and dy: 8 bytes per lane (dy alone: 16), even step count");
  static_assert(!GATED || sizeof(Tout) * VEC == 8, "gated scan: dy at 8 bytes per lane");
  constexpr bool GW = CLDS && sizeof(Tout) * VEC == 16;   // dy alone in LDS, 16 bytes per lane
  constexpr bool CREG = !CLDS || GW;                       // c in registers
  extern __shared__ __align__(16) float lds[];
  const Geometry& g = p.g;
  const int G = 1 << g.g_log2;
  const int NG = NTH >> g.g_log2;
  const int cols = G * VEC;
  const int R = g.cluster;
  // Flag value of this launch: the host's, or one more than the launches counted in the control block.
  const unsigned epoch = g.launch_count != nullptr ? *g.launch_count + 1u : g.epoch;
  float* sA = lds;                       // [NTH * VEC] per-lane map, multiplier (both directions)
  float* sXf = sA + NTH * VEC;           // [NTH * VEC] forward offset
  float* sXe = sXf + NTH * VEC;          // [NTH * VEC] reverse offset
  float* sPA = sXe + NTH * VEC;          // [(R-1) * cols] reverse maps of the later tiles of the cluster
  float* sPX = sPA + (R - 1) * cols;
  float* sE = sPX + (R - 1) * cols;      // [cols] reverse carry entering the tile
  int* sSeg = reinterpret_cast<int*>(sE + cols);
  char* sC = reinterpret_cast<char*>(sSeg) + 16 + ((int)threadIdx.x >> 6) * (T * 512);  // CLDS: this wave's [T rows][512 bytes] of c
  // and of dy; with 16 bytes per lane dy has the block to itself: [T rows][64 lanes x 16 bytes] per wave
  char* sG = GW ? reinterpret_cast<char*>(sSeg) + 16 + ((int)threadIdx.x >> 6) * (T * 1024) : sC + (NTH / 64) * (T * 512);
  char* sC2 = sG + (NTH / 64) * (T * 512);                                 // GATED: and of Cb (sC then holds Ca)
  // Where step i of this lane sits in its wavefront's LDS block: the loads that fill it deposit 1024 bytes per
  // instruction in lane order, i.e. per pair of steps [group in wavefront][step parity][G * 8 bytes].
  const int lds_lane = (((int)threadIdx.x & 63) >> g.g_log2) * (G * 16) + ((int)threadIdx.x & (G - 1)) * 8;
  auto lds_row = [&](int i) { return (i >> 1) * 1024 + (i & 1) * (G * 8); };
  auto g_slot = [&](int i) -> char* {   // where dy of this lane's step i sits
    return GW ? sG + i * 1024 + ((int)threadIdx.x & 63) * 16 : sG + lds_row(i) + lds_lane;
  };

  const int tid = threadIdx.x;
  // Workgroups go to the eight XCDs in turn, so workgroup i runs on XCD i mod 8.  Chains are dealt out so that each
  // XCD gets a run of adjacent chains (the strips of one batch row, when there are eight of each) rather than
  // every eighth one: its workgroups then stream whole rows of few batch rows instead of one 512-byte column of
  // all of them, which its L2 and address translation reward.  All tiles of a chain still run on one XCD.
  int chain = blockIdx.x % g.n_chains;
  if ((g.n_chains & 7) == 0) chain = (chain & 7) * (g.n_chains >> 3) + (chain >> 3);

  // ---- claim a tile of this chain, last tile in time first -----------------------------------
  int seg = 0;
  if (g.n_seg > 1) {
    if (tid == 0) *sSeg = (int)claim_ticket(g.tickets, chain, g.n_seg);
    __syncthreads();
    const int tk = __builtin_amdgcn_readfirstlane(*sSeg);
    if ((unsigned)tk >= (unsigned)g.n_seg) {
      // The control block was not zero on entry: no tile can be claimed in order.  Every workgroup then poisons
      // the tile its index names (the grid has one workgroup per tile), so that the caller never reads memory
      // nobody wrote, and reports it.
      if (tid == 0) raise_status(g.status, 2);
      const int pseg = blockIdx.x / g.n_chains, pbi = chain / g.n_strips, pstrip = chain - pbi * g.n_strips;
      const int pd = pstrip * cols + (tid & (G - 1)) * VEC;
      float nanv[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) nanv[v] = __uint_as_float(0x7fc00000u);
      for (int i = 0; i < T; ++i) {
        const int t = pseg * g.seg_len + (tid >> g.g_log2) * T + i;
        if (pd < g.D && t < g.L) {
          if (p.dx != nullptr)
            store_stream<Tin, VEC>((char*)p.dx + ((int64_t)pbi * p.dx_sb + (int64_t)t * p.dx_sl + pd) * (int64_t)sizeof(Tin), 0u, nanv);
          if (p.da != nullptr)
            store_stream<Tin, VEC>((char*)p.da + ((int64_t)pbi * p.da_sb + (int64_t)t * p.da_sl + pd) * (int64_t)sizeof(Tin), 0u, nanv);
          if (p.db != nullptr)
            store_stream<Tin, VEC>((char*)p.db + ((int64_t)pbi * p.db_sb + (int64_t)t * p.db_sl + pd) * (int64_t)sizeof(Tin), 0u, nanv);
          if (p.dc != nullptr)
            store_stream<Tin, VEC>((char*)p.dc + ((int64_t)pbi * p.dc_sb + (int64_t)t * p.dc_sl + pd) * (int64_t)sizeof(Tin), 0u, nanv);
          if (GATED && p.dc2 != nullptr)
            store_stream<Tin, VEC>((char*)p.dc2 + ((int64_t)pbi * p.dc2_sb + (int64_t)t * p.dc2_sl + pd) * (int64_t)sizeof(Tin), 0u, nanv);
        }
      }
      if (p.dh_init != nullptr && pseg == 0 && (tid >> g.g_log2) == 0 && pd < g.D)
        store_stream<float, VEC>((char*)p.dh_init + ((int64_t)pbi * g.D + pd) * (int64_t)sizeof(float), 0u, nanv);
      return;
    }
    seg = g.n_seg - 1 - tk;
  }

  const int bi = chain / g.n_strips;
  const int strip = chain - bi * g.n_strips;
  const int j = tid >> g.g_log2;
  const int dl = (tid & (G - 1)) * VEC;
  const int d = strip * cols + dl;
  const bool dok = d < g.D;
  const int t_tile = seg * g.seg_len;
  const int t0 = t_tile + j * T;
  const bool have_h = p.h != nullptr;

  const int64_t col0 = (int64_t)strip * cols;
  const char* xb = (const char*)p.x + ((int64_t)bi * p.x_sb + (int64_t)t_tile * p.x_sl + col0) * (int64_t)sizeof(Tin);
  const char* ab = (const char*)p.a + ((int64_t)bi * p.a_sb + (int64_t)t_tile * p.a_sl + col0) * (int64_t)sizeof(Tin);
  const char* bb = (const char*)p.b + ((int64_t)bi * p.b_sb + (int64_t)t_tile * p.b_sl + col0) * (int64_t)sizeof(Tin);
  const char* cb = (const char*)p.c + ((int64_t)bi * p.c_sb + (int64_t)t_tile * p.c_sl + col0) * (int64_t)sizeof(Tin);
  const char* gb = (const char*)p.dy + ((int64_t)bi * p.dy_sb + (int64_t)t_tile * p.dy_sl + col0) * (int64_t)sizeof(Tout);
  const uint32_t xo = (uint32_t)((j * T * (int)p.x_sl + dl) * (int)sizeof(Tin)), xs = (uint32_t)p.x_sl * sizeof(Tin);
  const uint32_t ao = (uint32_t)((j * T * (int)p.a_sl + dl) * (int)sizeof(Tin)), as = (uint32_t)p.a_sl * sizeof(Tin);
  const uint32_t bo = (uint32_t)((j * T * (int)p.b_sl + dl) * (int)sizeof(Tin)), bs = (uint32_t)p.b_sl * sizeof(Tin);
  const uint32_t co = (uint32_t)((j * T * (int)p.c_sl + dl) * (int)sizeof(Tin)), cs = (uint32_t)p.c_sl * sizeof(Tin);
  const uint32_t go = (uint32_t)((j * T * (int)p.dy_sl + dl) * (int)sizeof(Tout)), gs = (uint32_t)p.dy_sl * sizeof(Tout);
  const char* c2b = GATED ? (const char*)p.c2 + ((int64_t)bi * p.c2_sb + (int64_t)t_tile * p.c2_sl + col0) * (int64_t)sizeof(Tin) : nullptr;
  const uint32_t c2o = GATED ? (uint32_t)((j * T * (int)p.c2_sl + dl) * (int)sizeof(Tin)) : 0u, c2s = GATED ? (uint32_t)p.c2_sl * sizeof(Tin) : 0u;
  const float* hp = p.h + (int64_t)bi * p.h_sb + (int64_t)t0 * p.h_sl + d;

  // ---- ask for the neighbours' words first: they are looked at once the answers are back ------
  const bool multi = g.n_seg > 1;
  const int s = seg / R;                                     // cluster of this tile
  const int m = seg - s * R;                                 // tiles of the cluster before this one
  const int last = ((s + 1) * R < g.n_seg ? (s + 1) * R : g.n_seg) - 1;
  const int cnt = last - seg;                                // tiles of the cluster after this one
  const bool edge = (j == 0);  // the first lane group holds the tile's total reverse map
  const int lane = tid & (G - 1);  // position inside the lane group = position inside a word plane
  const unsigned long long* next_state = g.states + ((int64_t)chain * g.n_super + (s + 1)) * cols + lane;
  const bool want_state = multi && dok && edge && s + 1 < g.n_super;   // the first group fetches the next cluster's carry
  Peek<VEC> pk_state;
  pk_state.clear();
  if (want_state) pk_state.issue(next_state, G);

  // ---- issue every load of the tile before touching any of them ------------------------------
  Words<Tin, VEC> rx[T], ra[T], rb[T], rc[CREG ? T : 1];
  Words<Tout, VEC> rg[CLDS ? 1 : T];
  float hs[T][VEC];   // h(t0 + i)
  float hprev[VEC];   // h(t0 - 1); before the rebuild, the state at the tile's first step
  const bool tile_full = (t_tile + g.seg_len <= g.L) && ((strip + 1) * cols <= g.D);
  if (tile_full) {
    if (CLDS) {
      // register operands first, one tensor after the other (0.7 us of 211 faster than step by step on the headline
      // shape; c and dy ahead of them costs 6 us)
#pragma unroll
      for (int i = 0; i < T; ++i) ra[i] = load_stream<Tin, VEC>(ab, ao + i * as);
#pragma unroll
      for (int i = 0; i < T; ++i) rb[i] = load_stream<Tin, VEC>(bb, bo + i * bs);
#pragma unroll
      for (int i = 0; i < T; ++i) rx[i] = load_stream<Tin, VEC>(xb, xo + i * xs);
      if constexpr (GW) {
#pragma unroll
        for (int i = 0; i < T; ++i) rc[i] = load_stream<Tin, VEC>(cb, co + i * cs);
#pragma unroll
        for (int i = 0; i < T; ++i)
          __builtin_amdgcn_global_load_lds((global_ptr_t)(gb + go + i * gs), (lds_ptr_t)(sG + i * 1024), 16, 0, 2);
      } else {
      // 16 bytes per lane: the first half of a lane group's lanes fetches one row of the strip, the second half
      // the next one (64 lanes per row: a wavefront covers two rows of one group; 32: two rows of two groups)
      const int wl = tid & 63;
      const int half = (wl >> (g.g_log2 - 1)) & 1, piece = wl & ((G >> 1) - 1);
      const char* csrc = cb + (uint32_t)(j * T + half) * cs + (uint32_t)piece * 16u;
      const char* gsrc = gb + (uint32_t)(j * T + half) * gs + (uint32_t)piece * 16u;
      // one tensor after the other here as well (1.8 us of 211 on the headline shape against c and dy in turn)
#pragma unroll
      for (int k = 0; k < T / 2; ++k)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(csrc + (uint32_t)(2 * k) * cs), (lds_ptr_t)(sC + k * 1024), 16, 0, 2);
#pragma unroll
      for (int k = 0; k < T / 2; ++k)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(gsrc + (uint32_t)(2 * k) * gs), (lds_ptr_t)(sG + k * 1024), 16, 0, 2);
      if constexpr (GATED) {
        const char* c2src = c2b + (uint32_t)(j * T + half) * c2s + (uint32_t)piece * 16u;
#pragma unroll
        for (int k = 0; k < T / 2; ++k)
          __builtin_amdgcn_global_load_lds((global_ptr_t)(c2src + (uint32_t)(2 * k) * c2s), (lds_ptr_t)(sC2 + k * 1024), 16, 0, 2);
      }
      }
    } else {
#pragma unroll
      for (int i = 0; i < T; ++i) {
        ra[i] = load_stream<Tin, VEC>(ab, ao + i * as);
        rc[i] = load_stream<Tin, VEC>(cb, co + i * cs);
        rg[i] = load_stream<Tout, VEC>(gb, go + i * gs);
      }
#pragma unroll
      for (int i = 0; i < T; ++i) {
        rb[i] = load_stream<Tin, VEC>(bb, bo + i * bs);
        rx[i] = load_stream<Tin, VEC>(xb, xo + i * xs);
      }
    }
  } else {
    // Steps past L and columns past D act as the identity map (a = 1, everything else 0).
#pragma unroll
    for (int i = 0; i < T; ++i) {
      ra[i] = fill_words<Tin, VEC>(true);
      rb[i] = fill_words<Tin, VEC>(false);
      rx[i] = fill_words<Tin, VEC>(false);
      if (CREG) rc[i] = fill_words<Tin, VEC>(false);
      if (!CLDS) rg[i] = fill_words<Tout, VEC>(false);
    }
#pragma unroll
    for (int i = 0; i < T; ++i) {
      if (dok && t0 + i < g.L) {
        ra[i] = load_stream<Tin, VEC>(ab, ao + i * as);
        if (CREG) rc[i] = load_stream<Tin, VEC>(cb, co + i * cs);
        if (!CLDS) rg[i] = load_stream<Tout, VEC>(gb, go + i * gs);
        rb[i] = load_stream<Tin, VEC>(bb, bo + i * bs);
        rx[i] = load_stream<Tin, VEC>(xb, xo + i * xs);
      }
    }
    if (CLDS) {
      // Ragged tile (a partial last strip, or the end of the sequence): c and dy go through registers, half the
      // tile's steps at a time: rolled up so that it does not bring the registers back, but with the loads of a
      // half in flight together (one step at a time, a strip of D = 2000 behind seven whole ones cost the backward
      // 285 us against 219 us for D = 2048).
      constexpr int HB = T / 2;
#pragma unroll 1
      for (int i0 = 0; i0 < T; i0 += HB) {
        Words<Tin, VEC> cw[HB], cw2[GATED ? HB : 1];
        Words<Tout, VEC> gw[HB];
#pragma unroll
        for (int u = 0; u < HB; ++u) {
          const int i = i0 + u;
          cw[u] = fill_words<Tin, VEC>(false);
          gw[u] = fill_words<Tout, VEC>(false);
          if constexpr (GATED) cw2[u] = fill_words<Tin, VEC>(false);
          if (dok && t0 + i < g.L) {
            if (!CREG) cw[u] = load_stream<Tin, VEC>(cb, co + i * cs);
            gw[u] = load_stream<Tout, VEC>(gb, go + i * gs);
            if constexpr (GATED) cw2[u] = load_stream<Tin, VEC>(c2b, c2o + i * c2s);
          }
        }
#pragma unroll
        for (int u = 0; u < HB; ++u) {
          const int i = i0 + u;
          if (!CREG) *reinterpret_cast<Words<Tin, VEC>*>(sC + lds_row(i) + lds_lane) = cw[u];
          *reinterpret_cast<Words<Tout, VEC>*>(g_slot(i)) = gw[u];
          if constexpr (GATED) *reinterpret_cast<Words<Tin, VEC>*>(sC2 + lds_row(i) + lds_lane) = cw2[u];
        }
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
    } else if (dok && t0 == 0 && p.h_init != nullptr) {
      const Pack<float, VEC> hv = load_pack<float, VEC>(p.h_init + (int64_t)bi * g.D + d);
#pragma unroll
      for (int v = 0; v < VEC; ++v) hprev[v] = hv.v[v];
    }
  } else if (dok && t_tile > 0) {
    // state at the tile's first step, saved by the forward
    const Pack<float, VEC> hv = load_pack<float, VEC>(
        p.ckpt + ((int64_t)bi * g.n_ckpt + t_tile / g.ckpt_stride) * g.D + d);
#pragma unroll
    for (int v = 0; v < VEC; ++v) hprev[v] = hv.v[v];
  } else if (dok && p.h_init != nullptr) {
    // the first tile starts from the carried-in state
    const Pack<float, VEC> hv = load_pack<float, VEC>(p.h_init + (int64_t)bi * g.D + d);
#pragma unroll
    for (int v = 0; v < VEC; ++v) hprev[v] = hv.v[v];
  }

  // ---- the neighbours' answers (they were asked for before the operands, so they are back first)
  pk_state.pin();
  bool map_here = false, state_here = false;
  float ein[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) ein[v] = 0.0f;
  // A gradient arriving at the final state enters where the zero carry would: at the last cluster's
  // tiles (the lane group that folds the neighbours' maps onto it), or at every lane of a lone tile.
  if (p.dh_final != nullptr && s == g.n_super - 1 && dok && (edge || !multi)) {
    const Pack<float, VEC> ev = load_pack<float, VEC>(p.dh_final + (int64_t)bi * g.D + d);
#pragma unroll
    for (int v = 0; v < VEC; ++v) ein[v] = ev.v[v];
  }
  if (want_state && pk_state.ready(epoch)) {
    state_here = true;
#pragma unroll
    for (int v = 0; v < VEC; ++v) ein[v] = pk_state.value(v);
  }
  // Second look for what was not there yet; the answers travel while sweep 1 runs.
  const bool ask_state = want_state && !state_here;
  if (ask_state) pk_state.issue(next_state, G);

  // ---- sweep 1: fold this lane's T steps into the forward and the reverse affine map ----------
  float A[VEC], Xf[VEC], Xe[VEC];
  Words<Tin, VEC> za[GATED ? T : 1], zd[GATED ? T : 1];   // GATED: the derivatives of the two sigmoid gates
#pragma unroll
  for (int v = 0; v < VEC; ++v) { A[v] = 1.0f; Xf[v] = 0.0f; Xe[v] = 0.0f; }
#pragma unroll
  for (int i = 0; i < T; ++i) {
    if constexpr (GATED) {
      // The derivatives a (1 - a), b (1 - b) of the unrounded gates take the pre-activations' registers, rounded to
      // the storage type on their own (1 - a loses most of its digits when a, close to one, is first rounded to 16
      // bits): the last sweep multiplies by them instead of evaluating two more sigmoids per element.  Steps past L
      // and columns past D hold the identity (a = 1, b = 0) and keep it.
      za[i] = ra[i];
      zd[i] = rb[i];
      if (tile_full || (dok && t0 + i < g.L)) {
        float ga[VEC], gb[VEC], fa[VEC], fb[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          ga[v] = sigmoid_f(elem(ra[i], v));
          gb[v] = sigmoid_f(elem(rb[i], v));
          fa[v] = ga[v] * (1.0f - ga[v]);
          fb[v] = gb[v] * (1.0f - gb[v]);
        }
        if constexpr (ROUND) {
          float gx[VEC];
#pragma unroll
          for (int v = 0; v < VEC; ++v) gx[v] = elem(rx[i], v);
          round_through<Tc, VEC>(ga);
          round_through<Tc, VEC>(gb);
          round_through<Tc, VEC>(gx);
          ElemBits<Tin>::template set<VEC>(rx[i], gx);
        }
        ElemBits<Tin>::template set<VEC>(ra[i], ga);
        ElemBits<Tin>::template set<VEC>(rb[i], gb);
        ElemBits<Tin>::template set<VEC>(za[i], fa);
        ElemBits<Tin>::template set<VEC>(zd[i], fb);
      }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float av = elem(ra[i], v);
      Xf[v] = av * Xf[v] + elem(rb[i], v) * elem(rx[i], v);
      A[v] = av * A[v];
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // The loads that write c and dy into LDS are tracked by the vector memory counter only; this wave
  // is the only reader of the rows it fetched.  No store of the tile has been issued yet.
  if (CLDS) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
  for (int i = T - 1; i >= 0; --i) {
    Words<Tin, VEC> cw;
    Words<Tout, VEC> gw;
    if (CREG) cw = rc[i];
    else cw = *reinterpret_cast<const Words<Tin, VEC>*>(sC + lds_row(i) + lds_lane);
    if (CLDS) gw = *reinterpret_cast<const Words<Tout, VEC>*>(g_slot(i));
    else gw = rg[i];
    if constexpr (GATED) {
      const Words<Tin, VEC> cw2 = *reinterpret_cast<const Words<Tin, VEC>*>(sC2 + lds_row(i) + lds_lane);
      float gc[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) { const float ca = elem(cw, v); gc[v] = ca * sigmoid_f(ca) * elem(cw2, v); }
      if constexpr (ROUND) round_through<Tc, VEC>(gc);
      ElemBits<Tin>::template set<VEC>(cw, gc);
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v)
      Xe[v] = elem(ra[i], v) * (elem(cw, v) * elem(gw, v) + Xe[v]);
    __builtin_amdgcn_sched_barrier(0);
  }
  // ---- compose: groups before this one (forward state), groups after it (reverse carry) --------
  // Aq, Xq: the part of the reverse carry's map that the tile's total still has to be joined with; own: where the
  // map that closes the total sits in LDS (see the edge group below).
  float Ap[VEC], Xp[VEC], As[VEC], Xs[VEC], Aq[VEC], Xq[VEC];
  const float* own;
  if constexpr (XLANE) {
    // Cross-lane scans, one each way: the groups of one wavefront combine their maps with log2(64 / G) exchanges
    // between lanes, and one total per wavefront and direction goes through LDS.
    const int wl = tid & 63, w = tid >> 6;
    float* sAr = sA + NTH * VEC / 2;   // reverse totals of the wavefronts (the forward ones fill a quarter of sA at most)
    float Ar[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) Ar[v] = A[v];
    for (int off = G; off < 64; off <<= 1) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float pa = __shfl_up(A[v], off, 64), px = __shfl_up(Xf[v], off, 64);
        const float qa = __shfl_down(Ar[v], off, 64), qx = __shfl_down(Xe[v], off, 64);
        if (wl >= off) {        // forward: the earlier groups' map, then this one
          Xf[v] = A[v] * px + Xf[v];
          A[v] = A[v] * pa;
        }
        if (wl + off < 64) {    // reverse: the later groups' map, then this one
          Xe[v] = Ar[v] * qx + Xe[v];
          Ar[v] = Ar[v] * qa;
        }
      }
    }
    float Aef[VEC], Xef[VEC], Aer[VEC], Xer[VEC];   // the wavefront's groups before / after this one
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      Aef[v] = __shfl_up(A[v], G, 64);
      Xef[v] = __shfl_up(Xf[v], G, 64);
      Aer[v] = __shfl_down(Ar[v], G, 64);
      Xer[v] = __shfl_down(Xe[v], G, 64);
      if (wl < G) { Aef[v] = 1.0f; Xef[v] = 0.0f; }
      if (wl >= 64 - G) { Aer[v] = 1.0f; Xer[v] = 0.0f; }
    }
    own = sAr + dl;   // the first wavefront's reverse total: the edge group is its first group
    if (wl >= 64 - G) {
      lds_put<VEC>(sA + w * cols + dl, A);
      lds_put<VEC>(sXf + w * cols + dl, Xf);
    }
    if (wl < G) {
      lds_put<VEC>(sAr + w * cols + dl, Ar);
      lds_put<VEC>(sXe + w * cols + dl, Xe);
    }
#pragma unroll
    for (int i = 0; i < T; ++i) {
      forget(ra[i]); forget(rb[i]); forget(rx[i]); forget(rc[i]); forget(rg[i]);
    }
    lds_barrier();
    float Aw[VEC], Xw[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) { Aw[v] = 1.0f; Xw[v] = 0.0f; Aq[v] = 1.0f; Xq[v] = 0.0f; }
    if (!have_h) {
      for (int k = 0; k < w; ++k) {   // forward totals of the wavefronts before this one
        float ak[VEC], xk[VEC];
        lds_get<VEC>(sA + k * cols + dl, ak);
        lds_get<VEC>(sXf + k * cols + dl, xk);
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          Xw[v] = ak[v] * Xw[v] + xk[v];
          Aw[v] = ak[v] * Aw[v];
        }
      }
    }
    for (int k = (NTH >> 6) - 1; k > w; --k) {   // reverse totals of the wavefronts after this one
      float ak[VEC], xk[VEC];
      lds_get<VEC>(sAr + k * cols + dl, ak);
      lds_get<VEC>(sXe + k * cols + dl, xk);
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        Xq[v] = ak[v] * Xq[v] + xk[v];
        Aq[v] = ak[v] * Aq[v];
      }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      Ap[v] = Aef[v] * Aw[v];
      Xp[v] = Aef[v] * Xw[v] + Xef[v];
      As[v] = Aer[v] * Aq[v];
      Xs[v] = Aer[v] * Xq[v] + Xer[v];
    }
  } else {
    own = sA + tid * VEC;
    lds_put<VEC>(sA + tid * VEC, A);
    lds_put<VEC>(sXf + tid * VEC, Xf);
    lds_put<VEC>(sXe + tid * VEC, Xe);
#pragma unroll
    for (int i = 0; i < T; ++i) {
      forget(ra[i]); forget(rb[i]); forget(rx[i]);
      if (CREG) forget(rc[i]);
      if (!CLDS) forget(rg[i]);
    }
    lds_barrier();
#pragma unroll
    for (int v = 0; v < VEC; ++v) { Ap[v] = 1.0f; Xp[v] = 0.0f; As[v] = 1.0f; Xs[v] = 0.0f; }
    if (!have_h) {
#pragma unroll 4
      for (int k = 0; k < j; ++k) {
        float ak[VEC], xk[VEC];
        lds_get<VEC>(sA + k * cols + dl, ak);
        lds_get<VEC>(sXf + k * cols + dl, xk);
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          Xp[v] = ak[v] * Xp[v] + xk[v];
          Ap[v] = ak[v] * Ap[v];
        }
      }
    }
#pragma unroll 4
    for (int k = NG - 1; k > j; --k) {
      float ak[VEC], xk[VEC];
      lds_get<VEC>(sA + k * cols + dl, ak);
      lds_get<VEC>(sXe + k * cols + dl, xk);
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        Xs[v] = ak[v] * Xs[v] + xk[v];
        As[v] = ak[v] * As[v];
      }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) { Aq[v] = As[v]; Xq[v] = Xs[v]; }
  }

  // ---- reverse carry entering the tile -----------------------------------------------------------
  if (multi) {
    float At[VEC], Xt[VEC];
    if (edge) {
      // the map that closes the tile's total (this group's own, or its wavefront's) after everything after it
      float av[VEC], xv[VEC];
      lds_get<VEC>(own, av);
      lds_get<VEC>(XLANE ? sXe + dl : sXe + tid * VEC, xv);
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        At[v] = av[v] * Aq[v];
        Xt[v] = av[v] * Xq[v] + xv[v];
      }
      // Earlier tiles of the cluster need this tile's map; it depends on nothing, so it goes out first.
      if (dok && m > 0) {
        unsigned long long* mw = g.maps + ((int64_t)chain * g.n_seg + seg) * cols * 2 + lane;
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          word_publish(mw + (2 * v) * G, epoch, At[v]);
          word_publish(mw + (2 * v + 1) * G, epoch, Xt[v]);
        }
      }
    }
    // The second look's answers.
    if (ask_state && pk_state.ready(epoch)) {
      state_here = true;
#pragma unroll
      for (int v = 0; v < VEC; ++v) ein[v] = pk_state.value(v);
    }
    // Whatever is still missing is waited for: lane group j takes the maps of the later tiles
    // seg+1+j, seg+1+j+NG, ... of the cluster, and the first group, at the same time, the carry the
    // next cluster in time hands back (the one serial hop of the launch).
    for (int i = j; i < cnt; i += NG) {
      if (dok && !(i == j && map_here)) {
        float w[2 * VEC];
        const unsigned long long* mw = g.maps + ((int64_t)chain * g.n_seg + (seg + 1 + i)) * cols * 2 + lane;
        if (!words_wait<2 * VEC>(mw, G, epoch, w, kPollSlow)) raise_status(g.status, 1);
        float wa[VEC], wx[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) { wa[v] = w[2 * v]; wx[v] = w[2 * v + 1]; }
        lds_put<VEC>(sPA + i * cols + dl, wa);
        lds_put<VEC>(sPX + i * cols + dl, wx);
      }
    }
    if (want_state && !state_here) {
      if (!words_wait<VEC>(next_state, G, epoch, ein, m == 0 ? kPollChain : kPollUrgent)) raise_status(g.status, 1);
    }
    if (cnt > 0) lds_barrier();
    if (edge) {
      for (int i = cnt - 1; i >= 0; --i) {
        float pa[VEC], px[VEC];
        lds_get<VEC>(sPA + i * cols + dl, pa);
        lds_get<VEC>(sPX + i * cols + dl, px);
#pragma unroll
        for (int v = 0; v < VEC; ++v) ein[v] = pa[v] * ein[v] + px[v];
      }
      if (dok && m == 0 && s > 0) {
        unsigned long long* sw = g.states + ((int64_t)chain * g.n_super + s) * cols + lane;
#pragma unroll
        for (int v = 0; v < VEC; ++v) word_publish(sw + v * G, epoch, At[v] * ein[v] + Xt[v]);
      }
      lds_put<VEC>(sE + dl, ein);
    }
    lds_barrier();
    lds_get<VEC>(sE + dl, ein);
  }

  float E[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) E[v] = As[v] * ein[v] + Xs[v];

  // ---- sweep 2: rebuild h over this lane's steps -------------------------------------------------
  if (!have_h) {
#pragma unroll
    for (int v = 0; v < VEC; ++v) hprev[v] = Ap[v] * hprev[v] + Xp[v];
#pragma unroll
    for (int i = 0; i < T; ++i) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float hm = (i == 0) ? hprev[v] : hs[i - 1][v];
        hs[i][v] = elem(ra[i], v) * hm + elem(rb[i], v) * elem(rx[i], v);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  // ---- sweep 3: reverse recurrence and the four gradients ---------------------------------------
  char* dxb = (char*)p.dx + ((int64_t)bi * p.dx_sb + (int64_t)t_tile * p.dx_sl + col0) * (int64_t)sizeof(Tin);
  char* dab = (char*)p.da + ((int64_t)bi * p.da_sb + (int64_t)t_tile * p.da_sl + col0) * (int64_t)sizeof(Tin);
  char* dbb = (char*)p.db + ((int64_t)bi * p.db_sb + (int64_t)t_tile * p.db_sl + col0) * (int64_t)sizeof(Tin);
  char* dcb = (char*)p.dc + ((int64_t)bi * p.dc_sb + (int64_t)t_tile * p.dc_sl + col0) * (int64_t)sizeof(Tin);
  const uint32_t dxo = (uint32_t)((j * T * (int)p.dx_sl + dl) * (int)sizeof(Tin)), dxs = (uint32_t)p.dx_sl * sizeof(Tin);
  const uint32_t dao = (uint32_t)((j * T * (int)p.da_sl + dl) * (int)sizeof(Tin)), das = (uint32_t)p.da_sl * sizeof(Tin);
  const uint32_t dbo = (uint32_t)((j * T * (int)p.db_sl + dl) * (int)sizeof(Tin)), dbs = (uint32_t)p.db_sl * sizeof(Tin);
  const uint32_t dco = (uint32_t)((j * T * (int)p.dc_sl + dl) * (int)sizeof(Tin)), dcs = (uint32_t)p.dc_sl * sizeof(Tin);
  char* dc2b = GATED ? (char*)p.dc2 + ((int64_t)bi * p.dc2_sb + (int64_t)t_tile * p.dc2_sl + col0) * (int64_t)sizeof(Tin) : nullptr;
  const uint32_t dc2o = GATED ? (uint32_t)((j * T * (int)p.dc2_sl + dl) * (int)sizeof(Tin)) : 0u, dc2s = GATED ? (uint32_t)p.dc2_sl * sizeof(Tin) : 0u;
#pragma unroll
  for (int i = T - 1; i >= 0; --i) {
    float vdx[VEC], vda[VEC], vdb[VEC], vdc[VEC], vdc2[VEC];
    Words<Tin, VEC> cw;
    Words<Tout, VEC> gw;
    if (CREG) cw = rc[i];
    else cw = *reinterpret_cast<const Words<Tin, VEC>*>(sC + lds_row(i) + lds_lane);
    if (CLDS) gw = *reinterpret_cast<const Words<Tout, VEC>*>(g_slot(i));
    else gw = rg[i];
    float zca[VEC], zcb[VEC], sg[VEC];   // GATED: Ca, Cb and sigmoid(Ca) of this step
    if constexpr (GATED) {
      const Words<Tin, VEC> cw2 = *reinterpret_cast<const Words<Tin, VEC>*>(sC2 + lds_row(i) + lds_lane);
      float gc[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        zca[v] = elem(cw, v);
        zcb[v] = elem(cw2, v);
        sg[v] = sigmoid_f(zca[v]);
        gc[v] = zca[v] * sg[v] * zcb[v];
      }
      if constexpr (ROUND) round_through<Tc, VEC>(gc);
      ElemBits<Tin>::template set<VEC>(cw, gc);
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float gy = elem(gw, v);
      const float dH = elem(cw, v) * gy + E[v];
      const float hm = (i == 0) ? hprev[v] : hs[i - 1][v];
      vdc[v] = gy * hs[i][v];
      vdx[v] = elem(rb[i], v) * dH;
      vdb[v] = elem(rx[i], v) * dH;
      vda[v] = hm * dH;
      E[v] = elem(ra[i], v) * dH;
    }
    if constexpr (GATED) {
      // the scan's gradients as it would have stored them, then through the activations' derivatives
      if constexpr (ROUND) round_through<Tc, VEC>(vdx);   // (stored as Tin below: the same rounding when Tc is Tin)
      round_through<Tc, VEC>(vda);
      round_through<Tc, VEC>(vdb);
      round_through<Tc, VEC>(vdc);
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        vda[v] = vda[v] * elem(za[i], v);
        vdb[v] = vdb[v] * elem(zd[i], v);
        vdc2[v] = vdc[v] * zca[v] * sg[v];
        vdc[v] = vdc[v] * zcb[v] * sg[v] * (1.0f + zca[v] * (1.0f - sg[v]));
      }
    }
    if (tile_full || (dok && t0 + i < g.L)) {
      if (p.dx != nullptr) store_stream<Tin, VEC>(dxb, dxo + i * dxs, vdx);
      if (p.da != nullptr) store_stream<Tin, VEC>(dab, dao + i * das, vda);
      if (p.db != nullptr) store_stream<Tin, VEC>(dbb, dbo + i * dbs, vdb);
      if (p.dc != nullptr) store_stream<Tin, VEC>(dcb, dco + i * dcs, vdc);
      if constexpr (GATED) {
        if (p.dc2 != nullptr) store_stream<Tin, VEC>(dc2b, dc2o + i * dc2s, vdc2);
      }
    }
    // Keep each step's conversions next to their use (register footprint).
    __builtin_amdgcn_sched_barrier(0);
  }
  // What leaves the first step backwards, a(0) * dH(0), is the gradient of the carried-in state.
  if (p.dh_init != nullptr && seg == 0 && j == 0 && dok) {
    Pack<float, VEC> ev;
#pragma unroll
    for (int v = 0; v < VEC; ++v) ev.v[v] = E[v];
    store_pack<float, VEC>(p.dh_init + (int64_t)bi * g.D + d, ev);
  }
}

template <typename Tin, typename Tout>
static bool launch_bwd(const BwdArgs& args, int vec, int steps, int threads, bool cg_in_lds, int gated, dim3 grid,
                       size_t lds, hipStream_t stream) {
  if (gated != kNotGated) {
    // `gated` names the layer's compute dtype: the projections' storage type itself, or a 16-bit type for fp32 ones
    if constexpr (sizeof(Tin) == 2 && sizeof(Tout) == 2) {
      if (vec == 4 && steps == 8 && threads == 256 && cg_in_lds && gated == dtype_code<Tin>()) {
        hipLaunchKernelGGL((scan_bwd_kernel<Tin, Tout, 4, 8, 256, true, true, false>), grid, dim3(256), lds, stream, args);
        return true;
      }
    } else if constexpr (sizeof(Tin) == 4 && sizeof(Tout) == 4) {
      if (vec == 2 && steps == 8 && threads == 256 && cg_in_lds) {
        if (gated == QSSM_F32)
          hipLaunchKernelGGL((scan_bwd_kernel<float, float, 2, 8, 256, true, true, false, float>), grid, dim3(256), lds, stream, args);
        else if (gated == QSSM_F16)
          hipLaunchKernelGGL((scan_bwd_kernel<float, float, 2, 8, 256, true, true, false, f16_t>), grid, dim3(256), lds, stream, args);
        else
          hipLaunchKernelGGL((scan_bwd_kernel<float, float, 2, 8, 256, true, true, false, bf16_t>), grid, dim3(256), lds, stream, args);
        return true;
      }
    }
    return false;
  }
  // rows of at most 16 lanes in a 256-lane tile: 16 or more lane groups, folded across lanes
  const bool xlane = threads == 256 && !cg_in_lds && args.g.g_log2 <= 4;
#define QSSM_BWD_XCASE(V, S)                                                                                          \
  if (xlane && vec == V && steps == S) {                                                                              \
    hipLaunchKernelGGL((scan_bwd_kernel<Tin, Tout, V, S, 256, false, false, true>), grid, dim3(256), lds, stream, args); \
    return true;                                                                                                      \
  }
  QSSM_BWD_XCASE(1, 4)
  QSSM_BWD_XCASE(1, 8)
  QSSM_BWD_XCASE(2, 4)
  QSSM_BWD_XCASE(2, 8)
  QSSM_BWD_XCASE(4, 4)
  QSSM_BWD_XCASE(4, 8)
#undef QSSM_BWD_XCASE
#define QSSM_BWD_CASE(V, S, N, C)                                                                                   \
  if (vec == V && steps == S && threads == N && cg_in_lds == C) {                                                   \
    hipLaunchKernelGGL((scan_bwd_kernel<Tin, Tout, V, S, N, C, false, false>), grid, dim3(N), lds, stream, args);    \
    return true;                                                                                                    \
  }
  if constexpr (sizeof(Tin) == 2) {
    QSSM_BWD_CASE(4, 8, 256, true)
  }
  QSSM_BWD_CASE(1, 4, 256, false)
  QSSM_BWD_CASE(1, 8, 256, false)
  QSSM_BWD_CASE(2, 4, 256, false)
  QSSM_BWD_CASE(2, 8, 256, false)
  QSSM_BWD_CASE(4, 4, 256, false)
  QSSM_BWD_CASE(4, 8, 256, false)
  QSSM_BWD_CASE(2, 4, 512, false)
  QSSM_BWD_CASE(2, 8, 512, false)
  QSSM_BWD_CASE(4, 4, 512, false)
  QSSM_BWD_CASE(4, 8, 512, false)
  QSSM_BWD_CASE(2, 4, 1024, false)
  QSSM_BWD_CASE(2, 8, 1024, false)
  QSSM_BWD_CASE(4, 4, 1024, false)
#undef QSSM_BWD_CASE
  return false;
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
