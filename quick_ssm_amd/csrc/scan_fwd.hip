// Forward gated linear scan for gfx950: h(t) = a(t) h(t-1) + b(t) x(t), y(t) = c(t) h(t).
//
// One launch, one pass: x, a, b, c are read once and y is written once.  It takes the place
// of the reference's three forward launches and their N-sized fp32 scratch
// (ssm_local_forward_kernel / ssm_forward_carry_scan_kernel / ssm_fwd_apply_kernel,
// quick_ssm/triton_forwards.py:33-131) and of the y = c*h multiply and cast that follow them
// (quick_ssm/scan_interface.py:104-107).  The affine-map composition is the reference's
// combine_fn (quick_ssm/triton_forwards.py:26-30): (aL,xL) then (aR,xR) = (aR*aL, aR*xL+xR).
#include <type_traits>

#include "scan_common.h"

namespace qssm {

typedef __attribute__((address_space(1))) const void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// CLDS: the c operand is not needed before the last sweep, so it is loaded straight into LDS
// (no destination registers) and read from there step by step: 16 VGPRs fewer across the
// tile's whole life, which is one more resident workgroup per SIMD.  Needs 64 or 32 lanes per row and
// 8 bytes per lane, so that one wavefront-wide 16-byte-per-lane load covers whole rows of the strip.
//
// GATED: the operands are the SSM layer's projection outputs (quick_ssm/layers.py:76-88) and the gate activations
// happen here instead of in a pass of their own: a = sigmoid(A_pre) and b = sigmoid(D_pre) replace their
// pre-activations in the registers that hold them (rounded to the storage type, as the layer's cast to its
// compute dtype rounds them), c = silu(Ca) * Cb is formed step by step in the last sweep from two LDS-resident
// operands.  The a, x, b, c tensors of the layer never exist in HBM.
//
// Tc is the type the layer rounds the gates' outputs to (its compute dtype): the projections' own storage type, or,
// for fp32 projections (the reference's default layer: fp32 parameters, fp16 compute), a 16-bit type that only
// ever exists in registers; a = sigmoid(A_pre), x = B_in, b and c are rounded through it before they are used.
//
// XLANE: rows of 16 lanes or fewer (a few columns of D), where a tile has 16 to 256 lane groups: their maps are
// combined by exchanges between the lanes of a wavefront instead of a walk through LDS.
template <typename Tin, typename Tout, int VEC, int T, int NTH, bool CLDS, bool GATED, bool XLANE, typename Tc = Tin>
__global__ void __launch_bounds__(NTH) scan_fwd_kernel(const FwdArgs p) {
  static_assert(!XLANE || (!CLDS && !GATED), "cross-lane fold: register-only operands");
  static_assert(!GATED || (CLDS && sizeof(Tin) * VEC == 8), "gated scan: 8 bytes per lane, Ca and Cb through LDS");
  static_assert(GATED || std::is_same<Tc, Tin>::value, "a compute dtype of its own only means something to the gated scan");
  constexpr bool ROUND = !std::is_same<Tc, Tin>::value;   // the gates' outputs are rounded to a type narrower than their storage
  static_assert(!CLDS || ((sizeof(Tin) * VEC == 8 || sizeof(Tin) * VEC == 16) && T % 2 == 0),
                "LDS-resident c: 8 or 16 bytes per lane, even step count");
  // 16 bytes per lane: the load that deposits c in LDS gives every lane exactly its own columns of one step.
  constexpr bool WIDE = sizeof(Tin) * VEC == 16;
  constexpr int CROW = WIDE ? 1024 : 512;   // bytes of c one wavefront holds per step
  extern __shared__ __align__(16) float lds[];
  const Geometry& g = p.g;
  const int G = 1 << g.g_log2;
  const int NG = NTH >> g.g_log2;
  const int cols = G * VEC;
  const int R = g.cluster;
  // Flag value of this launch: the host's, or one more than the launches counted in the control block.
  const unsigned epoch = g.launch_count != nullptr ? *g.launch_count + 1u : g.epoch;
  float* sA = lds;                       // [NTH * VEC] per-lane map, multiplier
  float* sX = sA + NTH * VEC;            // [NTH * VEC] per-lane map, offset
  float* sPA = sX + NTH * VEC;           // [(R-1) * cols] maps of the earlier tiles of the cluster
  float* sPX = sPA + (R - 1) * cols;
  float* sH = sPX + (R - 1) * cols;      // [cols] state entering the tile
  int* sSeg = reinterpret_cast<int*>(sH + cols);
  char* sC = reinterpret_cast<char*>(sSeg) + 16;  // CLDS: [NTH / 64 waves][T rows][CROW bytes] of c
  char* sC2 = sC + (NTH / 64) * (T * CROW);       // GATED: the same of Cb (sC then holds Ca)

  const int tid = threadIdx.x;
  // Workgroups go to the eight XCDs in turn, so workgroup i runs on XCD i mod 8.  Chains are dealt out so that each
  // XCD gets a run of adjacent chains (the strips of one batch row, when there are eight of each) rather than
  // every eighth one: its workgroups then stream whole rows of few batch rows instead of one 512-byte column of
  // all of them, which its L2 and address translation reward.  All tiles of a chain still run on one XCD.
  int chain = blockIdx.x % g.n_chains;
  if ((g.n_chains & 7) == 0) chain = (chain & 7) * (g.n_chains >> 3) + (chain >> 3);
  // Where step i of this lane sits in its wavefront's block of sC: the loads that fill it deposit 1024 bytes
  // per instruction in lane order, i.e. per pair of steps [group in wavefront][step parity][G * 8 bytes].
  const int lds_lane = WIDE ? (tid & 63) * 16 : ((tid & 63) >> g.g_log2) * (G * 16) + (tid & (G - 1)) * 8;
  auto lds_row = [&](int i) { return WIDE ? i * 1024 : (i >> 1) * 1024 + (i & 1) * (G * 8); };

  // ---- claim a tile of this chain, in time order -------------------------------------------
  int seg = 0;
  if (g.n_seg > 1) {
    if (tid == 0) *sSeg = (int)claim_ticket(g.tickets, chain, g.n_seg);
    __syncthreads();
    seg = __builtin_amdgcn_readfirstlane(*sSeg);
    if ((unsigned)seg >= (unsigned)g.n_seg) {
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
          if (p.y != nullptr)
            store_stream<Tout, VEC>((char*)p.y + ((int64_t)pbi * p.y_sb + (int64_t)t * p.y_sl + pd) * (int64_t)sizeof(Tout), 0u, nanv);
          if (p.h_out != nullptr)
            store_stream<float, VEC>((char*)p.h_out + ((int64_t)pbi * p.h_sb + (int64_t)t * p.h_sl + pd) * (int64_t)sizeof(float), 0u, nanv);
          if (p.ckpt != nullptr && t % g.ckpt_stride == 0)
            store_stream<float, VEC>((char*)p.ckpt + (((int64_t)pbi * g.n_ckpt + t / g.ckpt_stride) * g.D + pd) * (int64_t)sizeof(float), 0u, nanv);
        }
      }
      if (p.h_final != nullptr && pseg == g.n_seg - 1 && (tid >> g.g_log2) == 0 && pd < g.D)
        store_stream<float, VEC>((char*)p.h_final + ((int64_t)pbi * g.D + pd) * (int64_t)sizeof(float), 0u, nanv);
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
  const char* c2b = GATED ? (const char*)p.c2 + ((int64_t)bi * p.c2_sb + (int64_t)t_tile * p.c2_sl + col0) * (int64_t)sizeof(Tin) : nullptr;
  const uint32_t c2o = GATED ? (uint32_t)((j * T * (int)p.c2_sl + dl) * (int)sizeof(Tin)) : 0u, c2s = GATED ? (uint32_t)p.c2_sl * sizeof(Tin) : 0u;
  const bool want_y = p.y != nullptr;
  const bool has_c = want_y && p.c != nullptr;

  // ---- ask for the neighbours' words first: they are looked at once the answers are back ------
  const bool multi = g.n_seg > 1;
  const int s = seg / R;               // cluster of this tile
  const int m = seg - s * R;           // tiles of the cluster before this one
  const bool edge = (j == NG - 1);     // the last lane group holds the tile's total map
  const int lane = tid & (G - 1);      // position inside the lane group = position inside a word plane
  const unsigned long long* my_map = g.maps + ((int64_t)chain * g.n_seg + (seg - m + j)) * cols * 2 + lane;
  const unsigned long long* prev_state = g.states + ((int64_t)chain * g.n_super + (s - 1)) * cols + lane;
  const bool want_map = multi && dok && j < m;            // this lane group fetches the map of tile (seg - m + j)
  const bool want_state = multi && dok && edge && s > 0;  // and the last group the previous cluster's state
  Peek<2 * VEC> pk_map;
  Peek<VEC> pk_state;
  pk_map.clear();
  pk_state.clear();
  if (want_map) pk_map.issue(my_map, G);
  if (want_state) pk_state.issue(prev_state, G);

  // ---- issue every load of the tile before touching any of them ------------------------------
  Words<Tin, VEC> rx[T], ra[T], rb[T], rc[CLDS ? 1 : T];
  const bool tile_full = (t_tile + g.seg_len <= g.L) && ((strip + 1) * cols <= g.D);
  // Operand loads of a whole tile.  KEEP: ordinary loads, which leave the lines in the cache hierarchy, for the last
  // tiles of a chain: a backward that follows the forward reads exactly those first.  Everything else streams.
  auto load_tile = [&](auto keep_tag) {
    constexpr bool KEEP = decltype(keep_tag)::value;
    constexpr int AUX = KEEP ? 0 : 2;   // cache policy bits of the loads into LDS: 2 = non-temporal
    // Loads that differ in nothing but their cache policy look alike to the optimizer, which would hoist one
    // (ordinary) copy in front of the branch; a fence at the head of one flavour keeps them apart.
    if constexpr (KEEP) asm volatile("" ::: "memory");
    // one tensor after the other rather than step by step: a hair faster (0.4 us of 125 on the headline shape)
#pragma unroll
    for (int i = 0; i < T; ++i) ra[i] = load_stream<Tin, VEC, KEEP>(ab, ao + i * as);
#pragma unroll
    for (int i = 0; i < T; ++i) rb[i] = load_stream<Tin, VEC, KEEP>(bb, bo + i * bs);
#pragma unroll
    for (int i = 0; i < T; ++i) rx[i] = load_stream<Tin, VEC, KEEP>(xb, xo + i * xs);
    if (CLDS && WIDE) {
      char* dst = sC + (tid >> 6) * (T * CROW);
#pragma unroll
      for (int i = 0; i < T; ++i)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(cb + co + i * cs), (lds_ptr_t)(dst + i * 1024), 16, 0, AUX);
    } else if (CLDS) {
      // 16 bytes per lane: the first half of a lane group's lanes fetches one row of the strip, the second half
      // the next one (64 lanes per row: a wavefront covers two rows of one group; 32: two rows of two groups)
      const int wl = tid & 63;
      const int half = (wl >> (g.g_log2 - 1)) & 1, piece = wl & ((G >> 1) - 1);
      const char* src = cb + (uint32_t)(j * T + half) * cs + (uint32_t)piece * 16u;
      char* dst = sC + (tid >> 6) * (T * 512);
#pragma unroll
      for (int k = 0; k < T / 2; ++k)
        __builtin_amdgcn_global_load_lds((global_ptr_t)(src + (uint32_t)(2 * k) * cs), (lds_ptr_t)(dst + k * 1024), 16, 0, AUX);
      if constexpr (GATED) {
        const char* src2 = c2b + (uint32_t)(j * T + half) * c2s + (uint32_t)piece * 16u;
        char* dst2 = sC2 + (tid >> 6) * (T * 512);
#pragma unroll
        for (int k = 0; k < T / 2; ++k)
          __builtin_amdgcn_global_load_lds((global_ptr_t)(src2 + (uint32_t)(2 * k) * c2s), (lds_ptr_t)(dst2 + k * 1024), 16, 0, AUX);
      }
    } else if (has_c) {
#pragma unroll
      for (int i = 0; i < T; ++i) rc[i] = load_stream<Tin, VEC, KEEP>(cb, co + i * cs);
    }
  };
  if (tile_full) {
    if (seg >= g.keep_from) load_tile(std::true_type{});
    else load_tile(std::false_type{});
  } else {
    // Steps past L and columns past D act as the identity map (a = 1, b*x = 0).
#pragma unroll
    for (int i = 0; i < T; ++i) {
      ra[i] = fill_words<Tin, VEC>(true);
      rb[i] = fill_words<Tin, VEC>(false);
      rx[i] = fill_words<Tin, VEC>(false);
      if (!CLDS) rc[i] = fill_words<Tin, VEC>(false);
    }
#pragma unroll
    for (int i = 0; i < T; ++i) {
      if (dok && t0 + i < g.L) {
        ra[i] = load_stream<Tin, VEC>(ab, ao + i * as);
        rb[i] = load_stream<Tin, VEC>(bb, bo + i * bs);
        rx[i] = load_stream<Tin, VEC>(xb, xo + i * xs);
        if (!CLDS && has_c) rc[i] = load_stream<Tin, VEC>(cb, co + i * cs);
      }
    }
    if (CLDS) {
      // Ragged tile (a partial last strip, or the end of the sequence): c goes through registers, half the tile's
      // steps at a time: rolled up so that it does not bring the registers back, but with the loads of a half in
      // flight together.
      char* dst = sC + (tid >> 6) * (T * CROW) + lds_lane;
      constexpr int HB = T / 2;
#pragma unroll 1
      for (int i0 = 0; i0 < T; i0 += HB) {
        Words<Tin, VEC> cw[HB], cw2[GATED ? HB : 1];
#pragma unroll
        for (int u = 0; u < HB; ++u) {
          const int i = i0 + u;
          cw[u] = fill_words<Tin, VEC>(false);
          if constexpr (GATED) cw2[u] = fill_words<Tin, VEC>(false);
          if (dok && t0 + i < g.L) {
            cw[u] = load_stream<Tin, VEC>(cb, co + i * cs);
            if constexpr (GATED) cw2[u] = load_stream<Tin, VEC>(c2b, c2o + i * c2s);
          }
        }
#pragma unroll
        for (int u = 0; u < HB; ++u) {
          const int i = i0 + u;
          *reinterpret_cast<Words<Tin, VEC>*>(dst + lds_row(i)) = cw[u];
          if constexpr (GATED) *reinterpret_cast<Words<Tin, VEC>*>(dst + (sC2 - sC) + lds_row(i)) = cw2[u];
        }
      }
    }
  }

  // ---- the neighbours' answers (they were asked for before the operands, so they are back first)
  pk_map.pin();
  pk_state.pin();
  bool map_here = false, state_here = false;
  float hin[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) hin[v] = 0.0f;
  // A carried-in state enters where the zero state would: at the first cluster's tiles (the lane group
  // that folds the neighbours' maps onto it), or at every lane when the chain has a single tile.
  if (p.h_init != nullptr && s == 0 && dok && (edge || !multi)) {
    const Pack<float, VEC> hv = load_pack<float, VEC>(p.h_init + (int64_t)bi * g.D + d);
#pragma unroll
    for (int v = 0; v < VEC; ++v) hin[v] = hv.v[v];
  }
  if (want_map && pk_map.ready(epoch)) {
    map_here = true;
    float wa[VEC], wx[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) { wa[v] = pk_map.value(2 * v); wx[v] = pk_map.value(2 * v + 1); }
    lds_put<VEC>(sPA + j * cols + dl, wa);
    lds_put<VEC>(sPX + j * cols + dl, wx);
  }
  if (want_state && pk_state.ready(epoch)) {
    state_here = true;
#pragma unroll
    for (int v = 0; v < VEC; ++v) hin[v] = pk_state.value(v);
  }
  // Second look for what was not there yet; the answers travel while sweep 1 runs.
  const bool ask_map = want_map && !map_here, ask_state = want_state && !state_here;
  if (ask_map) pk_map.issue(my_map, G);
  if (ask_state) pk_state.issue(prev_state, G);

  // ---- sweep 1: fold this lane's T steps into one affine map ---------------------------------
  float A[VEC], X[VEC];
#pragma unroll
  for (int v = 0; v < VEC; ++v) { A[v] = 1.0f; X[v] = 0.0f; }
#pragma unroll
  for (int i = 0; i < T; ++i) {
    if constexpr (GATED) {
      // Steps past L and columns past D hold the identity (a = 1, b = 0) already and keep it.
      if (tile_full || (dok && t0 + i < g.L)) {
        float ga[VEC], gb[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) { ga[v] = sigmoid_f(elem(ra[i], v)); gb[v] = sigmoid_f(elem(rb[i], v)); }
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
      }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const float av = elem(ra[i], v);
      X[v] = av * X[v] + elem(rb[i], v) * elem(rx[i], v);
      A[v] = av * A[v];
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // ---- compose the maps of the lane groups before this one ------------------------------------
  // Ap, Xp: the map of the tile's steps before this lane's; Aq, Xq: the part of it that the tile's total still
  // has to be joined with (see the edge group below); own: where the map that closes the total sits in LDS.
  float Ap[VEC], Xp[VEC], Aq[VEC], Xq[VEC];
  const float* own;
  if constexpr (XLANE) {   // several lane groups share a wavefront (g_log2 < 6)
    // Cross-lane scan: the groups of one wavefront combine their maps with log2(64 / G) exchanges between lanes
    // (group k takes the running map of group k - 2^s), whatever their number; only one total per wavefront
    // goes through LDS.  With one lane per row (D of a few columns) a 256-lane tile has 256 groups: 6 exchanges
    // and 3 LDS reads instead of up to 255 dependent LDS reads.
    const int wl = tid & 63;
    for (int off = G; off < 64; off <<= 1) {
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        const float pa = __shfl_up(A[v], off, 64), px = __shfl_up(X[v], off, 64);
        if (wl >= off) {   // the earlier groups' map (pa, px), then this one
          X[v] = A[v] * px + X[v];
          A[v] = A[v] * pa;
        }
      }
    }
    float Ae[VEC], Xe[VEC];   // map of the wavefront's groups before this one
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      Ae[v] = __shfl_up(A[v], G, 64);
      Xe[v] = __shfl_up(X[v], G, 64);
      if (wl < G) { Ae[v] = 1.0f; Xe[v] = 0.0f; }
    }
    const int w = tid >> 6;
    own = sA + w * cols + dl;
    if (wl >= 64 - G) {   // the wavefront's last group now holds its total
      lds_put<VEC>(sA + w * cols + dl, A);
      lds_put<VEC>(sX + w * cols + dl, X);
    }
#pragma unroll
    for (int i = 0; i < T; ++i) { forget(ra[i]); forget(rb[i]); forget(rx[i]); }
    lds_barrier();
#pragma unroll
    for (int v = 0; v < VEC; ++v) { Aq[v] = 1.0f; Xq[v] = 0.0f; }
    for (int k = 0; k < w; ++k) {   // totals of the wavefronts before this one
      float ak[VEC], xk[VEC];
      lds_get<VEC>(sA + k * cols + dl, ak);
      lds_get<VEC>(sX + k * cols + dl, xk);
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        Xq[v] = ak[v] * Xq[v] + xk[v];
        Aq[v] = ak[v] * Aq[v];
      }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      Ap[v] = Ae[v] * Aq[v];
      Xp[v] = Ae[v] * Xq[v] + Xe[v];
    }
  } else {
    own = sA + tid * VEC;
    lds_put<VEC>(sA + tid * VEC, A);
    lds_put<VEC>(sX + tid * VEC, X);
#pragma unroll
    for (int i = 0; i < T; ++i) { forget(ra[i]); forget(rb[i]); forget(rx[i]); }
    lds_barrier();
#pragma unroll
    for (int v = 0; v < VEC; ++v) { Ap[v] = 1.0f; Xp[v] = 0.0f; }
#pragma unroll 4
    for (int k = 0; k < j; ++k) {
      float ak[VEC], xk[VEC];
      lds_get<VEC>(sA + k * cols + dl, ak);
      lds_get<VEC>(sX + k * cols + dl, xk);
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        Xp[v] = ak[v] * Xp[v] + xk[v];
        Ap[v] = ak[v] * Ap[v];
      }
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) { Aq[v] = Ap[v]; Xq[v] = Xp[v]; }
  }

  // The loads that write c into LDS are tracked by the vector memory counter only; this wave is the
  // only reader of the rows it fetched.  Waiting here, before any store of the tile is issued, waits
  // for nothing but loads, and c, asked for last, has had the fold above to arrive.
  if (CLDS) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  // ---- state entering the tile ------------------------------------------------------------------
  if (multi) {
    float At[VEC], Xt[VEC];
    if (edge) {
      // the map that closes the tile's total (this group's own, or its wavefront's) after everything before it
      float av[VEC], xv[VEC];
      lds_get<VEC>(own, av);
      lds_get<VEC>(own + (sX - sA), xv);
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        At[v] = av[v] * Aq[v];
        Xt[v] = av[v] * Xq[v] + xv[v];
      }
      // Later tiles of the cluster need this tile's map; it depends on nothing, so it goes out first.
      if (dok && m + 1 < R && seg + 1 < g.n_seg) {
        unsigned long long* mw = g.maps + ((int64_t)chain * g.n_seg + seg) * cols * 2 + lane;
#pragma unroll
        for (int v = 0; v < VEC; ++v) {
          word_publish(mw + (2 * v) * G, epoch, At[v]);
          word_publish(mw + (2 * v + 1) * G, epoch, Xt[v]);
        }
      }
    }
    // The second look's answers.
    if (ask_map && pk_map.ready(epoch)) {
      map_here = true;
      float wa[VEC], wx[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) { wa[v] = pk_map.value(2 * v); wx[v] = pk_map.value(2 * v + 1); }
      lds_put<VEC>(sPA + j * cols + dl, wa);
      lds_put<VEC>(sPX + j * cols + dl, wx);
    }
    if (ask_state && pk_state.ready(epoch)) {
      state_here = true;
#pragma unroll
      for (int v = 0; v < VEC; ++v) hin[v] = pk_state.value(v);
    }
    // Whatever is still missing is waited for: lane group j takes the maps of the earlier tiles
    // j, j+NG, ... of the cluster, and the last group, at the same time, the previous cluster's
    // state (the one serial hop of the launch).
    for (int i = j; i < m; i += NG) {
      if (dok && !(i == j && map_here)) {
        float w[2 * VEC];
        const unsigned long long* mw = g.maps + ((int64_t)chain * g.n_seg + (seg - m + i)) * cols * 2 + lane;
        if (!words_wait<2 * VEC>(mw, G, epoch, w, kPollSlow)) raise_status(g.status, 1);
        float wa[VEC], wx[VEC];
#pragma unroll
        for (int v = 0; v < VEC; ++v) { wa[v] = w[2 * v]; wx[v] = w[2 * v + 1]; }
        lds_put<VEC>(sPA + i * cols + dl, wa);
        lds_put<VEC>(sPX + i * cols + dl, wx);
      }
    }
    if (want_state && !state_here) {
      if (!words_wait<VEC>(prev_state, G, epoch, hin, m == R - 1 ? kPollChain : kPollUrgent)) raise_status(g.status, 1);
    }
    if (m > 0) lds_barrier();
    if (edge) {
      for (int i = 0; i < m; ++i) {
        float pa[VEC], px[VEC];
        lds_get<VEC>(sPA + i * cols + dl, pa);
        lds_get<VEC>(sPX + i * cols + dl, px);
#pragma unroll
        for (int v = 0; v < VEC; ++v) hin[v] = pa[v] * hin[v] + px[v];
      }
      if (dok && m == R - 1 && s + 1 < g.n_super) {
        unsigned long long* sw = g.states + ((int64_t)chain * g.n_super + s) * cols + lane;
#pragma unroll
        for (int v = 0; v < VEC; ++v) word_publish(sw + v * G, epoch, At[v] * hin[v] + Xt[v]);
      }
      lds_put<VEC>(sH + dl, hin);
    }
    lds_barrier();
    lds_get<VEC>(sH + dl, hin);
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
  const bool want_final = p.h_final != nullptr && seg == g.n_seg - 1 && edge;
  if (!want_y && p.h_out == nullptr && p.h_final == nullptr) return;

  // ---- sweep 2: the recurrence proper, from the true carry-in -----------------------------------
  char* yb = (char*)p.y + ((int64_t)bi * p.y_sb + (int64_t)t_tile * p.y_sl + col0) * (int64_t)sizeof(Tout);
  char* hb = (char*)p.h_out + ((int64_t)bi * p.h_sb + (int64_t)t_tile * p.h_sl + col0) * (int64_t)sizeof(float);
  const uint32_t yo = (uint32_t)((j * T * (int)p.y_sl + dl) * (int)sizeof(Tout)), ys = (uint32_t)p.y_sl * sizeof(Tout);
  const uint32_t ho = (uint32_t)((j * T * (int)p.h_sl + dl) * (int)sizeof(float)), hs = (uint32_t)p.h_sl * sizeof(float);
#pragma unroll
  for (int i = 0; i < T; ++i) {
    float yv[VEC];
    Words<Tin, VEC> cw;
    if (CLDS) cw = *reinterpret_cast<const Words<Tin, VEC>*>(sC + (tid >> 6) * (T * CROW) + lds_row(i) + lds_lane);
    else cw = rc[i];
    if constexpr (GATED) {
      const Words<Tin, VEC> cw2 = *reinterpret_cast<const Words<Tin, VEC>*>(sC2 + (tid >> 6) * (T * CROW) + lds_row(i) + lds_lane);
      float gc[VEC];
#pragma unroll
      for (int v = 0; v < VEC; ++v) { const float ca = elem(cw, v); gc[v] = ca * sigmoid_f(ca) * elem(cw2, v); }
      if constexpr (ROUND) round_through<Tc, VEC>(gc);
      ElemBits<Tin>::template set<VEC>(cw, gc);
    }
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      h[v] = elem(ra[i], v) * h[v] + elem(rb[i], v) * elem(rx[i], v);
      yv[v] = (CLDS || has_c) ? elem(cw, v) * h[v] : h[v];
    }
    if (tile_full || (dok && t0 + i < g.L)) {
      if (want_y) store_stream<Tout, VEC>(yb, yo + i * ys, yv);
      if (p.h_out != nullptr) store_stream<float, VEC>(hb, ho + i * hs, h);
    }
    // Keep each step's conversions next to their use: hoisting them all above the recurrence
    // would hold an fp32 copy of the whole tile in registers.
    __builtin_amdgcn_sched_barrier(0);
  }
  // Steps past L are identity steps, so the last lane group of the last tile ends on h(L-1).
  if (want_final && dok) {
    Pack<float, VEC> hv;
#pragma unroll
    for (int v = 0; v < VEC; ++v) hv.v[v] = h[v];
    store_pack<float, VEC>(p.h_final + (int64_t)bi * g.D + d, hv);
  }
}

template <typename Tin, typename Tout>
static bool launch_fwd(const FwdArgs& args, int vec, int steps, int threads, bool c_in_lds, int gated, dim3 grid,
                       size_t lds, hipStream_t stream) {
  if (gated != kNotGated) {
    // `gated` names the layer's compute dtype: the projections' storage type itself, or a 16-bit type for fp32 ones
    if constexpr (sizeof(Tin) == 2) {
      if (vec == 4 && steps == 8 && threads == 256 && c_in_lds && gated == dtype_code<Tin>()) {
        hipLaunchKernelGGL((scan_fwd_kernel<Tin, Tout, 4, 8, 256, true, true, false>), grid, dim3(256), lds, stream, args);
        return true;
      }
    } else if constexpr (sizeof(Tout) == 4) {
      if (vec == 2 && steps == 8 && threads == 256 && c_in_lds) {
        if (gated == QSSM_F32)
          hipLaunchKernelGGL((scan_fwd_kernel<float, float, 2, 8, 256, true, true, false, float>), grid, dim3(256), lds, stream, args);
        else if (gated == QSSM_F16)
          hipLaunchKernelGGL((scan_fwd_kernel<float, float, 2, 8, 256, true, true, false, f16_t>), grid, dim3(256), lds, stream, args);
        else
          hipLaunchKernelGGL((scan_fwd_kernel<float, float, 2, 8, 256, true, true, false, bf16_t>), grid, dim3(256), lds, stream, args);
        return true;
      }
    }
    return false;
  }
  // rows of at most 16 lanes in a 256-lane tile: 16 or more lane groups, folded across lanes
  const bool xlane = threads == 256 && !c_in_lds && args.g.g_log2 <= 4;
#define QSSM_FWD_XCASE(V, S)                                                                                          \
  if (xlane && vec == V && steps == S) {                                                                              \
    hipLaunchKernelGGL((scan_fwd_kernel<Tin, Tout, V, S, 256, false, false, true>), grid, dim3(256), lds, stream, args); \
    return true;                                                                                                      \
  }
  QSSM_FWD_XCASE(1, 4)
  QSSM_FWD_XCASE(1, 8)
  QSSM_FWD_XCASE(2, 4)
  QSSM_FWD_XCASE(2, 8)
  QSSM_FWD_XCASE(4, 4)
  QSSM_FWD_XCASE(4, 8)
#undef QSSM_FWD_XCASE
#define QSSM_FWD_CASE(V, S, N, C)                                                                                   \
  if (vec == V && steps == S && threads == N && c_in_lds == C) {                                                    \
    hipLaunchKernelGGL((scan_fwd_kernel<Tin, Tout, V, S, N, C, false, false>), grid, dim3(N), lds, stream, args);    \
    return true;                                                                                                    \
  }
  if constexpr (sizeof(Tin) == 2) {
    QSSM_FWD_CASE(4, 8, 256, true)
    QSSM_FWD_CASE(4, 8, 512, true)
    QSSM_FWD_CASE(8, 8, 256, true)
    QSSM_FWD_CASE(8, 8, 256, false)
    QSSM_FWD_CASE(8, 4, 256, true)
    QSSM_FWD_CASE(8, 4, 256, false)
    QSSM_FWD_CASE(8, 4, 512, true)
    QSSM_FWD_CASE(8, 4, 512, false)
  }
  QSSM_FWD_CASE(1, 4, 256, false)
  QSSM_FWD_CASE(1, 8, 256, false)
  QSSM_FWD_CASE(2, 4, 256, false)
  QSSM_FWD_CASE(2, 8, 256, false)
  QSSM_FWD_CASE(4, 4, 256, false)
  QSSM_FWD_CASE(4, 8, 256, false)
  QSSM_FWD_CASE(2, 4, 512, false)
  QSSM_FWD_CASE(2, 8, 512, false)
  QSSM_FWD_CASE(4, 4, 512, false)
  QSSM_FWD_CASE(4, 8, 512, false)
  QSSM_FWD_CASE(2, 4, 1024, false)
  QSSM_FWD_CASE(2, 8, 1024, false)
  QSSM_FWD_CASE(4, 4, 1024, false)
  QSSM_FWD_CASE(4, 8, 1024, false)
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
