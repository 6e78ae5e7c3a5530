// C ABI of libquick_ssm_hip.so: launch planning, argument checks and kernel launches.
// Declarations and the reference functions each entry point stands in for: include/quick_ssm_hip.h.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <initializer_list>
#include <mutex>
#include <utility>

#include "scan_common.h"

namespace qssm {

static thread_local char g_err[256] = "";

static int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

static int hip_fail(hipError_t e, const char* what) {
  snprintf(g_err, sizeof(g_err), "%s: %s", what, hipGetErrorString(e));
  return (int)e;
}

static int dtype_size(int dt) {
  switch (dt) {
    case QSSM_F32: return 4;
    case QSSM_F16: return 2;
    case QSSM_BF16: return 2;
    default: return 0;
  }
}

static int pow2_ceil(int64_t n) {
  int p = 1;
  while (p < n) p <<= 1;
  return p;
}

// Lanes that one row of D columns can feed at `vec` columns per lane (a power of two <= 1024).
static int lanes_cap(int D, int vec) {
  const int lanes = pow2_ceil(D > 0 ? (D + vec - 1) / vec : 1);
  return lanes < 1024 ? lanes : 1024;
}

static int ilog2(int n) {
  int l = 0;
  while ((1 << l) < n) ++l;
  return l;
}

__global__ void __launch_bounds__(256) fill_zero_kernel(uint4* p, uint64_t n16) {
  uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (; i < n16; i += stride) p[i] = make_uint4(0, 0, 0, 0);
}

// 16-byte copy, the calibration kernel of known traffic (bytes read = bytes written): one workgroup per
// 16 KiB, started in index order and gone after one step, so that the resident workgroups cover one
// narrow window of both buffers (workgroups that stay and stride through the buffers copy a fifth slower).
__global__ void __launch_bounds__(256) copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                   uint64_t n16) {
  for (uint64_t base = (uint64_t)blockIdx.x * 1024u; base < n16; base += (uint64_t)gridDim.x * 1024u) {
    typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
    const u32x4* s = reinterpret_cast<const u32x4*>(src);
    u32x4* d = reinterpret_cast<u32x4*>(dst);
    const uint64_t i = base + threadIdx.x;
    u32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (i + 256u * k < n16) v[k] = __builtin_nontemporal_load(s + i + 256u * k);
#pragma unroll
    for (int k = 0; k < 4; ++k)
      if (i + 256u * k < n16) __builtin_nontemporal_store(v[k], d + i + 256u * k);
  }
}

static bool aligned_to(const void* p, int64_t sb, int64_t sl, int elem_bytes, int vec) {
  if (p == nullptr) return true;
  if (((uintptr_t)p) % ((uintptr_t)elem_bytes * vec) != 0) return false;
  return (sb % vec == 0) && (sl % vec == 0);
}

static const int kMaxThreads = 1024;
static const int kMaxLdsBytes = 64 * 1024;
static const int kCUs = 256;
static const uint64_t kKeepBytes = 224ull << 20;  // operand bytes a forward leaves in the caches for its backward

static bool threads_ok(int t) { return t == 256 || t == 512 || t == 1024; }

static int check_plan(const qssm_plan* pl, int direction) {
  if (pl == nullptr) return fail(QSSM_EINVAL, "plan is NULL");
  if (pl->direction != direction) return fail(QSSM_EINVAL, "plan was made for the other direction");
  if (pl->B < 0 || pl->L < 0 || pl->D < 0) return fail(QSSM_EINVAL, "negative dimension");
  if (pl->vec != 1 && pl->vec != 2 && pl->vec != 4 && !(pl->vec == 8 && direction == QSSM_FORWARD && dtype_size(pl->in_dtype) == 2))
    return fail(QSSM_EINVAL, "plan.vec must be 1, 2 or 4 (8 for a forward over 16-bit storage)");
  if (pl->steps != 4 && pl->steps != 8) return fail(QSSM_EINVAL, "plan.steps must be 4 or 8");
  if (!threads_ok(pl->threads)) return fail(QSSM_EINVAL, "plan.threads must be 256, 512 or 1024");
  if (pl->g_log2 < 0 || (1 << pl->g_log2) > pl->threads) return fail(QSSM_EINVAL, "plan.g_log2 out of range");
  if (pl->D % pl->vec != 0) return fail(QSSM_EALIGN, "D=%d is not a multiple of plan.vec=%d", pl->D, pl->vec);
  const int ng = pl->threads >> pl->g_log2;
  if (pl->strip_cols != (pl->vec << pl->g_log2) || pl->seg_len != pl->steps * ng)
    return fail(QSSM_EINVAL, "plan geometry is inconsistent");
  if (pl->keep_tiles < 0) return fail(QSSM_EINVAL, "plan.keep_tiles is negative");
  if (pl->B == 0 || pl->L == 0 || pl->D == 0) return 0;
  if (pl->n_strips != (pl->D + pl->strip_cols - 1) / pl->strip_cols ||
      pl->n_seg != (pl->L + pl->seg_len - 1) / pl->seg_len)
    return fail(QSSM_EINVAL, "plan tile counts are inconsistent");
  if (pl->cluster < 1 || (pl->cluster & (pl->cluster - 1)) != 0 ||
      pl->n_super != (pl->n_seg + pl->cluster - 1) / pl->cluster)
    return fail(QSSM_EINVAL, "plan cluster counts are inconsistent");
  const size_t lds = direction == QSSM_FORWARD ? fwd_lds_bytes(pl->threads, pl->vec, pl->strip_cols, pl->cluster)
                                               : bwd_lds_bytes(pl->threads, pl->vec, pl->strip_cols, pl->cluster);
  if ((size_t)pl->lds_bytes != lds || lds > (size_t)kMaxLdsBytes)
    return fail(QSSM_EINVAL, "plan.lds_bytes=%d does not fit the geometry", pl->lds_bytes);
  // Forward lanes write a saved state only at their own first step; backward tiles read one
  // only at the tile's first step.
  if (pl->ckpt_stride <= 0 || pl->seg_len % pl->ckpt_stride != 0 ||
      (direction == QSSM_FORWARD && pl->ckpt_stride % pl->steps != 0) ||
      pl->n_ckpt != (pl->L + pl->ckpt_stride - 1) / pl->ckpt_stride)
    return fail(QSSM_EINVAL, "plan.ckpt_stride=%d does not fit seg_len=%d / steps=%d", pl->ckpt_stride,
                pl->seg_len, pl->steps);
  return 0;
}

// Lane offsets inside a tile are 32-bit: the tile of every tensor must span less than 2 GiB.
static bool tile_span_ok(const qssm_plan* pl, const void* p, int64_t sb, int64_t sl, int elem_bytes) {
  if (p == nullptr) return true;
  if (sl < 0 || sb < 0) return false;
  const int64_t span = ((int64_t)pl->seg_len * sl + pl->strip_cols) * elem_bytes;
  return span < ((int64_t)1 << 31);
}

// One lane behind every launch that uses device-counted epochs: the next launch on the stream gets
// the next flag value.  A kernel of its own, so that every workgroup of the scan has read the
// count before it changes, and so that a captured graph replays correctly (the count lives in device
// memory, not in a kernel argument).  The count never takes the value whose successor is zero: from
// `reset_at` on it starts again at zero (the caller-owned buffers wrap at the end of the 32-bit range;
// the library's own scratch array wraps earlier, after its workspace has been wiped).
static const unsigned kCountWrapAt = 0xfffffffeu;
__global__ void count_launch_kernel(unsigned* count, unsigned reset_at) {
  *count = launch_count_next(*count, reset_at);
}

static void fill_geometry(Geometry* g, const qssm_plan* pl, void* control, void* workspace, uint32_t epoch) {
  g->B = pl->B;
  g->L = pl->L;
  g->D = pl->D;
  g->g_log2 = pl->g_log2;
  g->n_strips = pl->n_strips;
  g->n_chains = pl->B * pl->n_strips;
  g->n_seg = pl->n_seg;
  g->seg_len = pl->seg_len;
  g->cluster = pl->cluster;
  g->n_super = pl->n_super;
  g->ckpt_stride = pl->ckpt_stride;
  g->n_ckpt = pl->n_ckpt;
  g->keep_from = pl->n_seg - (pl->keep_tiles < pl->n_seg ? pl->keep_tiles : pl->n_seg);
  g->epoch = epoch;
  // epoch 0: the launches are counted in the control block itself (see count_launch_kernel)
  g->launch_count = epoch != 0 ? nullptr : (const unsigned*)((const char*)control + kLaunchCountOffset);
  char* ws = (char*)workspace;
  g->status = (int*)control;
  g->tickets = (unsigned*)((char*)control + kStatusBytes);
  g->maps = (unsigned long long*)ws;
  g->states = (unsigned long long*)(ws + ws_states_offset((uint64_t)g->n_chains, (uint64_t)g->n_seg,
                                                          (uint64_t)pl->strip_cols));
}

}  // namespace qssm

using namespace qssm;

// What a gated launch has beyond a plain one: the second factor of c and, backwards, where its gradient goes.
struct GateExtras {
  const void* c2;
  qssm_strides sc2;
  void* dc2;
  qssm_strides sdc2;
};

// What a launch tells its kernel table about gating: the plan's compute dtype for a gated launch.
static int gated_code(const qssm_plan* plan, const GateExtras* gate) {
  return gate == nullptr ? kNotGated : plan->compute_dtype;
}

static int forward_launch(const qssm_plan* plan, const void* x, qssm_strides sx, const void* a, qssm_strides sa,
                          const void* b, qssm_strides sb, const void* c, qssm_strides sc, void* y, qssm_strides sy,
                          float* h_out, qssm_strides sh, float* ckpt, const float* h_init, float* h_final,
                          void* control, uint64_t control_size, void* workspace, uint64_t workspace_bytes,
                          uint32_t epoch, unsigned count_reset_at, void* stream, const GateExtras* gate = nullptr);
static int backward_launch(const qssm_plan* plan, const void* x, qssm_strides sx, const void* a, qssm_strides sa,
                           const void* b, qssm_strides sb, const void* c, qssm_strides sc, const void* dy,
                           qssm_strides sdy, const float* h, qssm_strides sh, const float* ckpt, const float* h_init,
                           const float* dh_final, float* dh_init, void* dx, qssm_strides sdx, void* da,
                           qssm_strides sda, void* db, qssm_strides sdb, void* dc, qssm_strides sdc, void* control,
                           uint64_t control_size, void* workspace, uint64_t workspace_bytes, uint32_t epoch,
                           void* stream, const GateExtras* gate = nullptr);

extern "C" {

int qssm_version(void) { return QSSM_VERSION; }

const char* qssm_error_string(void) { return g_err; }

int qssm_plan_scan(int32_t B, int32_t L, int32_t D, int32_t in_dtype, int32_t out_dtype, int32_t direction,
                   int32_t align_elems, int32_t ckpt_stride, qssm_plan* plan) {
  return qssm_plan_scan_tuned(B, L, D, in_dtype, out_dtype, direction, align_elems, ckpt_stride, 0, plan);
}

// The gated kernels exist in one shape: 4 columns (8 bytes of 16-bit storage) and 8 steps per lane, 256 lanes,
// rows of 64 or 32 lanes, clusters of at most two tiles (the backward's three LDS-resident operands leave LDS
// for no more neighbour maps).
int qssm_plan_scan_gated(int32_t B, int32_t L, int32_t D, int32_t dtype, int32_t compute_dtype, int32_t out_dtype,
                         int32_t direction, int32_t align_elems, int32_t ckpt_stride, qssm_plan* plan) {
  const int es = dtype_size(dtype);
  if (es == 0 || dtype_size(compute_dtype) == 0) return fail(QSSM_EINVAL, "unknown dtype code");
  if (es == 2 && compute_dtype != dtype)
    return fail(QSSM_EINVAL, "16-bit projections are their own compute dtype");
  if (es == 4 && out_dtype != QSSM_F32)
    return fail(QSSM_EINVAL, "the gated scan over fp32 projections stores y and dy as fp32");
  // 8 bytes per lane and 8 steps per lane, 256 lanes: 4 columns of 16-bit storage, 2 of fp32
  const int vec = 8 / es;
  if (D % 4 != 0 || (align_elems * es) % 16 != 0 || D < 128)
    return fail(QSSM_EALIGN, "the gated scan needs D >= 128, a multiple of 4, and 16-byte aligned rows");
  const int32_t kGatedTune = (8 << 8) | (vec << 16) | (1 << 24);
  // The row width comes from a plan without a given spacing of saved states, so that the forward (which is handed
  // the backward's tile length as that spacing) and the backward (which is handed it back) agree on it; the gated
  // kernels exist for rows of 32 and 64 lanes.
  int rc = qssm_plan_scan_tuned(B, L, D, dtype, out_dtype, direction, align_elems, 0, kGatedTune, plan);
  if (rc != 0) return rc;
  if (B == 0 || L == 0) {
    rc = qssm_plan_scan_tuned(B, L, D, dtype, out_dtype, direction, align_elems, ckpt_stride, kGatedTune, plan);
    if (rc == 0) plan->compute_dtype = compute_dtype;
    return rc;
  }
  const int g_log2 = plan->g_log2 > 6 ? 6 : (plan->g_log2 < 5 ? 5 : plan->g_log2);
  if (g_log2 != plan->g_log2 || ckpt_stride != 0)
    rc = qssm_plan_scan_tuned(B, L, D, dtype, out_dtype, direction, align_elems, ckpt_stride,
                              kGatedTune | (g_log2 + 1), plan);
  if (rc == 0 && plan->cluster > 2)   // same strips, more hand-overs, less LDS
    rc = qssm_plan_scan_tuned(B, L, D, dtype, out_dtype, direction, align_elems, ckpt_stride,
                              kGatedTune | (g_log2 + 1) | (2 << 28), plan);
  if (rc != 0) return rc;
  plan->compute_dtype = compute_dtype;
  if (plan->vec != vec || plan->steps != 8 || plan->threads != 256 || (plan->g_log2 != 6 && plan->g_log2 != 5) ||
      plan->cluster > 2)
    return fail(QSSM_EINVAL, "no gated geometry for this shape");
  return 0;
}

int qssm_plan_scan_tuned(int32_t B, int32_t L, int32_t D, int32_t in_dtype, int32_t out_dtype, int32_t direction,
                         int32_t align_elems, int32_t ckpt_stride, int32_t tune, qssm_plan* plan) {
  if (plan == nullptr) return fail(QSSM_EINVAL, "plan is NULL");
  if (B < 0 || L < 0 || D < 0) return fail(QSSM_EINVAL, "negative dimension");
  if (direction != QSSM_FORWARD && direction != QSSM_BACKWARD) return fail(QSSM_EINVAL, "bad direction");
  const int es = dtype_size(in_dtype), os = dtype_size(out_dtype);
  if (es == 0 || os == 0) return fail(QSSM_EINVAL, "unknown dtype code");
  if (direction == QSSM_FORWARD ? find_fwd_launcher(in_dtype, out_dtype) == nullptr
                                : find_bwd_launcher(in_dtype, out_dtype) == nullptr)
    return fail(QSSM_EINVAL, "dtype pair (in=%d, out=%d) is not built; cast on the host", in_dtype, out_dtype);
  if (align_elems < 1) align_elems = 1;

  memset(plan, 0, sizeof(*plan));
  plan->B = B;
  plan->L = L;
  plan->D = D;
  plan->in_dtype = in_dtype;
  plan->out_dtype = out_dtype;
  plan->compute_dtype = in_dtype;
  plan->direction = direction;

  // Widest lane vector the alignment allows: 8 bytes per lane for 16-bit storage, 16 for fp32
  // forward; the backward keeps 5 operands + h in registers, so fp32 stays at 8 bytes there.
  int vec = 4;
  if (es == 4 && direction == QSSM_BACKWARD) vec = 2;
  const int tune_vec = (tune >> 16) & 0xff;
  if (tune_vec == 1 || tune_vec == 2) vec = tune_vec < vec ? tune_vec : vec;
  // The forward over 16-bit storage takes 16 bytes per lane (8 columns) when the launch is large enough to fill the
  // GPU with such tiles: half the wavefronts per tile for the same bytes, and every load, store and LDS access
  // twice as wide (bf16 B=8 L=4096 D=2048: 124 us against 130 with 8 bytes per lane).  Its register footprint
  // (a, b, x of 8 steps: 96 registers) does not leave room for the backward's rebuilt states, so the backward
  // stays at 8 bytes per lane (16 bytes at 4 steps per lane measured 240 us against 220).
  const bool wide_ok = direction == QSSM_FORWARD && es == 2 && align_elems % 8 == 0 && D % 8 == 0;
  // It pays from about a dozen tiles per compute unit on (bf16 B=12 L=4096 D=2048: 179 us against 195; B=16
  // L=2048 D=1024, 2048 tiles: 76 against 71), and not where few chains over a long sequence call for rows of half
  // the width further down (fp16 B=1 L=65536 D=4096: 508 against 491 with 8 bytes per lane and 512 lanes).
  const int64_t wide_chains = (int64_t)B * ((D + 255) / 256);
  const bool wide_auto = direction == QSSM_FORWARD && tune_vec == 0 && os == 2 && D >= 256 &&
                         wide_chains * ((L + 63) / 64) >= 12 * kCUs && !(wide_chains < 32 && L >= 256 * 64);
  if (wide_ok && (tune_vec == 8 || wide_auto)) vec = 8;
  while (vec > 1 && (align_elems % vec != 0 || (D > 0 && D % vec != 0))) vec >>= 1;
  plan->vec = vec;

  // Steps per lane: 8.  Fewer steps mean more, shorter tiles, and every tile pays the same fixed
  // hand-over cost; 8 steps of five operands still fit the register file at two waves per SIMD.
  int steps = 8;
  const int tune_steps = (tune >> 8) & 0xff;
  if (tune_steps == 4 || tune_steps == 8) steps = tune_steps;

  // Lanes per row: 512-byte row pieces (what HBM needs to stream at full rate) when D allows,
  // never more lanes than the row has vectors.  Workgroup: 256 lanes; small workgroups overlap
  // each other's waits best, and clusters (below) keep the number of serial hand-overs down.
  const int cap = lanes_cap(D, vec);
  int g = 512 / (vec * es);
  if (g > cap) g = cap;
  int threads = 256;
  // The forward for 16-bit storage keeps c in LDS when rows can be fetched 16 bytes at a time, which
  // leaves room for two 512-lane workgroups per compute unit: tiles twice as long, half the hand-overs.
  if (direction == QSSM_FORWARD && es == 2 && vec == 4 && steps == 8 && align_elems % 8 == 0) threads = 512;
  if (vec == 8) threads = 256;
  const int tune_g = (tune & 0xff) - 1, tune_t = (tune >> 24) & 0xf;
  const bool fixed_g = tune_g >= 0 && tune_g <= 10, fixed_t = tune_t >= 1 && tune_t <= 3;
  if (fixed_g) g = 1 << tune_g;
  if (fixed_t) threads = 256 << (tune_t - 1);
  if (vec == 1 && threads != 256) threads = 256;
  if (g > threads) g = threads;
  auto tiles = [&](int gg, int tt) -> int64_t {
    const int64_t strips = (D + (int64_t)gg * vec - 1) / ((int64_t)gg * vec);
    const int64_t seg = (int64_t)steps * (tt / gg);
    return (int64_t)B * strips * ((L + seg - 1) / seg);
  };
  if (B > 0 && L > 0 && D > 0) {
    const int64_t lp2 = pow2_ceil(L);
    // A tile longer than the sequence only idles lanes: shed time groups first.
    auto fit_threads = [&]() {
      if (!fixed_t)
        while (threads > 256 && threads / 2 >= g && (int64_t)steps * (threads / 2 / g) >= lp2) threads >>= 1;
    };
    fit_threads();
    // Small problems: rather more workgroups than idle compute units.  Narrow the strips first
    // (more chains, no extra hand-overs), then cut the tiles shorter in time.
    if (!fixed_g) {
      while (g * vec * es > 128 && g > 1 && tiles(g, threads) < 2 * kCUs) {
        g >>= 1;
        fit_threads();
      }
    }
    if (!fixed_t)
      while (threads > 256 && threads / 2 >= g && tiles(g, threads) < 2 * kCUs) threads >>= 1;
    // Few chains and a long sequence (16-bit storage): every chain then has dozens of tiles in flight, its
    // clusters are long and every tile reads the maps of the tiles before it.  Twice the chains at 256-byte
    // row pieces is the better trade (B=1 L=65536 D=4096: backward 932 us against 998 us, forward 531
    // against 548).
    if (!fixed_g && es == 2 && g * vec * es == 512) {
      const int64_t strips = (D + (int64_t)g * vec - 1) / ((int64_t)g * vec);
      const int64_t seg = (int64_t)steps * (threads / g);
      if ((int64_t)B * strips < 32 && L >= 256 * seg) g >>= 1;
    }
    // Very short sequences: widen the rows instead of idling most time groups of a workgroup.
    if (!fixed_g)
      while (g < cap && g < threads && (int64_t)steps * (threads / g) / 2 >= lp2) g <<= 1;
  }
  if (ckpt_stride > 0) {
    // A tile must cover a whole number of saved-state intervals and a forward lane must not
    // straddle one.
    if ((ckpt_stride & (ckpt_stride - 1)) != 0 || ckpt_stride < 4)
      return fail(QSSM_EINVAL, "ckpt_stride=%d must be a power of two >= 4", ckpt_stride);
    if (direction == QSSM_FORWARD && ckpt_stride % steps != 0) steps = 4;
    // Longer tiles first through more lanes (as far as the kernels and the caller's choice go), then through
    // narrower rows.
    const int most_threads = (direction == QSSM_BACKWARD && vec == 4 && steps == 8) ? 512 : kMaxThreads;
    while (steps * (threads / g) < ckpt_stride && !fixed_t && threads < most_threads && vec > 1 && vec < 8) threads <<= 1;
    while (steps * (threads / g) < ckpt_stride && g > 1) g >>= 1;
    if ((steps * (threads / g)) % ckpt_stride != 0)
      return fail(QSSM_EINVAL, "ckpt_stride=%d does not fit any tile length", ckpt_stride);
  }
  // Wide workgroups exist for vec >= 2 only, and the 1024-lane backward at 4 columns per lane
  // only at 4 steps (register file).
  if (direction == QSSM_BACKWARD && vec == 4 && steps == 8 && threads == 1024) threads = 512;
  if (g > threads) g = threads;
  plan->steps = steps;
  plan->threads = threads;
  plan->g_log2 = ilog2(g);
  plan->strip_cols = vec << plan->g_log2;
  plan->seg_len = steps * (threads >> plan->g_log2);
  if (ckpt_stride > 0 && plan->seg_len % ckpt_stride != 0)
    return fail(QSSM_EINVAL, "ckpt_stride=%d does not divide seg_len=%d", ckpt_stride, plan->seg_len);
  plan->ckpt_stride = ckpt_stride > 0 ? ckpt_stride : plan->seg_len;
  plan->cluster = 1;
  if (B == 0 || L == 0 || D == 0) {
    plan->lds_bytes = (int32_t)(direction == QSSM_FORWARD ? fwd_lds_bytes(threads, vec, plan->strip_cols, 1)
                                                          : bwd_lds_bytes(threads, vec, plan->strip_cols, 1));
    return 0;
  }
  plan->n_strips = (D + plan->strip_cols - 1) / plan->strip_cols;
  plan->n_seg = (L + plan->seg_len - 1) / plan->seg_len;
  plan->n_ckpt = (L + plan->ckpt_stride - 1) / plan->ckpt_stride;

  // Cluster size R.  Each cluster boundary is one serial hand-over (about 2.1 us forward, 1.8 us backward under
  // load on MI355X) that every chain pays in turn; inside a cluster a tile reads the maps of all earlier tiles,
  // which costs traffic and LDS (measured against R = 2 on bf16 B=8 L=4096 D=2048: forward +2 % at R = 4 and
  // +3.5 % at R = 8; backward -0.7 % at R = 4, whose fewer hand-overs outweigh the maps, and +14 % at R = 8; R = 1
  // has no maps at all, -2 %).  A launch takes the longer of its stream time
  // (operands at 5.6 TB/s, with that factor) and its chain (clusters x hand-over): the R with the smaller estimate
  // wins, the smaller R on a tie.  Large launches so get R = 1 or 2, long or narrow ones, whose chains would set
  // the pace, up to 8 (bf16 B=2 L=8192 D=512: forward 84.5 -> 36.3 us, backward 75.6 -> 43.1 us; B=2 L=4096
  // D=2048: 46.9 -> 36.3 and 86.2 -> 68.2 us), and single long sequences of small width 16 or 32, where the maps
  // cost 15 - 40 % (B=1 L=16384 D=256: 28.7 -> 19.4 and 55.9 -> 31.6 us; B=1 L=65536 D=512: 94 -> 74 and
  // 213 -> 158 us).  Single tiles per cluster only with a wide margin (chain within
  // 0.6 of the stream time): bf16 B=16 L=4096 D=2048 forward 233 us against 237, but at B=8 its 64 hand-overs in
  // 116 us would set the pace.
  auto lds_for = [&](int r) -> size_t {
    return direction == QSSM_FORWARD ? fwd_lds_bytes(threads, vec, plan->strip_cols, r)
                                     : bwd_lds_bytes(threads, vec, plan->strip_cols, r);
  };
  int cluster = 1;
  const int tune_r = (tune >> 28) & 0xf;
  if (tune_r >= 1) {
    cluster = 1 << (tune_r - 1);
  } else if (plan->n_seg > 1) {
    static const double kMapCost[2][6] = {{-0.02, 0.0, 0.02, 0.035, 0.15, 0.40}, {-0.02, 0.0, -0.005, 0.14, 0.30, 0.35}};
    const double hop_us = direction == QSSM_FORWARD ? 2.1 : 1.8;
    const double stream_us = (double)B * L * D * (direction == QSSM_FORWARD ? 4 * es + os : 8 * es + os) / 5.6e6;
    double best = 0.0;
    cluster = 0;
    // what the kernels that load operands straight into LDS need on top (16-bit storage): clusters beyond 8 must
    // leave that room, or the launch would fall back to the register-only kernels
    const size_t staging = es != 2 ? 0 : direction == QSSM_FORWARD ? fwd_c_lds_bytes(threads, steps, vec * es)
                                                                    : bwd_cg_lds_bytes(threads, steps);
    for (int k = 0; k < 6; ++k) {
      const int r = 1 << k;
      if (lds_for(r) + (k > 3 ? staging : 0) > (size_t)kMaxLdsBytes) break;
      const double chain_us = (double)((plan->n_seg + r - 1) / r) * hop_us;
      if (r == 1 && chain_us > 0.6 * stream_us) continue;
      const double a = stream_us * (1.0 + kMapCost[direction == QSSM_FORWARD ? 0 : 1][k]);
      const double est = a > chain_us ? a : chain_us;
      if (cluster == 0 || est < best) { best = est; cluster = r; }
    }
    if (cluster == 0) cluster = 1;
  }
  while (cluster > 1 && lds_for(cluster) > (size_t)kMaxLdsBytes) cluster >>= 1;
  if (lds_for(cluster) > (size_t)kMaxLdsBytes) return fail(QSSM_EINVAL, "geometry needs too much LDS");
  plan->cluster = cluster;
  plan->n_super = (plan->n_seg + cluster - 1) / cluster;
  plan->lds_bytes = (int32_t)lds_for(cluster);

  const uint64_t n_chains = (uint64_t)B * plan->n_strips;
  if (n_chains * plan->n_seg > 0x7fffffffull) return fail(QSSM_EINVAL, "shape needs more than 2^31 tiles");
  plan->control_bytes = control_bytes(n_chains);
  plan->workspace_bytes = plan->n_seg > 1 ? ws_total_bytes(n_chains, (uint64_t)plan->n_seg, (uint64_t)plan->n_super,
                                                           (uint64_t)plan->strip_cols)
                                          : 0;
  plan->ckpt_elems = (uint64_t)B * plan->n_ckpt * D;
  // The backward starts where the forward ends.  The last tiles of every chain therefore load their operands with
  // ordinary loads, which leave them in the 256 MiB memory-side cache, as far as seven eighths of it reach; the
  // tiles before them stream past the caches (bf16 B=8 L=4096 D=2048: the last 28 of 64 tiles; with everything at
  // fixed addresses the step takes 347.0 us with none kept, 339.7 with 8, 338.2 with 24 or 32, 343.2 with 48).
  // A launch whose operands fit altogether keeps all of them.
  if (direction == QSSM_FORWARD) {
    const uint64_t per_index = n_chains * (uint64_t)plan->strip_cols * plan->seg_len * 4u * (uint64_t)es;
    const uint64_t keep = kKeepBytes / (per_index > 0 ? per_index : 1);
    plan->keep_tiles = (int32_t)(keep < (uint64_t)plan->n_seg ? keep : (uint64_t)plan->n_seg);
  }
  return 0;
}

int qssm_zero_fill(void* workspace, uint64_t bytes, void* stream) {
  if (workspace == nullptr || bytes == 0) return 0;
  if (((uintptr_t)workspace) % 16 != 0 || bytes % 16 != 0)
    return fail(QSSM_EALIGN, "buffer must be 16-byte aligned and a multiple of 16 bytes");
  const uint64_t n16 = bytes / 16;
  uint64_t blocks = (n16 + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (uint4*)workspace,
                     n16);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e, "fill_zero_kernel launch");
}

int qssm_control_status(const void* control, void* stream, int32_t* status) {
  if (control == nullptr || status == nullptr) return fail(QSSM_EINVAL, "NULL argument");
  hipError_t e = hipMemcpyAsync(status, control, sizeof(int32_t), hipMemcpyDeviceToHost, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "hipMemcpyAsync(status)");
  e = hipStreamSynchronize((hipStream_t)stream);
  return e == hipSuccess ? 0 : hip_fail(e, "hipStreamSynchronize");
}

int qssm_control_status_async(const void* control, int32_t* host_status, void* stream) {
  if (control == nullptr || host_status == nullptr) return fail(QSSM_EINVAL, "NULL argument");
  hipError_t e = hipMemcpyAsync(host_status, control, sizeof(int32_t), hipMemcpyDeviceToHost, (hipStream_t)stream);
  return e == hipSuccess ? 0 : hip_fail(e, "hipMemcpyAsync(status)");
}

int qssm_scan_forward_call(const qssm_forward_call* k) {
  if (k == nullptr) return fail(QSSM_EINVAL, "call is NULL");
  return forward_launch(k->plan, k->x, k->sx, k->a, k->sa, k->b, k->sb, k->c, k->sc, k->y, k->sy, k->h_out, k->sh,
                        k->ckpt, k->h_init, k->h_final, k->control, k->control_size, k->workspace,
                        k->workspace_bytes, k->epoch, kCountWrapAt, k->stream);
}

int qssm_scan_backward_call(const qssm_backward_call* k) {
  if (k == nullptr) return fail(QSSM_EINVAL, "call is NULL");
  return qssm_scan_backward_carry(k->plan, k->x, k->sx, k->a, k->sa, k->b, k->sb, k->c, k->sc, k->dy, k->sdy, k->h,
                                  k->sh, k->ckpt, k->h_init, k->dh_final, k->dh_init, k->dx, k->sdx, k->da, k->sda,
                                  k->db, k->sdb, k->dc, k->sdc, k->control, k->control_size, k->workspace,
                                  k->workspace_bytes, k->epoch, k->stream);
}

int qssm_scan_forward(const qssm_plan* plan, const void* x, qssm_strides sx, const void* a, qssm_strides sa,
                      const void* b, qssm_strides sb, const void* c, qssm_strides sc, void* y, qssm_strides sy,
                      float* h_out, qssm_strides sh, float* ckpt, void* control, uint64_t control_size,
                      void* workspace, uint64_t workspace_bytes, uint32_t epoch, void* stream) {
  return qssm_scan_forward_carry(plan, x, sx, a, sa, b, sb, c, sc, y, sy, h_out, sh, ckpt, nullptr, nullptr, control,
                                 control_size, workspace, workspace_bytes, epoch, stream);
}

int qssm_scan_forward_carry(const qssm_plan* plan, const void* x, qssm_strides sx, const void* a, qssm_strides sa,
                            const void* b, qssm_strides sb, const void* c, qssm_strides sc, void* y, qssm_strides sy,
                            float* h_out, qssm_strides sh, float* ckpt, const float* h_init, float* h_final,
                            void* control, uint64_t control_size, void* workspace, uint64_t workspace_bytes,
                            uint32_t epoch, void* stream) {
  return forward_launch(plan, x, sx, a, sa, b, sb, c, sc, y, sy, h_out, sh, ckpt, h_init, h_final, control,
                        control_size, workspace, workspace_bytes, epoch, kCountWrapAt, stream);
}

}  // extern "C"

static int forward_launch(const qssm_plan* plan, const void* x, qssm_strides sx, const void* a, qssm_strides sa,
                          const void* b, qssm_strides sb, const void* c, qssm_strides sc, void* y, qssm_strides sy,
                          float* h_out, qssm_strides sh, float* ckpt, const float* h_init, float* h_final,
                          void* control, uint64_t control_size, void* workspace, uint64_t workspace_bytes,
                          uint32_t epoch, unsigned count_reset_at, void* stream, const GateExtras* gate) {
  int rc = check_plan(plan, QSSM_FORWARD);
  if (rc != 0) return rc;
  if (plan->B == 0 || plan->L == 0 || plan->D == 0) return 0;
  if (x == nullptr || a == nullptr || b == nullptr) return fail(QSSM_EINVAL, "x, a, b must not be NULL");
  if (y == nullptr && h_out == nullptr && ckpt == nullptr && h_final == nullptr)
    return fail(QSSM_EINVAL, "no output requested");
  fwd_launch_fn fn = find_fwd_launcher(plan->in_dtype, plan->out_dtype);
  if (fn == nullptr) return fail(QSSM_EINVAL, "dtype pair is not built");
  const int es = dtype_size(plan->in_dtype), os = dtype_size(plan->out_dtype), v = plan->vec;
  if (!aligned_to(x, sx.b, sx.l, es, v) || !aligned_to(a, sa.b, sa.l, es, v) || !aligned_to(b, sb.b, sb.l, es, v) ||
      !aligned_to(c, sc.b, sc.l, es, v) || !aligned_to(y, sy.b, sy.l, os, v) ||
      !aligned_to(h_out, sh.b, sh.l, 4, v) || !aligned_to(ckpt, 0, 0, 4, v) || !aligned_to(h_init, 0, 0, 4, v) ||
      !aligned_to(h_final, 0, 0, 4, v))
    return fail(QSSM_EALIGN, "a pointer or stride is not aligned to plan.vec=%d elements", v);
  if (control == nullptr || control_size < plan->control_bytes)
    return fail(QSSM_EWORKSPACE, "control block has %llu bytes, plan needs %llu", (unsigned long long)control_size,
                (unsigned long long)plan->control_bytes);
  if (plan->workspace_bytes > 0 && (workspace == nullptr || workspace_bytes < plan->workspace_bytes))
    return fail(QSSM_EWORKSPACE, "workspace has %llu bytes, plan needs %llu", (unsigned long long)workspace_bytes,
                (unsigned long long)plan->workspace_bytes);
  if (((uintptr_t)control) % 8 != 0 || ((uintptr_t)workspace) % 8 != 0)
    return fail(QSSM_EALIGN, "control block and workspace must be 8-byte aligned");

  if (!tile_span_ok(plan, x, sx.b, sx.l, es) || !tile_span_ok(plan, a, sa.b, sa.l, es) ||
      !tile_span_ok(plan, b, sb.b, sb.l, es) || !tile_span_ok(plan, c, sc.b, sc.l, es) ||
      !tile_span_ok(plan, y, sy.b, sy.l, os) || !tile_span_ok(plan, h_out, sh.b, sh.l, 4))
    return fail(QSSM_EINVAL, "a time stride is negative or too large for 32-bit tile offsets; pass a contiguous copy");

  FwdArgs args;
  fill_geometry(&args.g, plan, control, workspace, epoch);
  args.x = x; args.a = a; args.b = b; args.c = c; args.y = y; args.h_out = h_out; args.ckpt = ckpt;
  args.h_init = h_init; args.h_final = h_final;
  args.x_sb = sx.b; args.x_sl = sx.l; args.a_sb = sa.b; args.a_sl = sa.l;
  args.b_sb = sb.b; args.b_sl = sb.l; args.c_sb = sc.b; args.c_sl = sc.l;
  args.y_sb = sy.b; args.y_sl = sy.l; args.h_sb = sh.b; args.h_sl = sh.l;
  const dim3 grid((unsigned)((uint64_t)args.g.n_chains * args.g.n_seg));
  // c can live in LDS instead of registers when a row of the strip is one wavefront of 8-byte lanes
  // and c's rows can be fetched 16 bytes at a time.
  size_t lds = (size_t)plan->lds_bytes;
  // (8 bytes per lane: 4 columns of 16-bit storage; 2 columns of fp32 only in the gated scan's kernels)
  const bool narrow_rows = v * es == 8 && (es == 2 || gate != nullptr) && (plan->g_log2 == 6 || plan->g_log2 == 5) &&
                           (plan->threads == 256 || plan->threads == 512);
  const bool wide_rows = es == 2 && v == 8 && (plan->threads == 256 || plan->threads == 512);   // every lane fetches its own 16 bytes
  bool c_in_lds = y != nullptr && c != nullptr && ((narrow_rows && plan->steps == 8) || wide_rows) &&
                  ((uintptr_t)c) % 16 == 0 && (sc.b * es) % 16 == 0 && (sc.l * es) % 16 == 0 &&
                  lds + fwd_c_lds_bytes(plan->threads, plan->steps, v * es) <= (size_t)kMaxLdsBytes;
  if (c_in_lds) lds += fwd_c_lds_bytes(plan->threads, plan->steps, v * es);
  args.c2 = nullptr; args.c2_sb = args.c2_sl = 0;
  if (gate != nullptr && dtype_size(plan->compute_dtype) == 0) return fail(QSSM_EINVAL, "plan.compute_dtype is not a dtype code");
  if (gate != nullptr) {
    // Ca and Cb both go through LDS: the same conditions again for Cb, and room for the second array
    if (!c_in_lds || !narrow_rows || plan->threads != 256 || gate->c2 == nullptr || ((uintptr_t)gate->c2) % 16 != 0 ||
        (gate->sc2.b * es) % 16 != 0 || (gate->sc2.l * es) % 16 != 0 || !tile_span_ok(plan, gate->c2, gate->sc2.b, gate->sc2.l, es) ||
        lds + fwd_c_lds_bytes(plan->threads, plan->steps, v * es) > (size_t)kMaxLdsBytes)
      return fail(QSSM_EALIGN, "gated scan needs a plan of qssm_plan_scan_gated, y, and Ca, Cb with 16-byte aligned rows");
    lds += fwd_c_lds_bytes(plan->threads, plan->steps, v * es);
    args.c2 = gate->c2; args.c2_sb = gate->sc2.b; args.c2_sl = gate->sc2.l;
  }
  if (!fn(args, plan->vec, plan->steps, plan->threads, c_in_lds, gated_code(plan, gate), grid, lds, (hipStream_t)stream))
    return fail(QSSM_EINVAL, "no forward kernel for vec=%d steps=%d threads=%d", plan->vec, plan->steps, plan->threads);
  if (epoch == 0 && plan->n_seg > 1)
    hipLaunchKernelGGL(count_launch_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream,
                       (unsigned*)((char*)control + kLaunchCountOffset), count_reset_at);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e, "scan_fwd_kernel launch");
}

extern "C" {

int qssm_scan_backward(const qssm_plan* plan, const void* x, qssm_strides sx, const void* a, qssm_strides sa,
                       const void* b, qssm_strides sb, const void* c, qssm_strides sc, const void* dy,
                       qssm_strides sdy, const float* h, qssm_strides sh, const float* ckpt, void* dx,
                       qssm_strides sdx, void* da, qssm_strides sda, void* db, qssm_strides sdb, void* dc,
                       qssm_strides sdc, void* control, uint64_t control_size, void* workspace,
                       uint64_t workspace_bytes, uint32_t epoch, void* stream) {
  return qssm_scan_backward_carry(plan, x, sx, a, sa, b, sb, c, sc, dy, sdy, h, sh, ckpt, nullptr, nullptr, nullptr, dx,
                                  sdx, da, sda, db, sdb, dc, sdc, control, control_size, workspace, workspace_bytes,
                                  epoch, stream);
}

int qssm_scan_backward_carry(const qssm_plan* plan, const void* x, qssm_strides sx, const void* a, qssm_strides sa,
                             const void* b, qssm_strides sb, const void* c, qssm_strides sc, const void* dy,
                             qssm_strides sdy, const float* h, qssm_strides sh, const float* ckpt,
                             const float* h_init, const float* dh_final, float* dh_init, void* dx, qssm_strides sdx,
                             void* da, qssm_strides sda, void* db, qssm_strides sdb, void* dc, qssm_strides sdc,
                             void* control, uint64_t control_size, void* workspace, uint64_t workspace_bytes,
                             uint32_t epoch, void* stream) {
  return backward_launch(plan, x, sx, a, sa, b, sb, c, sc, dy, sdy, h, sh, ckpt, h_init, dh_final, dh_init, dx, sdx, da,
                         sda, db, sdb, dc, sdc, control, control_size, workspace, workspace_bytes, epoch, stream);
}

}  // extern "C"

static int backward_launch(const qssm_plan* plan, const void* x, qssm_strides sx, const void* a, qssm_strides sa,
                           const void* b, qssm_strides sb, const void* c, qssm_strides sc, const void* dy,
                           qssm_strides sdy, const float* h, qssm_strides sh, const float* ckpt, const float* h_init,
                           const float* dh_final, float* dh_init, void* dx, qssm_strides sdx, void* da,
                           qssm_strides sda, void* db, qssm_strides sdb, void* dc, qssm_strides sdc, void* control,
                           uint64_t control_size, void* workspace, uint64_t workspace_bytes, uint32_t epoch,
                           void* stream, const GateExtras* gate) {
  int rc = check_plan(plan, QSSM_BACKWARD);
  if (rc != 0) return rc;
  if (plan->B == 0 || plan->L == 0 || plan->D == 0) return 0;
  if (x == nullptr || a == nullptr || b == nullptr || c == nullptr || dy == nullptr)
    return fail(QSSM_EINVAL, "x, a, b, c, dy must not be NULL");
  if ((h == nullptr) == (ckpt == nullptr)) return fail(QSSM_EINVAL, "pass exactly one of h and ckpt");
  bwd_launch_fn fn = find_bwd_launcher(plan->in_dtype, plan->out_dtype);
  if (fn == nullptr) return fail(QSSM_EINVAL, "dtype pair is not built");
  const int es = dtype_size(plan->in_dtype), os = dtype_size(plan->out_dtype), v = plan->vec;
  if (!aligned_to(x, sx.b, sx.l, es, v) || !aligned_to(a, sa.b, sa.l, es, v) || !aligned_to(b, sb.b, sb.l, es, v) ||
      !aligned_to(c, sc.b, sc.l, es, v) || !aligned_to(dy, sdy.b, sdy.l, os, v) ||
      !aligned_to(h, sh.b, sh.l, 4, v) || !aligned_to(ckpt, 0, 0, 4, v) || !aligned_to(h_init, 0, 0, 4, v) ||
      !aligned_to(dh_final, 0, 0, 4, v) || !aligned_to(dh_init, 0, 0, 4, v) || !aligned_to(dx, sdx.b, sdx.l, es, v) ||
      !aligned_to(da, sda.b, sda.l, es, v) || !aligned_to(db, sdb.b, sdb.l, es, v) ||
      !aligned_to(dc, sdc.b, sdc.l, es, v))
    return fail(QSSM_EALIGN, "a pointer or stride is not aligned to plan.vec=%d elements", v);
  if (control == nullptr || control_size < plan->control_bytes)
    return fail(QSSM_EWORKSPACE, "control block has %llu bytes, plan needs %llu", (unsigned long long)control_size,
                (unsigned long long)plan->control_bytes);
  if (plan->workspace_bytes > 0 && (workspace == nullptr || workspace_bytes < plan->workspace_bytes))
    return fail(QSSM_EWORKSPACE, "workspace has %llu bytes, plan needs %llu", (unsigned long long)workspace_bytes,
                (unsigned long long)plan->workspace_bytes);
  if (((uintptr_t)control) % 8 != 0 || ((uintptr_t)workspace) % 8 != 0)
    return fail(QSSM_EALIGN, "control block and workspace must be 8-byte aligned");

  if (!tile_span_ok(plan, x, sx.b, sx.l, es) || !tile_span_ok(plan, a, sa.b, sa.l, es) ||
      !tile_span_ok(plan, b, sb.b, sb.l, es) || !tile_span_ok(plan, c, sc.b, sc.l, es) ||
      !tile_span_ok(plan, dy, sdy.b, sdy.l, os) || !tile_span_ok(plan, dx, sdx.b, sdx.l, es) ||
      !tile_span_ok(plan, da, sda.b, sda.l, es) || !tile_span_ok(plan, db, sdb.b, sdb.l, es) ||
      !tile_span_ok(plan, dc, sdc.b, sdc.l, es))
    return fail(QSSM_EINVAL, "a time stride is negative or too large for 32-bit tile offsets; pass a contiguous copy");

  BwdArgs args;
  fill_geometry(&args.g, plan, control, workspace, epoch);
  args.x = x; args.a = a; args.b = b; args.c = c; args.dy = dy; args.h = h; args.ckpt = ckpt;
  args.h_init = h_init; args.dh_final = dh_final; args.dh_init = dh_init;
  args.dx = dx; args.da = da; args.db = db; args.dc = dc;
  args.x_sb = sx.b; args.x_sl = sx.l; args.a_sb = sa.b; args.a_sl = sa.l;
  args.b_sb = sb.b; args.b_sl = sb.l; args.c_sb = sc.b; args.c_sl = sc.l;
  args.dy_sb = sdy.b; args.dy_sl = sdy.l; args.h_sb = sh.b; args.h_sl = sh.l;
  args.dx_sb = sdx.b; args.dx_sl = sdx.l; args.da_sb = sda.b; args.da_sl = sda.l;
  args.db_sb = sdb.b; args.db_sl = sdb.l; args.dc_sb = sdc.b; args.dc_sl = sdc.l;
  const dim3 grid((unsigned)((uint64_t)args.g.n_chains * args.g.n_seg));
  // c and dy can live in LDS instead of registers when a row of the strip is one wavefront of 8-byte
  // lanes in both and their rows can be fetched 16 bytes at a time.
  size_t lds = (size_t)plan->lds_bytes;
  // (8 bytes per lane: 4 columns of 16-bit storage; 2 columns of fp32, with fp32 dy, only in the gated scan's kernels)
  bool cg_in_lds = ((es == 2 && (os == 2 || os == 4) && v == 4) || (gate != nullptr && es == 4 && os == 4 && v == 2)) &&
                   (plan->g_log2 == 6 || plan->g_log2 == 5) && plan->steps == 8 && plan->threads == 256 &&
                   ((uintptr_t)c) % 16 == 0 && (sc.b * es) % 16 == 0 && (sc.l * es) % 16 == 0 &&
                   ((uintptr_t)dy) % 16 == 0 && (sdy.b * os) % 16 == 0 && (sdy.l * os) % 16 == 0 &&
                   lds + bwd_cg_lds_bytes(plan->threads, plan->steps) <= (size_t)kMaxLdsBytes;
  if (cg_in_lds) lds += bwd_cg_lds_bytes(plan->threads, plan->steps);
  args.c2 = nullptr; args.c2_sb = args.c2_sl = 0; args.dc2 = nullptr; args.dc2_sb = args.dc2_sl = 0;
  if (gate != nullptr && dtype_size(plan->compute_dtype) == 0) return fail(QSSM_EINVAL, "plan.compute_dtype is not a dtype code");
  if (gate != nullptr) {
    // Ca, Cb and dy all go through LDS: the same conditions again for Cb, and room for the third array
    const size_t one = bwd_cg_lds_bytes(plan->threads, plan->steps) / 2;
    if (!cg_in_lds || h != nullptr || gate->c2 == nullptr || ((uintptr_t)gate->c2) % 16 != 0 || (gate->sc2.b * es) % 16 != 0 ||
        (gate->sc2.l * es) % 16 != 0 || !tile_span_ok(plan, gate->c2, gate->sc2.b, gate->sc2.l, es) ||
        !aligned_to(gate->dc2, gate->sdc2.b, gate->sdc2.l, es, v) || !tile_span_ok(plan, gate->dc2, gate->sdc2.b, gate->sdc2.l, es) ||
        lds + one > (size_t)kMaxLdsBytes)
      return fail(QSSM_EALIGN, "gated scan needs a plan of qssm_plan_scan_gated, dy stored as the projections are, saved "
                               "states, and Ca, Cb, dy with 16-byte aligned rows");
    lds += one;
    args.c2 = gate->c2; args.c2_sb = gate->sc2.b; args.c2_sl = gate->sc2.l;
    args.dc2 = gate->dc2; args.dc2_sb = gate->sdc2.b; args.dc2_sl = gate->sdc2.l;
  }
  if (!fn(args, plan->vec, plan->steps, plan->threads, cg_in_lds, gated_code(plan, gate), grid, lds, (hipStream_t)stream))
    return fail(QSSM_EINVAL, "no backward kernel for vec=%d steps=%d threads=%d", plan->vec, plan->steps, plan->threads);
  if (epoch == 0 && plan->n_seg > 1)
    hipLaunchKernelGGL(count_launch_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream,
                       (unsigned*)((char*)control + kLaunchCountOffset), kCountWrapAt);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e, "scan_bwd_kernel launch");
}

extern "C" {

int qssm_scan_gated_forward(const qssm_plan* plan, const void* A_pre, qssm_strides sA, const void* B_in, qssm_strides sB,
                            const void* Ca, qssm_strides sCa, const void* Cb, qssm_strides sCb, const void* D_pre,
                            qssm_strides sD, void* y, qssm_strides sy, float* ckpt, void* control,
                            uint64_t control_size, void* workspace, uint64_t workspace_bytes, uint32_t epoch,
                            void* stream) {
  if (A_pre == nullptr || B_in == nullptr || Ca == nullptr || Cb == nullptr || D_pre == nullptr || y == nullptr)
    return fail(QSSM_EINVAL, "the five projection outputs and y must not be NULL");
  const GateExtras gate{Cb, sCb, nullptr, qssm_strides{0, 0}};
  return forward_launch(plan, B_in, sB, A_pre, sA, D_pre, sD, Ca, sCa, y, sy, nullptr, qssm_strides{0, 0}, ckpt, nullptr,
                        nullptr, control, control_size, workspace, workspace_bytes, epoch, kCountWrapAt, stream, &gate);
}

int qssm_scan_gated_backward(const qssm_plan* plan, const void* A_pre, qssm_strides sA, const void* B_in,
                             qssm_strides sB, const void* Ca, qssm_strides sCa, const void* Cb, qssm_strides sCb,
                             const void* D_pre, qssm_strides sD, const void* dy, qssm_strides sdy, const float* ckpt,
                             void* dA_pre, qssm_strides sdA, void* dB_in, qssm_strides sdB, void* dCa,
                             qssm_strides sdCa, void* dCb, qssm_strides sdCb, void* dD_pre, qssm_strides sdD,
                             void* control, uint64_t control_size, void* workspace, uint64_t workspace_bytes,
                             uint32_t epoch, void* stream) {
  if (A_pre == nullptr || B_in == nullptr || Ca == nullptr || Cb == nullptr || D_pre == nullptr || dy == nullptr ||
      ckpt == nullptr)
    return fail(QSSM_EINVAL, "the five projection outputs, dy and the saved states must not be NULL");
  const GateExtras gate{Cb, sCb, dCb, sdCb};
  return backward_launch(plan, B_in, sB, A_pre, sA, D_pre, sD, Ca, sCa, dy, sdy, nullptr, qssm_strides{0, 0}, ckpt, nullptr,
                         nullptr, nullptr, dB_in, sdB, dA_pre, sdA, dD_pre, sdD, dCa, sdCa, control, control_size,
                         workspace, workspace_bytes, epoch, stream, &gate);
}

// Widest lane vector (4, 2 or 1 elements) every listed tensor allows.
static int gate_vec(int S, std::initializer_list<std::pair<const void*, int64_t>> tensors, int elem_bytes_in,
                    std::initializer_list<const void*> dense, int elem_bytes_dense) {
  for (int v = 4; v > 1; v >>= 1) {
    bool ok = S % v == 0;
    for (const auto& t : tensors) ok = ok && ((uintptr_t)t.first) % (size_t)(v * elem_bytes_in) == 0 && t.second % v == 0;
    for (const void* d : dense) ok = ok && ((uintptr_t)d) % (size_t)(v * elem_bytes_dense) == 0;
    if (ok) return v;
  }
  return 1;
}

int qssm_gates_forward(const void* A_pre, int64_t ld_a, const void* B_in, int64_t ld_b, const void* Ca, int64_t ld_ca,
                       const void* Cb, int64_t ld_cb, const void* D_pre, int64_t ld_d, void* a, void* x, void* c,
                       void* b, int64_t rows, int32_t S, int32_t in_dtype, int32_t out_dtype, void* stream) {
  const int es = dtype_size(in_dtype), os = dtype_size(out_dtype);
  if (es == 0 || os == 0) return fail(QSSM_EINVAL, "unknown dtype code");
  if (rows < 0 || S < 0) return fail(QSSM_EINVAL, "negative dimension");
  if (rows == 0 || S == 0) return 0;
  if (!A_pre || !B_in || !Ca || !Cb || !D_pre || !a || !x || !c || !b) return fail(QSSM_EINVAL, "NULL tensor");
  if (ld_a < S || ld_b < S || ld_ca < S || ld_cb < S || ld_d < S) return fail(QSSM_EINVAL, "row stride below S");
  GateFwdArgs args{A_pre, B_in, Ca, Cb, D_pre, ld_a, ld_b, ld_ca, ld_cb, ld_d, a, x, c, b, rows, S};
  const int vec = gate_vec(S, {{A_pre, ld_a}, {B_in, ld_b}, {Ca, ld_ca}, {Cb, ld_cb}, {D_pre, ld_d}}, es,
                           {a, x, c, b}, os);
  if (!launch_gates_any(in_dtype, out_dtype, &args, nullptr, vec, (hipStream_t)stream))
    return fail(QSSM_EINVAL, "gate dtype pair (in=%d, out=%d) is not built", in_dtype, out_dtype);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e, "gates_fwd_kernel launch");
}

int qssm_gates_backward(const void* g_a, const void* g_x, const void* g_c, const void* g_b, const void* A_pre,
                        int64_t ld_a, const void* Ca, int64_t ld_ca, const void* Cb, int64_t ld_cb, const void* D_pre,
                        int64_t ld_d, void* dA_pre, void* dB_in, void* dCa, void* dCb, void* dD_pre, int64_t rows,
                        int32_t S, int32_t in_dtype, int32_t out_dtype, void* stream) {
  return qssm_gates_backward_strided(g_a, g_x, g_c, g_b, A_pre, ld_a, Ca, ld_ca, Cb, ld_cb, D_pre, ld_d, dA_pre, dB_in,
                                     dCa, dCb, dD_pre, S, rows, S, in_dtype, out_dtype, stream);
}

int qssm_gates_backward_strided(const void* g_a, const void* g_x, const void* g_c, const void* g_b, const void* A_pre,
                                int64_t ld_a, const void* Ca, int64_t ld_ca, const void* Cb, int64_t ld_cb,
                                const void* D_pre, int64_t ld_d, void* dA_pre, void* dB_in, void* dCa, void* dCb,
                                void* dD_pre, int64_t ld_grad, int64_t rows, int32_t S, int32_t in_dtype,
                                int32_t out_dtype, void* stream) {
  const int es = dtype_size(in_dtype), os = dtype_size(out_dtype);
  if (es == 0 || os == 0) return fail(QSSM_EINVAL, "unknown dtype code");
  if (rows < 0 || S < 0) return fail(QSSM_EINVAL, "negative dimension");
  if (rows == 0 || S == 0) return 0;
  if (!g_a || !g_x || !g_c || !g_b || !A_pre || !Ca || !Cb || !D_pre || !dA_pre || !dB_in || !dCa || !dCb || !dD_pre)
    return fail(QSSM_EINVAL, "NULL tensor");
  if (ld_a < S || ld_ca < S || ld_cb < S || ld_d < S || ld_grad < S) return fail(QSSM_EINVAL, "row stride below S");
  GateBwdArgs args{g_a, g_x, g_c, g_b, A_pre, Ca, Cb, D_pre, ld_a, ld_ca, ld_cb, ld_d,
                   dA_pre, dB_in, dCa, dCb, dD_pre, rows, S, ld_grad};
  int vec = gate_vec(S, {{A_pre, ld_a}, {Ca, ld_ca}, {Cb, ld_cb}, {D_pre, ld_d}, {dA_pre, ld_grad}, {dB_in, ld_grad},
                         {dCa, ld_grad}, {dCb, ld_grad}, {dD_pre, ld_grad}}, es, {g_a, g_x, g_c, g_b}, os);
  if (!launch_gates_any(in_dtype, out_dtype, nullptr, &args, vec, (hipStream_t)stream))
    return fail(QSSM_EINVAL, "gate dtype pair (in=%d, out=%d) is not built", in_dtype, out_dtype);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e, "gates_bwd_kernel launch");
}

int qssm_rmsnorm_forward(const void* x, int64_t ld_x, const void* weight, void* y, float* rstd, int64_t rows,
                         int32_t H, float eps, int32_t dtype, void* stream) {
  const int es = dtype_size(dtype);
  if (es == 0) return fail(QSSM_EINVAL, "unknown dtype code");
  if (rows < 0 || H < 0) return fail(QSSM_EINVAL, "negative dimension");
  if (rows == 0 || H == 0) return 0;
  if (!x || !weight || !y) return fail(QSSM_EINVAL, "NULL tensor");
  if (ld_x < H) return fail(QSSM_EINVAL, "row stride below H");
  if ((int64_t)H * es > 0x7fffffffll) return fail(QSSM_EINVAL, "row too wide");
  NormFwdArgs args{x, ld_x, weight, y, rstd, rows, H, eps};
  const int vec = gate_vec(H, {{x, ld_x}, {weight, H}, {y, H}}, es, {}, es);
  if (!launch_norm_any(dtype, &args, nullptr, vec, 0, nullptr, (hipStream_t)stream))
    return fail(QSSM_EINVAL, "rmsnorm storage type %d is not built", dtype);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e, "rmsnorm_fwd_kernel launch");
}

int qssm_rmsnorm_backward(const void* dy, int64_t ld_dy, const void* x, int64_t ld_x, const void* weight,
                          const float* rstd, void* dx, void* dweight, float* partial, int32_t partial_rows,
                          int64_t rows, int32_t H, float eps, int32_t dtype, void* stream) {
  const int es = dtype_size(dtype);
  if (es == 0) return fail(QSSM_EINVAL, "unknown dtype code");
  if (rows < 0 || H < 0) return fail(QSSM_EINVAL, "negative dimension");
  if (H == 0) return 0;
  if (!dweight || !partial) return fail(QSSM_EINVAL, "NULL tensor");
  if (rows > 0 && (!dy || !x || !weight || !dx)) return fail(QSSM_EINVAL, "NULL tensor");
  if (ld_dy < H || ld_x < H) return fail(QSSM_EINVAL, "row stride below H");
  if ((int64_t)H * es > 0x7fffffffll) return fail(QSSM_EINVAL, "row too wide");
  if (partial_rows < QSSM_RMSNORM_MIN_PARTIAL_ROWS)
    return fail(QSSM_EINVAL, "partial needs at least %d rows of H floats", QSSM_RMSNORM_MIN_PARTIAL_ROWS);
  NormBwdArgs args{dy, ld_dy, x, ld_x, weight, rstd, dx, partial, rows, H, eps};
  const int vec = rows == 0 ? 1 : gate_vec(H, {{dy, ld_dy}, {x, ld_x}, {weight, H}, {dx, H}}, es, {}, es);
  if (!launch_norm_any(dtype, nullptr, &args, vec, partial_rows, dweight, (hipStream_t)stream))
    return fail(QSSM_EINVAL, "rmsnorm storage type %d is not built", dtype);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e, "rmsnorm_bwd_kernel launch");
}

}  // extern "C"

// ---- the forward scan for callers that cannot allocate ----------------------------------------------------
//
// Control block and workspace of this entry point live in one array in the library's device image: nothing is
// allocated, by the caller or here.  Every GPU the library runs on holds its own copy of the array, at its own
// address, until the process ends.  `g_scratch` below is only the host-side handle of that array: its device
// address is asked for once per device (hipGetSymbolAddress) and kept in g_scratch_ptr; host code uses that
// pointer wherever it needs the array's memory.
static const uint64_t kScratchControlBytes = 256u << 10;                  // status, count, up to 4095 chains
static const uint64_t kScratchBytes = (uint64_t)QSSM_STATIC_SCRATCH_BYTES;  // control block + workspace
static const unsigned kScratchWipeAt = 0xfffffff0u;  // launch count from which the array is wiped and the count restarts
static __device__ __align__(256) unsigned char g_scratch[QSSM_STATIC_SCRATCH_BYTES];

static const int kMaxDevices = 64;
static unsigned char* g_scratch_ptr[kMaxDevices];   // per device: where that device keeps the array
static std::mutex g_scratch_mutex;

// Before every launch on the array: status word and ticket counters back to zero (a launch that failed may have
// left them dirty), the launch count kept.  Once the count has reached kScratchWipeAt the words of the whole
// array are cleared as well, and the counting kernel behind the scan then restarts the count, so that no word of
// an old launch can ever carry the flag value of a new one.  Every workgroup reads the count before anyone
// rewrites the word beside it with the same value.
__global__ void __launch_bounds__(256) scratch_prologue_kernel(uint4* scratch, uint64_t control16, uint64_t total16) {
  static_assert(kLaunchCountOffset == 4, "the count is the second word of the control block's first 16 bytes");
  const unsigned count = reinterpret_cast<const unsigned*>(scratch)[kLaunchCountOffset / 4];
  const uint64_t n16 = scratch_wipe_due(count, kScratchWipeAt) ? total16 : control16;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
    scratch[i] = i == 0 ? make_uint4(0u, count, 0u, 0u) : make_uint4(0u, 0u, 0u, 0u);
}

static int scratch_for_current_device(unsigned char** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) return fail(QSSM_EINVAL, "device index %d beyond the %d this entry point keeps", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_scratch));
    if (e != hipSuccess) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    if (p == nullptr || ((uintptr_t)p) % 256 != 0) return fail(QSSM_EINVAL, "scratch array has no usable device address");
    g_scratch_ptr[dev] = static_cast<unsigned char*>(p);
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

extern "C" int qssm_scan_forward_static(const qssm_plan* plan, const void* x, qssm_strides sx, const void* a,
                                        qssm_strides sa, const void* b, qssm_strides sb, const void* c,
                                        qssm_strides sc, void* y, qssm_strides sy, float* h_out, qssm_strides sh,
                                        float* ckpt, void* stream) {
  int rc = check_plan(plan, QSSM_FORWARD);
  if (rc != 0) return rc;
  if (plan->B == 0 || plan->L == 0 || plan->D == 0) return 0;
  if (plan->control_bytes > kScratchControlBytes || plan->workspace_bytes > kScratchBytes - kScratchControlBytes)
    return fail(QSSM_EWORKSPACE,
                "shape needs %llu bytes of control block and %llu of workspace; the built-in scratch array holds %llu "
                "and %llu: use qssm_scan_forward with buffers of the caller",
                (unsigned long long)plan->control_bytes, (unsigned long long)plan->workspace_bytes,
                (unsigned long long)kScratchControlBytes, (unsigned long long)(kScratchBytes - kScratchControlBytes));
  unsigned char* scratch = nullptr;
  rc = scratch_for_current_device(&scratch);
  if (rc != 0) return rc;
  if (plan->n_seg > 1) {
    hipLaunchKernelGGL(scratch_prologue_kernel, dim3(64), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<uint4*>(scratch), (uint64_t)(plan->control_bytes + 15) / 16, kScratchBytes / 16);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, "scratch_prologue_kernel launch");
  }
  return forward_launch(plan, x, sx, a, sa, b, sb, c, sc, y, sy, h_out, sh, ckpt, nullptr, nullptr, scratch,
                        kScratchControlBytes, scratch + kScratchControlBytes, kScratchBytes - kScratchControlBytes,
                        /*epoch=*/0, kScratchWipeAt, stream);
}

extern "C" {

int qssm_colsum(const void* x, int64_t ld, int64_t rows, int32_t S, int32_t dtype, float* partial, int32_t partial_rows,
                void* out, void* stream) {
  const int es = dtype_size(dtype);
  if (es == 0) return fail(QSSM_EINVAL, "unknown dtype code");
  if (rows < 0 || S < 0) return fail(QSSM_EINVAL, "negative dimension");
  if (S == 0) return 0;
  if (!out || !partial || (rows > 0 && !x)) return fail(QSSM_EINVAL, "NULL tensor");
  if (ld < S) return fail(QSSM_EINVAL, "row stride below S");
  if (partial_rows < 1) return fail(QSSM_EINVAL, "partial needs at least one row of S floats");
  // about 64 rows per chunk, as many chunks as `partial` has rows for
  int64_t chunks = (rows + 63) / 64;
  if (chunks > partial_rows) chunks = partial_rows;
  if (chunks < 1) chunks = 1;
  const int vec = rows == 0 ? 1 : gate_vec(S, {{x, ld}}, es, {}, es);
  if (!launch_colsum_any(dtype, x, ld, rows, S, vec, partial, (int)chunks, out, (hipStream_t)stream))
    return fail(QSSM_EINVAL, "column sum for storage type %d is not built", dtype);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e, "colsum kernel launch");
}

int qssm_launch_count_step(uint32_t count, int32_t static_scratch, uint32_t* flag, uint32_t* next, int32_t* wipes) {
  if (flag == nullptr || next == nullptr || wipes == nullptr) return fail(QSSM_EINVAL, "NULL argument");
  const unsigned reset_at = static_scratch ? kScratchWipeAt : kCountWrapAt;
  *flag = count + 1u;
  *next = launch_count_next(count, reset_at);
  *wipes = static_scratch && scratch_wipe_due(count, kScratchWipeAt) ? 1 : 0;
  return 0;
}

int qssm_copy_bytes(void* dst, const void* src, uint64_t bytes, void* stream) {
  if (bytes == 0) return 0;
  if (dst == nullptr || src == nullptr) return fail(QSSM_EINVAL, "NULL argument");
  if (((uintptr_t)dst) % 16 != 0 || ((uintptr_t)src) % 16 != 0 || bytes % 16 != 0)
    return fail(QSSM_EALIGN, "copy needs 16-byte alignment and a multiple of 16 bytes");
  const uint64_t n16 = bytes / 16;
  uint64_t blocks = (n16 + 1023) / 1024;
  if (blocks > (1u << 30)) blocks = 1u << 30;
  if (blocks == 0) blocks = 1;
  hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (uint4*)dst,
                     (const uint4*)src, n16);
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : hip_fail(e, "copy_kernel launch");
}

}  // extern "C"
