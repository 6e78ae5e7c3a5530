// Shared device-side pieces of the gfx950 gated linear scan kernels.
//
// Tile model (both directions).  A workgroup of 256 lanes owns one tile: a strip of
// `G * VEC` adjacent columns of one batch row, times `seg_len = NG * T` consecutive time
// steps, where G = lanes per row (a power of two, runtime), NG = 256 / G lane groups, and each
// lane keeps T steps x VEC columns of every operand in registers.  Lanes of one group read one
// contiguous row piece (G * VEC * sizeof(elem) bytes, 128 B at the default geometry), so all
// global traffic is coalesced along D while the recurrence runs along L inside a lane.
//
//   sweep 1   every lane folds its T steps into one affine map (A, X) starting from identity
//   LDS       the NG maps of each column are exchanged; lane group j composes the maps of the
//             groups before it (forward) / after it (reverse) into its carry-in
//   chain     the tile-level carry comes from the neighbouring tile of the same chain through
//             a 64-bit {flag, fp32} word in the workspace (one word per column)
//   sweep 2   every lane re-runs its T steps from the true carry-in and stores the results
//
// Tiles of a chain are claimed in time order through a per-chain ticket counter, so the tile a
// workgroup waits for was always claimed by a workgroup that is already running.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/quick_ssm_hip.h"

namespace qssm {

constexpr int kThreads = 256;
// Polls before a tile gives up on its neighbour's carry (each poll sleeps ~64 clocks and costs
// a round trip to the coherent level of the memory system: about a second in total).
constexpr int kSpinLimit = 1 << 20;

// Workspace layout (bytes): [0,64) status word; then one 64-byte slot per chain holding its
// ticket counter; then, 256-byte aligned, n_chains * n_seg * strip_cols carry words of 8 bytes.
constexpr uint64_t kStatusBytes = 64;
constexpr uint64_t kTicketStride = 64;

__host__ __device__ inline uint64_t ws_carry_offset(uint64_t n_chains) {
  uint64_t off = kStatusBytes + n_chains * kTicketStride;
  return (off + 255u) & ~uint64_t(255);
}

typedef _Float16 f16_t;
typedef __bf16 bf16_t;

template <typename T, int V>
struct alignas(sizeof(T) * V) Pack {
  T v[V];
};

template <int BYTES> struct RawOf;
template <> struct RawOf<2> { typedef unsigned short type; };
template <> struct RawOf<4> { typedef unsigned int type; };
template <> struct RawOf<8> { typedef unsigned int type __attribute__((ext_vector_type(2))); };
template <> struct RawOf<16> { typedef unsigned int type __attribute__((ext_vector_type(4))); };

// One vector load / store of VEC elements (the pointer is VEC-element aligned by contract).
template <typename T, int V>
__device__ __forceinline__ Pack<T, V> load_pack(const T* p) {
  typedef typename RawOf<sizeof(T) * V>::type raw_t;
  raw_t r = *reinterpret_cast<const raw_t*>(p);
  return __builtin_bit_cast(Pack<T, V>, r);
}

template <typename T, int V>
__device__ __forceinline__ void store_pack(T* p, const Pack<T, V>& v) {
  typedef typename RawOf<sizeof(T) * V>::type raw_t;
  *reinterpret_cast<raw_t*>(p) = __builtin_bit_cast(raw_t, v);
}

template <typename T, int V>
__device__ __forceinline__ Pack<T, V> fill_pack(float f) {
  Pack<T, V> r;
#pragma unroll
  for (int v = 0; v < V; ++v) r.v[v] = (T)f;
  return r;
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(f16_t v) { return (float)v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

// ---- cross-workgroup carry words ------------------------------------------------------------
// A carry word is {flag:32 | fp32 bits:32}.  Flag and payload travel in one 64-bit access, so
// no fence is needed between them; agent scope makes the access coherent across the XCDs'
// separate L2 caches.

constexpr unsigned kFlagReady = 1u;

__device__ __forceinline__ void carry_publish(unsigned long long* w, float v) {
  unsigned long long word = ((unsigned long long)kFlagReady << 32) | (unsigned long long)__float_as_uint(v);
  __hip_atomic_store(w, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Wait for a published word, take its payload and leave the word zero for the next launch.
// Returns false (and a NaN payload) if the neighbour never published within kSpinLimit polls.
__device__ __forceinline__ bool carry_consume(unsigned long long* w, float* out) {
  int spins = 0;
  for (;;) {
    unsigned long long word = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if ((unsigned)(word >> 32) == kFlagReady) {
      *out = __uint_as_float((unsigned)word);
      __hip_atomic_store(w, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      return true;
    }
    if (++spins >= kSpinLimit) {
      *out = __uint_as_float(0x7fc00000u);
      return false;
    }
    __builtin_amdgcn_s_sleep(1);
  }
}

// Claim the next tile of `chain` in time order.  The holder of the last ticket puts the
// counter back to zero: by then every other tile of the chain has taken its ticket.
__device__ __forceinline__ unsigned claim_ticket(unsigned* tickets, int chain, int n_seg) {
  unsigned* slot = tickets + (size_t)chain * (kTicketStride / sizeof(unsigned));
  unsigned tk = __hip_atomic_fetch_add(slot, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (tk == (unsigned)(n_seg - 1)) __hip_atomic_store(slot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return tk;
}

__device__ __forceinline__ void raise_status(int* status, int code) {
  __hip_atomic_store(status, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- kernel arguments -----------------------------------------------------------------------

struct Geometry {
  int B, L, D;
  int g_log2;       // log2 lanes per row
  int n_strips;     // strips per batch row
  int n_chains;     // B * n_strips
  int n_seg;        // tiles per chain
  int seg_len;      // time steps per tile
  int ckpt_stride;  // spacing of saved states
  int n_ckpt;       // saved states per (batch, column)
  int* status;
  unsigned* tickets;
  unsigned long long* carry;
};

struct FwdArgs {
  Geometry g;
  const void *x, *a, *b, *c;
  void* y;
  float* h_out;
  float* ckpt;
  int64_t x_sb, x_sl, a_sb, a_sl, b_sb, b_sl, c_sb, c_sl, y_sb, y_sl, h_sb, h_sl;
};

struct BwdArgs {
  Geometry g;
  const void *x, *a, *b, *c, *dy;
  const float* h;
  const float* ckpt;
  void *dx, *da, *db, *dc;
  int64_t x_sb, x_sl, a_sb, a_sl, b_sb, b_sl, c_sb, c_sl, dy_sb, dy_sl, h_sb, h_sl;
  int64_t dx_sb, dx_sl, da_sb, da_sl, db_sb, db_sl, dc_sb, dc_sl;
};

// Host-side launch tables, one entry per (in dtype, out dtype) pair the library instantiates.
typedef void (*fwd_launch_fn)(const FwdArgs&, int vec, int steps, dim3 grid, hipStream_t stream);
typedef void (*bwd_launch_fn)(const BwdArgs&, int vec, int steps, dim3 grid, hipStream_t stream);

fwd_launch_fn find_fwd_launcher(int in_dtype, int out_dtype);
bwd_launch_fn find_bwd_launcher(int in_dtype, int out_dtype);

}  // namespace qssm
