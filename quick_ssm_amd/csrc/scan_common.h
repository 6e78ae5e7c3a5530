// Shared device-side pieces of the gfx950 gated linear scan kernels.
//
// Tile model (both directions).  A workgroup of NTH lanes owns one tile: a strip of `G * VEC`
// adjacent columns of one batch row, times `seg_len = NG * T` consecutive time steps, where
// G = lanes per row (a power of two, runtime), NG = NTH / G lane groups, and each lane keeps
// T steps x VEC columns of every operand in registers.  Lanes of one group read one contiguous
// row piece (G * VEC * sizeof(elem) bytes; 512 B at the default geometry, which is what HBM
// needs to stream at full rate), so all global traffic is coalesced along D while the
// recurrence runs along L inside a lane.  A tile that waits for its neighbours holds its operands
// in registers, so the number of tiles a compute unit can hold bounds the bytes in flight; for
// 16-bit storage the operands the first sweep's recurrence does not need are therefore loaded
// straight into LDS instead (the CLDS variants of the kernels).
//
//   sweep 1   every lane folds its T steps into one affine map (A, X) starting from identity
//   LDS       the NG maps of each column are exchanged; lane group j composes the maps of the
//             groups before it (forward) / after it (reverse) into its carry-in
//   chain     tiles of one (batch row, strip) chain are grouped in clusters of R consecutive
//             tiles.  A tile publishes its own affine map as soon as it has it (it depends on
//             nothing), reads the maps of the tiles before it in its cluster, and takes the
//             state at the cluster's edge from the previous cluster.  Only that last hand-over
//             is a serial dependency: one hop per cluster, not per tile.
//   sweep 2   every lane re-runs its T steps from the true carry-in and stores the results
//
// Words exchanged between workgroups are {epoch:32 | fp32 bits:32}: flag and payload travel
// in one 64-bit access, so no fence is needed between them, and a word left over from an
// earlier launch (older epoch) reads as "not there yet".  Agent scope makes the accesses
// coherent across the XCDs' separate L2 caches.  A tile asks for its neighbours' words before
// it issues its own operand loads and looks at the answers when they are back; in steady
// state (tiles are claimed in time order, so neighbours ran a generation earlier) the words
// are there and the hand-over costs no extra round trip.  Every exchanged word is HBM traffic
// (agent-scope accesses do not stay in an XCD's L2), and the work around the words lengthens the
// tile's stay on its compute unit: both, not the waiting, are what the hand-over costs.
//
// Tiles of a chain are claimed in time order through a per-chain ticket counter in a small
// control block, so every tile a workgroup waits for was claimed by a workgroup that is already
// running.  The control block holds the status word, a count of launches and the counters; the
// holder of a chain's last ticket puts its counter back to zero.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/quick_ssm_hip.h"

namespace qssm {

// Polls before a tile gives up on a neighbour's word.  Each poll is a round trip to the
// coherent level of the memory system plus a sleep of up to half a microsecond: about a second
// in total.
constexpr int kSpinLimit = 1 << 20;

// Control block layout (bytes): [0,4) status word, [4,8) launches counted on the device (the epoch
// of a launch whose host passes epoch 0 is this count + 1; a one-lane kernel behind the launch
// adds one), rest of the first 64 bytes unused; then one 64-byte slot per chain holding its
// ticket counter.  Workspace layout: the tile maps (2 words per column per tile), then,
// 256-byte aligned, the cluster states (1 word per column per cluster).
constexpr uint64_t kStatusBytes = 64;
constexpr uint64_t kLaunchCountOffset = 4;
constexpr uint64_t kTicketStride = 64;

__host__ __device__ inline uint64_t ws_align(uint64_t off) { return (off + 255u) & ~uint64_t(255); }
__host__ __device__ inline uint64_t control_bytes(uint64_t n_chains) {
  return ws_align(kStatusBytes + n_chains * kTicketStride);
}
__host__ __device__ inline uint64_t ws_states_offset(uint64_t n_chains, uint64_t n_seg, uint64_t cols) {
  return ws_align(n_chains * n_seg * cols * 16u);
}
__host__ __device__ inline uint64_t ws_total_bytes(uint64_t n_chains, uint64_t n_seg, uint64_t n_super,
                                                   uint64_t cols) {
  return ws_align(ws_states_offset(n_chains, n_seg, cols) + n_chains * n_super * cols * 8u);
}

typedef _Float16 f16_t;
typedef __bf16 bf16_t;

template <typename T, int V>
struct alignas(sizeof(T) * V > 16 ? 16 : sizeof(T) * V) Pack {
  T v[V];
};

template <int BYTES> struct RawOf;
template <> struct RawOf<2> { typedef unsigned short type; };
template <> struct RawOf<4> { typedef unsigned int type; };
template <> struct RawOf<8> { typedef unsigned int type __attribute__((ext_vector_type(2))); };
template <> struct RawOf<16> { typedef unsigned int type __attribute__((ext_vector_type(4))); };

// VEC stored elements of one operand at one time step, kept as the 32-bit words they were
// loaded as.  16-bit elements stay packed two to a register until the instruction that uses
// them (a struct of halves would be split into one register per element).
template <typename T, int V>
struct Words {
  static constexpr int N = (int)((sizeof(T) * V + 3) / 4);
  uint32_t w[N];
};

template <typename T> struct ElemBits;
template <> struct ElemBits<float> {
  static __device__ __forceinline__ uint32_t one() { return 0x3f800000u; }
  template <int V> static __device__ __forceinline__ float get(const Words<float, V>& p, int v) {
    return __uint_as_float(p.w[v]);
  }
  template <int V> static __device__ __forceinline__ void set(Words<float, V>& p, const float* f) {
#pragma unroll
    for (int v = 0; v < V; ++v) p.w[v] = __float_as_uint(f[v]);
  }
};
template <> struct ElemBits<bf16_t> {
  static __device__ __forceinline__ uint32_t one() { return 0x3f803f80u; }
  template <int V> static __device__ __forceinline__ float get(const Words<bf16_t, V>& p, int v) {
    const uint32_t w = p.w[v >> 1];
    return __uint_as_float((v & 1) ? (w & 0xffff0000u) : (w << 16));
  }
  template <int V> static __device__ __forceinline__ void set(Words<bf16_t, V>& p, const float* f) {
    if (V == 1) {
      p.w[0] = (uint32_t)__builtin_bit_cast(unsigned short, (bf16_t)f[0]);
    } else {
      // two values per conversion instruction, already packed
      typedef float f32x2 __attribute__((ext_vector_type(2)));
      typedef bf16_t bf16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
      for (int k = 0; k < V / 2; ++k) {
        const f32x2 pair = {f[2 * k], f[2 * k + 1]};
        p.w[k] = __builtin_bit_cast(uint32_t, __builtin_convertvector(pair, bf16x2));
      }
    }
  }
};
template <> struct ElemBits<f16_t> {
  static __device__ __forceinline__ uint32_t one() { return 0x3c003c00u; }
  template <int V> static __device__ __forceinline__ float get(const Words<f16_t, V>& p, int v) {
    const uint32_t w = p.w[v >> 1];
    const unsigned short h = (unsigned short)((v & 1) ? (w >> 16) : (w & 0xffffu));
    return (float)__builtin_bit_cast(f16_t, h);
  }
  template <int V> static __device__ __forceinline__ void set(Words<f16_t, V>& p, const float* f) {
    if (V == 1) {
      p.w[0] = (uint32_t)__builtin_bit_cast(unsigned short, (f16_t)f[0]);
    } else {
#pragma unroll
      for (int k = 0; k < V / 2; ++k) {
        const uint32_t lo = __builtin_bit_cast(unsigned short, (f16_t)f[2 * k]);
        const uint32_t hi = __builtin_bit_cast(unsigned short, (f16_t)f[2 * k + 1]);
        p.w[k] = lo | (hi << 16);
      }
    }
  }
};

template <typename T, int V>
__device__ __forceinline__ float elem(const Words<T, V>& p, int v) {
  return ElemBits<T>::template get<V>(p, v);
}

// One vector load / store of VEC elements at a byte offset from a workgroup-uniform base.
// Operands and results are touched exactly once by a launch, so they are marked non-temporal (streaming); KEEP
// asks for an ordinary load instead, whose lines stay in the caches for a launch that follows.
template <typename T, int V, bool KEEP = false>
__device__ __forceinline__ Words<T, V> load_stream(const char* base, uint32_t byte_off) {
  if constexpr (sizeof(T) * V == 32) {   // two 16-byte halves
    const Words<T, V / 2> lo = load_stream<T, V / 2, KEEP>(base, byte_off), hi = load_stream<T, V / 2, KEEP>(base, byte_off + 16u);
    Words<T, V> out;
#pragma unroll
    for (int k = 0; k < 4; ++k) { out.w[k] = lo.w[k]; out.w[4 + k] = hi.w[k]; }
    return out;
  } else {
  typedef typename RawOf<sizeof(T) * V>::type raw_t;
  raw_t r;
  if constexpr (KEEP) r = *reinterpret_cast<const raw_t*>(base + byte_off);
  else r = __builtin_nontemporal_load(reinterpret_cast<const raw_t*>(base + byte_off));
  Words<T, V> out;
  if constexpr (sizeof(T) * V <= 4) {
    out.w[0] = (uint32_t)r;
  } else {
#pragma unroll
    for (int k = 0; k < Words<T, V>::N; ++k) out.w[k] = r[k];
  }
  return out;
  }
}

template <typename T, int V>
__device__ __forceinline__ void store_stream(char* base, uint32_t byte_off, const float* f) {
  if constexpr (sizeof(T) * V == 32) {   // two 16-byte halves
    store_stream<T, V / 2>(base, byte_off, f);
    store_stream<T, V / 2>(base, byte_off + 16u, f + V / 2);
  } else {
  typedef typename RawOf<sizeof(T) * V>::type raw_t;
  Words<T, V> p;
  ElemBits<T>::template set<V>(p, f);
  raw_t r;
  if constexpr (sizeof(T) * V <= 4) {
    r = (raw_t)p.w[0];
  } else {
#pragma unroll
    for (int k = 0; k < Words<T, V>::N; ++k) r[k] = p.w[k];
  }
  __builtin_nontemporal_store(r, reinterpret_cast<raw_t*>(base + byte_off));
  }
}

// All VEC elements equal to 1 (`one`) or 0.
template <typename T, int V>
__device__ __forceinline__ Words<T, V> fill_words(bool one) {
  Words<T, V> p;
  uint32_t w = one ? ElemBits<T>::one() : 0u;
  if (sizeof(T) * V < 4) w &= 0xffffu;
#pragma unroll
  for (int k = 0; k < Words<T, V>::N; ++k) p.w[k] = w;
  return p;
}

template <typename T, int V>
__device__ __forceinline__ Pack<T, V> load_pack(const T* p) {
  if constexpr (sizeof(T) * V == 32) {   // two 16-byte halves
    const Pack<T, V / 2> lo = load_pack<T, V / 2>(p), hi = load_pack<T, V / 2>(p + V / 2);
    Pack<T, V> out;
#pragma unroll
    for (int k = 0; k < V / 2; ++k) { out.v[k] = lo.v[k]; out.v[V / 2 + k] = hi.v[k]; }
    return out;
  } else {
    typedef typename RawOf<sizeof(T) * V>::type raw_t;
    raw_t r = *reinterpret_cast<const raw_t*>(p);
    return __builtin_bit_cast(Pack<T, V>, r);
  }
}

template <typename T, int V>
__device__ __forceinline__ void store_pack(T* p, const Pack<T, V>& v) {
  if constexpr (sizeof(T) * V == 32) {   // two 16-byte halves
    Pack<T, V / 2> lo, hi;
#pragma unroll
    for (int k = 0; k < V / 2; ++k) { lo.v[k] = v.v[k]; hi.v[k] = v.v[V / 2 + k]; }
    store_pack<T, V / 2>(p, lo);
    store_pack<T, V / 2>(p + V / 2, hi);
  } else {
    typedef typename RawOf<sizeof(T) * V>::type raw_t;
    *reinterpret_cast<raw_t*>(p) = __builtin_bit_cast(raw_t, v);
  }
}

// VEC adjacent floats in LDS as one access (a lane's VEC columns sit next to each other, so a
// wavefront's access is dense and free of bank conflicts, which VEC separate 4-byte accesses at a
// stride of VEC words are not).
template <int V>
__device__ __forceinline__ void lds_get(const float* p, float* out) {
  const Pack<float, V> v = *reinterpret_cast<const Pack<float, V>*>(p);
#pragma unroll
  for (int k = 0; k < V; ++k) out[k] = v.v[k];
}
template <int V>
__device__ __forceinline__ void lds_put(float* p, const float* in) {
  Pack<float, V> v;
#pragma unroll
  for (int k = 0; k < V; ++k) v.v[k] = in[k];
  *reinterpret_cast<Pack<float, V>*>(p) = v;
}

// Gate activations of the SSM layer (quick_ssm/layers.py:76-82), shared by the gate prologue and the gated scans
// so that both routes round the same values: the hardware's exp2 and reciprocal (1 ulp each), fp32 throughout.
__device__ __forceinline__ float sigmoid_f(float z) { return __builtin_amdgcn_rcpf(1.0f + __expf(-z)); }

// The value `f` has after being stored as T and read back (the rounding the layer applies when it casts the
// scan's operands to its compute dtype, and the scan when it stores a gradient).
template <typename T, int V>
__device__ __forceinline__ void round_through(float* f) {
  Words<T, V> w;
  ElemBits<T>::template set<V>(w, f);
#pragma unroll
  for (int v = 0; v < V; ++v) f[v] = elem(w, v);
}

// Makes the compiler forget what it knows about a loaded operand, so that the later sweeps
// convert it to fp32 again instead of keeping an fp32 copy of every operand alive across the
// barriers (which would double the register footprint of a tile).
template <typename T, int V>
__device__ __forceinline__ void forget(Words<T, V>& p) {
#pragma unroll
  for (int k = 0; k < Words<T, V>::N; ++k) asm volatile("" : "+v"(p.w[k]));
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// outstanding global load and store of the wave (operands still in flight, words just published
// to other workgroups), which would put a memory round trip into each of the tile's barriers.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// ---- words exchanged between workgroups ------------------------------------------------------

__device__ __forceinline__ void word_publish(unsigned long long* w, unsigned epoch, float v) {
  const unsigned long long word = ((unsigned long long)epoch << 32) | (unsigned long long)__float_as_uint(v);
  __hip_atomic_store(w, word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// One look at N consecutive words (all N loads in flight together).
template <int N>
struct Peek {
  unsigned long long r[N];
  // Start from "nothing there" (epoch 0 is never used), so that lanes which do not ask keep
  // defined values and no branch has to be joined, and waited for, before later loads go out.
  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int n = 0; n < N; ++n) r[n] = 0ull;
  }
  // Word n of this lane sits at w + n * plane: the lanes of a group are adjacent within a plane,
  // so that one load (or store) instruction of a wavefront covers whole cache lines.  Publishing
  // 8-byte words scattered one per 32 or 64 bytes would reach memory as partial-line writes.
  __device__ __forceinline__ void issue(const unsigned long long* w, int plane) {
#pragma unroll
    for (int n = 0; n < N; ++n)
      r[n] = __hip_atomic_load(const_cast<unsigned long long*>(w) + (size_t)n * plane, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
  }
  // Compiler fence: whatever looks at the answers stays behind the memory operations issued
  // before this point (the operand loads), instead of being hoisted in front of them.
  __device__ __forceinline__ void pin() {
#pragma unroll
    for (int n = 0; n < N; ++n) asm volatile("" : "+v"(r[n]) : : "memory");
  }
  __device__ __forceinline__ bool ready(unsigned epoch) const {
    bool ok = true;
#pragma unroll
    for (int n = 0; n < N; ++n) ok = ok && ((unsigned)(r[n] >> 32) == epoch);
    return ok;
  }
  __device__ __forceinline__ float value(int n) const { return __uint_as_float((unsigned)r[n]); }
};

// Wait until this lane's N words (at w + n * plane) carry this launch's epoch.  Returns false (and
// NaN payloads) if the words never arrive.  Three ways of polling:
//   kPollSlow    one word per wavefront (its first active lane's first word, read by every lane at
//                the same address, i.e. one 8-byte request), about half a microsecond apart; only
//                when that one has arrived do the lanes read their own words, which the producer
//                stored with the same instructions and which are then there as a rule.  For words
//                that are needed later than they are published as a rule: a waiting tile must not
//                load the memory system.
//   kPollUrgent  the same, almost back to back at first, backing off when the wait drags on.  For
//                the state a tile needs but does not hand on.
//   kPollChain   every lane polls its own words, back to back: the answer that shows the words is
//                the answer that carries them, which saves a round trip per hand-over.  Only for the
//                one tile per cluster that hands the state on, i.e. one waiting tile per chain: the
//                hand-overs from cluster to cluster are the serial path of the whole launch.
enum PollMode { kPollSlow = 0, kPollUrgent = 1, kPollChain = 2 };

template <int N>
__device__ __forceinline__ bool words_wait(const unsigned long long* w, int plane, unsigned epoch, float* out,
                                           const PollMode mode) {
  if (mode == kPollChain) {
    for (int spins = 0; spins < kSpinLimit; ++spins) {
      Peek<N> pk;
      pk.issue(w, plane);
      if (pk.ready(epoch)) {
#pragma unroll
        for (int n = 0; n < N; ++n) out[n] = pk.value(n);
        return true;
      }
      if (spins >= 64) {
        for (int k = 0; k < 8; ++k) __builtin_amdgcn_s_sleep(2);
      }
    }
  } else {
    const uint64_t mine = reinterpret_cast<uint64_t>(w);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)mine);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(mine >> 32));
    unsigned long long* lead = reinterpret_cast<unsigned long long*>(((uint64_t)hi << 32) | lo);
    const bool urgent = mode == kPollUrgent;
    for (int spins = 0; spins < kSpinLimit; ++spins) {
      const unsigned long long first = __hip_atomic_load(lead, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((unsigned)(first >> 32) == epoch) {
        Peek<N> pk;
        pk.issue(w, plane);
        if (pk.ready(epoch)) {
#pragma unroll
          for (int n = 0; n < N; ++n) out[n] = pk.value(n);
          return true;
        }
      }
      if (urgent && spins < 32) {
        __builtin_amdgcn_s_sleep(1);
      } else {
        const int nap = (urgent && spins < 256) ? 2 : 8;
        for (int k = 0; k < nap; ++k) __builtin_amdgcn_s_sleep(2);
      }
    }
  }
#pragma unroll
  for (int n = 0; n < N; ++n) out[n] = __uint_as_float(0x7fc00000u);
  return false;
}

// Claim the next tile of `chain` in time order: one atomic add.  The holder of the last ticket
// puts the counter back to zero; by then every other tile of the chain has taken its ticket.
__device__ __forceinline__ unsigned claim_ticket(unsigned* tickets, int chain, int n_seg) {
  unsigned* slot = tickets + (size_t)chain * (kTicketStride / sizeof(unsigned));
  const unsigned tk = __hip_atomic_fetch_add(slot, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (tk == (unsigned)(n_seg - 1)) __hip_atomic_store(slot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return tk;
}

// Status codes are bits (1: a tile gave up waiting, 2: the control block was dirty on entry) and accumulate.
__device__ __forceinline__ void raise_status(int* status, int code) {
  __hip_atomic_fetch_or(status, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The launch count kept in the control block (device-counted epochs).  A launch uses flag value count + 1; the
// counting kernel behind it stores launch_count_next(count, reset_at).  The count never takes the value whose
// successor is zero: from `reset_at` on it starts again at zero, and a caller that lets it do so must have
// cleared every word of the old numbering first (scratch_wipe_due: the library's own scratch array does that in
// the prologue of the launch that finds the count at or beyond its wipe mark).
__host__ __device__ inline unsigned launch_count_next(unsigned count, unsigned reset_at) {
  return count >= reset_at ? 0u : count + 1u;
}
__host__ __device__ inline bool scratch_wipe_due(unsigned count, unsigned wipe_at) { return count >= wipe_at; }

// ---- kernel arguments -----------------------------------------------------------------------

struct Geometry {
  int B, L, D;
  int g_log2;       // log2 lanes per row
  int n_strips;     // strips per batch row
  int n_chains;     // B * n_strips
  int n_seg;        // tiles per chain
  int seg_len;      // time steps per tile
  int cluster;      // tiles per cluster (R, power of two)
  int n_super;      // clusters per chain
  int ckpt_stride;  // spacing of saved states
  int n_ckpt;       // saved states per (batch, column)
  int keep_from;    // forward: tiles from this index on load their operands with ordinary (cached) loads
  unsigned epoch;   // this launch's flag value (nonzero), when the host counts launches
  const unsigned* launch_count;  // else: launches counted on the device; the flag value is *launch_count + 1
  int* status;
  unsigned* tickets;
  unsigned long long* maps;    // [chain][tile][2 * VEC planes][G lanes]: the tile's affine map (A, X)
  unsigned long long* states;  // [chain][cluster][VEC planes][G lanes]: state handed to the next cluster
};

struct FwdArgs {
  Geometry g;
  const void *x, *a, *b, *c;
  void* y;
  float* h_out;
  float* ckpt;
  const float* h_init;  // [B, D] state before the first step (null: zero)
  float* h_final;       // [B, D] state after the last step (null: not wanted)
  int64_t x_sb, x_sl, a_sb, a_sl, b_sb, b_sl, c_sb, c_sl, y_sb, y_sl, h_sb, h_sl;
  // Gated launches: a, b, x, c point at the projection outputs A_pre, D_pre, B_in, Ca and c2 at Cb; the kernel
  // forms a = sigmoid(A_pre), b = sigmoid(D_pre), c = silu(Ca) * Cb itself.
  const void* c2;
  int64_t c2_sb, c2_sl;
};

struct BwdArgs {
  Geometry g;
  const void *x, *a, *b, *c, *dy;
  const float* h;
  const float* ckpt;
  const float* h_init;    // [B, D] state before the first step (null: zero)
  const float* dh_final;  // [B, D] gradient arriving at the state after the last step (null: zero)
  float* dh_init;         // [B, D] gradient of the state before the first step (null: not wanted)
  void *dx, *da, *db, *dc;
  int64_t x_sb, x_sl, a_sb, a_sl, b_sb, b_sl, c_sb, c_sl, dy_sb, dy_sl, h_sb, h_sl;
  int64_t dx_sb, dx_sl, da_sb, da_sl, db_sb, db_sl, dc_sb, dc_sl;
  // Gated launches: operands as in FwdArgs; dx, da, db, dc receive dB_in, dA_pre, dD_pre, dCa and dc2 dCb.
  const void* c2;
  int64_t c2_sb, c2_sl;
  void* dc2;
  int64_t dc2_sb, dc2_sl;
};

// Dynamic LDS a launch needs: per-lane maps plus the cluster's neighbour maps and one row of state.
inline size_t fwd_lds_bytes(int nth, int vec, int cols, int cluster) {
  return sizeof(float) * ((size_t)2 * nth * vec + (size_t)2 * (cluster - 1) * cols + cols) + 16;
}
inline size_t bwd_lds_bytes(int nth, int vec, int cols, int cluster) {
  return sizeof(float) * ((size_t)3 * nth * vec + (size_t)2 * (cluster - 1) * cols + cols) + 16;
}

// Host-side launch tables, one entry per (in dtype, out dtype) pair the library instantiates.
// Return false if (vec, steps, threads) is not an instantiated combination.
// `gated`: kNotGated for the plain scan, else the storage code of the layer's compute dtype (gated scan).
constexpr int kNotGated = -1;
template <typename T> constexpr int dtype_code();
template <> constexpr int dtype_code<float>() { return QSSM_F32; }
template <> constexpr int dtype_code<f16_t>() { return QSSM_F16; }
template <> constexpr int dtype_code<bf16_t>() { return QSSM_BF16; }
typedef bool (*fwd_launch_fn)(const FwdArgs&, int vec, int steps, int threads, bool c_in_lds, int gated, dim3 grid,
                              size_t lds, hipStream_t stream);
// Extra dynamic LDS of the forward kernel that keeps c in LDS: 8 or 16 bytes per lane and step.
inline size_t fwd_c_lds_bytes(int nth, int steps, int lane_bytes) { return (size_t)nth * steps * lane_bytes; }
typedef bool (*bwd_launch_fn)(const BwdArgs&, int vec, int steps, int threads, bool cg_in_lds, int gated, dim3 grid,
                              size_t lds, hipStream_t stream);
// Extra dynamic LDS of the backward kernel that keeps c and dy in LDS.
inline size_t bwd_cg_lds_bytes(int nth, int steps) { return (size_t)2 * nth * steps * 8; }

fwd_launch_fn find_fwd_launcher(int in_dtype, int out_dtype);
bwd_launch_fn find_bwd_launcher(int in_dtype, int out_dtype);

// ---- gate prologue of the SSM layer (gates.hip) --------------------------------------------------

struct GateFwdArgs {
  const void *A_pre, *B_in, *Ca, *Cb, *D_pre;  // [rows, S], row strides in elements
  int64_t ld_a, ld_b, ld_ca, ld_cb, ld_d;
  void *a, *x, *c, *b;                          // [rows, S] contiguous
  int64_t rows;
  int S;
};

struct GateBwdArgs {
  const void *g_a, *g_x, *g_c, *g_b;            // [rows, S] contiguous, storage of the scan's operands
  const void *A_pre, *Ca, *Cb, *D_pre;          // [rows, S], row strides in elements
  int64_t ld_a, ld_ca, ld_cb, ld_d;
  void *dA_pre, *dB_in, *dCa, *dCb, *dD_pre;    // [rows, S], storage of the projections, one row stride for all five
  int64_t rows;
  int S;
  int64_t ld_grad;                               // row stride (elements) of the five gradients: S when contiguous
};

// One entry per (projection storage, operand storage) pair; exactly one of f, b is non-null.
// Returns false if the pair or vec is not built.
bool launch_gates_any(int in_dtype, int out_dtype, const GateFwdArgs* f, const GateBwdArgs* b, int vec,
                      hipStream_t stream);

// ---- RMSNorm of the SSM layer (rmsnorm.hip) ----------------------------------------------------------

struct NormFwdArgs {
  const void* x;      // [rows, H], row stride ld_x elements
  int64_t ld_x;
  const void* w;      // [H]
  void* y;            // [rows, H] contiguous
  float* rstd;        // [rows] 1 / sqrt(mean(x^2) + eps), or null
  int64_t rows;
  int H;
  float eps;
};

struct NormBwdArgs {
  const void* dy;     // [rows, H], row stride ld_dy elements
  int64_t ld_dy;
  const void* x;      // [rows, H], row stride ld_x elements
  int64_t ld_x;
  const void* w;      // [H]
  const float* rstd;  // [rows] as the forward stored it, or null (recomputed from x and eps)
  void* dx;           // [rows, H] contiguous
  float* partial;     // [partial rows, H] fp32 scratch for dw
  int64_t rows;
  int H;
  float eps;
};

// Exactly one of f, b is non-null; dw and max_partial_rows belong to the backward.  False if the
// storage type or vec is not built, or `partial` is too small for one launch.
bool launch_norm_any(int dtype, const NormFwdArgs* f, const NormBwdArgs* b, int vec, int max_partial_rows, void* dw,
                     hipStream_t stream);

// ---- column sums (colsum.hip): bias gradients of the layer's linear maps ---------------------------------------
// `partial` holds `chunks` rows of S floats.  False if the storage type is not built.
bool launch_colsum_any(int dtype, const void* x, int64_t ld, int64_t rows, int S, int vec, float* partial, int chunks,
                       void* out, hipStream_t stream);

}  // namespace qssm
