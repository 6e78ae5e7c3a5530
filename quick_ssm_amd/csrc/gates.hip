// Gate prologue of the SSM layer for gfx950: the five projection outputs become the scan's four
// operands in one pass, and their gradients go back in one pass.
//
//   a = sigmoid(A_pre)   x = B_in   c = silu(Ca) * Cb   b = sigmoid(D_pre)       (forward)
//   dA_pre = da * a (1 - a)          dB_in = dx          dD_pre = db * b (1 - b)
//   dCa = dc * Cb * s (1 + Ca (1 - s)),  dCb = dc * Ca * s,  s = sigmoid(Ca)     (backward)
//
// It takes the place of the elementwise chain in the reference's SSM.forward
// (quick_ssm/layers.py:76-88: two sigmoids, silu, a product and four dtype casts, each its own
// pass over a [B, L, state] tensor, and as many again recorded for autograd).  Arithmetic is
// fp32 whatever the storage; each result is rounded once to its storage type.  Pure streaming:
// 16 or 8 bytes per lane and tensor, nothing is read twice.
#include "scan_common.h"

namespace qssm {

template <typename T, int V>
__device__ __forceinline__ void load_f32(const void* base, int64_t elem_off, float* out) {
  const Words<T, V> w = load_stream<T, V>(reinterpret_cast<const char*>(base) + elem_off * (int64_t)sizeof(T), 0u);
#pragma unroll
  for (int v = 0; v < V; ++v) out[v] = elem(w, v);
}

template <typename T, int V>
__device__ __forceinline__ void store_f32(void* base, int64_t elem_off, const float* in) {
  store_stream<T, V>(reinterpret_cast<char*>(base) + elem_off * (int64_t)sizeof(T), 0u, in);
}

template <typename Tin, typename Tout, int V>
__global__ void __launch_bounds__(256) gates_fwd_kernel(const GateFwdArgs p) {
  const int64_t per_row = p.S / V;
  const int64_t total = p.rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = i / per_row;
    const int64_t col = (i - row * per_row) * V;
    float za[V], zx[V], zca[V], zcb[V], zd[V];
    load_f32<Tin, V>(p.A_pre, row * p.ld_a + col, za);
    load_f32<Tin, V>(p.B_in, row * p.ld_b + col, zx);
    load_f32<Tin, V>(p.Ca, row * p.ld_ca + col, zca);
    load_f32<Tin, V>(p.Cb, row * p.ld_cb + col, zcb);
    load_f32<Tin, V>(p.D_pre, row * p.ld_d + col, zd);
    float a[V], c[V], b[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      a[v] = sigmoid_f(za[v]);
      c[v] = zca[v] * sigmoid_f(zca[v]) * zcb[v];
      b[v] = sigmoid_f(zd[v]);
    }
    const int64_t o = row * p.S + col;
    store_f32<Tout, V>(p.a, o, a);
    store_f32<Tout, V>(p.x, o, zx);
    store_f32<Tout, V>(p.c, o, c);
    store_f32<Tout, V>(p.b, o, b);
  }
}

template <typename Tin, typename Tout, int V>
__global__ void __launch_bounds__(256) gates_bwd_kernel(const GateBwdArgs p) {
  const int64_t per_row = p.S / V;
  const int64_t total = p.rows * per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = i / per_row;
    const int64_t col = (i - row * per_row) * V;
    const int64_t o = row * p.S + col;
    float ga[V], gx[V], gc[V], gb[V], za[V], zca[V], zcb[V], zd[V];
    load_f32<Tout, V>(p.g_a, o, ga);
    load_f32<Tout, V>(p.g_x, o, gx);
    load_f32<Tout, V>(p.g_c, o, gc);
    load_f32<Tout, V>(p.g_b, o, gb);
    load_f32<Tin, V>(p.A_pre, row * p.ld_a + col, za);
    load_f32<Tin, V>(p.Ca, row * p.ld_ca + col, zca);
    load_f32<Tin, V>(p.Cb, row * p.ld_cb + col, zcb);
    load_f32<Tin, V>(p.D_pre, row * p.ld_d + col, zd);
    float dA[V], dCa[V], dCb[V], dD[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      const float a = sigmoid_f(za[v]);
      const float b = sigmoid_f(zd[v]);
      const float s = sigmoid_f(zca[v]);
      dA[v] = ga[v] * a * (1.0f - a);
      dD[v] = gb[v] * b * (1.0f - b);
      dCa[v] = gc[v] * zcb[v] * s * (1.0f + zca[v] * (1.0f - s));
      dCb[v] = gc[v] * zca[v] * s;
    }
    const int64_t og = row * p.ld_grad + col;
    store_f32<Tin, V>(p.dA_pre, og, dA);
    store_f32<Tin, V>(p.dB_in, og, gx);
    store_f32<Tin, V>(p.dCa, og, dCa);
    store_f32<Tin, V>(p.dCb, og, dCb);
    store_f32<Tin, V>(p.dD_pre, og, dD);
  }
}

// One 256-lane workgroup per 256 vectors: workgroups start in index order and end after one step, so at
// any moment the resident ones cover one narrow window of every tensor, which is what DRAM pages and
// address translation like best (6.1 / 5.8 TB/s forward / backward on 32768 x 4096 fp32 -> fp16, against
// 4.4 / 4.3 TB/s for 4096 workgroups that stay and stride through the tensors).  The kernels keep their
// grid-stride loop for tensors with more than 2^30 x 256 vectors.
static unsigned gate_grid(int64_t vectors) {
  const int64_t blocks = (vectors + 255) / 256;
  const int64_t cap = (int64_t)1 << 30;
  return (unsigned)(blocks < cap ? (blocks > 0 ? blocks : 1) : cap);
}

template <typename Tin, typename Tout>
static bool launch_gates(const GateFwdArgs* f, const GateBwdArgs* b, int vec, hipStream_t stream) {
  const int64_t rows = f ? f->rows : b->rows;
  const int S = f ? f->S : b->S;
  const unsigned grid = gate_grid(rows * (S / vec));
#define QSSM_GATE_CASE(V)                                                                                 \
  if (vec == V) {                                                                                         \
    if (f) hipLaunchKernelGGL((gates_fwd_kernel<Tin, Tout, V>), dim3(grid), dim3(256), 0, stream, *f);     \
    else hipLaunchKernelGGL((gates_bwd_kernel<Tin, Tout, V>), dim3(grid), dim3(256), 0, stream, *b);       \
    return true;                                                                                          \
  }
  QSSM_GATE_CASE(4)
  QSSM_GATE_CASE(2)
  QSSM_GATE_CASE(1)
#undef QSSM_GATE_CASE
  return false;
}

// One entry per (projection storage, operand storage) pair; false if the pair or vec is unknown.
bool launch_gates_any(int in_dtype, int out_dtype, const GateFwdArgs* f, const GateBwdArgs* b, int vec,
                      hipStream_t stream) {
#define QSSM_GATE_PAIR(IN, TIN, OUT, TOUT) \
  if (in_dtype == IN && out_dtype == OUT) return launch_gates<TIN, TOUT>(f, b, vec, stream);
  QSSM_GATE_PAIR(QSSM_F32, float, QSSM_F32, float)
  QSSM_GATE_PAIR(QSSM_F32, float, QSSM_F16, f16_t)
  QSSM_GATE_PAIR(QSSM_F32, float, QSSM_BF16, bf16_t)
  QSSM_GATE_PAIR(QSSM_F16, f16_t, QSSM_F16, f16_t)
  QSSM_GATE_PAIR(QSSM_F16, f16_t, QSSM_F32, float)
  QSSM_GATE_PAIR(QSSM_BF16, bf16_t, QSSM_BF16, bf16_t)
  QSSM_GATE_PAIR(QSSM_BF16, bf16_t, QSSM_F32, float)
#undef QSSM_GATE_PAIR
  return false;
}

}  // namespace qssm
