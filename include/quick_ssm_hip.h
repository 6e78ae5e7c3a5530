/*
 * quick_ssm_hip.h -- C ABI of libquick_ssm_hip.so, the gfx950 (MI355X) implementation of
 * quick_ssm's gated linear scan
 *
 *     h(t) = a(t) * h(t-1) + b(t) * x(t),   h(-1) = 0
 *     y(t) = c(t) * h(t)
 *
 * and of its reverse-time gradient
 *
 *     dH(t) = c(t) * dy(t) + a(t+1) * dH(t+1),   dH(L) = 0
 *     dx = b * dH,  db = x * dH,  da(t) = h(t-1) * dH(t),  dc = dy * h.
 *
 * The reference has no native layer (its device code is six Triton kernels launched from
 * Python), so the entry points below are what a binding of its device path would call.  Each
 * one names the reference function it stands in for.
 *
 * Conventions
 *   - All tensors are [B, L, D] with D contiguous (element stride 1).  Batch and time strides
 *     are passed in elements, so sliced views need no copy.
 *   - Plain pointers and sizes only; every buffer is owned by the caller.  The library never
 *     allocates device memory and never synchronises: kernels are enqueued on `stream`.
 *     (qssm_scan_forward_static alone works in an array of the library's own; it says so below.)
 *   - Arithmetic is fp32 whatever the storage type; y and the gradients are rounded once.
 *   - Return value: 0 on success, a QSSM_E* code or a hipError_t (> 0) otherwise;
 *     qssm_error_string() describes the last failure on the calling thread.
 *   - Entry points are re-entrant (no global state), with the same one exception.
 */
#ifndef QUICK_SSM_HIP_H
#define QUICK_SSM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define QSSM_API __attribute__((visibility("default")))
#else
#define QSSM_API
#endif

#define QSSM_VERSION 200 /* major*10000 + minor*100 + patch; 0.2.0: qssm_plan_scan without `tune`, qssm_plan.keep_tiles */

/* storage types */
#define QSSM_F32 0
#define QSSM_F16 1
#define QSSM_BF16 2

/* error codes (negative; positive values are hipError_t) */
#define QSSM_EINVAL (-1)    /* bad argument (null pointer, size, dtype, plan mismatch) */
#define QSSM_EALIGN (-2)    /* pointer or stride not aligned to plan.vec elements */
#define QSSM_EWORKSPACE (-3)/* workspace smaller than plan.workspace_bytes */
#define QSSM_ESTATE (-4)    /* device status word reports a failed launch */

/* plan directions */
#define QSSM_FORWARD 0
#define QSSM_BACKWARD 1

/*
 * Launch geometry of one scan launch.  A "tile" is one workgroup's share: a strip of
 * `strip_cols` adjacent columns of one batch row, times `seg_len` consecutive time steps.
 * Tiles of one (batch, strip) chain are grouped in clusters of `cluster` consecutive tiles; a
 * tile reads the per-tile maps of its cluster through the workspace and one state per cluster
 * is handed from cluster to cluster.  `ckpt_stride` is the spacing of the fp32 states h(t-1)
 * kept for the backward.
 */
typedef struct qssm_plan {
  int32_t B, L, D;
  int32_t in_dtype;       /* x, a, b, c and dx, da, db, dc */
  int32_t out_dtype;      /* y and dy */
  int32_t direction;      /* QSSM_FORWARD / QSSM_BACKWARD */
  int32_t vec;            /* adjacent columns per lane: 1, 2 or 4; 8 for a forward over 16-bit storage */
  int32_t steps;          /* consecutive time steps per lane: 4 or 8 */
  int32_t threads;        /* lanes per workgroup: 256, 512 or 1024 */
  int32_t g_log2;         /* log2(lanes per row of a strip) */
  int32_t strip_cols;     /* vec << g_log2 */
  int32_t seg_len;        /* steps * (threads >> g_log2) */
  int32_t n_strips;       /* ceil(D / strip_cols) */
  int32_t n_seg;          /* ceil(L / seg_len) */
  int32_t cluster;        /* tiles per cluster (power of two) */
  int32_t n_super;        /* ceil(n_seg / cluster) */
  int32_t ckpt_stride;    /* spacing (time steps) of saved states; divides seg_len */
  int32_t n_ckpt;         /* ceil(L / ckpt_stride) */
  int32_t lds_bytes;      /* dynamic LDS per workgroup */
  int32_t keep_tiles;     /* forward: the last keep_tiles tiles of every chain load their operands with ordinary
                             loads, so that the backward, which starts there, finds them in the caches; the rest
                             streams past the caches.  0 switches it off. */
  int32_t compute_dtype;  /* gated scans: the type the layer rounds its gates' outputs to (its compute dtype): the
                             projections' storage type, or QSSM_F16 / QSSM_BF16 for fp32 projections.  Plain scans:
                             in_dtype. */
  uint64_t control_bytes;   /* control block the launch needs (status word + ticket counters) */
  uint64_t workspace_bytes; /* workspace the launch needs (words exchanged between workgroups) */
  uint64_t ckpt_elems;      /* B * n_ckpt * D floats */
} qssm_plan;

/* element strides of one [B, L, D] tensor; the D stride is 1 by contract */
typedef struct qssm_strides {
  int64_t b, l;
} qssm_strides;

/* Library version (QSSM_VERSION of the build). */
QSSM_API int qssm_version(void);

/* Text for the last error raised on the calling thread ("" if none). */
QSSM_API const char* qssm_error_string(void);

/*
 * Choose the launch geometry for a shape.
 *   align_elems : largest power of two (<= 8) that divides D, every batch/time stride, and
 *                 every base address expressed in elements, over all tensors of the launch.
 *   ckpt_stride : 0 lets the forward plan pick; a backward plan (and a forward plan that must
 *                 match one) passes the stride the saved states were written with.
 * Stands in for the grid/block arithmetic of block_scan_forward_3d
 * (quick_ssm/triton_forwards.py:157-167) and block_scan_backward_3d
 * (quick_ssm/triton_backwards.py:195-204).
 */
QSSM_API int qssm_plan_scan(int32_t B, int32_t L, int32_t D, int32_t in_dtype, int32_t out_dtype,
                   int32_t direction, int32_t align_elems, int32_t ckpt_stride, qssm_plan* plan);

/*
 * qssm_plan_scan with single choices of the planner overridden.  For tests (which force every launch geometry
 * through the same inputs) and for geometry sweeps; a binding of the reference has no use for it.
 *   tune : bit fields, a zero field keeping the automatic choice: (g_log2 + 1) | steps << 8 | max vec << 16 |
 *          threads code << 24 (1: 256, 2: 512, 3: 1024) | (log2(cluster) + 1) << 28.  tune = 0 is qssm_plan_scan.
 * No counterpart in the reference.
 */
QSSM_API int qssm_plan_scan_tuned(int32_t B, int32_t L, int32_t D, int32_t in_dtype, int32_t out_dtype,
                         int32_t direction, int32_t align_elems, int32_t ckpt_stride, int32_t tune,
                         qssm_plan* plan);

/*
 * Two device buffers accompany every launch, both owned by the caller and both zero-filled
 * (qssm_zero_fill) when they are allocated:
 *
 *   control    status word, a launch count and one ticket counter per chain (plan.control_bytes).
 *              A launch needs the status word and the ticket counters zero on entry and leaves them
 *              zero, except that the status word becomes 1 if a tile gave up waiting for a neighbour
 *              (outputs downstream of it are NaN), and 2 if a ticket counter was not zero on entry
 *              (every output of the launch is NaN).  Either way the results are invalid and both
 *              buffers must be zero-filled again before the next launch.
 *   workspace  the words tiles hand to each other (plan.workspace_bytes; may be 0).  Words are
 *              tagged with the launch's epoch, so nothing has to be cleared between launches:
 *              zero-fill it once, and again before an epoch value would be reused.
 *
 * Launches that share these buffers must be ordered on one stream and carry different epochs.  Two
 * ways to number them; use one per pair of buffers from zero-fill to zero-fill:
 *   epoch != 0   the caller counts (1, 2, 3, ...).
 *   epoch == 0   the library counts in the control block: the launch reads its epoch from device
 *                memory and a one-lane kernel behind it adds one.  Nothing launch-specific is then
 *                baked into kernel arguments, so launches captured in a HIP graph replay correctly
 *                (the count wraps after 2^32 - 1 launches; zero-fill the workspace before that).
 */

/* Zero-fill a buffer with a fill kernel on `stream` (safe under graph capture; no hipMemset). */
QSSM_API int qssm_zero_fill(void* buffer, uint64_t bytes, void* stream);

/* Read back the status word of a control block (synchronises `stream`).  0 = every launch since
 * the last zero-fill completed. */
QSSM_API int qssm_control_status(const void* control, void* stream, int32_t* status);

/* Enqueue a copy of the status word into `host_status` (pinned host memory) on `stream`, without waiting:
 * the word is sticky until the control block is zero-filled, so a later look at `host_status` sees any failure
 * of a launch ordered before the copy.  What a training loop polls instead of synchronising. */
QSSM_API int qssm_control_status_async(const void* control, int32_t* host_status, void* stream);

/*
 * Forward scan: one pass that reads x, a, b, c once and writes y once.
 *   c          may be NULL (treated as 1, so y = h): the block_scan_forward_3d case.
 *   y          may be NULL (state-only pass: only `ckpt` is produced).
 *   h_out      optional fp32 [B, L, D] (strides sh): every h(t); the checkpoint=False case.
 *   ckpt       optional fp32 [B, n_ckpt, D] contiguous: h(t-1) at t = k * ckpt_stride.
 *   epoch      0 (the library counts launches in the control block), or a nonzero value different
 *              from the epoch of every earlier launch that used this workspace since it was last
 *              zero-filled (a per-workspace counter does it).
 *   control, workspace: see above.
 * Replaces _TritonScanFunction.forward's per-tile body (quick_ssm/scan_interface.py:91-107):
 * block_scan_forward_3d (quick_ssm/triton_forwards.py:134-172, three launches + fp32 scratch)
 * followed by y = c * h and the cast to out_dtype.
 */
QSSM_API int qssm_scan_forward(const qssm_plan* plan,
                      const void* x, qssm_strides sx,
                      const void* a, qssm_strides sa,
                      const void* b, qssm_strides sb,
                      const void* c, qssm_strides sc,
                      void* y, qssm_strides sy,
                      float* h_out, qssm_strides sh,
                      float* ckpt,
                      void* control, uint64_t control_size,
                      void* workspace, uint64_t workspace_bytes, uint32_t epoch,
                      void* stream);

/*
 * Forward scan for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): qssm_scan_forward without the control block, workspace and epoch
 * arguments.  Both buffers live in one array of QSSM_STATIC_SCRATCH_BYTES inside the library's device image;
 * every GPU the library runs on holds its own copy until the process ends.  The call allocates nothing and
 * never synchronises; its first call on a device looks the array's address up (make that call outside a
 * capture).  Launches number themselves in the array (as with epoch 0), so a captured call replays correctly.
 *   - Shapes whose plan needs more than 256 KiB of control block (4095 chains) or more workspace than the rest
 *     of the array are refused with QSSM_EWORKSPACE; the headline shape (bf16, B=8 L=4096 D=2048: 20 MiB) fits.
 *   - All calls on one GPU share that GPU's array: they must be ordered on one stream (or otherwise not
 *     overlap); calls that overlap on one GPU race.  The array keeps the last call's words, which their flag
 *     values make harmless; status word and ticket counters are cleared at the start of every call.
 * Results are those of qssm_scan_forward for the same plan, bit for bit.
 * No counterpart in the reference (its Triton launches allocate their scratch through torch,
 * quick_ssm/triton_forwards.py:150-156); it exists for the callers named above.
 */
#define QSSM_STATIC_SCRATCH_BYTES (32u << 20)
QSSM_API int qssm_scan_forward_static(const qssm_plan* plan,
                             const void* x, qssm_strides sx,
                             const void* a, qssm_strides sa,
                             const void* b, qssm_strides sb,
                             const void* c, qssm_strides sc,
                             void* y, qssm_strides sy,
                             float* h_out, qssm_strides sh,
                             float* ckpt,
                             void* stream);

/*
 * Forward scan with a carried state: the same launch, started from `h_init` instead of zero and/or
 * reporting the state after the last step, so that a sequence can be scanned in pieces (chunked
 * prefill, token-by-token generation) with results identical to one scan over the whole of it.
 *   h_init     optional fp32 [B, D] contiguous: h(-1).  NULL = zero.
 *   h_final    optional fp32 [B, D] contiguous: receives h(L-1).  NULL = not wanted.
 * All other arguments as qssm_scan_forward, which is this call with both set to NULL.
 * No counterpart in the reference, whose recurrence always starts from h(-1) = 0
 * (quick_ssm/scan_interface.py:15-21); its README lists a generation mode as future work
 * (README.md:176-184).
 */
QSSM_API int qssm_scan_forward_carry(const qssm_plan* plan,
                            const void* x, qssm_strides sx,
                            const void* a, qssm_strides sa,
                            const void* b, qssm_strides sb,
                            const void* c, qssm_strides sc,
                            void* y, qssm_strides sy,
                            float* h_out, qssm_strides sh,
                            float* ckpt,
                            const float* h_init, float* h_final,
                            void* control, uint64_t control_size,
                            void* workspace, uint64_t workspace_bytes, uint32_t epoch,
                            void* stream);

/*
 * Backward scan: one reverse-time pass that reads x, a, b, c, dy once and writes dx, da, db,
 * dc once.  h is rebuilt inside each tile from `ckpt` (the checkpoint=True case), or read from
 * `h` when that is given (the checkpoint=False case and block_scan_backward_3d's signature);
 * exactly one of `ckpt` / `h` must be non-NULL.  Any of dx, da, db, dc may be NULL (skipped).
 * Replaces _TritonScanFunction.backward's per-tile body (quick_ssm/scan_interface.py:125-145):
 * the forward re-run (:133-134) plus block_scan_backward_3d
 * (quick_ssm/triton_backwards.py:168-209) plus the casts at :148-152.
 */
QSSM_API int qssm_scan_backward(const qssm_plan* plan,
                       const void* x, qssm_strides sx,
                       const void* a, qssm_strides sa,
                       const void* b, qssm_strides sb,
                       const void* c, qssm_strides sc,
                       const void* dy, qssm_strides sdy,
                       const float* h, qssm_strides sh,
                       const float* ckpt,
                       void* dx, qssm_strides sdx,
                       void* da, qssm_strides sda,
                       void* db, qssm_strides sdb,
                       void* dc, qssm_strides sdc,
                       void* control, uint64_t control_size,
                       void* workspace, uint64_t workspace_bytes, uint32_t epoch,
                       void* stream);

/*
 * Backward scan with a carried state: the mirror image of qssm_scan_forward_carry.
 *   h_init     the h(-1) the forward started from (needed for da at t = 0).  NULL = zero.
 *   dh_final   optional fp32 [B, D]: gradient arriving at h(L-1) from whatever consumed h_final
 *              (the next piece's dh_init when a sequence is scanned in pieces).  NULL = zero.
 *   dh_init    optional fp32 [B, D]: receives the gradient of h(-1), a(0) * dH(0).  NULL = not wanted.
 * All other arguments as qssm_scan_backward, which is this call with the three set to NULL.
 * No counterpart in the reference (see qssm_scan_forward_carry).
 */
QSSM_API int qssm_scan_backward_carry(const qssm_plan* plan,
                             const void* x, qssm_strides sx,
                             const void* a, qssm_strides sa,
                             const void* b, qssm_strides sb,
                             const void* c, qssm_strides sc,
                             const void* dy, qssm_strides sdy,
                             const float* h, qssm_strides sh,
                             const float* ckpt,
                             const float* h_init, const float* dh_final, float* dh_init,
                             void* dx, qssm_strides sdx,
                             void* da, qssm_strides sda,
                             void* db, qssm_strides sdb,
                             void* dc, qssm_strides sdc,
                             void* control, uint64_t control_size,
                             void* workspace, uint64_t workspace_bytes, uint32_t epoch,
                             void* stream);

/*
 * The same two launches with their arguments in one block: a binding that keeps such a block per shape only
 * patches the pointers between calls, which matters where launches are small enough for the host side of a call
 * to bound the step (the reference's copy task: B=32, L=64, 12 layers).  Fields as the arguments of
 * qssm_scan_forward_carry / qssm_scan_backward_carry of the same names.
 */
typedef struct qssm_forward_call {
  const qssm_plan* plan;
  const void *x, *a, *b, *c;
  void* y;
  float* h_out;
  float* ckpt;
  const float* h_init;
  float* h_final;
  qssm_strides sx, sa, sb, sc, sy, sh;
  void* control;
  uint64_t control_size;
  void* workspace;
  uint64_t workspace_bytes;
  uint32_t epoch;
  uint32_t reserved;
  void* stream;
} qssm_forward_call;

typedef struct qssm_backward_call {
  const qssm_plan* plan;
  const void *x, *a, *b, *c, *dy;
  const float* h;
  const float* ckpt;
  const float* h_init;
  const float* dh_final;
  float* dh_init;
  void *dx, *da, *db, *dc;
  qssm_strides sx, sa, sb, sc, sdy, sh, sdx, sda, sdb, sdc;
  void* control;
  uint64_t control_size;
  void* workspace;
  uint64_t workspace_bytes;
  uint32_t epoch;
  uint32_t reserved;
  void* stream;
} qssm_backward_call;

QSSM_API int qssm_scan_forward_call(const qssm_forward_call* call);
QSSM_API int qssm_scan_backward_call(const qssm_backward_call* call);

/*
 * Gate prologue of the SSM layer: the five projection outputs [rows, S] (row strides ld_* in elements,
 * so they may be column slices of one wide GEMM output) become the scan's four operands, contiguous
 * [rows, S] in `out_dtype`, in one pass:
 *   a = sigmoid(A_pre), x = B_in, c = silu(Ca) * Cb, b = sigmoid(D_pre)
 * fp32 arithmetic, one rounding per result.  Built pairs (in, out): (f32, f32|f16|bf16), (f16, f16|f32),
 * (bf16, bf16|f32).  Replaces the elementwise chain of SSM.forward, quick_ssm/layers.py:76-88.
 */
QSSM_API int qssm_gates_forward(const void* A_pre, int64_t ld_a, const void* B_in, int64_t ld_b,
                       const void* Ca, int64_t ld_ca, const void* Cb, int64_t ld_cb,
                       const void* D_pre, int64_t ld_d,
                       void* a, void* x, void* c, void* b,
                       int64_t rows, int32_t S, int32_t in_dtype, int32_t out_dtype, void* stream);

/*
 * Backward of the gate prologue in one pass: gradients of the scan's operands (contiguous [rows, S] in
 * `out_dtype`) and the saved projection outputs give the gradients of the projection outputs (contiguous
 * [rows, S] in `in_dtype`):
 *   dA_pre = g_a * a (1 - a), dB_in = g_x, dD_pre = g_b * b (1 - b),
 *   dCa = g_c * Cb * s (1 + Ca (1 - s)), dCb = g_c * Ca * s, with s = sigmoid(Ca).
 * Replaces what autograd records for quick_ssm/layers.py:76-88.
 */
QSSM_API int qssm_gates_backward(const void* g_a, const void* g_x, const void* g_c, const void* g_b,
                        const void* A_pre, int64_t ld_a, const void* Ca, int64_t ld_ca,
                        const void* Cb, int64_t ld_cb, const void* D_pre, int64_t ld_d,
                        void* dA_pre, void* dB_in, void* dCa, void* dCb, void* dD_pre,
                        int64_t rows, int32_t S, int32_t in_dtype, int32_t out_dtype, void* stream);

/*
 * The same with a row stride `ld_grad` (elements, >= S) for the five gradients, so that they can be written as
 * column slices of one wide [rows, 5 S] tensor: the gradient of a single GEMM that produced all five projections.
 */
QSSM_API int qssm_gates_backward_strided(const void* g_a, const void* g_x, const void* g_c, const void* g_b,
                                const void* A_pre, int64_t ld_a, const void* Ca, int64_t ld_ca,
                                const void* Cb, int64_t ld_cb, const void* D_pre, int64_t ld_d,
                                void* dA_pre, void* dB_in, void* dCa, void* dCb, void* dD_pre, int64_t ld_grad,
                                int64_t rows, int32_t S, int32_t in_dtype, int32_t out_dtype, void* stream);

/*
 * The scan with the layer's gate activations inside it (quick_ssm/layers.py:76-104 as one launch each way): the
 * operands are the five projection outputs, [B, L, S] with batch and time strides in elements (so they may be
 * column slices of one wide GEMM output), stored as f16 or bf16, and
 *     a = sigmoid(A_pre), x = B_in, b = sigmoid(D_pre), c = silu(Ca) * Cb
 * are formed in registers, rounded to the projections' storage type exactly where the layer's cast to its compute
 * dtype rounds them (layers.py:85-88); then h(t) = a h(t-1) + b x, y = c h as in qssm_scan_forward.  The backward
 * returns the projections' gradients directly,
 *     dA_pre = da a (1 - a), dB_in = dx, dD_pre = db b (1 - b), dCa = dc Cb s (1 + Ca (1 - s)), dCb = dc Ca s,
 * s = sigmoid(Ca), with da, db, dc rounded to the storage type as qssm_scan_backward stores them.  The tensors a,
 * x, b, c and their gradients never reach HBM: 12 instead of 30 bytes per element forward and 22 instead of 46
 * backward for bf16.
 *   - fp32 projections (the reference's default layer: fp32 parameters, 16-bit compute dtype) are taken as well:
 *     `compute_dtype` then names the 16-bit type (or QSSM_F32) the gates' outputs and the scan's gradients are
 *     rounded to, in registers, where the layer's casts round them; y and dy are f32.  20 + 4 instead of 28 + 12
 *     bytes per element forward, 24 + 20 instead of 44 + 20 backward.
 *   - Plans come from qssm_plan_scan_gated (one geometry: 8 bytes x 8 steps per lane, 256 lanes); shapes it
 *     refuses (D < 128, rows not 16-byte aligned) take qssm_gates_* + qssm_scan_*.
 *   - ckpt, control, workspace, epoch: as for qssm_scan_forward / qssm_scan_backward; the backward needs the saved
 *     states (the checkpoint=True case) and y / dy stored as the projections are (16-bit projections forward: or
 *     as f32).
 * Replaces SSM.forward's elementwise chain and scan call, quick_ssm/layers.py:76-104, and what autograd records
 * for them.
 */
QSSM_API int qssm_plan_scan_gated(int32_t B, int32_t L, int32_t D, int32_t dtype, int32_t compute_dtype,
                         int32_t out_dtype, int32_t direction, int32_t align_elems, int32_t ckpt_stride,
                         qssm_plan* plan);

QSSM_API int qssm_scan_gated_forward(const qssm_plan* plan,
                            const void* A_pre, qssm_strides sA,
                            const void* B_in, qssm_strides sB,
                            const void* Ca, qssm_strides sCa,
                            const void* Cb, qssm_strides sCb,
                            const void* D_pre, qssm_strides sD,
                            void* y, qssm_strides sy,
                            float* ckpt,
                            void* control, uint64_t control_size,
                            void* workspace, uint64_t workspace_bytes, uint32_t epoch,
                            void* stream);

QSSM_API int qssm_scan_gated_backward(const qssm_plan* plan,
                             const void* A_pre, qssm_strides sA,
                             const void* B_in, qssm_strides sB,
                             const void* Ca, qssm_strides sCa,
                             const void* Cb, qssm_strides sCb,
                             const void* D_pre, qssm_strides sD,
                             const void* dy, qssm_strides sdy,
                             const float* ckpt,
                             void* dA_pre, qssm_strides sdA,
                             void* dB_in, qssm_strides sdB,
                             void* dCa, qssm_strides sdCa,
                             void* dCb, qssm_strides sdCb,
                             void* dD_pre, qssm_strides sdD,
                             void* control, uint64_t control_size,
                             void* workspace, uint64_t workspace_bytes, uint32_t epoch,
                             void* stream);

/*
 * RMSNorm of the SSM layer over the last axis: y = x * weight / sqrt(mean(x^2) + eps).
 * x is [rows, H] with row stride ld_x elements, weight [H], y [rows, H] contiguous, all stored as `dtype`
 * (f32, f16 or bf16); fp32 arithmetic, one rounding per result.  `rstd` ([rows] fp32, or NULL) receives
 * 1 / sqrt(mean(x^2) + eps) per row for the backward.  One pass: x is read once, y written once.
 * Replaces RMSNorm.forward, quick_ssm/layers.py:14-17 (pow, mean, add, sqrt, divide, multiply as six
 * passes).
 */
QSSM_API int qssm_rmsnorm_forward(const void* x, int64_t ld_x, const void* weight, void* y, float* rstd,
                         int64_t rows, int32_t H, float eps, int32_t dtype, void* stream);

/*
 * Backward of the RMSNorm in one pass over dy and x (row strides ld_dy, ld_x elements):
 *   g = dy * weight, s = sum(g * x), r = rstd:  dx = r * g - x * r^3 * s / H,  dweight = sum over rows dy * x * r.
 * dx is [rows, H] contiguous and dweight [H], both stored as `dtype`.  `rstd` may be NULL (r is then
 * recomputed from x and eps).  `partial` is fp32 scratch of `partial_rows` x H floats
 * (partial_rows >= QSSM_RMSNORM_MIN_PARTIAL_ROWS; more rows, up to 512, let more workgroups run); dweight
 * is summed from it in a fixed order by a second small launch, so results repeat bit for bit.
 * Replaces what autograd records for quick_ssm/layers.py:14-17.
 */
#define QSSM_RMSNORM_MIN_PARTIAL_ROWS 8
QSSM_API int qssm_rmsnorm_backward(const void* dy, int64_t ld_dy, const void* x, int64_t ld_x, const void* weight,
                          const float* rstd, void* dx, void* dweight, float* partial, int32_t partial_rows,
                          int64_t rows, int32_t H, float eps, int32_t dtype, void* stream);

/*
 * Column sums of a [rows, S] matrix with row stride `ld` (elements; a column block of a wider matrix is fine):
 * out[s] = sum over r of x[r, s], accumulated in fp32 in a fixed order (results repeat bit for bit) and stored in
 * x's storage type.  `partial` is fp32 scratch of `partial_rows` x S floats (64 rows suit a few thousand rows of x;
 * more rows of x per row of scratch only make the first of the two launches longer).
 * This is the bias gradient of a linear map, which autograd otherwise computes with a library reduction per bias:
 * replaces what autograd records for the `+ bias` of A_proj and out_proj, quick_ssm/layers.py:50-58,76,106.
 */
QSSM_API int qssm_colsum(const void* x, int64_t ld, int64_t rows, int32_t S, int32_t dtype, float* partial,
                         int32_t partial_rows, void* out, void* stream);

/*
 * Streaming copy of `bytes` bytes (16-byte aligned, multiple of 16) on `stream`.  Not part of
 * the scan: it is the known-size kernel against which rocprof's FETCH_SIZE / WRITE_SIZE
 * counters and the achievable-bandwidth ceiling are calibrated by the benchmark.
 */
QSSM_API int qssm_copy_bytes(void* dst, const void* src, uint64_t bytes, void* stream);

/*
 * Host-side mirror of the launch counter that launches with epoch argument 0 keep in their control
 * block (no GPU work): for a counter reading `count` before a launch, `*flag` is the flag value the
 * launch tags its words with, `*next` the reading afterwards, and `*wipes` whether the launch's
 * prologue clears the whole scratch array first (only qssm_scan_forward_static, `static_scratch`
 * nonzero, ever does).  No counterpart in the reference; it lets a caller, or a test, follow the
 * numbering across its wrap without driving a GPU through 2^32 launches.
 */
QSSM_API int qssm_launch_count_step(uint32_t count, int32_t static_scratch, uint32_t* flag, uint32_t* next,
                                    int32_t* wipes);

#ifdef __cplusplus
}
#endif
#endif /* QUICK_SSM_HIP_H */
