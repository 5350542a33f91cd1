/*
 * mi355x_rownorm.h -- C ABI of the MI355X (gfx950) row-wise reduce-then-normalize kernels.
 *
 * This is the whole surface the host operator layer binds.  It replaces the
 * kernel-entry functions of intel/torch-xpu-ops that take at::Tensor
 * (src/ATen/native/xpu/sycl/LayerNormKernels.h:19-59 and
 * src/ATen/native/xpu/sycl/SoftMaxKernels.h:19-43) with plain pointers and
 * sizes, so that any host (the C++ ATen layer in csrc/host, ctypes, a test
 * binary) can call the kernels without linking libtorch.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer into memory the caller owns.  No
 *    alignment beyond the element size is required of any pointer.
 *  - Tensors are dense row-major [M, N] (rows x normalized size); mean/rstd
 *    are float32 [M] whatever the input dtype, as at::toAccumulateType gives
 *    in src/ATen/native/xpu/LayerNorm.cpp:72-75.
 *  - Nothing here allocates, frees, synchronizes or throws.  Work is enqueued
 *    on `stream` (a hipStream_t passed as void*; NULL = the default stream)
 *    and the call returns at once; it is safe to call from several threads.
 *  - Return value: 0 on success, a negative ROWNORM_ERR_* for a rejected
 *    argument (nothing was launched), or a positive hipError_t value when a
 *    launch failed.  mi355x_rownorm_error_string() renders either.
 *  - M == 0 or N == 0 is a successful no-op, like the `if (M > 0)` guards in
 *    LayerNorm.cpp:77,236,301 and `numel() > 0` in SoftMaxKernels.cpp:2150
 *    (mean / rstd are not written then; the host layer fills them).
 *  - `eps` is a float where the reference's kernel entries take a double
 *    (LayerNormKernels.h:25): every supported dtype accumulates in float32, and
 *    the reference converts eps to that accumulate type before use
 *    (LayerNormKernels.cpp:1434), so nothing is lost; float64 rows are not
 *    computed here at all (the host layer passes them to the stock kernels).
 */
#ifndef MI355X_ROWNORM_H_
#define MI355X_ROWNORM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  ROWNORM_F32 = 0,
  ROWNORM_F16 = 1,
  ROWNORM_BF16 = 2
} rownorm_dtype;

enum {
  ROWNORM_OK = 0,
  ROWNORM_ERR_DTYPE = -1,     /* unknown dtype code or unsupported dtype pair */
  ROWNORM_ERR_SHAPE = -2,     /* negative size, or N beyond 2^30 elements */
  ROWNORM_ERR_NULL = -3,      /* a required pointer is NULL */
  ROWNORM_ERR_WORKSPACE = -4, /* workspace missing or smaller than *_workspace_bytes() */
  ROWNORM_ERR_OVERRIDE = -5,  /* a forced variant cannot run this shape */
  ROWNORM_ERR_SCRATCH_LIMIT = -6 /* mi355x_rms_norm_bwd_static: the call needs more than the static scratch */
};

/* Operation ids for mi355x_rownorm_plan / mi355x_rownorm_set_override. */
typedef enum {
  ROWNORM_OP_LAYER_NORM_FWD = 0,
  ROWNORM_OP_LAYER_NORM_BWD = 1,
  ROWNORM_OP_RMS_NORM_FWD = 2,
  ROWNORM_OP_RMS_NORM_BWD = 3,
  ROWNORM_OP_SOFTMAX_FWD = 4,
  ROWNORM_OP_SOFTMAX_BWD = 5,
  ROWNORM_OP_SOFTMAX_STRIDED_FWD = 6, /* mi355x_softmax_strided_fwd (override / strided_plan only) */
  ROWNORM_OP_SOFTMAX_STRIDED_BWD = 7,
  ROWNORM_OP_GROUP_NORM_FWD = 8,      /* mi355x_group_norm_fwd (override / group_norm_plan only) */
  ROWNORM_OP_GROUP_NORM_BWD = 9,
  ROWNORM_OP_COUNT = 10
} rownorm_op;

/* `mode` of the strided softmax entry points. */
enum {
  ROWNORM_SOFTMAX = 0,
  ROWNORM_LOG_SOFTMAX = 1,
  ROWNORM_SAFE_SOFTMAX = 2 /* forward only: slices with no finite element give 0 */
};

/* How one call is laid out on the GPU.  Replaces the reference's NormConfig
 * heuristics (src/ATen/native/xpu/sycl/Norm.h:225-370) and get_wgroup_size
 * (SoftMaxKernels.cpp:139-182); exposed so tests and logs can see the choice. */
typedef struct {
  int32_t resident;        /* 1: the row lives in registers (one HBM pass); 0: multi-pass streaming kernel */
  int32_t lanes_per_row;   /* G: lanes that share one row (8..1024) */
  int32_t packs_per_lane;  /* V: 16-byte packs each lane holds per row */
  int32_t block_threads;   /* threads per workgroup */
  int32_t rows_per_block;  /* rows a workgroup handles per iteration: block_threads / lanes_per_row */
  int32_t reserved;        /* mi355x_rownorm_plan: workgroups a row is split over or held by (norm ops,
                              rows beyond one workgroup's registers), else 0; mi355x_group_norm_plan:
                              1 when every pack lies in one channel */
  int64_t grid_blocks;     /* workgroups launched (persistent, grid-stride over rows) */
  int64_t partial_rows;    /* rows of the fp32 [partial_rows, N] column-sum workspace (backward only) */
} rownorm_plan;

const char* mi355x_rownorm_error_string(int code);

/* ABI revision; bumped when a signature changes. */
int mi355x_rownorm_abi_version(void);

/* native_layer_norm forward.  Replaces layer_norm_kernel(X, gamma, beta, M, N, eps, Y*, mean*, rstd*)
 * (LayerNormKernels.h:19-28).  gamma/beta may be NULL (treated as 1 / 0,
 * LayerNormKernels.cpp:281-285); mean/rstd may be NULL (not written; a few
 * rows far too long for the registers are then not split over workgroups).
 * w_dtype is the dtype of gamma and beta: equal to x_dtype, or ROWNORM_F32
 * with a 16-bit x (mixed precision, a CPU-ATen feature the reference lacks). */
int mi355x_layer_norm_fwd(const void* x, const void* gamma, const void* beta, void* y,
                          float* mean, float* rstd, int64_t M, int64_t N, float eps,
                          rownorm_dtype x_dtype, rownorm_dtype w_dtype, void* stream);

/* Bytes of scratch mi355x_layer_norm_bwd takes for this call.  Replaces the
 * at::empty/at::zeros scratch the reference allocates inside its entry point
 * (LayerNormKernels.cpp:1255-1264, Norm.h:263-283).  Two parts: the fp32 column
 * sums behind dgamma/dbeta (0 when neither is wanted; a shorter workspace is
 * ROWNORM_ERR_WORKSPACE), and, for a few rows far too long for the registers,
 * the partial sums of the split-row dX (the regime of Norm.h:632-812), which
 * follow the column sums.  A workspace that holds the first part only is
 * accepted: every row's dX then stays on one workgroup.  Rows beyond one
 * workgroup's registers in calls of many rows may be held four at a time by teams
 * of workgroups (dY and X read once; whole packs, 16-byte aligned tensors and
 * workspace, dx apart from dy and x, the bookkeeping and the bounded wait of
 * mi355x_rownorm_set_team_wait_us): the first part then holds one row a team,
 * which this query counts. */
size_t mi355x_layer_norm_bwd_workspace_bytes(int64_t M, int64_t N, rownorm_dtype x_dtype,
                                             rownorm_dtype w_dtype, int want_dgamma,
                                             int want_dbeta);

/* native_layer_norm_backward.  Replaces layer_norm_backward_kernel(dY, X, mean, rstd, gamma, M, N,
 * dX*, dgamma*, dbeta*) (LayerNormKernels.h:30-40).  Any of dx/dgamma/dbeta
 * may be NULL and is then skipped (LayerNormKernels.cpp:1140,1270-1406).
 * dx has x_dtype; dgamma/dbeta have w_dtype and are written in full (no
 * accumulation into previous contents).  Column sums are accumulated in fp32
 * and reduced in a fixed order: results are run-to-run deterministic. */
int mi355x_layer_norm_bwd(const void* dy, const void* x, const float* mean, const float* rstd,
                          const void* gamma, void* dx, void* dgamma, void* dbeta,
                          void* workspace, size_t workspace_bytes, int64_t M, int64_t N,
                          rownorm_dtype x_dtype, rownorm_dtype w_dtype, void* stream);

/* _fused_rms_norm forward.  Replaces rms_norm_kernel(X, gamma, M, N, eps, Y*, rstd*)
 * (LayerNormKernels.h:42-49). */
int mi355x_rms_norm_fwd(const void* x, const void* gamma, void* y, float* rstd, int64_t M,
                        int64_t N, float eps, rownorm_dtype x_dtype, rownorm_dtype w_dtype,
                        void* stream);

size_t mi355x_rms_norm_bwd_workspace_bytes(int64_t M, int64_t N, rownorm_dtype x_dtype,
                                           rownorm_dtype w_dtype, int want_dgamma);

/* _fused_rms_norm_backward.  Replaces rms_norm_backward_kernel(dY, X, rstd, gamma, M, N, dX*, dgamma*)
 * (LayerNormKernels.h:51-59). */
int mi355x_rms_norm_bwd(const void* dy, const void* x, const float* rstd, const void* gamma,
                        void* dx, void* dgamma, void* workspace, size_t workspace_bytes,
                        int64_t M, int64_t N, rownorm_dtype x_dtype, rownorm_dtype w_dtype,
                        void* stream);

/* Fused residual add -> norm (-> output cast), forward.  The step that precedes
 * the norm in a transformer block, h = x + residual, is formed in float32,
 * rounded once to x_dtype -- exactly what an elementwise add of the two tensors
 * gives -- written to `h` and normalized in the same pass: one read of x, one of
 * residual, one write of h and one of y, where an add followed by the norm reads
 * three tensors and writes two.  The reference has no such operator (its
 * forward, VectorizedLayerNormKernelFunctor in LayerNormKernels.cpp:469-586,
 * starts from the summed row); results equal the reference's norm applied to
 * that sum.  x, residual and h share x_dtype and the shape [M, N]; h may be the
 * memory of x or of residual (the usual in-place update of the residual
 * stream), y may not overlap them.  residual == NULL: no add, h is not touched
 * (may be NULL): the plain norm with the output cast.
 * y_dtype: x_dtype, or ROWNORM_F16 / ROWNORM_BF16 for float32 rows (a float32
 * residual stream feeding a 16-bit matrix multiply): y is rounded once, from
 * the float32 result.  Other arguments as mi355x_layer_norm_fwd /
 * mi355x_rms_norm_fwd. */
int mi355x_add_layer_norm_fwd(const void* x, const void* residual, const void* gamma,
                              const void* beta, void* h, void* y, float* mean, float* rstd,
                              int64_t M, int64_t N, float eps, rownorm_dtype x_dtype,
                              rownorm_dtype w_dtype, rownorm_dtype y_dtype, void* stream);
int mi355x_add_rms_norm_fwd(const void* x, const void* residual, const void* gamma, void* h,
                            void* y, float* rstd, int64_t M, int64_t N, float eps,
                            rownorm_dtype x_dtype, rownorm_dtype w_dtype, rownorm_dtype y_dtype,
                            void* stream);

/* Backward of the fused add -> norm.  h is the saved sum (the row that was
 * normalized), dy the gradient of y (x_dtype: the backward has no cast), dh_in
 * the gradient that reaches h by the residual path (NULL: none).  dh = the norm's
 * input gradient + dh_in, added in float32 and rounded once; it is the gradient
 * of both x and residual.  dh may be the memory of dh_in.  Workspace as for
 * mi355x_layer_norm_bwd / mi355x_rms_norm_bwd (same *_workspace_bytes). */
int mi355x_add_layer_norm_bwd(const void* dy, const void* dh_in, const void* h, const float* mean,
                              const float* rstd, const void* gamma, void* dh, void* dgamma,
                              void* dbeta, void* workspace, size_t workspace_bytes, int64_t M,
                              int64_t N, rownorm_dtype x_dtype, rownorm_dtype w_dtype,
                              void* stream);
int mi355x_add_rms_norm_bwd(const void* dy, const void* dh_in, const void* h, const float* rstd,
                            const void* gamma, void* dh, void* dgamma, void* workspace,
                            size_t workspace_bytes, int64_t M, int64_t N, rownorm_dtype x_dtype,
                            rownorm_dtype w_dtype, void* stream);

/* mi355x_rms_norm_bwd for callers that cannot allocate device memory: code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference, whose entry point
 * allocates its scratch itself (LayerNormKernels.cpp:1255-1264).  Same
 * arguments and results as mi355x_rms_norm_bwd (bit for bit, given the full
 * workspace) minus the workspace: the fp32 partial rows live in a 32 MiB array
 * inside the library's device image, one copy per GPU, held until the process
 * ends.  A call that would need more (mi355x_rms_norm_bwd_workspace_bytes()
 * above mi355x_rms_norm_bwd_static_limit_bytes(): on 256 compute units no launch
 * plan of the library itself, only a forced larger grid) fails with
 * ROWNORM_ERR_SCRATCH_LIMIT and
 * launches nothing.  Calls no hipMalloc / hipFree and no allocating library
 * routine.  Every call on one GPU shares that GPU's array: calls that overlap
 * in time on one GPU (two streams, two threads) race; calls on one stream are
 * ordered and safe.  Nothing in the array has to start at zero: each launch
 * writes every partial row before its second stage reads it.
 * Two rules for callers.  (1) The current device must be the device of
 * `stream` (as for any launch): the array's address is looked up for the current
 * device, each GPU holding its own copy.  (2) Before a call is recorded into a
 * HIP graph, make one ordinary call of the same shape on that device: the first
 * call on a device resolves the array's address (hipGetSymbolAddress), and the
 * first launch of a kernel loads its code object together with the 32 MiB array;
 * neither belongs inside a capture. */
size_t mi355x_rms_norm_bwd_static_limit_bytes(void);
int mi355x_rms_norm_bwd_static(const void* dy, const void* x, const float* rstd,
                               const void* gamma, void* dx, void* dgamma, int64_t M, int64_t N,
                               rownorm_dtype x_dtype, rownorm_dtype w_dtype, void* stream);

/* _softmax / _log_softmax over the innermost dimension of a dense [rows, N]
 * tensor.  Replaces _softmax_kernel / _log_softmax_kernel (SoftMaxKernels.h:19-29)
 * for the inner_size == 1 case (SoftMaxKernels.cpp:1663-1720).  out_dtype is
 * in_dtype, or ROWNORM_F32 with a ROWNORM_F16 input (half_to_float,
 * SoftMaxKernels.cpp:2131-2135).  Few, very long rows (fewer rows than half the
 * compute units, 4096 16-byte packs a row or more, 16-byte aligned x and y that do
 * not overlap) are each held by a team of workgroups, under the rules described at
 * mi355x_rownorm_set_team_wait_us; mi355x_softmax_bwd likewise (gi apart from grad
 * and y). */
int mi355x_softmax_fwd(const void* x, void* y, int64_t rows, int64_t N, rownorm_dtype in_dtype,
                       rownorm_dtype out_dtype, int is_log, void* stream);

/* _softmax_backward_data / _log_softmax_backward_data.  Replaces
 * _softmax_backward_kernel / _log_softmax_backward_kernel (SoftMaxKernels.h:31-43).
 * grad and y (the forward OUTPUT) share grad_dtype; gi has gi_dtype, which is
 * grad_dtype, or ROWNORM_F16 with ROWNORM_F32 grads (half_to_float,
 * src/ATen/native/xpu/SoftMax.cpp:49-55). */
int mi355x_softmax_bwd(const void* grad, const void* y, void* gi, int64_t rows, int64_t N,
                       rownorm_dtype grad_dtype, rownorm_dtype gi_dtype, int is_log,
                       void* stream);

/* _safe_softmax: softmax whose rows without any finite element (all -inf) come
 * out as zeros instead of NaN.  Replaces _safe_softmax_kernel
 * (SoftMaxKernels.h:45-46, SoftMaxKernels.cpp:2278-2299; the is_safe_softmax
 * branches at SoftMaxKernels.cpp:328-346).  Dtypes as for mi355x_softmax_fwd. */
int mi355x_safe_softmax_fwd(const void* x, void* y, int64_t rows, int64_t N,
                            rownorm_dtype in_dtype, rownorm_dtype out_dtype, void* stream);

/* _masked_softmax over the innermost dimension: elements whose mask byte is
 * non-zero are left out (treated as -inf); a row with every element masked is
 * NaN.  Replaces masked_softmax_kernel (SoftMaxKernels.h:48-52,
 * SoftMaxKernels.cpp:1901-2020 and 2301-2359).  `mask` is a dense
 * [mask_rows, N] buffer of one-byte booleans in device memory; data row r uses
 * mask row (r / mask_row_div) * mask_row_stride + r % mask_row_mod:
 *   mask of the input's shape            mask_rows = rows, div 1,   stride 1, mod 1
 *   [B, T] under a [B, H, T, T] input    mask_rows = B,    div H*T, stride 1, mod 1
 *   [T, T] under a [B, H, T, T] input    mask_rows = T,    div 1,   stride 0, mod T
 *   [B, 1, T, T] under [B, H, T, T]      mask_rows = B*T,  div H*T, stride T, mod T
 * A mapping that could leave the mask buffer, or rows >= 2^31, is rejected
 * with ROWNORM_ERR_SHAPE.  Input and output share `dtype`. */
int mi355x_masked_softmax_fwd(const void* x, const void* mask, void* y, int64_t rows, int64_t N,
                              int64_t mask_rows, int64_t mask_row_div, int64_t mask_row_stride,
                              int64_t mask_row_mod, rownorm_dtype dtype, void* stream);

/* _masked_softmax_backward: softmax backward with the saved output taken as 0
 * where the mask byte is non-zero, so those positions get a zero gradient.
 * Replaces masked_softmax_backward_kernel (SoftMaxKernels.h:54-58,
 * SoftMaxKernels.cpp:2022-2118 and 2361-2401).  Mask arguments as above;
 * grad, y and gi share `dtype`. */
int mi355x_masked_softmax_bwd(const void* grad, const void* y, const void* mask, void* gi,
                              int64_t rows, int64_t N, int64_t mask_rows, int64_t mask_row_div,
                              int64_t mask_row_stride, int64_t mask_row_mod, rownorm_dtype dtype,
                              void* stream);

/* native_group_norm on a dense NCHW-contiguous [N, C, HxW] input with `groups`
 * groups of C / groups channels.  Replaces group_norm_kernel
 * (src/ATen/native/xpu/sycl/GroupNormKernels.h:17-28, GroupNormKernels.cpp:
 * 364-530).  gamma/beta are [C] of w_dtype and may be NULL (1 / 0).  mean and
 * rstd are [N * groups] of w_dtype -- x_dtype, or ROWNORM_F32 beside fp32
 * weights -- as native_group_norm returns them; either may be NULL.  Pass
 * w_dtype = x_dtype when there are no weights.  C must be a multiple of
 * groups; N * groups < 2^31 and (C / groups) * HxW <= 2^30. */
int mi355x_group_norm_fwd(const void* x, const void* gamma, const void* beta, void* y, void* mean,
                          void* rstd, int64_t N, int64_t C, int64_t HxW, int64_t groups, float eps,
                          rownorm_dtype x_dtype, rownorm_dtype w_dtype, void* stream);

/* Bytes of device scratch mi355x_group_norm_bwd needs: two float32 [N, C]
 * arrays of per-sample channel sums; 0 when neither dgamma nor dbeta is wanted
 * and a (sample, group) row fits the registers (longer rows get dX from the
 * channel sums, so they always need the scratch).
 * The reference allocates the same two (ds, db) with at::empty
 * (GroupNormKernels.cpp:1398-1399). */
size_t mi355x_group_norm_bwd_workspace_bytes(int64_t N, int64_t C, int64_t HxW, int64_t groups,
                                             rownorm_dtype x_dtype, rownorm_dtype w_dtype,
                                             int want_dgamma, int want_dbeta);

/* native_group_norm_backward.  Replaces group_norm_backward_kernel
 * (GroupNormKernels.h:30-42, GroupNormKernels.cpp:1353-1589).  mean/rstd are
 * the forward's [N * groups] statistics in w_dtype.  dx, dgamma, dbeta may each
 * be NULL (not computed); dgamma/dbeta are [C] of w_dtype, summed in float32 in
 * a fixed order. */
int mi355x_group_norm_bwd(const void* dy, const void* x, const void* mean, const void* rstd,
                          const void* gamma, void* dx, void* dgamma, void* dbeta, void* workspace,
                          size_t workspace_bytes, int64_t N, int64_t C, int64_t HxW,
                          int64_t groups, rownorm_dtype x_dtype, rownorm_dtype w_dtype,
                          void* stream);

/* Launch layout of a GroupNorm call (no launch): one row is one (n, group)
 * slab of (C / groups) * HxW elements; `reserved` is 1 when HxW is a whole
 * number of 16-byte packs (per-pack weight lookup, channel sums fused into the
 * backward), 2 when only the rows are (a pack may straddle two channels: two
 * lookups per pack, sums still fused; needs HxW >= one pack and at most 512
 * channels a group), 0 for the general kernels; partial_rows is N for the
 * backward.  resident == 0: slabs beyond one workgroup's registers; the forward
 * of such slabs whose channels are whole packs is held by teams of workgroups
 * (one pass; the rules of mi355x_rownorm_set_team_wait_us apply), and
 * grid_blocks is then that launch's grid. */
int mi355x_group_norm_plan(int backward, int64_t N, int64_t C, int64_t HxW, int64_t groups,
                           rownorm_dtype x_dtype, rownorm_plan* out);

/* _softmax / _log_softmax / _safe_softmax over a dimension that is not
 * innermost: the dense tensor is viewed as [outer, dim_size, inner] and each of
 * the outer * inner columns of dim_size elements (inner apart in memory) is
 * normalized.  Replaces the spatial branch of host_softmax
 * (SoftMaxKernels.cpp:1721-1736, SpatialSoftmaxForwardKernelFunctor :725-950),
 * which the reference takes whenever inner_size != 1.  inner == 1 forwards to
 * the innermost-dimension kernels.  Dtypes as for mi355x_softmax_fwd; dim_size
 * and inner are limited to 2^30. */
int mi355x_softmax_strided_fwd(const void* x, void* y, int64_t outer, int64_t dim_size,
                               int64_t inner, rownorm_dtype in_dtype, rownorm_dtype out_dtype,
                               int mode, void* stream);

/* Backward of the above (SpatialSoftmaxBackwardKernelFunctor,
 * SoftMaxKernels.cpp:1387-1564, dispatched at :1877-1894).  mode is
 * ROWNORM_SOFTMAX or ROWNORM_LOG_SOFTMAX; dtypes as for mi355x_softmax_bwd. */
int mi355x_softmax_strided_bwd(const void* grad, const void* y, void* gi, int64_t outer,
                               int64_t dim_size, int64_t inner, rownorm_dtype grad_dtype,
                               rownorm_dtype gi_dtype, int mode, void* stream);

/* Launch layout of a strided softmax call (no launch).  In the result,
 * lanes_per_row is the number of lanes along `inner` (one 16-byte pack each),
 * rows_per_block the number of threads along dim_size that share one such
 * lane position, packs_per_lane the dim_size rows each of those holds;
 * resident == 0 means the multi-pass kernels, and then `reserved` is the number
 * of chunks the dim_size rows of a tile are cut into, one workgroup each (0: not
 * cut; the cut needs an output that does not overlap an input). */
int mi355x_softmax_strided_plan(int backward, int64_t outer, int64_t dim_size, int64_t inner,
                                rownorm_dtype dtype, rownorm_plan* out);

/* Reports the launch layout a call with these sizes would use on the current
 * device (no launch; needs no GPU when the device query fails: 256 compute
 * units are assumed).  x_dtype is the row dtype, w_dtype the weight dtype
 * (ignored by the softmax ops).  The strided softmax ops have their own query above.
 * The norm forwards and the softmax ops also look at their pointers: this reports the layout for
 * tensors that start on a 128-byte line; rows of at most 64 packs in tensors
 * that do not take one pack a lane (lanes_per_row = packs rounded up to a
 * power of two).  Unmasked softmax calls on ragged rows (N not a whole number
 * of packs) of at most 2048 16-bit / 1024 float32 elements, and on rows of up to
 * 12 whole packs that fit the reported layout badly, with 16-byte aligned
 * tensors and one dtype, run through LDS-staged kernels instead of the layout
 * reported here (a forced layout keeps the reported kernels).  The query
 * describes the plain call: the fused residual add keeps 1024 lanes for 16-bit
 * rows of 16392..24576 elements and takes the multi-pass kernel beyond 12 packs a
 * lane (float32 LayerNorm: 10), and the masked softmax calls beyond 32 elements a
 * lane on 1024 lanes (rows of more than 32768 elements; a forced layout beyond
 * that is ROWNORM_ERR_OVERRIDE for a masked call). */
int mi355x_rownorm_plan(rownorm_op op, int64_t M, int64_t N, rownorm_dtype x_dtype,
                        rownorm_dtype w_dtype, rownorm_plan* out);

/* The same query for tensors that do NOT all start on a 128-byte line
 * (off_line != 0), which is what the norm forwards and the softmax ops see
 * through their pointers: rows of at most 64 packs then take one pack a lane.
 * off_line == 0 is mi355x_rownorm_plan. */
int mi355x_rownorm_plan_at(rownorm_op op, int64_t M, int64_t N, rownorm_dtype x_dtype,
                           rownorm_dtype w_dtype, int off_line, rownorm_plan* out);

/* Test and tuning hook: force lanes_per_row / packs_per_lane / threads per
 * workgroup / workgroups per compute unit for one op (0 keeps the automatic
 * choice for that field; lanes_per_row == -1 forces the multi-pass kernel, and with
 * block_threads == 1 beside it a norm backward goes to teams of workgroups however few
 * rounds of rows they make).  Process-global;
 * the four fields of an op are stored as one atomic word, so a call that runs
 * while another thread changes the override uses the old or the new variant,
 * never a mix.  Production callers never use it: with no override set (the
 * state a process starts in) every entry point is re-entrant, and the only
 * mutable global state any of them touches is the call counter and the
 * bookkeeping slots of the team forward described at
 * mi355x_rownorm_set_team_wait_us.  A call whose shape the forced variant cannot hold
 * fails with ROWNORM_ERR_OVERRIDE instead of silently choosing another, and so
 * does a field outside 0..65535. */
int mi355x_rownorm_set_override(rownorm_op op, int lanes_per_row, int packs_per_lane,
                                int block_threads, int blocks_per_cu);

/* Test hook for the rows that a team of workgroups holds in registers (LayerNorm /
 * RMSNorm forward rows beyond 131072 16-bit or 65536 float32 elements, whole
 * 16-byte packs, no residual add, no cast, y not overlapping x; GroupNorm forward
 * slabs of that size; softmax / log_softmax forward and backward of few, very long
 * rows; LayerNorm / RMSNorm backward rows beyond one workgroup's registers in calls of
 * many rows; GroupNorm backward slabs of long whole-pack channels): how long a workgroup waits for the others of its team before it sums the
 * whole row itself (a second pass over the inputs, the same result to rounding), in
 * microseconds; 0xffffffff
 * restores the default, one second.  0 makes every wait give up at once, which is
 * how the tests exercise that path without making any kernel hang.  Process-global.
 * Such calls draw an id and one of 16 bookkeeping slots in library-owned device
 * memory from process-wide counters; results do not depend on which slot a call
 * gets, and two calls that share a slot while both run (more than 16 such calls in
 * flight across streams) each detect it, their workgroups summing their rows
 * themselves.  On a stream under capture these rows take the multi-launch kernels
 * instead. */
int mi355x_rownorm_set_team_wait_us(unsigned int microseconds);

/* Measurement aid, no counterpart in the reference: a plain streaming kernel over
 * `bytes` bytes (a multiple of 16; 16-byte aligned device pointers) of each
 * tensor, in the read : write mixes of this operator family -- mode 0: c = a
 * (1 : 1, a forward's traffic), mode 1: c = a + b as 32-bit integers (2 : 1, a
 * backward's), mode 2: a and b are read and summed, and only
 * min(bytes / 16384, 2048) * 4096 bytes of c are written.  What such a kernel
 * reaches is the practical ceiling an operator's fraction of the HBM peak is read
 * against, and the kernel of known size that rocprofv3's FETCH_SIZE / WRITE_SIZE
 * readings are scaled by.  Launches on `stream`, allocates nothing. */
int mi355x_rownorm_stream_probe(const void* a, const void* b, void* c, size_t bytes, int mode,
                                void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355X_ROWNORM_H_ */
