/*
 * Operator-level C ABI of the MI355X (gfx950) CVM backend.
 *
 * One entry point per reference operator kernel.  These are what a
 * `CVM_REGISTER_GLOBAL("cvm.runtime.hip.<op>")` wrapper calls after unpacking
 * its DLTensor arguments -- the role the `cuda_*` wrappers declared in the
 * reference's src/runtime/cuda/ops/cuda_ops.h:111-235 play for the CUDA
 * device.  Plain pointers and sizes only; no HIP or torch types.
 *
 * Conventions
 *  - every tensor pointer is DEVICE memory holding contiguous row-major int32
 *    (the reference's storage contract, src/runtime/graph_runtime.cc:505-506);
 *  - shape arrays are HOST memory, int64, length ndim (ndim <= 6);
 *  - `stream` is a hipStream_t passed as void* (NULL = default stream); calls
 *    only enqueue work, they never synchronise the device;
 *  - return value: CVMHIP_OK, or an error code.  Codes 10..19 are argument /
 *    logic errors (map to VERIFY -> std::logic_error -> ERROR_LOGIC), codes
 *    >= 20 are runtime failures (map to CHECK -> ERROR_RUNTIME), the same
 *    split the reference uses in src/runtime/cuda/ops/ops_cuda.cc:33-43.
 *    cvmhip_last_error() returns a message for the calling thread.
 *  - results are bit-identical to the reference CPU operators
 *    (src/runtime/cpu/ops) on the same inputs, including int32 wrap-around.
 */
#ifndef CVM_HIP_OPS_H_
#define CVM_HIP_OPS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif
#pragma GCC visibility push(default)

#define CVMHIP_OK 0
#define CVMHIP_ERR_ARG 10
#define CVMHIP_ERR_RUNTIME 20

enum { CVMHIP_ADD = 0, CVMHIP_SUB = 1, CVMHIP_MUL = 2, CVMHIP_MAX = 3, CVMHIP_DIV = 4, CVMHIP_GREATER = 5 };
enum { CVMHIP_SUM = 0, CVMHIP_RMAX = 1 };

const char* cvmhip_last_error(void);

/* ---- conv2d: replaces cuda_conv2d / cuda_depthwise_conv2d / cuda_groupwise_conv2d
 * (cuda_ops.h:113-142, conv.cu:394-700); semantics of cvm.runtime.cpu.conv2d
 * (src/runtime/cpu/ops/ops.cc:368-456).  NCHW data, OIHW filter, bias[oc] or NULL.
 * groups == 1: data and filter are narrowed to int8 (ops.cc:234,431) and the
 * product runs on i8 MFMA as an implicit GEMM; groups > 1: exact int32 direct
 * convolution, no narrowing (ops.cc:333-366).
 * `workspace` is device scratch of at least cvmhip_conv2d_workspace_bytes()
 * bytes -- the role args.ext_space plays for the CUDA backend
 * (src/top/nn/convolution.cc:237-272). */
size_t cvmhip_conv2d_workspace_bytes(int n, int ic, int h, int w, int oc, int kh, int kw, int groups);
int cvmhip_conv2d(const int32_t* x, const int32_t* w, const int32_t* bias, int32_t* y,
                  int n, int ic, int h, int wd, int oc, int kh, int kw,
                  int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w,
                  int groups, void* workspace, size_t workspace_bytes, void* stream);

/* ---- dense: replaces cuda_dense (cuda_ops.h:149, cuda_ops.cu:9-66); semantics of
 * cvm.runtime.cpu.dense (ops.cc:34-75): y[m][n] = sum_k x[m][k]*w[n][k] (+ bias[n]).
 * operand_bits <= 8 promises |x|,|w| <= 127 (what DenseInferPrecision,
 * src/top/nn/nn.cc:22-44, guarantees inside a verified graph) and selects the
 * i8 MFMA path; larger values select the exact int32 path. */
size_t cvmhip_dense_workspace_bytes(int m, int k, int n);
int cvmhip_dense(const int32_t* x, const int32_t* w, const int32_t* bias, int32_t* y,
                 int m, int k, int n, int operand_bits,
                 void* workspace, size_t workspace_bytes, void* stream);

/* ---- unary elementwise (y may alias x): cuda_relu / cuda_cvm_clip /
 * cuda_cvm_right_shift / cuda_cvm_left_shift / cuda_clip / cuda_abs /
 * cuda_negative / cuda_log (cuda_ops.h:154-211); CPU semantics in
 * src/runtime/cpu/ops/ops.cc:12-26,525-553,632-642 and elemwise.cc:47-193. */
int cvmhip_relu(const int32_t* x, int32_t* y, int64_t size, void* stream);
int cvmhip_cvm_clip(const int32_t* x, int32_t* y, int64_t size, int precision, void* stream);
int cvmhip_cvm_right_shift(const int32_t* x, int32_t* y, int64_t size, int precision, int shift_bit, void* stream);
int cvmhip_cvm_left_shift(const int32_t* x, int32_t* y, int64_t size, int precision, int shift_bit, void* stream);
int cvmhip_clip(const int32_t* x, int32_t* y, int64_t size, int32_t a_min, int32_t a_max, void* stream);
int cvmhip_abs(const int32_t* x, int32_t* y, int64_t size, void* stream);
int cvmhip_negative(const int32_t* x, int32_t* y, int64_t size, void* stream);
int cvmhip_cvm_precision(const int32_t* x, int32_t* y, int64_t size, void* stream);

/* ---- elemwise_add / elemwise_sub (c may alias a or b): cuda_elemwise_add/sub
 * (cuda_ops.h:111-112); CPU elemwise.cc:8-45.  op is CVMHIP_ADD or CVMHIP_SUB. */
int cvmhip_elemwise(int op, const int32_t* a, const int32_t* b, int32_t* c, int64_t size, void* stream);

/* ---- broadcast_{add,sub,mul,max,div,greater}: cuda_broadcast_* (cuda_ops.h:157-188);
 * CPU broadcast.cc:6-125 (right-aligned numpy broadcasting, div by 0 -> 0). */
int cvmhip_broadcast(int op, const int32_t* a, const int64_t* ashape, int andim,
                     const int32_t* b, const int64_t* bshape, int bndim,
                     int32_t* c, const int64_t* cshape, int cndim, void* stream);

/* ---- max_pool2d: cuda_max_pool (cuda_ops.h:143, conv.cu:704-760); CPU ops.cc:466-523
 * (padding counts as INT32_MIN; output extent given by the caller). */
int cvmhip_max_pool2d(const int32_t* x, int32_t* y, int n, int c, int h, int w,
                      int oh, int ow, int kh, int kw, int stride_h, int stride_w,
                      int pad_h, int pad_w, void* stream);

/* ---- sum / max over an axis set: cuda_sum / cuda_max (cuda_ops.h:189-201);
 * CPU reduce.cc:6-140.  `axes` as written in the attribute (negatives allowed). */
int cvmhip_reduce(int op, const int32_t* x, const int64_t* xshape, int ndim,
                  int32_t* y, int64_t ysize, const int64_t* axes, int naxes, int exclude,
                  void* stream);

/* ---- index-remap copies: cuda_concatenate, cuda_transpose, cuda_stride_slice,
 * cuda_slice_like, cuda_take, cuda_repeat, cuda_tile, cuda_upsampling_nearest,
 * cuda_where, cuda_flatten/reshape/expand_dims/squeeze (cuda_ops.h:156-235);
 * CPU ops.cc:567-989,1049-1075 and elemwise.cc:64-86. */
int cvmhip_copy(const int32_t* x, int32_t* y, int64_t size, void* stream); /* flatten/reshape/expand_dims/squeeze */
/* inputs[m] == NULL skips that input: its slice of y is taken to be in place already */
int cvmhip_concatenate(const int32_t* const* inputs, const int64_t* const* ishapes, int ninputs,
                       int ndim, int axis, int32_t* y, const int64_t* yshape, void* stream);
int cvmhip_transpose(const int32_t* x, const int64_t* xshape, int ndim,
                     const int64_t* axes, int naxes, int32_t* y, void* stream);
int cvmhip_strided_slice(const int32_t* x, const int64_t* xshape, int ndim,
                         const int64_t* begin, int nbegin, const int64_t* stride, int nstride,
                         int32_t* y, const int64_t* yshape, void* stream);
int cvmhip_slice_like(const int32_t* x, const int64_t* xshape, int ndim,
                      int32_t* y, const int64_t* yshape, void* stream);
int cvmhip_take(const int32_t* x, const int64_t* xshape, int xndim,
                const int32_t* indices, const int64_t* ishape, int indim,
                int32_t* y, const int64_t* yshape, int yndim, int has_axis, int axis, void* stream);
int cvmhip_repeat(const int32_t* x, const int64_t* xshape, int32_t* y, const int64_t* yshape,
                  int ndim, int axis, int repeats, void* stream);
int cvmhip_tile(const int32_t* x, const int64_t* xshape, int xndim,
                int32_t* y, const int64_t* yshape, int yndim, void* stream);
int cvmhip_upsampling(const int32_t* x, int32_t* y, int n, int c, int h, int w, int scale, void* stream);
int cvmhip_where(const int32_t* cond, const int32_t* x, const int32_t* y, int32_t* out,
                 const int64_t* oshape, int ndim, int same_shape, void* stream);

/* ---- get_valid_counts: cuda_get_valid_counts (cuda_ops.h:225, nms.cu:11-127);
 * CPU nms.cc:42-63.  Rows with row[1] > score_threshold are compacted in their
 * original order, the rest of y is -1, valid_count[b] is the count.
 * `workspace`: cvmhip_get_valid_counts_workspace_bytes() bytes of device scratch. */
size_t cvmhip_get_valid_counts_workspace_bytes(int batches, int n);
int cvmhip_get_valid_counts(const int32_t* x, int32_t* valid_count, int32_t* y,
                            int batches, int n, int k, int32_t score_threshold,
                            void* workspace, size_t workspace_bytes, void* stream);

/* ---- non_max_suppression: cuda_non_max_suppression (cuda_ops.h:228, nms.cu:310-430);
 * semantics of the CPU operator (nms.cc:65-140), including its early exit on a
 * batch with no valid rows, its stop at the first negative id and its in-place
 * overwrite of x rows past top_k (x is therefore written, and must not alias y).
 * No host synchronisation: valid_count is read on the device.
 * `workspace`: cvmhip_nms_workspace_bytes() bytes of scratch. */
size_t cvmhip_nms_workspace_bytes(int batches, int n, int k);
int cvmhip_non_max_suppression(int32_t* x, const int32_t* valid_count, int32_t* y,
                               int batches, int n, int k, int max_output_size,
                               int iou_threshold, int topk, int coord_start,
                               int score_index, int id_index, int force_suppress,
                               void* workspace, size_t workspace_bytes, void* stream);
/* The same operator for callers that cannot allocate device memory or bring a workspace (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The scratch is
 * a fixed array inside the library's code object, cvmhip_nms_static_capacity_bytes() bytes (2 MiB) per GPU,
 * held until the process ends; a call whose cvmhip_nms_workspace_bytes(batches, n, k) exceeds it returns
 * CVMHIP_ERR_ARG.  The call allocates and frees nothing.  All calls on one GPU share the array: calls that
 * overlap in time on one GPU (two streams, two threads) race and must be serialised by the caller.  The
 * first call on a device looks the array's address up (hipGetSymbolAddress); make it outside stream capture. */
size_t cvmhip_nms_static_capacity_bytes(void);
int cvmhip_non_max_suppression_static(int32_t* x, const int32_t* valid_count, int32_t* y,
                                      int batches, int n, int k, int max_output_size,
                                      int iou_threshold, int topk, int coord_start,
                                      int score_index, int id_index, int force_suppress, void* stream);

/* ---- device memory and streams: what a DeviceAPI subclass registered as
 * "device_api.hip" needs (include/cvm/runtime/device_api.h:43-108: SetDevice,
 * AllocDataSpace, FreeDataSpace, CopyDataFromTo, StreamSync).  Allocations are
 * aligned to at least 256 bytes. */
int cvmhip_device_count(int* count);
int cvmhip_set_device(int device_id);
int cvmhip_alloc(void** ptr, size_t bytes);
int cvmhip_free(void* ptr);
int cvmhip_memset32(void* ptr, int32_t value, size_t count, void* stream);
int cvmhip_host_alloc(void** ptr, size_t bytes);   /* pinned host memory for staging copies */
int cvmhip_host_free(void* ptr);
/* int8 bytes already on the device -> the int32 `data` tensor, clamped to [-range, range]: the input
 * path of CvmRuntime::SetInput (src/runtime/graph_runtime.cc:317-397) without widening on the host */
int cvmhip_widen_clamp_i8(const void* src, int32_t* dst, int64_t count, int32_t range, void* stream);
int cvmhip_copy_h2d(void* dst, const void* src, size_t bytes, void* stream);
int cvmhip_copy_d2h(void* dst, const void* src, size_t bytes, void* stream);
int cvmhip_copy_d2d(void* dst, const void* src, size_t bytes, void* stream);
/* device-to-device copy done by a compute kernel (16-byte granules) instead of the copy engine: a launch of
 * exactly known HBM traffic, 2*bytes, against which hardware traffic counters can be scaled */
int cvmhip_copy_kernel(void* dst, const void* src, size_t bytes, void* stream);
int cvmhip_stream_create(void** stream);
int cvmhip_stream_destroy(void* stream);
int cvmhip_stream_sync(void* stream);
/* elapsed-time probes for the per-operator time table (the reference's -DPROFILE
 * table, src/runtime/graph_runtime.cc:62-87, measured with device events) */
int cvmhip_event_create(void** event);
int cvmhip_event_destroy(void* event);
int cvmhip_event_record(void* event, void* stream);
int cvmhip_event_elapsed_ms(void* start, void* stop, float* ms);
int cvmhip_device_sync(void);                               /* every stream of the current device */
int cvmhip_stream_wait_event(void* stream, void* event);   /* work issued to `stream` later waits for `event` */
/* Per-kernel device time for a measurement harness: between begin and end the
 * implicit-GEMM and packing launches are bracketed by event pairs on their own
 * stream; end synchronises and writes {"kernel": {"launches", "ms", "work"}}
 * where work is the algorithmic operation (or byte) count of the launches. */
int cvmhip_kernel_timing_begin(void);
int cvmhip_kernel_timing_end(char* json_out, int capacity);
/* The same end call, but the text is a list with one entry per bracketed launch, in launch order:
 * [{"kernel", "desc" (layer shape and kernel configuration), "work", "bytes" (algorithmic HBM bytes), "ms"}] */
int cvmhip_kernel_timing_end_launches(char* json_out, int capacity);
int cvmhip_kernel_timing_active(void);   /* 1 between begin and end */

/* ---- stream capture: the launches issued on `stream` between begin and end
 * become one executable graph that replays them with a single submission
 * (hipStreamBeginCapture / hipGraphInstantiate / hipGraphLaunch).
 * No counterpart in the reference: its GPU runtime launches node by node. */
int cvmhip_capture_begin(void* stream);
int cvmhip_capture_end(void* stream, void** graph_exec);
int cvmhip_graph_launch(void* graph_exec, void* stream);
int cvmhip_graph_destroy(void* graph_exec);

/* ---- conv2d / dense with the filter packed once at model-load time.  The
 * filter of a graph node is a constant parameter, so the int32 OIHW -> int8
 * MFMA-row layout conversion that cuda_conv2d redoes on every call
 * (conv.cu:430-438) is hoisted out of the inference path.
 * `wp` is cvmhip_packed_weight_bytes() bytes; `workspace` holds the packed
 * activations, cvmhip_packed_act_bytes(n*h*w, ic) bytes. */
size_t cvmhip_packed_weight_bytes(int oc, int ic, int kh, int kw);
size_t cvmhip_packed_act_bytes(int64_t npix, int channels);
int cvmhip_pack_weights(const int32_t* w, void* wp, int oc, int ic, int kh, int kw, void* stream);
int cvmhip_conv2d_packed(const int32_t* x, const void* wp, const int32_t* bias, int32_t* y,
                         int n, int ic, int h, int wd, int oc, int kh, int kw,
                         int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w,
                         void* workspace, size_t workspace_bytes, void* stream);

/* ---- fused int8 path.  No counterpart in the reference: it runs every node as
 * its own int32 kernel.  Inside a verified graph every conv2d/dense operand is
 * proven to fit 8 bits (src/top/nn/convolution.cc:153-158, src/top/nn/nn.cc:26-31),
 * so the graph executor keeps such activations as int8 between layers and folds
 * the requantisation chain that follows a producer -- any sequence of relu /
 * cvm_right_shift / cvm_clip / clip -- into the producer's epilogue.  Results
 * are bit-identical to running the nodes one by one.
 * int8 activation layout ("act" below): channels padded to cp =
 * cvmhip_pad_channels(c) = 4, 8, 16 or a multiple of 32.  cp <= 16: NHWC.
 * Otherwise blocks of 32 consecutive pixels (linear index over n, h, w) x 32
 * channels, each stored as the 1 KiB operand fragment of v_mfma_i32_32x32x32_i8:
 *   offset(p, c) = ((p/32)*(cp/32) + c/32)*1024 + ((c/16)%2)*512 + (p%32)*16 + c%16
 * A buffer for npix pixels has cvmhip_packed_act_bytes(npix, c) bytes, 16-byte aligned. */
enum { CVMHIP_STAGE_RELU = 1, CVMHIP_STAGE_RSHIFT = 2, CVMHIP_STAGE_CLIP = 3, CVMHIP_STAGE_MUL = 4, CVMHIP_STAGE_CLAMP_SHIFT = 5 };
typedef struct {
  int32_t kind;        /* CVMHIP_STAGE_* */
  int32_t precision;   /* RSHIFT */
  int32_t shift_bit;   /* RSHIFT */
  int32_t lo, hi;      /* CLIP: max(min(v, hi), lo).  MUL: v * lo, wrapping (broadcast_mul by a constant scalar,
                          the requantisation scale in front of a cvm_right_shift; broadcast.cc:75-86).
                          CLAMP_SHIFT: min(max(v, lo), hi) >> shift_bit (arithmetic, 0..31, no rounding term): what is
                          left of a cvm_right_shift whose rounding term the caller has added to the value beforehand,
                          see cvmhip_fold_requant */
} cvmhip_stage;
typedef struct {
  int32_t count;       /* 0..4 stages, applied in order to the int32 value */
  cvmhip_stage stage[4];
} cvmhip_chain;

/* Host-side, no device needed.  cvmhip_chain_apply_host evaluates a chain on n int32 values exactly as the kernels do
 * (the form the library prepares from the stages, with adjacent clamps merged).
 * cvmhip_fold_requant rewrites the epilogue of a convolution  v = chain(acc + bias[oc]); if (residual) v = chain2(v + r)
 * into an equivalent one with fewer instructions per value: the rounding terms of the cvm_right_shift stages are
 * added to the bias (oc values, host memory; NULL = zeros) once per channel, and what remains of the stages are
 * CVMHIP_STAGE_CLAMP_SHIFT stages.  max_abs_acc bounds |acc| (e.g. taps * channels * 128 * 128 for int8 operands);
 * the rewrite is only made when acc + bias + rounding terms provably never wraps.  Returns 1 and fills bias_out
 * (oc values), chain_out, chain2_out, or returns 0 and leaves them alone (chain shapes it does not handle, or no proof). */
int cvmhip_chain_apply_host(const cvmhip_chain* chain, const int32_t* in, int64_t n, int32_t* out);
int cvmhip_fold_requant(const int32_t* bias, int oc, int64_t max_abs_acc, const cvmhip_chain* chain,
                        const cvmhip_chain* chain2, int has_residual, int32_t* bias_out, cvmhip_chain* chain_out,
                        cvmhip_chain* chain2_out);
int cvmhip_pad_channels(int channels);
/* Test and tuning hook: forces, for the calling thread's later convolution launches, the implicit-GEMM kernel
 * (0 automatic, 1 LDS-tiled, 2 wavefront-private, 3 large-tile wherever the layout allows it), a configuration of the
 * wavefront kernel (-1 automatic) and a tile of the tiled kernel (wm, wn in 1..2; 0 automatic; with kernel 3, wm = 1..3
 * picks the 256x256, 128x256 or 64x512 tile).  The library never reads the environment on a launch. */
int cvmhip_set_conv_tuning(int kernel, int wave_cfg, int tile_wm, int tile_wn);
/* The same for layer-sequence launches (cvmhip_conv_seq_*) of the calling thread: `spin_limit` = polls after which a wait
 * at a layer boundary gives up and raises the launch's error word (default 2 000 000; 0 makes every wait give up at
 * once, which is how the fall-back of a caller is tested without hanging a kernel). */
int cvmhip_set_seq_tuning(int spin_limit);
/* Measurement hook: later layer-sequence launches of the calling thread write time stamps (shader clock) into `stamps`,
 * device memory of 256 x layers x 8 64-bit words: per workgroup (XCD * 32 + rank among the XCD's workgroups)
 * and layer, words 0..7 = tile entered, boundary passed, first operands multiplied, K loop done, K-split exchange
 * done, epilogue issued, counted out, layer begun.  NULL switches them off (the default).  A launch captured into a
 * graph keeps the pointer it was captured with.  Only a library built with -DCVM_SEQ_STAMPS has them (the stamps cost
 * the kernel waits even when unused); otherwise a non-NULL pointer is refused with CVMHIP_ERR_ARG. */
int cvmhip_set_seq_stamps(void* stamps, int layers);
/* Tuning hook: the configuration of the tile kernel for entry `index` (< 64) of the sequence tables that
 * cvmhip_conv_seq_layer fills next on this thread; -1 = automatic; index < 0 resets every entry. */
int cvmhip_set_seq_layer_config(int index, int config);
/* int32 NCHW <-> int8 act layout (narrowing is static_cast<int8_t>) */
int cvmhip_pack_nhwc_i8(const int32_t* x, void* xp, int n, int c, int hw, void* stream);
int cvmhip_unpack_nhwc_i8(const void* xp, int32_t* x, int n, int c, int hw, void* stream);
/* conv2d / dense on int8 act input with packed filter (cvmhip_pack_weights):
 *   v = chain(acc + bias);  if (residual) v = chain2(v + residual);
 * out is int8 act layout when out_is_i8, else int32 NCHW.  residual is an int8 act
 * tensor with the output's geometry, or NULL. */
int cvmhip_conv2d_i8(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                     const void* residual, const cvmhip_chain* chain2, void* out, int out_is_i8,
                     int n, int ic, int h, int wd, int oc, int kh, int kw,
                     int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream);
/* The same with a workspace.  A layer with at most 64 output pixels and K = kh*kw*ic >= 8192 (dense at a small
 * batch: ops.cc:34-75 computed as a convolution; VGG-16's 25088 -> 4096 layer) is all filter streaming, and
 * one workgroup per 32 output channels cannot keep HBM busy: with a workspace K is cut into up to 4 slices
 * computed by different workgroups (int32 partial sums, added in a fixed order by a second kernel, so the
 * result is the same wrap-around sum).  cvmhip_conv2d_i8_workspace_bytes returns the size needed (0: the
 * layer does not qualify, pass NULL); with workspace NULL the call equals cvmhip_conv2d_i8. */
size_t cvmhip_conv2d_i8_workspace_bytes(int has_residual, int n, int ic, int h, int wd, int oc, int kh, int kw,
                                        int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w);
int cvmhip_conv2d_i8_ws(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                        const void* residual, const cvmhip_chain* chain2, void* out, int out_is_i8,
                        int n, int ic, int h, int wd, int oc, int kh, int kw,
                        int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w,
                        void* workspace, size_t workspace_bytes, void* stream);
/* conv2d + chain followed by max_pool2d with a 2x2 window, stride 2 and no padding (ops.cc:466-523: the maximum of the
 * four values of a window, all of which exist when the convolution's output extent is even) in ONE launch: the
 * kernel numbers the convolution's output pixels window by window, takes the maximum of the four requantised
 * values across lanes and stores only that.  out is the int8 act tensor of the POOLED result (n, oc, OH/2, OW/2);
 * the full-resolution tensor is never written.  Eligible (..._eligible returns 1): input and output channels
 * padded to a multiple of 32 (ic, oc > 16), OH and OW even, filter side <= 32; otherwise the call fails with
 * CVMHIP_ERR_ARG and the caller runs cvmhip_conv2d_i8 and cvmhip_max_pool2d_i8. */
int cvmhip_conv2d_pool2_i8_eligible(int n, int ic, int h, int wd, int oc, int kh, int kw,
                                    int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w);
int cvmhip_conv2d_pool2_i8(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain, void* out,
                           int n, int ic, int h, int wd, int oc, int kh, int kw,
                           int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream);
/* A run of convolutions in ONE launch.  No counterpart in the reference.  The images are dealt to
 * cvmhip_conv_seq_shares() XCDs (8) when the batch is a multiple of it, else to the largest of 4, 2, 1 that divides
 * the batch (the other XCDs' workgroups leave at once).  Images are independent, so every XCD computes all layers
 * of the run for its own share of the images; a layer boundary is then a counter in that XCD's L2 instead of a
 * kernel boundary (no L2 write-back, the next layer's operands are still in the L2).  Use: fill a host table of
 * n * cvmhip_conv_seq_layer_bytes() bytes with cvmhip_conv_seq_layer (entry i describes what
 * cvmhip_conv2d_i8 with the same arguments and an int8 output would compute; it returns 10 when that layer
 * cannot be part of a run), copy the table to the device, and launch it.  Layer i may read what layers < i of
 * the run or earlier launches wrote.  `sync` is cvmhip_conv_seq_sync_bytes() of device memory, zeroed once,
 * 256-byte aligned; its last 256-byte block starts with an error word that is non-zero after a launch whose
 * bounded waits ran out (results invalid; the caller falls back to one launch per layer).  The launch needs
 * every compute unit: two of them must never be in flight at the same time on one device. */
size_t cvmhip_conv_seq_layer_bytes(void);
size_t cvmhip_conv_seq_sync_bytes(void);
int cvmhip_conv_seq_shares(void);
int cvmhip_conv_seq_layer(void* table, int index, const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                          const void* residual, const cvmhip_chain* chain2, void* out,
                          int n, int ic, int h, int wd, int oc, int kh, int kw,
                          int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w);
/* configuration of the tile kernel that cvmhip_conv_seq_layer chose for entry `index` of a host table (7: the entry
 * begins a chain, see cvmhip_conv_seq_link) */
int cvmhip_conv_seq_layer_config(const void* table, int index);
/* Optional, on a finished host table of `count` entries, before it is copied to the device.  A 1x1 convolution with
 * stride 1 and no padding (conv2d: ops.cc:368-456) needs, for a block of 32 pixels, only the same 32 pixels of its
 * input.  Where an entry with 64 output channels is followed by one or two such layers, each reading the one before it
 * (the 3x3 -> 1x1 (+ residual) -> 1x1 run of a ResNet bottleneck), the wavefront that holds the first layer's result
 * for a pixel block computes the followers there and then, from registers: one layer boundary instead of three, and
 * the intermediate tensors are written (other layers may read them) but never read back.  Linked only when no output
 * of the three lies over anything the run still reads (the first layer's input, the residual) and all channel
 * counts are multiples of 32; results are bit for bit those of the unlinked table.  The call also marks pairs of
 * consecutive layers that have nothing to do with one another (the second reads nothing the first writes and writes
 * nothing the first reads or writes: the first 1x1 layer and the shortcut projection of a ResNet block): no layer
 * boundary is kept between the two.  Returns the number of chains and pairs.
 * cvmhip_set_seq_chains(0) switches linking off for the calling thread (on by default); a forced tile configuration
 * (cvmhip_set_conv_tuning, cvmhip_set_seq_layer_config) leaves the layers concerned unlinked. */
int cvmhip_conv_seq_link(void* table, int count);
int cvmhip_set_seq_chains(int on);
/* entries chained behind entry `index` of a host table (0, 1 or 2), plus 16 when no boundary follows the entry */
int cvmhip_conv_seq_layer_chain(const void* table, int index);
/* ops, bytes: algorithmic operations and HBM bytes of the layers, only reported by the kernel-timing session */
int cvmhip_conv_seq_launch(const void* dev_table, int nlayers, void* sync, double ops, double bytes, void* stream);
/* The same convolution with its int32 result written pixel-major (NHWC): image n's OH*OW*OC values
 * are contiguous at out + n*image_stride (elements).  This is what conv2d -> transpose(0,2,3,1) ->
 * reshape -> concatenate produces for a detection head (transpose: ops.cc:743-789, concatenate:
 * ops.cc:567-602), written in one pass straight into the head's slice of the concatenated tensor. */
int cvmhip_conv2d_i8_nhwc(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                          int32_t* out, int64_t image_stride, int n, int ic, int h, int wd, int oc, int kh, int kw,
                          int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream);
/* Two such convolutions over the SAME input with the same filter size, strides, padding, dilation and chain (the
 * class and the box head of one feature map of a detector) in ONE launch: the filters are packed behind one another by
 * cvmhip_pack_weights_pair (the first one's rows padded to a multiple of 32), `bias` has
 * ceil32(oc_a) + oc_b entries (the first head's, zeros up to the multiple of 32, the second head's) or is NULL, and
 * every workgroup writes the rows of the head its channels belong to.  Same values as two cvmhip_conv2d_i8_nhwc calls. */
size_t cvmhip_packed_weight_pair_bytes(int oc_a, int oc_b, int ic, int kh, int kw);
int cvmhip_pack_weights_pair(const int32_t* w_a, int oc_a, const int32_t* w_b, int oc_b, void* wp, int ic, int kh, int kw, void* stream);
int cvmhip_conv2d_i8_nhwc_pair(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                               int32_t* out_a, int64_t image_stride_a, int oc_a, int32_t* out_b, int64_t image_stride_b, int oc_b,
                               int n, int ic, int h, int wd, int kh, int kw,
                               int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream);
/* Detection heads of different feature maps do not depend on one another and are a handful of workgroups each: they can
 * share ONE launch.  No counterpart in the reference.  Use: fill a host table of n * cvmhip_conv_group_layer_bytes()
 * bytes with cvmhip_conv_group_heads (entry i describes what cvmhip_conv2d_i8_nhwc -- out_b NULL -- or
 * cvmhip_conv2d_i8_nhwc_pair with the same arguments would compute; first_block is the sum of the *blocks of the entries
 * before it; status 10 when the layer cannot be an entry: input channels not padded to 32), copy the table to the device
 * and call cvmhip_conv_group_launch with the number of entries and the sum of all *blocks.  The entries must not read what
 * another entry of the same launch writes. */
size_t cvmhip_conv_group_layer_bytes(void);
int cvmhip_conv_group_heads(void* table, int index, int first_block, int* blocks, const void* xp, const void* wp, const int32_t* bias,
                            const cvmhip_chain* chain, int32_t* out_a, int64_t image_stride_a, int oc_a, int32_t* out_b,
                            int64_t image_stride_b, int oc_b, int n, int ic, int h, int wd, int kh, int kw,
                            int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w);
/* ops, bytes: algorithmic operations and HBM bytes of the layers, only reported by the kernel-timing session */
int cvmhip_conv_group_launch(const void* dev_table, int nlayers, int total_blocks, double ops, double bytes, void* stream);
/* The same for convolutions with int8 output that do not depend on one another (at a small batch the first 1x1 layer and
 * the shortcut projection of a ResNet block are 50-400 workgroups each): entry i describes what cvmhip_conv2d_i8 with the
 * same arguments and an int8 output would compute; a table holds either int32 entries or int8 entries, launched by
 * cvmhip_conv_group_launch or cvmhip_conv_group_launch_i8. */
int cvmhip_conv_group_conv_i8(void* table, int index, int first_block, int* blocks, const void* xp, const void* wp, const int32_t* bias,
                              const cvmhip_chain* chain, const void* residual, const cvmhip_chain* chain2, void* out,
                              int n, int ic, int h, int wd, int oc, int kh, int kw,
                              int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w);
int cvmhip_conv_group_launch_i8(const void* dev_table, int nlayers, int total_blocks, double ops, double bytes, void* stream);
/* conv2d over at most 4 input channels with kw <= 8, dilation 1 (the RGB stem of a network), in
 * row-window form: the input is packed once per inference into int8 [n][hp][wp][4], zero padded, so
 * that the kw taps x 4 channel bytes of a filter row are one contiguous window and no tap lies
 * outside the stored tensor; K is ordered (kh, window byte).  Same arithmetic as cvmhip_conv2d_i8. */
int cvmhip_stem_eligible(int c, int kh, int kw, int dil_h, int dil_w);
size_t cvmhip_stem_input_bytes(int n, int h, int w, int kh, int kw, int stride_h, int stride_w, int pad_h, int pad_w);
int cvmhip_pack_stem_input(const int32_t* x, void* xs, int n, int c, int h, int w, int kh, int kw,
                           int stride_h, int stride_w, int pad_h, int pad_w, void* stream);
size_t cvmhip_packed_stem_weight_bytes(int oc, int kh, int kw);
int cvmhip_pack_stem_weights(const int32_t* w, void* wp, int oc, int c, int kh, int kw, void* stream);
int cvmhip_conv2d_stem_i8(const void* xs, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                          void* out, int out_is_i8, int n, int c, int h, int wd, int oc, int kh, int kw,
                          int stride_h, int stride_w, int pad_h, int pad_w, void* stream);
/* The same convolution followed by max_pool2d with a 3x3 window, stride 2 and padding 1 (ops.cc:466-523; the head of a
 * ResNet) in ONE launch: a workgroup computes the convolution pixels under a patch of 4 x 8 pooled pixels into LDS
 * (requantised to int8; pixels outside the convolution's output count as the smallest value, like the reference's
 * INT32_MIN padding) and takes the maxima there.  out: the pooled int8 act tensor (n, oc, pool_oh, pool_ow), with
 * pool_oh, pool_ow as the graph's shape inference gives them.  Eligible: the convolution is (cvmhip_stem_eligible),
 * oc is 32 or 64, and every window touches the convolution's output. */
int cvmhip_conv2d_stem_pool3_i8_eligible(int n, int c, int h, int wd, int oc, int kh, int kw, int stride_h, int stride_w,
                                         int pad_h, int pad_w, int pool_oh, int pool_ow);
int cvmhip_conv2d_stem_pool3_i8(const void* xs, const void* wp, const int32_t* bias, const cvmhip_chain* chain, void* out,
                                int n, int c, int h, int wd, int oc, int kh, int kw, int stride_h, int stride_w,
                                int pad_h, int pad_w, int pool_oh, int pool_ow, void* stream);
/* depthwise conv2d (groups == channels == out channels) on int8 act tensors, filter packed by
 * cvmhip_pack_depthwise_weights into [kh*kw][cp] int8 */
size_t cvmhip_packed_depthwise_bytes(int c, int kh, int kw);
int cvmhip_pack_depthwise_weights(const int32_t* w, void* wp, int c, int kh, int kw, void* stream);
int cvmhip_depthwise_conv2d_i8(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                               void* out, int out_is_i8, int n, int c, int h, int wd, int kh, int kw,
                               int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream);
/* The same depthwise convolution on the matrix cores, for channel counts padded to a multiple of 32 and
 * filter sides up to 32: a tile of 32 output channels is a convolution over its own 32 input channels
 * whose filter matrix is diagonal for every tap (groupwise_conv2d with groups == channels:
 * ops.cc:333-366), so it runs in the implicit-GEMM kernel of cvmhip_conv2d_i8 with K = taps * 32.  The
 * filter is packed by cvmhip_pack_depthwise_weights_mfma into cvmhip_packed_depthwise_mfma_bytes bytes.
 * Operands must be known to fit int8 (this path, like cvmhip_depthwise_conv2d_i8, does not narrow). */
int cvmhip_depthwise_mfma_eligible(int c, int kh, int kw);
size_t cvmhip_packed_depthwise_mfma_bytes(int c, int kh, int kw);
int cvmhip_pack_depthwise_weights_mfma(const int32_t* w, void* wp, int c, int kh, int kw, void* stream);
int cvmhip_depthwise_conv2d_mfma_i8(const void* xp, const void* wp, const int32_t* bias, const cvmhip_chain* chain,
                                    void* out, int out_is_i8, int n, int c, int h, int wd, int kh, int kw,
                                    int stride_h, int stride_w, int pad_h, int pad_w, int dil_h, int dil_w, void* stream);
/* flatten (elemwise.cc:64-76: a copy, the rows of an image one behind the other) of an int8 act tensor of n images,
 * hw pixels each, c channels (a multiple of 32), in the order a dense layer computed as a convolution over the whole
 * map takes its K axis: yp is the act tensor of n pixels (one per image) x hw * c channels, channel p * c + ch = channel
 * ch of pixel p (cvmhip_packed_act_bytes(n, hw * c) bytes, rows n .. 31 of its pixel block untouched).  With it that
 * dense layer is a 1x1 convolution over hw * c channels whose operand blocks are contiguous KiB: cvmhip_conv2d_i8_ws
 * with the filter packed for (ic = c, kh x kw = the map) and the geometry (ic = hw * c, 1 x 1 map, 1 x 1 filter) --
 * the packed filter is byte for byte the same for both readings. */
int cvmhip_flatten_act_i8(const void* xp, void* yp, int n, int c, int hw, void* stream);
/* out = chain(a + b) on int8 act tensors of identical geometry */
int cvmhip_add_i8(const void* a, const void* b, const cvmhip_chain* chain, void* out, int out_is_i8,
                  int n, int c, int hw, void* stream);
/* max_pool2d on int8 act tensors (padding counts as the smallest value, as INT32_MIN does) */
int cvmhip_max_pool2d_i8(const void* xp, void* yp, int n, int c, int h, int w, int oh, int ow,
                         int kh, int kw, int stride_h, int stride_w, int pad_h, int pad_w, void* stream);
/* out[n][c] = chain(sum over h,w of x[n][h][w][c]); out int8 act tensor of n pixels, or int32 [n][c] */
int cvmhip_sum_hw_i8(const void* xp, const cvmhip_chain* chain, void* out, int out_is_i8,
                     int n, int c, int hw, void* stream);

#pragma GCC visibility pop
#ifdef __cplusplus
}
#endif
#endif /* CVM_HIP_OPS_H_ */
