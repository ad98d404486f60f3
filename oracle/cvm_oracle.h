/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the reference CVM CPU
 * operators (src/runtime/cpu/ops/{ops,elemwise,broadcast,reduce,nms}.cc) in
 * plain C.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg may load this library; the product never links or calls it.
 *
 * Every tensor is contiguous row-major int32.  Shapes are passed as int64
 * arrays of length ndim (ndim <= 6).  All functions return 0 on success, a
 * positive code on rejected arguments.
 *
 * Pinned by tests/test_oracle.py: against the compiled reference (oracle/_ref) where it is built, against the
 * golden outputs it wrote (tests/golden/), and against closed forms / brute force.
 */
#ifndef CVM_ORACLE_H_
#define CVM_ORACLE_H_
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum { CVMO_ADD = 0, CVMO_SUB = 1, CVMO_MUL = 2, CVMO_MAX = 3, CVMO_DIV = 4, CVMO_GREATER = 5 };
enum { CVMO_SUM = 0, CVMO_RMAX = 1 };

/* ops.cc:368-456 (conv2d), :204-246 (im2col), :148-200 (matrix_mul), :333-366 (groupwise) */
int cvmo_conv2d(const int32_t* x, const int32_t* w, const int32_t* bias, int32_t* y,
                int n, int ic, int h, int wd, int oc, int kh, int kw,
                int stride_h, int stride_w, int pad_h, int pad_w,
                int dil_h, int dil_w, int groups);
/* ops.cc:34-75 */
int cvmo_dense(const int32_t* x, const int32_t* w, const int32_t* bias, int32_t* y,
               int m, int k, int n);
/* ops.cc:12-26 */
int cvmo_relu(const int32_t* x, int32_t* y, int64_t size);
/* elemwise.cc:88-112 */
int cvmo_cvm_clip(const int32_t* x, int32_t* y, int64_t size, int precision);
/* elemwise.cc:114-173 */
int cvmo_cvm_right_shift(const int32_t* x, int32_t* y, int64_t size, int precision, int shift_bit);
/* elemwise.cc:175-193 */
int cvmo_cvm_left_shift(const int32_t* x, int32_t* y, int64_t size, int precision, int shift_bit);
/* elemwise.cc:47-62 */
int cvmo_clip(const int32_t* x, int32_t* y, int64_t size, int32_t a_min, int32_t a_max);
/* elemwise.cc:8-45; op is CVMO_ADD or CVMO_SUB */
int cvmo_elemwise(int op, const int32_t* a, const int32_t* b, int32_t* c, int64_t size);
/* ops.cc:525-553, :632-642 */
int cvmo_abs(const int32_t* x, int32_t* y, int64_t size);
int cvmo_negative(const int32_t* x, int32_t* y, int64_t size);
int cvmo_cvm_precision(const int32_t* x, int32_t* y, int64_t size);
/* broadcast.cc:6-125 */
int cvmo_broadcast(int op, const int32_t* a, const int64_t* ashape, int andim,
                   const int32_t* b, const int64_t* bshape, int bndim,
                   int32_t* c, const int64_t* cshape, int cndim);
/* ops.cc:466-523 */
int cvmo_max_pool2d(const int32_t* x, int32_t* y, int n, int c, int h, int w,
                    int oh, int ow, int kh, int kw, int stride_h, int stride_w,
                    int pad_h, int pad_w);
/* reduce.cc:6-140; axes are the attribute's axes (may be negative), exclude as in ReduceParam */
int cvmo_reduce(int op, const int32_t* x, const int64_t* xshape, int ndim,
                int32_t* y, int64_t ysize, const int64_t* axes, int naxes, int exclude);
/* ops.cc:567-602 */
int cvmo_concatenate(const int32_t* const* inputs, const int64_t* const* ishapes, int ninputs,
                     int ndim, int axis, int32_t* y, const int64_t* yshape);
/* ops.cc:743-789; naxes == 0 reverses dims */
int cvmo_transpose(const int32_t* x, const int64_t* xshape, int ndim,
                   const int64_t* axes, int naxes, int32_t* y);
/* ops.cc:791-841 */
int cvmo_strided_slice(const int32_t* x, const int64_t* xshape, int ndim,
                       const int64_t* begin, int nbegin, const int64_t* stride, int nstride,
                       int32_t* y, const int64_t* yshape);
/* ops.cc:843-866 */
int cvmo_slice_like(const int32_t* x, const int64_t* xshape, int ndim,
                    int32_t* y, const int64_t* yshape);
/* ops.cc:868-956; has_axis == 0 is the flattened take (also cvm_lut) */
int cvmo_take(const int32_t* x, const int64_t* xshape, int xndim,
              const int32_t* indices, const int64_t* ishape, int indim,
              int32_t* y, const int64_t* yshape, int yndim, int has_axis, int axis);
/* ops.cc:604-630 */
int cvmo_repeat(const int32_t* x, const int64_t* xshape, int32_t* y, const int64_t* yshape,
                int ndim, int axis, int repeats);
/* ops.cc:644-681 */
int cvmo_tile(const int32_t* x, const int64_t* xshape, int xndim,
              int32_t* y, const int64_t* yshape, int yndim);
/* ops.cc:958-989 */
int cvmo_upsampling(const int32_t* x, int32_t* y, int n, int c, int h, int w, int scale);
/* ops.cc:1049-1075; same_shape != 0 when condition has x's ndim */
int cvmo_where(const int32_t* cond, const int32_t* x, const int32_t* y, int32_t* out,
               const int64_t* oshape, int ndim, int same_shape);
/* nms.cc:42-63 */
int cvmo_get_valid_counts(const int32_t* x, int32_t* valid_count, int32_t* y,
                          int batches, int n, int k, int32_t score_threshold);
/* nms.cc:4-40 */
int64_t cvmo_iou(const int32_t* rect1, const int32_t* rect2);
/* nms.cc:65-140; x is mutated exactly as the reference mutates it (rows past top_k set to -1) */
int cvmo_non_max_suppression(int32_t* x, const int32_t* valid_count, int32_t* y,
                             int batches, int n, int k, int max_output_size,
                             int iou_threshold, int topk, int coord_start,
                             int score_index, int id_index, int force_suppress);

#ifdef __cplusplus
}
#endif
#endif
