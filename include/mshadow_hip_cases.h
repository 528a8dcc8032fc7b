/*
 * libmshadow_cases - caller-style programs written against <mshadow/tensor.h>
 * (Tensor<gpu>, Stream<gpu>, expression templates), compiled by hipcc and exported as
 * C functions so that tests and the benchmark can drive the C++ expression API from
 * any language. They play the role of the reference's guide/ and test/ programs
 * (guide/neuralnet/convnet.cu:81-122 calls every one of these operations); each body
 * is the line of mshadow code quoted in its comment.
 *
 * All pointers are DEVICE pointers owned by the caller; pitches in elements; `stream`
 * is a handle from mshadow_hip_stream_create. `variant` 0 writes the expression on
 * plain tensors (the library recognises it and runs the tuned kernel); variant 1 wraps
 * the source in F<op::identity>() so that the same operation runs through the generic
 * expression kernel instead. Return value: 0, or non-zero with the text available from
 * mshadow_case_last_error() when a CHECK failed (DMLC_LOG_FATAL_THROW build).
 */
#ifndef MSHADOW_HIP_CASES_H_
#define MSHADOW_HIP_CASES_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *mshadow_case_last_error(void);

/* dst <saver>= A * B + 0.5f * F<sigmoid>(C) - D        (saver: 0 = 1 += 2 -= 3 *= 4 /=) */
int mshadow_case_map_fused_f32(float *dst, int dstride, const float *a, int astride,
                               const float *b, int bstride, const float *c, int cstride,
                               const float *d, int dstride_d, int rows, int cols, int saver,
                               void *stream);
/* dst <saver>= scalar */
int mshadow_case_map_scalar_f32(float *dst, int dstride, int rows, int cols, float scalar,
                                int saver, void *stream);
/* dst <saver>= (A + s1) / s2 + s3 */
int mshadow_case_map_axpb_f32(float *dst, int dstride, const float *a, int astride, int rows,
                              int cols, float s1, float s2, float s3, int saver, void *stream);

/* dst <saver>= scale * reduce_except_dim<1, Reducer>(src2d)   (sum_rows when Reducer = sum) */
int mshadow_case_reduce_keep_lowest_f32(float *dst, const float *src, int sstride, int rows,
                                        int cols, int reducer, int saver, float scale,
                                        int variant, void *stream);
/* dst <saver>= scale * reduce_except_dim<1, Reducer>(src4d)   (sumall_except_dim<1>) */
int mshadow_case_reduce_keep_highdim_f32(float *dst, const float *src, int sstride, int n, int c,
                                         int y, int x, int reducer, int saver, float scale,
                                         int variant, void *stream);

/* Softmax(dst, src) and SoftmaxGrad(dst, src, label) */
int mshadow_case_softmax_f32(float *dst, int dstride, const float *src, int sstride, int rows,
                             int cols, void *stream);
int mshadow_case_softmax_grad_f32(float *dst, int dstride, const float *src, int sstride,
                                  const float *label, int rows, int cols, void *stream);

/* The same four on half_t tensors, passed as their 16-bit patterns (scale too), and Softmax on
   double tensors: the element-type-generic paths of the header API */
int mshadow_case_reduce_keep_lowest_f16(uint16_t *dst, const uint16_t *src, int sstride, int rows,
                                        int cols, int reducer, int saver, uint16_t scale,
                                        int variant, void *stream);
int mshadow_case_reduce_keep_highdim_f16(uint16_t *dst, const uint16_t *src, int sstride, int n,
                                         int c, int y, int x, int reducer, int saver,
                                         uint16_t scale, int variant, void *stream);
int mshadow_case_softmax_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride,
                             int rows, int cols, void *stream);
int mshadow_case_softmax_grad_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride,
                                  const uint16_t *label, int rows, int cols, void *stream);
/* dst <saver>= a * b + c, and dst = pool<Reducer>(src, (ph, pw), ky, kx, sy, sx), on half_t tensors */
int mshadow_case_map_muladd_f16(uint16_t *dst, int dstride, const uint16_t *a, int astride,
                                const uint16_t *b, int bstride, const uint16_t *c, int cstride,
                                int rows, int cols, int saver, void *stream);
int mshadow_case_pool_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride, int planes,
                          int h, int w, int ph, int pw, int ky, int kx, int sy, int sx,
                          int reducer, void *stream);
/* dst = scale * reduce_except_dim<1, Reducer>(src) on double tensors: n == 0 takes src as y rows of
   x columns and keeps the columns (sum_rows), otherwise src is (n, c, y, x) and c is kept */
int mshadow_case_reduce_f64(double *dst, const double *src, int sstride, int n, int c, int y, int x,
                            int reducer, double scale, void *stream);
/* op 0: dst = a * b + c; op 1: dst = pad(crop(a, (rows - 2, cols - 2)), 1); dense rows x cols tensors of
   the element type named by the mshadow::TypeFlag code (float32 0, float64 1, float16 2, uint8 3,
   int32 4, int8 5, int64 6), dispatched with MSHADOW_TYPE_SWITCH */
int mshadow_case_map_any(int op, int type_flag, void *dst, const void *a, const void *b,
                         const void *c, int rows, int cols, void *stream);
int mshadow_case_softmax_f64(double *dst, int dstride, const double *src, int sstride, int rows,
                             int cols, void *stream);

/* SoftmaxGrad / SmoothSoftmaxGrad with and without ignore_label, on 2-D tensors (d0 == 0:
   rows x cols, label of `rows` floats) or 3-D tensors (d0, d1, d2; label (d0, d2) with
   pitch lstride); flags as MSHADOW_HIP_GRAD_* */
int mshadow_case_grad_family_f32(float *dst, int dstride, const float *src, int sstride,
                                 const float *label, int lstride, int d0, int rows_or_d1,
                                 int cols_or_d2, int flags, float ignore_label, float alpha,
                                 void *stream);
/* Softmax(dst, src) on 3-D tensors */
int mshadow_case_softmax3d_f32(float *dst, int dstride, const float *src, int sstride, int d0,
                               int d1, int d2, void *stream);
/* op 0: AddTakeGrad(dst, index, src); 1: AddTakeGradLargeBatch(dst, sorted, index, src);
   2: IndexFill(dst, index, src); int32 index vectors */
int mshadow_case_rows_by_index_f32(int op, float *dst, int dstride, int k_rows, const int *sorted,
                                   const int *index, int n_index, const float *src, int sstride,
                                   int src_rows, int cols, void *stream);
/* the gradient family (d0 == 0: 2-D), the 3-D Softmax and the row functions on tensors of
   another element type: type_flag 0 float, 1 double, 2 half_t (mshadow::TypeFlag codes);
   index_flag 0 float, 2 half_t, 4 int32, 6 int64. ignore_label is converted to the element
   type before the call, as a caller holding a DType would pass it. */
int mshadow_case_grad_family_any(int type_flag, void *dst, int dstride, const void *src, int sstride,
                                 const void *label, int lstride, int d0, int rows_or_d1,
                                 int cols_or_d2, int flags, double ignore_label, float alpha,
                                 void *stream);
int mshadow_case_softmax3d_any(int type_flag, void *dst, int dstride, const void *src, int sstride,
                               int d0, int d1, int d2, void *stream);
int mshadow_case_rows_by_index_any(int op, int type_flag, int index_flag, void *dst, int dstride,
                                   int k_rows, const void *sorted, const void *index, int n_index,
                                   const void *src, int sstride, int src_rows, int cols,
                                   void *stream);

/* broadcast<1> / repmat / reshape / swapaxis / mirror / upsampling_nearest /
   broadcast_scalar expressions over a dense (n, c, h, w) input `a` and a vector `v`
   (op 0..9, listed with the expression each evaluates in cases.hip) */
int mshadow_case_shaping_f32(int op, float *out, const float *a, const float *v, int n, int c,
                             int h, int w, void *stream);

/* Random<gpu>(seed): op 0 SampleUniform(p0, p1) into the two halves of out in turn; 1
   SampleGaussian(p0, p1); 2 out = uniform(Shape1(n)) * 2; 3 GetRandInt (unsigned words) */
int mshadow_case_random_f32(int op, int seed, float *out, int n, float p0, float p1, void *stream);
/* Random<gpu, double>(seed): ops 0-2 as above */
int mshadow_case_random_f64(int op, int seed, double *out, int n, double p0, double p1, void *stream);

/* op 0: SortByKey(keys, values, is_ascend); 1: VectorizedSort(keys, values as segment numbers).
   key_kind 0: float keys with int values, 1: int keys with float values (int segments for op 1) */
int mshadow_case_sort_by_key_32(int op, void *keys, int key_kind, void *values, int n,
                                int is_ascend, void *stream);
/* SortByKey for keys and values of any type of the type switch (mshadow::TypeFlag codes:
   0 float, 1 double, 2 half_t, 3 uint8, 4 int32, 5 int8, 6 int64) */
int mshadow_case_sort_by_key_any(int key_flag, int value_flag, void *keys, void *values, int n,
                                 int is_ascend, void *stream);

/* chpool / ch_unpool, reduce_with_axis / reduce_keepdim, broadcast_with_axis /
   broadcast_keepdim, transpose / transpose_indices, concat / slice / flip (also as the
   target of an assignment), take / take_grad / one_hot_encode / mat_choose_row_element /
   mat_fill_row_element / mask / range over a dense (n, ch, h, w) input `a`, operands `b`,
   `c` and parameters p0..p2 (op 0..27, listed with the expression each evaluates in
   cases.hip) */
int mshadow_case_extensions_f32(int op, float *out, const float *a, const float *b, const float *c,
                                int n, int ch, int h, int w, int p0, int p1, int p2,
                                void *stream);

/* dst <saver>= scale * dot(a[.T()], b[.T()]) for matrices and vectors, VectorDot, BatchGEMM and
   batch_dot over dense operands (op 0..16, listed with shapes in cases/dot_cases.inc) */
int mshadow_case_dot_f32(int op, float *out, const float *a, const float *b, int m, int k, int n,
                         int batch, void *stream);

/* out = x * x + x over a Tensor<gpu, 1, half2_t> of n_pairs elements (2 * n_pairs binary16 values) */
int mshadow_case_half2_map(uint16_t *out, const uint16_t *x, int n_pairs, void *stream);

/* a two-layer perceptron trained for `steps` full-batch updates on the device
   (cases/two_layer_net.h): x (batch, n_in), label (batch), w1 (n_in, n_hidden) and w2
   (n_hidden, n_out) in / out, probs (batch, n_out) out. Unlike the other cases every pointer
   is HOST memory: the program moves its data itself, and returns when the device is done */
int mshadow_case_two_layer_net_f32(int steps, float eta, float decay, int batch, int n_in,
                                   int n_hidden, int n_out, const float *x, const float *label,
                                   float *w1, float *w2, float *probs, void *stream);

/* dst = pool<Reducer>(src, Shape2(ph, pw), ky, kx, sy, sx) */
int mshadow_case_pool_f32(float *dst, int dstride, const float *src, int sstride, int planes,
                          int h, int w, int ph, int pw, int ky, int kx, int sy, int sx,
                          int reducer, int variant, void *stream);
/* dst = unpool<Reducer>(src, pooled, grad, ky, kx, sy, sx) */
int mshadow_case_unpool_f32(float *dst, int dstride, const float *src, int sstride,
                            const float *pooled, int pstride, const float *grad, int gstride,
                            int planes, int h, int w, int ph, int pw, int ky, int kx, int sy,
                            int sx, int reducer, int variant, void *stream);

/* col = unpack_patch2col(pad(img, pad_y, pad_x), ky, kx, sy, sx, dy, dx) */
int mshadow_case_im2col_f16(uint16_t *col, int cstride, const uint16_t *img, int istride, int n,
                            int c, int h, int w, int ky, int kx, int sy, int sx, int dy, int dx,
                            int pad_y, int pad_x, int variant, void *stream);
int mshadow_case_im2col_f32(float *col, int cstride, const float *img, int istride, int n, int c,
                            int h, int w, int ky, int kx, int sy, int sx, int dy, int dx,
                            int pad_y, int pad_x, int variant, void *stream);
/* img = crop(pack_col2patch(col, Shape4(n, c, h+2*pad_y, w+2*pad_x), ky, kx, sy, sx, dy, dx),
              Shape2(h, w), pad_y, pad_x) */
int mshadow_case_col2im_f16(uint16_t *img, int istride, const uint16_t *col, int cstride, int n,
                            int c, int h, int w, int ky, int kx, int sy, int sx, int dy, int dx,
                            int pad_y, int pad_x, int variant, void *stream);
int mshadow_case_col2im_f32(float *img, int istride, const float *col, int cstride, int n, int c,
                            int h, int w, int ky, int kx, int sy, int sx, int dy, int dx,
                            int pad_y, int pad_x, int variant, void *stream);

/* A convolutional network as one caller program (cases/conv_net.h; the network of the
   reference's guide/neuralnet/convnet.cu:81-122 with today's signatures): `steps` rounds of
   forward, backward and update on one batch, on one stream. geometry = {batch, in_channels,
   in_size, channels, ksize, kstride, pad, psize, num_out}. Every pointer is host memory:
   images (batch, in_channels, in_size, in_size), labels (batch, class numbers as floats),
   fixed_grad NULL or (batch, num_out) to enter the backward pass instead of probs -
   onehot(label), kernel (channels, in_channels * ksize^2) and weight (flat, num_out) in and
   out, keep NULL or an array of host pointers (NULL each) that receive the tensors of the
   last round in the order of conv_net::Kept. */
int mshadow_case_conv_net_f32(const int *geometry, int steps, float eta, float decay,
                              const float *images, const float *labels, const float *fixed_grad,
                              float *kernel, float *weight, float *const *keep, void *stream);
/* The convolution of that network and the gradient of its input alone, on float (half == 0)
   or binary16 tensors: image -> pad -> unpack_patch2col -> product -> swapaxis(reshape), and
   grad_out -> reshape(swapaxis) -> product -> pack_col2patch -> crop. Host memory. */
int mshadow_case_conv_pair(int half, const int *geometry, const void *image, const void *kernel,
                           const void *grad_out, void *col_forward, void *out, void *col_backward,
                           void *image_grad, void *stream);

/* Copy(Tensor<gpu,2,float> dst, Tensor<gpu,2,float> src, stream): device to device, either
   side possibly pitched */
int mshadow_case_copy_d2d_f32(float *dst, int dstride, const float *src, int sstride, int rows,
                              int cols, void *stream);

/* InitTensorEngine / NewStream / TensorContainer<gpu> / Copy (host -> device -> device ->
   host) / DeleteStream on host buffers of rows x cols floats; *device_stride receives the
   pitch AllocSpace chose with pad on or off. */
int mshadow_case_copy_roundtrip_f32(float *host_out, const float *host_in, int rows, int cols,
                                    int pad, int *device_stride);

#ifdef __cplusplus
}
#endif
#endif /* MSHADOW_HIP_CASES_H_ */
