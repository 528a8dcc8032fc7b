/*
 * TEST INFRASTRUCTURE - not part of the shipped library.
 *
 * Plain-C restatement of the CPU path of dmlc/mshadow for the nine hot-path
 * operations (elementwise map, two reduce-to-1D forms, softmax forward and
 * gradient, pool / unpool, patch2col / col2patch with pad / crop). Every
 * function follows the loop order and the rounding points of the reference
 * file:line it cites, so that results are bit-identical to the reference built
 * with -ffp-contract=off. Only tests, the smoke check and the benchmark's CPU
 * baseline may call into this file; the GPU library never does.
 *
 * All sizes and indices are 32-bit signed like the reference's index_t
 * (mshadow/base.h:288-292). Strides are row pitches in elements
 * (mshadow/tensor.h:419-423).
 */
#ifndef MSHADOW_ORACLE_H_
#define MSHADOW_ORACLE_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* savers, mshadow/base.h:539-602 */
enum { ORC_SAVETO = 0, ORC_PLUSTO = 1, ORC_MINUSTO = 2, ORC_MULTO = 3, ORC_DIVTO = 4 };
/* reducers, mshadow/base.h:604-862 */
enum { ORC_SUM = 0, ORC_MAX = 1, ORC_MIN = 2 };

/* number of OpenMP threads the loops below will use */
int orc_num_threads(void);

/* half <-> float, mshadow/half.h:197-242 (round to nearest even) and :285-330 */
uint16_t orc_float2half(float v);
float orc_half2float(uint16_t h);
void orc_float2half_n(uint16_t *dst, const float *src, int64_t n);
void orc_half2float_n(float *dst, const uint16_t *src, int64_t n);

/* dst <saver>= a*b + 0.5f*sigmoid(c) - d, sigmoid = pmath_sigmoid (caller functor) */
void orc_map_fused_f32(float *dst, int dstride, const float *a, int astride,
                       const float *b, int bstride, const float *c, int cstride,
                       const float *d, int dstride_d, int rows, int cols, int saver);
/* dst <saver>= scalar */
void orc_map_scalar_f32(float *dst, int dstride, int rows, int cols, float scalar, int saver);
/* dst <saver>= (a + s1) / s2 + s3   (guide/basic.cpp:25-30 shape of expression) */
void orc_map_axpb_f32(float *dst, int dstride, const float *a, int astride, int rows, int cols,
                      float s1, float s2, float s3, int saver);

void orc_reduce_keep_lowest_f32(float *dst, const float *src, int sstride, int rows, int cols,
                                int reducer, int saver, float scale);
void orc_reduce_keep_highdim_f32(float *dst, const float *src, int sstride, int n, int c, int y,
                                 int x, int reducer, int saver, float scale);

void orc_softmax_f32(float *dst, int dstride, const float *src, int sstride, int rows, int cols);
void orc_softmax_grad_f32(float *dst, int dstride, const float *src, int sstride,
                          const float *label, int rows, int cols);

/* The reductions and the softmax pair on half_t tensors (16-bit storage; every operation
   rounds to 16 bits, so accumulations round after each step). `scale` is a half_t too. */
void orc_reduce_keep_lowest_f16(uint16_t *dst, const uint16_t *src, int sstride, int rows,
                                int cols, int reducer, int saver, uint16_t scale);
void orc_reduce_keep_highdim_f16(uint16_t *dst, const uint16_t *src, int sstride, int n, int c,
                                 int y, int x, int reducer, int saver, uint16_t scale);
void orc_map_muladd_f16(uint16_t *dst, int dstride, const uint16_t *a, int astride,
                        const uint16_t *b, int bstride, const uint16_t *c, int cstride, int rows,
                        int cols, int saver);
void orc_pool_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride, int planes, int h,
                  int w, int ph, int pw, int ky, int kx, int sy, int sx, int reducer);
void orc_softmax_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride, int rows,
                     int cols);
void orc_softmax_grad_f16(uint16_t *dst, int dstride, const uint16_t *src, int sstride,
                          const uint16_t *label, int rows, int cols);

/* The rest of the softmax family and the row scatter / gather functions
   (mshadow/tensor_cpu-inl.h:304-528). `flags`: bit 0 = smooth (alpha used), bit 1 = the
   ignore_label argument is used. 3-D tensors are (d0, d1, d2) with the softmax over d1
   and a row pitch on d2; their label is (d0, d2) with pitch lstride. */
#define ORC_GRAD_SMOOTH 1
#define ORC_GRAD_IGNORE 2
void orc_softmax_grad_ex_f32(float *dst, int dstride, const float *src, int sstride,
                             const float *label, int rows, int cols, int flags,
                             float ignore_label, float alpha);
void orc_softmax3d_f32(float *dst, int dstride, const float *src, int sstride, int d0, int d1,
                       int d2);
void orc_softmax3d_grad_f32(float *dst, int dstride, const float *src, int sstride,
                            const float *label, int lstride, int d0, int d1, int d2, int flags,
                            float ignore_label, float alpha);
/* index_is_int: the index array holds int32 (else float, truncated like a label) */
void orc_add_take_grad_f32(float *dst, int dstride, int k_rows, const void *index,
                           int index_is_int, int n_index, const float *src, int sstride,
                           int cols);
void orc_add_take_grad_large_batch_f32(float *dst, int dstride, const void *sorted,
                                       const void *index, int index_is_int, int n_index,
                                       const float *src, int sstride, int cols);
void orc_index_fill_f32(float *dst, int dstride, const void *index, int index_is_int,
                        int n_index, const float *src, int sstride, int cols);

/* the same families for another element type (type_flag 0 float, 1 double, 2 half_t) and, for the
   row functions, another index type (index_flag 0 float, 2 half_t, 4 int32, 6 int64) */
void orc_grad_family_any(int type_flag, void *dst, int dstride, const void *src, int sstride,
                         const void *label, int lstride, int d0, int rows_or_d1, int cols_or_d2,
                         int flags, double ignore_label, float alpha);
void orc_softmax3d_any(int type_flag, void *dst, int dstride, const void *src, int sstride, int d0,
                       int d1, int d2);
void orc_rows_by_index_any(int op, int type_flag, int index_flag, void *dst, int dstride, int k_rows,
                           const void *sorted, const void *index, int n_index, const void *src,
                           int sstride, int cols);

void orc_sort_by_key_32(void *keys, int key_kind, void *values, int n, int is_ascend);
void orc_vectorized_sort_32(void *values, int value_kind, void *segments, int n);

void orc_pool_f32(float *dst, int dstride, const float *src, int sstride, int planes, int h, int w,
                  int ph, int pw, int ky, int kx, int sy, int sx, int reducer);
void orc_unpool_f32(float *dst, int dstride, const float *src, int sstride, const float *pooled,
                    int pstride, const float *grad, int gstride, int planes, int h, int w, int ph,
                    int pw, int ky, int kx, int sy, int sx, int reducer);

/* col = unpack_patch2col(pad(img, pad_y, pad_x), ky, kx, sy, sx, dy, dx) */
void orc_im2col_f16(uint16_t *col, int cstride, const uint16_t *img, int istride, int n, int c,
                    int h, int w, int ky, int kx, int sy, int sx, int dy, int dx, int pad_y,
                    int pad_x);
void orc_im2col_f32(float *col, int cstride, const float *img, int istride, int n, int c, int h,
                    int w, int ky, int kx, int sy, int sx, int dy, int dx, int pad_y, int pad_x);
/* img = crop(pack_col2patch(col, (n,c,h+2pad_y,w+2pad_x), ...), (h,w), pad_y, pad_x) */
void orc_col2im_f16(uint16_t *img, int istride, const uint16_t *col, int cstride, int n, int c,
                    int h, int w, int ky, int kx, int sy, int sx, int dy, int dx, int pad_y,
                    int pad_x);
void orc_col2im_f32(float *img, int istride, const float *col, int cstride, int n, int c, int h,
                    int w, int ky, int kx, int sy, int sx, int dy, int dx, int pad_y, int pad_x);

#ifdef __cplusplus
}
#endif
#endif  /* MSHADOW_ORACLE_H_ */
