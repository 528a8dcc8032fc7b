/*
 * libmshadow_probe - measurement aids used by bench.py (`--only softmax_phases`,
 * `--only ceiling_chain`). They have no counterpart in the reference and are no part of
 * the device layer: libmshadow_hip.so and the mshadow headers do not depend on them.
 * Same conventions as mshadow_hip.h: 0 on success, text from mshadow_probe_last_error().
 */
#ifndef MSHADOW_HIP_PROBE_H_
#define MSHADOW_HIP_PROBE_H_

#ifdef __cplusplus
extern "C" {
#endif

const char *mshadow_probe_last_error(void);

/* Cost of one dependent float32 add for a single wave, in ns, measured over 131072 adds
   with `workgroups` one-wave workgroups running at once (1: an otherwise idle chip; one per
   CU or more: the clock the chip keeps under load). Modes: */
#define MSHADOW_PROBE_CHAIN_REGISTER 0 /* s = s + a, both in vector registers */
#define MSHADOW_PROBE_CHAIN_LDS 1      /* the column reduction's chain: 16 lanes, operands by
                                          128-bit LDS reads fetched 32 adds ahead */
#define MSHADOW_PROBE_CHAIN_LANES 2    /* the softmax row sum's chain: the sum handed to the
                                          next lane by a DPP add */
#define MSHADOW_PROBE_CHAIN_REGISTER_F16 3 /* s = s + a on binary16 values (a half_t sum) */
int mshadow_probe_add_chain(int mode, int workgroups, double *ns_per_add, void *stream);

/* The softmax kernel for rows of 16385..32768 columns (one 512-thread workgroup per row, the
   row in registers), with a 100 MHz time stamp taken by thread 0 of every row at each step
   named below, after all of the thread's outstanding memory operations have completed.
   mean_us[i] = mean over rows of the time from the previous step of the list to step i
   (-1: no row reached it); resident_us = mean time from entry to the last step;
   kernel_us = duration of the launch by HIP events; fallback_rows = rows whose plan did not
   hold and that were summed by wave scans instead. dst may alias src. */
#define MSHADOW_PROBE_STAMP_FALLBACK 7
#define MSHADOW_PROBE_STAMPS 16
#define MSHADOW_PROBE_STAMP_ORDER {10, 11, 12, 13, 1, 2, 6, 8, 3, 4, 5, 14}
#define MSHADOW_PROBE_STAMP_NAMES                                                        \
  {"10 entry", "11 row loaded, thread maxima", "12 row maximum (barrier)", "13 exp",      \
   "1 chunk sums and maxima exchanged (barrier)", "2 chunk plan", \
   "6 certain chunks quantised", "8 lists of the other chunks written",               \
   "3 every wave's chunks done (barrier)", "4 row's list of addends assembled (barrier)",           \
   "5 chain (wave 0; barrier)", "14 divided and stored (stores completed)"}
int mshadow_probe_softmax_phases(float *dst, int dstride, const float *src, int sstride, int rows,
                                 int cols, double *mean_us, double *resident_us,
                                 double *kernel_us, int *fallback_rows, void *stream);

/* The memory side of that kernel alone: every workgroup loads its row into registers as the
   softmax kernel does, meets `barriers` workgroup barriers with `spin` multiply-adds per
   element before each, and stores the row. barriers = 0: what the access pattern itself
   allows (one workgroup per row, two rows resident per CU); with spin > 0: how much work
   between load and store the machine hides. resident = 2: two rows per CU as in the softmax
   kernel; 1: one (a second workgroup is kept off the CU). kernel_us = duration of the launch. */
int mshadow_probe_row_copy(float *dst, int dstride, const float *src, int sstride, int rows,
                           int cols, int barriers, int spin, int resident, double *kernel_us,
                           void *stream);

/* Rate of loads from global memory straight into LDS (the loads of the reduction kernels),
   with nothing consuming the data: `waves` waves per workgroup keep window .. window + 16
   loads (window = 16 or 32) of `width` bytes per lane (4 or 16) outstanding each. strip = 0: the matrix is read as one buffer,
   1024 workgroups take a contiguous piece each and an instruction fetches 64 * width
   consecutive bytes; strip = 16, 32 or 64: a workgroup reads that many columns of every
   row, as a reduction over the rows does, cols / strip workgroups, neighbouring strips
   behind the same L2; strip = -1: the matrix is read as 64 x 256 segments, 256 workgroups
   take 64 segments each (every 256th) and read them side by side, one instruction's worth
   (64 * width bytes) of each in turn, as a reduction that keeps the second of four
   dimensions does. kernel_us = duration of the
   launch that reads rows x cols floats once. */
int mshadow_probe_dma_rate(const float *src, int sstride, int rows, int cols, int strip, int width,
                           int waves, int window, double *kernel_us, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MSHADOW_HIP_PROBE_H_ */
