/*
 * libmshadow_probe - measurement aids used by bench.py (`--only softmax_phases`,
 * `--only ceiling_chain`, ...). They have no counterpart in the reference and are no part of
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
   hold and that were summed by wave scans instead. dst may alias src. variant 0: the kernel as
   the library launches it (two rows resident per CU); 1: the same with one row per CU; 2: one
   row per CU on 1024 threads - how long a row's steps take when the row has the CU to itself. */
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
                                 int cols, int variant, double *mean_us, double *resident_us,
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

/* The row copy as persistent workgroups fed from their own next row: `workgroups` workgroups
   of `threads` threads (1024: one per CU, 512: two) take rows in turn; while a row is in
   registers (stand-in work as above, then its stores) the first `prefetch_slabs` kilobytes per
   wave of the workgroup's next row are loaded straight into LDS, the rest when the row's turn
   comes. 28672 < cols <= 32768. */
int mshadow_probe_row_copy_prefetch(float *dst, int dstride, const float *src, int sstride, int rows,
                                    int cols, int threads, int prefetch_slabs, int barriers, int spin,
                                    int workgroups, double *kernel_us, void *stream);

/* A copy of `floats` floats by `workgroups` workgroups of four waves that stay until it is done
   (floats a multiple of workgroups x 16 KB), each wave moving 1 KB pieces, four on their way.
   own_run = 1: a wave's pieces are one contiguous run - the resident waves are as many separate
   sequential streams; 0: piece i of wave w is piece i * waves + w - the resident waves work side
   by side on one region that moves through memory. kernel_us = duration of the launch. */
int mshadow_probe_stream_copy(float *dst, const float *src, size_t floats, int workgroups, int own_run,
                              double *kernel_us, void *stream);

/* Rate of loads into LDS when workgroup b reads segments b * segs .. b * segs + segs - 1 of
   `seg_len` floats each (they lie one after the other in memory) side by side, `piece_instr`
   instructions (64 * width bytes each) of one segment, then of the next: nseg / segs
   workgroups of `waves` waves. The part of a segment that does not fill a round of pieces is
   not read. */
int mshadow_probe_seg_rate(const float *src, size_t floats, int seg_len, int nseg, int segs, int width,
                           int waves, int piece_instr, double *kernel_us, void *stream);

/* sumall_except_dim<1> over a dense (n, c, y, x) float tensor with the inner chains dealt out
   in groups of segments (kernels/reduce_dma.h), for a choice of segments per workgroup, loader
   waves, ring slots and bytes per lane and load: config 0..8 = (64,8,8,4) (32,8,8,4) (16,8,4,16)
   (32,8,4,16) (16,4,8,4) (32,8,6,4) (64,8,6,4) (32,4,8,4) (16,8,8,4); config -1 = one workgroup
   per kept index. The timed launch reads `src`
   after a launch on `warm` (another tensor of the shape). kernel_us = its duration. */
int mshadow_probe_highdim_split(float *dst, const float *warm, const float *src, int n, int c, int y,
                                int x, int config, double *kernel_us, void *stream);

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
