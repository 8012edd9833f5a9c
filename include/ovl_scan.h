/*
 * C ABI of the hand-written row scan kernels for AMD GPUs (libovl_scan.so).
 *
 * The reference's `accumulate` operator (opveclib/examples/test_accumulate.py:22-78; `cumsum` 81-113, `cumprod`
 * 116-147) is generated for one fixed shape per trace: one worker per row runs
 * `acc = x[row, 0]; out[row, 0] = acc; for i in 1 .. n-1: acc = f(acc, x[row, i]); out[row, i] = acc`
 * strictly left to right in the tensor's type.  These entry points compute the running sum and the running product
 * along the last axis of a dense C-ordered [rows, cols] tensor with exactly that order of operations - so results
 * equal the generated operator's and `numpy.cumsum` / `numpy.cumprod` bit for bit - but take the shape at run time
 * and need no code generation or compiler on the machine that calls them:
 *
 *   reference interface                                   replaced by
 *   ----------------------------------------------------  ------------------------------------------
 *   cumsum(x, axis=-1)    test_accumulate.py:81-113        ovl_cumsum_f32 / ovl_cumsum_f64
 *   cumprod(x, axis=-1)   test_accumulate.py:116-147       ovl_cumprod_f32 / ovl_cumprod_f64
 *
 * Kernel: the lane-skewed order-preserving scan.  Sixteen neighbouring lanes share a row; a lane owns a run of
 * consecutive columns of the current group (one 128-bit access for float32, two for float64), runs the recurrence
 * over its run from the carried state it holds and hands its state to its right neighbour with a lane-to-lane move;
 * after sixteen such phases the group is exact and the last lane's state is the carry into the next group.  The
 * columns after a row's last whole group run as one more, partial group across the same sixteen lanes (element-wise
 * loads with the index clamped to the row's end, element-wise stores); rows that do not start on 16-byte boundaries
 * are moved with unaligned vectors; rows shorter than one group take a plain kernel with one lane per row.
 * float64 rows whose length is a multiple of 512 columns (and 16-byte aligned tensors) run the same recurrence fed
 * from LDS, four rows per workgroup.  When the tensor gives every compute unit at most one workgroup (or whole rounds
 * of them with rows of 12288 columns and more) the workgroup has five wavefronts: two load chunks of 512 columns into
 * LDS, one runs the recurrence with 32 columns per lane and phase and publishes only the exact state that enters each
 * lane's segment, one recomputes the segments from those states (same order of operations, same bits) and one stores
 * them.  Otherwise three wavefronts move the chunks and the fourth scans them in place, 16 columns per lane and phase.
 * The result is the same bits whichever kernel runs.
 *
 * Conventions: tensor memory belongs to the caller and must be device accessible; `out` may not overlap `x`; the
 * functions enqueue one kernel on `hip_stream` (a hipStream_t; NULL is the default stream), return without
 * synchronising and allocate nothing.  They return an ovl_status (ovl_launch.h): OVL_EINVAL for null pointers, zero
 * sizes, rows * cols of 2^32 or more, or more than 2^32 - 257 rows, OVL_EHIP for a HIP error (text from ovl_scan_last_error).
 */
#ifndef OVL_SCAN_H_
#define OVL_SCAN_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

int ovl_cumsum_f32(const float* x, uint32_t rows, uint32_t cols, float* out, void* hip_stream);
int ovl_cumprod_f32(const float* x, uint32_t rows, uint32_t cols, float* out, void* hip_stream);
int ovl_cumsum_f64(const double* x, uint32_t rows, uint32_t cols, double* out, void* hip_stream);
int ovl_cumprod_f64(const double* x, uint32_t rows, uint32_t cols, double* out, void* hip_stream);

/*
 * The same functions with the operands associated as a tree instead of left to right: one workgroup per row, every
 * thread scans one 128-bit vector, the threads' totals are combined with wavefront shuffles and through LDS, the total
 * of the steps before travels in a register.  The reference's accumulate (examples/test_accumulate.py:63-76) is the
 * sequential recurrence, so these results are NOT its bits: they differ by rounding (for float32 sums of 16384 values
 * of order one typically in the last one or two digits; relative to a running sum that passes near zero the distance is
 * unbounded, as for any reordering).  In exchange the kernel runs at the speed of memory for every element type.  Rows
 * that are not whole 16-byte aligned vectors, and 2^24 rows or more, take the order-preserving kernels above.
 */
int ovl_cumsum_f32_reassociated(const float* x, uint32_t rows, uint32_t cols, float* out, void* hip_stream);
int ovl_cumprod_f32_reassociated(const float* x, uint32_t rows, uint32_t cols, float* out, void* hip_stream);
int ovl_cumsum_f64_reassociated(const double* x, uint32_t rows, uint32_t cols, double* out, void* hip_stream);
int ovl_cumprod_f64_reassociated(const double* x, uint32_t rows, uint32_t cols, double* out, void* hip_stream);

/*
 * Measurement aid with no counterpart in the reference: moves a dense [rows, cols] float64 tensor the way the
 * generated kernels that scan along the FIRST axis do, without scanning.  One workgroup owns `lines` (4, 8 or 16)
 * neighbouring columns and walks down the rows, so every row contributes `lines` * 8 consecutive bytes to it.
 * `mode` 1 only loads x, 2 only stores (the row index) to out, 3 copies x to out.  Timed beside a scan along the first
 * axis it says how much of that scan's time is the access pattern and how much the recurrence.  Same conventions and
 * status codes as the functions above.
 */
int ovl_strip_copy_f64(const double* x, uint32_t rows, uint32_t cols, double* out, uint32_t lines, uint32_t mode,
                       void* hip_stream);

/* Text of the last error on the calling thread ("" if none). */
const char* ovl_scan_last_error(void);

#ifdef __cplusplus
}
#endif

#endif  /* OVL_SCAN_H_ */
