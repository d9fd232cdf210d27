/*
 * megagemm_hip_tuning.h -- measurement and tuning aids of libmegagemm_hip.so.
 *
 * Nothing here has a counterpart in the reference, and no normal caller needs it: the
 * operators are declared in megagemm_hip.h.  These functions exist for benchmarks, profiler
 * runs and tests.  mg_set_option changes PROCESS-WIDE state: it is not synchronised with
 * calls running on other threads (a call reads each option once when it starts), and while
 * an override is in force the launch shape, the workspace shape that
 * mg_rmsnorm_bwd_workspace reports and hence the summation order of dW depend on it.
 */
#ifndef MEGAGEMM_HIP_TUNING_H
#define MEGAGEMM_HIP_TUNING_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Reports the launch shape mg_rmsnorm_fwd (backward == 0) or mg_rmsnorm_bwd (backward != 0)
 * takes for rows of `cols` elements; no counterpart in
 * the reference (whose launchers always use 256 threads per row, src/rmsnorm_kernel.cu:530).
 * Host-only: needs no device.  *generic = 1 means the element-wise kernels (one 256-thread
 * workgroup per row, *vectors_per_thread = 0).  *generic = 0 with *vectors_per_thread = 0
 * means a row too wide for registers, streamed twice by a 1024-thread workgroup.
 * *threads_per_row below 64 means that
 * 64 / *threads_per_row consecutive rows share a wave (rows of at most 2 KiB; at most
 * 640 bytes when the pitch is not a multiple of 16 bytes).
 * *vectors_per_thread = -G (G = 1, 2 or 4) means the row-group layout of rows of at most 64
 * vectors: a lane holds one vector of its row, *threads_per_row (1, 2, 4 ... 64) lanes serve
 * a row, and a wave keeps G groups of 64 / *threads_per_row consecutive rows in flight.
 */
int mg_rmsnorm_launch_info(int backward, int64_t cols, int dtype, int* generic, int* threads_per_row,
                           int* vectors_per_thread, int* workgroup_threads);

/*
 * Measurement aid with no counterpart in the reference: a plain device-to-device copy of
 * `bytes` (a multiple of 16; both pointers 16-byte aligned) done by one kernel that moves
 * one 16-byte vector per thread.  Its HBM traffic is exactly 2*bytes, which makes it the
 * yardstick for calibrating hardware traffic counters when profiling the other kernels.
 */
int mg_copy_bytes(void* dst, const void* src, int64_t bytes, void* stream);

/*
 * Streaming yardstick: one kernel that moves `bytes` (a multiple of 16; pointers aligned
 * to 4 bytes at least -- 16 for the aligned case the operators see with row pitches that are
 * multiples of 16) with the same 16-byte non-temporal buffer accesses as the operators,
 * 4 KiB per workgroup.  b == NULL: dst = a (one read, one write per byte); otherwise dst = a + b as
 * 32-bit words (two reads, one write).  The time such a launch takes at a given size is
 * the ceiling for an operator with the same read/write mix at that size.
 */
int mg_stream_probe(void* dst, const void* a, const void* b, int64_t bytes, void* stream);

/*
 * The same traffic with the operators' division of work: one workgroup (256 threads for rows
 * of up to 4 KiB, 512 up to 16 KiB, 1024 beyond) owns whole rows of `row_bytes` (a multiple of
 * 16, at most 65536) and walks the rows g, g + G, g + 2G ... of [rows, row_bytes] matrices,
 * requesting its next row before it stores the current one: dst = a (b == NULL) or
 * dst = a + b on 32-bit words.  workgroups = 0 (or >= rows) gives every row a workgroup of
 * its own, as the forward pass does; a smaller number G is a persistent grid, as backward
 * pass 1 uses.  It shows what the machine delivers when a workgroup has to take a whole row
 * at a time: the same as 4 KiB pieces for rows of up to 16 KiB, 5-15 % less at 32 KiB.
 */
int mg_row_probe(void* dst, const void* a, const void* b, int64_t rows, int64_t row_bytes,
                 int64_t workgroups, void* stream);

/*
 * mg_rmsnorm_bwd with a clock: the same launch (same results, same arguments), from a build of
 * the kernel in which thread 0 of every workgroup writes time stamps of the GPU's constant
 * 100 MHz clock (10 ns units, comparable across workgroups) to records[num_partials]
 * [MG_TIMELINE_WORDS]: word 0 = start of the workgroup, word 1 + i = end of its i-th sweep over
 * its row slots (the first MG_TIMELINE_ITERATIONS of them; 0 where there was none), word
 * MG_TIMELINE_WORDS - 3 = end of the row loop, MG_TIMELINE_WORDS - 2 = end of the workgroup (its
 * partial row written), MG_TIMELINE_WORDS - 1 = the die (XCC) it ran on.  It shows where a launch
 * spends its time: how long the first rows take to arrive, what a sweep costs once the memory
 * pipeline is full, and how far the last workgroup finishes behind the median one.  Only rows
 * that take the register-ring kernel on 512 threads (385-512 vectors of 16 bytes at a 16-byte
 * pitch: 4096 bf16/fp16 columns, 2048 fp32 columns) have such a build; other shapes return
 * MG_ERR_UNSUPPORTED.  records must be zeroed by the caller if unwritten words are to read 0.
 */
#define MG_TIMELINE_WORDS 32
#define MG_TIMELINE_ITERATIONS 24
int mg_rmsnorm_bwd_timeline(void* dx, float* dw_partial, const void* dy, const void* x, const void* w,
                            const float* inv_rms, int64_t rows, int64_t cols, int dtype, int64_t num_partials,
                            int64_t ld, uint64_t* records, void* stream);

/*
 * Tuning hook (not needed for normal use): overrides one launch parameter for the
 * calling process.  Keys: "fwd_tpr", "bwd_tpr" (threads per row: 64...1024, or 8 / 16 / 32 for
 * rows of at most 4 vectors per thread; -1 = never fewer than 64), "fwd_items" (target
 * 16-byte vectors per thread; 0 = automatic), "bwd_block" (1024 or 512 threads per
 * workgroup; 256 = one row slot of 256 threads per workgroup, two workgroups per compute unit,
 * for rows of up to 512 vectors), "bwd_wg_per_cu", "bwd_partials" (workgroups of the persistent backward grid, which is
 * also the number of partial rows; 0 = automatic), "bwd_partial_policy" (how the register-ring kernel
 * on 512 threads per row stores its partial row: 0 default, 1 non-temporal, 2 written through to
 * memory; other kernels ignore it), "bwd_prefetch" (1/0: request the next row before reducing
 * the current one; -1 = automatic), "narrow_groups" (the row-group layout for rows of at most
 * 64 vectors: 1, 2 or 4 groups in flight, 0 = never, -1 = automatic; a "fwd_tpr" / "fwd_items" /
 * "bwd_tpr" / "bwd_block" override switches the automatic choice off), "bwd_lds" (backward rows
 * of 1025-4096 vectors on 1024 threads with the dW sums in LDS: 0 = never, 1 = from 1025
 * vectors on, -1 = automatic), "bwd_ring" (backward rows at 16-byte pitches that fill their
 * lanes at one vector per thread, kept in flight through a ring of register buffers: 0 = never,
 * 2 or 4 = that many buffers, -1 = automatic; a "bwd_tpr" / "bwd_block" override switches it
 * off as well), "fwd_lines" (1 = forward rows of more than 256 vectors whose pitch is a multiple of 8 but not of
 * 128 bytes take the layout with the 16-byte vectors on the 128-byte lines of the output instead of
 * counted from the row's first byte, which is faster for some such shapes and slower for others;
 * 0 = never, the default; a "fwd_tpr" / "fwd_items" override switches it off as well), "swiglu_unroll",
 * "force_generic" (1 = always take the one-element-per-thread kernels, which nothing selects by itself), "xcd_group" (consecutive workgroups
 * handled by one die at a time, 0 = off, -1 = automatic), "swiglu_max_units" (vectors or
 * elements one SwiGLU launch may cover before the input is split by rows; 0 = 2^31).  Returns MG_ERR_INVALID_ARG for
 * an unknown key.  Values that do not fit a given problem are ignored for that call.
 */
int mg_set_option(const char* key, int value);

/*
 * Number of successful mg_set_option calls in this process so far.  The answers of
 * mg_rmsnorm_bwd_workspace and mg_rmsnorm_launch_info depend on the options: a caller that
 * remembers them (the ctypes binding does) keeps this number beside them and asks again when it
 * has moved, whoever moved it.
 */
int mg_option_generation(void);

#ifdef __cplusplus
}
#endif
#endif /* MEGAGEMM_HIP_TUNING_H */
