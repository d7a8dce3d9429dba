/*
 * pylo_mi355_bench.h -- measurement instrumentation of libpylo_mi355.so.
 *
 * NOT part of the drop-in boundary (include/pylo_mi355.h): nothing here has a counterpart in the
 * reference, and no optimizer step depends on it.  bench.py uses these entry points to time the launches of
 * a step with HIP events on the stream they run on, and to measure what the memory system delivers for the
 * access mixes of the element passes with nothing computed.
 */
#ifndef PYLO_MI355_BENCH_H
#define PYLO_MI355_BENCH_H

#include "pylo_mi355.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Optional per-launch timing, for benchmarks (no counterpart in the reference).  Between begin and
   end every *_step call records one HIP event before its first launch and one after each launch,
   on the call's stream, for at most `max_steps` calls.  end synchronises the last event and
   writes steps x num_launches durations in milliseconds (row-major) into ms_out. */
int pylo_mi355_plan_timing_begin(PyloPlan* plan, int max_steps);
int pylo_mi355_plan_timing_end(PyloPlan* plan, float* ms_out, int capacity, int* steps_out);

/* Names of the launches of one step, in launch order (static strings). */
const char* pylo_mi355_plan_launch_name(const PyloPlan* plan, int launch);

/* Bare streaming kernel, for benchmarks (no counterpart in the reference): per element, `reads` arrays of n
   floats are read (in[r * n + i]) and `writes` arrays written (out[w * n + i]), 16 bytes per lane and access,
   nothing computed.  It measures what the memory system delivers for an access mix -- 6 reads and 5 writes
   is the apply pass of the ELO-CELO2 step, 6 reads its statistics pass.  reads in {1, 6}, writes in
   {0, 1, 5}; n a multiple of 4; nontemporal != 0 uses non-temporal loads and stores. */
int pylo_mi355_stream_probe(const float* in, float* out, size_t n, int reads, int writes, int nontemporal,
                            void* stream);

/* Bare matrix-pipe kernel, for benchmarks (no counterpart in the reference): the main loop of the Newton-Schulz
   update product (tiles of 128 x 256 outputs, six v_mfma_f32_32x32x16_bf16 per fp32 tile product) over caller-
   provided operand planes, every tile job over k_steps reduction steps.  x_planes: rows_x rows (a multiple of
   128), b_planes: rows_b rows (a multiple of 256), both laid out [k_steps / 16][rows][3 planes][16] bf16
   (96 bytes a row and block of 16 steps).  mode 0: the product's own loop (operands staged from memory into
   LDS every 16 steps); 1: the operands of the first 16 steps staged once and read from LDS in every step;
   2: their fragments kept in registers, matrix instructions only.  out: (rows_x / 128) (rows_b / 256) x 256
   floats.  What the planes hold decides the power the matrix pipe draws and with it the clock: zeros run
   faster than data. */
int pylo_mi355_matrix_probe(const void* x_planes, int rows_x, const void* b_planes, int rows_b, int k_steps, int mode,
                            float* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* PYLO_MI355_BENCH_H */
