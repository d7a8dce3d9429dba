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

#ifdef __cplusplus
}
#endif
#endif /* PYLO_MI355_BENCH_H */
