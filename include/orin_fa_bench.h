/*
 * orin_fa_bench -- measurement aids, in libraries of their own beside the product library.  None of them
 * has a counterpart in the reference and none is part of the attention path: bench.py uses them for the
 * yardsticks its figures are read against.  An engine has no reason to call them, and liborin_fa.so exports
 * none of them.
 *
 *   liborin_fa_bench.so   (orin_llm_amd/csrc/bench_aids.hip alone; independent of liborin_fa.so) exports the
 *                         read-only stand-ins below.  Every call names the HIP stream it launches on and the
 *                         device buffers it uses; nothing is allocated, no state is kept.  Returns 0, -1 for a
 *                         refused argument, or minus the hipError_t of the launch.
 *   liborin_fa_stamps.so  (the product's sources with -DORIN_FA_STAMPS: the timeline build) exports the product
 *                         ABI plus orin_fa_bench_stamps.
 */
#ifndef ORIN_FA_BENCH_H
#define ORIN_FA_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* One launch of a kernel that does nothing but read `bytes` bytes at src (device, 16-byte aligned) once with
 * streaming 128-bit loads spread over every CU: loads_per_thread (2, 4, 8 or 16) 16-byte loads per thread of
 * 512-thread workgroups.  What a decode step's cache read costs when nothing else is done with the bytes.
 * sink: one device word that is never written (it keeps the loads alive).  Asynchronous. */
int orin_fa_bench_hbm_read(const void* src, size_t bytes, int loads_per_thread, unsigned* sink, void* stream);

/* One launch of a kernel that only reads a pair of Q4_K-shaped matrices (n_rows rows of n_blocks 144-byte blocks
 * each; the second matrix mat_bytes behind the first; w 16-byte aligned, n_rows a multiple of 16, n_blocks of 8)
 * the way a matrix-vector kernel would: workgroups of four waves over 16-row tiles.  pattern 0: per load
 * instruction 64 bytes of each of 16 rows (header, and a piece of each half of a block's nibbles); pattern 1, 2,
 * 4: runs of that many whole blocks of a row, lane after lane, with streaming loads.  What the load pattern alone
 * costs, nothing computed.  Asynchronous. */
int orin_fa_bench_read_pattern(const void* w, size_t mat_bytes, int n_rows, int n_blocks, int pattern, int workgroups,
                               unsigned* sink, void* stream);

/* A stand-in for one split-KV decode step, to price the two ways of merging its partial results: 256 workgroups
 * stream orin_fa_bench_handoff_stream_bytes() (32 MiB) at src and leave 784-float partial results that are then
 * added up into out[784] -- fused = 0: by a second kernel (two launches, what the library does); fused = 1:
 * inside the one launch, by a two-level last-arriver reduction over write-through stores and relaxed agent-scope
 * atomics (no cache-wide fence).  scratch: orin_fa_bench_handoff_scratch_bytes() of device memory, zeroed once by
 * the caller before the first call.  out is the same either way (784 floats: element 4i of every group is the
 * sum of 1..256 = 32896).  Asynchronous. */
int orin_fa_bench_handoff(const void* src, int fused, void* scratch, float* out, void* stream);
size_t orin_fa_bench_handoff_scratch_bytes(void);
size_t orin_fa_bench_handoff_stream_bytes(void);

/* One launch of a one-wave kernel that reads one word at src: the cost of a launch as such, when timed back to
 * back.  Asynchronous. */
int orin_fa_bench_tiny_launch(const unsigned* src, unsigned* sink, void* stream);

/* liborin_fa_stamps.so only (in the timeline build lane 0 of every wave of the prefill kernel, of the decode split
 * kernel and of the matrix-vector kernel that reads rows in long runs stores the 100 MHz wall clock at the end of
 * each stage).  Copies the table of the kernel's last launch to host memory: which = 0 prefill, n <= 1024
 * workgroups x 4 waves x 16 slots; which = 1 decode split kernel, n <= 1024 x 8 x 16; which = 2 matrix-vector
 * kernel, n <= 1024 x 4 x 16 (waves 0-3 of a workgroup); entry [workgroup][wave][slot], workgroups numbered
 * x + gridDim.x * (y + gridDim.y * z); a mark a wave did not pass reads 0.  Clears the table afterwards.
 * Synchronous.  Return codes as in orin_fa.h. */
int orin_fa_bench_stamps(int which, long long* host, size_t n);

/* (The cut-off builds liborin_fa_probe_<flags>.so / liborin_fa_pprobe_<flags>.so, built only on request by
 * `python -m orin_llm_amd.build --probes`, export the product ABI with parts of the decode split kernel or of the
 * prefill kernel taken out, as orin_llm_amd/csrc/fa_decode.hip and fa_prefill.hip describe under
 * ORIN_FA_DECODE_PROBE / ORIN_FA_PREFILL_PROBE: their results are wrong by design and only bench_aids.py loads
 * them.) */

#ifdef __cplusplus
}
#endif
#endif
