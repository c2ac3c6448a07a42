/*
 * orin_fa_bench -- measurement aids exported by liborin_fa.so beside the product ABI of
 * include/orin_fa.h.  None of them has a counterpart in the reference and none is part of the
 * attention path: bench.py uses them for the yardsticks its figures are read against.  An
 * engine has no reason to call them.
 */
#ifndef ORIN_FA_BENCH_H
#define ORIN_FA_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* orin_fa_decode_ind with HIP events recorded before, between and after its two kernels on the
 * library's stream.  Synchronises on the last event and returns the elapsed time of the split
 * kernel and of the combine kernel in microseconds (the latter 0 when the shape needs no
 * split).  Not capture-safe. */
int orin_fa_decode_ind_timed(const float* q, const uint16_t* kc, const uint16_t* vc, float* out,
                             int n_head, int n_kv, int head_dim, int n_ctx, const int* d_pos, float scale,
                             float* us_split, float* us_combine);

/* One launch, on the library's stream, of a kernel that does nothing but read `bytes` bytes at
 * src (device, 16-byte aligned) once with streaming 128-bit loads spread over every CU:
 * loads_per_thread (2, 4, 8 or 16) 16-byte loads per thread of 512-thread workgroups.  What a
 * decode step's cache read costs when nothing else is done with the bytes.  Asynchronous. */
int orin_fa_bench_hbm_read(const void* src, size_t bytes, int loads_per_thread);

/* One launch, on the library's stream, of a kernel that only reads a pair of Q4_K-shaped matrices (n_rows rows of
 * n_blocks 144-byte blocks each; the second matrix mat_bytes behind the first; w 16-byte aligned, n_rows a multiple
 * of 16, n_blocks of 8) the way a matrix-vector kernel would: workgroups of four waves over 16-row tiles.
 * pattern 0: per load instruction 64 bytes of each of 16 rows (header, and a piece of each half of a block's nibbles);
 * pattern 1, 2, 4: runs of that many whole blocks of a row, lane after lane, with streaming loads.  What the load
 * pattern alone costs, nothing computed.  Asynchronous. */
int orin_fa_bench_read_pattern(const void* w, size_t mat_bytes, int n_rows, int n_blocks, int pattern, int workgroups);

/* A stand-in for one split-KV decode step, to price the two ways of merging its partial results:
 * 256 workgroups stream orin_fa_bench_handoff_stream_bytes() (32 MiB) at src and leave 784-float
 * partial results that are then added up into out[784] -- fused = 0: by a second kernel (two
 * launches, what the library does); fused = 1: inside the one launch, by a two-level
 * last-arriver reduction over write-through stores and relaxed agent-scope atomics (no
 * cache-wide fence).  scratch: orin_fa_bench_handoff_scratch_bytes() of device memory, zeroed
 * once by the caller before the first call.  out is the same either way (784 floats: element
 * 4i of every group is the sum of 1..256 = 32896).  Asynchronous, on the library's stream. */
int orin_fa_bench_handoff(const void* src, int fused, void* scratch, float* out);
size_t orin_fa_bench_handoff_scratch_bytes(void);
size_t orin_fa_bench_handoff_stream_bytes(void);

/* One launch, on the library's stream, of a one-wave kernel that reads one word: the cost of
 * a launch as such, when timed back to back.  Asynchronous. */
int orin_fa_bench_tiny_launch(void);

/* (The cut-off builds liborin_fa_probe_<flags>.so export the product ABI too, with the decode split kernel's
 * parts taken out as orin_llm_amd/csrc/fa_decode.hip describes under ORIN_FA_DECODE_PROBE: their results are
 * wrong by design and only bench.py's cut-off workloads load them.) */

/* Timeline build only (liborin_fa_stamps.so: the same sources compiled with -DORIN_FA_STAMPS, in which
 * lane 0 of every wave of the prefill kernel, of the decode split kernel and of the matrix-vector kernel that
 * reads rows in long runs stores the 100 MHz wall clock at the end of each stage).  Copies the table of the
 * kernel's last launch to host memory: which = 0 prefill, n <= 1024 workgroups x 4 waves x 16 slots; which = 1
 * decode split kernel, n <= 1024 x 8 x 16; which = 2 matrix-vector kernel, n <= 1024 x 4 x 16 (waves 0-3 of a
 * workgroup); entry [workgroup][wave][slot], workgroups numbered x + gridDim.x * (y +
 * gridDim.y * z); a mark a wave did not pass reads 0.  Clears the table afterwards.  Synchronous.  The ordinary library returns a HIP "not supported" error. */
int orin_fa_bench_stamps(int which, long long* host, size_t n);

#ifdef __cplusplus
}
#endif
#endif
