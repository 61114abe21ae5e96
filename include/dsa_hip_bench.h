/*
 * Measurement aids of the MI355X DSA kernels: built into libdsa_bench.so, which only the benchmark
 * loads.  Nothing here is part of the drop-in boundary (include/dsa_hip.h) and nothing here has a
 * counterpart in the reference.  Status codes and dsa_last_error() as in dsa_hip.h.
 */
#ifndef DSA_HIP_BENCH_H
#define DSA_HIP_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * Profiling variant of dsa_sparse_mla_bwd: same arguments and results, plus the time of each launch
 * group in milliseconds, measured with HIP events on `stream` and summed over query chunks:
 *   pass_ms[0] key-sorted order   [1] P and dS   [2] per-pair dKV rows   [3] dQ beside the ordered dKV reduce   [4] 0
 * It creates and destroys HIP events and waits for the stream before returning, so it is for
 * benchmarks only.  No counterpart in the reference (its kernels are timed with do_bench from
 * Python, ops/tilelang_ops/sparse_mla_bwd.py:359-368).
 */
int dsa_sparse_mla_bwd_profile(const void* q, const void* kv, const void* out, const void* dout,
                               const int32_t* ids, const float* lse, int S, int H, int Skv, int K,
                               int q_start, float sm_scale, int d_v, void* dq, void* dkv,
                               void* workspace, size_t workspace_bytes, void* stream, float* pass_ms);

/*
 * Measurement aids; no counterpart in the reference.  Plain data movers with the traffic shape of
 * the two bandwidth-bound backward passes, and a kernel of nothing but bf16 MFMAs, so that a
 * benchmark can quote the kernels against what the memory system and the matrix pipes give a
 * kernel that does nothing else.
 *
 * dsa_probe_hbm_rows: `workgroups` x `rows_per_workgroup` (a multiple of 4) rows of 1152 bytes are
 * written to `rows` (at permuted row positions when scatter != 0, in order otherwise) while each
 * workgroup streams 4608 bytes from `src` on read_fifths (0..5) of every 5 steps of 4 rows; with
 * n = rows_per_workgroup / 4 steps, src must hold
 * workgroups * (n / 5 * read_fifths + min(n % 5, read_fifths)) * 4608 bytes.
 * dsa_probe_hbm_read: streams `bytes` from src; sink16 points at 16 writable bytes.
 */
int dsa_probe_hbm_rows(const void* src, void* rows, int workgroups, int rows_per_workgroup, int read_fifths,
                       int scatter, void* stream);
int dsa_probe_hbm_read(const void* src, size_t bytes, void* sink16, void* stream);
/* dsa_probe_mfma_bf16: `workgroups` x 4 waves each issue iters x 16 v_mfma_f32_32x32x16_bf16 and nothing else;
 * *flops (may be NULL) receives the flop count of the launch; sink4 points at 4 writable bytes. */
int dsa_probe_mfma_bf16(int workgroups, int iters, void* sink4, double* flops, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DSA_HIP_BENCH_H */
