// The sparse-MLA backward once more, with its per-launch timing entry point (dsa_sparse_mla_bwd_profile),
// for the benchmark library only.
#define DSA_BENCH_BUILD 1
#include "../../../include/dsa_hip_bench.h"
#include "../mla_bwd.hip"
