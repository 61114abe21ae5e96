// Plain data movers with the traffic shapes of the two HBM-bound backward passes.  They do no
// arithmetic worth the name, so their rate is what the memory system gives a kernel that moves the
// same bytes the same way: 1152-byte rows written at scattered row positions beside a streaming read
// (the dKV-row pass), and a pure streaming read (the ordered dKV sum).  The benchmark quotes the
// passes against these rates next to the nominal HBM peak.
#include "../dsa_common.h"
#include "../../../include/dsa_hip_bench.h"

namespace {

// 288 threads = 4 groups of 72 lanes; a group writes one 1152-byte row per iteration (16 B per
// lane).  On read_fifths of every 5 iterations each thread also reads 16 B from a stream of its own
// workgroup (4608 B per 4 rows written).
__global__ __launch_bounds__(288) void probe_rows_kernel(const uint4* __restrict__ src, uint4* __restrict__ rows,
                                                         long long nrows, int rows_per_wg, int read_fifths,
                                                         long long mult) {
  const int grp = threadIdx.x / 72, ch = threadIdx.x % 72;
  const long long wg = blockIdx.x;
  const int iters = rows_per_wg / 4;
  uint4 acc = {1u, 2u, 3u, 4u};
  const int rem = iters % 5;
  const int reads = iters / 5 * read_fifths + (rem < read_fifths ? rem : read_fifths);   // iterations that read
  long long rd = wg * (long long)reads * 288 + threadIdx.x;
  for (int it = 0; it < iters; it++) {
    if (it % 5 < read_fifths) {
      const uint4 v = src[rd];
      rd += 288;
      acc.x ^= v.x; acc.y += v.y; acc.z ^= v.z; acc.w += v.w;
    }
    long long r = wg * rows_per_wg + it * 4 + grp;
    if (mult) r = (r * mult) % nrows;
    rows[r * 72 + ch] = acc;
  }
}

__global__ __launch_bounds__(256) void probe_read_kernel(const uint4* __restrict__ src, size_t n16, uint4* __restrict__ sink) {
  uint4 acc = {0u, 0u, 0u, 0u};
  const size_t stride = (size_t)gridDim.x * 256;
  size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
  for (; e + 3 * stride < n16; e += 4 * stride) {
    const uint4 a = src[e], b = src[e + stride], c = src[e + 2 * stride], d = src[e + 3 * stride];
    acc.x ^= a.x ^ b.x ^ c.x ^ d.x; acc.y += a.y + b.y + c.y + d.y;
    acc.z ^= a.z ^ b.z ^ c.z ^ d.z; acc.w += a.w + b.w + c.w + d.w;
  }
  for (; e < n16; e += stride) { const uint4 a = src[e]; acc.x ^= a.x; acc.y += a.y; acc.z ^= a.z; acc.w += a.w; }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u) sink[0] = acc;     // keeps the loads alive; practically never taken
}

// Nothing but bf16 MFMAs: each wave runs `iters` rounds of 16 back-to-back v_mfma_f32_32x32x16_bf16 on four
// independent accumulators with non-trivial operands; what the matrix pipes sustain at the clock the
// part holds under that load.
__global__ __launch_bounds__(256, 1) void probe_mfma_kernel(float* __restrict__ sink, int iters) {
  const int lane = threadIdx.x & 63;
  bf16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    // pseudo-random values in [-1, 1): operands with busy mantissa bits (the clock the part holds depends
    // on how many bits toggle; all-zero operands run a fifth faster)
    const unsigned ha = (unsigned)(lane * 8 + e + 1) * 2654435761u, hb = (unsigned)(lane * 8 + e + 977) * 2246822519u;
    a[e] = (__bf16)((float)(ha >> 16) * (1.0f / 32768.0f) - 1.0f);
    b[e] = (__bf16)((float)(hb >> 16) * (1.0f / 32768.0f) - 1.0f);
  }
  f32x16 acc[4];
#pragma unroll
  for (int u = 0; u < 4; u++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[u][e] = 0.f;
  for (int it = 0; it < iters; it++) {
    asm volatile("" : "+v"(a), "+v"(b));          // keeps the loop body in the loop
#pragma unroll
    for (int r = 0; r < 4; r++)
#pragma unroll
      for (int u = 0; u < 4; u++) acc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[u], 0, 0, 0);
  }
  float keep = 0.f;
#pragma unroll
  for (int u = 0; u < 4; u++) keep += acc[u][0];
  if (keep == 123.456f) sink[0] = keep;           // practically never taken
}

}  // namespace

extern "C" int dsa_probe_mfma_bf16(int workgroups, int iters, void* sink4, double* flops, void* stream) {
  DSA_REQUIRE(workgroups > 0 && iters > 0 && sink4 != nullptr, "dsa_probe_mfma_bf16: bad arguments");
  probe_mfma_kernel<<<dim3(workgroups), dim3(256), 0, (hipStream_t)stream>>>((float*)sink4, iters);
  DSA_CHECK_LAUNCH("dsa_probe_mfma_bf16");
  if (flops) *flops = (double)workgroups * 4.0 * (double)iters * 16.0 * (2.0 * 32 * 32 * 16);
  return DSA_OK;
}

extern "C" int dsa_probe_hbm_rows(const void* src, void* rows, int workgroups, int rows_per_workgroup, int read_fifths,
                                  int scatter, void* stream) {
  DSA_REQUIRE(workgroups > 0 && rows_per_workgroup > 0 && rows_per_workgroup % 4 == 0, "dsa_probe_hbm_rows: bad sizes");
  DSA_REQUIRE(read_fifths >= 0 && read_fifths <= 5, "dsa_probe_hbm_rows: read_fifths must be 0..5");
  DSA_REQUIRE(((uintptr_t)src % 16) == 0 && ((uintptr_t)rows % 16) == 0, "dsa_probe_hbm_rows: misaligned pointer");
  const long long nrows = (long long)workgroups * rows_per_workgroup;
  // an odd multiplier that shares no factor with nrows permutes the rows
  long long mult = 0;
  if (scatter) {
    mult = 1000003;
    auto gcd = [](long long a, long long b) { while (b) { long long t = a % b; a = b; b = t; } return a; };
    while (gcd(mult, nrows) != 1) mult += 2;
    DSA_REQUIRE(nrows < ((long long)1 << 40), "dsa_probe_hbm_rows: too many rows");
  }
  probe_rows_kernel<<<dim3(workgroups), dim3(288), 0, (hipStream_t)stream>>>((const uint4*)src, (uint4*)rows, nrows,
                                                                            rows_per_workgroup, read_fifths, mult);
  DSA_CHECK_LAUNCH("dsa_probe_hbm_rows");
  return DSA_OK;
}

extern "C" int dsa_probe_hbm_read(const void* src, size_t bytes, void* sink16, void* stream) {
  DSA_REQUIRE(bytes >= 16 && ((uintptr_t)src % 16) == 0 && sink16 != nullptr, "dsa_probe_hbm_read: bad arguments");
  probe_read_kernel<<<dim3(8192), dim3(256), 0, (hipStream_t)stream>>>((const uint4*)src, bytes / 16, (uint4*)sink16);
  DSA_CHECK_LAUNCH("dsa_probe_hbm_read");
  return DSA_OK;
}
