// Head-averaged attention distribution over the selected slots, recomputed from q, kv, ids and the
// forward's lse instead of read from materialised logits:
//   target[i, t] = (1 / Hm) * sum_{h < Hm} exp(q[i,h,:] . kv[ids[i,t],:] * sm_scale - lse[i,h])
// which equals mean_h softmax_t(logits[i,h,:] * sm_scale)[t] when lse[i,h] is the log-sum-exp of
// that row over the same slots.  Nothing of size [S, H, K] exists: the forward need not write its
// logits (4.3 GB at seq 8192, 17 GB at 32k tokens) and this kernel need not read them back.
//
// One workgroup per query, a wave owns 32 heads and keeps its slice of Q in registers as the MFMA's
// A operand; the gathered key tile is the B operand, so an accumulator holds one key
// per lane and 16 heads per lane: the sum over heads is 15 additions inside a lane, one exchange
// between the half-waves, and one pass over per-wave partial sums in LDS at the end (fixed order).
// Slots are walked in the caller's order, so target lines up with the indexer's scores.
#include "mla_tile.h"

namespace {
using namespace mla;

// Four waves, one tile at a time, per-wave partial sums of all slots kept in LDS until the end.
// (Eight waves on alternate tiles - two per SIMD, 144 registers of Q each - measured the same
// 2.5 ms at [8192, 128, 2048]: the four waves' reads of the whole key tile, not latency, set the pace.)
template <int STAGES>
__global__ __launch_bounds__(256, 1) void attn_dist_qk_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ kv, const int* __restrict__ ids,
    const float* __restrict__ lse, float* __restrict__ target, int H, int Hm, int Skv, int K, int q_start,
    float sm_scale) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int qi = (int)gridDim.x - 1 - (int)blockIdx.x;
  const int NT = K / BI;
  // [STAGES][TILE_BYTES] key tiles | ids arrays | per-wave partial sums [4][K]
  int* idx_s = (int*)(smem + STAGES * TILE_BYTES);
  unsigned* tmask = (unsigned*)(idx_s + K);
  int* tlist = (int*)(tmask + NT);
  int* ntile_s = tlist + NT;
  float* part_s = (float*)(ntile_s + 4);
  for (int t = tid; t < 4 * K; t += 256) part_s[t] = 0.f;   // tiles without a valid slot are never visited
  // the query's rows are requested before the ids are staged: one round trip to memory for both
  const int h = wave * 32 + r;
  const size_t hrow = (size_t)qi * H + (h < H ? h : 0);
  bf16x8 qreg[KSTEPS];
  {
    const bf16x8* qp = (const bf16x8*)(q + hrow * DQK) + g;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) qreg[ks] = qp[2 * ks];
  }
  float lse2[16];
#pragma unroll
  for (int e = 0; e < 16; e++) {
    const int hh = wave * 32 + 8 * (e >> 2) + 4 * g + (e & 3);
    lse2[e] = hh < Hm ? lse[(size_t)qi * H + hh] * LOG2E : INFINITY;
  }
  __builtin_amdgcn_sched_barrier(0);
  const int ntiles = stage_ids(ids, qi, K, Skv, q_start + qi, idx_s, tmask, tlist, ntile_s);
  DSA_WAIT_VMCNT(0);
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ks++) asm volatile("" : "+a"(qreg[ks]));
#pragma unroll
  for (int e = 0; e < 16; e++) asm volatile("" : "+v"(lse2[e]));
  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  const LaneOffsets lo = lane_offsets();
  const float c2 = sm_scale * LOG2E;
  auto issue = [&](int n) { gather_tile(kv, idx_s, tlist[n], lds0 + (unsigned)((n % STAGES) * TILE_BYTES)); };
  for (int n = 0; n < STAGES - 1 && n < ntiles; n++) issue(n);
  for (int n = 0; n < ntiles; n++) {
    const int ahead = min(STAGES - 2, ntiles - 1 - n);      // gathers issued after this tile's: 9 operations each
    if (ahead >= 2) { DSA_WAIT_VMCNT(18); } else if (ahead == 1) { DSA_WAIT_VMCNT(9); } else { DSA_WAIT_VMCNT(0); }
    __syncthreads();
    // the next tile's nine transfers go out between the MFMA steps: issued in a row they would hold the
    // wave until the memory pipeline has taken them all
    const bool more = n + STAGES - 1 < ntiles;
    unsigned g_goff = 0, g_lb = 0;
    if (more) {
      const int nn = n + STAGES - 1;
      const int gkey = tid >> 3, gsub = tid & 7;
      int kid = idx_s[tlist[nn] * BI + gkey];
      kid = kid < 0 ? 0 : kid;
      g_goff = (unsigned)kid * (DQK * 2) + (unsigned)((gsub ^ swz(gkey)) * 16);
      g_lb = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)((nn % STAGES) * TILE_BYTES + wave * 1024));
    }
    const int tile = tlist[n];
    const unsigned mask = tmask[tile];
    const unsigned char* tb = smem + (n % STAGES) * TILE_BYTES;
    f32x16 sacc;
    {
      bf16x8 f[4];
#pragma unroll
      for (int ks = 0; ks < 4; ks++) f[ks] = *(const bf16x8*)(tb + (ks >> 2) * GRP_BYTES + lo.row_off[ks & 3]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
        if (ks == 0) mfma_v_av_first(sacc, qreg[0], f[0]);
        else mfma_v_av(sacc, qreg[ks], f[ks & 3]);
        if (ks + 4 < KSTEPS) f[ks & 3] = *(const bf16x8*)(tb + ((ks + 4) >> 2) * GRP_BYTES + lo.row_off[ks & 3]);
        if (ks % 4 == 1 && more) dma16(g_lb + (ks / 4) * GRP_BYTES, g_goff + (ks / 4) * 128, kv);
        __builtin_amdgcn_sched_barrier(0);
      }
      mfma_done_v(sacc);
    }
    const bool valid = (mask >> r) & 1u;
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 16; e++) s += valid ? __builtin_amdgcn_exp2f(fmaf(sacc[e], c2, -lse2[e])) : 0.f;
    s += __shfl_xor(s, 32, 64);
    if (g == 0) part_s[wave * K + tile * BI + r] = s;
  }
  __syncthreads();
  const float inv = 1.0f / (float)Hm;
  for (int t = tid; t < K; t += 256)
    target[(size_t)qi * K + t] = ((part_s[t] + part_s[K + t]) + (part_s[2 * K + t] + part_s[3 * K + t])) * inv;
}

}  // namespace

extern "C" int dsa_attn_dist_qk(const void* q, const void* kv, const int32_t* ids, const float* lse, int S, int H,
                                int heads_in_mean, int Skv, int K, int q_start, float sm_scale, float* target,
                                void* stream) {
  DSA_REQUIRE(S >= 0 && Skv > 0, "dsa_attn_dist_qk: bad sequence sizes S=%d Skv=%d", S, Skv);
  DSA_REQUIRE(H > 0 && H <= 128 && H % 32 == 0, "dsa_attn_dist_qk: head count must be 32, 64, 96 or 128, got %d", H);
  DSA_REQUIRE(heads_in_mean > 0 && heads_in_mean <= H, "dsa_attn_dist_qk: heads_in_mean=%d must be in 1 .. %d", heads_in_mean, H);
  DSA_REQUIRE(K > 0 && K % 64 == 0 && K <= 4096, "dsa_attn_dist_qk: top-k must be a multiple of 64 up to 4096, got %d", K);
  DSA_REQUIRE((size_t)Skv * DQK * 2 <= 0xffffffffull, "dsa_attn_dist_qk: kv larger than 4 GiB is not supported");
  DSA_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)kv % 16) == 0, "dsa_attn_dist_qk: misaligned pointer");
  if (S == 0) return DSA_OK;
  hipStream_t st = (hipStream_t)stream;
  const size_t tail = ids_lds_bytes(K) + 16 + (size_t)4 * K * 4;
  // as many key tiles in flight as LDS allows next to the ids and the partial sums
  const int stages = (size_t)3 * TILE_BYTES + tail <= 160 * 1024 ? 3 : 2;
  const size_t smem = (size_t)stages * TILE_BYTES + tail;
  auto kern = stages == 3 ? attn_dist_qk_kernel<3> : attn_dist_qk_kernel<2>;
  if (dsa_reserve_lds((const void*)kern, smem) != hipSuccess)
    DSA_FAIL(DSA_ERR_LAUNCH, "dsa_attn_dist_qk: cannot reserve %zu bytes of LDS", smem);
  kern<<<dim3(S), dim3(256), smem, st>>>((const __bf16*)q, (const __bf16*)kv, ids, lse, target, H, heads_in_mean, Skv, K,
                                         q_start, sm_scale);
  DSA_CHECK_LAUNCH("dsa_attn_dist_qk");
  return DSA_OK;
}
