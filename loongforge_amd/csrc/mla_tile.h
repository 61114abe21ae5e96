// Pieces shared by the sparse-MLA kernels: the LDS layout of a gathered tile of 32 latent rows,
// the asynchronous gather that fills it, and the per-query list of tiles holding a valid slot.
#pragma once
#include "dsa_common.h"

namespace mla {

constexpr int DQK = 576;
constexpr int DV = 512;
constexpr int BI = 32;                       // keys (slots) per tile
constexpr int TILE_BYTES = BI * DQK * 2;     // 36864
constexpr int GRP_BYTES = BI * 128;          // one 128-byte group of every key row of the tile
constexpr int KSTEPS = DQK / 16;             // 36 MFMA k-steps over d_qk
constexpr int VSTEPS = DV / 16;              // 32 MFMA k-steps over d_v
constexpr float LOG2E = 1.4426950408889634f;

// A key row (1152 bytes) is stored as nine 128-byte groups; group p of all 32 rows is contiguous
// (GRP_BYTES).  Inside a group the 16-byte slot of chunk c of row r is (c & 7) ^ swz(r).  swz
// permutes the bits of r so that (a) the rows of one parity in any aligned block of 16 hit 8
// different slots - 128-bit row reads by 16 lanes are conflict free - and (b) bit 2 of the slot
// follows bit 1 of the row, so the four keys a transpose read touches in a half wave fall into
// four different 64-byte bank regions - transpose reads by 32 lanes are conflict free as well.
__device__ __forceinline__ int swz(int r) {
  return (((r >> 1) & 1) << 2) | (((r >> 2) & 1) << 1) | ((r ^ (r >> 3)) & 1);
}

// Each lane fetches 16 bytes at gbase + goff; the wave's 64 chunks land at lds_base + 16*lane.
// (m0 carries the LDS base; nothing else in these kernels uses m0.)  The transfer is counted by
// the vector-memory counter but invisible to the compiler, which therefore never waits for it:
// callers wait with DSA_WAIT_VMCNT before a barrier.
__device__ __forceinline__ void dma16(unsigned lds_base, unsigned goff, const void* gbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_base), "v"(goff), "s"(gbase) : "memory");
}

// A pointer that is the same for every lane, forced into scalar registers.
template <typename T>
__device__ __forceinline__ const T* uniform_ptr(const T* p) {
  const unsigned long long v = (unsigned long long)p;
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v);
  const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
  return (const T*)(((unsigned long long)hi << 32) | lo);
}

// Stages the K ids of query qi in LDS (invalid slots become -1), builds the 32-bit validity mask
// of every tile and the ordered list of tiles with at least one valid slot.  Returns the number
// of such tiles.  Ends with a barrier.  K % 64 == 0.
__device__ __forceinline__ int stage_ids(const int* __restrict__ ids, int qi, int K, int Skv, int qpos,
                                         int* idx_s, unsigned* tmask, int* tlist, int* ntile_s) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int NT = K / BI;
  for (int t0 = tid; t0 < K; t0 += 8 * 256) {     // eight loads in flight per thread
    int v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = t0 + i * 256 < K ? ids[(size_t)qi * K + t0 + i * 256] : -1;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const bool ok = (v[i] >= 0) && (v[i] < Skv) && (v[i] <= qpos);
      if (t0 + i * 256 < K) idx_s[t0 + i * 256] = ok ? v[i] : -1;
    }
  }
  __syncthreads();
  for (int t2 = wave; t2 * 2 < NT; t2 += 4) {
    int e = t2 * 64 + lane;
    bool ok = idx_s[e] >= 0;
    unsigned long long b = __ballot(ok);
    if (lane == 0) { tmask[2 * t2] = (unsigned)b; tmask[2 * t2 + 1] = (unsigned)(b >> 32); }
  }
  __syncthreads();
  if (wave == 0) {
    int base = 0;
    for (int t0 = 0; t0 < NT; t0 += 64) {
      int t = t0 + lane;
      bool nz = t < NT && tmask[t] != 0u;
      unsigned long long b = __ballot(nz);
      if (nz) tlist[base + __popcll(b & ((1ull << lane) - 1ull))] = t;
      base += __popcll(b);
    }
    if (lane == 0) *ntile_s = base;
  }
  __syncthreads();
  return *ntile_s;
}

// LDS bytes needed by stage_ids' arrays.
__host__ __device__ inline size_t ids_lds_bytes(int K) { return (size_t)K * 4 + (size_t)(K / BI) * 8 + 16; }

// Gather of one tile: thread (key = tid/8, sub = tid%8) moves slot `sub` of each of the 9 groups.
__device__ __forceinline__ void gather_tile(const void* kv, const int* idx_s, int tile, unsigned lds_tile_base) {
  const int tid = threadIdx.x, wave = tid >> 6;
  const int gkey = tid >> 3, gsub = tid & 7;
  int kid = idx_s[tile * BI + gkey];
  kid = kid < 0 ? 0 : kid;
  const unsigned goff = (unsigned)kid * (DQK * 2) + (unsigned)((gsub ^ swz(gkey)) * 16);
  const unsigned lb = __builtin_amdgcn_readfirstlane(lds_tile_base + (unsigned)(wave * 1024));
#pragma unroll
  for (int grp = 0; grp < 9; grp++) dma16(lb + grp * GRP_BYTES, goff + grp * 128, kv);
}

// Tile-relative LDS byte offsets for this lane.
//   row_off[j]: 128-bit read of row (lane & 31), chunk c with (c & 7) == 2*j + (lane >> 5); add
//               (c >> 3) * GRP_BYTES.  This is the MFMA operand "32 rows x 16 contiguous d".
//   tr_off[s][t][par]: ds_read_b64_tr_b16 address for the transposed operand "32 columns (d) x 16
//               keys": keys 16s + 8t + 4g + (0..3), d columns 32*dt + (lane & 31) with par = dt & 1;
//               add (dt >> 1) * GRP_BYTES.  Two reads (t = 0, 1) give a lane its 8 keys of step s.
struct LaneOffsets {
  unsigned row_off[4];
  unsigned tr_off[2][2][2];
};
__device__ __forceinline__ LaneOffsets lane_offsets() {
  LaneOffsets o;
  const int lane = threadIdx.x & 63, r = lane & 31, g = lane >> 5;
#pragma unroll
  for (int j = 0; j < 4; j++) o.row_off[j] = (unsigned)(r * 128 + (((2 * j + g) ^ swz(r)) << 4));
  const int blk = lane >> 4, ii = lane & 15;
  const int cl = 2 * (blk & 1) + ((ii & 3) >> 1), half = ii & 1;
#pragma unroll
  for (int s = 0; s < 2; s++)
#pragma unroll
    for (int t = 0; t < 2; t++) {
      const int key = 16 * s + 8 * t + 4 * g + (ii >> 2);
#pragma unroll
      for (int par = 0; par < 2; par++)
        o.tr_off[s][t][par] = (unsigned)(key * 128 + (((4 * par + cl) ^ swz(key)) << 4) + half * 8);
    }
  return o;
}

// ---------------------------------------------------------------------------------------------
// MFMA through inline asm with explicit register files ("v" architectural, "a" accumulation).
// Back-to-back MFMAs accumulating into the same registers need no software wait states; whoever
// reads a finished accumulator with a non-MFMA instruction calls mfma_done first.
// ---------------------------------------------------------------------------------------------
#define DSA_MFMA_FN(name, ACC, A, B)                                                              \
  __device__ __forceinline__ void name##_first(f32x16& acc, const bf16x8& a, const bf16x8& b) {   \
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&" ACC(acc) : A(a), B(b));           \
  }                                                                                               \
  __device__ __forceinline__ void name(f32x16& acc, const bf16x8& a, const bf16x8& b) {           \
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+" ACC(acc) : A(a), B(b));           \
  }
DSA_MFMA_FN(mfma_v_av, "v", "a", "v")   // acc VGPR, A in AGPR, B in VGPR
DSA_MFMA_FN(mfma_v_vv, "v", "v", "v")
DSA_MFMA_FN(mfma_a_vv, "a", "v", "v")
DSA_MFMA_FN(mfma_a_av, "a", "a", "v")
#undef DSA_MFMA_FN
__device__ __forceinline__ void mfma_done_v(f32x16& acc) { asm volatile("s_nop 15\n\ts_nop 3" : "+v"(acc)); }
__device__ __forceinline__ void mfma_done_a(f32x16& acc) { asm volatile("s_nop 15\n\ts_nop 3" : "+a"(acc)); }


}  // namespace mla
