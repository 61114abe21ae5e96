// Sparse MQA-MLA attention backward for gfx950, deterministic.
//
// Per (query, selected key) pair the backward needs five products:
//   S  = Q.KV^T (576)   dP = dO.V^T (512)   dQ += dS.KV (576)   dKV[key] += dS^T.Q (576) + P^T.dO (512)
// The operands Q and dO of one query (278 KB in bf16) plus the fp32 dQ accumulators (295 KB) do
// not fit one compute unit (512 KB of registers, 160 KB of LDS) next to the gathered key tiles, and
// the products over d and over heads need the same operands in two register orientations.  The
// work is therefore split into passes that each keep ONE orientation resident in registers:
//   pass A  (bwd_pds_kernel)   S and dP per 32-key tile -> P and dS, written to HBM as bf16 in the
//                              exact MFMA operand layout of pass C (16 KB per query and tile)
//   pass B  (bwd_dq_kernel)    dQ^T += KV^T.dS^T, both operands by LDS transpose reads
//   pass C  (bwd_dkv_kernel)   per-pair rows  dS^T.Q + P^T.dO  (sum over all 128 heads) -> one
//                              bf16 row of 576 values
//                              in a pair buffer, at the position given by a key-sorted order
//   pass D  (bwd_reduce_kernel) dKV[key] = sum of that key's rows, in ascending query order
// The key-sorted order (pass 0) comes from a bitmap key x query, its row-wise prefix popcounts and
// an exclusive scan over keys: integer work only, so the order - and with it every fp32 sum - is
// identical from run to run.  No floating-point atomics anywhere.
#include "mla_tile.h"
#include "order.h"

namespace {
using namespace mla;

constexpr int PDS_TILE_BYTES = 16384;        // P and dS of one (query, tile): 2 x [16 chunk groups][32 keys][8 heads] bf16
constexpr int PDS_KIND_BYTES = 8192;
constexpr int ROW_BYTES = DQK * 2;           // one pair row of the dKV buffer
constexpr int PDS_THREADS = 512;

// ---------------------------------------------------------------------------------------------
// pass A: P and dS of every (query, tile)
// ---------------------------------------------------------------------------------------------
// One workgroup of eight waves per query; wave w owns heads [16w, 16w+16).  S = Q.KV^T and dP = dO.V^T
// are 16x16x32 MFMAs with the heads on the rows (Q and dO rows resident in registers, 8 d-values per
// lane and step) and the 16 keys of a half tile on the columns (key rows read from LDS, one 1 KB read
// feeding both products).  At under 256 registers per lane two waves share a SIMD.  Measured against
// four waves of 32 heads with 32x32x16 MFMAs (one wave per SIMD, half the LDS reads): the backward
// takes 14.5 instead of 15.1 ms; LDS reads (288 KB per tile) and the MFMAs (2176 clocks per tile and
// SIMD) are then about level.  A lane ends with 4 heads x 2 half tiles; lanes 32 apart trade halves
// (one v_permlane32_swap per register pair) so that every lane holds one key's 8 heads in the chunk
// order pass C reads: chunk group 2w + g = heads 16w + {4g .. 4g+3, 8+4g .. 8+4g+3}.
template <int STAGES>
__device__ __forceinline__ void pds_body(
    const __bf16* __restrict__ q, const __bf16* __restrict__ kv, const int* __restrict__ ids,
    const __bf16* __restrict__ out, const __bf16* __restrict__ dout, const float* __restrict__ lse,
    unsigned char* __restrict__ pds, int q0, int ql, int H, int Skv, int K, int q_start, float sm_scale,
    unsigned char* smem) {
  constexpr int KS = DQK / 32, VS = DV / 32;   // 18 and 16 steps of 32 d-values
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m = lane & 15, kg = lane >> 4;
  const int qi = q0 + ql;
  const int NT = K / BI;
  int* idx_s = (int*)(smem + STAGES * TILE_BYTES);
  unsigned* tmask = (unsigned*)(idx_s + K);
  int* tlist = (int*)(tmask + NT);
  int* ntile_s = tlist + NT;
  float* stat_s = (float*)(ntile_s + 4);       // [2][128]: lse * log2(e), delta
  // All of the query's rows are requested before the ids are staged: one round trip to memory for
  // both, instead of one after the other.
  const int h = wave * 16 + m;
  const bool head_ok = h < H;
  const size_t hrow = (size_t)qi * H + (head_ok ? h : 0);
  bf16x8 qreg[KS], doreg[VS], oreg[VS];
  {
    const bf16x8* qp = (const bf16x8*)(q + hrow * DQK) + kg;
    const bf16x8* dp = (const bf16x8*)(dout + hrow * DV) + kg;
    const bf16x8* op = (const bf16x8*)(out + hrow * DV) + kg;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qreg[ks] = qp[4 * ks];
#pragma unroll
    for (int ks = 0; ks < VS; ks++) doreg[ks] = dp[4 * ks];
#pragma unroll
    for (int ks = 0; ks < VS; ks++) oreg[ks] = op[4 * ks];
  }
  const float lse_h = lse[hrow];
  __builtin_amdgcn_sched_barrier(0);
  // (the helper is written for four waves; the other four repeat part of its work with equal results)
  const int ntiles = stage_ids(ids, ql, K, Skv, q_start + qi, idx_s, tmask, tlist, ntile_s);
  // Q and part of dO live in accumulation registers, which MFMA reads directly
#pragma unroll
  for (int ks = 0; ks < KS; ks++) asm volatile("" : "+a"(qreg[ks]));
#pragma unroll
  for (int ks = 0; ks < VS; ks++) {
    if (ks < 6) asm volatile("" : "+a"(doreg[ks]));
    else asm volatile("" : "+v"(doreg[ks]));
  }
#pragma unroll
  for (int ks = 0; ks < VS; ks++) asm volatile("" : "+v"(oreg[ks]));

  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  // transfers of a tile: thread (key, sub) of either half of the workgroup moves 16 bytes of a 128-byte
  // group of the key's row; waves 0-3 take groups 0-4, waves 4-7 groups 5-8 (a fifth step does nothing)
  const int hh = wave >> 2;
  const int gkey = (tid & 255) >> 3, gsub = tid & 7;
  // Within a 128-byte group the 16-byte chunk c of key row r sits in slot c ^ (r & 7).  (The slot function of
  // the other kernels' tiles also serves their transposing reads; with it this kernel's reads - 16 rows x 4
  // chunks per instruction - take two LDS cycles where one is needed.)
  const unsigned gslot = (unsigned)((gsub ^ (gkey & 7)) * 16) + (unsigned)(hh * 5 * 128);
  unsigned t_goff = 0, t_lb = 0;
  auto issue_prepare = [&](int n) {
    const int tile = tlist[n];
    int kid = idx_s[tile * BI + gkey];
    kid = kid < 0 ? 0 : kid;
    t_goff = (unsigned)kid * (DQK * 2) + gslot;
    t_lb = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)((n % STAGES) * TILE_BYTES + (wave & 3) * 1024 + hh * 5 * GRP_BYTES));
  };
  auto issue_step = [&](int i) {
    if (hh == 0 || i < 4) dma16(t_lb + i * GRP_BYTES, t_goff + i * 128, kv);
  };
  for (int n = 0; n < STAGES - 1 && n < ntiles; n++) {
    issue_prepare(n);
#pragma unroll
    for (int i = 0; i < 5; i++) issue_step(i);
  }
  // delta = rowsum(O . dO) while the first tiles travel
  {
    float part = 0.f;
#pragma unroll
    for (int ks = 0; ks < VS; ks++)
#pragma unroll
      for (int e = 0; e < 8; e++) part = fmaf((float)oreg[ks][e], (float)doreg[ks][e], part);
    part += __shfl_xor(part, 16, 64);
    part += __shfl_xor(part, 32, 64);
    if (kg == 0) {
      stat_s[h] = head_ok ? lse_h * LOG2E : INFINITY;
      stat_s[128 + h] = head_ok ? part : 0.f;
    }
  }
  __syncthreads();
  // accumulator i of a lane is head 16*wave + 4*kg + i, for key 16*kt + m
  const f32x4 lse2 = *(const f32x4*)(stat_s + wave * 16 + 4 * kg);
  const f32x4 delta = *(const f32x4*)(stat_s + 128 + wave * 16 + 4 * kg);

  // key-row operand of half tile kt and step ks: row 16*kt + m, 16-byte chunk 4*ks + kg of the row
  unsigned boff[2][2];
#pragma unroll
  for (int kt = 0; kt < 2; kt++)
#pragma unroll
    for (int par = 0; par < 2; par++) {
      const int row = 16 * kt + m;
      boff[kt][par] = (unsigned)(row * 128 + (((4 * par + kg) ^ (row & 7)) << 4));
    }
  const float c2 = sm_scale * LOG2E;

  f32x4 sacc[2], dpacc[2];
  // P and dS of the accumulated tile: the lane's 4 heads for its key of either half tile are two
  // registers (4 bf16) each
  auto finish = [&](int tile, unsigned mask) {
    unsigned pw[2][2], dw[2][2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
      const bool valid = (mask >> (16 * kt + m)) & 1u;
      float pf[4], df[4];
#pragma unroll
      for (int i = 0; i < 4; i++) {
        pf[i] = valid ? __builtin_amdgcn_exp2f(fmaf(sacc[kt][i], c2, -lse2[i])) : 0.f;
        df[i] = pf[i] * (dpacc[kt][i] - delta[i]) * sm_scale;
      }
      pw[kt][0] = cvt_pk_bf16(pf[0], pf[1]); pw[kt][1] = cvt_pk_bf16(pf[2], pf[3]);
      dw[kt][0] = cvt_pk_bf16(df[0], df[1]); dw[kt][1] = cvt_pk_bf16(df[2], df[3]);
    }
    // lanes 32 apart trade: the lower lane keeps half tile 0 and gets the partner's heads of it, the
    // upper lane keeps half tile 1.  Afterwards (x[0], x[1]) is the chunk of key 16*(lane/32) + m:
    // heads 4g .. 4g+3 then 8+4g .. 8+4g+3 of the wave's 16, g = kg & 1.
#pragma unroll
    for (int r2 = 0; r2 < 2; r2++) {
      swap_halves(pw[0][r2], pw[1][r2]);
      swap_halves(dw[0][r2], dw[1][r2]);
    }
    const int key = 16 * (lane >> 5) + m, g = kg & 1;
    unsigned char* base = pds + ((size_t)ql * NT + tile) * PDS_TILE_BYTES + (size_t)(2 * wave + g) * 512 + key * 16;
    *(uint4*)base = make_uint4(dw[0][0], dw[0][1], dw[1][0], dw[1][1]);
    *(uint4*)(base + PDS_KIND_BYTES) = make_uint4(pw[0][0], pw[0][1], pw[1][0], pw[1][1]);
  };

  // Between two barriers every wave runs the MFMAs of one tile and one `finish`; waves 0-3 finish the
  // tile they just accumulated, waves 4-7 first finish the previous one.  The two waves of a SIMD (w and
  // w + 4) are thus half a step apart: the arithmetic and stores of one run under the other's MFMAs.
  int tile = 0;
  unsigned mask = 0;
  for (int n = 0; n < ntiles; n++) {
    // operations a lane issued after this tile's transfers: D per later tile in flight (5 in waves
    // 0-3, 4 in waves 4-7), 2 stores per finished tile (waves 4-7 are one tile behind with those)
    {
      const int ahead = min(STAGES - 2, ntiles - 1 - n);
      if (hh == 0) {
        constexpr int D = 5;
        const int behind = min(n, STAGES - 1);
        if (ahead == STAGES - 2 && behind == STAGES - 1) { DSA_WAIT_VMCNT(D * (STAGES - 2) + 2 * (STAGES - 1)); }
        else if (ahead == STAGES - 2) { DSA_WAIT_VMCNT(D * (STAGES - 2)); }
        else if (ahead >= 1) { DSA_WAIT_VMCNT(D); }
        else { DSA_WAIT_VMCNT(0); }
      } else {
        constexpr int D = 4;             // (their stores of a step come before its transfers)
        const int behind = min(n - 1, STAGES - 2);
        if (ahead == STAGES - 2 && behind == STAGES - 2) { DSA_WAIT_VMCNT(D * (STAGES - 2) + 2 * (STAGES - 2)); }
        else if (ahead == STAGES - 2) { DSA_WAIT_VMCNT(D * (STAGES - 2)); }
        else if (ahead >= 1) { DSA_WAIT_VMCNT(D); }
        else { DSA_WAIT_VMCNT(0); }
      }
    }
    __syncthreads();
    // the next tile's transfers go out one at a time between the MFMA steps below: issued together they
    // would hold every wave at the address unit, which takes 64 bytes per clock for the compute unit
    const bool more = n + STAGES - 1 < ntiles;
    if (more) issue_prepare(n + STAGES - 1);
    const int prev_tile = tile;
    const unsigned prev_mask = mask;
    tile = __builtin_amdgcn_readfirstlane(tlist[n]);
    mask = __builtin_amdgcn_readfirstlane(tmask[tile]);
    if (hh == 1 && n > 0) finish(prev_tile, prev_mask);
    __builtin_amdgcn_sched_barrier(0);
    const unsigned char* tb = smem + (n % STAGES) * TILE_BYTES;
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int e = 0; e < 4; e++) { sacc[kt][e] = 0.f; dpacc[kt][e] = 0.f; }
    {
      // step j = 2 * ks + kt; FD operand reads in flight
      constexpr int FD = 4;
      bf16x8 f[FD];
#pragma unroll
      for (int j = 0; j < FD; j++) f[j] = *(const bf16x8*)(tb + ((j >> 1) >> 1) * GRP_BYTES + boff[j & 1][(j >> 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < 2 * KS; j++) {
        const int ks = j >> 1, kt = j & 1;
        sacc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qreg[ks], f[j % FD], sacc[kt], 0, 0, 0);
        if (ks < VS) dpacc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(doreg[ks], f[j % FD], dpacc[kt], 0, 0, 0);
        if (j + FD < 2 * KS) {
          const int j2 = j + FD, ks2 = j2 >> 1;
          f[j % FD] = *(const bf16x8*)(tb + (ks2 >> 1) * GRP_BYTES + boff[j2 & 1][ks2 & 1]);
        }
        if (j % 7 == 2 && more) issue_step(j / 7);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (hh == 0) finish(tile, mask);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (hh == 1 && ntiles > 0) finish(tile, mask);
}

// ---------------------------------------------------------------------------------------------
// pass B: dQ
// ---------------------------------------------------------------------------------------------
// dQ^T[d, head] += KV^T[d, key] . dS^T[key, head] per 32-key tile.  Both operands are LDS transpose
// reads: of the gathered key tile (18 d-tiles) and of the tile's dS block copied verbatim from the
// pass-A buffer.  Twelve waves share the 72 accumulator tiles (18 d-tiles x 4 head groups): wave
// (dg, hp) = (wave % 6, wave / 6) owns d-tiles 3dg .. 3dg+2 for the head groups 2hp, 2hp+1: 6 tiles
// (96 accumulator registers), 12 MFMAs and 20 transposing reads per wave and tile.  A wave issues one
// LDS instruction per 40-odd cycles whatever its width, and a transposing read carries 8 bytes per
// lane: with eight waves (9 tiles, 28 reads each) the reads of a wave took longer than the MFMAs of
// the two waves of a SIMD together (1 200 against 1 152 cycles per tile).  Three waves per SIMD at
// under 168 registers per lane issue them in two thirds of the time, and one wave's transfer issue and
// waits run under the MFMAs of the other two.
constexpr int DQ_THREADS = 768;
template <int STAGES>
__device__ __forceinline__ void dq_body(
    const __bf16* __restrict__ kv, const int* __restrict__ ids, const unsigned char* __restrict__ pds,
    __bf16* __restrict__ dq, int q0, int ql, int H, int Skv, int K, int q_start, const int* __restrict__ dup_flag,
    unsigned char* smem) {
  constexpr int STAGE_BYTES = TILE_BYTES + PDS_KIND_BYTES;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int dg = wave % 6, hp = wave / 6;
  const int r = lane & 31, g = lane >> 5;
  const int qi = q0 + ql;
  const int NT = K / BI;
  int* idx_s = (int*)(smem + STAGES * STAGE_BYTES);
  unsigned* tmask = (unsigned*)(idx_s + K);
  int* tlist = (int*)(tmask + NT);
  int* ntile_s = tlist + NT;
  // (the helper is written for four waves; the others repeat part of its work with equal results)
  const int ntiles = stage_ids(ids, ql, K, Skv, q_start + qi, idx_s, tmask, tlist, ntile_s);

  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  // transposed read of the dS block: lane (blk, ii) points at key 16s + 8t + 4g + ii/4 and the 4 heads
  // 16*(blk&1) + 4*(ii&3) .. +3 of a head group.  In HBM the block is [head group][s'][g'][key][8 heads];
  // in LDS the 16-byte pieces of a head group are reordered to [key][s'][g'], so that the 16 pieces a
  // half-wave reads at once (4 keys x 4 head octets) are 256 consecutive bytes: no bank conflicts.
  unsigned ds_off[2][2];
  // transposed read of the key tile for the wave's d-tiles 3dg + i (same formula as LaneOffsets::tr_off,
  // with the parity of the d-tile known only at run time)
  unsigned a_off[3][2][2];
  {
    const int blk = lane >> 4, ii = lane & 15, qq = ii & 3;
    const int cl = 2 * (blk & 1) + ((ii & 3) >> 1), half = ii & 1;
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const int key = 16 * s + 8 * t + 4 * g + (ii >> 2);
        ds_off[s][t] = (unsigned)(TILE_BYTES + key * 64 + (blk & 1) * 32 + (qq & 1) * 16 + (qq >> 1) * 8);
#pragma unroll
        for (int i = 0; i < 3; i++) {
          const int dt = 3 * dg + i;
          a_off[i][s][t] = (unsigned)((dt >> 1) * GRP_BYTES + key * 128 + (((4 * (dt & 1) + cl) ^ swz(key)) << 4) + half * 8);
        }
      }
  }
  // Transfers of a tile: 44 of 1 KB each.  Transfer t < 36 is slot t % 4 (keys 8*slot .. +7, thread (key,
  // sub) moving 16 bytes) of the 128-byte group t / 4 of the key rows; transfer 36 + b is 1 KB of the dS
  // block, piece P of the LDS order coming from piece src_piece(P) of the HBM order.  Wave v takes
  // transfers v, v + 12, v + 24 (groups v/4, v/4 + 3, v/4 + 6 of its slot v % 4) and, for v < 8, 36 + v.
  auto src_piece = [](int P) { return (P >> 7) * 128 + ((P >> 1) & 1) * 64 + (P & 1) * 32 + ((P >> 2) & 31); };
  const unsigned ds_src = (unsigned)src_piece((wave & 7) * 64 + lane) * 16u;
  const int gkey = 8 * (wave & 3) + (lane >> 3), gsub = lane & 7;
  const unsigned gslot = (unsigned)((gsub ^ swz(gkey)) * 16) + (unsigned)((wave >> 2) * 128);
  unsigned t_goff = 0, t_lb = 0, t_lbd = 0;
  const unsigned char* t_src = nullptr;
  auto issue_prepare = [&](int n) {
    const int tile = tlist[n];
    const unsigned sb = lds0 + (unsigned)((n % STAGES) * STAGE_BYTES);
    int kid = idx_s[tile * BI + gkey];
    kid = kid < 0 ? 0 : kid;
    t_goff = (unsigned)kid * (DQK * 2) + gslot;
    t_lb = __builtin_amdgcn_readfirstlane(sb + (unsigned)((wave & 3) * 1024 + (wave >> 2) * GRP_BYTES));
    t_lbd = __builtin_amdgcn_readfirstlane(sb + (unsigned)(TILE_BYTES + (wave & 7) * 1024));
    t_src = uniform_ptr(pds + ((size_t)ql * NT + tile) * PDS_TILE_BYTES);     // dS half
  };
  // step 0 .. 2: the wave's three groups of the key rows; step 3: its part of the dS block (waves 0-7)
  auto issue_step = [&](int j) {
    if (j < 3) dma16(t_lb + 3 * j * GRP_BYTES, t_goff + 3 * j * 128, kv);
    else if (wave < 8) dma16(t_lbd, ds_src, t_src);
  };

  const int hg0 = 2 * hp, hg1 = 2 * hp + 1;
  f32x16 acc[6];      // u = 2 * i + j: d-tile 3dg + i, head group 2hp + j
#pragma unroll
  for (int u = 0; u < 6; u++)
#pragma unroll
    for (int e = 0; e < 16; e++) acc[u][e] = 0.f;
  typedef short i16x8 __attribute__((ext_vector_type(8)));
  auto tr_pair = [&](const unsigned char* p0, const unsigned char* p1) {
    const i16x4 x0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, p0));
    const i16x4 x1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, p1));
    return __builtin_bit_cast(bf16x8, (i16x8)__builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7));
  };
  for (int n = 0; n < STAGES - 1 && n < ntiles; n++) {
    issue_prepare(n);
#pragma unroll
    for (int j = 0; j < 4; j++) issue_step(j);
  }
  for (int n = 0; n < ntiles; n++) {
    static_assert(STAGES == 3, "one tile of transfers in flight behind the awaited one");
    // transfers per wave and tile: 4 for waves 0-7, 3 for waves 8-11
    if (n + 1 < ntiles) { if (wave < 8) { DSA_WAIT_VMCNT(4); } else { DSA_WAIT_VMCNT(3); } } else { DSA_WAIT_VMCNT(0); }
    __syncthreads();
    const bool more = n + STAGES - 1 < ntiles;
    if (more) { issue_prepare(n + STAGES - 1); issue_step(3); }
    const unsigned char* tb = smem + (n % STAGES) * STAGE_BYTES;
    // key-tile operands one d-tile ahead, the four dS operands of the wave's two head groups: [hg0 or hg1][k-step]
    bf16x8 a[2][2], bds[2][2];
#pragma unroll
    for (int s = 0; s < 2; s++) a[0][s] = tr_pair(tb + a_off[0][s][0], tb + a_off[0][s][1]);
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int s = 0; s < 2; s++)
        bds[j][s] = tr_pair(tb + (j ? hg1 : hg0) * 2048 + ds_off[s][0], tb + (j ? hg1 : hg0) * 2048 + ds_off[s][1]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < 3; i++) {
      if (i + 1 < 3) {
#pragma unroll
        for (int s = 0; s < 2; s++) a[(i + 1) & 1][s] = tr_pair(tb + a_off[i + 1][s][0], tb + a_off[i + 1][s][1]);
      }
#pragma unroll
      for (int s = 0; s < 2; s++)
#pragma unroll
        for (int j = 0; j < 2; j++)
          acc[2 * i + j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i & 1][s], bds[j][s], acc[2 * i + j], 0, 0, 0);
      if (more) issue_step(i);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  // ---- write dQ: accumulator e of a lane is d = 32*dt + 8*(e/4) + 4*g + (e%4), head = 32*hg + r ----
  const bool poison = *dup_flag != 0;          // a query row with a repeated id: NaN instead of a sum that misses a term
#pragma unroll
  for (int u = 0; u < 6; u++) {
    const int dt = 3 * dg + (u >> 1);
    const int hg = (u & 1) ? hg1 : hg0;
    const int h = hg * 32 + r;
    if (h < H) {                               // the same for all lanes of a wave (H is a multiple of 32)
      unsigned short* op = (unsigned short*)dq + ((size_t)qi * H + h) * DQK + 32 * dt + 8 * g;
      uint4 o[2];
      acc_row_to_16B(acc[u], 1.0f, o);
      if (poison) o[0] = o[1] = make_uint4(0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u, 0x7fc07fc0u);
      *(uint4*)op = o[0];
      *(uint4*)(op + 16) = o[1];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// pass C: per-pair dKV rows
// ---------------------------------------------------------------------------------------------
// row[key, d] = sum_h dS[h,key] Q[h,d] + (d < 512) sum_h P[h,key] dO[h,d], all 128 heads, as
// row^T = X^T . coef with X = [Q; dO] (k = heads).  X^T is the register-resident operand: wave w
// owns the 32-column d-tiles {w, w+4, w+8, w+12, w+16} (the last only for w < 2) and loads its
// columns once per query through LDS transpose reads.  The 16 coefficient operands of a tile
// (pass-A layout, read from LDS as stored) also sit in registers, so a column tile is finished by
// 16 (or 8) back-to-back MFMAs on one accumulator.  Everything else runs in the shadow of the
// matrix pipe, a few instructions after each MFMA: while column tile c+1 accumulates, tile c is
// rounded to bf16, its four 8-byte pieces per lane are turned into two 16-byte pieces by a trade
// between the half-waves (the accumulator already holds one key per lane), and these are stored
// as 32-byte halves of the tile's 64 bytes in each of its 32 rows, at the positions of the
// key-sorted order; while the last column tile of a tile accumulates, the coefficient registers are
// refilled for the next tile.  The loop touches LDS for the coefficients only (16 reads per wave
// and tile).  One barrier per tile (the coefficient transfer is shared by the four waves); the
// per-pair rows are bf16.
constexpr int DKV_COEF_STAGES = 5;           // coefficient tiles in the LDS ring

// NC = column tiles of this wave (5 for waves 0 and 1, else 4).
template <int NC>
__device__ __forceinline__ void dkv_body(
    const __bf16* __restrict__ q, const __bf16* __restrict__ dout, const int* __restrict__ ids,
    const unsigned char* __restrict__ pds, const int* __restrict__ dst, unsigned char* __restrict__ rows,
    int q0, int ql, int H, int Skv, int K, int q_start, int dummy_row, unsigned char* smem) {
  constexpr int CST = DKV_COEF_STAGES;
  constexpr int NU = NC == 5 ? 9 : 8;          // units of 8 MFMAs per tile
  // [CST][PDS_TILE_BYTES] coefficient ring, shared with the set-up's per-wave X staging [4][8192] |
  // ids arrays | dst rows of the query [K + 32]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int qi = q0 + ql;
  const int NT = K / BI;
  unsigned char* xs = smem + wave * 8192;
  int* idx_s = (int*)(smem + CST * PDS_TILE_BYTES);
  unsigned* tmask = (unsigned*)(idx_s + K);
  int* tlist = (int*)(tmask + NT);
  int* ntile_s = tlist + NT;
  int* dst_s = ntile_s + 4;
  for (int t0 = tid; t0 < K + BI; t0 += 8 * 256) {   // eight loads in flight per thread
    int d[8];
#pragma unroll
    for (int i = 0; i < 8; i++) d[i] = t0 + i * 256 < K ? dst[(size_t)ql * K + t0 + i * 256] : -1;
#pragma unroll
    for (int i = 0; i < 8; i++)       // invalid slots land in a scratch row: the store count stays fixed
      if (t0 + i * 256 < K + BI) dst_s[t0 + i * 256] = d[i] >= 0 ? d[i] : dummy_row;
  }
  const int ntiles = stage_ids(ids, ql, K, Skv, q_start + qi, idx_s, tmask, tlist, ntile_s);
  if (ntiles == 0) return;

  // ---- X^T operands: x?[c][kk], kk = 2*w' + s' over the 8 groups of 16 heads ------------------
  // Q columns 0..3 and all dO columns live in accumulation registers (MFMA reads them there), the
  // fifth Q column, the coefficients and the accumulators in architectural registers.
  bf16x8 xqa[4][8], xqv[8], xo[4][8];
  {
    typedef short i16x8 __attribute__((ext_vector_type(8)));
    const int blk = lane >> 4, ii = lane & 15;
    // transpose read of a [128 heads][32 d] block (64-byte rows): lane points at head
    // 32w' + 8(2s'+t) + 4g + ii/4, d chunk 16*(blk&1) + 4*(ii&3)
    const unsigned xoff = (unsigned)((4 * g + (ii >> 2)) * 64 + (16 * (blk & 1) + 4 * (ii & 3)) * 2);
    constexpr int NP = NC + 4;                 // passes: Q column tiles, then dO column tiles
    uint4 ld[3][8];                            // three passes of global loads in flight
    auto pass_load = [&](int pass, uint4 (&dstv)[8]) {
      const bool isq = pass < NC;
      const int ci = isq ? pass : pass - NC;
      const int c = wave + 4 * ci;
      const __bf16* src = isq ? q + (size_t)qi * H * DQK + 32 * c : dout + (size_t)qi * H * DV + 32 * c;
      const int stride = isq ? DQK : DV;
      // rows of 64 bytes: lane covers head (lane/4 + 16*it), 16-byte piece lane%4
#pragma unroll
      for (int it = 0; it < 8; it++) {
        const int hh = (lane >> 2) + 16 * it;
        dstv[it] = make_uint4(0, 0, 0, 0);
        if (hh < H) dstv[it] = *(const uint4*)(src + (size_t)hh * stride + (lane & 3) * 8);
      }
    };
    pass_load(0, ld[0]);
    pass_load(1, ld[1]);
    pass_load(2, ld[2]);
#pragma unroll
    for (int pass = 0; pass < NP; pass++) {
      const bool isq = pass < NC;
      const int ci = isq ? pass : pass - NC;
#pragma unroll
      for (int it = 0; it < 8; it++) *(uint4*)(xs + ((lane >> 2) + 16 * it) * 64 + (lane & 3) * 16) = ld[pass % 3][it];
      if (pass + 3 < NP) pass_load(pass + 3, ld[pass % 3]);
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int kk = 0; kk < 8; kk++) {
        const unsigned char* hb = xs + (32 * (kk >> 1) + 16 * (kk & 1)) * 64;
        i16x4 x0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, hb + xoff));
        i16x4 x1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, hb + 8 * 64 + xoff));
        const bf16x8 val = __builtin_bit_cast(bf16x8, (i16x8)__builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7));
        if (!isq) xo[ci][kk] = val;
        else if (ci < 4) xqa[ci][kk] = val;
        else xqv[kk] = val;
      }
      __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int kk = 0; kk < 8; kk++) {
#pragma unroll
      for (int ci = 0; ci < 4; ci++) asm volatile("" : "+a"(xqa[ci][kk]));
      if (NC == 5) asm volatile("" : "+v"(xqv[kk]));
#pragma unroll
      for (int ci = 0; ci < 4; ci++) asm volatile("" : "+a"(xo[ci][kk]));
    }
  }
  __syncthreads();                             // the X staging shares LDS with the coefficient ring

  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  auto issue = [&](int n) {
    const unsigned lb = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)((n % CST) * PDS_TILE_BYTES + wave * 1024));
    const unsigned char* src = uniform_ptr(pds + ((size_t)ql * NT + tlist[n]) * PDS_TILE_BYTES);
#pragma unroll
    for (int c = 0; c < 4; c++) dma16(lb + c * 4096, (unsigned)(c * 4096 + tid * 16), src);
  };
  // Vector-memory operations retire in issue order, so "the transfer of tile t has landed" is a
  // bound on the number of operations issued after it: `issued` counts every operation of this
  // wave, mk[j] is the count right after the transfer of the (j+1)-th tile ahead.  Stores younger
  // than the awaited transfer stay in flight: the deeper the ring, the more of them.
  int issued = 0;
  int mk[CST - 1];
#pragma unroll
  for (int j = 0; j < CST - 1; j++) mk[j] = 0;
  auto issue_marked = [&](int n) {
    if (n < ntiles) {
      issue(n);
      issued += 4;
    }
    return issued;
  };
  // coefficient chunk of k-step kk: [kind][kk][g][key r] 16 bytes
  const unsigned coff = (unsigned)(g * 512 + r * 16);
  bf16x8 cf[16];
  issue_marked(0);
  mk[0] = issue_marked(1);
  if (ntiles > 1) { DSA_WAIT_VMCNT(4); } else { DSA_WAIT_VMCNT(0); }
  __syncthreads();
#pragma unroll
  for (int j = 1; j < CST - 1; j++) mk[j] = issue_marked(j + 1);
#pragma unroll
  for (int k = 0; k < 16; k++) cf[k] = *(const bf16x8*)(smem + k * 1024 + coff);

  // copy-out state: the rounded column tile in flight (four 8-byte pieces, then two 16-byte ones) and
  // the pointer to this lane's 16 bytes in the row of its key (lane & 31), first column tile of the wave
  const size_t lane_off = (size_t)(wave * 64 + g * 16);
  unsigned char* rptr = rows + (size_t)dummy_row * ROW_BYTES + lane_off;
  unsigned pc[4][2];
#pragma unroll
  for (int j = 0; j < 4; j++) pc[j][0] = pc[j][1] = 0u;
  uint4 piece[2] = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
  f32x16 acc[5];
#pragma unroll
  for (int e = 0; e < 16; e++) acc[NC - 1][e] = 0.f;   // rounded (to the scratch row) before its first MFMA

  // tasks of column tile ci, spread over MFMA slots: round (4 slots), trade between the half-waves
  // (2 slots: piece it = elements 16*it + 8*g .. +7 of the lane's key), store (2 slots of the following unit)
  auto conv = [&](int ci, int j) {
    pc[j][0] = cvt_pk_bf16(acc[ci][4 * j], acc[ci][4 * j + 1]);
    pc[j][1] = cvt_pk_bf16(acc[ci][4 * j + 2], acc[ci][4 * j + 3]);
  };
  auto piece_read = [&](int it) {
    const int jj = 2 * it;
    swap_halves(pc[jj][0], pc[jj + 1][0]);
    swap_halves(pc[jj][1], pc[jj + 1][1]);
    piece[it] = make_uint4(pc[jj][0], pc[jj][1], pc[jj + 1][0], pc[jj + 1][1]);
  };
  auto piece_store = [&](int ci, int it) {
    *(uint4*)(rptr + ci * 256 + it * 32) = piece[it];
    issued += 1;
  };
  // Operations a wave has issued, in the steady state, since the transfer it waits for at unit 6 of a
  // tile (that of the next tile, issued CST - 1 tiles earlier): the stores of unit 7 (and 8) of that
  // tile, CST - 2 whole tiles of 4 transfers + 2 NC stores, and this tile's stores before unit 6.
  constexpr int STEADY = 2 + (CST - 2) * (4 + 2 * NC) + (NC == 5 ? 8 : 6);
  static_assert(STEADY <= 63, "the vector-memory counter holds 63 at most");

  for (int n = 0; n < ntiles; n++) {
    const int tile = tlist[n];
    const int drow = dst_s[tile * BI + r];
    const unsigned char* nb = smem + ((n + 1) % CST) * PDS_TILE_BYTES;   // next tile's coefficients
#pragma unroll
    for (int u = 0; u < NU; u++) {
      const int ci = u < 8 ? u >> 1 : 4, half = u < 8 ? (u & 1) : 0;
      // column tile finished one unit ago (rounded now) and two units ago (stored now)
      const int p1 = (u + NU - 1) % NU, p2 = (u + NU - 2) % NU;
      const int conv_ci = p1 == 8 ? 4 : ((p1 & 1) ? p1 >> 1 : -1);
      const int store_ci = p2 == 8 ? 4 : ((p2 & 1) ? p2 >> 1 : -1);
      const bool reload = half == 1 ? u == 7 : u == (NC == 5 ? 8 : 6);
      if (u == 6) {
        // the next tile's coefficients have landed once at most (issued - mk[0]) younger operations
        // are in flight; anything below the steady-state count (first and last tiles of a query)
        // waits for everything, which is always enough
        if (n + 1 < ntiles) {
          if (issued - mk[0] >= STEADY) { DSA_WAIT_VMCNT(STEADY); } else { DSA_WAIT_VMCNT(0); }
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j + 1 < CST - 1; j++) mk[j] = mk[j + 1];
        mk[CST - 2] = issue_marked(n + CST);
      }
      if (u == 2) rptr = rows + (size_t)drow * ROW_BYTES + lane_off;      // all stores of the previous tile are issued
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < 8; m++) {
        const bf16x8 b = cf[half * 8 + m];
        if (half == 1) {
          mfma_v_av(acc[ci], xo[ci][m], b);
        } else if (ci == 4) {
          if (m == 0) mfma_v_vv_first(acc[4], xqv[m], b); else mfma_v_vv(acc[4], xqv[m], b);
        } else {
          if (m == 0) mfma_v_av_first(acc[ci], xqa[ci][m], b); else mfma_v_av(acc[ci], xqa[ci][m], b);
        }
        if (reload) cf[half * 8 + m] = *(const bf16x8*)(nb + (half * 8 + m) * 1024 + coff);
        if (conv_ci >= 0 && m >= 2 && m < 6) conv(conv_ci, m - 2);
        if (conv_ci >= 0 && m >= 6) piece_read(m - 6);
        if (store_ci >= 0 && (m == 3 || m == 4)) piece_store(store_ci, m - 3);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  // ---- drain: the last tile's final column tiles -------------------------------------------------
  if (NC == 5) {
    piece_store(3, 0);
    piece_store(3, 1);
  }
  mfma_done_v(acc[NC - 1]);
#pragma unroll
  for (int j = 0; j < 4; j++) conv(NC - 1, j);
  piece_read(0);
  piece_read(1);
  piece_store(NC - 1, 0);
  piece_store(NC - 1, 1);
}

// ---------------------------------------------------------------------------------------------
// pass D: dKV[key] = sum of that key's rows, ascending query order
// ---------------------------------------------------------------------------------------------
// One key per workgroup (504 of its threads): 72 column chunks of 8 elements x 7 row groups (row r of the
// segment goes to group r % 7); the seven partial sums are combined in a fixed order, so the result
// depends only on the segment, never on scheduling.  Pure streaming reads of 1152-byte rows, RED_FLIGHT
// of them in flight per thread.
// The rows are read once: a non-temporal load keeps them from displacing other lines in the caches
// (a streaming read of this size runs at 6.8 TB/s with it against 6.1 TB/s without).
typedef unsigned u32x4_nt __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 row_load16(const void* p) {
  const u32x4_nt v = __builtin_nontemporal_load((const u32x4_nt*)p);
  return make_uint4(v.x, v.y, v.z, v.w);
}
constexpr int RED_GROUPS = 7;
constexpr int RED_FLIGHT = 16;               // row pieces a thread has in flight
constexpr int RED_KEYS = 4;                  // consecutive keys per workgroup
// A workgroup sums RED_KEYS consecutive keys (their rows follow one another in the buffer): every thread walks its
// share of the first key's rows, then of the next one's, without a barrier in between, so that the loads of one
// key are in flight while the previous one is summed; one barrier, then the seven partial sums of each key are
// combined.  (One key per workgroup left the per-key latencies - segment bounds, first loads, barrier, combine -
// exposed once a key has few rows per launch: with the queries of 32768 tokens walked in four chunks the launch
// took 27.1 ms against 18.9 ms for one sweep; per key the sums and their order are the same as before.)
__device__ __forceinline__ void reduce_body(const unsigned char* __restrict__ rows, const int* __restrict__ start,
                                            float* __restrict__ dkv_acc, int key0, int n_keys, int accumulate,
                                            unsigned char* smem) {
  float* part = (float*)smem;                  // [RED_KEYS][RED_GROUPS][DQK]
  const int tid = threadIdx.x;
  const int ch = tid % 72, grp = tid / 72;
  const int nk = min(RED_KEYS, n_keys - key0);
  if (grp < RED_GROUPS) {
    int bounds[RED_KEYS + 1];
#pragma unroll
    for (int k = 0; k <= RED_KEYS; k++) bounds[k] = start[min(key0 + k, n_keys)];
#pragma unroll
    for (int k = 0; k < RED_KEYS; k++) {
      if (k >= nk) break;
      const int s0 = bounds[k], s1 = bounds[k + 1];
      float acc[8];
#pragma unroll
      for (int e = 0; e < 8; e++) acc[e] = 0.f;
      int rr = s0 + grp;
      for (; rr + (RED_FLIGHT - 1) * RED_GROUPS < s1; rr += RED_FLIGHT * RED_GROUPS) {
        uint4 v[RED_FLIGHT];
#pragma unroll
        for (int u = 0; u < RED_FLIGHT; u++) v[u] = row_load16(rows + (size_t)(rr + u * RED_GROUPS) * ROW_BYTES + ch * 16);
#pragma unroll
        for (int u = 0; u < RED_FLIGHT; u++) {
          const unsigned w[4] = {v[u].x, v[u].y, v[u].z, v[u].w};
#pragma unroll
          for (int e = 0; e < 4; e++) {
            acc[2 * e] += __builtin_bit_cast(float, w[e] << 16);
            acc[2 * e + 1] += __builtin_bit_cast(float, w[e] & 0xffff0000u);
          }
        }
      }
      for (; rr < s1; rr += RED_GROUPS) {
        const uint4 v = row_load16(rows + (size_t)rr * ROW_BYTES + ch * 16);
        const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
          acc[2 * e] += __builtin_bit_cast(float, w[e] << 16);
          acc[2 * e + 1] += __builtin_bit_cast(float, w[e] & 0xffff0000u);
        }
      }
#pragma unroll
      for (int e = 0; e < 8; e++) part[(k * RED_GROUPS + grp) * DQK + ch * 8 + e] = acc[e];
    }
  }
  __syncthreads();
  for (int o = tid; o < nk * DQK; o += (int)blockDim.x) {
    const int k = o / DQK, d = o % DQK;
    float sum = part[k * RED_GROUPS * DQK + d];
#pragma unroll
    for (int gq = 1; gq < RED_GROUPS; gq++) sum += part[(k * RED_GROUPS + gq) * DQK + d];
    float* p = dkv_acc + (size_t)(key0 + k) * DQK + d;
    *p = accumulate ? *p + sum : sum;
  }
}

// ---------------------------------------------------------------------------------------------
// kernels: two roles each, chosen per workgroup
// ---------------------------------------------------------------------------------------------
// Pass B is bound by LDS reads and leaves HBM nearly idle; pass D is a pure stream of HBM reads and
// leaves everything else idle; each occupies a whole compute unit (140 KB of LDS, or all its
// memory-level parallelism).  One launch carries the workgroups of both, spread evenly over the
// dispatch order, so that both kinds of work are in flight from the first workgroup to the last:
//   bwd_dq_reduce_kernel   pass B of all queries | pass D of all keys      (4.5 ms against 2.6 + 2.75)
// Within a role, the longest work (latest query, earliest key) comes first.
// Passes A and C, carried by one launch in the same way (pass A of one block of queries beside
// pass C of the block before it, 2 - 64 interleaved blocks), took as long side by side as one after
// the other: neither gets faster when it has fewer compute units - a compute unit that alternates
// cold loads (the P / dS tiles) with stores (the rows) drains either queue before it serves the
// other, which bounds pass C per compute unit at about the rate at which HBM bounds it for the
// whole chip.  They are separate kernels.
struct RoleSlot { bool first; int i; };
// nX workgroups of the first role and nY of the second, spread evenly over the launch: workgroup b belongs to the
// second role when the count floor(b * nY / (nX + nY)) steps up after it.
__device__ __forceinline__ RoleSlot role_slot(int b, int nX, int nY) {
  const long long tot = (long long)nX + nY;
  const int y0 = (int)((long long)b * nY / tot), y1 = (int)((long long)(b + 1) * nY / tot);
  if (y1 > y0) return {false, y0};
  return {true, b - y0};
}

__global__ __launch_bounds__(PDS_THREADS, 1) void bwd_pds_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ kv, const int* __restrict__ ids,
    const __bf16* __restrict__ out, const __bf16* __restrict__ dout, const float* __restrict__ lse,
    unsigned char* __restrict__ pds, int q0, int cnt, int H, int Skv, int K, int q_start, float sm_scale) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  pds_body<4>(q, kv, ids, out, dout, lse, pds, q0, cnt - 1 - (int)blockIdx.x, H, Skv, K, q_start, sm_scale, smem);
}

__global__ __launch_bounds__(256, 1) void bwd_dkv_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ dout, const int* __restrict__ ids,
    const unsigned char* __restrict__ pds, const int* __restrict__ dst, unsigned char* __restrict__ rows,
    int q0, int cnt, int H, int Skv, int K, int q_start, int dummy_row) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int ql = cnt - 1 - (int)blockIdx.x;
  // waves 0 and 1 own five column tiles, waves 2 and 3 four: two copies of the whole body, so that
  // no branch sits between the MFMAs; every copy meets the same barriers
  if (threadIdx.x < 128) dkv_body<5>(q, dout, ids, pds, dst, rows, q0, ql, H, Skv, K, q_start, dummy_row, smem);
  else dkv_body<4>(q, dout, ids, pds, dst, rows, q0, ql, H, Skv, K, q_start, dummy_row, smem);
}

__global__ __launch_bounds__(DQ_THREADS, 1) void bwd_dq_reduce_kernel(
    const __bf16* __restrict__ kv, const int* __restrict__ ids, const unsigned char* __restrict__ pds,
    __bf16* __restrict__ dq, int q0, int cnt, int H, int Skv, int K, int q_start, const int* __restrict__ dup_flag,
    const unsigned char* __restrict__ rows, const int* __restrict__ start, float* __restrict__ dkv_acc, int n_keys,
    int accumulate) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const RoleSlot rs = role_slot((int)blockIdx.x, cnt, (n_keys + RED_KEYS - 1) / RED_KEYS);
  if (rs.first) dq_body<3>(kv, ids, pds, dq, q0, cnt - 1 - rs.i, H, Skv, K, q_start, dup_flag, smem);
  else reduce_body(rows, start, dkv_acc, rs.i * RED_KEYS, n_keys, accumulate, smem);
}

// fp32 accumulator -> bf16 dKV; NaN everywhere when a query row held a repeated id
__global__ void cast_bf16_kernel(const float* __restrict__ src, unsigned short* __restrict__ dstp, size_t n,
                                 const int* __restrict__ dup_flag) {
  const bool poison = *dup_flag != 0;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x)
    dstp[e] = poison ? (unsigned short)0x7fc0 : f32_to_bf16_bits(src[e]);
}

// dQ of the chunks that ran before the flag was raised still holds sums: NaN everywhere in that case
__global__ void poison_bf16_kernel(unsigned short* __restrict__ p, size_t n, const int* __restrict__ dup_flag) {
  if (*dup_flag == 0) return;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x)
    p[e] = (unsigned short)0x7fc0;
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
struct BwdPlan {
  int chunk;            // queries per pass over the buffers
  int W;                // bitmap words per key
  size_t off_bitmap, off_prefix, off_count, off_start, off_flag, off_dst, off_sorted, off_pds, off_rows, off_acc, total;
};

size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }

BwdPlan layout_plan(int chunk, int Skv, int K) {
  BwdPlan p;
  p.chunk = chunk;
  p.W = (chunk + 31) / 32;
  size_t o = 0;
  p.off_bitmap = o; o = align_up(o + (size_t)Skv * p.W * 4);
  p.off_prefix = o; o = align_up(o + order::prefix_words(chunk, Skv) * 4);
  p.off_count = o; o = align_up(o + (size_t)(Skv + 1) * 4);
  p.off_start = o; o = align_up(o + (size_t)(Skv + 1) * 4);
  p.off_flag = o; o = align_up(o + 4);
  p.off_dst = o; o = align_up(o + (size_t)chunk * K * 4);
  p.off_sorted = o; o = align_up(o + (size_t)chunk * K * 4);
  p.off_pds = o; o = align_up(o + (size_t)chunk * (K / BI) * PDS_TILE_BYTES);
  p.off_rows = o; o = align_up(o + ((size_t)chunk * K + 1) * ROW_BYTES);
  p.off_acc = o; o = align_up(o + (size_t)Skv * DQK * 4);
  p.total = o;
  return p;
}

// Largest chunk of queries (all of them if possible, else repeated halving, at least 64) whose
// buffers fit the budget.
BwdPlan make_plan(int S, int Skv, int K, size_t budget) {
  int chunk = S;
  BwdPlan p = layout_plan(chunk, Skv, K);
  while (p.total > budget && chunk > 64) {
    chunk = (chunk + 1) / 2;
    p = layout_plan(chunk, Skv, K);
  }
  return p;
}

constexpr size_t DEFAULT_BUDGET = (size_t)160 << 30;

}  // namespace

extern "C" size_t dsa_sparse_mla_bwd_workspace_bytes(int S, int H, int Skv, int K) {
  (void)H;
  if (S <= 0 || Skv <= 0 || K <= 0) return 0;
  return make_plan(S, Skv, K, DEFAULT_BUDGET).total;
}

extern "C" size_t dsa_sparse_mla_bwd_workspace_bytes_min(int S, int H, int Skv, int K) {
  (void)H;
  if (S <= 0 || Skv <= 0 || K <= 0) return 0;
  return layout_plan(S < 64 ? S : 64, Skv, K).total;
}

static int bwd_impl(const void* q, const void* kv, const void* out, const void* dout, const int32_t* ids,
                    const float* lse, int S, int H, int Skv, int K, int q_start, float sm_scale, int d_v,
                    void* dq, void* dkv, void* workspace, size_t workspace_bytes, void* stream, float* pass_ms) {
  DSA_REQUIRE(d_v == DV, "dsa_sparse_mla_bwd: only d_v = 512 (d_qk = 576) is supported, got d_v = %d", d_v);
  DSA_REQUIRE(S >= 0 && Skv > 0, "dsa_sparse_mla_bwd: bad sequence sizes S=%d Skv=%d", S, Skv);
  DSA_REQUIRE(H > 0 && H <= 128 && H % 32 == 0, "dsa_sparse_mla_bwd: head count must be 32, 64, 96 or 128, got %d", H);
  DSA_REQUIRE(K > 0 && K % 64 == 0 && K <= 2048, "dsa_sparse_mla_bwd: top-k must be a multiple of 64 up to 2048, got %d", K);
  DSA_REQUIRE((size_t)Skv * DQK * 2 <= 0xffffffffull, "dsa_sparse_mla_bwd: kv larger than 4 GiB is not supported");
  DSA_REQUIRE(Skv <= order::MAX_KEYS, "dsa_sparse_mla_bwd: at most %d keys are supported, got %d", order::MAX_KEYS, Skv);
  DSA_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)kv % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
              ((uintptr_t)dout % 16) == 0 && ((uintptr_t)dq % 16) == 0 && ((uintptr_t)workspace % 256) == 0,
              "dsa_sparse_mla_bwd: misaligned pointer");
  hipStream_t st = (hipStream_t)stream;
  // choose the largest chunk the given workspace allows
  BwdPlan p = make_plan(S > 0 ? S : 1, Skv, K, workspace_bytes);
  if (p.total > workspace_bytes || workspace == nullptr)
    DSA_FAIL(DSA_ERR_WORKSPACE, "dsa_sparse_mla_bwd: workspace of %zu bytes is too small (need at least %zu)",
             workspace_bytes, make_plan(64, Skv, K, 1).total);
  unsigned char* ws = (unsigned char*)workspace;
  unsigned* bitmap = (unsigned*)(ws + p.off_bitmap);
  unsigned* prefix = (unsigned*)(ws + p.off_prefix);
  int* count = (int*)(ws + p.off_count);
  int* start = (int*)(ws + p.off_start);
  int* dup_flag = (int*)(ws + p.off_flag);
  int* dstp = (int*)(ws + p.off_dst);
  int* sorted = (int*)(ws + p.off_sorted);
  unsigned char* pds = ws + p.off_pds;
  unsigned char* rows = ws + p.off_rows;
  float* acc = (float*)(ws + p.off_acc);
  const int NT = K / BI;

  const size_t smemA = (size_t)4 * TILE_BYTES + ids_lds_bytes(K) + 16 + 1024;
  const size_t smemB = (size_t)3 * (TILE_BYTES + PDS_KIND_BYTES) + ids_lds_bytes(K);
  const size_t smemC = (size_t)DKV_COEF_STAGES * PDS_TILE_BYTES + ids_lds_bytes(K) + 16 + (size_t)(K + BI) * 4;
  if (dsa_reserve_lds((const void*)bwd_pds_kernel, smemA) != hipSuccess ||
      dsa_reserve_lds((const void*)bwd_dkv_kernel, smemC) != hipSuccess ||
      dsa_reserve_lds((const void*)bwd_dq_reduce_kernel, smemB) != hipSuccess)
    DSA_FAIL(DSA_ERR_LAUNCH, "dsa_sparse_mla_bwd: cannot reserve LDS");

  // optional timing (profiling entry point only): events between the launch groups
  hipEvent_t ev[5];
  if (pass_ms) {
    for (int i = 0; i < 5; i++) pass_ms[i] = 0.f;
    int made = 0;
    for (; made < 5; made++) if (hipEventCreate(&ev[made]) != hipSuccess) break;
    if (made < 5) {
      for (int i = 0; i < made; i++) hipEventDestroy(ev[i]);
      DSA_FAIL(DSA_ERR_LAUNCH, "dsa_sparse_mla_bwd_profile: cannot create events");
    }
  }
#define DSA_MARK(i) do { if (pass_ms) hipEventRecord(ev[i], st); } while (0)
  bool first = true;
  order::clear_flag(dup_flag, st);
  for (int q0 = 0; q0 < S; q0 += p.chunk) {
    const int cnt = S - q0 < p.chunk ? S - q0 : p.chunk;
    DSA_MARK(0);
    // The passes are free to choose their slot order (P, dS and the dKV rows never leave the workspace):
    // they walk each query's valid ids in ascending key order, so that the queries in flight on an XCD
    // gather neighbouring latent rows at the same time.
    // (The list is put together in LDS next to a bitmap over all keys; with more keys than fit there the
    // passes walk the caller's slot order instead.)
    const bool sort_ids = order::sorted_list_fits(Skv, K);
    order::build(ids, q0, cnt, K, Skv, q_start, bitmap, prefix, count, start, dstp, p.W, st, dup_flag, sort_ids ? sorted : nullptr);
    DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(order)");
    const int* sids = sort_ids ? sorted : ids + (size_t)q0 * K;      // row ql belongs to query q0 + ql
    DSA_MARK(1);
    bwd_pds_kernel<<<dim3(cnt), dim3(PDS_THREADS), smemA, st>>>((const __bf16*)q, (const __bf16*)kv, sids, (const __bf16*)out,
                                                       (const __bf16*)dout, lse, pds, q0, cnt, H, Skv, K, q_start, sm_scale);
    DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(P, dS)");
    DSA_MARK(2);
    bwd_dkv_kernel<<<dim3(cnt), dim3(256), smemC, st>>>((const __bf16*)q, (const __bf16*)dout, sids, pds, dstp, rows, q0, cnt,
                                                       H, Skv, K, q_start, p.chunk * K);
    DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(dKV rows)");
    DSA_MARK(3);
    // Pass B of every query beside pass D of every key.
    bwd_dq_reduce_kernel<<<dim3(cnt + (Skv + RED_KEYS - 1) / RED_KEYS), dim3(DQ_THREADS), smemB, st>>>((const __bf16*)kv, sids, pds, (__bf16*)dq, q0, cnt, H, Skv,
                                                                   K, q_start, dup_flag, rows, start, acc, Skv, first ? 0 : 1);
    DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(dQ | dKV reduce)");
    DSA_MARK(4);
    if (pass_ms) {
      hipEventSynchronize(ev[4]);
      for (int i = 0; i < 4; i++) { float ms = 0.f; hipEventElapsedTime(&ms, ev[i], ev[i + 1]); pass_ms[i] += ms; }
    }
    first = false;
  }
  if (S == 0) {
    order::zero_u32_kernel<<<dim3(256), dim3(256), 0, st>>>((unsigned*)acc, (size_t)Skv * DQK);
  }
  cast_bf16_kernel<<<dim3(2048), dim3(256), 0, st>>>(acc, (unsigned short*)dkv, (size_t)Skv * DQK, dup_flag);
  if (S > p.chunk)      // more than one chunk: the flag may have come up after earlier chunks wrote their dQ
    poison_bf16_kernel<<<dim3(2048), dim3(256), 0, st>>>((unsigned short*)dq, (size_t)S * H * DQK, dup_flag);
  DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(cast)");
  (void)NT;
  if (pass_ms) for (int i = 0; i < 5; i++) hipEventDestroy(ev[i]);
#undef DSA_MARK
  return DSA_OK;
}

extern "C" int dsa_sparse_mla_bwd(const void* q, const void* kv, const void* out, const void* dout, const int32_t* ids,
                                  const float* lse, int S, int H, int Skv, int K, int q_start, float sm_scale, int d_v,
                                  void* dq, void* dkv, void* workspace, size_t workspace_bytes, void* stream) {
  return bwd_impl(q, kv, out, dout, ids, lse, S, H, Skv, K, q_start, sm_scale, d_v, dq, dkv, workspace, workspace_bytes,
                  stream, nullptr);
}

#ifdef DSA_BENCH_BUILD     // the benchmark library compiles this file a second time, with the timed entry point
extern "C" int dsa_sparse_mla_bwd_profile(const void* q, const void* kv, const void* out, const void* dout,
                                          const int32_t* ids, const float* lse, int S, int H, int Skv, int K, int q_start,
                                          float sm_scale, int d_v, void* dq, void* dkv, void* workspace,
                                          size_t workspace_bytes, void* stream, float* pass_ms) {
  DSA_REQUIRE(pass_ms != nullptr, "dsa_sparse_mla_bwd_profile: pass_ms must point at 5 floats");
  return bwd_impl(q, kv, out, dout, ids, lse, S, H, Skv, K, q_start, sm_scale, d_v, dq, dkv, workspace, workspace_bytes,
                  stream, pass_ms);
}
#endif
