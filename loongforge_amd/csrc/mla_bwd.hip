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
//                              16-bit block-floating-point row (int16 mantissas + one fp32 scale)
//                              in a pair buffer, at the position given by a key-sorted order
//   pass D  (bwd_reduce_kernel) dKV[key] = sum of that key's rows, in ascending query order
// The key-sorted order (pass 0) comes from a bitmap key x query, its row-wise prefix popcounts and
// an exclusive scan over keys: integer work only, so the order - and with it every fp32 sum - is
// identical from run to run.  No floating-point atomics anywhere.
#include "mla_tile.h"
#include "order.h"

namespace {
using namespace mla;

constexpr int PDS_TILE_BYTES = 16384;        // P and dS of one (query, tile): 2 x [4 waves][2][2][32 keys][8 heads] bf16
constexpr int PDS_KIND_BYTES = 8192;
constexpr int ROW_BYTES = DQK * 2;           // one pair row of the dKV buffer

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

// vmcnt wait with a run-time bound (the instruction needs an immediate)
__device__ __forceinline__ void wait_vmcnt_le(int n) {
  switch (n) {
#define C(k) case k: DSA_WAIT_VMCNT(k); break;
    C(0) C(1) C(2) C(3) C(4) C(5) C(6) C(7) C(8) C(9) C(10) C(11) C(12) C(13) C(14) C(15) C(16) C(17) C(18) C(19)
    C(20) C(21) C(22) C(23) C(24) C(25) C(26) C(27) C(28) C(29) C(30) C(31) C(32) C(33) C(34) C(35) C(36) C(37)
    C(38) C(39) C(40) C(41) C(42) C(43) C(44) C(45) C(46) C(47) C(48)
#undef C
    default: DSA_WAIT_VMCNT(0); break;
  }
}

// ---------------------------------------------------------------------------------------------
// pass A: P and dS of every (query, tile)
// ---------------------------------------------------------------------------------------------
// One workgroup per query, wave w owns heads [32w, 32w+32).  S = Q.KV^T and dP = dO.V^T share the
// key-row operand read from LDS; Q and dO are the other MFMA operand, resident in registers (Q and
// half of dO in accumulation registers, which MFMA can read directly).  The accumulators then hold
// one key per lane and 16 heads per lane, which is the k-vector layout pass C needs, so P and dS go
// to HBM as 16-byte chunks without any shuffle.
template <int STAGES>
__global__ __launch_bounds__(256, 1) void bwd_pds_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ kv, const int* __restrict__ ids,
    const __bf16* __restrict__ out, const __bf16* __restrict__ dout, const float* __restrict__ lse,
    unsigned char* __restrict__ pds, int q0, int cnt, int H, int Skv, int K, int q_start, float sm_scale) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int ql = cnt - 1 - (int)blockIdx.x;
  const int qi = q0 + ql;
  const int NT = K / BI;
  int* idx_s = (int*)(smem + STAGES * TILE_BYTES);
  unsigned* tmask = (unsigned*)(idx_s + K);
  int* tlist = (int*)(tmask + NT);
  int* ntile_s = tlist + NT;
  float* stat_s = (float*)(ntile_s + 4);       // [2][128]: lse * log2(e), delta
  const int ntiles = stage_ids(ids, qi, K, Skv, q_start + qi, idx_s, tmask, tlist, ntile_s);

  const int h = wave * 32 + r;
  const bool head_ok = h < H;
  const size_t hrow = (size_t)qi * H + (head_ok ? h : 0);
  bf16x8 qreg[KSTEPS], doreg[VSTEPS];
  {
    const bf16x8* qp = (const bf16x8*)(q + hrow * DQK) + g;
    const bf16x8* dp = (const bf16x8*)(dout + hrow * DV) + g;
    const bf16x8* op = (const bf16x8*)(out + hrow * DV) + g;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) qreg[ks] = qp[2 * ks];
    float part = 0.f;
#pragma unroll
    for (int ks = 0; ks < VSTEPS; ks++) {
      doreg[ks] = dp[2 * ks];
      const bf16x8 o = op[2 * ks];
#pragma unroll
      for (int e = 0; e < 8; e++) part = fmaf((float)o[e], (float)doreg[ks][e], part);
    }
    part += __shfl_xor(part, 32, 64);
    if (g == 0) {
      stat_s[h] = head_ok ? lse[hrow] * LOG2E : INFINITY;
      stat_s[128 + h] = head_ok ? part : 0.f;
    }
    DSA_WAIT_VMCNT(0);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) asm volatile("" : "+a"(qreg[ks]));
#pragma unroll
    for (int ks = 0; ks < VSTEPS; ks++) {
      if (ks < 16) asm volatile("" : "+a"(doreg[ks]));
      else asm volatile("" : "+v"(doreg[ks]));
    }
  }
  __syncthreads();
  // accumulator e of a lane is head 32*wave + 8*(e/4) + 4*g + (e%4), for key (lane & 31)
  float lse2[16], delta[16];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const f32x4 a = *(const f32x4*)(stat_s + wave * 32 + 8 * j + 4 * g);
    const f32x4 b = *(const f32x4*)(stat_s + 128 + wave * 32 + 8 * j + 4 * g);
#pragma unroll
    for (int e = 0; e < 4; e++) { lse2[4 * j + e] = a[e]; delta[4 * j + e] = b[e]; }
  }

  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  const LaneOffsets lo = lane_offsets();
  const float c2 = sm_scale * LOG2E;
  auto issue = [&](int n) { gather_tile(kv, idx_s, tlist[n], lds0 + (unsigned)((n % STAGES) * TILE_BYTES)); };
  for (int n = 0; n < STAGES - 1 && n < ntiles; n++) issue(n);

  for (int n = 0; n < ntiles; n++) {
    // operations issued after this tile's gather: 9 per later gather, 4 stores per finished tile
    wait_vmcnt_le(9 * min(STAGES - 2, ntiles - 1 - n) + 4 * min(n, STAGES - 1));
    __syncthreads();
    if (n + STAGES - 1 < ntiles) issue(n + STAGES - 1);
    const int tile = tlist[n];
    const unsigned mask = tmask[tile];
    const unsigned char* tb = smem + (n % STAGES) * TILE_BYTES;

    f32x16 sacc, dpacc;
    {
      bf16x8 f[4];
#pragma unroll
      for (int ks = 0; ks < 4; ks++) f[ks] = *(const bf16x8*)(tb + (ks >> 2) * GRP_BYTES + lo.row_off[ks & 3]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ks++) {
        if (ks == 0) { mfma_v_av_first(sacc, qreg[0], f[0]); mfma_v_av_first(dpacc, doreg[0], f[0]); }
        else {
          mfma_v_av(sacc, qreg[ks], f[ks & 3]);
          if (ks < 16) mfma_v_av(dpacc, doreg[ks], f[ks & 3]);
          else if (ks < VSTEPS) mfma_v_vv(dpacc, doreg[ks], f[ks & 3]);
        }
        if (ks + 4 < KSTEPS) f[ks & 3] = *(const bf16x8*)(tb + ((ks + 4) >> 2) * GRP_BYTES + lo.row_off[ks & 3]);
        __builtin_amdgcn_sched_barrier(0);
      }
      mfma_done_v(sacc);
      mfma_done_v(dpacc);
    }
    const bool valid = (mask >> r) & 1u;
    bf16x8 pv[2], dsv[2];
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const int a = 8 * s + e;
        const float p = valid ? __builtin_amdgcn_exp2f(fmaf(sacc[a], c2, -lse2[a])) : 0.f;
        const float ds = p * (dpacc[a] - delta[a]) * sm_scale;
        pv[s][e] = (__bf16)p;
        dsv[s][e] = (__bf16)ds;
      }
    unsigned char* base = pds + ((size_t)ql * NT + tile) * PDS_TILE_BYTES + (size_t)((wave * 2) * 2 + g) * 512 + r * 16;
#pragma unroll
    for (int s = 0; s < 2; s++) {
      *(bf16x8*)(base + s * 1024) = dsv[s];
      *(bf16x8*)(base + PDS_KIND_BYTES + s * 1024) = pv[s];
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// ---------------------------------------------------------------------------------------------
// pass B: dQ
// ---------------------------------------------------------------------------------------------
// dQ^T[d, head] += KV^T[d, key] . dS^T[key, head] per 32-key tile.  Both operands are LDS transpose
// reads: of the gathered key tile (18 d-tiles) and of the tile's dS block copied verbatim from the
// pass-A buffer.  The 18 accumulator tiles of a wave (288 registers) sit in the 256 accumulation
// registers plus 32 architectural ones.
template <int STAGES>
__global__ __launch_bounds__(256, 1) void bwd_dq_kernel(
    const __bf16* __restrict__ kv, const int* __restrict__ ids, const unsigned char* __restrict__ pds,
    __bf16* __restrict__ dq, int q0, int cnt, int H, int Skv, int K, int q_start) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  constexpr int STAGE_BYTES = TILE_BYTES + PDS_KIND_BYTES;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int ql = cnt - 1 - (int)blockIdx.x;
  const int qi = q0 + ql;
  const int NT = K / BI;
  int* idx_s = (int*)(smem + STAGES * STAGE_BYTES);
  unsigned* tmask = (unsigned*)(idx_s + K);
  int* tlist = (int*)(tmask + NT);
  int* ntile_s = tlist + NT;
  const int ntiles = stage_ids(ids, qi, K, Skv, q_start + qi, idx_s, tmask, tlist, ntile_s);

  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  const LaneOffsets lo = lane_offsets();
  // transposed read of the dS block [wave][s'][g'][key][8 heads]: lane (blk, ii) points at key
  // 16s + 8t + 4g + ii/4 and the 4 heads 16*(blk&1) + 4*(ii&3) .. +3 of this wave
  unsigned ds_off[2][2];
  {
    const int blk = lane >> 4, ii = lane & 15, qq = ii & 3;
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
      for (int t = 0; t < 2; t++) {
        const int key = 16 * s + 8 * t + 4 * g + (ii >> 2);
        ds_off[s][t] = (unsigned)(TILE_BYTES + wave * 2048 + (blk & 1) * 1024 + (qq & 1) * 512 + key * 16 + (qq >> 1) * 8);
      }
  }
  auto issue = [&](int n) {
    const int tile = tlist[n];
    const unsigned sb = lds0 + (unsigned)((n % STAGES) * STAGE_BYTES);
    gather_tile(kv, idx_s, tile, sb);
    const unsigned lb = __builtin_amdgcn_readfirstlane(sb + (unsigned)(TILE_BYTES + wave * 1024));
    const unsigned char* src = uniform_ptr(pds + ((size_t)ql * NT + tile) * PDS_TILE_BYTES);     // dS half
    dma16(lb, (unsigned)(tid * 16), src);
    dma16(lb + 4096, (unsigned)(4096 + tid * 16), src);
  };

  f32x16 acc[18];
#pragma unroll
  for (int dt = 0; dt < 18; dt++) {
#pragma unroll
    for (int e = 0; e < 16; e++) acc[dt][e] = 0.f;
    if (dt < 16) asm volatile("" : "+a"(acc[dt])); else asm volatile("" : "+v"(acc[dt]));
  }
  for (int n = 0; n < STAGES - 1 && n < ntiles; n++) issue(n);
  for (int n = 0; n < ntiles; n++) {
    wait_vmcnt_le(11 * min(STAGES - 2, ntiles - 1 - n));
    __syncthreads();
    if (n + STAGES - 1 < ntiles) issue(n + STAGES - 1);
    const unsigned char* tb = smem + (n % STAGES) * STAGE_BYTES;
    typedef short i16x8 __attribute__((ext_vector_type(8)));
    bf16x8 bds[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
      i16x4 x0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, tb + ds_off[s][0]));
      i16x4 x1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, tb + ds_off[s][1]));
      bds[s] = __builtin_bit_cast(bf16x8, (i16x8)__builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7));
    }
    i16x4 v[2][2][2];
#pragma unroll
    for (int dt = 0; dt < 2; dt++)
#pragma unroll
      for (int s = 0; s < 2; s++)
#pragma unroll
        for (int t = 0; t < 2; t++)
          v[dt][s][t] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, tb + (dt >> 1) * GRP_BYTES + lo.tr_off[s][t][dt & 1]));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int dt = 0; dt < 18; dt++) {
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const bf16x8 a = __builtin_bit_cast(bf16x8, (i16x8)__builtin_shufflevector(v[dt & 1][s][0], v[dt & 1][s][1], 0, 1, 2, 3, 4, 5, 6, 7));
        if (dt < 16) mfma_a_vv(acc[dt], a, bds[s]);
        else mfma_v_vv(acc[dt], a, bds[s]);
      }
      if (dt + 2 < 18) {
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
          for (int t = 0; t < 2; t++)
            v[dt & 1][s][t] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, tb + ((dt + 2) >> 1) * GRP_BYTES + lo.tr_off[s][t][dt & 1]));
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  const int h = wave * 32 + r;
  if (h < H) {
    unsigned short* op = (unsigned short*)dq + ((size_t)qi * H + h) * DQK + 4 * g;
#pragma unroll
    for (int dt = 0; dt < 18; dt++) {
      if (dt < 16) mfma_done_a(acc[dt]); else mfma_done_v(acc[dt]);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        uint2 w = make_uint2(pack_bf16x2(acc[dt][4 * j], acc[dt][4 * j + 1]), pack_bf16x2(acc[dt][4 * j + 2], acc[dt][4 * j + 3]));
        *(uint2*)(op + 32 * dt + 8 * j) = w;
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// pass C: per-pair dKV rows
// ---------------------------------------------------------------------------------------------
// row[key, d] = sum_h dS[h,key] Q[h,d] + (d < 512) sum_h P[h,key] dO[h,d], all 128 heads, as
// row^T = X^T . coef with X = [Q; dO] (k = heads).  X^T is the register-resident operand: wave w
// owns the 32-column d-tiles {w, w+4, w+8, w+12, w+16} (the last only for w < 2) and loads its
// columns once per query through LDS transpose reads; the coefficient operand is the pass-A tile
// read from LDS as stored.  The finished 32 x 576 fp32 tile is staged in LDS, each row is scaled
// by 32767 / max|row| and written as one contiguous 1152-byte row of int16 (plus its fp32 scale)
// to the row index of the key-sorted order: the rounding error of a row is 2^-16 of its largest
// element, 128 times less than a bf16 row of the same size.
constexpr int OUT_STRIDE = DQK * 4 + 16;     // fp32 staging row stride in bytes (bank spread)

__global__ __launch_bounds__(256, 1) void bwd_dkv_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ dout, const int* __restrict__ ids,
    const unsigned char* __restrict__ pds, const int* __restrict__ dst, unsigned char* __restrict__ rows,
    float* __restrict__ row_scale, int q0, int cnt, int H, int Skv, int K, int q_start, int dummy_row) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  // [2][PDS_TILE_BYTES] coefficient tiles | [32][OUT_STRIDE] staging | [4][8192] per-wave X staging |
  // ids arrays | dst rows of the query [K] | row inverse scales [32]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int ql = cnt - 1 - (int)blockIdx.x;
  const int qi = q0 + ql;
  const int NT = K / BI;
  unsigned char* out_s = smem + 2 * PDS_TILE_BYTES;
  unsigned char* xs = out_s + BI * OUT_STRIDE + wave * 8192;
  int* idx_s = (int*)(out_s + BI * OUT_STRIDE + 4 * 8192);
  unsigned* tmask = (unsigned*)(idx_s + K);
  int* tlist = (int*)(tmask + NT);
  int* ntile_s = tlist + NT;
  int* dst_s = ntile_s + 4;
  float* inv_s = (float*)(dst_s + K);
  for (int t = tid; t < K; t += 256) {
    const int d = dst[(size_t)ql * K + t];
    dst_s[t] = d >= 0 ? d : dummy_row;       // invalid slots land in a scratch row: the store count stays fixed
  }
  const int ntiles = stage_ids(ids, qi, K, Skv, q_start + qi, idx_s, tmask, tlist, ntile_s);
  if (ntiles == 0) return;

  // ---- X^T operands: xq[c][kk] / xo[c][kk], kk = 2*w' + s' over the 8 groups of 16 heads ------
  const int ncol = wave < 2 ? 5 : 4;
  bf16x8 xq[5][8], xo[4][8];
  {
    typedef short i16x8 __attribute__((ext_vector_type(8)));
    const int blk = lane >> 4, ii = lane & 15;
    // transpose read of a [128 heads][32 d] block (64-byte rows): lane points at head
    // 32w' + 8(2s'+t) + 4g + ii/4, d chunk 16*(blk&1) + 4*(ii&3)
    const unsigned xoff = (unsigned)((4 * g + (ii >> 2)) * 64 + (16 * (blk & 1) + 4 * (ii & 3)) * 2);
#pragma unroll
    for (int pass = 0; pass < 9; pass++) {
      const bool isq = pass < 5;
      const int ci = isq ? pass : pass - 5;
      if (isq && ci >= ncol) continue;
      const int c = wave + 4 * ci;                      // d-tile
      const __bf16* src = isq ? q + (size_t)qi * H * DQK + 32 * c : dout + (size_t)qi * H * DV + 32 * c;
      const int stride = isq ? DQK : DV;
      // stage rows of 64 bytes: lane covers head (lane/4 + 16*it), 16-byte piece lane%4
#pragma unroll
      for (int it = 0; it < 8; it++) {
        const int hh = (lane >> 2) + 16 * it;
        uint4 val = make_uint4(0, 0, 0, 0);
        if (hh < H) val = *(const uint4*)(src + (size_t)hh * stride + (lane & 3) * 8);
        *(uint4*)(xs + hh * 64 + (lane & 3) * 16) = val;
      }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int kk = 0; kk < 8; kk++) {
        const unsigned char* hb = xs + (32 * (kk >> 1) + 16 * (kk & 1)) * 64;
        i16x4 x0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, hb + xoff));
        i16x4 x1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, hb + 8 * 64 + xoff));
        const bf16x8 val = __builtin_bit_cast(bf16x8, (i16x8)__builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7));
        if (isq) xq[ci][kk] = val; else xo[ci][kk] = val;
      }
      __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int ci = 0; ci < 5; ci++)
#pragma unroll
      for (int kk = 0; kk < 8; kk++) asm volatile("" : "+v"(xq[ci][kk]));
#pragma unroll
    for (int ci = 0; ci < 4; ci++)
#pragma unroll
      for (int kk = 0; kk < 8; kk++) asm volatile("" : "+a"(xo[ci][kk]));
  }

  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  auto issue = [&](int n) {
    const unsigned lb = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)((n & 1) * PDS_TILE_BYTES + wave * 1024));
    const unsigned char* src = uniform_ptr(pds + ((size_t)ql * NT + tlist[n]) * PDS_TILE_BYTES);
#pragma unroll
    for (int c = 0; c < 4; c++) dma16(lb + c * 4096, (unsigned)(c * 4096 + tid * 16), src);
  };
  issue(0);
  for (int n = 0; n < ntiles; n++) {
    // issued after this tile's 4 transfers: the 9 row stores and the scale store of the previous tile
    if (n > 0) { DSA_WAIT_VMCNT(10); } else { DSA_WAIT_VMCNT(0); }
    __syncthreads();
    if (n + 1 < ntiles) issue(n + 1);
    const unsigned char* cb = smem + (n & 1) * PDS_TILE_BYTES;
    const int tile = tlist[n];
    f32x16 acc[5];
    // coefficient chunk of k-step kk: [kind][kk][g][key r] 16 bytes
    const unsigned coff = (unsigned)(g * 512 + r * 16);
    bf16x8 cf[2];
    cf[0] = *(const bf16x8*)(cb + coff);
    cf[1] = *(const bf16x8*)(cb + 1024 + coff);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int step = 0; step < 16; step++) {            // 0..7: dS with Q, 8..15: P with dO
      const int kk = step & 7;
#pragma unroll
      for (int ci = 0; ci < 5; ci++) {
        if (step < 8) {
          if (ci < 4 || wave < 2) {
            if (step == 0) mfma_a_vv_first(acc[ci], xq[ci][kk], cf[step & 1]);
            else mfma_a_vv(acc[ci], xq[ci][kk], cf[step & 1]);
          }
        } else if (ci < 4) {
          mfma_a_av(acc[ci], xo[ci][kk], cf[step & 1]);
        }
      }
      if (step + 2 < 16) cf[step & 1] = *(const bf16x8*)(cb + (step + 2) * 1024 + coff);
      __builtin_amdgcn_sched_barrier(0);
    }
    // accumulator e of a lane: d = 32c + 8*(e/4) + 4g + (e%4), key = lane & 31
#pragma unroll
    for (int ci = 0; ci < 5; ci++) {
      if (ci == 4 && wave >= 2) continue;
      mfma_done_a(acc[ci]);
      const int c = wave + 4 * ci;
      float* orow = (float*)(out_s + r * OUT_STRIDE) + 32 * c + 4 * g;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const f32x4 w = {acc[ci][4 * j], acc[ci][4 * j + 1], acc[ci][4 * j + 2], acc[ci][4 * j + 3]};
        *(f32x4*)(orow + 8 * j) = w;
      }
    }
    __syncthreads();
    {   // per-row scale: 8 threads per row, 72 elements each
      const int row = tid >> 3, part = tid & 7;
      const float* src = (const float*)(out_s + row * OUT_STRIDE) + part * 72;
      float mx = 0.f;
#pragma unroll
      for (int e = 0; e < 72; e += 4) {
        const f32x4 w = *(const f32x4*)(src + e);
        mx = fmaxf(fmaxf(mx, fmaxf(fabsf(w[0]), fabsf(w[1]))), fmaxf(fabsf(w[2]), fabsf(w[3])));
      }
      mx = fmaxf(mx, __shfl_xor(mx, 1, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 2, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 4, 64));
      const bool finite = mx > 0.f && mx < INFINITY;
      if (part == 0) {
        inv_s[row] = finite ? 32767.0f / mx : 0.f;
        row_scale[dst_s[tile * BI + row]] = finite ? mx / 32767.0f : 0.f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 9; it++) {
      const int id = it * 256 + tid;
      const int key = id / 72, ch = id % 72;
      const float inv = inv_s[key];
      const float* src = (const float*)(out_s + key * OUT_STRIDE) + ch * 8;
      const f32x4 lo4 = *(const f32x4*)src, hi4 = *(const f32x4*)(src + 4);
      int qv[8];
#pragma unroll
      for (int e = 0; e < 4; e++) { qv[e] = __float2int_rn(lo4[e] * inv); qv[4 + e] = __float2int_rn(hi4[e] * inv); }
      uint4 val;
      val.x = (unsigned)(qv[0] & 0xffff) | ((unsigned)qv[1] << 16);
      val.y = (unsigned)(qv[2] & 0xffff) | ((unsigned)qv[3] << 16);
      val.z = (unsigned)(qv[4] & 0xffff) | ((unsigned)qv[5] << 16);
      val.w = (unsigned)(qv[6] & 0xffff) | ((unsigned)qv[7] << 16);
      *(uint4*)(rows + (size_t)dst_s[tile * BI + key] * ROW_BYTES + ch * 16) = val;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// pass D: dKV[key] = sum of the key's rows, ascending query order
// ---------------------------------------------------------------------------------------------
// One 288-thread workgroup per key: 72 column chunks of 8 elements x 4 row groups (row r of the
// segment goes to group r % 4); the four partial sums are combined in a fixed order, so the result
// depends only on the segment, never on scheduling.  Pure streaming reads of 1152-byte rows.
__global__ __launch_bounds__(288) void bwd_reduce_kernel(const unsigned char* __restrict__ rows, const float* __restrict__ row_scale,
                                                         const int* __restrict__ start, float* __restrict__ dkv_acc, int Skv,
                                                         int accumulate) {
  __shared__ float part[4][DQK];
  const int key = blockIdx.x;
  const int ch = threadIdx.x % 72, grp = threadIdx.x / 72;
  const int s0 = start[key], s1 = start[key + 1];
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; e++) acc[e] = 0.f;
  for (int rr = s0 + grp; rr < s1; rr += 4) {
    const uint4 v = *(const uint4*)(rows + (size_t)rr * ROW_BYTES + ch * 16);
    const float sc = row_scale[rr];
    const int w[4] = {(int)v.x, (int)v.y, (int)v.z, (int)v.w};
#pragma unroll
    for (int e = 0; e < 4; e++) {
      acc[2 * e] = fmaf((float)((w[e] << 16) >> 16), sc, acc[2 * e]);
      acc[2 * e + 1] = fmaf((float)(w[e] >> 16), sc, acc[2 * e + 1]);
    }
  }
#pragma unroll
  for (int e = 0; e < 8; e++) part[grp][ch * 8 + e] = acc[e];
  __syncthreads();
  for (int d = threadIdx.x; d < DQK; d += 288) {
    const float s = (part[0][d] + part[1][d]) + (part[2][d] + part[3][d]);
    float* p = dkv_acc + (size_t)key * DQK + d;
    *p = accumulate ? *p + s : s;
  }
}

__global__ void cast_bf16_kernel(const float* __restrict__ src, unsigned short* __restrict__ dstp, size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x)
    dstp[e] = f32_to_bf16_bits(src[e]);
}

// ---------------------------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------------------------
struct BwdPlan {
  int chunk;            // queries per pass over the buffers
  int W;                // bitmap words per key
  size_t off_bitmap, off_prefix, off_count, off_start, off_dst, off_pds, off_rows, off_scale, off_acc, total;
};

size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }

BwdPlan layout_plan(int chunk, int Skv, int K) {
  BwdPlan p;
  p.chunk = chunk;
  p.W = (chunk + 31) / 32;
  size_t o = 0;
  p.off_bitmap = o; o = align_up(o + (size_t)Skv * p.W * 4);
  p.off_prefix = o; o = align_up(o + (size_t)Skv * p.W * 4);
  p.off_count = o; o = align_up(o + (size_t)(Skv + 1) * 4);
  p.off_start = o; o = align_up(o + (size_t)(Skv + 1) * 4);
  p.off_dst = o; o = align_up(o + (size_t)chunk * K * 4);
  p.off_pds = o; o = align_up(o + (size_t)chunk * (K / BI) * PDS_TILE_BYTES);
  p.off_rows = o; o = align_up(o + ((size_t)chunk * K + 1) * ROW_BYTES);
  p.off_scale = o; o = align_up(o + ((size_t)chunk * K + 1) * 4);
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

constexpr size_t DEFAULT_BUDGET = (size_t)40 << 30;

}  // namespace

extern "C" size_t dsa_sparse_mla_bwd_workspace_bytes(int S, int H, int Skv, int K) {
  (void)H;
  if (S <= 0 || Skv <= 0 || K <= 0) return 0;
  return make_plan(S, Skv, K, DEFAULT_BUDGET).total;
}

static int bwd_impl(const void* q, const void* kv, const void* out, const void* dout, const int32_t* ids,
                    const float* lse, int S, int H, int Skv, int K, int q_start, float sm_scale, int d_v,
                    void* dq, void* dkv, void* workspace, size_t workspace_bytes, void* stream, float* pass_ms) {
  DSA_REQUIRE(d_v == DV, "dsa_sparse_mla_bwd: only d_v = 512 (d_qk = 576) is supported, got d_v = %d", d_v);
  DSA_REQUIRE(S >= 0 && Skv > 0, "dsa_sparse_mla_bwd: bad sequence sizes S=%d Skv=%d", S, Skv);
  DSA_REQUIRE(H > 0 && H <= 128 && H % 32 == 0, "dsa_sparse_mla_bwd: head count must be 32, 64, 96 or 128, got %d", H);
  DSA_REQUIRE(K > 0 && K % 64 == 0 && K <= 2048, "dsa_sparse_mla_bwd: top-k must be a multiple of 64 up to 2048, got %d", K);
  DSA_REQUIRE((size_t)Skv * DQK * 2 <= 0xffffffffull, "dsa_sparse_mla_bwd: kv larger than 4 GiB is not supported");
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
  int* dstp = (int*)(ws + p.off_dst);
  unsigned char* pds = ws + p.off_pds;
  unsigned char* rows = ws + p.off_rows;
  float* row_scale = (float*)(ws + p.off_scale);
  float* acc = (float*)(ws + p.off_acc);
  const int NT = K / BI;

  const size_t smemA = (size_t)4 * TILE_BYTES + ids_lds_bytes(K) + 16 + 1024;
  const size_t smemB = (size_t)3 * (TILE_BYTES + PDS_KIND_BYTES) + ids_lds_bytes(K);
  const size_t smemC = (size_t)2 * PDS_TILE_BYTES + (size_t)BI * OUT_STRIDE + 4 * 8192 + ids_lds_bytes(K) + 16 + (size_t)K * 4 + 128;
  if (hipFuncSetAttribute((const void*)bwd_pds_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smemA) != hipSuccess ||
      hipFuncSetAttribute((const void*)bwd_dq_kernel<3>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smemB) != hipSuccess ||
      hipFuncSetAttribute((const void*)bwd_dkv_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smemC) != hipSuccess)
    DSA_FAIL(DSA_ERR_LAUNCH, "dsa_sparse_mla_bwd: cannot reserve LDS");

  // optional per-pass timing (profiling entry point only): events between the passes
  hipEvent_t ev[6];
  if (pass_ms) {
    for (int i = 0; i < 5; i++) pass_ms[i] = 0.f;
    for (int i = 0; i < 6; i++) if (hipEventCreate(&ev[i]) != hipSuccess) DSA_FAIL(DSA_ERR_LAUNCH, "dsa_sparse_mla_bwd_profile: cannot create events");
  }
#define DSA_MARK(i) do { if (pass_ms) hipEventRecord(ev[i], st); } while (0)
  bool first = true;
  for (int q0 = 0; q0 < S; q0 += p.chunk) {
    const int cnt = S - q0 < p.chunk ? S - q0 : p.chunk;
    DSA_MARK(0);
    order::build(ids, q0, cnt, K, Skv, q_start, bitmap, prefix, count, start, dstp, p.W, st);
    DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(order)");
    DSA_MARK(1);
    bwd_pds_kernel<4><<<dim3(cnt), dim3(256), smemA, st>>>((const __bf16*)q, (const __bf16*)kv, ids, (const __bf16*)out,
                                                          (const __bf16*)dout, lse, pds, q0, cnt, H, Skv, K, q_start, sm_scale);
    DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(P, dS)");
    DSA_MARK(2);
    bwd_dq_kernel<3><<<dim3(cnt), dim3(256), smemB, st>>>((const __bf16*)kv, ids, pds, (__bf16*)dq, q0, cnt, H, Skv, K, q_start);
    DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(dQ)");
    DSA_MARK(3);
    bwd_dkv_kernel<<<dim3(cnt), dim3(256), smemC, st>>>((const __bf16*)q, (const __bf16*)dout, ids, pds, dstp, rows, row_scale, q0, cnt,
                                                       H, Skv, K, q_start, p.chunk * K);
    DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(dKV rows)");
    DSA_MARK(4);
    bwd_reduce_kernel<<<dim3(Skv), dim3(288), 0, st>>>(rows, row_scale, start, acc, Skv, first ? 0 : 1);
    DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(dKV reduce)");
    DSA_MARK(5);
    if (pass_ms) {
      hipEventSynchronize(ev[5]);
      for (int i = 0; i < 5; i++) { float ms = 0.f; hipEventElapsedTime(&ms, ev[i], ev[i + 1]); pass_ms[i] += ms; }
    }
    first = false;
  }
  if (S == 0) {
    order::zero_u32_kernel<<<dim3(256), dim3(256), 0, st>>>((unsigned*)acc, (size_t)Skv * DQK);
  }
  cast_bf16_kernel<<<dim3(2048), dim3(256), 0, st>>>(acc, (unsigned short*)dkv, (size_t)Skv * DQK);
  DSA_CHECK_LAUNCH("dsa_sparse_mla_bwd(cast)");
  (void)NT;
  if (pass_ms) for (int i = 0; i < 6; i++) hipEventDestroy(ev[i]);
#undef DSA_MARK
  return DSA_OK;
}

extern "C" int dsa_sparse_mla_bwd(const void* q, const void* kv, const void* out, const void* dout, const int32_t* ids,
                                  const float* lse, int S, int H, int Skv, int K, int q_start, float sm_scale, int d_v,
                                  void* dq, void* dkv, void* workspace, size_t workspace_bytes, void* stream) {
  return bwd_impl(q, kv, out, dout, ids, lse, S, H, Skv, K, q_start, sm_scale, d_v, dq, dkv, workspace, workspace_bytes,
                  stream, nullptr);
}

extern "C" int dsa_sparse_mla_bwd_profile(const void* q, const void* kv, const void* out, const void* dout,
                                          const int32_t* ids, const float* lse, int S, int H, int Skv, int K, int q_start,
                                          float sm_scale, int d_v, void* dq, void* dkv, void* workspace,
                                          size_t workspace_bytes, void* stream, float* pass_ms) {
  DSA_REQUIRE(pass_ms != nullptr, "dsa_sparse_mla_bwd_profile: pass_ms must point at 5 floats");
  return bwd_impl(q, kv, out, dout, ids, lse, S, H, Skv, K, q_start, sm_scale, d_v, dq, dkv, workspace, workspace_bytes,
                  stream, pass_ms);
}
