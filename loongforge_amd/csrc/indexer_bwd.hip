// Sparse backward of the lightning-indexer logits for gfx950, deterministic.
//
// For every selected pair (query i, slot t, key j = ids[i,t]) with upstream gradient g[i,t]:
//   r_h = q8[i,h,:] . k8[j,:]            a = g[i,t] * k_scale[j]          e_h = a * q_w[i,h] * [r_h > 0]
//   d_qw[i,h]   += a * relu(r_h)
//   d_q8[i,h,:] += e_h * k8[j,:]
//   d_k8[j,:]   += sum_h e_h * q8[i,h,:]
// One 256-thread workgroup per query; the four waves each take 32 of the 128 slots of a tile.
//   r        fp8 MFMA (exact products, as in the forward), one key per lane, heads down the registers
//   d_k8 row bf16 MFMA  row^T[d, key] = Q^T[d, head] . E[head, key];  E = the r-accumulator layout,
//            Q^T resident in accumulation registers; the row, rounded to bf16, goes to a pair buffer at
//            the position of a key-sorted order and a second kernel sums every key's rows in fp32 in
//            ascending query order
//   d_q8     bf16 MFMA  dq^T[d, head] += K^T[d, key] . E^T[key, head], both operands by LDS transpose
//            reads (the wave's key rows converted to bf16, and E written back to LDS)
// For d_q8 E is carried as a bf16 pair (hi + lo), so the bf16 products lose nothing visible in fp32
// (q8 and k8 are exact in bf16); the d_k8 rows use the hi part alone, as they are rounded to bf16
// anyway.  No floating-point atomics: every sum has a fixed order.
#include "dsa_common.h"
#include "order.h"

namespace {

constexpr int D = 128;
constexpr int TK = 128;                 // slots per tile
constexpr int TILE_BYTES = TK * D;      // fp8 key rows
constexpr int RED_STRIDE = 132;         // floats per head row of the cross-wave reduction buffer
constexpr int STRIP_STRIDE = 136;       // bytes per key row of the d_k transpose strip (two d-tiles of 64 bytes + bank spread)

typedef short i16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ int swz(int r) { return (r & 7) ^ ((r >> 3) & 1); }
__device__ __forceinline__ int kb_swz(int key) { return ((key & 3) << 2) | ((key >> 2) & 3); }
__device__ __forceinline__ int es_swz(int key) { return 2 * ((key >> 1) & 3) + ((key >> 3) & 1); }
__device__ __forceinline__ void dma16(unsigned lds_base, unsigned goff, const void* gbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_base), "v"(goff), "s"(gbase) : "memory");
}
__device__ __forceinline__ void mfma_a_vv(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_v_av_first(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "a"(a), "v"(b));
}
__device__ __forceinline__ void mfma_v_av(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "a"(a), "v"(b));
}
__device__ __forceinline__ void mfma_done_v(f32x16& acc) { asm volatile("s_nop 15\n\ts_nop 3" : "+v"(acc)); }
__device__ __forceinline__ void mfma_done_a(f32x16& acc) { asm volatile("s_nop 15\n\ts_nop 3" : "+a"(acc)); }

__device__ __forceinline__ bf16x8 tr_pair(const unsigned char* p0, const unsigned char* p1) {
  i16x4 x0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, p0));
  i16x4 x1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(i16x4, p1));
  return __builtin_bit_cast(bf16x8, (i16x8)__builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7));
}

template <int NHT>
__global__ __launch_bounds__(256, 1) void indexer_bwd_kernel(
    const float* __restrict__ gsc, const unsigned char* __restrict__ q8, const unsigned char* __restrict__ k8,
    const float* __restrict__ k_scale, const float* __restrict__ q_w, const int* __restrict__ ids,
    const int* __restrict__ dst, unsigned short* __restrict__ rows, float* __restrict__ d_q8, float* __restrict__ d_qw,
    int q0, int cnt, int Sk, int K, int dummy_row) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  constexpr int HI = 32 * NHT;
  // [2][TILE_BYTES] fp8 key tiles | kb [4 waves][32 keys][256 B] bf16 keys | es [4 waves][2][32 keys][HI] bf16 E |
  // idx_s [K] | a_s [K] | dst_s [K] | dw_red [4][64] | strip [4 waves][32][STRIP_STRIDE]
  unsigned char* kb = smem + 2 * TILE_BYTES;
  unsigned char* es = kb + 4 * 32 * 256;
  int* idx_s = (int*)(es + 4 * 2 * 32 * 128);
  float* a_s = (float*)(idx_s + K);
  int* dst_s = (int*)(a_s + K);
  float* dw_red = (float*)(dst_s + K);
  unsigned char* strip = (unsigned char*)(dw_red + 4 * 64) + (threadIdx.x >> 6) * (32 * STRIP_STRIDE);   // per wave
  float* red = (float*)smem;                        // [HI][RED_STRIDE], reuses the tile area at the end
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int ql = cnt - 1 - (int)blockIdx.x;
  const int qi = q0 + ql;

  for (int t0 = tid; t0 < K; t0 += 8 * 256) {     // eight slots per thread with all their loads in flight
    int v[8], d[8];
    float gv[8], kv[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int t = min(t0 + i * 256, K - 1);
      v[i] = ids[(size_t)qi * K + t];
      gv[i] = gsc[(size_t)qi * K + t];
      d[i] = dst[(size_t)ql * K + t];
    }
#pragma unroll
    for (int i = 0; i < 8; i++) kv[i] = k_scale[(v[i] >= 0 && v[i] < Sk) ? v[i] : 0];
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int t = t0 + i * 256;
      if (t < K) {
        const bool ok = v[i] >= 0 && v[i] < Sk;
        idx_s[t] = ok ? v[i] : -1;
        a_s[t] = ok ? gv[i] * kv[i] : 0.f;
        dst_s[t] = (ok && d[i] >= 0) ? d[i] : dummy_row;
      }
    }
  }
  // stage q8[i] (HI x 128 bytes) in the kb area to build the transposed bf16 operand
  for (int c = tid; c < HI * 8; c += 256) *(uint4*)(kb + c * 16) = *(const uint4*)(q8 + (size_t)qi * HI * D + c * 16);
  __syncthreads();

  // ---- register-resident operands ---------------------------------------------------------
  i32x8 aq[NHT][2];          // fp8 rows of the query: A operand of r
  float wq[NHT][16];         // q_w of the 16 heads a lane sees per head tile
  float dwp[NHT][16];
  bf16x8 qt[4][2 * NHT];     // Q^T: lane = d row (32*dt + r), 8 heads of k-step kk = 2*ht + s
#pragma unroll
  for (int t = 0; t < NHT; t++) {
    const unsigned char* row = q8 + ((size_t)qi * HI + 32 * t + r) * D + 32 * g;
#pragma unroll
    for (int s = 0; s < 2; s++) {
      const i32x4 lo = *(const i32x4*)(row + 64 * s);
      const i32x4 hi = *(const i32x4*)(row + 64 * s + 16);
      aq[t][s] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
    const float* wrow = q_w + (size_t)qi * HI + 32 * t + 4 * g;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const f32x4 w4 = *(const f32x4*)(wrow + 8 * j);
#pragma unroll
      for (int e = 0; e < 4; e++) { wq[t][4 * j + e] = w4[e]; dwp[t][4 * j + e] = 0.f; }
    }
  }
#pragma unroll
  for (int dt = 0; dt < 4; dt++)
#pragma unroll
    for (int kk = 0; kk < 2 * NHT; kk++) {
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const int head = 16 * kk + 8 * (e >> 2) + 4 * g + (e & 3);
        const int byte = kb[head * D + 32 * dt + r];
        qt[dt][kk][e] = (__bf16)__builtin_amdgcn_cvt_f32_fp8(byte, 0);
      }
      asm volatile("" : "+a"(qt[dt][kk]));
    }
  f32x16 dq_acc[NHT][4];
#pragma unroll
  for (int t = 0; t < NHT; t++)
#pragma unroll
    for (int dt = 0; dt < 4; dt++) {
#pragma unroll
      for (int e = 0; e < 16; e++) dq_acc[t][dt][e] = 0.f;
      asm volatile("" : "+a"(dq_acc[t][dt]));
    }
  DSA_WAIT_VMCNT(0);
  __syncthreads();

  // ---- lane-dependent LDS offsets -------------------------------------------------------------
  unsigned b_off[2][2];      // B operand of r: key row r of the wave's 32, bytes [64s + 32g, +32)
#pragma unroll
  for (int s = 0; s < 2; s++)
#pragma unroll
    for (int x = 0; x < 2; x++) b_off[s][x] = (unsigned)((32 * wave + r) * D + (((4 * s + 2 * g + x) ^ swz(r)) << 4));
  const int blk = lane >> 4, ii = lane & 15;
  // transpose reads: lane (blk, ii) points at key 16*s2 + 8*t + 4*g + ii/4, column chunk 16*(blk&1) + 4*(ii&3)
  // Both wave-private buffers XOR the 16-byte slot index with a permutation of the key's bits
  // (kb_swz: 16 slots per 256-byte row, es_swz: 8 slots per 128-byte row), chosen so that the
  // row-wise writes by 16 lanes and the transpose reads by 32 lanes spread over all banks.
  unsigned kt_off[2][2][4], et_off[2][2][NHT];
#pragma unroll
  for (int s2 = 0; s2 < 2; s2++)
#pragma unroll
    for (int t = 0; t < 2; t++) {
      const int key = 16 * s2 + 8 * t + 4 * g + (ii >> 2);
      const int sub = 2 * (blk & 1) + ((ii & 3) >> 1), half = (ii & 1) * 8;
#pragma unroll
      for (int dt = 0; dt < 4; dt++)
        kt_off[s2][t][dt] = (unsigned)(wave * 8192 + key * 256 + (((4 * dt + sub) ^ kb_swz(key)) << 4) + half);
#pragma unroll
      for (int tt = 0; tt < NHT; tt++)
        et_off[s2][t][tt] = (unsigned)(wave * 8192 + key * 128 + (((4 * tt + sub) ^ es_swz(key)) << 4) + half);
    }

  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  const int gkey = tid >> 3, gsub = tid & 7;
  const int ntile = K / TK;
  auto issue = [&](int t) {
    const unsigned lb = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)((t & 1) * TILE_BYTES + wave * 1024));
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const int key = c * 32 + gkey;
      int kid = idx_s[t * TK + key];
      kid = kid < 0 ? 0 : kid;
      dma16(lb + c * 4096, (unsigned)kid * D + (unsigned)((gsub ^ swz(key)) * 16), k8);
    }
  };
  issue(0);
  for (int t = 0; t < ntile; t++) {
    // issued after this tile's 4 transfers: the 16 row stores of the previous tile
    if (t > 0) { DSA_WAIT_VMCNT(16); } else { DSA_WAIT_VMCNT(0); }
    __syncthreads();
    if (t + 1 < ntile) issue(t + 1);
    const unsigned char* tb = smem + (t & 1) * TILE_BYTES;
    const int slot = t * TK + 32 * wave + r;
    const float a = a_s[slot];

    // ---- r, E, d_qw -----------------------------------------------------------------------------
    i32x8 bk[2];
#pragma unroll
    for (int s = 0; s < 2; s++) {
      const i32x4 lo = *(const i32x4*)(tb + b_off[s][0]);
      const i32x4 hi = *(const i32x4*)(tb + b_off[s][1]);
      bk[s] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
    bf16x8 ehi[NHT][2], elo[NHT][2];
#pragma unroll
    for (int tt = 0; tt < NHT; tt++) {
      f32x16 acc;
#pragma unroll
      for (int e = 0; e < 16; e++) acc[e] = 0.f;
      acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(aq[tt][0], bk[0], acc, 0, 0, 0, 127, 0, 127);
      acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(aq[tt][1], bk[1], acc, 0, 0, 0, 127, 0, 127);
#pragma unroll
      for (int e = 0; e < 16; e += 2) {
        // two neighbouring heads at a time: one packed conversion for the bf16 heads of E, one for what they miss
        float ev[2];
#pragma unroll
        for (int x = 0; x < 2; x++) {
          const float rr = acc[e + x];
          dwp[tt][e + x] = fmaf(a, __builtin_bit_cast(float, max(__builtin_bit_cast(int, rr), 0)), dwp[tt][e + x]);   // relu on the bit pattern
          ev[x] = rr > 0.f ? a * wq[tt][e + x] : 0.f;
        }
        const unsigned ph = cvt_pk_bf16(ev[0], ev[1]);
        const unsigned pl = cvt_pk_bf16(ev[0] - __builtin_bit_cast(float, ph << 16), ev[1] - __builtin_bit_cast(float, ph & 0xffff0000u));
        const bf16x2 h2 = __builtin_bit_cast(bf16x2, ph), l2 = __builtin_bit_cast(bf16x2, pl);
        ehi[tt][e >> 3][e & 7] = h2[0]; ehi[tt][e >> 3][(e & 7) + 1] = h2[1];
        elo[tt][e >> 3][e & 7] = l2[0]; elo[tt][e >> 3][(e & 7) + 1] = l2[1];
      }
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- d_k8 rows: row^T[d, key] = Q^T . E, 32 keys of this wave --------------------------------
    {
      // Rows leave as bf16 (the ordered sum over a key's rows runs in fp32; one row carries 2^-9 of
      // relative rounding, so E enters these products as its bf16 head alone).  Two 32 x 32 d-tiles at a
      // time are rounded, transposed through a wave-private LDS strip and stored, so that a store
      // instruction writes eight complete 128-byte row segments (lane: key 8*i + lane/8, 16-byte piece
      // lane%8) instead of scattered 8-byte pieces.
      unsigned short* rowp[4];
#pragma unroll
      for (int i = 0; i < 4; i++)
        rowp[i] = rows + (size_t)dst_s[t * TK + 32 * wave + 8 * i + (lane >> 3)] * D + 8 * (lane & 7);
      unsigned char* sw = strip + r * STRIP_STRIDE + 8 * g;
      const unsigned char* sr = strip + (lane >> 3) * STRIP_STRIDE + (lane & 7) * 16;
      auto row_mfmas = [&](int dt, f32x16& racc) {
        mfma_v_av_first(racc, qt[dt][0], ehi[0][0]);
#pragma unroll
        for (int kk = 1; kk < 2 * NHT; kk++) mfma_v_av(racc, qt[dt][kk], ehi[kk >> 1][kk & 1]);
      };
      f32x16 racc[2];
      row_mfmas(0, racc[0]);
#pragma unroll
      for (int dt = 0; dt < 4; dt++) {
        // the next d-tile's MFMAs run while this one is rounded into the strip
        if (dt + 1 < 4) row_mfmas(dt + 1, racc[(dt + 1) & 1]);
        else mfma_done_v(racc[dt & 1]);
#pragma unroll
        for (int j = 0; j < 4; j++) {                // d = 32*dt + 8*j + 4*g .. +3 of key r
          const uint2 w = make_uint2(cvt_pk_bf16(racc[dt & 1][4 * j], racc[dt & 1][4 * j + 1]),
                                     cvt_pk_bf16(racc[dt & 1][4 * j + 2], racc[dt & 1][4 * j + 3]));
          *(uint2*)(sw + 64 * (dt & 1) + 16 * j) = w;
        }
        if (dt & 1) {
          __builtin_amdgcn_wave_barrier();
#pragma unroll
          for (int i = 0; i < 4; i++) *(uint4*)(rowp[i] + 64 * (dt >> 1)) = *(const uint4*)(sr + 8 * i * STRIP_STRIDE);
          __builtin_amdgcn_wave_barrier();
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- d_q8: this wave's key rows as bf16, E back to LDS, then transpose reads ------------------
    {
      // lane (key r, half g) converts bytes [64g, 64g + 64) of its key row
      const unsigned char* krow = tb + (32 * wave + r) * D;
      unsigned char* kdst = kb + wave * 8192 + r * 256;
      const int ksw = kb_swz(r);
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const int slot16 = (4 * g + c) ^ swz(r);
        const i32x4 w = *(const i32x4*)(krow + slot16 * 16);
        // e4m3 -> bf16 is exact; one instruction converts two bytes of a word
        bf16x8 o0, o1;
#pragma unroll
        for (int x = 0; x < 4; x++) {
          const bf16x2 lo2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[x], 1.0f, false);
          const bf16x2 hi2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[x], 1.0f, true);
          if (x < 2) { o0[4 * x] = lo2[0]; o0[4 * x + 1] = lo2[1]; o0[4 * x + 2] = hi2[0]; o0[4 * x + 3] = hi2[1]; }
          else { o1[4 * (x - 2)] = lo2[0]; o1[4 * (x - 2) + 1] = lo2[1]; o1[4 * (x - 2) + 2] = hi2[0]; o1[4 * (x - 2) + 3] = hi2[1]; }
        }
        *(bf16x8*)(kdst + (((8 * g + 2 * c) ^ ksw) << 4)) = o0;
        *(bf16x8*)(kdst + (((8 * g + 2 * c + 1) ^ ksw) << 4)) = o1;
      }
      // E[key r][heads]: the lane holds heads 32*tt + 8*j + 4*g + (0..3)
      unsigned char* edst = es + wave * 8192 + r * 128;
      const int esw = es_swz(r);
#pragma unroll
      for (int tt = 0; tt < NHT; tt++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const int hb = (((4 * tt + j) ^ esw) << 4) + 8 * g;      // heads 32*tt + 8*j + 4*g .. +3
          bf16x4 vh, vl;
#pragma unroll
          for (int e = 0; e < 4; e++) { vh[e] = ehi[tt][j >> 1][4 * (j & 1) + e]; vl[e] = elo[tt][j >> 1][4 * (j & 1) + e]; }
          *(bf16x4*)(edst + hb) = vh;
          *(bf16x4*)(edst + 4096 + hb) = vl;
        }
      __builtin_amdgcn_wave_barrier();
#pragma unroll
      for (int s2 = 0; s2 < 2; s2++) {
        bf16x8 bh[NHT], bl[NHT];
#pragma unroll
        for (int tt = 0; tt < NHT; tt++) {
          bh[tt] = tr_pair(es + et_off[s2][0][tt], es + et_off[s2][1][tt]);
          bl[tt] = tr_pair(es + 4096 + et_off[s2][0][tt], es + 4096 + et_off[s2][1][tt]);
        }
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
          const bf16x8 ak = tr_pair(kb + kt_off[s2][0][dt], kb + kt_off[s2][1][dt]);
#pragma unroll
          for (int tt = 0; tt < NHT; tt++) {
            mfma_a_vv(dq_acc[tt][dt], ak, bh[tt]);
            mfma_a_vv(dq_acc[tt][dt], ak, bl[tt]);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      __builtin_amdgcn_wave_barrier();
    }
  }

  // ---- d_qw: sum the per-lane partials over the 32 keys of a half-wave, then over waves -----------
#pragma unroll
  for (int tt = 0; tt < NHT; tt++)
#pragma unroll
    for (int e = 0; e < 16; e++) {
      float v = dwp[tt][e];
#pragma unroll
      for (int o = 1; o < 32; o <<= 1) v += __shfl_xor(v, o, 64);
      if (r == 0) dw_red[wave * 64 + 32 * tt + 8 * (e >> 2) + 4 * g + (e & 3)] = v;
    }
  // ---- d_q8: fixed-order sum of the four waves' accumulators through LDS ----------------------------
  DSA_WAIT_VMCNT(0);
  __syncthreads();
  for (int w = 0; w < 4; w++) {
    if (wave == w) {
#pragma unroll
      for (int tt = 0; tt < NHT; tt++)
#pragma unroll
        for (int dt = 0; dt < 4; dt++) {
          mfma_done_a(dq_acc[tt][dt]);
          float* rp = red + (32 * tt + r) * RED_STRIDE + 32 * dt + 4 * g;
#pragma unroll
          for (int j = 0; j < 4; j++) {
            f32x4 v = {dq_acc[tt][dt][4 * j], dq_acc[tt][dt][4 * j + 1], dq_acc[tt][dt][4 * j + 2], dq_acc[tt][dt][4 * j + 3]};
            if (w > 0) { const f32x4 old = *(const f32x4*)(rp + 8 * j); v += old; }
            *(f32x4*)(rp + 8 * j) = v;
          }
        }
    }
    __syncthreads();
  }
  for (int c = tid; c < HI * 32; c += 256) {
    const int h = c >> 5, d4 = c & 31;
    *(f32x4*)(d_q8 + ((size_t)qi * HI + h) * D + 4 * d4) = *(const f32x4*)(red + h * RED_STRIDE + 4 * d4);
  }
  if (tid < HI) d_qw[(size_t)qi * HI + tid] = (dw_red[tid] + dw_red[64 + tid]) + (dw_red[128 + tid] + dw_red[192 + tid]);
}

// d_k8[key] (+)= sum of the key's bf16 rows in fp32, ascending query order; 128 threads = 16 chunks of 8
// columns x 8 row groups (row r of the segment goes to group r % 8), the groups combined in a fixed order
__global__ __launch_bounds__(128) void indexer_reduce_kernel(const unsigned short* __restrict__ rows, const int* __restrict__ start,
                                                             float* __restrict__ d_k8, int accumulate,
                                                             const int* __restrict__ dup_flag) {
  __shared__ float part[8][D];
  const int key = blockIdx.x, ch = threadIdx.x & 15, grp = threadIdx.x >> 4;
  const int s0 = start[key], s1 = start[key + 1];
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; e++) acc[e] = 0.f;
  for (int rr = s0 + grp; rr < s1; rr += 8) {
    const uint4 v = *(const uint4*)(rows + (size_t)rr * D + 8 * ch);
    const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; e++) {
      acc[2 * e] += __builtin_bit_cast(float, w[e] << 16);
      acc[2 * e + 1] += __builtin_bit_cast(float, w[e] & 0xffff0000u);
    }
  }
#pragma unroll
  for (int e = 0; e < 8; e++) part[grp][8 * ch + e] = acc[e];
  __syncthreads();
  {
    const int c = threadIdx.x;      // one column per thread
    float s = ((part[0][c] + part[1][c]) + (part[2][c] + part[3][c])) + ((part[4][c] + part[5][c]) + (part[6][c] + part[7][c]));
    float* p = d_k8 + (size_t)key * D + c;
    if (accumulate) s += *p;
    if (*dup_flag) s = __builtin_nanf("");       // a query row held a repeated id: no sum that misses a term
    *p = s;
  }
}

struct Plan {
  int chunk, W;
  size_t off_bitmap, off_prefix, off_count, off_start, off_flag, off_dst, off_rows, total;
};
size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }
Plan layout_plan(int chunk, int Sk, int K) {
  Plan p;
  p.chunk = chunk;
  p.W = (chunk + 31) / 32;
  size_t o = 0;
  p.off_bitmap = o; o = align_up(o + (size_t)Sk * p.W * 4);
  p.off_prefix = o; o = align_up(o + order::prefix_words(chunk, Sk) * 4);
  p.off_count = o; o = align_up(o + (size_t)(Sk + 1) * 4);
  p.off_start = o; o = align_up(o + (size_t)(Sk + 1) * 4);
  p.off_flag = o; o = align_up(o + 4);
  p.off_dst = o; o = align_up(o + (size_t)chunk * K * 4);
  p.off_rows = o; o = align_up(o + ((size_t)chunk * K + 1) * D * 2);
  p.total = o;
  return p;
}
Plan make_plan(int S, int Sk, int K, size_t budget) {
  int chunk = S;
  Plan p = layout_plan(chunk, Sk, K);
  while (p.total > budget && chunk > 64) {
    chunk = (chunk + 1) / 2;
    p = layout_plan(chunk, Sk, K);
  }
  return p;
}
constexpr size_t DEFAULT_BUDGET = (size_t)16 << 30;

}  // namespace

extern "C" size_t dsa_indexer_bwd_workspace_bytes(int S, int Hi, int Sk, int K) {
  (void)Hi;
  if (S <= 0 || Sk <= 0 || K <= 0) return 0;
  return make_plan(S, Sk, K, DEFAULT_BUDGET).total;
}

extern "C" int dsa_indexer_bwd(const float* g, const void* q8, const void* k8, const float* k_scale, const float* q_w,
                               const int32_t* ids, int S, int Hi, int Sk, int K, float* d_q8, float* d_k8, float* d_qw,
                               void* workspace, size_t workspace_bytes, void* stream) {
  DSA_REQUIRE(Hi == 32 || Hi == 64, "dsa_indexer_bwd: head count must be 32 or 64, got %d", Hi);
  DSA_REQUIRE(S >= 0 && Sk > 0, "dsa_indexer_bwd: bad sizes S=%d Sk=%d", S, Sk);
  DSA_REQUIRE(K > 0 && K % TK == 0 && K <= 4096, "dsa_indexer_bwd: top-k must be a multiple of 128 up to 4096, got %d", K);
  DSA_REQUIRE((size_t)Sk * D <= 0xffffffffull, "dsa_indexer_bwd: key array too large");
  DSA_REQUIRE(Sk <= order::MAX_KEYS, "dsa_indexer_bwd: at most %d keys are supported, got %d", order::MAX_KEYS, Sk);
  DSA_REQUIRE(((uintptr_t)q8 % 16) == 0 && ((uintptr_t)k8 % 16) == 0 && ((uintptr_t)q_w % 16) == 0 &&
              ((uintptr_t)d_q8 % 16) == 0 && ((uintptr_t)d_k8 % 16) == 0 && ((uintptr_t)workspace % 256) == 0,
              "dsa_indexer_bwd: misaligned pointer");
  hipStream_t st = (hipStream_t)stream;
  Plan p = make_plan(S > 0 ? S : 1, Sk, K, workspace_bytes);
  if (p.total > workspace_bytes || workspace == nullptr)
    DSA_FAIL(DSA_ERR_WORKSPACE, "dsa_indexer_bwd: workspace of %zu bytes is too small (need at least %zu)",
             workspace_bytes, layout_plan(64, Sk, K).total);
  unsigned char* ws = (unsigned char*)workspace;
  unsigned* bitmap = (unsigned*)(ws + p.off_bitmap);
  unsigned* prefix = (unsigned*)(ws + p.off_prefix);
  int* count = (int*)(ws + p.off_count);
  int* start = (int*)(ws + p.off_start);
  int* dup_flag = (int*)(ws + p.off_flag);
  int* dstp = (int*)(ws + p.off_dst);
  unsigned short* rows = (unsigned short*)(ws + p.off_rows);
  size_t smem = (size_t)2 * TILE_BYTES + 4 * 32 * 256 + 4 * 2 * 32 * 128 + (size_t)K * 12 + 4 * 64 * 4 + 4 * 32 * STRIP_STRIDE;
  const size_t red_bytes = (size_t)Hi * RED_STRIDE * 4;
  if (red_bytes > (size_t)2 * TILE_BYTES + 4 * 32 * 256) smem += red_bytes;
  auto kern = Hi == 32 ? indexer_bwd_kernel<1> : indexer_bwd_kernel<2>;
  if (dsa_reserve_lds((const void*)kern, smem) != hipSuccess)
    DSA_FAIL(DSA_ERR_LAUNCH, "dsa_indexer_bwd: cannot reserve LDS");
  bool first = true;
  order::clear_flag(dup_flag, st);
  for (int q0 = 0; q0 < S; q0 += p.chunk) {
    const int cnt = S - q0 < p.chunk ? S - q0 : p.chunk;
    // every id inside [0, Sk) counts: the causal window was already applied when the ids were selected
    order::build(ids, q0, cnt, K, Sk, 0x3fffffff, bitmap, prefix, count, start, dstp, p.W, st, dup_flag);
    DSA_CHECK_LAUNCH("dsa_indexer_bwd(order)");
    kern<<<dim3(cnt), dim3(256), smem, st>>>(g, (const unsigned char*)q8, (const unsigned char*)k8, k_scale, q_w, ids, dstp,
                                             rows, d_q8, d_qw, q0, cnt, Sk, K, p.chunk * K);
    DSA_CHECK_LAUNCH("dsa_indexer_bwd");
    indexer_reduce_kernel<<<dim3(Sk), dim3(128), 0, st>>>(rows, start, d_k8, first ? 0 : 1, dup_flag);
    DSA_CHECK_LAUNCH("dsa_indexer_bwd(reduce)");
    first = false;
  }
  if (S == 0) order::zero_u32_kernel<<<dim3(256), dim3(256), 0, st>>>((unsigned*)d_k8, (size_t)Sk * D);
  return DSA_OK;
}
