// Sparse MQA-MLA attention forward for gfx950.
//
// One 256-thread workgroup (4 waves) per query; wave w owns heads [32w, 32w+32).  The query's
// selected latent rows are gathered 32 at a time straight from global memory into LDS
// (global_load_lds, 16 B per lane, STAGES tiles in flight) in a layout of nine 128-byte groups per
// key row with an XOR swizzle on the 16-byte slot, so both MFMA operand reads below are spread
// over the LDS banks:
//   S^T[key, head] = KV_tile . Q^T      36 x v_mfma_f32_32x32x16_bf16, A = KV rows from LDS
//                                         (ds_read_b128), B = this wave's Q slice held in registers
//   O^T[dv, head] += V_tile^T . P^T     32 x MFMA, A = LDS transpose reads (ds_read_b64_tr_b16),
//                                         B = the softmaxed S^T accumulators re-used in place
// With S^T a lane owns one head (column), so the online-softmax statistics are per lane and need
// one cross-lane exchange per tile; the accumulator layout of S^T is, up to a fixed permutation
// of the keys inside a tile, the B-operand layout of the second product, so P never touches LDS.
// MFMA-bound: 2*H*(576+512) flop per (query, key) pair against 1152 gathered bytes.
#include "mla_tile.h"

namespace {
using namespace mla;

constexpr int DTILES = DV / 32;              // 16

// S^T MFMAs are issued through inline asm so that their accumulator lives in architectural VGPRs:
// the 256 accumulation registers are exactly the O^T accumulators, and a 17th accumulator tuple
// there would force the register allocator to shuffle tuples between the two register files.
// Back-to-back MFMAs that accumulate into the same registers need no software wait states; the
// consumer of the finished chain does (mfma_chain_done).
__device__ __forceinline__ void mfma_first(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_next(f32x16& acc, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_chain_done(f32x16& acc) {
  // 8-pass MFMA result -> VALU read needs 11 wait states; leave a margin
  asm volatile("s_nop 15\n\ts_nop 3" : "+v"(acc));
}

// The softmax of a head is taken relative to a reference point fixed before the first P.V
// product, so the O^T accumulators are never rescaled.  The fast pass (EXACT = false) uses the
// maximum of the first tile; a query in which a later tile exceeds that by more than 2^64 is
// marked (NaN with a payload in lse) and redone by the EXACT = true pass, which first finds the
// true row maximum with an extra sweep of S^T over all tiles.
constexpr unsigned LSE_REDO_MARK = 0x7fc0d5a0u;

// One query, by the 256 threads of a workgroup.
template <int STAGES, int POUT, bool EXACT>   // POUT: 0 none, 1 bf16, 2 f32
__device__ __forceinline__ void fwd_query(
    const __bf16* __restrict__ q, const __bf16* __restrict__ kv, const int* __restrict__ ids,
    __bf16* __restrict__ out, float* __restrict__ lse, void* __restrict__ p_out,
    int S, int H, int Skv, int K, int q_start, float sm_scale, const float* __restrict__ sink, int p_skip, int qi) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, g = lane >> 5;
  const int qpos = q_start + qi;
  const int NT = K / BI;

  int* idx_s = (int*)(smem + STAGES * TILE_BYTES);
  unsigned* tmask = (unsigned*)(idx_s + K);
  int* tlist = (int*)(tmask + NT);
  int* ntile_s = tlist + NT;

  // ---- this wave's Q slice as the B operand of S^T = KV . Q^T, requested before the ids are staged
  // so that both come back in one round trip to memory ---------------------------------------------
  const int h = wave * 32 + r;
  const bool head_ok = h < H;
  bf16x8 qreg[KSTEPS];
  {
    const bf16x8* qp = (const bf16x8*)(q + ((size_t)qi * H + (head_ok ? h : 0)) * DQK) + g;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) qreg[ks] = qp[2 * ks];
  }
  __builtin_amdgcn_sched_barrier(0);

  // ---- stage the ids, mark valid slots, list the tiles that have any ---------------------
  const int ntiles = stage_ids(ids, qi, K, Skv, qpos, idx_s, tmask, tlist, ntile_s);
  // the slice must have landed before the gather pipeline starts: the loop below counts
  // outstanding vector-memory operations by hand
  DSA_WAIT_VMCNT(0);
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ks++) asm volatile("" : "+v"(qreg[ks]));

  // slots of tiles that are never visited still need their -inf in p_out
  // (p_out holds the slots from p_skip on: its rows are K - p_skip wide)
  if (POUT != 0 && head_ok && ntiles < NT) {
    for (int t = p_skip / BI; t < NT; t++) {
      if (tmask[t] != 0u) continue;
      const size_t pbase = ((size_t)qi * H + h) * (K - p_skip) + (size_t)(t * BI - p_skip) + 16 * g;
      if (POUT == 2) {
        const f32x4 ninf = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
#pragma unroll
        for (int j = 0; j < 4; j++) *(f32x4*)((float*)p_out + pbase + 4 * j) = ninf;
      } else {
        const uint4 ninf = make_uint4(0xff80ff80u, 0xff80ff80u, 0xff80ff80u, 0xff80ff80u);
#pragma unroll
        for (int j = 0; j < 2; j++) *(uint4*)((unsigned short*)p_out + pbase + 8 * j) = ninf;
      }
    }
  }

  // ---- gather of tile n of the list into ring slot n % STAGES; lane-dependent LDS offsets ----
  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  auto issue = [&](int n) { gather_tile(kv, idx_s, tlist[n], lds0 + (unsigned)((n % STAGES) * TILE_BYTES)); };
  // The same gather in nine steps (one 128-byte group of the key rows each), issued between MFMAs:
  // nine transfers in a row hold the wave until the memory pipeline has taken them all (about 520
  // clocks per tile of 4200).
  unsigned g_goff = 0, g_lb = 0;
  auto gather_prepare = [&](int n) {
    const int gkey = tid >> 3, gsub = tid & 7;
    int kid = idx_s[tlist[n] * BI + gkey];
    kid = kid < 0 ? 0 : kid;
    g_goff = (unsigned)kid * (DQK * 2) + (unsigned)((gsub ^ swz(gkey)) * 16);
    g_lb = __builtin_amdgcn_readfirstlane(lds0 + (unsigned)((n % STAGES) * TILE_BYTES + wave * 1024));
  };
  auto gather_step = [&](int grp) { dma16(g_lb + grp * GRP_BYTES, g_goff + grp * 128, kv); };
  const LaneOffsets lo = lane_offsets();
  const unsigned (&qk_off)[4] = lo.row_off;          // A operand of S^T: row r, 16-byte chunk 2*ks + g
  const unsigned (&pv_off)[2][2][2] = lo.tr_off;     // A operand of O^T: transpose reads, [s][t][dt & 1]

  const float c2 = sm_scale * LOG2E;
  float m_ref = -1e30f, l_run = 0.f;
  bool overflow = false;
  f32x16 oacc[DTILES];
#pragma unroll
  for (int dt = 0; dt < DTILES; dt++)
#pragma unroll
    for (int e = 0; e < 16; e++) oacc[dt][e] = 0.f;

  // S^T of the tile in stage buffer tb.  Operand reads run four k-steps ahead of the MFMAs; the
  // scheduling fences keep that order (and with it the register budget: Q slice 144 + O^T
  // accumulators 256 of 512 per lane).
  auto qk_tile = [&](const unsigned char* tb, unsigned mask, f32x16& sacc, bool gather) {
    bf16x8 a[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) a[ks] = *(const bf16x8*)(tb + (ks >> 2) * GRP_BYTES + qk_off[ks & 3]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ks++) {
      if (ks == 0) mfma_first(sacc, a[0], qreg[0]);
      else mfma_next(sacc, a[ks & 3], qreg[ks]);
      if (ks + 4 < KSTEPS) a[ks & 3] = *(const bf16x8*)(tb + ((ks + 4) >> 2) * GRP_BYTES + qk_off[ks & 3]);
      if (ks % 7 == 3 && gather) gather_step(ks / 7);          // groups 0 .. 4
      __builtin_amdgcn_sched_barrier(0);
    }
    mfma_chain_done(sacc);
    // accumulator e of this lane is key 8*(e/4) + 4*g + (e%4) of the tile
    if (mask != 0xffffffffu) {
      const unsigned mg = mask >> (4 * g);
#pragma unroll
      for (int e = 0; e < 16; e++)
        if (!((mg >> (8 * (e >> 2) + (e & 3))) & 1u)) sacc[e] = -INFINITY;
    }
  };
  auto tile_max = [&](const f32x16& sacc) {
    float mx = sacc[0];
#pragma unroll
    for (int e = 1; e < 16; e++) mx = fmaxf(mx, sacc[e]);
    return fmaxf(mx, __shfl_xor(mx, 32, 64)) * c2;
  };
  auto wait_tile = [&](int n) {
    const int ahead = min(STAGES - 2, ntiles - 1 - n);   // tiles allowed to stay in flight
    if (ahead >= 2) { DSA_WAIT_VMCNT(18); }
    else if (ahead == 1) { DSA_WAIT_VMCNT(9); }
    else { DSA_WAIT_VMCNT(0); }
    __syncthreads();
  };

  if (EXACT) {   // extra sweep: true maximum of every head over all valid slots
    for (int n = 0; n < STAGES - 1 && n < ntiles; n++) issue(n);
    for (int n = 0; n < ntiles; n++) {
      wait_tile(n);
      if (n + STAGES - 1 < ntiles) issue(n + STAGES - 1);
      f32x16 sacc;
      qk_tile(smem + (n % STAGES) * TILE_BYTES, tmask[tlist[n]], sacc, false);
      m_ref = fmaxf(m_ref, tile_max(sacc));
    }
    __syncthreads();
  }

  for (int n = 0; n < STAGES - 1 && n < ntiles; n++) issue(n);

  for (int n = 0; n < ntiles; n++) {
    wait_tile(n);
    const bool more = n + STAGES - 1 < ntiles;
    if (more) gather_prepare(n + STAGES - 1);

    const int tile = tlist[n];
    const unsigned mask = tmask[tile];
    const unsigned char* tb = smem + (n % STAGES) * TILE_BYTES;

    f32x16 sacc;
    qk_tile(tb, mask, sacc, more);
    if (POUT != 0 && head_ok && tile * BI >= p_skip) {
      const size_t prow = ((size_t)qi * H + h) * (K - p_skip) + (size_t)(tile * BI - p_skip);
      if (POUT == 2) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
          f32x4 v = {sacc[4 * j], sacc[4 * j + 1], sacc[4 * j + 2], sacc[4 * j + 3]};
          *(f32x4*)((float*)p_out + prow + 4 * g + 8 * j) = v;
        }
      } else {
        // A lane holds keys 8j + 4g .. +3 of its head (j = 0..3): 8-byte pieces.  The two half-waves
        // trade pieces so that each lane ends up with 8 consecutive keys, twice: 16-byte stores.
        uint4 o[2];
        acc_row_to_16B(sacc, 1.0f, o);
        *(uint4*)((unsigned short*)p_out + prow + 8 * g) = o[0];
        *(uint4*)((unsigned short*)p_out + prow + 16 + 8 * g) = o[1];
      }
    }

    // ---- softmax numerators (base 2), one head per lane -----------------------------------
    {
      const float mx = tile_max(sacc);
      if (!EXACT) {
        if (n == 0) m_ref = mx;
        overflow |= (mx > m_ref + 64.0f);
      }
    }
    bf16x8 pb[2];
    {
      float psum = 0.f;
#pragma unroll
      for (int s = 0; s < 2; s++)
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float pe = __builtin_amdgcn_exp2f(fmaf(sacc[8 * s + e], c2, -m_ref));
          psum += pe;
          pb[s][e] = (__bf16)pe;
        }
      l_run += psum;
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- O^T += V^T . P^T -----------------------------------------------------------------
    {
      typedef short i16x8 __attribute__((ext_vector_type(8)));
      i16x4 v[2][2][2];   // [ring][s][t]
#pragma unroll
      for (int dt = 0; dt < 2; dt++)
#pragma unroll
        for (int s = 0; s < 2; s++)
#pragma unroll
          for (int t = 0; t < 2; t++)
            v[dt][s][t] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                LDS_PTR(i16x4, tb + (dt >> 1) * GRP_BYTES + pv_off[s][t][dt & 1]));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int dt = 0; dt < DTILES; dt++) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
          i16x8 av = __builtin_shufflevector(v[dt & 1][s][0], v[dt & 1][s][1], 0, 1, 2, 3, 4, 5, 6, 7);
          oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av), pb[s], oacc[dt], 0, 0, 0);
        }
        if (dt + 2 < DTILES) {
#pragma unroll
          for (int s = 0; s < 2; s++)
#pragma unroll
            for (int t = 0; t < 2; t++)
              v[dt & 1][s][t] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                  LDS_PTR(i16x4, tb + ((dt + 2) >> 1) * GRP_BYTES + pv_off[s][t][dt & 1]));
        }
        if (dt % 4 == 1 && more) gather_step(5 + dt / 4);        // groups 5 .. 8
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // ---- epilogue: normalise, write out[i,h,:] and lse[i,h] ---------------------------------
  float l_tot = l_run + __shfl_xor(l_run, 32, 64);
  if (!EXACT && __ballot(overflow) != 0ull) {
    // leave the query to the exact pass (it rewrites out, lse and p_out of all heads)
    if (lane == 0 && wave * 32 < H) ((unsigned*)lse)[(size_t)qi * H + wave * 32] = LSE_REDO_MARK;
    return;
  }
  float o_scale = 1.0f;
  if (sink) {
    // per-head sink logit: one more term exp(sink) in the denominator, with no value row.  The
    // reference point moves to max(reference, sink) so that neither term can overflow; a query
    // without any valid slot ends with lse = sink and a zero output row.
    const float sk2 = sink[head_ok ? h : 0] * LOG2E;
    const float nm = fmaxf(m_ref, sk2);
    o_scale = exp2f(m_ref - nm);
    l_tot = l_tot * o_scale + exp2f(sk2 - nm);
    m_ref = nm;
  }
  const float inv = l_tot > 0.f ? o_scale / l_tot : 0.f;
  if (head_ok) {
    if (g == 0) lse[(size_t)qi * H + h] = l_tot > 0.f ? (m_ref + log2f(l_tot)) * 0.6931471805599453f : INFINITY;
    unsigned short* op = (unsigned short*)out + ((size_t)qi * H + h) * DV + 8 * g;
#pragma unroll
    for (int dt = 0; dt < DTILES; dt++) {
      uint4 o[2];
      acc_row_to_16B(oacc[dt], inv, o);       // head_ok is the same for all lanes of a wave
      *(uint4*)(op + 32 * dt) = o[0];
      *(uint4*)(op + 32 * dt + 16) = o[1];
    }
  }
}

// Fast pass: workgroup b takes query S - 1 - b (longest prefixes first).  Exact pass: workgroup b
// looks at the marks of queries 32b .. 32b + 31 with one load per lane and redoes the marked ones,
// so that a launch in which nothing is marked costs a few microseconds, not a full-size workgroup
// per query.
template <int STAGES, int POUT, bool EXACT>
__global__ __launch_bounds__(256, 1) void mla_fwd_kernel(
    const __bf16* __restrict__ q, const __bf16* __restrict__ kv, const int* __restrict__ ids,
    __bf16* __restrict__ out, float* __restrict__ lse, void* __restrict__ p_out,
    int S, int H, int Skv, int K, int q_start, float sm_scale, const float* __restrict__ sink, int p_skip) {
  if (!EXACT) {
    fwd_query<STAGES, POUT, false>(q, kv, ids, out, lse, p_out, S, H, Skv, K, q_start, sm_scale, sink, p_skip,
                                   S - 1 - (int)blockIdx.x);
    return;
  }
  const int qc = (int)blockIdx.x * 32 + (int)(threadIdx.x & 31);
  bool redo = false;
  if (qc < S) {
    const unsigned* lw = (const unsigned*)lse + (size_t)qc * H;
    for (int w = 0; w * 32 < H; w++) redo |= (lw[w * 32] == LSE_REDO_MARK);
  }
  unsigned todo = (unsigned)__ballot(redo);      // every wave reads the same 32 marks before any of them is rewritten
  while (todo) {
    const int b = __builtin_ctz(todo);
    todo &= todo - 1;
    fwd_query<STAGES, POUT, true>(q, kv, ids, out, lse, p_out, S, H, Skv, K, q_start, sm_scale, sink, p_skip,
                                  (int)blockIdx.x * 32 + b);
    __syncthreads();
  }
}

template <int STAGES>
int launch_fwd(const void* q, const void* kv, const int32_t* ids, int S, int H, int Skv, int K, int q_start,
               float sm_scale, void* out, float* lse, void* p_out, int p_out_f32, const float* sink, int p_skip, hipStream_t st) {
  const size_t smem = (size_t)STAGES * TILE_BYTES + (size_t)K * 4 + (size_t)(K / BI) * 8 + 16;   // ids, tile masks, tile list, counters
  if (smem > 160 * 1024) return -1;
  dim3 grid(S), block(256);
#define DSA_FWD_LAUNCH(P) do { \
    auto kern = mla_fwd_kernel<STAGES, P, false>; \
    auto kern2 = mla_fwd_kernel<STAGES, P, true>; \
    if (dsa_reserve_lds((const void*)kern, smem) != hipSuccess) return -2; \
    if (dsa_reserve_lds((const void*)kern2, smem) != hipSuccess) return -2; \
    kern<<<grid, block, smem, st>>>((const __bf16*)q, (const __bf16*)kv, ids, (__bf16*)out, lse, p_out, S, H, Skv, K, q_start, sm_scale, sink, p_skip); \
    kern2<<<dim3((S + 31) / 32), block, smem, st>>>((const __bf16*)q, (const __bf16*)kv, ids, (__bf16*)out, lse, p_out, S, H, Skv, K, q_start, sm_scale, sink, p_skip); \
  } while (0)
  if (!p_out) DSA_FWD_LAUNCH(0);
  else if (!p_out_f32) DSA_FWD_LAUNCH(1);
  else DSA_FWD_LAUNCH(2);
#undef DSA_FWD_LAUNCH
  return 0;
}

}  // namespace

extern "C" int dsa_sparse_mla_fwd_ex(const void* q, const void* kv, const int32_t* ids, int S, int H, int Skv, int K,
                                     int q_start, float sm_scale, int d_v, void* out, float* lse, void* p_out,
                                     int p_out_f32, const float* attn_sink, int p_out_skip, void* stream) {
  DSA_REQUIRE(d_v == DV, "dsa_sparse_mla_fwd: only d_v = 512 (d_qk = 576) is supported, got d_v = %d", d_v);
  DSA_REQUIRE(S >= 0 && Skv > 0, "dsa_sparse_mla_fwd: bad sequence sizes S=%d Skv=%d", S, Skv);
  DSA_REQUIRE(H > 0 && H <= 128 && H % 32 == 0, "dsa_sparse_mla_fwd: head count must be 32, 64, 96 or 128, got %d", H);
  DSA_REQUIRE(K > 0 && K % 64 == 0, "dsa_sparse_mla_fwd: top-k must be a positive multiple of 64, got %d", K);
  DSA_REQUIRE(p_out_skip >= 0 && p_out_skip < K && p_out_skip % BI == 0,
              "dsa_sparse_mla_fwd: p_out_skip must be a multiple of %d in [0, top-k), got %d", BI, p_out_skip);
  DSA_REQUIRE((size_t)Skv * DQK * 2 <= 0xffffffffull, "dsa_sparse_mla_fwd: kv larger than 4 GiB is not supported");
  DSA_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)kv % 16) == 0 && ((uintptr_t)out % 8) == 0 &&
              ((uintptr_t)p_out % 16) == 0 && ((uintptr_t)attn_sink % 4) == 0, "dsa_sparse_mla_fwd: misaligned pointer");
  if (S == 0) return DSA_OK;
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (K <= 2048) rc = launch_fwd<4>(q, kv, ids, S, H, Skv, K, q_start, sm_scale, out, lse, p_out, p_out_f32, attn_sink, p_out ? p_out_skip : 0, st);
  else if (K <= 8192) rc = launch_fwd<3>(q, kv, ids, S, H, Skv, K, q_start, sm_scale, out, lse, p_out, p_out_f32, attn_sink, p_out ? p_out_skip : 0, st);
  else rc = -1;
  DSA_REQUIRE(rc != -1, "dsa_sparse_mla_fwd: top-k %d exceeds the supported maximum 8192", K);
  if (rc == -2) DSA_FAIL(DSA_ERR_LAUNCH, "dsa_sparse_mla_fwd: cannot reserve LDS");
  DSA_CHECK_LAUNCH("dsa_sparse_mla_fwd");
  return DSA_OK;
}

extern "C" int dsa_sparse_mla_fwd(const void* q, const void* kv, const int32_t* ids, int S, int H, int Skv, int K,
                                  int q_start, float sm_scale, int d_v, void* out, float* lse, void* p_out,
                                  int p_out_f32, void* stream) {
  return dsa_sparse_mla_fwd_ex(q, kv, ids, S, H, Skv, K, q_start, sm_scale, d_v, out, lse, p_out, p_out_f32, nullptr, 0, stream);
}
