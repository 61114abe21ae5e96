// MLA weight absorption around the sparse attention kernels, for gfx950: per-head projections
//
//     C[s, h, n] = sum_k A[s, h, k] * W[h, n, k]            (bf16 in, fp32 accumulate, bf16 out)
//
// read and written in place inside larger tensors, so that no permute / split / concatenate copy
// surrounds them:
//   * query side   A = the no-position part of the up-projected query, [S, H, 128] inside [S, H, 192];
//                  W = W_UK^T [H, 512, 128]; C = the latent part of the attention query,
//                  [S, H, 512] inside [S, H, 576] (the rotary part is written by the rotary kernel)
//   * output side  A = the attention output [S, H, 512]; W = W_UV [H, 128, 512];
//                  C = [S, H * 128], the input of the output projection
// HBM-bound (137 GFLOP against 1.3 GB at S = 8192, H = 128): one workgroup holds a head's 128 KB weight
// matrix in LDS for many row blocks; a wave computes C^T[n, s] = W[n, :] . A[s, :]^T for 32 rows s at a
// time, the weights as the MFMA A operand (LDS row reads), the activation rows as the B operand straight
// from global memory (16 bytes per lane, next block requested before this block's MFMAs).  With C^T in
// the accumulators a lane owns one output row, so the result leaves in 16-byte pieces.
#include "mla_tile.h"

namespace {

constexpr int ROWS = 128;                 // activation rows per workgroup step (32 per wave)

template <int K, int N>
__global__ __launch_bounds__(256, 1) void absorb_kernel(
    const __bf16* __restrict__ a, long a_tok, long a_head, const __bf16* __restrict__ w,
    __bf16* __restrict__ c, long c_tok, long c_head, int S, int H, int splits) {
  // W[h] in LDS as K / 64 column groups of [N rows][128 bytes]; inside a group the 16-byte chunk c of row n sits in slot
  // (c & 7) ^ swz(n): the layout of the attention kernels' key tiles, whose 128-bit row reads are bank-conflict free
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  constexpr int KS = K / 16, NT = N / 32, CH = K / 8;                          // k-steps, output tiles, chunks per row
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, g = lane >> 5;
  const int h = blockIdx.x / splits, part = blockIdx.x % splits;

  // ---- the head's weights into LDS -------------------------------------------------------
  {
    const uint4* src = (const uint4*)(w + (size_t)h * N * K);
    for (int e = tid; e < N * CH; e += 256) {
      const int n = e / CH, ch = e % CH;
      *(uint4*)(smem + (size_t)(ch >> 3) * (N * 128) + n * 128 + (((ch & 7) ^ mla::swz(n & 31)) << 4)) = src[e];
    }
  }
  __syncthreads();

  const int nblk = (S + ROWS - 1) / ROWS;
  const int b_lo = (int)((long)nblk * part / splits), b_hi = (int)((long)nblk * (part + 1) / splits);
  auto load_rows = [&](int blk, bf16x8 (&t)[KS]) {
    const int s = min(blk * ROWS + wave * 32 + r, S - 1);
    const bf16x8* p = (const bf16x8*)(a + (size_t)s * a_tok + (size_t)h * a_head) + g;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) t[ks] = p[2 * ks];
  };
  bf16x8 cur[KS], nxt[KS];
  if (b_lo < b_hi) load_rows(b_lo, cur);
  for (int blk = b_lo; blk < b_hi; blk++) {
    if (blk + 1 < b_hi) load_rows(blk + 1, nxt);
    const int s = blk * ROWS + wave * 32 + r;
    unsigned short* out = (unsigned short*)c + (size_t)min(s, S - 1) * c_tok + (size_t)h * c_head + 8 * g;
#pragma unroll 2
    for (int nt = 0; nt < NT; nt++) {
      f32x16 acc;
#pragma unroll
      for (int e = 0; e < 16; e++) acc[e] = 0.f;
      const int n = 32 * nt + r;
      const unsigned char* wrow = smem + n * 128;
      const int sw = mla::swz(r);
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const bf16x8 wv = *(const bf16x8*)(wrow + (ks >> 2) * (N * 128) + ((((2 * ks + g) & 7) ^ sw) << 4));
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wv, cur[ks], acc, 0, 0, 0);
      }
      uint4 o[2];
      acc_row_to_16B(acc, 1.0f, o);          // every lane takes part; rows past the end are not stored
      if (s < S) {
        *(uint4*)(out + 32 * nt) = o[0];
        *(uint4*)(out + 32 * nt + 16) = o[1];
      }
    }
    if (blk + 1 < b_hi) {
#pragma unroll
      for (int ks = 0; ks < KS; ks++) cur[ks] = nxt[ks];
    }
  }
}

template <int K, int N>
int launch(const void* a, int64_t a_tok, int64_t a_head, const void* w, void* c, int64_t c_tok, int64_t c_head,
           int S, int H, hipStream_t st) {
  const int nblk = (S + ROWS - 1) / ROWS;
  int splits = (512 + H - 1) / H;
  if (splits > nblk) splits = nblk;
  if (splits < 1) splits = 1;
  const size_t smem = (size_t)K * N * 2;
  auto kern = absorb_kernel<K, N>;
  static bool configured = false;            // per template instance
  if (!configured) {
    if (dsa_reserve_lds((const void*)kern, smem) != hipSuccess) return -2;
    configured = true;
  }
  kern<<<dim3((unsigned)(H * splits)), dim3(256), smem, st>>>((const __bf16*)a, (long)a_tok, (long)a_head, (const __bf16*)w,
                                                               (__bf16*)c, (long)c_tok, (long)c_head, S, H, splits);
  return 0;
}

}  // namespace

extern "C" int dsa_mla_absorb(const void* a, int64_t a_tok, int64_t a_head, const void* w, void* c, int64_t c_tok,
                              int64_t c_head, int S, int H, int k_dim, int n_dim, void* stream) {
  DSA_REQUIRE(S >= 0 && H > 0, "dsa_mla_absorb: bad sizes S=%d H=%d", S, H);
  DSA_REQUIRE((k_dim == 128 && n_dim == 512) || (k_dim == 512 && n_dim == 128),
              "dsa_mla_absorb: (k, n) must be (128, 512) (query side) or (512, 128) (output side), got (%d, %d)", k_dim, n_dim);
  DSA_REQUIRE(a_tok % 8 == 0 && a_head % 8 == 0 && c_tok % 8 == 0 && c_head % 8 == 0,
              "dsa_mla_absorb: row strides must be multiples of 8 elements");
  DSA_REQUIRE(((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0 && ((uintptr_t)c % 16) == 0, "dsa_mla_absorb: misaligned pointer");
  if (S == 0) return DSA_OK;
  int rc;
  if (k_dim == 128) rc = launch<128, 512>(a, a_tok, a_head, w, c, c_tok, c_head, S, H, (hipStream_t)stream);
  else rc = launch<512, 128>(a, a_tok, a_head, w, c, c_tok, c_head, S, H, (hipStream_t)stream);
  if (rc == -2) DSA_FAIL(DSA_ERR_LAUNCH, "dsa_mla_absorb: cannot reserve LDS");
  DSA_CHECK_LAUNCH("dsa_mla_absorb");
  return DSA_OK;
}
