// Rotary position embedding for the MLA query / key rows around the sparse attention kernels,
// fused with the copies (layout permutation, concatenation) that surround it.  HBM-bound
// elementwise work: every row is read once and written once in 16-byte pieces.
//
// One kernel covers the whole family.  Per (token, head) it
//   * copies a "main" part of d_main elements from one strided tensor to another, and
//   * rotates a "pe" part of emb_dim elements: pair i is (x1_i, x2_i) with
//         y1_i = x1_i * c1_i - x2_i * s1_i          y2_i = x2_i * c2_i + x1_i * s2_i      (forward)
//         y1_i = x1_i * c1_i + x2_i * s2_i          y2_i = x2_i * c2_i - x1_i * s1_i      (inverse: the transpose)
//     in fp32 without fused multiply-adds, rounded once to bf16.
// Where the pair sits in a row is the "pairing": adjacent (elements 2i, 2i+1) or split
// (elements i, i + emb_dim/2); source and destination pairings are independent, and the cos / sin
// rows are indexed with the pairing of the rotated side (destination in the forward direction,
// source in the inverse one): c1_i = cos[2i], c2_i = cos[2i+1] or c1_i = cos[i], c2_i = cos[i + emb_dim/2].
#include "dsa_common.h"

namespace {

constexpr int ADJ = 0, SPLIT = 1;

struct RopeArgs {
  const unsigned short* main_src; long ms_tok, ms_head;     // strides in elements; nullptr: no main part
  unsigned short* main_dst; long md_tok, md_head;
  int d_main;
  const unsigned short* pe_src; long ps_tok, ps_head;
  unsigned short* pe_dst; long pd_tok, pd_head;
  int emb;
  const void* cos; const void* sin; int cs_f32;             // [positions][emb], fp32 or bf16
  const int* positions; int batch;                          // position of a token: positions[t] or t / batch
  int tokens, heads;
};

__device__ __forceinline__ void load4(const void* base, long idx, int f32, float (&o)[4]) {
  if (f32) {
    const f32x4 v = *(const f32x4*)((const float*)base + idx);
    o[0] = v[0]; o[1] = v[1]; o[2] = v[2]; o[3] = v[3];
  } else {
    const uint2 v = *(const uint2*)((const unsigned short*)base + idx);
    o[0] = __builtin_bit_cast(float, v.x << 16); o[1] = __builtin_bit_cast(float, v.x & 0xffff0000u);
    o[2] = __builtin_bit_cast(float, v.y << 16); o[3] = __builtin_bit_cast(float, v.y & 0xffff0000u);
  }
}

template <int IN, int OUT, bool INVERSE>
__global__ __launch_bounds__(256) void rope_rows_kernel(RopeArgs a) {
#pragma clang fp contract(off)     // products and sums stay separate IEEE operations
  const int half = a.emb >> 1;
  const int main_chunks = a.main_src ? a.d_main >> 3 : 0;
  const int quads = a.emb >> 3;                       // groups of four pairs
  const int per_head = main_chunks + quads;
  const int items = a.heads * per_head;
  for (long tok = blockIdx.x; tok < a.tokens; tok += gridDim.x) {
    const long pos = a.emb == 0 ? 0 : (a.positions ? a.positions[tok] : tok / a.batch);
    for (int it = threadIdx.x; it < items; it += 256) {
      const int head = it / per_head, c = it - head * per_head;
      if (c < main_chunks) {
        const uint4 v = *(const uint4*)(a.main_src + tok * a.ms_tok + head * a.ms_head + 8 * c);
        *(uint4*)(a.main_dst + tok * a.md_tok + head * a.md_head + 8 * c) = v;
        continue;
      }
      const int q = c - main_chunks;
      const unsigned short* src = a.pe_src + tok * a.ps_tok + head * a.ps_head;
      unsigned short* dst = a.pe_dst + tok * a.pd_tok + head * a.pd_head;
      float x1[4], x2[4];
      if (IN == ADJ) {
        const uint4 v = *(const uint4*)(src + 8 * q);
        const unsigned w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
          x1[k] = __builtin_bit_cast(float, w[k] << 16);
          x2[k] = __builtin_bit_cast(float, w[k] & 0xffff0000u);
        }
      } else {
        load4(src, 4 * q, 0, x1);
        load4(src, half + 4 * q, 0, x2);
      }
      constexpr int CS = INVERSE ? IN : OUT;           // pairing of the rotated side
      float c1[4], c2[4], s1[4], s2[4];
      const long crow = pos * a.emb;
      if (CS == ADJ) {
        float ca[4], cb[4], sa[4], sb[4];
        load4(a.cos, crow + 8 * q, a.cs_f32, ca);
        load4(a.cos, crow + 8 * q + 4, a.cs_f32, cb);
        load4(a.sin, crow + 8 * q, a.cs_f32, sa);
        load4(a.sin, crow + 8 * q + 4, a.cs_f32, sb);
        c1[0] = ca[0]; c2[0] = ca[1]; c1[1] = ca[2]; c2[1] = ca[3]; c1[2] = cb[0]; c2[2] = cb[1]; c1[3] = cb[2]; c2[3] = cb[3];
        s1[0] = sa[0]; s2[0] = sa[1]; s1[1] = sa[2]; s2[1] = sa[3]; s1[2] = sb[0]; s2[2] = sb[1]; s1[3] = sb[2]; s2[3] = sb[3];
      } else {
        load4(a.cos, crow + 4 * q, a.cs_f32, c1);
        load4(a.cos, crow + half + 4 * q, a.cs_f32, c2);
        load4(a.sin, crow + 4 * q, a.cs_f32, s1);
        load4(a.sin, crow + half + 4 * q, a.cs_f32, s2);
      }
      float y1[4], y2[4];
#pragma unroll
      for (int k = 0; k < 4; k++) {
        if (!INVERSE) {
          y1[k] = x1[k] * c1[k] - x2[k] * s1[k];
          y2[k] = x2[k] * c2[k] + x1[k] * s2[k];
        } else {
          y1[k] = x1[k] * c1[k] + x2[k] * s2[k];
          y2[k] = (-x1[k]) * s1[k] + x2[k] * c2[k];
        }
      }
      if (OUT == ADJ) {
        uint4 o;
        o.x = pack_bf16x2(y1[0], y2[0]); o.y = pack_bf16x2(y1[1], y2[1]);
        o.z = pack_bf16x2(y1[2], y2[2]); o.w = pack_bf16x2(y1[3], y2[3]);
        *(uint4*)(dst + 8 * q) = o;
      } else {
        *(uint2*)(dst + 4 * q) = make_uint2(pack_bf16x2(y1[0], y1[1]), pack_bf16x2(y1[2], y1[3]));
        *(uint2*)(dst + half + 4 * q) = make_uint2(pack_bf16x2(y2[0], y2[1]), pack_bf16x2(y2[2], y2[3]));
      }
    }
  }
}

// Gradient of a pe row that the forward broadcast to every head: the head-sum of the incoming
// gradient (fp32, heads added in ascending order within 256 / emb_dim interleaved groups, the groups
// then in order), rounded to bf16, then the inverse rotation; written with adjacent pairing.
template <int IN>
__global__ __launch_bounds__(256) void rope_headsum_inverse_kernel(
    const unsigned short* __restrict__ g, long g_tok, long g_head, unsigned short* __restrict__ d_emb, long de_tok,
    int emb, const void* cos, const void* sin, int cs_f32, const int* __restrict__ positions, int batch,
    int tokens, int heads) {
#pragma clang fp contract(off)
  __shared__ float part[256];
  __shared__ float tot[256];
  const int half = emb >> 1;
  const int groups = 256 / emb;
  const int e = threadIdx.x % emb, grp = threadIdx.x / emb;
  for (long tok = blockIdx.x; tok < tokens; tok += gridDim.x) {
    const long pos = positions ? positions[tok] : tok / batch;
    float s = 0.f;
    if (grp < groups)
      for (int h = grp; h < heads; h += groups) s += bf16_bits_to_f32(g[tok * g_tok + h * g_head + e]);
    part[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x < emb) {
      float t = 0.f;
      for (int k = 0; k < groups; k++) t += part[k * emb + e];
      tot[e] = bf16_bits_to_f32(f32_to_bf16_bits(t));
    }
    __syncthreads();
    if (threadIdx.x < half) {
      const int i = threadIdx.x;
      const int i1 = IN == ADJ ? 2 * i : i, i2 = IN == ADJ ? 2 * i + 1 : i + half;
      const float x1 = tot[i1], x2 = tot[i2];
      float c1, c2, s1, s2;
      const long crow = pos * emb;
      if (cs_f32) {
        c1 = ((const float*)cos)[crow + i1]; c2 = ((const float*)cos)[crow + i2];
        s1 = ((const float*)sin)[crow + i1]; s2 = ((const float*)sin)[crow + i2];
      } else {
        c1 = bf16_bits_to_f32(((const unsigned short*)cos)[crow + i1]); c2 = bf16_bits_to_f32(((const unsigned short*)cos)[crow + i2]);
        s1 = bf16_bits_to_f32(((const unsigned short*)sin)[crow + i1]); s2 = bf16_bits_to_f32(((const unsigned short*)sin)[crow + i2]);
      }
      const float y1 = x1 * c1 + x2 * s2;
      const float y2 = (-x1) * s1 + x2 * c2;
      *(unsigned*)(d_emb + tok * de_tok + 2 * i) = pack_bf16x2(y1, y2);
    }
    __syncthreads();
  }
}

bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }
bool aligned8(const void* p) { return ((uintptr_t)p % 8) == 0; }

}  // namespace

extern "C" int dsa_rope_rows(const void* main_src, int64_t ms_tok, int64_t ms_head, void* main_dst, int64_t md_tok,
                             int64_t md_head, int d_main, const void* pe_src, int64_t ps_tok, int64_t ps_head,
                             void* pe_dst, int64_t pd_tok, int64_t pd_head, int emb_dim, const void* cos,
                             const void* sin, int cos_sin_f32, const int32_t* positions, int batch, int tokens,
                             int heads, int in_pairing, int out_pairing, int inverse, void* stream) {
  DSA_REQUIRE(tokens >= 0 && heads > 0, "dsa_rope_rows: bad sizes tokens=%d heads=%d", tokens, heads);
  DSA_REQUIRE(emb_dim >= 0 && emb_dim % 8 == 0, "dsa_rope_rows: emb_dim must be a multiple of 8, got %d", emb_dim);
  DSA_REQUIRE(emb_dim > 0 || main_src != nullptr, "dsa_rope_rows: nothing to do (no main part and emb_dim = 0)");
  DSA_REQUIRE((in_pairing == 0 || in_pairing == 1) && (out_pairing == 0 || out_pairing == 1),
              "dsa_rope_rows: pairing must be 0 (adjacent) or 1 (split)");
  DSA_REQUIRE(emb_dim == 0 || (pe_src && pe_dst && cos && sin), "dsa_rope_rows: null pointer");
  DSA_REQUIRE(emb_dim == 0 || positions != nullptr || batch > 0, "dsa_rope_rows: batch must be positive when no positions are given");
  DSA_REQUIRE(emb_dim == 0 || aligned16(pe_src) && aligned16(pe_dst) && aligned16(cos) && aligned16(sin) && ps_tok % 8 == 0 &&
              ps_head % 8 == 0 && pd_tok % 8 == 0 && pd_head % 8 == 0,
              "dsa_rope_rows: pe rows must start on 16-byte boundaries");
  if (main_src) {
    DSA_REQUIRE(main_dst != nullptr && d_main > 0 && d_main % 8 == 0, "dsa_rope_rows: d_main must be a positive multiple of 8, got %d", d_main);
    DSA_REQUIRE(aligned16(main_src) && aligned16(main_dst) && ms_tok % 8 == 0 && ms_head % 8 == 0 && md_tok % 8 == 0 &&
                md_head % 8 == 0, "dsa_rope_rows: main rows must start on 16-byte boundaries");
  }
  if (tokens == 0) return DSA_OK;
  RopeArgs a;
  a.main_src = (const unsigned short*)main_src; a.ms_tok = ms_tok; a.ms_head = ms_head;
  a.main_dst = (unsigned short*)main_dst; a.md_tok = md_tok; a.md_head = md_head; a.d_main = d_main;
  a.pe_src = (const unsigned short*)pe_src; a.ps_tok = ps_tok; a.ps_head = ps_head;
  a.pe_dst = (unsigned short*)pe_dst; a.pd_tok = pd_tok; a.pd_head = pd_head; a.emb = emb_dim;
  a.cos = cos; a.sin = sin; a.cs_f32 = cos_sin_f32; a.positions = positions; a.batch = batch;
  a.tokens = tokens; a.heads = heads;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(tokens < (1 << 20) ? tokens : (1 << 20)), block(256);
  const int sel = (in_pairing << 2) | (out_pairing << 1) | (inverse ? 1 : 0);
  switch (sel) {
    case 0: rope_rows_kernel<ADJ, ADJ, false><<<grid, block, 0, st>>>(a); break;
    case 1: rope_rows_kernel<ADJ, ADJ, true><<<grid, block, 0, st>>>(a); break;
    case 2: rope_rows_kernel<ADJ, SPLIT, false><<<grid, block, 0, st>>>(a); break;
    case 3: rope_rows_kernel<ADJ, SPLIT, true><<<grid, block, 0, st>>>(a); break;
    case 4: rope_rows_kernel<SPLIT, ADJ, false><<<grid, block, 0, st>>>(a); break;
    case 5: rope_rows_kernel<SPLIT, ADJ, true><<<grid, block, 0, st>>>(a); break;
    case 6: rope_rows_kernel<SPLIT, SPLIT, false><<<grid, block, 0, st>>>(a); break;
    default: rope_rows_kernel<SPLIT, SPLIT, true><<<grid, block, 0, st>>>(a); break;
  }
  DSA_CHECK_LAUNCH("dsa_rope_rows");
  return DSA_OK;
}

extern "C" int dsa_rope_headsum_inverse(const void* grad, int64_t g_tok, int64_t g_head, void* d_emb, int64_t de_tok,
                                        int emb_dim, const void* cos, const void* sin, int cos_sin_f32,
                                        const int32_t* positions, int batch, int tokens, int heads, int in_pairing,
                                        void* stream) {
  DSA_REQUIRE(tokens >= 0 && heads > 0, "dsa_rope_headsum_inverse: bad sizes tokens=%d heads=%d", tokens, heads);
  DSA_REQUIRE(emb_dim >= 2 && emb_dim <= 256 && (emb_dim & (emb_dim - 1)) == 0,
              "dsa_rope_headsum_inverse: emb_dim must be a power of two up to 256, got %d", emb_dim);
  DSA_REQUIRE(in_pairing == 0 || in_pairing == 1, "dsa_rope_headsum_inverse: pairing must be 0 (adjacent) or 1 (split)");
  DSA_REQUIRE(positions != nullptr || batch > 0, "dsa_rope_headsum_inverse: batch must be positive when no positions are given");
  DSA_REQUIRE(grad && d_emb && cos && sin, "dsa_rope_headsum_inverse: null pointer");
  DSA_REQUIRE(((uintptr_t)d_emb % 4) == 0 && de_tok % 2 == 0, "dsa_rope_headsum_inverse: d_emb rows must start on 4-byte boundaries");
  if (tokens == 0) return DSA_OK;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(tokens < (1 << 20) ? tokens : (1 << 20)), block(256);
  if (in_pairing == 0)
    rope_headsum_inverse_kernel<ADJ><<<grid, block, 0, st>>>((const unsigned short*)grad, g_tok, g_head, (unsigned short*)d_emb,
                                                            de_tok, emb_dim, cos, sin, cos_sin_f32, positions, batch, tokens, heads);
  else
    rope_headsum_inverse_kernel<SPLIT><<<grid, block, 0, st>>>((const unsigned short*)grad, g_tok, g_head, (unsigned short*)d_emb,
                                                              de_tok, emb_dim, cos, sin, cos_sin_f32, positions, batch, tokens, heads);
  DSA_CHECK_LAUNCH("dsa_rope_headsum_inverse");
  return DSA_OK;
}
