/*
 * C ABI of the MI355X (gfx950) fused DeepSeek-Sparse-Attention kernels.
 *
 * One entry point per external kernel the reference's DSA path calls.  Every function takes raw
 * device pointers plus sizes and a HIP stream (passed as void*; NULL = the null stream), launches
 * asynchronously on that stream, allocates nothing, keeps no state between calls and returns an
 * int status: 0 on success, negative on error (see dsa_last_error()).  All tensors are dense and
 * row-major ("contiguous") unless a leading dimension is given.  Paths in the comments are
 * relative to the reference tree.
 */
#ifndef DSA_HIP_H
#define DSA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DSA_OK 0
#define DSA_ERR_BAD_ARG (-1)     /* shape / alignment / unsupported size */
#define DSA_ERR_LAUNCH (-2)      /* HIP reported a launch error */
#define DSA_ERR_WORKSPACE (-3)   /* caller-provided workspace too small */

/* ABI version; bumped whenever a signature changes. */
int dsa_version(void);
/* Human-readable description of the last error on the calling thread ("" if none). */
const char* dsa_last_error(void);

/*
 * Row-wise e4m3 quantiser: amax -> max(amax, eps) -> scale = 448/amax (floored to a power of two
 * when pow2 != 0) -> x8 = e4m3_rne(clamp(x * scale)), scale_inv = 1/scale.
 * Replaces TransformerEngine's Float8BlockQuantizer as configured at
 * loongforge/models/common/experimental_attention_variant/dsa_fused_kernels.py:2308-2315 and
 * used at :2341-2346 (1x128 blocks => one scale per row of `cols` = 128 elements).
 *   x        [rows, cols] bf16     x8 [rows, cols] fp8-e4m3 (OCP)     scale_inv [rows] f32
 */
int dsa_quant_rowwise_e4m3(const void* x, int64_t rows, int cols, void* x8, float* scale_inv,
                           float eps, int pow2, void* stream);

/*
 * Hadamard rotation fused with the quantiser above: y = bf16(H_128 . x * 128^-0.5) (Sylvester
 * order), then (x8, scale_inv) = quantise(y).  Replaces the pair rotate_activation ->
 * Float8BlockQuantizer of the indexer front end: rotate_activation at
 * loongforge/models/common/experimental_attention_variant/dsa_fused.py:74-90 (applied at :604-606)
 * followed by the quantiser at dsa_fused_kernels.py:2341-2346, without the bf16 round trip
 * through memory.  Either output may be NULL: x8 == NULL gives the rotation only (y), y == NULL the
 * quantised payload only.
 *   x, y [rows, 128] bf16     x8 [rows, 128] fp8-e4m3 (OCP)     scale_inv [rows] f32
 */
int dsa_rotate_quant_e4m3(const void* x, int64_t rows, int cols, void* x8, float* scale_inv, void* y,
                          float eps, int pow2, void* stream);

/*
 * The quantiser above (after the rotation when rotate != 0) that also writes, per row,
 *   weight_scaled[row] = (weights[row] * scale_inv[row]) * factor
 * i.e. the indexer's `weight_scaled = weights * q_scale * softmax_scale`
 * (dsa_fused_kernels.py:2362, deepseek_v4_csa.py:1386) with rows = (token, head) and
 * factor = head_dim^-0.5, in the same kernel that produces q_scale instead of two elementwise
 * launches after it.  The products are rounded one after the other, as the separate operations are.
 *   weights, weight_scaled [rows] f32
 */
int dsa_quant_rowwise_e4m3_weights(const void* x, int64_t rows, int cols, void* x8, float* scale_inv,
                                   float eps, int pow2, int rotate, const float* weights, float factor,
                                   float* weight_scaled, void* stream);

/*
 * The indexer front end behind its projections in one pass per 128-element row:
 *   [LayerNorm ->] [RoPE on the leading 64 elements ->] [Hadamard rotation ->] quantiser [-> weight scaling]
 * Replaces, on the key side, k_norm -> _apply_rope -> rotate_activation at
 * loongforge/models/common/experimental_attention_variant/dsa_fused.py:583-606 followed by the quantiser
 * at dsa_fused_kernels.py:2341-2346, and on the query side _apply_rope -> rotate_activation -> quantiser
 * -> weight_scaled (dsa_fused.py:568-578, :604-606; dsa_fused_kernels.py:2341-2346, :2362).  Every stage
 * rounds to bf16 where the separate operations do.  The rotary part uses the formula, rounding and cos /
 * sin indexing of dsa_rope_rows with equal source and destination pairing (0 adjacent pairs, 1 split pairs
 * (i, i + 32), -1 none): fused_apply_mla_rope(..., pe_first=True), dsa_fused.py:435-451.
 *   x [rows, 128] bf16, rows = tokens * rows_per_token; position of a row's token: positions[token], or
 *   token / batch when positions is NULL; cos, sin [max position + 1, 64] bf16 or f32 (cos_sin_f32): the tables must
 *   reach the largest position given - the entry point does not know their length and checks nothing there;
 *   ln_weight, ln_bias [128] f32 or both NULL (no LayerNorm); rotate != 0 applies the Hadamard rotation.
 *   Outputs as dsa_rotate_quant_e4m3 (x8 / scale_inv and / or y) and dsa_quant_rowwise_e4m3_weights
 *   (weights, weight_scaled [rows] f32, or both NULL).
 */
int dsa_indexer_front_e4m3(const void* x, int64_t rows, int cols, int rows_per_token, const float* ln_weight,
                           const float* ln_bias, float ln_eps, const void* cos, const void* sin,
                           int cos_sin_f32, int pairing, const int32_t* positions, int batch, int rotate,
                           void* x8, float* scale_inv, void* y, float eps, int pow2, const float* weights,
                           float factor, float* weight_scaled, void* stream);

/*
 * Lightning-indexer logits:
 *   logits[i, j - base_i] = k_scale[j] * sum_h q_w[i,h] * relu(q8[i,h,:] . k8[j,:]),  ks[i] <= j < ke[i]
 * and -inf for every other column of row i.  base_i = 0 when `relative` == 0 (dense layout, width
 * Sk) and ks[i] when `relative` != 0 (packed layout of the reference, width = max_seqlen_k).
 * Replaces deep_gemm.fp8_mqa_logits as called at dsa_fused_kernels.py:2366 and :2370-2380.
 *   q8 [S, Hi, 128] e4m3   q_w [S, Hi] f32 (= weights * q_scale * 128^-0.5)   k8 [Sk, 128] e4m3
 *   k_scale [Sk] f32   ks, ke [S] i32   logits [S, ld] f32 (ld >= width)
 */
int dsa_indexer_logits(const void* q8, const float* q_w, const void* k8, const float* k_scale,
                       const int32_t* ks, const int32_t* ke, int S, int Hi, int Sk,
                       float* logits, int64_t ld, int width, int relative, void* stream);

/*
 * Per-row top-k by value.  Row i considers columns [row_begin[i], row_end[i]) of logits, clipped to
 * [0, width) (NULL: 0 / width for every row); -inf entries are never selected.  Outputs K slots per
 * row: the selected scores (descending when `sorted` != 0, otherwise in ascending column order) and
 * column ids + id_base[i] (id_base == NULL: 0); unused slots hold score -inf and id -1.  Ties at the
 * K-th value are broken towards the lower column, so the result is deterministic.
 * Replaces flashinfer.top_k behind padded_flashinfer_topk, dsa_fused_kernels.py:1958-1998, and the
 * id globalisation at :2386-2387.
 *   logits [S, ld] f32   scores [S, K] f32   ids [S, K] i32
 */
int dsa_topk(const float* logits, int S, int64_t ld, const int32_t* row_begin, const int32_t* row_end,
             int width, const int32_t* id_base, int K, int sorted, float* scores, int32_t* ids,
             void* stream);

/*
 * Fused indexer forward = dsa_indexer_logits + dsa_topk without a caller-visible [S, Sk] matrix:
 * `workspace` (>= dsa_indexer_topk_workspace_bytes) holds the logits of one query block at a time.
 * Replaces DSAIndexerKernelFunction.forward after quantisation, dsa_fused_kernels.py:2348-2387.
 * ids are global key rows; rows with fewer than K visible keys are padded with id -1 / score -inf.
 */
size_t dsa_indexer_topk_workspace_bytes(int S, int Sk, int K);
int dsa_indexer_topk_fwd(const void* q8, const float* q_w, const void* k8, const float* k_scale,
                         const int32_t* ks, const int32_t* ke, int S, int Hi, int Sk, int K,
                         int sorted, float* scores, int32_t* ids, void* workspace,
                         size_t workspace_bytes, void* stream);

/*
 * dsa_indexer_topk_fwd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): same inputs, outputs and results, no
 * workspace argument.  The logits blocks live in a 64 MiB device array inside the library, which every
 * GPU the library runs on holds until the process ends; at most 65536 keys (a block of 256 queries
 * must fit), more is refused with DSA_ERR_BAD_ARG.  The call allocates nothing; calls that overlap on
 * one GPU share the array and race, so order them on one stream.  The first call on a device looks
 * up the array's address there (not a stream operation: make it outside a graph capture).
 * No counterpart in the reference, whose wrapper lets torch allocate the logits
 * (dsa_fused_kernels.py:2366-2380).
 */
int dsa_indexer_topk_fwd_static(const void* q8, const float* q_w, const void* k8, const float* k_scale,
                                const int32_t* ks, const int32_t* ke, int S, int Hi, int Sk, int K,
                                int sorted, float* scores, int32_t* ids, void* stream);

/*
 * Sparse gradients of the selected logits w.r.t. the fp8 payloads and the scaled weights
 * (scales are constants):  with j = ids[i,t] >= 0, r_h = q8[i,h,:] . k8[j,:],
 *   d_qw[i,h]   = sum_t g[i,t] k_scale[j] relu(r_h)
 *   d_q8[i,h,:] = sum_t g[i,t] k_scale[j] q_w[i,h] [r_h > 0] k8[j,:]
 *   d_k8[j,:]   = sum_{(i,t): ids[i,t]=j} g[i,t] k_scale[j] sum_h q_w[i,h] [r_h > 0] q8[i,h,:]
 * d_k8 is accumulated in a fixed order (bit-reproducible); the ids of one query must be distinct
 * (a row with a repeated id makes the call return d_k8 filled with NaN).  Replaces
 * lightning_indexer_bwd.fp8_mqa_logits_bwd as called at dsa_fused_kernels.py:2421-2430.
 *   g [S, K] f32   d_q8 [S, Hi, 128] f32   d_k8 [Sk, 128] f32   d_qw [S, Hi] f32
 */
size_t dsa_indexer_bwd_workspace_bytes(int S, int Hi, int Sk, int K);
int dsa_indexer_bwd(const float* g, const void* q8, const void* k8, const float* k_scale,
                    const float* q_w, const int32_t* ids, int S, int Hi, int Sk, int K,
                    float* d_q8, float* d_k8, float* d_qw, void* workspace, size_t workspace_bytes,
                    void* stream);

/*
 * Sparse MQA-MLA attention forward.  Slot t of query i (global position q_start + i) is valid iff
 * ids[i,t] != -1, 0 <= ids[i,t] < Skv and ids[i,t] <= q_start + i.  Over the valid slots:
 *   s = q[i,h,:] . kv[ids[i,t],:]   P = softmax_t(s * sm_scale)   out[i,h,:] = sum_t P kv[ids[i,t], :d_v]
 *   lse[i,h] = natural-log sum-exp of s * sm_scale  (+inf, with out = 0, when no slot is valid)
 *   p_out[i,h,t] = s (raw logit) on valid slots, -inf elsewhere; optional (NULL to skip);
 *                  p_out_f32 selects f32 (1) or bf16 (0) storage.
 * Replaces flash_mla_fwd.flash_mla_sparse_fwd as called at dsa_fused_kernels.py:2048-2059
 * (math: ops/tilelang_ops/sparse_mla_fwd.py:129-180).
 *   q [S, H, 576] bf16   kv [Skv, 576] bf16   ids [S, K] i32 (K % 64 == 0)
 *   out [S, H, 512] bf16   lse [S, H] f32   p_out [S, H, K]
 */
int dsa_sparse_mla_fwd(const void* q, const void* kv, const int32_t* ids, int S, int H, int Skv,
                       int K, int q_start, float sm_scale, int d_v, void* out, float* lse,
                       void* p_out, int p_out_f32, void* stream);

/*
 * The same with a per-head attention-sink logit (attn_sink [H] f32, NULL = none): the softmax
 * denominator gains the term exp(attn_sink[h]), which has no value row, so
 *   P = exp(s * sm_scale) / (sum_t exp(s * sm_scale) + exp(attn_sink[h]))   and lse includes the sink;
 * a query without valid slots gets lse = attn_sink[h] and a zero output row.  This is the
 * `attn_sink` argument of flash_mla_sparse_fwd at dsa_fused_kernels.py:2040-2057; its math is the
 * torch formulation at loongforge/models/foundation/deepseek_v4/deepseek_v4_csa.py:571-579.
 * dsa_sparse_mla_bwd needs no sink argument: the sink enters dQ / dKV only through lse.
 * p_out_skip (a multiple of 32, < K; 0 = none): p_out leaves out the first p_out_skip slots of every
 * query and is [S,H,K - p_out_skip]; attention itself still runs over all K slots.  This is the
 * `window_size` argument of the same call (:2058): the DeepSeek-V4 caller puts its sliding-window
 * keys in the leading slots and documents the resulting p_out width at deepseek_v4_csa.py:2341-2346.
 */
int dsa_sparse_mla_fwd_ex(const void* q, const void* kv, const int32_t* ids, int S, int H, int Skv,
                          int K, int q_start, float sm_scale, int d_v, void* out, float* lse,
                          void* p_out, int p_out_f32, const float* attn_sink, int p_out_skip, void* stream);

/*
 * Sparse MQA-MLA attention backward: dQ and dKV of dsa_sparse_mla_fwd given dO, the saved out and
 * natural-log lse.  P and dS enter the matrix products as bf16 (as in the reference's kernel); the
 * contribution of one (query, key) pair to dKV - a row of 576 values, summed over all heads in
 * fp32 - is rounded to bf16 once, and the rows of a key are then summed in fp32 in a fixed order
 * (bit-reproducible, no float atomics); dKV is returned as bf16.  The ids of one query must be
 * distinct (any top-k is): a row with a repeated valid id makes the call return dq and dkv filled
 * with NaN rather than sums that miss a term.  Replaces flash_mla_bwd.flash_mla_sparse_bwd /
 * sparse_mla_bwd_interface as called at dsa_fused_kernels.py:2086-2110
 * (math: loongforge/models/common/experimental_attention_variant/sparse_mla_bwd.py:292-356).
 *   dout [S, H, 512] bf16   dq [S, H, 576] bf16   dkv [Skv, 576] bf16
 * Workspace: dsa_sparse_mla_bwd_workspace_bytes is the largest size the call can use - all queries in one
 * sweep (26 GiB at S = Skv = 8192, K = 2048; 105 GiB at 32768 tokens).  Any size from
 * dsa_sparse_mla_bwd_workspace_bytes_min on is accepted: with less than the full size the queries are walked in
 * chunks (the largest of S, S/2, S/4, ... that fits, at least 64), a few per cent slower per extra chunk; the
 * chunking follows from the sizes alone, and dKV is bit-reproducible for a given workspace size.
 */
size_t dsa_sparse_mla_bwd_workspace_bytes(int S, int H, int Skv, int K);
size_t dsa_sparse_mla_bwd_workspace_bytes_min(int S, int H, int Skv, int K);
int dsa_sparse_mla_bwd(const void* q, const void* kv, const void* out, const void* dout,
                       const int32_t* ids, const float* lse, int S, int H, int Skv, int K,
                       int q_start, float sm_scale, int d_v, void* dq, void* dkv,
                       void* workspace, size_t workspace_bytes, void* stream);

/*
 * KL loss of the indexer's scores against the attention distribution, and its gradient, per query row:
 *   pred = softmax_t(scores[i,:])    u = target[i,:] + eps
 *   row_loss[i] = sum_t u_t (log u_t - log(pred_t + eps))      grad[i,t] = d row_loss[i] / d scores[i,t]
 * sum_i row_loss[i] is F.kl_div((pred + eps).log(), target + eps, reduction="sum") of
 * dsa_fused.py:931-944 (eps = 1e-10 there); padded slots (score -inf, target 0) add nothing and get
 * gradient 0.  `ld_s` / `ld_t` are the row strides of scores / target in elements.
 *   scores [S, K] f32   target [S, K] f32   row_loss [S] f32   grad [S, K] f32
 */
int dsa_indexer_kl_loss(const float* scores, int64_t ld_s, const float* target, int64_t ld_t, int S,
                        int K, float eps, float* row_loss, float* grad, void* stream);

/*
 * Head-averaged attention distribution over the selected slots:
 *   target[i,t] = (1/H) sum_h softmax_t(p_out[i,h,:] * sm_scale)[t]
 * Replaces triton_attn_dist, dsa_fused_kernels.py:1844-1955.  `ld_s` / `ld_h` are the element
 * strides of p_out between queries / heads (so a head-sliced view can be passed).
 *   p_out [S, H, K] bf16 or f32   target [S, K] f32
 */
int dsa_attn_dist(const void* p_out, int p_out_f32, int S, int H, int K, int64_t ld_s,
                  int64_t ld_h, float sm_scale, float* target, void* stream);

/*
 * The same distribution without materialised logits: recomputed from q, kv, ids and the forward's
 * natural-log lse,
 *   target[i,t] = (1/heads_in_mean) sum_{h < heads_in_mean} exp(q[i,h,:] . kv[ids[i,t],:] * sm_scale - lse[i,h])
 * (0 for invalid slots; validity as in dsa_sparse_mla_fwd), which is mean_h softmax_t when lse[i,h]
 * is the log-sum-exp over the same slots.  Replaces the pair `return_p_out=True` +
 * triton_attn_dist of the training path (loongforge/models/common/experimental_attention_variant/
 * dsa_fused.py:903-929): the [S, H, K] logits (4.3 GB at seq 8192) are neither written nor read.
 * heads_in_mean < H leaves out padded heads, as the slice at dsa_fused.py:915-917 does.
 *   q [S, H, 576] bf16   kv [Skv, 576] bf16   ids [S, K] i32 (K % 64 == 0, K <= 4096)   lse [S, H] f32
 */
int dsa_attn_dist_qk(const void* q, const void* kv, const int32_t* ids, const float* lse, int S, int H,
                     int heads_in_mean, int Skv, int K, int q_start, float sm_scale, float* target,
                     void* stream);

/*
 * MLA weight absorption, one head's projection per (token, head) row, read and written in place inside
 * larger tensors:  c[s, h, n] = sum_k a[s, h, k] * w[h, n, k]   (bf16, fp32 accumulation).
 * Replaces the two per-head products around the sparse attention call at
 * loongforge/models/common/experimental_attention_variant/multi_latent_attention.py:1177-1194 / :1304-1316
 * (q_content = einsum("...hd,hdk->...hk", q_no_pe, k_up), or the TEGroupedLinear linear_kv_up_proj_absorb_q
 * with its permutes) and :955-974 (core_attn_out = einsum("...hk,hdk->...hd", core_attn_out, v_up), or
 * linear_kv_up_proj_absorb_output with movedim / transpose), together with the copies that surround them:
 * `a` may be the no-position columns of the [S, H, 192] query projection and `c` the latent columns of the
 * [S, H, 576] attention query (k_dim = 128, n_dim = 512, w = W_UK transposed to [H, 512, 128]); or `a` the
 * attention output [S, H, 512] and `c` the [S, H * 128] input of the output projection (k_dim = 512,
 * n_dim = 128, w = W_UV [H, 128, 512]).
 *   a_tok, a_head, c_tok, c_head: strides in elements between tokens / heads (multiples of 8);
 *   rows of a, c and w start on 16-byte boundaries.
 */
int dsa_mla_absorb(const void* a, int64_t a_tok, int64_t a_head, const void* w, void* c, int64_t c_tok,
                   int64_t c_head, int S, int H, int k_dim, int n_dim, void* stream);

/*
 * Rotary position embedding of the MLA query / key rows, fused with the copies around it.  Per
 * (token, head) the call copies a "main" part of d_main bf16 elements between two strided tensors
 * (main_src NULL: no main part) and rotates a "pe" part of emb_dim bf16 elements, pair by pair:
 *     y1 = x1 * c1 - x2 * s1     y2 = x2 * c2 + x1 * s2          (inverse = 0)
 *     y1 = x1 * c1 + x2 * s2     y2 = x2 * c2 - x1 * s1          (inverse = 1: the transpose, for gradients)
 * in fp32 without fused multiply-adds, rounded once to bf16.  A pairing says where pair i sits in
 * a row: 0 = adjacent (elements 2i, 2i+1), 1 = split (elements i, i + emb_dim/2); in_pairing and
 * out_pairing are independent, and cos / sin ([positions, emb_dim], fp32 or bf16) are indexed
 * with the pairing of the rotated side (out_pairing when inverse = 0, in_pairing when inverse = 1).
 * Strides are in elements; a pe head stride of 0 broadcasts one row to every head; pe_src may
 * equal pe_dst when the pairings are equal (in place).  The position of token t is positions[t],
 * or t / batch when positions is NULL.  Rows must start on 16-byte boundaries, d_main and emb_dim
 * are multiples of 8.
 *
 * This one entry point replaces the reference's Triton kernels
 *   rotary_{fwd,bwd}_q_kernel_interleaved            dsa_fused_kernels.py:68-228    (in = out = 0, no main part, in place)
 *   rotary_{fwd,bwd}_q_kernel_non_interleaved        dsa_fused_kernels.py:366-499   (in = out = 1, no main part, in place)
 *   fused_rope_permute_cat_{fwd,bwd}_kernel_*        dsa_fused_kernels.py:619-1008  (main: [h,S,d] <-> [S,h,d]; in 0 -> out 1 or 0)
 *   rotary_fwd_absorb_kv_kernel_*                    dsa_fused_kernels.py:1228-1502 (pe head stride 0; in 0 -> out 1 or 0)
 * and, with emb_dim = 0 (main part only), the k_dim copy of rotary_bwd_absorb_kv_kernel_* (:1327-1371,
 * :1517-1562); dsa_rope_headsum_inverse is the rest of that kernel.
 */
int dsa_rope_rows(const void* main_src, int64_t ms_tok, int64_t ms_head, void* main_dst, int64_t md_tok,
                  int64_t md_head, int d_main, const void* pe_src, int64_t ps_tok, int64_t ps_head,
                  void* pe_dst, int64_t pd_tok, int64_t pd_head, int emb_dim, const void* cos,
                  const void* sin, int cos_sin_f32, const int32_t* positions, int batch, int tokens,
                  int heads, int in_pairing, int out_pairing, int inverse, void* stream);

/*
 * Gradient of a pe row that the forward broadcast to every head (the key's rotary part):
 *   d_emb[t, :] = inverse rotation of bf16( sum_h grad[t, h, :] )   written with adjacent pairing,
 * the head-sum in fp32 in a fixed order.  grad points at the pe part of the incoming gradient
 * (element strides g_tok, g_head), in_pairing is the pairing the forward wrote it with.
 * Replaces the `pid_head == 0` branch of rotary_bwd_absorb_kv_kernel_{non_interleaved,interleaved},
 * dsa_fused_kernels.py:1372-1410 and :1563-1608.
 */
int dsa_rope_headsum_inverse(const void* grad, int64_t g_tok, int64_t g_head, void* d_emb, int64_t de_tok,
                             int emb_dim, const void* cos, const void* sin, int cos_sin_f32,
                             const int32_t* positions, int batch, int tokens, int heads, int in_pairing,
                             void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DSA_HIP_H */
