/*
 * libssdhip -- C ABI of the MI355X (gfx950) draft->verify hot path.
 *
 * The reference (tanishqkumar/ssd) has no FFI of its own: its hot ops are Python call sites into
 * third-party CUDA wheels (torch/cuBLAS, Inductor, Triton, sgl-kernel FA3, flashinfer).  Each entry point
 * below replaces one such call site; the citation names the reference file:line it stands in for.
 * INTEGRATION.md shows the ctypes stub a maintainer would add at that call site.
 *
 * Conventions
 *   - every function returns 0 (SSD_OK) or a negative error code; nothing throws, allocates, or
 *     synchronises; all work is enqueued on `stream` (a hipStream_t passed as void*), so every call is
 *     hipGraph-capturable.
 *   - all pointers are DEVICE pointers owned by the caller; bf16 tensors are raw 16-bit words.
 *   - "rows"  = row-major [M][K] bf16.
 *     "frag"  = fragment-major [ceil(M/16)][K/32][64 lanes][8] bf16: 16x32 tiles of 1 KiB stored in
 *               MFMA-16x16x32 lane order, lane = (row & 15) + 16 * ((col & 31) >> 3).  Weights are
 *               pre-shuffled into this layout once at load (ssd_rows_to_frag); activations are
 *               produced in it directly by the kernel that feeds a GEMM.
 *   - token ids / positions are int64, every other index is int32 (as the reference,
 *     ssd/engine/helpers/runner_helpers.py:99-106).
 *   - KV cache layout per layer and per K/V: [num_blocks][n_kv_heads][block_size][head_dim] bf16;
 *     slot = block_id * block_size + pos_in_block, slot -1 = do not store (reference semantics,
 *     ssd/layers/attention.py:23-25).
 */
#ifndef SSD_HIP_H
#define SSD_HIP_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* Bumped whenever a signature or a semantic of this header changes; ssd_abi_version() returns the value the library was built
 * with, so a consumer compiled against another header can tell (tests/abi_consumer.c does). */
#define SSD_HIP_ABI_VERSION 6

#define SSD_OK 0
#define SSD_ERR_SHAPE (-1)
#define SSD_ERR_LAUNCH (-2)
#define SSD_ERR_ARG (-3)

/* GEMM epilogues */
#define SSD_EPI_ROWS 0      /* y rows bf16 [M][ldy]                                             */
#define SSD_EPI_SILU_FRAG 1 /* W row groups alternate gate/up; y = frag bf16 [M][N/2] = silu(g)*u */
#define SSD_EPI_ROWS_F32 2  /* y rows fp32 [M][ldy] (diagnostics: logits before the bf16 rounding) */

int ssd_abi_version(void);

/* Layout conversion.  mode 0: identity; mode 1: source rows are [gate ; up] halves and destination
 * 16-row groups alternate gate/up (MergedColumnParallelLinear, ssd/layers/linear.py:101-122). */
int ssd_rows_to_frag(const void* src_rows, void* dst_frag, int R, int K, int mode, void* stream);
int ssd_frag_to_rows(const void* src_frag, void* dst_rows, int R, int K, void* stream);
/* QKV weights [q heads | k heads | v heads] (QKVParallelLinear, ssd/layers/linear.py:125-162) -> fragment-major with the
 * "rotation-paired" row order: in every q/k head, 16-row group j = dims [8j..8j+7] ++ [hd/2+8j..hd/2+8j+7], so both members of
 * a neox RoPE pair share an MFMA accumulator tile.  GEMMs on such weights emit q/k in that order (qkv_perm = 1 below). */
int ssd_rows_to_frag_qkv(const void* src_rows, void* dst_frag, int nh, int nkv, int hd, int K, void* stream);

/* VocabParallelEmbedding.forward -- ssd/layers/embed_head.py:49-57 (rows outside
 * [vocab_start, vocab_start+vocab_count) produce zeros, the TP-masked form). */
int ssd_embedding(const int64_t* ids, const void* table_rows, void* out_rows, int T, int H, long vocab_start,
                  long vocab_count, void* stream);

/* RMSDNorm.norm_forward / add_norm_forward -- ssd/layers/layernorm.py:64-88 (as compiled: fp32 math,
 * res_out = bf16(x+res), y = bf16((x+res) * rsqrt(mean^2 + eps) * w)).  res_in/res_out/out_rows/out_frag
 * may be NULL; gather_rows (int32[T], optional) selects input rows (prefill last-token logits,
 * ssd/layers/embed_head.py:81-84). */
int ssd_rmsnorm(const void* x_rows, const void* res_in, void* res_out, const void* weight, float eps,
                void* out_rows, void* out_frag, const int32_t* gather_rows, int T, int H, void* stream);

/* ssd_rmsnorm whose x is the bf16 rounding of the sum of `splits` fp32 partial slabs [splits][slab_rows][H] written by
 * ssd_gemm_parts (the row-parallel GEMM that precedes every add_norm_forward, ssd/models/llama3.py:185-199). */
int ssd_rmsnorm_parts(const void* parts, int splits, int slab_rows, const void* res_in, void* res_out, const void* weight,
                      float eps, void* out_rows, void* out_frag, int T, int H, void* stream);

/* RMSHeadNorm.forward -- ssd/layers/layernorm.py:16-40 (Qwen3's q_norm / k_norm, ssd/models/qwen3.py:96-104) as a call of its own:
 * x_rows [T][heads][hd] normalised over hd per (token, head), weight bf16[hd].  The hot path runs it inside ssd_rope_store_kv
 * (q_norm_w / k_norm_w); this entry point is bit-identical to that fused form and exists for a binding at the module boundary. */
int ssd_head_rmsnorm(const void* x_rows, const void* weight, float eps, void* out_rows, int T, int heads, int hd, void* stream);

/* SiluAndMul.forward -- ssd/layers/activation.py:11-14 as a call of its own: x_rows [T][2 I] = [gate | up] ->
 * bf16(silu(gate) * up) as rows [T][I] and / or fragment-major (either may be NULL).  The hot path runs it as the gate_up GEMM's
 * epilogue (SSD_EPI_SILU_FRAG), same arithmetic. */
int ssd_silu_mul(const void* x_rows, void* out_rows, void* out_frag, int T, int I, void* stream);

/* The EAGLE-3 draft layer's QKV input, torch.cat([input_layernorm(token_embeddings), conditioning_feature_ln(features)], -1)
 * -- ssd/models/eagle3_draft_llama3.py:148-150 -- written directly as ONE fragment-major [T][2H] activation (each half is
 * RMSDNorm.norm_forward as in ssd_rmsnorm). */
int ssd_rmsnorm_pair(const void* x0_rows, const void* weight0, const void* x1_rows, const void* weight1, float eps,
                     void* out_frag, int T, int H, void* stream);

/* F.linear(x, W, b) -- ssd/layers/linear.py:65,98,196; ssd/layers/embed_head.py:88,95,111.
 * x_frag [M][K] frag, w_frag [N][K] frag, bias bf16[N] or NULL.  M <= 128 per call.
 * SSD_EPI_SILU_FRAG additionally fuses SiluAndMul.forward -- ssd/layers/activation.py:11-14. */
int ssd_gemm_wf(const void* x_frag, const void* w_frag, const void* bias, void* y, int M, int N, int K, int ldy,
                int epilogue, void* stream);
/* The same F.linear for matrices with too few 16-row groups to fill the chip (csrc/gemm_sk.hip; the 1B draft's o_proj /
 * down_proj): K is split across `splits` workgroups per row group, the last one to arrive reduces the fp32 partials in a
 * fixed order.  workspace >= (N/16)*splits KiB; counters >= N/16 uint32, zeroed once.  M <= 16, bf16 rows. */
int ssd_gemm_splitk(const void* x_frag, const void* w_frag, const void* bias, void* y, int M, int N, int K, int ldy,
                    int splits, int waves, void* workspace, void* counters, void* stream);

/* The same F.linear in its latency-optimal form for small matrices at M <= 16 (csrc/gemm_sk.hip gemm_sp_kernel): K is
 * split over `splits` workgroups per 16-row group, every wave keeps all its k-tiles in flight, and the partial sums are
 * NOT combined here: `parts` receives fp32 slabs [splits][M][N] which the consumer (ssd_gemm_fused_parts /
 * ssd_rmsnorm_parts) sums in slab order while forming x = bf16(sum) + residual -- the kernel boundary is the only
 * synchronisation.  parts == NULL: splits must be 1 and bf16 rows (+ bias) go to y.  ceil(K/32/splits/waves) <= 8. */
int ssd_gemm_parts(const void* x_frag, const void* w_frag, const void* bias, void* y, void* parts, int M, int N, int K,
                   int ldy, int splits, int waves, void* stream);

/* Prefill-chunk GEMM, 16 < M <= 128 (csrc/gemm_pf.hip): the reference's eager prefill F.linear calls
 * (ssd/engine/model_runner.py:602 -> ssd/layers/linear.py:65,98,196).  Same operands and epilogues (SSD_EPI_ROWS,
 * SSD_EPI_SILU_FRAG) as ssd_gemm_wf; the x tile of a k-step is shared by a workgroup through LDS and K is split
 * across workgroups into fp32 partials in `workspace` (>= ssd_gemm_pf_workspace_bytes), summed in a fixed order.
 * N % 128 == 0, K % 128 == 0; splits <= 0 picks the default.  epilogue 2 (partials only, y may be NULL, no bias): the fp32
 * partials [splits][M][N] in `workspace` ARE the output (splits = ssd_gemm_pf_workspace_bytes(M, N, K) / (4 M N)), to be
 * summed by ssd_rmsnorm_parts -- the add + RMSNorm that follows o_proj / down_proj -- instead of an epilogue launch. */
int ssd_gemm_pf_workspace_bytes(int M, int N, int K, int64_t* bytes);
int ssd_gemm_pf(const void* x_frag, const void* w_frag, const void* bias, void* y, int M, int N, int K, int ldy,
                int epilogue, void* workspace, int64_t workspace_bytes, int splits, void* stream);
/* Fused decode-layer GEMM for M <= 16 (csrc/gemm_fused.hip): [residual add + RMSNorm] -> F.linear ->
 * [RoPE + paged KV store | SiLU*mul | rows] in ONE launch; replaces add_norm_forward (layernorm.py:76-88) + F.linear
 * (linear.py:97-98) + RotaryEmbedding.forward (rotary_embedding.py:40-60) + store_kvcache (attention.py:10-41), or
 * + SiluAndMul (activation.py:11-14).  x comes either fragment-major (x_frag) or as row-major h (+ res_in) normalised on
 * the fly with norm_w / eps; then res_out (!= res_in) receives bf16(h + res_in).  epilogue: 0 rows, 1 SiLU*mul -> frag,
 * 3 RoPE + KV store (weights from ssd_rows_to_frag_qkv; q_out rows [M][nh*hd], K/V into the paged cache at `slots`).
 * nt / waves <= 0 pick the default decomposition. */
int ssd_gemm_fused(const void* x_frag, const void* h_rows, const void* res_in, void* res_out, const void* norm_w, float eps,
                   const void* w_frag, const void* bias, int M, int N, int K, int epilogue, void* y, int ldy,
                   const int64_t* positions, const float* cos_sin, const int32_t* slots, void* q_out, void* k_cache,
                   void* v_cache, int nh, int nkv, int hd, int block_size, int nt, int waves, void* stream);

/* ssd_gemm_fused with the norm prologue fed by the producer GEMM's fp32 partial slabs [splits][M][K] (ssd_gemm_parts)
 * instead of bf16 rows: h = bf16(sum over the slabs, in order), the value the reference's F.linear would have stored. */
int ssd_gemm_fused_parts(const void* h_parts, int splits, const void* res_in, void* res_out, const void* norm_w, float eps,
                         const void* w_frag, const void* bias, int M, int N, int K, int epilogue, void* y, int ldy,
                         const int64_t* positions, const float* cos_sin, const int32_t* slots, void* q_out, void* k_cache,
                         void* v_cache, int nh, int nkv, int hd, int block_size, int nt, int waves, void* stream);

/* (RMSHeadNorm q/k, Qwen3: ssd/models/qwen3.py:96-104) + RotaryEmbedding.forward
 * (ssd/layers/rotary_embedding.py:40-60) + store_kvcache (ssd/layers/attention.py:10-41).
 * qkv_rows [T][(nh+2nkv)*hd]; cos_sin fp32 [max_pos][hd] (cos || sin); q_norm_w/k_norm_w bf16[hd] or NULL. */
int ssd_rope_store_kv(const void* qkv_rows, const int64_t* positions, const float* cos_sin,
                      const int32_t* slot_mapping, void* q_out_rows, void* k_cache, void* v_cache,
                      const void* q_norm_w, const void* k_norm_w, float eps, int T, int nh, int nkv, int hd,
                      int block_size, int qkv_perm, void* stream);
/* Same, with the QKV rows given as `splits` fp32 split-K slabs parts[s][T][(nh+2nkv)*hd] of the prefill GEMM (ssd_gemm_pf with
 * epilogue 2): a value is bf16(slab 0 + slab 1 + ...), what the GEMM's own epilogue (the F.linear store, ssd/layers/linear.py:98)
 * would have written -- bit-identical to ssd_gemm_pf rows + ssd_rope_store_kv, one launch less per prefill layer. */
int ssd_rope_store_kv_parts(const float* parts, int splits, const int64_t* positions, const float* cos_sin,
                            const int32_t* slot_mapping, void* q_out_rows, void* k_cache, void* v_cache,
                            const void* q_norm_w, const void* k_norm_w, float eps, int T, int nh, int nkv, int hd,
                            int block_size, int qkv_perm, void* stream);

/* Attention.forward, all branches -- ssd/layers/attention.py:73-134.
 *   mode 0: causal, bottom-right aligned over context_lens (prefill :90-93, verify/glue :105-111,
 *           single-query decode :126-131).  cu_q int32[B+1] or NULL (then q_per_seq queries per sequence).
 *   mode 1: draft-tree decode (:113-125): tree_mq queries per sequence, structural mask of
 *           ssd/engine/helpers/mask_helpers.py:12-21 at tree step `tree_step`; tree_jidx int32[B][tree_mq]
 *           gives each branch's glue position (NULL -> branch / tree_F).
 * splits = key-range splits per (sequence, kv head) (static per launch; ranges derive from context_lens on
 * device).  ws_o fp32[T*nh*splits*hd], ws_ml fp32[T*nh*splits*2] needed when splits > 1.
 * flags bit0: use scalar LDS gathers instead of ds_read_b64_tr_b16 (diagnostic).
 * flags bit1: single-bf16 probabilities in P.V (FlashAttention's rounding) instead of the default hi+lo split.
 * flags bit2: one 16-row tile per workgroup also for query blocks of more than 8 row tiles per kv head (default: two) -- bit-identical,
 *             twice the workgroups; the host takes it for prefill chunks (ssd_amd/model.py _attn_flags).
 * flags bits 8..11: waves per workgroup (1..8, 0 = 1) that split the key range and merge in LDS. */
int ssd_attn_paged(const void* q_rows, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                   int max_blocks, const int32_t* context_lens, const int32_t* cu_q, int q_per_seq, int B, int T,
                   int max_q, int nh, int nkv, int hd, int block_size, float scale, int mode, int tree_K,
                   int tree_mq, int tree_step, int tree_F, const int32_t* tree_jidx, int splits, int flags,
                   void* ws_o, void* ws_ml, void* out_rows, void* out_frag, void* stream);

/* The same kernel under the names of the reference's two other attention call sites (thin forms: no split workspaces, one key range):
 *   ssd_attn_prefill_varlen  flash_attn_varlen_func, ssd/layers/attention.py:90-93 -- B packed causal sequences (cu_q int32[B + 1]) over the
 *                            paged cache this forward has just filled (context_lens = total lengths; T = cu_q[B] rows, max_q the longest)
 *   ssd_attn_tree            the draft tree's custom-mask prefill, ssd/layers/attention.py:113-125 + ssd/engine/helpers/mask_helpers.py:12-21 --
 *                            tree_mq branch rows per sequence at step tree_step (T = B * tree_mq), mask computed from (branch, step) */
int ssd_attn_prefill_varlen(const void* q_rows, const void* k_cache, const void* v_cache, const int32_t* block_tables, int max_blocks,
                            const int32_t* context_lens, const int32_t* cu_q, int B, int T, int max_q, int nh, int nkv, int hd,
                            int block_size, float scale, void* out_rows, void* out_frag, void* stream);
int ssd_attn_tree(const void* q_rows, const void* k_cache, const void* v_cache, const int32_t* block_tables, int max_blocks,
                  const int32_t* context_lens, int B, int tree_K, int tree_mq, int tree_step, int tree_F, const int32_t* tree_jidx,
                  int nh, int nkv, int hd, int block_size, float scale, void* out_rows, void* out_frag, void* stream);

/* Attention + o_proj in ONE launch for the single-GPU drafts' decode / glue forwards: flash_attn_with_kvcache
 * (ssd/layers/attention.py:105-111,126-131) followed by RowParallelLinear o_proj (ssd/layers/linear.py:186-199, no all-reduce
 * at tp = 1).  One sequence, T causal (bottom-right aligned) query rows; parts = fp32 slabs [nkv][T][N], slab h = o_proj
 * restricted to the columns of kv head h's q heads: their sum over h is o_proj(attention output), consumed exactly like
 * ssd_gemm_parts' slabs (ssd_gemm_fused_parts / ssd_rmsnorm_parts with splits = nkv).  T * (nh / nkv) <= 32 (hd 64) or 16
 * (hd 128), (nh / nkv) * hd <= 256, N % 128 == 0, nkv <= 16; the whole context is scanned by the 8 waves of a workgroup (use
 * it up to ~1 K keys). */
int ssd_attn_oproj_parts(const void* q_rows, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                         int max_blocks, const int32_t* context_lens, int T, int nh, int nkv, int hd, int block_size,
                         float scale, const void* w_o_frag, int N, void* parts, void* stream);

/* LM head on the greedy path: F.linear + logits.argmax(-1) -- ssd/layers/embed_head.py:88-116 followed by
 * ssd/layers/sampler.py:15-20 / ssd/utils/verify.py:34.  ssd_gemm_wf_argmax writes the bf16 logits rows like ssd_gemm_wf
 * (M <= 32) AND, per workgroup, the (max value, lowest index) of each token row over the features that workgroup produced
 * (compared on the bf16-rounded logits): part_val / part_idx [m * part_stride + p], p < ssd_gemm_wf_argmax_parts(M, N, K)
 * (a host-side query; returns the count, or a negative error).  ssd_argmax_parts* finish the argmax from those candidates
 * (larger value, then lower index == argmax over the stored logits) and, in the same launch, do what the loop does with
 * the tokens next:
 *   ssd_argmax_parts          out / out2 / out3[row * out3_stride] (any may be NULL) = idx + idx_offset; out_val (optional)
 *                             = the row maximum (vocab-parallel merge input, see ssd_argmax_merge)
 *   ssd_argmax_parts_verify   + ssd_verify_greedy (K + 1 <= 16 rows per sequence; preds optional [B*(K+1)])
 *   ssd_argmax_parts_advance  + ssd_draft_advance */
int ssd_gemm_wf_argmax_parts(int M, int N, int K);
int ssd_gemm_wf_argmax(const void* x_frag, const void* w_frag, const void* bias, void* y, int M, int N, int K, int ldy,
                       float* part_val, int32_t* part_idx, int part_stride, void* stream);

/* The single-token decode chain (one sequence, M = 1: SpeculatorSync's draft chain, ssd/engine/speculator_sync.py:25-69, and the
 * JIT chain of ssd/engine/draft_runner.py:186-378): everything of a decoder layer between two attention launches in ONE launch --
 * LlamaDecoderLayer.forward (ssd/models/llama3.py:128-199) minus the attention call: o_proj, residual add + post-attention
 * RMSNorm, gate_up + SiluAndMul, down_proj, residual add, and then EITHER the next layer's input RMSNorm + QKV projection + RoPE +
 * store_kvcache (w_qkv_next != NULL; q_out / k_cache / v_cache / positions / slots / cos_sin are the NEXT layer's) OR, on the last
 * layer (h_out != NULL), the hand-over to the final norm: h_out = down_proj rows, res_out = the residual they are added to.
 * 256 resident workgroups; the three all-to-all edges inside are all-gathers of finished bf16 vectors through data-tagged
 * 8-byte granules (csrc/chain.hip).  Same rounding points as the separate launches; fp32 summation order differs (tolerance).
 *   granules  ssd_chain_granule_bytes(h, I) bytes, zeroed ONCE at allocation
 *   gen       uint32 device word; ssd_chain_tick(gen, stream) once per forward, before its first segment
 *   err       uint32 device word, set to 1 if a bounded wait gave up (the forward's results are then invalid)
 * Shapes: ssd_chain_segment_ok(...) == SSD_OK (h, qn, I multiples of 128; h <= 4096; I <= 16384; no biases, no q/k norm). */
int ssd_chain_tick(void* gen, void* stream);
int ssd_chain_granule_bytes(int h, int I);
int ssd_chain_segment_ok(int h, int qn, int I, int qkv_n, int nh, int nkv, int hd);
int ssd_chain_segment(const void* a_frag, const void* res_in, void* res_out, void* h_out, const void* w_o, const void* w_gu,
                      const void* w_d, const void* w_qkv_next, const void* ln_post, const void* ln_next, float eps,
                      const int64_t* positions, const float* cos_sin, const int32_t* slots, void* q_out, void* k_cache, void* v_cache,
                      int h, int qn, int I, int qkv_n, int nh, int nkv, int hd, int block_size, int layer, void* granules,
                      const void* gen, void* err, void* stream);

/* The same layer segment for 2..30 token rows (csrc/tree_segment.hip): the MQ_LEN-branch tree-decode step of asynchronous speculation
 * (DraftRunner._decode_tree, ssd/engine/draft_runner.py:713-812: K forwards of (K+1)*F rows through LlamaDecoderLayer.forward,
 * ssd/models/llama3.py:128-199) and the K+1-row glue decode (draft_runner.py:560-640).  Operands as ssd_chain_segment with M rows:
 * a_frag frag [M][qn], res_in / res_out / h_out rows [M][h] (res_out != res_in), positions / slots [M], q_out rows [M][nh*hd].
 * 256 resident workgroups; the all-to-all edges are 16-byte write-through stores + one flag word per producer workgroup, payload
 * read with sc1 loads; x^ of all M rows lives in LDS.  h in {1024, 2048}; no biases.
 * qkv_rows_next (models with a per-head q / k RMSNorm, ssd/models/qwen3.py:96-104: the norm needs a whole head, i.e. eight of this
 * kernel's workgroups): instead of the RoPE + KV-store epilogue the NEXT layer's raw QKV projection rows [M][qkv_n] are written (in the
 * rotation-paired order of its weights, qkv_perm = 1) for ssd_rope_store_kv; positions / cos_sin / slots / q_out /
 * k_cache / v_cache are then NULL.
 *   workspace  ssd_tree_segment_workspace_bytes(h, I) bytes, zeroed ONCE at allocation (flags + the three hand-off buffers)
 *   gen / err  as ssd_chain_segment (one ssd_chain_tick per forward)
 * Returns SSD_ERR_LAUNCH when the device cannot keep 256 of its workgroups resident at once (they wait for each other). */
int ssd_tree_segment_workspace_bytes(int h, int I);
int ssd_tree_segment_ok(int M, int h, int qn, int I, int qkv_n, int nh, int nkv, int hd);
int ssd_tree_segment(const void* a_frag, const void* res_in, void* res_out, void* h_out, const void* w_o, const void* w_gu,
                     const void* w_d, const void* w_qkv_next, const void* ln_post, const void* ln_next, float eps,
                     const int64_t* positions, const float* cos_sin, const int32_t* slots, void* q_out, void* k_cache, void* v_cache,
                     void* qkv_rows_next, int M, int h, int qn, int I, int qkv_n, int nh, int nkv, int hd, int block_size, int layer,
                     void* workspace, const void* gen, void* err, void* stream);
int ssd_argmax_parts(const float* part_val, const int32_t* part_idx, int nparts, long part_stride, int T, long idx_offset,
                     int64_t* out, int64_t* out2, int64_t* out3, long out3_stride, float* out_val, void* stream);
int ssd_argmax_parts_verify(const float* part_val, const int32_t* part_idx, int nparts, long part_stride,
                            const int64_t* speculations, int B, int K, int64_t* preds, int32_t* accept_len,
                            int64_t* recovery, int64_t* packed, void* stream);
int ssd_argmax_parts_advance(const float* part_val, const int32_t* part_idx, int nparts, long part_stride, int64_t* next,
                             int64_t* input_ids, int64_t* positions, int32_t* slots, int32_t* context_lens,
                             const int32_t* block_tables, int max_blocks, int block_size, int64_t* spec, int K,
                             int32_t* step, int B, void* stream);

/* Sampler.forward at temperature 0 -- ssd/layers/sampler.py:15-20; verify.py:34.  out2 optional copy. */
int ssd_argmax_rows(const void* logits_rows, long ld, int T, int V, int64_t* out, int64_t* out2, void* stream);
/* Vocab-parallel form of the same argmax (ParallelLMHead gather + cat, ssd/layers/embed_head.py:88-92, followed by
 * argmax): each rank reduces its shard to (max value, global index = local + idx_offset); the per-rank rows (strides in elements of each array) are
 * all-gathered (16 bytes per row instead of the logits) and merged: larger value, then lower index. */
int ssd_argmax_rows_val(const void* logits_rows, long ld, int T, int V, long idx_offset, int64_t* out_idx,
                        float* out_val, void* stream);
int ssd_argmax_merge(const float* vals, const int64_t* idxs, int tp, int T, long stride, long stride_idx, int64_t* out,
                     int64_t* out2, void* stream);

/* verify(), greedy branch -- ssd/utils/verify.py:28-48.  preds/speculations int64 [B][K+1].
 * packed (optional) int64 [B][K+3] = (accept_len, recovery, spec_0..spec_K): the step's whole result in one D2H
 * copy instead of the reference's four .tolist() syncs (verify.py:173-181). */
int ssd_verify_greedy(const int64_t* preds, const int64_t* speculations, int B, int K, int32_t* accept_len,
                      int64_t* recovery, int64_t* packed, void* stream);

/* Temperature > 0 (csrc/stochastic.hip).  rng_state: uint64 device word (seed); advance it with ssd_rng_advance after each
 * use so hipGraph replays draw fresh numbers.  temps float[T / rows_per_temp] (one temperature per sequence).
 * ssd_sample_rows: Sampler.forward -- ssd/layers/sampler.py:15-36 (T == 0 -> argmax; else Gumbel-max == the reference's
 * argmax(softmax / Exp(1))).  ssd_row_lse: log-sum-exp of logits / T per row (softmax normaliser of verify.py:76-99).
 * ssd_verify_ratio: verify() with ratio acceptance and residual resampling -- ssd/utils/verify.py:50-167.  ratio_rows
 * int32[B]: 1 where the draft tokens were really drawn from q (cache hit or JIT), else greedy acceptance + recovery ~ p.
 * accept_prob (optional) float[B][K] receives min(1, p/q) per position.
 * sampler_x (apply_sampler_x_rescaling -- ssd/utils/async_helpers/async_spec_helpers.py:79-105; sampler.py:29-31;
 * verify.py:101-105): boost_idx int32[rows][boost_k] = the F+1 most probable tokens of each row (ssd_topk_rows),
 * boost_x = sampler_x; NULL disables it.  ssd_row_lse and ssd_verify_ratio must see the same boost rows for q. */
int ssd_topk_rows(const void* logits_rows, long ld, int T, int V, int k, int32_t* out_idx, void* stream);
int ssd_sample_rows(const void* logits_rows, long ld, int T, int V, const float* temps, int rows_per_temp,
                    const void* rng_state, unsigned salt, int64_t* out, int64_t* out2, const int32_t* boost_idx,
                    int boost_k, float boost_x, void* stream);
int ssd_rng_advance(void* rng_state, void* stream);
int ssd_row_lse(const void* logits_rows, long ld, int T, int V, const float* temps, int rows_per_temp, float* lse,
                const int32_t* boost_idx, int boost_k, float boost_x, void* stream);
int ssd_verify_ratio(const void* logits_p, long ld_p, const void* logits_q, long ld_q, int V, int B, int K,
                     const int64_t* speculations, const int64_t* preds_p, const float* lse_p, const float* lse_q,
                     const float* temps_t, const float* temps_q, const int32_t* ratio_rows, const void* rng_state,
                     unsigned salt, int32_t* accept_len, int64_t* recovery, int64_t* packed, float* accept_prob,
                     const int32_t* boost_idx_q, int boost_k, float boost_x, void* stream);

/* get_forked_recovery_tokens_from_logits -- ssd/utils/async_helpers/async_spec_helpers.py:26-78.
 * counts/offsets int32 [B][K+1]: fan-out and output offset of each glue position. */
int ssd_fork_topf(const void* logits_rows, long ld, int V, const int64_t* returned_tokens, const int32_t* counts,
                  const int32_t* offsets, int B, int K, int mq, int64_t* out, void* stream);
/* The same selection spread over the chip (every row cut into slices of <= 4096 logits, per-slice top-F candidates in `workspace`
 * -- ssd_fork_topf_workspace_bytes(V, B, K) bytes -- then one wave per row merges them): bit-equal to ssd_fork_topf, two short
 * launches instead of B*(K+1) workgroups walking whole vocabulary rows F times (84.7 -> ~8 us at V = 128256).  V % 8 == 0 and
 * V <= 196608 (48 slices): ssd_fork_topf_workspace_bytes returns SSD_ERR_SHAPE (< 0) for a vocabulary the split form refuses --
 * the predicate a caller gates on before it captures the call in a graph. */
int ssd_fork_topf_workspace_bytes(int V, int B, int K);
int ssd_fork_topf_split(const void* logits_rows, long ld, int V, const int64_t* returned_tokens, const int32_t* counts,
                        const int32_t* offsets, int B, int K, int mq, void* workspace, int64_t* out, void* stream);

/* Speculation-cache lookup -- the tensor compare of DraftRunner.hit_cache_and_respond, ssd/engine/draft_runner.py:215-252.
 * The cache of a round has Bc * W entries: entry c = b * W + i has key (cache_seq[b], cache_j[c], cache_forks[c]) =
 * (sequence id, glue position of branch i, fork token of branch i).  out_idx[r] (int32[B]) = first entry equal to request key
 * r = req_keys[r][0..2] (int64 [B][3]: seq id, accepted length - 1, recovery token), or -1. */
int ssd_cache_lookup(const int64_t* req_keys, const int64_t* cache_seq, const int32_t* cache_j, const int64_t* cache_forks,
                     int B, int Bc, int W, int32_t* out_idx, void* stream);

/* Device-side replacement for the host loop body of SpeculatorSync.speculate --
 * ssd/engine/speculator_sync.py:47-66 (+ runner_helpers.py:59-75): append the sampled token, bump
 * position / context length, recompute the KV slot from the block table. */
int ssd_draft_advance(const int64_t* next, int64_t* input_ids, int64_t* positions, int32_t* slots,
                      int32_t* context_lens, const int32_t* block_tables, int max_blocks, int block_size,
                      int64_t* spec, int K, int32_t* step, int B, void* stream);

/* logits_q[b][*step] <- src row b (bf16 [B][K][V]); collects the draft logits of a device-side chain step
 * (torch.stack(logits_q), ssd/engine/speculator_sync.py:58,67). */
int ssd_store_step_rows(const void* src_rows, long src_ld, void* dst, int B, int V, int K, const int32_t* step, void* stream);

/* One-shot full-mesh all-reduce (sum, bf16 in/out, fp32 accumulate in rank order) over hipIpc-shared fine-grained
 * buffers -- replaces dist.all_reduce after o_proj / down_proj / the embedding (ssd/layers/linear.py:195-199,
 * ssd/layers/embed_head.py:53-56) for the small decode-time messages; csrc/comm.hip describes the protocol.
 * Setup (not hot path): ssd_comm_alloc (fine-grained device memory, zeroed) / ssd_comm_ipc_export (64-byte handle) /
 * ssd_comm_ipc_open (map a peer's allocation) / ssd_comm_ipc_close / ssd_comm_free.
 * ssd_allreduce_bf16: slots[r] / flags[r] = rank r's staging area (2 * slot_elems bf16) and flag array (8*8 uint32);
 * counters uint32[8] and err uint32[1] are local device words (zeroed once); err becomes 1 if a peer did not arrive
 * within spin_budget polls (the call then leaves `out` undefined and the caller must fall back). */
int ssd_comm_alloc(void** out, long bytes);
int ssd_comm_free(void* p);
int ssd_comm_ipc_export(void* p, void* handle64);
int ssd_comm_ipc_open(const void* handle64, void** out);
int ssd_comm_ipc_close(void* p);
int ssd_allreduce_bf16(const void* in, void* out, long n, int rank, int world, void* const* slots, void* const* flags,
                       long slot_elems, void* counters, void* err, long spin_budget, void* stream);
/* Same transport as an all-gather of n8 opaque 8-byte words per rank: out [world][n8] (replaces the logits gather of
 * ParallelLMHead, ssd/layers/embed_head.py:88-92, by a (value, index) exchange of 12 bytes per row). */
int ssd_allgather_u64(const void* in, void* out, long n8, int rank, int world, void* const* slots, void* const* flags,
                      long slot_elems, void* counters, void* err, long spin_budget, void* stream);

/* RowParallelLinear's all_reduce (ssd/layers/linear.py:195-199) fused with the add + RMSNorm that always follows it
 * (ssd/layers/layernorm.py:76-88; ssd/models/llama3.py:185-199): res_out = bf16(allreduce(in) + res_in),
 * out = bf16(x32 * rsqrt(mean(x32^2) + eps) * weight) row-major and/or fragment-major.  Bit-identical to
 * ssd_allreduce_bf16 followed by ssd_rmsnorm; same slots / flags / counters.  T*H <= slot_elems. */
int ssd_allreduce_add_rmsnorm_bf16(const void* in, const void* res_in, void* res_out, const void* weight, float eps,
                                   void* out_rows, void* out_frag, int T, int H, int rank, int world, void* const* slots,
                                   void* const* flags, long slot_elems, void* counters, void* err, long spin_budget,
                                   void* stream);

/* The same two collectives over DATA-TAGGED GRANULES (round 4; csrc/comm.hip): every rank pushes its values into each peer's
 * inbox as 8-byte {2 x bf16, epoch} words -- one write-through store each, single-copy atomic -- and polls its OWN inbox: one
 * hop, no drain / flag / remote read, no ordering between separate payload and flag stores to rely on.  2x the wire bytes, so
 * for messages up to 64 Ki elements (every decode / verify sum of the tensor-parallel target); larger ones use the calls above.
 * inboxes[r] = rank r's inbox (2 * 8 * gr_cap granules, zeroed); counters / err are the SAME as in the calls above -- the two
 * protocols share one epoch and may be interleaved.  Replace ssd/layers/linear.py:195-199 (+ layernorm.py:76-88) like them. */
int ssd_allreduce_gr_bf16(const void* in, void* out, long n, int rank, int world, void* const* inboxes, long gr_cap,
                          void* counters, void* err, long spin_budget, void* stream);
int ssd_allreduce_add_rmsnorm_gr_bf16(const void* in, const void* res_in, void* res_out, const void* weight, float eps,
                                      void* out_rows, void* out_frag, int T, int H, int rank, int world, void* const* inboxes,
                                      long gr_cap, void* counters, void* err, long spin_budget, void* stream);

/* ---- decoders with an fp32 residual stream, sandwich norms, differential attention and a routed feed-forward (the Fatulix design;
 * no counterpart in the reference).  `f32` selects the element type of weights, GEMM-input rows and the KV cache: 0 = bf16, 1 = fp32
 * (true fp32 arithmetic throughout).  Residual rows, norm statistics, attention scores / weights and router logits are fp32 in both. ---- */

/* x_out[t] = table[ids[t]] as fp32 residual rows [T][W]; x0_out (optional) receives the same rows (designs that add the embedding
 * output again before a repeated pass keep it). */
int ssd_embed_res32(const int64_t* ids, const void* table_rows, void* x_out, void* x0_out, int T, int W, long vocab, int f32,
                    void* stream);
/* out[r] = weight * x[i] / sqrt(mean(x[i]^2) + eps), i = gather[r] or r; x fp32 [.][W].  add (optional, fp32 [T][W], no gather):
 * x += add first, written back in place. */
int ssd_rmsnorm_res32(void* x, const void* add, const void* weight, float eps, void* out_rows, const int32_t* gather, int T, int W,
                      int f32, void* stream);
/* x += weight * y / sqrt(mean(y^2) + eps): the norm AFTER a sublayer and the residual sum; y fp32 [T][W]. */
int ssd_rmsnorm_add_res32(const void* y, const void* weight, float eps, void* x, int T, int W, int f32, void* stream);
/* The tail of a sandwich sublayer in one launch: y = y_rows (fp32 [T][W]) or, when y_rows is NULL, the routed mix
 * sum_j weights[t][j] * ydn_rows[inv[t*top+j]] (+ shared_rows[t]) (written to y_scratch); x += post_weight * rms(y); then, with
 * next_weight / next_out: x += next_add (optional), next_out = next_weight * rms(x).  Same arithmetic as ssd_moe_combine +
 * ssd_rmsnorm_add_res32 + ssd_rmsnorm_res32. */
int ssd_sandwich_tail(const void* y_rows, const void* ydn_rows, const int32_t* inv, const float* weights, const void* shared_rows,
                      int top, void* y_scratch, const void* post_weight, float eps, void* x, const void* next_add,
                      const void* next_weight, void* next_out, int T, int W, int f32, void* stream);
/* fp32 rows [rows][ld_src] -> bf16 rows [rows][ld_dst]; columns cols .. ld_dst-1 of dst are set to -inf. */
int ssd_rows_f32_to_bf16(const void* src, void* dst, int rows, int cols, long ld_src, long ld_dst, void* stream);

/* y = x w^T for row-major x [M][K] and w [N][K] of ANY sizes (csrc/gemm_rows.hip).  epilogue 0: fp32 rows; 1: relu(y)^2 as
 * element-type rows; 2: element-type rows; 3 / 4 (bf16 only, N even): w rows are (gate, up) pairs -- row 2i, row 2i + 1 -- and y is
 * act(gate) * up as element-type rows [M][N / 2], act = silu (3) or tanh-form gelu (4). */
int ssd_gemm_rows(const void* x_rows, const void* w_rows, void* y, int M, int N, int K, int epilogue, int f32, void* stream);
/* The same product per group: sorted rows offsets[e] .. offsets[e+1]-1 (e < E) multiply by w_rows + e * N * K; row_idx (optional)
 * names the x row of sorted row r as row_idx[r] / idx_div, y rows are the sorted rows.  rows = offsets[E]'s upper bound. */
int ssd_gemm_rows_grouped(const void* x_rows, const void* w_rows, void* y, const int32_t* offsets, int E, const int32_t* row_idx,
                          int idx_div, int rows, int N, int K, int epilogue, int f32, void* stream);

/* Differential attention (csrc/attention_diff.hip).  qkvg_rows fp32 [T][H*2*D + G*2*D + G*Dv + H] = [q | k | v | gate logits] with
 * q and k laid out head by head as [map 1 | map 2]; q_norm_w / k_norm_w [D]; K cache [blocks][G][block_size][2*D], V cache
 * transposed per page [blocks][G][Dv][block_size]; slots int32 [T] (-1: no store); q_out [T][H*2*D]; gate_out fp32 [T][H] = sigmoid(gate logits). */
int ssd_diffattn_store(const void* qkvg_rows, const void* q_norm_w, const void* k_norm_w, float eps, const int32_t* slots,
                       void* q_out, void* gate_out, void* k_cache, void* v_cache, int T, int H, int G, int D, int Dv, int block_size,
                       int f32, void* stream);
/* out[t][h] = out_scale * gate[t][h] * rms_noweight(a_1 - lambda * a_2), a_m = softmax(scale * q_m . k_m) v over keys
 * 0 .. positions[t] of the token's sequence (cu_q int32 [B+1] row ranges, or q_per_seq rows per sequence when cu_q is NULL).
 * context_lens int32 [B] (keys each sequence holds) and max_q (most rows of one sequence) are optional (NULL / 0); with them, bf16,
 * D % 8 == 0, D <= 128, Dv % 16 == 0, Dv <= 128 and block_size % 32 == 0 the MFMA form runs, else the fp32 scalar form.
 * workspace (optional, fp32, workspace_bytes) + ctx_hint (host-side bound of the context lengths): decoding rows cut their keys
 * over up to 16 workgroups per (sequence, kv head); 4160 floats per (sequence, kv head, slice). */
int ssd_diffattn_paged(const void* q_rows, const void* k_cache, const void* v_cache, const void* gate, const int32_t* block_tables,
                       int max_blocks, const int64_t* positions, const int32_t* context_lens, const int32_t* cu_q, int q_per_seq,
                       int max_q, int B, int T, int H, int G, int D, int Dv, int block_size, float scale, float lambda, float out_scale,
                       float eps, void* out_rows, int f32, void* workspace, long workspace_bytes, int ctx_hint, void* stream);

/* Routed feed-forward (csrc/moe.hip): from the router's fp32 logits [T][E] (ssd_gemm_rows, fp32 rows out) the `top` largest per token,
 * softmax over the chosen ones;
 * counting sort of the (token, slot) pairs by expert; weighted sum of the experts' fp32 output rows (+ the shared expert's). */
int ssd_moe_route(const float* logits, int32_t* idx, float* weights, int T, int E, int top, void* stream);
int ssd_moe_plan(const int32_t* idx, int T, int top, int E, int32_t* offsets, int32_t* perm, int32_t* inv, void* stream);
int ssd_moe_combine(const void* y_rows, const int32_t* inv, const float* weights, const void* shared_rows, void* out_rows, int T,
                    int top, int W, void* stream);

/* G products in one launch (per-head matrices over column slices of token-major rows): group g multiplies x_rows + g * gsx (row
 * stride ldx) by w_rows + g * N * K and writes y + g * gsy (row stride ldy; strides in elements of the respective type). */
int ssd_gemm_rows_batched(const void* x_rows, const void* w_rows, void* y, int M, int N, int K, int G, long ldx, long gsx, long ldy,
                          long gsy, int epilogue, int f32, void* stream);

/* Parallel layers with Dynamic-Tanh norms, dyt(x) = tanh(alpha * x) * weight + bias (csrc/dyt.hip); alpha: one fp32 number in
 * device memory.  ssd_dyt_embed: x (fp32 [T][W]) = dyt(table[ids]); x0 (optional) a second fp32 copy; cat (optional) an element-type
 * copy with row stride ld_cat.  ssd_dyt_rows: out[r] = dyt(x[i]), i = gather[r] or r; add_vec (optional, [W], no gather): x += add_vec
 * first, written back. */
int ssd_dyt_embed(const int64_t* ids, const void* table, const float* alpha, const void* weight, const void* bias, void* x, void* x0,
                  void* cat, long ld_cat, int T, int W, long vocab, int f32, void* stream);
int ssd_dyt_rows(void* x, const void* add_vec, const float* alpha, const void* weight, const void* bias, void* out_rows,
                 const int32_t* gather, int T, int W, int f32, void* stream);
/* x += y_mix + ff: ff = y_ff (fp32 [T][W]) or, when y_ff is NULL and ydn_rows is given, sum_j weights[t][j] * ydn_rows[inv[t*top+j]]
 * (+ sigmoid(shared_gate[t * ld_shared_gate]) * shared_rows[t]; a NULL shared_gate means 1), or 0.  Then next_out = dyt(x) with
 * next_alpha / next_weight / next_bias (optional) and cat = x as element-type rows of stride ld_cat (optional). */
int ssd_parallel_tail(void* x, const void* y_mix, const void* y_ff, const void* ydn_rows, const int32_t* inv, const float* weights,
                      int top, const void* shared_rows, const float* shared_gate, long ld_shared_gate, const float* next_alpha,
                      const void* next_weight, const void* next_bias, void* next_out, void* cat, long ld_cat, int T, int W, int f32,
                      void* stream);
/* out[r][c] = act(ab[r][c]) * ab[r][F + c] for fp32 rows [rows][2F]; act 0: silu, 1: tanh-form gelu. */
int ssd_glu_rows(const void* ab_rows, void* out_rows, int rows, int F, int act, int f32, void* stream);

/* Latent attention with a sliding window (csrc/attention_latent.hip).  proj_rows fp32 [T][ld] = [dq (q_rank) | latent (kv_rank) |
 * rotated key part (rot) | gate logits (H)].  Store: cq_out [T][q_rank] = rms(dq) * q_norm_w; cache row slots[t] (-1: none) of
 * cache [rows][kv_rank + rot] = [rms(latent) * kv_norm_w | rope(rotated key part)]; gate_out fp32 [T][H] = sigmoid.  rope turns the
 * first rot_dims entries (entry i pairs with i + rot_dims / 2) by positions[t] * freqs[i] with cos and sin times mag.
 * q_norm_w NULL: cq_out = the first q_rank entries as they are (queries that pass through no latent); gate_out NULL: no gates (the
 * row then need not hold gate logits).  ssd_latent_attn: gate NULL = 1. */
int ssd_latent_store(const void* proj_rows, long ld, int q_rank, int kv_rank, int rot, int H, const void* q_norm_w,
                     const void* kv_norm_w, float eps, const int64_t* positions, const float* freqs, float mag, int rot_dims,
                     const int32_t* slots, void* cq_out, void* cache, void* gate_out, int T, int f32, void* stream);
/* out[t][h] (kv_rank wide) = gate[t][h] * sum_j softmax_j(scale * (<q_abs[t][h], c_j> + <rope(q_rows[t][h][D:]), k_j>)) c_j over the
 * keys j of the token's sequence with 0 <= positions[t] - j < window (window <= 0: all keys up to the token); q_abs fp32
 * [T][H][kv_rank] (element-type rows when q_abs_elem), q_rows [T][H][D + rot].  workspace (optional, fp32): with few rows the MFMA
 * form cuts the window over up to 16 workgroups per (token, 16 heads), kv_rank * 16 + 32 floats per slice, and merges.  Sequences: cu_q int32 [B+1] row ranges, or q_per_seq rows each when cu_q is NULL. */
int ssd_latent_attn(const void* q_abs, const void* q_rows, const void* cache, const void* gate, const int32_t* block_tables,
                    int max_blocks, const int64_t* positions, const int32_t* cu_q, int q_per_seq, int B, int T, int H, int D, int rot,
                    int kv_rank, int block_size, int window, float scale, const float* freqs, float mag, int rot_dims, void* out_rows,
                    int f32, int q_abs_elem, void* workspace, long workspace_bytes, void* stream);
/* 1 when the MFMA form of ssd_latent_attn takes these sizes (then the caller may hand q_abs over as element-type rows, q_abs_elem = 1:
 * 16 heads of a token per workgroup, keys in steps of 32), 0 when only the scalar form (fp32 q_abs, q_abs_elem = 0) does. */
int ssd_latent_attn_mfma_ok(int kv_rank, int rot, int f32);

/* Linear attention with per-head decay over a recurrent fp32 state (csrc/lightning.hip).  proj_rows fp32 [T][ld] holds q at q_off
 * ([H][D]), k at k_off ([H][D]), v at v_off ([H][Dv]), each passed through silu.  Per sequence b (rows cu_q[b] .. cu_q[b+1]-1, or
 * q_per_seq rows each) and head: S = state[state_slots[b]][h] (zero when the first row's position is 0), per row S = decay[h] * S +
 * k v^T, out = S^T q (fp32 [T][H*Dv]); S is written back.  act 0: q, k, v = silu of the row's values; act 1: the values as they are. */
int ssd_lightning_scan(const void* proj_rows, long ld, int q_off, int k_off, int v_off, const float* decay, const int64_t* positions,
                       const int32_t* cu_q, int q_per_seq, const int32_t* state_slots, void* state, void* out_rows, int B, int H, int D,
                       int Dv, int act, void* stream);
/* out[t] = weight * o[t] / sqrt(mean(o[t]^2) + eps) * sigmoid(proj_rows[t][g_off ..]) over N = H * Dv entries, element-type rows. */
int ssd_lightning_gate_norm(const void* o_rows, const void* proj_rows, long ld, int g_off, const void* weight, float eps,
                            void* out_rows, int T, int N, int f32, void* stream);

/* Router of the softmax-then-choose kind: scores = softmax(logits[t][0..E)) (row stride ld), experts in `groups` contiguous groups of
 * which the `keep` with the largest best score stay eligible, the `top` largest eligible scores -> idx, weights = score / (sum of
 * the chosen + 1e-20) * scale. */
int ssd_moe_route_softmax(const float* logits, long ld, int32_t* idx, float* weights, int T, int E, int top, int groups, int keep,
                          float scale, void* stream);

/* Pre-norm layers over an fp32 residual stream (csrc/prenorm.hip).  ssd_embed_pos_res32: x (fp32 [T][W]) = table[ids[t]] +
 * pos_table[positions[t]] (a learned position vector per position, unscaled; an id or position out of range gives a zero row) and,
 * when norm_weight is given, norm_out = norm_weight * x / sqrt(mean(x^2) + eps) as element-type rows.
 * ssd_prenorm_tail: x += y_rows (fp32 [T][W]) or, when y_rows is NULL, sum_j (weights ? weights[t*top+j] : 1) * ydn_rows[inv[t*top+j]];
 * then (optional) next_out = next_weight * rms(x), the input rows of the next sublayer's first GEMM. */
int ssd_embed_pos_res32(const int64_t* ids, const int64_t* positions, const void* table, const void* pos_table, void* x_out,
                        const void* norm_weight, float eps, void* norm_out, int T, int W, long vocab, long max_pos, int f32,
                        void* stream);
int ssd_prenorm_tail(void* x, const void* y_rows, const void* ydn_rows, const int32_t* inv, const float* weights, int top, float eps,
                     const void* next_weight, void* next_out, int T, int W, int f32, void* stream);
/* out[t] = coef[0] rms(z) + coef[1] rms(z^2) + coef[2] rms(z^3) + coef[3] over fp32 rows [T][F] (powers element by element, rms(v) =
 * v / sqrt(mean(v^2) + eps) per row), element-type rows out; coef: four fp32 numbers in device memory. */
int ssd_polynorm_rows(const void* z_rows, const float* coef, float eps, void* out_rows, int T, int F, int f32, void* stream);
/* Clamped swish-GLU over fp32 rows [rows][2F] = [zg | zu]: s = row_scale ? row_scale[perm ? perm[r] : r] : 1; g = min(s zg, limit),
 * u = clamp(s zu, -limit, limit); out = g * sigmoid(alpha * g) * (u + 1), element-type rows [rows][F]. */
int ssd_glu_clamp_rows(const void* ab_rows, const float* row_scale, const int32_t* perm, void* out_rows, int rows, int F, float limit,
                       float alpha, int f32, void* stream);
/* The same clamped swish-GLU as the epilogue of the grouped product (bf16 only): w_rows [E][N][K] with the rows of every expert in
 * (gate_i, up_i) pairs, y element-type rows [rows][N / 2]; s = row_scale ? row_scale[row_idx ? row_idx[m] : m] : 1 for sorted row m. */
int ssd_gemm_rows_grouped_glu_clamp(const void* x_rows, const void* w_rows, void* y, const int32_t* offsets, int E,
                                    const int32_t* row_idx, int idx_div, int rows, int N, int K, const float* row_scale, float limit,
                                    float alpha, void* stream);
/* The dense form of the same epilogue (no groups, no row factor): y [M][N / 2] = g sigmoid(alpha g) (u + 1) of the (gate, up) row pairs. */
int ssd_gemm_rows_glu_clamp(const void* x_rows, const void* w_rows, void* y, int M, int N, int K, float limit, float alpha, void* stream);
/* fp32 logit rows in place: z = scale * z, then (cap > 0) z = cap * tanh(z / cap). */
int ssd_logits_cap_rows(void* logits, int rows, int V, long ld, float scale, float cap, void* stream);
/* Router of the sigmoid kind: scores = sigmoid(logits[t][0..E)) (row stride ld), the `top` largest (lowest index wins a tie) -> idx,
 * weights = those scores as they are. */
int ssd_moe_route_sigmoid(const float* logits, long ld, int32_t* idx, float* weights, int T, int E, int top, void* stream);
/* The sigmoid router with a choice correction and group-limited choice: choice = sigmoid(logit) + correction[e] (NULL: 0); experts in
 * `groups` contiguous groups, a group's score = the sum of its `group_top` (<= 8) largest choice scores, experts outside the best
 * `keep` groups cannot be chosen (their choice score counts as -inf); the `top` largest choice scores -> idx; weights = sigmoid(logit)
 * of the chosen, as they are. */
int ssd_moe_route_sigmoid_grouped(const float* logits, long ld, const float* correction, int32_t* idx, float* weights, int T, int E,
                                  int top, int groups, int keep, int group_top, void* stream);

/* Sliding-window attention with unit-RMS q / k, capped scores, a per-head distance penalty and a softmax sink
 * (csrc/attention_window.hip).  Store: qkv_rows fp32 [T][ld] = [q (H*D) | k (G*D) | v (G*Dv)]; q_out [T][H*D] = q / rms(q) per head;
 * K cache [blocks][G][block_size][D] row slots[t] (-1: none) = k / rms(k); V cache [blocks][G][Dv][block_size] (transposed per page).
 * Attention: out[t][h] (Dv wide) = sum_j p_j v_j over the keys j of the token's sequence with 0 <= positions[t] - j < window
 * (window 0: all keys up to the token), s_j = cap * tanh(scale * <q, k_j> / cap) - slopes[h] * (positions[t] - j) (cap <= 0: no cap;
 * slopes NULL: no penalty), p_j = exp(s_j) / (sum_j' exp(s_j') + exp(sinks[h])) (sinks NULL: no sink).  max_q > 0 (an upper bound of
 * the rows any sequence of the batch brings) admits the MFMA form for bf16 and D % 32 == 0, Dv % 16 == 0, block_size % 32 == 0; max_q = 0
 * or other sizes or fp32: the scalar form. */
int ssd_winattn_store(const void* qkv_rows, long ld, float eps, const int32_t* slots, void* q_out, void* k_cache, void* v_cache, int T,
                      int H, int G, int D, int Dv, int block_size, int f32, void* stream);
int ssd_winattn_paged(const void* q_rows, const void* k_cache, const void* v_cache, const float* slopes, const float* sinks,
                      const int32_t* block_tables, int max_blocks, const int64_t* positions, const int32_t* cu_q, int q_per_seq,
                      int max_q, int B, int T, int H, int G, int D, int Dv, int block_size, int window, float scale, float cap,
                      const float* out_freqs, void* out_rows, int f32, void* stream);
/* The store of the rotary variant: q_out = rope(q_norm_w * q / rms(q)) with the RMS over ALL H * D entries of the row's q (k alike,
 * over G * D, into the K cache); rope turns the first rot_dims entries of every head (entry i pairs with i + rot_dims / 2) by
 * positions[t] * qk_freqs[i].  v_freqs (fp32 [Dv / 2], NULL: none): every value head turns over all Dv entries by positions[t] *
 * v_freqs[i] before it is cached; ssd_winattn_paged's out_freqs (NULL: none) then turns every head's output back by the query's
 * position (pair (m, m + Dv / 2) by -positions[t] * out_freqs[m]; the MFMA form takes Dv % 32 == 0 then). */
int ssd_winattn_store_rope(const void* qkv_rows, long ld, const void* q_norm_w, const void* k_norm_w, float eps, const int64_t* positions,
                           const float* qk_freqs, int rot_dims, const float* v_freqs, const int32_t* slots, void* q_out, void* k_cache,
                           void* v_cache, int T, int H, int G, int D, int Dv, int block_size, int f32, void* stream);

/* Layers that normalise a sublayer's output only, with a weighted average over the depth (csrc/postnorm.hip).
 * ssd_embed_hist: x_out fp32 [T][W] = table[ids[t]] (zeros for an id outside the table), the same into hist0 (optional) and as
 * element-type rows into rows_out (optional).
 * ssd_postnorm_tail: v = y_rows[t] (fp32) or sum_j weights[t * top + j] * ydn_rows[inv[t * top + j]];  x[t] += post_weight * v /
 * sqrt(mean(v^2) + eps) (post_weight fp32 [W]).  hist (optional, fp32 levels of hist_stride floats): level hist_levels - 1 receives
 * x[t], then x[t] = sum_(j < hist_levels) coef[j] * level_j[t].  next_out (optional): x[t] as element-type rows.
 * ssd_rmsnorm_w32_rows: out_rows[r] = weight * x[g] / sqrt(mean(x[g]^2) + eps), g = gather[r] or r; weight fp32.
 * ssd_rope_rows: in place on fp32 rows [T][ld]: blocks of `heads` heads of D entries at columns off_a and off_b (off_b < 0: one block);
 * the first rot_dims entries of a head turn (entry i pairs with i + rot_dims / 2) by positions[t] * freqs[i], then the head is
 * multiplied by the block's scale.
 * ssd_gate_rows: out_rows[t][c] = o_rows[t * ldo + c] * sigmoid(gate_rows[t * ldg + c]) for c < N, element-type rows out. */
int ssd_embed_hist(const int64_t* ids, const void* table, void* x_out, void* hist0, void* rows_out, int T, int W, long vocab, int f32,
                   void* stream);
int ssd_postnorm_tail(const void* y_rows, const void* ydn_rows, const int32_t* inv, const float* weights, int top,
                      const float* post_weight, float eps, void* x, void* hist, long hist_stride, int hist_levels, const float* coef,
                      void* next_out, int T, int W, int f32, void* stream);
int ssd_rmsnorm_w32_rows(const void* x, const float* weight, float eps, void* out_rows, const int32_t* gather, int T, int W, int f32,
                         void* stream);
int ssd_rope_rows(void* rows, long ld, const int64_t* positions, const float* freqs, int rot_dims, int heads, int D, int off_a,
                  float scale_a, int off_b, float scale_b, int T, void* stream);
int ssd_gate_rows(const void* o_rows, long ldo, const void* gate_rows, long ldg, void* out_rows, int T, int N, int f32, void* stream);

/* Recurrent mixers over per-sequence state slots (csrc/recurrent.hip).  Sequences: cu_q int32 [B+1] row ranges, or q_per_seq rows
 * each; state_slots int32 [B]; a sequence whose first row has position 0 starts from zero whatever its slot holds.
 * ssd_token_shift_mix: out[t][s] (W wide, s < S) = h + (h_prev - h) * mu[s] for element-type rows hn_rows [T][W]; h_prev = the row
 * before in the batch, shift_state[slot] (fp32 [slots][W]) for a portion's first row, zero at position 0.
 * ssd_wkv_scan: proj_rows fp32 [T][ld] holds r, k, v ([H][D] each) at r_off / k_off / v_off, decay_rows fp32 [T][ldw] the decay
 * logits; per head w = exp(-exp(decay + w0)), o = (S + diag(u) k v^T)^T r, S = diag(w) S + k v^T over state fp32 [slots][H][D][D];
 * out fp32 [T][H*D]; also shift_state[slot] = the sequence's last row of hn_rows.
 * ssd_causal_conv_silu: out fp32 [T][C] = silu(conv_b[c] + sum_j conv_w[c][j] * in[t - (taps - 1 - j)][c]), in = proj_rows columns
 * col_off .. col_off + C; inputs before a portion come from conv_state fp32 [slots][taps - 1][C] (last row = most recent).
 * ssd_ssd_scan: per head (group h / (H / G)) dt = softplus(proj_rows[t][dt_off + h] + dt_bias[h]), S = exp(-exp(a_log[h]) dt) S +
 * dt B x^T over state fp32 [slots][H][N][Dv], y = S^T C + skip[h] x; x / B / C = xbc_rows fp32 [T][ldx] at x_off ([H][Dv]), b_off,
 * c_off ([G][N] each); out fp32 [T][H*Dv]; also saves the last taps - 1 rows of proj_rows columns conv_off .. conv_off + C into
 * conv_state[slot].
 * ssd_group_gate_norm: rows of N entries in `groups` equal parts, g = silu(gate_rows[t][c]) (fp32, row stride ldg): gate_first ?
 * weight * rms_part(o * g) : weight * rms_part(o) * g, element-type rows. */
int ssd_token_shift_mix(const void* hn_rows, const void* mu, const float* shift_state, const int64_t* positions, const int32_t* cu_q,
                        int q_per_seq, const int32_t* state_slots, int B, void* out_rows, int T, int W, int S, int f32, void* stream);
int ssd_wkv_scan(const void* proj_rows, long ld, int r_off, int k_off, int v_off, const void* decay_rows, long ldw, const float* w0,
                 const float* u, const int64_t* positions, const int32_t* cu_q, int q_per_seq, const int32_t* state_slots, void* state,
                 void* out_rows, const void* hn_rows, void* shift_state, int W, int B, int H, int D, int f32, void* stream);
int ssd_causal_conv_silu(const void* proj_rows, long ld, int col_off, int C, const void* conv_w, const void* conv_b,
                         const float* conv_state, const int64_t* positions, const int32_t* cu_q, int q_per_seq,
                         const int32_t* state_slots, int B, void* out_rows, int T, int taps, int f32, void* stream);
int ssd_ssd_scan(const void* xbc_rows, long ldx, int x_off, int b_off, int c_off, const void* proj_rows, long ld, int dt_off,
                 const float* dt_bias, const float* a_log, const float* skip, const int64_t* positions, const int32_t* cu_q,
                 int q_per_seq, const int32_t* state_slots, void* state, void* out_rows, int conv_off, int C, void* conv_state,
                 int taps, int B, int H, int G, int N, int Dv, void* stream);
int ssd_group_gate_norm(const void* o_rows, const void* gate_rows, long ldg, const void* weight, float eps, void* out_rows, int T,
                        int N, int groups, int gate_first, int f32, void* stream);

/* hipGraph capture for a host that is not PyTorch -- the reference captures its decode / verify / glue / tree steps with
 * torch.cuda.CUDAGraph (ssd/engine/helpers/cudagraph_helpers.py:20-120); every entry point above only enqueues on `stream`, so the calls
 * between ssd_graph_begin and ssd_graph_end become ONE replayable graph.  stream: a non-null hipStream_t; *out_exec: the executable graph. */
int ssd_graph_begin(void* stream);
int ssd_graph_end(void* stream, void** out_exec);
int ssd_graph_launch(void* exec, void* stream);
int ssd_graph_destroy(void* exec);

#ifdef __cplusplus
}
#endif
#endif
