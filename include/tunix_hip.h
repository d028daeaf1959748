/*
 * tunix_hip.h -- C ABI of libtunix_hip.so: hand-written gfx950 (MI355X) kernels for the
 * quantized rollout-decode path of google/tunix (Sampler decode step on int4/NF4 QLoRA
 * models + per-token logps).
 *
 * Conventions (all entry points):
 *   - extern "C"; `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *   - every pointer is a DEVICE pointer unless its name starts with `h_`;
 *   - no allocation, no synchronisation, no host callback inside; outputs are caller-allocated;
 *   - in-place updates (KV cache, token buffer) use the same pointer for input and output;
 *   - return 0 on success, a negative TNX_E* code otherwise; tnx_last_error() returns the
 *     calling thread's last message;
 *   - bf16 values are raw uint16_t bit patterns; all matrices are row-major;
 *   - scalars that change from one decode step to the next (step index, positions) are read
 *     from device memory so that a captured HIP graph of one step can be replayed unchanged.
 *
 * Each declaration cites the reference code (paths relative to the google/tunix tree) whose
 * arithmetic the entry point replaces.
 */
#ifndef TUNIX_HIP_H_
#define TUNIX_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TNX_OK 0
#define TNX_EINVAL (-22)  /* bad shape / alignment / enum                         */
#define TNX_ELAUNCH (-5)  /* hipGetLastError() != hipSuccess after a kernel launch */
#define TNX_ENOSYS (-38)  /* combination not built                                 */

/* Weight code books. INT4: code u in [0,15] means the integer u-8. NF4: the 16 QLoRA levels. */
#define TNX_Q_INT4 0
#define TNX_Q_NF4 1

/* RMSNorm dtype flows (tunix/models/llama3/model.py:290-297, qwen3/model.py:450-456,
 * gemma3/model.py:940-950). */
#define TNX_NORM_LLAMA 0
#define TNX_NORM_QWEN3 1
#define TNX_NORM_GEMMA3 2

/* RoPE dtype flows (llama3/model.py:249-270 fp32 sin/cos; qwen3/model.py:404-425 sin/cos
 * rounded to bf16 first; gemma3/model.py:402-430 fp32 with base frequency + scale factor). */
#define TNX_ROPE_LLAMA 0
#define TNX_ROPE_QWEN3 1
#define TNX_ROPE_GEMMA3 2

/* Epilogues of tnx_qlinear_lora. */
#define TNX_EPI_STORE 0     /* y = bf16(acc)                                               */
#define TNX_EPI_RESIDUAL 1  /* y = bf16(bf16(acc) + residual)      (llama3/model.py:560-563) */
#define TNX_EPI_SILU_MUL 2  /* y = bf16(bf16(silu(bf16 g)) * bf16 u) (llama3/model.py:493)    */
#define TNX_EPI_GELU_MUL 3  /* y = bf16(bf16(gelu_tanh(bf16 g)) * bf16 u) (gemma3/model.py:785-797) */
#define TNX_EPI_F32 4       /* y(fp32) = acc, no rounding                                   */

const char* tnx_last_error(void);
/* Library / ABI version: (major << 16) | minor, the value tnx_version() returns.
 * Rule: the MAJOR number changes whenever an existing entry point changes its argument list or
 * meaning, or a descriptor struct changes its layout (a field added, removed, moved or retyped):
 * a caller built against another major number must not call the library.  The MINOR number counts
 * additions that leave every existing entry point and struct exactly as they were (new entry
 * points, new enum values); a caller built against minor m runs on any minor >= m of the same
 * major.  A caller checks tnx_version() >> 16 == TNX_ABI_VERSION_MAJOR and
 * (tnx_version() & 0xffff) >= TNX_ABI_VERSION_MINOR before its first call.
 * History: 1.0 first ABI; 1.1 added tnx_rmsnorm_moe_combine (and, against this rule, an argument
 * of tnx_quantize_pack and a field of tnx_lmhead_desc); 2.0 states the rule, keeps those changes,
 * adds tnx_attn_desc.segment_ids, reads top_k == V in tnx_sample_topk as a real top-k, and moves
 * the measurement probe tnx_stream_read out of the library; 3.0 adds tnx_qw_expand /
 * tnx_qw_expanded_bytes, tnx_dense_expand and the w_expanded field of tnx_qlinear_desc and
 * tnx_lmhead_desc; 3.1 adds tnx_sample_topk_head / tnx_sample_topk_head_ok. */
#define TNX_ABI_VERSION_MAJOR 3
#define TNX_ABI_VERSION_MINOR 1
#define TNX_ABI_VERSION ((TNX_ABI_VERSION_MAJOR << 16) | TNX_ABI_VERSION_MINOR)
int tnx_version(void);

/* ---------------------------------------------------------------------------------------
 * Packed weight format ("QW"), defined by this library (qwix's QArray layout is third-party
 * and not part of the reference tree; tunix only passes weight_qtype / tile_size through at
 * tunix/cli/utils/model.py:31-77).
 *
 * A linear y[M,N] = x[M,K] . W[K,N] is quantized in groups of `group` consecutive K indices
 * per output column: scale[g,n] = bf16(absmax / 7) (INT4) or bf16(absmax) (NF4); the code of
 * an element is the nearest code-book entry of w / f32(scale) (round-half-even for INT4,
 * clamped to [-8,7]; nearest level, ties to the lower code, for NF4).  The value a kernel
 * uses is the weight dequantised to bf16,  w^[k,n] = bf16( bf16(level(code)) * scale[g(k),n] ),
 * multiplied into bf16 activations with fp32 accumulation:  y[m,n] = sum_k x[m,k] * w^[k,n].
 *
 * Storage: N is padded to a multiple of 16 and K to a multiple of 128. Codes are tiled as
 * [N/16][K/128][64 lanes][4 dwords]; lane l of a tile owns column n = 16*nt + l%16; its dword
 * j holds the 8 codes of k = 128*kt + 32*j + 8*(l/16) + i, i = 0..7, code i in bits 4i..4i+3.
 * Scales are tiled as [N/16][K/128][16][S] bf16 with S = max(2, 128/group) slots per k-tile
 * and column, slot s holding the scale of k = 128*kt + s*(128/S) .. (a group wider than a slot
 * repeats its scale), so that a lane reads its scales as one aligned 4- or 8-byte word.
 * tnx_qw_sizes() gives the byte sizes; tnx_quantize_pack() produces both arrays on device.
 * ------------------------------------------------------------------------------------- */
int tnx_qw_sizes(int64_t K, int64_t N, int group, size_t* codes_bytes, size_t* scales_bytes);

/* w: bf16 or fp32 [K,N] row-major (w_is_f32 selects).  If `interleave2` != 0 the N columns
 * are the concatenation [gate | up] of two N/2-wide matrices and are stored interleaved in
 * blocks of 16 (gate block, up block, ...) so that TNX_EPI_*_MUL sees matching columns in
 * adjacent tiles.  int4_bound: the integer the group's absmax maps to, scale = bf16(absmax /
 * int4_bound) (ignored for NF4); 7 is this format's definition above, and the parameter is there
 * so that a quantiser with another symmetric bound (7.5, 8: codes still clamp to [-8, 7]) can be
 * mirrored without an ABI change; <= 0 selects 7.  Replaces qwix's quantizer reached from
 * tunix/cli/utils/model.py:51-68. */
int tnx_quantize_pack(void* stream, const void* w, int w_is_f32, int64_t K, int64_t N,
                      int group, int qtype, int interleave2, float int4_bound, uint32_t* codes,
                      uint16_t* scales);

/* Inverse of the packing for tests and export: w_out fp32 [K,N] = w^ (bf16 values). */
int tnx_qw_dequant(void* stream, const uint32_t* codes, const uint16_t* scales, int64_t K,
                   int64_t N, int group, int qtype, int interleave2, float* w_out);

/* Optional second copy of a frozen weight for calls with many rows (512 and more: prefill,
 * compute_per_token_logps): the same values w^ = bf16(bf16(level) * scale), 2 bytes per weight,
 * laid out as the matrix-instruction fragments of the many-row kernel, which then loads them as
 * they are instead of converting codes in its loop (results are bit-identical; the kernel is
 * bound by its instruction mix there, not by the 4x larger weight stream).  288 GB of HBM hold
 * it beside the packed weights: 14 GB for the 7 G linear weights of Llama-3.1-8B.  Pass the copy
 * as tnx_qlinear_desc.w_expanded / tnx_lmhead_desc.w_expanded; calls with few rows ignore it.
 * No counterpart in the reference (XLA materialises a dequantised bf16 W on every call). */
size_t tnx_qw_expanded_bytes(int64_t K, int64_t N);
int tnx_qw_expand(void* stream, const uint32_t* codes, const uint16_t* scales, int64_t K, int64_t N,
                  int group, int qtype, uint16_t* w_expanded /* 16-byte aligned */);
/* The same layout from a dense bf16 matrix w[N][K] (an unquantised or tied lm_head, [V][D]): a
 * log-probability pass over 512 rows or more then runs the head on the many-row kernel
 * (tnx_lmhead_desc.w_expanded next to w_bf16) instead of the 128 x 128 one. */
int tnx_dense_expand(void* stream, const uint16_t* w_bf16, int64_t K, int64_t N, uint16_t* w_expanded);

/* ---------------------------------------------------------------------------------------
 * Quantized linear fused with the LoRA delta:  y = epi( x . dequant(W) + lora_scale * t . B )
 * replaces Einsum.__call__ / nnx.Linear as rewritten by qwix (llama3/model.py:216-218,
 * :461-496; qwen3/model.py:361-365; gemma3/model.py:398-399) and the merge formula
 * W + (A @ B) * alpha / rank pinned at tunix/models/safetensors_saver.py:107.
 * ------------------------------------------------------------------------------------- */
typedef struct tnx_qlinear_desc {
  int64_t M, K, N;          /* N counts packed columns (after interleave2 it is 2*F)        */
  int group, qtype;
  const uint16_t* x;        /* bf16 [M,K]                                                   */
  const uint32_t* codes;    /* QW codes                                                     */
  const uint16_t* scales;   /* QW scales                                                    */
  /* LoRA (optional: lora_rank == 0 disables). t = bf16(x . A) comes from tnx_lora_down.    */
  int lora_rank;            /* r, multiple of 32                                            */
  int lora_nseg;            /* 1..4 column segments, each with its own t columns; -1: the
                               columns are an interleaved gate/up pair (even tiles use t
                               columns [0,r), odd tiles [r,2r))                             */
  int64_t lora_seg_end[4];  /* exclusive end column (packed order) of each segment, %16==0  */
  int lora_seg_toff[4];     /* first t column of each segment                               */
  int64_t t_ld;             /* row stride of t in elements                                  */
  const uint16_t* t;        /* bf16 [M, t_ld]                                               */
  const uint16_t* lora_b;   /* bf16 [N, r] (B transposed: r contiguous)                     */
  float lora_scale;         /* alpha / rank                                                 */
  int epilogue;             /* TNX_EPI_*                                                    */
  const uint16_t* residual; /* bf16 [M, N] for TNX_EPI_RESIDUAL                             */
  void* y;                  /* bf16 [M,N]; *_MUL: bf16 [M,N/2]; TNX_EPI_F32: fp32 [M,N]     */
  int split_k;              /* >1: the K range is split over work-groups, each writing its
                               partial tile into `ws`                                       */
  float* ws;                /* fp32 [split_k, M, N] workspace (need not be initialised);
                               required when split_k > 1; tnx_splitk_finish adds the
                               partial tiles in split order and applies the epilogue        */
  /* Optional (next_tpart != NULL), *_MUL epilogues with split_k == 1 only: the LoRA
   * down-projection of the NEXT linear -- the one that consumes y, e.g. down_proj after
   * gate|up -- fused into this epilogue.  Each (up to) 128-row x 128-column work-group tile leaves
   * its share of y . A_next as one fp32 fragment plane; tnx_lora_reduce adds the planes in a fixed
   * order and writes t_next = bf16(y . A_next), which tnx_lora_down would have produced.    */
  const uint16_t* next_a_t; /* bf16 [next_rank, N/2]: A_next transposed                     */
  int next_rank;            /* multiple of 16, <= 64                                        */
  float* next_tpart;        /* fp32 [ceil(M/128) * ceil(N/128)][8192]                       */
  const uint16_t* w_expanded; /* optional: tnx_qw_expand of (codes, scales); NULL: none       */
} tnx_qlinear_desc;

int tnx_qlinear_lora(void* stream, const tnx_qlinear_desc* h_desc);
/* Epilogue for split_k > 1 (same desc): y = epi(sum_z ws[z]). */
int tnx_splitk_finish(void* stream, const tnx_qlinear_desc* h_desc);

/* t[M, :R] = bf16(sum over the n_col_blocks fragment planes that tnx_qlinear_lora left in
 * tpart through next_tpart), planes added in column-block order. */
int tnx_lora_reduce(void* stream, const float* tpart, int64_t M, int64_t n_col_blocks, int R,
                    uint16_t* t, int64_t t_ld);

/* t[M, R] = bf16( x[M,K] . A ), a_t = A transposed: bf16 [R, K].  R multiple of 16.
 * The LoRA "down" half of qwix's x @ lora_a @ lora_b (shapes at
 * tunix/models/llama3/mapping_sglang_jax.py:64-145). */
int tnx_lora_down(void* stream, const uint16_t* x, int64_t M, int64_t K, const uint16_t* a_t,
                  int R, uint16_t* t, int64_t t_ld);

/* ---------------------------------------------------------------------------------------
 * Embedding gather: out[m,:] = table[ids[m],:] * scale_bf16  (scale 1.0 = plain copy).
 * Embedder.encode llama3/model.py:238-242, qwen3/model.py:390-395, gemma3/model.py:353-358
 * (gemma3 multiplies by bf16(sqrt(D))).  ids are read as ids[row_stride*b + col(+t)].
 * ------------------------------------------------------------------------------------- */
int tnx_embed(void* stream, const uint16_t* table, int64_t V, int64_t D, const int32_t* ids,
              int64_t ids_ld, const int32_t* col_ptr, int64_t B, int64_t T, float scale,
              uint16_t* out);

/* RMSNorm over the last axis, three dtype flows.
 *   h = (res_pre ? bf16(x + res_pre) : x);  if (h_out) h_out = h;
 *   y = norm(h) ;  if (res_post) y = bf16(y + res_post)
 * llama3/model.py:290-297, qwen3/model.py:450-456, gemma3/model.py:940-950; residual adds
 * llama3/model.py:560-563, gemma3/model.py:875-898. */
int tnx_rmsnorm(void* stream, const uint16_t* x, const uint16_t* res_pre, uint16_t* h_out,
                const uint16_t* w, const uint16_t* res_post, uint16_t* y, int64_t M, int64_t D,
                float eps, int flavor);
/* The same, with the input row taken from the fp32 partial planes ws[split_k][M][D] that
 * tnx_qlinear_lora leaves when split_k > 1 (N == D): x = bf16(sum_z ws[z]) in split order.  It
 * replaces tnx_splitk_finish + tnx_rmsnorm for a linear whose output feeds a residual add and a
 * norm (o_proj / down_proj: llama3/model.py:560-563).  D % 8 == 0. */
int tnx_rmsnorm_splitk(void* stream, const float* ws, int split_k, const uint16_t* res_pre,
                       uint16_t* h_out, const uint16_t* w, const uint16_t* res_post, uint16_t* y,
                       int64_t M, int64_t D, float eps, int flavor);
/* The same, with the input row taken from the k routed rows of a token: x = bf16(sum_j topk_w[m,j]
 * * y_route[m*k + j]), j ascending (tnx_moe_combine's arithmetic).  It replaces tnx_moe_combine +
 * tnx_rmsnorm where an MoE layer's output feeds the residual add and the next norm
 * (qwen3/model.py:826-832 into :450-456).  D % 8 == 0. */
int tnx_rmsnorm_moe_combine(void* stream, const uint16_t* y_route, const uint16_t* topk_w, int k,
                            const uint16_t* res_pre, uint16_t* h_out, const uint16_t* w,
                            const uint16_t* res_post, uint16_t* y, int64_t M, int64_t D, float eps,
                            int flavor);
/* Two norms in a row in one launch: y as above (input x, or the partial planes ws of a split-k
 * linear when x is NULL), then y2 = norm(y) with weight w2.  Gemma-3's block applies
 * post_attention_norm, adds the residual and applies pre_ffw_norm to the sum, and likewise
 * post_ffw_norm + residual followed by the next block's pre_attention_norm
 * (gemma3/model.py:882-898): y = h + norm(x) . w is the new residual stream, y2 the next
 * linear's input.  Results equal those of two tnx_rmsnorm launches bit for bit.  D % 8 == 0. */
int tnx_rmsnorm_pair(void* stream, const uint16_t* x, const float* ws, int split_k,
                     const uint16_t* res_pre, uint16_t* h_out, const uint16_t* w,
                     const uint16_t* res_post, uint16_t* y, const uint16_t* w2, uint16_t* y2,
                     int64_t M, int64_t D, float eps, int flavor);

/* ---------------------------------------------------------------------------------------
 * Per-head q/k RMSNorm (optional) + RoPE + KV-cache write for T tokens per row.
 *   qkv: bf16 [B*T, (Hq+2*Hkv)*dh] (q heads, then k heads, then v heads)
 *   positions[b*pos_ld + col + t], col = *col_ptr (device) : RoPE position of token t of row b
 *   cache slot of token t = (*col_ptr + t) % S
 *   q_out: bf16 [B*T, Hq*dh];  kcache/vcache: bf16 [B, Hkv, S, dh]
 * apply_rope llama3/model.py:249-270 (call sites :356-365 never pass rope_theta, so theta is
 * 1e6), qwen3/model.py:404-425 (+ q_norm/k_norm :531-532), gemma3/model.py:402-430 (+ q/k
 * norm :586-587, query pre-scale :596); cache write llama3/model.py:367-377.
 * ------------------------------------------------------------------------------------- */
typedef struct tnx_rope_desc {
  int64_t B, T, S;
  int Hq, Hkv, dh;
  int rope_flavor;           /* TNX_ROPE_*                                                  */
  float rope_scale;          /* gemma3: angles are divided by this scale factor (>= 1)      */
  const float* timescale;    /* fp32 [dh/2] device: theta^(2i/dh), computed once by the host */
  int qk_norm;               /* -1 none, else TNX_NORM_* flavour applied per head to q and k */
  float norm_eps;
  const uint16_t* q_norm_w;  /* bf16 [dh] or NULL                                           */
  const uint16_t* k_norm_w;
  float q_prescale;          /* 0 = none; gemma3 multiplies q by bf16(this) after RoPE      */
  const uint16_t* qkv;
  const int32_t* positions;
  int64_t pos_ld;
  const int32_t* col_ptr;    /* device int32: first token-buffer column of this call        */
  uint16_t* q_out;
  uint16_t* kcache;
  uint16_t* vcache;
  const float* qkv_ws;       /* optional: split_k fp32 partial planes [split_k][B*T][(Hq+2Hkv)*dh]
                                of the qkv linear (tnx_qlinear_lora with finish skipped); the
                                input is then bf16(sum of the planes, in split order) and qkv
                                may be NULL                                                   */
  int split_k;
} tnx_rope_desc;
int tnx_qknorm_rope_kvwrite(void* stream, const tnx_rope_desc* h_desc);
/* sin / cos of positions[b, *col_ptr] / timescale[i], fp32 [B, dh/2] each: the angles of the
 * Llama rotation above for one decode step, shared by all layers (input of the fused mode of
 * tnx_gqa_attn). */
int tnx_rope_table(void* stream, const int32_t* positions, int64_t pos_ld, const int32_t* col_ptr,
                   int64_t B, const float* timescale, int dh, float* sin_out, float* cos_out);

/* ---------------------------------------------------------------------------------------
 * GQA attention over the KV cache for T query tokens per row (T = 1: decode).
 * Query token t of row b sits in cache slot c = *col_ptr + t (the caller keeps *col_ptr + T <=
 * tok_ld, the ids one row of `tokens` holds) and attends slot j iff
 *   j <= c  and  tokens[b*tok_ld + j] != pad_id  and (window == 0 or j > c - window),
 * i.e. the mask of compute_attention_masks (tunix/generate/utils.py:34-58) /
 * make_causal_attn_mask (:61-83) and create_sliding_window_mask (gemma3/model.py:477-496),
 * evaluated from the token buffer instead of a dense [B,T,S] mask.
 * scores: s = bf16(q.k) ; s = bf16(s * bf16(scale)) (scale 0: skip, gemma3 pre-scales q);
 * softmax in fp32, probabilities rounded to bf16 before the PV product, fp32 accumulation,
 * output rounded to bf16 (llama3/model.py:379-396, qwen3/model.py:674-686,
 * gemma3/model.py:618-660).
 *   q: bf16 [B*T, Hq*dh]; out: bf16 [B*T, Hq*dh]; caches bf16 [B,Hkv,S,dh]
 *   Every slot of both caches must hold finite values, also the slots no token was written to
 *   yet (allocate the caches zero-filled): a masked key gets probability exactly 0, but its value
 *   row still enters the P.V product, and 0 * NaN or 0 * Inf would poison the output.
 *   ws: fp32 workspace of tnx_attn_ws_bytes() bytes (only touched when the key range is split)
 * ------------------------------------------------------------------------------------- */
typedef struct tnx_attn_desc {
  int64_t B, T, S;
  int Hq, Hkv, dh;
  float scale;
  int window;
  int32_t pad_id;
  const uint16_t* q;
  const uint16_t* kcache;
  const uint16_t* vcache;
  const int32_t* tokens;
  int64_t tok_ld;
  const int32_t* col_ptr;
  int kv_chunk;              /* keys per work-group when splitting (multiple of 32); 0: no split */
  float* ws;
  uint16_t* out;
  /* Optional fused RoPE + cache write for decode (rope_sin != NULL; needs T == 1,
   * dh == 128, a model without q/k norm and the Llama rotation): the kernel takes the step's
   * q, k and v from the qkv linear's output (finished bf16 `qkv` [B, (Hq+2Hkv)*dh], or its
   * `qkv_split` fp32 partial planes `qkv_ws`), rotates q and k exactly as
   * tnx_qknorm_rope_kvwrite does (with the step's sines / cosines from tnx_rope_table), writes k
   * and v into cache slot *col_ptr and attends them from registers; `q` is not read and that
   * separate launch is not needed. */
  const float* qkv_ws;
  const uint16_t* qkv;
  int qkv_split;
  const float* rope_sin;     /* fp32 [B, dh/2] from tnx_rope_table                           */
  const float* rope_cos;
  /* Optional, packed batches (several sequences per row, compute_per_token_logps with
   * segment_ids, tunix/rl/common.py:260-271, :408-418; qwen3/model.py:622-655): int32
   * [B, tok_ld] segment id of every slot.  When given, slot j is attended iff j <= c (and the
   * window test) and segment_ids[b, j] == segment_ids[b, c]; `tokens` and pad_id are not read
   * (padding is its own segment, as the reference's packed callers arrange it). */
  const int32_t* segment_ids;
} tnx_attn_desc;
size_t tnx_attn_ws_bytes(int64_t B, int64_t T, int64_t S, int Hq, int dh, int kv_chunk);
int tnx_gqa_attn(void* stream, const tnx_attn_desc* h_desc);

/* ---------------------------------------------------------------------------------------
 * Fused lm_head -> fp32 log-softmax statistics, never writing [M,V] logits:
 *   logit[m,v] = f32(bf16( x[m,:] . W[v,:] (+ lora) )) / temperature
 * per row m: best id (first maximal index), best logit, logsumexp, and optionally the logit
 * of a given target id.  compute_final_logits llama3/model.py:688-697; sample_best
 * tunix/generate/sampler.py:151-161; selective_log_softmax tunix/rl/common.py:187-203;
 * compute_chunked_logps :485-571.
 *   head weights: dense bf16 [V,D] (w_bf16 != NULL; also the tied embedding table), or QW
 *   part: fp32 workspace [M, n_vblocks, 4]; n_vblocks from tnx_lmhead_nblocks(V)
 *   logits_out (optional) receives the raw logits f32(bf16(x . W)): neither the temperature nor
 *   the forbidden mask is applied to it (the sampler's logits buffer, sampler.py:724-728)
 * ------------------------------------------------------------------------------------- */
typedef struct tnx_lmhead_desc {
  int64_t M, D, V;
  const uint16_t* x;          /* bf16 [M,D]                                                  */
  const uint16_t* w_bf16;     /* bf16 [V,D] or NULL                                          */
  const uint32_t* codes;      /* QW (K = D, N = V) when w_bf16 == NULL                       */
  const uint16_t* scales;
  int group, qtype;
  int lora_rank;
  const uint16_t* t;          /* bf16 [M, t_ld]                                              */
  int64_t t_ld;
  const uint16_t* lora_b;     /* bf16 [V, r]                                                 */
  float lora_scale;
  float temperature;          /* fp32 logits are divided by this (0 or 1.0 = no scaling)     */
  const int32_t* forbidden;   /* device list of ids forced to -inf, or NULL                  */
  int n_forbidden;
  const int32_t* targets;     /* int32 [M] or NULL                                           */
  float* part;
  int32_t* best_id;           /* int32 [M] or NULL                                           */
  float* best_logp;           /* fp32 [M]: log-softmax at best_id, or NULL                   */
  float* target_logp;         /* fp32 [M]: log-softmax at targets[m], or NULL                */
  float* lse;                 /* fp32 [M] or NULL                                            */
  float* logits_out;          /* fp32 [M,V] or NULL: materialise logits (return_logits /
                                 top-k sampling path)                                       */
  float* part_entropy;        /* fp32 workspace [M, n_vblocks], needed when entropy != NULL  */
  float* entropy;             /* fp32 [M] or NULL: -sum_v p_v log p_v of the (temperature-
                                 scaled) distribution, compute_entropy_from_logits
                                 tunix/rl/common.py:1136-1148                                */
  /* Optional whole-vocabulary categorical draw inside the head (draw_id != NULL): what
   * tnx_sample_topk does for top_p >= 1 without top_k (sample_top_p, sampler.py:119-121),
   * jax.random.categorical over logits / temperature with the noise of fold_in(key, *step),
   * without materialising the logits. */
  float* part_draw;           /* fp32 workspace [M, n_vblocks, 3]                            */
  uint32_t draw_key0, draw_key1;
  int draw_rng_variant;       /* as rng_variant of tnx_sample_topk                           */
  const int32_t* draw_step_ptr;
  int32_t* draw_id;           /* int32 [M]                                                   */
  float* draw_logp;           /* fp32 [M]: log-softmax at the drawn id, or NULL              */
  /* fp32-accumulate reference mode: != 0 keeps the fp32 accumulator as the logit instead of
   * rounding it to bf16 first (the reference's head is a bf16 einsum cast to fp32,
   * llama3/model.py:688-697; this mode is what that einsum would give with an fp32 result).
   * Inputs are what they are in the normal mode (bf16 x, weights dequantised to bf16, bf16 t);
   * every sum and the log-softmax run in fp32.  Log-probabilities then agree with an fp64
   * evaluation of the same bf16 operands to 1e-4 instead of to bf16 resolution. */
  int logits_fp32;
  const uint16_t* w_expanded; /* optional: tnx_qw_expand of (codes, scales), or
                                 tnx_dense_expand of w_bf16                                   */
} tnx_lmhead_desc;
int64_t tnx_lmhead_nblocks(int64_t V);
int tnx_lmhead_logp(void* stream, const tnx_lmhead_desc* h_desc);

/* Top-k / top-p sampling from materialised raw fp32 logits, which are divided by `temperature`
 * on the fly: sample_top_p tunix/generate/sampler.py:105-148.  `forbidden` ids (may be NULL) are
 * treated as -inf (:490-491).  The k largest logits per row (descending,
 * lower index first among equals) are softmaxed, entries whose exclusive cumulative
 * probability exceeds top_p are dropped, and one is drawn by Gumbel-max (jax.random.categorical)
 * with noise from threefry2x32 keyed by fold_in((key0,key1), *step_ptr) (sampler.py:516).
 * rng_variant selects jax's random_bits layout: 1 = partitionable (counter (0,n), x0^x1),
 * 0 = original (counter array split in halves).  k <= 0 (no top-k) with top_p >= 1 draws from
 * the whole vocabulary, noise indexed by vocabulary id (:118-121).  logp_out = full-vocabulary
 * log-softmax at the drawn id (:141-144).
 * 0 < k < V: k <= 1024.  With a workspace `ws` of tnx_sample_topk_ws_bytes(M, V, k) bytes (and
 * ceil(V / 8192) * k <= 4096, k <= 512) the row is processed in segments by many work-groups and a merging
 * launch; with ws = NULL one work-group per row does everything.  Both give the same result.
 * k <= 0 with top_p < 1, and k == V with any top_p, sort every row completely, as the reference
 * does with jax.lax.top_k(k = V) (:126-127), draw over SORTED positions, and need ws of
 * tnx_sample_fullsort_ws_bytes(M, V) bytes (two pairs of [M, V] key / id arrays for the library's
 * own stable radix sort; M * V < 2^31).  k > V returns TNX_EINVAL
 * (jax.lax.top_k raises). */
size_t tnx_sample_topk_ws_bytes(int64_t M, int64_t V, int k);
size_t tnx_sample_fullsort_ws_bytes(int64_t M, int64_t V);
int tnx_sample_topk(void* stream, const float* logits, int64_t M, int64_t V, int k, float top_p,
                    float temperature, uint32_t key0, uint32_t key1, int rng_variant,
                    const int32_t* forbidden, int n_forbidden, const int32_t* step_ptr, float* ws,
                    int32_t* ids_out, float* logp_out);

/* The same draw for 0 < k < V straight after a tnx_lmhead_logp call over the same rows, in one
 * launch that reads k x 128 logits per row instead of the row: the k best logits of a row lie in
 * the k blocks of 128 columns with the largest block maxima, which the head has left in its
 * workspace.  `logits` is that call's logits_out, `part` its workspace, `lse` its lse output
 * (needed when logp_out is given); the call must have used the same `temperature` and the same
 * `forbidden` list.  Ids are those of tnx_sample_topk on the same logits; logp_out is taken
 * against the head's log-sum-exp (the two sum the row's exponentials in different orders).
 * Shapes: tnx_sample_topk_head_ok(V, k) != 0, i.e. k <= 64 and V <= 524288; otherwise TNX_EINVAL
 * and the caller uses tnx_sample_topk.  No workspace. */
int tnx_sample_topk_head_ok(int64_t V, int k);
int tnx_sample_topk_head(void* stream, const float* logits, const float* part, const float* lse,
                         int64_t M, int64_t V, int k, float top_p, float temperature, uint32_t key0,
                         uint32_t key1, int rng_variant, const int32_t* forbidden, int n_forbidden,
                         const int32_t* step_ptr, int32_t* ids_out, float* logp_out);

/* Sampler bookkeeping of one step (tunix/generate/sampler.py:529-535, :692-703):
 *   col = *step_ptr; tokens[b, col+1] = ids[b]; logprobs[b, col+1] = logp[b] (if given);
 *   done[b] |= ids[b] in eos[];  then *step_ptr = col + 1 (by the last thread). */
int tnx_sample_commit(void* stream, const int32_t* ids, const float* logp, int64_t B,
                      int32_t* tokens, int64_t tok_ld, float* logprobs, int32_t* done,
                      const int32_t* eos, int n_eos, int32_t* step_ptr);

/* ---------------------------------------------------------------------------------------
 * MoE (qwen3/model.py:787-832): router softmax -> top-k -> renormalise (weights bf16), and an
 * int4/NF4 grouped GEMM over routed tokens (operator shape of megablox.gmm, :975-995).
 * ------------------------------------------------------------------------------------- */
/* scores: bf16 [M,E] router outputs.  topk_w: bf16 [M,k]; topk_id: int32 [M,k] (descending
 * probability, lower expert id first among equals).  A row with a NaN score still gets k distinct
 * ids inside [0,E) (so that the sort and the grouped GEMM stay in bounds) and NaN weights. */
int tnx_moe_route_topk(void* stream, const uint16_t* scores, int64_t M, int E, int k,
                       uint16_t* topk_w, int32_t* topk_id);
/* Builds the expert-sorted route list: counts[E], offsets[E+1], sorted_route[M*k] (route =
 * m*k + j).  Single work-group; M*k <= 1<<20. */
int tnx_moe_sort_routes(void* stream, const int32_t* topk_id, int64_t M, int k, int E,
                        int32_t* counts, int32_t* offsets, int32_t* sorted_route);
typedef struct tnx_moe_gmm_desc {
  int64_t n_routes;          /* M*k                                                          */
  int E, k;
  int64_t K, N;              /* per-expert linear: x[.,K] . W_e[K,N]                          */
  int group, qtype;
  const uint16_t* x;         /* bf16 rows; row of route r is r / x_div (x_div = k for the
                                token activations, 1 for per-route activations)             */
  int x_div;
  const uint32_t* codes;     /* QW per expert, expert stride = tnx_qw_sizes().codes_bytes    */
  const uint16_t* scales;
  const int32_t* offsets;    /* int32 [E+1]                                                  */
  const int32_t* sorted_route;
  int epilogue;              /* TNX_EPI_STORE or TNX_EPI_SILU_MUL (interleave2 packing)      */
  uint16_t* y;               /* bf16 [n_routes, N or N/2], indexed by route                  */
} tnx_moe_gmm_desc;
int tnx_moe_int4_gmm(void* stream, const tnx_moe_gmm_desc* h_desc);
/* out[m,:] = bf16( sum_j f32(topk_w[m,j]) * f32(y[m*k+j,:]) )  (qwen3/model.py:827-832). */
int tnx_moe_combine(void* stream, const uint16_t* y, const uint16_t* topk_w, int64_t M, int k,
                    int64_t D, const uint16_t* residual, uint16_t* out);

/* GRPO clipped ratio (tunix/rl/algo_core.py:440-489): lr = clip(logp - old, -20, 20);
 * ratio = exp(lr); loss = max(-A*ratio, -A*clip(ratio, 1-eps_lo, 1+eps_hi)).
 * adv has one value per sequence: adv[n / tokens_per_seq].  Outputs may be NULL. */
int tnx_grpo_ratio(void* stream, const float* logp, const float* old_logp, const float* adv,
                   int64_t N, int64_t tokens_per_seq, float eps_lo, float eps_hi, float* ratio,
                   float* loss, int32_t* clipped);

/* Per-token KL estimators between the trained and the reference policy
 * (tunix/rl/common.py:135-184): TNX_KL_KL logp - ref; TNX_KL_MSE 0.5 * (logp - ref)^2;
 * TNX_KL_LOW_VAR exp(d) - d - 1 with d = ref - logp.  clamp >= 0 clips the result to
 * [-clamp, clamp]; a negative clamp means none (the reference's clamp_value=None). */
enum { TNX_KL_KL = 0, TNX_KL_MSE = 1, TNX_KL_LOW_VAR = 2 };
int tnx_kl_divergence(void* stream, const float* logp, const float* ref_logp, int64_t N, int method,
                      float clamp, float* kl);

/* Loss aggregation without packing segments (tunix/rl/common.py:763-854, the per-row branch): out[0] = unreduced sum,
 * out[1] = denominator of the mode; the caller divides as WeightedMetric.compute does
 * (tunix/sft/utils.py:201-219).  per_token_loss, mask: fp32 [B, T]; row_ws: [B, 2] fp32 workspace
 * (per-row sum of loss * mask, per-row sum of mask).  norm: the `norm` keyword of the two modes
 * that take one (the caller passes the reference's default, T or B, when the keyword is absent).
 * Sums run in a fixed order: the result is the same on every launch. */
enum {
  TNX_AGG_TOKEN_MEAN = 0,              /* "token-mean" */
  TNX_AGG_SEQ_MEAN_TOKEN_MEAN = 1,     /* "sequence-mean-token-mean" */
  TNX_AGG_SEQ_MEAN_TOKEN_SCALE = 2,    /* "sequence-mean-token-scale" */
  TNX_AGG_SEQ_MEAN_TOKEN_SUM = 3,      /* "seq-mean-token-sum" */
  TNX_AGG_SEQ_MEAN_TOKEN_SUM_NORM = 4  /* "sequence-mean-token-sum-norm" */
};
int tnx_aggregate_loss(void* stream, const float* per_token_loss, const float* mask, int64_t B, int64_t T,
                       int mode, float norm, float* row_ws, float* out);

/* The same over packed batches (the segment branch, tunix/rl/common.py:857-940 with the segment
 * sums of :704-760): a row holds several sequences, segment_ids int32 [B, T] tells them apart
 * (0 = padding, ids outside [0, num_segments) belong to no segment), and the per-sequence modes
 * reduce per segment: a segment counts when it has at least one token with mask != 0, segment 0
 * never counts, the denominator is the number of counted segments.  "token-mean" and
 * "sequence-mean-token-sum-norm" sum over all tokens as without packing; norm <= 0 in the latter
 * selects the reference's default there, the number of counted segments.
 * "sequence-mean-token-scale" needs an explicit norm > 0.  ws: tnx_aggregate_loss_segmented_ws_bytes
 * bytes.  Every sum runs in a fixed order. */
size_t tnx_aggregate_loss_segmented_ws_bytes(int64_t B, int num_segments);
int tnx_aggregate_loss_segmented(void* stream, const float* per_token_loss, const float* mask,
                                 const int32_t* segment_ids, int64_t B, int64_t T, int num_segments,
                                 int mode, float norm, float* ws, float* out);

/* Agreement between the log-probabilities the rollout recorded and the ones the trainer
 * recomputes for the same tokens (tunix/rl/grpo/grpo_learner.py:405-440), over the positions
 * where mask != 0.  rollout_logp, trainer_logp, mask: fp32 [B, T].  out5 = { mean |dlogp|,
 * max |dlogp|, mean |dp|, max |dp|, Pearson correlation of the probabilities } with
 * p = exp(logp), means over max(mask count, 1), correlation = cov / sqrt(max(var_r * var_t, 1e-12)).
 * ws: tnx_logp_drift_ws_bytes(B) bytes, 8-byte aligned.  The moments are accumulated in double. */
size_t tnx_logp_drift_ws_bytes(int64_t B);
int tnx_logp_drift(void* stream, const float* rollout_logp, const float* trainer_logp, const float* mask,
                   int64_t B, int64_t T, void* ws, float* out5);

/* tnx_logp_drift for callers that cannot allocate device memory (code under HIP-graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): no counterpart in the reference.  Same
 * arguments and results as tnx_logp_drift without the workspace: the per-row moments go to an
 * array built into the library (tnx_logp_drift_static_max_rows() = 4096 rows, 320 KiB, one copy
 * per GPU for the life of the process).  B above that limit returns TNX_EINVAL.  The call
 * allocates and frees nothing; its first call on a device looks the array's address up
 * (hipGetSymbolAddress), so make that call outside a capture.  Every call on one GPU shares
 * that GPU's array: calls that overlap on one GPU (different streams, no ordering) race. */
int64_t tnx_logp_drift_static_max_rows(void);
int tnx_logp_drift_static(void* stream, const float* rollout_logp, const float* trainer_logp,
                          const float* mask, int64_t B, int64_t T, float* out5);

/* Fill n 32-bit words with `value` (graph-capturable replacement for hipMemsetAsync). */
int tnx_fill_u32(void* stream, uint32_t* p, int64_t n, uint32_t value);

#ifdef __cplusplus
}
#endif
#endif /* TUNIX_HIP_H_ */
