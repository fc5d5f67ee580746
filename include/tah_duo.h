/* tah_duo.h -- C ABI of the MI355X (gfx950) duo-causal attention library.
 *
 * The reference (thu-nics/TaH) has no FFI on this path: it expresses duo-causal
 * attention as a dense additive mask + a concatenating Python KV cache + Hugging
 * Face SDPA.  Each entry point below names the reference code whose device work
 * it replaces.  All pointers are device pointers unless stated otherwise; all
 * functions enqueue on `stream`, never allocate, never synchronise, keep no
 * global state and return 0 or a negative TAH_E_* code (never throw).
 *
 * Layout.  Tokens are packed ("varlen"): sequence b owns rows
 * [cu[b], cu[b+1]) of a [rows, heads, D] bf16 tensor whose innermost D elements
 * are contiguous; row and head strides are given in elements.  Only valid tokens
 * are packed, so within a sequence the depth-0 ("iteration 1") key at local
 * index j has position j, and a depth-0 query at local index i has position
 * i + (Lk1 - Lq1) (queries are the newest rows of the sequence).  Depth-1
 * ("iteration 2") rows exist only for hard tokens and carry their position
 * explicitly (pos_q2 / pos_k2, int32).  Inside a sequence the depth-1 query rows
 * come in ascending position (pos_q2 non-decreasing between cu_q2[b] and
 * cu_q2[b+1]), the order in which gather_active packs hard tokens
 * (tah/model/tah_model.py:114-117): the backward pass skips depth-1 query tiles
 * by the position of their last row.
 *
 * Visibility (tah/model/tah_model.py:788): key (pos_k, depth_k) is visible to
 * query (pos_q, depth_q) iff pos_k <= pos_q and depth_k <= depth_q.  The two
 * streams are what that rule needs for any depth: queries at depth d >= 2 go
 * where depth-1 queries go, with the keys of depths 1 .. d together as their
 * position-carrying key stream (rows of a sequence in any order; all of them
 * satisfy depth_k <= depth_q).
 * GQA: query head h reads kv head h / (Hq / Hkv)
 * (transformers/integrations/sdpa_attention.py:15-24, repeat_kv).
 */
#ifndef TAH_DUO_H
#define TAH_DUO_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TAH_DUO_ABI_VERSION 7

enum {
    TAH_OK = 0,
    TAH_E_NULL = -1,      /* a required pointer is NULL */
    TAH_E_SHAPE = -2,     /* unsupported head_dim / head counts / negative sizes */
    TAH_E_ALIGN = -3,     /* pointer or stride not 16-byte aligned */
    TAH_E_LAUNCH = -4,    /* the HIP runtime rejected the launch */
    TAH_E_WORKSPACE = -5, /* workspace too small */
    TAH_E_SCRATCH = -6    /* tah_duo_decode_static: the call needs more than TAH_DUO_STATIC_SCRATCH_BYTES */
};

typedef void* tah_stream_t; /* hipStream_t */

/* One query stream + its key/value segment at one depth. */
typedef struct tah_duo_stream {
    const void* q;          /* bf16 [total_q, Hq,  D] */
    const void* k;          /* bf16 [total_k, Hkv, D] */
    const void* v;          /* bf16 [total_k, Hkv, D] */
    void* o;                /* bf16 [total_q, Hq,  D]  (forward output) */
    float* lse;             /* f32  [Hq, total_q] natural-log normaliser (forward output) */
    const int32_t* cu_q;    /* int32 [nseq+1] */
    const int32_t* cu_k;    /* int32 [nseq+1] */
    const int32_t* pos_q;   /* int32 [total_q]; NULL at depth 0 (implicit positions) */
    const int32_t* pos_k;   /* int32 [total_k]; NULL at depth 0 */
    int64_t q_row_stride, q_head_stride;
    int64_t k_row_stride, k_head_stride;
    int64_t v_row_stride, v_head_stride;
    int64_t o_row_stride, o_head_stride;
    int32_t total_q, total_k;
} tah_duo_stream;

typedef struct tah_duo_fwd_args {
    tah_duo_stream s1;      /* depth 0: every token */
    tah_duo_stream s2;      /* depth 1: hard tokens; total_q may be 0 */
    int32_t nseq, hq, hkv, d;
    float scale;            /* softmax scale, head_dim**-0.5 in Qwen3 */
    const void* schedule;   /* launch-order table from tah_duo_schedule_build for these boundaries, or NULL */
} tah_duo_fwd_args;

int tah_duo_abi_version(void);
const char* tah_duo_error_string(int code);

/* Prefill / training forward of duo-causal attention.
 * Replaces, per decoder layer and for both depths at once:
 *   TaHForCausalLM._build_attention_mask        tah/model/tah_model.py:744-791
 *   TaHCache.update / get_cache_upto_iter (cat)  tah/model/causal_cache.py:63-109
 *   sdpa_attention_forward (repeat_kv + SDPA)    transformers/integrations/sdpa_attention.py:79-166
 * Depth-0 queries attend to depth-0 keys; depth-1 queries attend to depth-0
 * keys and depth-1 keys, both cut at the query's position.  `args` is a host
 * pointer and is read before the call returns.  Rows with no visible key get
 * o = 0, lse = -inf. */
int tah_duo_fwd_varlen(const tah_duo_fwd_args* args, tah_stream_t stream);

/* Launch order of a varlen call's tiles, heaviest first (optional).  The kernels start one workgroup per
 * (kv head, 128-row tile); with several documents of unequal length in a batch, handing the tiles out in
 * sequence order leaves the long tiles of later documents for the end of the launch.  This call sorts the
 * tiles of both depths by the work they will do, on the device, from the same boundary arrays the
 * attention calls take; pass the table as `schedule` to tah_duo_fwd_varlen / tah_duo_bwd_varlen as long as
 * nseq, the totals, hq / hkv and the contents of cu_* and pos_q2 stay what they were when it was built
 * (one table serves every layer and the backward pass of a batch).  A table whose sizes (nseq, the totals,
 * hq / hkv) differ from a call's is ignored by that call.  The table is a permutation of the tile numbers, which
 * the kernels turn into tiles from the call's own boundaries: it changes the order in which tiles are started,
 * never a result -- one built for other boundaries of the same sizes still makes a call visit each of its tiles
 * once, only no longer heaviest first (build a new one when cu_* change: one small launch, 0.015 ms for the four
 * sequences of a 16 384-token batch).  Tiles of equal weight are listed in no particular order, which can differ
 * between two builds.
 * No counterpart in the reference, whose SDPA call launches a dense rectangular problem
 * (transformers/integrations/sdpa_attention.py:79-166). */
typedef struct tah_duo_schedule_args {
    const int32_t* cu_q1;   /* int32 [nseq+1] depth-0 query boundaries */
    const int32_t* cu_k1;   /* int32 [nseq+1] depth-0 key boundaries */
    const int32_t* cu_q2;   /* depth 1; may be NULL when total_q2 == 0 */
    const int32_t* cu_k2;   /* may be NULL when total_k2 == 0 */
    const int32_t* pos_q2;  /* int32 [total_q2] positions of the depth-1 query rows */
    int32_t nseq, hq, hkv;  /* nseq <= 4095 */
    int32_t total_q1, total_k1, total_q2, total_k2;
    void* schedule;         /* >= tah_duo_schedule_bytes(...) bytes, 4-byte aligned */
    size_t schedule_bytes;
} tah_duo_schedule_args;

size_t tah_duo_schedule_bytes(int32_t nseq, int32_t hq, int32_t hkv, int32_t total_q1, int32_t total_k1,
                              int32_t total_q2, int32_t total_k2);
int tah_duo_schedule_build(const tah_duo_schedule_args* args, tah_stream_t stream);

/* A dense additive attention mask as Hugging Face passes it: element
 * [seq b][head h][query i][key j], i and j counted inside sequence b (row
 * cu_q[b] + i, key row cu_k[b] + j), strides in elements (head_stride 0 for the
 * usual (B,1,Tq,Tkv) mask). */
typedef struct tah_additive_mask {
    const void* mask;
    int64_t seq_stride, head_stride, q_stride, k_stride;
    int32_t dtype; /* 0: bf16, 1: float */
} tah_additive_mask;

/* Compatibility mode: softmax(q k^T * scale + mask) v with an explicit additive
 * mask, exactly the arithmetic the reference runs today
 *   TaHForCausalLM._build_attention_mask (the mask)  tah/model/tah_model.py:744-791
 *   sdpa_attention_forward (repeat_kv + SDPA)         transformers/integrations/sdpa_attention.py:79-166
 * for callers that still build the (B,1,Tq,Tkv) mask.  Only stream s1 of `args`
 * is used (s2 must be empty); every query sees every key of its sequence and the
 * mask alone decides.  Entries of finfo.min or -inf hide a key; a row whose keys
 * are all hidden gets o = 0, lse = -inf.  The mask is read once per (head, tile):
 * O(Tq*Tkv) traffic that the duo-causal entry point avoids. */
int tah_duo_fwd_masked(const tah_duo_fwd_args* args, const tah_additive_mask* mask, tah_stream_t stream);

/* Gradient tensors of one stream (same row/head layout as the forward tensors). */
typedef struct tah_duo_bwd_stream {
    const void* d_o;        /* bf16 [total_q, Hq,  D] upstream gradient of o */
    void* dq;               /* bf16 [total_q, Hq,  D] */
    void* dk;               /* bf16 [total_k, Hkv, D] */
    void* dv;               /* bf16 [total_k, Hkv, D] */
    float* delta;           /* f32  [2, Hq, total_q] scratch written by the call: rowsum(dO*O), then lse * log2(e) */
    int64_t do_row_stride, do_head_stride;
    int64_t dq_row_stride, dq_head_stride;
    int64_t dk_row_stride, dk_head_stride;
    int64_t dv_row_stride, dv_head_stride;
} tah_duo_bwd_stream;

typedef struct tah_duo_bwd_args {
    tah_duo_fwd_args fwd;   /* the forward call's tensors; o and lse are inputs here */
    tah_duo_bwd_stream g1;  /* depth 0 */
    tah_duo_bwd_stream g2;  /* depth 1 */
    void* ds_workspace;         /* NULL, or >= tah_duo_bwd_workspace_bytes(...) bytes, 16-byte aligned; contents need no
                                 * initialisation and mean nothing after the call */
    size_t ds_workspace_bytes;
    int32_t max_seqlen_k1;      /* upper bound on one sequence's depth-0 key rows, 0: unknown (total_k is used) */
    int32_t max_seqlen_k2;      /* same for depth 1 */
} tah_duo_bwd_args;

/* Backward of tah_duo_fwd_varlen: dQ, dK, dV of both depths.  Replaces torch
 * autograd through SDPA + torch.cat + repeat_kv on this path; the reference
 * keeps cached K/V attached to the graph (tah/model/causal_cache.py:92-93), so
 * depth-0 dK/dV collect the contributions of depth-0 and depth-1 queries, summed
 * over the query heads of each kv head.  Deterministic (no atomics).
 *
 * Without `ds_workspace`: three kernels, dQ and dK/dV each recompute the scores (7 matrix products per
 * visible (query tile, key tile) pair).  With it (hq / hkv <= 4): the dK/dV kernel also writes
 * dS = P o (dP - delta) in bf16, one 16 KiB block per (64 query rows, head, 128 keys), and dQ = scale * dS K
 * reads it back (5 products per pair; the workspace is written and read once).  Both give the same dK / dV
 * to the bit; dQ then uses the dS the dK product uses.  The bound the size function returns covers every
 * (64-row query tile, 128-key tile) pair of the call: about total_q * max_seqlen_k * hq * 2 bytes. */
int tah_duo_bwd_varlen(const tah_duo_bwd_args* args, tah_stream_t stream);
size_t tah_duo_bwd_workspace_bytes(int32_t nseq, int32_t hq, int32_t hkv, int32_t total_q1, int32_t total_k1,
                                   int32_t total_q2, int32_t total_k2, int32_t max_seqlen_k1, int32_t max_seqlen_k2);

/* Backward of tah_duo_fwd_masked (same additive mask; no gradient is formed for
 * the mask itself, which the reference builds from integers).  Replaces torch
 * autograd through sdpa_attention_forward with attn_mask
 * (transformers/integrations/sdpa_attention.py:79-166). */
int tah_duo_bwd_masked(const tah_duo_bwd_args* args, const tah_additive_mask* mask, tah_stream_t stream);

/* One depth of the native KV cache of one decoder layer.  Each sequence slot s
 * owns a slab: row j of kv head h lives at
 *   base + (start[s] + j) * row_stride + h * head_stride      (elements, D contiguous)
 * which covers both token-major [rows, Hkv, D] slabs and the head-major
 * [slot, Hkv, capacity, D] layout the decode kernel streams best.  len[s] rows
 * are in use.  Depth 0 holds every token of the sequence in position order
 * (position of row j is j); depth 1 holds hard tokens only, with pos[] giving
 * each row's position.
 * Replaces the per-(layer, depth) tensors of TaHCache (tah/model/causal_cache.py:43-48). */
typedef struct tah_kv_segment {
    void* k;                 /* bf16 */
    void* v;                 /* bf16 */
    int32_t* pos;            /* int32 [nslots * capacity], row j of slot s at pos[s*capacity + j]; NULL at depth 0 */
    const int32_t* start;    /* int32 [nslots] first row of each slab, in rows of row_stride */
    int32_t* len;            /* int32 [nslots] rows in use */
    int64_t k_row_stride, k_head_stride, v_row_stride, v_head_stride;
    int32_t capacity;        /* rows per slab; also the upper bound on len[] used to size grids */
    int32_t nslots;
} tah_kv_segment;

typedef struct tah_duo_decode_args {
    const void* q;           /* bf16 [nq, Hq, D]: one query row per (sequence, depth) being decoded */
    void* o;                 /* bf16 [nq, Hq, D] */
    float* lse;              /* f32 [nq, Hq] natural-log normaliser, may be NULL */
    int64_t q_row_stride, q_head_stride, o_row_stride, o_head_stride;
    const int32_t* q_slot;   /* int32 [nq] cache slot of each query's sequence; negative: no sequence (nothing is read
                              * for the query, its output row is zeros) */
    const int32_t* q_pos;    /* int32 [nq] position of each query */
    const int32_t* q_depth;  /* int32 [nq] 0 or 1; NULL: every query is at `depth` */
    int32_t depth;
    tah_kv_segment c1;       /* depth-0 cache, already holding the new token's K/V */
    tah_kv_segment c2;       /* depth-1 cache; only read by depth-1 queries */
    void* workspace;         /* >= tah_duo_decode_workspace_bytes(...) bytes, 16-byte aligned */
    size_t workspace_bytes;
    int32_t nq, hq, hkv, d;
    float scale;
    void* o_packed;          /* NULL, or bf16 [hq * d * 32]: the output once more as the rows operand of tah_linear_rows
                              * (the o projection that follows), nq <= 32; rows nq .. 31 are left as they are */
} tah_duo_decode_args;

/* Bytes of split-K scratch tah_duo_decode needs for nq queries. */
size_t tah_duo_decode_workspace_bytes(int32_t nq, int32_t hq, int32_t capacity1, int32_t capacity2);

/* Decode step of duo-causal attention against the KV cache: every query row
 * attends to the depth-0 rows of its sequence with index <= q_pos, and, if it
 * is a depth-1 query, to the depth-1 rows with pos <= q_pos.  Split-K over
 * chunks of both segments (1024 rows; 256 rows when nq * hq * chunks is too small to fill the chip), then a
 * merge kernel.
 * Calls that share a workspace must be ordered on one stream.  Replaces, for Tq == 1:
 *   TaHForCausalLM._build_attention_mask        tah/model/tah_model.py:744-791
 *   TaHCache.get_cache_upto_iter (cat it1|it2)   tah/model/causal_cache.py:101-109
 *   sdpa_attention_forward                       transformers/integrations/sdpa_attention.py:79-166
 * Queries with no visible row get o = 0, lse = -inf. */
int tah_duo_decode(const tah_duo_decode_args* args, tah_stream_t stream);

/* Split-K scratch held inside the library for tah_duo_decode_static, per GPU. */
#define TAH_DUO_STATIC_SCRATCH_BYTES (16u << 20)

/* tah_duo_decode for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): same arguments, same kernels and same results, but the
 * split-K partials go to a buffer of TAH_DUO_STATIC_SCRATCH_BYTES that the library itself holds on each GPU
 * (`workspace` / `workspace_bytes` are ignored).  It has no counterpart in the reference.  Calls needing
 * more than that -- tah_duo_decode_workspace_bytes(nq, hq, capacity1, capacity2) bytes, e.g. nq * hq *
 * (chunks of 1024 or 256 rows over both capacities) * 520 -- return TAH_E_SCRATCH and launch nothing.  It calls no
 * hipMalloc / hipFree; the first call on a device looks the buffer's address up once.  All calls on one
 * GPU share the buffer (nothing in it needs clearing between calls): two calls that overlap in time on
 * one GPU -- different streams, or graphs replayed concurrently -- race. */
int tah_duo_decode_static(const tah_duo_decode_args* args, tah_stream_t stream);

typedef struct tah_kv_append_args {
    const void* k_new;       /* bf16 [total_new, Hkv, D] */
    const void* v_new;
    const int32_t* pos_new;  /* int32 [total_new] or NULL (depth 0) */
    int64_t k_row_stride, k_head_stride, v_row_stride, v_head_stride;
    const int32_t* cu_new;   /* int32 [nseq+1]: rows [cu_new[i], cu_new[i+1]) go to slot slot_of[i] */
    const int32_t* slot_of;  /* int32 [nseq] or NULL (slot i); a negative entry: that sequence's rows are skipped */
    int32_t nseq, total_new, hkv, d;
    tah_kv_segment cache;    /* destination; len[] is advanced by the number of rows appended */
    int32_t* overflow;       /* optional device flag, set to 1 if a slab would exceed capacity (rows dropped) */
} tah_kv_append_args;

/* In-place append of new K/V rows (and positions) to the per-sequence slabs.
 * Replaces the torch.cat growth of TaHCache.update (tah/model/causal_cache.py:84-95). */
int tah_kv_append(const tah_kv_append_args* args, tah_stream_t stream);

typedef struct tah_qk_prep_args {
    const void* q;           /* bf16 [rows, Hq, D]  projected queries, one row per token */
    const void* k;           /* bf16 [rows, Hkv, D] */
    const void* v;           /* bf16 [rows, Hkv, D]; may be NULL when V is neither copied nor appended */
    void* q_out;             /* bf16 [rows, Hq, D]; may alias q */
    void* k_out;             /* bf16 [rows, Hkv, D]; may alias k; unused with append */
    void* v_out;             /* optional copy of v; unused with append */
    int64_t q_row_stride, q_head_stride, k_row_stride, k_head_stride, v_row_stride, v_head_stride;
    int64_t q_out_row_stride, q_out_head_stride, k_out_row_stride, k_out_head_stride, v_out_row_stride, v_out_head_stride;
    const void* q_weight;    /* bf16 [D] RMSNorm weight of the query heads */
    const void* k_weight;    /* bf16 [D] */
    const void* cos;         /* bf16 [rows, D] rotary cosines of each token's position */
    const void* sin;         /* bf16 [rows, D] */
    int64_t cos_sin_row_stride;
    float eps;               /* RMSNorm epsilon */
    int32_t rows, hq, hkv, d;
    /* append != 0: K (after norm and rotation) and V go to the slabs of `cache`, rows
     * [cu_new[i], cu_new[i+1]) to slot slot_of[i], and len[] advances, as in tah_kv_append */
    int32_t append;
    const int32_t* cu_new;   /* int32 [nseq+1] */
    const int32_t* slot_of;  /* int32 [nseq] or NULL (slot i); a negative entry: q is prepared, K/V of those rows are not cached */
    const int32_t* pos_new;  /* int32 [rows] or NULL (depth 0) */
    int32_t nseq;
    tah_kv_segment cache;
    int32_t* overflow;       /* optional device flag, as in tah_kv_append */
    /* != 0: the caller promises that every sequence brings at most one row and that the slots named are all
     * different (a decode step): the lengths are then advanced by the same launch instead of a second one */
    int32_t append_one_row_per_seq;
    /* Optional: the layer's input RMSNorm folded in.  With `norm_input` set, q, k and v are projections of the
     * un-normalised rows norm_input[rows, norm_cols] through weights that already carry the norm's weight
     * (W' = W diag(g)), and every head is first multiplied by the row's rsqrt(mean(norm_input[row]^2) + norm_eps):
     * the norm needs no launch of its own (Qwen3DecoderLayer.forward: input_layernorm, then q|k|v projections).
     * V is then scaled as well (to v_out, or on its way into the slabs).  norm_cols % 8 == 0. */
    const void* norm_input;
    int64_t norm_input_row_stride;
    int32_t norm_cols;
    float norm_eps;
} tah_qk_prep_args;

/* Per-head RMSNorm of q and k, rotary embedding of both, and optionally the KV-cache append,
 * in one pass over the token rows; each arithmetic step rounds to bf16 where the reference's
 * eager bf16 modules do.  Replaces, between the projections and the attention call of
 *   Qwen3Attention.forward        transformers/models/qwen3/modeling_qwen3.py (q_norm, k_norm,
 *                                 apply_rotary_pos_emb; third party, pinned 4.52.4 by the reference)
 *   TaHCache.update               tah/model/causal_cache.py:63-97 (with append)
 * head_dim 128 only.  In-place use (q_out == q, k_out == k) is allowed. */
int tah_qk_prep(const tah_qk_prep_args* args, tah_stream_t stream);

typedef struct tah_qk_prep_bwd_args {
    const void* q;           /* bf16 [rows, Hq, D]: what tah_qk_prep was given */
    const void* k;           /* bf16 [rows, Hkv, D] */
    const void* dq_out;      /* bf16 [rows, Hq, D]: gradient of tah_qk_prep's q_out */
    const void* dk_out;      /* bf16 [rows, Hkv, D]: gradient of its k_out */
    void* dq;                /* bf16 [rows, Hq, D]: gradient of q; may alias dq_out */
    void* dk;                /* bf16 [rows, Hkv, D]; may alias dk_out */
    int64_t q_row_stride, q_head_stride, k_row_stride, k_head_stride;
    int64_t dq_out_row_stride, dq_out_head_stride, dk_out_row_stride, dk_out_head_stride;
    int64_t dq_row_stride, dq_head_stride, dk_row_stride, dk_head_stride;
    const void* q_weight;    /* bf16 [D] */
    const void* k_weight;    /* bf16 [D] */
    const void* cos;         /* bf16 [rows, D] */
    const void* sin;         /* bf16 [rows, D] */
    int64_t cos_sin_row_stride;
    float eps;
    int32_t rows, hq, hkv, d;
    /* float32 [n_partial, 2, D]: row i holds the sums, over the token rows i, i + n_partial, ... and over the heads, of
     * the gradients of q_weight ([i, 0, :]) and k_weight ([i, 1, :]); every row is written (zeros when n_partial > rows).
     * The caller adds the rows up (a fixed order: results do not vary from run to run). */
    float* dw_partial;
    int32_t n_partial;       /* workgroups to launch, >= 1; a few per compute unit is enough */
} tah_qk_prep_bwd_args;

/* Backward of tah_qk_prep without append and without a folded input norm: gradients of the projected q and k and of
 * the two RMSNorm weights, given the gradients of the prepared q and k (V passes through tah_qk_prep unchanged, so
 * its gradient is the caller's already).  Differentiates Qwen3RMSNorm.forward and apply_rotary_pos_emb
 * (transformers/models/qwen3/modeling_qwen3.py; third party, pinned 4.52.4 by the reference) in float32 on the bf16
 * inputs.  head_dim 128 only. */
int tah_qk_prep_bwd(const tah_qk_prep_bwd_args* args, tah_stream_t stream);

typedef struct tah_topk_mix_args {
    const void* logits;        /* bf16 [rows, vocab], vocab contiguous */
    const void* embedding;     /* bf16 [vocab, hidden], 16-byte aligned rows */
    void* out;                 /* bf16 [rows, hidden] */
    const uint8_t* row_enable; /* optional, one byte per row: rows whose byte is 0 are skipped (out untouched, or zeroed) */
    int64_t logits_row_stride, embedding_row_stride, out_row_stride; /* elements */
    int32_t rows, vocab, hidden, topk; /* topk <= 256, vocab <= 155648, hidden a multiple of 8 */
    void* out_packed;          /* optional: the rows once more as the rows operand of tah_linear_rows, bf16 [32 * hidden]
                                * (rows <= 32, hidden % 32 == 0; rows past `rows` are not touched) */
    int32_t zero_disabled;     /* != 0: rows whose row_enable byte is 0 are written as zeros instead of left alone */
    /* Optional: the row's top-k logits themselves, largest first: bf16 [rows, min(topk, vocab)], what
     * torch.topk(logits, topk).values holds (equal values make the choice among ties invisible here).  The input of
     * MLPIterDecider's logits_projection (tah/model/iter_decider.py:281).  With values_out set, `out` may be NULL:
     * then only the values are produced (`embedding`, `hidden` are not used). */
    void* values_out;
    int64_t values_row_stride; /* elements */
    /* Optional, with values_out: the vocabulary index of each of those values, int32 [rows, values_row_stride]; equal
     * values in ascending index order (among equal values at the k-th place the lower indices are the ones taken). */
    int32_t* indices_out;
} tah_topk_mix_args;

/* Next-iteration input of hard tokens: softmax over each row's top-k logits, then the probability-weighted
 * sum of the corresponding embedding rows.  Replaces topk_softmax_input_update (tah/model/tah_model.py:57-75:
 * torch.topk + softmax + gather of (rows, k, hidden) embedding rows + sum) with one pass per row and no
 * (rows, k, hidden) intermediate.  Among equal logits at the k-th place the lower vocabulary indices are
 * taken (torch.topk leaves that choice open).  Probabilities and products round to bf16 where the bf16
 * eager arithmetic rounds; sums are float32 in index order, so results do not vary from run to run. */
int tah_topk_mix(const tah_topk_mix_args* args, tah_stream_t stream);

typedef struct tah_sample_rows_args {
    const void* logits;        /* bf16 [rows, vocab], vocab contiguous */
    const void* logits_prev;   /* optional bf16 [rows, vocab]: see add_prev */
    const int32_t* add_prev;   /* optional int32 [rows]: a row whose entry is not 0 draws from logits_prev + logits, the sum
                                * rounded to bf16 (the final logits of a token that took a second latent iteration) */
    const uint8_t* row_enable; /* optional, one byte per row: rows whose byte is 0 are skipped (outputs untouched) */
    const float* uniforms;     /* float32 [rows], each in [0, 1): the caller's random numbers, one per row and call */
    int64_t* tokens;           /* optional int64 [rows]: the drawn vocabulary index */
    float* probs;              /* optional float32 [rows, probs_row_stride]: the distribution drawn from (0 outside the filters) */
    int64_t logits_row_stride, prev_row_stride, probs_row_stride; /* elements */
    int32_t rows, vocab;       /* vocab <= 155648 */
    float temperature;         /* > 0 */
    float top_p;               /* in (0, 1]; 1: no filter */
    float min_p;               /* in [0, 1]; 0: no filter */
} tah_sample_rows_args;

/* One token per row by temperature sampling with the min_p and top_p filters, in one launch and without a sort over
 * the vocabulary.  Replaces sample_next_token (tah/model/utils.py:84-125) for do_sample=True and top_k == 0:
 * softmax(logits / temperature); tokens below min_p times the largest probability dropped, renormalised; tokens
 * dropped once the probability mass before them, in descending order, exceeds top_p, renormalised; one draw.  Tokens
 * of equal probability are ordered by vocabulary index, lower first (a stable descending sort; torch.sort leaves it
 * open).  The draw is the inverse-CDF draw over that same order with the caller's uniform number u: the first token
 * at which the kept mass passes u times the kept total (torch.multinomial draws from the same distribution with its
 * own generator).  Sums are float32; the row maximum must be finite.  `probs`, when given, receives the filtered and
 * renormalised distribution itself. */
int tah_sample_rows(const tah_sample_rows_args* args, tah_stream_t stream);

/* tah_qk_prep (append, one row per sequence) and tah_duo_decode in one launch, for a generation step: the workgroup
 * of a (query, kv head) prepares its query heads and the new K and V itself, stores K and V into the slabs and attends
 * over the cached rows and the new one.  `prep` and `dec` mean what they mean for the two calls (prep->q_out / k_out,
 * dec->q and the workspace are not used; prep->cache must be dec->c1 or dec->c2; row i of prep is query i of dec and
 * prep->slot_of[i], where not negative, is dec->q_slot[i]); cache contents and lengths are bit for bit those of the
 * two calls, the outputs too up to the last bit of a rare element (the same arithmetic in the same order, compiled
 * twice).  append_at: int32 [rows], the number of rows sequence i's segment of prep->cache holds before the
 * call, i.e. cache.len[slot] -- handed in because the workgroups of a sequence cannot read the length while one of
 * them advances it (len[slot] becomes append_at[i] + 1; a row whose append_at differs from the length sets
 * *prep->overflow to 2 where that flag is given: the slab then has a gap or an overwritten row; one query row per
 * slot and call).  Only for calls tah_duo_decode_step_supported() accepts (256
 * or more (query, kv head) pairs, slabs of at most 4096 rows, one or two query heads per kv head: cases
 * tah_duo_decode runs without split-K); others return TAH_E_SHAPE and the caller makes the two calls.  append_depth: NULL,
 * or int32 [rows], 0 / 1 per row: the segment (dec->c1 / dec->c2) that row's K and V go to, for a batch whose rows are at
 * different latent iterations (append_at[i] then counts the rows of that segment, and prep->cache only has to be one of
 * the two).  Replaces, with
 * tah_qk_prep's and tah_duo_decode's lists, one more launch per layer and latent iteration. */
int tah_duo_decode_step_supported(int32_t nq, int32_t hq, int32_t hkv, int32_t capacity1);
int tah_duo_decode_step(const tah_qk_prep_args* prep, const tah_duo_decode_args* dec, const int32_t* append_at,
                        const int32_t* append_depth, tah_stream_t stream);

/* Gate of the Qwen3 MLP for a decode step: out[r][i] = silu(gate_up[r][i]) * gate_up[r][inter + i], both
 * steps rounded to bf16 as the eager modules round them -- `act_fn(gate_proj(x)) * up_proj(x)` of Qwen3MLP.forward
 * (transformers/models/qwen3/modeling_qwen3.py, third party; the layer the reference's base model runs,
 * tah/model/tah_model.py:616-623) on the output of one fused gate|up projection.  One launch instead of two. */
int tah_silu_mul(const void* gate_up, void* out, int32_t rows, int32_t inter, int64_t gate_up_row_stride,
                 int64_t out_row_stride, tah_stream_t stream);
/* The same with the MLP's input RMSNorm folded in (post_attention_layernorm, then gate|up projections): gate_up is the
 * projection of the un-normalised rows norm_input[rows, norm_cols] through a weight that carries the norm's weight;
 * gate and up are multiplied by the row's rsqrt(mean(norm_input[row]^2) + norm_eps) before the gate. */
int tah_silu_mul_normed(const void* gate_up, void* out, int32_t rows, int32_t inter, int64_t gate_up_row_stride,
                        int64_t out_row_stride, const void* norm_input, int64_t norm_input_row_stride, int32_t norm_cols,
                        float norm_eps, tah_stream_t stream);

/* Linear layers of a decode step: at most 32 rows (one token per sequence) against a weight of megabytes.  The work
 * is streaming the weight once, so weight and rows are kept in the order the kernel reads them:
 *   packed weight  tiles of 16 output columns x 32 k, the 64 16-byte operands of the lanes of one
 *                  v_mfma_f32_16x16x32_bf16 step next to each other, a tile's k steps one after another;
 *                  n * k elements (2 n * k for TAH_LINEAR_GATE_UP), made once by tah_linear_pack_weight;
 *   packed rows    bf16 [k / 32][2][64][8]: unit (step, half, lane) holds row 16 half + lane % 16, columns
 *                  32 step + 8 (lane / 16) ... + 8; always 32 rows, the rows past `rows` are zero.  Made by
 *                  tah_linear_pack_rows, by tah_linear_rows (out_packed) and by tah_duo_decode (o_packed).
 * Replaces, for the rows of a decode step, in Qwen3DecoderLayer.forward / Qwen3Attention.forward / Qwen3MLP.forward
 * of the base model the reference runs (transformers/models/qwen3/modeling_qwen3.py, third party;
 * tah/model/tah_model.py:616-623): the q|k|v projections, o_proj + residual add, gate|up projections +
 * act_fn(gate) * up, down_proj + residual add.  Products accumulate in float32 in a fixed order (results do not
 * vary from run to run) and are rounded to bf16 where the eager modules round. */
enum { TAH_LINEAR_PLAIN = 0, TAH_LINEAR_GATE_UP = 1 };
enum { TAH_ACT_NONE = 0, TAH_ACT_RELU = 1, TAH_ACT_GELU = 2 };      /* GELU: x Phi(x), nn.GELU's default */
enum { TAH_NORM_NONE = 0, TAH_NORM_RMS = 1, TAH_NORM_LAYER = 2 };

/* w bf16 [n, k] row-major (nn.Linear weight), or [2 n, k] = [gate; up] stacked for TAH_LINEAR_GATE_UP; k % 32 == 0,
 * n % 16 == 0 (gate|up: n % 24 == 0 or n % 16 == 0).  packed: n * k (2 n * k) elements, 16-byte aligned. */
int tah_linear_pack_weight(const void* w, int64_t w_row_stride, void* packed, int32_t n, int32_t k, int32_t kind,
                           tah_stream_t stream);
/* x bf16 [rows, k] row-major, rows <= 32 -> x_packed bf16 [32 * k] (rows past `rows` zero). */
int tah_linear_pack_rows(const void* x, int64_t x_row_stride, void* x_packed, int32_t rows, int32_t k, tah_stream_t stream);

typedef struct tah_linear_rows_args {
    const void* w_packed;     /* from tah_linear_pack_weight(n, k, kind) */
    const void* x_packed;     /* packed rows [32 * k] */
    const void* residual;     /* bf16 [rows, n] added to the product, or NULL (TAH_LINEAR_PLAIN only); may be `out` */
    void* out;                /* bf16 [rows, n] row-major, or NULL */
    void* out_packed;         /* packed rows [32 * n] for the next layer (n % 32 == 0), or NULL; one of out / out_packed
                               * is needed */
    int64_t residual_row_stride, out_row_stride; /* elements */
    int32_t rows, n, k;       /* rows <= 32 */
    int32_t kind;             /* TAH_LINEAR_PLAIN: out = act(bf16(r (x W^T - m c)) [+ bias] [+ residual])
                               * TAH_LINEAR_GATE_UP: out = bf16(silu(g)) * u, g = bf16(r x Wg^T), u = bf16(r x Wu^T) */
    int32_t input_norm;       /* TAH_NORM_RMS: r = rsqrt(mean(x[row]^2) + norm_eps), an RMSNorm of the rows whose weight is
                               * already inside W (the MLP's input norm for gate|up, the final norm for an output head);
                               * TAH_NORM_LAYER (plain only): a LayerNorm of the rows, m = mean(x[row]), r = rsqrt(var(x[row])
                               * + norm_eps), c = ln_colsum; W holds W0 diag(gamma) and bias bf16(W0 beta + b0) for the
                               * layer W0, b0 behind LayerNorm(gamma, beta) (the blocks of the learned iteration decider,
                               * tah/model/iter_decider.py:139-152, :166-169);  TAH_NORM_NONE: r = 1, m = 0 */
    float norm_eps;
    const void* bias;         /* TAH_LINEAR_PLAIN: bf16 [n] added to the product (after its rounding to bf16, before the
                               * residual), or NULL */
    int32_t activation;       /* TAH_LINEAR_PLAIN: TAH_ACT_RELU / TAH_ACT_GELU applied last (a small MLP's first layer) */
    const float* ln_colsum;   /* TAH_NORM_LAYER: float32 [n], sum over k of the bf16 weight row as packed; else ignored */
} tah_linear_rows_args;
int tah_linear_rows(const tah_linear_rows_args* args, tah_stream_t stream);

/* One greedy generation step after the logits exist: per row, the final logits (first-iteration logits, plus
 * the second iteration's for rows that took one, summed in bf16 as the model's logits buffers are,
 * tah/model/tah_model.py:543,628), their arg-max (the lower index among equals), and the generation loop's
 * bookkeeping of tah/model/utils.py:228-262 without its per-row `.item()`: a row whose token is `eos` is finished
 * and the token is not part of its output; finished rows write 0; positions advance for the rows that decoded.
 * The final logits are never written out.  One launch instead of about thirty small ones per step. */
typedef struct tah_greedy_step_args {
    const void* logits0;      /* bf16 [rows, vocab] */
    const void* logits1;      /* bf16 [rows, vocab] or NULL (then hard is NULL too) */
    const uint8_t* hard;      /* [rows] nonzero: the row's logits are bf16(logits0 + logits1) */
    int64_t row_stride0, row_stride1; /* elements, multiples of 8 */
    int32_t rows, vocab;
    int32_t eos;              /* end-of-sequence token id, < 0 for none */
    int64_t* tok;             /* [rows] out: the token chosen, 0 for finished rows (input of the next step) */
    uint8_t* finished;        /* [rows] in/out */
    int32_t* pos;             /* [rows] += 1 for rows that were not finished */
    int64_t* out_tokens;      /* [rows, out_stride] column step_idx[0] is written */
    int64_t out_stride;
    const int64_t* step_idx;  /* [1] */
    int32_t out_cols;         /* columns of out_tokens: with step_idx[0] >= out_cols (a captured step replayed more often
                               * than the buffer has columns) nothing is stored and the row is marked finished */
    int32_t* out_len;         /* [rows] += 1 for rows still unfinished after this step */
    int64_t* n_hard;          /* += hard rows among those that decoded */
    int64_t* n_steps;         /* += rows that decoded */
} tah_greedy_step_args;
int tah_greedy_step(const tah_greedy_step_args* args, tah_stream_t stream);

/* Start of a generation step (one token per sequence), in one launch: for row i, active[i] = !finished[i]; slot[i] = i
 * and q_pos[i] = pos[i] for active rows, -1 for finished ones (nothing cached, nothing seen); the rotary rows of
 * position pos[i] (clamped into the tables); and the embedding row of tok[i], row-major and, when x_packed is given
 * (rows <= 32, hidden % 32 == 0), in the rows form of tah_linear_rows (rows past `rows` are not touched).  Replaces the
 * embed_tokens lookup of the base model and the rotary lookup (Qwen3Model.forward / Qwen3RotaryEmbedding, third party)
 * for the generation loop of tah/model/utils.py:228-262, plus the masks a fixed-shape step needs. */
typedef struct tah_step_begin_args {
    const int64_t* tok;       /* [rows] */
    const int32_t* pos;       /* [rows] */
    const uint8_t* finished;  /* [rows] */
    const void* embed;        /* bf16 [vocab, hidden] */
    int64_t embed_row_stride;
    const void* cos_table;    /* bf16 [table_rows, 128] */
    const void* sin_table;
    int32_t rows, vocab, hidden, table_rows;
    void* x;                  /* bf16 [rows, hidden] out */
    int64_t x_row_stride;
    void* x_packed;           /* bf16 [32 * hidden] out, or NULL */
    void* cos_rows;           /* bf16 [rows, 128] out */
    void* sin_rows;
    int32_t* slot;            /* [rows] out */
    int32_t* q_pos;           /* [rows] out */
    uint8_t* active;          /* [rows] out */
    /* Optional, for a batch whose rows are at different latent iterations (tah_greedy_tick): phase[i] != 0 means row i
     * runs the second iteration of its token -- its input is x_alt[i] (the top-k mix the previous tick left there)
     * instead of the embedding row; q_depth[i] = phase[i]; append_at[i] = hard_len[i] for such rows, pos[i] for the
     * others (the row count of the segment the row appends to); eligible[i] = active and at the first iteration. */
    const int32_t* phase;     /* [rows] or NULL */
    const void* x_alt;        /* bf16 [rows, hidden]; needed with phase */
    int64_t x_alt_row_stride;
    const int32_t* hard_len;  /* [rows]; needed with append_at */
    int32_t* q_depth;         /* [rows] out or NULL */
    int32_t* append_at;       /* [rows] out or NULL */
    uint8_t* eligible;        /* [rows] out or NULL */
} tah_step_begin_args;
int tah_step_begin(const tah_step_begin_args* args, tah_stream_t stream);

/* Second layer of a two-layer decider MLP and the decision, in one launch: hard[i] = sigmoid(bf16(bf16(hidden[i] . w2) +
 * b2)) > threshold and active[i] (the roundings of the eager `h @ w2.T + b2` in bf16, then .float().sigmoid()), and for
 * the second latent iteration hard_i32[i] (0/1), slot[i] = i and q_pos[i] = pos[i] for hard rows, -1 otherwise (each
 * optional).  The first layer is a tah_linear_rows call with bias and relu.  The decider of the end-to-end workload
 * (hidden -> 512 -> 1); the reference's MLPIterDecider (tah/model/iter_decider.py:193-301) is a larger network. */
typedef struct tah_decider_tail_args {
    const void* hidden;       /* bf16 [rows, width], after the first layer's ReLU */
    int64_t hidden_row_stride;
    const void* w2;           /* bf16 [width] */
    const void* b2;           /* bf16 [1] or NULL */
    float threshold;
    int32_t rows, width;      /* width % 8 == 0 */
    const uint8_t* active;    /* [rows] or NULL (all) */
    const int32_t* pos;       /* [rows]; needed with q_pos */
    uint8_t* hard;            /* [rows] out */
    int32_t* hard_i32;        /* [rows] out or NULL */
    int32_t* slot;            /* [rows] out or NULL */
    int32_t* q_pos;           /* [rows] out or NULL */
} tah_decider_tail_args;
int tah_decider_tail(const tah_decider_tail_args* args, tah_stream_t stream);

/* End of a tick of a generation loop in which every row advances by one latent iteration of its own token, so that a
 * row whose token needs no second iteration does not wait for those that do (the reference's loop,
 * tah/model/tah_model.py:580-706 + tah/model/utils.py:228-262, keeps the batch in step; per row the computation and its
 * result are the same).  phase[i]: 0 = row i just ran the first iteration of a token, 1 = the second.  Rows with
 * phase 0 and hard_now[i] set only move to phase 1.  Every other unfinished row gets its token -- the arg-max of
 * `logits`, or of bf16(logits_prev + logits) at phase 1 (logits_prev: what the previous tick's launch left there, the
 * row's first iteration) -- written to out_tokens[i, out_len[i]]; out_len, pos, tok, finished (end-of-sequence, which is
 * not written, or `limit` tokens reached), phase = 0, hard_len += 1 and n_hard += 1 after a second iteration,
 * n_steps += 1.  With `chosen` set the token of row i is chosen[i] instead of the arg-max (a sampled token, drawn by the
 * caller from the same final logits); the logits are then not read and may be NULL. */
typedef struct tah_greedy_tick_args {
    const void* logits;       /* bf16 [rows, vocab]: this tick's */
    const void* logits_prev;  /* bf16 [rows, vocab]: the previous tick's */
    int64_t row_stride, row_stride_prev; /* elements, multiples of 8 */
    int32_t rows, vocab;
    int32_t eos;              /* end-of-sequence token id, < 0 for none */
    int32_t limit;            /* a row is finished when out_len reaches it */
    const uint8_t* hard_now;  /* [rows] */
    int32_t* phase;           /* [rows] in/out */
    int64_t* tok;             /* [rows] out */
    uint8_t* finished;        /* [rows] in/out */
    int32_t* pos;             /* [rows] in/out */
    int64_t* out_tokens;      /* [rows, out_stride] */
    int64_t out_stride;
    int32_t* out_len;         /* [rows] in/out */
    int32_t* hard_len;        /* [rows] in/out */
    int64_t* n_hard;
    int64_t* n_steps;
    const int64_t* chosen;    /* [rows] or NULL: take these tokens instead of the arg-max */
} tah_greedy_tick_args;
int tah_greedy_tick(const tah_greedy_tick_args* args, tah_stream_t stream);

/* Hard-token index build: stream compaction of a (B, S) byte mask in row-major
 * order.  Replaces the stable sort + nonzero of gather_active / scatter_back
 * (tah/model/tah_model.py:111-119, :160-167).  For the r-th True entry, at
 * (b, s): pos_out[r] = s, flat_out[r] = b*S + s, seq_out[r] = b (each may be
 * NULL; capacity B*S when given); cu_out[b] = number of True entries in rows
 * < b, cu_out[B] = total (required, B+1 entries).  Bit-exact. */
int tah_hard_index_build(const uint8_t* mask, int32_t B, int32_t S, int32_t* pos_out, int32_t* flat_out,
                         int32_t* seq_out, int32_t* cu_out, tah_stream_t stream);

/* Destination rows of the right-padded (B, width) form used by gather_active
 * (tah/model/tah_model.py:117-134): out[r] = seq_of[r]*width + (r - cu[seq_of[r]]) for r < n.  When n_dev is
 * given (a device int32, e.g. &cu[B] as tah_hard_index_build wrote it) only the first min(n, *n_dev) entries
 * are produced, so that a caller that never reads the count back can pass an upper bound as n.  An entry
 * whose rank inside its row is >= width gets -1 (tah_rows_copy skips it) and sets *overflow (optional). */
int tah_pad_rows_build(const int32_t* cu, const int32_t* seq_of, int32_t n, const int32_t* n_dev, int32_t width,
                       int32_t* out, int32_t* overflow, tah_stream_t stream);

/* Row gather / scatter: dst[dst_rows ? dst_rows[r] : r] = src[src_rows ? src_rows[r] : r]
 * for r < n (and r < *n_dev when n_dev is given: the count stays on the device), rows of row_bytes bytes at
 * the given byte strides; when dst_enable is given (one byte per destination row) rows whose byte is 0 are
 * left untouched -- the assignment_mask of scatter_back; a negative row index skips the entry.  Replaces
 * torch.gather (tah_model.py:127-133) and the boolean-mask index_put (tah_model.py:163-175), and with n_dev
 * the host synchronisation of tah_model.py:116.  Rows named twice in dst_rows race.  Bit-exact. */
int tah_rows_copy(const void* src, const int32_t* src_rows, void* dst, const int32_t* dst_rows,
                  const uint8_t* dst_enable, int32_t n, const int32_t* n_dev, int64_t row_bytes,
                  int64_t src_stride_bytes, int64_t dst_stride_bytes, tah_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* TAH_DUO_H */
