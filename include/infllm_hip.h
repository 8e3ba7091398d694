/*
 * C ABI of libinfllm_hip.so: the gfx950 (MI355X) kernels behind the InfLLM
 * streaming memory-attention path.
 *
 * Conventions
 *  - every pointer named d_* is a device address, h_* a (pinned) host address;
 *  - bf16 buffers are passed as `const void*` / `void*`, fp32 as float*;
 *  - all strides are in ELEMENTS, the innermost (head_dim) axis is contiguous;
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream);
 *  - every call only enqueues work; buffers are borrowed until that work ends;
 *  - return value 0 = ok, negative = rejected arguments or a launch error, with
 *    the message available from infllm_last_error() (thread local);
 *  - head_dim must be 128; dtype of q/k/v is bf16.
 *
 * Each entry point names the part of the reference it replaces (file:line in
 * thunlp/InfLLM).
 */
#ifndef INFLLM_HIP_H
#define INFLLM_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define INFLLM_ABI_VERSION 1
#define INFLLM_HEAD_DIM 128
#define INFLLM_KEY_TILE 64

/* Library identity; no counterpart in the reference (a pure-Python package). */
int infllm_version(void);
const char *infllm_last_error(void);

/* ---------------------------------------------------------------------------
 * Prologue: RoPE + staging of new tokens.
 * Replaces RotaryEmbeddingESM.forward / apply_rotary_pos_emb_one_angle
 * (inf_llm/attention/rope.py:89-112) and the torch.cat of the local window and
 * the remainder (inf_llm/attention/context_manager.py:719-747).
 *
 * For the n new tokens at absolute stream positions pos0 .. pos0+n-1:
 *   ring_k_raw / ring_v  <- k, v                 (row  pos % ring_cap)
 *   ring_k_rot           <- RoPE(k, angle pos)
 *   q_loc                <- RoPE(q, angle pos)
 *   q_glb                <- RoPE(q, angle glb_pos)      (glb_pos = n_local - 1)
 *   ring_score rows of the new tokens <- 0
 * The relative rotation between q_loc[i] and ring_k_rot[j] is exactly
 * (pos_i - pos_j) * inv_freq, which is what the reference's window-relative
 * tables produce.  Angles are formed in fp64 (pos * distance_scale * inv_freq)
 * so that positions of 10^6 and beyond keep full precision.
 * q: [B,H,n,128], k/v: [B,Hkv,n,128]; rings: [B,Hkv,ring_cap,128];
 * q_loc/q_glb: [B,H,n,128] contiguous; ring_score: fp32 [B,H,ring_cap].
 */
typedef struct {
    const void *d_q, *d_k, *d_v;
    int64_t q_sb, q_sh, q_sl;      /* strides of q */
    int64_t k_sb, k_sh, k_sl;      /* strides of k */
    int64_t v_sb, v_sh, v_sl;      /* strides of v */
    int32_t B, H, Hkv, n;
    int64_t pos0;
    int64_t glb_pos;
    const float *d_inv_freq;       /* [64] fp32, as the reference computes it */
    double distance_scale;
    void *d_ring_k_raw, *d_ring_k_rot, *d_ring_v;
    float *d_ring_score;
    int64_t ring_cap;
    void *d_q_loc, *d_q_glb;
    float *d_qpart;                /* optional fp32 [B, ceil(n/16), H*128]: sums of q_glb over each run of 16 positions */
} infllm_ingest_args;
int infllm_ingest(const infllm_ingest_args *a, void *stream);

/* out[b,c] = scale * sum_p parts[b,p,c] (p ascending): turns the d_qpart sums of infllm_ingest into
 * the mean global query of a block (context_manager.py:373-375) with scale = 1/n. */
int infllm_reduce_partials(const float *d_parts, int32_t B, int32_t n_parts, int32_t C, float scale,
                           float *d_out, void *stream);

/* Mean of q_glb over each execution block (context_manager.py:373-375):
 * q_glb [B,H,n,128] contiguous -> d_qbar fp32 [B, n_blocks, H*128],
 * block j covers rows [j*exc, min((j+1)*exc, n)). */
int infllm_block_mean(const void *d_q_glb, int32_t B, int32_t H, int32_t n, int32_t exc,
                      float *d_qbar, void *stream);
/* The same means for a whole chunk of un-rotated input rows q [B,H,n,128] (strides in elements), as
 * get_batched_topk needs them (context_manager.py:548-612, with the one-angle rotation of :744-746):
 * d_qbar fp32 [B, n_blocks, H*128] = RoPE(mean of the block's rows, angle glb_pos). */
int infllm_chunk_qbar(const void *d_q, int64_t q_sb, int64_t q_sh, int64_t q_sl, int32_t B, int32_t H,
                      int32_t n, int32_t exc, const float *d_inv_freq, double distance_scale,
                      int64_t glb_pos, float *d_qbar, void *stream);

/* RoPE of plain rows, for the attention types that rotate tensors themselves (stream_llm.py:62-73,
 * infinite_lm.py:59-66, origin.py:36; rope.py:27-47, 93-112): x [B,H,L,128] bf16 with element strides
 * sb/sh/sl -> d_out [B,H,L,128] contiguous, row r rotated by the angle of position pos0 + r*pos_step
 * (pos_step 1: consecutive positions; 0: one angle for every row).  Angles in fp64. */
int infllm_rope_rows(const void *d_x, int64_t sb, int64_t sh, int64_t sl, int32_t B, int32_t H, int32_t L,
                     int64_t pos0, int32_t pos_step, const float *d_inv_freq, double distance_scale,
                     void *d_out, void *stream);

/* ---------------------------------------------------------------------------
 * One stage of the multi-stage attention (bf16 MFMA flash kernel).
 * Replaces MultiStageDotProductionAttention.append
 * (inf_llm/attention/dot_production_attention/torch_impl.py:39-96,
 *  triton_impl.py:488-556) for one stage; stages are joined by
 * infllm_attn_merge.  Keys come either from a "linear" source (a tensor or a
 * ring: key index j lives in row j % cap) with the reference's mask
 *      dist = i - j + offset;  window: 0 <= dist < size;  complement: dist >= size
 * or from a page table of 64-key tiles (memory units, init tokens, overflow
 * remainder: context_manager.py:386-451), all keys of which are visible.
 * Output: per split s, un-merged partial results
 *      o_part [nsplit,B,H,Lq,128] fp16 bit patterns (normalised by the split's own sum, so bounded by
 *                                 max |v|; 11 significant bits against the 8 of the bf16 result)
 *      lse_part [nsplit,B,H,Lq]   fp32 (base-2 log-sum-exp of scaled logits)
 */
typedef struct {
    const void *k;            /* device address of key row 0 of kv head 0 */
    const void *v;
    int64_t head_stride;      /* elements between kv heads */
    int32_t n_valid;          /* 1..64 rows */
    int32_t reserved;
} infllm_page;

enum { INFLLM_MASK_NONE = 0, INFLLM_MASK_WINDOW = 1, INFLLM_MASK_COMPLEMENT = 2 };

typedef struct {
    const void *d_q;               /* [B,H,Lq,128] */
    int64_t q_sb, q_sh, q_sl;
    int32_t B, H, Hkv, Lq;
    /* linear source (d_pages == NULL) */
    const void *d_k, *d_v;
    int64_t k_sb, k_sh, k_sl, v_sb, v_sh, v_sl;
    int64_t cap;                   /* rows of the ring; >= j_hi for a plain tensor */
    int64_t j_lo, j_hi;            /* key index range held by the source */
    int32_t mask;                  /* INFLLM_MASK_* */
    int32_t reserved;
    int64_t offset, window;
    /* paged source (d_pages != NULL): [B, n_pages] */
    const infllm_page *d_pages;
    int32_t n_pages;
    int32_t nsplit;
    float softmax_scale;           /* 1/sqrt(128) */
    uint16_t *d_o_part;            /* fp16 */
    float *d_lse_part;
} infllm_attn_args;
int infllm_attn_stage(const infllm_attn_args *a, void *stream);

/* Joint softmax across stages/splits (torch_impl.py:15-36):
 * o = sum_p 2^(lse_p - LSE) o_p, LSE = log2 sum_p 2^lse_p.
 * d_o_part fp16 [P,B,H,Lq,128], d_lse_part [P,B,H,Lq] -> d_out bf16 [B,H,Lq,128]
 * (strides given, multiples of 8 elements), d_lse fp32 [B,H,Lq].  d_lse may be NULL (output only); d_out may be NULL (log-sum-exp
 * only, a much smaller launch: the scores of infllm_local_score need nothing else). */
int infllm_attn_merge(const uint16_t *d_o_part, const float *d_lse_part, int32_t P,
                      int32_t B, int32_t H, int32_t Lq,
                      void *d_out, int64_t o_sb, int64_t o_sh, int64_t o_sl,
                      float *d_lse, void *stream);
/* The operator's whole forward in one call (attn.append(local...), attn.append(global..., end=True),
 * attn.get_result(): context_manager.py:486-489, 526-533): the local stage over a ring or tensor, the global
 * stage over a page table (either may be NULL), and their merge into d_out / d_lse.  The stages keep their own
 * nsplit; the global stage's partial buffers must directly follow the local stage's
 * (global->d_o_part == local->d_o_part + local->nsplit*B*H*Lq*128, likewise d_lse_part). */
int infllm_attn_fwd(const infllm_attn_args *local, const infllm_attn_args *global,
                    void *d_out, int64_t o_sb, int64_t o_sh, int64_t o_sl, float *d_lse, void *stream);

/* Both stages of the operator in ONE launch (attn.append(local...) + attn.append(global..., end=True),
 * context_manager.py:486-489, 526-533; the reference's fused implementation carries the softmax state across its
 * stages the same way, triton_impl.py:488-556): the linear stage's tiles and the paged stage's pages form one list
 * that `nsplit` key splits divide between them, each with the queries of its own stage (local->d_q, global->d_q).
 * Both blocks must agree on B, H, Hkv, Lq and softmax_scale; nsplit and the partial buffers are taken from `local`:
 * d_o_part [nsplit,B,H,Lq,128] fp16, d_lse_part [nsplit,B,H,Lq] - one set of partials for both stages, to be joined
 * by infllm_attn_merge with P = nsplit. */
int infllm_attn_stages_fused(const infllm_attn_args *local, const infllm_attn_args *global, void *stream);

/* infllm_attn_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The stages' partial rows, which
 * infllm_attn_fwd takes from the caller as a workspace (d_o_part / d_lse_part), live in an array inside the library's
 * own image instead: the d_o_part / d_lse_part fields of both argument blocks are ignored, everything else is as for
 * infllm_attn_fwd, and the results are the same bit for bit.  The call allocates nothing (no hipMalloc / hipFree, no
 * allocating library routine).  Limit: (local nsplit + global nsplit) * B * H * Lq <= INFLLM_NOALLOC_MAX_PART_ROWS
 * partial rows (260 bytes each: 16.25 MiB of device memory per GPU, held until the process ends); larger calls are
 * rejected with an error.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams,
 * two threads) race - serialise them, or use infllm_attn_fwd with workspaces of your own.  The first call on a device
 * also looks up that device's copy of the array and sets the kernels' attributes (safe from several threads at once,
 * but not something a graph capture records): make one call per device before capturing. */
#define INFLLM_NOALLOC_MAX_PART_ROWS 65536
int infllm_attn_fwd_noalloc(const infllm_attn_args *local, const infllm_attn_args *global,
                            void *d_out, int64_t o_sb, int64_t o_sh, int64_t o_sl, float *d_lse, void *stream);

/* ---------------------------------------------------------------------------
 * Column sums of the final probabilities of one linear stage
 * (torch_impl.py:27-28; triton_impl.py:232-335):
 *   score[b,h,j] (+)= sum_i 2^(scale*log2e*q_i.k_j - lse[b,h,i]) * visible(i,j)
 * for j in [j_lo, j_hi); score row index is j % score_cap.
 */
typedef struct {
    const void *d_q;
    int64_t q_sb, q_sh, q_sl;
    int32_t B, H, Hkv, Lq;
    const void *d_k;
    int64_t k_sb, k_sh, k_sl;
    int64_t cap;
    int64_t j_lo, j_hi;
    int32_t mask;
    int32_t accumulate;            /* 1: add to d_score, 0: overwrite */
    int64_t offset, window;
    const float *d_lse;            /* n_parts == 0: [B,H,Lq] from infllm_attn_merge;  n_parts > 0: the
                                      partial log-sum-exps [n_parts,B,H,Lq] of infllm_attn_stage, joined on the
                                      fly (saves the merge launch when nothing else needs the joint value yet) */
    float softmax_scale;
    int32_t n_parts;
    float *d_score;                /* fp32 [B,H,score_cap] */
    int64_t score_sb, score_sh, score_cap;
} infllm_score_args;
int infllm_local_score(const infllm_score_args *a, void *stream);

/* ---------------------------------------------------------------------------
 * Retrieval: unit scores + top-k.
 * Replaces VectorTensor.get_topk and calc_block_topk
 * (context_manager.py:159-163, 366-383).
 *   scores[n] = sum_c reps[n,c] * qbar[c]   (bf16 reps, fp32 qbar, fp32 out)
 *   idx[0..k)  = indices of the k largest scores in descending score order, as torch.topk
 *                returns them (the residency policy inserts a block's missed units in this
 *                order, context_manager.py:495-515); equal scores go to the lower index
 *                first, at the boundary and in the order.
 * reps [N,C] bf16 row stride rep_stride; C = H*128.  k <= 1024.
 */
int infllm_score_topk(const void *d_reps, int64_t rep_stride, int32_t N, int32_t C,
                      const float *d_qbar, int32_t k,
                      float *d_scores, int32_t *d_idx, void *stream);
/* The selection over ALL units from two parts (what the stream does between blocks): d_cand[n_cand] are the k best,
 * in any order, of units [0, first_new) (infllm_topk over their scores, taken while other work was in flight);
 * this scores the n_new units [first_new, first_new + n_new) (d_scores[first_new ...] = reps . qbar, the same
 * arithmetic as infllm_unit_scores) and ranks them against the candidates in the same launch: d_idx[k] as
 * infllm_topk over all first_new + n_new scores would give (a unit of the overall top-k that is not new is among
 * the k best of the old ones).  n_cand + n_new <= 64; rows of 512, 1024, 2048 or 4096 elements. */
int infllm_score_new_topk(const void *d_reps, int64_t rep_stride, int32_t C, const float *d_qbar, float *d_scores,
                          const int32_t *d_cand, int32_t n_cand, int32_t first_new, int32_t n_new, int32_t k, int32_t *d_idx,
                          void *stream);
/* infllm_score_topk for several mean queries over the same N units, every representative read once per 8 queries
 * (the selections of all execution blocks of a chunk or call against the units that exist at its start:
 * get_batched_topk, context_manager.py:548-612; the stream uses it once per prepared call).  Query q's scores go to
 * d_scores + q * scores_qs (the same bits as infllm_unit_scores gives), its ids to d_idx + q * idx_qs, its mean query
 * is at d_qbars + q * qbar_qs.  Rows of 512, 1024, 2048 or 4096 elements; returns 1, with nothing launched, for other
 * row lengths. */
int infllm_score_topk_queries(const void *d_reps, int64_t rep_stride, int32_t N, int32_t C, const float *d_qbars, int64_t qbar_qs,
                              int32_t n_queries, int32_t k, float *d_scores, int64_t scores_qs, int32_t *d_idx, int64_t idx_qs,
                              void *stream);
/* The two halves of infllm_score_topk: scores of rows [first, first+count) into d_scores[first..], and the
 * selection over d_scores[0..N).  Scoring the units that exist early and only the newly carved ones late keeps
 * the retrieval of the next block short. */
int infllm_unit_scores(const void *d_reps, int64_t rep_stride, int32_t first, int32_t count, int32_t C,
                       const float *d_qbar, float *d_scores, void *stream);
int infllm_topk(const float *d_scores, int32_t N, int32_t k, int32_t *d_idx, void *stream);

/* Representative key of carved units.
 * Replaces get_block_k + mean (context_manager.py:268-277, 664-670).
 * For unit u (0 <= u < n_units) made of the tokens at ring rows
 * (t0 + u*bs + r) % ring_cap, r < bs:
 *   per query head h: the repr_topk highest ring_score[b,h,row] (ties -> lower r),
 *   rep[b, u, h*128 + d] = mean of those rows of ring_k_raw[b, h / (H/Hkv)].
 * d_rep_out: bf16 [B] rows at d_rep_out + b*rep_sb + u*rep_su; d_idx_out (optional,
 * may be NULL): int32 [B,n_units,H,repr_topk] chosen r's in descending score order.
 */
int infllm_repr_keys(const float *d_ring_score, const void *d_ring_k_raw, int64_t ring_cap,
                     int32_t B, int32_t H, int32_t Hkv, int64_t t0, int32_t bs,
                     int32_t n_units, int32_t repr_topk,
                     void *d_rep_out, int64_t rep_sb, int64_t rep_su,
                     int32_t *d_idx_out, void *stream);

/* ---------------------------------------------------------------------------
 * Unit cache traffic.  Replaces MemoryUnit.__init__/load
 * (context_manager.py:39-45, 76-91).
 * infllm_gather_rows: ring rows (t0 + r) % ring_cap, r < n, of every kv head ->
 *   out[b*out_sb + (r / unit_rows)*out_su + h*out_sh + (r % unit_rows)*128 ...] (device);
 *   with unit_rows = n this is a plain [B,Hkv,n,128] copy.  Used to carve units and
 *   init tokens out of the ring.
 * infllm_copy_async: hipMemcpyAsync of nbytes, kind 1 = host->device,
 *   2 = device->host, 3 = device->device, on `stream`.
 */
int infllm_gather_rows(const void *d_ring, int64_t ring_cap, int32_t B, int32_t Hkv,
                       int64_t t0, int32_t n, int32_t unit_rows, void *d_out, int64_t out_sb,
                       int64_t out_su, int64_t out_sh, void *stream);
int infllm_copy_async(void *dst, const void *src, int64_t nbytes, int32_t kind, void *stream);
/* the same under the name the cache's own transfers go by (MemoryUnit.load / offload, context_manager.py:64-109) */
int infllm_cache_copy_async(void *dst, const void *src, int64_t nbytes, int32_t kind, void *stream);
/* infllm_fetch_units: n copies of nbytes each, pinned host -> device, in ONE kernel launch that reads the
 *   device-mapped pinned memory directly (the misses of a block are scattered over the host arena; issuing a
 *   hipMemcpyAsync per 512 KiB unit costs more than moving it).  h_src[i] must be the device-visible address
 *   of pinned memory (infllm_host_device_pointer), both sides 16-byte aligned.  Replaces the H2D half of
 *   MemoryUnit.load (context_manager.py:76-91).
 * infllm_host_device_pointer: hipHostGetDevicePointer of a pinned allocation (NULL on failure). */
int infllm_fetch_units(const void *const *h_src, void *const *d_dst, int32_t n, int64_t nbytes, void *stream);
void *infllm_host_device_pointer(void *h_pinned);

/* ---------------------------------------------------------------------------
 * One execution block in three calls (four with the fetch ahead of the selection).
 * Replaces the device work of ContextManager._append and append_global
 * (context_manager.py:474-545, 614-679) for one block of at most exc_block_size
 * queries; the host keeps the state machine (what is carved when), the cache policy is
 * infllm_cache_* further down:
 *
 *   infllm_block_front   the block's prologue (RoPE + rings) and retrieval (mean query, unit
 *                        scores, top-k, asynchronous copy of the ids to pinned memory) unless
 *                        the previous block already did them ahead; when the caller passes the NEXT
 *                        block's rows, that block's prologue, the scores of the units that already
 *                        exist and their k best (the candidates of the next selection); then the local
 *                        stage (inside a call prepared by infllm_call_front: no prologue, and the
 *                        local stage of two blocks per launch);
 *   infllm_block_select  waits until the ids of this block are readable on the host, runs the cache
 *                        policy and issues the fetch of the missed units (copy stream); the same in
 *                        separate steps: infllm_layer_wait_topk, the caller's own policy,
 *                        infllm_block_fetch;
 *   infllm_block_back    (the fetch, if nothing issued it yet,) page table, global stage, merge,
 *                        local score of the tokens about to be carved, init peeling,
 *                        representatives of the new units, and - when the next block was
 *                        prepared - the scores of the new units, the next block's top-k and
 *                        the copy of its ids; only then the block's output rows, the rest of the
 *                        local score and the gather of the new units into a staging slot
 *                        (while fetches run ahead of the selection: ONE local-score launch over the whole
 *                        window before the representatives, with the merge riding in it as extra
 *                        workgroups, since nothing waits for the selection at once);
 *   infllm_block_prefetch  (optional, further down) starts the NEXT block's fetch from its candidates.
 *
 * The fetch of missed units goes through 7 DMA engines (ROCr copies) for blocks of 64 queries or more, and the
 * main stream waits with hipStreamWaitValue32 for a sequence number the engines write behind the units; shorter
 * blocks, and processes without usable engines (or with INFLLM_NO_DMA_FETCH=1), use the zero-copy kernel
 * of infllm_fetch_units on the copy stream.  Either way the fetch is ordered behind the last reader of the slots
 * and behind the offload of units that are still on their way to the host.  A missed unit whose rows are still in
 * the staging slot they were gathered into when it was carved is copied from there on the main stream instead.
 * An eighth engine is kept for the carved units' way to the host.
 *
 * The chain from one block's ids to the next block's ids is therefore: fetch, global stage,
 * a small local-score launch (which joins the stages' log-sum-exps itself), representatives, a
 * small unit-score launch, the final ranking; the merge runs behind it.
 *
 * The copy of newly carved units from the staging slot to pinned host memory is deferred and
 * ordered by the host: once the gather's event has fired (checked at the next block's calls) it
 * goes to the DMA engine (ROCr asynchronous copy), whose completion signal is checked before the
 * staging slot is reused and before a fetch reads one of those units.  Where that is not
 * possible (no ROCr agents, INFLLM_NO_DMA_ENGINE=1, or a fetch needs the units at once) it is a
 * hipMemcpyAsync on the copy stream.  infllm_layer_flush issues whatever is still pending, waits
 * for the engine copies, and must be called when no further block follows (end of an append()
 * call); after it and a synchronisation of the copy stream the host copies are complete.
 *
 * The next block's selection is prepared in two parts: the top-k of the units that exist when
 * infllm_block_front prepares the next block is taken there (off the chain), and after the block only
 * those k candidates and the units carved in between are ranked (same result as one top-k over all).
 *
 * A layer handle owns only events, ROCr signals, a [B,topk] device array and a pinned copy for those
 * candidates, 8 bytes of signal memory, shadow policy objects for the guess in flight, the rotation of the
 * pinned page-table staging slots and of the carve staging slots; every other buffer is the caller's.
 */
typedef struct {
    int32_t B, H, Hkv;
    int32_t n_local, n_init, block_size, exc, topk, repr_topk, max_cached;
    int32_t max_splits, num_cus;
    int64_t ring_cap;
    void *d_ring_k_raw, *d_ring_k_rot, *d_ring_v;     /* [B,Hkv,ring_cap,128] */
    float *d_ring_score;                              /* [B,H,ring_cap] */
    void *d_init_kv;                                  /* [B,2,Hkv,init_cap,128] */
    int64_t init_cap;
    void *d_slab;                                     /* [B,max_cached,2,Hkv,block_size,128] */
    /* two slots each (a block and the one prepared ahead) */
    void *d_q_loc, *d_q_glb;                          /* [2][B*H*exc*128] */
    float *d_qbar;                                    /* [2][B,H*128] */
    float *d_qpart;                                   /* [2][B,ceil(exc/16),H*128] */
    uint16_t *d_o_part;                               /* fp16 [2*max_splits,B,H,exc,128] */
    float *d_lse_part, *d_lse;                        /* [2*max_splits,B,H,exc], [B,H,exc] */
    int32_t *d_topk_idx, *h_topk_idx;                 /* [B,topk] device / pinned host; h_topk_idx may be NULL when
                                                         d_topk_idx is the device-visible address of pinned memory:
                                                         the top-k kernel then writes the ids where the host reads them */
    infllm_page *d_pages;                             /* [B,max_pages] */
    infllm_page *h_pages;                             /* pinned, [page_slots,B,max_pages] */
    int32_t max_pages, page_slots;
    void *d_carve_stage;                              /* [carve_slots,max_carve,B,2,Hkv,block_size,128] */
    int32_t max_carve, carve_slots;
    const float *d_inv_freq;
    double distance_scale;
    float softmax_scale;
    int32_t reserved;
    /* Optional (both or neither): one pinned int32, as the device sees it and as the host sees it.  With
     * h_topk_idx == NULL the selection kernel stores a sequence number there after the ids, and
     * infllm_layer_wait_topk polls it instead of sleeping on an event (falls back to the event after 2 ms). */
    int32_t *d_topk_flag;
    const volatile int32_t *h_topk_flag;
} infllm_layer_desc;

void *infllm_layer_create(const infllm_layer_desc *desc);    /* NULL + infllm_last_error() on failure */
int infllm_layer_destroy(void *layer);

typedef struct {
    const void *d_q, *d_k, *d_v;                      /* this block's rows: [B,H,n,128], [B,Hkv,n,128] */
    int64_t q_sb, q_sh, q_sl, k_sb, k_sh, k_sl, v_sb, v_sh, v_sl;
    int32_t n;                                        /* queries in the block, 1..exc */
    int32_t n_units;                                  /* units carved so far (per batch row) */
    int64_t b0;                                       /* stream position of the first query */
    const void *d_reps;                               /* [B, rows, H*128] bf16 representatives */
    int64_t rep_sb, rep_su;
    float *d_unit_scores;                             /* [B, >= n_units] */
    int64_t unit_scores_sb;
    const void *d_q_next, *d_k_next, *d_v_next;       /* rows of the next block (same strides), or NULL */
    int32_t n_next, flags;                            /* INFLLM_NO_RETRIEVAL: the caller supplies the selection */
    /* infllm_call_front only, optional: [ceil(n / exc), B, call_scores_cols] floats, call_scores_cols >= n_units + the
     * units the call can carve.  Given, the k best of the units that exist now are chosen for every block of the call
     * in one go (VectorTensor.get_topk, context_manager.py:159-163, once per call instead of once per block); a
     * block's selection then only weighs its list against the units carved since the call began - the same ids in
     * the same order.  The buffer is in use until the call's last infllm_block_back. */
    float *d_call_scores;
    int64_t call_scores_cols;
} infllm_front_args;
int infllm_block_front(void *layer, const infllm_front_args *a, void *stream);

/* A whole append() call prepared in one go.  ContextManager.append (context_manager.py:749-798) works its tokens off
 * in execution blocks, and the sliding-window half of a block's attention (context_manager.py:474-482) needs nothing
 * but the block's own rows and the rows before it - so, once the call's rows are in the rings, it can run for several
 * blocks in one launch, ahead of the blocks' retrieval:
 *
 *   infllm_layer_set_batch  hands the layer the buffers this takes (the caller's allocation, like the workspaces of
 *                           infllm_layer_desc): rotated queries of a call, the blocks' mean queries and the local
 *                           stage's partial rows.  Needs exc_block_size to be a multiple of 32.
 *   infllm_call_front       a->d_q/d_k/d_v are the rows of the next a->n <= max_tokens tokens (a->b0 the first one's
 *                           position); runs the prologue for all of them (the rings must have room: ring_cap >=
 *                           a->b0 - cursor + a->n), every block's mean query, the first block's retrieval when
 *                           a->n_units > topk (and, with a->d_call_scores, the lists of the other blocks'
 *                           selections, see there).  The blocks then go through infllm_block_front / select / back as
 *                           ever, in order; block_front finds their prologue done (its d_q / d_k / d_v and
 *                           next-block pointers are not read, n_next still says whether a block of this call
 *                           follows) and launches the local stage for group_blocks blocks at a time, at the first
 *                           block of each group.  infllm_layer_end_call (or infllm_layer_flush) ends the call.
 * Without these two calls every block runs its own prologue and local stage (block_front). */
typedef struct {
    void *d_q_loc, *d_q_glb;          /* [B, H, max_tokens, 128] bf16 each */
    float *d_qpart;                   /* [B, ceil(max_tokens / 16), H*128] */
    float *d_qbar;                    /* [ceil(max_tokens / exc), B, H*128] */
    uint16_t *d_o_part;               /* [part_rows, 128] fp16: partial rows of the local stage, by block */
    float *d_lse_part;                /* [part_rows] */
    int64_t part_rows;                /* >= B * H * exc * max(8, 4 * group_blocks) */
    int32_t max_tokens;
    int32_t group_blocks;             /* blocks per local-stage launch (0: 2) */
} infllm_batch_desc;
int infllm_layer_set_batch(void *layer, const infllm_batch_desc *b);
int infllm_call_front(void *layer, const infllm_front_args *a, void *stream);
int infllm_layer_wait_topk(void *layer);

/* flags of infllm_front_args / infllm_back_args: skip mean query, unit scores and top-k (the selection was made
 * elsewhere, e.g. for a whole chunk at once: context_manager.py:548-612, 749-770) */
enum { INFLLM_NO_RETRIEVAL = 1 };
typedef struct {
    int32_t n, n_sel;                                 /* queries; selected units per batch row */
    int64_t b0;
    const int32_t *h_sel_slots;                       /* host [B,n_sel]: slab slot of each selected unit */
    int32_t n_miss, init_len;                         /* units to fetch; init tokens present */
    const int32_t *h_miss_row, *h_miss_slot;          /* host [n_miss] */
    const int32_t *h_miss_unit;                       /* host [n_miss]: unit ids (to order a fetch after that unit's offload) */
    const void *const *h_miss_src;                    /* host [n_miss]: device-visible address of pinned [2,Hkv,block_size,128] */
    int64_t cursor;                                   /* first un-carved stream position */
    void *d_out;                                      /* [B,H,n,128] bf16 */
    int64_t o_sb, o_sh, o_sl;
    int32_t init_take, n_carve;                       /* state-machine actions after the block */
    void *d_rep_out;                                  /* representative row of the first new unit */
    int64_t rep_sb, rep_su;
    int32_t *d_repr_idx;                              /* optional [B,n_carve,H,repr_topk] */
    void *const *h_carve_dst;                         /* host [n_carve]: pinned [B,2,Hkv,block_size,128] */
    int32_t n_units, flags;                           /* units before this block's carving; INFLLM_NO_RETRIEVAL */
    const void *d_reps;                               /* [B, rows, H*128] (rep_sb / rep_su above) */
    float *d_unit_scores;                             /* [B, >= n_units + n_carve] */
    int64_t unit_scores_sb;
    /* Optional (NULL = off), for cache_strategy "lru-s" (context_manager.py:454-470, 529-543): d_unit_mass
     * [B,n_sel] fp32, device-visible, receives for every selected unit the sum over heads, queries and the
     * unit's tokens of the block's final attention probabilities; d_mass_scratch fp32 [B,n_sel,H,block_size].
     * infllm_layer_wait_mass blocks the host until the last such result is written. */
    float *d_unit_mass, *d_mass_scratch;
} infllm_back_args;
int infllm_layer_wait_mass(void *layer);
/* Optional: issue the fetch of infllm_block_back ahead of it, as soon as the misses are known (the rest of
 * the host's bookkeeping then overlaps the transfer); infllm_block_back must follow with the same lists. */
int infllm_block_fetch(void *layer, int32_t n_miss, const int32_t *h_miss_row, const int32_t *h_miss_slot,
                       const int32_t *h_miss_unit, const void *const *h_miss_src, void *stream, void *copy_stream);
int infllm_block_back(void *layer, const infllm_back_args *a, void *stream, void *copy_stream);

int infllm_layer_flush(void *layer, void *copy_stream);
/* The end of an append() call without the wait: what infllm_layer_flush does, except that the copy of the units the
 * last blocks carved to their pinned home (MemoryUnit.cpu_data, context_manager.py:39-45) is left to go on in the
 * background, as it does between the blocks of a call - the next call's blocks, or a later infllm_layer_flush, see
 * it through (a unit that is selected before its copy has landed is served from its staging slot as ever).  For a
 * caller that does not read the pinned copies between calls: the host then goes straight on to the next call instead
 * of waiting 50-120 us for the copy engine.  infllm_layer_flush before reading pinned units or freeing them. */
int infllm_layer_end_call(void *layer, void *copy_stream);

/* ---- residency policy of the device unit cache, one object per batch row (context_manager.py:246-265 for the
 * values, 495-515 for the eviction): lru = clock of the last use, fifo = clock of the first load, lru-s = decayed
 * attention mass; eviction takes the smallest values first (first inserted first on ties) and never a unit of the
 * current selection.  Host code (no device work): it sits between the arrival of the top-k ids and the fetch. */
enum { INFLLM_CACHE_LRU = 0, INFLLM_CACHE_FIFO = 1, INFLLM_CACHE_LRU_S = 2 };
void *infllm_cache_create(int32_t capacity, int32_t strategy, double score_decay);
int infllm_cache_destroy(void *cache);
/* One block: selected[n_sel] unit ids -> slots[n_sel] (their slab slots); the misses in selection order with the
 * slots they get; the evicted ids in eviction order (evicted / n_evicted may be NULL).  Returns the number of misses. */
int infllm_cache_touch(void *cache, const int32_t *selected, int32_t n_sel, int32_t *slots, int32_t *miss_units,
                       int32_t *miss_slots, int32_t *evicted, int32_t *n_evicted);
/* The same with slot wishes: a missed unit listed in hint_units takes its hint_slots entry when that slot is free
 * once the evictions are done (a caller that has moved the unit there already, see infllm_block_prefetch); which slot
 * a unit occupies changes nothing else. */
int infllm_cache_touch_hinted(void *cache, const int32_t *selected, int32_t n_sel, int32_t *slots, int32_t *miss_units,
                              int32_t *miss_slots, int32_t *evicted, int32_t *n_evicted, const int32_t *hint_units,
                              const int32_t *hint_slots, int32_t n_hints);
/* lru-s (context_manager.py:529-543): every resident's value decays, then the given units gain their scores */
int infllm_cache_add_scores(void *cache, const int32_t *units, const double *scores, int32_t n);
/* residents in insertion order (any output may be NULL); returns their number */
int infllm_cache_residents(void *cache, int32_t *units, double *values, int32_t *slots, int32_t capacity);
/* the slot of a resident unit, -1 when it is not resident */
int infllm_cache_slot_of(void *cache, int32_t unit);
/* a second policy object in the same state / bring dst (same capacity and strategy) into the state of src:
 * what a caller needs to try a selection out before it is final (see infllm_block_prefetch) */
void *infllm_cache_clone(const void *src);
int infllm_cache_copy(void *dst, const void *src);

/* Selection -> policy -> fetch in one native call (replaces a host loop between infllm_layer_wait_topk and
 * infllm_block_fetch): runs infllm_cache_touch for every batch row, fills the lists infllm_block_back takes and
 * issues the fetch.  Returns the number of misses (>= 0) or an error (< 0). */
typedef struct {
    void *const *caches;                              /* [B] */
    const int32_t *h_selected;                        /* host [B,n_sel] unit ids (e.g. the pinned top-k ids) */
    int32_t n_sel;
    int32_t wait_topk;                                /* != 0: infllm_layer_wait_topk first, then read h_selected */
    /* host arena of the units: unit u of batch row b is at h_chunk_base[u / units_per_chunk]
     * + (u % units_per_chunk) * unit_bytes + b * row_bytes (device-visible addresses of pinned memory) */
    const uint64_t *h_chunk_base;
    int32_t n_chunks, units_per_chunk;
    int64_t unit_bytes, row_bytes;
    int32_t *h_sel_slots;                             /* out [B,n_sel] */
    int32_t *h_miss_row, *h_miss_slot, *h_miss_unit;  /* out [<= B*n_sel] */
    const void **h_miss_src;                          /* out [<= B*n_sel] */
    int32_t *h_evicted;                               /* out, optional: [B,n_sel], row b holds h_n_evicted[b] ids */
    int32_t *h_n_evicted, *h_n_miss;                  /* out, optional: [B] */
} infllm_select_args;
int infllm_block_select(void *layer, const infllm_select_args *a, void *stream, void *copy_stream);
/* The ids the last infllm_block_select worked on ([B, n_sel], the order it read them in), from the library's own
 * copy: the pinned ids themselves are overwritten by the next selection as soon as infllm_block_back has been
 * enqueued, so a caller that wants them afterwards (the lru-s scores of `selected_block`, context_manager.py:529-543;
 * traces) reads them here.  Returns the number of ids written (<= capacity) or an error (< 0). */
int infllm_layer_last_selection(void *layer, int32_t *ids, int32_t capacity);
/* The fetch ahead of the selection.  infllm_block_front ranks the units that exist before its block for the NEXT
 * block already (the selection proper, late in infllm_block_back, only weighs these candidates against the units
 * carved in between) and publishes them to the host.  Called after infllm_block_back, this runs the residency
 * policy for the candidates on a copy of the policy objects and starts the fetch of their misses, a block's length
 * before the selection is final, so that the transfer is no longer part of the chain selection -> fetch -> global
 * stage -> next selection.  The next infllm_block_select settles it: when the selection equals the candidates
 * (all but the blocks in which a freshly carved unit makes the top-k) the copy becomes the policy state, the lists
 * and the return value are what the call would have produced, and nothing is left to fetch; otherwise the copy is
 * dropped and the call proceeds from the untouched state, except that a missed unit which the guess has moved
 * already takes the slot it was moved to where that slot is free (infllm_cache_touch_hinted), so that only the other
 * misses are fetched, together with the residents whose slots the guess overwrote.  The hit / miss / eviction
 * sequence is therefore the reference's either way; which slot a unit occupies may differ from a run without guesses.
 * No guess is made (return 0) when no candidates are pending, when the policy would evict a unit of the
 * selection whose global stage may still be running, or when the DMA engines are not in use (beside the block's
 * own kernels the fetch kernel costs more than the shorter chain gains; INFLLM_FETCH_AHEAD_ALWAYS=1 guesses anyway).  Valid only for policies whose state does not change between
 * this call and the selection (lru, fifo: the lru-s scores arrive with the block's attention mass).
 * `a` as for infllm_block_select (h_selected, wait_topk and the output lists are not used).  Returns the number of
 * units whose fetch was started (>= 0) or an error (< 0).  A guess still open at infllm_layer_flush is undone there. */
int infllm_block_prefetch(void *layer, const infllm_select_args *a, void *stream, void *copy_stream);
/* how many guesses were made / turned out to be the selection */
int infllm_layer_prefetch_stats(void *layer, int64_t *issued, int64_t *confirmed);
/* Missed units that were served from a carve staging slot so far (a device-to-device copy on the main stream instead
 * of a transfer from pinned host memory; MemoryUnit.load, context_manager.py:76-91, for a unit whose gather into
 * staging is at most four carving blocks old).  INFLLM_NO_STAGING_COPY=1 (read by infllm_layer_create) turns it off. */
int64_t infllm_layer_staged_units(void *layer);
/* Which of two interchangeable paths the blocks of this layer took so far (for tests that compare the paths): counts[0]
 * page tables of the global stage (get_global_hidden_and_mask, context_manager.py:386-451) carried in the stage's own
 * launch, [1] written to device memory by the table kernel, [2] uploaded from the host; [3] merges of a block's partial
 * outputs (torch_impl.py:15-36) carried by the block's local-score launch, [4] launched on their own in a block whose
 * order of launches allowed the carried form; [5] selections ranked from the lists of a prepared call
 * (infllm_front_args.d_call_scores) instead of a pass over all units.  INFLLM_PAGE_TABLE_KERNEL=1,
 * INFLLM_SCORE_MERGE_APART=1 and INFLLM_NO_CALL_LISTS=1, read by infllm_layer_create, move blocks from [0] to [1],
 * from [3] to [4] and out of [5]. */
int infllm_layer_path_counts(void *layer, int64_t *counts /* [6] */);
/* Units moved from pinned host memory to the slab so far, whichever way (DMA engines or the fetch kernel): the misses
 * of the selections, the candidates a guess fetched that were not selected after all, and what a wrong guess's
 * repair brought back - the host-to-device traffic of MemoryUnit.load (context_manager.py:76-91) in units. */
int64_t infllm_layer_fetched_units(void *layer);

/* Event timing of the two attention stages (for benchmarks): enable with a record
 * capacity and a stride (every stride-th launch of each stage is bracketed by two events; an event pair
 * costs the stream several microseconds, so a throughput run samples), read back (which: 0 local stage,
 * 1 global stage, 2 the main stream's wait for the fetch in infllm_block_back); the read waits for launches
 * that are still running.
 * ms[i] is the launch-to-finish time of one stage launch, n_queries[i] its block size,
 * n_keys[i] the key rows its source held. */
int infllm_layer_timing(void *layer, int32_t capacity, int32_t stride);
int infllm_layer_read_timing(void *layer, int32_t which, float *ms, int32_t *n_queries, int32_t *n_keys,
                             int32_t capacity);

#ifdef __cplusplus
}
#endif
#endif /* INFLLM_HIP_H */
