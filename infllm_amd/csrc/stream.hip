// One execution block of the streaming path in a few native calls
// (inf_llm/attention/context_manager.py:474-545, 614-679): front (local stage, the next block's prologue and
// candidates), select (selection -> residency policy -> fetch), back (global stage, merge, scores, new units) and,
// optionally, prefetch (the next block's fetch from its candidates, settled by the next select).  The launches of a
// block are issued back to back so that the host interpreter is not on the GPU's critical path; missed units and
// carved units travel through the DMA engines (ROCr), ordered by the host and by a flag the stream waits on.
// What is carved when stays with the caller; the residency policy is infllm_cache_* (cache.hip).
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <utility>
#include <vector>

#include <hsa/hsa.h>
#include <hsa/hsa_ext_amd.h>

#include "common.h"

namespace {

struct StageTimer {
    std::vector<hipEvent_t> ev;       // pairs
    std::vector<int> n_queries, n_keys;
    int used = 0;
    int seen = 0;                     // launches since timing was enabled
};

struct Layer {
    infllm_layer_desc d;
    hipEvent_t topk_done = nullptr;       // indices of the last front() are in pinned memory
    hipEvent_t global_done = nullptr;     // last global stage has read the slab
    hipEvent_t fetch_done = nullptr;      // missed units are in their slots
    hipEvent_t carve_ready = nullptr;     // carve staging filled
    std::vector<hipEvent_t> page_evt, carve_evt;
    std::vector<char> page_busy, carve_busy;
    std::vector<void *> fetch_dst;
    hipStream_t copy_stream = nullptr;
    bool fetch_issued = false;            // infllm_block_fetch ran for the block in flight
    bool fetch_wait = false;              // the main stream still has to wait for fetch_done
    // device-to-host copy of the units carved by the previous block: issued on the copy stream
    // right AFTER the next block's fetch, so that it never delays a fetch
    struct Offload {
        bool pending = false;
        int slot = 0, first_unit = 0, count = 0;
        std::vector<void *> dst;
        // how the host learns that the copy into staging has finished: the selection kernel launched behind it has
        // published its sequence number (after_seq != 0), or the event carve_ready (has_event)
        int32_t after_seq = 0;
        bool has_event = false;
    } off;
    int32_t seen_seq = 0;                 // last selection sequence number the host has read
    hipStream_t main_stream = nullptr;    // of the last infllm_block_front / infllm_block_back
    bool main_stream_known = false;
    // The same copy through the DMA engine (see issue_offload_dma): agents of this layer's GPU and of the host,
    // one completion signal per carve staging slot, and which units a slot's copy in flight carries
    bool dma_ok = false;
    hsa_agent_t dma_gpu{}, dma_cpu{};
    std::vector<hsa_signal_t> dma_sig;
    std::vector<char> dma_busy;
    std::vector<int> dma_first, dma_count;
    // The fetch of missed units through several DMA engines (see fetch_by_engines): engines, the signal the unit
    // copies count down, a 4-byte flag in signal memory that the main stream waits on and the engines write last,
    // its pinned source values, and the sequence number of the fetch in flight.
    bool efetch_ok = false;
    std::vector<uint32_t> efetch_engines;
    hsa_signal_t efetch_sig[2]{}, efetch_flag_sig[2]{};   // two sets, used in turn: a fetch may be issued while the one before is in flight
    bool efetch_prev_in_use = false;                   // the last fetch wrote only slots of the selection in use
    uint32_t *d_efetch_flag = nullptr, *h_efetch_val = nullptr;
    int efetch_dev = 0;
    uint32_t off_engine = 0;                           // the engine that takes carved units to the host (0: the runtime's choice)
    uint32_t efetch_seq = 0;
    bool efetch_wait = false;
    int cur_n = 0;                                     // queries of the block in flight
    bool guessing = false;                             // the last selection settled a fetch made ahead of it
    // The fetch ahead of the selection (see infllm_block_prefetch): the candidates' host copy with the sequence number
    // the kernel publishes behind them, the selection whose global stage may still be running, and the guess in flight.
    int32_t *h_cand = nullptr;                         // pinned 2 x [B*topk + 1]: two lists may be on their way at a time
    int32_t cand_seq = 0;
    struct CandPub {
        int64_t b0 = -1;                               // first position of the block the list is for, -1: none
        int32_t seq = 0;                               // what the kernel stores behind the list
    } cand_pub[2];
    int cand_next = 0;                                 // the buffer the next list goes to
    int64_t next_b0 = -1;                              // first position after the block whose second half was enqueued last
    std::vector<int32_t> last_sel;                     // [B, last_n_sel]
    int last_n_sel = 0;
    struct Ahead {
        bool active = false;
        int n_sel = 0, n_miss_all = 0;
        std::vector<void *> shadow;                    // [B] policy state after the guessed selection
        std::vector<int32_t> cand, sel_slots;          // [B, n_sel]
        std::vector<int32_t> miss_row, miss_slot, miss_unit;
        std::vector<const void *> miss_src;
        std::vector<int32_t> evicted, n_evicted, n_miss;             // [B, n_sel], [B], [B]
        std::vector<int32_t> victim_row, victim_unit, victim_slot;   // residents whose slots the guess overwrote
        std::vector<const void *> victim_src;
    } ahead;
    int64_t ahead_issued = 0, ahead_confirmed = 0;
    bool ahead_any_path = false;                       // guess also when the fetch kernel has to move the units
    int page_cur = 0, carve_cur = 0;
    // which units each staging slot of the carve holds (the launch that fills it is in the main stream's queue or done):
    // a missed unit that is still there is copied from there, device to device, instead of coming back over PCIe
    std::vector<int> stage_first, stage_count;
    hipEvent_t stage_copied = nullptr;                 // behind the last such copy
    std::vector<int64_t> stage_copy_dst;               // slots (row * max_cached + slot) such copies may still be on their way to
    bool stage_copy_ok = true;                         // INFLLM_NO_STAGING_COPY=1: every missed unit comes from the host
    bool page_table_kernel = false;                    // INFLLM_PAGE_TABLE_KERNEL=1: short page tables are written by a kernel too
    bool score_merge_apart = false;                    // INFLLM_SCORE_MERGE_APART=1: the merge never rides in the score launch
    // which of those paths the blocks took (infllm_layer_path_counts): page tables carried by the launch / written by
    // the kernel / uploaded; merges carried by the score launch / launched on their own in a block that could carry one
    int64_t n_tables_inline = 0, n_tables_kernel = 0, n_tables_upload = 0, n_score_merged = 0, n_score_apart = 0;
    int64_t staged_units = 0;                          // missed units served from a staging slot so far
    int64_t fetched_units = 0;                         // units moved from pinned host memory so far (guessed ones and repairs included)
    hipEvent_t mass_done = nullptr;
    bool mass_pending = false;
    int32_t topk_seq = 0;
    hipStream_t topk_stream = nullptr;    // stream of the last selection (to fall back on when the poll gives up)
    // the top-k of the units that existed when the next block was prepared, chosen ahead of the chain: [B,topk]
    // device ids (this handle's own allocation) and the unit count they were chosen from (-1: none)
    int32_t *d_cand = nullptr;
    int cand_units = -1;
    int scored_units = -1;                // block_front scored units [0, scored_units) under the next block's mean query (-1: none)
    // Lists made once per prepared call (infllm_front_args.d_call_scores): for every block of the call the k best of
    // the units that existed when the call began (d_base: [kMaxCallBlocks, B, topk], this handle's allocation) and
    // those units' scores under the block's mean query (the caller's buffer).  While call_lists is set, a block's
    // selection and the next block's candidates are ranked from them (run_call_rank).
    int32_t *d_base = nullptr;
    bool call_lists = false, no_call_lists = false;    // INFLLM_NO_CALL_LISTS=1 turns them off
    bool call_lists_pending = false;                   // the call in flight wants them: its first block's second half makes them
    int call_room = 0;                                 // entries a ranking takes (INFLLM_CALL_LISTS_ROOM lowers it: the rest of
                                                       // such a call goes back to selections over all units)
    int call_n0 = 0, call_blocks = 0;
    float *call_scores = nullptr;
    int64_t call_cols = 0;
    int64_t n_call_ranked = 0;
    bool has_global = false;
    bool global_unmarked = false;         // the last global stage ran without recording global_done (see block_back)
    hipEvent_t idle_main = nullptr, idle_copy = nullptr;      // recorded by layer_flush: this layer's work up to there
    bool idle_recorded = false;
    bool unflushed = false;               // work was enqueued since the last layer_flush (a call that ended half way)
    hipStream_t last_copy_stream = nullptr;
    // where the carving stood after the last block (rows from there on are still needed): infllm_call_front checks
    // the rings' room against it
    bool cursor_known = false;
    int64_t cursor = 0;
    bool topk_pending = false;
    int slot = 0;                         // workspace slot written last
    // Where a block's rotated queries, mean query and (when its local stage already ran) local partials are: a slot of
    // the per-block workspaces, or a slice of the buffers of a call that was prepared in one go (infllm_call_front).
    struct QView {
        const bf16_t *q_loc = nullptr, *q_glb = nullptr;
        int64_t q_sh = 0, q_sb = 0;
        const float *qbar = nullptr;
        bool batched = false;
        const uint16_t *o_loc = nullptr;   // batched: the block's local partials [nsplit, B, H, n, 128] and log-sum-exps
        const float *lse_loc = nullptr;
        int nsplit = 0;
    };
    QView fresh;                          // the block whose prologue ran last
    QView cur;                            // the block between front() and back()
    infllm_batch_desc bd{};               // buffers for calls prepared in one go
    bool batch_ok = false;
    bool batch_live = false;              // a prepared call whose blocks are being worked off
    int64_t batch_b0 = 0;
    int batch_n = 0, batch_nsplit = 0;
    int64_t batch_block_rows = 0;
    bool batch_retrieved = false;         // the first block's retrieval was launched by infllm_call_front
    int batch_group = 1;                  // blocks per local-stage launch of the prepared call
    int batch_regions = 1;                // block-sized regions of the partial rows, used in turn (a multiple of the group)
    bool prepared = false;                // the next block's prologue already ran
    int64_t prepared_b0 = 0;
    int prepared_n = 0;
    int timing_cap = 0, timing_stride = 1;
    StageTimer timer[3];               // local stage, global stage, the main stream's wait for the fetch
};

#define HIP_OK(call, what)                                                              \
    do {                                                                                \
        hipError_t e_ = (call);                                                         \
        if (e_ != hipSuccess) return infllm_fail(-2, "%s: %s", what, hipGetErrorString(e_)); \
    } while (0)

// out[b, i] = sum of the `count` floats at scratch[(b * n_sel + i) * count ...]: the attention mass of one selected unit
// (context_manager.py:457-460: sum over the unit's tokens, then over the heads)
__global__ __launch_bounds__(256) void unit_mass_kernel(const float *scratch, int count, float *out) {
    __shared__ float red[4];
    const int idx = blockIdx.y * gridDim.x + blockIdx.x;
    const float *src = scratch + (int64_t)idx * count;
    float acc = 0.f;
    for (int e = threadIdx.x; e < count; e += 256) acc += src[e];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) out[idx] = (red[0] + red[1]) + (red[2] + red[3]);
}

}  // namespace
int infllm_topk_publish(const float *d_scores, int32_t N, int32_t k, int32_t *d_idx, int32_t *d_flag, int32_t flag_value, void *stream);
int infllm_call_rank(const CallRankJob *job, int32_t C, int32_t n_wgs, void *stream);
int infllm_call_rank_room();
constexpr int kMaxCallBlocks = 16;
int infllm_retrieve_fused(const void *d_reps, int64_t rep_stride, int32_t N, int32_t C, const float *d_qbar, int32_t k, float *d_scores,
                          int32_t *d_idx, int32_t *d_idx2, int32_t *d_flag, int32_t flag_value, void *stream);
int infllm_inline_page_limit();
int infllm_copy_units(const void *const *d_src, void *const *d_dst, int32_t n, int64_t nbytes, void *stream);
int infllm_merge_job(const uint16_t *d_o_part, const float *d_lse_part, int32_t P1, const uint16_t *d_o_part2, const float *d_lse_part2,
                     int32_t P2, int32_t B, int32_t H, int32_t Lq, void *d_out, int64_t o_sb, int64_t o_sh, int64_t o_sl, float *d_lse,
                     MergeJob *job);
int infllm_local_score_merged(const infllm_score_args *a, const MergeJob *job, void *stream);
int infllm_attn_stage_blocked(const infllm_attn_args *a, int32_t exc, int64_t block_rows, void *stream);
int infllm_attn_merge2(const uint16_t *d_o_part, const float *d_lse_part, int32_t P1, const uint16_t *d_o_part2, const float *d_lse_part2,
                       int32_t P2, int32_t B, int32_t H, int32_t Lq, void *d_out, int64_t o_sb, int64_t o_sh, int64_t o_sl, float *d_lse,
                       void *stream);
int infllm_reduce_partials_blocks(const float *d_parts, int32_t B, int32_t n, int32_t exc, int32_t C, float *d_out, void *stream);
int infllm_attn_paged_inline(const infllm_attn_args *local, const infllm_attn_args *global, const infllm_page *h_pages, void *stream);
int infllm_score_new_rank(const void *d_reps, int64_t rep_stride, int32_t C, const float *d_qbar, float *d_scores, const int32_t *d_cand,
                          int32_t n_cand, int32_t first_new, int32_t n_new, int32_t k, int32_t *d_idx, int32_t *d_flag,
                          int32_t flag_value, void *stream);
int infllm_repr_keys_carve(const float *d_ring_score, const void *d_ring_k_raw, int64_t ring_cap, int32_t B, int32_t H, int32_t Hkv,
                           int64_t t0, int32_t bs, int32_t n_units, int32_t repr_topk, void *d_rep_out, int64_t rep_sb, int64_t rep_su,
                           int32_t *d_idx_out, const void *d_ring_v, void *d_out_k, void *d_out_v, int64_t out_sb, int64_t out_su,
                           int64_t out_sh, void *stream);
int infllm_topk_publish_pair(const float *d_scores, int32_t N, int32_t k, int32_t *d_idx, int32_t *d_idx2, int32_t *d_flag,
                             int32_t flag_value, void *stream);
int infllm_gather_rows_pair(const void *d_ring_a, void *d_out_a, const void *d_ring_b, void *d_out_b, int64_t ring_cap, int32_t B,
                            int32_t Hkv, int64_t t0, int32_t n, int32_t unit_rows, int64_t out_sb, int64_t out_su, int64_t out_sh,
                            void *stream);
int infllm_topk_merge_publish(const float *d_scores, const int32_t *d_cand, int32_t n_cand, int32_t first_new, int32_t n_new, int32_t k,
                              int32_t *d_idx, int32_t *d_flag, int32_t flag_value, void *stream);
namespace {

int splits_for(const infllm_layer_desc &d, int n_queries, int n_tiles) {
    const int G = d.H / d.Hkv;
    const int wgs = (((n_queries + 31) / 32) * G + 7) / 8 * d.Hkv * d.B;      // 8 wave tasks per workgroup
    int want = (d.num_cus + wgs - 1) / wgs;                                      // one workgroup per CU (LDS bound)
    int cap = n_tiles / 8, limit = d.max_splits;
    if (n_queries <= 32) {
        // decode-sized blocks: the stage is a read of K/V, bound by how many workgroups pull on HBM at once, so a
        // workgroup may get as little as one tile pair; the partials still fit: 2 * limit * n_queries rows of the
        // 2 * max_splits * exc the caller allocated
        cap = n_tiles / 2;
        const int room = d.max_splits * d.exc / n_queries;
        limit = room < 32 ? room : 32;
    }
    int s = want < limit ? want : limit;
    if (s > cap) s = cap;
    return s < 1 ? 1 : s;
}

// ---- page table built on the device from the slot list (no host staging, no copy in the chain)
constexpr int kPageJobSlots = 64;
struct PageJob {
    int32_t B, Hkv, bs, max_cached, n_sel, init_len;
    int32_t n_unit_pages, n_init_pages, n_pages;
    int64_t cursor, overflow_end, ring_cap, init_cap;
    const bf16_t *slab, *init_kv, *ring_k, *ring_v;
    int32_t slots[kPageJobSlots];
};

__global__ __launch_bounds__(64) void build_pages_kernel(PageJob j, infllm_page *out) {
    const int p = blockIdx.x * 64 + threadIdx.x, u = blockIdx.y;
    if (p >= j.n_pages) return;
    const int64_t unit_elems = (int64_t)j.Hkv * j.bs * kD;
    infllm_page pg;
    pg.reserved = 0;
    if (p < j.n_unit_pages) {
        const int tpu = (j.bs + kTile - 1) / kTile;
        const int s = p / tpu, t0 = (p % tpu) * kTile;
        const bf16_t *kb = j.slab + ((int64_t)u * j.max_cached + j.slots[u * j.n_sel + s]) * 2 * unit_elems;
        pg.k = kb + (int64_t)t0 * kD;
        pg.v = kb + unit_elems + (int64_t)t0 * kD;
        pg.head_stride = (int64_t)j.bs * kD;
        pg.n_valid = j.bs - t0 < kTile ? j.bs - t0 : kTile;
    } else if (p < j.n_unit_pages + j.n_init_pages) {
        const int t0 = (p - j.n_unit_pages) * kTile;
        const bf16_t *ik = j.init_kv + (int64_t)u * 2 * j.Hkv * j.init_cap * kD;
        pg.k = ik + (int64_t)t0 * kD;
        pg.v = ik + (int64_t)j.Hkv * j.init_cap * kD + (int64_t)t0 * kD;
        pg.head_stride = j.init_cap * kD;
        pg.n_valid = j.init_len - t0 < kTile ? j.init_len - t0 : kTile;
    } else {
        const int want = p - j.n_unit_pages - j.n_init_pages;
        int64_t pos = j.cursor, len = 0;
        for (int i = 0; i <= want; ++i) {          // runs of <= 64 rows that do not cross the end of the ring
            pos += len;
            len = j.overflow_end - pos;
            if (len > kTile) len = kTile;
            const int64_t row = pos % j.ring_cap;
            if (len > j.ring_cap - row) len = j.ring_cap - row;
        }
        const int64_t row = pos % j.ring_cap;
        pg.k = j.ring_k + ((int64_t)u * j.Hkv * j.ring_cap + row) * kD;
        pg.v = j.ring_v + ((int64_t)u * j.Hkv * j.ring_cap + row) * kD;
        pg.head_stride = j.ring_cap * kD;
        pg.n_valid = (int)len;
    }
    out[(int64_t)u * j.n_pages + p] = pg;
}

// ---- the DMA engine for the device-to-host copy of carved units
// hipMemcpyAsync may run a 2 MiB device-to-host copy as a shader kernel.  Its writes leave through the L2, and
// every kernel that ends while they drain over PCIe waits for them in its end-of-kernel cache write-back: the kernels
// of the block chain stretched by the length of the copy.  The ROCr copy below goes through the SDMA engine, which
// reads HBM and writes host memory without the shader caches.  It is ordered by the host instead of by a stream:
// it is issued only once the gather kernels that fill the staging slot have finished (event query), and its
// completion signal is checked before the slot is written again or a fetch reads the units from the host.
hsa_status_t collect_agent(hsa_agent_t a, void *data) {
    ((std::vector<hsa_agent_t> *)data)->push_back(a);
    return HSA_STATUS_SUCCESS;
}

// Agents for the current HIP device: matched by PCI address; false when ROCr cannot be used (the stream-ordered
// hipMemcpyAsync path is then the only one).  INFLLM_NO_DMA_ENGINE=1 in the environment turns the engine path off.
bool dma_find_agents(hsa_agent_t *gpu, hsa_agent_t *cpu) {
    const char *off = getenv("INFLLM_NO_DMA_ENGINE");
    if (off && off[0] && off[0] != '0') return false;
    if (hsa_init() != HSA_STATUS_SUCCESS) return false;            // reference counted: the HIP runtime holds it already
    std::vector<hsa_agent_t> all;
    if (hsa_iterate_agents(collect_agent, &all) != HSA_STATUS_SUCCESS) return false;
    int dev = 0, bus = -1, devid = -1, domain = -1;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    (void)hipDeviceGetAttribute(&bus, hipDeviceAttributePciBusId, dev);
    (void)hipDeviceGetAttribute(&devid, hipDeviceAttributePciDeviceId, dev);
    (void)hipDeviceGetAttribute(&domain, hipDeviceAttributePciDomainID, dev);
    bool have_cpu = false, have_gpu = false;
    int n_gpu = 0;
    hsa_agent_t only_gpu{};
    for (hsa_agent_t a : all) {
        hsa_device_type_t type;
        if (hsa_agent_get_info(a, HSA_AGENT_INFO_DEVICE, &type) != HSA_STATUS_SUCCESS) continue;
        if (type == HSA_DEVICE_TYPE_CPU && !have_cpu) {
            *cpu = a;
            have_cpu = true;
        } else if (type == HSA_DEVICE_TYPE_GPU) {
            ++n_gpu;
            only_gpu = a;
            uint32_t bdf = 0, dom = 0;
            if (hsa_agent_get_info(a, (hsa_agent_info_t)HSA_AMD_AGENT_INFO_BDFID, &bdf) != HSA_STATUS_SUCCESS) continue;
            if (hsa_agent_get_info(a, (hsa_agent_info_t)HSA_AMD_AGENT_INFO_DOMAIN, &dom) != HSA_STATUS_SUCCESS) continue;
            if (!have_gpu && (int)((bdf >> 8) & 0xff) == bus && (int)((bdf >> 3) & 0x1f) == devid && (int)dom == domain) {
                *gpu = a;
                have_gpu = true;
            }
        }
    }
    if (!have_gpu && n_gpu == 1) {
        *gpu = only_gpu;
        have_gpu = true;
    }
    return have_cpu && have_gpu;
}

// wait (bounded) until the engine copy out of staging slot `slot` has completed
int dma_wait_slot(Layer *L, int slot, const char *what) {
    if (!L->dma_busy[slot]) return 0;
    const auto t0 = std::chrono::steady_clock::now();
    while (hsa_signal_load_scacquire(L->dma_sig[slot]) > 0) {
        if (std::chrono::steady_clock::now() - t0 > std::chrono::seconds(10))
            return infllm_fail(-2, "%s: the DMA engine copy of carved units did not complete within 10 s", what);
    }
    L->dma_busy[slot] = 0;
    return 0;
}

// Has the copy of the pending units into their staging slot finished?  1 yes, 0 not yet, < 0 error.
int carve_copied(Layer *L) {
    if (L->off.has_event) {
        const hipError_t q = hipEventQuery(L->carve_ready);
        if (q == hipErrorNotReady) {
            (void)hipGetLastError();               // "not ready" is an answer, not a failure of a later launch
            return 0;
        }
        if (q != hipSuccess) return infllm_fail(-2, "offload: %s", hipGetErrorString(q));
        return 1;
    }
    if (L->off.after_seq == 0) return 1;           // nothing was launched
    if (L->seen_seq - L->off.after_seq >= 0) return 1;
    const volatile int32_t *flag = L->d.h_topk_flag;
    return flag && *flag - L->off.after_seq >= 0 ? 1 : 0;
}

// an event for it after all (recorded late it covers more than the copy, which is harmless)
int carve_event(Layer *L) {
    if (!L->off.has_event) {
        HIP_OK(hipEventRecord(L->carve_ready, L->main_stream), "offload: event");
        L->off.has_event = true;
    }
    return 0;
}

// host wait for the same
int carve_wait(Layer *L) {
    const auto t0 = std::chrono::steady_clock::now();
    for (uint32_t spins = 0; !L->off.has_event; ++spins) {
        const int c = carve_copied(L);
        if (c) return c < 0 ? c : 0;
        if ((spins & 1023u) == 1023u && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(2)) {
            const int erc = carve_event(L);
            if (erc) return erc;
        }
        __builtin_ia32_pause();
    }
    HIP_OK(hipEventSynchronize(L->carve_ready), "offload: wait for the copy into staging");
    return 0;
}

// Try to hand the pending units to the DMA engine.  Returns 1 when issued, 0 when not possible right now (the gather
// kernels have not finished, or there is no engine path), < 0 on error.
int issue_offload_dma(Layer *L) {
    if (!L->dma_ok || !L->off.pending) return 0;
    const int ready = carve_copied(L);
    if (ready <= 0) return ready;
    const infllm_layer_desc &d = L->d;
    const int slot = L->off.slot, n = L->off.count;
    int rc = dma_wait_slot(L, slot, "offload");                                  // an older copy out of the same slot
    if (rc) return rc;
    const int64_t unit_all = (int64_t)d.B * 2 * d.Hkv * d.block_size * kD;
    const bf16_t *stage = (const bf16_t *)d.d_carve_stage + (int64_t)slot * d.max_carve * unit_all;
    int runs = 0;
    for (int i = 0; i < n;) {
        int j = i + 1;
        while (j < n && (char *)L->off.dst[j] == (char *)L->off.dst[j - 1] + unit_all * sizeof(bf16_t)) ++j;
        ++runs;
        i = j;
    }
    hsa_signal_store_relaxed(L->dma_sig[slot], runs);                            // every finished copy takes one off
    int issued = 0;
    for (int i = 0; i < n;) {                    // one copy per run of units that are contiguous on the host
        int j = i + 1;
        while (j < n && (char *)L->off.dst[j] == (char *)L->off.dst[j - 1] + unit_all * sizeof(bf16_t)) ++j;
        // on the engine kept for this direction where there is one (see efetch_setup), else wherever the runtime puts it
        const size_t bytes = (size_t)(j - i) * unit_all * sizeof(bf16_t);
        const hsa_status_t hs = L->off_engine ? hsa_amd_memory_async_copy_on_engine(L->off.dst[i], L->dma_cpu, stage + (int64_t)i * unit_all, L->dma_gpu,
                                                                                    bytes, 0, nullptr, L->dma_sig[slot],
                                                                                    (hsa_amd_sdma_engine_id_t)L->off_engine, false)
                                              : hsa_amd_memory_async_copy(L->off.dst[i], L->dma_cpu, stage + (int64_t)i * unit_all, L->dma_gpu, bytes, 0,
                                                                          nullptr, L->dma_sig[slot]);
        if (hs != HSA_STATUS_SUCCESS) {
            // give the engine path up for this layer: let what was issued finish, the stream path copies the units again
            hsa_signal_subtract_relaxed(L->dma_sig[slot], runs - issued);
            L->dma_busy[slot] = issued > 0;
            rc = dma_wait_slot(L, slot, "offload");
            L->dma_ok = false;
            return rc;
        }
        ++issued;
        i = j;
    }
    L->dma_busy[slot] = 1;
    L->dma_first[slot] = L->off.first_unit;
    L->dma_count[slot] = n;
    L->off.pending = false;
    return 1;
}

// copy the pending units from their staging slot to pinned host memory on `cs` (stream ordered)
int issue_offload(Layer *L, hipStream_t cs) {
    const infllm_layer_desc &d = L->d;
    const int64_t unit_all = (int64_t)d.B * 2 * d.Hkv * d.block_size * kD;        // one unit, all batch rows
    const bf16_t *stage = (const bf16_t *)d.d_carve_stage + (int64_t)L->off.slot * d.max_carve * unit_all;
    const int erc = carve_event(L);
    if (erc) return erc;
    HIP_OK(hipStreamWaitEvent(cs, L->carve_ready, 0), "offload: wait carve");
    const int n = L->off.count;
    for (int i = 0; i < n;) {                   // one copy per run of units that are contiguous on the host
        int j = i + 1;
        while (j < n && (char *)L->off.dst[j] == (char *)L->off.dst[j - 1] + unit_all * sizeof(bf16_t)) ++j;
        HIP_OK(hipMemcpyAsync(L->off.dst[i], stage + (int64_t)i * unit_all, (size_t)(j - i) * unit_all * sizeof(bf16_t),
                              hipMemcpyDeviceToHost, cs),
               "offload: copy");
        i = j;
    }
    HIP_OK(hipEventRecord(L->carve_evt[L->off.slot], cs), "offload: event");
    L->carve_busy[L->off.slot] = 1;
    L->off.pending = false;
    return 0;
}

// ---- the fetch of missed units through the DMA engines
// A kernel that reads pinned memory keeps thousands of PCIe reads outstanding in the L2, and everything else on the
// chip runs 1.5-2x longer beside it.  The SDMA engines do not go through the shader caches: 8 of them together move
// a block's misses as fast as the kernel does (a single engine reaches half of that on 512 KiB pieces), and the
// kernels beside them run at their own speed.  Ordering: the host issues the copies (it has just seen the selection,
// so the previous global stage, the last reader of the slots, has finished - otherwise it waits for that event
// here), and the last thing the engines write is a sequence number into a flag in signal memory, on which the main
// stream waits (hipStreamWaitValue32) before the global stage.
constexpr int kEfetchEngines = 8;
constexpr int kEngineMinQueries = 64;
constexpr int kEfetchVals = 8;

int efetch_wait_signal(hsa_signal_t sig, const char *what) {
    const auto t0 = std::chrono::steady_clock::now();
    while (hsa_signal_load_scacquire(sig) > 0) {
        if (std::chrono::steady_clock::now() - t0 > std::chrono::seconds(10)) return infllm_fail(-2, "%s: DMA engine copies did not complete within 10 s", what);
    }
    return 0;
}

// every fetch issued so far has landed (flag copies included)
int efetch_wait_all(Layer *L, const char *what) {
    for (int i = 0; i < 2; ++i) {
        if (!L->efetch_flag_sig[i].handle) continue;
        const int rc = efetch_wait_signal(L->efetch_flag_sig[i], what);
        if (rc) return rc;
    }
    return 0;
}

// Flag words in signal memory are never given back to the runtime: memory of that kind that a kernel has read (the
// stream's wait is a kernel) is best not freed while the process lives, so a layer that goes away leaves its word
// to the next one on the same device.
struct FlagPool {
    std::mutex mu;
    std::vector<std::pair<int, uint32_t *>> spare;          // (device, word)
};
FlagPool &flag_pool() {
    static FlagPool *p = new FlagPool();                     // outlives static destruction order
    return *p;
}
uint32_t *flag_take(int dev) {
    {
        std::lock_guard<std::mutex> g(flag_pool().mu);
        auto &v = flag_pool().spare;
        for (size_t i = 0; i < v.size(); ++i)
            if (v[i].first == dev) {
                uint32_t *w = v[i].second;
                v.erase(v.begin() + i);
                return w;
            }
    }
    uint32_t *w = nullptr;
    if (hipExtMallocWithFlags((void **)&w, 8, hipMallocSignalMemory) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return w;
}
void flag_give(int dev, uint32_t *w) {
    std::lock_guard<std::mutex> g(flag_pool().mu);
    flag_pool().spare.emplace_back(dev, w);
}

// set the engine fetch up for this layer; on any failure the kernel fetch stays the only path
void efetch_setup(Layer *L) {
    const char *off = getenv("INFLLM_NO_DMA_FETCH");
    if (!L->dma_ok || (off && off[0] && off[0] != '0')) return;
    int dev = 0, can = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&can, hipDeviceAttributeCanUseStreamWaitValue, dev) != hipSuccess || !can) {
        (void)hipGetLastError();
        return;
    }
    uint32_t mask = 0;
    if (hsa_amd_memory_copy_engine_status(L->dma_gpu, L->dma_cpu, &mask) != HSA_STATUS_SUCCESS) return;
    // The engines of the low eight bits of the status mask are the ones that move data without getting in the way of
    // kernels (with a ninth or a tenth the block's own kernels ran 10-40 % longer, measured).  One of them is kept for
    // the carved units' way to the host: while that copy (2 MiB per block) shared an engine with the fetch, the units
    // queued behind it on that engine landed last and the whole fetch waited for them - 47.6 ms per 128K stream
    // against 44.2 with the engines apart.
    uint32_t d2h = 0;
    if (hsa_amd_memory_copy_engine_status(L->dma_cpu, L->dma_gpu, &d2h) != HSA_STATUS_SUCCESS) d2h = 0;
    std::vector<uint32_t> low;
    for (int b = 0; b < 8; ++b)
        if (mask & (1u << b)) low.push_back(1u << b);
    L->off_engine = 0;
    if (low.size() >= 4 && (d2h & low[1])) L->off_engine = low[1];      // the second one: the first is the fetch's flag engine
    for (uint32_t e : low)
        if (e != L->off_engine && (int)L->efetch_engines.size() < kEfetchEngines) L->efetch_engines.push_back(e);
    if (L->efetch_engines.size() < 2) return;
    L->efetch_dev = dev;
    if (!(L->d_efetch_flag = flag_take(dev)) || hipHostMalloc((void **)&L->h_efetch_val, kEfetchVals * sizeof(uint32_t)) != hipSuccess ||
        hsa_signal_create(0, 0, nullptr, &L->efetch_sig[0]) != HSA_STATUS_SUCCESS ||
        hsa_signal_create(0, 0, nullptr, &L->efetch_flag_sig[0]) != HSA_STATUS_SUCCESS ||
        hsa_signal_create(0, 0, nullptr, &L->efetch_sig[1]) != HSA_STATUS_SUCCESS ||
        hsa_signal_create(0, 0, nullptr, &L->efetch_flag_sig[1]) != HSA_STATUS_SUCCESS) {
        (void)hipGetLastError();
        return;
    }
    // the first copy on an engine creates its queue (milliseconds): do that here, once per process and engine
    for (int i = 0; i < kEfetchVals; ++i) L->h_efetch_val[i] = 0;
    hsa_signal_store_relaxed(L->efetch_sig[0], (hsa_signal_value_t)L->efetch_engines.size());
    int issued = 0;
    for (uint32_t e : L->efetch_engines) {
        if (hsa_amd_memory_async_copy_on_engine(L->d_efetch_flag, L->dma_gpu, L->h_efetch_val, L->dma_cpu, 4, 0, nullptr, L->efetch_sig[0],
                                                (hsa_amd_sdma_engine_id_t)e, false) != HSA_STATUS_SUCCESS)
            break;
        ++issued;
    }
    hsa_signal_subtract_relaxed(L->efetch_sig[0], (hsa_signal_value_t)(L->efetch_engines.size() - issued));
    if (efetch_wait_signal(L->efetch_sig[0], "layer_create") != 0 || issued != (int)L->efetch_engines.size()) return;
    if (L->off_engine) {                 // the same for the engine of the other direction; if it refuses, the runtime chooses
        hsa_signal_store_relaxed(L->efetch_sig[0], 1);
        if (hsa_amd_memory_async_copy_on_engine(L->h_efetch_val + (kEfetchVals - 1), L->dma_cpu, L->d_efetch_flag, L->dma_gpu, 4, 0, nullptr,
                                                L->efetch_sig[0], (hsa_amd_sdma_engine_id_t)L->off_engine, false) != HSA_STATUS_SUCCESS) {
            hsa_signal_store_relaxed(L->efetch_sig[0], 0);
            L->off_engine = 0;
        } else if (efetch_wait_signal(L->efetch_sig[0], "layer_create") != 0)
            return;
        L->h_efetch_val[kEfetchVals - 1] = 0;
    }
    L->efetch_ok = true;
}

// Returns 1 when the engines took the fetch, 0 when the caller should use the kernel, < 0 on error.
int fetch_by_engines(Layer *L, int n_miss, const void *const *srcs, int64_t nbytes, bool ahead) {
    if (!L->efetch_ok || !L->dma_ok) return 0;          // stream-ordered offloads are not ordered before the engines
    for (size_t s = 0; s < L->carve_busy.size(); ++s) {  // ... and the few that were issued (layer_flush) have to land first
        if (!L->carve_busy[s]) continue;
        HIP_OK(hipEventSynchronize(L->carve_evt[s]), "fetch: wait offload");
        L->carve_busy[s] = 0;
    }
    // slots may still be read by the previous global stage unless the host has seen a later result of the stream
    // (a fetch ahead writes no slot of the selection in use, and the stage before that has finished)
    if (!ahead && L->has_global && hipEventQuery(L->global_done) != hipSuccess) {
        (void)hipGetLastError();
        HIP_OK(hipEventSynchronize(L->global_done), "fetch: wait global");
    }
    // A fetch ahead writes no slot of the selection in use, and those are all that the fetch before it writes (unless
    // that one also put back what a wrong guess had overwritten): the two may be in flight together, each engine
    // taking its copies in the order they were issued, so the link does not idle between one fetch's landing and the
    // host's issue of the next; the host only makes sure that the fetch before the last has landed (whose signals this
    // one takes over).  Any other fetch lets everything land first.  Measured with the engines told apart (see
    // efetch_setup): 43.1-43.6 ms per 128K stream against 43.7-43.8 with one fetch at a time;
    // while the carved units' copy to the host still shared an engine with the fetch the overlap lost (the next
    // fetch's copies took bandwidth from the stragglers the stream was waiting for).
    const int set = (int)((L->efetch_seq + 1) & 1u);
    int rc = ahead && L->efetch_prev_in_use ? efetch_wait_signal(L->efetch_flag_sig[set], "fetch") : efetch_wait_all(L, "fetch");
    if (rc) return rc;
    const uint32_t seq = ++L->efetch_seq;
    uint32_t *val = L->h_efetch_val + (seq % (kEfetchVals - 1));
    *val = seq;
    hsa_signal_t sig = L->efetch_sig[set], flag_sig = L->efetch_flag_sig[set];
    hsa_signal_store_relaxed(sig, n_miss);
    hsa_signal_store_relaxed(flag_sig, 1);
    int issued = 0;
    bool ok = true;
    for (int i = 0; i < n_miss && ok; ++i) {
        ok = hsa_amd_memory_async_copy_on_engine(L->fetch_dst[i], L->dma_gpu, srcs[i], L->dma_cpu, (size_t)nbytes, 0, nullptr, sig,
                                                 (hsa_amd_sdma_engine_id_t)L->efetch_engines[i % L->efetch_engines.size()], false) ==
             HSA_STATUS_SUCCESS;
        issued += ok ? 1 : 0;
    }
    // the sequence number goes out behind the units, on the engine that wrote the one before: the flag never steps back
    if (ok)
        ok = hsa_amd_memory_async_copy_on_engine(L->d_efetch_flag, L->dma_gpu, val, L->dma_cpu, 4, 1, &sig, flag_sig,
                                                 (hsa_amd_sdma_engine_id_t)L->efetch_engines[0], false) == HSA_STATUS_SUCCESS;
    if (!ok) {
        // give the engine path up: let what was issued land, then the kernel copies everything again
        hsa_signal_subtract_relaxed(sig, n_miss - issued);
        hsa_signal_store_relaxed(flag_sig, 0);
        rc = efetch_wait_signal(sig, "fetch");
        if (!rc) rc = efetch_wait_all(L, "fetch");
        L->efetch_ok = false;
        --L->efetch_seq;
        return rc;
    }
    L->efetch_wait = true;
    L->efetch_prev_in_use = true;
    return 1;
}

// missed units -> their slab slots on the copy stream; then the pending offload (never ahead of a fetch
// unless the fetch needs one of the units that are still on their way to the host)
int do_fetch(Layer *L, int n_miss, const int32_t *rows, const int32_t *slots, const int32_t *units, const void *const *srcs,
             hipStream_t st, hipStream_t cs, bool ahead = false) {
    const infllm_layer_desc &d = L->d;
    const bool side = cs != st;
    L->unflushed = true;
    L->last_copy_stream = cs;
    const int64_t slot_elems = 2 * (int64_t)d.Hkv * d.block_size * kD;
    // A unit carved a few blocks ago is still in the staging slot it was gathered into (the launch that filled it is
    // ahead of this point in the main stream): it is copied from there.  A unit that makes a selection right after it
    // was carved - which is when a guessed selection turns out wrong - would otherwise have to wait for its own way
    // to the host to end before it could come back.
    std::vector<int32_t> rows_k, slots_k, units_k;
    std::vector<const void *> srcs_k;
    if (n_miss > 0) {
        INFLLM_REQUIRE(rows && slots && units && srcs, "fetch: null miss list");
        // slots that an earlier copy out of staging may still be on its way to: a fetch that is not ordered by the
        // main stream (engines, copy stream) lets it land before it writes one of them again
        if (!L->stage_copy_dst.empty()) {
            const hipError_t q = hipEventQuery(L->stage_copied);
            if (q == hipSuccess)
                L->stage_copy_dst.clear();
            else {
                (void)hipGetLastError();
                bool hit = false;
                for (int i = 0; i < n_miss && !hit; ++i)
                    for (int64_t dst : L->stage_copy_dst) hit = hit || dst == (int64_t)rows[i] * d.max_cached + slots[i];
                if (hit) {
                    HIP_OK(hipEventSynchronize(L->stage_copied), "fetch: wait staging copy");
                    L->stage_copy_dst.clear();
                }
            }
        }
        hipStream_t ms = L->main_stream_known ? L->main_stream : st;       // the stream the staging slots are filled on
        std::vector<char> staged(n_miss, 0);
        std::vector<const void *> st_src;
        std::vector<void *> st_dst;
        int n_staged = 0;
        const int64_t unit_all = (int64_t)d.B * slot_elems;
        for (int i = 0; i < n_miss; ++i) {
            int at = -1;
            for (size_t sl = 0; L->stage_copy_ok && sl < L->stage_count.size() && at < 0; ++sl)
                if (units[i] >= L->stage_first[sl] && units[i] < L->stage_first[sl] + L->stage_count[sl]) at = (int)sl;
            if (at < 0) continue;
            INFLLM_REQUIRE(rows[i] >= 0 && rows[i] < d.B && slots[i] >= 0 && slots[i] < d.max_cached, "fetch: bad miss entry");
            if (n_staged == 0) {
                // an earlier fetch may still be on its way to the same slot (a guess that turned out wrong put another
                // unit there; a repair put back one that is evicted again): it lands first
                if (L->efetch_ok) {
                    const int wrc = efetch_wait_all(L, "fetch");
                    if (wrc) return wrc;
                }
                if (L->fetch_wait && ms != cs) HIP_OK(hipStreamWaitEvent(ms, L->fetch_done, 0), "fetch: wait fetch");
            }
            const bf16_t *src = (const bf16_t *)d.d_carve_stage + ((int64_t)at * d.max_carve + (units[i] - L->stage_first[at])) * unit_all +
                                (int64_t)rows[i] * slot_elems;
            bf16_t *dst = (bf16_t *)d.d_slab + ((int64_t)rows[i] * d.max_cached + slots[i]) * slot_elems;
            st_src.push_back(src);
            st_dst.push_back(dst);
            L->stage_copy_dst.push_back((int64_t)rows[i] * d.max_cached + slots[i]);
            staged[i] = 1;
            ++n_staged;
            ++L->staged_units;
        }
        if (n_staged > 0) {
            const int crc = infllm_copy_units(st_src.data(), st_dst.data(), n_staged, slot_elems * (int64_t)sizeof(bf16_t), ms);      // one launch for all
            if (crc) return crc;
            HIP_OK(hipEventRecord(L->stage_copied, ms), "fetch: event");
            for (int i = 0; i < n_miss; ++i) {
                if (staged[i]) continue;
                rows_k.push_back(rows[i]); slots_k.push_back(slots[i]); units_k.push_back(units[i]); srcs_k.push_back(srcs[i]);
            }
            rows = rows_k.data(); slots = slots_k.data(); units = units_k.data(); srcs = srcs_k.data();
            n_miss = (int)rows_k.size();
        }
    }
    if (n_miss > 0) {
        if (L->off.pending) {
            bool hit = false;
            for (int i = 0; i < n_miss && !hit; ++i) hit = units[i] >= L->off.first_unit && units[i] < L->off.first_unit + L->off.count;
            if (hit) {
                // the DMA engines that fetch are not ordered behind `cs`: there, the units go out by the engine too
                // (waited for just below), or the host waits for the stream copy
                int orc = 0;
                if (L->efetch_ok && L->dma_ok) {
                    orc = carve_wait(L);
                    if (orc) return orc;
                    orc = issue_offload_dma(L);
                    if (orc < 0) return orc;
                }
                if (L->off.pending) {
                    orc = issue_offload(L, cs);
                    if (orc) return orc;
                    if (L->efetch_ok) HIP_OK(hipStreamSynchronize(cs), "fetch: wait offload");
                }
            }
        }
        for (size_t s = 0; s < L->dma_busy.size(); ++s) {           // units still on their way to the host by the engine
            if (!L->dma_busy[s]) continue;
            bool hit = false;
            for (int i = 0; i < n_miss && !hit; ++i) hit = units[i] >= L->dma_first[s] && units[i] < L->dma_first[s] + L->dma_count[s];
            if (hit) {
                int wrc = dma_wait_slot(L, (int)s, "fetch");
                if (wrc) return wrc;
            }
        }
        L->fetched_units += n_miss;
        L->fetch_dst.resize(n_miss);
        for (int i = 0; i < n_miss; ++i) {
            INFLLM_REQUIRE(rows[i] >= 0 && rows[i] < d.B && slots[i] >= 0 && slots[i] < d.max_cached && srcs[i], "fetch: bad miss entry");
            L->fetch_dst[i] = (bf16_t *)d.d_slab + ((int64_t)rows[i] * d.max_cached + slots[i]) * slot_elems;
        }
        // The engines pay where other kernels run beside the fetch; a short block (a decode step) has nothing to
        // run beside it, and there the fetch kernel gets the units into place a little sooner (measured).
        const int erc = ahead || L->cur_n >= kEngineMinQueries ? fetch_by_engines(L, n_miss, srcs, slot_elems * (int64_t)sizeof(bf16_t), ahead) : 0;
        if (erc < 0) return erc;
        if (erc == 0) {
            if (L->efetch_ok) {                   // engine copies of an earlier fetch may aim at the same slots
                const int wrc = efetch_wait_all(L, "fetch");
                if (wrc) return wrc;
            }
            if (side && L->has_global && !ahead) HIP_OK(hipStreamWaitEvent(cs, L->global_done, 0), "fetch: wait global");
            int frc = infllm_fetch_units(srcs, L->fetch_dst.data(), n_miss, slot_elems * (int64_t)sizeof(bf16_t), cs);
            if (frc) return frc;
            if (side) {
                HIP_OK(hipEventRecord(L->fetch_done, cs), "fetch: event");
                L->fetch_wait = true;
            }
        }
    }
    if (L->off.pending) {
        if (L->dma_ok) {                          // the engine takes it as soon as the gathers have finished (see block_back)
            const int drc = issue_offload_dma(L);
            return drc < 0 ? drc : 0;
        }
        return issue_offload(L, cs);
    }
    return 0;
}

int timer_begin(Layer *L, int which, int n_queries, int n_keys, hipStream_t st) {
    StageTimer &t = L->timer[which];
    if (L->timing_cap <= 0 || t.used >= L->timing_cap) return -1;
    if (t.seen++ % L->timing_stride) return -1;
    const int i = t.used++;
    t.n_queries[i] = n_queries;
    t.n_keys[i] = n_keys;
    (void)hipEventRecord(t.ev[2 * i], st);
    return i;
}

void timer_end(Layer *L, int which, int i, hipStream_t st) {
    if (i >= 0) (void)hipEventRecord(L->timer[which].ev[2 * i + 1], st);
}

}  // namespace

extern "C" void *infllm_layer_create(const infllm_layer_desc *desc) {
    auto bad = [](const char *m) -> void * {
        infllm_fail(-1, "layer_create: %s", m);
        return nullptr;
    };
    if (!desc) return bad("null descriptor");
    const infllm_layer_desc &d = *desc;
    if (d.B <= 0 || d.H <= 0 || d.Hkv <= 0 || d.H % d.Hkv) return bad("bad head geometry");
    if (d.exc <= 0 || d.exc > d.n_local || d.block_size <= 0 || d.topk < 0 || d.topk > d.max_cached) return bad("bad knobs");
    if (d.ring_cap % kTile || d.ring_cap < (int64_t)d.n_local + 2 * d.exc + d.block_size) return bad("ring too small or unaligned");
    if (!d.d_ring_k_raw || !d.d_ring_k_rot || !d.d_ring_v || !d.d_ring_score || !d.d_init_kv || !d.d_slab || !d.d_q_loc ||
        !d.d_q_glb || !d.d_qbar || !d.d_qpart || !d.d_o_part || !d.d_lse_part || !d.d_lse || !d.d_topk_idx || !d.d_pages ||
        !d.h_pages || !d.d_carve_stage || !d.d_inv_freq)
        return bad("null buffer");
    if (d.topk > 64) return bad("topk above 64 (the selection lists of a block are fixed 64-entry arrays)");
    if (d.max_splits < 1 || d.max_splits > 64 || d.num_cus < 1 || d.page_slots < 1 || d.carve_slots < 1 || d.max_carve < 1 ||
        d.max_pages < 1 || d.init_cap < 1)
        return bad("bad capacities");
    Layer *L = new Layer();
    L->d = d;
    bool ok = hipEventCreateWithFlags(&L->topk_done, hipEventDisableTiming) == hipSuccess &&
              hipEventCreateWithFlags(&L->global_done, hipEventDisableTiming) == hipSuccess &&
              hipEventCreateWithFlags(&L->fetch_done, hipEventDisableTiming) == hipSuccess &&
              hipEventCreateWithFlags(&L->carve_ready, hipEventDisableTiming) == hipSuccess &&
              hipEventCreateWithFlags(&L->mass_done, hipEventDisableTiming) == hipSuccess &&
              hipEventCreateWithFlags(&L->idle_main, hipEventDisableTiming) == hipSuccess &&
              hipEventCreateWithFlags(&L->idle_copy, hipEventDisableTiming) == hipSuccess &&
              hipEventCreateWithFlags(&L->stage_copied, hipEventDisableTiming) == hipSuccess;
    L->page_evt.resize(d.page_slots, nullptr);
    L->carve_evt.resize(d.carve_slots, nullptr);
    L->page_busy.assign(d.page_slots, 0);
    L->carve_busy.assign(d.carve_slots, 0);
    L->stage_first.assign(d.carve_slots, 0);
    L->stage_count.assign(d.carve_slots, 0);

    for (auto &e : L->page_evt) ok = ok && hipEventCreateWithFlags(&e, hipEventDisableTiming) == hipSuccess;
    for (auto &e : L->carve_evt) ok = ok && hipEventCreateWithFlags(&e, hipEventDisableTiming) == hipSuccess;
    if (!ok) {
        infllm_layer_destroy(L);
        return bad("hipEventCreate failed");
    }
    if (d.topk > 0 && hipMalloc((void **)&L->d_cand, sizeof(int32_t) * d.B * d.topk) != hipSuccess) {
        L->d_cand = nullptr;                        // not fatal: selections then run over all units every time
        (void)hipGetLastError();
    }
    L->dma_busy.assign(d.carve_slots, 0);
    L->dma_first.assign(d.carve_slots, 0);
    L->dma_count.assign(d.carve_slots, 0);
    if (dma_find_agents(&L->dma_gpu, &L->dma_cpu)) {
        L->dma_ok = true;
        for (int i = 0; i < d.carve_slots && L->dma_ok; ++i) {
            hsa_signal_t sig;
            if (hsa_signal_create(0, 0, nullptr, &sig) == HSA_STATUS_SUCCESS) L->dma_sig.push_back(sig);
            else L->dma_ok = false;                 // without signals the stream-ordered copy is used
        }
    }
    efetch_setup(L);
    {
        const char *any = getenv("INFLLM_FETCH_AHEAD_ALWAYS");
        L->ahead_any_path = any && any[0] && any[0] != '0';
        const char *ns = getenv("INFLLM_NO_STAGING_COPY");
        L->stage_copy_ok = !(ns && ns[0] && ns[0] != '0');
        const char *pk = getenv("INFLLM_PAGE_TABLE_KERNEL");
        L->page_table_kernel = pk && pk[0] && pk[0] != '0';
        const char *ma = getenv("INFLLM_SCORE_MERGE_APART");
        L->score_merge_apart = ma && ma[0] && ma[0] != '0';
        const char *nl = getenv("INFLLM_NO_CALL_LISTS");
        L->no_call_lists = nl && nl[0] && nl[0] != '0';
        const char *room = getenv("INFLLM_CALL_LISTS_ROOM");
        L->call_room = infllm_call_rank_room();
        if (room && atoi(room) > 0 && atoi(room) < L->call_room) L->call_room = atoi(room);
    }
    if (hipHostMalloc((void **)&L->h_cand, 2 * ((size_t)d.B * d.topk + 1) * sizeof(int32_t)) != hipSuccess) {
        (void)hipGetLastError();
        L->h_cand = nullptr;                        // no fetch ahead of the selection then
    } else
        std::memset(L->h_cand, 0, 2 * ((size_t)d.B * d.topk + 1) * sizeof(int32_t));
    if (d.topk > 0 && hipMalloc((void **)&L->d_base, sizeof(int32_t) * kMaxCallBlocks * d.B * d.topk) != hipSuccess) {
        (void)hipGetLastError();
        L->d_base = nullptr;                        // not fatal: every block's selection then runs over all units
    }
    return L;
}

extern "C" int infllm_layer_destroy(void *layer) {
    if (!layer) return 0;
    Layer *L = (Layer *)layer;
    // The caller frees the layer's buffers next: wait for the work that uses them - what layer_flush marked on the two
    // streams (every append ends with it), not for the device, which may be busy with other layers.
    // A layer destroyed between a block's calls and the flush (an append() that raised, a C caller that skipped the
    // flush) has work in flight that no such mark covers: then the two streams themselves are waited for.
    if (L->unflushed) {
        if (L->main_stream_known) (void)hipStreamSynchronize(L->main_stream);
        if (L->last_copy_stream) (void)hipStreamSynchronize(L->last_copy_stream);
        if (L->efetch_ok) (void)efetch_wait_all(L, "layer_destroy");
        (void)hipGetLastError();
    } else if (L->idle_recorded) {
        (void)hipEventSynchronize(L->idle_main);
        (void)hipEventSynchronize(L->idle_copy);
    }
    for (hipEvent_t e : {L->topk_done, L->global_done, L->fetch_done, L->carve_ready, L->mass_done, L->idle_main, L->idle_copy, L->stage_copied})
        if (e) (void)hipEventDestroy(e);
    for (hipEvent_t e : L->page_evt)
        if (e) (void)hipEventDestroy(e);
    for (hipEvent_t e : L->carve_evt)
        if (e) (void)hipEventDestroy(e);
    for (size_t i = 0; i < L->dma_sig.size(); ++i) {
        if (i < L->dma_busy.size()) (void)dma_wait_slot(L, (int)i, "layer_destroy");
        (void)hsa_signal_destroy(L->dma_sig[i]);
    }
    for (auto &t : L->timer)
        for (hipEvent_t e : t.ev)
            if (e) (void)hipEventDestroy(e);
    if (L->d_cand) (void)hipFree(L->d_cand);
    if (L->d_base) (void)hipFree(L->d_base);
    if (L->h_cand) (void)hipHostFree(L->h_cand);
    for (void *c : L->ahead.shadow)
        if (c) (void)infllm_cache_destroy(c);
    for (int i = 0; i < 2; ++i) {
        if (L->efetch_sig[i].handle) {
            (void)efetch_wait_signal(L->efetch_sig[i], "layer_destroy");
            (void)hsa_signal_destroy(L->efetch_sig[i]);
        }
        if (L->efetch_flag_sig[i].handle) {
            (void)efetch_wait_signal(L->efetch_flag_sig[i], "layer_destroy");
            (void)hsa_signal_destroy(L->efetch_flag_sig[i]);
        }
    }
    if (L->d_efetch_flag) flag_give(L->efetch_dev, L->d_efetch_flag);
    if (L->h_efetch_val) (void)hipHostFree(L->h_efetch_val);
    delete L;
    return 0;
}

extern "C" int infllm_layer_timing(void *layer, int32_t capacity, int32_t stride) {
    INFLLM_REQUIRE(layer && capacity >= 0 && stride >= 1, "layer_timing: bad arguments");
    Layer *L = (Layer *)layer;
    for (auto &t : L->timer) {
        while ((int)t.ev.size() < 2 * capacity) {
            hipEvent_t e;
            HIP_OK(hipEventCreate(&e), "layer_timing");
            t.ev.push_back(e);
        }
        t.n_queries.resize(capacity);
        t.n_keys.resize(capacity);
        t.used = 0;
        t.seen = 0;
    }
    L->timing_cap = capacity;
    L->timing_stride = stride;
    return 0;
}

extern "C" int infllm_layer_read_timing(void *layer, int32_t which, float *ms, int32_t *n_queries, int32_t *n_keys,
                                        int32_t capacity) {
    INFLLM_REQUIRE(layer && which >= 0 && which <= 2 && ms && capacity >= 0, "layer_read_timing: bad arguments");
    Layer *L = (Layer *)layer;
    StageTimer &t = L->timer[which];
    int n = t.used < capacity ? t.used : capacity;
    for (int i = 0; i < n; ++i) {
        HIP_OK(hipEventSynchronize(t.ev[2 * i + 1]), "layer_read_timing");            // no wait when the launch has finished
        HIP_OK(hipEventElapsedTime(&ms[i], t.ev[2 * i], t.ev[2 * i + 1]), "layer_read_timing");
        if (n_queries) n_queries[i] = t.n_queries[i];
        if (n_keys) n_keys[i] = t.n_keys[i];
    }
    return n;
}

namespace {

int run_ingest(Layer *L, const infllm_front_args *a, const void *q, const void *k, const void *v, int n, int64_t b0, int slot,
               bool want_mean, void *stream) {
    const infllm_layer_desc &d = L->d;
    infllm_ingest_args in{};
    in.d_q = q; in.d_k = k; in.d_v = v;
    in.q_sb = a->q_sb; in.q_sh = a->q_sh; in.q_sl = a->q_sl;
    in.k_sb = a->k_sb; in.k_sh = a->k_sh; in.k_sl = a->k_sl;
    in.v_sb = a->v_sb; in.v_sh = a->v_sh; in.v_sl = a->v_sl;
    in.B = d.B; in.H = d.H; in.Hkv = d.Hkv; in.n = n;
    in.pos0 = b0; in.glb_pos = d.n_local - 1;
    in.d_inv_freq = d.d_inv_freq; in.distance_scale = d.distance_scale;
    in.d_ring_k_raw = d.d_ring_k_raw; in.d_ring_k_rot = d.d_ring_k_rot; in.d_ring_v = d.d_ring_v;
    in.d_ring_score = d.d_ring_score; in.ring_cap = d.ring_cap;
    const int64_t qws = (int64_t)d.B * d.H * d.exc * kD;
    in.d_q_loc = (bf16_t *)d.d_q_loc + slot * qws;
    in.d_q_glb = (bf16_t *)d.d_q_glb + slot * qws;
    const int C = d.H * kD;
    float *qpart = d.d_qpart + (int64_t)slot * d.B * ((d.exc + 15) / 16) * C;
    in.d_qpart = want_mean ? qpart : nullptr;
    Layer::QView qv;
    qv.q_loc = (const bf16_t *)in.d_q_loc; qv.q_glb = (const bf16_t *)in.d_q_glb;
    qv.q_sh = (int64_t)n * kD; qv.q_sb = (int64_t)d.H * n * kD;
    qv.qbar = d.d_qbar + (int64_t)slot * d.B * C;
    L->fresh = qv;
    int rc = infllm_ingest(&in, stream);
    if (rc || !want_mean) return rc;
    return infllm_reduce_partials(qpart, d.B, (n + 15) / 16, C, 1.f / (float)n, d.d_qbar + (int64_t)slot * d.B * C, stream);
}

// a block of the call that infllm_call_front prepared?
bool block_in_batch(const Layer *L, int64_t b0, int n) {
    if (!L->batch_live || b0 < L->batch_b0 || b0 + n > L->batch_b0 + L->batch_n) return false;
    return (b0 - L->batch_b0) % L->d.exc == 0 && (n == L->d.exc || b0 + n == L->batch_b0 + L->batch_n);
}

Layer::QView batch_view(const Layer *L, int64_t b0) {
    const infllm_layer_desc &d = L->d;
    const int64_t off = b0 - L->batch_b0;
    const int blk = (int)(off / d.exc);
    Layer::QView v;
    v.q_loc = (const bf16_t *)L->bd.d_q_loc + off * kD; v.q_glb = (const bf16_t *)L->bd.d_q_glb + off * kD;
    v.q_sh = (int64_t)L->batch_n * kD; v.q_sb = (int64_t)d.H * L->batch_n * kD;
    v.qbar = L->bd.d_qbar + (int64_t)blk * d.B * d.H * kD;
    v.batched = true;
    // a block's partials live from its group's launch to its merge: the regions are used in turn
    const int region = blk % L->batch_regions;
    v.o_loc = L->bd.d_o_part + (int64_t)region * L->batch_block_rows * kD;
    v.lse_loc = L->bd.d_lse_part + (int64_t)region * L->batch_block_rows;
    v.nsplit = L->batch_nsplit;
    return v;
}

int run_unit_scores(Layer *L, const void *reps, int64_t rep_sb, int64_t rep_su, float *scores, int64_t scores_sb, int first,
                    int count, const float *qbar, void *stream) {
    const infllm_layer_desc &d = L->d;
    const int C = d.H * kD;
    for (int u = 0; u < d.B; ++u) {
        int rc = infllm_unit_scores((const bf16_t *)reps + (int64_t)u * rep_sb, rep_su, first, count, C,
                                    qbar + (int64_t)u * C, scores + (int64_t)u * scores_sb, stream);
        if (rc) return rc;
    }
    return 0;
}

int run_topk(Layer *L, const float *scores, int64_t scores_sb, int n_units, void *stream) {
    const infllm_layer_desc &d = L->d;
    hipStream_t st = (hipStream_t)stream;
    // the last row's kernel also publishes a sequence number the host can poll (kernels of a stream finish in order)
    const bool poll = d.d_topk_flag && d.h_topk_flag && !d.h_topk_idx;
    if (poll) ++L->topk_seq;
    for (int u = 0; u < d.B; ++u) {
        const bool last = poll && u == d.B - 1;
        int rc = infllm_topk_publish(scores + (int64_t)u * scores_sb, n_units, d.topk, d.d_topk_idx + (int64_t)u * d.topk,
                                     last ? d.d_topk_flag : nullptr, L->topk_seq, stream);
        if (rc) return rc;
    }
    if (d.h_topk_idx)      // NULL: d_topk_idx is itself host-visible pinned memory, the kernel wrote there
        HIP_OK(hipMemcpyAsync(d.h_topk_idx, d.d_topk_idx, sizeof(int32_t) * d.B * d.topk, hipMemcpyDeviceToHost, st), "index copy");
    // an event record costs the stream 2-3 us; with the polled sequence number it would only back up the rare case
    // in which the poll gives up, and a stream synchronisation does that as well
    if (!poll) HIP_OK(hipEventRecord(L->topk_done, st), "event");
    L->topk_stream = st;
    L->topk_pending = true;
    return 0;
}

// scores of all units and the selection among them (run_unit_scores + run_topk), one launch per batch row where the
// geometry has the kernel for it
int run_retrieval(Layer *L, const void *reps, int64_t rep_sb, int64_t rep_su, float *scores, int64_t scores_sb, int n_units,
                  const float *qbar, void *stream) {
    const infllm_layer_desc &d = L->d;
    hipStream_t st = (hipStream_t)stream;
    const int C = d.H * kD;
    const bool poll = d.d_topk_flag && d.h_topk_flag && !d.h_topk_idx;
    if (poll) ++L->topk_seq;
    for (int u = 0; u < d.B; ++u) {
        const bool last = poll && u == d.B - 1;
        const bf16_t *reps_u = (const bf16_t *)reps + (int64_t)u * rep_sb;
        float *scores_u = scores + (int64_t)u * scores_sb;
        int rc = infllm_retrieve_fused(reps_u, rep_su, n_units, C, qbar + (int64_t)u * C, d.topk, scores_u, d.d_topk_idx + (int64_t)u * d.topk,
                                       nullptr, last ? d.d_topk_flag : nullptr, L->topk_seq, stream);
        if (rc < 0) return rc;
        if (rc == 1) {
            rc = infllm_unit_scores(reps_u, rep_su, 0, n_units, C, qbar + (int64_t)u * C, scores_u, stream);
            if (rc) return rc;
            rc = infllm_topk_publish(scores_u, n_units, d.topk, d.d_topk_idx + (int64_t)u * d.topk, last ? d.d_topk_flag : nullptr,
                                     L->topk_seq, stream);
            if (rc) return rc;
        }
    }
    if (d.h_topk_idx)      // NULL: d_topk_idx is itself host-visible pinned memory, the kernel wrote there
        HIP_OK(hipMemcpyAsync(d.h_topk_idx, d.d_topk_idx, sizeof(int32_t) * d.B * d.topk, hipMemcpyDeviceToHost, st), "index copy");
    if (!poll) HIP_OK(hipEventRecord(L->topk_done, st), "event");
    L->topk_stream = st;
    L->topk_pending = true;
    return 0;
}

// the selection for the next block from the candidates chosen ahead and the n_new units carved since
int run_topk_merge(Layer *L, const float *scores, int64_t scores_sb, int n_old, int n_new, void *stream) {
    const infllm_layer_desc &d = L->d;
    hipStream_t st = (hipStream_t)stream;
    const bool poll = d.d_topk_flag && d.h_topk_flag && !d.h_topk_idx;
    if (poll) ++L->topk_seq;
    for (int u = 0; u < d.B; ++u) {
        const bool last = poll && u == d.B - 1;
        int rc = infllm_topk_merge_publish(scores + (int64_t)u * scores_sb, L->d_cand + (int64_t)u * d.topk, d.topk, n_old, n_new, d.topk,
                                           d.d_topk_idx + (int64_t)u * d.topk, last ? d.d_topk_flag : nullptr, L->topk_seq, stream);
        if (rc) return rc;
    }
    if (d.h_topk_idx)
        HIP_OK(hipMemcpyAsync(d.h_topk_idx, d.d_topk_idx, sizeof(int32_t) * d.B * d.topk, hipMemcpyDeviceToHost, st), "index copy");
    if (!poll) HIP_OK(hipEventRecord(L->topk_done, st), "event");
    L->topk_stream = st;
    L->topk_pending = true;
    return 0;
}

// the scores of the n_new units carved since the candidates were chosen and the ranking, one launch per batch row;
// returns 1 (nothing launched) when there is no such kernel for this geometry
int run_score_new_rank(Layer *L, const void *reps, int64_t rep_sb, int64_t rep_su, float *scores, int64_t scores_sb, int n_old, int n_new,
                       void *stream) {
    const infllm_layer_desc &d = L->d;
    hipStream_t st = (hipStream_t)stream;
    const int C = d.H * kD;
    if (C % 512 != 0 || (C / 512 != 1 && C / 512 != 2 && C / 512 != 4 && C / 512 != 8) || n_new < 1) return 1;
    const bool poll = d.d_topk_flag && d.h_topk_flag && !d.h_topk_idx;
    if (poll) ++L->topk_seq;
    for (int u = 0; u < d.B; ++u) {
        const bool last = poll && u == d.B - 1;
        int rc = infllm_score_new_rank((const bf16_t *)reps + (int64_t)u * rep_sb, rep_su, C, L->fresh.qbar + (int64_t)u * C,
                                       scores + (int64_t)u * scores_sb, L->d_cand + (int64_t)u * d.topk, d.topk, n_old, n_new, d.topk,
                                       d.d_topk_idx + (int64_t)u * d.topk, last ? d.d_topk_flag : nullptr, L->topk_seq, stream);
        if (rc) return rc < 0 ? rc : infllm_fail(-2, "score_new_rank: no kernel after the geometry check");
    }
    if (d.h_topk_idx)
        HIP_OK(hipMemcpyAsync(d.h_topk_idx, d.d_topk_idx, sizeof(int32_t) * d.B * d.topk, hipMemcpyDeviceToHost, st), "index copy");
    if (!poll) HIP_OK(hipEventRecord(L->topk_done, st), "event");
    L->topk_stream = st;
    L->topk_pending = true;
    return 0;
}

int32_t *cand_buffer(Layer *L, int buf) { return L->h_cand + (int64_t)buf * ((int64_t)L->d.B * L->d.topk + 1); }

// where the next candidate list goes: the buffer, and the note by which infllm_block_prefetch finds it
int cand_publication(Layer *L, int64_t for_b0) {
    const int buf = L->cand_next;
    L->cand_next ^= 1;
    ++L->cand_seq;
    L->cand_pub[buf].b0 = for_b0;
    L->cand_pub[buf].seq = L->cand_seq;
    return buf;
}

bool call_rank_fits(const Layer *L, int first_new, int n_new) {
    return n_new <= 64 && L->d.topk + (first_new + n_new - L->call_n0) <= L->call_room;
}

// From the lists of the prepared call (Layer::call_lists): the n_new units from first_new on were carved just now;
// their scores under the mean queries of the call's later blocks, the selection of block j_sel and the candidates of
// block j_cand (block numbers within the call, -1: none) in one launch.  The caller has checked call_rank_fits.
int run_call_rank(Layer *L, const void *reps, int64_t rep_sb, int64_t rep_su, int first_new, int n_new, int j_sel, int j_cand, void *stream) {
    const infllm_layer_desc &d = L->d;
    hipStream_t st = (hipStream_t)stream;
    if (j_cand >= 0 && !L->h_cand) j_cand = -1;
    const int j0 = j_sel >= 0 ? j_sel : j_cand;
    if (j0 < 0) return 0;                                   // (new units are only ever carved with a block to follow)
    CallRankJob jb{};
    jb.reps = (const bf16_t *)reps; jb.rep_sb = rep_sb; jb.rep_su = rep_su;
    jb.qbars = L->bd.d_qbar; jb.scores = L->call_scores; jb.cols = L->call_cols; jb.base = L->d_base;
    jb.B = d.B; jb.k = d.topk; jb.n_base = L->call_n0; jb.first_new = first_new; jb.n_new = n_new;
    jb.j0 = j0; jb.j_sel = j_sel; jb.j_cand = j_cand;
    const bool poll = d.d_topk_flag && d.h_topk_flag && !d.h_topk_idx;
    if (j_sel >= 0) {
        if (poll) ++L->topk_seq;
        jb.sel_out = d.d_topk_idx; jb.sel_flag = poll ? d.d_topk_flag : nullptr; jb.sel_seq = L->topk_seq;
    }
    if (j_cand >= 0) {
        const int buf = cand_publication(L, L->batch_b0 + (int64_t)j_cand * d.exc);
        jb.cand_out = cand_buffer(L, buf); jb.cand_flag = jb.cand_out + (int64_t)d.B * d.topk; jb.cand_seq = L->cand_seq;
    }
    const int last = j_cand >= 0 ? j_cand : j_sel;
    const int n_wgs = n_new > 0 ? L->call_blocks - j0 : last - j0 + 1;
    int rc = infllm_call_rank(&jb, d.H * kD, n_wgs, stream);
    if (rc) return rc < 0 ? rc : infllm_fail(-2, "call_rank: no kernel after the checks");
    if (j_sel >= 0) {
        if (d.h_topk_idx)
            HIP_OK(hipMemcpyAsync(d.h_topk_idx, d.d_topk_idx, sizeof(int32_t) * d.B * d.topk, hipMemcpyDeviceToHost, st), "index copy");
        if (!poll) HIP_OK(hipEventRecord(L->topk_done, st), "event");
        L->topk_stream = st;
        L->topk_pending = true;
        ++L->n_call_ranked;
    }
    return 0;
}

// n_parts > 0: the stages' partial log-sum-exps are joined inside the launch (d_lse is not ready yet)
infllm_score_args local_score_args(Layer *L, int n, int64_t b0, const Layer::QView &qv, int64_t j_lo, int64_t j_hi, int n_parts) {
    const infllm_layer_desc &d = L->d;
    infllm_score_args sc{};
    sc.d_q = qv.q_loc;
    sc.q_sl = kD; sc.q_sh = qv.q_sh; sc.q_sb = qv.q_sb;
    sc.B = d.B; sc.H = d.H; sc.Hkv = d.Hkv; sc.Lq = n;
    sc.d_k = d.d_ring_k_rot;
    sc.k_sl = kD; sc.k_sh = d.ring_cap * kD; sc.k_sb = (int64_t)d.Hkv * d.ring_cap * kD;
    sc.cap = d.ring_cap; sc.j_lo = j_lo; sc.j_hi = j_hi;
    sc.mask = INFLLM_MASK_WINDOW; sc.accumulate = 1; sc.offset = b0; sc.window = d.n_local;
    sc.d_lse = n_parts > 0 ? d.d_lse_part : d.d_lse; sc.n_parts = n_parts; sc.softmax_scale = d.softmax_scale;
    sc.d_score = d.d_ring_score; sc.score_sh = d.ring_cap; sc.score_sb = (int64_t)d.H * d.ring_cap; sc.score_cap = d.ring_cap;
    return sc;
}

int run_local_score(Layer *L, int n, int64_t b0, const Layer::QView &qv, int64_t j_lo, int64_t j_hi, int n_parts, void *stream) {
    if (j_hi <= j_lo) return 0;
    const infllm_score_args sc = local_score_args(L, n, b0, qv, j_lo, j_hi, n_parts);
    return infllm_local_score(&sc, stream);
}

// the local stage of a block: causal sliding window over the ring
infllm_attn_args local_stage_args(Layer *L, int n, int64_t b0, const Layer::QView &qv, int nsplit) {
    const infllm_layer_desc &d = L->d;
    const int64_t b1 = b0 + n;
    const int64_t lo = b0 > d.n_local ? b0 - d.n_local : 0;
    infllm_attn_args at{};
    at.d_q = qv.q_loc;
    at.q_sl = kD; at.q_sh = qv.q_sh; at.q_sb = qv.q_sb;
    at.B = d.B; at.H = d.H; at.Hkv = d.Hkv; at.Lq = n;
    at.d_k = d.d_ring_k_rot; at.d_v = d.d_ring_v;
    at.k_sl = at.v_sl = kD;
    at.k_sh = at.v_sh = d.ring_cap * kD;
    at.k_sb = at.v_sb = (int64_t)d.Hkv * d.ring_cap * kD;
    at.cap = d.ring_cap; at.j_lo = lo; at.j_hi = b1;
    at.mask = INFLLM_MASK_WINDOW; at.offset = b0; at.window = d.n_local;
    at.nsplit = nsplit;
    at.softmax_scale = d.softmax_scale;
    at.d_o_part = d.d_o_part; at.d_lse_part = d.d_lse_part;
    return at;
}

}  // namespace

extern "C" int infllm_layer_set_batch(void *layer, const infllm_batch_desc *b) {
    INFLLM_REQUIRE(layer && b, "layer_set_batch: null argument");
    Layer *L = (Layer *)layer;
    const infllm_layer_desc &d = L->d;
    INFLLM_REQUIRE(b->d_q_loc && b->d_q_glb && b->d_qpart && b->d_qbar && b->d_o_part && b->d_lse_part, "layer_set_batch: null buffer");
    INFLLM_REQUIRE(d.exc % 32 == 0, "layer_set_batch: execution blocks of %d rows are not whole query tiles", d.exc);
    INFLLM_REQUIRE(b->max_tokens >= d.exc, "layer_set_batch: %d tokens are less than one execution block", b->max_tokens);
    INFLLM_REQUIRE(b->group_blocks >= 0 && b->group_blocks <= 64, "layer_set_batch: %d blocks per launch", b->group_blocks);
    const int group = b->group_blocks > 0 ? b->group_blocks : 2;
    INFLLM_REQUIRE(b->part_rows >= (int64_t)d.B * d.H * d.exc * (4 * group > 8 ? 4 * group : 8), "layer_set_batch: too few partial rows");
    INFLLM_REQUIRE(!L->batch_live, "layer_set_batch: a prepared call is still being worked off");
    L->bd = *b;
    L->batch_ok = true;
    return 0;
}

extern "C" int infllm_call_front(void *layer, const infllm_front_args *a, void *stream) {
    INFLLM_REQUIRE(layer && a, "call_front: null argument");
    Layer *L = (Layer *)layer;
    const infllm_layer_desc &d = L->d;
    hipStream_t st = (hipStream_t)stream;
    INFLLM_REQUIRE(L->batch_ok, "call_front: no buffers (infllm_layer_set_batch)");
    INFLLM_REQUIRE(a->n >= 1 && a->n <= L->bd.max_tokens, "call_front: %d tokens do not fit the buffers (%d)", a->n, L->bd.max_tokens);
    INFLLM_REQUIRE(a->n <= d.ring_cap, "call_front: %d tokens do not fit a ring of %lld rows", a->n, (long long)d.ring_cap);
    INFLLM_REQUIRE(a->n_units >= 0 && a->b0 >= 0, "call_front: negative state");
    INFLLM_REQUIRE(a->d_q && a->d_k && a->d_v, "call_front: null q / k / v");
    // the rows from the carving cursor on are still needed (remainder, window, score track): writing a->n rows at b0
    // must not reach around the ring to them
    INFLLM_REQUIRE(!L->cursor_known || a->b0 - L->cursor + a->n <= d.ring_cap,
                   "call_front: %d tokens at %lld would overwrite ring rows from %lld on (ring of %lld rows)", a->n, (long long)a->b0,
                   (long long)L->cursor, (long long)d.ring_cap);
    L->main_stream = st;
    L->main_stream_known = true;
    L->unflushed = true;
    L->batch_live = false;
    L->prepared = false;
    const int C = d.H * kD;
    const int n_blocks = (a->n + d.exc - 1) / d.exc;

    // ---- the first block's retrieval first: the host waits for its ids before it can fetch anything for this call,
    //      and the prologue of the whole call would put 50-60 us in front of them.  The first block's rows go through
    //      the prologue twice (the second time with the rest of the call, to the same effect).
    int rc;
    L->topk_pending = false;
    L->batch_retrieved = false;
    const bool retrieve = a->n_units > d.topk && !(a->flags & INFLLM_NO_RETRIEVAL);
    if (retrieve) {
        INFLLM_REQUIRE(a->d_reps && a->d_unit_scores, "call_front: null representative / score buffer");
        L->slot ^= 1;
        rc = run_ingest(L, a, a->d_q, a->d_k, a->d_v, a->n < d.exc ? a->n : d.exc, a->b0, L->slot, true, stream);
        if (rc) return rc;
        rc = run_retrieval(L, a->d_reps, a->rep_sb, a->rep_su, a->d_unit_scores, a->unit_scores_sb, a->n_units, L->fresh.qbar, stream);
        if (rc) return rc;
    }

    // ---- prologue of every token, mean query of every block
    infllm_ingest_args in{};
    in.d_q = a->d_q; in.d_k = a->d_k; in.d_v = a->d_v;
    in.q_sb = a->q_sb; in.q_sh = a->q_sh; in.q_sl = a->q_sl;
    in.k_sb = a->k_sb; in.k_sh = a->k_sh; in.k_sl = a->k_sl;
    in.v_sb = a->v_sb; in.v_sh = a->v_sh; in.v_sl = a->v_sl;
    in.B = d.B; in.H = d.H; in.Hkv = d.Hkv; in.n = a->n;
    in.pos0 = a->b0; in.glb_pos = d.n_local - 1;
    in.d_inv_freq = d.d_inv_freq; in.distance_scale = d.distance_scale;
    in.d_ring_k_raw = d.d_ring_k_raw; in.d_ring_k_rot = d.d_ring_k_rot; in.d_ring_v = d.d_ring_v;
    in.d_ring_score = d.d_ring_score; in.ring_cap = d.ring_cap;
    in.d_q_loc = L->bd.d_q_loc; in.d_q_glb = L->bd.d_q_glb;
    in.d_qpart = L->bd.d_qpart;
    rc = infllm_ingest(&in, stream);
    if (rc) return rc;
    rc = infllm_reduce_partials_blocks(L->bd.d_qpart, d.B, a->n, d.exc, C, L->bd.d_qbar, stream);
    if (rc) return rc;

    // ---- how the local stage cuts its keys: as few splits as fill the chip, and no more than the partial rows hold.
    //      It is launched for a group of blocks at a time (block_front, at the group's first block), every launch
    //      with the same number of splits.
    const int group = L->bd.group_blocks > 0 ? L->bd.group_blocks : 2;
    const int group_n = a->n < group * d.exc ? a->n : group * d.exc;
    const int64_t b1 = a->b0 + group_n;
    const int64_t lo = a->b0 > d.n_local ? a->b0 - d.n_local : 0;
    int nsplit = splits_for(d, group_n, (int)((b1 - lo + kTile - 1) / kTile));
    // room for the partials of two groups: the one being merged block by block and the one launched ahead of it
    const int64_t rows_one = (int64_t)d.B * d.H * (n_blocks > 1 ? d.exc : a->n);
    const int need = n_blocks > 1 ? 2 * group : 1;
    while (nsplit > 1 && L->bd.part_rows / (nsplit * rows_one) < need) --nsplit;
    int regions = (int)(L->bd.part_rows / (nsplit * rows_one));
    INFLLM_REQUIRE(regions >= need, "call_front: partial rows do not fit");
    regions = regions / group * group;
    L->batch_live = true;
    L->batch_b0 = a->b0;
    L->batch_n = a->n;
    L->batch_nsplit = nsplit;
    L->batch_group = group;
    L->batch_regions = n_blocks > 1 ? regions : 1;
    L->batch_block_rows = (int64_t)nsplit * d.B * d.H * (n_blocks > 1 ? d.exc : a->n);
    L->fresh = batch_view(L, a->b0);

    L->batch_retrieved = retrieve;

    // ---- the lists of the call's other blocks (the k best of the units that exist now under each block's mean query)
    //      are made behind the first block's global stage (block_back): here they would sit between the first
    //      selection and the first global stage, a stretch in which the stream only waits for the first fetch
    L->call_lists = false;
    L->call_lists_pending = false;
    const int max_new = (a->n + d.block_size - 1) / d.block_size + 1;
    const int cpl = C % 512 == 0 ? C / 512 : 0;
    if (retrieve && n_blocks > 1 && n_blocks <= kMaxCallBlocks && a->d_call_scores && L->d_base && !L->no_call_lists && d.topk <= 64 &&
        (cpl == 1 || cpl == 2 || cpl == 4 || cpl == 8) && a->call_scores_cols >= (int64_t)a->n_units + max_new &&
        d.topk + max_new <= infllm_call_rank_room() && d.max_carve <= 64) {
        L->call_lists_pending = true;
        L->call_n0 = a->n_units;
        L->call_blocks = n_blocks;
        L->call_scores = a->d_call_scores;
        L->call_cols = a->call_scores_cols;
    }
    return 0;
}

extern "C" int infllm_block_front(void *layer, const infllm_front_args *a, void *stream) {
    INFLLM_REQUIRE(layer && a, "block_front: null argument");
    Layer *L = (Layer *)layer;
    const infllm_layer_desc &d = L->d;
    hipStream_t st = (hipStream_t)stream;
    INFLLM_REQUIRE(a->n >= 1 && a->n <= d.exc, "block_front: %d queries do not fit an execution block of %d", a->n, d.exc);
    INFLLM_REQUIRE(a->n_units >= 0 && a->b0 >= 0, "block_front: negative state");
    INFLLM_REQUIRE(a->n_next >= 0 && a->n_next <= d.exc, "block_front: bad next block size %d", a->n_next);
    int rc;
    L->main_stream = st;
    L->main_stream_known = true;
    L->unflushed = true;

    // ---- this block's prologue and retrieval, unless the previous block prepared them
    const bool batched = block_in_batch(L, a->b0, a->n);       // its prologue and local stage ran in infllm_call_front
    if (!(L->prepared && L->prepared_b0 == a->b0 && L->prepared_n == a->n)) {
        const bool retrieve = a->n_units > d.topk && !(a->flags & INFLLM_NO_RETRIEVAL);
        const bool retrieved = batched && L->batch_retrieved && a->b0 == L->batch_b0;
        if (batched)
            L->fresh = batch_view(L, a->b0);
        else {
            L->slot ^= 1;
            rc = run_ingest(L, a, a->d_q, a->d_k, a->d_v, a->n, a->b0, L->slot, retrieve, stream);
            if (rc) return rc;
        }
        if (!retrieved) L->topk_pending = false;
        if (retrieve && !retrieved) {
            INFLLM_REQUIRE(a->d_reps && a->d_unit_scores, "block_front: null representative / score buffer");
            rc = run_retrieval(L, a->d_reps, a->rep_sb, a->rep_su, a->d_unit_scores, a->unit_scores_sb, a->n_units, L->fresh.qbar, stream);
            if (rc) return rc;
        }
    }
    L->batch_retrieved = false;
    L->prepared = false;
    L->cur = L->fresh;
    L->cur_n = a->n;
    if (!batched) L->call_lists = L->call_lists_pending = false;

    const int64_t b1 = a->b0 + a->n;
    const int64_t lo = a->b0 > d.n_local ? a->b0 - d.n_local : 0;

    // ---- the next block's prologue and the scores of the units that exist already.  Ahead of the local stage: the
    //      host starts the next block's fetch from the candidates chosen here, and everything queued before them
    //      delays that fetch.
    const bool next_batched = a->n_next > 0 && block_in_batch(L, b1, a->n_next);
    if (next_batched || (a->n_next > 0 && a->d_q_next && a->d_k_next && a->d_v_next)) {
        if (next_batched)
            L->fresh = batch_view(L, b1);
        else {
            L->slot ^= 1;
            rc = run_ingest(L, a, a->d_q_next, a->d_k_next, a->d_v_next, a->n_next, b1, L->slot, true, stream);
            if (rc) return rc;
        }
        // (with the lists of a prepared call the next block's candidates were ranked when the previous block had
        //  carved its units: nothing to do here)
        L->scored_units = -1;
        if (a->n_units > 0 && !(a->flags & INFLLM_NO_RETRIEVAL) && !(L->call_lists && next_batched)) {
            L->scored_units = a->n_units;
            INFLLM_REQUIRE(a->d_reps && a->d_unit_scores, "block_front: null representative / score buffer");
            // The scores of the existing units and their k best now, while the fetch is in flight: the selection after the
            // block then only has to weigh these against the few units carved in between, instead of running over every
            // unit on the chain.  One launch per batch row where the geometry has the kernel for it, else two.
            L->cand_units = -1;
            const bool want_cand = L->d_cand && a->n_units > d.topk;
            // the host gets a copy, with a sequence number behind the last row's: it may fetch them ahead
            const int buf = want_cand && L->h_cand ? cand_publication(L, b1) : -1;
            const int C = d.H * kD;
            for (int u = 0; u < d.B; ++u) {
                const bf16_t *reps_u = (const bf16_t *)a->d_reps + (int64_t)u * a->rep_sb;
                float *scores_u = a->d_unit_scores + (int64_t)u * a->unit_scores_sb;
                const float *qbar_u = L->fresh.qbar + (int64_t)u * C;
                int32_t *cand_host = buf >= 0 ? cand_buffer(L, buf) + (int64_t)u * d.topk : nullptr;
                int32_t *cand_flag = buf >= 0 && u == d.B - 1 ? cand_buffer(L, buf) + (int64_t)d.B * d.topk : nullptr;
                rc = want_cand ? infllm_retrieve_fused(reps_u, a->rep_su, a->n_units, C, qbar_u, d.topk, scores_u, L->d_cand + (int64_t)u * d.topk,
                                                       cand_host, cand_flag, L->cand_seq, stream)
                               : 1;
                if (rc < 0) return rc;
                if (rc == 1) {
                    rc = infllm_unit_scores(reps_u, a->rep_su, 0, a->n_units, C, qbar_u, scores_u, stream);
                    if (rc) return rc;
                    if (want_cand) {
                        rc = infllm_topk_publish_pair(scores_u, a->n_units, d.topk, L->d_cand + (int64_t)u * d.topk, cand_host, cand_flag,
                                                      L->cand_seq, stream);
                        if (rc) return rc;
                    }
                }
            }
            if (want_cand) L->cand_units = a->n_units;
        }
        L->prepared = true;
        L->prepared_b0 = b1;
        L->prepared_n = a->n_next;
    }

    // ---- local stage: causal sliding window over the ring.  Launched here, ahead of the host's wait for the selection
    //      and of the stream's wait for the fetched units, both of which it covers.  (Both stages of a block as ONE
    //      launch behind that wait was measured: the launch is 6 us shorter than the two and the merge reads half the
    //      partials, but the stream then reaches its wait for the fetch a local stage earlier and idles longer than it
    //      saved.  infllm_attn_stages_fused remains an entry point of the library.)
    if (batched && ((a->b0 - L->batch_b0) / d.exc) % L->batch_group == 0) {
        // the local stage of this block and the next ones of its group in one launch (more queries per launch: fewer
        // key splits, fewer partial rows, the launch's fixed cost once); each block's partials go where its merge
        // expects them
        const int64_t left = L->batch_b0 + L->batch_n - a->b0;
        const int gn = (int)(left < (int64_t)L->batch_group * d.exc ? left : (int64_t)L->batch_group * d.exc);
        infllm_attn_args at = local_stage_args(L, gn, a->b0, L->cur, L->batch_nsplit);
        at.d_o_part = (uint16_t *)L->cur.o_loc; at.d_lse_part = (float *)L->cur.lse_loc;
        const int ti = timer_begin(L, 0, gn, (int)(a->b0 + gn - lo), st);
        rc = infllm_attn_stage_blocked(&at, d.exc, L->batch_block_rows, stream);
        timer_end(L, 0, ti, st);
        if (rc) return rc;
    }
    if (!batched) {
        infllm_attn_args at = local_stage_args(L, a->n, a->b0, L->cur, splits_for(d, a->n, (int)((b1 - lo + kTile - 1) / kTile)));
        const int ti = timer_begin(L, 0, a->n, (int)(b1 - lo), st);
        rc = infllm_attn_stage(&at, stream);
        timer_end(L, 0, ti, st);
        if (rc) return rc;
    }
    return 0;
}

extern "C" int infllm_layer_wait_topk(void *layer) {
    INFLLM_REQUIRE(layer, "layer_wait_topk: null layer");
    Layer *L = (Layer *)layer;
    if (!L->topk_pending) return 0;
    if (L->d.d_topk_flag && L->d.h_topk_flag && !L->d.h_topk_idx) {
        // poll the pinned sequence number for a while: waking up from an event wait costs tens of microseconds,
        // and this wait sits on the chain from one block's selection to the next
        const volatile int32_t *flag = L->d.h_topk_flag;
        const auto t0 = std::chrono::steady_clock::now();
        for (uint32_t spins = 0; *flag != L->topk_seq; ++spins) {
            if ((spins & 1023u) == 1023u && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(2)) break;
            __builtin_ia32_pause();
        }
        if (*flag == L->topk_seq) {
            std::atomic_thread_fence(std::memory_order_acquire);
            L->topk_pending = false;
            L->seen_seq = L->topk_seq;
            return 0;
        }
        HIP_OK(hipStreamSynchronize(L->topk_stream), "layer_wait_topk");        // no event was recorded in this mode
        L->topk_pending = false;
        L->seen_seq = L->topk_seq;
        return 0;
    }
    HIP_OK(hipEventSynchronize(L->topk_done), "layer_wait_topk");
    L->topk_pending = false;
    return 0;
}

extern "C" int infllm_layer_wait_mass(void *layer) {
    INFLLM_REQUIRE(layer, "layer_wait_mass: null layer");
    Layer *L = (Layer *)layer;
    if (!L->mass_pending) return 0;
    HIP_OK(hipEventSynchronize(L->mass_done), "layer_wait_mass");
    L->mass_pending = false;
    return 0;
}

extern "C" int infllm_block_fetch(void *layer, int32_t n_miss, const int32_t *h_miss_row, const int32_t *h_miss_slot,
                                  const int32_t *h_miss_unit, const void *const *h_miss_src, void *stream, void *copy_stream) {
    INFLLM_REQUIRE(layer && n_miss >= 0, "block_fetch: bad arguments");
    Layer *L = (Layer *)layer;
    INFLLM_REQUIRE(n_miss <= L->d.B * L->d.topk, "block_fetch: %d misses exceed what a block can select", n_miss);
    int rc = do_fetch(L, n_miss, h_miss_row, h_miss_slot, h_miss_unit, h_miss_src, (hipStream_t)stream, (hipStream_t)copy_stream);
    if (rc == 0) L->fetch_issued = true;
    return rc;
}

namespace {

const void *host_unit(const infllm_select_args *a, int unit, int row) {
    const int chunk = unit / a->units_per_chunk, idx = unit % a->units_per_chunk;
    if (chunk >= a->n_chunks || !a->h_chunk_base[chunk]) return nullptr;
    return (const void *)(uintptr_t)(a->h_chunk_base[chunk] + (uint64_t)idx * a->unit_bytes + (uint64_t)row * a->row_bytes);
}

// A guess that is not confirmed leaves residents behind whose slots it overwrote: they are fetched again (those
// that are still resident, in the slot they had; all of them when no policy objects are given, i.e. when the policy
// has not moved since the guess).  `extra` lists misses to fetch in the same go.
int ahead_repair(Layer *L, void *const *caches, int n_extra, const int32_t *rows, const int32_t *slots, const int32_t *units,
                 const void *const *srcs, hipStream_t st, hipStream_t cs) {
    Layer::Ahead &g = L->ahead;
    std::vector<int32_t> r(rows, rows + n_extra), sl(slots, slots + n_extra), un(units, units + n_extra);
    std::vector<const void *> sr(srcs, srcs + n_extra);
    for (size_t i = 0; i < g.victim_unit.size(); ++i) {
        if (caches && infllm_cache_slot_of(caches[g.victim_row[i]], g.victim_unit[i]) != g.victim_slot[i]) continue;     // gone by now
        r.push_back(g.victim_row[i]);
        sl.push_back(g.victim_slot[i]);
        un.push_back(g.victim_unit[i]);
        sr.push_back(g.victim_src[i]);
    }
    g.victim_unit.clear();
    const int rc = do_fetch(L, (int)r.size(), r.data(), sl.data(), un.data(), sr.data(), st, cs);
    L->efetch_prev_in_use = false;            // it also wrote slots of units that are not selected: the next guess may evict those
    return rc;
}

}  // namespace

extern "C" int infllm_block_prefetch(void *layer, const infllm_select_args *a, void *stream, void *copy_stream) {
    INFLLM_REQUIRE(layer && a, "block_prefetch: null argument");
    Layer *L = (Layer *)layer;
    const infllm_layer_desc &d = L->d;
    Layer::Ahead &g = L->ahead;
    INFLLM_REQUIRE(!g.active, "block_prefetch: the previous guess has not been settled by infllm_block_select");
    const int k = d.topk, B = d.B;
    if (!L->h_cand || k > 64 || L->next_b0 < 0) return 0;
    int buf = -1;                                        // the list that was chosen for the block that comes next
    for (int i = 0; i < 2; ++i)
        if (L->cand_pub[i].b0 == L->next_b0) buf = i;
    if (buf < 0) return 0;
    const int32_t cand_seq = L->cand_pub[buf].seq;
    L->cand_pub[buf].b0 = -1;
    const int32_t *h_cand = cand_buffer(L, buf);
    // Beside the block's own kernels the fetch kernel slows them down by more than the shorter chain gains (measured):
    // without the DMA engines the fetch stays behind the selection, unless INFLLM_FETCH_AHEAD_ALWAYS=1 asks for it.
    if (!L->efetch_ok && !L->ahead_any_path) return 0;
    INFLLM_REQUIRE(a->caches && a->h_chunk_base && a->units_per_chunk > 0 && a->n_chunks >= 0 && a->unit_bytes > 0 && a->row_bytes > 0,
                   "block_prefetch: bad cache list / host arena description");
    // (the list was launched ahead of the local stage of the block in flight, or behind the block before it)
    const volatile int32_t *flag = h_cand + (int64_t)B * k;
    const auto t0 = std::chrono::steady_clock::now();
    for (uint32_t spins = 0; *flag != cand_seq; ++spins) {
        if ((spins & 1023u) == 1023u && std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(2)) return 0;
        __builtin_ia32_pause();
    }
    std::atomic_thread_fence(std::memory_order_acquire);
    g.n_sel = k;
    g.cand.assign(h_cand, h_cand + (int64_t)B * k);
    g.sel_slots.resize((size_t)B * k);
    g.evicted.resize((size_t)B * k);
    g.n_evicted.assign(B, 0);
    g.n_miss.assign(B, 0);
    g.miss_row.clear(); g.miss_slot.clear(); g.miss_unit.clear(); g.miss_src.clear();
    g.victim_row.clear(); g.victim_unit.clear(); g.victim_slot.clear(); g.victim_src.clear();
    g.shadow.resize(B, nullptr);
    for (int u = 0; u < B; ++u) {
        INFLLM_REQUIRE(a->caches[u], "block_prefetch: null cache of row %d", u);
        if (!g.shadow[u]) {
            g.shadow[u] = infllm_cache_clone(a->caches[u]);
            INFLLM_REQUIRE(g.shadow[u], "block_prefetch: no shadow cache");
        } else {
            const int crc = infllm_cache_copy(g.shadow[u], a->caches[u]);
            if (crc) return crc;
        }
        int32_t units[64], slots[64], n_ev = 0;
        const int32_t *cand = g.cand.data() + (int64_t)u * k;
        for (int i = 0; i < k; ++i)
            if (cand[i] < 0 || !host_unit(a, cand[i], u)) return 0;                 // not a list of units: no guess
        const int m = infllm_cache_touch(g.shadow[u], cand, k, g.sel_slots.data() + (int64_t)u * k, units, slots,
                                         g.evicted.data() + (int64_t)u * k, &n_ev);
        if (m < 0) return m;
        g.n_evicted[u] = n_ev;
        g.n_miss[u] = m;
        for (int e = 0; e < n_ev; ++e) {
            const int32_t unit = g.evicted[(int64_t)u * k + e];
            // a victim that the block in flight still reads: no fetch ahead this time
            if ((int64_t)(u + 1) * L->last_n_sel <= (int64_t)L->last_sel.size())
                for (int j = 0; j < L->last_n_sel; ++j)
                    if (L->last_sel[(int64_t)u * L->last_n_sel + j] == unit) return 0;
            g.victim_row.push_back(u);
            g.victim_unit.push_back(unit);
            g.victim_slot.push_back(infllm_cache_slot_of(a->caches[u], unit));
            g.victim_src.push_back(host_unit(a, unit, u));
        }
        for (int i = 0; i < m; ++i) {
            g.miss_row.push_back(u);
            g.miss_slot.push_back(slots[i]);
            g.miss_unit.push_back(units[i]);
            g.miss_src.push_back(host_unit(a, units[i], u));
        }
    }
    g.n_miss_all = (int)g.miss_unit.size();
    const int rc = do_fetch(L, g.n_miss_all, g.miss_row.data(), g.miss_slot.data(), g.miss_unit.data(), g.miss_src.data(),
                            (hipStream_t)stream, (hipStream_t)copy_stream, true);
    if (rc) return rc;
    g.active = true;
    ++L->ahead_issued;
    return g.n_miss_all;
}

extern "C" int64_t infllm_layer_staged_units(void *layer) {
    if (!layer) return infllm_fail(-1, "layer_staged_units: null layer");
    return ((Layer *)layer)->staged_units;
}

extern "C" int infllm_layer_path_counts(void *layer, int64_t *counts) {
    INFLLM_REQUIRE(layer && counts, "layer_path_counts: null argument");
    const Layer *L = (const Layer *)layer;
    counts[0] = L->n_tables_inline;
    counts[1] = L->n_tables_kernel;
    counts[2] = L->n_tables_upload;
    counts[3] = L->n_score_merged;
    counts[4] = L->n_score_apart;
    counts[5] = L->n_call_ranked;
    return 0;
}

extern "C" int64_t infllm_layer_fetched_units(void *layer) {
    if (!layer) return infllm_fail(-1, "layer_fetched_units: null layer");
    return ((Layer *)layer)->fetched_units;
}

extern "C" int infllm_layer_prefetch_stats(void *layer, int64_t *issued, int64_t *confirmed) {
    INFLLM_REQUIRE(layer, "layer_prefetch_stats: null layer");
    Layer *L = (Layer *)layer;
    if (issued) *issued = L->ahead_issued;
    if (confirmed) *confirmed = L->ahead_confirmed;
    return 0;
}

extern "C" int infllm_layer_last_selection(void *layer, int32_t *ids, int32_t capacity) {
    INFLLM_REQUIRE(layer && (ids || capacity == 0) && capacity >= 0, "layer_last_selection: bad arguments");
    Layer *L = (Layer *)layer;
    const int64_t n = (int64_t)L->last_sel.size();
    INFLLM_REQUIRE(n <= capacity, "layer_last_selection: %lld ids do not fit %d", (long long)n, capacity);
    if (n) std::memcpy(ids, L->last_sel.data(), sizeof(int32_t) * n);
    return (int)n;
}

extern "C" int infllm_block_select(void *layer, const infllm_select_args *a, void *stream, void *copy_stream) {
    INFLLM_REQUIRE(layer && a, "block_select: null argument");
    Layer *L = (Layer *)layer;
    const infllm_layer_desc &d = L->d;
    INFLLM_REQUIRE(a->caches && a->n_sel >= 0 && a->n_sel <= d.topk, "block_select: bad selection size %d", a->n_sel);
    INFLLM_REQUIRE(a->n_sel == 0 || (a->h_selected && a->h_sel_slots && a->h_miss_row && a->h_miss_slot && a->h_miss_unit && a->h_miss_src),
                   "block_select: null list");
    INFLLM_REQUIRE(a->n_sel == 0 || (a->h_chunk_base && a->units_per_chunk > 0 && a->n_chunks >= 0 && a->unit_bytes > 0 && a->row_bytes > 0),
                   "block_select: bad host arena description");
    if (a->wait_topk) {
        const int wrc = infllm_layer_wait_topk(layer);
        if (wrc) return wrc;
    }
    if (L->global_unmarked && !a->wait_topk && L->main_stream) {
        // The previous global stage left no event behind because the host was expected to read this block's selection
        // (which the stream produces after that stage) before fetching.  A caller that brings its own selection has not
        // waited for anything: the slots may still be read, so wait here.
        HIP_OK(hipStreamSynchronize(L->main_stream), "block_select: wait for the previous global stage");
    }
    L->global_unmarked = false;
    L->last_n_sel = a->n_sel;
    if (a->n_sel > 0) L->last_sel.assign(a->h_selected, a->h_selected + (int64_t)d.B * a->n_sel);
    else L->last_sel.clear();
    bool repair = false;
    L->guessing = L->ahead.active;
    if (L->ahead.active) {
        Layer::Ahead &g = L->ahead;
        g.active = false;
        if (a->n_sel == g.n_sel && std::memcmp(a->h_selected, g.cand.data(), sizeof(int32_t) * d.B * a->n_sel) == 0) {
            // the guess was the selection: its policy state becomes the state, its fetch is the block's fetch
            for (int u = 0; u < d.B; ++u) {
                INFLLM_REQUIRE(a->caches[u], "block_select: null cache of row %d", u);
                const int crc = infllm_cache_copy(a->caches[u], g.shadow[u]);
                if (crc) return crc;
                if (a->h_n_evicted) a->h_n_evicted[u] = g.n_evicted[u];
                if (a->h_n_miss) a->h_n_miss[u] = g.n_miss[u];
            }
            std::memcpy(a->h_sel_slots, g.sel_slots.data(), sizeof(int32_t) * d.B * a->n_sel);
            if (a->h_evicted) std::memcpy(a->h_evicted, g.evicted.data(), sizeof(int32_t) * d.B * a->n_sel);
            for (int i = 0; i < g.n_miss_all; ++i) {
                a->h_miss_row[i] = g.miss_row[i];
                a->h_miss_slot[i] = g.miss_slot[i];
                a->h_miss_unit[i] = g.miss_unit[i];
                a->h_miss_src[i] = g.miss_src[i];
            }
            g.victim_unit.clear();
            ++L->ahead_confirmed;
            L->fetch_issued = true;
            return g.n_miss_all;
        }
        repair = true;
    }
    // From here on the policy state is the one before any guess.  After a guess that was not the selection, most of
    // what it moved is still wanted: a missed unit takes the slot the guess put it in where that slot is free (the
    // policy does not care which slot a unit has), and only the others are left to fetch.
    Layer::Ahead &g = L->ahead;
    int n_miss = 0, n_todo = 0;
    int32_t units[64], slots[64], hint_units[64], hint_slots[64];
    INFLLM_REQUIRE(a->n_sel <= 64, "block_select: more than 64 units per row");
    for (int u = 0; u < d.B; ++u) {
        INFLLM_REQUIRE(a->caches[u], "block_select: null cache of row %d", u);
        int32_t n_ev = 0, n_hints = 0;
        if (repair)
            for (int i = 0; i < g.n_miss_all && n_hints < 64; ++i)
                if (g.miss_row[i] == u) hint_units[n_hints] = g.miss_unit[i], hint_slots[n_hints++] = g.miss_slot[i];
        const int m = infllm_cache_touch_hinted(a->caches[u], a->h_selected + (int64_t)u * a->n_sel, a->n_sel,
                                                a->h_sel_slots + (int64_t)u * a->n_sel, units, slots,
                                                a->h_evicted ? a->h_evicted + (int64_t)u * a->n_sel : nullptr, &n_ev, hint_units, hint_slots, n_hints);
        if (m < 0) return m;
        if (a->h_n_evicted) a->h_n_evicted[u] = n_ev;
        if (a->h_n_miss) a->h_n_miss[u] = m;
        for (int i = 0; i < m; ++i, ++n_miss) {
            bool in_place = false;                                  // the guess has put (or is putting) it there
            for (int h = 0; h < n_hints && !in_place; ++h) in_place = hint_units[h] == units[i] && hint_slots[h] == slots[i];
            if (in_place) continue;
            const void *src = host_unit(a, units[i], u);
            INFLLM_REQUIRE(src, "block_select: unit %d has no host copy", units[i]);
            a->h_miss_row[n_todo] = u;
            a->h_miss_slot[n_todo] = slots[i];
            a->h_miss_unit[n_todo] = units[i];
            a->h_miss_src[n_todo] = src;
            ++n_todo;
        }
    }
    const int rc = repair ? ahead_repair(L, a->caches, n_todo, a->h_miss_row, a->h_miss_slot, a->h_miss_unit, a->h_miss_src,
                                         (hipStream_t)stream, (hipStream_t)copy_stream)
                          : do_fetch(L, n_todo, a->h_miss_row, a->h_miss_slot, a->h_miss_unit, a->h_miss_src, (hipStream_t)stream,
                                     (hipStream_t)copy_stream);
    if (rc) return rc;
    L->fetch_issued = true;
    return n_miss;
}

namespace {

// The global stage's page table of batch row u, on the host: units (by slot) | init tokens | overflow remainder of the
// ring.  Writes at most `room` entries to pg and returns how many the row has (slots are checked by the caller).
int host_pages(const infllm_layer_desc &d, const infllm_back_args *a, int u, int64_t overflow_end, infllm_page *pg, int room) {
    const int bs = d.block_size;
    const int64_t unit_elems = (int64_t)d.Hkv * bs * kD, slot_elems = 2 * unit_elems;
    int n = 0;
    auto push = [&](const bf16_t *k, const bf16_t *v, int64_t hs, int valid) {
        if (n < room) pg[n] = infllm_page{k, v, hs, valid, 0};
        ++n;
    };
    for (int s = 0; s < a->n_sel; ++s) {
        const int sl = a->h_sel_slots[u * a->n_sel + s];
        const bf16_t *kb = (const bf16_t *)d.d_slab + ((int64_t)u * d.max_cached + sl) * slot_elems;
        for (int t0 = 0; t0 < bs; t0 += kTile)
            push(kb + (int64_t)t0 * kD, kb + unit_elems + (int64_t)t0 * kD, (int64_t)bs * kD, bs - t0 < kTile ? bs - t0 : kTile);
    }
    const bf16_t *ik = (const bf16_t *)d.d_init_kv + (int64_t)u * 2 * d.Hkv * d.init_cap * kD;
    const bf16_t *iv = ik + (int64_t)d.Hkv * d.init_cap * kD;
    for (int t0 = 0; t0 < a->init_len; t0 += kTile)
        push(ik + (int64_t)t0 * kD, iv + (int64_t)t0 * kD, d.init_cap * kD, a->init_len - t0 < kTile ? a->init_len - t0 : kTile);
    const bf16_t *rk = (const bf16_t *)d.d_ring_k_raw + (int64_t)u * d.Hkv * d.ring_cap * kD;
    const bf16_t *rv = (const bf16_t *)d.d_ring_v + (int64_t)u * d.Hkv * d.ring_cap * kD;
    for (int64_t pos = a->cursor; pos < overflow_end;) {
        const int64_t row = pos % d.ring_cap;
        int64_t len = overflow_end - pos;
        if (len > kTile) len = kTile;
        if (len > d.ring_cap - row) len = d.ring_cap - row;
        push(rk + row * kD, rv + row * kD, d.ring_cap * kD, (int)len);
        pos += len;
    }
    return n;
}

}  // namespace

extern "C" int infllm_block_back(void *layer, const infllm_back_args *a, void *stream, void *copy_stream) {
    INFLLM_REQUIRE(layer && a, "block_back: null argument");
    Layer *L = (Layer *)layer;
    const infllm_layer_desc &d = L->d;
    hipStream_t st = (hipStream_t)stream, cs = (hipStream_t)copy_stream;
    const bool side = cs != st;
    const int bs = d.block_size;
    L->unflushed = true;
    L->last_copy_stream = cs;
    INFLLM_REQUIRE(a->n >= 1 && a->n <= d.exc && a->n_sel >= 0 && a->n_sel <= d.topk, "block_back: bad block sizes");
    INFLLM_REQUIRE(a->n_miss >= 0 && a->n_miss <= d.B * a->n_sel && a->init_len >= 0 && a->init_len <= d.init_cap,
                   "block_back: bad miss / init counts");
    INFLLM_REQUIRE(a->n_sel == 0 || a->h_sel_slots, "block_back: null slot list");
    INFLLM_REQUIRE(a->d_out && a->cursor >= 0 && a->init_take >= 0 && a->n_carve >= 0 && a->n_carve <= d.max_carve,
                   "block_back: bad output / carve arguments");
    INFLLM_REQUIRE(a->n_units >= 0, "block_back: negative unit count");
    const int64_t b1 = a->b0 + a->n;
    L->next_b0 = b1;
    const int64_t unit_elems = (int64_t)d.Hkv * bs * kD;          // K (or V) of one unit
    const int64_t slot_elems = 2 * unit_elems;
    const Layer::QView &cur = L->cur;
    const bool batched = cur.batched;

    // ---- 1. fetch missed units into their slots (copy stream), unless infllm_block_fetch already did
    if (!L->fetch_issued) {
        int frc = do_fetch(L, a->n_miss, a->h_miss_row, a->h_miss_slot, a->h_miss_unit, a->h_miss_src, st, cs);
        if (frc) return frc;
    }
    L->fetch_issued = false;

    // ---- 2. page table of the global stage: units | init | overflow remainder (slot numbers only: it does not
    //         wait for the fetch, so it is out of the way when the units arrive)
    const int64_t overflow_end = b1 - d.n_local > a->cursor ? b1 - d.n_local : a->cursor;
    int n_pages = 0;
    for (int i = 0; i < d.B * a->n_sel; ++i)
        INFLLM_REQUIRE(a->h_sel_slots[i] >= 0 && a->h_sel_slots[i] < d.max_cached, "block_back: slot %d out of range", a->h_sel_slots[i]);
    // A table of up to 64 entries travels in the launch of the stage that reads it; a longer one is written by a small
    // kernel from the slot list, or uploaded.  INFLLM_PAGE_TABLE_KERNEL=1 keeps the kernel for short tables too.
    infllm_page inline_pages[64];
    bool pages_inline = false;
    if (!L->page_table_kernel) {
        const int room = infllm_inline_page_limit() < 64 ? infllm_inline_page_limit() : 64;
        int n0 = host_pages(d, a, 0, overflow_end, inline_pages, room);
        if (n0 > 0 && (int64_t)d.B * n0 <= room) {
            INFLLM_REQUIRE(n0 <= d.max_pages, "block_back: %d pages exceed the table (%d)", n0, d.max_pages);
            for (int u = 1; u < d.B; ++u) {
                const int nu = host_pages(d, a, u, overflow_end, inline_pages + (int64_t)u * n0, n0);
                INFLLM_REQUIRE(nu == n0, "block_back: batch rows disagree on the page count");
            }
            n_pages = n0;
            pages_inline = true;
        }
    }
    if (pages_inline) {
        ++L->n_tables_inline;
    } else if (d.B * a->n_sel <= kPageJobSlots) {
        PageJob j{};
        j.B = d.B; j.Hkv = d.Hkv; j.bs = bs; j.max_cached = d.max_cached; j.n_sel = a->n_sel; j.init_len = a->init_len;
        j.n_unit_pages = a->n_sel * ((bs + kTile - 1) / kTile);
        j.n_init_pages = (a->init_len + kTile - 1) / kTile;
        int n_over = 0;
        for (int64_t pos = a->cursor; pos < overflow_end; ++n_over) {
            const int64_t row = pos % d.ring_cap;
            int64_t len = overflow_end - pos;
            if (len > kTile) len = kTile;
            if (len > d.ring_cap - row) len = d.ring_cap - row;
            pos += len;
        }
        j.n_pages = n_pages = j.n_unit_pages + j.n_init_pages + n_over;
        INFLLM_REQUIRE(n_pages <= d.max_pages, "block_back: %d pages exceed the table (%d)", n_pages, d.max_pages);
        j.cursor = a->cursor; j.overflow_end = overflow_end; j.ring_cap = d.ring_cap; j.init_cap = d.init_cap;
        j.slab = (const bf16_t *)d.d_slab; j.init_kv = (const bf16_t *)d.d_init_kv;
        j.ring_k = (const bf16_t *)d.d_ring_k_raw; j.ring_v = (const bf16_t *)d.d_ring_v;
        for (int i = 0; i < d.B * a->n_sel; ++i) {
            INFLLM_REQUIRE(a->h_sel_slots[i] >= 0 && a->h_sel_slots[i] < d.max_cached, "block_back: slot %d out of range", a->h_sel_slots[i]);
            j.slots[i] = a->h_sel_slots[i];
        }
        if (n_pages > 0) {
            hipLaunchKernelGGL(build_pages_kernel, dim3((n_pages + 63) / 64, d.B), dim3(64), 0, st, j, d.d_pages);
            INFLLM_CHECK_LAUNCH("build_pages");
            ++L->n_tables_kernel;
        }
    } else
    {
        const int slot = L->page_cur;
        L->page_cur = (slot + 1) % d.page_slots;
        if (L->page_busy[slot]) HIP_OK(hipEventSynchronize(L->page_evt[slot]), "block_back: page slot");
        infllm_page *base = d.h_pages + (int64_t)slot * d.B * d.max_pages;
        for (int u = 0; u < d.B; ++u) {
            infllm_page *pg = base + (int64_t)u * d.max_pages;     // packed to n_pages below
            int n = 0;
            auto push = [&](const bf16_t *k, const bf16_t *v, int64_t hs, int valid) {
                if (n < d.max_pages) pg[n] = infllm_page{k, v, hs, valid, 0};
                ++n;
            };
            for (int s = 0; s < a->n_sel; ++s) {
                const int sl = a->h_sel_slots[u * a->n_sel + s];
                INFLLM_REQUIRE(sl >= 0 && sl < d.max_cached, "block_back: slot %d out of range", sl);
                const bf16_t *kb = (const bf16_t *)d.d_slab + ((int64_t)u * d.max_cached + sl) * slot_elems;
                for (int t0 = 0; t0 < bs; t0 += kTile)
                    push(kb + (int64_t)t0 * kD, kb + unit_elems + (int64_t)t0 * kD, (int64_t)bs * kD, bs - t0 < kTile ? bs - t0 : kTile);
            }
            const bf16_t *ik = (const bf16_t *)d.d_init_kv + (int64_t)u * 2 * d.Hkv * d.init_cap * kD;
            const bf16_t *iv = ik + (int64_t)d.Hkv * d.init_cap * kD;
            for (int t0 = 0; t0 < a->init_len; t0 += kTile)
                push(ik + (int64_t)t0 * kD, iv + (int64_t)t0 * kD, d.init_cap * kD, a->init_len - t0 < kTile ? a->init_len - t0 : kTile);
            const bf16_t *rk = (const bf16_t *)d.d_ring_k_raw + (int64_t)u * d.Hkv * d.ring_cap * kD;
            const bf16_t *rv = (const bf16_t *)d.d_ring_v + (int64_t)u * d.Hkv * d.ring_cap * kD;
            for (int64_t pos = a->cursor; pos < overflow_end;) {
                const int64_t row = pos % d.ring_cap;
                int64_t len = overflow_end - pos;
                if (len > kTile) len = kTile;
                if (len > d.ring_cap - row) len = d.ring_cap - row;
                push(rk + row * kD, rv + row * kD, d.ring_cap * kD, (int)len);
                pos += len;
            }
            INFLLM_REQUIRE(n <= d.max_pages, "block_back: %d pages exceed the table (%d)", n, d.max_pages);
            if (u == 0) n_pages = n;
            INFLLM_REQUIRE(n == n_pages, "block_back: batch rows disagree on the page count");
        }
        if (n_pages > 0) {
            // device layout is [B, n_pages]: pack the rows
            for (int u = 1; u < d.B; ++u)
                for (int i = 0; i < n_pages; ++i) base[(int64_t)u * n_pages + i] = base[(int64_t)u * d.max_pages + i];
            HIP_OK(hipMemcpyAsync(d.d_pages, base, sizeof(infllm_page) * d.B * n_pages, hipMemcpyHostToDevice, st),
                   "block_back: page upload");
            HIP_OK(hipEventRecord(L->page_evt[slot], st), "block_back: event");
            L->page_busy[slot] = 1;
            ++L->n_tables_upload;
        }
    }

    // ---- 3. the global stage and merge (the local stage was launched by block_front or infllm_call_front)
    const int64_t lo = a->b0 > d.n_local ? a->b0 - d.n_local : 0;
    const int lin_tiles = (int)((b1 - lo + kTile - 1) / kTile);
    const int64_t part_o = (int64_t)d.B * d.H * a->n * kD, part_l = (int64_t)d.B * d.H * a->n;
    int rc;
    const int sl = batched ? cur.nsplit : splits_for(d, a->n, lin_tiles);       // key splits of the local stage's partials
    const int tw = L->fetch_wait || L->efetch_wait ? timer_begin(L, 2, a->n, a->n_miss, st) : -1;
    if (L->fetch_wait) {
        HIP_OK(hipStreamWaitEvent(st, L->fetch_done, 0), "block_back: wait fetch");
        L->fetch_wait = false;
    }
    if (L->efetch_wait) {           // the engines write the fetch's sequence number behind the units (a later fetch a larger one)
        HIP_OK(hipStreamWaitValue32(st, L->d_efetch_flag, L->efetch_seq, hipStreamWaitValueGte, 0xffffffffu), "block_back: wait fetch flag");
        L->efetch_wait = false;
    }
    timer_end(L, 2, tw, st);
    int parts = sl;
    if (n_pages > 0) {
        infllm_attn_args at{};
        at.d_q = cur.q_glb;
        at.q_sl = kD; at.q_sh = cur.q_sh; at.q_sb = cur.q_sb;
        at.B = d.B; at.H = d.H; at.Hkv = d.Hkv; at.Lq = a->n;
        at.cap = kTile;
        at.d_pages = d.d_pages; at.n_pages = n_pages;
        at.softmax_scale = d.softmax_scale;
        at.nsplit = splits_for(d, a->n, n_pages);
        // behind the local stage's partials - unless those lie with the call's (then the merge takes two sets)
        at.d_o_part = d.d_o_part + (batched ? 0 : sl * part_o);
        at.d_lse_part = d.d_lse_part + (batched ? 0 : sl * part_l);
        const int ti = timer_begin(L, 1, a->n, n_pages * kTile, st);
        rc = pages_inline ? infllm_attn_paged_inline(nullptr, &at, inline_pages, stream) : infllm_attn_stage(&at, stream);
        timer_end(L, 1, ti, st);
        if (rc) return rc;
        parts += at.nsplit;
        // The next fetch (copy stream or DMA engines) must not overtake these reads.  While guesses are being settled
        // no event is needed for that: a fetch ahead never writes a slot of the selection in use, and a fetch behind
        // a selection is issued by a host that has read that selection, which the stream produced after this stage.
        if ((side || L->efetch_ok) && !L->guessing) {
            HIP_OK(hipEventRecord(L->global_done, st), "block_back: event");
            L->has_global = true;
            L->global_unmarked = false;
        } else
            L->global_unmarked = side || L->efetch_ok;
    }
    // Only the joint log-sum-exp is needed on the way to the next selection, and only by the small score launch of
    // step 4, which joins the partial values itself; the merge (output rows and the joint value for the bulk of the
    // scores) runs once that selection is out (step 5b).  The score-decay policy needs the joint value here.
    const bool lse_now = a->d_unit_mass && a->n_sel > 0;
    const bool one_pass = L->guessing && !lse_now;
    // partials in two places cannot be joined by the score launch: the joint value comes first then as well
    const bool lse_early = lse_now || (batched && !one_pass);
    auto merge = [&](void *out, float *lse) {
        return batched ? infllm_attn_merge2(cur.o_loc, cur.lse_loc, sl, d.d_o_part, d.d_lse_part, parts - sl, d.B, d.H, a->n, out, a->o_sb,
                                            a->o_sh, a->o_sl, lse, stream)
                       : infllm_attn_merge(d.d_o_part, d.d_lse_part, parts, d.B, d.H, a->n, out, a->o_sb, a->o_sh, a->o_sl, lse, stream);
    };
    if (lse_early) {
        rc = merge(nullptr, d.d_lse);
        if (rc) return rc;
    }

    // ---- 3b. attention mass each selected unit received (only the score-decay policy asks for it)
    if (a->d_unit_mass && a->n_sel > 0) {
        INFLLM_REQUIRE(a->d_mass_scratch, "block_back: unit mass without scratch");
        for (int u = 0; u < d.B; ++u)
            for (int i = 0; i < a->n_sel; ++i) {
                infllm_score_args sc{};
                sc.d_q = cur.q_glb + (int64_t)u * cur.q_sb;
                sc.q_sl = kD; sc.q_sh = cur.q_sh; sc.q_sb = 0;
                sc.B = 1; sc.H = d.H; sc.Hkv = d.Hkv; sc.Lq = a->n;
                sc.d_k = (const bf16_t *)d.d_slab + ((int64_t)u * d.max_cached + a->h_sel_slots[u * a->n_sel + i]) * slot_elems;
                sc.k_sl = kD; sc.k_sh = (int64_t)bs * kD; sc.k_sb = 0;
                sc.cap = bs; sc.j_lo = 0; sc.j_hi = bs;
                sc.mask = INFLLM_MASK_NONE; sc.accumulate = 0;
                sc.d_lse = d.d_lse + (int64_t)u * d.H * a->n; sc.softmax_scale = d.softmax_scale;
                sc.d_score = a->d_mass_scratch + ((int64_t)u * a->n_sel + i) * d.H * bs;
                sc.score_sh = bs; sc.score_sb = 0; sc.score_cap = bs;
                rc = infllm_local_score(&sc, stream);
                if (rc) return rc;
            }
        hipLaunchKernelGGL(unit_mass_kernel, dim3(a->n_sel, d.B), dim3(256), 0, st, a->d_mass_scratch, d.H * bs, a->d_unit_mass);
        INFLLM_CHECK_LAUNCH("unit_mass");
        HIP_OK(hipEventRecord(L->mass_done, st), "block_back: event");
        L->mass_pending = true;
    }

    // ---- 4. what the next block's retrieval waits for: scores of the tokens that leave the ring now,
    //         init peeling, representatives of the new units
    bool carved = false;
    int carved_slot = 0;
    L->main_stream = st;
    const int64_t new_cursor = a->cursor + a->init_take + (int64_t)a->n_carve * bs;
    L->cursor = new_cursor;
    L->cursor_known = true;
    const int64_t urgent_hi = new_cursor < b1 ? new_cursor : b1;
    // While the fetches run ahead of the selection nothing waits for this block's selection at once, and the split
    // into an urgent and a bulk score launch only costs stream time: the merge and one score launch come first then.
    if (one_pass) {
        // ... in ONE launch where the key range is long enough for the scoring kernel to have workgroups to spare
        MergeJob job;
        rc = batched ? infllm_merge_job(cur.o_loc, cur.lse_loc, sl, d.d_o_part, d.d_lse_part, parts - sl, d.B, d.H, a->n, a->d_out, a->o_sb,
                                        a->o_sh, a->o_sl, d.d_lse, &job)
                     : infllm_merge_job(d.d_o_part, d.d_lse_part, parts, nullptr, nullptr, 0, d.B, d.H, a->n, a->d_out, a->o_sb, a->o_sh,
                                        a->o_sl, d.d_lse, &job);
        if (rc) return rc;
        rc = 1;
        if (!L->score_merge_apart && parts <= 8 && b1 > lo) {
            const infllm_score_args sc = local_score_args(L, a->n, a->b0, cur, lo, b1, 0);
            rc = infllm_local_score_merged(&sc, &job, stream);
            if (rc < 0) return rc;
            if (rc == 0) ++L->n_score_merged;
        }
        if (rc == 1) {
            ++L->n_score_apart;
            rc = merge(a->d_out, d.d_lse);
            if (rc) return rc;
            rc = run_local_score(L, a->n, a->b0, cur, lo, b1, 0, stream);
        }
    } else
        rc = run_local_score(L, a->n, a->b0, cur, lo, urgent_hi, lse_early ? 0 : parts, stream);
    if (rc) return rc;
    int64_t cursor = a->cursor;
    if (a->init_take > 0) {
        INFLLM_REQUIRE(a->init_len + a->init_take <= d.init_cap, "block_back: init overflow");
        bf16_t *ik = (bf16_t *)d.d_init_kv + (int64_t)a->init_len * kD;
        const int64_t sb = 2 * (int64_t)d.Hkv * d.init_cap * kD, sh = d.init_cap * kD;
        rc = infllm_gather_rows(d.d_ring_k_raw, d.ring_cap, d.B, d.Hkv, cursor, a->init_take, a->init_take, ik, sb, 0, sh, stream);
        if (rc) return rc;
        rc = infllm_gather_rows(d.d_ring_v, d.ring_cap, d.B, d.Hkv, cursor, a->init_take, a->init_take,
                                ik + (int64_t)d.Hkv * d.init_cap * kD, sb, 0, sh, stream);
        if (rc) return rc;
        cursor += a->init_take;
    }
    if (a->n_carve > 0) {
        // representatives of the new units, and in the same launch their rows out of the rings into a staging slot
        // (from there they go to pinned host memory, off the critical path)
        INFLLM_REQUIRE(a->d_rep_out && a->h_carve_dst, "block_back: null carve outputs");
        for (int i = 0; i < a->n_carve; ++i) INFLLM_REQUIRE(a->h_carve_dst[i], "block_back: null carve destination");
        if (L->off.pending && d.carve_slots < 2) {      // one staging slot: the earlier units have to leave it first
            int drc = 0;
            if (L->dma_ok) {
                drc = carve_wait(L);
                if (drc) return drc;
                drc = issue_offload_dma(L);
                if (drc < 0) return drc;
            }
            if (drc == 0) {
                rc = issue_offload(L, cs);
                if (rc) return rc;
            }
        }
        const int slot = L->carve_cur;
        L->carve_cur = (slot + 1) % d.carve_slots;
        if (L->carve_busy[slot]) HIP_OK(hipEventSynchronize(L->carve_evt[slot]), "block_back: carve slot");
        rc = dma_wait_slot(L, slot, "block_back");
        if (rc) return rc;
        const int64_t unit_all = (int64_t)d.B * slot_elems;                       // one unit, all batch rows
        bf16_t *stage = (bf16_t *)d.d_carve_stage + (int64_t)slot * d.max_carve * unit_all;
        rc = infllm_repr_keys_carve(d.d_ring_score, d.d_ring_k_raw, d.ring_cap, d.B, d.H, d.Hkv, cursor, bs, a->n_carve, d.repr_topk,
                                    a->d_rep_out, a->rep_sb, a->rep_su, a->d_repr_idx, d.d_ring_v, stage, stage + unit_elems, slot_elems,
                                    unit_all, (int64_t)bs * kD, stream);
        if (rc) return rc;
        L->stage_first[slot] = a->n_units;
        L->stage_count[slot] = a->n_carve;
        carved = true;
        carved_slot = slot;
    }
    // ---- 5. the next block's retrieval (its prologue ran in block_front)
    const int32_t seq_before = L->topk_seq;
    L->topk_pending = false;
    const int n_units_next = a->n_units + a->n_carve;
    if (L->prepared && n_units_next > d.topk && !(a->flags & INFLLM_NO_RETRIEVAL)) {
        INFLLM_REQUIRE(a->d_reps && a->d_unit_scores, "block_back: null representative / score buffer");
        // with the lists of a prepared call: the new units' scores for the call's later blocks, the next block's
        // selection and the candidates of the block after it, one launch.  (The first block of such a call selects
        // for the second as a block on its own would, from the candidates block_front chose, and makes the lists
        // behind that selection: see below.)
        const bool make_lists = L->call_lists_pending && batched && a->b0 == L->batch_b0 && a->n_units == L->call_n0 &&
                                call_rank_fits(L, a->n_units, a->n_carve);
        if (batched && a->b0 == L->batch_b0) L->call_lists_pending = false;
        const int j_next = L->call_lists && batched ? (int)((b1 - L->batch_b0) / d.exc) : -1;
        if (j_next >= 1 && j_next < L->call_blocks && block_in_batch(L, b1, L->prepared_n) && call_rank_fits(L, a->n_units, a->n_carve)) {
            rc = run_call_rank(L, a->d_reps, a->rep_sb, a->rep_su, a->n_units, a->n_carve, j_next, j_next + 1 < L->call_blocks ? j_next + 1 : -1,
                               stream);
            if (rc) return rc;
            rc = 0;
        } else {
            L->call_lists = false;      // (lists that no longer fit their kernel: the rest of the call selects over all units)
            const bool merge = L->cand_units == a->n_units && d.topk + a->n_carve <= 64;
            rc = merge ? run_score_new_rank(L, a->d_reps, a->rep_sb, a->rep_su, a->d_unit_scores, a->unit_scores_sb, a->n_units, a->n_carve, stream)
                       : 1;
        }
        if (rc < 0) return rc;
        if (rc == 1) {                  // the two steps on their own
            const bool merge = L->cand_units == a->n_units && d.topk + a->n_carve <= 64;
            // (the older units were scored by block_front, unless the call's lists stood in for that)
            const int first = L->scored_units == a->n_units ? a->n_units : 0;
            rc = run_unit_scores(L, a->d_reps, a->rep_sb, a->rep_su, a->d_unit_scores, a->unit_scores_sb, first, n_units_next - first, L->fresh.qbar,
                                 stream);
            if (rc) return rc;
            if (merge)
                rc = run_topk_merge(L, a->d_unit_scores, a->unit_scores_sb, a->n_units, a->n_carve, stream);
            else
                rc = run_topk(L, a->d_unit_scores, a->unit_scores_sb, n_units_next, stream);
            if (rc) return rc;
        }
        if (make_lists) {
            // The lists of the call's other blocks, two launches for the whole call, BEHIND the second block's selection:
            // the host is busy with that selection and the stream with the wait for its fetch while they are made.
            // Then the first ranking from them: the units just carved under the later blocks' mean queries, and the
            // third block's candidates.
            const int C = d.H * kD;
            for (int u = 0; u < d.B; ++u) {
                rc = infllm_score_topk_queries((const bf16_t *)a->d_reps + (int64_t)u * a->rep_sb, a->rep_su, L->call_n0, C,
                                               L->bd.d_qbar + ((int64_t)d.B + u) * C, (int64_t)d.B * C, L->call_blocks - 1, d.topk,
                                               L->call_scores + ((int64_t)d.B + u) * L->call_cols, (int64_t)d.B * L->call_cols,
                                               L->d_base + ((int64_t)d.B + u) * d.topk, (int64_t)d.B * d.topk, stream);
                if (rc) return rc < 0 ? rc : infllm_fail(-2, "block_back: no scoring kernel after the geometry check");
            }
            L->call_lists = true;
            if (L->call_blocks > 2) {
                rc = run_call_rank(L, a->d_reps, a->rep_sb, a->rep_su, a->n_units, a->n_carve, -1, 2, stream);
                if (rc) return rc;
            }
        }
    }
    L->cand_units = -1;
    if (carved) {
        // host work that the selection just launched does not have to wait for
        if (L->off.pending) {
            // the units of an earlier block are still waiting: their copy into staging was queued a whole block ago, so
            // the host gets through this wait at once and the engine can take them; else the copy stream does
            int drc = 0;
            if (L->dma_ok) {
                drc = carve_wait(L);
                if (drc) return drc;
                drc = issue_offload_dma(L);
                if (drc < 0) return drc;
            }
            if (drc == 0) {
                rc = issue_offload(L, cs);
                if (rc) return rc;
            }
        }
        L->off.after_seq = 0;
        L->off.has_event = false;
        L->off.pending = true;
        L->off.slot = carved_slot;
        L->off.first_unit = a->n_units;
        L->off.count = a->n_carve;
        L->off.dst.assign(a->h_carve_dst, a->h_carve_dst + a->n_carve);
        L->copy_stream = cs;
        // An event record costs the stream 2-3 us.  When a selection kernel that publishes a sequence number follows
        // the copy into staging, that number tells the host as much; otherwise the event does.
        if (L->dma_ok && L->topk_seq != seq_before) L->off.after_seq = L->topk_seq;
        else {
            rc = carve_event(L);
            if (rc) return rc;
        }
    }
    // ---- 5b. the block's output rows
    if (!one_pass) {
        rc = merge(a->d_out, lse_early ? nullptr : d.d_lse);
        if (rc) return rc;
        // ---- 6. off the critical path: the rest of the local score, new units to pinned host memory
        rc = run_local_score(L, a->n, a->b0, cur, urgent_hi > lo ? urgent_hi : lo, b1, 0, stream);
        if (rc) return rc;
    }
    return 0;
}

namespace {
int end_of_call(Layer *L, void *copy_stream, bool finish_copies);
}

extern "C" int infllm_layer_flush(void *layer, void *copy_stream) {
    INFLLM_REQUIRE(layer, "layer_flush: null layer");
    return end_of_call((Layer *)layer, copy_stream, true);
}

extern "C" int infllm_layer_end_call(void *layer, void *copy_stream) {
    INFLLM_REQUIRE(layer, "layer_end_call: null layer");
    return end_of_call((Layer *)layer, copy_stream, false);
}

namespace {
int end_of_call(Layer *L, void *copy_stream, bool finish_copies) {
    if (L->ahead.active) {                      // a guess nobody settled: put back what it overwrote
        L->ahead.active = false;
        hipStream_t cs = (hipStream_t)copy_stream;
        int rrc = ahead_repair(L, nullptr, 0, nullptr, nullptr, nullptr, nullptr, cs, cs);
        if (rrc) return rrc;
        // nothing later is ordered behind this repair by itself: finish it here (it is not a path a stream takes)
        if (L->efetch_ok) {
            rrc = efetch_wait_all(L, "layer_flush");
            if (rrc) return rrc;
        }
        HIP_OK(hipStreamSynchronize(cs), "layer_flush: repair");
        L->fetch_wait = L->efetch_wait = false;
    }
    if (L->off.pending && finish_copies) {
        int drc = issue_offload_dma(L);
        if (drc < 0) return drc;
        if (drc == 0) {
            drc = issue_offload(L, (hipStream_t)copy_stream);
            if (drc) return drc;
        }
    }
    for (size_t s = 0; s < L->dma_busy.size() && finish_copies; ++s) {       // engine copies are not ordered by any stream: finish them here
        const int wrc = dma_wait_slot(L, (int)s, "layer_flush");
        if (wrc) return wrc;
    }
    L->batch_live = false;
    if (L->main_stream_known) {
        HIP_OK(hipEventRecord(L->idle_main, L->main_stream), "layer_flush: event");
        HIP_OK(hipEventRecord(L->idle_copy, (hipStream_t)copy_stream), "layer_flush: event");
        L->idle_recorded = true;
        L->unflushed = false;
    }
    return 0;
}
}  // namespace
