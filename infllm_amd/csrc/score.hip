// Column sums of the final attention probabilities of one linear stage
// (inf_llm/attention/dot_production_attention/torch_impl.py:27-28): the "local score"
// that InfLLM accumulates per token to choose representative keys
// (inf_llm/attention/context_manager.py:623-625).
//
// It needs the final log-sum-exp of every query, so it runs after the merge and
// recomputes Q.K^T.  Orientation: S[query, key] with keys in the MFMA column, so a lane
// owns one key and the column sum is a running per-lane scalar.  A workgroup owns 256
// consecutive keys of one query head: each of its 4 waves keeps 64 keys in registers
// (B operand) for the whole kernel, while tiles of 64 or 128 queries stream through LDS
// (A operand, shared by the 4 waves, double buffered).  Exactly one lane writes each
// (head, key) cell, so results are deterministic.
#include "common.h"
#include <type_traits>

namespace {

constexpr int kQPad = kD + 8;              // LDS row of Q (bf16 elements): 272 bytes rotates the banks

// KS = 32-key halves per wave: 2 for long key ranges; 1 halves the work of a wave per query stage, which is what
// bounds the short launches that sit on the critical path between two blocks.  QS = queries per LDS stage: a short
// launch is a chain of stages that each wait for one global load (there is next to no arithmetic to hide it behind),
// so it takes stages of 128 queries and half as many of them.
//
// MERGE: the launch also carries the merge of the block's partial attention outputs: every scoring workgroup merges
// two (row, 8 dims) pieces per thread (merge_issue / merge_finish of common.h) while it waits for its keys.  The two
// kinds of work do not depend on each other - the scoring workgroups join the partial log-sum-exps themselves, by
// the merge's own arithmetic - and the merge is a handful of loads per thread that are in flight during a wait the
// workgroup has anyway: one launch instead of two on the chain from one block's selection to the next, and no
// workgroups of its own that would queue for the scoring workgroups' places.  In this form the joined log-sum-exps of
// ALL the launch's queries are put into LDS once, in the same wait, instead of stage by stage.
struct ScoreMerge {
    MergeJob job;
    int32_t score_tiles;               // blockIdx.y below this scores, from there on merges
};
struct NoScoreMerge {};

template <int KS, int QS, bool MERGE = false>
__global__ __launch_bounds__(256, 2) void local_score_kernel(infllm_score_args a, std::conditional_t<MERGE, ScoreMerge, NoScoreMerge> sm) {
    constexpr int kWaveKeys = 32 * KS, kKeysPerWg = 4 * kWaveKeys, kQStage = QS;
    int n_tiles = gridDim.y;
    PartSets lps{a.n_parts, 0, 0};
    if constexpr (MERGE) {
        n_tiles = sm.score_tiles;
        if ((int)blockIdx.y >= n_tiles) {
            merge_piece(sm.job, ((int64_t)((int)blockIdx.y - n_tiles) * gridDim.x + blockIdx.x) * 256 + threadIdx.x);
            return;
        }
        lps = sm.job.ps;
    }
    extern __shared__ __attribute__((aligned(16))) char score_lds[];
    bf16_t(*Qs)[kQStage][kQPad] = (bf16_t(*)[kQStage][kQPad])score_lds;                               // [2][QS][kQPad]
    float(*Ls)[kQStage] = (float(*)[kQStage])(score_lds + 2 * kQStage * kQPad * sizeof(bf16_t));      // [2][QS]
    [[maybe_unused]] float *Lall = (float *)Ls;                                                        // MERGE: [Lq rounded up to QS]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int col = lane & 31, grp = lane >> 5;
    const int G = a.H / a.Hkv;
    // blockIdx.x walks the kv heads first, then the query heads of a group: workgroups go to the 8 XCDs round-robin by
    // linear id, so with 8 (16, ...) kv heads the query heads that share a K tile sit behind the same L2 and that tile
    // leaves HBM once instead of once per query head
    const int b = blockIdx.x / a.H, hx = blockIdx.x % a.H, g = hx % a.Hkv, h = g * G + hx / a.Hkv;
    // Workgroups are dispatched x fastest: all heads of one key tile, then the next tile.  The two tiles at either end
    // of a masked key range see only part of the queries and finish early, so they go last: when the grid is a little
    // more than what the chip holds at once, the workgroups that start late are then the short ones.
    const int slot = blockIdx.y;
    int tile = slot;
    if (n_tiles >= 6 && a.mask != INFLLM_MASK_NONE)
        tile = slot < n_tiles - 4 ? slot + 2 : slot == n_tiles - 4 ? 1 : slot == n_tiles - 3 ? n_tiles - 2 : slot == n_tiles - 2 ? 0 : n_tiles - 1;
    const int64_t jg = (a.j_lo / kWaveKeys + (int64_t)tile * 4) * kWaveKeys;         // first key of the workgroup
    const int64_t j0 = jg + (int64_t)wave * kWaveKeys;                               // first key of this wave
    const float scale = a.softmax_scale * 1.4426950408889634f;

    // ---- this wave's 64 keys as the B operand (lane = key column)
    bf16x8 kreg[KS][kD / 16];
    bool jok[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const int64_t j = j0 + ks * 32 + col;
        jok[ks] = j >= a.j_lo && j < a.j_hi;
        const bf16_t *krow = (const bf16_t *)a.d_k + (int64_t)b * a.k_sb + (int64_t)g * a.k_sh + (j % a.cap) * a.k_sl;
#pragma unroll
        for (int kk = 0; kk < kD / 16; ++kk) {
            u32x4 raw = jok[ks] ? *(const u32x4 *)(krow + kk * 16 + grp * 8) : u32x4{0, 0, 0, 0};
            kreg[ks][kk] = __builtin_bit_cast(bf16x8, raw);
        }
    }

    // ---- query range: what the workgroup stages, and what this wave needs of it
    auto query_range = [&](int64_t jf, int64_t jl, int64_t &lo, int64_t &hi) {   // keys [jf, jl] -> queries [lo, hi)
        lo = 0;
        hi = a.Lq;
        jf = max(jf, a.j_lo);
        jl = min(jl, a.j_hi - 1);
        if (jl < jf) {
            hi = 0;
            return;
        }
        if (a.mask == INFLLM_MASK_WINDOW) {
            lo = max(lo, jf - a.offset);
            hi = min(hi, jl - a.offset + a.window);
        } else if (a.mask == INFLLM_MASK_COMPLEMENT) {
            lo = max(lo, jf - a.offset + a.window);
        }
    };
    int64_t g_lo, g_hi, w_lo, w_hi;
    query_range(jg, jg + kKeysPerWg - 1, g_lo, g_hi);
    query_range(j0, j0 + kWaveKeys - 1, w_lo, w_hi);
    const int st_lo = (int)(g_lo / kQStage), st_hi = g_hi > g_lo ? (int)((g_hi - 1) / kQStage) + 1 : st_lo;

    const bf16_t *qbase = (const bf16_t *)a.d_q + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh;
    const float *lse = a.d_lse + ((int64_t)b * a.H + h) * a.Lq;
    const int ld_chunk = tid & 15, ld_row = tid >> 4;
    u32x4 qbuf[kQStage / 16];
    float lbuf = 0.f;
    auto load_stage = [&](int s) {
        const int i0 = s * kQStage;
#pragma unroll
        for (int i = 0; i < kQStage / 16; ++i) {
            const int qi = i0 + ld_row + 16 * i;
            qbuf[i] = qi < a.Lq ? *(const u32x4 *)(qbase + (int64_t)qi * a.q_sl + ld_chunk * 8) : u32x4{0, 0, 0, 0};
        }
        if (!MERGE && tid < kQStage) {
            if (i0 + tid >= a.Lq) {
                lbuf = INFINITY;                                                  // +inf => probability 0
            } else if (a.n_parts <= 0) {
                lbuf = lse[i0 + tid];
            } else {                                                              // join the stages' partial values here
                const int64_t rows = (int64_t)a.B * a.H * a.Lq;
                float m = -INFINITY, den = 0.f;
                for (int p0 = 0; p0 < a.n_parts; p0 += 8) {
                    float l8[8], m8 = -INFINITY;
#pragma unroll
                    for (int i = 0; i < 8; ++i) l8[i] = p0 + i < a.n_parts ? lse[lps.l(p0 + i, rows) + i0 + tid] : -INFINITY;
#pragma unroll
                    for (int i = 0; i < 8; ++i) m8 = fmaxf(m8, l8[i]);
                    if (m8 == -INFINITY) continue;
                    const float m_new = fmaxf(m, m8);
                    den *= __builtin_amdgcn_exp2f(m - m_new);
#pragma unroll
                    for (int i = 0; i < 8; ++i) den += __builtin_amdgcn_exp2f(l8[i] - m_new);
                    m = m_new;
                }
                lbuf = den > 0.f ? m + log2f(den) : INFINITY;
            }
        }
    };
    auto store_stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < kQStage / 16; ++i) *(u32x4 *)&Qs[buf][ld_row + 16 * i][ld_chunk * 8] = qbuf[i];
        if (!MERGE && tid < kQStage) Ls[buf][tid] = lbuf;
    };

    float colsum[KS] = {};
    if (st_hi > st_lo) load_stage(st_lo);
    if constexpr (MERGE) {
        // joined log-sum-exps of every query of the launch (the per-stage join above for one group of 8 partials)
        const int64_t rows = (int64_t)a.B * a.H * a.Lq;
        const int lq_pad = (a.Lq + kQStage - 1) / kQStage * kQStage;
        for (int i = tid; i < lq_pad; i += 256) {
            float l8[8], m8 = -INFINITY, den = 0.f;
#pragma unroll
            for (int p = 0; p < 8; ++p) l8[p] = i < a.Lq && p < a.n_parts ? lse[lps.l(p, rows) + i] : -INFINITY;
#pragma unroll
            for (int p = 0; p < 8; ++p) m8 = fmaxf(m8, l8[p]);
            if (m8 != -INFINITY) {
#pragma unroll
                for (int p = 0; p < 8; ++p) den += __builtin_amdgcn_exp2f(l8[p] - m8);
            }
            Lall[i] = den > 0.f ? m8 + log2f(den) : INFINITY;              // +inf => probability 0
        }
    }
    if (st_hi > st_lo) {
        store_stage(0);
        if (st_lo + 1 < st_hi) load_stage(st_lo + 1);
    }
    __syncthreads();
    for (int s = st_lo; s < st_hi; ++s) {
        const int cur = (s - st_lo) & 1;
        const int64_t i0 = (int64_t)s * kQStage;
        // Fast path: every (query, key) pair of this stage and this wave's keys is visible.  Then the sub-tiles of 32
        // queries are software pipelined: the MFMAs of sub-tile qs+1 are issued before the exponentials of sub-tile qs,
        // in ONE basic block, so that the scheduler can interleave them (an MFMA runs for 32 cycles in the background
        // of the VALU); with everything behind per-sub-tile branches the two kinds of work only ever alternated.
        bool fast = i0 >= w_lo && i0 + kQStage <= w_hi && i0 + kQStage <= a.Lq && j0 >= a.j_lo && j0 + kWaveKeys <= a.j_hi;
        if (a.mask == INFLLM_MASK_WINDOW)
            fast = fast && (i0 - (j0 + kWaveKeys - 1) + a.offset >= 0) && (i0 + kQStage - 1 - j0 + a.offset < a.window);
        if (a.mask == INFLLM_MASK_COMPLEMENT) fast = fast && (i0 - (j0 + kWaveKeys - 1) + a.offset >= a.window);
        if (fast) {
            constexpr int kSub = kQStage / 32;
            f32x16 sacc[2][KS];
            f32x4 l4[2][4];
            auto issue = [&](int qs, int pb) {
                bf16x8 qa[kD / 16];                              // A operand: lane = query row
                const bf16_t *qrow = &Qs[cur][qs * 32 + col][grp * 8];
#pragma unroll
                for (int kk = 0; kk < kD / 16; ++kk) qa[kk] = *(const bf16x8 *)(qrow + kk * 16);
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) l4[pb][q4] = *(const f32x4 *)(MERGE ? &Lall[i0 + qs * 32 + 8 * q4 + 4 * grp] : &Ls[cur][qs * 32 + 8 * q4 + 4 * grp]);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int r = 0; r < 16; ++r) sacc[pb][ks][r] = 0.f;
#pragma unroll
                for (int kk = 0; kk < kD / 16; ++kk)
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        sacc[pb][ks] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa[kk], kreg[ks][kk], sacc[pb][ks], 0, 0, 0);
            };
            issue(0, 0);
#pragma unroll
            for (int qs = 0; qs < kSub; ++qs) {
                const int pb = qs & 1;
                if (qs + 1 < kSub) issue(qs + 1, pb ^ 1);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    float acc = 0.f;
#pragma unroll
                    for (int r = 0; r < 16; ++r)
                        acc += __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[pb][ks][r], scale, -l4[pb][r >> 2][r & 3]));
                    colsum[ks] += acc;
                }
                if (qs + 1 < kSub) {
                    // one MFMA, then its share of the exponentials (16 * KS of each per sub-tile)
#pragma unroll
                    for (int i = 0; i < 8 * KS; ++i) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      // MFMA
                        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);      // VALU
                        __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);      // transcendental
                    }
                }
            }
        } else
        if (i0 < w_hi && i0 + kQStage > w_lo) {                  // wave-uniform
#pragma unroll
            for (int qs = 0; qs < kQStage / 32; ++qs) {
                const int64_t iq = i0 + qs * 32;
                if (iq >= w_hi || iq + 32 <= w_lo) continue;
                bf16x8 qa[kD / 16];                              // A operand: lane = query row
                const bf16_t *qrow = &Qs[cur][qs * 32 + col][grp * 8];
#pragma unroll
                for (int kk = 0; kk < kD / 16; ++kk) qa[kk] = *(const bf16x8 *)(qrow + kk * 16);
                f32x4 l4[4];                                     // lse of rows 8*(r>>2) + 4*grp + (r&3)
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) l4[q4] = *(const f32x4 *)(MERGE ? &Lall[i0 + qs * 32 + 8 * q4 + 4 * grp] : &Ls[cur][qs * 32 + 8 * q4 + 4 * grp]);
                // both key halves at once: two independent accumulator chains keep the matrix pipe busy
                f32x16 sacc2[KS];
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int r = 0; r < 16; ++r) sacc2[ks][r] = 0.f;
#pragma unroll
                for (int kk = 0; kk < kD / 16; ++kk)
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks)
                        sacc2[ks] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa[kk], kreg[ks][kk], sacc2[ks], 0, 0, 0);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const f32x16 sacc = sacc2[ks];
                    // dist(i, j) = i - j + offset for the first query row and this lane's key
                    const int64_t jk = j0 + ks * 32;
                    const int64_t e0 = iq - jk + a.offset;       // query iq, key jk
                    bool need_mask = false;
                    if (a.mask == INFLLM_MASK_WINDOW) need_mask = (e0 - 31 < 0) || (e0 + 31 >= a.window);
                    if (a.mask == INFLLM_MASK_COMPLEMENT) need_mask = (e0 - 31 < a.window);
                    float acc = 0.f;
                    if (!need_mask) {
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            acc += __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[r], scale, -l4[r >> 2][r & 3]));
                    } else {
                        const int d0 = (int)min(max(e0, (int64_t)-(1 << 29)), (int64_t)(1 << 29)) - col;
                        const int win = (int)min(a.window, (int64_t)(1 << 30));
#pragma unroll
                        for (int r = 0; r < 16; ++r) {
                            const int dist = d0 + 8 * (r >> 2) + 4 * grp + (r & 3);
                            bool vis = true;
                            if (a.mask == INFLLM_MASK_WINDOW) vis = dist >= 0 && dist < win;
                            if (a.mask == INFLLM_MASK_COMPLEMENT) vis = dist >= win;
                            const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[r], scale, -l4[r >> 2][r & 3]));
                            acc += vis ? p : 0.f;
                        }
                    }
                    colsum[ks] += acc;
                }
            }
        }
        if (s + 1 < st_hi) {
            store_stage(cur ^ 1);
            if (s + 2 < st_hi) load_stage(s + 2);
        }
        __syncthreads();
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        const float tot = colsum[ks] + wave_xor32(colsum[ks]);
        const int64_t j = j0 + ks * 32 + col;
        if (grp == 0 && jok[ks]) {
            float *dst = a.d_score + (int64_t)b * a.score_sb + (int64_t)h * a.score_sh + (j % a.score_cap);
            *dst = a.accumulate ? *dst + tot : tot;
        }
    }
}

}  // namespace

namespace {

int check_score_args(const infllm_score_args *a) {
    INFLLM_REQUIRE(a != nullptr, "local_score: null argument block");
    INFLLM_REQUIRE(a->d_q && a->d_k && a->d_lse && a->d_score, "local_score: null pointer");
    INFLLM_REQUIRE(a->B > 0 && a->H > 0 && a->Hkv > 0 && a->H % a->Hkv == 0 && a->Lq > 0,
                   "local_score: bad geometry B=%d H=%d Hkv=%d Lq=%d", a->B, a->H, a->Hkv, a->Lq);
    INFLLM_REQUIRE(a->cap > 0 && a->score_cap > 0 && a->j_lo >= 0, "local_score: bad ring sizes");
    INFLLM_REQUIRE(a->j_hi - a->j_lo <= a->cap && a->j_hi - a->j_lo <= a->score_cap,
                   "local_score: key range [%lld,%lld) exceeds the ring", (long long)a->j_lo, (long long)a->j_hi);
    INFLLM_REQUIRE(a->mask >= 0 && a->mask <= 2, "local_score: unknown mask %d", a->mask);
    INFLLM_REQUIRE(a->n_parts >= 0 && a->n_parts <= 1024, "local_score: %d partial log-sum-exps", a->n_parts);
    INFLLM_REQUIRE((a->q_sl % 8 | a->q_sh % 8 | a->q_sb % 8 | a->k_sl % 8 | a->k_sh % 8 | a->k_sb % 8) == 0,
                   "local_score: strides must be multiples of 8");
    INFLLM_REQUIRE(a->j_hi - a->j_lo <= (int64_t)65000 * 256, "local_score: key range of %lld rows exceeds one launch",
                   (long long)(a->j_hi - a->j_lo));
    return 0;
}

size_t score_lds_bytes(int qs) { return (size_t)(2 * qs * kQPad * sizeof(bf16_t) + 2 * qs * sizeof(float)); }
constexpr int kMergedMaxLq = 2048;                     // MERGE: 4 bytes of LDS per query of the launch
size_t score_lds_bytes_merged(int qs, int lq) { return (size_t)(2 * qs * kQPad * sizeof(bf16_t) + (size_t)((lq + qs - 1) / qs * qs) * sizeof(float)); }

int score_lds_setup() {
    static bool lds_set = false;                       // dynamic LDS above 64 KiB must be enabled once per kernel
    if (!lds_set) {
        hipError_t e = hipFuncSetAttribute((const void *)local_score_kernel<1, 128>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)score_lds_bytes(128));
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void *)local_score_kernel<2, 128>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)score_lds_bytes(128));
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void *)local_score_kernel<2, 128, true>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)score_lds_bytes_merged(128, kMergedMaxLq));
        if (e != hipSuccess) return infllm_fail(-2, "local_score: %s", hipGetErrorString(e));
        lds_set = true;
    }
    return 0;
}

}  // namespace

extern "C" int infllm_local_score(const infllm_score_args *a, void *stream) {
    int rc = check_score_args(a);
    if (rc) return rc;
    if (a->j_hi <= a->j_lo) return 0;
    rc = score_lds_setup();
    if (rc) return rc;
    if (a->j_hi - a->j_lo > 1024) {
        const int64_t tiles = (a->j_hi - 1) / 64 - a->j_lo / 64 + 1;
        hipLaunchKernelGGL((local_score_kernel<2, 128>), dim3(a->B * a->H, (unsigned)((tiles + 3) / 4)), dim3(256), score_lds_bytes(128),
                           (hipStream_t)stream, *a, NoScoreMerge{});
    } else {
        const int64_t tiles = (a->j_hi - 1) / 32 - a->j_lo / 32 + 1;
        hipLaunchKernelGGL((local_score_kernel<1, 128>), dim3(a->B * a->H, (unsigned)((tiles + 3) / 4)), dim3(256), score_lds_bytes(128),
                           (hipStream_t)stream, *a, NoScoreMerge{});
    }
    INFLLM_CHECK_LAUNCH("local_score");
    return 0;
}

// library-internal: the local score of a block and the merge of its partial attention outputs in one launch.  The
// scores are taken against the joint log-sum-exp of the job's partials (a->d_lse and a->n_parts are set from the job);
// returns 1, with nothing launched, where the one-launch form does not apply (short key ranges).
int infllm_local_score_merged(const infllm_score_args *a, const MergeJob *job, void *stream) {
    INFLLM_REQUIRE(a && job, "local_score_merged: null argument");
    INFLLM_REQUIRE(job->out && job->B == a->B && job->H == a->H && job->Lq == a->Lq && job->P >= 1 && job->P <= 8,
                   "local_score_merged: the merge does not belong to these queries");
    infllm_score_args sc = *a;
    sc.d_lse = job->lse_part;
    sc.n_parts = job->P;
    int rc = check_score_args(&sc);
    if (rc) return rc;
    if (sc.j_hi - sc.j_lo <= 1024 || sc.Lq > kMergedMaxLq) return 1;
    rc = score_lds_setup();
    if (rc) return rc;
    const int64_t tiles = (sc.j_hi - 1) / 64 - sc.j_lo / 64 + 1;
    const int score_tiles = (int)((tiles + 3) / 4);
    const int64_t merge_wgs = ((int64_t)job->B * job->H * job->Lq * 16 + 255) / 256;
    const int gx = sc.B * sc.H;
    const int merge_slots = (int)((merge_wgs + gx - 1) / gx);
    hipLaunchKernelGGL((local_score_kernel<2, 128, true>), dim3(gx, (unsigned)(score_tiles + merge_slots)), dim3(256),
                       score_lds_bytes_merged(128, sc.Lq), (hipStream_t)stream, sc, ScoreMerge{*job, score_tiles});
    INFLLM_CHECK_LAUNCH("local_score_merged");
    return 0;
}
