// Column sums of the final attention probabilities of one linear stage
// (inf_llm/attention/dot_production_attention/torch_impl.py:27-28): the "local score"
// that InfLLM accumulates per token to choose representative keys
// (inf_llm/attention/context_manager.py:623-625).
//
// It needs the final log-sum-exp of every query, so it runs after the merge and
// recomputes Q.K^T.  Orientation: S[query, key] with keys in the MFMA column, so a lane
// owns one key and the column sum is a running per-lane scalar.  A workgroup owns 64
// keys of one kv head; its waves take the query heads of the group (two waves per head,
// one 32-key half each, when the group has fewer than 4 heads); K stays in registers
// and query tiles stream from L2.  Exactly one lane writes each (head, key) cell, so
// results are deterministic.
#include "common.h"

namespace {

constexpr int kQT = 32;

__global__ __launch_bounds__(256, 2) void local_score_kernel(infllm_score_args a) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int col = lane & 31, grp = lane >> 5;
    const int G = a.H / a.Hkv;
    const int b = blockIdx.y / a.Hkv, g = blockIdx.y % a.Hkv;
    const int64_t j0 = ((a.j_lo >> 6) + blockIdx.x) * (int64_t)kTile;       // first key of this tile

    const int halves = G >= 4 ? 1 : 2;          // waves per head
    const int head_step = 4 / halves;
    const int ks_lo = halves == 1 ? 0 : (wave & 1), ks_hi = halves == 1 ? 2 : (wave & 1) + 1;
    const float scale = a.softmax_scale * 1.4426950408889634f;

    // queries that can see any key of the tile
    int64_t i_lo = 0, i_hi = a.Lq;               // [i_lo, i_hi)
    const int64_t jf = max(j0, a.j_lo), jl = min(j0 + kTile, a.j_hi) - 1;
    if (a.mask == INFLLM_MASK_WINDOW) {
        i_lo = max(i_lo, jf - a.offset);
        i_hi = min(i_hi, jl - a.offset + a.window);
    } else if (a.mask == INFLLM_MASK_COMPLEMENT) {
        i_lo = max(i_lo, jf - a.offset + a.window);
    }
    const int qt_lo = (int)(i_lo / kQT), qt_hi = i_hi > i_lo ? (int)((i_hi - 1) / kQT) + 1 : qt_lo;

    for (int hg = wave / halves; hg < G; hg += head_step) {
        const int h = g * G + hg;
        // ---- keys of this wave in registers (B operand: lane = key column)
        bf16x8 kreg[2][kD / 16];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            const int64_t j = j0 + ks * 32 + col;
            const bool ok = ks >= ks_lo && ks < ks_hi && j >= a.j_lo && j < a.j_hi;
            const bf16_t *krow = (const bf16_t *)a.d_k + (int64_t)b * a.k_sb + (int64_t)g * a.k_sh + (j % a.cap) * a.k_sl;
#pragma unroll
            for (int kk = 0; kk < kD / 16; ++kk) {
                u32x4 raw = ok ? *(const u32x4 *)(krow + kk * 16 + grp * 8) : u32x4{0, 0, 0, 0};
                kreg[ks][kk] = __builtin_bit_cast(bf16x8, raw);
            }
        }
        float colsum[2] = {0.f, 0.f};
        const bf16_t *qbase = (const bf16_t *)a.d_q + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh;
        const float *lse = a.d_lse + ((int64_t)b * a.H + h) * a.Lq;

        for (int qt = qt_lo; qt < qt_hi; ++qt) {
            const int i0 = qt * kQT;
            bf16x8 qa[kD / 16];                  // A operand: lane = query row
            {
                const int qi = i0 + col;
                const bool ok = qi < a.Lq;
                const bf16_t *qrow = qbase + (int64_t)qi * a.q_sl;
#pragma unroll
                for (int kk = 0; kk < kD / 16; ++kk) {
                    u32x4 raw = ok ? *(const u32x4 *)(qrow + kk * 16 + grp * 8) : u32x4{0, 0, 0, 0};
                    qa[kk] = __builtin_bit_cast(bf16x8, raw);
                }
            }
            float lrow[16];                      // lse of the 16 query rows this lane sees
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int qi = i0 + 8 * (r >> 2) + 4 * grp + (r & 3);
                lrow[r] = qi < a.Lq ? lse[qi] : INFINITY;          // +inf => probability 0
            }
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                if (ks < ks_lo || ks >= ks_hi) continue;
                f32x16 s;
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = 0.f;
#pragma unroll
                for (int kk = 0; kk < kD / 16; ++kk)
                    s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(qa[kk], kreg[ks][kk], s, 0, 0, 0);
                const int64_t j = j0 + ks * 32 + col;
                const bool jok = j >= a.j_lo && j < a.j_hi;
                float acc = 0.f;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t qi = i0 + 8 * (r >> 2) + 4 * grp + (r & 3);
                    const int64_t dist = qi - j + a.offset;
                    bool vis = jok;
                    if (a.mask == INFLLM_MASK_WINDOW) vis = vis && dist >= 0 && dist < a.window;
                    if (a.mask == INFLLM_MASK_COMPLEMENT) vis = vis && dist >= a.window;
                    float p = __builtin_amdgcn_exp2f(s[r] * scale - lrow[r]);
                    acc += vis ? p : 0.f;
                }
                colsum[ks] += acc;
            }
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            if (ks < ks_lo || ks >= ks_hi) continue;
            const float tot = colsum[ks] + wave_xor32(colsum[ks]);
            const int64_t j = j0 + ks * 32 + col;
            if (grp == 0 && j >= a.j_lo && j < a.j_hi) {
                float *dst = a.d_score + (int64_t)b * a.score_sb + (int64_t)h * a.score_sh + (j % a.score_cap);
                *dst = a.accumulate ? *dst + tot : tot;
            }
        }
    }
}

}  // namespace

extern "C" int infllm_local_score(const infllm_score_args *a, void *stream) {
    INFLLM_REQUIRE(a != nullptr, "local_score: null argument block");
    INFLLM_REQUIRE(a->d_q && a->d_k && a->d_lse && a->d_score, "local_score: null pointer");
    INFLLM_REQUIRE(a->B > 0 && a->H > 0 && a->Hkv > 0 && a->H % a->Hkv == 0 && a->Lq > 0,
                   "local_score: bad geometry B=%d H=%d Hkv=%d Lq=%d", a->B, a->H, a->Hkv, a->Lq);
    INFLLM_REQUIRE(a->cap > 0 && a->score_cap > 0 && a->j_lo >= 0, "local_score: bad ring sizes");
    INFLLM_REQUIRE(a->j_hi - a->j_lo <= a->cap && a->j_hi - a->j_lo <= a->score_cap,
                   "local_score: key range [%lld,%lld) exceeds the ring", (long long)a->j_lo, (long long)a->j_hi);
    INFLLM_REQUIRE(a->mask >= 0 && a->mask <= 2, "local_score: unknown mask %d", a->mask);
    INFLLM_REQUIRE((a->q_sl % 8 | a->q_sh % 8 | a->q_sb % 8 | a->k_sl % 8 | a->k_sh % 8 | a->k_sb % 8) == 0,
                   "local_score: strides must be multiples of 8");
    if (a->j_hi <= a->j_lo) return 0;
    const int64_t tiles = ((a->j_hi - 1) >> 6) - (a->j_lo >> 6) + 1;
    hipLaunchKernelGGL(local_score_kernel, dim3((unsigned)tiles, a->B * a->Hkv), dim3(256), 0, (hipStream_t)stream, *a);
    INFLLM_CHECK_LAUNCH("local_score");
    return 0;
}
