// Retrieval side of the streaming path: unit scores, top-k selection and the
// representative key of a carved unit
// (inf_llm/attention/context_manager.py:159-163, 268-277, 366-383, 664-670).
// All three are memory-bound; reductions are wavefront-wide with a fixed order, so the
// outputs are deterministic.
#include "common.h"

#include <algorithm>
#include <atomic>

namespace {

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

// ---------------------------------------------------------------- unit scores (GEMV)
// Generic shape: one wave per representative row; the mean query sits in LDS as fp32.
__global__ __launch_bounds__(256) void unit_scores_kernel(const bf16_t *reps, int64_t rep_stride, int N, int C,
                                                          const float *qbar, float *scores) {
    extern __shared__ float qs[];
    for (int e = threadIdx.x; e < C; e += 256) qs[e] = qbar[e];
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int wave_global = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int n_waves = gridDim.x * 4;
    const int chunks = C / 8;
    for (int n = wave_global; n < N; n += n_waves) {
        const bf16_t *row = reps + (int64_t)n * rep_stride;
        float acc = 0.f;
        for (int c = lane; c < chunks; c += 64) {
            u32x4 w = *(const u32x4 *)(row + c * 8);
            const float *qv = qs + c * 8;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc += bf16_bits_to_f32(w[i] & 0xffffu) * qv[2 * i];
                acc += bf16_bits_to_f32(w[i] >> 16) * qv[2 * i + 1];
            }
        }
        acc = wave_sum(acc);
        if (lane == 0) scores[n] = acc;
    }
}

// Rows of CPL*512 elements: a lane owns CPL 16-byte chunks of every row and keeps its slice of the mean
// query in registers, so the row loop is nothing but CPL independent loads followed by FMAs.  The first
// row's loads are issued before the query is staged, and a wave walks its rows with a fixed stride so
// that all waves of the chip stream disjoint rows at once.
template <int CPL, int ROWS>
__global__ __launch_bounds__(256) void unit_scores_rows_kernel(const bf16_t *reps, int64_t rep_stride, int N,
                                                                const float *qbar, float *scores, int64_t qbar_ys, int64_t scores_ys) {
    extern __shared__ float qs[];
    qbar += blockIdx.y * qbar_ys;                               // blockIdx.y: one of several queries over the same rows
    scores += blockIdx.y * scores_ys;
    constexpr int C = CPL * 512;
    const int lane = threadIdx.x & 63;
    const int waves_per_wg = blockDim.x >> 6;
    const int n_waves = gridDim.x * waves_per_wg;
    int n = blockIdx.x * waves_per_wg + (threadIdx.x >> 6);     // rows n, n + n_waves, ... belong to this wave
    u32x4 w[ROWS][CPL];
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
        if (n + r * n_waves < N) {
            const bf16_t *row = reps + (int64_t)(n + r * n_waves) * rep_stride + lane * 8;
#pragma unroll
            for (int j = 0; j < CPL; ++j) w[r][j] = __builtin_nontemporal_load((const u32x4 *)(row + j * 512));
        }
    for (int e = threadIdx.x * 4; e < C; e += blockDim.x * 4) *(f32x4 *)(qs + e) = *(const f32x4 *)(qbar + e);
    __syncthreads();
    float q[CPL][8];
#pragma unroll
    for (int j = 0; j < CPL; ++j) {
        const f32x4 lo = *(const f32x4 *)(qs + j * 512 + lane * 8), hi = *(const f32x4 *)(qs + j * 512 + lane * 8 + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) q[j][i] = lo[i], q[j][4 + i] = hi[i];
    }
    while (n < N) {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int cur = n + r * n_waves;
            if (cur >= N) break;
            float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc0 += bf16_bits_to_f32(w[r][j][i] & 0xffffu) * q[j][2 * i];
                    acc1 += bf16_bits_to_f32(w[r][j][i] >> 16) * q[j][2 * i + 1];
                }
            }
            const int nxt = cur + ROWS * n_waves;
            if (nxt < N) {
                const bf16_t *row = reps + (int64_t)nxt * rep_stride + lane * 8;
#pragma unroll
                for (int j = 0; j < CPL; ++j) w[r][j] = __builtin_nontemporal_load((const u32x4 *)(row + j * 512));
            }
            const float acc = wave_sum(acc0 + acc1);
            if (lane == 0) scores[cur] = acc;
        }
        n += ROWS * n_waves;
    }
}

// At most 512 workgroups (two per CU, all resident at once: a second round of workgroups costs more than
// it gains); long tables keep two rows per wave in flight.
template <int CPL>
void launch_unit_scores_rows(const bf16_t *reps, int64_t rep_stride, int N, const float *qbar, float *scores, hipStream_t st,
                             int n_queries = 1, int64_t qbar_ys = 0, int64_t scores_ys = 0) {
    constexpr int kRowsDeep = CPL <= 8 ? 2 : 1;
    const bool deep = kRowsDeep > 1 && N >= 4096;
    const int per_wg = 4 * (deep ? kRowsDeep : 1);
    int wgs = (N + per_wg - 1) / per_wg;
    if (wgs > 512) wgs = 512;
    auto kern = deep ? unit_scores_rows_kernel<CPL, kRowsDeep> : unit_scores_rows_kernel<CPL, 1>;
    hipLaunchKernelGGL(kern, dim3(wgs, n_queries), dim3(256), (size_t)CPL * 512 * sizeof(float), st, reps, rep_stride, N, qbar, scores,
                       qbar_ys, scores_ys);
}

// ---------------------------------------------------------------- top-k (radix select)
constexpr int kSelThreads = 1024;

__device__ __forceinline__ uint32_t order_key(float f) {
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);       // larger float <=> larger key
}

// exclusive scan of one int per thread over the workgroup; returns the total in *total
__device__ int block_exclusive_scan(int v, int *wave_tot, int *total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        int n = __shfl_up(incl, o, 64);
        if (lane >= o) incl += n;
    }
    __syncthreads();                      // wave_tot free to overwrite
    if (lane == 63) wave_tot[wave] = incl;
    __syncthreads();
    int base = 0, tot = 0;
    for (int w = 0; w < kSelThreads / 64; ++w) {
        int t = wave_tot[w];
        if (w < wave) base += t;
        tot += t;
    }
    *total = tot;
    return base + incl - v;
}

// Both selection kernels can end by publishing a sequence number next to the ids (flag may be NULL): every
// thread fences its id stores to system scope, the workgroup meets, then one thread stores the number.  A host
// that polls the (pinned) flag sees the ids no later than the number.
// ids go to one place or two (the second, when given, is a host-visible copy of a device-side list)
__device__ __forceinline__ void put_id(int32_t *a, int32_t *b, int pos, int32_t v) {
    a[pos] = v;
    if (b) b[pos] = v;
}

__device__ __forceinline__ void publish(int32_t *flag, int32_t value) {
    if (!flag) return;
    __threadfence_system();
    __syncthreads();
    if (threadIdx.x == 0) __hip_atomic_store(flag, value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

// The k selected (id, key) pairs sit in LDS in ascending id; they leave in the order torch.topk returns them
// (context_manager.py:163: descending score), equal keys in ascending id.  The residency policy inserts a block's
// missed units in that order (context_manager.py:495-515), so the order decides later evictions.
__device__ __forceinline__ void emit_descending(const int32_t *sel_id, const uint32_t *sel_key, int k, int32_t *idx_out,
                                                int32_t *idx_out2) {
    const int t = threadIdx.x;
    if (t >= k) return;
    const uint32_t mine = sel_key[t];
    int rank = 0;
    for (int j = 0; j < k; ++j) {
        const uint32_t kj = sel_key[j];
        rank += (kj > mine || (kj == mine && j < t)) ? 1 : 0;
    }
    put_id(idx_out, idx_out2, rank, sel_id[t]);
}

__global__ __launch_bounds__(kSelThreads) void topk_kernel(const float *scores, int N, int k, int32_t *idx_out, int32_t *idx_out2,
                                                           int32_t *flag, int32_t flag_value, int64_t scores_xs, int64_t idx_xs) {
    scores += blockIdx.x * scores_xs;                           // blockIdx.x: one of several tables
    idx_out += blockIdx.x * idx_xs;
    if (idx_out2) idx_out2 += blockIdx.x * idx_xs;
    __shared__ int hist[256];
    __shared__ int wave_tot[kSelThreads / 64];
    __shared__ int32_t sel_id[kSelThreads];
    __shared__ uint32_t sel_key[kSelThreads];
    __shared__ uint32_t sh_prefix;
    __shared__ int sh_need;
    const int tid = threadIdx.x;

    // ---- find the k-th largest key, 8 bits per pass from the top
    uint32_t prefix = 0, pmask = 0;
    int need = k;                          // how many of the keys matching `prefix` are still wanted
    for (int shift = 24; shift >= 0; shift -= 8) {
        if (tid < 256) hist[tid] = 0;
        __syncthreads();
        for (int n = tid; n < N; n += kSelThreads) {
            uint32_t key = order_key(scores[n]);
            if ((key & pmask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1);
        }
        __syncthreads();
        {
            // digit of the need-th largest key: scan the buckets from the top (thread t <-> digit 255 - t)
            const int v = tid < 256 ? hist[255 - tid] : 0;
            int tot;
            const int excl = block_exclusive_scan(v, wave_tot, &tot);
            if (tid < 256 && excl < need && excl + v >= need) {
                sh_prefix = prefix | ((uint32_t)(255 - tid) << shift);
                sh_need = need - excl;
            }
        }
        __syncthreads();
        prefix = sh_prefix;
        need = sh_need;
        pmask |= 255u << shift;
        __syncthreads();
    }
    // prefix = key of the k-th largest; take all keys above it and the first `need` equal to it
    int out_base = 0, eq_base = 0;
    for (int n0 = 0; n0 < N; n0 += kSelThreads) {
        const int n = n0 + tid;
        uint32_t key = n < N ? order_key(scores[n]) : 0u;
        const int is_eq = (n < N && key == prefix) ? 1 : 0;
        int tot_eq, tot_sel;
        const int eq_rank = eq_base + block_exclusive_scan(is_eq, wave_tot, &tot_eq);
        const int sel = (n < N && (key > prefix || (is_eq && eq_rank < need))) ? 1 : 0;
        const int pos = out_base + block_exclusive_scan(sel, wave_tot, &tot_sel);
        if (sel && pos < k) sel_id[pos] = n, sel_key[pos] = key;
        eq_base += tot_eq;
        out_base += tot_sel;
    }
    __syncthreads();
    emit_descending(sel_id, sel_key, k, idx_out, idx_out2);
    publish(flag, flag_value);
}

// Tables of up to 16384 scores: every thread keeps its R consecutive keys in registers, so the scores are read
// once.  Three digit passes (12, 12 and 8 bits from the top; 4096 bins spread the keys of one binade over
// many LDS counters) find the key of the k-th largest; a pass whose bucket is wanted whole ends the search.
// Output contract as above: lowest indices among keys equal to the k-th; ids leave in descending score.
template <int R>
__global__ __launch_bounds__(kSelThreads) void topk_regs_kernel(const float *scores, int N, int k, int32_t *idx_out, int32_t *idx_out2,
                                                                int32_t *flag, int32_t flag_value, int64_t scores_xs, int64_t idx_xs) {
    scores += blockIdx.x * scores_xs;                           // blockIdx.x: one of several tables
    idx_out += blockIdx.x * idx_xs;
    if (idx_out2) idx_out2 += blockIdx.x * idx_xs;
    __shared__ __align__(16) int hist[4096];
    __shared__ int wave_tot[kSelThreads / 64];
    __shared__ uint32_t sh_prefix;
    __shared__ int sh_need, sh_done;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n_valid = min(max(N - tid * R, 0), R);
    uint32_t key[R];
#pragma unroll
    for (int j = 0; j < R; ++j) key[j] = j < n_valid ? order_key(scores[tid * R + j]) : 0u;

    uint32_t prefix = 0, pmask = 0;
    int need = k;
    bool done = false;
    for (int p = 0; p < 3 && !done; ++p) {
        const int shift = p == 0 ? 20 : p == 1 ? 8 : 0;
        const uint32_t dmask = p == 2 ? 255u : 4095u;
#pragma unroll
        for (int i = 0; i < 4; ++i) hist[tid + i * kSelThreads] = 0;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < R; ++j)
            if (j < n_valid && (key[j] & pmask) == prefix) atomicAdd(&hist[dmask - ((key[j] >> shift) & dmask)], 1);
        __syncthreads();
        // bins are stored from the largest digit down; thread t owns bins 4t..4t+3
        const int h0 = hist[4 * tid], h1 = hist[4 * tid + 1], h2 = hist[4 * tid + 2], h3 = hist[4 * tid + 3];
        const int s = h0 + h1 + h2 + h3;
        int incl = s;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const int up = __shfl_up(incl, o, 64);
            if (lane >= o) incl += up;
        }
        if (lane == 63) wave_tot[wave] = incl;
        __syncthreads();
        int excl = incl - s;
        for (int w = 0; w < kSelThreads / 64; ++w) excl += w < wave ? wave_tot[w] : 0;
        if (excl < need && excl + s >= need) {                 // exactly one thread holds the bucket of the k-th
            const int hv[4] = {h0, h1, h2, h3};
            int e = excl, bin = 0;
#pragma unroll
            for (int i = 0; i < 3; ++i)
                if (e + hv[bin] < need) e += hv[bin], ++bin;
            sh_prefix = prefix | ((dmask - (uint32_t)(4 * tid + bin)) << shift);
            sh_need = need - e;
            sh_done = hv[bin] == need - e;
        }
        __syncthreads();
        prefix = sh_prefix;
        need = sh_need;
        done = sh_done != 0;
        pmask |= dmask << shift;
    }
    // keys above the prefix are all taken; of those equal to it (under pmask) the first `need` by index
    int cg = 0, ce = 0;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        const uint32_t mk = key[j] & pmask;
        cg += (j < n_valid && mk > prefix) ? 1 : 0;
        ce += (j < n_valid && mk == prefix) ? 1 : 0;
    }
    const int packed = (ce << 16) | cg;                        // cg < k <= 1024 and ce <= 16384: no carry between the fields
    int incl = packed;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
    }
    __syncthreads();                                           // wave_tot of the last pass fully read
    if (lane == 63) wave_tot[wave] = incl;
    __syncthreads();
    int excl = incl - packed;
    for (int w = 0; w < kSelThreads / 64; ++w) excl += w < wave ? wave_tot[w] : 0;
    int g_before = excl & 0xffff, e_before = excl >> 16;
    // the histogram is free now: ids and keys of the selection in ascending id, then out in descending score
    int32_t *sel_id = hist;
    uint32_t *sel_key = (uint32_t *)hist + kSelThreads;
#pragma unroll
    for (int j = 0; j < R; ++j) {
        if (j >= n_valid) break;
        const uint32_t mk = key[j] & pmask;
        if (mk > prefix) {
            const int pos = g_before + min(e_before, need);
            sel_id[pos] = tid * R + j, sel_key[pos] = key[j];
            ++g_before;
        } else if (mk == prefix) {
            if (e_before < need) {
                const int pos = g_before + e_before;
                sel_id[pos] = tid * R + j, sel_key[pos] = key[j];
            }
            ++e_before;
        }
    }
    __syncthreads();
    emit_descending(sel_id, sel_key, k, idx_out, idx_out2);
    publish(flag, flag_value);
}

// The selection over ALL units from two parts: the k best of the units that existed earlier (`cand`, any order,
// chosen by the kernels above while other work was still in flight) and the n_new units carved since, whose scores
// arrive last.  A unit of the overall top-k that is not new is among the k best of the old ones, so ranking these
// n_cand + n_new <= 64 candidates by (key, lower id first) gives the same list, in the same order, as above.
__global__ __launch_bounds__(64) void topk_merge_kernel(const float *scores, const int32_t *cand, int n_cand, int first_new,
                                                        int n_new, int k, int32_t *idx_out, int32_t *flag, int32_t flag_value) {
    const int lane = threadIdx.x, n = n_cand + n_new;
    const bool valid = lane < n;
    const int id = lane < n_cand ? cand[lane] : first_new + (lane - n_cand);
    const uint32_t key = valid ? order_key(scores[id]) : 0u;
    int rank = 0;
    for (int j = 0; j < n; ++j) {
        const uint32_t kj = __shfl(key, j, 64);
        const int idj = __shfl(id, j, 64);
        rank += (kj > key || (kj == key && idj < id)) ? 1 : 0;
    }
    if (valid && rank < k) idx_out[rank] = id;              // descending score, equal scores in ascending id
    publish(flag, flag_value);
}

// The two steps above in one launch for the few units carved since the candidates were chosen: wave w of the
// one workgroup scores new units w, w + 4, ... (the arithmetic of unit_scores_rows_kernel, term by term, so a
// unit's score does not depend on which kernel computed it), then the first wave ranks candidates and new units.
template <int CPL>
__global__ __launch_bounds__(256) void score_new_rank_kernel(const bf16_t *reps, int64_t rep_stride, const float *qbar, float *scores,
                                                             const int32_t *cand, int n_cand, int first_new, int n_new, int k,
                                                             int32_t *idx_out, int32_t *flag, int32_t flag_value) {
    __shared__ float fresh[64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float q[CPL][8];
#pragma unroll
    for (int j = 0; j < CPL; ++j) {
        const f32x4 lo = *(const f32x4 *)(qbar + j * 512 + lane * 8), hi = *(const f32x4 *)(qbar + j * 512 + lane * 8 + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) q[j][i] = lo[i], q[j][4 + i] = hi[i];
    }
    for (int r = wave; r < n_new; r += 4) {
        const bf16_t *row = reps + (int64_t)(first_new + r) * rep_stride + lane * 8;
        u32x4 w[CPL];
#pragma unroll
        for (int j = 0; j < CPL; ++j) w[j] = *(const u32x4 *)(row + j * 512);
        float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc0 += bf16_bits_to_f32(w[j][i] & 0xffffu) * q[j][2 * i];
                acc1 += bf16_bits_to_f32(w[j][i] >> 16) * q[j][2 * i + 1];
            }
        }
        const float acc = wave_sum(acc0 + acc1);
        if (lane == 0) {
            scores[first_new + r] = acc;
            fresh[r] = acc;
        }
    }
    __syncthreads();
    if (wave == 0) {
        const int n = n_cand + n_new;
        const bool valid = lane < n;
        const int id = lane < n_cand ? cand[lane] : first_new + (lane - n_cand);
        const uint32_t key = !valid ? 0u : order_key(lane < n_cand ? scores[id] : fresh[lane - n_cand]);
        int rank = 0;
        for (int j = 0; j < n; ++j) {
            const uint32_t kj = __shfl(key, j, 64);
            const int idj = __shfl(id, j, 64);
            rank += (kj > key || (kj == key && idj < id)) ? 1 : 0;
        }
        if (valid && rank < k) idx_out[rank] = id;          // descending score, equal scores in ascending id
    }
    publish(flag, flag_value);
}


// ---------------------------------------------------------------- unit scores and their top-k in ONE launch
// (context_manager.py:159-163: logits = block_k @ mean query, topk(...).indices)
// The scoring is unit_scores_rows_kernel's, term by term (a unit's score does not depend on which kernel computed it).
// Every workgroup then takes a ticket; the one that draws the last ticket knows that all scores are written and
// selects.  What crosses workgroups - the scores, the ticket - moves through agent-scope atomic accesses, which are
// performed at the level of the memory hierarchy that all XCDs share, so no workgroup has to write its L2 back.
//
// The selection orders the units by the 64-bit composite (order_key(score) << 32 | ~id): all distinct, larger =
// better score, equal scores by ascending id - torch.topk's order as the residency policy sees it.  The keys are
// dealt to G >= k groups of threads; the smallest of the groups' maxima is a threshold that at least k composites
// reach, and with scores that do not depend on the unit number in a regular way only about G ln G do.  Those few are
// ranked against each other by counting.  When more than kSurvivorCap reach it (scores that fall with the unit
// number, say) the exact k-th largest composite is built bit by bit instead - slower, never wrong.
constexpr int kRetrThreads = 512;
constexpr int kSurvivorCap = 1024;
constexpr int kTicketSlots = 64;
static __device__ unsigned int retrieval_tickets[kTicketSlots];       // zero at load; the last workgroup puts its slot back to zero

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int o) {
    const uint32_t lo = __shfl_xor((uint32_t)v, o, 64), hi = __shfl_xor((uint32_t)(v >> 32), o, 64);
    return ((uint64_t)hi << 32) | lo;
}

// the selection by one workgroup of kRetrThreads threads over N <= NB * 16 * kRetrThreads scores; a thread keeps its
// keys (units tid, tid + kRetrThreads, ...) in registers
template <int NB>
__device__ __forceinline__ void select_topk_block(const float *scores, int N, int k, int32_t *idx_out, int32_t *idx_out2) {
    __shared__ uint64_t surv[kSurvivorCap + 8];
    __shared__ __align__(16) uint32_t gmax[64];
    __shared__ int wave_cnt[kRetrThreads / 64];
    __shared__ int s_count;
    constexpr int R = NB * 16;                                   // 16 loads in flight per thread and round trip
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint32_t key[R];
    uint32_t best = 0;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        float sc[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int n = tid + (b * 16 + j) * kRetrThreads;
            // an agent-scope load: it is served from where the other workgroups' agent-scope stores went
            sc[j] = n < N ? __hip_atomic_load(scores + n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int n = tid + (b * 16 + j) * kRetrThreads;
            key[b * 16 + j] = n < N ? order_key(sc[j]) : 0u;
            best = key[b * 16 + j] > best ? key[b * 16 + j] : best;
        }
    }
    auto composite = [&](int j) { return ((uint64_t)key[j] << 32) | (uint32_t)(0xffffffffu - (uint32_t)(tid + j * kRetrThreads)); };
    if (tid == 0) s_count = 0;
    if (tid < 64) gmax[tid] = 0xffffffffu;
    __syncthreads();
    // groups of 32, 16 or 8 lanes: 16, 32 or 64 groups; the threshold is on the score's key alone (units that tie with
    // it all pass, and are told apart by the composites afterwards)
    const int width = k <= 16 ? 32 : k <= 32 ? 16 : 8;
    for (int o = 1; o < width; o <<= 1) {
        const uint32_t other = __shfl_xor(best, o, 64);
        best = other > best ? other : best;
    }
    if ((lane & (width - 1)) == 0) gmax[tid / width] = best;
    __syncthreads();
    uint32_t tau = 0xffffffffu;
#pragma unroll
    for (int g = 0; g < 64; g += 4) {
        const u32x4 m = *(const u32x4 *)(gmax + g);
        tau = min(min(tau, m[0]), min(m[1], min(m[2], m[3])));
    }
    auto collect = [&](uint64_t thr) {                           // composites >= thr into surv[]; s_count = how many there are
#pragma unroll
        for (int j = 0; j < R; ++j) {
            const uint64_t c = composite(j);
            if (tid + j * kRetrThreads < N && c >= thr) {
                const int pos = atomicAdd(&s_count, 1);
                if (pos < kSurvivorCap) surv[pos] = c;
            }
        }
        __syncthreads();
    };
    collect((uint64_t)tau << 32);
    if (s_count > kSurvivorCap) {
        // exact: the largest t with at least k composites >= t, one bit at a time from the top
        uint64_t t = 0;
        for (int bit = 63; bit >= 0; --bit) {
            const uint64_t trial = t | (1ull << bit);
            int c = 0;
#pragma unroll
            for (int j = 0; j < R; ++j) c += (tid + j * kRetrThreads < N && composite(j) >= trial) ? 1 : 0;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) c += __shfl_xor(c, o, 64);
            __syncthreads();                                     // wave_cnt of the previous round fully read
            if (lane == 0) wave_cnt[wave] = c;
            __syncthreads();
            int tot = 0;
#pragma unroll
            for (int w = 0; w < kRetrThreads / 64; ++w) tot += wave_cnt[w];
            if (tot >= k) t = trial;
        }
        __syncthreads();
        if (tid == 0) s_count = 0;
        __syncthreads();
        collect(t);                                              // exactly k of them now
    }
    const int S = s_count;
    const int S8 = (S + 7) & ~7;                                 // padded with composites below every real one: the
    for (int i = S + tid; i < S8; i += kRetrThreads) surv[i] = 0;  // ranking loop then reads eight entries per round trip
    __syncthreads();
    for (int i = tid; i < S; i += kRetrThreads) {
        const uint64_t mine = surv[i];
        int rank = 0;
        for (int j = 0; j < S8; j += 8) {
            uint64_t o[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = surv[j + e];
#pragma unroll
            for (int e = 0; e < 8; ++e) rank += o[e] > mine ? 1 : 0;
        }
        if (rank < k) put_id(idx_out, idx_out2, rank, (int32_t)(0xffffffffu - (uint32_t)mine));
    }
}

template <int CPL, int ROWS>
__global__ __launch_bounds__(kRetrThreads) void retrieve_fused_kernel(const bf16_t *reps, int64_t rep_stride, int N, const float *qbar,
                                                                      float *scores, int k, int32_t *idx_out, int32_t *idx_out2,
                                                                      int32_t *flag, int32_t flag_value, int ticket_slot) {
    extern __shared__ float qs[];                                // the mean query
    __shared__ int is_last;
    constexpr int C = CPL * 512;
    const int lane = threadIdx.x & 63;
    const int waves_per_wg = kRetrThreads / 64;
    const int n_waves = gridDim.x * waves_per_wg;
    int n = blockIdx.x * waves_per_wg + (threadIdx.x >> 6);     // rows n, n + n_waves, ... belong to this wave
    u32x4 w[ROWS][CPL];
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
        if (n + r * n_waves < N) {
            const bf16_t *row = reps + (int64_t)(n + r * n_waves) * rep_stride + lane * 8;
#pragma unroll
            for (int j = 0; j < CPL; ++j) w[r][j] = __builtin_nontemporal_load((const u32x4 *)(row + j * 512));
        }
    for (int e = threadIdx.x * 4; e < C; e += kRetrThreads * 4) *(f32x4 *)(qs + e) = *(const f32x4 *)(qbar + e);
    __syncthreads();
    float q[CPL][8];
#pragma unroll
    for (int j = 0; j < CPL; ++j) {
        const f32x4 lo = *(const f32x4 *)(qs + j * 512 + lane * 8), hi = *(const f32x4 *)(qs + j * 512 + lane * 8 + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) q[j][i] = lo[i], q[j][4 + i] = hi[i];
    }
    while (n < N) {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int cur = n + r * n_waves;
            if (cur >= N) break;
            float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc0 += bf16_bits_to_f32(w[r][j][i] & 0xffffu) * q[j][2 * i];
                    acc1 += bf16_bits_to_f32(w[r][j][i] >> 16) * q[j][2 * i + 1];
                }
            }
            const int nxt = cur + ROWS * n_waves;
            if (nxt < N) {
                const bf16_t *row = reps + (int64_t)nxt * rep_stride + lane * 8;
#pragma unroll
                for (int j = 0; j < CPL; ++j) w[r][j] = __builtin_nontemporal_load((const u32x4 *)(row + j * 512));
            }
            const float acc = wave_sum(acc0 + acc1);
            if (lane == 0) __hip_atomic_store(scores + cur, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        n += ROWS * n_waves;
    }
    // every wave's score stores have been performed before the workgroup takes its ticket
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned int drawn = __hip_atomic_fetch_add(&retrieval_tickets[ticket_slot], 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        is_last = drawn == gridDim.x - 1;
    }
    __syncthreads();
    if (!is_last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    if (threadIdx.x == 0) __hip_atomic_store(&retrieval_tickets[ticket_slot], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (N <= 16 * kRetrThreads) select_topk_block<1>(scores, N, k, idx_out, idx_out2);
    else select_topk_block<2>(scores, N, k, idx_out, idx_out2);
    publish(flag, flag_value);
}

// ---------------------------------------------------------------- representative keys
constexpr int kMaxUnit = 2048;             // largest supported unit (block_size)

// The copy of the same units' K and V rows out of the rings into contiguous staging (what infllm_gather_rows does)
// can ride in the launch that picks their representatives: independent work, one launch less in the stream.
struct CarveCopy {
    const bf16_t *ring_a, *ring_b;
    bf16_t *out_a, *out_b;
    int64_t ring_cap, t0, out_sb, out_su, out_sh;
    int32_t Hkv, B, n, unit_rows, x_extra;         // n rows from t0 on; x_extra = extra workgroups along x (0: no copy)
};

// one wave per (query head, unit, batch row); workgroups with blockIdx.x >= H copy
__global__ __launch_bounds__(64) void repr_keys_kernel(const float *ring_score, const bf16_t *ring_k, int64_t ring_cap,
                                                       int H, int Hkv, int64_t t0, int bs, int repr_topk, bf16_t *rep_out,
                                                       int64_t rep_sb, int64_t rep_su, int32_t *idx_out, CarveCopy cc) {
    __shared__ float sc[kMaxUnit];
    if ((int)blockIdx.x >= H) {
        const int64_t g = ((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * cc.x_extra + ((int)blockIdx.x - H);
        const int64_t e = g * 64 + threadIdx.x;                        // (ring, batch row, kv head, row, 16-byte chunk)
        if (e >= (int64_t)2 * cc.B * cc.Hkv * cc.n * 16) return;
        const int c = (int)(e & 15);
        int64_t rest = e >> 4;
        const int r = (int)(rest % cc.n);
        rest /= cc.n;
        const int hk = (int)(rest % cc.Hkv);
        rest /= cc.Hkv;
        const int bb = (int)(rest % cc.B);
        const bool second = rest / cc.B != 0;
        const bf16_t *src = (second ? cc.ring_b : cc.ring_a) + (((int64_t)bb * cc.Hkv + hk) * cc.ring_cap + (cc.t0 + r) % cc.ring_cap) * kD + c * 8;
        bf16_t *dst = (second ? cc.out_b : cc.out_a) + (int64_t)bb * cc.out_sb + (int64_t)(r / cc.unit_rows) * cc.out_su +
                      (int64_t)hk * cc.out_sh + (int64_t)(r % cc.unit_rows) * kD + c * 8;
        *(u32x4 *)dst = *(const u32x4 *)src;
        return;
    }
    const int h = blockIdx.x, u = blockIdx.y, b = blockIdx.z, lane = threadIdx.x;
    const int n_units = gridDim.y;
    const int g = h / (H / Hkv);
    const int64_t first = t0 + (int64_t)u * bs;
    const float *srow = ring_score + ((int64_t)b * H + h) * ring_cap;
    for (int r = lane; r < bs; r += 64) sc[r] = srow[(first + r) % ring_cap];
    __syncthreads();
    const bf16_t *kbase = ring_k + ((int64_t)b * Hkv + g) * ring_cap * kD;
    float a0 = 0.f, a1 = 0.f;
    for (int it = 0; it < repr_topk; ++it) {
        float best = -INFINITY;
        int best_r = INT32_MAX;
        for (int r = lane; r < bs; r += 64) {
            float x = sc[r];
            if (x > best || (x == best && r < best_r)) {     // NaN never wins
                best = x;
                best_r = r;
            }
        }
        if (best_r == INT32_MAX && lane < bs) best_r = lane;   // all -inf / NaN: still pick a valid row
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            float ob = __shfl_xor(best, o, 64);
            int orr = __shfl_xor(best_r, o, 64);
            if (ob > best || (ob == best && orr < best_r) || best_r == INT32_MAX) {
                best = ob;
                best_r = orr;
            }
        }
        if (lane == 0) {
            sc[best_r] = -INFINITY;
            if (idx_out) idx_out[(((int64_t)b * n_units + u) * H + h) * repr_topk + it] = best_r;
        }
        uint32_t w = *(const uint32_t *)(kbase + ((first + best_r) % ring_cap) * kD + lane * 2);
        a0 += bf16_bits_to_f32(w & 0xffffu);
        a1 += bf16_bits_to_f32(w >> 16);
        __syncthreads();
    }
    const float inv = 1.f / (float)repr_topk;
    *(uint32_t *)(rep_out + (int64_t)b * rep_sb + (int64_t)u * rep_su + (int64_t)h * kD + lane * 2) =
        pack_bf16x2(a0 * inv, a1 * inv);
}

}  // namespace

extern "C" int infllm_unit_scores(const void *d_reps, int64_t rep_stride, int32_t first, int32_t count, int32_t C,
                                  const float *d_qbar, float *d_scores, void *stream) {
    INFLLM_REQUIRE(d_reps && d_qbar && d_scores, "unit_scores: null pointer");
    INFLLM_REQUIRE(first >= 0 && count >= 0 && C > 0 && C % 8 == 0 && C <= 16384, "unit_scores: bad sizes first=%d count=%d C=%d",
                   first, count, C);
    INFLLM_REQUIRE(rep_stride >= C && rep_stride % 8 == 0, "unit_scores: row stride %lld", (long long)rep_stride);
    if (count == 0) return 0;
    const bf16_t *rows = (const bf16_t *)d_reps + (int64_t)first * rep_stride;
    float *out = d_scores + first;
    switch (C % 512 == 0 ? C / 512 : 0) {
#define ROWS_CASE(n) case n: launch_unit_scores_rows<n>(rows, rep_stride, count, d_qbar, out, (hipStream_t)stream); break
        ROWS_CASE(1); ROWS_CASE(2); ROWS_CASE(4); ROWS_CASE(5); ROWS_CASE(6); ROWS_CASE(8); ROWS_CASE(10); ROWS_CASE(12); ROWS_CASE(16);
#undef ROWS_CASE
    default: {
        const int wgs = count < 4 * 2048 ? (count + 3) / 4 : 2048;
        hipLaunchKernelGGL(unit_scores_kernel, dim3(wgs), dim3(256), (size_t)C * sizeof(float), (hipStream_t)stream, rows,
                           rep_stride, count, C, d_qbar, out);
    }
    }
    INFLLM_CHECK_LAUNCH("unit_scores");
    return 0;
}

int infllm_topk_publish_pair(const float *d_scores, int32_t N, int32_t k, int32_t *d_idx, int32_t *d_idx2, int32_t *d_flag,
                             int32_t flag_value, void *stream);

extern "C" int infllm_topk(const float *d_scores, int32_t N, int32_t k, int32_t *d_idx, void *stream) {
    return infllm_topk_publish_pair(d_scores, N, k, d_idx, nullptr, nullptr, 0, stream);
}

// library-internal: the selection followed by `*d_flag = flag_value` (system scope) once the ids are written
int infllm_topk_publish(const float *d_scores, int32_t N, int32_t k, int32_t *d_idx, int32_t *d_flag, int32_t flag_value, void *stream) {
    return infllm_topk_publish_pair(d_scores, N, k, d_idx, nullptr, d_flag, flag_value, stream);
}

// the selection over `tables` tables of N scores each (scores_xs apart), table t's ids to d_idx + t * idx_xs
static int launch_topk(const float *d_scores, int32_t N, int32_t k, int32_t *d_idx, int32_t *d_idx2, int32_t *d_flag, int32_t flag_value,
                       int tables, int64_t scores_xs, int64_t idx_xs, void *stream) {
    INFLLM_REQUIRE(d_scores && d_idx, "topk: null pointer");
    INFLLM_REQUIRE(N > 0 && k > 0 && k <= N && k <= 1024 && tables >= 1, "topk: k=%d with N=%d, %d tables", k, N, tables);
    const hipStream_t st = (hipStream_t)stream;
    switch (N <= 16384 ? (N + kSelThreads - 1) / kSelThreads : 0) {       // keys per thread
#define REGS_CASE(r) hipLaunchKernelGGL(topk_regs_kernel<r>, dim3(tables), dim3(kSelThreads), 0, st, d_scores, N, k, d_idx, d_idx2, d_flag, flag_value, scores_xs, idx_xs); break
    case 1: REGS_CASE(1);
    case 2: REGS_CASE(2);
    case 3: REGS_CASE(3);
    case 4: REGS_CASE(4);
    case 5: case 6: REGS_CASE(6);
    case 7: case 8: REGS_CASE(8);
    case 9: case 10: REGS_CASE(10);
    case 11: case 12: REGS_CASE(12);
    case 13: case 14: case 15: case 16: REGS_CASE(16);
#undef REGS_CASE
    default: hipLaunchKernelGGL(topk_kernel, dim3(tables), dim3(kSelThreads), 0, st, d_scores, N, k, d_idx, d_idx2, d_flag, flag_value, scores_xs, idx_xs);
    }
    INFLLM_CHECK_LAUNCH("topk");
    return 0;
}

// ... with a second copy of the ids in d_idx2 (may be NULL)
int infllm_topk_publish_pair(const float *d_scores, int32_t N, int32_t k, int32_t *d_idx, int32_t *d_idx2, int32_t *d_flag,
                             int32_t flag_value, void *stream) {
    return launch_topk(d_scores, N, k, d_idx, d_idx2, d_flag, flag_value, 1, 0, 0, stream);
}

// internal: see topk_merge_kernel
int infllm_topk_merge_publish(const float *d_scores, const int32_t *d_cand, int32_t n_cand, int32_t first_new, int32_t n_new, int32_t k,
                              int32_t *d_idx, int32_t *d_flag, int32_t flag_value, void *stream) {
    INFLLM_REQUIRE(d_scores && d_cand && d_idx, "topk_merge: null pointer");
    INFLLM_REQUIRE(n_cand >= 0 && n_new >= 0 && n_cand + n_new <= 64 && k > 0 && k <= n_cand + n_new && first_new >= 0,
                   "topk_merge: %d + %d candidates for k=%d", n_cand, n_new, k);
    hipLaunchKernelGGL(topk_merge_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, d_scores, d_cand, n_cand, first_new, n_new, k,
                       d_idx, d_flag, flag_value);
    INFLLM_CHECK_LAUNCH("topk_merge");
    return 0;
}

// unit scores of the n_new units from first_new on, then the ranking of infllm_topk_merge_publish, in one launch.
// Returns 1 when the row length has no such kernel (the caller then launches the two steps).
int infllm_score_new_rank(const void *d_reps, int64_t rep_stride, int32_t C, const float *d_qbar, float *d_scores, const int32_t *d_cand,
                          int32_t n_cand, int32_t first_new, int32_t n_new, int32_t k, int32_t *d_idx, int32_t *d_flag,
                          int32_t flag_value, void *stream) {
    INFLLM_REQUIRE(d_reps && d_qbar && d_scores && d_cand && d_idx, "score_new_rank: null pointer");
    INFLLM_REQUIRE(n_cand >= 0 && n_new >= 0 && n_cand + n_new <= 64 && k > 0 && k <= n_cand + n_new && first_new >= 0,
                   "score_new_rank: %d + %d candidates for k=%d", n_cand, n_new, k);
    INFLLM_REQUIRE(rep_stride >= C && rep_stride % 8 == 0, "score_new_rank: row stride %lld", (long long)rep_stride);
    const bf16_t *reps = (const bf16_t *)d_reps;
    switch (C % 512 == 0 ? C / 512 : 0) {
#define RANK_CASE(n) case n: hipLaunchKernelGGL(score_new_rank_kernel<n>, dim3(1), dim3(256), 0, (hipStream_t)stream, reps, rep_stride, d_qbar, \
                                                 d_scores, d_cand, n_cand, first_new, n_new, k, d_idx, d_flag, flag_value); break
        RANK_CASE(1); RANK_CASE(2); RANK_CASE(4); RANK_CASE(8);
#undef RANK_CASE
    default: return 1;
    }
    INFLLM_CHECK_LAUNCH("score_new_rank");
    return 0;
}

extern "C" int infllm_score_new_topk(const void *d_reps, int64_t rep_stride, int32_t C, const float *d_qbar, float *d_scores,
                                     const int32_t *d_cand, int32_t n_cand, int32_t first_new, int32_t n_new, int32_t k, int32_t *d_idx,
                                     void *stream) {
    const int rc = infllm_score_new_rank(d_reps, rep_stride, C, d_qbar, d_scores, d_cand, n_cand, first_new, n_new, k, d_idx, nullptr, 0, stream);
    return rc == 1 ? infllm_fail(-1, "score_new_topk: rows of %d elements (supported: 512, 1024, 2048, 4096)", C) : rc;
}


// ---------------------------------------------------------------- a call's selections from lists made once per call
// (see CallRankJob in common.h).  Scoring is unit_scores_rows_kernel's arithmetic, term by term; the ranking orders
// base list and new units by (score, lower id first) as every selection here does, so the list that leaves is the
// one a selection over all units would give: a unit of the overall top-k that existed when the call began is among
// the k best of the units of that time.
constexpr int kCallRankEntries = 256;      // base list + units carved since the call began
constexpr int kCallRankNew = 64;           // units carved by one block

template <int CPL>
__global__ __launch_bounds__(256) void call_rank_kernel(CallRankJob jb) {
    __shared__ float fresh[kCallRankNew];
    __shared__ uint32_t e_key[kCallRankEntries];
    __shared__ int32_t e_id[kCallRankEntries];
    constexpr int C = CPL * 512;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j = jb.j0 + (int)blockIdx.x;
    const bool is_sel = j == jb.j_sel, is_cand = j == jb.j_cand;
    for (int u = 0; u < jb.B; ++u) {
        const float *qbar = jb.qbars + ((int64_t)j * jb.B + u) * C;
        float *scores = jb.scores + ((int64_t)j * jb.B + u) * jb.cols;
        // a ranking thread's entry, asked for ahead of the scoring: the base list's units and the units carved earlier
        // in the call have had their scores since then, so these loads travel beside those of the new units' rows
        const int n_late = jb.first_new + jb.n_new - jb.n_base;  // units carved since the call began
        const int n = jb.k + n_late;
        int my_id = -1;
        float my_score = 0.f;
        if ((is_sel || is_cand) && tid < n) {
            my_id = tid < jb.k ? jb.base[((int64_t)j * jb.B + u) * jb.k + tid] : jb.n_base + (tid - jb.k);
            if (my_id < jb.first_new) my_score = scores[my_id];
        }
        if (jb.n_new > 0) {
            float q[CPL][8];
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                const f32x4 lo = *(const f32x4 *)(qbar + c * 512 + lane * 8), hi = *(const f32x4 *)(qbar + c * 512 + lane * 8 + 4);
#pragma unroll
                for (int i = 0; i < 4; ++i) q[c][i] = lo[i], q[c][4 + i] = hi[i];
            }
            for (int r = wave; r < jb.n_new; r += 4) {
                const bf16_t *row = jb.reps + (int64_t)u * jb.rep_sb + (int64_t)(jb.first_new + r) * jb.rep_su + lane * 8;
                u32x4 w[CPL];
#pragma unroll
                for (int c = 0; c < CPL; ++c) w[c] = *(const u32x4 *)(row + c * 512);
                float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
                for (int c = 0; c < CPL; ++c) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        acc0 += bf16_bits_to_f32(w[c][i] & 0xffffu) * q[c][2 * i];
                        acc1 += bf16_bits_to_f32(w[c][i] >> 16) * q[c][2 * i + 1];
                    }
                }
                const float acc = wave_sum(acc0 + acc1);
                if (lane == 0) {
                    scores[jb.first_new + r] = acc;
                    fresh[r] = acc;
                }
            }
        }
        if (!is_sel && !is_cand) continue;                       // workgroup-uniform
        __syncthreads();
        if (tid < n) {
            e_id[tid] = my_id;
            e_key[tid] = order_key(my_id >= jb.first_new ? fresh[my_id - jb.first_new] : my_score);
        }
        __syncthreads();
        if (tid < n) {
            const uint32_t key = e_key[tid];
            const int id = e_id[tid];
            int rank = 0;
            for (int e = 0; e < n; ++e) {
                const uint32_t ke = e_key[e];
                const int ide = e_id[e];
                rank += (ke > key || (ke == key && ide < id)) ? 1 : 0;
            }
            if (rank < jb.k) (is_sel ? jb.sel_out : jb.cand_out)[(int64_t)u * jb.k + rank] = id;
        }
        __syncthreads();                                         // fresh / e_key / e_id are rewritten for the next row
    }
    if (is_sel) publish(jb.sel_flag, jb.sel_seq);
    else if (is_cand) publish(jb.cand_flag, jb.cand_seq);
}

// library-internal: launches call_rank_kernel for n_wgs blocks of the call from job->j0 on.  Returns 1, with nothing
// launched, where the kernel does not apply (row lengths other than 512 * {1, 2, 4, 8}, lists that do not fit).
int infllm_call_rank(const CallRankJob *job, int32_t C, int32_t n_wgs, void *stream) {
    INFLLM_REQUIRE(job && job->reps && job->qbars && job->scores && job->base, "call_rank: null pointer");
    INFLLM_REQUIRE(n_wgs >= 1 && job->B >= 1 && job->k >= 1 && job->n_new >= 0 && job->n_base >= job->k && job->first_new >= job->n_base,
                   "call_rank: bad job");
    INFLLM_REQUIRE(job->first_new + job->n_new <= job->cols, "call_rank: %d units do not fit score rows of %lld", job->first_new + job->n_new,
                   (long long)job->cols);
    INFLLM_REQUIRE(job->j_sel < 0 || job->sel_out, "call_rank: no place for the selection");
    INFLLM_REQUIRE(job->j_cand < 0 || job->cand_out, "call_rank: no place for the candidates");
    if (job->n_new > kCallRankNew || job->k + (job->first_new + job->n_new - job->n_base) > kCallRankEntries) return 1;
    switch (C % 512 == 0 ? C / 512 : 0) {
#define CALL_RANK_CASE(n) case n: hipLaunchKernelGGL(call_rank_kernel<n>, dim3(n_wgs), dim3(256), 0, (hipStream_t)stream, *job); break
        CALL_RANK_CASE(1); CALL_RANK_CASE(2); CALL_RANK_CASE(4); CALL_RANK_CASE(8);
#undef CALL_RANK_CASE
    default: return 1;
    }
    INFLLM_CHECK_LAUNCH("call_rank");
    return 0;
}
int infllm_call_rank_room() { return kCallRankEntries; }

// select_topk_block over several tables, one workgroup each (table t at scores + t * scores_xs, its ids to
// idx_out + t * idx_xs)
template <int NB>
__global__ __launch_bounds__(kRetrThreads) void select_rows_kernel(const float *scores, int N, int k, int32_t *idx_out, int64_t scores_xs,
                                                                   int64_t idx_xs) {
    select_topk_block<NB>(scores + blockIdx.x * scores_xs, N, k, idx_out + blockIdx.x * idx_xs, nullptr);
}

// Scores of the same N rows under several queries, every row read once per group of QG queries: the group's queries
// sit in LDS (QG x C floats), a wave keeps two rows in registers and walks the group's queries over them.  The sums
// are unit_scores_rows_kernel's, term by term.
constexpr int kQueryGroup = 8;
template <int CPL>
__global__ __launch_bounds__(512) void unit_scores_queries_kernel(const bf16_t *reps, int64_t rep_stride, int N, const float *qbars,
                                                                   int64_t qbar_qs, int n_queries, float *scores, int64_t scores_qs) {
    extern __shared__ float qs[];                               // [kQueryGroup][C]
    constexpr int C = CPL * 512;
    const int lane = threadIdx.x & 63;
    // Workgroups go to the 8 XCDs round-robin by their id.  The workgroups that walk the same rows for different
    // groups of queries get ids 8 apart: they run on the same XCD at about the same time, and all but the first of
    // them find the rows in that XCD's L2.
    const int groups = (n_queries + kQueryGroup - 1) / kQueryGroup;
    const int wgs = gridDim.x / groups;                         // workgroups per group of queries (a multiple of 8)
    const int slot = blockIdx.x / 8, xcd = blockIdx.x % 8;
    const int wg = (slot / groups) * 8 + xcd;
    const int n_waves = wgs * 8;
    const int q0 = (slot % groups) * kQueryGroup;
    const int nq = min(kQueryGroup, n_queries - q0);
    int n = wg * 8 + (threadIdx.x >> 6);                        // rows n, n + n_waves, ... belong to this wave
    u32x4 w[2][CPL], w_next[2][CPL];
    auto load_rows = [&](u32x4 (&dst)[2][CPL], int first) {
#pragma unroll
        for (int r = 0; r < 2; ++r)
            if (first + r * n_waves < N) {
                const bf16_t *row = reps + (int64_t)(first + r * n_waves) * rep_stride + lane * 8;
#pragma unroll
                for (int j = 0; j < CPL; ++j) dst[r][j] = *(const u32x4 *)(row + j * 512);
            }
    };
    load_rows(w, n);
    for (int e = threadIdx.x * 4; e < nq * C; e += 512 * 4)
        *(f32x4 *)(qs + e) = *(const f32x4 *)(qbars + (int64_t)(q0 + e / C) * qbar_qs + e % C);
    __syncthreads();
    while (n < N) {
        const bool two = n + n_waves < N;
        load_rows(w_next, n + 2 * n_waves);                     // the next two rows travel while these are multiplied
        // a row's elements are unpacked once and meet every query of the group; per (row, query) the two running sums
        // take their terms in unit_scores_rows_kernel's order (chunk by chunk, element by element)
        float acc[2][kQueryGroup][2];
#pragma unroll
        for (int q = 0; q < kQueryGroup; ++q) acc[0][q][0] = acc[0][q][1] = acc[1][q][0] = acc[1][q][1] = 0.f;
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
            float lo[2][4], hi[2][4];
#pragma unroll
            for (int r = 0; r < 2; ++r)
#pragma unroll
                for (int i = 0; i < 4; ++i) lo[r][i] = bf16_bits_to_f32(w[r][j][i] & 0xffffu), hi[r][i] = bf16_bits_to_f32(w[r][j][i] >> 16);
#pragma unroll
            for (int q = 0; q < kQueryGroup; ++q) {
                if (q >= nq) break;
                const float *qq = qs + q * C + j * 512 + lane * 8;
                const f32x4 q_lo = *(const f32x4 *)qq, q_hi = *(const f32x4 *)(qq + 4);
                const float qv[8] = {q_lo[0], q_lo[1], q_lo[2], q_lo[3], q_hi[0], q_hi[1], q_hi[2], q_hi[3]};
#pragma unroll
                for (int r = 0; r < 2; ++r)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        acc[r][q][0] += lo[r][i] * qv[2 * i];
                        acc[r][q][1] += hi[r][i] * qv[2 * i + 1];
                    }
            }
        }
#pragma unroll
        for (int q = 0; q < kQueryGroup; ++q) {
            if (q >= nq) break;
            const float s0 = wave_sum(acc[0][q][0] + acc[0][q][1]), s1 = wave_sum(acc[1][q][0] + acc[1][q][1]);
            if (lane == 0) {
                scores[(int64_t)(q0 + q) * scores_qs + n] = s0;
                if (two) scores[(int64_t)(q0 + q) * scores_qs + n + n_waves] = s1;
            }
        }
        n += 2 * n_waves;
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int j = 0; j < CPL; ++j) w[r][j] = w_next[r][j];
    }
}

extern "C" int infllm_score_topk_queries(const void *d_reps, int64_t rep_stride, int32_t N, int32_t C, const float *d_qbars, int64_t qbar_qs,
                              int32_t n_queries, int32_t k, float *d_scores, int64_t scores_qs, int32_t *d_idx, int64_t idx_qs, void *stream) {
    INFLLM_REQUIRE(d_reps && d_qbars && d_scores && d_idx, "score_topk_queries: null pointer");
    INFLLM_REQUIRE(N > 0 && k > 0 && k <= N && n_queries >= 1 && n_queries <= 65535, "score_topk_queries: k=%d N=%d queries=%d", k, N, n_queries);
    INFLLM_REQUIRE(rep_stride >= C && rep_stride % 8 == 0, "score_topk_queries: row stride %lld", (long long)rep_stride);
    const bf16_t *rows = (const bf16_t *)d_reps;
    const int groups = (n_queries + kQueryGroup - 1) / kQueryGroup;
    int wgs = ((N + 15) / 16 + 7) / 8 * 8;                 // two rows per wave and trip; a multiple of the 8 XCDs
    if (wgs > 256) wgs = 256;                              // one workgroup per CU: the queries take most of its LDS
    static bool lds_set = false;                           // dynamic LDS above 64 KiB must be enabled once per kernel
    if (!lds_set) {
        hipError_t e = hipFuncSetAttribute((const void *)unit_scores_queries_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                           kQueryGroup * 4096 * (int)sizeof(float));
        if (e != hipSuccess) return infllm_fail(-2, "score_topk_queries: %s", hipGetErrorString(e));
        lds_set = true;
    }
    switch (C % 512 == 0 ? C / 512 : 0) {
#define QUERIES_CASE(n) case n: hipLaunchKernelGGL(unit_scores_queries_kernel<n>, dim3(wgs * groups), dim3(512), (size_t)kQueryGroup * n * 512 * sizeof(float), \
                                                    (hipStream_t)stream, rows, rep_stride, N, d_qbars, qbar_qs, n_queries, d_scores, scores_qs); break
        QUERIES_CASE(1); QUERIES_CASE(2); QUERIES_CASE(4); QUERIES_CASE(8);
#undef QUERIES_CASE
    default: return 1;
    }
    INFLLM_CHECK_LAUNCH("score_topk_queries");
    if (N > 32 * kRetrThreads || k > 64) return launch_topk(d_scores, N, k, d_idx, nullptr, nullptr, 0, n_queries, scores_qs, idx_qs, stream);
    if (N <= 16 * kRetrThreads)
        hipLaunchKernelGGL(select_rows_kernel<1>, dim3(n_queries), dim3(kRetrThreads), 0, (hipStream_t)stream, d_scores, N, k, d_idx, scores_qs, idx_qs);
    else
        hipLaunchKernelGGL(select_rows_kernel<2>, dim3(n_queries), dim3(kRetrThreads), 0, (hipStream_t)stream, d_scores, N, k, d_idx, scores_qs, idx_qs);
    INFLLM_CHECK_LAUNCH("score_topk_queries (selection)");
    return 0;
}

// library-internal: unit scores of all N units and the k best of them in ONE launch (retrieve_fused_kernel), the ids
// leaving as infllm_topk_publish_pair leaves them.  Returns 1, with nothing launched, where that kernel does not apply
// (row lengths other than 512 * {1, 2, 4, 8}, more than 16384 units, k > 64): the caller then launches the two steps.
int infllm_retrieve_fused(const void *d_reps, int64_t rep_stride, int32_t N, int32_t C, const float *d_qbar, int32_t k, float *d_scores,
                          int32_t *d_idx, int32_t *d_idx2, int32_t *d_flag, int32_t flag_value, void *stream) {
    INFLLM_REQUIRE(d_reps && d_qbar && d_scores && d_idx, "retrieve: null pointer");
    INFLLM_REQUIRE(N > 0 && k > 0 && k <= N, "retrieve: k=%d with N=%d", k, N);
    INFLLM_REQUIRE(rep_stride >= C && rep_stride % 8 == 0, "retrieve: row stride %lld", (long long)rep_stride);
    if (N > 16384 || k > 64 || C % 512 != 0) return 1;
    const int cpl = C / 512;
    if (cpl != 1 && cpl != 2 && cpl != 4 && cpl != 8) return 1;
    static std::atomic<unsigned int> next_slot{0};
    const int slot = (int)(next_slot.fetch_add(1, std::memory_order_relaxed) % kTicketSlots);
    constexpr int waves_per_wg = kRetrThreads / 64;
    const bool deep = N >= 4096;
    const int per_wg = waves_per_wg * (deep ? 2 : 1);
    int wgs = (N + per_wg - 1) / per_wg;
    if (wgs > 256) wgs = 256;
    const size_t lds = (size_t)C * sizeof(float);
    const bf16_t *reps = (const bf16_t *)d_reps;
    const hipStream_t st = (hipStream_t)stream;
#define FUSED_CASE(c)                                                                                                              \
    case c: {                                                                                                                      \
        auto kern = deep ? retrieve_fused_kernel<c, 2> : retrieve_fused_kernel<c, 1>;                                              \
        hipLaunchKernelGGL(kern, dim3(wgs), dim3(kRetrThreads), lds, st, reps, rep_stride, N, d_qbar, d_scores, k, d_idx, d_idx2,   \
                           d_flag, flag_value, slot);                                                                              \
        break;                                                                                                                     \
    }
    switch (cpl) {
        FUSED_CASE(1) FUSED_CASE(2) FUSED_CASE(4) FUSED_CASE(8)
    }
#undef FUSED_CASE
    INFLLM_CHECK_LAUNCH("retrieve");
    return 0;
}

extern "C" int infllm_score_topk(const void *d_reps, int64_t rep_stride, int32_t N, int32_t C, const float *d_qbar,
                                 int32_t k, float *d_scores, int32_t *d_idx, void *stream) {
    INFLLM_REQUIRE(N > 0 && k >= 0 && k <= N, "score_topk: k=%d with N=%d", k, N);
    if (k > 0) {
        INFLLM_REQUIRE(d_idx, "score_topk: null index pointer");
        const int frc = infllm_retrieve_fused(d_reps, rep_stride, N, C, d_qbar, k, d_scores, d_idx, nullptr, nullptr, 0, stream);
        if (frc != 1) return frc;
    }
    int rc = infllm_unit_scores(d_reps, rep_stride, 0, N, C, d_qbar, d_scores, stream);
    if (rc == 0 && k > 0) rc = infllm_topk(d_scores, N, k, d_idx, stream);
    return rc;
}

// internal: infllm_repr_keys, and in the same launch the K (ring_v: V) rows of those units out of the rings into
// d_out_k / d_out_v as infllm_gather_rows lays them out (unit_rows = bs); d_ring_v == NULL: no copy
int infllm_repr_keys_carve(const float *d_ring_score, const void *d_ring_k_raw, int64_t ring_cap, int32_t B, int32_t H, int32_t Hkv,
                           int64_t t0, int32_t bs, int32_t n_units, int32_t repr_topk, void *d_rep_out, int64_t rep_sb, int64_t rep_su,
                           int32_t *d_idx_out, const void *d_ring_v, void *d_out_k, void *d_out_v, int64_t out_sb, int64_t out_su,
                           int64_t out_sh, void *stream) {
    INFLLM_REQUIRE(d_ring_score && d_ring_k_raw && d_rep_out, "repr_keys: null pointer");
    INFLLM_REQUIRE(B > 0 && H > 0 && Hkv > 0 && H % Hkv == 0, "repr_keys: bad geometry B=%d H=%d Hkv=%d", B, H, Hkv);
    INFLLM_REQUIRE(bs > 0 && bs <= kMaxUnit, "repr_keys: unit size %d not in 1..%d", bs, kMaxUnit);
    INFLLM_REQUIRE(repr_topk > 0 && repr_topk <= bs, "repr_keys: repr_topk %d not in 1..%d", repr_topk, bs);
    INFLLM_REQUIRE(n_units >= 0 && t0 >= 0 && (int64_t)n_units * bs <= ring_cap, "repr_keys: %d units do not fit the ring",
                   n_units);
    INFLLM_REQUIRE(rep_sb % 2 == 0 && rep_su % 2 == 0, "repr_keys: output strides must be even");
    if (n_units == 0) return 0;
    CarveCopy cc{};
    if (d_ring_v) {
        INFLLM_REQUIRE(d_out_k && d_out_v && (out_sb % 8 | out_su % 8 | out_sh % 8) == 0, "repr_keys: bad copy destination");
        cc.ring_a = (const bf16_t *)d_ring_k_raw; cc.ring_b = (const bf16_t *)d_ring_v;
        cc.out_a = (bf16_t *)d_out_k; cc.out_b = (bf16_t *)d_out_v;
        cc.ring_cap = ring_cap; cc.t0 = t0; cc.out_sb = out_sb; cc.out_su = out_su; cc.out_sh = out_sh;
        cc.Hkv = Hkv; cc.B = B; cc.n = n_units * bs; cc.unit_rows = bs;
        const int64_t waves = ((int64_t)2 * B * Hkv * cc.n * 16 + 63) / 64, per_x = (int64_t)n_units * B;
        cc.x_extra = (int32_t)((waves + per_x - 1) / per_x);
    }
    hipLaunchKernelGGL(repr_keys_kernel, dim3(H + cc.x_extra, n_units, B), dim3(64), 0, (hipStream_t)stream, d_ring_score,
                       (const bf16_t *)d_ring_k_raw, ring_cap, H, Hkv, t0, bs, repr_topk, (bf16_t *)d_rep_out, rep_sb,
                       rep_su, d_idx_out, cc);
    INFLLM_CHECK_LAUNCH("repr_keys");
    return 0;
}

extern "C" int infllm_repr_keys(const float *d_ring_score, const void *d_ring_k_raw, int64_t ring_cap, int32_t B, int32_t H,
                                int32_t Hkv, int64_t t0, int32_t bs, int32_t n_units, int32_t repr_topk, void *d_rep_out,
                                int64_t rep_sb, int64_t rep_su, int32_t *d_idx_out, void *stream) {
    return infllm_repr_keys_carve(d_ring_score, d_ring_k_raw, ring_cap, B, H, Hkv, t0, bs, n_units, repr_topk, d_rep_out, rep_sb, rep_su,
                                  d_idx_out, nullptr, nullptr, nullptr, 0, 0, 0, stream);
}
