// Multi-stage attention for gfx950: one flash-style MFMA kernel per stage, and the
// merge that realises the joint softmax across stages
// (inf_llm/attention/dot_production_attention/torch_impl.py:15-96).
//
// Work split.  For one kv head the query heads that share it (GQA) are laid out as
// "wave tasks" (query tile of 32 rows, head-in-group); a workgroup of 8 waves takes 8
// consecutive tasks ordered tile-major/head-minor, so with 4 query heads per kv head
// the 8 waves hold two tiles of 32 queries of the 4 heads and walk the same keys.
// K and V tiles of 64 keys are staged through LDS once per workgroup.
//
// MFMA formulation (v_mfma_f32_32x32x16_bf16), all operands read as 16-byte vectors:
//   S^T[key, query] = K[key, :] . Q[query, :]       A = K rows (LDS), B = Q (registers)
//   O^T[d, query]  += V^T[d, key] . P^T[key, query]  A = V^T rows (LDS), B = P (registers)
// A lane owns ONE query column, so the running max / sum / rescale are per-lane scalars
// and P never leaves registers.  MFMA row r of a 32-key sub-tile is bound to key
// pi(r) = 16*(r>>4) + 8*((r>>2)&1) + 4*((r>>3)&1) + (r&3); with that binding the 16
// accumulator registers of a lane are two runs of 8 consecutive keys, which is exactly
// the k-slice the second MFMA wants from the lane.  V is transposed on its way into LDS.
#include <cstdlib>

#include "common.h"

#include <atomic>
#include <cstddef>
#include <cstring>
#include <type_traits>

namespace {

constexpr int kWaves = 8;                  // 2 per SIMD inside ONE workgroup: a K/V tile in LDS feeds 256 query rows
constexpr int kStages = 4;                 // K/V tiles resident in LDS: the pair being multiplied and the pair in flight
constexpr int kThreads = kWaves * kWave;
constexpr int kQTile = 32;                 // queries per wave
constexpr int kBig = 1 << 29;              // clamp for mask distances held in int32

struct StageRange {
    int64_t lo, hi;   // key index range [lo, hi) visible to a span of queries
};

// keys visible to queries [i0, i1] under the stage mask, clipped to the source range
__device__ __forceinline__ StageRange visible_range(const infllm_attn_args &a, int64_t i0, int64_t i1) {
    StageRange r{a.j_lo, a.j_hi};
    if (a.mask == INFLLM_MASK_WINDOW) {
        r.lo = max(r.lo, i0 + a.offset - a.window + 1);
        r.hi = min(r.hi, i1 + a.offset + 1);
    } else if (a.mask == INFLLM_MASK_COMPLEMENT) {
        r.hi = min(r.hi, i1 + a.offset - a.window + 1);
    }
    return r;
}

__device__ __forceinline__ int floordiv64(int64_t x) { return (int)(x >> 6); }   // arithmetic shift = floor

// Division by a launch constant without the divide: q = (n * mul) >> shift is exact for every n < 2^31 when
// mul = floor(2^shift / d) + 1 and shift = 31 + ceil(log2 d) (the excess mul*d - 2^shift is at most d <= 2^ceil(log2 d),
// so the error term n * excess / (d * 2^shift) stays below 1/d).  The kernel's set-up is a chain of such divisions on
// the critical path of a workgroup that lives for only a handful of tiles; a hardware-less 64-bit divide costs
// some two hundred instructions.
struct FastDiv {
    uint32_t d, mul, shift;
};
inline FastDiv fast_div(uint32_t d) {
    uint32_t l = 0;
    while ((1ull << l) < d) ++l;
    return FastDiv{d, (uint32_t)((1ull << (31 + l)) / d + 1), 31 + l};
}
__device__ __forceinline__ uint32_t fdiv(uint32_t n, const FastDiv &f) { return (uint32_t)(((uint64_t)n * f.mul) >> f.shift); }

// launch constants the kernel would otherwise derive with divisions
struct StageGeom {
    FastDiv gx, gy, hkv, group, nsplit, cap_tiles;
    int32_t n_tasks;
    // Partial rows by execution block (out_exc > 0): the queries are those of several consecutive execution blocks of
    // out_exc rows (the last one may be shorter), and block k's partials form a [nsplit, B, H, n_k, 128] array of their
    // own at row k * out_block_rows of the partial buffers - where the merge of that block expects them.
    int32_t out_exc;
    int64_t out_block_rows;
    FastDiv out_exc_div;
};

// LDS layouts.  Tiles go from global memory straight into LDS (global_load_lds_dwordx4: lane l of a
// wave deposits its 16 bytes at base + 16*l, so one instruction fills 4 rows of 256 bytes), which leaves
// no staging registers; which 16-byte chunk of which row a lane FETCHES is free, and that is where the
// layout is decided:
//   Ks[buf][R][16 chunks]  LDS row R holds key k_lds_row(R) (bits 2 and 3 swapped inside each 32-key
//                          half, so the lane that owns MFMA row r reads LDS row r); chunk c of the row
//                          sits at position c ^ swz(R).  The LDS serves 256 bytes per cycle from 64 banks: a
//                          16-byte read is conflict free when the 16 lanes of a quarter wave hit 16 different
//                          chunk positions, an 8-byte transposing read when the 32 lanes of a half wave hit 32
//                          different 8-byte slots; swz() is a permutation of the 4 low row bits that gives both
//                          (K: 16 consecutive rows, one chunk each; V: 4 rows x 4 chunks x 2 halves).
//   Vs[buf][R][16 chunks]  natural rows, same swizzle; the V^T operand of the second MFMA is formed by
//                          the transposing read ds_read_b64_tr_b16: in a group of 16 lanes, lane 4*j + q
//                          supplies the address of 4 consecutive d of key j, and lane i receives element
//                          i of keys j = 0..3, i.e. 4 consecutive keys at one d.
__device__ __forceinline__ int k_lds_row(int key) { return (key & ~12) | ((key & 4) << 1) | ((key & 8) >> 1); }
__device__ __forceinline__ int swz(int row) { return ((row & 3) << 2) | ((row >> 2) & 3); }

typedef short s16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ s16x4 lds_read_tr(const bf16_t *p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)p);
}
// Issued as inline assembly on purpose.  With the builtin, the compiler tracks the transfer as an LDS store that
// may alias every later LDS read and puts `s_waitcnt vmcnt(0)` in front of the first operand read of the tile being
// multiplied - which waits for the tiles just requested for LATER and serialises load and math completely.  The
// kernel orders the transfers itself: vmcnt(0) and a barrier before a buffer is read, a barrier before it is refilled.
__device__ __forceinline__ void load_to_lds16(const bf16_t *g, bf16_t *lds_wave_base) {
    const uint32_t lds = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) void *)lds_wave_base);
    uint32_t saved_m0;                    // M0 is the compiler's to manage: put back what it held
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "s"(lds), "v"(g)
                 : "memory");
}

constexpr int kTileBytes = kTile * kD * 2;        // one K (or V) tile in LDS
constexpr float kLazyLog2 = 8.f;                  // the running max may lag the true max by 2^8

template <int N>
struct IntC {
    static constexpr int value = N;
};

// MODE: what the launch walks.  kLinear: the linear source of `a`; kPaged: the page table of `a`; kBoth: the linear
// source of `a`, then the page table of `a2` with `a2`'s queries - both stages of the operator in one launch, as ONE
// list of tiles that the key splits divide between them (one set of partials, one fixed cost instead of two).
enum { kLinear = 0, kPaged = 1, kBoth = 2 };

// The page table can ride in the launch itself (INLINE): the host passes up to kInlinePages entries by value, and the
// kernel reads them where they lie in its argument segment - scalar loads through the constant address space, like the
// table in device memory, but no kernel has to run beforehand to put it there.  The parameter is never touched as a
// C++ object (that would copy it to scratch memory for the dynamic index).
constexpr int kInlinePages = 64;
struct InlinePages {
    infllm_page p[kInlinePages];
};
struct NoInlinePages {};
struct KernargLayout {                     // the arguments as the launch lays them out: in order, naturally aligned
    infllm_attn_args a, a2;
    StageGeom geo;
    InlinePages pages;
};

template <int MODE, bool INLINE = false>
__global__ __launch_bounds__(kThreads, 2) void attn_stage_kernel(infllm_attn_args a, infllm_attn_args a2, StageGeom geo,
                                                                 std::conditional_t<INLINE, InlinePages, NoInlinePages>) {
    constexpr bool HAS_LIN = MODE != kPaged, HAS_PAG = MODE != kLinear;
    const infllm_attn_args &ap = MODE == kBoth ? a2 : a;                 // the paged stage's arguments
    extern __shared__ __attribute__((aligned(16))) char lds_dyn[];      // kStages K tiles, then kStages V tiles
    char *const Ks = lds_dyn, *const Vs = lds_dyn + kStages * kTileBytes;
    __shared__ int wg_lo[kWaves], wg_hi[kWaves];

    // the wave index is the same in every lane: said so, what derives from it (the wave's queries, tile range, mask
    // distances) stays in scalar registers
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int col = lane & 31, grp = lane >> 5;
    const int G = (int)geo.group.d;
    // Workgroups go to the 8 XCDs round-robin by linear id, and each XCD has its own L2.  Renumber so that
    // one XCD runs a contiguous run of ids: the workgroups that share a (kv head, split) K/V range then sit
    // behind one L2 and that range leaves HBM once instead of once per XCD.
    int bx = blockIdx.x, by = blockIdx.y, bz = blockIdx.z;
    {
        const int gx = gridDim.x, gy = gridDim.y, total = gx * gy * (int)gridDim.z;
        if ((total & 7) == 0) {
            const int lin = bx + gx * (by + gy * bz);
            const int id = (lin & 7) * (total >> 3) + (lin >> 3);
            const int rest = (int)fdiv(id, geo.gx);     // id = bx + gx * (by + gy * bz)
            bx = id - rest * gx;
            bz = (int)fdiv(rest, geo.gy);
            by = rest - bz * gy;
        }
    }
    const int b = (int)fdiv(by, geo.hkv), g = by - b * a.Hkv;
    const int split = bz;
    const int n_tasks = geo.n_tasks;

    // ---- this wave's task and the tiles it needs
    const int task = bx * kWaves + wave;
    const bool live = task < n_tasks;
    const int qt = live ? (int)fdiv(task, geo.group) : 0, hg = live ? task - qt * G : 0;
    const int h = g * G + hg;
    const int i0 = qt * kQTile, i1 = min(i0 + kQTile, a.Lq) - 1;

    int w_t0 = 0, w_t1 = 0;              // this wave's range of LINEAR tiles (absolute tile numbers)
    if (HAS_LIN && live) {
        StageRange r = visible_range(a, i0, i1);
        if (r.hi > r.lo) {
            w_t0 = floordiv64(r.lo);
            w_t1 = floordiv64(r.hi - 1) + 1;
        }
    }
    // ---- workgroup range of linear tiles = union over its waves
    if (lane == 0) {
        wg_lo[wave] = w_t1 > w_t0 ? w_t0 : INT32_MAX;
        wg_hi[wave] = w_t1 > w_t0 ? w_t1 : INT32_MIN;
    }
    __syncthreads();
    int lin_t0 = INT32_MAX, lin_t1 = INT32_MIN;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
        lin_t0 = min(lin_t0, wg_lo[w]);
        lin_t1 = max(lin_t1, wg_hi[w]);
    }
    if (lin_t1 <= lin_t0) lin_t0 = lin_t1 = 0;
    // The unified tile list: u in [0, n_lin) is linear tile lin_t0 + u, u in [n_lin, n_lin + n_pag) is page u - n_lin.
    const int n_lin = lin_t1 - lin_t0, n_pag = HAS_PAG ? ap.n_pages : 0;
    int g_t0, g_t1;                      // this split's share of the list
    {
        // n / nsplit tiles each; the n % nsplit left over go one each to a run of splits in the middle: the first and
        // the last split hold the tiles that need the mask (window start, causal diagonal) and take 1-2 us longer over
        // the same number of tiles, so with the extras at the ends the whole launch waited for them
        const uint32_t n = (uint32_t)(n_lin + n_pag), per = fdiv(n, geo.nsplit), rem = n - per * a.nsplit;
        const int first_extra = (int)((a.nsplit - rem) >> 1);
        const int before = min(max(split - first_extra, 0), (int)rem);            // extras given to lower splits
        const int mine = (split >= first_extra && split < first_extra + (int)rem) ? 1 : 0;
        g_t0 = (int)per * split + before;
        g_t1 = g_t0 + (int)per + mine;
    }
    const int wu0 = w_t0 - lin_t0, wu1 = w_t1 - lin_t0;     // this wave's linear tiles in list indices

    bf16x8 qreg[kD / 16];                     // Q as the B operand: lane = (query col, k-group); loaded behind the first tiles

    // ---- per-lane LDS byte offsets of the MFMA operands (inside one tile buffer)
    uint32_t k_off[kD / 16];                  // K operand kk of sub-tile 0 (sub-tile 1: + 32 rows)
#pragma unroll
    for (int kk = 0; kk < kD / 16; ++kk) k_off[kk] = col * 256 + (((kk * 2 + grp) ^ swz(col)) * 16);
    uint32_t v_off[kD / 32][2];               // V^T operand of d-tile dt, key half e, of 16-key step 0 (step gi: + 16*gi rows)
    {
        const int lam = lane & 15, g16 = lane >> 4;
        const int vr = 8 * (g16 >> 1) + (lam >> 2);              // lane 4*j + q addresses key j ...
        const int vc = 2 * (g16 & 1) + ((lam & 3) >> 1);         // ... at 4 consecutive d: 16-byte chunk
        const int vh = 8 * (lam & 1);                            //     and byte offset inside it
#pragma unroll
        for (int dt = 0; dt < kD / 32; ++dt)
#pragma unroll
            for (int e = 0; e < 2; ++e) v_off[dt][e] = (vr + 4 * e) * 256 + (((dt * 4 + vc) ^ swz(vr + 4 * e)) * 16) + vh;
    }

    // ---- tile loads: wave w, instruction i fills LDS rows 8*w + 4*i .. +3; lane -> (row, position).
    //      The wave-uniform tile base advances with the loop; the per-lane offsets are loop invariant.
    constexpr int kLd = kTile / (4 * kWaves);  // load instructions per wave and tile, for K and for V
    uint32_t gk_off[kLd], gv_off[kLd];        // element offsets inside a linear tile
    uint32_t pk_off[kLd], pv_off[kLd];        // ... inside a page (rows of kD elements)
    int gk_row[kLd], gv_row[kLd];
    {
        const int ld_pos = lane & 15, ld_sub = lane >> 4;
#pragma unroll
        for (int i = 0; i < kLd; ++i) {
            const int R = 4 * kLd * wave + 4 * i + ld_sub, chunk = ld_pos ^ swz(R);
            gk_row[i] = k_lds_row(R);
            gv_row[i] = R;
            if (HAS_LIN) {
                gk_off[i] = (uint32_t)(gk_row[i] * a.k_sl + chunk * 8);
                gv_off[i] = (uint32_t)(R * a.v_sl + chunk * 8);
            }
            if (HAS_PAG) {
                pk_off[i] = (uint32_t)(gk_row[i] * kD + chunk * 8);
                pv_off[i] = (uint32_t)(R * kD + chunk * 8);
            }
        }
    }
    const bf16_t *k_head = nullptr, *v_head = nullptr;          // linear source: row 0 of this kv head
    int64_t ring_row = 0;                                        // ring row of the linear tile to load next
    if (HAS_LIN) {
        k_head = (const bf16_t *)a.d_k + (int64_t)b * a.k_sb + (int64_t)g * a.k_sh;
        v_head = (const bf16_t *)a.d_v + (int64_t)b * a.v_sb + (int64_t)g * a.v_sh;
        const int first = lin_t0 + min(g_t0, n_lin);
        ring_row = (int64_t)(first - (int)(fdiv(first, geo.cap_tiles) * geo.cap_tiles.d)) * kTile;
    }
    // The page table is read through the constant address space: the index is wave-uniform, so these become scalar
    // loads.  As vector loads they would share the vmcnt counter with the tile transfers, and waiting for a page
    // entry would wait for every tile in flight.  The table is written by an earlier kernel and is read-only here.
    const __attribute__((address_space(4))) infllm_page *page_table;
    if constexpr (INLINE)
        page_table = (const __attribute__((address_space(4))) infllm_page *)((const __attribute__((address_space(4))) char *)
                                                                             __builtin_amdgcn_kernarg_segment_ptr() +
                                                                             offsetof(KernargLayout, pages)) + (int64_t)b * n_pag;
    else
        page_table = (const __attribute__((address_space(4))) infllm_page *)(uintptr_t)ap.d_pages + (int64_t)b * n_pag;
    auto load_tile = [&](int u, int buf) {     // list index; linear tiles are requested in ascending order
        const bf16_t *kbase, *vbase;
        int row_lo, row_hi;                   // valid rows of this tile: [row_lo, row_hi)
        const bool paged = MODE == kPaged || (MODE == kBoth && u >= n_lin);
        if (paged) {
            const __attribute__((address_space(4))) infllm_page *entry = page_table + (u - n_lin);
            const int64_t hs = entry->head_stride;
            kbase = (const bf16_t *)entry->k + (int64_t)g * hs;
            vbase = (const bf16_t *)entry->v + (int64_t)g * hs;
            row_lo = 0;
            row_hi = entry->n_valid;
        } else {
            const int64_t j0 = (int64_t)(lin_t0 + u) * kTile;
            kbase = k_head + ring_row * a.k_sl;       // cap is a multiple of the tile, so a tile never wraps
            vbase = v_head + ring_row * a.v_sl;
            ring_row += kTile;
            if (ring_row >= a.cap) ring_row -= a.cap;
            row_lo = (int)max((int64_t)0, a.j_lo - j0);
            row_hi = (int)min((int64_t)kTile, a.j_hi - j0);
        }
        char *kdst = Ks + buf * kTileBytes + wave * (kLd * 1024), *vdst = Vs + buf * kTileBytes + wave * (kLd * 1024);
        if (row_lo == 0 && row_hi == kTile) {          // the common case: no per-lane predicate
#pragma unroll
            for (int i = 0; i < kLd; ++i) {
                load_to_lds16(kbase + (paged ? pk_off[i] : gk_off[i]), (bf16_t *)(kdst + i * 1024));
                load_to_lds16(vbase + (paged ? pv_off[i] : gv_off[i]), (bf16_t *)(vdst + i * 1024));
            }
        } else {
#pragma unroll
            for (int i = 0; i < kLd; ++i) {
                // rows outside the source are written as zeros: their keys are masked, but 0 * stale must stay 0
                if (gk_row[i] >= row_lo && gk_row[i] < row_hi) load_to_lds16(kbase + (paged ? pk_off[i] : gk_off[i]), (bf16_t *)(kdst + i * 1024));
                else *(u32x4 *)(kdst + i * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
                if (gv_row[i] >= row_lo && gv_row[i] < row_hi) load_to_lds16(vbase + (paged ? pv_off[i] : gv_off[i]), (bf16_t *)(vdst + i * 1024));
                else *(u32x4 *)(vdst + i * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
            }
        }
    };

    // ---- running softmax state of this lane's query (max kept in raw logit units, allowed to lag)
    float m_run = -INFINITY, l_run = 0.f, neg_ms = 0.f;
    f32x16 oacc[kD / 32];
#pragma unroll
    for (int dt = 0; dt < kD / 32; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[dt][r] = 0.f;

    const float scale = a.softmax_scale * 1.4426950408889634f;
    const float lazy = kLazyLog2 / scale;

    auto tile_math = [&](int buf, int t) {
        const char *kb = Ks + buf * kTileBytes, *vb = Vs + buf * kTileBytes;
        f32x16 s[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int r = 0; r < 16; ++r) s[ks][r] = 0.f;
        {
            // 16 K operands in groups of 4 (kk pair x both sub-tiles): a group is requested from LDS while the
            // MFMAs of the previous one run; scheduling fences keep the compiler from serialising read -> MFMA
            bf16x8 ka[4][4];
            auto k_operand = [&](int i) {          // i = kk * 2 + ks
                return *(const bf16x8 *)(kb + (i & 1) * 32 * 256 + k_off[i >> 1]);
            };
#pragma unroll
            for (int j = 0; j < 4; ++j) ka[0][j] = k_operand(j);
#pragma unroll
            for (int gi = 0; gi < 4; ++gi) {
                __builtin_amdgcn_sched_barrier(0);
                if (gi < 3) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) ka[gi + 1][j] = k_operand((gi + 1) * 4 + j);
                    __builtin_amdgcn_sched_barrier(0);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int i = gi * 4 + j;
                    s[i & 1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[gi][j], qreg[i >> 1], s[i & 1], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- mask (only tiles that touch a boundary); distances are clamped into int32
        bool need_mask;
        int row_lo = 0, row_hi = kTile;
        int d0 = 0;                            // dist of (this lane's query, key 0 of the tile)
        const bool paged = MODE == kPaged || (MODE == kBoth && t >= n_lin);
        if (paged) {
            row_hi = page_table[t - n_lin].n_valid;
            need_mask = row_hi < kTile;
        } else {
            const int64_t j0 = (int64_t)(lin_t0 + t) * kTile;
            row_lo = (int)max((int64_t)0, a.j_lo - j0);
            row_hi = (int)min((int64_t)kTile, a.j_hi - j0);
            need_mask = row_lo > 0 || row_hi < kTile;
            const int64_t e0 = (int64_t)i0 + a.offset - j0;       // dist(query i0, key j0)
            if (a.mask == INFLLM_MASK_WINDOW) {
                need_mask |= (e0 < kTile - 1) || (e0 + (i1 - i0) >= a.window);
            } else if (a.mask == INFLLM_MASK_COMPLEMENT) {
                need_mask |= (e0 - (kTile - 1) < a.window);
            }
            d0 = (int)min(max(e0, (int64_t)-kBig), (int64_t)kBig) + col;
        }
        if (need_mask) {
            const int win = (int)min(a.window, (int64_t)2 * kBig);
            const int lo_l = row_lo - 8 * grp, hi_l = row_hi - 8 * grp;      // bounds on kc for this lane
            const int dl = d0 - 8 * grp;                                       // dist = dl - kc
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    // key of register r: ko = kc + 8*grp with the compile-time part kc; everything is
                    // expressed relative to the per-lane bases so that no per-register value is kept
                    const int kc = ks * 32 + 16 * (r >> 3) + (r & 7);
                    bool vis = (kc >= lo_l) && (kc < hi_l);
                    if (!paged) {
                        if (a.mask == INFLLM_MASK_WINDOW) vis = vis && (kc <= dl) && (kc > dl - win);
                        if (a.mask == INFLLM_MASK_COMPLEMENT) vis = vis && (kc <= dl - win);
                    }
                    s[ks][r] = vis ? s[ks][r] : -INFINITY;
                }
        }
        float tmax = -INFINITY;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, s[ks][r]);
        tmax = fmaxf(tmax, wave_xor32(tmax));
        // lazy running max: it only moves when a score would exceed it by more than 2^kLazyLog2 after scaling,
        // so the rescale of the output accumulators is rare; probabilities stay below 2^kLazyLog2
        const bool moved = tmax > m_run + lazy;
        if (__builtin_amdgcn_ballot_w64(moved) != 0) {
            const float m_new = moved ? tmax : m_run;
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * scale);      // exp2(-inf) = 0 on the first move
            const float al = moved ? alpha : 1.f;
            l_run *= al;
#pragma unroll
            for (int dt = 0; dt < kD / 32; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) oacc[dt][r] *= al;
            m_run = m_new;
            neg_ms = (m_run == -INFINITY) ? 0.f : -m_run * scale;
        }
        // The row sum is taken over the probabilities AS ROUNDED to bf16, the values the second MFMA multiplies: the
        // output is then an exact convex combination of value rows (a row on which one key carries nearly all the
        // weight comes out as that value row, whatever the rounding of its weight), and a pair costs one dot
        // instruction instead of two additions.
        float psum[2] = {0.f, 0.f};
        uint32_t pw[2][8];
        auto exps = [&](int ks, int r0, int r1) {
#pragma unroll
            for (int r = r0; r < r1; r += 2) {
                float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[ks][r], scale, neg_ms));
                float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[ks][r + 1], scale, neg_ms));
                pw[ks][r >> 1] = pack_bf16x2(p0, p1);
                psum[ks] = sum_bf16x2(pw[ks][r >> 1], psum[ks]);
            }
        };
        exps(0, 0, 16);                        // the first 32 keys now; the other 32 beside the MFMAs that consume these
        {
            // 4 steps of 16 keys, 4 MFMAs each; the V^T operands of a step are requested from LDS while the
            // MFMAs of the previous step run
            typedef short s16x8 __attribute__((ext_vector_type(8)));
            s16x8 va[2][kD / 32];
            auto v_operands = [&](int gi, s16x8 *dst) {
#pragma unroll
                for (int dt = 0; dt < kD / 32; ++dt) {
                    dst[dt].lo = lds_read_tr((const bf16_t *)(vb + gi * 16 * 256 + v_off[dt][0]));
                    dst[dt].hi = lds_read_tr((const bf16_t *)(vb + gi * 16 * 256 + v_off[dt][1]));
                }
            };
            v_operands(0, va[0]);
#pragma unroll
            for (int gi = 0; gi < 4; ++gi) {
                __builtin_amdgcn_sched_barrier(0);
                if (gi < 3) {
                    v_operands(gi + 1, va[(gi + 1) & 1]);
                    __builtin_amdgcn_sched_barrier(0);
                }
                const int ks = gi >> 1, mm = gi & 1;
                u32x4 praw{pw[ks][4 * mm], pw[ks][4 * mm + 1], pw[ks][4 * mm + 2], pw[ks][4 * mm + 3]};
                bf16x8 pb = __builtin_bit_cast(bf16x8, praw);
                // A wave's own vector-ALU work hides under its MFMAs when the two are interleaved instruction by
                // instruction (an MFMA holds the matrix pipe for 32 cycles and the issue port for a few): the
                // exponentials of the tile's second half go between the MFMAs of its first half.
                if (gi < 2) exps(1, 8 * gi, 8 * gi + 8);
#pragma unroll
                for (int dt = 0; dt < kD / 32; ++dt)
                    oacc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, va[gi & 1][dt]), pb, oacc[dt], 0, 0, 0);
                if (gi < 2) {
#pragma unroll
                    for (int dt = 0; dt < kD / 32; ++dt) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);      // one MFMA
                        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);      // multiply-adds, rounding, row sum
                        __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);      // two exponentials
                        __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        l_run += psum[0] + psum[1];
    };

    // Tiles are handled in pairs: one barrier per two tiles.  While the pair (t, t+1) is multiplied, the next
    // pair is on its way into the other two buffers, which were last read before the previous barrier; the
    // loads of a pair are the only ones outstanding, so landing = vmcnt(0).
    static_assert(kStages == 4, "two buffer pairs");
    for (int p = 0; p < 2; ++p)
        if (g_t0 + p < g_t1) load_tile(g_t0 + p, p);
    auto load_q = [&](const infllm_attn_args &src) {
        const int qi = i0 + col;
        const bool ok = live && qi < src.Lq;
        const bf16_t *qrow = (const bf16_t *)src.d_q + (int64_t)b * src.q_sb + (int64_t)h * src.q_sh + (int64_t)qi * src.q_sl;
#pragma unroll
        for (int kk = 0; kk < kD / 16; ++kk) {
            u32x4 raw = ok ? *(const u32x4 *)(qrow + kk * 16 + grp * 8) : u32x4{0, 0, 0, 0};
            qreg[kk] = __builtin_bit_cast(bf16x8, raw);
        }
    };
    // the queries of the stage this split starts in; a split that crosses from the linear tiles into the pages swaps
    // them for the paged stage's queries at its first page (once per workgroup: that wait also covers the tiles in flight)
    bool q_paged = MODE == kPaged || (MODE == kBoth && g_t0 >= n_lin);
    load_q(q_paged ? ap : a);

    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // The compiler does not know that the wait above also covered the query rows; passing them through an empty
    // asm makes it place its own wait for them HERE rather than in front of their first use inside the loop,
    // where a vmcnt(0) would wait for the tiles in flight.
#pragma unroll
    for (int kk = 0; kk < kD / 16; ++kk) asm volatile("" : "+v"(qreg[kk]));
    __syncthreads();
    // does this wave see tile u at all?  (pages: every live wave; linear tiles: the wave's own visible range)
    auto mine = [&](int u) { return (HAS_PAG && u >= n_lin) ? live : (u >= wu0 && u < wu1); };
    for (int t = g_t0; t < g_t1; t += 2) {
        const int buf = (t - g_t0) & 3;                          // 0 or 2
        if (t + 2 < g_t1) load_tile(t + 2, buf ^ 2);
        if (t + 3 < g_t1) load_tile(t + 3, (buf ^ 2) + 1);
#pragma unroll
        for (int e = 0; e < 2; ++e) {                            // wave-uniform conditions; barriers stay outside
            const int u = t + e;
            if (u >= g_t1) break;
            if (MODE == kBoth && u >= n_lin && !q_paged) {
                load_q(ap);
                q_paged = true;
            }
            if (mine(u)) tile_math(buf + e, u);
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
    }

    // ---- epilogue: normalised partial + base-2 log-sum-exp.  The accumulators hold O^T (a lane owns a query and
    //      scattered 4-float pieces of its row); they go through this wave's 16 KB of the now idle tile buffers so
    //      that every store instruction writes two whole 512-byte rows.
    if (!live) return;
    const float l_tot = l_run + wave_xor32(l_run);
    const int qi = i0 + col;
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    int64_t row0 = (((int64_t)split * a.B + b) * a.H + h) * a.Lq + i0;            // row of this wave's first query
    int rows_left = a.Lq - i0;                                                     // valid queries of this tile
    if (geo.out_exc > 0) {                    // a query tile lies inside one execution block (out_exc is a multiple of the tile)
        const int blk = (int)fdiv(i0, geo.out_exc_div), in_blk = i0 - blk * geo.out_exc;
        const int n_blk = min(geo.out_exc, a.Lq - blk * geo.out_exc);
        row0 = (int64_t)blk * geo.out_block_rows + (((int64_t)split * a.B + b) * a.H + h) * n_blk + in_blk;
        rows_left = n_blk - in_blk;
    }
    const int64_t row = row0 + col;
    {
        // fp16 keeps 11 bits of a value that ends up rounded to bf16's 8, and halves what the partials cost in HBM
        // (with few tiles per workgroup their write is a tenth of the kernel); staged rows are 256 bytes, a lane's
        // 4-value piece is 8 bytes, and 16-byte chunks are swizzled by the row
        char *stage = lds_dyn + wave * (kQTile * kD * 2);
#pragma unroll
        for (int dt = 0; dt < kD / 32; ++dt)
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const f16x4 o4{(_Float16)(oacc[dt][4 * q4] * inv), (_Float16)(oacc[dt][4 * q4 + 1] * inv),
                               (_Float16)(oacc[dt][4 * q4 + 2] * inv), (_Float16)(oacc[dt][4 * q4 + 3] * inv)};
                const int chunk = dt * 4 + q4;                                     // 16-byte chunk of the row; grp picks its half
                *(f16x4 *)(stage + col * (kD * 2) + ((chunk ^ col) & 15) * 16 + grp * 8) = o4;
            }
        const int piece = lane & 15;
        _Float16 *o_part = (_Float16 *)a.d_o_part;
#pragma unroll
        for (int k4 = 0; k4 < kQTile / 4; ++k4) {
            const int qr = 4 * k4 + (lane >> 4);
            const u32x4 o8 = *(const u32x4 *)(stage + qr * (kD * 2) + ((piece ^ qr) & 15) * 16);
            if (qr < rows_left) *(u32x4 *)(o_part + (row0 + qr) * kD + piece * 8) = o8;
        }
    }
    if (qi >= a.Lq) return;
    if (grp == 0) a.d_lse_part[row] = l_tot > 0.f ? m_run * scale + log2f(l_tot) : -INFINITY;
}

// one thread per (row, 8 dims): P fp16 partials -> bf16 output row + final lse (merge_piece, common.h)
__global__ __launch_bounds__(256) void attn_merge_kernel(MergeJob job) { merge_piece(job, (int64_t)blockIdx.x * 256 + threadIdx.x); }

// the log-sum-exp half of the merge alone: one thread per row
__global__ __launch_bounds__(256) void attn_merge_lse_kernel(const float *lse_part, int P, int64_t rows, float *lse_out, PartSets ps) {
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= rows) return;
    float m = -INFINITY, den = 0.f;
    for (int p0 = 0; p0 < P; p0 += 8) {                 // online over batches of 8 independent loads
        float l8[8], m8 = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; ++i) l8[i] = p0 + i < P ? lse_part[ps.l(p0 + i, rows) + row] : -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; ++i) m8 = fmaxf(m8, l8[i]);
        if (m8 == -INFINITY) continue;
        const float m_new = fmaxf(m, m8);
        den *= __builtin_amdgcn_exp2f(m - m_new);
#pragma unroll
        for (int i = 0; i < 8; ++i) den += __builtin_amdgcn_exp2f(l8[i] - m_new);
        m = m_new;
    }
    lse_out[row] = den > 0.f ? m + log2f(den) : -INFINITY;
}

// The same two merges for few rows and many partials (decode-sized blocks: a handful of query rows, dozens of key
// splits).  16 adjacent lanes share a row piece and take every 16th partial each, so all partials are one or two
// round trips to memory instead of a chain; the lanes' sums are then joined by a fixed butterfly.
__device__ __forceinline__ float group16_max(float v) {
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
__device__ __forceinline__ float group16_sum(float v) {
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

__global__ __launch_bounds__(256) void attn_merge_wide_kernel(const _Float16 *o_part, const float *lse_part, int P, int B, int H,
                                                              int Lq, bf16_t *out, int64_t o_sb, int64_t o_sh, int64_t o_sl,
                                                              float *lse_out, PartSets ps) {
    const int64_t rows = (int64_t)B * H * Lq;
    const int64_t e = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 4;       // (row, 8 dims)
    const int pl = threadIdx.x & 15;
    const int64_t row = e >> 4;
    const int c = (int)(e & 15);
    if (row >= rows) return;                                                 // whole 16-lane groups leave together
    constexpr int kMine = 8;                                                 // partials per lane: P <= 128
    float l[kMine];
    f16x8 o[kMine];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < kMine; ++i) {
        const int p = pl + 16 * i;
        const bool on = p < P;
        l[i] = on ? lse_part[ps.l(p, rows) + row] : -INFINITY;
        o[i] = on ? *(const f16x8 *)(o_part + (ps.l(p, rows) + row) * kD + ps.o(p) + c * 8) : f16x8{0, 0, 0, 0, 0, 0, 0, 0};
        m = fmaxf(m, l[i]);
    }
    m = group16_max(m);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, den = 0.f;
    if (m > -INFINITY) {
#pragma unroll
        for (int i = 0; i < kMine; ++i) {
            const float w = __builtin_amdgcn_exp2f(l[i] - m);
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] += (float)o[i][j] * w;
            den += w;
        }
    }
    den = group16_sum(den);
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = group16_sum(acc[j]);
    if (pl != 0) return;
    const float inv = den > 0.f ? 1.f / den : 0.f;
    const int i = (int)(row % Lq), h = (int)((row / Lq) % H), b = (int)(row / ((int64_t)Lq * H));
    u32x4 packed{pack_bf16x2(acc[0] * inv, acc[1] * inv), pack_bf16x2(acc[2] * inv, acc[3] * inv),
                 pack_bf16x2(acc[4] * inv, acc[5] * inv), pack_bf16x2(acc[6] * inv, acc[7] * inv)};
    *(u32x4 *)(out + (int64_t)b * o_sb + (int64_t)h * o_sh + (int64_t)i * o_sl + c * 8) = packed;
    if (c == 0 && lse_out) lse_out[row] = den > 0.f ? m + log2f(den) : -INFINITY;
}

__global__ __launch_bounds__(256) void attn_merge_lse_wide_kernel(const float *lse_part, int P, int64_t rows, float *lse_out, PartSets ps) {
    const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 4;
    const int pl = threadIdx.x & 15;
    if (row >= rows) return;
    constexpr int kMine = 8;
    float l[kMine], m = -INFINITY;
#pragma unroll
    for (int i = 0; i < kMine; ++i) {
        const int p = pl + 16 * i;
        l[i] = p < P ? lse_part[ps.l(p, rows) + row] : -INFINITY;
        m = fmaxf(m, l[i]);
    }
    m = group16_max(m);
    float den = 0.f;
    if (m > -INFINITY) {
#pragma unroll
        for (int i = 0; i < kMine; ++i) den += __builtin_amdgcn_exp2f(l[i] - m);
    }
    den = group16_sum(den);
    if (pl == 0) lse_out[row] = den > 0.f ? m + log2f(den) : -INFINITY;
}

}  // namespace

#define HIP_OK_ATTN(call, what)                                                         \
    do {                                                                                \
        hipError_t e_ = (call);                                                         \
        if (e_ != hipSuccess) return infllm_fail(-2, "%s: %s", what, hipGetErrorString(e_)); \
    } while (0)

namespace {

int check_linear_stage(const infllm_attn_args *a) {
    INFLLM_REQUIRE(a->j_hi <= a->j_lo || (a->d_k && a->d_v), "attn_stage: null k / v pointer");
    INFLLM_REQUIRE(a->cap > 0 && a->cap % kTile == 0, "attn_stage: cap %lld is not a positive multiple of %d",
                   (long long)a->cap, kTile);
    INFLLM_REQUIRE(a->j_lo >= 0 && a->j_hi - a->j_lo <= a->cap, "attn_stage: key range [%lld,%lld) exceeds cap %lld",
                   (long long)a->j_lo, (long long)a->j_hi, (long long)a->cap);
    INFLLM_REQUIRE(a->mask >= 0 && a->mask <= 2, "attn_stage: unknown mask %d", a->mask);
    INFLLM_REQUIRE(a->j_hi < (1ll << 36), "attn_stage: key range beyond 2^36 rows");
    INFLLM_REQUIRE((a->k_sl % 8 | a->k_sh % 8 | a->k_sb % 8 | a->v_sl % 8 | a->v_sh % 8 | a->v_sb % 8) == 0,
                   "attn_stage: k/v strides must be multiples of 8");
    return 0;
}

int check_common(const infllm_attn_args *a) {
    INFLLM_REQUIRE(a->d_q, "attn_stage: null q pointer");
    INFLLM_REQUIRE(a->B > 0 && a->H > 0 && a->Hkv > 0 && a->H % a->Hkv == 0 && a->Lq > 0,
                   "attn_stage: bad geometry B=%d H=%d Hkv=%d Lq=%d", a->B, a->H, a->Hkv, a->Lq);
    INFLLM_REQUIRE(a->nsplit >= 1 && a->nsplit <= 64, "attn_stage: nsplit %d out of range", a->nsplit);
    INFLLM_REQUIRE((a->q_sl % 8 | a->q_sh % 8 | a->q_sb % 8) == 0, "attn_stage: q strides must be multiples of 8");
    return 0;
}

// mode: kLinear (a), kPaged (a), kBoth (a = linear stage, a2 = paged stage); h_pages: NULL, or the paged stage's table
// [B, n_pages] in HOST memory, B * n_pages <= kInlinePages, which then travels in the launch (d_pages is not read)
int launch_stage(int mode, const infllm_attn_args *a, const infllm_attn_args *a2, void *stream, const infllm_page *h_pages = nullptr,
                 int out_exc = 0, int64_t out_block_rows = 0) {
    const int G = a->H / a->Hkv;
    const int n_tasks = ((a->Lq + kQTile - 1) / kQTile) * G;
    dim3 grid((n_tasks + kWaves - 1) / kWaves, a->B * a->Hkv, a->nsplit);
    INFLLM_REQUIRE((int64_t)grid.x * grid.y * grid.z < (1ll << 31), "attn_stage: grid too large");
    StageGeom geo{fast_div(grid.x), fast_div(grid.y), fast_div((uint32_t)a->Hkv), fast_div((uint32_t)G),
                  fast_div((uint32_t)a->nsplit), fast_div(1), n_tasks, out_exc, out_block_rows, fast_div((uint32_t)(out_exc > 0 ? out_exc : 1))};
    // tile indices stay below 2^30, so any ring of 2^31 tiles or more never wraps: one divisor stands for all of them
    if (mode != kPaged) geo.cap_tiles = fast_div((uint32_t)std::min<int64_t>(a->cap / kTile, 1ll << 31));
    constexpr size_t lds_bytes = 2 * kStages * kTileBytes;
    static bool lds_set[3] = {false, false, false};           // dynamic LDS above 64 KiB must be enabled once per kernel
    const infllm_attn_args &second = a2 ? *a2 : *a;
    if (h_pages) {
        const infllm_attn_args &pg = mode == kBoth ? second : *a;
        INFLLM_REQUIRE(mode != kLinear && pg.n_pages >= 0 && (int64_t)pg.B * pg.n_pages <= kInlinePages,
                       "attn_stage: %d x %d pages do not fit a launch", pg.B, pg.n_pages);
        static bool lds_set_inline[3] = {false, false, false};
        const void *fn = mode == kPaged ? (const void *)attn_stage_kernel<kPaged, true> : (const void *)attn_stage_kernel<kBoth, true>;
        if (!lds_set_inline[mode]) {
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
            if (e != hipSuccess) return infllm_fail(-2, "attn_stage: %s", hipGetErrorString(e));
            lds_set_inline[mode] = true;
        }
        InlinePages table;
        memcpy(table.p, h_pages, sizeof(infllm_page) * pg.B * pg.n_pages);
        if (mode == kPaged) hipLaunchKernelGGL((attn_stage_kernel<kPaged, true>), grid, dim3(kThreads), lds_bytes, (hipStream_t)stream, *a, second, geo, table);
        else hipLaunchKernelGGL((attn_stage_kernel<kBoth, true>), grid, dim3(kThreads), lds_bytes, (hipStream_t)stream, *a, second, geo, table);
        INFLLM_CHECK_LAUNCH("attn_stage");
        return 0;
    }
    const void *fn = mode == kLinear ? (const void *)attn_stage_kernel<kLinear>
                     : mode == kPaged ? (const void *)attn_stage_kernel<kPaged> : (const void *)attn_stage_kernel<kBoth>;
    if (!lds_set[mode]) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) return infllm_fail(-2, "attn_stage: %s", hipGetErrorString(e));
        lds_set[mode] = true;
    }
    if (mode == kLinear) hipLaunchKernelGGL(attn_stage_kernel<kLinear>, grid, dim3(kThreads), lds_bytes, (hipStream_t)stream, *a, second, geo, NoInlinePages{});
    else if (mode == kPaged) hipLaunchKernelGGL(attn_stage_kernel<kPaged>, grid, dim3(kThreads), lds_bytes, (hipStream_t)stream, *a, second, geo, NoInlinePages{});
    else hipLaunchKernelGGL(attn_stage_kernel<kBoth>, grid, dim3(kThreads), lds_bytes, (hipStream_t)stream, *a, second, geo, NoInlinePages{});
    INFLLM_CHECK_LAUNCH("attn_stage");
    return 0;
}

}  // namespace

extern "C" int infllm_attn_stage(const infllm_attn_args *a, void *stream) {
    INFLLM_REQUIRE(a != nullptr, "attn_stage: null argument block");
    INFLLM_REQUIRE(a->d_o_part && a->d_lse_part, "attn_stage: null output pointer");
    int rc = check_common(a);
    if (rc) return rc;
    if (a->d_pages) {
        INFLLM_REQUIRE(a->n_pages >= 0, "attn_stage: negative page count");
        return launch_stage(kPaged, a, nullptr, stream);
    }
    rc = check_linear_stage(a);
    return rc ? rc : launch_stage(kLinear, a, nullptr, stream);
}

// library-internal: a linear stage over the queries of several consecutive execution blocks of `exc` rows (the last
// may be shorter); block k's partial rows and log-sum-exps start at row k * block_rows of d_o_part / d_lse_part and
// are laid out [nsplit, B, H, n_k, 128] / [nsplit, B, H, n_k], as infllm_attn_merge takes them for that block.
int infllm_attn_stage_blocked(const infllm_attn_args *a, int32_t exc, int64_t block_rows, void *stream) {
    INFLLM_REQUIRE(a && a->d_o_part && a->d_lse_part && !a->d_pages, "attn_stage_blocked: null argument or paged source");
    INFLLM_REQUIRE(exc > 0 && exc % kQTile == 0, "attn_stage_blocked: blocks of %d rows are not whole query tiles", exc);
    INFLLM_REQUIRE(block_rows >= (int64_t)a->nsplit * a->B * a->H * (a->Lq < exc ? a->Lq : exc), "attn_stage_blocked: block stride too small");
    int rc = check_common(a);
    if (rc) return rc;
    rc = check_linear_stage(a);
    return rc ? rc : launch_stage(kLinear, a, nullptr, stream, nullptr, exc, block_rows);
}

// library-internal: the paged stage (local == NULL) or both stages in one launch, with the page table [B, n_pages]
// given in HOST memory and carried by the launch; global->d_pages is not read.  B * n_pages <= infllm_inline_page_limit().
int infllm_inline_page_limit() { return kInlinePages; }
int infllm_attn_paged_inline(const infllm_attn_args *local, const infllm_attn_args *global, const infllm_page *h_pages, void *stream) {
    INFLLM_REQUIRE(global && h_pages && global->d_o_part && global->d_lse_part, "attn_paged_inline: null argument");
    int rc = check_common(global);
    if (rc) return rc;
    if (!local) return launch_stage(kPaged, global, nullptr, stream, h_pages);
    INFLLM_REQUIRE(local->d_o_part && local->d_lse_part && !local->d_pages, "attn_paged_inline: bad local stage");
    INFLLM_REQUIRE(local->B == global->B && local->H == global->H && local->Hkv == global->Hkv && local->Lq == global->Lq &&
                       local->softmax_scale == global->softmax_scale,
                   "attn_paged_inline: the two stages disagree");
    rc = check_common(local);
    if (rc) return rc;
    rc = check_linear_stage(local);
    return rc ? rc : launch_stage(kBoth, local, global, stream, h_pages);
}

extern "C" int infllm_attn_stages_fused(const infllm_attn_args *local, const infllm_attn_args *global, void *stream) {
    INFLLM_REQUIRE(local && global, "attn_stages_fused: null argument block");
    INFLLM_REQUIRE(local->d_o_part && local->d_lse_part, "attn_stages_fused: null output pointer");
    INFLLM_REQUIRE(!local->d_pages && global->d_pages && global->n_pages >= 0,
                   "attn_stages_fused: the first stage must be linear, the second paged");
    INFLLM_REQUIRE(local->B == global->B && local->H == global->H && local->Hkv == global->Hkv && local->Lq == global->Lq,
                   "attn_stages_fused: the two stages disagree on B / H / Hkv / Lq");
    INFLLM_REQUIRE(local->softmax_scale == global->softmax_scale, "attn_stages_fused: the two stages disagree on the softmax scale");
    int rc = check_common(local);
    if (rc) return rc;
    rc = check_common(global);
    if (rc) return rc;
    rc = check_linear_stage(local);
    return rc ? rc : launch_stage(kBoth, local, global, stream);
}

extern "C" int infllm_attn_merge(const uint16_t *d_o_part, const float *d_lse_part, int32_t P, int32_t B, int32_t H,
                                 int32_t Lq, void *d_out, int64_t o_sb, int64_t o_sh, int64_t o_sl, float *d_lse,
                                 void *stream);

extern "C" int infllm_attn_fwd(const infllm_attn_args *local, const infllm_attn_args *global, void *d_out, int64_t o_sb,
                               int64_t o_sh, int64_t o_sl, float *d_lse, void *stream) {
    INFLLM_REQUIRE(local || global, "attn_fwd: no stage given");
    INFLLM_REQUIRE(d_out || d_lse, "attn_fwd: neither output nor lse requested");
    const infllm_attn_args *first = local ? local : global;
    int parts = first->nsplit;
    if (local && global) {
        INFLLM_REQUIRE(local->B == global->B && local->H == global->H && local->Lq == global->Lq,
                       "attn_fwd: the two stages disagree on B / H / Lq");
        const int64_t rows = (int64_t)local->B * local->H * local->Lq;
        INFLLM_REQUIRE(global->d_o_part == local->d_o_part + (int64_t)local->nsplit * rows * kD &&
                           global->d_lse_part == local->d_lse_part + (int64_t)local->nsplit * rows,
                       "attn_fwd: the global stage's partials must follow the local stage's in one buffer");
        parts += global->nsplit;
    }
    int rc = local ? infllm_attn_stage(local, stream) : 0;
    if (rc) return rc;
    rc = global ? infllm_attn_stage(global, stream) : 0;
    if (rc) return rc;
    return infllm_attn_merge(first->d_o_part, first->d_lse_part, parts, first->B, first->H, first->Lq, d_out, o_sb, o_sh, o_sl,
                             d_lse, stream);
}

// ---- the forward for callers that cannot allocate
// The stages' partial rows are scratch memory: infllm_attn_fwd takes them from the caller.  A caller under HIP graph
// capture, in a tight serving loop or in a harness that forbids hipMalloc has nowhere to get them from, so this
// variant keeps them in an array of the library's own image.  Every GPU the library runs on holds its own copy of the
// array (at its own address) until the process ends; every call on a GPU uses that GPU's copy, so calls that overlap on
// one GPU race.  Nothing has to be cleared between calls: each split writes all of its rows and log-sum-exps before
// the merge reads them.
constexpr int64_t kStaticPartRows = INFLLM_NOALLOC_MAX_PART_ROWS;            // (split, batch row, head, query) rows
static __device__ __align__(256) unsigned char attn_static_scratch[kStaticPartRows * (kD * 2 + 4)];
constexpr int kMaxDevices = 64;
// per device: where ITS copy of the array lives.  Atomic: two threads making their first call on a device both look the
// address up and store the same value
static std::atomic<unsigned char *> static_scratch_ptr[kMaxDevices];

extern "C" int infllm_attn_fwd_noalloc(const infllm_attn_args *local, const infllm_attn_args *global, void *d_out, int64_t o_sb,
                                       int64_t o_sh, int64_t o_sl, float *d_lse, void *stream) {
    INFLLM_REQUIRE(local || global, "attn_fwd_noalloc: no stage given");
    const infllm_attn_args *first = local ? local : global;
    INFLLM_REQUIRE(first->B > 0 && first->H > 0 && first->Lq > 0, "attn_fwd_noalloc: bad geometry");
    if (local && global)
        INFLLM_REQUIRE(local->B == global->B && local->H == global->H && local->Lq == global->Lq,
                       "attn_fwd_noalloc: the two stages disagree on B / H / Lq");
    const int parts = (local ? local->nsplit : 0) + (global ? global->nsplit : 0);
    const int64_t rows = (int64_t)first->B * first->H * first->Lq;
    INFLLM_REQUIRE(parts >= 1 && parts <= 128, "attn_fwd_noalloc: %d key splits", parts);
    INFLLM_REQUIRE(parts * rows <= kStaticPartRows,
                   "attn_fwd_noalloc: %d splits x %lld rows exceed the built-in scratch of %lld partial rows (use infllm_attn_fwd "
                   "with a workspace of your own)", parts, (long long)rows, (long long)kStaticPartRows);
    int dev = -1;
    HIP_OK_ATTN(hipGetDevice(&dev), "attn_fwd_noalloc");
    INFLLM_REQUIRE(dev >= 0 && dev < kMaxDevices, "attn_fwd_noalloc: device %d", dev);
    unsigned char *scratch = static_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!scratch) {                            // once per device, with that device current: the symbol's address THERE
        void *p = nullptr;
        HIP_OK_ATTN(hipGetSymbolAddress(&p, HIP_SYMBOL(attn_static_scratch)), "attn_fwd_noalloc: hipGetSymbolAddress");
        INFLLM_REQUIRE(p != nullptr, "attn_fwd_noalloc: no address for the scratch array");
        scratch = (unsigned char *)p;
        static_scratch_ptr[dev].store(scratch, std::memory_order_release);
    }
    // o partials first (fp16 rows), the log-sum-exps behind all of them; the global stage's follow the local stage's
    uint16_t *o_part = (uint16_t *)scratch;
    float *lse_part = (float *)(scratch + kStaticPartRows * kD * 2);
    infllm_attn_args l{}, g{};
    if (local) {
        l = *local;
        l.d_o_part = o_part;
        l.d_lse_part = lse_part;
    }
    if (global) {
        g = *global;
        const int64_t skip = local ? (int64_t)local->nsplit * rows : 0;
        g.d_o_part = o_part + skip * kD;
        g.d_lse_part = lse_part + skip;
    }
    return infllm_attn_fwd(local ? &l : nullptr, global ? &g : nullptr, d_out, o_sb, o_sh, o_sl, d_lse, stream);
}

// library-internal: the description of a merge over two sets of partials, P1 behind (d_o_part, d_lse_part) and P2
// behind (d_o_part2, d_lse_part2), in that order; P2 == 0 is the plain merge
int infllm_merge_job(const uint16_t *d_o_part, const float *d_lse_part, int32_t P1, const uint16_t *d_o_part2, const float *d_lse_part2,
                     int32_t P2, int32_t B, int32_t H, int32_t Lq, void *d_out, int64_t o_sb, int64_t o_sh, int64_t o_sl, float *d_lse,
                     MergeJob *job) {
    INFLLM_REQUIRE(d_o_part && d_lse_part && job, "attn_merge: null pointer");
    INFLLM_REQUIRE(P1 >= 1 && P2 >= 0 && (P2 == 0 || (d_o_part2 && d_lse_part2)), "attn_merge: bad partial sets %d + %d", P1, P2);
    INFLLM_REQUIRE(B > 0 && H > 0 && Lq > 0, "attn_merge: bad sizes B=%d H=%d Lq=%d", B, H, Lq);
    INFLLM_REQUIRE((o_sl % 8 | o_sh % 8 | o_sb % 8) == 0, "attn_merge: output strides must be multiples of 8");
    PartSets ps{P1 + P2, 0, 0};
    if (P2 > 0) {
        const int64_t rows_ = (int64_t)B * H * Lq;
        ps.n_first = P1;
        // index (p * rows + row) of the first buffers -> index ((p - P1) * rows + row) of the second
        ps.skip_l = (int64_t)(((intptr_t)d_lse_part2 - (intptr_t)d_lse_part) / (intptr_t)sizeof(float)) - (int64_t)P1 * rows_;
        ps.skip_o = (int64_t)(((intptr_t)d_o_part2 - (intptr_t)d_o_part) / 2) - (int64_t)P1 * rows_ * kD - ps.skip_l * kD;
    }
    *job = MergeJob{(const _Float16 *)d_o_part, d_lse_part, P1 + P2, B, H, Lq, (bf16_t *)d_out, o_sb, o_sh, o_sl, d_lse, ps};
    return 0;
}

// library-internal: the merge over two sets of partials
int infllm_attn_merge2(const uint16_t *d_o_part, const float *d_lse_part, int32_t P1, const uint16_t *d_o_part2,
                       const float *d_lse_part2, int32_t P2, int32_t B, int32_t H, int32_t Lq, void *d_out, int64_t o_sb,
                       int64_t o_sh, int64_t o_sl, float *d_lse, void *stream) {
    MergeJob job;
    const int jrc = infllm_merge_job(d_o_part, d_lse_part, P1, d_o_part2, d_lse_part2, P2, B, H, Lq, d_out, o_sb, o_sh, o_sl, d_lse, &job);
    if (jrc) return jrc;
    const int32_t P = P1 + P2;
    const PartSets ps = job.ps;
    // few rows, many partials (decode-sized blocks): 16 lanes per row piece, each taking every 16th partial
    const bool wide = P > 8 && P <= 128 && (int64_t)B * H * Lq <= 2048;
    if (!d_out) {                                     // log-sum-exp only
        INFLLM_REQUIRE(d_lse, "attn_merge: neither output nor lse requested");
        const int64_t rows = (int64_t)B * H * Lq;
        if (wide)
            hipLaunchKernelGGL(attn_merge_lse_wide_kernel, dim3((unsigned)((rows * 16 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                               d_lse_part, P, rows, d_lse, ps);
        else
            hipLaunchKernelGGL(attn_merge_lse_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, (hipStream_t)stream, d_lse_part,
                               P, rows, d_lse, ps);
        INFLLM_CHECK_LAUNCH("attn_merge (lse)");
        return 0;
    }
    const int64_t threads = (int64_t)B * H * Lq * 16;
    if (wide)
        hipLaunchKernelGGL(attn_merge_wide_kernel, dim3((unsigned)((threads * 16 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                           (const _Float16 *)d_o_part, d_lse_part, P, B, H, Lq, (bf16_t *)d_out, o_sb, o_sh, o_sl, d_lse, ps);
    else
        hipLaunchKernelGGL(attn_merge_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                           job);
    INFLLM_CHECK_LAUNCH("attn_merge");
    return 0;
}

extern "C" int infllm_attn_merge(const uint16_t *d_o_part, const float *d_lse_part, int32_t P, int32_t B, int32_t H,
                                 int32_t Lq, void *d_out, int64_t o_sb, int64_t o_sh, int64_t o_sl, float *d_lse,
                                 void *stream) {
    return infllm_attn_merge2(d_o_part, d_lse_part, P, nullptr, nullptr, 0, B, H, Lq, d_out, o_sb, o_sh, o_sl, d_lse, stream);
}
