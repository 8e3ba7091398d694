// Shared helpers for the gfx950 kernels of libinfllm_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/infllm_hip.h"

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int kD = INFLLM_HEAD_DIM;       // head_dim
constexpr int kTile = INFLLM_KEY_TILE;    // keys per tile
constexpr int kWave = 64;

// thread-local error text, returned by infllm_last_error()
char *infllm_err_buf();
int infllm_fail(int code, const char *fmt, ...);

#define INFLLM_REQUIRE(cond, ...)                      \
    do {                                               \
        if (!(cond)) return infllm_fail(-1, __VA_ARGS__); \
    } while (0)

#define INFLLM_CHECK_LAUNCH(name)                                                     \
    do {                                                                              \
        hipError_t e_ = hipGetLastError();                                            \
        if (e_ != hipSuccess) return infllm_fail(-2, "%s: %s", name, hipGetErrorString(e_)); \
    } while (0)

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
    return __uint_as_float(bits16 << 16);
}
// round-to-nearest-even fp32 -> bf16 bits (inputs are finite here; NaN kept quiet)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
// two fp32 -> packed bf16 pair, round-to-nearest-even (one v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
// acc + lo + hi of a packed bf16 pair, exactly (v_dot2c_f32_bf16 against a pair of ones)
__device__ __forceinline__ float sum_bf16x2(uint32_t pair, float acc) {
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pair), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), acc, false);
}
__device__ __forceinline__ float wave_xor32(float x) {
    return __shfl_xor(x, 32, 64);
}

// ---- the merge of partial attention outputs, shared by the merge kernels (attn.hip) and by the local-score launch
//      that carries the merge of its block along (score.hip)
// The partials of a merge may lie in two places: the first n_first of them behind the pointers the kernel is given,
// the rest wherever the second stage wrote them.  skip_l / skip_o are what has to be added to an index into the first
// buffers (log-sum-exps; fp16 elements beyond the row term) to land in the second.
struct PartSets {
    int32_t n_first;
    int64_t skip_l, skip_o;
    __device__ __forceinline__ int64_t l(int p, int64_t rows) const { return (int64_t)p * rows + (p >= n_first ? skip_l : 0); }
    __device__ __forceinline__ int64_t o(int p) const { return p >= n_first ? skip_o : 0; }
};

struct MergeJob {
    const _Float16 *o_part;            // [P, B, H, Lq, 128] normalised partial rows (see PartSets)
    const float *lse_part;             // [P, B, H, Lq] their base-2 log-sum-exps
    int32_t P, B, H, Lq;
    bf16_t *out;                       // rows [b, h, i] at b * o_sb + h * o_sh + i * o_sl
    int64_t o_sb, o_sh, o_sl;
    float *lse_out;                    // [B, H, Lq] or NULL
    PartSets ps;
};

// thread e of the merge: (row, 8 dims) = (e / 16, e % 16).  (inf_llm/attention/dot_production_attention/torch_impl.py:15-36)
__device__ __forceinline__ void merge_piece(const MergeJob &mj, int64_t e) {
    const _Float16 *o_part = mj.o_part;
    const float *lse_part = mj.lse_part;
    const PartSets ps = mj.ps;
    const int P = mj.P, H = mj.H, Lq = mj.Lq;
    const int64_t rows = (int64_t)mj.B * H * Lq;
    const int64_t row = e >> 4;
    const int c = (int)(e & 15);
    if (row >= rows) return;
    // partials in batches of 8 so that the loads of a batch are in flight together (decode-sized blocks merge
    // dozens of partials of very few rows: a chain of dependent loads would be all latency)
    float m = -INFINITY;
    for (int p0 = 0; p0 < P; p0 += 8) {
        float l8[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) l8[i] = p0 + i < P ? lse_part[ps.l(p0 + i, rows) + row] : -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; ++i) m = fmaxf(m, l8[i]);
    }
    float acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = 0.f;
    float den = 0.f;
    if (m > -INFINITY) {
        for (int p0 = 0; p0 < P; p0 += 8) {
            float l8[8];
            f16x8 o8[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const bool on = p0 + i < P;
                l8[i] = on ? lse_part[ps.l(p0 + i, rows) + row] : -INFINITY;
                o8[i] = on ? *(const f16x8 *)(o_part + (ps.l(p0 + i, rows) + row) * kD + ps.o(p0 + i) + c * 8) : f16x8{0, 0, 0, 0, 0, 0, 0, 0};
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float w = __builtin_amdgcn_exp2f(l8[i] - m);       // exp2(-inf) = 0: empty partials hold zeros
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[j] += (float)o8[i][j] * w;
                den += w;
            }
        }
    }
    const float inv = den > 0.f ? 1.f / den : 0.f;
    const int i = (int)(row % Lq), h = (int)((row / Lq) % H), b = (int)(row / ((int64_t)Lq * H));
    u32x4 packed{pack_bf16x2(acc[0] * inv, acc[1] * inv), pack_bf16x2(acc[2] * inv, acc[3] * inv),
                 pack_bf16x2(acc[4] * inv, acc[5] * inv), pack_bf16x2(acc[6] * inv, acc[7] * inv)};
    *(u32x4 *)(mj.out + (int64_t)b * mj.o_sb + (int64_t)h * mj.o_sh + (int64_t)i * mj.o_sl + c * 8) = packed;
    if (c == 0 && mj.lse_out) mj.lse_out[row] = den > 0.f ? m + log2f(den) : -INFINITY;
}


// ---- a call's selections from lists made once per call (retrieve.hip: call_rank_kernel; stream.hip drives it)
// For every later block of a prepared call the k best of the units that existed when the call began are known
// (`base`), and so are those units' scores under the block's mean query (`scores`).  After a block has carved
// n_new units, workgroup x of one launch scores them under the mean query of block j0 + x and, for the two blocks
// that need a list now, ranks the base list against all the units carved since the call began.
struct CallRankJob {
    const bf16_t *reps;                // [B][units][C] representatives
    int64_t rep_sb, rep_su;
    const float *qbars;                // [blocks][B][C] mean queries of the call's blocks
    float *scores;                     // [blocks][B][cols]
    int64_t cols;
    const int32_t *base;               // [blocks][B][k]
    int32_t B, k;
    int32_t n_base;                    // units that existed when the call began
    int32_t first_new, n_new;          // the units carved just now: [first_new, first_new + n_new)
    int32_t j0;                        // workgroup x works for block j0 + x
    int32_t j_sel, j_cand;             // blocks whose selection / candidate list leaves now (-1: none)
    int32_t *sel_out, *sel_flag;       // [B][k] ids, then the sequence number
    int32_t sel_seq;
    int32_t *cand_out, *cand_flag;
    int32_t cand_seq;
};
