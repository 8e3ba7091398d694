// Prologue of the streaming path: RoPE of new tokens and their staging into the
// per-layer rings (inf_llm/attention/rope.py:89-112,
// inf_llm/attention/context_manager.py:719-747, 373-375).
#include "common.h"

namespace {

constexpr int kPosPerBlock = 16;   // stream positions handled by one workgroup
constexpr int kHalf = kD / 2;      // 64 rotation pairs per head

struct Rot8 {
    u32x4 lo, hi;
};

// rotate 8 pairs (lo[i], hi[i]) by (c[i], s[i]); fp32 math, one rounding to bf16
__device__ __forceinline__ Rot8 rotate8(u32x4 xlo, u32x4 xhi, const float2 *cs) {
    Rot8 r;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        float a0 = bf16_bits_to_f32(xlo[w] & 0xffffu), a1 = bf16_bits_to_f32(xlo[w] >> 16);
        float b0 = bf16_bits_to_f32(xhi[w] & 0xffffu), b1 = bf16_bits_to_f32(xhi[w] >> 16);
        float2 c0 = cs[2 * w], c1 = cs[2 * w + 1];
        // x*cos + rotate_half(x)*sin, rotate_half = (-hi, lo)
        r.lo[w] = pack_bf16x2(a0 * c0.x - b0 * c0.y, a1 * c1.x - b1 * c1.y);
        r.hi[w] = pack_bf16x2(b0 * c0.x + a0 * c0.y, b1 * c1.x + a1 * c1.y);
    }
    return r;
}

__global__ __launch_bounds__(256) void ingest_kernel(infllm_ingest_args a) {
    __shared__ float2 cs_pos[kPosPerBlock][kHalf];
    __shared__ float2 cs_glb[kHalf];
    const int tid = threadIdx.x;
    const int b = blockIdx.y;
    const int p0 = blockIdx.x * kPosPerBlock;
    const int np = min(kPosPerBlock, a.n - p0);

    for (int e = tid; e < kPosPerBlock * kHalf; e += 256) {
        int p = e / kHalf, f = e % kHalf;
        double ang = (double)(a.pos0 + p0 + p) * a.distance_scale * (double)a.d_inv_freq[f];
        double s, c;
        sincos(ang, &s, &c);
        cs_pos[p][f] = make_float2((float)c, (float)s);
    }
    if (tid < kHalf) {
        double ang = (double)a.glb_pos * a.distance_scale * (double)a.d_inv_freq[tid];
        double s, c;
        sincos(ang, &s, &c);
        cs_glb[tid] = make_float2((float)c, (float)s);
    }
    __syncthreads();

    const bf16_t *q = (const bf16_t *)a.d_q + (int64_t)b * a.q_sb;
    const bf16_t *k = (const bf16_t *)a.d_k + (int64_t)b * a.k_sb;
    const bf16_t *v = (const bf16_t *)a.d_v + (int64_t)b * a.v_sb;
    bf16_t *q_loc = (bf16_t *)a.d_q_loc + (int64_t)b * a.H * a.n * kD;
    bf16_t *q_glb = (bf16_t *)a.d_q_glb + (int64_t)b * a.H * a.n * kD;
    const int64_t ring_b = (int64_t)b * a.Hkv * a.ring_cap * kD;
    bf16_t *rk_raw = (bf16_t *)a.d_ring_k_raw + ring_b;
    bf16_t *rk_rot = (bf16_t *)a.d_ring_k_rot + ring_b;
    bf16_t *rv = (bf16_t *)a.d_ring_v + ring_b;

    // query heads: 8 threads per (head, position) row
    for (int e = tid; e < a.H * np * 8; e += 256) {
        int c = e & 7, p = (e >> 3) % np, h = (e >> 3) / np;
        const bf16_t *src = q + (int64_t)h * a.q_sh + (int64_t)(p0 + p) * a.q_sl;
        u32x4 lo = *(const u32x4 *)(src + c * 8), hi = *(const u32x4 *)(src + kHalf + c * 8);
        int64_t o = ((int64_t)h * a.n + p0 + p) * kD;
        Rot8 r = rotate8(lo, hi, &cs_pos[p][c * 8]);
        *(u32x4 *)(q_loc + o + c * 8) = r.lo;
        *(u32x4 *)(q_loc + o + kHalf + c * 8) = r.hi;
        r = rotate8(lo, hi, &cs_glb[c * 8]);
        *(u32x4 *)(q_glb + o + c * 8) = r.lo;
        *(u32x4 *)(q_glb + o + kHalf + c * 8) = r.hi;
    }
    // key heads: raw copy + rotated copy into the rings
    for (int e = tid; e < a.Hkv * np * 8; e += 256) {
        int c = e & 7, p = (e >> 3) % np, h = (e >> 3) / np;
        const bf16_t *src = k + (int64_t)h * a.k_sh + (int64_t)(p0 + p) * a.k_sl;
        u32x4 lo = *(const u32x4 *)(src + c * 8), hi = *(const u32x4 *)(src + kHalf + c * 8);
        int64_t row = (a.pos0 + p0 + p) % a.ring_cap;
        int64_t o = ((int64_t)h * a.ring_cap + row) * kD;
        *(u32x4 *)(rk_raw + o + c * 8) = lo;
        *(u32x4 *)(rk_raw + o + kHalf + c * 8) = hi;
        Rot8 r = rotate8(lo, hi, &cs_pos[p][c * 8]);
        *(u32x4 *)(rk_rot + o + c * 8) = r.lo;
        *(u32x4 *)(rk_rot + o + kHalf + c * 8) = r.hi;
    }
    // values: plain copy, 16 threads per row
    for (int e = tid; e < a.Hkv * np * 16; e += 256) {
        int c = e & 15, p = (e >> 4) % np, h = (e >> 4) / np;
        const bf16_t *src = v + (int64_t)h * a.v_sh + (int64_t)(p0 + p) * a.v_sl;
        int64_t row = (a.pos0 + p0 + p) % a.ring_cap;
        *(u32x4 *)(rv + ((int64_t)h * a.ring_cap + row) * kD + c * 8) = *(const u32x4 *)(src + c * 8);
    }
    // the score track of a new token starts at zero (context_manager.py:733-741)
    for (int e = tid; e < a.H * np; e += 256) {
        int p = e % np, h = e / np;
        int64_t row = (a.pos0 + p0 + p) % a.ring_cap;
        a.d_ring_score[((int64_t)b * a.H + h) * a.ring_cap + row] = 0.f;
    }
}

constexpr int kMeanThreads = 512;

// one workgroup per (block, head, batch row); fixed summation order => deterministic
__global__ __launch_bounds__(kMeanThreads) void block_mean_kernel(const bf16_t *q_glb, int H, int n, int exc,
                                                                 float *qbar, int n_blocks) {
    __shared__ float2 part[kMeanThreads / 64][64];
    const int blk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int r0 = blk * exc, r1 = min(r0 + exc, n);
    const bf16_t *src = q_glb + ((int64_t)b * H + h) * (int64_t)n * kD;
    float s0 = 0.f, s1 = 0.f;
    for (int r = r0 + grp; r < r1; r += kMeanThreads / 64) {
        uint32_t w = *(const uint32_t *)(src + (int64_t)r * kD + lane * 2);
        s0 += bf16_bits_to_f32(w & 0xffffu);
        s1 += bf16_bits_to_f32(w >> 16);
    }
    part[grp][lane] = make_float2(s0, s1);
    __syncthreads();
    if (grp == 0) {
        float t0 = 0.f, t1 = 0.f;
        for (int g = 0; g < kMeanThreads / 64; ++g) {
            t0 += part[g][lane].x;
            t1 += part[g][lane].y;
        }
        float inv = 1.f / (float)(r1 - r0);
        float *dst = qbar + (((int64_t)b * n_blocks + blk) * H + h) * kD + lane * 2;
        dst[0] = t0 * inv;
        dst[1] = t1 * inv;
    }
}

__global__ __launch_bounds__(256) void gather_rows_kernel(const bf16_t *ring, int64_t ring_cap, int Hkv, int64_t t0,
                                                          int n, int unit_rows, bf16_t *out, int64_t out_sb,
                                                          int64_t out_su, int64_t out_sh) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int e = blockIdx.x * 256 + threadIdx.x;      // (row, 16-byte chunk)
    if (e >= n * 16) return;
    int r = e >> 4, c = e & 15;
    int64_t row = (t0 + r) % ring_cap;
    const bf16_t *src = ring + (((int64_t)b * Hkv + h) * ring_cap + row) * kD + c * 8;
    *(u32x4 *)(out + (int64_t)b * out_sb + (int64_t)(r / unit_rows) * out_su + (int64_t)h * out_sh +
               (int64_t)(r % unit_rows) * kD + c * 8) = *(const u32x4 *)src;
}

}  // namespace

extern "C" int infllm_ingest(const infllm_ingest_args *a, void *stream) {
    INFLLM_REQUIRE(a != nullptr, "ingest: null argument block");
    INFLLM_REQUIRE(a->d_q && a->d_k && a->d_v && a->d_inv_freq, "ingest: null input pointer");
    INFLLM_REQUIRE(a->d_ring_k_raw && a->d_ring_k_rot && a->d_ring_v && a->d_ring_score && a->d_q_loc && a->d_q_glb,
                   "ingest: null output pointer");
    INFLLM_REQUIRE(a->B > 0 && a->H > 0 && a->Hkv > 0 && a->H % a->Hkv == 0, "ingest: bad head geometry B=%d H=%d Hkv=%d",
                   a->B, a->H, a->Hkv);
    INFLLM_REQUIRE(a->n >= 0 && a->pos0 >= 0, "ingest: negative length or position");
    INFLLM_REQUIRE(a->ring_cap > 0 && a->n <= a->ring_cap, "ingest: %d new tokens do not fit a ring of %lld rows", a->n,
                   (long long)a->ring_cap);
    INFLLM_REQUIRE((a->q_sl % 8 | a->q_sh % 8 | a->q_sb % 8 | a->k_sl % 8 | a->k_sh % 8 | a->k_sb % 8 | a->v_sl % 8 |
                    a->v_sh % 8 | a->v_sb % 8) == 0,
                   "ingest: strides must be multiples of 8 elements (16-byte rows)");
    if (a->n == 0) return 0;
    dim3 grid((a->n + kPosPerBlock - 1) / kPosPerBlock, a->B);
    hipLaunchKernelGGL(ingest_kernel, grid, dim3(256), 0, (hipStream_t)stream, *a);
    INFLLM_CHECK_LAUNCH("ingest");
    return 0;
}

extern "C" int infllm_block_mean(const void *d_q_glb, int32_t B, int32_t H, int32_t n, int32_t exc, float *d_qbar,
                                 void *stream) {
    INFLLM_REQUIRE(d_q_glb && d_qbar, "block_mean: null pointer");
    INFLLM_REQUIRE(B > 0 && H > 0 && n > 0 && exc > 0, "block_mean: bad sizes B=%d H=%d n=%d exc=%d", B, H, n, exc);
    int n_blocks = (n + exc - 1) / exc;
    hipLaunchKernelGGL(block_mean_kernel, dim3(n_blocks, H, B), dim3(kMeanThreads), 0, (hipStream_t)stream,
                       (const bf16_t *)d_q_glb, H, n, exc, d_qbar, n_blocks);
    INFLLM_CHECK_LAUNCH("block_mean");
    return 0;
}

extern "C" int infllm_gather_rows(const void *d_ring, int64_t ring_cap, int32_t B, int32_t Hkv, int64_t t0, int32_t n,
                                  int32_t unit_rows, void *d_out, int64_t out_sb, int64_t out_su, int64_t out_sh,
                                  void *stream) {
    INFLLM_REQUIRE(d_ring && d_out, "gather_rows: null pointer");
    INFLLM_REQUIRE(B > 0 && Hkv > 0 && ring_cap > 0 && t0 >= 0 && n >= 0 && n <= ring_cap,
                   "gather_rows: bad sizes B=%d Hkv=%d cap=%lld t0=%lld n=%d", B, Hkv, (long long)ring_cap, (long long)t0, n);
    INFLLM_REQUIRE(unit_rows > 0, "gather_rows: unit_rows must be positive");
    INFLLM_REQUIRE((out_sb % 8 | out_su % 8 | out_sh % 8) == 0, "gather_rows: output strides must be multiples of 8");
    if (n == 0) return 0;
    hipLaunchKernelGGL(gather_rows_kernel, dim3((n * 16 + 255) / 256, Hkv, B), dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t *)d_ring, ring_cap, Hkv, t0, n, unit_rows, (bf16_t *)d_out, out_sb, out_su, out_sh);
    INFLLM_CHECK_LAUNCH("gather_rows");
    return 0;
}
