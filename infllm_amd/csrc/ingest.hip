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

// rotate 8 pairs (lo[i], hi[i]) by (c[i], s[i]); fp32 math, one rounding to bf16.  `raw` (optional) receives the 16
// rotated values before that rounding: lo pairs first, then hi pairs.
__device__ __forceinline__ Rot8 rotate8(u32x4 xlo, u32x4 xhi, const float2 *cs, float *raw = nullptr) {
    Rot8 r;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        float a0 = bf16_bits_to_f32(xlo[w] & 0xffffu), a1 = bf16_bits_to_f32(xlo[w] >> 16);
        float b0 = bf16_bits_to_f32(xhi[w] & 0xffffu), b1 = bf16_bits_to_f32(xhi[w] >> 16);
        float2 c0 = cs[2 * w], c1 = cs[2 * w + 1];
        // x*cos + rotate_half(x)*sin, rotate_half = (-hi, lo)
        const float l0 = a0 * c0.x - b0 * c0.y, l1 = a1 * c1.x - b1 * c1.y;
        const float h0 = b0 * c0.x + a0 * c0.y, h1 = b1 * c1.x + a1 * c1.y;
        r.lo[w] = pack_bf16x2(l0, l1);
        r.hi[w] = pack_bf16x2(h0, h1);
        if (raw) {
            raw[2 * w] = l0, raw[2 * w + 1] = l1;
            raw[8 + 2 * w] = h0, raw[8 + 2 * w + 1] = h1;
        }
    }
    return r;
}

// grid = (position tiles of 16, batch rows, kv heads): a workgroup rotates the query heads of one
// kv-head group plus that group's key head, copies its value head, and leaves the sum of its
// rotated-to-one-position queries over its positions in d_qpart (for the block's mean query; summed
// before the rounding to bf16, so the mean query carries no rounding of its own).
//
// Angles.  cos / sin of (position x frequency) are needed for 16 positions x 64 frequencies per workgroup.
// Only the workgroup's FIRST position and the step of one position are evaluated (fp64 sincos, one call
// per thread for 128 threads); the other 15 positions follow by the angle-addition recurrence in fp64,
// whose error after 15 steps is a few 1e-16 - far below the fp32 value the rotation consumes.  The rows
// the workgroup will rotate are requested from memory BEFORE that arithmetic, so the two overlap.
__global__ __launch_bounds__(256) void ingest_kernel(infllm_ingest_args a) {
    __shared__ float2 cs_pos[kPosPerBlock][kHalf];
    __shared__ float2 cs_glb[kHalf];
    __shared__ double2 cs_step[kHalf];                // (cos, sin) of one position's step per frequency
    __shared__ float red[4][kPosPerBlock][kD];        // q_glb of 4 heads x 16 positions, for the partial sums
    const int tid = threadIdx.x;
    const int b = blockIdx.y, g = blockIdx.z;
    const int G = a.H / a.Hkv;
    const int p0 = blockIdx.x * kPosPerBlock;
    const int np = min(kPosPerBlock, a.n - p0);

    const bf16_t *q = (const bf16_t *)a.d_q + (int64_t)b * a.q_sb;
    const bf16_t *k = (const bf16_t *)a.d_k + (int64_t)b * a.k_sb + (int64_t)g * a.k_sh;
    const bf16_t *v = (const bf16_t *)a.d_v + (int64_t)b * a.v_sb + (int64_t)g * a.v_sh;
    bf16_t *q_loc = (bf16_t *)a.d_q_loc + (int64_t)b * a.H * a.n * kD;
    bf16_t *q_glb = (bf16_t *)a.d_q_glb + (int64_t)b * a.H * a.n * kD;
    const int64_t ring_g = ((int64_t)b * a.Hkv + g) * a.ring_cap * kD;
    bf16_t *rk_raw = (bf16_t *)a.d_ring_k_raw + ring_g;
    bf16_t *rk_rot = (bf16_t *)a.d_ring_k_rot + ring_g;
    bf16_t *rv = (bf16_t *)a.d_ring_v + ring_g;
    const int n_tiles = (a.n + kPosPerBlock - 1) / kPosPerBlock;

    // ---- requests first: the first group of (up to) 4 query heads, the key head, the value head
    constexpr int kQItems = 2;                        // 4 heads x 16 positions x 8 chunk pairs = 512 items over 256 threads
    u32x4 q_lo[kQItems], q_hi[kQItems], k_lo, k_hi, v_row;
    const int nh0 = min(4, G);
#pragma unroll
    for (int i = 0; i < kQItems; ++i) {
        const int e = tid + i * 256;
        if (e < nh0 * np * 8) {
            const int c = e & 7, p = (e >> 3) % np, hl = (e >> 3) / np;
            const bf16_t *src = q + (int64_t)(g * G + hl) * a.q_sh + (int64_t)(p0 + p) * a.q_sl;
            q_lo[i] = *(const u32x4 *)(src + c * 8);
            q_hi[i] = *(const u32x4 *)(src + kHalf + c * 8);
        }
    }
    if (tid < np * 8) {
        const bf16_t *src = k + (int64_t)(p0 + (tid >> 3)) * a.k_sl;
        k_lo = *(const u32x4 *)(src + (tid & 7) * 8);
        k_hi = *(const u32x4 *)(src + kHalf + (tid & 7) * 8);
    }
    if (tid < np * 16) v_row = *(const u32x4 *)(v + (int64_t)(p0 + (tid >> 4)) * a.v_sl + (tid & 15) * 8);

    // ---- angles
    if (tid < kHalf) {
        const double w = a.distance_scale * (double)a.d_inv_freq[tid];
        double s, c;
        sincos((double)(a.pos0 + p0) * w, &s, &c);
        cs_pos[0][tid] = make_float2((float)c, (float)s);
        cs_step[tid] = make_double2(c, s);            // parked here until the step values arrive
    } else if (tid < 2 * kHalf) {
        const int f = tid - kHalf;
        double s, c;
        sincos((double)a.glb_pos * a.distance_scale * (double)a.d_inv_freq[f], &s, &c);
        cs_glb[f] = make_float2((float)c, (float)s);
    }
    double2 step = make_double2(1.0, 0.0);
    if (tid < kHalf) {
        double s, c;
        sincos(a.distance_scale * (double)a.d_inv_freq[tid], &s, &c);
        step = make_double2(c, s);
        double2 cur = cs_step[tid];
        for (int p = 1; p < kPosPerBlock; ++p) {      // (cos, sin)(x + w) from (cos, sin)(x)
            const double c2 = cur.x * step.x - cur.y * step.y, s2 = cur.y * step.x + cur.x * step.y;
            cur = make_double2(c2, s2);
            cs_pos[p][tid] = make_float2((float)c2, (float)s2);
        }
    }
    __syncthreads();

    // query heads of the group, 4 at a time: 8 threads per (head, position) row
    for (int hg0 = 0; hg0 < G; hg0 += 4) {
        const int nh = min(4, G - hg0);
#pragma unroll
        for (int i = 0; i < kQItems; ++i) {
            const int e = tid + i * 256;
            if (e >= nh * np * 8) continue;
            const int c = e & 7, p = (e >> 3) % np, hl = (e >> 3) / np;
            const int h = g * G + hg0 + hl;
            u32x4 lo = q_lo[i], hi = q_hi[i];
            if (hg0 > 0) {
                const bf16_t *src = q + (int64_t)h * a.q_sh + (int64_t)(p0 + p) * a.q_sl;
                lo = *(const u32x4 *)(src + c * 8), hi = *(const u32x4 *)(src + kHalf + c * 8);
            }
            int64_t o = ((int64_t)h * a.n + p0 + p) * kD;
            Rot8 r = rotate8(lo, hi, &cs_pos[p][c * 8]);
            *(u32x4 *)(q_loc + o + c * 8) = r.lo;
            *(u32x4 *)(q_loc + o + kHalf + c * 8) = r.hi;
            float raw[16];
            r = rotate8(lo, hi, &cs_glb[c * 8], raw);
            *(u32x4 *)(q_glb + o + c * 8) = r.lo;
            *(u32x4 *)(q_glb + o + kHalf + c * 8) = r.hi;
            if (a.d_qpart) {
                *(f32x4 *)&red[hl][p][c * 8] = f32x4{raw[0], raw[1], raw[2], raw[3]};
                *(f32x4 *)&red[hl][p][c * 8 + 4] = f32x4{raw[4], raw[5], raw[6], raw[7]};
                *(f32x4 *)&red[hl][p][kHalf + c * 8] = f32x4{raw[8], raw[9], raw[10], raw[11]};
                *(f32x4 *)&red[hl][p][kHalf + c * 8 + 4] = f32x4{raw[12], raw[13], raw[14], raw[15]};
            }
        }
        if (a.d_qpart) {
            __syncthreads();
            for (int e = tid; e < nh * kD; e += 256) {
                const int d = e % kD, hl = e / kD;
                float s = 0.f;
                for (int p = 0; p < np; ++p) s += red[hl][p][d];          // fixed order
                a.d_qpart[(((int64_t)b * n_tiles + blockIdx.x) * a.H + g * G + hg0 + hl) * kD + d] = s;
            }
            __syncthreads();
        }
    }
    // key head: raw copy + rotated copy into the rings
    if (tid < np * 8) {
        const int c = tid & 7, p = tid >> 3;
        const int64_t o = ((a.pos0 + p0 + p) % a.ring_cap) * kD;
        *(u32x4 *)(rk_raw + o + c * 8) = k_lo;
        *(u32x4 *)(rk_raw + o + kHalf + c * 8) = k_hi;
        Rot8 r = rotate8(k_lo, k_hi, &cs_pos[p][c * 8]);
        *(u32x4 *)(rk_rot + o + c * 8) = r.lo;
        *(u32x4 *)(rk_rot + o + kHalf + c * 8) = r.hi;
    }
    // value head: plain copy, 16 threads per row
    if (tid < np * 16) *(u32x4 *)(rv + ((a.pos0 + p0 + (tid >> 4)) % a.ring_cap) * kD + (tid & 15) * 8) = v_row;
    // the score track of a new token starts at zero (context_manager.py:733-741)
    for (int e = tid; e < G * np; e += 256) {
        const int p = e % np, h = g * G + e / np;
        a.d_ring_score[((int64_t)b * a.H + h) * a.ring_cap + (a.pos0 + p0 + p) % a.ring_cap] = 0.f;
    }
}

// out[b, c] = scale * sum_p parts[b, p, c], p ascending.  A workgroup owns 64 columns; its 4 waves fetch different
// partials, so that 32 of them are one round trip to memory (a chain of dependent loads is all latency, and that
// latency multiplies while a unit fetch keeps the memory fabric busy); the sum itself runs in the fixed order.
// With blockIdx.z > 0 the partials are those of several execution blocks ingested by one launch: block z owns
// blk_parts consecutive partials (the last block what is left of n_parts) and exc positions (the last what is left of
// n_rows), its mean goes to out[z, b, :] and its scale is 1 / (its positions).
__global__ __launch_bounds__(256) void reduce_partials_kernel(const float *parts, int n_parts, int C, float scale,
                                                              float *out, int blk_parts, int n_rows, int exc) {
    __shared__ float stage[32][64];
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int c = blockIdx.x * 64 + lane, b = blockIdx.y, z = blockIdx.z;
    const float *src = parts + ((int64_t)b * n_parts + (int64_t)z * blk_parts) * C + c;
    out += (int64_t)z * gridDim.y * C;
    if (blk_parts < n_parts) {
        n_parts = min(blk_parts, n_parts - z * blk_parts);
        scale = 1.f / (float)min(exc, n_rows - z * exc);
    }
    float s = 0.f;
    for (int p0 = 0; p0 < n_parts; p0 += 32) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int p = p0 + grp + 4 * i;
            v[i] = (c < C && p < n_parts) ? src[(int64_t)p * C] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) stage[grp + 4 * i][lane] = v[i];
        __syncthreads();
        if (grp == 0) {
            const int m = min(32, n_parts - p0);
            for (int p = 0; p < m; ++p) s += stage[p][lane];
        }
        __syncthreads();
    }
    if (grp == 0 && c < C) out[(int64_t)b * C + c] = s * scale;
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

// Mean global query of every execution block of a chunk, straight from the un-rotated input rows: the global
// query is rotated by ONE angle (rope.py:93-104), and a rotation is linear, so the mean is taken first (fp32)
// and rotated once.  One workgroup per (block, head, batch row).
__global__ __launch_bounds__(kMeanThreads) void chunk_qbar_kernel(const bf16_t *q, int64_t q_sb, int64_t q_sh, int64_t q_sl,
                                                                 int H, int n, int exc, const float *inv_freq,
                                                                 double distance_scale, int64_t glb_pos, float *qbar,
                                                                 int n_blocks) {
    __shared__ float2 part[kMeanThreads / 64][64];
    __shared__ float mean[kD];
    const int blk = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int r0 = blk * exc, r1 = min(r0 + exc, n);
    const bf16_t *src = q + (int64_t)b * q_sb + (int64_t)h * q_sh;
    float s0 = 0.f, s1 = 0.f;
    for (int r = r0 + grp; r < r1; r += kMeanThreads / 64) {
        uint32_t w = *(const uint32_t *)(src + (int64_t)r * q_sl + lane * 2);
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
        const float inv = 1.f / (float)(r1 - r0);
        mean[lane * 2] = t0 * inv;
        mean[lane * 2 + 1] = t1 * inv;
    }
    __syncthreads();
    if (threadIdx.x < kD / 2) {
        const int f = threadIdx.x;
        double sn, cs;
        sincos((double)glb_pos * distance_scale * (double)inv_freq[f], &sn, &cs);
        const float c = (float)cs, sgn = (float)sn, lo = mean[f], hi = mean[f + kD / 2];
        float *dst = qbar + (((int64_t)b * n_blocks + blk) * H + h) * kD;
        dst[f] = lo * c - hi * sgn;
        dst[f + kD / 2] = hi * c + lo * sgn;
    }
}

// RoPE of plain rows (rope.py:27-47, 93-104): out[b,h,r,:] = x[b,h,r,:] rotated by the angle of position
// pos0 + r * pos_step (pos_step 0: every row by the same angle).  One wave per row, a lane owns the pair
// (d, d + 64); the angle is formed in fp64 like in the stream prologue.
__global__ __launch_bounds__(256) void rope_rows_kernel(const bf16_t *x, int64_t sb, int64_t sh, int64_t sl, int H, int L,
                                                        int64_t pos0, int pos_step, const float *inv_freq,
                                                        double distance_scale, bf16_t *out) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6), h = blockIdx.y, b = blockIdx.z;
    if (r >= L) return;
    const bf16_t *src = x + (int64_t)b * sb + (int64_t)h * sh + (int64_t)r * sl;
    bf16_t *dst = out + (((int64_t)b * H + h) * L + r) * kD;
    double sn, cs;
    sincos((double)(pos0 + (int64_t)r * pos_step) * distance_scale * (double)inv_freq[lane], &sn, &cs);
    const float c = (float)cs, s = (float)sn;
    const float lo = bf16_bits_to_f32(((const uint16_t *)src)[lane]), hi = bf16_bits_to_f32(((const uint16_t *)src)[lane + kD / 2]);
    ((uint16_t *)dst)[lane] = (uint16_t)(pack_bf16x2(lo * c - hi * s, 0.f) & 0xffffu);
    ((uint16_t *)dst)[lane + kD / 2] = (uint16_t)(pack_bf16x2(hi * c + lo * s, 0.f) & 0xffffu);
}

// grid.z = B, or 2*B to gather from a second ring (ring2 -> out2, same geometry) in the same launch
__global__ __launch_bounds__(256) void gather_rows_kernel(const bf16_t *ring, int64_t ring_cap, int Hkv, int64_t t0,
                                                          int n, int unit_rows, bf16_t *out, int64_t out_sb,
                                                          int64_t out_su, int64_t out_sh, int B, const bf16_t *ring2, bf16_t *out2) {
    const int b = blockIdx.z % B, h = blockIdx.y;
    if ((int)blockIdx.z >= B) {
        ring = ring2;
        out = out2;
    }
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
    dim3 grid((a->n + kPosPerBlock - 1) / kPosPerBlock, a->B, a->Hkv);
    hipLaunchKernelGGL(ingest_kernel, grid, dim3(256), 0, (hipStream_t)stream, *a);
    INFLLM_CHECK_LAUNCH("ingest");
    return 0;
}

extern "C" int infllm_reduce_partials(const float *d_parts, int32_t B, int32_t n_parts, int32_t C, float scale, float *d_out,
                                      void *stream) {
    INFLLM_REQUIRE(d_parts && d_out, "reduce_partials: null pointer");
    INFLLM_REQUIRE(B > 0 && n_parts > 0 && C > 0, "reduce_partials: bad sizes B=%d n_parts=%d C=%d", B, n_parts, C);
    hipLaunchKernelGGL(reduce_partials_kernel, dim3((C + 63) / 64, B), dim3(256), 0, (hipStream_t)stream, d_parts, n_parts, C,
                       scale, d_out, n_parts, 0, 0);
    INFLLM_CHECK_LAUNCH("reduce_partials");
    return 0;
}

// library-internal: the mean rotated query of every execution block of one ingest launch over n positions (blocks of
// exc, a multiple of the ingest tile; the last may be shorter): d_parts [B, ceil(n / tile), C] -> d_out [blocks, B, C]
int infllm_reduce_partials_blocks(const float *d_parts, int32_t B, int32_t n, int32_t exc, int32_t C, float *d_out, void *stream) {
    INFLLM_REQUIRE(d_parts && d_out, "reduce_partials_blocks: null pointer");
    INFLLM_REQUIRE(B > 0 && n > 0 && C > 0 && exc > 0 && exc % kPosPerBlock == 0, "reduce_partials_blocks: bad sizes B=%d n=%d exc=%d C=%d", B, n, exc, C);
    const int n_parts = (n + kPosPerBlock - 1) / kPosPerBlock, n_blocks = (n + exc - 1) / exc;
    hipLaunchKernelGGL(reduce_partials_kernel, dim3((C + 63) / 64, B, n_blocks), dim3(256), 0, (hipStream_t)stream, d_parts, n_parts, C,
                       1.f / (float)n, d_out, n_blocks > 1 ? exc / kPosPerBlock : n_parts, n, exc);
    INFLLM_CHECK_LAUNCH("reduce_partials_blocks");
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

extern "C" int infllm_chunk_qbar(const void *d_q, int64_t q_sb, int64_t q_sh, int64_t q_sl, int32_t B, int32_t H, int32_t n,
                                 int32_t exc, const float *d_inv_freq, double distance_scale, int64_t glb_pos, float *d_qbar,
                                 void *stream) {
    INFLLM_REQUIRE(d_q && d_inv_freq && d_qbar, "chunk_qbar: null pointer");
    INFLLM_REQUIRE(B > 0 && H > 0 && n > 0 && exc > 0, "chunk_qbar: bad sizes B=%d H=%d n=%d exc=%d", B, H, n, exc);
    INFLLM_REQUIRE(q_sl % 2 == 0 && q_sh % 2 == 0 && q_sb % 2 == 0 && (uintptr_t)d_q % 4 == 0, "chunk_qbar: q rows must be 4-byte aligned");
    const int n_blocks = (n + exc - 1) / exc;
    hipLaunchKernelGGL(chunk_qbar_kernel, dim3(n_blocks, H, B), dim3(kMeanThreads), 0, (hipStream_t)stream, (const bf16_t *)d_q,
                       q_sb, q_sh, q_sl, H, n, exc, d_inv_freq, distance_scale, glb_pos, d_qbar, n_blocks);
    INFLLM_CHECK_LAUNCH("chunk_qbar");
    return 0;
}

extern "C" int infllm_rope_rows(const void *d_x, int64_t sb, int64_t sh, int64_t sl, int32_t B, int32_t H, int32_t L, int64_t pos0,
                                int32_t pos_step, const float *d_inv_freq, double distance_scale, void *d_out, void *stream) {
    INFLLM_REQUIRE(B >= 0 && H >= 0 && L >= 0 && pos0 >= 0 && (pos_step == 0 || pos_step == 1), "rope_rows: bad sizes B=%d H=%d L=%d", B, H, L);
    if (B == 0 || H == 0 || L == 0) return 0;
    INFLLM_REQUIRE(d_x && d_inv_freq && d_out, "rope_rows: null pointer");
    hipLaunchKernelGGL(rope_rows_kernel, dim3((L + 3) / 4, H, B), dim3(256), 0, (hipStream_t)stream, (const bf16_t *)d_x, sb, sh, sl,
                       H, L, pos0, pos_step, d_inv_freq, distance_scale, (bf16_t *)d_out);
    INFLLM_CHECK_LAUNCH("rope_rows");
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
                       (const bf16_t *)d_ring, ring_cap, Hkv, t0, n, unit_rows, (bf16_t *)d_out, out_sb, out_su, out_sh, B,
                       (const bf16_t *)nullptr, (bf16_t *)nullptr);
    INFLLM_CHECK_LAUNCH("gather_rows");
    return 0;
}

// internal: the K and the V rows of the same stream positions in one launch (same arguments as infllm_gather_rows)
int infllm_gather_rows_pair(const void *d_ring_a, void *d_out_a, const void *d_ring_b, void *d_out_b, int64_t ring_cap, int32_t B,
                            int32_t Hkv, int64_t t0, int32_t n, int32_t unit_rows, int64_t out_sb, int64_t out_su, int64_t out_sh,
                            void *stream) {
    INFLLM_REQUIRE(d_ring_a && d_out_a && d_ring_b && d_out_b, "gather_rows: null pointer");
    INFLLM_REQUIRE(B > 0 && Hkv > 0 && ring_cap > 0 && n >= 0 && n <= ring_cap && t0 >= 0 && unit_rows > 0, "gather_rows: bad sizes");
    INFLLM_REQUIRE((out_sb % 8 | out_su % 8 | out_sh % 8) == 0, "gather_rows: output strides must be multiples of 8");
    if (n == 0) return 0;
    hipLaunchKernelGGL(gather_rows_kernel, dim3((n * 16 + 255) / 256, Hkv, 2 * B), dim3(256), 0, (hipStream_t)stream,
                       (const bf16_t *)d_ring_a, ring_cap, Hkv, t0, n, unit_rows, (bf16_t *)d_out_a, out_sb, out_su, out_sh, B,
                       (const bf16_t *)d_ring_b, (bf16_t *)d_out_b);
    INFLLM_CHECK_LAUNCH("gather_rows");
    return 0;
}
