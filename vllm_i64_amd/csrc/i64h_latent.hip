// Latent attention of libi64hip_dense.so (include/i64h_dense.h): every token caches ONE row per layer - a normalised low-rank
// latent and a rotated key part shared by all heads.  The per-head key and value projections of the latent are never
// materialised: the caller carries the query through the key projection (q' = W_uk^T q, a batched Linear) and the attention
// output back through the value projection (a batched Linear over the summed latents), so a head's score is
// q'_latent . latent_j + q_rot . key_rot_j and all heads read the same cached rows.
//   latent_prep_kernel     : RMS norm of the latent, rotation of the shared key part and of every head's rotated query part,
//                            cache write - one workgroup per token
//   latent_attn_row_kernel : one wave per (token, head): 64 keys at a time, one key per lane for the scores (fp32 dot over the
//                            cached row), online softmax over the wave, weighted row sum with the columns spread over the lanes
#include "i64h_common.h"
#include "i64h_dense.h"

__device__ __forceinline__ float lt_load(const void* cache, int dtype, int64_t idx) {
    return dtype == 0 ? ((const float*)cache)[idx] : __uint_as_float((uint32_t)((const uint16_t*)cache)[idx] << 16);
}
__device__ __forceinline__ void lt_store(void* cache, int dtype, int64_t idx, float v) {
    if (dtype == 0) {
        ((float*)cache)[idx] = v;
    } else {
        uint32_t u = __float_as_uint(v);
        u = (u & 0x7fffffffu) > 0x7f800000u ? ((u >> 16) | 0x40u) : ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
        ((uint16_t*)cache)[idx] = (uint16_t)u;
    }
}

__global__ __launch_bounds__(256) void latent_prep_kernel(const i64h_latent_prep_args p) {
    __shared__ float red[4];
    const int tid = threadIdx.x;
    const int64_t t = blockIdx.x;
    const int pos = p.positions[t], slot = p.slot_ids[t];
    const int r = p.kv_rank, rd = p.rot_dim, D = r + rd, half = p.rot_dims / 2;
    const int64_t row = (int64_t)p.block_table[(int64_t)slot * p.max_blocks_per_seq + pos / p.block_size] * p.block_size + pos % p.block_size;
    const float* pr = p.P + t * p.ldp;
    const float* dkv = pr + p.dkv_off;
    float s = 0.0f;
    for (int c = tid; c < r; c += 256) s += dkv[c] * dkv[c];
    s = wave_sum(s);
    if ((tid & 63) == 0) red[tid >> 6] = s;
    __syncthreads();
    const float den = sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)r + p.eps);
    for (int c = tid; c < r; c += 256) lt_store(p.cache, p.cache_dtype, row * D + c, dkv[c] / den * p.c_norm_w[c]);
    const float fpos = (float)pos;
    // the shared key part and every head's query part: index 0 is the key, 1 + h the heads
    for (int e = tid; e < (p.heads + 1) * rd; e += 256) {
        const int who = e / rd, c = e % rd;
        const float* src = who == 0 ? dkv + r : pr + p.q_off + (int64_t)(who - 1) * (p.dim + rd) + p.dim;
        float v;
        if (c < 2 * half) {
            float sn, cs;
            sincosf(fpos * p.inv_freq[c >> 1], &sn, &cs);
            const float a = src[c & ~1], b = src[c | 1];
            v = (c & 1) ? (b * cs + a * sn) : (a * cs - b * sn);
        } else {
            v = src[c];
        }
        if (who == 0) lt_store(p.cache, p.cache_dtype, row * D + r + c, v);
        else p.Q[(t * p.heads + (who - 1)) * D + r + c] = v;
    }
}

#define LT_MAXC 16  // latent columns per lane: kv_rank <= 64 * LT_MAXC

__global__ __launch_bounds__(256) void latent_attn_row_kernel(const i64h_latent_attn_args p) {
    extern __shared__ float lds[];  // [4][D] scaled queries, [4][64] weights, [4][64] cache rows
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int64_t t = blockIdx.x;
    const int r = p.kv_rank, D = r + p.rot_dim;
    float* sq = lds + w * D;
    float* sp = lds + 4 * D + w * 64;
    int* srow = (int*)(lds + 4 * D + 256) + w * 64;
    const int h_raw = blockIdx.y * 4 + w;
    const bool active = h_raw < p.heads;
    const int h = active ? h_raw : p.heads - 1;
    const int pos = p.positions[t], slot = p.slot_ids[t];
    const float* q = p.Q + (t * p.heads + h) * D;
    for (int d = lane; d < D; d += 64) sq[d] = q[d] * p.scale;
    __syncthreads();
    const int j0 = p.window > 0 ? max(0, pos - p.window + 1) : 0;
    const int32_t* bt = p.block_table + (int64_t)slot * p.max_blocks_per_seq;
    float m = -INFINITY, l = 0.0f, acc[LT_MAXC];
#pragma unroll
    for (int i = 0; i < LT_MAXC; ++i) acc[i] = 0.0f;
    for (int jb = j0; jb <= pos; jb += 64) {
        const int j = jb + lane;
        const bool valid = j <= pos;
        const int jj = valid ? j : pos;
        const int64_t rj = (int64_t)bt[jj / p.block_size] * p.block_size + jj % p.block_size;
        float s = 0.0f;
        if (p.cache_dtype == 0) {
            const float* kr = (const float*)p.cache + rj * D;
            if ((D & 3) == 0) {
                for (int d = 0; d < D; d += 4) {
                    const float4 kv = *(const float4*)(kr + d);
                    s += sq[d] * kv.x; s += sq[d + 1] * kv.y; s += sq[d + 2] * kv.z; s += sq[d + 3] * kv.w;
                }
            } else {
                for (int d = 0; d < D; ++d) s += sq[d] * kr[d];
            }
        } else {
            const uint16_t* kr = (const uint16_t*)p.cache + rj * D;
            if ((D & 7) == 0) {
                for (int d = 0; d < D; d += 8) {
                    const uint4 kv = *(const uint4*)(kr + d);
                    const uint32_t kw[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s += sq[d + 2 * i] * __uint_as_float(kw[i] << 16);
                        s += sq[d + 2 * i + 1] * __uint_as_float(kw[i] & 0xffff0000u);
                    }
                }
            } else {
                for (int d = 0; d < D; ++d) s += sq[d] * __uint_as_float((uint32_t)kr[d] << 16);
            }
        }
        s = valid ? s : -INFINITY;
        const float mn = fmaxf(m, wave_max(s));
        const float alpha = expf(m - mn);
        const float pj = valid ? expf(s - mn) : 0.0f;
        l = l * alpha + wave_sum(pj);
        m = mn;
        __syncthreads();  // the previous block's weights have been read by every lane
        sp[lane] = pj;
        srow[lane] = (int)rj;
        __syncthreads();
        const int cnt = min(64, pos - jb + 1);
#pragma unroll
        for (int i = 0; i < LT_MAXC; ++i) acc[i] *= alpha;
        for (int k = 0; k < cnt; ++k) {
            const float pk = sp[k];
            const int64_t base = (int64_t)srow[k] * D;
#pragma unroll
            for (int i = 0; i < LT_MAXC; ++i) {
                const int c = lane + 64 * i;
                if (c < r) acc[i] += pk * lt_load(p.cache, p.cache_dtype, base + c);
            }
        }
    }
    if (active) {
        float* o = p.out + (t * p.heads + h) * r;
#pragma unroll
        for (int i = 0; i < LT_MAXC; ++i) {
            const int c = lane + 64 * i;
            if (c < r) o[c] = acc[i] / l;
        }
    }
}

extern "C" {

int i64h_latent_prep(const i64h_latent_prep_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "latent_prep: no descriptor");
    const i64h_latent_prep_args& d = *dp;
    I64H_CHECK_ARG(d.n >= 0 && d.heads > 0 && d.dim > 0 && d.rot_dim >= 0 && d.kv_rank > 0 && d.block_size > 0, "latent_prep: bad sizes");
    I64H_CHECK_ARG(d.rot_dims >= 0 && d.rot_dims <= d.rot_dim && d.rot_dims % 2 == 0, "latent_prep: %d rotated dimensions of %d", d.rot_dims, d.rot_dim);
    I64H_CHECK_ARG(d.cache_dtype == 0 || d.cache_dtype == 2, "latent_prep: cache dtype %d", d.cache_dtype);
    I64H_CHECK_ARG(d.P && d.c_norm_w && d.positions && d.slot_ids && d.block_table && d.cache && d.Q && (d.inv_freq || d.rot_dims == 0), "latent_prep: null operand");
    if (d.n == 0) return 0;
    hipLaunchKernelGGL(latent_prep_kernel, dim3((unsigned)d.n), dim3(256), 0, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

int i64h_latent_attn(const i64h_latent_attn_args* dp, void* stream) {
    I64H_CHECK_ARG(dp != nullptr, "latent_attn: no descriptor");
    const i64h_latent_attn_args& d = *dp;
    I64H_CHECK_ARG(d.n >= 0 && d.heads > 0 && d.kv_rank > 0 && d.rot_dim >= 0 && d.block_size > 0, "latent_attn: bad sizes");
    I64H_CHECK_ARG(d.kv_rank <= 64 * LT_MAXC, "latent_attn: kv_rank %d above %d", d.kv_rank, 64 * LT_MAXC);
    I64H_CHECK_ARG(d.cache_dtype == 0 || d.cache_dtype == 2, "latent_attn: cache dtype %d", d.cache_dtype);
    I64H_CHECK_ARG(d.Q && d.cache && d.block_table && d.slot_ids && d.positions && d.out, "latent_attn: null operand");
    if (d.n == 0) return 0;
    const int D = d.kv_rank + d.rot_dim;
    const size_t lds = (size_t)(4 * D + 512) * 4;
    I64H_CHECK_ARG(lds <= 64 * 1024, "latent_attn: cached rows of %d values do not fit", D);
    hipLaunchKernelGGL(latent_attn_row_kernel, dim3((unsigned)d.n, (unsigned)((d.heads + 3) / 4)), dim3(256), lds, (hipStream_t)stream, d);
    I64H_CHECK_LAUNCH();
    return 0;
}

}  // extern "C"
