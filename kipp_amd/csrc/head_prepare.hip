// Queries, keys and values of an attention mixer made ready from its input product, for mixers with any of: biases,
// a per-head RMS norm with or without a weight, a rotation over part of the head, a factor on the queries that grows
// with the position, keys and values of different widths, values mixed with those of an earlier layer; and the write
// into the paged cache.
//
// `proj` is the float32 product [tokens][stride] (or slabs [parts][tokens][stride] that are added in order) with
// the columns [n_q heads of d | n_kv key heads of d | n_kv value heads of dv | ...].  One wave takes one head of
// one token:
//     bias    u += bias[column]                               (bias over the q | k | v columns, or none)
//     norm    u *= rsqrt(mean(u^2) + eps) [* w]               (queries and keys; mode 0 none, 1 plain, 2 weighted)
//     rotate  queries and keys: number i < r / 2 of a head turns with number i + r / 2 by the token's angle i
//             (`angles` [tokens][r]: r / 2 cosines, then r / 2 sines; none: no rotation)
//     factor  queries at position p times 1 + coef * ln(floor((p + 1) / every) + 1)     (every 0: none)
//     head    queries of head h times q_head_scale[h]                                    (or none)
//     values  every value head over its root mean square, rsqrt(mean(u^2) + v_norm_eps)  (v_norm_eps < 0: none)
//     mix     `v_first_out` [tokens][n_kv dv] receives the values as they are here; with `v_first_in` (another layer's,
//             of the same tokens) the value becomes (1 - lambda) v + lambda v_first, lambda = *v_lambda
//     write   q to q_out [tokens][n_q d]; the key and value of position p to page table[p / page], slot p % page;
//             caches [page][kv head][slot][d] and [page][kv head][slot][v_row], v_row >= dv (the rest of a row is zeros)
// All arithmetic is float32.
#include "common.h"
#include <math.h>

#define HEADS_PER_BLOCK 4
#define MAX_D 256

template <typename TO, typename TC>
__global__ void head_prepare_kernel(
    const float* __restrict__ proj, int parts, size_t part_stride, int stride, const float* __restrict__ bias,
    TO* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks, int norm_mode, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, float eps, float temp_coef, int temp_every,
    int n_q, int n_kv, int d, int dv, int page, int write_kv, const float* __restrict__ q_head_scale, float v_norm_eps,
    const float* __restrict__ angles, int rotary_dim, const float* __restrict__ v_first_in, float* __restrict__ v_first_out,
    const float* __restrict__ v_lambda, int v_row) {
    const int wave = threadIdx.x / KIPP_WAVE;
    const int lane = threadIdx.x & (KIPP_WAVE - 1);
    const int t = blockIdx.y;
    const int slot = blockIdx.x * HEADS_PER_BLOCK + wave;
    const int n_slots = write_kv ? n_q + 2 * n_kv : n_q;
    if (slot >= n_slots) return;    // no barrier below: a wave is on its own
    const int kind = slot < n_q ? 0 : (slot < n_q + n_kv ? 1 : 2);
    const int head = kind == 0 ? slot : (kind == 1 ? slot - n_q : slot - n_q - n_kv);
    const int width = kind == 2 ? dv : d;
    const int column = kind == 0 ? head * d : (kind == 1 ? n_q * d + head * d : (n_q + n_kv) * d + head * dv);
    const float* src = proj + (size_t)t * stride + column;
    const int pos = positions[t];

    float vals[MAX_D / KIPP_WAVE];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
        const int e = lane + c * KIPP_WAVE;
        float v = 0.0f;
        if (e < width) {
            for (int p = 0; p < parts; ++p) v += src[p * part_stride + e];
            if (bias != nullptr) v += bias[column + e];
        }
        vals[c] = v;
        ss = fmaf(v, v, ss);
    }
    if (kind != 2 && norm_mode != 0) {
        ss = wave_sum(ss);
        float scale = 1.0f / sqrtf(ss / (float)d + eps);
        if (kind == 0 && temp_every > 0)
            scale *= 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
        const float* w = norm_mode == 2 ? (kind == 0 ? q_norm_w : k_norm_w) : nullptr;
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
            const int e = lane + c * KIPP_WAVE;
            if (e < d) vals[c] = vals[c] * scale * (w != nullptr ? w[e] : 1.0f);
        }
    } else if (kind == 0 && temp_every > 0) {
        const float factor = 1.0f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.0f);
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) vals[c] *= factor;
    }
    if (kind != 2 && angles != nullptr) {
        // a number's partner lies in another lane (and maybe another register): every lane takes part in every move
        const int half = rotary_dim / 2;
        float turned[MAX_D / KIPP_WAVE];
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
            const int e = lane + c * KIPP_WAVE;
            const bool in = e < rotary_dim, low = e < half;
            const int pe = in ? (low ? e + half : e - half) : e;
            float partner = 0.0f;
#pragma unroll
            for (int c2 = 0; c2 < MAX_D / KIPP_WAVE; ++c2) {
                const float got = __shfl(vals[c2], pe & (KIPP_WAVE - 1), KIPP_WAVE);
                if ((pe / KIPP_WAVE) == c2) partner = got;
            }
            const int i = low ? e : e - half;
            const float cs = in ? angles[(size_t)t * rotary_dim + i] : 1.0f;
            const float sn = in ? angles[(size_t)t * rotary_dim + half + i] : 0.0f;
            turned[c] = !in ? vals[c] : (low ? rotate_lo(vals[c], partner, cs, sn) : rotate_hi(partner, vals[c], cs, sn));
        }
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) vals[c] = turned[c];
    }
    if (kind == 0 && q_head_scale != nullptr) {
        const float factor = q_head_scale[head];
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) vals[c] *= factor;
    }
    if (kind == 2 && v_norm_eps >= 0.0f) {
        const float scale = 1.0f / sqrtf(wave_sum(ss) / (float)dv + v_norm_eps);
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) vals[c] *= scale;
    }
    if (kind == 2 && (v_first_in != nullptr || v_first_out != nullptr)) {
        const size_t at = (size_t)t * n_kv * dv + (size_t)head * dv;
        const float lam = v_first_in != nullptr ? v_lambda[0] : 0.0f;
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
            const int e = lane + c * KIPP_WAVE;
            if (e < dv) {
                if (v_first_out != nullptr) v_first_out[at + e] = vals[c];
                if (v_first_in != nullptr) vals[c] = (1.0f - lam) * vals[c] + lam * v_first_in[at + e];
            }
        }
    }
    if (kind == 0) {
        TO* dst = q_out + ((size_t)t * n_q + head) * d;
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
            const int e = lane + c * KIPP_WAVE;
            if (e < d) store_f(dst, e, vals[c]);
        }
    } else {
        const int seq = seq_of_token[t];
        const int page_id = block_table[(size_t)seq * max_blocks + pos / page];
        // a value's row in the cache may be wider than the value (v_row >= dv): the rest is written as zeros
        const int row = kind == 1 ? d : v_row;
        TC* dst = (kind == 1 ? k_cache : v_cache) + (((size_t)page_id * n_kv + head) * page + pos % page) * row;
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
            const int e = lane + c * KIPP_WAVE;
            if (e < row) store_f(dst, e, e < width ? vals[c] : 0.0f);
        }
    }
}

extern "C" int kipp_head_prepare_rotated(
    const float* proj, int parts, int stride, const float* bias, void* q_out, int q_dtype, void* k_cache, void* v_cache,
    int cache_dtype, const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
    int norm_mode, const float* q_norm_w, const float* k_norm_w, float eps, float temp_coef, int temp_every,
    int n_tokens, int n_q, int n_kv, int d, int dv, int page, int write_kv, const float* q_head_scale, float v_norm_eps,
    const float* angles, int rotary_dim, const float* v_first_in, float* v_first_out, const float* v_lambda, int v_row,
    hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (v_row < dv || v_row > MAX_D) return -1;
    if (angles != nullptr && (rotary_dim <= 0 || rotary_dim % 2 || rotary_dim > d)) return -1;
    if (v_first_in != nullptr && (v_lambda == nullptr || v_first_in == v_first_out)) return -1;
    if (d <= 0 || d > MAX_D || dv <= 0 || dv > MAX_D || n_q <= 0 || n_kv <= 0 || page <= 0) return -1;
    if (stride < n_q * d + (write_kv ? n_kv * (d + dv) : 0) || norm_mode < 0 || norm_mode > 2 || temp_every < 0) return -1;
    if (norm_mode == 2 && (q_norm_w == nullptr || k_norm_w == nullptr)) return -1;
    const int n_slots = write_kv ? n_q + 2 * n_kv : n_q;
    dim3 grid((n_slots + HEADS_PER_BLOCK - 1) / HEADS_PER_BLOCK, n_tokens), block(HEADS_PER_BLOCK * KIPP_WAVE);
    const size_t part_stride = (size_t)n_tokens * stride;
#define KIPP_HP(TO, TC)                                                                                              \
    hipLaunchKernelGGL((head_prepare_kernel<TO, TC>), grid, block, 0, stream, proj, parts, part_stride, stride, bias, \
                       (TO*)q_out, (TC*)k_cache, (TC*)v_cache, positions, seq_of_token, block_table, max_blocks,      \
                       norm_mode, q_norm_w, k_norm_w, eps, temp_coef, temp_every, n_q, n_kv, d, dv, page, write_kv,     \
                       q_head_scale, v_norm_eps, angles, rotary_dim, v_first_in, v_first_out, v_lambda, v_row)
    if (q_dtype == KIPP_F32 && cache_dtype == KIPP_F32) KIPP_HP(float, float);
    else if (q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16) KIPP_HP(bf16_t, bf16_t);
    else return -2;
#undef KIPP_HP
    return KIPP_LAUNCH_CHECK();
}

extern "C" int kipp_head_prepare_scaled(
    const float* proj, int parts, int stride, const float* bias, void* q_out, int q_dtype, void* k_cache, void* v_cache,
    int cache_dtype, const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
    int norm_mode, const float* q_norm_w, const float* k_norm_w, float eps, float temp_coef, int temp_every,
    int n_tokens, int n_q, int n_kv, int d, int dv, int page, int write_kv, const float* q_head_scale, float v_norm_eps,
    hipStream_t stream) {
    return kipp_head_prepare_rotated(proj, parts, stride, bias, q_out, q_dtype, k_cache, v_cache, cache_dtype, positions, seq_of_token,
                                     block_table, max_blocks, norm_mode, q_norm_w, k_norm_w, eps, temp_coef, temp_every, n_tokens, n_q,
                                     n_kv, d, dv, page, write_kv, q_head_scale, v_norm_eps, nullptr, 0, nullptr, nullptr, nullptr, dv, stream);
}

extern "C" int kipp_head_prepare(
    const float* proj, int parts, int stride, const float* bias, void* q_out, int q_dtype, void* k_cache, void* v_cache,
    int cache_dtype, const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
    int norm_mode, const float* q_norm_w, const float* k_norm_w, float eps, float temp_coef, int temp_every,
    int n_tokens, int n_q, int n_kv, int d, int dv, int page, int write_kv, hipStream_t stream) {
    return kipp_head_prepare_scaled(proj, parts, stride, bias, q_out, q_dtype, k_cache, v_cache, cache_dtype, positions, seq_of_token,
                                    block_table, max_blocks, norm_mode, q_norm_w, k_norm_w, eps, temp_coef, temp_every, n_tokens, n_q,
                                    n_kv, d, dv, page, write_kv, nullptr, -1.0f, stream);
}
