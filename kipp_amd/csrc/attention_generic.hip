// Causal grouped-query attention over the paged cache for any mix of query
// tokens (prompt portions and single decoded tokens alike), any key size up
// to 1,024, values of their own width (`dv`; the value cache may be the key
// cache itself, a value then being the first dv numbers of its key's row of
// `v_row` numbers) and any storage type.  One wave per (token, query head); this is the
// float32 path's kernel and the fallback of sizes the MFMA kernels refuse.
//
// For query position p of a sequence the keys are s in [max(0, p-window+1), p]
// (window 0: from 0; with `chunk` c > 0 from p - p % c, the start of p's chunk of c positions counted from 0), score = (q . k_s) * scale (with `softcap` c > 0: c tanh(score / c)), softmax with the maximum
// subtracted (with `sink` one more term e^0 joins the denominator: a key of score 0 without a value),
// out = sum p_s v_s  (/root/reference/src/kipp.c:2882-2922).  Keys are
// taken in tiles of 64 aligned to absolute key index, so the sequence of
// operations for one query depends on its own position only, never on what
// else is in the batch.
#include "common.h"
#include <math.h>

#define HEADS_PER_BLOCK 4
#define MAX_D 1024

// q . k over d numbers, added in index order whatever the width of the loads (16 bytes where the row allows).
__device__ __forceinline__ float dot_row(const float* q, const float* k, int d) {
    float dot = 0.0f;
    int e = 0;
    if ((((uintptr_t)k) & 15) == 0)
#pragma unroll 4
        for (; e + 4 <= d; e += 4) {
            const float4 v = *reinterpret_cast<const float4*>(k + e);
            dot += q[e] * v.x;
            dot += q[e + 1] * v.y;
            dot += q[e + 2] * v.z;
            dot += q[e + 3] * v.w;
        }
    for (; e < d; ++e) dot += q[e] * k[e];
    return dot;
}

__device__ __forceinline__ float dot_row(const float* q, const bf16_t* k, int d) {
    float dot = 0.0f;
    int e = 0;
    if ((((uintptr_t)k) & 15) == 0)
#pragma unroll 4
        for (; e + 8 <= d; e += 8) {
            const uint4 v = *reinterpret_cast<const uint4*>(k + e);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                dot += q[e + 2 * i] * __uint_as_float(w[i] << 16);
                dot += q[e + 2 * i + 1] * __uint_as_float(w[i] & 0xffff0000u);
            }
        }
    for (; e < d; ++e) dot += q[e] * bf16_to_f32(k[e]);
    return dot;
}

template <typename TQ, typename TC, typename TO>
__global__ void paged_attention_generic_kernel(
    const TQ* __restrict__ q, const TC* __restrict__ k_cache, const TC* __restrict__ v_cache, TO* __restrict__ out,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks,
    int n_q, int n_kv, int d, int dv, int v_row, int page, float scale, int window, float softcap, int chunk, int sink) {
    __shared__ float q_s[HEADS_PER_BLOCK][MAX_D];
    __shared__ float p_s[HEADS_PER_BLOCK][KIPP_WAVE];
    __shared__ unsigned long long off_s[HEADS_PER_BLOCK][KIPP_WAVE];
    const int wave = threadIdx.x / KIPP_WAVE;
    const int lane = threadIdx.x & (KIPP_WAVE - 1);
    const int t = blockIdx.y;
    int head = blockIdx.x * HEADS_PER_BLOCK + wave;
    const bool active = head < n_q;
    if (!active) head = n_q - 1;
    const int g = head / (n_q / n_kv);
    const int pos = positions[t];
    const int seq = seq_of_token[t];
    const int32_t* table = block_table + (size_t)seq * max_blocks;
    const int lo = chunk > 0 ? pos - pos % chunk : (window > 0 ? max(0, pos - window + 1) : 0);

    const TQ* q_row = q + ((size_t)t * n_q + head) * d;
    for (int e = lane; e < d; e += KIPP_WAVE) q_s[wave][e] = load_f(q_row, e);
    __syncthreads();

    float m = -INFINITY, l = 0.0f;
    float acc[MAX_D / KIPP_WAVE];
#pragma unroll
    for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) acc[c] = 0.0f;

    for (int s0 = (lo / KIPP_WAVE) * KIPP_WAVE; s0 <= pos; s0 += KIPP_WAVE) {
        const int s = s0 + lane;
        const bool valid = s >= lo && s <= pos;
        float score = -INFINITY;
        unsigned long long off = 0;
        if (valid) {
            const int page_id = table[s / page];
            off = ((unsigned long long)page_id * n_kv + g) * page + s % page;
            const TC* k_row = k_cache + off * d;
            score = dot_row(q_s[wave], k_row, d) * scale;
            if (softcap > 0.0f) score = softcap * tanhf(score / softcap);
        }
        const float m_new = fmaxf(m, wave_max(score));
        const float alpha = expf(m - m_new);
        const float p = valid ? expf(score - m_new) : 0.0f;
        l = l * alpha + wave_sum(p);
        m = m_new;
        __syncthreads();
        p_s[wave][lane] = p;
        off_s[wave][lane] = off;
        __syncthreads();
        const int j_lo = max(0, lo - s0);
        const int j_hi = min(KIPP_WAVE, pos - s0 + 1);
        // every column's sum still runs over the keys in order; the keys are the outer loop so that a key's loads (one a
        // column of this lane) and those of the next keys are on their way together
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) acc[c] *= alpha;
#pragma unroll 4
        for (int j = j_lo; j < j_hi; ++j) {
            const float pj = p_s[wave][j];
            const TC* v_at = v_cache + off_s[wave][j] * v_row;
#pragma unroll
            for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
                const int e = lane + c * KIPP_WAVE;
                if (e < dv) acc[c] += pj * load_f(v_at, e);
            }
        }
    }
    if (!active) return;
    TO* o_row = out + ((size_t)t * n_q + head) * dv;
    if (sink) l += expf(-m);        // the term of score 0 (m is finite: a position sees itself)
    const float inv = 1.0f / l;
#pragma unroll
    for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
        const int e = lane + c * KIPP_WAVE;
        if (e < dv) store_f(o_row, e, acc[c] * inv);
    }
}

// Values of width dv in rows of v_row numbers (v_row = dv for a value cache of its own).
extern "C" int kipp_paged_attention_generic_masked(
    const void* q, int q_dtype, const void* k_cache, const void* v_cache, int cache_dtype, void* out, int out_dtype,
    const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
    int n_tokens, int n_q, int n_kv, int d, int dv, int v_row, int page, float scale, int window, float softcap,
    int chunk, int sink, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (chunk < 0 || (chunk > 0 && window > 0)) return -1;
    if (d > MAX_D || d <= 0 || dv > MAX_D || dv <= 0 || v_row < dv || n_kv <= 0 || n_q % n_kv) return -1;
    dim3 grid((n_q + HEADS_PER_BLOCK - 1) / HEADS_PER_BLOCK, n_tokens), block(HEADS_PER_BLOCK * KIPP_WAVE);
#define KIPP_PA(TQ, TC, TO)                                                                                    \
    hipLaunchKernelGGL((paged_attention_generic_kernel<TQ, TC, TO>), grid, block, 0, stream, (const TQ*)q,     \
                       (const TC*)k_cache, (const TC*)v_cache, (TO*)out, positions, seq_of_token, block_table, \
                       max_blocks, n_q, n_kv, d, dv, v_row, page, scale, window, softcap, chunk, sink)
    if (q_dtype == KIPP_F32 && cache_dtype == KIPP_F32 && out_dtype == KIPP_F32) KIPP_PA(float, float, float);
    else if (q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16 && out_dtype == KIPP_BF16) KIPP_PA(bf16_t, bf16_t, bf16_t);
    else return -2;
#undef KIPP_PA
    return KIPP_LAUNCH_CHECK();
}

extern "C" int kipp_paged_attention_generic_capped(
    const void* q, int q_dtype, const void* k_cache, const void* v_cache, int cache_dtype, void* out, int out_dtype,
    const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
    int n_tokens, int n_q, int n_kv, int d, int dv, int v_row, int page, float scale, int window, float softcap,
    hipStream_t stream) {
    return kipp_paged_attention_generic_masked(q, q_dtype, k_cache, v_cache, cache_dtype, out, out_dtype, positions, seq_of_token,
                                               block_table, max_blocks, n_tokens, n_q, n_kv, d, dv, v_row, page, scale, window, softcap,
                                               0, 0, stream);
}

extern "C" int kipp_paged_attention_generic_v(
    const void* q, int q_dtype, const void* k_cache, const void* v_cache, int cache_dtype, void* out, int out_dtype,
    const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
    int n_tokens, int n_q, int n_kv, int d, int dv, int v_row, int page, float scale, int window, hipStream_t stream) {
    return kipp_paged_attention_generic_capped(q, q_dtype, k_cache, v_cache, cache_dtype, out, out_dtype, positions, seq_of_token,
                                               block_table, max_blocks, n_tokens, n_q, n_kv, d, dv, v_row, page, scale, window, 0.0f, stream);
}

extern "C" int kipp_paged_attention_generic(
    const void* q, int q_dtype, const void* k_cache, const void* v_cache, int cache_dtype, void* out, int out_dtype,
    const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
    int n_tokens, int n_q, int n_kv, int d, int page, float scale, int window, hipStream_t stream) {
    if (d > 256) return -1;
    return kipp_paged_attention_generic_v(q, q_dtype, k_cache, v_cache, cache_dtype, out, out_dtype, positions, seq_of_token,
                                          block_table, max_blocks, n_tokens, n_q, n_kv, d, d, d, page, scale, window, stream);
}
