// Recurrent mixers whose memory is a matrix S [d, dv] a head, carried from token to token in float32 in the
// request's slot: linear attention with a fixed decay a head, and the gated delta rule.
//
//     decay   S <- a_h S + k v^T;                               o = S^T q      (q, k, v = silu of the projections)
//     delta   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q      (q, k, v, beta, g made ready by `prepare`)
//
// `scan`: a workgroup takes (entry, head, a run of columns of S) and walks the entry's tokens in order.  A column of S is
// shared by L lanes side by side in a wave (L a power of two, 8 or 16 rows a lane, row r with lane r % L), so the sums over
// rows end in moves between the lanes of a wave and the walk has no barrier of its own; tokens come in chunks through
// LDS.  What is computed for a token depends on the state and the token alone, never on where a chunk or a portion
// begins: prompt portions and single tokens give the same bits.  State in the slot: S as [head][column][row].
//
// `prepare` (delta rule): the short causal convolutions over q | k | v with their silu, the unit norm of every q and k head,
// beta and g, from the input product and the slot's last taps - 1 inputs; `conv_keep` then writes the slot's new last
// inputs.  `finish`: a root mean square over a span of columns, a weight, a gate.
#include "common.h"
#include <math.h>

#define SCAN_THREADS 256
#define MAX_TAPS 16

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// sum over the L lanes that share a column (they are neighbours in the wave); every one of them gets the same bits
__device__ __forceinline__ float column_sum(float v, int lanes) {
    for (int off = 1; off < lanes; off <<= 1) v += __shfl_xor(v, off, KIPP_WAVE);
    return v;
}

// MODE 0: fixed decay, inputs through silu.  MODE 1: delta rule, inputs as they are.
template <int MODE, int R>
__global__ void __launch_bounds__(SCAN_THREADS)
matrix_scan_kernel(const float* __restrict__ src, int stride, int q_at, int k_at, int v_at, int beta_at, int g_at,
                   const float* __restrict__ decays, float* __restrict__ state, size_t state_stride,
                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ slots,
                   float* __restrict__ o_raw, int heads, int qk_rep, int d, int dv, int lanes, int chunk) {
    extern __shared__ float lds[];
    const int cols = SCAN_THREADS / lanes;
    float* k_s = lds;                       // [chunk][d]
    float* q_s = k_s + (size_t)chunk * d;   // [chunk][d]
    float* v_s = q_s + (size_t)chunk * d;   // [chunk][cols]
    float* s_s = v_s + (size_t)chunk * cols;  // [chunk][2]: beta, g
    const int entry = blockIdx.z, head = blockIdx.y;
    const int col0 = blockIdx.x * cols;
    const int sub = threadIdx.x % lanes;
    const int col = col0 + threadIdx.x / lanes;
    const bool live = col < dv;
    const int qk_head = head / qk_rep;
    const int first = q_start[entry], n = q_len[entry];
    float* S_col = state + (size_t)slots[entry] * state_stride + ((size_t)head * dv + (live ? col : 0)) * d;

    float S[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int r = sub + i * lanes;
        S[i] = (live && r < d) ? S_col[r] : 0.0f;
    }
    const float decay = MODE == 0 ? decays[head] : 0.0f;

    for (int t0 = 0; t0 < n; t0 += chunk) {
        const int m = min(chunk, n - t0);
        __syncthreads();
        for (int i = threadIdx.x; i < m * d; i += SCAN_THREADS) {
            const int tt = i / d, r = i - tt * d;
            const float* row = src + (size_t)(first + t0 + tt) * stride;
            const float kv = row[k_at + qk_head * d + r], qv = row[q_at + qk_head * d + r];
            k_s[tt * d + r] = MODE == 0 ? silu_f(kv) : kv;
            q_s[tt * d + r] = MODE == 0 ? silu_f(qv) : qv;
        }
        for (int i = threadIdx.x; i < m * cols; i += SCAN_THREADS) {
            const int tt = i / cols, c = i - tt * cols;
            float vv = 0.0f;
            if (col0 + c < dv) {
                vv = src[(size_t)(first + t0 + tt) * stride + v_at + head * dv + col0 + c];
                if (MODE == 0) vv = silu_f(vv);
            }
            v_s[tt * cols + c] = vv;
        }
        if (MODE == 1)
            for (int i = threadIdx.x; i < m; i += SCAN_THREADS) {
                const float* row = src + (size_t)(first + t0 + i) * stride;
                s_s[2 * i] = row[beta_at + head];
                s_s[2 * i + 1] = row[g_at + head];
            }
        __syncthreads();
        for (int tt = 0; tt < m; ++tt) {
            const float* kt = k_s + tt * d;
            const float* qt = q_s + tt * d;
            const float vv = v_s[tt * cols + threadIdx.x / lanes];
            float acc = 0.0f;
            if (MODE == 0) {
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    const int r = sub + i * lanes;
                    if (r < d) {
                        S[i] = fmaf(decay, S[i], kt[r] * vv);
                        acc = fmaf(S[i], qt[r], acc);
                    }
                }
            } else {
                const float beta = s_s[2 * tt], g = s_s[2 * tt + 1];
                float read = 0.0f;
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    const int r = sub + i * lanes;
                    if (r < d) {
                        S[i] *= g;
                        read = fmaf(S[i], kt[r], read);
                    }
                }
                const float u = beta * (vv - column_sum(read, lanes));
#pragma unroll
                for (int i = 0; i < R; ++i) {
                    const int r = sub + i * lanes;
                    if (r < d) {
                        S[i] = fmaf(kt[r], u, S[i]);
                        acc = fmaf(S[i], qt[r], acc);
                    }
                }
            }
            acc = column_sum(acc, lanes);
            if (live && sub == 0) o_raw[(size_t)(first + t0 + tt) * heads * dv + head * dv + col] = acc;
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int r = sub + i * lanes;
            if (r < d) S_col[r] = S[i];
        }
    }
}

// Lanes a column and tokens a chunk for key size d; false if d is out of range.
static bool scan_shape(int d, int* lanes, int* rows, int* chunk) {
    if (d <= 0 || d > 1024) return false;
    *rows = d <= 512 ? 8 : 16;
    int l = 1;
    while (l * *rows < d) l <<= 1;
    *lanes = l;
    int c = 4096 / d;
    *chunk = c < 1 ? 1 : (c > 16 ? 16 : c);
    return true;
}

template <int MODE>
static int launch_scan(const float* src, int stride, int q_at, int k_at, int v_at, int beta_at, int g_at, const float* decays,
                       float* state, size_t state_stride, const int32_t* q_start, const int32_t* q_len, const int32_t* slots,
                       float* o_raw, int entries, int heads, int qk_rep, int d, int dv, hipStream_t stream) {
    int lanes, rows, chunk;
    if (!scan_shape(d, &lanes, &rows, &chunk) || heads <= 0 || dv <= 0 || qk_rep <= 0 || heads % qk_rep) return -1;
    if (state_stride < (size_t)heads * d * dv) return -1;
    const int cols = SCAN_THREADS / lanes;
    dim3 grid((dv + cols - 1) / cols, heads, entries), block(SCAN_THREADS);
    const size_t lds = ((size_t)2 * chunk * d + (size_t)chunk * cols + 2 * chunk) * sizeof(float);
    if (rows == 8)
        hipLaunchKernelGGL((matrix_scan_kernel<MODE, 8>), grid, block, lds, stream, src, stride, q_at, k_at, v_at, beta_at, g_at, decays,
                           state, state_stride, q_start, q_len, slots, o_raw, heads, qk_rep, d, dv, lanes, chunk);
    else
        hipLaunchKernelGGL((matrix_scan_kernel<MODE, 16>), grid, block, lds, stream, src, stride, q_at, k_at, v_at, beta_at, g_at, decays,
                           state, state_stride, q_start, q_len, slots, o_raw, heads, qk_rep, d, dv, lanes, chunk);
    return KIPP_LAUNCH_CHECK();
}

// proj: float32 [tokens][stride], columns q [heads d] | k [heads d] | v [heads dv] | ... before their silu.
extern "C" int kipp_decay_scan(const float* proj, int stride, const float* decays, float* state, size_t state_stride,
                               const int32_t* q_start, const int32_t* q_len, const int32_t* slots, float* o_raw, int entries,
                               int heads, int d, int dv, hipStream_t stream) {
    if (entries <= 0) return 0;
    if (stride < 2 * heads * d + heads * dv) return -1;
    return launch_scan<0>(proj, stride, 0, heads * d, 2 * heads * d, 0, 0, decays, state, state_stride, q_start, q_len, slots, o_raw,
                          entries, heads, 1, d, dv, stream);
}

// prep: float32 [tokens][stride], columns q [kv_heads d] | k [kv_heads d] | v [heads dv] | beta [heads] | g [heads], ready.
extern "C" int kipp_delta_scan(const float* prep, int stride, float* state, size_t state_stride, const int32_t* q_start,
                               const int32_t* q_len, const int32_t* slots, float* o_raw, int entries, int heads, int kv_heads,
                               int d, int dv, hipStream_t stream) {
    if (entries <= 0) return 0;
    if (kv_heads <= 0 || heads % kv_heads || stride < 2 * kv_heads * d + heads * dv + 2 * heads) return -1;
    const int c = 2 * kv_heads * d + heads * dv;
    return launch_scan<1>(prep, stride, 0, kv_heads * d, 2 * kv_heads * d, c, c + heads, nullptr, state, state_stride, q_start, q_len,
                          slots, o_raw, entries, heads, heads / kv_heads, d, dv, stream);
}

// One workgroup a token.  conv_w [channels][taps]; kept [slot][taps - 1][channels] at `kept_at` floats into the slot.
__global__ void __launch_bounds__(SCAN_THREADS)
delta_prepare_kernel(const float* __restrict__ proj, int stride, const float* __restrict__ conv_w, int taps,
                     const float* __restrict__ a_log, const float* __restrict__ dt_bias, const float* __restrict__ state,
                     size_t state_stride, size_t kept_at, const int32_t* __restrict__ seq_of_token,
                     const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots, float* __restrict__ prep,
                     int prep_stride, int heads, int kv_heads, int d, int dv, int beta_col, int a_col, float unit_eps) {
    const int t = blockIdx.x;
    const int entry = seq_of_token[t];
    const int first = q_start[entry];
    const int channels = 2 * kv_heads * d + heads * dv;
    const float* kept = state + (size_t)slots[entry] * state_stride + kept_at;
    float* dst = prep + (size_t)t * prep_stride;
    for (int c = threadIdx.x; c < channels; c += SCAN_THREADS) {
        float y = 0.0f;
        for (int j = 0; j < taps; ++j) {
            const int at = t - (taps - 1) + j;      // the row of the input `taps - 1 - j` tokens back
            const float in = at >= first ? proj[(size_t)at * stride + c] : kept[(size_t)(taps - 1 + (at - first)) * channels + c];
            y = fmaf(conv_w[(size_t)c * taps + j], in, y);
        }
        dst[c] = silu_f(y);
    }
    for (int h = threadIdx.x; h < heads; h += SCAN_THREADS) {
        const float* row = proj + (size_t)t * stride;
        dst[channels + h] = sigmoid_f(row[beta_col + h]);
        dst[channels + heads + h] = expf(-expf(a_log[h]) * softplus_f(row[a_col + h] + dt_bias[h]));
    }
    __syncthreads();
    // every q and k head over the root of its sum of squares; q also over the root of d
    const int wave = threadIdx.x / KIPP_WAVE, lane = threadIdx.x & (KIPP_WAVE - 1);
    for (int hh = wave; hh < 2 * kv_heads; hh += SCAN_THREADS / KIPP_WAVE) {
        float* head = dst + (size_t)hh * d;
        float ss = 0.0f;
        for (int e = lane; e < d; e += KIPP_WAVE) ss = fmaf(head[e], head[e], ss);
        ss = wave_sum(ss);
        float scale = 1.0f / sqrtf(ss + unit_eps);
        if (hh < kv_heads) scale *= 1.0f / sqrtf((float)d);
        for (int e = lane; e < d; e += KIPP_WAVE) head[e] *= scale;
    }
}

// The slot's new last inputs: new[i] = the input at place n - (taps - 1) + i of the portion (from the old ones where that is before it).
__global__ void conv_keep_kernel(const float* __restrict__ proj, int stride, int taps, float* __restrict__ state, size_t state_stride,
                                 size_t kept_at, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                 const int32_t* __restrict__ slots, int channels) {
    const int entry = blockIdx.y;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= channels) return;
    const int first = q_start[entry], n = q_len[entry];
    float* kept = state + (size_t)slots[entry] * state_stride + kept_at;
    float vals[MAX_TAPS];
#pragma unroll
    for (int i = 0; i < MAX_TAPS - 1; ++i) {
        if (i < taps - 1) {
            const int p = n - (taps - 1) + i;
            vals[i] = p >= 0 ? proj[(size_t)(first + p) * stride + c] : kept[(size_t)(taps - 1 + p) * channels + c];
        }
    }
#pragma unroll
    for (int i = 0; i < MAX_TAPS - 1; ++i)
        if (i < taps - 1) kept[(size_t)i * channels + c] = vals[i];
}

extern "C" int kipp_delta_prepare(const float* proj, int stride, const float* conv_w, int taps, const float* a_log, const float* dt_bias,
                                  float* state, size_t state_stride, size_t kept_at, const int32_t* seq_of_token, const int32_t* q_start,
                                  const int32_t* q_len, const int32_t* slots, float* prep, int prep_stride, int tokens, int entries,
                                  int heads, int kv_heads, int d, int dv, int beta_col, int a_col, float unit_eps, hipStream_t stream) {
    if (tokens <= 0) return 0;
    const int channels = 2 * kv_heads * d + heads * dv;
    if (taps < 1 || taps > MAX_TAPS || heads <= 0 || kv_heads <= 0 || d <= 0 || dv <= 0) return -1;
    if (stride < channels || prep_stride < channels + 2 * heads || state_stride < kept_at + (size_t)(taps - 1) * channels) return -1;
    hipLaunchKernelGGL(delta_prepare_kernel, dim3(tokens), dim3(SCAN_THREADS), 0, stream, proj, stride, conv_w, taps, a_log, dt_bias,
                       (const float*)state, state_stride, kept_at, seq_of_token, q_start, slots, prep, prep_stride, heads, kv_heads, d, dv,
                       beta_col, a_col, unit_eps);
    if (taps > 1)
        hipLaunchKernelGGL(conv_keep_kernel, dim3((channels + 255) / 256, entries), dim3(256), 0, stream, proj, stride, taps, state,
                           state_stride, kept_at, q_start, q_len, slots, channels);
    return KIPP_LAUNCH_CHECK();
}

// out[t][c] = o[t][c] * rsqrt(mean over c's span of o^2 + eps) * w[c % w_len] * gate(gates[t][gate_at + c]); gate 0 sigmoid, 1 silu.
template <typename TO>
__global__ void __launch_bounds__(SCAN_THREADS)
scan_finish_kernel(const float* __restrict__ o_raw, const float* __restrict__ gates, int gate_stride, int gate_at,
                   const float* __restrict__ w, int w_len, float eps, int gate_kind, TO* __restrict__ out, int width, int span) {
    __shared__ float scratch[16];
    const size_t t = blockIdx.y;
    const int c0 = blockIdx.x * span;
    const float* src = o_raw + t * width + c0;
    float ss = 0.0f;
    for (int e = threadIdx.x; e < span; e += SCAN_THREADS) ss = fmaf(src[e], src[e], ss);
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)span + eps);
    const float* gate = gates + t * gate_stride + gate_at + c0;
    for (int e = threadIdx.x; e < span; e += SCAN_THREADS) {
        const float z = gate[e];
        const float gv = gate_kind == 0 ? sigmoid_f(z) : silu_f(z);
        store_f(out, t * width + c0 + e, src[e] * inv * w[(c0 + e) % w_len] * gv);
    }
}

extern "C" int kipp_scan_finish(const float* o_raw, const float* gates, int gate_stride, int gate_at, const float* w, int w_len, float eps,
                                int gate_kind, void* out, int out_dtype, int tokens, int width, int span, hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (width <= 0 || span <= 0 || width % span || w_len <= 0 || gate_stride < gate_at + width || gate_kind < 0 || gate_kind > 1) return -1;
    dim3 grid(width / span, tokens), block(SCAN_THREADS);
    if (out_dtype == KIPP_F32)
        hipLaunchKernelGGL((scan_finish_kernel<float>), grid, block, 0, stream, o_raw, gates, gate_stride, gate_at, w, w_len, eps, gate_kind,
                           (float*)out, width, span);
    else if (out_dtype == KIPP_BF16)
        hipLaunchKernelGGL((scan_finish_kernel<bf16_t>), grid, block, 0, stream, o_raw, gates, gate_stride, gate_at, w, w_len, eps, gate_kind,
                           (bf16_t*)out, width, span);
    else
        return -2;
    return KIPP_LAUNCH_CHECK();
}
