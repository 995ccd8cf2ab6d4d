// Recurrent mixers whose memory is a matrix S [d, dv] a head, carried from token to token in float32 in the
// request's slot: linear attention with a fixed decay a head, the gated delta rule, and the selective state space
// recurrence in its dual form (a decay a token and head).
//
//     decay   S <- a_h S + k v^T;                               o = S^T q      (q, k, v = silu of the projections)
//     delta   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q      (q, k, v, beta, g made ready by `prepare`)
//     gated   S <- g S + k v^T;                                 o = S^T q      (q, k, v, g made ready by `ssd_prepare`:
//             k = B, q = C, v = dt x, g = exp(-exp(A_h) dt), dt = softplus(. + dt_bias))
//
// `scan`: a workgroup takes (entry, head, a run of columns of S) and walks the entry's tokens in order.  A column of S is
// shared by L lanes side by side in a wave (L a power of two, 8 or 16 rows in a run a lane), so the sums over rows end in
// data-parallel moves between the lanes of a wave and the walk has no barrier of its own; tokens come in chunks through
// LDS, four at a time, so that the sums of four tokens' outputs run side by side.  What is computed for a token depends on the state and the token alone, never on where a chunk or a portion
// begins: prompt portions and single tokens give the same bits.  State in the slot: S as [head][column][row].
//
// `prepare` (delta rule): the short causal convolutions over q | k | v with their silu, the unit norm of every q and k head,
// beta and g, from the input product and the slot's last taps - 1 inputs; `conv_keep` then writes the slot's new last
// inputs.  `finish`: a root mean square over a span of columns, a weight, a gate.
#include "common.h"
#include "lane_sums.h"
#include <math.h>

#define SCAN_THREADS 256
#define MAX_TAPS 16

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// One token of the walk for a lane's R rows of a column: the new rows, and the lane's share of o (summed over the
// column's lanes by the caller, so that the sums of several tokens run side by side).  The same code whether the token
// stands alone or among others: a position's bits do not depend on how the tokens were cut.
template <int MODE, int R, int LANES>
__device__ __forceinline__ float scan_token(float (&S)[R], const float* __restrict__ kt, const float* __restrict__ qt, float vv,
                                            float decay, float beta, float g) {
    float k[R], q[R];
#pragma unroll
    for (int i = 0; i < R; i += 4) {
        const float4 k4 = *(const float4*)(kt + i), q4 = *(const float4*)(qt + i);
        k[i] = k4.x; k[i + 1] = k4.y; k[i + 2] = k4.z; k[i + 3] = k4.w;
        q[i] = q4.x; q[i + 1] = q4.y; q[i + 2] = q4.z; q[i + 3] = q4.w;
    }
    float acc = 0.0f;
    if (MODE == 0 || MODE == 2) {
        const float a = MODE == 2 ? g : decay;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            S[i] = fmaf(a, S[i], k[i] * vv);
            acc = fmaf(S[i], q[i], acc);
        }
    } else {
        float read = 0.0f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            S[i] *= g;
            read = fmaf(S[i], k[i], read);
        }
        const float u = beta * (vv - column_sum<LANES>(read));
#pragma unroll
        for (int i = 0; i < R; ++i) {
            S[i] = fmaf(k[i], u, S[i]);
            acc = fmaf(S[i], q[i], acc);
        }
    }
    return acc;
}

// MODE 0: fixed decay, inputs through silu.  MODE 1: delta rule, inputs as they are.  MODE 2: a decay a token, inputs as
// they are.  A column of S is shared by LANES
// lanes side by side, lane `sub` with the R rows sub R .. sub R + R - 1 (read from LDS 16 bytes at a time; rows beyond d
// are zeros there and stay zeros in S).
template <int MODE, int R, int LANES>
__global__ void __launch_bounds__(SCAN_THREADS)
matrix_scan_kernel(const float* __restrict__ src, int stride, int q_at, int k_at, int v_at, int beta_at, int g_at,
                   const float* __restrict__ decays, float* __restrict__ state, size_t state_stride,
                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ slots,
                   float* __restrict__ o_raw, int heads, int qk_rep, int d, int dv, int chunk) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    constexpr int COLS = SCAN_THREADS / LANES;
    constexpr int DP = R * LANES;           // a key's numbers in LDS, filled up with zeros
    float* k_s = lds;                       // [chunk][DP]
    float* q_s = k_s + (size_t)chunk * DP;  // [chunk][DP]
    float* v_s = q_s + (size_t)chunk * DP;  // [chunk][COLS]
    float* s_s = v_s + (size_t)chunk * COLS;  // [chunk][2]: beta, g
    const int entry = blockIdx.z, head = blockIdx.y;
    const int col0 = blockIdx.x * COLS;
    const int sub = threadIdx.x % LANES, colw = threadIdx.x / LANES;
    const int col = col0 + colw;
    const bool live = col < dv;
    const int qk_head = head / qk_rep;
    const int first = q_start[entry], n = q_len[entry];
    float* S_col = state + (size_t)slots[entry] * state_stride + ((size_t)head * dv + (live ? col : 0)) * d;

    // a lane's rows lie together: 16 bytes at a time where every column begins at a multiple of 16 bytes
    const bool wide = (d & 3) == 0 && (state_stride & 3) == 0;
    float S[R];
#pragma unroll
    for (int i = 0; i < R; i += 4) {
        const int r = sub * R + i;
        if (wide) {
            const float4 s4 = (live && r < d) ? *(const float4*)(S_col + r) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            S[i] = s4.x; S[i + 1] = s4.y; S[i + 2] = s4.z; S[i + 3] = s4.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) S[i + j] = (live && r + j < d) ? S_col[r + j] : 0.0f;
        }
    }
    const float decay = MODE == 0 ? decays[head] : 0.0f;
    float* o_col = o_raw + (size_t)head * dv + col;
    const size_t o_stride = (size_t)heads * dv;

    for (int t0 = 0; t0 < n; t0 += chunk) {
        const int m = min(chunk, n - t0);
        __syncthreads();
        for (int i = threadIdx.x; i < m * DP; i += SCAN_THREADS) {
            const int tt = i / DP, r = i - tt * DP;
            float kv = 0.0f, qv = 0.0f;
            if (r < d) {
                const float* row = src + (size_t)(first + t0 + tt) * stride;
                kv = row[k_at + qk_head * d + r];
                qv = row[q_at + qk_head * d + r];
                if (MODE == 0) { kv = silu_f(kv); qv = silu_f(qv); }
            }
            k_s[i] = kv;
            q_s[i] = qv;
        }
        for (int i = threadIdx.x; i < m * COLS; i += SCAN_THREADS) {
            const int tt = i / COLS, c = i - tt * COLS;
            float vv = 0.0f;
            if (col0 + c < dv) {
                vv = src[(size_t)(first + t0 + tt) * stride + v_at + head * dv + col0 + c];
                if (MODE == 0) vv = silu_f(vv);
            }
            v_s[i] = vv;
        }
        if (MODE >= 1)
            for (int i = threadIdx.x; i < m; i += SCAN_THREADS) {
                const float* row = src + (size_t)(first + t0 + i) * stride;
                s_s[2 * i] = MODE == 1 ? row[beta_at + head] : 0.0f;
                s_s[2 * i + 1] = row[g_at + head];
            }
        __syncthreads();
        const float* kt = k_s + sub * R;
        const float* qt = q_s + sub * R;
        int tt = 0;
        for (; tt + 4 <= m; tt += 4) {
            float acc[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                acc[u] = scan_token<MODE, R, LANES>(S, kt + (tt + u) * DP, qt + (tt + u) * DP, v_s[(tt + u) * COLS + colw], decay,
                                                    MODE >= 1 ? s_s[2 * (tt + u)] : 0.0f, MODE >= 1 ? s_s[2 * (tt + u) + 1] : 0.0f);
#pragma unroll
            for (int u = 0; u < 4; ++u) acc[u] = column_sum<LANES>(acc[u]);
            if (live && sub == 0) {
#pragma unroll
                for (int u = 0; u < 4; ++u) o_col[(size_t)(first + t0 + tt + u) * o_stride] = acc[u];
            }
        }
        for (; tt < m; ++tt) {
            float acc = scan_token<MODE, R, LANES>(S, kt + tt * DP, qt + tt * DP, v_s[tt * COLS + colw], decay,
                                                   MODE >= 1 ? s_s[2 * tt] : 0.0f, MODE >= 1 ? s_s[2 * tt + 1] : 0.0f);
            acc = column_sum<LANES>(acc);
            if (live && sub == 0) o_col[(size_t)(first + t0 + tt) * o_stride] = acc;
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < R; i += 4) {
            const int r = sub * R + i;
            if (wide) {
                if (r < d) *(float4*)(S_col + r) = make_float4(S[i], S[i + 1], S[i + 2], S[i + 3]);
            } else {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (r + j < d) S_col[r + j] = S[i + j];
            }
        }
    }
}

// Lanes a column, rows a lane and tokens a chunk for key size d; false if d is out of range.
static bool scan_shape(int d, int longest, int* lanes, int* rows, int* chunk) {
    if (d <= 0 || d > 1024) return false;
    *rows = d <= 512 ? 8 : 16;
    int l = 1;
    while (l * *rows < d) l <<= 1;
    *lanes = l;
    int c = 6144 / (l * *rows);      // k and q of a chunk stay under 48 KB of LDS
    *chunk = c < 1 ? 1 : (c > 32 ? 32 : c);
    // no more LDS than the longest entry fills (single tokens: a few hundred bytes, so that many workgroups share a compute unit)
    if (longest > 0 && longest < *chunk) *chunk = longest;
    return true;
}

template <int MODE>
static int launch_scan(const float* src, int stride, int q_at, int k_at, int v_at, int beta_at, int g_at, const float* decays,
                       float* state, size_t state_stride, const int32_t* q_start, const int32_t* q_len, const int32_t* slots,
                       float* o_raw, int entries, int heads, int qk_rep, int d, int dv, int longest, hipStream_t stream) {
    int lanes, rows, chunk;
    if (!scan_shape(d, longest, &lanes, &rows, &chunk) || heads <= 0 || dv <= 0 || qk_rep <= 0 || heads % qk_rep) return -1;
    if (state_stride < (size_t)heads * d * dv) return -1;
    const int cols = SCAN_THREADS / lanes;
    dim3 grid((dv + cols - 1) / cols, heads, entries), block(SCAN_THREADS);
    const size_t lds = ((size_t)2 * chunk * lanes * rows + (size_t)chunk * cols + 2 * chunk) * sizeof(float);
#define KIPP_SCAN(R, L)                                                                                                        \
    hipLaunchKernelGGL((matrix_scan_kernel<MODE, R, L>), grid, block, lds, stream, src, stride, q_at, k_at, v_at, beta_at, g_at, \
                       decays, state, state_stride, q_start, q_len, slots, o_raw, heads, qk_rep, d, dv, chunk)
    if (rows == 16) KIPP_SCAN(16, 64);
    else if (lanes == 1) KIPP_SCAN(8, 1);
    else if (lanes == 2) KIPP_SCAN(8, 2);
    else if (lanes == 4) KIPP_SCAN(8, 4);
    else if (lanes == 8) KIPP_SCAN(8, 8);
    else if (lanes == 16) KIPP_SCAN(8, 16);
    else if (lanes == 32) KIPP_SCAN(8, 32);
    else KIPP_SCAN(8, 64);
#undef KIPP_SCAN
    return KIPP_LAUNCH_CHECK();
}

// proj: float32 [tokens][stride], columns q [heads d] | k [heads d] | v [heads dv] | ... before their silu.
// `longest`: the most tokens an entry brings, if the host knows (0: it does not); it only sizes the chunks.
extern "C" int kipp_decay_scan(const float* proj, int stride, const float* decays, float* state, size_t state_stride,
                               const int32_t* q_start, const int32_t* q_len, const int32_t* slots, float* o_raw, int entries,
                               int heads, int d, int dv, int longest, hipStream_t stream) {
    if (entries <= 0) return 0;
    if (stride < 2 * heads * d + heads * dv) return -1;
    return launch_scan<0>(proj, stride, 0, heads * d, 2 * heads * d, 0, 0, decays, state, state_stride, q_start, q_len, slots, o_raw,
                          entries, heads, 1, d, dv, longest, stream);
}

// prep: float32 [tokens][stride], columns q [kv_heads d] | k [kv_heads d] | v [heads dv] | beta [heads] | g [heads], ready.
extern "C" int kipp_delta_scan(const float* prep, int stride, float* state, size_t state_stride, const int32_t* q_start,
                               const int32_t* q_len, const int32_t* slots, float* o_raw, int entries, int heads, int kv_heads,
                               int d, int dv, int longest, hipStream_t stream) {
    if (entries <= 0) return 0;
    if (kv_heads <= 0 || heads % kv_heads || stride < 2 * kv_heads * d + heads * dv + 2 * heads) return -1;
    const int c = 2 * kv_heads * d + heads * dv;
    return launch_scan<1>(prep, stride, 0, kv_heads * d, 2 * kv_heads * d, c, c + heads, nullptr, state, state_stride, q_start, q_len,
                          slots, o_raw, entries, heads, heads / kv_heads, d, dv, longest, stream);
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

// prep: float32 [tokens][stride], columns q = C [groups n] | k = B [groups n] | v = dt x [heads p] | x [heads p] | g [heads], ready.
extern "C" int kipp_gated_scan(const float* prep, int stride, float* state, size_t state_stride, const int32_t* q_start,
                               const int32_t* q_len, const int32_t* slots, float* o_raw, int entries, int heads, int groups,
                               int n, int p, int longest, hipStream_t stream) {
    if (entries <= 0) return 0;
    if (groups <= 0 || heads % groups || stride < 2 * groups * n + 2 * heads * p + heads) return -1;
    return launch_scan<2>(prep, stride, 0, groups * n, 2 * groups * n, 0, 2 * groups * n + 2 * heads * p, nullptr, state, state_stride,
                          q_start, q_len, slots, o_raw, entries, heads, heads / groups, n, p, longest, stream);
}

#define SSD_MAX_HEADS 1024

// One workgroup a token.  proj: [z: inner | x: inner | B: groups n | C: groups n | dt: heads] (inner = heads p); the
// channels x | B | C pass a causal filter (conv_w [channels][taps] with conv_b [channels], the slot's kept inputs ahead of a
// portion; kept [taps - 1][channels] at `kept_at` floats into the slot) and silu.  prep as `kipp_gated_scan` reads it.
__global__ void __launch_bounds__(SCAN_THREADS)
ssd_prepare_kernel(const float* __restrict__ proj, int stride, const float* __restrict__ conv_w, const float* __restrict__ conv_b, int taps,
                   const float* __restrict__ a_log, const float* __restrict__ dt_bias, const float* __restrict__ state,
                   size_t state_stride, size_t kept_at, const int32_t* __restrict__ seq_of_token,
                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots, float* __restrict__ prep,
                   int prep_stride, int heads, int groups, int n, int p) {
    __shared__ float dt_s[SSD_MAX_HEADS];
    const int t = blockIdx.x;
    const int entry = seq_of_token[t];
    const int first = q_start[entry];
    const int inner = heads * p, gn = groups * n;
    const int channels = inner + 2 * gn;
    const float* kept = state + (size_t)slots[entry] * state_stride + kept_at;
    const float* row = proj + (size_t)t * stride;
    float* dst = prep + (size_t)t * prep_stride;
    for (int h = threadIdx.x; h < heads; h += SCAN_THREADS) {
        const float dt = softplus_f(row[2 * inner + 2 * gn + h] + dt_bias[h]);
        dt_s[h] = dt;
        dst[2 * gn + 2 * inner + h] = expf(-expf(a_log[h]) * dt);
    }
    __syncthreads();
    for (int c = threadIdx.x; c < channels; c += SCAN_THREADS) {
        float y = conv_b[c];
        for (int j = 0; j < taps; ++j) {
            const int at = t - (taps - 1) + j;      // the row of the input `taps - 1 - j` tokens back
            const float in = at >= first ? proj[(size_t)at * stride + inner + c] : kept[(size_t)(taps - 1 + (at - first)) * channels + c];
            y = fmaf(conv_w[(size_t)c * taps + j], in, y);
        }
        y = silu_f(y);
        if (c < inner) {
            dst[2 * gn + c] = dt_s[c / p] * y;
            dst[2 * gn + inner + c] = y;
        } else if (c < inner + gn) {
            dst[gn + (c - inner)] = y;          // B: the keys
        } else {
            dst[c - inner - gn] = y;            // C: the queries
        }
    }
}

extern "C" int kipp_ssd_prepare(const float* proj, int stride, const float* conv_w, const float* conv_b, int taps, const float* a_log,
                                const float* dt_bias, float* state, size_t state_stride, size_t kept_at, const int32_t* seq_of_token,
                                const int32_t* q_start, const int32_t* q_len, const int32_t* slots, float* prep, int prep_stride,
                                int tokens, int entries, int heads, int groups, int n, int p, hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (taps < 1 || taps > MAX_TAPS || heads <= 0 || heads > SSD_MAX_HEADS || groups <= 0 || heads % groups || n <= 0 || p <= 0) return -1;
    const int inner = heads * p, channels = inner + 2 * groups * n;
    if (stride < inner + channels + heads || prep_stride < 2 * groups * n + 2 * inner + heads ||
        state_stride < kept_at + (size_t)(taps - 1) * channels) return -1;
    hipLaunchKernelGGL(ssd_prepare_kernel, dim3(tokens), dim3(SCAN_THREADS), 0, stream, proj, stride, conv_w, conv_b, taps, a_log, dt_bias,
                       (const float*)state, state_stride, kept_at, seq_of_token, q_start, slots, prep, prep_stride, heads, groups, n, p);
    if (taps > 1)
        hipLaunchKernelGGL(conv_keep_kernel, dim3((channels + 255) / 256, entries), dim3(256), 0, stream, proj + inner, stride, taps, state,
                           state_stride, kept_at, q_start, q_len, slots, channels);
    return KIPP_LAUNCH_CHECK();
}

// y[t][c] = (o[t][c] + skip[c / p] x[t][c]) * silu(z[t][c]); out = y * rsqrt(mean over c's span of y^2 + eps) * w[c]: the gate
// comes before the norm.  x at column `x_at` of prep, z at column `z_at` of proj.
template <typename TO>
__global__ void __launch_bounds__(SCAN_THREADS)
ssd_finish_kernel(const float* __restrict__ o_raw, const float* __restrict__ prep, int prep_stride, int x_at,
                  const float* __restrict__ proj, int proj_stride, int z_at, const float* __restrict__ skip, int p,
                  const float* __restrict__ w, float eps, TO* __restrict__ out, int width, int span) {
    __shared__ float scratch[16];
    const size_t t = blockIdx.y;
    const int c0 = blockIdx.x * span;
    const float* o = o_raw + t * width + c0;
    const float* x = prep + t * prep_stride + x_at + c0;
    const float* z = proj + t * proj_stride + z_at + c0;
    float ss = 0.0f;
    for (int e = threadIdx.x; e < span; e += SCAN_THREADS) {
        const float y = fmaf(skip[(c0 + e) / p], x[e], o[e]) * silu_f(z[e]);
        ss = fmaf(y, y, ss);
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)span + eps);
    for (int e = threadIdx.x; e < span; e += SCAN_THREADS) {
        const float y = fmaf(skip[(c0 + e) / p], x[e], o[e]) * silu_f(z[e]);
        store_f(out, t * width + c0 + e, y * inv * w[c0 + e]);
    }
}

extern "C" int kipp_ssd_finish(const float* o_raw, const float* prep, int prep_stride, int x_at, const float* proj, int proj_stride,
                               int z_at, const float* skip, int p, const float* w, float eps, void* out, int out_dtype, int tokens,
                               int width, int span, hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (width <= 0 || span <= 0 || width % span || p <= 0 || width % p || prep_stride < x_at + width || proj_stride < z_at + width) return -1;
    dim3 grid(width / span, tokens), block(SCAN_THREADS);
    if (out_dtype == KIPP_F32)
        hipLaunchKernelGGL((ssd_finish_kernel<float>), grid, block, 0, stream, o_raw, prep, prep_stride, x_at, proj, proj_stride, z_at, skip, p,
                           w, eps, (float*)out, width, span);
    else if (out_dtype == KIPP_BF16)
        hipLaunchKernelGGL((ssd_finish_kernel<bf16_t>), grid, block, 0, stream, o_raw, prep, prep_stride, x_at, proj, proj_stride, z_at, skip, p,
                           w, eps, (bf16_t*)out, width, span);
    else
        return -2;
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
