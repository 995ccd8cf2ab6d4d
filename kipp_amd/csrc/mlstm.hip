// The matrix memory of an mLSTM layer: the recurrence itself, for prompt portions and single tokens alike, and
// the step between it and the output projection.
//
// Per head, with a query q (already times d^(-1/2)), key k (d numbers), value v (dv numbers) and the two gate
// pre-activations zi, zf of a token:
//     li = cap * tanh((zi + bi) / cap)                   the log of the input gate
//     lf = logsigmoid(cap * tanh((zf + bf) / cap))       the log of the forget gate
//     m' = max(lf + m, li)
//     S' = exp(lf + m - m') S + exp(li - m') k v^T       (d x dv),   n' likewise with k alone
//     o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
// S, n and m live in the request's state slot as float32 [heads][dv][d] | [Z][heads][d] | [Z][heads], Z = ceil(dv / columns of a workgroup)
// (a column of S, the d numbers that meet one value, lies together):
// every workgroup of a head keeps a copy of n and m of its own (all equal), so that none reads what another has
// already written for the next step.  A slot that was just claimed holds zeros, which is the recurrence's start.
// Everything here is float32.
//
// scan    a workgroup takes (entry of the batch, head, a run of columns of S) and walks the entry's tokens in order.
//         A column is shared by 4, 16 or 64 lanes that stand side by side in a wave, each with 8 (or 16) rows of it,
//         so the sum over rows ends in a few lane exchanges and no wave waits for another inside the walk.  Every
//         lane also keeps its rows of n (the same arithmetic in every column, hence the same bits), so the
//         denominator needs no exchange between columns either.  The tokens come in chunks: while one chunk is
//         walked out of LDS, the next one's k, q, v and gate pre-activations are on their way from memory into
//         registers; when a chunk is put into LDS the first wave takes the gates of its tokens (tanh and logarithms a lane a
//         token, the running maximum in token order, the exponentials a lane a token again), so the walk itself is
//         multiply-adds, and the sums over a column's lanes are data-parallel moves inside the wave, not trips through LDS.
//         The order of a token's operations does not depend on where its chunk begins: a position's bits are the
//         same however the prompt was cut.
// finish  every head of a token divided by its root mean square, times the norm's weight, times sigmoid(gate),
//         in the type the output projection reads.
//
// `proj` is the input product, float32 [tokens][stride], with the columns
//     [q: heads d | k: heads d | v: heads dv | gate: heads dv | zi: heads | zf: heads].
#include "common.h"
#include "lane_sums.h"
#include <math.h>

#define SCAN_THREADS 256
#define SCAN_GROUP 8
#define SCAN_STAGE 4096     // most numbers of k (and of q) that a chunk of tokens stages: 16 a thread

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.0f) - log1pf(expf(-fabsf(z))); }

// ROWS rows of a column a lane (a multiple of 4), PARTS lanes a column (side by side in a wave), 256 / PARTS columns a
// workgroup.  BASE: the rows a lane has in the build for prompt portions of this key size; a build with more rows a lane
// adds them in runs of BASE and the runs pairwise, which is the order in which the lanes of that build add theirs.  `unit`: columns that share one copy of n and m in the state (a workgroup's columns are a multiple of it).
// LDS: chunk * (2 ROWS PARTS + columns + 4) + 4 floats; rows of k and q are padded with zeros to ROWS * PARTS numbers.
template <int ROWS, int PARTS, int BASE>
__global__ void __launch_bounds__(SCAN_THREADS) mlstm_scan_kernel(
    const float* __restrict__ proj, int stride, const float* __restrict__ bias_i, const float* __restrict__ bias_f, float cap,
    float* __restrict__ state, size_t state_stride, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
    const int32_t* __restrict__ slots, float* __restrict__ o_raw, int heads, int d, int dv, int chunk, int unit, int copies) {
    constexpr int COLS = SCAN_THREADS / PARTS;
    constexpr int DP = ROWS * PARTS;                        // a staged row of k or q
    constexpr int PER = SCAN_STAGE / SCAN_THREADS;          // staged numbers of k, and of q, a thread
    constexpr int PER_V = 32 * COLS / SCAN_THREADS > 0 ? 32 * COLS / SCAN_THREADS : 1;
    extern __shared__ __align__(16) float lds[];
    float* k_s = lds;
    float* q_s = k_s + (size_t)chunk * DP;
    float* v_s = q_s + (size_t)chunk * DP;
    float* g_s = v_s + (size_t)chunk * COLS;              // a token's (keep, take, floor of the denominator, -)
    float* m_s = g_s + (size_t)chunk * 4;                  // m after the chunk
    const int seq = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    const int part = tid & (PARTS - 1), col_l = tid / PARTS;
    const int col = blockIdx.z * COLS + col_l;
    const bool live = col < dv;
    const int row0 = part * ROWS;
    const int first = q_start[seq], count = q_len[seq];
    float* slot = state + (size_t)slots[seq] * state_stride;
    float* S_g = slot + ((size_t)head * dv + (live ? col : 0)) * d;
    float* n_all = slot + (size_t)heads * d * dv;
    float* m_all = n_all + (size_t)copies * heads * d;
    const int copy_in = blockIdx.z * COLS / unit;            // every copy holds the same numbers: the first of this workgroup's is read
    const float* n_g = n_all + ((size_t)copy_in * heads + head) * d;
    const bool writes_copy = live && col % unit == 0;       // this column's lanes write the copy of the column's unit
    float* n_w = n_all + ((size_t)((live ? col : 0) / unit) * heads + head) * d;

    float S[ROWS], nv[ROWS];
    // a lane's rows of a column lie together: 16 bytes a load where the addresses allow
    const bool wide = d % 4 == 0 && (((uintptr_t)S_g | (uintptr_t)n_g | (uintptr_t)n_w) & 15) == 0 && row0 + ROWS <= d;
    if (wide) {
#pragma unroll
        for (int r = 0; r < ROWS; r += 4) {
            *reinterpret_cast<float4*>(S + r) = live ? *reinterpret_cast<const float4*>(S_g + row0 + r) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            *reinterpret_cast<float4*>(nv + r) = *reinterpret_cast<const float4*>(n_g + row0 + r);
        }
    } else {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int row = row0 + r;
            S[r] = (live && row < d) ? S_g[row] : 0.0f;
            nv[r] = row < d ? n_g[row] : 0.0f;
        }
    }
    float m = m_all[(size_t)copy_in * heads + head];
    const float q_scale = 1.0f / sqrtf((float)d);
    const float bi = bias_i[head], bf = bias_f[head];
    const int at_q = head * d, at_k = heads * d + head * d, at_v = 2 * heads * d + head * dv;
    const int at_i = 2 * heads * d + 2 * heads * dv + head, at_f = at_i + heads;

    // a chunk's numbers on their way: asked for before the chunk ahead of it is walked, put into LDS after
    float k_r[PER], q_r[PER], v_r[PER_V], zi = 0.0f, zf = 0.0f;
    auto fetch = [&](int c0, int n_tok) {
        const float* base = proj + (size_t)(first + c0) * stride;
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int i = tid + j * SCAN_THREADS;
            k_r[j] = q_r[j] = 0.0f;
            if (i < n_tok * DP) {
                const int tt = i / DP, e = i - tt * DP;
                if (e < d) {
                    k_r[j] = base[(size_t)tt * stride + at_k + e];
                    q_r[j] = base[(size_t)tt * stride + at_q + e];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < PER_V; ++j) {
            const int i = tid + j * SCAN_THREADS;
            if (i < n_tok * COLS) {
                const int tt = i / COLS, cc = blockIdx.z * COLS + (i - tt * COLS);
                v_r[j] = cc < dv ? base[(size_t)tt * stride + at_v + cc] : 0.0f;
            }
        }
        if (tid < n_tok) {
            zi = base[(size_t)tid * stride + at_i];
            zf = base[(size_t)tid * stride + at_f];
        }
    };
    int n_tok = min(chunk, count);
    fetch(0, n_tok);
    for (int c0 = 0; c0 < count; c0 += chunk) {
        __syncthreads();        // the chunk before has been walked by every wave
#pragma unroll
        for (int j = 0; j < PER; ++j) {
            const int i = tid + j * SCAN_THREADS;
            if (i < n_tok * DP) {
                k_s[i] = k_r[j];
                q_s[i] = q_r[j] * q_scale;
            }
        }
#pragma unroll
        for (int j = 0; j < PER_V; ++j) {
            const int i = tid + j * SCAN_THREADS;
            if (i < n_tok * COLS) v_s[i] = v_r[j];
        }
        if (tid < KIPP_WAVE) {
            // The gates, by the first wave: a lane a token takes tanh and the logarithms; then the running maximum walks the
            // chunk's tokens in order (m' = max(lf + m, li): an add and a maximum a token, the lanes' numbers read across
            // the wave), and every lane takes its token's three exponentials.  The walk below is left with multiply-adds.
            const float li = tid < n_tok ? cap * tanhf((zi + bi) / cap) : 0.0f;
            const float lf = tid < n_tok ? log_sigmoid(cap * tanhf((zf + bf) / cap)) : 0.0f;
            float m_before = 0.0f, m_after = 0.0f;
            for (int t = 0; t < n_tok; ++t) {
                const float lf_t = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(lf), t));
                const float li_t = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(li), t));
                const float m_new = fmaxf(lf_t + m, li_t);
                if (tid == t) {
                    m_before = m;
                    m_after = m_new;
                }
                m = m_new;
            }
            if (tid < n_tok)
                *reinterpret_cast<float4*>(g_s + 4 * tid) = make_float4(expf(lf + m_before - m_after), expf(li - m_after), expf(-m_after), 0.0f);
            if (tid == 0) m_s[0] = m;
        }
        __syncthreads();
        const int n_next = min(chunk, count - c0 - chunk);
        if (n_next > 0) fetch(c0 + chunk, n_next);
        // eight tokens at a time: their gates out of LDS, then the multiply-adds over a lane's rows, then the sums over the
        // lanes of a column for all eight (data-parallel moves inside a row of 16 lanes; only a column of 64 lanes takes
        // its last two steps through LDS)
        for (int t8 = 0; t8 < n_tok; t8 += SCAN_GROUP) {
            float keep[SCAN_GROUP], take[SCAN_GROUP], floor_p[SCAN_GROUP], num_p[SCAN_GROUP], den_p[SCAN_GROUP];
#pragma unroll
            for (int u = 0; u < SCAN_GROUP; ++u) {
                const float4 g = *reinterpret_cast<const float4*>(g_s + 4 * min(t8 + u, n_tok - 1));
                keep[u] = g.x;
                take[u] = g.y;
                floor_p[u] = g.z;
            }
#pragma unroll
            for (int u = 0; u < SCAN_GROUP; ++u) {
                num_p[u] = den_p[u] = 0.0f;
                if (t8 + u < n_tok) {
                    const int tt = t8 + u;
                    const float tv = take[u] * v_s[tt * COLS + col_l];
                    const float* k_t = k_s + (size_t)tt * DP + row0;
                    const float* q_t = q_s + (size_t)tt * DP + row0;
                    float kk[ROWS], qq[ROWS];
#pragma unroll
                    for (int r = 0; r < ROWS; r += 4) {
                        *reinterpret_cast<float4*>(kk + r) = *reinterpret_cast<const float4*>(k_t + r);
                        *reinterpret_cast<float4*>(qq + r) = *reinterpret_cast<const float4*>(q_t + r);
                    }
                    constexpr int RUNS = ROWS / BASE;
                    static_assert(RUNS == 1 || RUNS == 2 || RUNS == 4 || RUNS == 8, "runs of rows");
                    float num[RUNS], den[RUNS];
#pragma unroll
                    for (int g = 0; g < RUNS; ++g) num[g] = den[g] = 0.0f;
#pragma unroll
                    for (int r = 0; r < ROWS; ++r) {
                        S[r] = fmaf(keep[u], S[r], kk[r] * tv);
                        nv[r] = fmaf(keep[u], nv[r], take[u] * kk[r]);
                        num[r / BASE] = fmaf(S[r], qq[r], num[r / BASE]);
                        den[r / BASE] = fmaf(nv[r], qq[r], den[r / BASE]);
                    }
#pragma unroll
                    for (int w = 1; w < RUNS; w <<= 1)
#pragma unroll
                        for (int i = 0; i + w < RUNS; i += 2 * w) {
                            num[i] += num[i + w];
                            den[i] += den[i + w];
                        }
                    num_p[u] = num[0];
                    den_p[u] = den[0];
                }
            }
#pragma unroll
            for (int u = 0; u < SCAN_GROUP; ++u) {
                num_p[u] = column_sum<PARTS>(num_p[u]);
                den_p[u] = column_sum<PARTS>(den_p[u]);
            }
            if (live && part == 0) {
#pragma unroll
                for (int u = 0; u < SCAN_GROUP; ++u)
                    if (t8 + u < n_tok)
                        o_raw[((size_t)(first + c0 + t8 + u) * heads + head) * dv + col] = num_p[u] / (fmaxf(fabsf(den_p[u]), floor_p[u]) + 1e-6f);
            }
        }
        n_tok = n_next;
    }
    if (wide) {
#pragma unroll
        for (int r = 0; r < ROWS; r += 4) {
            if (live) *reinterpret_cast<float4*>(S_g + row0 + r) = *reinterpret_cast<float4*>(S + r);
            if (writes_copy) *reinterpret_cast<float4*>(n_w + row0 + r) = *reinterpret_cast<float4*>(nv + r);
        }
    } else {
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int row = row0 + r;
            if (live && row < d) S_g[row] = S[r];
            if (writes_copy && row < d) n_w[row] = nv[r];
        }
    }
    if (writes_copy && part == 0) m_all[(size_t)(col / unit) * heads + head] = m_s[0];
}

#define FINISH_HEADS 4

template <typename TO>
__global__ void mlstm_finish_kernel(const float* __restrict__ o_raw, const float* __restrict__ proj, int stride, int gate_at,
                                    const float* __restrict__ norm_w, float eps, TO* __restrict__ out, int heads, int dv) {
    const int wave = threadIdx.x / KIPP_WAVE, lane = threadIdx.x & (KIPP_WAVE - 1);
    const int t = blockIdx.y, head = blockIdx.x * FINISH_HEADS + wave;
    if (head >= heads) return;
    const float* src = o_raw + ((size_t)t * heads + head) * dv;
    float ss = 0.0f;
    for (int e = lane; e < dv; e += KIPP_WAVE) ss = fmaf(src[e], src[e], ss);
    ss = wave_sum(ss);
    const float scale = 1.0f / sqrtf(ss / (float)dv + eps);
    const float* gate = proj + (size_t)t * stride + gate_at + head * dv;
    TO* dst = out + ((size_t)t * heads + head) * dv;
    for (int e = lane; e < dv; e += KIPP_WAVE)
        store_f(dst, e, src[e] * scale * norm_w[head * dv + e] * (1.0f / (1.0f + expf(-gate[e]))));
}

// Lanes that share a column of the memory in the walk over prompt portions: 8 rows a lane (16 for keys of 129 to 256 and
// of more than 512 numbers).  256 / lanes is the `unit`: the columns that share a copy of n and m in the state.
static int kipp_mlstm_parts(int d) { return d <= 32 ? 4 : (d <= 256 ? 16 : 64); }

extern "C" {

// `few`: every entry brings few tokens (single decoded tokens): where the key size allows, a workgroup takes 64 columns
// with 4 lanes each, a quarter of the workgroups, each reading longer runs of the state.
int kipp_mlstm_scan(const float* proj, int stride, const float* bias_i, const float* bias_f, float cap, float* state,
                    size_t state_stride, const int32_t* q_start, const int32_t* q_len, const int32_t* slots, float* o_raw,
                    int n_seqs, int heads, int d, int dv, int few, hipStream_t stream) {
    if (n_seqs <= 0) return 0;
    if (heads <= 0 || d <= 0 || d > 1024 || dv <= 0 || !(cap > 0.0f)) return -1;
    const int unit = SCAN_THREADS / kipp_mlstm_parts(d);
    const int copies = (dv + unit - 1) / unit;
    if (stride < 2 * heads * d + 2 * heads * dv + 2 * heads || state_stride < (size_t)heads * d * dv + (size_t)copies * (heads * d + heads)) return -1;
    const int base_parts = kipp_mlstm_parts(d);
    const int base_rows = d <= 128 ? 8 : (d <= 256 ? 16 : (d <= 512 ? 8 : 16));
    int parts = base_parts, rows = base_rows;
    if (few && d > 32 && d <= 128) parts = 4, rows = 32;
    else if (few && d > 128 && d <= 256) parts = 8, rows = 32;
    const int cols = SCAN_THREADS / parts;
    dim3 grid(n_seqs, heads, (dv + cols - 1) / cols), block(SCAN_THREADS);
    int chunk = SCAN_STAGE / (rows * parts);          // tokens whose k and q fit the staging registers
    if (chunk > 32) chunk = 32;
    const size_t lds = ((size_t)chunk * (2 * rows * parts + cols + 4) + 4) * sizeof(float);
#define KIPP_SCAN(R, P, B)                                                                                                          \
    hipLaunchKernelGGL((mlstm_scan_kernel<R, P, B>), grid, block, lds, stream, proj, stride, bias_i, bias_f, cap, state, state_stride, \
                       q_start, q_len, slots, o_raw, heads, d, dv, chunk, unit, copies)
    if (parts == 4 && rows == 8) KIPP_SCAN(8, 4, 8);
    else if (parts == 4) KIPP_SCAN(32, 4, 8);
    else if (parts == 8) KIPP_SCAN(32, 8, 16);
    else if (parts == 16 && rows == 8) KIPP_SCAN(8, 16, 8);
    else if (parts == 16) KIPP_SCAN(16, 16, 16);
    else if (rows == 8) KIPP_SCAN(8, 64, 8);
    else KIPP_SCAN(16, 64, 16);
#undef KIPP_SCAN
    return KIPP_LAUNCH_CHECK();
}

int kipp_mlstm_finish(const float* o_raw, const float* proj, int stride, int gate_at, const float* norm_w, float eps,
                      void* out, int out_dtype, int n_tokens, int heads, int dv, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (heads <= 0 || dv <= 0 || stride < gate_at + heads * dv) return -1;
    dim3 grid((heads + FINISH_HEADS - 1) / FINISH_HEADS, n_tokens), block(FINISH_HEADS * KIPP_WAVE);
    if (out_dtype == KIPP_BF16)
        hipLaunchKernelGGL(mlstm_finish_kernel<bf16_t>, grid, block, 0, stream, o_raw, proj, stride, gate_at, norm_w, eps, (bf16_t*)out, heads, dv);
    else
        hipLaunchKernelGGL(mlstm_finish_kernel<float>, grid, block, 0, stream, o_raw, proj, stride, gate_at, norm_w, eps, (float*)out, heads, dv);
    return KIPP_LAUNCH_CHECK();
}

}  // extern "C"
