// A routed feed-forward (mixture of experts): the router's choice, the tokens sorted by expert, the experts'
// two products over those runs of rows, and the weighted sum.
//
//     route    p = softmax(z) over all experts (float32); the `top` largest p (the lower index first among equals);
//              weight = p / (sum of the chosen p + eps)
//     route (grouped)  s = sigmoid(z); choice scores c = s + correction; experts in equal groups of neighbours, a group's
//              score the sum of its two largest c; only experts of the `keep` best groups can be chosen; the `top` largest
//              c among them; weight = s / (sum of the chosen s + eps) * scale
//     sort     the (token, choice) pairs in runs of one expert each, cut into tiles of up to 16 (or 128) rows; the list of tiles
//              is made on the device, so the host never learns the counts and the launches have a fixed shape
//     expert   a tile's rows against its expert's matrix: out[row][n] = act(sum_k W_e[n][k] x[row][k]).  bfloat16 with K a
//              multiple of 32: on the matrix cores, a workgroup a (tile of up to 128 rows, 128 columns), a wave 32 of the
//              columns in 8 x 2 fragments of 16 x 16 (two workgroups share a compute unit's registers); steps of 64 numbers of k come from memory 128 bytes a row (eight
//              lanes side by side) into registers while the step before is multiplied out of LDS; a tile of a few rows
//              (single tokens) multiplies only the fragments it has, and is then bound by the read of its expert's matrix.  Else (float32, other K): a lane takes a column of a tile of 16 rows.
//              Either way the sum over k runs in one order for every row, so a row's result does not depend on its tile
//     combine  out[t] = sum_j weight[t][j] y[place of (t, j)] (+ the shared expert's result, slabs added in order)
#include "common.h"
#include <math.h>

#define ROUTE_WAVES 4
#define MAX_EXPERTS 1024
#define MAX_TOP 32
#define TILE_ROWS 16
#define EXPERT_COLS 256
#define EXPERT_KC 128
#define MFMA_ROWS 128       // rows of a tile of the matrix-core product: eight fragments of 16
#define MFMA_COLS 128       // columns of a workgroup: four waves with two fragments each
#define MFMA_NF (MFMA_COLS / 64)
#define MFMA_KC 64          // numbers of k a step brings into LDS
#define MFMA_PITCH 72       // bfloat16 numbers from a row to the next in LDS
#define MFMA_THREADS 256
#define XCDS 8              // dies of the chip; consecutive workgroups of a launch go to them in turn

enum { ACT_NONE = -1, ACT_SILU = 0, ACT_RELU = 1, ACT_GELU = 2, ACT_GELU_TANH = 3, ACT_RELU2 = 4 };

__device__ __forceinline__ float activate(float z, int act) {
    switch (act) {
        case ACT_SILU: return z / (1.0f + expf(-z));
        case ACT_RELU: return fmaxf(z, 0.0f);
        case ACT_GELU: return 0.5f * z * (1.0f + erff(z * 0.70710678118654752440f));
        case ACT_GELU_TANH: return 0.5f * z * (1.0f + tanhf(0.79788456080286535588f * (z + 0.044715f * z * z * z)));
        case ACT_RELU2: { const float r = fmaxf(z, 0.0f); return r * r; }
        default: return z;
    }
}

// One wave a token.  z: float32 [tokens][stride] (or slabs of it, added in order).
__global__ void __launch_bounds__(ROUTE_WAVES * KIPP_WAVE)
moe_route_kernel(const float* __restrict__ z, int parts, size_t part_stride, int stride, int32_t* __restrict__ chosen,
                 float* __restrict__ weight, int tokens, int experts, int top, float eps) {
    const int wave = threadIdx.x / KIPP_WAVE, lane = threadIdx.x & (KIPP_WAVE - 1);
    const int t = blockIdx.x * ROUTE_WAVES + wave;
    if (t >= tokens) return;        // no barrier below
    float p[MAX_EXPERTS / KIPP_WAVE];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < MAX_EXPERTS / KIPP_WAVE; ++i) {
        const int e = lane + i * KIPP_WAVE;
        float v = -INFINITY;
        if (e < experts) {
            v = z[(size_t)t * stride + e];
            for (int q = 1; q < parts; ++q) v += z[q * part_stride + (size_t)t * stride + e];
        }
        p[i] = v;
        m = fmaxf(m, v);
    }
    m = wave_max(m);
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < MAX_EXPERTS / KIPP_WAVE; ++i) {
        p[i] = (lane + i * KIPP_WAVE < experts) ? expf(p[i] - m) : -1.0f;
        if (p[i] > 0.0f) sum += p[i];
    }
    sum = wave_sum(sum);
    float picked_sum = 0.0f;
    float mine = 0.0f;          // lane j keeps the j-th choice
    int mine_e = 0;
    for (int j = 0; j < top; ++j) {
        float best = -1.0f;
        int best_e = MAX_EXPERTS;
#pragma unroll
        for (int i = 0; i < MAX_EXPERTS / KIPP_WAVE; ++i)
            if (p[i] > best) { best = p[i]; best_e = lane + i * KIPP_WAVE; }     // the lowest index of a lane's largest
        for (int off = 32; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, KIPP_WAVE);
            const int oe = __shfl_xor(best_e, off, KIPP_WAVE);
            if (ob > best || (ob == best && oe < best_e)) { best = ob; best_e = oe; }
        }
#pragma unroll
        for (int i = 0; i < MAX_EXPERTS / KIPP_WAVE; ++i)
            if (lane + i * KIPP_WAVE == best_e) p[i] = -1.0f;
        const float s = best / sum;
        picked_sum += s;
        if (lane == j) { mine = s; mine_e = best_e; }
    }
    if (lane < top) {
        chosen[(size_t)t * top + lane] = mine_e;
        weight[(size_t)t * top + lane] = mine / (picked_sum + eps);
    }
}

// One wave a token: sigmoid scores, a correction for the choice alone, groups of neighbouring experts of which the best stay.
__global__ void __launch_bounds__(ROUTE_WAVES * KIPP_WAVE)
moe_route_grouped_kernel(const float* __restrict__ z, int parts, size_t part_stride, int stride, const float* __restrict__ correction,
                         int32_t* __restrict__ chosen, float* __restrict__ weight, int tokens, int experts, int top, float eps,
                         int group_count, int group_keep, float scale) {
    __shared__ float c_s[ROUTE_WAVES][MAX_EXPERTS];     // choice scores, then -inf for experts of groups that do not stay
    __shared__ float g_s[ROUTE_WAVES][MAX_EXPERTS];     // group scores, -inf once a group is taken
    const int wave = threadIdx.x / KIPP_WAVE, lane = threadIdx.x & (KIPP_WAVE - 1);
    int t = blockIdx.x * ROUTE_WAVES + wave;
    const bool live = t < tokens;
    if (!live) t = tokens - 1;      // stay in step with the barriers
    const int size = experts / group_count;
    float s[MAX_EXPERTS / KIPP_WAVE];
#pragma unroll
    for (int i = 0; i < MAX_EXPERTS / KIPP_WAVE; ++i) {
        const int e = lane + i * KIPP_WAVE;
        s[i] = 0.0f;
        if (e < experts) {
            float v = z[(size_t)t * stride + e];
            for (int q = 1; q < parts; ++q) v += z[q * part_stride + (size_t)t * stride + e];
            s[i] = 1.0f / (1.0f + expf(-v));
            c_s[wave][e] = s[i] + (correction != nullptr ? correction[e] : 0.0f);
        }
    }
    __syncthreads();
    if (group_keep < group_count) {
        for (int g = lane; g < group_count; g += KIPP_WAVE) {
            float a = -INFINITY, b = -INFINITY;      // the two largest of the group
            for (int j = 0; j < size; ++j) {
                const float v = c_s[wave][g * size + j];
                if (v > a) { b = a; a = v; } else if (v > b) { b = v; }
            }
            g_s[wave][g] = size > 1 ? a + b : a;
        }
        __syncthreads();
        for (int round = 0; round < group_keep; ++round) {
            float best = -INFINITY;
            int best_g = MAX_EXPERTS;
            for (int g = lane; g < group_count; g += KIPP_WAVE) {
                const float v = g_s[wave][g];
                if (v > best || (best_g == MAX_EXPERTS && v != -INFINITY)) { best = v; best_g = g; }
            }
            for (int off = 32; off > 0; off >>= 1) {
                const float ob = __shfl_xor(best, off, KIPP_WAVE);
                const int og = __shfl_xor(best_g, off, KIPP_WAVE);
                if (og != MAX_EXPERTS && (best_g == MAX_EXPERTS || ob > best || (ob == best && og < best_g))) { best = ob; best_g = og; }
            }
            __syncthreads();
            if (lane == 0 && best_g != MAX_EXPERTS) g_s[wave][best_g] = -INFINITY;      // taken: it stays
            __syncthreads();
        }
        for (int e = lane; e < experts; e += KIPP_WAVE)
            if (g_s[wave][e / size] != -INFINITY) c_s[wave][e] = -INFINITY;             // its group was not taken
        __syncthreads();
    }
    float c[MAX_EXPERTS / KIPP_WAVE];
#pragma unroll
    for (int i = 0; i < MAX_EXPERTS / KIPP_WAVE; ++i) {
        const int e = lane + i * KIPP_WAVE;
        c[i] = e < experts ? c_s[wave][e] : -INFINITY;
    }
    float picked_sum = 0.0f, mine = 0.0f;       // lane j keeps the j-th choice
    int mine_e = 0;
    for (int j = 0; j < top; ++j) {
        float best = -INFINITY, best_s = 0.0f;
        int best_e = MAX_EXPERTS;
#pragma unroll
        for (int i = 0; i < MAX_EXPERTS / KIPP_WAVE; ++i)
            if (c[i] > best) { best = c[i]; best_e = lane + i * KIPP_WAVE; best_s = s[i]; }     // the lowest index of a lane's largest
        for (int off = 32; off > 0; off >>= 1) {
            const float ob = __shfl_xor(best, off, KIPP_WAVE), os = __shfl_xor(best_s, off, KIPP_WAVE);
            const int oe = __shfl_xor(best_e, off, KIPP_WAVE);
            if (ob > best || (ob == best && oe < best_e)) { best = ob; best_e = oe; best_s = os; }
        }
#pragma unroll
        for (int i = 0; i < MAX_EXPERTS / KIPP_WAVE; ++i)
            if (lane + i * KIPP_WAVE == best_e) c[i] = -INFINITY;
        picked_sum += best_s;
        if (lane == j) { mine = best_s; mine_e = best_e < experts ? best_e : 0; }
    }
    if (live && lane < top) {
        chosen[(size_t)t * top + lane] = mine_e;
        weight[(size_t)t * top + lane] = mine / (picked_sum + eps) * scale;
    }
}

// One workgroup sorts all pairs.  tiles: int32 [max_tiles][3] = (expert, first row, rows); rows 0 marks an unused tile.
__global__ void __launch_bounds__(1024)
moe_sort_kernel(const int32_t* __restrict__ chosen, int pairs, int experts, int top, int32_t* __restrict__ pair_token,
                int32_t* __restrict__ place_of_pair, int32_t* __restrict__ tiles, int max_tiles, int tile_rows) {
    __shared__ int count[MAX_EXPERTS];
    __shared__ int first[MAX_EXPERTS + 1];
    __shared__ int tile_first[MAX_EXPERTS + 1];
    for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) atomicAdd(&count[chosen[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int rows = 0, tl = 0;
        for (int e = 0; e < experts; ++e) {
            first[e] = rows;
            tile_first[e] = tl;
            rows += count[e];
            tl += (count[e] + tile_rows - 1) / tile_rows;
        }
        first[experts] = rows;
        tile_first[experts] = tl;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += blockDim.x) {
        const int n = count[e];
        for (int j = 0; j * tile_rows < n; ++j) {
            int32_t* tile = tiles + (size_t)(tile_first[e] + j) * 3;
            tile[0] = e;
            tile[1] = first[e] + j * tile_rows;
            tile[2] = min(tile_rows, n - j * tile_rows);
        }
    }
    for (int i = tile_first[experts] + threadIdx.x; i < max_tiles; i += blockDim.x) {
        tiles[(size_t)i * 3] = 0;
        tiles[(size_t)i * 3 + 1] = 0;
        tiles[(size_t)i * 3 + 2] = 0;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += blockDim.x) count[e] = 0;     // now the next free place of a run
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = chosen[p];
        const int at = first[e] + atomicAdd(&count[e], 1);
        pair_token[at] = p / top;
        place_of_pair[p] = at;
    }
}

// x rows are x[gather[row]] (gather null: x[row]); w: [experts][n_out][k]; out[row][n_out].
template <typename TX, typename TW, typename TO>
__global__ void __launch_bounds__(EXPERT_COLS)
moe_expert_kernel(const TX* __restrict__ x, const int32_t* __restrict__ gather, const TW* __restrict__ w,
                  const int32_t* __restrict__ tiles, TO* __restrict__ out, int n_out, int k, int act) {
    __shared__ float x_s[TILE_ROWS][EXPERT_KC];
    const int32_t* tile = tiles + (size_t)blockIdx.x * 3;
    const int rows = tile[2];
    if (rows == 0) return;      // uniform over the workgroup
    const int expert = tile[0], row0 = tile[1];
    const int col = blockIdx.y * EXPERT_COLS + threadIdx.x;
    const TW* w_row = w + ((size_t)expert * n_out + (col < n_out ? col : 0)) * k;
    float acc[TILE_ROWS];
#pragma unroll
    for (int r = 0; r < TILE_ROWS; ++r) acc[r] = 0.0f;
    for (int k0 = 0; k0 < k; k0 += EXPERT_KC) {
        const int kc = min(EXPERT_KC, k - k0);
        __syncthreads();
        for (int i = threadIdx.x; i < TILE_ROWS * EXPERT_KC; i += EXPERT_COLS) {
            const int r = i / EXPERT_KC, e = i - r * EXPERT_KC;
            float v = 0.0f;
            if (r < rows && e < kc) {
                const size_t src_row = gather != nullptr ? (size_t)gather[row0 + r] : (size_t)(row0 + r);
                v = load_f(x + src_row * k, k0 + e);
            }
            x_s[r][e] = v;
        }
        __syncthreads();
        if (col < n_out) {
            for (int e = 0; e < kc; ++e) {
                const float wv = load_f(w_row, k0 + e);
#pragma unroll
                for (int r = 0; r < TILE_ROWS; ++r) acc[r] = fmaf(wv, x_s[r][e], acc[r]);
            }
        }
    }
    if (col >= n_out) return;
#pragma unroll
    for (int r = 0; r < TILE_ROWS; ++r)
        if (r < rows) store_f(out + (size_t)(row0 + r) * n_out, col, activate(acc[r], act));
}

// The same on the matrix cores: bfloat16 x and w, K a multiple of 32, tiles of up to MFMA_ROWS rows.  A 16 x 16 x 32
// product takes, from lane l, 8 numbers of row l % 16 at k = 8 (l / 16) .. + 7 of either operand, and leaves
// C[4 (l / 16) + v][l % 16] in its register v.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
union Frag {
    u32x4 u;
    bf16x8 v;
};

template <typename TO>
__global__ void __launch_bounds__(MFMA_THREADS)
moe_expert_mfma_kernel(const bf16_t* __restrict__ x, const int32_t* __restrict__ gather, const bf16_t* __restrict__ w,
                       const int32_t* __restrict__ tiles, TO* __restrict__ out, int n_out, int k, int act) {
    // 64 numbers of k of every row of the tile and of every column of the workgroup, a row 144 bytes apart from the next
    // (the fragments' reads of 16 bytes a lane then spread over the banks)
    __shared__ __attribute__((aligned(16))) bf16_t a_s[MFMA_ROWS * MFMA_PITCH];
    __shared__ __attribute__((aligned(16))) bf16_t b_s[MFMA_COLS * MFMA_PITCH];
    // Workgroups go to the chip's 8 dies in turn, each with an L2 of its own: the launch's workgroups are renumbered so
    // that a die works on neighbouring tiles at a time, which are mostly row tiles of one expert and read the same
    // columns of its matrix.
    const unsigned launched = blockIdx.x + blockIdx.y * gridDim.x, total = gridDim.x * gridDim.y;
    const unsigned die = launched % XCDS, turn = launched / XCDS, each = total / XCDS, more = total % XCDS;
    const unsigned item = (die < more ? die * (each + 1) : more * (each + 1) + (die - more) * each) + turn;
    const int32_t* tile = tiles + (size_t)(item % gridDim.x) * 3;
    const int rows = tile[2];
    if (rows == 0) return;      // uniform over the workgroup
    const int expert = tile[0], row0 = tile[1];
    const int tid = threadIdx.x;
    const int wave = tid / KIPP_WAVE, lane = tid & (KIPP_WAVE - 1), l16 = lane & 15, h = lane >> 4;
    const int col_base = (item / gridDim.x) * MFMA_COLS;
    const int mfrags = (rows + 15) >> 4;
    // from memory, 8 threads take the 128 bytes of a row's step: thread t rows t / 8 + 32 i, bytes 16 (t % 8) ..
    const int ld_row = tid >> 3, ld_ch = tid & 7;
    // where a lane's rows begin, in numbers from x and from the expert's matrix (the launcher has checked that 32 bits hold them)
    unsigned a_src[MFMA_ROWS / 32], b_src[MFMA_COLS / 32];
    const bf16_t* w_e = w + (size_t)expert * n_out * k;
#pragma unroll
    for (int i = 0; i < MFMA_ROWS / 32; ++i) {
        const int r = min(ld_row + 32 * i, rows - 1);       // rows beyond the tile's read its last one and are not stored
        const unsigned src = gather != nullptr ? (unsigned)gather[row0 + r] : (unsigned)(row0 + r);
        a_src[i] = src * (unsigned)k + 8 * ld_ch;
    }
#pragma unroll
    for (int i = 0; i < MFMA_COLS / 32; ++i) {
        const int c = min(col_base + ld_row + 32 * i, n_out - 1);
        b_src[i] = (unsigned)c * (unsigned)k + 8 * ld_ch;
    }
    u32x4 a_r[MFMA_ROWS / 32], b_r[MFMA_COLS / 32];
    const u32x4 zero = (u32x4){0u, 0u, 0u, 0u};
    auto fetch = [&](int k0) {
        const bool there = k0 + 8 * ld_ch < k;              // k is a multiple of 32: the last step may be half a step
#pragma unroll
        for (int i = 0; i < MFMA_ROWS / 32; ++i)
            if (32 * i < 16 * mfrags) a_r[i] = there ? *(const u32x4*)(x + a_src[i] + k0) : zero;
#pragma unroll
        for (int i = 0; i < MFMA_COLS / 32; ++i) b_r[i] = there ? *(const u32x4*)(w_e + b_src[i] + k0) : zero;
    };
    f32x4 acc[MFMA_ROWS / 16][MFMA_NF];
#pragma unroll
    for (int i = 0; i < MFMA_ROWS / 16; ++i)
#pragma unroll
        for (int j = 0; j < MFMA_NF; ++j) acc[i][j] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    fetch(0);
    for (int k0 = 0; k0 < k; k0 += MFMA_KC) {
        __syncthreads();        // the step before has been multiplied
#pragma unroll
        for (int i = 0; i < MFMA_ROWS / 32; ++i)
            if (32 * i < 16 * mfrags) *(u32x4*)(a_s + (ld_row + 32 * i) * MFMA_PITCH + 8 * ld_ch) = a_r[i];
#pragma unroll
        for (int i = 0; i < MFMA_COLS / 32; ++i) *(u32x4*)(b_s + (ld_row + 32 * i) * MFMA_PITCH + 8 * ld_ch) = b_r[i];
        __syncthreads();
        if (k0 + MFMA_KC < k) fetch(k0 + MFMA_KC);      // on its way while this step is multiplied
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            Frag b[MFMA_NF];
#pragma unroll
            for (int j = 0; j < MFMA_NF; ++j) b[j].u = *(const u32x4*)(b_s + (wave * 16 * MFMA_NF + 16 * j + l16) * MFMA_PITCH + 32 * half + 8 * h);
            if (mfrags == MFMA_ROWS / 16) {          // a whole tile: nothing to ask between the fragments
#pragma unroll
                for (int i = 0; i < MFMA_ROWS / 16; ++i) {
                    Frag a;
                    a.u = *(const u32x4*)(a_s + (16 * i + l16) * MFMA_PITCH + 32 * half + 8 * h);
#pragma unroll
                    for (int j = 0; j < MFMA_NF; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b[j].v, acc[i][j], 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int i = 0; i < MFMA_ROWS / 16 - 1; ++i) {
                    if (i < mfrags) {
                        Frag a;
                        a.u = *(const u32x4*)(a_s + (16 * i + l16) * MFMA_PITCH + 32 * half + 8 * h);
#pragma unroll
                        for (int j = 0; j < MFMA_NF; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b[j].v, acc[i][j], 0, 0, 0);
                    }
                }
            }
        }
    }
    const int col0 = col_base + wave * 16 * MFMA_NF;
#pragma unroll
    for (int i = 0; i < MFMA_ROWS / 16; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int r = 16 * i + 4 * h + v;
            if (r < rows) {
                TO* dst = out + (size_t)(row0 + r) * n_out;
#pragma unroll
                for (int j = 0; j < MFMA_NF; ++j) {
                    const int c = col0 + 16 * j + l16;
                    if (c < n_out) store_f(dst, c, activate(acc[i][j][v], act));
                }
            }
        }
}

// out[t][c] = sum_j weight[t][j] y[place[t top + j]][c] + sum of the slabs of shared[t][c]
__global__ void moe_combine_kernel(const float* __restrict__ y, const int32_t* __restrict__ place, const float* __restrict__ weight,
                                   const float* __restrict__ shared, int shared_parts, size_t shared_stride,
                                   float* __restrict__ out, int tokens, int width, int top) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)tokens * width) return;
    const int t = (int)(i / width), c = (int)(i - (size_t)t * width);
    float acc = 0.0f;
    for (int j = 0; j < top; ++j)
        acc = fmaf(weight[(size_t)t * top + j], y[(size_t)place[(size_t)t * top + j] * width + c], acc);
    for (int p = 0; p < shared_parts; ++p) acc += shared[p * shared_stride + i];
    out[i] = acc;
}

extern "C" int kipp_moe_route(const float* z, int parts, int stride, int32_t* chosen, float* weight, int tokens, int experts, int top,
                              float eps, int32_t* pair_token, int32_t* place_of_pair, int32_t* tiles, int max_tiles, int tile_rows,
                              hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (experts <= 0 || experts > MAX_EXPERTS || top <= 0 || top > MAX_TOP || top > experts || stride < experts || parts <= 0) return -1;
    const int pairs = tokens * top;
    if (tile_rows != TILE_ROWS && tile_rows != MFMA_ROWS) return -1;
    if (max_tiles < (pairs + tile_rows - 1) / tile_rows + (experts < pairs ? experts : pairs)) return -1;
    hipLaunchKernelGGL(moe_route_kernel, dim3((tokens + ROUTE_WAVES - 1) / ROUTE_WAVES), dim3(ROUTE_WAVES * KIPP_WAVE), 0, stream, z, parts,
                       (size_t)tokens * stride, stride, chosen, weight, tokens, experts, top, eps);
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, (const int32_t*)chosen, pairs, experts, top, pair_token,
                       place_of_pair, tiles, max_tiles, tile_rows);
    return KIPP_LAUNCH_CHECK();
}

// The same with sigmoid scores, a correction of the choice (or none) and groups of which `group_keep` of `group_count` stay.
extern "C" int kipp_moe_route_grouped(const float* z, int parts, int stride, const float* correction, int32_t* chosen, float* weight,
                                      int tokens, int experts, int top, float eps, int group_count, int group_keep, float scale,
                                      int32_t* pair_token, int32_t* place_of_pair, int32_t* tiles, int max_tiles, int tile_rows,
                                      hipStream_t stream) {
    if (tokens <= 0) return 0;
    if (experts <= 0 || experts > MAX_EXPERTS || top <= 0 || top > MAX_TOP || top > experts || stride < experts || parts <= 0) return -1;
    if (group_count <= 0 || experts % group_count || group_keep <= 0 || group_keep > group_count ||
        top > group_keep * (experts / group_count)) return -1;
    const int pairs = tokens * top;
    if (tile_rows != TILE_ROWS && tile_rows != MFMA_ROWS) return -1;
    if (max_tiles < (pairs + tile_rows - 1) / tile_rows + (experts < pairs ? experts : pairs)) return -1;
    hipLaunchKernelGGL(moe_route_grouped_kernel, dim3((tokens + ROUTE_WAVES - 1) / ROUTE_WAVES), dim3(ROUTE_WAVES * KIPP_WAVE), 0, stream, z,
                       parts, (size_t)tokens * stride, stride, correction, chosen, weight, tokens, experts, top, eps, group_count, group_keep,
                       scale);
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, (const int32_t*)chosen, pairs, experts, top, pair_token,
                       place_of_pair, tiles, max_tiles, tile_rows);
    return KIPP_LAUNCH_CHECK();
}

// `tile_rows`: the rows of the tiles that `kipp_moe_route` was asked for: 128 takes the matrix cores (bfloat16 x and w, K a multiple of 32), 16 the plain kernel.
extern "C" int kipp_moe_expert(const void* x, int x_dtype, const int32_t* gather, const void* w, int w_dtype, const int32_t* tiles,
                               int max_tiles, void* out, int out_dtype, int n_out, int k, int act, int tile_rows, hipStream_t stream) {
    if (max_tiles <= 0) return 0;
    if (n_out <= 0 || k <= 0 || act < ACT_NONE || act > ACT_RELU2) return -1;
    if (tile_rows == MFMA_ROWS) {
        if (x_dtype != KIPP_BF16 || w_dtype != KIPP_BF16 || k % 32) return -2;
        // a lane's offsets into x and into an expert's matrix are 32 bits wide
        if ((long long)max_tiles * MFMA_ROWS * k >= (1ll << 31) || (long long)n_out * k >= (1ll << 31)) return -2;
        dim3 grid(max_tiles, (n_out + MFMA_COLS - 1) / MFMA_COLS), block(MFMA_THREADS);
        if (out_dtype == KIPP_BF16)
            hipLaunchKernelGGL((moe_expert_mfma_kernel<bf16_t>), grid, block, 0, stream, (const bf16_t*)x, gather, (const bf16_t*)w, tiles,
                               (bf16_t*)out, n_out, k, act);
        else if (out_dtype == KIPP_F32)
            hipLaunchKernelGGL((moe_expert_mfma_kernel<float>), grid, block, 0, stream, (const bf16_t*)x, gather, (const bf16_t*)w, tiles,
                               (float*)out, n_out, k, act);
        else
            return -2;
        return KIPP_LAUNCH_CHECK();
    }
    if (tile_rows != TILE_ROWS) return -1;
    dim3 grid(max_tiles, (n_out + EXPERT_COLS - 1) / EXPERT_COLS), block(EXPERT_COLS);
#define KIPP_ME(TX, TW, TO)                                                                                                  \
    hipLaunchKernelGGL((moe_expert_kernel<TX, TW, TO>), grid, block, 0, stream, (const TX*)x, gather, (const TW*)w, tiles, \
                       (TO*)out, n_out, k, act)
    if (x_dtype == KIPP_F32 && w_dtype == KIPP_F32 && out_dtype == KIPP_F32) KIPP_ME(float, float, float);
    else if (x_dtype == KIPP_BF16 && w_dtype == KIPP_BF16 && out_dtype == KIPP_BF16) KIPP_ME(bf16_t, bf16_t, bf16_t);
    else if (x_dtype == KIPP_BF16 && w_dtype == KIPP_BF16 && out_dtype == KIPP_F32) KIPP_ME(bf16_t, bf16_t, float);
    else return -2;
#undef KIPP_ME
    return KIPP_LAUNCH_CHECK();
}

extern "C" int kipp_moe_combine(const float* y, const int32_t* place, const float* weight, const float* shared, int shared_parts,
                                float* out, int tokens, int width, int top, hipStream_t stream) {
    if (tokens <= 0) return 0;
    const size_t total = (size_t)tokens * width;
    hipLaunchKernelGGL(moe_combine_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, y, place, weight, shared,
                       shared != nullptr ? shared_parts : 0, total, out, tokens, width, top);
    return KIPP_LAUNCH_CHECK();
}

// out[r][i] = act(sum of the slabs of u[r][i]) [* sum of the slabs of u[r][inner + i] when `glu`]; with `bias` (over u's
// columns) each sum has its column's bias added first
template <typename TO>
__global__ void activate_kernel(const float* __restrict__ u, int parts, size_t part_stride, TO* __restrict__ out, size_t total,
                                int inner, int glu, int act, const float* __restrict__ bias) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t r = i / inner;
    const int c = (int)(i - r * inner);
    const size_t at = glu ? r * 2 * inner + c : i;
    float a = u[at], b = glu ? u[at + inner] : 1.0f;
    for (int p = 1; p < parts; ++p) {
        a += u[p * part_stride + at];
        if (glu) b += u[p * part_stride + at + inner];
    }
    if (bias != nullptr) {
        a += bias[c];
        if (glu) b += bias[inner + c];
    }
    store_f(out, i, glu ? activate(a, act) * b : activate(a, act));
}

extern "C" int kipp_activate_biased(const float* u, int parts, void* out, int out_dtype, int rows, int inner, int glu, int act,
                                    const float* bias, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (inner <= 0 || parts <= 0 || act < ACT_SILU || act > ACT_RELU2) return -1;
    const size_t total = (size_t)rows * inner;
    const size_t part_stride = total * (glu ? 2 : 1);
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (out_dtype == KIPP_F32)
        hipLaunchKernelGGL((activate_kernel<float>), grid, block, 0, stream, u, parts, part_stride, (float*)out, total, inner, glu, act, bias);
    else if (out_dtype == KIPP_BF16)
        hipLaunchKernelGGL((activate_kernel<bf16_t>), grid, block, 0, stream, u, parts, part_stride, (bf16_t*)out, total, inner, glu, act, bias);
    else
        return -2;
    return KIPP_LAUNCH_CHECK();
}

extern "C" int kipp_activate(const float* u, int parts, void* out, int out_dtype, int rows, int inner, int glu, int act,
                             hipStream_t stream) {
    return kipp_activate_biased(u, parts, out, out_dtype, rows, inner, glu, act, nullptr, stream);
}
