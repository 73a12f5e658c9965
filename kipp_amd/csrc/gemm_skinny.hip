// Matrix product for few rows (decode): Y[M, N] = X[M, K] . W[N, K]^T with
// bfloat16 operands, float32 accumulation, M <= 64.  The cost is reading W
// once from HBM, so everything serves one aim: many 16-byte loads of W in
// flight in every wave, all the time.
//
// A wave owns 16 rows of W and a slice of K.  It keeps a ring of DEPTH steps
// (32 columns each) in registers: while the matrix core works on step s, the
// loads of steps s+1 .. s+DEPTH are on their way (plain loads: streaming hints made this
// access pattern slower in measurements).  The 4 waves of a workgroup
// are KW slices of K times 4/KW row tiles; slices are added in LDS in slice
// order.  `parts` > 1 splits K over workgroups as well (for products with few
// output rows): part p writes its own [M, N] slab and the consumer adds the
// slabs in order, so there are no atomics and the same bits come out every run.
//
// v_mfma_f32_16x16x32_bf16: A = W tile (lane: row l % 16, k = 8 (l / 16) + j),
// B = X^T (lane: token l % 16, same k), D: lane holds features 4 (l / 16) + v of
// token l % 16, i.e. 16 contiguous bytes of a Y row.
//
// TILED: W comes in the streaming layout, in which the 1 KB that a wave reads in
// one step (16 rows x 32 columns) is contiguous: [tile of 16 rows][step of 32
// columns][lane][8 values], lane l holding row l % 16, columns 8 (l / 16) .. + 7 of
// the step; rows are padded to whole tiles with zeros and K is a multiple of 32.
// Every request then covers full memory lines, which a compute unit issues at a
// bounded rate: the same kernel streams a fifth faster than from [N, K] rows.
//
// With SWIGLU the weight is [gate rows; up rows] ([2 I, K]) and the kernel writes
// silu(gate) * up as bfloat16 [M, I]  (/root/reference/src/kipp.c:2644-2648).
// From rows, a wave computes a gate tile and the matching up tile together.  In
// the streaming layout the two lie in ONE tile, 8 gate rows over the 8 matching
// up rows, so a wave has 8 outputs: there are twice as many, half as heavy
// workgroups, which fill the last round of 256 better (9,728 outputs: 4.75
// rounds instead of 2.4, so 5 % lost instead of 26 %).
//
// Two optional ends spare the decode step its norm kernels (a launch costs more than the
// norm's work there).  `AddNorm`: the product is a delta of the residual stream and is not
// split over workgroups; the wave that holds a tile's sums adds the residual, writes the new
// residual, its product with the next norm's weight as bfloat16, and the sum of squares of
// every row over the tile's 16 columns.  (Split over workgroups, the last to arrive would
// have to add the slabs: the device-wide fences that takes cost several times the kernel,
// measured 27 instead of 6 microseconds.)  `RowScale`: X holds such rows; the kernel sums a
// row's partial sums and multiplies the row of the product by rsqrt(sum / K + eps), which is
// the product of the normalized row (the scale of a row commutes with the contraction).
#include "common.h"

#define WAVES 4
#define THREADS (WAVES * KIPP_WAVE)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

union Frag {
    u32x4 u;
    bf16x8 v;
};

struct RowScale {               // sumsq == nullptr: none
    const float* sumsq;         // [M, stride]: `parts` partial sums of squares of each row X was made from
    int parts, stride;          // stride: parts rounded up to a multiple of 4, so that a lane loads four sums at once
    float inv_width, eps;
};

struct AddNorm {                // residual == nullptr: none
    float* residual;            // [M, N], updated in place
    const float* norm_w;        // [N]
    bf16_t* rows_out;           // [M, N] = bfloat16(residual * norm_w)
    float* sumsq_out;           // [M, stride]: ceil(N / 16) sums a row, stride as in RowScale
    int stride;
    int steps_major;            // rows_out as [N / 32][M][32] (N a multiple of 32)
};

// Where element (row, column) of bfloat16 rows lies: [row][width], or [column / 32][row][32] for `rows` rows.
__device__ __forceinline__ size_t rows_at(int row, int col, int width, int rows, int steps_major) {
    return steps_major ? ((size_t)(col >> 5) * rows + row) * 32 + (col & 31) : (size_t)row * width + col;
}

#define SCALE_LOADS 10          // 16-byte loads of partial sums a lane has in flight: 160 sums of a row, what 2,560 columns give

template <int MT, bool SWIGLU, int KW, int DEPTH, bool TILED>
__global__ void __launch_bounds__(THREADS) gemm_skinny_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, float* Y, bf16_t* __restrict__ act,
    int M, int N, int K, RowScale rs, AddNorm an, int x_major, int act_major) {
    constexpr bool PAIRS = SWIGLU && TILED;          // gate and up rows share a tile
    constexpr int NT = SWIGLU && !TILED ? 2 : 1;
    constexpr int TW = WAVES / KW;                   // row tiles of a workgroup
    __shared__ float red[KW > 1 ? WAVES : 1][NT][MT][256];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: the loop bounds below are scalars
    const int l16 = lane & 15, h = lane >> 4;
    const int tile_in_wg = wave / KW, slice = wave % KW;
    const int n0 = (blockIdx.x * TW + tile_in_wg) * 16;
    const int part = blockIdx.y;
    const int inner = SWIGLU ? N / 2 : N;            // rows of one of the stacked matrices
    const int out0 = PAIRS ? n0 / 2 : n0;            // first output feature of the tile
    // The contraction in groups of DEPTH steps of 32 columns.  Groups are dealt out evenly to
    // the gridDim.y * KW slices; what is left beyond the last whole group (fewer than DEPTH
    // steps and a rest of 8, 16 or 24 columns) goes to the very last slice.
    const int full_steps = K / 32;
    const int groups = full_steps / DEPTH;
    const int slices = (int)gridDim.y * KW;
    const int my_slice = part * KW + slice;
    const int g_begin = (int)((long long)groups * my_slice / slices);
    const int g_end = (int)((long long)groups * (my_slice + 1) / slices);

    const bool row_ok = n0 + l16 < inner;
    const int row = row_ok ? n0 + l16 : 0;           // clamped: the loads stay in bounds, the result is dropped
    const bf16_t* w_row[NT];
    if (TILED) {
        // a tile index beyond the last (the grid is rounded up) is clamped and dropped
        const int tiles = PAIRS ? (inner + 7) / 8 : (inner + 15) / 16;
        const size_t tile = (size_t)min(n0 >> 4, tiles - 1);
        w_row[0] = W + tile * full_steps * 512 + lane * 8;
    } else {
        w_row[0] = W + (size_t)row * K + 8 * h;
        if (SWIGLU) w_row[NT - 1] = W + (size_t)(inner + row) * K + 8 * h;
    }
    const bf16_t* x_row[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) x_row[mt] = X + (size_t)min(16 * mt + l16, M - 1) * (x_major ? 32 : K) + 8 * h;
    const int x_step = x_major ? 32 * M : 32;        // from one step's columns of a row to the next step's

    // the partial sums of the rows' scales, asked for first, all at once, and added once the first
    // weights are on their way (up to 16 rows): lane group h takes every fourth run of four sums of token l % 16.
    // Of the waves that share a tile one does this for all (the one of the second slice; the scale is wanted
    // after the slices have met in LDS anyway): every load a compute unit issues counts against the weights'.
    __shared__ float s_scale[KW > 1 ? TW : 1][16];
    float4 scale_part[MT == 1 ? SCALE_LOADS : 1];
    const float* scale_src = nullptr;
    if (MT == 1 && rs.sumsq != nullptr && (KW == 1 || slice == 1)) {
        scale_src = rs.sumsq + (size_t)min(l16, M - 1) * rs.stride;
#pragma unroll
        for (int i = 0; i < SCALE_LOADS; ++i)   // beyond the last run: read the last again, dropped below
            scale_part[i] = *(const float4*)(scale_src + min(4 * (h + 4 * i), rs.stride - 4));
        __builtin_amdgcn_sched_barrier(0);
    }

    // what the residual end adds to, asked for first as well (nobody writes these elements before that end does)
    const bool wide = (N & 3) == 0;                  // a lane's four columns are 16 aligned bytes
    float res[MT][4], norm_w[4];
    if (!SWIGLU && an.residual != nullptr && slice == 0) {       // the wave that will hold the tile's sums
        const int col = min(n0 + 4 * h, wide ? N - 4 : N - 1);
        if (wide) {
            const float4 w4 = *(const float4*)(an.norm_w + col);
            norm_w[0] = w4.x, norm_w[1] = w4.y, norm_w[2] = w4.z, norm_w[3] = w4.w;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const float4 r4 = *(const float4*)(an.residual + (size_t)min(16 * mt + l16, M - 1) * N + col);
                res[mt][0] = r4.x, res[mt][1] = r4.y, res[mt][2] = r4.z, res[mt][3] = r4.w;
            }
        } else {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int c = min(n0 + 4 * h + v, N - 1);
                norm_w[v] = an.norm_w[c];
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) res[mt][v] = an.residual[(size_t)min(16 * mt + l16, M - 1) * N + c];
            }
        }
    }

    f32x4 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

    Frag wf[DEPTH][NT], xf[DEPTH][MT];
    // No value is touched between its load and its product: the loads stay in flight.
    auto fetch = [&](int u, int step) {
        const int k = 32 * step;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wf[u][nt].u = *(const u32x4*)(w_row[nt] + (TILED ? 512 * step : k));
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xf[u][mt].u = *(const u32x4*)(x_row[mt] + (size_t)step * x_step);
    };
    auto multiply = [&](int u) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][nt].v, xf[u][mt].v, acc[nt][mt], 0, 0, 0);
    };

    // the rows' scales: added up once the first weights have been asked for (asked for first, the partial sums
    // arrive first, and the weights are on their way meanwhile).  The sum starts from a zero that exists only
    // after those requests, or the compiler would add before it asks for the weights and the wave would wait idle;
    // and it stands in the same block as those requests, so that the wait counts them and is not for all of them.
    float row_scale[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) row_scale[mt] = 1.0f;
    auto finish_scale = [&]() {
        if (MT == 1 && scale_src != nullptr) {
            float t;
            asm volatile("v_mov_b32 %0, 0" : "=v"(t) : : "memory");
#pragma unroll
            for (int i = 0; i < SCALE_LOADS; ++i) {
                const int p = 4 * (h + 4 * i);
                t += p < rs.parts ? scale_part[i].x : 0.0f;
                t += p + 1 < rs.parts ? scale_part[i].y : 0.0f;
                t += p + 2 < rs.parts ? scale_part[i].z : 0.0f;
                t += p + 3 < rs.parts ? scale_part[i].w : 0.0f;
            }
            for (int p0 = 16 * SCALE_LOADS; p0 < rs.parts; p0 += 16 * SCALE_LOADS) {   // wider rows: as many again at a time
                float4 more[SCALE_LOADS];
#pragma unroll
                for (int i = 0; i < SCALE_LOADS; ++i) more[i] = *(const float4*)(scale_src + min(p0 + 4 * (h + 4 * i), rs.stride - 4));
#pragma unroll
                for (int i = 0; i < SCALE_LOADS; ++i) {
                    const int p = p0 + 4 * (h + 4 * i);
                    t += p < rs.parts ? more[i].x : 0.0f;
                    t += p + 1 < rs.parts ? more[i].y : 0.0f;
                    t += p + 2 < rs.parts ? more[i].z : 0.0f;
                    t += p + 3 < rs.parts ? more[i].w : 0.0f;
                }
            }
            t += __shfl_xor(t, 16, KIPP_WAVE);     // the four lane groups of a token
            t += __shfl_xor(t, 32, KIPP_WAVE);
            row_scale[0] = 1.0f / sqrtf(t * rs.inv_width + rs.eps);
            if (KW > 1 && h == 0) s_scale[tile_in_wg][l16] = row_scale[0];
        }
    };
    if (g_begin >= g_end) finish_scale();
    if (g_begin < g_end) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) fetch(u, g_begin * DEPTH + u);
        finish_scale();
        for (int g = g_begin; g + 1 < g_end; ++g) {      // while step s is multiplied, step s + DEPTH is fetched
#pragma unroll
            for (int u = 0; u < DEPTH; ++u) {
                multiply(u);
                fetch(u, (g + 1) * DEPTH + u);
                __builtin_amdgcn_sched_barrier(0);    // keep the loads here: the compiler would gather them after the products
            }
        }
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) multiply(u);
    }
    // what is left of K, by the last slice: whole steps one at a time, then the rest with a mask
    if (my_slice == slices - 1) {
        for (int step = groups * DEPTH; step < full_steps; ++step) {
            fetch(0, step);
            multiply(0);
        }
        if (!TILED && (K & 31) != 0) {
            const int k = 32 * full_steps;
            const bool ok = k + 8 * h < K;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                wf[0][nt].u = (u32x4){0u, 0u, 0u, 0u};
                if (ok) wf[0][nt].u = *(const u32x4*)(w_row[nt] + k);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                xf[0][mt].u = (u32x4){0u, 0u, 0u, 0u};
                if (ok) xf[0][mt].u = *(const u32x4*)(x_row[mt] + k);
            }
            multiply(0);
        }
    }
    // tokens beyond M and rows beyond N were computed from clamped addresses and are dropped below

    float sum[NT][MT][4];
    bool writer = true;                               // this wave holds finished sums
    if (KW > 1) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) red[wave][nt][mt][lane * 4 + v] = acc[nt][mt][v];
        __syncthreads();
        writer = slice == 0;
        if (MT == 1 && rs.sumsq != nullptr) row_scale[0] = s_scale[tile_in_wg][l16];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float a = 0.0f;
                    if (writer) {
#pragma unroll
                        for (int w = 0; w < KW; ++w) a += red[tile_in_wg * KW + w][nt][mt][lane * 4 + v];
                    }
                    sum[nt][mt][v] = a * row_scale[mt];
                }
    } else {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) sum[nt][mt][v] = acc[nt][mt][v] * row_scale[mt];
    }
    const int n = n0 + 4 * h;
    if (!SWIGLU && an.residual != nullptr) {
        // ---- the product is a delta of the residual stream (never split over workgroups: the launcher sees to it)
        if (!writer) return;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int token = 16 * mt + l16;
            float x[4], ss = 0.0f;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                x[v] = res[mt][v] + sum[0][mt][v];
                if (token < M && n + v < N) ss = fmaf(x[v], x[v], ss);
            }
            if (token < M && wide && n + 3 < N) {
                const size_t at = (size_t)token * N + n;
                *(float4*)(an.residual + at) = make_float4(x[0], x[1], x[2], x[3]);
                uint2 packed;
                packed.x = (uint32_t)f32_to_bf16(x[0] * norm_w[0]) | ((uint32_t)f32_to_bf16(x[1] * norm_w[1]) << 16);
                packed.y = (uint32_t)f32_to_bf16(x[2] * norm_w[2]) | ((uint32_t)f32_to_bf16(x[3] * norm_w[3]) << 16);
                *(uint2*)(an.rows_out + rows_at(token, n, N, M, an.steps_major)) = packed;   // four columns of one run of 32
            } else if (token < M) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    if (n + v < N) {
                        an.residual[(size_t)token * N + n + v] = x[v];
                        an.rows_out[rows_at(token, n + v, N, M, an.steps_major)] = f32_to_bf16(x[v] * norm_w[v]);
                    }
                }
            }
            ss += __shfl_xor(ss, 16, KIPP_WAVE);      // the four lane groups hold a tile's 16 columns of a token
            ss += __shfl_xor(ss, 32, KIPP_WAVE);
            if (h == 0 && token < M && n0 < N) an.sumsq_out[(size_t)token * an.stride + (n0 >> 4)] = ss;
        }
        return;
    }
    if (!writer) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int token = 16 * mt + l16;
        if (PAIRS) {
            // rows 0..7 of the tile are gates, rows 8..15 the matching ups: they sit 32 lanes apart
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float g = sum[0][mt][v], up = __shfl_xor(g, 32, KIPP_WAVE);
                const int o = out0 + 4 * h + v;
                if (h < 2 && token < M && o < inner) act[rows_at(token, o, inner, M, act_major)] = f32_to_bf16(g / (1.0f + expf(-g)) * up);
            }
            continue;
        }
        if (token >= M) continue;
        if (SWIGLU) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if (n + v < inner) {
                    const float g = sum[0][mt][v], up = sum[NT - 1][mt][v];
                    act[rows_at(token, n + v, inner, M, act_major)] = f32_to_bf16(g / (1.0f + expf(-g)) * up);
                }
            }
        } else {
            float* y = Y + ((size_t)part * M + token) * N + n;
            if (n + 3 < N && (N & 3) == 0) {
                *(float4*)y = make_float4(sum[0][mt][0], sum[0][mt][1], sum[0][mt][2], sum[0][mt][3]);
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < N) y[v] = sum[0][mt][v];
            }
        }
    }
}

template <bool SWIGLU, int KW, bool TILED>
static int launch_kw(const bf16_t* X, const bf16_t* W, float* Y, bf16_t* act, int M, int N, int K, int parts,
                     RowScale rs, AddNorm an, int x_major, int act_major, hipStream_t stream) {
    const int inner = SWIGLU ? N / 2 : N;
    const int tiles = SWIGLU && TILED ? (inner + 7) / 8 : (inner + 15) / 16;
    constexpr int TW = WAVES / KW;
    dim3 grid((tiles + TW - 1) / TW, parts), block(THREADS);
    if (an.residual != nullptr && parts != 1) return -1;
    if (rs.sumsq != nullptr && M > 16) return -1;
    const int mt = (M + 15) / 16;
#define KIPP_SK(MT, D) \
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, SWIGLU, KW, D, TILED>), grid, block, 0, stream, X, W, Y, act, M, N, K, rs, an, x_major, \
                       act_major)
    switch (mt) {
        case 1:
            // fewer workgroups than compute units: what is in flight is what the busy ones ask for, so they ask for twice as much
            if (grid.x * grid.y < 256 && K / 32 / 16 >= KW) KIPP_SK(1, 16);
            else KIPP_SK(1, 8);
            break;
        case 2: KIPP_SK(2, 8); break;
        case 3: KIPP_SK(3, 4); break;
        case 4: KIPP_SK(4, 4); break;
        default: return -1;
    }
#undef KIPP_SK
    return KIPP_LAUNCH_CHECK();
}

template <bool SWIGLU>
static int launch(const bf16_t* X, const bf16_t* W, float* Y, bf16_t* act, int M, int N, int K, int parts, int kw,
                  int tiled, RowScale rs, AddNorm an, int x_major, int act_major, hipStream_t stream) {
    if (tiled && (K & 31)) return -1;
    if (x_major && (K & 31)) return -1;              // whole runs of 32 columns only
    if (an.residual != nullptr && an.steps_major && (N & 31)) return -1;
    if (act_major && ((N / 2) & 31)) return -1;
#define KIPP_KW(KW)                                                                          \
    return tiled ? launch_kw<SWIGLU, KW, true>(X, W, Y, act, M, N, K, parts, rs, an, x_major, act_major, stream)         \
                 : launch_kw<SWIGLU, KW, false>(X, W, Y, act, M, N, K, parts, rs, an, x_major, act_major, stream)
    switch (kw) {
        case 1: KIPP_KW(1);
        case 2: KIPP_KW(2);
        case 4: KIPP_KW(4);
        default: return -1;
    }
#undef KIPP_KW
}

// How the contraction is split: `kw` slices inside a workgroup and `parts` across
// workgroups.  A compute unit draws a bounded number of bytes a second however many
// waves ask, so what counts is that all 256 of them stream all the time: the
// workgroups run in rounds of 256, and a round costs what one workgroup reads plus
// a fixed start.  The plan takes the split with the cheapest rounds (each slice at
// least one whole group of 8 steps, a small charge for every slab the consumer has
// to add).  A function of the shape only, never of the data.
static void plan(int tiles, int K, int max_parts, int* kw, int* parts) {
    const int groups = K / 32 / 8 > 0 ? K / 32 / 8 : 1;
    const double start = 300.0;                       // a workgroup's fixed cost, in columns of its rows
    double best = 1e300;
    *kw = 1;
    *parts = 1;
    for (int k = 4; k >= 1; k /= 2) {
        const int tw = WAVES / k;
        const int cols = (tiles + tw - 1) / tw;
        for (int p = 1; p <= max_parts && k * p <= groups; ++p) {
            const int rounds = (cols * p + 255) / 256;
            const double cost = rounds * (tw * (double)K / p + start) * (1.0 + 0.02 * p);
            if (cost < best * 0.999) {
                best = cost;
                *kw = k;
                *parts = p;
            }
        }
    }
}

extern "C" {

// Slabs the product of this shape comes in when the caller allows up to `max_parts`.
int kipp_gemm_skinny_parts(int N, int K, int max_parts) {
    int kw, parts;
    plan((N + 15) / 16, K, max_parts, &kw, &parts);
    return parts;
}

// Floats of a row of `parts` partial sums: whole runs of four.
static int sumsq_stride(int parts) { return (parts + 3) / 4 * 4; }

static RowScale row_scale_of(const float* sumsq, int sumsq_parts, int K, float eps) {
    RowScale rs = {sumsq, sumsq_parts, sumsq_stride(sumsq_parts), 1.0f / (float)K, eps};
    return rs;
}

// Floats of a row of the partial sums a product of N columns writes (ceil(N / 16) sums, in whole runs of four).
int kipp_gemm_skinny_sumsq_stride(int N) { return sumsq_stride((N + 15) / 16); }

// Y: float32 [parts, M, N] with parts = kipp_gemm_skinny_parts(N, K, max_parts).
// K must be a multiple of 8 (16-byte loads), M <= 64.  `tiled`: W is in the
// streaming layout (K a multiple of 32), else [N, K] rows.
// `sumsq` [M, sumsq_parts rounded up to a multiple of 4] (or null; M <= 16 then): every row of the product is multiplied by
// rsqrt(sum of the row's sumsq / K + eps).
// `x_steps_major`: X comes as [K / 32][M][32] (K a multiple of 32); `rows_out_steps_major`: rows_out is written as
// [N / 32][M][32] (N a multiple of 32).
// `residual` [M, N] (or null): the product is added to it in place (Y is not written and there is
// one part), `rows_out` [M, N] = bfloat16(residual * norm_w) and `sumsq_out`
// [M, kipp_gemm_skinny_sumsq_stride(N)] = every row's sums of squares of the new residual over each 16 columns
// (M <= 16 with a residual).
int kipp_gemm_skinny(const void* X, const void* W, float* Y, int M, int N, int K, int max_parts, int tiled,
                     const float* sumsq, int sumsq_parts, float eps, float* residual, const float* norm_w, void* rows_out,
                     float* sumsq_out, int x_steps_major, int rows_out_steps_major, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || (K & 7) || max_parts <= 0) return -1;
    if (sumsq != nullptr && (sumsq_parts <= 0 || M > 16)) return -1;
    if (residual != nullptr && (norm_w == nullptr || rows_out == nullptr || sumsq_out == nullptr || M > 16)) return -1;
    int kw, parts;
    plan((N + 15) / 16, K, residual != nullptr ? 1 : max_parts, &kw, &parts);
    AddNorm an = {residual, norm_w, (bf16_t*)rows_out, sumsq_out, sumsq_stride((N + 15) / 16), rows_out_steps_major};
    return launch<false>((const bf16_t*)X, (const bf16_t*)W, Y, nullptr, M, N, K, parts, kw, tiled,
                         row_scale_of(sumsq, sumsq_parts, K, eps), an, x_steps_major, 0, stream);
}

// W: [2 I, K] = [gate; up] (tiled: tiles of 8 gate rows over the 8 matching up rows); act: bfloat16 [M, I].
// The contraction is cut the same way from both layouts, so both give the same bits.
// `sumsq`, `sumsq_parts`, `eps`, `x_steps_major`: as above; `act_steps_major`: act is written as [I / 32][M][32] (I a multiple of 32).
int kipp_gemm_skinny_swiglu(const void* X, const void* W, void* act, int M, int two_inner, int K, int tiled,
                            const float* sumsq, int sumsq_parts, float eps, int x_steps_major, int act_steps_major,
                            hipStream_t stream) {
    if (M <= 0 || two_inner <= 0) return 0;
    if (M > 64 || K <= 0 || (K & 7) || (two_inner & 1)) return -1;
    if (sumsq != nullptr && (sumsq_parts <= 0 || M > 16)) return -1;
    int kw, parts;
    plan((two_inner / 2 + 7) / 8, K, 1, &kw, &parts);
    AddNorm none = {nullptr, nullptr, nullptr, nullptr, 4, 0};
    return launch<true>((const bf16_t*)X, (const bf16_t*)W, nullptr, (bf16_t*)act, M, two_inner, K, 1, kw, tiled,
                        row_scale_of(sumsq, sumsq_parts, K, eps), none, x_steps_major, act_steps_major, stream);
}

}  // extern "C"
