// Matrix product for a few dozen rows (decode at larger batches):
// Y[M, N] = X[M, K] . W[N, K]^T, bfloat16 operands, float32 accumulation,
// M <= 256.  Like the few-rows kernel it is bound by reading W once (up to about
// 128 rows; beyond, the matrix cores' work shows), but here
// the rows of X are too many to fetch per wave: every wave would read as much
// of X from L2 as of W from HBM.  So the TW waves of a workgroup share one
// range of K and stage X through LDS in chunks of 256 columns (128 from 65
// rows on, 64 from 129, so that two workgroups still fit a compute unit; double buffered,
// one barrier a chunk), while each wave streams its own 16 rows of W through a
// ring of one chunk's steps in registers.
//
// K is split over `parts` workgroups (grid.y): part p writes slab p of
// Y[parts, M, N]; the consumer adds the slabs in order.
//
// A workgroup has 4 to 8 waves (its size is the launch's, not the kernel's), so that the tiles of W can be
// dealt out to about as many workgroups as there are compute units without splitting K: the SwiGLU end
// (W = [gate; up] in paired tiles, act = silu(gate) * up written straight from the sums) needs the whole of K
// in one workgroup.
//
// v_mfma_f32_16x16x32_bf16: A = W tile (lane: row l % 16, k = 8 (l / 16) + j),
// B = X^T from LDS (lane: token l % 16, same k), D: lane holds features
// 4 (l / 16) + v of token l % 16.
#include "common.h"

#define MAX_ROWS 256

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

union Frag {
    u32x4 u;
    bf16x8 v;
};

// TILED: W in the streaming layout [tile of 16 rows][step of 32 columns][lane][8 values]
// (rows padded to whole tiles with zeros, K a multiple of 32), in which a wave's load is
// one contiguous KB.
// DEPTH: steps of 32 columns in one chunk.  NTW: 16-row tiles of W a wave streams (every fragment of X
// read from LDS then serves NTW products, and a workgroup's staging of X serves NTW times the rows).
// END 1: W is [gate; up] in paired tiles (8 gate rows over the 8 matching up rows), N = 16 tiles' columns, K is not split and
// act[M, inner] = bfloat16(silu(gate) * up) is written instead of Y.
#define MIN_WAVES 4
#define MAX_WAVES 8

template <int MT, bool TILED, int DEPTH, int NTW, int END>
__global__ void __launch_bounds__(MAX_WAVES * KIPP_WAVE) gemm_rows_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, float* __restrict__ Y, bf16_t* __restrict__ act, int M, int N, int K,
    int inner) {
    constexpr int CHUNK = 32 * DEPTH;                          // columns of X staged at a time
    constexpr int X_PITCH = CHUNK + 8;                         // bf16 elements per staged row (the pad spreads the banks)
    constexpr int UNITS = MT * 16 * (CHUNK / 8);              // 16-byte units of one staged chunk
    constexpr int XR = UNITS / (MIN_WAVES * KIPP_WAVE);        // units a thread of the smallest workgroup moves
    static_assert(UNITS % (MIN_WAVES * KIPP_WAVE) == 0, "whole waves stage whole runs of units");
    __shared__ __attribute__((aligned(16))) bf16_t xs[2][MT * 16 * X_PITCH];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int threads = blockDim.x, tw = threads >> 6;         // MIN_WAVES to MAX_WAVES waves
    const int l16 = lane & 15, h = lane >> 4;
    const int n0 = (blockIdx.x * tw + wave) * (16 * NTW);
    const int part = blockIdx.y, parts = gridDim.y;
    const int groups = K / CHUNK;                              // whole chunks; the rest of K goes to the last part
    const int g_begin = (int)((long long)groups * part / parts);
    const int g_end = (int)((long long)groups * (part + 1) / parts);

    const bf16_t* w_row[NTW];                                  // clamped: in bounds, dropped at the store
#pragma unroll
    for (int i = 0; i < NTW; ++i)
        w_row[i] = TILED ? W + (size_t)min((n0 >> 4) + i, (N + 15) / 16 - 1) * (K / 32) * 512 + lane * 8
                         : W + (size_t)min(n0 + 16 * i + l16, N - 1) * K + 8 * h;

    // the units of X this thread stages: unit -> (row, 8-column chunk); a larger workgroup has fewer a thread
    const bf16_t* x_src[XR];
    int x_dst[XR];
    bool x_mine[XR];
#pragma unroll
    for (int i = 0; i < XR; ++i) {
        const int unit = tid + i * threads;
        x_mine[i] = unit < UNITS;
        const int r = min(unit, UNITS - 1) / (CHUNK / 8), c = unit % (CHUNK / 8);
        x_src[i] = X + (size_t)min(r, M - 1) * K + c * 8;
        x_dst[i] = r * X_PITCH + c * 8;
    }

    f32x4 acc[NTW][MT];
#pragma unroll
    for (int i = 0; i < NTW; ++i)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[i][mt] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    Frag wf[DEPTH][NTW];
    u32x4 xr[XR];

    auto fetch_w = [&](int u, int step) {
#pragma unroll
        for (int i = 0; i < NTW; ++i) wf[u][i].u = *(const u32x4*)(w_row[i] + (TILED ? 512 : 32) * step);
    };
    auto fetch_x = [&](int g) {
#pragma unroll
        for (int i = 0; i < XR; ++i)
            if (x_mine[i]) xr[i] = *(const u32x4*)(x_src[i] + (size_t)g * CHUNK);
    };
    auto stage_x = [&](int buf) {
#pragma unroll
        for (int i = 0; i < XR; ++i)
            if (x_mine[i]) *(u32x4*)(xs[buf] + x_dst[i]) = xr[i];
    };
    auto multiply = [&](int u, int buf) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            Frag xf;
            xf.u = *(const u32x4*)(xs[buf] + (mt * 16 + l16) * X_PITCH + 32 * u + 8 * h);
#pragma unroll
            for (int i = 0; i < NTW; ++i) acc[i][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][i].v, xf.v, acc[i][mt], 0, 0, 0);
        }
    };

    // The last chunk stands outside the loop, so that inside it every load has a fixed
    // place in the order of the loads in flight and no wait covers more than it must.
    if (g_begin < g_end) {
        fetch_x(g_begin);                             // asked for first: needed first
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) fetch_w(u, g_begin * DEPTH + u);
        stage_x(0);
        __syncthreads();
        int buf = 0;
        for (int g = g_begin; g + 1 < g_end; ++g) {
            fetch_x(g + 1);
#pragma unroll
            for (int u = 0; u < DEPTH; ++u) {
                multiply(u, buf);
                fetch_w(u, (g + 1) * DEPTH + u);
                __builtin_amdgcn_sched_barrier(0);    // keep the load here: the compiler would gather all eight after the products
            }
            stage_x(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) multiply(u, buf);
    }
    // the rest of K (less than a chunk), by the last part, straight from global memory
    if (part == parts - 1) {
        for (int k = groups * CHUNK; k < K; k += 32) {
            const bool ok = k + 8 * h < K;
            Frag w_t[NTW];
#pragma unroll
            for (int i = 0; i < NTW; ++i) {
                w_t[i].u = (u32x4){0u, 0u, 0u, 0u};
                if (ok) w_t[i].u = *(const u32x4*)(w_row[i] + (TILED ? 16 * k : k));
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                Frag x_t;
                x_t.u = (u32x4){0u, 0u, 0u, 0u};
                if (ok) x_t.u = *(const u32x4*)(X + (size_t)min(16 * mt + l16, M - 1) * K + 8 * h + k);
#pragma unroll
                for (int i = 0; i < NTW; ++i) acc[i][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_t[i].v, x_t.v, acc[i][mt], 0, 0, 0);
            }
        }
    }
    if (END == 1) {
        // rows 0..7 of a tile are gates, rows 8..15 the matching ups: they sit 32 lanes apart
#pragma unroll
        for (int i = 0; i < NTW; ++i) {
            const int o = (n0 / 2) + 8 * i + 4 * h;                // first of this lane's four features (lane groups 0 and 1)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                const int token = 16 * mt + l16;
                float a[4];
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const float g = acc[i][mt][v], up = __shfl_xor(g, 32, KIPP_WAVE);
                    a[v] = g / (1.0f + expf(-g)) * up;
                }
                if (h >= 2 || token >= M) continue;
                bf16_t* out = act + (size_t)token * inner + o;
                if (o + 3 < inner && (inner & 3) == 0) {
                    uint2 packed;
                    packed.x = (uint32_t)f32_to_bf16(a[0]) | ((uint32_t)f32_to_bf16(a[1]) << 16);
                    packed.y = (uint32_t)f32_to_bf16(a[2]) | ((uint32_t)f32_to_bf16(a[3]) << 16);
                    *(uint2*)out = packed;
                } else {
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (o + v < inner) out[v] = f32_to_bf16(a[v]);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < NTW; ++i) {
        const int n = n0 + 16 * i + 4 * h;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int token = 16 * mt + l16;
            if (token >= M) continue;
            float* y = Y + ((size_t)part * M + token) * N + n;
            if (n + 3 < N && (N & 3) == 0) {
                *(float4*)y = make_float4(acc[i][mt][0], acc[i][mt][1], acc[i][mt][2], acc[i][mt][3]);
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < N) y[v] = acc[i][mt][v];
            }
        }
    }
}

// Tiles of 16 rows of W per workgroup (4 to 8 waves with one tile each, or 5 to 8 waves with two) and parts of
// K, from the shape only.  A compute unit draws a bounded number of bytes a second, so the workgroups run
// in rounds of 256 and a round costs what one workgroup reads, its rows of W and (from L2, at about a
// quarter of the price a row) all rows of X, plus a fixed start; the plan takes the cheapest rounds, with a
// small charge for every slab the consumer has to add and every part at least one whole chunk.  (Fitted to
// sweeps over these splits at 32, 64 and 128 rows: the more rows X has, the larger the workgroups.)
static int chunk_of(int M) { return M > 128 ? 64 : (M > 64 ? 128 : 256); }

static double plan(int M, int N, int K, int max_parts, int* tw, int* ntw, int* parts) {
    static const int tiles_of_a_workgroup[] = {4, 5, 6, 7, 8, 10, 12, 14, 16};
    const int tiles = (N + 15) / 16;
    const int groups = K / chunk_of(M) > 0 ? K / chunk_of(M) : 1;
    double best = 1e300;
    *tw = 4;
    *ntw = 1;
    *parts = 1;
    for (int t : tiles_of_a_workgroup) {
        const int cols = (tiles + t - 1) / t;
        for (int p = 1; p <= max_parts && p <= groups; ++p) {
            const int rounds = (cols * p + 255) / 256;
            const double cost = rounds * ((t + 0.27 * M / 16.0) * (double)K / p + 150.0 * t) * (1.0 + 0.02 * p);
            if (cost < best * 0.999) {
                best = cost;
                *tw = t > 8 ? t / 2 : t;
                *ntw = t > 8 ? 2 : 1;
                *parts = p;
            }
        }
    }
    return best;
}

// `cut` (for measurements and tests): 10 x waves + tiles a wave, with exactly max_parts parts of K (as many as K has chunks).
static int cut_or_plan(int M, int N, int K, int max_parts, int cut, int* tw, int* ntw, int* parts) {
    if (cut == 0) {
        plan(M, N, K, max_parts, tw, ntw, parts);
        return 0;
    }
    *tw = cut / 10;
    *ntw = cut % 10;
    const int groups = K / chunk_of(M) > 0 ? K / chunk_of(M) : 1;
    *parts = max_parts < groups ? max_parts : groups;
    return (*tw < MIN_WAVES || *tw > MAX_WAVES || *ntw < 1 || *ntw > 2) ? -1 : 0;
}

template <int END>
static int launch(const void* X, const void* W, float* Y, void* act, int M, int N, int K, int inner, int tw, int ntw, int parts,
                  int tiled, hipStream_t stream) {
    const int tiles = (N + 15) / 16;
    dim3 grid((tiles + tw * ntw - 1) / (tw * ntw), parts), block(tw * KIPP_WAVE);
    const int mt = (M + 15) / 16;       // from 65 rows on an even number of 16-row tiles is staged (whole waves move whole runs of units)
#define KIPP_GR(MT, DEPTH, NTW)                                                                                          \
    do {                                                                                                                 \
        if (tiled)                                                                                                       \
            hipLaunchKernelGGL((gemm_rows_kernel<MT, true, DEPTH, NTW, END>), grid, block, 0, stream, (const bf16_t*)X,  \
                               (const bf16_t*)W, Y, (bf16_t*)act, M, N, K, inner);                                       \
        else if (END == 0)                                                                                               \
            hipLaunchKernelGGL((gemm_rows_kernel<MT, false, DEPTH, NTW, 0>), grid, block, 0, stream, (const bf16_t*)X,   \
                               (const bf16_t*)W, Y, (bf16_t*)act, M, N, K, inner);                                       \
        else                                                                                                             \
            return -1;                                                                                                   \
    } while (0)
#define KIPP_GR_NTW(NTW)                   \
    switch (mt) {                          \
        case 1: KIPP_GR(1, 8, NTW); break; \
        case 2: KIPP_GR(2, 8, NTW); break; \
        case 3: KIPP_GR(3, 8, NTW); break; \
        case 4: KIPP_GR(4, 8, NTW); break; \
        case 5:                            \
        case 6: KIPP_GR(6, 4, NTW); break; \
        case 7:                            \
        case 8: KIPP_GR(8, 4, NTW); break; \
        case 9:                            \
        case 10:                           \
        case 11:                           \
        case 12: KIPP_GR(12, 2, NTW); break; \
        case 13:                           \
        case 14:                           \
        case 15:                           \
        case 16: KIPP_GR(16, 2, NTW); break; \
        default: return -1;                \
    }
    if (ntw == 2) {
        KIPP_GR_NTW(2)
    } else {
        KIPP_GR_NTW(1)
    }
#undef KIPP_GR_NTW
#undef KIPP_GR
    return KIPP_LAUNCH_CHECK();
}

extern "C" {

int kipp_gemm_rows_max_rows() { return MAX_ROWS; }

int kipp_gemm_rows_parts(int M, int N, int K, int max_parts) {
    int tw, ntw, parts;
    plan(M, N, K, max_parts, &tw, &ntw, &parts);
    return parts;
}

// Y: float32 [parts, M, N] with parts = kipp_gemm_rows_parts(M, N, K, max_parts).
// M <= 256, K a multiple of 8; `tiled`: W in the streaming layout (K a multiple of 32).
int kipp_gemm_rows(const void* X, const void* W, float* Y, int M, int N, int K, int max_parts, int tiled, int cut,
                   hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > MAX_ROWS || K <= 0 || (K & 7) || max_parts <= 0 || (tiled && (K & 31))) return -1;
    int tw, ntw, parts;
    if (cut_or_plan(M, N, K, max_parts, cut, &tw, &ntw, &parts) != 0) return -1;
    return launch<0>(X, W, Y, nullptr, M, N, K, 0, tw, ntw, parts, tiled, stream);
}

// Whether the product that ends in SwiGLU is taken for this shape: K is not split there, and where the tiles of W are
// too few for that (or leave most of a round of workgroups idle) the split product and an activation kernel are faster.
int kipp_gemm_rows_swiglu_pays(int M, int two_inner, int K) {
    if (M <= 0 || M > MAX_ROWS || two_inner <= 0 || (two_inner & 1) || K <= 0 || (K & 31)) return 0;
    // beyond 64 rows the activation's arithmetic at the end of every workgroup costs what the second launch does (measured at
    // 2560 x 19456: 2 to 3 us saved of 23 to 27 up to 64 rows, nothing from 80 rows on)
    if (M > 64) return 0;
    const int N = 16 * ((two_inner / 2 + 7) / 8);
    int tw, ntw, parts;
    const double whole = plan(M, N, K, 1, &tw, &ntw, &parts), split = plan(M, N, K, 12, &tw, &ntw, &parts);
    // the split product's slabs are written, read again and the activation is a launch of its own: about a fifth of its time
    return whole <= 1.2 * split;
}

// act: bfloat16 [M, I] = silu(X . gate^T) * (X . up^T); W: the paired tiles of [gate; up] ([2 I, K], tiles of 8 gate rows
// over the 8 matching up rows, K a multiple of 32).
int kipp_gemm_rows_swiglu(const void* X, const void* W, void* act, int M, int two_inner, int K, int cut, hipStream_t stream) {
    if (M <= 0 || two_inner <= 0) return 0;
    if (M > MAX_ROWS || K <= 0 || (K & 31) || (two_inner & 1)) return -1;
    const int inner = two_inner / 2, N = 16 * ((inner + 7) / 8);
    int tw, ntw, parts;
    if (cut_or_plan(M, N, K, 1, cut, &tw, &ntw, &parts) != 0 || parts != 1) return -1;
    return launch<1>(X, W, nullptr, act, M, N, K, inner, tw, ntw, 1, 1, stream);
}

}  // extern "C"
