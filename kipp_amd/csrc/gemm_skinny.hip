// Matrix product for few rows (decode): Y[M, N] = X[M, K] . W[N, K]^T with
// bfloat16 operands, float32 accumulation, M <= 64.  The cost is reading W
// once from HBM, so everything serves one aim: many 16-byte loads of W in
// flight in every wave, all the time.
//
// A wave owns 16 rows of W and a slice of K.  It keeps a ring of DEPTH steps
// (32 columns each) in registers: while the matrix core works on step s, the
// loads of steps s+1 .. s+DEPTH are on their way.  The 4 waves of a workgroup
// are KW slices of K times 4/KW row tiles; slices are added in LDS in slice
// order.  `parts` > 1 splits K over workgroups as well (for products with few
// output rows): part p writes its own [M, N] slab and the consumer adds the
// slabs in order, so there are no atomics and the same bits come out every run.
//
// v_mfma_f32_16x16x32_bf16: A = W tile (lane: row l % 16, k = 8 (l / 16) + j),
// B = X^T (lane: token l % 16, same k), D: lane holds features 4 (l / 16) + v of
// token l % 16, i.e. 16 contiguous bytes of a Y row.
//
// With SWIGLU the weight is [gate rows; up rows] ([2 I, K]); a wave computes the
// gate tile and the matching up tile together and writes
// silu(gate) * up as bfloat16 [M, I]  (/root/reference/src/kipp.c:2644-2648).
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

template <int MT, bool SWIGLU, int KW, int DEPTH>
__global__ void __launch_bounds__(THREADS) gemm_skinny_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, float* __restrict__ Y, bf16_t* __restrict__ act,
    int M, int N, int K, int steps_per_part) {
    constexpr int NT = SWIGLU ? 2 : 1;
    constexpr int TW = WAVES / KW;                   // row tiles of a workgroup
    __shared__ float red[KW > 1 ? WAVES : 1][NT][MT][256];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // uniform: the loop bounds below are scalars
    const int l16 = lane & 15, h = lane >> 4;
    const int tile_in_wg = wave / KW, slice = wave % KW;
    const int n0 = (blockIdx.x * TW + tile_in_wg) * 16;
    const int part = blockIdx.y;
    const int inner = SWIGLU ? N / 2 : N;            // rows of one of the stacked matrices
    const int full_steps = K / 32;                   // steps of 32 columns; a rest of 8, 16 or 24 comes last
    const int part_begin = min(full_steps, part * steps_per_part);
    const int part_end = min(full_steps, part_begin + steps_per_part);
    const int per_slice = (part_end - part_begin + KW - 1) / KW;
    const int s_begin = min(part_end, part_begin + slice * per_slice);
    const int s_end = min(part_end, s_begin + per_slice);

    const bool row_ok = n0 + l16 < inner;
    const int row = row_ok ? n0 + l16 : 0;           // clamped: the loads stay in bounds, the result is dropped
    const bf16_t* w_row[NT];
    w_row[0] = W + (size_t)row * K + 8 * h;
    if (SWIGLU) w_row[NT - 1] = W + (size_t)(inner + row) * K + 8 * h;
    const bf16_t* x_row[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) x_row[mt] = X + (size_t)min(16 * mt + l16, M - 1) * K + 8 * h;

    f32x4 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

    Frag wf[DEPTH][NT], xf[DEPTH][MT];
    // A step beyond the slice reads the slice's last step again (in bounds) and is never used.
    // No value is touched between its load and its product: the loads stay in flight.
    auto fetch = [&](int u, int s) {
        const int k = 32 * min(s, s_end - 1);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) wf[u][nt].u = __builtin_nontemporal_load((const u32x4*)(w_row[nt] + k));
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xf[u][mt].u = *(const u32x4*)(x_row[mt] + k);
    };
    auto multiply = [&](int u) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][nt].v, xf[u][mt].v, acc[nt][mt], 0, 0, 0);
    };

    if (s_begin < s_end) {
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) fetch(u, s_begin + u);
        int s = s_begin;
        for (; s + 2 * DEPTH <= s_end; s += DEPTH) {     // every step used and every step fetched is inside the slice
#pragma unroll
            for (int u = 0; u < DEPTH; ++u) {
                multiply(u);
                fetch(u, s + DEPTH + u);
            }
        }
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            if (s + u < s_end) multiply(u);
            fetch(u, s + DEPTH + u);
        }
        s += DEPTH;
#pragma unroll
        for (int u = 0; u < DEPTH; ++u)
            if (s + u < s_end) multiply(u);
    }
    // the rest of K beyond the last full step, by the wave that owns the end of the contraction
    if ((K & 31) != 0 && part == (int)gridDim.y - 1 && slice == KW - 1) {
        const int k = 32 * full_steps;
        const bool ok = k + 8 * h < K;
        Frag w_t[NT], x_t[MT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            w_t[nt].u = (u32x4){0u, 0u, 0u, 0u};
            if (ok) w_t[nt].u = *(const u32x4*)(w_row[nt] + k);
        }
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            x_t[mt].u = (u32x4){0u, 0u, 0u, 0u};
            if (ok) x_t[mt].u = *(const u32x4*)(x_row[mt] + k);
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_t[nt].v, x_t[mt].v, acc[nt][mt], 0, 0, 0);
    }
    // tokens beyond M and rows beyond N were computed from clamped addresses and are dropped below

    float sum[NT][MT][4];
    if (KW > 1) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) red[wave][nt][mt][lane * 4 + v] = acc[nt][mt][v];
        __syncthreads();
        if (slice != 0) return;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float a = 0.0f;
#pragma unroll
                    for (int w = 0; w < KW; ++w) a += red[tile_in_wg * KW + w][nt][mt][lane * 4 + v];
                    sum[nt][mt][v] = a;
                }
    } else {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int v = 0; v < 4; ++v) sum[nt][mt][v] = acc[nt][mt][v];
    }
    const int n = n0 + 4 * h;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int token = 16 * mt + l16;
        if (token >= M) continue;
        if (SWIGLU) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if (n + v < inner) {
                    const float g = sum[0][mt][v], up = sum[NT - 1][mt][v];
                    act[(size_t)token * inner + n + v] = f32_to_bf16(g / (1.0f + expf(-g)) * up);
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

template <bool SWIGLU, int KW>
static int launch_kw(const bf16_t* X, const bf16_t* W, float* Y, bf16_t* act, int M, int N, int K, int parts,
                     hipStream_t stream) {
    const int inner = SWIGLU ? N / 2 : N;
    const int full_steps = K / 32;
    const int steps_per_part = (full_steps + parts - 1) / parts;
    const int tiles = (inner + 15) / 16;
    constexpr int TW = WAVES / KW;
    dim3 grid((tiles + TW - 1) / TW, parts), block(THREADS);
    const int mt = (M + 15) / 16;
#define KIPP_SK(MT, D) \
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, SWIGLU, KW, D>), grid, block, 0, stream, X, W, Y, act, M, N, K, steps_per_part)
    switch (mt) {
        case 1: KIPP_SK(1, 8); break;
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
                  hipStream_t stream) {
    switch (kw) {
        case 1: return launch_kw<SWIGLU, 1>(X, W, Y, act, M, N, K, parts, stream);
        case 2: return launch_kw<SWIGLU, 2>(X, W, Y, act, M, N, K, parts, stream);
        case 4: return launch_kw<SWIGLU, 4>(X, W, Y, act, M, N, K, parts, stream);
        default: return -1;
    }
}

// How the contraction is split: `kw` slices inside a workgroup and `parts`
// across workgroups, so that about 1500 waves stream the weight and each has
// at least 16 steps.  A function of the shape only, never of the data.
static void plan(int tiles, int total_steps, int max_parts, int* kw, int* parts) {
    int want = (1536 + tiles - 1) / tiles;                 // slices per tile to reach ~1536 waves
    const int by_steps = total_steps / 16 > 0 ? total_steps / 16 : 1;
    if (want > by_steps) want = by_steps;
    if (want >= 4) {
        *kw = 4;
        *parts = want / 4;
    } else if (want >= 2) {
        *kw = 2;
        *parts = 1;
    } else {
        *kw = 1;
        *parts = 1;
    }
    if (*parts > max_parts) *parts = max_parts;
    if (*parts < 1) *parts = 1;
}

extern "C" {

// Slabs the product of this shape comes in when the caller allows up to `max_parts`.
int kipp_gemm_skinny_parts(int N, int K, int max_parts) {
    int kw, parts;
    plan((N + 15) / 16, (K + 31) / 32, max_parts, &kw, &parts);
    return parts;
}

// Y: float32 [parts, M, N] with parts = kipp_gemm_skinny_parts(N, K, max_parts).
// K must be a multiple of 8 (16-byte loads), M <= 64.
int kipp_gemm_skinny(const void* X, const void* W, float* Y, int M, int N, int K, int max_parts, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || (K & 7) || max_parts <= 0) return -1;
    int kw, parts;
    plan((N + 15) / 16, (K + 31) / 32, max_parts, &kw, &parts);
    return launch<false>((const bf16_t*)X, (const bf16_t*)W, Y, nullptr, M, N, K, parts, kw, stream);
}

// W: [2 I, K] = [gate; up]; act: bfloat16 [M, I].
int kipp_gemm_skinny_swiglu(const void* X, const void* W, void* act, int M, int two_inner, int K, hipStream_t stream) {
    if (M <= 0 || two_inner <= 0) return 0;
    if (M > 64 || K <= 0 || (K & 7) || (two_inner & 1)) return -1;
    int kw, parts;
    plan((two_inner / 2 + 15) / 16, (K + 31) / 32, 1, &kw, &parts);
    return launch<true>((const bf16_t*)X, (const bf16_t*)W, nullptr, (bf16_t*)act, M, two_inner, K, 1, kw, stream);
}

}  // extern "C"
