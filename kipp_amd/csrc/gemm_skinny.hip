// Matrix product for few rows (decode): Y[M, N] = X[M, K] . W[N, K]^T with
// bfloat16 operands, float32 accumulation, M <= 64.  The cost is reading W
// once from HBM; everything is arranged so that a wave streams 16 rows of W
// with 16-byte loads and feeds them to the matrix cores as they arrive.
//
// A workgroup is 4 waves on the same 16 rows of W, each with a quarter of the
// workgroup's K range; their partial tiles are added in LDS in wave order.
// `parts` > 1 splits K over workgroups as well (for products with few output
// rows): part p writes its own [M, N] slab and the consumer adds the slabs in
// order, so no atomics and the same bits every run.
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
#define UNROLL 4

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

union Frag {
    u32x4 u;
    bf16x8 v;
};

template <int MT, bool SWIGLU>
__global__ void __launch_bounds__(THREADS) gemm_skinny_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, float* __restrict__ Y, bf16_t* __restrict__ act,
    int M, int N, int K, int steps_per_part) {
    constexpr int NT = SWIGLU ? 2 : 1;
    __shared__ float red[WAVES][NT][MT][256];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, h = lane >> 4;
    const int n0 = blockIdx.x * 16;
    const int part = blockIdx.y;
    const int inner = SWIGLU ? N / 2 : N;            // rows of one of the stacked matrices
    const int total_steps = (K + 31) / 32;
    const int part_begin = part * steps_per_part;
    const int part_end = min(total_steps, part_begin + steps_per_part);
    const int per_wave = (part_end - part_begin + WAVES - 1) / WAVES;
    const int s_begin = part_begin + wave * per_wave;
    const int s_end = min(part_end, s_begin + per_wave);

    const bool row_ok = n0 + l16 < inner;
    const bf16_t* w_row[NT];
    w_row[0] = W + (size_t)(n0 + l16) * K;
    if (SWIGLU) w_row[NT - 1] = W + (size_t)(inner + n0 + l16) * K;
    const bf16_t* x_row[MT];
    bool tok_ok[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        tok_ok[mt] = 16 * mt + l16 < M;
        x_row[mt] = X + (size_t)(16 * mt + l16) * K;
    }

    f32x4 acc[NT][MT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};

    for (int s0 = s_begin; s0 < s_end; s0 += UNROLL) {
        Frag wf[UNROLL][NT], xf[UNROLL][MT];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int k = 32 * (s0 + u) + 8 * h;
            const bool k_ok = s0 + u < s_end && k < K;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                wf[u][nt].u = (u32x4){0u, 0u, 0u, 0u};
                if (k_ok && row_ok) wf[u][nt].u = __builtin_nontemporal_load((const u32x4*)(w_row[nt] + k));
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                xf[u][mt].u = (u32x4){0u, 0u, 0u, 0u};
                if (k_ok && tok_ok[mt]) xf[u][mt].u = *(const u32x4*)(x_row[mt] + k);
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][nt].v, xf[u][mt].v, acc[nt][mt], 0, 0, 0);
    }
    // add the four waves in order
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][nt][mt][lane * 4 + v] = acc[nt][mt][v];
    __syncthreads();
    // thread (mt, lane) of the first MT waves finishes tile mt
    for (int mt = wave; mt < MT; mt += WAVES) {
        const int token = 16 * mt + l16;
        float sum[NT][4];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float a = 0.0f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) a += red[w][nt][mt][lane * 4 + v];
                sum[nt][v] = a;
            }
        if (token >= M) continue;
        const int n = n0 + 4 * h;
        if (SWIGLU) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if (n + v < inner) {
                    const float g = sum[0][v], up = sum[NT - 1][v];
                    act[(size_t)token * inner + n + v] = f32_to_bf16(g / (1.0f + expf(-g)) * up);
                }
            }
        } else {
            float* y = Y + ((size_t)part * M + token) * N + n;
            if (n + 3 < N && (N & 3) == 0) {
                *(float4*)y = make_float4(sum[0][0], sum[0][1], sum[0][2], sum[0][3]);
            } else {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (n + v < N) y[v] = sum[0][v];
            }
        }
    }
}

template <bool SWIGLU>
static int launch(const bf16_t* X, const bf16_t* W, float* Y, bf16_t* act, int M, int N, int K, int parts,
                  hipStream_t stream) {
    const int inner = SWIGLU ? N / 2 : N;
    const int total_steps = (K + 31) / 32;
    const int steps_per_part = (total_steps + parts - 1) / parts;
    dim3 grid((inner + 15) / 16, parts), block(THREADS);
    const int mt = (M + 15) / 16;
#define KIPP_SK(MT) hipLaunchKernelGGL((gemm_skinny_kernel<MT, SWIGLU>), grid, block, 0, stream, X, W, Y, act, M, N, K, steps_per_part)
    switch (mt) {
        case 1: KIPP_SK(1); break;
        case 2: KIPP_SK(2); break;
        case 3: KIPP_SK(3); break;
        case 4: KIPP_SK(4); break;
        default: return -1;
    }
#undef KIPP_SK
    return KIPP_LAUNCH_CHECK();
}

extern "C" {

// Y: float32 [parts, M, N].  K must be a multiple of 8 (16-byte loads), M <= 64.
int kipp_gemm_skinny(const void* X, const void* W, float* Y, int M, int N, int K, int parts, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 64 || K <= 0 || (K & 7) || parts <= 0) return -1;
    return launch<false>((const bf16_t*)X, (const bf16_t*)W, Y, nullptr, M, N, K, parts, stream);
}

// W: [2 I, K] = [gate; up]; act: bfloat16 [M, I].
int kipp_gemm_skinny_swiglu(const void* X, const void* W, void* act, int M, int two_inner, int K, hipStream_t stream) {
    if (M <= 0 || two_inner <= 0) return 0;
    if (M > 64 || K <= 0 || (K & 7) || (two_inner & 1)) return -1;
    return launch<true>((const bf16_t*)X, (const bf16_t*)W, nullptr, (bf16_t*)act, M, two_inner, K, 1, stream);
}

}  // extern "C"
