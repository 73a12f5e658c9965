// Per-head q/k RMSNorm, rotary position encoding and the write of keys and
// values into the paged cache, in one pass over the projection output.
//
// Input row layout of `qkv`: [n_q heads | n_kv key heads | n_kv value heads],
// each head `d` wide; `qkv` may come in `parts` slabs [parts, tokens, width] that are added
// in order (a product whose contraction was split over workgroups).  One wave handles one head of one token.
//   norm   u_j *= rsqrt(mean(u^2) + eps) * w_j, the same w for every head
//          (/root/reference/src/kipp.c:2480-2500), before the rotation;
//   rotary (u_i, u_{i+r/2}) <- (u_i c - u_{i+r/2} s, u_{i+r/2} c + u_i s),
//          angle = float(pos) * inv_freq[i]  (kipp.c:2368-2382); dims >= r pass;
//          with `interleaved` pair i is (u_{2i}, u_{2i+1}) instead (another pairing that
//          checkpoints of other families use; the general kernel only);
//          with `angles` ([tokens][r]: r/2 cosines, then r/2 sines, made once a step by
//          rotary_angles_kernel for all layers) the kernel reads them instead of computing them;
//   write  key/value row of position pos goes to page table[pos / page], slot
//          pos % page; cache layout [page][kv head][slot][d].
#include "common.h"

#define HEADS_PER_BLOCK 4
#define MAX_D 256

template <typename TI, typename TO, typename TC>
__global__ void qk_norm_rope_kv_kernel(
    const TI* __restrict__ qkv, TO* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ inv_freq, const float* __restrict__ angles, int rotary_dim, int interleaved,
    int n_q, int n_kv, int d, int page, int n_slots, int parts, size_t part_stride) {
    __shared__ float buf[HEADS_PER_BLOCK][MAX_D];
    const int wave = threadIdx.x / KIPP_WAVE;
    const int lane = threadIdx.x & (KIPP_WAVE - 1);
    const int t = blockIdx.y;
    int slot = blockIdx.x * HEADS_PER_BLOCK + wave;
    const bool active = slot < n_slots;
    if (!active) slot = n_slots - 1;  // stay in step with the barriers below
    const int kind = slot < n_q ? 0 : (slot < n_q + n_kv ? 1 : 2);  // q, k, v
    const int row_width = (n_q + 2 * n_kv) * d;
    const TI* src = qkv + (size_t)t * row_width + (size_t)slot * d;
    const int pos = positions[t];

    float vals[MAX_D / KIPP_WAVE];
    float ss = 0.0f;
#pragma unroll
    for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
        const int e = lane + c * KIPP_WAVE;
        float v = 0.0f;
        if (e < d)
            for (int p = 0; p < parts; ++p) v += load_f(src, p * part_stride + e);   // slabs of a split product, in order
        vals[c] = v;
        ss = square_add(ss, v);
    }
    const float* norm_w = kind == 0 ? q_norm_w : (kind == 1 ? k_norm_w : nullptr);
    if (norm_w != nullptr) {
        ss = wave_sum(ss);
        const float scale = head_norm_scale(ss, (float)d, eps);
#pragma unroll
        for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
            const int e = lane + c * KIPP_WAVE;
            if (e < d) vals[c] *= scale * norm_w[e];
        }
    }
#pragma unroll
    for (int c = 0; c < MAX_D / KIPP_WAVE; ++c) {
        const int e = lane + c * KIPP_WAVE;
        if (e < d) buf[wave][e] = vals[c];
    }
    __syncthreads();
    // Barriers stay outside the conditions: waves of one workgroup hold heads
    // of different kinds.
    const bool rotate = kind != 2 && (inv_freq != nullptr || angles != nullptr);
    const int half = rotary_dim / 2;
    float lo[MAX_D / 2 / KIPP_WAVE], hi[MAX_D / 2 / KIPP_WAVE];
#pragma unroll
    for (int c = 0; c < MAX_D / 2 / KIPP_WAVE; ++c) {
        const int i = lane + c * KIPP_WAVE;
        lo[c] = hi[c] = 0.0f;
        if (rotate && i < half) {
            float cs, sn;
            if (angles != nullptr) {
                cs = angles[(size_t)t * rotary_dim + i];
                sn = angles[(size_t)t * rotary_dim + half + i];
            } else {
                const float angle = (float)pos * inv_freq[i];
                cs = cosf(angle);
                sn = sinf(angle);
            }
            const float a = buf[wave][interleaved ? 2 * i : i], b = buf[wave][interleaved ? 2 * i + 1 : i + half];
            lo[c] = rotate_lo(a, b, cs, sn);
            hi[c] = rotate_hi(a, b, cs, sn);
        }
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < MAX_D / 2 / KIPP_WAVE; ++c) {
        const int i = lane + c * KIPP_WAVE;
        if (rotate && i < half) {
            buf[wave][interleaved ? 2 * i : i] = lo[c];
            buf[wave][interleaved ? 2 * i + 1 : i + half] = hi[c];
        }
    }
    __syncthreads();
    if (!active) return;
    if (kind == 0) {
        TO* dst = q_out + ((size_t)t * n_q + slot) * d;
        for (int e = lane; e < d; e += KIPP_WAVE) store_f(dst, e, buf[wave][e]);
    } else {
        const int head = kind == 1 ? slot - n_q : slot - n_q - n_kv;
        const int seq = seq_of_token[t];
        const int page_id = block_table[(size_t)seq * max_blocks + pos / page];
        TC* dst = (kind == 1 ? k_cache : v_cache) +
                  (((size_t)page_id * n_kv + head) * page + pos % page) * d;
        for (int e = lane; e < d; e += KIPP_WAVE) store_f(dst, e, buf[wave][e]);
    }
}

// The same for head sizes of 128 and 256 rotated over their whole width: element
// i and its partner i + d/2 then lie in the same lane (lane i % 64 holds elements
// i % 64 + 64 c), so nothing passes through LDS; a wave takes several heads of one
// token, four at a time with all their loads issued first, and computes the
// token's sines and cosines once for all of them.
template <int NC, bool SLABS, typename TI, typename TO, typename TC>
__global__ void __launch_bounds__(HEADS_PER_BLOCK * KIPP_WAVE) qk_norm_rope_kv_regs_kernel(
    const TI* __restrict__ qkv, TO* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ inv_freq, const float* __restrict__ angles, int n_q, int n_kv, int page, int n_slots,
    int parts, size_t part_stride) {
    constexpr int D = NC * KIPP_WAVE, HC = NC / 2, BATCH = 4;
    const int wave = threadIdx.x / KIPP_WAVE;
    const int lane = threadIdx.x & (KIPP_WAVE - 1);
    const int t = blockIdx.y;
    const int waves = gridDim.x * HEADS_PER_BLOCK;
    const int pos = positions[t];
    const size_t row = (size_t)t * (n_q + 2 * n_kv) * D;

    float cs[HC], sn[HC], qw[NC], kw[NC];
#pragma unroll
    for (int c = 0; c < HC; ++c) {
        cs[c] = 1.0f;
        sn[c] = 0.0f;
        if (angles != nullptr) {
            cs[c] = angles[(size_t)t * D + lane + c * KIPP_WAVE];
            sn[c] = angles[(size_t)t * D + D / 2 + lane + c * KIPP_WAVE];
        } else if (inv_freq != nullptr) {
            const float angle = (float)pos * inv_freq[lane + c * KIPP_WAVE];
            cs[c] = cosf(angle);
            sn[c] = sinf(angle);
        }
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
        qw[c] = q_norm_w != nullptr ? q_norm_w[lane + c * KIPP_WAVE] : 1.0f;
        kw[c] = k_norm_w != nullptr ? k_norm_w[lane + c * KIPP_WAVE] : 1.0f;
    }
    size_t cache_row = 0;
    if (n_slots > n_q) {
        const int page_id = block_table[(size_t)seq_of_token[t] * max_blocks + pos / page];
        cache_row = (size_t)page_id * n_kv * page + pos % page;
    }

    for (int s0 = blockIdx.x * HEADS_PER_BLOCK + wave; s0 < n_slots; s0 += waves * BATCH) {
        float v[BATCH][NC];
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const int slot = min(s0 + u * waves, n_slots - 1);
            const TI* src = qkv + row + (size_t)slot * D + lane;
#pragma unroll
            for (int c = 0; c < NC; ++c) v[u][c] = load_f(src, c * KIPP_WAVE);
        }
        if (SLABS) {
            // the other slabs, four at a time: all their loads are asked for before the first is added (slabs in order)
            for (int p0 = 1; p0 < parts; p0 += 4) {
                float more[4][BATCH][NC];
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int u = 0; u < BATCH; ++u) {
                        const int slot = min(s0 + u * waves, n_slots - 1);
                        const TI* src = qkv + row + (size_t)slot * D + lane;
#pragma unroll
                        for (int c = 0; c < NC; ++c)
                            more[q][u][c] = p0 + q < parts ? load_f(src, (size_t)(p0 + q) * part_stride + c * KIPP_WAVE) : 0.0f;
                    }
#pragma unroll
                for (int q = 0; q < 4; ++q)
#pragma unroll
                    for (int u = 0; u < BATCH; ++u)
#pragma unroll
                        for (int c = 0; c < NC; ++c) v[u][c] += more[q][u][c];
            }
        }
#pragma unroll
        for (int u = 0; u < BATCH; ++u) {
            const int slot = s0 + u * waves;
            if (slot >= n_slots) break;
            const int kind = slot < n_q ? 0 : (slot < n_q + n_kv ? 1 : 2);
            if (kind != 2) {
                if ((kind == 0 ? q_norm_w : k_norm_w) != nullptr) {
                    float ss = 0.0f;
#pragma unroll
                    for (int c = 0; c < NC; ++c) ss = square_add(ss, v[u][c]);
                    ss = wave_sum(ss);
                    const float scale = head_norm_scale(ss, (float)D, eps);
#pragma unroll
                    for (int c = 0; c < NC; ++c) v[u][c] *= scale * (kind == 0 ? qw[c] : kw[c]);
                }
#pragma unroll
                for (int c = 0; c < HC; ++c) {
                    const float a = v[u][c], b = v[u][c + HC];
                    v[u][c] = rotate_lo(a, b, cs[c], sn[c]);
                    v[u][c + HC] = rotate_hi(a, b, cs[c], sn[c]);
                }
            }
            if (kind == 0) {
                TO* dst = q_out + ((size_t)t * n_q + slot) * D + lane;
#pragma unroll
                for (int c = 0; c < NC; ++c) store_f(dst, c * KIPP_WAVE, v[u][c]);
            } else {
                const int head = kind == 1 ? slot - n_q : slot - n_q - n_kv;
                TC* dst = (kind == 1 ? k_cache : v_cache) + (cache_row + (size_t)head * page) * D + lane;
#pragma unroll
                for (int c = 0; c < NC; ++c) store_f(dst, c * KIPP_WAVE, v[u][c]);
            }
        }
    }
}

template <typename TI, typename TO, typename TC>
static void launch_regs(const void* qkv, void* q_out, void* k_cache, void* v_cache, const int32_t* positions,
                        const int32_t* seq_of_token, const int32_t* block_table, int max_blocks, const float* q_norm_w,
                        const float* k_norm_w, float eps, const float* inv_freq, const float* angles, int n_tokens,
                        int n_q, int n_kv, int d, int page, int n_slots, int parts, hipStream_t stream) {
    // few tokens: a wave for every head; many: a workgroup for a token
    const int per_token = n_tokens >= 256 ? 1 : (n_slots + HEADS_PER_BLOCK - 1) / HEADS_PER_BLOCK;
    dim3 grid(per_token, n_tokens), block(HEADS_PER_BLOCK * KIPP_WAVE);
    const size_t stride = (size_t)n_tokens * (n_q + 2 * n_kv) * d;
#define KIPP_RR(NC, SLABS)                                                                                          \
    hipLaunchKernelGGL((qk_norm_rope_kv_regs_kernel<NC, SLABS, TI, TO, TC>), grid, block, 0, stream, (const TI*)qkv, \
                       (TO*)q_out, (TC*)k_cache, (TC*)v_cache, positions, seq_of_token, block_table, max_blocks,     \
                       q_norm_w, k_norm_w, eps, inv_freq, angles, n_q, n_kv, page, n_slots, parts, stride)
    if (d == 128) {
        if (parts > 1) KIPP_RR(2, true); else KIPP_RR(2, false);
    } else {
        if (parts > 1) KIPP_RR(4, true); else KIPP_RR(4, false);
    }
#undef KIPP_RR
}

// angles[t][i] = cos(float(pos_t) * inv_freq[i]), angles[t][half + i] = sin(...): once a step, for every
// layer that rotates with these frequencies.
__global__ void rotary_angles_kernel(const int32_t* __restrict__ positions, const float* __restrict__ inv_freq,
                                     float* __restrict__ angles, int n_tokens, int half) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_tokens * half) return;
    const int t = idx / half, i = idx % half;
    const float angle = (float)positions[t] * inv_freq[i];
    angles[(size_t)t * 2 * half + i] = cosf(angle);
    angles[(size_t)t * 2 * half + half + i] = sinf(angle);
}

extern "C" int kipp_rotary_angles(const int32_t* positions, const float* inv_freq, float* angles, int n_tokens, int half,
                                  hipStream_t stream) {
    if (n_tokens <= 0 || half <= 0) return 0;
    const int total = n_tokens * half;
    hipLaunchKernelGGL(rotary_angles_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, positions, inv_freq, angles,
                       n_tokens, half);
    return KIPP_LAUNCH_CHECK();
}

extern "C" int kipp_qk_norm_rope_kv(
    const void* qkv, int in_dtype, void* q_out, int q_dtype, void* k_cache, void* v_cache, int cache_dtype,
    const int32_t* positions, const int32_t* seq_of_token, const int32_t* block_table, int max_blocks,
    const float* q_norm_w, const float* k_norm_w, float eps, const float* inv_freq, const float* angles, int rotary_dim,
    int interleaved, int n_tokens, int n_q, int n_kv, int d, int page, int write_kv, int parts, hipStream_t stream) {
    if (n_tokens <= 0) return 0;
    if (d > MAX_D || d <= 0 || rotary_dim > d || (rotary_dim & 1)) return -1;
    const int n_slots = write_kv ? n_q + 2 * n_kv : n_q;
    const bool rotates = inv_freq != nullptr || angles != nullptr;
    if ((d == 128 || d == 256) && (!rotates || (rotary_dim == d && !interleaved))) {
#define KIPP_RL(TI, TO, TC)                                                                                        \
    launch_regs<TI, TO, TC>(qkv, q_out, k_cache, v_cache, positions, seq_of_token, block_table, max_blocks, q_norm_w, \
                            k_norm_w, eps, inv_freq, angles, n_tokens, n_q, n_kv, d, page, n_slots, parts, stream)
        if (in_dtype == KIPP_F32 && q_dtype == KIPP_F32 && cache_dtype == KIPP_F32) KIPP_RL(float, float, float);
        else if (in_dtype == KIPP_F32 && q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16) KIPP_RL(float, bf16_t, bf16_t);
        else if (in_dtype == KIPP_BF16 && q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16) KIPP_RL(bf16_t, bf16_t, bf16_t);
        else return -2;
#undef KIPP_RL
        return KIPP_LAUNCH_CHECK();
    }
    dim3 grid((n_slots + HEADS_PER_BLOCK - 1) / HEADS_PER_BLOCK, n_tokens), block(HEADS_PER_BLOCK * KIPP_WAVE);
#define KIPP_RK(TI, TO, TC)                                                                                  \
    hipLaunchKernelGGL((qk_norm_rope_kv_kernel<TI, TO, TC>), grid, block, 0, stream, (const TI*)qkv,         \
                       (TO*)q_out, (TC*)k_cache, (TC*)v_cache, positions, seq_of_token, block_table,         \
                       max_blocks, q_norm_w, k_norm_w, eps, inv_freq, angles, rotary_dim, interleaved, n_q, n_kv, d, page, n_slots, parts,      \
                       (size_t)n_tokens * (n_q + 2 * n_kv) * d)
    if (in_dtype == KIPP_F32 && q_dtype == KIPP_F32 && cache_dtype == KIPP_F32) KIPP_RK(float, float, float);
    else if (in_dtype == KIPP_F32 && q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16) KIPP_RK(float, bf16_t, bf16_t);
    else if (in_dtype == KIPP_BF16 && q_dtype == KIPP_BF16 && cache_dtype == KIPP_BF16) KIPP_RK(bf16_t, bf16_t, bf16_t);
    else return -2;
#undef KIPP_RK
    return KIPP_LAUNCH_CHECK();
}
