// Prefill attention over the paged cache, bfloat16: causal grouped-query
// attention for portions of prompts (two tokens and more), with the online
// softmax of flash attention and both products on the matrix cores
// (/root/reference/metal/kipp_kernels.metal:1380-1611 plays this role in the reference).
//
// A workgroup (4 waves) takes 128 consecutive query rows of one sequence and
// one query head; a wave owns 32 of them.  Keys and values of the sequence are
// streamed through LDS in tiles of 64 positions, found through the block table
// (the portion may start at any position; keys 0..pos are in the cache, this
// step's own keys included).
//
//   S^T = K Q^T   v_mfma_f32_32x32x16_bf16, A = key tile from LDS, B = the wave's
//                 queries held in registers.  In the result a lane holds 16
//                 keys of ONE query (its column), so the row statistics of the
//                 softmax are per lane plus one exchange with lane ^ 32.
//   O^T = V^T P^T A = value tile stored transposed in LDS, B = the probabilities
//                 straight from the S^T registers (the contraction index of the
//                 instruction is a dummy, so the key order a lane happens to
//                 hold is simply used for both operands).  O^T again has the
//                 query as its column: rescaling needs no exchange at all.
//
// Softmax in float32, base 2; probabilities are rounded to bfloat16 for the
// second product, the row sum is taken from the float32 values.
//
// Compile-time: HEAD_DIM (multiple of 16, <= 256).
#include "common.h"
#include <math.h>
#include <type_traits>

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif

#define BM 128
#define BN 64
#define WAVES 4
#define THREADS (WAVES * KIPP_WAVE)
#define QSTEPS (HEAD_DIM / 16)                 // contraction steps of S^T
#define DP (((HEAD_DIM + 31) / 32) * 32)       // value columns rounded up to the 32-row tile of O^T
#define DTILES (DP / 32)
#define K_PITCH (HEAD_DIM + 8)                 // bf16 elements per key row in LDS
#define V_PITCH (BN + 4)                       // bf16 elements per value column in LDS
#define DCHUNKS (HEAD_DIM / 8)
#define K_LOADS ((BN * DCHUNKS + THREADS - 1) / THREADS)
#define V_TASKS (((BN / 2) * DCHUNKS + THREADS - 1) / THREADS)
#define MAX_PAGES 4096

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

union Frag {
    u32x4 u;
    bf16x8 v;
};


typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

// two floats to two bfloat16 (round to nearest even) in one 32-bit word: the conversion
// instruction of gfx950
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    union {
        bf16x2 v;
        uint32_t u;
    } r;
    r.v = __builtin_convertvector((f32x2){a, b}, bf16x2);
    return r.u;
}

__global__ void __launch_bounds__(THREADS, 2) attention_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int32_t* __restrict__ item_seq, const int32_t* __restrict__ item_tile,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ block_table, int max_blocks, int n_q, int n_kv, int page, float scale_log2e,
    int window, int tile_rows, const int32_t* __restrict__ item_split, int split_keys, float* __restrict__ part_acc,
    float* __restrict__ part_ml, int max_splits) {
    __shared__ __attribute__((aligned(16))) bf16_t Ks[BN * K_PITCH];
    __shared__ __attribute__((aligned(16))) bf16_t Vt[DP * V_PITCH];
    __shared__ int s_page[MAX_PAGES];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, hh = lane >> 5;
    // Work = (item, head), items sorted by the host from the longest key range to the
    // shortest.  The first half of the grid takes the work in that order, the second half
    // from the light end: workgroups that come to share a compute unit (k and k + half, when
    // the whole grid is resident at once) then carry about the same load together.
    const int total = gridDim.x, half = (total + 1) / 2;
    const int work = (int)blockIdx.x < half ? (int)blockIdx.x : total - 1 - ((int)blockIdx.x - half);
    const int item = work / n_q, head = work % n_q;
    const int kvh = head / (n_q / n_kv);
    const int seq = item_seq[item];
    const int tile_row0 = item_tile[item] * tile_rows;          // first row of the tile within the portion
    const int row0 = q_start[seq] + tile_row0;                  // ... within the batch
    const int rows_in_tile = min(tile_rows, q_len[seq] - tile_row0);
    const int pos0 = positions[row0];                           // position of the tile's first query
    const int last_pos = pos0 + rows_in_tile - 1;
    const int32_t* table = block_table + (size_t)seq * max_blocks;

    const int my_row = wave * 32 + l32;                         // this lane's query within the tile
    const bool wave_active = wave * 32 < rows_in_tile;
    const bool row_valid = my_row < rows_in_tile;
    const int my_pos = pos0 + my_row;
    const int my_lo = window > 0 ? max(0, my_pos - window + 1) : 0;

    // the wave's queries as B operand: lane (query l32, half hh) holds q[16 t + 8 hh .. + 7]
    Frag qf[QSTEPS];
#pragma unroll
    for (int t = 0; t < QSTEPS; ++t) {
        qf[t].u = (u32x4){0u, 0u, 0u, 0u};
        if (row_valid) qf[t].u = *(const u32x4*)(q + ((size_t)(row0 + my_row) * n_q + head) * HEAD_DIM + 16 * t + 8 * hh);
    }

    f32x16 o[DTILES];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[dt][v] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;

    // value rows beyond the head size stay zero for the whole kernel
    if (DP > HEAD_DIM) {
        for (int i = tid; i < (DP - HEAD_DIM) * V_PITCH; i += THREADS) Vt[HEAD_DIM * V_PITCH + i] = 0;
    }

    // with `split_keys` the keys are cut at multiples of it and this work item takes one cut (windows are not split)
    const int split = split_keys > 0 ? item_split[item] : 0;
    const int tile_lo = split_keys > 0 ? split * (split_keys / BN) : (window > 0 ? max(0, pos0 - window + 1) : 0) / BN;
    const int tile_hi = split_keys > 0 ? min(last_pos / BN, (split + 1) * (split_keys / BN) - 1) : last_pos / BN;

    // The pages of the keys this workgroup reads, once, into LDS: the loads of a tile then
    // depend on nothing in flight and are issued back to back.  The page size is a power of
    // two and the table row fits s_page (both checked by the launcher).
    const int page_shift = __builtin_ctz(page);
    const int first_block = (tile_lo * BN) >> page_shift, last_block = min(last_pos, tile_hi * BN + BN - 1) >> page_shift;
    for (int i = tid; i <= last_block - first_block; i += THREADS) s_page[i] = table[first_block + i];
    __syncthreads();
    // address of key s of this sequence and head; s is clamped to the last key of the portion
    // (beyond it the scores are masked, the values only have to be finite)
    auto row_offset = [&](int s) -> size_t {
        const int sc = min(s, last_pos);
        return (((size_t)s_page[(sc >> page_shift) - first_block] * n_kv + kvh) * page + (sc & (page - 1))) * HEAD_DIM;
    };

    // registers for one tile: keys (K_LOADS 16-byte chunks a thread), values (2 chunks for each of V_TASKS key pairs)
    Frag k_reg[K_LOADS];
    Frag v_reg[V_TASKS][2];
    auto fetch_tile = [&](int key0) {
#pragma unroll
        for (int i = 0; i < K_LOADS; ++i) {
            const int c = min(tid + i * THREADS, BN * DCHUNKS - 1);
            const int key = c / DCHUNKS, chunk = c % DCHUNKS;
            k_reg[i].u = *(const u32x4*)(k_cache + row_offset(key0 + key) + chunk * 8);
        }
#pragma unroll
        for (int i = 0; i < V_TASKS; ++i) {
            const int c = min(tid + i * THREADS, (BN / 2) * DCHUNKS - 1);
            const int pair = c % (BN / 2), chunk = c / (BN / 2);
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                v_reg[i][e].u = *(const u32x4*)(v_cache + row_offset(key0 + 2 * pair + e) + chunk * 8);
            }
        }
    };
    auto store_tile = [&]() {
        // keys: [key][d]; values transposed: [d][key], two keys to a 32-bit word
#pragma unroll
        for (int i = 0; i < K_LOADS; ++i) {
            const int c = tid + i * THREADS;
            if (c < BN * DCHUNKS) *(u32x4*)(Ks + (c / DCHUNKS) * K_PITCH + (c % DCHUNKS) * 8) = k_reg[i].u;
        }
#pragma unroll
        for (int i = 0; i < V_TASKS; ++i) {
            const int c = tid + i * THREADS;
            if (c < (BN / 2) * DCHUNKS) {
                const int pair = c % (BN / 2), chunk = c / (BN / 2);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t a = v_reg[i][0].u[j >> 1], b = v_reg[i][1].u[j >> 1];
                    *(uint32_t*)(Vt + (chunk * 8 + j) * V_PITCH + 2 * pair) =
                        (j & 1) ? (a >> 16) | (b & 0xffff0000u) : (a & 0xffffu) | (b << 16);
                }
            }
        }
    };

    fetch_tile(tile_lo * BN);
    for (int kt = tile_lo; kt <= tile_hi; ++kt) {
        const int key0 = kt * BN;
        __syncthreads();   // the tile before has been read by every wave
        store_tile();
        __syncthreads();
        if (kt < tile_hi) fetch_tile(key0 + BN);   // on its way while this tile is worked on
        if (!wave_active) continue;

        // ---- S^T = K Q^T for the two 32-key halves of the tile
        f32x16 s_acc[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int v = 0; v < 16; ++v) s_acc[j][v] = 0.0f;
#pragma unroll
            for (int t = 0; t < QSTEPS; ++t) {
                Frag kf;
                kf.u = *(const u32x4*)(Ks + (32 * j + l32) * K_PITCH + 16 * t + 8 * hh);
                s_acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf.v, qf[t].v, s_acc[j], 0, 0, 0);
            }
        }
        // ---- online softmax in base 2; register v of half j is key 32 j + 8 (v / 4) + 4 hh + v % 4.
        //      The scale is folded into the exponent: p = 2^(s c - m c), one FMA and one exp a key.
        //      Only tiles that touch the diagonal (or a window's edge) pay for a mask.
        const bool masked = key0 + BN - 1 > pos0 + wave * 32 || window > 0;
        if (masked) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int s = key0 + 32 * j + 8 * (v / 4) + 4 * hh + (v % 4);
                    if (s > my_pos || s < my_lo) s_acc[j][v] = -INFINITY;
                }
        }
        float m_tile = -INFINITY;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) m_tile = fmaxf(m_tile, s_acc[j][v]);
        m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, KIPP_WAVE));
        const float m_new = fmaxf(m_run, m_tile);                 // raw scores; scale_log2e > 0 keeps the order
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;    // a row with nothing visible yet
        const float m_scaled = m_use * scale_log2e;
        const float alpha = __builtin_amdgcn_exp2f(m_run * scale_log2e - m_scaled);
        float l_tile = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float p = __builtin_amdgcn_exp2f(fmaf(s_acc[j][v], scale_log2e, -m_scaled));   // -inf gives 0
                s_acc[j][v] = p;
                l_tile += p;
            }
        l_tile += __shfl_xor(l_tile, 32, KIPP_WAVE);
        l_run = l_run * alpha + l_tile;
        m_run = m_new;
        if (__any(alpha != 1.0f)) {                               // the maximum moved for some query of the wave
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[dt][v] *= alpha;
        }
        // ---- O^T += V^T P^T; step st of half j uses registers 8 st .. 8 st + 7, which are the keys
        //      32 j + 16 st + {4 hh .. 4 hh + 3} and 32 j + 16 st + 8 + {4 hh .. 4 hh + 3}
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int st = 0; st < 2; ++st) {
                Frag pf;
                pf.u = (u32x4){pack_bf16(s_acc[j][8 * st + 0], s_acc[j][8 * st + 1]),
                               pack_bf16(s_acc[j][8 * st + 2], s_acc[j][8 * st + 3]),
                               pack_bf16(s_acc[j][8 * st + 4], s_acc[j][8 * st + 5]),
                               pack_bf16(s_acc[j][8 * st + 6], s_acc[j][8 * st + 7])};
#pragma unroll
                for (int dt = 0; dt < DTILES; ++dt) {
                    Frag vf;
                    const bf16_t* col = Vt + (32 * dt + l32) * V_PITCH + 32 * j + 16 * st + 4 * hh;
                    const u32x2 lo = *(const u32x2*)(col), hi = *(const u32x2*)(col + 8);
                    vf.u = (u32x4){lo[0], lo[1], hi[0], hi[1]};
                    o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf.v, o[dt], 0, 0, 0);
                }
            }
    }
    if (!row_valid) return;
    if (split_keys > 0) {
        // one cut of the keys: the sums as they are, with their reference maximum (base 2) and their
        // denominator; attention_prefill_merge_kernel adds the cuts of a row in order
        const size_t slot = ((size_t)(row0 + my_row) * n_q + head) * max_splits + split;
        if (hh == 0) {
            part_ml[slot * 2] = m_run == -INFINITY ? -INFINITY : m_run * scale_log2e;
            part_ml[slot * 2 + 1] = l_run;
        }
        float* p_row = part_acc + slot * HEAD_DIM;
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int dcol = 32 * dt + 8 * g + 4 * hh;
                if (dcol < HEAD_DIM) *(f32x4*)(p_row + dcol) = (f32x4){o[dt][4 * g + 0], o[dt][4 * g + 1], o[dt][4 * g + 2], o[dt][4 * g + 3]};
            }
        return;
    }
    // O^T register v of tile dt is column 32 dt + 8 (v / 4) + 4 hh + v % 4 of this lane's query
    const float inv = 1.0f / l_run;
    bf16_t* o_row = out + ((size_t)(row0 + my_row) * n_q + head) * HEAD_DIM;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int dcol = 32 * dt + 8 * g + 4 * hh;
            if (dcol < HEAD_DIM) {
                *(u32x2*)(o_row + dcol) = (u32x2){pack_bf16(o[dt][4 * g + 0] * inv, o[dt][4 * g + 1] * inv),
                                                  pack_bf16(o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv)};
            }
        }
}

// ---------------------------------------------------------------------------------------------
// The same kernel for head size 128 with the tiles brought into LDS by the memory pipeline
// itself (global_load_lds_dwordx4: 16 bytes a lane from global memory straight into LDS).
// No register holds a tile on its way, nothing is packed or transposed by the lanes, and two
// buffers take turns, so a tile costs one barrier: while tile i is worked on, tile i + 1 lands.
//
// Keys and values lie in LDS as in the cache, [key][d], 256 bytes a row.  Row r keeps its
// 16-byte chunk c at slot c ^ (r % 16) (keys) or c ^ 4 (r % 4) (values): the rows that one
// matrix-core operand reads at once then fall into different banks.  The lane that fills slot p
// of row r simply asks for chunk p ^ ... of that row.  The value operand V^T comes out of LDS
// transposed by ds_read_b64_tr_b16 (within 16 lanes, lane i receives element i % 4 of the
// 8-byte pieces addressed by lanes i / 4, 4 + i / 4, 8 + i / 4, 12 + i / 4).
#if HEAD_DIM == 128
#ifndef PREFILL_DMA
#define PREFILL_DMA 1                            // 0: head size 128 takes the kernel above as well
#endif
#define TILE_BYTES (BN * HEAD_DIM * 2)           // the keys (or the values) of one tile
#define DMA_LDS_BYTES (2 * TILE_BYTES)           // dynamic LDS: the second tile buffer; the page table lies behind it

typedef __attribute__((ext_vector_type(4))) short s16x4;
#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

__global__ void __launch_bounds__(THREADS, 2) attention_prefill_dma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int32_t* __restrict__ item_seq, const int32_t* __restrict__ item_tile,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ block_table, int max_blocks, int n_q, int n_kv, int page, float scale_log2e,
    int window, int tile_rows, const int32_t* __restrict__ item_split, int split_keys, float* __restrict__ part_acc,
    float* __restrict__ part_ml, int max_splits) {
    // the two tile buffers are two objects (one static, one dynamic): the compiler then sees that the loads
    // into one never touch what is read from the other, and makes no read wait for them
    __shared__ __attribute__((aligned(1024))) unsigned char tile_a[2 * TILE_BYTES];
    extern __shared__ __attribute__((aligned(1024))) unsigned char tile_b[];
    int* s_page = (int*)(tile_b + 2 * TILE_BYTES);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, hh = lane >> 5;
    const int l16 = lane & 15, quarter = lane >> 4;
    const int total = gridDim.x, half = (total + 1) / 2;
    const int work = (int)blockIdx.x < half ? (int)blockIdx.x : total - 1 - ((int)blockIdx.x - half);
    const int item = work / n_q, head = work % n_q;
    const int kvh = head / (n_q / n_kv);
    const int seq = item_seq[item];
    const int tile_row0 = item_tile[item] * tile_rows;
    const int row0 = q_start[seq] + tile_row0;
    const int rows_in_tile = min(tile_rows, q_len[seq] - tile_row0);
    const int pos0 = positions[row0];
    const int last_pos = pos0 + rows_in_tile - 1;
    const int32_t* table = block_table + (size_t)seq * max_blocks;

    const int my_row = wave * 32 + l32;
    const bool wave_active = wave * 32 < rows_in_tile;
    const bool row_valid = my_row < rows_in_tile;
    const int my_pos = pos0 + my_row;
    const int my_lo = window > 0 ? max(0, my_pos - window + 1) : 0;

    Frag qf[QSTEPS];
#pragma unroll
    for (int t = 0; t < QSTEPS; ++t) {
        qf[t].u = (u32x4){0u, 0u, 0u, 0u};
        if (row_valid) qf[t].u = *(const u32x4*)(q + ((size_t)(row0 + my_row) * n_q + head) * HEAD_DIM + 16 * t + 8 * hh);
    }

    f32x16 o[DTILES];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) o[dt][v] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;

    // with `split_keys` the keys are cut at multiples of it and this work item takes one cut (windows are not split)
    const int split = split_keys > 0 ? item_split[item] : 0;
    const int tile_lo = split_keys > 0 ? split * (split_keys / BN) : (window > 0 ? max(0, pos0 - window + 1) : 0) / BN;
    const int tile_hi = split_keys > 0 ? min(last_pos / BN, (split + 1) * (split_keys / BN) - 1) : last_pos / BN;
    const int page_shift = __builtin_ctz(page);
    const int first_block = (tile_lo * BN) >> page_shift, last_block = min(last_pos, tile_hi * BN + BN - 1) >> page_shift;
    for (int i = tid; i <= last_block - first_block; i += THREADS) s_page[i] = table[first_block + i];
    __syncthreads();

    // A wave brings 16 keys of a tile (and their values): instruction i the rows 4 i + quarter, a lane one
    // 16-byte slot of a row.  Keys beyond the portion's last read its last row again (masked below).
    // Where the 16 keys lie in one page and none is beyond the last (all tiles but a portion's last, pages
    // of 16 keys and more), their rows are one run of memory: a base the whole wave shares plus a lane's own
    // offset, which never changes.
    uint32_t k_off[4], v_off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = 4 * i + quarter;
        k_off[i] = (uint32_t)(r * HEAD_DIM + ((l16 ^ r) << 3)) * 2;
        v_off[i] = (uint32_t)(r * HEAD_DIM + ((l16 ^ (4 * (r & 3))) << 3)) * 2;
    }
    auto issue = [&](int kt, unsigned char* tile) {
        unsigned char* kdst = tile + wave * (16 * HEAD_DIM * 2);
        const int s0 = kt * BN + 16 * wave;                                 // the wave's first key
        if (page >= 16 && s0 + 15 <= last_pos) {
            const int pg = __builtin_amdgcn_readfirstlane(s_page[(s0 >> page_shift) - first_block]);
            const size_t base = (((size_t)pg * n_kv + kvh) * page + (s0 & (page - 1))) * (HEAD_DIM * 2);
            const unsigned char* kb = (const unsigned char*)k_cache + base;
            const unsigned char* vb = (const unsigned char*)v_cache + base;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                __builtin_amdgcn_global_load_lds(GLOBAL_PTR(kb + k_off[i]), LDS_PTR(kdst + 1024 * i), 16, 0, 0);
                __builtin_amdgcn_global_load_lds(GLOBAL_PTR(vb + v_off[i]), LDS_PTR(kdst + TILE_BYTES + 1024 * i), 16, 0, 0);
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 16 * wave + 4 * i + quarter;                      // row of the tile
            const int sc = min(kt * BN + r, last_pos);
            const size_t at = (((size_t)s_page[(sc >> page_shift) - first_block] * n_kv + kvh) * page + (sc & (page - 1))) * HEAD_DIM;
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(k_cache + at + ((l16 ^ (r & 15)) << 3)), LDS_PTR(kdst + 1024 * i), 16, 0, 0);
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(v_cache + at + ((l16 ^ (4 * (r & 3))) << 3)),
                                             LDS_PTR(kdst + TILE_BYTES + 1024 * i), 16, 0, 0);
        }
    };

    // a lane's places in the operands.  Keys: row 32 j + l32, chunk 2 t + hh.  Values, transposed read for the
    // 32 columns of tile dt: this lane gives the address of row 4 hh + l16 / 4 (+ 32 j + 16 st, + 8 for the second
    // half of the step), columns 32 dt + 16 (quarter % 2) + 4 (l16 % 4) .. + 3
    const int v_row = 4 * hh + (l16 >> 2);
    int v_at[DTILES], k_at[QSTEPS];
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
        v_at[dt] = TILE_BYTES + v_row * 256 +
                   ((((4 * dt + 2 * (quarter & 1) + ((l16 & 3) >> 1)) ^ (4 * (v_row & 3))) << 4) | ((l16 & 1) << 3));
#pragma unroll
    for (int t = 0; t < QSTEPS; ++t) k_at[t] = l32 * 256 + (((2 * t + hh) ^ (l32 & 15)) << 4);

    // one tile: `Ks` holds it (keys, then values), the next one goes to `next`
    auto work_tile = [&](int kt, const unsigned char* Ks, unsigned char* next) {
        const int key0 = kt * BN;
        __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0): this wave's part of the tile is in LDS
        __syncthreads();                         // every part is; and the other buffer has been read by every wave
        if (kt < tile_hi) issue(kt + 1, next);
        if (!wave_active) return;

        // ---- S^T = K Q^T for the two 32-key halves of the tile
        // The key operands of step t + 2 are asked for before the products of step t: a read out of LDS takes
        // longer than the two products of a step, and asked for right in front of them it is waited for every
        // step.  Written out, with waits that count: left to the compiler every wait is for all reads on their way.
        static_assert(QSTEPS == 8, "the waits below are written for eight steps");
        f32x16 s_acc[2];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) s_acc[j][v] = 0.0f;
        u32x4 kf[3][2];
        const uint32_t k_lds = (uint32_t)(uintptr_t)LDS_PTR(Ks);
#define KIPP_K_READ(T)                                                                                              \
    _Pragma("unroll") for (int j = 0; j < 2; ++j)                                                                   \
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(kf[(T) % 3][j]) : "v"(k_lds + k_at[T]), "i"(j * (32 * 256)))
#define KIPP_K_STEP(T, N)                                                                                           \
    do {                                                                                                            \
        asm volatile("s_waitcnt lgkmcnt(" #N ")" : "+v"(kf[(T) % 3][0]), "+v"(kf[(T) % 3][1]));                      \
        _Pragma("unroll") for (int j = 0; j < 2; ++j) {                                                             \
            Frag f;                                                                                                 \
            f.u = kf[(T) % 3][j];                                                                                   \
            s_acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.v, qf[T].v, s_acc[j], 0, 0, 0);                    \
        }                                                                                                           \
        __builtin_amdgcn_sched_barrier(0);   /* the order written here is the order meant */                       \
    } while (0)
        KIPP_K_READ(0);
        KIPP_K_READ(1);
        KIPP_K_READ(2);
        KIPP_K_STEP(0, 4);
        KIPP_K_READ(3);
        KIPP_K_STEP(1, 4);
        KIPP_K_READ(4);
        KIPP_K_STEP(2, 4);
        KIPP_K_READ(5);
        KIPP_K_STEP(3, 4);
        KIPP_K_READ(6);
        KIPP_K_STEP(4, 4);
        KIPP_K_READ(7);
        KIPP_K_STEP(5, 4);
        KIPP_K_STEP(6, 2);
        KIPP_K_STEP(7, 0);
#undef KIPP_K_READ
#undef KIPP_K_STEP
        const bool masked = key0 + BN - 1 > pos0 + wave * 32 || window > 0;
        if (masked) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int s = key0 + 32 * j + 8 * (v / 4) + 4 * hh + (v % 4);
                    if (s > my_pos || s < my_lo) s_acc[j][v] = -INFINITY;
                }
        }
        float m_tile = -INFINITY;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) m_tile = fmaxf(m_tile, s_acc[j][v]);
        m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, KIPP_WAVE));
        // The exponents are taken against a reference maximum that follows the true one only when some
        // query's maximum has moved by more than 8 (a weight is then at most 2^8, sums and products stay
        // far inside float32): what has been gathered is rescaled on few tiles instead of on most.
        const float m_new = fmaxf(m_run, m_tile);
        if (__any((m_new - m_run) * scale_log2e > 8.0f)) {           // the first visible key: -inf to finite
            // 0 at a query's first visible key, 1 where nothing moved or nothing is visible yet
            const float alpha = m_new == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f((m_run - m_new) * scale_log2e);
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
                for (int v = 0; v < 16; ++v) o[dt][v] *= alpha;
            m_run = m_new;
        }
        const float m_scaled = (m_run == -INFINITY ? 0.0f : m_run) * scale_log2e;   // nothing visible yet: every weight is 0
        float l_tile = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float p = __builtin_amdgcn_exp2f(fmaf(s_acc[j][v], scale_log2e, -m_scaled));
                s_acc[j][v] = p;
                l_tile += p;
            }
        l_tile += __shfl_xor(l_tile, 32, KIPP_WAVE);
        l_run += l_tile;
        // ---- O^T += V^T P^T in four steps of 16 keys; the second half of a step lies 8 rows (2,048 bytes)
        //      further.  The transposed reads are written out: through the intrinsic the compiler makes each wait
        //      for every load into LDS that is on its way, the next tile's included.  The reads of step s + 1 are
        //      asked for before step s is multiplied.
        static_assert(DTILES == 4, "the waits below count eight transposed reads a step");
        uint32_t v_lds[DTILES];
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt) v_lds[dt] = (uint32_t)(uintptr_t)LDS_PTR(Ks + v_at[dt]);
        u32x2 vt[2][2 * DTILES];
#define KIPP_READ_STEP(S, STEP)                                                                                      \
    _Pragma("unroll") for (int dt = 0; dt < DTILES; ++dt) {                                                          \
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(vt[S][2 * dt]) : "v"(v_lds[dt]), "i"((STEP) * 4096)); \
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2"                                                           \
                     : "=v"(vt[S][2 * dt + 1])                                                                       \
                     : "v"(v_lds[dt]), "i"((STEP) * 4096 + 2048));                                                   \
    }
#define KIPP_WAIT_STEP(S, N)                                                                                     \
    asm volatile("s_waitcnt lgkmcnt(" #N ")"                                                                     \
                 : "+v"(vt[S][0]), "+v"(vt[S][1]), "+v"(vt[S][2]), "+v"(vt[S][3]), "+v"(vt[S][4]), "+v"(vt[S][5]), \
                   "+v"(vt[S][6]), "+v"(vt[S][7]))
        auto multiply_step = [&](const u32x2* set, int step) {
            const int j = step >> 1, st = step & 1;
            Frag pf;
            pf.u = (u32x4){pack_bf16(s_acc[j][8 * st + 0], s_acc[j][8 * st + 1]), pack_bf16(s_acc[j][8 * st + 2], s_acc[j][8 * st + 3]),
                           pack_bf16(s_acc[j][8 * st + 4], s_acc[j][8 * st + 5]), pack_bf16(s_acc[j][8 * st + 6], s_acc[j][8 * st + 7])};
#pragma unroll
            for (int dt = 0; dt < DTILES; ++dt) {
                Frag vf;
                vf.u = (u32x4){set[2 * dt][0], set[2 * dt][1], set[2 * dt + 1][0], set[2 * dt + 1][1]};
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf.v, pf.v, o[dt], 0, 0, 0);
            }
        };
        KIPP_READ_STEP(0, 0)
        KIPP_READ_STEP(1, 1)
        KIPP_WAIT_STEP(0, 8);
        multiply_step(vt[0], 0);
        KIPP_READ_STEP(0, 2)
        KIPP_WAIT_STEP(1, 8);
        multiply_step(vt[1], 1);
        KIPP_READ_STEP(1, 3)
        KIPP_WAIT_STEP(0, 8);
        multiply_step(vt[0], 2);
        KIPP_WAIT_STEP(1, 0);
        multiply_step(vt[1], 3);
#undef KIPP_READ_STEP
#undef KIPP_WAIT_STEP
    };
    issue(tile_lo, tile_a);
    for (int kt = tile_lo; kt <= tile_hi; kt += 2) {
        work_tile(kt, tile_a, tile_b);
        if (kt + 1 <= tile_hi) work_tile(kt + 1, tile_b, tile_a);
    }
    if (!row_valid) return;
    if (split_keys > 0) {
        // one cut of the keys: the sums as they are, with their reference maximum (base 2) and their
        // denominator; attention_prefill_merge_kernel adds the cuts of a row in order
        const size_t slot = ((size_t)(row0 + my_row) * n_q + head) * max_splits + split;
        if (hh == 0) {
            part_ml[slot * 2] = m_run == -INFINITY ? -INFINITY : m_run * scale_log2e;
            part_ml[slot * 2 + 1] = l_run;
        }
        float* p_row = part_acc + slot * HEAD_DIM;
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int dcol = 32 * dt + 8 * g + 4 * hh;
                if (dcol < HEAD_DIM) *(f32x4*)(p_row + dcol) = (f32x4){o[dt][4 * g + 0], o[dt][4 * g + 1], o[dt][4 * g + 2], o[dt][4 * g + 3]};
            }
        return;
    }
    const float inv = 1.0f / l_run;
    bf16_t* o_row = out + ((size_t)(row0 + my_row) * n_q + head) * HEAD_DIM;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int dcol = 32 * dt + 8 * g + 4 * hh;
            *(u32x2*)(o_row + dcol) = (u32x2){pack_bf16(o[dt][4 * g + 0] * inv, o[dt][4 * g + 1] * inv),
                                              pack_bf16(o[dt][4 * g + 2] * inv, o[dt][4 * g + 3] * inv)};
        }
}
#endif  // HEAD_DIM == 128

// The cuts of a row's keys, added in order: out = sum_s acc_s 2^(m_s - m) / sum_s l_s 2^(m_s - m).  A workgroup takes
// MERGE_HEADS heads of a row, a thread four neighbouring elements of one of them; the cuts are read four at a time, all
// asked for before the first is added.  How many cuts a row has follows from the last position of the tile of query
// rows it lies in (every row of a tile has the tile's cuts; a cut that begins behind a row's own position holds
// nothing: m = -inf, l = 0).
#define MERGE_LANES (HEAD_DIM / 4)               // threads of a head
#define MERGE_HEADS (256 / MERGE_LANES > 0 ? 256 / MERGE_LANES : 1)
__global__ void __launch_bounds__(MERGE_HEADS * MERGE_LANES) attention_prefill_merge_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml, bf16_t* __restrict__ out,
    const int32_t* __restrict__ merge_rows, const int32_t* __restrict__ merge_cuts, int n_q, int max_splits) {
    // rows on the grid's x, which takes as many as a step has (y ends at 65,535)
    const int head = blockIdx.y * MERGE_HEADS + threadIdx.x / MERGE_LANES, dcol = 4 * (threadIdx.x % MERGE_LANES);
    if (head >= n_q) return;
    const int row = merge_rows[blockIdx.x], cuts = merge_cuts[blockIdx.x];
    const size_t slot0 = ((size_t)row * n_q + head) * max_splits;
    const float2* ml = (const float2*)part_ml + slot0;
    float m = -INFINITY;
    for (int s0 = 0; s0 < cuts; s0 += 4) {
        float ms[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) ms[q] = s0 + q < cuts ? ml[s0 + q].x : -INFINITY;
#pragma unroll
        for (int q = 0; q < 4; ++q) m = fmaxf(m, ms[q]);
    }
    float denom = 0.0f;
    f32x4 a = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    for (int s0 = 0; s0 < cuts; s0 += 4) {
        float2 one[4];
        f32x4 acc[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int s = min(s0 + q, cuts - 1);
            one[q] = ml[s];
            acc[q] = *(const f32x4*)(part_acc + (slot0 + s) * HEAD_DIM + dcol);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (s0 + q < cuts && one[q].x != -INFINITY) {
                const float w = exp2f(one[q].x - m);
                denom += one[q].y * w;
                a += acc[q] * w;
            }
        }
    }
    bf16_t* o = out + ((size_t)row * n_q + head) * HEAD_DIM + dcol;
    *(u32x2*)o = (u32x2){pack_bf16(a[0] / denom, a[1] / denom), pack_bf16(a[2] / denom, a[3] / denom)};
}

extern "C" {

int kipp_attention_prefill_rows() { return BM; }

// `item_seq[i]`, `item_tile[i]`: sequence (row of the block table) and tile of `tile_rows` query rows
// of its portion for work item i; best sorted from the longest key range to the shortest.
// `tile_rows`: 128, or 64 or 32 where the items of 128 rows would leave compute units idle (a wave takes
// 32 rows; with fewer rows the other waves of a workgroup only help to bring keys and values in).
int kipp_attention_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                           const int32_t* item_seq, const int32_t* item_tile, const int32_t* q_start,
                           const int32_t* q_len, const int32_t* positions, const int32_t* block_table, int max_blocks,
                           int n_items, int n_q, int n_kv, int head_dim, int page, float scale, int window,
                           int tile_rows, const int32_t* item_split, int split_keys, float* part_acc, float* part_ml,
                           int max_splits, const int32_t* merge_rows, const int32_t* merge_cuts, int n_merge,
                           hipStream_t stream) {
    if (n_items <= 0) return 0;
    if (head_dim != HEAD_DIM || n_kv <= 0 || n_q % n_kv) return -1;
    if (tile_rows != 128 && tile_rows != 64 && tile_rows != 32) return -7;
    // keys cut at multiples of `split_keys` (0: not cut): work item i then takes cut item_split[i] and writes sums that
    // are not normalised yet into part_acc [rows, n_q, max_splits, head_dim] / part_ml [.., 2]; rows merge_rows[j] with
    // merge_cuts[j] cuts are merged afterwards.  Windows are not cut.
    if (split_keys < 0 || (split_keys % BN) || (split_keys > 0 && (window > 0 || !item_split || !part_acc || !part_ml ||
                                                                    max_splits <= 0 || !merge_rows || !merge_cuts)))
        return -8;
    if (page <= 0 || (page & (page - 1))) return -4;   // pages of a power of two only
    if (max_blocks > MAX_PAGES) return -5;             // the table row is staged in LDS
    const float scale_log2e = scale * 1.4426950408889634f;
#if HEAD_DIM == 128 && PREFILL_DMA
    if (true) {
        static bool prepared = false;
        if (!prepared) {
            if (hipFuncSetAttribute((const void*)attention_prefill_dma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    DMA_LDS_BYTES + MAX_PAGES * 4) != hipSuccess) return -6;
            prepared = true;
        }
        hipLaunchKernelGGL(attention_prefill_dma_kernel, dim3(n_items * n_q), dim3(THREADS), DMA_LDS_BYTES + max_blocks * 4,
                           stream, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, item_seq,
                           item_tile, q_start, q_len, positions, block_table, max_blocks, n_q, n_kv, page, scale_log2e, window, tile_rows,
                           item_split, split_keys, part_acc, part_ml, max_splits);
    } else
#endif
    hipLaunchKernelGGL(attention_prefill_kernel, dim3(n_items * n_q), dim3(THREADS), 0, stream, (const bf16_t*)q,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, item_seq, item_tile, q_start, q_len,
                       positions, block_table, max_blocks, n_q, n_kv, page, scale_log2e, window, tile_rows, item_split,
                       split_keys, part_acc, part_ml, max_splits);
    if (split_keys > 0 && n_merge > 0)
        hipLaunchKernelGGL(attention_prefill_merge_kernel, dim3(n_merge, (n_q + MERGE_HEADS - 1) / MERGE_HEADS), dim3(MERGE_HEADS * MERGE_LANES), 0, stream, part_acc, part_ml,
                           (bf16_t*)out, merge_rows, merge_cuts, n_q, max_splits);
    return KIPP_LAUNCH_CHECK();
}

}  // extern "C"
