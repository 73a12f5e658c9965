// Decode attention over the paged cache, bfloat16, split over the keys.
//
// One query token per sequence.  A workgroup (4 waves) takes one sequence, one
// key/value head and one split of SPLIT keys; the GROUP query heads that share
// the key/value head are computed together, so every key and value is read
// once for all of them (/root/reference/metal/kipp_kernels.metal:517-626 plays this
// role in the reference, with 1024-key splits and no sharing across heads).
//
//   scores   S^T[key][head] = K . Q^T on the matrix cores: the A operand of
//            v_mfma_f32_16x16x32_bf16 is a block of 16 key rows read straight
//            from global memory (16 bytes a lane), B holds the GROUP queries;
//   softmax  over the split's keys in float32, in LDS, base 2;
//   values   lanes own 8 columns of a value row; 16 lanes read one row (256 B
//            at head size 128), the 16 lane groups of the workgroup take every
//            16th key; products in float32 FMA, summed over the groups in LDS.
//
// Split boundaries are multiples of the split's length in absolute key index, and the
// merge adds the splits in index order, so within one launch shape the result for a
// token does not depend on what else is in the batch.  The split's length (192, 256 or
// 320 keys) and the kernel follow from the launch's shape (rows, key/value heads,
// longest context), so between shapes, batch 1 and batch 8 say, a token's bits may
// differ in the last place.  A sequence that needs one split only is written
// normalised at once.  The merge is done by whichever workgroup of a (token,
// key/value head) finishes last: every workgroup writes its partial result
// through to memory (stores of device scope: the dies' L2 caches do not see each
// other's lines), waits until the stores have arrived, and adds one to the
// head's count with an atomic of device scope; the one that brings the count to
// the number of splits reads all partial results from memory (loads of device
// scope), merges them and sets the count back to zero.  Nobody waits for
// anybody, no fence is needed (a fence of device scope writes a die's whole L2
// back: 40 us), and the sums are those of attention_decode_reduce_kernel in the
// same order, which a caller without the counts still gets as a second launch
// (4.7 us a layer; merged here a decode step at batch 8 is 1 % shorter).
//
// FUSED: the kernel starts from the output of the QKV projection instead of from
// finished queries.  Each workgroup norms and rotates the GROUP queries of its
// key/value head itself (a wave a head, element i and its rotation partner
// i + d/2 in one lane, as in the rotary kernel), and the workgroup of the split
// that holds the token's own position does the same for the new key, takes the
// new value, writes both into the cache and uses them from LDS.  A decode step
// then needs no rotary kernel.  Head sizes that are multiples of 128, rotated
// over their whole width.
//
// Compile-time: HEAD_DIM (multiple of 16, <= 256), GROUP (query heads per
// key/value head, <= 16).
#include "common.h"
#include <math.h>
#include <type_traits>

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
#ifndef GROUP
#error "compile with -DGROUP=<query heads per key/value head>"
#endif

#define SPLIT 256                              // keys of a split (the kernel that takes one a workgroup also has longer ones)
#define SPLIT_MIN 192                          // the shortest (few sequences)
#define SPLIT_MAX 320                          // the longest (the fused form has registers for no more with two workgroups a compute unit)
#define WAVES 4
#define THREADS (WAVES * KIPP_WAVE)
#define KSTEPS ((HEAD_DIM + 31) / 32)          // MFMA steps of 32 over the head size
#define CHUNKS (HEAD_DIM / 8)                  // 16-byte chunks of a row
#define CHUNKS_PER_LANE ((CHUNKS + 15) / 16)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

union Frag {
    u32x4 u;
    bf16x8 v;
};

#define FUSED_OK ((HEAD_DIM % 128) == 0)
#define NC (HEAD_DIM / KIPP_WAVE)              // elements of a head a lane holds when a wave takes a head
#define JOBS ((GROUP + 2 + WAVES - 1) / WAVES)  // heads a wave prepares: GROUP queries, the new key, the new value
#define MAX_SLABS 4                            // slabs of the projection the fused kernel adds

// What the fused kernel needs beside the attention itself.
struct Projected {
    const float* qkv;        // [parts][tokens][(n_q + 2 n_kv) HEAD_DIM], slabs added in order
    int parts;
    size_t part_stride;
    const float* q_norm_w;   // null: no norm
    const float* k_norm_w;
    float eps;
    const float* inv_freq;   // null (and angles null): no rotation
    const float* angles;     // [tokens][HEAD_DIM]: cosines then sines of every token's angles, or null: computed here
    int write_kv;            // 0: the cache is another layer's, keys and values are already there
    int out_rows;            // > 0: `out` is written as [n_q HEAD_DIM / 32][out_rows][32] for the product that reads it next (below)
};

// Where element `col` of row `row` of the mixed heads lies: [row][width], or with `out_rows` > 0 in the order the
// few-rows products read their rows fastest, [width / 32][out_rows][32] (a wave's 64 bytes of each row are then one run).
__device__ __forceinline__ size_t out_at(int row, int col, int width, int out_rows) {
    return out_rows > 0 ? ((size_t)(col >> 5) * out_rows + row) * 32 + (col & 31) : (size_t)row * width + col;
}

// Values that another workgroup of the same launch reads: written through to memory and read from there (the
// dies' L2 caches do not see each other's lines).  A store is known to have arrived once the wave's count of
// outstanding memory operations is back to zero.
__device__ __forceinline__ void store_through(float* p, float v) {
    __hip_atomic_store((unsigned*)p, __float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_through(const float* p) {
    return __uint_as_float(__hip_atomic_load((const unsigned*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}

// two neighbouring values at an address that 8 divides
__device__ __forceinline__ float2 load_through2(const float* p) {
    const unsigned long long bits = __hip_atomic_load((const unsigned long long*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return make_float2(__uint_as_float((unsigned)bits), __uint_as_float((unsigned)(bits >> 32)));
}

// The merge of attention_decode_reduce_kernel (the same sums in the same order) by the workgroup that finished
// last among the splits of a (token, key/value head): elements `dcol` and `dcol` + 1 (dcol even) of head `head`.
// A split costs a thread two loads of 8 bytes: its maximum with its denominator, and the two sums.
__device__ __forceinline__ float2 merge_splits_here(const float* part_acc, const float* part_ml, size_t slot0, int n_splits, int dcol) {
    constexpr int AT_ONCE = 16;
    float2 ml_s[AT_ONCE], a_s[AT_ONCE];
    // the first 16 splits are asked for together
#pragma unroll
    for (int i = 0; i < AT_ONCE; ++i) {
        ml_s[i] = make_float2(-INFINITY, 0.0f);
        a_s[i] = make_float2(0.0f, 0.0f);
        if (i < n_splits) {
            ml_s[i] = load_through2(part_ml + (slot0 + i) * 2);
            a_s[i] = load_through2(part_acc + (slot0 + i) * HEAD_DIM + dcol);
        }
    }
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < AT_ONCE; ++i) m = fmaxf(m, ml_s[i].x);
    for (int s = AT_ONCE; s < n_splits; ++s) m = fmaxf(m, load_through(part_ml + (slot0 + s) * 2));
    float denom = 0.0f;
    float2 a = make_float2(0.0f, 0.0f);
#pragma unroll
    for (int i = 0; i < AT_ONCE; ++i) {
        if (i < n_splits) {
            const float w = exp2f(ml_s[i].x - m);
            denom += ml_s[i].y * w;
            a.x += a_s[i].x * w;
            a.y += a_s[i].y * w;
        }
    }
    for (int s = AT_ONCE; s < n_splits; ++s) {
        const float2 ml = load_through2(part_ml + (slot0 + s) * 2), more = load_through2(part_acc + (slot0 + s) * HEAD_DIM + dcol);
        const float w = exp2f(ml.x - m);
        denom += ml.y * w;
        a.x += more.x * w;
        a.y += more.y * w;
    }
    return make_float2(a.x / denom, a.y / denom);
}

__device__ __forceinline__ void store_through2(float* p, float a, float b) {
    __hip_atomic_store((unsigned long long*)p, (unsigned long long)__float_as_uint(a) | ((unsigned long long)__float_as_uint(b) << 32),
                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Two neighbouring elements (dcol even) of a split's partial result.  With `arrivals` the splits are merged inside this launch.
__device__ __forceinline__ void put_partial2(const unsigned* arrivals, float* part_acc, float* part_ml, size_t slot, int dcol,
                                             float a0, float a1, float m, float l) {
    if (arrivals != nullptr) {
        store_through2(part_acc + slot * HEAD_DIM + dcol, a0, a1);
        if (dcol == 0) store_through2(part_ml + slot * 2, m, l);
    } else {
        *(float2*)(part_acc + slot * HEAD_DIM + dcol) = make_float2(a0, a1);
        if (dcol == 0) *(float2*)(part_ml + slot * 2) = make_float2(m, l);
    }
}

// One element of a split's partial result.  With `arrivals` the splits are merged inside this launch.
__device__ __forceinline__ void put_partial(const unsigned* arrivals, float* part_acc, float* part_ml, size_t slot, int dcol,
                                            float a, float m, float l) {
    if (arrivals != nullptr) {
        store_through(part_acc + slot * HEAD_DIM + dcol, a);
        if (dcol == 0) {
            store_through(part_ml + slot * 2, m);
            store_through(part_ml + slot * 2 + 1, l);
        }
    } else {
        part_acc[slot * HEAD_DIM + dcol] = a;
        if (dcol == 0) {
            part_ml[slot * 2] = m;
            part_ml[slot * 2 + 1] = l;
        }
    }
}

// The end of a workgroup that has put one of several splits of (token `item`, key/value head `kvh`): it counts
// itself once what it wrote has arrived, and the one that counts last merges the splits, in split order.  Nobody
// waits for anybody.  Called by all threads of the workgroup.
__device__ __forceinline__ void merge_by_the_last(unsigned* arrivals, const float* part_acc, const float* part_ml, bf16_t* out,
                                                  int item, int row, int kvh, int n_q, int n_kv, int max_splits, int n_splits,
                                                  int out_rows = 0) {
    __shared__ int s_last;
    const int tid = threadIdx.x;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
        unsigned* count = arrivals + (size_t)item * n_kv + kvh;
        const unsigned before = __hip_atomic_fetch_add(count, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int last = before + 1u == (unsigned)n_splits;
        if (last) __hip_atomic_store(count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // as the next launch expects it
        s_last = last;
    }
    __syncthreads();
    if (!s_last) return;
    for (int idx = tid; idx < GROUP * HEAD_DIM / 2; idx += THREADS) {
        const int g = idx / (HEAD_DIM / 2), dcol = 2 * (idx % (HEAD_DIM / 2));
        const int head = kvh * GROUP + g;
        const size_t slot0 = ((size_t)item * n_q + head) * max_splits;
        const float2 merged = merge_splits_here(part_acc, part_ml, slot0, n_splits, dcol);
        // two neighbouring columns lie side by side in either order of the rows (runs of 32 columns)
        *(uint32_t*)(out + out_at(row, head * HEAD_DIM + dcol, n_q * HEAD_DIM, out_rows)) =
            (uint32_t)f32_to_bf16(merged.x) | ((uint32_t)f32_to_bf16(merged.y) << 16);
    }
}

template <bool FUSED, int SPLIT_T>
__global__ void __launch_bounds__(THREADS) attention_decode_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const int32_t* __restrict__ rows, const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks, int n_q, int n_kv, int page, float scale_log2e,
    int window, int max_splits, Projected pj, unsigned* arrivals) {
    static_assert(SPLIT_T % (16 * WAVES) == 0 && SPLIT_T <= 2 * THREADS, "whole blocks of 16 keys a wave; at most two pages a thread");
    constexpr int BPW = SPLIT_T / 16 / WAVES;         // 16-key blocks a wave scores
    constexpr int KPG = SPLIT_T / 16;                 // keys a lane group multiplies with values
    __shared__ float s_scores[GROUP][SPLIT_T + 4];
    __shared__ __attribute__((aligned(16))) bf16_t s_new[FUSED ? GROUP + 2 : 1][HEAD_DIM];
    __shared__ float s_red[WAVES][GROUP][HEAD_DIM];
    __shared__ float s_m[GROUP], s_l[GROUP];
    __shared__ int s_page[SPLIT_T + 2];                 // page of every key of the split (any page size)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, h = lane >> 4;
    const int kvh = blockIdx.y;
    // The grid is (query tokens, key/value heads, splits): workgroups are handed out in that order, so those of
    // splits beyond a sequence's position, which the grid has for the longest context it was recorded for,
    // come last and leave at once instead of holding a place that a working one waits for.
    const int row = rows[blockIdx.x];                 // row of this query token in the batch
    const int pos = positions[row];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int first_split = lo / SPLIT_T, last_split = pos / SPLIT_T;
    const int split = first_split + blockIdx.z;
    if (split > last_split) return;                   // the grid covers the longest sequence
    const int n_splits = last_split - first_split + 1;
    const int base = split * SPLIT_T;
    const int32_t* table = block_table + (size_t)seq_of_token[row] * max_blocks;

    // Pages first, once, into LDS: the loads of keys and values below then depend on
    // nothing that is still in flight and can all be issued back to back.  Keys beyond
    // the query's position read the last valid page (finite values, masked later).
    const int page_shift = __builtin_ctz(page);          // the page size is a power of two (checked by the launcher)
    int my_page[2] = {0, 0};
#pragma unroll
    for (int i = 0; i < 2; ++i)
        if (tid + THREADS * i < SPLIT_T) my_page[i] = table[min(base + tid + THREADS * i, pos) >> page_shift];

    // ---- fused: ask for the projected heads this wave prepares, and for what their norm and
    // rotation need, before the keys and values are asked for: they are wanted first
    const bool owner = FUSED && pj.write_kv && split == last_split;   // this workgroup holds the token's own position
#if FUSED_OK
    float raw[JOBS][NC], norm_q[NC], norm_k[NC], freq[NC / 2], cs[NC / 2], sn[NC / 2];
    if (FUSED) {
        const size_t width = (size_t)(n_q + 2 * n_kv) * HEAD_DIM;
        int last_slab = pj.parts - 1;
        asm volatile("" : "+s"(last_slab));          // opaque: every slab load below is issued, none waits for a branch
#pragma unroll
        for (int jj = 0; jj < JOBS; ++jj) {
            const int j = wave + jj * WAVES;
            const bool valid = j < GROUP || (owner && j < GROUP + 2);
            const int slot = !valid ? 0 : (j < GROUP ? kvh * GROUP + j : (j == GROUP ? n_q + kvh : n_q + n_kv + kvh));
            const float* src = pj.qkv + (size_t)row * width + (size_t)slot * HEAD_DIM + lane;
            // every slab is asked for before any is used, then they are added in order.  A slab index
            // beyond `parts` reads the last slab again and enters with the factor 0: no branch, so no
            // load can be moved behind one and waited for on its own
            float slab[NC][MAX_SLABS];
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int p = 0; p < MAX_SLABS; ++p)
                    slab[c][p] = src[(size_t)min(p, last_slab) * pj.part_stride + c * KIPP_WAVE];
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                raw[jj][c] = slab[c][0];
#pragma unroll
                for (int p = 1; p < MAX_SLABS; ++p) raw[jj][c] += (p <= last_slab ? 1.0f : 0.0f) * slab[c][p];
            }
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            norm_q[c] = pj.q_norm_w != nullptr ? pj.q_norm_w[lane + c * KIPP_WAVE] : 1.0f;
            norm_k[c] = pj.k_norm_w != nullptr ? pj.k_norm_w[lane + c * KIPP_WAVE] : 1.0f;
        }
#pragma unroll
        for (int c = 0; c < NC / 2; ++c) {
            freq[c] = 0.0f;
            cs[c] = 1.0f;
            sn[c] = 0.0f;
            if (pj.angles != nullptr) {
                cs[c] = pj.angles[(size_t)row * HEAD_DIM + lane + c * KIPP_WAVE];
                sn[c] = pj.angles[(size_t)row * HEAD_DIM + HEAD_DIM / 2 + lane + c * KIPP_WAVE];
            } else if (pj.inv_freq != nullptr) {
                freq[c] = pj.inv_freq[lane + c * KIPP_WAVE];
            }
        }
    }
#endif
#pragma unroll
    for (int i = 0; i < 2; ++i)
        if (tid + THREADS * i < SPLIT_T) s_page[tid + THREADS * i] = my_page[i];
    __syncthreads();

    // ---- the GROUP queries as B operand: lane (slot l16, quarter h) holds q[slot][32 t + 8 h .. + 7]
    Frag qf[KSTEPS];
    if (!FUSED) {
#pragma unroll
        for (int t = 0; t < KSTEPS; ++t) {
            const int dcol = min(32 * t + 8 * h, HEAD_DIM - 8);
            qf[t].u = *(const u32x4*)(q + ((size_t)row * n_q + (size_t)kvh * GROUP + min(l16, GROUP - 1)) * HEAD_DIM + dcol);
        }
    }

    // ---- scores: each wave takes BPW blocks of 16 keys; every load is unconditional
    Frag kf[BPW][KSTEPS];
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
        const int kl = (wave * BPW + b) * 16 + l16;
        const int s = min(base + kl, pos);
        const bf16_t* k_row = k_cache + (((size_t)s_page[kl] * n_kv + kvh) * page + (s & (page - 1))) * HEAD_DIM;
#pragma unroll
        for (int t = 0; t < KSTEPS; ++t) kf[b][t].u = *(const u32x4*)(k_row + min(32 * t + 8 * h, HEAD_DIM - 8));
    }
    // ---- values are asked for now, so that they arrive while the scores are worked on
    Frag vf[KPG][CHUNKS_PER_LANE];
    const int kg = wave * 4 + h;                      // this lane group's keys: base + kg + 16 i
#pragma unroll
    for (int i = 0; i < KPG; ++i) {
        const int kl = kg + 16 * i;
        const int s = min(base + kl, pos);
        const bf16_t* v_row = v_cache + (((size_t)s_page[kl] * n_kv + kvh) * page + (s & (page - 1))) * HEAD_DIM;
#pragma unroll
        for (int c = 0; c < CHUNKS_PER_LANE; ++c) vf[i][c].u = *(const u32x4*)(v_row + min(l16 + 16 * c, CHUNKS - 1) * 8);
    }
#if FUSED_OK
    if (FUSED) {
        // norm (/root/reference/src/kipp.c:2480-2500), rotation (kipp.c:2368-2382), in the arithmetic of
        // the rotary kernel; the keys and values asked for above are on their way meanwhile
        if (pj.angles == nullptr && pj.inv_freq != nullptr) {
#pragma unroll
            for (int c = 0; c < NC / 2; ++c) {
                const float angle = (float)pos * freq[c];
                cs[c] = cosf(angle);
                sn[c] = sinf(angle);
            }
        }
        const int own_slot = pos - base;             // the token's own key within this split (owner only)
#pragma unroll
        for (int jj = 0; jj < JOBS; ++jj) {
            const int j = wave + jj * WAVES;
            if (!(j < GROUP || (owner && j < GROUP + 2))) continue;
            if (j <= GROUP) {
                if ((j < GROUP ? pj.q_norm_w : pj.k_norm_w) != nullptr) {
                    float ss = 0.0f;
#pragma unroll
                    for (int c = 0; c < NC; ++c) ss = square_add(ss, raw[jj][c]);
                    ss = wave_sum(ss);
                    const float r = head_norm_scale(ss, (float)HEAD_DIM, pj.eps);
#pragma unroll
                    for (int c = 0; c < NC; ++c) raw[jj][c] *= r * (j < GROUP ? norm_q[c] : norm_k[c]);
                }
#pragma unroll
                for (int c = 0; c < NC / 2; ++c) {
                    const float a = raw[jj][c], b = raw[jj][c + NC / 2];
                    raw[jj][c] = rotate_lo(a, b, cs[c], sn[c]);
                    raw[jj][c + NC / 2] = rotate_hi(a, b, cs[c], sn[c]);
                }
            }
            bf16_t* dst = nullptr;
            if (j >= GROUP)
                dst = (j == GROUP ? k_cache : v_cache) +
                      (((size_t)s_page[own_slot] * n_kv + kvh) * page + (pos & (page - 1))) * HEAD_DIM;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const bf16_t bits = f32_to_bf16(raw[jj][c]);
                s_new[j][lane + c * KIPP_WAVE] = bits;
                if (dst != nullptr) dst[lane + c * KIPP_WAVE] = bits;
            }
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < KSTEPS; ++t)
            qf[t].u = *(const u32x4*)(&s_new[min(l16, GROUP - 1)][min(32 * t + 8 * h, HEAD_DIM - 8)]);
        if (owner) {                                  // the token's own key and value come from LDS, not from the cache
#pragma unroll
            for (int b = 0; b < BPW; ++b)
                if ((wave * BPW + b) * 16 + l16 == own_slot) {
#pragma unroll
                    for (int t = 0; t < KSTEPS; ++t)
                        kf[b][t].u = *(const u32x4*)(&s_new[GROUP][min(32 * t + 8 * h, HEAD_DIM - 8)]);
                }
#pragma unroll
            for (int i = 0; i < KPG; ++i)
                if (kg + 16 * i == own_slot) {
#pragma unroll
                    for (int c = 0; c < CHUNKS_PER_LANE; ++c)
                        vf[i][c].u = *(const u32x4*)(&s_new[GROUP + 1][min(l16 + 16 * c, CHUNKS - 1) * 8]);
                }
        }
    }
#endif
    // operands that reach beyond the head size or the group were read from clamped addresses: zero them
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t)
        if (32 * t + 8 * h >= HEAD_DIM || l16 >= GROUP) qf[t].u = (u32x4){0u, 0u, 0u, 0u};
#pragma unroll
    for (int b = 0; b < BPW; ++b) {
        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int t = 0; t < KSTEPS; ++t) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[b][t].v, qf[t].v, acc, 0, 0, 0);
        // acc[v] = S^T[key 4 h + v][slot l16]
        if (l16 < GROUP) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int kl = (wave * BPW + b) * 16 + 4 * h + v;
                const int s = base + kl;
                s_scores[l16][kl] = (s >= lo && s <= pos) ? acc[v] * scale_log2e : -INFINITY;
            }
        }
    }
    __syncthreads();

    // ---- softmax over the split's keys, one head per wave at a time
    for (int g = wave; g < GROUP; g += WAVES) {
        float sc[SPLIT_T / KIPP_WAVE];
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < SPLIT_T / KIPP_WAVE; ++i) {
            sc[i] = s_scores[g][lane + KIPP_WAVE * i];
            m = fmaxf(m, sc[i]);
        }
        m = wave_max(m);
        float l = 0.0f;
#pragma unroll
        for (int i = 0; i < SPLIT_T / KIPP_WAVE; ++i) {
            const float p = exp2f(sc[i] - m);          // -inf gives 0
            s_scores[g][lane + KIPP_WAVE * i] = p;
            l += p;
        }
        l = wave_sum(l);
        if (lane == 0) {
            s_m[g] = m;
            s_l[g] = l;
        }
    }
    __syncthreads();

    // ---- values: acc[g][c][j] += p[g][key] * v[key][8 chunk + j]
    float acc[GROUP][CHUNKS_PER_LANE][8];
#pragma unroll
    for (int g = 0; g < GROUP; ++g)
#pragma unroll
        for (int c = 0; c < CHUNKS_PER_LANE; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[g][c][j] = 0.0f;
#pragma unroll
    for (int i = 0; i < KPG; ++i) {
        const int kl = kg + 16 * i;
        float p[GROUP];
#pragma unroll
        for (int g = 0; g < GROUP; ++g) p[g] = s_scores[g][kl];
#pragma unroll
        for (int c = 0; c < CHUNKS_PER_LANE; ++c) {
            float vv[8];
#pragma unroll
            for (int j = 0; j < 8; ++j)
                vv[j] = __uint_as_float((j & 1) ? (vf[i][c].u[j >> 1] & 0xffff0000u) : (vf[i][c].u[j >> 1] << 16));
#pragma unroll
            for (int g = 0; g < GROUP; ++g)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[g][c][j] = fmaf(p[g], vv[j], acc[g][c][j]);
        }
    }
    // sum the four lane groups of the wave, then the waves
#pragma unroll
    for (int g = 0; g < GROUP; ++g)
#pragma unroll
        for (int c = 0; c < CHUNKS_PER_LANE; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float a = acc[g][c][j];
                a += __shfl_xor(a, 16, KIPP_WAVE);
                a += __shfl_xor(a, 32, KIPP_WAVE);
                acc[g][c][j] = a;
            }
    if (h == 0) {
#pragma unroll
        for (int g = 0; g < GROUP; ++g)
#pragma unroll
            for (int c = 0; c < CHUNKS_PER_LANE; ++c) {
                const int chunk = l16 + 16 * c;
                if (chunk < CHUNKS) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) s_red[wave][g][chunk * 8 + j] = acc[g][c][j];
                }
            }
    }
    __syncthreads();
    for (int idx = tid; idx < GROUP * HEAD_DIM / 2; idx += THREADS) {      // two neighbouring columns a thread
        const int g = idx / (HEAD_DIM / 2), dcol = 2 * (idx % (HEAD_DIM / 2));
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            a0 += s_red[w][g][dcol];
            a1 += s_red[w][g][dcol + 1];
        }
        const int head = kvh * GROUP + g;
        if (n_splits == 1) {
            *(uint32_t*)(out + out_at(row, head * HEAD_DIM + dcol, n_q * HEAD_DIM, FUSED ? pj.out_rows : 0)) =
                (uint32_t)f32_to_bf16(a0 / s_l[g]) | ((uint32_t)f32_to_bf16(a1 / s_l[g]) << 16);
        } else {
            put_partial2(arrivals, part_acc, part_ml, ((size_t)blockIdx.x * n_q + head) * max_splits + blockIdx.z, dcol, a0, a1, s_m[g], s_l[g]);
        }
    }
    if (arrivals != nullptr && n_splits > 1)
        merge_by_the_last(arrivals, part_acc, part_ml, out, blockIdx.x, row, kvh, n_q, n_kv, max_splits, n_splits, FUSED ? pj.out_rows : 0);
}

// ---------------------------------------------------------------------------------------------
// The same attention for long contexts.  A workgroup takes a long range of keys (BIG) and walks
// it in blocks of SUB keys with a running maximum and sum per head; while block i is worked on,
// the keys and values of block i + 1 are on their way into a second set of registers.  Against
// the kernel above this saves page lookups, partial results and merge work per key, which pays
// from several thousand keys on (measured: a sixth faster at 30,000 keys); at a few thousand
// keys the kernel above, which has more bytes in flight, is faster.  Partial results have the
// same layout, and the same merge kernel adds the ranges in order.
#define SUB 128
#define BIG 1024
#ifndef STREAM_FROM
#define STREAM_FROM 8192                         // keys from which the launcher takes this kernel
#endif
#define SUB_BLOCKS_PER_WAVE (SUB / 16 / WAVES)   // 16-key blocks of a sub-block that a wave scores
#define SUB_KEYS_PER_GROUP (SUB / 16)            // keys of a sub-block that a lane group multiplies with values

__global__ void __launch_bounds__(THREADS) attention_decode_stream_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const int32_t* __restrict__ rows, const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks, int n_q, int n_kv, int page, float scale_log2e,
    int window, int max_splits, unsigned* arrivals) {
    __shared__ float s_scores[GROUP][SUB + 4];
    __shared__ float s_red[WAVES][GROUP][HEAD_DIM];
    __shared__ float s_m[GROUP], s_l[GROUP], s_alpha[GROUP];
    __shared__ int s_page[BIG];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, h = lane >> 4;
    const int kvh = blockIdx.y;
    const int row = rows[blockIdx.z];
    const int pos = positions[row];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int first_split = lo / BIG, last_split = pos / BIG;
    const int split = first_split + blockIdx.x;
    if (split > last_split) return;
    const int n_splits = last_split - first_split + 1;
    const int base = split * BIG;
    const int n_sub = (min(BIG, pos + 1 - base) + SUB - 1) / SUB;      // blocks that hold a key up to the query's own
    const int32_t* table = block_table + (size_t)seq_of_token[row] * max_blocks;
    const int page_shift = __builtin_ctz(page);

    for (int i = tid; i < n_sub * SUB; i += THREADS) s_page[i] = table[min(base + i, pos) >> page_shift];
    if (tid < GROUP) {
        s_m[tid] = -INFINITY;
        s_l[tid] = 0.0f;
    }
    Frag qf[KSTEPS];
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t) {
        const int dcol = min(32 * t + 8 * h, HEAD_DIM - 8);
        qf[t].u = *(const u32x4*)(q + ((size_t)row * n_q + (size_t)kvh * GROUP + min(l16, GROUP - 1)) * HEAD_DIM + dcol);
    }
    __syncthreads();

    Frag kf[2][SUB_BLOCKS_PER_WAVE][KSTEPS], vf[2][SUB_KEYS_PER_GROUP][CHUNKS_PER_LANE];
    const int kg = wave * 4 + h;                      // this lane group's keys of a sub-block: kg + 16 i
    auto fetch = [&](auto set, int sub) {
        constexpr int S = decltype(set)::value;
        const int first = sub * SUB;
#pragma unroll
        for (int b = 0; b < SUB_BLOCKS_PER_WAVE; ++b) {
            const int kl = first + (wave * SUB_BLOCKS_PER_WAVE + b) * 16 + l16;
            const int sk = min(base + kl, pos);
            const bf16_t* k_row = k_cache + (((size_t)s_page[kl] * n_kv + kvh) * page + (sk & (page - 1))) * HEAD_DIM;
#pragma unroll
            for (int t = 0; t < KSTEPS; ++t) kf[S][b][t].u = *(const u32x4*)(k_row + min(32 * t + 8 * h, HEAD_DIM - 8));
        }
#pragma unroll
        for (int i = 0; i < SUB_KEYS_PER_GROUP; ++i) {
            const int kl = first + kg + 16 * i;
            const int sk = min(base + kl, pos);
            const bf16_t* v_row = v_cache + (((size_t)s_page[kl] * n_kv + kvh) * page + (sk & (page - 1))) * HEAD_DIM;
#pragma unroll
            for (int c = 0; c < CHUNKS_PER_LANE; ++c) vf[S][i][c].u = *(const u32x4*)(v_row + min(l16 + 16 * c, CHUNKS - 1) * 8);
        }
    };

    float acc[GROUP][CHUNKS_PER_LANE][8];
#pragma unroll
    for (int g = 0; g < GROUP; ++g)
#pragma unroll
        for (int c = 0; c < CHUNKS_PER_LANE; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[g][c][j] = 0.0f;
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t)
        if (32 * t + 8 * h >= HEAD_DIM || l16 >= GROUP) qf[t].u = (u32x4){0u, 0u, 0u, 0u};

    auto work = [&](auto set, int sub) {
        constexpr int S = decltype(set)::value;
        const int first = base + sub * SUB;
        // ---- scores of this sub-block
#pragma unroll
        for (int b = 0; b < SUB_BLOCKS_PER_WAVE; ++b) {
            f32x4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int t = 0; t < KSTEPS; ++t) sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[S][b][t].v, qf[t].v, sc, 0, 0, 0);
            if (l16 < GROUP) {
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int kl = (wave * SUB_BLOCKS_PER_WAVE + b) * 16 + 4 * h + v;
                    const int sk = first + kl;
                    s_scores[l16][kl] = (sk >= lo && sk <= pos) ? sc[v] * scale_log2e : -INFINITY;
                }
            }
        }
        __syncthreads();
        // ---- running maximum and sum, one head per wave at a time
        for (int g = wave; g < GROUP; g += WAVES) {
            float sc[SUB / KIPP_WAVE];
            float m = -INFINITY;
#pragma unroll
            for (int i = 0; i < SUB / KIPP_WAVE; ++i) {
                sc[i] = s_scores[g][lane + KIPP_WAVE * i];
                m = fmaxf(m, sc[i]);
            }
            m = wave_max(m);
            const float m_old = s_m[g];
            const float m_new = fmaxf(m_old, m);
            const float m_use = m_new == -INFINITY ? 0.0f : m_new;     // nothing visible yet: every weight is 0
            float l = 0.0f;
#pragma unroll
            for (int i = 0; i < SUB / KIPP_WAVE; ++i) {
                const float pw = exp2f(sc[i] - m_use);
                s_scores[g][lane + KIPP_WAVE * i] = pw;
                l += pw;
            }
            l = wave_sum(l);
            if (lane == 0) {
                const float alpha = exp2f(m_old - m_use);                // m_old = -inf gives 0
                s_alpha[g] = alpha;
                s_l[g] = s_l[g] * alpha + l;
                s_m[g] = m_new;
            }
        }
        __syncthreads();
        // ---- values: what was gathered so far is brought to the new maximum, then this sub-block is added
        float alpha[GROUP];
#pragma unroll
        for (int g = 0; g < GROUP; ++g) alpha[g] = s_alpha[g];
#pragma unroll
        for (int g = 0; g < GROUP; ++g)
#pragma unroll
            for (int c = 0; c < CHUNKS_PER_LANE; ++c)
#pragma unroll
                for (int j = 0; j < 8; ++j) acc[g][c][j] *= alpha[g];
#pragma unroll
        for (int i = 0; i < SUB_KEYS_PER_GROUP; ++i) {
            const int kl = kg + 16 * i;
            float pw[GROUP];
#pragma unroll
            for (int g = 0; g < GROUP; ++g) pw[g] = s_scores[g][kl];
#pragma unroll
            for (int c = 0; c < CHUNKS_PER_LANE; ++c) {
                float vv[8];
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    vv[j] = __uint_as_float((j & 1) ? (vf[S][i][c].u[j >> 1] & 0xffff0000u) : (vf[S][i][c].u[j >> 1] << 16));
#pragma unroll
                for (int g = 0; g < GROUP; ++g)
#pragma unroll
                    for (int j = 0; j < 8; ++j) acc[g][c][j] = fmaf(pw[g], vv[j], acc[g][c][j]);
            }
        }
        __syncthreads();                              // the scores are overwritten by the next sub-block
    };

    using Set0 = std::integral_constant<int, 0>;
    using Set1 = std::integral_constant<int, 1>;
    fetch(Set0{}, 0);
    for (int sub = 0; sub < n_sub; sub += 2) {
        if (sub + 1 < n_sub) fetch(Set1{}, sub + 1);
        work(Set0{}, sub);
        if (sub + 1 < n_sub) {
            if (sub + 2 < n_sub) fetch(Set0{}, sub + 2);
            work(Set1{}, sub + 1);
        }
    }

    // sum the four lane groups of the wave, then the waves
#pragma unroll
    for (int g = 0; g < GROUP; ++g)
#pragma unroll
        for (int c = 0; c < CHUNKS_PER_LANE; ++c)
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float a = acc[g][c][j];
                a += __shfl_xor(a, 16, KIPP_WAVE);
                a += __shfl_xor(a, 32, KIPP_WAVE);
                acc[g][c][j] = a;
            }
    if (h == 0) {
#pragma unroll
        for (int g = 0; g < GROUP; ++g)
#pragma unroll
            for (int c = 0; c < CHUNKS_PER_LANE; ++c) {
                const int chunk = l16 + 16 * c;
                if (chunk < CHUNKS) {
#pragma unroll
                    for (int j = 0; j < 8; ++j) s_red[wave][g][chunk * 8 + j] = acc[g][c][j];
                }
            }
    }
    __syncthreads();
    for (int idx = tid; idx < GROUP * HEAD_DIM; idx += THREADS) {
        const int g = idx / HEAD_DIM, dcol = idx % HEAD_DIM;
        float a = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) a += s_red[w][g][dcol];
        const int head = kvh * GROUP + g;
        if (n_splits == 1) {
            out[((size_t)row * n_q + head) * HEAD_DIM + dcol] = f32_to_bf16(a / s_l[g]);
        } else {
            put_partial(arrivals, part_acc, part_ml, ((size_t)blockIdx.z * n_q + head) * max_splits + blockIdx.x, dcol, a, s_m[g], s_l[g]);
        }
    }
    if (arrivals != nullptr && n_splits > 1)
        merge_by_the_last(arrivals, part_acc, part_ml, out, blockIdx.z, row, kvh, n_q, n_kv, max_splits, n_splits);
}

// ---------------------------------------------------------------------------------------------
// The same attention with keys and values streamed through LDS by the memory pipeline itself
// (global_load_lds_dwordx4: 16 bytes a lane straight into LDS, no register in between), for
// head size 128 and pages that are multiples of 16 keys.
//
// Every wave is a stream of its own: it takes every fourth block of 16 keys of the workgroup's
// range, keeps a ring of RING_STAGES blocks (keys and values, 8 KB a block) in its own part of
// LDS and, while it works on one block, the next is on its way; no barrier until the waves merge
// at the end.  The loads therefore never stop while a wave has keys left, where the kernels above
// load everything, then compute everything (and all workgroups of a launch do so in step).
//
//   scores   S^T[key][head] = K . Q^T, v_mfma_f32_16x16x32_bf16, A = the block's keys from LDS;
//   softmax  online, per wave: a lane holds 4 keys of one head, the lanes of the other key
//            quarters are two exchanges away; running maximum and sum per head in registers;
//   values   O^T[d][head] += V^T . P^T, v_mfma_f32_16x16x16_bf16: P^T is the score registers as
//            they are (rounded to bfloat16), V^T comes out of LDS transposed by
//            ds_read_b64_tr_b16 (values lie in LDS as in the cache, [key][d]).
//
// The launcher takes this kernel from 96 (sequence, key/value head) pairs on (measured in the decode step at
// 2,100 keys: from there it is at least as fast as splitting the keys, merge kernel included, with pages
// scattered over the pool; at 80 pairs it is a tenth slower):
// a workgroup then walks a sequence's whole context (up to RING_RANGE keys), the partial results
// and the merge kernel fall away, and in the FUSED form every query is normed and rotated once (by
// the one workgroup of its key/value head) while the first blocks are on their way; that workgroup
// also writes the token's key and value into the cache and puts them into the block it has in LDS.
// With fewer pairs it is taken for long contexts, in ranges that still give 256 workgroups (1,024 keys
// at least: measured a tenth faster than the kernel above at 8 sequences of 9,000 and of 30,000 keys).
//
// LDS layout of a block: key row r at 256 r, its 16-byte chunk c at slot c ^ r (keys) or
// c ^ 2 (r % 8) (values): the 16 rows a matrix-core operand reads at once then fall into
// different banks.  The lane that brings slot p of row r simply asks for chunk p ^ r of that row.
#define RING_OK (HEAD_DIM == 128)
#define RING_STAGES 2
#define RING_HALF (16 * HEAD_DIM * 2)                          // bytes of a block's keys (or values)
#define RING_BYTES (WAVES * RING_STAGES * 2 * RING_HALF)
#define RING_RANGE (KIPP_WAVE * WAVES * 16)                    // keys of a workgroup at most: a wave holds its blocks' pages one a lane
#ifndef RING_FROM_PAIRS
#define RING_FROM_PAIRS 96                                    // sequences x key/value heads from which this kernel is taken
#endif

typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

#if RING_OK
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
    union {
        bf16x2 v;
        uint32_t u;
    } r;
    r.v = __builtin_convertvector((f32x2){a, b}, bf16x2);
    return r.u;
}

#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

template <bool FUSED>
__global__ void __launch_bounds__(THREADS, 2) attention_decode_ring_kernel(
    const bf16_t* __restrict__ q, bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const int32_t* __restrict__ rows, const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_of_token,
    const int32_t* __restrict__ block_table, int max_blocks, int n_q, int n_kv, int page, float scale_log2e,
    int window, int max_splits, int range, Projected pj, unsigned* arrivals) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char ring[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, h = lane >> 4;
    const int kvh = blockIdx.y;
    const int row = rows[blockIdx.x];                 // the grid is (query tokens, key/value heads, ranges): ranges beyond a sequence's position come last
    const int pos = positions[row];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int first_split = lo / range, last_split = pos / range;
    const int split = first_split + blockIdx.z;
    if (split > last_split) return;
    const int n_splits = last_split - first_split + 1;
    const int base = split * range;
    const int32_t* table = block_table + (size_t)seq_of_token[row] * max_blocks;
    const int page_shift = __builtin_ctz(page);

    // blocks of 16 keys (absolute index) that hold a visible key of this range; the wave's are every fourth
    const int kb_lo = max(lo, base) >> 4, kb_hi = min(pos, base + range - 1) >> 4;
    const int kb_first = kb_lo + wave;
    const int n_mine = kb_first <= kb_hi ? (kb_hi - kb_first) / WAVES + 1 : 0;
    // the page of the wave's j-th block in lane j (a block lies within one page)
    int my_pages = 0;
    if (lane < n_mine) my_pages = table[((kb_first + WAVES * lane) << 4) >> page_shift];

    unsigned char* my_ring = ring + wave * (RING_STAGES * 2 * RING_HALF);
    auto issue = [&](int j, int stage) {
        const int kb = kb_first + WAVES * j;
        const int pg = __builtin_amdgcn_readlane(my_pages, j);
        const size_t off = (((size_t)pg * n_kv + kvh) * page + ((kb << 4) & (page - 1))) * HEAD_DIM;
        const int last = pos - (kb << 4);            // keys beyond the query's own read its row again (masked below)
        unsigned char* dst = my_ring + stage * (2 * RING_HALF);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 4 * i + h;
            const bf16_t* src = k_cache + off + (size_t)min(r, last) * HEAD_DIM + ((l16 ^ r) << 3);
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(src), LDS_PTR(dst + 1024 * i), 16, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 4 * i + h;
            const bf16_t* src = v_cache + off + (size_t)min(r, last) * HEAD_DIM + ((l16 ^ (2 * (r & 7))) << 3);
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(src), LDS_PTR(dst + RING_HALF + 1024 * i), 16, 0, 0);
        }
    };
    if (n_mine > 0) issue(0, 0);
    if (n_mine > 1) issue(1, 1);

    // ---- the GROUP queries as B operand: lane (slot l16, quarter h) holds q[slot][32 t + 8 h .. + 7]
    Frag qf[KSTEPS];
    bf16_t (*s_new)[HEAD_DIM] = (bf16_t(*)[HEAD_DIM])(ring + RING_BYTES);   // FUSED: the GROUP queries, the new key, the new value
    const bool owner = FUSED && pj.write_kv && split == last_split;        // this workgroup holds the token's own position
    if (FUSED) {
        // norm (/root/reference/src/kipp.c:2480-2500) and rotation (kipp.c:2368-2382) of the heads this wave
        // prepares, in the arithmetic of the rotary kernel: a wave a head, element i and its rotation
        // partner i + d/2 in one lane; the slabs of the projection are added in order
        const size_t width = (size_t)(n_q + 2 * n_kv) * HEAD_DIM;
        int last_slab = pj.parts - 1;
        asm volatile("" : "+s"(last_slab));          // opaque: every slab load below is issued, none waits for a branch
        float cs[NC / 2], sn[NC / 2];
#pragma unroll
        for (int c = 0; c < NC / 2; ++c) {
            cs[c] = 1.0f;
            sn[c] = 0.0f;
            if (pj.angles != nullptr) {
                cs[c] = pj.angles[(size_t)row * HEAD_DIM + lane + c * KIPP_WAVE];
                sn[c] = pj.angles[(size_t)row * HEAD_DIM + HEAD_DIM / 2 + lane + c * KIPP_WAVE];
            } else if (pj.inv_freq != nullptr) {
                const float angle = (float)pos * pj.inv_freq[lane + c * KIPP_WAVE];
                cs[c] = cosf(angle);
                sn[c] = sinf(angle);
            }
        }
#pragma unroll
        for (int jj = 0; jj < JOBS; ++jj) {
            const int j = wave + jj * WAVES;
            if (!(j < GROUP || (owner && j < GROUP + 2))) continue;
            const int slot = j < GROUP ? kvh * GROUP + j : (j == GROUP ? n_q + kvh : n_q + n_kv + kvh);
            const float* src = pj.qkv + (size_t)row * width + (size_t)slot * HEAD_DIM + lane;
            float slab[NC][MAX_SLABS], raw[NC];
#pragma unroll
            for (int c = 0; c < NC; ++c)
#pragma unroll
                for (int p = 0; p < MAX_SLABS; ++p)
                    slab[c][p] = src[(size_t)min(p, last_slab) * pj.part_stride + c * KIPP_WAVE];
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                raw[c] = slab[c][0];
#pragma unroll
                for (int p = 1; p < MAX_SLABS; ++p) raw[c] += (p <= last_slab ? 1.0f : 0.0f) * slab[c][p];
            }
            if (j <= GROUP) {
                const float* norm_w = j < GROUP ? pj.q_norm_w : pj.k_norm_w;
                if (norm_w != nullptr) {
                    float ss = 0.0f;
#pragma unroll
                    for (int c = 0; c < NC; ++c) ss = square_add(ss, raw[c]);
                    ss = wave_sum(ss);
                    const float r = head_norm_scale(ss, (float)HEAD_DIM, pj.eps);
#pragma unroll
                    for (int c = 0; c < NC; ++c) raw[c] *= r * norm_w[lane + c * KIPP_WAVE];
                }
#pragma unroll
                for (int c = 0; c < NC / 2; ++c) {
                    const float a = raw[c], b = raw[c + NC / 2];
                    raw[c] = rotate_lo(a, b, cs[c], sn[c]);
                    raw[c + NC / 2] = rotate_hi(a, b, cs[c], sn[c]);
                }
            }
            bf16_t* dst = nullptr;
            if (j >= GROUP)
                dst = (j == GROUP ? k_cache : v_cache) +
                      (((size_t)table[pos >> page_shift] * n_kv + kvh) * page + (pos & (page - 1))) * HEAD_DIM;
#pragma unroll
            for (int c = 0; c < NC; ++c) {
                const bf16_t bits = f32_to_bf16(raw[c]);
                s_new[j][lane + c * KIPP_WAVE] = bits;
                if (dst != nullptr) dst[lane + c * KIPP_WAVE] = bits;
            }
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < KSTEPS; ++t) qf[t].u = *(const u32x4*)(&s_new[min(l16, GROUP - 1)][32 * t + 8 * h]);
    } else {
#pragma unroll
        for (int t = 0; t < KSTEPS; ++t)
            qf[t].u = *(const u32x4*)(q + ((size_t)row * n_q + (size_t)kvh * GROUP + min(l16, GROUP - 1)) * HEAD_DIM + 32 * t + 8 * h);
    }
#pragma unroll
    for (int t = 0; t < KSTEPS; ++t)
        if (l16 >= GROUP) qf[t].u = (u32x4){0u, 0u, 0u, 0u};

    f32x4 o[HEAD_DIM / 16];
#pragma unroll
    for (int b = 0; b < HEAD_DIM / 16; ++b) o[b] = (f32x4){0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY, l_run = 0.0f;
    // a lane's place in the operands: key row l16 of the keys; for the transposed read of the values, the
    // 8 bytes at row 4 h + l16 / 4, columns 4 (l16 % 4) .. + 3 of a 16-column block
    const int v_row = 4 * h + (l16 >> 2);
    uint32_t v_addr[HEAD_DIM / 16];                  // LDS addresses of those 8 bytes in stage 0, one per block of columns
#pragma unroll
    for (int b = 0; b < HEAD_DIM / 16; ++b)
        v_addr[b] = (uint32_t)(uintptr_t)LDS_PTR(my_ring + RING_HALF) + v_row * 256 + 8 * (l16 & 3) + 32 * (b ^ (v_row & 7));

    for (int j = 0; j < n_mine; ++j) {
        const int stage = j & 1;
        // the block's 8 loads have landed when at most the next block's 8 are still out
        if (j + 1 < n_mine) __builtin_amdgcn_s_waitcnt(0x0F78);      // vmcnt(8)
        else __builtin_amdgcn_s_waitcnt(0x0F70);                     // vmcnt(0)
        unsigned char* kbuf = my_ring + stage * (2 * RING_HALF);
        const int kb = kb_first + WAVES * j;
        if (owner && kb == (pos >> 4)) {
            // the token's own key and value (the cache row may or may not have them yet): from s_new into the block
            const int r = pos & 15;
            if (lane < 16) {
                *(u32x4*)(kbuf + r * 256 + ((lane ^ r) << 4)) = *(const u32x4*)(&s_new[GROUP][8 * lane]);
                *(u32x4*)(kbuf + RING_HALF + r * 256 + ((lane ^ (2 * (r & 7))) << 4)) = *(const u32x4*)(&s_new[GROUP + 1][8 * lane]);
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // written before the transposed reads below are asked for
        }
        f32x4 sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int t = 0; t < KSTEPS; ++t) {
            Frag kf;
            kf.u = *(const u32x4*)(kbuf + l16 * 256 + (((4 * t + h) ^ l16) << 4));
            sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[t].v, sc, 0, 0, 0);
        }
        // The values, transposed, are asked for now and arrive during the softmax.  The instruction is
        // written out: the compiler would make a read through the intrinsic wait for every load into
        // LDS that is still on its way, the next block's included.
        s16x4 vt[HEAD_DIM / 16];
#pragma unroll
        for (int b = 0; b < HEAD_DIM / 16; ++b)
            asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(vt[b]) : "v"(v_addr[b] + stage * (2 * RING_HALF)));
        // sc[v] = S^T[key 4 h + v][head l16]
        float m_blk = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int s = (kb << 4) + 4 * h + v;
            sc[v] = (s >= lo && s <= pos) ? __fmul_rn(sc[v], scale_log2e) : -INFINITY;   // every rounding spelt out: both forms of the kernel give the same bits
            m_blk = fmaxf(m_blk, sc[v]);
        }
        m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 16, KIPP_WAVE));
        m_blk = fmaxf(m_blk, __shfl_xor(m_blk, 32, KIPP_WAVE));
        const float m_new = fmaxf(m_run, m_blk);
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;       // nothing visible yet: every weight is 0
        const float alpha = exp2f(__fsub_rn(m_run, m_use));          // m_run = -inf gives 0
        float l_blk = 0.0f;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            sc[v] = exp2f(__fsub_rn(sc[v], m_use));                  // -inf gives 0
            l_blk = __fadd_rn(l_blk, sc[v]);
        }
        l_blk += __shfl_xor(l_blk, 16, KIPP_WAVE);
        l_blk += __shfl_xor(l_blk, 32, KIPP_WAVE);
        l_run = fmaf(l_run, alpha, l_blk);
        m_run = m_new;
        union {
            u32x2 u;
            s16x4 v;
        } pb;
        pb.u = (u32x2){pack_bf16(sc[0], sc[1]), pack_bf16(sc[2], sc[3])};
        static_assert(HEAD_DIM / 16 == 8, "the wait below names the eight transposed reads");
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(vt[0]), "+v"(vt[1]), "+v"(vt[2]), "+v"(vt[3]), "+v"(vt[4]), "+v"(vt[5]), "+v"(vt[6]), "+v"(vt[7]));
        // every read of the stage has come back: the block after next is asked for
        if (j + 2 < n_mine) issue(j + 2, stage);
#pragma unroll
        for (int b = 0; b < HEAD_DIM / 16; ++b) {
#pragma unroll
            for (int v = 0; v < 4; ++v) o[b][v] = __fmul_rn(o[b][v], alpha);
            o[b] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vt[b], pb.v, o[b], 0, 0, 0);
        }
    }

    // ---- merge the waves: o[b][v] = O[head l16][16 b + 4 h + v]
    __syncthreads();                                                 // every ring has been read for the last time
    float* s_red = (float*)ring;                                     // [WAVES][GROUP][HEAD_DIM]
    float* s_ml = s_red + WAVES * GROUP * HEAD_DIM;                  // [WAVES][GROUP][2]
    if (l16 < GROUP) {
#pragma unroll
        for (int b = 0; b < HEAD_DIM / 16; ++b)
            *(f32x4*)(s_red + ((size_t)wave * GROUP + l16) * HEAD_DIM + 16 * b + 4 * h) = o[b];
        if (h == 0) {
            s_ml[(wave * GROUP + l16) * 2] = m_run;
            s_ml[(wave * GROUP + l16) * 2 + 1] = l_run;
        }
    }
    __syncthreads();
    for (int idx = tid; idx < GROUP * HEAD_DIM / 2; idx += THREADS) {      // two neighbouring columns a thread
        const int g = idx / (HEAD_DIM / 2), dcol = 2 * (idx % (HEAD_DIM / 2));
        float m = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) m = fmaxf(m, s_ml[(w * GROUP + g) * 2]);
        float a0 = 0.0f, a1 = 0.0f, l = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float f = exp2f(__fsub_rn(s_ml[(w * GROUP + g) * 2], m));    // a wave without keys: 2^-inf = 0
            a0 = fmaf(s_red[((size_t)w * GROUP + g) * HEAD_DIM + dcol], f, a0);
            a1 = fmaf(s_red[((size_t)w * GROUP + g) * HEAD_DIM + dcol + 1], f, a1);
            l = fmaf(s_ml[(w * GROUP + g) * 2 + 1], f, l);
        }
        const int head = kvh * GROUP + g;
        if (n_splits == 1) {
            *(uint32_t*)(out + out_at(row, head * HEAD_DIM + dcol, n_q * HEAD_DIM, FUSED ? pj.out_rows : 0)) =
                (uint32_t)f32_to_bf16(a0 / l) | ((uint32_t)f32_to_bf16(a1 / l) << 16);
        } else {
            put_partial2(arrivals, part_acc, part_ml, ((size_t)blockIdx.x * n_q + head) * max_splits + blockIdx.z, dcol, a0, a1, m, l);
        }
    }
    if (arrivals != nullptr && n_splits > 1)
        merge_by_the_last(arrivals, part_acc, part_ml, out, blockIdx.x, row, kvh, n_q, n_kv, max_splits, n_splits, FUSED ? pj.out_rows : 0);
}
#endif  // RING_OK

// Merge the splits of every (token, head) in index order:
// m* = max m_s, out = sum_s acc_s 2^(m_s - m*) / sum_s l_s 2^(m_s - m*)
// (/root/reference/metal/kipp_kernels.metal:741-779).
__global__ void attention_decode_reduce_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml, bf16_t* __restrict__ out,
    const int32_t* __restrict__ rows, const int32_t* __restrict__ positions, int n_q, int window, int max_splits,
    int split_keys, int out_rows) {
    const int head = blockIdx.x, item = blockIdx.y;
    const int row = rows[item];
    const int pos = positions[row];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int n_splits = pos / split_keys - lo / split_keys + 1;
    if (n_splits == 1) return;
    const size_t slot0 = ((size_t)item * n_q + head) * max_splits;
    // the (m, l) pairs of all splits, one a lane, so that they arrive together
    const int lane = threadIdx.x & 63;
    float m = -INFINITY;
    for (int s0 = 0; s0 < n_splits; s0 += KIPP_WAVE)
        if (s0 + lane < n_splits) m = fmaxf(m, part_ml[(slot0 + s0 + lane) * 2]);
    m = wave_max(m);
    float denom = 0.0f;
    for (int s = 0; s < n_splits; ++s) denom += part_ml[(slot0 + s) * 2 + 1] * exp2f(part_ml[(slot0 + s) * 2] - m);
    for (int dcol = threadIdx.x; dcol < HEAD_DIM; dcol += blockDim.x) {
        float a = 0.0f;
        int s = 0;
        for (; s + 4 <= n_splits; s += 4) {       // four loads in flight; added in split order
            const float a0 = part_acc[(slot0 + s) * HEAD_DIM + dcol], a1 = part_acc[(slot0 + s + 1) * HEAD_DIM + dcol];
            const float a2 = part_acc[(slot0 + s + 2) * HEAD_DIM + dcol], a3 = part_acc[(slot0 + s + 3) * HEAD_DIM + dcol];
            a += a0 * exp2f(part_ml[(slot0 + s) * 2] - m);
            a += a1 * exp2f(part_ml[(slot0 + s + 1) * 2] - m);
            a += a2 * exp2f(part_ml[(slot0 + s + 2) * 2] - m);
            a += a3 * exp2f(part_ml[(slot0 + s + 3) * 2] - m);
        }
        for (; s < n_splits; ++s) a += part_acc[(slot0 + s) * HEAD_DIM + dcol] * exp2f(part_ml[(slot0 + s) * 2] - m);
        out[out_at(row, head * HEAD_DIM + dcol, n_q * HEAD_DIM, out_rows)] = f32_to_bf16(a / denom);
    }
}


// The same merge for launches of up to MAXS splits: the (m, l) pairs and the partial sums of every split the
// launch has are asked for at once, before the token's position says how many of them count, so the kernel is
// two round trips to memory long instead of four.  The same sums in the same order as above.
template <int MAXS>
__global__ void __launch_bounds__(KIPP_WAVE) attention_decode_reduce_few_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml, bf16_t* __restrict__ out,
    const int32_t* __restrict__ rows, const int32_t* __restrict__ positions, int n_q, int window, int max_splits,
    int split_keys, int grid_splits, int out_rows) {
    constexpr int COLS = (HEAD_DIM + KIPP_WAVE - 1) / KIPP_WAVE;     // columns of a head a lane merges
    const int head = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
    const size_t slot0 = ((size_t)item * n_q + head) * max_splits;
    float m_s[MAXS], l_s[MAXS], a_s[MAXS][COLS];
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
        const size_t slot = slot0 + min(s, grid_splits - 1);         // beyond the launch's splits: the last again, dropped below
        m_s[s] = part_ml[slot * 2];
        l_s[s] = part_ml[slot * 2 + 1];
#pragma unroll
        for (int c = 0; c < COLS; ++c) a_s[s][c] = part_acc[slot * HEAD_DIM + min(lane + KIPP_WAVE * c, HEAD_DIM - 1)];
    }
    const int row = rows[item];
    const int pos = positions[row];
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int n_splits = pos / split_keys - lo / split_keys + 1;
    if (n_splits == 1) return;                                        // written by the attention kernel itself
    // slots of splits that did not run hold whatever was there before: they are chosen away, never multiplied
    float m = -INFINITY;
#pragma unroll
    for (int s = 0; s < MAXS; ++s) m = fmaxf(m, s < n_splits ? m_s[s] : -INFINITY);
    float denom = 0.0f, a[COLS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) a[c] = 0.0f;
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
        if (s < n_splits) {
            const float w = exp2f(m_s[s] - m);
            denom += l_s[s] * w;
#pragma unroll
            for (int c = 0; c < COLS; ++c) a[c] += a_s[s][c] * w;
        }
    }
#pragma unroll
    for (int c = 0; c < COLS; ++c) {
        const int dcol = lane + KIPP_WAVE * c;
        if (dcol < HEAD_DIM) out[out_at(row, head * HEAD_DIM + dcol, n_q * HEAD_DIM, out_rows)] = f32_to_bf16(a[c] / denom);
    }
}

// The merge of a launch's splits (`grid_splits` of `split_keys` keys each at most).
static int launch_reduce(const float* part_acc, const float* part_ml, bf16_t* out, const int32_t* rows,
                         const int32_t* positions, int n_items, int n_q, int window, int max_splits, int split_keys,
                         int grid_splits, hipStream_t stream, int out_rows = 0) {
    const dim3 grid(n_q, n_items);
    if (grid_splits <= 8)
        hipLaunchKernelGGL(attention_decode_reduce_few_kernel<8>, grid, dim3(KIPP_WAVE), 0, stream, part_acc, part_ml, out,
                           rows, positions, n_q, window, max_splits, split_keys, grid_splits, out_rows);
    else if (grid_splits <= 16)
        hipLaunchKernelGGL(attention_decode_reduce_few_kernel<16>, grid, dim3(KIPP_WAVE), 0, stream, part_acc, part_ml, out,
                           rows, positions, n_q, window, max_splits, split_keys, grid_splits, out_rows);
    else
        hipLaunchKernelGGL(attention_decode_reduce_kernel, grid, dim3(HEAD_DIM >= 64 ? 64 : HEAD_DIM), 0, stream, part_acc,
                           part_ml, out, rows, positions, n_q, window, max_splits, split_keys, out_rows);
    return KIPP_LAUNCH_CHECK();
}


#if RING_OK
// Keys a workgroup of the kernel that streams through LDS walks in a launch of this shape; 0: the launch
// is not for it.  RING_WHOLE_FROM_PAIRS (sequence, key/value head) pairs and more: whole contexts (RING_RANGE
// keys at most).  Fewer: ranges that give 256 workgroups, if those are 1,024 keys and more; else whole contexts
// from RING_FROM_PAIRS pairs on.  Measured in the decode step at 2,100 keys, 8 heads: 12 sequences in two ranges
// (192 workgroups at work instead of 96) 3.24 instead of 3.54 ms; 16 sequences 3.31 instead of 3.39 (they were
// level while the merge asked for its partial results four bytes at a time); 24 sequences in two ranges 4.11
// instead of 3.97 (the partial results and their merge cost more than the second workgroup on every compute
// unit brings).  A function of the launch's shape, never of the data.
#define RING_WHOLE_FROM_PAIRS 160
static int ring_range(int n_items, int n_kv, int page, int grid_splits) {
    if (page % 16 != 0) return 0;
    const long long pairs = (long long)n_items * n_kv, span = (long long)grid_splits * SPLIT;
    const long long whole = span < RING_RANGE ? span : RING_RANGE;
    if (pairs >= RING_WHOLE_FROM_PAIRS) return (int)whole;
    const long long range = span * pairs / 256 / SPLIT * SPLIT;
    if (range < 1024) return pairs >= RING_FROM_PAIRS ? (int)whole : 0;
    return (int)(range < RING_RANGE ? range : RING_RANGE);
}

// That kernel, if it takes this launch (0 if not).
template <bool FUSED>
static int launch_ring(const bf16_t* q, bf16_t* k_cache, bf16_t* v_cache, bf16_t* out, float* part_acc, float* part_ml,
                       const int32_t* rows, const int32_t* positions, const int32_t* seq_of_token,
                       const int32_t* block_table, int max_blocks, int n_items, int n_q, int n_kv, int page,
                       float scale_log2e, int window, int grid_splits, int max_splits, Projected pj, unsigned* arrivals,
                       hipStream_t stream, int* rc) {
    const int range = ring_range(n_items, n_kv, page, grid_splits);
    if (range == 0) return 0;
    const int lds = RING_BYTES + (FUSED ? (GROUP + 2) * HEAD_DIM * 2 : 0);
    static bool prepared = false;
    if (!prepared) {
        if (hipFuncSetAttribute((const void*)attention_decode_ring_kernel<FUSED>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                lds) != hipSuccess) {
            *rc = -6;
            return 1;
        }
        prepared = true;
    }
    const int span = grid_splits * SPLIT;
    const int ring_splits = (span + range - 1) / range + (window > 0 ? 1 : 0);   // a window may straddle one more edge
    if (ring_splits > max_splits) return 0;
    hipLaunchKernelGGL(attention_decode_ring_kernel<FUSED>, dim3(n_items, n_kv, ring_splits), dim3(THREADS), lds, stream, q,
                       k_cache, v_cache, out, part_acc, part_ml, rows, positions, seq_of_token, block_table, max_blocks, n_q,
                       n_kv, page, scale_log2e, window, max_splits, range, pj, arrivals);
    *rc = KIPP_LAUNCH_CHECK();
    if (*rc != 0 || ring_splits == 1 || arrivals != nullptr) return 1;
    *rc = launch_reduce(part_acc, part_ml, (bf16_t*)out, rows, positions, n_items, n_q, window, max_splits, range, ring_splits, stream,
                        FUSED ? pj.out_rows : 0);
    return 1;
}
#endif

// The kernel that takes one split a workgroup, with splits of 192, 256 or 320 keys (head sizes above 128: 256): the
// length whose workgroups take the fewest keys one after the other on a compute unit.  The workgroups of a launch run in
// rounds of 256, and a round costs what one split reads, so a length is priced as rounds x keys, with the rounds of the
// splits that contexts really have: a recorded step is launched for the longest context of its class of 1,024, and the
// splits beyond a sequence's position leave at once, so the price is the mean over the contexts of that class.
// Measured in the decode step behind 2,048 to 2,304 keys (a class up to 3,072), 32 query over 8 key/value heads, for
// 192 / 256 / 320 keys: 4 sequences 2.353 / 2.416 / 2.340 ms, 5: 2.394 / 2.454 / 2.531, 6: 2.550 / 2.493 / 2.575,
// 8: 2.620 / 2.741 / 2.648; every order is the price's.  (While the merge of the splits asked for its partial results
// four bytes at a time the shorter splits' merges cost more than that, and 8 sequences took 320.)  A function of the
// launch's shape, never of the data.
static int split_keys_for(int n_items, int n_kv, int span_keys, int window, int longest, int max_splits) {
    const long long pairs = (long long)n_items * n_kv;
    const int extra = window > 0 ? 1 : 0;
    static const int lengths[] = {SPLIT_MAX, SPLIT, SPLIT_MIN};          // of equal price the longest: fewer partial results
    const bool a_class = span_keys > 1024 && span_keys % 1024 == 0;      // every context of the last 1,024 keys may come
    long long best = -1;
    int keys = 0;
    for (int length : lengths) {
        if (length > longest || (span_keys + length - 1) / length + extra > max_splits) continue;
        long long price = 0;
        for (int i = a_class ? 1 : 16; i <= 16; ++i) {
            const int context = span_keys - (16 - i) * 64;
            price += (pairs * ((context + length - 1) / length + extra) + 255) / 256 * length;
        }
        if (best < 0 || price < best) {
            best = price;
            keys = length;
        }
    }
    return keys != 0 ? keys : longest;                // (no length fits the room for partial results: the launcher refuses)
}

template <bool FUSED>
static int launch_split(const bf16_t* q, bf16_t* k_cache, bf16_t* v_cache, bf16_t* out, float* part_acc, float* part_ml,
                        const int32_t* rows, const int32_t* positions, const int32_t* seq_of_token,
                        const int32_t* block_table, int max_blocks, int n_items, int n_q, int n_kv, int page,
                        float scale_log2e, int window, int grid_splits, int max_splits, Projected pj, unsigned* arrivals,
                        hipStream_t stream) {
    const int extra = window > 0 ? 1 : 0;
    const int span_keys = (grid_splits - extra) * SPLIT;           // the caller counts splits of SPLIT keys
    // one rule for both forms, so that they cut alike and give the same bits
    // (head sizes above 128 stay with 256 keys: a longer split's keys and values would not fit the registers)
    const int keys = split_keys_for(n_items, n_kv, span_keys, window, HEAD_DIM <= 128 ? SPLIT_MAX : SPLIT, max_splits);
    const int splits = keys == SPLIT ? grid_splits : (span_keys + keys - 1) / keys + extra;
#define KIPP_SPLIT_LAUNCH(KEYS)                                                                                       \
    hipLaunchKernelGGL((attention_decode_kernel<FUSED, KEYS>), dim3(n_items, n_kv, splits), dim3(THREADS), 0, stream, q, \
                       k_cache, v_cache, out, part_acc, part_ml, rows, positions, seq_of_token, block_table, max_blocks, \
                       n_q, n_kv, page, scale_log2e, window, max_splits, pj, arrivals)
    switch (keys) {
        case SPLIT_MIN: KIPP_SPLIT_LAUNCH(SPLIT_MIN); break;
        case 256: KIPP_SPLIT_LAUNCH(256); break;
        case 320: KIPP_SPLIT_LAUNCH(320); break;
        default: return -1;
    }
#undef KIPP_SPLIT_LAUNCH
    int rc = KIPP_LAUNCH_CHECK();
    if (rc != 0 || splits == 1 || arrivals != nullptr) return rc;      // with `arrivals` the last workgroup of a head has merged
    return launch_reduce(part_acc, part_ml, out, rows, positions, n_items, n_q, window, max_splits, keys, splits, stream, FUSED ? pj.out_rows : 0);
}

extern "C" {

int kipp_attention_decode_split() { return SPLIT; }
// The shortest split a launch may be cut into: what the workspace has to hold partial results for.
int kipp_attention_decode_split_min() { return SPLIT_MIN; }

// 1 if a launch of this shape goes to the kernel that streams through LDS (its fused form has no limit
// on the rows or the context).
int kipp_attention_decode_ring_takes(int n_items, int n_kv, int page, int grid_splits) {
#if RING_OK
    return ring_range(n_items, n_kv, page, grid_splits) > 0 ? 1 : 0;
#else
    return 0;
#endif
}

// `rows[i]` is the batch row of the i-th decode token.  `grid_splits` is how
// many splits the launch covers (at least those of the longest sequence);
// `part_acc` holds n_items * n_q * max_splits * HEAD_DIM floats, `part_ml`
// n_items * n_q * max_splits * 2.
int kipp_attention_decode(const void* q, const void* k_cache, const void* v_cache, void* out, float* part_acc,
                          float* part_ml, const int32_t* rows, const int32_t* positions, const int32_t* seq_of_token,
                          const int32_t* block_table, int max_blocks, int n_items, int n_q, int n_kv, int head_dim,
                          int page, float scale, int window, int grid_splits, int max_splits, int32_t* arrivals,
                          hipStream_t stream) {
    if (n_items <= 0) return 0;
    if (head_dim != HEAD_DIM || n_kv <= 0 || n_q != n_kv * GROUP) return -1;
    if (grid_splits <= 0 || grid_splits > max_splits) return -3;
    if (page <= 0 || (page & (page - 1))) return -4;   // pages of a power of two only
    const float scale_log2e = scale * 1.4426950408889634f;
#if RING_OK
    {
        int rc = 0;
        if (launch_ring<false>((const bf16_t*)q, (bf16_t*)k_cache, (bf16_t*)v_cache, (bf16_t*)out, part_acc, part_ml, rows,
                               positions, seq_of_token, block_table, max_blocks, n_items, n_q, n_kv, page, scale_log2e, window,
                               grid_splits, max_splits, Projected{}, (unsigned*)arrivals, stream, &rc))
            return rc;
    }
#endif
    // Long contexts: long ranges of keys walked by each workgroup, if that still gives every compute
    // unit two workgroups.  A function of the launch's shape, never of the data.
    const int big_splits = (grid_splits * SPLIT + BIG - 1) / BIG + (window > 0 ? 1 : 0);
    if (grid_splits * SPLIT >= STREAM_FROM && (long long)n_items * n_kv * big_splits >= 2 * 256 && big_splits <= max_splits) {
        hipLaunchKernelGGL(attention_decode_stream_kernel, dim3(big_splits, n_kv, n_items), dim3(THREADS), 0, stream,
                           (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, part_acc,
                           part_ml, rows, positions, seq_of_token, block_table, max_blocks, n_q, n_kv, page, scale_log2e,
                           window, max_splits, (unsigned*)arrivals);
        int rc = KIPP_LAUNCH_CHECK();
        if (rc != 0 || big_splits == 1 || arrivals != nullptr) return rc;
        return launch_reduce(part_acc, part_ml, (bf16_t*)out, rows, positions, n_items, n_q, window, max_splits, BIG, big_splits, stream);
    }
    return launch_split<false>((const bf16_t*)q, (bf16_t*)k_cache, (bf16_t*)v_cache, (bf16_t*)out, part_acc, part_ml, rows, positions,
                               seq_of_token, block_table, max_blocks, n_items, n_q, n_kv, page, scale_log2e, window, grid_splits,
                               max_splits, Projected{}, (unsigned*)arrivals, stream);
}

// 1 if this build has the fused kernel (head sizes that are multiples of 128).
int kipp_attention_decode_fused_ok() { return FUSED_OK ? 1 : 0; }
int kipp_attention_decode_fused_slabs() { return MAX_SLABS; }

// The same from the output of the QKV projection: `qkv` float32 [parts][tokens][(n_q + 2 n_kv) head_dim];
// norm weights, `inv_freq` and `angles` may be null (no norm; no rotation if both are null; a rotation covers
// the whole head; `angles` [tokens][head_dim] holds every token's cosines, then sines);
// with `write_kv` the token's key and value are written into the cache as well; with `out_steps_major` `out` is written
// as [n_q head_dim / 32][n_tokens][32], the order in which the few-rows product that follows reads its rows fastest.
int kipp_attention_decode_fused(const float* qkv, int parts, int n_tokens, const float* q_norm_w, const float* k_norm_w,
                                float eps, const float* inv_freq, const float* angles, int write_kv, void* k_cache,
                                void* v_cache, void* out,
                                float* part_acc, float* part_ml, const int32_t* rows, const int32_t* positions,
                                const int32_t* seq_of_token, const int32_t* block_table, int max_blocks, int n_items,
                                int n_q, int n_kv, int head_dim, int page, float scale, int window, int grid_splits,
                                int max_splits, int32_t* arrivals, int out_steps_major, hipStream_t stream) {
#if FUSED_OK
    if (n_items <= 0) return 0;
    if (head_dim != HEAD_DIM || n_kv <= 0 || n_q != n_kv * GROUP || parts <= 0 || parts > MAX_SLABS) return -1;
    if (grid_splits <= 0 || grid_splits > max_splits) return -3;
    if (page <= 0 || (page & (page - 1))) return -4;
    const float scale_log2e = scale * 1.4426950408889634f;
    Projected pj{qkv, parts, (size_t)n_tokens * (n_q + 2 * n_kv) * HEAD_DIM, q_norm_w, k_norm_w, eps, inv_freq, angles,
                 write_kv, out_steps_major ? n_tokens : 0};
#if RING_OK
    {
        int rc = 0;
        if (launch_ring<true>((const bf16_t*)nullptr, (bf16_t*)k_cache, (bf16_t*)v_cache, (bf16_t*)out, part_acc, part_ml, rows,
                              positions, seq_of_token, block_table, max_blocks, n_items, n_q, n_kv, page, scale_log2e, window,
                              grid_splits, max_splits, pj, (unsigned*)arrivals, stream, &rc))
            return rc;
    }
#endif
    return launch_split<true>((const bf16_t*)nullptr, (bf16_t*)k_cache, (bf16_t*)v_cache, (bf16_t*)out, part_acc, part_ml, rows,
                              positions, seq_of_token, block_table, max_blocks, n_items, n_q, n_kv, page, scale_log2e, window,
                              grid_splits, max_splits, pj, (unsigned*)arrivals, stream);
#else
    return -5;
#endif
}

}  // extern "C"
