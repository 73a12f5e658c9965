// Token choice on the device, one workgroup per row of float32 logits.
#include "common.h"
#include <math.h>

// Greedy: the largest logit, the lowest index among equals
// (/root/reference/src/kipp.c:3459-3464: strict '>' in index order).
__global__ void __launch_bounds__(1024) argmax_kernel(const float* __restrict__ logits, int32_t* __restrict__ out,
                                                      int vocab) {
    __shared__ float best_v[16];
    __shared__ int best_i[16];
    const float* row = logits + (size_t)blockIdx.x * vocab;
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
        const float v = row[i];
        if (v > bv || (bi == 0x7fffffff && !(v != v))) {
            bv = v;
            bi = i;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, KIPP_WAVE);
        const int oi = __shfl_xor(bi, off, KIPP_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    const int lane = threadIdx.x & (KIPP_WAVE - 1), wave = threadIdx.x / KIPP_WAVE;
    if (lane == 0) {
        best_v[wave] = bv;
        best_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        const int waves = blockDim.x / KIPP_WAVE;
        for (int w = 1; w < waves; ++w) {
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        }
        out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
    }
}

// The same in two stages for large vocabularies: ARGMAX_CHUNKS workgroups a row each find the
// best of their stretch, then one workgroup a row picks among them (again the lowest index
// among equals: stretches are in index order).
#define ARGMAX_CHUNKS 32

__global__ void __launch_bounds__(256) argmax_chunks_kernel(const float* __restrict__ logits, float* __restrict__ part_v,
                                                            int32_t* __restrict__ part_i, int vocab) {
    __shared__ float best_v[4];
    __shared__ int best_i[4];
    const float* row = logits + (size_t)blockIdx.y * vocab;
    const int per = (vocab + ARGMAX_CHUNKS - 1) / ARGMAX_CHUNKS;
    const int begin = blockIdx.x * per, end = min(vocab, begin + per);
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
        const float v = row[i];
        if (v > bv || (bi == 0x7fffffff && !(v != v))) {
            bv = v;
            bi = i;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, KIPP_WAVE);
        const int oi = __shfl_xor(bi, off, KIPP_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        best_v[threadIdx.x >> 6] = bv;
        best_i[threadIdx.x >> 6] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w)
            if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
                bv = best_v[w];
                bi = best_i[w];
            }
        part_v[blockIdx.y * ARGMAX_CHUNKS + blockIdx.x] = bv;
        part_i[blockIdx.y * ARGMAX_CHUNKS + blockIdx.x] = bi;
    }
}

__global__ void argmax_pick_kernel(const float* __restrict__ part_v, const int32_t* __restrict__ part_i,
                                   int32_t* __restrict__ out) {
    float bv = part_v[blockIdx.x * ARGMAX_CHUNKS + threadIdx.x];
    int bi = part_i[blockIdx.x * ARGMAX_CHUNKS + threadIdx.x];
#pragma unroll
    for (int off = ARGMAX_CHUNKS / 2; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, KIPP_WAVE);
        const int oi = __shfl_xor(bi, off, KIPP_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

extern "C" int kipp_argmax_scratch_floats(int rows) { return rows * ARGMAX_CHUNKS * 2; }

// `scratch`: kipp_argmax_scratch_floats(rows) 4-byte words, used when the vocabulary is large.
extern "C" int kipp_argmax(const float* logits, int32_t* out, int rows, int vocab, float* scratch, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return -1;
    if (vocab < 16384 || scratch == nullptr) {
        hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(1024), 0, stream, logits, out, vocab);
        return KIPP_LAUNCH_CHECK();
    }
    float* part_v = scratch;
    int32_t* part_i = (int32_t*)(scratch + (size_t)rows * ARGMAX_CHUNKS);
    hipLaunchKernelGGL(argmax_chunks_kernel, dim3(ARGMAX_CHUNKS, rows), dim3(256), 0, stream, logits, part_v, part_i, vocab);
    hipLaunchKernelGGL(argmax_pick_kernel, dim3(rows), dim3(ARGMAX_CHUNKS), 0, stream, part_v, part_i, out);
    return KIPP_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// The same choice for callers that cannot allocate (declared in no_alloc.h).  The partial
// results of the two-stage form live in a file-scope device array instead of a buffer the
// caller brings.  Every GPU holds its own copy of the array at its own address: in host code
// the array's name is only a stand-in, so its address on the current device is looked up
// once per device and that pointer is what the kernels get.
#include "no_alloc.h"

static __device__ __align__(256) unsigned char scratch[KIPP_ARGMAX_STATIC_MAX_ROWS * ARGMAX_CHUNKS * 2 * 4];

#define KIPP_MAX_DEVICES 64
static void* scratch_of_device[KIPP_MAX_DEVICES];   // the array's address on each device, once looked up

static int static_scratch(float** ptr) {
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return (int)err;
    if (device < 0 || device >= KIPP_MAX_DEVICES) return -3;
    void* p = __atomic_load_n(&scratch_of_device[device], __ATOMIC_ACQUIRE);
    if (p == nullptr) {
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return (int)err;
        if (p == nullptr) return -4;
        __atomic_store_n(&scratch_of_device[device], p, __ATOMIC_RELEASE);   // two first callers store the same address
    }
    *ptr = (float*)p;
    return 0;
}

extern "C" int kipp_argmax_static_max_rows(void) { return KIPP_ARGMAX_STATIC_MAX_ROWS; }

extern "C" int kipp_argmax_static(const float* logits, int32_t* out, int rows, int vocab, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0 || logits == nullptr || out == nullptr) return -1;
    if (rows > KIPP_ARGMAX_STATIC_MAX_ROWS) return -2;      // beyond what the array holds: refused, nothing launched
    float* ptr = nullptr;
    const int rc = static_scratch(&ptr);
    if (rc != 0) return rc;
    // every slot that the second kernel reads is written by the first one of the same call,
    // so nothing of an earlier call has to be cleared
    return kipp_argmax(logits, out, rows, vocab, ptr, stream);
}

// ---------------------------------------------------------------------------------------
// What a row of logits gives for its target token: -log softmax(row)[target], as the
// reference's perplexity run computes it (/root/reference/src/kipp_cli.c:759-778): the row's
// maximum in float32, the exponentials of (logit - maximum) and their sum in float64,
// maximum + log(sum) - logit[target].  One workgroup a row; the sum is added in a fixed tree
// (every lane its stride, then lanes, then waves), so a row gives the same bits every time.
#define NLL_THREADS 256
__global__ void __launch_bounds__(NLL_THREADS) row_nll_kernel(const float* __restrict__ logits, int vocab,
                                                               const int32_t* __restrict__ targets, double* __restrict__ out) {
    __shared__ float s_max[NLL_THREADS / KIPP_WAVE];
    __shared__ double s_sum[NLL_THREADS / KIPP_WAVE];
    const float* row = logits + (size_t)blockIdx.x * vocab;
    float top = -INFINITY;
    for (int i = threadIdx.x; i < vocab; i += NLL_THREADS) top = fmaxf(top, row[i]);
    top = wave_max(top);
    if ((threadIdx.x & (KIPP_WAVE - 1)) == 0) s_max[threadIdx.x / KIPP_WAVE] = top;
    __syncthreads();
    top = s_max[0];
    for (int w = 1; w < NLL_THREADS / KIPP_WAVE; ++w) top = fmaxf(top, s_max[w]);
    double sum = 0.0;
    for (int i = threadIdx.x; i < vocab; i += NLL_THREADS) sum += exp((double)row[i] - (double)top);
    for (int off = KIPP_WAVE / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, KIPP_WAVE);
    if ((threadIdx.x & (KIPP_WAVE - 1)) == 0) s_sum[threadIdx.x / KIPP_WAVE] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        double total = s_sum[0];
        for (int w = 1; w < NLL_THREADS / KIPP_WAVE; ++w) total += s_sum[w];
        out[blockIdx.x] = (double)top + log(total) - (double)row[targets[blockIdx.x]];
    }
}

// out[r] = -log softmax(logits[r, :])[targets[r]] (float64); every target inside the vocabulary.
extern "C" int kipp_row_nll(const float* logits, int rows, int vocab, const int32_t* targets, double* out, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return -1;
    hipLaunchKernelGGL(row_nll_kernel, dim3(rows), dim3(NLL_THREADS), 0, stream, logits, vocab, targets, out);
    return KIPP_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// Logit bias and the penalties over a request's recent tokens, applied to rows of logits where
// they lie, before a token is chosen from them (/root/reference/src/kipp.c:3386-3431): first every
// bias entry in its order, l[token] += bias; then, for every distinct recent token with its count,
// l = l > 0 ? l / repetition : l * repetition (unless repetition is 0 or 1), l -= presence,
// l -= frequency * count.  A row's entries are few (its biases, at most 64 recent tokens) and
// their order counts, so one lane walks them; every operation is one IEEE float operation as on
// the host (the kernel is compiled without contraction into fused multiply-adds).
// `begin` [rows + 1]: a row's entries are begin[r] .. begin[r + 1]; the first `biases[r]` of them
// are biases (`value`: the bias), the rest penalties (`value`: the token's count).  The host has
// dropped tokens outside the vocabulary and recent tokens that came before.
__global__ void adjust_logits_kernel(float* __restrict__ logits, int rows, int vocab, const int32_t* __restrict__ begin,
                                     const int32_t* __restrict__ biases, const int32_t* __restrict__ token,
                                     const float* __restrict__ value, const float* __restrict__ repetition,
                                     const float* __restrict__ presence, const float* __restrict__ frequency) {
#pragma clang fp contract(off)   // the product freq * count is rounded before it is taken off, as on the host
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    float* row = logits + (size_t)r * vocab;
    const int first = begin[r], last = begin[r + 1], first_penalty = first + biases[r];
    for (int e = first; e < first_penalty && e < last; ++e) row[token[e]] = row[token[e]] + value[e];
    const float rep = repetition[r], pres = presence[r], freq = frequency[r];
    for (int e = first_penalty; e < last; ++e) {
        float v = row[token[e]];
        if (rep != 0.0f && rep != 1.0f) v = v > 0.0f ? v / rep : v * rep;
        v = v - pres;
        const float off = freq * value[e];
        v = v - off;
        row[token[e]] = v;
    }
}

extern "C" int kipp_adjust_logits(float* logits, int rows, int vocab, const int32_t* begin, const int32_t* biases,
                                  const int32_t* token, const float* value, const float* repetition, const float* presence,
                                  const float* frequency, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return -1;
    hipLaunchKernelGGL(adjust_logits_kernel, dim3((rows + 63) / 64), dim3(64), 0, stream, logits, rows, vocab, begin, biases, token,
                       value, repetition, presence, frequency);
    return KIPP_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------
// Temperature sampling with top-k, min-p and top-p, one workgroup per row, with the
// meaning of the host sampler (/root/reference/src/kipp.c:3433-3559): scale by 1/T,
// keep candidates within 20 of the maximum, order them by descending logit (ties: lower
// id first), cut to the k first, drop what is below min_p times the top weight, keep
// the shortest prefix whose mass reaches top_p of the total, and take the first
// candidate whose cumulative mass exceeds u times the kept mass, u drawn on the host.
//
// Nothing is sorted.  A candidate's place in the order is its 64-bit key
// (monotone image of the scaled logit above the inverted index), and every question
// ("which key is the k-th", "where does the cumulative mass reach x") is answered by
// walking down the key one byte at a time with a 256-bin histogram of counts or of
// masses.  Masses are weights exp(l - max) in 44-bit fixed point, added with integer
// atomics: the sums are exact and do not depend on the order of the additions.
// A walk ends where the chosen byte has one candidate alone; the total mass is what the
// top level's histogram adds up to; and where few candidates are left (at most
// SAMPLE_LIST: after top-k, or counted) they are gathered into LDS once and the two
// mass questions are answered there, by the candidate at which the running mass
// crosses the target.

#define SAMPLE_THREADS 1024
#define SAMPLE_LIST SAMPLE_THREADS       // candidates that are finished in LDS, a lane each
#define MASS_SCALE 17592186044416.0f   // 2^44

__device__ __forceinline__ uint32_t float_order(float x) {
    uint32_t b = __float_as_uint(x);
    if (b == 0x80000000u) b = 0u;                        // -0 is 0: equal logits are ordered by their ids alone, as on the host
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);   // larger float, larger integer
}

// The float whose order is `o`, for the ends of a range of orders: orders beyond the infinities (the patterns of NaN)
// give the infinity on their side, so that a comparison with the end never turns false for a number inside the range.
__device__ __forceinline__ float float_of_order(uint32_t o) {
    if (o > 0xff800000u) return INFINITY;
    if (o < 0x007fffffu) return -INFINITY;
    return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o);
}

struct SampleRow {
    const float* row;
    int vocab;
    float inv_t, scaled_max, cutoff;
    unsigned long long key_floor;   // candidates of the top-k cut have key >= key_floor
    double min_weight;              // ... and weight >= min_weight (0: no min-p)

    // a candidate by its logit and the top-k cut alone (no exponential yet): its key and its scaled logit
    __device__ __forceinline__ bool candidate(int i, float logit, unsigned long long* key, float* scaled) const {
        *scaled = logit * inv_t;
        if (!(*scaled >= cutoff)) return false;
        *key = ((unsigned long long)float_order(*scaled) << 32) | (uint32_t)(0xffffffffu - (uint32_t)i);
        return *key >= key_floor;
    }
    // its weight, and whether min-p keeps it
    __device__ __forceinline__ bool weighs(float scaled, float* weight) const {
        *weight = expf(scaled - scaled_max);
        return (double)*weight >= min_weight;
    }
    __device__ __forceinline__ bool member(int i, float logit, unsigned long long* key, float* weight) const {
        float scaled;
        return candidate(i, logit, key, &scaled) && weighs(scaled, weight);
    }
};

// f(i, row[i]) for every logit of a row, a lane's in ascending order, eight loads asked for before the first is used (a pass
// over a row is a chain of loads otherwise, each waiting for the one before); loads of 16 bytes where the row allows them
// (a vocabulary that is a multiple of four: a quarter of the loads, and of the waits).
#define SAMPLE_AHEAD 8
template <typename F>
__device__ __forceinline__ void for_each_logit(const float* __restrict__ row, int vocab, F f) {
    if ((vocab & 3) == 0 && ((size_t)row & 15) == 0) {
        const float4* __restrict__ row4 = (const float4*)row;
        const int quads = vocab >> 2;
        constexpr int QUADS_AHEAD = SAMPLE_AHEAD / 2;               // as many bytes on their way as fit the registers of 1,024 lanes
        for (int base = threadIdx.x; base < quads; base += QUADS_AHEAD * blockDim.x) {
            float4 v[QUADS_AHEAD];
#pragma unroll
            for (int j = 0; j < QUADS_AHEAD; ++j) {
                const int q = base + j * blockDim.x;
                v[j] = q < quads ? row4[q] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
#pragma unroll
            for (int j = 0; j < QUADS_AHEAD; ++j) {
                const int q = base + j * blockDim.x;
                if (q < quads) {
                    f(4 * q, v[j].x);
                    f(4 * q + 1, v[j].y);
                    f(4 * q + 2, v[j].z);
                    f(4 * q + 3, v[j].w);
                }
            }
        }
        return;
    }
    for (int base = threadIdx.x; base < vocab; base += SAMPLE_AHEAD * blockDim.x) {
        float v[SAMPLE_AHEAD];
#pragma unroll
        for (int j = 0; j < SAMPLE_AHEAD; ++j) {
            const int i = base + j * blockDim.x;
            v[j] = i < vocab ? row[i] : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < SAMPLE_AHEAD; ++j) {
            const int i = base + j * blockDim.x;
            if (i < vocab) f(i, v[j]);
        }
    }
}

// The histogram of one level: for each value of the key's byte the measure of the candidates that have it (masses or
// counts), how many they are, and the key of one of them (the key of the only one, where there is one).
struct Bins {
    unsigned long long measure[256];
    unsigned long long key[256];
    unsigned int count[256];
};

// What a lane has gathered for one bin goes to the workgroup's histogram: where all lanes of the wave mean the same bin (the
// usual case: neighbouring logits share their leading bits) the wave adds up first and one lane goes to memory.  Integer
// sums: the order of the additions changes nothing.
__device__ __forceinline__ void add_to_bin(Bins* bins, int bin, unsigned long long m, unsigned int n, unsigned long long key) {
    const int first = __builtin_amdgcn_readfirstlane(bin);
    if (__all(bin == first)) {
        if (n != 0) bins->key[first] = key;       // any of them: the key is only looked at where the bin holds one candidate
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            m += __shfl_xor(m, off, KIPP_WAVE);
            n += __shfl_xor(n, off, KIPP_WAVE);
        }
        if ((threadIdx.x & (KIPP_WAVE - 1)) == 0 && n != 0) {
            atomicAdd(&bins->measure[first], m);
            atomicAdd(&bins->count[first], n);
        }
    } else if (n != 0) {
        atomicAdd(&bins->measure[bin], m);
        atomicAdd(&bins->count[bin], n);
        bins->key[bin] = key;
    }
}

// One pass over the row: the candidates whose key begins with `prefix` above `level` (level 7: all; `only_byte` >= 0: those
// with that top byte alone) go into `bins` by the key's byte at `level`.  A lane keeps what it has gathered for the bin it met
// last and goes to the histogram only when the bin changes; the exponential is taken only of candidates under the prefix.
template <bool MASS>
__device__ __forceinline__ void gather(const SampleRow& r, int level, unsigned long long prefix, int only_byte, Bins* bins) {
    int at_bin = 0;
    unsigned int n = 0;
    unsigned long long sum = 0, last_key = 0;
    // Most logits of a pass fall to a comparison of two floats: the key's upper half is a monotone image of the scaled logit,
    // so the keys at or above the floor, under a prefix that lies within that half (levels 6 to 4), or with one top byte, are
    // the scaled logits of a range, and only what lies in it goes through the exact tests below.
    uint32_t order_lo = (uint32_t)(r.key_floor >> 32), order_hi = 0xffffffffu;
    if (level >= 4 && level < 7) {
        const int free_bits = 8 * (level + 1) - 32;
        const uint32_t first = (uint32_t)(prefix << free_bits);
        order_lo = first > order_lo ? first : order_lo;
        order_hi = first | ((1u << free_bits) - 1u);
    } else if (level == 7 && only_byte >= 0) {
        const uint32_t first = (uint32_t)only_byte << 24;
        order_lo = first > order_lo ? first : order_lo;
        order_hi = first | 0x00ffffffu;
    }
    const float range_lo = fmaxf(float_of_order(order_lo), r.cutoff), range_hi = float_of_order(order_hi);
    for_each_logit(r.row, r.vocab, [&](int i, float logit) {
        unsigned long long key;
        float scaled, w = 1.0f;
        if (!(logit * r.inv_t >= range_lo && logit * r.inv_t <= range_hi)) return;
        if (!r.candidate(i, logit, &key, &scaled)) return;
        if (level < 7 && (key >> (8 * (level + 1))) != prefix) return;
        if (only_byte >= 0 && (int)(key >> 56) != only_byte) return;
        if ((MASS || r.min_weight > 0.0) && !r.weighs(scaled, &w)) return;
        const int bin = (int)((key >> (8 * level)) & 0xff);
        if (bin != at_bin && n != 0) {
            atomicAdd(&bins->measure[at_bin], sum);
            atomicAdd(&bins->count[at_bin], n);
            bins->key[at_bin] = last_key;
            sum = 0;
            n = 0;
        }
        at_bin = bin;
        sum += MASS ? (unsigned long long)(w * MASS_SCALE) : 1ull;
        n += 1;
        last_key = key;
    });
    add_to_bin(bins, at_bin, sum, n, last_key);
}

// Walk down the key bytes.  With MASS the measure of a candidate is its fixed-point weight,
// else 1.  Finds the first candidate in key order (descending) at which the running measure
// reaches `target` (STRICT: exceeds it).  Returns its key; *before gets the measure of the
// candidates ahead of it, *own its own measure.  If the target is beyond the total, the
// last candidate is returned.  The walk ends at the level whose chosen byte one candidate alone
// has: that candidate is the answer, and the levels below would add nothing ahead of it.
// `fraction` (not null): the target is *fraction times the measure of all candidates, which the
// top level's histogram adds up to.  `top` (not null) with `keep`: the top level's histogram is
// left there; without `keep`: it is taken from there for the bytes above the floor's (their
// candidates have not changed since: only the floor was raised), and the floor's own byte is
// gathered again.
template <bool MASS, bool STRICT>
__device__ unsigned long long descend(const SampleRow& r, double target, const double* fraction, Bins* bins, Bins* top, bool keep,
                                      unsigned long long* shared, double* before, double* own) {
    unsigned long long prefix = 0;      // the key bytes fixed so far, right-aligned
    unsigned long long ahead = 0;       // the measure of the candidates ahead of the prefix: an integer, exact
    for (int level = 7; level >= 0; --level) {
        if (level == 3) {               // byte 3 is the top byte of the inverted index: always 0xff (vocab < 2^24)
            prefix = (prefix << 8) | 0xffull;
            continue;
        }
        const int floor_byte = (int)(r.key_floor >> 56);
        const bool reuse = level == 7 && top != nullptr && !keep;
        for (int b = threadIdx.x; b < 256; b += blockDim.x) {
            const bool from_top = reuse && b > floor_byte;
            bins->measure[b] = from_top ? top->measure[b] : 0;
            bins->count[b] = from_top ? top->count[b] : 0;
            if (from_top) bins->key[b] = top->key[b];
        }
        __syncthreads();
        gather<MASS>(r, level, prefix, reuse ? floor_byte : -1, bins);
        __syncthreads();
        if (level == 7 && top != nullptr && keep) {
            for (int b = threadIdx.x; b < 256; b += blockDim.x) {
                top->measure[b] = bins->measure[b];
                top->count[b] = bins->count[b];
                top->key[b] = bins->key[b];
            }
        }
        // The byte at which the running measure reaches the target, found by the first wave: a lane takes four bins (the
        // highest bytes first), the lanes' sums are scanned across the wave, and every lane looks for the place among its own.
        if (threadIdx.x < KIPP_WAVE) {
            const int l = threadIdx.x;
            unsigned long long h[4], mine = 0;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                h[q] = bins->measure[255 - 4 * l - q];
                mine += h[q];
            }
            unsigned long long through = mine;                     // of this lane's bins and of all lanes before it
#pragma unroll
            for (int off = 1; off < KIPP_WAVE; off <<= 1) {
                const unsigned long long other = __shfl_up(through, off, KIPP_WAVE);
                if (l >= off) through += other;
            }
            const unsigned long long total = __shfl(through, KIPP_WAVE - 1, KIPP_WAVE);
            if (level == 7 && fraction != nullptr) target = *fraction * (double)total;
            unsigned long long run = ahead + (through - mine), run_there = 0;
            int found = -1, low = -1;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (h[q] == 0) continue;
                low = 255 - 4 * l - q;
                if (found >= 0) continue;
                const unsigned long long next = run + h[q];
                if (STRICT ? (double)next > target : (double)next >= target) {
                    found = 255 - 4 * l - q;
                    run_there = run;
                } else {
                    run = next;
                }
            }
            const unsigned long long reached = __ballot(found >= 0), filled = __ballot(mine != 0);
            int chosen = 0;
            unsigned long long chosen_run = ahead;
            if (reached != 0) {
                const int from = __ffsll((long long)reached) - 1;
                chosen = __shfl(found, from, KIPP_WAVE);
                chosen_run = __shfl(run_there, from, KIPP_WAVE);
            } else if (filled != 0) {   // the target lies beyond everything: the last candidate
                chosen = __shfl(low, 63 - __clzll((long long)filled), KIPP_WAVE);
                chosen_run = ahead + total - bins->measure[chosen];
            }
            if (l == 0) {
                shared[0] = (unsigned long long)chosen;
                shared[1] = chosen_run;
                shared[2] = bins->measure[chosen];
                shared[3] = bins->count[chosen] == 1 ? bins->key[chosen] : 0;       // (no key is 0: byte 3 is 0xff)
                shared[4] = (unsigned long long)__double_as_longlong(target);
            }
        }
        __syncthreads();
        prefix = (prefix << 8) | shared[0];
        ahead = shared[1];
        *own = (double)shared[2];
        const unsigned long long alone = shared[3];
        target = __longlong_as_double((long long)shared[4]);
        __syncthreads();
        if (alone != 0) {
            prefix = alone;
            break;
        }
    }
    *before = (double)ahead;
    return prefix;
}

__global__ void __launch_bounds__(SAMPLE_THREADS) sample_kernel(
    const float* __restrict__ logits, int vocab, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const float* __restrict__ min_p, const double* __restrict__ uniform,
    int32_t* __restrict__ out) {
    __shared__ Bins bins, top;
    __shared__ unsigned long long shared[5];
    __shared__ unsigned long long list_key[SAMPLE_LIST], list_mass[SAMPLE_LIST];
    __shared__ unsigned int list_n;
    __shared__ float best_v[16];
    __shared__ int best_i[16];
    const int rowi = blockIdx.x;
    const float* row = logits + (size_t)rowi * vocab;
    // ---- the maximum, the lowest index among equals
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for_each_logit(row, vocab, [&](int i, float v) {
        if (v > bv || (bi == 0x7fffffff && !(v != v))) {
            bv = v;
            bi = i;
        }
    });
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off, KIPP_WAVE);
        const int oi = __shfl_xor(bi, off, KIPP_WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        best_v[threadIdx.x >> 6] = bv;
        best_i[threadIdx.x >> 6] = bi;
    }
    __syncthreads();
    bv = best_v[0];
    bi = best_i[0];
    for (int w = 1; w < SAMPLE_THREADS / KIPP_WAVE; ++w)
        if (best_v[w] > bv || (best_v[w] == bv && best_i[w] < bi)) {
            bv = best_v[w];
            bi = best_i[w];
        }
    if (bi == 0x7fffffff) bi = 0;
    const float t = temperature[rowi];
    if (!(t > 0.0f)) {                      // greedy
        if (threadIdx.x == 0) out[rowi] = bi;
        return;
    }
    SampleRow r;
    r.row = row;
    r.vocab = vocab;
    r.inv_t = 1.0f / t;
    r.scaled_max = bv * r.inv_t;
    r.cutoff = r.scaled_max - 20.0f;
    r.key_floor = 0;
    r.min_weight = 0.0;
    double before, own;
    // ---- top-k: the key of the k-th candidate is the floor of what stays
    const int k = top_k[rowi];
    if (k > 0) r.key_floor = descend<false, false>(r, (double)k, nullptr, &bins, nullptr, false, shared, &before, &own);
    // ---- min-p relative to the top weight, which is exp(0) = 1
    const float mp = min_p[rowi];
    if (mp > 0.0f) r.min_weight = (double)mp;
    const double share = (double)top_p[rowi];
    bool few = k > 0 && k <= SAMPLE_LIST;
    if (!few) {
        // how many candidates there are (logits within 20 of the largest, after the temperature: a few hundred of a trained
        // model's 150,000): a pass that takes no exponential
        if (threadIdx.x == 0) list_n = 0;
        __syncthreads();
        unsigned int mine = 0;
        for_each_logit(row, vocab, [&](int i, float logit) {
            unsigned long long key;
            float scaled;
            if (logit * r.inv_t >= r.cutoff && r.candidate(i, logit, &key, &scaled)) ++mine;
        });
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) mine += __shfl_xor(mine, off, KIPP_WAVE);
        if ((threadIdx.x & (KIPP_WAVE - 1)) == 0 && mine != 0) atomicAdd(&list_n, mine);
        __syncthreads();
        few = list_n <= SAMPLE_LIST;
        __syncthreads();
    }
    if (few) {
        // ---- few candidates are left: one pass gathers them, key and mass, into LDS, a lane a candidate; each
        //      adds up the masses of those ahead of it in key order, and the two questions (where does the mass reach
        //      top_p of the total; where does it exceed the draw's share of what is kept) are answered by the one candidate
        //      at which the running mass crosses the target: the answers of the two walks below, without their passes
        if (threadIdx.x == 0) list_n = 0;
        __syncthreads();
        for_each_logit(row, vocab, [&](int i, float logit) {
            unsigned long long key;
            float w;
            if (!r.member(i, logit, &key, &w)) return;
            const unsigned int at = atomicAdd(&list_n, 1u);
            if (at < SAMPLE_LIST) {
                list_key[at] = key;
                list_mass[at] = (unsigned long long)(w * MASS_SCALE);
            }
        });
        __syncthreads();
        const int n = (int)(list_n < SAMPLE_LIST ? list_n : SAMPLE_LIST);
        const bool have = (int)threadIdx.x < n;
        const unsigned long long my_key = have ? list_key[threadIdx.x] : 0, my_mass = have ? list_mass[threadIdx.x] : 0;
        unsigned long long ahead_of_me = 0, total = 0;
        int rank = 0;
        for (int j = 0; j < n; ++j) {
            const unsigned long long other = list_key[j], mass = list_mass[j];
            total += mass;
            if (other > my_key) {
                ahead_of_me += mass;
                ++rank;
            }
        }
        if (threadIdx.x == 0) shared[0] = 0;
        __syncthreads();
        const double reach = share * (double)total;
        if (have && (double)(ahead_of_me + my_mass) >= reach && (rank == 0 || !((double)ahead_of_me >= reach))) {
            shared[0] = my_key;                                                     // the last candidate that top-p keeps
            shared[1] = (unsigned long long)__double_as_longlong((double)ahead_of_me + (double)my_mass);
        }
        __syncthreads();
        if (shared[0] == 0 && have && rank == n - 1) {                              // (beyond everything: the last candidate)
            shared[0] = my_key;
            shared[1] = (unsigned long long)__double_as_longlong((double)ahead_of_me + (double)my_mass);
        }
        __syncthreads();
        const unsigned long long last_kept = shared[0];
        const double kept_mass = __longlong_as_double((long long)shared[1]), draw = uniform[rowi] * kept_mass;
        __syncthreads();
        if (threadIdx.x == 0) shared[2] = 0;
        __syncthreads();
        const bool kept_one = have && my_key >= last_kept;
        if (kept_one && (double)(ahead_of_me + my_mass) > draw && (rank == 0 || !((double)ahead_of_me > draw))) shared[2] = my_key;
        __syncthreads();
        if (shared[2] == 0 && kept_one && my_key == last_kept) shared[2] = my_key;  // (beyond everything: the last one kept)
        __syncthreads();
        if (threadIdx.x == 0) out[rowi] = (int32_t)(0xffffffffu - (uint32_t)(shared[2] & 0xffffffffu));
        return;
    }
    if (!(share < 1.0)) {
        // ---- top-p keeps everything: the draw's share of the total mass, in one walk
        const double part = uniform[rowi];
        const unsigned long long pick = descend<true, true>(r, 0.0, &part, &bins, nullptr, false, shared, &before, &own);
        if (threadIdx.x == 0) out[rowi] = (int32_t)(0xffffffffu - (uint32_t)(pick & 0xffffffffu));
        return;
    }
    // ---- top-p: the shortest prefix whose mass reaches top_p of the total (the total: what the top level's histogram adds up to)
    const unsigned long long last = descend<true, false>(r, 0.0, &share, &bins, &top, true, shared, &before, &own);
    if (last > r.key_floor) r.key_floor = last;
    const double kept = before + own;
    // ---- the draw, among what is kept: above the floor's byte the top level's histogram still holds
    const unsigned long long pick = descend<true, true>(r, uniform[rowi] * kept, nullptr, &bins, &top, false, shared, &before, &own);
    if (threadIdx.x == 0) out[rowi] = (int32_t)(0xffffffffu - (uint32_t)(pick & 0xffffffffu));
}

extern "C" int kipp_sample(const float* logits, int rows, int vocab, const float* temperature, const int32_t* top_k,
                           const float* top_p, const float* min_p, const double* uniform, int32_t* out,
                           hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0 || vocab >= (1 << 24)) return -1;
    hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(SAMPLE_THREADS), 0, stream, logits, vocab, temperature, top_k,
                       top_p, min_p, uniform, out);
    return KIPP_LAUNCH_CHECK();
}
