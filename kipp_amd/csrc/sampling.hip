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

#define SAMPLE_THREADS 1024
#define MASS_SCALE 17592186044416.0f   // 2^44

__device__ __forceinline__ uint32_t float_order(float x) {
    const uint32_t b = __float_as_uint(x);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);   // larger float, larger integer
}

struct SampleRow {
    const float* row;
    int vocab;
    float inv_t, scaled_max, cutoff;
    unsigned long long key_floor;   // candidates of the top-k cut have key >= key_floor
    double min_weight;              // ... and weight >= min_weight (0: no min-p)

    __device__ __forceinline__ bool member(int i, unsigned long long* key, float* weight) const {
        const float scaled = row[i] * inv_t;
        if (!(scaled >= cutoff)) return false;
        *key = ((unsigned long long)float_order(scaled) << 32) | (uint32_t)(0xffffffffu - (uint32_t)i);
        if (*key < key_floor) return false;
        *weight = expf(scaled - scaled_max);
        return (double)*weight >= min_weight;
    }
};

// Walk down the key bytes.  With MASS the measure of a candidate is its fixed-point weight,
// else 1.  Finds the first candidate in key order (descending) at which the running measure
// reaches `target` (STRICT: exceeds it).  Returns its key; *before gets the measure of the
// candidates ahead of it, *own its own measure.  If the target is beyond the total, the
// last candidate is returned.
template <bool MASS, bool STRICT>
__device__ unsigned long long descend(const SampleRow& r, double target, unsigned long long* hist,
                                      unsigned long long* shared, double* before, double* own) {
    unsigned long long prefix = 0;      // the key bytes fixed so far, right-aligned
    double ahead = 0.0;
    for (int level = 7; level >= 0; --level) {
        if (level == 3) {               // byte 3 is the top byte of the inverted index: always 0xff (vocab < 2^24)
            prefix = (prefix << 8) | 0xffull;
            continue;
        }
        for (int b = threadIdx.x; b < 256; b += blockDim.x) hist[b] = 0;
        __syncthreads();
        for (int i = threadIdx.x; i < r.vocab; i += blockDim.x) {
            unsigned long long key;
            float w;
            if (!r.member(i, &key, &w)) continue;
            if (level < 7 && (key >> (8 * (level + 1))) != prefix) continue;
            const unsigned long long m = MASS ? (unsigned long long)(w * MASS_SCALE) : 1ull;
            atomicAdd(&hist[(key >> (8 * level)) & 0xff], m);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            int chosen = -1, lowest = 0;
            double run = ahead;
            for (int b = 255; b >= 0; --b) {
                if (hist[b] == 0) continue;
                lowest = b;
                const double next = run + (double)hist[b];
                if (STRICT ? next > target : next >= target) {
                    chosen = b;
                    break;
                }
                run = next;
            }
            if (chosen < 0) {           // the target lies beyond everything: the last candidate
                chosen = lowest;
                run -= (double)hist[lowest];
            }
            shared[0] = (unsigned long long)chosen;
            shared[1] = (unsigned long long)__double_as_longlong(run);
            shared[2] = hist[chosen];
        }
        __syncthreads();
        prefix = (prefix << 8) | shared[0];
        ahead = __longlong_as_double((long long)shared[1]);
        *own = (double)shared[2];
        __syncthreads();
    }
    *before = ahead;
    return prefix;
}

__global__ void __launch_bounds__(SAMPLE_THREADS) sample_kernel(
    const float* __restrict__ logits, int vocab, const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
    const float* __restrict__ top_p, const float* __restrict__ min_p, const double* __restrict__ uniform,
    int32_t* __restrict__ out) {
    __shared__ unsigned long long hist[256];
    __shared__ unsigned long long shared[4];
    __shared__ float best_v[16];
    __shared__ int best_i[16];
    const int rowi = blockIdx.x;
    const float* row = logits + (size_t)rowi * vocab;
    // ---- the maximum, the lowest index among equals
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
    if (k > 0) r.key_floor = descend<false, false>(r, (double)k, hist, shared, &before, &own);
    // ---- min-p relative to the top weight, which is exp(0) = 1
    const float mp = min_p[rowi];
    if (mp > 0.0f) r.min_weight = (double)mp;
    // ---- top-p: the shortest prefix whose mass reaches top_p of the total
    for (int b = threadIdx.x; b < 4; b += blockDim.x) shared[b] = 0;
    __syncthreads();
    unsigned long long mine = 0;
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
        unsigned long long key;
        float w;
        if (r.member(i, &key, &w)) mine += (unsigned long long)(w * MASS_SCALE);
    }
    atomicAdd(&shared[3], mine);
    __syncthreads();
    const double total = (double)shared[3];
    __syncthreads();
    const unsigned long long last = descend<true, false>(r, (double)top_p[rowi] * total, hist, shared, &before, &own);
    if (last > r.key_floor) r.key_floor = last;
    const double kept = before + own;
    // ---- the draw
    const unsigned long long pick = descend<true, true>(r, uniform[rowi] * kept, hist, shared, &before, &own);
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
