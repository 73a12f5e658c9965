// Matrix product for prompt portions (hundreds to thousands of rows):
// Y[M, N] = X[M, K] . W[N, K]^T, bfloat16 operands, float32 accumulation on
// v_mfma_f32_32x32x16_bf16, K a multiple of 32.
//
// A workgroup of 4 waves (2 x 2, one a SIMD) or of 8 (2 x 4, two a SIMD) owns a tile of outputs; a wave holds
// WM x WN accumulator tiles of 32 x 32 (4 waves of 4 x 4, or 8 waves of 4 x 2: a workgroup tile of 256 x 256;
// also smaller ones, chosen by the launcher so that the tiles of a product fill the 256 compute units in whole
// rounds, or by the caller).  It walks K in steps of 32 columns.  The pieces of X and W of a step go from
// global memory straight into LDS (global_load_lds_dwordx4: no registers, no waiting wave), four
// steps deep.  In LDS four rows of a piece share 256 bytes, whose sixteen 16-byte slots are permuted
// by the low bits of the group's index: the 16 lanes that read one operand column together then hit
// sixteen different slots (no bank conflict is counted), and a wave's DMA instruction still writes
// one contiguous KB.
//
// With one wave a SIMD, whatever holds up its instruction stream idles the matrix cores.  Every other
// instruction of the walk (the reads of the next operands out of LDS, the DMA of the steps ahead) is
// therefore placed between two products, a few at a time, and the barrier of a step falls between its two
// halves.  Measured with the shader clock around the walk: 37.5 cycles a
// product where the matrix core needs 32; 33.5 with the DMA taken out: a wave that issues
// a DMA instruction cannot issue its next product in time, which a second wave on the SIMD hides.  In the
// run of a prefill the chip is at its power limit, and the time of a product is set by that, not by the
// cycles: the cuts differ by a few per cent, and which is fastest for a shape is found by the clock.
//
// An output element is summed over K in the same order whatever the tile and the number of waves: cuts
// with the same parts of K give the same bits.
//
// The result leaves through one of three ends:
//   slabs   float32 [parts, M, N]: K is split over `parts` workgroups (grid.z) where the tiles
//           alone would leave compute units idle, and the consumer adds the slabs in order
//           (the residual add, the rotary kernel: no atomics, the same bits every time);
//   swiglu  W = [gate; up] ([2 I, K]): a wave's columns are gate rows and the up rows that belong
//           to them, a lane holds both values of an output, and bfloat16(silu(gate) * up)
//           [M, I] is all that is written (/root/reference/src/kipp.c:2633-2653);
//   bf16    bfloat16 [M, N].
// The bfloat16 ends pass through LDS so that a lane stores 16 bytes of one row.
//
// Tiles are handed to the 8 dies of the GPU in blocks: workgroups that run on one die (every
// eighth one) take tiles that share their rows of W, which that die's L2 then serves.
#include "common.h"

#define BK 32                                      // columns of a step
#define CHUNKS (BK / 8)                            // 16-byte chunks of a row of a piece
#define GROUP_ROWS (16 / CHUNKS)                   // rows that share 256 bytes of LDS
#define INSTR_ROWS (4 * GROUP_ROWS)                // rows one DMA instruction of a wave brings (1 KB)

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

union Frag {
    u32x4 u;
    bf16x8 v;
};

#define LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

enum { END_SLABS = 0, END_SWIGLU = 1, END_BF16 = 2 };

// silu(g) * u with the exponential of the hardware (base 2)
__device__ __forceinline__ float swiglu_of(float g, float u) {
    return g / (1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g)) * u;
}

// every operand register of a set is tied to the wait for its reads, so that no product moves in front of it
template <int WM, int WN>
__device__ __forceinline__ void wait_reads(u32x4 (&fa)[WM], u32x4 (&fb)[WN]) {
    if constexpr (WM == 4 && WN == 4)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]));
    else if constexpr (WM == 4 && WN == 3)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]));
    else if constexpr (WM == 2 && WN == 3)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]));
    else if constexpr (WM == 4)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]), "+v"(fa[3]), "+v"(fb[0]), "+v"(fb[1]));
    else if constexpr (WN == 4)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fb[0]), "+v"(fb[1]), "+v"(fb[2]), "+v"(fb[3]));
    else
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[0]), "+v"(fa[1]), "+v"(fb[0]), "+v"(fb[1]));
}

// Steps of K that are in LDS or on their way there: four.  (Tiles of half the size with three steps and two
// workgroups a compute unit, i.e. two waves a SIMD from two workgroups, were measured and are no faster: those
// tiles move half as many bytes again through the DMA for the same products.  Two waves a SIMD on the full tile
// are the 8-wave cuts.)
template <int WM, int WN>
struct Depth {
    static constexpr int value = 4;
};

template <int WM, int WN, int END, int WGN = 2>
__global__ void __launch_bounds__(64 * 2 * WGN, 1) gemm_tiles_kernel(
    const bf16_t* __restrict__ X, const bf16_t* __restrict__ W, void* __restrict__ Y, int M, int N, int K,
    int tiles_m, int tiles_n, int parts, int inner, int col_begin, int col_end) {
    constexpr int STAGES = Depth<WM, WN>::value;
    constexpr int WAVES = 2 * WGN;                                // 2 down, WGN across (2: one wave a SIMD, 4: two)
    constexpr int TM = 64 * WM, TN = 32 * WN * WGN;               // the workgroup's tile
    constexpr int X_PIECE = TM * BK * 2, W_PIECE = TN * BK * 2;   // bytes of a step's pieces
    constexpr int STAGE_BYTES = X_PIECE + W_PIECE;
    constexpr int XI = TM / INSTR_ROWS / WAVES, WI = TN / INSTR_ROWS / WAVES;   // DMA instructions of a wave for each piece
    static_assert(XI >= 1 && XI * INSTR_ROWS * WAVES == TM && WI * INSTR_ROWS * WAVES == TN, "the waves share the pieces evenly");
    constexpr int LOADS = XI + WI;                                // DMA instructions a wave issues a step
    constexpr int NM = WM * WN;                                   // products of a half step
    constexpr int NR = WM + WN;                                   // operand reads of a half step
    constexpr int OUT_N = END == END_SWIGLU ? TN / 2 : TN;        // output columns of a tile
    static_assert((WM == 2 || WM == 4) && (WN == 2 || WN == 3 || WN == 4), "wave tiles of 2 or 4 MFMA tiles down, 2 to 4 across");
    static_assert(WN != 3 || END == END_SLABS, "three tiles across only for the float32 end");
    static_assert((STAGES - 1) * LOADS < 64, "the wait counts below must fit the counter");
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31, hh = lane >> 5;
    const int wm = wave / WGN, wn = wave % WGN;

    // ---- which tile: workgroups id, id + 8, id + 16, ... run on one die; each die takes a run of
    //      consecutive tiles, rows of X fastest, so that its tiles share rows of W
    const int n_tiles = tiles_m * tiles_n;
    const int id = blockIdx.x;
    const int per_die = (n_tiles + 7) / 8;
    const int tile = (id & 7) * per_die + (id >> 3);
    if ((id >> 3) >= per_die || tile >= n_tiles) return;          // the grid is rounded up to whole dies
    const int tm = tile % tiles_m, tn = tile / tiles_m;
    const int part = blockIdx.z;
    const int steps_all = K / BK;
    const int s_begin = (int)((long long)steps_all * part / parts);
    const int nk = (int)((long long)steps_all * (part + 1) / parts) - s_begin;

    // ---- the DMA: a wave brings a quarter of each piece, INSTR_ROWS rows an instruction; a lane brings the
    //      16 bytes that belong at its place of the KB: group g = 4 i + lane / 16 of GROUP_ROWS rows, slot
    //      s = lane % 16, which holds chunk s ^ (g % CHUNKS) of the group: row (that / CHUNKS) of the group,
    //      columns 8 (that % CHUNKS) .. + 7
    const int q4 = lane >> 4, s16 = lane & 15;
    const int in_group = s16 ^ (q4 & (CHUNKS - 1));
    const int lane_row = GROUP_ROWS * q4 + in_group / CHUNKS, col8 = (in_group % CHUNKS) * 8;
    // an address is a base that all lanes share (it walks along K in scalar registers) plus a lane's own 32-bit
    // offset, which never changes: no vector arithmetic for an address inside the walk (the launcher refuses
    // operands of 4 GiB and more)
    uint32_t x_src[XI], w_src[WI];
    const unsigned char* x_base = (const unsigned char*)(X + (size_t)s_begin * BK);
    const unsigned char* w_base = (const unsigned char*)(W + (size_t)s_begin * BK);
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        const int r = (TM / WAVES) * wave + INSTR_ROWS * i + lane_row;
        x_src[i] = (uint32_t)(((size_t)min(tm * TM + r, M - 1) * K + col8) * 2);
    }
#pragma unroll
    for (int i = 0; i < WI; ++i) {
        const int r = (TN / WAVES) * wave + INSTR_ROWS * i + lane_row;    // row of the piece
        int wr;
        if (END == END_SWIGLU) {
            // the 32 WN rows of the piece that a wave multiplies are 16 WN gate rows, then the 16 WN up rows that
            // belong to them (`half`: which of the WGN waves across)
            const int half = r / (32 * WN), within = r % (32 * WN);
            const int c = col_begin + tn * OUT_N + 16 * WN * half + within % (16 * WN);
            wr = min(c, col_end - 1) + (within >= 16 * WN ? inner : 0);
        } else {
            wr = min(col_begin + tn * TN + r, col_end - 1);
        }
        w_src[i] = (uint32_t)(((size_t)wr * K + col8) * 2);
    }
    // where step `step` of an operand begins, for every lane: pinned to scalar registers (left to itself the
    // compiler adds the lane's offset first and then walks a 64-bit vector address along K)
    auto step_base = [&](const unsigned char* base, int step) {
        const unsigned char* at = base + (size_t)step * (BK * 2);
        asm volatile("" : "+s"(at));
        return at;
    };
    auto issue_one = [&](const unsigned char* x_at, const unsigned char* w_at, int stage, int n) {   // DMA instruction n (0 .. LOADS - 1) of a step
        // the lane's offset passes through an empty asm here, so that its widening to 64 bits stands beside the
        // load: the compiler then takes the form "scalar base + 32-bit vector offset" and adds nothing per load
        // (widened once outside the walk, the offset would cost a 64-bit vector add for every load)
        // (in place: the offset keeps its own register for the whole walk.  A copy in a scratch register could be
        // handed to a read out of LDS as its destination right behind the DMA instruction, and nothing says how
        // long the memory pipeline takes to fetch an instruction's address registers)
        unsigned char* dst = lds + stage * STAGE_BYTES;
        if (n < XI) {
            uint32_t& off = x_src[n < XI ? n : 0];
            asm volatile("" : "+v"(off));
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(x_at + off), LDS_PTR(dst + wave * (X_PIECE / WAVES) + 1024 * n), 16, 0, 0);
        } else {
            uint32_t& off = w_src[n < XI ? 0 : n - XI];
            asm volatile("" : "+v"(off));
            __builtin_amdgcn_global_load_lds(GLOBAL_PTR(w_at + off), LDS_PTR(dst + X_PIECE + wave * (W_PIECE / WAVES) + 1024 * (n - XI)), 16, 0, 0);
        }
    };

    // ---- a lane's place in the operands: row 32 j + l32 of the wave's rows, chunk 2 t + hh of the step
    int frag_at[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        const int group = l32 / GROUP_ROWS;
        frag_at[t] = group * 256 + (((CHUNKS * (l32 % GROUP_ROWS) + 2 * t + hh) ^ (group & (CHUNKS - 1))) << 4);
    }
    const int a_base = wm * (X_PIECE / 2), b_base = X_PIECE + wn * (W_PIECE / WGN);

    f32x16 acc[WM][WN];
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // ---- the walk over K.  The operands of a product leave LDS through reads written out by hand (through
    //      ordinary loads the compiler would make every read wait for all DMA into LDS that is on its way), asked
    //      for one half step ahead.  Steps beyond the last are asked for again from the last one (into a buffer
    //      that nobody reads any more), so that the count of loads on their way is the same at every step.
    u32x4 a[2][WM], b[2][WN];
    // read R of a half step: the first row operand, every column operand, then the other row operands (the
    // order in which the products below want them)
#define KIPP_READ_ONE(T, STEP, KS, R)                                                                              \
    do {                                                                                                           \
        const uint32_t st_ = (uint32_t)(uintptr_t)LDS_PTR(lds + ((STEP) % STAGES) * STAGE_BYTES);                  \
        const uint32_t a_at_ = st_ + a_base + frag_at[KS], b_at_ = st_ + b_base + frag_at[KS];                     \
        if ((R) == 0) asm volatile("ds_read_b128 %0, %1" : "=v"(a[T][0]) : "v"(a_at_));                            \
        else if ((R) <= WN)                                                                                        \
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(b[T][(R) <= WN ? (R) - 1 : 0]) : "v"(b_at_), "i"(((R) - 1) * 32 * BK * 2)); \
        else                                                                                                       \
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(a[T][(R) > WN ? (R) - WN : 0]) : "v"(a_at_), "i"(((R) - WN) * 32 * BK * 2)); \
    } while (0)
#define KIPP_PRODUCT(T, M_)                                                                         \
    do {                                                                                            \
        Frag fa, fb;                                                                                \
        fa.u = a[T][(M_) / WN];                                                                     \
        fb.u = b[T][(M_) % WN];                                                                     \
        acc[(M_) / WN][(M_) % WN] =                                                                 \
            __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa.v, fb.v, acc[(M_) / WN][(M_) % WN], 0, 0, 0); \
    } while (0)

    // The DMA instructions of a step go out in two groups, half a step apart: the first LOADS_EARLY of step
    // kt + STAGES behind the products of the second half of step kt (into the buffer of step kt, which every wave
    // has left at the barrier in the middle of step kt), the others behind the products of the first half of
    // step kt + 1.  So a wave asks for 1 KB every third product and not every product for half of the time:
    // the four waves' requests together then stay under what the compute unit's path to memory takes, and no
    // wave waits to hand one in (measured: 20 cycles an instruction when they all came behind one another).
    constexpr int LOADS_EARLY = (LOADS + 1) / 2, LOADS_LATE = LOADS - LOADS_EARLY;
    // the items of a half step: NR reads of operands, one behind each of the first products, then D DMA
    // instructions spread over the products that are left (all spread evenly where there are more items than products)
#define KIPP_ITEMS(D, M_, READ, DMA)                                                          \
    do {                                                                                      \
        constexpr int T_ = NR + (D);                                                          \
        _Pragma("unroll") for (int p_ = 0; p_ < T_; ++p_) {                                   \
            const int behind_ = T_ > NM ? p_ * NM / T_ : (p_ < NR ? p_ : NR + (p_ - NR) * (NM - NR) / (D)); \
            if (behind_ != (M_)) continue;                                                    \
            if (p_ >= NR) { DMA(p_ - NR); }                                                   \
            else { READ(p_); }                                                                \
        }                                                                                     \
    } while (0)

#pragma unroll
    for (int s = 0; s < STAGES; ++s) {
        const unsigned char* x_at = step_base(x_base, min(s, nk - 1));
        const unsigned char* w_at = step_base(w_base, min(s, nk - 1));
#pragma unroll
        for (int n = 0; n < (s == STAGES - 1 ? LOADS_EARLY : LOADS); ++n) issue_one(x_at, w_at, s, n);
    }
    // step 0 has arrived when steps 1 .. STAGES - 2 and the early part of step STAGES - 1 may still be on their way
    constexpr int AFTER_FIRST = (STAGES - 2) * LOADS + LOADS_EARLY;
    static_assert(AFTER_FIRST < 64, "the wait counts must fit the counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (AFTER_FIRST & 15) | ((AFTER_FIRST >> 4) << 14));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();                                  // bare, as in the walk below
    asm volatile("" ::: "memory");
#pragma unroll
    for (int r = 0; r < NR; ++r) KIPP_READ_ONE(0, 0, 0, r);
    for (int kt = 0; kt < nk; ++kt) {
        // first half: products of columns 0 .. 15 of the step; the operands of the second half arrive meanwhile,
        // and the late DMA instructions of step kt + STAGES - 1 go out, into the buffer of step kt - 1
        // (the scheduler may not carry instructions over the marks: the order written here is the order meant)
        wait_reads<WM, WN>(a[0], b[0]);
        __builtin_amdgcn_sched_barrier(0);
        const int late = min(kt + STAGES - 1, nk - 1), late_stage = (kt + STAGES - 1) % STAGES;
        const unsigned char* x_late = step_base(x_base, late);
        const unsigned char* w_late = step_base(w_base, late);
#define KIPP_READ_A(R) KIPP_READ_ONE(1, kt, 1, R)
#define KIPP_DMA_A(N_) issue_one(x_late, w_late, late_stage, LOADS_EARLY + (N_))
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            KIPP_PRODUCT(0, m);
            KIPP_ITEMS(LOADS_LATE, m, KIPP_READ_A, KIPP_DMA_A);
            __builtin_amdgcn_sched_barrier(0);
        }
        // second half: every wave's part of the next step has arrived (what may still be on its way: the steps
        // behind it), and every wave is done with this step's buffer (its operands are in registers), into which
        // the early DMA instructions of step kt + STAGES now go
        wait_reads<WM, WN>(a[1], b[1]);
        __builtin_amdgcn_s_waitcnt(0x0F70 | (((STAGES - 2) * LOADS) & 15) | ((((STAGES - 2) * LOADS) >> 4) << 14));
        // the bare barrier: __syncthreads() also fences, and the fence waits for EVERY load into LDS that is on
        // its way (the compiler writes vmcnt(0) for it), which would leave nothing in flight across a step
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        const int ahead = min(kt + STAGES, nk - 1);
        const unsigned char* x_ahead = step_base(x_base, ahead);
        const unsigned char* w_ahead = step_base(w_base, ahead);
#define KIPP_READ_B(R) KIPP_READ_ONE(0, kt + 1, 0, R)
#define KIPP_DMA_B(N_) issue_one(x_ahead, w_ahead, kt % STAGES, N_)
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            KIPP_PRODUCT(1, m);
            KIPP_ITEMS(LOADS_EARLY, m, KIPP_READ_B, KIPP_DMA_B);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#undef KIPP_READ_A
#undef KIPP_DMA_A
#undef KIPP_READ_B
#undef KIPP_DMA_B
#undef KIPP_ITEMS
    wait_reads<WM, WN>(a[0], b[0]);
    __builtin_amdgcn_s_waitcnt(0x0F70);      // nothing may still be on its way into LDS when the buffers are used again
#undef KIPP_READ_ONE
#undef KIPP_PRODUCT

    // ---- the ends.  In accumulator tile (i, j) a lane holds column l32 and rows 8 (v / 4) + 4 hh + v % 4.
    const int row0 = tm * TM + wm * (32 * WM);
    if (END == END_SLABS) {
        // a lane stores 4 bytes; the 32 lanes of a half wave 128 bytes of one row
        float* out = (float*)Y + (size_t)part * M * N;
        const int col0 = col_begin + tn * TN + wn * (32 * WN);
#pragma unroll
        for (int i = 0; i < WM; ++i)
#pragma unroll
            for (int j = 0; j < WN; ++j) {
                const int col = col0 + 32 * j + l32;
                if (col >= col_end) continue;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = row0 + 32 * i + 8 * (v / 4) + 4 * hh + (v % 4);
                    if (row < M) out[(size_t)row * N + col] = acc[i][j][v];
                }
            }
        return;
    }
    if constexpr (WN == 3) return;
    // bfloat16 ends: the wave's outputs, 32 rows at a time, go through its own corner of LDS (now free), from
    // which a lane takes 8 neighbouring columns of one row: 16 bytes a store, whole memory lines a row
    constexpr int WCOLS = END == END_SWIGLU ? 16 * WN : 32 * WN;   // output columns of a wave
    constexpr int PITCH = WCOLS + 8;                               // bf16 elements a staged row (the pad spreads the banks)
    static_assert(32 * PITCH * 2 <= STAGES * STAGE_BYTES / WAVES, "a wave's staging fits its share of LDS");
    __syncthreads();                                               // every wave is done reading operands
    bf16_t* stage = (bf16_t*)(lds + wave * (STAGES * STAGE_BYTES / WAVES));
    bf16_t* out = (bf16_t*)Y;
    const int out_width = END == END_SWIGLU ? inner : N;
    const int col0 = col_begin + tn * OUT_N + wn * WCOLS;
    constexpr int LANES_PER_ROW = WCOLS / 8, ROWS_PER_PASS = 64 / LANES_PER_ROW;
#pragma unroll
    for (int i = 0; i < WM; ++i) {
#pragma unroll
        for (int j = 0; j < WCOLS / 32; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = 8 * (v / 4) + 4 * hh + (v % 4);
                const float value = END == END_SWIGLU ? swiglu_of(acc[i][j][v], acc[i][(j + WN / 2) % WN][v]) : acc[i][j][v];
                stage[r * PITCH + 32 * j + l32] = f32_to_bf16(value);
            }
        // (a wave's lanes run in step: what the wave wrote it can read back without a barrier of the workgroup)
        __builtin_amdgcn_s_waitcnt(0xC07F);                        // lgkmcnt(0): the writes above have landed
#pragma unroll
        for (int pass = 0; pass < 32 / ROWS_PER_PASS; ++pass) {
            const int r = pass * ROWS_PER_PASS + lane / LANES_PER_ROW, c = (lane % LANES_PER_ROW) * 8;
            const u32x4 v = *(const u32x4*)(stage + r * PITCH + c);
            const int row = row0 + 32 * i + r, col = col0 + c;
            if (row < M) {
                if (col + 8 <= col_end && (out_width & 7) == 0) {
                    *(u32x4*)(out + (size_t)row * out_width + col) = v;
                } else {
                    const bf16_t* e = (const bf16_t*)&v;
                    for (int k = 0; k < 8; ++k)
                        if (col + k < col_end) out[(size_t)row * out_width + col + k] = e[k];
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);                        // the reads are done before the next 32 rows overwrite them
    }
}

// How a product is cut: the wave's tile (WM x WN MFMA tiles) and the parts of K, for a range of output columns.
// The cost of a cut is what its slowest compute unit does: rounds of tiles over the 256 units, each a fixed cost
// (first data, the stores of the end) plus the steps of its part of K.  Times in microseconds, measured at the
// benchmark's sizes; smaller wave tiles move more bytes through LDS for the same products and cost more a product.
struct Cut {
    int wm, wn, parts;
    int col_begin, col_end;     // output columns
    int wgn = 2;                // waves across: 2 (4 waves, one a SIMD) or 4 (8 waves, two a SIMD)
};

#define N_SHAPES 5
static const int kShapes[N_SHAPES][2] = {{4, 4}, {4, 3}, {4, 2}, {2, 4}, {2, 2}};
static const double kStep[N_SHAPES] = {0.80, 0.62, 0.47, 0.47, 0.27};    // one step of 32 columns of one tile
static const double kFixed[N_SHAPES] = {13.0, 11.0, 9.0, 9.0, 6.0};      // start and end of a tile

static double cut_cost(int M, int cols, int steps, int end, int shape, int parts) {
    const int tm = 64 * kShapes[shape][0], tn = end == END_SWIGLU ? 32 * kShapes[shape][1] : 64 * kShapes[shape][1];
    const long long tiles = (long long)((M + tm - 1) / tm) * ((cols + tn - 1) / tn);
    const long long rounds = (tiles * parts + 255) / 256;
    return rounds * (kFixed[shape] + kStep[shape] * ((steps + parts - 1) / parts)) + 1.0 * (parts - 1);
}

// Workgroups of 8 waves (wave tiles of 4 x 2, four across: the 256 x 256 tile with two waves a SIMD) for the whole rounds of
// 256 tiles, and the columns that are left, which would hold every compute unit for a round that few of them have a tile
// in, in smaller tiles: 8 waves on half the rows and columns, or (`rest` = 1, 2, 3) 4 waves on 256 x 64, 128 x 128, 128 x 64.
// Without whole rounds, or with nothing left, one cut of the 8-wave tile.
static int whole_rounds_then_rest(int M, int cols, int end, int rest, Cut* cuts) {
    cuts[0] = {4, 2, 1, 0, cols, 4};
    const int tm = 256, tn = (end == END_SWIGLU ? 16 : 32) * 2 * 4;
    const int tiles_m = (M + tm - 1) / tm;
    const long long whole = ((long long)tiles_m * (cols / tn)) / 256 * 256;
    const int first_cols = (int)(whole / tiles_m) * tn;
    if (first_cols <= 0 || first_cols >= cols) return 1;
    cuts[0].col_end = first_cols;
    static const int tiles[4][3] = {{2, 2, 4}, {4, 2, 2}, {2, 4, 2}, {2, 2, 2}};
    cuts[1] = {tiles[rest & 3][0], tiles[rest & 3][1], 1, first_cols, cols, tiles[rest & 3][2]};
    return 2;
}

// Up to two cuts, side by side in the output's columns.  The float32 end takes one cut, whose parts of K may be
// more than one.  The bfloat16 ends cannot split K; where whole rounds of the largest tile leave a rest of tiles
// that would hold the 256 units for another whole round, the rest of the columns is cut into smaller tiles.
static int plan(int M, int N, int K, int end, int max_parts, Cut* cuts) {
    const int steps = K / BK;
    const int cols = end == END_SWIGLU ? N / 2 : N;
    double best = 1e30;
    int n_cuts = 1;
    for (int s = 0; s < N_SHAPES; ++s) {
        if (kShapes[s][1] == 3 && end != END_SLABS) continue;
        for (int parts = 1; parts <= (end == END_SLABS ? max_parts : 1) && parts <= steps; ++parts) {
            const double cost = cut_cost(M, cols, steps, end, s, parts);
            if (cost < best - 1e-9) {
                best = cost;
                cuts[0] = {kShapes[s][0], kShapes[s][1], parts, 0, cols};
            }
        }
    }
    if (end == END_SWIGLU && M >= 512) {
        // from 512 rows on the 8-wave tile is the faster one for this end, measured at 512, 1,024 and 2,048 rows of the 4B
        // shape (57 against 65 us, 115 against 114, 196 against 209); an element's sum does not depend on the tile
        return whole_rounds_then_rest(M, cols, end, 0, cuts);
    }
    if (end != END_SLABS) {
        // whole rounds of the largest tile first, the rest of the columns in smaller tiles
        const int tn = end == END_SWIGLU ? 128 : 256;
        const int tiles_m = (M + 255) / 256;
        const long long whole = ((long long)tiles_m * (cols / tn)) / 256 * 256;      // tiles of whole rounds
        const int first_cols = (int)(whole / tiles_m) * tn;
        if (first_cols > 0 && first_cols < cols) {
            for (int s = 2; s < N_SHAPES; ++s) {
                const double cost = cut_cost(M, first_cols, steps, end, 0, 1) + cut_cost(M, cols - first_cols, steps, end, s, 1);
                if (cost < best - 1e-9) {
                    best = cost;
                    n_cuts = 2;
                    cuts[0] = {4, 4, 1, 0, first_cols};
                    cuts[1] = {kShapes[s][0], kShapes[s][1], 1, first_cols, cols};
                }
            }
        }
    }
    return n_cuts;
}

template <int WM, int WN, int END, int WGN = 2>
static int launch_cut(const void* X, const void* W, void* Y, int M, int N, int K, const Cut& cut, hipStream_t stream) {
    constexpr int lds_bytes = Depth<WM, WN>::value * (64 * WM + 32 * WN * WGN) * BK * 2;
    static bool prepared = false;
    if (!prepared) {
        if (hipFuncSetAttribute((const void*)gemm_tiles_kernel<WM, WN, END, WGN>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                lds_bytes) != hipSuccess)
            return -6;
        prepared = true;
    }
    const int tm = 64 * WM, tn = (END == END_SWIGLU ? 16 : 32) * WN * WGN;
    const int tiles_m = (M + tm - 1) / tm, tiles_n = (cut.col_end - cut.col_begin + tn - 1) / tn;
    const int per_die = (tiles_m * tiles_n + 7) / 8;
    hipLaunchKernelGGL((gemm_tiles_kernel<WM, WN, END, WGN>), dim3(per_die * 8, 1, cut.parts), dim3(64 * 2 * WGN), lds_bytes, stream,
                       (const bf16_t*)X, (const bf16_t*)W, Y, M, N, K, tiles_m, tiles_n, cut.parts, N / 2, cut.col_begin,
                       cut.col_end);
    return KIPP_LAUNCH_CHECK();
}

template <int END>
static int launch_end(const void* X, const void* W, void* Y, int M, int N, int K, const Cut& cut, hipStream_t stream) {
    if (cut.wgn == 4) {
        // 8 waves, two a SIMD: the same workgroup tiles from wave tiles half as wide
        if (cut.wm == 4 && cut.wn == 2) return launch_cut<4, 2, END, 4>(X, W, Y, M, N, K, cut, stream);
        if (cut.wm == 2 && cut.wn == 2) return launch_cut<2, 2, END, 4>(X, W, Y, M, N, K, cut, stream);
        return -5;
    }
    if (cut.wm == 4 && cut.wn == 4) return launch_cut<4, 4, END>(X, W, Y, M, N, K, cut, stream);
    if (cut.wm == 4 && cut.wn == 2) return launch_cut<4, 2, END>(X, W, Y, M, N, K, cut, stream);
    if (cut.wm == 2 && cut.wn == 4) return launch_cut<2, 4, END>(X, W, Y, M, N, K, cut, stream);
    if (cut.wm == 2 && cut.wn == 2) return launch_cut<2, 2, END>(X, W, Y, M, N, K, cut, stream);
    if constexpr (END == END_SLABS) {
        if (cut.wm == 4 && cut.wn == 3) return launch_cut<4, 3, END>(X, W, Y, M, N, K, cut, stream);
        if (cut.wm == 2 && cut.wn == 3) return launch_cut<2, 3, END>(X, W, Y, M, N, K, cut, stream);
    }
    return -5;
}

extern "C" {
// parts that kipp_gemm_tiles cuts K into for these sizes when it may use up to `max_parts` (1 for the ends that are not slabs)
int kipp_gemm_tiles_parts(int M, int N, int K, int end, int max_parts) {
    if (K <= 0 || (K % BK) || M <= 0 || N <= 0) return -1;
    Cut cuts[2];
    plan(M, N, K, end, max_parts, cuts);
    return cuts[0].parts;
}

// Y: float32 [parts, M, N] with parts = kipp_gemm_tiles_parts(...) (end 0), bfloat16 [M, N / 2] = silu(gate) * up for
// W = [gate; up] (end 1), bfloat16 [M, N] (end 2).  K a multiple of 32.  `force`: 0, or 100 wm + 10 wn + parts (+ 1000: 8 waves, four across; + 2000: the same for whole rounds of tiles, the
// rest of the columns in smaller ones, which + 10000 r chooses) to take that cut whatever the plan says (the runtime's timed choice, tests).
int kipp_gemm_tiles(const void* X, const void* W, void* Y, int M, int N, int K, int end, int max_parts, int force,
                    hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0 || (K % BK) || max_parts <= 0) return -1;
    if (end != END_SLABS && end != END_SWIGLU && end != END_BF16) return -3;
    if (end == END_SWIGLU && (N & 1)) return -4;
    // a lane's offset into an operand is 32 bits wide
    if ((unsigned long long)M * K * 2 >= (1ull << 32) || (unsigned long long)N * K * 2 >= (1ull << 32)) return -6;
    Cut cuts[2];
    int n_cuts = plan(M, N, K, end, max_parts, cuts);
    if (force) {
        const int cols = end == END_SWIGLU ? N / 2 : N;
        n_cuts = 1;
        const int rest_code = force / 10000;         // + 10000 r: the tile of the columns that + 2000 leaves (below)
        force %= 10000;
        cuts[0] = {(force / 100) % 10, (force / 10) % 10, force % 10, 0, cols, force >= 1000 ? 4 : 2};
        if (force >= 2000 && end != END_SLABS) n_cuts = whole_rounds_then_rest(M, cols, end, rest_code, cuts);   // + 2000 (above)
    }
    for (int c = 0; c < n_cuts; ++c) {
        const Cut& cut = cuts[c];
        if (cut.parts < 1 || cut.parts > K / BK || (end != END_SLABS && cut.parts != 1)) return -2;
        const int rc = end == END_SLABS ? launch_end<END_SLABS>(X, W, Y, M, N, K, cut, stream)
                       : end == END_SWIGLU ? launch_end<END_SWIGLU>(X, W, Y, M, N, K, cut, stream)
                                           : launch_end<END_BF16>(X, W, Y, M, N, K, cut, stream);
        if (rc != 0) return rc;
    }
    return 0;
}

}  // extern "C"
