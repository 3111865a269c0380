// Sparse form of a population's linear layer: per-member weights = base ^ flips with few flips per row.
//
//   popcount(x ^ (b ^ f)) = popcount(x ^ b) + |f| - 2 * popcount(f & (x ^ b))
//
// so a member's row sum is the SHARED product popcount(x_d ^ b_r) (one base matrix for the whole population: a real
// matrix product with reuse, done on the matrix cores) plus a correction that only touches the member's flipped
// columns.  With flip probability p the correction reads 2 bytes per flip (16 p bits per weight bit) instead of the
// 1 bit per weight bit of the materialised weights: 12 % of the bytes at p = 0.01.  The result is the same integer.
//
// Flip lists ("sorted slices"): the rows of a member are ordered by flip count inside blocks of 1024 rows and cut into
// slices of 64 rows; a slice stores its rows' flips interleaved in 16-byte pieces: piece j of lane l = flips 8j ..
// 8j+7 of the slice's l-th row, padded with a sentinel to the slice's longest row.  A wave takes one slice: every
// load is one 1 KB run of 16 bytes per lane, no per-row offsets, no cross-lane reduction.  A flip is 16 bits:
//     [4:0]  bit inside a 32-bit piece of the input row        [15:5]  2 * (column / 32) + b
// where b is the BASE bit at that column: the kernel keeps the pieces of the member's input row interleaved with
// their complements in LDS (piece, ~piece, piece, ~piece ...: 4Kw dwords, then one zero dword for the sentinel 4Kw),
// so that the looked-up bit already is x ^ b.  The rows of a slice move through the columns at about the same pace,
// so at any moment the 64 lanes look into a narrow window of the table: neighbouring dwords, different banks.
#include <cmath>
#include <type_traits>

#include "nb_common.hpp"

namespace nb {

typedef int fl_v4i __attribute__((ext_vector_type(4)));
typedef int fl_v8i __attribute__((ext_vector_type(8)));
typedef float fl_v4f __attribute__((ext_vector_type(4)));

constexpr int kFlipMaxKw = 511;       // 4 * Kw must fit the 11-bit piece index
constexpr int kFlipBlockRows = 1024;  // rows are ordered inside blocks of this many (16 slices, one workgroup)

// ---- bits -> FP4 (E2M1) codes: bit 1 -> 0x2 (+1.0), bit 0 -> 0xA (-1.0); bit j of the byte -> nibble j ------------
__device__ __forceinline__ uint32_t fl_codes8(uint32_t b)
{
    uint32_t x = (b | (b << 12)) & 0x000F000Fu;
    x = (x | (x << 6)) & 0x03030303u;
    x = (x | (x << 3)) & 0x11111111u;
    return 0xAAAAAAAAu ^ (x << 3);
}

// in [rows, Kw] 64-bit words -> out [rows_p, 32 * Kw_p] bytes: 32 bits become 16 bytes; rows past `rows` and words
// past Kw become zero codes (0.0), which add nothing to a dot product.
__global__ __launch_bounds__(256) void fl_expand_kernel(uint4 *__restrict__ out, const uint32_t *__restrict__ in,
                                                        int64_t rows, int pieces, int64_t rows_p, int pieces_p)
{
    NB_FLAT_LOOP(t, rows_p * pieces_p)
    {
        if (t < rows_p * pieces_p) {
            const int64_t r = t / pieces_p;
            const int p = (int)(t - r * pieces_p);
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (r < rows && p < pieces) {
                const uint32_t b = in[r * pieces + p];
                v = make_uint4(fl_codes8(b & 255u), fl_codes8((b >> 8) & 255u), fl_codes8((b >> 16) & 255u),
                               fl_codes8(b >> 24));
            }
            out[t] = v;
        }
    }
}

// ---- shared product on the matrix cores ---------------------------------------------------------------------------
// C[m, n] = popcount(A_m ^ B_n) = (K - dot(+-1 codes)) / 2 with v_mfma_scale_f32_16x16x128_f8f6f4 on FP4 codes at
// unit scales (exact: +-1 and 0 are E2M1 values, the fp32 sums are integers below 2^24).  A workgroup of four waves
// owns a 128 x 128 tile (a wave 64 x 64 = 4 x 4 MFMA tiles: 8 KB of fragment reads per 16 products; eight waves of
// 64 x 32 measured slower, 37.6 against 31.4 us at 4096 x 1024 x 8192, the LDS traffic per product grows); a step
// stages 128 positions (64 bytes) of the tile's 128 + 128 rows in LDS (rows 80 bytes apart: the 16 rows of a fragment
// read land in different banks) while the previous step's fragments are multiplied; one barrier per step.  Fragment layout: lane l supplies row l % 16 and
// the 32 positions of 16-byte piece l / 16 (any assignment works as long as both operands use the same one);
// acc[r] is C[4 * (l / 16) + r][l % 16].
constexpr int kGemmTile = 128, kGemmStepBytes = 64, kGemmLd = kGemmStepBytes + 16;
constexpr int kGemmBufBytes = 2 * kGemmTile * kGemmLd;  // both operands of one step
constexpr int kGemmAhead = 4;                           // steps whose bytes are in flight, held in registers

__global__ __launch_bounds__(256) void fl_gemm_fp4_kernel(int32_t *__restrict__ C, const uint8_t *__restrict__ A,
                                                          const uint8_t *__restrict__ B, int64_t M, int64_t N,
                                                          int rowbytes, int kbits, int mtiles, int ntiles)
{
    constexpr int P = kGemmAhead;
    __shared__ __align__(16) uint8_t lds[2 * kGemmBufBytes];
    // workgroup b runs on XCD b % 8: give each XCD a contiguous run of tiles (neighbours share their A rows in L2)
    const int T = mtiles * ntiles, per = (T + 7) / 8;
    const int L = (int)(blockIdx.x % 8) * per + (int)(blockIdx.x / 8);
    if (L >= T) return;  // whole workgroup, before any barrier
    const int mt = L / ntiles, nt = L - mt * ntiles;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = tid >> 1, lhalf = tid & 1;  // staging: two threads per row, 32 bytes each
    const uint8_t *ga = A + ((int64_t)mt * kGemmTile + lrow) * rowbytes + lhalf * 32;
    const uint8_t *gb = B + ((int64_t)nt * kGemmTile + lrow) * rowbytes + lhalf * 32;
    const int st_off = lrow * kGemmLd + lhalf * 32;
    const int fa_off = (wm * 64 + (lane & 15)) * kGemmLd + (lane >> 4) * 16;
    const int fb_off = kGemmTile * kGemmLd + (wn * 64 + (lane & 15)) * kGemmLd + (lane >> 4) * 16;
    fl_v4f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = fl_v4f{0.f, 0.f, 0.f, 0.f};
    const int steps = rowbytes / kGemmStepBytes;
    // Register sets: a set holds the bytes of a step that is still to come.  Memory latency is several steps long and
    // a CU runs one workgroup, so four steps are kept in flight; a step past the end asks for the last one again (every
    // step issues the same loads, which keeps the wait counts exact).  The sets are separate named variables: indexing
    // an array of sets, even by a constant that only appears after inlining, sends them to scratch memory.
    static_assert(kGemmAhead == 4, "the step sequence below is written for four register sets");
    uint4 a0x, a0y, b0x, b0y, a1x, a1y, b1x, b1y, a2x, a2y, b2x, b2y, a3x, a3y, b3x, b3y;
#define NB_GEMM_REQUEST(ax, ay, bx, by, step)                                        \
    do {                                                                             \
        const int nx_ = ((step) < steps ? (step) : steps - 1) * kGemmStepBytes;      \
        ax = *reinterpret_cast<const uint4 *>(ga + nx_);                             \
        ay = *reinterpret_cast<const uint4 *>(ga + nx_ + 16);                        \
        bx = *reinterpret_cast<const uint4 *>(gb + nx_);                             \
        by = *reinterpret_cast<const uint4 *>(gb + nx_ + 16);                        \
    } while (0)
#define NB_GEMM_STAGE(ax, ay, bx, by, bufno)                                         \
    do {                                                                             \
        uint8_t *w_ = lds + (bufno) * kGemmBufBytes + st_off;                        \
        *reinterpret_cast<uint4 *>(w_) = ax;                                         \
        *reinterpret_cast<uint4 *>(w_ + 16) = ay;                                    \
        *reinterpret_cast<uint4 *>(w_ + kGemmTile * kGemmLd) = bx;                   \
        *reinterpret_cast<uint4 *>(w_ + kGemmTile * kGemmLd + 16) = by;              \
    } while (0)
    auto multiply = [&](int cur) {
        const uint8_t *buf = lds + (cur & 1) * kGemmBufBytes;
        fl_v4i fa[4], fb[4];
#pragma unroll
        for (int i = 0; i < 4; i++) fa[i] = *reinterpret_cast<const fl_v4i *>(buf + fa_off + i * 16 * kGemmLd);
#pragma unroll
        for (int j = 0; j < 4; j++) fb[j] = *reinterpret_cast<const fl_v4i *>(buf + fb_off + j * 16 * kGemmLd);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const fl_v8i a8 = __builtin_shufflevector(fa[i], fa[i], 0, 1, 2, 3, -1, -1, -1, -1);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const fl_v8i b8 = __builtin_shufflevector(fb[j], fb[j], 0, 1, 2, 3, -1, -1, -1, -1);
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, acc[i][j], 4, 4, 0, 0x7F7F7F7F, 0,
                                                                             0x7F7F7F7F);
            }
        }
    };
    // One step: the set that holds step cur + 1 goes to the buffer that step cur - 1 has left (every wave passed the
    // barrier that ended it) and is asked for step cur + 5; then the products of step cur; then the barrier.
#define NB_GEMM_STEP(ax, ay, bx, by, cur)                        \
    do {                                                         \
        NB_GEMM_STAGE(ax, ay, bx, by, ((cur) + 1) & 1);          \
        NB_GEMM_REQUEST(ax, ay, bx, by, (cur) + 1 + kGemmAhead); \
        __builtin_amdgcn_sched_barrier(0);                       \
        multiply(cur);                                           \
        __syncthreads();                                         \
    } while (0)
    NB_GEMM_REQUEST(a0x, a0y, b0x, b0y, 0);
    NB_GEMM_REQUEST(a1x, a1y, b1x, b1y, 1);
    NB_GEMM_REQUEST(a2x, a2y, b2x, b2y, 2);
    NB_GEMM_REQUEST(a3x, a3y, b3x, b3y, 3);
    NB_GEMM_STAGE(a0x, a0y, b0x, b0y, 0);
    NB_GEMM_REQUEST(a0x, a0y, b0x, b0y, 4);
    __syncthreads();
    int s = 0;
    for (; s + 4 <= steps; s += 4) {
        NB_GEMM_STEP(a1x, a1y, b1x, b1y, s);
        NB_GEMM_STEP(a2x, a2y, b2x, b2y, s + 1);
        NB_GEMM_STEP(a3x, a3y, b3x, b3y, s + 2);
        NB_GEMM_STEP(a0x, a0y, b0x, b0y, s + 3);
    }
    if (s < steps) NB_GEMM_STEP(a1x, a1y, b1x, b1y, s);  // uniform tails
    if (s + 1 < steps) NB_GEMM_STEP(a2x, a2y, b2x, b2y, s + 1);
    if (s + 2 < steps) NB_GEMM_STEP(a3x, a3y, b3x, b3y, s + 2);
#undef NB_GEMM_STEP
#undef NB_GEMM_STAGE
#undef NB_GEMM_REQUEST
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int64_t m = (int64_t)mt * kGemmTile + wm * 64 + i * 16 + 4 * (lane >> 4) + r;
                const int64_t n = (int64_t)nt * kGemmTile + wn * 64 + j * 16 + (lane & 15);
                if (m < M && n < N) C[m * N + n] = (kbits - (int)acc[i][j][r]) >> 1;
            }
}

// ---- flip counts: cnt[d, r] = popcount(W[d, r, :] ^ base[r, :]), sixteen lanes per row ---------------------------
__global__ __launch_bounds__(256) void fl_count_kernel(uint16_t *__restrict__ cnt, const uint64_t *__restrict__ W,
                                                       const uint64_t *__restrict__ base, int64_t rows, int64_t R,
                                                       int Kw)
{
    const int64_t gid = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 4;
    const int sub = threadIdx.x & 15;
    const bool live = gid < rows;
    const int64_t row = live ? gid : rows - 1;
    const int64_t r = row % R;
    const uint64_t *w = W + row * Kw, *b = base + r * Kw;
    int acc = 0;
    for (int k = sub; k < Kw; k += 16) acc += __popcll(__builtin_nontemporal_load(w + k) ^ b[k]);
    acc += __shfl_xor(acc, 8);
    acc += __shfl_xor(acc, 4);
    acc += __shfl_xor(acc, 2);
    acc += __shfl_xor(acc, 1);
    if (live && sub == 0) cnt[row] = (uint16_t)acc;
}

// ---- flip lists: one wave per slice, lane l walks the row perm[d, 64 s + l] ---------------------------------------
__global__ __launch_bounds__(256) void fl_fill_kernel(uint32_t *__restrict__ entries, const uint64_t *__restrict__ W,
                                                      const uint64_t *__restrict__ base,
                                                      const uint16_t *__restrict__ perm,
                                                      const int64_t *__restrict__ slice_off,
                                                      const int32_t *__restrict__ slice_len, int64_t nslices, int S,
                                                      int64_t R, int Kw)
{
    const int lane = threadIdx.x & 63;
    const int64_t sl = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (sl >= nslices) return;
    const int64_t d = sl / S;
    const int s = (int)(sl - d * S);
    const int64_t p = (int64_t)s * 64 + lane;
    const bool valid = p < R;
    int64_t r = valid ? perm[d * R + p] : 0;
    r = r < R ? r : R - 1;
    const int L = 4 * slice_len[sl];  // dwords per lane; dword j of lane l sits at piece j / 4, component j % 4
    uint4 *dst = reinterpret_cast<uint4 *>(entries + slice_off[sl]) + lane;
    const uint32_t sentinel = (uint32_t)(4 * Kw) << 5;
    int j = 0;
    uint32_t pend = 0;
    bool half = false;
    // a lane's dwords leave four at a time, as whole 16-byte pieces (L is a multiple of 4); never past the slice,
    // whatever the inputs
    uint32_t q0 = 0, q1 = 0, q2 = 0;
    auto put = [&](uint32_t v) {
        const int c = j & 3;
        if (c == 0) q0 = v;
        else if (c == 1) q1 = v;
        else if (c == 2) q2 = v;
        else if (j < L) dst[(int64_t)(j >> 2) * 64] = make_uint4(q0, q1, q2, v);
        j++;
    };
    if (valid) {
        const uint64_t *w = W + (d * R + r) * Kw, *b = base + r * Kw;
        for (int k = 0; k < Kw; k++) {
            const uint64_t bw = b[k];
            uint64_t m = w[k] ^ bw;
            while (m) {
                const int bit = __builtin_ctzll(m);
                m &= m - 1;
                const uint32_t col = (uint32_t)k * 64u + (uint32_t)bit;
                const uint32_t bb = (uint32_t)(bw >> bit) & 1u;
                const uint32_t e = ((2u * (col >> 5) + bb) << 5) | (col & 31u);
                if (!half) {
                    pend = e;
                    half = true;
                } else {
                    put(pend | (e << 16));
                    half = false;
                }
            }
        }
    }
    if (half) put(pend | (sentinel << 16));
    while (j < L) put(sentinel | (sentinel << 16));
}

// ---- skip sampler: flip lists straight from the generator, without ever drawing the bits that do not flip -----------
// For a uniform flip probability p the columns that flip in a row form a renewal process with geometric gaps.  Row q
// (flat over members and rows) reads the Philox words first + q*C + i, i = 0, 1, ...; word i has the rank
// #{k < Kt : cdf[k] <= word} (cdf[k-1] = floor(2^32 * (1 - (1-p)^k)), supplied by the caller; Kt == 0 means no
// flips): a rank below Kt moves the position on by rank + 1 columns and flips the column reached, rank Kt (a word
// beyond the table) moves it on by Kt columns without a flip; the row ends when the position passes C.  About
// C*p + 1 words per row instead of C: 100 times fewer at p = 0.01.  The same law as the per-bit compare (i.i.d. Bernoulli(p), quantised to
// 2^-32), not the same stream.
constexpr int kSkipMaxTable = 4096;

struct SkipChain {
    PhiloxKey key;
    uint64_t g;   // index of the next word
    uint4 blk;
    bool fresh;
    __device__ __forceinline__ SkipChain(const PhiloxKey &k, uint64_t start) : key(k), g(start), fresh(true) {}
    __device__ __forceinline__ uint32_t next()
    {
        if (fresh || (g & 3u) == 0) blk = philox_block(key, g >> 2);
        fresh = false;
        const uint32_t e = (uint32_t)g & 3u;
        g++;
        return e == 0 ? blk.x : e == 1 ? blk.y : e == 2 ? blk.z : blk.w;
    }
};

// Number of table entries <= u (the table is sorted).  The entries follow 2^32 * (1 - q^k), so
// log2(1 - u / 2^32) / log2(q) lands within a step or two of the answer; the walk from there is against the table
// itself, which keeps the result exact whatever the float arithmetic does (a wrong estimate only costs probes).
__device__ __forceinline__ int skip_rank(const uint32_t *tab, int Kt, uint32_t u, float inv_log2q)
{
    const float s = ((float)(~u) + 1.0f) * 2.3283064365386963e-10f;  // 1 - u / 2^32, from the complement: no cancellation
    int est = (int)(__log2f(s) * inv_log2q);
    est = est < 0 ? 0 : (est > Kt ? Kt : est);
    while (est < Kt && tab[est] <= u) est++;
    while (est > 0 && tab[est - 1] > u) est--;
    return est;
}

__global__ __launch_bounds__(256) void fl_skip_count_kernel(uint16_t *__restrict__ cnt, const uint32_t *__restrict__ cdf,
                                                            int Kt, float inv_log2q, PhiloxKey key, int64_t rows, int C)
{
    __shared__ uint32_t tab[kSkipMaxTable];
    for (int i = threadIdx.x; i < Kt; i += 256) tab[i] = cdf[i];
    __syncthreads();
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= rows) return;
    int n = 0;
    if (Kt > 0) {
        SkipChain chain(key, key.first + (uint64_t)q * (uint64_t)C);
        int pos = -1;
        for (;;) {
            const int rank = skip_rank(tab, Kt, chain.next(), inv_log2q);
            pos += rank < Kt ? rank + 1 : Kt;
            if (pos >= C) break;
            n += rank < Kt ? 1 : 0;
        }
    }
    cnt[q] = (uint16_t)n;
}

// ---- the same walk when every row starts on a block boundary of the stream (C and first multiples of 4) ------------
// All lanes then take word e of their current block at the same time, so a block's four words are four straight-line
// steps without a per-lane word select.  The table sits in LDS with one entry of padding on either side
// (tab1[k] = cdf[k - 1], tab1[0] = 0, tab1[Kt + 1] = 2^32 - 1): the float estimate is almost always the rank itself,
// and one two-entry read confirms it (tab1[est] <= u < tab1[est + 1]); a wave in which any lane fails that test walks
// the table as skip_rank does.  Same ranks, same words, same results as the kernels above.
__device__ __forceinline__ void skip_table_load(uint32_t *tab1, const uint32_t *cdf, int Kt)
{
    for (int i = threadIdx.x; i < Kt + 2; i += 256) tab1[i] = i == 0 ? 0u : (i <= Kt ? cdf[i - 1] : 0xFFFFFFFFu);
    __syncthreads();
}

// ranks of a block's four words: estimates and table reads first, one test for all four
__device__ __forceinline__ void skip_rank4(int (&rank)[4], const uint32_t *tab1, int Kt, const uint4 &w, float inv_log2q,
                                           float c0)
{
    const uint32_t u[4] = {w.x, w.y, w.z, w.w};
    uint32_t lo[4], hi[4];
    const float kt_f = (float)Kt;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        // log2((2^32 - 1 - u) / 2^32) / log2(q): never negative, +inf for u = 2^32 - 1; the missing 1 moves the
        // estimate for about two words in a million
        const int est = (int)fminf(fmaf(__log2f((float)(~u[e])), inv_log2q, c0), kt_f);
        rank[e] = est;
        lo[e] = tab1[est];
        hi[e] = tab1[est + 1];
    }
    uint32_t bad = 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) bad |= (uint32_t)(lo[e] > u[e]) | (uint32_t)(hi[e] <= u[e]);
    if (__any(bad != 0)) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            int est = rank[e];
            while (est < Kt && tab1[est + 1] <= u[e]) est++;
            while (est > 0 && tab1[est] > u[e]) est--;
            rank[e] = est;
        }
    }
}

// A lane counts rows q, q + T, q + 2T, ... (T = threads of the grid): lanes whose rows end early start their next
// one at the following block instead of idling until the longest row of the wave has ended.
__global__ __launch_bounds__(256) void fl_skip_count_aligned_kernel(uint16_t *__restrict__ cnt,
                                                                    const uint32_t *__restrict__ cdf, int Kt,
                                                                    float inv_log2q, PhiloxKey key, int64_t rows, int C)
{
    __shared__ uint32_t tab1[kSkipMaxTable + 2];
    skip_table_load(tab1, cdf, Kt);
    const int64_t T = (int64_t)gridDim.x * 256;
    int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const uint64_t row_blocks = (uint64_t)C >> 2;
    uint64_t row_blk = (key.first >> 2) + (uint64_t)q * row_blocks, blk = row_blk;
    const uint64_t blk_step = (uint64_t)T * row_blocks;
    const float c0 = -32.0f * inv_log2q;
    int pos = -1, n = 0;
    bool live = q < rows;
    while (__any(live)) {
        int rank[4];
        skip_rank4(rank, tab1, Kt, philox_block(key, blk++), inv_log2q, c0);
#pragma unroll
        for (int e = 0; e < 4; ++e) {   // past the row's end pos stays >= C and nothing more is counted
            pos += rank[e] < Kt ? rank[e] + 1 : Kt;
            n += (rank[e] < Kt && pos < C) ? 1 : 0;
        }
        if (pos >= C) {
            if (live) cnt[q] = (uint16_t)n;
            q += T;
            row_blk += blk_step;
            blk = row_blk;
            pos = -1;
            n = 0;
            live = q < rows;
        }
    }
}

// One lane's row, walked word by word (any C, any first): its entries into dwords lane, lane + 64, ... of the slice.
// A lane's dwords leave four at a time, as whole 16-byte pieces (L is a multiple of 4); never past the slice,
// whatever the inputs.  The walk writes its entries without the base bit; when a piece is complete, the base
// words of its (up to eight) columns are asked for together and the bits put in before the piece is stored: one
// wait for memory per piece instead of one per flip (a wait for a load also waits for the stores before it).
__device__ __forceinline__ void skip_fill_row(uint4 *__restrict__ dst, int L, const uint64_t *__restrict__ b, int Kw,
                                              const uint32_t *tab, int Kt, float inv_log2q, const PhiloxKey &key,
                                              uint64_t start, bool valid, int C)
{
    const uint32_t sentinel = (uint32_t)(4 * Kw) << 5;
    const uint32_t npieces = (uint32_t)(4 * Kw);
    int j = 0;
    uint32_t pend = 0;
    bool half = false;
    uint32_t q0 = 0, q1 = 0, q2 = 0;
    auto base_bit = [&](uint32_t e) -> uint32_t {  // e: one 16-bit entry; 0 for a sentinel
        const uint32_t piece = e >> 5;
        const uint32_t col = (piece >> 1) * 32u + (e & 31u);
        const uint32_t live = piece < npieces;
        const uint64_t word = live ? b[col >> 6] : 0ull;  // nothing is read for a sentinel
        return (uint32_t)(word >> (col & 63u)) & 1u;
    };
    auto patched = [&](uint32_t v) { return v | (base_bit(v & 0xFFFFu) << 5) | (base_bit(v >> 16) << 21); };
    auto put = [&](uint32_t v) {
        const int c = j & 3;
        if (c == 0) q0 = v;
        else if (c == 1) q1 = v;
        else if (c == 2) q2 = v;
        else if (j < L) {
            const uint32_t p0 = patched(q0), p1 = patched(q1), p2 = patched(q2), p3 = patched(v);
            dst[(int64_t)(j >> 2) * 64] = make_uint4(p0, p1, p2, p3);
        }
        j++;
    };
    if (valid && Kt > 0) {
        SkipChain chain(key, start);
        int pos = -1;
        for (;;) {
            const int rank = skip_rank(tab, Kt, chain.next(), inv_log2q);
            pos += rank < Kt ? rank + 1 : Kt;
            if (pos >= C) break;
            if (rank >= Kt) continue;  // a word beyond the table: moved on, no flip
            const uint32_t col = (uint32_t)pos;
            const uint32_t e = ((2u * (col >> 5)) << 5) | (col & 31u);  // base bit still to come
            if (!half) {
                pend = e;
                half = true;
            } else {
                put(pend | (e << 16));
                half = false;
            }
        }
    }
    if (half) put(pend | (sentinel << 16));
    while (j < L) put(sentinel | (sentinel << 16));
}

__global__ __launch_bounds__(256) void fl_skip_fill_kernel(uint32_t *__restrict__ entries,
                                                           const uint64_t *__restrict__ base,
                                                           const uint16_t *__restrict__ perm,
                                                           const int64_t *__restrict__ slice_off,
                                                           const int32_t *__restrict__ slice_len,
                                                           const uint32_t *__restrict__ cdf, int Kt, float inv_log2q,
                                                           PhiloxKey key, int64_t nslices, int S, int64_t R, int Kw,
                                                           int C)
{
    __shared__ uint32_t tab[kSkipMaxTable];
    for (int i = threadIdx.x; i < Kt; i += 256) tab[i] = cdf[i];
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const int64_t sl = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (sl >= nslices) return;
    const int64_t d = sl / S;
    const int s = (int)(sl - d * S);
    const int64_t p = (int64_t)s * 64 + lane;
    const bool valid = p < R;
    int64_t r = valid ? perm[d * R + p] : 0;
    r = r < R ? r : R - 1;
    uint4 *dst = reinterpret_cast<uint4 *>(entries + slice_off[sl]) + lane;
    skip_fill_row(dst, 4 * slice_len[sl], base + r * Kw, Kw, tab, Kt, inv_log2q, key,
                  key.first + (uint64_t)(d * R + r) * (uint64_t)C, valid, C);
}

// Rows on block boundaries of the stream (C and first multiples of 4, a table with entries): the lanes of a slice
// walk in step, eight words (two blocks) to a 16-byte piece.  As long as every word of a live row yields a flip, word
// i of a row is its flip i, so the piece a wave is on is the same for all its lanes and nothing about the entry's
// place is per lane; a row that has ended gives sentinels.  A word beyond the table (no flip) in any live row breaks
// that: the wave then starts its slice again, row by row as above (with a table that runs to saturation this takes a
// word of 2^32 - 1).
__global__ __launch_bounds__(256) void fl_skip_fill_aligned_kernel(uint32_t *__restrict__ entries,
                                                                   const uint64_t *__restrict__ base,
                                                                   const uint16_t *__restrict__ perm,
                                                                   const int64_t *__restrict__ slice_off,
                                                                   const int32_t *__restrict__ slice_len,
                                                                   const uint32_t *__restrict__ cdf, int Kt,
                                                                   float inv_log2q, PhiloxKey key, int64_t nslices,
                                                                   int S, int64_t R, int Kw, int C)
{
    __shared__ uint32_t tab1[kSkipMaxTable + 2];
    skip_table_load(tab1, cdf, Kt);
    const int lane = threadIdx.x & 63;
    const int64_t sl = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (sl >= nslices) return;
    const int64_t d = sl / S;
    const int s = (int)(sl - d * S);
    const int64_t p = (int64_t)s * 64 + lane;
    const bool valid = p < R;
    int64_t r = valid ? perm[d * R + p] : 0;
    r = r < R ? r : R - 1;
    const int P = slice_len[sl];
    uint4 *dst = reinterpret_cast<uint4 *>(entries + slice_off[sl]) + lane;
    const uint32_t *b32 = reinterpret_cast<const uint32_t *>(base + r * Kw);
    const uint32_t sentinel = (uint32_t)(4 * Kw) << 5;
    const float c0 = -32.0f * inv_log2q;
    uint64_t blk = (key.first >> 2) + (uint64_t)(d * R + r) * ((uint64_t)C >> 2);
    int pos = valid ? -1 : C;
    bool irregular = false;
    uint4 cur = make_uint4(0u, 0u, 0u, 0u);   // the row's window that the last entry lay in, and its first dword
    uint32_t curwin = 0xFFFFFFFFu;
    const uint32_t last_start = (uint32_t)(2 * Kw - 4);
    int piece = 0;
    for (; piece < P; ++piece) {
        uint32_t e[8];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            int rank4[4];
            skip_rank4(rank4, tab1, Kt, philox_block(key, blk++), inv_log2q, c0);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int rank = rank4[k];
                irregular |= rank >= Kt && pos < C;
                pos += rank < Kt ? rank + 1 : Kt;
                const uint32_t col = (uint32_t)pos;
                e[4 * h + k] = pos < C ? (((col >> 5) << 6) | (col & 31u)) : sentinel;
            }
        }
        if (__any(irregular)) break;
        // Base bits from 16-byte windows of the row (128 columns; the last one ends with the row): a window is asked
        // for only where an entry leaves the one before it, since what the look-ups cost is the number of lanes that
        // ask, not the bytes.  Four entries' windows are asked for together; nothing is read for a sentinel.
#pragma unroll
        for (int h = 0; h < 8; h += 4) {
            uint32_t st[4];
            bool need[4];
            uint4 w[4];
            uint32_t prev = curwin;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const uint32_t dw = e[h + k] >> 6, a = dw & ~3u;
                st[k] = a < last_start ? a : last_start;
                const bool live = e[h + k] != sentinel;
                need[k] = live && st[k] != prev;
                prev = live ? st[k] : prev;
            }
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (need[k]) __builtin_memcpy(&w[k], b32 + st[k], 16);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                if (need[k]) {
                    cur = w[k];
                    curwin = st[k];
                }
                const uint32_t d = (e[h + k] >> 6) - curwin;
                const uint32_t word = d == 0 ? cur.x : d == 1 ? cur.y : d == 2 ? cur.z : cur.w;
                const uint32_t bit = e[h + k] != sentinel ? (word >> (e[h + k] & 31u)) & 1u : 0u;
                e[h + k] |= bit << 5;
            }
        }
        dst[(int64_t)piece * 64] = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16),
                                              e[6] | (e[7] << 16));
    }
    if (piece < P)
        skip_fill_row(dst, 4 * P, base + r * Kw, Kw, tab1 + 1, Kt, inv_log2q, key,
                      key.first + (uint64_t)(d * R + r) * (uint64_t)C, valid, C);
}

// v of lane (lane ^ j), j a power of two below 64: quad permutes, swizzles inside 32 lanes, a general exchange for 32
__device__ __forceinline__ uint32_t xor_lane(uint32_t v, int j)
{
    switch (j) {
    case 1: return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);   // quad_perm [1, 0, 3, 2]
    case 2: return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xF, 0xF, true);   // quad_perm [2, 3, 0, 1]
    case 4: return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, (4 << 10) | 0x1F);    // bit mode: and 31, xor j
    case 8: return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, (8 << 10) | 0x1F);
    case 16: return (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, (16 << 10) | 0x1F);
    default: return (uint32_t)__shfl_xor((int)v, j);
    }
}

// Row order and slice lengths from the counts: workgroup (d, block of 1024 rows) sorts its rows by (count, row) with a
// bitonic network, a key per thread, partners inside a wave by lane exchange and others through LDS (keys
// count << 10 | row-in-block are distinct, so the order is the stable one; rows past R
// sort last) and writes perm and, from the last row of every run of 64, the slice's pieces per lane.
__global__ __launch_bounds__(1024) void fl_layout_kernel(uint16_t *__restrict__ perm, int32_t *__restrict__ slice_len,
                                                         const uint16_t *__restrict__ cnt, int64_t R, int nblk, int S)
{
    __shared__ uint32_t key[1024];
    const int t = threadIdx.x;
    const int64_t d = blockIdx.x / nblk;
    const int blk = (int)(blockIdx.x - d * nblk);
    const int64_t r0 = (int64_t)blk * 1024;
    const int valid = (int)(R - r0 < 1024 ? R - r0 : 1024);
    uint32_t v = t < valid ? ((uint32_t)cnt[d * R + r0 + t] << 10) | (uint32_t)t : 0xFFFFFC00u | (uint32_t)t;
#pragma unroll
    for (int k = 2; k <= 1024; k <<= 1) {
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1) {
            uint32_t o;
            if (j >= 64) {  // the partner sits in another wave: through LDS
                __syncthreads();
                key[t] = v;
                __syncthreads();
                o = key[t ^ j];
            } else {
                o = xor_lane(v, j);
            }
            const bool keep_min = ((t & j) == 0) == ((t & k) == 0);
            v = keep_min ? (v < o ? v : o) : (v > o ? v : o);
        }
    }
    if (t < valid) {
        perm[d * R + r0 + t] = (uint16_t)(r0 + (v & 1023u));
        if ((t & 63) == 63 || t == valid - 1) slice_len[d * S + (r0 + t) / 64] = (int32_t)(((v >> 10) + 7) >> 3);
    }
}

// slice_off = running sum of slice_len * 256 dwords (exclusive), total[0] = the sum.  Workgroup b owns slices
// 8192 b .. 8192 b + 8191, eight per thread, and first adds up everything before them itself.
__device__ __forceinline__ int64_t block_sum_1024(int64_t v, int64_t *wave_sum, int64_t *incl_out)
{
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    int64_t incl = v;  // inclusive sum over the wave's lanes
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int64_t up = __shfl_up(incl, o);
        if (lane >= o) incl += up;
    }
    __syncthreads();
    if (lane == 63) wave_sum[wv] = incl;
    __syncthreads();
    int64_t before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
        before += w < wv ? wave_sum[w] : 0;
        all += wave_sum[w];
    }
    *incl_out = before + incl;
    return all;
}

__global__ __launch_bounds__(1024) void fl_offsets_kernel(int64_t *__restrict__ slice_off, int64_t *__restrict__ total,
                                                          const int32_t *__restrict__ slice_len, int64_t n)
{
    __shared__ int64_t wave_sum[16];
    const int t = threadIdx.x;
    const int64_t tile = (int64_t)blockIdx.x * 8192;
    int64_t head = 0, unused;
    const int4 *len4 = reinterpret_cast<const int4 *>(slice_len);  // a tile is 2048 of these
#pragma unroll 4
    for (int64_t i = t; i < tile / 4; i += 1024) {
        const int4 q = len4[i];
        head += (int64_t)q.x + q.y + q.z + q.w;
    }
    const int64_t carry = block_sum_1024(head, wave_sum, &unused) * 256;
    const int64_t i0 = tile + (int64_t)t * 8;
    int64_t v[8], mine = 0, incl;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        v[k] = i0 + k < n ? (int64_t)slice_len[i0 + k] * 256 : 0;
        mine += v[k];
    }
    const int64_t all = block_sum_1024(mine, wave_sum, &incl);
    int64_t run = carry + incl - mine;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        if (i0 + k < n) slice_off[i0 + k] = run;
        run += v[k];
    }
    if (t == 0 && blockIdx.x == gridDim.x - 1) total[0] = carry + all;
}

// whether every row of the walk starts on a block boundary of the stream (and there is a table to look up)
static inline bool skip_rows_aligned(int64_t C, uint64_t first, int64_t Kt) { return Kt > 0 && C % 4 == 0 && first % 4 == 0; }
// the aligned fill reads the base in 16-byte windows: rows of at least two words
static inline bool skip_fill_aligned(int64_t C, uint64_t first, int64_t Kt) { return skip_rows_aligned(C, first, Kt) && C > 64; }

// Flip lists -> materialised weights: W must hold the base in every member on entry; every flip is XOR-ed in.  A
// lane owns its row, so plain read-modify-writes suffice (flips come in column order: one write per touched word).
__global__ __launch_bounds__(256) void fl_to_dense_kernel(uint64_t *__restrict__ W, const uint32_t *__restrict__ entries,
                                                          const int64_t *__restrict__ slice_off,
                                                          const int32_t *__restrict__ slice_len,
                                                          const uint16_t *__restrict__ perm, int64_t nslices, int S,
                                                          int64_t R, int Kw)
{
    const int lane = threadIdx.x & 63;
    const int64_t sl = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (sl >= nslices) return;
    const int64_t d = sl / S;
    const int s = (int)(sl - d * S);
    const int64_t p = (int64_t)s * 64 + lane;
    if (p >= R) return;
    int64_t r = perm[d * R + p];
    r = r < R ? r : R - 1;
    uint64_t *row = W + (d * R + r) * Kw;
    const uint32_t *src = entries + slice_off[sl] + lane * 4;
    const int L = 4 * slice_len[sl];
    int curw = -1;
    uint64_t mask = 0;
    for (int j = 0; j < L; j++) {
        const uint32_t pair = src[(int64_t)(j >> 2) * 256 + (j & 3)];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t e = h ? pair >> 16 : pair & 0xFFFFu;
            const uint32_t piece = e >> 5;
            if (piece >= (uint32_t)(4 * Kw)) continue;  // sentinel
            const uint32_t col = (piece >> 1) * 32u + (e & 31u);
            const int w = (int)(col >> 6);
            if (w != curw) {
                if (curw >= 0) row[curw] ^= mask;
                curw = w;
                mask = 0;
            }
            mask |= (uint64_t)1 << (col & 63u);
        }
    }
    if (curw >= 0) row[curw] ^= mask;
}

// ---- the members' corrections, threshold and pack --------------------------------------------------------------------
// One workgroup per (member, block of 1024 rows), one wave per slice.  PACK: out = bits (2 * sum > thresh) of the
// block's rows, OR-ed into an LDS bit array (the rows of a slice are scattered over the block) and written as 32-bit
// pieces; else out = the int32 sums.
template <bool PACK>
__global__ __launch_bounds__(1024) void fl_bmv_kernel(void *__restrict__ out, const int32_t *__restrict__ G,
                                                      const uint32_t *__restrict__ entries,
                                                      const int64_t *__restrict__ slice_off,
                                                      const int32_t *__restrict__ slice_len,
                                                      const uint16_t *__restrict__ perm,
                                                      const uint16_t *__restrict__ cnt, const uint32_t *__restrict__ x32,
                                                      const int32_t *__restrict__ thresh, int64_t R, int S, int Kw,
                                                      int blocks_per_member)
{
    // x and ~x interleaved, one zero dword (the sentinel's entry: 4 * Kw), then the block's bit array.  A static
    // array: its address is then known when the look-ups are compiled and needs no add per look-up.
    __shared__ uint32_t fl_tab[4 * kFlipMaxKw + 1 + 32];
    constexpr int U = 4;                  // 16-byte pieces of a lane's list requested together
    const int64_t d = blockIdx.x / blocks_per_member;
    const int blk = (int)(blockIdx.x - d * blocks_per_member);
    const int nd = 2 * Kw;
    const int lane = threadIdx.x & 63;
    // the slice is uniform over the wave, and visibly so: the tests on the slice's length below are scalar branches
    const int s = blk * (kFlipBlockRows / 64) + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const bool active = s < S;
    const int64_t sl = d * S + (active ? s : S - 1);
    const int L = active ? __builtin_amdgcn_readfirstlane(slice_len[sl]) : 0;
    const uint4 *src = reinterpret_cast<const uint4 *>(entries + slice_off[sl]) + lane;
    // Two register sets take turns: while one batch is looked up, the batch after it is in flight.  Only pieces
    // that exist are requested (L is wave-uniform, so every such test is a scalar branch).  The first two batches
    // are requested before anything else: they do not depend on the table.
    uint4 e0[U], e1[U];
    auto request = [&](uint4(&e)[U], int j) {
#pragma unroll
        for (int u = 0; u < U; u++)
            if (j + u < L) e[u] = load_stream16(src + (int64_t)(j + u) * 64);
    };
    request(e0, 0);
    request(e1, U);
    for (int i = threadIdx.x; i < nd; i += blockDim.x) {
        const uint32_t v = x32[d * nd + i];
        fl_tab[2 * i] = v;
        fl_tab[2 * i + 1] = ~v;
    }
    uint32_t *bitmap = fl_tab + 2 * nd + 1;
    if (threadIdx.x == 0) fl_tab[2 * nd] = 0u;
    if (threadIdx.x < 32) bitmap[threadIdx.x] = 0u;
    const int64_t p = (int64_t)s * 64 + lane;
    const bool valid = active && p < R;
    int64_t r = perm[d * R + (valid ? p : R - 1)];
    r = r < R ? r : R - 1;
    const int n = cnt[d * R + r];
    const int g = G[d * R + r];
    const int t = PACK ? thresh[d * R + r] : 0;
    __syncthreads();
    int sy = 0;
    auto take = [&](uint32_t e) {
        const uint32_t w0 = fl_tab[(e >> 5) & 0x7FFu];
        const uint32_t w1 = fl_tab[e >> 21];
        sy += (int)((w0 >> (e & 31u)) & 1u) + (int)((w1 >> ((e >> 16) & 31u)) & 1u);
    };
    auto look_up = [&](const uint4(&e)[U], int j) {
#pragma unroll
        for (int u = 0; u < U; u++)
            if (j + u < L) {
                take(e[u].x);
                take(e[u].y);
                take(e[u].z);
                take(e[u].w);
            }
    };
    for (int j = 0; j < L; j += 2 * U) {
        look_up(e0, j);
        request(e0, j + 2 * U);
        look_up(e1, j + U);
        request(e1, j + 3 * U);
    }
    if (active) {
        const int sum = g + n - 2 * sy;
        if (PACK) {
            const int local = (int)(r - (int64_t)blk * kFlipBlockRows);
            if (valid && 2 * sum > t) atomicOr(&bitmap[(local >> 5) & 31], 1u << (local & 31));
        } else if (valid) {
            static_cast<int32_t *>(out)[d * R + r] = sum;
        }
    }
    if (PACK) {
        __syncthreads();
        const int pieces = 2 * (int)((R + 63) / 64);  // 32-bit pieces of a member's output row
        const int q = blk * 32 + (int)threadIdx.x;
        if (threadIdx.x < 32 && q < pieces) static_cast<uint32_t *>(out)[d * pieces + q] = bitmap[threadIdx.x];
    }
}

static int flip_shape_check(int64_t D, int64_t R, int64_t Kw, const char *who)
{
    NB_REQUIRE(D >= 0 && R >= 0 && Kw >= 0, "%s: negative shape D=%lld R=%lld Kw=%lld", who, (long long)D, (long long)R,
               (long long)Kw);
    NB_REQUIRE(Kw <= kFlipMaxKw, "%s: rows of %lld words, at most %d", who, (long long)Kw, kFlipMaxKw);
    NB_REQUIRE(R <= 65536, "%s: %lld rows per member, at most 65536", who, (long long)R);
    NB_REQUIRE(D * ((R + 63) / 64) <= (1LL << 31) && D * R < (1LL << 40), "%s: too many rows", who);
    return NB_OK;
}

}  // namespace nb

extern "C" {
int nb_expand_fp4_i64(uint8_t *out, const int64_t *in, int64_t rows, int64_t Kw, int64_t rows_padded, int64_t Kw_padded,
                      nb_stream_t stream)
{
    const char *who = "nb_expand_fp4_i64";
    NB_REQUIRE(rows >= 0 && Kw >= 0 && rows_padded >= rows && Kw_padded >= Kw, "%s: bad shape", who);
    NB_REQUIRE(Kw_padded < (1 << 20) && rows_padded < (1LL << 40), "%s: too large", who);
    if (rows_padded * Kw_padded == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_ALIGNED(out, 16);
    if (rows * Kw > 0) {
        NB_REQUIRE_PTR(in);
        NB_REQUIRE_ALIGNED(in, 8);
    }
    nb::fl_expand_kernel<<<dim3(nb::grid_for(rows_padded * Kw_padded * 2)), dim3(256), 0, nb::as_stream(stream)>>>(
        reinterpret_cast<uint4 *>(out), reinterpret_cast<const uint32_t *>(in), rows, (int)(2 * Kw), rows_padded,
        (int)(2 * Kw_padded));
    return nb::check_launch(who);
}

int nb_bmm_nt_fp4(int32_t *C, const uint8_t *A, const uint8_t *B, int64_t M, int64_t N, int64_t Kw, int64_t M_padded,
                  int64_t N_padded, int64_t Kw_padded, nb_stream_t stream)
{
    const char *who = "nb_bmm_nt_fp4";
    NB_REQUIRE(M >= 0 && N >= 0 && Kw >= 0 && Kw_padded >= Kw, "%s: bad shape", who);
    if (M * N == 0) return NB_OK;
    NB_REQUIRE(M_padded >= nb::ceil_div(M, nb::kGemmTile) * nb::kGemmTile &&
                   N_padded >= nb::ceil_div(N, nb::kGemmTile) * nb::kGemmTile,
               "%s: operands must be padded to whole tiles of %d rows (M_padded=%lld, N_padded=%lld)", who,
               nb::kGemmTile, (long long)M_padded, (long long)N_padded);
    NB_REQUIRE(Kw_padded >= 2 && Kw_padded % 2 == 0, "%s: padded row of %lld words, a positive even count needed", who,
               (long long)Kw_padded);
    NB_REQUIRE(Kw_padded * 64 < (1 << 24), "%s: rows too long for exact fp32 sums", who);
    NB_REQUIRE_PTR(C);
    NB_REQUIRE_PTR(A);
    NB_REQUIRE_PTR(B);
    NB_REQUIRE_ALIGNED(C, 4);
    NB_REQUIRE_ALIGNED(A, 16);
    NB_REQUIRE_ALIGNED(B, 16);
    const int64_t mt = nb::ceil_div(M, nb::kGemmTile), nt = nb::ceil_div(N, nb::kGemmTile);
    NB_REQUIRE(mt * nt < (1 << 24), "%s: too many tiles", who);
    const int64_t grid = nb::ceil_div(mt * nt, 8) * 8;
    nb::fl_gemm_fp4_kernel<<<dim3((unsigned)grid), dim3(256), 0, nb::as_stream(stream)>>>(
        C, A, B, M, N, (int)(Kw_padded * 32), (int)(Kw * 64), (int)mt, (int)nt);
    return nb::check_launch(who);
}

int nb_flip_count_i64(uint16_t *cnt, const int64_t *W, const int64_t *base, int64_t D, int64_t R, int64_t Kw,
                      nb_stream_t stream)
{
    const char *who = "nb_flip_count_i64";
    if (int rc = nb::flip_shape_check(D, R, Kw, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_PTR(cnt);
    NB_REQUIRE_ALIGNED(cnt, 2);
    if (Kw > 0) {
        NB_REQUIRE_PTR(W);
        NB_REQUIRE_PTR(base);
        NB_REQUIRE_ALIGNED(W, 8);
        NB_REQUIRE_ALIGNED(base, 8);
    }
    const int64_t blocks = nb::ceil_div(D * R * 16, 256);
    NB_REQUIRE(blocks <= nb::kMaxGridX, "%s: too many rows for one launch", who);
    nb::fl_count_kernel<<<dim3((unsigned)blocks), dim3(256), 0, nb::as_stream(stream)>>>(
        cnt, reinterpret_cast<const uint64_t *>(W), reinterpret_cast<const uint64_t *>(base), D * R, R, (int)Kw);
    return nb::check_launch(who);
}

int nb_flip_fill_i64(uint32_t *entries, const int64_t *W, const int64_t *base, const uint16_t *perm,
                     const int64_t *slice_off, const int32_t *slice_len, int64_t D, int64_t R, int64_t Kw,
                     nb_stream_t stream)
{
    const char *who = "nb_flip_fill_i64";
    if (int rc = nb::flip_shape_check(D, R, Kw, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_PTR(entries);
    NB_REQUIRE_PTR(perm);
    NB_REQUIRE_PTR(slice_off);
    NB_REQUIRE_PTR(slice_len);
    NB_REQUIRE_ALIGNED(entries, 16);
    NB_REQUIRE_ALIGNED(perm, 2);
    NB_REQUIRE_ALIGNED(slice_off, 8);
    NB_REQUIRE_ALIGNED(slice_len, 4);
    if (Kw > 0) {
        NB_REQUIRE_PTR(W);
        NB_REQUIRE_PTR(base);
        NB_REQUIRE_ALIGNED(W, 8);
        NB_REQUIRE_ALIGNED(base, 8);
    }
    const int64_t S = (R + 63) / 64;
    nb::fl_fill_kernel<<<dim3((unsigned)nb::ceil_div(D * S, 4)), dim3(256), 0, nb::as_stream(stream)>>>(
        entries, reinterpret_cast<const uint64_t *>(W), reinterpret_cast<const uint64_t *>(base), perm, slice_off,
        slice_len, D * S, (int)S, R, (int)Kw);
    return nb::check_launch(who);
}

// 1 / log2(1 - p) for the table's first entry p * 2^32: only a hint for where a look-up starts probing
static float skip_hint(uint32_t cdf0)
{
    const double p = (double)cdf0 / 4294967296.0;
    if (p <= 0.0 || p >= 1.0) return 0.0f;
    return (float)(1.0 / std::log2(1.0 - p));
}

int nb_flip_skip_count_i64(uint16_t *cnt, const uint32_t *cdf, uint32_t cdf0, int64_t Kt, uint64_t seed, uint64_t subseq,
                           uint64_t first, int64_t D, int64_t R, int64_t C, nb_stream_t stream)
{
    const char *who = "nb_flip_skip_count_i64";
    const float inv_log2q = skip_hint(cdf0);
    NB_REQUIRE(C >= 0 && Kt >= 0 && Kt <= nb::kSkipMaxTable, "%s: bad C=%lld or table of %lld entries (at most %d)", who,
               (long long)C, (long long)Kt, nb::kSkipMaxTable);
    if (int rc = nb::flip_shape_check(D, R, (C + 63) / 64, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_PTR(cnt);
    NB_REQUIRE_ALIGNED(cnt, 2);
    if (Kt > 0) NB_REQUIRE_PTR(cdf);
    NB_REQUIRE_ALIGNED(cdf, 4);
    const int64_t blocks = nb::ceil_div(D * R, 256);
    NB_REQUIRE(blocks <= nb::kMaxGridX, "%s: too many rows for one launch", who);
    if (nb::skip_rows_aligned(C, first, Kt)) {
        // beyond 2048 workgroups (eight per compute unit) a lane takes several rows, up to eight
        const int64_t grid = blocks <= 2048 ? blocks : std::max<int64_t>(2048, nb::ceil_div(blocks, 8));
        nb::fl_skip_count_aligned_kernel<<<dim3((unsigned)grid), dim3(256), 0, nb::as_stream(stream)>>>(
            cnt, cdf, (int)Kt, inv_log2q, nb::PhiloxKey{seed, subseq, first}, D * R, (int)C);
    } else {
        nb::fl_skip_count_kernel<<<dim3((unsigned)blocks), dim3(256), 0, nb::as_stream(stream)>>>(
            cnt, cdf, (int)Kt, inv_log2q, nb::PhiloxKey{seed, subseq, first}, D * R, (int)C);
    }
    return nb::check_launch(who);
}

int nb_flip_skip_fill_i64(uint32_t *entries, const int64_t *base, const uint16_t *perm, const int64_t *slice_off,
                          const int32_t *slice_len, const uint32_t *cdf, uint32_t cdf0, int64_t Kt, uint64_t seed,
                          uint64_t subseq, uint64_t first, int64_t D, int64_t R, int64_t C, nb_stream_t stream)
{
    const char *who = "nb_flip_skip_fill_i64";
    const float inv_log2q = skip_hint(cdf0);
    NB_REQUIRE(C >= 0 && Kt >= 0 && Kt <= nb::kSkipMaxTable, "%s: bad C=%lld or table of %lld entries (at most %d)", who,
               (long long)C, (long long)Kt, nb::kSkipMaxTable);
    const int64_t Kw = (C + 63) / 64;
    if (int rc = nb::flip_shape_check(D, R, Kw, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_PTR(entries);
    NB_REQUIRE_PTR(perm);
    NB_REQUIRE_PTR(slice_off);
    NB_REQUIRE_PTR(slice_len);
    NB_REQUIRE_ALIGNED(entries, 16);
    NB_REQUIRE_ALIGNED(perm, 2);
    NB_REQUIRE_ALIGNED(slice_off, 8);
    NB_REQUIRE_ALIGNED(slice_len, 4);
    if (Kt > 0) NB_REQUIRE_PTR(cdf);
    NB_REQUIRE_ALIGNED(cdf, 4);
    if (Kw > 0) NB_REQUIRE_PTR(base);
    NB_REQUIRE_ALIGNED(base, 8);
    const int64_t S = (R + 63) / 64;
    const dim3 grid((unsigned)nb::ceil_div(D * S, 4));
    if (nb::skip_fill_aligned(C, first, Kt))
        nb::fl_skip_fill_aligned_kernel<<<grid, dim3(256), 0, nb::as_stream(stream)>>>(
            entries, reinterpret_cast<const uint64_t *>(base), perm, slice_off, slice_len, cdf, (int)Kt, inv_log2q,
            nb::PhiloxKey{seed, subseq, first}, D * S, (int)S, R, (int)Kw, (int)C);
    else
        nb::fl_skip_fill_kernel<<<grid, dim3(256), 0, nb::as_stream(stream)>>>(
            entries, reinterpret_cast<const uint64_t *>(base), perm, slice_off, slice_len, cdf, (int)Kt, inv_log2q,
            nb::PhiloxKey{seed, subseq, first}, D * S, (int)S, R, (int)Kw, (int)C);
    return nb::check_launch(who);
}

int nb_flip_layout(uint16_t *perm, int32_t *slice_len, int64_t *slice_off, int64_t *total, const uint16_t *cnt, int64_t D,
                   int64_t R, nb_stream_t stream)
{
    const char *who = "nb_flip_layout";
    if (int rc = nb::flip_shape_check(D, R, 0, who)) return rc;
    NB_REQUIRE_PTR(total);
    NB_REQUIRE_ALIGNED(total, 8);
    const int64_t S = (R + 63) / 64;
    if (D * R > 0) {
        NB_REQUIRE_PTR(perm);
        NB_REQUIRE_PTR(slice_len);
        NB_REQUIRE_PTR(slice_off);
        NB_REQUIRE_PTR(cnt);
        NB_REQUIRE_ALIGNED(perm, 2);
        NB_REQUIRE_ALIGNED(slice_len, 16);
        NB_REQUIRE_ALIGNED(slice_off, 8);
        NB_REQUIRE_ALIGNED(cnt, 2);
        const int64_t nblk = nb::ceil_div(R, 1024);
        NB_REQUIRE(D * nblk <= nb::kMaxGridX / 4, "%s: too many rows for one launch", who);
        nb::fl_layout_kernel<<<dim3((unsigned)(D * nblk)), dim3(1024), 0, nb::as_stream(stream)>>>(
            perm, slice_len, cnt, R, (int)nblk, (int)S);
        if (int rc = nb::check_launch(who)) return rc;
    }
    const int64_t n = D * R > 0 ? D * S : 0;
    nb::fl_offsets_kernel<<<dim3((unsigned)std::max<int64_t>(1, nb::ceil_div(n, 8192))), dim3(1024), 0,
                            nb::as_stream(stream)>>>(slice_off, total, slice_len, n);
    return nb::check_launch(who);
}

int nb_flip_to_dense_i64(int64_t *W, const uint32_t *entries, const int64_t *slice_off, const int32_t *slice_len,
                         const uint16_t *perm, int64_t D, int64_t R, int64_t Kw, nb_stream_t stream)
{
    const char *who = "nb_flip_to_dense_i64";
    if (int rc = nb::flip_shape_check(D, R, Kw, who)) return rc;
    if (D * R * Kw == 0) return NB_OK;
    NB_REQUIRE_PTR(W);
    NB_REQUIRE_PTR(entries);
    NB_REQUIRE_PTR(perm);
    NB_REQUIRE_PTR(slice_off);
    NB_REQUIRE_PTR(slice_len);
    NB_REQUIRE_ALIGNED(W, 8);
    NB_REQUIRE_ALIGNED(entries, 16);
    NB_REQUIRE_ALIGNED(perm, 2);
    NB_REQUIRE_ALIGNED(slice_off, 8);
    NB_REQUIRE_ALIGNED(slice_len, 4);
    const int64_t S = (R + 63) / 64;
    nb::fl_to_dense_kernel<<<dim3((unsigned)nb::ceil_div(D * S, 4)), dim3(256), 0, nb::as_stream(stream)>>>(
        reinterpret_cast<uint64_t *>(W), entries, slice_off, slice_len, perm, D * S, (int)S, R, (int)Kw);
    return nb::check_launch(who);
}

static int flip_bmv(void *out, const int32_t *G, const uint32_t *entries, const int64_t *slice_off,
                    const int32_t *slice_len, const uint16_t *perm, const uint16_t *cnt, const int64_t *x,
                    const int32_t *thresh, int64_t D, int64_t R, int64_t Kw, bool pack, nb_stream_t stream,
                    const char *who)
{
    if (int rc = nb::flip_shape_check(D, R, Kw, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(G);
    NB_REQUIRE_PTR(entries);
    NB_REQUIRE_PTR(slice_off);
    NB_REQUIRE_PTR(slice_len);
    NB_REQUIRE_PTR(perm);
    NB_REQUIRE_PTR(cnt);
    if (pack) NB_REQUIRE_PTR(thresh);
    if (Kw > 0) NB_REQUIRE_PTR(x);
    NB_REQUIRE_ALIGNED(out, pack ? 8 : 4);
    NB_REQUIRE_ALIGNED(G, 4);
    NB_REQUIRE_ALIGNED(entries, 16);
    NB_REQUIRE_ALIGNED(slice_off, 8);
    NB_REQUIRE_ALIGNED(slice_len, 4);
    NB_REQUIRE_ALIGNED(perm, 2);
    NB_REQUIRE_ALIGNED(cnt, 2);
    NB_REQUIRE_ALIGNED(x, 8);
    NB_REQUIRE_ALIGNED(thresh, 4);
    const int64_t S = (R + 63) / 64;
    const int per_block = nb::kFlipBlockRows / 64;
    const int64_t bpm = nb::ceil_div(S, per_block);
    NB_REQUIRE(D * bpm <= nb::kMaxGridX, "%s: too many rows for one launch", who);
    const unsigned threads = 64u * (unsigned)(S < per_block ? S : per_block);
    const dim3 grid((unsigned)(D * bpm));
    if (pack)
        nb::fl_bmv_kernel<true><<<grid, dim3(threads), 0, nb::as_stream(stream)>>>(
            out, G, entries, slice_off, slice_len, perm, cnt, reinterpret_cast<const uint32_t *>(x), thresh, R, (int)S,
            (int)Kw, (int)bpm);
    else
        nb::fl_bmv_kernel<false><<<grid, dim3(threads), 0, nb::as_stream(stream)>>>(
            out, G, entries, slice_off, slice_len, perm, cnt, reinterpret_cast<const uint32_t *>(x), thresh, R, (int)S,
            (int)Kw, (int)bpm);
    return nb::check_launch(who);
}

int nb_bmv_flip_i64(int32_t *out, const int32_t *G, const uint32_t *entries, const int64_t *slice_off,
                    const int32_t *slice_len, const uint16_t *perm, const uint16_t *cnt, const int64_t *x, int64_t D,
                    int64_t R, int64_t Kw, nb_stream_t stream)
{
    return flip_bmv(out, G, entries, slice_off, slice_len, perm, cnt, x, nullptr, D, R, Kw, false, stream,
                    "nb_bmv_flip_i64");
}

int nb_bmv_flip_act_pack_i64(int64_t *out, const int32_t *G, const uint32_t *entries, const int64_t *slice_off,
                             const int32_t *slice_len, const uint16_t *perm, const uint16_t *cnt, const int64_t *x,
                             const int32_t *thresh, int64_t D, int64_t R, int64_t Kw, nb_stream_t stream)
{
    return flip_bmv(out, G, entries, slice_off, slice_len, perm, cnt, x, thresh, D, R, Kw, true, stream,
                    "nb_bmv_flip_act_pack_i64");
}
}
