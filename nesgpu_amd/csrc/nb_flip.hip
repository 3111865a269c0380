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
#include <algorithm>
#include <cmath>
#include <mutex>
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

// ---- flip lists ("fixed slices") -----------------------------------------------------------------------------------
// Slice (d, s) = rows 64 s .. 64 s + 63 of member d owns `cap` 16-byte pieces per lane at entries + ((d * S + s) * cap
// + j) * 256 + 4 * l dwords (piece j of lane l = row 64 s + l): the row's flips 8j .. 8j+7 in column order, the last
// piece padded with sentinels.  info[d, r] = flips | pieces << 16: only the first `pieces` pieces of a row's lane were
// written, and nothing else of the lane is ever read.  Every slice sits at a fixed place, so lists can be written in
// one pass, by rows in any order, without knowing the other rows' lengths.
// info[d, r] from materialised weights: popcount(W[d, r, :] ^ base[r, :]), sixteen lanes per row
__global__ __launch_bounds__(256) void fl_count_kernel(uint32_t *__restrict__ info, const uint64_t *__restrict__ W,
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
    if (live && sub == 0) info[row] = flip_info((uint32_t)acc, (uint32_t)(acc + 7) >> 3);
}

// the lists from materialised weights: one wave per slice, lane l walks row 64 s + l.  A row with more flips than
// cap * 8 keeps its first cap * 8 and is counted in overflow[0].
__global__ __launch_bounds__(256) void fl_fill_kernel(uint32_t *__restrict__ entries, uint32_t *__restrict__ info,
                                                      uint32_t *__restrict__ overflow, const uint64_t *__restrict__ W,
                                                      const uint64_t *__restrict__ base, int64_t nslices, int S,
                                                      int64_t R, int Kw, int cap)
{
    const int lane = threadIdx.x & 63;
    const int64_t sl = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (sl >= nslices) return;
    const int64_t d = sl / S;
    const int s = (int)(sl - d * S);
    const int64_t r = (int64_t)s * 64 + lane;
    if (r >= R) return;
    uint4 *dst = reinterpret_cast<uint4 *>(entries) + sl * (int64_t)cap * 64 + lane;
    const uint32_t sentinel = (uint32_t)(4 * Kw) << 5;
    const int limit = 4 * cap;  // dwords of a lane
    int j = 0, n = 0;
    uint32_t pend = 0;
    bool half = false;
    uint32_t q0 = 0, q1 = 0, q2 = 0;
    auto put = [&](uint32_t v) {  // a lane's dwords leave four at a time, as whole pieces; never past the lane's share
        const int c = j & 3;
        if (c == 0) q0 = v;
        else if (c == 1) q1 = v;
        else if (c == 2) q2 = v;
        else if (j < limit) dst[(int64_t)(j >> 2) * 64] = make_uint4(q0, q1, q2, v);
        j++;
    };
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
            n++;
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
    while (j & 3) put(sentinel | (sentinel << 16));
    const int pieces = j >> 2;
    if (pieces > cap) {
        atomicAdd(overflow, 1u);
        info[d * R + r] = flip_info((uint32_t)(8 * cap), (uint32_t)cap);
    } else {
        info[d * R + r] = flip_info((uint32_t)n, (uint32_t)pieces);
    }
}

// Flip lists -> materialised weights: W must hold the base in every member on entry; every flip is XOR-ed in.  A
// lane owns its row, so plain read-modify-writes suffice (flips in column order: one write per touched word; any
// other order just writes more often).
__global__ __launch_bounds__(256) void fl_to_dense_kernel(uint64_t *__restrict__ W, const uint32_t *__restrict__ entries,
                                                          const uint32_t *__restrict__ info, int64_t nslices, int S,
                                                          int64_t R, int Kw, int cap)
{
    const int lane = threadIdx.x & 63;
    const int64_t sl = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (sl >= nslices) return;
    const int64_t d = sl / S;
    const int s = (int)(sl - d * S);
    const int64_t r = (int64_t)s * 64 + lane;
    if (r >= R) return;
    uint64_t *row = W + (d * R + r) * Kw;
    const uint32_t *src = entries + sl * (int64_t)cap * 256 + lane * 4;
    int pieces = (int)(info[d * R + r] >> 16);
    pieces = pieces < cap ? pieces : cap;
    int curw = -1;
    uint64_t mask = 0;
    for (int j = 0; j < 4 * pieces; j++) {
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
// One workgroup per (member, block of 1024 rows), one wave per slice, lane l on row 64 s + l.  A lane asks only for
// the pieces its own row has (a lane that is done requests nothing: the bytes a slice costs follow its rows' lengths
// in 64-byte sectors, not its longest row); the wave walks to its longest row.  PACK: out = bits (2 * sum > thresh)
// of the block's rows, collected in an LDS bit array and written as 32-bit pieces; else out = the int32 sums.
template <bool PACK>
__global__ __launch_bounds__(1024) void fl_bmv_kernel(void *__restrict__ out, const int32_t *__restrict__ G,
                                                      const uint32_t *__restrict__ entries,
                                                      const uint32_t *__restrict__ info, const uint32_t *__restrict__ x32,
                                                      const int32_t *__restrict__ thresh, int64_t R, int S, int Kw,
                                                      int blocks_per_member, int cap)
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
    const int64_t r = (int64_t)s * 64 + lane;
    const bool valid = active && r < R;
    const uint32_t inf = valid ? info[d * R + r] : 0u;
    const int n = (int)(inf & 0xFFFFu);
    int mine = (int)(inf >> 16);          // pieces of this lane's row
    mine = mine < cap ? mine : cap;
    int longest = mine;                   // of the slice
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const int other = __shfl_xor(longest, o);
        longest = longest > other ? longest : other;
    }
    const int L = __builtin_amdgcn_readfirstlane(longest);
    const uint4 *src = reinterpret_cast<const uint4 *>(entries) + sl * (int64_t)cap * 64 + lane;
    const uint32_t sent2 = ((uint32_t)(4 * Kw) << 5) * 0x00010001u;
    // Two register sets take turns: while one batch is looked up, the batch after it is in flight.  The first two
    // batches are requested before anything else: they do not depend on the table.
    uint4 e0[U], e1[U];
    auto request = [&](uint4(&e)[U], int j) {
#pragma unroll
        for (int u = 0; u < U; u++)
            if (j + u < L) {
                e[u] = make_uint4(sent2, sent2, sent2, sent2);
                if (j + u < mine) e[u] = load_stream16(src + (int64_t)(j + u) * 64);
            }
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
    const int g = valid ? G[d * R + r] : 0;
    const int t = (PACK && valid) ? thresh[d * R + r] : 0;
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
    if (valid) {
        const int sum = g + n - 2 * sy;
        if (PACK) {
            const int local = (int)(r - (int64_t)blk * kFlipBlockRows);
            // the 32 rows of a bitmap word are 32 consecutive lanes of this wave: one ballot half per word
            const unsigned long long m = __ballot(2 * sum > t);
            if ((lane & 31) == 0) bitmap[(local >> 5) & 31] = (uint32_t)(m >> (lane & 32));
        } else {
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

// ---- weighted sum over the lists: out[r, c] = fp16( sum_d w[d] * bit_d[r, c] ), bit = base ^ flip -------------------
//   = base[r, c] * (sum_d w[d])  +  (1 - 2 base[r, c]) * sum over the members d that flip (r, c) of w[d]
// The entry carries the base bit, so a flip adds +-w[d] to its column.  A workgroup owns RB rows (four where LDS has
// room: 64 bytes of every piece, whole sectors) and keeps their columns' sums in LDS as 32-bit fixed-point integers
// (weights scaled by a power of two chosen from sum |w[d]|, so that no sum can overflow, populations below 2^30
// members: integer adds commute, the result does not depend on the order in which the members arrive);
// lane = (row, member), 64 / RB members per wave and step; a lane asks for four pieces at a time, the next four
// before it adds the current ones.  Bound by how the lists are read (64-byte halves of lines a kilobyte apart).
__global__ __launch_bounds__(1024) void fl_wsum_kernel(_Float16 *__restrict__ out, const uint32_t *__restrict__ entries,
                                                       const uint32_t *__restrict__ info,
                                                       const uint64_t *__restrict__ base,
                                                       const _Float16 *__restrict__ wts, int64_t D, int64_t R, int C,
                                                       int Kw, int S, int cap, int RB)
{
    extern __shared__ int32_t fl_ws_acc[];  // [RB][64 * Kw] column sums, 16 x 8 bytes of scratch, 64 spare words
    float *red = reinterpret_cast<float *>(fl_ws_acc + RB * 64 * Kw);
    int32_t *spare = fl_ws_acc + RB * 64 * Kw + 32 + (threadIdx.x & 63);   // after the scratch: a word per lane
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cols = 64 * Kw;
    for (int i = tid; i < RB * cols; i += 1024) fl_ws_acc[i] = 0;
    // A = sum |w[d]| (every workgroup adds in the same order, so all agree on the scale)
    float part = 0.f;
    for (int64_t i = tid; i < D; i += 1024) part += fabsf((float)wts[i]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o);
    if (lane == 0) red[wave] = part;
    __syncthreads();
    float A = 0.f;
#pragma unroll
    for (int w = 0; w < 16; w++) A += red[w];
    // scale = 2^k with A * 2^k < 2^30 (and the rounding of each term, at most D / 2 in all, stays below 2^30 as well)
    int ex;
    (void)frexpf(A + 1.0f, &ex);  // A + 1 < 2^ex
    const int k = 29 - ex;
    const float scale = ldexpf(1.0f, k), inv_scale = ldexpf(1.0f, -k);
    // Workgroups go round the eight XCDs in turn; the 64 / RB workgroups that share a slice of 64 rows (their rows'
    // pieces lie next to each other, two workgroups to a 128-byte line) should share an L2: XCD x takes a contiguous
    // eighth of the row groups.
    int bid = (int)blockIdx.x;
    if ((gridDim.x & 7u) == 0) bid = (bid & 7) * (int)(gridDim.x >> 3) + (bid >> 3);
    const int row = lane & (RB - 1);
    const int64_t r = (int64_t)bid * RB + row;
    const bool rvalid = r < R;
    const int s = (int)(r >> 6), l = (int)(r & 63);
    int32_t *acc = fl_ws_acc + row * cols;
    const uint32_t npieces = (uint32_t)(4 * Kw);
    long long total = 0;  // sum of the scaled weights (this lane's members)
    const int per_wave = 64 / RB, shift = RB == 4 ? 2 : (RB == 2 ? 1 : 0);
    // Four pieces of a row are asked for together and the next four while those are added (a lane with one request in
    // flight leaves the memory system idle: 16 KB per compute unit); the next member's row info comes a member ahead.
    // Plain loads, not streaming ones: a 128-byte line holds a piece of eight rows, i.e. of two workgroups, and should
    // stay in L2 until the second has read its half.
    constexpr int U = 4;
    const int64_t dstep = 16 * per_wave;
    int64_t d = (int64_t)wave * per_wave + (lane >> shift);
    uint32_t inf = (rvalid && d < D) ? info[d * R + r] : 0u;
    for (; d < D; d += dstep) {
        const uint32_t inf_next = (rvalid && d + dstep < D) ? info[(d + dstep) * R + r] : 0u;
        const int wq = (int)rintf((float)wts[d] * scale);
        if (row == 0) total += wq;
        int pieces = (int)(inf >> 16);
        pieces = pieces < cap ? pieces : cap;
        inf = inf_next;
        if (!rvalid) continue;
        const uint4 *src = reinterpret_cast<const uint4 *>(entries) + (d * S + s) * (int64_t)cap * 64 + l;
        uint4 cur[U], nxt[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            cur[u] = make_uint4(0u, 0u, 0u, 0u);
            if (u < pieces) cur[u] = src[(int64_t)u * 64];
        }
        for (int j0 = 0; j0 < pieces; j0 += U) {
#pragma unroll
            for (int u = 0; u < U; u++) {
                nxt[u] = make_uint4(0u, 0u, 0u, 0u);
                if (j0 + U + u < pieces) nxt[u] = src[(int64_t)(j0 + U + u) * 64];
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                if (j0 + u < pieces) {
                    const uint32_t e[4] = {cur[u].x, cur[u].y, cur[u].z, cur[u].w};
#pragma unroll
                    for (int h = 0; h < 8; h++) {
                        // no branch per entry: a sentinel adds zero to a word of the lane's own
                        const uint32_t v = (h & 1) ? e[h >> 1] >> 16 : e[h >> 1] & 0xFFFFu;
                        const bool flip = (v >> 5) < npieces;
                        const uint32_t col = ((v >> 1) & 0xFFE0u) | (v & 31u);   // 32 * (piece / 2) + bit
                        atomicAdd(flip ? acc + col : spare, flip ? ((v & 32u) ? -wq : wq) : 0);
                    }
                }
                cur[u] = nxt[u];
            }
        }
    }
    // total of the scaled weights over all members
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) total += __shfl_xor(total, o);
    __syncthreads();
    long long *tred = reinterpret_cast<long long *>(red);
    if (lane == 0) tred[wave] = total;
    __syncthreads();
    long long F = 0;
#pragma unroll
    for (int w = 0; w < 16; w++) F += tred[w];
    for (int i = tid; i < RB * C; i += 1024) {
        const int rr = i / C, c = i - rr * C;
        const int64_t ro = (int64_t)bid * RB + rr;
        if (ro < R) {
            const long long b = (long long)((base[ro * Kw + (c >> 6)] >> (c & 63)) & 1ull);
            out[ro * C + c] = (_Float16)((float)(b * F + (long long)fl_ws_acc[rr * cols + c]) * inv_scale);
        }
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

static int flip_list_check(const uint32_t *entries, const uint32_t *info, int64_t D, int64_t R, int64_t Kw, int64_t cap,
                           const char *who)
{
    if (int rc = nb::flip_shape_check(D, R, Kw, who)) return rc;
    NB_REQUIRE(cap >= 0 && cap <= 8191, "%s: %lld pieces per row, at most 8191", who, (long long)cap);
    NB_REQUIRE(D * ((R + 63) / 64) * std::max<int64_t>(cap, 1) < (1LL << 36), "%s: lists too large", who);
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_PTR(info);
    NB_REQUIRE_ALIGNED(info, 4);
    if (cap > 0) NB_REQUIRE_PTR(entries);
    NB_REQUIRE_ALIGNED(entries, 16);
    return NB_OK;
}

int nb_flip_count_i64(uint32_t *info, const int64_t *W, const int64_t *base, int64_t D, int64_t R, int64_t Kw,
                      nb_stream_t stream)
{
    const char *who = "nb_flip_count_i64";
    if (int rc = nb::flip_shape_check(D, R, Kw, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_PTR(info);
    NB_REQUIRE_ALIGNED(info, 4);
    if (Kw > 0) {
        NB_REQUIRE_PTR(W);
        NB_REQUIRE_PTR(base);
        NB_REQUIRE_ALIGNED(W, 8);
        NB_REQUIRE_ALIGNED(base, 8);
    }
    const int64_t blocks = nb::ceil_div(D * R * 16, 256);
    NB_REQUIRE(blocks <= nb::kMaxGridX, "%s: too many rows for one launch", who);
    nb::fl_count_kernel<<<dim3((unsigned)blocks), dim3(256), 0, nb::as_stream(stream)>>>(
        info, reinterpret_cast<const uint64_t *>(W), reinterpret_cast<const uint64_t *>(base), D * R, R, (int)Kw);
    return nb::check_launch(who);
}

int nb_flip_fill_i64(uint32_t *entries, uint32_t *info, uint32_t *overflow, const int64_t *W, const int64_t *base,
                     int64_t D, int64_t R, int64_t Kw, int64_t cap, nb_stream_t stream)
{
    const char *who = "nb_flip_fill_i64";
    if (int rc = flip_list_check(entries, info, D, R, Kw, cap, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_PTR(overflow);
    NB_REQUIRE_ALIGNED(overflow, 4);
    if (Kw > 0) {
        NB_REQUIRE_PTR(W);
        NB_REQUIRE_PTR(base);
        NB_REQUIRE_ALIGNED(W, 8);
        NB_REQUIRE_ALIGNED(base, 8);
    }
    const int64_t S = (R + 63) / 64;
    nb::fl_fill_kernel<<<dim3((unsigned)nb::ceil_div(D * S, 4)), dim3(256), 0, nb::as_stream(stream)>>>(
        entries, info, overflow, reinterpret_cast<const uint64_t *>(W), reinterpret_cast<const uint64_t *>(base), D * S,
        (int)S, R, (int)Kw, (int)cap);
    return nb::check_launch(who);
}

int nb_flip_to_dense_i64(int64_t *W, const uint32_t *entries, const uint32_t *info, int64_t D, int64_t R, int64_t Kw,
                         int64_t cap, nb_stream_t stream)
{
    const char *who = "nb_flip_to_dense_i64";
    if (int rc = flip_list_check(entries, info, D, R, Kw, cap, who)) return rc;
    if (D * R * Kw == 0) return NB_OK;
    NB_REQUIRE_PTR(W);
    NB_REQUIRE_ALIGNED(W, 8);
    const int64_t S = (R + 63) / 64;
    nb::fl_to_dense_kernel<<<dim3((unsigned)nb::ceil_div(D * S, 4)), dim3(256), 0, nb::as_stream(stream)>>>(
        reinterpret_cast<uint64_t *>(W), entries, info, D * S, (int)S, R, (int)Kw, (int)cap);
    return nb::check_launch(who);
}

static int flip_bmv(void *out, const int32_t *G, const uint32_t *entries, const uint32_t *info, const int64_t *x,
                    const int32_t *thresh, int64_t D, int64_t R, int64_t Kw, int64_t cap, bool pack, nb_stream_t stream,
                    const char *who)
{
    if (int rc = flip_list_check(entries, info, D, R, Kw, cap, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(G);
    if (pack) NB_REQUIRE_PTR(thresh);
    if (Kw > 0) NB_REQUIRE_PTR(x);
    NB_REQUIRE_ALIGNED(out, pack ? 8 : 4);
    NB_REQUIRE_ALIGNED(G, 4);
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
            out, G, entries, info, reinterpret_cast<const uint32_t *>(x), thresh, R, (int)S, (int)Kw, (int)bpm, (int)cap);
    else
        nb::fl_bmv_kernel<false><<<grid, dim3(threads), 0, nb::as_stream(stream)>>>(
            out, G, entries, info, reinterpret_cast<const uint32_t *>(x), thresh, R, (int)S, (int)Kw, (int)bpm, (int)cap);
    return nb::check_launch(who);
}

int nb_bmv_flip_i64(int32_t *out, const int32_t *G, const uint32_t *entries, const uint32_t *info, const int64_t *x,
                    int64_t D, int64_t R, int64_t Kw, int64_t cap, nb_stream_t stream)
{
    return flip_bmv(out, G, entries, info, x, nullptr, D, R, Kw, cap, false, stream, "nb_bmv_flip_i64");
}

int nb_bmv_flip_act_pack_i64(int64_t *out, const int32_t *G, const uint32_t *entries, const uint32_t *info,
                             const int64_t *x, const int32_t *thresh, int64_t D, int64_t R, int64_t Kw, int64_t cap,
                             nb_stream_t stream)
{
    return flip_bmv(out, G, entries, info, x, thresh, D, R, Kw, cap, true, stream, "nb_bmv_flip_act_pack_i64");
}

int nb_flip_weighted_sum_i64(uint16_t *out, const uint32_t *entries, const uint32_t *info, const int64_t *base,
                             const uint16_t *weights, int64_t D, int64_t R, int64_t C, int64_t cap, nb_stream_t stream)
{
    const char *who = "nb_flip_weighted_sum_i64";
    NB_REQUIRE(C >= 0, "%s: negative C", who);
    const int64_t Kw = (C + 63) / 64;
    if (int rc = flip_list_check(entries, info, D, R, Kw, cap, who)) return rc;
    NB_REQUIRE(D < (1LL << 30), "%s: at most 2^30 - 1 members", who);
    if (R * C == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_ALIGNED(out, 2);
    NB_REQUIRE_PTR(base);
    NB_REQUIRE_ALIGNED(base, 8);
    if (D > 0) NB_REQUIRE_PTR(weights);
    NB_REQUIRE_ALIGNED(weights, 2);
    // rows per workgroup: as many of 4, 2, 1 as LDS (160 KB per workgroup on this part) holds
    int RB = 4;
    while (RB > 1 && (size_t)RB * 64 * Kw * 4 + 384 > 150 * 1024) RB >>= 1;
    const size_t lds = (size_t)RB * 64 * Kw * 4 + 384;   // sums, 128 bytes of scratch, a spare word per lane
    static std::once_flag once;
    static hipError_t attr = hipSuccess;
    std::call_once(once, [] {
        attr = hipFuncSetAttribute(reinterpret_cast<const void *>(nb::fl_wsum_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024 + 128);
    });
    if (attr != hipSuccess) {
        (void)hipGetLastError();
        return nb::fail(NB_ERR_UNSUPPORTED, "%s: cannot raise the kernel's LDS limit: %s", who, hipGetErrorString(attr));
    }
    const int64_t S = (R + 63) / 64;
    nb::fl_wsum_kernel<<<dim3((unsigned)nb::ceil_div(R, RB)), dim3(1024), lds, nb::as_stream(stream)>>>(
        reinterpret_cast<_Float16 *>(out), entries, info, reinterpret_cast<const uint64_t *>(base),
        reinterpret_cast<const _Float16 *>(weights), D, R, (int)C, (int)Kw, (int)S, (int)cap, RB);
    return nb::check_launch(who);
}
}
