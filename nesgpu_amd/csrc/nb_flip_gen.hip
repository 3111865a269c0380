// Drawing the flip lists of the sparse linear form straight from the generator, in one pass and without a read-back.
//
// Skip sampler: with flip probability p the flipped columns of a row are a renewal process with geometric gaps, so
// only the gaps are drawn (about C*p + 1 random words per row instead of C).  Row q = d*R + r reads the Philox words
// first + q*C + i, i = 0, 1, ...; a word's rank in the table cdf[k-1] = floor(2^32 (1 - (1-p)^k)) (how many entries
// are <= the word) moves the position on by rank + 1 columns to a flip, or, beyond the table, by the table's length
// without one; the row ends when the position passes C.
//
// Thinning (per-element probabilities): the walk runs at the LARGEST flip probability p_max of the layer; words come
// in pairs (gap, accept), and a column c reached by the walk flips only if accept * T_max < Tf[r, c] * 2^32, i.e.
// with probability Tf / T_max: every column then flips with its own probability Tf[r, c] / 2^32, independently.
//
// Work is laid out by ROWS, not by members: a workgroup owns a few rows and keeps what a look-up needs of them in LDS
// (their base bits, or their probabilities), its lanes walk those rows for member after member (a lane that has
// finished a row starts its next member at once), and every row's entries go to the fixed place the list layout
// gives them (nb_flip.hip), so nothing has to be counted first.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <mutex>

#include "nb_common.hpp"
#include "nb_conv_common.hpp"

namespace nb {

constexpr int kSkipMaxTable = 4096;
// The table as the kernels take it, in device memory: [0] entries Kt, [1] the bits of the float 1 / log2(1 - p) (a hint
// for where a look-up starts probing; it changes no result), [2] the threshold p * 2^32 the table was made for, [3] 0,
// [4 + k] = cdf[k].
constexpr int kSkipHeader = 4;
constexpr int kSkipTableWords = kSkipHeader + kSkipMaxTable;

struct SkipChain {
    PhiloxKey key;
    uint64_t g;   // index of the next word
    uint4 blk;
    bool fresh;
    __device__ __forceinline__ SkipChain(const PhiloxKey &k, uint64_t start) : key(k), g(start), fresh(true) {}
    __device__ __forceinline__ void restart(uint64_t start)
    {
        g = start;
        fresh = true;
    }
    __device__ __forceinline__ uint32_t next()
    {
        if (fresh || (g & 3u) == 0) blk = philox_block(key, g >> 2);
        fresh = false;
        const uint32_t e = (uint32_t)g & 3u;
        g++;
        return e == 0 ? blk.x : e == 1 ? blk.y : e == 2 ? blk.z : blk.w;
    }
};

// Ranks of N words in the padded table tab1 (tab1[0] = 0, tab1[k] = cdf[k - 1], tab1[Kt + 1] = 2^32 - 1): the number of
// cdf entries <= the word.  The entries follow 2^32 (1 - q^k), so log2((2^32 - 1 - u) / 2^32) / log2(q) is almost always
// the rank itself; one two-entry read confirms it (tab1[est] <= u < tab1[est + 1]), and a wave in which any lane fails
// that test walks the table from its estimate.  The result never depends on the float arithmetic.
template <int N>
__device__ __forceinline__ void skip_ranks(int (&rank)[N], const uint32_t *tab1, int Kt, const uint32_t (&u)[N],
                                           float inv_log2q, float c0)
{
    uint32_t lo[N], hi[N];
    const float kt_f = (float)Kt;
#pragma unroll
    for (int e = 0; e < N; ++e) {
        const int est = (int)fminf(fmaf(__log2f((float)(~u[e])), inv_log2q, c0), kt_f);
        rank[e] = est;
        lo[e] = tab1[est];
        hi[e] = tab1[est + 1];
    }
    uint32_t bad = 0;
#pragma unroll
    for (int e = 0; e < N; ++e) bad |= (uint32_t)(lo[e] > u[e]) | (uint32_t)(hi[e] <= u[e]);
    if (__any(bad != 0)) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
            int est = rank[e];
            while (est < Kt && tab1[est + 1] <= u[e]) est++;
            while (est > 0 && tab1[est] > u[e]) est--;
            rank[e] = est;
        }
    }
}

struct GenArgs {
    uint4 *entries;
    uint32_t *info, *overflow;
    const void *rows;        // uniform: base bits [R, 2 Kw] dwords; thinning: [R, C] 16-bit flip laws
    const uint32_t *table;   // kSkipTableWords
    PhiloxKey key;
    int64_t D, R;
    int C, Kw, S, cap, MC, rb_shift;  // MC members per workgroup; 1 << rb_shift rows per workgroup
    int group;                        // lanes (rows of one member) that start their members together
};

// ALIGNED: every row starts on a block boundary of the stream (C and first multiples of 4): a block's four words are
// four straight-line steps.  THIN: words in (gap, accept) pairs against the 16-bit laws of the columns:
// bit 15 = base bit, bits 14:0 = the fp16 flip probability y <= 1/2, Tf = floor(y * 2^32).
template <bool ALIGNED, bool THIN>
__global__ __launch_bounds__(1024) void fl_gen_kernel(const GenArgs a)
{
    extern __shared__ uint32_t gen_lds[];
    uint32_t *tab1 = gen_lds;                              // kSkipMaxTable + 2
    uint32_t *rowdata = gen_lds + kSkipMaxTable + 2;       // the workgroup's rows
    const int Kt = (int)a.table[0];
    const float inv_log2q = __uint_as_float(a.table[1]);
    const uint32_t Tmax = a.table[2];
    const int RB = 1 << a.rb_shift;
    const int nrg = (int)((a.R + RB - 1) >> a.rb_shift);
    const int rg = (int)(blockIdx.x % (unsigned)nrg), mc = (int)(blockIdx.x / (unsigned)nrg);
    const int64_t r0 = (int64_t)rg << a.rb_shift;
    for (int i = threadIdx.x; i < Kt + 2; i += blockDim.x)
        tab1[i] = i == 0 ? 0u : (i <= Kt ? a.table[kSkipHeader + i - 1] : 0xFFFFFFFFu);
    const int row_dwords = THIN ? (a.C + 1) / 2 : 2 * a.Kw;   // LDS dwords of a row
    if (THIN) {
        const uint16_t *src = static_cast<const uint16_t *>(a.rows);
        uint16_t *dst16 = reinterpret_cast<uint16_t *>(rowdata);
        for (int rr = 0; rr < RB && r0 + rr < a.R; rr++)
            for (int i = threadIdx.x; i < a.C; i += blockDim.x) dst16[rr * 2 * row_dwords + i] = src[(r0 + rr) * a.C + i];
    } else {
        const uint32_t *src = static_cast<const uint32_t *>(a.rows);
        for (int rr = 0; rr < RB && r0 + rr < a.R; rr++)
            for (int i = threadIdx.x; i < row_dwords; i += blockDim.x)
                rowdata[rr * row_dwords + i] = src[(r0 + rr) * row_dwords + i];
    }
    __syncthreads();
    const int rr = (int)threadIdx.x & (RB - 1);
    const int64_t r = r0 + rr;
    const int slots = (int)blockDim.x >> a.rb_shift;         // members a workgroup walks at a time
    const int64_t dend = (int64_t)(mc + 1) * a.MC < a.D ? (int64_t)(mc + 1) * a.MC : a.D;
    int64_t d = (int64_t)mc * a.MC + ((int)threadIdx.x >> a.rb_shift);
    const uint32_t *myrow = rowdata + rr * row_dwords;
    const uint16_t *myrow16 = reinterpret_cast<const uint16_t *>(myrow);
    const uint32_t sentinel = (uint32_t)(4 * a.Kw) << 5;
    const float c0 = -32.0f * inv_log2q;
    const int C = a.C;
    if (r >= a.R) d = dend;                                   // a lane without a row
    if (Kt == 0) {                                            // p = 0: no flips anywhere
        for (; d < dend; d += slots) a.info[d * a.R + r] = 0u;
        return;
    }
    // per-lane walk state
    bool live = d < dend;
    int64_t q = 0;
    uint64_t blk = 0;
    SkipChain chain(a.key, 0);
    uint4 *dst = a.entries;
    int pos = -1, n = 0, k = 0, piece = 0;
    uint32_t q0 = 0, q1 = 0, q2 = 0, q3 = 0;
    auto start_row = [&]() {
        live = d < dend;
        if (live) {
            q = d * a.R + r;
            const uint64_t g0 = a.key.first + (uint64_t)q * (uint64_t)C;
            if (ALIGNED) blk = g0 >> 2;
            else chain.restart(g0);
            dst = a.entries + ((d * a.S + (r >> 6)) * (int64_t)a.cap) * 64 + (r & 63);
        }
        pos = live ? -1 : C;
        n = 0;
        k = 0;
        piece = 0;
    };
    auto insert = [&](uint32_t e) {                          // the piece as a 128-bit shift register: oldest entry lowest
        q0 = __builtin_amdgcn_alignbit(q1, q0, 16);
        q1 = __builtin_amdgcn_alignbit(q2, q1, 16);
        q2 = __builtin_amdgcn_alignbit(q3, q2, 16);
        q3 = (q3 >> 16) | (e << 16);
    };
    auto flush = [&]() {
        if (piece < a.cap) dst[(int64_t)piece * 64] = make_uint4(q0, q1, q2, q3);
        piece++;
        k = 0;
    };
    // one step of the walk: `rank` of the gap word; `acc` the pair's second word (THIN)
    auto step = [&](int rank, uint32_t acc) {
        pos += rank < Kt ? rank + 1 : Kt;
        bool flip = rank < Kt && pos < C;
        const int pc = pos < C ? pos : 0;
        uint32_t b;
        if (THIN) {
            const uint32_t h = myrow16[pc];
            b = h >> 15;
            const float y = (float)__builtin_bit_cast(_Float16, (uint16_t)(h & 0x7FFFu));
            const uint32_t Tf = (uint32_t)fminf(y * 4294967296.0f, 4294967040.0f);
            flip = flip && ((uint64_t)acc * (uint64_t)Tmax < ((uint64_t)Tf << 32));
        } else {
            b = (myrow[pc >> 5] >> (pc & 31)) & 1u;
        }
        if (flip) {
            insert((((2u * ((uint32_t)pc >> 5)) + b) << 5) | ((uint32_t)pc & 31u));
            n++;
            if (++k == 8) flush();
        }
    };
    auto finish_row = [&]() {
        if (k) {
            for (; k < 8; k++) insert(sentinel);
            flush();
        }
        const bool over = piece > a.cap;
        a.info[q] = over ? flip_info((uint32_t)(8 * a.cap), (uint32_t)a.cap) : flip_info((uint32_t)n, (uint32_t)piece);
        if (over) atomicAdd(a.overflow, 1u);
        d += slots;
        start_row();
    };
    start_row();
    while (__any(live)) {
        if (ALIGNED) {
            const uint4 w = philox_block(a.key, blk++);
            if (THIN) {
                const uint32_t u[2] = {w.x, w.z};
                int rank[2];
                skip_ranks<2>(rank, tab1, Kt, u, inv_log2q, c0);
                step(rank[0], w.y);
                step(rank[1], w.w);
            } else {
                const uint32_t u[4] = {w.x, w.y, w.z, w.w};
                int rank[4];
                skip_ranks<4>(rank, tab1, Kt, u, inv_log2q, c0);
#pragma unroll
                for (int e = 0; e < 4; ++e) step(rank[e], 0u);
            }
        } else {
            const uint32_t u[1] = {chain.next()};
            const uint32_t acc = THIN ? chain.next() : 0u;
            int rank[1];
            skip_ranks<1>(rank, tab1, Kt, u, inv_log2q, c0);
            step(rank[0], acc);
        }
        if (live && pos >= C) finish_row();
    }
}

// Uniform probability, rows on block boundaries of the stream: the lanes of a wave walk in step, eight words (two
// blocks) to a 16-byte piece.  Every word of a live row is a flip unless it lies beyond the table (rank Kt: the slot
// gets a sentinel, which the list layout allows anywhere) or the row has ended (sentinels to the end of the piece),
// so word i of an iteration is slot i of the piece for every lane: nothing about an entry's place is per lane, and a
// lane that has finished its row starts its next member with the next piece.  Same words, same ranks, same flips as
// fl_gen_kernel<true, false>; the lists differ only in where sentinels stand.
__global__ __launch_bounds__(1024) void fl_gen_static_kernel(const GenArgs a)
{
    extern __shared__ uint32_t gen_lds[];
    uint32_t *tab1 = gen_lds;
    uint32_t *rowdata = gen_lds + kSkipMaxTable + 2;
    const int Kt = (int)a.table[0];
    const float inv_log2q = __uint_as_float(a.table[1]);
    const int RB = 1 << a.rb_shift;
    const int nrg = (int)((a.R + RB - 1) >> a.rb_shift);
    const int rg = (int)(blockIdx.x % (unsigned)nrg), mc = (int)(blockIdx.x / (unsigned)nrg);
    const int64_t r0 = (int64_t)rg << a.rb_shift;
    for (int i = threadIdx.x; i < Kt + 2; i += blockDim.x)
        tab1[i] = i == 0 ? 0u : (i <= Kt ? a.table[kSkipHeader + i - 1] : 0xFFFFFFFFu);
    const int row_dwords = 2 * a.Kw;
    {
        const uint32_t *src = static_cast<const uint32_t *>(a.rows);
        for (int rr = 0; rr < RB && r0 + rr < a.R; rr++)
            for (int i = threadIdx.x; i < row_dwords; i += blockDim.x)
                rowdata[rr * row_dwords + i] = src[(r0 + rr) * row_dwords + i];
    }
    __syncthreads();
    const int rr = (int)threadIdx.x & (RB - 1);
    const int64_t r = r0 + rr;
    const int slots = (int)blockDim.x >> a.rb_shift;
    const int64_t dend = (int64_t)(mc + 1) * a.MC < a.D ? (int64_t)(mc + 1) * a.MC : a.D;
    int64_t d = (int64_t)mc * a.MC + ((int)threadIdx.x >> a.rb_shift);
    const uint32_t *myrow = rowdata + rr * row_dwords;
    const uint32_t sentinel = (uint32_t)(4 * a.Kw) << 5;
    const float c0 = -32.0f * inv_log2q;
    const int C = a.C;
    if (r >= a.R) d = dend;
    if (Kt == 0) {
        for (; d < dend; d += slots) a.info[d * a.R + r] = 0u;
        return;
    }
    bool live = d < dend;
    int64_t q = 0;
    uint64_t blk = 0;
    uint4 *dst = a.entries;
    int pos = C, n = 0, piece = 0;
    auto start_row = [&]() {
        live = d < dend;
        if (live) {
            q = d * a.R + r;
            blk = (a.key.first + (uint64_t)q * (uint64_t)C) >> 2;
            dst = a.entries + ((d * a.S + (r >> 6)) * (int64_t)a.cap) * 64 + (r & 63);
        }
        pos = live ? -1 : C;
        n = 0;
        piece = 0;
    };
    start_row();
    // The RB lanes that hold the rows of one 16 RB-byte run of a member's pieces (a whole 128-byte line for eight
    // rows) start every member together: they are then on the same piece in every iteration and one store
    // instruction writes the run in one piece (single 16-byte stores to scattered lines reach a third of the
    // memory's write rate).  A lane whose row has ended waits for the longest of the group's rows.
    bool rowlive = live;
    const int G = RB < a.group ? RB : a.group;
    const int gshift = (int)(threadIdx.x & 63u) & ~(G - 1);
    const unsigned long long gmask = (1ull << G) - 1ull;
    while (__any(live)) {
        uint32_t e[8];
        const int n_before = n;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const uint4 w = philox_block(a.key, blk++);
            const uint32_t u[4] = {w.x, w.y, w.z, w.w};
            int rank[4];
            skip_ranks<4>(rank, tab1, Kt, u, inv_log2q, c0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const bool beyond = rank[i] >= Kt;               // the word lies past the table: Kt columns on, no flip
                pos = pos + rank[i] + (beyond ? 0 : 1);
                const bool flip = !beyond && pos < C;
                const uint32_t pc = (uint32_t)(pos < C ? pos : 0);
                const uint32_t b = __builtin_amdgcn_ubfe(myrow[pc >> 5], pc, 1);
                const uint32_t ent = pc + (pc & ~31u) + (b << 5);   // ((2 * (pc >> 5) + b) << 5) | (pc & 31)
                e[4 * h + i] = flip ? ent : sentinel;
                n += flip ? 1 : 0;
            }
        }
        if (rowlive) {
            if (!(pos >= C && n == n_before)) {   // a last piece without a flip is not part of the list
                if (piece < a.cap)
                    dst[(int64_t)piece * 64] = make_uint4(e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16),
                                                          e[6] | (e[7] << 16));
                piece++;
            }
            if (pos >= C) {
                const bool over = piece > a.cap;
                a.info[q] = over ? flip_info((uint32_t)(8 * a.cap), (uint32_t)a.cap) : flip_info((uint32_t)n, (uint32_t)piece);
                if (over) atomicAdd(a.overflow, 1u);
                rowlive = false;
            }
        }
        pos = rowlive ? pos : C;                  // a finished lane draws on, and nothing comes of it
        const unsigned long long busy = __ballot(rowlive);
        if (live && ((busy >> gshift) & gmask) == 0ull) {
            d += slots;
            start_row();
            rowlive = live;
        }
    }
}

// ---- the table, made on the device from a threshold that lives there ---------------------------------------------------
// cdf[k - 1] = floor(2^32 (1 - (1 - p)^k)), p = T / 2^32, cdf[0] = T itself, made non-decreasing, cut where it
// saturates at 2^32 - 1 (at most kSkipMaxTable entries); T == 0: an empty table.  One workgroup of 1024 threads, four
// entries each.
__device__ __forceinline__ void skip_table_build(uint32_t *table, const uint32_t *thr)
{
    __shared__ uint32_t wave_max[16];
    __shared__ int first_full;
    const int t = threadIdx.x, lane = t & 63, wv = t >> 6;
    const uint32_t T = thr[0];
    const double p = (double)T / 4294967296.0;
    if (t == 0) first_full = kSkipMaxTable;   // index of the first saturated entry
    uint32_t v[4];
    const double l1p = p < 1.0 ? log1p(-p) : -INFINITY;
    uint32_t run = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int k = 4 * t + i + 1;
        double x = floor(-expm1((double)k * l1p) * 4294967296.0);
        x = x < 4294967295.0 ? x : 4294967295.0;
        uint32_t e = T == 0 ? 0u : (uint32_t)x;
        if (k == 1) e = T;
        run = run > e ? run : e;
        v[i] = run;
    }
    // running maximum across threads: inside the wave, then over the waves before
    uint32_t incl = run;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t up = (uint32_t)__shfl_up((int)incl, o);
        if (lane >= o) incl = incl > up ? incl : up;
    }
    if (lane == 63) wave_max[wv] = incl;
    __syncthreads();
    uint32_t before = 0;
    for (int w = 0; w < wv; w++) before = before > wave_max[w] ? before : wave_max[w];
    uint32_t prev = (uint32_t)__shfl_up((int)incl, 1);
    prev = lane == 0 ? 0u : prev;
    prev = prev > before ? prev : before;   // maximum of everything before this thread's entries
#pragma unroll
    for (int i = 0; i < 4; i++) {
        v[i] = v[i] > prev ? v[i] : prev;
        if (v[i] == 0xFFFFFFFFu) atomicMin(&first_full, 4 * t + i);
        table[kSkipHeader + 4 * t + i] = v[i];
    }
    __syncthreads();
    if (t == 0) {
        const int Kt = T == 0 ? 0 : (first_full < kSkipMaxTable ? first_full + 1 : kSkipMaxTable);
        table[0] = (uint32_t)Kt;
        const float hint = (p > 0.0 && p < 1.0) ? (float)(1.0 / log2(1.0 - p)) : 0.0f;
        table[1] = __float_as_uint(hint);
        table[2] = T;
        table[3] = 0u;
    }
}

// ---- the layers' law: weights -> probabilities --------------------------------------------------------------------------
// P = fp16(sigmoid(float(fp16(fp16(w / m) * 5)))) with m = fp16(mean|w| + 1e-5), every step rounded to fp16 where the
// tensor expression of modules/binary.py:59-60 rounds it.  mean|w| is the exact sum (fp16 values add exactly in a
// double) divided by the count and rounded once to fp16.
constexpr int kLawBlocks = 256;   // partial sums (doubles of workspace)

__global__ __launch_bounds__(256) void law_abs_sum_kernel(double *__restrict__ partial, uint32_t *__restrict__ table,
                                                          const _Float16 *__restrict__ w, int64_t n)
{
    __shared__ double red[4];
    double s = 0.0;
    // eight weights per load where the array allows it
    const int64_t n8 = (reinterpret_cast<uintptr_t>(w) & 15u) == 0 ? n >> 3 : 0;
    const uint4 *w8 = reinterpret_cast<const uint4 *>(w);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
        const uint4 v = w8[i];
        const uint32_t d[4] = {v.x, v.y, v.z, v.w};
        double t = 0.0, u = 0.0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            t += (double)fabsf((float)__builtin_bit_cast(_Float16, (uint16_t)(d[e] & 0xFFFFu)));
            u += (double)fabsf((float)__builtin_bit_cast(_Float16, (uint16_t)(d[e] >> 16)));
        }
        s += t + u;
    }
    for (int64_t i = 8 * n8 + (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        s += (double)fabsf((float)w[i]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        partial[blockIdx.x] = red[0] + red[1] + red[2] + red[3];
        if (blockIdx.x == 0 && table) table[2] = 0u;   // the largest flip threshold is collected there next
    }
}

// The denominator fp16(mean|w| + 1e-5), made by every workgroup for itself: the partial sums are fetched by as many
// threads, added in index order by one (the same additions in every workgroup: all agree), and handed round in LDS.
__device__ __forceinline__ _Float16 law_denominator(const double *partial, int nparts, int64_t n)
{
    __shared__ double part[kLawBlocks];
    __shared__ float denom_sh;
    for (int i = threadIdx.x; i < nparts; i += blockDim.x) part[i] = partial[i];
    __syncthreads();
    if (threadIdx.x == 0) {
        double s = 0.0;
        for (int i = 0; i < nparts; i++) s += part[i];
        const _Float16 mean = double_round_once_fp16(s / (double)n);
        denom_sh = (float)(_Float16)((float)mean + 1e-5f);
    }
    __syncthreads();
    return (_Float16)denom_sh;
}

__device__ __forceinline__ _Float16 law_probability(_Float16 w, _Float16 denom)
{
    const _Float16 qn = (_Float16)((float)w / (float)denom);
    const _Float16 nw = (_Float16)((float)qn * 5.0f);
    return (_Float16)(1.0f / (1.0f + expf(-(float)nw)));
}

__device__ __forceinline__ uint32_t law_threshold(_Float16 p)   // min(floor(p * 2^32), 2^32 - 1); 0 for NaN
{
    const float v = (float)p * 4294967296.0f;
    return v >= 4294967296.0f ? 0xFFFFFFFFu : (v > 0.0f ? (uint32_t)v : 0u);
}

// MODE 0: out32 = thresholds; 1: out16 = probabilities (fp16)
template <int MODE>
__global__ __launch_bounds__(256) void law_dense_kernel(uint32_t *__restrict__ out32, _Float16 *__restrict__ out16,
                                                        const _Float16 *__restrict__ w, const double *__restrict__ partial,
                                                        int nparts, int64_t n)
{
    const _Float16 denom = law_denominator(partial, nparts, n);
    NB_FLAT_LOOP(t, n)
    {
        if (t < n) {
            const _Float16 p = law_probability(w[t], denom);
            if (MODE == 0) out32[t] = law_threshold(p);
            else out16[t] = p;
        }
    }
}

// Sparse form: law[r, c] = base bit << 15 | fp16 bits of the flip probability y = min(P, 1 - P) (exact in fp16),
// base[r, :] packed, and the largest flip threshold floor(y * 2^32) of the layer into table[2] (cleared by the sum
// kernel).  One wave per 64 columns of a row: the ballot of the base bits is the packed word.
__global__ __launch_bounds__(256) void law_sparse_kernel(uint16_t *__restrict__ law, uint64_t *__restrict__ base,
                                                         uint32_t *__restrict__ table, const _Float16 *__restrict__ w,
                                                         const double *__restrict__ partial, int nparts, int64_t R,
                                                         int C, int Kw)
{
    const _Float16 denom = law_denominator(partial, nparts, R * (int64_t)C);
    const int lane = threadIdx.x & 63;
    uint32_t tmax = 0;
    for (int64_t wd = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); wd < R * Kw; wd += (int64_t)gridDim.x * 4) {
        const int64_t r = wd / Kw;
        const int c = (int)(wd - r * Kw) * 64 + lane;
        bool one = false;
        if (c < C) {
            const float p = (float)law_probability(w[r * C + c], denom);
            one = p >= 0.5f;
            const _Float16 y = (_Float16)(one ? 1.0f - p : p);   // exact: p is a multiple of 2^-11 from 1/2 on
            const uint16_t ybits = __builtin_bit_cast(uint16_t, y) & 0x7FFFu;   // NaN weights: some probability, no fault
            law[r * C + c] = (uint16_t)(ybits | (one ? 0x8000u : 0u));
            const uint32_t tf = (uint32_t)fminf((float)__builtin_bit_cast(_Float16, ybits) * 4294967296.0f, 4294967040.0f);
            tmax = tmax > tf ? tmax : tf;
        }
        const unsigned long long word = __ballot(one);
        if (lane == 0) base[wd] = word;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t other = (uint32_t)__shfl_xor((int)tmax, o);
        tmax = tmax > other ? tmax : other;
    }
    // one atomic per workgroup: they all go to the same word
    __shared__ uint32_t wave_tmax[4];
    if (lane == 0) wave_tmax[threadIdx.x >> 6] = tmax;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++) tmax = tmax > wave_tmax[w] ? tmax : wave_tmax[w];
        if (tmax) atomicMax(table + 2, tmax);
    }
}

// What the host decides from (sparse form or not, which walk, the lists' capacity), in one read-back of three
// doubles: the mean flip probability of the layer, the largest mean of a row, the largest flip probability.
__global__ __launch_bounds__(256) void law_row_sums_kernel(float *__restrict__ rows, const uint16_t *__restrict__ law, int C)
{
    __shared__ float red[4];
    const uint16_t *row = law + (int64_t)blockIdx.x * C;
    float s = 0.f;
    for (int c = threadIdx.x; c < C; c += 256) s += (float)__builtin_bit_cast(_Float16, (uint16_t)(row[c] & 0x7FFFu));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) rows[blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
}

__global__ __launch_bounds__(256) void law_stats_kernel(double *__restrict__ stats, const float *__restrict__ rows,
                                                        const uint32_t *__restrict__ table, int64_t R, int C)
{
    __shared__ double sum_sh[4];
    __shared__ float max_sh[4];
    double s = 0.0;
    float m = 0.f;
    for (int64_t r = threadIdx.x; r < R; r += 256) {
        const float v = rows[r];
        s += (double)v;
        m = fmaxf(m, v);
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        s += __shfl_xor(s, o);
        m = fmaxf(m, __shfl_xor(m, o));
    }
    if ((threadIdx.x & 63) == 0) {
        sum_sh[threadIdx.x >> 6] = s;
        max_sh[threadIdx.x >> 6] = m;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        stats[0] = ((sum_sh[0] + sum_sh[1]) + (sum_sh[2] + sum_sh[3])) / ((double)R * (double)C);
        stats[1] = (double)fmaxf(fmaxf(max_sh[0], max_sh[1]), fmaxf(max_sh[2], max_sh[3])) / (double)C;
        stats[2] = (double)table[2] / 4294967296.0;
    }
}

// thr may be table + 2 (the threshold read before anything is written, and written back unchanged)
__global__ __launch_bounds__(1024) void fl_skip_table_kernel(uint32_t *table, const uint32_t *thr)
{
    skip_table_build(table, thr);
}

static int gen_launch(GenArgs a, bool thin, bool force_walk, hipStream_t s, const char *who)
{
    const bool aligned = a.C % 4 == 0 && a.key.first % 4 == 0;
    // rows per workgroup: eight (a 128-byte line of every piece) where LDS holds them
    const size_t tab_bytes = (size_t)(kSkipMaxTable + 2) * 4;
    const size_t row_bytes = thin ? (size_t)((a.C + 1) / 2) * 4 : (size_t)a.Kw * 8;
    int shift = 3;
    while (shift > 0 && tab_bytes + (row_bytes << shift) > 150 * 1024) shift--;
    NB_REQUIRE(tab_bytes + (row_bytes << shift) <= 150 * 1024, "%s: a row of %d columns does not fit LDS", who, a.C);
    a.rb_shift = shift;
    a.group = getenv("NESBIN_FLIP_GROUP") ? atoi(getenv("NESBIN_FLIP_GROUP")) : 8;
    const size_t lds = tab_bytes + (row_bytes << shift);
    // large workgroups when the rows fill LDS (one workgroup per compute unit then), else four waves each
    const int threads = lds > 40 * 1024 ? 1024 : 256;
    const int slots = threads >> shift;
    // about eight members per lane, so that a wave does not wait long for its slowest lane at the end
    int64_t MC = (int64_t)slots * 8;
    if (MC > a.D) MC = ceil_div(a.D, slots) * slots;
    a.MC = (int)MC;
    const int64_t nrg = ceil_div(a.R, (int64_t)1 << shift), nmc = ceil_div(a.D, MC);
    NB_REQUIRE(nrg * nmc <= kMaxGridX, "%s: too many rows for one launch", who);
    static std::once_flag once;
    static hipError_t attr = hipSuccess;
    std::call_once(once, [] {
        const void *fns[5] = {reinterpret_cast<const void *>(fl_gen_kernel<false, false>),
                              reinterpret_cast<const void *>(fl_gen_kernel<false, true>),
                              reinterpret_cast<const void *>(fl_gen_kernel<true, false>),
                              reinterpret_cast<const void *>(fl_gen_kernel<true, true>),
                              reinterpret_cast<const void *>(fl_gen_static_kernel)};
        for (const void *f : fns) {
            const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
            if (e != hipSuccess) attr = e;
        }
    });
    if (attr != hipSuccess) {
        (void)hipGetLastError();
        return fail(NB_ERR_UNSUPPORTED, "%s: cannot raise the kernel's LDS limit: %s", who, hipGetErrorString(attr));
    }
    const dim3 grid((unsigned)(nrg * nmc)), block((unsigned)threads);
    if (aligned && thin) fl_gen_kernel<true, true><<<grid, block, lds, s>>>(a);
    else if (aligned && !force_walk) fl_gen_static_kernel<<<grid, block, lds, s>>>(a);
    else if (aligned) fl_gen_kernel<true, false><<<grid, block, lds, s>>>(a);
    else if (thin) fl_gen_kernel<false, true><<<grid, block, lds, s>>>(a);
    else fl_gen_kernel<false, false><<<grid, block, lds, s>>>(a);
    return check_launch(who);
}

// ---- per-element probabilities by layers ---------------------------------------------------------------------------
// Thinning at the largest probability of a layer draws C * p_max candidates per row whatever the mean: a law with a long
// tail pays for its tail.  Here the columns of a row are sorted into 16 classes by the size of their flip threshold Tf,
// class k holding 2^(30-k) < Tf <= 2^(31-k) (class 15: everything down to Tf = 1; Tf = 0 never flips and is left out),
// and the walk goes class by class over the class's columns at the class's own rate 2^-(k+1): a column it reaches flips
// iff accept < Tf * 2^(k+1), i.e. with probability Tf / 2^(31-k) >= 1/2 (class 15 aside).  The candidates of a row
// are then at most twice its flips plus a step or two per class.
//
// Contract (restated in oracle/nesbin_oracle.c, nbo_skip_flips_layered_i64): pl[r, i] = column | law << 16 lists the row's
// columns class by class, in increasing column order inside a class; cls[r, k] is where class k starts (cls[r, 16]:
// the end).  Row q = d*R + r reads the Philox words first + q*C + 2i (gap) and + 2i + 1 (accept), i = 0, 1, ...: the
// walk starts at position -1 of the first non-empty class; a gap word's rank in the class's table (the first
// kLayerTab entries of the gap table of threshold 2^(31-k)) moves it on by rank + 1 positions to a candidate, or,
// beyond the table, by the table's length without one; past the class's end the next non-empty class starts at -1
// with the next word pair; the row ends with the last class.
constexpr int kLayers = 16, kLayerTab = 512, kLayerStride = kLayerTab + 2, kLayerWords = kSkipTableWords;

__device__ __forceinline__ uint32_t law_threshold16(uint32_t law16)
{
    const float y = (float)__builtin_bit_cast(_Float16, (uint16_t)(law16 & 0x7FFFu));
    return (uint32_t)fminf(y * 4294967296.0f, 4294967040.0f);
}

// class of a flip threshold: 0 .. 15, or 16 for Tf = 0 (never flips)
__device__ __forceinline__ int law_class(uint32_t tf)
{
    if (tf == 0) return kLayers;
    const int k = __clz((int)(tf - 1u)) - 1;   // __clz(0) = 32
    return k < 0 ? 0 : (k > kLayers - 1 ? kLayers - 1 : k);
}

// The 16 gap tables, whole (kSkipTableWords each; the walk keeps the first kLayerTab entries): class k's is the table of
// threshold 2^(31-k).  A workgroup per class.
__global__ __launch_bounds__(1024) void fl_layer_tables_kernel(uint32_t *tables)
{
    __shared__ uint32_t thr;
    if (threadIdx.x == 0) thr = 0x80000000u >> blockIdx.x;
    __syncthreads();
    skip_table_build(tables + (size_t)blockIdx.x * kLayerWords, &thr);
}

// One workgroup of 16 waves per row, a wave per stretch of its columns: count the classes, then place every column
// (stable: increasing column inside a class; a class's columns of an earlier stretch come first).
__global__ __launch_bounds__(1024) void law_layers_kernel(uint32_t *__restrict__ pl, uint32_t *__restrict__ cls,
                                                          const uint16_t *__restrict__ law, int C)
{
    extern __shared__ uint32_t gen_lds[];
    uint32_t *sorted = gen_lds;                                         // the row in its new order: C words
    __shared__ uint32_t cnt[16][kLayers];
    __shared__ uint32_t cstart[kLayers + 1];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t r = blockIdx.x;
    const uint16_t *row = law + r * C;
    const int per = ((C + 63) / 64 + 15) / 16 * 64;                    // columns of a stretch
    const int cbeg = wv * per, cend = cbeg + per < C ? cbeg + per : C;
    uint32_t count[kLayers];
#pragma unroll
    for (int k = 0; k < kLayers; k++) count[k] = 0;
    for (int c0 = cbeg; c0 < cend; c0 += 64) {
        const int c = c0 + lane;
        const int k = c < cend ? law_class(law_threshold16(row[c])) : kLayers;
#pragma unroll
        for (int kk = 0; kk < kLayers; kk++) count[kk] += (uint32_t)__popcll(__ballot(k == kk));
    }
#pragma unroll
    for (int k = 0; k < kLayers; k++)
        if (lane == 0) cnt[wv][k] = count[k];
    __syncthreads();
    // thread k < 16: where each wave's columns of class k go, inside the class; then where the classes start
    if (threadIdx.x < kLayers) {
        uint32_t acc = 0;
        for (int w = 0; w < 16; w++) {
            const uint32_t v = cnt[w][threadIdx.x];
            cnt[w][threadIdx.x] = acc;
            acc += v;
        }
        cstart[threadIdx.x] = acc;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t acc = 0;
        for (int k = 0; k < kLayers; k++) {
            const uint32_t v = cstart[k];
            cstart[k] = acc;
            cls[r * (kLayers + 1) + k] = acc;
            acc += v;
        }
        cstart[kLayers] = acc;
        cls[r * (kLayers + 1) + kLayers] = acc;
    }
    __syncthreads();
    uint32_t offs[kLayers];
#pragma unroll
    for (int k = 0; k < kLayers; k++) offs[k] = cstart[k] + cnt[wv][k];
    const uint32_t run = cstart[kLayers];
    const unsigned long long below = (1ull << lane) - 1ull;
    for (int c0 = cbeg; c0 < cend; c0 += 64) {
        const int c = c0 + lane;
        const uint32_t l = c < cend ? row[c] : 0u;
        const int k = c < cend ? law_class(law_threshold16(l)) : kLayers;
#pragma unroll
        for (int kk = 0; kk < kLayers; kk++) {
            const unsigned long long m = __ballot(k == kk);
            if (k == kk) sorted[offs[kk] + (uint32_t)__popcll(m & below)] = (uint32_t)c | (l << 16);
            offs[kk] += (uint32_t)__popcll(m);
        }
    }
    __syncthreads();
    // the row leaves in whole lines; the columns that never flip fill its end (never read by the walk)
    uint32_t *out = pl + r * C;
    for (uint32_t i = threadIdx.x; i < (uint32_t)C; i += 1024) out[i] = i < run ? sorted[i] : 0xFFFFu;
}

struct LayerArgs {
    uint4 *entries;
    uint32_t *info, *overflow;
    const uint32_t *pl, *cls, *tables;   // [R, C], [R, 17], [16, kLayerWords]
    PhiloxKey key;
    int64_t D, R;
    int C, Kw, S, cap, MC, rb_shift;
    int batch;   // lanes of a wave that end their rows together
};

// INLDS: the workgroup's rows of pl are staged in LDS; else (rows too long for that) read where they lie.
template <bool ALIGNED, bool INLDS>
__global__ __launch_bounds__(1024) void fl_gen_layered_kernel(const LayerArgs a)
{
    extern __shared__ uint32_t gen_lds[];
    uint32_t *tabs = gen_lds;                                                 // kLayers tables of kLayerStride words
    int *kts = reinterpret_cast<int *>(tabs + kLayers * kLayerStride);        // entries of each
    float *hints = reinterpret_cast<float *>(kts + kLayers);                  // 1 / log2(1 - p_k)
    const int RB = 1 << a.rb_shift;
    uint32_t *cl = reinterpret_cast<uint32_t *>(hints + kLayers);             // RB x (kLayers + 1) class starts
    uint32_t *rowdata = cl + 8 * (kLayers + 1);                               // RB x C (column | law << 16)
    const int nrg = (int)((a.R + RB - 1) >> a.rb_shift);
    const int rg = (int)(blockIdx.x % (unsigned)nrg), mc = (int)(blockIdx.x / (unsigned)nrg);
    const int64_t r0 = (int64_t)rg << a.rb_shift;
    for (int idx = threadIdx.x; idx < kLayers * kLayerStride; idx += blockDim.x) {
        const int k = idx / kLayerStride, i = idx - k * kLayerStride;
        const uint32_t *t = a.tables + k * kLayerWords;
        const int kt = (int)t[0] < kLayerTab ? (int)t[0] : kLayerTab;
        tabs[idx] = i == 0 ? 0u : (i <= kt ? t[kSkipHeader + i - 1] : 0xFFFFFFFFu);
        if (i == 0) {
            kts[k] = kt;
            hints[k] = __uint_as_float(t[1]);
        }
    }
    for (int rr = 0; rr < RB && r0 + rr < a.R; rr++) {
        if (INLDS)
            for (int i = threadIdx.x; i < a.C; i += blockDim.x) rowdata[rr * a.C + i] = a.pl[(r0 + rr) * a.C + i];
        for (int i = threadIdx.x; i <= kLayers; i += blockDim.x) cl[rr * (kLayers + 1) + i] = a.cls[(r0 + rr) * (kLayers + 1) + i];
    }
    __syncthreads();
    const int rr = (int)threadIdx.x & (RB - 1);
    const int64_t r = r0 + rr;
    const int slots = (int)blockDim.x >> a.rb_shift;
    const int64_t dend = (int64_t)(mc + 1) * a.MC < a.D ? (int64_t)(mc + 1) * a.MC : a.D;
    int64_t d = (int64_t)mc * a.MC + ((int)threadIdx.x >> a.rb_shift);
    const uint32_t *myrow = INLDS ? rowdata + rr * a.C : a.pl + (r < a.R ? r : 0) * a.C;
    const uint32_t *mycl = cl + rr * (kLayers + 1);
    const uint32_t sentinel = (uint32_t)(4 * a.Kw) << 5;
    if (r >= a.R) d = dend;
    // the lane keeps its row for all its members: which classes have columns, once
    uint32_t nonempty = 0;
    if (r < a.R)
        for (int c = 0; c < kLayers; c++) nonempty |= (mycl[c + 1] != mycl[c] ? 1u : 0u) << c;
    bool live = d < dend;
    int64_t q = 0;
    uint64_t blk = 0;
    SkipChain chain(a.key, 0);
    uint4 *dst = a.entries;
    int cur = 0, pos = -1, nk = 0, startk = 0, n = 0, k = 0, piece = 0;
    // the current class's table: where it starts in LDS, its length, the hint of its look-ups
    const uint32_t *tab1 = tabs;
    int kt = 0;
    float hint = -1.0f;
    uint32_t q0 = 0, q1 = 0, q2 = 0, q3 = 0;
    auto insert = [&](uint32_t e) {
        q0 = __builtin_amdgcn_alignbit(q1, q0, 16);
        q1 = __builtin_amdgcn_alignbit(q2, q1, 16);
        q2 = __builtin_amdgcn_alignbit(q3, q2, 16);
        q3 = (q3 >> 16) | (e << 16);
    };
    auto flush = [&]() {
        if (piece < a.cap) dst[(int64_t)piece * 64] = make_uint4(q0, q1, q2, q3);
        piece++;
        k = 0;
    };
    // the next class that has columns, from `from` on; kLayers: none left
    auto enter_class = [&](int from) {
        const uint32_t left = from < kLayers ? nonempty >> from : 0u;
        cur = left ? from + (int)__builtin_ctz(left) : kLayers;
        const int c = cur < kLayers ? cur : 0;
        // (class starts beyond the row, which only a caller's own faulty sort can hold, end the class at once)
        startk = (int)(mycl[c] < (uint32_t)a.C ? mycl[c] : (uint32_t)a.C);
        nk = (int)(mycl[c + 1] < (uint32_t)a.C ? mycl[c + 1] : (uint32_t)a.C) - startk;
        kt = kts[c];
        hint = hints[c];
        tab1 = tabs + c * kLayerStride;
        pos = -1;
    };
    auto start_row = [&]() {
        live = d < dend;
        if (live) {
            q = d * a.R + r;
            const uint64_t g0 = a.key.first + (uint64_t)q * (uint64_t)a.C;
            if (ALIGNED) blk = g0 >> 2;
            else chain.restart(g0);
            dst = a.entries + ((d * a.S + (r >> 6)) * (int64_t)a.cap) * 64 + (r & 63);
            enter_class(0);
        } else {
            cur = kLayers;
        }
        n = 0;
        k = 0;
        piece = 0;
    };
    auto finish_row = [&]() {
        if (k) {
            for (; k < 8; k++) insert(sentinel);
            flush();
        }
        const bool over = piece > a.cap;
        a.info[q] = over ? flip_info((uint32_t)(8 * a.cap), (uint32_t)a.cap) : flip_info((uint32_t)n, (uint32_t)piece);
        if (over) atomicAdd(a.overflow, 1u);
        d += slots;
        start_row();
    };
    auto rank_of = [&](uint32_t gap) {
        const uint32_t u[1] = {gap};
        int rank[1];
        skip_ranks<1>(rank, tab1, kt, u, hint, -32.0f * hint);
        return rank[0];
    };
    // one step of the walk in the lane's current class: the rank of a gap word and the pair's accept word
    auto step = [&](int rank, uint32_t acc) {
        pos += rank < kt ? rank + 1 : kt;
        if (pos >= nk) {
            enter_class(cur + 1);
        } else if (rank < kt) {
            const uint32_t e = myrow[startk + pos];
            const uint32_t col = e & 0xFFFFu, l = e >> 16;
            // accept < Tf * 2^(k+1) in 32 bits: the right side is even, so halve both (Tf * 2^k <= 2^31)
            if ((acc >> 1) < (law_threshold16(l) << cur)) {
                insert((((2u * (col >> 5)) + (l >> 15)) << 5) | (col & 31u));
                n++;
                if (++k == 8) flush();
            }
        }
    };
    start_row();
    while (__any(live)) {
        // A lane whose row has ended waits until `batch` lanes of the wave have (or none is walking): the wave then
        // goes through the end of a row and the start of the next once for all of them, not in every turn.
        const bool ended = live && cur >= kLayers;   // also rows without a column that can flip
        if (__popcll(__ballot(ended)) >= a.batch || !__any(live && !ended)) {
            if (ended) finish_row();
        }
        if (live && cur < kLayers) {
            if (ALIGNED) {
                const uint4 w = philox_block(a.key, blk++);
                step(rank_of(w.x), w.y);
                if (cur < kLayers) step(rank_of(w.z), w.w);
            } else {
                const uint32_t gap = chain.next();
                const uint32_t acc = chain.next();
                step(rank_of(gap), acc);
            }
        }
    }
}

static int layered_launch(LayerArgs a, hipStream_t s, const char *who)
{
    const bool aligned = a.C % 4 == 0 && a.key.first % 4 == 0;
    const size_t fixed = (size_t)(kLayers * kLayerStride + 2 * kLayers + 8 * (kLayers + 1)) * 4;
    const size_t row_bytes = (size_t)a.C * 4;
    // rows per workgroup: eight (a 128-byte line of every piece) where LDS holds them; two at least, else none in LDS
    int shift = 3;
    while (shift > 1 && fixed + (row_bytes << shift) > 150 * 1024) shift--;
    bool inlds = fixed + (row_bytes << shift) <= 150 * 1024;
    if (const char *e = getenv("NESBIN_LAYERED_LDS")) inlds = inlds && atoi(e) != 0;
    if (!inlds) shift = 3;
    a.rb_shift = shift;
    a.batch = 4;
    if (const char *e = getenv("NESBIN_LAYERED_BATCH")) a.batch = std::max(1, std::min(64, atoi(e)));
    const size_t lds = fixed + (inlds ? row_bytes << shift : 0);
    const int threads = 1024;
    const int slots = threads >> shift;
    int64_t MC = (int64_t)slots * 8;
    if (MC > a.D) MC = ceil_div(a.D, slots) * slots;
    a.MC = (int)MC;
    const int64_t nrg = ceil_div(a.R, (int64_t)1 << shift), nmc = ceil_div(a.D, MC);
    NB_REQUIRE(nrg * nmc <= kMaxGridX, "%s: too many rows for one launch", who);
    static std::once_flag once;
    static hipError_t attr = hipSuccess;
    std::call_once(once, [] {
        const void *fns[2] = {reinterpret_cast<const void *>(fl_gen_layered_kernel<false, true>),
                              reinterpret_cast<const void *>(fl_gen_layered_kernel<true, true>)};
        for (const void *f : fns) {
            const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);
            if (e != hipSuccess) attr = e;
        }
    });
    if (attr != hipSuccess) {
        (void)hipGetLastError();
        return fail(NB_ERR_UNSUPPORTED, "%s: cannot raise the kernel's LDS limit: %s", who, hipGetErrorString(attr));
    }
    const dim3 grid((unsigned)(nrg * nmc)), block((unsigned)threads);
    if (aligned && inlds) fl_gen_layered_kernel<true, true><<<grid, block, lds, s>>>(a);
    else if (aligned) fl_gen_layered_kernel<true, false><<<grid, block, lds, s>>>(a);
    else if (inlds) fl_gen_layered_kernel<false, true><<<grid, block, lds, s>>>(a);
    else fl_gen_layered_kernel<false, false><<<grid, block, lds, s>>>(a);
    return check_launch(who);
}

static int gen_check(const uint32_t *entries, const uint32_t *info, const uint32_t *overflow, const void *rows,
                     const uint32_t *table, int64_t D, int64_t R, int64_t C, int64_t cap, const char *who)
{
    NB_REQUIRE(D >= 0 && R >= 0 && C >= 0, "%s: negative shape D=%lld R=%lld C=%lld", who, (long long)D, (long long)R,
               (long long)C);
    const int64_t Kw = (C + 63) / 64;
    NB_REQUIRE(Kw <= 511, "%s: rows of %lld words, at most 511", who, (long long)Kw);
    NB_REQUIRE(R <= 65536, "%s: %lld rows per member, at most 65536", who, (long long)R);
    NB_REQUIRE(D * ((R + 63) / 64) <= (1LL << 31) && D * R < (1LL << 40), "%s: too many rows", who);
    NB_REQUIRE(cap >= 0 && cap <= 8191, "%s: %lld pieces per row, at most 8191", who, (long long)cap);
    NB_REQUIRE(D * ((R + 63) / 64) * std::max<int64_t>(cap, 1) < (1LL << 36), "%s: lists too large", who);
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_PTR(info);
    NB_REQUIRE_PTR(overflow);
    NB_REQUIRE_PTR(table);
    NB_REQUIRE_ALIGNED(info, 4);
    NB_REQUIRE_ALIGNED(overflow, 4);
    NB_REQUIRE_ALIGNED(table, 4);
    if (cap > 0) NB_REQUIRE_PTR(entries);
    NB_REQUIRE_ALIGNED(entries, 16);
    if (C > 0) NB_REQUIRE_PTR(rows);
    return NB_OK;
}


// ---- the skip sampler's masks as packed words (short rows) ---------------------------------------------------------
// out = base ^ mask for rows of at most KW words, the mask being the one the lists above describe: row q = m*R + r
// walks the Philox words first + q*C + i exactly as fl_gen_kernel does, so the result is what expanding
// nb_flip_skip's lists gives.  For the filters of a conv layer (64 to 512 channels per tap, a few flips per row at
// most) that is one or two random words per row instead of one per bit.
// A workgroup takes a chunk of `rc` rows (conv: whole output channels, rc = oc * KK) of `mc` members: a lane walks
// row after row and leaves their words in LDS, then the workgroup writes the chunks where the update
// step reads it ([n, R, Rw]) and, for a conv layer, where the conv multiplies it ([n, KK * Rw, O], word k of row
// (o, t) at [m][t * Rw + k][o]), both in runs of whole lines.
template <typename W>
struct SkipDenseArgs {
    W *out_rows, *out_conv;   // either may be null
    const W *base;            // may be null: the mask alone
    const uint32_t *table;
    PhiloxKey key;
    int64_t n, R;
    int C, Rw, O, KK, oc, mc, nchunk;   // a chunk: oc output channels = oc * KK rows; nchunk chunks; mc members per workgroup
    int tabw;                 // LDS words kept for the table: min(C, kSkipMaxTable) + 2, rounded up to even
};

template <typename W, int KW>
__global__ __launch_bounds__(256) void sample_skip_kernel(const SkipDenseArgs<W> a)
{
    constexpr int bits = WordTraits<W>::bits, lb = WordTraits<W>::log2bits;
    extern __shared__ uint32_t gen_lds[];
    uint32_t *tab1 = gen_lds;                                            // a.tabw words
    W *basebuf = reinterpret_cast<W *>(gen_lds + a.tabw);                // rc * Rw words: the chunk's base rows
    W *stage = basebuf + a.oc * a.KK * a.Rw;                             // mc * rc * Rw words
    // a rank of C or more ends the row whatever it is: only the first C entries of the table are ever looked at
    const int Kfull = (int)a.table[0];
    const int Kt = Kfull < a.C ? Kfull : a.C;
    const float inv_log2q = __uint_as_float(a.table[1]);
    const float c0 = -32.0f * inv_log2q;
    for (int i = threadIdx.x; i < Kt + 2; i += 256)
        tab1[i] = i == 0 ? 0u : (i <= Kt ? a.table[kSkipHeader + i - 1] : 0xFFFFFFFFu);
    // 32-bit arithmetic throughout (the host checks the ranges): a 64-bit division costs as much as a row's walk
    const unsigned ch = blockIdx.x % (unsigned)a.nchunk, mg = blockIdx.x / (unsigned)a.nchunk;
    const int o0 = (int)ch * a.oc;                                      // first output channel of the chunk
    const int ocl = a.O - o0 < a.oc ? a.O - o0 : a.oc;                  // its channels
    const int r0 = o0 * a.KK, rows = ocl * a.KK;
    const int64_t m0 = (int64_t)mg * a.mc;
    const int members = (int)(a.n - m0 < a.mc ? a.n - m0 : a.mc);      // members of this workgroup
    const int C = a.C, Rw = a.Rw;
    const int words = rows * Rw;                                        // of one member's chunk
    const int items = members * rows;                                   // rows to walk: item = ml * rows + rl
    // the chunk's base rows, four loads in flight per lane
    for (int j0 = 0; j0 < words; j0 += 1024) {
        W v[4];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int j = j0 + e * 256 + (int)threadIdx.x;
            v[e] = (a.base && j < words) ? a.base[(int64_t)r0 * Rw + j] : (W)0;
        }
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int j = j0 + e * 256 + (int)threadIdx.x;
            if (j < words) basebuf[j] = v[e];
        }
    }
    __syncthreads();
    // A lane walks item after item (lane, lane + 256, ...) without waiting for the others: a row takes one word or
    // many, and lanes in step row by row would idle through the longest row of every pass.  One step of the walk is
    // the same straight code for every lane (a lane out of items computes on and is ignored); only handing a finished
    // row over is a branch.
    const int qd = 256 / rows, qr = 256 - qd * rows;                    // the next item: 256 further
    int it = (int)threadIdx.x;
    int ml = it / rows, rl = it - ml * rows;
    bool live = it < items;
    auto first_word = [&]() { return a.key.first + (uint64_t)((m0 + ml) * a.R + r0 + rl) * (uint64_t)C; };
    uint64_t g = live ? first_word() : 0;
    W mask[KW];
#pragma unroll
    for (int k = 0; k < KW; k++) mask[k] = 0;
    int pos = -1;
    while (__any(live)) {
        int rank[1] = {0};
        if (Kt > 0) {                                                   // p = 0: no word is drawn, every row ends at once
            const uint4 b = philox_block(a.key, g >> 2);
            const uint32_t e = (uint32_t)g & 3u;
            const uint32_t u[1] = {e == 0 ? b.x : e == 1 ? b.y : e == 2 ? b.z : b.w};
            skip_ranks<1>(rank, tab1, Kt, u, inv_log2q, c0);
        }
        g++;
        pos += rank[0] < Kt ? rank[0] + 1 : (Kt == Kfull && Kt > 0 ? Kt : C);
        const bool done = pos >= C;
        const W bit = (!done && rank[0] < Kt) ? (W)1 << (pos & (bits - 1)) : (W)0;
#pragma unroll
        for (int k = 0; k < KW; k++) mask[k] |= (pos >> lb) == k ? bit : (W)0;
        if (live && done) {
#pragma unroll
            for (int k = 0; k < KW; k++) {
                if (k < Rw) stage[ml * words + rl * Rw + k] = mask[k] ^ basebuf[rl * Rw + k];
                mask[k] = 0;
            }
            it += 256;
            ml += qd;
            rl += qr;
            if (rl >= rows) {
                rl -= rows;
                ml++;
            }
            live = it < items;
            g = first_word();
            pos = -1;
        }
    }
    __syncthreads();
    for (int mm = 0; mm < members; mm++) {
        const int64_t m = m0 + mm;
        const W *src = stage + mm * words;
        if (a.out_rows) {
            W *dst = a.out_rows + (m * a.R + r0) * Rw;
            for (int j = threadIdx.x; j < words; j += 256) __builtin_nontemporal_store(src[j], dst + j);
        }
        if (a.out_conv) {
            // the chunk's output channels o0 .. o0 + oc - 1; j = (t * Rw + k) * oc + ol.  No division per word where
            // oc is a power of two (it almost always is) and a row is one word
            const int oc = ocl;
            const int sh = (oc & (oc - 1)) == 0 ? 31 - __builtin_clz((unsigned)oc) : -1;
            W *dst = a.out_conv + m * (int64_t)a.KK * Rw * a.O + o0;
            for (int j = threadIdx.x; j < words; j += 256) {
                const int tk = sh >= 0 ? j >> sh : j / oc, ol = j - tk * oc;
                int t = tk, k = 0;
                if (KW > 1) {
                    t = tk / Rw;
                    k = tk - t * Rw;
                }
                __builtin_nontemporal_store(src[(ol * a.KK + t) * Rw + k], dst + (int64_t)tk * a.O + ol);
            }
        }
    }
}

template <typename W>
static int sample_skip_launch(W *out_conv, W *out_rows, const W *base, const uint32_t *table, uint64_t seed,
                              uint64_t subseq, uint64_t first, int64_t n, int64_t O, int64_t KK, int64_t C,
                              hipStream_t s, const char *who)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_REQUIRE(n >= 0 && O >= 0 && KK >= 1 && C >= 0, "%s: negative shape", who);
    const int64_t R = O * KK, Rw = ceil_div(C, bits);
    if (n * R * Rw == 0) return NB_OK;
    NB_REQUIRE(out_conv || out_rows, "%s: no output", who);
    NB_REQUIRE_PTR(table);
    NB_REQUIRE_ALIGNED(table, 4);
    NB_REQUIRE_ALIGNED(out_conv, sizeof(W));
    NB_REQUIRE_ALIGNED(out_rows, sizeof(W));
    NB_REQUIRE_ALIGNED(base, sizeof(W));
    if (Rw > 8)
        return fail(NB_ERR_UNSUPPORTED, "%s: rows of more than 8 words (%lld): use the flip lists or the per-bit sampler",
                    who, (long long)Rw);
    NB_REQUIRE(KK * Rw <= 2048 && R * Rw < (1LL << 31) && n < (1LL << 40), "%s: shape too large", who);
    // rows per chunk: whole output channels, about 2048 words of staging at most; members per workgroup: enough rows
    // to spread the table's load over, while the launch keeps a few thousand workgroups
    int64_t oc = std::max<int64_t>(1, 2048 / (KK * Rw));
    if (oc > O) oc = O;
    if (oc >= 16) oc &= ~15LL;  // runs of whole 128-byte lines in the conv layout
    const int64_t rc = oc * KK, nchunk = ceil_div(R, rc);
    // members per workgroup: as many as 4096 words of staging hold (long queues of rows per lane even out the lanes),
    // while the launch keeps a thousand workgroups
    int64_t mc = std::max<int64_t>(1, 4096 / (rc * Rw));
    while (mc > 1 && nchunk * ceil_div(n, mc) < 2048) mc >>= 1;
    const int64_t blocks = nchunk * ceil_div(n, mc);
    NB_REQUIRE(blocks <= kMaxGridX, "%s: too many workgroups for one launch", who);
    SkipDenseArgs<W> a{};
    a.out_rows = out_rows;
    a.out_conv = out_conv;
    a.base = base;
    a.table = table;
    a.key = PhiloxKey{seed, subseq, first};
    a.n = n;
    a.R = R;
    a.C = (int)C;
    a.Rw = (int)Rw;
    a.O = (int)O;
    a.KK = (int)KK;
    a.oc = (int)oc;
    a.mc = (int)mc;
    a.nchunk = (int)nchunk;
    a.tabw = (int)((std::min<int64_t>(C, kSkipMaxTable) + 3) & ~1LL);
    const size_t lds = (size_t)a.tabw * 4 + (size_t)((mc + 1) * rc * Rw) * sizeof(W);
    const dim3 grid((unsigned)blocks), block(256);
    if (Rw == 1) sample_skip_kernel<W, 1><<<grid, block, lds, s>>>(a);
    else if (Rw == 2) sample_skip_kernel<W, 2><<<grid, block, lds, s>>>(a);
    else if (Rw <= 4) sample_skip_kernel<W, 4><<<grid, block, lds, s>>>(a);
    else sample_skip_kernel<W, 8><<<grid, block, lds, s>>>(a);
    return check_launch(who);
}

}  // namespace nb

extern "C" {
int64_t nb_skip_table_words(void) { return nb::kSkipTableWords; }

int nb_skip_table(uint32_t *table, const uint32_t *threshold, nb_stream_t stream)
{
    const char *who = "nb_skip_table";
    NB_REQUIRE_PTR(table);
    NB_REQUIRE_PTR(threshold);
    NB_REQUIRE_ALIGNED(table, 4);
    NB_REQUIRE_ALIGNED(threshold, 4);
    nb::fl_skip_table_kernel<<<dim3(1), dim3(1024), 0, nb::as_stream(stream)>>>(table, threshold);
    return nb::check_launch(who);
}

int nb_flip_skip_i64(uint32_t *entries, uint32_t *info, uint32_t *overflow, const int64_t *base, const uint32_t *table,
                     uint64_t seed, uint64_t subseq, uint64_t first, int64_t D, int64_t R, int64_t C, int64_t cap,
                     nb_stream_t stream)
{
    const char *who = "nb_flip_skip_i64";
    if (int rc = nb::gen_check(entries, info, overflow, base, table, D, R, C, cap, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_ALIGNED(base, 8);
    nb::GenArgs a{};
    a.entries = reinterpret_cast<uint4 *>(entries);
    a.info = info;
    a.overflow = overflow;
    a.rows = base;
    a.table = table;
    a.key = nb::PhiloxKey{seed, subseq, first};
    a.D = D;
    a.R = R;
    a.C = (int)C;
    a.Kw = (int)((C + 63) / 64);
    a.S = (int)((R + 63) / 64);
    a.cap = (int)cap;
    return nb::gen_launch(a, false, getenv("NESBIN_FLIP_WALK") != nullptr, nb::as_stream(stream), who);
}

int nb_flip_skip_thin_i64(uint32_t *entries, uint32_t *info, uint32_t *overflow, const uint16_t *law,
                          const uint32_t *table, uint64_t seed, uint64_t subseq, uint64_t first, int64_t D, int64_t R,
                          int64_t C, int64_t cap, nb_stream_t stream)
{
    const char *who = "nb_flip_skip_thin_i64";
    if (int rc = nb::gen_check(entries, info, overflow, law, table, D, R, C, cap, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE_ALIGNED(law, 2);
    nb::GenArgs a{};
    a.entries = reinterpret_cast<uint4 *>(entries);
    a.info = info;
    a.overflow = overflow;
    a.rows = law;
    a.table = table;
    a.key = nb::PhiloxKey{seed, subseq, first};
    a.D = D;
    a.R = R;
    a.C = (int)C;
    a.Kw = (int)((C + 63) / 64);
    a.S = (int)((R + 63) / 64);
    a.cap = (int)cap;
    return nb::gen_launch(a, true, false, nb::as_stream(stream), who);
}

int64_t nb_flip_layer_table_words(void) { return nb::kLayers * nb::kLayerWords; }

int nb_flip_layer_tables(uint32_t *tables, nb_stream_t stream)
{
    const char *who = "nb_flip_layer_tables";
    NB_REQUIRE_PTR(tables);
    NB_REQUIRE_ALIGNED(tables, 4);
    nb::fl_layer_tables_kernel<<<dim3(nb::kLayers), dim3(1024), 0, nb::as_stream(stream)>>>(tables);
    return nb::check_launch(who);
}

int nb_flip_law_layers(uint32_t *pl, uint32_t *cls, const uint16_t *law, int64_t R, int64_t C, nb_stream_t stream)
{
    const char *who = "nb_flip_law_layers";
    NB_REQUIRE(R >= 0 && C >= 0, "%s: negative shape R=%lld, C=%lld", who, (long long)R, (long long)C);
    if (R == 0) return NB_OK;
    NB_REQUIRE_PTR(cls);
    NB_REQUIRE_ALIGNED(cls, 4);
    if (C > 0) {
        NB_REQUIRE_PTR(pl);
        NB_REQUIRE_PTR(law);
        NB_REQUIRE_ALIGNED(pl, 4);
        NB_REQUIRE_ALIGNED(law, 2);
    }
    NB_REQUIRE(R <= nb::kMaxGridX, "%s: too many rows for one launch", who);
    NB_REQUIRE(C <= 511 * 64, "%s: rows of %lld columns, at most %d", who, (long long)C, 511 * 64);
    static std::once_flag once;
    static hipError_t attr = hipSuccess;
    std::call_once(once, [] {
        attr = hipFuncSetAttribute(reinterpret_cast<const void *>(nb::law_layers_kernel),
                                   hipFuncAttributeMaxDynamicSharedMemorySize, 511 * 64 * 4);
    });
    if (attr != hipSuccess) {
        (void)hipGetLastError();
        return nb::fail(NB_ERR_UNSUPPORTED, "%s: cannot raise the kernel's LDS limit: %s", who, hipGetErrorString(attr));
    }
    nb::law_layers_kernel<<<dim3((unsigned)R), dim3(1024), (size_t)C * 4, nb::as_stream(stream)>>>(pl, cls, law, (int)C);
    return nb::check_launch(who);
}

int nb_flip_skip_layered_i64(uint32_t *entries, uint32_t *info, uint32_t *overflow, const uint32_t *pl,
                             const uint32_t *cls, const uint32_t *tables, uint64_t seed, uint64_t subseq, uint64_t first,
                             int64_t D, int64_t R, int64_t C, int64_t cap, nb_stream_t stream)
{
    const char *who = "nb_flip_skip_layered_i64";
    if (int rc = nb::gen_check(entries, info, overflow, pl, tables, D, R, C, cap, who)) return rc;
    if (D * R == 0) return NB_OK;
    NB_REQUIRE(C <= 65535, "%s: C=%lld, at most 65535 columns", who, (long long)C);
    NB_REQUIRE_PTR(cls);
    NB_REQUIRE_ALIGNED(pl, 4);
    NB_REQUIRE_ALIGNED(cls, 4);
    nb::LayerArgs a{};
    a.entries = reinterpret_cast<uint4 *>(entries);
    a.info = info;
    a.overflow = overflow;
    a.pl = pl;
    a.cls = cls;
    a.tables = tables;
    a.key = nb::PhiloxKey{seed, subseq, first};
    a.D = D;
    a.R = R;
    a.C = (int)C;
    a.Kw = (int)((C + 63) / 64);
    a.S = (int)((R + 63) / 64);
    a.cap = (int)cap;
    return nb::layered_launch(a, nb::as_stream(stream), who);
}

int nb_sample_skip_i64(int64_t *out, const int64_t *base, const uint32_t *table, uint64_t seed, uint64_t subseq,
                       uint64_t first, int64_t n, int64_t R, int64_t C, nb_stream_t stream)
{
    NB_REQUIRE_PTR(out);
    return nb::sample_skip_launch<uint64_t>(nullptr, reinterpret_cast<uint64_t *>(out),
                                            reinterpret_cast<const uint64_t *>(base), table, seed, subseq, first, n, R, 1,
                                            C, nb::as_stream(stream), "nb_sample_skip_i64");
}
int nb_sample_skip_i32(int32_t *out, const int32_t *base, const uint32_t *table, uint64_t seed, uint64_t subseq,
                       uint64_t first, int64_t n, int64_t R, int64_t C, nb_stream_t stream)
{
    NB_REQUIRE_PTR(out);
    return nb::sample_skip_launch<uint32_t>(nullptr, reinterpret_cast<uint32_t *>(out),
                                            reinterpret_cast<const uint32_t *>(base), table, seed, subseq, first, n, R, 1,
                                            C, nb::as_stream(stream), "nb_sample_skip_i32");
}
int nb_sample_conv_skip_i64(int64_t *out_conv, int64_t *out_rows, const int64_t *base, const uint32_t *table,
                            uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t O, int64_t KK, int64_t C,
                            nb_stream_t stream)
{
    return nb::sample_skip_launch<uint64_t>(reinterpret_cast<uint64_t *>(out_conv), reinterpret_cast<uint64_t *>(out_rows),
                                            reinterpret_cast<const uint64_t *>(base), table, seed, subseq, first, n, O, KK,
                                            C, nb::as_stream(stream), "nb_sample_conv_skip_i64");
}
int nb_sample_conv_skip_i32(int32_t *out_conv, int32_t *out_rows, const int32_t *base, const uint32_t *table,
                            uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t O, int64_t KK, int64_t C,
                            nb_stream_t stream)
{
    return nb::sample_skip_launch<uint32_t>(reinterpret_cast<uint32_t *>(out_conv), reinterpret_cast<uint32_t *>(out_rows),
                                            reinterpret_cast<const uint32_t *>(base), table, seed, subseq, first, n, O, KK,
                                            C, nb::as_stream(stream), "nb_sample_conv_skip_i32");
}

int64_t nb_law_workspace_bytes(void) { return nb::kLawBlocks * 8; }

static int law_sum(double *ws, uint32_t *table, const uint16_t *w, int64_t n, hipStream_t s, int *nparts,
                   const char *who)
{
    NB_REQUIRE_PTR(ws);
    NB_REQUIRE_ALIGNED(ws, 8);
    NB_REQUIRE_PTR(w);
    NB_REQUIRE_ALIGNED(w, 2);
    const int64_t blocks = std::min<int64_t>(nb::kLawBlocks, nb::ceil_div(n, 2048));
    *nparts = (int)blocks;
    nb::law_abs_sum_kernel<<<dim3((unsigned)blocks), dim3(256), 0, s>>>(ws, table, reinterpret_cast<const _Float16 *>(w), n);
    return nb::check_launch(who);
}

int nb_thresholds_from_weights(uint32_t *thresholds, const uint16_t *weights, int64_t n, void *workspace,
                               nb_stream_t stream)
{
    const char *who = "nb_thresholds_from_weights";
    NB_REQUIRE(n >= 0 && n < (1LL << 40), "%s: bad element count %lld", who, (long long)n);
    if (n == 0) return NB_OK;
    NB_REQUIRE_PTR(thresholds);
    NB_REQUIRE_ALIGNED(thresholds, 4);
    int nparts = 0;
    if (int rc = law_sum(static_cast<double *>(workspace), nullptr, weights, n, nb::as_stream(stream), &nparts, who))
        return rc;
    nb::law_dense_kernel<0><<<dim3(nb::grid_for(n)), dim3(256), 0, nb::as_stream(stream)>>>(
        thresholds, nullptr, reinterpret_cast<const _Float16 *>(weights), static_cast<const double *>(workspace), nparts, n);
    return nb::check_launch(who);
}

int nb_probabilities_from_weights(uint16_t *p, const uint16_t *weights, int64_t n, void *workspace, nb_stream_t stream)
{
    const char *who = "nb_probabilities_from_weights";
    NB_REQUIRE(n >= 0 && n < (1LL << 40), "%s: bad element count %lld", who, (long long)n);
    if (n == 0) return NB_OK;
    NB_REQUIRE_PTR(p);
    NB_REQUIRE_ALIGNED(p, 2);
    int nparts = 0;
    if (int rc = law_sum(static_cast<double *>(workspace), nullptr, weights, n, nb::as_stream(stream), &nparts, who))
        return rc;
    nb::law_dense_kernel<1><<<dim3(nb::grid_for(n)), dim3(256), 0, nb::as_stream(stream)>>>(
        nullptr, reinterpret_cast<_Float16 *>(p), reinterpret_cast<const _Float16 *>(weights),
        static_cast<const double *>(workspace), nparts, n);
    return nb::check_launch(who);
}

int nb_flip_law_stats(double *stats, float *row_sums, const uint16_t *law, const uint32_t *table, int64_t R, int64_t C,
                      nb_stream_t stream)
{
    const char *who = "nb_flip_law_stats";
    NB_REQUIRE(R > 0 && C > 0 && C <= 511 * 64 && R <= nb::kMaxGridX, "%s: bad shape R=%lld C=%lld", who, (long long)R,
               (long long)C);
    NB_REQUIRE_PTR(stats);
    NB_REQUIRE_PTR(row_sums);
    NB_REQUIRE_PTR(law);
    NB_REQUIRE_PTR(table);
    NB_REQUIRE_ALIGNED(stats, 8);
    NB_REQUIRE_ALIGNED(row_sums, 4);
    NB_REQUIRE_ALIGNED(law, 2);
    NB_REQUIRE_ALIGNED(table, 4);
    nb::law_row_sums_kernel<<<dim3((unsigned)R), dim3(256), 0, nb::as_stream(stream)>>>(row_sums, law, (int)C);
    if (int rc = nb::check_launch(who)) return rc;
    nb::law_stats_kernel<<<dim3(1), dim3(256), 0, nb::as_stream(stream)>>>(stats, row_sums, table, R, (int)C);
    return nb::check_launch(who);
}

int nb_flip_law_from_weights(uint16_t *law, int64_t *base, uint32_t *table, const uint16_t *weights, int64_t R, int64_t C,
                             void *workspace, nb_stream_t stream)
{
    const char *who = "nb_flip_law_from_weights";
    NB_REQUIRE(R >= 0 && C >= 0 && R * C < (1LL << 40) && C <= 511 * 64, "%s: bad shape R=%lld C=%lld", who, (long long)R,
               (long long)C);
    NB_REQUIRE_PTR(table);
    NB_REQUIRE_ALIGNED(table, 4);
    NB_REQUIRE(R * C > 0, "%s: empty layer", who);
    NB_REQUIRE_PTR(law);
    NB_REQUIRE_PTR(base);
    NB_REQUIRE_ALIGNED(law, 2);
    NB_REQUIRE_ALIGNED(base, 8);
    const int64_t Kw = (C + 63) / 64;
    int nparts = 0;
    if (int rc = law_sum(static_cast<double *>(workspace), table, weights, R * C, nb::as_stream(stream), &nparts, who))
        return rc;
    const int64_t blocks = std::min<int64_t>(nb::ceil_div(R * Kw, 4), 2048);
    nb::law_sparse_kernel<<<dim3((unsigned)blocks), dim3(256), 0, nb::as_stream(stream)>>>(
        law, reinterpret_cast<uint64_t *>(base), table, reinterpret_cast<const _Float16 *>(weights),
        static_cast<const double *>(workspace), nparts, R, (int)C, (int)Kw);
    if (int rc = nb::check_launch(who)) return rc;
    nb::fl_skip_table_kernel<<<dim3(1), dim3(1024), 0, nb::as_stream(stream)>>>(table, table + 2);
    return nb::check_launch(who);
}
}
