// Bernoulli bit sampling by threshold compare, materialised ([n,R,Rw] packed words) or fused into
// the XOR-popcount matrix-vector product so the per-member weights never reach memory.
//
// The draw for (member m, row r, column c) is one uint32 word: either words[(m*R+r)*C+c]
// (supplied) or word first+(m*R+r)*C+c of a Philox4x32-10 stream.  The supplied stream is
// 4 bytes per weight bit, so these kernels are HBM-bound on it: lanes read it with 16-byte
// loads at consecutive addresses and every word is touched exactly once.
#include <type_traits>

#include "nb_common.hpp"

namespace nb {

struct WordsSrc {
    const uint32_t *__restrict__ p;
    // four words starting at flat index g (g % 4 == 0, p 16-byte aligned)
    __device__ __forceinline__ uint4 load4(int64_t g) const { return load_stream16(p + g); }
    __device__ __forceinline__ uint32_t load1(int64_t g) const { return load_stream4(p + g); }
    // wave-uniform row start `row0` (flat index) plus a 32-bit per-lane offset: lets the load use a
    // scalar base register and a 32-bit vector offset
    __device__ __forceinline__ uint4 load4(int64_t row0, uint32_t off) const { return load_stream16(p + row0 + off); }
};

struct PhiloxSrc {
    PhiloxKey key;
    // (first + g) % 4 == 0 is guaranteed by the host for load4
    __device__ __forceinline__ uint4 load4(int64_t g) const { return philox_block(key, (key.first + (uint64_t)g) >> 2); }
    __device__ __forceinline__ uint32_t load1(int64_t g) const { return philox_word(key, key.first + (uint64_t)g); }
    __device__ __forceinline__ uint4 load4(int64_t row0, uint32_t off) const { return load4(row0 + off); }
};

// threshold of columns c..c+3 of row r
__device__ __forceinline__ uint4 thr4(const uint32_t *__restrict__ thresh, uint32_t ts, int64_t idx)
{
    return thresh ? *reinterpret_cast<const uint4 *>(thresh + idx) : make_uint4(ts, ts, ts, ts);
}

// bit j of the result = (word j < threshold j).  Each compare's carry is shifted in by an add-with-carry of the
// running value to itself: two vector instructions per word instead of compare, select and shift-or.
__device__ __forceinline__ uint32_t nibble_lt(uint4 w, uint4 t)
{
    uint32_t r;
    asm("v_cmp_lt_u32 vcc, %1, %5\n\tv_addc_co_u32 %0, vcc, 0, 0, vcc\n\t"
        "v_cmp_lt_u32 vcc, %2, %6\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc\n\t"
        "v_cmp_lt_u32 vcc, %3, %7\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc\n\t"
        "v_cmp_lt_u32 vcc, %4, %8\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc"
        : "=&v"(r)
        : "v"(w.w), "v"(w.z), "v"(w.y), "v"(w.x), "v"(t.w), "v"(t.z), "v"(t.y), "v"(t.x)
        : "vcc");
    return r;
}

// ---- materialised sampler, wide path: C % bits == 0 and 16-byte aligned streams ------------------
// One lane per 4 columns; bits/4 neighbouring lanes assemble one output word by OR-ing their
// shifted nibbles across the lane group.
// A workgroup owns BS consecutive quads of the [R, C] plane and U consecutive members: the thresholds and
// the base word of a quad are fetched once and reused for the U members, whose stream loads (U independent
// 16-byte non-temporal loads per lane, 16 KiB contiguous per member and workgroup) are all issued before
// the first use.
// Second, optional output in the layout a conv layer multiplies with (modules/binary.py:134-137): the rows are
// (out channel o, tap t) pairs, r = o * KK + t, and word wi of row r goes to out2[m][(t * Rw + wi) * O + o].
template <typename W>
struct ConvOut {
    W *__restrict__ out2;
    uint32_t KK, O;
    __device__ __forceinline__ int64_t at(uint32_t r, uint32_t wi, uint32_t Rw) const
    {
        const uint32_t o = r / KK, t = r - o * KK;
        return (int64_t)(t * Rw + wi) * O + o;
    }
};

template <typename W, class Src, int U, int BS, bool HAS_THR, bool HAS_BASE>
__global__ __launch_bounds__(BS) void sample_wide_kernel(W *__restrict__ out, const W *__restrict__ base,
                                                         const uint32_t *__restrict__ thresh, uint32_t ts, Src src,
                                                         int64_t n, uint32_t RC4, uint32_t plane_tiles,
                                                         int64_t total_blocks, ConvOut<W> conv, uint32_t Rw)
{
    constexpr int bits = WordTraits<W>::bits;
    constexpr int G = bits / 4;      // lanes per output word
    constexpr int WPB = BS / G;      // words a workgroup makes per member
    __shared__ W stage[U * WPB];
    for (int64_t b = blockIdx.x; b < total_blocks; b += gridDim.x) {  // block-uniform
        const int64_t mg = b / plane_tiles;
        const uint32_t pt = (uint32_t)(b - mg * plane_tiles);
        const uint32_t p = pt * BS + threadIdx.x;           // quad inside the plane
        const uint32_t pc = p < RC4 ? p : RC4 - 1;          // clamp: no branch around the loads
        const uint4 t = HAS_THR ? *reinterpret_cast<const uint4 *>(thresh + (int64_t)pc * 4) : make_uint4(ts, ts, ts, ts);
        const W bw = HAS_BASE ? base[pc / G] : (W)0;
        uint4 w[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            int64_t m = mg * U + u;
            m = m < n ? m : n - 1;
            w[u] = src.load4(m * RC4 * 4, pc * 4u);
        }
        __builtin_amdgcn_sched_barrier(0);
        // The words go out through LDS: written one per lane group they would be 8-byte pieces scattered over the U
        // members; collected first, every wave writes whole runs of consecutive words, with streaming stores.
        // (The write traffic itself, 1/32 of the read stream, is what costs most: with the same stores aimed at one
        // cache-resident 4 KB region the kernel runs 10 % faster.)
        if (b != (int64_t)blockIdx.x) __syncthreads();  // the previous round's words have been read
#pragma unroll
        for (int u = 0; u < U; u++) {
            W v = (W)nibble_lt(w[u], t) << (4 * (int)(threadIdx.x & (G - 1)));  // BS % G == 0
            v = or_reduce_group<G>(v) ^ bw;
            if ((threadIdx.x & (G - 1)) == 0) stage[u * WPB + threadIdx.x / G] = v;
        }
        __syncthreads();
        for (int i = threadIdx.x; i < U * WPB; i += BS) {
            const int u = i / WPB, wi = i - u * WPB;
            const int64_t m = mg * U + u;
            const uint32_t pw = pt * WPB + wi;  // word inside the plane; C % bits == 0: words never straddle rows
            if (m < n && pw < RC4 / G) {
                if (out) __builtin_nontemporal_store(stage[i], out + m * (RC4 / G) + pw);
                if (conv.out2) {
                    const uint32_t r = pw / Rw;
                    conv.out2[m * (RC4 / G) + conv.at(r, pw - r * Rw, Rw)] = stage[i];
                }
            }
        }
    }
}

// ---- materialised sampler from the generator, C % bits == 0: one lane per output word ---------------------------
// A lane draws the bits/4 generator blocks of one word of the [R, C] plane for U members, block by block: a block's
// four thresholds come in one 16-byte load that serves the U members, nothing crosses lanes or goes through LDS, and
// the words leave as runs of consecutive lanes.  (With supplied words the stream's bytes are what counts and the
// kernel above, a lane per four columns, reads them coalesced; with the generator the instructions per word are:
// about 14.5 here, 19 there.)
template <typename W, int U, bool HAS_THR, bool HAS_BASE>
__global__ __launch_bounds__(256) void sample_word_philox_kernel(W *__restrict__ out, const W *__restrict__ base,
                                                                 const uint32_t *__restrict__ thresh, uint32_t ts,
                                                                 PhiloxKey key, int64_t n, uint32_t PW, int64_t total,
                                                                 ConvOut<W> conv, uint32_t Rw)
{
    constexpr int bits = WordTraits<W>::bits;
    constexpr int NB = bits / 4;  // generator blocks per word
    NB_FLAT_LOOP(i, total)
    {
        if (i < total) {
            const int64_t mg = i / PW;
            const uint32_t pw = (uint32_t)(i - mg * PW);
            const uint4 *__restrict__ tq = reinterpret_cast<const uint4 *>(thresh) + (int64_t)pw * NB;
            uint64_t blk[U];
            W v[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                blk[u] = (key.first >> 2) + (uint64_t)((mg * U + u) * PW + pw) * NB;  // first % 4 == 0 (host)
                v[u] = 0;
            }
            for (int k = 0; k < NB; k++) {
                const uint4 t = HAS_THR ? tq[k] : make_uint4(ts, ts, ts, ts);
#pragma unroll
                for (int u = 0; u < U; u++) v[u] |= (W)nibble_lt(philox_block(key, blk[u] + (uint64_t)k), t) << (4 * k);
            }
            const W bw = HAS_BASE ? base[pw] : (W)0;
            const uint32_t r = pw / Rw;
            const int64_t at2 = conv.out2 ? conv.at(r, pw - r * Rw, Rw) : 0;
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int64_t m = mg * U + u;
                if (m < n) {
                    if (out) __builtin_nontemporal_store((W)(v[u] ^ bw), out + m * PW + pw);
                    if (conv.out2) conv.out2[m * PW + at2] = v[u] ^ bw;
                }
            }
        }
    }
}

// ---- the same with 16-bit draws: two weight bits per generated word -----------------------------------------------
// Column g (flat index first + (m*R + r)*C + c) takes the half-word h = half g % 2 (low half first) of element g / 2 of
// the stream (seed, subsequence) and is set iff h < T >> 16, or h == T >> 16 and l < (T & 0xFFFF) with l the low 16
// bits of element g of the stream (seed, subsequence ^ 2^63): every bit is set with probability exactly T / 2^32,
// independently, like the 32-bit compare, at half the generator work; the second stream is only read on a tie
// (2^-16 of the columns).  A generator block serves 8 columns.
//
// One column: the subtraction's borrow IS h < T >> 16 when the half-word sits in the upper 16 bits and the threshold's
// lower 16 bits are cleared, and is shifted in by an add-with-carry as in nibble_lt; the difference is below 65536
// exactly on a tie, and the smallest difference of a block says whether any of its columns had one.
__device__ __forceinline__ void col_lt16(uint32_t &r, uint32_t &zmin, uint32_t w_hi, uint32_t t_hi)
{
    uint32_t d;
    asm("v_sub_co_u32 %1, vcc, %2, %3\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc" : "+v"(r), "=&v"(d) : "v"(w_hi), "v"(t_hi) : "vcc");
    zmin = d < zmin ? d : zmin;
}

// the 8 columns of a block, column 0 in bit 0; ta / tb: thresholds of columns 0..3 / 4..7 with their low halves cleared
__device__ __forceinline__ uint32_t byte_lt16(uint4 w, uint4 ta, uint4 tb, uint32_t &zmin)
{
    uint32_t r = 0;
    col_lt16(r, zmin, w.w, tb.w);
    col_lt16(r, zmin, w.w << 16, tb.z);
    col_lt16(r, zmin, w.z, tb.y);
    col_lt16(r, zmin, w.z << 16, tb.x);
    col_lt16(r, zmin, w.y, ta.w);
    col_lt16(r, zmin, w.y << 16, ta.z);
    col_lt16(r, zmin, w.x, ta.y);
    col_lt16(r, zmin, w.x << 16, ta.x);
    return r;
}

// the columns of a block that tied, decided by the second stream; g0: flat index of the block's column 0
__device__ __forceinline__ uint32_t byte_ties16(uint32_t byte, uint4 w, uint4 ta, uint4 tb, const PhiloxKey &key, uint64_t g0)
{
    const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
    const uint32_t tt[8] = {ta.x, ta.y, ta.z, ta.w, tb.x, tb.y, tb.z, tb.w};
    const PhiloxKey tie{key.seed, key.subseq ^ 0x8000000000000000ull, 0};
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t h = (j & 1) ? ww[j >> 1] >> 16 : ww[j >> 1] & 0xFFFFu;
        if (h == tt[j] >> 16) {
            const uint32_t l = philox_word(tie, g0 + (uint64_t)j) & 0xFFFFu;
            byte = (byte & ~(1u << j)) | ((uint32_t)(l < (tt[j] & 0xFFFFu)) << j);
        }
    }
    return byte;
}

template <typename W, int U, bool HAS_THR, bool HAS_BASE>
__global__ __launch_bounds__(256) void sample_word_philox16_kernel(W *__restrict__ out, const W *__restrict__ base,
                                                                   const uint32_t *__restrict__ thresh, uint32_t ts,
                                                                   PhiloxKey key, int64_t n, uint32_t PW, int64_t total,
                                                                   ConvOut<W> conv, uint32_t Rw)
{
    constexpr int bits = WordTraits<W>::bits;
    constexpr int NB = bits / 8;  // generator blocks per word
    NB_FLAT_LOOP(i, total)
    {
        if (i < total) {
            const int64_t mg = i / PW;
            const uint32_t pw = (uint32_t)(i - mg * PW);
            const uint4 *__restrict__ tq = reinterpret_cast<const uint4 *>(thresh) + (int64_t)pw * (2 * NB);
            uint64_t blk[U];
            W v[U];
#pragma unroll
            for (int u = 0; u < U; u++) {
                blk[u] = (key.first >> 3) + (uint64_t)((mg * U + u) * PW + pw) * NB;  // first % 8 == 0 (host)
                v[u] = 0;
            }
            uint64_t tied = 0;  // bit 8 * u + k: member u's block k had a tie (U <= 8, NB <= 8)
            for (int k = 0; k < NB; k++) {
                const uint4 ta = HAS_THR ? tq[2 * k] : make_uint4(ts, ts, ts, ts);
                const uint4 tb = HAS_THR ? tq[2 * k + 1] : ta;
                const uint4 ha = make_uint4(ta.x & 0xFFFF0000u, ta.y & 0xFFFF0000u, ta.z & 0xFFFF0000u, ta.w & 0xFFFF0000u);
                const uint4 hb = make_uint4(tb.x & 0xFFFF0000u, tb.y & 0xFFFF0000u, tb.z & 0xFFFF0000u, tb.w & 0xFFFF0000u);
#pragma unroll
                for (int u = 0; u < U; u++) {
                    uint32_t zmin = 0xFFFFFFFFu;
                    const uint32_t byte = byte_lt16(philox_block(key, blk[u] + (uint64_t)k), ha, hb, zmin);
                    tied |= (uint64_t)(zmin < 65536u) << (8 * u + k);
                    v[u] |= (W)byte << (8 * k);
                }
            }
            // ties (2^-16 of the columns): the blocks that had one are drawn again and decided by the second stream
            if (__any(tied != 0)) {
                while (tied) {
                    const int bit = __builtin_ctzll(tied);
                    tied &= tied - 1;
                    const int uu = bit >> 3, k = bit & 7;
                    const uint64_t b = (key.first >> 3) + (uint64_t)((mg * U + uu) * PW + pw) * NB + (uint64_t)k;
                    const uint4 ta = HAS_THR ? tq[2 * k] : make_uint4(ts, ts, ts, ts);
                    const uint4 tb = HAS_THR ? tq[2 * k + 1] : ta;
                    const uint4 w = philox_block(key, b);
                    uint32_t zmin = 0xFFFFFFFFu;
                    const uint4 ha = make_uint4(ta.x & 0xFFFF0000u, ta.y & 0xFFFF0000u, ta.z & 0xFFFF0000u, ta.w & 0xFFFF0000u);
                    const uint4 hb = make_uint4(tb.x & 0xFFFF0000u, tb.y & 0xFFFF0000u, tb.z & 0xFFFF0000u, tb.w & 0xFFFF0000u);
                    const uint32_t byte = byte_ties16(byte_lt16(w, ha, hb, zmin), w, ta, tb, key, b << 3);
                    const W clear = ~((W)0xFF << (8 * k)), put = (W)byte << (8 * k);
#pragma unroll
                    for (int u = 0; u < U; u++) v[u] = u == uu ? (v[u] & clear) | put : v[u];
                }
            }
            const W bw = HAS_BASE ? base[pw] : (W)0;
            const uint32_t r = pw / Rw;
            const int64_t at2 = conv.out2 ? conv.at(r, pw - r * Rw, Rw) : 0;
#pragma unroll
            for (int u = 0; u < U; u++) {
                const int64_t m = mg * U + u;
                if (m < n) {
                    if (out) __builtin_nontemporal_store((W)(v[u] ^ bw), out + m * PW + pw);
                    if (conv.out2) conv.out2[m * PW + at2] = v[u] ^ bw;
                }
            }
        }
    }
}

// ---- materialised sampler, generic path: one wave per (member,row), ballot builds the words ------
template <typename W, class Src>
__global__ __launch_bounds__(256) void sample_ballot_kernel(W *__restrict__ out, const W *__restrict__ base,
                                                            const uint32_t *__restrict__ thresh, uint32_t ts, Src src,
                                                            int64_t nrows, int64_t R, int C, int Rw, ConvOut<W> conv)
{
    constexpr int bits = WordTraits<W>::bits;
    const int lane = threadIdx.x & 63;
    // one wave per (m, r) row; wave-uniform stride loop
    for (int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6); row < nrows; row += (int64_t)gridDim.x * 4) {
        const int64_t r = row % R;
        for (int c0 = 0; c0 < C; c0 += 64) {
            const int c = c0 + lane;
            bool bit = false;
            if (c < C) {
                const uint32_t t = thresh ? thresh[r * C + c] : ts;
                bit = src.load1(row * C + c) < t;
            }
            const uint64_t m = __ballot(bit);
            if (lane == 0) {
                auto put = [&](int wi, W v) {
                    v ^= base ? base[r * Rw + wi] : (W)0;
                    if (out) out[row * Rw + wi] = v;
                    if (conv.out2) conv.out2[(row / R) * (R * Rw) + conv.at((uint32_t)r, (uint32_t)wi, (uint32_t)Rw)] = v;
                };
                if (bits == 64) {
                    put(c0 >> 6, (W)m);
                } else {
                    const int wi = c0 >> 5;
                    put(wi, (W)m);
                    if (wi + 1 < Rw) put(wi + 1, (W)(m >> 32));
                }
            }
        }
    }
}

// ---- materialised sampler, rows shorter than a word: one lane per (member,row) -----------------------------------------
// (the first conv layer of an RGB network has 3 columns per row, a 16-channel layer 16: a wave per row would leave
// most lanes idle).  The generator is asked block by block: a block's four words are consecutive columns.
template <typename W, class Src>
__global__ __launch_bounds__(256) void sample_narrow_kernel(W *__restrict__ out, const W *__restrict__ base,
                                                            const uint32_t *__restrict__ thresh, uint32_t ts, Src src,
                                                            int64_t nrows, int64_t R, int C, ConvOut<W> conv, bool quads)
{
    NB_FLAT_LOOP(row, nrows)
    {
        if (row < nrows) {
            const int64_t r = row % R;
            const uint32_t *__restrict__ tr = thresh ? thresh + r * C : nullptr;
            W v = 0;
            if constexpr (std::is_same<Src, PhiloxSrc>::value) {
                const uint64_t g0 = src.key.first + (uint64_t)row * (uint64_t)C;
                if (quads) {
                    // whole generator blocks: four columns per block, their thresholds in one 16-byte load (the rows
                    // of neighbouring lanes lie C words apart: single loads would touch a cache line per lane and word)
                    const uint4 *__restrict__ tq = reinterpret_cast<const uint4 *>(tr);
#pragma unroll 4  // four blocks' thresholds asked for together
                    for (int k = 0; k < (C >> 2); k++) {
                        const uint4 b = philox_block(src.key, (g0 >> 2) + (uint64_t)k);
                        const uint4 t = tr ? tq[k] : make_uint4(ts, ts, ts, ts);
                        const uint32_t nib = (uint32_t)(b.x < t.x) | ((uint32_t)(b.y < t.y) << 1) |
                                             ((uint32_t)(b.z < t.z) << 2) | ((uint32_t)(b.w < t.w) << 3);
                        v |= (W)nib << (4 * k);
                    }
                } else
                for (uint64_t blk = g0 >> 2; blk <= (g0 + (uint64_t)C - 1) >> 2; blk++) {
                    const uint4 b = philox_block(src.key, blk);
                    const uint32_t w4[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int64_t c = (int64_t)(blk * 4 + e - g0);  // column of this word, if it is one of the row's
                        if (c >= 0 && c < C) v |= (W)(w4[e] < (tr ? tr[c] : ts)) << c;
                    }
                }
            } else {
                for (int c = 0; c < C; c++) v |= (W)(src.load1(row * C + c) < (tr ? tr[c] : ts)) << c;
            }
            v ^= base ? base[r] : (W)0;
            if (out) out[row] = v;
            if (conv.out2) conv.out2[(row / R) * R + conv.at((uint32_t)r, 0u, 1u)] = v;
        }
    }
}

// ---- fused sample + XOR-popcount matrix-vector product -------------------------------------------------
// Wide path (C % 4 == 0, aligned streams): one wave per RPW consecutive rows of one member; lane
// l covers columns 4*(l+64*it)..+3.  The lane XORs its 4 sampled bits with the matching nibbles
// of base[r] and x[m] and counts; a wave reduction per row finishes the sum.
template <typename W, class Src, int RPW>
__global__ __launch_bounds__(256) void seeded_bmv_wide_kernel(int32_t *__restrict__ Cout, const W *__restrict__ base,
                                                              const uint32_t *__restrict__ thresh, uint32_t ts,
                                                              const W *__restrict__ x, Src src, int64_t n, int64_t R,
                                                              int C4, int Rw, int64_t groups_per_member)
{
    constexpr int bits = WordTraits<W>::bits;
    constexpr int G = bits / 4;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t m = wave / groups_per_member;
    if (m >= n) return;  // wave-uniform; the host keeps n * groups_per_member within one launch
    const int64_t r0 = (wave - m * groups_per_member) * RPW;
    int acc[RPW];
#pragma unroll
    for (int q = 0; q < RPW; q++) acc[q] = 0;
    const int64_t C = (int64_t)C4 * 4;
    for (int c4 = lane; c4 < C4; c4 += 64) {
        const int wi = c4 / G, sh = 4 * (c4 & (G - 1));
        const uint32_t xn = (uint32_t)(x[m * Rw + wi] >> sh) & 0xFu;
#pragma unroll
        for (int q = 0; q < RPW; q++) {
            const int64_t r = r0 + q;
            if (r < R) {
                const uint4 w = src.load4((m * R + r) * C + 4 * (int64_t)c4);
                const uint4 t = thr4(thresh, ts, r * C + 4 * (int64_t)c4);
                uint32_t nib = nibble_lt(w, t) ^ xn;
                if (base) nib ^= (uint32_t)(base[r * Rw + wi] >> sh) & 0xFu;
                acc[q] += __popc(nib);
            }
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
#pragma unroll
        for (int q = 0; q < RPW; q++) acc[q] += __shfl_xor(acc[q], off);
    }
    if (lane == 0) {
#pragma unroll
        for (int q = 0; q < RPW; q++)
            if (r0 + q < R) Cout[m * R + r0 + q] = acc[q];
    }
}

// Streaming path (C % 256 == 0, aligned streams): every lane issues RPW*ITU independent 16-byte loads of
// the word stream before it consumes any of them, a 1024-thread workgroup covers a contiguous span of
// rows, and the per-lane work is four compares, a nibble XOR and one v_bcnt per load.
template <typename W, class Src, int RPW, int ITU, bool HAS_THR, bool HAS_BASE>
__global__ __launch_bounds__(1024) void seeded_bmv_stream_kernel(int32_t *__restrict__ Cout,
                                                                 const W *__restrict__ base,
                                                                 const uint32_t *__restrict__ thresh, uint32_t ts,
                                                                 const W *__restrict__ x, Src src, int64_t n, int R,
                                                                 int C4, int Rw, int groups_per_member)
{
    constexpr int bits = WordTraits<W>::bits;
    constexpr int G = bits / 4;
    const int lane = threadIdx.x & 63;
    // wave-uniform quantities are forced into scalar registers (the host keeps n*groups below 2^31)
    // Consecutive workgroups are dispatched round-robin over the 8 XCDs: workgroup b goes to XCD b % 8.  Give each
    // XCD one contiguous eighth of the word stream instead of every eighth 128 KB piece (0.5 % faster, measured).
    const uint32_t vb = (gridDim.x & 7u) == 0u ? (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3) : blockIdx.x;
    const uint32_t wave = vb * 16u + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t m32 = wave / (uint32_t)groups_per_member;
    if (m32 >= n) return;
    const int64_t m = m32;
    const int r0 = (int)(wave - m32 * (uint32_t)groups_per_member) * RPW;
    const int64_t C = (int64_t)C4 * 4;
    int rows[RPW];
#pragma unroll
    for (int q = 0; q < RPW; q++) rows[q] = r0 + q < R ? r0 + q : R - 1;  // tail rows are recomputed, not stored
    int acc[RPW];
#pragma unroll
    for (int q = 0; q < RPW; q++) acc[q] = 0;
    const int sh = 4 * (lane & (G - 1));
    for (int c40 = 0; c40 < C4; c40 += 64 * ITU) {
        // Issue every load of this step before consuming any: the small cached operands (x, base,
        // thresholds) first, then the RPW*ITU 16-byte loads of the word stream.
        W bx[RPW][ITU];
        uint4 t[RPW][ITU];
        uint4 w[RPW][ITU];
#pragma unroll
        for (int it = 0; it < ITU; it++) {
            const int c4 = c40 + it * 64 + lane;
            const int wi = c4 / G;
            const W xw = x[m * Rw + wi];
#pragma unroll
            for (int q = 0; q < RPW; q++) {
                bx[q][it] = HAS_BASE ? (W)(xw ^ base[(int64_t)rows[q] * Rw + wi]) : xw;
                t[q][it] = HAS_THR ? *reinterpret_cast<const uint4 *>(thresh + rows[q] * C + 4 * (int64_t)c4)
                                   : make_uint4(ts, ts, ts, ts);
            }
        }
#pragma unroll
        for (int q = 0; q < RPW; q++)
#pragma unroll
            for (int it = 0; it < ITU; it++)
                w[q][it] = src.load4((m * R + rows[q]) * C, 4u * (uint32_t)(c40 + it * 64 + lane));
        __builtin_amdgcn_sched_barrier(0);  // do not let the scheduler sink a load next to its use
#pragma unroll
        for (int it = 0; it < ITU; it++)
#pragma unroll
            for (int q = 0; q < RPW; q++)
                acc[q] += __popc(nibble_lt(w[q][it], t[q][it]) ^ ((uint32_t)(bx[q][it] >> sh) & 0xFu));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
#pragma unroll
        for (int q = 0; q < RPW; q++) acc[q] += __shfl_xor(acc[q], off);
    }
    if (lane == 0) {
#pragma unroll
        for (int q = 0; q < RPW; q++)
            if (r0 + q < R) Cout[m * R + r0 + q] = acc[q];
    }
}

template <typename W, class Src, int RPW, int ITU>
static void launch_bmv_stream(int32_t *Cout, const W *base, const uint32_t *thresh, uint32_t ts, const W *x, Src src,
                              int64_t n, int64_t R, int64_t C, int Rw, hipStream_t s)
{
    const int gpm = (int)ceil_div(R, RPW);
    const int64_t waves = n * gpm;
    const dim3 grid((unsigned)ceil_div(waves, 16)), block(1024);
#define NB_LAUNCH_STREAM(T, B)                                                                                   \
    seeded_bmv_stream_kernel<W, Src, RPW, ITU, T, B><<<grid, block, 0, s>>>(Cout, base, thresh, ts, x, src, n, (int)R, \
                                                                            (int)(C / 4), Rw, gpm)
    if (thresh && base) NB_LAUNCH_STREAM(true, true);
    else if (thresh) NB_LAUNCH_STREAM(true, false);
    else if (base) NB_LAUNCH_STREAM(false, true);
    else NB_LAUNCH_STREAM(false, false);
#undef NB_LAUNCH_STREAM
}

// Generic path: one wave per (member,row), one column per lane and step.
template <typename W, class Src>
__global__ __launch_bounds__(256) void seeded_bmv_generic_kernel(int32_t *__restrict__ Cout,
                                                                 const W *__restrict__ base,
                                                                 const uint32_t *__restrict__ thresh, uint32_t ts,
                                                                 const W *__restrict__ x, Src src, int64_t nrows,
                                                                 int64_t R, int C, int Rw)
{
    constexpr int lb = WordTraits<W>::log2bits;
    constexpr int bits = WordTraits<W>::bits;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= nrows) return;  // wave-uniform
    const int64_t m = row / R, r = row - m * R;
    int acc = 0;
    for (int c = lane; c < C; c += 64) {
        const uint32_t t = thresh ? thresh[r * C + c] : ts;
        uint32_t bit = src.load1(row * C + c) < t;
        const int wi = c >> lb, sh = c & (bits - 1);
        bit ^= (uint32_t)(x[m * Rw + wi] >> sh) & 1u;
        if (base) bit ^= (uint32_t)(base[r * Rw + wi] >> sh) & 1u;
        acc += bit;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
    if (lane == 0) Cout[row] = acc;
}

__global__ __launch_bounds__(256) void philox_words_kernel(uint32_t *__restrict__ out, PhiloxKey key, int64_t count)
{
    // one thread per aligned block of the stream; head/tail blocks are partial
    const uint64_t blk0 = key.first >> 2;
    const int64_t nblk = (int64_t)(((key.first + (uint64_t)count + 3) >> 2) - blk0);
    NB_FLAT_LOOP(t, nblk)
    {
        if (t >= nblk) continue;
        const uint64_t blk = blk0 + (uint64_t)t;
        const uint64_t gbeg = blk << 2;
        const uint4 b = philox_block(key, blk);
        const uint32_t v[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint64_t g = gbeg + e;
            if (g >= key.first && g < key.first + (uint64_t)count) out[g - key.first] = v[e];
        }
    }
}

template <typename W>
static int sample_check(const void *out, const W *base, const uint32_t *thresh, int64_t n, int64_t R, int64_t C,
                        const char *who, bool *empty)
{
    NB_REQUIRE(n >= 0 && R >= 0 && C >= 0, "%s: negative shape n=%lld R=%lld C=%lld", who, (long long)n, (long long)R,
               (long long)C);
    *empty = (n * R * C == 0);
    if (*empty) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE(C <= (1 << 30), "%s: C=%lld too large", who, (long long)C);
    NB_REQUIRE(n * R <= (1LL << 40), "%s: n*R=%lld rows is too many", who, (long long)(n * R));
    if (base) NB_REQUIRE_ALIGNED(base, sizeof(W));
    if (thresh) NB_REQUIRE_ALIGNED(thresh, 4);
    return NB_OK;
}

template <typename W, class Src>
int sample_impl(W *out, const W *base, const uint32_t *thresh, uint32_t ts, Src src, bool src_vec_ok, int64_t n,
                int64_t R, int64_t C, nb_stream_t stream, const char *who, W *out_conv = nullptr, int64_t KK = 1)
{
    constexpr int bits = WordTraits<W>::bits;
    bool empty;
    if (int rc = sample_check<W>(out ? out : out_conv, base, thresh, n, R, C, who, &empty)) return rc;
    if (empty) return NB_OK;
    NB_REQUIRE_ALIGNED(out, sizeof(W));
    NB_REQUIRE_ALIGNED(out_conv, sizeof(W));
    NB_REQUIRE(KK >= 1 && R % KK == 0 && R < (1LL << 31), "%s: %lld rows are not whole groups of %lld taps", who,
               (long long)R, (long long)KK);
    const ConvOut<W> conv{out_conv, (uint32_t)KK, (uint32_t)(R / KK)};
    hipStream_t s = as_stream(stream);
    const int64_t Rw = ceil_div(C, bits);
    const bool wide_ok = C % bits == 0 && src_vec_ok && (!thresh || aligned(thresh, 16)) &&
                         R * (C / 4) < (1LL << 30);  // 32-bit word offsets 4 * (R * C / 4) inside a member's plane
    if constexpr (std::is_same<Src, PhiloxSrc>::value) {
        if (wide_ok) {
            const uint32_t PW = (uint32_t)(R * Rw);
            // eight members per lane while that leaves two waves for every SIMD, else two
            const bool many = ceil_div(n, 8) * PW >= 131072;
            const int64_t total = ceil_div(n, many ? 8 : 2) * PW;
            const dim3 grid(grid_for(total)), block(256);
#define NB_LAUNCH_WORD(UU, T, B)                                                                                        \
    sample_word_philox_kernel<W, UU, T, B><<<grid, block, 0, s>>>(out, base, thresh, ts, src.key, n, PW, total, conv, \
                                                                 (uint32_t)Rw)
#define NB_LAUNCH_WORD_U(T, B)            \
    do {                                  \
        if (many) NB_LAUNCH_WORD(8, T, B); \
        else NB_LAUNCH_WORD(2, T, B);      \
    } while (0)
            if (thresh && base) NB_LAUNCH_WORD_U(true, true);
            else if (thresh) NB_LAUNCH_WORD_U(true, false);
            else if (base) NB_LAUNCH_WORD_U(false, true);
            else NB_LAUNCH_WORD_U(false, false);
#undef NB_LAUNCH_WORD_U
#undef NB_LAUNCH_WORD
            return check_launch(who);
        }
    }
    if (wide_ok) {
        constexpr int U = 8, BS = 1024;
        const uint32_t rc4 = (uint32_t)(R * (C / 4));
        const uint32_t plane_tiles = (uint32_t)ceil_div(rc4, BS);
        const int64_t total_blocks = ceil_div(n, U) * plane_tiles;
        const dim3 grid((unsigned)(total_blocks < kMaxBlocks ? total_blocks : kMaxBlocks)), block(BS);
#define NB_LAUNCH_WIDE(T, B)                                                                                   \
    sample_wide_kernel<W, Src, U, BS, T, B><<<grid, block, 0, s>>>(out, base, thresh, ts, src, n, rc4, plane_tiles, \
                                                                   total_blocks, conv, (uint32_t)Rw)
        if (thresh && base) NB_LAUNCH_WIDE(true, true);
        else if (thresh) NB_LAUNCH_WIDE(true, false);
        else if (base) NB_LAUNCH_WIDE(false, true);
        else NB_LAUNCH_WIDE(false, false);
#undef NB_LAUNCH_WIDE
    } else if (C < bits) {
        // rows that are whole generator blocks with 16-byte aligned thresholds (src_vec_ok: the stream starts on a block)
        const bool quads = C % 4 == 0 && src_vec_ok && (!thresh || aligned(thresh, 16));
        sample_narrow_kernel<W, Src><<<dim3(grid_for(n * R)), dim3(256), 0, s>>>(out, base, thresh, ts, src, n * R, R,
                                                                               (int)C, conv, quads);
    } else {
        sample_ballot_kernel<W, Src><<<dim3(grid_for(n * R * 64)), dim3(256), 0, s>>>(
            out, base, thresh, ts, src, n * R, R, (int)C, (int)Rw, conv);
    }
    return check_launch(who);
}

// 16-bit draws: rows of whole words, a stream that starts on a block of 8 columns, thresholds (if any) 16-byte aligned
template <typename W>
int sample16_impl(W *out, const W *base, const uint32_t *thresh, uint32_t ts, PhiloxKey key, int64_t n, int64_t R,
                  int64_t C, nb_stream_t stream, const char *who, W *out_conv = nullptr, int64_t KK = 1)
{
    constexpr int bits = WordTraits<W>::bits;
    bool empty;
    if (int rc = sample_check<W>(out ? out : out_conv, base, thresh, n, R, C, who, &empty)) return rc;
    if (empty) return NB_OK;
    NB_REQUIRE_ALIGNED(out, sizeof(W));
    NB_REQUIRE_ALIGNED(out_conv, sizeof(W));
    NB_REQUIRE(KK >= 1 && R % KK == 0 && R < (1LL << 31), "%s: %lld rows are not whole groups of %lld taps", who,
               (long long)R, (long long)KK);
    if (C % bits != 0 || (key.first & 7) != 0 || (thresh && !aligned(thresh, 16)) || R * (C / 4) >= (1LL << 30))
        return fail(NB_ERR_UNSUPPORTED,
                    "%s: 16-bit draws take rows of whole words, first %% 8 == 0 and 16-byte aligned thresholds", who);
    const ConvOut<W> conv{out_conv, (uint32_t)KK, (uint32_t)(R / KK)};
    hipStream_t s = as_stream(stream);
    const int64_t Rw = C / bits;
    const uint32_t PW = (uint32_t)(R * Rw);
    const bool many = ceil_div(n, 8) * PW >= 131072;
    const int64_t total = ceil_div(n, many ? 8 : 2) * PW;
    const dim3 grid(grid_for(total)), block(256);
#define NB_LAUNCH_WORD(UU, T, B)                                                                                       \
    sample_word_philox16_kernel<W, UU, T, B><<<grid, block, 0, s>>>(out, base, thresh, ts, key, n, PW, total, conv, \
                                                                   (uint32_t)Rw)
#define NB_LAUNCH_WORD_U(T, B)            \
    do {                                  \
        if (many) NB_LAUNCH_WORD(8, T, B); \
        else NB_LAUNCH_WORD(2, T, B);      \
    } while (0)
    if (thresh && base) NB_LAUNCH_WORD_U(true, true);
    else if (thresh) NB_LAUNCH_WORD_U(true, false);
    else if (base) NB_LAUNCH_WORD_U(false, true);
    else NB_LAUNCH_WORD_U(false, false);
#undef NB_LAUNCH_WORD_U
#undef NB_LAUNCH_WORD
    return check_launch(who);
}

// ---- fused sample + XOR-popcount with 16-bit draws -----------------------------------------------------------------
// C[m, r] = sum_k popcount(w(m, r, k) ^ x[m, k]) with w what sample_word_philox16_kernel would have written.  A wave
// takes RPW rows of one member (they share the member's input bytes); a lane takes 8 columns per step, i.e. one
// generator block per row: eight borrow/shift pairs, an XOR with the byte of base ^ x, one v_bcnt.  Needs C % 8 == 0
// and first % 8 == 0 (blocks do not straddle rows), thresholds 16-byte aligned.
template <typename W, int RPW, bool HAS_THR, bool HAS_BASE>
__global__ __launch_bounds__(256) void seeded_bmv_philox16_kernel(int32_t *__restrict__ Cout, const W *__restrict__ base,
                                                                  const uint32_t *__restrict__ thresh, uint32_t ts,
                                                                  const W *__restrict__ x, PhiloxKey key, int64_t n,
                                                                  int R, int C8, int Rw, int groups_per_member)
{
    constexpr int bits = WordTraits<W>::bits;
    constexpr int BPW = bits / 8;  // bytes (blocks of 8 columns) per word
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int64_t m = wave / groups_per_member;
    if (m >= n) return;
    const int r0 = (int)(wave - m * groups_per_member) * RPW;
    int rows[RPW];
#pragma unroll
    for (int q = 0; q < RPW; q++) rows[q] = r0 + q < R ? r0 + q : R - 1;  // tail rows are recomputed, not stored
    int acc[RPW];
#pragma unroll
    for (int q = 0; q < RPW; q++) acc[q] = 0;
    const uint64_t blk0 = key.first >> 3;
    // every lane runs the same number of steps (the tie test below is a wave-wide vote); lanes past the row's end
    // compute on the last block and add nothing
    for (int c0 = 0; c0 < C8; c0 += 64) {
        const bool live = c0 + lane < C8;
        const int c8 = live ? c0 + lane : C8 - 1;
        const int wi = c8 / BPW, sh = 8 * (c8 - wi * BPW);
        const W xw = x[m * Rw + wi];
#pragma unroll
        for (int q = 0; q < RPW; q++) {
            const int r = rows[q];
            const uint32_t bx = (uint32_t)((HAS_BASE ? (W)(xw ^ base[(int64_t)r * Rw + wi]) : xw) >> sh) & 0xFFu;
            const uint4 *tq = reinterpret_cast<const uint4 *>(thresh + ((int64_t)r * C8 + c8) * 8);
            const uint4 ta = HAS_THR ? tq[0] : make_uint4(ts, ts, ts, ts);
            const uint4 tb = HAS_THR ? tq[1] : ta;
            const uint4 ha = make_uint4(ta.x & 0xFFFF0000u, ta.y & 0xFFFF0000u, ta.z & 0xFFFF0000u, ta.w & 0xFFFF0000u);
            const uint4 hb = make_uint4(tb.x & 0xFFFF0000u, tb.y & 0xFFFF0000u, tb.z & 0xFFFF0000u, tb.w & 0xFFFF0000u);
            const uint64_t b = blk0 + (uint64_t)((m * R + r) * C8 + c8);
            const uint4 w = philox_block(key, b);
            uint32_t zmin = 0xFFFFFFFFu;
            uint32_t byte = byte_lt16(w, ha, hb, zmin);
            if (__any(zmin < 65536u)) {
                if (zmin < 65536u) byte = byte_ties16(byte, w, ta, tb, key, b << 3);
            }
            acc[q] += live ? __popc(byte ^ bx) : 0;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
#pragma unroll
        for (int q = 0; q < RPW; q++) acc[q] += __shfl_xor(acc[q], off);
    }
    if (lane == 0) {
#pragma unroll
        for (int q = 0; q < RPW; q++)
            if (r0 + q < R) Cout[m * R + r0 + q] = acc[q];
    }
}

template <typename W>
int seeded_bmv16_impl(int32_t *Cout, const W *base, const uint32_t *thresh, uint32_t ts, const W *x, PhiloxKey key,
                      int64_t n, int64_t R, int64_t C, nb_stream_t stream, const char *who)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_REQUIRE(n >= 0 && R >= 0 && C >= 0, "%s: negative shape n=%lld R=%lld C=%lld", who, (long long)n, (long long)R,
               (long long)C);
    if (n * R == 0) return NB_OK;
    NB_REQUIRE_PTR(Cout);
    NB_REQUIRE_ALIGNED(Cout, 4);
    NB_REQUIRE(C > 0 && C <= (1 << 30) && R < (1LL << 31), "%s: C=%lld, R=%lld out of range", who, (long long)C, (long long)R);
    NB_REQUIRE_PTR(x);
    NB_REQUIRE_ALIGNED(x, sizeof(W));
    if (base) NB_REQUIRE_ALIGNED(base, sizeof(W));
    if (C % 8 != 0 || (key.first & 7) != 0 || (thresh && !aligned(thresh, 16)))
        return fail(NB_ERR_UNSUPPORTED,
                    "%s: 16-bit draws take C %% 8 == 0, first %% 8 == 0 and 16-byte aligned thresholds", who);
    constexpr int RPW = 4;
    const int64_t gpm = ceil_div(R, RPW), waves = n * gpm;
    NB_REQUIRE(ceil_div(waves, 4) <= kMaxGridX, "%s: n*R=%lld rows exceed one launch", who, (long long)(n * R));
    const dim3 grid((unsigned)ceil_div(waves, 4)), block(256);
    const int Rw = (int)ceil_div(C, bits);
    hipStream_t s = as_stream(stream);
#define NB_LAUNCH16(T, B)                                                                                              \
    seeded_bmv_philox16_kernel<W, RPW, T, B><<<grid, block, 0, s>>>(Cout, base, thresh, ts, x, key, n, (int)R, (int)(C / 8), \
                                                                    Rw, (int)gpm)
    if (thresh && base) NB_LAUNCH16(true, true);
    else if (thresh) NB_LAUNCH16(true, false);
    else if (base) NB_LAUNCH16(false, true);
    else NB_LAUNCH16(false, false);
#undef NB_LAUNCH16
    return check_launch(who);
}

template <typename W, class Src>
int seeded_bmv_impl(int32_t *Cout, const W *base, const uint32_t *thresh, uint32_t ts, const W *x, Src src,
                    bool src_vec_ok, int64_t n, int64_t R, int64_t C, nb_stream_t stream, const char *who)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_REQUIRE(n >= 0 && R >= 0 && C >= 0, "%s: negative shape n=%lld R=%lld C=%lld", who, (long long)n, (long long)R,
               (long long)C);
    if (n * R == 0) return NB_OK;
    NB_REQUIRE_PTR(Cout);
    NB_REQUIRE_ALIGNED(Cout, 4);
    NB_REQUIRE(C <= (1 << 30), "%s: C=%lld too large", who, (long long)C);
    NB_REQUIRE(n * R <= (1LL << 40) && ceil_div(n * R, 4) <= kMaxGridX, "%s: n*R=%lld rows exceed one launch", who,
               (long long)(n * R));
    if (C > 0) {
        NB_REQUIRE_PTR(x);
        NB_REQUIRE_ALIGNED(x, sizeof(W));
    }
    if (base) NB_REQUIRE_ALIGNED(base, sizeof(W));
    if (thresh) NB_REQUIRE_ALIGNED(thresh, 4);
    hipStream_t s = as_stream(stream);
    const int64_t Rw = ceil_div(C, bits);
    constexpr int RPW = 4;
    const bool vec_ok = C > 0 && (C & 3) == 0 && src_vec_ok && (!thresh || aligned(thresh, 16));
    if (vec_ok && (C & 255) == 0 && n * R < (1LL << 31) && ceil_div(n * R, 16) <= kMaxBlocks) {
        const int64_t it = C / 256;  // wave-steps per row
        if ((it & 7) == 0) launch_bmv_stream<W, Src, 1, 8>(Cout, base, thresh, ts, x, src, n, R, C, (int)Rw, s);
        else if ((it & 3) == 0) launch_bmv_stream<W, Src, 2, 4>(Cout, base, thresh, ts, x, src, n, R, C, (int)Rw, s);
        else if ((it & 1) == 0) launch_bmv_stream<W, Src, 4, 2>(Cout, base, thresh, ts, x, src, n, R, C, (int)Rw, s);
        else launch_bmv_stream<W, Src, 8, 1>(Cout, base, thresh, ts, x, src, n, R, C, (int)Rw, s);
    } else if (vec_ok) {
        const int64_t gpm = ceil_div(R, RPW);
        const int64_t waves = n * gpm;
        seeded_bmv_wide_kernel<W, Src, RPW><<<dim3((unsigned)ceil_div(waves, 4)), dim3(256), 0, s>>>(
            Cout, base, thresh, ts, x, src, n, R, (int)(C / 4), (int)Rw, gpm);
    } else {
        seeded_bmv_generic_kernel<W, Src><<<dim3((unsigned)ceil_div(n * R, 4)), dim3(256), 0, s>>>(
            Cout, base, thresh, ts, x, src, n * R, R, (int)C, (int)Rw);
    }
    return check_launch(who);
}

// Probabilities -> sampler thresholds: T = min(floor(p * 2^32), 2^32 - 1), 0 for p <= 0 and for NaN.  p is fp16 (11
// significant bits), so p * 2^32 is exact in fp32.
__global__ __launch_bounds__(256) void thresholds_from_p_kernel(uint32_t *__restrict__ T, const _Float16 *__restrict__ P,
                                                                int64_t n)
{
    NB_FLAT_LOOP(i, n)
    {
        if (i < n) {
            const float v = (float)P[i] * 4294967296.0f;
            T[i] = v >= 4294967295.0f ? 0xFFFFFFFFu : (v > 0.0f ? (uint32_t)floorf(v) : 0u);
        }
    }
}

}  // namespace nb

using nb::PhiloxSrc;
using nb::WordsSrc;
#define U64(p) reinterpret_cast<uint64_t *>(p)
#define U32(p) reinterpret_cast<uint32_t *>(p)
#define CU64(p) reinterpret_cast<const uint64_t *>(p)
#define CU32(p) reinterpret_cast<const uint32_t *>(p)

extern "C" {
int nb_sample_from_words_i64(int64_t *out, const int64_t *base, const uint32_t *thresh, uint32_t ts,
                             const uint32_t *words, int64_t n, int64_t R, int64_t C, nb_stream_t s)
{
    if (n * R * C > 0 && !words) return nb::fail(NB_ERR_NULL, "nb_sample_from_words_i64: words is NULL");
    return nb::sample_impl<uint64_t, WordsSrc>(U64(out), CU64(base), thresh, ts, WordsSrc{words},
                                               nb::aligned(words, 16) && (C & 3) == 0, n, R, C, s,
                                               "nb_sample_from_words_i64");
}
int nb_sample_from_words_i32(int32_t *out, const int32_t *base, const uint32_t *thresh, uint32_t ts,
                             const uint32_t *words, int64_t n, int64_t R, int64_t C, nb_stream_t s)
{
    if (n * R * C > 0 && !words) return nb::fail(NB_ERR_NULL, "nb_sample_from_words_i32: words is NULL");
    return nb::sample_impl<uint32_t, WordsSrc>(U32(out), CU32(base), thresh, ts, WordsSrc{words},
                                               nb::aligned(words, 16) && (C & 3) == 0, n, R, C, s,
                                               "nb_sample_from_words_i32");
}
int nb_sample_philox_i64(int64_t *out, const int64_t *base, const uint32_t *thresh, uint32_t ts, uint64_t seed,
                         uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t C, nb_stream_t s)
{
    return nb::sample_impl<uint64_t, PhiloxSrc>(U64(out), CU64(base), thresh, ts, PhiloxSrc{{seed, subseq, first}},
                                                (first & 3) == 0 && (C & 3) == 0, n, R, C, s, "nb_sample_philox_i64");
}
int nb_sample_philox_i32(int32_t *out, const int32_t *base, const uint32_t *thresh, uint32_t ts, uint64_t seed,
                         uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t C, nb_stream_t s)
{
    return nb::sample_impl<uint32_t, PhiloxSrc>(U32(out), CU32(base), thresh, ts, PhiloxSrc{{seed, subseq, first}},
                                                (first & 3) == 0 && (C & 3) == 0, n, R, C, s, "nb_sample_philox_i32");
}
int nb_sample_philox16_i64(int64_t *out, const int64_t *base, const uint32_t *thresh, uint32_t ts, uint64_t seed,
                           uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t C, nb_stream_t s)
{
    return nb::sample16_impl<uint64_t>(U64(out), CU64(base), thresh, ts, nb::PhiloxKey{seed, subseq, first}, n, R, C, s,
                                       "nb_sample_philox16_i64");
}
int nb_sample_philox16_i32(int32_t *out, const int32_t *base, const uint32_t *thresh, uint32_t ts, uint64_t seed,
                           uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t C, nb_stream_t s)
{
    return nb::sample16_impl<uint32_t>(U32(out), CU32(base), thresh, ts, nb::PhiloxKey{seed, subseq, first}, n, R, C, s,
                                       "nb_sample_philox16_i32");
}
int nb_sample_conv_philox16_i64(int64_t *out_conv, int64_t *out_rows, const int64_t *base, const uint32_t *thresh,
                                uint32_t ts, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t O,
                                int64_t KK, int64_t C, nb_stream_t s)
{
    const char *who = "nb_sample_conv_philox16_i64";
    if (O < 0 || KK < 1) return nb::fail(NB_ERR_SHAPE, "%s: bad shape O=%lld KK=%lld", who, (long long)O, (long long)KK);
    if (n * O * KK * C > 0 && !out_conv) return nb::fail(NB_ERR_NULL, "%s: out_conv is NULL", who);
    return nb::sample16_impl<uint64_t>(U64(out_rows), CU64(base), thresh, ts, nb::PhiloxKey{seed, subseq, first}, n,
                                       O * KK, C, s, who, U64(out_conv), KK);
}
int nb_sample_conv_philox16_i32(int32_t *out_conv, int32_t *out_rows, const int32_t *base, const uint32_t *thresh,
                                uint32_t ts, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t O,
                                int64_t KK, int64_t C, nb_stream_t s)
{
    const char *who = "nb_sample_conv_philox16_i32";
    if (O < 0 || KK < 1) return nb::fail(NB_ERR_SHAPE, "%s: bad shape O=%lld KK=%lld", who, (long long)O, (long long)KK);
    if (n * O * KK * C > 0 && !out_conv) return nb::fail(NB_ERR_NULL, "%s: out_conv is NULL", who);
    return nb::sample16_impl<uint32_t>(U32(out_rows), CU32(base), thresh, ts, nb::PhiloxKey{seed, subseq, first}, n,
                                       O * KK, C, s, who, U32(out_conv), KK);
}
int nb_sample_conv_from_words_i64(int64_t *out_conv, int64_t *out_rows, const int64_t *base, const uint32_t *thresh,
                                  uint32_t ts, const uint32_t *words, int64_t n, int64_t O, int64_t KK, int64_t C,
                                  nb_stream_t s)
{
    const char *who = "nb_sample_conv_from_words_i64";
    if (O < 0 || KK < 1) return nb::fail(NB_ERR_SHAPE, "%s: bad shape O=%lld KK=%lld", who, (long long)O, (long long)KK);
    if (n * O * KK * C > 0 && !words) return nb::fail(NB_ERR_NULL, "%s: words is NULL", who);
    if (n * O * KK * C > 0 && !out_conv) return nb::fail(NB_ERR_NULL, "%s: out_conv is NULL", who);
    return nb::sample_impl<uint64_t, WordsSrc>(U64(out_rows), CU64(base), thresh, ts, WordsSrc{words},
                                               nb::aligned(words, 16) && (C & 3) == 0, n, O * KK, C, s, who,
                                               U64(out_conv), KK);
}
int nb_sample_conv_from_words_i32(int32_t *out_conv, int32_t *out_rows, const int32_t *base, const uint32_t *thresh,
                                  uint32_t ts, const uint32_t *words, int64_t n, int64_t O, int64_t KK, int64_t C,
                                  nb_stream_t s)
{
    const char *who = "nb_sample_conv_from_words_i32";
    if (O < 0 || KK < 1) return nb::fail(NB_ERR_SHAPE, "%s: bad shape O=%lld KK=%lld", who, (long long)O, (long long)KK);
    if (n * O * KK * C > 0 && !words) return nb::fail(NB_ERR_NULL, "%s: words is NULL", who);
    if (n * O * KK * C > 0 && !out_conv) return nb::fail(NB_ERR_NULL, "%s: out_conv is NULL", who);
    return nb::sample_impl<uint32_t, WordsSrc>(U32(out_rows), CU32(base), thresh, ts, WordsSrc{words},
                                               nb::aligned(words, 16) && (C & 3) == 0, n, O * KK, C, s, who,
                                               U32(out_conv), KK);
}
int nb_sample_conv_philox_i64(int64_t *out_conv, int64_t *out_rows, const int64_t *base, const uint32_t *thresh,
                              uint32_t ts, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t O,
                              int64_t KK, int64_t C, nb_stream_t s)
{
    const char *who = "nb_sample_conv_philox_i64";
    if (O < 0 || KK < 1) return nb::fail(NB_ERR_SHAPE, "%s: bad shape O=%lld KK=%lld", who, (long long)O, (long long)KK);
    if (n * O * KK * C > 0 && !out_conv) return nb::fail(NB_ERR_NULL, "%s: out_conv is NULL", who);
    return nb::sample_impl<uint64_t, PhiloxSrc>(U64(out_rows), CU64(base), thresh, ts, PhiloxSrc{{seed, subseq, first}},
                                                (first & 3) == 0 && (C & 3) == 0, n, O * KK, C, s, who, U64(out_conv),
                                                KK);
}
int nb_sample_conv_philox_i32(int32_t *out_conv, int32_t *out_rows, const int32_t *base, const uint32_t *thresh,
                              uint32_t ts, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t O,
                              int64_t KK, int64_t C, nb_stream_t s)
{
    const char *who = "nb_sample_conv_philox_i32";
    if (O < 0 || KK < 1) return nb::fail(NB_ERR_SHAPE, "%s: bad shape O=%lld KK=%lld", who, (long long)O, (long long)KK);
    if (n * O * KK * C > 0 && !out_conv) return nb::fail(NB_ERR_NULL, "%s: out_conv is NULL", who);
    return nb::sample_impl<uint32_t, PhiloxSrc>(U32(out_rows), CU32(base), thresh, ts, PhiloxSrc{{seed, subseq, first}},
                                                (first & 3) == 0 && (C & 3) == 0, n, O * KK, C, s, who, U32(out_conv),
                                                KK);
}
int nb_philox_words(uint32_t *out, uint64_t seed, uint64_t subseq, uint64_t first, int64_t count, nb_stream_t s)
{
    if (count < 0) return nb::fail(NB_ERR_SHAPE, "nb_philox_words: negative count");
    if (count == 0) return NB_OK;
    if (!out) return nb::fail(NB_ERR_NULL, "nb_philox_words: out is NULL");
    if (!nb::aligned(out, 4)) return nb::fail(NB_ERR_ALIGN, "nb_philox_words: out is not 4-byte aligned");
    const int64_t blocks4 = (int64_t)(((first + (uint64_t)count + 3) >> 2) - (first >> 2));
    nb::philox_words_kernel<<<dim3(nb::grid_for(blocks4)), dim3(256), 0, nb::as_stream(s)>>>(
        out, nb::PhiloxKey{seed, subseq, first}, count);
    return nb::check_launch("nb_philox_words");
}
int nb_seeded_bmv_from_words_i64(int32_t *C, const int64_t *base, const uint32_t *thresh, uint32_t ts, const int64_t *x,
                                 const uint32_t *words, int64_t n, int64_t R, int64_t Cbits, nb_stream_t s)
{
    if (n * R * Cbits > 0 && !words) return nb::fail(NB_ERR_NULL, "nb_seeded_bmv_from_words_i64: words is NULL");
    return nb::seeded_bmv_impl<uint64_t, WordsSrc>(C, CU64(base), thresh, ts, CU64(x), WordsSrc{words},
                                                   nb::aligned(words, 16), n, R, Cbits, s,
                                                   "nb_seeded_bmv_from_words_i64");
}
int nb_seeded_bmv_from_words_i32(int32_t *C, const int32_t *base, const uint32_t *thresh, uint32_t ts, const int32_t *x,
                                 const uint32_t *words, int64_t n, int64_t R, int64_t Cbits, nb_stream_t s)
{
    if (n * R * Cbits > 0 && !words) return nb::fail(NB_ERR_NULL, "nb_seeded_bmv_from_words_i32: words is NULL");
    return nb::seeded_bmv_impl<uint32_t, WordsSrc>(C, CU32(base), thresh, ts, CU32(x), WordsSrc{words},
                                                   nb::aligned(words, 16), n, R, Cbits, s,
                                                   "nb_seeded_bmv_from_words_i32");
}
int nb_seeded_bmv_philox16_i64(int32_t *C, const int64_t *base, const uint32_t *thresh, uint32_t ts, const int64_t *x,
                               uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t Cbits,
                               nb_stream_t s)
{
    return nb::seeded_bmv16_impl<uint64_t>(C, CU64(base), thresh, ts, CU64(x), nb::PhiloxKey{seed, subseq, first}, n, R,
                                           Cbits, s, "nb_seeded_bmv_philox16_i64");
}
int nb_seeded_bmv_philox16_i32(int32_t *C, const int32_t *base, const uint32_t *thresh, uint32_t ts, const int32_t *x,
                               uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t Cbits,
                               nb_stream_t s)
{
    return nb::seeded_bmv16_impl<uint32_t>(C, CU32(base), thresh, ts, CU32(x), nb::PhiloxKey{seed, subseq, first}, n, R,
                                           Cbits, s, "nb_seeded_bmv_philox16_i32");
}
int nb_seeded_bmv_philox_i64(int32_t *C, const int64_t *base, const uint32_t *thresh, uint32_t ts, const int64_t *x,
                             uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t Cbits,
                             nb_stream_t s)
{
    return nb::seeded_bmv_impl<uint64_t, PhiloxSrc>(C, CU64(base), thresh, ts, CU64(x),
                                                    PhiloxSrc{{seed, subseq, first}}, (first & 3) == 0, n, R, Cbits, s,
                                                    "nb_seeded_bmv_philox_i64");
}
int nb_seeded_bmv_philox_i32(int32_t *C, const int32_t *base, const uint32_t *thresh, uint32_t ts, const int32_t *x,
                             uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t Cbits,
                             nb_stream_t s)
{
    return nb::seeded_bmv_impl<uint32_t, PhiloxSrc>(C, CU32(base), thresh, ts, CU32(x),
                                                    PhiloxSrc{{seed, subseq, first}}, (first & 3) == 0, n, R, Cbits, s,
                                                    "nb_seeded_bmv_philox_i32");
}
int nb_thresholds_from_p(uint32_t *T, const uint16_t *P, int64_t n, nb_stream_t stream)
{
    const char *who = "nb_thresholds_from_p";
    NB_REQUIRE(n >= 0 && n < (1LL << 40), "%s: bad count %lld", who, (long long)n);
    if (n == 0) return NB_OK;
    NB_REQUIRE_PTR(T);
    NB_REQUIRE_PTR(P);
    NB_REQUIRE_ALIGNED(T, 4);
    NB_REQUIRE_ALIGNED(P, 2);
    nb::thresholds_from_p_kernel<<<dim3(nb::grid_for(n)), dim3(256), 0, nb::as_stream(stream)>>>(
        T, reinterpret_cast<const _Float16 *>(P), n);
    return nb::check_launch(who);
}
}
