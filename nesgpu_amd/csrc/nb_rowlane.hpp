// "Row per lane" XOR-popcount tile kernel shared by bmm and the implicit-im2col conv.
//
// Mapping: one lane owns one row x of the product (an output pixel for conv) and keeps that
// row's packed words a[k] in VGPRs.  All lanes of a workgroup belong to the same member z, so
// the second operand B[z,k,y] is wave-uniform: the compiler fetches it with scalar loads and
// feeds it to v_xor_b32 as an SGPR operand -- no LDS staging and no per-lane traffic for B.
// Per 64-bit word and output the VALU work is 2 v_xor_b32 + 2 accumulating v_bcnt_u32_b32.
#pragma once
#include "nb_common.hpp"

namespace nb {

// ---- A-operand loaders ---------------------------------------------------------------------
// Explicit rows: A [Z, M, Kw].
template <typename W>
struct RowsA {
    const W *__restrict__ A;
    int64_t M;
    int Kw;
    struct Lane {
        const W *row;
        bool valid;
    };
    __device__ __forceinline__ Lane lane(int64_t z, int64_t m) const
    {
        Lane l;
        l.valid = m < M;
        l.row = A + (z * M + (l.valid ? m : 0)) * Kw;
        return l;
    }
    template <int KC>
    __device__ __forceinline__ void load(const Lane &l, int k0, W (&a)[KC]) const
    {
#pragma unroll
        for (int i = 0; i < KC; i++) a[i] = (l.valid && k0 + i < Kw) ? l.row[k0 + i] : (W)0;
    }
};

// Implicit im2col: input [D, H, W, Cw]; word k of output pixel (yo, xo) is channel word k%Cw
// of tap k/Cw = i*fy + j at input position (i + yo*sx - px, j + xo*sy - py), zero outside
// (extensions/src/batch_im2col.cu:14-29).
struct ConvGeom {
    int H, Wd, Cw, fx, fy, px, py, sx, sy, h, w;
};

template <typename W>
struct ConvA {
    const W *__restrict__ in;
    ConvGeom g;
    struct Lane {
        const W *img;
        int y0, x0;
        bool valid;
    };
    // (yo, xo) output pixel of this lane
    __device__ __forceinline__ Lane lane_at(int64_t z, int yo, int xo, bool valid) const
    {
        Lane l;
        l.valid = valid;
        l.img = in + z * (int64_t)g.H * g.Wd * g.Cw;
        l.y0 = yo * g.sx - g.px;
        l.x0 = xo * g.sy - g.py;
        return l;
    }
    template <int KC>
    __device__ __forceinline__ void load(const Lane &l, int k0, W (&a)[KC]) const
    {
        const int Kw = g.fx * g.fy * g.Cw;
        // tap counters for k0, then advanced incrementally (all wave-uniform)
        const int cw = g.Cw > 0 ? g.Cw : 1;
        int tap = k0 / cw;
        int c = k0 - tap * cw;
        int ti = tap / g.fy;
        int tj = tap - ti * g.fy;
#pragma unroll
        for (int i = 0; i < KC; i++) {
            const int y = l.y0 + ti, x = l.x0 + tj;
            const bool ok = l.valid && (k0 + i < Kw) && y >= 0 && y < g.H && x >= 0 && x < g.Wd;
            a[i] = ok ? l.img[((int64_t)y * g.Wd + x) * g.Cw + c] : (W)0;
            if (++c == g.Cw) {
                c = 0;
                if (++tj == g.fy) {
                    tj = 0;
                    ++ti;
                }
            }
        }
    }
};

// Implicit im2col with TAP PACKING for narrow channels (Cw == 1, tap_bits = true channel count <= bits/2):
// T = bits / tap_bits taps share one word, word w of an output pixel is OR_t tap(w*T + t) << (tap_bits*t).
// The filter must be packed the same way (tap_pack_filter_kernel).  The popcount sum is unchanged because
// both operands are zero above tap_bits (extensions/src/pack.cu:17; input bits above them are masked off here, so a
// stray bit counts for nothing, as in the matrix-core kernels) and an out-of-range tap is the zero word.
template <typename W>
struct ConvTapA {
    const W *__restrict__ in;
    ConvGeom g;
    int tap_bits, T;
    typedef typename ConvA<W>::Lane Lane;
    __device__ __forceinline__ Lane lane_at(int64_t z, int yo, int xo, bool valid) const
    {
        Lane l;
        l.valid = valid;
        l.img = in + z * (int64_t)g.H * g.Wd;
        l.y0 = yo * g.sx - g.px;
        l.x0 = xo * g.sy - g.py;
        return l;
    }
    template <int KC>
    __device__ __forceinline__ void load(const Lane &l, int k0, W (&a)[KC]) const
    {
        const int taps = g.fx * g.fy;
        const W cmask = (W)(((W)1 << tap_bits) - 1);
        int tap = k0 * T;
        int ti = tap / g.fy;
        int tj = tap - ti * g.fy;
#pragma unroll
        for (int i = 0; i < KC; i++) {
            W wv = 0;
            for (int t = 0; t < T && tap < taps; t++, tap++) {
                const int y = l.y0 + ti, x = l.x0 + tj;
                const bool ok = l.valid && y >= 0 && y < g.H && x >= 0 && x < g.Wd;
                const W v = ok ? (l.img[(int64_t)y * g.Wd + x] & cmask) : (W)0;
                wv |= v << (tap_bits * t);
                if (++tj == g.fy) {
                    tj = 0;
                    ++ti;
                }
            }
            a[i] = wv;
        }
    }
};

// ---- accumulate one K-chunk into an N-tile ----------------------------------------------------
// EXACT: the chunk is complete (k0 + KC <= Kw), so the k-steps carry no guards and the scalar loads of
// later steps can be issued while earlier steps compute.
template <typename W, int KC, int NT, bool EXACT>
__device__ __forceinline__ void mac_chunk(int (&acc)[NT], const W (&a)[KC], const W *__restrict__ Bz, int k0, int Kw,
                                          int n0, int N)
{
    if (EXACT && n0 + NT <= N) {
        // software pipeline over k: the scalar loads of step i+1 are issued before step i computes
        const W *__restrict__ brow = Bz + (int64_t)k0 * N + n0;
        W bcur[NT], bnxt[NT];
#pragma unroll
        for (int j = 0; j < NT; j++) bcur[j] = brow[j];
#pragma unroll
        for (int i = 0; i < KC; i++) {
            if (i + 1 < KC) {
#pragma unroll
                for (int j = 0; j < NT; j++) bnxt[j] = brow[(int64_t)(i + 1) * N + j];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NT; j++) acc_popc_xor(acc[j], a[i], bcur[j]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < NT; j++) bcur[j] = bnxt[j];
        }
    } else if (n0 + NT <= N) {
#pragma unroll
        for (int i = 0; i < KC; i++) {
            if (EXACT || k0 + i < Kw) {
                const W *__restrict__ brow = Bz + (int64_t)(k0 + i) * N + n0;
#pragma unroll
                for (int j = 0; j < NT; j++) acc_popc_xor(acc[j], a[i], brow[j]);
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < KC; i++) {
            if (EXACT || k0 + i < Kw) {
                const W *__restrict__ brow = Bz + (int64_t)(k0 + i) * N + n0;
#pragma unroll
                for (int j = 0; j < NT; j++)
                    if (n0 + j < N) acc_popc_xor(acc[j], a[i], brow[j]);
            }
        }
    }
}

// ---- epilogues -----------------------------------------------------------------------------------
// int32 popcount sums, C [Z, M, N].  A full N-tile is transposed through LDS so that every store
// instruction of a wave writes whole 64-byte row segments (4 lanes x int4 per row), and the stores are
// non-temporal: the output is written once and never re-read by this kernel.  The lanes of a wave own
// consecutive rows (row - lane is the wave's first row).
typedef int nb_i32x4 __attribute__((ext_vector_type(4)));
struct EpiI32 {
    int32_t *__restrict__ C;
    bool vec;  // rows are 16-byte aligned and N % 4 == 0
    struct State {};
    template <int NT>
    __device__ __forceinline__ void tile(State &, int64_t row, bool valid, int64_t z, int n0, int N,
                                         const int (&acc)[NT]) const
    {
        static_assert(NT == 16, "the transposed store assumes 16-wide tiles");
        const int wv = threadIdx.x >> 6, lane = threadIdx.x & 63;
        const bool full = __all(valid);
        if (n0 + NT <= N && vec && full) {
            __shared__ int stage[4][64][NT + 1];  // +1: conflict-free column writes
#pragma unroll
            for (int j = 0; j < NT; j++) stage[wv][lane][j] = acc[j];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const int64_t row0 = row - lane;
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const int r = p * 16 + (lane >> 2), c = (lane & 3) * 4;
                const nb_i32x4 v = {stage[wv][r][c], stage[wv][r][c + 1], stage[wv][r][c + 2], stage[wv][r][c + 3]};
                __builtin_nontemporal_store(v, reinterpret_cast<nb_i32x4 *>(C + (row0 + r) * N + n0 + c));
            }
            __builtin_amdgcn_wave_barrier();
            return;
        }
        if (!valid) return;
        int32_t *dst = C + row * N + n0;
#pragma unroll
        for (int j = 0; j < NT; j++)
            if (n0 + j < N) dst[j] = acc[j];
    }
    __device__ __forceinline__ void finish(State &, int64_t, bool) const {}
};

// popcount sums added up over the rows of a member: S [Z, N] (zeroed beforehand), one atomic add per wave and
// column.  Every lane of a wave works on the same member z.
struct EpiSum {
    int32_t *__restrict__ S;
    struct State {};
    template <int NT>
    __device__ __forceinline__ void tile(State &, int64_t, bool valid, int64_t z, int n0, int N,
                                         const int (&acc)[NT]) const
    {
#pragma unroll
        for (int j = 0; j < NT; j++) {
            int v = valid ? acc[j] : 0;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
            if ((threadIdx.x & 63) == 0 && n0 + j < N) atomicAdd(S + z * N + n0 + j, v);
        }
    }
    __device__ __forceinline__ void finish(State &, int64_t, bool) const {}
};

// bool bytes (2*popc > thresh[z,y]), C [Z, M, N]   (extensions/src/bmm_act.cu:56)
struct EpiBool {
    uint8_t *__restrict__ C;
    const int32_t *__restrict__ thresh;
    bool vec;  // rows are 4-byte aligned and N % 4 == 0: store four bools per dword
    struct State {};
    template <int NT>
    __device__ __forceinline__ void tile(State &, int64_t row, bool valid, int64_t z, int n0, int N,
                                         const int (&acc)[NT]) const
    {
        const int32_t *__restrict__ t = thresh + z * N + n0;
        uint8_t *dst = C + row * N + n0;
        if (n0 + NT <= N && vec) {
#pragma unroll
            for (int j = 0; j < NT; j += 4) {
                uint32_t v = 0;
#pragma unroll
                for (int q = 0; q < 4; q++) v |= (uint32_t)(2 * acc[j + q] > t[j + q]) << (8 * q);
                if (valid) *reinterpret_cast<uint32_t *>(dst + j) = v;
            }
        } else {
#pragma unroll
            for (int j = 0; j < NT; j++)
                if (n0 + j < N && valid) dst[j] = (uint8_t)(2 * acc[j] > t[j]);
        }
    }
    __device__ __forceinline__ void finish(State &, int64_t, bool) const {}
};

// Threshold bits packed along y into words, out [rows, Ow]; with POOL the four lanes of a quad
// hold the 2x2 window of one pooled pixel and their words are ORed before lane 0 stores
// (extensions/src/bmm_act.cu:56 + extensions/src/pack.cu:26 + extensions/src/max_pool2d.cu:19-32).
template <typename W, bool POOL>
struct EpiPack {
    W *__restrict__ out;
    const int32_t *__restrict__ thresh;
    int Ow;
    struct State {
        uint32_t cur = 0;   // the 32-bit half being filled
        uint32_t lo = 0;    // finished low half of a 64-bit word
    };
    template <int NT>
    __device__ __forceinline__ void tile(State &st, int64_t row, bool valid, int64_t z, int n0, int N,
                                         const int (&acc)[NT]) const
    {
        constexpr int bits = WordTraits<W>::bits;
        static_assert(32 % NT == 0, "an N-tile must not straddle two 32-bit halves");
        const int32_t *__restrict__ t = thresh + z * N + n0;
        const int sh = n0 & 31;
        // 2*popc > t  <=>  popc > (t >> 1) for every integer t (arithmetic shift)
        if (n0 + NT <= N) {
#pragma unroll
            for (int j = 0; j < NT; j++) st.cur |= (uint32_t)(acc[j] > (t[j] >> 1)) << (sh + j);
        } else {
#pragma unroll
            for (int j = 0; j < NT; j++)
                if (n0 + j < N) st.cur |= (uint32_t)(acc[j] > (t[j] >> 1)) << (sh + j);
        }
        const bool last = n0 + NT >= N;
        if (((n0 + NT) & 31) == 0 || last) {               // a 32-bit half is complete
            const bool high = bits == 64 && ((n0 >> 5) & 1);
            if (bits == 64 && !high && !last) {            // low half of a 64-bit word: keep it, go on
                st.lo = st.cur;
                st.cur = 0;
                return;
            }
            W v = bits == 64 ? (W)(((uint64_t)(high ? st.cur : 0u) << 32) | (high ? st.lo : st.cur)) : (W)st.cur;
            v = valid ? v : (W)0;
            bool writer = valid;
            if (POOL) {
                v = or_reduce_group<4>(v);
                writer = valid && (threadIdx.x & 3) == 0;
            }
            if (writer) out[row * Ow + n0 / bits] = v;
            st.cur = 0;
            st.lo = 0;
        }
    }
    __device__ __forceinline__ void finish(State &, int64_t, bool) const {}
};

// The loop nest shared by every row-per-lane kernel.
// SINGLE: Kw <= KC (one chunk, A words stay in registers for every N-tile); EXACT: Kw == KC.
template <typename W, int KC, int NT, bool SINGLE, bool EXACT, class ALoad, class Epi>
__device__ __forceinline__ void rowlane_body(const ALoad &al, const typename ALoad::Lane &lane,
                                             const W *__restrict__ Bz, const Epi &epi, int64_t orow, int64_t z,
                                             int Kw, int N)
{
    typename Epi::State st;
    W a[KC];
    if (SINGLE) al.template load<KC>(lane, 0, a);
    for (int n0 = 0; n0 < N; n0 += NT) {
        int acc[NT];
#pragma unroll
        for (int j = 0; j < NT; j++) acc[j] = 0;
        if (SINGLE) {
            mac_chunk<W, KC, NT, EXACT>(acc, a, Bz, 0, Kw, n0, N);
        } else {
            int k0 = 0;
            for (; k0 + KC <= Kw; k0 += KC) {
                al.template load<KC>(lane, k0, a);
                mac_chunk<W, KC, NT, true>(acc, a, Bz, k0, Kw, n0, N);
            }
            if (k0 < Kw) {
                al.template load<KC>(lane, k0, a);
                mac_chunk<W, KC, NT, false>(acc, a, Bz, k0, Kw, n0, N);
            }
        }
        epi.template tile<NT>(st, orow, lane.valid, z, n0, N, acc);
    }
    epi.finish(st, orow, lane.valid);
}

}  // namespace nb
