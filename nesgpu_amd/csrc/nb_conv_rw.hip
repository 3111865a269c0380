// Binary conv on the int8 matrix cores, row-walking variant (3-row filters, stride 1).
//
// CDNA4 has no 1-bit MFMA, but v_mfma_i32_16x16x64_i8 does 16384 int8 MACs per wave in 16 cycles: 4x the
// bit-MAC rate of v_xor + v_bcnt.  Bits are expanded to +-1 bytes (bit 1 -> +1, bit 0 -> -1; an out-of-range
// pixel is the zero word, i.e. all -1), the int32 dot product over the K expanded positions is exact, and
//     popcount(x ^ w) = (K - dot) / 2
// gives back the reference's sum bit for bit.
//
// Work split.  A workgroup owns a band of output rows of one member; the band's input rows (with the zero-word
// border, so the implicit im2col needs no bounds checks) are expanded once into LDS.  A wave owns a strip of 16
// output columns, 16*NT output channels and a sub-band of rows.  It builds its filter fragments straight from
// global memory into registers (no LDS staging) and then walks DOWN the strip: the A fragment of image row r and
// tap column j is the same 16 pixels x 64 positions whichever filter row it meets, so it is read from LDS once
// and multiplied into the three output rows r, r-1, r-2 that are live in a ring of three accumulator sets.  One
// ds_read_b128 therefore feeds 3*NT MFMAs and the LDS pipe stays far from its limit even for 16 channels.
// Finished rows leave through the epilogue straight to global memory: int32 sums via a per-wave LDS transpose
// (full pixel rows, non-temporal), or threshold bits gathered with ballots into packed words, optionally
// 2x2 OR-pooled (pooling in x is a min over neighbouring accumulator registers, in y over two walked rows).
//
// Fragment layout of v_mfma_i32_16x16x64_i8 (checked on hardware): lane l supplies row l%16 of A and
// column l%16 of B, its 16 bytes are the K-positions 16*(l/16)..+15 of the 64-chunk (any bijection works as
// long as A and B use the same one), and acc[r] is D[4*(l/16) + r][l%16].
//
// K chunks of one filter row (the per-pixel byte count CB is 16, 32 or 64*Cw):
//   CB = 16: one chunk, lane group g holds tap column g (up to 4 columns);
//   CB = 32: chunk q holds tap columns 2q and 2q+1, 32 positions each;
//   CB >= 64: one chunk per (tap column, 64-position channel word).
// Chunks of tap columns past the filter width multiply by zero bytes.
#include "nb_conv_common.hpp"

namespace nb {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kRwThreads = 256;
constexpr int kRwWaves = kRwThreads / 64;
constexpr int kRwLutBytes = 256;  // 4 bits -> 4 bytes of +-1, four interleaved copies
constexpr int kRwMaxCPR = 6;
constexpr int kRwTabBytes = 3 * kRwMaxCPR * 4 * 8;  // (chunk, lane group) -> filter word offset, shift, mask

struct RwConv {
    const uint64_t *in;
    const uint64_t *filt;
    const int32_t *thresh;
    void *out;
    int H, Wd, Cw, px, py, h, w, O, fy;
    int CB;            // expanded bytes per pixel: 16, 32 or 64*Cw
    int PS;            // pixel stride in the LDS image, bytes (PS/16 odd: conflict-free 16-lane b128 reads)
    int RW;            // pixels per LDS image row
    int hs, S;         // output rows per band, bands per member
    int hb, nsub;      // output rows per sub-band (even), sub-bands per band
    int cgl, ngw;      // channel groups per workgroup, workgroups per band
    int bst_off;       // LDS offset of the filter-fragment staging area (the image area itself when cgl == 1)
    int ntx, ncg;      // 16-column strips, channel groups of 16*NT
    int K;             // expanded positions that count: taps * CB
    int in_bits;       // valid channel bits per pixel
    int tapT, tapM;    // tap-packed filter: taps per word and ceil(65536 / tapT) + 1 (0: one word per tap and channel word)
    int img_bytes;
    int fwords;        // filter words per member
    int pix_q, pix_r;  // threads / RW and % RW: image-pixel advance of one fill pass
    short qj[kRwMaxCPR];  // chunk q of a filter row: first tap column ...
    short qc[kRwMaxCPR];  // ... and first position inside the pixel
    int jsh, cmask;    // lane group g adds (g >> jsh) tap columns and 16 * (g & cmask) positions
};

// 4 bits -> 4 bytes of +-1 (bit j -> byte j): 1 -> 0x01, 0 -> 0xFF
__device__ __forceinline__ uint32_t rw_pm1_bytes(uint32_t nib)
{
    const uint32_t s1 = (nib << 7) | nib;
    const uint32_t s2 = (s1 << 14) | s1;
    const uint32_t u = ~s2 & 0x01010101u;        // 1 where the bit is 0
    return ((u << 8) - (u << 1)) | 0x01010101u;  // 0xFE where the bit is 0, then | 1
}

__device__ __forceinline__ uint64_t rw_sel4(int r, uint64_t a, uint64_t b, uint64_t c, uint64_t d)
{
    return r == 0 ? a : r == 1 ? b : r == 2 ? c : d;
}

// MODE 0: int32 popcount sums [D,h,w,O]; 2: threshold bits packed along O; 3: the same, 2x2 OR-pooled.
template <int CPR, int NT, int MODE>
__global__ __launch_bounds__(kRwThreads, 2) void conv_rw_kernel(const RwConv p)
{
    constexpr int FX = 3;
    constexpr int NK = FX * CPR;
    extern __shared__ __align__(16) unsigned char lds[];
    unsigned char *img = lds + kRwLutBytes + kRwTabBytes;

    const int tid = threadIdx.x, lane = tid & 63;
    // The wave index must be visibly uniform: every branch around MFMAs below has to be a scalar branch, because
    // MFMA ignores EXEC and a masked-off block that is not jumped over would still accumulate.
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, lg = lane >> 4;
    // workgroup = (member, band of rows, set of cgl channel groups), channel groups fastest
    const unsigned zb = blockIdx.x / (unsigned)p.ngw;
    const int cg0 = (int)(blockIdx.x - zb * p.ngw) * p.cgl;
    const int cg1 = cg0 + p.cgl < p.ncg ? cg0 + p.cgl : p.ncg;
    const int64_t z = zb / (unsigned)p.S;                       // member
    const int row0 = (int)(zb - (unsigned)z * p.S) * p.hs;      // first output row of this band
    const int hloc = p.h - row0 < p.hs ? p.h - row0 : p.hs;     // its output rows
    const int Ow = (p.O + 63) >> 6;
    const int nunits = p.ntx * p.nsub;                          // (strip, sub-band) units for the four waves

    // Expansion table: dword 4*n + c (c = 0..3) holds the +-1 bytes of the four bits of n.  A lane always reads copy
    // c = lane % 4, so every address a wave asks for sits in a bank of its own: the look-ups never conflict.
    if (tid < 64) reinterpret_cast<uint32_t *>(lds)[tid] = rw_pm1_bytes((unsigned)tid >> 2);
    const unsigned char *lut = lds + (lane & 3) * 4;
    auto expand16 = [&](uint32_t h16) {  // 16 bits -> 16 bytes of +-1, bit b -> byte b
        uint4 r;
        r.x = *reinterpret_cast<const uint32_t *>(lut + ((h16 & 0xFu) << 4));
        r.y = *reinterpret_cast<const uint32_t *>(lut + (((h16 >> 4) & 0xFu) << 4));
        r.z = *reinterpret_cast<const uint32_t *>(lut + (((h16 >> 8) & 0xFu) << 4));
        r.w = *reinterpret_cast<const uint32_t *>(lut + (((h16 >> 12) & 0xFu) << 4));
        return r;
    };

    // ---- fragment geometry ---------------------------------------------------------------------------------
    // chunk kq = i*CPR + q (filter row i) and lane group g: tap column j, first position c0.  Table entry:
    //   x = byte offset of the filter word holding the group's 16 bits (without the channel),
    //   y = shift of those bits | mask of the channel bits among them << 8 | (tap column inside the filter) << 31;
    // a tap column past the filter multiplies by zero bytes, channel positions past in_bits by -1 (they equal the
    // pixel's zero tail and are part of K).
    uint2 *tab = reinterpret_cast<uint2 *>(lds + kRwLutBytes);
    if (tid < NK * 4) {
        const int kq = tid >> 2, g = tid & 3;
        const int i = kq / CPR, q = kq - i * CPR;
        int qj = 0, qc = 0;
        if (p.CB == 32) {
            qj = 2 * q;
        } else if (p.CB >= 64) {
            qj = q / p.Cw;
            qc = 64 * (q - qj * p.Cw);
        }
        const int j = qj + (g >> p.jsh), c0 = qc + 16 * (g & p.cmask);
        const int tap = i * p.fy + j;
        const int left = p.in_bits - c0;
        const int nv = left < 0 ? 0 : (left > 16 ? 16 : left);
        int fr, sh;
        if (p.tapT > 0) {
            fr = (tap * p.tapM) >> 16;  // tap / tapT
            sh = p.in_bits * (tap - fr * p.tapT) + c0;
            sh = sh > 63 ? 63 : sh;     // only when nv == 0: the bits are masked off anyway
        } else {
            fr = tap * p.Cw + (c0 >> 6);
            sh = c0 & 63;
        }
        const bool inside = j < p.fy;
        tab[tid] = make_uint2(inside ? (uint32_t)(fr * p.O) * 8u : 0u,
                              (uint32_t)sh | (((1u << nv) - 1u) << 8) | (inside ? 0x80000000u : 0u));
    }
    int koff[CPR];  // byte offset of the lane's 16 positions relative to the strip's first pixel
#pragma unroll
    for (int q = 0; q < CPR; q++) {
        const int j = p.qj[q] + (lg >> p.jsh);
        koff[q] = __mul24((j < p.fy ? j : 0) + li, p.PS) + p.qc[q] + 16 * (lg & p.cmask);
    }
    __syncthreads();  // tables complete

    // The four waves build a channel group's NK*NT filter fragments together: wave w takes fragments w, w+4, ...
    // (fragment f = chunk f/NT, channel tile f%NT) from global memory, expands them into the staging area, and
    // after a barrier every wave copies all of them into registers.  Every address is valid (channels past O read
    // channel O-1, dead tap columns word 0); the expansion zeroes them.
    constexpr int NF = NK * NT, FPW = (NF + kRwWaves - 1) / kRwWaves;
    const unsigned char *fz = reinterpret_cast<const unsigned char *>(p.filt + z * (int64_t)p.fwords);
    unsigned char *bst = lds + p.bst_off;
    uint64_t fw[FPW];
    int traw[NT];
    auto request_filter = [&](int n0) {
#pragma unroll
        for (int t = 0; t < FPW; t++) {
            const int f = wv + kRwWaves * t;  // uniform
            const int kq = f < NF ? f / NT : 0, nt = f < NF ? f - kq * NT : 0;
            const int ch = n0 + nt * 16 + li;
            fw[t] = *reinterpret_cast<const uint64_t *>(fz + (tab[kq * 4 + lg].x + (uint32_t)(ch < p.O ? ch : p.O - 1) * 8u));
        }
        if (MODE != 0) {
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                const int ch = n0 + nt * 16 + li;
                traw[nt] = p.thresh[z * p.O + (ch < p.O ? ch : p.O - 1)];
            }
        }
    };
    auto stage_filter = [&](int n0) {
#pragma unroll
        for (int t = 0; t < FPW; t++) {
            const int f = wv + kRwWaves * t;
            if (f < NF) {  // uniform
                const int kq = f / NT, nt = f - kq * NT;
                const uint32_t e = tab[kq * 4 + lg].y;
                const uint32_t sh = e & 63u, vmask = (e >> 8) & 0xFFFFu;
                const bool live = (int)e < 0 && n0 + nt * 16 + li < p.O;
                const uint32_t h16 = (uint32_t)(fw[t] >> sh) & vmask;
                const uint4 e16 = expand16(h16);
                *reinterpret_cast<uint4 *>(bst + (f * 64 + lane) * 16) =
                    live ? e16 : make_uint4(0u, 0u, 0u, 0u);
            }
        }
    };
    v4i B[NK][NT];
    int tdot[NT];
    auto fetch_fragments = [&](int n0) {
#pragma unroll
        for (int kq = 0; kq < NK; kq++)
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
                B[kq][nt] = *reinterpret_cast<const v4i *>(bst + ((kq * NT + nt) * 64 + lane) * 16);
        // thresholds in dot-product terms: 2*popc > t  <=>  popc > (t>>1)  <=>  dot < K - 2*(t>>1)
        if (MODE != 0) {
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                int64_t td = n0 + nt * 16 + li < p.O ? (int64_t)p.K - 2 * (int64_t)(traw[nt] >> 1) : -2147483648LL;
                td = td > 2147483647LL ? 2147483647LL : (td < -2147483648LL ? -2147483648LL : td);
                tdot[nt] = (int)td;
            }
        }
    };
    request_filter(cg0 * 16 * NT);

    // ---- phase 1: request the band's input words (with border) --------------------------------------------------
    // one pixel word per item, up to U items per thread in flight; (row, column, offset) advance incrementally; an
    // out-of-range pixel reads word 0 of the member and is replaced by the zero word
    const unsigned char *src = reinterpret_cast<const unsigned char *>(p.in + z * (int64_t)p.H * p.Wd * p.Cw);
    const int npix = (hloc + FX - 1) * p.RW;
    const int pixb = p.Cw * 8, rowb = p.Wd * pixb;                          // bytes per pixel / image row
    const int stepb = p.pix_q * rowb + p.pix_r * pixb, wrapb = rowb - p.RW * pixb;
    const int xend = p.RW - p.py;
    constexpr int U = 8;
    int yy, xs, off;  // running position of the thread's next item
    {
        const int row = tid / p.RW, xx = tid - row * p.RW;
        yy = row0 + row - p.px;
        xs = xx - p.py;
        off = yy * rowb + xs * pixb;
    }
    uint64_t wd[U];
    auto load_items = [&](int cw8) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const bool inb = yy >= 0 && yy < p.H && xs >= 0 && xs < p.Wd;  // false past the last image row too
            const uint64_t v = *reinterpret_cast<const uint64_t *>(src + (uint32_t)(inb ? off + cw8 : 0));
            wd[u] = inb ? v : 0ull;
            yy += p.pix_q;
            xs += p.pix_r;
            off += stepb;
            if (xs >= xend) {
                xs -= p.RW;
                yy++;
                off += wrapb;
            }
        }
    };
    load_items(0);

    // ---- phase 2: first channel group's fragments (staged over the still empty image area when cgl == 1) ---------
    stage_filter(cg0 * 16 * NT);
    __syncthreads();  // fragments complete
    fetch_fragments(cg0 * 16 * NT);
    __syncthreads();  // fragments in registers: the area is free again

    // ---- phase 3: expand the input words into +-1 bytes in LDS -----------------------------------------------------
    for (int cw = 0; cw < p.Cw; cw++) {
        const int nbytes = p.CB - cw * 64 < 64 ? p.CB - cw * 64 : 64;  // positions held by this word
        unsigned char *dst = img + __mul24(tid, p.PS) + cw * 64;
        const int dstep = kRwThreads * p.PS;
        for (int pix0 = tid; pix0 < npix; pix0 += kRwThreads * U) {
            if (pix0 != tid || cw != 0) load_items(cw * 8);
#pragma unroll
            for (int u = 0; u < U; u++) {
                if (pix0 + u * kRwThreads < npix) {
                    for (int c = 0; c < nbytes; c += 16) {
                        *reinterpret_cast<uint4 *>(dst + c) = expand16((uint32_t)(wd[u] >> c) & 0xFFFFu);
                    }
                }
                dst += dstep;
            }
        }
        if (cw + 1 < p.Cw) {  // rewind to the thread's first item for the next channel word
            const int row = tid / p.RW, xx = tid - row * p.RW;
            yy = row0 + row - p.px;
            xs = xx - p.py;
            off = yy * rowb + xs * pixb;
        }
    }
    __syncthreads();  // image complete

    int *stage = reinterpret_cast<int *>(img + p.img_bytes) + wv * (16 * 16 * NT);  // MODE 0 only

    for (int cg = cg0;;) {
    const int n0 = cg * 16 * NT;  // first channel of the group
    for (int u = wv; u < nunits; u += kRwWaves) {
        const int sub = u / p.ntx, strip = u - sub * p.ntx;
        const int ys = sub * p.hb;
        const int ye = ys + p.hb < hloc ? ys + p.hb : hloc;
        if (ys >= ye) continue;  // wave-uniform
        const int x0 = strip * 16;

        int pend[NT][2];  // MODE 3: x-pooled minima of the even row of a pair
#pragma unroll
        for (int nt = 0; nt < NT; nt++) pend[nt][0] = pend[nt][1] = 0;

        // ---- epilogue of one finished output row (band-relative y) -------------------------------------------
        // Output addresses: a uniform row pointer (scalar arithmetic) plus a per-lane 32-bit byte offset.
        unsigned char *obase;   // first element of the strip's row 0 (band-relative) for this channel group
        int64_t orowb;          // bytes from one (pooled) output row to the next
        uint32_t olane[MODE == 0 ? 16 / (64 / (4 * NT)) : 1];
        bool olive[MODE == 0 ? 16 / (64 / (4 * NT)) : 1];
        const bool halfword = NT == 2 && p.ncg > 1;  // a 32-channel group is half a word
        if (MODE == 0) {
            constexpr int LPP = 4 * NT, PPI = 64 / LPP;  // lanes per pixel (one int4 each), pixels per store
            obase = static_cast<unsigned char *>(p.out) + ((((z * p.h + row0) * (int64_t)p.w + x0) * p.O + n0) << 2);
            orowb = ((int64_t)p.w * p.O) << 2;
#pragma unroll
            for (int s = 0; s < 16 / PPI; s++) {
                const int pi = s * PPI + lane / LPP, c4 = (lane % LPP) * 4;
                olane[s] = (uint32_t)(__mul24(pi, p.O) + c4) << 2;
                olive[s] = x0 + pi < p.w && n0 + c4 < p.O;
            }
        } else {
            const int hh = MODE == 3 ? p.h >> 1 : p.h, ww = MODE == 3 ? p.w >> 1 : p.w;
            const int r0 = MODE == 3 ? row0 >> 1 : row0, xx0 = MODE == 3 ? x0 >> 1 : x0;
            const int64_t e0 = ((z * hh + r0) * (int64_t)ww + xx0) * Ow;  // word index of the strip's first pixel
            obase = static_cast<unsigned char *>(p.out) + (halfword ? (e0 << 3) + 4 * cg : (e0 + cg) << 3);
            orowb = ((int64_t)ww * Ow) << 3;
            olane[0] = (uint32_t)__mul24(lane, Ow) << 3;
            olive[0] = lane < (MODE == 3 ? 8 : 16) && xx0 + lane < ww;
        }
        auto finish_row = [&](v4i (&a)[NT], int y) {
            if (MODE == 0) {
                // stage the 16 x (16*NT) tile in LDS, then store whole pixel rows (non-temporal)
#pragma unroll
                for (int nt = 0; nt < NT; nt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) stage[(4 * lg + r) * (16 * NT) + nt * 16 + li] = (p.K - a[nt][r]) >> 1;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                constexpr int LPP = 4 * NT, PPI = 64 / LPP;
                unsigned char *orow = obase + y * orowb;
#pragma unroll
                for (int s = 0; s < 16 / PPI; s++) {
                    const int pi = s * PPI + lane / LPP, c4 = (lane % LPP) * 4;
                    if (olive[s]) {
                        const nb_i32x4 v = *reinterpret_cast<const nb_i32x4 *>(stage + pi * (16 * NT) + c4);
                        __builtin_nontemporal_store(v, reinterpret_cast<nb_i32x4 *>(orow + olane[s]));
                    }
                }
                __builtin_amdgcn_wave_barrier();
                return;
            }
            uint64_t word = 0;
            if (MODE == 2) {
                // ballot r of lane (pixel 4*g+r, channel li): bits 16*g.. are the 16-channel piece of pixel 4*g+r.
                // Lane j < 16 assembles the pieces of pixel j over the NT channel tiles and writes them.
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    uint64_t m[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) m[r] = __ballot(a[nt][r] < tdot[nt]);
                    const uint64_t mine = rw_sel4(lane & 3, m[0], m[1], m[2], m[3]);
                    word |= ((mine >> (16 * ((lane >> 2) & 3))) & 0xFFFFull) << (16 * nt);
                }
            } else {
                // pixels 4g, 4g+1 and 4g+2, 4g+3 pool in x; rows y (even) and y+1 pool in y
                if ((y & 1) == 0) {
#pragma unroll
                    for (int nt = 0; nt < NT; nt++) {
                        pend[nt][0] = a[nt][0] < a[nt][1] ? a[nt][0] : a[nt][1];
                        pend[nt][1] = a[nt][2] < a[nt][3] ? a[nt][2] : a[nt][3];
                    }
                    return;
                }
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    int v0 = a[nt][0] < a[nt][1] ? a[nt][0] : a[nt][1];
                    int v1 = a[nt][2] < a[nt][3] ? a[nt][2] : a[nt][3];
                    v0 = v0 < pend[nt][0] ? v0 : pend[nt][0];
                    v1 = v1 < pend[nt][1] ? v1 : pend[nt][1];
                    const uint64_t m0 = __ballot(v0 < tdot[nt]), m1 = __ballot(v1 < tdot[nt]);
                    const uint64_t mine = (lane & 1) ? m1 : m0;  // pooled pixel 2g + q <-> lane 2g + q
                    word |= ((mine >> (16 * ((lane >> 1) & 3))) & 0xFFFFull) << (16 * nt);
                }
            }
            unsigned char *orow = obase + (MODE == 3 ? y >> 1 : y) * orowb;
            if (olive[0]) {
                if (halfword) {
                    uint32_t *o = reinterpret_cast<uint32_t *>(orow + olane[0]);
                    o[0] = (uint32_t)word;
                    if (cg == p.ncg - 1 && (cg & 1) == 0) o[1] = 0u;
                } else {
                    *reinterpret_cast<uint64_t *>(orow + olane[0]) = word;
                }
            }
        };

        // ---- walk down the strip: image row rr (band-relative) feeds output rows rr, rr-1, rr-2 --------------
        // a0 holds the partial sums of output row rr-2 (two filter rows done), a1 those of row rr-1 (one done).
        // Image row rr completes row rr-2 (emitted), continues row rr-1 and opens row rr with a zero C operand,
        // so nothing is ever cleared or rotated.  Rows rr in [ys+2, ye) take the branch-free loop.
        const unsigned char *arow = img + (ys * p.RW + x0) * p.PS;
        const int rowbytes = p.RW * p.PS;
        const int rend = ye + FX - 1;
        const int ylast = MODE == 3 ? (p.h & ~1) - row0 : ye;  // pooled maps drop an odd last row
        v4i F[CPR], a0[NT], a1[NT];
#pragma unroll
        for (int q = 0; q < CPR; q++) F[q] = *reinterpret_cast<const v4i *>(arow + koff[q]);
#pragma unroll
        for (int nt = 0; nt < NT; nt++) a0[nt] = a1[nt] = (v4i){0, 0, 0, 0};
        auto edge_step = [&](int rr) {  // first two and last two image rows of the sub-band: some parts are missing
            v4i Fn[CPR];
            arow += rowbytes;
#pragma unroll
            for (int q = 0; q < CPR; q++) Fn[q] = F[q];
            if (rr + 1 < rend) {
#pragma unroll
                for (int q = 0; q < CPR; q++) Fn[q] = *reinterpret_cast<const v4i *>(arow + koff[q]);
            }
            if (rr - 2 >= ys) {
#pragma unroll
                for (int q = 0; q < CPR; q++)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        a0[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(F[q], B[2 * CPR + q][nt], a0[nt], 0, 0, 0);
                if (rr - 2 < ylast) finish_row(a0, rr - 2);
            }
            if (rr - 1 >= ys && rr - 1 < ye) {
#pragma unroll
                for (int nt = 0; nt < NT; nt++) a0[nt] = a1[nt];
#pragma unroll
                for (int q = 0; q < CPR; q++)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        a0[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(F[q], B[CPR + q][nt], a0[nt], 0, 0, 0);
            }
            if (rr < ye) {
#pragma unroll
                for (int nt = 0; nt < NT; nt++) a1[nt] = (v4i){0, 0, 0, 0};
#pragma unroll
                for (int q = 0; q < CPR; q++)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        a1[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(F[q], B[q][nt], a1[nt], 0, 0, 0);
            }
#pragma unroll
            for (int q = 0; q < CPR; q++) F[q] = Fn[q];
        };
        int rr = ys;
        const int lead = ys + 2 < rend ? ys + 2 : rend;
        for (; rr < lead; rr++) edge_step(rr);
        for (; rr < ye; rr++) {
            v4i Fn[CPR], done[NT];
            arow += rowbytes;
#pragma unroll
            for (int q = 0; q < CPR; q++) Fn[q] = *reinterpret_cast<const v4i *>(arow + koff[q]);
#pragma unroll
            for (int nt = 0; nt < NT; nt++) done[nt] = a0[nt];
#pragma unroll
            for (int q = 0; q < CPR; q++)
#pragma unroll
                for (int nt = 0; nt < NT; nt++)
                    done[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(F[q], B[2 * CPR + q][nt], done[nt], 0, 0, 0);
#pragma unroll
            for (int nt = 0; nt < NT; nt++) a0[nt] = a1[nt];
#pragma unroll
            for (int q = 0; q < CPR; q++)
#pragma unroll
                for (int nt = 0; nt < NT; nt++)
                    a0[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(F[q], B[CPR + q][nt], a0[nt], 0, 0, 0);
#pragma unroll
            for (int nt = 0; nt < NT; nt++) a1[nt] = (v4i){0, 0, 0, 0};
#pragma unroll
            for (int q = 0; q < CPR; q++)
#pragma unroll
                for (int nt = 0; nt < NT; nt++)
                    a1[nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(F[q], B[q][nt], a1[nt], 0, 0, 0);
            finish_row(done, rr - 2);  // rr - 2 < ye - 2 <= ylast
#pragma unroll
            for (int q = 0; q < CPR; q++) F[q] = Fn[q];
        }
        for (; rr < rend; rr++) edge_step(rr);
    }
    if (++cg >= cg1) break;
    // next channel group: no wave reads the staging area during a walk, so a wave that is done starts at once
    request_filter(cg * 16 * NT);
    stage_filter(cg * 16 * NT);
    __syncthreads();
    fetch_fragments(cg * 16 * NT);
    __syncthreads();  // a fast wave must not restage while a slow one still fetches
    }
}

static inline int rw_round_up(int a, int b) { return (a + b - 1) / b * b; }

template <int CPR, int NT, int MODE>
static bool rw_launch_one(const RwConv &p, int64_t D, size_t lds_bytes, hipStream_t s)
{
    static bool attr_set = false;  // benign race: setting the same attribute twice is harmless
    auto *kfn = conv_rw_kernel<CPR, NT, MODE>;
    if (!attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                160 * 1024) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        attr_set = true;
    }
    kfn<<<dim3((unsigned)(D * p.S * p.ngw)), dim3(kRwThreads), lds_bytes, s>>>(p);
    return true;
}

template <int MODE>
static bool rw_launch_mode(const RwConv &p, int64_t D, int CPR, int NT, size_t lds, hipStream_t s)
{
#define NB_RW(cpr, nt) \
    if (CPR == cpr && NT == nt) return rw_launch_one<cpr, nt, MODE>(p, D, lds, s)
    NB_RW(1, 1);
    NB_RW(1, 2);
    NB_RW(1, 4);
    NB_RW(2, 1);
    NB_RW(2, 2);
    NB_RW(2, 4);
    NB_RW(3, 1);
    NB_RW(3, 2);
    NB_RW(3, 4);
    NB_RW(6, 2);
#undef NB_RW
    return false;
}

// mode as in conv_impl (0 int32, 2 packed, 3 packed+pooled).  tap_bits > 0: the filter is tap-packed and the
// input has tap_bits true channels in one word per pixel.  Returns false when this shape has no kernel here;
// nothing has been launched then.
bool conv_rw_try(void *out, const uint64_t *in, const uint64_t *filt, const int32_t *thresh, const ConvGeom &g,
                 int64_t D, int O, int tap_bits, int mode, hipStream_t s)
{
    if (!aligned(out, 16)) return false;
    if (mode != 0 && mode != 2 && mode != 3) return false;
    if (g.sx != 1 || g.sy != 1 || g.h < 1 || g.w < 1 || D < 1) return false;
    if (g.fx != 3 || g.fy < 1 || g.fy > 3 || g.Cw < 1) return false;
    if (O < 16 || (O & 15) != 0) return false;
    if (mode == 3 && (g.h < 2 || g.w < 2)) return false;
    if (tap_bits > 0 && (g.Cw != 1 || tap_bits > 32)) return false;
    // 32-bit byte offsets inside one member's image and filter block
    if ((int64_t)g.H * g.Wd * g.Cw * 8 >= (1LL << 31) || (int64_t)9 * g.Cw * O * 8 >= (1LL << 31)) return false;
    RwConv p;
    p.in = in;
    p.filt = filt;
    p.thresh = thresh;
    p.out = out;
    p.H = g.H; p.Wd = g.Wd; p.Cw = g.Cw; p.px = g.px; p.py = g.py; p.h = g.h; p.w = g.w;
    p.O = O;
    p.fy = g.fy;
    const int CB = tap_bits > 0 ? (tap_bits <= 16 ? 16 : 32) : 64 * g.Cw;
    p.CB = CB;
    p.in_bits = tap_bits > 0 ? tap_bits : 64 * g.Cw;
    p.tapT = tap_bits > 0 ? 64 / tap_bits : 0;
    p.tapM = tap_bits > 0 ? 65536 / p.tapT + 1 : 0;
    p.fwords = (tap_bits > 0 ? (3 * g.fy + p.tapT - 1) / p.tapT : 3 * g.fy * g.Cw) * O;
    int CPR;
    if (CB == 16) {
        CPR = 1;
        p.jsh = 0; p.cmask = 0;
        p.qj[0] = 0; p.qc[0] = 0;
    } else if (CB == 32) {
        CPR = (g.fy + 1) / 2;
        p.jsh = 1; p.cmask = 1;
        for (int q = 0; q < CPR; q++) { p.qj[q] = (short)(2 * q); p.qc[q] = 0; }
    } else {
        CPR = g.fy * g.Cw;
        if (CPR > kRwMaxCPR) return false;
        p.jsh = 2; p.cmask = 3;
        for (int q = 0; q < CPR; q++) { p.qj[q] = (short)(q / g.Cw); p.qc[q] = (short)(64 * (q % g.Cw)); }
    }
    for (int q = CPR; q < kRwMaxCPR; q++) p.qj[q] = p.qc[q] = 0;
    if (CPR == 4 || CPR == 5) return false;
    int NT = O >= 64 ? 4 : O / 16;
    if (NT == 3) return false;
    if (CPR == 6) NT = O >= 32 ? 2 : 0;
    if (CPR == 6 && O == 16) return false;
    p.ncg = (O + 16 * NT - 1) / (16 * NT);
    p.PS = ((CB >> 4) & 1) ? CB : CB + 16;
    p.ntx = (g.w + 15) / 16;
    p.RW = 16 * p.ntx + g.fy - 1;
    p.K = 3 * g.fy * CB;
    p.pix_q = kRwThreads / p.RW;
    p.pix_r = kRwThreads % p.RW;
    // Bands: as few as keep a workgroup's LDS at or below 78 KB (two workgroups per CU), rows per band even.
    // The NK*NT filter fragments (1 KB each) are staged in LDS on their way to the registers.  With one channel
    // group they borrow the image area before the image is written.  With several, a workgroup walks all groups
    // over one expanded image if a separate staging area fits (bands of at least 8 rows); otherwise every channel
    // group gets workgroups of its own, each expanding the image again.
    const int stage = mode == 0 ? kRwWaves * 16 * 16 * NT * 4 : 0;
    const int rowbytes = p.RW * p.PS;
    const int frag_bytes = 3 * CPR * NT * 1024;
    const size_t fixed = (size_t)kRwLutBytes + kRwTabBytes + stage, budget = 78 * 1024;
    size_t lds = 0;
    p.cgl = 0;
    for (p.S = 1;; p.S++) {
        p.hs = rw_round_up((g.h + p.S - 1) / p.S, 2);
        const int img = rw_round_up((p.hs + 2) * rowbytes + 64, 16);
        if (p.ncg > 1 && fixed + img + frag_bytes <= budget && (p.hs >= 8 || p.S == 1)) {
            p.cgl = p.ncg;
            p.img_bytes = img;
            p.bst_off = (int)(fixed + img);
            lds = fixed + img + frag_bytes;
            break;
        }
        if (p.hs <= 2 || (p.ncg > 1 && p.hs < 8)) break;
    }
    if (p.cgl == 0) {
        for (p.S = 1;; p.S++) {
            p.hs = rw_round_up((g.h + p.S - 1) / p.S, 2);
            p.img_bytes = rw_round_up((p.hs + 2) * rowbytes + 64, 16);
            if (p.img_bytes < frag_bytes) p.img_bytes = frag_bytes;
            lds = fixed + p.img_bytes;
            if (lds <= budget || p.hs <= 2) break;
        }
        p.cgl = 1;
        p.bst_off = kRwLutBytes + kRwTabBytes;  // the image area
    }
    if (lds > 158 * 1024) return false;
    p.ngw = (p.ncg + p.cgl - 1) / p.cgl;
    p.S = (g.h + p.hs - 1) / p.hs;  // bands that own at least one row
    if (D * p.S * p.ngw > kMaxBlocks) return false;
    // Sub-bands: enough (strip, sub-band) units for the four waves of a workgroup.
    int nsub = p.ntx >= kRwWaves ? 1 : (kRwWaves + p.ntx - 1) / p.ntx;
    p.hb = rw_round_up((p.hs + nsub - 1) / nsub, 2);
    p.nsub = (p.hs + p.hb - 1) / p.hb;
    if (mode == 0) return rw_launch_mode<0>(p, D, CPR, NT, lds, s);
    if (mode == 2) return rw_launch_mode<2>(p, D, CPR, NT, lds, s);
    return rw_launch_mode<3>(p, D, CPR, NT, lds, s);
}

}  // namespace nb
