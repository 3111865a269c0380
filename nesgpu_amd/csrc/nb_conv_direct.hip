// Binary conv on the matrix cores for narrow layers: at most 16 input channels (tap-packed filters), at most 64
// output channels (one output word), 3-row filters of up to 3 columns, stride 1, threshold bits out (optionally 2x2
// OR-pooled).
//
// Such a layer has too little arithmetic per pixel to pay for a staged image: one v_mfma_i32_16x16x64_i8 covers 16
// pixels x 16 channels x one filter row (3 tap columns x 16 channel positions + 16 idle positions), three of them
// finish a row of 16 output pixels for 16 channels (a wave takes NT = 1, 2 or 4 such channel tiles).  So there is no producer / consumer split and no image in LDS here.  Every wave
// is on its own: it owns a strip of 16 output columns of one sub-band of one member's rows and walks down the strip.
// Lane (pixel li, tap column g) fetches the word of input pixel (row, x0 + li + g - py) itself (a buffer load whose
// range check returns the zero word for every pixel outside the image: the implicit im2col needs no bounds
// arithmetic), takes its 16 channel bits through a 256-entry LDS table to 16 bytes of +-1, and has its A fragment.
// The fragment of image row r is the same whichever filter row it meets, so it is multiplied into the three output
// rows r, r-1, r-2 (three independent accumulators); finished rows are compared with the thresholds (as dot
// products: popcount(x ^ w) = (K - dot) / 2), gathered with ballots, pooled (in x a min over neighbouring
// accumulator registers, in y over two walked rows) and stored as packed words.  Loads run four rows ahead.
// No barrier after the table is filled, about 60 registers: eight waves per SIMD hide each other's latencies.
//
// Bits are +-1 bytes (1 -> +1, 0 -> -1); channel positions past the layer's channel count and tap columns past the
// filter's width are zero bytes in the filter fragment, so K counts true positions only and stray bits above the
// channel count in an input word do not matter.
#include "nb_conv_common.hpp"

namespace nb {

typedef int dc_v4i __attribute__((ext_vector_type(4)));

struct DcConv {
    const uint64_t *in, *filt;
    const int32_t *thresh;
    uint64_t *out;
    int H, Wd, px, py, h, w, O, fy;
    int in_bits, tapT, tapM, fwords, K;
    int ntx, nsb, hb;       // strips of 16 columns, sub-bands per member, rows per sub-band (even)
    int wbytes;             // 8: 64-bit words; 4: 32-bit words (pixels 4 bytes apart, 32-bit filter words, and
                            // 4-byte output words when O <= 32)
    uint32_t units;         // D * nsb * ntx
    uint32_t mntx, mnsb;    // floor(2^32 / ntx), floor(2^32 / nsb): quotients by multiplication
};

// n / d for n < 2^31 with m = floor(2^32 / d): the estimate is at most two short
__device__ __forceinline__ uint32_t dc_div(uint32_t n, uint32_t d, uint32_t m)
{
    uint32_t q = d == 1 ? n : __umulhi(n, m);
    q += n - q * d >= d;
    q += n - q * d >= d;
    return q;
}

// lane `LANE` (a constant) of w = the scalar value v; the other lanes keep theirs
#define NB_DC_WRITELANE(w, v, LANE) asm("v_writelane_b32 %0, %1, %2" : "+v"(w) : "s"(v), "n"(LANE))

// entry b: the +-1 bytes of bits 0..7 of b
struct DcLut {
    uint2 e[256];
};
constexpr uint32_t dc_pm1_const(uint32_t nib)
{
    uint32_t w = 0;
    for (int j = 0; j < 4; j++) w |= (((nib >> j) & 1u) ? 0x01u : 0xFFu) << (8 * j);
    return w;
}
constexpr DcLut dc_make_lut()
{
    DcLut t{};
    for (uint32_t b = 0; b < 256; b++) {
        t.e[b].x = dc_pm1_const(b & 15u);
        t.e[b].y = dc_pm1_const(b >> 4);
    }
    return t;
}
__device__ const DcLut dc_lut_src = dc_make_lut();

// MODE 2: threshold bits packed along the channels; 3: the same, 2x2 OR-pooled
template <int NT, int MODE>
__global__ __launch_bounds__(256) void conv_direct_kernel(const DcConv p)
{
    __shared__ __align__(16) uint2 lut[256];
    lut[threadIdx.x] = dc_lut_src.e[threadIdx.x];
    __syncthreads();
    const unsigned char *lutb = reinterpret_cast<const unsigned char *>(lut);
    auto expand16 = [&](uint32_t x) {  // bits 0..15 of x -> 16 bytes
        const uint2 a = *reinterpret_cast<const uint2 *>(lutb + ((x & 0xFFu) << 3));
        const uint2 b = *reinterpret_cast<const uint2 *>(lutb + (((x >> 8) & 0xFFu) << 3));
        return (dc_v4i){(int)a.x, (int)a.y, (int)b.x, (int)b.y};
    };
    const int lane = threadIdx.x & 63;
    // the unit is uniform over the wave, and visibly so: every branch around an MFMA must be a scalar branch,
    // because MFMA ignores EXEC
    const uint32_t u = blockIdx.x * 4u + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (u >= p.units) return;
    const uint32_t t = dc_div(u, (uint32_t)p.ntx, p.mntx);
    const int st = (int)(u - t * (uint32_t)p.ntx);
    const int64_t z = dc_div(t, (uint32_t)p.nsb, p.mnsb);
    const int sb = (int)(t - (uint32_t)z * (uint32_t)p.nsb);
    const int li = lane & 15, lg = lane >> 4;

    // ---- filter fragments: filter row i, lane (channel li, tap column lg) -----------------------------------------
    dc_v4i B0[NT], B1[NT], B2[NT];
    int tdot[NT];
    {
        const uint64_t *fz = p.filt + z * (int64_t)p.fwords;
        const uint32_t *fz32 = reinterpret_cast<const uint32_t *>(p.filt) + z * (int64_t)p.fwords;
        const uint32_t vbits = (1u << p.in_bits) - 1u;  // in_bits <= 16
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
            const int chn = nt * 16 + li;
            const int ch = chn < p.O ? chn : p.O - 1;
            const bool live = lg < p.fy && chn < p.O;
            uint32_t pmask[4];  // bytes of the true channel positions
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const int nv = p.in_bits - 4 * d;
                pmask[d] = !live || nv <= 0 ? 0u : (nv >= 4 ? 0xFFFFFFFFu : (1u << (8 * nv)) - 1u);
            }
            dc_v4i e[3];
#pragma unroll
            for (int i = 0; i < 3; i++) {
                const int tap = i * p.fy + (lg < p.fy ? lg : 0);
                const int fr = (tap * p.tapM) >> 16, sh = p.in_bits * (tap - fr * p.tapT);  // fr = tap / tapT
                const uint64_t fword = p.wbytes == 8 ? fz[(int64_t)fr * p.O + ch] : (uint64_t)fz32[(int64_t)fr * p.O + ch];
                const uint32_t fbits = (uint32_t)(fword >> sh) & vbits;
                e[i] = expand16(fbits);
                e[i][0] &= (int)pmask[0];
                e[i][1] &= (int)pmask[1];
                e[i][2] &= (int)pmask[2];
                e[i][3] &= (int)pmask[3];
            }
            B0[nt] = e[0], B1[nt] = e[1], B2[nt] = e[2];
            // thresholds in dot-product terms: 2*popc > t  <=>  popc > (t>>1)  <=>  dot < K - 2*(t>>1)
            int64_t td = (int64_t)p.K - 2 * (int64_t)(p.thresh[z * p.O + ch] >> 1);
            td = td > 2147483647LL ? 2147483647LL : td;
            tdot[nt] = chn < p.O ? (int)td : -2147483647 - 1;  // channels past O never fire
        }
    }

    // ---- input addressing ------------------------------------------------------------------------------------------
    const int x0 = st * 16;
    const int ys = sb * p.hb;
    const int hout = MODE == 3 ? (p.h & ~1) : p.h;  // pooled maps drop an odd last row
    const int ye = ys + p.hb < hout ? ys + p.hb : hout;
    if (ys >= ye) return;
    const int rowb = p.Wd * p.wbytes;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char *>(reinterpret_cast<const char *>(p.in) + z * (int64_t)p.H * rowb), (short)0, p.H * rowb,
        0x00020000);
    // A column outside the image (or the idle fourth lane group) gets an offset that is out of range whatever row
    // offset (below 2^30 either way) is added; a row outside gives a negative or too large offset by itself.
    constexpr uint32_t kOutside = 0xC0000000u;
    const int xc = x0 + li + lg - p.py;
    const uint32_t coloff = (lg < p.fy && xc >= 0 && xc < p.Wd) ? (uint32_t)(xc * p.wbytes) : kOutside;
    auto load_row = [&](int rr) {  // band row rr is image row rr - px
        return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)(coloff + (uint32_t)((rr - p.px) * rowb)), 0, 0);
    };

    // ---- output ----------------------------------------------------------------------------------------------------
    const int hh = MODE == 3 ? p.h >> 1 : p.h, ww = MODE == 3 ? p.w >> 1 : p.w;
    const int xx0 = MODE == 3 ? x0 >> 1 : x0;
    // The words leave through buffer stores whose range is the member's map: a lane with nothing to store is given an
    // offset beyond the range and the hardware drops its store.  No branch on the lane then, which matters here: an
    // MFMA that the compiler sinks into a branch taken by some lanes only (its results being used only there) runs
    // with the other lanes' operands and results masked off and gives wrong sums, so the walk has no divergent
    // branch at all.
    const bool olive = lane < (MODE == 3 ? 8 : 16) && xx0 + lane < ww;
    // one 64-bit word per pixel (O <= 64), or, with 32-bit words and O <= 32, one 32-bit word
    const int obytes = (p.wbytes == 4 && p.O <= 32) ? 4 : 8;
    const __amdgpu_buffer_rsrc_t orsrc = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<char *>(p.out) + z * hh * (int64_t)ww * obytes, (short)0, hh * ww * obytes, 0x00020000);
    const uint32_t ooff = olive ? (uint32_t)((xx0 + lane) * obytes) : 0xC0000000u;
    int pend[NT][2];  // MODE 3: x-pooled minima of the even row of a pair
#pragma unroll
    for (int nt = 0; nt < NT; nt++) pend[nt][0] = pend[nt][1] = 0;
    // 16-bit field gq (0..3) of ballot a in the low half, that of ballot b in the high half: scalar instructions
    auto fields = [](uint64_t a, uint64_t b, int gq, bool both) {
        const uint32_t x = gq < 2 ? (uint32_t)a : (uint32_t)(a >> 32), y = gq < 2 ? (uint32_t)b : (uint32_t)(b >> 32);
        if (!both) return (gq & 1) ? x >> 16 : x & 0xFFFFu;  // b is a constant zero
        uint32_t r;  // one instruction; the compiler spells the same thing out as a shift, an and and an or
        if (gq & 1)
            asm("s_pack_hh_b32_b16 %0, %1, %2" : "=s"(r) : "s"(x), "s"(y));
        else
            asm("s_pack_ll_b32_b16 %0, %1, %2" : "=s"(r) : "s"(x), "s"(y));
        return r;
    };
    typedef int dc_v2i __attribute__((ext_vector_type(2)));
    auto finish_row = [&](dc_v4i (&a)[NT], int y, int par) {
        int wlo = 0, whi = 0;
        if (NT == 1) {
            // one channel tile: the storing lane picks its ballot and shifts its 16 bits down itself
            uint64_t word;
            if (MODE == 2) {
                // ballot r of lane (pixel 4*g+r, channel li): bits 16*g.. are the channels of pixel 4*g+r; lane
                // j < 16 takes the piece of pixel j
                const uint64_t m0 = __ballot(a[0][0] < tdot[0]), m1 = __ballot(a[0][1] < tdot[0]),
                               m2 = __ballot(a[0][2] < tdot[0]), m3 = __ballot(a[0][3] < tdot[0]);
                const int r = lane & 3;
                const uint64_t mine = r == 0 ? m0 : r == 1 ? m1 : r == 2 ? m2 : m3;
                word = (mine >> (16 * ((lane >> 2) & 3))) & 0xFFFFull;
            } else {
                // pixels 4g, 4g+1 and 4g+2, 4g+3 pool in x; rows y (even) and y+1 pool in y
                const int v0 = a[0][0] < a[0][1] ? a[0][0] : a[0][1], v1 = a[0][2] < a[0][3] ? a[0][2] : a[0][3];
                if (par == 0) {
                    pend[0][0] = v0, pend[0][1] = v1;
                    return;
                }
                const int w0 = v0 < pend[0][0] ? v0 : pend[0][0], w1 = v1 < pend[0][1] ? v1 : pend[0][1];
                const uint64_t m0 = __ballot(w0 < tdot[0]), m1 = __ballot(w1 < tdot[0]);
                const uint64_t mine = (lane & 1) ? m1 : m0;  // pooled pixel 2g + q <-> lane 2g + q
                word = (mine >> (16 * ((lane >> 1) & 3))) & 0xFFFFull;
            }
            wlo = (int)(uint32_t)word;
        } else if (MODE == 2) {
            // several tiles: the word of pixel j = 4*g + r is put together from field g of the tiles' ballots r with
            // scalar instructions and written into lane j's registers with v_writelane
            uint64_t m[4][4];
#pragma unroll
            for (int nt = 0; nt < 4; nt++)
#pragma unroll
                for (int r = 0; r < 4; r++) m[nt][r] = nt < NT ? __ballot(a[nt < NT ? nt : 0][r] < tdot[nt < NT ? nt : 0]) : 0;
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    NB_DC_WRITELANE(wlo, fields(m[0][r], m[1][r], g, NT > 1), 4 * g + r);
                    if (NT > 2) NB_DC_WRITELANE(whi, fields(m[2][r], m[3][r], g, NT > 3), 4 * g + r);
                }
        } else {
            if (par == 0) {
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    pend[nt][0] = a[nt][0] < a[nt][1] ? a[nt][0] : a[nt][1];
                    pend[nt][1] = a[nt][2] < a[nt][3] ? a[nt][2] : a[nt][3];
                }
                return;
            }
            // lane P < 8 stores pooled pixel P = 2*g + q: field g of ballot q
            uint64_t m[4][2];
#pragma unroll
            for (int nt = 0; nt < 4; nt++) {
                m[nt][0] = m[nt][1] = 0;
                if (nt < NT) {
                    const int n = nt < NT ? nt : 0;
                    int v0 = a[n][0] < a[n][1] ? a[n][0] : a[n][1];
                    int v1 = a[n][2] < a[n][3] ? a[n][2] : a[n][3];
                    v0 = v0 < pend[n][0] ? v0 : pend[n][0];
                    v1 = v1 < pend[n][1] ? v1 : pend[n][1];
                    m[nt][0] = __ballot(v0 < tdot[n]);
                    m[nt][1] = __ballot(v1 < tdot[n]);
                }
            }
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    NB_DC_WRITELANE(wlo, fields(m[0][q], m[1][q], g, NT > 1), 2 * g + q);
                    if (NT > 2) NB_DC_WRITELANE(whi, fields(m[2][q], m[3][q], g, NT > 3), 2 * g + q);
                }
        }
        if (obytes == 8)   // uniform
            __builtin_amdgcn_raw_buffer_store_b64((dc_v2i){wlo, whi}, orsrc,
                                                  (int)(ooff + (uint32_t)((MODE == 3 ? y >> 1 : y) * ww * 8)), 0, 2);
        else
            __builtin_amdgcn_raw_buffer_store_b32(wlo, orsrc, (int)(ooff + (uint32_t)((MODE == 3 ? y >> 1 : y) * ww * 4)),
                                                  0, 2);
    };

    // ---- walk down the strip: band row rr feeds output rows rr (filter row 0), rr-1 (1) and rr-2 (2) ---------------
    // a0 holds the partial sums of output row rr-2 (two filter rows done), a1 those of row rr-1 (one done).  Band row
    // rr completes row rr-2 (emitted), continues row rr-1 and opens row rr with a zero C operand.
    dc_v4i a0[NT], a1[NT];
    const dc_v4i zero = {0, 0, 0, 0};
#pragma unroll
    for (int nt = 0; nt < NT; nt++) a0[nt] = a1[nt] = zero;
    uint32_t r0 = load_row(ys), r1 = load_row(ys + 1), r2 = load_row(ys + 2), r3 = load_row(ys + 3);
#define NB_DC_MFMA(A, B, C) __builtin_amdgcn_mfma_i32_16x16x64_i8(A, B, C, 0, 0, 0)
    // the parts of a step: C = last (third) row of output row rr-2, M = middle row of rr-1, F = first row of rr
#define NB_DC_PART_C(done) _Pragma("unroll") for (int nt = 0; nt < NT; nt++) done[nt] = NB_DC_MFMA(A, B2[nt], a0[nt]);
#define NB_DC_PART_M _Pragma("unroll") for (int nt = 0; nt < NT; nt++) a0[nt] = NB_DC_MFMA(A, B1[nt], a1[nt]);
#define NB_DC_PART_F _Pragma("unroll") for (int nt = 0; nt < NT; nt++) a1[nt] = NB_DC_MFMA(A, B0[nt], zero);
    if (ye - ys < 4) {
        // short sub-band (a few last rows of an image): every part of a step under its own (uniform) condition
#define NB_DC_ANY(RR, X, PAR)                                          \
    {                                                                  \
        const int rr_ = (RR);                                          \
        const dc_v4i A = expand16(X);                                  \
        X = load_row(rr_ + 4);                                         \
        dc_v4i done[NT];                                               \
        if (rr_ - 2 >= ys) { NB_DC_PART_C(done) }                      \
        if (rr_ - 1 >= ys && rr_ - 1 < ye) { NB_DC_PART_M }            \
        if (rr_ < ye) { NB_DC_PART_F }                                 \
        if (rr_ - 2 >= ys) finish_row(done, rr_ - 2, PAR);             \
    }
        for (int rr = ys; rr < ye + 2; rr += 4) {
            NB_DC_ANY(rr, r0, 0)
            if (rr + 1 < ye + 2) NB_DC_ANY(rr + 1, r1, 1)
            if (rr + 2 < ye + 2) NB_DC_ANY(rr + 2, r2, 0)
            if (rr + 3 < ye + 2) NB_DC_ANY(rr + 3, r3, 1)
        }
#undef NB_DC_ANY
        return;
    }
    // The steady rows carry no conditions and always issue the same load, so that the wait for a row's word is a
    // wait for exactly the loads issued before it (four rows ahead).
    int rr = ys + 2;
    {
        dc_v4i A = expand16(r0);
        r0 = load_row(ys + 4);
        NB_DC_PART_F
        A = expand16(r1);
        r1 = load_row(ys + 5);
        NB_DC_PART_M
        NB_DC_PART_F
    }
#define NB_DC_ROW(X, PAR)                                \
    {                                                    \
        const dc_v4i A = expand16(X);                    \
        X = load_row(rr + 4);                            \
        dc_v4i done[NT];                                 \
        NB_DC_PART_C(done)                               \
        NB_DC_PART_M                                     \
        NB_DC_PART_F                                     \
        finish_row(done, rr - 2, PAR);                   \
        rr++;                                            \
    }
    // sub-bands start on even rows, so the parity of a finished row is known where the loop is unrolled
    const int nsteady = ye - ys - 2, rem = nsteady & 3;
    for (int q = nsteady >> 2; q > 0; q--) {
        NB_DC_ROW(r2, 0)
        NB_DC_ROW(r3, 1)
        NB_DC_ROW(r0, 0)
        NB_DC_ROW(r1, 1)
    }
    if (rem >= 1) NB_DC_ROW(r2, 0)
    if (rem >= 2) NB_DC_ROW(r3, 1)
    if (rem >= 3) NB_DC_ROW(r0, 0)
#undef NB_DC_ROW
    // band rows ye and ye + 1 finish the last two output rows; their words sit in the ring behind the steady rows
    {
        const uint32_t ta = rem == 0 ? r2 : rem == 1 ? r3 : rem == 2 ? r0 : r1;
        const uint32_t tb = rem == 0 ? r3 : rem == 1 ? r0 : rem == 2 ? r1 : r2;
        dc_v4i A = expand16(ta);
        dc_v4i done[NT];
        NB_DC_PART_C(done)
        NB_DC_PART_M
        finish_row(done, ye - 2, (ye - ys) & 1);
        A = expand16(tb);
        NB_DC_PART_C(done)
        finish_row(done, ye - 1, (ye - 1 - ys) & 1);
    }
#undef NB_DC_PART_C
#undef NB_DC_PART_M
#undef NB_DC_PART_F
#undef NB_DC_MFMA
}

// mode 2 (packed threshold bits) or 3 (2x2 OR-pooled) on a tap-packed filter.  false = not this shape, nothing
// launched.
bool conv_direct_try(void *out, const uint64_t *in, const uint64_t *filt, const int32_t *thresh, const ConvGeom &g,
                     int64_t D, int O, int tap_bits, int mode, hipStream_t s, int word_bytes)
{
    if (mode != 2 && mode != 3) return false;
    if (tap_bits < 1 || tap_bits > 16 || g.Cw != 1) return false;
    if (g.sx != 1 || g.sy != 1 || g.fx != 3 || g.fy < 1 || g.fy > 3) return false;
    if (O < 1 || O > 64 || D < 1 || g.h < 1 || g.w < 1) return false;
    if (mode == 3 && (g.h < 2 || g.w < 2)) return false;
    // 32-bit byte offsets inside one member's image, far enough below 2^30 for the out-of-range marker
    if ((int64_t)(g.H + g.px + 8) * g.Wd * 8 >= (1LL << 29) || (int64_t)g.h * g.w * 8 >= (1LL << 30)) return false;
    DcConv p;
    p.in = in;
    p.filt = filt;
    p.thresh = thresh;
    p.out = static_cast<uint64_t *>(out);
    p.H = g.H; p.Wd = g.Wd; p.px = g.px; p.py = g.py; p.h = g.h; p.w = g.w;
    p.O = O;
    p.fy = g.fy;
    p.in_bits = tap_bits;
    p.wbytes = word_bytes;
    p.tapT = 8 * word_bytes / tap_bits;
    p.tapM = 65536 / p.tapT + 1;  // (tap * tapM) >> 16 = tap / tapT for the nine taps
    p.fwords = (3 * g.fy + p.tapT - 1) / p.tapT * O;
    p.K = 3 * g.fy * tap_bits;
    p.ntx = (g.w + 15) / 16;
    // Sub-bands: a wave spends about as much on its start (filter fragments, thresholds) as on ten rows, and two
    // rows of every sub-band on the overlap, so sub-bands are as tall as the population allows: whole images once
    // that gives every SIMD about four waves (4096 units), else down to 16 rows.
    {
        const int64_t per = D * p.ntx;
        int64_t want = per >= 4096 ? 1 : (4096 + per - 1) / per;
        const int64_t most = g.h / 16 > 1 ? g.h / 16 : 1;
        want = want > most ? most : want;
        p.hb = (int)((g.h + want - 1) / want + 1) & ~1;
    }
    p.nsb = (g.h + p.hb - 1) / p.hb;
    const int64_t units = D * p.nsb * p.ntx;
    if (units >= (1LL << 31)) return false;
    p.units = (uint32_t)units;
    p.mntx = (uint32_t)((1ULL << 32) / (uint32_t)p.ntx);  // unused for a divisor of 1
    p.mnsb = (uint32_t)((1ULL << 32) / (uint32_t)p.nsb);
    const int64_t blocks = ceil_div(units, 4);
    const int NT = O <= 16 ? 1 : O <= 32 ? 2 : 4;
#define NB_DC_LAUNCH(nt)                                                   \
    if (NT == nt) {                                                        \
        if (mode == 2)                                                     \
            conv_direct_kernel<nt, 2><<<dim3((unsigned)blocks), dim3(256), 0, s>>>(p); \
        else                                                               \
            conv_direct_kernel<nt, 3><<<dim3((unsigned)blocks), dim3(256), 0, s>>>(p); \
    }
    NB_DC_LAUNCH(1)
    NB_DC_LAUNCH(2)
    NB_DC_LAUNCH(4)
#undef NB_DC_LAUNCH
    return true;
}

}  // namespace nb
