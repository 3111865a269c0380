// Binary conv on the FP4 matrix cores for layers with one full channel word per pixel (33 to 64 channels), 3x3
// windows, stride 1: threshold bits out (optionally 2x2 OR-pooled), the popcount maps' sums over the pixels, or the
// int32 maps themselves (a finished row goes through an LDS tile, so that whole pixels leave in 16-byte stores; written
// straight from the accumulators' layout, as 64-byte pieces, they took 78-90 us where 50 are possible).  The
// wave-per-strip scheme of nb_conv_direct.hip with v_mfma_scale_f32_16x16x128_f8f6f4 at unit scales.
//
// Bits become FP4 (E2M1) codes, 1 -> +1.0 (0x2), 0 -> -1.0 (0xA), two positions per byte; +-1 and 0 are exact, the
// fp32 sums are integers far below 2^24, so popcount(x ^ w) = (K - dot) / 2 is the reference's sum bit for bit.  An
// out-of-range pixel is the zero word, i.e. all -1; the zero tail of a channel word multiplies -1 by -1 and is part
// of K.
//
// A wave owns 16 output columns of a sub-band of one member's rows for 16*NT output channels (one output word when
// NT = 4) and walks down.  One MFMA takes 128 positions = two (pixel column, 64 channels) pairs: lane (pixel li,
// group g) supplies the 32 channels of half g&1 of pixel column g>>1, which it fetches itself (a 4-byte buffer load
// whose range check returns zero outside the image) and takes through a 256-entry LDS table, 8 bits -> 4 bytes.
// Per image row r two fragments:
//   A0(r) = [row r, tap column 0 | row r, tap column 1]            x filter rows 0, 1, 2  -> output rows r, r-1, r-2
//   A1(r) = [row r, tap column 2 | row r+1, tap column 2]          x [f(0,2) | f(1,2)]    -> output row r
//                                                                  x [f(2,2) |   0   ]    -> output row r-2
// so the third tap column costs two MFMAs per row instead of three: five per row and 16 channels, not six.
// Finished rows are compared with the thresholds (as dot products), gathered with ballots, pooled (in x a min over
// neighbouring accumulator registers, in y over two walked rows) and stored as whole words.
//
// The same kernel has an int8 flavour (Q = 0) for tap-packed layers of 17 to 32 channels (the first layer of a
// network fed with 3 x 8 bit planes): a pixel is 32 positions of +-1 bytes, a lane supplies 16 of them, one
// v_mfma_i32_16x16x64_i8 takes two (pixel column, 32 channels) pairs, and everything else is as above with integer
// sums (no bias needed).  Positions past the channel count are zero bytes in the filter fragments.
#include "nb_conv_common.hpp"

namespace nb {

typedef int dw_v4i __attribute__((ext_vector_type(4)));
typedef int dw_v8i __attribute__((ext_vector_type(8)));
typedef float dw_v4f __attribute__((ext_vector_type(4)));

struct DwConv {
    const uint64_t *in, *filt;
    const int32_t *thresh;
    void *out;
    int H, Wd, px, py, h, w, O, Ow, K;
    int in_bits, tapT, tapM, fwords;  // Q = 0: channels, taps per filter word, (tap * tapM) >> 16 = tap / tapT, words
    int ntx, ncg, nsb, hb;  // strips of 16 columns, channel groups of 16*NT, sub-bands per member, rows per sub-band
    uint32_t units;         // D * nsb * ncg * ntx
    uint32_t mntx, mncg, mnsb;
};

__device__ __forceinline__ uint32_t dw_div(uint32_t n, uint32_t d, uint32_t m)  // n / d, m = floor(2^32 / d)
{
    uint32_t q = d == 1 ? n : __umulhi(n, m);
    q += n - q * d >= d;
    q += n - q * d >= d;
    return q;
}

// entry b: the FP4 codes of bits 0..7 of b, bit j -> nibble j
struct DwLut {
    uint32_t e[256];
};
constexpr DwLut dw_make_lut()
{
    DwLut t{};
    for (uint32_t b = 0; b < 256; b++) {
        uint32_t w = 0;
        for (int j = 0; j < 8; j++) w |= (((b >> j) & 1u) ? 0x2u : 0xAu) << (4 * j);
        t.e[b] = w;
    }
    return t;
}
__device__ const DwLut dw_lut_src = dw_make_lut();

// entry b: the +-1 bytes of bits 0..7 of b (1 -> 0x01, 0 -> 0xFF)
struct DwLut8 {
    uint2 e[256];
};
constexpr uint32_t dw_pm1_const(uint32_t nib)
{
    uint32_t w = 0;
    for (int j = 0; j < 4; j++) w |= (((nib >> j) & 1u) ? 0x01u : 0xFFu) << (8 * j);
    return w;
}
constexpr DwLut8 dw_make_lut8()
{
    DwLut8 t{};
    for (uint32_t b = 0; b < 256; b++) {
        t.e[b].x = dw_pm1_const(b & 15u);
        t.e[b].y = dw_pm1_const(b >> 4);
    }
    return t;
}
__device__ const DwLut8 dw_lut8_src = dw_make_lut8();

// lane `LANE` (a constant) of w = the scalar value v; the other lanes keep theirs
#define NB_DW_WRITELANE(w, v, LANE) asm("v_writelane_b32 %0, %1, %2" : "+v"(w) : "s"(v), "n"(LANE))

__device__ __forceinline__ dw_v4f dw_mfma(dw_v4i a, dw_v4i b, dw_v4f c)
{
    const dw_v8i a8 = __builtin_shufflevector(a, a, 0, 1, 2, 3, -1, -1, -1, -1);
    const dw_v8i b8 = __builtin_shufflevector(b, b, 0, 1, 2, 3, -1, -1, -1, -1);
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, c, 4, 4, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
}
__device__ __forceinline__ dw_v4i dw_mfma(dw_v4i a, dw_v4i b, dw_v4i c)
{
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
}
template <int Q>
struct DwAcc {
    typedef dw_v4f type;
};
template <>
struct DwAcc<0> {
    typedef dw_v4i type;
};

// MODE 0: the popcount maps themselves, int32 [D,h,w,O]; 2: threshold bits packed along the channels; 3: the same, 2x2
// OR-pooled; 4: the popcount sums added up over the pixels, int32 [D,O] (atomic adds into a zeroed array)
// Q: 1 = FP4 codes, one full channel word per pixel; 0 = +-1 bytes, 17 to 32 channels (tap-packed filter)
template <int NT, int MODE, int Q>
__global__ __launch_bounds__(256) void conv_direct_fp4_kernel(const DwConv p)
{
    typedef typename DwAcc<Q>::type acc_t;
    __shared__ __align__(16) uint2 lut_s[Q ? 128 : 256];  // Q = 1: 256 four-byte entries; Q = 0: 256 eight-byte entries
    // MODE 0: a wave's finished row, 16 pixels x 16*NT channels of int32, on its way from the accumulators' layout
    // (a lane holds 4 pixels of one channel) to whole pixels (a lane stores 4 channels of one pixel); pixel rows
    // 16*NT + 4 dwords apart, so that the four lane groups' writes fall into different banks
    constexpr int kTileRow = 16 * NT + 4;
    __shared__ __align__(16) int tile_s[MODE == 0 ? 4 * 16 * kTileRow : 4];
    if (Q)
        reinterpret_cast<uint32_t *>(lut_s)[threadIdx.x] = dw_lut_src.e[threadIdx.x];
    else
        lut_s[threadIdx.x] = dw_lut8_src.e[threadIdx.x];
    __syncthreads();
    const unsigned char *lutb = reinterpret_cast<const unsigned char *>(lut_s);
    // the lane's 16 bytes of a pixel: Q = 1: the 32 bits x -> 32 codes; Q = 0: bits 0..15 of x -> 16 bytes of +-1
    auto expand32 = [&](uint32_t x) {
        if (Q) {
            const uint32_t a = *reinterpret_cast<const uint32_t *>(lutb + ((x & 0xFFu) << 2));
            const uint32_t b = *reinterpret_cast<const uint32_t *>(lutb + (((x >> 8) & 0xFFu) << 2));
            const uint32_t c = *reinterpret_cast<const uint32_t *>(lutb + (((x >> 16) & 0xFFu) << 2));
            const uint32_t d = *reinterpret_cast<const uint32_t *>(lutb + ((x >> 24) << 2));
            return (dw_v4i){(int)a, (int)b, (int)c, (int)d};
        } else {
            const uint2 a = *reinterpret_cast<const uint2 *>(lutb + ((x & 0xFFu) << 3));
            const uint2 b = *reinterpret_cast<const uint2 *>(lutb + (((x >> 8) & 0xFFu) << 3));
            return (dw_v4i){(int)a.x, (int)a.y, (int)b.x, (int)b.y};
        }
    };
    const int lane = threadIdx.x & 63;
    // the unit is uniform over the wave, and visibly so: every branch around an MFMA must be a scalar branch,
    // because MFMA ignores EXEC
    const uint32_t u = blockIdx.x * 4u + (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (u >= p.units) return;
    const uint32_t t1 = dw_div(u, (uint32_t)p.ntx, p.mntx);
    const int st = (int)(u - t1 * (uint32_t)p.ntx);
    const uint32_t t2 = dw_div(t1, (uint32_t)p.ncg, p.mncg);
    const int cg = (int)(t1 - t2 * (uint32_t)p.ncg);
    const int64_t z = dw_div(t2, (uint32_t)p.nsb, p.mnsb);
    const int sb = (int)(t2 - (uint32_t)z * (uint32_t)p.nsb);
    const int li = lane & 15, lg = lane >> 4;
    const int tc = lg >> 1, hf = lg & 1;  // pixel column inside the 128-position chunk, half of the channel word

    // ---- filter fragments: lane (channel li of tile nt, group lg) ---------------------------------------------------
    const dw_v4i zero_i = {0, 0, 0, 0};
    dw_v4i B0[3][NT], B1a[NT], B1b[NT];
    int tdot[NT];
    {
        const uint64_t *fz = p.filt + z * (int64_t)(Q ? 9 * p.O : p.fwords);
        // the lane's half of the filter word of (tap, channel): Q = 1: 32 of its 64 bits; Q = 0: bits 16*hf.. of the
        // tap's in_bits bits inside a tap-packed word
        auto half = [&](int tap, int ch) {
            if (Q) {
                const uint64_t wd = fz[(int64_t)tap * p.O + ch];
                return hf ? (uint32_t)(wd >> 32) : (uint32_t)wd;
            } else {
                const int fr = (tap * p.tapM) >> 16, sh = p.in_bits * (tap - fr * p.tapT);  // fr = tap / tapT
                const uint32_t bits = (uint32_t)(fz[(int64_t)fr * p.O + ch] >> sh) & (uint32_t)((1ull << p.in_bits) - 1ull);
                return (bits >> (16 * hf)) & 0xFFFFu;
            }
        };
        // Q = 0: the bytes of positions past the channel count are cleared (the upper half holds positions 16..31)
        dw_v4i pmask = {-1, -1, -1, -1};
        if (!Q && hf) {
#pragma unroll
            for (int d = 0; d < 4; d++) {
                const int nv = p.in_bits - 16 - 4 * d;
                pmask[d] = nv <= 0 ? 0 : (nv >= 4 ? -1 : (int)((1u << (8 * nv)) - 1u));
            }
        }
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
            const int ch = (cg * NT + nt) * 16 + li;
            const bool live = ch < p.O;
            const int chc = live ? ch : p.O - 1;
#pragma unroll
            for (int i = 0; i < 3; i++) {
                B0[i][nt] = expand32(half(i * 3 + tc, chc)) & pmask;  // a channel past O multiplies whatever: it never fires
            }
            B1a[nt] = expand32(half(tc * 3 + 2, chc)) & pmask;    // f(0,2) | f(1,2)
            const dw_v4i eb = expand32(half(8, chc)) & pmask;     // f(2,2) | 0
            B1b[nt] = tc == 0 ? eb : zero_i;
            // thresholds in dot-product terms: 2*popc > t  <=>  popc > (t>>1)  <=>  dot < K - 2*(t>>1); every dot
            // product lies in [-K, K], so thresholds outside mean always / never and are pulled in to K + 1 / -K - 1
            int t = MODE == 2 || MODE == 3 ? p.thresh[z * p.O + chc] : 0;
            t = t > 2 * p.K + 4 ? 2 * p.K + 4 : (t < -2 * p.K - 4 ? -2 * p.K - 4 : t);  // beyond: always / never, too
            int td = live ? p.K - 2 * (t >> 1) : -p.K - 1;
            td = td > p.K + 1 ? p.K + 1 : (td < -p.K - 1 ? -p.K - 1 : td);
            // Q = 1: the accumulators start at K + 1 instead of 0, so every sum is a positive float and its bit
            // pattern orders like the value: minima and comparisons are integer instructions (one each; the float
            // forms cost a compare and a select).
            tdot[nt] = Q ? __builtin_bit_cast(int, (float)(td + p.K + 1)) : td;
        }
    }

    // ---- input addressing ------------------------------------------------------------------------------------------
    const int x0 = st * 16;
    const int ys = sb * p.hb;
    const int hout = MODE == 3 ? (p.h & ~1) : p.h;  // pooled maps drop an odd last row
    const int ye = ys + p.hb < hout ? ys + p.hb : hout;
    if (ys >= ye) return;
    const int rowb = p.Wd * 8;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint64_t *>(p.in + z * (int64_t)p.H * p.Wd), (short)0, p.H * rowb, 0x00020000);
    // A column outside the image gets an offset that is out of range whatever row offset (below 2^29 either way) is
    // added; a row outside gives a negative or too large offset by itself.
    constexpr uint32_t kOutside = 0xC0000000u;
    const int xa = x0 + li + tc - p.py, xb = x0 + li + 2 - p.py;
    const int hoff = Q ? 4 * hf : 0;  // Q = 0: both halves of a pixel come from the low dword of its word
    const uint32_t offa = (xa >= 0 && xa < p.Wd) ? (uint32_t)(xa * 8 + hoff) : kOutside;
    const uint32_t offb = (xb >= 0 && xb < p.Wd) ? (uint32_t)(xb * 8 + hoff + tc * rowb) : kOutside;
    const int hsh = Q ? 0 : 16 * hf;  // Q = 0: the lane's 16 channel bits inside the loaded dword
    auto load_a = [&](int rr) {  // band row rr is image row rr - px
        return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)(offa + (uint32_t)((rr - p.px) * rowb)), 0, 0) >> hsh;
    };
    auto load_b = [&](int rr) {
        return (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)(offb + (uint32_t)((rr - p.px) * rowb)), 0, 0) >> hsh;
    };

    // ---- output ----------------------------------------------------------------------------------------------------
    const int hh = MODE == 3 ? p.h >> 1 : p.h, ww = MODE == 3 ? p.w >> 1 : p.w;
    const int xx0 = MODE == 3 ? x0 >> 1 : x0;
    // a channel group is a whole output word (NT = 4), or the layer has one group and one word (O = 16 or 32; the
    // upper part of the word is written as zero)
    const bool olive = lane < (MODE == 3 ? 8 : 16) && xx0 + lane < ww;
    int pend[NT][2];  // MODE 3: x-pooled minima of the even row of a pair
#pragma unroll
    for (int nt = 0; nt < NT; nt++) pend[nt][0] = pend[nt][1] = 0;
    // 16-bit field gq (0..3) of ballot a in the low half, that of ballot b in the high half: scalar pack instructions
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
    // A finished row's comparison results are ballots (scalar registers): bit 16*g + li of the ballot of accumulator
    // register r is (pixel 4*g + r, channel li of the tile).  The output word of a pixel is put together from 16-bit
    // fields of the NT tiles' ballots with scalar pack instructions and written into the storing lane's registers
    // with v_writelane: two vector instructions per stored word, whatever NT is.
    // MODE 4: the lane's running sum over its four pixel columns (columns past the image masked off) and all rows
    int csum[NT];
    int cmask[4];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) csum[nt] = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) cmask[r] = x0 + 4 * lg + r < p.w ? -1 : 0;
    // The words leave through buffer stores whose range is the member's map: a lane with nothing to store is given an
    // offset beyond the range and the hardware drops its store.  No branch on the lane then, which matters here: an
    // MFMA that the compiler sinks into a branch taken by some lanes only (its results being used only there) runs
    // with the other lanes' operands and results masked off and gives wrong sums, so the walk has no divergent
    // branch at all.
    __amdgpu_buffer_rsrc_t orsrc = rsrc;
    uint32_t ooff = 0;
    if (MODE == 2 || MODE == 3) {  // lane P < 8 (16) stores the word of (pooled) pixel xx0 + P for channel group cg
        orsrc = __builtin_amdgcn_make_buffer_rsrc(static_cast<uint64_t *>(p.out) + z * hh * (int64_t)ww * p.Ow, (short)0,
                                                  hh * ww * p.Ow * 8, 0x00020000);
        ooff = olive ? (uint32_t)(((xx0 + lane) * p.Ow + cg) * 8) : 0xC0000000u;
    }
    // MODE 0: int32 [h, w, O]; step s of a row stores pixels 4s .. 4s+3: lane l the channels 4*(l % (4*NT)) .. +3 of the
    // group of pixel 4s + l / (4*NT) (NT = 4: one pixel per 16 lanes = 256 bytes, a whole run of lines)
    constexpr int kLpp = 4 * NT, kPps = 64 / kLpp;  // lanes per pixel, pixels per store step
    int *tile = tile_s + (threadIdx.x >> 6) * 16 * kTileRow;
    uint32_t ooff0[16 / kPps];
    if (MODE == 0) {
        orsrc = __builtin_amdgcn_make_buffer_rsrc(static_cast<int32_t *>(p.out) + z * p.h * (int64_t)p.w * p.O, (short)0,
                                                  p.h * p.w * p.O * 4, 0x00020000);
#pragma unroll
        for (int s2 = 0; s2 < 16 / kPps; s2++) {
            const int px = s2 * kPps + lane / kLpp, ch = cg * 16 * NT + 4 * (lane % kLpp);
            ooff0[s2] = (x0 + px < p.w && ch < p.O) ? (uint32_t)(((x0 + px) * p.O + ch) * 4) : 0xC0000000u;
        }
    }
    auto finish_row = [&](acc_t (&af)[NT], int y, int par) {
        if (MODE == 4) {
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
                csum[nt] += (int)((cmask[0] ? af[nt][0] : 0) + (cmask[1] ? af[nt][1] : 0) + (cmask[2] ? af[nt][2] : 0) +
                                  (cmask[3] ? af[nt][3] : 0));  // Q = 1: float sums, exact: below 2^13
            return;
        }
        if (MODE == 0) {
            // popcount = (K - dot) / 2; Q = 1: the sums carry the bias K + 1
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const auto f = af[nt][r];
                    tile[(4 * lg + r) * kTileRow + 16 * nt + li] =
                        Q ? (int)(((float)(2 * p.K + 1) - (float)f) * 0.5f) : (p.K - (int)f) >> 1;
                }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            typedef int dw_v4s __attribute__((ext_vector_type(4)));
#pragma unroll
            for (int s2 = 0; s2 < 16 / kPps; s2++) {
                const dw_v4s v = *reinterpret_cast<const dw_v4s *>(tile + (s2 * kPps + lane / kLpp) * kTileRow +
                                                                    4 * (lane % kLpp));
                __builtin_amdgcn_raw_buffer_store_b128(v, orsrc, (int)(ooff0[s2] + (uint32_t)(y * p.w * p.O * 4)), 0, 0);
            }
            __builtin_amdgcn_wave_barrier();
            return;
        }
        int a[NT][4];
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const auto f = af[nt][r];  // a copy first: the cast below wants an object, not a vector element
                a[nt][r] = __builtin_bit_cast(int, f);
            }
        int wlo = 0, whi = 0;
        if (MODE == 2) {
            // lane j < 16 stores pixel j = 4*g + r: field g of ballot r
            uint64_t m[4][4];
#pragma unroll
            for (int nt = 0; nt < 4; nt++)
#pragma unroll
                for (int r = 0; r < 4; r++) m[nt][r] = nt < NT ? __ballot(a[nt < NT ? nt : 0][r] < tdot[nt < NT ? nt : 0]) : 0;
#pragma unroll
            for (int g = 0; g < 4; g++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    NB_DW_WRITELANE(wlo, fields(m[0][r], m[1][r], g, NT > 1), 4 * g + r);
                    if (NT > 2) NB_DW_WRITELANE(whi, fields(m[2][r], m[3][r], g, NT > 3), 4 * g + r);
                }
        } else {
            // pixels 4g, 4g+1 and 4g+2, 4g+3 pool in x; rows y (even) and y+1 pool in y
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
                    NB_DW_WRITELANE(wlo, fields(m[0][q], m[1][q], g, NT > 1), 2 * g + q);
                    if (NT > 2) NB_DW_WRITELANE(whi, fields(m[2][q], m[3][q], g, NT > 3), 2 * g + q);
                }
        }
        typedef int dw_v2i __attribute__((ext_vector_type(2)));
        __builtin_amdgcn_raw_buffer_store_b64((dw_v2i){wlo, whi}, orsrc,
                                              (int)(ooff + (uint32_t)((MODE == 3 ? y >> 1 : y) * ww * p.Ow * 8)), 0, 2);
    };

    // ---- walk down the strip: band row rr feeds output rows rr (filter row 0), rr-1 (1) and rr-2 (2) ---------------
    // a0 holds the partial sums of output row rr-2, a1 those of row rr-1; band row rr completes row rr-2 (emitted),
    // continues row rr-1 and opens row rr with a zero C operand.
    acc_t a0[NT], a1[NT];
    typedef decltype(a0[0][0] + a0[0][0]) acc_s;
    const acc_s kb = Q ? (acc_s)(p.K + 1) : (acc_s)0;
    const acc_t zero = {kb, kb, kb, kb};  // the C operand that opens an output row: Q = 1: the bias described above
#pragma unroll
    for (int nt = 0; nt < NT; nt++) a0[nt] = a1[nt] = zero;
    uint32_t ra0 = load_a(ys), rb0 = load_b(ys), ra1 = load_a(ys + 1), rb1 = load_b(ys + 1);
    uint32_t ra2 = load_a(ys + 2), rb2 = load_b(ys + 2), ra3 = load_a(ys + 3), rb3 = load_b(ys + 3);
    // the parts of a step: C = last (third) row of output row rr-2, M = middle row of rr-1, F = first row of rr
    // image fragment x filter fragment: register r of a lane is (pixel 4g + r, channel li)
#define NB_DW_MM(A, B, C) dw_mfma(A, B, C)
#define NB_DW_PART_C(done, A0, A1)                                                           \
    _Pragma("unroll") for (int nt = 0; nt < NT; nt++) done[nt] = NB_DW_MM(A0, B0[2][nt], a0[nt]); \
    _Pragma("unroll") for (int nt = 0; nt < NT; nt++) done[nt] = NB_DW_MM(A1, B1b[nt], done[nt]);
#define NB_DW_PART_M(A0) _Pragma("unroll") for (int nt = 0; nt < NT; nt++) a0[nt] = NB_DW_MM(A0, B0[1][nt], a1[nt]);
#define NB_DW_PART_F(A0, A1)                                                                 \
    _Pragma("unroll") for (int nt = 0; nt < NT; nt++) a1[nt] = NB_DW_MM(A0, B0[0][nt], zero); \
    _Pragma("unroll") for (int nt = 0; nt < NT; nt++) a1[nt] = NB_DW_MM(A1, B1a[nt], a1[nt]);
    if (ye - ys < 4) {
        // short sub-band (a few last rows of an image): every part of a step under its own (uniform) condition
#define NB_DW_ANY(RR, XA, XB, PAR)                                      \
    {                                                                   \
        const int rr_ = (RR);                                           \
        const dw_v4i A0 = expand32(XA), A1 = expand32(XB);              \
        XA = load_a(rr_ + 4);                                           \
        XB = load_b(rr_ + 4);                                           \
        acc_t done[NT];                                                 \
        if (rr_ - 2 >= ys) { NB_DW_PART_C(done, A0, A1) }               \
        if (rr_ - 1 >= ys && rr_ - 1 < ye) { NB_DW_PART_M(A0) }         \
        if (rr_ < ye) { NB_DW_PART_F(A0, A1) }                          \
        if (rr_ - 2 >= ys) finish_row(done, rr_ - 2, PAR);              \
    }
        for (int rr = ys; rr < ye + 2; rr += 4) {
            NB_DW_ANY(rr, ra0, rb0, 0)
            if (rr + 1 < ye + 2) NB_DW_ANY(rr + 1, ra1, rb1, 1)
            if (rr + 2 < ye + 2) NB_DW_ANY(rr + 2, ra2, rb2, 0)
            if (rr + 3 < ye + 2) NB_DW_ANY(rr + 3, ra3, rb3, 1)
        }
#undef NB_DW_ANY
    } else {
        // The steady rows carry no conditions and always issue the same loads, so that the wait for a row's words is a
        // wait for exactly the loads issued before them (four rows ahead).  The fragments of the next row are looked up
        // while the current row is multiplied: two fragment sets, P and Q, used in turn.
        int rr = ys + 2;
        dw_v4i P0 = expand32(ra0), P1 = expand32(rb0), Q0, Q1;
        {
            Q0 = expand32(ra1), Q1 = expand32(rb1);
            ra0 = load_a(ys + 4);
            rb0 = load_b(ys + 4);
            NB_DW_PART_F(P0, P1)
            P0 = expand32(ra2), P1 = expand32(rb2);
            ra1 = load_a(ys + 5);
            rb1 = load_b(ys + 5);
            NB_DW_PART_M(Q0)
            NB_DW_PART_F(Q0, Q1)
        }
        // C0, C1: the current row's fragments; N0, N1: set for the next row, whose words are XNA, XNB; XCA, XCB: the ring
        // slot of the current row, free since its words were looked up a step ago
#define NB_DW_ROW(C0, C1, N0, N1, XNA, XNB, XCA, XCB, PAR)     \
    {                                                          \
        N0 = expand32(XNA), N1 = expand32(XNB);                \
        XCA = load_a(rr + 4);                                  \
        XCB = load_b(rr + 4);                                  \
        acc_t done[NT];                                        \
        NB_DW_PART_C(done, C0, C1)                             \
        NB_DW_PART_M(C0)                                       \
        NB_DW_PART_F(C0, C1)                                   \
        finish_row(done, rr - 2, PAR);                         \
        rr++;                                                  \
    }
        // sub-bands start on even rows, so the parity of a finished row is known where the loop is unrolled
        const int nsteady = ye - ys - 2, rem = nsteady & 3;
        for (int q = nsteady >> 2; q > 0; q--) {
            NB_DW_ROW(P0, P1, Q0, Q1, ra3, rb3, ra2, rb2, 0)
            NB_DW_ROW(Q0, Q1, P0, P1, ra0, rb0, ra3, rb3, 1)
            NB_DW_ROW(P0, P1, Q0, Q1, ra1, rb1, ra0, rb0, 0)
            NB_DW_ROW(Q0, Q1, P0, P1, ra2, rb2, ra1, rb1, 1)
        }
        if (rem >= 1) NB_DW_ROW(P0, P1, Q0, Q1, ra3, rb3, ra2, rb2, 0)
        if (rem >= 2) NB_DW_ROW(Q0, Q1, P0, P1, ra0, rb0, ra3, rb3, 1)
        if (rem >= 3) NB_DW_ROW(P0, P1, Q0, Q1, ra1, rb1, ra0, rb0, 0)
#undef NB_DW_ROW
        // band rows ye and ye + 1 finish the last two output rows: row ye's fragments are in the current set, row
        // ye + 1's words in the ring slot behind it
        {
            if (rem & 1) P0 = Q0, P1 = Q1;
            const uint32_t ua = rem == 0 ? ra3 : rem == 1 ? ra0 : rem == 2 ? ra1 : ra2;
            const uint32_t ub = rem == 0 ? rb3 : rem == 1 ? rb0 : rem == 2 ? rb1 : rb2;
            Q0 = expand32(ua), Q1 = expand32(ub);
            acc_t done[NT];
            NB_DW_PART_C(done, P0, P1)
            NB_DW_PART_M(P0)
            finish_row(done, ye - 2, (ye - ys) & 1);
            NB_DW_PART_C(done, Q0, Q1)
            finish_row(done, ye - 1, (ye - 1 - ys) & 1);
        }
    }
#undef NB_DW_PART_C
#undef NB_DW_PART_M
#undef NB_DW_PART_F
#undef NB_DW_MM
    if (MODE == 4) {
        // popcount = (K - dot) / 2 per pixel (Q = 1: the sums carry the bias K + 1): add the four lane groups, then
        // one atomic per channel
        const int cols = p.w - x0 < 16 ? p.w - x0 : 16;
        const int kn = (Q ? 2 * p.K + 1 : p.K) * (ye - ys) * cols;
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
            int v = csum[nt];
            v += __shfl_xor(v, 16);
            v += __shfl_xor(v, 32);
            const int ch = (cg * NT + nt) * 16 + li;
            if (lg == 0 && ch < p.O) atomicAdd(reinterpret_cast<int *>(p.out) + z * p.O + ch, (kn - v) >> 1);
        }
    }
}

// mode 0 (int32 maps), 2 (packed threshold bits), 3 (2x2 OR-pooled) or 4 (pixel sums into a zeroed array).  tap_bits == 0: one full
// channel word per pixel, filter [D, 9, O], FP4 (returns 4; only with allow_fp4); tap_bits in 17..32: tap-packed filter,
// +-1 bytes (returns 2).  0 = not this shape, nothing launched.
int conv_direct_fp4_try(void *out, const uint64_t *in, const uint64_t *filt, const int32_t *thresh, const ConvGeom &g,
                        int64_t D, int O, int tap_bits, int mode, bool allow_fp4, hipStream_t s)
{
    if (mode != 0 && mode != 2 && mode != 3 && mode != 4) return 0;
    const int q = tap_bits == 0 ? 1 : 0;
    if (q ? !allow_fp4 : (tap_bits < 17 || tap_bits > 32)) return 0;
    // 32-bit byte offsets inside one member's output, below 2^30 for the out-of-range marker of the stores
    if ((mode == 2 || mode == 3) && (int64_t)g.h * g.w * ((O + 63) / 64) * 8 >= (1LL << 30)) return 0;
    if (g.Cw != 1) return 0;
    if (g.sx != 1 || g.sy != 1 || g.fx != 3 || g.fy != 3) return 0;
    if (D < 1 || g.h < 1 || g.w < 1) return 0;
    if (!(O == 16 || O == 32 || (O >= 64 && O % 16 == 0))) return 0;
    if (mode == 3 && (g.h < 2 || g.w < 2)) return 0;
    if (mode == 0 && (int64_t)g.h * g.w * O * 4 >= (1LL << 30)) return 0;  // 32-bit byte offsets inside a member's maps
    // 32-bit byte offsets inside one member's image, far enough below 2^30 for the out-of-range marker
    if ((int64_t)(g.H + g.px + 8) * g.Wd * 8 >= (1LL << 29) || (int64_t)9 * O * 8 >= (1LL << 31)) return 0;
    // 64 channels per wave from 64 channels on (32 per wave, with twice the waves per SIMD, measured 5-8 % slower)
    const int NT = O >= 64 ? 4 : O / 16;
    DwConv p;
    p.in = in;
    p.filt = filt;
    p.thresh = thresh;
    p.out = out;
    p.H = g.H; p.Wd = g.Wd; p.px = g.px; p.py = g.py; p.h = g.h; p.w = g.w;
    p.O = O;
    p.Ow = (O + 63) / 64;
    p.K = q ? 9 * 64 : 9 * tap_bits;
    p.in_bits = q ? 64 : tap_bits;
    p.tapT = q ? 1 : 64 / tap_bits;
    p.tapM = 65536 / p.tapT + 1;  // (tap * tapM) >> 16 = tap / tapT for the nine taps
    p.fwords = (9 + p.tapT - 1) / p.tapT * O;
    p.ntx = (g.w + 15) / 16;
    p.ncg = p.Ow;  // groups cover whole output words (dead channels give zero bits)
    // Sub-bands as tall as the population allows: whole images once that gives every SIMD a few waves, else down
    // to 16 rows (a wave's start, the filter fragments, costs about as much as six rows).
    {
        const int64_t per = D * p.ntx * p.ncg;
        int64_t want = per >= 2048 ? 1 : (2048 + per - 1) / per;
        const int64_t most = g.h / 16 > 1 ? g.h / 16 : 1;
        want = want > most ? most : want;
        p.hb = (int)((g.h + want - 1) / want + 1) & ~1;
    }
    p.nsb = (g.h + p.hb - 1) / p.hb;
    const int64_t units = D * p.nsb * p.ncg * p.ntx;
    if (units >= (1LL << 31)) return 0;
    p.units = (uint32_t)units;
    p.mntx = (uint32_t)((1ULL << 32) / (uint32_t)p.ntx);  // unused for a divisor of 1
    p.mncg = (uint32_t)((1ULL << 32) / (uint32_t)p.ncg);
    p.mnsb = (uint32_t)((1ULL << 32) / (uint32_t)p.nsb);
    const dim3 grid((unsigned)ceil_div(units, 4)), block(256);
#define NB_DW_LAUNCH(nt, qq)                                                   \
    if (NT == nt && q == qq) {                                                 \
        if (mode == 0)                                                         \
            conv_direct_fp4_kernel<nt, 0, qq><<<grid, block, 0, s>>>(p);       \
        else if (mode == 2)                                                    \
            conv_direct_fp4_kernel<nt, 2, qq><<<grid, block, 0, s>>>(p);       \
        else if (mode == 3)                                                    \
            conv_direct_fp4_kernel<nt, 3, qq><<<grid, block, 0, s>>>(p);       \
        else                                                                   \
            conv_direct_fp4_kernel<nt, 4, qq><<<grid, block, 0, s>>>(p);       \
    }
    NB_DW_LAUNCH(1, 1)
    NB_DW_LAUNCH(2, 1)
    NB_DW_LAUNCH(4, 1)
    NB_DW_LAUNCH(1, 0)
    NB_DW_LAUNCH(2, 0)
    NB_DW_LAUNCH(4, 0)
#undef NB_DW_LAUNCH
    return q ? 4 : 2;
}

}  // namespace nb
