// Tap-packed binary conv for narrow channels (Cw == 1, true channel count tap_bits <= bits/2): several filter
// taps share one word, which cuts the XOR-popcount work by the number of taps per word (4x at 16 channels,
// one word for the whole 3x3x3 window at 3 channels) without changing any sum.
#include <type_traits>
#include "nb_conv_common.hpp"

namespace nb {

// filt [D, taps, O] (one word per tap, only the low tap_bits bits used) -> out [D, ceil(taps/T), O] with
// out[d,w,o] = OR_t (filt[d, w*T+t, o] & mask) << (tap_bits*t).
template <typename W>
__global__ __launch_bounds__(256) void tap_pack_filter_kernel(W *__restrict__ out, const W *__restrict__ filt,
                                                              int64_t total, int taps, int Kp, int O, int tap_bits,
                                                              int T)
{
    const W mask = (W)(((W)1 << tap_bits) - 1);
    NB_FLAT_LOOP(i, total)
    {
        if (i >= total) continue;
        const int o = (int)(i % O);
        const int64_t dw = i / O;
        const int w = (int)(dw % Kp);
        const int64_t d = dw / Kp;
        W v = 0;
        for (int t = 0; t < T; t++) {
            const int tap = w * T + t;
            if (tap < taps) v |= (filt[(d * taps + tap) * O + o] & mask) << (tap_bits * t);
        }
        out[i] = v;
    }
}

template <typename W, bool POOLMAP, class Epi>
static void dispatch_tap(const ConvTapA<W> &al, const W *filt, const Epi &epi, int64_t D, int64_t lanes, int Kp, int N,
                         hipStream_t s)
{
    typedef ConvTapA<W> AL;
    const int pblocks = (int)ceil_div(lanes, 256);
    const dim3 grid((unsigned)(D * pblocks)), block(256);
#define NB_TAP(KC, SINGLE, EXACT) \
    conv_rowlane_kernel<W, AL, KC, 16, SINGLE, EXACT, POOLMAP, Epi><<<grid, block, 0, s>>>(al, filt, epi, pblocks, Kp, N)
    if (Kp == 1) NB_TAP(1, true, true);
    else if (Kp == 3) NB_TAP(3, true, true);
    else if (Kp <= 5) NB_TAP(5, true, false);
    else if (Kp <= 16) NB_TAP(16, true, false);
    else NB_TAP(16, false, false);
#undef NB_TAP
}

template <typename W>
void conv_tap_launch(void *out, const W *in, const W *filt, const int32_t *thresh, const ConvGeom &g, int64_t D,
                     int64_t lanes, int N, int tap_bits, int mode, hipStream_t s)
{
    constexpr int bits = WordTraits<W>::bits;
    const int T = taps_per_word(bits, tap_bits);
    const int Kp = (int)ceil_div(g.fx * g.fy, T);
    ConvTapA<W> al{in, g, tap_bits, T};
    if (mode == 0) {
        EpiI32 epi{static_cast<int32_t *>(out), (N & 3) == 0 && aligned(out, 16)};
        dispatch_tap<W, false, EpiI32>(al, filt, epi, D, lanes, Kp, N, s);
    } else if (mode == 1) {
        EpiBool epi{static_cast<uint8_t *>(out), thresh, (N & 3) == 0 && aligned(out, 4)};
        dispatch_tap<W, false, EpiBool>(al, filt, epi, D, lanes, Kp, N, s);
    } else if (mode == 4) {
        EpiSum epi{static_cast<int32_t *>(out)};
        dispatch_tap<W, false, EpiSum>(al, filt, epi, D, lanes, Kp, N, s);
    } else if (mode == 2) {
        EpiPack<W, false> epi{static_cast<W *>(out), thresh, (int)ceil_div(N, bits)};
        dispatch_tap<W, false, EpiPack<W, false>>(al, filt, epi, D, lanes, Kp, N, s);
    } else {
        EpiPack<W, true> epi{static_cast<W *>(out), thresh, (int)ceil_div(N, bits)};
        dispatch_tap<W, true, EpiPack<W, true>>(al, filt, epi, D, lanes, Kp, N, s);
    }
}

template void conv_tap_launch<uint64_t>(void *, const uint64_t *, const uint64_t *, const int32_t *, const ConvGeom &,
                                        int64_t, int64_t, int, int, int, hipStream_t);
template void conv_tap_launch<uint32_t>(void *, const uint32_t *, const uint32_t *, const int32_t *, const ConvGeom &,
                                        int64_t, int64_t, int, int, int, hipStream_t);

// ---- whole window in one register --------------------------------------------------------------------------------
// When all taps of the window fit one tap-packed filter word and taps * tap_bits <= 32 (a 3x3 window on up to 3
// channels: the first layer of a network on RGB images), a lane gathers its pixel's whole window into ONE 32-bit
// register in the filter word's tap order.  The member's filter words and thresholds are wave-uniform (scalar
// loads), and an output channel then costs three vector instructions per pixel: v_xor with the filter word as
// scalar operand, v_bcnt with minus the halved threshold as its accumulate operand, and one funnel shift that
// moves the running output word left and takes the sign of that difference in (channels from the top down, so
// bit o lands at position o; the bits arrive inverted and are flipped once per 32 channels).
// Output: threshold bits packed along O (mode 2).
constexpr uint32_t kWinOutside = 0xC0000000u;  // a buffer offset no image reaches: the load returns zero
constexpr int kWinPix = 4;  // pixels per lane: one batch of scalar loads serves four windows
// GATHER: 0 = any geometry, one pixel's window at a time; 1 = rows of four neighbouring pixels straight from memory;
// 2 = the same rows out of an LDS copy of the image rows the workgroup's pixels touch.
template <typename W, int GATHER>
__global__ __launch_bounds__(256) void conv_window_pack_kernel(W *__restrict__ out, const W *__restrict__ in,
                                                               const W *__restrict__ ftap,
                                                               const int32_t *__restrict__ thresh, ConvGeom g, int O,
                                                               int tap_bits, int pixblocks)
{
    constexpr int bits = WordTraits<W>::bits;
    const int64_t z = blockIdx.x / pixblocks;  // wave-uniform: a workgroup stays inside one member
    const int hw = g.h * g.w;
    const W *__restrict__ img = in + z * (int64_t)g.H * g.Wd;  // Cw == 1
    const uint32_t cm = (1u << tap_bits) - 1u;
    uint32_t win[kWinPix];
    bool live[kWinPix];
    int pcs[kWinPix];
    if (GATHER != 0) {
        // stride 1, windows at most 5 wide: a lane takes four neighbouring pixels of one output row, whose windows
        // share their columns: fx * (fy + 3) words are fetched instead of 4 * fx * fy, with one row / column test each
        const int wq = (g.w + kWinPix - 1) / kWinPix;  // quads per output row
        const int quad = (int)(blockIdx.x - z * pixblocks) * 256 + threadIdx.x;
        const int qc = quad < g.h * wq ? quad : g.h * wq - 1;
        const int yo = qc / wq, x0 = (qc - yo * wq) * kWinPix;
#pragma unroll
        for (int q = 0; q < kWinPix; q++) {
            live[q] = quad < g.h * wq && x0 + q < g.w;
            pcs[q] = yo * g.w + (x0 + q < g.w ? x0 + q : g.w - 1);
            win[q] = 0;
        }
        // all words of the window rows are requested before the first one is used: range-checked buffer loads
        // (an offset outside the member's image reads as zero, the padding word) need no branch around them
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<W *>(img), (short)0, g.H * g.Wd * (int)sizeof(W), 0x00020000);
        // GATHER == 2: the input rows that the workgroup's 256 quads touch are copied to LDS first, every word
        // fetched once with coalesced loads (low 32 bits, masked to the channel bits; rows outside the image as
        // zeros).  A row is stored as four runs, columns 0,4,8.. then 1,5,9.. and so on, so that the lanes of a
        // wave, which stand four columns apart, read neighbouring LDS words.
        extern __shared__ uint32_t wl[];
        const int qs = (g.Wd + 3) / 4 + 1;  // words per run, one spare
        const int qfirst = (int)(blockIdx.x - z * pixblocks) * 256;
        const int ya = qfirst / wq - g.px;  // first input row staged
        if (GATHER == 2) {
            const int qlast = qfirst + 255 < g.h * wq ? qfirst + 255 : g.h * wq - 1;
            const int total = (qlast / wq - qfirst / wq + g.fx) * g.Wd;  // staged rows x words per row
            // word idx = base + 256 * u + thread sits in staged row r at column xx; one division per thread, then
            // steps of 256 words = rstep rows and xstep columns (wave-uniform)
            const int rstep = 256 / g.Wd, xstep = 256 - rstep * g.Wd;
            int r = (int)threadIdx.x / g.Wd, xx = (int)threadIdx.x - r * g.Wd;
            for (int base = 0; base < total; base += 1024) {
                uint32_t val[4];
                int at[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int idx = base + u * 256 + (int)threadIdx.x;
                    const int yy = ya + r;
                    const bool ok = (idx < total) & ((unsigned)yy < (unsigned)g.H);
                    const uint32_t off = ok ? (uint32_t)(yy * g.Wd + xx) * (uint32_t)sizeof(W) : kWinOutside;
                    val[u] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)off, 0, 0) & cm;
                    at[u] = idx < total ? r * 4 * qs + (xx & 3) * qs + (xx >> 2) : -1;
                    r += rstep;
                    xx += xstep;
                    if (xx >= g.Wd) {
                        xx -= g.Wd;
                        r++;
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; u++)
                    if (at[u] >= 0) wl[at[u]] = val[u];
            }
            __syncthreads();
        }
        auto gather = [&](auto fxc, auto fyc) {
            constexpr int FX = decltype(fxc)::value, FY = decltype(fyc)::value;  // FY: upper bound of g.fy
            constexpr int NC = FY + kWinPix - 1;
            uint32_t v[FX][NC];
            bool cv[NC];  // column x0 - py + jc lies inside the image (and inside the window's span)
#pragma unroll
            for (int jc = 0; jc < NC; jc++)
                cv[jc] = ((unsigned)(x0 - g.py + jc) < (unsigned)g.Wd) & (jc < g.fy + kWinPix - 1);
            if (GATHER == 2) {
                int ci[NC];  // place of column x0 - py + jc inside a staged row
#pragma unroll
                for (int jc = 0; jc < NC; jc++) {
                    const int xx = x0 - g.py + jc;
                    ci[jc] = cv[jc] ? (xx & 3) * qs + (xx >> 2) : 0;
                }
                const int rbase = (yo - g.px - ya) * 4 * qs;
#pragma unroll
                for (int i = 0; i < FX; i++)
#pragma unroll
                    for (int jc = 0; jc < NC; jc++) {
                        const uint32_t t = wl[rbase + i * 4 * qs + ci[jc]];
                        v[i][jc] = cv[jc] ? t : 0u;  // rows outside the image were staged as zeros
                    }
            } else {
#pragma unroll
                for (int i = 0; i < FX; i++) {
                    const int yy = yo - g.px + i;
                    const bool rv = (unsigned)yy < (unsigned)g.H;
                    const int rb = yy * g.Wd + x0 - g.py;  // word index of the row's first column
#pragma unroll
                    for (int jc = 0; jc < NC; jc++) {  // column x0 - py + jc serves pixel q as tap column jc - q
                        const uint32_t off = (rv & cv[jc]) ? (uint32_t)(rb + jc) * (uint32_t)sizeof(W) : kWinOutside;
                        v[i][jc] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)off, 0, 0) & cm;
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < FX; i++)
#pragma unroll
                for (int j = 0; j < FY; j++)
                    if (j < g.fy) {  // uniform
                        const int sh = tap_bits * (i * g.fy + j);
#pragma unroll
                        for (int q = 0; q < kWinPix; q++) win[q] |= v[i][j + q] << sh;
                    }
        };
        using I1 = std::integral_constant<int, 1>;
        using I2 = std::integral_constant<int, 2>;
        using I3 = std::integral_constant<int, 3>;
        using I4 = std::integral_constant<int, 4>;
        using I5 = std::integral_constant<int, 5>;
        if (g.fx == 3 && g.fy == 3) {  // uniform
            gather(I3{}, I3{});
        } else {
            switch (g.fx) {
            case 1: gather(I1{}, I5{}); break;
            case 2: gather(I2{}, I5{}); break;
            case 3: gather(I3{}, I5{}); break;
            case 4: gather(I4{}, I5{}); break;
            default: gather(I5{}, I5{}); break;
            }
        }
    } else {
        const int pix0 = (int)(blockIdx.x - z * pixblocks) * (256 * kWinPix) + threadIdx.x;
#pragma unroll
        for (int q = 0; q < kWinPix; q++) {
            const int pix = pix0 + 256 * q;
            live[q] = pix < hw;
            pcs[q] = live[q] ? pix : hw - 1;
            const int yo = pcs[q] / g.w, xo = pcs[q] - yo * g.w;
            uint32_t wv = 0;
            for (int i = 0; i < g.fx; i++) {
                const int yy = yo * g.sx - g.px + i;
                for (int j = 0; j < g.fy; j++) {
                    const int xx = xo * g.sy - g.py + j;
                    const bool inside = (unsigned)yy < (unsigned)g.H && (unsigned)xx < (unsigned)g.Wd;
                    const uint32_t v = inside ? (uint32_t)img[yy * g.Wd + xx] : 0u;  // out of range: the zero word
                    wv |= (v & cm) << (tap_bits * (i * g.fy + j));
                }
            }
            win[q] = wv;
        }
    }
    const W *__restrict__ fz = ftap + z * (int64_t)O;  // tap-packed filter [D, 1, O]
    const int32_t *__restrict__ tz = thresh + z * (int64_t)O;
    const int Ow = (O + bits - 1) / bits;
    for (int ow = 0; ow < Ow; ow++) {
        W word[kWinPix];
#pragma unroll
        for (int q = 0; q < kWinPix; q++) word[q] = 0;
#pragma unroll
        for (int half = 0; half < bits / 32; half++) {
            const int base = ow * bits + half * 32;
            const int nch = O - base < 32 ? O - base : 32;  // uniform; channels past O leave zero bits
            uint32_t acc[kWinPix];
#pragma unroll
            for (int q = 0; q < kWinPix; q++) acc[q] = 0;
            if (nch == 32) {
                // sixteen channels at a time: their filter words and thresholds come in with a few wide scalar loads
#pragma unroll
                for (int blk = 1; blk >= 0; blk--) {
                    uint32_t fwv[16], nth[16];
#pragma unroll
                    for (int o = 0; o < 16; o++) {
                        fwv[o] = (uint32_t)fz[base + 16 * blk + o];
                        nth[o] = ~(uint32_t)(tz[base + 16 * blk + o] >> 1);  // -(floor(t / 2)) - 1
                    }
#pragma unroll
                    for (int o = 15; o >= 0; o--) {
                        // 2*popc > t  <=>  popc > floor(t/2)  <=>  popc - floor(t/2) - 1 >= 0: the sign bit of
                        // that difference is the INVERTED output bit; it is shifted in at the bottom of acc by
                        // one funnel shift ({acc, d} >> 31)
#pragma unroll
                        for (int q = 0; q < kWinPix; q++) {
                            const uint32_t d = (uint32_t)__popc(win[q] ^ fwv[o]) + nth[o];
                            acc[q] = __builtin_amdgcn_alignbit(acc[q], d, 31);
                        }
                    }
                }
#pragma unroll
                for (int q = 0; q < kWinPix; q++) acc[q] = ~acc[q];
            } else {
                for (int o = nch - 1; o >= 0; o--) {
                    const uint32_t fw = (uint32_t)fz[base + o];
                    const int th = tz[base + o] >> 1;
#pragma unroll
                    for (int q = 0; q < kWinPix; q++) acc[q] = acc[q] + acc[q] + (uint32_t)((int)__popc(win[q] ^ fw) > th);
                }
            }
#pragma unroll
            for (int q = 0; q < kWinPix; q++) word[q] |= (W)acc[q] << (32 * half);
        }
#pragma unroll
        for (int q = 0; q < kWinPix; q++)
            if (live[q]) out[(z * hw + pcs[q]) * (int64_t)Ow + ow] = word[q];
    }
}

template <typename W>
bool conv_window_try(void *out, const W *in, const W *filt, const int32_t *thresh, const ConvGeom &g, int64_t D, int O,
                     int tap_bits, int mode, hipStream_t s)
{
    constexpr int bits = WordTraits<W>::bits;
    const int taps = g.fx * g.fy;
    if (mode != 2 || tap_bits <= 0 || g.Cw != 1 || taps * tap_bits > 32 || taps > taps_per_word(bits, tap_bits)) return false;
    const int64_t hw = (int64_t)g.h * g.w;
    if (hw < 1 || hw >= (1LL << 30) || (int64_t)g.H * g.Wd >= (1LL << 31)) return false;
    if (g.H < 1 || g.Wd < 1) return false;  // an empty image under padding: the general kernels take it
    if (g.sx == 1 && g.sy == 1 && g.fy <= 5 && g.fx <= 5 && (int64_t)g.H * g.Wd * (int64_t)sizeof(W) < (1 << 30)) {
        const int wq = (int)ceil_div(g.w, kWinPix);
        const int64_t pixblocks = ceil_div((int64_t)g.h * wq, 256);
        if (D * pixblocks > kMaxGridX) return false;
        // LDS copy of the rows a workgroup touches: (rows of 256 quads + fx - 1) x four runs of Wd/4 + 1 words, and
        // a few words of slack for the reads of columns just past a row (dropped by the column test)
        const int64_t rows = (255 + wq - 1) / wq + 1 + g.fx - 1;
        const int64_t lds = (rows * 4 * ((g.Wd + 3) / 4 + 1) + 8) * 4;
        if (lds <= 48 * 1024)
            conv_window_pack_kernel<W, 2><<<dim3((unsigned)(D * pixblocks)), dim3(256), (size_t)lds, s>>>(
                static_cast<W *>(out), in, filt, thresh, g, O, tap_bits, (int)pixblocks);
        else
            conv_window_pack_kernel<W, 1><<<dim3((unsigned)(D * pixblocks)), dim3(256), 0, s>>>(
                static_cast<W *>(out), in, filt, thresh, g, O, tap_bits, (int)pixblocks);
    } else {
        const int64_t pixblocks = ceil_div(hw, 256 * kWinPix);
        if (D * pixblocks > kMaxGridX) return false;
        conv_window_pack_kernel<W, 0><<<dim3((unsigned)(D * pixblocks)), dim3(256), 0, s>>>(
            static_cast<W *>(out), in, filt, thresh, g, O, tap_bits, (int)pixblocks);
    }
    return true;
}
template bool conv_window_try<uint64_t>(void *, const uint64_t *, const uint64_t *, const int32_t *, const ConvGeom &,
                                        int64_t, int, int, int, hipStream_t);
template bool conv_window_try<uint32_t>(void *, const uint32_t *, const uint32_t *, const int32_t *, const ConvGeom &,
                                        int64_t, int, int, int, hipStream_t);

template <typename W>
static int tap_pack_filter_impl(W *out, const W *filt, int64_t D, int64_t taps, int64_t O, int tap_bits,
                                nb_stream_t stream, const char *who)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_REQUIRE(D >= 0 && taps >= 0 && O >= 0, "%s: negative shape", who);
    NB_REQUIRE(tap_bits >= 1 && 2 * tap_bits <= bits, "%s: tap_bits must be in [1, %d], got %d", who, bits / 2, tap_bits);
    NB_REQUIRE(taps <= (1 << 20) && O <= (1 << 24), "%s: taps=%lld or O=%lld too large", who, (long long)taps,
               (long long)O);
    const int T = taps_per_word(bits, tap_bits);
    const int64_t Kp = ceil_div(taps, T);
    const int64_t total = D * Kp * O;
    if (total == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(filt);
    NB_REQUIRE_ALIGNED(out, sizeof(W));
    NB_REQUIRE_ALIGNED(filt, sizeof(W));
    tap_pack_filter_kernel<W><<<dim3(grid_for(total)), dim3(256), 0, as_stream(stream)>>>(out, filt, total, (int)taps,
                                                                                         (int)Kp, (int)O, tap_bits, T);
    return check_launch(who);
}

}  // namespace nb

extern "C" {
int nb_tap_pack_filter_i64(int64_t *out, const int64_t *filt, int64_t D, int64_t taps, int64_t O, int tap_bits,
                           nb_stream_t s)
{
    return nb::tap_pack_filter_impl<uint64_t>(reinterpret_cast<uint64_t *>(out),
                                              reinterpret_cast<const uint64_t *>(filt), D, taps, O, tap_bits, s,
                                              "nb_tap_pack_filter_i64");
}
int nb_tap_pack_filter_i32(int32_t *out, const int32_t *filt, int64_t D, int64_t taps, int64_t O, int tap_bits,
                           nb_stream_t s)
{
    return nb::tap_pack_filter_impl<uint32_t>(reinterpret_cast<uint32_t *>(out),
                                              reinterpret_cast<const uint32_t *>(filt), D, taps, O, tap_bits, s,
                                              "nb_tap_pack_filter_i32");
}
}
