// Tap-packed binary conv for narrow channels (Cw == 1, true channel count tap_bits <= bits/2): several filter
// taps share one word, which cuts the XOR-popcount work by the number of taps per word (4x at 16 channels,
// one word for the whole 3x3x3 window at 3 channels) without changing any sum.
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
