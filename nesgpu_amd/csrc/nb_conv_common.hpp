// Shared by the conv translation units: geometry validation and the row-per-lane conv kernel.
#pragma once
#include "nb_rowlane.hpp"

namespace nb {

inline int geom_check(ConvGeom *g, int64_t D, int64_t H, int64_t Wd, int64_t Cw, int fx, int fy, int px, int py,
                      int sx, int sy, const char *who)
{
    NB_REQUIRE(D >= 0 && H >= 0 && Wd >= 0 && Cw >= 0, "%s: negative shape D=%lld H=%lld W=%lld Cw=%lld", who,
               (long long)D, (long long)H, (long long)Wd, (long long)Cw);
    NB_REQUIRE(fx >= 1 && fy >= 1 && sx >= 1 && sy >= 1 && px >= 0 && py >= 0,
               "%s: bad window fx=%d fy=%d px=%d py=%d sx=%d sy=%d", who, fx, fy, px, py, sx, sy);
    NB_REQUIRE(H <= 32768 && Wd <= 32768 && Cw <= 32768 && fx <= 1024 && fy <= 1024 && px <= 32768 && py <= 32768,
               "%s: dimension too large (H=%lld W=%lld Cw=%lld fx=%d fy=%d)", who, (long long)H, (long long)Wd,
               (long long)Cw, fx, fy);
    const int64_t h = out_dim(H, fx, px, sx), w = out_dim(Wd, fy, py, sy);
    NB_REQUIRE(H - fx + 2 * (int64_t)px >= 0 && Wd - fy + 2 * (int64_t)py >= 0,
               "%s: window %dx%d larger than padded input %lldx%lld", who, fx, fy, (long long)(H + 2 * px),
               (long long)(Wd + 2 * py));
    NB_REQUIRE(h * w < (1LL << 30) && (int64_t)fx * fy * Cw < (1LL << 24), "%s: output %lldx%lld too large", who,
               (long long)h, (long long)w);
    g->H = (int)H;
    g->Wd = (int)Wd;
    g->Cw = (int)Cw;
    g->fx = fx;
    g->fy = fy;
    g->px = px;
    g->py = py;
    g->sx = sx;
    g->sy = sy;
    g->h = (int)h;
    g->w = (int)w;
    return NB_OK;
}

// ---- conv: row-per-lane kernel with the implicit-im2col loader ----------------------------------
// POOLMAP: lanes 4q..4q+3 hold the 2x2 window of pooled pixel q (needed by EpiPack<.,true>);
// otherwise lane p of a member is output pixel p in row-major order.
template <typename W, class AL, int KC, int NT, bool SINGLE, bool EXACT, bool POOLMAP, class Epi>
__global__ __launch_bounds__(256) void conv_rowlane_kernel(AL al, const W *__restrict__ filt, Epi epi, int pblocks,
                                                           int Kw, int N)
{
    const ConvGeom &g = al.g;
    const int64_t z = blockIdx.x / pblocks;
    const int p = (int)(blockIdx.x - z * pblocks) * 256 + threadIdx.x;
    int yo, xo;
    bool valid;
    int64_t orow;
    if (POOLMAP) {
        const int h2 = g.h >> 1, w2 = g.w >> 1;
        const int q = p >> 2, sub = p & 3;
        valid = q < h2 * w2;
        const int qy = q / w2, qx = q - qy * w2;
        yo = 2 * qy + (sub >> 1);
        xo = 2 * qx + (sub & 1);
        orow = z * (int64_t)(h2 * w2) + q;
    } else {
        valid = p < g.h * g.w;
        yo = p / g.w;
        xo = p - yo * g.w;
        orow = z * (int64_t)(g.h * g.w) + p;
    }
    const typename AL::Lane lane = al.lane_at(z, yo, xo, valid);
    const W *__restrict__ Fz = filt + z * (int64_t)Kw * N;
    rowlane_body<W, KC, NT, SINGLE, EXACT>(al, lane, Fz, epi, orow, z, Kw, N);
}

// Tap-packed conv (narrow channels), defined in nb_conv_tap.hip.  `filt` is the tap-packed filter
// [D, ceil(fx*fy / (bits/tap_bits)), N]; mode as in conv_impl.
template <typename W>
void conv_tap_launch(void *out, const W *in, const W *filt, const int32_t *thresh, const ConvGeom &g, int64_t D,
                     int64_t lanes, int N, int tap_bits, int mode, hipStream_t s);

// Window-in-a-register kernel (nb_conv_tap.hip): mode 2 on tap-packed filters whose whole window fits 32 bits.
// false = not this shape, nothing launched.
template <typename W>
bool conv_window_try(void *out, const W *in, const W *filt, const int32_t *thresh, const ConvGeom &g, int64_t D, int O,
                     int tap_bits, int mode, hipStream_t s);

// Matrix-core conv (nb_conv_mfma.hip): 3-row filters, stride 1, O % 16 == 0; mode as in conv_impl (0, 2, 3, 4).
// 0 = no kernel for this shape, nothing launched; 2 = the int8 kernel ran; 4 = the FP4 kernel ran (allow_fp4 only).
int conv_mfma_try(void *out, const uint64_t *in, const uint64_t *filt, const int32_t *thresh, const ConvGeom &g,
                  int64_t D, int O, int tap_bits, int mode, bool allow_fp4, hipStream_t s);

// Matrix-core conv for narrow layers (nb_conv_direct.hip): tap-packed filters of at most 16 channels, O <= 64, 3-row
// filters of up to 3 columns, stride 1, mode 2 or 3.  false = not this shape, nothing launched.
bool conv_direct_try(void *out, const uint64_t *in, const uint64_t *filt, const int32_t *thresh, const ConvGeom &g,
                     int64_t D, int O, int tap_bits, int mode, hipStream_t s, int word_bytes = 8);

// The same scheme for wider pixels (nb_conv_direct_fp4.hip), 3x3 windows, stride 1, O = 16, 32 or a multiple of 16 from
// 64 on, mode 0, 2, 3 or 4: one full channel word per pixel with filter [D, 9, O] on the FP4 matrix cores (returns 4; only
// with allow_fp4), tap-packed filters of 17 to 32 channels on the int8 matrix cores (returns 2).  0 = not this shape.
int conv_direct_fp4_try(void *out, const uint64_t *in, const uint64_t *filt, const int32_t *thresh, const ConvGeom &g,
                        int64_t D, int O, int tap_bits, int mode, bool allow_fp4, hipStream_t s);

// Pixel sums (mode 4) from counts of the image's bits per tap, without a conv (nb_conv_sums.hip): 64-bit words, stride
// 1, filters of at most 5 x 5; tap_bits > 0: tap-packed filter.  false = not this shape, nothing launched.
// With bias != nullptr the kernel writes the batch-norm layer's thresholds (bn_conv_threshold below, K channels x taps)
// instead of the sums.
bool conv_sums_count_try(int32_t *out, const uint64_t *in, const uint64_t *filt, const ConvGeom &g, int64_t D, int O,
                         int tap_bits, hipStream_t s, const _Float16 *bias = nullptr, const _Float16 *noise = nullptr,
                         int64_t K = 0);

// What torch's mean over `in_elems` elements reduced to `out_elems` results multiplies its fp32 sums by: the quotient of
// the two counts, each converted to fp32 first.
inline float mean_factor(int64_t out_elems, int64_t in_elems) { return (float)out_elems / (float)in_elems; }

// A double rounded ONCE to fp16: brought to fp32 with round-to-odd (an inexact result keeps a set last bit), after
// which the rounding to fp16 is the one of the exact value.
__device__ __forceinline__ _Float16 double_round_once_fp16(double p)
{
    float r = (float)p;
    if ((double)r != p) {
        uint32_t u = __float_as_uint(r);
        if (fabs((double)r) > fabs(p)) u -= 1u;  // towards zero (r is not zero here: |r| > |p| > 0)
        r = __uint_as_float(u | 1u);
    }
    return (_Float16)r;
}

// fp16(a * b) with one rounding, which is what torch's fp16 mean does with its fp32 sum and that factor (its kernel
// converts the product straight to fp16); the product of two floats is exact in a double.  Written out so that the
// result does not depend on which instructions the compiler picks for `(_Float16)(a * b)`.
__device__ __forceinline__ _Float16 mul_round_once_fp16(float a, float b)
{
    return double_round_once_fp16((double)a * (double)b);
}

// Threshold of BinarizedConv2d(batch_norm=True) for one (member, channel) from the sum of its popcount map over the HW
// output pixels (modules/binary.py:147-155): act = 2*popc - K, mean = fp16(float(sum of act) * factor), rounded once,
// with factor = mean_factor(D * O, D * O * HW) (torch's fp16 mean: fp32 sum times that quotient; the same number
// whenever the fp32 sum is exact, i.e. up to 2^24 in magnitude), thr = fp16(fp16(bias + noise) + mean);
// act > thr  <=>  2*popc > floor(thr) + K, which is what is returned (clamped to int32; INT32_MAX, never exceeded,
// for NaN).
__device__ __forceinline__ int32_t bn_conv_threshold(long long popc_sum, _Float16 bias, _Float16 noise, long long K,
                                                     long long HW, float factor)
{
    const long long sum_act = 2ll * popc_sum - K * HW;
    const _Float16 mean = mul_round_once_fp16((float)sum_act, factor);
    const _Float16 tb = bias + noise;
    const float v = (float)(_Float16)(tb + mean);
    if (v != v) return 2147483647;
    long long th = (long long)floorf(fminf(fmaxf(v, -3.0e9f), 3.0e9f)) + K;
    th = th > 2147483647ll ? 2147483647ll : (th < -2147483648ll ? -2147483648ll : th);
    return (int32_t)th;
}

// thresh[d,o] = bn_conv_threshold(sums[d,o], ...), in place if thresh == sums (nb_linear_bn.hip)
void bn_conv_thresh_launch(int32_t *thresh, const int32_t *sums, const _Float16 *bias, const _Float16 *noise, int64_t D,
                           int64_t O, int64_t K, int64_t HW, hipStream_t s);

inline int taps_per_word(int bits, int tap_bits) { return bits / tap_bits; }

}  // namespace nb
