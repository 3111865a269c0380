// Packed im2col, implicit-im2col binary conv (int32 / bool / packed / packed+pooled outputs) and
// the packed-bit max-pool.
#include <atomic>
#include <cstdlib>

#include "nb_conv_common.hpp"

namespace nb {

// ---- im2col (kept for API parity; conv itself never materialises the columns) ----------------
// One thread per output word; consecutive threads write consecutive words.  Members are walked by blockIdx.y so
// that the index arithmetic inside a member stays in 32 bits (the host checks that a member's columns fit).
template <typename W>
__global__ __launch_bounds__(256) void im2col_kernel(W *__restrict__ out, const W *__restrict__ in, int64_t D,
                                                     uint32_t per_member, ConvGeom g)
{
    const uint32_t idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= per_member) return;
    const uint32_t K = (uint32_t)(g.fx * g.fy * g.Cw);
    const uint32_t loc = idx / K, e = idx - loc * K;
    const uint32_t xo = loc / (uint32_t)g.w, yo = loc - xo * (uint32_t)g.w;
    const uint32_t tap = e / (uint32_t)g.Cw, c = e - tap * (uint32_t)g.Cw;
    const uint32_t i = tap / (uint32_t)g.fy, j = tap - i * (uint32_t)g.fy;
    const int xi = (int)(i + xo * g.sx) - g.px, yi = (int)(j + yo * g.sy) - g.py;
    const bool ok = xi >= 0 && xi < g.H && yi >= 0 && yi < g.Wd;
    const int64_t img = (int64_t)g.H * g.Wd * g.Cw;
    const int64_t off = ok ? ((int64_t)xi * g.Wd + yi) * g.Cw + c : 0;
    for (int64_t b = blockIdx.y; b < D; b += gridDim.y) {
        const W v = in[b * img + off];  // an element outside re-reads the member's first word and is dropped
        __builtin_nontemporal_store(ok ? v : (W)0, out + b * (int64_t)per_member + idx);
    }
}

// ---- max-pool: OR over the fixed 2x2 window (extensions/src/max_pool2d.cu:19-32) ---------------
template <typename W>
__global__ __launch_bounds__(256) void max_pool_kernel(W *__restrict__ out, const W *__restrict__ in, int64_t total,
                                                       ConvGeom g)
{
    NB_FLAT_LOOP(t, total)
    {
        if (t >= total) continue;
        const int64_t pix = t / g.Cw;
        const int c = (int)(t - pix * g.Cw);
        const int hw = g.h * g.w;
        const int64_t b = pix / hw;
        const int loc = (int)(pix - b * hw);
        const int xo = loc / g.w, yo = loc - xo * g.w;
        const W *img = in + b * (int64_t)g.H * g.Wd * g.Cw;
        W v = 0;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int xi = i + xo * g.sx - g.px, yi = j + yo * g.sy - g.py;
                if (xi >= 0 && xi < g.H && yi >= 0 && yi < g.Wd) v |= img[((int64_t)xi * g.Wd + yi) * g.Cw + c];
            }
        out[t] = v;
    }
}

// Fast path for the usual pooling geometry (2x2 window, stride 2, no padding, 64-bit words, every window inside
// the image): 16-byte streaming loads, four in flight per thread.
// PAIR = true  (Cw == 1, even output width): a thread ORs a 2x4 block of input words into two output words;
// PAIR = false (Cw even; used for Cw == 2): a thread ORs the same word pair of the window's four pixels into an
// output word pair.
template <bool PAIR>
__global__ __launch_bounds__(256) void max_pool_2x2_kernel(uint64_t *__restrict__ out, const uint64_t *__restrict__ in,
                                                           uint32_t total, ConvGeom g, uint32_t units_per_row)
{
    // 32-bit unit indices (the host checks that they fit); a thread handles units t and t + half with all eight
    // loads requested before the first OR
    const uint32_t half = (total + 1) >> 1;
    const uint32_t t0 = blockIdx.x * 256u + threadIdx.x;
    if (t0 >= half) return;
    const uint32_t tt[2] = {t0, t0 + half < total ? t0 + half : t0};
    uint4 a0[2], a1[2], b0[2], b1[2];
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const uint32_t rowi = tt[k] / units_per_row, e = tt[k] - rowi * units_per_row;  // (b, xo), unit in the row
        const uint32_t b = rowi / (uint32_t)g.h, xo = rowi - b * (uint32_t)g.h;
        const int64_t rowstride = (int64_t)g.Wd * g.Cw, inrow = ((int64_t)b * g.H + 2 * xo) * rowstride;
        int64_t i0, i1;  // word offsets of the two 16-byte pieces inside an input row
        if (PAIR) {
            i0 = 4 * (int64_t)e;
            i1 = i0 + 2;
        } else {
            const uint32_t hw = (uint32_t)g.Cw >> 1, yo = e / hw, cp = e - yo * hw;
            i0 = (int64_t)(2 * yo) * g.Cw + 2 * cp;
            i1 = i0 + g.Cw;
        }
        a0[k] = load_stream16(in + inrow + i0);
        a1[k] = load_stream16(in + inrow + i1);
        b0[k] = load_stream16(in + inrow + rowstride + i0);
        b1[k] = load_stream16(in + inrow + rowstride + i1);
    }
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const uint4 u = make_uint4(a0[k].x | b0[k].x, a0[k].y | b0[k].y, a0[k].z | b0[k].z, a0[k].w | b0[k].w);
        const uint4 v = make_uint4(a1[k].x | b1[k].x, a1[k].y | b1[k].y, a1[k].z | b1[k].z, a1[k].w | b1[k].w);
        // PAIR: u holds input pixels 4e, 4e+1 -> output pixel 2e; v holds 4e+2, 4e+3 -> output pixel 2e+1
        const uint4 r = PAIR ? make_uint4(u.x | u.z, u.y | u.w, v.x | v.z, v.y | v.w)
                             : make_uint4(u.x | v.x, u.y | v.y, u.z | v.z, u.w | v.w);
        if (k == 0 || t0 + half < total) {
            u32x4_t rv = {r.x, r.y, r.z, r.w};
            __builtin_nontemporal_store(rv, reinterpret_cast<u32x4_t *>(out) + tt[k]);
        }
    }
}

template <typename W, bool POOLMAP, class Epi>
static void dispatch_conv(const ConvA<W> &al, const W *filt, const Epi &epi, int64_t D, int64_t lanes_per_member,
                          int N, hipStream_t s)
{
    typedef ConvA<W> AL;
    const int Kw = al.g.fx * al.g.fy * al.g.Cw;
    const int pblocks = (int)ceil_div(lanes_per_member, 256);
    const dim3 grid((unsigned)(D * pblocks)), block(256);
#define NB_CONV(KC, SINGLE, EXACT) \
    conv_rowlane_kernel<W, AL, KC, 16, SINGLE, EXACT, POOLMAP, Epi><<<grid, block, 0, s>>>(al, filt, epi, pblocks, Kw, N)
    if (Kw == 9) NB_CONV(9, true, true);
    else if (Kw == 18) NB_CONV(18, true, true);
    else if (Kw <= 4) NB_CONV(4, true, false);
    else if (Kw <= 9) NB_CONV(9, true, false);
    else if (Kw <= 18) NB_CONV(18, true, false);
    else NB_CONV(16, false, false);
#undef NB_CONV
}

template <typename W>
int im2col_impl(W *out, const W *in, int64_t D, int64_t H, int64_t Wd, int64_t Cw, int fx, int fy, int px, int py,
                int sx, int sy, nb_stream_t stream, const char *who)
{
    ConvGeom g;
    if (int rc = geom_check(&g, D, H, Wd, Cw, fx, fy, px, py, sx, sy, who)) return rc;
    const int64_t total = D * g.h * g.w * (int64_t)fx * fy * Cw;
    if (total == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(in);
    NB_REQUIRE_ALIGNED(out, sizeof(W));
    NB_REQUIRE_ALIGNED(in, sizeof(W));
    const int64_t per_member = total / D;
    NB_REQUIRE(per_member < (1LL << 31) && H * Wd * Cw > 0, "%s: a member's columns exceed 2^31 words or its image is empty",
               who);
    const dim3 grid((unsigned)ceil_div(per_member, 256), (unsigned)(D < 65535 ? D : 65535));
    im2col_kernel<W><<<grid, dim3(256), 0, as_stream(stream)>>>(out, in, D, (uint32_t)per_member, g);
    return check_launch(who);
}

template <typename W>
int max_pool_impl(W *out, const W *in, int64_t B, int64_t H, int64_t Wd, int64_t Cw, int fx, int fy, int px, int py,
                  int sx, int sy, nb_stream_t stream, const char *who)
{
    ConvGeom g;
    if (int rc = geom_check(&g, B, H, Wd, Cw, fx, fy, px, py, sx, sy, who)) return rc;
    const int64_t total = B * g.h * g.w * Cw;
    if (total == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(in);
    NB_REQUIRE_ALIGNED(out, sizeof(W));
    NB_REQUIRE_ALIGNED(in, sizeof(W));
    if (sizeof(W) == 8 && sx == 2 && sy == 2 && px == 0 && py == 0 && 2 * g.h <= g.H && 2 * g.w <= g.Wd &&
        aligned(out, 16) && aligned(in, 16) && ((int64_t)g.Wd * Cw) % 2 == 0) {
        const bool pair = Cw == 1 && g.w % 2 == 0;
        if (pair || Cw == 2) {  // measured: with four or more words per pixel the word-per-thread kernel is faster
            const int units_per_row = pair ? g.w / 2 : g.w * (int)(Cw / 2);
            const int64_t units = B * g.h * units_per_row;
            if (units < (1LL << 31)) {
                uint64_t *o = reinterpret_cast<uint64_t *>(out);
                const uint64_t *i = reinterpret_cast<const uint64_t *>(in);
                const unsigned blocks = (unsigned)ceil_div((units + 1) / 2, 256);
                if (pair)
                    max_pool_2x2_kernel<true><<<dim3(blocks), dim3(256), 0, as_stream(stream)>>>(
                        o, i, (uint32_t)units, g, (uint32_t)units_per_row);
                else
                    max_pool_2x2_kernel<false><<<dim3(blocks), dim3(256), 0, as_stream(stream)>>>(
                        o, i, (uint32_t)units, g, (uint32_t)units_per_row);
                return check_launch(who);
            }
        }
    }
    const unsigned blocks = grid_for(total);
    max_pool_kernel<W><<<dim3(blocks), dim3(256), 0, as_stream(stream)>>>(out, in, total, g);
    return check_launch(who);
}

// Process-wide choice between the conv engines (all give identical results): 0 = automatic (matrix cores
// on the shapes where they measured faster, else XOR-popcount), 1 = XOR-popcount only, 2 = matrix cores wherever
// a kernel covers the shape (FP4 codes where that flavour exists, else +-1 bytes), 3 = as 2 but +-1 bytes only.
// Initialised from the environment variable NESBIN_CONV_ENGINE ("valu" -> 1, "mfma" -> 2, "int8" -> 3);
// nb_conv_engine() changes it.
// The one piece of process-wide state of the library: an atomic, read once per conv call.
static int conv_engine_from_env()
{
    const char *v = getenv("NESBIN_CONV_ENGINE");
    return (v && v[0] == 'v') ? 1 : (v && v[0] == 'm') ? 2 : (v && v[0] == 'i') ? 3 : 0;
}
static std::atomic<int> &conv_engine_cell()
{
    static std::atomic<int> cell{conv_engine_from_env()};  // initialised once, thread-safe (function-local static)
    return cell;
}
static int conv_engine() { return conv_engine_cell().load(std::memory_order_relaxed); }
// engine of this thread's latest conv launch: 1 XOR-popcount, 2 matrix cores on +-1 bytes, 4 matrix cores on FP4 codes,
// 5 pixel sums from bit counts (no conv)
static thread_local int t_last_engine = 0;
int set_conv_engine(int e)
{
    if (e >= 0 && e <= 3) return conv_engine_cell().exchange(e, std::memory_order_relaxed);
    return conv_engine();
}

__global__ __launch_bounds__(256) void zero_i32_kernel(int32_t *__restrict__ out, int64_t total)
{
    NB_FLAT_LOOP(t, total)
    {
        if (t < total) out[t] = 0;
    }
}

// mode 0: int32 sums, 1: bool bytes, 2: packed words, 3: packed + 2x2 pooled words, 4: int32 sums added up over
// the pixels, [D, O]
template <typename W>
int conv_impl(void *out, const W *in, const W *filt, const int32_t *thresh, int64_t D, int64_t H, int64_t Wd,
              int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy, int mode, int tap_bits,
              nb_stream_t stream, const char *who, const _Float16 *bn_bias = nullptr, const _Float16 *bn_noise = nullptr,
              int64_t bn_K = 0)
{
    constexpr int bits = WordTraits<W>::bits;
    ConvGeom g;
    if (int rc = geom_check(&g, D, H, Wd, Cw, fx, fy, px, py, sx, sy, who)) return rc;
    NB_REQUIRE(O >= 0 && O <= (1 << 24), "%s: bad output channel count %lld", who, (long long)O);
    const int64_t hw = (int64_t)g.h * g.w;
    const int64_t h2w2 = (int64_t)(g.h >> 1) * (g.w >> 1);
    const int64_t lanes = mode == 3 ? 4 * h2w2 : hw;
    if (mode == 4 && D * O > 0 && lanes == 0) {  // no output pixels: the sums are zero
        NB_REQUIRE_PTR(out);
        NB_REQUIRE_ALIGNED(out, 4);
        zero_i32_kernel<<<dim3(grid_for(D * O)), dim3(256), 0, as_stream(stream)>>>(static_cast<int32_t *>(out), D * O);
        return check_launch(who);
    }
    if (D * lanes * O == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    if (Cw > 0) {
        NB_REQUIRE_PTR(in);
        NB_REQUIRE_PTR(filt);
        NB_REQUIRE_ALIGNED(in, sizeof(W));
        NB_REQUIRE_ALIGNED(filt, sizeof(W));
    }
    if (mode != 0 && mode != 4) {
        NB_REQUIRE_PTR(thresh);
        NB_REQUIRE_ALIGNED(thresh, 4);
    }
    NB_REQUIRE(D * ceil_div(lanes, 256) <= kMaxGridX, "%s: %lld members x %lld pixels exceed one launch", who,
               (long long)D, (long long)lanes);
    ConvA<W> al{in, g};
    hipStream_t s = as_stream(stream);
    const int N = (int)O;
    NB_REQUIRE(tap_bits >= 0, "%s: negative tap_bits", who);
    if (tap_bits > 0)
        NB_REQUIRE(Cw == 1 && 2 * tap_bits <= bits, "%s: tap packing needs Cw == 1 and tap_bits <= %d (got Cw=%lld, %d)",
                   who, bits / 2, (long long)Cw, tap_bits);
    if (mode == 0 || mode == 4) NB_REQUIRE_ALIGNED(out, 4);
    if (mode == 2 || mode == 3) NB_REQUIRE_ALIGNED(out, sizeof(W));
    // int8 matrix-core path (64-bit words, stride 1, O % 16 == 0, member fits LDS); same results
    const int engine = conv_engine();
    if (mode == 4) {
        NB_REQUIRE(hw * (int64_t)fx * fy * Cw * bits < (1LL << 31), "%s: a member's pixel sum may overflow int32", who);
        // Automatic choice: the sums over the pixels need no conv at all (counts of the image's bits per tap, then one
        // small dot product per output channel); a pinned engine still runs its conv kernels.
        if (bits == 64 && engine == 0 && Cw > 0 &&
            conv_sums_count_try(static_cast<int32_t *>(out), reinterpret_cast<const uint64_t *>(in),
                                reinterpret_cast<const uint64_t *>(filt), g, D, N, tap_bits, s, bn_bias, bn_noise, bn_K)) {
            t_last_engine = 5;
            return check_launch(who);
        }
        zero_i32_kernel<<<dim3(grid_for(D * O)), dim3(256), 0, s>>>(static_cast<int32_t *>(out), D * O);
    }
    // Automatic choice, measured on MI355X: one workgroup per CU walks whole members, so the matrix-core kernel needs
    // a population that fills at least half of the CUs; below that the XOR-popcount kernels, which spread one
    // member's pixels over many workgroups, are faster.
    // A window of at most 32 bits (3x3 on up to 3 channels) with packed output: one register per pixel, four vector
    // instructions per output channel; faster than either engine on that shape.
    if (engine <= 1 && Cw > 0 && conv_window_try<W>(out, in, filt, thresh, g, D, N, tap_bits, mode, s)) {
        t_last_engine = 1;
        return check_launch(who);
    }
    // Narrow layers (at most 16 channels in, at most 64 out, threshold bits out): a wave per strip of 16 output columns on
    // the int8 matrix cores, no staged image; any population size.
    if (Cw > 0 && engine != 1 &&
        conv_direct_try(out, reinterpret_cast<const uint64_t *>(in), reinterpret_cast<const uint64_t *>(filt), thresh, g,
                        D, N, tap_bits, mode, s, bits / 8)) {
        t_last_engine = 2;
        return check_launch(who);
    }
    // One word per pixel, 3x3: the same wave-per-strip scheme for full channel words (FP4 matrix cores) and for
    // tap-packed layers of 17 to 32 channels (int8).  Packed outputs and pixel sums always; the int32 maps unless they
    // are large (images of 1024 pixels or more and 256 MiB or more to write: there the staged-image kernel below
    // measured 5-10 % faster, on smaller maps the strip kernel 10-50 %).
    const bool big_maps = mode == 0 && hw >= 1024 && D * hw * O * 4 >= (1LL << 28);
    if (bits == 64 && Cw == 1 && engine != 1 && (engine >= 2 || D >= 128) && !big_maps) {
        const int ran = conv_direct_fp4_try(out, reinterpret_cast<const uint64_t *>(in),
                                            reinterpret_cast<const uint64_t *>(filt), thresh, g, D, N, tap_bits, mode,
                                            engine != 3, s);
        if (ran) {
            t_last_engine = ran;
            return check_launch(who);
        }
    }
    if (bits == 64 && Cw > 0 && engine != 1 && (engine >= 2 || D >= 128)) {
        const int ran = conv_mfma_try(out, reinterpret_cast<const uint64_t *>(in), reinterpret_cast<const uint64_t *>(filt),
                                      thresh, g, D, N, tap_bits, mode, engine != 3, s);
        if (ran) {
            t_last_engine = ran;
            return check_launch(who);
        }
    }
    t_last_engine = 1;
    if (tap_bits > 0) {
        conv_tap_launch<W>(out, in, filt, thresh, g, D, lanes, N, tap_bits, mode, s);
        return check_launch(who);
    }
    if (mode == 0) {
        NB_REQUIRE_ALIGNED(out, 4);
        EpiI32 epi{static_cast<int32_t *>(out), (N & 3) == 0 && aligned(out, 16)};
        dispatch_conv<W, false, EpiI32>(al, filt, epi, D, lanes, N, s);
    } else if (mode == 4) {
        EpiSum epi{static_cast<int32_t *>(out)};
        dispatch_conv<W, false, EpiSum>(al, filt, epi, D, lanes, N, s);
    } else if (mode == 1) {
        EpiBool epi{static_cast<uint8_t *>(out), thresh, (N & 3) == 0 && aligned(out, 4)};
        dispatch_conv<W, false, EpiBool>(al, filt, epi, D, lanes, N, s);
    } else if (mode == 2) {
        NB_REQUIRE_ALIGNED(out, sizeof(W));
        EpiPack<W, false> epi{static_cast<W *>(out), thresh, (int)ceil_div(O, bits)};
        dispatch_conv<W, false, EpiPack<W, false>>(al, filt, epi, D, lanes, N, s);
    } else {
        NB_REQUIRE_ALIGNED(out, sizeof(W));
        EpiPack<W, true> epi{static_cast<W *>(out), thresh, (int)ceil_div(O, bits)};
        dispatch_conv<W, true, EpiPack<W, true>>(al, filt, epi, D, lanes, N, s);
    }
    return check_launch(who);
}

}  // namespace nb

#define W64(p) reinterpret_cast<const uint64_t *>(p)
#define W32(p) reinterpret_cast<const uint32_t *>(p)

// Thresholds of the batch-norm conv layer straight from the image: the pixel sums (mode 4, whatever kernel serves them)
// and the threshold arithmetic; one kernel where the sums come from bit counts, else the sums land in `thresh` and
// are turned into thresholds in place.
template <typename W>
static int conv_bn_thresholds_impl(int32_t *thresh, const W *in, const W *filt, const uint16_t *bias,
                                   const uint16_t *bias_noise, int64_t D, int64_t H, int64_t Wd, int64_t Cw, int64_t O,
                                   int fx, int fy, int px, int py, int sx, int sy, int tap_bits, int64_t K,
                                   nb_stream_t stream, const char *who)
{
    nb::ConvGeom g;
    if (int rc = nb::geom_check(&g, D, H, Wd, Cw, fx, fy, px, py, sx, sy, who)) return rc;
    NB_REQUIRE(O >= 0 && O <= (1 << 24), "%s: bad output channel count %lld", who, (long long)O);
    NB_REQUIRE(K >= 0 && K < (1LL << 31), "%s: bad K=%lld", who, (long long)K);
    if (D * O == 0) return NB_OK;
    const int64_t hw = (int64_t)g.h * g.w;
    NB_REQUIRE(hw >= 1, "%s: no output pixels to take a mean over", who);
    NB_REQUIRE_PTR(thresh);
    NB_REQUIRE_PTR(bias);
    NB_REQUIRE_PTR(bias_noise);
    NB_REQUIRE_ALIGNED(bias, 2);
    NB_REQUIRE_ALIGNED(bias_noise, 2);
    const _Float16 *b = reinterpret_cast<const _Float16 *>(bias), *n = reinterpret_cast<const _Float16 *>(bias_noise);
    nb::t_last_engine = 0;
    if (int rc = nb::conv_impl<W>(thresh, in, filt, nullptr, D, H, Wd, Cw, O, fx, fy, px, py, sx, sy, 4, tap_bits, stream,
                                  who, b, n, K))
        return rc;
    if (nb::t_last_engine == 5) return NB_OK;  // the counting kernel wrote thresholds
    nb::bn_conv_thresh_launch(thresh, thresh, b, n, D, O, K, hw, nb::as_stream(stream));
    return nb::check_launch(who);
}

extern "C" {
int nb_conv_engine(int engine) { return nb::set_conv_engine(engine); }
int nb_conv_last_engine(void) { return nb::t_last_engine; }
int nb_im2col_i64(int64_t *out, const int64_t *in, int64_t D, int64_t H, int64_t W, int64_t Cw, int fx, int fy, int px,
                  int py, int sx, int sy, nb_stream_t s)
{
    return nb::im2col_impl<uint64_t>(reinterpret_cast<uint64_t *>(out), W64(in), D, H, W, Cw, fx, fy, px, py, sx, sy, s,
                                     "nb_im2col_i64");
}
int nb_im2col_i32(int32_t *out, const int32_t *in, int64_t D, int64_t H, int64_t W, int64_t Cw, int fx, int fy, int px,
                  int py, int sx, int sy, nb_stream_t s)
{
    return nb::im2col_impl<uint32_t>(reinterpret_cast<uint32_t *>(out), W32(in), D, H, W, Cw, fx, fy, px, py, sx, sy, s,
                                     "nb_im2col_i32");
}
int nb_max_pool2d_i64(int64_t *out, const int64_t *in, int64_t B, int64_t H, int64_t W, int64_t Cw, int fx, int fy,
                      int px, int py, int sx, int sy, nb_stream_t s)
{
    return nb::max_pool_impl<uint64_t>(reinterpret_cast<uint64_t *>(out), W64(in), B, H, W, Cw, fx, fy, px, py, sx, sy,
                                       s, "nb_max_pool2d_i64");
}
int nb_max_pool2d_i32(int32_t *out, const int32_t *in, int64_t B, int64_t H, int64_t W, int64_t Cw, int fx, int fy,
                      int px, int py, int sx, int sy, nb_stream_t s)
{
    return nb::max_pool_impl<uint32_t>(reinterpret_cast<uint32_t *>(out), W32(in), B, H, W, Cw, fx, fy, px, py, sx, sy,
                                       s, "nb_max_pool2d_i32");
}
int nb_conv_i64(int32_t *out, const int64_t *in, const int64_t *filt, int64_t D, int64_t H, int64_t W, int64_t Cw,
                int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits, nb_stream_t s)
{
    return nb::conv_impl<uint64_t>(out, W64(in), W64(filt), nullptr, D, H, W, Cw, O, fx, fy, px, py, sx, sy, 0,
                                   tap_bits, s, "nb_conv_i64");
}
int nb_conv_i32(int32_t *out, const int32_t *in, const int32_t *filt, int64_t D, int64_t H, int64_t W, int64_t Cw,
                int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits, nb_stream_t s)
{
    return nb::conv_impl<uint32_t>(out, W32(in), W32(filt), nullptr, D, H, W, Cw, O, fx, fy, px, py, sx, sy, 0,
                                   tap_bits, s, "nb_conv_i32");
}
int nb_conv_bn_thresholds_from_input_i64(int32_t *thresh, const int64_t *in, const int64_t *filt, const uint16_t *bias,
                                         const uint16_t *bias_noise, int64_t D, int64_t H, int64_t W, int64_t Cw,
                                         int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits,
                                         int64_t K, nb_stream_t s)
{
    return conv_bn_thresholds_impl<uint64_t>(thresh, W64(in), W64(filt), bias, bias_noise, D, H, W, Cw, O, fx, fy, px, py,
                                             sx, sy, tap_bits, K, s, "nb_conv_bn_thresholds_from_input_i64");
}
int nb_conv_bn_thresholds_from_input_i32(int32_t *thresh, const int32_t *in, const int32_t *filt, const uint16_t *bias,
                                         const uint16_t *bias_noise, int64_t D, int64_t H, int64_t W, int64_t Cw,
                                         int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits,
                                         int64_t K, nb_stream_t s)
{
    return conv_bn_thresholds_impl<uint32_t>(thresh, W32(in), W32(filt), bias, bias_noise, D, H, W, Cw, O, fx, fy, px, py,
                                             sx, sy, tap_bits, K, s, "nb_conv_bn_thresholds_from_input_i32");
}
int nb_conv_popc_sums_i64(int32_t *sums, const int64_t *in, const int64_t *filt, int64_t D, int64_t H, int64_t W,
                          int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits,
                          nb_stream_t s)
{
    return nb::conv_impl<uint64_t>(sums, W64(in), W64(filt), nullptr, D, H, W, Cw, O, fx, fy, px, py, sx, sy, 4,
                                   tap_bits, s, "nb_conv_popc_sums_i64");
}
int nb_conv_popc_sums_i32(int32_t *sums, const int32_t *in, const int32_t *filt, int64_t D, int64_t H, int64_t W,
                          int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits,
                          nb_stream_t s)
{
    return nb::conv_impl<uint32_t>(sums, W32(in), W32(filt), nullptr, D, H, W, Cw, O, fx, fy, px, py, sx, sy, 4,
                                   tap_bits, s, "nb_conv_popc_sums_i32");
}
int nb_conv_act_i64(uint8_t *out, const int64_t *in, const int64_t *filt, const int32_t *thresh, int64_t D, int64_t H,
                    int64_t W, int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits,
                    nb_stream_t s)
{
    return nb::conv_impl<uint64_t>(out, W64(in), W64(filt), thresh, D, H, W, Cw, O, fx, fy, px, py, sx, sy, 1,
                                   tap_bits, s, "nb_conv_act_i64");
}
int nb_conv_act_i32(uint8_t *out, const int32_t *in, const int32_t *filt, const int32_t *thresh, int64_t D, int64_t H,
                    int64_t W, int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits,
                    nb_stream_t s)
{
    return nb::conv_impl<uint32_t>(out, W32(in), W32(filt), thresh, D, H, W, Cw, O, fx, fy, px, py, sx, sy, 1,
                                   tap_bits, s, "nb_conv_act_i32");
}
int nb_conv_act_pack_i64(int64_t *out, const int64_t *in, const int64_t *filt, const int32_t *thresh, int64_t D,
                         int64_t H, int64_t W, int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy,
                         int pool, int tap_bits, nb_stream_t s)
{
    return nb::conv_impl<uint64_t>(out, W64(in), W64(filt), thresh, D, H, W, Cw, O, fx, fy, px, py, sx, sy,
                                   pool ? 3 : 2, tap_bits, s, "nb_conv_act_pack_i64");
}
int nb_conv_act_pack_i32(int32_t *out, const int32_t *in, const int32_t *filt, const int32_t *thresh, int64_t D,
                         int64_t H, int64_t W, int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy,
                         int pool, int tap_bits, nb_stream_t s)
{
    return nb::conv_impl<uint32_t>(out, W32(in), W32(filt), thresh, D, H, W, Cw, O, fx, fy, px, py, sx, sy,
                                   pool ? 3 : 2, tap_bits, s, "nb_conv_act_pack_i32");
}
}
