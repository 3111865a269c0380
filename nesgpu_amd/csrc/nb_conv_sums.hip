// Pixel sums of a binary conv without the conv: sums[d, o] = sum over the output pixels of
// sum_k popcount(window word k ^ filter word k) (what conv_popc_sums returns; the statistic behind the per-member mean
// of BinarizedConv2d(batch_norm=True), modules/binary.py:147-155).
//
// The sum over the pixels can be taken first.  For tap t = (i, j) and channel bit c let n1[t][c] be the number of
// output pixels whose window has a 1 at (t, c) (a position outside the image is a 0, extensions/src/batch_im2col.cu:
// 14-29).  A filter bit 0 meets n1 ones, a filter bit 1 meets hw - n1 zeros, so
//     sums[o] = sum_t sum_c ( n1[t][c] + f[t][c][o] * (hw - 2 * n1[t][c]) )
// and n1 does not depend on the filter: it is a count of image bits over the rectangle of input pixels that tap t
// sees (stride 1: rows [i - px, h + i - px) x columns [j - py, w + j - py), clipped to the image).  The work is one
// pass over the image (a few vector instructions per pixel) plus, per output channel and tap, a dot product of the
// filter word with n1, taken bit plane by bit plane: sum_c f_c * n1_c = sum_k 2^k popcount(f & plane_k).  The result
// is the same integer as the conv's; a 64->128 3x3 layer on 16x16 images takes about 3 700 vector instructions per
// member this way (measured), where the conv needs 2 300 matrix instructions and as many vector ones around them.
//
// One workgroup per member.  Counting: the member's image goes through LDS; lane c of a wave owns channel bit c of
// the current channel word and first counts every pixel for every tap (a flat pass, 16 pixels per step, the four waves
// in turn), then takes the few border rows, border columns and corner pixels off the taps that do not see them.  The
// four waves' counts meet in LDS and are cut into bit planes with ballots; then wave w takes the filter words w, w + 4,
// ... of every output channel (a lane per channel) and the waves' parts of a channel meet in an LDS sum.
#include "nb_conv_common.hpp"

namespace nb {

constexpr int kCsMaxF = 5;        // filter extent per axis
constexpr int kCsMaxPlanes = 24;  // bits of hw (the planes are spelled out below)
constexpr int kCsMaxWords = 100;  // taps * Cw: plane words kept in LDS (19 KB at 24 planes)
constexpr int kCsChunkWords = 4096;  // pixels of an image chunk in LDS (32 KB)
constexpr int kCsBatch = 8;          // filter words a thread has in flight
constexpr int kCsChanChunk = 2048;   // output channels summed in LDS at a time, at most

// lane `LANE` (a literal) of w = the scalar value v; the other lanes keep theirs
#define NB_CS_WRITELANE(w, v, LANE) asm("v_writelane_b32 %0, %1, %2" : "+v"(w) : "s"(v), "n"(LANE))

struct CsConv {
    const uint64_t *in, *filt;
    int32_t *out;
    int H, Wd, Cw, h, w, fx, fy, px, py, O;
    int taps, nplanes, hw, rows_chunk, chunk_words, n1_ints, chan_chunk;
    int tap_bits, tapT, fwords;  // tap-packed filters: bits per tap, taps per word, filter words per channel
    const _Float16 *bias, *noise;  // not null: write the batch-norm layer's thresholds instead of the sums
    long long K;
    float mean_factor;  // what the fp32 sum of a (member, channel)'s activations is multiplied by for its mean
};

// F: the largest filter extent the instance is built for (3 or kCsMaxF); the per-tap code is spelled out F x F times
template <int F>
__global__ __launch_bounds__(256) void conv_sums_count_kernel(const CsConv p)
{
    // LDS, sized by the launch (small layers leave room for many workgroups per CU): the image chunk, the bit planes
    // of the counts, the counts n1[taps][64] (later the channels' sums), and asum[t * Cw + cw] = sum_c n1[t][c]
    extern __shared__ uint64_t cs_lds[];
    uint64_t *chunk = cs_lds;
    uint64_t *planes = chunk + p.chunk_words;
    int *n1 = reinterpret_cast<int *>(planes + p.taps * p.Cw * p.nplanes);
    int *asum = n1 + p.n1_ints;
    const int64_t d = blockIdx.x;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int bit = lane & 31, half = lane >> 5;
    // column and row ranges of the taps (uniform)
    int clo[F], chi[F], rlo[F], rhi[F];
#pragma unroll
    for (int j = 0; j < F; j++) {
        const int a = j - p.py, b = p.w + j - p.py;
        clo[j] = a < 0 ? 0 : (a > p.Wd ? p.Wd : a);
        chi[j] = b > p.Wd ? p.Wd : (b < clo[j] ? clo[j] : b);
        const int ar = j - p.px, br = p.h + j - p.px;
        rlo[j] = ar < 0 ? 0 : (ar > p.H ? p.H : ar);
        rhi[j] = br > p.H ? p.H : (br < rlo[j] ? rlo[j] : br);
    }
    // inner rows / columns: seen by every tap (possibly none)
    int irlo = 0, irhi = p.H, iclo = 0, ichi = p.Wd;
#pragma unroll
    for (int j = 0; j < F; j++) {
        if (j < p.fx) irlo = rlo[j] > irlo ? rlo[j] : irlo, irhi = rhi[j] < irhi ? rhi[j] : irhi;
        if (j < p.fy) iclo = clo[j] > iclo ? clo[j] : iclo, ichi = chi[j] < ichi ? chi[j] : ichi;
    }
    irhi = irhi < irlo ? irlo : irhi;
    ichi = ichi < iclo ? iclo : ichi;
    const uint64_t *img = p.in + d * (int64_t)p.H * p.Wd * p.Cw;
    // The last part gives wave w the filter words tw = w, w + 4, ... of every output channel (lane l: channels l,
    // l + 64, ...); the first kCsBatch of them are requested here, before the counting.
    const uint64_t *fz = p.filt + d * (int64_t)p.fwords * p.O;
    const uint64_t tmask = p.tap_bits ? ((1ull << p.tap_bits) - 1ull) : ~0ull;
    const int TW = p.taps * p.Cw;
    auto fword = [&](int o, int tw) -> uint64_t {  // tw is uniform: the division is a scalar one
        if (o >= p.O || tw >= TW) return 0ull;
        return fz[(int64_t)(p.tap_bits ? tw / p.tapT : tw) * p.O + o];
    };
    uint64_t fpre[kCsBatch];
#pragma unroll
    for (int b2 = 0; b2 < kCsBatch; b2++) fpre[b2] = fword(lane, wv + 4 * b2);
    for (int cw = 0; cw < p.Cw; cw++) {
        for (int i = threadIdx.x; i < p.taps * 64; i += 256) n1[i] = 0;
        int acc[F][F];
#pragma unroll
        for (int i = 0; i < F; i++)
#pragma unroll
            for (int j = 0; j < F; j++) acc[i][j] = 0;
        // The image goes through LDS in chunks of whole rows (word cw of every pixel, low halves and high halves apart):
        // the loads of a chunk are all in flight together, and a lane then reads the halves that hold its bit, four
        // pixels at a time (one address per half wave: a broadcast).
        //
        // Every pixel is first counted for every tap (one flat pass, a quarter of the chunk per wave).  The rows and
        // columns that some tap does not see are few (filter extent - 1 at either end) and are set right afterwards:
        // a border row's sum over the inner columns comes off the taps that do not see the row, a border column's sum
        // over the inner rows off those that do not see the column, a corner pixel off those that miss either.
        for (int r0 = 0; r0 < p.H; r0 += p.rows_chunk) {
            const int nr = p.H - r0 < p.rows_chunk ? p.H - r0 : p.rows_chunk;
            const int npix = nr * p.Wd, npad = (npix + 15) & ~15;
            __syncthreads();  // the chunk before has been read (and n1 is zero)
            uint32_t *c32 = reinterpret_cast<uint32_t *>(chunk);
            for (int i = threadIdx.x; i < npad; i += 256) {
                const uint64_t v = i < npix ? __builtin_nontemporal_load(img + ((int64_t)r0 * p.Wd + i) * p.Cw + cw) : 0ull;
                c32[i] = (uint32_t)v;
                c32[p.chunk_words + i] = (uint32_t)(v >> 32);
            }
            __syncthreads();
            const uint32_t *mine = c32 + half * p.chunk_words;
            auto pix = [&](int rr, int col) { return (int)((mine[rr * p.Wd + col] >> bit) & 1u); };
            // flat pass: groups of 16 pixels, dealt out to the waves in turn
            int tot = 0;
            for (int q = wv * 16; q < npad; q += 64) {
                const uint4 a = *reinterpret_cast<const uint4 *>(mine + q), b = *reinterpret_cast<const uint4 *>(mine + q + 4);
                const uint4 c = *reinterpret_cast<const uint4 *>(mine + q + 8), e = *reinterpret_cast<const uint4 *>(mine + q + 12);
                tot += (int)(((a.x >> bit) & 1u) + ((a.y >> bit) & 1u)) + (int)(((a.z >> bit) & 1u) + ((a.w >> bit) & 1u));
                tot += (int)(((b.x >> bit) & 1u) + ((b.y >> bit) & 1u)) + (int)(((b.z >> bit) & 1u) + ((b.w >> bit) & 1u));
                tot += (int)(((c.x >> bit) & 1u) + ((c.y >> bit) & 1u)) + (int)(((c.z >> bit) & 1u) + ((c.w >> bit) & 1u));
                tot += (int)(((e.x >> bit) & 1u) + ((e.y >> bit) & 1u)) + (int)(((e.z >> bit) & 1u) + ((e.w >> bit) & 1u));
            }
#pragma unroll
            for (int i = 0; i < F; i++)
#pragma unroll
                for (int j = 0; j < F; j++) acc[i][j] += tot;
            // border rows of this chunk and border columns, dealt out to the waves in turn
            int item = 0;
            for (int rr = 0; rr < nr; rr++) {
                const int r = r0 + rr;
                if (r >= irlo && r < irhi) {  // inner rows: skip to their end
                    rr += (irhi < r0 + nr ? irhi : r0 + nr) - r - 1;
                    continue;
                }
                if ((item++ & 3) != wv) continue;
                int s = 0;
#pragma unroll 8
                for (int col = iclo; col < ichi; col++) s += pix(rr, col);
                // what tap column j sees of the row: the inner columns and the corner pixels inside its range
                int full = s, seen[F];
#pragma unroll
                for (int j = 0; j < F; j++) seen[j] = s;
                for (int col = 0; col < p.Wd; col++) {
                    if (col >= iclo && col < ichi) {
                        col = ichi - 1;
                        continue;
                    }
                    const int v = pix(rr, col);
                    full += v;
#pragma unroll
                    for (int j = 0; j < F; j++) seen[j] += (col >= clo[j] && col < chi[j]) ? v : 0;
                }
#pragma unroll
                for (int i = 0; i < F; i++) {
                    const bool in = r >= rlo[i] && r < rhi[i];
#pragma unroll
                    for (int j = 0; j < F; j++) acc[i][j] -= in ? full - seen[j] : full;
                }
            }
            for (int col = 0; col < p.Wd; col++) {
                if (col >= iclo && col < ichi) {
                    col = ichi - 1;
                    continue;
                }
                if ((item++ & 3) != wv) continue;
                int s = 0;
                const int ra = irlo > r0 ? irlo : r0, rb = irhi < r0 + nr ? irhi : r0 + nr;
#pragma unroll 8
                for (int r = ra; r < rb; r++) s += pix(r - r0, col);
#pragma unroll
                for (int j = 0; j < F; j++) {
                    const int off = (col >= clo[j] && col < chi[j]) ? 0 : s;
#pragma unroll
                    for (int i = 0; i < F; i++) acc[i][j] -= off;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < F; i++)
#pragma unroll
            for (int j = 0; j < F; j++)
                if (i < p.fx && j < p.fy) atomicAdd(&n1[(i * p.fy + j) * 64 + lane], acc[i][j]);
        __syncthreads();
        // bit planes of the counts: plane k of (tap, cw) is the ballot of bit k over the 64 channel bits; the ballots
        // of a tap are handed to lanes 0 .. nplanes-1 and stored together
        for (int t = wv; t < p.taps; t += 4) {
            // tap-packed filters only see the channel bits: input bits above them count for nothing, as in the conv kernels
            const int v = (p.tap_bits && lane >= p.tap_bits) ? 0 : n1[t * 64 + lane];
            int a = 0;
            uint32_t lo = 0, hi = 0;
#define NB_CS_PLANE(K)                                    \
    if (K < p.nplanes) {                                  \
        const uint64_t m = __ballot(v & (1 << K));        \
        a += __popcll(m) << K;                            \
        NB_CS_WRITELANE(lo, (uint32_t)m, K);              \
        NB_CS_WRITELANE(hi, (uint32_t)(m >> 32), K);      \
    }
            NB_CS_PLANE(0) NB_CS_PLANE(1) NB_CS_PLANE(2) NB_CS_PLANE(3) NB_CS_PLANE(4) NB_CS_PLANE(5)
            NB_CS_PLANE(6) NB_CS_PLANE(7) NB_CS_PLANE(8) NB_CS_PLANE(9) NB_CS_PLANE(10) NB_CS_PLANE(11)
            NB_CS_PLANE(12) NB_CS_PLANE(13) NB_CS_PLANE(14) NB_CS_PLANE(15) NB_CS_PLANE(16) NB_CS_PLANE(17)
            NB_CS_PLANE(18) NB_CS_PLANE(19) NB_CS_PLANE(20) NB_CS_PLANE(21) NB_CS_PLANE(22) NB_CS_PLANE(23)
#undef NB_CS_PLANE
            if (lane < p.nplanes) planes[(t * p.Cw + cw) * p.nplanes + lane] = ((uint64_t)hi << 32) | lo;
            if (lane == 0) asum[t * p.Cw + cw] = a;
        }
        __syncthreads();
    }
    // ---- sums[o] = sum over (tap, cw) of ( asum + hw * popcount(f) - 2 * sum_k 2^k popcount(f & plane_k) ) ------------
    // Wave w takes the words tw = w, w + 4, ... (uniform over the wave: the planes are read at one address), lane l the
    // channels l, l + 64, ...; kCsBatch filter words are requested together; the four waves' parts of a channel meet in
    // an LDS sum.
    int *osum = n1;  // the counts are in the planes by now
    for (int o0 = 0; o0 < p.O; o0 += p.chan_chunk) {
        const int oc = p.O - o0 < p.chan_chunk ? p.O - o0 : p.chan_chunk;
        for (int i = threadIdx.x; i < oc; i += 256) osum[i] = 0;
        __syncthreads();
        for (int oq = lane; oq < oc; oq += 64) {
            int part = 0, dot = 0;
            for (int tb = wv; tb < TW; tb += 4 * kCsBatch) {
                uint64_t f[kCsBatch];
                if (o0 == 0 && oq == lane && tb == wv) {
#pragma unroll
                    for (int b2 = 0; b2 < kCsBatch; b2++) f[b2] = fpre[b2];
                } else {
#pragma unroll
                    for (int b2 = 0; b2 < kCsBatch; b2++) f[b2] = fword(o0 + oq, tb + 4 * b2);
                }
#pragma unroll
                for (int b2 = 0; b2 < kCsBatch; b2++) {
                    const int tw = tb + 4 * b2;
                    if (tw >= TW) break;
                    uint64_t fv = f[b2];
                    if (p.tap_bits) fv = (fv >> (p.tap_bits * (tw % p.tapT))) & tmask;
                    const uint64_t *pl = planes + tw * p.nplanes;
                    int k = 0;
                    for (; k + 2 <= p.nplanes; k += 2) {
                        const uint64_t p0 = pl[k], p1 = pl[k + 1];
                        dot += (__popcll(fv & p0) << k) + (__popcll(fv & p1) << (k + 1));
                    }
                    if (k < p.nplanes) dot += __popcll(fv & pl[k]) << k;
                    part += asum[tw] + p.hw * __popcll(fv);
                }
            }
            atomicAdd(&osum[oq], part - 2 * dot);
        }
        __syncthreads();
        for (int i = threadIdx.x; i < oc; i += 256) {
            const int64_t at = d * p.O + o0 + i;
            p.out[at] = p.bias ? bn_conv_threshold(osum[i], p.bias[o0 + i], p.noise[at], p.K, p.hw, p.mean_factor) : osum[i];
        }
        __syncthreads();
    }
}

// Pixel sums (mode 4 of the conv) for 64-bit words, stride 1, filters of at most 5 x 5: true = launched.  With bias /
// noise the batch-norm layer's thresholds are written instead (K = channels x taps).
bool conv_sums_count_try(int32_t *out, const uint64_t *in, const uint64_t *filt, const ConvGeom &g, int64_t D, int O,
                         int tap_bits, hipStream_t s, const _Float16 *bias, const _Float16 *noise, int64_t K)
{
    if (g.sx != 1 || g.sy != 1 || g.fx > kCsMaxF || g.fy > kCsMaxF || g.fx < 1 || g.fy < 1) return false;
    if (g.Cw < 1 || D < 1 || O < 1 || g.h < 1 || g.w < 1 || D > kMaxGridX) return false;
    const int taps = g.fx * g.fy;
    if ((int64_t)taps * g.Cw > kCsMaxWords) return false;
    const int64_t hw = (int64_t)g.h * g.w;
    if (hw >= (1LL << (kCsMaxPlanes - 1)) || hw * taps * g.Cw * 64 >= (1LL << 31)) return false;
    if (g.Wd > kCsChunkWords) return false;  // a row of the image must fit the LDS chunk
    CsConv p;
    p.in = in; p.filt = filt; p.out = out;
    p.bias = bias; p.noise = noise; p.K = K;
    p.H = g.H; p.Wd = g.Wd; p.Cw = g.Cw; p.h = g.h; p.w = g.w; p.fx = g.fx; p.fy = g.fy; p.px = g.px; p.py = g.py;
    p.O = O;
    p.taps = taps;
    const int64_t pixels = (int64_t)g.H * g.Wd;
    p.rows_chunk = pixels <= kCsChunkWords ? g.H : kCsChunkWords / g.Wd;
    p.chunk_words = (p.rows_chunk * g.Wd + 15) & ~15;  // dwords of a half; padded for the 16-pixel groups
    p.chan_chunk = O < kCsChanChunk ? O : kCsChanChunk;
    p.n1_ints = taps * 64 > p.chan_chunk ? taps * 64 : p.chan_chunk;
    p.hw = (int)hw;
    p.mean_factor = mean_factor(D * O, D * O * hw);
    p.nplanes = 1;
    while ((1LL << p.nplanes) <= hw) p.nplanes++;
    p.tap_bits = tap_bits;
    p.tapT = tap_bits ? 64 / tap_bits : 1;
    p.fwords = tap_bits ? (taps + p.tapT - 1) / p.tapT : taps * g.Cw;
    const size_t lds = (size_t)p.chunk_words * 8 + (size_t)taps * g.Cw * p.nplanes * 8 + (size_t)p.n1_ints * 4 +
                       (size_t)taps * g.Cw * 4;
    if (g.fx <= 3 && g.fy <= 3)
        conv_sums_count_kernel<3><<<dim3((unsigned)D), dim3(256), lds, s>>>(p);
    else
        conv_sums_count_kernel<kCsMaxF><<<dim3((unsigned)D), dim3(256), lds, s>>>(p);
    return true;
}

}  // namespace nb
