// Binary conv on the matrix cores (3-row filters, stride 1): a persistent producer / consumer kernel.
//
// CDNA4 has no 1-bit MFMA, but v_mfma_i32_16x16x64_i8 does 16384 int8 MACs per wave in 16 cycles: 4x the
// bit-MAC rate of v_xor + v_bcnt.  Bits are expanded to +-1 bytes (bit 1 -> +1, bit 0 -> -1; an out-of-range
// pixel is the zero word, i.e. all -1), the int32 dot product over the K expanded positions is exact, and
//     popcount(x ^ w) = (K - dot) / 2
// gives back the reference's sum bit for bit.
// A second flavour (template parameter Q = 1) expands to FP4 (E2M1) codes instead, two positions per byte, and
// multiplies with v_mfma_scale_f32_16x16x128_f8f6f4 at unit scales: 128 positions per instruction in the same 16
// cycles.  +1, -1 and 0 are exact in E2M1, the fp32 sums are integers far below 2^24, so the result is the same
// integer.  It exists for full channel words (64, 128 or 256 channels), where a filter row then takes 2, 3 or 6
// instructions instead of 3, 6 or 12; its byte geometry is that of the +-1 flavour with half the bytes per pixel.
//
// One workgroup per CU (8 or 12 consumer waves + 4 producer waves) walks through its share of the population.  A
// task is a band of output rows of one member for one group of up to 64 output channels.  The producer waves
// prepare task k while the consumer waves multiply task k-1, one barrier per step:
//   producer: the band's input words and, when the (member, channel group) changes, the filter words were
//     requested one step ahead; it expands the input rows (with the zero-word border, so the implicit im2col
//     needs no bounds checks) into one of two LDS image buffers and the filter words into MFMA B fragments in an
//     LDS staging area, then requests the words of task k+1;
//   consumer: a wave owns 16*NT of the task's channels; it copies new fragments into registers (they stay there
//     for all bands of the member), then walks DOWN a strip of 16 output columns: the A fragment of image row r
//     and tap column j is the same 16 pixels x 64 positions whichever filter row it meets, so it is read from LDS
//     once and multiplied into the three output rows r, r-1, r-2.  One ds_read_b128 feeds 3*NT MFMAs.  Finished rows leave straight to
//     global memory: int32 sums via a per-wave LDS transpose (full pixel rows, non-temporal), or threshold bits
//     gathered with ballots into packed words, optionally 2x2 OR-pooled (in x a min over neighbouring
//     accumulator registers, in y over two walked rows), or sums over the pixels (atomic adds).
// Each SIMD holds two or three consumer waves and one producer wave: one wave alone cannot issue MFMAs back to
// back, and the expansion work (VALU, LDS, memory latency) runs beside the MFMAs instead of in front of them.
// The producer waves run at raised issue priority and issue the same loads on every step (which keeps the
// compiler's wait counts exact), so that they are done early in the step and the consumers set its length.
//
// Fragment layout of v_mfma_i32_16x16x64_i8 (checked on hardware): lane l supplies row l%16 of A and
// column l%16 of B, its 16 bytes are the K-positions 16*(l/16)..+15 of the 64-chunk (any bijection works as
// long as A and B use the same one), and acc[r] is D[4*(l/16) + r][l%16].
//
// K chunks of one filter row (the per-pixel byte count CB is 16, 32 or 64*Cw as +-1 bytes, 32*Cw as FP4 codes):
//   CB = 16: one chunk, lane group g holds tap column g (up to 4 columns);
//   CB = 32: chunk q holds tap columns 2q and 2q+1, 32 positions each;
//   CB >= 64: one chunk per (tap column, 64-position channel word).
// Chunks of tap columns past the filter width multiply by zero bytes.
#include <atomic>
#include <type_traits>

#include "nb_conv_common.hpp"

namespace nb {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

// Consumer waves: two per SIMD keep the matrix core issuing back to back; kernels whose filter fragments are few
// (at most 128 registers in all) run three per SIMD, which hides more of the per-row latency chains that dominate
// when a row step has only a handful of MFMAs.
constexpr int rw_cwaves(int CPR, int NT) { return CPR * NT <= 4 ? 12 : 8; }
constexpr int kRwPWaves = 4;      // producer waves
constexpr int kRwTeam = 64 * kRwPWaves;  // producer threads
constexpr int kRwLutBytes = 256 * 8;  // byte -> 8 bytes of +-1
constexpr int kRwMaxCPR = 6;
constexpr int kRwTabBytes = 3 * kRwMaxCPR * 4 * 8;  // (chunk, lane group) -> filter word offset, shift, mask
// dynamic LDS a launch may ask for: the CU's 160 KB minus the kernel's two static tables
constexpr int kRwMaxDynLds = 160 * 1024 - kRwLutBytes - kRwTabBytes - 512;
constexpr int kRwItems = 10;      // input words a producer thread holds in flight

struct RwConv {
    const uint64_t *in;
    const uint64_t *filt;
    const int32_t *thresh;
    void *out;
    int64_t D;
    int H, Wd, Cw, px, py, h, w, O, fy;
    int CB;            // expanded bytes per pixel: 16, 32 or 64*Cw as +-1 bytes; 32*Cw as FP4 codes
    int PS;            // pixel stride in the LDS image, bytes (PS/16 odd: conflict-free 16-lane b128 reads)
    int RW;            // pixels per LDS image row
    int hs, S;         // output rows per band, bands per member
    int hb, nsub;      // output rows per sub-band (even), sub-bands per band
    int ntx, ncg;      // 16-column strips, channel groups (of 16*NT*cgt channels) = tasks per band
    int cgt;           // consumer channel tiles (of 16*NT channels) per task: 1, 2 or 4
    int K;             // expanded positions that count: taps * CB
    int in_bits;       // valid channel bits per pixel
    int tapT, tapM;    // tap-packed filter: taps per word and ceil(65536 / tapT) + 1 (0: one word per tap and channel word)
    int img_bytes;     // one image buffer
    int nbst;          // fragment staging areas: 1, or 2 when every task brings new fragments
    int fwords;        // filter words per member
    int pix_q, pix_r;  // team threads / RW and % RW: image-pixel advance of one fill pass
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

// 8 bits -> 8 FP4 (E2M1) codes, bit j -> nibble j: 1 -> 0x2 (+1.0), 0 -> 0xA (-1.0)
__device__ __forceinline__ uint32_t rw_pm1_fp4(uint32_t b)
{
    uint32_t w = 0;
#pragma unroll
    for (int j = 0; j < 8; j++) w |= (((b >> j) & 1u) ? 0x2u : 0xAu) << (4 * j);
    return w;
}

// One matrix-core step on 16-byte fragments.  Q = 0: v_mfma_i32_16x16x64_i8 on +-1 bytes (64 positions).  Q = 1:
// v_mfma_scale_f32_16x16x128_f8f6f4 on FP4 codes with unit scales (128 positions, the same issue time: twice the
// rate); +-1 and 0 are exact in E2M1 and the fp32 sums are integers far below 2^24, so the result is exact too.
template <int Q>
struct RwAcc {
    typedef v4i type;
    typedef int scalar;
};
template <>
struct RwAcc<1> {
    typedef v4f type;
    typedef float scalar;
};
__device__ __forceinline__ v4i rw_mfma(v4i a, v4i b, v4i c) { return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0); }
__device__ __forceinline__ v4f rw_mfma(v4i a, v4i b, v4f c)
{
    const v8i a8 = __builtin_shufflevector(a, a, 0, 1, 2, 3, -1, -1, -1, -1);
    const v8i b8 = __builtin_shufflevector(b, b, 0, 1, 2, 3, -1, -1, -1, -1);
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b8, c, 4, 4, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
}

__device__ __forceinline__ uint64_t rw_sel4(int r, uint64_t a, uint64_t b, uint64_t c, uint64_t d)
{
    return r == 0 ? a : r == 1 ? b : r == 2 ? c : d;
}

// Position of a workgroup in its task sequence: members blockIdx.x, blockIdx.x + gridDim.x, ...; per member the
// channel groups, per channel group the bands.
struct RwTask {
    int64_t z;
    int cg, band;
};
__device__ __forceinline__ void rw_next(RwTask &t, const RwConv &p)
{
    if (++t.band == p.S) {
        t.band = 0;
        if (++t.cg == p.ncg) {
            t.cg = 0;
            t.z += gridDim.x;
        }
    }
}

// MODE 0: int32 popcount sums [D,h,w,O]; 2: threshold bits packed along O; 3: the same, 2x2 OR-pooled;
// 4: the popcount sums added up over the pixels, int32 [D,O] (atomic adds into a zeroed array).
// Q: 0 = +-1 bytes and the int8 MFMA, 1 = FP4 codes and the FP4 MFMA (full channel words only).
template <int CPR, int NT, int MODE, int Q>
__global__ __launch_bounds__(64 * (rw_cwaves(CPR, NT) + kRwPWaves)) void conv_mfma_kernel(const RwConv p)
{
    typedef typename RwAcc<Q>::type acc_t;    // accumulator fragment
    typedef typename RwAcc<Q>::scalar acc_s;  // one dot product
    constexpr int PPL = Q ? 32 : 16;          // positions in a lane's 16 bytes
    constexpr int kRwCWaves = rw_cwaves(CPR, NT);
    constexpr int FX = 3;
    constexpr int NK = FX * CPR;
    constexpr int NF = NK * NT;                  // fragments of one consumer channel tile
    constexpr int CGTMAX = 4 / NT;               // a task covers at most 64 channels
    constexpr int FPW = (NF * CGTMAX + kRwPWaves - 1) / kRwPWaves;  // fragments per producer wave, at most
    constexpr int kFragBytes = NF * CGTMAX * 1024 + 64 * 4;         // + the task's thresholds
    // The two small tables are objects of their own, so that the compiler knows that the stores into the image and
    // staging buffers never alias the table look-ups and can keep many look-ups in flight.
    __shared__ __align__(16) uint2 lut_s[kRwLutBytes / 8];
    __shared__ __align__(16) uint2 tab[kRwTabBytes / 8];
    extern __shared__ __align__(16) unsigned char lds[];
    unsigned char *img0 = lds;
    unsigned char *bst0 = img0 + 2 * p.img_bytes;
    int *stage0 = reinterpret_cast<int *>(bst0 + p.nbst * kFragBytes);  // MODE 0 only

    const int tid = threadIdx.x, lane = tid & 63;
    // The wave index must be visibly uniform: every branch around MFMAs below has to be a scalar branch, because
    // MFMA ignores EXEC and a masked-off block that is not jumped over would still accumulate.
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool producer = wv >= kRwCWaves;
    const int tw = producer ? wv - kRwCWaves : wv;            // wave inside the team
    const int ttid = tid - (producer ? 64 * kRwCWaves : 0);   // thread inside the team
    const int li = lane & 15, lg = lane >> 4;
    const int Ow = (p.O + 63) >> 6;

    // Expansion table: entry b holds the +-1 bytes of bits 0..7 of b.  The expansion work shares the SIMDs' issue
    // slots with the MFMAs, so it is written for the fewest instructions: two ALU operations and one 8-byte look-up
    // per 8 bits (bank conflicts between look-ups cost LDS time, which is plentiful, not issue slots).
    // (FP4: entry b holds the 8 codes of b in 4 bytes.)
    if (tid < 256) {
        if (Q) {
            reinterpret_cast<uint32_t *>(lut_s)[tid] = rw_pm1_fp4(tid);
        } else {
            lut_s[tid] = make_uint2(rw_pm1_bytes(tid & 0xFu), rw_pm1_bytes((unsigned)tid >> 4));
        }
    }
    const unsigned char *lutb = reinterpret_cast<const unsigned char *>(lut_s);
    // FP4: 32 bits -> 16 bytes of codes, four 4-byte look-ups
    auto expand32_fp4 = [&](uint32_t x) {
        const uint32_t a = *reinterpret_cast<const uint32_t *>(lutb + ((x << 2) & 0x3FCu));
        const uint32_t b = *reinterpret_cast<const uint32_t *>(lutb + ((x >> 6) & 0x3FCu));
        const uint32_t c = *reinterpret_cast<const uint32_t *>(lutb + ((x >> 14) & 0x3FCu));
        const uint32_t d = *reinterpret_cast<const uint32_t *>(lutb + ((x >> 22) & 0x3FCu));
        return make_uint4(a, b, c, d);
    };
    // bits 16*hi .. 16*hi+15 of x -> 16 bytes of +-1, bit b -> byte b
    auto expand_half = [&](uint32_t x, int hi) {
        const uint32_t i0 = hi ? (x >> 13) & 0x7F8u : (x << 3) & 0x7F8u;
        const uint32_t i1 = hi ? (x >> 21) & 0x7F8u : (x >> 5) & 0x7F8u;
        const uint2 a = *reinterpret_cast<const uint2 *>(lutb + i0), b = *reinterpret_cast<const uint2 *>(lutb + i1);
        return make_uint4(a.x, a.y, b.x, b.y);
    };

    // ---- fragment geometry ---------------------------------------------------------------------------------
    // chunk kq = i*CPR + q (filter row i) and lane group g: tap column j, first position c0.  Table entry:
    //   x = byte offset of the filter word holding the group's 16 (FP4: 32) bits (without the channel),
    //   y = shift of those bits | number of channel bits among them << 8 | (tap column inside the filter) << 31;
    // a tap column past the filter multiplies by zero bytes, channel positions past in_bits by -1 (they equal the
    // pixel's zero tail and are part of K).
    if (tid >= 64 && tid < 64 + NK * 4) {
        const int e = tid - 64;
        const int kq = e >> 2, g = e & 3;
        const int i = kq / CPR, q = kq - i * CPR;
        int qj = 0, qc = 0;
        if (p.CB == 32) {
            qj = 2 * q;
        } else if (p.CB >= 64) {
            const int nch = p.CB >> 6;  // 64-byte pieces of a pixel
            qj = q / nch;
            qc = 64 * (q - qj * nch);
        }
        const int j = qj + (g >> p.jsh);
        const int c0 = (qc + 16 * (g & p.cmask)) * (PPL / 16);  // first position of the lane group inside the pixel
        const int tap = i * p.fy + j;
        const int left = p.in_bits - c0;
        const int nv = left < 0 ? 0 : (left > PPL ? PPL : left);
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
        tab[e] = make_uint2(inside ? (uint32_t)(fr * p.O) * 8u : 0u,
                            (uint32_t)sh | ((uint32_t)nv << 8) | (inside ? 0x80000000u : 0u));
    }
    __syncthreads();  // tables complete

    // number of tasks of this workgroup
    const int64_t nmem = (int64_t)blockIdx.x < p.D ? (p.D - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    const int nsteps = (int)(nmem * p.ncg * p.S);

    if (producer) {
        // =========================================== producer ===================================================
        // Team thread ttid owns the items (pixel words) ttid, ttid + 256, ... of a band; all of a band's items are
        // in flight at once (the host sizes bands so that they fit).  The words are fetched with buffer loads whose
        // range is the member's image: a row above or below the image gives a byte offset outside the range and the
        // hardware returns the zero word, which is what an out-of-range pixel is; a column outside the image is
        // given an offset that is out of range for every row.  No bounds arithmetic per item, no select afterwards.
        // The producers' few instructions per step go first: they are the last waves of the workgroup, which the
        // SIMD's oldest-first issue would otherwise serve only when its three consumer waves stall, and the
        // consumers then wait for them at the step's barrier.
        __builtin_amdgcn_s_setprio(3);
        const int pixb = p.Cw * 8, rowb = p.Wd * pixb;  // bytes per pixel / image row
        const int prow = ttid / p.RW, pxx = ttid - prow * p.RW;
        // input words of this step's and of the next task
        uint64_t wda[kRwItems], wdb[kRwItems];
        uint64_t fw[FPW];
        int traw = 0;
        // item u of this thread is pixel ttid + 256*u of the band's LDS image: its byte offset relative to the band's
        // first input row (kOutside for a column outside the image)
        constexpr uint32_t kOutside = 0xC0000000u;  // +- any band offset (below 2^30 in size) stays past every image
        uint32_t ioff[kRwItems];
        {
            int r = prow, x = pxx;
#pragma unroll
            for (int u = 0; u < kRwItems; u++) {
                ioff[u] = (x - p.py >= 0 && x - p.py < p.Wd) ? (uint32_t)(r * rowb + (x - p.py) * pixb) : kOutside;
                r += p.pix_q;
                x += p.pix_r;
                if (x >= p.RW) {
                    x -= p.RW;
                    r++;
                }
            }
        }
        const int img_range = p.H * rowb;  // bytes of one member's image
        auto request = [&](uint64_t (&wd)[kRwItems], const RwTask &t, int cw) {
            const uint64_t *src = p.in + t.z * (int64_t)p.H * p.Wd * p.Cw;
            const __amdgpu_buffer_rsrc_t rsrc =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<uint64_t *>(src), (short)0, img_range, 0x00020000);
            const uint32_t off0 = (uint32_t)((t.band * p.hs - p.px) * rowb + cw * 8);
#pragma unroll
            for (int u = 0; u < kRwItems; u++) {
                const v2i v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)(off0 + ioff[u]), 0, 0);
                wd[u] = ((uint64_t)(uint32_t)v[1] << 32) | (uint32_t)v[0];
            }
        };
        // Filter words of a channel group: wave tw takes fragments tw, tw+4, ... (fragment f = chunk f/NT, channel
        // tile f%NT).  Every address is valid (channels past O read channel O-1, dead tap columns word 0); the
        // expansion zeroes them.
        auto request_filter = [&](const RwTask &t) {
            const unsigned char *fz = reinterpret_cast<const unsigned char *>(p.filt + t.z * (int64_t)p.fwords);
            const int n0 = t.cg * 16 * NT * p.cgt;
            const int nft = NF * p.cgt;  // fragments of the task: f = (channel tile * NK + chunk) * NT + 16-channel piece
#pragma unroll
            for (int i = 0; i < FPW; i++) {
                const int f = tw + kRwPWaves * i;  // uniform
                const int fc = f < nft ? f : 0;
                const int ct = fc / NF, r = fc - ct * NF, kq = r / NT, nt = r - kq * NT;
                const int ch = n0 + (ct * NT + nt) * 16 + li;
                fw[i] = *reinterpret_cast<const uint64_t *>(fz + (tab[kq * 4 + lg].x + (uint32_t)(ch < p.O ? ch : p.O - 1) * 8u));
            }
            if (MODE == 2 || MODE == 3) {
                const int ch = n0 + ttid;
                traw = p.thresh[t.z * p.O + (ch < p.O ? ch : p.O - 1)];
            }
        };
        RwTask cur{(int64_t)blockIdx.x, 0, 0};
        if (nsteps > 0) {
            request_filter(cur);
            request(wda, cur, 0);
        }
        int nb = 0;      // fragment sets staged so far
        int imgseq = 0;  // images expanded so far; image i sits in buffer i & 1
        // One step: `wd` holds the input words of task k (requested a step ago); those of task k+1 go to `wn` first
        // thing, so that their latency hides behind this step's work.
        auto step = [&](int k, uint64_t (&wd)[kRwItems], uint64_t (&wn)[kRwItems]) {
            if (k < nsteps) {
                RwTask nxt = cur;
                rw_next(nxt, p);
                // Every step issues the same loads (the last one asks for its own task again, a step that keeps the
                // image for another channel group asks for it anyway): the number of loads in flight behind the
                // words used below is then known when the kernel is compiled, and waiting for this task's words
                // does not wait for the next task's as well.
                const RwTask ahead = k + 1 < nsteps ? nxt : cur;
                request(wn, ahead, 0);
                const int n0 = cur.cg * 16 * NT * p.cgt;
                if (cur.band == 0) {
                    // ---- new (member, channel group): fragments and thresholds -> staging area -------------------
                    unsigned char *bst = bst0 + (nb & (p.nbst - 1)) * kFragBytes;
                    nb++;
#pragma unroll
                    for (int i = 0; i < FPW; i++) {
                        const int f = tw + kRwPWaves * i;
                        if (f < NF * p.cgt) {  // uniform
                            const int ct = f / NF, r = f - ct * NF, kq = r / NT, nt = r - kq * NT;
                            const uint32_t e = tab[kq * 4 + lg].y;
                            const uint32_t sh = e & 63u, nv = (e >> 8) & 63u;
                            const uint32_t vmask = nv >= 32u ? 0xFFFFFFFFu : (1u << nv) - 1u;
                            const bool live = (int)e < 0 && n0 + (ct * NT + nt) * 16 + li < p.O;
                            const uint32_t fbits = (uint32_t)(fw[i] >> sh) & vmask;
                            const uint4 e16 = Q ? expand32_fp4(fbits) : expand_half(fbits, 0);
                            *reinterpret_cast<uint4 *>(bst + (f * 64 + lane) * 16) = live ? e16 : make_uint4(0u, 0u, 0u, 0u);
                        }
                    }
                    // thresholds in dot-product terms: 2*popc > t  <=>  popc > (t>>1)  <=>  dot < K - 2*(t>>1)
                    if ((MODE == 2 || MODE == 3) && ttid < 64) {
                        int64_t td = n0 + ttid < p.O ? (int64_t)p.K - 2 * (int64_t)(traw >> 1) : -2147483648LL;
                        if (Q) {
                            // every dot product lies in [-K, K]: thresholds outside mean always / never and are
                            // pulled in to K + 1 / -K - 1, which fp32 holds exactly
                            td = td > p.K + 1 ? p.K + 1 : (td < -p.K - 1 ? -p.K - 1 : td);
                            reinterpret_cast<float *>(bst + NF * CGTMAX * 1024)[ttid] = (float)td;
                        } else {
                            td = td > 2147483647LL ? 2147483647LL : (td < -2147483648LL ? -2147483648LL : td);
                            reinterpret_cast<int *>(bst + NF * CGTMAX * 1024)[ttid] = (int)td;
                        }
                    }
                }
                // the filter words of the next task get the whole image expansion as a head start
                request_filter(ahead);
                // ---- input words -> +-1 bytes in an image buffer (kept when only the channel group changed) ---------
                if (k == 0 || p.S > 1 || cur.cg == 0) {
                    unsigned char *img = img0 + (imgseq & 1) * p.img_bytes;
                    imgseq++;
                    const int row0 = cur.band * p.hs;
                    const int hloc = p.h - row0 < p.hs ? p.h - row0 : p.hs;
                    const int npix = (hloc + FX - 1) * p.RW;
                    // Narrow pixels (at most 32 positions, one input word): the look-ups of several items are issued
                    // before the first store, so that no item waits for the LDS round trip of the one before.
                    auto fill_narrow = [&](auto pieces) {
                        constexpr int P = decltype(pieces)::value;
                        constexpr int G = P == 1 ? 5 : 2;  // items per batch: kRwItems is a multiple of both
                        unsigned char *dst = img + __mul24(ttid, p.PS);
                        const int dstep = kRwTeam * p.PS;
                        // input bits above the channel count count for nothing (the positions they would take stand
                        // for the zero tail)
                        const uint32_t inmask = p.in_bits >= 32 ? 0xFFFFFFFFu : (1u << p.in_bits) - 1u;
#pragma unroll
                        for (int u0 = 0; u0 < kRwItems; u0 += G) {
                            uint4 e[G][P];
#pragma unroll
                            for (int v = 0; v < G; v++) {
                                const uint32_t lo = (uint32_t)wd[u0 + v] & inmask;
#pragma unroll
                                for (int c = 0; c < P; c++) e[v][c] = expand_half(lo, c);
                            }
#pragma unroll
                            for (int v = 0; v < G; v++) {
                                if (ttid + (u0 + v) * kRwTeam < npix) {
#pragma unroll
                                    for (int c = 0; c < P; c++) *reinterpret_cast<uint4 *>(dst + 16 * c) = e[v][c];
                                }
                                dst += dstep;
                            }
                        }
                    };
                    if (Q == 0 && CPR == 1 && p.CB == 16) {
                        fill_narrow(std::integral_constant<int, 1>{});
                    } else if (Q == 0 && CPR <= 2 && p.CB == 32) {
                        fill_narrow(std::integral_constant<int, 2>{});
                    } else
                    for (int cw = 0; cw < p.Cw; cw++) {
                        if (cw > 0) request(wd, cur, cw);
                        const int nbytes = Q ? 32 : (p.CB - cw * 64 < 64 ? p.CB - cw * 64 : 64);  // bytes this word expands to
                        unsigned char *dst = img + __mul24(ttid, p.PS) + cw * (Q ? 32 : 64);
                        const int dstep = kRwTeam * p.PS;
#pragma unroll
                        for (int u = 0; u < kRwItems; u++) {
                            if (ttid + u * kRwTeam < npix) {
                                const uint32_t lo = (uint32_t)wd[u], hi = (uint32_t)(wd[u] >> 32);
                                if (Q) {
                                    *reinterpret_cast<uint4 *>(dst) = expand32_fp4(lo);
                                    *reinterpret_cast<uint4 *>(dst + 16) = expand32_fp4(hi);
                                } else {
#pragma unroll
                                    for (int c = 0; c < 4; c++)
                                        if (16 * c < nbytes)  // uniform
                                            *reinterpret_cast<uint4 *>(dst + 16 * c) = expand_half(c < 2 ? lo : hi, c & 1);
                                }
                            }
                            dst += dstep;
                        }
                    }
                }
                cur = nxt;
            }
            __syncthreads();
        };
        for (int k = 0; k <= nsteps; k += 2) {
            step(k, wda, wdb);
            if (k + 1 <= nsteps) step(k + 1, wdb, wda);
        }
        return;
    }

    // ============================================= consumer =====================================================
    int koff[CPR];  // byte offset of the lane's 16 positions relative to the strip's first pixel
#pragma unroll
    for (int q = 0; q < CPR; q++) {
        const int j = p.qj[q] + (lg >> p.jsh);
        koff[q] = __mul24((j < p.fy ? j : 0) + li, p.PS) + p.qc[q] + 16 * (lg & p.cmask);
    }
    v4i B[NK][NT];
    acc_s tdot[NT];
#pragma unroll
    for (int kq = 0; kq < NK; kq++)
#pragma unroll
        for (int nt = 0; nt < NT; nt++) B[kq][nt] = (v4i){0, 0, 0, 0};
#pragma unroll
    for (int nt = 0; nt < NT; nt++) tdot[nt] = 0;
    int *stage = stage0 + tw * (16 * 16 * NT);  // MODE 0 only
    // Wave tw always works on channel tile ct of a task (so its fragments stay valid over a member's bands) and
    // shares the (strip, sub-band) units of that tile with the other waves of the same tile.
    const int ct = tw % p.cgt, uw = tw / p.cgt, ustep = kRwCWaves / p.cgt;
    const int nunits = p.ntx * p.nsub;
    RwTask cur{(int64_t)blockIdx.x, 0, 0};
    int nb = 0, imgseq = 0;
    for (int k = 0; k <= nsteps; k++) {
        if (k > 0) {
            // task k-1: image number imgseq, new fragments in staging area nb % nbst
            const int64_t z = cur.z;
            const int cg = cur.cg;
            const int n0 = (cg * p.cgt + ct) * 16 * NT;  // first channel of the wave's tile
            const int row0 = cur.band * p.hs;
            const int hloc = p.h - row0 < p.hs ? p.h - row0 : p.hs;
            if (k == 1 || p.S > 1 || cg == 0) imgseq++;
            const unsigned char *img = img0 + ((imgseq - 1) & 1) * p.img_bytes;
            if (cur.band == 0) {
                const unsigned char *bst = bst0 + (nb & (p.nbst - 1)) * kFragBytes;
                nb++;
#pragma unroll
                for (int kq = 0; kq < NK; kq++)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        B[kq][nt] = *reinterpret_cast<const v4i *>(bst + (((ct * NK + kq) * NT + nt) * 64 + lane) * 16);
                if (MODE == 2 || MODE == 3) {
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        tdot[nt] = reinterpret_cast<const acc_s *>(bst + NF * CGTMAX * 1024)[(ct * NT + nt) * 16 + li];
                }
            }
            for (int u = uw; u < nunits; u += ustep) {
                const int sub = u / p.ntx, strip = u - sub * p.ntx;
                const int ys = sub * p.hb;
                const int ye = ys + p.hb < hloc ? ys + p.hb : hloc;
                if (ys >= ye) continue;  // wave-uniform
                const int x0 = strip * 16;

            acc_s pend[NT][2];  // MODE 3: x-pooled minima of the even row of a pair
#pragma unroll
            for (int nt = 0; nt < NT; nt++) pend[nt][0] = pend[nt][1] = 0;
            // MODE 4: the lane's running sum of dot products over its four pixel columns (columns past the image
            // masked off) and all rows of the unit
            acc_s csum[NT];
            int cmask[4];
#pragma unroll
            for (int nt = 0; nt < NT; nt++) csum[nt] = 0;
#pragma unroll
            for (int r = 0; r < 4; r++) cmask[r] = x0 + 4 * lg + r < p.w ? -1 : 0;

            // ---- epilogue of one finished output row (band-relative y) -------------------------------------------
            // Output addresses: a uniform row pointer (scalar arithmetic) plus a per-lane 32-bit byte offset.
            unsigned char *obase;   // first element of the strip's row 0 (band-relative) for this channel group
            int64_t orowb;          // bytes from one (pooled) output row to the next
            uint32_t olane[MODE == 0 ? 16 / (64 / (4 * NT)) : 1];
            bool olive[MODE == 0 ? 16 / (64 / (4 * NT)) : 1];
            const bool piece = p.O >= 64;  // the tile's 16*NT bits are one of several pieces of the pixel's word(s)
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
                obase = static_cast<unsigned char *>(p.out) + (piece ? ((e0 + cg) << 3) + 2 * NT * ct : e0 << 3);
                orowb = ((int64_t)ww * Ow) << 3;
                olane[0] = (uint32_t)__mul24(lane, Ow) << 3;
                olive[0] = lane < (MODE == 3 ? 8 : 16) && xx0 + lane < ww;
            }
            auto finish_row = [&](acc_t (&a)[NT], int y, int par = -1) {  // par: y & 1 when the caller knows it
                if (MODE == 4) {
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        csum[nt] += (cmask[0] ? a[nt][0] : 0) + (cmask[1] ? a[nt][1] : 0) + (cmask[2] ? a[nt][2] : 0) +
                                    (cmask[3] ? a[nt][3] : 0);
                    return;
                }
                if (MODE == 0) {
                    // stage the 16 x (16*NT) tile in LDS, then store whole pixel rows (non-temporal)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            stage[(4 * lg + r) * (16 * NT) + nt * 16 + li] =
                                Q ? (int)__builtin_fmaf((float)a[nt][r], -0.5f, 0.5f * (float)p.K) : (p.K - (int)a[nt][r]) >> 1;
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
                    if ((par < 0 ? y & 1 : par) == 0) {
#pragma unroll
                        for (int nt = 0; nt < NT; nt++) {
                            pend[nt][0] = a[nt][0] < a[nt][1] ? a[nt][0] : a[nt][1];
                            pend[nt][1] = a[nt][2] < a[nt][3] ? a[nt][2] : a[nt][3];
                        }
                        return;
                    }
#pragma unroll
                    for (int nt = 0; nt < NT; nt++) {
                        acc_s v0 = a[nt][0] < a[nt][1] ? a[nt][0] : a[nt][1];
                        acc_s v1 = a[nt][2] < a[nt][3] ? a[nt][2] : a[nt][3];
                        v0 = v0 < pend[nt][0] ? v0 : pend[nt][0];
                        v1 = v1 < pend[nt][1] ? v1 : pend[nt][1];
                        const uint64_t m0 = __ballot(v0 < tdot[nt]), m1 = __ballot(v1 < tdot[nt]);
                        const uint64_t mine = (lane & 1) ? m1 : m0;  // pooled pixel 2g + q <-> lane 2g + q
                        word |= ((mine >> (16 * ((lane >> 1) & 3))) & 0xFFFFull) << (16 * nt);
                    }
                }
                unsigned char *orow = obase + (MODE == 3 ? y >> 1 : y) * orowb;
                if (olive[0]) {
                    if (piece && NT == 1) {
                        __builtin_nontemporal_store((uint16_t)(uint16_t)word, reinterpret_cast<uint16_t *>(orow + olane[0]));
                    } else if (piece) {
                        __builtin_nontemporal_store((uint32_t)(uint32_t)word, reinterpret_cast<uint32_t *>(orow + olane[0]));
                    } else {
                        __builtin_nontemporal_store((uint64_t)word, reinterpret_cast<uint64_t *>(orow + olane[0]));
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
            v4i F[CPR];
            acc_t a0[NT], a1[NT];
#pragma unroll
            for (int q = 0; q < CPR; q++) F[q] = *reinterpret_cast<const v4i *>(arow + koff[q]);
#pragma unroll
            for (int nt = 0; nt < NT; nt++) a0[nt] = a1[nt] = (acc_t){0, 0, 0, 0};
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
                            a0[nt] = rw_mfma(F[q], B[2 * CPR + q][nt], a0[nt]);
                    if (rr - 2 < ylast) finish_row(a0, rr - 2);
                }
                if (rr - 1 >= ys && rr - 1 < ye) {
#pragma unroll
                    for (int nt = 0; nt < NT; nt++) a0[nt] = a1[nt];
#pragma unroll
                    for (int q = 0; q < CPR; q++)
#pragma unroll
                        for (int nt = 0; nt < NT; nt++)
                            a0[nt] = rw_mfma(F[q], B[CPR + q][nt], a0[nt]);
                }
                if (rr < ye) {
#pragma unroll
                    for (int nt = 0; nt < NT; nt++) a1[nt] = (acc_t){0, 0, 0, 0};
#pragma unroll
                    for (int q = 0; q < CPR; q++)
#pragma unroll
                        for (int nt = 0; nt < NT; nt++)
                            a1[nt] = rw_mfma(F[q], B[q][nt], a1[nt]);
                }
#pragma unroll
                for (int q = 0; q < CPR; q++) F[q] = Fn[q];
            };
            int rr = ys;
            const int lead = ys + 2 < rend ? ys + 2 : rend;
            for (; rr < lead; rr++) edge_step(rr);
            // Steady rows two at a time: the fragments alternate between F and G (no register copies), and the first
            // row of a pair is an even output row (sub-bands start on even rows), which the pooled epilogue needs to
            // know at compile time to be free of branches.
            v4i G[CPR];
            auto row_step = [&](v4i (&Fu)[CPR], v4i (&Fl)[CPR], int r, int par) {
                acc_t done[NT];
                arow += rowbytes;
#pragma unroll
                for (int q = 0; q < CPR; q++) Fl[q] = *reinterpret_cast<const v4i *>(arow + koff[q]);
#pragma unroll
                for (int nt = 0; nt < NT; nt++) done[nt] = a0[nt];
#pragma unroll
                for (int q = 0; q < CPR; q++)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        done[nt] = rw_mfma(Fu[q], B[2 * CPR + q][nt], done[nt]);
#pragma unroll
                for (int nt = 0; nt < NT; nt++) a0[nt] = a1[nt];
#pragma unroll
                for (int q = 0; q < CPR; q++)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        a0[nt] = rw_mfma(Fu[q], B[CPR + q][nt], a0[nt]);
#pragma unroll
                for (int nt = 0; nt < NT; nt++) a1[nt] = (acc_t){0, 0, 0, 0};
#pragma unroll
                for (int q = 0; q < CPR; q++)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        a1[nt] = rw_mfma(Fu[q], B[q][nt], a1[nt]);
                finish_row(done, r - 2, par);  // r - 2 < ye - 2 <= ylast
            };
            for (; rr + 1 < ye; rr += 2) {
                row_step(F, G, rr, 0);
                row_step(G, F, rr + 1, 1);
            }
            if (rr < ye) {
                row_step(F, G, rr, 0);
#pragma unroll
                for (int q = 0; q < CPR; q++) F[q] = G[q];
                rr++;
            }
            for (; rr < rend; rr++) edge_step(rr);
            if (MODE == 4) {
                // popcount = (K - dot) / 2 per pixel: add the four lane groups, then one atomic per channel
                const int cols = p.w - x0 < 16 ? p.w - x0 : 16;
                const int kn = p.K * (ye - ys) * cols;
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    int v = (int)csum[nt];
                    v += __shfl_xor(v, 16);
                    v += __shfl_xor(v, 32);
                    const int ch = n0 + nt * 16 + li;
                    if (lg == 0 && ch < p.O) atomicAdd(static_cast<int *>(p.out) + z * p.O + ch, (kn - v) >> 1);
                }
            }
            }
            rw_next(cur, p);
        }
        __syncthreads();
    }
}

static inline int rw_round_up(int a, int b) { return (a + b - 1) / b * b; }

// Registers of a kernel instantiation and the CU count of the current device (for the workgroups-per-CU estimate).
// Written once per device: regs first, then cus with release order; a reader that sees cus != 0 sees regs too.
struct RwFit {
    std::atomic<int> cus{0}, regs{0};
};
template <int CPR, int NT, int MODE, int Q>
static bool rw_launch_one(const RwConv &p, int64_t D, size_t lds_bytes, hipStream_t s)
{
    // Per device (the attribute belongs to the device's copy of the kernel).  Threads that arrive together all
    // compute the same values and publish them through the atomics.
    constexpr int kMaxDevices = 16;
    static RwFit fits[kMaxDevices];
    auto *kfn = conv_mfma_kernel<CPR, NT, MODE, Q>;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return false;
    }
    RwFit &fit = fits[dev];
    int fit_cus = fit.cus.load(std::memory_order_acquire);
    if (fit_cus == 0) {
        hipFuncAttributes fa;
        int cus = 0;
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                kRwMaxDynLds) != hipSuccess ||
            hipFuncGetAttributes(&fa, reinterpret_cast<const void *>(kfn)) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) {
            (void)hipGetLastError();
            return false;
        }
        fit.regs.store(fa.numRegs > 0 ? fa.numRegs : 256, std::memory_order_relaxed);
        fit.cus.store(cus, std::memory_order_release);
        fit_cus = cus;
    }
    const int fit_regs = fit.regs.load(std::memory_order_relaxed);
    // 512 registers per lane and SIMD, three or four waves of a workgroup per SIMD; 160 KB of LDS per CU
    int per_cu = 512 / ((fit_regs + 7) / 8 * 8) / ((rw_cwaves(CPR, NT) + kRwPWaves) / 4);
    const int by_lds = (int)(160 * 1024 / (lds_bytes + kRwLutBytes + kRwTabBytes));
    per_cu = per_cu < by_lds ? per_cu : by_lds;
    per_cu = per_cu < 1 ? 1 : (per_cu > 4 ? 4 : per_cu);
    const int64_t wgs = D < (int64_t)fit_cus * per_cu ? D : (int64_t)fit_cus * per_cu;
    kfn<<<dim3((unsigned)wgs), dim3(64 * (rw_cwaves(CPR, NT) + kRwPWaves)), lds_bytes, s>>>(p);
    return true;
}

template <int MODE>
static bool rw_launch_mode(const RwConv &p, int64_t D, int CPR, int NT, int q, size_t lds, hipStream_t s)
{
#define NB_RW(cpr, nt, qq) \
    if (CPR == cpr && NT == nt && q == qq) return rw_launch_one<cpr, nt, MODE, qq>(p, D, lds, s)
    NB_RW(1, 1, 0);
    NB_RW(1, 2, 0);
    NB_RW(2, 1, 0);
    NB_RW(2, 2, 0);
    NB_RW(3, 1, 0);
    NB_RW(3, 2, 0);
    NB_RW(6, 1, 0);
    NB_RW(2, 1, 1);  // FP4: 64 channels (one word per pixel, two tap columns per 128-position chunk)
    NB_RW(2, 2, 1);
    NB_RW(3, 1, 1);  // FP4: 128 channels (one chunk per tap column)
    NB_RW(3, 2, 1);
    NB_RW(6, 1, 1);  // FP4: 256 channels
#undef NB_RW
    return false;
}

// One attempt with +-1 bytes (q = 0) or FP4 codes (q = 1).  Returns false when this shape has no kernel in that
// flavour; nothing has been launched then.
static bool rw_try(void *out, const uint64_t *in, const uint64_t *filt, const int32_t *thresh, const ConvGeom &g,
                   int64_t D, int O, int tap_bits, int mode, int q, hipStream_t s)
{
    if (!aligned(out, 16)) return false;
    if (mode != 0 && mode != 2 && mode != 3 && mode != 4) return false;
    if (g.sx != 1 || g.sy != 1 || g.h < 1 || g.w < 1 || D < 1) return false;
    if (g.fx != 3 || g.fy < 1 || g.fy > 3 || g.Cw < 1) return false;
    if (O < 16 || (O & 15) != 0) return false;
    if (mode == 3 && (g.h < 2 || g.w < 2)) return false;
    if (tap_bits > 0 && (g.Cw != 1 || tap_bits > 32)) return false;
    // 32-bit byte offsets inside one member's image (below 2^30, so that the out-of-range marker of the producers'
    // buffer loads stays out of range for every band offset) and filter block
    if ((int64_t)g.H * g.Wd * g.Cw * 8 >= (1LL << 30) || (int64_t)9 * g.Cw * O * 8 >= (1LL << 31)) return false;
    RwConv p;
    p.in = in;
    p.filt = filt;
    p.thresh = thresh;
    p.out = out;
    p.H = g.H; p.Wd = g.Wd; p.Cw = g.Cw; p.px = g.px; p.py = g.py; p.h = g.h; p.w = g.w;
    p.O = O;
    p.fy = g.fy;
    if (q && (tap_bits > 0 || (g.Cw != 1 && g.Cw != 2 && g.Cw != 4))) return false;
    const int CB = q ? 32 * g.Cw : tap_bits > 0 ? (tap_bits <= 16 ? 16 : 32) : 64 * g.Cw;  // bytes per pixel
    const int nch = CB >> 6;                                                              // 64-byte pieces of a pixel
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
        for (int c = 0; c < CPR; c++) { p.qj[c] = (short)(2 * c); p.qc[c] = 0; }
    } else {
        CPR = g.fy * nch;
        if (CPR > kRwMaxCPR) return false;
        p.jsh = 2; p.cmask = 3;
        for (int c = 0; c < CPR; c++) { p.qj[c] = (short)(c / nch); p.qc[c] = (short)(64 * (c % nch)); }
    }
    for (int c = CPR; c < kRwMaxCPR; c++) p.qj[c] = p.qc[c] = 0;
    if (CPR == 4 || CPR == 5) return false;
    // A consumer wave keeps the fragments of 16*NT channels in registers (at most 72 of its 168); a task covers
    // cgt such tiles: 64 channels when there are that many, else all of them.
    int NT, cgt;
    if (O >= 64) {
        NT = CPR == 6 ? 1 : 2;
        cgt = 4 / NT;
    } else if (O == 16 || (O == 32 && CPR != 6)) {
        NT = O / 16;
        cgt = 1;
    } else {
        return false;
    }
    p.cgt = cgt;
    p.ncg = (O + 16 * NT * cgt - 1) / (16 * NT * cgt);
    p.PS = ((CB >> 4) & 1) ? CB : CB + 16;
    p.ntx = (g.w + 15) / 16;
    p.RW = 16 * p.ntx + g.fy - 1;
    p.K = 3 * g.fy * (q ? 64 * g.Cw : CB);  // positions
    p.pix_q = kRwTeam / p.RW;
    p.pix_r = kRwTeam % p.RW;
    p.D = D;
    // Bands: as few as possible such that the producers hold a band's input words in flight at once and two image
    // buffers, the fragment staging areas and the int32 transpose tiles fit the CU's LDS; rows per band even.
    const int cwaves = rw_cwaves(CPR, NT);
    const int stage = mode == 0 ? cwaves * 16 * 16 * NT * 4 : 0;
    const int rowbytes = p.RW * p.PS;
    const int frag_bytes = 3 * CPR * 4 * 1024 + 64 * 4;  // NK * NT * (4 / NT) fragments + thresholds
    size_t lds = 0;
    for (p.S = 1;; p.S++) {
        p.hs = rw_round_up((g.h + p.S - 1) / p.S, 2);
        const int bands = (g.h + p.hs - 1) / p.hs;
        p.nbst = bands == 1 ? 2 : 1;  // every task brings new fragments: stage them alternately
        p.img_bytes = rw_round_up((p.hs + 2) * rowbytes + 64, 16);
        lds = 2 * (size_t)p.img_bytes + (size_t)p.nbst * frag_bytes + stage;
        if ((lds <= (size_t)kRwMaxDynLds && (p.hs + 2) * p.RW <= kRwItems * kRwTeam) || p.hs <= 2) break;
    }
    if (lds > (size_t)kRwMaxDynLds || (p.hs + 2) * p.RW > kRwItems * kRwTeam) return false;
    p.S = (g.h + p.hs - 1) / p.hs;  // bands that own at least one row
    // Sub-bands: enough (strip, sub-band) units for the consumer waves of one channel tile.
    const int wpt = cwaves / cgt;
    int nsub = p.ntx >= wpt ? 1 : (wpt + p.ntx - 1) / p.ntx;
    p.hb = rw_round_up((p.hs + nsub - 1) / nsub, 2);
    p.nsub = (p.hs + p.hb - 1) / p.hb;
    if (mode == 0) return rw_launch_mode<0>(p, D, CPR, NT, q, lds, s);
    if (mode == 2) return rw_launch_mode<2>(p, D, CPR, NT, q, lds, s);
    if (mode == 4) return rw_launch_mode<4>(p, D, CPR, NT, q, lds, s);
    return rw_launch_mode<3>(p, D, CPR, NT, q, lds, s);
}

// mode as in conv_impl (0 int32, 2 packed, 3 packed+pooled, 4 pixel sums).  tap_bits > 0: the filter is tap-packed
// and the input has tap_bits true channels in one word per pixel.  Returns 0 when this shape has no kernel here
// (nothing has been launched then), 2 when the int8 kernel ran, 4 when the FP4 kernel ran (full channel words of 64,
// 128 or 256 channels; results are identical).
int conv_mfma_try(void *out, const uint64_t *in, const uint64_t *filt, const int32_t *thresh, const ConvGeom &g,
                  int64_t D, int O, int tap_bits, int mode, bool allow_fp4, hipStream_t s)
{
    // int32 maps of a 64-channel layer with up to 64 output channels are bound by writing the maps; there the FP4
    // flavour measured no faster (52.9 against 49.6 us at 32x32, population 1024) and the +-1 bytes stay.
    if (mode == 0 && g.Cw == 1 && O <= 64) allow_fp4 = false;
    if (allow_fp4 && rw_try(out, in, filt, thresh, g, D, O, tap_bits, mode, 1, s)) return 4;
    return rw_try(out, in, filt, thresh, g, D, O, tap_bits, mode, 0, s) ? 2 : 0;
}

}  // namespace nb
