// Binary conv on the int8 matrix cores (measured alternative to the VALU popcount path).
//
// CDNA4 has no 1-bit MFMA, but v_mfma_i32_16x16x64_i8 does 16384 int8 MACs per wave in 16 cycles: 4x the
// bit-MAC rate of v_xor + v_bcnt.  Bits are expanded to +-1 bytes (bit 1 -> +1, bit 0 -> -1; an out-of-range
// pixel is the zero word, i.e. all -1), the int32 dot product over K = taps*CB positions is exact, and
//     popcount(x ^ w) = (K - dot) / 2
// gives back the reference's sum bit for bit.  One workgroup owns one member: its image is expanded once
// into LDS (with the zero-word border, so the implicit im2col needs no bounds checks), the member's filter
// fragments are expanded once, cooperatively, and then stay in VGPRs, and every wave streams 16-pixel A
// fragments out of LDS with one ds_read_b128 per fragment.
//
// Fragment layout of v_mfma_i32_16x16x64_i8 (checked on hardware): lane l supplies row l%16 of A and
// column l%16 of B, its 16 bytes are the K-positions 16*(l/16)..+15 of the 64-chunk (any bijection works as
// long as A and B use the same one), and acc[r] is D[4*(l/16) + r][l%16].
//
// All index arithmetic that needs a division (K position -> tap / channel, tile -> row / column) is done on
// the host and handed over in the kernel argument block, or advanced incrementally.
#include "nb_conv_common.hpp"

namespace nb {

typedef int v4i __attribute__((ext_vector_type(4)));

// 512 threads = two waves per SIMD: one wave's LDS reads and epilogue overlap the other's MFMAs.  The filter
// fragments of up to 36 (chunk, channel tile) pairs stay in registers (144 VGPRs); with more than 18 of them a
// wave works on two pixel tiles per step instead of four to stay inside 256 VGPRs.
constexpr int kMfmaThreads = 512;
constexpr int mfma_mt(int NK, int NT) { return NK * NT > 18 ? 2 : 4; }
constexpr int kLutBytes = 256 * 8;  // byte -> 8 bytes of +-1
constexpr int kMaxNK = 18;
constexpr int kTab = kMaxNK * 16;   // (chunk, lane group, dword) entries

struct MfmaConv {
    const uint64_t *in;
    const uint64_t *filt;
    const int32_t *thresh;
    void *out;
    int H, Wd, Cw, px, py, h, w, O;
    int CB;          // bytes (channel positions) per pixel, multiple of 4
    int PS;          // pixel stride in the LDS image, bytes
    int RW;          // pixels per LDS image row
    int RIN;         // LDS image rows = hs + fx - 1
    int K;           // taps * CB
    int ntx;         // 16-pixel tiles per output row
    int frows;       // filter rows per member (words per output channel)
    int img_bytes, bfr_bytes;
    int step_q, step_r;  // (waves*MT) / ntx and % ntx: tile advance of one step
    int pix_q, pix_r;    // threads / RW and % RW: image-pixel advance of one fill pass
    int taps, fy, tapT, in_bits;  // tapT > 1: tap-packed filter with in_bits channel bits per tap
    int S, hs;  // a member's output rows are split over S workgroups, hs rows each (even when pooling)
};

// Per K position 64*kc + 16*lg + 4*d (index (kc*4 + lg)*4 + d), computed once per workgroup into LDS:
struct MfmaTables {
    int koff[kTab];            // byte offset of that position relative to a tile's pixel in the LDS image
    short frow[kTab];          // filter row holding the 4 positions
    unsigned char fsh[kTab];   // bit position inside that filter word
    unsigned char flf[kTab];   // valid bits from there on (0: multiply by zero)
};
constexpr int kTabBytes = (sizeof(MfmaTables) + 15) / 16 * 16;

// 4 bits -> 4 bytes of +-1 (bit j -> byte j): 1 -> 0x01, 0 -> 0xFF
__device__ __forceinline__ uint32_t pm1_bytes(uint32_t nib)
{
    const uint32_t s1 = (nib << 7) | nib;
    const uint32_t s2 = (s1 << 14) | s1;
    const uint32_t u = ~s2 & 0x01010101u;        // 1 where the bit is 0
    return ((u << 8) - (u << 1)) | 0x01010101u;  // 0xFE where the bit is 0, then | 1
}

// MODE 0: int32 popcount sums [D,h,w,O]; 2: threshold bits packed along O; 3: the same, 2x2 OR-pooled.
template <int NK, int NT, int MODE, bool PB16, int MT>
__global__ __launch_bounds__(kMfmaThreads) void conv_mfma_kernel(const MfmaConv p)
{
    constexpr int kMfmaWaves = kMfmaThreads / 64;
    extern __shared__ __align__(16) unsigned char lds[];
    const uint2 *lut = reinterpret_cast<const uint2 *>(lds);
    MfmaTables &tab = *reinterpret_cast<MfmaTables *>(lds + kLutBytes);
    unsigned char *img = lds + kLutBytes + kTabBytes;
    unsigned char *bfr = img + p.img_bytes;
    // MODE 0: the per-wave int32 staging tiles reuse the fragment area once the fragments sit in registers;
    // MODE 2/3: packed words per pixel, behind the fragment area.
    unsigned char *obuf = MODE == 0 ? bfr : bfr + p.bfr_bytes;

    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int li = lane & 15, lg = lane >> 4;
    const int64_t z = blockIdx.x / (unsigned)p.S;  // member
    const int row0 = (int)(blockIdx.x - z * p.S) * p.hs;  // first output row of this workgroup
    const int hloc = p.h - row0 < p.hs ? p.h - row0 : p.hs;  // its output rows
    const int Ow = (p.O + 63) >> 6;

    if (tid < 256)  // expansion table: entry b holds the +-1 bytes of bits 0..7 of b
        reinterpret_cast<uint2 *>(lds)[tid] = make_uint2(pm1_bytes(tid & 0xFu), pm1_bytes((unsigned)tid >> 4));
    for (int ti = tid; ti < NK * 16; ti += kMfmaThreads) {  // K-position tables, one entry per thread
        const int k = 64 * (ti >> 4) + 16 * ((ti >> 2) & 3) + 4 * (ti & 3);
        int tap = k / p.CB;
        const int c = k - tap * p.CB;
        const bool valid = tap < p.taps;
        tap = valid ? tap : p.taps - 1;  // K padding: the filter side is zero, read any valid pixel
        const int i = tap / p.fy, j = tap - i * p.fy;
        tab.koff[ti] = (i * p.RW + j) * p.PS + c;
        int frow = 0, fsh = 0, flf = 0;
        if (valid && p.tapT > 1) {
            // tap t sits at bits in_bits*(t % T) of word t / T; c < in_bits for every position that is asked for
            // (CB = in_bits rounded up to 4, 8 or a multiple of 16)
            const int tq = tap / p.tapT;
            frow = tq;
            fsh = p.in_bits * (tap - tq * p.tapT) + (c < p.in_bits ? c : 0);
            flf = c < p.in_bits ? p.in_bits - c : 0;
        } else if (valid) {
            frow = tap * p.Cw + (c >> 6);
            fsh = c & 63;
            flf = 64;
        }
        tab.frow[ti] = (short)frow;
        tab.fsh[ti] = (unsigned char)fsh;
        tab.flf[ti] = (unsigned char)flf;
    }
    __syncthreads();

    // Filter words of one channel group: wave wv owns fragments wv, wv + waves, ...  The words of group 0 are
    // requested before the image is touched and those of group cg + 1 before the MFMA loop of group cg, so
    // their latency never sits on the critical path.
    constexpr int FPW = (NK * NT + kMfmaWaves - 1) / kMfmaWaves;  // fragments per wave
    constexpr int LD = PB16 ? 1 : 4;                               // filter words per fragment and lane
    uint64_t fw[FPW][LD];
    const uint64_t *fz = p.filt + z * (int64_t)p.frows * p.O;
    auto load_filter = [&](int n0g) {
#pragma unroll
        for (int q = 0; q < FPW; q++) {
            const int f = wv + kMfmaWaves * q;
            const int kc = f / NT, nt = f - kc * NT;  // NT is a compile-time constant
            const int ch = n0g + nt * 16 + li;
#pragma unroll
            for (int d = 0; d < LD; d++) {
                const int ti = f < NK * NT ? (kc * 4 + lg) * 4 + d : 0;
                const bool need = f < NK * NT && ch < p.O && tab.flf[ti] > 0;
                fw[q][d] = need ? fz[(int64_t)tab.frow[ti] * p.O + ch] : 0ull;
            }
        }
    };
    load_filter(0);

    // ---- phase 1: expand the member's image (with border) into LDS -----------------------------------------------
    // one pixel word per item, 8 items per thread loaded before any is expanded; (row, xx) advance incrementally
    {
        const uint64_t *src = p.in + z * (int64_t)p.H * p.Wd * p.Cw;
        const int npix = (hloc + p.RIN - p.hs) * p.RW;  // RIN = hs + fx - 1 rows at most
        const int row = tid / p.RW, xx = tid - row * p.RW;
        for (int cw = 0; cw < p.Cw; cw++) {
            const int nbits = p.CB - cw * 64 < 64 ? p.CB - cw * 64 : 64;  // positions held by this word
            int r0 = row, x0 = xx;
            constexpr int U = 8;
            for (int pix0 = tid; pix0 < npix; pix0 += kMfmaThreads * U) {
                uint64_t wd[U];
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const int yy = row0 + r0 - p.px, xs = x0 - p.py;
                    const bool inb = yy >= 0 && yy < p.H && xs >= 0 && xs < p.Wd;  // false past the last image row too
                    wd[u] = inb ? src[((int64_t)yy * p.Wd + xs) * p.Cw + cw] : 0ull;
                    r0 += p.pix_q;
                    x0 += p.pix_r;
                    if (x0 >= p.RW) {
                        x0 -= p.RW;
                        r0++;
                    }
                }
#pragma unroll
                for (int u = 0; u < U; u++) {
                    const int pix = pix0 + u * kMfmaThreads;
                    if (pix >= npix) continue;
                    unsigned char *dst = img + pix * p.PS + cw * 64;
                    if (nbits >= 16) {
                        for (int c = 0; c < nbits; c += 16) {
                            const uint2 lo = lut[(uint32_t)(wd[u] >> c) & 0xFFu];
                            const uint2 hi = lut[(uint32_t)(wd[u] >> (c + 8)) & 0xFFu];
                            *reinterpret_cast<uint4 *>(dst + c) = make_uint4(lo.x, lo.y, hi.x, hi.y);
                        }
                    } else if (nbits == 8) {
                        *reinterpret_cast<uint2 *>(dst) = lut[(uint32_t)wd[u] & 0xFFu];
                    } else {
                        *reinterpret_cast<uint32_t *>(dst) = lut[(uint32_t)wd[u] & 0xFu].x;
                    }
                }
            }
        }
    }

    // per-lane K offsets into the LDS image
    int koff[NK][PB16 ? 1 : 4];
#pragma unroll
    for (int kc = 0; kc < NK; kc++)
#pragma unroll
        for (int d = 0; d < (PB16 ? 1 : 4); d++) koff[kc][d] = tab.koff[(kc * 4 + lg) * 4 + d];

    const int mtiles = hloc * p.ntx;
    const int ngroups = (p.O + 16 * NT - 1) / (16 * NT);
    for (int cg = 0; cg < ngroups; cg++) {
        const int n0g = cg * 16 * NT;  // first channel of this group
        __syncthreads();               // image complete / previous group's use of the fragment area finished
        // ---- phase 2: expand the prefetched filter words of this channel group into fragments ------------------
#pragma unroll
        for (int q = 0; q < FPW; q++) {
            const int f = wv + kMfmaWaves * q;
            if (f >= NK * NT) continue;  // wave-uniform
            const int kc = f / NT, nt = f - kc * NT;
            const bool chv = n0g + nt * 16 + li < p.O;
            uint32_t e[4];
            if (PB16) {
                const int ti = (kc * 4 + lg) * 4;
                const int left = chv ? tab.flf[ti] : 0;  // valid bits from this position on (0: multiply by zero)
                uint32_t h16 = (uint32_t)(fw[q][0] >> tab.fsh[ti]) & 0xFFFFu;
                h16 = left >= 16 ? h16 : h16 & ((1u << left) - 1);
                const uint2 lo = lut[h16 & 0xFFu], hi = lut[h16 >> 8];
                e[0] = left > 0 ? lo.x : 0u;
                e[1] = left > 0 ? lo.y : 0u;
                e[2] = left > 0 ? hi.x : 0u;
                e[3] = left > 0 ? hi.y : 0u;
            } else {
#pragma unroll
                for (int d = 0; d < 4; d++) {
                    const int ti = (kc * 4 + lg) * 4 + d;
                    const int left = chv ? tab.flf[ti] : 0;
                    uint32_t nib = (uint32_t)(fw[q][d] >> tab.fsh[ti]) & 0xFu;
                    nib = left >= 4 ? nib : nib & ((1u << left) - 1);
                    e[d] = left > 0 ? lut[nib].x : 0u;
                }
            }
            *reinterpret_cast<uint4 *>(bfr + (f * 64 + lane) * 16) = make_uint4(e[0], e[1], e[2], e[3]);
        }
        __syncthreads();
        v4i B[NK][NT];
#pragma unroll
        for (int kc = 0; kc < NK; kc++)
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
                B[kc][nt] = *reinterpret_cast<const v4i *>(bfr + ((kc * NT + nt) * 64 + lane) * 16);
        if (MODE == 0) __syncthreads();  // the staging tiles below overwrite the fragment area

        // thresholds in dot-product terms: 2*popc > t  <=>  popc > (t>>1)  <=>  dot < K - 2*(t>>1)
        int tdot[NT];
        if (MODE != 0) {
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                const int ch = n0g + nt * 16 + li;
                int64_t td = ch < p.O ? (int64_t)p.K - 2 * (int64_t)(p.thresh[z * p.O + ch] >> 1) : -2147483648LL;
                td = td > 2147483647LL ? 2147483647LL : (td < -2147483648LL ? -2147483648LL : td);
                tdot[nt] = (int)td;
            }
        }

        if (cg + 1 < ngroups) load_filter(n0g + 16 * NT);

        // ---- phase 3: MT pixel tiles x NT channel tiles per wave and step ---------------------------------------
        // tile t = ty * ntx + txi; the wave's first tile of a step advances by kMfmaWaves*MT tiles
        int sty = (wv * MT) / p.ntx, stx = wv * MT - sty * p.ntx;
        for (int t0 = wv * MT; t0 < mtiles; t0 += kMfmaWaves * MT) {
            int tbase[MT], ty[MT], tx[MT];
            {
                int cy = sty, cx = stx;
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    const bool live = t0 + mt < mtiles;
                    ty[mt] = live ? cy : 0;  // dead tiles compute on tile 0 and are dropped below
                    tx[mt] = live ? cx * 16 : 0;
                    tbase[mt] = (ty[mt] * p.RW + tx[mt] + li) * p.PS;
                    if (++cx == p.ntx) {
                        cx = 0;
                        cy++;
                    }
                }
                sty += p.step_q;
                stx += p.step_r;
                if (stx >= p.ntx) {
                    stx -= p.ntx;
                    sty++;
                }
            }
            v4i acc[MT][NT];
#pragma unroll
            for (int mt = 0; mt < MT; mt++)
#pragma unroll
                for (int nt = 0; nt < NT; nt++) acc[mt][nt] = (v4i){0, 0, 0, 0};
#pragma unroll
            for (int kc = 0; kc < NK; kc++) {
                v4i A[MT];
#pragma unroll
                for (int mt = 0; mt < MT; mt++) {
                    if (PB16) {
                        A[mt] = *reinterpret_cast<const v4i *>(img + tbase[mt] + koff[kc][0]);
                    } else {
#pragma unroll
                        for (int d = 0; d < 4; d++)
                            A[mt][d] = *reinterpret_cast<const int *>(img + tbase[mt] + koff[kc][PB16 ? 0 : d]);
                    }
                }
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
                        acc[mt][nt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[mt], B[kc][nt], acc[mt][nt], 0, 0, 0);
            }
            // ---- epilogue of the step ----------------------------------------------------------------------
#pragma unroll
            for (int mt = 0; mt < MT; mt++) {
                if (t0 + mt >= mtiles) continue;  // wave-uniform
                if (MODE == 0) {
                    // stage the 16 x (16*NT) tile in LDS, then store whole pixel rows (non-temporal)
                    int *stage = reinterpret_cast<int *>(obuf) + wv * (16 * 16 * NT);
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            stage[(4 * lg + r) * (16 * NT) + nt * 16 + li] = (p.K - acc[mt][nt][r]) >> 1;
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    int32_t *o32 = static_cast<int32_t *>(p.out);
                    constexpr int LPP = 4 * NT;    // lanes per pixel, one int4 each
                    constexpr int PPI = 64 / LPP;  // pixels per store instruction
                    int32_t *orow = o32 + ((z * p.h + row0 + ty[mt]) * (int64_t)p.w + tx[mt]) * p.O + n0g;
#pragma unroll
                    for (int s = 0; s < 16 / PPI; s++) {
                        const int pi = s * PPI + lane / LPP, c4 = (lane % LPP) * 4;
                        if (tx[mt] + pi < p.w && n0g + c4 < p.O) {
                            const nb_i32x4 v = *reinterpret_cast<const nb_i32x4 *>(stage + pi * (16 * NT) + c4);
                            __builtin_nontemporal_store(v, reinterpret_cast<nb_i32x4 *>(orow + (int64_t)pi * p.O + c4));
                        }
                    }
                    __builtin_amdgcn_wave_barrier();
                } else {
                    // ballot r of lane (pixel 4*lg+r, channel li): bits 16*g.. are the 16-channel piece of pixel
                    // 4*g+r.  Lane j < 16 extracts the piece of pixel j and writes it.
                    uint16_t *ob16 = reinterpret_cast<uint16_t *>(obuf);
#pragma unroll
                    for (int nt = 0; nt < NT; nt++) {
                        uint64_t m[4];
#pragma unroll
                        for (int r = 0; r < 4; r++) m[r] = __ballot(acc[mt][nt][r] < tdot[nt]);
                        const int r = lane & 3;
                        const uint64_t mine = r == 0 ? m[0] : r == 1 ? m[1] : r == 2 ? m[2] : m[3];
                        const uint32_t piece16 = (uint32_t)(mine >> (16 * ((lane >> 2) & 3))) & 0xFFFFu;
                        const int x = tx[mt] + lane;  // lanes 0..15 <-> the tile's 16 pixels
                        if (lane < 16 && x < p.w)
                            ob16[((ty[mt] * p.w + x) * Ow) * 4 + (n0g >> 4) + nt] = (uint16_t)piece16;
                    }
                }
            }
        }
    }

    // ---- phase 4 (packed modes): write the member's packed map, optionally 2x2 OR-pooled ----------------------
    if (MODE != 0) {
        __syncthreads();
        const uint64_t *ob = reinterpret_cast<const uint64_t *>(obuf);
        uint64_t *o64 = static_cast<uint64_t *>(p.out);
        // 16-bit pieces of channels past O in the last word were never written: mask them off
        const int lastv = p.O - 64 * (Ow - 1);
        const uint64_t lastmask = lastv >= 64 ? ~0ull : ((1ull << lastv) - 1);
        if (MODE == 2) {
            const int total = hloc * p.w * Ow;
            uint64_t *dst = o64 + (z * p.h + row0) * (int64_t)p.w * Ow;
            int wi = tid % Ow;
            const int dwi = kMfmaThreads % Ow;
            for (int i = tid; i < total; i += kMfmaThreads) {
                dst[i] = ob[i] & (wi == Ow - 1 ? lastmask : ~0ull);
                wi += dwi;
                wi = wi >= Ow ? wi - Ow : wi;
            }
        } else {
            const int h2 = hloc >> 1, w2 = p.w >> 1;  // row0 is even: hs is
            const int total = h2 * w2 * Ow;
            uint64_t *dst = o64 + (z * (p.h >> 1) + (row0 >> 1)) * (int64_t)w2 * Ow;
            for (int i = tid; i < total; i += kMfmaThreads) {
                const int q = i / Ow, wi = i - q * Ow;
                const int qy = q / w2, qx = q - qy * w2;
                const int b0 = ((2 * qy) * p.w + 2 * qx) * Ow + wi;
                const uint64_t v = ob[b0] | ob[b0 + Ow] | ob[b0 + p.w * Ow] | ob[b0 + p.w * Ow + Ow];
                dst[i] = v & (wi == Ow - 1 ? lastmask : ~0ull);
            }
        }
    }
}

static inline int round_up(int a, int b) { return (a + b - 1) / b * b; }

// Returns false when the launch could not be set up (the caller then uses the XOR-popcount path).
template <int NK, int NT, int MODE, bool PB16>
static bool launch_one(const MfmaConv &p, int64_t D, size_t lds_bytes, hipStream_t s)
{
    static bool attr_set = false;  // benign race: setting the same attribute twice is harmless
    auto *kfn = conv_mfma_kernel<NK, NT, MODE, PB16, mfma_mt(NK, NT)>;
    if (!attr_set) {
        if (hipFuncSetAttribute(reinterpret_cast<const void *>(kfn), hipFuncAttributeMaxDynamicSharedMemorySize,
                                160 * 1024) != hipSuccess) {
            (void)hipGetLastError();
            return false;
        }
        attr_set = true;
    }
    kfn<<<dim3((unsigned)(D * p.S)), dim3(kMfmaThreads), lds_bytes, s>>>(p);
    return true;
}

template <int MODE>
static bool launch_mode(const MfmaConv &p, int64_t D, int NK, int NT, bool pb16, size_t lds, hipStream_t s)
{
#define NB_MFMA(nk, nt)                                                           \
    if (NK == nk && NT == nt)                                                     \
        return pb16 ? launch_one<nk, nt, MODE, true>(p, D, lds, s) : launch_one<nk, nt, MODE, false>(p, D, lds, s)
#define NB_MFMA16(nk, nt) \
    if (NK == nk && NT == nt && pb16) return launch_one<nk, nt, MODE, true>(p, D, lds, s)
    NB_MFMA(1, 4);
    NB_MFMA(1, 1);
    NB_MFMA(3, 1);
    NB_MFMA(3, 4);
    NB_MFMA16(9, 4);  // pixels narrower than 16 positions never reach 9 chunks with the usual filter sizes
    NB_MFMA16(9, 1);
    NB_MFMA16(18, 2);
#undef NB_MFMA16
#undef NB_MFMA
    return false;
}

// mode as in conv_impl (0 int32, 2 packed, 3 packed+pooled).  in_bits = true channel count if known, else 0.
// Returns false when this shape has no matrix-core kernel or, unless force is set, when the XOR-popcount
// kernels measured faster on shapes of its kind; nothing has been launched then.
bool conv_mfma_try(void *out, const uint64_t *in, const uint64_t *filt, const int32_t *thresh, const ConvGeom &g,
                   int64_t D, int O, int in_bits, bool filter_tap_packed, int mode, bool force, hipStream_t s)
{
    if (!aligned(out, 16)) return false;
    if (mode != 0 && mode != 2 && mode != 3) return false;
    if (g.sx != 1 || g.sy != 1 || g.h < 1 || g.w < 1 || D < 1 || D > kMaxBlocks) return false;
    if (O < 1 || (O & 15) != 0) return false;
    if (mode == 3 && (g.h < 2 || g.w < 2)) return false;
    if (filter_tap_packed && (in_bits < 1 || g.Cw != 1)) return false;
    MfmaConv p;
    p.in = in;
    p.filt = filt;
    p.thresh = thresh;
    p.out = out;
    p.H = g.H; p.Wd = g.Wd; p.Cw = g.Cw; p.px = g.px; p.py = g.py; p.h = g.h; p.w = g.w;
    p.O = O;
    const int taps = g.fx * g.fy;
    const int tapT = filter_tap_packed ? 64 / in_bits : 1;
    int CB = g.Cw * 64;
    if (in_bits > 0 && g.Cw == 1) CB = round_up(in_bits, 4);
    if (CB != 4 && CB != 8 && (CB & 15) != 0) CB = round_up(CB, 16);
    if (CB > g.Cw * 64) return false;
    p.CB = CB;
    const bool pb16 = (CB & 15) == 0;
    p.PS = CB > 32 ? CB + 16 : CB;
    p.ntx = (g.w + 15) / 16;
    p.RW = round_up(16 * p.ntx + g.fy - 1, 4);
    p.K = taps * CB;
    p.frows = filter_tap_packed ? (taps + tapT - 1) / tapT : taps * g.Cw;
    if (p.frows > 32767) return false;
    const int NK = (p.K + 63) / 64;
    if (NK > kMaxNK) return false;
    int NT = O >= 64 ? 4 : (O == 16 ? 1 : 0);
    if (NK == 18) NT = O >= 32 ? 2 : 0;
    if (NT == 0) return false;
    // Measured on MI355X (64-bit words, 3x3 filters, 1024-4096 members): the per-member set-up (image and filter
    // expansion) is paid back from 32x32 output pixels on, or from 16x16 when K = taps*channels reaches 1152;
    // below that the XOR-popcount kernels win.
    const int64_t pixels = (int64_t)g.h * g.w;
    if (!force && !(pixels >= 1024 || (NK >= 18 && pixels >= 256))) return false;
    const int threads = kMfmaThreads, waves = threads / 64, MT = mfma_mt(NK, NT);
    p.step_q = (waves * MT) / p.ntx;
    p.step_r = (waves * MT) % p.ntx;
    p.pix_q = threads / p.RW;
    p.pix_r = threads % p.RW;
    p.taps = taps;
    p.fy = g.fy;
    p.tapT = tapT;
    p.in_bits = in_bits;
    p.bfr_bytes = NK * NT * 1024;
    const int Ow = (O + 63) / 64;
    const int stage = waves * 16 * 16 * NT * 4;
    if (mode == 0 && p.bfr_bytes < stage) p.bfr_bytes = stage;
    // Kernels with few filter fragments need few registers, so several workgroups fit a CU and one's set-up
    // overlaps another's MFMAs -- if their LDS footprints allow it: split a member's rows until a workgroup
    // needs at most 48 KB (each part re-expands fx - 1 halo rows and rebuilds the small fragment set).
    const int max_split = NK * NT <= 4 ? 8 : 1;
    size_t lds = 0;
    for (p.S = 1;; p.S++) {
        p.hs = round_up((g.h + p.S - 1) / p.S, 2);
        p.RIN = p.hs + g.fx - 1;
        p.img_bytes = round_up(p.RIN * p.RW * p.PS + 64, 16);
        const int obuf = mode == 0 ? 0 : round_up(p.hs * g.w * Ow * 8, 16);
        lds = (size_t)kLutBytes + kTabBytes + p.img_bytes + p.bfr_bytes + obuf;
        if (lds <= 48 * 1024 || p.S >= max_split || p.hs <= 8) break;
    }
    p.S = (g.h + p.hs - 1) / p.hs;  // parts that own at least one row
    if (lds > 158 * 1024 || D * p.S > kMaxBlocks) return false;
    if (mode == 0) return launch_mode<0>(p, D, NK, NT, pb16, lds, s);
    if (mode == 2) return launch_mode<2>(p, D, NK, NT, pb16, lds, s);
    return launch_mode<3>(p, D, NK, NT, pb16, lds, s);
}

}  // namespace nb
