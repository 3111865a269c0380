/*
 * TEST INFRASTRUCTURE ONLY.  CPU oracle for the packed binary forward path of
 * jamesal1/NESgpu: a plain-C restatement of the reference kernels' arithmetic.
 * Only tests, the smoke check and the benchmark's cpu_baseline leg load this
 * library; the product (libnesbin.so) never links or calls it.
 *
 * What pins each function (checked by the CPU test-suite):
 *   pack / unpack        numpy.packbits(bitorder="little") closed form + round trip
 *   int8pack             numpy little-endian byte view of a zero-padded row
 *   im2col               independent numpy gather over unpacked, explicitly padded bits
 *   bmm / bmm_act        integer matmul on +-1 values: 2*popc - K == a.(-b)
 *                        (booloptests.py:150-160) and brute force on bits
 *   conv / conv_act      grouped torch.conv2d on +-1 with pad value -1 and
 *                        sign-inverted filters (booloptests.py:150-155,157-160)
 *   max_pool2d           pack(F.max_pool2d(bits)) for 2x2/s2 (booloptests.py:94-95,138-141)
 *                        and an OR-of-window brute force for padded cases
 *   sample_from_words    numpy (words < thresh) + packbits; rate check mean ~= p
 *   seeded_bmv           must equal bmm(sample_from_words(...), x)
 *   philox4x32_10        Random123 known-answer vectors and rocRAND's host engine
 *   weighted_sum         float64 numpy einsum over unpacked bits (tolerance)
 *   skip_flips           numpy searchsorted + cumsum over the (pinned) Philox words; flip rate,
 *                        gap histogram against the geometric law, neighbouring columns uncorrelated
 *   skip_flips_thin      the same numpy walk with the pair's second word deciding each column
 *                        (Python integers); per-column flip rates against their own probabilities,
 *                        neighbouring columns uncorrelated, reduction to skip_flips' law when all
 *                        probabilities equal the largest one
 *   skip_flips_layered   rows whose columns all share a class: equal to skip_flips_thin on the same words with the
 *                        class's table and tmax = 2^(31-k) (every class); mixed rows: an independent numpy walk
 *                        per class over the (pinned) Philox words; per-column flip rates against their own
 *                        probabilities over a law spanning many classes, neighbouring columns uncorrelated
 *   draws16              an independent numpy evaluation from the (pinned) Philox words of the two streams,
 *                        with thresholds that force ties; rates of columns whose thresholds have non-zero
 *                        low halves; neighbouring columns (the two halves of one word) uncorrelated
 * The cuRAND XORWOW stream of the reference samplers (sample_bits.cu:23-25,54) is NOT
 * reproduced anywhere: parity unpinned for that stream; supplied-word parity replaces it.
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp, see Makefile)
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)

#define WORD uint64_t
#define WBITS 64
#define POPC(x) __builtin_popcountll(x)
#define FN(x) CAT(x, _i64)
#include "nesbin_oracle_impl.h"
#undef WORD
#undef WBITS
#undef POPC
#undef FN

#define WORD uint32_t
#define WBITS 32
#define POPC(x) __builtin_popcount(x)
#define FN(x) CAT(x, _i32)
#include "nesbin_oracle_impl.h"
#undef WORD
#undef WBITS
#undef POPC
#undef FN

/* booleanOperations.py:162-166 -- conv = bmm(im2col(input), filter); filter is
 * [D, fx*fy*Cw, O] (modules/binary.py:136-137).  Done one member at a time so the
 * column buffer stays small.  out is [D, h, w, O] int32. */
#define DEFINE_CONV(SUF, WORD_T)                                                                   \
    void nbo_conv_##SUF(int32_t *out, const WORD_T *in, const WORD_T *filt, int64_t D, int64_t H,  \
                        int64_t W, int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx,  \
                        int sy)                                                                    \
    {                                                                                              \
        const int64_t h = (H - fx + 2 * px) / sx + 1, w = (W - fy + 2 * py) / sy + 1;              \
        const int64_t K = (int64_t)fx * fy * Cw;                                                   \
        _Pragma("omp parallel")                                                                    \
        {                                                                                          \
            WORD_T *cols = (WORD_T *)malloc(sizeof(WORD_T) * (size_t)(h * w * K + 1));             \
            _Pragma("omp for schedule(static)")                                                    \
            for (int64_t d = 0; d < D; d++) {                                                      \
                nbo_im2col_##SUF(cols, in + d * H * W * Cw, 1, H, W, Cw, fx, fy, px, py, sx, sy);  \
                nbo_bmm_##SUF(out + d * h * w * O, cols, filt + d * K * O, 1, h * w, K, O);        \
            }                                                                                      \
            free(cols);                                                                            \
        }                                                                                          \
    }                                                                                              \
    /* booleanOperations.py:168-172 -- conv_act = bmm_act(im2col(input), filter, thresh). */       \
    void nbo_conv_act_##SUF(uint8_t *out, const WORD_T *in, const WORD_T *filt,                    \
                            const int32_t *thresh, int64_t D, int64_t H, int64_t W, int64_t Cw,    \
                            int64_t O, int fx, int fy, int px, int py, int sx, int sy)             \
    {                                                                                              \
        const int64_t h = (H - fx + 2 * px) / sx + 1, w = (W - fy + 2 * py) / sy + 1;              \
        const int64_t K = (int64_t)fx * fy * Cw;                                                   \
        _Pragma("omp parallel")                                                                    \
        {                                                                                          \
            WORD_T *cols = (WORD_T *)malloc(sizeof(WORD_T) * (size_t)(h * w * K + 1));             \
            _Pragma("omp for schedule(static)")                                                    \
            for (int64_t d = 0; d < D; d++) {                                                      \
                nbo_im2col_##SUF(cols, in + d * H * W * Cw, 1, H, W, Cw, fx, fy, px, py, sx, sy);  \
                nbo_bmm_act_##SUF(out + d * h * w * O, cols, filt + d * K * O, thresh + d * O, 1,  \
                                  h * w, K, O);                                                    \
            }                                                                                      \
            free(cols);                                                                            \
        }                                                                                          \
    }

DEFINE_CONV(i64, uint64_t)
DEFINE_CONV(i32, uint32_t)

/* Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy as 1, 2, 3",
 * SC'11).  Not part of the reference (it draws from cuRAND XORWOW, sample_bits.cu:23-25);
 * this is the generator the replacement uses when the random words are not supplied.
 * ctr[4], key[2] -> out[4]. */
void nbo_philox4x32_10(uint32_t out[4], const uint32_t ctr[4], const uint32_t key[2])
{
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; r++) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* The word stream the replacement's generator mode defines: word number g (a flat index into
 * the [n, R, C] draw tensor, plus first) is lane g%4 of the Philox block with counter
 * (lo32(g/4), hi32(g/4), lo32(subseq), hi32(subseq)) and key (lo32(seed), hi32(seed)). */
void nbo_philox_words(uint32_t *out, uint64_t seed, uint64_t subseq, uint64_t first, int64_t count)
{
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < count; i++) {
        const uint64_t g = first + (uint64_t)i;
        const uint64_t blk = g >> 2;
        const uint32_t ctr[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)subseq,
                                 (uint32_t)(subseq >> 32)};
        uint32_t o[4];
        nbo_philox4x32_10(o, ctr, key);
        out[i] = o[g & 3];
    }
}

/* Bernoulli draws from 16-bit half-words: the contract of nb_sample_philox16_* (no counterpart in the reference,
 * whose sampler compares a 32-bit uniform per bit, extensions/src/sample_bits.cu:47-57).  Column g = first + row*C + c
 * (rows flat over members and rows) takes half-word g % 2 (low half first) of element g / 2 of the stream
 * (seed, subseq): h; with T the column's threshold (thresh[(row % R)*C + c] or thr_scalar) the bit is set iff
 * h < T >> 16, or h == T >> 16 and l < (T & 0xFFFF), l = the low 16 bits of element g of the stream
 * (seed, subseq ^ 2^63).  P(bit) = T / 2^32 exactly.  bit: [rows, C] bytes. */
void nbo_draws16(uint8_t *bit, const uint32_t *thresh, uint32_t thr_scalar, uint64_t seed, uint64_t subseq,
                 uint64_t first, int64_t rows, int64_t R, int64_t C)
{
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    const uint64_t sub2 = subseq ^ 0x8000000000000000ull;
#pragma omp parallel for schedule(static)
    for (int64_t row = 0; row < rows; row++) {
        for (int64_t c = 0; c < C; c++) {
            const uint64_t g = first + (uint64_t)row * (uint64_t)C + (uint64_t)c;
            const uint64_t e = g >> 1, blk = e >> 2;
            const uint32_t ctr[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)subseq, (uint32_t)(subseq >> 32)};
            uint32_t o[4];
            nbo_philox4x32_10(o, ctr, key);
            const uint32_t w = o[e & 3];
            const uint32_t h = (g & 1) ? w >> 16 : w & 0xFFFFu;
            const uint32_t t = thresh ? thresh[(row % R) * C + c] : thr_scalar;
            uint8_t b = h < (t >> 16);
            if (h == (t >> 16)) {
                const uint64_t blk2 = g >> 2;
                const uint32_t ctr2[4] = {(uint32_t)blk2, (uint32_t)(blk2 >> 32), (uint32_t)sub2, (uint32_t)(sub2 >> 32)};
                nbo_philox4x32_10(o, ctr2, key);
                b = (o[g & 3] & 0xFFFFu) < (t & 0xFFFFu);
            }
            bit[row * C + c] = b;
        }
    }
}

/* Flip masks by gap sampling: the contract of the library's skip sampler (nb_flip_skip_*; no counterpart in the
 * reference, whose sampler draws every bit, extensions/src/sample_bits.cu:47-57).  Row q (flat over members and rows)
 * reads the Philox words first + q*C + i, i = 0, 1, ...; word i has rank #{k < Kt : cdf[k] <= word}: a rank below Kt
 * moves the position on by rank + 1 columns and flips the column reached; rank Kt (the word lies beyond the table)
 * moves it on by Kt columns without a flip (the geometric law has no memory, so the walk just continues); the row
 * ends when the position passes C.  With cdf[k-1] = floor(2^32 * (1 - (1-p)^k)) the gaps are geometric and the
 * columns i.i.d. Bernoulli(p), quantised to 2^-32.  An empty table (Kt == 0) stands for p = 0: no flips.  mask is
 * [rows, ceil(C/64)] 64-bit words, LSB first. */
void nbo_skip_flips_i64(uint64_t *mask, const uint32_t *cdf, int64_t Kt, uint64_t seed, uint64_t subseq, uint64_t first,
                        int64_t rows, int64_t C)
{
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    const int64_t Kw = (C + 63) / 64;
#pragma omp parallel for schedule(static)
    for (int64_t q = 0; q < rows; q++) {
        uint64_t *row = mask + q * Kw;
        memset(row, 0, (size_t)Kw * 8);
        if (Kt == 0) continue;
        int64_t pos = -1;
        for (int64_t i = 0;; i++) {
            const uint64_t g = first + (uint64_t)q * (uint64_t)C + (uint64_t)i;
            const uint64_t blk = g >> 2;
            const uint32_t ctr[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)subseq, (uint32_t)(subseq >> 32)};
            uint32_t o[4];
            nbo_philox4x32_10(o, ctr, key);
            const uint32_t u = o[g & 3];
            int64_t lo = 0, hi = Kt; /* first index whose entry exceeds u */
            while (lo < hi) {
                const int64_t mid = (lo + hi) / 2;
                if (cdf[mid] <= u) lo = mid + 1;
                else hi = mid;
            }
            pos += lo < Kt ? 1 + lo : Kt;
            if (pos >= C) break;
            if (lo < Kt) row[pos >> 6] |= (uint64_t)1 << (pos & 63);
        }
    }
}

/* fp16 bit pattern (sign ignored by the caller) -> float, exactly */
static float nbo_half_bits_to_float(uint16_t h)
{
    const uint32_t e = (h >> 10) & 31u, m = h & 1023u;
    if (e == 0) return (float)m * 5.9604644775390625e-08f;              /* m * 2^-24 */
    if (e == 31) return m ? __builtin_nanf("") : __builtin_inff();
    float v = (float)(1024u + m) * 0.0009765625f;                       /* 1.m */
    int sh = (int)e - 15;
    while (sh > 0) { v *= 2.0f; sh--; }
    while (sh < 0) { v *= 0.5f; sh++; }
    return v;
}

/* Flip masks under a per-element law, by thinning: the contract of nb_flip_skip_thin_i64 (no counterpart in the
 * reference, whose sampler compares every bit's probability with its own draw, extensions/src/sample_bits.cu:47-57).
 * law [R, C]: bit 15 = base bit of the column (not used here), bits 14:0 = fp16 pattern of its flip probability
 * y <= 1/2, Tf = floor(y * 2^32).  Row q = d*R + r reads the Philox words first + q*C + 2i (a gap, ranked in cdf as
 * in nbo_skip_flips_i64; cdf belongs to the largest Tf of the layer, tmax) and first + q*C + 2i + 1: the column the
 * gap reaches flips iff that second word times tmax is below Tf * 2^32, i.e. with probability Tf / tmax.  mask is
 * [D*R, ceil(C/64)] 64-bit words, LSB first. */
void nbo_skip_flips_thin_i64(uint64_t *mask, const uint16_t *law, const uint32_t *cdf, int64_t Kt, uint32_t tmax,
                             uint64_t seed, uint64_t subseq, uint64_t first, int64_t D, int64_t R, int64_t C)
{
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    const int64_t Kw = (C + 63) / 64;
#pragma omp parallel for schedule(static)
    for (int64_t q = 0; q < D * R; q++) {
        uint64_t *row = mask + q * Kw;
        const uint16_t *lr = law + (q % R) * C;
        memset(row, 0, (size_t)Kw * 8);
        if (Kt == 0) continue;
        int64_t pos = -1;
        for (int64_t i = 0;; i++) {
            uint32_t pair[2];
            for (int h = 0; h < 2; h++) {
                const uint64_t g = first + (uint64_t)q * (uint64_t)C + (uint64_t)(2 * i + h);
                const uint64_t blk = g >> 2;
                const uint32_t ctr[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)subseq, (uint32_t)(subseq >> 32)};
                uint32_t o[4];
                nbo_philox4x32_10(o, ctr, key);
                pair[h] = o[g & 3];
            }
            int64_t lo = 0, hi = Kt; /* first index whose entry exceeds the gap word */
            while (lo < hi) {
                const int64_t mid = (lo + hi) / 2;
                if (cdf[mid] <= pair[0]) lo = mid + 1;
                else hi = mid;
            }
            pos += lo < Kt ? 1 + lo : Kt;
            if (pos >= C) break;
            if (lo >= Kt) continue;
            float t = nbo_half_bits_to_float((uint16_t)(lr[pos] & 0x7FFFu)) * 4294967296.0f;
            if (!(t <= 4294967040.0f)) t = 4294967040.0f;
            const uint64_t tf = (uint64_t)(uint32_t)t;
            if ((uint64_t)pair[1] * (uint64_t)tmax < (tf << 32)) row[pos >> 6] |= (uint64_t)1 << (pos & 63);
        }
    }
}

/* Flip masks under a per-element law, class by class: the contract of nb_flip_skip_layered_i64 (no counterpart in the
 * reference, as above).  The columns of row r that can flip are listed in pl[r, :] = column | law << 16, sorted by the
 * class of their flip threshold Tf (class k: 2^(30-k) < Tf <= 2^(31-k), k < 15; class 15: 0 < Tf <= 2^16), in
 * increasing column order inside a class; cls[r, k] .. cls[r, k+1] is class k's stretch of the list.  Row q = d*R + r
 * reads the Philox words first + q*C + 2i (a gap) and + 2i + 1 (accept), i = 0, 1, ..., without a break from class to
 * class: in class k the gap is ranked in cdfs[k] (kts[k] entries of the gap table of threshold 2^(31-k)) and moves the
 * position in the class's stretch (start: -1) as in nbo_skip_flips_i64; the column reached flips iff
 * accept < Tf * 2^(k+1); a position past the stretch ends the class, and the next class that has columns starts with
 * the next pair.  cdfs is [16, tabw] uint32.  mask is [D*R, ceil(C/64)] 64-bit words, LSB first. */
void nbo_skip_flips_layered_i64(uint64_t *mask, const uint32_t *pl, const uint32_t *cls, const uint32_t *cdfs,
                                const int32_t *kts, int64_t tabw, uint64_t seed, uint64_t subseq, uint64_t first,
                                int64_t D, int64_t R, int64_t C)
{
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    const int64_t Kw = (C + 63) / 64;
#pragma omp parallel for schedule(static)
    for (int64_t q = 0; q < D * R; q++) {
        uint64_t *row = mask + q * Kw;
        const uint32_t *list = pl + (q % R) * C;
        const uint32_t *starts = cls + (q % R) * 17;
        memset(row, 0, (size_t)Kw * 8);
        uint64_t g = first + (uint64_t)q * (uint64_t)C; /* the next word of the row */
        for (int k = 0; k < 16; k++) {
            const int64_t nk = (int64_t)starts[k + 1] - (int64_t)starts[k];
            const uint32_t *cdf = cdfs + (int64_t)k * tabw;
            const int64_t Kt = kts[k];
            if (nk <= 0) continue;
            int64_t pos = -1;
            for (;;) {
                uint32_t pair[2];
                for (int h = 0; h < 2; h++, g++) {
                    const uint64_t blk = g >> 2;
                    const uint32_t ctr[4] = {(uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)subseq, (uint32_t)(subseq >> 32)};
                    uint32_t o[4];
                    nbo_philox4x32_10(o, ctr, key);
                    pair[h] = o[g & 3];
                }
                int64_t lo = 0, hi = Kt;
                while (lo < hi) {
                    const int64_t mid = (lo + hi) / 2;
                    if (cdf[mid] <= pair[0]) lo = mid + 1;
                    else hi = mid;
                }
                pos += lo < Kt ? 1 + lo : Kt;
                if (pos >= nk) break;
                if (lo >= Kt) continue;
                const uint32_t e = list[starts[k] + pos];
                float t = nbo_half_bits_to_float((uint16_t)((e >> 16) & 0x7FFFu)) * 4294967296.0f;
                if (!(t <= 4294967040.0f)) t = 4294967040.0f;
                const uint64_t tf = (uint64_t)(uint32_t)t;
                const uint32_t col = e & 0xFFFFu;
                if ((uint64_t)pair[1] < (tf << (k + 1))) row[col >> 6] |= (uint64_t)1 << (col & 63);
            }
        }
    }
}

#ifdef _OPENMP
#include <omp.h>
int nbo_max_threads(void) { return omp_get_max_threads(); }
void nbo_set_threads(int n) { omp_set_num_threads(n); }
#else
int nbo_max_threads(void) { return 1; }
void nbo_set_threads(int n) { (void)n; }
#endif
