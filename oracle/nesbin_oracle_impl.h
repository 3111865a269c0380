/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's packed binary
 * forward ops, instantiated once per word width by nesbin_oracle.c.
 *
 * Included with these macros defined:
 *   WORD   unsigned word type (uint64_t / uint32_t)
 *   WBITS  bits per word (64 / 32)
 *   POPC   popcount builtin for WORD
 *   FN(x)  name mangler (appends _i64 / _i32)
 *
 * Every function walks the index space exactly the way the reference kernel it
 * cites does (one scalar loop nest, no tiling), so that a reader can compare it
 * line by line with the cited file.  OpenMP splits only the outermost
 * (population / row) axis, which the reference treats as independent as well.
 */

/* extensions/src/pack.cu:22-28 -- bit i of word y of row x is input[x][y*bits+i],
 * LSB first; columns past input1 read as 0 (pack.cu:17). */
void FN(nbo_pack)(WORD *ret, const uint8_t *input, int64_t R, int64_t C)
{
    const int64_t Rw = (C + WBITS - 1) / WBITS;
#pragma omp parallel for schedule(static)
    for (int64_t x = 0; x < R; x++) {
        for (int64_t y = 0; y < Rw; y++) {
            WORD tmp = 0;
            for (int i = 0; i < WBITS; i++) {
                const int64_t col = y * WBITS + i;
                const WORD b = (col < C && input[x * C + col]) ? 1 : 0;
                tmp |= b << i;
            }
            ret[x * Rw + y] = tmp;
        }
    }
}

/* extensions/booleanUtilitiesCuda.cu:77-90 -- ret[x][y*bits+i] = bit i of input[x][y];
 * output has Rw*bits columns (booleanUtilitiesCuda.cu:186). */
void FN(nbo_unpack)(uint8_t *ret, const WORD *input, int64_t R, int64_t Rw)
{
#pragma omp parallel for schedule(static)
    for (int64_t x = 0; x < R; x++)
        for (int64_t y = 0; y < Rw; y++)
            for (int i = 0; i < WBITS; i++)
                ret[(x * Rw + y) * WBITS + i] = (uint8_t)((input[x * Rw + y] >> i) & 1);
}

/* extensions/src/int8pack.cu:22-28 -- byte i of word y is input[x][y*(bits/8)+i],
 * little endian, bytes past input1 read as 0 (int8pack.cu:17). */
void FN(nbo_int8pack)(WORD *ret, const uint8_t *input, int64_t R, int64_t C)
{
    const int64_t per = WBITS / 8;
    const int64_t Rw = (C + per - 1) / per;
#pragma omp parallel for schedule(static)
    for (int64_t x = 0; x < R; x++) {
        for (int64_t y = 0; y < Rw; y++) {
            WORD tmp = 0;
            for (int i = 0; i < per; i++) {
                const int64_t col = y * per + i;
                const WORD b = col < C ? input[x * C + col] : 0;
                tmp |= b << (8 * i);
            }
            ret[x * Rw + y] = tmp;
        }
    }
}

/* extensions/src/batch_im2col.cu:14-29 and booleanOperations.py:83-87.
 * input [B,H,W,Cw] -> output [B, h*w, fx*fy*Cw]; element e=(i*fy+j)*Cw+c reads
 * input[b][i + xo*sx - px][j + yo*sy - py][c], out of bounds -> the zero word. */
void FN(nbo_im2col)(WORD *out, const WORD *in, int64_t B, int64_t H, int64_t W, int64_t Cw,
                    int fx, int fy, int px, int py, int sx, int sy)
{
    const int64_t h = (H - fx + 2 * px) / sx + 1;
    const int64_t w = (W - fy + 2 * py) / sy + 1;
    const int64_t K = (int64_t)fx * fy * Cw;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; b++) {
        for (int64_t loc = 0; loc < h * w; loc++) {
            const int64_t xo = loc / w, yo = loc - xo * w;
            for (int64_t e = 0; e < K; e++) {
                const int64_t eidx = e / Cw, c = e - eidx * Cw;
                const int64_t i = eidx / fy, j = eidx - i * fy;
                const int64_t xi = i + xo * sx - px, yi = j + yo * sy - py;
                const int inb = xi >= 0 && xi < H && yi >= 0 && yi < W;
                out[(b * h * w + loc) * K + e] = inb ? in[((b * H + xi) * W + yi) * Cw + c] : 0;
            }
        }
    }
}

/* extensions/src/bmm.cu:40,52 -- C[z][x][y] = sum_k popc(A[z][x][k] ^ B[z][k][y]). */
void FN(nbo_bmm)(int32_t *Cc, const WORD *A, const WORD *Bm, int64_t Z, int64_t M, int64_t K, int64_t N)
{
#pragma omp parallel for schedule(static)
    for (int64_t z = 0; z < Z; z++)
        for (int64_t x = 0; x < M; x++)
            for (int64_t y = 0; y < N; y++) {
                int32_t acc = 0;
                for (int64_t k = 0; k < K; k++)
                    acc += POPC(A[(z * M + x) * K + k] ^ Bm[(z * K + k) * N + y]);
                Cc[(z * M + x) * N + y] = acc;
            }
}

/* extensions/src/bmm_act.cu:56 -- C = (2*popc > thresh[z][y]) as a bool byte. */
void FN(nbo_bmm_act)(uint8_t *Cc, const WORD *A, const WORD *Bm, const int32_t *thresh,
                     int64_t Z, int64_t M, int64_t K, int64_t N)
{
#pragma omp parallel for schedule(static)
    for (int64_t z = 0; z < Z; z++)
        for (int64_t x = 0; x < M; x++)
            for (int64_t y = 0; y < N; y++) {
                int32_t acc = 0;
                for (int64_t k = 0; k < K; k++)
                    acc += POPC(A[(z * M + x) * K + k] ^ Bm[(z * K + k) * N + y]);
                Cc[(z * M + x) * N + y] = (uint8_t)(2 * acc > thresh[z * N + y]);
            }
}

/* extensions/src/max_pool2d.cu:14-32 -- bitwise OR over a window that the kernel fixes
 * at 2x2 whatever filterx/filtery say (max_pool2d.cu:21,23); the filter sizes only
 * enter the output size (booleanOperations.py:234-235, max_pool2d.cu:14). */
void FN(nbo_max_pool2d)(WORD *out, const WORD *in, int64_t B, int64_t H, int64_t W, int64_t Cw,
                        int fx, int fy, int px, int py, int sx, int sy)
{
    const int64_t h = (H - fx + 2 * px) / sx + 1;
    const int64_t w = (W - fy + 2 * py) / sy + 1;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; b++)
        for (int64_t loc = 0; loc < h * w; loc++) {
            const int64_t xo = loc / w, yo = loc - xo * w;
            for (int64_t c = 0; c < Cw; c++) {
                WORD tmp = 0;
                for (int i = 0; i < 2; i++)
                    for (int j = 0; j < 2; j++) {
                        const int64_t xi = i + xo * sx - px, yi = j + yo * sy - py;
                        if (xi >= 0 && xi < H && yi >= 0 && yi < W)
                            tmp |= in[((b * H + xi) * W + yi) * Cw + c];
                    }
                out[(b * h * w + loc) * Cw + c] = tmp;
            }
        }
}

/* Law and layout of extensions/src/sample_bits.cu:47-57 (ret[x][y][z] bit i set when the
 * probability of column z*bits+i beats the draw; tail columns have p=0, sample_bits.cu:35)
 * with the cuRAND draw replaced by a supplied uint32 word per bit:
 *     bit = words[x][y][z*bits+i] < thresh[y][z*bits+i]
 * thresh == NULL means the same scalar threshold thr_scalar everywhere.
 * base  != NULL XORs the sampled mask onto base[y][z] (flip form); NULL means 0. */
void FN(nbo_sample_from_words)(WORD *ret, const WORD *base, const uint32_t *thresh, uint32_t thr_scalar,
                               const uint32_t *words, int64_t n, int64_t R, int64_t C)
{
    const int64_t Rw = (C + WBITS - 1) / WBITS;
#pragma omp parallel for schedule(static)
    for (int64_t x = 0; x < n; x++)
        for (int64_t y = 0; y < R; y++)
            for (int64_t z = 0; z < Rw; z++) {
                WORD tmp = 0;
                for (int i = 0; i < WBITS; i++) {
                    const int64_t col = z * WBITS + i;
                    if (col < C) {
                        const uint32_t t = thresh ? thresh[y * C + col] : thr_scalar;
                        const WORD b = words[(x * R + y) * C + col] < t ? 1 : 0;
                        tmp |= b << i;
                    }
                }
                ret[(x * R + y) * Rw + z] = tmp ^ (base ? base[y * Rw + z] : 0);
            }
}

/* Structure of extensions/booleanOperationsCuda.cu:184-200 (cuda_binary_seeded_bmv_kernel):
 * output (member x, row y) regenerates its weight words one at a time and accumulates
 * popc(word ^ B[x][i]); the weights never exist in memory.  The draw is a supplied word:
 *     wbit = basebit ^ (words[x][y][col] < thresh)      (same law as nbo_sample_from_words)
 * C is [n, R] int32 (booleanOperationsCuda.cu:303). */
void FN(nbo_seeded_bmv_from_words)(int32_t *Cc, const WORD *base, const uint32_t *thresh, uint32_t thr_scalar,
                                   const WORD *xin, const uint32_t *words, int64_t n, int64_t R, int64_t C)
{
    const int64_t Rw = (C + WBITS - 1) / WBITS;
#pragma omp parallel for schedule(static)
    for (int64_t x = 0; x < n; x++)
        for (int64_t y = 0; y < R; y++) {
            int32_t acc = 0;
            for (int64_t z = 0; z < Rw; z++) {
                WORD wv = base ? base[y * Rw + z] : 0;
                int64_t end = C - z * WBITS;
                if (end > WBITS) end = WBITS;
                for (int64_t i = 0; i < end; i++) {
                    const int64_t col = z * WBITS + i;
                    const uint32_t t = thresh ? thresh[y * C + col] : thr_scalar;
                    const WORD b = words[(x * R + y) * C + col] < t ? 1 : 0;
                    wv ^= b << i;
                }
                acc += POPC(wv ^ xin[x * Rw + z]);
            }
            Cc[x * R + y] = acc;
        }
}

/* extensions/src/weighted_sum.cu:28-46 -- ret[y][z] = sum_x w[x] * bit(in[x][y][z/bits], z%bits),
 * accumulated in fp32 in member order (weighted_sum.cu:26,39).  The fp16 rounding of the
 * result is left to the caller; this returns the fp32 sum. */
void FN(nbo_weighted_sum)(float *ret, const WORD *in, const float *w, int64_t n, int64_t R, int64_t Rw, int64_t zbits)
{
#pragma omp parallel for schedule(static)
    for (int64_t y = 0; y < R; y++)
        for (int64_t z = 0; z < zbits; z++) {
            float tmp = 0.f;
            const int64_t ze = z / WBITS;
            const int zb = (int)(z - ze * WBITS);
            for (int64_t x = 0; x < n; x++)
                if ((in[(x * R + y) * Rw + ze] >> zb) & 1)
                    tmp += w[x];
            ret[y * zbits + z] = tmp;
        }
}
