/*
 * nesbin.h -- C ABI of libnesbin.so: population-batched packed binary layer forward ops for
 * AMD Instinct MI355X (gfx950), a from-scratch replacement for the CUDA/CuPy kernels behind
 * jamesal1/NESgpu's extensions/booleanOperations.py, boolop_cuda and boolutil_cuda.
 *
 * Conventions (all entry points)
 *   - every pointer is a DEVICE pointer into dense row-major memory owned by the caller; the
 *     library allocates nothing and keeps no per-call state, so calls from several threads do not
 *     interfere.  The only process-wide state is the conv engine selector (nb_conv_engine, an atomic
 *     that every conv call reads once; all engines give identical results) and a per-device cache of
 *     kernel attributes;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); launches are
 *     asynchronous on it and the call never synchronises;
 *   - packed words are LSB-first: bit i of word y of a row is element y*bits+i
 *     (extensions/src/pack.cu:26); `_i64` entry points use 64-bit words, `_i32` 32-bit words
 *     (the reference retargets its kernels the same way, extensions/booleanOperations.py:10-11);
 *   - the return value is 0 on success, NB_ERR_* for rejected arguments (nothing launched), or
 *     NB_ERR_HIP_BASE + hipError_t when the runtime refused a launch.  Nothing throws.
 *     nb_last_error_string() describes the last failure on the calling thread.
 */
#ifndef NESBIN_H
#define NESBIN_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define NB_OK 0
#define NB_ERR_NULL 1        /* a required pointer is NULL */
#define NB_ERR_SHAPE 2       /* negative / inconsistent / too large dimension */
#define NB_ERR_ALIGN 3       /* pointer not aligned to its element size */
#define NB_ERR_UNSUPPORTED 4 /* combination this build has no kernel for */
#define NB_ERR_HIP_BASE 1000

typedef void *nb_stream_t;

int nb_version(void);
const char *nb_last_error_string(void);

/* ---- pack / unpack -------------------------------------------------------------------
 * pack: bool bytes [R, C] -> words [R, ceil(C/bits)], zero-filled tail.
 *   replaces extensions/booleanOperations.py:175-187 (pack_kernel, extensions/src/pack.cu:4-30)
 *   and boolutil_cuda.pack (extensions/booleanUtilities.cpp:36-40). */
int nb_pack_i64(int64_t *out, const uint8_t *in, int64_t R, int64_t C, nb_stream_t stream);
int nb_pack_i32(int32_t *out, const uint8_t *in, int64_t R, int64_t C, nb_stream_t stream);
/* unpack: words [R, Rw] -> bool bytes [R, Rw*bits].
 *   replaces boolutil_cuda.unpack (extensions/booleanUtilities.cpp:43-46,
 *   extensions/booleanUtilitiesCuda.cu:77-90,182-195). */
int nb_unpack_i64(uint8_t *out, const int64_t *in, int64_t R, int64_t Rw, nb_stream_t stream);
int nb_unpack_i32(uint8_t *out, const int32_t *in, int64_t R, int64_t Rw, nb_stream_t stream);
/* int8pack: uint8 [R, C] -> words [R, ceil(C/(bits/8))], little-endian bytes, zero tail.
 *   replaces extensions/booleanOperations.py:189-201 (extensions/src/int8pack.cu:4-30). */
int nb_int8pack_i64(int64_t *out, const uint8_t *in, int64_t R, int64_t C, nb_stream_t stream);
int nb_int8pack_i32(int32_t *out, const uint8_t *in, int64_t R, int64_t C, nb_stream_t stream);

/* ---- XOR-popcount batched matmul --------------------------------------------------------
 * C[z,x,y] = sum_k popcount(A[z,x,k] ^ B[z,k,y]);  A [Z,M,Kw], B [Z,Kw,N], C [Z,M,N] int32.
 *   replaces extensions/booleanOperations.py:107-129 (bmm_kernel, extensions/src/bmm.cu:5-58)
 *   and boolop_cuda.binary_bmm (extensions/booleanOperations.cpp:34-41). */
int nb_bmm_i64(int32_t *C, const int64_t *A, const int64_t *B, int64_t Z, int64_t M, int64_t Kw, int64_t N,
               nb_stream_t stream);
int nb_bmm_i32(int32_t *C, const int32_t *A, const int32_t *B, int64_t Z, int64_t M, int64_t Kw, int64_t N,
               nb_stream_t stream);
/* The linear layer's activations in one kernel: C[z, x] (int32 [Z, M]) = 2 * sum_k popc(A[z,x,k] ^ x[z,k]) - K, K the
 * true number of input bits (modules/binary.py:97: `2 * bmm(...) - in_features`); A [Z, M, Kw], x [Z, Kw].  The
 * matrix-vector kernels of nb_bmm (N = 1) with the affine map applied as the sums are stored. */
int nb_bmv_pm1_i64(int32_t *C, const int64_t *A, const int64_t *x, int64_t Z, int64_t M, int64_t Kw, int64_t K,
                   nb_stream_t stream);
int nb_bmv_pm1_i32(int32_t *C, const int32_t *A, const int32_t *x, int64_t Z, int64_t M, int64_t Kw, int64_t K,
                   nb_stream_t stream);
/* same with the output (2*popc > thresh[z,y]) as bool bytes; thresh [Z,N] int32.
 *   replaces extensions/booleanOperations.py:131-158 (extensions/src/bmm_act.cu:5-63). */
int nb_bmm_act_i64(uint8_t *C, const int64_t *A, const int64_t *B, const int32_t *thresh, int64_t Z, int64_t M,
                   int64_t Kw, int64_t N, nb_stream_t stream);
int nb_bmm_act_i32(uint8_t *C, const int32_t *A, const int32_t *B, const int32_t *thresh, int64_t Z, int64_t M,
                   int64_t Kw, int64_t N, nb_stream_t stream);
/* Matrix-vector form of a linear layer with the threshold and the pack fused: bit m of member z's output row is
 * (2 * sum_k popcount(A[z,m,k] ^ x[z,k]) > thresh[z,m]); A [Z,M,Kw], x [Z,Kw], thresh [Z,M] int32,
 * out [Z, ceil(M/bits)] words, LSB-first, tail bits zero.
 *   no single counterpart in the reference: it is BinarizedLinear.forward's bmm -> compare (modules/binary.py:97-106)
 *   followed by the next layer's pack (extensions/src/pack.cu:5-30), without the int32 and bool maps in between. */
int nb_bmv_act_pack_i64(int64_t *out, const int64_t *A, const int64_t *x, const int32_t *thresh, int64_t Z, int64_t M,
                        int64_t Kw, nb_stream_t stream);
int nb_bmv_act_pack_i32(int32_t *out, const int32_t *A, const int32_t *x, const int32_t *thresh, int64_t Z, int64_t M,
                        int64_t Kw, nb_stream_t stream);

/* ---- linear layer with the population-mean threshold --------------------------------------------------
 * BinarizedLinear(batch_norm=True) in one call: with popc[z,m] = sum_k popcount(A[z,m,k] ^ x[z,k]) and
 * act = 2*popc - K,
 *     mean[m]  = fp16( float(sum_z act[z,m]) * (float(M) / float(Z*M)) )   (the sum is exact integer arithmetic; the
 *                factor is what torch's fp16 mean multiplies its fp32 sum by: the quotient of the element counts;
 *                the exact product is rounded once, to fp16, as torch's kernel does)
 *     thr[z,m] = fp16( fp16(bias[m] + bias_noise[z,m]) + mean[m] )
 *     bit[z,m] = act[z,m] > thr[z,m]                            (compared exactly; false for a NaN threshold)
 * A [Z,M,Kw], x [Z,Kw], bias [M] fp16, bias_noise [Z,M] fp16 (raw 16-bit patterns), K = true bit count of a row.
 * pack bit 0 clear: out = bool bytes [Z,M]; set: out = words [Z, ceil(M/bits)], LSB-first, tail bits zero.
 * pack bit 1 set (values 2, 3): act is rounded to fp16 before it is summed and before it is compared, which is what the
 * reference's tensor expression does; it matters for K > 2048 only (K <= 65504 then).
 * workspace: device memory, 256-byte aligned, at least nb_bmv_bn_workspace_bytes(Z, M) bytes (the members' int32
 * sums and the per-output totals pass through it; contents undefined afterwards).  The weights are read once.
 *   replaces the composition of modules/binary.py:97-102 (bmm -> 2*popc - in_features -> .type(float16).mean(dim=0)
 *   -> thresh -> compare); equal to it wherever act is exact in fp16 (K <= 2048), or with pack bit 1 set, and torch's
 *   fp32 sum over the population is exact (Z * K < 2^24); beyond that torch's sum depends on its summation order. */
int64_t nb_bmv_bn_workspace_bytes(int64_t Z, int64_t M);
int nb_bmv_bn_act_i64(void *out, const int64_t *A, const int64_t *x, const uint16_t *bias, const uint16_t *bias_noise,
                      int64_t Z, int64_t M, int64_t Kw, int64_t K, int pack, void *workspace, int64_t workspace_bytes,
                      nb_stream_t stream);
int nb_bmv_bn_act_i32(void *out, const int32_t *A, const int32_t *x, const uint16_t *bias, const uint16_t *bias_noise,
                      int64_t Z, int64_t M, int64_t Kw, int64_t K, int pack, void *workspace, int64_t workspace_bytes,
                      nb_stream_t stream);
/* nb_bmv_bn_act_i64 for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the same computation with the workspace in a fixed device array of
 * nb_bmv_bn_static_bytes() bytes (4 MiB + 64 KiB) that the library holds on every GPU it runs on until the process
 * ends.  Calls no hipMalloc / hipFree / allocating routine.  Shapes that need more
 * (nb_bmv_bn_workspace_bytes(Z, M) > nb_bmv_bn_static_bytes(), i.e. beyond about a million outputs) are rejected with
 * NB_ERR_SHAPE.  All calls on one GPU share that array: calls that overlap in time on one GPU (different streams or
 * threads) race; calls on one stream do not.  No counterpart in the reference. */
int64_t nb_bmv_bn_static_bytes(void);
int nb_bmv_bn_act_static_i64(void *out, const int64_t *A, const int64_t *x, const uint16_t *bias,
                             const uint16_t *bias_noise, int64_t Z, int64_t M, int64_t Kw, int64_t K, int pack,
                             nb_stream_t stream);

/* Thresholds of BinarizedConv2d(batch_norm=True) (modules/binary.py:147-155) from the pixel sums that
 * nb_conv_popc_sums_* returns: with act = 2*popc - K over the HW output pixels,
 *     mean[d,o] = fp16(float(sum_pixels act) * (float(D*O) / float(D*O*HW)))   (the exact product rounded once: torch's
 *                 fp16 mean of a [D,h,w,O] map over its pixels wherever the fp32 sum is exact, K * HW <= 2^24),
 *     thr = fp16(fp16(bias[o] + bias_noise[d,o]) + mean),
 *     thresh[d,o] = floor(thr) + K  (int32, clamped; INT32_MAX for NaN),
 * so that nb_conv_act*(..., thresh, ...) (2*popc > thresh) decides act > thr exactly as long as the activations are
 * integers that fp16 holds exactly (K <= 2048).  sums, thresh int32 [D,O]; bias fp16 [O]; bias_noise fp16 [D,O].
 * Replaces a dozen elementwise tensor operations of the layer; no single counterpart in the reference. */
int nb_conv_bn_thresholds(int32_t *thresh, const int32_t *sums, const uint16_t *bias, const uint16_t *bias_noise,
                          int64_t D, int64_t O, int64_t K, int64_t HW, nb_stream_t stream);
/* The same thresholds straight from the layer's input: nb_conv_popc_sums_* and nb_conv_bn_thresholds in one call, without
 * a sums array (arguments as nb_conv_popc_sums_*, K = channels x taps, at least one output pixel).  Where the sums
 * come from bit counts (see the engine selector below) it is a single kernel; else the sums are written into thresh
 * and turned into thresholds in place. */
int nb_conv_bn_thresholds_from_input_i64(int32_t *thresh, const int64_t *in, const int64_t *filt, const uint16_t *bias,
                                         const uint16_t *bias_noise, int64_t D, int64_t H, int64_t W, int64_t Cw,
                                         int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits,
                                         int64_t K, nb_stream_t stream);
int nb_conv_bn_thresholds_from_input_i32(int32_t *thresh, const int32_t *in, const int32_t *filt, const uint16_t *bias,
                                         const uint16_t *bias_noise, int64_t D, int64_t H, int64_t W, int64_t Cw,
                                         int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits,
                                         int64_t K, nb_stream_t stream);

/* ---- sparse form of a population's linear layer: shared base + per-member flip lists ------------------------
 * For per-member weights W[d] = base ^ flips[d] with few flips per row (BASELINE's "base XOR Bernoulli(p) flip mask"),
 *     popcount(x ^ W[d,r]) = popcount(x ^ base[r]) + |flips[d,r]| - 2 * popcount(flips[d,r] & (x ^ base[r])):
 * one shared product for the whole population plus a correction that reads 2 bytes per flip instead of 1 bit per
 * weight bit.  Same integers as nb_bmm_i64 / nb_bmv_act_pack_i64 on the materialised W.  64-bit words only (a row of
 * 32-bit words with an even count has the same bytes).  No counterpart in the reference, whose linear layer always
 * streams materialised weights (modules/binary.py:97).
 *
 * Flip lists ("fixed slices"): with S = ceil(R / 64) and a capacity of `cap` 16-byte pieces per row, piece j of row
 * r of member d sits at dword offset (((d * S + r / 64) * cap + j) * 64 + r % 64) * 4 of entries (16-byte aligned,
 * D * S * cap * 256 dwords): the row's flips 8j .. 8j+7 (in column order from every producer but
 * nb_flip_skip_layered, which lists them class by class; no consumer needs an order, each column at most once is
 * what counts), low half of a dword first, 16 bits each:
 * [4:0] = column % 32, [15:5] = 2 * (column / 32) + b with b the base bit at that column; the last piece is padded
 * with the sentinel (4Kw) << 5, which may also stand between flips.  info[d, r] (uint32) = flips | pieces << 16: only the
 * first `pieces` pieces of a row are ever written or read.  Every row has a fixed place, so lists are written in one
 * pass, in any order, without a count first.  A row that needs more than cap pieces keeps its first 8 * cap flips and
 * adds one to overflow[0] (uint32, device memory, cleared by the caller): check it when convenient, choose a larger
 * cap and draw again.  Kw <= 511, R <= 65536, cap <= 8191.
 *
 * nb_flip_count: info[d, r] = popcount(W[d, r, :] ^ base[r, :]) | ceil(that / 8) << 16; W [D, R, Kw], base [R, Kw].
 * nb_flip_fill:  the entries and info of every row from W ^ base.
 * nb_expand_fp4: packed rows [rows, Kw] -> FP4 (E2M1) codes [rows_padded, 32 * Kw_padded] bytes, bit 1 -> +1.0,
 *                bit 0 -> -1.0, padding -> 0.0: the operand form of nb_bmm_nt_fp4.
 * nb_bmm_nt_fp4: C[m, n] = popcount(A_m ^ B_n), int32 [M, N], for two expanded operands (rows padded to multiples of
 *                128, Kw_padded even); the shared-base form of the product of extensions/src/bmm.cu:5-58 on the matrix
 *                cores (FP4 MFMA, exact for +-1).
 * nb_bmv_flip:   out[d, r] = G[d, r] + flips(d, r) - 2 * (number of member d's flips in row r whose looked-up bit is
 *                set), int32 [D, R], with G = nb_bmm_nt_fp4(x, base): equal to nb_bmm_i64(W, x) with N = 1.
 * nb_bmv_flip_act_pack: the same sums thresholded (2 * sum > thresh[d, r]) and packed along r into
 *                [D, ceil(R/64)] words: equal to nb_bmv_act_pack_i64(W, x, thresh).
 * nb_flip_to_dense: materialises flip lists: W [D, R, Kw] must hold base in every member on entry, every listed
 *                flip is XOR-ed in (interop with the dense kernels, and what the tests compare through).
 * nb_flip_weighted_sum: out[r, c] (fp16 [R, C]) = sum_d weights[d] * bit_d[r, c] with bit = base ^ flip, i.e.
 *                base[r, c] * sum_d weights[d] +- the weights of the members that flip (r, c): what
 *                nb_weighted_sum_i64 gives on the materialised weights (extensions/src/weighted_sum.cu:28-46, the
 *                update step of modules/binary.py:70), up to the order of the additions: the weights are scaled by a
 *                power of two to 32-bit integers (sum |w| * scale < 2^29) and added exactly, in any order.
 *
 * Skip sampler (generator mode of the flip form): the flipped columns of a row are a renewal process with geometric
 * gaps, so the lists can be drawn directly, about C*p + 1 random words per row instead of the C words of the per-bit
 * compare.  Row q = d*R + r reads the Philox4x32-10 words first + q*C + i, i = 0, 1, ... (stream (seed, subseq), as
 * nb_philox_words numbers them); a word has the rank #{k < Kt : cdf[k] <= word}: a rank below Kt moves the position
 * (start: -1) on by rank + 1 columns and flips the column reached, rank Kt moves it on by Kt columns without a flip;
 * the row ends when the position passes C.  The table is device memory of nb_skip_table_words() uint32: [0] = Kt
 * (<= 4096), [1] = the bits of the float 1 / log2(1 - p) (a hint for where a look-up starts probing; it changes no
 * result), [2] = the threshold p * 2^32, [3] = 0, [4 + k] = cdf[k] = floor(2^32 * (1 - (1-p)^(k+1))), sorted; Kt == 0
 * means no flips.  Written by the caller, or by nb_skip_table from a threshold in device memory (which may be
 * table + 2).  Same law as nb_sample_philox with a base and thr_scalar = p * 2^32 (i.i.d. Bernoulli(p), quantised to
 * 2^-32), another stream.  One kernel, nothing read back: the call can be captured into a HIP graph.
 * nb_flip_skip: lists with a uniform flip probability against base [R, Kw].
 * nb_flip_skip_thin: per-element probabilities by thinning.  law [R, C] uint16: bit 15 = the base bit of the column,
 *                bits 14:0 = the fp16 pattern of its flip probability y <= 1/2, Tf = floor(y * 2^32); table: made for
 *                the largest Tf of the layer (T_max = table[2]).  The words of a row come in pairs: word 2i is a gap as
 *                above, and the column it reaches flips only if word 2i+1 times T_max is below Tf * 2^32 (64-bit
 *                integers): each column flips with probability Tf / 2^32, independently.
 * nb_flip_skip_layered: per-element probabilities class by class, for laws whose largest probability is far above
 *                their mean (thinning draws C * p_max pairs per row, this about twice the row's flips plus one or
 *                two per class).  nb_flip_law_layers sorts a law [R, C] (as nb_flip_skip_thin takes it; the base
 *                bit travels along) into pl [R, C] uint32 = column | law << 16, the columns of class k
 *                (2^(30-k) < Tf <= 2^(31-k) for k < 15, 0 < Tf <= 2^16 for k = 15; Tf = 0 is left out, the tail of
 *                pl holds 0xFFFF) at pl[r, cls[r, k] .. cls[r, k+1]) in increasing column order; cls [R, 17]
 *                uint32.  tables: nb_flip_layer_table_words() uint32 of device memory filled once by
 *                nb_flip_layer_tables: 16 tables as nb_skip_table makes them, class k's for the threshold
 *                2^(31-k), of which the walk uses the first 512 entries.  The words of a row come in pairs as for
 *                nb_flip_skip_thin, class after class without a break: in class k the gap's rank in that table
 *                (a rank of 512 = beyond it) moves the position in the class's stretch of pl (start: -1), the
 *                column reached flips iff the second word is below Tf * 2^(k+1); a position past the stretch ends
 *                the class and the next class that has columns starts with the next pair.  Same law as
 *                nb_flip_skip_thin (every column flips with probability Tf / 2^32, independently), other masks.
 * Both per-element walks give row q the words from first + q*C on and use two per step, so a row that takes more than
 * C/2 steps reads into the words of row q + 1 and the two rows' draws are no longer independent: they are meant for
 * sparse laws (thinning takes about C * p_max steps, the class-by-class walk about 1.5 per flip plus 16;
 * BinarizedLinear uses them for mean flip probabilities of at most 0.04).
 * The layers' law (modules/binary.py:59-60), P = sigmoid(5 w / (mean|w| + 1e-5)), rounded to fp16 wherever the tensor
 * expression rounds; mean|w| = the exact sum over the count, rounded once to fp16.  workspace: nb_law_workspace_bytes()
 * bytes of device memory, 8-byte aligned.
 * nb_thresholds_from_weights: thresholds[i] = min(floor(P_i * 2^32), 2^32 - 1), what nb_sample_philox takes.
 * nb_probabilities_from_weights: the fp16 probabilities themselves.
 * nb_flip_law_from_weights: the sparse form of the same law: law [R, C] as nb_flip_skip_thin takes it (base bit =
 *                P >= 1/2, y = min(P, 1 - P)), base [R, Kw] packed, and table made for the layer's largest Tf. */
int64_t nb_skip_table_words(void);
int nb_skip_table(uint32_t *table, const uint32_t *threshold, nb_stream_t stream);
int nb_flip_skip_i64(uint32_t *entries, uint32_t *info, uint32_t *overflow, const int64_t *base, const uint32_t *table,
                     uint64_t seed, uint64_t subseq, uint64_t first, int64_t D, int64_t R, int64_t C, int64_t cap,
                     nb_stream_t stream);
int nb_flip_skip_thin_i64(uint32_t *entries, uint32_t *info, uint32_t *overflow, const uint16_t *law,
                          const uint32_t *table, uint64_t seed, uint64_t subseq, uint64_t first, int64_t D, int64_t R,
                          int64_t C, int64_t cap, nb_stream_t stream);
/* stats[0..2] (doubles, device memory) = the mean flip probability of a law [R, C], the largest mean of a row, the
 * largest flip probability (table[2] / 2^32, table as nb_flip_law_from_weights left it): what a host needs to choose
 * between the dense and the sparse form, between the two walks, and the lists' capacity, in one read-back.
 * row_sums: R floats of workspace. */
int nb_flip_law_stats(double *stats, float *row_sums, const uint16_t *law, const uint32_t *table, int64_t R, int64_t C,
                      nb_stream_t stream);
int64_t nb_flip_layer_table_words(void);
int nb_flip_layer_tables(uint32_t *tables, nb_stream_t stream);
int nb_flip_law_layers(uint32_t *pl, uint32_t *cls, const uint16_t *law, int64_t R, int64_t C, nb_stream_t stream);
int nb_flip_skip_layered_i64(uint32_t *entries, uint32_t *info, uint32_t *overflow, const uint32_t *pl,
                             const uint32_t *cls, const uint32_t *tables, uint64_t seed, uint64_t subseq, uint64_t first,
                             int64_t D, int64_t R, int64_t C, int64_t cap, nb_stream_t stream);
/* The skip sampler's masks as packed words, for short rows (at most 8 words): out = base ^ mask (base NULL: the mask
 * alone), the mask of row q = m*R + r being exactly the flips nb_flip_skip_i64 lists for it (same table, same words
 * first + q*C + i of the stream), i.e. what nb_flip_to_dense_i64 makes of those lists.  Same layouts as the per-bit
 * samplers: nb_sample_skip writes [n, R, ceil(C/bits)]; nb_sample_conv_skip takes the rows as (out channel, tap) pairs,
 * R = O * KK, and writes out_rows [n, R, Rw] and / or out_conv [n, KK * Rw, O] like nb_sample_conv_philox (either may
 * be NULL, not both).  About C*p + 1 random words per row instead of C: the conv layers' filters at small flip
 * probabilities.  No counterpart in the reference (extensions/src/sample_bits.cu:47-57 draws every bit). */
int nb_sample_skip_i64(int64_t *out, const int64_t *base, const uint32_t *table, uint64_t seed, uint64_t subseq,
                       uint64_t first, int64_t n, int64_t R, int64_t C, nb_stream_t stream);
int nb_sample_skip_i32(int32_t *out, const int32_t *base, const uint32_t *table, uint64_t seed, uint64_t subseq,
                       uint64_t first, int64_t n, int64_t R, int64_t C, nb_stream_t stream);
int nb_sample_conv_skip_i64(int64_t *out_conv, int64_t *out_rows, const int64_t *base, const uint32_t *table,
                            uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t O, int64_t KK, int64_t C,
                            nb_stream_t stream);
int nb_sample_conv_skip_i32(int32_t *out_conv, int32_t *out_rows, const int32_t *base, const uint32_t *table,
                            uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t O, int64_t KK, int64_t C,
                            nb_stream_t stream);
int64_t nb_law_workspace_bytes(void);
int nb_thresholds_from_weights(uint32_t *thresholds, const uint16_t *weights, int64_t n, void *workspace,
                               nb_stream_t stream);
int nb_probabilities_from_weights(uint16_t *p, const uint16_t *weights, int64_t n, void *workspace, nb_stream_t stream);
int nb_flip_law_from_weights(uint16_t *law, int64_t *base, uint32_t *table, const uint16_t *weights, int64_t R, int64_t C,
                             void *workspace, nb_stream_t stream);
int nb_flip_to_dense_i64(int64_t *W, const uint32_t *entries, const uint32_t *info, int64_t D, int64_t R, int64_t Kw,
                         int64_t cap, nb_stream_t stream);
int nb_flip_count_i64(uint32_t *info, const int64_t *W, const int64_t *base, int64_t D, int64_t R, int64_t Kw,
                      nb_stream_t stream);
int nb_flip_fill_i64(uint32_t *entries, uint32_t *info, uint32_t *overflow, const int64_t *W, const int64_t *base,
                     int64_t D, int64_t R, int64_t Kw, int64_t cap, nb_stream_t stream);
int nb_expand_fp4_i64(uint8_t *out, const int64_t *in, int64_t rows, int64_t Kw, int64_t rows_padded, int64_t Kw_padded,
                      nb_stream_t stream);
int nb_bmm_nt_fp4(int32_t *C, const uint8_t *A, const uint8_t *B, int64_t M, int64_t N, int64_t Kw, int64_t M_padded,
                  int64_t N_padded, int64_t Kw_padded, nb_stream_t stream);
int nb_bmv_flip_i64(int32_t *out, const int32_t *G, const uint32_t *entries, const uint32_t *info, const int64_t *x,
                    int64_t D, int64_t R, int64_t Kw, int64_t cap, nb_stream_t stream);
int nb_bmv_flip_act_pack_i64(int64_t *out, const int32_t *G, const uint32_t *entries, const uint32_t *info,
                             const int64_t *x, const int32_t *thresh, int64_t D, int64_t R, int64_t Kw, int64_t cap,
                             nb_stream_t stream);
int nb_flip_weighted_sum_i64(uint16_t *out, const uint32_t *entries, const uint32_t *info, const int64_t *base,
                             const uint16_t *weights, int64_t D, int64_t R, int64_t C, int64_t cap, nb_stream_t stream);

/* ---- packed im2col / conv -----------------------------------------------------------------
 * Geometry: input [D,H,W,Cw] (channels-last packed), fx taps along H, fy taps along W,
 * h=(H-fx+2px)/sx+1, w=(W-fy+2py)/sy+1, out-of-range taps read the zero word.
 * im2col: -> [D, h*w, fx*fy*Cw], element (i*fy+j)*Cw+c.
 *   replaces extensions/booleanOperations.py:82-102 (extensions/src/batch_im2col.cu:3-33) and
 *   boolop_cuda.batch_im2col (extensions/booleanOperations.cpp:52-55). */
int nb_im2col_i64(int64_t *out, const int64_t *in, int64_t D, int64_t H, int64_t W, int64_t Cw, int fx, int fy,
                  int px, int py, int sx, int sy, nb_stream_t stream);
int nb_im2col_i32(int32_t *out, const int32_t *in, int64_t D, int64_t H, int64_t W, int64_t Cw, int fx, int fy,
                  int px, int py, int sx, int sy, nb_stream_t stream);
/* conv: filt [D, fx*fy*Cw, O] -> out [D,h,w,O] int32 popcount sums; equals
 * bmm(im2col(in), filt) without materialising the columns.
 *   replaces extensions/booleanOperations.py:162-166 and boolop_cuda.binary_batch_conv2d
 *   (extensions/booleanOperations.cpp:43-50, extensions/booleanOperationsCuda.cu:295-298).
 * tap_bits (all conv entry points): 0 = the layout above.  tap_bits = C > 0 declares that Cw == 1 and only
 * the low C <= bits/2 bits of every input word are used (C true channels, zero tail as pack writes it); filt
 * must then be the TAP-PACKED filter [D, ceil(fx*fy/T), O], T = bits/C, produced by nb_tap_pack_filter_*.
 * T taps share a word, the sums are identical, the work is T times smaller. */
int nb_conv_i64(int32_t *out, const int64_t *in, const int64_t *filt, int64_t D, int64_t H, int64_t W, int64_t Cw,
                int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits, nb_stream_t stream);
int nb_conv_i32(int32_t *out, const int32_t *in, const int32_t *filt, int64_t D, int64_t H, int64_t W, int64_t Cw,
                int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits, nb_stream_t stream);
/* conv_act: out [D,h,w,O] bool bytes = 2*popc > thresh[d,o]; thresh [D,O] int32.
 *   replaces extensions/booleanOperations.py:168-172. */
int nb_conv_act_i64(uint8_t *out, const int64_t *in, const int64_t *filt, const int32_t *thresh, int64_t D,
                    int64_t H, int64_t W, int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy,
                    int tap_bits, nb_stream_t stream);
int nb_conv_act_i32(uint8_t *out, const int32_t *in, const int32_t *filt, const int32_t *thresh, int64_t D,
                    int64_t H, int64_t W, int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy,
                    int tap_bits, nb_stream_t stream);
/* conv_act_pack: the same bits packed along O into [D,h,w,ceil(O/bits)] words; with pool != 0
 * the 2x2 / stride-2 / no-padding OR-pool of those words, [D,h/2,w/2,ceil(O/bits)].
 * Equals pack(conv_act(...)) followed (pool) by max_pool2d(.,2,2,0,0,2,2); it fuses the chain
 * conv_act -> pack -> max_pool2d of modules/binary.py:156-157,141-142,177-182 so the bool map
 * never reaches memory.  No single counterpart in the reference. */
int nb_conv_act_pack_i64(int64_t *out, const int64_t *in, const int64_t *filt, const int32_t *thresh, int64_t D,
                         int64_t H, int64_t W, int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx,
                         int sy, int pool, int tap_bits, nb_stream_t stream);
int nb_conv_act_pack_i32(int32_t *out, const int32_t *in, const int32_t *filt, const int32_t *thresh, int64_t D,
                         int64_t H, int64_t W, int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx,
                         int sy, int pool, int tap_bits, nb_stream_t stream);
/* conv_popc_sums: sums[d,o] = sum over the output pixels of conv(...)[d,:,:,o], int32 [D,O] (the library zeroes
 * it first; rejected when a member's sum could overflow int32).  This is what the per-member mean of
 * BinarizedConv2d(batch_norm=True) needs (modules/binary.py:147-155: thresh = bias + bias_noise +
 * activation.mean over h,w with activation = 2*conv - K), without the int32 maps reaching memory.  No single
 * counterpart in the reference. */
int nb_conv_popc_sums_i64(int32_t *sums, const int64_t *in, const int64_t *filt, int64_t D, int64_t H, int64_t W,
                          int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits,
                          nb_stream_t stream);
int nb_conv_popc_sums_i32(int32_t *sums, const int32_t *in, const int32_t *filt, int64_t D, int64_t H, int64_t W,
                          int64_t Cw, int64_t O, int fx, int fy, int px, int py, int sx, int sy, int tap_bits,
                          nb_stream_t stream);
/* Conv engine selector (process-wide tunable, not per call).  The engines compute the same sums bit for bit: the
 * XOR-popcount kernels (any shape) and a matrix-core kernel (64-bit words, 3-row windows, stride 1, O % 16 == 0,
 * one band of a member's image fits LDS) that feeds the bits to the matrix cores as +-1 bytes (int8 MFMA) or, for
 * full channel words of 64, 128 or 256 channels, as FP4 codes (FP4 MFMA, twice the rate, exact for +-1).
 * Narrow layers (tap-packed filters of at most 16 channels, at most 64 output channels, 3-row windows of up to 3
 * columns, stride 1, packed output) have a matrix-core kernel of their own that serves any population; packed
 * outputs and pixel sums of 3x3 windows over one word per pixel have another (tap-packed filters of 17 to 32
 * channels as +-1 bytes; full channel words as FP4 codes, engines 0 and 2).
 * 0 = automatic: the matrix-core kernels for populations of 128 members or more (the narrow one always), else
 * XOR-popcount; nb_conv_popc_sums_i64 of a stride-1 layer with filters of at most 5 x 5 runs no conv at all then: it
 * counts the image's bits per tap and finishes with one small dot product per output channel (same integers);
 * 1 = XOR-popcount only; 2 = matrix cores wherever a kernel covers the shape; 3 = as 2, +-1 bytes only.  Returns
 * the previous setting; any other argument only queries.  Initial value from the environment variable
 * NESBIN_CONV_ENGINE: first letter 'v' -> 1, 'm' -> 2, 'i' -> 3, else 0.  No counterpart in the reference. */
int nb_conv_engine(int engine);
/* Engine that served the calling thread's latest conv / conv_act / conv_act_pack launch: 1 = XOR-popcount,
 * 2 = matrix cores on +-1 bytes, 4 = matrix cores on FP4 codes, 5 = pixel sums from bit counts, 0 = none yet.  For tests and tuning.  No
 * counterpart in the reference. */
int nb_conv_last_engine(void);
/* tap_pack_filter: filt [D, taps, O] (one word per tap, Cw == 1) -> out [D, ceil(taps/T), O], T = bits/tap_bits,
 * out[d,w,o] = OR_t (filt[d,w*T+t,o] & (2^tap_bits - 1)) << (tap_bits*t).  A layout transform of the
 * per-member filters of modules/binary.py:136-137; no counterpart in the reference. */
int nb_tap_pack_filter_i64(int64_t *out, const int64_t *filt, int64_t D, int64_t taps, int64_t O, int tap_bits,
                           nb_stream_t stream);
int nb_tap_pack_filter_i32(int32_t *out, const int32_t *filt, int64_t D, int64_t taps, int64_t O, int tap_bits,
                           nb_stream_t stream);

/* ---- packed max-pool -------------------------------------------------------------------------
 * [B,H,W,Cw] -> [B,h,w,Cw]; bitwise OR over the 2x2 window anchored at (xo*sx-px, yo*sy-py),
 * zero outside.  fx, fy only set the output size, as in the reference kernel whose window
 * loops are fixed at 2 (extensions/src/max_pool2d.cu:21-23).
 *   replaces extensions/booleanOperations.py:232-252 (extensions/src/max_pool2d.cu:3-36). */
int nb_max_pool2d_i64(int64_t *out, const int64_t *in, int64_t B, int64_t H, int64_t W, int64_t Cw, int fx, int fy,
                      int px, int py, int sx, int sy, nb_stream_t stream);
int nb_max_pool2d_i32(int32_t *out, const int32_t *in, int64_t B, int64_t H, int64_t W, int64_t Cw, int fx, int fy,
                      int px, int py, int sx, int sy, nb_stream_t stream);

/* ---- Bernoulli bit sampling ------------------------------------------------------------------
 * Law and layout of sample_bits (extensions/booleanOperations.py:203-215,
 * extensions/src/sample_bits.cu:47-57; boolutil_cuda.sample_bits,
 * extensions/booleanUtilities.cpp:49-52): out [n,R,ceil(C/bits)], one independent draw per
 * (member, row, column), tail bits zero.  The cuRAND XORWOW draw is replaced by a uint32 word:
 *     bit(m,r,c) = word(m,r,c) < threshold(r,c)
 * threshold(r,c) = thresh[r*C+c] if thresh != NULL else thr_scalar.  If base != NULL
 * ([R,ceil(C/bits)]) the sampled mask is XORed onto it: out = base ^ mask (bit-flip form).
 * from_words: word(m,r,c) = words[(m*R+r)*C+c], supplied by the caller.
 * philox:     word(m,r,c) = lane g%4 of Philox4x32-10(counter=(lo(g/4),hi(g/4),lo(subseq),
 *             hi(subseq)), key=(lo(seed),hi(seed))), g = first + (m*R+r)*C+c  -- the same
 *             numbers nb_philox_words writes, so the two forms agree bit for bit. */
int nb_sample_from_words_i64(int64_t *out, const int64_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                             const uint32_t *words, int64_t n, int64_t R, int64_t C, nb_stream_t stream);
int nb_sample_from_words_i32(int32_t *out, const int32_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                             const uint32_t *words, int64_t n, int64_t R, int64_t C, nb_stream_t stream);
int nb_sample_philox_i64(int64_t *out, const int64_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                         uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t C,
                         nb_stream_t stream);
int nb_sample_philox_i32(int32_t *out, const int32_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                         uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t C,
                         nb_stream_t stream);
int nb_philox_words(uint32_t *out, uint64_t seed, uint64_t subseq, uint64_t first, int64_t count,
                    nb_stream_t stream);
/* philox16: the same law from 16-bit draws, two columns per generated word (the generator's vector instructions,
 * not memory, bound the per-bit samplers above).  Column g = first + (m*R+r)*C + c takes half-word g % 2 (low half
 * first) of element g / 2 of the stream (seed, subseq): h; the bit is set iff h < T >> 16, or h == T >> 16 and
 * l < (T & 0xFFFF) with l the low 16 bits of element g of the stream (seed, subseq ^ 2^63): probability exactly
 * T / 2^32, independent columns; the second stream is read on ties only (2^-16 of the columns).  Other bits than
 * nb_sample_philox draws from the same seed.  Needs rows of whole words (C % bits == 0), first % 8 == 0 and 16-byte
 * aligned thresholds; NB_ERR_UNSUPPORTED otherwise.  The conv forms write the second layout like
 * nb_sample_conv_philox.  No counterpart in the reference (one 32-bit uniform per bit, extensions/src/sample_bits.cu:54). */
int nb_sample_philox16_i64(int64_t *out, const int64_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                           uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t C,
                           nb_stream_t stream);
int nb_sample_philox16_i32(int32_t *out, const int32_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                           uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R, int64_t C,
                           nb_stream_t stream);
int nb_sample_conv_philox16_i64(int64_t *out_conv, int64_t *out_rows, const int64_t *base, const uint32_t *thresh,
                                uint32_t thr_scalar, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n,
                                int64_t O, int64_t KK, int64_t C, nb_stream_t stream);
int nb_sample_conv_philox16_i32(int32_t *out_conv, int32_t *out_rows, const int32_t *base, const uint32_t *thresh,
                                uint32_t thr_scalar, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n,
                                int64_t O, int64_t KK, int64_t C, nb_stream_t stream);
/* Sampler thresholds from fp16 probabilities (what the layers' set_noise feeds the samplers, modules/binary.py:59-62):
 * T[i] = min(floor(P[i] * 2^32), 2^32 - 1), 0 for P <= 0 and NaN; exact (fp16 has 11 significant bits).  P = 1.0 fails
 * only for the word 0xFFFFFFFF, like `p > u` with u in (0, 1] (extensions/src/sample_bits.cu:54). */
int nb_thresholds_from_p(uint32_t *T, const uint16_t *P, int64_t n, nb_stream_t stream);
/* The same samplers for a conv layer's filters: the R = O * KK rows are (out channel o, tap t) pairs, r = o * KK + t
 * (the layer's weight is [O*kx*ky, C], modules/binary.py:125), and the kernel writes every sampled word ALSO (or
 * only, when out_rows is NULL) where the conv multiplies it: out_conv [n, KK * Rw, O] with word wi of row (o, t) at
 * [m][t * Rw + wi][o], Rw = ceil(C/bits).  One pass instead of sample -> view -> permute(0,2,3,4,1) -> contiguous
 * (modules/binary.py:134-137); out_rows keeps the [n, R, Rw] layout that the update step sums over. */
int nb_sample_conv_from_words_i64(int64_t *out_conv, int64_t *out_rows, const int64_t *base, const uint32_t *thresh,
                                  uint32_t thr_scalar, const uint32_t *words, int64_t n, int64_t O, int64_t KK,
                                  int64_t C, nb_stream_t stream);
int nb_sample_conv_from_words_i32(int32_t *out_conv, int32_t *out_rows, const int32_t *base, const uint32_t *thresh,
                                  uint32_t thr_scalar, const uint32_t *words, int64_t n, int64_t O, int64_t KK,
                                  int64_t C, nb_stream_t stream);
int nb_sample_conv_philox_i64(int64_t *out_conv, int64_t *out_rows, const int64_t *base, const uint32_t *thresh,
                              uint32_t thr_scalar, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t O,
                              int64_t KK, int64_t C, nb_stream_t stream);
int nb_sample_conv_philox_i32(int32_t *out_conv, int32_t *out_rows, const int32_t *base, const uint32_t *thresh,
                              uint32_t thr_scalar, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t O,
                              int64_t KK, int64_t C, nb_stream_t stream);

/* ---- fused sample + XOR-popcount matrix-vector product -------------------------------------------
 * C[m,r] = sum_k popcount(w(m,r,k) ^ x[m,k]) where w is what nb_sample_* would have written;
 * the per-member weights never exist in memory.  x [n,ceil(C/bits)], C [n,R] int32.
 *   replaces boolop_cuda.binary_seeded_bmv (extensions/booleanOperations.cpp:58-63,
 *   extensions/booleanOperationsCuda.cu:172-202,301-322). */
int nb_seeded_bmv_from_words_i64(int32_t *C, const int64_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                                 const int64_t *x, const uint32_t *words, int64_t n, int64_t R, int64_t Cbits,
                                 nb_stream_t stream);
int nb_seeded_bmv_from_words_i32(int32_t *C, const int32_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                                 const int32_t *x, const uint32_t *words, int64_t n, int64_t R, int64_t Cbits,
                                 nb_stream_t stream);
int nb_seeded_bmv_philox_i64(int32_t *C, const int64_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                             const int64_t *x, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R,
                             int64_t Cbits, nb_stream_t stream);
int nb_seeded_bmv_philox_i32(int32_t *C, const int32_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                             const int32_t *x, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R,
                             int64_t Cbits, nb_stream_t stream);
/* The same product over the 16-bit draws of nb_sample_philox16 (C[m,r] = what nb_bmm gives on nb_sample_philox16's
 * output and x): needs Cbits % 8 == 0, first % 8 == 0 and 16-byte aligned thresholds, NB_ERR_UNSUPPORTED otherwise. */
int nb_seeded_bmv_philox16_i64(int32_t *C, const int64_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                               const int64_t *x, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R,
                               int64_t Cbits, nb_stream_t stream);
int nb_seeded_bmv_philox16_i32(int32_t *C, const int32_t *base, const uint32_t *thresh, uint32_t thr_scalar,
                               const int32_t *x, uint64_t seed, uint64_t subseq, uint64_t first, int64_t n, int64_t R,
                               int64_t Cbits, nb_stream_t stream);

/* ---- weighted sum of packed masks (update step) ---------------------------------------------------
 * ret[r,z] = fp16( sum_m float(w[m]) * bit(in[m,r,z/bits], z%bits) ), fp32 accumulation in member
 * order; in [n,R,Rw], w [n] fp16, ret [R,zbits] fp16.
 *   replaces extensions/booleanOperations.py:218-229 (extensions/src/weighted_sum.cu:8-48) and
 *   boolutil_cuda.binary_weighted_sum (extensions/booleanUtilities.cpp:54-59). */
int nb_weighted_sum_i64(uint16_t *ret, const int64_t *in, const uint16_t *w, int64_t n, int64_t R, int64_t Rw,
                        int64_t zbits, nb_stream_t stream);
int nb_weighted_sum_i32(uint16_t *ret, const int32_t *in, const uint16_t *w, int64_t n, int64_t R, int64_t Rw,
                        int64_t zbits, nb_stream_t stream);
/* The same sum with the fp32 additions blocked instead of in member order: per output bit the members are taken 8
 * at a time through tables of partial sums (sum of the weights of the set bits of a byte), the groups of a chunk of 64
 * members and then the chunks are added in a fixed order (the same result on every run).  It differs from
 * nb_weighted_sum by fp32 rounding of the partial sums only (a few 1e-7 of sum |w|), inside the reference's own
 * tolerance for this op (booloptests.py:284-285, rtol 1e-2), and runs about three times as fast.  Same arguments
 * and checks; needs R * Rw * (word bytes / 4) < 2^25. */
int nb_weighted_sum_fast_i64(uint16_t *ret, const int64_t *in, const uint16_t *w, int64_t n, int64_t R, int64_t Rw,
                             int64_t zbits, nb_stream_t stream);
int nb_weighted_sum_fast_i32(uint16_t *ret, const int32_t *in, const uint16_t *w, int64_t n, int64_t R, int64_t Rw,
                             int64_t zbits, nb_stream_t stream);

/* ---- the steps around weighted_sum in a layer's update ---------------------------------------------
 * The tensor expressions of modules/binary.py:67-77 other than the weighted sum, one launch each.
 *
 * nb_center_fitness: out[i] (fp16) = fp16(x[i] - mean), x = fp16(in[i]) (round to nearest even), mean = the mean of the
 *   x[i] rounded once to fp16 (the sum taken in double precision); replaces modules/binary.py:68-69
 *   (weights.type(torch.float16); weights - weights.mean()).  torch's fp16 mean adds in fp32 in an order of its own
 *   and multiplies by a rounded 1/n, so the two means can differ by one fp16 step when the exact mean lies within a
 *   few 1e-7 (relative) of the middle between two fp16 numbers.  in: fp16 (_f16) or fp32 (_f32), n values.
 * nb_grad_regularize: grad[i] = fp16(fp16(grad[i] + fp16(l1 * sign(weight[i]))) + fp16(l2 * weight[i])), in place, a
 *   zero coefficient skipping its step; replaces modules/binary.py:73-76 with the same roundings (products in fp32
 *   with the coefficient as a float, every tensor fp16).  sign(NaN) = 0.
 * nb_bias_grad: out[o] (fp16 [O]) = fp16(sum_d centered[d] * bias_noise[d, o]), fp32 accumulation in a fixed order;
 *   replaces modules/binary.py:77 (weights @ self.bias_noise; a library product there, whose order is its own).
 *   centered fp16 [n], bias_noise fp16 [n, O]. */
int nb_center_fitness_f16(uint16_t *out, const uint16_t *in, int64_t n, nb_stream_t stream);
int nb_center_fitness_f32(uint16_t *out, const float *in, int64_t n, nb_stream_t stream);
int nb_grad_regularize(uint16_t *grad, const uint16_t *weight, float l1, float l2, int64_t n, nb_stream_t stream);
int nb_bias_grad(uint16_t *out, const uint16_t *centered, const uint16_t *bias_noise, int64_t n, int64_t O,
                 nb_stream_t stream);
/* nb_bias_noise_scale: x[i] (fp16, in place) = fp16(fp16(x[i] - 0.5) * 6): the arithmetic of the bias noise of
 *   modules/binary.py:63-64 on the uniform draw (which stays torch.rand), with the tensor expression's roundings. */
int nb_bias_noise_scale(uint16_t *x, int64_t n, nb_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* NESBIN_H */
