// weighted_sum: ret[r,z] = fp16( sum_m float(w[m]) * bit(in[m,r,z/bits], z%bits) ), the reduction over
// the population that the update step applies to the sampled masks
// (extensions/src/weighted_sum.cu:28-46).  fp32 accumulation in member order, like the reference.
#include <stdlib.h>

#include <mutex>
#include <type_traits>

#include "nb_common.hpp"

namespace nb {

// Rows shorter than 32 bytes.  One wave per (row, 64-bit column): lane z owns output bit z of the column and adds the members' weights in member
// order (the reference's order, so the fp32 sums are the same).  Members are taken 64 at a time: lane j fetches the
// column word of member m0 + j (64 strided loads in flight at once instead of one load per loop step), the
// workgroup's four waves share the chunk's weights as fp32 in LDS, and then for each member its word, read out of
// lane j into a scalar register pair, is used directly as the lane mask of one v_cndmask (bit z <-> lane z):
// two v_readlane + one LDS broadcast read + v_cndmask + v_add per member and wave.
template <typename W>
__global__ __launch_bounds__(256) void weighted_sum_kernel(_Float16 *__restrict__ ret, const W *__restrict__ in,
                                                           const _Float16 *__restrict__ w, int64_t n, int64_t R,
                                                           int Rw, int zbits, int ncol)
{
    constexpr int bits = WordTraits<W>::bits;
    constexpr int wpc = 64 / bits;  // words per 64-bit column
    __shared__ float wsh[2][64];
    const int lane = threadIdx.x & 63;
    const int64_t cid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (row, column); past the end: idle but in step
    const bool live = cid < R * ncol;
    const int64_t r = live ? cid / ncol : 0;
    const int c = live ? (int)(cid - r * ncol) : 0;
    const int64_t stride = R * (int64_t)Rw;
    const W *p = in + r * Rw + (int64_t)c * wpc;
    const bool has_hi = wpc == 1 || c * wpc + 1 < Rw;
    const uint16_t *wr = reinterpret_cast<const uint16_t *>(w);
    // The next chunk's words and weights are fetched before the current chunk is summed, always and from a valid place
    // (members past n: the last member again; idle waves: row 0), and masked where they are used: a load whose result
    // joins a zero from another path would be waited for right where it is issued.
    uint32_t vlo, vhi, wa;
    auto fetch = [&](int64_t m) {
        const W *q = p + (m < n ? m : n - 1) * stride;
        if (wpc == 1) {
            const uint64_t v = (uint64_t)q[0];
            vlo = (uint32_t)v;
            vhi = (uint32_t)(v >> 32);
        } else {
            vlo = (uint32_t)q[0];
            vhi = (uint32_t)q[has_hi ? 1 : 0];
        }
        wa = wr[m < n ? m : n - 1];
    };
    if (n <= 0) {  // no members: zeros, and nothing to fetch
        if (live && c * 64 + lane < zbits) ret[r * zbits + c * 64 + lane] = (_Float16)0.f;
        return;
    }
    fetch(lane);
    float acc = 0.f;
    int buf = 0;
    for (int64_t m0 = 0; m0 < n; m0 += 64, buf ^= 1) {
        const int64_t m = m0 + lane;
        const uint32_t keep = live && m < n ? 0xFFFFFFFFu : 0u;  // members past n: the zero word, nothing is added
        const uint32_t clo = vlo & keep, chi = has_hi ? vhi & keep : 0u;
        if (threadIdx.x < 64) wsh[buf][lane] = m < n ? (float)__builtin_bit_cast(_Float16, (uint16_t)wa) : 0.f;
        // one barrier per chunk: a buffer is written again two chunks later, after every wave has passed the barrier
        // of the chunk in between
        __syncthreads();
        fetch(m + 64);
#pragma unroll 8
        for (int j = 0; j < 64; j++) {
            const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)clo, j);
            const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)chi, j);
            const uint64_t mask = ((uint64_t)hi << 32) | lo;
            const float wm = wsh[buf][j];
            float t;
            asm("v_cndmask_b32_e64 %0, 0, %1, %2" : "=v"(t) : "v"(wm), "s"(mask));  // t = bit z of the word ? wm : 0
            acc += t;  // adding zero for a clear bit leaves the running sum unchanged
        }
    }
    const int z = c * 64 + lane;
    if (live && z < zbits) ret[r * zbits + z] = (_Float16)acc;
}

// Rows of 32 bytes or more: one wave per (row, 32-byte piece), a workgroup's four waves on four
// consecutive pieces, so that every 128-byte line of every member's row is fetched by one workgroup, once, in one
// 32-byte access per lane (lane j holds the piece of member m0 + j in 8 registers; the next 64 members' pieces are
// requested before the current ones are used).  The piece holds four 64-bit columns; lane z owns output bit z of
// each and keeps four running sums, all in member order.  The members' words reach the lanes through LDS instead
// of v_readlane: the wave stores its 64 pieces split into the low and the high halves of the four columns, and lane
// z reads, per member, the 16 bytes that hold its half of all four columns (one broadcast read).  Per member and
// column that leaves v_bfe_i32 (bit z as 0 / -1), v_and with the member's weight and v_add: three vector
// instructions and no scalar operand, against two lane reads, an LDS read, a select and an add above.  (A wave per
// 64-byte piece with eight sums measured the same or slower: half as many waves to hide the LDS reads behind.)
#define NB_WS_COL(ACC, D) ACC += __builtin_bit_cast(float, __builtin_amdgcn_sbfe((int)(D), zz, 1u) & wbits);

// VEC: rows are whole pieces and 16-byte aligned (16-byte loads); otherwise the piece is fetched as 4-byte loads, those
// past the end of the row left out (rows of 9 words, say: a conv layer's filters).
// COLS: 64-bit columns per wave, 4 (a 32-byte piece) or 2 (16 bytes: twice the waves, for outputs too small to give
// every SIMD a wave otherwise).
template <bool VEC, int COLS>
__global__ __launch_bounds__(256) void weighted_sum_line_kernel(_Float16 *__restrict__ ret,
                                                                const uint32_t *__restrict__ in,
                                                                const _Float16 *__restrict__ w, int64_t n, int64_t R,
                                                                int rowdw, int zbits, int npiece)
{
    typedef typename std::conditional<COLS == 4, uint4, uint2>::type half_t;  // one half (low or high) of the columns
    __shared__ half_t msk[2][4][2][64];  // [buffer][wave][low halves, high halves][member]
    __shared__ float wsh[2][64];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t pid = (int64_t)blockIdx.x * 4 + wv;  // (row, piece); past the end: idle but in step
    const bool live = pid < R * npiece;
    const int64_t r = live ? pid / npiece : 0;
    const int g = live ? (int)(pid - r * npiece) : 0;
    const int64_t stride = R * (int64_t)rowdw;  // dwords from one member's row to the next member's
    const uint32_t *p = in + r * rowdw + (int64_t)g * (2 * COLS);
    const int left = rowdw - g * (2 * COLS);    // dwords of the row from this piece on
    // The fetch is unconditional and what it brings is masked where it is used, a chunk later: a load whose result
    // joins a zero from another path (a member past n, a dword past the row's end) gets moved out of the registers it
    // arrives in, and the wait for it would then sit right behind the load instead of behind the chunk's arithmetic.
    // Members past n read the last member's piece, dwords past the row's end the row's last dword; idle waves read
    // row 0.  The weight stays fp16 until then for the same reason.  (Fetching two or four chunks ahead measured slower.)
    auto fetch = [&](uint4 &x, uint4 &y, int64_t m) {
        const uint32_t *q = p + (m < n ? m : n - 1) * stride;
        if (VEC) {
            x = load_stream16(q);
            if (COLS == 4) y = load_stream16(q + 4);
        } else {
            // plain loads: those of a lane share a cache line, which streaming loads would fetch once per load
            const int last = left - 1;  // >= 0: a piece holds output bits
            x.x = q[0];
            x.y = q[last < 1 ? last : 1];
            x.z = q[last < 2 ? last : 2];
            x.w = q[last < 3 ? last : 3];
            if (COLS == 4) {
                y.x = q[last < 4 ? last : 4];
                y.y = q[last < 5 ? last : 5];
                y.z = q[last < 6 ? last : 6];
                y.w = q[last < 7 ? last : 7];
            }
        }
    };
    // keep(k): the mask that dword k of the piece fetched for member m has to pass
    auto keep = [&](int k, int64_t m) -> uint32_t { return (live && m < n && (VEC || k < left)) ? 0xFFFFFFFFu : 0u; };
    const uint32_t zz = lane & 31;
    const int half = lane >> 5;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    uint4 a0, a1 = make_uint4(0u, 0u, 0u, 0u);
    const uint16_t *wr = reinterpret_cast<const uint16_t *>(w);
    uint32_t wa;  // the weight's fp16 bits, as loaded
    fetch(a0, a1, lane);
    wa = wr[lane < n ? lane : n - 1];
    int buf = 0;
    for (int64_t m0 = 0; m0 < n; m0 += 64, buf ^= 1) {
        const int64_t m = m0 + lane;
        if constexpr (COLS == 4) {
            msk[buf][wv][0][lane] = make_uint4(a0.x & keep(0, m), a0.z & keep(2, m), a1.x & keep(4, m), a1.z & keep(6, m));
            msk[buf][wv][1][lane] = make_uint4(a0.y & keep(1, m), a0.w & keep(3, m), a1.y & keep(5, m), a1.w & keep(7, m));
        } else {
            msk[buf][wv][0][lane] = make_uint2(a0.x & keep(0, m), a0.z & keep(2, m));
            msk[buf][wv][1][lane] = make_uint2(a0.y & keep(1, m), a0.w & keep(3, m));
        }
        if (wv == 0) wsh[buf][lane] = m < n ? (float)__builtin_bit_cast(_Float16, (uint16_t)wa) : 0.f;
        // one barrier per chunk: a buffer is written again two chunks later, after every wave has passed the barrier
        // of the chunk in between and so has finished reading it
        __syncthreads();
        // the next chunk, always (past n: the last member's piece again, masked when used)
        fetch(a0, a1, m + 64);
        wa = wr[m + 64 < n ? m + 64 : n - 1];
        const half_t *mine = &msk[buf][wv][half][0];
#pragma unroll 8
        for (int j = 0; j < 64; j++) {
            const int wbits = __builtin_bit_cast(int, wsh[buf][j]);
            const half_t d = mine[j];
            NB_WS_COL(s0, d.x)
            NB_WS_COL(s1, d.y)
            if constexpr (COLS == 4) {
                NB_WS_COL(s2, d.z)
                NB_WS_COL(s3, d.w)
            }
        }
    }
    if (!live) return;
    _Float16 *o = ret + r * zbits;
    const int z = g * (64 * COLS) + lane;
    if (z < zbits) o[z] = (_Float16)s0;
    if (z + 64 < zbits) o[z + 64] = (_Float16)s1;
    if (COLS == 4) {
        if (z + 128 < zbits) o[z + 128] = (_Float16)s2;
        if (z + 192 < zbits) o[z + 192] = (_Float16)s3;
    }
}
#undef NB_WS_COL

template <typename W>
int weighted_sum_impl(uint16_t *ret, const W *in, const uint16_t *w, int64_t n, int64_t R, int64_t Rw, int64_t zbits,
                      nb_stream_t stream, const char *who)
{
    NB_REQUIRE(n >= 0 && R >= 0 && Rw >= 0 && zbits >= 0, "%s: negative shape", who);
    if (R * zbits == 0) return NB_OK;
    NB_REQUIRE_PTR(ret);
    NB_REQUIRE_ALIGNED(ret, 2);
    if (n > 0 && Rw > 0) {
        NB_REQUIRE_PTR(in);
        NB_REQUIRE_PTR(w);
        NB_REQUIRE_ALIGNED(in, sizeof(W));
        NB_REQUIRE_ALIGNED(w, 2);
    }
    NB_REQUIRE(zbits <= (1 << 30) && Rw <= (1 << 30), "%s: row too long", who);
    NB_REQUIRE(zbits <= Rw * (int64_t)WordTraits<W>::bits, "%s: zbits exceeds the Rw words of a row", who);
    // Rows without a tail (every bit of every word is an output bit) are one long row: the output [R, zbits] and the
    // members' [R, Rw] words are the same memory as [1, R * zbits] and [1, R * Rw].  One-word rows (a conv layer's
    // 64-channel taps) get the wide kernel that way.
    if (R > 1 && zbits == Rw * (int64_t)WordTraits<W>::bits && R * zbits <= (1 << 30)) {
        Rw *= R;
        zbits *= R;
        R = 1;
    }
    const int64_t rowbytes = Rw * (int64_t)sizeof(W);
    // a wave per 32-byte piece once that gives every SIMD a wave, a wave per 16-byte piece for outputs half that size;
    // smaller outputs spread better with a wave per column
    if (n > 0 && rowbytes >= 32 && R * ceil_div(zbits, 128) >= 1024) {
        const bool wide = R * ceil_div(zbits, 256) >= 1024;
        const int pbits = wide ? 256 : 128;
        const int64_t npiece = ceil_div(zbits, pbits);  // pieces of a row that hold output bits
        const int64_t blocks = ceil_div(R * npiece, 4);
        NB_REQUIRE(blocks <= kMaxGridX, "%s: output exceeds one launch", who);
        const bool vec = rowbytes % (pbits / 8) == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0;
        auto *kern = wide ? (vec ? weighted_sum_line_kernel<true, 4> : weighted_sum_line_kernel<false, 4>)
                          : (vec ? weighted_sum_line_kernel<true, 2> : weighted_sum_line_kernel<false, 2>);
        kern<<<dim3((unsigned)blocks), dim3(256), 0, as_stream(stream)>>>(
            reinterpret_cast<_Float16 *>(ret), reinterpret_cast<const uint32_t *>(in),
            reinterpret_cast<const _Float16 *>(w), n, R, (int)(rowbytes / 4), (int)zbits, (int)npiece);
        return check_launch(who);
    }
    const int64_t ncol = ceil_div(zbits, 64);
    const int64_t blocks = ceil_div(R * ncol, 4);
    NB_REQUIRE(blocks <= kMaxGridX, "%s: output exceeds one launch", who);
    weighted_sum_kernel<W><<<dim3((unsigned)blocks), dim3(256), 0, as_stream(stream)>>>(
        reinterpret_cast<_Float16 *>(ret), in, reinterpret_cast<const _Float16 *>(w), n, R, (int)Rw, (int)zbits,
        (int)ncol);
    return check_launch(who);
}


// ---- fast mode: blocked sums through tables of partial sums -----------------------------------------------------
// The member-order kernels above spend three vector instructions per member and output bit (one bit test, one mask,
// one add).  Here a lane owns a 32-bit column of the members' words (lanes side by side: every load of a wave is one
// 256-byte run), takes the members 32 at a time, transposes the 32 x 32 bit block in its registers (word k then
// holds output bit k of the 32 members), and adds, per output bit and group of 8 members, one entry of a table
// T[group][byte] = sum of the weights of the members whose bit is set in `byte`: a quarter of an instruction per
// transposed bit plus 3 instructions and one LDS read per 8 members.  Sums are fp32; their order is by groups of 8,
// chunks of 64 and the waves that share a column set, not by member: results differ from the member-order kernel by
// fp32 rounding only (about 1e-7 of the sum of |weights|), far inside the fp16 spacing of any result that is not
// dominated by cancellation.
//
// A workgroup has 16 waves = (16 >> SPLIT) column sets of 64 columns x (1 << SPLIT) member shares; wave (cs, ms)
// takes the chunks of 64 members ms, ms + shares, ... of its column set and builds the 8 tables of each chunk
// itself (8 KB of LDS per wave, no workgroup barrier in the loop).  At the end the shares of a column set are
// added in a fixed order through LDS (so the result does not change from run to run).
constexpr int kLutRedStride = 33;                                      // floats per lane in the reduction buffer
constexpr int kLutLdsBytes = 16 * 64 * kLutRedStride * 4;              // >= 16 waves x 8 KB of tables

template <int J>
__device__ __forceinline__ void transpose_stage(uint32_t (&a)[32])
{
    constexpr uint32_t m = J == 4 ? 0x0F0F0F0Fu : J == 2 ? 0x33333333u : 0x55555555u;
#pragma unroll
    for (int k = 0; k < 32; k++) {
        if (k & J) continue;
        // v_bitop3_b32 with table 0xE4: third operand set ? first : second, bit by bit
        const uint32_t lo = a[k], hi = a[k + J];
        a[k] = __builtin_amdgcn_bitop3_b32(lo, hi << J, m, 0xE4);
        a[k + J] = __builtin_amdgcn_bitop3_b32(lo >> J, hi, m, 0xE4);
    }
}

__device__ __forceinline__ void transpose_bits_32x32(uint32_t (&a)[32])
{
    // stage j swaps, for every k with bit j clear, the bits of a[k] at positions with bit j set with the bits of
    // a[k + j] at positions with bit j clear; after the five stages bit p of a[k] is what bit k of a[p] was
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const uint32_t lo = a[k], hi = a[k + 16];
        a[k] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);       // low halves: lo.b0 lo.b1 hi.b0 hi.b1
        a[k + 16] = __builtin_amdgcn_perm(hi, lo, 0x07060302u);  // high halves
    }
#pragma unroll
    for (int k0 = 0; k0 < 32; k0 += 16)
#pragma unroll
        for (int k = k0; k < k0 + 8; k++) {
            const uint32_t lo = a[k], hi = a[k + 8];
            a[k] = __builtin_amdgcn_perm(hi, lo, 0x06020400u);      // lo.b0 hi.b0 lo.b2 hi.b2
            a[k + 8] = __builtin_amdgcn_perm(hi, lo, 0x07030501u);  // lo.b1 hi.b1 lo.b3 hi.b3
        }
    transpose_stage<4>(a);
    transpose_stage<2>(a);
    transpose_stage<1>(a);
}

// The 8 tables of a chunk of 64 members (tbl[g * 256 + byte] = sum of the weights of the members 8 g + j whose bit j
// is set in byte), built by the wave that uses them.
__device__ __forceinline__ void lut_build_tables(float *tbl, const uint16_t *wr, int64_t m0, int64_t n, int lane)
{
    // lane (g, s): group g of the chunk, the entries whose bits 2..4 are s; bits 0, 1, 5, 6 by doubling
    const int g = lane >> 3, s = lane & 7;
    float wj[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int64_t m = m0 + 8 * g + j;
        wj[j] = m < n ? (float)__builtin_bit_cast(_Float16, wr[m]) : 0.f;
    }
    // 16 entries at a time (bit 7 clear, then set) to keep the registers for the members' words
    float e[16];
    e[0] = ((s & 1) ? wj[2] : 0.f) + ((s & 2) ? wj[3] : 0.f) + ((s & 4) ? wj[4] : 0.f);
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const float wk = wj[k < 2 ? k : k + 3];
#pragma unroll
        for (int t = 0; t < (1 << k); t++) e[t + (1 << k)] = e[t] + wk;
    }
    // register index = (bits 5, 6) << 2 | bits 0..1: the eight lanes of a group write 128 contiguous bytes
    float4 *dst = reinterpret_cast<float4 *>(tbl + g * 256 + 4 * s);
#pragma unroll
    for (int i = 0; i < 4; i++) dst[8 * i] = make_float4(e[4 * i], e[4 * i + 1], e[4 * i + 2], e[4 * i + 3]);
#pragma unroll
    for (int t = 0; t < 16; t++) e[t] += wj[7];
#pragma unroll
    for (int i = 0; i < 4; i++) dst[8 * (i + 4)] = make_float4(e[4 * i], e[4 * i + 1], e[4 * i + 2], e[4 * i + 3]);
}

template <int SPLIT>
__global__ __launch_bounds__(1024) void weighted_sum_lut_kernel(_Float16 *__restrict__ ret,
                                                                 const uint32_t *__restrict__ in,
                                                                 const _Float16 *__restrict__ w, int64_t n, int64_t Q,
                                                                 int rowdw, int zbits, int whole_rows)
{
    extern __shared__ __align__(16) float lds[];
    constexpr int SHARES = 1 << SPLIT, SETS = 16 >> SPLIT;
    const int lane = threadIdx.x & 63;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ms = wv & (SHARES - 1), cs = wv >> SPLIT;
    const int64_t q = ((int64_t)blockIdx.x * SETS + cs) * 64 + lane;  // this lane's column of 32-bit words
    // byte offset of the lane's column (past the end: the last column, never stored): 32 bits, so that a load is a
    // wave-uniform base plus a lane offset
    const uint32_t qoff = (uint32_t)(q < Q ? q : Q - 1) * 4u;
    float *tbl = lds + wv * 2048;
    const uint16_t *wr = reinterpret_cast<const uint16_t *>(w);
    float acc[32];
#pragma unroll
    for (int k = 0; k < 32; k++) acc[k] = 0.f;
    const int64_t nchunks = (n + 63) >> 6;
    for (int64_t c = ms; c < nchunks; c += SHARES) {
        const int64_t m0 = c * 64;
        uint32_t a[32];
        // the block's 32 loads: one buffer per block that ends with the last member, so that members past n read as
        // zero words (their weights are zero too); per load a wave-uniform offset and the lane's column offset
        auto fetch = [&](int64_t mb) {
            const int64_t left = n - mb;
            const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<uint32_t *>(in + mb * Q), (short)0, (int)((left < 32 ? left : 32) * Q * 4), 0x00020000);
#pragma unroll
            for (int j = 0; j < 32; j++)
                a[j] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)qoff, (int)(j * (uint32_t)Q * 4u), 2);
        };
        fetch(m0);
        lut_build_tables(tbl, wr, m0, n, lane);
        // the tables are read by other lanes of this wave only: LDS accesses of a wave are served in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        auto block = [&](auto blk) {
            transpose_bits_32x32(a);
#pragma unroll
            for (int k = 0; k < 32; k++) {
                const float t0 = tbl[(blk * 4 + 0) * 256 + (a[k] & 255u)];
                const float t1 = tbl[(blk * 4 + 1) * 256 + ((a[k] >> 8) & 255u)];
                const float t2 = tbl[(blk * 4 + 2) * 256 + ((a[k] >> 16) & 255u)];
                const float t3 = tbl[(blk * 4 + 3) * 256 + (a[k] >> 24)];
                acc[k] += (t0 + t1) + (t2 + t3);
                if ((k & 3) == 3) __builtin_amdgcn_sched_barrier(0);  // 16 lookups in flight, not all 128
            }
        };
        block(std::integral_constant<int, 0>());
        if (m0 + 32 < n) {
            fetch(m0 + 32);
            block(std::integral_constant<int, 1>());
        }
        // the next chunk's tables overwrite these: same wave, in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    if (SPLIT == 0) {
        if (q >= Q) return;
        const int64_t r = q / rowdw;
        const int z0 = (int)(q - r * rowdw) * 32;
        if (whole_rows) {
            uint4 *o = reinterpret_cast<uint4 *>(ret + q * 32);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                uint32_t h[4];
#pragma unroll
                for (int e = 0; e < 4; e++)
                    h[e] = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)acc[8 * i + 2 * e]) |
                           ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)acc[8 * i + 2 * e + 1]) << 16);
                o[i] = make_uint4(h[0], h[1], h[2], h[3]);
            }
        } else {
#pragma unroll
            for (int k = 0; k < 32; k++)
                if (z0 + k < zbits) ret[r * zbits + z0 + k] = (_Float16)acc[k];
        }
        return;
    }
    __syncthreads();  // every wave is done with its tables
#pragma unroll
    for (int k = 0; k < 32; k++) lds[(wv * 64 + lane) * kLutRedStride + k] = acc[k];
    __syncthreads();
    // thread t adds the shares of 32 / SHARES consecutive output bits of one column
    constexpr int KP = 32 >> SPLIT;
    const int col = threadIdx.x >> SPLIT, part = threadIdx.x & (SHARES - 1);
    const int cs2 = col >> 6, l2 = col & 63;
    const int64_t q2 = ((int64_t)blockIdx.x * SETS + cs2) * 64 + l2;
    if (q2 >= Q) return;
    float sum[KP];
#pragma unroll
    for (int i = 0; i < KP; i++) sum[i] = 0.f;
#pragma unroll
    for (int m = 0; m < SHARES; m++)
#pragma unroll
        for (int i = 0; i < KP; i++) sum[i] += lds[(((cs2 << SPLIT) + m) * 64 + l2) * kLutRedStride + part * KP + i];
    const int64_t r = q2 / rowdw;
    const int z0 = (int)(q2 - r * rowdw) * 32 + part * KP;
    if (whole_rows) {
        uint32_t *o = reinterpret_cast<uint32_t *>(ret + q2 * 32 + part * KP);
#pragma unroll
        for (int i = 0; i < KP; i += 2)
            o[i >> 1] = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)sum[i]) |
                        ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)sum[i + 1]) << 16);
    } else {
#pragma unroll
        for (int i = 0; i < KP; i++)
            if (z0 + i < zbits) ret[r * zbits + z0 + i] = (_Float16)sum[i];
    }
}

// The same for small outputs: a wave takes 32 columns and its two halves take the two blocks of 32 members of a
// chunk, so that twice as many waves share the work (a small layer's sum is bound by the pace of one wave over its
// chunk, not by the machine).  Lane = (half h, column): members m0 + 32 h .., tables 4 h .. 4 h + 3; the halves are two
// more shares in the final addition.
template <int SPLIT>
__global__ __launch_bounds__(1024) void weighted_sum_lut_half_kernel(_Float16 *__restrict__ ret,
                                                                      const uint32_t *__restrict__ in,
                                                                      const _Float16 *__restrict__ w, int64_t n, int64_t Q,
                                                                      int rowdw, int zbits, int whole_rows)
{
    extern __shared__ __align__(16) float lds[];
    constexpr int SHARES = 1 << SPLIT, SETS = 16 >> SPLIT;
    const int lane = threadIdx.x & 63, hb = lane >> 5;
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ms = wv & (SHARES - 1), cs = wv >> SPLIT;
    const int64_t q = ((int64_t)blockIdx.x * SETS + cs) * 32 + (lane & 31);
    float *tbl = lds + wv * 2048;
    const float *mine = tbl + hb * 1024;
    const uint16_t *wr = reinterpret_cast<const uint16_t *>(w);
    float acc[32];
#pragma unroll
    for (int k = 0; k < 32; k++) acc[k] = 0.f;
    const int64_t nchunks = (n + 63) >> 6;
    // the lane's column and its half's first member of a chunk, as one byte offset into the chunk's buffer
    const uint32_t off = (uint32_t)(q < Q ? q : Q - 1) * 4u + (uint32_t)hb * 32u * (uint32_t)Q * 4u;
    for (int64_t c = ms; c < nchunks; c += SHARES) {
        const int64_t m0 = c * 64;
        uint32_t a[32];
        const int64_t left = n - m0;
        // one buffer per chunk that ends with the last member: members past n read as zero words
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<uint32_t *>(in + m0 * Q), (short)0, (int)((left < 64 ? left : 64) * Q * 4), 0x00020000);
#pragma unroll
        for (int j = 0; j < 32; j++)
            a[j] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)off, (int)(j * (uint32_t)Q * 4u), 2);
        lut_build_tables(tbl, wr, m0, n, lane);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        transpose_bits_32x32(a);
#pragma unroll
        for (int k = 0; k < 32; k++) {
            const float t0 = mine[0 * 256 + (a[k] & 255u)];
            const float t1 = mine[1 * 256 + ((a[k] >> 8) & 255u)];
            const float t2 = mine[2 * 256 + ((a[k] >> 16) & 255u)];
            const float t3 = mine[3 * 256 + (a[k] >> 24)];
            acc[k] += (t0 + t1) + (t2 + t3);
            if ((k & 3) == 3) __builtin_amdgcn_sched_barrier(0);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();  // every wave is done with its tables
#pragma unroll
    for (int k = 0; k < 32; k++) lds[(wv * 64 + lane) * kLutRedStride + k] = acc[k];
    __syncthreads();
    // thread t < 512 adds the 2 * SHARES partial sums of 32 / SHARES consecutive output bits of one column
    constexpr int KP = 32 >> SPLIT;
    const int col = threadIdx.x >> SPLIT, part = threadIdx.x & (SHARES - 1);
    const int cs2 = col >> 5, l2 = col & 31;
    const int64_t q2 = ((int64_t)blockIdx.x * SETS + cs2) * 32 + l2;
    if (col >= SETS * 32 || q2 >= Q) return;
    float sum[KP];
#pragma unroll
    for (int i = 0; i < KP; i++) sum[i] = 0.f;
#pragma unroll
    for (int m = 0; m < SHARES; m++)
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int i = 0; i < KP; i++)
                sum[i] += lds[(((cs2 << SPLIT) + m) * 64 + h * 32 + l2) * kLutRedStride + part * KP + i];
    const int64_t r = q2 / rowdw;
    const int z0 = (int)(q2 - r * rowdw) * 32 + part * KP;
    if (whole_rows) {
        uint32_t *o = reinterpret_cast<uint32_t *>(ret + q2 * 32 + part * KP);
#pragma unroll
        for (int i = 0; i < KP; i += 2)
            o[i >> 1] = (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)sum[i]) |
                        ((uint32_t)__builtin_bit_cast(uint16_t, (_Float16)sum[i + 1]) << 16);
    } else {
#pragma unroll
        for (int i = 0; i < KP; i++)
            if (z0 + i < zbits) ret[r * zbits + z0 + i] = (_Float16)sum[i];
    }
}

template <typename W>
int weighted_sum_fast_impl(uint16_t *ret, const W *in, const uint16_t *w, int64_t n, int64_t R, int64_t Rw,
                           int64_t zbits, nb_stream_t stream, const char *who)
{
    NB_REQUIRE(n >= 0 && R >= 0 && Rw >= 0 && zbits >= 0, "%s: negative shape", who);
    if (R * zbits == 0) return NB_OK;
    NB_REQUIRE_PTR(ret);
    NB_REQUIRE_ALIGNED(ret, 2);
    if (n > 0) {
        NB_REQUIRE_PTR(in);
        NB_REQUIRE_PTR(w);
        NB_REQUIRE_ALIGNED(in, sizeof(W));
        NB_REQUIRE_ALIGNED(w, 2);
    }
    NB_REQUIRE(zbits <= (1 << 30) && Rw <= (1 << 30), "%s: row too long", who);
    NB_REQUIRE(zbits <= Rw * (int64_t)WordTraits<W>::bits, "%s: zbits exceeds the Rw words of a row", who);
    const int64_t rowdw = Rw * (int64_t)(sizeof(W) / 4), Q = R * rowdw;
    NB_REQUIRE(Q < (1LL << 25), "%s: more than 2^25 32-bit columns", who);
    const int64_t sets = ceil_div(Q, 64), nchunks = ceil_div(n, 64);
    // member shares per column set: as many as it takes to give the chip about 4096 waves, while every share has a chunk
    int split = 0;
    while (split < 4 && (sets << split) < 4096 && (2LL << split) <= nchunks) split++;
    if (const char *v = getenv("NESBIN_WSUM_SPLIT")) {
        const int f = atoi(v);
        if (f >= 0 && f <= 4) split = f;
    }
    const int whole = zbits == rowdw * 32 && aligned(ret, 16);
    const int64_t blocks = ceil_div(sets, 16 >> split);
    NB_REQUIRE(blocks <= kMaxGridX, "%s: output exceeds one launch", who);
    // small outputs: 32 columns per wave, the wave's halves on the two blocks of a chunk (twice the waves)
    bool halves = split == 4 && (sets << split) < 2048 && nchunks >= 1 && Q < (1LL << 23);
    if (const char *v = getenv("NESBIN_WSUM_HALVES")) halves = atoi(v) != 0 && split >= 3 && Q < (1LL << 23);
    static std::once_flag once;
    static hipError_t attr = hipSuccess;
    std::call_once(once, [] {
        const void *fns[7] = {reinterpret_cast<const void *>(weighted_sum_lut_kernel<0>),
                              reinterpret_cast<const void *>(weighted_sum_lut_kernel<1>),
                              reinterpret_cast<const void *>(weighted_sum_lut_kernel<2>),
                              reinterpret_cast<const void *>(weighted_sum_lut_kernel<3>),
                              reinterpret_cast<const void *>(weighted_sum_lut_kernel<4>),
                              reinterpret_cast<const void *>(weighted_sum_lut_half_kernel<3>),
                              reinterpret_cast<const void *>(weighted_sum_lut_half_kernel<4>)};
        for (const void *f : fns) {
            const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, kLutLdsBytes);
            if (e != hipSuccess) attr = e;
        }
    });
    if (attr != hipSuccess) {
        (void)hipGetLastError();
        return fail(NB_ERR_UNSUPPORTED, "%s: cannot raise the kernel's LDS limit: %s", who, hipGetErrorString(attr));
    }
    const int64_t nblocks = halves ? ceil_div(ceil_div(Q, 32), 16 >> split) : blocks;
    auto launch = [&](auto kern) {
        kern<<<dim3((unsigned)nblocks), dim3(1024), kLutLdsBytes, as_stream(stream)>>>(
            reinterpret_cast<_Float16 *>(ret), reinterpret_cast<const uint32_t *>(in),
            reinterpret_cast<const _Float16 *>(w), n, Q, (int)rowdw, (int)zbits, whole);
    };
    if (halves) {
        if (split == 3) launch(weighted_sum_lut_half_kernel<3>);
        else launch(weighted_sum_lut_half_kernel<4>);
        return check_launch(who);
    }
    switch (split) {
        case 0: launch(weighted_sum_lut_kernel<0>); break;
        case 1: launch(weighted_sum_lut_kernel<1>); break;
        case 2: launch(weighted_sum_lut_kernel<2>); break;
        case 3: launch(weighted_sum_lut_kernel<3>); break;
        default: launch(weighted_sum_lut_kernel<4>); break;
    }
    return check_launch(who);
}

}  // namespace nb

extern "C" {
int nb_weighted_sum_i64(uint16_t *ret, const int64_t *in, const uint16_t *w, int64_t n, int64_t R, int64_t Rw,
                        int64_t zbits, nb_stream_t s)
{
    return nb::weighted_sum_impl<uint64_t>(ret, reinterpret_cast<const uint64_t *>(in), w, n, R, Rw, zbits, s,
                                           "nb_weighted_sum_i64");
}
int nb_weighted_sum_i32(uint16_t *ret, const int32_t *in, const uint16_t *w, int64_t n, int64_t R, int64_t Rw,
                        int64_t zbits, nb_stream_t s)
{
    return nb::weighted_sum_impl<uint32_t>(ret, reinterpret_cast<const uint32_t *>(in), w, n, R, Rw, zbits, s,
                                           "nb_weighted_sum_i32");
}
int nb_weighted_sum_fast_i64(uint16_t *ret, const int64_t *in, const uint16_t *w, int64_t n, int64_t R, int64_t Rw,
                             int64_t zbits, nb_stream_t s)
{
    return nb::weighted_sum_fast_impl<uint64_t>(ret, reinterpret_cast<const uint64_t *>(in), w, n, R, Rw, zbits, s,
                                                "nb_weighted_sum_fast_i64");
}
int nb_weighted_sum_fast_i32(uint16_t *ret, const int32_t *in, const uint16_t *w, int64_t n, int64_t R, int64_t Rw,
                             int64_t zbits, nb_stream_t s)
{
    return nb::weighted_sum_fast_impl<uint32_t>(ret, reinterpret_cast<const uint32_t *>(in), w, n, R, Rw, zbits, s,
                                                "nb_weighted_sum_fast_i32");
}
}
