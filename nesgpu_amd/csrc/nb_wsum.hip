// weighted_sum: ret[r,z] = fp16( sum_m float(w[m]) * bit(in[m,r,z/bits], z%bits) ), the reduction over
// the population that the update step applies to the sampled masks
// (extensions/src/weighted_sum.cu:28-46).  fp32 accumulation in member order, like the reference.
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
}
