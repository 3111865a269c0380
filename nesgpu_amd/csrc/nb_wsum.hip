// weighted_sum: ret[r,z] = fp16( sum_m float(w[m]) * bit(in[m,r,z/bits], z%bits) ), the reduction over
// the population that the update step applies to the sampled masks
// (extensions/src/weighted_sum.cu:28-46).  fp32 accumulation in member order, like the reference.
#include "nb_common.hpp"

namespace nb {

// One wave per (row, 64-bit column): lane z owns output bit z of the column and adds the members' weights in member
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
    __shared__ float wsh[64];
    const int lane = threadIdx.x & 63;
    const int64_t cid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // (row, column); past the end: idle but in step
    const bool live = cid < R * ncol;
    const int64_t r = live ? cid / ncol : 0;
    const int c = live ? (int)(cid - r * ncol) : 0;
    const int64_t stride = R * (int64_t)Rw;
    const W *p = in + r * Rw + (int64_t)c * wpc;
    const bool has_hi = wpc == 1 || c * wpc + 1 < Rw;
    float acc = 0.f;
    for (int64_t m0 = 0; m0 < n; m0 += 64) {
        __syncthreads();
        if (threadIdx.x < 64) wsh[threadIdx.x] = m0 + threadIdx.x < n ? (float)w[m0 + threadIdx.x] : 0.f;
        __syncthreads();
        uint32_t vlo = 0, vhi = 0;  // members past n contribute the zero word: nothing is added for them
        if (live && m0 + lane < n) {
            if (wpc == 1) {
                const uint64_t v = (uint64_t)p[(m0 + lane) * stride];
                vlo = (uint32_t)v;
                vhi = (uint32_t)(v >> 32);
            } else {
                vlo = (uint32_t)p[(m0 + lane) * stride];
                vhi = has_hi ? (uint32_t)p[(m0 + lane) * stride + 1] : 0u;
            }
        }
#pragma unroll 8
        for (int j = 0; j < 64; j++) {
            const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)vlo, j);
            const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)vhi, j);
            const uint64_t mask = ((uint64_t)hi << 32) | lo;
            const float wm = wsh[j];
            float t;
            asm("v_cndmask_b32_e64 %0, 0, %1, %2" : "=v"(t) : "v"(wm), "s"(mask));  // t = bit z of the word ? wm : 0
            acc += t;  // adding zero for a clear bit leaves the running sum unchanged
        }
    }
    const int z = c * 64 + lane;
    if (live && z < zbits) ret[r * zbits + z] = (_Float16)acc;
}

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
