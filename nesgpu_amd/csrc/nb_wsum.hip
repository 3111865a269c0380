// weighted_sum: ret[r,z] = fp16( sum_m float(w[m]) * bit(in[m,r,z/bits], z%bits) ), the reduction over
// the population that the update step applies to the sampled masks
// (extensions/src/weighted_sum.cu:28-46).  fp32 accumulation in member order, like the reference.
#include "nb_common.hpp"

namespace nb {

// One lane per output column z; the 64 lanes of a wave cover one 64-bit word (or two 32-bit
// words) of the row, so each mask word is fetched once per wave and broadcast.
template <typename W>
__global__ __launch_bounds__(256) void weighted_sum_kernel(_Float16 *__restrict__ ret, const W *__restrict__ in,
                                                           const _Float16 *__restrict__ w, int64_t n, int64_t R,
                                                           int Rw, int zbits, int zblocks)
{
    constexpr int bits = WordTraits<W>::bits;
    constexpr int lb = WordTraits<W>::log2bits;
    const int64_t r = blockIdx.x / zblocks;
    const int z = (int)(blockIdx.x - r * zblocks) * 256 + threadIdx.x;
    if (z >= zbits) return;
    const int ze = z >> lb, zb = z & (bits - 1);
    float acc = 0.f;
    if (ze < Rw) {
        const W *p = in + r * Rw + ze;
        const int64_t stride = R * (int64_t)Rw;
        for (int64_t m = 0; m < n; m++) {
            const float wm = (float)w[m];
            if ((p[m * stride] >> zb) & 1) acc += wm;
        }
    }
    ret[r * zbits + z] = (_Float16)acc;
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
    const int64_t zblocks = ceil_div(zbits, 256);
    NB_REQUIRE(R * zblocks <= kMaxGridX, "%s: output exceeds one launch", who);
    weighted_sum_kernel<W><<<dim3((unsigned)(R * zblocks)), dim3(256), 0, as_stream(stream)>>>(
        reinterpret_cast<_Float16 *>(ret), in, reinterpret_cast<const _Float16 *>(w), n, R, (int)Rw, (int)zbits,
        (int)zblocks);
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
