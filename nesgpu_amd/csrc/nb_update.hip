// The small steps around weighted_sum in a layer's update (modules/binary.py:67-77), one kernel each instead of
// three to four tensor expressions: the fitness vector centred in fp16, the l1 / l2 terms added to the gradient
// estimate, and the bias gradient fitness @ bias_noise; and set_noise's scaling of the uniform bias draw.
#include <algorithm>
#include "nb_common.hpp"
#include "nb_conv_common.hpp"

namespace nb {

// out[i] = fp16(x[i] - mean) with x = fp16(in) and mean = the mean of the x[i] rounded once to fp16
// (modules/binary.py:68-69: weights.type(float16), then weights - weights.mean()).  The sum of the x[i] is taken in
// double precision (exact for any fitness vector whose values span less than 53 bits), where torch's fp16 mean adds
// in fp32 in an order of its own and multiplies by a rounded 1/n: the two means agree unless the exact one lies
// within a few 1e-7 (relative) of the middle between two fp16 numbers.  One workgroup.
template <typename T>
__global__ __launch_bounds__(1024) void center_fitness_kernel(_Float16 *__restrict__ out, const T *__restrict__ in,
                                                              int64_t n)
{
    __shared__ double part[16];
    __shared__ float mean_sh;
    double s = 0.0;
    for (int64_t i = threadIdx.x; i < n; i += 1024) s += (double)(float)(_Float16)in[i];
#pragma unroll
    for (int o = 32; o; o >>= 1) s += __shfl_xor(s, o);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int k = 0; k < 16; k++) t += part[k];
        mean_sh = (float)double_round_once_fp16(t / (double)n);
    }
    __syncthreads();
    const float m = mean_sh;
    for (int64_t i = threadIdx.x; i < n; i += 1024) out[i] = (_Float16)((float)(_Float16)in[i] - m);
}

// grad += l1 * sign(w), then grad += l2 * w, each with the roundings of the fp16 tensor expressions of
// modules/binary.py:73-76: the product with the coefficient (a float) rounded to fp16, then the sum rounded to fp16;
// a coefficient of zero skips its step, as the `if` there does.  sign(NaN) = 0, like torch.sign.
__device__ __forceinline__ _Float16 grad_regularize_one(_Float16 g, _Float16 wv, float l1, float l2)
{
    const float x = (float)wv;
    if (l1 != 0.f) {
        const float sg = (float)((0.f < x) - (x < 0.f));
        g = (_Float16)((float)g + (float)(_Float16)(l1 * sg));
    }
    if (l2 != 0.f) g = (_Float16)((float)g + (float)(_Float16)(l2 * x));
    return g;
}

// VEC: eight elements (16 bytes) per thread and step; n8 = n / 8 groups, the tail one by one.
template <bool VEC>
__global__ __launch_bounds__(256) void grad_regularize_kernel(_Float16 *__restrict__ grad, const _Float16 *__restrict__ w,
                                                              float l1, float l2, int64_t n)
{
    const int64_t n8 = VEC ? n >> 3 : 0;
    if (VEC) {
        uint4 *g8 = reinterpret_cast<uint4 *>(grad);
        const uint4 *w8 = reinterpret_cast<const uint4 *>(w);
        for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n8; i += (int64_t)gridDim.x * 256) {
            const uint4 gv = g8[i], wv = w8[i];
            const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, ww[4] = {wv.x, wv.y, wv.z, wv.w};
            uint32_t r[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const _Float16 lo = grad_regularize_one(__builtin_bit_cast(_Float16, (uint16_t)(gw[e] & 0xFFFFu)),
                                                        __builtin_bit_cast(_Float16, (uint16_t)(ww[e] & 0xFFFFu)), l1, l2);
                const _Float16 hi = grad_regularize_one(__builtin_bit_cast(_Float16, (uint16_t)(gw[e] >> 16)),
                                                        __builtin_bit_cast(_Float16, (uint16_t)(ww[e] >> 16)), l1, l2);
                r[e] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
            }
            g8[i] = make_uint4(r[0], r[1], r[2], r[3]);
        }
    }
    for (int64_t i = 8 * n8 + (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        grad[i] = grad_regularize_one(grad[i], w[i], l1, l2);
}

// x = (x - 0.5) * 6 with the roundings of the fp16 tensor expression of modules/binary.py:63-64 (the uniform draw itself
// stays torch.rand on the device's global generator, as in the reference): fp16(fp16(x - 0.5) * 6), in place.
__global__ __launch_bounds__(256) void bias_noise_scale_kernel(_Float16 *__restrict__ x, int64_t n)
{
    NB_FLAT_LOOP(i, n)
    {
        if (i >= n) continue;
        const _Float16 c = (_Float16)((float)x[i] - 0.5f);
        x[i] = (_Float16)((float)c * 6.0f);
    }
}

// out[o] = fp16(sum_d c[d] * noise[d, o]), fp32 accumulation (modules/binary.py:77: weights @ bias_noise).  A workgroup
// takes 8 outputs (16 contiguous bytes per member: one load where the row length allows it); thread t takes the
// members t, t + 1024, ... with a fused multiply-add per output, and the 1024 partial sums of an output are added
// in a fixed order (butterflies inside a wave, then the 16 waves in turn): the same bits on every run, not the order
// of a library GEMV.  Every thread has all its loads in flight at once.
template <bool VEC>
__global__ __launch_bounds__(1024) void bias_grad_kernel(_Float16 *__restrict__ out, const _Float16 *__restrict__ c,
                                                         const _Float16 *__restrict__ noise, int64_t n, int64_t O)
{
    __shared__ float part[16][8];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int64_t o0 = (int64_t)blockIdx.x * 8;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.f;
#pragma unroll 4
    for (int64_t d = threadIdx.x; d < n; d += 1024) {
        const float cd = (float)c[d];
        if (VEC) {
            const uint4 v = *reinterpret_cast<const uint4 *>(noise + d * O + o0);
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                acc[2 * e] = fmaf(cd, (float)__builtin_bit_cast(_Float16, (uint16_t)(w[e] & 0xFFFFu)), acc[2 * e]);
                acc[2 * e + 1] = fmaf(cd, (float)__builtin_bit_cast(_Float16, (uint16_t)(w[e] >> 16)), acc[2 * e + 1]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++)
                if (o0 + e < O) acc[e] = fmaf(cd, (float)noise[d * O + o0 + e], acc[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; e++) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) acc[e] += __shfl_xor(acc[e], o);
        if (lane == 0) part[wv][e] = acc[e];
    }
    __syncthreads();
    if (threadIdx.x < 8 && o0 + threadIdx.x < O) {
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < 16; k++) t += part[k][threadIdx.x];
        out[o0 + threadIdx.x] = (_Float16)t;
    }
}

template <typename T>
static int center_fitness_impl(uint16_t *out, const T *in, int64_t n, nb_stream_t stream, const char *who)
{
    NB_REQUIRE(n >= 0, "%s: negative length", who);
    if (n == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(in);
    NB_REQUIRE_ALIGNED(out, 2);
    NB_REQUIRE_ALIGNED(in, sizeof(T));
    center_fitness_kernel<<<dim3(1), dim3(1024), 0, as_stream(stream)>>>(reinterpret_cast<_Float16 *>(out), in, n);
    return check_launch(who);
}

}  // namespace nb

extern "C" {
int nb_center_fitness_f16(uint16_t *out, const uint16_t *in, int64_t n, nb_stream_t stream)
{
    return nb::center_fitness_impl(out, reinterpret_cast<const _Float16 *>(in), n, stream, "nb_center_fitness_f16");
}
int nb_center_fitness_f32(uint16_t *out, const float *in, int64_t n, nb_stream_t stream)
{
    return nb::center_fitness_impl(out, in, n, stream, "nb_center_fitness_f32");
}

int nb_grad_regularize(uint16_t *grad, const uint16_t *weight, float l1, float l2, int64_t n, nb_stream_t stream)
{
    NB_REQUIRE(n >= 0, "nb_grad_regularize: negative length");
    if (n == 0 || (l1 == 0.f && l2 == 0.f)) return NB_OK;
    NB_REQUIRE_PTR(grad);
    NB_REQUIRE_PTR(weight);
    NB_REQUIRE_ALIGNED(grad, 2);
    NB_REQUIRE_ALIGNED(weight, 2);
    const bool vec = nb::aligned(grad, 16) && nb::aligned(weight, 16) && n >= 8;
    const unsigned blocks = (unsigned)std::min<int64_t>(nb::ceil_div(vec ? n / 8 + 7 : n, 256), 8192);
    if (vec)
        nb::grad_regularize_kernel<true><<<dim3(blocks), dim3(256), 0, nb::as_stream(stream)>>>(
            reinterpret_cast<_Float16 *>(grad), reinterpret_cast<const _Float16 *>(weight), l1, l2, n);
    else
        nb::grad_regularize_kernel<false><<<dim3(blocks), dim3(256), 0, nb::as_stream(stream)>>>(
            reinterpret_cast<_Float16 *>(grad), reinterpret_cast<const _Float16 *>(weight), l1, l2, n);
    return nb::check_launch("nb_grad_regularize");
}

int nb_bias_noise_scale(uint16_t *x, int64_t n, nb_stream_t stream)
{
    NB_REQUIRE(n >= 0, "nb_bias_noise_scale: negative length");
    if (n == 0) return NB_OK;
    NB_REQUIRE_PTR(x);
    NB_REQUIRE_ALIGNED(x, 2);
    nb::bias_noise_scale_kernel<<<dim3(nb::grid_for(n)), dim3(256), 0, nb::as_stream(stream)>>>(
        reinterpret_cast<_Float16 *>(x), n);
    return nb::check_launch("nb_bias_noise_scale");
}

int nb_bias_grad(uint16_t *out, const uint16_t *centered, const uint16_t *bias_noise, int64_t n, int64_t O,
                 nb_stream_t stream)
{
    NB_REQUIRE(n >= 0 && O >= 0, "nb_bias_grad: negative shape");
    if (O == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_ALIGNED(out, 2);
    if (n > 0) {
        NB_REQUIRE_PTR(centered);
        NB_REQUIRE_PTR(bias_noise);
        NB_REQUIRE_ALIGNED(centered, 2);
        NB_REQUIRE_ALIGNED(bias_noise, 2);
    }
    const int64_t blocks = nb::ceil_div(O, 8);
    NB_REQUIRE(blocks <= nb::kMaxGridX, "nb_bias_grad: too many outputs for one launch");
    if (O % 8 == 0 && nb::aligned(bias_noise, 16))
        nb::bias_grad_kernel<true><<<dim3((unsigned)blocks), dim3(1024), 0, nb::as_stream(stream)>>>(
            reinterpret_cast<_Float16 *>(out), reinterpret_cast<const _Float16 *>(centered),
            reinterpret_cast<const _Float16 *>(bias_noise), n, O);
    else
        nb::bias_grad_kernel<false><<<dim3((unsigned)blocks), dim3(1024), 0, nb::as_stream(stream)>>>(
            reinterpret_cast<_Float16 *>(out), reinterpret_cast<const _Float16 *>(centered),
            reinterpret_cast<const _Float16 *>(bias_noise), n, O);
    return nb::check_launch("nb_bias_grad");
}
}
