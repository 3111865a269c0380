// Calibration kernels for the benchmark (built into libnesbin_calib.so, not part of the product ABI):
// a plain streaming copy, a streaming read and an XOR+popcount register loop.  They give the measured
// ceilings that the datasheet roofline numbers are reported beside.
#include "nb_common.hpp"

namespace nb {

__global__ __launch_bounds__(256) void calib_copy_kernel(uint4 *__restrict__ dst, const uint4 *__restrict__ src,
                                                         int64_t n16)
{
    const int64_t stride = (int64_t)gridDim.x * 256;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// Each thread owns UNR consecutive 16-byte chunks at wave-contiguous addresses.
template <int UNR>
__global__ __launch_bounds__(256) void calib_read_kernel(uint32_t *__restrict__ sink, const uint4 *__restrict__ src,
                                                         int64_t n16)
{
    const int64_t base = ((int64_t)blockIdx.x * 256 * UNR) + threadIdx.x;
    uint32_t acc = 0;
#pragma unroll
    for (int u = 0; u < UNR; u++) {
        const int64_t i = base + (int64_t)u * 256;
        if (i < n16) {
            const uint4 v = src[i];
            acc ^= v.x ^ v.y ^ v.z ^ v.w;
        }
    }
    if (acc == 0x9E3779B9u) sink[0] = acc;  // practically never; keeps the loads alive
}

// iters x 16 independent (v_xor_b32 with an SGPR operand, accumulating v_bcnt_u32_b32) pairs per lane.
__global__ __launch_bounds__(256) void calib_popc_kernel(int32_t *__restrict__ out, const uint32_t *__restrict__ s,
                                                         int iters)
{
    uint32_t a[8];
#pragma unroll
    for (int i = 0; i < 8; i++) a[i] = threadIdx.x * 2654435761u + i * 40503u + blockIdx.x;
    int acc[16];
#pragma unroll
    for (int j = 0; j < 16; j++) acc[j] = 0;
    for (int it = 0; it < iters; it++) {
        const uint32_t *__restrict__ row = s + (it & 63) * 16;  // wave-uniform -> scalar loads
#pragma unroll
        for (int i = 0; i < 8; i++) {
#pragma unroll
            for (int j = 0; j < 16; j++) acc[j] += __popc(a[i] ^ row[j]);
        }
    }
    int t = 0;
#pragma unroll
    for (int j = 0; j < 16; j++) t += acc[j];
    out[(int64_t)blockIdx.x * 256 + threadIdx.x] = t;
}

}  // namespace nb

extern "C" {
int nb_calib_copy(void *dst, const void *src, int64_t bytes, int blocks, nb_stream_t s)
{
    nb::calib_copy_kernel<<<dim3((unsigned)blocks), dim3(256), 0, nb::as_stream(s)>>>(
        static_cast<uint4 *>(dst), static_cast<const uint4 *>(src), bytes / 16);
    return nb::check_launch("nb_calib_copy");
}
int nb_calib_read(void *sink, const void *src, int64_t bytes, nb_stream_t s)
{
    const int64_t n16 = bytes / 16;
    constexpr int UNR = 8;
    const int64_t blocks = nb::ceil_div(n16, 256 * UNR);
    nb::calib_read_kernel<UNR><<<dim3((unsigned)blocks), dim3(256), 0, nb::as_stream(s)>>>(
        static_cast<uint32_t *>(sink), static_cast<const uint4 *>(src), n16);
    return nb::check_launch("nb_calib_read");
}
// lane-ops executed = blocks*256 * iters * 8*16 * 2 (one xor + one bcnt per pair)
int nb_calib_popc(void *out, const void *s1024, int blocks, int iters, nb_stream_t s)
{
    nb::calib_popc_kernel<<<dim3((unsigned)blocks), dim3(256), 0, nb::as_stream(s)>>>(
        static_cast<int32_t *>(out), static_cast<const uint32_t *>(s1024), iters);
    return nb::check_launch("nb_calib_popc");
}
}
