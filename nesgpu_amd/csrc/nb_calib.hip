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

// Streaming writes alone: every thread stores 16-byte chunks at wave-contiguous addresses.
__global__ __launch_bounds__(256) void calib_fill_kernel(uint4 *__restrict__ dst, int64_t n16, uint32_t v)
{
    const int64_t stride = (int64_t)gridDim.x * 256;
    const uint4 w = make_uint4(v, v + 1u, v + 2u, v + 3u);
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) dst[i] = w;
}

// The store pattern of the conv kernels' int32 maps without any arithmetic: members of [32 rows][32 pixels][64
// channels] int32 (256 KB each); a wave owns 16 pixel columns of a member and writes, row after row, its 4 KB of the
// row (four 16-byte stores per lane), 8 KB apart from row to row.
__global__ __launch_bounds__(256) void calib_store_rows_kernel(int *__restrict__ out, int units)
{
    const int u = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (u >= units) return;
    const int st = u & 1, z = u >> 1;
    uint4 *base = reinterpret_cast<uint4 *>(out + (int64_t)z * 65536);
    const uint4 v = make_uint4(1u, 2u, 3u, (uint32_t)lane);
    for (int y = 0; y < 32; y++) {
#pragma unroll
        for (int s = 0; s < 4; s++) base[((y * 32 + st * 16 + 4 * s + lane / 16) * 64 + 4 * (lane % 16)) / 4] = v;
    }
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

// The same read with the load the streaming kernels of the library use: non-temporal 16-byte loads, all of a
// thread's UNR requests issued before the first use, 1024-thread workgroups.
template <int UNR>
__global__ __launch_bounds__(1024) void calib_read_stream_kernel(uint32_t *__restrict__ sink, const uint4 *__restrict__ src,
                                                                 int64_t n16)
{
    const int64_t base = ((int64_t)blockIdx.x * 1024 * UNR) + threadIdx.x;
    uint4 v[UNR];
#pragma unroll
    for (int u = 0; u < UNR; u++) {
        const int64_t i = base + (int64_t)u * 1024;
        v[u] = load_stream16(src + (i < n16 ? i : n16 - 1));
    }
    __builtin_amdgcn_sched_barrier(0);
    uint32_t acc = 0;
#pragma unroll
    for (int u = 0; u < UNR; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    if (acc == 0x9E3779B9u) sink[0] = acc;
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

typedef int calib_v4i __attribute__((ext_vector_type(4)));

// How int8 MFMAs and ordinary vector instructions share a SIMD's issue.  Every iteration has eight
// v_mfma_i32_16x16x64_i8 on independent accumulators, each followed by V independent v_add_u32.
// SPLIT = false: every wave runs that mixed stream.  SPLIT = true: even waves of a workgroup issue only the MFMAs,
// odd waves only the adds (16*V per iteration... the same totals per SIMD pair), at wave priorities PM and PV.
template <int V, bool SPLIT, int PM, int PV>
__global__ __launch_bounds__(256) void calib_mfma_valu_kernel(int32_t *__restrict__ out, int iters)
{
    calib_v4i a = {(int)threadIdx.x, 1, 2, 3}, b = {5, 6, 7, (int)blockIdx.x};
    calib_v4i acc[8];
    int x[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        acc[i] = (calib_v4i){0, 0, 0, 0};
        x[i] = threadIdx.x + i;
    }
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar branches only: MFMA ignores EXEC
    const bool do_m = !SPLIT || (wv & 1) == 0, do_v = !SPLIT || (wv & 1) == 1;
    if (SPLIT) {
        if (do_m) {
            __builtin_amdgcn_s_setprio(PM);
        } else {
            __builtin_amdgcn_s_setprio(PV);
        }
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (do_m) asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a), "v"(b));
            if (do_v) {
#pragma unroll
                for (int j = 0; j < V; j++) asm volatile("v_add_u32 %0, %0, %1" : "+v"(x[(i + j) & 7]) : "v"(it));
            }
        }
    }
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15");  // the accumulators are read below without the compiler's hazard padding
    int t = 0;
#pragma unroll
    for (int i = 0; i < 8; i++) t += acc[i][0] + acc[i][3] + x[i];
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
int nb_calib_fill(void *dst, int64_t bytes, int blocks, nb_stream_t s)
{
    nb::calib_fill_kernel<<<dim3((unsigned)blocks), dim3(256), 0, nb::as_stream(s)>>>(static_cast<uint4 *>(dst),
                                                                                     bytes / 16, 7u);
    return nb::check_launch("nb_calib_fill");
}
// members x 256 KB written
int nb_calib_store_rows(void *dst, int members, nb_stream_t s)
{
    const int units = members * 2;
    nb::calib_store_rows_kernel<<<dim3((unsigned)((units + 3) / 4)), dim3(256), 0, nb::as_stream(s)>>>(
        static_cast<int *>(dst), units);
    return nb::check_launch("nb_calib_store_rows");
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
int nb_calib_read_stream(void *sink, const void *src, int64_t bytes, nb_stream_t s)
{
    const int64_t n16 = bytes / 16;
    constexpr int UNR = 8;
    const int64_t blocks = nb::ceil_div(n16, 1024 * UNR);
    nb::calib_read_stream_kernel<UNR><<<dim3((unsigned)blocks), dim3(1024), 0, nb::as_stream(s)>>>(
        static_cast<uint32_t *>(sink), static_cast<const uint4 *>(src), n16);
    return nb::check_launch("nb_calib_read_stream");
}
// lane-ops executed = blocks*256 * iters * 8*16 * 2 (one xor + one bcnt per pair)
int nb_calib_popc(void *out, const void *s1024, int blocks, int iters, nb_stream_t s)
{
    nb::calib_popc_kernel<<<dim3((unsigned)blocks), dim3(256), 0, nb::as_stream(s)>>>(
        static_cast<int32_t *>(out), static_cast<const uint32_t *>(s1024), iters);
    return nb::check_launch("nb_calib_popc");
}
// variant 0: MFMAs alone; 1: + 2 adds per MFMA in the same wave; 2: + 4 adds in the same wave; 3: MFMA waves and
// add waves (4 adds per MFMA) at equal priority; 4: the same with the MFMA waves at priority 3; 5: with the add waves
// at priority 3.  MFMAs executed per SIMD = blocks * 4 / 1024 * iters * 8 (half of that for variants 3-5).
int nb_calib_mfma_valu(void *out, int blocks, int iters, int variant, nb_stream_t s)
{
    int32_t *o = static_cast<int32_t *>(out);
    const dim3 g((unsigned)blocks), b(256);
    hipStream_t st = nb::as_stream(s);
    switch (variant) {
    case 0: nb::calib_mfma_valu_kernel<0, false, 0, 0><<<g, b, 0, st>>>(o, iters); break;
    case 1: nb::calib_mfma_valu_kernel<2, false, 0, 0><<<g, b, 0, st>>>(o, iters); break;
    case 2: nb::calib_mfma_valu_kernel<4, false, 0, 0><<<g, b, 0, st>>>(o, iters); break;
    case 3: nb::calib_mfma_valu_kernel<4, true, 0, 0><<<g, b, 0, st>>>(o, iters); break;
    case 4: nb::calib_mfma_valu_kernel<4, true, 3, 0><<<g, b, 0, st>>>(o, iters); break;
    case 5: nb::calib_mfma_valu_kernel<4, true, 0, 3><<<g, b, 0, st>>>(o, iters); break;
    default: return NB_ERR_SHAPE;
    }
    return nb::check_launch("nb_calib_mfma_valu");
}
}
