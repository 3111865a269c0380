// pack / unpack / int8pack: HBM-bound layout conversions between bool bytes and packed words.
#include "nb_common.hpp"

namespace nb {

// 4 bool bytes of a dword -> 4 bits.  Any non-zero byte counts as 1.
__device__ __forceinline__ uint32_t nibble_of_bools(uint32_t v)
{
    // high bit of every byte := byte != 0
    const uint32_t nz = (((v & 0x7F7F7F7Fu) + 0x7F7F7F7Fu) | v) & 0x80808080u;
    const uint32_t t = nz >> 7;                 // b0@0 b1@8 b2@16 b3@24
    const uint32_t y = (t << 7) | t;            // b0@7 b1@8 ...
    const uint32_t z = (y << 14) | y;           // b0@21 b1@22 b2@23 b3@24
    return (z >> 21) & 0xFu;
}

__device__ __forceinline__ uint32_t bits16_of_bools(uint4 v)
{
    return nibble_of_bools(v.x) | (nibble_of_bools(v.y) << 4) | (nibble_of_bools(v.z) << 8) |
           (nibble_of_bools(v.w) << 12);
}

// One thread per output word, 16-byte loads.  Requires C % 16 == 0 and a 16-byte aligned input,
// so every 16-byte chunk lies inside one row.
template <typename W>
__global__ __launch_bounds__(256) void pack_vec16_kernel(W *__restrict__ out, const uint8_t *__restrict__ in,
                                                         int64_t total_words, int Rw, int64_t C)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_FLAT_LOOP(t, total_words)
    {
        if (t >= total_words) continue;
        const int64_t row = t / Rw;
        const int y = (int)(t - row * Rw);
        const int64_t col0 = (int64_t)y * bits;
        const uint4 *src = reinterpret_cast<const uint4 *>(in + row * C + col0);
        int64_t left = C - col0;
        const int chunks = (int)((left < bits ? left : bits) >> 4);
        // all loads first and none behind a branch (a chunk past the row re-reads the first one and is dropped):
        // a load behind a branch waits for the one before it
        const int cmax = (int)((C < bits ? C : bits) >> 4);  // the same for every thread
        uint4 v[bits / 16];
#pragma unroll
        for (int c = 0; c < bits / 16; c++)
            v[c] = c < cmax ? load_stream16(reinterpret_cast<const uint8_t *>(src + (c < chunks ? c : 0))) : make_uint4(0, 0, 0, 0);
        W w = 0;
#pragma unroll
        for (int c = 0; c < bits / 16; c++) w |= (W)(c < chunks ? bits16_of_bools(v[c]) : 0u) << (16 * c);
        __builtin_nontemporal_store(w, out + t);
    }
}

// Rows of exactly 16 bools (one 16-byte chunk per row, one word per row): a workgroup takes 1024 consecutive rows,
// thread i the rows i, i + 256, i + 512, i + 768: every load instruction of a wave reads 1 KiB in one piece, all four
// of a thread are in flight before the first is used, and the words leave as runs of 64.
template <typename W>
__global__ __launch_bounds__(256) void pack_rows16_kernel(W *__restrict__ out, const uint8_t *__restrict__ in, int64_t rows)
{
    const int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x;
    uint4 v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int64_t r = base + 256 * j;
        v[j] = load_stream16(in + (r < rows ? r : rows - 1) * 16);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int64_t r = base + 256 * j;
        if (r < rows) __builtin_nontemporal_store((W)bits16_of_bools(v[j]), out + r);
    }
}

// One thread per output word, 8-byte loads.  Requires C % 8 == 0 and an 8-byte aligned input, so every 8-byte chunk
// lies inside one row (rows of 24 or 40 bools: 3 x 8 bit planes of an image, say).
template <typename W>
__global__ __launch_bounds__(256) void pack_vec8_kernel(W *__restrict__ out, const uint8_t *__restrict__ in,
                                                        int64_t total_words, int Rw, int64_t C)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_FLAT_LOOP(t, total_words)
    {
        if (t >= total_words) continue;
        const int64_t row = t / Rw;
        const int y = (int)(t - row * Rw);
        const int64_t col0 = (int64_t)y * bits;
        const uint2 *src = reinterpret_cast<const uint2 *>(in + row * C + col0);
        const int64_t left = C - col0;
        const int chunks = (int)((left < bits ? left : bits) >> 3);
        // all loads first and none behind a branch (a chunk past the row re-reads the first one and is dropped)
        const int cmax = (int)((C < bits ? C : bits) >> 3);  // the same for every thread
        uint2 v[bits / 8];
#pragma unroll
        for (int c = 0; c < bits / 8; c++) v[c] = c < cmax ? src[c < chunks ? c : 0] : make_uint2(0u, 0u);
        W w = 0;
#pragma unroll
        for (int c = 0; c < bits / 8; c++)
            w |= (W)(c < chunks ? nibble_of_bools(v[c].x) | (nibble_of_bools(v[c].y) << 4) : 0u) << (8 * c);
        __builtin_nontemporal_store(w, out + t);
    }
}

// 64-bit words, C % 64 == 0, 16-byte aligned input: a wave converts 4 KiB of bools (64 words) per step.
// Load i (0..3) takes the 1 KiB slice i with lanes at consecutive 16-byte chunks (fully coalesced); the four
// lanes of a quad then hold the four 16-bit quarters of word i*16 + lane/4 and OR them together, and lane
// 4q+i stores word i*16+q, so one store instruction writes the 64 finished words.
__global__ __launch_bounds__(256) void pack_quad_kernel(uint64_t *__restrict__ out, const uint8_t *__restrict__ in,
                                                        int64_t total_words)
{
    const int lane = threadIdx.x & 63;
    const int64_t nwaves = (int64_t)gridDim.x * 4;
    for (int64_t w0 = ((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) * 64; w0 < total_words; w0 += nwaves * 64) {
        const uint8_t *src = in + w0 * 64;
        const int64_t left = total_words - w0;  // words left from w0 (>= 1)
        uint4 v[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int64_t word = i * 16 + (lane >> 2);
            if (word >= left) word = left - 1;  // clamp: tail lanes re-read a valid word and do not store
            v[i] = load_stream16(src + word * 64 + (lane & 3) * 16);
        }
        __builtin_amdgcn_sched_barrier(0);
        uint64_t mine = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint64_t q = (uint64_t)bits16_of_bools(v[i]) << (16 * (lane & 3));
            q = or_reduce_group<4>(q);
            if ((lane & 3) == i) mine = q;
        }
        const int64_t word = (lane & 3) * 16 + (lane >> 2);
        if (word < left) __builtin_nontemporal_store(mine, out + w0 + word);
    }
}

// Generic: one thread per output word, byte loads, any C.
template <typename W>
__global__ __launch_bounds__(256) void pack_generic_kernel(W *__restrict__ out, const uint8_t *__restrict__ in,
                                                           int64_t total_words, int Rw, int64_t C)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_FLAT_LOOP(t, total_words)
    {
        if (t >= total_words) continue;
        const int64_t row = t / Rw;
        const int y = (int)(t - row * Rw);
        const int64_t col0 = (int64_t)y * bits;
        const uint8_t *src = in + row * C + col0;
        int64_t left = C - col0;
        const int nb_ = (int)(left < bits ? left : bits);
        W w = 0;
        for (int i = 0; i < nb_; i++) w |= (W)(src[i] != 0) << i;
        out[t] = w;
    }
}

// One thread per 16 output bytes (16 bits of a word).
template <typename W>
__global__ __launch_bounds__(256) void unpack_kernel(uint8_t *__restrict__ out, const W *__restrict__ in,
                                                     int64_t total_chunks)
{
    constexpr int bits = WordTraits<W>::bits;
    constexpr int per = bits / 16;
    NB_FLAT_LOOP(t, total_chunks)
    {
        if (t >= total_chunks) continue;
        const W w = in[t / per];
        const uint32_t h = (uint32_t)(w >> (16 * (int)(t % per))) & 0xFFFFu;
        uint32_t d[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t nib = (h >> (4 * q)) & 0xFu;
            d[q] = (nib * 0x00204081u) & 0x01010101u;   // bit j -> byte j
        }
        u32x4_t dv = {d[0], d[1], d[2], d[3]};
        __builtin_nontemporal_store(dv, reinterpret_cast<u32x4_t *>(out) + t);  // written once, read by another kernel
    }
}

template <typename W>
__global__ __launch_bounds__(256) void int8pack_kernel(W *__restrict__ out, const uint8_t *__restrict__ in,
                                                       int64_t total_words, int Rw, int64_t C)
{
    constexpr int per = WordTraits<W>::bits / 8;
    NB_FLAT_LOOP(t, total_words)
    {
        if (t >= total_words) continue;
        const int64_t row = t / Rw;
        const int y = (int)(t - row * Rw);
        const int64_t col0 = (int64_t)y * per;
        const uint8_t *src = in + row * C + col0;
        int64_t left = C - col0;
        const int nb_ = (int)(left < per ? left : per);
        W w = 0;
        for (int i = 0; i < nb_; i++) w |= (W)src[i] << (8 * i);
        out[t] = w;
    }
}

template <typename W>
int pack_impl(W *out, const uint8_t *in, int64_t R, int64_t C, nb_stream_t stream, const char *who)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_REQUIRE(R >= 0 && C >= 0, "%s: negative shape R=%lld C=%lld", who, (long long)R, (long long)C);
    const int64_t Rw = ceil_div(C, bits);
    const int64_t total = R * Rw;
    if (total == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(in);
    NB_REQUIRE_ALIGNED(out, sizeof(W));
    NB_REQUIRE(Rw <= 2147483647LL, "%s: row of %lld words is too long", who, (long long)Rw);
    const unsigned blocks = grid_for(total);
    if (bits == 64 && (C & 63) == 0 && aligned(in, 16)) {
        const unsigned qb = grid_for(ceil_div(total, 64) * 64);  // one wave per 64 words
        pack_quad_kernel<<<dim3(qb), dim3(256), 0, as_stream(stream)>>>(reinterpret_cast<uint64_t *>(out), in, total);
    } else if (C == 16 && aligned(in, 16) && ceil_div(R, 1024) <= kMaxGridX)
        pack_rows16_kernel<W><<<dim3((unsigned)ceil_div(R, 1024)), dim3(256), 0, as_stream(stream)>>>(out, in, R);
    else if ((C & 15) == 0 && aligned(in, 16))
        pack_vec16_kernel<W><<<dim3(blocks), dim3(256), 0, as_stream(stream)>>>(out, in, total, (int)Rw, C);
    else if ((C & 7) == 0 && aligned(in, 8))
        pack_vec8_kernel<W><<<dim3(blocks), dim3(256), 0, as_stream(stream)>>>(out, in, total, (int)Rw, C);
    else
        pack_generic_kernel<W><<<dim3(blocks), dim3(256), 0, as_stream(stream)>>>(out, in, total, (int)Rw, C);
    return check_launch(who);
}

template <typename W>
int unpack_impl(uint8_t *out, const W *in, int64_t R, int64_t Rw, nb_stream_t stream, const char *who)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_REQUIRE(R >= 0 && Rw >= 0, "%s: negative shape R=%lld Rw=%lld", who, (long long)R, (long long)Rw);
    const int64_t chunks = R * Rw * (bits / 16);
    if (chunks == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(in);
    NB_REQUIRE_ALIGNED(in, sizeof(W));
    NB_REQUIRE_ALIGNED(out, 16);
    const unsigned blocks = grid_for(chunks);
    unpack_kernel<W><<<dim3(blocks), dim3(256), 0, as_stream(stream)>>>(out, in, chunks);
    return check_launch(who);
}

template <typename W>
int int8pack_impl(W *out, const uint8_t *in, int64_t R, int64_t C, nb_stream_t stream, const char *who)
{
    constexpr int per = WordTraits<W>::bits / 8;
    NB_REQUIRE(R >= 0 && C >= 0, "%s: negative shape R=%lld C=%lld", who, (long long)R, (long long)C);
    const int64_t Rw = ceil_div(C, per);
    const int64_t total = R * Rw;
    if (total == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(in);
    NB_REQUIRE_ALIGNED(out, sizeof(W));
    NB_REQUIRE(Rw <= 2147483647LL, "%s: row of %lld words is too long", who, (long long)Rw);
    const unsigned blocks = grid_for(total);
    int8pack_kernel<W><<<dim3(blocks), dim3(256), 0, as_stream(stream)>>>(out, in, total, (int)Rw, C);
    return check_launch(who);
}

}  // namespace nb

extern "C" {
int nb_pack_i64(int64_t *out, const uint8_t *in, int64_t R, int64_t C, nb_stream_t s)
{
    return nb::pack_impl<uint64_t>(reinterpret_cast<uint64_t *>(out), in, R, C, s, "nb_pack_i64");
}
int nb_pack_i32(int32_t *out, const uint8_t *in, int64_t R, int64_t C, nb_stream_t s)
{
    return nb::pack_impl<uint32_t>(reinterpret_cast<uint32_t *>(out), in, R, C, s, "nb_pack_i32");
}
int nb_unpack_i64(uint8_t *out, const int64_t *in, int64_t R, int64_t Rw, nb_stream_t s)
{
    return nb::unpack_impl<uint64_t>(out, reinterpret_cast<const uint64_t *>(in), R, Rw, s, "nb_unpack_i64");
}
int nb_unpack_i32(uint8_t *out, const int32_t *in, int64_t R, int64_t Rw, nb_stream_t s)
{
    return nb::unpack_impl<uint32_t>(out, reinterpret_cast<const uint32_t *>(in), R, Rw, s, "nb_unpack_i32");
}
int nb_int8pack_i64(int64_t *out, const uint8_t *in, int64_t R, int64_t C, nb_stream_t s)
{
    return nb::int8pack_impl<uint64_t>(reinterpret_cast<uint64_t *>(out), in, R, C, s, "nb_int8pack_i64");
}
int nb_int8pack_i32(int32_t *out, const uint8_t *in, int64_t R, int64_t C, nb_stream_t s)
{
    return nb::int8pack_impl<uint32_t>(reinterpret_cast<uint32_t *>(out), in, R, C, s, "nb_int8pack_i32");
}
}
