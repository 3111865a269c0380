// Shared definitions for the gfx950 kernels of libnesbin.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/nesbin.h"

namespace nb {

constexpr int kWave = 64;  // CDNA4 wavefront width

template <typename W>
struct WordTraits;
template <>
struct WordTraits<uint64_t> {
    static constexpr int bits = 64;
    static constexpr int log2bits = 6;
};
template <>
struct WordTraits<uint32_t> {
    static constexpr int bits = 32;
    static constexpr int log2bits = 5;
};

// XOR + popcount of one packed word.  A 64-bit word compiles to two v_xor_b32 and two
// v_bcnt_u32_b32; the add into `acc` folds into v_bcnt's accumulate operand.
__device__ __forceinline__ int popc_xor(uint64_t a, uint64_t b) { return __popcll(a ^ b); }
__device__ __forceinline__ int popc_xor(uint32_t a, uint32_t b) { return __popc(a ^ b); }

// acc += popcount(a ^ b).  The v_bcnt_u32_b32 is emitted by hand so that its third operand carries the
// running sum: per 32-bit half exactly one v_xor_b32 and one v_bcnt_u32_b32, no separate add (the
// compiler otherwise rewrites the sum of two popcounts and the accumulator into bcnt,bcnt,v_add3).
__device__ __forceinline__ int bcnt_acc(uint32_t x, int acc)
{
    int r;
    asm("v_bcnt_u32_b32 %0, %1, %2" : "=v"(r) : "v"(x), "v"(acc));
    return r;
}
__device__ __forceinline__ void acc_popc_xor(int &acc, uint64_t a, uint64_t b)
{
    acc = bcnt_acc((uint32_t)a ^ (uint32_t)b, acc);
    acc = bcnt_acc((uint32_t)(a >> 32) ^ (uint32_t)(b >> 32), acc);
}
__device__ __forceinline__ void acc_popc_xor(int &acc, uint32_t a, uint32_t b) { acc = bcnt_acc(a ^ b, acc); }

// Streaming (read-once) loads: the non-temporal hint keeps a multi-GiB stream from displacing the small
// reused operands in L2 and measurably raises achieved HBM bandwidth on MI355X.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint64_t u64x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 load_stream16(const void *p)
{
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint32_t load_stream4(const uint32_t *p) { return __builtin_nontemporal_load(p); }

// OR-reduction over aligned groups of G lanes (G = 4, 8 or 16) with DPP lane permutes instead of
// LDS-crossbar shuffles: xor-1 and xor-2 inside a quad, then the mirrored half-row and row.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_mov(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}
template <int G>
__device__ __forceinline__ uint32_t or_reduce_group(uint32_t v)
{
    static_assert(G == 4 || G == 8 || G == 16, "group must be 4, 8 or 16 lanes");
    v |= dpp_mov<0xB1>(v);               // quad_perm [1,0,3,2]
    v |= dpp_mov<0x4E>(v);               // quad_perm [2,3,0,1]
    if (G >= 8) v |= dpp_mov<0x141>(v);  // row_half_mirror: lane i <-> 7-i within 8
    if (G >= 16) v |= dpp_mov<0x140>(v); // row_mirror: lane i <-> 15-i within 16
    return v;
}
template <int G>
__device__ __forceinline__ uint64_t or_reduce_group(uint64_t v)
{
    const uint32_t lo = or_reduce_group<G>((uint32_t)v), hi = or_reduce_group<G>((uint32_t)(v >> 32));
    return ((uint64_t)hi << 32) | lo;
}

// Philox4x32-10 (Salmon et al., SC'11): counter-based generator used when the caller does not
// supply the random words.
__device__ __forceinline__ uint4 philox4x32_10(uint4 c, uint2 k)
{
#pragma unroll
    for (int r = 0; r < 10; r++) {
        // full 64-bit products: one v_mad_u64_u32 each instead of a v_mul_lo / v_mul_hi pair (the generator is bound
        // by the number of vector instructions per word)
        const uint64_t p0 = (uint64_t)0xD2511F53u * c.x, p1 = (uint64_t)0xCD9E8D57u * c.z;
        const uint32_t lo0 = (uint32_t)p0, hi0 = (uint32_t)(p0 >> 32);
        const uint32_t lo1 = (uint32_t)p1, hi1 = (uint32_t)(p1 >> 32);
        // three-input XOR in one instruction (v_bitop3_b32, truth table 0x96)
        c = make_uint4(__builtin_amdgcn_bitop3_b32(hi1, c.y, k.x, 0x96), lo1, __builtin_amdgcn_bitop3_b32(hi0, c.w, k.y, 0x96), lo0);
        k.x += 0x9E3779B9u;
        k.y += 0xBB67AE85u;
    }
    return c;
}

struct PhiloxKey {
    uint64_t seed, subseq, first;
};

// Block number `blk` (= word index / 4) of the stream described by `key`.
__device__ __forceinline__ uint4 philox_block(const PhiloxKey &key, uint64_t blk)
{
    return philox4x32_10(make_uint4((uint32_t)blk, (uint32_t)(blk >> 32), (uint32_t)key.subseq,
                                    (uint32_t)(key.subseq >> 32)),
                         make_uint2((uint32_t)key.seed, (uint32_t)(key.seed >> 32)));
}

__device__ __forceinline__ uint32_t philox_word(const PhiloxKey &key, uint64_t g)
{
    const uint4 b = philox_block(key, g >> 2);
    const uint32_t e = (uint32_t)g & 3u;
    return e == 0 ? b.x : e == 1 ? b.y : e == 2 ? b.z : b.w;
}

// Flip lists of the sparse linear form: what info[d, r] holds for a row with `flips` entries in `pieces` 16-byte pieces
__host__ __device__ __forceinline__ uint32_t flip_info(uint32_t flips, uint32_t pieces) { return flips | (pieces << 16); }

// Block-uniform stride loop over a flat index space: every thread of a workgroup runs the same number of
// iterations (so wave-level collectives inside the body are safe); `T` may be >= TOTAL on the last one.
#define NB_FLAT_LOOP(T, TOTAL)                                                                            \
    for (int64_t T##_base = (int64_t)blockIdx.x * 256, T = T##_base + threadIdx.x; T##_base < (TOTAL); \
         T##_base += (int64_t)gridDim.x * 256, T = T##_base + threadIdx.x)

// ---- host side -----------------------------------------------------------------------------
void set_error(const char *fmt, ...);
int fail(int code, const char *fmt, ...);
int check_launch(const char *what);

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
inline hipStream_t as_stream(nb_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// The runtime rejects launches whose gridDim.x * blockDim.x does not fit in 32 bits.  One-dimensional
// kernels therefore cap the grid at kMaxBlocks workgroups of 256 and walk larger problems with a
// block-uniform stride loop; kernels that map one workgroup to one tile reject larger problems.
constexpr int64_t kMaxBlocks = 1LL << 23;
constexpr int64_t kMaxGridX = kMaxBlocks;
inline unsigned grid_for(int64_t threads) { int64_t b = ceil_div(threads, 256); return (unsigned)(b < kMaxBlocks ? b : kMaxBlocks); }

// Output size of a strided window op (extensions/booleanOperations.py:83-84,234-235).
inline int64_t out_dim(int64_t in, int f, int p, int s) { return (in - f + 2 * (int64_t)p) / s + 1; }

}  // namespace nb

#define NB_REQUIRE_PTR(p)                                            \
    do {                                                             \
        if ((p) == nullptr) return nb::fail(NB_ERR_NULL, "%s: %s is NULL", __func__, #p); \
    } while (0)
#define NB_REQUIRE_ALIGNED(p, a)                                                                        \
    do {                                                                                                \
        if (!nb::aligned((p), (a))) return nb::fail(NB_ERR_ALIGN, "%s: %s is not %d-byte aligned", __func__, #p, (int)(a)); \
    } while (0)
#define NB_REQUIRE(cond, ...)                                        \
    do {                                                             \
        if (!(cond)) return nb::fail(NB_ERR_SHAPE, __VA_ARGS__);     \
    } while (0)
