// Linear layer with the population-mean threshold (BinarizedLinear(batch_norm=True), modules/binary.py:97-102) as one
// call: XOR-popcount matrix-vector products of all members -> per-output sum over the population -> threshold
// bias + bias_noise + mean in fp16 -> compare (-> pack).  The weights are streamed once; what the steps hand to each
// other (the int32 sums of every member and the per-output totals) lives in a workspace: caller-supplied, or the
// library's own fixed device array for callers that cannot allocate.
#include <mutex>

#include "nb_common.hpp"
#include "nb_conv_common.hpp"

namespace nb {

// Fixed device array behind nb_bmv_bn_act_static_i64: per-output totals first, then the members' sums.
constexpr int64_t kBnStaticBytes = (4 << 20) + (64 << 10);
static __device__ __align__(256) unsigned char scratch[kBnStaticBytes];

static int64_t bn_colsum_bytes(int64_t M) { return ceil_div(M * 8, 256) * 256; }
static int64_t bn_workspace_bytes(int64_t Z, int64_t M) { return bn_colsum_bytes(M) + ceil_div(Z * M * 4, 256) * 256; }

// Clears by a kernel, not a memset node, so that the call can be captured into a HIP graph.
__global__ __launch_bounds__(256) void bn_zero_kernel(uint32_t *__restrict__ p, int64_t n)
{
    NB_FLAT_LOOP(t, n)
    {
        if (t < n) p[t] = 0u;
    }
}

// colsum[m] += sum of popc[z, m] over one chunk of members; consecutive threads take consecutive m.
constexpr int kBnChunk = 64;
// ROUND: the activations 2*popc - K are rounded to fp16 first, as `activation.type(torch.float16)` does, and their
// (signed) sum is what is added up, in two's complement.
template <bool ROUND>
__global__ __launch_bounds__(256) void bn_colsum_kernel(unsigned long long *__restrict__ colsum,
                                                        const int32_t *__restrict__ popc, int64_t Z, int64_t M, int64_t K)
{
    const int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (m >= M) return;
    const int64_t z0 = (int64_t)blockIdx.y * kBnChunk;
    const int64_t z1 = z0 + kBnChunk < Z ? z0 + kBnChunk : Z;
    unsigned long long s = 0;
    // unrolled: the loads of sixteen members are in flight together (with few columns a workgroup has few lanes at
    // work and nothing else hides their round trips)
#pragma unroll 16
    for (int64_t z = z0; z < z1; z++) {
        const int32_t pc = popc[z * M + m];
        if (ROUND)
            s += (unsigned long long)(long long)(float)(_Float16)(float)(2ll * pc - K);  // an integer again: |.| <= 65504
        else
            s += (unsigned long long)(uint32_t)pc;
    }
    atomicAdd(colsum + m, s);
}

// act = 2*popc - K against thr = fp16(fp16(bias + bias_noise) + mean), mean = fp16(float(sum of act) * factor), the
// exact product rounded once, with factor = float(M) / float(Z * M): torch's fp16 mean accumulates in fp32 and
// multiplies by that quotient of the output and input element counts, so this is its result whenever the fp32 sum
// is exact (up to 2^24 in magnitude).
// act is an integer and thr an fp16 number, so act > thr <=> act > floor(thr) (never for NaN).
// ROUND: total is the sum of the fp16-rounded activations, and the activation is rounded to fp16 for the compare as
// well (torch compares an int32 tensor with an fp16 one in fp16): the reference's arithmetic for rows of more than
// 2048 bits, where 2*popc - K is no longer exact in fp16.
template <bool ROUND>
__device__ __forceinline__ bool bn_bit(int32_t popc, unsigned long long total, _Float16 bias, _Float16 noise, int64_t Z,
                                       int64_t K, float factor)
{
    const long long sum_act = ROUND ? (long long)total : 2ll * (long long)total - (long long)K * (long long)Z;
    const _Float16 mean = mul_round_once_fp16((float)sum_act, factor);
    const _Float16 tb = bias + noise;
    const float t = (float)(_Float16)(tb + mean);
    if (t != t) return false;
    const long long act = 2ll * popc - (long long)K;
    if (ROUND) return (float)(_Float16)(float)act > t;
    const float tc = fminf(fmaxf(t, -1.0e9f), 1.0e9f);
    return act > (long long)floorf(tc);
}

template <bool ROUND>
__global__ __launch_bounds__(256) void bn_bool_kernel(uint8_t *__restrict__ out, const int32_t *__restrict__ popc,
                                                      const unsigned long long *__restrict__ colsum,
                                                      const _Float16 *__restrict__ bias,
                                                      const _Float16 *__restrict__ noise, int64_t Z, int64_t M,
                                                      int64_t K, float factor)
{
    NB_FLAT_LOOP(t, Z * M)
    {
        if (t < Z * M) {
            const int64_t m = t % M;
            out[t] = bn_bit<ROUND>(popc[t], colsum[m], bias[m], noise[t], Z, K, factor) ? 1 : 0;
        }
    }
}

// One wave per output word: lane i < bits decides bit i, the ballot is the word.
template <typename W, bool ROUND>
__global__ __launch_bounds__(256) void bn_pack_kernel(W *__restrict__ out, const int32_t *__restrict__ popc,
                                                      const unsigned long long *__restrict__ colsum,
                                                      const _Float16 *__restrict__ bias,
                                                      const _Float16 *__restrict__ noise, int64_t Z, int64_t M,
                                                      int64_t Mw, int64_t K, float factor)
{
    constexpr int bits = WordTraits<W>::bits;
    const int lane = threadIdx.x & 63;
    const int64_t wd = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wd >= Z * Mw) return;  // wave-uniform
    const int64_t z = wd / Mw;
    const int64_t m = (wd - z * Mw) * bits + lane;
    bool bit = false;
    if (lane < bits && m < M) bit = bn_bit<ROUND>(popc[z * M + m], colsum[m], bias[m], noise[z * M + m], Z, K, factor);
    const unsigned long long word = __ballot(bit);
    if (lane == 0) out[wd] = (W)word;
}

template <typename W>
static int bn_impl(void *out, const W *A, const W *x, const uint16_t *bias, const uint16_t *noise, int64_t Z, int64_t M,
                   int64_t Kw, int64_t K, int pack, void *workspace, int64_t workspace_bytes, nb_stream_t stream,
                   const char *who)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_REQUIRE(pack >= 0 && pack <= 3, "%s: pack must be 0..3 (bit 0: packed output, bit 1: fp16-rounded activations)", who);
    const bool round16 = (pack & 2) != 0;
    pack &= 1;
    NB_REQUIRE(!round16 || K <= 65504, "%s: K=%lld is beyond fp16", who, (long long)K);
    NB_REQUIRE(Z >= 0 && M >= 0 && Kw >= 0 && K >= 0, "%s: negative shape Z=%lld M=%lld Kw=%lld K=%lld", who,
               (long long)Z, (long long)M, (long long)Kw, (long long)K);
    NB_REQUIRE(K <= Kw * (int64_t)bits, "%s: K=%lld exceeds the %lld bits of a row", who, (long long)K,
               (long long)(Kw * bits));
    if (Z * M == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(bias);
    NB_REQUIRE_PTR(noise);
    NB_REQUIRE_ALIGNED(bias, 2);
    NB_REQUIRE_ALIGNED(noise, 2);
    if (pack) NB_REQUIRE_ALIGNED(out, sizeof(W));
    NB_REQUIRE(Z < (1LL << 31) && M < (1LL << 31) && Z * M < (1LL << 40), "%s: Z=%lld or M=%lld too large", who,
               (long long)Z, (long long)M);
    NB_REQUIRE(Z <= 65535 * (int64_t)kBnChunk, "%s: more than %lld members", who, (long long)(65535 * (int64_t)kBnChunk));
    const int64_t Mw = ceil_div(M, bits);
    NB_REQUIRE(!pack || ceil_div(Z * Mw, 4) <= kMaxGridX, "%s: output exceeds one launch", who);
    NB_REQUIRE_PTR(workspace);
    NB_REQUIRE_ALIGNED(workspace, 256);
    NB_REQUIRE(workspace_bytes >= bn_workspace_bytes(Z, M), "%s: workspace of %lld bytes, %lld needed", who,
               (long long)workspace_bytes, (long long)bn_workspace_bytes(Z, M));
    hipStream_t s = as_stream(stream);
    auto *colsum = static_cast<unsigned long long *>(workspace);
    auto *popc = reinterpret_cast<int32_t *>(static_cast<unsigned char *>(workspace) + bn_colsum_bytes(M));
    const unsigned mblocks = (unsigned)ceil_div(M, 256);
    bn_zero_kernel<<<dim3(grid_for(2 * M)), dim3(256), 0, s>>>(reinterpret_cast<uint32_t *>(colsum), 2 * M);
    if (int rc = check_launch(who)) return rc;
    // the members' sums: the matrix-vector form of the XOR-popcount product (Kw == 0: all zero)
    int rc;
    if (Kw == 0) {
        bn_zero_kernel<<<dim3(grid_for(Z * M)), dim3(256), 0, s>>>(reinterpret_cast<uint32_t *>(popc), Z * M);
        rc = check_launch(who);
    } else if (sizeof(W) == 8) {
        rc = nb_bmm_i64(popc, reinterpret_cast<const int64_t *>(A), reinterpret_cast<const int64_t *>(x), Z, M, Kw, 1,
                        stream);
    } else {
        rc = nb_bmm_i32(popc, reinterpret_cast<const int32_t *>(A), reinterpret_cast<const int32_t *>(x), Z, M, Kw, 1,
                        stream);
    }
    if (rc) return rc;
    const dim3 cgrid(mblocks, (unsigned)ceil_div(Z, kBnChunk));
    if (round16)
        bn_colsum_kernel<true><<<cgrid, dim3(256), 0, s>>>(colsum, popc, Z, M, K);
    else
        bn_colsum_kernel<false><<<cgrid, dim3(256), 0, s>>>(colsum, popc, Z, M, K);
    if (int rc2 = check_launch(who)) return rc2;
    const auto *b16 = reinterpret_cast<const _Float16 *>(bias), *n16 = reinterpret_cast<const _Float16 *>(noise);
    const float factor = mean_factor(M, Z * M);
    if (pack) {
        const dim3 pgrid((unsigned)ceil_div(Z * Mw, 4));
        if (round16)
            bn_pack_kernel<W, true><<<pgrid, dim3(256), 0, s>>>(static_cast<W *>(out), popc, colsum, b16, n16, Z, M, Mw, K, factor);
        else
            bn_pack_kernel<W, false><<<pgrid, dim3(256), 0, s>>>(static_cast<W *>(out), popc, colsum, b16, n16, Z, M, Mw, K, factor);
    } else {
        const dim3 bgrid(grid_for(Z * M));
        if (round16)
            bn_bool_kernel<true><<<bgrid, dim3(256), 0, s>>>(static_cast<uint8_t *>(out), popc, colsum, b16, n16, Z, M, K, factor);
        else
            bn_bool_kernel<false><<<bgrid, dim3(256), 0, s>>>(static_cast<uint8_t *>(out), popc, colsum, b16, n16, Z, M, K, factor);
    }
    return check_launch(who);
}

// Device address of `scratch` on the current device, looked up once per device (each GPU holds its own copy of the
// array at its own address).
static int bn_static_ptr(void **ptr, const char *who)
{
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void *ptrs[kMaxDevices] = {};
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return fail(NB_ERR_UNSUPPORTED, "%s: no current device", who);
    }
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            set_error("%s: hipGetSymbolAddress failed: %s", who, hipGetErrorString(e));
            return NB_ERR_HIP_BASE + (int)e;
        }
        ptrs[dev] = p;
    }
    *ptr = ptrs[dev];
    return NB_OK;
}

// Thresholds of BinarizedConv2d(batch_norm=True) from the pixel sums of the popcount maps (bn_conv_threshold in
// nb_conv_common.hpp holds the arithmetic).  One thread per (member, channel); thresh may be sums.
__global__ __launch_bounds__(256) void bn_conv_thresh_kernel(int32_t *thresh, const int32_t *sums,
                                                             const _Float16 *__restrict__ bias,
                                                             const _Float16 *__restrict__ noise, int64_t D, int64_t O,
                                                             int64_t K, int64_t HW, float factor)
{
    NB_FLAT_LOOP(t, D * O)
    {
        if (t < D * O) thresh[t] = bn_conv_threshold(sums[t], bias[t % O], noise[t], K, HW, factor);
    }
}

void bn_conv_thresh_launch(int32_t *thresh, const int32_t *sums, const _Float16 *bias, const _Float16 *noise, int64_t D,
                           int64_t O, int64_t K, int64_t HW, hipStream_t s)
{
    bn_conv_thresh_kernel<<<dim3(grid_for(D * O)), dim3(256), 0, s>>>(thresh, sums, bias, noise, D, O, K, HW,
                                                                      mean_factor(D * O, D * O * HW));
}

}  // namespace nb

extern "C" {
int nb_conv_bn_thresholds(int32_t *thresh, const int32_t *sums, const uint16_t *bias, const uint16_t *bias_noise,
                           int64_t D, int64_t O, int64_t K, int64_t HW, nb_stream_t stream)
{
    const char *who = "nb_conv_bn_thresholds";
    NB_REQUIRE(D >= 0 && O >= 0 && K >= 0 && HW >= 1, "%s: bad shape D=%lld O=%lld K=%lld HW=%lld", who, (long long)D,
               (long long)O, (long long)K, (long long)HW);
    NB_REQUIRE(K < (1LL << 31) && HW < (1LL << 31) && D * O < (1LL << 40), "%s: too large", who);
    if (D * O == 0) return NB_OK;
    NB_REQUIRE_PTR(thresh);
    NB_REQUIRE_PTR(sums);
    NB_REQUIRE_PTR(bias);
    NB_REQUIRE_PTR(bias_noise);
    NB_REQUIRE_ALIGNED(thresh, 4);
    NB_REQUIRE_ALIGNED(sums, 4);
    NB_REQUIRE_ALIGNED(bias, 2);
    NB_REQUIRE_ALIGNED(bias_noise, 2);
    nb::bn_conv_thresh_launch(thresh, sums, reinterpret_cast<const _Float16 *>(bias),
                              reinterpret_cast<const _Float16 *>(bias_noise), D, O, K, HW, nb::as_stream(stream));
    return nb::check_launch(who);
}
int64_t nb_bmv_bn_workspace_bytes(int64_t Z, int64_t M)
{
    if (Z < 0 || M < 0 || Z >= (1LL << 31) || M >= (1LL << 31)) return -1;
    return nb::bn_workspace_bytes(Z, M);
}
int64_t nb_bmv_bn_static_bytes(void) { return nb::kBnStaticBytes; }
int nb_bmv_bn_act_i64(void *out, const int64_t *A, const int64_t *x, const uint16_t *bias, const uint16_t *bias_noise,
                      int64_t Z, int64_t M, int64_t Kw, int64_t K, int pack, void *workspace, int64_t workspace_bytes,
                      nb_stream_t s)
{
    return nb::bn_impl<uint64_t>(out, reinterpret_cast<const uint64_t *>(A), reinterpret_cast<const uint64_t *>(x), bias,
                                 bias_noise, Z, M, Kw, K, pack, workspace, workspace_bytes, s, "nb_bmv_bn_act_i64");
}
int nb_bmv_bn_act_i32(void *out, const int32_t *A, const int32_t *x, const uint16_t *bias, const uint16_t *bias_noise,
                      int64_t Z, int64_t M, int64_t Kw, int64_t K, int pack, void *workspace, int64_t workspace_bytes,
                      nb_stream_t s)
{
    return nb::bn_impl<uint32_t>(out, reinterpret_cast<const uint32_t *>(A), reinterpret_cast<const uint32_t *>(x), bias,
                                 bias_noise, Z, M, Kw, K, pack, workspace, workspace_bytes, s, "nb_bmv_bn_act_i32");
}
int nb_bmv_bn_act_static_i64(void *out, const int64_t *A, const int64_t *x, const uint16_t *bias,
                             const uint16_t *bias_noise, int64_t Z, int64_t M, int64_t Kw, int64_t K, int pack,
                             nb_stream_t s)
{
    const char *who = "nb_bmv_bn_act_static_i64";
    if (Z >= 0 && M >= 0 && Z < (1LL << 31) && M < (1LL << 31) && nb::bn_workspace_bytes(Z, M) > nb::kBnStaticBytes)
        return nb::fail(NB_ERR_SHAPE, "%s: Z=%lld, M=%lld need %lld bytes of workspace, the fixed array holds %lld", who,
                        (long long)Z, (long long)M, (long long)nb::bn_workspace_bytes(Z, M),
                        (long long)nb::kBnStaticBytes);
    void *ptr = nullptr;
    if (Z * M != 0)
        if (int rc = nb::bn_static_ptr(&ptr, who)) return rc;
    return nb::bn_impl<uint64_t>(out, reinterpret_cast<const uint64_t *>(A), reinterpret_cast<const uint64_t *>(x), bias,
                                 bias_noise, Z, M, Kw, K, pack, ptr, nb::kBnStaticBytes, s, who);
}
}
