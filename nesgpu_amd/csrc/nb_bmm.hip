// XOR-popcount batched matmul: C[z,x,y] = sum_k popc(A[z,x,k] ^ B[z,k,y]).
//
// Two kernels:
//  * N == 1 (the linear layer's matrix-vector form, modules/binary.py:97): the weight stream is
//    read exactly once, so the kernel is HBM-bound.  A group of L lanes walks one weight row
//    with 16-byte loads (consecutive lanes read consecutive addresses), XORs with the member's
//    input words and reduces the popcounts across the group.
//  * otherwise: the row-per-lane kernel of nb_rowlane.hpp (B fetched through scalar loads).
#include "nb_rowlane.hpp"

namespace nb {

template <typename W, int L, int V, int RPG, int BS>
__global__ __launch_bounds__(BS) void bmv_kernel(int32_t *__restrict__ C, const W *__restrict__ A,
                                                 const W *__restrict__ X, int64_t rows, int64_t M, int Kw)
{
    typedef W WV __attribute__((ext_vector_type(V == 2 ? 2 : 1)));
    const int64_t gid = ((int64_t)blockIdx.x * BS + threadIdx.x) / L;
    const int sub = threadIdx.x % L;
    const int64_t r0 = gid * RPG;
    int acc[RPG];
#pragma unroll
    for (int q = 0; q < RPG; q++) acc[q] = 0;
    // rows past the end are clamped (recomputed, never stored) so that the loads need no branches
    int64_t rr[RPG], zz[RPG];
    {
        const int64_t last = rows - 1;
        const int64_t rc = r0 < last ? r0 : last;
        int64_t z = rc / M, m = rc - z * M;
#pragma unroll
        for (int q = 0; q < RPG; q++) {
            rr[q] = r0 + q < last ? r0 + q : last;
            zz[q] = z;
            if (r0 + q < last && ++m == M) {
                m = 0;
                z++;
            }
        }
    }
    for (int k = sub * V; k < Kw; k += L * V) {
        WV av[RPG], xv[RPG];
#pragma unroll
        for (int q = 0; q < RPG; q++) xv[q] = *reinterpret_cast<const WV *>(X + zz[q] * Kw + k);
#pragma unroll
        for (int q = 0; q < RPG; q++)
            av[q] = __builtin_nontemporal_load(reinterpret_cast<const WV *>(A + rr[q] * Kw + k));  // read once
        __builtin_amdgcn_sched_barrier(0);  // all loads of the step in flight before the first use
#pragma unroll
        for (int q = 0; q < RPG; q++) {
            if (V == 2) acc[q] += popc_xor(av[q][0], xv[q][0]) + popc_xor(av[q][V - 1], xv[q][V - 1]);
            else acc[q] += popc_xor(av[q][0], xv[q][0]);
        }
    }
#pragma unroll
    for (int off = L / 2; off > 0; off >>= 1) {
#pragma unroll
        for (int q = 0; q < RPG; q++) acc[q] += __shfl_xor(acc[q], off);
    }
    if (sub == 0) {
#pragma unroll
        for (int q = 0; q < RPG; q++)
            if (r0 + q < rows) C[r0 + q] = acc[q];
    }
}

template <typename W, int KC, int NT, bool SINGLE, bool EXACT, class Epi>
__global__ __launch_bounds__(256) void bmm_rowlane_kernel(RowsA<W> al, const W *__restrict__ Bm, Epi epi, int mblocks,
                                                          int N)
{
    const int64_t z = blockIdx.x / mblocks;
    const int64_t m = (int64_t)(blockIdx.x - z * mblocks) * 256 + threadIdx.x;
    const typename RowsA<W>::Lane lane = al.lane(z, m);
    const W *__restrict__ Bz = Bm + z * al.Kw * (int64_t)N;
    rowlane_body<W, KC, NT, SINGLE, EXACT>(al, lane, Bz, epi, z * al.M + m, z, al.Kw, N);
}

template <typename W, int L, int V>
static void launch_bmv(int32_t *C, const W *A, const W *X, int64_t rows, int64_t M, int Kw, hipStream_t s)
{
    constexpr int RPG = 4, BS = 1024;  // 8 rows per group measured slower (fewer waves fit)
    const int64_t groups = ceil_div(rows, RPG);
    const int64_t blocks = ceil_div(groups * L, BS);
    bmv_kernel<W, L, V, RPG, BS><<<dim3((unsigned)blocks), dim3(BS), 0, s>>>(C, A, X, rows, M, Kw);
}

template <typename W, int V>
static void dispatch_bmv(int32_t *C, const W *A, const W *X, int64_t rows, int64_t M, int Kw, hipStream_t s)
{
    const int per = (Kw + V - 1) / V;  // lane-steps needed to cover a row once
    if (per <= 1) launch_bmv<W, 1, V>(C, A, X, rows, M, Kw, s);
    else if (per <= 2) launch_bmv<W, 2, V>(C, A, X, rows, M, Kw, s);
    else if (per <= 4) launch_bmv<W, 4, V>(C, A, X, rows, M, Kw, s);
    else if (per <= 8) launch_bmv<W, 8, V>(C, A, X, rows, M, Kw, s);
    else if (per <= 16) launch_bmv<W, 16, V>(C, A, X, rows, M, Kw, s);
    else if (per <= 32) launch_bmv<W, 32, V>(C, A, X, rows, M, Kw, s);
    else launch_bmv<W, 64, V>(C, A, X, rows, M, Kw, s);
}

template <typename W, class Epi>
static void dispatch_rowlane(const RowsA<W> &al, const W *B, const Epi &epi, int64_t Z, int64_t M, int Kw, int N,
                             hipStream_t s)
{
    const int mblocks = (int)ceil_div(M, 256);
    const dim3 grid((unsigned)(Z * mblocks)), block(256);
    if (Kw == 9) bmm_rowlane_kernel<W, 9, 16, true, true, Epi><<<grid, block, 0, s>>>(al, B, epi, mblocks, N);
    else if (Kw == 18) bmm_rowlane_kernel<W, 18, 16, true, true, Epi><<<grid, block, 0, s>>>(al, B, epi, mblocks, N);
    else if (Kw <= 4) bmm_rowlane_kernel<W, 4, 16, true, false, Epi><<<grid, block, 0, s>>>(al, B, epi, mblocks, N);
    else if (Kw <= 9) bmm_rowlane_kernel<W, 9, 16, true, false, Epi><<<grid, block, 0, s>>>(al, B, epi, mblocks, N);
    else if (Kw <= 18) bmm_rowlane_kernel<W, 18, 16, true, false, Epi><<<grid, block, 0, s>>>(al, B, epi, mblocks, N);
    else bmm_rowlane_kernel<W, 16, 16, false, false, Epi><<<grid, block, 0, s>>>(al, B, epi, mblocks, N);
}

template <typename W>
static int bmm_check(const void *C, const W *A, const W *B, int64_t Z, int64_t M, int64_t Kw, int64_t N,
                     const char *who, bool *empty)
{
    NB_REQUIRE(Z >= 0 && M >= 0 && Kw >= 0 && N >= 0, "%s: negative shape Z=%lld M=%lld Kw=%lld N=%lld", who,
               (long long)Z, (long long)M, (long long)Kw, (long long)N);
    *empty = (Z * M * N == 0);
    if (*empty) return NB_OK;
    NB_REQUIRE_PTR(C);
    if (Kw > 0) {
        NB_REQUIRE_PTR(A);
        NB_REQUIRE_PTR(B);
        NB_REQUIRE_ALIGNED(A, sizeof(W));
        NB_REQUIRE_ALIGNED(B, sizeof(W));
    }
    NB_REQUIRE(Kw <= (1 << 24) && N <= (1 << 24), "%s: Kw=%lld or N=%lld above 2^24", who, (long long)Kw,
               (long long)N);
    NB_REQUIRE(Z * ceil_div(M, 256) <= kMaxGridX && Z * M < (1LL << 40), "%s: Z*M=%lld rows exceed one launch", who,
               (long long)(Z * M));
    return NB_OK;
}

template <typename W>
int bmm_impl(int32_t *C, const W *A, const W *B, int64_t Z, int64_t M, int64_t Kw, int64_t N, nb_stream_t stream,
             const char *who)
{
    bool empty;
    if (int rc = bmm_check<W>(C, A, B, Z, M, Kw, N, who, &empty)) return rc;
    if (empty) return NB_OK;
    NB_REQUIRE_ALIGNED(C, 4);
    hipStream_t s = as_stream(stream);
    if (N == 1 && Kw > 0) {
        const int64_t rows = Z * M;
        NB_REQUIRE(ceil_div(ceil_div(rows, 4) * 64, 256) <= kMaxGridX, "%s: %lld rows exceed one launch", who,
                   (long long)rows);
        if ((Kw & 1) == 0 && aligned(A, 2 * sizeof(W)) && aligned(B, 2 * sizeof(W)))
            dispatch_bmv<W, 2>(C, A, B, rows, M, (int)Kw, s);
        else
            dispatch_bmv<W, 1>(C, A, B, rows, M, (int)Kw, s);
    } else {
        RowsA<W> al{A, M, (int)Kw};
        EpiI32 epi{C, (N & 3) == 0 && aligned(C, 16)};
        dispatch_rowlane<W, EpiI32>(al, B, epi, Z, M, (int)Kw, (int)N, s);
    }
    return check_launch(who);
}

template <typename W>
int bmm_act_impl(uint8_t *C, const W *A, const W *B, const int32_t *thresh, int64_t Z, int64_t M, int64_t Kw,
                 int64_t N, nb_stream_t stream, const char *who)
{
    bool empty;
    if (int rc = bmm_check<W>(C, A, B, Z, M, Kw, N, who, &empty)) return rc;
    if (empty) return NB_OK;
    NB_REQUIRE_PTR(thresh);
    NB_REQUIRE_ALIGNED(thresh, 4);
    RowsA<W> al{A, M, (int)Kw};
    EpiBool epi{C, thresh, (N & 3) == 0 && aligned(C, 4)};
    dispatch_rowlane<W, EpiBool>(al, B, epi, Z, M, (int)Kw, (int)N, as_stream(stream));
    return check_launch(who);
}

}  // namespace nb

extern "C" {
int nb_bmm_i64(int32_t *C, const int64_t *A, const int64_t *B, int64_t Z, int64_t M, int64_t Kw, int64_t N,
               nb_stream_t s)
{
    return nb::bmm_impl<uint64_t>(C, reinterpret_cast<const uint64_t *>(A), reinterpret_cast<const uint64_t *>(B), Z,
                                  M, Kw, N, s, "nb_bmm_i64");
}
int nb_bmm_i32(int32_t *C, const int32_t *A, const int32_t *B, int64_t Z, int64_t M, int64_t Kw, int64_t N,
               nb_stream_t s)
{
    return nb::bmm_impl<uint32_t>(C, reinterpret_cast<const uint32_t *>(A), reinterpret_cast<const uint32_t *>(B), Z,
                                  M, Kw, N, s, "nb_bmm_i32");
}
int nb_bmm_act_i64(uint8_t *C, const int64_t *A, const int64_t *B, const int32_t *thresh, int64_t Z, int64_t M,
                   int64_t Kw, int64_t N, nb_stream_t s)
{
    return nb::bmm_act_impl<uint64_t>(C, reinterpret_cast<const uint64_t *>(A), reinterpret_cast<const uint64_t *>(B),
                                      thresh, Z, M, Kw, N, s, "nb_bmm_act_i64");
}
int nb_bmm_act_i32(uint8_t *C, const int32_t *A, const int32_t *B, const int32_t *thresh, int64_t Z, int64_t M,
                   int64_t Kw, int64_t N, nb_stream_t s)
{
    return nb::bmm_act_impl<uint32_t>(C, reinterpret_cast<const uint32_t *>(A), reinterpret_cast<const uint32_t *>(B),
                                      thresh, Z, M, Kw, N, s, "nb_bmm_act_i32");
}
}
