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
                                                 const W *__restrict__ X, int64_t rows, int64_t M, int Kw,
                                                 int omul, int osub)
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
            if (r0 + q < rows) C[r0 + q] = acc[q] * omul - osub;
    }
}

// Matrix-vector form for short rows (16, 32 or 64 bytes: VPR 16-byte vectors): a lane owns whole rows, so there is no
// cross-lane reduction at all.  A wave takes Q runs of 64 consecutive rows (every load instruction reads one
// contiguous run of 64 rows), all Q * VPR streaming loads of a lane are requested before the first use, and the
// member's input vector (the same few bytes for all lanes of a run, or two neighbouring ones) comes through the cache.
template <int VPR, int Q>
__global__ __launch_bounds__(256) void bmv_short_kernel(int32_t *__restrict__ C, const uint4 *__restrict__ A,
                                                        const uint4 *__restrict__ X, uint32_t rows, uint32_t M,
                                                        int omul, int osub)
{
    const uint32_t wave_first = (blockIdx.x * 256u + (threadIdx.x & ~63u)) * Q;
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t row[Q];
    uint4 a[Q][VPR], x[Q][VPR];
#pragma unroll
    for (int q = 0; q < Q; q++) {
        row[q] = wave_first + q * 64u + lane;
        const uint32_t rc = row[q] < rows ? row[q] : rows - 1;  // rows past the end are recomputed, never stored
#pragma unroll
        for (int v = 0; v < VPR; v++) a[q][v] = load_stream16(A + (int64_t)rc * VPR + v);
        const uint32_t z = rc / M;
#pragma unroll
        for (int v = 0; v < VPR; v++) x[q][v] = X[(int64_t)z * VPR + v];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int q = 0; q < Q; q++) {
        int acc = 0;
#pragma unroll
        for (int v = 0; v < VPR; v++) {
            acc = bcnt_acc(a[q][v].x ^ x[q][v].x, acc);
            acc = bcnt_acc(a[q][v].y ^ x[q][v].y, acc);
            acc = bcnt_acc(a[q][v].z ^ x[q][v].z, acc);
            acc = bcnt_acc(a[q][v].w ^ x[q][v].w, acc);
        }
        if (row[q] < rows) C[row[q]] = acc * omul - osub;
    }
}

template <int VPR>
static void launch_bmv_short(int32_t *C, const void *A, const void *X, int64_t rows, int64_t M, hipStream_t s, int omul,
                             int osub)
{
    constexpr int Q = 4;
    bmv_short_kernel<VPR, Q><<<dim3((unsigned)ceil_div(rows, 256 * Q)), dim3(256), 0, s>>>(
        C, static_cast<const uint4 *>(A), static_cast<const uint4 *>(X), (uint32_t)rows, (uint32_t)M, omul, osub);
}

// Matrix-vector form for long rows: L lanes (16, 32 or 64) walk FOUR rows of one member with 16-byte streaming
// loads, so the input vector is loaded once per step for all four, and the four per-lane sums are reduced by a
// transposing butterfly: two quad steps halve the rows a lane carries (4 -> 2 -> 1) while they add, then two
// rotations inside the row of 16 and at most two cross-row exchanges finish the one remaining value.  That is 9
// cross-lane operations instead of 24, which matters because at HBM speed the vector ALUs, not the memory
// system, are what this kernel runs out of.  Popcounts do not care about the word width: rows are handled as
// 16-byte vectors.  Needs M % 4 == 0 (the four rows share the member's input) and rows of whole 16-byte vectors.
// U steps of the row walk are requested together (4*U loads of 16 bytes in flight per lane); needs
// rowvecs % (U*L) == 0.
// PACK: instead of the int32 sums, the bits (2*sum > thresh[row]) of the workgroup's 4*BS/L consecutive rows, packed
// LSB-first (C is then the output bit array in 32-bit pieces; the host makes sure that a member's rows fill whole
// words, so the flat row number is the flat bit number).
template <int L, int U, int BS, bool PACK = false>
__global__ __launch_bounds__(BS) void bmv_quad_kernel(int32_t *__restrict__ C, const uint4 *__restrict__ A,
                                                      const uint4 *__restrict__ X, int64_t quads, int64_t M,
                                                      int rowvecs, const int32_t *__restrict__ thresh = nullptr,
                                                      int omul = 1, int osub = 0)
{
    constexpr int RPB = 4 * BS / L;  // rows of a workgroup
    __shared__ uint32_t pieces[PACK ? RPB / 32 : 1];
    if (PACK) {
        if (threadIdx.x < RPB / 32) pieces[threadIdx.x] = 0u;
        __syncthreads();
    }
    const int64_t gid = ((int64_t)blockIdx.x * BS + threadIdx.x) / L;
    const int sub = threadIdx.x % L;
    const bool live = gid < quads;
    const int64_t r0 = (live ? gid : quads - 1) * 4;  // dead groups recompute the last quad and store nothing
    const int64_t z = r0 / M;
    const uint4 *a = A + r0 * rowvecs, *x = X + z * rowvecs;
    int acc[4] = {0, 0, 0, 0};
    for (int k = sub; k < rowvecs; k += L * U) {
        uint4 xv[U], av[U][4];
#pragma unroll
        for (int u = 0; u < U; u++) xv[u] = x[k + u * L];
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int q = 0; q < 4; q++) av[u][q] = load_stream16(a + (int64_t)q * rowvecs + k + u * L);  // read once
        __builtin_amdgcn_sched_barrier(0);  // all loads of the step in flight before the first use
#pragma unroll
        for (int u = 0; u < U; u++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                acc[q] = bcnt_acc(av[u][q].x ^ xv[u].x, acc[q]);
                acc[q] = bcnt_acc(av[u][q].y ^ xv[u].y, acc[q]);
                acc[q] = bcnt_acc(av[u][q].z ^ xv[u].z, acc[q]);
                acc[q] = bcnt_acc(av[u][q].w ^ xv[u].w, acc[q]);
            }
    }
    const bool b0 = threadIdx.x & 1, b1 = threadIdx.x & 2;
    // lanes with bit 0 clear keep rows 0,1 and hand rows 2,3 to their neighbour, the others the reverse
    int k0 = b0 ? acc[2] : acc[0], k1 = b0 ? acc[3] : acc[1];
    const int s0 = b0 ? acc[0] : acc[2], s1 = b0 ? acc[1] : acc[3];
    k0 += (int)dpp_mov<0xB1>((uint32_t)s0);  // quad_perm [1,0,3,2]
    k1 += (int)dpp_mov<0xB1>((uint32_t)s1);
    // bit 1 clear: keep the first of the two rows
    int v = b1 ? k1 : k0;
    v += (int)dpp_mov<0x4E>((uint32_t)(b1 ? k0 : k1));  // quad_perm [2,3,0,1]
    v += (int)dpp_mov<0x124>((uint32_t)v);               // row_ror:4
    v += (int)dpp_mov<0x128>((uint32_t)v);               // row_ror:8
    if (L >= 32) v += __shfl_xor(v, 16);
    if (L >= 64) v += __shfl_xor(v, 32);
    // lane q < 4 of the group now holds row 2*(q&1) + (q>>1); streaming stores: the results are read by another
    // kernel, and ordinary stores between the row loads cost this kernel 2 % of its bandwidth (measured)
    if (!PACK) {
        if (live && sub < 4) __builtin_nontemporal_store(v * omul - osub, C + r0 + 2 * (sub & 1) + (sub >> 1));
    } else {
        if (live && sub < 4) {
            const int64_t row = r0 + 2 * (sub & 1) + (sub >> 1);
            const int local = (int)(row - (int64_t)blockIdx.x * RPB);
            if (2 * v > thresh[row]) atomicOr(&pieces[local >> 5], 1u << (local & 31));
        }
        __syncthreads();
        const int64_t piece = (int64_t)blockIdx.x * (RPB / 32) + threadIdx.x;
        if (threadIdx.x < RPB / 32 && piece * 32 < quads * 4) reinterpret_cast<uint32_t *>(C)[piece] = pieces[threadIdx.x];
    }
}

template <int L, int U>
static void launch_bmv_quad(int32_t *C, const void *A, const void *X, int64_t rows, int64_t M, int rowvecs, hipStream_t s,
                            const int32_t *thresh = nullptr, int omul = 1, int osub = 0)
{
    constexpr int BS = 1024;
    const int64_t quads = rows / 4;
    const int64_t blocks = ceil_div(quads * L, BS);
    if (thresh)
        bmv_quad_kernel<L, U, BS, true><<<dim3((unsigned)blocks), dim3(BS), 0, s>>>(
            C, static_cast<const uint4 *>(A), static_cast<const uint4 *>(X), quads, M, rowvecs, thresh);
    else
        bmv_quad_kernel<L, U, BS><<<dim3((unsigned)blocks), dim3(BS), 0, s>>>(
            C, static_cast<const uint4 *>(A), static_cast<const uint4 *>(X), quads, M, rowvecs, nullptr, omul, osub);
}

// Any shape: one wave per output word, its rows one after the other (lanes stride over the row's words).
template <typename W>
__global__ __launch_bounds__(256) void bmv_act_pack_generic_kernel(W *__restrict__ out, const W *__restrict__ A,
                                                                   const W *__restrict__ X,
                                                                   const int32_t *__restrict__ thresh, int64_t words,
                                                                   int64_t M, int Mw, int Kw)
{
    constexpr int bits = WordTraits<W>::bits;
    const int lane = threadIdx.x & 63;
    const int64_t wd = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (wd >= words) return;  // wave-uniform, no barrier below
    const int64_t z = wd / Mw;
    const int64_t m0 = (wd - z * Mw) * bits;
    W word = 0;
    for (int i = 0; i < bits && m0 + i < M; i++) {
        const W *a = A + (z * M + m0 + i) * Kw, *x = X + z * Kw;
        int acc = 0;
        for (int k = lane; k < Kw; k += 64) acc += popc_xor(a[k], x[k]);
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off);
        if (2 * acc > thresh[z * M + m0 + i]) word |= (W)1 << i;
    }
    if (lane == 0) out[wd] = word;
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
static void launch_bmv(int32_t *C, const W *A, const W *X, int64_t rows, int64_t M, int Kw, hipStream_t s, int omul,
                       int osub)
{
    constexpr int RPG = 4, BS = 1024;  // 8 rows per group measured slower (fewer waves fit)
    const int64_t groups = ceil_div(rows, RPG);
    const int64_t blocks = ceil_div(groups * L, BS);
    bmv_kernel<W, L, V, RPG, BS><<<dim3((unsigned)blocks), dim3(BS), 0, s>>>(C, A, X, rows, M, Kw, omul, osub);
}

template <typename W, int V>
static void dispatch_bmv(int32_t *C, const W *A, const W *X, int64_t rows, int64_t M, int Kw, hipStream_t s, int omul,
                         int osub)
{
    const int per = (Kw + V - 1) / V;  // lane-steps needed to cover a row once
    if (per <= 1) launch_bmv<W, 1, V>(C, A, X, rows, M, Kw, s, omul, osub);
    else if (per <= 2) launch_bmv<W, 2, V>(C, A, X, rows, M, Kw, s, omul, osub);
    else if (per <= 4) launch_bmv<W, 4, V>(C, A, X, rows, M, Kw, s, omul, osub);
    else if (per <= 8) launch_bmv<W, 8, V>(C, A, X, rows, M, Kw, s, omul, osub);
    else if (per <= 16) launch_bmv<W, 16, V>(C, A, X, rows, M, Kw, s, omul, osub);
    else if (per <= 32) launch_bmv<W, 32, V>(C, A, X, rows, M, Kw, s, omul, osub);
    else launch_bmv<W, 64, V>(C, A, X, rows, M, Kw, s, omul, osub);
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
             const char *who, int omul = 1, int osub = 0)  // N == 1 only: the sums leave as sum * omul - osub
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
        const int64_t rowbytes = Kw * (int64_t)sizeof(W);
        if ((rowbytes == 16 || rowbytes == 32 || rowbytes == 64) && rows < (1LL << 31) && aligned(A, 16) &&
            aligned(B, 16)) {
            if (rowbytes == 16) launch_bmv_short<1>(C, A, B, rows, M, s, omul, osub);
            else if (rowbytes == 32) launch_bmv_short<2>(C, A, B, rows, M, s, omul, osub);
            else launch_bmv_short<4>(C, A, B, rows, M, s, omul, osub);
        } else if (rowbytes % 16 == 0 && rowbytes >= 256 && M % 4 == 0 && aligned(A, 16) && aligned(B, 16)) {
            const int rowvecs = (int)(rowbytes / 16);
            // as many row steps in flight as divide the row (up to 16 loads of 16 bytes per lane), fewest lanes per row
            if (rowvecs % 256 == 0) launch_bmv_quad<64, 4>(C, A, B, rows, M, rowvecs, s, nullptr, omul, osub);
            else if (rowvecs % 128 == 0) launch_bmv_quad<32, 4>(C, A, B, rows, M, rowvecs, s, nullptr, omul, osub);
            else if (rowvecs % 64 == 0) launch_bmv_quad<16, 4>(C, A, B, rows, M, rowvecs, s, nullptr, omul, osub);
            else if (rowvecs % 32 == 0) launch_bmv_quad<16, 2>(C, A, B, rows, M, rowvecs, s, nullptr, omul, osub);
            else if (rowvecs >= 64) launch_bmv_quad<64, 1>(C, A, B, rows, M, rowvecs, s, nullptr, omul, osub);
            else if (rowvecs >= 32) launch_bmv_quad<32, 1>(C, A, B, rows, M, rowvecs, s, nullptr, omul, osub);
            else launch_bmv_quad<16, 1>(C, A, B, rows, M, rowvecs, s, nullptr, omul, osub);
        } else if ((Kw & 1) == 0 && aligned(A, 2 * sizeof(W)) && aligned(B, 2 * sizeof(W)))
            dispatch_bmv<W, 2>(C, A, B, rows, M, (int)Kw, s, omul, osub);
        else
            dispatch_bmv<W, 1>(C, A, B, rows, M, (int)Kw, s, omul, osub);
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

template <typename W>
int bmv_act_pack_impl(W *out, const W *A, const W *X, const int32_t *thresh, int64_t Z, int64_t M, int64_t Kw,
                      nb_stream_t stream, const char *who)
{
    constexpr int bits = WordTraits<W>::bits;
    NB_REQUIRE(Z >= 0 && M >= 0 && Kw >= 0, "%s: negative shape Z=%lld M=%lld Kw=%lld", who, (long long)Z, (long long)M,
               (long long)Kw);
    if (Z * M == 0) return NB_OK;
    NB_REQUIRE_PTR(out);
    NB_REQUIRE_PTR(thresh);
    NB_REQUIRE_ALIGNED(out, sizeof(W));
    NB_REQUIRE_ALIGNED(thresh, 4);
    if (Kw > 0) {
        NB_REQUIRE_PTR(A);
        NB_REQUIRE_PTR(X);
        NB_REQUIRE_ALIGNED(A, sizeof(W));
        NB_REQUIRE_ALIGNED(X, sizeof(W));
    }
    NB_REQUIRE(Kw <= (1 << 24) && Z * M < (1LL << 40), "%s: Kw=%lld or Z*M=%lld too large", who, (long long)Kw,
               (long long)(Z * M));
    hipStream_t s = as_stream(stream);
    const int64_t rows = Z * M;
    const int64_t rowbytes = Kw * (int64_t)sizeof(W);
    const int64_t Mw = ceil_div(M, bits);
    NB_REQUIRE(ceil_div(Z * Mw, 4) <= kMaxGridX && ceil_div(ceil_div(rows, 4) * 64, 256) <= kMaxGridX,
               "%s: %lld rows exceed one launch", who, (long long)rows);
    if (rowbytes % 16 == 0 && rowbytes >= 256 && M % bits == 0 && aligned(A, 16) && aligned(X, 16)) {
        const int rowvecs = (int)(rowbytes / 16);
        int32_t *C = reinterpret_cast<int32_t *>(out);
        if (rowvecs % 256 == 0) launch_bmv_quad<64, 4>(C, A, X, rows, M, rowvecs, s, thresh);
        else if (rowvecs % 128 == 0) launch_bmv_quad<32, 4>(C, A, X, rows, M, rowvecs, s, thresh);
        else if (rowvecs % 64 == 0) launch_bmv_quad<16, 4>(C, A, X, rows, M, rowvecs, s, thresh);
        else if (rowvecs % 32 == 0) launch_bmv_quad<16, 2>(C, A, X, rows, M, rowvecs, s, thresh);
        else if (rowvecs >= 64) launch_bmv_quad<64, 1>(C, A, X, rows, M, rowvecs, s, thresh);
        else if (rowvecs >= 32) launch_bmv_quad<32, 1>(C, A, X, rows, M, rowvecs, s, thresh);
        else launch_bmv_quad<16, 1>(C, A, X, rows, M, rowvecs, s, thresh);
    } else {
        bmv_act_pack_generic_kernel<W><<<dim3((unsigned)ceil_div(Z * Mw, 4)), dim3(256), 0, s>>>(
            out, A, X, thresh, Z * Mw, M, (int)Mw, (int)Kw);
    }
    return check_launch(who);
}

}  // namespace nb

extern "C" {
int nb_bmv_act_pack_i64(int64_t *out, const int64_t *A, const int64_t *x, const int32_t *thresh, int64_t Z, int64_t M,
                        int64_t Kw, nb_stream_t s)
{
    return nb::bmv_act_pack_impl<uint64_t>(reinterpret_cast<uint64_t *>(out), reinterpret_cast<const uint64_t *>(A),
                                           reinterpret_cast<const uint64_t *>(x), thresh, Z, M, Kw, s,
                                           "nb_bmv_act_pack_i64");
}
int nb_bmv_act_pack_i32(int32_t *out, const int32_t *A, const int32_t *x, const int32_t *thresh, int64_t Z, int64_t M,
                        int64_t Kw, nb_stream_t s)
{
    return nb::bmv_act_pack_impl<uint32_t>(reinterpret_cast<uint32_t *>(out), reinterpret_cast<const uint32_t *>(A),
                                           reinterpret_cast<const uint32_t *>(x), thresh, Z, M, Kw, s,
                                           "nb_bmv_act_pack_i32");
}
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
int nb_bmv_pm1_i64(int32_t *C, const int64_t *A, const int64_t *x, int64_t Z, int64_t M, int64_t Kw, int64_t K,
                   nb_stream_t s)
{
    NB_REQUIRE(K >= 0 && K <= Kw * 64 && K < (1LL << 31), "nb_bmv_pm1_i64: K = %lld bits does not fit the rows' %lld words", (long long)K,
               (long long)Kw);
    if (Kw == 0) return nb::fail(NB_ERR_SHAPE, "nb_bmv_pm1_i64: empty rows");
    return nb::bmm_impl<uint64_t>(C, reinterpret_cast<const uint64_t *>(A), reinterpret_cast<const uint64_t *>(x), Z, M, Kw, 1, s,
                                  "nb_bmv_pm1_i64", 2, (int)K);
}
int nb_bmv_pm1_i32(int32_t *C, const int32_t *A, const int32_t *x, int64_t Z, int64_t M, int64_t Kw, int64_t K,
                   nb_stream_t s)
{
    NB_REQUIRE(K >= 0 && K <= Kw * 32 && K < (1LL << 31), "nb_bmv_pm1_i32: K = %lld bits does not fit the rows' %lld words", (long long)K,
               (long long)Kw);
    if (Kw == 0) return nb::fail(NB_ERR_SHAPE, "nb_bmv_pm1_i32: empty rows");
    return nb::bmm_impl<uint32_t>(C, reinterpret_cast<const uint32_t *>(A), reinterpret_cast<const uint32_t *>(x), Z, M, Kw, 1, s,
                                  "nb_bmv_pm1_i32", 2, (int)K);
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
