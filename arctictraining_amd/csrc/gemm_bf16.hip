// Ragged grouped GEMMs on bf16 MFMA (v_mfma_f32_32x32x16_bf16), f32 accumulate.
//
// One kernel template covers the three operand layouts of the expert FFN:
//   rows / NN   C[rows_e,:] = A[rows_e,:] @ B[e]        (forward; B is [Kd,N], N contiguous)
//   rows / NT   C[rows_e,:] = A[rows_e,:] @ B[e]^T      (data gradient; B is [N',Kd'] so both K-contiguous)
//   wgrad / TN  C[e] = A[rows_e,:]^T @ B[rows_e,:]      (weight gradient; the reduction runs over the ragged rows)
//
// Tiles of BM x BN x 32 move from global memory straight into LDS (global_load_lds, 16 bytes
// per lane, four stages in flight); the XOR swizzle of the LDS layout is applied on the source
// side.  Fragments are read back with
//   * ds_read_b128 when the operand is K-contiguous in LDS.  A 32-wide K row is 4 chunks of
//     16 bytes; chunk kc of row r sits at position kc ^ ((r >> 2) & 3), which makes the 32
//     rows a half-wave reads cover every group of 4 banks exactly twice and the 4 lanes of
//     each quad distinct groups: conflict-free on the 64-bank LDS of gfx950;
//   * eight ds_read_b32 + v_perm when it is K-strided: a dword holds two ADJACENT columns of
//     one k row, so one set of reads feeds a PAIR of MFMA tiles, one taking the even and one
//     the odd columns.  The pair's accumulators then hold (col 2j, col 2j+1) in the same lane
//     and register, which makes the stores packed 4-byte and lets the gated activation
//     (gate = even, up = odd column) run on registers in the epilogue.
//
// Row-grouped launches take their (expert, first row, end row) per M tile from a tile map
// that a small kernel builds on the device from the expert offsets: no host sync, empty
// experts simply own no tile.  Workgroups are dealt to the 8 XCDs so that the ~32 resident on
// one XCD cover one super-tile of gm x gn tiles (shared A and B panels in that XCD's L2),
// and super-tiles rotate over the XCDs, which keeps them evenly loaded whatever the routing
// skew.
#include "amoe_common.h"

#include <type_traits>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 mfma_bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float mfma_f32x16;

namespace {

constexpr int BK = 32;      // K extent of one LDS stage
constexpr int NSTAGE = 4;   // LDS stages in flight

struct GemmArgs {
    const bf16_t* A;
    const bf16_t* B;
    bf16_t* C;
    bf16_t* C2;
    const int32_t* a_row_map;
    const int32_t* b_row_map;  // weight gradient only
    const float* row_scale;  // gated epilogue: inter[r,:] is multiplied by row_scale[r] (null = 1)
    const int32_t* offsets;
    const int4* tile_map;
    const int32_t* n_mtiles;
    int lda, ldb, ldc, ldc2;
    long long strideB, strideC;
    int E;
    int Kd;       // rows mode: reduction length
    int M;        // wgrad mode: output rows per expert
    int N;        // output columns
    int n_ntiles;
    int n_mt;     // wgrad mode: M tiles per expert
    int rows_total;  // weight gradient: length of the row maps
    int gm, gn;   // blocks of one XCD work on super-tiles of gm x gn tiles
    int sn;       // super-tiles along N
};

enum { EPI_STORE = 0, EPI_GATED = 1 };

// tile map: one int4 {expert, first row, end row, 0} per M tile
__global__ void __launch_bounds__(512)
tile_map_kernel(const int32_t* __restrict__ offsets, int E, int bm, int4* __restrict__ tile_map,
                int32_t* __restrict__ n_mtiles, int max_mtiles)
{
    __shared__ int32_t start[AMOE_MAX_EXPERTS + 1];  // start[e] = first M tile of expert e
    __shared__ int32_t off[AMOE_MAX_EXPERTS + 1];
    const int e = threadIdx.x;  // 512 threads, one per possible expert
    int nt = 0;
    if (e < E) {
        int a = offsets[e], b = offsets[e + 1];
        off[e] = a;
        if (e == E - 1) off[E] = b;
        nt = (b - a + bm - 1) / bm;
    }
    start[e + 1] = nt;
    if (e == 0) start[0] = 0;
    __syncthreads();
    // inclusive Hillis-Steele scan of start[1..512]
    for (int o = 1; o < AMOE_MAX_EXPERTS; o <<= 1) {
        int add = (e >= o) ? start[e + 1 - o] : 0;
        __syncthreads();
        start[e + 1] += add;
        __syncthreads();
    }
    const int total = start[E];
    if (e == 0) *n_mtiles = total < max_mtiles ? total : max_mtiles;
    for (int mt = threadIdx.x; mt < total && mt < max_mtiles; mt += blockDim.x) {
        // largest ex with start[ex] <= mt
        int lo = 0, hi = E - 1;
        while (lo < hi) {
            int mid = (lo + hi + 1) >> 1;
            if (start[mid] <= mt) lo = mid; else hi = mid - 1;
        }
        int4 v;
        v.x = lo;
        v.y = off[lo] + (mt - start[lo]) * bm;
        v.z = off[lo + 1];
        v.w = 0;
        tile_map[mt] = v;
    }
}

__device__ __forceinline__ uint32_t perm_lo(uint32_t w1, uint32_t w0) { return __builtin_amdgcn_perm(w1, w0, 0x05040100u); }
__device__ __forceinline__ uint32_t perm_hi(uint32_t w1, uint32_t w0) { return __builtin_amdgcn_perm(w1, w0, 0x07060302u); }

// 16 zero bytes that masked lanes of a direct-to-LDS load read instead of out-of-range rows
__device__ __attribute__((aligned(16))) uint32_t g_zero_chunk[4] = {0u, 0u, 0u, 0u};

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// wave-level half of a workgroup barrier for LDS data: this wave's LDS reads have returned and
// all but N of its loads have landed; then the hardware barrier.  (No memory fence: LDS is not
// cached and the direct-to-LDS loads are tracked by vmcnt.)
template <int N>
__device__ __forceinline__ void lds_barrier()
{
    static_assert(N >= 0 && N <= 63, "vmcnt is 6 bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (0 << 8) | ((N >> 4) << 14));
    __builtin_amdgcn_s_barrier();
}
using T_ = std::true_type;
using F_ = std::false_type;

// MAPS (weight gradient only): 1 = the rows of A, 2 = the rows of B are gathered through a row map
template <int BM, int BN, int WGM, int WGN, bool A_KC, bool B_KC, int EPI, int ACT, int MAPS = 0>
__global__ void __launch_bounds__(WGM * WGN * 64)
grouped_gemm_bf16_kernel(GemmArgs p)
{
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr bool WGRAD = !A_KC;
    constexpr bool A_MAP = WGRAD && (MAPS & 1), B_MAP = WGRAD && (MAPS & 2);
    static_assert(WGRAD || MAPS == 0, "row-grouped launches gather through the per-thread row plan");
    static_assert(TN % 2 == 0, "N tiles come in even/odd pairs");
    static_assert(!WGRAD || (TM % 2 == 0 && !B_KC), "wgrad pairs both operands");
    static_assert(BM >= 128 && BN >= 128, "K-strided swizzle needs 16 chunks per row");
    constexpr int A_CH = BM * 4, B_CH = BN * 4;   // 16-byte chunks per stage (a 32-wide K row is 4 chunks)
    constexpr int STAGE = A_CH + B_CH;
    constexpr int PER_A = A_CH / NT, PER_B = B_CH / NT;
    static_assert(A_CH % NT == 0 && B_CH % NT == 0, "tile must split evenly over the block");

    extern __shared__ u32x4_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int lj = lane & 31, lg = lane >> 5;

    // ------------------------------------------------------------ block -> tile
    // Workgroups are dealt to the 8 XCDs round-robin.  The ~32 workgroups resident on one XCD
    // are made to cover one gm x gn super-tile, so its gm A panels and gn B panels are fetched
    // into that XCD's L2 once and shared; super-tiles themselves rotate over the XCDs.
    const int b = blockIdx.x;
    const int xcd = b & 7;
    const int q = b >> 3;
    const int per_super = p.gm * p.gn;
    const int sid = (q / per_super) * 8 + xcd;
    const int w = q % per_super;
    const int sm = sid / p.sn, sn_i = sid - sm * p.sn;
    const int pm = sm * p.gm + w / p.gn;
    const int nt = sn_i * p.gn + w % p.gn;
    if (nt >= p.n_ntiles) return;
    int e, m0, mend, kt_count;
    int r0 = 0, r1 = 0;
    if (!WGRAD) {
        if (pm >= *p.n_mtiles) return;
        int4 tm = p.tile_map[pm];
        e = tm.x;
        m0 = tm.y;
        mend = tm.z;
        kt_count = p.Kd / BK;
    } else {
        e = pm / p.n_mt;
        if (e >= p.E) return;
        m0 = (pm - e * p.n_mt) * BM;
        mend = p.M;
        r0 = p.offsets[e];
        r1 = p.offsets[e + 1];
        kt_count = (r1 - r0 + BK - 1) / BK;
    }
    const int n0 = nt * BN;

    // ------------------------------------------------------------ global load plans
    // Loads go straight from global memory into LDS: lane l of a wave fills the 16-byte chunk
    // (wave's base + l), so chunk c = tid + NT*i of a stage is filled by thread tid in its i-th
    // load.  The XOR swizzle of the LDS layout is applied on the SOURCE side: the thread that
    // fills physical chunk c fetches the logical chunk that belongs there.
    uint32_t aoff[PER_A], boff[PER_B];
    int a_kr[PER_A], b_kr[PER_B];  // wgrad: k row of the chunk, for the ragged-end mask
    const bf16_t* Ab = p.A;
    const bf16_t* Bb = p.B;
#pragma unroll
    for (int i = 0; i < PER_A; ++i) {
        const int c = tid + NT * i;
        if (A_KC) {
            const int row = c >> 2, kc = (c & 3) ^ ((row >> 2) & 3);
            int gr = min(m0 + row, mend - 1);
            if (p.a_row_map) gr = p.a_row_map[gr];
            aoff[i] = (uint32_t)gr * (uint32_t)p.lda + kc * 8;
            a_kr[i] = 0;
        } else {
            constexpr int CPR = BM / 8;
            const int krow = c / CPR, mc = (c % CPR) ^ (((krow >> 3) & 1) << 3);
            const int col = min(m0 + mc * 8, p.M - 8);
            aoff[i] = A_MAP ? (uint32_t)col : (uint32_t)krow * (uint32_t)p.lda + col;
            a_kr[i] = krow;
        }
    }
#pragma unroll
    for (int i = 0; i < PER_B; ++i) {
        const int c = tid + NT * i;
        if (B_KC) {
            // LDS row slot s of a 64-row block holds column 2*(s%32) + s/32 of that block, so the
            // even columns (one MFMA tile) and the odd columns (its partner) are each 32
            // consecutive LDS rows
            const int row = c >> 2, kc = (c & 3) ^ ((row >> 2) & 3);
            const int gn = min(n0 + (row & ~63) + 2 * (row & 31) + ((row >> 5) & 1), p.N - 1);
            boff[i] = (uint32_t)gn * (uint32_t)p.ldb + kc * 8;
            b_kr[i] = 0;
        } else {
            constexpr int CPR = BN / 8;
            const int krow = c / CPR, nc = (c % CPR) ^ (((krow >> 3) & 1) << 3);
            const int col = min(n0 + nc * 8, p.N - 8);
            boff[i] = B_MAP ? (uint32_t)col : (uint32_t)krow * (uint32_t)p.ldb + col;
            b_kr[i] = krow;
        }
    }
    if (!WGRAD) {
        Bb += (long long)e * p.strideB;
    } else {
        if (!A_MAP) Ab += (long long)r0 * p.lda;
        if (!B_MAP) Bb += (long long)r0 * p.ldb;
    }
    const int k_rows = r1 - r0;  // wgrad: rows of this expert

    // Gathered operands of the weight gradient: the source row of a chunk changes with every K
    // tile, so it is looked up one tile ahead (a_nxt / b_nxt, fetched right before the loads of
    // the previous tile are issued) and moved to a_use / b_use when its own loads go out.
    int a_use[PER_A], a_nxt[PER_A], b_use[PER_B], b_nxt[PER_B];
    auto fetch_a_idx = [&](int kt, int (&dst)[PER_A]) {
#pragma unroll
        for (int i = 0; i < PER_A; ++i) dst[i] = p.a_row_map[min(r0 + kt * BK + a_kr[i], p.rows_total - 1)];
    };
    auto fetch_b_idx = [&](int kt, int (&dst)[PER_B]) {
#pragma unroll
        for (int i = 0; i < PER_B; ++i) dst[i] = p.b_row_map[min(r0 + kt * BK + b_kr[i], p.rows_total - 1)];
    };

    // wgrad: rows past the end of the expert read a block of zeros instead (only the last K
    // tile of an expert can be ragged, the select costs two VALU ops per load)
    auto dma_a = [&](int kt, auto LO, auto HI, const int (&idx)[PER_A]) {
        constexpr int lo = decltype(LO)::value, hi = decltype(HI)::value;
        const int k0 = kt * BK;
        u32x4_t* sa = smem + (kt & (NSTAGE - 1)) * STAGE + wave * 64;
        const bf16_t* a_base = A_KC ? Ab + k0 : (A_MAP ? Ab : Ab + (long long)k0 * p.lda);
#pragma unroll
        for (int i = lo; i < hi; ++i) {
            const bf16_t* src = a_base + aoff[i];
            if (A_MAP) src += (long long)idx[i] * p.lda;
            if (WGRAD) src = (k0 + a_kr[i] < k_rows) ? src : reinterpret_cast<const bf16_t*>(g_zero_chunk);
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(sa + NT * i), 16, 0, 0);
        }
    };
    auto dma_b = [&](int kt, auto LO, auto HI, const int (&idx)[PER_B]) {
        constexpr int lo = decltype(LO)::value, hi = decltype(HI)::value;
        const int k0 = kt * BK;
        u32x4_t* sb = smem + (kt & (NSTAGE - 1)) * STAGE + A_CH + wave * 64;
        const bf16_t* b_base = B_KC ? Bb + k0 : (B_MAP ? Bb : Bb + (long long)k0 * p.ldb);
#pragma unroll
        for (int i = lo; i < hi; ++i) {
            const bf16_t* src = b_base + boff[i];
            if (B_MAP) src += (long long)idx[i] * p.ldb;
            if (WGRAD) src = (k0 + b_kr[i] < k_rows) ? src : reinterpret_cast<const bf16_t*>(g_zero_chunk);
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(sb + NT * i), 16, 0, 0);
        }
    };
    // steady-state issue: rotate the looked-up rows when the first half of a tile goes out
    auto issue_a = [&](int kt, auto LO, auto HI) {
        if (A_MAP && decltype(LO)::value == 0) {
#pragma unroll
            for (int i = 0; i < PER_A; ++i) a_use[i] = a_nxt[i];
            fetch_a_idx(kt + 1, a_nxt);
        }
        dma_a(kt, LO, HI, a_use);
    };
    auto issue_b = [&](int kt, auto LO, auto HI) {
        if (B_MAP && decltype(LO)::value == 0) {
#pragma unroll
            for (int i = 0; i < PER_B; ++i) b_use[i] = b_nxt[i];
            fetch_b_idx(kt + 1, b_nxt);
        }
        dma_b(kt, LO, HI, b_use);
    };

    mfma_f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // ------------------------------------------------------------ fragment readers
    // "raw" fragments are what comes out of LDS: for a K-contiguous operand the MFMA operand
    // itself, for a K-strided operand eight dwords per tile pair still to be split by v_perm.
    constexpr int RAW_A = A_KC ? TM : TM * 2;   // u32x4 registers
    constexpr int RAW_B = B_KC ? TN : TN * 2;
    auto read_a = [&](const u32x4_t* sa, int ks, u32x4_t (&ra)[RAW_A]) {
        if (A_KC) {
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                const int row = wm * WTM + t * 32 + lj;
                const int kc = ks * 2 + lg;
                ra[t] = sa[row * 4 + (kc ^ ((row >> 2) & 3))];
            }
        } else {
            constexpr int CPR = BM / 8;
            const uint32_t* sw = reinterpret_cast<const uint32_t*>(sa);
#pragma unroll
            for (int pr = 0; pr < TM / 2; ++pr) {
                const int word = (wm * WTM + pr * 64) / 2 + lj;
                const int chunk = (word >> 2) ^ (lg << 3);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int krow = ks * 16 + lg * 8 + i;
                    ra[pr * 2 + (i >> 2)][i & 3] = sw[(krow * CPR + chunk) * 4 + (word & 3)];
                }
            }
        }
    };
    auto read_b = [&](const u32x4_t* sb, int ks, u32x4_t (&rb)[RAW_B]) {
        if (B_KC) {
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                const int row = wn * WTN + t * 32 + lj;
                const int kc = ks * 2 + lg;
                rb[t] = sb[row * 4 + (kc ^ ((row >> 2) & 3))];
            }
        } else {
            constexpr int CPR = BN / 8;
            const uint32_t* sw = reinterpret_cast<const uint32_t*>(sb);
#pragma unroll
            for (int pr = 0; pr < TN / 2; ++pr) {
                const int word = (wn * WTN + pr * 64) / 2 + lj;
                const int chunk = (word >> 2) ^ (lg << 3);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int krow = ks * 16 + lg * 8 + i;
                    rb[pr * 2 + (i >> 2)][i & 3] = sw[(krow * CPR + chunk) * 4 + (word & 3)];
                }
            }
        }
    };
    // raw -> MFMA operands (identity for K-contiguous operands)
    auto to_frag_pair = [&](const u32x4_t& w03, const u32x4_t& w47, mfma_bf16x8& even, mfma_bf16x8& odd) {
        u32x4_t lo = {perm_lo(w03[1], w03[0]), perm_lo(w03[3], w03[2]), perm_lo(w47[1], w47[0]), perm_lo(w47[3], w47[2])};
        u32x4_t hi = {perm_hi(w03[1], w03[0]), perm_hi(w03[3], w03[2]), perm_hi(w47[1], w47[0]), perm_hi(w47[3], w47[2])};
        even = __builtin_bit_cast(mfma_bf16x8, lo);
        odd = __builtin_bit_cast(mfma_bf16x8, hi);
    };
    auto make_fa = [&](const u32x4_t (&ra)[RAW_A], mfma_bf16x8 (&fa)[TM]) {
        if (A_KC) {
#pragma unroll
            for (int t = 0; t < TM; ++t) fa[t] = __builtin_bit_cast(mfma_bf16x8, ra[t]);
        } else {
#pragma unroll
            for (int pr = 0; pr < TM / 2; ++pr) to_frag_pair(ra[2 * pr], ra[2 * pr + 1], fa[2 * pr], fa[2 * pr + 1]);
        }
    };
    auto make_fb = [&](const u32x4_t (&rb)[RAW_B], mfma_bf16x8 (&fb)[TN]) {
        if (B_KC) {
#pragma unroll
            for (int t = 0; t < TN; ++t) fb[t] = __builtin_bit_cast(mfma_bf16x8, rb[t]);
        } else {
#pragma unroll
            for (int pr = 0; pr < TN / 2; ++pr) to_frag_pair(rb[2 * pr], rb[2 * pr + 1], fb[2 * pr], fb[2 * pr + 1]);
        }
    };
    // quarter Q of a K step's MFMAs (A tile outer, B tile inner)
    constexpr int N_MFMA = TM * TN;
    static_assert(N_MFMA % 4 == 0, "a K step is issued in four chunks");
    auto mma_quarter = [&](const mfma_bf16x8 (&fa)[TM], const mfma_bf16x8 (&fb)[TN], auto Q) {
        constexpr int q = decltype(Q)::value;
#pragma unroll
        for (int f = q * (N_MFMA / 4); f < (q + 1) * (N_MFMA / 4); ++f) {
            const int i = f / TN, j = f % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    };

    // ------------------------------------------------------------ main loop
    // NSTAGE = 4 LDS stages of one 32-wide K tile each (two MFMA K steps).  Iteration j works
    // on tile j (stage j % 4):
    //   step A: MFMAs on the ks=0 fragments | fetch the ks=1 fragments of tile j
    //           | issue the B half of the loads of tile j+3
    //   wait until tile j+1 has landed (the loads of tiles j+2, j+3 may stay in flight), barrier:
    //           tile j+1 is visible and stage j % 4 is free (every wave holds its last fragments)
    //   step B: MFMAs on the ks=1 fragments | fetch the ks=0 fragments of tile j+1
    //           | issue the A half of the loads of tile j+4 into the stage just freed
    // so the direct-to-LDS loads trickle out evenly (the L1 path moves 64 bytes a clock, half of
    // what the MFMAs consume at full rate) and each has about two iterations to land.
    // A step is written as four chunks fenced by scheduling barriers, each pairing a quarter of
    // the MFMAs with one kind of side work: A-fragment reads, B-fragment reads, loads, loads +
    // the v_perm splitting of K-strided fragments for the next step.
    constexpr int PER = PER_A + PER_B;
    static_assert(2 * PER + PER_A <= 63, "vmcnt is a 6-bit counter");
    using IC0 = std::integral_constant<int, 0>;
    using IC1 = std::integral_constant<int, 1>;
    using IC2 = std::integral_constant<int, 2>;
    using IC3 = std::integral_constant<int, 3>;
    using A_HALF = std::integral_constant<int, (PER_A + 1) / 2>;
    using A_ALL = std::integral_constant<int, PER_A>;
    using B_HALF = std::integral_constant<int, (PER_B + 1) / 2>;
    using B_ALL = std::integral_constant<int, PER_B>;
    u32x4_t ra[RAW_A], rb[RAW_B];
    mfma_bf16x8 fa0[TM], fb0[TN], fa1[TM], fb1[TN];

    // prologue: tiles 0..2 and the A half of tile 3 go out, tile 0 is awaited
    {
        // row lookups of the first four tiles go out together, ahead of their loads
        int ia[NSTAGE][PER_A], ib[NSTAGE][PER_B];
#pragma unroll
        for (int t = 0; t < NSTAGE; ++t) {
            if (A_MAP) fetch_a_idx(t, ia[t]);
            if (B_MAP) fetch_b_idx(t, ib[t]);
        }
#pragma unroll
        for (int t = 0; t < NSTAGE - 1; ++t) {
            if (t < kt_count) {
                dma_a(t, IC0{}, A_ALL{}, ia[t]);
                dma_b(t, IC0{}, B_ALL{}, ib[t]);
            }
        }
        if (kt_count > NSTAGE - 1) dma_a(NSTAGE - 1, IC0{}, A_ALL{}, ia[NSTAGE - 1]);
        if (A_MAP) fetch_a_idx(NSTAGE, a_nxt);          // next A tile to go out is tile 4
        if (B_MAP) {
#pragma unroll
            for (int i = 0; i < PER_B; ++i) b_nxt[i] = ib[NSTAGE - 1][i];  // next B tile is tile 3
        }
    }
    if (kt_count > NSTAGE - 1) {
        lds_barrier<2 * PER + PER_A>();
    } else {
        lds_barrier<0>();
    }
    if (kt_count > 0) {
        read_a(smem, 0, ra);
        read_b(smem + A_CH, 0, rb);
        make_fa(ra, fa0);
        make_fb(rb, fb0);
    }
    __builtin_amdgcn_sched_barrier(0);

    // LOAD_B: tile kt+3 exists; LOAD_A: tile kt+4 exists; WAITN: loads younger than tile kt+1
    auto k_tile = [&](auto LOAD_B, auto LOAD_A, auto WAITN, auto NEXT, int kt) {
        constexpr bool load_b = decltype(LOAD_B)::value, load_a = decltype(LOAD_A)::value;
        constexpr bool next = decltype(NEXT)::value;
        constexpr int waitn = decltype(WAITN)::value;
        const u32x4_t* sa = smem + (kt & (NSTAGE - 1)) * STAGE;
        const u32x4_t* sb = sa + A_CH;
        // ---- step A: MFMAs on (fa0, fb0)
        read_a(sa, 1, ra);
        mma_quarter(fa0, fb0, IC0{});
        __builtin_amdgcn_sched_barrier(0);
        read_b(sb, 1, rb);
        mma_quarter(fa0, fb0, IC1{});
        __builtin_amdgcn_sched_barrier(0);
        if (load_b) issue_b(kt + 3, IC0{}, B_HALF{});
        mma_quarter(fa0, fb0, IC2{});
        __builtin_amdgcn_sched_barrier(0);
        if (load_b) issue_b(kt + 3, B_HALF{}, B_ALL{});
        make_fa(ra, fa1);
        make_fb(rb, fb1);
        mma_quarter(fa0, fb0, IC3{});
        __builtin_amdgcn_sched_barrier(0);
        lds_barrier<waitn>();
        __builtin_amdgcn_sched_barrier(0);
        // ---- step B: MFMAs on (fa1, fb1)
        const u32x4_t* na = smem + ((kt + 1) & (NSTAGE - 1)) * STAGE;
        if (next) read_a(na, 0, ra);
        mma_quarter(fa1, fb1, IC0{});
        __builtin_amdgcn_sched_barrier(0);
        if (next) read_b(na + A_CH, 0, rb);
        mma_quarter(fa1, fb1, IC1{});
        __builtin_amdgcn_sched_barrier(0);
        if (load_a) issue_a(kt + 4, IC0{}, A_HALF{});
        mma_quarter(fa1, fb1, IC2{});
        __builtin_amdgcn_sched_barrier(0);
        if (load_a) issue_a(kt + 4, A_HALF{}, A_ALL{});
        if (next) {
            make_fa(ra, fa0);
            make_fb(rb, fb0);
        }
        mma_quarter(fa1, fb1, IC3{});
        __builtin_amdgcn_sched_barrier(0);
    };
    {
        using W0 = std::integral_constant<int, 0>;
        using W1 = std::integral_constant<int, PER>;
        using W2 = std::integral_constant<int, 2 * PER>;
        int kt = 0;
        for (; kt + 4 < kt_count; ++kt) k_tile(T_{}, T_{}, W2{}, T_{}, kt);
        if (kt + 4 == kt_count) { k_tile(T_{}, F_{}, W2{}, T_{}, kt); ++kt; }
        if (kt + 3 == kt_count) { k_tile(F_{}, F_{}, W1{}, T_{}, kt); ++kt; }
        if (kt + 2 == kt_count) { k_tile(F_{}, F_{}, W0{}, T_{}, kt); ++kt; }
        if (kt + 1 == kt_count) k_tile(F_{}, F_{}, W0{}, F_{}, kt);
    }

    // ------------------------------------------------------------ epilogue
    if (!WGRAD) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * WTM + i * 32 + 8 * (v >> 2) + 4 * lg + (v & 3);
                if (row >= mend) continue;
                float rs = 1.0f;
                if (EPI == EPI_GATED && p.row_scale) rs = p.row_scale[row];
#pragma unroll
                for (int pr = 0; pr < TN / 2; ++pr) {
                    const int col = n0 + wn * WTN + pr * 64 + 2 * lj;
                    if (col >= p.N) continue;
                    const uint32_t packed = pack_bf16x2(acc[i][2 * pr][v], acc[i][2 * pr + 1][v]);
                    if (EPI == EPI_GATED) {
                        if (p.C) *reinterpret_cast<uint32_t*>(p.C + (size_t)row * p.ldc + col) = packed;
                        const float gte = bf16_lo(packed), up = bf16_hi(packed);
                        p.C2[(size_t)row * p.ldc2 + (col >> 1)] = (bf16_t)(rs * up * act_fwd<ACT>(gte));
                    } else {
                        *reinterpret_cast<uint32_t*>(p.C + (size_t)row * p.ldc + col) = packed;
                    }
                }
            }
        }
    } else {
        bf16_t* Ce = p.C + (long long)e * p.strideC;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * WTM + (i >> 1) * 64 + 2 * (8 * (v >> 2) + 4 * lg + (v & 3)) + (i & 1);
                if (row >= p.M) continue;
#pragma unroll
                for (int pr = 0; pr < TN / 2; ++pr) {
                    const int col = n0 + wn * WTN + pr * 64 + 2 * lj;
                    if (col >= p.N) continue;
                    *reinterpret_cast<uint32_t*>(Ce + (size_t)row * p.ldc + col) =
                        pack_bf16x2(acc[i][2 * pr][v], acc[i][2 * pr + 1][v]);
                }
            }
        }
    }
}

// ------------------------------------------------------------------ host side
template <int BM, int BN, int WGM, int WGN, bool A_KC, bool B_KC, int EPI, int ACT, int MAPS = 0>
int launch_cfg(const GemmArgs& a, int grid, hipStream_t s)
{
    auto kern = grouped_gemm_bf16_kernel<BM, BN, WGM, WGN, A_KC, B_KC, EPI, ACT, MAPS>;
    constexpr int lds_bytes = NSTAGE * (BM + BN) * BK * 2;
    static bool attr_done = false;
    if (!attr_done) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (err != hipSuccess) {
            amoe_set_error("grouped_gemm: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(err));
            return AMOE_ERR_LAUNCH;
        }
        attr_done = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WGM * WGN * 64), lds_bytes, s, a);
    return amoe_check_launch("grouped_gemm_bf16");
}

struct TileCfg {
    int bm, bn;
};

inline TileCfg pick_cfg(int tile_cfg)
{
    switch (tile_cfg) {
        case 1: return {128, 128};
        case 2: return {256, 128};
        case 3: return {256, 256};
        case 5: return {256, 256};
        default: return {256, 256};
    }
}

template <bool A_KC, bool B_KC, int EPI, int ACT, int MAPS = 0>
int launch_any(const GemmArgs& a, int tile_cfg, int grid, hipStream_t s)
{
    switch (tile_cfg) {
        case 1: return launch_cfg<128, 128, 2, 2, A_KC, B_KC, EPI, ACT, MAPS>(a, grid, s);
        case 3: return launch_cfg<256, 256, 2, 2, A_KC, B_KC, EPI, ACT, MAPS>(a, grid, s);
        case 5: return launch_cfg<256, 256, 4, 2, A_KC, B_KC, EPI, ACT, MAPS>(a, grid, s);
        case 2: return launch_cfg<256, 128, 2, 2, A_KC, B_KC, EPI, ACT, MAPS>(a, grid, s);
        default: return launch_cfg<256, 256, 2, 4, A_KC, B_KC, EPI, ACT, MAPS>(a, grid, s);  // 8 waves, 128x64 per wave
    }
}

}  // namespace

// super-tile shape and grid size for `m_tiles` (upper bound) x `n_ntiles` tiles
static int set_supertiles(GemmArgs& a, long long m_tiles, long long* grid)
{
    a.gn = a.n_ntiles < 8 ? a.n_ntiles : 8;
    a.gm = 32 / a.gn;
    a.sn = (a.n_ntiles + a.gn - 1) / a.gn;
    const long long sm = (m_tiles + a.gm - 1) / a.gm;
    const long long supers = sm * a.sn;
    *grid = 8 * ((supers + 7) / 8) * a.gm * a.gn;
    AMOE_REQUIRE(*grid < (1ll << 31), AMOE_ERR_UNSUPPORTED, "grouped_gemm: grid too large");
    return AMOE_OK;
}

// workspace: [0,16) tile count, then one int4 per M tile for the smallest tile height (64)
static inline int ws_max_mtiles(int R, int E, int bm) { return R / bm + E + 1; }

AMOE_EXPORT size_t amoe_grouped_gemm_workspace_bytes(int R, int E)
{
    if (R <= 0 || E <= 0) return 0;
    return 16 + sizeof(int4) * (size_t)ws_max_mtiles(R, E, 64);
}

int amoe_build_tile_map(const int32_t* offsets, int R, int E, int bm, void* workspace, size_t workspace_bytes,
                        const int4** tile_map, const int32_t** n_mtiles, int* max_mtiles, hipStream_t s)
{
    AMOE_REQUIRE(workspace_bytes >= amoe_grouped_gemm_workspace_bytes(R, E), AMOE_ERR_WORKSPACE,
                 "grouped_gemm: workspace %zu < %zu bytes", workspace_bytes, amoe_grouped_gemm_workspace_bytes(R, E));
    int32_t* cnt = (int32_t*)workspace;
    int4* map = (int4*)((char*)workspace + 16);
    *max_mtiles = ws_max_mtiles(R, E, bm);
    hipLaunchKernelGGL(tile_map_kernel, dim3(1), dim3(512), 0, s, offsets, E, bm, map, cnt, *max_mtiles);
    *tile_map = map;
    *n_mtiles = cnt;
    return amoe_check_launch("tile_map");
}

// rows mode driver shared by the three row-grouped entry points
template <bool B_KC, int EPI, int ACT>
static int run_rows_bf16(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C,
                         void* C2, const float* row_scale, int R, int E, int Kred, int N, int ldb, long long strideB, void* workspace,
                         size_t workspace_bytes, int tile_cfg, hipStream_t s)
{
    TileCfg tc = pick_cfg(tile_cfg);
    GemmArgs a = {};
    int max_mtiles = 0;
    int rc = amoe_build_tile_map(offsets, R, E, tc.bm, workspace, workspace_bytes, &a.tile_map, &a.n_mtiles,
                                 &max_mtiles, s);
    if (rc) return rc;
    a.A = (const bf16_t*)A;
    a.B = (const bf16_t*)B;
    a.C = (bf16_t*)C;
    a.C2 = (bf16_t*)C2;
    a.a_row_map = a_row_map;
    a.row_scale = row_scale;
    a.offsets = offsets;
    a.lda = Kred;
    a.ldb = ldb;
    a.ldc = N;
    a.ldc2 = N / 2;
    a.strideB = strideB;
    a.strideC = 0;
    a.E = E;
    a.Kd = Kred;
    a.M = R;
    a.N = N;
    a.n_ntiles = (N + tc.bn - 1) / tc.bn;
    a.n_mt = 0;
    long long grid = 0;
    rc = set_supertiles(a, max_mtiles, &grid);
    if (rc) return rc;
    return launch_any<true, B_KC, EPI, ACT>(a, tile_cfg, (int)grid, s);
}

int amoe_bf16_gateup_act(const void* xp, const int32_t* a_row_map, const void* w, const int32_t* offsets, void* gate_up,
                         void* inter, const float* row_scale, int R, int E, int H, int I, int act, void* workspace, size_t workspace_bytes,
                         int tile_cfg, hipStream_t s)
{
    AMOE_DISPATCH_ACT(act, return (run_rows_bf16<false, EPI_GATED, ACT>(xp, a_row_map, w, offsets, gate_up, inter, row_scale, R, E, H,
                                                                        2 * I, 2 * I, (long long)H * 2 * I, workspace,
                                                                        workspace_bytes, tile_cfg, s)))
    return AMOE_ERR_BAD_ARG;
}

int amoe_bf16_nn(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C, int R, int E,
                 int Kd, int N, void* workspace, size_t workspace_bytes, int tile_cfg, hipStream_t s)
{
    return run_rows_bf16<false, EPI_STORE, 0>(A, a_row_map, B, offsets, C, nullptr, nullptr, R, E, Kd, N, N, (long long)Kd * N,
                                              workspace, workspace_bytes, tile_cfg, s);
}

// C[rows_e, :Kd] = A[rows_e, :N] @ B[e]^T with B [E, Kd, N]: the reduction runs over N
int amoe_bf16_nt(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C, int R, int E,
                 int Kd, int N, void* workspace, size_t workspace_bytes, int tile_cfg, hipStream_t s)
{
    return run_rows_bf16<true, EPI_STORE, 0>(A, a_row_map, B, offsets, C, nullptr, nullptr, R, E, /*Kred=*/N, /*N out=*/Kd,
                                             /*ldb=*/N, (long long)Kd * N, workspace, workspace_bytes, tile_cfg, s);
}

int amoe_bf16_wgrad(const void* A, const int32_t* a_row_map, const void* B, const int32_t* b_row_map,
                    const int32_t* offsets, void* C, int R, int E, int Kd, int N, int tile_cfg, hipStream_t s)
{
    TileCfg tc = pick_cfg(tile_cfg);
    GemmArgs a = {};
    a.A = (const bf16_t*)A;
    a.B = (const bf16_t*)B;
    a.C = (bf16_t*)C;
    a.a_row_map = a_row_map;
    a.b_row_map = b_row_map;
    a.rows_total = R;
    a.offsets = offsets;
    a.lda = Kd;
    a.ldb = N;
    a.ldc = N;
    a.strideC = (long long)Kd * N;
    a.E = E;
    a.M = Kd;
    a.N = N;
    a.n_ntiles = (N + tc.bn - 1) / tc.bn;
    a.n_mt = (Kd + tc.bm - 1) / tc.bm;
    long long grid = 0;
    int rc = set_supertiles(a, (long long)E * a.n_mt, &grid);
    if (rc) return rc;
    if (a_row_map) return launch_any<false, false, EPI_STORE, 0, 1>(a, tile_cfg, (int)grid, s);
    if (b_row_map) return launch_any<false, false, EPI_STORE, 0, 2>(a, tile_cfg, (int)grid, s);
    return launch_any<false, false, EPI_STORE, 0>(a, tile_cfg, (int)grid, s);
}
