// Ragged grouped GEMMs on bf16 MFMA (v_mfma_f32_32x32x16_bf16), f32 accumulate.
//
// One kernel template covers the three operand layouts of the expert FFN:
//   rows / NN   C[rows_e,:] = A[rows_e,:] @ B[e]        (forward; B is [Kd,N], N contiguous)
//   rows / NT   C[rows_e,:] = A[rows_e,:] @ B[e]^T      (data gradient; B is [N',Kd'] so both K-contiguous)
//   wgrad / TN  C[e] = A[rows_e,:]^T @ B[rows_e,:]      (weight gradient; the reduction runs over the ragged rows)
//
// Tiles of BM x BN x 64 are staged through LDS (double buffered, one barrier per K step) by
// 16-byte global loads; fragments are read back with
//   * ds_read_b128 when the operand is K-contiguous in LDS (XOR-swizzled 16-byte chunks), or
//   * eight ds_read_b32 + v_perm when it is K-strided: a dword holds two ADJACENT columns of
//     one k row, so one set of reads feeds a PAIR of MFMA tiles, one taking the even and one
//     the odd columns.  The pair's accumulators then hold (col 2j, col 2j+1) in the same lane
//     and register, which makes the stores packed 4-byte and lets the gated activation
//     (gate = even, up = odd column) run on registers in the epilogue.
//
// Row-grouped launches take their (expert, first row, end row) per M tile from a tile map
// that a small kernel builds on the device from the expert offsets: no host sync, empty
// experts simply own no tile.  Blocks are dealt to the 8 XCDs so that all N tiles of one M
// tile run on the same XCD (shared A rows and expert weights in that XCD's L2) while
// consecutive M tiles rotate over XCDs, which keeps the XCDs evenly loaded whatever the
// routing skew.
#include "amoe_common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 mfma_bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float mfma_f32x16;

namespace {

constexpr int BK = 64;

struct GemmArgs {
    const bf16_t* A;
    const bf16_t* B;
    bf16_t* C;
    bf16_t* C2;
    const int32_t* a_row_map;
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

template <int BM, int BN, int WGM, int WGN, bool A_KC, bool B_KC, int EPI, int ACT>
__global__ void __launch_bounds__(WGM * WGN * 64)
grouped_gemm_bf16_kernel(GemmArgs p)
{
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr bool WGRAD = !A_KC;
    static_assert(TN % 2 == 0, "N tiles come in even/odd pairs");
    static_assert(!WGRAD || (TM % 2 == 0 && !B_KC), "wgrad pairs both operands");
    static_assert(BM >= 128 && BN >= 128, "K-strided swizzle needs 16 chunks per row");
    constexpr int A_CH = BM * 8, B_CH = BN * 8;   // 16-byte chunks per stage
    constexpr int PER_A = A_CH / NT, PER_B = B_CH / NT;
    static_assert(A_CH % NT == 0 && B_CH % NT == 0, "tile must split evenly over the block");

    extern __shared__ u32x4_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int lj = lane & 31, lg = lane >> 5;

    // ------------------------------------------------------------ block -> tile
    const int b = blockIdx.x;
    const int xcd = b & 7;
    const int q = b >> 3;
    const int grp = q / p.n_ntiles;
    const int nt = q - grp * p.n_ntiles;
    const int pm = grp * 8 + xcd;
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
    uint32_t aoff[PER_A], boff[PER_B];
    int a_lds[PER_A], b_lds[PER_B];
    int a_kr[PER_A], b_kr[PER_B];  // wgrad: k row of the chunk, for the ragged-end mask
    const bf16_t* Ab = p.A;
    const bf16_t* Bb = p.B;
#pragma unroll
    for (int i = 0; i < PER_A; ++i) {
        const int c = tid + NT * i;
        if (A_KC) {
            const int row = c >> 3, kc = c & 7;
            int gr = min(m0 + row, mend - 1);
            if (p.a_row_map) gr = p.a_row_map[gr];
            aoff[i] = (uint32_t)gr * (uint32_t)p.lda + kc * 8;
            a_lds[i] = row * 8 + (kc ^ (row & 7));
            a_kr[i] = 0;
        } else {
            constexpr int CPR = BM / 8;
            const int krow = c / CPR, mc = c % CPR;
            const int col = min(m0 + mc * 8, p.M - 8);
            aoff[i] = (uint32_t)krow * (uint32_t)p.lda + col;
            a_lds[i] = krow * CPR + (mc ^ (((krow >> 3) & 1) << 3));
            a_kr[i] = krow;
        }
    }
#pragma unroll
    for (int i = 0; i < PER_B; ++i) {
        const int c = tid + NT * i;
        if (B_KC) {
            const int row = c >> 3, kc = c & 7;
            const int gn = min(n0 + row, p.N - 1);
            boff[i] = (uint32_t)gn * (uint32_t)p.ldb + kc * 8;
            b_lds[i] = row * 8 + (kc ^ ((row >> 1) & 7));
            b_kr[i] = 0;
        } else {
            constexpr int CPR = BN / 8;
            const int krow = c / CPR, nc = c % CPR;
            const int col = min(n0 + nc * 8, p.N - 8);
            boff[i] = (uint32_t)krow * (uint32_t)p.ldb + col;
            b_lds[i] = krow * CPR + (nc ^ (((krow >> 3) & 1) << 3));
            b_kr[i] = krow;
        }
    }
    if (!WGRAD) {
        Bb += (long long)e * p.strideB;
    } else {
        Ab += (long long)r0 * p.lda;
        Bb += (long long)r0 * p.ldb;
    }
    const int k_rows = r1 - r0;  // wgrad: rows of this expert

    u32x4_t ra[PER_A], rb[PER_B];
    auto load_global = [&](int kt) {
        const int k0 = kt * BK;
#pragma unroll
        for (int i = 0; i < PER_A; ++i) {
            if (A_KC) {
                ra[i] = *reinterpret_cast<const u32x4_t*>(Ab + aoff[i] + k0);
            } else {
                const bool ok = k0 + a_kr[i] < k_rows;
                const bf16_t* src = Ab + (ok ? aoff[i] + (uint32_t)k0 * (uint32_t)p.lda : 0u);
                u32x4_t v = *reinterpret_cast<const u32x4_t*>(ok ? src : p.A);
                u32x4_t z = {0u, 0u, 0u, 0u};
                ra[i] = ok ? v : z;
            }
        }
#pragma unroll
        for (int i = 0; i < PER_B; ++i) {
            if (B_KC) {
                rb[i] = *reinterpret_cast<const u32x4_t*>(Bb + boff[i] + k0);
            } else if (!WGRAD) {
                rb[i] = *reinterpret_cast<const u32x4_t*>(Bb + boff[i] + (uint32_t)k0 * (uint32_t)p.ldb);
            } else {
                const bool ok = k0 + b_kr[i] < k_rows;
                const bf16_t* src = Bb + (ok ? boff[i] + (uint32_t)k0 * (uint32_t)p.ldb : 0u);
                u32x4_t v = *reinterpret_cast<const u32x4_t*>(ok ? src : p.B);
                u32x4_t z = {0u, 0u, 0u, 0u};
                rb[i] = ok ? v : z;
            }
        }
    };
    auto store_lds = [&](int buf) {
        u32x4_t* sa = smem + buf * (A_CH + B_CH);
        u32x4_t* sb = sa + A_CH;
#pragma unroll
        for (int i = 0; i < PER_A; ++i) sa[a_lds[i]] = ra[i];
#pragma unroll
        for (int i = 0; i < PER_B; ++i) sb[b_lds[i]] = rb[i];
    };

    mfma_f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // ------------------------------------------------------------ fragment readers
    auto read_a = [&](const u32x4_t* sa, int ks, mfma_bf16x8 (&fa)[TM]) {
        if (A_KC) {
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                const int row = wm * WTM + t * 32 + lj;
                const int kc = ks * 2 + lg;
                u32x4_t v = sa[row * 8 + (kc ^ (row & 7))];
                fa[t] = __builtin_bit_cast(mfma_bf16x8, v);
            }
        } else {
            constexpr int CPR = BM / 8;
            const uint32_t* sw = reinterpret_cast<const uint32_t*>(sa);
#pragma unroll
            for (int pr = 0; pr < TM / 2; ++pr) {
                const int word = (wm * WTM + pr * 64) / 2 + lj;
                const int chunk = (word >> 2) ^ (lg << 3);
                uint32_t w[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int krow = ks * 16 + lg * 8 + i;
                    w[i] = sw[(krow * CPR + chunk) * 4 + (word & 3)];
                }
                u32x4_t lo = {perm_lo(w[1], w[0]), perm_lo(w[3], w[2]), perm_lo(w[5], w[4]), perm_lo(w[7], w[6])};
                u32x4_t hi = {perm_hi(w[1], w[0]), perm_hi(w[3], w[2]), perm_hi(w[5], w[4]), perm_hi(w[7], w[6])};
                fa[2 * pr] = __builtin_bit_cast(mfma_bf16x8, lo);
                fa[2 * pr + 1] = __builtin_bit_cast(mfma_bf16x8, hi);
            }
        }
    };
    auto read_b = [&](const u32x4_t* sb, int ks, mfma_bf16x8 (&fb)[TN]) {
        if (B_KC) {
#pragma unroll
            for (int t = 0; t < TN; ++t) {
                const int row = wn * WTN + (t >> 1) * 64 + 2 * lj + (t & 1);
                const int kc = ks * 2 + lg;
                u32x4_t v = sb[row * 8 + (kc ^ ((row >> 1) & 7))];
                fb[t] = __builtin_bit_cast(mfma_bf16x8, v);
            }
        } else {
            constexpr int CPR = BN / 8;
            const uint32_t* sw = reinterpret_cast<const uint32_t*>(sb);
#pragma unroll
            for (int pr = 0; pr < TN / 2; ++pr) {
                const int word = (wn * WTN + pr * 64) / 2 + lj;
                const int chunk = (word >> 2) ^ (lg << 3);
                uint32_t w[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int krow = ks * 16 + lg * 8 + i;
                    w[i] = sw[(krow * CPR + chunk) * 4 + (word & 3)];
                }
                u32x4_t lo = {perm_lo(w[1], w[0]), perm_lo(w[3], w[2]), perm_lo(w[5], w[4]), perm_lo(w[7], w[6])};
                u32x4_t hi = {perm_hi(w[1], w[0]), perm_hi(w[3], w[2]), perm_hi(w[5], w[4]), perm_hi(w[7], w[6])};
                fb[2 * pr] = __builtin_bit_cast(mfma_bf16x8, lo);
                fb[2 * pr + 1] = __builtin_bit_cast(mfma_bf16x8, hi);
            }
        }
    };

    // ------------------------------------------------------------ main loop
    if (kt_count > 0) {
        load_global(0);
        store_lds(0);
    }
    __syncthreads();
    for (int kt = 0; kt < kt_count; ++kt) {
        const int cur = kt & 1;
        const bool more = kt + 1 < kt_count;
        if (more) load_global(kt + 1);
        const u32x4_t* sa = smem + cur * (A_CH + B_CH);
        const u32x4_t* sb = sa + A_CH;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            mfma_bf16x8 fa[TM], fb[TN];
            read_a(sa, ks, fa);
            read_b(sb, ks, fb);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (more) store_lds(cur ^ 1);
        __syncthreads();
    }

    // ------------------------------------------------------------ epilogue
    if (!WGRAD) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * WTM + i * 32 + 8 * (v >> 2) + 4 * lg + (v & 3);
                if (row >= mend) continue;
#pragma unroll
                for (int pr = 0; pr < TN / 2; ++pr) {
                    const int col = n0 + wn * WTN + pr * 64 + 2 * lj;
                    if (col >= p.N) continue;
                    const uint32_t packed = pack_bf16x2(acc[i][2 * pr][v], acc[i][2 * pr + 1][v]);
                    if (EPI == EPI_GATED) {
                        if (p.C) *reinterpret_cast<uint32_t*>(p.C + (size_t)row * p.ldc + col) = packed;
                        const float gte = bf16_lo(packed), up = bf16_hi(packed);
                        p.C2[(size_t)row * p.ldc2 + (col >> 1)] = (bf16_t)(up * act_fwd<ACT>(gte));
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
template <int BM, int BN, int WGM, int WGN, bool A_KC, bool B_KC, int EPI, int ACT>
int launch_cfg(const GemmArgs& a, int grid, hipStream_t s)
{
    auto kern = grouped_gemm_bf16_kernel<BM, BN, WGM, WGN, A_KC, B_KC, EPI, ACT>;
    constexpr int lds_bytes = 2 * (BM + BN) * BK * 2;
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
        default: return {256, 128};
    }
}

template <bool A_KC, bool B_KC, int EPI, int ACT>
int launch_any(const GemmArgs& a, int tile_cfg, int grid, hipStream_t s)
{
    switch (tile_cfg) {
        case 1: return launch_cfg<128, 128, 2, 2, A_KC, B_KC, EPI, ACT>(a, grid, s);
        case 3: return launch_cfg<256, 256, 2, 2, A_KC, B_KC, EPI, ACT>(a, grid, s);
        default: return launch_cfg<256, 128, 2, 2, A_KC, B_KC, EPI, ACT>(a, grid, s);
    }
}

}  // namespace

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
                         void* C2, int R, int E, int Kred, int N, int ldb, long long strideB, void* workspace,
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
    const int grid = 8 * ((max_mtiles + 7) / 8) * a.n_ntiles;
    return launch_any<true, B_KC, EPI, ACT>(a, tile_cfg, grid, s);
}

int amoe_bf16_gateup_act(const void* xp, const int32_t* a_row_map, const void* w, const int32_t* offsets, void* gate_up,
                         void* inter, int R, int E, int H, int I, int act, void* workspace, size_t workspace_bytes,
                         int tile_cfg, hipStream_t s)
{
    AMOE_DISPATCH_ACT(act, return (run_rows_bf16<false, EPI_GATED, ACT>(xp, a_row_map, w, offsets, gate_up, inter, R, E, H,
                                                                        2 * I, 2 * I, (long long)H * 2 * I, workspace,
                                                                        workspace_bytes, tile_cfg, s)))
    return AMOE_ERR_BAD_ARG;
}

int amoe_bf16_nn(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C, int R, int E,
                 int Kd, int N, void* workspace, size_t workspace_bytes, int tile_cfg, hipStream_t s)
{
    return run_rows_bf16<false, EPI_STORE, 0>(A, a_row_map, B, offsets, C, nullptr, R, E, Kd, N, N, (long long)Kd * N,
                                              workspace, workspace_bytes, tile_cfg, s);
}

// C[rows_e, :Kd] = A[rows_e, :N] @ B[e]^T with B [E, Kd, N]: the reduction runs over N
int amoe_bf16_nt(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C, int R, int E,
                 int Kd, int N, void* workspace, size_t workspace_bytes, int tile_cfg, hipStream_t s)
{
    return run_rows_bf16<true, EPI_STORE, 0>(A, a_row_map, B, offsets, C, nullptr, R, E, /*Kred=*/N, /*N out=*/Kd,
                                             /*ldb=*/N, (long long)Kd * N, workspace, workspace_bytes, tile_cfg, s);
}

int amoe_bf16_wgrad(const void* A, const void* B, const int32_t* offsets, void* C, int R, int E, int Kd, int N,
                    int tile_cfg, hipStream_t s)
{
    TileCfg tc = pick_cfg(tile_cfg);
    GemmArgs a = {};
    a.A = (const bf16_t*)A;
    a.B = (const bf16_t*)B;
    a.C = (bf16_t*)C;
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
    const long long pm_total = (long long)E * a.n_mt;
    const long long grid = 8 * ((pm_total + 7) / 8) * a.n_ntiles;
    AMOE_REQUIRE(grid < (1ll << 31), AMOE_ERR_UNSUPPORTED, "grouped_gemm_wgrad: grid too large");
    return launch_any<false, false, EPI_STORE, 0>(a, tile_cfg, (int)grid, s);
}
