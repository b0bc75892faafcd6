// Ragged grouped GEMMs on bf16 / f16 MFMA (v_mfma_f32_32x32x16_bf16 / _f16), f32 accumulate.
//
// Two kernel templates cover the three operand layouts of the expert FFN:
//   grouped_gemm_rows_body (persistent, one workgroup per CU)
//     rows / NN   C[rows_e,:] = A[rows_e,:] @ B[e]        (forward; B is [Kd,N], N contiguous)
//     rows / NT   C[rows_e,:] = A[rows_e,:] @ B[e]^T      (data gradient; B is [N',Kd'] so both K-contiguous)
//   grouped_gemm_wgrad_body (one tile per workgroup)
//     wgrad / TN  C[e] = A[rows_e,:]^T @ B[rows_e,:]      (weight gradient; the reduction runs over the ragged rows)
//
// Tiles of BM x BN x 32 move from global memory straight into LDS (global_load_lds, 16 bytes
// per lane, four stages in flight); the XOR swizzle of the LDS layout is applied on the source
// side.  Fragments are read back with
//   * ds_read_b128 when the operand is K-contiguous in LDS.  A 32-wide K row is 4 chunks of
//     16 bytes; chunk kc of row r sits at position kc ^ ((r >> 2) & 3), which makes the 32
//     rows a half-wave reads cover every group of 4 banks exactly twice and the 4 lanes of
//     each quad distinct groups: conflict-free on the 64-bank LDS of gfx950;
//   * two ds_read_b64_tr_b16 (the transposing LDS read of gfx950) when it is K-strided, i.e.
//     stored [k][column] with the columns contiguous.  The 16 lanes of a group together read a
//     4 (k) x 16 (columns) block -- lane j supplies the address of k row j/4, columns
//     4*(j%4)..+3 -- and lane i of the group receives column i for the 4 k rows, which is the
//     MFMA operand layout.  16-byte chunk c of k row k sits at position c ^ ((k & 3) << 2), so
//     the four k rows a half-wave reads fall into the four different quarters of the banks.
// Every operand layout therefore yields the same accumulator layout: lane l of a 32x32 tile
// holds column l%32.  In the epilogue neighbouring lanes swap one value (DPP) so that each
// lane stores a packed pair of adjacent columns of ONE row; for the gate_up GEMM that pair is
// (gate, up) of one intermediate column, so the gated activation runs on registers.
//
// Row-grouped launches take their (expert, first row, end row) per M tile from a tile map
// that a small kernel builds on the device from the expert offsets: no host sync, empty
// experts simply own no tile.  Tiles are dealt to the 8 XCDs so that the ~32 workgroups resident
// on one XCD cover one super-tile of gm x gn tiles (shared A and B panels in that XCD's L2),
// and super-tiles rotate over the XCDs, which keeps them evenly loaded whatever the routing
// skew.
#include "amoe_common.h"

// This file is compiled once per group of entry points (-DAMOE_GEMM_PART=0..3), in parallel: the
// kernels of all groups are instances of the same two templates.
//   0: gate_up forward with the gated activation   1: plain row-grouped products (NN, NT)
//   2: data gradient of down + gated-activation backward   3: weight gradients, tile map, shared host helpers
#ifndef AMOE_GEMM_PART
#define AMOE_GEMM_PART -1   // everything in one translation unit
#endif
#define AMOE_PART(n) (AMOE_GEMM_PART < 0 || AMOE_GEMM_PART == (n))

#include <atomic>
#include <type_traits>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 mfma_bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 mfma_f16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float mfma_f32x16;

// What the kernel needs to know about its 16-bit element type: the MFMA operand vector and
// instruction, and the conversions of the epilogues (round to nearest even on the way out).
// Addresses, tiles and the LDS layout only depend on the element size, which the two types share.
template <typename ET>
struct Elem16;
template <>
struct Elem16<bf16_t> {
    typedef mfma_bf16x8 frag_t;
    __device__ static __forceinline__ float lo(uint32_t w) { return bf16_lo(w); }
    __device__ static __forceinline__ float hi(uint32_t w) { return bf16_hi(w); }
    __device__ static __forceinline__ uint32_t pack2(float a, float b) { return pack_bf16x2(a, b); }
    __device__ static __forceinline__ mfma_f32x16 mfma(frag_t a, frag_t b, mfma_f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Elem16<f16_t> {
    typedef mfma_f16x8 frag_t;
    __device__ static __forceinline__ float lo(uint32_t w) { return f16_lo(w); }
    __device__ static __forceinline__ float hi(uint32_t w) { return f16_hi(w); }
    __device__ static __forceinline__ uint32_t pack2(float a, float b) { return pack_f16x2(a, b); }
    __device__ static __forceinline__ mfma_f32x16 mfma(frag_t a, frag_t b, mfma_f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

namespace {

constexpr int BK = 32;      // K extent of one LDS stage
constexpr int NSTAGE = 4;   // LDS stages: one being consumed, the others landed or in flight.  (5 stages fit
                            // the 160 KB of LDS and were measured: no faster.)

struct GemmArgs {
    const bf16_t* A;
    const bf16_t* B;
    bf16_t* C;
    bf16_t* C2;
    const int32_t* a_row_map;
    const int32_t* b_row_map;  // weight gradient only
    const float* row_scale;  // gated epilogues: the per-row factor of the gated activation (null = 1)
    const bf16_t* G;         // gated-backward epilogue: gate_up [R, 2N] of the forward pass
    float* partials;         // gated-backward epilogue: [n_ntiles][part_stride] row sums, or null
    int ldg, part_stride;
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
    int max_mtiles;  // rows mode: entries of tile_map (those past the last tile hold expert -1)
    int f16;         // host side only: the operands are float16 (launch the f16 instance), else bf16
};

enum { EPI_STORE = 0, EPI_GATED = 1, EPI_GATED_BWD = 2 };

#if AMOE_PART(3)
// tile map of a caller that brings its own expert offsets (amoe_emit_tile_map has the layout)
__global__ void __launch_bounds__(512)
tile_map_kernel(const int32_t* __restrict__ offsets, int E, int bm, int4* __restrict__ tile_map,
                int32_t* __restrict__ header, int max_mtiles)
{
    __shared__ int32_t row_end[AMOE_MAX_EXPERTS];
    __shared__ int32_t tscan[AMOE_MAX_EXPERTS];
    const int e = threadIdx.x;  // 512 threads, one per possible expert
    if (e < E) row_end[e] = offsets[e + 1] - offsets[0];
    __syncthreads();
    amoe_emit_tile_map<512>(row_end, offsets[0], E, bm, tile_map, header, max_mtiles, tscan);
}
#endif

typedef short tr_i16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) tr_i16x4* tr_lptr_t;

// value of the lane whose index differs in bit 0 / bit 1 (DPP quad permutes, no LDS traffic)
__device__ __forceinline__ float lane_xor1(float x)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
}
__device__ __forceinline__ float lane_xor2(float x)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
}

// 16 zero bytes that masked lanes of a direct-to-LDS load read instead of out-of-range rows
static __device__ __attribute__((aligned(16))) uint32_t g_zero_chunk[4] = {0u, 0u, 0u, 0u};

// Wave-uniform load of one int32 from memory this kernel never writes: read through the
// constant address space, which makes it a scalar load (its own counter, tracked by the
// compiler) instead of a vector load.
__device__ __forceinline__ int scalar_load_i32(const int32_t* ptr)
{
    return *(const __attribute__((address_space(4))) int32_t*)ptr;
}

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
// One direct-to-LDS load of 16 bytes per lane in its scalar-base form: a wave-uniform 64-bit base, a
// 32-bit byte offset per lane, the wave's LDS destination in M0 (lane l lands at M0 + 16 l).  The
// builtin only produces the form with a 64-bit address per lane, which costs a register pair per
// load and a 64-bit vector add per issue.  The load is not known to the compiler: whoever issues it
// waits for it (vmcnt) before the data is read.  M0 is written and consumed inside one asm statement
// (the compiler reserves M0 and sets it anew before each use of its own; the build's assembly check
// verifies that every write of M0 in these kernels is followed at once by the load that reads it).
__device__ __forceinline__ void dma16_sbase(const void* base, uint32_t lane_offset, uint32_t lds_addr)
{
    // (operands the compiler may hold in vector registers although they are wave-uniform)
    const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_addr);
    const uint64_t b64 = (uint64_t)(uintptr_t)base;
    const uint64_t sb = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b64) |
                        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32)) << 32);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(m0v), "v"(lane_offset), "s"(sb)
                 : "memory");
}
// the same for 4 bytes per lane (lane l lands at M0 + 4 l)
__device__ __forceinline__ void dma4_sbase(const void* base, uint32_t lane_offset, uint32_t lds_addr)
{
    // (operands the compiler may hold in vector registers although they are wave-uniform)
    const uint32_t m0v = __builtin_amdgcn_readfirstlane(lds_addr);
    const uint64_t b64 = (uint64_t)(uintptr_t)base;
    const uint64_t sb = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b64) |
                        ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b64 >> 32)) << 32);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :
                 : "s"(m0v), "v"(lane_offset), "s"(sb)
                 : "memory");
}
// workgroup barrier for data exchanged through LDS by ordinary LDS accesses: this wave's LDS traffic
// has completed, then the hardware barrier (loads and stores to global memory stay in flight)
__device__ __forceinline__ void lds_sync()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// Activation for the bf16 epilogue: the sigmoid's division by the hardware reciprocal (1 ulp; the
// result is rounded to bf16 next) instead of the ten-instruction IEEE division sequence.
template <int ACT>
__device__ __forceinline__ float act_fwd_fast(float g)
{
    if (ACT == AMOE_ACT_SILU) return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g));
    if (ACT == AMOE_ACT_GPT_OSS) return g * __builtin_amdgcn_rcpf(1.0f + __expf(-1.702f * g));
    return act_fwd<ACT>(g);
}
// act(g) and act'(g) for the backward epilogue, sharing one sigmoid (hardware reciprocal, see above)
template <int ACT>
__device__ __forceinline__ void act_both_fast(float g, float& f, float& df)
{
    if (ACT == AMOE_ACT_SILU || ACT == AMOE_ACT_GPT_OSS) {
        const float a = ACT == AMOE_ACT_SILU ? 1.0f : 1.702f;
        const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-a * g));
        f = g * sg;
        df = sg * (1.0f + a * g * (1.0f - sg));
    } else {
        f = act_fwd<ACT>(g);
        df = act_bwd<ACT>(g);
    }
}
using T_ = std::true_type;
using F_ = std::false_type;

// ------------------------------------------------------------------ weight gradient: one tile per workgroup
// C[e] = A[rows_e,:]^T @ B[rows_e,:]: the reduction runs over the expert's rows, both operands are
// K-strided ([k][column] in LDS, transposing reads).
// MAPS: 1 = the rows of A, 2 = the rows of B are gathered through a row map
// ET: the 16-bit element type (bf16_t or f16_t); GemmArgs names its pointers bf16_t for both
template <int BM, int BN, int WGM, int WGN, int MAPS, typename ET>
__device__ __forceinline__ void grouped_gemm_wgrad_body(const GemmArgs& p)
{
    typedef typename Elem16<ET>::frag_t frag_t;
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr bool A_MAP = (MAPS & 1) != 0, B_MAP = (MAPS & 2) != 0;
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
    const int e = pm / p.n_mt;
    if (e >= p.E) return;
    const int m0 = (pm - e * p.n_mt) * BM;
    const int mend = p.M;   // output rows per expert
    const int r0 = p.offsets[e], r1 = p.offsets[e + 1];
    const int kt_count = (r1 - r0 + BK - 1) / BK;
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
        constexpr int CPR = BM / 8;
        const int krow = c / CPR, mc = (c % CPR) ^ ((krow & 3) << 2);
        const int col = min(m0 + mc * 8, p.M - 8);
        aoff[i] = A_MAP ? (uint32_t)col : (uint32_t)krow * (uint32_t)p.lda + col;
        a_kr[i] = krow;
    }
#pragma unroll
    for (int i = 0; i < PER_B; ++i) {
        const int c = tid + NT * i;
        constexpr int CPR = BN / 8;
        const int krow = c / CPR, nc = (c % CPR) ^ ((krow & 3) << 2);
        const int col = min(n0 + nc * 8, p.N - 8);
        boff[i] = B_MAP ? (uint32_t)col : (uint32_t)krow * (uint32_t)p.ldb + col;
        b_kr[i] = krow;
    }
    if (!A_MAP) Ab += (long long)r0 * p.lda;
    if (!B_MAP) Bb += (long long)r0 * p.ldb;
    const int k_rows = r1 - r0;  // rows of this expert

    // Gathered operands of the weight gradient: the source row of a chunk changes with every K
    // tile.  One wave-wide load covers RPW consecutive k rows starting at a wave-uniform row, so
    // the row indices are fetched with SCALAR loads (their own counter: a vector load here would
    // have to be awaited together with every direct-to-LDS load issued before it; the maps are
    // only ever read by this kernel, which is what a scalar load requires) into a_snx /
    // b_snx one tile ahead, and spread to the lanes (a_use / b_use) right after the fragment
    // wait at the start of the step whose loads use them.
    constexpr int RPW_A = 64 / (BM / 8), RPW_B = 64 / (BN / 8);
    int a_use[PER_A], b_use[PER_B];
    int a_snx[PER_A][RPW_A], b_snx[PER_B][RPW_B];
    auto sfetch_a = [&](int kt, int (&dst)[PER_A][RPW_A]) {
#pragma unroll
        for (int i = 0; i < PER_A; ++i)
#pragma unroll
            for (int q = 0; q < RPW_A; ++q)
                dst[i][q] = scalar_load_i32(p.a_row_map + min(r0 + kt * BK + (wave * 64 + NT * i) / (BM / 8) + q, p.rows_total - 1));
    };
    auto sfetch_b = [&](int kt, int (&dst)[PER_B][RPW_B]) {
#pragma unroll
        for (int i = 0; i < PER_B; ++i)
#pragma unroll
            for (int q = 0; q < RPW_B; ++q)
                dst[i][q] = scalar_load_i32(p.b_row_map + min(r0 + kt * BK + (wave * 64 + NT * i) / (BN / 8) + q, p.rows_total - 1));
    };
    // Each fetched index passes through an empty asm statement as a scalar register first: a
    // select between two values that are still loads from the index array would be folded into
    // one load at a selected address, which turns the array into scratch memory.
    auto spread_a = [&](const int (&src)[PER_A][RPW_A], int (&dst)[PER_A]) {
#pragma unroll
        for (int i = 0; i < PER_A; ++i) {
            int v = 0;
#pragma unroll
            for (int q = 0; q < RPW_A; ++q) {
                int sq = src[i][q];
                asm("" : "+s"(sq));
                v = (q == 0 || lane / (BM / 8) == q) ? sq : v;
            }
            dst[i] = v;
        }
    };
    auto spread_b = [&](const int (&src)[PER_B][RPW_B], int (&dst)[PER_B]) {
#pragma unroll
        for (int i = 0; i < PER_B; ++i) {
            int v = 0;
#pragma unroll
            for (int q = 0; q < RPW_B; ++q) {
                int sq = src[i][q];
                asm("" : "+s"(sq));
                v = (q == 0 || lane / (BN / 8) == q) ? sq : v;
            }
            dst[i] = v;
        }
    };

    const bf16_t* zero_src = reinterpret_cast<const bf16_t*>(g_zero_chunk);
    asm volatile("" : "+s"(zero_src));  // keep the address in registers (not re-derived per load)
    // wgrad: rows past the end of the expert read a block of zeros instead (only the last K
    // tile of an expert can be ragged, the select costs two VALU ops per load)
    auto dma_a = [&](int kt, auto LO, auto HI, const int (&idx)[PER_A]) {
        constexpr int lo = decltype(LO)::value, hi = decltype(HI)::value;
        const int k0 = kt * BK;
        u32x4_t* sa = smem + (kt % NSTAGE) * STAGE + wave * 64;
        const bf16_t* a_base = A_MAP ? Ab : Ab + (long long)k0 * p.lda;
#pragma unroll
        for (int i = lo; i < hi; ++i) {
            const bf16_t* src = a_base + aoff[i];
            if (A_MAP) src += (long long)idx[i] * p.lda;
            src = (k0 + a_kr[i] < k_rows) ? src : zero_src;
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(sa + NT * i), 16, 0, 0);
        }
    };
    auto dma_b = [&](int kt, auto LO, auto HI, const int (&idx)[PER_B]) {
        constexpr int lo = decltype(LO)::value, hi = decltype(HI)::value;
        const int k0 = kt * BK;
        u32x4_t* sb = smem + (kt % NSTAGE) * STAGE + A_CH + wave * 64;
        const bf16_t* b_base = B_MAP ? Bb : Bb + (long long)k0 * p.ldb;
#pragma unroll
        for (int i = lo; i < hi; ++i) {
            const bf16_t* src = b_base + boff[i];
            if (B_MAP) src += (long long)idx[i] * p.ldb;
            src = (k0 + b_kr[i] < k_rows) ? src : zero_src;
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(sb + NT * i), 16, 0, 0);
        }
    };
    auto issue_a = [&](int kt, auto LO, auto HI) { dma_a(kt, LO, HI, a_use); };
    auto issue_b = [&](int kt, auto LO, auto HI) { dma_b(kt, LO, HI, b_use); };

    mfma_f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // ------------------------------------------------------------ fragment readers
    // One 16-byte register quad per 32-wide tile and 16-deep K step.  Lane -> (k row, 4 columns) inside the 4x16 block its 16-lane group
    // transposes; groups 0/1 take columns 0-15 / 16-31 of the tile, groups 2/3 the k rows 8-15.
    // The transposing read is issued as inline assembly: through the builtin the compiler treats
    // it as possibly aliasing the direct-to-LDS loads in flight and drains them all (vmcnt(0))
    // before every read.  The compiler therefore does not track these reads; settle() below
    // waits for them and ties the fragments to the wait.
    const int tr_j = lane & 15, tr_blk = lane >> 4;
    const int tr_col = 16 * (tr_blk & 1) + 4 * (tr_j & 3);   // first of this lane's 4 columns in the tile
    const int tr_k = 8 * (tr_blk >> 1) + (tr_j >> 2);        // its k row inside the K step (+4 for the second read)
    auto read_tr = [&](const u32x4_t* st, auto CPR_, int col0, auto KS) -> u32x4_t {
        constexpr int cpr = decltype(CPR_)::value, ks = decltype(KS)::value;
        const int col = col0 + tr_col;
        const int chunk = (col >> 3) ^ ((tr_j >> 2) << 2);
        const uint32_t addr = (uint32_t)(uintptr_t)(lptr_t)st + (uint32_t)((tr_k * cpr + chunk) * 16 + (col & 7) * 2);
        u32x2_t lo, hi;
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo) : "v"(addr), "i"(ks * 16 * cpr * 16));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "i"((ks * 16 + 4) * cpr * 16));
        return u32x4_t{lo[0], lo[1], hi[0], hi[1]};
    };
    auto read_a = [&](const u32x4_t* sa, auto KS, frag_t (&fa)[TM], auto LIVE) {
        constexpr int ks = decltype(KS)::value;
#pragma unroll
        for (int t = 0; t < decltype(LIVE)::value; ++t) {
            fa[t] = __builtin_bit_cast(frag_t, read_tr(sa, std::integral_constant<int, BM / 8>{}, wm * WTM + t * 32, KS));
        }
    };
    auto read_b = [&](const u32x4_t* sb, auto KS, frag_t (&fb)[TN]) {
        constexpr int ks = decltype(KS)::value;
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            fb[t] = __builtin_bit_cast(frag_t, read_tr(sb, std::integral_constant<int, BN / 8>{}, wn * WTN + t * 32, KS));
        }
    };
    // Called before the first MFMA that consumes fragments fetched by read_tr: waits for this
    // wave's LDS reads and makes the fragments depend on the wait (an MFMA is otherwise free to
    // be scheduled ahead of it).
    auto settle = [&](frag_t (&fa)[TM], frag_t (&fb)[TN], auto LIVE) {
        asm volatile("s_waitcnt lgkmcnt(0)");
#pragma unroll
        for (int t = 0; t < decltype(LIVE)::value; ++t) asm volatile("" : "+v"(fa[t]));   // only the blocks that were read
#pragma unroll
        for (int t = 0; t < TN; ++t) asm volatile("" : "+v"(fb[t]));
    };
    // quarter Q of a K step's MFMAs (A tile outer, B tile inner)
    constexpr int N_MFMA = TM * TN;
    static_assert(N_MFMA % 4 == 0, "a K step is issued in four chunks");
    auto mma_quarter = [&](const frag_t (&fa)[TM], const frag_t (&fb)[TN], auto Q, auto LIVE) {
        constexpr int q = decltype(Q)::value;
#pragma unroll
        for (int f = q * (N_MFMA / 4); f < (q + 1) * (N_MFMA / 4); ++f) {
            const int i = f / TN, j = f % TN;
            if (i >= decltype(LIVE)::value) continue;   // a 32-row block past the end of the expert
            acc[i][j] = Elem16<ET>::mfma(fa[i], fb[j], acc[i][j]);
        }
    };

    // ------------------------------------------------------------ main loop
    // NSTAGE LDS stages of one 32-wide K tile each (two MFMA K steps); the offsets below are
    // those of NSTAGE = 4.  Iteration j works on tile j (stage j % 4):
    //   step A: MFMAs on the ks=0 fragments | fetch the ks=1 fragments of tile j
    //           | issue the B half of the loads of tile j+3
    //   wait until tile j+1 has landed (the loads of tiles j+2, j+3 may stay in flight), barrier:
    //           tile j+1 is visible and stage j % 4 is free (every wave holds its last fragments)
    //   step B: MFMAs on the ks=1 fragments | fetch the ks=0 fragments of tile j+1
    //           | issue the A half of the loads of tile j+4 into the stage just freed
    // so the direct-to-LDS loads trickle out evenly (the L1 path moves 64 bytes a clock, half of
    // what the MFMAs consume at full rate) and each has about two iterations to land.
    // A step is written as four chunks fenced by scheduling barriers, each pairing a quarter of
    // the MFMAs with one kind of side work: A-fragment reads, B-fragment reads, loads, loads.
    // Fragments are double-buffered: a step's reads fill the set the other step consumes.
    constexpr int PER = PER_A + PER_B;
    static_assert((NSTAGE - 2) * PER + PER_A <= 63, "vmcnt is a 6-bit counter");
    using IC0 = std::integral_constant<int, 0>;
    using IC1 = std::integral_constant<int, 1>;
    using IC2 = std::integral_constant<int, 2>;
    using IC3 = std::integral_constant<int, 3>;
    using A_HALF = std::integral_constant<int, (PER_A + 1) / 2>;
    using A_ALL = std::integral_constant<int, PER_A>;
    using B_HALF = std::integral_constant<int, (PER_B + 1) / 2>;
    using B_ALL = std::integral_constant<int, PER_B>;
    frag_t fa0[TM], fb0[TN], fa1[TM], fb1[TN];

    // prologue: tiles 0..2 and the A half of tile 3 go out, tile 0 is awaited
    {
        // row lookups of the first four tiles go out together, ahead of their loads
        int sa4[NSTAGE][PER_A][RPW_A], sb4[NSTAGE][PER_B][RPW_B];
#pragma unroll
        for (int t = 0; t < NSTAGE; ++t) {
            if (A_MAP) sfetch_a(t, sa4[t]);
            if (B_MAP && t < NSTAGE - 1) sfetch_b(t, sb4[t]);
        }
        if (A_MAP) sfetch_a(NSTAGE, a_snx);      // next A tile to go out in the loop
        if (B_MAP) sfetch_b(NSTAGE - 1, b_snx);  // next B tile to go out in the loop
#pragma unroll
        for (int t = 0; t < NSTAGE - 1; ++t) {
            if (t < kt_count) {
                if (A_MAP) spread_a(sa4[t], a_use);
                if (B_MAP) spread_b(sb4[t], b_use);
                // B first: its addresses are known, those of A may still wait for the row map
                dma_b(t, IC0{}, B_ALL{}, b_use);
                dma_a(t, IC0{}, A_ALL{}, a_use);
            }
        }
        if (kt_count > NSTAGE - 1) {
            if (A_MAP) spread_a(sa4[NSTAGE - 1], a_use);
            dma_a(NSTAGE - 1, IC0{}, A_ALL{}, a_use);
        }
    }
    if (kt_count > NSTAGE - 1) {
        lds_barrier<(NSTAGE - 2) * PER + PER_A>();
    } else {
        lds_barrier<0>();
    }
    __builtin_amdgcn_sched_barrier(0);

    // LOAD_B: tile kt+3 exists; LOAD_A: tile kt+4 exists; WAITN: loads younger than tile kt+1
    auto k_tile = [&](auto LIVE, auto LOAD_B, auto LOAD_A, auto WAITN, auto NEXT, int kt) {
        constexpr bool idle = decltype(LIVE)::value == 0;   // this wave owns no live row: it only takes part in the loads
        constexpr bool load_b = decltype(LOAD_B)::value, load_a = decltype(LOAD_A)::value;
        constexpr bool next = decltype(NEXT)::value;
        constexpr int waitn = decltype(WAITN)::value;
        const u32x4_t* sa = smem + (kt % NSTAGE) * STAGE;
        const u32x4_t* sb = sa + A_CH;
        // ---- step A: MFMAs on (fa0, fb0)
        if (!idle) settle(fa0, fb0, LIVE);
        if (B_MAP && load_b) {
            spread_b(b_snx, b_use);     // rows of the B tile whose loads go out in this step
            sfetch_b(kt + NSTAGE, b_snx);
        }
        read_a(sa, IC1{}, fa1, LIVE);
        mma_quarter(fa0, fb0, IC0{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (!idle) read_b(sb, IC1{}, fb1);
        mma_quarter(fa0, fb0, IC1{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (load_b) issue_b(kt + NSTAGE - 1, IC0{}, B_HALF{});
        mma_quarter(fa0, fb0, IC2{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (load_b) issue_b(kt + NSTAGE - 1, B_HALF{}, B_ALL{});
        mma_quarter(fa0, fb0, IC3{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        lds_barrier<waitn>();
        __builtin_amdgcn_sched_barrier(0);
        // ---- step B: MFMAs on (fa1, fb1)
        const u32x4_t* na = smem + ((kt + 1) % NSTAGE) * STAGE;
        if (!idle) settle(fa1, fb1, LIVE);
        if (A_MAP && load_a) {
            spread_a(a_snx, a_use);     // rows of the A tile whose loads go out in this step
            sfetch_a(kt + NSTAGE + 1, a_snx);
        }
        if (next) read_a(na, IC0{}, fa0, LIVE);
        mma_quarter(fa1, fb1, IC0{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (next && !idle) read_b(na + A_CH, IC0{}, fb0);
        mma_quarter(fa1, fb1, IC1{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (load_a) issue_a(kt + NSTAGE, IC0{}, A_HALF{});
        mma_quarter(fa1, fb1, IC2{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (load_a) issue_a(kt + NSTAGE, A_HALF{}, A_ALL{});
        mma_quarter(fa1, fb1, IC3{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
    };
    // Every path through this block ends in the final k_tile, whose first action waits for the
    // fragment reads still outstanding: none is in flight when the epilogue reuses the registers.
    auto run_tiles = [&](auto LIVE) {
    if (kt_count > 0) {
        // W<r>: loads younger than tile kt+1 when r tiles (kt included) remain and none is left to issue
        using W0 = std::integral_constant<int, 0>;
        using W1 = std::integral_constant<int, PER>;
        using W2 = std::integral_constant<int, 2 * PER>;
        using WFULL = std::integral_constant<int, (NSTAGE - 2) * PER>;
        static_assert(NSTAGE == 4 || NSTAGE == 5, "the drain below is written out for 4 or 5 stages");
        read_a(smem, IC0{}, fa0, LIVE);
        if (decltype(LIVE)::value) read_b(smem + A_CH, IC0{}, fb0);
        __builtin_amdgcn_sched_barrier(0);
        int kt = 0;
        for (; kt + NSTAGE < kt_count; ++kt) k_tile(LIVE, T_{}, T_{}, WFULL{}, T_{}, kt);
        if (kt + NSTAGE == kt_count) { k_tile(LIVE, T_{}, F_{}, WFULL{}, T_{}, kt); ++kt; }
        if (NSTAGE == 5) {
            if (kt + 4 == kt_count) { k_tile(LIVE, F_{}, F_{}, W2{}, T_{}, kt); ++kt; }
        }
        if (kt + 3 == kt_count) { k_tile(LIVE, F_{}, F_{}, W1{}, T_{}, kt); ++kt; }
        if (kt + 2 == kt_count) { k_tile(LIVE, F_{}, F_{}, W0{}, T_{}, kt); ++kt; }
        k_tile(LIVE, F_{}, F_{}, W0{}, F_{}, kt);  // kt + 1 == kt_count here, whichever way it was reached
    }
    };
    // Only the 32-row blocks of this wave that hold live rows are read and multiplied: the last tile
    // of an expert is often a sliver, and a block of clamped duplicate rows costs as much as a live
    // one.  The count is wave-uniform and picks one copy of the loop; a wave without live rows still
    // issues its share of the loads and meets the barriers.  (Tests inside one shared loop were
    // measured slower than no skipping at all: they cost the full tiles more than the slivers gain.)
    {
        // (weight gradient: mend is the number of output rows per expert; a wave whose columns all lie
        // past the matrix edge has nothing to multiply either)
        const int live_rows = n0 + wn * WTN < p.N ? min(max(mend - (m0 + wm * WTM), 0), WTM) : 0;
        const int live = (live_rows + 31) >> 5;
        static_assert(TM == 2 || TM == 4, "the dispatch below is written for two or four 32-row blocks per wave");
        if (live >= TM) {
            run_tiles(std::integral_constant<int, TM>{});
        } else if (live == 0) {
            run_tiles(std::integral_constant<int, 0>{});
        } else if (live == 1) {
            run_tiles(std::integral_constant<int, 1>{});
        } else {
            if constexpr (TM == 4) {
                if (live == 2) run_tiles(std::integral_constant<int, 2>{});
                else run_tiles(std::integral_constant<int, 3>{});
            }
        }
    }

    // ------------------------------------------------------------ epilogue
    // Lane l of tile (i, j) holds column j*32 + l%32 for 16 rows; registers v, v+1 (v even) are
    // rows r, r+1.  Each lane converts its two values to one packed pair, lanes 2c and 2c+1
    // exchange the pairs (DPP) and a byte permute leaves the even lane with columns (2c, 2c+1) of
    // row r and the odd lane with those of row r+1: three VALU operations per 4-byte store.
    // Addresses are a wave-uniform row base (scalar arithmetic) plus one per-lane 32-bit offset;
    // tiles that lie entirely inside the matrix take the FULL form without per-store bounds tests.
    bf16_t* Cb = p.C + (long long)e * p.strideC;
    const int odd1 = lj & 1;
    const uint32_t swap_sel = odd1 ? 0x03020706u : 0x05040100u;
    // wave-uniform origin of this wave's part of the tile, and the lane's offset from it (bytes)
    const long long worg = (long long)(m0 + wm * WTM) * p.ldc + n0 + wn * WTN;
    char* cbase = reinterpret_cast<char*>(Cb + worg);
    const uint32_t loff = (uint32_t)((4 * lg + odd1) * p.ldc + (lj & ~1)) * 2u;
    auto epilogue = [&](auto FULL) {
        constexpr bool full = decltype(FULL)::value;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const bool col_ok = full || (n0 + wn * WTN + j * 32 + (lj & ~1) < p.N);
#pragma unroll
                for (int v = 0; v < 16; v += 4) {
                    const int rq = i * 32 + 8 * (v >> 2);           // first of 8 rows, relative to the wave's origin
                    const int rt = wm * WTM + rq + 4 * lg;          // rows rt..rt+3 of the tile
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        const uint32_t own = Elem16<ET>::pack2(acc[i][j][v + 2 * u], acc[i][j][v + 2 * u + 1]);
                        const uint32_t got = __builtin_amdgcn_update_dpp(0, own, 0xB1, 0xF, 0xF, true);
                        const uint32_t pk = __builtin_amdgcn_perm(got, own, swap_sel);
                        const bool ok = full || (col_ok && m0 + rt + 2 * u + odd1 < mend);
                        if (ok) {
                            char* rowp = cbase + ((long long)(rq + 2 * u) * p.ldc + j * 32) * 2;
                            *reinterpret_cast<uint32_t*>(rowp + loff) = pk;
                        }
                    }
                }
            }
        }
    };
    if (m0 + BM <= mend && n0 + BN <= p.N) epilogue(T_{}); else epilogue(F_{});
}

// ------------------------------------------------------------------ row-grouped GEMMs: persistent kernel
// One workgroup per CU walks over its share of the tiles (virtual block b, b + grid, b + 2 grid, ...
// with the same virtual block -> tile mapping a one-tile-per-workgroup launch would use, so the
// workgroups of one XCD still work on one super-tile at a time).  The K loops of consecutive tiles
// form one software pipeline: the last four iterations of a tile issue the loads of the first four
// K tiles of the next one, so a tile starts with its operands already in LDS, and what remains
// between two tiles is the epilogue.  What the next tile needs is fetched a tile ahead: its entry
// of the tile map by a scalar load, its gathered row indices by a direct-to-LDS load at the start
// of the current tile (a vector load to registers would have to be awaited together with every
// operand load issued after it).  The row scales of the gated epilogues arrive the same way.
template <int BM, int BN, int WGM, int WGN, bool B_KC, int EPI, int ACT, typename ET>
__device__ __forceinline__ void grouped_gemm_rows_body(const GemmArgs& p)
{
    typedef typename Elem16<ET>::frag_t frag_t;
    constexpr int NT = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    static_assert(NSTAGE == 4, "the cross-tile pipeline is written for four stages");
    static_assert(BM >= 128 && BN >= 128, "K-strided swizzle needs 16 chunks per row");
    static_assert(NT >= BM, "one thread per tile row for the row-index and row-scale loads");
    constexpr int A_CH = BM * 4, B_CH = BN * 4;   // 16-byte chunks per stage (a 32-wide K row is 4 chunks)
    constexpr int STAGE = A_CH + B_CH;
    constexpr int PER_A = A_CH / NT, PER_B = B_CH / NT;
    constexpr int PER = PER_A + PER_B;
    static_assert(A_CH % NT == 0 && B_CH % NT == 0, "tile must split evenly over the block");
    static_assert((NSTAGE - 2) * PER + PER_A <= 63, "vmcnt is a 6-bit counter");
    // stores every wave issues in the epilogue of a tile without edge tests (at least)
    constexpr int EPI_STORES = EPI == EPI_GATED_BWD ? TM * TN * 16 : (EPI == EPI_GATED ? TM * TN * 4 : TM * TN * 8);
    constexpr int W_AFTER_STORES = -1;
    constexpr int W_LOOSE = (NSTAGE - 2) * PER + EPI_STORES < 63 ? (NSTAGE - 2) * PER + EPI_STORES : 63;

    extern __shared__ u32x4_t smem[];
    // LDS: the stages | row indices of the next tile [NT] | row scales of two tiles [2][BM] | row-sum partials [2 WGN][BM]
    int32_t* s_idx = reinterpret_cast<int32_t*>(smem + NSTAGE * STAGE);
    float* s_rs2 = reinterpret_cast<float*>(s_idx + NT);
    float* s_part = s_rs2 + 2 * BM;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WGN, wn = wave % WGN;
    const int lj = lane & 31, lg = lane >> 5;
    const int KT = p.Kd / BK;

    // ------------------------------------------------------------ this workgroup's tiles
    // Virtual blocks b, b + grid, b + 2 grid, ...; virtual block v belongs to XCD v % 8 (the hardware deals
    // workgroups to the XCDs round-robin) and is slot (v / 8) % (gm gn) of super-tile ((v / 8) / (gm gn)) * 8
    // + v % 8: the workgroups resident on one XCD work on one super-tile of gm x gn tiles at a time (its gm A
    // panels and gn B panels are shared in that XCD's L2) and the super-tiles rotate over the XCDs.  Only whole
    // groups of 8 super-tiles are dealt that way: the up to 7 left over would give some XCDs a whole super-tile
    // (about one round of tiles) more than the others, so their tiles go to the XCDs one by one.
    const int per_super = p.gm * p.gn;
    const int n_mtiles = min(scalar_load_i32(p.n_mtiles), p.max_mtiles);
    const int supers = ((n_mtiles + p.gm - 1) / p.gm) * p.sn;
    const int vb_rot = (supers >> 3) * 8 * per_super;      // virtual blocks of the rotated part
    const int vb_total = supers * per_super;
    int vb_next = blockIdx.x;
    auto advance = [&](int& pm, int& nt) -> bool {  // this workgroup's next tile; false: none is left
        while (vb_next < vb_total) {
            const int vb = vb_next;
            vb_next += gridDim.x;
            int sid, w;
            if (vb < vb_rot) {
                const int xcd = vb & 7, q = vb >> 3;
                sid = (q / per_super) * 8 + xcd;
                w = q % per_super;
            } else {
                sid = vb / per_super;
                w = vb - sid * per_super;
            }
            const int sm = sid / p.sn, sn_i = sid - sm * p.sn;
            pm = sm * p.gm + w / p.gn;
            nt = sn_i * p.gn + w % p.gn;
            if (nt < p.n_ntiles && pm < n_mtiles) return true;
        }
        return false;
    };
    auto load_entry = [&](int pm) -> int4 {
        const int32_t* ent = reinterpret_cast<const int32_t*>(p.tile_map + pm);
        int4 v;
        v.x = scalar_load_i32(ent);
        v.y = scalar_load_i32(ent + 1);
        v.z = scalar_load_i32(ent + 2);
        v.w = 0;
        return v;
    };

    // ------------------------------------------------------------ load plans
    // Lane l of a wave fills the 16-byte chunk (wave's base + l) of a stage, so chunk c = tid + NT*i is
    // filled by thread tid in its i-th load; the XOR swizzle of the LDS layout is applied on the
    // source side.  A plan is one 32-bit BYTE offset per load, from the operand's base (A) or the
    // expert's base (B): the loads then take a wave-uniform 64-bit base that moves along K by scalar
    // arithmetic plus that constant per-lane offset, and the K loop spends no vector instruction on
    // addresses.  (The host side rejects operands of 4 GiB or more.)
    auto plan_a = [&](int m0, int mend, bool from_lds, uint32_t (&aoff)[PER_A]) {
#pragma unroll
        for (int i = 0; i < PER_A; ++i) {
            const int c = tid + NT * i;
            const int row = c >> 2, kc = (c & 3) ^ ((row >> 2) & 3);
            int gr = min(m0 + row, mend - 1);
            if (p.a_row_map) gr = from_lds ? s_idx[row] : p.a_row_map[gr];
            aoff[i] = ((uint32_t)gr * (uint32_t)p.lda + kc * 8) * 2u;
        }
    };
    auto plan_b = [&](int n0, uint32_t (&boff)[PER_B]) {
#pragma unroll
        for (int i = 0; i < PER_B; ++i) {
            const int c = tid + NT * i;
            if (B_KC) {
                const int row = c >> 2, kc = (c & 3) ^ ((row >> 2) & 3);
                const int gn = min(n0 + row, p.N - 1);
                boff[i] = ((uint32_t)gn * (uint32_t)p.ldb + kc * 8) * 2u;
            } else {
                constexpr int CPR = BN / 8;
                const int krow = c / CPR, nc = (c % CPR) ^ ((krow & 3) << 2);
                const int col = min(n0 + nc * 8, p.N - 8);
                boff[i] = ((uint32_t)krow * (uint32_t)p.ldb + col) * 2u;
            }
        }
    };
    auto dma_a = [&](int stage, int k0, const uint32_t (&off)[PER_A], auto LO, auto HI) {
        u32x4_t* sa = smem + stage * STAGE + wave * 64;
        const char* a_base = reinterpret_cast<const char*>(p.A + k0);
#pragma unroll
        for (int i = decltype(LO)::value; i < decltype(HI)::value; ++i)
            dma16_sbase(a_base, off[i], (uint32_t)(uintptr_t)(lptr_t)(sa + NT * i));
    };
    auto dma_b = [&](int stage, int k0, const bf16_t* Bb, const uint32_t (&off)[PER_B], auto LO, auto HI) {
        u32x4_t* sb = smem + stage * STAGE + A_CH + wave * 64;
        const char* b_base = reinterpret_cast<const char*>(B_KC ? Bb + k0 : Bb + (long long)k0 * p.ldb);
#pragma unroll
        for (int i = decltype(LO)::value; i < decltype(HI)::value; ++i)
            dma16_sbase(b_base, off[i], (uint32_t)(uintptr_t)(lptr_t)(sb + NT * i));
    };

    mfma_f32x16 acc[TM][TN];

    // ------------------------------------------------------------ fragment readers (see grouped_gemm_wgrad_body)
    const int tr_j = lane & 15, tr_blk = lane >> 4;
    const int tr_col = 16 * (tr_blk & 1) + 4 * (tr_j & 3);
    const int tr_k = 8 * (tr_blk >> 1) + (tr_j >> 2);
    auto read_tr = [&](const u32x4_t* st, auto CPR_, int col0, auto KS) -> u32x4_t {
        constexpr int cpr = decltype(CPR_)::value, ks = decltype(KS)::value;
        const int col = col0 + tr_col;
        const int chunk = (col >> 3) ^ ((tr_j >> 2) << 2);
        const uint32_t addr = (uint32_t)(uintptr_t)(lptr_t)st + (uint32_t)((tr_k * cpr + chunk) * 16 + (col & 7) * 2);
        u32x2_t lo, hi;
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo) : "v"(addr), "i"(ks * 16 * cpr * 16));
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(addr), "i"((ks * 16 + 4) * cpr * 16));
        return u32x4_t{lo[0], lo[1], hi[0], hi[1]};
    };
    auto read_a = [&](const u32x4_t* sa, auto KS, frag_t (&fa)[TM], auto LIVE) {
        constexpr int ks = decltype(KS)::value;
#pragma unroll
        for (int t = 0; t < decltype(LIVE)::value; ++t) {
            const int row = wm * WTM + t * 32 + lj;
            const int kc = ks * 2 + lg;
            fa[t] = __builtin_bit_cast(frag_t, sa[row * 4 + (kc ^ ((row >> 2) & 3))]);
        }
    };
    auto read_b = [&](const u32x4_t* sb, auto KS, frag_t (&fb)[TN]) {
        constexpr int ks = decltype(KS)::value;
#pragma unroll
        for (int t = 0; t < TN; ++t) {
            u32x4_t r;
            if (B_KC) {
                const int row = wn * WTN + t * 32 + lj;
                const int kc = ks * 2 + lg;
                r = sb[row * 4 + (kc ^ ((row >> 2) & 3))];
            } else {
                r = read_tr(sb, std::integral_constant<int, BN / 8>{}, wn * WTN + t * 32, KS);
            }
            fb[t] = __builtin_bit_cast(frag_t, r);
        }
    };
    auto settle = [&](frag_t (&fb)[TN]) {
        if (B_KC) return;
        asm volatile("s_waitcnt lgkmcnt(0)");
#pragma unroll
        for (int t = 0; t < TN; ++t) asm volatile("" : "+v"(fb[t]));
    };
    constexpr int N_MFMA = TM * TN;
    static_assert(N_MFMA % 4 == 0, "a K step is issued in four chunks");
    auto mma_quarter = [&](const frag_t (&fa)[TM], const frag_t (&fb)[TN], auto Q, auto LIVE) {
        constexpr int q = decltype(Q)::value;
#pragma unroll
        for (int f = q * (N_MFMA / 4); f < (q + 1) * (N_MFMA / 4); ++f) {
            const int i = f / TN, j = f % TN;
            if (i >= decltype(LIVE)::value) continue;
            acc[i][j] = Elem16<ET>::mfma(fa[i], fb[j], acc[i][j]);
        }
    };

    using IC0 = std::integral_constant<int, 0>;
    using IC1 = std::integral_constant<int, 1>;
    using IC2 = std::integral_constant<int, 2>;
    using IC3 = std::integral_constant<int, 3>;
    using A_HALF = std::integral_constant<int, (PER_A + 1) / 2>;
    using A_ALL = std::integral_constant<int, PER_A>;
    using B_HALF = std::integral_constant<int, (PER_B + 1) / 2>;
    using B_ALL = std::integral_constant<int, PER_B>;
    frag_t fa0[TM], fb0[TN], fa1[TM], fb1[TN];

    // ------------------------------------------------------------ tile state
    // this tile
    int e, m0, mend, nt, n0;
    uint32_t aoff[PER_A], boff[PER_B];
    const bf16_t* Bb;
    // the next tile of this workgroup, if it has one
    bool have_n;
    int pm_n = 0, nt_n = 0;
    int4 tm_n;
    uint32_t aoff_n[PER_A], boff_n[PER_B];
    const bf16_t* Bb_n = p.B;
#pragma unroll
    for (int i = 0; i < PER_A; ++i) aoff_n[i] = 0;
#pragma unroll
    for (int i = 0; i < PER_B; ++i) boff_n[i] = 0;
    {
        int pm = 0;
        nt = 0;
        if (!advance(pm, nt)) return;
        const int4 tm = load_entry(pm);
        e = tm.x;
        m0 = tm.y;
        mend = tm.z;
        have_n = advance(pm_n, nt_n);
        tm_n = have_n ? load_entry(pm_n) : make_int4(0, 0, 1, 0);
    }
    n0 = nt * BN;
    plan_a(m0, mend, false, aoff);
    plan_b(n0, boff);
    Bb = p.B + (long long)e * p.strideB;

    bool loose = false;     // the previous tile issued this tile's first loads and its epilogue stored without edge tests

    // One 32-wide K tile kt of the current tile; g = running K-tile count of this workgroup (stage g % 4).
    //   step A: MFMAs on the ks=0 fragments | fetch the ks=1 fragments | issue the B loads of K tile g+3
    //   wait until K tile g+1 has landed (the loads of g+2, g+3 may stay in flight), barrier
    //   step B: MFMAs on the ks=1 fragments | fetch the ks=0 fragments of K tile g+1 | issue the A loads
    //           of K tile g+4 into the stage just freed
    // LB / LA: 0 = nothing to load, 1 = K tile kt+3 / kt+4 of this tile, 2 = K tile kt+3-KT / kt+4-KT of the next
    auto k_tile = [&](auto LIVE, auto LB, auto LA, auto WAITN, auto NEXT, int kt, int g) {
        constexpr bool idle = decltype(LIVE)::value == 0;
        constexpr int lb = decltype(LB)::value, la = decltype(LA)::value;
        constexpr bool next = decltype(NEXT)::value;
        constexpr int waitn = decltype(WAITN)::value;
        const u32x4_t* sa = smem + (g & 3) * STAGE;
        const u32x4_t* sb = sa + A_CH;
        const int kb = (lb == 2 ? kt + 3 - KT : kt + 3) * BK;
        const int ka = (la == 2 ? kt + 4 - KT : kt + 4) * BK;
        // ---- step A
        if (!idle) settle(fb0);
        read_a(sa, IC1{}, fa1, LIVE);
        mma_quarter(fa0, fb0, IC0{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (!idle) read_b(sb, IC1{}, fb1);
        mma_quarter(fa0, fb0, IC1{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (lb == 1) dma_b((g + 3) & 3, kb, Bb, boff, IC0{}, B_HALF{});
        if (lb == 2) dma_b((g + 3) & 3, kb, Bb_n, boff_n, IC0{}, B_HALF{});
        mma_quarter(fa0, fb0, IC2{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (lb == 1) dma_b((g + 3) & 3, kb, Bb, boff, B_HALF{}, B_ALL{});
        if (lb == 2) dma_b((g + 3) & 3, kb, Bb_n, boff_n, B_HALF{}, B_ALL{});
        mma_quarter(fa0, fb0, IC3{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (waitn == W_AFTER_STORES) {
            // first two K tiles of a tile whose loads went out before the previous tile's epilogue: the
            // stores of that epilogue are younger than the loads awaited here.  When their number is
            // known (a tile without edge tests stores unconditionally) they may stay in flight.
            if (loose) lds_barrier<W_LOOSE>(); else lds_barrier<(NSTAGE - 2) * PER>();
        } else {
            lds_barrier<waitn>();
        }
        __builtin_amdgcn_sched_barrier(0);
        // ---- step B
        const u32x4_t* na = smem + ((g + 1) & 3) * STAGE;
        if (!idle) settle(fb1);
        if (next) read_a(na, IC0{}, fa0, LIVE);
        mma_quarter(fa1, fb1, IC0{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (next && !idle) read_b(na + A_CH, IC0{}, fb0);
        mma_quarter(fa1, fb1, IC1{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (la == 1) dma_a(g & 3, ka, aoff, IC0{}, A_HALF{});
        if (la == 2) dma_a(g & 3, ka, aoff_n, IC0{}, A_HALF{});
        mma_quarter(fa1, fb1, IC2{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
        if (la == 1) dma_a(g & 3, ka, aoff, A_HALF{}, A_ALL{});
        if (la == 2) dma_a(g & 3, ka, aoff_n, A_HALF{}, A_ALL{});
        mma_quarter(fa1, fb1, IC3{}, LIVE);
        __builtin_amdgcn_sched_barrier(0);
    };
    using W0 = std::integral_constant<int, 0>;
    using W1 = std::integral_constant<int, PER>;
    using WFULL = std::integral_constant<int, (NSTAGE - 2) * PER>;
    using WDYN = std::integral_constant<int, W_AFTER_STORES>;
    // The K loop of one tile, for a wave with LIVE 32-row blocks of live rows.  chain: the loop ends by
    // issuing the first loads of the next tile (whose plan is made here, once its row indices are in LDS).
    auto run_tile = [&](auto LIVE, bool chain, int g0) {
        read_a(smem + (g0 & 3) * STAGE, IC0{}, fa0, LIVE);
        if (decltype(LIVE)::value) {
            read_b(smem + (g0 & 3) * STAGE + A_CH, IC0{}, fb0);
            settle(fb0);   // (nothing to overlap with here; every path below then starts with no read outstanding)
        }
        __builtin_amdgcn_sched_barrier(0);
        int kt = 0;
        if (chain) {
            k_tile(LIVE, IC1{}, IC1{}, WDYN{}, T_{}, kt, g0 + kt); ++kt;
            k_tile(LIVE, IC1{}, IC1{}, WDYN{}, T_{}, kt, g0 + kt); ++kt;
            for (; kt < KT - 4; ++kt) k_tile(LIVE, IC1{}, IC1{}, WFULL{}, T_{}, kt, g0 + kt);
            if (decltype(LIVE)::value) settle(fb0);   // before the plan of the next tile is made in this wave's registers
            plan_a(tm_n.y, tm_n.z, true, aoff_n);
            plan_b(nt_n * BN, boff_n);
            Bb_n = p.B + (long long)tm_n.x * p.strideB;
            __builtin_amdgcn_sched_barrier(0);
            k_tile(LIVE, IC1{}, IC2{}, WFULL{}, T_{}, kt, g0 + kt); ++kt;
            k_tile(LIVE, IC2{}, IC2{}, WFULL{}, T_{}, kt, g0 + kt); ++kt;
            k_tile(LIVE, IC2{}, IC2{}, WFULL{}, T_{}, kt, g0 + kt); ++kt;
            k_tile(LIVE, IC2{}, IC2{}, WFULL{}, F_{}, kt, g0 + kt);
        } else {
            for (; kt + NSTAGE < KT; ++kt) k_tile(LIVE, IC1{}, IC1{}, WFULL{}, T_{}, kt, g0 + kt);
            if (kt + NSTAGE == KT) { k_tile(LIVE, IC1{}, IC0{}, WFULL{}, T_{}, kt, g0 + kt); ++kt; }
            if (kt + 3 == KT) { k_tile(LIVE, IC0{}, IC0{}, W1{}, T_{}, kt, g0 + kt); ++kt; }
            if (kt + 2 == KT) { k_tile(LIVE, IC0{}, IC0{}, W0{}, T_{}, kt, g0 + kt); ++kt; }
            k_tile(LIVE, IC0{}, IC0{}, W0{}, F_{}, kt, g0 + kt);
        }
    };

    // ------------------------------------------------------------ the workgroup's tiles
    int g0 = 0, par = 0;
    bool chained = false;   // the previous tile issued this tile's first loads
    for (;;) {
        const bool have_next = have_n;
        const bool chain = have_next && KT >= 8;
        float* s_rs = s_rs2 + par * BM;
        // the row scales of this tile, parked in LDS for its epilogue (visible after the loop's barriers)
        if (EPI != EPI_STORE) {
            if (p.row_scale) {
                dma4_sbase(p.row_scale, (uint32_t)min(m0 + tid % BM, mend - 1) * 4u,
                           (uint32_t)(uintptr_t)(lptr_t)(s_rs + (wave * 64) % BM));
            } else if (tid < BM) {
                s_rs[tid] = 1.0f;
            }
        }
        // the gathered row indices of the next tile
        if (chain && p.a_row_map) {
            dma4_sbase(p.a_row_map, (uint32_t)min(tm_n.y + tid % BM, tm_n.z - 1) * 4u,
                       (uint32_t)(uintptr_t)(lptr_t)(s_idx + wave * 64));
        }
        // and the tile after the next: which one it is, and its entry of the tile map
        int pm_nn = 0, nt_nn = 0;
        const bool have_nn = have_next && advance(pm_nn, nt_nn);
        const int4 tm_nn = have_nn ? load_entry(pm_nn) : make_int4(0, 0, 1, 0);

        if (!chained) {
            // tiles 0..2 and the A half of tile 3 go out, tile 0 is awaited
#pragma unroll
            for (int t = 0; t < NSTAGE - 1; ++t) {
                if (t < KT) {
                    dma_b((g0 + t) & 3, t * BK, Bb, boff, IC0{}, B_ALL{});
                    dma_a((g0 + t) & 3, t * BK, aoff, IC0{}, A_ALL{});
                }
            }
            if (KT > NSTAGE - 1) {
                dma_a((g0 + NSTAGE - 1) & 3, (NSTAGE - 1) * BK, aoff, IC0{}, A_ALL{});
                lds_barrier<(NSTAGE - 2) * PER + PER_A>();
            } else {
                lds_barrier<0>();
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
        {
            // Only the 32-row blocks of this wave that hold live rows are read and multiplied; the count
            // is wave-uniform and picks one copy of the loop (a wave without live rows still issues its
            // share of the loads and meets the barriers).
            const int live_rows = n0 + wn * WTN < p.N ? min(max(mend - (m0 + wm * WTM), 0), WTM) : 0;
            const int live = (live_rows + 31) >> 5;
            static_assert(TM == 2 || TM == 4, "the dispatch below is written for two or four 32-row blocks per wave");
            if (live >= TM) {
                run_tile(std::integral_constant<int, TM>{}, chain, g0);
            } else if (live == 0) {
                run_tile(std::integral_constant<int, 0>{}, chain, g0);
            } else if (live == 1) {
                run_tile(std::integral_constant<int, 1>{}, chain, g0);
            } else {
                if constexpr (TM == 4) {
                    if (live == 2) run_tile(std::integral_constant<int, 2>{}, chain, g0);
                    else run_tile(std::integral_constant<int, 3>{}, chain, g0);
                }
            }
        }

        // ---------------------------------------------------------- epilogue
        // Lane l of tile (i, j) holds column j*32 + l%32 for 16 rows; registers v, v+1 (v even) are
        // rows r, r+1.  Each lane converts its two values to one packed pair, lanes 2c and 2c+1
        // exchange the pairs (DPP) and a byte permute leaves the even lane with columns (2c, 2c+1) of
        // row r and the odd lane with those of row r+1: three VALU operations per 4-byte store.
        // Gated: that pair is (gate, up) of intermediate column c; a second exchange between lanes l
        // and l^2 over two row pairs packs two neighbouring intermediate columns of one row.
        // Addresses are a wave-uniform row base (scalar arithmetic) plus one per-lane 32-bit offset;
        // tiles that lie entirely inside their expert's rows and the matrix take the FULL form
        // without per-store bounds tests.
        const bool tile_full = m0 + BM <= mend && n0 + BN <= p.N;
        // (the lane index passes through an empty asm statement: everything the epilogue derives from
        // it would otherwise be hoisted out of the tile loop and held in registers across the K loops)
        int lane_e = lane;
        asm volatile("" : "+v"(lane_e));
        const int lj = lane_e & 31, lg = lane_e >> 5;
        const int odd1 = lj & 1, odd2 = (lj >> 1) & 1;
        const uint32_t swap_sel = odd1 ? 0x03020706u : 0x05040100u;
        if (EPI == EPI_GATED_BWD) {
            // The accumulators are d_inter[r, c] (c = intermediate column); nothing of it is stored.
            // With (gate, up) = gate_up[r, 2c], gate_up[r, 2c+1] re-read from the forward pass and
            // s = row_scale[r]:  d_gate_up[r, 2c] = s * d * up * act'(gate),  d_gate_up[r, 2c+1] =
            // s * d * act(gate)  (one packed pair per element, no lane exchange needed), and the row
            // sums  sum_c d * up * act(gate)  -- the gradient of s -- are reduced over the tile's columns
            // in a fixed order and written to partials[N tile][row].
            const long long gorg = (long long)(m0 + wm * WTM) * p.ldg + 2 * (n0 + wn * WTN);
            const char* gbase = reinterpret_cast<const char*>(p.G + gorg);
            char* dbase = reinterpret_cast<char*>(p.C + gorg);
            const uint32_t goff = (uint32_t)(4 * lg * p.ldg + 2 * lj) * 2u;
            auto run = [&](auto FULL) {
                constexpr bool full = decltype(FULL)::value;
                // a block = 8 of the 16 values a lane holds of one 32x32 tile (half hh: registers 8hh..8hh+7)
                auto load_block = [&](int i, int j, int hh, uint32_t (&g)[8]) {
                    const bool col_ok = full || (n0 + wn * WTN + j * 32 + lj < p.N);
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int v = 8 * hh + u;
                        const int rr = i * 32 + 8 * (v >> 2) + (v & 3);   // row relative to the wave's origin (+ 4*lg in goff)
                        const bool ok = full || (col_ok && m0 + wm * WTM + rr + 4 * lg < mend);
                        const char* rowp = gbase + ((long long)rr * p.ldg + 2 * j * 32) * 2;
                        g[u] = ok ? *reinterpret_cast<const uint32_t*>(rowp + goff) : 0u;
                    }
                };
                uint32_t gcur[8], gnxt[8];
                load_block(0, 0, 0, gcur);
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    float dot[16];
#pragma unroll
                    for (int v = 0; v < 16; ++v) dot[v] = 0.f;
#pragma unroll
                    for (int jh = 0; jh < 2 * TN; ++jh) {
                        const int j = jh >> 1, hh = jh & 1;
                        // the next block's pairs are requested before this block is worked on
                        constexpr int NB = TM * TN * 2;
                        const int b_next = i * 2 * TN + jh + 1;
                        if (b_next < NB) load_block(b_next / (2 * TN), (b_next % (2 * TN)) >> 1, b_next & 1, gnxt);
                        __builtin_amdgcn_sched_barrier(0);
                        const bool col_ok = full || (n0 + wn * WTN + j * 32 + lj < p.N);
#pragma unroll
                        for (int u = 0; u < 8; ++u) {
                            // (fenced every four elements: left alone, the scheduler interleaves all the
                            // activation chains and their temporaries no longer fit beside the accumulators)
                            if (u == 4) __builtin_amdgcn_sched_barrier(0);
                            const int v = 8 * hh + u;
                            const int rr = i * 32 + 8 * (v >> 2) + (v & 3);
                            const float d = acc[i][j][v];
                            const float gate = Elem16<ET>::lo(gcur[u]), up = Elem16<ET>::hi(gcur[u]);
                            float f, df;
                            act_both_fast<ACT>(gate, f, df);
                            const float sd = s_rs[wm * WTM + rr + 4 * lg] * d;
                            dot[v] += d * up * f;
                            const bool ok = full || (col_ok && m0 + wm * WTM + rr + 4 * lg < mend);
                            if (ok) {
                                char* rowp = dbase + ((long long)rr * p.ldg + 2 * j * 32) * 2;
                                *reinterpret_cast<uint32_t*>(rowp + goff) = Elem16<ET>::pack2(sd * up * df, sd * f);
                            }
                        }
                        __builtin_amdgcn_sched_barrier(0);
                        if (b_next < NB) {
#pragma unroll
                            for (int u = 0; u < 8; ++u) gcur[u] = gnxt[u];
                        }
                    }
                    if (p.partials) {
                        // sum over the 16 lanes of a row group (its 16 columns), then one slot per
                        // (wave column, half-wave group) and tile row
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            float x = dot[v];
                            x += dpp_f32<AMOE_DPP_QUAD_XOR1>(x);
                            x += dpp_f32<AMOE_DPP_QUAD_XOR2>(x);
                            x += dpp_f32<AMOE_DPP_HALF_MIRROR>(x);
                            x += dpp_f32<AMOE_DPP_MIRROR>(x);
                            if ((lane_e & 15) == 0)
                                s_part[(wn * 2 + ((lane_e >> 4) & 1)) * BM + wm * WTM + i * 32 + 8 * (v >> 2) + 4 * lg + (v & 3)] = x;
                        }
                    }
                }
            };
            if (tile_full) run(T_{}); else run(F_{});
            if (p.partials) {
                lds_sync();
                if (tid < BM && m0 + tid < mend) {
                    float tot = 0.f;
#pragma unroll
                    for (int q = 0; q < 2 * WGN; ++q) tot += s_part[q * BM + tid];
                    p.partials[(long long)nt * p.part_stride + m0 + tid] = tot;
                }
            }
        } else {
            // wave-uniform origin of this wave's part of the tile, and the lane's offset from it (bytes)
            const long long worg = (long long)(m0 + wm * WTM) * p.ldc + n0 + wn * WTN;
            const long long worg2 = (long long)(m0 + wm * WTM) * p.ldc2 + ((n0 + wn * WTN) >> 1);
            char* cbase = reinterpret_cast<char*>(p.C + worg);
            char* c2base = EPI == EPI_GATED ? reinterpret_cast<char*>(p.C2 + worg2) : nullptr;
            const uint32_t loff = (uint32_t)((4 * lg + odd1) * p.ldc + (lj & ~1)) * 2u;
            const uint32_t loff2 = EPI == EPI_GATED ? (uint32_t)((4 * lg + 2 * odd2 + odd1) * p.ldc2 + ((lj >> 1) & ~1)) * 2u : 0u;
            const bool want_c = EPI != EPI_GATED || p.C != nullptr;
            auto epilogue = [&](auto FULL) {
                constexpr bool full = decltype(FULL)::value;
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    // gated: the scales of this lane's 8 rows of tile row i, fetched together ahead of
                    // the column loop (one wait for the batch instead of one per use)
                    float sc[4][2];
                    if (EPI == EPI_GATED) {
#pragma unroll
                        for (int v4 = 0; v4 < 4; ++v4)
#pragma unroll
                            for (int u = 0; u < 2; ++u) sc[v4][u] = s_rs[wm * WTM + i * 32 + 8 * v4 + 4 * lg + 2 * u + odd1];
                    }
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        const bool col_ok = full || (n0 + wn * WTN + j * 32 + (lj & ~1) < p.N);
#pragma unroll
                        for (int v = 0; v < 16; v += 4) {
                            const int rq = i * 32 + 8 * (v >> 2);           // first of 8 rows, relative to the wave's origin
                            const int rt = wm * WTM + rq + 4 * lg;          // rows rt..rt+3 of the tile
                            float h[2];
#pragma unroll
                            for (int u = 0; u < 2; ++u) {
                                const uint32_t own = Elem16<ET>::pack2(acc[i][j][v + 2 * u], acc[i][j][v + 2 * u + 1]);
                                const uint32_t got = __builtin_amdgcn_update_dpp(0, own, 0xB1, 0xF, 0xF, true);
                                const uint32_t pk = __builtin_amdgcn_perm(got, own, swap_sel);
                                const bool ok = full || (col_ok && m0 + rt + 2 * u + odd1 < mend);
                                if (EPI == EPI_GATED)
                                    h[u] = sc[v >> 2][u] * Elem16<ET>::hi(pk) * act_fwd_fast<ACT>(Elem16<ET>::lo(pk));
                                if (want_c && ok) {
                                    char* rowp = cbase + ((long long)(rq + 2 * u) * p.ldc + j * 32) * 2;
                                    *reinterpret_cast<uint32_t*>(rowp + loff) = pk;
                                }
                            }
                            if (EPI == EPI_GATED) {
                                // lanes with bit 1 clear keep the first row pair, the others the second
                                const float got = lane_xor2(odd2 ? h[0] : h[1]);
                                const uint32_t hp = odd2 ? Elem16<ET>::pack2(got, h[1]) : Elem16<ET>::pack2(h[0], got);
                                const bool ok = full || (col_ok && m0 + rt + 2 * odd2 + odd1 < mend);
                                if (ok) {
                                    char* rowp = c2base + ((long long)rq * p.ldc2 + j * 16) * 2;
                                    *reinterpret_cast<uint32_t*>(rowp + loff2) = hp;
                                }
                            }
                        }
                    }
                }
            };
            if (tile_full) epilogue(T_{}); else epilogue(F_{});
        }

        if (!have_next) break;
        // ---- the next tile becomes this tile
        e = tm_n.x;
        m0 = tm_n.y;
        mend = tm_n.z;
        nt = nt_n;
        n0 = nt * BN;
        if (chain) {
#pragma unroll
            for (int i = 0; i < PER_A; ++i) aoff[i] = aoff_n[i];
#pragma unroll
            for (int i = 0; i < PER_B; ++i) boff[i] = boff_n[i];
            Bb = Bb_n;
        } else {
            plan_a(m0, mend, false, aoff);
            plan_b(n0, boff);
            Bb = p.B + (long long)e * p.strideB;
        }
        have_n = have_nn;
        pm_n = pm_nn;
        nt_n = nt_nn;
        tm_n = tm_nn;
        chained = chain;
        loose = chain && tile_full;
        g0 += KT;
        par ^= 1;
    }
}

// ------------------------------------------------------------------ host side

template <int BM, int BN, int WGM, int WGN, int MAPS>
__global__ void __launch_bounds__(WGM * WGN * 64)
grouped_gemm_wgrad_bf16_kernel(GemmArgs p)
{
    grouped_gemm_wgrad_body<BM, BN, WGM, WGN, MAPS, bf16_t>(p);
}

// the same kernel on float16 operands (v_mfma_f32_32x32x16_f16)
template <int BM, int BN, int WGM, int WGN, int MAPS>
__global__ void __launch_bounds__(WGM * WGN * 64)
grouped_gemm_wgrad_f16_kernel(GemmArgs p)
{
    grouped_gemm_wgrad_body<BM, BN, WGM, WGN, MAPS, f16_t>(p);
}

template <int BM, int BN, int WGM, int WGN, bool B_KC, int EPI, int ACT>
__global__ void __launch_bounds__(WGM * WGN * 64)
grouped_gemm_rows_bf16_kernel(GemmArgs p)
{
    grouped_gemm_rows_body<BM, BN, WGM, WGN, B_KC, EPI, ACT, bf16_t>(p);
}
template <int BM, int BN, int WGM, int WGN, bool B_KC, int EPI, int ACT>
__global__ void __launch_bounds__(WGM * WGN * 64)
grouped_gemm_rows_f16_kernel(GemmArgs p)
{
    grouped_gemm_rows_body<BM, BN, WGM, WGN, B_KC, EPI, ACT, f16_t>(p);
}

// compute units of the current device (0 if it cannot be read)
static int device_cu_count()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 0;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

template <auto KERN, int THREADS, int LDS_BYTES>
int launch_kernel(const GemmArgs& a, int grid, hipStream_t s)
{
    // The LDS limit is an attribute of the kernel on one device: set once per device (bit d of the
    // mask); setting it twice from racing threads is harmless.
    static std::atomic<unsigned long long> attr_done{0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 63;   // 63: never cached
    if (dev == 63 || !(attr_done.load(std::memory_order_relaxed) >> dev & 1ull)) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(KERN),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        if (err != hipSuccess) {
            amoe_set_error("grouped_gemm: cannot reserve %d bytes of LDS: %s", LDS_BYTES, hipGetErrorString(err));
            return AMOE_ERR_LAUNCH;
        }
        if (dev != 63) attr_done.fetch_or(1ull << dev, std::memory_order_relaxed);
    }
    hipLaunchKernelGGL(KERN, dim3(grid), dim3(THREADS), LDS_BYTES, s, a);
    return amoe_check_launch("grouped_gemm_16bit");
}

// F16_OK = false leaves the float16 instance of this shape out of the library
template <int BM, int BN, int WGM, int WGN, bool A_KC, bool B_KC, int EPI, int ACT, int MAPS = 0, bool F16_OK = true>
int launch_cfg(const GemmArgs& a, int grid, hipStream_t s)
{
    constexpr int NT = WGM * WGN * 64;
    constexpr int stage_bytes = NSTAGE * (BM + BN) * BK * 2;
    if (a.f16 && !F16_OK) {
        amoe_set_error("grouped_gemm: this tile_cfg is not available for float16 with this epilogue");
        return AMOE_ERR_UNSUPPORTED;
    }
    if constexpr (A_KC) {
        // row-grouped: persistent workgroups, as many as fit on the device at once
        constexpr int lds_bytes = stage_bytes + NT * 4 + 2 * BM * 4 + (EPI == EPI_GATED_BWD ? 2 * WGN * BM * 4 : 0);
        constexpr int per_cu = (lds_bytes <= 80 * 1024 && NT <= 256) ? 2 : 1;
        const int cus = device_cu_count();
        AMOE_REQUIRE(cus > 0, AMOE_ERR_LAUNCH, "grouped_gemm: cannot read the number of compute units");
        // (a multiple of 8: every XCD then runs the same number of workgroups; `grid` bounds the number of tiles)
        int g = grid < cus * per_cu ? grid : cus * per_cu;
        g = (g + 7) & ~7;
        if constexpr (F16_OK) {
            if (a.f16) return launch_kernel<grouped_gemm_rows_f16_kernel<BM, BN, WGM, WGN, B_KC, EPI, ACT>, NT, lds_bytes>(a, g, s);
        }
        return launch_kernel<grouped_gemm_rows_bf16_kernel<BM, BN, WGM, WGN, B_KC, EPI, ACT>, NT, lds_bytes>(a, g, s);
    } else {
        if constexpr (F16_OK) {
            if (a.f16) return launch_kernel<grouped_gemm_wgrad_f16_kernel<BM, BN, WGM, WGN, MAPS>, NT, stage_bytes>(a, grid, s);
        }
        return launch_kernel<grouped_gemm_wgrad_bf16_kernel<BM, BN, WGM, WGN, MAPS>, NT, stage_bytes>(a, grid, s);
    }
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
        case 3:
            // four waves with 256 accumulator registers each leave the gated-backward epilogue no
            // room for its operands: that shape is not built for it
            if constexpr (EPI == EPI_GATED_BWD) {
                amoe_set_error("grouped_gemm: tile_cfg 3 is not available with the gated-backward epilogue");
                return AMOE_ERR_UNSUPPORTED;
            } else {
                // (in float16 the conversions of the epilogues do not fit beside 256 accumulators in the
                // row-grouped kernel: bfloat16 only there)
                return launch_cfg<256, 256, 2, 2, A_KC, B_KC, EPI, ACT, MAPS, !A_KC>(a, grid, s);
            }
        case 5:
            if constexpr (EPI == EPI_GATED_BWD) {   // spills as well (four tile columns per wave)
                amoe_set_error("grouped_gemm: tile_cfg 5 is not available with the gated-backward epilogue");
                return AMOE_ERR_UNSUPPORTED;
            } else {
                return launch_cfg<256, 256, 4, 2, A_KC, B_KC, EPI, ACT, MAPS>(a, grid, s);
            }
        case 2: return launch_cfg<256, 128, 2, 2, A_KC, B_KC, EPI, ACT, MAPS>(a, grid, s);
        default: return launch_cfg<256, 256, 2, 4, A_KC, B_KC, EPI, ACT, MAPS>(a, grid, s);  // 8 waves, 128x64 per wave
    }
}

}  // namespace

// super-tile shape and grid size for `m_tiles` (upper bound) x `n_ntiles` tiles
static int set_supertiles(GemmArgs& a, long long m_tiles, long long* grid)
{
    // at most 8 N tiles per super-tile, the N super-columns of equal width (11 -> 6 + 5, not 8 + 3)
    const int n_super = (a.n_ntiles + 7) / 8;
    a.gn = (a.n_ntiles + n_super - 1) / n_super;
    a.gm = 32 / a.gn;
    // weight gradient: when all tiles of one expert fit in one round of an XCD's 32 CUs, the
    // expert is the super-tile, so its rows are fetched into one L2 only
    if (a.n_mt > 0 && (long long)a.n_mt * a.n_ntiles <= 32) {
        a.gm = a.n_mt;
        a.gn = a.n_ntiles;
    }
    a.sn = (a.n_ntiles + a.gn - 1) / a.gn;
    const long long sm = (m_tiles + a.gm - 1) / a.gm;
    const long long supers = sm * a.sn;
    *grid = 8 * ((supers + 7) / 8) * a.gm * a.gn;
    AMOE_REQUIRE(*grid < (1ll << 31), AMOE_ERR_UNSUPPORTED, "grouped_gemm: grid too large");
    return AMOE_OK;
}

// workspace: [0,16) tile count, then one int4 per M tile for the smallest tile height (64)
static inline int ws_max_mtiles(int R, int E, int bm) { return R / bm + E + 1; }

int amoe_build_tile_map(const int32_t* offsets, int R, int E, int bm, void* workspace, size_t workspace_bytes,
                        const int4** tile_map, const int32_t** n_mtiles, int* max_mtiles, hipStream_t s, bool ready);

#if AMOE_PART(3)
AMOE_EXPORT size_t amoe_grouped_gemm_workspace_bytes(int R, int E)
{
    if (R <= 0 || E <= 0) return 0;
    return 16 + sizeof(int4) * (size_t)ws_max_mtiles(R, E, 64);
}

// ready: the workspace already holds the map for these arguments (AMOE_TILE_MAP_READY); nothing is launched
int amoe_build_tile_map(const int32_t* offsets, int R, int E, int bm, void* workspace, size_t workspace_bytes,
                        const int4** tile_map, const int32_t** n_mtiles, int* max_mtiles, hipStream_t s, bool ready)
{
    AMOE_REQUIRE(workspace_bytes >= amoe_grouped_gemm_workspace_bytes(R, E), AMOE_ERR_WORKSPACE,
                 "grouped_gemm: workspace %zu < %zu bytes", workspace_bytes, amoe_grouped_gemm_workspace_bytes(R, E));
    int32_t* cnt = (int32_t*)workspace;
    int4* map = (int4*)((char*)workspace + 16);
    *max_mtiles = ws_max_mtiles(R, E, bm);
    *tile_map = map;
    *n_mtiles = cnt;
    if (ready) return AMOE_OK;
    hipLaunchKernelGGL(tile_map_kernel, dim3(1), dim3(512), 0, s, offsets, E, bm, map, cnt, *max_mtiles);
    return amoe_check_launch("tile_map");
}

// Where the tile map of a row-grouped GEMM lives inside its workspace and how tall its tiles are, for a
// caller that builds the map itself (the permutation plan): the float32 kernels use 64-row tiles.
int amoe_tile_map_layout(int R, int E, int dtype, int tile_cfg, void* workspace, size_t workspace_bytes, int4** tile_map,
                         int32_t** n_mtiles, int* bm, int* max_mtiles)
{
    AMOE_REQUIRE(dtype == AMOE_F32 || dtype == AMOE_BF16 || dtype == AMOE_F16, AMOE_ERR_BAD_ARG, "tile map: bad dtype %d", dtype);
    const int shape = tile_cfg & ~AMOE_TILE_MAP_READY;
    AMOE_REQUIRE(tile_cfg >= 0 && shape <= 5 && shape != 4, AMOE_ERR_BAD_ARG, "tile map: bad tile_cfg %d", tile_cfg);
    AMOE_REQUIRE(R > 0 && E > 0 && E <= AMOE_MAX_EXPERTS, AMOE_ERR_BAD_ARG, "tile map: bad sizes R=%d E=%d", R, E);
    AMOE_REQUIRE(workspace_bytes >= amoe_grouped_gemm_workspace_bytes(R, E), AMOE_ERR_WORKSPACE,
                 "tile map: workspace %zu < %zu bytes", workspace_bytes, amoe_grouped_gemm_workspace_bytes(R, E));
    *bm = dtype == AMOE_F32 ? 64 : pick_cfg(shape).bm;
    *max_mtiles = ws_max_mtiles(R, E, *bm);
    *n_mtiles = (int32_t*)workspace;
    *tile_map = (int4*)((char*)workspace + 16);
    return AMOE_OK;
}

#endif

// rows mode driver shared by the three row-grouped entry points
template <bool B_KC, int EPI, int ACT>
static int run_rows_bf16(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C,
                         void* C2, const float* row_scale, int R, int E, int Kred, int N, int ldb, long long strideB, void* workspace,
                         size_t workspace_bytes, int tile_cfg, hipStream_t s, int dtype, const void* G = nullptr, float* partials = nullptr)
{
    const bool map_ready = (tile_cfg & AMOE_TILE_MAP_READY) != 0;
    tile_cfg &= ~AMOE_TILE_MAP_READY;
    TileCfg tc = pick_cfg(tile_cfg);
    // the kernel addresses A (at most R source rows) and one expert of B with 32-bit byte offsets
    AMOE_REQUIRE((unsigned long long)R * (unsigned long long)Kred * 2ull < (1ull << 32) &&
                     (unsigned long long)Kred * (unsigned long long)N * 2ull < (1ull << 32),
                 AMOE_ERR_UNSUPPORTED, "grouped_gemm: operand of 4 GiB or more (R=%d, K=%d, N=%d)", R, Kred, N);
    GemmArgs a = {};
    int max_mtiles = 0;
    int rc = amoe_build_tile_map(offsets, R, E, tc.bm, workspace, workspace_bytes, &a.tile_map, &a.n_mtiles,
                                 &max_mtiles, s, map_ready);
    if (rc) return rc;
    a.A = (const bf16_t*)A;
    a.B = (const bf16_t*)B;
    a.C = (bf16_t*)C;
    a.C2 = (bf16_t*)C2;
    a.f16 = dtype == AMOE_F16;
    a.a_row_map = a_row_map;
    a.row_scale = row_scale;
    a.offsets = offsets;
    a.lda = Kred;
    a.ldb = ldb;
    a.ldc = EPI == EPI_GATED_BWD ? 2 * N : N;
    a.ldc2 = N / 2;
    a.G = (const bf16_t*)G;
    a.ldg = 2 * N;
    a.partials = partials;
    a.part_stride = R;
    a.strideB = strideB;
    a.strideC = 0;
    a.E = E;
    a.Kd = Kred;
    a.M = R;
    a.N = N;
    a.n_ntiles = (N + tc.bn - 1) / tc.bn;
    a.n_mt = 0;
    long long grid = 0;
    a.max_mtiles = max_mtiles;
    rc = set_supertiles(a, max_mtiles, &grid);
    if (rc) return rc;
    return launch_any<true, B_KC, EPI, ACT>(a, tile_cfg, (int)grid, s);
}

#if AMOE_PART(0)
int amoe_bf16_gateup_act(const void* xp, const int32_t* a_row_map, const void* w, const int32_t* offsets, void* gate_up,
                         void* inter, const float* row_scale, int R, int E, int H, int I, int act, void* workspace, size_t workspace_bytes,
                         int tile_cfg, hipStream_t s, int dtype)
{
    AMOE_DISPATCH_ACT(act, return (run_rows_bf16<false, EPI_GATED, ACT>(xp, a_row_map, w, offsets, gate_up, inter, row_scale, R, E, H,
                                                                        2 * I, 2 * I, (long long)H * 2 * I, workspace,
                                                                        workspace_bytes, tile_cfg, s, dtype)))
    return AMOE_ERR_BAD_ARG;
}

#endif

#if AMOE_PART(1)
int amoe_bf16_nn(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C, int R, int E,
                 int Kd, int N, void* workspace, size_t workspace_bytes, int tile_cfg, hipStream_t s, int dtype)
{
    return run_rows_bf16<false, EPI_STORE, 0>(A, a_row_map, B, offsets, C, nullptr, nullptr, R, E, Kd, N, N, (long long)Kd * N,
                                              workspace, workspace_bytes, tile_cfg, s, dtype);
}

// C[rows_e, :Kd] = A[rows_e, :N] @ B[e]^T with B [E, Kd, N]: the reduction runs over N
int amoe_bf16_nt(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C, int R, int E,
                 int Kd, int N, void* workspace, size_t workspace_bytes, int tile_cfg, hipStream_t s, int dtype)
{
    return run_rows_bf16<true, EPI_STORE, 0>(A, a_row_map, B, offsets, C, nullptr, nullptr, R, E, /*Kred=*/N, /*N out=*/Kd,
                                             /*ldb=*/N, (long long)Kd * N, workspace, workspace_bytes, tile_cfg, s, dtype);
}

#endif

#if AMOE_PART(2)
// d_gate_up [R, 2I] and the row sums of the score gradient from dy rows [., H], w_down [E, I, H] and the
// forward's gate_up [R, 2I]: the data gradient of the down projection with the backward of the gated
// activation as its epilogue.  The reduction runs over H, the output columns are the I intermediate columns.
int amoe_bf16_nt_gated_bwd(const void* dy, const int32_t* a_row_map, const void* w_down, const int32_t* offsets,
                           const void* gate_up, const float* row_scale, void* d_gate_up, float* partials, int R, int E,
                           int I, int H, int act, void* workspace, size_t workspace_bytes, int tile_cfg, hipStream_t s, int dtype)
{
    AMOE_DISPATCH_ACT(act, return (run_rows_bf16<true, EPI_GATED_BWD, ACT>(dy, a_row_map, w_down, offsets, d_gate_up, nullptr,
                                                                           row_scale, R, E, /*Kred=*/H, /*N out=*/I, /*ldb=*/H,
                                                                           (long long)I * H, workspace, workspace_bytes,
                                                                           tile_cfg, s, dtype, gate_up, partials)))
    return AMOE_ERR_BAD_ARG;
}

#endif

#if AMOE_PART(3)
// number of row-sum partials per routed row that amoe_bf16_nt_gated_bwd writes: one per N tile
int amoe_bf16_gated_bwd_parts(int I, int tile_cfg)
{
    TileCfg tc = pick_cfg(tile_cfg & ~AMOE_TILE_MAP_READY);
    return (I + tc.bn - 1) / tc.bn;
}

int amoe_bf16_wgrad(const void* A, const int32_t* a_row_map, const void* B, const int32_t* b_row_map,
                    const int32_t* offsets, void* C, int R, int E, int Kd, int N, int tile_cfg, hipStream_t s, int dtype)
{
    tile_cfg &= ~AMOE_TILE_MAP_READY;   // no tile map in the weight gradient
    TileCfg tc = pick_cfg(tile_cfg);
    GemmArgs a = {};
    a.f16 = dtype == AMOE_F16;
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
#endif
