// Ragged grouped GEMMs in float32 on v_mfma_f32_32x32x2_f32 (full-precision FMA in the
// matrix core).  One 64x64x16 kernel serves the three layouts; operands are staged in LDS
// K-major ([k][m]) so that the one-float-per-lane MFMA operands are read conflict-free
// whatever the layout in memory.  This is the path of the small float32 configuration; the
// bf16 kernels are the performance path.
#include "amoe_common.h"

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float mfma_f32x16;

int amoe_build_tile_map(const int32_t* offsets, int R, int E, int bm, void* workspace, size_t workspace_bytes,
                        const int4** tile_map, const int32_t** n_mtiles, int* max_mtiles, hipStream_t s, bool ready);

namespace {

constexpr int BM = 64, BN = 64, BK = 16, NT = 256, PAD = 4;

struct GemmArgsF32 {
    const float* A;
    const float* B;
    float* C;
    const int32_t* a_row_map;
    const int32_t* b_row_map;  // weight gradient only
    const int32_t* offsets;
    const int4* tile_map;
    const int32_t* n_mtiles;
    int lda, ldb, ldc;
    long long strideB, strideC;
    int E, Kd, M, N, n_ntiles, n_mt;
};

template <bool A_KC, bool B_KC>
__global__ void __launch_bounds__(NT)
grouped_gemm_f32_kernel(GemmArgsF32 p)
{
    constexpr bool WGRAD = !A_KC;
    __shared__ float As[BK][BM + PAD];
    __shared__ float Bs[BK][BN + PAD];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lj = lane & 31, lg = lane >> 5;

    const int q = blockIdx.x;
    const int pm = q / p.n_ntiles;
    const int nt = q - pm * p.n_ntiles;
    int e, m0, mend, k_len;
    int r0 = 0;
    if (!WGRAD) {
        if (pm >= *p.n_mtiles) return;
        int4 tm = p.tile_map[pm];
        e = tm.x;
        m0 = tm.y;
        mend = tm.z;
        k_len = p.Kd;
    } else {
        e = pm / p.n_mt;
        if (e >= p.E) return;
        m0 = (pm - e * p.n_mt) * BM;
        mend = p.M;
        r0 = p.offsets[e];
        k_len = p.offsets[e + 1] - r0;
    }
    const int n0 = nt * BN;
    const float* Ab = WGRAD ? p.A + (long long)r0 * p.lda : p.A;
    const float* Bb = WGRAD ? p.B + (long long)r0 * p.ldb : p.B + (long long)e * p.strideB;

    // per-thread source coordinates
    long long a_src;
    int a_col = 0, b_col = 0;  // column offsets of the gathered weight-gradient operands
    int a_k;  // k offset inside the tile
    if (A_KC) {
        const int m = tid >> 2;
        a_k = (tid & 3) * 4;
        int gr = min(m0 + m, mend - 1);
        if (p.a_row_map) gr = p.a_row_map[gr];
        a_src = (long long)gr * p.lda + a_k;
    } else {
        a_k = tid >> 4;
        const int m4 = (tid & 15) * 4;
        a_col = min(m0 + m4, p.M - 4);
        a_src = (long long)a_k * p.lda + a_col;
    }
    long long b_src;
    int b_k;
    if (B_KC) {
        const int n = tid >> 2;
        b_k = (tid & 3) * 4;
        b_src = (long long)min(n0 + n, p.N - 1) * p.ldb + b_k;
    } else {
        b_k = tid >> 4;
        const int n4 = (tid & 15) * 4;
        b_col = min(n0 + n4, p.N - 4);
        b_src = (long long)b_k * p.ldb + b_col;
    }

    mfma_f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.f;

    const f32x4_t zero4 = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < k_len; k0 += BK) {
        f32x4_t va, vb;
        if (A_KC) {
            va = (k0 + a_k < k_len) ? *reinterpret_cast<const f32x4_t*>(Ab + a_src + k0) : zero4;
        } else if (p.a_row_map) {
            va = (k0 + a_k < k_len) ? *reinterpret_cast<const f32x4_t*>(
                                          p.A + (long long)p.a_row_map[r0 + k0 + a_k] * p.lda + a_col)
                                    : zero4;
        } else {
            va = (k0 + a_k < k_len) ? *reinterpret_cast<const f32x4_t*>(Ab + a_src + (long long)k0 * p.lda) : zero4;
        }
        if (B_KC) {
            vb = (k0 + b_k < k_len) ? *reinterpret_cast<const f32x4_t*>(Bb + b_src + k0) : zero4;
        } else if (WGRAD && p.b_row_map) {
            vb = (k0 + b_k < k_len) ? *reinterpret_cast<const f32x4_t*>(
                                          p.B + (long long)p.b_row_map[r0 + k0 + b_k] * p.ldb + b_col)
                                    : zero4;
        } else {
            vb = (k0 + b_k < k_len) ? *reinterpret_cast<const f32x4_t*>(Bb + b_src + (long long)k0 * p.ldb) : zero4;
        }
        __syncthreads();  // previous step's reads are done
        if (A_KC) {
            const int m = tid >> 2;
#pragma unroll
            for (int i = 0; i < 4; ++i) As[a_k + i][m] = va[i];
        } else {
            *reinterpret_cast<f32x4_t*>(&As[a_k][(tid & 15) * 4]) = va;
        }
        if (B_KC) {
            const int n = tid >> 2;
#pragma unroll
            for (int i = 0; i < 4; ++i) Bs[b_k + i][n] = vb[i];
        } else {
            *reinterpret_cast<f32x4_t*>(&Bs[b_k][(tid & 15) * 4]) = vb;
        }
        __syncthreads();
#pragma unroll
        for (int kb = 0; kb < BK; kb += 2) {
            const float a = As[kb + lg][wm * 32 + lj];
            const float b = Bs[kb + lg][wn * 32 + lj];
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
        }
    }

    float* Cb = WGRAD ? p.C + (long long)e * p.strideC : p.C;
    const int col = n0 + wn * 32 + lj;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int row = m0 + wm * 32 + 8 * (v >> 2) + 4 * lg + (v & 3);
        if (row < mend && col < p.N) Cb[(long long)row * p.ldc + col] = acc[v];
    }
}

}  // namespace

// rows mode: C[rows_e, :N] = A[rows_e, :Kred] @ op(B[e]);  b_kc selects B stored [N,Kred]
int amoe_f32_rows(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C, int R, int E,
                  int Kred, int N, int ldb, long long strideB, bool b_kc, void* workspace, size_t workspace_bytes,
                  bool map_ready, hipStream_t s)
{
    GemmArgsF32 a = {};
    int max_mtiles = 0;
    // map_ready (AMOE_TILE_MAP_READY): the workspace already holds the map for these offsets, nothing is launched
    int rc = amoe_build_tile_map(offsets, R, E, BM, workspace, workspace_bytes, &a.tile_map, &a.n_mtiles, &max_mtiles, s,
                                 map_ready);
    if (rc) return rc;
    a.A = (const float*)A;
    a.B = (const float*)B;
    a.C = (float*)C;
    a.a_row_map = a_row_map;
    a.offsets = offsets;
    a.lda = Kred;
    a.ldb = ldb;
    a.ldc = N;
    a.strideB = strideB;
    a.E = E;
    a.Kd = Kred;
    a.M = R;
    a.N = N;
    a.n_ntiles = (N + BN - 1) / BN;
    const long long grid = (long long)max_mtiles * a.n_ntiles;
    AMOE_REQUIRE(grid < (1ll << 31), AMOE_ERR_UNSUPPORTED, "grouped_gemm(f32): grid too large");
    if (b_kc)
        hipLaunchKernelGGL((grouped_gemm_f32_kernel<true, true>), dim3((int)grid), dim3(NT), 0, s, a);
    else
        hipLaunchKernelGGL((grouped_gemm_f32_kernel<true, false>), dim3((int)grid), dim3(NT), 0, s, a);
    return amoe_check_launch("grouped_gemm_f32");
}

int amoe_f32_wgrad(const void* A, const int32_t* a_row_map, const void* B, const int32_t* b_row_map,
                   const int32_t* offsets, void* C, int R, int E, int Kd, int N, hipStream_t s)
{
    GemmArgsF32 a = {};
    a.a_row_map = a_row_map;
    a.b_row_map = b_row_map;
    a.A = (const float*)A;
    a.B = (const float*)B;
    a.C = (float*)C;
    a.offsets = offsets;
    a.lda = Kd;
    a.ldb = N;
    a.ldc = N;
    a.strideC = (long long)Kd * N;
    a.E = E;
    a.M = Kd;
    a.N = N;
    a.n_ntiles = (N + BN - 1) / BN;
    a.n_mt = (Kd + BM - 1) / BM;
    const long long grid = (long long)E * a.n_mt * a.n_ntiles;
    AMOE_REQUIRE(grid < (1ll << 31), AMOE_ERR_UNSUPPORTED, "grouped_gemm_wgrad(f32): grid too large");
    hipLaunchKernelGGL((grouped_gemm_f32_kernel<false, false>), dim3((int)grid), dim3(NT), 0, s, a);
    return amoe_check_launch("grouped_gemm_wgrad_f32");
}
