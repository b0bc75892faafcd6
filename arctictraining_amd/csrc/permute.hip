// Deterministic token-to-expert permutation plan: a stable counting sort of the k-major
// flattened assignment vector, in three launches
//   1. per-chunk expert histograms (LDS counters),
//   2. a one-block scan over chunks and experts (counts, offsets, per-chunk bases),
//   3. per-chunk ranking in ascending slot order (ballot match inside a wavefront, LDS
//      running counters across steps) and the scatter of the three index maps.
// A chunk is kChunk consecutive flat slots f = k*T + t handled by ONE wavefront, so the
// order inside an expert is ascending f by construction, with no global atomics.
#include "amoe_common.h"

#include <atomic>

namespace {

constexpr int kChunk = 512;         // flat slots per wavefront
constexpr int kWavesPerBlock = 4;   // independent chunks per block

__device__ __forceinline__ int load_expert(const int32_t* assign, int f, int T, int K, int E)
{
    int k = f / T;
    int t = f - k * T;
    int e = assign[(size_t)t * K + k];
    return min(max(e, 0), E - 1);  // memory safety for caller-supplied assignments
}

__global__ void __launch_bounds__(kWavesPerBlock * AMOE_WAVE)
permute_hist_kernel(const int32_t* __restrict__ assign, int T, int K, int E, int R, int n_chunks,
                    int32_t* __restrict__ chunk_counts)
{
    __shared__ int32_t cnt[kWavesPerBlock][AMOE_MAX_EXPERTS];
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = blockIdx.x * kWavesPerBlock + w;
    for (int e = lane; e < E; e += 64) cnt[w][e] = 0;
    __syncthreads();
    if (c < n_chunks) {
        const int f0 = c * kChunk;
        const int f1 = min(f0 + kChunk, R);
        for (int f = f0 + lane; f < f1; f += 64) atomicAdd(&cnt[w][load_expert(assign, f, T, K, E)], 1);
    }
    __syncthreads();
    if (c < n_chunks)
        for (int e = lane; e < E; e += 64) chunk_counts[(size_t)c * E + e] = cnt[w][e];
}

// One block of 1024 threads: with EP = E rounded up to a power of two, thread t works for
// expert t % EP on the (t / EP)-th slice of the chunks, so that the walk over chunks (the only
// sequential part) is 1024 / EP ways parallel and every load is coalesced over experts.  A
// thread holds its slice of counts in registers between the two passes (kScanBatch at a time):
// the exclusive bases overwrite the counts in place, and loads issued after such a store cannot
// be moved ahead of it, which would turn the second pass into a chain of dependent round trips.
// When tile_map is non-null the block also writes the row-grouped GEMMs' tile map (one int4
// {expert, first row, end row, 0} per `bm`-row tile, {-1,0,0,0} past the last) and its tile count.
constexpr int kScanThreads = 1024;
constexpr int kScanBatch = 16;

__global__ void __launch_bounds__(kScanThreads)
permute_scan_kernel(int32_t* __restrict__ chunk_counts /* in: counts, out: exclusive base inside expert */,
                    int E, int EP, int n_chunks, int32_t* __restrict__ counts, int32_t* __restrict__ offsets,
                    int4* __restrict__ tile_map, int32_t* __restrict__ n_mtiles, int bm, int max_mtiles)
{
    __shared__ int32_t part[kScanThreads];       // [slice][EP]
    __shared__ int32_t tot[AMOE_MAX_EXPERTS + 1];
    __shared__ int32_t tstart[AMOE_MAX_EXPERTS + 1];
    const int t = threadIdx.x;
    const int e = t & (EP - 1);
    const int g = t / EP;
    const int G = kScanThreads / EP;
    const int per = (n_chunks + G - 1) / G;
    const int c0 = min(g * per, n_chunks), c1 = min(c0 + per, n_chunks);
    int sum = 0;
    if (e < E)
        for (int cb = c0; cb < c1; cb += kScanBatch) {
            int v[kScanBatch];
#pragma unroll
            for (int i = 0; i < kScanBatch; ++i) v[i] = cb + i < c1 ? chunk_counts[(size_t)(cb + i) * E + e] : 0;
#pragma unroll
            for (int i = 0; i < kScanBatch; ++i) sum += v[i];
        }
    part[t] = sum;
    __syncthreads();
    int run = 0;
    for (int gg = 0; gg < g; ++gg) run += part[gg * EP + e];
    if (g == G - 1 && e < E) {
        counts[e] = run + sum;
        tot[e] = run + sum;
    }
    if (e < E)
        for (int cb = c0; cb < c1; cb += kScanBatch) {
            int v[kScanBatch];
#pragma unroll
            for (int i = 0; i < kScanBatch; ++i) v[i] = cb + i < c1 ? chunk_counts[(size_t)(cb + i) * E + e] : 0;
#pragma unroll
            for (int i = 0; i < kScanBatch; ++i) {
                if (cb + i < c1) chunk_counts[(size_t)(cb + i) * E + e] = run;
                run += v[i];
            }
        }
    if (t < AMOE_MAX_EXPERTS && t >= E) tot[t] = 0;
    __syncthreads();
    // Inclusive scan over the experts of the row counts, by ONE wavefront: 8 consecutive entries per
    // lane serially, the lane sums by cross-lane shuffles (a block-wide Hillis-Steele scan costs 18
    // barriers of 16 wavefronts).
    static_assert(AMOE_MAX_EXPERTS == 8 * AMOE_WAVE, "one wavefront scans 8 entries per lane");
    if (t < AMOE_WAVE) {
        int r[8];
        int s_rows = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            r[i] = tot[t * 8 + i];
            s_rows += r[i];
        }
        int in_rows = s_rows;
#pragma unroll
        for (int o = 1; o < AMOE_WAVE; o <<= 1) {
            const int u = __shfl_up(in_rows, o, AMOE_WAVE);
            if (t >= o) in_rows += u;
        }
        int run_rows = in_rows - s_rows;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            run_rows += r[i];
            tot[t * 8 + i] = run_rows;
        }
    }
    __syncthreads();
    if (t < E) offsets[t + 1] = tot[t];
    if (t == 0) offsets[0] = 0;
    if (tile_map == nullptr) return;
    // tot[e] = end row of expert e
    amoe_emit_tile_map<kScanThreads>(tot, 0, E, bm, tile_map, n_mtiles, max_mtiles, tstart);
}

__global__ void __launch_bounds__(kWavesPerBlock * AMOE_WAVE)
permute_scatter_kernel(const int32_t* __restrict__ assign, int T, int K, int E, int R, int n_chunks,
                       const int32_t* __restrict__ chunk_base, const int32_t* __restrict__ offsets,
                       const float* __restrict__ scores, int32_t* __restrict__ token_of, int32_t* __restrict__ slot_of,
                       int32_t* __restrict__ row_of, float* __restrict__ scores_perm)
{
    __shared__ int32_t run[kWavesPerBlock][AMOE_MAX_EXPERTS];
    const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int c = blockIdx.x * kWavesPerBlock + w;
    if (c >= n_chunks) return;  // no block-wide barrier below: every wavefront is independent
    for (int e = lane; e < E; e += 64) run[w][e] = offsets[e] + chunk_base[(size_t)c * E + e];
    __builtin_amdgcn_wave_barrier();
    const int f0 = c * kChunk;
    const int f1 = min(f0 + kChunk, R);
    const unsigned long long lt_mask = (1ull << lane) - 1ull;
    for (int fb = f0; fb < f1; fb += 64) {
        const int f = fb + lane;
        const bool valid = f < f1;
        const int e = valid ? load_expert(assign, f, T, K, E) : 0;
        // lanes that hold the same expert
        unsigned long long same = __ballot(valid);
#pragma unroll
        for (int b = 0; b < 9; ++b) {
            unsigned long long bits = __ballot((e >> b) & 1);
            same &= ((e >> b) & 1) ? bits : ~bits;
        }
        const int rank = __popcll(same & lt_mask);
        int row = 0;
        if (valid) row = run[w][e] + rank;
        __builtin_amdgcn_wave_barrier();
        // the highest lane of each group advances the running counter
        if (valid && (same >> lane) == 1ull) run[w][e] = row + 1;
        __builtin_amdgcn_wave_barrier();
        if (valid) {
            int k = f / T;
            int t = f - k * T;
            token_of[row] = t;
            slot_of[row] = f;
            row_of[(size_t)t * K + k] = row;
            if (scores_perm) scores_perm[row] = scores[(size_t)t * K + k];
        }
    }
}

}  // namespace

static inline int permute_chunks(int R) { return (R + kChunk - 1) / kChunk; }

AMOE_EXPORT size_t amoe_permute_workspace_bytes(int R, int E)
{
    if (R <= 0 || E <= 0) return 0;
    return (size_t)permute_chunks(R) * (size_t)E * sizeof(int32_t);
}

// argument checks shared by the two entry points (all before the first HIP call)
static int check_plan_args(const int32_t* assign, const float* scores, int T, int K, int E, int32_t* counts,
                           int32_t* offsets, int32_t* token_of, int32_t* slot_of, int32_t* row_of, float* scores_perm)
{
    AMOE_REQUIRE(assign && counts && offsets && token_of && slot_of && row_of, AMOE_ERR_BAD_ARG,
                 "permute_plan: null pointer");
    AMOE_REQUIRE(!scores_perm || scores, AMOE_ERR_BAD_ARG, "permute_plan: scores_perm needs scores");
    AMOE_REQUIRE(T > 0 && K > 0 && E > 0, AMOE_ERR_BAD_ARG, "permute_plan: T, K, E must be positive");
    AMOE_REQUIRE(E <= AMOE_MAX_EXPERTS, AMOE_ERR_UNSUPPORTED, "permute_plan: E=%d exceeds %d", E, AMOE_MAX_EXPERTS);
    AMOE_REQUIRE((long long)T * K < (1ll << 31), AMOE_ERR_UNSUPPORTED, "permute_plan: T*K does not fit int32");
    return AMOE_OK;
}

// the three launches; cc = per-chunk expert counts, permute_chunks(R) * E int32 (every entry is
// written by the histogram kernel before it is read: nothing has to be cleared)
static int launch_plan(const int32_t* assign, const float* scores, int T, int K, int E, int32_t* counts,
                       int32_t* offsets, int32_t* token_of, int32_t* slot_of, int32_t* row_of, float* scores_perm,
                       int32_t* cc, hipStream_t s, int4* tile_map = nullptr, int32_t* n_mtiles = nullptr, int bm = 1,
                       int max_mtiles = 0)
{
    const int R = T * K;
    const int n_chunks = permute_chunks(R);
    const int n_blocks = (n_chunks + kWavesPerBlock - 1) / kWavesPerBlock;
    hipLaunchKernelGGL(permute_hist_kernel, dim3(n_blocks), dim3(kWavesPerBlock * AMOE_WAVE), 0, s, assign, T, K, E, R,
                       n_chunks, cc);
    int EP = 1;
    while (EP < E) EP <<= 1;
    hipLaunchKernelGGL(permute_scan_kernel, dim3(1), dim3(kScanThreads), 0, s, cc, E, EP, n_chunks, counts, offsets,
                       tile_map, n_mtiles, bm, max_mtiles);
    hipLaunchKernelGGL(permute_scatter_kernel, dim3(n_blocks), dim3(kWavesPerBlock * AMOE_WAVE), 0, s, assign, T, K, E,
                       R, n_chunks, cc, offsets, scores, token_of, slot_of, row_of, scores_perm);
    return amoe_check_launch("permute_plan");
}

AMOE_EXPORT int amoe_permute_plan(const int32_t* assign, const float* scores, int T, int K, int E, int32_t* counts,
                                  int32_t* offsets, int32_t* token_of, int32_t* slot_of, int32_t* row_of,
                                  float* scores_perm, void* workspace, size_t workspace_bytes, void* stream)
{
    int rc = check_plan_args(assign, scores, T, K, E, counts, offsets, token_of, slot_of, row_of, scores_perm);
    if (rc) return rc;
    AMOE_REQUIRE(workspace, AMOE_ERR_BAD_ARG, "permute_plan: null workspace");
    AMOE_REQUIRE(workspace_bytes >= amoe_permute_workspace_bytes(T * K, E), AMOE_ERR_WORKSPACE,
                 "permute_plan: workspace %zu < %zu bytes", workspace_bytes, amoe_permute_workspace_bytes(T * K, E));
    return launch_plan(assign, scores, T, K, E, counts, offsets, token_of, slot_of, row_of, scores_perm,
                       (int32_t*)workspace, (hipStream_t)stream);
}

// The plan together with the tile map of the row-grouped GEMMs that will run over its offsets: the
// scan kernel holds the offsets anyway, so the map costs no launch of its own.
int amoe_tile_map_layout(int R, int E, int dtype, int tile_cfg, void* workspace, size_t workspace_bytes, int4** tile_map,
                         int32_t** n_mtiles, int* bm, int* max_mtiles);

AMOE_EXPORT int amoe_permute_plan_tiled(const int32_t* assign, const float* scores, int T, int K, int E, int32_t* counts,
                                        int32_t* offsets, int32_t* token_of, int32_t* slot_of, int32_t* row_of,
                                        float* scores_perm, void* workspace, size_t workspace_bytes, void* gemm_workspace,
                                        size_t gemm_workspace_bytes, int dtype, int tile_cfg, void* stream)
{
    int rc = check_plan_args(assign, scores, T, K, E, counts, offsets, token_of, slot_of, row_of, scores_perm);
    if (rc) return rc;
    AMOE_REQUIRE(workspace && gemm_workspace, AMOE_ERR_BAD_ARG, "permute_plan_tiled: null workspace");
    AMOE_REQUIRE(workspace_bytes >= amoe_permute_workspace_bytes(T * K, E), AMOE_ERR_WORKSPACE,
                 "permute_plan_tiled: workspace %zu < %zu bytes", workspace_bytes, amoe_permute_workspace_bytes(T * K, E));
    int4* tile_map = nullptr;
    int32_t* n_mtiles = nullptr;
    int bm = 0, max_mtiles = 0;
    rc = amoe_tile_map_layout(T * K, E, dtype, tile_cfg, gemm_workspace, gemm_workspace_bytes, &tile_map, &n_mtiles, &bm,
                              &max_mtiles);
    if (rc) return rc;
    return launch_plan(assign, scores, T, K, E, counts, offsets, token_of, slot_of, row_of, scores_perm,
                       (int32_t*)workspace, (hipStream_t)stream, tile_map, n_mtiles, bm, max_mtiles);
}

// ------------------------------------------------------------------ the variant that allocates nothing
// The per-chunk counts live in a fixed array in device memory that belongs to the library (each
// GPU the library runs on holds its own copy until the process ends).  Host code never uses the
// array's name as an address: the device address is looked up once per device and kept.
static __device__ __align__(256) int32_t scratch[AMOE_PERMUTE_STATIC_MAX_COUNTS];

static constexpr int kMaxDevices = 64;
static std::atomic<int32_t*> g_scratch_ptr[kMaxDevices];

// device address of `scratch` on the current device (resolved on the first call per device)
static int static_scratch(int32_t** out)
{
    int dev = -1;
    hipError_t err = hipGetDevice(&dev);
    if (err != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        amoe_set_error("permute_plan_static: no usable current device (%s)", hipGetErrorString(err));
        return AMOE_ERR_LAUNCH;
    }
    int32_t* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!ptr) {
        void* sym = nullptr;
        err = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !sym) {
            amoe_set_error("permute_plan_static: cannot resolve the scratch array on device %d: %s", dev,
                           hipGetErrorString(err));
            return AMOE_ERR_LAUNCH;
        }
        ptr = (int32_t*)sym;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // racing threads store the same address
    }
    *out = ptr;
    return AMOE_OK;
}

AMOE_EXPORT int amoe_permute_plan_static(const int32_t* assign, const float* scores, int T, int K, int E,
                                         int32_t* counts, int32_t* offsets, int32_t* token_of, int32_t* slot_of,
                                         int32_t* row_of, float* scores_perm, void* stream)
{
    int rc = check_plan_args(assign, scores, T, K, E, counts, offsets, token_of, slot_of, row_of, scores_perm);
    if (rc) return rc;
    const long long need = (long long)permute_chunks(T * K) * E;
    AMOE_REQUIRE(need <= (long long)AMOE_PERMUTE_STATIC_MAX_COUNTS, AMOE_ERR_UNSUPPORTED,
                 "permute_plan_static: ceil(T*K/%d)*E = %lld exceeds the built-in scratch of %d counters; "
                 "use amoe_permute_plan with a caller workspace",
                 kChunk, need, AMOE_PERMUTE_STATIC_MAX_COUNTS);
    int32_t* cc = nullptr;
    rc = static_scratch(&cc);
    if (rc) return rc;
    return launch_plan(assign, scores, T, K, E, counts, offsets, token_of, slot_of, row_of, scores_perm, cc,
                       (hipStream_t)stream);
}
