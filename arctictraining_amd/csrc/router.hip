// Router softmax / top-k and its backward: one 64-lane wavefront per token, expert values
// spread over lanes (expert e lives in lane e % 64, register e / 64), reductions by
// cross-lane shuffles.  HBM-bound: T*E logits in, T*E probabilities + T*K pairs out.
#include "amoe_common.h"

namespace {

constexpr int kTokensPerBlock = 4;  // 4 wavefronts

// total order used for selection: larger value first, then lower expert index.  The key is
// (monotone bits of the value) << 32 | (0xffffffff - index), maximised.
__device__ __forceinline__ unsigned long long sel_key(float v, int idx)
{
    v = v + 0.0f;  // -0.0 -> +0.0 so that both zeros tie
    uint32_t u = __float_as_uint(v);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return ((unsigned long long)u << 32) | (unsigned long long)(0xffffffffu - (uint32_t)idx);
}

template <int CTRL>
__device__ __forceinline__ unsigned long long max_with_dpp(unsigned long long k)
{
    const uint32_t hi = (uint32_t)(k >> 32), lo = (uint32_t)k;
    const unsigned long long other = ((unsigned long long)dpp_u32<CTRL>(hi) << 32) | dpp_u32<CTRL>(lo);
    return other > k ? other : k;
}

__device__ __forceinline__ unsigned long long row_lane_u64(unsigned long long k, int lane)
{
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(k >> 32), lane);
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)k, lane);
    return ((unsigned long long)hi << 32) | lo;
}

// The same order in 32 bits for bf16 logits: a bf16 value has 16 significant bits, so the upper
// half of the monotone pattern decides, and the lower half is free for the index (E <= 512).
// Half the instructions of the 64-bit key in every arg-max step.
__device__ __forceinline__ uint32_t sel_key32(float v, int idx)
{
    v = v + 0.0f;
    uint32_t u = __float_as_uint(v);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return (u & 0xffff0000u) | (0xffffu - (uint32_t)idx);
}

template <int CTRL>
__device__ __forceinline__ uint32_t max_with_dpp(uint32_t k)
{
    const uint32_t other = dpp_u32<CTRL>(k);
    return other > k ? other : k;
}

__device__ __forceinline__ uint32_t wave_max_key(uint32_t k)
{
    k = max_with_dpp<AMOE_DPP_QUAD_XOR1>(k);
    k = max_with_dpp<AMOE_DPP_QUAD_XOR2>(k);
    k = max_with_dpp<AMOE_DPP_HALF_MIRROR>(k);
    k = max_with_dpp<AMOE_DPP_MIRROR>(k);
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)k, 0), b = (uint32_t)__builtin_amdgcn_readlane((int)k, 16);
    const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)k, 32), d = (uint32_t)__builtin_amdgcn_readlane((int)k, 48);
    const uint32_t ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}

// key type, construction and index extraction per logit type (float16 logits take the 64-bit key:
// their 11 significant bits do not fit the upper half of the float32 pattern)
template <typename T>
struct SelKey {
    typedef unsigned long long type;
    __device__ static __forceinline__ type make(float v, int idx) { return sel_key(v, idx); }
    __device__ static __forceinline__ int index(type k) { return (int)(0xffffffffu - (uint32_t)(k & 0xffffffffull)); }
};
template <>
struct SelKey<bf16_t> {
    typedef uint32_t type;
    __device__ static __forceinline__ type make(float v, int idx) { return sel_key32(v, idx); }
    __device__ static __forceinline__ int index(type k) { return (int)(0xffffu - (k & 0xffffu)); }
};

// wave-uniform maximum of the 64 keys
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long k)
{
    k = max_with_dpp<AMOE_DPP_QUAD_XOR1>(k);
    k = max_with_dpp<AMOE_DPP_QUAD_XOR2>(k);
    k = max_with_dpp<AMOE_DPP_HALF_MIRROR>(k);
    k = max_with_dpp<AMOE_DPP_MIRROR>(k);
    const unsigned long long a = row_lane_u64(k, 0), b = row_lane_u64(k, 16);
    const unsigned long long c = row_lane_u64(k, 32), d = row_lane_u64(k, 48);
    const unsigned long long ab = a > b ? a : b, cd = c > d ? c : d;
    return ab > cd ? ab : cd;
}
__device__ __forceinline__ unsigned long long wave_max_key(unsigned long long k) { return wave_max_u64(k); }

template <typename T, int VPT>
__global__ void __launch_bounds__(kTokensPerBlock * AMOE_WAVE)
router_topk_fwd_kernel(const T* __restrict__ logits, int n_tokens, int E, int K, int normalize,
                       float* __restrict__ probs, int32_t* __restrict__ topk_idx, float* __restrict__ scores)
{
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * kTokensPerBlock + (threadIdx.x >> 6);
    if (t >= n_tokens) return;
    const T* row = logits + (size_t)t * E;

    typedef typename SelKey<T>::type key_t;
    float v[VPT];
    key_t key[VPT];
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        int e = lane + 64 * j;
        bool ok = e < E;
        v[j] = ok ? ElemTraits<T>::load1(row + (ok ? e : 0)) : -INFINITY;
        key[j] = ok ? SelKey<T>::make(v[j], e) : (key_t)0;
    }

    // K rounds of wave-wide arg-max; a taken entry's key drops to 0
    float top_v = 0.f;   // lane k keeps the k-th selected logit
    int top_e = 0;       // lane k keeps the k-th selected expert
    float row_max = 0.f;
    for (int k = 0; k < K; ++k) {
        key_t best = key[0];
#pragma unroll
        for (int j = 1; j < VPT; ++j) best = key[j] > best ? key[j] : best;
        best = wave_max_key(best);
        int e_sel = SelKey<T>::index(best);
        float v_sel = 0.f;
#pragma unroll
        for (int j = 0; j < VPT; ++j) {
            if (lane + 64 * j == e_sel) {
                key[j] = (key_t)0;
                v_sel = v[j];
            }
        }
        // the owning lane broadcasts the logit
        v_sel = row_lane_f32(v_sel, e_sel & 63);   // e_sel is wave-uniform
        if (k == 0) row_max = v_sel;
        if (lane == k) {
            top_v = v_sel;
            top_e = e_sel;
        }
    }

    // softmax in f32 around the row maximum (= the first selected logit)
    float ex[VPT];
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        ex[j] = (lane + 64 * j < E) ? expf(v[j] - row_max) : 0.f;
        part += ex[j];
    }
    const float z = wave_sum(part);
    float* prow = probs + (size_t)t * E;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        int e = lane + 64 * j;
        if (e < E) prow[e] = ex[j] / z;
    }
    // (the division stays an IEEE division: the probabilities are compared with the library softmax)

    float p_sel = (lane < K) ? expf(top_v - row_max) / z : 0.f;
    float s = p_sel;
    if (normalize) {
        float tot = wave_sum(p_sel);
        s = p_sel / tot;
    }
    if (lane < K) {
        topk_idx[(size_t)t * K + lane] = top_e;
        scores[(size_t)t * K + lane] = ElemTraits<T>::round(s);
    }
}

template <typename T, int VPT>
__global__ void __launch_bounds__(kTokensPerBlock * AMOE_WAVE)
router_bwd_kernel(const float* __restrict__ d_scores, const float* __restrict__ probs,
                  const int32_t* __restrict__ topk_idx, const int32_t* __restrict__ counts, int n_tokens, int E,
                  int K, int normalize, float lb_coeff, T* __restrict__ d_logits)
{
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * kTokensPerBlock + (threadIdx.x >> 6);
    if (t >= n_tokens) return;
    const float* prow = probs + (size_t)t * E;

    float p[VPT], dp[VPT];
    float cnt_part = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        int e = lane + 64 * j;
        bool ok = e < E;
        p[j] = ok ? prow[e] : 0.f;
        float c = ok ? (float)counts[e] : 0.f;
        dp[j] = c;  // scaled below once the total is known
        cnt_part += c;
    }
    const float total = wave_sum(cnt_part);
    const float lb = total > 0.f ? lb_coeff / total : 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) dp[j] *= lb;

    // lanes 0..K-1 hold one selected slot each
    int e_k = 0;
    float ds_k = 0.f, p_k = 0.f;
    if (lane < K) {
        e_k = topk_idx[(size_t)t * K + lane];
        ds_k = d_scores[(size_t)t * K + lane];
        p_k = prow[e_k];
    }
    float dptop = ds_k;
    if (normalize) {
        float S = wave_sum(p_k);
        float dot = wave_sum(ds_k * (p_k / S));
        dptop = (ds_k - dot) / S;
    }
    for (int k = 0; k < K; ++k) {
        int e = __shfl(e_k, k, AMOE_WAVE);
        float g = __shfl(dptop, k, AMOE_WAVE);
#pragma unroll
        for (int j = 0; j < VPT; ++j)
            if (lane + 64 * j == e) dp[j] += g;
    }
    float part = 0.f;
#pragma unroll
    for (int j = 0; j < VPT; ++j) part += p[j] * dp[j];
    const float inner = wave_sum(part);
    T* out = d_logits + (size_t)t * E;
#pragma unroll
    for (int j = 0; j < VPT; ++j) {
        int e = lane + 64 * j;
        if (e < E) ElemTraits<T>::store1(out + e, p[j] * (dp[j] - inner));
    }
}

int check_router_shape(int T, int E, int K)
{
    AMOE_REQUIRE(T > 0 && E > 0 && K > 0, AMOE_ERR_BAD_ARG, "router: T, E, K must be positive (T=%d E=%d K=%d)", T, E, K);
    AMOE_REQUIRE(E <= AMOE_MAX_EXPERTS, AMOE_ERR_UNSUPPORTED, "router: E=%d exceeds %d", E, AMOE_MAX_EXPERTS);
    AMOE_REQUIRE(K <= E && K <= AMOE_MAX_TOPK, AMOE_ERR_UNSUPPORTED, "router: K=%d must be <= min(E=%d, %d)", K, E,
                 AMOE_MAX_TOPK);
    return AMOE_OK;
}

}  // namespace

#define ROUTER_DISPATCH_VPT(E, ...)                              \
    if ((E) <= 64) { constexpr int VPT = 1; __VA_ARGS__; }       \
    else if ((E) <= 128) { constexpr int VPT = 2; __VA_ARGS__; } \
    else if ((E) <= 256) { constexpr int VPT = 4; __VA_ARGS__; } \
    else { constexpr int VPT = 8; __VA_ARGS__; }

AMOE_EXPORT int amoe_router_topk_fwd(const void* logits, int dtype, int T, int E, int K, int normalize, float* probs,
                                     int32_t* topk_idx, float* scores, void* stream)
{
    AMOE_REQUIRE(logits && probs && topk_idx && scores, AMOE_ERR_BAD_ARG, "router_topk_fwd: null pointer");
    AMOE_REQUIRE(dtype == AMOE_F32 || dtype == AMOE_BF16 || dtype == AMOE_F16, AMOE_ERR_BAD_ARG, "router_topk_fwd: bad dtype %d", dtype);
    int rc = check_router_shape(T, E, K);
    if (rc) return rc;
    dim3 grid((T + kTokensPerBlock - 1) / kTokensPerBlock), block(kTokensPerBlock * AMOE_WAVE);
    hipStream_t s = (hipStream_t)stream;
    ROUTER_DISPATCH_VPT(E, {
        AMOE_DISPATCH_ELEM(dtype, hipLaunchKernelGGL((router_topk_fwd_kernel<ELEM, VPT>), grid, block, 0, s,
                                                     (const ELEM*)logits, T, E, K, normalize, probs, topk_idx, scores))
    })
    return amoe_check_launch("router_topk_fwd");
}

AMOE_EXPORT int amoe_router_bwd(const float* d_scores, const float* probs, const int32_t* topk_idx,
                                const int32_t* counts, int dtype, int T, int E, int K, int normalize, float lb_coeff,
                                void* d_logits, void* stream)
{
    AMOE_REQUIRE(d_scores && probs && topk_idx && counts && d_logits, AMOE_ERR_BAD_ARG, "router_bwd: null pointer");
    AMOE_REQUIRE(dtype == AMOE_F32 || dtype == AMOE_BF16 || dtype == AMOE_F16, AMOE_ERR_BAD_ARG, "router_bwd: bad dtype %d", dtype);
    int rc = check_router_shape(T, E, K);
    if (rc) return rc;
    dim3 grid((T + kTokensPerBlock - 1) / kTokensPerBlock), block(kTokensPerBlock * AMOE_WAVE);
    hipStream_t s = (hipStream_t)stream;
    ROUTER_DISPATCH_VPT(E, {
        AMOE_DISPATCH_ELEM(dtype, hipLaunchKernelGGL((router_bwd_kernel<ELEM, VPT>), grid, block, 0, s, d_scores, probs,
                                                     topk_idx, counts, T, E, K, normalize, lb_coeff, (ELEM*)d_logits))
    })
    return amoe_check_launch("router_bwd");
}
