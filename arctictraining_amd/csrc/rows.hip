// HBM-bound row kernels: gather, weighted gather-reduce (combine / gather backward),
// combine backward, and the elementwise gated activation (forward for the f32 path,
// backward for both).  All move 16-byte vectors per lane; a row of H elements is walked by
// the 256 lanes of a block in steps of 256 vectors so every access is fully coalesced.
#include "amoe_common.h"

namespace {

constexpr int kBlock = 256;

// xp[r,:] = x[token_of[r],:]
template <typename T>
__global__ void __launch_bounds__(kBlock)
gather_rows_kernel(const T* __restrict__ x, const int32_t* __restrict__ token_of, T* __restrict__ xp, int R, int H)
{
    constexpr int V = ElemTraits<T>::kVec;
    const int nvec = H / V;
    for (int r = blockIdx.x; r < R; r += gridDim.x) {
        const u32x4_t* src = reinterpret_cast<const u32x4_t*>(x + (size_t)token_of[r] * H);
        u32x4_t* dst = reinterpret_cast<u32x4_t*>(xp + (size_t)r * H);
        for (int i = threadIdx.x; i < nvec; i += kBlock) dst[i] = src[i];
    }
}

// dst[t,:] = (addend ? addend[t,:] : 0) + sum_k w[t,k] * src[row_of[t,k],:]   (w == null -> 1)
template <typename T, int KMAX>
__global__ void __launch_bounds__(kBlock)
gather_reduce_kernel(const T* __restrict__ src, const int32_t* __restrict__ row_of, const float* __restrict__ w,
                     const T* __restrict__ addend, T* __restrict__ dst, int n_tokens, int K, int H)
{
    constexpr int V = ElemTraits<T>::kVec;
    const int nvec = H / V;
    for (int t = blockIdx.x; t < n_tokens; t += gridDim.x) {
        int rows[KMAX];
        float wk[KMAX];
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
            bool ok = k < K;
            rows[k] = ok ? row_of[(size_t)t * K + k] : 0;
            wk[k] = ok ? (w ? w[(size_t)t * K + k] : 1.0f) : 0.f;
        }
        for (int i = threadIdx.x; i < nvec; i += kBlock) {
            float acc[V];
            if (addend) {
                u32x4_t a = reinterpret_cast<const u32x4_t*>(addend + (size_t)t * H)[i];
                ElemTraits<T>::unpack(a, acc);
            } else {
#pragma unroll
                for (int j = 0; j < V; ++j) acc[j] = 0.f;
            }
#pragma unroll
            for (int k = 0; k < KMAX; ++k) {
                if (k < K) {
                    u32x4_t v = reinterpret_cast<const u32x4_t*>(src + (size_t)rows[k] * H)[i];
                    float f[V];
                    ElemTraits<T>::unpack(v, f);
#pragma unroll
                    for (int j = 0; j < V; ++j) acc[j] += wk[k] * f[j];
                }
            }
            reinterpret_cast<u32x4_t*>(dst + (size_t)t * H)[i] = ElemTraits<T>::pack(acc);
        }
    }
}

// d_out[row_of[t,k],:] = dy[t,:] * s[t,k];  d_s[t,k] = <dy[t,:], out[row_of[t,k],:]>
template <typename T>
__global__ void __launch_bounds__(kBlock)
combine_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ out, const int32_t* __restrict__ row_of,
                   const float* __restrict__ scores, T* __restrict__ d_out, float* __restrict__ d_scores,
                   int n_tokens, int K, int H)
{
    constexpr int V = ElemTraits<T>::kVec;
    __shared__ float red[kBlock / AMOE_WAVE];
    const int nvec = H / V;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int t = blockIdx.x; t < n_tokens; t += gridDim.x) {
        const u32x4_t* g = reinterpret_cast<const u32x4_t*>(dy + (size_t)t * H);
        for (int k = 0; k < K; ++k) {
            const int row = row_of[(size_t)t * K + k];
            const float s = scores[(size_t)t * K + k];
            const u32x4_t* o = reinterpret_cast<const u32x4_t*>(out + (size_t)row * H);
            u32x4_t* d = d_out ? reinterpret_cast<u32x4_t*>(d_out + (size_t)row * H) : nullptr;
            float part = 0.f;
            for (int i = threadIdx.x; i < nvec; i += kBlock) {
                float gv[V], ov[V], dv[V];
                ElemTraits<T>::unpack(g[i], gv);
                ElemTraits<T>::unpack(o[i], ov);
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    part += gv[j] * ov[j];
                    dv[j] = gv[j] * s;
                }
                if (d) d[i] = ElemTraits<T>::pack(dv);
            }
            part = wave_sum(part);
            __syncthreads();  // red[] free again
            if (lane == 0) red[wv] = part;
            __syncthreads();
            if (threadIdx.x == 0) {
                float tot = 0.f;
#pragma unroll
                for (int i = 0; i < kBlock / AMOE_WAVE; ++i) tot += red[i];
                d_scores[(size_t)t * K + k] = tot;
            }
        }
    }
}

// inter[r,i] = scale[r] * gu[r,2i+1] * act(gu[r,2i])     (one wavefront per row; scale == null -> 1)
template <typename T, int ACT>
__global__ void __launch_bounds__(kBlock)
gated_act_fwd_kernel(const T* __restrict__ gu, const float* __restrict__ scale, T* __restrict__ inter, int R, int I)
{
    constexpr int V = ElemTraits<T>::kVec;
    const int lane = threadIdx.x & 63;
    const int nvec = I / V;
    for (int r = blockIdx.x * (kBlock / AMOE_WAVE) + (threadIdx.x >> 6); r < R; r += gridDim.x * (kBlock / AMOE_WAVE)) {
        const float sc = scale ? scale[r] : 1.0f;
        const u32x4_t* g = reinterpret_cast<const u32x4_t*>(gu + (size_t)r * 2 * I);
        u32x4_t* o = reinterpret_cast<u32x4_t*>(inter + (size_t)r * I);
        for (int i = lane; i < nvec; i += AMOE_WAVE) {
            float a[V], b[V], out[V];
            ElemTraits<T>::unpack(g[2 * i], a);
            ElemTraits<T>::unpack(g[2 * i + 1], b);
#pragma unroll
            for (int j = 0; j < V / 2; ++j) {
                out[j] = sc * a[2 * j + 1] * act_fwd<ACT>(a[2 * j]);
                out[V / 2 + j] = sc * b[2 * j + 1] * act_fwd<ACT>(b[2 * j]);
            }
            o[i] = ElemTraits<T>::pack(out);
        }
    }
}

// Backward of inter[r,i] = scale[r] * up * act(gate)   (one wavefront per row):
//   d_gu[r,2i]   = scale[r] * d_inter[r,i] * up * act'(gate)
//   d_gu[r,2i+1] = scale[r] * d_inter[r,i] * act(gate)
//   d_scale[r]   = sum_i d_inter[r,i] * up * act(gate)        written at slot (t,k) of row r
template <typename T, int ACT>
__global__ void __launch_bounds__(kBlock)
gated_act_bwd_kernel(const T* __restrict__ gu, const T* __restrict__ d_inter, const float* __restrict__ scale,
                     const int32_t* __restrict__ slot_of, int n_tokens, int K, T* __restrict__ d_gu,
                     float* __restrict__ d_scale_tk, int R, int I)
{
    constexpr int V = ElemTraits<T>::kVec;
    const int lane = threadIdx.x & 63;
    const int nvec = I / V;
    for (int r = blockIdx.x * (kBlock / AMOE_WAVE) + (threadIdx.x >> 6); r < R; r += gridDim.x * (kBlock / AMOE_WAVE)) {
        const float sc = scale ? scale[r] : 1.0f;
        const u32x4_t* g = reinterpret_cast<const u32x4_t*>(gu + (size_t)r * 2 * I);
        const u32x4_t* di = reinterpret_cast<const u32x4_t*>(d_inter + (size_t)r * I);
        u32x4_t* o = reinterpret_cast<u32x4_t*>(d_gu + (size_t)r * 2 * I);
        float dot = 0.f;
        for (int i = lane; i < nvec; i += AMOE_WAVE) {
            float a[V], b[V], d[V], oa[V], ob[V];
            ElemTraits<T>::unpack(g[2 * i], a);
            ElemTraits<T>::unpack(g[2 * i + 1], b);
            ElemTraits<T>::unpack(di[i], d);
#pragma unroll
            for (int j = 0; j < V / 2; ++j) {
                const float fa = act_fwd<ACT>(a[2 * j]), fb = act_fwd<ACT>(b[2 * j]);
                dot += d[j] * a[2 * j + 1] * fa + d[V / 2 + j] * b[2 * j + 1] * fb;
                oa[2 * j] = sc * d[j] * a[2 * j + 1] * act_bwd<ACT>(a[2 * j]);
                oa[2 * j + 1] = sc * d[j] * fa;
                ob[2 * j] = sc * d[V / 2 + j] * b[2 * j + 1] * act_bwd<ACT>(b[2 * j]);
                ob[2 * j + 1] = sc * d[V / 2 + j] * fb;
            }
            o[2 * i] = ElemTraits<T>::pack(oa);
            o[2 * i + 1] = ElemTraits<T>::pack(ob);
        }
        if (d_scale_tk) {
            dot = wave_sum(dot);
            if (lane == 0) {
                const int f = slot_of[r];
                const int k = f / n_tokens;
                d_scale_tk[(size_t)(f - k * n_tokens) * K + k] = dot;
            }
        }
    }
}

// d_scores[t,k] = sum_p partials[p][row_of[t,k]]  (fixed order over p)
__global__ void __launch_bounds__(kBlock)
score_grad_gather_kernel(const float* __restrict__ partials, int n_parts, long long part_stride,
                         const int32_t* __restrict__ row_of, float* __restrict__ d_scores, int n_slots)
{
    const int s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= n_slots) return;
    const int row = row_of[s];
    float tot = 0.f;
    for (int p = 0; p < n_parts; ++p) tot += partials[p * part_stride + row];
    d_scores[s] = tot;
}

int check_rows(const char* what, int dtype, int rows, int H)
{
    AMOE_REQUIRE(dtype == AMOE_F32 || dtype == AMOE_BF16 || dtype == AMOE_F16, AMOE_ERR_BAD_ARG, "%s: bad dtype %d", what, dtype);
    AMOE_REQUIRE(rows > 0 && H > 0, AMOE_ERR_BAD_ARG, "%s: sizes must be positive (rows=%d H=%d)", what, rows, H);
    const int vec = dtype != AMOE_F32 ? 8 : 4;
    AMOE_REQUIRE(H % vec == 0, AMOE_ERR_UNSUPPORTED, "%s: row length %d must be a multiple of %d", what, H, vec);
    return AMOE_OK;
}

inline int row_grid(int rows) { return rows < 65536 ? rows : 65536; }

}  // namespace

AMOE_EXPORT int amoe_gather_rows_fwd(const void* x, const int32_t* token_of, void* xp, int dtype, int R, int H,
                                     void* stream)
{
    AMOE_REQUIRE(x && token_of && xp, AMOE_ERR_BAD_ARG, "gather_rows_fwd: null pointer");
    int rc = check_rows("gather_rows_fwd", dtype, R, H);
    if (rc) return rc;
    hipStream_t s = (hipStream_t)stream;
    AMOE_DISPATCH_ELEM(dtype, hipLaunchKernelGGL(gather_rows_kernel<ELEM>, dim3(row_grid(R)), dim3(kBlock), 0, s,
                                                 (const ELEM*)x, token_of, (ELEM*)xp, R, H))
    return amoe_check_launch("gather_rows_fwd");
}

template <typename T>
static void launch_gather_reduce(const void* src, const int32_t* row_of, const float* w, const void* addend, void* dst,
                                 int T_, int K, int H, hipStream_t s)
{
    dim3 grid(row_grid(T_)), block(kBlock);
    if (K <= 2)
        hipLaunchKernelGGL((gather_reduce_kernel<T, 2>), grid, block, 0, s, (const T*)src, row_of, w, (const T*)addend,
                           (T*)dst, T_, K, H);
    else if (K <= 4)
        hipLaunchKernelGGL((gather_reduce_kernel<T, 4>), grid, block, 0, s, (const T*)src, row_of, w, (const T*)addend,
                           (T*)dst, T_, K, H);
    else if (K <= 8)
        hipLaunchKernelGGL((gather_reduce_kernel<T, 8>), grid, block, 0, s, (const T*)src, row_of, w, (const T*)addend,
                           (T*)dst, T_, K, H);
    else
        hipLaunchKernelGGL((gather_reduce_kernel<T, AMOE_MAX_TOPK>), grid, block, 0, s, (const T*)src, row_of, w,
                           (const T*)addend, (T*)dst, T_, K, H);
}

AMOE_EXPORT int amoe_gather_rows_bwd(const void* d_xp, const int32_t* row_of, const void* addend, void* dx, int dtype,
                                     int T, int K, int H, void* stream)
{
    AMOE_REQUIRE(d_xp && row_of && dx, AMOE_ERR_BAD_ARG, "gather_rows_bwd: null pointer");
    int rc = check_rows("gather_rows_bwd", dtype, T, H);
    if (rc) return rc;
    AMOE_REQUIRE(K > 0 && K <= AMOE_MAX_TOPK, AMOE_ERR_UNSUPPORTED, "gather_rows_bwd: K=%d outside 1..%d", K,
                 AMOE_MAX_TOPK);
    AMOE_DISPATCH_ELEM(dtype, launch_gather_reduce<ELEM>(d_xp, row_of, nullptr, addend, dx, T, K, H, (hipStream_t)stream))
    return amoe_check_launch("gather_rows_bwd");
}

AMOE_EXPORT int amoe_combine_fwd(const void* moe_out, const int32_t* row_of, const float* scores, void* y, int dtype,
                                 int T, int K, int H, void* stream)
{
    AMOE_REQUIRE(moe_out && row_of && y, AMOE_ERR_BAD_ARG, "combine_fwd: null pointer");
    int rc = check_rows("combine_fwd", dtype, T, H);
    if (rc) return rc;
    AMOE_REQUIRE(K > 0 && K <= AMOE_MAX_TOPK, AMOE_ERR_UNSUPPORTED, "combine_fwd: K=%d outside 1..%d", K, AMOE_MAX_TOPK);
    AMOE_DISPATCH_ELEM(dtype, launch_gather_reduce<ELEM>(moe_out, row_of, scores, nullptr, y, T, K, H, (hipStream_t)stream))
    return amoe_check_launch("combine_fwd");
}

AMOE_EXPORT int amoe_combine_bwd(const void* dy, const void* moe_out, const int32_t* row_of, const float* scores,
                                 void* d_moe_out, float* d_scores, int dtype, int T, int K, int H, void* stream)
{
    AMOE_REQUIRE(dy && moe_out && row_of && scores && d_scores, AMOE_ERR_BAD_ARG, "combine_bwd: null pointer");
    int rc = check_rows("combine_bwd", dtype, T, H);
    if (rc) return rc;
    AMOE_REQUIRE(K > 0 && K <= AMOE_MAX_TOPK, AMOE_ERR_UNSUPPORTED, "combine_bwd: K=%d outside 1..%d", K, AMOE_MAX_TOPK);
    hipStream_t s = (hipStream_t)stream;
    AMOE_DISPATCH_ELEM(dtype, hipLaunchKernelGGL(combine_bwd_kernel<ELEM>, dim3(row_grid(T)), dim3(kBlock), 0, s,
                                                 (const ELEM*)dy, (const ELEM*)moe_out, row_of, scores, (ELEM*)d_moe_out,
                                                 d_scores, T, K, H))
    return amoe_check_launch("combine_bwd");
}

// used by the f32 gate_up path, which does not fuse the activation into its GEMM
int amoe_launch_gated_act_fwd(const void* gu, const float* row_scale, void* inter, int dtype, int R, int I, int act,
                              hipStream_t s)
{
    const int rows_per_block = kBlock / AMOE_WAVE;
    const int grid = (R + rows_per_block - 1) / rows_per_block < 65536 ? (R + rows_per_block - 1) / rows_per_block : 65536;
    AMOE_DISPATCH_ACT(act, {
        AMOE_DISPATCH_ELEM(dtype, hipLaunchKernelGGL((gated_act_fwd_kernel<ELEM, ACT>), dim3(grid), dim3(kBlock), 0, s,
                                                     (const ELEM*)gu, row_scale, (ELEM*)inter, R, I))
    })
    return amoe_check_launch("gated_act_fwd");
}

AMOE_EXPORT int amoe_gated_act_bwd(const void* gate_up, const void* d_inter, const float* row_scale,
                                   const int32_t* slot_of, void* d_gate_up, float* d_row_scale, int dtype, int R, int I,
                                   int T, int K, int act, void* stream)
{
    AMOE_REQUIRE(gate_up && d_inter && d_gate_up, AMOE_ERR_BAD_ARG, "gated_act_bwd: null pointer");
    int rc = check_rows("gated_act_bwd", dtype, R, I);
    if (rc) return rc;
    AMOE_REQUIRE(act >= AMOE_ACT_SILU && act <= AMOE_ACT_GPT_OSS, AMOE_ERR_BAD_ARG, "gated_act_bwd: bad activation %d",
                 act);
    if (d_row_scale) {
        AMOE_REQUIRE(slot_of, AMOE_ERR_BAD_ARG, "gated_act_bwd: d_row_scale needs slot_of");
        AMOE_REQUIRE(T > 0 && K > 0 && (long long)T * K == (long long)R, AMOE_ERR_BAD_ARG,
                     "gated_act_bwd: T*K must equal R (T=%d K=%d R=%d)", T, K, R);
    }
    const int rows_per_block = kBlock / AMOE_WAVE;
    const int grid = (R + rows_per_block - 1) / rows_per_block < 65536 ? (R + rows_per_block - 1) / rows_per_block : 65536;
    hipStream_t s = (hipStream_t)stream;
    AMOE_DISPATCH_ACT(act, {
        AMOE_DISPATCH_ELEM(dtype, hipLaunchKernelGGL((gated_act_bwd_kernel<ELEM, ACT>), dim3(grid), dim3(kBlock), 0, s,
                                                     (const ELEM*)gate_up, (const ELEM*)d_inter, row_scale, slot_of, T, K,
                                                     (ELEM*)d_gate_up, d_row_scale, R, I))
    })
    return amoe_check_launch("gated_act_bwd");
}

AMOE_EXPORT int amoe_score_grad_gather(const float* partials, int n_parts, const int32_t* row_of, float* d_scores, int T,
                                       int K, void* stream)
{
    AMOE_REQUIRE(partials && row_of && d_scores, AMOE_ERR_BAD_ARG, "score_grad_gather: null pointer");
    AMOE_REQUIRE(n_parts > 0 && T > 0 && K > 0, AMOE_ERR_BAD_ARG, "score_grad_gather: sizes must be positive");
    AMOE_REQUIRE((long long)T * K < (1ll << 31), AMOE_ERR_UNSUPPORTED, "score_grad_gather: T*K does not fit int32");
    const int n = T * K;
    hipLaunchKernelGGL(score_grad_gather_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, (hipStream_t)stream,
                       partials, n_parts, (long long)n, row_of, d_scores, n);
    return amoe_check_launch("score_grad_gather");
}
