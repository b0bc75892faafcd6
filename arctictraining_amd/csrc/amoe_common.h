// Shared host/device helpers for the gfx950 expert-layer kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/arctic_moe_hip.h"

#define AMOE_EXPORT extern "C" __attribute__((visibility("default")))

// ---------------------------------------------------------------- host side errors
void amoe_set_error(const char* fmt, ...);

#define AMOE_REQUIRE(cond, code, ...)  \
    do {                               \
        if (!(cond)) {                 \
            amoe_set_error(__VA_ARGS__); \
            return (code);             \
        }                              \
    } while (0)

static inline int amoe_check_launch(const char* what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        amoe_set_error("%s: %s", what, hipGetErrorString(e));
        return AMOE_ERR_LAUNCH;
    }
    return AMOE_OK;
}

// ---------------------------------------------------------------- device types
typedef __bf16 bf16_t;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16_t;
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

#define AMOE_WAVE 64

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t hi16) { return __uint_as_float(hi16 << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// round-to-nearest-even float -> bf16 pair packed into one dword (lo = a, hi = b)
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b)
{
    f32x2_t v = {a, b};
    bf16x2_t r = __builtin_convertvector(v, bf16x2_t);
    return __builtin_bit_cast(uint32_t, r);
}
__device__ __forceinline__ float round_bf16(float a)
{
    bf16_t r = (bf16_t)a;
    return (float)r;
}

// the same for IEEE half precision (v_cvt_f16_f32 rounds to nearest even in the default mode)
__device__ __forceinline__ float f16_lo(uint32_t w) { return (float)__builtin_bit_cast(f16x2_t, w)[0]; }
__device__ __forceinline__ float f16_hi(uint32_t w) { return (float)__builtin_bit_cast(f16x2_t, w)[1]; }
__device__ __forceinline__ uint32_t pack_f16x2(float a, float b)
{
    f16x2_t r = {(f16_t)a, (f16_t)b};
    return __builtin_bit_cast(uint32_t, r);
}

template <typename T>
struct ElemTraits;
template <>
struct ElemTraits<float> {
    static constexpr int kVec = 4;  // elements per 16-byte vector
    __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f)
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(v[i]);
    }
    __device__ static __forceinline__ u32x4_t pack(const float* f)
    {
        u32x4_t v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = __float_as_uint(f[i]);
        return v;
    }
    __device__ static __forceinline__ float load1(const float* p) { return *p; }
    __device__ static __forceinline__ void store1(float* p, float v) { *p = v; }
    __device__ static __forceinline__ float round(float v) { return v; }
};
template <>
struct ElemTraits<bf16_t> {
    static constexpr int kVec = 8;
    __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f)
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = bf16_lo(v[i]);
            f[2 * i + 1] = bf16_hi(v[i]);
        }
    }
    __device__ static __forceinline__ u32x4_t pack(const float* f)
    {
        u32x4_t v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = pack_bf16x2(f[2 * i], f[2 * i + 1]);
        return v;
    }
    __device__ static __forceinline__ float load1(const bf16_t* p) { return (float)(*p); }
    __device__ static __forceinline__ void store1(bf16_t* p, float v) { *p = (bf16_t)v; }
    __device__ static __forceinline__ float round(float v) { return round_bf16(v); }
};

template <>
struct ElemTraits<f16_t> {
    static constexpr int kVec = 8;
    __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f)
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = f16_lo(v[i]);
            f[2 * i + 1] = f16_hi(v[i]);
        }
    }
    __device__ static __forceinline__ u32x4_t pack(const float* f)
    {
        u32x4_t v;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = pack_f16x2(f[2 * i], f[2 * i + 1]);
        return v;
    }
    __device__ static __forceinline__ float load1(const f16_t* p) { return (float)(*p); }
    __device__ static __forceinline__ void store1(f16_t* p, float v) { *p = (f16_t)v; }
    __device__ static __forceinline__ float round(float v) { return (float)(f16_t)v; }
};

// runs the statement with ELEM = the element type of `dtype` (float for AMOE_F32)
#define AMOE_DISPATCH_ELEM(dtype, ...)                                   \
    if ((dtype) == AMOE_BF16) { typedef bf16_t ELEM; __VA_ARGS__; }      \
    else if ((dtype) == AMOE_F16) { typedef f16_t ELEM; __VA_ARGS__; }   \
    else { typedef float ELEM; __VA_ARGS__; }

// Wave-wide reductions without LDS traffic: four DPP steps leave every lane of a 16-lane row
// with the row's result (lanes exchanged inside quads, then between the quads of a half row,
// then between the half rows), and the four rows are combined from one lane each.
constexpr int AMOE_DPP_QUAD_XOR1 = 0xB1;     // quad_perm [1,0,3,2]
constexpr int AMOE_DPP_QUAD_XOR2 = 0x4E;     // quad_perm [2,3,0,1]
constexpr int AMOE_DPP_HALF_MIRROR = 0x141;  // row_half_mirror: lane i <- lane 7 - i of its half row
constexpr int AMOE_DPP_MIRROR = 0x140;       // row_mirror: lane i <- lane 15 - i of its row

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t x)
{
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xF, 0xF, true);
}

template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x)
{
    return __uint_as_float(dpp_u32<CTRL>(__float_as_uint(x)));
}

__device__ __forceinline__ float row_lane_f32(float v, int lane)
{
    return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), lane));
}

__device__ __forceinline__ float wave_sum(float v)
{
    v += dpp_f32<AMOE_DPP_QUAD_XOR1>(v);
    v += dpp_f32<AMOE_DPP_QUAD_XOR2>(v);
    v += dpp_f32<AMOE_DPP_HALF_MIRROR>(v);
    v += dpp_f32<AMOE_DPP_MIRROR>(v);
    return (row_lane_f32(v, 0) + row_lane_f32(v, 16)) + (row_lane_f32(v, 32) + row_lane_f32(v, 48));
}

// activations of the gated expert FFN (value and derivative)
template <int ACT>
__device__ __forceinline__ float act_fwd(float g)
{
    if (ACT == AMOE_ACT_SILU) return g / (1.0f + __expf(-g));
    if (ACT == AMOE_ACT_GPT_OSS) return g / (1.0f + __expf(-1.702f * g));
    if (ACT == AMOE_ACT_RELU) return g > 0.f ? g : 0.f;
    // exact (erf) gelu, the default of torch.nn.functional.gelu
    return 0.5f * g * (1.0f + erff(g * 0.70710678118654752f));
}
template <int ACT>
__device__ __forceinline__ float act_bwd(float g)
{
    if (ACT == AMOE_ACT_SILU) {
        float s = 1.0f / (1.0f + __expf(-g));
        return s * (1.0f + g * (1.0f - s));
    }
    if (ACT == AMOE_ACT_GPT_OSS) {
        float s = 1.0f / (1.0f + __expf(-1.702f * g));
        return s * (1.0f + 1.702f * g * (1.0f - s));
    }
    if (ACT == AMOE_ACT_RELU) return g > 0.f ? 1.f : 0.f;
    float cdf = 0.5f * (1.0f + erff(g * 0.70710678118654752f));
    float pdf = 0.3989422804014327f * __expf(-0.5f * g * g);
    return cdf + g * pdf;
}

#define AMOE_DISPATCH_ACT(act, ...)                                  \
    switch (act) {                                                   \
        case AMOE_ACT_SILU: { constexpr int ACT = AMOE_ACT_SILU; __VA_ARGS__; } break;       \
        case AMOE_ACT_GELU: { constexpr int ACT = AMOE_ACT_GELU; __VA_ARGS__; } break;       \
        case AMOE_ACT_RELU: { constexpr int ACT = AMOE_ACT_RELU; __VA_ARGS__; } break;       \
        default: { constexpr int ACT = AMOE_ACT_GPT_OSS; __VA_ARGS__; } break;               \
    }

// ---------------------------------------------------------------- tile map of the row-grouped GEMMs
// One int4 {expert, first row, end row, 0} per bm-row tile of the expert-grouped rows, written by ONE
// block: experts ascending, an expert's tiles in row order (its last one may be partly filled), entries
// past the last tile hold expert -1.  An expert's short last tile stays next to its full ones on
// purpose: the tiles of one expert share its weight panels in L2 when they are worked on together, and
// a short tile (same loads, fewer multiplications) next to full ones evens out the memory traffic over
// time -- a list with all the short tiles at the end was measured 4-7 % slower.
// header[0] = number of tiles, header[1..3] = 0.
//   row_end: inclusive scan of the experts' row counts, in LDS, visible to the block; row_base: first row of expert 0
//   tscan [AMOE_MAX_EXPERTS]: LDS scratch
// Called by all NTHREADS (>= 64) threads of the block.
template <int NTHREADS>
__device__ __forceinline__ void amoe_emit_tile_map(const int32_t* row_end, int row_base, int E, int bm, int4* tile_map,
                                                   int32_t* header, int max_mtiles, int32_t* tscan)
{
    static_assert(AMOE_MAX_EXPERTS == 8 * AMOE_WAVE, "one wavefront scans 8 entries per lane");
    const int t = threadIdx.x;
    for (int e = t; e < AMOE_MAX_EXPERTS; e += NTHREADS) {
        const int rows = e < E ? row_end[e] - (e ? row_end[e - 1] : 0) : 0;
        tscan[e] = (rows + bm - 1) / bm;
    }
    __syncthreads();
    if (t < AMOE_WAVE) {
        // inclusive scan of the tile counts: 8 consecutive entries per lane, lane sums by shuffles
        int f[8], s = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            f[i] = tscan[t * 8 + i];
            s += f[i];
        }
        int inc = s;
#pragma unroll
        for (int o = 1; o < AMOE_WAVE; o <<= 1) {
            const int u = __shfl_up(inc, o, AMOE_WAVE);
            if (t >= o) inc += u;
        }
        int run = inc - s;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            run += f[i];
            tscan[t * 8 + i] = run;
        }
    }
    __syncthreads();
    const int total = tscan[E - 1];
    for (int mt = t; mt < total && mt < max_mtiles; mt += NTHREADS) {
        // smallest ex with tscan[ex] > mt: the expert that owns tile mt
        int lo = 0, hi = E - 1;
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (tscan[mid] > mt) hi = mid; else lo = mid + 1;
        }
        const int first_tile = lo ? tscan[lo - 1] : 0;
        const int row0 = lo ? row_end[lo - 1] : 0;
        tile_map[mt] = make_int4(lo, row_base + row0 + (mt - first_tile) * bm, row_base + row_end[lo], 0);
    }
    for (int mt = total + t; mt < max_mtiles; mt += NTHREADS) tile_map[mt] = make_int4(-1, 0, 0, 0);
    if (t == 0) {
        header[0] = total < max_mtiles ? total : max_mtiles;
        header[1] = 0;
        header[2] = 0;
        header[3] = 0;
    }
}
