// Expert-weight re-layout between the checkpoint format of the original MoE blocks and the
// unified ArcticMoE parameters (arctic_training/model/moe/utils.py:249-266 and :366-395):
//
//   pack    out[e][h][G*i + g] = in_g[e][i][h]     nn.Linear weights [out=I, in=H] of the gate
//                                                  (g=0) and up (g=1) projections -> the
//                                                  interleaved expert_gate_up [E, H, 2I];
//                                                  G = 1 is a plain batched transpose
//                                                  (down_proj [E, H, I] -> expert_down [E, I, H])
//   unpack  out_g[e][i][h] = in[e][h][G*i + g]     the inverse, for saving a checkpoint
//
// Pure byte movement, HBM bound: 64 x 64 tiles go through LDS so that both the reads and the
// writes are 16-byte accesses along the contiguous dimension of their tensor.
#include "amoe_common.h"

namespace {

constexpr int TILE = 64;

// T is the element as raw bits (uint16_t / uint32_t); V = elements per 16-byte access
template <typename T, int G, bool PACK>
__global__ void __launch_bounds__(256)
remap_kernel(const T* __restrict__ a0, const T* __restrict__ a1, T* __restrict__ b0, T* __restrict__ b1, int I, int H,
             long long split_es /* expert stride of the [E,I,H] side */, long long joint_es /* of the [E,H,G*I] side */)
{
    constexpr int V = 16 / sizeof(T);
    constexpr int PAD = V;                       // keeps rows 16-byte aligned and staggers the banks
    // joint-side tile: TILE rows (h) x G*TILE columns; split-side tiles: G x TILE rows (i) x TILE columns (h)
    __shared__ __attribute__((aligned(16))) T tile[TILE][G * TILE + PAD];   // [hh][G*ii + g]
    const int tid = threadIdx.x;
    const int h0 = blockIdx.x * TILE, i0 = blockIdx.y * TILE, e = blockIdx.z;
    const T* s0 = a0;
    const T* s1 = a1;
    typedef T vec_t __attribute__((ext_vector_type(16 / sizeof(T))));

    if (PACK) {
        // read the split side: for each g, rows i, 16-byte vectors along h
        constexpr int VPR = TILE / V;            // vectors per row
        for (int g = 0; g < G; ++g) {
            const T* src = (g == 0 ? s0 : s1) + (long long)e * split_es;
            for (int v = tid; v < TILE * VPR; v += 256) {
                const int ii = v / VPR, hv = (v % VPR) * V;
                const int i = i0 + ii, h = h0 + hv;
                if (i < I && h < H) {
                    const vec_t x = *reinterpret_cast<const vec_t*>(src + (long long)i * H + h);
#pragma unroll
                    for (int k = 0; k < V; ++k) tile[hv + k][G * ii + g] = x[k];
                }
            }
        }
        __syncthreads();
        // write the joint side: rows h, 16-byte vectors along the G*I columns
        constexpr int VPJ = G * TILE / V;
        T* dst = b0 + (long long)e * joint_es;
        for (int v = tid; v < TILE * VPJ; v += 256) {
            const int hh = v / VPJ, cv = (v % VPJ) * V;
            const int h = h0 + hh, c = G * i0 + cv;
            if (h < H && c < G * I)
                *reinterpret_cast<vec_t*>(dst + (long long)h * (G * I) + c) = *reinterpret_cast<const vec_t*>(&tile[hh][cv]);
        }
    } else {
        constexpr int VPJ = G * TILE / V;
        const T* src = s0 + (long long)e * joint_es;
        for (int v = tid; v < TILE * VPJ; v += 256) {
            const int hh = v / VPJ, cv = (v % VPJ) * V;
            const int h = h0 + hh, c = G * i0 + cv;
            if (h < H && c < G * I)
                *reinterpret_cast<vec_t*>(&tile[hh][cv]) = *reinterpret_cast<const vec_t*>(src + (long long)h * (G * I) + c);
        }
        __syncthreads();
        constexpr int VPR = TILE / V;
        for (int g = 0; g < G; ++g) {
            T* dst = (g == 0 ? b0 : b1) + (long long)e * split_es;
            for (int v = tid; v < TILE * VPR; v += 256) {
                const int ii = v / VPR, hv = (v % VPR) * V;
                const int i = i0 + ii, h = h0 + hv;
                if (i < I && h < H) {
                    vec_t x;
#pragma unroll
                    for (int k = 0; k < V; ++k) x[k] = tile[hv + k][G * ii + g];
                    *reinterpret_cast<vec_t*>(dst + (long long)i * H + h) = x;
                }
            }
        }
    }
}

template <typename T>
int launch(bool pack, const void* a0, const void* a1, void* b0, void* b1, int E, int I, int H, long long split_es,
           hipStream_t s)
{
    const dim3 grid((H + TILE - 1) / TILE, (I + TILE - 1) / TILE, E), block(256);
    const bool two = pack ? a1 != nullptr : b1 != nullptr;
    const long long joint_es = (long long)H * I * (two ? 2 : 1);
    if (pack) {
        if (two)
            hipLaunchKernelGGL((remap_kernel<T, 2, true>), grid, block, 0, s, (const T*)a0, (const T*)a1, (T*)b0, (T*)nullptr,
                               I, H, split_es, joint_es);
        else
            hipLaunchKernelGGL((remap_kernel<T, 1, true>), grid, block, 0, s, (const T*)a0, (const T*)nullptr, (T*)b0,
                               (T*)nullptr, I, H, split_es, joint_es);
    } else {
        if (two)
            hipLaunchKernelGGL((remap_kernel<T, 2, false>), grid, block, 0, s, (const T*)a0, (const T*)nullptr, (T*)b0, (T*)b1,
                               I, H, split_es, joint_es);
        else
            hipLaunchKernelGGL((remap_kernel<T, 1, false>), grid, block, 0, s, (const T*)a0, (const T*)nullptr, (T*)b0,
                               (T*)nullptr, I, H, split_es, joint_es);
    }
    return amoe_check_launch(pack ? "remap_pack" : "remap_unpack");
}

int check(const char* what, const void* p0, const void* p1, int dtype, int E, int I, int H, long long split_es)
{
    AMOE_REQUIRE(p0 && p1, AMOE_ERR_BAD_ARG, "%s: null pointer", what);
    AMOE_REQUIRE(dtype == AMOE_F32 || dtype == AMOE_BF16 || dtype == AMOE_F16, AMOE_ERR_BAD_ARG, "%s: bad dtype %d", what, dtype);
    AMOE_REQUIRE(E > 0 && I > 0 && H > 0, AMOE_ERR_BAD_ARG, "%s: sizes must be positive (E=%d I=%d H=%d)", what, E, I, H);
    AMOE_REQUIRE(E <= 65535 && (I + TILE - 1) / TILE <= 65535, AMOE_ERR_UNSUPPORTED, "%s: grid too large", what);
    const int v = dtype != AMOE_F32 ? 8 : 4;
    AMOE_REQUIRE(I % v == 0 && H % v == 0, AMOE_ERR_UNSUPPORTED, "%s: I=%d and H=%d must be multiples of %d", what, I, H, v);
    AMOE_REQUIRE(split_es >= (long long)I * H && split_es % v == 0, AMOE_ERR_BAD_ARG,
                 "%s: expert stride %lld must be at least I*H and a multiple of %d", what, split_es, v);
    return AMOE_OK;
}

}  // namespace

AMOE_EXPORT int amoe_remap_pack(const void* in0, const void* in1, void* out, int dtype, int E, int I, int H,
                                long long in_expert_stride, void* stream)
{
    int rc = check("amoe_remap_pack", in0, out, dtype, E, I, H, in_expert_stride);
    if (rc) return rc;
    if (dtype != AMOE_F32) return launch<uint16_t>(true, in0, in1, out, nullptr, E, I, H, in_expert_stride, (hipStream_t)stream);
    return launch<uint32_t>(true, in0, in1, out, nullptr, E, I, H, in_expert_stride, (hipStream_t)stream);
}

AMOE_EXPORT int amoe_remap_unpack(const void* in, void* out0, void* out1, int dtype, int E, int I, int H,
                                  long long out_expert_stride, void* stream)
{
    int rc = check("amoe_remap_unpack", in, out0, dtype, E, I, H, out_expert_stride);
    if (rc) return rc;
    if (dtype != AMOE_F32) return launch<uint16_t>(false, in, nullptr, out0, out1, E, I, H, out_expert_stride, (hipStream_t)stream);
    return launch<uint32_t>(false, in, nullptr, out0, out1, E, I, H, out_expert_stride, (hipStream_t)stream);
}
