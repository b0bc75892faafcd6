// Exported grouped-GEMM entry points (argument validation + dtype dispatch), the version
// query and the per-thread error message.
#include "amoe_common.h"

#include <string.h>

static thread_local char g_err[512] = "";

void amoe_set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

AMOE_EXPORT int amoe_version(void) { return 100; }
AMOE_EXPORT const char* amoe_last_error(void) { return g_err; }

// implemented in gemm_bf16.hip / gemm_f32.hip / rows.hip
int amoe_bf16_gateup_act(const void* xp, const int32_t* a_row_map, const void* w, const int32_t* offsets, void* gate_up,
                         void* inter, const float* row_scale, int R, int E, int H, int I, int act, void* workspace, size_t workspace_bytes,
                         int tile_cfg, hipStream_t s, int dtype);
int amoe_bf16_nn(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C, int R, int E,
                 int Kd, int N, void* workspace, size_t workspace_bytes, int tile_cfg, hipStream_t s, int dtype);
int amoe_bf16_nt(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C, int R, int E,
                 int Kd, int N, void* workspace, size_t workspace_bytes, int tile_cfg, hipStream_t s, int dtype);
int amoe_bf16_wgrad(const void* A, const int32_t* a_row_map, const void* B, const int32_t* b_row_map,
                    const int32_t* offsets, void* C, int R, int E, int Kd, int N, int tile_cfg, hipStream_t s, int dtype);
int amoe_bf16_nt_gated_bwd(const void* dy, const int32_t* a_row_map, const void* w_down, const int32_t* offsets,
                           const void* gate_up, const float* row_scale, void* d_gate_up, float* partials, int R, int E,
                           int I, int H, int act, void* workspace, size_t workspace_bytes, int tile_cfg, hipStream_t s, int dtype);
int amoe_bf16_gated_bwd_parts(int I, int tile_cfg);
int amoe_f32_rows(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets, void* C, int R, int E,
                  int Kred, int N, int ldb, long long strideB, bool b_kc, void* workspace, size_t workspace_bytes,
                  bool map_ready, hipStream_t s);
int amoe_f32_wgrad(const void* A, const int32_t* a_row_map, const void* B, const int32_t* b_row_map,
                   const int32_t* offsets, void* C, int R, int E, int Kd, int N, hipStream_t s);
int amoe_launch_gated_act_fwd(const void* gu, const float* row_scale, void* inter, int dtype, int R, int I, int act,
                              hipStream_t s);

namespace {

// what both dtypes share: pointers, sizes, the int32 offset range
int check_gemm_common(const char* what, int dtype, int R, int E, int d0, int d1, int tile_cfg)
{
    AMOE_REQUIRE(dtype == AMOE_F32 || dtype == AMOE_BF16 || dtype == AMOE_F16, AMOE_ERR_BAD_ARG, "%s: bad dtype %d", what, dtype);
    AMOE_REQUIRE(R > 0 && E > 0 && d0 > 0 && d1 > 0, AMOE_ERR_BAD_ARG, "%s: sizes must be positive (R=%d E=%d %d %d)",
                 what, R, E, d0, d1);
    AMOE_REQUIRE(E <= AMOE_MAX_EXPERTS, AMOE_ERR_UNSUPPORTED, "%s: E=%d exceeds %d", what, E, AMOE_MAX_EXPERTS);
    const int shape = tile_cfg & ~AMOE_TILE_MAP_READY;
    AMOE_REQUIRE(tile_cfg >= 0 && shape <= 5 && shape != 4, AMOE_ERR_BAD_ARG,
                 "%s: tile_cfg %d is not one of 0, 1, 2, 3, 5 (optionally | AMOE_TILE_MAP_READY)", what, tile_cfg);
    AMOE_REQUIRE((long long)R * d0 < (1ll << 32) && (long long)R * d1 < (1ll << 32) && (long long)d0 * d1 < (1ll << 32),
                 AMOE_ERR_UNSUPPORTED, "%s: an operand exceeds 2^32 elements", what);
    return AMOE_OK;
}

// reduction length must be a multiple of `red_mult`, the other extents of `vec`
int check_gemm_dims(const char* what, int dtype, int red, int other)
{
    if (dtype != AMOE_F32) {
        AMOE_REQUIRE(red % 32 == 0, AMOE_ERR_UNSUPPORTED, "%s: 16-bit reduction length %d must be a multiple of 32", what,
                     red);
        AMOE_REQUIRE(other % 8 == 0, AMOE_ERR_UNSUPPORTED, "%s: 16-bit extent %d must be a multiple of 8", what, other);
    } else {
        AMOE_REQUIRE(red % 4 == 0 && other % 4 == 0, AMOE_ERR_UNSUPPORTED,
                     "%s: f32 extents (%d, %d) must be multiples of 4", what, red, other);
    }
    return AMOE_OK;
}

}  // namespace

AMOE_EXPORT int amoe_grouped_gemm_gateup_act_fwd(const void* xp, const int32_t* a_row_map, const void* w_gate_up,
                                                 const int32_t* offsets, const float* row_scale, void* gate_up,
                                                 void* inter, int dtype, int R,
                                                 int E, int H, int I, int act, void* workspace, size_t workspace_bytes,
                                                 int tile_cfg, void* stream)
{
    const char* what = "grouped_gemm_gateup_act_fwd";
    AMOE_REQUIRE(xp && w_gate_up && offsets && inter && workspace, AMOE_ERR_BAD_ARG, "%s: null pointer", what);
    int rc = check_gemm_common(what, dtype, R, E, H, I, tile_cfg);
    if (rc) return rc;
    AMOE_REQUIRE(act >= AMOE_ACT_SILU && act <= AMOE_ACT_GPT_OSS, AMOE_ERR_BAD_ARG, "%s: bad activation %d", what, act);
    AMOE_REQUIRE((long long)H * 2 * I < (1ll << 32) && (long long)R * 2 * I < (1ll << 32), AMOE_ERR_UNSUPPORTED,
                 "%s: an operand exceeds 2^32 elements", what);
    rc = check_gemm_dims(what, dtype, H, 2 * I);
    if (rc) return rc;
    AMOE_REQUIRE(workspace_bytes >= amoe_grouped_gemm_workspace_bytes(R, E), AMOE_ERR_WORKSPACE,
                 "%s: workspace %zu < %zu bytes", what, workspace_bytes, amoe_grouped_gemm_workspace_bytes(R, E));
    hipStream_t s = (hipStream_t)stream;
    if (dtype != AMOE_F32)
        return amoe_bf16_gateup_act(xp, a_row_map, w_gate_up, offsets, gate_up, inter, row_scale, R, E, H, I, act, workspace,
                                    workspace_bytes, tile_cfg, s, dtype);
    AMOE_REQUIRE(gate_up, AMOE_ERR_UNSUPPORTED, "%s: the f32 path needs the gate_up buffer", what);
    AMOE_REQUIRE(I % 4 == 0, AMOE_ERR_UNSUPPORTED, "%s: f32 intermediate size %d must be a multiple of 4", what, I);
    rc = amoe_f32_rows(xp, a_row_map, w_gate_up, offsets, gate_up, R, E, H, 2 * I, 2 * I, (long long)H * 2 * I, false,
                       workspace, workspace_bytes, (tile_cfg & AMOE_TILE_MAP_READY) != 0, s);
    if (rc) return rc;
    return amoe_launch_gated_act_fwd(gate_up, row_scale, inter, dtype, R, I, act, s);
}

AMOE_EXPORT int amoe_grouped_gemm_nn(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets,
                                     void* C, int dtype, int R, int E, int Kd, int N, void* workspace,
                                     size_t workspace_bytes, int tile_cfg, void* stream)
{
    const char* what = "grouped_gemm_nn";
    AMOE_REQUIRE(A && B && offsets && C && workspace, AMOE_ERR_BAD_ARG, "%s: null pointer", what);
    int rc = check_gemm_common(what, dtype, R, E, Kd, N, tile_cfg);
    if (rc) return rc;
    rc = check_gemm_dims(what, dtype, Kd, N);
    if (rc) return rc;
    AMOE_REQUIRE(workspace_bytes >= amoe_grouped_gemm_workspace_bytes(R, E), AMOE_ERR_WORKSPACE,
                 "%s: workspace %zu < %zu bytes", what, workspace_bytes, amoe_grouped_gemm_workspace_bytes(R, E));
    hipStream_t s = (hipStream_t)stream;
    if (dtype != AMOE_F32)
        return amoe_bf16_nn(A, a_row_map, B, offsets, C, R, E, Kd, N, workspace, workspace_bytes, tile_cfg, s, dtype);
    return amoe_f32_rows(A, a_row_map, B, offsets, C, R, E, Kd, N, N, (long long)Kd * N, false, workspace,
                         workspace_bytes, (tile_cfg & AMOE_TILE_MAP_READY) != 0, s);
}

AMOE_EXPORT int amoe_grouped_gemm_nt(const void* A, const int32_t* a_row_map, const void* B, const int32_t* offsets,
                                     void* C, int dtype, int R, int E, int Kd, int N, void* workspace,
                                     size_t workspace_bytes, int tile_cfg, void* stream)
{
    const char* what = "grouped_gemm_nt";
    AMOE_REQUIRE(A && B && offsets && C && workspace, AMOE_ERR_BAD_ARG, "%s: null pointer", what);
    int rc = check_gemm_common(what, dtype, R, E, Kd, N, tile_cfg);
    if (rc) return rc;
    rc = check_gemm_dims(what, dtype, N, Kd);  // the reduction runs over N here
    if (rc) return rc;
    AMOE_REQUIRE(workspace_bytes >= amoe_grouped_gemm_workspace_bytes(R, E), AMOE_ERR_WORKSPACE,
                 "%s: workspace %zu < %zu bytes", what, workspace_bytes, amoe_grouped_gemm_workspace_bytes(R, E));
    hipStream_t s = (hipStream_t)stream;
    if (dtype != AMOE_F32)
        return amoe_bf16_nt(A, a_row_map, B, offsets, C, R, E, Kd, N, workspace, workspace_bytes, tile_cfg, s, dtype);
    return amoe_f32_rows(A, a_row_map, B, offsets, C, R, E, /*Kred=*/N, /*N out=*/Kd, /*ldb=*/N, (long long)Kd * N, true,
                         workspace, workspace_bytes, (tile_cfg & AMOE_TILE_MAP_READY) != 0, s);
}

AMOE_EXPORT int amoe_grouped_gemm_wgrad(const void* A, const int32_t* a_row_map, const void* B,
                                        const int32_t* b_row_map, const int32_t* offsets, void* C, int dtype, int R,
                                        int E, int Kd, int N, int tile_cfg, void* stream)
{
    const char* what = "grouped_gemm_wgrad";
    AMOE_REQUIRE(A && B && offsets && C, AMOE_ERR_BAD_ARG, "%s: null pointer", what);
    AMOE_REQUIRE(!(a_row_map && b_row_map), AMOE_ERR_UNSUPPORTED, "%s: at most one operand may be gathered", what);
    int rc = check_gemm_common(what, dtype, R, E, Kd, N, tile_cfg);
    if (rc) return rc;
    const int vec = dtype != AMOE_F32 ? 8 : 4;
    AMOE_REQUIRE(Kd % vec == 0 && N % vec == 0, AMOE_ERR_UNSUPPORTED, "%s: extents (%d, %d) must be multiples of %d",
                 what, Kd, N, vec);
    hipStream_t s = (hipStream_t)stream;
    if (dtype != AMOE_F32) return amoe_bf16_wgrad(A, a_row_map, B, b_row_map, offsets, C, R, E, Kd, N, tile_cfg, s, dtype);
    return amoe_f32_wgrad(A, a_row_map, B, b_row_map, offsets, C, R, E, Kd, N, s);
}

AMOE_EXPORT int amoe_gated_bwd_score_parts(int I, int tile_cfg)
{
    if (I <= 0 || tile_cfg < 0) return 0;
    return amoe_bf16_gated_bwd_parts(I, tile_cfg);
}

AMOE_EXPORT int amoe_grouped_gemm_nt_gated_bwd(const void* dy, const int32_t* a_row_map, const void* w_down,
                                               const int32_t* offsets, const void* gate_up, const float* row_scale,
                                               void* d_gate_up, float* score_partials, int dtype, int R, int E, int I,
                                               int H, int act, void* workspace, size_t workspace_bytes, int tile_cfg,
                                               void* stream)
{
    const char* what = "grouped_gemm_nt_gated_bwd";
    AMOE_REQUIRE(dy && w_down && offsets && gate_up && d_gate_up && workspace, AMOE_ERR_BAD_ARG, "%s: null pointer", what);
    int rc = check_gemm_common(what, dtype, R, E, I, H, tile_cfg);
    if (rc) return rc;
    AMOE_REQUIRE(dtype != AMOE_F32, AMOE_ERR_UNSUPPORTED,
                 "%s: bf16 and float16 only (float32 callers run amoe_grouped_gemm_nt and amoe_gated_act_bwd)", what);
    AMOE_REQUIRE(act >= AMOE_ACT_SILU && act <= AMOE_ACT_GPT_OSS, AMOE_ERR_BAD_ARG, "%s: bad activation %d", what, act);
    AMOE_REQUIRE((long long)R * 2 * I < (1ll << 32), AMOE_ERR_UNSUPPORTED, "%s: an operand exceeds 2^32 elements", what);
    rc = check_gemm_dims(what, dtype, H, I);  // the reduction runs over H
    if (rc) return rc;
    AMOE_REQUIRE(workspace_bytes >= amoe_grouped_gemm_workspace_bytes(R, E), AMOE_ERR_WORKSPACE,
                 "%s: workspace %zu < %zu bytes", what, workspace_bytes, amoe_grouped_gemm_workspace_bytes(R, E));
    return amoe_bf16_nt_gated_bwd(dy, a_row_map, w_down, offsets, gate_up, row_scale, d_gate_up, score_partials, R, E, I, H,
                                  act, workspace, workspace_bytes, tile_cfg, (hipStream_t)stream, dtype);
}
