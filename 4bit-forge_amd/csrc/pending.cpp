// Entry points declared in forge_hip.h whose kernels are not written yet.
#include "common.h"
#define NOT_YET(name) return forge::fail(FORGE_ERR_INVALID, name " is not implemented yet")
extern "C" int forge_hessian_update_grouped(const void*, int, int64_t, int64_t, const int64_t*, int64_t, const float*, const float*, float*, forge_stream_t) { NOT_YET("forge_hessian_update_grouped"); }
extern "C" int forge_chol_inv_upper_batched(float*, const float*, float*, float*, int32_t*, int64_t, int64_t, int, void*, int64_t, forge_stream_t) { NOT_YET("forge_chol_inv_upper_batched"); }
extern "C" int64_t forge_chol_workspace_bytes(int64_t, int64_t) { return 0; }
extern "C" int forge_hessian_permute(const float*, const int64_t*, const uint8_t*, float*, float*, float, int64_t, int64_t, forge_stream_t) { NOT_YET("forge_hessian_permute"); }
extern "C" int forge_weight_to_solver_order(const void*, int, int64_t, int64_t, const int64_t*, const uint8_t*, float*, int64_t, int64_t, int64_t, forge_stream_t) { NOT_YET("forge_weight_to_solver_order"); }
extern "C" int forge_codes_to_layer_order(const uint8_t*, const int64_t*, uint8_t*, int64_t, int64_t, int64_t, forge_stream_t) { NOT_YET("forge_codes_to_layer_order"); }
extern "C" int forge_pack_int4(const uint8_t*, const float*, int32_t*, int64_t, int64_t, int64_t, forge_stream_t) { NOT_YET("forge_pack_int4"); }
