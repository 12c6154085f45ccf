#include "ql_host.h"
#include "llaminar_amd/ql_api.h"
namespace llamql {
bool q6k_gemv_launch(const char *fn, const void *, const void *, float *, int32_t *, int, int, int, int, int, int, int, hipStream_t) { return fail(fn, "Q6_K not built yet"); }
bool iq3s_gemv_launch(const char *fn, const void *, const void *, float *, int32_t *, int, int, int, int, int, int, int, hipStream_t) { return fail(fn, "IQ3_S not built yet"); }
}
extern "C" {
size_t llam_ql_prepared_bytes(uint8_t fmt, int N, int K) { return (size_t)N * (K / 256) * (fmt == 5 ? 144 : fmt == 8 ? 210 : 112); }
bool llam_ql_prepare_weights(uint8_t, const void *, void *, int, int, int, void *) { return llamql::fail("stub", "not built yet"); }
bool llam_ql_gemm(uint8_t, const void *, const void *, float *, int, int, int, int, int, void *) { return llamql::fail("stub", "not built yet"); }
bool llam_ql_epilogue(float *, const float *, const float *, int, int, int, float, float, int, void *) { return llamql::fail("stub", "not built yet"); }
bool llam_ql_moe_route(const float *, int, int, int, int, int32_t *, float *, int, void *) { return llamql::fail("stub", "not built yet"); }
bool llam_ql_moe_gate_up(uint8_t, const llam_ql_expert *, const int32_t *, const void *, float *, float *, int, int, int, int, int, void *) { return llamql::fail("stub", "not built yet"); }
bool llam_ql_swiglu_quantize(const float *, const float *, float *, void *, int, int, int, void *) { return llamql::fail("stub", "not built yet"); }
bool llam_ql_moe_down(uint8_t, const llam_ql_expert *, const int32_t *, const float *, const void *, float *, int, int, int, int, int, int, void *) { return llamql::fail("stub", "not built yet"); }
}
