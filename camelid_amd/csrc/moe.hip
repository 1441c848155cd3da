// Mixture-of-experts dispatch (placeholder until the routed kernels land).
#include "cml_host.hpp"

using namespace cml;

extern "C" {

int cml_moe_route_top_k(const float *, int64_t, int, int, int32_t *, float *, cml_stream_t) {
    return fail(CML_ERR_UNSUPPORTED, "cml_moe_route_top_k is not built yet");
}

size_t cml_moe_workspace_bytes(int, int64_t, int64_t, int64_t, int, int) { return 0; }

int cml_moe_ffn(const cml_weight *, const cml_weight *, const cml_weight *, int, int, const int32_t *, const float *,
                const float *, int64_t, float *, void *, size_t, cml_stream_t) {
    return fail(CML_ERR_UNSUPPORTED, "cml_moe_ffn is not built yet");
}

}  // extern "C"
