// Fused GAT layer core (placeholder until the kernels land).
#include "common.h"

using namespace jg;
#define JG_EXPORT extern "C" __attribute__((visibility("default")))

JG_EXPORT int32_t jgamd_gat_fwd_workspace(int32_t, int64_t, int32_t, int32_t, size_t *bytes)
{
    if (bytes) *bytes = 0;
    return fail(JGAMD_ERR_UNSUPPORTED, "gat_fwd: not implemented");
}
JG_EXPORT int32_t jgamd_gat_fwd(const int32_t *, const int32_t *, const float *, const float *, const float *, float,
                                float *, float *, float *, float *, float *, float *, int32_t, int64_t, int32_t,
                                int32_t, void *, size_t, void *)
{
    return fail(JGAMD_ERR_UNSUPPORTED, "gat_fwd: not implemented");
}
JG_EXPORT int32_t jgamd_gat_bwd_workspace(int32_t, int64_t, int32_t, int32_t, size_t *bytes)
{
    if (bytes) *bytes = 0;
    return fail(JGAMD_ERR_UNSUPPORTED, "gat_bwd: not implemented");
}
JG_EXPORT int32_t jgamd_gat_bwd(const int32_t *, const int32_t *, const int32_t *, const int32_t *, const float *,
                                const float *, const float *, float, const float *, const float *, const float *,
                                const float *, const float *, const float *, float *, float *, float *, int32_t,
                                int64_t, int32_t, int32_t, void *, size_t, void *)
{
    return fail(JGAMD_ERR_UNSUPPORTED, "gat_bwd: not implemented");
}
