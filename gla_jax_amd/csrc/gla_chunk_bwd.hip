#include "gla_chunk_common.hpp"
#include "gla_chunk_kernels.hpp"
namespace gla {
template <typename T, int C, int D>
int launch_chunk_grad(hipStream_t, int, int, int, const float *, const void *, const void *, const void *,
                      const void *, const void *, const void *, const float *, float *, void *, void *, void *)
{
    return GLA_ERR_UNSUPPORTED;
}
#define GLA_INST_GRAD(T, C, D)                                                                           \
    template int launch_chunk_grad<T, C, D>(hipStream_t, int, int, int, const float *, const void *,     \
                                            const void *, const void *, const void *, const void *,     \
                                            const void *, const float *, float *, void *, void *, void *);
GLA_FOR_EACH_CHUNK_CONFIG(GLA_INST_GRAD)
}  // namespace gla
