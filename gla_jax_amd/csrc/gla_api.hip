// Entry points of libgla_hip.so that carry no kernels of their own.
#include "gla_common.hpp"

extern "C" int gla_abi_version(void) { return GLA_HIP_ABI_VERSION; }

extern "C" const char *gla_status_string(int status)
{
    switch (status) {
    case GLA_OK: return "ok";
    case GLA_ERR_NULL: return "a required pointer is NULL";
    case GLA_ERR_SHAPE: return "unsupported shape (dimension <= 0, too large, or not a supported size)";
    case GLA_ERR_DTYPE: return "unsupported dtype combination";
    case GLA_ERR_CHUNK: return "chunk_size must be a supported power of two that divides T";
    case GLA_ERR_WORKSPACE: return "workspace missing or too small";
    case GLA_ERR_ALIGN: return "pointer not 16-byte aligned";
    case GLA_ERR_UNSUPPORTED: return "configuration not built in this library";
    default: break;
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "unknown status";
}
