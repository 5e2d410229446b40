#include "mhffn_common.hpp"
namespace mhffn {
size_t bwd_workspace_bytes_bf16(const Dims& d) { return 16; }
hipError_t launch_bwd_bf16(const void*, const void*, const void*, const void*, const float*, const void*, void*, void*,
                           void*, void*, float*, int, void*, const Dims&, hipStream_t)
{
    return hipErrorNotSupported;
}
}  // namespace mhffn
