// placeholder
#include "common.hpp"
#include "launch.hpp"
namespace d2dmoe {
bool mfma_dense_supported(const d2dmoe_shape&) { return false; }
size_t mfma_packed_bytes(const d2dmoe_shape&) { return 0; }
hipError_t launch_mfma_pack(const d2dmoe_shape&, const void*, const void*, const void*, const void*, const void*, const void*, void*, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_mfma_dense(const d2dmoe_shape&, const void*, const void*, const void*, const void*, void*, hipStream_t) { return hipErrorNotSupported; }
}
