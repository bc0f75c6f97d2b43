#include "common.hpp"
namespace hodu {
int launch_skinny(hodu_rocm_ctx *, int, int, const void *, const void *, void *, const DevProduct &) {
    return HODU_ROCM_UNSUPPORTED;
}
}  // namespace hodu
