// k_linear_mfma.hip -- the full-precision linear of the f32-stream designs on the matrix cores (kernels_stream32.h: linear_f32 with bf16 products).
#include "device_utils.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

bool linear_mfma_supported(const LinearF32Params& p) {
    (void)p;
    return false;
}
uzu_status linear_mfma(hipStream_t s, const LinearF32Params& p) {
    (void)s, (void)p;
    set_error("linear_mfma: shape not covered");
    return UZU_ERR_UNSUPPORTED;
}

} // namespace k
} // namespace uzu
