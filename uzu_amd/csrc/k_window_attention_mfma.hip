// k_window_attention_mfma.hip -- the matrix-core form of the attention over cached keys and values (kernels_stream32.h::window_attention).
#include "device_utils.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

bool window_attention_mfma_supported(const WindowAttentionParams& p) { return false; }

uzu_status window_attention_mfma(hipStream_t s, const WindowAttentionParams& p) {
    set_error("window_attention: the matrix-core form does not take this shape");
    return UZU_ERR_UNSUPPORTED;
}

} // namespace k
} // namespace uzu
