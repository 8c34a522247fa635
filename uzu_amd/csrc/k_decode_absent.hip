// k_decode_absent.hip -- stands in for k_decode.hip in the `stream32` flavor of the library (make stream32 -> lib/libuzu_hip_stream32.so).
//
// k_decode.hip holds the fused decode-step kernels of the bf16-stream models: hundreds of template instances, four minutes of compile time -- more than every
// other source together.  The f32-stream designs never launch them, so a first use that only serves such a design (bin/trace_run in a fresh checkout) builds
// this flavor in well under a minute.  Here every entry of k_decode.hip refuses by name; model creation refuses a bf16-stream model before it gets that far
// (uzu_hip_decode_kernels_present below, engine_build.hip).
#include "internal.h"
#include "kernels_decode.h"

namespace uzu {
namespace k {

namespace {
uzu_status absent(const char* what) {
    set_error("%s: this library was built without the fused decode kernels of the bf16-stream models (make stream32); run `make -C uzu_amd/csrc` for the full library", what);
    return UZU_ERR_UNSUPPORTED;
}
} // namespace

bool gemv_dec_stripe_supported(const DecGemvParams&, int) { return false; }
uzu_status gemv_dec(hipStream_t, const DecGemvParams&, int, uint32_t*) { return absent("gemv_dec"); }
bool gemv_dec_plain_in_rht_supported(uint32_t, uint32_t) { return false; }
uzu_status argmax_commit(hipStream_t, const float*, const uint32_t*, uint32_t, uint32_t*, uint32_t*, uint32_t*, uint32_t*, const CommitEmbed*) { return absent("argmax_commit"); }
void gemv_dec_plan_query(const DecGemvParams&, int, DecGemvPlan* out) {
    if (out) *out = DecGemvPlan{};
}
uzu_status delta_dec(hipStream_t, const DeltaDecParams&) { return absent("delta_dec"); }
uzu_status attn_dec(hipStream_t, const AttnDecParams&, uint32_t) { return absent("attn_dec"); }
bool attn_dec_fused_supported(uint32_t, uint32_t, uint32_t, uint32_t, int) { return false; }
uzu_status attn_dec_check() { return UZU_OK; }
uzu_status attn_merge(hipStream_t, const float*, const float*, const float*, const uint16_t*, uint16_t*, uint32_t, uint32_t, uint32_t) { return absent("attn_merge"); }

} // namespace k
} // namespace uzu

extern "C" {
int uzu_hip_decode_kernels_present(void) { return 0; }
void uzu_hip_debug_set_timeline(unsigned long long*, uint32_t) {}
void uzu_hip_debug_set_attn_fused(int) {}
int uzu_hip_debug_attn_fused_built(void) { return 0; }
}
