#include "fsta_common.h"
namespace fsta {
bool mfma_supported(int, int, int) { return false; }
int launch_attention_mfma(const AttnParams&, int, int, bool, hipStream_t) {
    return fail(FSTA_EUNSUPPORTED, "matrix-core kernel not built");
}
}
