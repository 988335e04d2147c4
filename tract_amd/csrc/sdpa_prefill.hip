// MFMA prefill attention for gfx950 (placeholder dispatch until the kernel lands).
#include "common.h"
namespace trocm {
int launch_sdpa_prefill(const SdpaArgs &, hipStream_t) { return 2; }
}  // namespace trocm
