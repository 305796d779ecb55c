// fp8 (e4m3) matrix-core attention kernel -- placeholder until the kernel lands.
#include "common.hpp"
namespace af3 {
bool mfma_fp8_eligible(const af3_dpa_params&) { return false; }
int  launch_dpa_mfma_fp8(const af3_dpa_params&, hipStream_t) { return AF3_ERR_BAD_DTYPE; }
}  // namespace af3
