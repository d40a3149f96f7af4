// placeholder until the MFMA backward lands
#include "sa2_common.h"
namespace sa2 {
bool mfma_bwd_supported(int, int, int, int, int, int, int) { return false; }
int launch_mfma_bwd(const Problem&, hipStream_t) { return SA2_ERR_UNSUPPORTED; }
size_t mfma_bwd_scratch_bytes(int, int, int, int, int, int) { return 0; }
}
