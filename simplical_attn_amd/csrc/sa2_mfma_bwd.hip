// placeholder until the MFMA backward lands
#include "sa2_common.h"
namespace sa2 {
int launch_mfma_bwd(const Problem&, hipStream_t) { return SA2_ERR_UNSUPPORTED; }
size_t mfma_bwd_scratch_bytes(int, int, int, int, int, int) { return 0; }
}
