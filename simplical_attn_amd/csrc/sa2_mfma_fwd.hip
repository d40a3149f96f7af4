// placeholder until the MFMA forward lands
#include "sa2_common.h"
namespace sa2 {
bool mfma_supported(int, int, int, int, int, int, int) { return false; }
bool mfma_layout_ok(const Problem&, bool) { return false; }
int launch_mfma_fwd(const Problem&, hipStream_t) { return SA2_ERR_UNSUPPORTED; }
}
