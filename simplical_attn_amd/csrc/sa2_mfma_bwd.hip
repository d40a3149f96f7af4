// MFMA backward for gfx950 (bf16 or fp16, head_dim 32, 64 or 128): dispatch to the two kernels,
// sa2_mfma_bwd_kp.hip for dQ, dK', dV' and sa2_mfma_bwd_kv.hip for dK, dV, after the row-dot kernel.
//
// Same expanded-row view as the forward: rows r = (i, delta), Q~[r] = q[i] *
// k2~[i-delta] * scale*log2(e) and dO~[r] = dO[i] * v2~[i-delta], both in the element type, with
// P = exp2(S - LSE*log2e) recomputed from the saved log-sum-exp and dS = P * (dO~.v1 - D_i).
// Both kernels take any K' window: one too wide for their LDS buffers is walked in segments of deltas.
//
// Every output element has one writer and a fixed summation order: no atomics,
// bitwise reproducible.
#include "sa2_mfma_common.h"

namespace sa2 {

bool mfma_bwd_supported(int B, int N, int H, int D, int w1, int w2, int dtype) {
    return mfma_supported(B, N, H, D, w1, w2, dtype);
}

// Workspace of the K'-side kernel (dQ partials, and the dK', dV' partials of a segmented launch),
// rounded up so that what follows it stays 256-byte aligned
size_t kp_side_scratch_bytes(int B, int N, int H, int D, int w2) {
    return (kp_scratch_bytes(B, N, H, D, w2) + 255) / 256 * 256;
}

size_t mfma_bwd_scratch_bytes(int B, int N, int H, int D, int w1, int w2) {
    return kp_side_scratch_bytes(B, N, H, D, w2) + kv_split_scratch_bytes(B, N, H, D, w1, w2);
}

int launch_mfma_bwd(const Problem& p, int dtype, hipStream_t st) {
    int rc = launch_rowdot(p.out, p.dout, p.dsum, p.B, p.N, p.H, p.D, dtype, st);
    if (rc != SA2_OK) return rc;
    if (p.dq.p || p.dk2.p || p.dv2.p) {
        rc = launch_mfma_bwd_kp(p, dtype, st);
        if (rc != SA2_OK) return rc;
    }
    if (p.dk1.p || p.dv1.p) rc = launch_mfma_bwd_kv(p, dtype, st);
    return rc;
}

}  // namespace sa2
