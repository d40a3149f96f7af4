// fp32 tensors on the matrix pipes of gfx950: forward and backward with v_mfma_f32_32x32x2_f32
// (fp32 products, fp32 accumulation), head_dim 32, 64 or 128.
//
// Same expanded-row view as the 16-bit kernels: rows r = (i, delta), Q~[r] = q[i] * (k2[i-delta] +
// k2_bias) * scale*log2(e), dO~[r] = dO[i] * (v2[i-delta] + v2_bias), everything in fp32.  A 32x32x2
// MFMA takes one fp32 value per lane for each operand (lane l: row or column l % 32, contraction slot
// l / 32) and leaves a 32x32 tile in 16 registers (register v of lane l: row 8*(v/4) + 4*(l/32) + v%4,
// column l % 32).  With the logits computed transposed (S^T = K1 . Q~^T) register v of a lane is the
// weight of its expanded row and of key 8*(v/4) + 4*(l/32) + v%4 of the tile: exactly the B operand of
// MFMA number v of the second contraction R^T += V1^T . P^T, whose A operand is one fp32 per lane read
// from the row-major V tile in LDS.  No transposed copies, no shuffles.
//
// These kernels are bound by the MFMA chains themselves (64 cycles per instruction, D MFMAs per
// tile and contraction), so the structure is kept simple: four wavefronts per workgroup, one per SIMD
// with the whole register file (accumulators in AGPRs), K/V tiles through a double-buffered LDS stage
// written from registers, one barrier per tile.
//
//   f32_fwd_kernel      32 queries per workgroup; wavefront w takes delta = w, w+4, ... and keeps one
//                       online softmax and one output accumulator across its units; the four are
//                       merged once at the end.
//   f32_bwd_kp_kernel   32 K' rows per workgroup and every delta.  After a unit's sweep its three
//                       reductions go to fp32 accumulators in LDS in column-rotated phases: dK' and
//                       dV' rows are aligned with the unit's rows, dQ rows are shifted by delta; the
//                       dQ accumulator is written once per workgroup as a partial that
//                       f32_dq_sum_kernel adds up in block order.
//   f32_bwd_kv_kernel   128 K/V rows per workgroup (32 per wavefront, resident in registers as B
//                       operands), streaming every unit (query block, delta) that can see them.
// Every output element has one writer and a fixed summation order: no atomics, bitwise reproducible.
#include "sa2_mfma_common.h"

namespace sa2 {
namespace {

constexpr int XW = 4;                  // wavefronts per workgroup
constexpr int XT = XW * 64;            // threads per workgroup
constexpr int XJ = XW * 32;            // K rows per workgroup of the K-side kernel

template <int D>
struct F32Cfg {
    static constexpr int DG = D / 8;           // groups of 8 contraction columns: one float4 per lane and group
    static constexpr int DT = D / 32;          // 32-column blocks of an output contraction
    static constexpr int RS = D + 4;           // row stride of a tile in LDS (floats)
    static constexpr int TILE = 32 * RS;       // floats
    static constexpr int STAGE = 2 * TILE;     // two tiles (K and V, or Q~ and dO~)
    static constexpr int KR = 32 * D / 4 / XT; // float4 per thread and tile
    static constexpr size_t TILES_BYTES = (size_t)2 * STAGE * 4;           // = XW * 32 * RS * 4: also the merge buffer
    static constexpr size_t FWD_LDS = TILES_BYTES + 2 * XW * 32 * 4;
    static constexpr size_t LDS_LIMIT = 160 * 1024;
    // K'-side kernel: the stages, the dQ accumulator (32 + w2 rows) and the dK' and dV' accumulators (32 rows each)
    static size_t kp_lds(int w2) { return TILES_BYTES + (size_t)(32 + w2 + 64) * RS * 4; }
    static bool kp_fits(int w2) { return kp_lds(w2) <= LDS_LIMIT; }
    // deltas whose dQ rows the accumulator holds at once: all w2 + 1 of them, or (wider K' windows) the largest
    // multiple of four that fits; the kernel then walks the window in segments of that many deltas
    static int kp_segment(int w2) {
        if (kp_fits(w2)) return w2 + 1;
        int segw = 32;
        while (kp_fits(segw + XW - 1)) segw += XW;
        return segw;
    }
    static constexpr size_t KV_LDS = TILES_BYTES + 2 * 2 * 32 * 4;
};

__device__ __forceinline__ floatx16 mfma_f32(float a, float b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ floatx16 zero16() {
    floatx16 z;
#pragma unroll
    for (int v = 0; v < 16; ++v) z[v] = 0.f;
    return z;
}
__device__ __forceinline__ int xcd_order(int pid, int total) {
    // workgroups are dealt round-robin to the 8 XCDs: neighbours in the problem share an L2
    return (total & 7) == 0 ? (pid & 7) * (total >> 3) + (pid >> 3) : pid;
}

typedef float fx4 __attribute__((ext_vector_type(4)));      // 16 bytes in flight (a plain vector: stays in registers)

// Rows [j0, j0+32) of two tensors (clamped to the sequence) from global memory to registers, and
// from there to the two tiles of a stage.
template <int D>
__device__ __forceinline__ void tile_load(fx4 (&a)[F32Cfg<D>::KR], fx4 (&b)[F32Cfg<D>::KR], const float* ap, int64_t as,
                                          const float* bp, int64_t bs, int j0, int N, int tid) {
#pragma unroll
    for (int u = 0; u < F32Cfg<D>::KR; ++u) {
        const int c = tid + XT * u;
        const int row = c / (D / 4), col = c - row * (D / 4);
        int j = j0 + row;
        j = j < N ? j : N - 1;
        a[u] = *(const fx4*)(ap + (int64_t)j * as + col * 4);
        b[u] = *(const fx4*)(bp + (int64_t)j * bs + col * 4);
    }
}
template <int D>
__device__ __forceinline__ void tile_store(const fx4 (&a)[F32Cfg<D>::KR], const fx4 (&b)[F32Cfg<D>::KR], float* stage, int tid) {
    using C = F32Cfg<D>;
#pragma unroll
    for (int u = 0; u < C::KR; ++u) {
        const int c = tid + XT * u;
        const int row = c / (D / 4), col = c - row * (D / 4);
        *(fx4*)(stage + row * C::RS + col * 4) = a[u];
        *(fx4*)(stage + C::TILE + row * C::RS + col * 4) = b[u];
    }
}

// ================================================================== forward =====
template <int D>
__global__ __launch_bounds__(XT) __attribute__((amdgpu_waves_per_eu(D <= 64 ? 2 : 1, D <= 64 ? 2 : 1)))
void f32_fwd_kernel(Problem p, int nqb, int total) {
    using C = F32Cfg<D>;
    extern __shared__ __attribute__((aligned(16))) float smem_f[];
    float* mrg_m = smem_f + 2 * C::STAGE;        // [XW][32]
    float* mrg_l = mrg_m + XW * 32;              // [XW][32]

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;
    const int pid = xcd_order(blockIdx.x, total);
    const int bh = pid / nqb, qb = pid - bh * nqb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int i0 = qb * BQ, i = i0 + ln, ic = i < N ? i : N - 1;
    const int i_last = i0 + BQ - 1 < N ? i0 + BQ - 1 : N - 1;

    const float* qp = (const float*)p.q.p + p.q.off(b, 0, h);
    const float* k1p = (const float*)p.k1.p + p.k1.off(b, 0, h);
    const float* k2p = (const float*)p.k2.p + p.k2.off(b, 0, h);
    const float* v1p = (const float*)p.v1.p + p.v1.off(b, 0, h);
    const float* v2p = (const float*)p.v2.p + p.v2.off(b, 0, h);

    const int jt_lo = (i0 - w1 > 0 ? i0 - w1 : 0) / TJ, jt_hi = i_last / TJ;
    const int nt = jt_hi - jt_lo + 1;
    const int n_units = (w2 < i_last ? w2 : i_last) + 1;
    const int nrounds = (n_units + XW - 1) / XW;
    const int total_steps = nrounds * nt;
    const float qscale = p.scale * LOG2E;

    fx4 tk[C::KR], tv[C::KR];                    // the tile on its way from global memory to LDS
    tile_load<D>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, jt_lo * TJ, N, tid);
    tile_store<D>(tk, tv, smem_f, tid);
    tile_load<D>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, (jt_lo + 1 % nt) * TJ, N, tid);
    __syncthreads();

    // the wavefront's running softmax over its units: reference exponent, sum, weighted output
    float M = -INFINITY, L = 0.f;
    floatx16 oacc[C::DT];
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt) oacc[dt] = zero16();

    int g = 0;
    for (int round = 0; round < nrounds; ++round) {
        const int delta = round * XW + wave;
        const bool ok = delta < n_units;
        const int kr = ic - delta > 0 ? ic - delta : 0;
        const bool row_ok = ok && i < N && i >= delta;
        const bool rows_full = i0 >= delta && i0 + BQ - 1 < N;

        float qf[D / 2];
        if (ok) {
#pragma unroll
            for (int gg = 0; gg < C::DG; ++gg) {
                const float4 qa = *(const float4*)(qp + (int64_t)ic * p.q.sn + 8 * gg + 4 * hf);
                const float4 kb = *(const float4*)(k2p + (int64_t)kr * p.k2.sn + 8 * gg + 4 * hf);
                qf[4 * gg + 0] = qa.x * qscale * (kb.x + p.k2_bias);
                qf[4 * gg + 1] = qa.y * qscale * (kb.y + p.k2_bias);
                qf[4 * gg + 2] = qa.z * qscale * (kb.z + p.k2_bias);
                qf[4 * gg + 3] = qa.w * qscale * (kb.w + p.k2_bias);
            }
        }
        float m = -INFINITY, l = 0.f;
        floatx16 racc[C::DT];
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) racc[dt] = zero16();

        for (int s = 0; s < nt; ++s, ++g) {
            if (ok) {
                const int j0 = (jt_lo + s) * TJ;
                const float* Ks = smem_f + (g & 1) * C::STAGE;
                const float* Vs = Ks + C::TILE;
                floatx16 sacc = zero16();
#pragma unroll
                for (int gg = 0; gg < C::DG; ++gg) {
                    const float4 ka = *(const float4*)(Ks + ln * C::RS + 8 * gg + 4 * hf);
                    sacc = mfma_f32(ka.x, qf[4 * gg + 0], sacc);
                    sacc = mfma_f32(ka.y, qf[4 * gg + 1], sacc);
                    sacc = mfma_f32(ka.z, qf[4 * gg + 2], sacc);
                    sacc = mfma_f32(ka.w, qf[4 * gg + 3], sacc);
                }
                // register v of this lane: key j0 + 8*(v/4) + 4*hf + v%4
                const bool interior = rows_full && (j0 + TJ - 1 <= i0) && (j0 >= i0 + BQ - 1 - w1);
                if (!interior) {
                    const int hi = i - j0 - 4 * hf, lo = hi - w1;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int c = 8 * (v >> 2) + (v & 3);
                        sacc[v] = (row_ok && c <= hi && c >= lo) ? sacc[v] : -INFINITY;
                    }
                }
                float mx = sacc[0];
#pragma unroll
                for (int v = 1; v < 16; ++v) mx = fmaxf(mx, sacc[v]);
                mx = fmaxf(mx, other_half(mx));
                const float m_new = fmaxf(m, mx);
                const float m_use = m_new == -INFINITY ? 0.f : m_new;
                const float alpha = fast_exp2(m - m_use);
                m = m_new;
                if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
                    l *= alpha;
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                        for (int v = 0; v < 16; ++v) racc[dt][v] *= alpha;
                }
                float pv[16];
                float rs = 0.f;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    pv[v] = fast_exp2(sacc[v] - m_use);
                    rs += pv[v];
                }
                l += rs;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float* vrow = Vs + (8 * (v >> 2) + 4 * hf + (v & 3)) * C::RS + ln;
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt) racc[dt] = mfma_f32(vrow[dt * 32], pv[v], racc[dt]);
                }
            }
            // (unconditional: past the last step this moves a tile nobody reads, which is cheaper than a branch
            // around register arrays)
            tile_store<D>(tk, tv, smem_f + ((g + 1) & 1) * C::STAGE, tid);
            tile_load<D>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, (jt_lo + (g + 2) % nt) * TJ, N, tid);
            __syncthreads();
        }

        if (ok) {
            // fold the unit into the wavefront's running result: O += e^(m-M) * (v2 + bias) * R
            const float lt = l + other_half(l);
            const float M_new = fmaxf(M, m);
            const float Mu = M_new == -INFINITY ? 0.f : M_new;
            const float a = fast_exp2(M - Mu), c = fast_exp2(m - Mu);
            L = L * a + lt * c;
            M = M_new;
            const float* vrow = v2p + (int64_t)kr * p.v2.sn + 4 * hf;
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const float4 x = *(const float4*)(vrow + dt * 32 + 8 * g4);
                    oacc[dt][4 * g4 + 0] = oacc[dt][4 * g4 + 0] * a + c * racc[dt][4 * g4 + 0] * (x.x + p.v2_bias);
                    oacc[dt][4 * g4 + 1] = oacc[dt][4 * g4 + 1] * a + c * racc[dt][4 * g4 + 1] * (x.y + p.v2_bias);
                    oacc[dt][4 * g4 + 2] = oacc[dt][4 * g4 + 2] * a + c * racc[dt][4 * g4 + 2] * (x.z + p.v2_bias);
                    oacc[dt][4 * g4 + 3] = oacc[dt][4 * g4 + 3] * a + c * racc[dt][4 * g4 + 3] * (x.w + p.v2_bias);
                }
        }
    }

    // ---- merge the four wavefronts (the tile stages are free: the sweep's last barrier is behind us) ----
    float* mrg = smem_f;                                   // [XW][32][RS]
    {
        float* row = mrg + (wave * 32 + ln) * C::RS + 4 * hf;
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)
                *(float4*)(row + dt * 32 + 8 * g4) = make_float4(oacc[dt][4 * g4], oacc[dt][4 * g4 + 1], oacc[dt][4 * g4 + 2],
                                                                 oacc[dt][4 * g4 + 3]);
        if (hf == 0) {
            mrg_m[wave * 32 + ln] = M;
            mrg_l[wave * 32 + ln] = L;
        }
    }
    __syncthreads();
    const int row = tid >> 3, io = i0 + row;
    if (io < N) {
        float Mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < XW; ++w) Mx = fmaxf(Mx, mrg_m[w * 32 + row]);
        const float Mu = Mx == -INFINITY ? 0.f : Mx;
        float wgt[XW], Ls = 0.f;
#pragma unroll
        for (int w = 0; w < XW; ++w) {
            wgt[w] = fast_exp2(mrg_m[w * 32 + row] - Mu);
            Ls += mrg_l[w * 32 + row] * wgt[w];
        }
        // sum_w + 1e-8 in units of 2^Mu (reference.py:74); for a tiny Mu the epsilon dominates
        const bool big = Mu > LOG2_EPS;
        const float denom = big ? Ls + 1e-8f * fast_exp2(-Mu) : Ls * fast_exp2(Mu - LOG2_EPS) + 1.f;
        const float inv = big ? 1.f / denom : fast_exp2(Mu - LOG2_EPS) / denom;
        float* orow = (float*)p.out.p + p.out.off(b, io, h);
#pragma unroll
        for (int x = 0; x < C::DT; ++x) {
            const int col = 32 * x + 4 * (tid & 7);
            float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int w = 0; w < XW; ++w) {
                const float4 y = *(const float4*)(mrg + (w * 32 + row) * C::RS + col);
                acc.x += wgt[w] * y.x; acc.y += wgt[w] * y.y; acc.z += wgt[w] * y.z; acc.w += wgt[w] * y.w;
            }
            *(float4*)(orow + col) = make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
        }
        if ((tid & 7) == 0)
            p.lse[(int64_t)bh * N + io] = big ? LN2 * Mu + logf(denom) : LN_EPS + logf(denom);
    }
}

// ============================================== backward, K' side: dQ, dK', dV' =====
// SEG: the K' window is walked in segments of segw deltas (a kernel of its own; segw = w2 + 1 otherwise)
template <int D, bool SEG>
__global__ __launch_bounds__(XT) __attribute__((amdgpu_waves_per_eu(D <= 64 ? 2 : 1, D <= 64 ? 2 : 1)))
void f32_bwd_kp_kernel(Problem p, int nkb, int total, float* __restrict__ dq_part, int segw) {
    using C = F32Cfg<D>;
    extern __shared__ __attribute__((aligned(16))) float smem_f[];
    float* dk_s = smem_f + 2 * C::STAGE;         // [32][RS]: dK' rows k0 .. k0+31 (before the scale)
    float* dv_s = dk_s + 32 * C::RS;             // [32][RS]: dV' rows
    float* dq_s = dv_s + 32 * C::RS;             // [32 + segw - 1][RS]: dQ rows k0 + dbase .. of the current segment (before the scale)

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;
    const int pid = xcd_order(blockIdx.x, total);
    const int bh = pid / nkb, kb = pid - bh * nkb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int k0 = kb * BQ, k = k0 + ln, kc = k < N ? k : N - 1;
    const int NR = 32 + w2;                      // rows of the block's dQ partial
    const int NRS = 32 + segw - 1;               // rows of the accumulator
    int dbase = 0;                               // first delta of the current segment

    const float* qp = (const float*)p.q.p + p.q.off(b, 0, h);
    const float* k1p = (const float*)p.k1.p + p.k1.off(b, 0, h);
    const float* k2p = (const float*)p.k2.p + p.k2.off(b, 0, h);
    const float* v1p = (const float*)p.v1.p + p.v1.off(b, 0, h);
    const float* v2p = (const float*)p.v2.p + p.v2.off(b, 0, h);
    const float* dop = (const float*)p.dout.p + p.dout.off(b, 0, h);
    const bool want_dq = p.dq.p != nullptr;

    const int n_units = (w2 < N - 1 - k0 ? w2 : N - 1 - k0) + 1;       // delta with k0 + delta < N
    const int nrounds = (n_units + XW - 1) / XW;
    const float qscale = p.scale * LOG2E;

    for (int c = tid; c < (NRS + 64) * C::RS; c += XT) dk_s[c] = 0.f;      // all three accumulators

    fx4 tk[C::KR], tv[C::KR];                    // the tile on its way from global memory to LDS
    for (int round = 0; round < nrounds; ++round) {
        // queries of the round's units: k0 + 4*round .. k0 + 31 + 4*round + 3 (within the sequence)
        const int d_first = round * XW, d_last = d_first + XW - 1 < n_units - 1 ? d_first + XW - 1 : n_units - 1;
        const int i_min = k0 + d_first, i_max = k0 + 31 + d_last < N - 1 ? k0 + 31 + d_last : N - 1;
        const int jt_lo = (i_min - w1 > 0 ? i_min - w1 : 0) / TJ, jt_hi = i_max / TJ;
        const int nt = jt_hi - jt_lo + 1;

        const int delta = d_first + wave;
        const bool ok = delta < n_units;
        const int i = k + delta, ic = i < N ? i : N - 1;
        const bool row_ok = ok && i < N;                  // (k <= i < N)
        const int iw_lo = k0 + delta, iw_hi = k0 + 31 + delta < N - 1 ? k0 + 31 + delta : N - 1;   // this unit's queries
        const bool rows_full = k0 + 31 + delta < N;

        float qf[D / 2], dof[D / 2];
        float lse2 = 0.f, dsum = 0.f;
        if (ok) {
#pragma unroll
            for (int gg = 0; gg < C::DG; ++gg) {
                const float4 qa = *(const float4*)(qp + (int64_t)ic * p.q.sn + 8 * gg + 4 * hf);
                const float4 ka = *(const float4*)(k2p + (int64_t)kc * p.k2.sn + 8 * gg + 4 * hf);
                const float4 da = *(const float4*)(dop + (int64_t)ic * p.dout.sn + 8 * gg + 4 * hf);
                const float4 va = *(const float4*)(v2p + (int64_t)kc * p.v2.sn + 8 * gg + 4 * hf);
                qf[4 * gg + 0] = qa.x * qscale * (ka.x + p.k2_bias);
                qf[4 * gg + 1] = qa.y * qscale * (ka.y + p.k2_bias);
                qf[4 * gg + 2] = qa.z * qscale * (ka.z + p.k2_bias);
                qf[4 * gg + 3] = qa.w * qscale * (ka.w + p.k2_bias);
                dof[4 * gg + 0] = da.x * (va.x + p.v2_bias);
                dof[4 * gg + 1] = da.y * (va.y + p.v2_bias);
                dof[4 * gg + 2] = da.z * (va.z + p.v2_bias);
                dof[4 * gg + 3] = da.w * (va.w + p.v2_bias);
            }
            lse2 = p.lse[(int64_t)bh * N + ic] * LOG2E;
            dsum = p.dsum[(int64_t)bh * N + ic];
        }
        floatx16 racc[C::DT], gacc[C::DT];
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) racc[dt] = gacc[dt] = zero16();

        // (the previous round's last barrier has passed: both stages are free)
        tile_load<D>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, jt_lo * TJ, N, tid);
        tile_store<D>(tk, tv, smem_f, tid);
        if (nt > 1) tile_load<D>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, (jt_lo + 1) * TJ, N, tid);
        __syncthreads();
        for (int s = 0; s < nt; ++s) {
            const int j0 = (jt_lo + s) * TJ;
            // tiles that hold no key of this unit's windows are skipped by the wavefront
            if (ok && j0 <= iw_hi && j0 + TJ - 1 >= iw_lo - w1) {
                const float* Ks = smem_f + (s & 1) * C::STAGE;
                const float* Vs = Ks + C::TILE;
                floatx16 sacc = zero16(), dpacc = zero16();
#pragma unroll
                for (int gg = 0; gg < C::DG; ++gg) {
                    const float4 ka = *(const float4*)(Ks + ln * C::RS + 8 * gg + 4 * hf);
                    const float4 va = *(const float4*)(Vs + ln * C::RS + 8 * gg + 4 * hf);
                    sacc = mfma_f32(ka.x, qf[4 * gg + 0], sacc);
                    dpacc = mfma_f32(va.x, dof[4 * gg + 0], dpacc);
                    sacc = mfma_f32(ka.y, qf[4 * gg + 1], sacc);
                    dpacc = mfma_f32(va.y, dof[4 * gg + 1], dpacc);
                    sacc = mfma_f32(ka.z, qf[4 * gg + 2], sacc);
                    dpacc = mfma_f32(va.z, dof[4 * gg + 2], dpacc);
                    sacc = mfma_f32(ka.w, qf[4 * gg + 3], sacc);
                    dpacc = mfma_f32(va.w, dof[4 * gg + 3], dpacc);
                }
                const bool interior = rows_full && (j0 + TJ - 1 <= iw_lo) && (j0 >= iw_lo + 31 - w1);
                float pv[16], dsv[16];
                const int hi = i - j0 - 4 * hf, lo = hi - w1;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int c = 8 * (v >> 2) + (v & 3);
                    const bool valid = interior || (row_ok && c <= hi && c >= lo);
                    pv[v] = valid ? fast_exp2(sacc[v] - lse2) : 0.f;
                    dsv[v] = pv[v] * (dpacc[v] - dsum);
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int rr = (8 * (v >> 2) + 4 * hf + (v & 3)) * C::RS + ln;
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt) {
                        racc[dt] = mfma_f32(Vs[rr + dt * 32], pv[v], racc[dt]);
                        gacc[dt] = mfma_f32(Ks[rr + dt * 32], dsv[v], gacc[dt]);
                    }
                }
            }
            if (s + 1 < nt) tile_store<D>(tk, tv, smem_f + ((s + 1) & 1) * C::STAGE, tid);
            if (s + 2 < nt) tile_load<D>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, (jt_lo + s + 2) * TJ, N, tid);
            __syncthreads();
        }

        // ---- the unit's reductions into the workgroup's LDS accumulators:
        //      dK'[k] += G*q[i], dV'[k] += R*dO[i] (rows ln), dQ[i] += G*k2~[k] (rows ln + delta).
        //      Four phases; in phase ph wavefront w owns column group (w + ph) % 4 of every row, so no
        //      two wavefronts touch an element at once and every element sums in a fixed order. ----
#pragma unroll
        for (int ph = 0; ph < 4; ++ph) {
            if (row_ok) {
                const int g4 = (wave + ph) & 3;
                const int col = 8 * g4 + 4 * hf;
                const float* qrow = qp + (int64_t)ic * p.q.sn + col;
                const float* drow = dop + (int64_t)ic * p.dout.sn + col;
                const float* krow = k2p + (int64_t)kc * p.k2.sn + col;
                float* dkrow = dk_s + ln * C::RS + col;
                float* dvrow = dv_s + ln * C::RS + col;
                float* dqrow = dq_s + (ln + delta - dbase) * C::RS + col;
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt) {
                    // (g4 is uniform over the wavefront: pick this group's four registers)
                    float gv[4], rv[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        gv[t] = g4 == 0 ? gacc[dt][t] : g4 == 1 ? gacc[dt][4 + t] : g4 == 2 ? gacc[dt][8 + t] : gacc[dt][12 + t];
                        rv[t] = g4 == 0 ? racc[dt][t] : g4 == 1 ? racc[dt][4 + t] : g4 == 2 ? racc[dt][8 + t] : racc[dt][12 + t];
                    }
                    const float4 qx = *(const float4*)(qrow + dt * 32);
                    const float4 dx = *(const float4*)(drow + dt * 32);
                    float4 a = *(float4*)(dkrow + dt * 32);
                    a.x += gv[0] * qx.x; a.y += gv[1] * qx.y; a.z += gv[2] * qx.z; a.w += gv[3] * qx.w;
                    *(float4*)(dkrow + dt * 32) = a;
                    float4 c = *(float4*)(dvrow + dt * 32);
                    c.x += rv[0] * dx.x; c.y += rv[1] * dx.y; c.z += rv[2] * dx.z; c.w += rv[3] * dx.w;
                    *(float4*)(dvrow + dt * 32) = c;
                    if (want_dq) {
                        const float4 kx = *(const float4*)(krow + dt * 32);
                        float4 o = *(float4*)(dqrow + dt * 32);
                        o.x += gv[0] * (kx.x + p.k2_bias); o.y += gv[1] * (kx.y + p.k2_bias);
                        o.z += gv[2] * (kx.z + p.k2_bias); o.w += gv[3] * (kx.w + p.k2_bias);
                        *(float4*)(dqrow + dt * 32) = o;
                    }
                }
            }
            __syncthreads();
        }
        // ---- end of a segment: its first segw dQ rows are complete and go to the partial; the 31 rows the next
        //      segment shares with it move to the front of the accumulator ----
        if (SEG && round + 1 < nrounds && (round + 1) * XW - dbase >= segw) {
            if (want_dq) {
                float* part = dq_part + (((int64_t)bh * nkb + kb) * (int64_t)NR + dbase) * D;
                for (int c = tid; c < segw * (D / 4); c += XT) {
                    const int r = c / (D / 4), col = c - r * (D / 4);
                    *(float4*)(part + (int64_t)r * D + col * 4) = *(const float4*)(dq_s + r * C::RS + col * 4);
                }
                __syncthreads();
                for (int c = tid; c < 31 * (D / 4); c += XT) {          // (segw >= 32: source and destination are disjoint)
                    const int r = c / (D / 4), col = c - r * (D / 4);
                    *(float4*)(dq_s + r * C::RS + col * 4) = *(const float4*)(dq_s + (segw + r) * C::RS + col * 4);
                }
                __syncthreads();
                for (int c = tid; c < (NRS - 31) * (D / 4); c += XT) {
                    const int r = 31 + c / (D / 4), col = c % (D / 4);
                    *(float4*)(dq_s + r * C::RS + col * 4) = make_float4(0.f, 0.f, 0.f, 0.f);
                }
                __syncthreads();
            }
            dbase += segw;
        }
    }

    // ---- dK' and dV' rows of the block ----
    {
        const int row = tid >> 3, ko = k0 + row;
        if (ko < N) {
#pragma unroll
            for (int x = 0; x < C::DT; ++x) {
                const int col = 32 * x + 4 * (tid & 7);
                if (p.dk2.p) {
                    const float4 a = *(const float4*)(dk_s + row * C::RS + col);
                    *(float4*)((float*)p.dk2.p + p.dk2.off(b, ko, h) + col) =
                        make_float4(a.x * p.scale, a.y * p.scale, a.z * p.scale, a.w * p.scale);
                }
                if (p.dv2.p) *(float4*)((float*)p.dv2.p + p.dv2.off(b, ko, h) + col) = *(const float4*)(dv_s + row * C::RS + col);
            }
        }
    }
    // ---- dQ partial of this block: rows k0 .. k0+31+w2, of which those from dbase on are still here
    //      (rows past the accumulator belong to deltas beyond the end of the sequence: zeros) ----
    if (want_dq) {
        float* part = dq_part + (((int64_t)bh * nkb + kb) * (int64_t)NR + dbase) * D;
        for (int c = tid; c < (NR - dbase) * (D / 4); c += XT) {
            const int r = c / (D / 4), col = c - r * (D / 4);
            *(float4*)(part + (int64_t)r * D + col * 4) =
                r < NRS ? *(const float4*)(dq_s + r * C::RS + col * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
}

// dQ[i] = scale * sum over the K' blocks kb with 32*kb <= i <= 32*kb + 31 + w2, in block order
template <int D>
__global__ __launch_bounds__(256) void f32_dq_sum_kernel(Problem p, int nkb, const float* __restrict__ dq_part, int64_t chunks) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= chunks) return;
    const int col = (int)(c % (D / 4));
    const int64_t rowid = c / (D / 4);
    const int i = (int)(rowid % p.N);
    const int bh = (int)(rowid / p.N);
    const int b = bh / p.H, h = bh - b * p.H;
    const int NR = 32 + p.w2;
    int kb_lo = (i - 31 - p.w2 + 31) / 32;                 // smallest kb with 32*kb + 31 + w2 >= i
    kb_lo = (i - 31 - p.w2) <= 0 ? 0 : kb_lo;
    const int kb_hi = i / 32;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int kb = kb_lo; kb <= kb_hi; ++kb) {
        const float4 y = *(const float4*)(dq_part + (((int64_t)bh * nkb + kb) * NR + (i - 32 * kb)) * D + col * 4);
        acc.x += y.x; acc.y += y.y; acc.z += y.z; acc.w += y.w;
    }
    float* orow = (float*)p.dq.p + p.dq.off(b, i, h);
    *(float4*)(orow + col * 4) = make_float4(acc.x * p.scale, acc.y * p.scale, acc.z * p.scale, acc.w * p.scale);
}

// =================================================== backward, K side: dK, dV =====
// nsplit > 1 (grids smaller than the chip): the workgroup takes the sp-th share of the key block's stream
// of units and writes fp32 partial sums to `part` ([dK | dV][nsplit][B*H][N][D]) for f32_kv_sum_kernel.
template <int D, bool SPLIT>
__global__ __launch_bounds__(XT) __attribute__((amdgpu_waves_per_eu(D <= 64 ? 2 : 1, D <= 64 ? 2 : 1)))
void f32_bwd_kv_kernel(Problem p, int njb, int total, int nsplit_arg, float* __restrict__ part) {
    const int nsplit = SPLIT ? nsplit_arg : 1;
    using C = F32Cfg<D>;
    extern __shared__ __attribute__((aligned(16))) float smem_f[];
    float* lse_s = smem_f + 2 * C::STAGE;        // [2][32]  LSE*log2(e) of the unit's queries
    float* dsum_s = lse_s + 2 * 32;              // [2][32]

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;
    const int pid = xcd_order(blockIdx.x, total);
    const int sp = pid % nsplit, pj = pid / nsplit;
    const int bh = pj / njb, jb = pj - bh * njb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int j0 = jb * XJ, jw = j0 + 32 * wave, j = jw + ln, jc = j < N ? j : N - 1;

    const float* qp = (const float*)p.q.p + p.q.off(b, 0, h);
    const float* k1p = (const float*)p.k1.p + p.k1.off(b, 0, h);
    const float* k2p = (const float*)p.k2.p + p.k2.off(b, 0, h);
    const float* v1p = (const float*)p.v1.p + p.v1.off(b, 0, h);
    const float* v2p = (const float*)p.v2.p + p.v2.off(b, 0, h);
    const float* dop = (const float*)p.dout.p + p.dout.off(b, 0, h);
    const float qscale = p.scale * LOG2E;

    // this wavefront's K and V rows as resident B operands (column = key j, slots d = 8g + 4hf + t)
    float kf[D / 2], vf[D / 2];
#pragma unroll
    for (int gg = 0; gg < C::DG; ++gg) {
        const float4 ka = *(const float4*)(k1p + (int64_t)jc * p.k1.sn + 8 * gg + 4 * hf);
        const float4 va = *(const float4*)(v1p + (int64_t)jc * p.v1.sn + 8 * gg + 4 * hf);
        kf[4 * gg] = ka.x; kf[4 * gg + 1] = ka.y; kf[4 * gg + 2] = ka.z; kf[4 * gg + 3] = ka.w;
        vf[4 * gg] = va.x; vf[4 * gg + 1] = va.y; vf[4 * gg + 2] = va.z; vf[4 * gg + 3] = va.w;
    }
    floatx16 dkacc[C::DT], dvacc[C::DT];
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt) dkacc[dt] = dvacc[dt] = zero16();

    const int j_last = j0 + XJ - 1 < N ? j0 + XJ - 1 : N - 1;
    const int i_max = (int)((int64_t)j_last + w1 < N - 1 ? j_last + w1 : N - 1);
    auto units_of = [&](int ib) {
        const int il = ib * BQ + BQ - 1 < N ? ib * BQ + BQ - 1 : N - 1;
        return (w2 < il ? w2 : il) + 1;
    };
    // The units (query block, delta) that see the key block, in stream order, and this workgroup's share of
    // them: from delta d_first of block ib_lo to delta d_last of block ib_hi.  The shares cut the stream
    // counted with w2 + 1 slots per block (a block near the start of the sequence has fewer units: the slots
    // beyond are skipped).
    int ib_lo = j0 / BQ, ib_hi = i_max / BQ, d_first = 0, d_last = w2;
    bool empty_share = ib_lo > ib_hi;
    if constexpr (SPLIT) {
        const int per = w2 + 1, ib0 = ib_lo;
        const int slots = (ib_hi - ib_lo + 1) * per;
        const int chunk = (slots + nsplit - 1) / nsplit;
        const int v_lo = sp * chunk, v_hi = (v_lo + chunk < slots ? v_lo + chunk : slots) - 1;
        empty_share = v_lo > v_hi;
        if (!empty_share) {
            ib_lo = ib0 + v_lo / per;
            d_first = v_lo - (ib_lo - ib0) * per;
            ib_hi = ib0 + v_hi / per;
            d_last = v_hi - (ib_hi - ib0) * per;
            if (d_first >= units_of(ib_lo)) {        // the share starts in the slots a short block does not have
                ++ib_lo;
                d_first = 0;
            }
            empty_share = !(ib_lo < ib_hi || (ib_lo == ib_hi && d_first <= d_last));
        }
    }
    // (a share of a split launch may be empty: it walks one unit without touching it and writes zeros)
    if (empty_share) {
        ib_lo = ib_hi = j0 / BQ;
        d_first = d_last = 0;
    }

    // ---- forming a unit: Q~ and dO~ tiles (32 rows), LSE and D of its queries ----
    float4 fq[C::KR], fk[C::KR], fd[C::KR], fv[C::KR];
    float f_lse = 0.f, f_dsum = 0.f;
    auto fetch_unit = [&](int ib, int delta) {
#pragma unroll
        for (int u = 0; u < C::KR; ++u) {
            const int c = tid + XT * u;
            const int row = c / (D / 4), col = c - row * (D / 4);
            int i = ib * BQ + row;
            i = i < N ? i : N - 1;
            const int k = i - delta > 0 ? i - delta : 0;
            fq[u] = *(const float4*)(qp + (int64_t)i * p.q.sn + col * 4);
            fk[u] = *(const float4*)(k2p + (int64_t)k * p.k2.sn + col * 4);
            fd[u] = *(const float4*)(dop + (int64_t)i * p.dout.sn + col * 4);
            fv[u] = *(const float4*)(v2p + (int64_t)k * p.v2.sn + col * 4);
        }
        if (tid < 32) {
            int i = ib * BQ + tid;
            i = i < N ? i : N - 1;
            f_lse = p.lse[(int64_t)bh * N + i] * LOG2E;
            f_dsum = p.dsum[(int64_t)bh * N + i];
        }
    };
    auto store_unit = [&](int buf) {
        float* Qs = smem_f + buf * C::STAGE;
        float* Ds = Qs + C::TILE;
#pragma unroll
        for (int u = 0; u < C::KR; ++u) {
            const int c = tid + XT * u;
            const int row = c / (D / 4), col = c - row * (D / 4);
            const float kb = p.k2_bias, vb = p.v2_bias;
            *(float4*)(Qs + row * C::RS + col * 4) = make_float4(fq[u].x * qscale * (fk[u].x + kb), fq[u].y * qscale * (fk[u].y + kb),
                                                                 fq[u].z * qscale * (fk[u].z + kb), fq[u].w * qscale * (fk[u].w + kb));
            *(float4*)(Ds + row * C::RS + col * 4) = make_float4(fd[u].x * (fv[u].x + vb), fd[u].y * (fv[u].y + vb),
                                                                 fd[u].z * (fv[u].z + vb), fd[u].w * (fv[u].w + vb));
        }
        if (tid < 32) {
            lse_s[buf * 32 + tid] = f_lse;
            dsum_s[buf * 32 + tid] = f_dsum;
        }
    };

    int ib = ib_lo, delta = d_first, nu = units_of(ib_lo), buf = 0;
    fetch_unit(ib, delta);
    store_unit(0);
    __syncthreads();
    while (true) {
        int nib = ib, ndelta = delta + 1;
        if (ndelta >= nu) {
            nib = ib + 1;
            ndelta = 0;
        }
        const bool more = SPLIT ? (nib < ib_hi || (nib == ib_hi && ndelta <= d_last)) : nib <= ib_hi;
        if (more) fetch_unit(nib, ndelta);

        const int i0 = ib * BQ;
        const bool touches = (i0 + BQ - 1 >= jw) && ((int64_t)i0 <= (int64_t)jw + 31 + w1) && jw < N && !empty_share;
        if (touches) {
            const float* Qs = smem_f + buf * C::STAGE;
            const float* Ds = Qs + C::TILE;
            floatx16 sacc = zero16(), dpacc = zero16();
#pragma unroll
            for (int gg = 0; gg < C::DG; ++gg) {
                const float4 qa = *(const float4*)(Qs + ln * C::RS + 8 * gg + 4 * hf);
                const float4 da = *(const float4*)(Ds + ln * C::RS + 8 * gg + 4 * hf);
                sacc = mfma_f32(qa.x, kf[4 * gg + 0], sacc);
                dpacc = mfma_f32(da.x, vf[4 * gg + 0], dpacc);
                sacc = mfma_f32(qa.y, kf[4 * gg + 1], sacc);
                dpacc = mfma_f32(da.y, vf[4 * gg + 1], dpacc);
                sacc = mfma_f32(qa.z, kf[4 * gg + 2], sacc);
                dpacc = mfma_f32(da.z, vf[4 * gg + 2], dpacc);
                sacc = mfma_f32(qa.w, kf[4 * gg + 3], sacc);
                dpacc = mfma_f32(da.w, vf[4 * gg + 3], dpacc);
            }
            // register v of this lane: query i0 + 8*(v/4) + 4*hf + v%4, key j
            const bool interior = (i0 >= jw + 31) && ((int64_t)i0 + 31 <= (int64_t)jw + w1) && (i0 + BQ - 1 < N) && (i0 >= delta);
            const int lo = j - i0 - 4 * hf;                                    // c >= lo  <=>  j <= i
            const int hi = (int)((int64_t)j + w1 - i0 < (1 << 20) ? j + w1 - i0 : (1 << 20)) - 4 * hf;   // i <= j + w1
            const int dlo = delta - i0 - 4 * hf, nhi = N - 1 - i0 - 4 * hf;
            float pv[16], dsv[16];
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const float4 ls = *(const float4*)(lse_s + buf * 32 + 8 * g4 + 4 * hf);
                const float4 dm = *(const float4*)(dsum_s + buf * 32 + 8 * g4 + 4 * hf);
                const float lsv[4] = {ls.x, ls.y, ls.z, ls.w}, dmv[4] = {dm.x, dm.y, dm.z, dm.w};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int v = 4 * g4 + t, c = 8 * g4 + t;
                    const bool valid = interior || ((j < N) && (c >= lo) && (c <= hi) && (c >= dlo) && (c <= nhi));
                    pv[v] = valid ? fast_exp2(sacc[v] - lsv[t]) : 0.f;
                    dsv[v] = pv[v] * (dpacc[v] - dmv[t]);
                }
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int rr = (8 * (v >> 2) + 4 * hf + (v & 3)) * C::RS + ln;
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt) {
                    dvacc[dt] = mfma_f32(Ds[rr + dt * 32], pv[v], dvacc[dt]);
                    dkacc[dt] = mfma_f32(Qs[rr + dt * 32], dsv[v], dkacc[dt]);
                }
            }
        }
        if (!more) break;
        store_unit(buf ^ 1);          // (the other buffer was last read one step ago, before that step's barrier)
        __syncthreads();
        if (nib != ib) nu = units_of(nib);
        ib = nib;
        delta = ndelta;
        buf ^= 1;
    }

    if (j < N) {
        float* dkp = p.dk1.p ? (float*)p.dk1.p + p.dk1.off(b, j, h) + 4 * hf : nullptr;
        float* dvp = p.dv1.p ? (float*)p.dv1.p + p.dv1.off(b, j, h) + 4 * hf : nullptr;
        if constexpr (SPLIT) {
            const int64_t BH = (int64_t)p.B * p.H;
            if (dkp) dkp = part + (((0 * (int64_t)nsplit + sp) * BH + bh) * N + j) * D + 4 * hf;
            if (dvp) dvp = part + (((1 * (int64_t)nsplit + sp) * BH + bh) * N + j) * D + 4 * hf;
        }
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                // Q~ carries scale*log2(e): dK = ln2 * sum dS * Q~
                if (dkp) *(float4*)(dkp + dt * 32 + 8 * g4) = make_float4(dkacc[dt][4 * g4] * LN2, dkacc[dt][4 * g4 + 1] * LN2,
                                                                           dkacc[dt][4 * g4 + 2] * LN2, dkacc[dt][4 * g4 + 3] * LN2);
                if (dvp) *(float4*)(dvp + dt * 32 + 8 * g4) = make_float4(dvacc[dt][4 * g4], dvacc[dt][4 * g4 + 1], dvacc[dt][4 * g4 + 2],
                                                                           dvacc[dt][4 * g4 + 3]);
            }
    }
}

// dK and dV from the partial sums of a split launch, shares added in their order
template <int D>
__global__ __launch_bounds__(256) void f32_kv_sum_kernel(Problem p, int nsplit, const float* __restrict__ part, int64_t chunks) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= chunks) return;
    const int col = (int)(c % (D / 4));
    const int64_t rowid = c / (D / 4);
    const int j = (int)(rowid % p.N);
    const int bh = (int)(rowid / p.N);
    const int b = bh / p.H, h = bh - b * p.H;
    const int64_t BH = (int64_t)p.B * p.H;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const Tensor& t = which ? p.dv1 : p.dk1;
        if (!t.p) continue;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int s = 0; s < nsplit; ++s) {
            const float4 y = *(const float4*)(part + (((which * (int64_t)nsplit + s) * BH + bh) * p.N + j) * D + col * 4);
            acc.x += y.x; acc.y += y.y; acc.z += y.z; acc.w += y.w;
        }
        *(float4*)((float*)t.p + t.off(b, j, h) + col * 4) = acc;
    }
}

// Shares a key block's query blocks are split into when the K-side grid is smaller than the chip
int f32_kv_nsplit(int B, int N, int H, int D, int w1, int w2) {
    const int64_t bh = (int64_t)B * H, base = bh * ((N + XJ - 1) / XJ);
    const int blocks = (XJ + (w1 < N ? w1 : N) + BQ - 1) / BQ + 1;
    const int64_t units = (int64_t)blocks * ((w2 < N - 1 ? w2 : N - 1) + 1);     // of a key block's stream, at most
    int ns = 1;                                                                  // shares of at least 8 units
    while (ns < 16 && base * ns * 2 <= 512 && (int64_t)ns * 2 * 8 <= units && (int64_t)2 * ns * 2 * bh * N * D * 4 <= ((int64_t)32 << 20))
        ns *= 2;
    return ns;
}
size_t f32_dq_part_bytes(int B, int N, int H, int D, int w2) {
    return ((size_t)B * H * ((N + BQ - 1) / BQ) * (size_t)(32 + w2) * D * sizeof(float) + 255) / 256 * 256;
}

// ------------------------------------------------------------------ launchers ----
template <int D>
int launch_f32_fwd(const Problem& p, hipStream_t st) {
    using C = F32Cfg<D>;
    const int nqb = (p.N + BQ - 1) / BQ;
    const int64_t total = (int64_t)nqb * p.B * p.H;
    if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    if (!allow_full_lds((const void*)f32_fwd_kernel<D>)) return SA2_ERR_LAUNCH_FAILED;
    hipLaunchKernelGGL((f32_fwd_kernel<D>), dim3((unsigned)total), dim3(XT), C::FWD_LDS, st, p, nqb, (int)total);
    return hipGetLastError() == hipSuccess ? SA2_OK : SA2_ERR_LAUNCH_FAILED;
}

template <int D>
int launch_f32_bwd(const Problem& p, hipStream_t st) {
    using C = F32Cfg<D>;
    int rc = launch_rowdot(p.out, p.dout, p.dsum, p.B, p.N, p.H, p.D, SA2_F32, st);
    if (rc != SA2_OK) return rc;
    if (p.dq.p || p.dk2.p || p.dv2.p) {
        const int nkb = (p.N + BQ - 1) / BQ;
        const int64_t total = (int64_t)nkb * p.B * p.H;
        if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
        if (p.scratch_bytes < f32_dq_part_bytes(p.B, p.N, p.H, D, p.w2)) return SA2_ERR_WORKSPACE_TOO_SMALL;
        float* part = (float*)p.scratch;
        const int segw = C::kp_segment(p.w2);
        if (!allow_full_lds((const void*)f32_bwd_kp_kernel<D, false>) || !allow_full_lds((const void*)f32_bwd_kp_kernel<D, true>))
            return SA2_ERR_LAUNCH_FAILED;
        if (segw < p.w2 + 1)
            hipLaunchKernelGGL((f32_bwd_kp_kernel<D, true>), dim3((unsigned)total), dim3(XT), C::kp_lds(segw - 1), st, p, nkb, (int)total, part, segw);
        else
            hipLaunchKernelGGL((f32_bwd_kp_kernel<D, false>), dim3((unsigned)total), dim3(XT), C::kp_lds(segw - 1), st, p, nkb, (int)total, part, segw);
        if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
        if (p.dq.p) {
            const int64_t chunks = (int64_t)p.B * p.H * p.N * (D / 4);
            hipLaunchKernelGGL((f32_dq_sum_kernel<D>), dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st, p, nkb, part, chunks);
            if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
        }
    }
    if (p.dk1.p || p.dv1.p) {
        const int njb = (p.N + XJ - 1) / XJ;
        const int nsplit = f32_kv_nsplit(p.B, p.N, p.H, D, p.w1, p.w2);
        const int64_t total = (int64_t)njb * p.B * p.H * nsplit;
        if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
        float* kv_part = nullptr;
        if (nsplit > 1) {
            if (p.scratch_bytes < f32_mfma_bwd_scratch_bytes(p.B, p.N, p.H, D, p.w1, p.w2)) return SA2_ERR_WORKSPACE_TOO_SMALL;
            kv_part = (float*)((char*)p.scratch + f32_dq_part_bytes(p.B, p.N, p.H, D, p.w2));
        }
        if (!allow_full_lds((const void*)f32_bwd_kv_kernel<D, false>) || !allow_full_lds((const void*)f32_bwd_kv_kernel<D, true>))
            return SA2_ERR_LAUNCH_FAILED;
        if (nsplit > 1)
            hipLaunchKernelGGL((f32_bwd_kv_kernel<D, true>), dim3((unsigned)total), dim3(XT), C::KV_LDS, st, p, njb, (int)total, nsplit, kv_part);
        else
            hipLaunchKernelGGL((f32_bwd_kv_kernel<D, false>), dim3((unsigned)total), dim3(XT), C::KV_LDS, st, p, njb, (int)total, 1, kv_part);
        if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
        if (nsplit > 1) {
            const int64_t chunks = (int64_t)p.B * p.H * p.N * (D / 4);
            hipLaunchKernelGGL((f32_kv_sum_kernel<D>), dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st, p, nsplit, kv_part, chunks);
            if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
        }
    }
    return SA2_OK;
}

bool rows16(const Tensor& t, int B, int N, int H) {
    if (!t.p) return true;
    if ((uintptr_t)t.p & 15u) return false;
    return !((B > 1 && (t.sb & 3)) || (N > 1 && (t.sn & 3)) || (H > 1 && (t.sh & 3)));
}

}  // namespace

bool f32_mfma_supported(int D, int dtype) { return dtype == SA2_F32 && (D == 32 || D == 64 || D == 128); }

bool f32_mfma_bwd_supported(int D, int w2, int dtype) {
    (void)w2;                // any K' window: wide ones are walked in segments
    return f32_mfma_supported(D, dtype);
}

bool f32_mfma_layout_ok(const Problem& p, bool backward) {
    const Tensor* fwd[] = {&p.q, &p.k1, &p.k2, &p.v1, &p.v2, &p.out};
    for (const Tensor* t : fwd)
        if (!rows16(*t, p.B, p.N, p.H)) return false;
    if (backward) {
        const Tensor* bwd[] = {&p.dout, &p.dq, &p.dk1, &p.dk2, &p.dv1, &p.dv2};
        for (const Tensor* t : bwd)
            if (!rows16(*t, p.B, p.N, p.H)) return false;
    }
    return true;
}

size_t f32_mfma_bwd_scratch_bytes(int B, int N, int H, int D, int w1, int w2) {
    const int ns = f32_kv_nsplit(B, N, H, D, w1, w2);
    return f32_dq_part_bytes(B, N, H, D, w2) + (ns > 1 ? (size_t)2 * ns * B * H * (size_t)N * D * sizeof(float) : 0);
}

int launch_f32_mfma_fwd(const Problem& p, hipStream_t st) {
    return p.D == 128 ? launch_f32_fwd<128>(p, st) : p.D == 64 ? launch_f32_fwd<64>(p, st) : launch_f32_fwd<32>(p, st);
}

int launch_f32_mfma_bwd(const Problem& p, hipStream_t st) {
    return p.D == 128 ? launch_f32_bwd<128>(p, st) : p.D == 64 ? launch_f32_bwd<64>(p, st) : launch_f32_bwd<32>(p, st);
}

}  // namespace sa2
