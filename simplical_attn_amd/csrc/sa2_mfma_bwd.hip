// MFMA backward for gfx950: dispatch to the on-chip kernels (sa2_mfma_bwd_kp.hip for dQ, dK',
// dV'; sa2_mfma_bwd_kv.hip for dK, dV; bf16 or fp16, head_dim 32, 64 or 128), and the workspace
// kernels (bf16 or fp16, head_dim 64 or 128) that serve shapes whose K' window is too wide for them.
//
// Same expanded-row view as the forward: rows r = (i, delta), Q~[r] = q[i] *
// k2~[i-delta] * scale*log2(e) and dO~[r] = dO[i] * v2~[i-delta], both in the element type.  With
// P = exp2(S - LSE*log2e) recomputed from the saved log-sum-exp and
// dS = P * (dO~.v1 - D_i), the workspace kernels are:
//
//   row kernel      owns 32 queries x one delta per wavefront, sweeps the K window:
//                   G[r,:] = scale * sum_j dS[r,j] k1[j,:]   and   R[r,:] = sum_j P[r,j] v1[j,:]
//                   are written once per expanded row to a 16-bit workspace;
//   finalize        dQ[i]  = sum_delta G[(i,delta)] * k2~[i-delta]
//                   dK'[k] = sum_delta G[(k+delta,delta)] * q[k+delta]
//                   dV'[k] = sum_delta R[(k+delta,delta)] * dO[k+delta]
//   column kernel   owns 128 K rows per workgroup (32 per wavefront, K/V operands
//                   resident in registers), streams every expanded row that can see
//                   them and accumulates dK = ln2 * sum_r dS[r,j] Q~[r], dV = sum_r P[r,j] dO~[r].
//
// Every output element has one writer and a fixed summation order: no atomics,
// bitwise reproducible.
#include "sa2_mfma_common.h"

namespace sa2 {
namespace {

// ============================================================ row kernel =====
template <int D>
struct RowCfg {
    static constexpr int DK = D / 16;
    static constexpr int DT = D / 32;
    static constexpr int KS = D + 8;           // row-major tile row stride (elements)
    static constexpr int VS = TJ + 8;          // transposed tile row stride (elements)
    static constexpr int RM_ELEMS = TJ * KS;
    static constexpr int TR_ELEMS = D * VS;
    static constexpr int STAGE = 2 * RM_ELEMS + 2 * TR_ELEMS;   // K, V row-major; K^T, V^T
    static constexpr int KR = TJ * D / 8 / NTHREADS;
    static constexpr int NDP = D / 2;
    static constexpr int VPASS = NDP / 32;
    static constexpr size_t LDS_BYTES = (size_t)2 * STAGE * 2;
};

// 4 rows x 2 columns of a [row][col] 16-bit tile (one dword per row) -> two 8-byte
// groups of the transposed tile.
__device__ __forceinline__ void transpose4x2(const uint32_t* x, uint2& lo, uint2& hi) {
    lo.x = (x[0] & 0xffffu) | (x[1] << 16);
    lo.y = (x[2] & 0xffffu) | (x[3] << 16);
    hi.x = (x[0] >> 16) | (x[1] & 0xffff0000u);
    hi.y = (x[2] >> 16) | (x[3] & 0xffff0000u);
}

template <class E, int D>
__global__ __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(1, 1)))
void mfma_bwd_row_kernel(Problem p, int nqb, int total, uint16_t* __restrict__ gws, uint16_t* __restrict__ rws) {
    typedef typename E::scalar EL;
    typedef typename E::x8 X8;
    using C = RowCfg<D>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t* smem = (uint16_t*)smem_raw;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;

    int pid = blockIdx.x;
    if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
    const int bh = pid / nqb, qb = pid - bh * nqb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int i0 = qb * BQ;
    const int i = i0 + ln;
    const int ic = i < N ? i : N - 1;
    const int i_last = (i0 + BQ - 1 < N ? i0 + BQ - 1 : N - 1);

    const uint16_t* qp = (const uint16_t*)p.q.p + p.q.off(b, 0, h);
    const uint16_t* k1p = (const uint16_t*)p.k1.p + p.k1.off(b, 0, h);
    const uint16_t* k2p = (const uint16_t*)p.k2.p + p.k2.off(b, 0, h);
    const uint16_t* v1p = (const uint16_t*)p.v1.p + p.v1.off(b, 0, h);
    const uint16_t* v2p = (const uint16_t*)p.v2.p + p.v2.off(b, 0, h);
    const uint16_t* dop = (const uint16_t*)p.dout.p + p.dout.off(b, 0, h);

    const int jt_lo = (i0 - w1 > 0 ? i0 - w1 : 0) / TJ;
    const int jt_hi = i_last / TJ;
    const int nt = jt_hi - jt_lo + 1;
    const int n_units = (w2 < i_last ? w2 : i_last) + 1;
    const int nrounds = (n_units + 3) >> 2;
    const int total_steps = nrounds * nt;
    const int nd = w2 + 1;                       // delta slots per query in the workspace

    // ---- staging: K and V tiles, row-major and transposed ---------------------
    uint4 kreg[C::KR], vreg[C::KR];
    uint32_t ktr[C::VPASS * 4], vtr[C::VPASS * 4];
    const int v_dp = tid % C::NDP, v_g0 = tid / C::NDP;
    auto load_tile = [&](int jt) {
        const int j0 = jt * TJ;
#pragma unroll
        for (int u = 0; u < C::KR; ++u) {
            const int c = tid + NTHREADS * u;
            const int row = c / (D / 8), col = c - row * (D / 8);
            int j = j0 + row;
            j = j < N ? j : N - 1;
            kreg[u] = *(const uint4*)(k1p + (int64_t)j * p.k1.sn + col * 8);
            vreg[u] = *(const uint4*)(v1p + (int64_t)j * p.v1.sn + col * 8);
        }
#pragma unroll
        for (int ps = 0; ps < C::VPASS; ++ps) {
            const int grp = v_g0 + ps * (NTHREADS / C::NDP);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                int j = j0 + grp * 4 + r;
                j = j < N ? j : N - 1;
                ktr[ps * 4 + r] = *(const uint32_t*)(k1p + (int64_t)j * p.k1.sn + 2 * v_dp);
                vtr[ps * 4 + r] = *(const uint32_t*)(v1p + (int64_t)j * p.v1.sn + 2 * v_dp);
            }
        }
    };
    auto store_tile = [&](int buf) {
        uint16_t* Kr = smem + buf * C::STAGE;
        uint16_t* Vr = Kr + C::RM_ELEMS;
        uint16_t* Kt = Vr + C::RM_ELEMS;
        uint16_t* Vt = Kt + C::TR_ELEMS;
#pragma unroll
        for (int u = 0; u < C::KR; ++u) {
            const int c = tid + NTHREADS * u;
            const int row = c / (D / 8), col = c - row * (D / 8);
            *(uint4*)(Kr + row * C::KS + col * 8) = kreg[u];
            *(uint4*)(Vr + row * C::KS + col * 8) = vreg[u];
        }
#pragma unroll
        for (int ps = 0; ps < C::VPASS; ++ps) {
            const int grp = v_g0 + ps * (NTHREADS / C::NDP);
            const int g = grp >> 1, hh = grp & 1;
            const int pos = (g >> 1) * 16 + hh * 8 + (g & 1) * 4;
            uint2 lo, hi;
            transpose4x2(ktr + ps * 4, lo, hi);
            *(uint2*)(Kt + (2 * v_dp) * C::VS + pos) = lo;
            *(uint2*)(Kt + (2 * v_dp + 1) * C::VS + pos) = hi;
            transpose4x2(vtr + ps * 4, lo, hi);
            *(uint2*)(Vt + (2 * v_dp) * C::VS + pos) = lo;
            *(uint2*)(Vt + (2 * v_dp + 1) * C::VS + pos) = hi;
        }
    };

    const float qscale = p.scale * LOG2E;
    const float lse2 = p.lse[(int64_t)bh * N + ic] * LOG2E;
    const float dsum = p.dsum[(int64_t)bh * N + ic];

    load_tile(jt_lo);
    store_tile(0);
    if (total_steps > 1) load_tile(jt_lo + (1 % nt));
    __syncthreads();

    int g = 0;
    for (int round = 0; round < nrounds; ++round) {
        const int delta = round * 4 + wave;
        if (delta >= n_units) {
            for (int s = 0; s < nt; ++s, ++g) {
                if (g + 1 < total_steps) store_tile((g + 1) & 1);
                if (g + 2 < total_steps) load_tile(jt_lo + (g + 2) % nt);
                __syncthreads();
            }
            continue;
        }

        X8 qf[C::DK], dof[C::DK];
        floatx16 gacc[C::DT], racc[C::DT];
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int v = 0; v < 16; ++v) gacc[dt][v] = racc[dt][v] = 0.f;
        int k = ic - delta;
        k = k > 0 ? k : 0;
#pragma unroll
        for (int kk = 0; kk < C::DK; ++kk) {
            const int col = kk * 16 + hf * 8;
            const uint4 qa = *(const uint4*)(qp + (int64_t)ic * p.q.sn + col);
            const uint4 kb = *(const uint4*)(k2p + (int64_t)k * p.k2.sn + col);
            const uint4 da = *(const uint4*)(dop + (int64_t)ic * p.dout.sn + col);
            const uint4 vb = *(const uint4*)(v2p + (int64_t)k * p.v2.sn + col);
            const uint32_t qw[4] = {qa.x, qa.y, qa.z, qa.w}, kw[4] = {kb.x, kb.y, kb.z, kb.w};
            const uint32_t dw[4] = {da.x, da.y, da.z, da.w}, vw[4] = {vb.x, vb.y, vb.z, vb.w};
            X8 r, d;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                r[2 * t] = (EL)(E::lo(qw[t]) * (E::lo(kw[t]) + p.k2_bias) * qscale);
                r[2 * t + 1] = (EL)(E::hi(qw[t]) * (E::hi(kw[t]) + p.k2_bias) * qscale);
                d[2 * t] = (EL)(E::lo(dw[t]) * (E::lo(vw[t]) + p.v2_bias));
                d[2 * t + 1] = (EL)(E::hi(dw[t]) * (E::hi(vw[t]) + p.v2_bias));
            }
            qf[kk] = r;
            dof[kk] = d;
        }
        const bool rows_full = i0 >= delta && i0 + BQ - 1 < N;
        const bool row_ok = i < N && i >= delta;

        for (int s = 0; s < nt; ++s, ++g) {
            const int j0 = (jt_lo + s) * TJ;
            const uint16_t* Kr = smem + (g & 1) * C::STAGE;
            const uint16_t* Vr = Kr + C::RM_ELEMS;
            const uint16_t* Kt = Vr + C::RM_ELEMS;
            const uint16_t* Vt = Kt + C::TR_ELEMS;
            floatx16 sacc, dpacc;
#pragma unroll
            for (int v = 0; v < 16; ++v) sacc[v] = dpacc[v] = 0.f;
#pragma unroll
            for (int kk = 0; kk < C::DK; ++kk) {
                const X8 ka = *(const X8*)(Kr + ln * C::KS + kk * 16 + hf * 8);
                const X8 va = *(const X8*)(Vr + ln * C::KS + kk * 16 + hf * 8);
                sacc = E::mfma(ka, qf[kk], sacc, 0, 0, 0);
                dpacc = E::mfma(va, dof[kk], dpacc, 0, 0, 0);
            }
            float pv[16], dsv[16];
#pragma unroll
            for (int v = 0; v < 16; ++v) pv[v] = sacc[v] - lse2;
            const bool interior = (j0 + TJ - 1 <= i0) && (j0 >= i0 + BQ - 1 - w1) && rows_full;
            if (__builtin_expect(!interior, 0)) {
                const int hi = i - j0 - 4 * hf, lo = hi - w1;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int c = 8 * (v >> 2) + (v & 3);
                    pv[v] = (row_ok && c <= hi && c >= lo) ? pv[v] : -INFINITY;
                }
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                pv[v] = fast_exp2(pv[v]);
                dsv[v] = pv[v] * (dpacc[v] - dsum);
            }
            X8 pb[2], dsb[2];
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    pb[ks][t] = (EL)pv[ks * 8 + t];
                    dsb[ks][t] = (EL)dsv[ks * 8 + t];
                }
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const X8 kt = *(const X8*)(Kt + (dt * 32 + ln) * C::VS + ks * 16 + hf * 8);
                    const X8 vt = *(const X8*)(Vt + (dt * 32 + ln) * C::VS + ks * 16 + hf * 8);
                    gacc[dt] = E::mfma(kt, dsb[ks], gacc[dt], 0, 0, 0);
                    racc[dt] = E::mfma(vt, pb[ks], racc[dt], 0, 0, 0);
                }

            if (g + 1 < total_steps) store_tile((g + 1) & 1);
            if (g + 2 < total_steps) load_tile(jt_lo + (g + 2) % nt);
            __syncthreads();
        }

        // ---- one expanded row per lane pair: G and R to the workspace ----------
        if (row_ok) {
            const int64_t base = (((int64_t)bh * N + i) * nd + delta) * D + 4 * hf;
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    union { EL h[4]; uint2 u; } a, c;
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        a.h[t] = (EL)(gacc[dt][4 * g4 + t] * p.scale);
                        c.h[t] = (EL)racc[dt][4 * g4 + t];
                    }
                    *(uint2*)(gws + base + dt * 32 + 8 * g4) = a.u;
                    *(uint2*)(rws + base + dt * 32 + 8 * g4) = c.u;
                }
        }
    }
}

// =============================================================== finalize ====
// One wavefront per (batch, head, position n): lanes own column pairs.
template <class E, int D>
__global__ __launch_bounds__(256) void mfma_bwd_finalize_kernel(Problem p, const uint16_t* __restrict__ gws,
                                                               const uint16_t* __restrict__ rws, int64_t rows) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    if (lane >= D / 2) return;
    const int N = p.N, w2 = p.w2, nd = w2 + 1;
    const int n = (int)(row % N);
    const int bh = (int)(row / N);
    const int b = bh / p.H, h = bh - b * p.H;
    const int c2 = 2 * lane;
    const uint16_t* qp = (const uint16_t*)p.q.p + p.q.off(b, 0, h) + c2;
    const uint16_t* k2p = (const uint16_t*)p.k2.p + p.k2.off(b, 0, h) + c2;
    const uint16_t* dop = (const uint16_t*)p.dout.p + p.dout.off(b, 0, h) + c2;
    const int64_t wrow = (int64_t)bh * N;

    if (p.dq.p) {
        float a0 = 0.f, a1 = 0.f;
        const int dmax = n < w2 ? n : w2;
        for (int dl = 0; dl <= dmax; ++dl) {
            const uint32_t gx = *(const uint32_t*)(gws + ((wrow + n) * nd + dl) * D + c2);
            const uint32_t kx = *(const uint32_t*)(k2p + (int64_t)(n - dl) * p.k2.sn);
            a0 = fmaf(E::lo(gx), E::lo(kx) + p.k2_bias, a0);
            a1 = fmaf(E::hi(gx), E::hi(kx) + p.k2_bias, a1);
        }
        const uint32_t o = E::pack(a0, a1);
        *(uint32_t*)((uint16_t*)p.dq.p + p.dq.off(b, n, h) + c2) = o;
    }
    if (p.dk2.p || p.dv2.p) {
        float k0 = 0.f, k1 = 0.f, v0 = 0.f, v1 = 0.f;
        const int dmax = (N - 1 - n) < w2 ? (N - 1 - n) : w2;
        for (int dl = 0; dl <= dmax; ++dl) {
            const int i = n + dl;
            const int64_t wo = ((wrow + i) * nd + dl) * D + c2;
            const uint32_t gx = *(const uint32_t*)(gws + wo);
            const uint32_t rx = *(const uint32_t*)(rws + wo);
            const uint32_t qx = *(const uint32_t*)(qp + (int64_t)i * p.q.sn);
            const uint32_t dx = *(const uint32_t*)(dop + (int64_t)i * p.dout.sn);
            k0 = fmaf(E::lo(gx), E::lo(qx), k0);
            k1 = fmaf(E::hi(gx), E::hi(qx), k1);
            v0 = fmaf(E::lo(rx), E::lo(dx), v0);
            v1 = fmaf(E::hi(rx), E::hi(dx), v1);
        }
        if (p.dk2.p)
            *(uint32_t*)((uint16_t*)p.dk2.p + p.dk2.off(b, n, h) + c2) =
                E::pack(k0, k1);
        if (p.dv2.p)
            *(uint32_t*)((uint16_t*)p.dv2.p + p.dv2.off(b, n, h) + c2) =
                E::pack(v0, v1);
    }
}

// ========================================================== column kernel ====
constexpr int CJ = 128;      // K rows per workgroup (32 per wavefront)

template <int D>
struct ColCfg {
    static constexpr int DK = D / 16;
    static constexpr int DT = D / 32;
    static constexpr int KS = D + 8;           // row-major unit tile row stride (elements)
    static constexpr int VS = BQ + 8;          // transposed unit tile row stride (elements)
    static constexpr int RM_ELEMS = BQ * KS;
    static constexpr int TR_ELEMS = D * VS;
    static constexpr int UNIT = 2 * RM_ELEMS + 2 * TR_ELEMS;    // Q~, dO~ row-major; Q~^T, dO~^T
    static constexpr int RAW_Q = BQ * D;                        // q and dO rows of the query block
    static constexpr int RAW_K = 2 * BQ * D;                    // 64 rows of k2 / v2 per delta chunk
    static constexpr int RAW = 2 * RAW_Q + 2 * RAW_K;
    static constexpr int NCP = D / 2;                           // column pairs
    static constexpr int COMBOS = 8 * NCP / NTHREADS;           // (4-row group, column pair) items per thread
    static constexpr size_t LDS_BYTES = (size_t)(2 * UNIT + RAW) * 2 + 2 * BQ * sizeof(float);
};

template <class E, int D>
__global__ __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(1, 1)))
void mfma_bwd_col_kernel(Problem p, int njb, int total) {
    typedef typename E::scalar EL;
    typedef typename E::x8 X8;
    using C = ColCfg<D>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t* units = (uint16_t*)smem_raw;                 // two formed units
    uint16_t* q_s = units + 2 * C::UNIT;
    uint16_t* do_s = q_s + C::RAW_Q;
    uint16_t* k2_s = do_s + C::RAW_Q;
    uint16_t* v2_s = k2_s + C::RAW_K;
    float* lse_s = (float*)(v2_s + C::RAW_K);
    float* dsum_s = lse_s + BQ;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;

    int pid = blockIdx.x;
    if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
    const int bh = pid / njb, jb = pid - bh * njb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int j0 = jb * CJ;
    const int jw = j0 + 32 * wave;               // this wavefront's K rows: jw .. jw+31
    const int j = jw + ln;
    const int jc = j < N ? j : N - 1;

    const uint16_t* qp = (const uint16_t*)p.q.p + p.q.off(b, 0, h);
    const uint16_t* k1p = (const uint16_t*)p.k1.p + p.k1.off(b, 0, h);
    const uint16_t* k2p = (const uint16_t*)p.k2.p + p.k2.off(b, 0, h);
    const uint16_t* v1p = (const uint16_t*)p.v1.p + p.v1.off(b, 0, h);
    const uint16_t* v2p = (const uint16_t*)p.v2.p + p.v2.off(b, 0, h);
    const uint16_t* dop = (const uint16_t*)p.dout.p + p.dout.off(b, 0, h);

    // K and V rows of this wavefront as resident MFMA B operands (column = K row)
    X8 kfr[C::DK], vfr[C::DK];
#pragma unroll
    for (int kk = 0; kk < C::DK; ++kk) {
        kfr[kk] = *(const X8*)(k1p + (int64_t)jc * p.k1.sn + kk * 16 + hf * 8);
        vfr[kk] = *(const X8*)(v1p + (int64_t)jc * p.v1.sn + kk * 16 + hf * 8);
    }
    floatx16 dkacc[C::DT], dvacc[C::DT];
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) dkacc[dt][v] = dvacc[dt][v] = 0.f;

    const float qscale = p.scale * LOG2E;
    const int j_last = (j0 + CJ - 1 < N ? j0 + CJ - 1 : N - 1);
    const int i_max = (int)((int64_t)j_last + w1 < N - 1 ? j_last + w1 : N - 1);
    const int ib_lo = j0 / BQ, ib_hi = i_max / BQ;

    for (int ib = ib_lo; ib <= ib_hi; ++ib) {
        const int i0 = ib * BQ;
        const int i_last = (i0 + BQ - 1 < N ? i0 + BQ - 1 : N - 1);
        const int n_units = (w2 < i_last ? w2 : i_last) + 1;
        // does this wavefront's K tile see any query of the block?
        const bool touches = (i0 + BQ - 1 >= jw) && ((int64_t)i0 <= (int64_t)jw + 31 + w1) && jw < N;
        float lse2r[16], dsumr[16];

        for (int dc = 0; dc < n_units; dc += BQ) {
            const int ndl = (n_units - dc < BQ ? n_units - dc : BQ);
            const int kbase = i0 - dc - BQ;         // k2_s / v2_s row 0
            __syncthreads();
            // ---- raw rows: q, dO of the block (once) and 64 rows of k2, v2 ------
            if (dc == 0) {
#pragma unroll
                for (int u = 0; u < BQ * D / 8 / NTHREADS; ++u) {
                    const int c = tid + NTHREADS * u;
                    const int row = c / (D / 8), col = c - row * (D / 8);
                    int i = i0 + row;
                    i = i < N ? i : N - 1;
                    *(uint4*)(q_s + row * D + col * 8) = *(const uint4*)(qp + (int64_t)i * p.q.sn + col * 8);
                    *(uint4*)(do_s + row * D + col * 8) = *(const uint4*)(dop + (int64_t)i * p.dout.sn + col * 8);
                }
                if (tid < BQ) {
                    int i = i0 + tid;
                    i = i < N ? i : N - 1;
                    lse_s[tid] = p.lse[(int64_t)bh * N + i] * LOG2E;
                    dsum_s[tid] = p.dsum[(int64_t)bh * N + i];
                }
            }
#pragma unroll
            for (int u = 0; u < 2 * BQ * D / 8 / NTHREADS; ++u) {
                const int c = tid + NTHREADS * u;
                const int row = c / (D / 8), col = c - row * (D / 8);
                int k = kbase + row;
                k = k < 0 ? 0 : (k < N ? k : N - 1);
                *(uint4*)(k2_s + row * D + col * 8) = *(const uint4*)(k2p + (int64_t)k * p.k2.sn + col * 8);
                *(uint4*)(v2_s + row * D + col * 8) = *(const uint4*)(v2p + (int64_t)k * p.v2.sn + col * 8);
            }
            __syncthreads();
            if (dc == 0) {
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const float4 a = *(const float4*)(lse_s + 8 * g4 + 4 * hf);
                    const float4 c = *(const float4*)(dsum_s + 8 * g4 + 4 * hf);
                    lse2r[4 * g4] = a.x; lse2r[4 * g4 + 1] = a.y; lse2r[4 * g4 + 2] = a.z; lse2r[4 * g4 + 3] = a.w;
                    dsumr[4 * g4] = c.x; dsumr[4 * g4 + 1] = c.y; dsumr[4 * g4 + 2] = c.z; dsumr[4 * g4 + 3] = c.w;
                }
            }

            // Form the expanded rows of one delta in all four layouts.
            auto form = [&](int delta, int buf) {
                uint16_t* Qr = units + buf * C::UNIT;
                uint16_t* Dr = Qr + C::RM_ELEMS;
                uint16_t* Qt = Dr + C::RM_ELEMS;
                uint16_t* Dt = Qt + C::TR_ELEMS;
                const int cp = tid % C::NCP;
#pragma unroll
                for (int cb = 0; cb < C::COMBOS; ++cb) {
                    const int rg = tid / C::NCP + cb * (NTHREADS / C::NCP);      // rows 4rg .. 4rg+3
                    uint32_t qx[4], dx[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int r = 4 * rg + t;
                        const int kr = r - delta + dc + BQ;                      // (i0 + r - delta) - kbase
                        const uint32_t qa = *(const uint32_t*)(q_s + r * D + 2 * cp);
                        const uint32_t ka = *(const uint32_t*)(k2_s + kr * D + 2 * cp);
                        const uint32_t da = *(const uint32_t*)(do_s + r * D + 2 * cp);
                        const uint32_t va = *(const uint32_t*)(v2_s + kr * D + 2 * cp);
                        const float q0 = E::lo(qa) * (E::lo(ka) + p.k2_bias) * qscale;
                        const float q1 = E::hi(qa) * (E::hi(ka) + p.k2_bias) * qscale;
                        const float d0 = E::lo(da) * (E::lo(va) + p.v2_bias);
                        const float d1 = E::hi(da) * (E::hi(va) + p.v2_bias);
                        union { EL h[2]; uint32_t u; } qq, dd;
                        qq.h[0] = (EL)q0; qq.h[1] = (EL)q1;
                        dd.h[0] = (EL)d0; dd.h[1] = (EL)d1;
                        qx[t] = qq.u;
                        dx[t] = dd.u;
                        *(uint32_t*)(Qr + r * C::KS + 2 * cp) = qq.u;
                        *(uint32_t*)(Dr + r * C::KS + 2 * cp) = dd.u;
                    }
                    // row r = 8g + 4hh + t sits at position (g/2)*16 + hh*8 + (g%2)*4 + t
                    const int g = rg >> 1, hh = rg & 1;
                    const int pos = (g >> 1) * 16 + hh * 8 + (g & 1) * 4;
                    uint2 lo, hi;
                    transpose4x2(qx, lo, hi);
                    *(uint2*)(Qt + (2 * cp) * C::VS + pos) = lo;
                    *(uint2*)(Qt + (2 * cp + 1) * C::VS + pos) = hi;
                    transpose4x2(dx, lo, hi);
                    *(uint2*)(Dt + (2 * cp) * C::VS + pos) = lo;
                    *(uint2*)(Dt + (2 * cp + 1) * C::VS + pos) = hi;
                }
            };

            form(dc, 0);
            __syncthreads();
            for (int x = 0; x < ndl; ++x) {
                const int delta = dc + x;
                if (x + 1 < ndl) form(delta + 1, (x + 1) & 1);
                if (touches) {
                    const uint16_t* Qr = units + (x & 1) * C::UNIT;
                    const uint16_t* Dr = Qr + C::RM_ELEMS;
                    const uint16_t* Qt = Dr + C::RM_ELEMS;
                    const uint16_t* Dt = Qt + C::TR_ELEMS;
                    // S[r, j] and dP[r, j]: rows = expanded rows, columns = this wavefront's K rows
                    floatx16 sacc, dpacc;
#pragma unroll
                    for (int v = 0; v < 16; ++v) sacc[v] = dpacc[v] = 0.f;
#pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) {
                        const X8 qa = *(const X8*)(Qr + ln * C::KS + kk * 16 + hf * 8);
                        const X8 da = *(const X8*)(Dr + ln * C::KS + kk * 16 + hf * 8);
                        sacc = E::mfma(qa, kfr[kk], sacc, 0, 0, 0);
                        dpacc = E::mfma(da, vfr[kk], dpacc, 0, 0, 0);
                    }
                    float pv[16], dsv[16];
#pragma unroll
                    for (int v = 0; v < 16; ++v) pv[v] = sacc[v] - lse2r[v];
                    const bool interior = (i0 >= jw + 31) && ((int64_t)i0 + 31 <= (int64_t)jw + w1) &&
                                          (i0 + BQ - 1 < N) && (i0 >= delta);
                    if (__builtin_expect(!interior, 0)) {
                        // element v of this lane is query i0 + 8*(v/4) + 4*hf + v%4, column j
                        const int lo = j - i0 - 4 * hf;            // need c >= lo
                        const int hi = (int)((int64_t)j + w1 - i0 < 1 << 20 ? j + w1 - i0 : 1 << 20) - 4 * hf;
                        const int dlo = delta - i0 - 4 * hf, nhi = N - 1 - i0 - 4 * hf;
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int c = 8 * (v >> 2) + (v & 3);
                            pv[v] = (j < N && c >= lo && c <= hi && c >= dlo && c <= nhi) ? pv[v] : -INFINITY;
                        }
                    }
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        pv[v] = fast_exp2(pv[v]);
                        dsv[v] = pv[v] * (dpacc[v] - dsumr[v]);
                    }
                    X8 pb[2], dsb[2];
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                        for (int t = 0; t < 8; ++t) {
                            pb[ks][t] = (EL)pv[ks * 8 + t];
                            dsb[ks][t] = (EL)dsv[ks * 8 + t];
                        }
                    // dV^T[d, j] += dO~^T[d, r] P[r, j];  dK^T[d, j] += Q~^T[d, r] dS[r, j]
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks) {
                            const X8 dta = *(const X8*)(Dt + (dt * 32 + ln) * C::VS + ks * 16 + hf * 8);
                            const X8 qta = *(const X8*)(Qt + (dt * 32 + ln) * C::VS + ks * 16 + hf * 8);
                            dvacc[dt] = E::mfma(dta, pb[ks], dvacc[dt], 0, 0, 0);
                            dkacc[dt] = E::mfma(qta, dsb[ks], dkacc[dt], 0, 0, 0);
                        }
                }
                __syncthreads();
            }
        }
    }

    if (j < N) {
        uint16_t* dkp = p.dk1.p ? (uint16_t*)p.dk1.p + p.dk1.off(b, j, h) + 4 * hf : nullptr;
        uint16_t* dvp = p.dv1.p ? (uint16_t*)p.dv1.p + p.dv1.off(b, j, h) + 4 * hf : nullptr;
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                union { EL h[4]; uint2 u; } a, c;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    a.h[t] = (EL)(dkacc[dt][4 * g4 + t] * LN2);     // Q~ carries scale*log2(e)
                    c.h[t] = (EL)dvacc[dt][4 * g4 + t];
                }
                if (dkp) *(uint2*)(dkp + dt * 32 + 8 * g4) = a.u;
                if (dvp) *(uint2*)(dvp + dt * 32 + 8 * g4) = c.u;
            }
    }
}

template <class E, int D>
int launch_col_part(const Problem& p, hipStream_t st) {
    using C = ColCfg<D>;
    const int njb = (p.N + CJ - 1) / CJ;
    const int64_t total = (int64_t)njb * p.B * p.H;
    if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    if (!allow_full_lds((const void*)mfma_bwd_col_kernel<E, D>)) return SA2_ERR_LAUNCH_FAILED;
    hipLaunchKernelGGL((mfma_bwd_col_kernel<E, D>), dim3((unsigned)total), dim3(NTHREADS), C::LDS_BYTES, st, p, njb,
                       (int)total);
    return hipGetLastError() == hipSuccess ? SA2_OK : SA2_ERR_LAUNCH_FAILED;
}

size_t expanded_ws_bytes(int B, int N, int H, int D, int w2) {
    return (size_t)B * H * N * (size_t)(w2 + 1) * D * sizeof(uint16_t);
}

template <class E, int D>
int launch_row_part(const Problem& p, hipStream_t st) {
    using C = RowCfg<D>;
    const int nqb = (p.N + BQ - 1) / BQ;
    const int64_t total = (int64_t)nqb * p.B * p.H;
    if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    const size_t one = (expanded_ws_bytes(p.B, p.N, p.H, D, p.w2) + 255) / 256 * 256;
    if (p.scratch_bytes < 2 * one) return SA2_ERR_WORKSPACE_TOO_SMALL;
    uint16_t* gws = (uint16_t*)p.scratch;
    uint16_t* rws = (uint16_t*)((char*)p.scratch + one);
    if (!allow_full_lds((const void*)mfma_bwd_row_kernel<E, D>)) return SA2_ERR_LAUNCH_FAILED;
    hipLaunchKernelGGL((mfma_bwd_row_kernel<E, D>), dim3((unsigned)total), dim3(NTHREADS), C::LDS_BYTES, st, p, nqb,
                       (int)total, gws, rws);
    if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
    const int64_t rows = (int64_t)p.B * p.H * p.N;
    hipLaunchKernelGGL((mfma_bwd_finalize_kernel<E, D>), dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, st, p, gws, rws,
                       rows);
    return hipGetLastError() == hipSuccess ? SA2_OK : SA2_ERR_LAUNCH_FAILED;
}

}  // namespace

bool mfma_bwd_supported(int B, int N, int H, int D, int w1, int w2, int dtype) {
    if (!mfma_supported(B, N, H, D, w1, w2, dtype)) return false;
    // the workspace kernels for wide K' windows exist for D = 64 and 128
    return D != 32 || (kp_fits(D, w2) && kv_fits(D, w2));
}

// Workspace of the K'-side kernels (dQ partials, or the expanded-row arrays of the workspace kernels),
// rounded up so that what follows it stays 256-byte aligned
size_t kp_side_scratch_bytes(int B, int N, int H, int D, int w2) {
    const size_t one = (expanded_ws_bytes(B, N, H, D, w2) + 255) / 256 * 256;
    return kp_fits(D, w2) ? (kp_scratch_bytes(B, N, H, D, w2) + 255) / 256 * 256 : 2 * one;
}

size_t mfma_bwd_scratch_bytes(int B, int N, int H, int D, int w1, int w2) {
    return kp_side_scratch_bytes(B, N, H, D, w2) + (kv_fits(D, w2) ? kv_split_scratch_bytes(B, N, H, D, w1) : 0);
}

int launch_mfma_bwd(const Problem& p, int dtype, hipStream_t st) {
    int rc = launch_rowdot(p.out, p.dout, p.dsum, p.B, p.N, p.H, p.D, dtype, st);
    if (rc != SA2_OK) return rc;
    if (p.dq.p || p.dk2.p || p.dv2.p) {
        if (kp_fits(p.D, p.w2)) rc = launch_mfma_bwd_kp(p, dtype, st);
        else if (dtype == SA2_F16) rc = p.D == 128 ? launch_row_part<ElemF16, 128>(p, st) : launch_row_part<ElemF16, 64>(p, st);
        else rc = p.D == 128 ? launch_row_part<ElemBF16, 128>(p, st) : launch_row_part<ElemBF16, 64>(p, st);
        if (rc != SA2_OK) return rc;
    }
    if (p.dk1.p || p.dv1.p) {
        if (kv_fits(p.D, p.w2)) rc = launch_mfma_bwd_kv(p, dtype, st);
        else if (dtype == SA2_F16) rc = p.D == 128 ? launch_col_part<ElemF16, 128>(p, st) : launch_col_part<ElemF16, 64>(p, st);
        else rc = p.D == 128 ? launch_col_part<ElemBF16, 128>(p, st) : launch_col_part<ElemBF16, 64>(p, st);
    }
    return rc;
}

}  // namespace sa2
