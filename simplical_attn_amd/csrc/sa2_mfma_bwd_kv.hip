// MFMA backward for gfx950 (bf16 or fp16 elements), the K-side kernel: dK and dV.
//
// A workgroup owns 128 consecutive K/V rows, 32 per wavefront pair, resident in registers
// as MFMA B operands.  It streams every unit of expanded rows that can see them: unit
// (query block ib, delta) is the 32 rows r = (i0 + r, k = i - delta) with
// Q~[r] = q[i] * k2~[k] * scale*log2(e) and dO~[r] = dO[i] * v2~[k], formed by the whole
// workgroup into a three-deep LDS ring one step ahead of their use.  Per unit and pair:
//   the "P" wavefront computes S = Q~.K^T - LSE, P = exp2(S), hands P (16 bit) to its partner
//       through LDS and accumulates dV^T += dO~^T.P;
//   the "dS" wavefront computes dP = dO~.V^T - D and, one unit behind, dS = P*dP and
//       dK^T += Q~^T.dS.
// Transposed operands come from the same unit tiles through ds_read_b64_tr_b16; the tiles are laid
// out in row groups so that both kinds of read are free of bank conflicts.
// Every output element has one writer and a fixed summation order.
#include <type_traits>

#include "sa2_mfma_common.h"

namespace sa2 {
namespace {

constexpr int VW = 8;                  // wavefronts per workgroup
constexpr int VT = VW * 64;            // threads per workgroup
constexpr int VPAIR = 4;
constexpr int VJ = VPAIR * 32;         // K rows per workgroup

template <int D>
struct KvCfg {
    static constexpr int DK = D / 16;
    static constexpr int DT = D / 32;
    // A unit tile (32 rows) in LDS keeps groups of RPW rows together: within a group the 16-byte
    // chunk c of row q sits at byte (c * RPW + q) * 16, groups lie GROUP bytes apart.  Row operand
    // reads (16 bytes per lane) and transposed operand reads are both bank-conflict free in it.
    static constexpr int RPW = 512 / D;        // rows per group: 4 (D = 128), 8 (D = 64), 16 (D = 32)
    static constexpr int GROUP = 1024 + 16 * RPW;
    static constexpr int TILE_BYTES = (BQ / RPW) * GROUP;
    static constexpr int UNIT_BYTES = 2 * TILE_BYTES;      // Q~ tile, then dO~ tile
    static constexpr int row_off(int r) { return (r / RPW) * GROUP + (r % RPW) * 16; }    // chunk 0 of row r
    static constexpr int NUNIT = 3;
    static constexpr int RS = D + D / 4;       // K'/V' row stride (bf16): the forming threads' reads (RPW rows x 16 bytes per 16 lanes) hit distinct banks
    static constexpr int FS = D;               // q / dO row stride (fp32); read once per query block, unpadded
    static constexpr int PX_BYTES = VPAIR * 2 * 64 * 32;
    static constexpr size_t LDS_LIMIT = 160 * 1024;
    static size_t lds_bytes(int w2) {
        return (size_t)NUNIT * UNIT_BYTES + PX_BYTES + 2 * BQ * FS * 4 + 2 * (size_t)(BQ + w2) * RS * 2 + 4 * BQ * 4;
    }
    static bool fits(int w2) { return lds_bytes(w2) <= LDS_LIMIT; }
};

// BIAS = false: k2_bias and v2_bias are both zero (the reference's default), the adds drop out.
template <class E, int D, bool BIAS>
__global__ __launch_bounds__(VT) __attribute__((amdgpu_waves_per_eu(2, 2)))
void mfma_bwd_kv_kernel(Problem p, int njb, int total) {
    typedef typename E::scalar EL;
    typedef typename E::x8 X8;
    using C = KvCfg<D>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int SR = BQ + w2;                                   // K'/V' rows kept per query block
    unsigned char* units = smem_raw;
    unsigned char* px = smem_raw + (size_t)C::NUNIT * C::UNIT_BYTES;
    float* q_s = (float*)(px + C::PX_BYTES);                  // [BQ][FS] q * scale*log2(e), fp32
    float* do_s = q_s + BQ * C::FS;                           // [BQ][FS] dO, fp32
    uint16_t* k2_s = (uint16_t*)(do_s + BQ * C::FS);          // [SR][RS] rows i0-w2 .. i0+31
    uint16_t* v2_s = k2_s + SR * C::RS;                       // [SR][RS]
    float* lse_s = (float*)(v2_s + SR * C::RS);               // [2][BQ]  -LSE*log2(e), by parity of ib
    float* dsum_s = lse_s + 2 * BQ;                           // [2][BQ]  -D_i

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int role = wave >> 2, pr = wave & 3;
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;

    int pid = blockIdx.x;
    if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
    const int bh = pid / njb, jb = pid - bh * njb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int j0 = jb * VJ;
    const int jw = j0 + 32 * pr;                 // this pair's K rows: jw .. jw+31
    const int j = jw + ln;
    const int jc = j < N ? j : N - 1;

    const uint16_t* qp = (const uint16_t*)p.q.p + p.q.off(b, 0, h);
    const uint16_t* k2p = (const uint16_t*)p.k2.p + p.k2.off(b, 0, h);
    const uint16_t* v2p = (const uint16_t*)p.v2.p + p.v2.off(b, 0, h);
    const uint16_t* dop = (const uint16_t*)p.dout.p + p.dout.off(b, 0, h);

    // K rows (P wavefront) or V rows (dS wavefront) of the pair as the resident B operand
    X8 kvf[C::DK];
    {
        const Tensor& t = role ? p.v1 : p.k1;
        const uint16_t* src = (const uint16_t*)t.p + t.off(b, jc, h) + hf * 8;
#pragma unroll
        for (int kk = 0; kk < C::DK; ++kk) kvf[kk] = *(const X8*)(src + kk * 16);
    }
    floatx16 oacc[C::DT];                        // dV^T (P wavefront) or dK^T (dS wavefront)
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) oacc[dt][v] = 0.f;

    const float qscale = p.scale * LOG2E;
    const int j_last = (j0 + VJ - 1 < N ? j0 + VJ - 1 : N - 1);
    const int i_max = (int)((int64_t)j_last + w1 < N - 1 ? j_last + w1 : N - 1);
    const int ib_lo = j0 / BQ, ib_hi = i_max / BQ;
    auto units_of = [&](int ib) {
        const int il = (ib * BQ + BQ - 1 < N ? ib * BQ + BQ - 1 : N - 1);
        return (w2 < il ? w2 : il) + 1;
    };

    // ---- raw rows of a query block: q, dO, the K'/V' rows its deltas reach, -LSE, -D ----
    auto load_raw = [&](int ib) {
        constexpr int CPR = D / 8;
        const int i0 = ib * BQ;
        for (int c = tid; c < BQ * CPR; c += VT) {
            const int row = c / CPR, col = c - row * CPR;
            int i = i0 + row;
            i = i < N ? i : N - 1;
            const uint4 qa = *(const uint4*)(qp + (int64_t)i * p.q.sn + col * 8);
            const uint4 da = *(const uint4*)(dop + (int64_t)i * p.dout.sn + col * 8);
            float* qd = q_s + row * C::FS + col * 8;
            float* dd = do_s + row * C::FS + col * 8;
            *(float4*)qd = make_float4(E::lo(qa.x) * qscale, E::hi(qa.x) * qscale, E::lo(qa.y) * qscale, E::hi(qa.y) * qscale);
            *(float4*)(qd + 4) = make_float4(E::lo(qa.z) * qscale, E::hi(qa.z) * qscale, E::lo(qa.w) * qscale, E::hi(qa.w) * qscale);
            *(float4*)dd = make_float4(E::lo(da.x), E::hi(da.x), E::lo(da.y), E::hi(da.y));
            *(float4*)(dd + 4) = make_float4(E::lo(da.z), E::hi(da.z), E::lo(da.w), E::hi(da.w));
        }
        for (int c = tid; c < SR * CPR; c += VT) {
            const int row = c / CPR, col = c - row * CPR;
            int k = i0 - w2 + row;
            k = k < 0 ? 0 : (k < N ? k : N - 1);
            *(uint4*)(k2_s + row * C::RS + col * 8) = *(const uint4*)(k2p + (int64_t)k * p.k2.sn + col * 8);
            *(uint4*)(v2_s + row * C::RS + col * 8) = *(const uint4*)(v2p + (int64_t)k * p.v2.sn + col * 8);
        }
        if (tid < BQ) {
            int i = i0 + tid;
            i = i < N ? i : N - 1;
            lse_s[(ib & 1) * BQ + tid] = -p.lse[(int64_t)bh * N + i] * LOG2E;
            dsum_s[(ib & 1) * BQ + tid] = -p.dsum[(int64_t)bh * N + i];
        }
    };
    // ---- form unit (ib, delta) into a ring slot: one 16-byte chunk of Q~ and of dO~ per thread ----
    // this thread's chunk of the block's q and dO rows stays in registers for the block's units
    float qv[8], dv[8];
#pragma unroll
    for (int t = 0; t < 8; ++t) qv[t] = dv[t] = 0.f;
    // Wavefront g < 32 / RPW forms row group g of a unit: lane L the 16-byte chunk L / RPW of row
    // L % RPW, so that a wavefront's stores fill the group's 1 KB contiguously.
    const bool former = wave < BQ / C::RPW;
    const int f_row = wave * C::RPW + lane % C::RPW, f_col = lane / C::RPW;
    auto fetch_qd = [&]() {
        if (!former) return;
        const int row = f_row, col = f_col;
        const float4 q0 = *(const float4*)(q_s + row * C::FS + col * 8), q1 = *(const float4*)(q_s + row * C::FS + col * 8 + 4);
        const float4 d0 = *(const float4*)(do_s + row * C::FS + col * 8), d1 = *(const float4*)(do_s + row * C::FS + col * 8 + 4);
        qv[0] = q0.x; qv[1] = q0.y; qv[2] = q0.z; qv[3] = q0.w; qv[4] = q1.x; qv[5] = q1.y; qv[6] = q1.z; qv[7] = q1.w;
        dv[0] = d0.x; dv[1] = d0.y; dv[2] = d0.z; dv[3] = d0.w; dv[4] = d1.x; dv[5] = d1.y; dv[6] = d1.z; dv[7] = d1.w;
    };
    auto form = [&](int delta, int slot) {
        if (!former) return;
        const int row = f_row, col = f_col;
        const int kr = row - delta + w2;
        const uint4 kx = *(const uint4*)(k2_s + kr * C::RS + col * 8);
        const uint4 vx = *(const uint4*)(v2_s + kr * C::RS + col * 8);
        const uint32_t kw[4] = {kx.x, kx.y, kx.z, kx.w}, vw[4] = {vx.x, vx.y, vx.z, vx.w};
        const float kb = BIAS ? p.k2_bias : 0.f, vb = BIAS ? p.v2_bias : 0.f;
        X8 r, d;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (BIAS) {
                r[2 * t] = (EL)(qv[2 * t] * (E::lo(kw[t]) + kb));
                r[2 * t + 1] = (EL)(qv[2 * t + 1] * (E::hi(kw[t]) + kb));
                d[2 * t] = (EL)(dv[2 * t] * (E::lo(vw[t]) + vb));
                d[2 * t + 1] = (EL)(dv[2 * t + 1] * (E::hi(vw[t]) + vb));
            } else {
                r[2 * t] = (EL)(qv[2 * t] * E::lo(kw[t]));
                r[2 * t + 1] = (EL)(qv[2 * t + 1] * E::hi(kw[t]));
                d[2 * t] = (EL)(dv[2 * t] * E::lo(vw[t]));
                d[2 * t + 1] = (EL)(dv[2 * t + 1] * E::hi(vw[t]));
            }
        }
        unsigned char* dst = units + slot * C::UNIT_BYTES + wave * C::GROUP + lane * 16;
        *(X8*)dst = r;
        *(X8*)(dst + C::TILE_BYTES) = d;
    };

    const uint32_t units_addr = lds_address(units);
    const uint32_t px_addr = lds_address(px) + (uint32_t)(pr * 2 * 64 * 32 + lane * 32);
    // this lane's part of a row operand read (row ln, the k-slots of its half; k-step kk adds
    // kk * KKB) and of a transposed operand read (32-column block dt adds dt * DTB)
    const uint32_t row_lane = (uint32_t)((ln / C::RPW) * C::GROUP + (hf * C::RPW + ln % C::RPW) * 16);
    const uint32_t col_lane = lds_group_column_lane_offset<C::RPW, C::GROUP>(lane);
    constexpr uint32_t KKB = 32 * C::RPW, DTB = 64 * C::RPW;

    // ---- prologue: first block's raw rows, first unit --------------------------------
    load_raw(ib_lo);
    __syncthreads();
    fetch_qd();
    form(0, 0);
    __syncthreads();

    // The sweep, instantiated once per role so that each keeps only its own registers live.
    auto sweep = [&](auto role_tag) {
        constexpr int ROLE = decltype(role_tag)::value;
        int ib = ib_lo, delta = 0, slot = 0, step = 0;
        int nu = units_of(ib_lo);
        int cur_ib = -1;
        floatx16 negr;                               // -LSE*log2e (P) or -D (dS) of the block's rows, per accumulator element
    #pragma unroll
        for (int v = 0; v < 16; ++v) negr[v] = 0.f;
        floatx16 dp_prev;
    #pragma unroll
        for (int v = 0; v < 16; ++v) dp_prev[v] = 0.f;
        bool act_prev = false;

        // dS of the previous unit and its dK MFMAs (dS wavefronts)
        auto consume = [&](int pslot, int pstep) {
            typedef const X8 __attribute__((address_space(3)))* lds_b8;
            const uint32_t a = px_addr + (uint32_t)((pstep & 1) * 64 * 32);
            const X8 p0 = *(lds_b8)(uintptr_t)a, p1 = *(lds_b8)(uintptr_t)(a + 16);
            const uint32_t qt_addr = units_addr + (uint32_t)(pslot * C::UNIT_BYTES) + col_lane;
            X8 qt[C::DT][2];
    #pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
    #pragma unroll
                for (int ks = 0; ks < 2; ++ks) qt[dt][ks] = lds_group_column_operand_at<C, X8>(qt_addr + dt * DTB, ks);
            X8 dsb[2];
    #pragma unroll
            for (int t = 0; t < 8; ++t) {
                dsb[0][t] = (EL)((float)p0[t] * dp_prev[t]);
                dsb[1][t] = (EL)((float)p1[t] * dp_prev[8 + t]);
            }
    #pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
    #pragma unroll
                for (int ks = 0; ks < 2; ++ks)
                    oacc[dt] = E::mfma(qt[dt][ks], dsb[ks], oacc[dt], 0, 0, 0);
        };

        while (true) {
            const int i0 = ib * BQ;
            // does this pair's K tile see any query of the block?
            const bool act = (i0 + BQ - 1 >= jw) && ((int64_t)i0 <= (int64_t)jw + 31 + w1) && jw < N;
            if (act && cur_ib != ib) {
                const float* src = (ROLE ? dsum_s : lse_s) + (ib & 1) * BQ + 4 * hf;
    #pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const float4 a = *(const float4*)(src + 8 * g4);
                    negr[4 * g4] = a.x; negr[4 * g4 + 1] = a.y; negr[4 * g4 + 2] = a.z; negr[4 * g4 + 3] = a.w;
                }
                cur_ib = ib;
            }
            const uint32_t u_addr = units_addr + (uint32_t)(slot * C::UNIT_BYTES);
            if (ROLE == 0) {
                if (act) {
                    X8 qa[C::DK];
    #pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) qa[kk] = lds_read_x8<X8>(u_addr + row_lane + kk * KKB);
                    floatx16 sh;
                    const bool interior = (i0 >= jw + 31) && ((int64_t)i0 + 31 <= (int64_t)jw + w1) && (i0 + BQ - 1 < N) &&
                                          (i0 >= delta);
                    if (__builtin_expect(interior, 1)) {
                        sh = E::mfma(qa[0], kvf[0], negr, 0, 0, 0);
                    } else {
                        asm volatile("" ::: "memory");
                        // element v of this lane is query i0 + 8*(v/4) + 4*hf + v%4, column j
                        const int lo = j - i0 - 4 * hf;
                        const int hi = (int)((int64_t)j + w1 - i0 < 1 << 20 ? j + w1 - i0 : 1 << 20) - 4 * hf;
                        const int dlo = delta - i0 - 4 * hf, nhi = N - 1 - i0 - 4 * hf;
                        floatx16 ct;
    #pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int c = 8 * (v >> 2) + (v & 3);
                            ct[v] = ((j < N) & (c >= lo) & (c <= hi) & (c >= dlo) & (c <= nhi)) ? negr[v] : -INFINITY;
                        }
                        sh = E::mfma(qa[0], kvf[0], ct, 0, 0, 0);
                    }
    #pragma unroll
                    for (int kk = 1; kk < C::DK; ++kk)
                        sh = E::mfma(qa[kk], kvf[kk], sh, 0, 0, 0);
                    X8 pb[2];
    #pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
    #pragma unroll
                        for (int t = 0; t < 8; ++t) pb[ks][t] = (EL)fast_exp2(sh[ks * 8 + t]);
                    {
                        typedef X8 __attribute__((address_space(3)))* lds_b8;
                        const uint32_t a = px_addr + (uint32_t)((step & 1) * 64 * 32);
                        *(lds_b8)(uintptr_t)a = pb[0];
                        *(lds_b8)(uintptr_t)(a + 16) = pb[1];
                    }
                    const uint32_t dt_addr = u_addr + (uint32_t)C::TILE_BYTES + col_lane;
                    X8 da[C::DT][2];
    #pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
    #pragma unroll
                        for (int ks = 0; ks < 2; ++ks) da[dt][ks] = lds_group_column_operand_at<C, X8>(dt_addr + dt * DTB, ks);
    #pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
    #pragma unroll
                        for (int ks = 0; ks < 2; ++ks)
                            oacc[dt] = E::mfma(da[dt][ks], pb[ks], oacc[dt], 0, 0, 0);
                }
            } else {
                // first the previous unit (its dP is still in dp_prev), then this unit's dP
                if (act_prev) consume(slot == 0 ? C::NUNIT - 1 : slot - 1, step - 1);
                if (act) {
                    const uint32_t d_addr = u_addr + (uint32_t)C::TILE_BYTES;
                    X8 da[C::DK];
    #pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) da[kk] = lds_read_x8<X8>(d_addr + row_lane + kk * KKB);
                    dp_prev = E::mfma(da[0], kvf[0], negr, 0, 0, 0);
    #pragma unroll
                    for (int kk = 1; kk < C::DK; ++kk)
                        dp_prev = E::mfma(da[kk], kvf[kk], dp_prev, 0, 0, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, C::DK, 0);
                    __builtin_amdgcn_sched_group_barrier(0x008, C::DK, 0);
                }
                act_prev = act;
            }

            // ---- next unit: form it one step ahead (after a change of block: its raw rows first)
            int nib = ib, ndelta = delta + 1;
            if (ndelta >= nu) {
                nib = ib + 1;
                ndelta = 0;
            }
            const bool more = nib <= ib_hi;
            const int nslot = slot + 1 == C::NUNIT ? 0 : slot + 1;
            if (more) {
                if (nib != ib) {
                    __syncthreads();         // nobody still forms from the old rows
                    load_raw(nib);
                    __syncthreads();
                    fetch_qd();
                    nu = units_of(nib);
                }
                form(ndelta, nslot);
            }
            __syncthreads();
            ++step;
            if (!more) break;
            ib = nib;
            delta = ndelta;
            slot = nslot;
        }
        if (ROLE == 1 && act_prev) consume(slot, step - 1);

    };
    if (role == 0) sweep(std::integral_constant<int, 0>());
    else sweep(std::integral_constant<int, 1>());

    if (j < N) {
        const Tensor& t = role ? p.dk1 : p.dv1;
        if (t.p) {
            uint16_t* dst = (uint16_t*)t.p + t.off(b, j, h) + 4 * hf;
            const float sc = role ? LN2 : 1.f;       // Q~ carries scale*log2(e)
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    union { EL hh[4]; uint2 u; } a;
#pragma unroll
                    for (int x = 0; x < 4; ++x) a.hh[x] = (EL)(oacc[dt][4 * g4 + x] * sc);
                    *(uint2*)(dst + dt * 32 + 8 * g4) = a.u;
                }
        }
    }
}

template <class E, int D>
int launch_kv(const Problem& p, hipStream_t st) {
    using C = KvCfg<D>;
    const int njb = (p.N + VJ - 1) / VJ;
    const int64_t total = (int64_t)njb * p.B * p.H;
    if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    const size_t lds = C::lds_bytes(p.w2);
    const bool bias = p.k2_bias != 0.f || p.v2_bias != 0.f;
    const void* fn = bias ? (const void*)mfma_bwd_kv_kernel<E, D, true> : (const void*)mfma_bwd_kv_kernel<E, D, false>;
    if (!allow_full_lds(fn)) return SA2_ERR_LAUNCH_FAILED;
    if (bias) hipLaunchKernelGGL((mfma_bwd_kv_kernel<E, D, true>), dim3((unsigned)total), dim3(VT), lds, st, p, njb, (int)total);
    else hipLaunchKernelGGL((mfma_bwd_kv_kernel<E, D, false>), dim3((unsigned)total), dim3(VT), lds, st, p, njb, (int)total);
    return hipGetLastError() == hipSuccess ? SA2_OK : SA2_ERR_LAUNCH_FAILED;
}

}  // namespace

bool kv_fits(int D, int w2) {
    return D == 128 ? KvCfg<128>::fits(w2) : D == 64 ? KvCfg<64>::fits(w2) : D == 32 ? KvCfg<32>::fits(w2) : false;
}

int launch_mfma_bwd_kv(const Problem& p, int dtype, hipStream_t st) {
    if (dtype == SA2_F16)
        return p.D == 128 ? launch_kv<ElemF16, 128>(p, st) : p.D == 64 ? launch_kv<ElemF16, 64>(p, st) : launch_kv<ElemF16, 32>(p, st);
    return p.D == 128 ? launch_kv<ElemBF16, 128>(p, st) : p.D == 64 ? launch_kv<ElemBF16, 64>(p, st) : launch_kv<ElemBF16, 32>(p, st);
}

}  // namespace sa2
