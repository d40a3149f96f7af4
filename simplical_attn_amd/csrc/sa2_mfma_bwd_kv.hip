// MFMA backward for gfx950 (bf16 or fp16 elements), the K-side kernel: dK and dV.
//
// A workgroup owns 128 consecutive K/V rows, 32 per wavefront pair (at head_dim 64, where the
// registers allow it and the grid stays large enough: 256 rows, two 32-row blocks per pair, so
// that a unit's forming, its operand reads and the step's barrier serve twice the MFMAs),
// resident in registers as MFMA B operands.  It streams every unit of expanded rows that can see them: unit
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
//
// Small grids (fewer workgroups than the chip holds) split a key block's stream of units over up to
// sixteen workgroups (shares of whole units, at least eight each); each writes its fp32 partial dK and
// dV to the workspace and kv_sum_kernel adds the partials in split order.
#include <type_traits>

#include "sa2_mfma_common.h"

namespace sa2 {
namespace {

constexpr int VW = 8;                  // wavefronts per workgroup
constexpr int VT = VW * 64;            // threads per workgroup
constexpr int VPAIR = 4;
constexpr int KV_MAX_SPLIT = 16;       // workgroups a key block's stream of units is split over, at most
constexpr int KV_MIN_SHARE = 8;        // units a share holds at least
constexpr int KV_GRID_TARGET = 512;    // a split stops once the grid holds this many workgroups

// KB: 32-row blocks of K/V rows per wavefront pair
template <int D, int KB>
struct KvCfg {
    static constexpr int VJ = VPAIR * 32 * KB;     // K rows per workgroup
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
    static constexpr int PX_BYTES = VPAIR * 2 * KB * 64 * 32;
    static constexpr size_t LDS_LIMIT = 160 * 1024;
    static size_t lds_bytes(int w2) {
        return (size_t)NUNIT * UNIT_BYTES + PX_BYTES + 2 * BQ * FS * 4 + 2 * (size_t)(BQ + w2) * RS * 2 + 4 * BQ * 4;
    }
    static bool fits(int w2) { return lds_bytes(w2) <= LDS_LIMIT; }
    // widest run of deltas (minus one) whose K'/V' rows LDS holds at once
    static int max_segment() {
        return (int)((LDS_LIMIT - lds_bytes(0)) / (2 * (size_t)RS * 2));
    }
};

// BIAS = false: k2_bias and v2_bias are both zero (the reference's default), the adds drop out.
// SPLIT (nsplit > 1): the workgroup takes the sp-th share of the key block's units and writes fp32
// partial sums to `part` ([2][nsplit][B*H][N][D]: dK before its scale, then dV).
// SEG = true: a K' window too wide for LDS is walked in segments of ws_arg + 1 deltas; LDS holds the K'/V'
// rows of one segment of a query block and they are reloaded at every segment.  (A kernel of its own, so that
// the common case carries none of it.)
template <class E, int D, bool BIAS, int KB, bool SEG, bool SPLIT>
__global__ __launch_bounds__(VT) __attribute__((amdgpu_waves_per_eu(2, 2)))
void mfma_bwd_kv_kernel(Problem p, int njb, int total, int nsplit_arg, float* __restrict__ part, int ws_arg) {
    const int nsplit = nsplit_arg;           // (1 unless SPLIT; kept a run-time value: the compiler's code for the sweep is better that way)
    typedef typename E::scalar EL;
    typedef typename E::x8 X8;
    using C = KvCfg<D, KB>;
    constexpr int VJ = C::VJ;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int ws = SEG ? ws_arg : w2;
    const int SR = BQ + ws;                                   // K'/V' rows kept per query block and segment
    unsigned char* units = smem_raw;
    unsigned char* px = smem_raw + (size_t)C::NUNIT * C::UNIT_BYTES;
    float* q_s = (float*)(px + C::PX_BYTES);                  // [BQ][FS] q * scale*log2(e), fp32
    float* do_s = q_s + BQ * C::FS;                           // [BQ][FS] dO, fp32
    uint16_t* k2_s = (uint16_t*)(do_s + BQ * C::FS);          // [SR][RS] rows i0-dbase-ws .. i0-dbase+31
    uint16_t* v2_s = k2_s + SR * C::RS;                       // [SR][RS]
    float* lse_s = (float*)(v2_s + SR * C::RS);               // [2][BQ]  -LSE*log2(e), by parity of ib
    float* dsum_s = lse_s + 2 * BQ;                           // [2][BQ]  -D_i

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int role = wave >> 2, pr = wave & 3;
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;

    int pid = blockIdx.x;
    if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
    const int sp = pid % nsplit, pj = pid / nsplit;
    const int bh = pj / njb, jb = pj - bh * njb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int j0 = jb * VJ;
    const int jw = j0 + 32 * KB * pr;            // this pair's K rows: jw .. jw+32*KB-1, in blocks of 32

    const uint16_t* qp = (const uint16_t*)p.q.p + p.q.off(b, 0, h);
    const uint16_t* k2p = (const uint16_t*)p.k2.p + p.k2.off(b, 0, h);
    const uint16_t* v2p = (const uint16_t*)p.v2.p + p.v2.off(b, 0, h);
    const uint16_t* dop = (const uint16_t*)p.dout.p + p.dout.off(b, 0, h);

    // K rows (P wavefront) or V rows (dS wavefront) of the pair as the resident B operand
    X8 kvf[KB][C::DK];
#pragma unroll
    for (int sb = 0; sb < KB; ++sb) {
        const Tensor& t = role ? p.v1 : p.k1;
        const int j = jw + 32 * sb + ln;
        const uint16_t* src = (const uint16_t*)t.p + t.off(b, j < N ? j : N - 1, h) + hf * 8;
#pragma unroll
        for (int kk = 0; kk < C::DK; ++kk) kvf[sb][kk] = *(const X8*)(src + kk * 16);
    }
    floatx16 oacc[KB][C::DT];                    // dV^T (P wavefront) or dK^T (dS wavefront)
#pragma unroll
    for (int sb = 0; sb < KB; ++sb)
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int v = 0; v < 16; ++v) oacc[sb][dt][v] = 0.f;

    const float qscale = p.scale * LOG2E;
    const int j_last = (j0 + VJ - 1 < N ? j0 + VJ - 1 : N - 1);
    const int i_max = (int)((int64_t)j_last + w1 < N - 1 ? j_last + w1 : N - 1);
    auto units_of = [&](int ib) {
        const int il = (ib * BQ + BQ - 1 < N ? ib * BQ + BQ - 1 : N - 1);
        return (w2 < il ? w2 : il) + 1;
    };
    // The units (query block, delta) that see the key block, in stream order, and this workgroup's share of
    // them: from delta d_first of block ib_lo to delta d_last of block ib_hi.  The shares cut the stream
    // counted with w2 + 1 slots per block (a block near the start of the sequence has fewer units: the slots
    // beyond are skipped).
    int ib_lo = j0 / BQ, ib_hi = i_max / BQ, d_first = 0, d_last = w2;
    bool has_work = ib_lo <= ib_hi;
    if constexpr (SPLIT) {
        const int per = w2 + 1, ib0 = ib_lo;
        const int slots = (ib_hi - ib_lo + 1) * per;
        const int chunk = (slots + nsplit - 1) / nsplit;
        const int v_lo = sp * chunk, v_hi = (v_lo + chunk < slots ? v_lo + chunk : slots) - 1;
        has_work = v_lo <= v_hi;
        if (has_work) {
            ib_lo = ib0 + v_lo / per;
            d_first = v_lo - (ib_lo - ib0) * per;
            ib_hi = ib0 + v_hi / per;
            d_last = v_hi - (ib_hi - ib0) * per;
            if (d_first >= units_of(ib_lo)) {        // the share starts in the slots a short block does not have
                ++ib_lo;
                d_first = 0;
            }
            has_work = ib_lo < ib_hi || (ib_lo == ib_hi && d_first <= d_last);
        }
    }
    const int dbase0 = SEG ? d_first : 0;            // first delta of the K'/V' rows loaded first

    // ---- raw rows of a query block: q, dO, the K'/V' rows its deltas reach, -LSE, -D ----
    auto load_raw = [&](int ib, int dbase) {
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
            int k = i0 - dbase - ws + row;
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
    auto form = [&](int dseg, int slot) {        // dseg: delta - first delta of its segment
        if (!former) return;
        const int row = f_row, col = f_col;
        const int kr = row - dseg + ws;
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
    const uint32_t px_addr = lds_address(px) + (uint32_t)(pr * 2 * KB * 64 * 32 + lane * 32);
    // this lane's part of a row operand read (row ln, the k-slots of its half; k-step kk adds
    // kk * KKB) and of a transposed operand read (32-column block dt adds dt * DTB)
    const uint32_t row_lane = (uint32_t)((ln / C::RPW) * C::GROUP + (hf * C::RPW + ln % C::RPW) * 16);
    const uint32_t col_lane = lds_group_column_lane_offset<C::RPW, C::GROUP>(lane);
    constexpr uint32_t KKB = 32 * C::RPW, DTB = 64 * C::RPW;

    // ---- prologue: first block's raw rows, first unit --------------------------------
    if (has_work) {
        load_raw(ib_lo, dbase0);
        __syncthreads();
        fetch_qd();
        form(d_first - dbase0, 0);
        __syncthreads();
    }

    // The sweep, instantiated once per role so that each keeps only its own registers live.
    auto sweep = [&](auto role_tag) {
        constexpr int ROLE = decltype(role_tag)::value;
        int ib = ib_lo, delta = d_first, slot = 0, step = 0, dbase = dbase0;
        int nu = units_of(ib_lo);
        int cur_ib = -1;
        floatx16 negr;                               // -LSE*log2e (P) or -D (dS) of the block's rows, per accumulator element
    #pragma unroll
        for (int v = 0; v < 16; ++v) negr[v] = 0.f;
        floatx16 dp_prev[KB];
    #pragma unroll
        for (int sb = 0; sb < KB; ++sb)
    #pragma unroll
            for (int v = 0; v < 16; ++v) dp_prev[sb][v] = 0.f;
        bool act_prev[KB];
    #pragma unroll
        for (int sb = 0; sb < KB; ++sb) act_prev[sb] = false;

        // dS of the previous unit and its dK MFMAs (dS wavefronts)
        auto consume = [&](int pslot, int pstep) {
            typedef const X8 __attribute__((address_space(3)))* lds_b8;
            const uint32_t qt_addr = units_addr + (uint32_t)(pslot * C::UNIT_BYTES) + col_lane;
            X8 qt[C::DT][2];
    #pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
    #pragma unroll
                for (int ks = 0; ks < 2; ++ks) qt[dt][ks] = lds_group_column_operand_at<C, X8>(qt_addr + dt * DTB, ks);
    #pragma unroll
            for (int sb = 0; sb < KB; ++sb) {
                if (!act_prev[sb]) continue;
                const uint32_t a = px_addr + (uint32_t)(((pstep & 1) * KB + sb) * 64 * 32);
                const X8 p0 = *(lds_b8)(uintptr_t)a, p1 = *(lds_b8)(uintptr_t)(a + 16);
                X8 dsb[2];
    #pragma unroll
                for (int t = 0; t < 8; ++t) {
                    dsb[0][t] = (EL)((float)p0[t] * dp_prev[sb][t]);
                    dsb[1][t] = (EL)((float)p1[t] * dp_prev[sb][8 + t]);
                }
    #pragma unroll
                for (int dt = 0; dt < C::DT; ++dt)
    #pragma unroll
                    for (int ks = 0; ks < 2; ++ks)
                        oacc[sb][dt] = E::mfma(qt[dt][ks], dsb[ks], oacc[sb][dt], 0, 0, 0);
            }
        };
        auto any_of = [&](const bool (&x)[KB]) {
            bool r = false;
    #pragma unroll
            for (int sb = 0; sb < KB; ++sb) r |= x[sb];
            return r;
        };

        while (true) {
            const int i0 = ib * BQ;
            // which of this pair's K blocks see a query of the block?
            bool act[KB];
    #pragma unroll
            for (int sb = 0; sb < KB; ++sb) {
                const int jb0 = jw + 32 * sb;
                act[sb] = (i0 + BQ - 1 >= jb0) && ((int64_t)i0 <= (int64_t)jb0 + 31 + w1) && jb0 < N;
            }
            const bool act_any = any_of(act);
            if (act_any && cur_ib != ib) {
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
                if (act_any) {
                    X8 qa[C::DK];
    #pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) qa[kk] = lds_read_x8<X8>(u_addr + row_lane + kk * KKB);
                    X8 pb[KB][2];
    #pragma unroll
                    for (int sb = 0; sb < KB; ++sb) {
                        if (!act[sb]) continue;
                        const int jb0 = jw + 32 * sb, j = jb0 + ln;
                        floatx16 sh;
                        const bool interior = (i0 >= jb0 + 31) && ((int64_t)i0 + 31 <= (int64_t)jb0 + w1) && (i0 + BQ - 1 < N) &&
                                              (i0 >= delta);
                        if (__builtin_expect(interior, 1)) {
                            sh = E::mfma(qa[0], kvf[sb][0], negr, 0, 0, 0);
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
                            sh = E::mfma(qa[0], kvf[sb][0], ct, 0, 0, 0);
                        }
    #pragma unroll
                        for (int kk = 1; kk < C::DK; ++kk)
                            sh = E::mfma(qa[kk], kvf[sb][kk], sh, 0, 0, 0);
    #pragma unroll
                        for (int ks = 0; ks < 2; ++ks)
    #pragma unroll
                            for (int t = 0; t < 8; ++t) pb[sb][ks][t] = (EL)fast_exp2(sh[ks * 8 + t]);
                        {
                            typedef X8 __attribute__((address_space(3)))* lds_b8;
                            const uint32_t a = px_addr + (uint32_t)(((step & 1) * KB + sb) * 64 * 32);
                            *(lds_b8)(uintptr_t)a = pb[sb][0];
                            *(lds_b8)(uintptr_t)(a + 16) = pb[sb][1];
                        }
                    }
                    const uint32_t dt_addr = u_addr + (uint32_t)C::TILE_BYTES + col_lane;
                    X8 da[C::DT][2];
    #pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
    #pragma unroll
                        for (int ks = 0; ks < 2; ++ks) da[dt][ks] = lds_group_column_operand_at<C, X8>(dt_addr + dt * DTB, ks);
    #pragma unroll
                    for (int sb = 0; sb < KB; ++sb) {
                        if (!act[sb]) continue;
    #pragma unroll
                        for (int dt = 0; dt < C::DT; ++dt)
    #pragma unroll
                            for (int ks = 0; ks < 2; ++ks)
                                oacc[sb][dt] = E::mfma(da[dt][ks], pb[sb][ks], oacc[sb][dt], 0, 0, 0);
                    }
                }
            } else {
                // first the previous unit (its dP is still in dp_prev), then this unit's dP
                if (any_of(act_prev)) consume(slot == 0 ? C::NUNIT - 1 : slot - 1, step - 1);
                if (act_any) {
                    const uint32_t d_addr = u_addr + (uint32_t)C::TILE_BYTES;
                    X8 da[C::DK];
    #pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) da[kk] = lds_read_x8<X8>(d_addr + row_lane + kk * KKB);
    #pragma unroll
                    for (int sb = 0; sb < KB; ++sb) {
                        if (!act[sb]) continue;
                        dp_prev[sb] = E::mfma(da[0], kvf[sb][0], negr, 0, 0, 0);
    #pragma unroll
                        for (int kk = 1; kk < C::DK; ++kk)
                            dp_prev[sb] = E::mfma(da[kk], kvf[sb][kk], dp_prev[sb], 0, 0, 0);
                    }
                    if constexpr (KB == 1) {
                        __builtin_amdgcn_sched_group_barrier(0x100, C::DK, 0);
                        __builtin_amdgcn_sched_group_barrier(0x008, C::DK, 0);
                    }
                }
    #pragma unroll
                for (int sb = 0; sb < KB; ++sb) act_prev[sb] = act[sb];
            }

            // ---- next unit: form it one step ahead (after a change of block: its raw rows first)
            int nib = ib, ndelta = delta + 1;
            if (ndelta >= nu) {
                nib = ib + 1;
                ndelta = 0;
            }
            const bool more = SPLIT ? (nib < ib_hi || (nib == ib_hi && ndelta <= d_last)) : nib <= ib_hi;
            const int nslot = slot + 1 == C::NUNIT ? 0 : slot + 1;
            if (more) {
                if (nib != ib || (SEG && ndelta - dbase > ws)) {
                    if constexpr (SEG) dbase = ndelta;
                    __syncthreads();         // nobody still forms from the old rows
                    load_raw(nib, dbase);
                    __syncthreads();
                    fetch_qd();
                    nu = units_of(nib);
                }
                form(ndelta - dbase, nslot);
            }
            __syncthreads();
            ++step;
            if (!more) break;
            ib = nib;
            delta = ndelta;
            slot = nslot;
        }
        if (ROLE == 1 && any_of(act_prev)) consume(slot, step - 1);

    };
    if (has_work) {
        if (role == 0) sweep(std::integral_constant<int, 0>());
        else sweep(std::integral_constant<int, 1>());
    }

    const Tensor& t = role ? p.dk1 : p.dv1;
    const float sc = role ? LN2 : 1.f;               // Q~ carries scale*log2(e)
#pragma unroll
    for (int sb = 0; sb < KB; ++sb) {
        const int j = jw + 32 * sb + ln;
        if (j >= N || !t.p) continue;
        if (nsplit == 1) {
            uint16_t* dst = (uint16_t*)t.p + t.off(b, j, h) + 4 * hf;
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    union { EL hh[4]; uint2 u; } a;
#pragma unroll
                    for (int x = 0; x < 4; ++x) a.hh[x] = (EL)(oacc[sb][dt][4 * g4 + x] * sc);
                    *(uint2*)(dst + dt * 32 + 8 * g4) = a.u;
                }
        } else {
            // fp32 partial of this share: [dK | dV][split][batch*head][position][column]
            const int64_t BH = (int64_t)p.B * p.H;
            float* dst = part + ((((role ? 0 : 1) * (int64_t)nsplit + sp) * BH + bh) * N + j) * D + 4 * hf;
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4)
                    *(float4*)(dst + dt * 32 + 8 * g4) = make_float4(oacc[sb][dt][4 * g4] * sc, oacc[sb][dt][4 * g4 + 1] * sc,
                                                                     oacc[sb][dt][4 * g4 + 2] * sc, oacc[sb][dt][4 * g4 + 3] * sc);
        }
    }
}

// dK and dV from the partial sums of a split launch, shares added in their order
template <class E>
__global__ __launch_bounds__(256) void kv_sum_kernel(Problem p, int nsplit, const float* __restrict__ part, int64_t chunks) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= chunks) return;
    const int D = p.D;
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
        *(uint2*)((uint16_t*)t.p + t.off(b, j, h) + col * 4) = make_uint2(E::pack(acc.x, acc.y), E::pack(acc.z, acc.w));
    }
}

// Geometry of a launch: 32-row K blocks per wavefront pair, and the number of shares a key block's
// stream of units is split into.  Both depend on the problem's sizes only.
struct KvPlan {
    int kb, nsplit;
};
KvPlan kv_plan(int B, int N, int H, int D, int w1, int w2) {
    KvPlan pl{1, 1};
    const int64_t bh = (int64_t)B * H;
    // two K blocks per pair at head_dim 64 when that still leaves a grid worth splitting no further than in two
    if (D == 64 && bh * ((N + 255) / 256) * 2 >= KV_GRID_TARGET / 2) pl.kb = 2;
    const int vj = VPAIR * 32 * pl.kb;
    const int64_t base = bh * ((N + vj - 1) / vj);
    const int blocks = (vj + (w1 < N ? w1 : N) + BQ - 1) / BQ + 1;          // query blocks a key block streams, at most
    // (the partial sums of a split launch stay under 32 MiB)
    auto part_bytes = [&](int ns) { return (int64_t)2 * ns * bh * N * D * 4; };
    const int64_t units = (int64_t)blocks * ((w2 < N - 1 ? w2 : N - 1) + 1);     // of a key block's stream, at most
    while (pl.nsplit < KV_MAX_SPLIT && base * pl.nsplit * 2 <= KV_GRID_TARGET && (int64_t)pl.nsplit * 2 * KV_MIN_SHARE <= units &&
           part_bytes(pl.nsplit * 2) <= ((int64_t)32 << 20))
        pl.nsplit *= 2;
    return pl;
}

template <class E, int D, int KB>
int launch_kv_geometry(const Problem& p, int nsplit, hipStream_t st) {
    using C = KvCfg<D, KB>;
    const int njb = (p.N + C::VJ - 1) / C::VJ;
    const int64_t total = (int64_t)njb * p.B * p.H * nsplit;
    if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    const int ws = p.w2 < C::max_segment() ? p.w2 : C::max_segment();
    const size_t lds = C::lds_bytes(ws);
    const bool bias = p.k2_bias != 0.f || p.v2_bias != 0.f;
    // the partial sums of a split launch lie behind the K'-side kernel's part of the workspace
    float* part = nullptr;
    if (nsplit > 1) {
        const size_t off = kp_side_scratch_bytes(p.B, p.N, p.H, D, p.w2);
        if (p.scratch_bytes < off + kv_split_scratch_bytes(p.B, p.N, p.H, D, p.w1, p.w2)) return SA2_ERR_WORKSPACE_TOO_SMALL;
        part = (float*)((char*)p.scratch + off);
    }
    const bool seg = ws < p.w2;
    // (the segmented kernel exists with the bias adds only)
    auto go = [&](auto kernel) {
        if (!allow_full_lds((const void*)kernel)) return false;
        hipLaunchKernelGGL(kernel, dim3((unsigned)total), dim3(VT), lds, st, p, njb, (int)total, nsplit, part, ws);
        return true;
    };
    bool ok;
    if (nsplit > 1)
        ok = seg    ? go(mfma_bwd_kv_kernel<E, D, true, KB, true, true>)
             : bias ? go(mfma_bwd_kv_kernel<E, D, true, KB, false, true>)
                    : go(mfma_bwd_kv_kernel<E, D, false, KB, false, true>);
    else
        ok = seg    ? go(mfma_bwd_kv_kernel<E, D, true, KB, true, false>)
             : bias ? go(mfma_bwd_kv_kernel<E, D, true, KB, false, false>)
                    : go(mfma_bwd_kv_kernel<E, D, false, KB, false, false>);
    if (!ok) return SA2_ERR_LAUNCH_FAILED;
    if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
    if (nsplit > 1) {
        const int64_t chunks = (int64_t)p.B * p.H * p.N * (D / 4);
        hipLaunchKernelGGL((kv_sum_kernel<E>), dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st, p, nsplit, part, chunks);
        if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
    }
    return SA2_OK;
}

template <class E, int D>
int launch_kv(const Problem& p, hipStream_t st) {
    const KvPlan pl = kv_plan(p.B, p.N, p.H, D, p.w1, p.w2);
    if constexpr (D == 64) {
        if (pl.kb == 2) return launch_kv_geometry<E, D, 2>(p, pl.nsplit, st);
    }
    return launch_kv_geometry<E, D, 1>(p, pl.nsplit, st);
}

}  // namespace

size_t kv_split_scratch_bytes(int B, int N, int H, int D, int w1, int w2) {
    const KvPlan pl = kv_plan(B, N, H, D, w1, w2);
    return pl.nsplit > 1 ? (size_t)2 * pl.nsplit * B * H * (size_t)N * D * sizeof(float) : 0;
}

int launch_mfma_bwd_kv(const Problem& p, int dtype, hipStream_t st) {
    if (dtype == SA2_F16)
        return p.D == 128 ? launch_kv<ElemF16, 128>(p, st) : p.D == 64 ? launch_kv<ElemF16, 64>(p, st) : launch_kv<ElemF16, 32>(p, st);
    return p.D == 128 ? launch_kv<ElemBF16, 128>(p, st) : p.D == 64 ? launch_kv<ElemBF16, 64>(p, st) : launch_kv<ElemBF16, 32>(p, st);
}

}  // namespace sa2
