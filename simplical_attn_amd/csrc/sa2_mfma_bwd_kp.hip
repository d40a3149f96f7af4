// MFMA backward for gfx950 (bf16 or fp16 elements), the K'-side kernel: dQ, dK' and dV'.
//
// Expanded rows r = (i, k), k = i - delta in the K' window of i.  A workgroup owns 32
// consecutive K' rows k0..k0+31 and every delta: unit delta is the 32 rows
// (i = k + delta, k).  With P = exp2(S - LSE*log2e) and dS = P * (dO~.v1 - D_i):
//
//   R[r,:] = sum_j P[r,j]  v1[j,:]        dV'[k] = sum_delta R[(k+delta,k)] * dO[k+delta]
//   G[r,:] = sum_j dS[r,j] k1[j,:]        dK'[k] = scale * sum_delta G[(k+delta,k)] * q[k+delta]
//                                         dQ[i]  = scale * sum_delta G[(i,i-delta)] * k2~[i-delta]
//
// dK' and dV' are aligned with the unit's rows, so they accumulate in registers over the
// deltas a wavefront handles; dQ is shifted by delta and goes through an fp32 accumulator
// in LDS (rows k0 .. k0+31+w2), written once per workgroup as a partial that a small
// kernel adds up (a query gets partials from at most 2 + w2/32 workgroups, summed in a
// fixed order: bitwise reproducible).  A K' window too wide for that accumulator is cut into
// segments of deltas, one workgroup per (K' block, segment); their fp32 partial dK' and dV' are
// added by kp_sum_kernel in segment order.
//
// Eight wavefronts, two per SIMD, form four pairs that each hold one unit per round (two
// consecutive deltas at head_dim 32 and 64, where the registers allow it: every K and V operand
// read, tile request and step barrier then serves twice the MFMAs) and
// sweep the K1/V1 window in 32-key tiles staged through a three-deep LDS ring:
//   the "P" wavefront computes S^T = K1.Q~^T, P = exp2(S - LSE), hands P (16 bit) to its
//       partner through LDS and accumulates R^T += V1^T.P^T;
//   the "dS" wavefront computes dP^T = V1.dO~^T and, one tile behind, dS = P*(dP - D) and
//       G^T += K1^T.dS^T.
// Every MFMA operand that streams from LDS is read once per 32x32x16 MFMA; transposed
// operands come from the row-major tiles through ds_read_b64_tr_b16.
#include <type_traits>

#include "sa2_mfma_common.h"

namespace sa2 {
namespace {

constexpr int KW = 8;                  // wavefronts per workgroup
constexpr int KT = KW * 64;            // threads per workgroup
constexpr int NPAIR = 4;

__device__ __forceinline__ int kp_recompute_here(int x) {
    asm volatile("" : "+v"(x));
    return x;
}

// U: units (consecutive deltas) a wavefront pair holds per round
template <int D, int U = 1>
struct KpCfg {
    static constexpr int DK = D / 16;
    static constexpr int DT = D / 32;
    // K and V tiles are written by direct global->LDS loads: one wavefront instruction fills a
    // group of RPW rows (1 KB), lane L putting the 16-byte chunk L / RPW of row L % RPW at byte
    // 16 * L; groups lie GROUP bytes apart.  Row and transposed operand reads are conflict free.
    static constexpr int RPW = 512 / D;
    // byte offset of row r of a tile (chunk 0)
    static constexpr int row_off(int r) { return (r / RPW) * GROUP + (r % RPW) * 16; }
    static constexpr int GROUP = 1024 + 16 * RPW;
    static constexpr int NGROUP = TJ / RPW;
    static constexpr int TILE_BYTES = NGROUP * GROUP;
    static constexpr int STAGE = TILE_BYTES;   // bf16 elements of a stage: K tile, then V tile
    static constexpr int NSTAGE = 3;
    static constexpr int RS = D + 8;           // raw row / slab row stride (bf16)
    static constexpr int AS = D + 4;           // fp32 accumulator row stride
    static constexpr int PX_BYTES = NPAIR * 2 * U * 64 * 32;     // P hand-over, double buffered
    static constexpr size_t LDS_LIMIT = 160 * 1024;
    // raw = true: the q and dO rows the workgroup touches are copied to LDS; otherwise the
    // wavefronts read them from global memory once per unit
    static size_t main_bytes(int w2, bool raw) {
        const size_t rq = BQ + w2;
        return (size_t)NSTAGE * STAGE * 2 + PX_BYTES + (raw ? 2 * rq * RS * 2 : 0) + 2 * BQ * RS * 2 +
               2 * ((rq + 3) / 4 * 4) * 4 + rq * AS * 4;
    }
    static size_t final_bytes() { return (size_t)KW * BQ * AS * 4; }
    static size_t lds_bytes(int w2, bool raw) {
        return main_bytes(w2, raw) > final_bytes() ? main_bytes(w2, raw) : final_bytes();
    }
    static bool raw_fits(int w2) { return lds_bytes(w2, true) <= LDS_LIMIT; }
    static bool fits(int w2) { return lds_bytes(w2, false) <= LDS_LIMIT; }
};

// RAW = true: the q and dO rows the workgroup touches are copied to LDS; otherwise the
// wavefronts read them from global memory once per unit.
//
// LEFT = true: the pre-pass for window sizes that leave one unit over after the rounds of
// four (w2 + 1 = 4n + 1).  A workgroup takes four consecutive K' blocks, one per wavefront
// pair, and computes the unit delta = w2 of each in one shared sweep of K/V tiles.  Its
// results go where the main kernel (launched next with left = 1) picks them up: dK'
// and dV' in the element type in the output tensors, the dQ contribution as fp32 in rows
// w2 .. w2+31 of the block's dQ partial.  The main kernel then handles delta < w2.
//
// U = 2 (head_dim 32 and 64, where the registers allow it): a pair holds two consecutive deltas per round, so
// that every K and V operand read, every tile request and every step barrier serves twice the MFMAs.
//
// SEG = true: a K' window too wide for the dQ accumulator in LDS is cut into nseg runs of segw deltas, one
// workgroup per (K' block, segment); a kernel of its own so that the common case carries none of it.  Each writes its own dQ partial (rows k0 + seg*segw ..) and, when
// nseg > 1, fp32 partial dK' and dV' to `kpart` ([dV' | dK'][nseg][B*H][N][D]) for kp_sum_kernel.
template <class E, int D, bool RAW, bool LEFT, int U, bool SEG = false>
__global__ __launch_bounds__(KT) __attribute__((amdgpu_waves_per_eu(2, 2)))
void mfma_bwd_kp_kernel(Problem p, int nkb, int total, float* __restrict__ dq_part, int left, int nseg_arg, int segw_arg,
                        float* __restrict__ kpart) {
    typedef typename E::scalar EL;
    typedef typename E::x8 X8;
    constexpr bool raw = RAW;
    static_assert(!(RAW && LEFT), "the pre-pass keeps no row copies in LDS");
    static_assert(!LEFT || U == 1, "the pre-pass holds one unit per pair");
    static_assert(!SEG || (!LEFT && !RAW), "segments: main kernel, rows from global memory");
    using C = KpCfg<D, U>;
    constexpr int UPR = NPAIR * U;                            // units per round
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int nseg = SEG ? nseg_arg : 1, segw = SEG ? segw_arg : w2 + 1;
    const int w2s = segw - 1;                                 // deltas of a segment, minus one (w2 when there is one segment)
    const int RQ = BQ + w2s;                                  // query rows this workgroup touches
    uint16_t* smem = (uint16_t*)smem_raw;                     // stage ring
    unsigned char* px = smem_raw + (size_t)C::NSTAGE * C::STAGE * 2;
    uint16_t* q_s = (uint16_t*)(px + C::PX_BYTES);            // [RQ][RS] q rows kq .. (when raw)
    uint16_t* do_s = q_s + RQ * C::RS;                        // [RQ][RS] dO rows      (when raw)
    uint16_t* k2_s = raw ? do_s + RQ * C::RS : q_s;           // [BQ][RS] K' rows k0 ..
    uint16_t* v2_s = k2_s + BQ * C::RS;                       // [BQ][RS] V' rows
    const int RQ4 = (RQ + 3) & ~3;
    float* lse_s = (float*)(v2_s + BQ * C::RS);               // [RQ] LSE * log2(e)
    float* dsum_s = lse_s + RQ4;                              // [RQ] D_i
    float* dqacc = dsum_s + RQ4;                              // [RQ][AS]

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int role = wave >> 2, pr = wave & 3;                // role 0: P wavefront, 1: dS wavefront
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;

    // Launch order: all (K' block, head) pairs of segment 0, then those of segment 1, ...: the last segment
    // is the short one, and workgroups that alternate between long and short in launch order end up with
    // the long ones on half of the CUs (measured: twice the time).  Within a segment consecutive blocks go
    // to the same XCD.
    const int per_seg = SEG ? total / nseg : total;
    const int seg = SEG ? (int)blockIdx.x / per_seg : 0;
    int pb = SEG ? (int)blockIdx.x - seg * per_seg : (int)blockIdx.x;
    if ((per_seg & 7) == 0) pb = (pb & 7) * (per_seg >> 3) + (pb >> 3);
    // (in the pre-pass nkb counts groups of four K' blocks and k0 belongs to the pair)
    const int bh = pb / nkb, kb = LEFT ? (pb - bh * nkb) * NPAIR + pr : pb - bh * nkb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int k0 = kb * BQ;
    const int dlo = seg * segw;                               // first delta of the segment
    const int dhi = dlo + w2s < w2 ? dlo + w2s : w2;          // last one
    const int kq = k0 + dlo;                                  // query of K' row k0 at the segment's first delta
    const int k0_wg = LEFT ? (kb - pr) * BQ : k0;
    const int k0_end = LEFT ? k0_wg + NPAIR * BQ - 1 : k0 + BQ - 1;               // last K' row of the workgroup
    const int i_hi = (int)((int64_t)k0_end + dhi < N - 1 ? k0_end + dhi : N - 1);
    const int nkb_all = (N + BQ - 1) / BQ;
    if (LEFT && k0_wg + w2 > N - 1) return;          // none of the four blocks has the unit delta = w2

    const uint16_t* qp = (const uint16_t*)p.q.p + p.q.off(b, 0, h);
    const uint16_t* k1p = (const uint16_t*)p.k1.p + p.k1.off(b, 0, h);
    const uint16_t* k2p = (const uint16_t*)p.k2.p + p.k2.off(b, 0, h);
    const uint16_t* v1p = (const uint16_t*)p.v1.p + p.v1.off(b, 0, h);
    const uint16_t* v2p = (const uint16_t*)p.v2.p + p.v2.off(b, 0, h);
    const uint16_t* dop = (const uint16_t*)p.dout.p + p.dout.off(b, 0, h);

    const int i_lo = LEFT ? k0_wg + w2 : kq;                                      // first query of the workgroup
    const int jt_lo = (i_lo - w1 > 0 ? i_lo - w1 : 0) / TJ;
    const int jt_hi = i_hi / TJ;
    const int nt = jt_hi - jt_lo + 1;
    // the unit delta = w2 exists for this block and the pre-pass took it
    const bool has_left = left && !LEFT && k0 + w2 <= N - 1;
    const int nu_all = (w2 < N - 1 - k0 ? w2 : N - 1 - k0) + 1 - (has_left ? 1 : 0);      // units of the K' block
    const int n_units = !SEG ? nu_all : nu_all - dlo < segw ? nu_all - dlo : segw;                        // of this segment (may be <= 0)
    const int nrounds = LEFT ? 1 : (n_units + UPR - 1) / UPR;
    // Tiles a round sweeps: from the first tile of its smallest delta to the last tile of its
    // largest one (tile indices relative to jt_lo).
    auto round_first = [&](int round) {
        if (LEFT) return 0;
        const int i_min = kq + round * UPR;
        return (i_min - w1 > 0 ? i_min - w1 : 0) / TJ - jt_lo;
    };
    auto round_last = [&](int round) {
        if (LEFT) return nt - 1;
        const int dl = (round + 1) * UPR - 1 < n_units - 1 ? (round + 1) * UPR - 1 : n_units - 1;
        const int i_max = kq + dl + BQ - 1 < N - 1 ? kq + dl + BQ - 1 : N - 1;
        return i_max / TJ - jt_lo;
    };
    const bool want_dq = p.dq.p != nullptr;

    // ---- staging of one K/V tile: wavefront w requests group w of both tiles, straight into LDS
    const bool t_owner = wave < C::NGROUP;
    const int t_row = wave * C::RPW + (lane % C::RPW), t_col = lane / C::RPW;
    const uint32_t k_off = ((uint32_t)t_row * (uint32_t)p.k1.sn + t_col * 8) * 2u;
    const uint32_t v_off = ((uint32_t)t_row * (uint32_t)p.v1.sn + t_col * 8) * 2u;
    typedef __attribute__((address_space(3))) void* lds_ptr;
    typedef const __attribute__((address_space(1))) void* glb_ptr;
    auto dma_tile = [&](int jt, int stage) {
        const int j0 = jt * TJ;
        if (!t_owner) return;
        uint32_t ko = k_off, vo = v_off;
        if (__builtin_expect(j0 + TJ > N, 0)) {
            const int r = t_row < N - 1 - j0 ? t_row : N - 1 - j0;        // clamp (masked later)
            ko = ((uint32_t)r * (uint32_t)p.k1.sn + t_col * 8) * 2u;
            vo = ((uint32_t)r * (uint32_t)p.v1.sn + t_col * 8) * 2u;
        }
        const char* kbp = (const char*)(k1p + (int64_t)j0 * p.k1.sn);
        const char* vbp = (const char*)(v1p + (int64_t)j0 * p.v1.sn);
        unsigned char* dst = smem_raw + (size_t)stage * (C::STAGE * 2) + wave * C::GROUP;
        __builtin_amdgcn_global_load_lds((glb_ptr)(kbp + ko), (lds_ptr)dst, 16, 0, 0);
        __builtin_amdgcn_global_load_lds((glb_ptr)(vbp + vo), (lds_ptr)(dst + C::TILE_BYTES), 16, 0, 0);
    };

    // ---- raw rows, LSE, D and the dQ accumulator -------------------------------------
    if constexpr (!LEFT) {
        constexpr int CPR = D / 8;
        for (int c = tid; c < (raw ? RQ * CPR : 0); c += KT) {
            const int row = c / CPR, col = c - row * CPR;
            int r = kq + row;
            r = r < N ? r : N - 1;
            *(uint4*)(q_s + row * C::RS + col * 8) = *(const uint4*)(qp + (int64_t)r * p.q.sn + col * 8);
            *(uint4*)(do_s + row * C::RS + col * 8) = *(const uint4*)(dop + (int64_t)r * p.dout.sn + col * 8);
        }
        for (int c = tid; c < BQ * CPR; c += KT) {
            const int row = c / CPR, col = c - row * CPR;
            int r = k0 + row;
            r = r < N ? r : N - 1;
            *(uint4*)(k2_s + row * C::RS + col * 8) = *(const uint4*)(k2p + (int64_t)r * p.k2.sn + col * 8);
            *(uint4*)(v2_s + row * C::RS + col * 8) = *(const uint4*)(v2p + (int64_t)r * p.v2.sn + col * 8);
        }
        for (int c = tid; c < RQ; c += KT) {
            int r = kq + c;
            r = r < N ? r : N - 1;
            lse_s[c] = p.lse[(int64_t)bh * N + r] * LOG2E;
            dsum_s[c] = p.dsum[(int64_t)bh * N + r];
        }
        for (int c = tid; c < RQ * C::AS; c += KT) dqacc[c] = 0.f;
        if (has_left && p.dq.p) {
            // rows w2 .. w2+31 of the accumulator start from the pre-pass contribution
            __syncthreads();
            constexpr int CH = D / 4;
            const float* src = dq_part + (((int64_t)bh * nkb + kb) * RQ + w2) * D;
            for (int it = tid; it < BQ * CH; it += KT) {
                const int row = it / CH, c0 = (it - row * CH) * 4;
                *(float4*)(dqacc + (w2 + row) * C::AS + c0) = *(const float4*)(src + (int64_t)row * D + c0);
            }
        }
    }

    // q / dO row of query kq + rel: the LDS copy or (clamped) global memory
    auto q_row = [&](int rel) {
        if constexpr (RAW) {
            return (const uint16_t*)(q_s + rel * C::RS);
        } else {
            const int r = kq + rel < N ? kq + rel : N - 1;
            return qp + (int64_t)r * p.q.sn;
        }
    };
    auto do_row = [&](int rel) {
        if constexpr (RAW) {
            return (const uint16_t*)(do_s + rel * C::RS);
        } else {
            const int r = kq + rel < N ? kq + rel : N - 1;
            return dop + (int64_t)r * p.dout.sn;
        }
    };
    // K' / V' row k0 + ln of this pair's block
    const int kc = k0 + ln < N ? k0 + ln : N - 1;
    auto k2_row = [&]() {
        if constexpr (LEFT) return k2p + (int64_t)kc * p.k2.sn;
        else return (const uint16_t*)(k2_s + ln * C::RS);
    };
    auto v2_row = [&]() {
        if constexpr (LEFT) return v2p + (int64_t)kc * p.v2.sn;
        else return (const uint16_t*)(v2_s + ln * C::RS);
    };
    const float qscale = p.scale * LOG2E;
    const uint32_t smem_addr = lds_address(smem);
    const uint32_t px_addr = lds_address(px) + (uint32_t)(pr * 2 * U * 64 * 32 + lane * 32);
    const uint32_t row_lane = (uint32_t)((ln / C::RPW) * C::GROUP + (hf * C::RPW + ln % C::RPW) * 16);   // row operand
    const uint32_t col_lane = lds_group_column_lane_offset<C::RPW, C::GROUP>(lane);                      // transposed operand
    constexpr uint32_t KKB = 32 * C::RPW, DTB = 64 * C::RPW;      // operand strides of a k-step / a 32-column block
    constexpr uint32_t GA = C::row_off(16), GB = C::row_off(8);
    // all transposed operand reads of a tile (opaque reads, settled before use)
    auto issue_tr = [&](uint32_t a, lds_half_operand (&h)[4 * C::DT]) {
        lds_tr_issue<0, GB>(a, h[0], h[1]);
        lds_tr_issue<GA, GA + GB>(a, h[2], h[3]);
        if constexpr (C::DT >= 2) {
            lds_tr_issue<DTB, DTB + GB>(a, h[4], h[5]);
            lds_tr_issue<DTB + GA, DTB + GA + GB>(a, h[6], h[7]);
        }
        if constexpr (C::DT == 4) {
            lds_tr_issue<2 * DTB, 2 * DTB + GB>(a, h[8], h[9]);
            lds_tr_issue<2 * DTB + GA, 2 * DTB + GA + GB>(a, h[10], h[11]);
            lds_tr_issue<3 * DTB, 3 * DTB + GB>(a, h[12], h[13]);
            lds_tr_issue<3 * DTB + GA, 3 * DTB + GA + GB>(a, h[14], h[15]);
        }
    };

    // Step g works on ring stage g % 3 (the dS wavefronts also on the one before).  The tile of
    // step g+1 (the next one of this round, or the first one of the next round) is requested at
    // the start of step g and must have landed at its end.
    int g = 0, buf = 0;
    int next_round = 0, next_tile = round_first(0), next_last = round_last(0);
    auto next_request = [&](int stage) {
        if (next_round < nrounds) dma_tile(jt_lo + next_tile, stage);
        if (next_tile == next_last) {
            ++next_round;
            next_tile = round_first(next_round);
            next_last = round_last(next_round);
        } else {
            ++next_tile;
        }
    };
    next_request(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    auto begin_step = [&]() { next_request(buf + 1 == C::NSTAGE ? 0 : buf + 1); };
    auto advance = [&]() {
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        buf = buf + 1 == C::NSTAGE ? 0 : buf + 1;
        ++g;
    };

    // dV' (P wavefronts) or dK' (dS wavefronts) of this wavefront's deltas, rows k0+ln
    floatx16 pacc[C::DT];
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
        for (int v = 0; v < 16; ++v) pacc[dt][v] = 0.f;
    if (role == 0) {
        // =============================== P wavefronts ================================
        for (int round = 0; round < nrounds; ++round) {
            int delta[U], i_min[U], i_max[U], sa[U], sb[U];
            bool ok[U], row_ok[U], rows_full[U];
            floatx16 racc[U][C::DT];
            X8 qf[U][C::DK];
            floatx16 negl[U];
            const int i_of_lane = kq + ln;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                delta[u] = LEFT ? w2 : round * UPR + pr * U + u;
                ok[u] = LEFT ? (kb < nkb_all && k0 + w2 <= N - 1) : delta[u] < n_units;
                row_ok[u] = i_of_lane + delta[u] < N;
                i_min[u] = kq + delta[u];
                i_max[u] = (i_min[u] + BQ - 1 < N ? i_min[u] + BQ - 1 : N - 1);
                rows_full[u] = i_min[u] + BQ - 1 < N;
                sa[u] = ok[u] ? (i_min[u] - w1 > 0 ? i_min[u] - w1 : 0) / TJ - jt_lo : nt;     // first and last tile of the unit
                sb[u] = ok[u] ? i_max[u] / TJ - jt_lo : -1;
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                    for (int v = 0; v < 16; ++v) racc[u][dt][v] = 0.f;
                float lse2 = 0.f;
                {
                    const uint16_t* qrow = q_row(ln + delta[u]) + hf * 8;
                    const uint16_t* krow = k2_row() + hf * 8;
                    uint4 qav[C::DK], kxv[C::DK];       // all reads of the two rows first
#pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) qav[kk] = *(const uint4*)(qrow + kk * 16);
#pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) kxv[kk] = *(const uint4*)(krow + kk * 16);
#pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) {
                        const uint4 qa = qav[kk];
                        const uint4 kx = kxv[kk];
                        const uint32_t qw[4] = {qa.x, qa.y, qa.z, qa.w};
                        const uint32_t kw[4] = {kx.x, kx.y, kx.z, kx.w};
                        X8 r;
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            r[2 * t] = (EL)(E::lo(qw[t]) * (E::lo(kw[t]) + p.k2_bias) * qscale);
                            r[2 * t + 1] = (EL)(E::hi(qw[t]) * (E::hi(kw[t]) + p.k2_bias) * qscale);
                        }
                        qf[u][kk] = r;
                    }
                    const int iu = i_of_lane + delta[u];
                    if constexpr (LEFT) lse2 = p.lse[(int64_t)bh * N + (iu < N ? iu : N - 1)] * LOG2E;
                    else if (ok[u]) lse2 = lse_s[ln + delta[u]];
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) negl[u][v] = -lse2;
            }
            const int s_end = round_last(round);
            for (int s = round_first(round); s <= s_end; ++s) {
                begin_step();
                bool in[U];
                bool any = false;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    in[u] = s >= sa[u] && s <= sb[u];
                    any |= in[u];
                }
                if (any) {
                    const int j0 = (jt_lo + s) * TJ;
                    const uint32_t ks_addr = smem_addr + (uint32_t)(buf * C::STAGE) * 2u;
                    X8 ka[C::DK];
#pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) ka[kk] = lds_read_x8<X8>(ks_addr + row_lane + kk * KKB);
                    X8 pb[U][2];
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        if (!in[u]) continue;
                        floatx16 sh;
                        const bool plain = rows_full[u] && j0 + TJ - 1 <= i_min[u] && j0 >= i_max[u] - w1;
                        if (__builtin_expect(plain, 1)) {
                            sh = E::mfma(ka[0], qf[u][0], negl[u], 0, 0, 0);
                        } else {
                            asm volatile("" ::: "memory");
                            // element v of this lane is key j0 + 8*(v/4) + 4*hf + v%4
                            const int hi = i_of_lane + delta[u] - j0 - 4 * hf, lo = hi - w1;
                            floatx16 ct;
#pragma unroll
                            for (int v = 0; v < 16; ++v) {
                                const int c = 8 * (v >> 2) + (v & 3);
                                ct[v] = (row_ok[u] & (c <= hi) & (c >= lo)) ? negl[u][0] : -INFINITY;
                            }
                            sh = E::mfma(ka[0], qf[u][0], ct, 0, 0, 0);
                        }
#pragma unroll
                        for (int kk = 1; kk < C::DK; ++kk)
                            sh = E::mfma(ka[kk], qf[u][kk], sh, 0, 0, 0);
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                            for (int t = 0; t < 8; ++t) pb[u][ks][t] = (EL)fast_exp2(sh[ks * 8 + t]);
                    }
                    lds_half_operand vh[4 * C::DT];
                    issue_tr(ks_addr + (uint32_t)C::TILE_BYTES + col_lane, vh);
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        if (!in[u]) continue;
                        // opaque stores: the compiler would wait for the tile request in flight
                        const uint32_t a = px_addr + (uint32_t)(((g & 1) * U + u) * 64 * 32);
                        asm volatile("ds_write_b128 %0, %1\n\tds_write_b128 %0, %2 offset:16" ::"v"(a), "v"(pb[u][0]), "v"(pb[u][1]) : "memory");
                    }
                    lds_settle(vh);
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        if (!in[u]) continue;
#pragma unroll
                        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                            for (int ks = 0; ks < 2; ++ks)
                                racc[u][dt] = E::mfma(lds_join<X8>(vh[4 * dt + 2 * ks], vh[4 * dt + 2 * ks + 1]),
                                                      pb[u][ks], racc[u][dt], 0, 0, 0);
                    }
                }
                advance();
            }
            // dV'[k] += R[(k+delta, k)] * dO[k+delta]
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (!ok[u]) continue;
                const uint16_t* drow = do_row(ln + delta[u]) + 4 * hf;
                uint2 dx[4 * C::DT];               // the dO row, read in one batch
#pragma unroll
                for (int e = 0; e < 4 * C::DT; ++e) dx[e] = *(const uint2*)(drow + (e >> 2) * 32 + 8 * (e & 3));
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        const uint2 x = dx[4 * dt + g4];
                        pacc[dt][4 * g4 + 0] += racc[u][dt][4 * g4 + 0] * E::lo(x.x);
                        pacc[dt][4 * g4 + 1] += racc[u][dt][4 * g4 + 1] * E::hi(x.x);
                        pacc[dt][4 * g4 + 2] += racc[u][dt][4 * g4 + 2] * E::lo(x.y);
                        pacc[dt][4 * g4 + 3] += racc[u][dt][4 * g4 + 3] * E::hi(x.y);
                    }
            }
            if constexpr (LEFT) {
                // pre-pass: dV' of the unit goes to the output tensor as it is
                if (ok[0] && p.dv2.p && k0 + ln < N) {
                    uint16_t* dst = (uint16_t*)p.dv2.p + p.dv2.off(b, k0 + ln, h) + 4 * hf;
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                        for (int g4 = 0; g4 < 4; ++g4) {
                            union { EL hh[4]; uint2 u; } o;
#pragma unroll
                            for (int x = 0; x < 4; ++x) o.hh[x] = (EL)pacc[dt][4 * g4 + x];
                            *(uint2*)(dst + dt * 32 + 8 * g4) = o.u;
                        }
                }
                return;
            }
            if (want_dq) {
                // the dS wavefronts add their dQ contributions in four phases
                __syncthreads();
                __syncthreads();
                __syncthreads();
            }
        }
    } else {
        // =============================== dS wavefronts ===============================
        for (int round = 0; round < nrounds; ++round) {
            int delta[U], sa[U], sb[U];
            bool ok[U];
            floatx16 gacc[U][C::DT];
            X8 dof[U][C::DK];
            floatx16 dp_prev[U], negd[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                delta[u] = LEFT ? w2 : round * UPR + pr * U + u;
                ok[u] = LEFT ? (kb < nkb_all && k0 + w2 <= N - 1) : delta[u] < n_units;
                const int i_min = kq + delta[u];
                const int i_max = (i_min + BQ - 1 < N ? i_min + BQ - 1 : N - 1);
                sa[u] = ok[u] ? (i_min - w1 > 0 ? i_min - w1 : 0) / TJ - jt_lo : nt;
                sb[u] = ok[u] ? i_max / TJ - jt_lo : -1;
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                    for (int v = 0; v < 16; ++v) gacc[u][dt][v] = 0.f;
                float dsum = 0.f;
                {
                    const uint16_t* drow = do_row(ln + delta[u]) + hf * 8;
                    const uint16_t* vrow = v2_row() + hf * 8;
                    uint4 dav[C::DK], vxv[C::DK];       // all reads of the two rows first
#pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) dav[kk] = *(const uint4*)(drow + kk * 16);
#pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) vxv[kk] = *(const uint4*)(vrow + kk * 16);
#pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) {
                        const uint4 da = dav[kk];
                        const uint4 vx = vxv[kk];
                        const uint32_t dw[4] = {da.x, da.y, da.z, da.w};
                        const uint32_t vw[4] = {vx.x, vx.y, vx.z, vx.w};
                        X8 r;
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            r[2 * t] = (EL)(E::lo(dw[t]) * (E::lo(vw[t]) + p.v2_bias));
                            r[2 * t + 1] = (EL)(E::hi(dw[t]) * (E::hi(vw[t]) + p.v2_bias));
                        }
                        dof[u][kk] = r;
                    }
                    if constexpr (LEFT) dsum = p.dsum[(int64_t)bh * N + (i_min + ln < N ? i_min + ln : N - 1)];
                    else if (ok[u]) dsum = dsum_s[ln + delta[u]];
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) { dp_prev[u][v] = 0.f; negd[u][v] = -dsum; }
            }
            // dS of the tile handled in the previous step (tile index sp) and its G MFMAs
            auto consume = [&](int sp) {
                typedef const X8 __attribute__((address_space(3)))* lds_b8;
                X8 p0[U], p1[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t a = px_addr + (uint32_t)((((g - 1) & 1) * U + u) * 64 * 32);
                    p0[u] = *(lds_b8)(uintptr_t)a;
                    p1[u] = *(lds_b8)(uintptr_t)(a + 16);
                }
                const int pb = buf == 0 ? C::NSTAGE - 1 : buf - 1;
                lds_half_operand kh[4 * C::DT];
                issue_tr(smem_addr + (uint32_t)(pb * C::STAGE) * 2u + col_lane, kh);
                lds_settle(kh);
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (U > 1 && !(sp >= sa[u] && sp <= sb[u])) continue;
                    X8 dsb[2];
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        dsb[0][t] = (EL)((float)p0[u][t] * dp_prev[u][t]);
                        dsb[1][t] = (EL)((float)p1[u][t] * dp_prev[u][8 + t]);
                    }
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks)
                            gacc[u][dt] = E::mfma(lds_join<X8>(kh[4 * dt + 2 * ks], kh[4 * dt + 2 * ks + 1]),
                                                  dsb[ks], gacc[u][dt], 0, 0, 0);
                }
            };
            auto any_in = [&](int sx) {
                bool r = false;
#pragma unroll
                for (int u = 0; u < U; ++u) r |= sx >= sa[u] && sx <= sb[u];
                return r;
            };
            const int s_end = round_last(round);
            for (int s = round_first(round); s <= s_end; ++s) {
                begin_step();
                if (any_in(s - 1)) consume(s - 1);
                if (any_in(s)) {
                    const uint32_t vs_addr = smem_addr + (uint32_t)(buf * C::STAGE) * 2u + (uint32_t)C::TILE_BYTES;
                    X8 va[C::DK];
#pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) va[kk] = lds_read_x8<X8>(vs_addr + row_lane + kk * KKB);
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        if (!(s >= sa[u] && s <= sb[u])) continue;
                        dp_prev[u] = E::mfma(va[0], dof[u][0], negd[u], 0, 0, 0);
#pragma unroll
                        for (int kk = 1; kk < C::DK; ++kk)
                            dp_prev[u] = E::mfma(va[kk], dof[u][kk], dp_prev[u], 0, 0, 0);
                    }
                    if constexpr (U == 1) {
                        __builtin_amdgcn_sched_group_barrier(0x100, C::DK, 0);
                        __builtin_amdgcn_sched_group_barrier(0x008, C::DK, 0);
                    }
                }
                advance();
            }
            if (any_in(s_end)) consume(s_end);
            // dK'[k] += G[(k+delta, k)] * q[k+delta]   (scale applied at the end)
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (!ok[u]) continue;
                const uint16_t* qrow = q_row(ln + delta[u]) + 4 * hf;
                uint2 qx[4 * C::DT];               // the q row, read in one batch
#pragma unroll
                for (int e = 0; e < 4 * C::DT; ++e) qx[e] = *(const uint2*)(qrow + (e >> 2) * 32 + 8 * (e & 3));
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        const uint2 x = qx[4 * dt + g4];
                        pacc[dt][4 * g4 + 0] += gacc[u][dt][4 * g4 + 0] * E::lo(x.x);
                        pacc[dt][4 * g4 + 1] += gacc[u][dt][4 * g4 + 1] * E::hi(x.x);
                        pacc[dt][4 * g4 + 2] += gacc[u][dt][4 * g4 + 2] * E::lo(x.y);
                        pacc[dt][4 * g4 + 3] += gacc[u][dt][4 * g4 + 3] * E::hi(x.y);
                    }
            }
            if constexpr (LEFT) {
                // pre-pass: dK' of the unit goes to the output tensor, its dQ
                // contribution G * k2~ (unscaled) to rows w2 .. w2+31 of the block's dQ partial
                if (ok[0] && k0 + ln < N) {
                    if (p.dk2.p) {
                        uint16_t* dst = (uint16_t*)p.dk2.p + p.dk2.off(b, k0 + ln, h) + 4 * hf;
#pragma unroll
                        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                            for (int g4 = 0; g4 < 4; ++g4) {
                                union { EL hh[4]; uint2 u; } o;
#pragma unroll
                                for (int x = 0; x < 4; ++x) o.hh[x] = (EL)(p.scale * pacc[dt][4 * g4 + x]);
                                *(uint2*)(dst + dt * 32 + 8 * g4) = o.u;
                            }
                    }
                }
                if (ok[0] && want_dq) {
                    // (rows of keys past the end of the sequence carry zeros: their G is zero)
                    float* dst = dq_part + (((int64_t)bh * nkb_all + kb) * RQ + w2 + ln) * D + 4 * hf;
                    const uint16_t* krow = k2_row() + 4 * hf;
                    uint2 kx[4 * C::DT];           // the K' row, read in one batch
#pragma unroll
                    for (int e = 0; e < 4 * C::DT; ++e) kx[e] = *(const uint2*)(krow + (e >> 2) * 32 + 8 * (e & 3));
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                        for (int g4 = 0; g4 < 4; ++g4) {
                            const uint2 x = kx[4 * dt + g4];
                            float4 a;
                            a.x = gacc[0][dt][4 * g4 + 0] * (E::lo(x.x) + p.k2_bias);
                            a.y = gacc[0][dt][4 * g4 + 1] * (E::hi(x.x) + p.k2_bias);
                            a.z = gacc[0][dt][4 * g4 + 2] * (E::lo(x.y) + p.k2_bias);
                            a.w = gacc[0][dt][4 * g4 + 3] * (E::hi(x.y) + p.k2_bias);
                            *(float4*)(dst + dt * 32 + 8 * g4) = a;
                        }
                }
                return;
            }
            if (want_dq) {
                // dQ contribution of the units: dqacc[ln + delta][:] += G * k2~.  The four dS
                // wavefronts add into the shared fp32 accumulator (scale is applied when the
                // partial is written out) in four phases; in phase t
                // wavefront pr owns the 16-column blocks (pr + t) % 4 (and that + 4 when D = 128),
                // so no two wavefronts touch an element at the same time and every element
                // receives its contributions in a fixed order (a wavefront's units one after the other).
                auto add_dq = [&](auto PR, auto BIASED) {
                    constexpr int P0 = decltype(PR)::value;
                    constexpr bool WITH_BIAS = decltype(BIASED)::value;
                    const int tid_q = kp_recompute_here(threadIdx.x);
                    const int ln_q = tid_q & 31, hf_q = (tid_q >> 5) & 1;
                    const uint16_t* krow = k2_s + ln_q * C::RS + 4 * hf_q;      // (main kernel only)
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
#pragma unroll
                        for (int u = 0; u < U; ++u) {
                            if (!ok[u]) continue;
                            float* arow = dqacc + (ln_q + delta[u]) * C::AS + 4 * hf_q;
                            constexpr int NV = C::DK / 2;             // float4 slots of this phase
                            float4 a[NV];
                            uint2 x[NV];
                            // slot e of the phase -> 32-column tile dt and 8-column group g4 (D = 32
                            // has one tile: the four phases take its four groups)
                            auto slot_dt = [&](int e) { return D == 32 ? 0 : (((P0 + t) & 3) + 4 * (e >> 1)) >> 1; };
                            auto slot_g4 = [&](int e) {
                                return D == 32 ? ((P0 + t) & 3) : 2 * ((((P0 + t) & 3) + 4 * (e >> 1)) & 1) + (e & 1);
                            };
#pragma unroll
                            for (int e = 0; e < NV; ++e) {
                                const int col = slot_dt(e) * 32 + 8 * slot_g4(e);
                                x[e] = *(const uint2*)(krow + col);
                                a[e] = *(float4*)(arow + col);
                            }
                            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                            for (int e = 0; e < NV; ++e) {
                                const int dt = slot_dt(e), g4 = slot_g4(e);
                                const float kb = WITH_BIAS ? p.k2_bias : 0.f;
                                a[e].x += gacc[u][dt][4 * g4 + 0] * (E::lo(x[e].x) + kb);
                                a[e].y += gacc[u][dt][4 * g4 + 1] * (E::hi(x[e].x) + kb);
                                a[e].z += gacc[u][dt][4 * g4 + 2] * (E::lo(x[e].y) + kb);
                                a[e].w += gacc[u][dt][4 * g4 + 3] * (E::hi(x[e].y) + kb);
                                *(float4*)(arow + dt * 32 + 8 * g4) = a[e];
                            }
                            // (the second unit's rows overlap the first one's, shifted by one: its reads
                            // must see the first unit's writes, which the same lanes' program order does not
                            // give across lanes)
                            if constexpr (U > 1) __builtin_amdgcn_wave_barrier();
                        }
                        if (t < 3) __syncthreads();
                    }
                };
                auto add_dq_of = [&](auto BIASED) {
                    switch (pr) {
                        case 0: add_dq(std::integral_constant<int, 0>{}, BIASED); break;
                        case 1: add_dq(std::integral_constant<int, 1>{}, BIASED); break;
                        case 2: add_dq(std::integral_constant<int, 2>{}, BIASED); break;
                        default: add_dq(std::integral_constant<int, 3>{}, BIASED); break;
                    }
                };
                if (p.k2_bias != 0.f) add_dq_of(std::true_type{});
                else add_dq_of(std::false_type{});
            }
        }
    }

    // ---- dQ partial of this workgroup ------------------------------------------------
    const int tid_f = kp_recompute_here(threadIdx.x);
    __syncthreads();
    if (want_dq) {
        constexpr int CH = D / 4;
        float* dst = dq_part + (((int64_t)bh * nkb + kb) * nseg + seg) * RQ * D;
        for (int it = tid_f; it < RQ * CH; it += KT) {
            const int row = it / CH, c0 = (it - row * CH) * 4;
            float4 a = *(const float4*)(dqacc + row * C::AS + c0);
            a.x *= p.scale; a.y *= p.scale; a.z *= p.scale; a.w *= p.scale;
            *(float4*)(dst + (int64_t)row * D + c0) = a;
        }
    }
    __syncthreads();
    // ---- dK' and dV': add the four wavefronts of each role through LDS ----------------
    // item -> (tensor, K' row, 8 columns); a thread's items are it = tid, tid + KT, ...
    constexpr int CHF = D / 8;
    constexpr int ITEMS = (2 * BQ * CHF + KT - 1) / KT;
    // what the pre-pass left in the output rows (the contribution of the unit delta = w2),
    // requested now so that it arrives while the wavefronts' sums go through LDS
    uint4 pre[ITEMS];
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        pre[j] = make_uint4(0, 0, 0, 0);
        const int it = tid_f + j * KT;
        if (it < 2 * BQ * CHF && has_left) {
            const int which = it / (BQ * CHF);
            const int rem = it - which * BQ * CHF;
            const int row = rem / CHF, c0 = (rem - row * CHF) * 8;
            const Tensor& t = which ? p.dk2 : p.dv2;
            if (k0 + row < N && t.p) pre[j] = *(const uint4*)((const uint16_t*)t.p + t.off(b, k0 + row, h) + c0);
        }
    }
    {
        float* region = (float*)smem_raw + (size_t)wave * BQ * C::AS;
        const int ln_f = tid_f & 31, hf_f = (tid_f >> 5) & 1;
        float* rrow = region + ln_f * C::AS + 4 * hf_f;
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                float4 a;
                a.x = pacc[dt][4 * g4 + 0]; a.y = pacc[dt][4 * g4 + 1];
                a.z = pacc[dt][4 * g4 + 2]; a.w = pacc[dt][4 * g4 + 3];
                *(float4*)(rrow + dt * 32 + 8 * g4) = a;
            }
    }
    __syncthreads();
    {
        constexpr int CH = CHF;
        const float* base = (const float*)smem_raw;
#pragma unroll
        for (int j = 0; j < ITEMS; ++j) {
            const int it = tid_f + j * KT;
            if (it >= 2 * BQ * CH) break;
            const int which = it / (BQ * CH);                       // 0: dV' (P wavefronts), 1: dK'
            const int rem = it - which * BQ * CH;
            const int row = rem / CH, c0 = (rem - row * CH) * 8;
            const int k = k0 + row;
            const Tensor& t = which ? p.dk2 : p.dv2;
            if (k >= N || !t.p) continue;
            float acc[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) acc[c] = 0.f;
#pragma unroll
            for (int w = 0; w < NPAIR; ++w) {
                const float* rp = base + (size_t)(which * NPAIR + w) * BQ * C::AS + row * C::AS + c0;
                const float4 a = *(const float4*)rp, c4 = *(const float4*)(rp + 4);
                acc[0] += a.x; acc[1] += a.y; acc[2] += a.z; acc[3] += a.w;
                acc[4] += c4.x; acc[5] += c4.y; acc[6] += c4.z; acc[7] += c4.w;
            }
            const float sc = which ? p.scale : 1.f;
            if (nseg > 1) {
                float* dst = kpart + ((((int64_t)which * nseg + seg) * p.B * p.H + bh) * N + k) * D + c0;
                *(float4*)dst = make_float4(acc[0] * sc, acc[1] * sc, acc[2] * sc, acc[3] * sc);
                *(float4*)(dst + 4) = make_float4(acc[4] * sc, acc[5] * sc, acc[6] * sc, acc[7] * sc);
                continue;
            }
            uint16_t* dst = (uint16_t*)t.p + t.off(b, k, h) + c0;
            const uint4 x = pre[j];                                 // zeros where the pre-pass did not run
            const float part[8] = {E::lo(x.x), E::hi(x.x), E::lo(x.y), E::hi(x.y),
                                   E::lo(x.z), E::hi(x.z), E::lo(x.w), E::hi(x.w)};
            union { EL hh[8]; uint4 u; } o;
#pragma unroll
            for (int c = 0; c < 8; ++c) o.hh[c] = (EL)(acc[c] * sc + part[c]);
            *(uint4*)dst = o.u;
        }
    }
}

// dQ[i] = sum of the partials of the K' blocks that reach query i, in block order.
template <class E, int D>
__global__ __launch_bounds__(256) void mfma_bwd_dq_sum_kernel(Problem p, const float* __restrict__ dq_part, int nkb,
                                                             int64_t items, int nseg, int segw) {
    typedef typename E::scalar EL;
    constexpr int CH = D / 8;
    const int64_t it = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (it >= items) return;
    const int c0 = (int)(it % CH) * 8;
    const int64_t row = it / CH;
    const int N = p.N, RQ = BQ + p.w2;       // queries a K' block reaches
    const int RS = BQ + segw - 1;            // rows of one segment's partial
    const int i = (int)(row % N);
    const int bh = (int)(row / N);
    const int b = bh / p.H, h = bh - b * p.H;
    const int kb_hi = i / BQ;
    int kb_lo = (i - RQ + BQ) / BQ;              // smallest kb with i - 32*kb <= RQ-1
    kb_lo = (i - RQ + 1 <= 0) ? 0 : kb_lo;
    float acc[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = 0.f;
    if (nseg == 1) {
        for (int kb = kb_lo; kb <= kb_hi; ++kb) {
            const float* src = dq_part + (((int64_t)bh * nkb + kb) * RQ + (i - kb * BQ)) * D + c0;
            const float4 a = *(const float4*)src, c4 = *(const float4*)(src + 4);
            acc[0] += a.x; acc[1] += a.y; acc[2] += a.z; acc[3] += a.w;
            acc[4] += c4.x; acc[5] += c4.y; acc[6] += c4.z; acc[7] += c4.w;
        }
        kb_lo = kb_hi + 1;
    }
    for (int kb = kb_lo; kb <= kb_hi; ++kb) {
        const int rel = i - kb * BQ;             // row of the block's reach; segment s holds rel - s*segw in [0, RS)
        const int s_hi = rel / segw < nseg - 1 ? rel / segw : nseg - 1;
        const int s_lo = rel - RS + 1 <= 0 ? 0 : (rel - RS + segw) / segw;
        for (int sg = s_lo; sg <= s_hi; ++sg) {
            const float* src = dq_part + ((((int64_t)bh * nkb + kb) * nseg + sg) * RS + (rel - sg * segw)) * D + c0;
            const float4 a = *(const float4*)src, c4 = *(const float4*)(src + 4);
            acc[0] += a.x; acc[1] += a.y; acc[2] += a.z; acc[3] += a.w;
            acc[4] += c4.x; acc[5] += c4.y; acc[6] += c4.z; acc[7] += c4.w;
        }
    }
    union { EL hh[8]; uint4 u; } o;
#pragma unroll
    for (int c = 0; c < 8; ++c) o.hh[c] = (EL)acc[c];
    *(uint4*)((uint16_t*)p.dq.p + p.dq.off(b, i, h) + c0) = o.u;
}

// dK' and dV' from the fp32 partial sums of a segmented launch, segments added in their order
template <class E>
__global__ __launch_bounds__(256) void kp_sum_kernel(Problem p, int nseg, const float* __restrict__ kpart, int64_t chunks) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= chunks) return;
    const int D = p.D;
    const int col = (int)(c % (D / 4));
    const int64_t rowid = c / (D / 4);
    const int k = (int)(rowid % p.N);
    const int bh = (int)(rowid / p.N);
    const int b = bh / p.H, h = bh - b * p.H;
    const int64_t BH = (int64_t)p.B * p.H;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        const Tensor& t = which ? p.dk2 : p.dv2;
        if (!t.p) continue;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int sg = 0; sg < nseg; ++sg) {
            const float4 y = *(const float4*)(kpart + (((which * (int64_t)nseg + sg) * BH + bh) * p.N + k) * D + col * 4);
            acc.x += y.x; acc.y += y.y; acc.z += y.z; acc.w += y.w;
        }
        *(uint2*)((uint16_t*)t.p + t.off(b, k, h) + col * 4) = make_uint2(E::pack(acc.x, acc.y), E::pack(acc.z, acc.w));
    }
}

// Geometry of a launch: deltas per segment and number of segments (one while the dQ accumulator of the
// whole K' window fits LDS).  A pair holds two deltas per round at head_dim 32 and 64, one at 128.
struct KpPlan {
    int segw, nseg;
};
template <int D>
constexpr int kp_units() { return D <= 64 ? 2 : 1; }
template <int D>
KpPlan kp_plan_of(int w2) {
    using C = KpCfg<D, kp_units<D>()>;
    if (C::fits(w2)) return KpPlan{w2 + 1, 1};
    constexpr int UPR = NPAIR * kp_units<D>();
    int segw = UPR;
    while (C::fits(segw + UPR - 1)) segw += UPR;           // whole rounds per segment
    return KpPlan{segw, (w2 + segw) / segw};
}
KpPlan kp_plan(int D, int w2) { return D == 128 ? kp_plan_of<128>(w2) : D == 64 ? kp_plan_of<64>(w2) : kp_plan_of<32>(w2); }

size_t kp_dq_part_bytes(int B, int N, int H, int D, const KpPlan& pl) {
    const size_t nkb = (size_t)(N + BQ - 1) / BQ;
    return ((size_t)B * H * nkb * pl.nseg * (size_t)(BQ + pl.segw - 1) * D * sizeof(float) + 255) / 256 * 256;
}

template <class E, int D>
int launch_kp(const Problem& p, hipStream_t st) {
    constexpr int U = kp_units<D>();
    using C = KpCfg<D, U>;
    const KpPlan pl = kp_plan(D, p.w2);
    const int nkb = (p.N + BQ - 1) / BQ;
    const int64_t total = (int64_t)nkb * p.B * p.H * pl.nseg;
    if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    if ((p.dq.p || pl.nseg > 1) && p.scratch_bytes < kp_scratch_bytes(p.B, p.N, p.H, D, p.w2)) return SA2_ERR_WORKSPACE_TOO_SMALL;
    const int w2s = pl.segw - 1;
    const bool raw = pl.nseg == 1 && C::raw_fits(w2s);
    const size_t lds = C::lds_bytes(w2s, raw);
    float* part = (float*)p.scratch;
    float* kpart = (float*)((char*)p.scratch + kp_dq_part_bytes(p.B, p.N, p.H, D, pl));
    // one unit left over after the rounds of four: the pre-pass takes it
    // (unless the grid is so small that a further launch costs more than the lone round)
    const int left = (pl.nseg == 1 && p.w2 >= NPAIR && p.w2 % NPAIR == 0 && (p.force_prepass || total >= 768)) ? 1 : 0;
    if (left) {
        const size_t lds_left = (size_t)C::NSTAGE * C::STAGE * 2 + KpCfg<D, 1>::PX_BYTES;
        const int ngrp = (nkb + NPAIR - 1) / NPAIR;
        const int64_t total_left = (int64_t)ngrp * p.B * p.H;
        if (!allow_full_lds((const void*)mfma_bwd_kp_kernel<E, D, false, true, 1>)) return SA2_ERR_LAUNCH_FAILED;
        hipLaunchKernelGGL((mfma_bwd_kp_kernel<E, D, false, true, 1>), dim3((unsigned)total_left), dim3(KT), lds_left, st, p, ngrp,
                           (int)total_left, part, 0, 1, p.w2 + 1, (float*)nullptr);
        if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
    }
    if (pl.nseg > 1) {
        if (!allow_full_lds((const void*)mfma_bwd_kp_kernel<E, D, false, false, U, true>)) return SA2_ERR_LAUNCH_FAILED;
        hipLaunchKernelGGL((mfma_bwd_kp_kernel<E, D, false, false, U, true>), dim3((unsigned)total), dim3(KT), lds, st, p, nkb,
                           (int)total, part, left, pl.nseg, pl.segw, kpart);
    } else {
        const void* fn = raw ? (const void*)mfma_bwd_kp_kernel<E, D, true, false, U> : (const void*)mfma_bwd_kp_kernel<E, D, false, false, U>;
        if (!allow_full_lds(fn)) return SA2_ERR_LAUNCH_FAILED;
        if (raw) hipLaunchKernelGGL((mfma_bwd_kp_kernel<E, D, true, false, U>), dim3((unsigned)total), dim3(KT), lds, st, p, nkb, (int)total, part, left, 1, p.w2 + 1, kpart);
        else hipLaunchKernelGGL((mfma_bwd_kp_kernel<E, D, false, false, U>), dim3((unsigned)total), dim3(KT), lds, st, p, nkb, (int)total, part, left, 1, p.w2 + 1, kpart);
    }
    if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
    if (p.dq.p) {
        const int64_t items = (int64_t)p.B * p.H * p.N * (D / 8);
        hipLaunchKernelGGL((mfma_bwd_dq_sum_kernel<E, D>), dim3((unsigned)((items + 255) / 256)), dim3(256), 0, st, p, part,
                           nkb, items, pl.nseg, pl.segw);
        if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
    }
    if (pl.nseg > 1 && (p.dk2.p || p.dv2.p)) {
        const int64_t chunks = (int64_t)p.B * p.H * p.N * (D / 4);
        hipLaunchKernelGGL((kp_sum_kernel<E>), dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st, p, pl.nseg, kpart, chunks);
        if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
    }
    return SA2_OK;
}

}  // namespace

// workspace of the K'-side kernel: the dQ partials, then (segmented launches) the dK' and dV' partials
size_t kp_scratch_bytes(int B, int N, int H, int D, int w2) {
    const KpPlan pl = kp_plan(D, w2);
    return kp_dq_part_bytes(B, N, H, D, pl) + (pl.nseg > 1 ? (size_t)2 * pl.nseg * B * H * (size_t)N * D * sizeof(float) : 0);
}

int launch_mfma_bwd_kp(const Problem& p, int dtype, hipStream_t st) {
    if (dtype == SA2_F16)
        return p.D == 128 ? launch_kp<ElemF16, 128>(p, st) : p.D == 64 ? launch_kp<ElemF16, 64>(p, st) : launch_kp<ElemF16, 32>(p, st);
    return p.D == 128 ? launch_kp<ElemBF16, 128>(p, st) : p.D == 64 ? launch_kp<ElemBF16, 64>(p, st) : launch_kp<ElemBF16, 32>(p, st);
}

}  // namespace sa2
