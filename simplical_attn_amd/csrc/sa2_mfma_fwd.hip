// MFMA forward for gfx950 (bf16 or fp16 elements), head_dim 32, 64 or 128.
//
// Formulation: expand every query i by its K' window into rows r = (i, delta),
// delta = i - k in [0, w2], with Q~[r,:] = q[i,:] * (k2[i-delta,:] + k2_bias) *
// scale*log2(e), rounded to bf16.  Then s[r,j] = Q~[r].k1[j] and
// R[r,:] = sum_j p[r,j] v1[j,:] are sliding-window flash attention on the
// expanded rows (both contractions on v_mfma_f32_32x32x16_bf16 / _f16, fp32 softmax
// per row), and the rows of a query are merged with a second online softmax:
// O[i] = sum_delta e^{m_r-M} (v2[i-delta]+v2_bias) * R[r] / (L + 1e-8 e^{-M}).
// No logit outside the K' window is ever computed.
//
// Work split: one workgroup of 8 wavefronts (two per SIMD, so that one
// wavefront's softmax arithmetic overlaps the other's MFMAs) owns 32 consecutive
// queries of one (batch, head).  A "unit" is (delta, those 32 queries) = one
// 32-row MFMA N-tile; each wavefront holds one unit at a time and sweeps the K
// window [i0-w1, i0+31] in 32-key tiles that go straight from global memory into a
// four-stage LDS ring (global_load_lds, two steps ahead of their use) in a grouped
// layout that both the 16-byte K operand reads and the transposed V operand reads
// (ds_read_b64_tr_b16) take without bank conflicts.  The q rows of the block and the
// K'/V' rows its deltas reach are copied to LDS once.  A step issues the logit MFMAs
// of tile t between the softmax instructions of tile t-1, then the step's barrier (every
// LDS read of the step is complete by then), then the value MFMAs of tile t-1, which
// only read registers and so run under the next step's tile request and operand reads.
// A step is one basic block (mask and request are compile-time variants of it), so that
// the compiler can place all of this between the MFMAs.  At head_dim 128, after each round of 8 units the
// wavefronts fold their (m, l, R*v2) into the workgroup's fp32 accumulator through bf16 slabs in LDS,
// each thread summing a fixed slice in a fixed order.  At head_dim 32 and 64 the registers allow a
// second accumulator per wavefront: every wavefront keeps the running (m, l, sum of R*v2) of its own
// units, rounds follow each other without a barrier of their own, and the eight are merged once at the
// end through fp32 LDS in wavefront order.
//
// The logits are computed transposed (S^T = K1 . Q~^T) so that an expanded row
// lives in one lane pair: exp2(S^T) is already laid out as the B operand of
// R^T = V^T . P^T.  The softmax reference point of a unit is fixed at the first
// tile that holds one of its keys and enters the logit MFMA as its C operand, so
// on unmasked tiles the vector ALU only does exp2, bf16 packing and a row sum.
#include <type_traits>

#include "sa2_mfma_common.h"

namespace sa2 {
namespace {

constexpr int FW = 8;                 // wavefronts per workgroup

// The value of x behind a barrier the optimiser cannot see through: what is derived from it
// is computed where it is used instead of being kept in a register across the tile sweep.
__device__ __forceinline__ int recompute_here(int x) {
    asm volatile("" : "+v"(x));
    return x;
}
constexpr int FT = FW * 64;           // threads per workgroup

template <int D>
struct Cfg {
    static constexpr int DK = D / 16;          // k-steps of the logit contraction
    static constexpr int DT = D / 32;          // 32-column tiles of the value contraction
    static constexpr int KS = D + 8;           // row stride of the q / K' / V' copies in LDS (bf16)
    // Keys per K/V tile and sweep step, in 32-key halves.  (64-key tiles at head_dim 64, so that a step
    // holds 16 MFMAs per wavefront as at head_dim 128, measured the same forward time as 32-key tiles at
    // B2 H8 N2048 w 512/32 and cost 90 registers: 32 everywhere.)
    static constexpr int TK = 32;
    static constexpr int NSUB = TK / 32;
    // Head dims up to 64: every wavefront keeps the running softmax state and the output accumulator
    // of its units in registers (32 more at head_dim 64) and the eight are merged once at the end,
    // instead of a fold through LDS with three barriers after every round of eight units.
    static constexpr bool NOFOLD = D <= 64;
    // A K or V tile in LDS is written by direct global->LDS loads: one wavefront instruction
    // fills a group of RPW rows (1 KB), lane L putting the 16-byte chunk L / RPW of row
    // L % RPW at byte 16 * L.  Groups lie GROUP bytes apart.  Row operand reads and
    // transposed operand reads are both bank-conflict free in this layout.
    static constexpr int RPW = 512 / D;                     // rows per group: 4 (D = 128), 8 (D = 64), 16 (D = 32)
    // byte offset of row r of a tile (chunk 0)
    static constexpr int row_off(int r) { return (r / RPW) * GROUP + (r % RPW) * 16; }
    static constexpr int GROUP = 1024 + 16 * RPW;           // bytes
    static constexpr int NGROUP = TK / RPW;
    static constexpr int TILE_BYTES = NGROUP * GROUP;
    static constexpr int STAGE = TILE_BYTES;                // bf16 elements of one stage = K tile + V tile
    static constexpr int SS = D + 8;                        // slab row stride (bf16)
    static constexpr int OS = D + 4;                        // accumulator row stride (fp32)
    // LDS carve-up (bytes)
    static constexpr int NSTAGE = 4;
    static constexpr size_t STAGE_BYTES = (size_t)NSTAGE * STAGE * 2;
    static constexpr size_t SLAB_BYTES = (size_t)3 * BQ * SS * 2;          // three slabs; four more live in idle stage buffers
    static_assert(2 * BQ * SS <= STAGE, "two slabs must fit one stage buffer");
    static constexpr size_t OACC_BYTES = (size_t)BQ * OS * 4;
    static constexpr size_t XCH_BYTES = (size_t)(2 * FW * BQ + 3 * BQ) * 4;
    static constexpr size_t QS_BYTES = (size_t)BQ * KS * 2;
    static constexpr size_t BASE_BYTES = STAGE_BYTES + SLAB_BYTES + OACC_BYTES + XCH_BYTES + QS_BYTES;
    static constexpr size_t LDS_LIMIT = 160 * 1024;
    // rows of K' and V' kept in LDS: the 32 of the block plus the w2 before it
    static size_t side_bytes(int w2) { return (size_t)2 * (BQ + w2) * KS * 2; }
    static bool side_fits(int w2) { return BASE_BYTES + side_bytes(w2) <= LDS_LIMIT; }
    static size_t lds_bytes(int w2) { return BASE_BYTES + (side_fits(w2) ? side_bytes(w2) : 0); }
};

// SAFE = false: the fast kernel.  A weight that overflows (logits growing by more
// than ~100 octaves along the window after the reference point was fixed) only marks
// the block by storing NaN in its first LSE slot.
// SAFE = true: the repair kernel, launched right after: a block that finds the mark
// recomputes itself refreshing the reference point on every tile; every other block
// exits at once.
// MODE_LEFT: the pre-pass for window sizes that leave one unit over after the rounds of
// eight (w2 + 1 = 8n + 1).  A workgroup takes eight consecutive query blocks, one per
// wavefront, and computes the unit delta = w2 of each while sharing one sweep of K/V tiles.
// Nothing is merged across wavefronts: every query's partial result goes to `out` as
// R * (v2 + bias) / l in bf16 and to `lse` as m + log2(l); the fast kernel, launched next with
// left = 1, starts its accumulator from that pair and handles delta < w2 in full rounds.
constexpr int MODE_FAST = 0, MODE_SAFE = 1, MODE_LEFT = 2;
constexpr int PREPASS_MIN_WORKGROUPS = 768;      // three workgroups per CU

// Transposed V operand reads of a whole tile, item I of N = (32-key half h, 32-column block dt,
// k-step ks): rows 32h + 16ks + {0..7, 8..15} of columns 32dt .. 32dt+31, into vh[2I], vh[2I+1].
template <class C, int I, int N, int M>
__device__ __forceinline__ void issue_v_all(uint32_t addr, lds_half_operand (&vh)[M]) {
    if constexpr (I < N) {
        constexpr int h = I / (2 * C::DT), dt = (I / 2) % C::DT, ks = I % 2;
        constexpr int base = dt * 64 * C::RPW;
        lds_tr_issue<base + C::row_off(32 * h + 16 * ks), base + C::row_off(32 * h + 16 * ks + 8)>(addr, vh[2 * I], vh[2 * I + 1]);
        issue_v_all<C, I + 1, N>(addr, vh);
    }
}

// SIDE: the K' and V' rows the block's deltas reach are copied to LDS (they fit); otherwise
// they are read from global memory where they are needed.
template <class E, int D, int MODE, bool SIDE>
__global__ __launch_bounds__(FT) __attribute__((amdgpu_waves_per_eu(2, 2)))
void mfma_fwd_kernel(Problem p, int nqb, int total, int left) {
    typedef typename E::scalar EL;
    typedef typename E::x8 X8;
    typedef typename E::x2 X2;
    constexpr bool SAFE = MODE == MODE_SAFE, LEFT = MODE == MODE_LEFT;
    static_assert(!(LEFT && SIDE), "the pre-pass keeps no row copies in LDS");
    using C = Cfg<D>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t* smem = (uint16_t*)smem_raw;
    uint16_t* slabs = (uint16_t*)(smem_raw + C::STAGE_BYTES);
    float* oacc = (float*)(smem_raw + C::STAGE_BYTES + C::SLAB_BYTES);
    float* xch_m = oacc + BQ * C::OS;           // [FW][BQ]
    float* xch_l = xch_m + FW * BQ;             // [FW][BQ]
    float* lam_s = xch_l + FW * BQ;             // [BQ] reference point of the pre-pass partial
    float* fin_m = lam_s + BQ;                  // [BQ] final M
    float* fin_l = fin_m + BQ;                  // [BQ] final L
    uint16_t* q_s = (uint16_t*)(fin_l + BQ);    // [BQ][KS] q rows of the block
    uint16_t* k2_s = q_s + BQ * C::KS;          // [BQ + w2][KS] K' rows i0-w2 .. i0+31 (when SIDE)

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;

    // Workgroups are dealt round-robin to the 8 XCDs; remap so that the
    // neighbouring query blocks of one head (which share almost all of their
    // K/V window) run on the same XCD and meet in its L2.
    int pid = blockIdx.x;
    if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
    // (in the pre-pass nqb counts groups of eight query blocks)
    const int bh = pid / nqb, qb = LEFT ? (pid - bh * nqb) * FW + wave : pid - bh * nqb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int i0 = qb * BQ;                      // per wavefront in the pre-pass
    const int i0_wg = LEFT ? (qb - wave) * BQ : i0;
    const int i = i0 + ln;
    const int ic = i < N ? i : N - 1;
    const int i_last = (i0 + BQ - 1 < N ? i0 + BQ - 1 : N - 1);
    if (SAFE) {
        const float mark = p.lse[(int64_t)bh * N + i0];
        if (mark == mark) return;                 // not NaN: the fast kernel's result stands
    }

    const uint16_t* qp = (const uint16_t*)p.q.p + p.q.off(b, 0, h);
    const uint16_t* k1p = (const uint16_t*)p.k1.p + p.k1.off(b, 0, h);
    const uint16_t* k2p = (const uint16_t*)p.k2.p + p.k2.off(b, 0, h);
    const uint16_t* v1p = (const uint16_t*)p.v1.p + p.v1.off(b, 0, h);
    const uint16_t* v2p = (const uint16_t*)p.v2.p + p.v2.off(b, 0, h);

    constexpr int TJ = C::TK;                    // keys per tile in this kernel
    const int jt_lo = (i0_wg - w1 > 0 ? i0_wg - w1 : 0) / TJ;
    const int jt_hi = LEFT ? (i0_wg + FW * BQ - 1 < N - 1 ? i0_wg + FW * BQ - 1 : N - 1) / TJ : i_last / TJ;
    const int nt = jt_hi - jt_lo + 1;
    // delta = 0 .. n_units-1; the fast kernel leaves delta = w2 to the pre-pass where that ran
    const bool has_left = left && i_last >= w2;
    const int n_units = LEFT ? 1 : (w2 < i_last ? w2 : i_last) + 1 - (has_left && !SAFE ? 1 : 0);
    const int nrounds = (n_units + FW - 1) / FW;
    const int total_steps = nrounds * nt;
    // tiles of the sweep that hold keys of this wavefront's rows (the whole sweep outside the pre-pass)
    const int ws0 = LEFT ? (i0 - w1 > 0 ? i0 - w1 : 0) / TJ - jt_lo : 0;
    const int ws1 = LEFT ? (i_last < 0 ? 0 : i_last) / TJ - jt_lo : nt - 1;

    // ---- staging of one K/V tile: direct global -> LDS loads ------------------------
    // Wavefront w fills group w of the K tile and of the V tile (the first NGROUP wavefronts
    // when D = 64).  Tiles are requested strictly in sweep order into consecutive ring stages.
    const bool t_owner = wave < C::NGROUP;
    const int t_row = wave * C::RPW + (lane % C::RPW), t_col = lane / C::RPW;
    const uint32_t k_off = ((uint32_t)t_row * (uint32_t)p.k1.sn + t_col * 8) * 2u;
    const uint32_t v_off = ((uint32_t)t_row * (uint32_t)p.v1.sn + t_col * 8) * 2u;
    // the same for the tile that holds the end of the sequence: rows past it are clamped to the
    // last one (they are masked later)
    const int jt_end = (N - 1) / TJ;
    const int t_row_c = t_row < N - 1 - jt_end * TJ ? t_row : N - 1 - jt_end * TJ;
    const uint32_t k_off_c = ((uint32_t)t_row_c * (uint32_t)p.k1.sn + t_col * 8) * 2u;
    const uint32_t v_off_c = ((uint32_t)t_row_c * (uint32_t)p.v1.sn + t_col * 8) * 2u;
    typedef __attribute__((address_space(3))) void* lds_ptr;
    typedef const __attribute__((address_space(1))) void* glb_ptr;
    int dma_tile = 0, dma_stage = 0, dma_count = 0;             // next tile (from jt_lo), its stage, tiles requested
    // (no branch in here when every wavefront owns a group, so that the request can be scheduled
    // into the middle of a step's arithmetic)
    auto dma_next = [&]() {
        const int j0 = (jt_lo + dma_tile) * TJ;
        if (C::NGROUP >= FW || t_owner) {
            const bool at_end = jt_lo + dma_tile == jt_end;
            const uint32_t ko = at_end ? k_off_c : k_off, vo = at_end ? v_off_c : v_off;
            const char* kb = (const char*)(k1p + (int64_t)j0 * p.k1.sn);
            const char* vb = (const char*)(v1p + (int64_t)j0 * p.v1.sn);
            unsigned char* dst = smem_raw + (size_t)dma_stage * (C::STAGE * 2) + wave * C::GROUP;
            __builtin_amdgcn_global_load_lds((glb_ptr)(kb + ko), (lds_ptr)dst, 16, 0, 0);
            __builtin_amdgcn_global_load_lds((glb_ptr)(vb + vo), (lds_ptr)(dst + C::TILE_BYTES), 16, 0, 0);
        }
        dma_tile = dma_tile + 1 == nt ? 0 : dma_tile + 1;
        dma_stage = (dma_stage + 1) & (C::NSTAGE - 1);
        ++dma_count;
    };

    // ---- workgroup accumulators ------------------------------------------------
    // thread -> (query aq, ACN columns from ac) of the fp32 accumulator in LDS
    constexpr int ACN = D / 16;                    // columns per thread (8, 4 or 2)
    bool bad = false;
    if constexpr (!LEFT) {
        // running maximum and sum of every query: fin_m / fin_l in LDS, read and updated at the
        // merges.  Where the pre-pass ran the accumulator starts from its partial result, which
        // enters the first merge with weight 1 at its own reference point m + log2 l.
        const int aq = tid >> 4, ac = (tid & 15) * ACN;
        const int io = i0 + aq < N ? i0 + aq : N - 1;
        if (has_left && !SAFE) {
            const uint16_t* prow = (const uint16_t*)p.out.p + p.out.off(b, io, h) + ac;
            uint32_t pw[ACN / 2];
            load_words(prow, pw);
            float* o = oacc + aq * C::OS + ac;
#pragma unroll
            for (int c = 0; c < ACN / 2; ++c) {
                o[2 * c] = E::lo(pw[c]);
                o[2 * c + 1] = E::hi(pw[c]);
            }
            if (tid < BQ) {
                const int it = i0 + tid < N ? i0 + tid : N - 1;
                const float lam = p.lse[(int64_t)bh * N + it];
                bad = !(lam == lam);                           // the pre-pass overflowed: repair the block
                lam_s[tid] = lam;
            }
        } else {
#pragma unroll
            for (int c = 0; c < ACN; ++c) oacc[aq * C::OS + ac + c] = 0.f;
        }
        if (tid < BQ) {
            fin_m[tid] = -INFINITY;
            fin_l[tid] = 0.f;
        }
    }

    // the first two tiles are requested before anything else so that their latency overlaps
    // the copies below
    dma_next();
    if (total_steps > 1) dma_next();

    // ---- q rows of the block and the K'/V' rows its deltas reach, once, to LDS ----
    const int side_rows = BQ + w2;
    uint16_t* v2_s = k2_s + side_rows * C::KS;
    if constexpr (!LEFT) {
        constexpr int CPR = D / 8;                 // 16-byte chunks per row
        for (int c = tid; c < BQ * CPR; c += FT) {
            const int row = c / CPR, col = c - row * CPR;
            int r = i0 + row;
            r = r < N ? r : N - 1;
            *(uint4*)(q_s + row * C::KS + col * 8) = *(const uint4*)(qp + (int64_t)r * p.q.sn + col * 8);
        }
        if constexpr (SIDE) {
            for (int c = tid; c < side_rows * CPR; c += FT) {
                const int row = c / CPR, col = c - row * CPR;
                int r = i0 - w2 + row;
                r = r < 0 ? 0 : (r < N ? r : N - 1);
                *(uint4*)(k2_s + row * C::KS + col * 8) = *(const uint4*)(k2p + (int64_t)r * p.k2.sn + col * 8);
                *(uint4*)(v2_s + row * C::KS + col * 8) = *(const uint4*)(v2p + (int64_t)r * p.v2.sn + col * 8);
            }
        }
    }
    // K'/V' row of this lane's query for a given delta: LDS copy or global memory
    auto k2_row = [&](int delta) {
        if constexpr (SIDE) {
            return (const uint16_t*)(k2_s + (ln + w2 - delta) * C::KS);       // row (i0 + ln - delta) - (i0 - w2)
        } else {
            const int k = ic - delta;
            return k2p + (int64_t)(k > 0 ? k : 0) * p.k2.sn;
        }
    };

    const float qscale = p.scale * LOG2E;
    // LDS byte addresses: the stage ring, this lane's part of a K operand read (row ln, k-slots of
    // its half) and of a transposed V operand read
    const uint32_t smem_addr = lds_address(smem);
    const uint32_t k_lane = (uint32_t)((ln / C::RPW) * C::GROUP + (hf * C::RPW + ln % C::RPW) * 16);
    const uint32_t v_lane = lds_group_column_lane_offset<C::RPW, C::GROUP>(lane);

    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    // Tiles [s_lo, s_hi] need no mask: every key of the tile is inside the K window of
    // every query of the block.
    int s_lo = (i0 + BQ - 1 - w1 + TJ - 1) / TJ - jt_lo;       // first tile with j0 >= i0+31-w1
    s_lo = (i0 + BQ - 1 - w1 <= jt_lo * TJ) ? 0 : s_lo;
    const int s_hi = (i0 + 1) / TJ - 1 - jt_lo;                 // last tile with j0+31 <= i0

    // Step g of the sweep works on ring stage g % NSTAGE.  At its start the tile of step g+2 is
    // requested (the stage it goes to was last read in step g-2); at its end the tile of step
    // g+1 must have landed.  Requests run on across rounds, so between two rounds the ring
    // holds the first tile of the next round, has its second one in flight, and two stages
    // are free for the merge.
    int g = 0, buf = 0;                                         // buf = g % NSTAGE
    bool requested = false;
    auto begin_step = [&](int) {
        requested = dma_count < total_steps;
        if (requested) dma_next();
    };
    auto advance = [&]() {
        if (requested) asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
        buf = (buf + 1) & (C::NSTAGE - 1);
        ++g;
    };

    // (NOFOLD) this wavefront's running result over its units: reference exponent and sum of every
    // row, output accumulator in the layout of the value MFMAs' result
    float Mw = -INFINITY, Lw = 0.f;
    floatx16 wacc[C::NOFOLD ? C::DT : 1];
    if constexpr (C::NOFOLD) {
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int v = 0; v < 16; ++v) wacc[dt][v] = 0.f;
    }

    for (int round = 0; round < nrounds; ++round) {
        const int delta = LEFT ? w2 : round * FW + wave;
        const bool ok = LEFT ? (i0 < N && i_last >= w2) : delta < n_units;
        // The unit starts from the query's running reference point (finite from the second
        // round on, or from the first where the pre-pass ran), so only then it looks for maxima.
        float m = -INFINITY, l = 0.f;
        if constexpr (!LEFT) m = C::NOFOLD ? Mw : (ok ? fin_m[ln] : -INFINITY);
        floatx16 racc[C::DT];
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int v = 0; v < 16; ++v) racc[dt][v] = 0.f;

        if (!ok) {
            // no unit for this wavefront in this round: keep the staging pipeline moving
            for (int s = 0; s < nt; ++s) {
                begin_step(s);
                advance();
            }
        } else {
            // ---- new unit: Q~ operand, fresh softmax state ----------------------
            X8 qf[C::DK];
            {
                const uint16_t* krow = k2_row(delta) + hf * 8;
                const uint16_t* qrow;
                if constexpr (LEFT) qrow = qp + (int64_t)ic * p.q.sn + hf * 8;
                else qrow = q_s + ln * C::KS + hf * 8;
                // (all reads of the two rows first: from global memory they overlap)
                uint4 qav[C::DK], kbv[C::DK];
#pragma unroll
                for (int kk = 0; kk < C::DK; ++kk) kbv[kk] = *(const uint4*)(krow + kk * 16);
#pragma unroll
                for (int kk = 0; kk < C::DK; ++kk) qav[kk] = *(const uint4*)(qrow + kk * 16);
                auto form_q = [&](auto BIASED) {
                    const float kbias = decltype(BIASED)::value ? p.k2_bias : 0.f;
#pragma unroll
                    for (int kk = 0; kk < C::DK; ++kk) {
                        const uint4 qa = qav[kk];
                        const uint4 kb = kbv[kk];
                        const uint32_t qw[4] = {qa.x, qa.y, qa.z, qa.w};
                        const uint32_t kw[4] = {kb.x, kb.y, kb.z, kb.w};
                        X8 r;
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            r[2 * t] = (EL)(E::lo(qw[t]) * qscale * (E::lo(kw[t]) + kbias));
                            r[2 * t + 1] = (EL)(E::hi(qw[t]) * qscale * (E::hi(kw[t]) + kbias));
                        }
                        qf[kk] = r;
                    }
                };
                if (p.k2_bias != 0.f) form_q(std::true_type{});
                else form_q(std::false_type{});
            }
            const bool rows_full = i0 >= delta && i0 + BQ - 1 < N;
            const bool row_ok = i < N && i >= delta;
            // -m (0 while the row has no finite logit yet), as a scalar and replicated over an
            // accumulator tuple: the tuple is the C operand of the first logit MFMA.
            float nm = (m == -INFINITY) ? 0.f : -m;    // (first round: fixed before the sweep)
            floatx16 negm;
#pragma unroll
            for (int v = 0; v < 16; ++v) negm[v] = nm;

            // exp2 of the shifted logits -> bf16 weights (MFMA B operand) and their row sum
            auto weights = [&](const floatx16& sh, X8* w, float& rsum) {
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                    for (int t = 0; t < 8; ++t) w[ks][t] = (EL)fast_exp2(sh[ks * 8 + t]);
                const X2 ones = {(EL)1.f, (EL)1.f};
                float r = 0.f;
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    r = E::dot2(__builtin_shufflevector(w[ks], w[ks], 0, 1), ones, r, false);
                    r = E::dot2(__builtin_shufflevector(w[ks], w[ks], 2, 3), ones, r, false);
                    r = E::dot2(__builtin_shufflevector(w[ks], w[ks], 4, 5), ones, r, false);
                    r = E::dot2(__builtin_shufflevector(w[ks], w[ks], 6, 7), ones, r, false);
                }
                rsum = r;
            };
            constexpr uint32_t KKB = 32 * C::RPW, DTB = 64 * C::RPW;      // operand strides of a k-step / a 32-column block
            auto stage_addr = [&](int st) { return smem_addr + (uint32_t)st * (uint32_t)(C::STAGE * 2); };
            constexpr uint32_t SUBB = C::row_off(32 % C::TK);                   // byte offset of a tile's second 32-key half
            // logits of the 32-key half `h` of the tile at ks_addr
            auto logit_mfmas = [&](uint32_t ks_addr, int h, floatx16 c) -> floatx16 {
#pragma unroll
                for (int kk = 0; kk < C::DK; ++kk) {
                    const X8 ka = lds_read_x8<X8>(ks_addr + k_lane + h * SUBB + kk * KKB);
                    c = E::mfma(ka, qf[kk], c, 0, 0, 0);
                }
                return c;
            };
            // all transposed V operand reads of a tile (opaque reads, settled before use):
            // vh[((h * DT + dt) * 2 + ks) * 2 + {0, 1}] = the two halves of the operand of half h,
            // 32-column block dt, k-step ks
            auto issue_v = [&](uint32_t vt_addr, lds_half_operand (&vh)[4 * C::DT * C::NSUB]) {
                issue_v_all<C, 0, 2 * C::DT * C::NSUB>(vt_addr, vh);
            };
            // value MFMAs of a whole tile: w[2 * h + ks] = the weights of half h, k-step ks
            auto value_mfmas = [&](uint32_t vt_addr, const X8* w) {
                lds_half_operand vh[4 * C::DT * C::NSUB];
                issue_v(vt_addr, vh);
                lds_settle(vh);
#pragma unroll
                for (int h = 0; h < C::NSUB; ++h)
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks) {
                            const int x = ((h * C::DT + dt) * 2 + ks) * 2;
                            const X8 va = lds_join<X8>(vh[x], vh[x + 1]);
                            racc[dt] = E::mfma(va, w[2 * h + ks], racc[dt], 0, 0, 0);
                        }
            };

            // Mask of a tile as the C operand of its logit MFMAs: -m where the key is inside
            // the window of the row, -inf elsewhere.  Element v of this lane is key
            // j0 + 8*(v/4) + 4*hf + v%4.
            auto masked_c = [&](int j0) -> floatx16 {
                const int hi = i - j0 - 4 * hf, lo = hi - w1;
                floatx16 ct;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int c = 8 * (v >> 2) + (v & 3);
                    const bool valid = row_ok & (c <= hi) & (c >= lo);
                    ct[v] = valid ? nm : -INFINITY;
                }
                return ct;
            };
            auto tile_plain = [&](int s) {
                return rows_full && s >= s_lo && s <= s_hi;
            };

            if (SAFE) {
                // ---- repair pass: the reference point follows the maxima on every tile ----
                for (int s = 0; s < nt; ++s) {
                    begin_step(s);
                    const uint32_t Ks = stage_addr(buf);
                    const bool plain = tile_plain(s);
                    floatx16 t[C::NSUB];
                    float mx = -INFINITY;
#pragma unroll
                    for (int h = 0; h < C::NSUB; ++h) {
                        const int j0 = (jt_lo + s) * TJ + 32 * h;
                        const int hi = i - j0 - 4 * hf, lo = hi - w1;
#pragma unroll
                        for (int v = 0; v < 16; ++v) t[h][v] = 0.f;
                        t[h] = logit_mfmas(Ks, h, t[h]);
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int c = 8 * (v >> 2) + (v & 3);
                            const bool valid = plain | (row_ok & (c <= hi) & (c >= lo));
                            t[h][v] = valid ? t[h][v] : -INFINITY;
                            mx = fmaxf(mx, t[h][v]);
                        }
                    }
                    mx = fmaxf(mx, other_half(mx));
                    const float m_new = fmaxf(m, mx);
                    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
                    const float alpha = fast_exp2(m - m_use);
                    m = m_new;
                    l *= alpha;
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                        for (int v = 0; v < 16; ++v) racc[dt][v] *= alpha;
                    X8 pb[2 * C::NSUB];
#pragma unroll
                    for (int h = 0; h < C::NSUB; ++h) {
#pragma unroll
                        for (int v = 0; v < 16; ++v) t[h][v] -= m_use;
                        float rs;
                        weights(t[h], pb + 2 * h, rs);
                        l += rs;
                    }
                    value_mfmas(Ks + C::TILE_BYTES + v_lane, pb);
                    advance();
                }
            } else {
                // ---- reference point: the query's running one, or (first round) the maximum of
                // the first tile, or 0 for a row with no key there.  Any finite reference is
                // exact as long as no weight overflows, which `bad` watches.
                for (int s = 0; s < ws0; ++s) {           // (pre-pass) tiles before this wavefront's window
                    begin_step(s);
                    advance();
                }
                if (__builtin_amdgcn_ballot_w64(m == -INFINITY) != 0) {
                    float mx = -INFINITY;
#pragma unroll
                    for (int h = 0; h < C::NSUB; ++h) {
                        const int j0 = (jt_lo + ws0) * TJ + 32 * h;
                        const int hi = i - j0 - 4 * hf, lo = hi - w1;
                        floatx16 t;
#pragma unroll
                        for (int v = 0; v < 16; ++v) t[v] = 0.f;
                        t = logit_mfmas(stage_addr(buf), h, t);
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            const int c = 8 * (v >> 2) + (v & 3);
                            const bool valid = row_ok & (c <= hi) & (c >= lo);
                            mx = fmaxf(mx, valid ? t[v] : -INFINITY);
                        }
                    }
                    mx = fmaxf(mx, other_half(mx));
                    if (m == -INFINITY) m = (mx == -INFINITY) ? 0.f : mx;
                    nm = -m;
#pragma unroll
                    for (int v = 0; v < 16; ++v) negm[v] = nm;
                }
                // ---- two-stage software pipeline over the tiles: step t issues the logit MFMAs
                // of tile t between the softmax instructions of tile t-1, then the value MFMAs
                // of tile t-1; the shifted logits of tile t wait in registers for step t+1.
                floatx16 sh_a[C::NSUB], sh_b[C::NSUB];
                {
                    const bool plain0 = tile_plain(ws0);
                    begin_step(ws0);
#pragma unroll
                    for (int h = 0; h < C::NSUB; ++h)
                        sh_a[h] = logit_mfmas(stage_addr(buf), h, plain0 ? negm : masked_c((jt_lo + ws0) * TJ + 32 * h));
                }
                uint32_t vt_prev = stage_addr(buf) + (uint32_t)C::TILE_BYTES + v_lane;
                advance();
                // One step: logits of tile s into `cur`, weights and value MFMAs of tile s-1 from `prev`.
                // PLAIN: the tile needs no mask.  DMA: the step requests a tile (all but the last
                // two steps of the kernel do).  Both are compile-time so that a step is one
                // basic block: the request's scalar arithmetic and the loads then sit between the
                // MFMAs instead of in front of them, where both wavefronts of a SIMD would wait.
                auto step = [&](int s, const floatx16 (&prev)[C::NSUB], floatx16 (&cur)[C::NSUB], auto PLAIN_TAG, auto DMA_TAG) {
                    constexpr bool PLAIN = decltype(PLAIN_TAG)::value, DMA = decltype(DMA_TAG)::value;
                    const uint32_t ks_addr = stage_addr(buf);
                    X8 ka[C::NSUB][C::DK];
#pragma unroll
                    for (int h = 0; h < C::NSUB; ++h)
#pragma unroll
                        for (int kk = 0; kk < C::DK; ++kk) ka[h][kk] = lds_read_x8<X8>(ks_addr + k_lane + h * SUBB + kk * KKB);
                    // the reference point (and, on the window-edge tiles, the mask) is the
                    // C operand of the first logit MFMA
                    if constexpr (PLAIN) cur[0] = E::mfma(ka[0][0], qf[0], negm, 0, 0, 0);
                    else cur[0] = E::mfma(ka[0][0], qf[0], masked_c((jt_lo + s) * TJ), 0, 0, 0);
                    if constexpr (DMA) dma_next();
                    lds_half_operand vh[4 * C::DT * C::NSUB];
                    issue_v(vt_prev, vh);
                    X8 pb[2 * C::NSUB];
#pragma unroll
                    for (int kk = 1; kk < C::DK; ++kk)
                        cur[0] = E::mfma(ka[0][kk], qf[kk], cur[0], 0, 0, 0);
#pragma unroll
                    for (int h = 1; h < C::NSUB; ++h) {
                        if constexpr (PLAIN) cur[h] = E::mfma(ka[h][0], qf[0], negm, 0, 0, 0);
                        else cur[h] = E::mfma(ka[h][0], qf[0], masked_c((jt_lo + s) * TJ + 32 * h), 0, 0, 0);
#pragma unroll
                        for (int kk = 1; kk < C::DK; ++kk)
                            cur[h] = E::mfma(ka[h][kk], qf[kk], cur[h], 0, 0, 0);
                    }
#pragma unroll
                    for (int h = 0; h < C::NSUB; ++h) {
                        float rs;
                        weights(prev[h], pb + 2 * h, rs);
                        l += rs;
                        bad |= !(rs < E::WEIGHT_LIMIT);
                    }
                    asm volatile("" : "+v"(pb[0]));              // (the wait below stays behind the first weights)
                    lds_settle(vh);
                    // The barrier stands in front of the value MFMAs: they only read registers.
                    vt_prev = ks_addr + (uint32_t)C::TILE_BYTES + v_lane;
                    if constexpr (DMA) asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
                    buf = (buf + 1) & (C::NSTAGE - 1);
                    ++g;
#pragma unroll
                    for (int h = 0; h < C::NSUB; ++h)
#pragma unroll
                        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                            for (int dt = 0; dt < C::DT; ++dt) {
                                const int x = ((h * C::DT + dt) * 2 + ks) * 2;
                                const X8 va = lds_join<X8>(vh[x], vh[x + 1]);
                                racc[dt] = E::mfma(va, pb[2 * h + ks], racc[dt], 0, 0, 0);
                            }
                    // the softmax arithmetic is spread over the MFMAs of the step
                    constexpr int NMFMA = C::NSUB * (C::DK + 2 * C::DT);
                    constexpr int PER = (36 * C::NSUB + NMFMA - 1) / NMFMA;
#pragma unroll
                    for (int x = 0; x < NMFMA; ++x) {
                        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);               // one MFMA
                        __builtin_amdgcn_sched_group_barrier(0x402, PER, 0);             // a slice of VALU / exp
                    }
                };
                // Steps s .. to of one kind; sh_a holds the shifted logits of the latest tile before
                // and after.  The steps that still request a tile come first.
                int s = ws0 + 1;
                auto run = [&](int to, auto PLAIN_TAG) {
                    const int left_to_request = total_steps - dma_count;
                    const int to_dma = to - s + 1 <= left_to_request ? to : s + left_to_request - 1;
                    for (; s + 1 <= to_dma; s += 2) {
                        step(s, sh_a, sh_b, PLAIN_TAG, std::true_type{});
                        step(s + 1, sh_b, sh_a, PLAIN_TAG, std::true_type{});
                    }
                    if (s <= to_dma) {
                        step(s, sh_a, sh_b, PLAIN_TAG, std::true_type{});
#pragma unroll
                        for (int h = 0; h < C::NSUB; ++h) sh_a[h] = sh_b[h];
                        ++s;
                    }
                    for (; s <= to; ++s) {               // the last two steps of the kernel
                        step(s, sh_a, sh_b, std::false_type{}, std::false_type{});
#pragma unroll
                        for (int h = 0; h < C::NSUB; ++h) sh_a[h] = sh_b[h];
                    }
                };
                // window-edge tiles, tiles that need no mask, window-edge tiles
                const int p_lo = rows_full ? (s_lo > s ? s_lo : s) : ws1 + 1;
                const int p_hi = rows_full ? (s_hi < ws1 ? s_hi : ws1) : ws1;
                if (p_lo <= p_hi) {
                    run(p_lo - 1, std::false_type{});
                    run(p_hi, std::true_type{});
                }
                run(ws1, std::false_type{});
                X8 pb[2 * C::NSUB];
#pragma unroll
                for (int h = 0; h < C::NSUB; ++h) {
                    float rs;
                    weights(sh_a[h], pb + 2 * h, rs);
                    l += rs;
                    bad |= !(rs < E::WEIGHT_LIMIT);
                }
                value_mfmas(vt_prev, pb);
                for (int s2 = ws1 + 1; s2 < nt; ++s2) {   // (pre-pass) tiles after this wavefront's window
                    begin_step(s2);
                    advance();
                }
            }
        }

        if constexpr (LEFT) {
            // ---- pre-pass: every wavefront stores the partial result of its own unit -------
            const float lt = l + other_half(l);
            const bool any_bad = __builtin_amdgcn_ballot_w64(bad) != 0;
            if (ok && i < N) {
                const float inv = lt > 0.f ? 1.f / lt : 0.f;
                const int kr = i - delta > 0 ? i - delta : 0;
                const uint16_t* vrow = v2p + (int64_t)kr * p.v2.sn + 4 * hf;
                uint16_t* orow = (uint16_t*)p.out.p + p.out.off(b, i, h) + 4 * hf;
                uint2 vx[4 * C::DT];               // the V' row, read in one batch
#pragma unroll
                for (int e = 0; e < 4 * C::DT; ++e) vx[e] = *(const uint2*)(vrow + (e >> 2) * 32 + 8 * (e & 3));
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        const uint2 x = vx[4 * dt + g4];
                        union { EL h[4]; uint2 u; } o;
                        o.h[0] = (EL)(inv * racc[dt][4 * g4 + 0] * (E::lo(x.x) + p.v2_bias));
                        o.h[1] = (EL)(inv * racc[dt][4 * g4 + 1] * (E::hi(x.x) + p.v2_bias));
                        o.h[2] = (EL)(inv * racc[dt][4 * g4 + 2] * (E::lo(x.y) + p.v2_bias));
                        o.h[3] = (EL)(inv * racc[dt][4 * g4 + 3] * (E::hi(x.y) + p.v2_bias));
                        *(uint2*)(orow + dt * 32 + 8 * g4) = o.u;
                    }
                if (hf == 0) {
                    const float lam = lt > 0.f ? m + __log2f(lt) : -INFINITY;
                    p.lse[(int64_t)bh * N + i] = any_bad ? __builtin_nanf("") : lam;
                }
            }
            return;
        }

        if constexpr (C::NOFOLD) {
            // ---- the unit joins the wavefront's running result: O += e^(m-M) * (v2 + bias) * R ----
            if (ok) {
                const int tid_u = recompute_here(threadIdx.x);
                const int ln_u = tid_u & 31, hf_u = (tid_u >> 5) & 1;
                const uint16_t* vrow;
                if constexpr (SIDE) {
                    vrow = v2_s + (ln_u + w2 - delta) * C::KS + 4 * hf_u;
                } else {
                    const int iq = i0 + ln_u < N ? i0 + ln_u : N - 1;
                    vrow = v2p + (int64_t)(iq - delta > 0 ? iq - delta : 0) * p.v2.sn + 4 * hf_u;
                }
                uint2 vx[4 * C::DT];
#pragma unroll
                for (int e = 0; e < 4 * C::DT; ++e) vx[e] = *(const uint2*)(vrow + (e >> 2) * 32 + 8 * (e & 3));
                const float lt = l + other_half(l);
                const bool row_has = (i0 + ln_u < N) & (i0 + ln_u >= delta);
                // The fast kernel keeps a unit's reference point fixed, and every unit after the wavefront's
                // first starts from the running one: all weights are 1.  The repair kernel moves it.
                float a = 1.f, c = 1.f;
                if (SAFE) {
                    const float Mn = fmaxf(Mw, m), Mu = Mn == -INFINITY ? 0.f : Mn;
                    a = fast_exp2(Mw - Mu);
                    c = fast_exp2(m - Mu);
                    Mw = Mn;
                } else {
                    Mw = row_has ? m : Mw;           // (a row without a key in this unit keeps its state)
                }
                Lw = Lw * a + lt * c;
                const float vb = p.v2_bias;
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        const uint2 x = vx[4 * dt + g4];
                        if (SAFE) {
                            wacc[dt][4 * g4 + 0] = wacc[dt][4 * g4 + 0] * a + c * racc[dt][4 * g4 + 0] * (E::lo(x.x) + vb);
                            wacc[dt][4 * g4 + 1] = wacc[dt][4 * g4 + 1] * a + c * racc[dt][4 * g4 + 1] * (E::hi(x.x) + vb);
                            wacc[dt][4 * g4 + 2] = wacc[dt][4 * g4 + 2] * a + c * racc[dt][4 * g4 + 2] * (E::lo(x.y) + vb);
                            wacc[dt][4 * g4 + 3] = wacc[dt][4 * g4 + 3] * a + c * racc[dt][4 * g4 + 3] * (E::hi(x.y) + vb);
                        } else {
                            wacc[dt][4 * g4 + 0] += racc[dt][4 * g4 + 0] * (E::lo(x.x) + vb);
                            wacc[dt][4 * g4 + 1] += racc[dt][4 * g4 + 1] * (E::hi(x.x) + vb);
                            wacc[dt][4 * g4 + 2] += racc[dt][4 * g4 + 2] * (E::lo(x.y) + vb);
                            wacc[dt][4 * g4 + 3] += racc[dt][4 * g4 + 3] * (E::hi(x.y) + vb);
                        }
                    }
            }
            continue;
        }

        // ---- fold the round's units into the workgroup accumulator --------------
        // (lane coordinates are derived again here so that they do not occupy registers
        // during the sweep)
        const int tid_m = recompute_here(threadIdx.x);
        const int ln_m = tid_m & 31, hf_m = (tid_m >> 5) & 1;
        const int aq = tid_m >> 4, ac = (tid_m & 15) * ACN;
        // the V' row of this lane's query, read in one batch before the exchange below
        const uint16_t* vrow;
        if constexpr (SIDE) {
            vrow = v2_s + (ok ? ln_m + w2 - delta : 0) * C::KS + 4 * hf_m;
        } else {
            const int iq = i0 + ln_m < N ? i0 + ln_m : N - 1;
            const int vr = ok && iq - delta > 0 ? iq - delta : 0;
            vrow = v2p + (int64_t)vr * p.v2.sn + 4 * hf_m;
        }
        uint2 vx[4 * C::DT];
#pragma unroll
        for (int e = 0; e < 4 * C::DT; ++e) vx[e] = *(const uint2*)(vrow + (e >> 2) * 32 + 8 * (e & 3));
        const float lt = l + other_half(l);
        if (hf_m == 0) {
            xch_m[wave * BQ + ln_m] = m;
            xch_l[wave * BQ + ln_m] = lt;
        }
        __syncthreads();
        float Mrun = fin_m[ln_m], Lrun = fin_l[ln_m];
        float Mn = Mrun;
#pragma unroll
        for (int w = 0; w < FW; ++w) Mn = fmaxf(Mn, xch_m[w * BQ + ln_m]);
        const float Muse = (Mn == -INFINITY) ? 0.f : Mn;
        if (has_left && !SAFE && round == 0) {
            // the pre-pass partial: weight 1 at its own reference point, which stays out of the
            // running maximum (that remains the value of a logit)
            Mrun = lam_s[ln_m];
            Lrun = Mrun > -INFINITY ? 1.f : 0.f;
        }
        const float a = fast_exp2(Mrun - Muse);
        bad |= !(a < E::WEIGHT_LIMIT);
        float Ln = Lrun * a;
#pragma unroll
        for (int w = 0; w < FW; ++w) Ln += xch_l[w * BQ + ln_m] * fast_exp2(xch_m[w * BQ + ln_m] - Muse);
        // Wavefront 0 rescales the accumulator rows by a and adds its contribution
        // c * (v2 + bias) * R in place (its lanes own whole rows there).  Every other wavefront
        // writes its contribution as bf16 into its own slab: three slabs have their own LDS, the
        // other four use the two stage buffers that hold no tile of the next round.  Then
        // every thread adds its slice of the seven slabs in wavefront order.
        const float cw = ok ? fast_exp2(m - Muse) : 0.f;
        auto slab_of = [&](int w) -> uint16_t* {
            if (w < 4) return slabs + (w - 1) * (BQ * C::SS);
            const int fb = (buf + 2 + ((w - 4) >> 1)) & (C::NSTAGE - 1);      // the two stages after the next round's first two
            return smem + fb * C::STAGE + (w & 1) * (BQ * C::SS);
        };
        // PLAIN: every weight this wavefront applies is 1 (its unit started from the query's
        // running reference point and that did not move) and there is no V' bias.
        auto contribute = [&](auto PLAIN_TAG) {
            constexpr bool PLAIN = decltype(PLAIN_TAG)::value;
            const float vb = PLAIN ? 0.f : p.v2_bias;
            if (wave == 0) {
                float* arow = oacc + ln_m * C::OS + 4 * hf_m;
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        const uint2 x = vx[4 * dt + g4];
                        float4 o = *(float4*)(arow + dt * 32 + 8 * g4);
                        if (PLAIN) {
                            o.x += racc[dt][4 * g4 + 0] * E::lo(x.x);
                            o.y += racc[dt][4 * g4 + 1] * E::hi(x.x);
                            o.z += racc[dt][4 * g4 + 2] * E::lo(x.y);
                            o.w += racc[dt][4 * g4 + 3] * E::hi(x.y);
                        } else {
                            o.x = o.x * a + cw * racc[dt][4 * g4 + 0] * (E::lo(x.x) + vb);
                            o.y = o.y * a + cw * racc[dt][4 * g4 + 1] * (E::hi(x.x) + vb);
                            o.z = o.z * a + cw * racc[dt][4 * g4 + 2] * (E::lo(x.y) + vb);
                            o.w = o.w * a + cw * racc[dt][4 * g4 + 3] * (E::hi(x.y) + vb);
                        }
                        *(float4*)(arow + dt * 32 + 8 * g4) = o;
                    }
            } else {
                uint16_t* srow = slab_of(wave) + ln_m * C::SS + 4 * hf_m;
                const float c1 = PLAIN ? 1.f : cw;
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4) {
                        const uint2 x = vx[4 * dt + g4];
                        union { __bf16 h[4]; uint2 u; } o;      // slabs are bf16 whatever the element type
                        if (PLAIN) {
                            o.h[0] = (__bf16)(racc[dt][4 * g4 + 0] * E::lo(x.x));
                            o.h[1] = (__bf16)(racc[dt][4 * g4 + 1] * E::hi(x.x));
                            o.h[2] = (__bf16)(racc[dt][4 * g4 + 2] * E::lo(x.y));
                            o.h[3] = (__bf16)(racc[dt][4 * g4 + 3] * E::hi(x.y));
                        } else {
                            o.h[0] = (__bf16)(c1 * racc[dt][4 * g4 + 0] * (E::lo(x.x) + vb));
                            o.h[1] = (__bf16)(c1 * racc[dt][4 * g4 + 1] * (E::hi(x.x) + vb));
                            o.h[2] = (__bf16)(c1 * racc[dt][4 * g4 + 2] * (E::lo(x.y) + vb));
                            o.h[3] = (__bf16)(c1 * racc[dt][4 * g4 + 3] * (E::hi(x.y) + vb));
                        }
                        *(uint2*)(srow + dt * 32 + 8 * g4) = o.u;
                    }
            }
        };
        // (a unit that does not exist has cw = 0 and R = 0: it may take either path)
        const bool plain_lane = ((a == 1.f) | (wave != 0)) & ((cw == 1.f) | !ok) & (p.v2_bias == 0.f);
        if (__builtin_amdgcn_ballot_w64(!plain_lane) == 0) contribute(std::true_type{});
        else contribute(std::false_type{});
        __syncthreads();
        if (wave == 0 && hf_m == 0) {
            fin_m[ln_m] = Mn;
            fin_l[ln_m] = Ln;
        }
        {
            float acc[ACN];
#pragma unroll
            for (int c = 0; c < ACN; ++c) acc[c] = oacc[aq * C::OS + ac + c];
#pragma unroll
            for (int w = 1; w < FW; ++w) {
                const uint16_t* sp = slab_of(w) + aq * C::SS + ac;
                uint32_t sw[ACN / 2];
                load_words(sp, sw);
#pragma unroll
                for (int c = 0; c < ACN / 2; ++c) {
                    acc[2 * c] += bf16_lo(sw[c]);
                    acc[2 * c + 1] += bf16_hi(sw[c]);
                }
            }
#pragma unroll
            for (int c = 0; c < ACN; ++c) oacc[aq * C::OS + ac + c] = acc[c];
        }
        __syncthreads();       // the stage buffers that served as slabs are requested again in the next steps
    }

    if constexpr (C::NOFOLD && !LEFT) {
        // ---- merge the eight wavefronts (and the pre-pass partial) into the LDS accumulator ----
        const int tid_m = recompute_here(threadIdx.x);
        const int ln_m = tid_m & 31, hf_m = (tid_m >> 5) & 1;
        const int aq = tid_m >> 4, ac = (tid_m & 15) * ACN;
        if (hf_m == 0) {
            xch_m[wave * BQ + ln_m] = Mw;
            xch_l[wave * BQ + ln_m] = Lw;
        }
        __syncthreads();           // (also: every wavefront is done with the tile ring, which the sums go through)
        const bool with_left = has_left && !SAFE;
        auto reference = [&](int row) {
            float mx = with_left ? lam_s[row] : -INFINITY;
#pragma unroll
            for (int w = 0; w < FW; ++w) mx = fmaxf(mx, xch_m[w * BQ + row]);
            return mx;
        };
        // writer side: this wavefront's rows scaled to the common reference
        const float Mrow = reference(ln_m);
        const float cw = Mw == -INFINITY ? 0.f : fast_exp2(Mw - Mrow);
        // reader side: this thread's slice of the accumulator
        const float Mq = reference(aq), Mq_use = Mq == -INFINITY ? 0.f : Mq;
        float Ln = 0.f;
#pragma unroll
        for (int w = 0; w < FW; ++w) {
            const float mw = xch_m[w * BQ + aq];
            Ln += mw == -INFINITY ? 0.f : xch_l[w * BQ + aq] * fast_exp2(mw - Mq_use);
        }
        float acc[ACN];
        {
            const float al = (with_left && lam_s[aq] > -INFINITY) ? fast_exp2(lam_s[aq] - Mq_use) : 0.f;
            Ln += al;                                                     // the pre-pass partial has sum 1 at its reference
#pragma unroll
            for (int c = 0; c < ACN; ++c) acc[c] = with_left ? al * oacc[aq * C::OS + ac + c] : 0.f;
        }
        float* mbuf = (float*)smem_raw;                                   // [4][BQ][OS] fp32, over the tile ring
        static_assert((size_t)4 * BQ * C::OS * 4 <= C::STAGE_BYTES, "the merge buffer lies over the tile ring");
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            if ((wave >> 2) == pass) {
                float* mrow = mbuf + ((wave & 3) * BQ + ln_m) * C::OS + 4 * hf_m;
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                    for (int g4 = 0; g4 < 4; ++g4)
                        *(float4*)(mrow + dt * 32 + 8 * g4) = make_float4(cw * wacc[dt][4 * g4], cw * wacc[dt][4 * g4 + 1],
                                                                          cw * wacc[dt][4 * g4 + 2], cw * wacc[dt][4 * g4 + 3]);
            }
            __syncthreads();
#pragma unroll
            for (int w = 0; w < 4; ++w)
#pragma unroll
                for (int c = 0; c < ACN; ++c) acc[c] += mbuf[(w * BQ + aq) * C::OS + ac + c];
            __syncthreads();
        }
#pragma unroll
        for (int c = 0; c < ACN; ++c) oacc[aq * C::OS + ac + c] = acc[c];
        if ((tid_m & 15) == 0) {
            fin_m[aq] = Mq;
            fin_l[aq] = Ln;
        }
        __syncthreads();
    }

    // ---- normalise and store ------------------------------------------------------
    const bool any_bad = !SAFE && __syncthreads_or(bad ? 1 : 0);
    const int tid_f = recompute_here(threadIdx.x);
    const int aq = tid_f >> 4, ac = (tid_f & 15) * ACN;
    const int io = i0 + aq;
    if (io < N) {
        const float Ms = fin_m[aq], L = fin_l[aq];
        const float inv = 1.f / (L + 1e-8f * fast_exp2(-Ms));
        uint16_t* orow = (uint16_t*)p.out.p + p.out.off(b, io, h) + ac;
        union { EL h[ACN]; uint32_t w[ACN / 2]; } o;
#pragma unroll
        for (int c = 0; c < ACN; ++c) o.h[c] = (EL)(oacc[aq * C::OS + ac + c] * inv);
        store_words(orow, o.w);
        if ((tid_f & 15) == 0) {
            float lse;
            if (Ms > LOG2_EPS) lse = LN2 * (Ms + __log2f(L + 1e-8f * fast_exp2(-Ms)));
            else lse = LN_EPS + log1pf(L * fast_exp2(Ms - LOG2_EPS));
            p.lse[(int64_t)bh * N + io] = (any_bad && aq == 0) ? __builtin_nanf("") : lse;
        }
    }
}

template <class E, int D, bool SIDE>
int launch_fwd_kernels(const Problem& p, int nqb, int total, hipStream_t st) {
    using C = Cfg<D>;
    const size_t lds = C::lds_bytes(p.w2);
    // one unit left over after the rounds of eight: the pre-pass takes it, unless the grid is so
    // small that a further launch costs more than the lone round
    const int left = (p.w2 >= FW && p.w2 % FW == 0 && (p.force_prepass || total >= PREPASS_MIN_WORKGROUPS)) ? 1 : 0;
    if (!allow_full_lds((const void*)mfma_fwd_kernel<E, D, MODE_FAST, SIDE>) ||
        !allow_full_lds((const void*)mfma_fwd_kernel<E, D, MODE_SAFE, SIDE>) ||
        !allow_full_lds((const void*)mfma_fwd_kernel<E, D, MODE_LEFT, false>))
        return SA2_ERR_LAUNCH_FAILED;
    if (left) {
        const int ngrp = (nqb + FW - 1) / FW;
        const int total_left = ngrp * (total / nqb);
        hipLaunchKernelGGL((mfma_fwd_kernel<E, D, MODE_LEFT, false>), dim3((unsigned)total_left), dim3(FT), C::STAGE_BYTES, st, p,
                           ngrp, total_left, 0);
        if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
    }
    hipLaunchKernelGGL((mfma_fwd_kernel<E, D, MODE_FAST, SIDE>), dim3((unsigned)total), dim3(FT), lds, st, p, nqb, total, left);
    if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
    hipLaunchKernelGGL((mfma_fwd_kernel<E, D, MODE_SAFE, SIDE>), dim3((unsigned)total), dim3(FT), lds, st, p, nqb, total, left);
    return hipGetLastError() == hipSuccess ? SA2_OK : SA2_ERR_LAUNCH_FAILED;
}

template <class E, int D>
int launch_fwd_pair(const Problem& p, int nqb, int total, hipStream_t st) {
    return Cfg<D>::side_fits(p.w2) ? launch_fwd_kernels<E, D, true>(p, nqb, total, st)
                                   : launch_fwd_kernels<E, D, false>(p, nqb, total, st);
}

bool aligned16(const Tensor& t, int B, int N, int H) {
    if (!t.p) return true;
    if ((uintptr_t)t.p & 15u) return false;
    if (B > 1 && (t.sb & 7)) return false;
    if (N > 1 && (t.sn & 7)) return false;
    if (H > 1 && (t.sh & 7)) return false;
    // the kernels address rows of one (batch, head) slice with 32-bit element offsets
    if (N > 1 && (int64_t)(N - 1) * t.sn + 256 >= (int64_t)1 << 31) return false;
    return true;
}

}  // namespace

bool mfma_supported(int B, int N, int H, int D, int w1, int w2, int dtype) {
    (void)B; (void)H; (void)w1; (void)w2; (void)N;
    return (dtype == SA2_BF16 || dtype == SA2_F16) && (D == 32 || D == 64 || D == 128);
}

bool mfma_layout_ok(const Problem& p, bool backward) {
    const Tensor* fwd[] = {&p.q, &p.k1, &p.k2, &p.v1, &p.v2, &p.out};
    for (const Tensor* t : fwd)
        if (!aligned16(*t, p.B, p.N, p.H)) return false;
    if (backward) {
        const Tensor* bwd[] = {&p.dout, &p.dq, &p.dk1, &p.dk2, &p.dv1, &p.dv2};
        for (const Tensor* t : bwd)
            if (!aligned16(*t, p.B, p.N, p.H)) return false;
    }
    return true;
}

int launch_mfma_fwd(const Problem& p, int dtype, hipStream_t st) {
    const int nqb = (p.N + BQ - 1) / BQ;
    const int64_t total = (int64_t)nqb * p.B * p.H;
    if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    if (dtype == SA2_F16)
        return p.D == 128 ? launch_fwd_pair<ElemF16, 128>(p, nqb, (int)total, st)
               : p.D == 64 ? launch_fwd_pair<ElemF16, 64>(p, nqb, (int)total, st)
                           : launch_fwd_pair<ElemF16, 32>(p, nqb, (int)total, st);
    return p.D == 128 ? launch_fwd_pair<ElemBF16, 128>(p, nqb, (int)total, st)
           : p.D == 64 ? launch_fwd_pair<ElemBF16, 64>(p, nqb, (int)total, st)
                       : launch_fwd_pair<ElemBF16, 32>(p, nqb, (int)total, st);
}

}  // namespace sa2
