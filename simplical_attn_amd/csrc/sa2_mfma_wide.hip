// MFMA kernels for 16-bit tensors whose head_dim the tuned kernels do not take: head_dim 256
// (bf16 or fp16), forward and backward, on v_mfma_f32_32x32x16_bf16 / _f16.
//
// Same expanded-row view as the tuned kernels (rows r = (i, delta), Q~[r] = q[i] * k2~[i-delta] *
// scale*log2(e), dO~[r] = dO[i] * v2~[i-delta], both rounded to the element type), in the simple
// arrangement of the fp32 MFMA kernels: four wavefronts per workgroup, one per SIMD with the whole
// register file, 32-row tiles row-major in a double-buffered LDS stage written from registers, one
// barrier per tile.  Row operands are 16-byte reads of a tile row; transposed operands (the tile's
// rows as the contraction index) come from the same tile through ds_read_b64_tr_b16, with a row
// stride that keeps both kinds of read free of bank conflicts.
//
// A head_dim of 256 does not leave room for the operands of the logit contraction (64 registers) next
// to accumulators for all 256 output columns of two contractions, so every kernel takes the output
// columns in passes of DV = 128 (grid dimension y): a pass contracts the logits over the whole
// head_dim and accumulates its own 128 columns of R, G, dK, dV.  The logits (and dP) are computed
// once per pass: 1.5x the forward's and 1.33x the backward's algorithmic MFMA work.
//
//   wide_fwd_kernel   32 queries per workgroup; wavefront w takes delta = w, w+4, ... with one online
//                     softmax and one output accumulator across its units, merged once at the end.
//   wide_kp_kernel    32 K' rows per workgroup and every delta; the unit's reductions (dK', dV' rows
//                     aligned with the unit's rows, dQ rows shifted by delta) go to fp32 accumulators
//                     in LDS in column-rotated phases; dQ leaves as a per-workgroup partial that
//                     wide_dq_sum_kernel adds up in block order.
//   wide_kv_kernel    128 K/V rows per workgroup (32 per wavefront, resident in registers as B
//                     operands), streaming every unit (query block, delta) that can see them.
// Every output element has one writer and a fixed summation order: no atomics, bitwise reproducible.
#include "sa2_mfma_common.h"

namespace sa2 {
namespace {

constexpr int WW = 4;                  // wavefronts per workgroup
constexpr int WT = WW * 64;            // threads per workgroup
constexpr int WJ = WW * 32;            // K rows per workgroup of the K-side kernel

typedef unsigned ux4 __attribute__((ext_vector_type(4)));     // 16 bytes in flight (a plain vector: stays in registers)

template <int D, int DV>
struct WideCfg {
    static_assert(D % 32 == 0 && DV % 32 == 0 && D % DV == 0, "32-column blocks");
    static constexpr int DK = D / 16;          // k-steps of a contraction over head_dim
    static constexpr int DT = DV / 32;         // 32-column blocks of a pass's output columns
    static constexpr int NPASS = D / DV;
    static constexpr int RS = D + 16;          // tile row stride (elements): rows lie 8 banks apart
    static constexpr int RSB = RS * 2;         // ... in bytes
    static constexpr int TILE = 32 * RS;       // elements
    static constexpr int STAGE = 2 * TILE;     // two tiles (K and V, or Q~ and dO~)
    static constexpr int KR = 32 * D / 8 / WT; // 16-byte chunks per thread and tile
    static constexpr int AS = DV + 4;          // row stride of the fp32 accumulators in LDS
    static constexpr size_t TILES_BYTES = (size_t)2 * STAGE * 2;
    static constexpr size_t MERGE_BYTES = (size_t)WW * 32 * AS * 4;
    static constexpr size_t FWD_LDS = (TILES_BYTES > MERGE_BYTES ? TILES_BYTES : MERGE_BYTES) + 2 * WW * 32 * 4;
    static constexpr size_t LDS_LIMIT = 160 * 1024;
    static size_t kp_lds(int w2) { return TILES_BYTES + (size_t)(32 + w2 + 64) * AS * 4; }
    static bool kp_fits(int w2) { return kp_lds(w2) <= LDS_LIMIT; }
    // deltas whose dQ rows the accumulator holds at once: all w2 + 1 of them, or (wider K' windows) the largest
    // multiple of four that fits; the kernel then walks the window in segments of that many deltas
    static int kp_segment(int w2) {
        if (kp_fits(w2)) return w2 + 1;
        int segw = 32;
        while (kp_fits(segw + WW - 1)) segw += WW;
        return segw;
    }
    static constexpr size_t KV_LDS = TILES_BYTES + 2 * 2 * 32 * 4;
};

__device__ __forceinline__ floatx16 zeros16() {
    floatx16 z;
#pragma unroll
    for (int v = 0; v < 16; ++v) z[v] = 0.f;
    return z;
}
__device__ __forceinline__ int xcd_neighbours(int pid, int total) {
    // workgroups are dealt round-robin to the 8 XCDs: neighbours in the problem share an L2
    return (total & 7) == 0 ? (pid & 7) * (total >> 3) + (pid >> 3) : pid;
}

// Rows [j0, j0+32) of two tensors (clamped to the sequence) from global memory to registers, and
// from there to the two tiles of a stage.
template <int D, int DV, int KR>
__device__ __forceinline__ void wide_load(ux4 (&a)[KR], ux4 (&b)[KR], const uint16_t* ap, int64_t as,
                                          const uint16_t* bp, int64_t bs, int j0, int N, int tid) {
#pragma unroll
    for (int u = 0; u < KR; ++u) {
        const int c = tid + WT * u;
        const int row = c / (D / 8), col = c - row * (D / 8);
        int j = j0 + row;
        j = j < N ? j : N - 1;
        a[u] = *(const ux4*)(ap + (int64_t)j * as + col * 8);
        b[u] = *(const ux4*)(bp + (int64_t)j * bs + col * 8);
    }
}
template <int D, int DV, int KR>
__device__ __forceinline__ void wide_store(const ux4 (&a)[KR], const ux4 (&b)[KR], uint16_t* stage, int tid) {
    using C = WideCfg<D, DV>;
#pragma unroll
    for (int u = 0; u < KR; ++u) {
        const int c = tid + WT * u;
        const int row = c / (D / 8), col = c - row * (D / 8);
        *(ux4*)(stage + row * C::RS + col * 8) = a[u];
        *(ux4*)(stage + C::TILE + row * C::RS + col * 8) = b[u];
    }
}

// Lane part of a transposed operand read out of a row-major tile: within 16 lanes, lane s supplies the
// address of row s/4, columns 4*(s%4)..+3, and lane i receives column i of those four rows; the four
// 16-lane groups of a wavefront take the rows 0-3 / 4-7 (by half) of the 16-column halves of a 32-column
// block.  The operand of k-step ks and column block c is then the reads at
//   tile + lane part + (16*ks) * row stride + 2*c     and     ... + (16*ks + 8) * row stride ...
// whose eight values are, in order, the k-slots of a 32x32 accumulator handed on as the other operand.
template <int RSB>
__device__ __forceinline__ uint32_t tr_lane_offset(int lane) {
    const int grp = lane >> 4, s = lane & 15;
    return (uint32_t)((4 * (grp >> 1) + (s >> 2)) * RSB + (16 * (grp & 1) + 4 * (s & 3)) * 2);
}
template <class X8, int RSB>
__device__ __forceinline__ X8 tr_operand(uint32_t addr) {
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef v4s __attribute__((address_space(3)))* lds_v4s;
    union { v4s h[2]; X8 v; } u;
    u.h[0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(uintptr_t)addr);
    u.h[1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(uintptr_t)(addr + 8 * RSB));
    return u.v;
}

// a[r] * (b[r] + bias) [* mul] of two 16-byte chunks (8 elements), rounded to the element type
template <class E>
__device__ __forceinline__ typename E::x8 product8(const ux4& a, const ux4& b, float bias, float mul) {
    typedef typename E::scalar EL;
    typename E::x8 r;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        r[2 * t] = (EL)(E::lo(a[t]) * mul * (E::lo(b[t]) + bias));
        r[2 * t + 1] = (EL)(E::hi(a[t]) * mul * (E::hi(b[t]) + bias));
    }
    return r;
}

// ================================================================== forward =====
template <class E, int D, int DV>
__global__ __launch_bounds__(WT) __attribute__((amdgpu_waves_per_eu(1, 1)))
void wide_fwd_kernel(Problem p, int nqb, int total) {
    typedef typename E::scalar EL;
    typedef typename E::x8 X8;
    using C = WideCfg<D, DV>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_w[];
    uint16_t* tiles = (uint16_t*)smem_w;
    float* mrg_m = (float*)(smem_w + (C::TILES_BYTES > C::MERGE_BYTES ? C::TILES_BYTES : C::MERGE_BYTES));   // [WW][32]
    float* mrg_l = mrg_m + WW * 32;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;
    const int pid = xcd_neighbours(blockIdx.x, total);
    const int c0 = blockIdx.y * DV;                          // this pass's output columns
    const int bh = pid / nqb, qb = pid - bh * nqb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int i0 = qb * BQ, i = i0 + ln, ic = i < N ? i : N - 1;
    const int i_last = i0 + BQ - 1 < N ? i0 + BQ - 1 : N - 1;

    const uint16_t* qp = (const uint16_t*)p.q.p + p.q.off(b, 0, h);
    const uint16_t* k1p = (const uint16_t*)p.k1.p + p.k1.off(b, 0, h);
    const uint16_t* k2p = (const uint16_t*)p.k2.p + p.k2.off(b, 0, h);
    const uint16_t* v1p = (const uint16_t*)p.v1.p + p.v1.off(b, 0, h);
    const uint16_t* v2p = (const uint16_t*)p.v2.p + p.v2.off(b, 0, h);

    const int jt_lo = (i0 - w1 > 0 ? i0 - w1 : 0) / TJ, jt_hi = i_last / TJ;
    const int nt = jt_hi - jt_lo + 1;
    const int n_units = (w2 < i_last ? w2 : i_last) + 1;
    const int nrounds = (n_units + WW - 1) / WW;
    const float qscale = p.scale * LOG2E;
    const uint32_t tiles_addr = lds_address(tiles);
    const uint32_t tr_lane = tr_lane_offset<C::RSB>(lane);

    ux4 tk[C::KR], tv[C::KR];                    // the tile on its way from global memory to LDS
    wide_load<D, DV>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, jt_lo * TJ, N, tid);
    wide_store<D, DV>(tk, tv, tiles, tid);
    wide_load<D, DV>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, (jt_lo + 1 % nt) * TJ, N, tid);
    __syncthreads();

    // the wavefront's running softmax over its units: reference exponent, sum, weighted output
    float M = -INFINITY, L = 0.f;
    floatx16 oacc[C::DT];
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt) oacc[dt] = zeros16();

    int g = 0;
    for (int round = 0; round < nrounds; ++round) {
        const int delta = round * WW + wave;
        const bool ok = delta < n_units;
        const int kr = ic - delta > 0 ? ic - delta : 0;
        const bool row_ok = ok && i < N && i >= delta;
        const bool rows_full = i0 >= delta && i0 + BQ - 1 < N;

        X8 qf[C::DK];
        if (ok) {
#pragma unroll
            for (int kk = 0; kk < C::DK; ++kk) {
                const ux4 qa = *(const ux4*)(qp + (int64_t)ic * p.q.sn + kk * 16 + hf * 8);
                const ux4 kb = *(const ux4*)(k2p + (int64_t)kr * p.k2.sn + kk * 16 + hf * 8);
                qf[kk] = product8<E>(qa, kb, p.k2_bias, qscale);
            }
        }
        float m = -INFINITY, l = 0.f;
        floatx16 racc[C::DT];
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) racc[dt] = zeros16();

        for (int s = 0; s < nt; ++s, ++g) {
            if (ok) {
                const int j0 = (jt_lo + s) * TJ;
                const uint16_t* Ks = tiles + (g & 1) * C::STAGE;
                const uint32_t Vt = tiles_addr + (uint32_t)(((g & 1) * C::STAGE + C::TILE) * 2) + tr_lane + (uint32_t)(c0 * 2);
                floatx16 sacc = zeros16();
#pragma unroll
                for (int kk = 0; kk < C::DK; ++kk) {
                    const X8 ka = *(const X8*)(Ks + ln * C::RS + kk * 16 + hf * 8);
                    sacc = E::mfma(ka, qf[kk], sacc, 0, 0, 0);
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
                // the weights as the MFMA sees them (rounded), and their sum
                X8 pb[2];
                float rs = 0.f;
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        pb[ks][t] = (EL)fast_exp2(sacc[ks * 8 + t] - m_use);
                        rs += (float)pb[ks][t];
                    }
                l += rs;
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt) {
                        const X8 va = tr_operand<X8, C::RSB>(Vt + (uint32_t)(16 * ks * C::RSB + dt * 64));
                        racc[dt] = E::mfma(va, pb[ks], racc[dt], 0, 0, 0);
                    }
            }
            // (unconditional: past the last step this moves a tile nobody reads)
            wide_store<D, DV>(tk, tv, tiles + ((g + 1) & 1) * C::STAGE, tid);
            wide_load<D, DV>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, (jt_lo + (g + 2) % nt) * TJ, N, tid);
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
            const uint16_t* vrow = v2p + (int64_t)kr * p.v2.sn + c0 + 4 * hf;
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                for (int g4 = 0; g4 < 4; ++g4) {
                    const uint2 x = *(const uint2*)(vrow + dt * 32 + 8 * g4);
                    oacc[dt][4 * g4 + 0] = oacc[dt][4 * g4 + 0] * a + c * racc[dt][4 * g4 + 0] * (E::lo(x.x) + p.v2_bias);
                    oacc[dt][4 * g4 + 1] = oacc[dt][4 * g4 + 1] * a + c * racc[dt][4 * g4 + 1] * (E::hi(x.x) + p.v2_bias);
                    oacc[dt][4 * g4 + 2] = oacc[dt][4 * g4 + 2] * a + c * racc[dt][4 * g4 + 2] * (E::lo(x.y) + p.v2_bias);
                    oacc[dt][4 * g4 + 3] = oacc[dt][4 * g4 + 3] * a + c * racc[dt][4 * g4 + 3] * (E::hi(x.y) + p.v2_bias);
                }
        }
    }

    // ---- merge the four wavefronts (the tile stages are free: the sweep's last barrier is behind us) ----
    float* mrg = (float*)smem_w;                           // [WW][32][AS]
    {
        float* row = mrg + (wave * 32 + ln) * C::AS + 4 * hf;
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
        for (int w = 0; w < WW; ++w) Mx = fmaxf(Mx, mrg_m[w * 32 + row]);
        const float Mu = Mx == -INFINITY ? 0.f : Mx;
        float wgt[WW], Ls = 0.f;
#pragma unroll
        for (int w = 0; w < WW; ++w) {
            wgt[w] = fast_exp2(mrg_m[w * 32 + row] - Mu);
            Ls += mrg_l[w * 32 + row] * wgt[w];
        }
        // sum_w + 1e-8 in units of 2^Mu (reference.py:74); for a tiny Mu the epsilon dominates
        const bool big = Mu > LOG2_EPS;
        const float denom = big ? Ls + 1e-8f * fast_exp2(-Mu) : Ls * fast_exp2(Mu - LOG2_EPS) + 1.f;
        const float inv = big ? 1.f / denom : fast_exp2(Mu - LOG2_EPS) / denom;
        uint16_t* orow = (uint16_t*)p.out.p + p.out.off(b, io, h) + c0;
#pragma unroll
        for (int x = 0; x < C::DT; ++x) {
            const int col = 32 * x + 4 * (tid & 7);
            float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int w = 0; w < WW; ++w) {
                const float4 y = *(const float4*)(mrg + (w * 32 + row) * C::AS + col);
                acc.x += wgt[w] * y.x; acc.y += wgt[w] * y.y; acc.z += wgt[w] * y.z; acc.w += wgt[w] * y.w;
            }
            *(uint2*)(orow + col) = make_uint2(E::pack(acc.x * inv, acc.y * inv), E::pack(acc.z * inv, acc.w * inv));
        }
        if ((tid & 7) == 0 && blockIdx.y == 0)
            p.lse[(int64_t)bh * N + io] = big ? LN2 * Mu + logf(denom) : LN_EPS + logf(denom);
    }
}

// ============================================== backward, K' side: dQ, dK', dV' =====
// SEG: the K' window is walked in segments of segw deltas (a kernel of its own; segw = w2 + 1 otherwise)
template <class E, int D, int DV, bool SEG>
__global__ __launch_bounds__(WT) __attribute__((amdgpu_waves_per_eu(1, 1)))
void wide_kp_kernel(Problem p, int nkb, int total, float* __restrict__ dq_part, int segw) {
    typedef typename E::scalar EL;
    typedef typename E::x8 X8;
    using C = WideCfg<D, DV>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_w[];
    uint16_t* tiles = (uint16_t*)smem_w;
    float* dk_s = (float*)(smem_w + C::TILES_BYTES);     // [32][AS]: dK' rows k0 .. k0+31 (before the scale)
    float* dv_s = dk_s + 32 * C::AS;                     // [32][AS]: dV' rows
    float* dq_s = dv_s + 32 * C::AS;                     // [32 + segw - 1][AS]: dQ rows k0 + dbase .. of the current segment (before the scale)

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;
    const int pid = xcd_neighbours(blockIdx.x, total);
    const int c0 = blockIdx.y * DV;
    const int bh = pid / nkb, kb = pid - bh * nkb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int k0 = kb * BQ, k = k0 + ln, kc = k < N ? k : N - 1;
    const int NR = 32 + w2;                      // rows of the block's dQ partial
    const int NRS = 32 + segw - 1;               // rows of the accumulator
    int dbase = 0;                               // first delta of the current segment

    const uint16_t* qp = (const uint16_t*)p.q.p + p.q.off(b, 0, h);
    const uint16_t* k1p = (const uint16_t*)p.k1.p + p.k1.off(b, 0, h);
    const uint16_t* k2p = (const uint16_t*)p.k2.p + p.k2.off(b, 0, h);
    const uint16_t* v1p = (const uint16_t*)p.v1.p + p.v1.off(b, 0, h);
    const uint16_t* v2p = (const uint16_t*)p.v2.p + p.v2.off(b, 0, h);
    const uint16_t* dop = (const uint16_t*)p.dout.p + p.dout.off(b, 0, h);
    const bool want_dq = p.dq.p != nullptr;

    const int n_units = (w2 < N - 1 - k0 ? w2 : N - 1 - k0) + 1;       // delta with k0 + delta < N
    const int nrounds = (n_units + WW - 1) / WW;
    const float qscale = p.scale * LOG2E;
    const uint32_t tiles_addr = lds_address(tiles);
    const uint32_t tr_lane = tr_lane_offset<C::RSB>(lane);

    for (int c = tid; c < (NRS + 64) * C::AS; c += WT) dk_s[c] = 0.f;      // all three accumulators

    ux4 tk[C::KR], tv[C::KR];
    for (int round = 0; round < nrounds; ++round) {
        // queries of the round's units: k0 + 4*round .. k0 + 31 + 4*round + 3 (within the sequence)
        const int d_first = round * WW, d_last = d_first + WW - 1 < n_units - 1 ? d_first + WW - 1 : n_units - 1;
        const int i_min = k0 + d_first, i_max = k0 + 31 + d_last < N - 1 ? k0 + 31 + d_last : N - 1;
        const int jt_lo = (i_min - w1 > 0 ? i_min - w1 : 0) / TJ, jt_hi = i_max / TJ;
        const int nt = jt_hi - jt_lo + 1;

        const int delta = d_first + wave;
        const bool ok = delta < n_units;
        const int i = k + delta, ic = i < N ? i : N - 1;
        const bool row_ok = ok && i < N;
        const int iw_lo = k0 + delta, iw_hi = k0 + 31 + delta < N - 1 ? k0 + 31 + delta : N - 1;   // this unit's queries
        const bool rows_full = k0 + 31 + delta < N;

        X8 qf[C::DK], dof[C::DK];
        float lse2 = 0.f, dsum = 0.f;
        if (ok) {
#pragma unroll
            for (int kk = 0; kk < C::DK; ++kk) {
                const int col = kk * 16 + hf * 8;
                const ux4 qa = *(const ux4*)(qp + (int64_t)ic * p.q.sn + col);
                const ux4 ka = *(const ux4*)(k2p + (int64_t)kc * p.k2.sn + col);
                const ux4 da = *(const ux4*)(dop + (int64_t)ic * p.dout.sn + col);
                const ux4 va = *(const ux4*)(v2p + (int64_t)kc * p.v2.sn + col);
                qf[kk] = product8<E>(qa, ka, p.k2_bias, qscale);
                dof[kk] = product8<E>(da, va, p.v2_bias, 1.f);
            }
            lse2 = p.lse[(int64_t)bh * N + ic] * LOG2E;
            dsum = p.dsum[(int64_t)bh * N + ic];
        }
        floatx16 racc[C::DT], gacc[C::DT];
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt) racc[dt] = gacc[dt] = zeros16();

        // (the previous round's last barrier has passed: both stages are free)
        wide_load<D, DV>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, jt_lo * TJ, N, tid);
        wide_store<D, DV>(tk, tv, tiles, tid);
        wide_load<D, DV>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, (jt_lo + 1 % nt) * TJ, N, tid);
        __syncthreads();
        for (int s = 0; s < nt; ++s) {
            const int j0 = (jt_lo + s) * TJ;
            // tiles that hold no key of this unit's windows are skipped by the wavefront
            if (ok && j0 <= iw_hi && j0 + TJ - 1 >= iw_lo - w1) {
                const uint16_t* Ks = tiles + (s & 1) * C::STAGE;
                const uint16_t* Vs = Ks + C::TILE;
                const uint32_t Kt = tiles_addr + (uint32_t)((s & 1) * C::STAGE * 2) + tr_lane + (uint32_t)(c0 * 2);
                const uint32_t Vt = Kt + (uint32_t)(C::TILE * 2);
                floatx16 sacc = zeros16(), dpacc = zeros16();
#pragma unroll
                for (int kk = 0; kk < C::DK; ++kk) {
                    const X8 ka = *(const X8*)(Ks + ln * C::RS + kk * 16 + hf * 8);
                    const X8 va = *(const X8*)(Vs + ln * C::RS + kk * 16 + hf * 8);
                    sacc = E::mfma(ka, qf[kk], sacc, 0, 0, 0);
                    dpacc = E::mfma(va, dof[kk], dpacc, 0, 0, 0);
                }
                const bool interior = rows_full && (j0 + TJ - 1 <= iw_lo) && (j0 >= iw_lo + 31 - w1);
                const int hi = i - j0 - 4 * hf, lo = hi - w1;
                X8 pb[2], dsb[2];
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int c = 8 * (v >> 2) + (v & 3);
                    const bool valid = interior || (row_ok && c <= hi && c >= lo);
                    const float pv = valid ? fast_exp2(sacc[v] - lse2) : 0.f;
                    pb[v >> 3][v & 7] = (EL)pv;
                    dsb[v >> 3][v & 7] = (EL)(pv * (dpacc[v] - dsum));
                }
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt) {
                        const uint32_t o = (uint32_t)(16 * ks * C::RSB + dt * 64);
                        racc[dt] = E::mfma(tr_operand<X8, C::RSB>(Vt + o), pb[ks], racc[dt], 0, 0, 0);
                        gacc[dt] = E::mfma(tr_operand<X8, C::RSB>(Kt + o), dsb[ks], gacc[dt], 0, 0, 0);
                    }
            }
            wide_store<D, DV>(tk, tv, tiles + ((s + 1) & 1) * C::STAGE, tid);
            wide_load<D, DV>(tk, tv, k1p, p.k1.sn, v1p, p.v1.sn, (jt_lo + (s + 2) % nt) * TJ, N, tid);
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
                const uint16_t* qrow = qp + (int64_t)ic * p.q.sn + c0 + col;
                const uint16_t* drow = dop + (int64_t)ic * p.dout.sn + c0 + col;
                const uint16_t* krow = k2p + (int64_t)kc * p.k2.sn + c0 + col;
                float* dkrow = dk_s + ln * C::AS + col;
                float* dvrow = dv_s + ln * C::AS + col;
                float* dqrow = dq_s + (ln + delta - dbase) * C::AS + col;
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt) {
                    // (g4 is uniform over the wavefront: pick this group's four registers)
                    float gv[4], rv[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        gv[t] = g4 == 0 ? gacc[dt][t] : g4 == 1 ? gacc[dt][4 + t] : g4 == 2 ? gacc[dt][8 + t] : gacc[dt][12 + t];
                        rv[t] = g4 == 0 ? racc[dt][t] : g4 == 1 ? racc[dt][4 + t] : g4 == 2 ? racc[dt][8 + t] : racc[dt][12 + t];
                    }
                    const uint2 qx = *(const uint2*)(qrow + dt * 32);
                    const uint2 dx = *(const uint2*)(drow + dt * 32);
                    float4 a = *(float4*)(dkrow + dt * 32);
                    a.x += gv[0] * E::lo(qx.x); a.y += gv[1] * E::hi(qx.x); a.z += gv[2] * E::lo(qx.y); a.w += gv[3] * E::hi(qx.y);
                    *(float4*)(dkrow + dt * 32) = a;
                    float4 c = *(float4*)(dvrow + dt * 32);
                    c.x += rv[0] * E::lo(dx.x); c.y += rv[1] * E::hi(dx.x); c.z += rv[2] * E::lo(dx.y); c.w += rv[3] * E::hi(dx.y);
                    *(float4*)(dvrow + dt * 32) = c;
                    if (want_dq) {
                        const uint2 kx = *(const uint2*)(krow + dt * 32);
                        float4 o = *(float4*)(dqrow + dt * 32);
                        o.x += gv[0] * (E::lo(kx.x) + p.k2_bias); o.y += gv[1] * (E::hi(kx.x) + p.k2_bias);
                        o.z += gv[2] * (E::lo(kx.y) + p.k2_bias); o.w += gv[3] * (E::hi(kx.y) + p.k2_bias);
                        *(float4*)(dqrow + dt * 32) = o;
                    }
                }
            }
            __syncthreads();
        }
        // ---- end of a segment: its first segw dQ rows are complete and go to the partial; the 31 rows the next
        //      segment shares with it move to the front of the accumulator ----
        if (SEG && round + 1 < nrounds && (round + 1) * WW - dbase >= segw) {
            if (want_dq) {
                float* part = dq_part + (((int64_t)bh * nkb + kb) * (int64_t)NR + dbase) * D + c0;
                for (int c = tid; c < segw * (DV / 4); c += WT) {
                    const int r = c / (DV / 4), col = c - r * (DV / 4);
                    *(float4*)(part + (int64_t)r * D + col * 4) = *(const float4*)(dq_s + r * C::AS + col * 4);
                }
                __syncthreads();
                for (int c = tid; c < 31 * (DV / 4); c += WT) {         // (segw >= 32: source and destination are disjoint)
                    const int r = c / (DV / 4), col = c - r * (DV / 4);
                    *(float4*)(dq_s + r * C::AS + col * 4) = *(const float4*)(dq_s + (segw + r) * C::AS + col * 4);
                }
                __syncthreads();
                for (int c = tid; c < (NRS - 31) * (DV / 4); c += WT) {
                    const int r = 31 + c / (DV / 4), col = c % (DV / 4);
                    *(float4*)(dq_s + r * C::AS + col * 4) = make_float4(0.f, 0.f, 0.f, 0.f);
                }
                __syncthreads();
            }
            dbase += segw;
        }
    }

    // ---- dK' and dV' rows of the block (this pass's columns) ----
    {
        const int row = tid >> 3, ko = k0 + row;
        if (ko < N) {
#pragma unroll
            for (int x = 0; x < C::DT; ++x) {
                const int col = 32 * x + 4 * (tid & 7);
                if (p.dk2.p) {
                    const float4 a = *(const float4*)(dk_s + row * C::AS + col);
                    *(uint2*)((uint16_t*)p.dk2.p + p.dk2.off(b, ko, h) + c0 + col) =
                        make_uint2(E::pack(a.x * p.scale, a.y * p.scale), E::pack(a.z * p.scale, a.w * p.scale));
                }
                if (p.dv2.p) {
                    const float4 a = *(const float4*)(dv_s + row * C::AS + col);
                    *(uint2*)((uint16_t*)p.dv2.p + p.dv2.off(b, ko, h) + c0 + col) = make_uint2(E::pack(a.x, a.y), E::pack(a.z, a.w));
                }
            }
        }
    }
    // ---- dQ partial of this block: rows k0 .. k0+31+w2, this pass's columns ----
    //      (those from dbase on are still here; rows past the accumulator belong to deltas beyond the end of the
    //      sequence: zeros)
    if (want_dq) {
        float* part = dq_part + (((int64_t)bh * nkb + kb) * (int64_t)NR + dbase) * D + c0;
        for (int c = tid; c < (NR - dbase) * (DV / 4); c += WT) {
            const int r = c / (DV / 4), col = c - r * (DV / 4);
            *(float4*)(part + (int64_t)r * D + col * 4) =
                r < NRS ? *(const float4*)(dq_s + r * C::AS + col * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
}

// dQ[i] = scale * sum over the K' blocks kb with 32*kb <= i <= 32*kb + 31 + w2, in block order
template <class E, int D>
__global__ __launch_bounds__(256) void wide_dq_sum_kernel(Problem p, int nkb, const float* __restrict__ dq_part, int64_t chunks) {
    const int64_t c = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (c >= chunks) return;
    const int col = (int)(c % (D / 4));
    const int64_t rowid = c / (D / 4);
    const int i = (int)(rowid % p.N);
    const int bh = (int)(rowid / p.N);
    const int b = bh / p.H, h = bh - b * p.H;
    const int NR = 32 + p.w2;
    const int kb_lo = (i - 31 - p.w2) <= 0 ? 0 : (i - p.w2) / 32;      // smallest kb with 32*kb + 31 + w2 >= i
    const int kb_hi = i / 32;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int kb = kb_lo; kb <= kb_hi; ++kb) {
        const float4 y = *(const float4*)(dq_part + (((int64_t)bh * nkb + kb) * NR + (i - 32 * kb)) * D + col * 4);
        acc.x += y.x; acc.y += y.y; acc.z += y.z; acc.w += y.w;
    }
    *(uint2*)((uint16_t*)p.dq.p + p.dq.off(b, i, h) + col * 4) =
        make_uint2(E::pack(acc.x * p.scale, acc.y * p.scale), E::pack(acc.z * p.scale, acc.w * p.scale));
}

// =================================================== backward, K side: dK, dV =====
// nsplit > 1 (grids smaller than the chip): the workgroup takes the sp-th share of the key block's stream
// of units and writes fp32 partial sums to `part` ([dK | dV][nsplit][B*H][N][D]) for wide_kv_sum_kernel.
template <class E, int D, int DV, bool SPLIT>
__global__ __launch_bounds__(WT) __attribute__((amdgpu_waves_per_eu(1, 1)))
void wide_kv_kernel(Problem p, int njb, int total, int nsplit_arg, float* __restrict__ part) {
    const int nsplit = SPLIT ? nsplit_arg : 1;
    typedef typename E::scalar EL;
    typedef typename E::x8 X8;
    using C = WideCfg<D, DV>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_w[];
    uint16_t* tiles = (uint16_t*)smem_w;
    float* lse_s = (float*)(smem_w + C::TILES_BYTES);    // [2][32]  LSE*log2(e) of the unit's queries
    float* dsum_s = lse_s + 2 * 32;                      // [2][32]

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;
    const int pid = xcd_neighbours(blockIdx.x, total);
    const int c0 = blockIdx.y * DV;
    const int sp = pid % nsplit, pj = pid / nsplit;
    const int bh = pj / njb, jb = pj - bh * njb;
    const int b = bh / p.H, h = bh - b * p.H;
    const int N = p.N, w1 = p.w1, w2 = p.w2;
    const int j0 = jb * WJ, jw = j0 + 32 * wave, j = jw + ln, jc = j < N ? j : N - 1;

    const uint16_t* qp = (const uint16_t*)p.q.p + p.q.off(b, 0, h);
    const uint16_t* k1p = (const uint16_t*)p.k1.p + p.k1.off(b, 0, h);
    const uint16_t* k2p = (const uint16_t*)p.k2.p + p.k2.off(b, 0, h);
    const uint16_t* v1p = (const uint16_t*)p.v1.p + p.v1.off(b, 0, h);
    const uint16_t* v2p = (const uint16_t*)p.v2.p + p.v2.off(b, 0, h);
    const uint16_t* dop = (const uint16_t*)p.dout.p + p.dout.off(b, 0, h);
    const float qscale = p.scale * LOG2E;
    const uint32_t tiles_addr = lds_address(tiles);
    const uint32_t tr_lane = tr_lane_offset<C::RSB>(lane);

    // this wavefront's K and V rows as resident B operands (column = key j)
    X8 kf[C::DK], vf[C::DK];
#pragma unroll
    for (int kk = 0; kk < C::DK; ++kk) {
        kf[kk] = *(const X8*)(k1p + (int64_t)jc * p.k1.sn + kk * 16 + hf * 8);
        vf[kk] = *(const X8*)(v1p + (int64_t)jc * p.v1.sn + kk * 16 + hf * 8);
    }
    floatx16 dkacc[C::DT], dvacc[C::DT];
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt) dkacc[dt] = dvacc[dt] = zeros16();

    const int j_last = j0 + WJ - 1 < N ? j0 + WJ - 1 : N - 1;
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
    ux4 fq[C::KR], fk[C::KR], fd[C::KR], fv[C::KR];
    float f_lse = 0.f, f_dsum = 0.f;
    auto fetch_unit = [&](int ib, int delta) {
#pragma unroll
        for (int u = 0; u < C::KR; ++u) {
            const int c = tid + WT * u;
            const int row = c / (D / 8), col = c - row * (D / 8);
            int i = ib * BQ + row;
            i = i < N ? i : N - 1;
            const int k = i - delta > 0 ? i - delta : 0;
            fq[u] = *(const ux4*)(qp + (int64_t)i * p.q.sn + col * 8);
            fk[u] = *(const ux4*)(k2p + (int64_t)k * p.k2.sn + col * 8);
            fd[u] = *(const ux4*)(dop + (int64_t)i * p.dout.sn + col * 8);
            fv[u] = *(const ux4*)(v2p + (int64_t)k * p.v2.sn + col * 8);
        }
        if (tid < 32) {
            int i = ib * BQ + tid;
            i = i < N ? i : N - 1;
            f_lse = p.lse[(int64_t)bh * N + i] * LOG2E;
            f_dsum = p.dsum[(int64_t)bh * N + i];
        }
    };
    auto store_unit = [&](int buf) {
        uint16_t* Qs = tiles + buf * C::STAGE;
        uint16_t* Ds = Qs + C::TILE;
#pragma unroll
        for (int u = 0; u < C::KR; ++u) {
            const int c = tid + WT * u;
            const int row = c / (D / 8), col = c - row * (D / 8);
            *(X8*)(Qs + row * C::RS + col * 8) = product8<E>(fq[u], fk[u], p.k2_bias, qscale);
            *(X8*)(Ds + row * C::RS + col * 8) = product8<E>(fd[u], fv[u], p.v2_bias, 1.f);
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
            const uint16_t* Qs = tiles + buf * C::STAGE;
            const uint16_t* Ds = Qs + C::TILE;
            const uint32_t Qt = tiles_addr + (uint32_t)(buf * C::STAGE * 2) + tr_lane + (uint32_t)(c0 * 2);
            const uint32_t Dt = Qt + (uint32_t)(C::TILE * 2);
            floatx16 sacc = zeros16(), dpacc = zeros16();
#pragma unroll
            for (int kk = 0; kk < C::DK; ++kk) {
                const X8 qa = *(const X8*)(Qs + ln * C::RS + kk * 16 + hf * 8);
                const X8 da = *(const X8*)(Ds + ln * C::RS + kk * 16 + hf * 8);
                sacc = E::mfma(qa, kf[kk], sacc, 0, 0, 0);
                dpacc = E::mfma(da, vf[kk], dpacc, 0, 0, 0);
            }
            // register v of this lane: query i0 + 8*(v/4) + 4*hf + v%4, key j
            const bool interior = (i0 >= jw + 31) && ((int64_t)i0 + 31 <= (int64_t)jw + w1) && (i0 + BQ - 1 < N) && (i0 >= delta);
            const int lo = j - i0 - 4 * hf;                                    // c >= lo  <=>  j <= i
            const int hi = (int)((int64_t)j + w1 - i0 < (1 << 20) ? j + w1 - i0 : (1 << 20)) - 4 * hf;   // i <= j + w1
            const int dlo = delta - i0 - 4 * hf, nhi = N - 1 - i0 - 4 * hf;
            X8 pb[2], dsb[2];
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const float4 ls = *(const float4*)(lse_s + buf * 32 + 8 * g4 + 4 * hf);
                const float4 dm = *(const float4*)(dsum_s + buf * 32 + 8 * g4 + 4 * hf);
                const float lsv[4] = {ls.x, ls.y, ls.z, ls.w}, dmv[4] = {dm.x, dm.y, dm.z, dm.w};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int v = 4 * g4 + t, c = 8 * g4 + t;
                    const bool valid = interior || ((j < N) && (c >= lo) && (c <= hi) && (c >= dlo) && (c <= nhi));
                    const float pv = valid ? fast_exp2(sacc[v] - lsv[t]) : 0.f;
                    pb[v >> 3][v & 7] = (EL)pv;
                    dsb[v >> 3][v & 7] = (EL)(pv * (dpacc[v] - dmv[t]));
                }
            }
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int dt = 0; dt < C::DT; ++dt) {
                    const uint32_t o = (uint32_t)(16 * ks * C::RSB + dt * 64);
                    dvacc[dt] = E::mfma(tr_operand<X8, C::RSB>(Dt + o), pb[ks], dvacc[dt], 0, 0, 0);
                    dkacc[dt] = E::mfma(tr_operand<X8, C::RSB>(Qt + o), dsb[ks], dkacc[dt], 0, 0, 0);
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

    if (j < N && SPLIT) {
        const int64_t BH = (int64_t)p.B * p.H;
        float* dkp = p.dk1.p ? part + (((0 * (int64_t)nsplit + sp) * BH + bh) * N + j) * D + c0 + 4 * hf : nullptr;
        float* dvp = p.dv1.p ? part + (((1 * (int64_t)nsplit + sp) * BH + bh) * N + j) * D + c0 + 4 * hf : nullptr;
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                if (dkp) *(float4*)(dkp + dt * 32 + 8 * g4) = make_float4(dkacc[dt][4 * g4] * LN2, dkacc[dt][4 * g4 + 1] * LN2,
                                                                           dkacc[dt][4 * g4 + 2] * LN2, dkacc[dt][4 * g4 + 3] * LN2);
                if (dvp) *(float4*)(dvp + dt * 32 + 8 * g4) = make_float4(dvacc[dt][4 * g4], dvacc[dt][4 * g4 + 1], dvacc[dt][4 * g4 + 2],
                                                                           dvacc[dt][4 * g4 + 3]);
            }
    } else if (j < N) {
        uint16_t* dkp = p.dk1.p ? (uint16_t*)p.dk1.p + p.dk1.off(b, j, h) + c0 + 4 * hf : nullptr;
        uint16_t* dvp = p.dv1.p ? (uint16_t*)p.dv1.p + p.dv1.off(b, j, h) + c0 + 4 * hf : nullptr;
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                // Q~ carries scale*log2(e): dK = ln2 * sum dS * Q~
                if (dkp) *(uint2*)(dkp + dt * 32 + 8 * g4) = make_uint2(E::pack(dkacc[dt][4 * g4] * LN2, dkacc[dt][4 * g4 + 1] * LN2),
                                                                         E::pack(dkacc[dt][4 * g4 + 2] * LN2, dkacc[dt][4 * g4 + 3] * LN2));
                if (dvp) *(uint2*)(dvp + dt * 32 + 8 * g4) = make_uint2(E::pack(dvacc[dt][4 * g4], dvacc[dt][4 * g4 + 1]),
                                                                         E::pack(dvacc[dt][4 * g4 + 2], dvacc[dt][4 * g4 + 3]));
            }
    }
}

// dK and dV from the partial sums of a split launch, shares added in their order
template <class E, int D>
__global__ __launch_bounds__(256) void wide_kv_sum_kernel(Problem p, int nsplit, const float* __restrict__ part, int64_t chunks) {
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
        *(uint2*)((uint16_t*)t.p + t.off(b, j, h) + col * 4) = make_uint2(E::pack(acc.x, acc.y), E::pack(acc.z, acc.w));
    }
}

// Shares a key block's query blocks are split into when the K-side grid is smaller than the chip
int wide_kv_nsplit(int B, int N, int H, int D, int w1, int w2, int npass) {
    const int64_t bh = (int64_t)B * H, base = bh * ((N + WJ - 1) / WJ) * npass;
    const int blocks = (WJ + (w1 < N ? w1 : N) + BQ - 1) / BQ + 1;
    const int64_t units = (int64_t)blocks * ((w2 < N - 1 ? w2 : N - 1) + 1);     // of a key block's stream, at most
    int ns = 1;                                                                  // shares of at least 8 units
    while (ns < 16 && base * ns * 2 <= 512 && (int64_t)ns * 2 * 8 <= units && (int64_t)2 * ns * 2 * bh * N * D * 4 <= ((int64_t)32 << 20))
        ns *= 2;
    return ns;
}
size_t wide_dq_part_bytes(int B, int N, int H, int D, int w2) {
    return ((size_t)B * H * ((N + BQ - 1) / BQ) * (size_t)(32 + w2) * D * sizeof(float) + 255) / 256 * 256;
}

// ------------------------------------------------------------------ launchers ----
template <class E, int D, int DV>
int launch_wide_fwd(const Problem& p, hipStream_t st) {
    using C = WideCfg<D, DV>;
    const int nqb = (p.N + BQ - 1) / BQ;
    const int64_t total = (int64_t)nqb * p.B * p.H;
    if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    if (!allow_full_lds((const void*)wide_fwd_kernel<E, D, DV>)) return SA2_ERR_LAUNCH_FAILED;
    hipLaunchKernelGGL((wide_fwd_kernel<E, D, DV>), dim3((unsigned)total, C::NPASS), dim3(WT), C::FWD_LDS, st, p, nqb, (int)total);
    return hipGetLastError() == hipSuccess ? SA2_OK : SA2_ERR_LAUNCH_FAILED;
}

template <class E, int D, int DV>
int launch_wide_bwd(const Problem& p, hipStream_t st) {
    using C = WideCfg<D, DV>;
    int rc = launch_rowdot(p.out, p.dout, p.dsum, p.B, p.N, p.H, p.D, E::DTYPE, st);
    if (rc != SA2_OK) return rc;
    if (p.dq.p || p.dk2.p || p.dv2.p) {
        const int nkb = (p.N + BQ - 1) / BQ;
        const int64_t total = (int64_t)nkb * p.B * p.H;
        if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
        if (p.scratch_bytes < wide_dq_part_bytes(p.B, p.N, p.H, D, p.w2)) return SA2_ERR_WORKSPACE_TOO_SMALL;
        float* part = (float*)p.scratch;
        if (!allow_full_lds((const void*)wide_kp_kernel<E, D, DV, false>) || !allow_full_lds((const void*)wide_kp_kernel<E, D, DV, true>))
            return SA2_ERR_LAUNCH_FAILED;
        const int segw = C::kp_segment(p.w2);
        if (segw < p.w2 + 1)
            hipLaunchKernelGGL((wide_kp_kernel<E, D, DV, true>), dim3((unsigned)total, C::NPASS), dim3(WT), C::kp_lds(segw - 1), st, p, nkb,
                               (int)total, part, segw);
        else
            hipLaunchKernelGGL((wide_kp_kernel<E, D, DV, false>), dim3((unsigned)total, C::NPASS), dim3(WT), C::kp_lds(segw - 1), st, p, nkb,
                               (int)total, part, segw);
        if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
        if (p.dq.p) {
            const int64_t chunks = (int64_t)p.B * p.H * p.N * (D / 4);
            hipLaunchKernelGGL((wide_dq_sum_kernel<E, D>), dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st, p, nkb, part, chunks);
            if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
        }
    }
    if (p.dk1.p || p.dv1.p) {
        const int njb = (p.N + WJ - 1) / WJ;
        const int nsplit = wide_kv_nsplit(p.B, p.N, p.H, D, p.w1, p.w2, C::NPASS);
        const int64_t total = (int64_t)njb * p.B * p.H * nsplit;
        if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
        float* kv_part = nullptr;
        if (nsplit > 1) {
            if (p.scratch_bytes < wide_bwd_scratch_bytes(p.B, p.N, p.H, D, p.w1, p.w2)) return SA2_ERR_WORKSPACE_TOO_SMALL;
            kv_part = (float*)((char*)p.scratch + wide_dq_part_bytes(p.B, p.N, p.H, D, p.w2));
        }
        if (!allow_full_lds((const void*)wide_kv_kernel<E, D, DV, false>) || !allow_full_lds((const void*)wide_kv_kernel<E, D, DV, true>))
            return SA2_ERR_LAUNCH_FAILED;
        if (nsplit > 1)
            hipLaunchKernelGGL((wide_kv_kernel<E, D, DV, true>), dim3((unsigned)total, C::NPASS), dim3(WT), C::KV_LDS, st, p, njb, (int)total,
                               nsplit, kv_part);
        else
            hipLaunchKernelGGL((wide_kv_kernel<E, D, DV, false>), dim3((unsigned)total, C::NPASS), dim3(WT), C::KV_LDS, st, p, njb, (int)total,
                               1, kv_part);
        if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
        if (nsplit > 1) {
            const int64_t chunks = (int64_t)p.B * p.H * p.N * (D / 4);
            hipLaunchKernelGGL((wide_kv_sum_kernel<E, D>), dim3((unsigned)((chunks + 255) / 256)), dim3(256), 0, st, p, nsplit, kv_part, chunks);
            if (hipGetLastError() != hipSuccess) return SA2_ERR_LAUNCH_FAILED;
        }
    }
    return SA2_OK;
}

}  // namespace

bool wide_supported(int D, int dtype) { return (dtype == SA2_BF16 || dtype == SA2_F16) && D == 256; }

bool wide_bwd_supported(int D, int w2, int dtype) {
    (void)w2;                // any K' window: wide ones are walked in segments
    return wide_supported(D, dtype);
}

size_t wide_bwd_scratch_bytes(int B, int N, int H, int D, int w1, int w2) {
    const int ns = wide_kv_nsplit(B, N, H, D, w1, w2, 2);
    return wide_dq_part_bytes(B, N, H, D, w2) + (ns > 1 ? (size_t)2 * ns * B * H * (size_t)N * D * sizeof(float) : 0);
}

int launch_wide_fwd(const Problem& p, int dtype, hipStream_t st) {
    return dtype == SA2_F16 ? launch_wide_fwd<ElemF16, 256, 128>(p, st) : launch_wide_fwd<ElemBF16, 256, 128>(p, st);
}

int launch_wide_bwd(const Problem& p, int dtype, hipStream_t st) {
    return dtype == SA2_F16 ? launch_wide_bwd<ElemF16, 256, 128>(p, st) : launch_wide_bwd<ElemBF16, 256, 128>(p, st);
}

}  // namespace sa2
