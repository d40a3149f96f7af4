// bf16 MFMA forward for gfx950, head_dim 64 or 128.
//
// Formulation: expand every query i by its K' window into rows r = (i, delta),
// delta = i - k in [0, w2], with Q~[r,:] = q[i,:] * (k2[i-delta,:] + k2_bias) *
// scale*log2(e), rounded to bf16.  Then s[r,j] = Q~[r].k1[j] and
// R[r,:] = sum_j p[r,j] v1[j,:] are sliding-window flash attention on the
// expanded rows (both contractions on v_mfma_f32_32x32x16_bf16, fp32 online
// softmax per row), and the rows of a query are merged at the end with a
// second online softmax:  O[i] = sum_delta e^{m_r-M} (v2[i-delta]+v2_bias) * R[r]
// / (L + 1e-8 e^{-M}).  No logit outside the K' window is ever computed.
//
// Work split: one workgroup (4 wavefronts) owns 32 consecutive queries of one
// (batch, head).  A "unit" is (delta, those 32 queries) = one 32-row MFMA
// N-tile.  A wavefront holds two units at a time (they share every K/V operand
// fetched from LDS) and sweeps the K window [i0-w1, i0+31] in 32-key tiles that
// the workgroup stages through double-buffered LDS: K row-major, V transposed
// and permuted so that each MFMA operand is one 16-byte LDS read.
//
// The logits are computed transposed (S^T = K1 . Q~^T) so that an expanded row
// lives in one lane (pair): row maxima and sums are in-lane reductions plus one
// exchange with lane^32, and exp2(S^T) is already laid out as the B operand of
// R^T = V^T . P^T.
#include "sa2_mfma_common.h"

namespace sa2 {
namespace {

template <int D>
struct Cfg {
    static constexpr int DK = D / 16;          // k-steps of the logit contraction
    static constexpr int DT = D / 32;          // 32-column tiles of the value contraction
    static constexpr int KS = D + 8;           // K tile row stride in LDS (bf16), +16 B against bank conflicts
    static constexpr int VS = TJ + 8;          // V^T tile row stride in LDS (bf16)
    static constexpr int K_ELEMS = TJ * KS;
    static constexpr int V_ELEMS = D * VS;
    static constexpr int STAGE = K_ELEMS + V_ELEMS;
    static constexpr int KR = TJ * D / 8 / NTHREADS;       // 16-byte K chunks per thread per tile
    static constexpr int NDP = D / 2;                       // column pairs of V
    static constexpr int VPASS = NDP / 32;                  // 4-row groups per thread per tile
    static constexpr int OS = D + 4;                        // merge buffer row stride (fp32)
    static constexpr int MERGE_FLOATS = 4 * (BQ * OS + 2 * BQ);
    static constexpr size_t STAGE_BYTES = (size_t)2 * STAGE * 2;          // two staging buffers
    static constexpr size_t LDS_BYTES = STAGE_BYTES + (size_t)MERGE_FLOATS * 4;
};

template <int D>
__global__ __launch_bounds__(NTHREADS) __attribute__((amdgpu_waves_per_eu(1, 1)))
void mfma_fwd_kernel(Problem p, int nqb, int total) {
    using C = Cfg<D>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t* smem = (uint16_t*)smem_raw;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, ln = lane & 31, hf = lane >> 5;

    // Workgroups are dealt round-robin to the 8 XCDs; remap so that the
    // neighbouring query blocks of one head (which share almost all of their
    // K/V window) run on the same XCD and meet in its L2.
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

    const int jt_lo = (i0 - w1 > 0 ? i0 - w1 : 0) / TJ;
    const int jt_hi = i_last / TJ;
    const int nt = jt_hi - jt_lo + 1;
    const int n_units = (w2 < i_last ? w2 : i_last) + 1;     // delta = 0 .. n_units-1
    const int npairs = (n_units + 1) >> 1;
    const int nrounds = (npairs + 3) >> 2;
    const int total_steps = nrounds * nt;

    // ---- staging of one K/V tile: global -> registers -> LDS ----------------
    uint4 kreg[C::KR];
    uint32_t vreg[C::VPASS * 4];
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
        }
#pragma unroll
        for (int ps = 0; ps < C::VPASS; ++ps) {
            const int grp = v_g0 + ps * (NTHREADS / C::NDP);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                int j = j0 + grp * 4 + r;
                j = j < N ? j : N - 1;
                vreg[ps * 4 + r] = *(const uint32_t*)(v1p + (int64_t)j * p.v1.sn + 2 * v_dp);
            }
        }
    };
    auto store_tile = [&](int buf) {
        uint16_t* Ks = smem + buf * C::STAGE;
        uint16_t* Vt = Ks + C::K_ELEMS;
#pragma unroll
        for (int u = 0; u < C::KR; ++u) {
            const int c = tid + NTHREADS * u;
            const int row = c / (D / 8), col = c - row * (D / 8);
            *(uint4*)(Ks + row * C::KS + col * 8) = kreg[u];
        }
#pragma unroll
        for (int ps = 0; ps < C::VPASS; ++ps) {
            const int grp = v_g0 + ps * (NTHREADS / C::NDP);
            // key j = 8g + 4hh + t of the tile sits at position (g/2)*16 + hh*8 + (g%2)*4 + t
            const int g = grp >> 1, hh = grp & 1;
            const int pos = (g >> 1) * 16 + hh * 8 + (g & 1) * 4;
            const uint32_t x0 = vreg[ps * 4], x1 = vreg[ps * 4 + 1], x2 = vreg[ps * 4 + 2], x3 = vreg[ps * 4 + 3];
            uint2 lo, hi;
            lo.x = (x0 & 0xffffu) | (x1 << 16);
            lo.y = (x2 & 0xffffu) | (x3 << 16);
            hi.x = (x0 >> 16) | (x1 & 0xffff0000u);
            hi.y = (x2 >> 16) | (x3 & 0xffff0000u);
            *(uint2*)(Vt + (2 * v_dp) * C::VS + pos) = lo;
            *(uint2*)(Vt + (2 * v_dp + 1) * C::VS + pos) = hi;
        }
    };

    // ---- per-wavefront state -------------------------------------------------
    // The query accumulators O (fp32, unnormalised, relative to Mrun) live in
    // LDS behind the staging buffers: they are touched once per unit, and the
    // registers they would take are what keeps the sweep free of AGPR copies.
    float* fm = (float*)(smem_raw + C::STAGE_BYTES);
    float* Om = fm + wave * (BQ * C::OS + 2 * BQ);
    float* Mm = Om + BQ * C::OS;
    float* Lm = Mm + BQ;
#pragma unroll
    for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
            *(float4*)(Om + ln * C::OS + dt * 32 + 8 * g4 + 4 * hf) = make_float4(0.f, 0.f, 0.f, 0.f);
    float Mrun = -INFINITY, Lrun = 0.f;

    const float qscale = p.scale * LOG2E;

    load_tile(jt_lo);
    store_tile(0);
    if (total_steps > 1) load_tile(jt_lo + (1 % nt));
    __syncthreads();

    int g = 0;
    for (int round = 0; round < nrounds; ++round) {
        const int pair = round * 4 + wave;
        const int delta0 = 2 * pair, delta1 = 2 * pair + 1;
        const bool ok0 = delta0 < n_units, ok1 = delta1 < n_units;

        if (!ok0) {
            // nothing to compute this round: keep the staging pipeline moving
            for (int s = 0; s < nt; ++s, ++g) {
                if (g + 1 < total_steps) store_tile((g + 1) & 1);
                if (g + 2 < total_steps) load_tile(jt_lo + (g + 2) % nt);
                __syncthreads();
            }
            continue;
        }

        // ---- new pair of units: Q~ operands, fresh running softmax ----------
        bf16x8 qf[2][C::DK];
        floatx16 racc[2][C::DT];
        float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                for (int v = 0; v < 16; ++v) racc[u][dt][v] = 0.f;
            int k = ic - (u ? delta1 : delta0);
            k = k > 0 ? k : 0;
#pragma unroll
            for (int kk = 0; kk < C::DK; ++kk) {
                const uint4 qa = *(const uint4*)(qp + (int64_t)ic * p.q.sn + kk * 16 + hf * 8);
                const uint4 kb = *(const uint4*)(k2p + (int64_t)k * p.k2.sn + kk * 16 + hf * 8);
                const uint32_t qw[4] = {qa.x, qa.y, qa.z, qa.w};
                const uint32_t kw[4] = {kb.x, kb.y, kb.z, kb.w};
                bf16x8 r;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    r[2 * t] = (__bf16)(bf16_lo(qw[t]) * (bf16_lo(kw[t]) + p.k2_bias) * qscale);
                    r[2 * t + 1] = (__bf16)(bf16_hi(qw[t]) * (bf16_hi(kw[t]) + p.k2_bias) * qscale);
                }
                qf[u][kk] = r;
            }
        }
        const bool rows_full0 = i0 >= delta0 && i0 + BQ - 1 < N;
        const bool rows_full1 = ok1 && i0 >= delta1 && i0 + BQ - 1 < N;
        const bool row_ok0 = i < N && i >= delta0;
        const bool row_ok1 = ok1 && i < N && i >= delta1;

        for (int s = 0; s < nt; ++s, ++g) {
            const int j0 = (jt_lo + s) * TJ;
            const uint16_t* Ks = smem + (g & 1) * C::STAGE;
            const uint16_t* Vt = Ks + C::K_ELEMS;
            // S^T tiles: rows = keys of the tile, columns = expanded rows
            floatx16 sacc[2];
#pragma unroll
            for (int u = 0; u < 2; ++u)
#pragma unroll
                for (int v = 0; v < 16; ++v) sacc[u][v] = 0.f;
#pragma unroll
            for (int kk = 0; kk < C::DK; ++kk) {
                const bf16x8 ka = *(const bf16x8*)(Ks + ln * C::KS + kk * 16 + hf * 8);
                sacc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[0][kk], sacc[0], 0, 0, 0);
                sacc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka, qf[1][kk], sacc[1], 0, 0, 0);
            }
            const bool interior = (j0 + TJ - 1 <= i0) && (j0 >= i0 + BQ - 1 - w1);
            bf16x8 pb[2][2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                float pv[16];
#pragma unroll
                for (int v = 0; v < 16; ++v) pv[v] = sacc[u][v];
                if (__builtin_expect(!(interior && (u ? rows_full1 : rows_full0)), 0)) {
                    // element v of this lane is key j0 + 8*(v/4) + 4*hf + v%4
                    const bool row_ok = u ? row_ok1 : row_ok0;
                    const int hi = i - j0 - 4 * hf, lo = hi - w1;
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int c = 8 * (v >> 2) + (v & 3);
                        pv[v] = (row_ok && c <= hi && c >= lo) ? pv[v] : -INFINITY;
                    }
                }
                float mx = fmaxf(pv[0], pv[1]);
#pragma unroll
                for (int v = 2; v < 16; ++v) mx = fmaxf(mx, pv[v]);
                mx = fmaxf(mx, other_half(mx));
                // Lazy reference point: move it only when the maximum grows by more
                // than 2^RESCALE_LOG2, so the accumulator rescale is rare; weights
                // stay below 2^RESCALE_LOG2 and every later formula only needs m to
                // be a common reference, not the exact maximum.
                if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx > m[u] + RESCALE_LOG2) != 0, 0)) {
                    const float m_new = (mx > m[u] + RESCALE_LOG2) ? mx : m[u];
                    const float alpha = fast_exp2(m[u] - ((m_new == -INFINITY) ? 0.f : m_new));
                    m[u] = m_new;
                    l[u] *= alpha;
                    asm volatile("s_nop 15\n\ts_nop 15");
#pragma unroll
                    for (int dt = 0; dt < C::DT; ++dt) scale_acc(racc[u][dt], alpha);
                    asm volatile("s_nop 4");
                }
                const float m_use = (m[u] == -INFINITY) ? 0.f : m[u];
                float rs = 0.f;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    pv[v] = fast_exp2(pv[v] - m_use);
                    rs += pv[v];
                }
                l[u] += rs;
#pragma unroll
                for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                    for (int t = 0; t < 8; ++t) pb[u][ks][t] = (__bf16)pv[ks * 8 + t];
            }
            // R^T += V^T . P^T
#pragma unroll
            for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
                for (int ks = 0; ks < 2; ++ks) {
                    const bf16x8 va = *(const bf16x8*)(Vt + (dt * 32 + ln) * C::VS + ks * 16 + hf * 8);
                    racc[0][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[0][ks], racc[0][dt], 0, 0, 0);
                    racc[1][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, pb[1][ks], racc[1][dt], 0, 0, 0);
                }

            if (g + 1 < total_steps) store_tile((g + 1) & 1);
            if (g + 2 < total_steps) load_tile(jt_lo + (g + 2) % nt);
            __syncthreads();
        }

        // ---- fold the finished units into the query accumulators ------------
        float a_all = 1.f, bb[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const float lt = l[u] + other_half(l[u]);
            const float Mn = fmaxf(Mrun, m[u]);
            const float Muse = (Mn == -INFINITY) ? 0.f : Mn;
            const float a = fast_exp2(Mrun - Muse);
            bb[u] = fast_exp2(m[u] - Muse);
            // unit 0's factor must also shrink by unit 1's rescale of the accumulator
            if (u == 1) bb[0] *= a;
            a_all *= a;
            Lrun = Lrun * a + lt * bb[u];
            Mrun = Mn;
        }
        int kr0 = ic - delta0, kr1 = ic - delta1;
        kr0 = kr0 > 0 ? kr0 : 0;
        kr1 = kr1 > 0 ? kr1 : 0;
        const uint16_t* vrow0 = v2p + (int64_t)kr0 * p.v2.sn + 4 * hf;
        const uint16_t* vrow1 = v2p + (int64_t)kr1 * p.v2.sn + 4 * hf;
#pragma unroll
        for (int dt = 0; dt < C::DT; ++dt)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const uint2 x0 = *(const uint2*)(vrow0 + dt * 32 + 8 * g4);
                const uint2 x1 = *(const uint2*)(vrow1 + dt * 32 + 8 * g4);
                float* op = Om + ln * C::OS + dt * 32 + 8 * g4 + 4 * hf;
                float4 o = *(float4*)op;
                const float b0 = bb[0], b1 = bb[1];
                o.x = o.x * a_all + b0 * racc[0][dt][4 * g4 + 0] * (bf16_lo(x0.x) + p.v2_bias) +
                      b1 * racc[1][dt][4 * g4 + 0] * (bf16_lo(x1.x) + p.v2_bias);
                o.y = o.y * a_all + b0 * racc[0][dt][4 * g4 + 1] * (bf16_hi(x0.x) + p.v2_bias) +
                      b1 * racc[1][dt][4 * g4 + 1] * (bf16_hi(x1.x) + p.v2_bias);
                o.z = o.z * a_all + b0 * racc[0][dt][4 * g4 + 2] * (bf16_lo(x0.y) + p.v2_bias) +
                      b1 * racc[1][dt][4 * g4 + 2] * (bf16_lo(x1.y) + p.v2_bias);
                o.w = o.w * a_all + b0 * racc[0][dt][4 * g4 + 3] * (bf16_hi(x0.y) + p.v2_bias) +
                      b1 * racc[1][dt][4 * g4 + 3] * (bf16_hi(x1.y) + p.v2_bias);
                *(float4*)op = o;
            }
    }

    // ---- merge the four wavefronts' partial (M, L, O) through LDS ------------
    if (hf == 0) {
        Mm[ln] = Mrun;
        Lm[ln] = Lrun;
    }
    __syncthreads();

    constexpr int CH = D / 8;                 // output columns per thread
    const int qi = tid >> 3, dc = (tid & 7) * CH;
    const int io = i0 + qi;
    if (io < N) {
        float Mw[4], Ms = -INFINITY;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            Mw[w] = fm[w * (BQ * C::OS + 2 * BQ) + BQ * C::OS + qi];
            Ms = fmaxf(Ms, Mw[w]);
        }
        float cw[4], L = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            cw[w] = fast_exp2(Mw[w] - Ms);    // a wavefront without units has M = -inf -> weight 0
            L += cw[w] * fm[w * (BQ * C::OS + 2 * BQ) + BQ * C::OS + BQ + qi];
        }
        const float inv = 1.f / (L + 1e-8f * fast_exp2(-Ms));
        uint16_t* orow = (uint16_t*)p.out.p + p.out.off(b, io, h) + dc;
#pragma unroll
        for (int c4 = 0; c4 < CH; c4 += 8) {
            bf16x8 r;
#pragma unroll
            for (int t4 = 0; t4 < 8; t4 += 4) {
                float4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const float4 x = *(const float4*)(fm + w * (BQ * C::OS + 2 * BQ) + qi * C::OS + dc + c4 + t4);
                    acc.x += cw[w] * x.x;
                    acc.y += cw[w] * x.y;
                    acc.z += cw[w] * x.z;
                    acc.w += cw[w] * x.w;
                }
                r[t4 + 0] = (__bf16)(acc.x * inv);
                r[t4 + 1] = (__bf16)(acc.y * inv);
                r[t4 + 2] = (__bf16)(acc.z * inv);
                r[t4 + 3] = (__bf16)(acc.w * inv);
            }
            *(bf16x8*)(orow + c4) = r;
        }
        if ((tid & 7) == 0) {
            float lse;
            if (Ms > LOG2_EPS) lse = LN2 * (Ms + __log2f(L + 1e-8f * fast_exp2(-Ms)));
            else lse = LN_EPS + log1pf(L * fast_exp2(Ms - LOG2_EPS));
            p.lse[(int64_t)bh * N + io] = lse;
        }
    }
}

bool aligned16(const Tensor& t, int B, int N, int H) {
    if (!t.p) return true;
    if ((uintptr_t)t.p & 15u) return false;
    if (B > 1 && (t.sb & 7)) return false;
    if (N > 1 && (t.sn & 7)) return false;
    if (H > 1 && (t.sh & 7)) return false;
    return true;
}

}  // namespace

bool mfma_supported(int B, int N, int H, int D, int w1, int w2, int dtype) {
    (void)B; (void)H; (void)w1; (void)w2; (void)N;
    return dtype == SA2_BF16 && (D == 64 || D == 128);
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

int launch_mfma_fwd(const Problem& p, hipStream_t st) {
    const int nqb = (p.N + BQ - 1) / BQ;
    const int64_t total = (int64_t)nqb * p.B * p.H;
    if (total > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    if (p.D == 128) {
        using C = Cfg<128>;
        if (hipFuncSetAttribute((const void*)mfma_fwd_kernel<128>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)C::LDS_BYTES) != hipSuccess)
            return SA2_ERR_LAUNCH_FAILED;
        hipLaunchKernelGGL(mfma_fwd_kernel<128>, dim3((unsigned)total), dim3(NTHREADS), C::LDS_BYTES, st, p, nqb,
                           (int)total);
    } else {
        using C = Cfg<64>;
        if (hipFuncSetAttribute((const void*)mfma_fwd_kernel<64>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)C::LDS_BYTES) != hipSuccess)
            return SA2_ERR_LAUNCH_FAILED;
        hipLaunchKernelGGL(mfma_fwd_kernel<64>, dim3((unsigned)total), dim3(NTHREADS), C::LDS_BYTES, st, p, nqb,
                           (int)total);
    }
    return hipGetLastError() == hipSuccess ? SA2_OK : SA2_ERR_LAUNCH_FAILED;
}

}  // namespace sa2
