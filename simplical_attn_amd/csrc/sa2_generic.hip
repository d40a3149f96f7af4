// Generic fp32-FMA kernels: any element type (fp32 / bf16 / fp16 I/O), any
// D <= 256, any window.  All arithmetic is fp32 with accurate expf/logf, so
// this path carries the 1e-5 parity bar of the fp32 configuration and serves
// every shape the MFMA kernels do not take.
//
// Work split: one wavefront owns one row of the quantity it produces (an
// output row, a dQ row, a dK/dV row or a dK'/dV' row) and sweeps the rows it
// interacts with in 64-wide tiles staged in LDS; lanes map to the 64 inner
// keys for the logit and to the D columns for the accumulation.  Every result
// row has exactly one writer: no atomics, bitwise reproducible.
#include <type_traits>

#include "sa2_common.h"

namespace sa2 {
namespace {

constexpr int ROWS_PER_BLOCK = 4;   // wavefronts per workgroup, one owned row each
constexpr int TILE = 64;            // inner keys per LDS tile (one per lane)
constexpr int MAXC = 4;             // ceil(256 / 64) column slots per lane

__device__ __forceinline__ int imax(int a, int b) { return a > b ? a : b; }
__device__ __forceinline__ int imin(int a, int b) { return a < b ? a : b; }

// Stage rows [r0, r0+TILE) of key tensor `kt` and value tensor `vt` (+bias)
// into LDS as fp32, zero-filled outside [lo, hi] and beyond D.
template <typename T>
__device__ __forceinline__ void stage_tile(const Tensor& kt, const Tensor& vt, float kbias, float vbias,
                                           int b, int h, int r0, int lo, int hi, int D, int D4, int DP,
                                           float* Ks, float* Vs) {
    const T* kp = (const T*)kt.p;
    const T* vp = (const T*)vt.p;
    for (int idx = threadIdx.x; idx < TILE * D4; idx += blockDim.x) {
        const int r = idx / D4, d = idx - r * D4;
        const int row = r0 + r;
        float kv = 0.f, vv = 0.f;
        if (row >= lo && row <= hi && d < D) {
            kv = to_float(kp[kt.off(b, row, h) + d]) + kbias;
            vv = to_float(vp[vt.off(b, row, h) + d]) + vbias;
        }
        Ks[r * DP + d] = kv;
        Vs[r * DP + d] = vv;
    }
}

__device__ __forceinline__ float dot_row(const float* a, const float* row, int D4) {
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int d = 0; d < D4; d += 4) {
        const float4 x = *(const float4*)(a + d);
        const float4 y = *(const float4*)(row + d);
        s0 = fmaf(x.x, y.x, s0);
        s1 = fmaf(x.y, y.y, s1);
        s2 = fmaf(x.z, y.z, s2);
        s3 = fmaf(x.w, y.w, s3);
    }
    return (s0 + s1) + (s2 + s3);
}

struct Smem {
    float *Ks, *Vs, *a_s, *b_s, *p_s, *ds_s;
};
__device__ __forceinline__ Smem carve(float* base, int D4, int DP, int wave) {
    Smem s;
    s.Ks = base;
    s.Vs = s.Ks + TILE * DP;
    float* per_wave = s.Vs + TILE * DP;
    s.a_s = per_wave + wave * (2 * D4 + 2 * TILE);
    s.b_s = s.a_s + D4;
    s.p_s = s.b_s + D4;
    s.ds_s = s.p_s + TILE;
    return s;
}
size_t smem_bytes(int D) {
    const int D4 = (D + 3) & ~3, DP = D4 + 4;
    return sizeof(float) * (size_t)(2 * TILE * DP + ROWS_PER_BLOCK * (2 * D4 + 2 * TILE));
}

// ---------------------------------------------------------------- forward ----
template <typename T>
__global__ __launch_bounds__(ROWS_PER_BLOCK * 64) void generic_fwd_kernel(Problem p, int nblk) {
    extern __shared__ float smem[];
    const int D = p.D, D4 = (D + 3) & ~3, DP = D4 + 4, N = p.N;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const Smem sm = carve(smem, D4, DP, wave);
    const int bh = blockIdx.x / nblk, blk = blockIdx.x - bh * nblk;
    const int b = bh / p.H, h = bh - b * p.H;
    const int i_base = blk * ROWS_PER_BLOCK;
    const int i = i_base + wave;
    const bool active = i < N;
    const int nc = (D + 63) >> 6;

    const T* qp = (const T*)p.q.p;
    const T* k2p = (const T*)p.k2.p;
    const T* v2p = (const T*)p.v2.p;

    float qreg[MAXC], acc[MAXC];
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int d = lane + 64 * c;
        acc[c] = 0.f;
        qreg[c] = (active && d < D) ? to_float(qp[p.q.off(b, i, h) + d]) * p.scale : 0.f;
    }
    float m = -INFINITY, l = 0.f;

    const int j_lo_blk = imax(0, i_base - p.w1), j_hi_blk = imin(N - 1, i_base + ROWS_PER_BLOCK - 1);
    const int j_lo = imax(0, i - p.w1), k_lo = imax(0, i - p.w2);

    for (int jc = j_lo_blk; jc <= j_hi_blk; jc += TILE) {
        __syncthreads();
        stage_tile<T>(p.k1, p.v1, 0.f, 0.f, b, h, jc, j_lo_blk, j_hi_blk, D, D4, DP, sm.Ks, sm.Vs);
        __syncthreads();
        if (!active || jc > i || jc + TILE - 1 < j_lo) continue;
        const int j = jc + lane;
        const bool valid = j >= j_lo && j <= i;
        const int x_lo = imax(j_lo, jc) - jc, x_hi = imin(i, jc + TILE - 1) - jc;
        for (int k = k_lo; k <= i; ++k) {
            float v2r[MAXC];
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                const int d = lane + 64 * c;
                v2r[c] = 0.f;
                if (c < nc && d < D4) {
                    float kk = 0.f;
                    if (d < D) {
                        kk = to_float(k2p[p.k2.off(b, k, h) + d]) + p.k2_bias;
                        v2r[c] = to_float(v2p[p.v2.off(b, k, h) + d]) + p.v2_bias;
                    }
                    sm.a_s[d] = qreg[c] * kk;
                }
            }
            __builtin_amdgcn_wave_barrier();
            float s = dot_row(sm.a_s, sm.Ks + lane * DP, D4);
            s = valid ? s : -INFINITY;
            const float m_new = fmaxf(m, wave_max(s));
            const float alpha = expf(m - m_new);
            const float pj = valid ? expf(s - m_new) : 0.f;
            l = l * alpha + wave_sum(pj);
            m = m_new;
            sm.p_s[lane] = pj;
            __builtin_amdgcn_wave_barrier();
            float t[MAXC] = {0.f, 0.f, 0.f, 0.f};
            for (int x = x_lo; x <= x_hi; ++x) {
                const float px = sm.p_s[x];
#pragma unroll
                for (int c = 0; c < MAXC; ++c)
                    if (c < nc) t[c] = fmaf(px, sm.Vs[x * DP + imin(lane + 64 * c, D4 - 1)], t[c]);
            }
#pragma unroll
            for (int c = 0; c < MAXC; ++c) acc[c] = fmaf(t[c], v2r[c], acc[c] * alpha);
            __builtin_amdgcn_wave_barrier();
        }
    }
    if (!active) return;
    const float denom = l + 1e-8f * expf(-m);
    T* op = (T*)p.out.p;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int d = lane + 64 * c;
        if (c < nc && d < D) from_float(acc[c] / denom, op + p.out.off(b, i, h) + d);
    }
    if (lane == 0) p.lse[(int64_t)bh * N + i] = lse_with_eps(m, l);
}

// --------------------------------------------------------------- backward ----
// One expanded pair (query i, outer key o): logits against the staged inner
// tile, P and dS from the saved LSE, then
//   g[d] = sum_x dS[x] * Xs[x][d]     r[d] = sum_x P[x] * Ys[x][d].
template <bool NEED_R>
__device__ __forceinline__ void pair_pass(const Smem& sm, int lane, int DP, int D4, int nc, bool valid,
                                          int x_lo, int x_hi, float lse_i, float dsum_i,
                                          float* g, float* r) {
    __builtin_amdgcn_wave_barrier();
    const float s = dot_row(sm.a_s, sm.Ks + lane * DP, D4);
    const float dp = dot_row(sm.b_s, sm.Vs + lane * DP, D4);
    const float pj = valid ? expf(s - lse_i) : 0.f;
    sm.p_s[lane] = pj;
    sm.ds_s[lane] = pj * (dp - dsum_i);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int c = 0; c < MAXC; ++c) g[c] = r[c] = 0.f;
    for (int x = x_lo; x <= x_hi; ++x) {
        const float px = sm.p_s[x], dsx = sm.ds_s[x];
#pragma unroll
        for (int c = 0; c < MAXC; ++c)
            if (c < nc) {
                const int d = imin(lane + 64 * c, D4 - 1);
                g[c] = fmaf(dsx, sm.Ks[x * DP + d], g[c]);
                if (NEED_R) r[c] = fmaf(px, sm.Vs[x * DP + d], r[c]);
            }
    }
    __builtin_amdgcn_wave_barrier();
}

// dQ: one wavefront per query row.
template <typename T>
__global__ __launch_bounds__(ROWS_PER_BLOCK * 64) void generic_bwd_dq_kernel(Problem p, int nblk) {
    extern __shared__ float smem[];
    const int D = p.D, D4 = (D + 3) & ~3, DP = D4 + 4, N = p.N;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const Smem sm = carve(smem, D4, DP, wave);
    const int bh = blockIdx.x / nblk, blk = blockIdx.x - bh * nblk;
    const int b = bh / p.H, h = bh - b * p.H;
    const int i_base = blk * ROWS_PER_BLOCK;
    const int i = i_base + wave;
    const bool active = i < N;
    const int nc = (D + 63) >> 6;
    const T* k2p = (const T*)p.k2.p;
    const T* v2p = (const T*)p.v2.p;

    float qreg[MAXC], doreg[MAXC], dq[MAXC];
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int d = lane + 64 * c;
        const bool ok = active && d < D;
        dq[c] = 0.f;
        qreg[c] = ok ? to_float(((const T*)p.q.p)[p.q.off(b, i, h) + d]) * p.scale : 0.f;
        doreg[c] = ok ? to_float(((const T*)p.dout.p)[p.dout.off(b, i, h) + d]) : 0.f;
    }
    const float lse_i = active ? p.lse[(int64_t)bh * N + i] : 0.f;
    const float dsum_i = active ? p.dsum[(int64_t)bh * N + i] : 0.f;
    const int j_lo_blk = imax(0, i_base - p.w1), j_hi_blk = imin(N - 1, i_base + ROWS_PER_BLOCK - 1);
    const int j_lo = imax(0, i - p.w1), k_lo = imax(0, i - p.w2);

    for (int jc = j_lo_blk; jc <= j_hi_blk; jc += TILE) {
        __syncthreads();
        stage_tile<T>(p.k1, p.v1, 0.f, 0.f, b, h, jc, j_lo_blk, j_hi_blk, D, D4, DP, sm.Ks, sm.Vs);
        __syncthreads();
        if (!active || jc > i || jc + TILE - 1 < j_lo) continue;
        const int j = jc + lane;
        const bool valid = j >= j_lo && j <= i;
        const int x_lo = imax(j_lo, jc) - jc, x_hi = imin(i, jc + TILE - 1) - jc;
        for (int k = k_lo; k <= i; ++k) {
            float k2r[MAXC];
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                const int d = lane + 64 * c;
                k2r[c] = 0.f;
                if (c < nc && d < D4) {
                    float vv = 0.f;
                    if (d < D) {
                        k2r[c] = to_float(k2p[p.k2.off(b, k, h) + d]) + p.k2_bias;
                        vv = to_float(v2p[p.v2.off(b, k, h) + d]) + p.v2_bias;
                    }
                    sm.a_s[d] = qreg[c] * k2r[c];
                    sm.b_s[d] = doreg[c] * vv;
                }
            }
            float g[MAXC], r[MAXC];
            pair_pass<false>(sm, lane, DP, D4, nc, valid, x_lo, x_hi, lse_i, dsum_i, g, r);
#pragma unroll
            for (int c = 0; c < MAXC; ++c) dq[c] = fmaf(g[c], k2r[c] * p.scale, dq[c]);
        }
    }
    if (!active) return;
    T* gp = (T*)p.dq.p;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int d = lane + 64 * c;
        if (c < nc && d < D) from_float(dq[c], gp + p.dq.off(b, i, h) + d);
    }
}

// Gradients of one key/value pair (the "owner" side), one wavefront per owner
// row o.  Queries i in [o, o+w_own] attend to it; for each such query the other
// ("inner") pair is swept over its window [i-w_in, i].  With owner = (k1,v1),
// inner = (k2,v2) this produces dK, dV; with the roles swapped, dK', dV'.
struct OwnerArgs {
    Tensor own_k, own_v, in_k, in_v, d_own_k, d_own_v;
    float own_kbias, own_vbias, in_kbias, in_vbias;
    int w_own, w_in;
};
template <typename T>
__global__ __launch_bounds__(ROWS_PER_BLOCK * 64) void generic_bwd_owner_kernel(Problem p, OwnerArgs a, int nblk) {
    extern __shared__ float smem[];
    const int D = p.D, D4 = (D + 3) & ~3, DP = D4 + 4, N = p.N;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const Smem sm = carve(smem, D4, DP, wave);
    const int bh = blockIdx.x / nblk, blk = blockIdx.x - bh * nblk;
    const int b = bh / p.H, h = bh - b * p.H;
    const int o_base = blk * ROWS_PER_BLOCK;
    const int o = o_base + wave;
    const bool active = o < N;
    const int nc = (D + 63) >> 6;
    const T* qp = (const T*)p.q.p;
    const T* dop = (const T*)p.dout.p;

    float okreg[MAXC], ovreg[MAXC], dk[MAXC], dv[MAXC];
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int d = lane + 64 * c;
        const bool ok = active && d < D;
        dk[c] = dv[c] = 0.f;
        okreg[c] = ok ? (to_float(((const T*)a.own_k.p)[a.own_k.off(b, o, h) + d]) + a.own_kbias) * p.scale : 0.f;
        ovreg[c] = ok ? to_float(((const T*)a.own_v.p)[a.own_v.off(b, o, h) + d]) + a.own_vbias : 0.f;
    }
    const int x_lo_blk = imax(0, o_base - a.w_in);
    const int x_hi_blk = imin(N - 1, imin(N - 1, o_base + ROWS_PER_BLOCK - 1) + a.w_own);
    const int i_last = imin(N - 1, o + a.w_own);

    for (int xc = x_lo_blk; xc <= x_hi_blk; xc += TILE) {
        __syncthreads();
        stage_tile<T>(a.in_k, a.in_v, a.in_kbias, a.in_vbias, b, h, xc, x_lo_blk, x_hi_blk, D, D4, DP, sm.Ks, sm.Vs);
        __syncthreads();
        if (!active) continue;
        const int i_first = imax(o, xc);
        const int i_end = imin(i_last, (int)imin((int64_t)N - 1, (int64_t)xc + TILE - 1 + a.w_in));
        const int x = xc + lane;
        for (int i = i_first; i <= i_end; ++i) {
            float qr[MAXC], dor[MAXC];
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                const int d = lane + 64 * c;
                qr[c] = dor[c] = 0.f;
                if (c < nc && d < D4) {
                    if (d < D) {
                        qr[c] = to_float(qp[p.q.off(b, i, h) + d]);
                        dor[c] = to_float(dop[p.dout.off(b, i, h) + d]);
                    }
                    sm.a_s[d] = qr[c] * okreg[c];
                    sm.b_s[d] = dor[c] * ovreg[c];
                }
            }
            const int in_lo = imax(0, i - a.w_in);
            const bool valid = x >= in_lo && x <= i;
            const int x_lo = imax(in_lo, xc) - xc, x_hi = imin(i, xc + TILE - 1) - xc;
            const float lse_i = p.lse[(int64_t)bh * N + i];
            const float dsum_i = p.dsum[(int64_t)bh * N + i];
            float g[MAXC], r[MAXC];
            pair_pass<true>(sm, lane, DP, D4, nc, valid, x_lo, x_hi, lse_i, dsum_i, g, r);
#pragma unroll
            for (int c = 0; c < MAXC; ++c) {
                dk[c] = fmaf(g[c], qr[c] * p.scale, dk[c]);
                dv[c] = fmaf(r[c], dor[c], dv[c]);
            }
        }
    }
    if (!active) return;
#pragma unroll
    for (int c = 0; c < MAXC; ++c) {
        const int d = lane + 64 * c;
        if (c < nc && d < D) {
            if (a.d_own_k.p) from_float(dk[c], (T*)a.d_own_k.p + a.d_own_k.off(b, o, h) + d);
            if (a.d_own_v.p) from_float(dv[c], (T*)a.d_own_v.p + a.d_own_v.off(b, o, h) + d);
        }
    }
}

// dsum[b,h,i] = sum_d dout*out, one wavefront per row.
template <typename T>
__global__ __launch_bounds__(256) void rowdot_kernel(Tensor out, Tensor dout, float* dsum, int N, int H, int D,
                                                     int64_t rows) {
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int lane = threadIdx.x & 63;
    const int i = (int)(row % N);
    const int bh = (int)(row / N);
    const int b = bh / H, h = bh - b * H;
    const T* op = (const T*)out.p + out.off(b, i, h);
    const T* gp = (const T*)dout.p + dout.off(b, i, h);
    float s = 0.f;
    for (int d = lane; d < D; d += 64) s = fmaf(to_float(op[d]), to_float(gp[d]), s);
    s = wave_sum(s);
    if (lane == 0) dsum[row] = s;
}

// The same for 16-bit elements with 16-byte aligned rows and D = 8 << n: a lane takes eight
// consecutive elements of a row in one 16-byte load per tensor, D / 8 lanes share a row, a
// wavefront covers 512 / D rows.
template <typename T>
__global__ __launch_bounds__(256) void rowdot_vec_kernel(Tensor out, Tensor dout, float* dsum, int N, int H, int lpr_log2,
                                                         int64_t rows) {
    const int lane = threadIdx.x & 63;
    const int lpr = 1 << lpr_log2;                        // lanes per row
    const int64_t row = (((int64_t)blockIdx.x * 4 + (threadIdx.x >> 6)) << (6 - lpr_log2)) + (lane >> lpr_log2);
    const int sub = lane & (lpr - 1);
    float s = 0.f;
    if (row < rows) {
        const int i = (int)(row % N);
        const int bh = (int)(row / N);
        const int b = bh / H, h = bh - b * H;
        const uint4 o = *(const uint4*)((const T*)out.p + out.off(b, i, h) + sub * 8);
        const uint4 g = *(const uint4*)((const T*)dout.p + dout.off(b, i, h) + sub * 8);
        const uint32_t ow[4] = {o.x, o.y, o.z, o.w}, gw[4] = {g.x, g.y, g.z, g.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            union { uint32_t u; T h[2]; } a, c;
            a.u = ow[t];
            c.u = gw[t];
            s = fmaf(to_float(a.h[0]), to_float(c.h[0]), s);
            s = fmaf(to_float(a.h[1]), to_float(c.h[1]), s);
        }
    }
    for (int off = lpr >> 1; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if (row < rows && sub == 0) dsum[row] = s;
}

template <typename F>
int dispatch_dtype(int dtype, F&& f) {
    switch (dtype) {
        case SA2_F32: return f((float*)nullptr);
        case SA2_BF16: return f((bf16_t*)nullptr);
        case SA2_F16: return f((f16_t*)nullptr);
    }
    return SA2_ERR_BAD_DTYPE;
}

int check_launch() { return hipGetLastError() == hipSuccess ? SA2_OK : SA2_ERR_LAUNCH_FAILED; }

template <typename K>
bool allow_big_lds(K kernel, size_t bytes) {
    return bytes <= 64 * 1024 || allow_full_lds((const void*)kernel);
}

}  // namespace

int launch_rowdot(const Tensor& out, const Tensor& dout, float* dsum, int B, int N, int H, int D, int dtype,
                  hipStream_t st) {
    const int64_t rows = (int64_t)B * H * N;
    const int64_t blocks = (rows + 3) / 4;
    if (blocks > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    // 16-bit elements, D = 8, 16, .. 256 and 16-byte aligned rows: the vector kernel
    auto aligned = [&](const Tensor& t) {
        return ((uintptr_t)t.p & 15u) == 0 && (B == 1 || t.sb % 8 == 0) && (N == 1 || t.sn % 8 == 0) && (H == 1 || t.sh % 8 == 0);
    };
    int lpr_log2 = -1;
    for (int n = 0; n <= 5; ++n)
        if (D == (8 << n)) lpr_log2 = n;
    const bool vec = dtype != SA2_F32 && lpr_log2 >= 0 && aligned(out) && aligned(dout);
    return dispatch_dtype(dtype, [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if constexpr (sizeof(T) == 2) {
            if (vec) {
                const int64_t per_block = (int64_t)4 << (6 - lpr_log2);           // rows per workgroup
                const int64_t vblocks = (rows + per_block - 1) / per_block;
                hipLaunchKernelGGL(rowdot_vec_kernel<T>, dim3((unsigned)vblocks), dim3(256), 0, st, out, dout, dsum, N, H,
                                   lpr_log2, rows);
                return check_launch();
            }
        }
        hipLaunchKernelGGL(rowdot_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, st, out, dout, dsum, N, H, D, rows);
        return check_launch();
    });
}

int launch_generic_fwd(const Problem& p, int dtype, hipStream_t st) {
    const int nblk = (p.N + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
    const int64_t blocks = (int64_t)nblk * p.B * p.H;
    if (blocks > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    const size_t lds = smem_bytes(p.D);
    return dispatch_dtype(dtype, [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        if (!allow_big_lds(generic_fwd_kernel<T>, lds)) return (int)SA2_ERR_LAUNCH_FAILED;
        hipLaunchKernelGGL(generic_fwd_kernel<T>, dim3((unsigned)blocks), dim3(ROWS_PER_BLOCK * 64), lds, st, p, nblk);
        return check_launch();
    });
}

size_t generic_bwd_scratch_bytes(int, int, int, int, int, int) { return 0; }

int launch_generic_bwd(const Problem& p, int dtype, hipStream_t st) {
    const int nblk = (p.N + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK;
    const int64_t blocks = (int64_t)nblk * p.B * p.H;
    if (blocks > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    const size_t lds = smem_bytes(p.D);
    int rc = launch_rowdot(p.out, p.dout, p.dsum, p.B, p.N, p.H, p.D, dtype, st);
    if (rc != SA2_OK) return rc;
    return dispatch_dtype(dtype, [&](auto* tag) {
        using T = std::remove_pointer_t<decltype(tag)>;
        const dim3 grid((unsigned)blocks), block(ROWS_PER_BLOCK * 64);
        if (p.dq.p) {
            if (!allow_big_lds(generic_bwd_dq_kernel<T>, lds)) return (int)SA2_ERR_LAUNCH_FAILED;
            hipLaunchKernelGGL(generic_bwd_dq_kernel<T>, grid, block, lds, st, p, nblk);
            if (check_launch() != SA2_OK) return (int)SA2_ERR_LAUNCH_FAILED;
        }
        if (!allow_big_lds(generic_bwd_owner_kernel<T>, lds)) return (int)SA2_ERR_LAUNCH_FAILED;
        if (p.dk1.p || p.dv1.p) {
            OwnerArgs a{p.k1, p.v1, p.k2, p.v2, p.dk1, p.dv1, 0.f, 0.f, p.k2_bias, p.v2_bias, p.w1, p.w2};
            hipLaunchKernelGGL(generic_bwd_owner_kernel<T>, grid, block, lds, st, p, a, nblk);
            if (check_launch() != SA2_OK) return (int)SA2_ERR_LAUNCH_FAILED;
        }
        if (p.dk2.p || p.dv2.p) {
            OwnerArgs a{p.k2, p.v2, p.k1, p.v1, p.dk2, p.dv2, p.k2_bias, p.v2_bias, 0.f, 0.f, p.w2, p.w1};
            hipLaunchKernelGGL(generic_bwd_owner_kernel<T>, grid, block, lds, st, p, a, nblk);
            if (check_launch() != SA2_OK) return (int)SA2_ERR_LAUNCH_FAILED;
        }
        return (int)SA2_OK;
    });
}

}  // namespace sa2
