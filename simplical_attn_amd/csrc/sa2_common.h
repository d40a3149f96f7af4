// Shared declarations of the gfx950 2-simplicial attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sa2.h"

namespace sa2 {

// One [B,N,H,D] tensor: base pointer and element strides (D stride is 1).
struct Tensor {
    void* p;
    int64_t sb, sn, sh;
    __host__ __device__ int64_t off(int b, int n, int h) const { return b * sb + n * sn + h * sh; }
};

// Everything a kernel needs about one call.  w1/w2 are already the inclusive
// window reaches: query i sees keys [i-w, i].
struct Problem {
    int B, N, H, D;
    int w1, w2;
    float scale, k2_bias, v2_bias;
    Tensor q, k1, k2, v1, v2, out, dout;
    Tensor dq, dk1, dk2, dv1, dv2;   // p == nullptr: not requested
    float* lse;                      // [B,H,N]
    float* dsum;                     // [B,H,N]  sum_d dout*out
    void* scratch;                   // remaining workspace (path specific)
    size_t scratch_bytes;
    int force_prepass;               // take the pre-pass kernels whenever the window allows, whatever the size
};

// ---- element loads / stores -------------------------------------------------
struct bf16_t { uint16_t bits; };
struct f16_t { _Float16 v; };

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return __uint_as_float(((uint32_t)x.bits) << 16); }
__device__ __forceinline__ float to_float(f16_t x) { return (float)x.v; }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);   // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1u);                                             // round to nearest even
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ void from_float(float f, float* p) { *p = f; }
__device__ __forceinline__ void from_float(float f, bf16_t* p) { p->bits = f32_to_bf16_bits(f); }
__device__ __forceinline__ void from_float(float f, f16_t* p) { p->v = (_Float16)f; }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// log(sum_w + 1e-8) from the running maximum m and l = sum exp(s-m), for any m.
__device__ __forceinline__ float lse_with_eps(float m, float l) {
    const float log_eps = -18.420680743952367f;   // log(1e-8)
    if (m > log_eps) return m + logf(l + 1e-8f * expf(-m));
    return log_eps + log1pf(l * expf(m - log_eps));
}

// Lifts a kernel's limit on dynamic LDS to the CU's full 160 KB.  The value never depends on the
// call, and it is set once per (kernel, device) for the life of the process, so concurrent
// launches of one kernel with different LDS sizes cannot disturb each other.
constexpr int LDS_BYTES_PER_CU = 160 * 1024;
bool allow_full_lds(const void* kernel);

// ---- launchers (each returns a sa2_status) ----------------------------------
int launch_rowdot(const Tensor& out, const Tensor& dout, float* dsum, int B, int N, int H, int D,
                  int dtype, hipStream_t st);
int launch_generic_fwd(const Problem& p, int dtype, hipStream_t st);
int launch_generic_bwd(const Problem& p, int dtype, hipStream_t st);
size_t generic_bwd_scratch_bytes(int B, int N, int H, int D, int w1, int w2);

bool mfma_supported(int B, int N, int H, int D, int w1, int w2, int dtype);
bool mfma_bwd_supported(int B, int N, int H, int D, int w1, int w2, int dtype);
bool mfma_layout_ok(const Problem& p, bool backward);
int launch_mfma_fwd(const Problem& p, int dtype, hipStream_t st);
int launch_mfma_bwd(const Problem& p, int dtype, hipStream_t st);
size_t mfma_bwd_scratch_bytes(int B, int N, int H, int D, int w1, int w2);
// fp32 tensors on the fp32 MFMA (head_dim 32, 64, 128; rows 16-byte aligned)
bool f32_mfma_supported(int D, int dtype);
bool f32_mfma_bwd_supported(int D, int w2, int dtype);
bool f32_mfma_layout_ok(const Problem& p, bool backward);
size_t f32_mfma_bwd_scratch_bytes(int B, int N, int H, int D, int w1, int w2);
int launch_f32_mfma_fwd(const Problem& p, hipStream_t st);
int launch_f32_mfma_bwd(const Problem& p, hipStream_t st);
// 16-bit tensors with head_dim 256 on the 16-bit MFMA (rows 16-byte aligned)
bool wide_supported(int D, int dtype);
bool wide_bwd_supported(int D, int w2, int dtype);
size_t wide_bwd_scratch_bytes(int B, int N, int H, int D, int w1, int w2);
int launch_wide_fwd(const Problem& p, int dtype, hipStream_t st);
int launch_wide_bwd(const Problem& p, int dtype, hipStream_t st);
// K'-side backward kernel (dQ, dK', dV') that keeps its partial sums on chip (K' windows too wide for
// that are cut into segments of deltas, one workgroup each)
size_t kp_scratch_bytes(int B, int N, int H, int D, int w2);
int launch_mfma_bwd_kp(const Problem& p, int dtype, hipStream_t st);
// K-side backward kernel (dK, dV) with paired wavefronts; for small grids it splits a key block's
// query blocks over several workgroups, whose fp32 partial sums lie in the workspace behind the
// K'-side part (kp_side_scratch_bytes); K' windows too wide for its LDS rows are walked in segments
size_t kv_split_scratch_bytes(int B, int N, int H, int D, int w1, int w2);
size_t kp_side_scratch_bytes(int B, int N, int H, int D, int w2);
int launch_mfma_bwd_kv(const Problem& p, int dtype, hipStream_t st);

}  // namespace sa2
