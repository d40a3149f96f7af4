/*
 * sa2.h - C ABI of the MI355X (gfx950) 2-simplicial attention library.
 *
 * Plain C: pointers, sizes and scalars only; no torch types.  Every pointer
 * is a DEVICE pointer unless stated otherwise.  All entry points are
 * asynchronous on the HIP stream they are given, allocate nothing, never
 * synchronise, keep no state that depends on a call's arguments (each kernel's
 * LDS limit is raised once per process and device) and return 0 on success or
 * a negative sa2_status on error (nothing is launched on error).
 *
 * Tensors are [B, N, H, D] with per-tensor ELEMENT strides (batch, sequence,
 * head); the D stride must be 1.  LSE and workspace rows are [B, H, N] fp32,
 * contiguous.
 *
 * Maths (what the reference's operator computes):
 *   J(i) = [max(0,i-w1), i], K(i) = [max(0,i-w2), i]   simplicial/reference.py:41-45
 *   s[i,j,k] = scale * sum_d q[i,d] k1[j,d] (k2[k,d]+k2_bias)   reference.py:33,64
 *   O[i] = sum_{j,k} e^s (v1[j] * (v2[k]+v2_bias)) / (sum_{j,k} e^s + 1e-8)   reference.py:68-74
 *   LSE[i] = log(sum_{j,k} e^s + 1e-8)   (natural log; replaces simplicial/kernels.py:164)
 */
#ifndef SA2_H
#define SA2_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SA2_VERSION 1

typedef enum sa2_status {
    SA2_OK = 0,
    SA2_ERR_NULL_POINTER = -1,
    SA2_ERR_BAD_DTYPE = -2,
    SA2_ERR_BAD_SHAPE = -3,      /* B,N,H,D < 1 or D > 256 */
    SA2_ERR_BAD_STRIDE = -4,     /* a stride is not positive */
    SA2_ERR_BAD_WINDOW = -5,     /* w1 or w2 negative (or 0 with window_inclusive = 0) */
    SA2_ERR_WORKSPACE_TOO_SMALL = -6,
    SA2_ERR_LAUNCH_FAILED = -7,  /* hipGetLastError() after a launch */
    SA2_ERR_UNSUPPORTED = -8,    /* a forced kernel path does not support the shape/dtype */
    SA2_ERR_TOO_LARGE = -9,      /* an index would overflow the kernels' 32-bit grid */
    SA2_ERR_STATIC_WORKSPACE = -10 /* sa2_backward_static_workspace: the problem needs more than
                                      SA2_STATIC_WORKSPACE_BYTES, or the array's address is unavailable */
} sa2_status;

typedef enum sa2_dtype { SA2_F32 = 0, SA2_BF16 = 1, SA2_F16 = 2 } sa2_dtype;

/* flags */
#define SA2_FLAG_AUTO 0u            /* matrix-pipe (MFMA) kernels when the shape allows, fp32-FMA kernels otherwise */
#define SA2_FLAG_FORCE_GENERIC 1u   /* fp32-FMA kernels (any dtype, any D <= 256) */
#define SA2_FLAG_FORCE_MFMA 2u      /* MFMA kernels (bf16 or fp16 with D 32, 64, 128 or 256; fp32 with D 32, 64 or 128;
                                       16-byte aligned rows) or SA2_ERR_UNSUPPORTED; also takes the pre-pass kernels
                                       of the 16-bit D 32/64/128 path whenever the window sizes allow, whatever the
                                       problem size (SA2_FLAG_AUTO leaves them out for small grids) */

/* Tensor order of the `strides` argument (3 int64 per tensor: batch, sequence, head). */
enum { SA2_T_Q = 0, SA2_T_K1, SA2_T_K2, SA2_T_V1, SA2_T_V2, SA2_T_OUT, SA2_FWD_TENSORS,
       SA2_T_DOUT = SA2_FWD_TENSORS, SA2_T_DQ, SA2_T_DK1, SA2_T_DK2, SA2_T_DV1, SA2_T_DV2,
       SA2_BWD_TENSORS };

/* Library version (SA2_VERSION the library was built with). */
int sa2_version(void);

/* Static, NUL-terminated description of a status code. */
const char* sa2_strerror(int status);

/* 1 if sa2_forward would take MFMA kernels for this problem under SA2_FLAG_AUTO
 * (given 16-byte aligned rows), 0 if it would take the fp32-FMA kernels.  sa2_backward makes the
 * same choice: its MFMA kernels take any K' window (one wider than their on-chip accumulators hold
 * is walked in segments of deltas). */
int sa2_uses_mfma(int B, int N, int H, int D, int w1, int w2, int dtype);

/*
 * Forward.  Replaces the launch in TwoSimplicialAttentionFunction.forward
 * (simplicial/triton_impl.py:19-58) and the kernel it launches
 * (simplicial/kernels.py:11-171).
 *   q,k1,k2,v1,v2  inputs, element type `dtype`
 *   out            output, element type `dtype`        (triton_impl.py:23)
 *   lse            [B,H,N] fp32, natural-log LSE        (triton_impl.py:24)
 *   strides        SA2_FWD_TENSORS x 3 element strides  (HOST pointer)
 *   window_inclusive  1: windows [i-w, i] (reference.py); 0: (i-w, i] (kernels.py:133-136)
 * While the call runs, `out` and `lse` also hold intermediate results of its first kernel: their
 * contents are final only once the call's work on the stream has completed.
 */
int sa2_forward(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                void* out, float* lse,
                int B, int N, int H, int D,
                const int64_t* strides,
                int w1, int w2, float scale, float k2_bias, float v2_bias,
                int dtype, int window_inclusive, unsigned flags, void* hip_stream);

/* Bytes of device workspace sa2_backward needs for this problem (0 is never
 * returned for a valid problem; returns 0 for an invalid one). */
size_t sa2_bwd_workspace_bytes(int B, int N, int H, int D, int w1, int w2, int dtype, unsigned flags);

/*
 * Backward.  Replaces TwoSimplicialAttentionFunction.backward
 * (simplicial/triton_impl.py:61-158): the row term D = sum_d dO*O
 * (simplicial/kernels.py:569-571), the K-side kernel (kernels.py:175-382) and
 * the K'-side kernel (kernels.py:386-566).
 *   out, dout, lse   forward output, upstream gradient, forward LSE
 *   dq,dk1,dk2,dv1,dv2  gradients in `dtype`; a NULL pointer means "not needed"
 *                       (ctx.needs_input_grad, triton_impl.py:73-77); every
 *                       non-NULL gradient is fully overwritten (no pre-zeroing needed; dk2 and
 *                       dv2 also hold intermediate results while the call runs)
 *   workspace        >= sa2_bwd_workspace_bytes(...) bytes, 256-byte aligned; contents
 *                    on entry are ignored
 *   strides          SA2_BWD_TENSORS x 3 element strides (HOST pointer)
 * Deterministic: no atomics; two calls on the same inputs give identical bits.
 */
int sa2_backward(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                 const void* out, const void* dout, const float* lse,
                 void* dq, void* dk1, void* dk2, void* dv1, void* dv2,
                 void* workspace, size_t workspace_bytes,
                 int B, int N, int H, int D,
                 const int64_t* strides,
                 int w1, int w2, float scale, float k2_bias, float v2_bias,
                 int dtype, int window_inclusive, unsigned flags, void* hip_stream);

/*
 * sa2_backward for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart
 * in the reference.  Same arguments, kernels and results as sa2_backward, minus the
 * workspace: that is a file-scope device array of SA2_STATIC_WORKSPACE_BYTES inside the
 * library, one copy per GPU, held until the process ends.  The call itself allocates and
 * frees nothing.  A problem with sa2_bwd_workspace_bytes(...) > SA2_STATIC_WORKSPACE_BYTES
 * returns SA2_ERR_STATIC_WORKSPACE and launches nothing.  All calls on one GPU share the
 * array (the kernels overwrite what they read from it, so nothing needs clearing between
 * calls): calls that overlap on one GPU - different streams, or host threads - race;
 * calls on one stream are safe.
 */
#define SA2_STATIC_WORKSPACE_BYTES (64u << 20)
int sa2_backward_static_workspace(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                                  const void* out, const void* dout, const float* lse,
                                  void* dq, void* dk1, void* dk2, void* dv1, void* dv2,
                                  int B, int N, int H, int D,
                                  const int64_t* strides,
                                  int w1, int w2, float scale, float k2_bias, float v2_bias,
                                  int dtype, int window_inclusive, unsigned flags, void* hip_stream);

/*
 * Row term of the softmax Jacobian, dsum[b,h,i] = sum_d dout[b,i,h,d]*out[b,i,h,d]
 * in fp32.  Replaces compute_D_kernel (simplicial/kernels.py:569-571), with the
 * [B,H,N] fp32 layout the backward kernels index.
 *   strides   2 x 3 element strides: out, dout (HOST pointer)
 */
int sa2_rowdot(const void* out, const void* dout, float* dsum,
               int B, int N, int H, int D, const int64_t* strides, int dtype, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* SA2_H */
