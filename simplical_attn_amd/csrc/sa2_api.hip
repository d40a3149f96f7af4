// extern "C" boundary: argument validation and kernel-path selection.
// No allocation and no synchronisation.  The only process state is set-up that happens once and
// never depends on a call's arguments: each kernel's LDS limit (allow_full_lds) and, for
// sa2_backward_static_workspace, the per-device address of the library's own workspace array.
#include <string.h>

#include <mutex>
#include <utility>
#include <vector>

#include "sa2_common.h"

using namespace sa2;

namespace sa2 {

bool allow_full_lds(const void* kernel) {
    static std::mutex mu;
    static std::vector<std::pair<const void*, int>> done;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return false;
    std::lock_guard<std::mutex> lock(mu);
    for (const auto& e : done)
        if (e.first == kernel && e.second == dev) return true;
    // the limit covers dynamic LDS only: what the kernel declares statically comes off the 160 KB
    hipFuncAttributes attr;
    if (hipFuncGetAttributes(&attr, kernel) != hipSuccess) return false;
    const int room = LDS_BYTES_PER_CU - (int)attr.sharedSizeBytes;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, room) != hipSuccess) return false;
    done.emplace_back(kernel, dev);
    return true;
}

}  // namespace sa2

// Workspace of sa2_backward_static_workspace: one copy per GPU the library runs on, held until
// the process ends.  In host code this name is only a handle for hipGetSymbolAddress; the
// device address it yields (per device) is what the kernels are given.
static __device__ __align__(256) unsigned char scratch[SA2_STATIC_WORKSPACE_BYTES];

namespace {

bool valid_dtype(int dtype) { return dtype == SA2_F32 || dtype == SA2_BF16 || dtype == SA2_F16; }

int check_dims(int B, int N, int H, int D, int w1, int w2, int dtype, int window_inclusive) {
    if (!valid_dtype(dtype)) return SA2_ERR_BAD_DTYPE;
    if (B < 1 || N < 1 || H < 1 || D < 1 || D > 256) return SA2_ERR_BAD_SHAPE;
    const int wmin = window_inclusive ? 0 : 1;
    if (w1 < wmin || w2 < wmin) return SA2_ERR_BAD_WINDOW;
    if ((int64_t)B * H * N > 0x7fffffffLL) return SA2_ERR_TOO_LARGE;
    return SA2_OK;
}

// Inclusive reach of a window: [i-reach, i]; never more than N-1.
int reach(int w, int window_inclusive, int N) {
    const int r = window_inclusive ? w : w - 1;
    return r < N - 1 ? r : N - 1;
}

Tensor make_tensor(const void* p, const int64_t* strides, int which) {
    Tensor t;
    t.p = const_cast<void*>(p);
    t.sb = strides[3 * which + 0];
    t.sn = strides[3 * which + 1];
    t.sh = strides[3 * which + 2];
    return t;
}

bool strides_ok(const int64_t* strides, int count, int B, int N, int H) {
    for (int t = 0; t < count; ++t) {
        // a size-1 axis may carry any stride; otherwise strides must be positive
        if ((B > 1 && strides[3 * t] <= 0) || (N > 1 && strides[3 * t + 1] <= 0) || (H > 1 && strides[3 * t + 2] <= 0))
            return false;
    }
    return true;
}

size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Device address of `scratch` on the current device, looked up on the first call on that
// device (with that device current) and kept; NULL if the lookup fails.
void* static_workspace() {
    constexpr int MAX_DEVICES = 64;
    static std::mutex mu;
    static void* address[MAX_DEVICES] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> lock(mu);
    if (!address[dev]) {
        void* ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
        address[dev] = ptr;
    }
    return address[dev];
}

size_t dsum_bytes(int B, int N, int H) { return align_up((size_t)B * H * N * sizeof(float), 256); }

// Which kernels a call takes: the fp32 FMA kernels, the tuned 16-bit MFMA kernels (head_dim 32, 64, 128), the
// 16-bit MFMA kernels for head_dim 256, or the fp32 MFMA kernels.
enum KernelPath { PATH_GENERIC, PATH_MFMA16, PATH_WIDE16, PATH_MFMA32 };

KernelPath pick_path(const Problem& p, int dtype, unsigned flags, bool backward, int* status) {
    *status = SA2_OK;
    if (flags & SA2_FLAG_FORCE_GENERIC) return PATH_GENERIC;
    KernelPath path = PATH_GENERIC;
    if (dtype == SA2_F32) {
        const bool ok = (backward ? f32_mfma_bwd_supported(p.D, p.w2, dtype) : f32_mfma_supported(p.D, dtype)) &&
                        f32_mfma_layout_ok(p, backward);
        if (ok) path = PATH_MFMA32;
    } else {
        const bool ok = (backward ? mfma_bwd_supported(p.B, p.N, p.H, p.D, p.w1, p.w2, dtype)
                                  : mfma_supported(p.B, p.N, p.H, p.D, p.w1, p.w2, dtype)) &&
                        mfma_layout_ok(p, backward);
        if (ok) path = PATH_MFMA16;
        else if ((backward ? wide_bwd_supported(p.D, p.w2, dtype) : wide_supported(p.D, dtype)) && mfma_layout_ok(p, backward))
            path = PATH_WIDE16;
    }
    if (path == PATH_GENERIC && (flags & SA2_FLAG_FORCE_MFMA)) *status = SA2_ERR_UNSUPPORTED;
    return path;
}

}  // namespace

extern "C" {

int sa2_version(void) { return SA2_VERSION; }

const char* sa2_strerror(int status) {
    switch (status) {
        case SA2_OK: return "success";
        case SA2_ERR_NULL_POINTER: return "a required pointer is NULL";
        case SA2_ERR_BAD_DTYPE: return "unknown dtype (0 = fp32, 1 = bf16, 2 = fp16)";
        case SA2_ERR_BAD_SHAPE: return "bad shape: B, N, H, D must be >= 1 and D <= 256";
        case SA2_ERR_BAD_STRIDE: return "bad stride: batch/sequence/head strides must be positive (D stride is 1)";
        case SA2_ERR_BAD_WINDOW: return "bad window: w1 and w2 must be >= 0 (>= 1 for the half-open convention)";
        case SA2_ERR_WORKSPACE_TOO_SMALL: return "workspace is smaller than sa2_bwd_workspace_bytes() or not 256-byte aligned";
        case SA2_ERR_LAUNCH_FAILED: return "a HIP kernel launch failed";
        case SA2_ERR_UNSUPPORTED: return "the forced kernel path does not support this shape, dtype or layout";
        case SA2_ERR_TOO_LARGE: return "problem too large for the kernels' 32-bit grid (B*H*N must be < 2^31)";
        case SA2_ERR_STATIC_WORKSPACE: return "the problem needs more workspace than the library's own SA2_STATIC_WORKSPACE_BYTES, or "
                                              "the address of that array could not be obtained on this device";
    }
    return "unknown sa2 status";
}

int sa2_uses_mfma(int B, int N, int H, int D, int w1, int w2, int dtype) {
    if (check_dims(B, N, H, D, w1, w2, dtype, 1) != SA2_OK) return 0;
    return (mfma_supported(B, N, H, D, reach(w1, 1, N), reach(w2, 1, N), dtype) || wide_supported(D, dtype) ||
            f32_mfma_supported(D, dtype)) ? 1 : 0;
}

int sa2_forward(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                void* out, float* lse, int B, int N, int H, int D, const int64_t* strides,
                int w1, int w2, float scale, float k2_bias, float v2_bias,
                int dtype, int window_inclusive, unsigned flags, void* hip_stream) {
    if (!q || !k1 || !k2 || !v1 || !v2 || !out || !lse || !strides) return SA2_ERR_NULL_POINTER;
    int rc = check_dims(B, N, H, D, w1, w2, dtype, window_inclusive);
    if (rc != SA2_OK) return rc;
    if (!strides_ok(strides, SA2_FWD_TENSORS, B, N, H)) return SA2_ERR_BAD_STRIDE;

    Problem p;
    memset(&p, 0, sizeof(p));
    p.B = B; p.N = N; p.H = H; p.D = D;
    p.w1 = reach(w1, window_inclusive, N);
    p.w2 = reach(w2, window_inclusive, N);
    p.scale = scale; p.k2_bias = k2_bias; p.v2_bias = v2_bias;
    p.q = make_tensor(q, strides, SA2_T_Q);
    p.k1 = make_tensor(k1, strides, SA2_T_K1);
    p.k2 = make_tensor(k2, strides, SA2_T_K2);
    p.v1 = make_tensor(v1, strides, SA2_T_V1);
    p.v2 = make_tensor(v2, strides, SA2_T_V2);
    p.out = make_tensor(out, strides, SA2_T_OUT);
    p.lse = lse;

    p.force_prepass = (flags & SA2_FLAG_FORCE_MFMA) ? 1 : 0;

    hipStream_t st = (hipStream_t)hip_stream;
    const KernelPath path = pick_path(p, dtype, flags, false, &rc);
    if (rc != SA2_OK) return rc;
    return path == PATH_MFMA16 ? launch_mfma_fwd(p, dtype, st)
           : path == PATH_WIDE16 ? launch_wide_fwd(p, dtype, st)
           : path == PATH_MFMA32 ? launch_f32_mfma_fwd(p, st) : launch_generic_fwd(p, dtype, st);
}

size_t sa2_bwd_workspace_bytes(int B, int N, int H, int D, int w1, int w2, int dtype, unsigned flags) {
    if (check_dims(B, N, H, D, w1, w2, dtype, 1) != SA2_OK) return 0;
    size_t scratch = generic_bwd_scratch_bytes(B, N, H, D, w1, w2);
    if (!(flags & SA2_FLAG_FORCE_GENERIC) && mfma_bwd_supported(B, N, H, D, reach(w1, 1, N), reach(w2, 1, N), dtype)) {
        const size_t m = mfma_bwd_scratch_bytes(B, N, H, D, reach(w1, 1, N), reach(w2, 1, N));
        if (m > scratch) scratch = m;
    }
    if (!(flags & SA2_FLAG_FORCE_GENERIC) && wide_bwd_supported(D, reach(w2, 1, N), dtype)) {
        const size_t m = wide_bwd_scratch_bytes(B, N, H, D, reach(w1, 1, N), reach(w2, 1, N));
        if (m > scratch) scratch = m;
    }
    if (!(flags & SA2_FLAG_FORCE_GENERIC) && f32_mfma_bwd_supported(D, reach(w2, 1, N), dtype)) {
        const size_t m = f32_mfma_bwd_scratch_bytes(B, N, H, D, reach(w1, 1, N), reach(w2, 1, N));
        if (m > scratch) scratch = m;
    }
    return dsum_bytes(B, N, H) + align_up(scratch, 256) + 256;
}

int sa2_backward(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                 const void* out, const void* dout, const float* lse,
                 void* dq, void* dk1, void* dk2, void* dv1, void* dv2,
                 void* workspace, size_t workspace_bytes,
                 int B, int N, int H, int D, const int64_t* strides,
                 int w1, int w2, float scale, float k2_bias, float v2_bias,
                 int dtype, int window_inclusive, unsigned flags, void* hip_stream) {
    if (!q || !k1 || !k2 || !v1 || !v2 || !out || !dout || !lse || !strides || !workspace) return SA2_ERR_NULL_POINTER;
    int rc = check_dims(B, N, H, D, w1, w2, dtype, window_inclusive);
    if (rc != SA2_OK) return rc;
    if (!strides_ok(strides, SA2_BWD_TENSORS, B, N, H)) return SA2_ERR_BAD_STRIDE;
    // The half-open convention with window w has the reach of the closed one with w-1.
    const size_t need = sa2_bwd_workspace_bytes(B, N, H, D, window_inclusive ? w1 : w1 - 1,
                                                window_inclusive ? w2 : w2 - 1, dtype, flags);
    if (workspace_bytes < need || ((uintptr_t)workspace & 255u)) return SA2_ERR_WORKSPACE_TOO_SMALL;
    if (!dq && !dk1 && !dk2 && !dv1 && !dv2) return SA2_OK;

    Problem p;
    memset(&p, 0, sizeof(p));
    p.B = B; p.N = N; p.H = H; p.D = D;
    p.w1 = reach(w1, window_inclusive, N);
    p.w2 = reach(w2, window_inclusive, N);
    p.scale = scale; p.k2_bias = k2_bias; p.v2_bias = v2_bias;
    p.q = make_tensor(q, strides, SA2_T_Q);
    p.k1 = make_tensor(k1, strides, SA2_T_K1);
    p.k2 = make_tensor(k2, strides, SA2_T_K2);
    p.v1 = make_tensor(v1, strides, SA2_T_V1);
    p.v2 = make_tensor(v2, strides, SA2_T_V2);
    p.out = make_tensor(out, strides, SA2_T_OUT);
    p.dout = make_tensor(dout, strides, SA2_T_DOUT);
    p.dq = make_tensor(dq, strides, SA2_T_DQ);
    p.dk1 = make_tensor(dk1, strides, SA2_T_DK1);
    p.dk2 = make_tensor(dk2, strides, SA2_T_DK2);
    p.dv1 = make_tensor(dv1, strides, SA2_T_DV1);
    p.dv2 = make_tensor(dv2, strides, SA2_T_DV2);
    p.lse = const_cast<float*>(lse);
    p.dsum = (float*)workspace;
    p.scratch = (char*)workspace + dsum_bytes(B, N, H);
    p.scratch_bytes = workspace_bytes - dsum_bytes(B, N, H);

    p.force_prepass = (flags & SA2_FLAG_FORCE_MFMA) ? 1 : 0;

    hipStream_t st = (hipStream_t)hip_stream;
    const KernelPath path = pick_path(p, dtype, flags, true, &rc);
    if (rc != SA2_OK) return rc;
    return path == PATH_MFMA16 ? launch_mfma_bwd(p, dtype, st)
           : path == PATH_WIDE16 ? launch_wide_bwd(p, dtype, st)
           : path == PATH_MFMA32 ? launch_f32_mfma_bwd(p, st) : launch_generic_bwd(p, dtype, st);
}

int sa2_backward_static_workspace(const void* q, const void* k1, const void* k2, const void* v1, const void* v2,
                                  const void* out, const void* dout, const float* lse,
                                  void* dq, void* dk1, void* dk2, void* dv1, void* dv2,
                                  int B, int N, int H, int D, const int64_t* strides,
                                  int w1, int w2, float scale, float k2_bias, float v2_bias,
                                  int dtype, int window_inclusive, unsigned flags, void* hip_stream) {
    int rc = check_dims(B, N, H, D, w1, w2, dtype, window_inclusive);
    if (rc != SA2_OK) return rc;
    const size_t need = sa2_bwd_workspace_bytes(B, N, H, D, window_inclusive ? w1 : w1 - 1,
                                                window_inclusive ? w2 : w2 - 1, dtype, flags);
    if (need == 0 || need > (size_t)SA2_STATIC_WORKSPACE_BYTES) return SA2_ERR_STATIC_WORKSPACE;
    void* ws = static_workspace();
    if (!ws) return SA2_ERR_STATIC_WORKSPACE;
    return sa2_backward(q, k1, k2, v1, v2, out, dout, lse, dq, dk1, dk2, dv1, dv2, ws, SA2_STATIC_WORKSPACE_BYTES,
                        B, N, H, D, strides, w1, w2, scale, k2_bias, v2_bias, dtype, window_inclusive, flags, hip_stream);
}

int sa2_rowdot(const void* out, const void* dout, float* dsum, int B, int N, int H, int D,
               const int64_t* strides, int dtype, void* hip_stream) {
    if (!out || !dout || !dsum || !strides) return SA2_ERR_NULL_POINTER;
    int rc = check_dims(B, N, H, D, 0, 0, dtype, 1);
    if (rc != SA2_OK) return rc;
    if (!strides_ok(strides, 2, B, N, H)) return SA2_ERR_BAD_STRIDE;
    return launch_rowdot(make_tensor(out, strides, 0), make_tensor(dout, strides, 1), dsum, B, N, H, D, dtype,
                         (hipStream_t)hip_stream);
}

}  // extern "C"
