// Internal declarations shared by the translation units of libffi_hip.so (gfx950 only).
#ifndef FFI_INTERNAL_H
#define FFI_INTERNAL_H

#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstddef>

#include "ffi_hip.h"

namespace ffi {

// Shape bundle, validated on the host before any launch.
struct Dims {
    int B;   // batch
    int N;   // num_features
    int L;   // num_units (labels)
    int K;   // fan_in
    bool tp; // features / feature_grad are [N,B]
};

// Records a failing HIP call for ffi_last_hip_error() and maps it to FFI_ERR_HIP.
int hip_fail(hipError_t e);

#define FFI_HIP_TRY(expr)                                   \
    do {                                                    \
        hipError_t e__ = (expr);                            \
        if (e__ != hipSuccess) return ::ffi::hip_fail(e__); \
    } while (0)

#define FFI_TRY(expr)                 \
    do {                              \
        int s__ = (expr);             \
        if (s__ != FFI_OK) return s__; \
    } while (0)

// Library-owned device scratch, one buffer per (device, stream, slot), grown on demand and kept.
// Work that uses a buffer is ordered by the stream it belongs to.
enum WorkspaceSlot { kWsFeaturesT = 0, kWsPartials = 1, kWsSlots = 2 };
int workspace_get(hipStream_t s, int slot, size_t bytes, void** out);
void workspace_clear(int device);
size_t workspace_bytes(int device);
int device_cu_count();

// dst[c][r] = src[r][c] for a row-major [rows, cols] matrix.
int launch_transpose(const float* src, float* dst, int rows, int cols, hipStream_t s);

// ---- launchers (each validates nothing; callers pass validated Dims) ---------------------------
int launch_forward(const float* x, const int32_t* idx, const float* w, float* out, const Dims& d,
                   hipStream_t s);
int launch_weight_grad(const float* x, const int32_t* idx, const float* g, float* gw, const Dims& d,
                       hipStream_t s);

}  // namespace ffi

// Column-ordered ("CSC") view of one lookup matrix.
struct ffi_plan {
    int device = -1;
    int L = 0, K = 0, N = 0;
    const int32_t* lookup = nullptr;  // the buffer this plan was built from (cache key)
    unsigned long long fingerprint = 0;
    // perm[e]: flat position j*K+k of the e-th entry in (column, position) order;
    // col_ptr[n]..col_ptr[n+1]: the entries of column n.
    int32_t* perm = nullptr;
    int32_t* col_ptr = nullptr;
    unsigned long long* d_scratch = nullptr;  // fingerprint / flags (device)
    unsigned long long* h_scratch = nullptr;  // pinned mirror
    size_t bytes = 0;
};

namespace ffi {
int plan_build(ffi_plan* p, const int32_t* lookup, hipStream_t s);
int plan_fingerprint(ffi_plan* p, const int32_t* lookup, hipStream_t s, unsigned long long* out,
                     unsigned long long* bad_ids);
void plan_free(ffi_plan* p);
int launch_input_grad(const ffi_plan* p, const float* w, const float* g, float* gx, int B, bool tp,
                      hipStream_t s);
}  // namespace ffi

#endif  // FFI_INTERNAL_H
