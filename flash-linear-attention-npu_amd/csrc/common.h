// Host-side helpers shared by every operator translation unit: status / error
// string, tensor-descriptor checks, variable-length metadata, pinned staging.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <exception>
#include <new>
#include <vector>

#include "../../include/fla_hip.h"

namespace fla {

// ---- error reporting -------------------------------------------------------
char *last_error_buffer();  // thread-local, 512 bytes
int fail(int status, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define FLA_REQUIRE(cond, status, ...)               \
    do {                                             \
        if (!(cond)) return ::fla::fail((status), __VA_ARGS__); \
    } while (0)

#define FLA_HIP_CHECK(expr)                                                           \
    do {                                                                              \
        hipError_t err__ = (expr);                                                    \
        if (err__ != hipSuccess)                                                      \
            return ::fla::fail(FLA_ERR_LAUNCH, "%s failed: %s", #expr, hipGetErrorString(err__)); \
    } while (0)

// Every extern "C" entry point runs its body through this: host-side bookkeeping uses std::vector and a mutex, and
// nothing they throw may cross the C boundary.
template <typename F> inline int guarded(F &&body) noexcept {
    try {
        return body();
    } catch (const std::bad_alloc &) {
        return fail(FLA_ERR_HOST, "host memory allocation failed inside the call.");
    } catch (const std::exception &e) {
        return fail(FLA_ERR_HOST, "host-side failure inside the call: %s", e.what());
    } catch (...) {
        return fail(FLA_ERR_HOST, "unknown host-side failure inside the call.");
    }
}

// ---- tensor descriptor helpers --------------------------------------------
inline size_t dtype_size(int dt) {
    switch (dt) {
        case FLA_F32: case FLA_I32: return 4;
        case FLA_F16: case FLA_BF16: return 2;
        case FLA_I64: return 8;
        default: return 0;
    }
}

inline bool is_contiguous(const fla_tensor *t) {
    int64_t expect = 1;
    for (int i = t->ndim - 1; i >= 0; --i) {
        if (t->shape[i] != 1 && t->stride[i] != expect) return false;
        expect *= t->shape[i];
    }
    return true;
}

inline int64_t numel(const fla_tensor *t) {
    int64_t n = 1;
    for (int i = 0; i < t->ndim; ++i) n *= t->shape[i];
    return n;
}

// Required tensor: non-null descriptor and data, given rank and dtype.
int check_tensor(const fla_tensor *t, const char *op, const char *name, int ndim, int dtype_mask);
inline int dt_bit(int dt) { return 1 << dt; }
bool same_shape(const fla_tensor *a, const fla_tensor *b);
// Innermost stride must be 1 (or extent 1).
inline bool inner_unit(const fla_tensor *t) {
    return t->ndim == 0 || t->shape[t->ndim - 1] == 1 || t->stride[t->ndim - 1] == 1;
}

// ---- variable-length metadata ---------------------------------------------
// Host view of cu_seqlens and the canonical (sequence, chunk) table derived from
// it.  Device copy layout (int32): cu[N+1] | chunk_offset[N+1] | table[2*NT].
struct Varlen {
    bool enabled = false;
    int N = 0;         // sequences
    int NT = 0;        // total chunks over all sequences
    int64_t total = 0; // cu[N]
    std::vector<int32_t> host;  // packed as above
    const int32_t *d_cu = nullptr;
    const int32_t *d_choff = nullptr;
    const int32_t *d_tab = nullptr;
    size_t bytes() const { return enabled ? ((host.size() * 4 + 255) / 256) * 256 : 0; }
};

// Builds the host table; validates cu_seqlens (non-decreasing, starts at 0,
// ends at total_t) and, when given, that chunk_indices is the canonical list.
int build_varlen(Varlen &vl, const char *op, const fla_int_array *cu_seqlens,
                 const fla_int_array *chunk_indices, int64_t chunk, int64_t total_t);
// Copies the table into `workspace` on `stream` through a pinned staging ring
// and fills the device pointers.
int upload_varlen(Varlen &vl, void *workspace, hipStream_t stream);

// Asynchronous host->device copy of a small host buffer that may be freed by
// the caller immediately after return.
int stage_to_device(void *dst, const void *src, size_t bytes, hipStream_t stream);

int num_cus();

// ---- optional per-kernel timing (off by default) ---------------------------
// When enabled through fla_profile_enable(1), every kernel launch site brackets
// its launch with two HIP events on the launch stream; fla_profile_report()
// synchronises them and returns "name count total_ms" lines.
bool profile_enabled();
bool profile_begin(const char *name, hipStream_t stream);   // false: nothing was recorded
void profile_end(hipStream_t stream);
struct ProfileScope {
    hipStream_t s;
    bool on;
    ProfileScope(const char *name, hipStream_t stream) : s(stream), on(profile_enabled()) {
        if (on) on = profile_begin(name, s);
    }
    ~ProfileScope() {
        if (on) profile_end(s);
    }
};

}  // namespace fla

#define FLA_LAUNCH(name, stream_, ...)                     \
    do {                                                   \
        ::fla::ProfileScope prof__(name, stream_);         \
        hipLaunchKernelGGL(__VA_ARGS__);                   \
    } while (0)

// Workspace-query / launch pair generator: each operator is written once as
//   static int impl(<operands>, void* ws, uint64_t ws_size, hipStream_t s, uint64_t* query)
// and, when `query` is non-null, reports its workspace size without launching.
