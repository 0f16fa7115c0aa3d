// Host-side helpers: error string, descriptor checks, varlen metadata, pinned
// staging ring for small host->device copies.
#include "common.h"

#include <mutex>

namespace fla {

char *last_error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}

int fail(int status, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(last_error_buffer(), 512, fmt, ap);
    va_end(ap);
    if (const char *env = getenv("FLA_HIP_LOG")) {
        if (env[0] && env[0] != '0') fprintf(stderr, "[fla_hip] error %d: %s\n", status, last_error_buffer());
    }
    return status;
}

int check_tensor(const fla_tensor *t, const char *op, const char *name, int ndim, int dtype_mask) {
    if (t == nullptr || t->data == nullptr) return fail(FLA_ERR_NULL, "%s: %s must not be null.", op, name);
    if (ndim >= 0 && t->ndim != ndim)
        return fail(FLA_ERR_SHAPE, "%s: %s must be rank %d, got rank %d.", op, name, ndim, t->ndim);
    if (t->ndim < 0 || t->ndim > FLA_MAX_DIMS) return fail(FLA_ERR_SHAPE, "%s: %s has invalid rank.", op, name);
    if (t->dtype < 0 || t->dtype > FLA_I64 || !(dtype_mask & dt_bit(t->dtype)))
        return fail(FLA_ERR_DTYPE, "%s: %s has unsupported dtype %d.", op, name, t->dtype);
    for (int i = 0; i < t->ndim; ++i)
        if (t->shape[i] < 0) return fail(FLA_ERR_SHAPE, "%s: %s has a negative extent.", op, name);
    return FLA_OK;
}

bool same_shape(const fla_tensor *a, const fla_tensor *b) {
    if (a->ndim != b->ndim) return false;
    for (int i = 0; i < a->ndim; ++i)
        if (a->shape[i] != b->shape[i]) return false;
    return true;
}

int build_varlen(Varlen &vl, const char *op, const fla_int_array *cu, const fla_int_array *ci,
                 int64_t chunk, int64_t total_t) {
    vl = Varlen();
    if (cu == nullptr || cu->data == nullptr || cu->size == 0) {
        if (ci != nullptr && ci->data != nullptr && ci->size != 0)
            return fail(FLA_ERR_METADATA, "%s: chunk_indices given without cu_seqlens.", op);
        return FLA_OK;
    }
    if (cu->size < 2) return fail(FLA_ERR_METADATA, "%s: cu_seqlens needs at least two entries.", op);
    if (chunk <= 0) return fail(FLA_ERR_SHAPE, "%s: chunk_size must be positive.", op);
    const int N = (int)cu->size - 1;
    if (cu->data[0] != 0) return fail(FLA_ERR_METADATA, "%s: cu_seqlens must start at 0.", op);
    if (cu->data[N] != total_t)
        return fail(FLA_ERR_METADATA, "%s: cu_seqlens must end at the token count %lld, got %lld.", op,
                    (long long)total_t, (long long)cu->data[N]);
    if (total_t >= (int64_t)1 << 31) return fail(FLA_ERR_SHAPE, "%s: token count exceeds int32.", op);
    std::vector<int32_t> tab;
    std::vector<int32_t> choff(N + 1, 0);
    for (int n = 0; n < N; ++n) {
        const int64_t len = cu->data[n + 1] - cu->data[n];
        if (len < 0) return fail(FLA_ERR_METADATA, "%s: cu_seqlens must be non-decreasing.", op);
        const int nc = (int)((len + chunk - 1) / chunk);
        for (int c = 0; c < nc; ++c) {
            tab.push_back(n);
            tab.push_back(c);
        }
        choff[n + 1] = choff[n] + nc;
    }
    if (ci != nullptr && ci->data != nullptr && ci->size != 0) {
        bool ok = ci->size == tab.size();
        for (size_t i = 0; ok && i < tab.size(); ++i) ok = ci->data[i] == tab[i];
        if (!ok)
            return fail(FLA_ERR_METADATA,
                        "%s: chunk_indices must be the canonical sequence-major list derived from cu_seqlens.", op);
    }
    vl.enabled = true;
    vl.N = N;
    vl.NT = choff[N];
    vl.total = total_t;
    vl.host.resize((size_t)(N + 1) * 2 + tab.size());
    for (int n = 0; n <= N; ++n) {
        vl.host[n] = (int32_t)cu->data[n];
        vl.host[N + 1 + n] = choff[n];
    }
    if (!tab.empty()) memcpy(vl.host.data() + 2 * (N + 1), tab.data(), tab.size() * 4);
    return FLA_OK;
}

int upload_varlen(Varlen &vl, void *workspace, hipStream_t stream) {
    if (!vl.enabled) return FLA_OK;
    if (workspace == nullptr) return fail(FLA_ERR_WORKSPACE, "workspace required for cu_seqlens metadata.");
    int rc = stage_to_device(workspace, vl.host.data(), vl.host.size() * 4, stream);
    if (rc != FLA_OK) return rc;
    const int32_t *base = static_cast<const int32_t *>(workspace);
    vl.d_cu = base;
    vl.d_choff = base + (vl.N + 1);
    vl.d_tab = base + 2 * (vl.N + 1);
    return FLA_OK;
}

// ---- pinned staging ring ---------------------------------------------------
// hipMemcpyAsync from pageable memory may still be reading the source after it
// returns, and the caller's int arrays die with the call.  Small metadata is
// therefore copied into a pinned slot first; an event per slot says when the
// device copy has drained it.  One ring per device, created on first use.
namespace {
struct Slot {
    void *host = nullptr;
    size_t cap = 0;
    hipEvent_t ev = nullptr;
    bool busy = false;
};
struct Ring {
    Slot slots[16];
    int next = 0;
};
std::mutex g_ring_mu;
Ring g_rings[16];
}  // namespace

int stage_to_device(void *dst, const void *src, size_t bytes, hipStream_t stream) {
    if (bytes == 0) return FLA_OK;
    // A captured copy would be replayed from a pinned slot that later calls recycle, i.e. with other calls' metadata,
    // never validated for the replayed launch; and the slot's event would belong to the capture.  Calls that carry host
    // integer arrays therefore stay out of graphs.
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone)
        return fail(FLA_ERR_UNSUPPORTED,
                    "host integer arrays (cu_seqlens, chunk_indices, query_start_loc, cache_indices, ...) cannot be uploaded "
                    "while the stream is being captured; keep this call out of the graph.");
    int dev = 0;
    FLA_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= 16) return fail(FLA_ERR_UNSUPPORTED, "device index %d out of range.", dev);
    std::lock_guard<std::mutex> lock(g_ring_mu);
    Ring &ring = g_rings[dev];
    Slot &s = ring.slots[ring.next];
    ring.next = (ring.next + 1) % 16;
    if (s.busy) {
        s.busy = false;
        if (hipEventSynchronize(s.ev) != hipSuccess) {
            // The copy that was reading this slot's buffer may never have completed.  The buffer and the event are
            // retired (dropped, not freed or reused: a stuck copy may still read the memory) and the slot starts
            // again with fresh ones on its next use, so that no later call writes into memory a copy still reads.
            (void)hipGetLastError();
            s.host = nullptr;
            s.cap = 0;
            s.ev = nullptr;
            return fail(FLA_ERR_LAUNCH, "waiting for an earlier upload of host integer arrays failed.");
        }
    }
    if (s.cap < bytes) {
        if (s.host) FLA_HIP_CHECK(hipHostFree(s.host));
        s.host = nullptr;
        s.cap = 0;
        size_t cap = 4096;
        while (cap < bytes) cap *= 2;
        FLA_HIP_CHECK(hipHostMalloc(&s.host, cap, hipHostMallocDefault));
        s.cap = cap;
    }
    if (s.ev == nullptr) FLA_HIP_CHECK(hipEventCreateWithFlags(&s.ev, hipEventDisableTiming));
    memcpy(s.host, src, bytes);
    FLA_HIP_CHECK(hipMemcpyAsync(dst, s.host, bytes, hipMemcpyHostToDevice, stream));
    FLA_HIP_CHECK(hipEventRecord(s.ev, stream));
    s.busy = true;
    return FLA_OK;
}

int num_cus() {
    static int cached[16] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

// ---- per-kernel timing -------------------------------------------------------
namespace {
struct ProfRec {
    const char *name;
    hipEvent_t start, stop;
};
std::mutex g_prof_mu;
std::vector<ProfRec> g_prof;
bool g_prof_on = false;
}  // namespace

bool profile_enabled() { return g_prof_on; }
int profile_report_impl(char *buf, uint64_t cap);

bool profile_begin(const char *name, hipStream_t stream) {
    ProfRec r{name, nullptr, nullptr};
    if (hipEventCreate(&r.start) != hipSuccess) return false;
    if (hipEventCreate(&r.stop) != hipSuccess) {
        (void)hipEventDestroy(r.start);
        return false;
    }
    (void)hipEventRecord(r.start, stream);
    try {
        std::lock_guard<std::mutex> lock(g_prof_mu);
        g_prof.push_back(r);
    } catch (...) {   // no room for the record: this launch goes untimed
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
        return false;
    }
    return true;
}

void profile_end(hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_prof_mu);
    if (!g_prof.empty()) (void)hipEventRecord(g_prof.back().stop, stream);
}

}  // namespace fla

extern "C" void fla_profile_enable(int on) { fla::g_prof_on = on != 0; }

// Waits for every recorded launch, writes one "name count total_ms" line per kernel
// name into buf (NUL-terminated, truncated to cap) and clears the records.
extern "C" int fla_profile_report(char *buf, uint64_t cap) {
    const int names = fla::guarded([&] { return fla::profile_report_impl(buf, cap); });
    return names;
}

namespace fla {
int profile_report_impl(char *buf, uint64_t cap) {
    std::lock_guard<std::mutex> lock(fla::g_prof_mu);
    struct Agg { const char *name; int n; double ms; };
    std::vector<Agg> agg;
    for (auto &r : fla::g_prof) {
        float ms = 0.f;
        if (hipEventSynchronize(r.stop) == hipSuccess && hipEventElapsedTime(&ms, r.start, r.stop) == hipSuccess) {
            bool found = false;
            for (auto &a : agg)
                if (!strcmp(a.name, r.name)) { a.n++; a.ms += ms; found = true; break; }
            if (!found) agg.push_back(Agg{r.name, 1, ms});
        }
        (void)hipEventDestroy(r.start);
        (void)hipEventDestroy(r.stop);
    }
    fla::g_prof.clear();
    size_t off = 0;
    if (buf && cap) buf[0] = 0;
    for (auto &a : agg) {
        if (!buf || off >= cap) break;
        int w = snprintf(buf + off, cap - off, "%s %d %.6f\n", a.name, a.n, a.ms);
        if (w < 0) break;
        off += (size_t)w;
    }
    return (int)agg.size();
}
}  // namespace fla

extern "C" const char *fla_last_error(void) { return fla::last_error_buffer(); }
extern "C" int fla_abi_version(void) { return 1; }
