// Geometry shared by the chunked gated-delta-rule kernels: how a launch maps to
// (batch row, sequence, chunk) for dense and packed variable-length inputs.
#pragma once

#include "common.h"
#include "device_utils.h"

namespace fla {

constexpr int kChunk = 64;  // tokens per chunk of every MFMA kernel
#ifdef FLA_ELEM_F16
constexpr int kElemDtype = FLA_F16;   // dtype code of `elem` in this translation unit
#else
constexpr int kElemDtype = FLA_BF16;
#endif

struct ChunkGeom {
    int B, T;            // batch rows, tokens per row (packed total when varlen)
    int Hk, Hv;          // key / value heads (Hv % Hk == 0)
    int K, V;
    int NT;              // chunks per batch row (varlen: over all sequences)
    int N;               // sequences
    const int32_t *cu;   // [N+1] or null (dense)
    const int32_t *choff;  // [N+1] first chunk of each sequence
    const int32_t *tab;  // [NT][2] (sequence, chunk within sequence)
    int C = kChunk;      // tokens per chunk (128 where an operator supports it)
    int head_fast = 0;   // chunk-parallel launches: 1 = grid (heads, chunks, batch), neighbouring workgroups take the heads
                         // of one chunk (token-major operands: those rows are neighbours in memory); 0 = (chunks, heads, batch)
};

// Chunk-parallel launches: the (x, head) pair of this workgroup, x = chunk index (times whatever the kernel packs into
// it).  The grid is (x, heads, batch), or (heads, x, batch) when geom.head_fast is set.
__device__ __forceinline__ void block_chunk_head(const ChunkGeom &g, int &x, int &head) {
    x = g.head_fast ? blockIdx.y : blockIdx.x;
    head = g.head_fast ? blockIdx.x : blockIdx.y;
}
inline dim3 chunk_head_grid(const ChunkGeom &g, int x, int heads) {
    return g.head_fast ? dim3(heads, x, g.B) : dim3(x, heads, g.B);
}

// Head-first activations [B, H, T, D] with arbitrary outer strides and unit inner stride.
struct View4 {
    const void *p;
    int64_t sb, sh, st;
};
// Per-token scalars [B, H, T] (or [B, T, H]) through strides; f32 or the element type of the matrices.
struct View3 {
    const void *p;
    int64_t sb, sh, st;
    int is_elem;
};

__device__ __forceinline__ float load_scalar(const View3 &v, int b, int h, int t) {
    const int64_t off = b * v.sb + h * v.sh + (int64_t)t * v.st;
    return v.is_elem ? (float)static_cast<const elem *>(v.p)[off] : static_cast<const float *>(v.p)[off];
}

// The matrix-core translation units are built twice, for bf16 and for f16 elements.  The f16 object exports
// each C entry point under a hidden name with the suffix _f16; the bf16 object owns the public name and
// forwards calls whose first matrix operand is f16.
#ifdef FLA_ELEM_F16
#define FLA_ENTRY(name) extern "C" __attribute__((visibility("hidden"))) int name##_f16
#define FLA_ROUTE_F16(t, name, ...)
#else
#define FLA_ENTRY(name)                                                             \
    extern "C" __attribute__((visibility("hidden"))) decltype(name) name##_f16;     \
    extern "C" int name
#define FLA_ROUTE_F16(t, name, ...) \
    if ((t) != nullptr && (t)->dtype == FLA_F16) return name##_f16(__VA_ARGS__)
#endif

// Chunk `c` of batch row `b` -> first token and length.
__device__ __forceinline__ void chunk_span(const ChunkGeom &g, int b, int c, int &seq, int &start, int &len) {
    if (g.cu == nullptr) {
        seq = b;
        start = c * g.C;
        len = min(g.C, g.T - start);
    } else {
        seq = g.tab[2 * c];
        start = g.cu[seq] + g.tab[2 * c + 1] * g.C;
        len = min(g.C, g.cu[seq + 1] - start);
    }
}

inline View4 view4(const fla_tensor *t) { return View4{t->data, t->stride[0], t->stride[1], t->stride[2]}; }
inline View3 view3(const fla_tensor *t) {
    return View3{t->data, t->stride[0], t->stride[1], t->stride[2], t->dtype == FLA_F32 ? 0 : 1};
}

// Common validation of the [B,H,T,D] / [B,H,T] operand family; fills geometry
// (without varlen pointers).  `v` may be null when the op has no V-sized operand.
// `elem_dtype` is the dtype code the matrices must have (per-token scalars: that or f32).
// `max_chunk` = 128 for the operators that are also built for 128-token chunks.
int gdn_geometry(const char *op, const fla_tensor *k, const fla_tensor *v_like, const fla_tensor *g_like,
                 int64_t chunk_size, ChunkGeom &geom, int elem_dtype = FLA_BF16, int max_chunk = kChunk);
int check_bhtd(const char *op, const char *name, const fla_tensor *t, int64_t B, int64_t H, int64_t T, int64_t D,
               int dtype_mask);
int check_bht(const char *op, const char *name, const fla_tensor *t, int64_t B, int64_t H, int64_t T,
              int elem_dtype = FLA_BF16);
// Validates cu_seqlens / chunk_indices, reports the workspace (query != null) or uploads the chunk table
// into `workspace` and completes `geom` with the device pointers.
int finish_varlen(const char *op, Varlen &vl, ChunkGeom &geom, const fla_int_array *cu, const fla_int_array *ci,
                  void *workspace, uint64_t workspace_size, hipStream_t stream, uint64_t *query, int chunk = 0);

}  // namespace fla
