// extern "C" entry points of libkascade_hip.so: argument validation, launch
// sequencing, error reporting.  No allocation happens here; every buffer is the
// caller's.  Validation failures are reported before anything is launched, so
// they can be exercised on a machine without a GPU.
#include "../../include/kascade_hip.h"
#include "../../include/kascade_hip_diag.h"

#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <mutex>

#include "decode.h"
#include "diag.h"
#include "paged.h"
#include "prefill.h"
#include "topk.h"

using namespace kascade;

namespace {

thread_local char g_err[1024] = "";
int g_cu_count = 0;

// Scratch of kascade_decode_reuse_paged_noalloc_call: the partial log-sums [batch,32,num_split]
// and partial outputs [batch,32,num_split,128] of the splits, fp32, for up to kNoAllocUnits
// (sequence, split) pairs.  Every device the library runs on holds its own copy of the array at
// its own address until the process ends; host code never uses the array's name as an address but
// the pointer hipGetSymbolAddress returns for the current device (g_noalloc_ptr).
constexpr int kNoAllocUnits = 1024;
constexpr size_t kNoAllocFloats = (size_t)kNoAllocUnits * kHeads * (1 + kDim);   // 16.9 MB
static __device__ __align__(256) float scratch[kNoAllocFloats];
constexpr int kMaxDevices = 64;
float* g_noalloc_ptr[kMaxDevices] = {};
std::mutex g_noalloc_mutex;   // host threads that meet in the first call on a device

int fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return -1;
}

int check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return 0;
    return fail("%s: %s", what, hipGetErrorString(e));
}

#define REQUIRE(cond, ...)                 \
    do {                                   \
        if (!(cond)) return fail(__VA_ARGS__); \
    } while (0)

inline const half_t* H(const kascade_half* p) { return reinterpret_cast<const half_t*>(p); }
inline half_t* H(kascade_half* p) { return reinterpret_cast<half_t*>(p); }
// element tensors whose type (fp16 or bf16) the shape decides
inline const void* E(const kascade_half* p) { return p; }
inline void* E(kascade_half* p) { return p; }

// Device address of `scratch` on the current device, looked up once per device.
int noalloc_scratch(float** out) {
    int dev = 0;
    if (check_hip(hipGetDevice(&dev), "hipGetDevice")) return -1;
    REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    if (!g_noalloc_ptr[dev]) {
        void* ptr = nullptr;
        if (check_hip(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)"))
            return -1;
        REQUIRE(ptr != nullptr, "hipGetSymbolAddress(scratch) returned a null address");
        g_noalloc_ptr[dev] = static_cast<float*>(ptr);
    }
    *out = g_noalloc_ptr[dev];
    return 0;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_strides(const kascade_strides& s, const char* name) {
    REQUIRE(s.b % 8 == 0 && s.l % 8 == 0 && s.h % 8 == 0,
            "%s strides must be multiples of 8 elements (16-byte rows)", name);
    REQUIRE(s.l > 0 && s.h > 0, "%s strides must be positive", name);
    REQUIRE(s.l < (1LL << 31), "%s row stride must be below 2^31 elements", name);
    return 0;
}

// Shape of the tensors a call works on: KV heads, head dimension, element kind, query heads per
// KV head.  The entry points without a shape argument use the reference's.
struct Shape {
    int G, D, elem, gs;
    int H() const { return G * gs; }
};
const Shape kRefShape{kGroups, kDim, kElemF16, kGroupSize};

int get_shape(const kascade_shape* in, Shape* out) {
    REQUIRE(in, "shape: null pointer argument");
    REQUIRE(in->kv_heads >= 1 && in->kv_heads <= 65535, "shape: kv_heads out of range");
    REQUIRE(in->head_dim == 64 || in->head_dim == 128, "shape: head_dim must be 64 or 128, got %d", in->head_dim);
    REQUIRE(in->dtype == KASCADE_F16 || in->dtype == KASCADE_BF16, "shape: dtype must be KASCADE_F16 or KASCADE_BF16");
    const int gs = in->group_size == 0 ? kGroupSize : in->group_size;
    REQUIRE(gs >= 1 && gs <= 16,
            "shape: group_size (query heads per KV head) must be 1 to 16 (0 = 4), got %d", in->group_size);
    REQUIRE((long long)in->kv_heads * gs <= 65535, "shape: too many query heads");
    out->G = in->kv_heads; out->D = in->head_dim; out->elem = in->dtype == KASCADE_BF16 ? kElemBF16 : kElemF16;
    out->gs = gs;
    return 0;
}

// what the reference's scratch shapes fix for its decode kernels (attention_utils.py:36-59)
constexpr int kRefNumSplit = 8;

// element strides of a contiguous [B,seq_len,heads,128] tensor
kascade_strides contiguous_strides(int seq_len, int heads) {
    return kascade_strides{(int64_t)seq_len * heads * kDim, (int64_t)heads * kDim, (int64_t)kDim};
}

int rows_per_split(long long max_rows, int num_split) {
    long long r = (max_rows + num_split - 1) / num_split;
    return (int)(((r + 63) / 64) * 64);
}

int check_paging(const int32_t* block_table, int max_pages, int page_size, int* page_shift) {
    if (!block_table) {
        *page_shift = 0;
        return 0;
    }
    int sh = ilog2_exact(page_size);
    REQUIRE(sh >= 0, "page_size must be a power of two, got %d", page_size);
    REQUIRE(max_pages > 0, "max_pages must be positive with a block table");
    *page_shift = sh;
    return 0;
}

// K/V addressing of the decode calls without a block table: `strides` (elements, may be NULL
// for the contiguous [B,kv_stride_tokens,G,D] cache).
int set_kv_strides(DecodeParams& p, const Shape& sh, const kascade_strides* strides,
                   const int32_t* block_table, int kv_stride_tokens) {
    p.G = sh.G; p.head_dim = sh.D; p.elem = sh.elem; p.gs = sh.gs;
    if (!strides) {
        p.kv_stride_b = (long long)kv_stride_tokens * sh.G * sh.D;
        p.kv_stride_l = sh.G * sh.D;
        p.kv_stride_h = sh.D;
        return 0;
    }
    REQUIRE(!block_table, "kv_strides and block_table exclude each other");
    if (check_strides(*strides, "decode K/V")) return -1;
    REQUIRE(strides->b >= 0, "decode K/V batch stride must not be negative");
    p.kv_stride_b = strides->b;
    p.kv_stride_l = (unsigned)strides->l;
    p.kv_stride_h = strides->h;
    return 0;
}

// Fused append of the decode calls: both rows or neither; the caches are written through the
// K / V arguments.
int set_append(DecodeParams& p, const kascade_half* k_new, const kascade_half* v_new,
               const kascade_half* K, const kascade_half* V) {
    if (!k_new && !v_new) return 0;
    REQUIRE(k_new && v_new && K && V, "k_new and v_new come together, with both caches");
    REQUIRE(aligned16(k_new) && aligned16(v_new), "k_new/v_new must be 16-byte aligned");
    p.k_new = H(k_new); p.v_new = H(v_new);
    p.k_cache = const_cast<half_t*>(H(K)); p.v_cache = const_cast<half_t*>(H(V));
    return 0;
}

}  // namespace

extern "C" {

int kascade_abi_version(void) { return 10; }

const char* kascade_get_last_error(void) { return g_err; }

int kascade_device_cu_count(void) { return g_cu_count; }

int kascade_init(void) {
    int dev = 0;
    if (check_hip(hipGetDevice(&dev), "hipGetDevice")) return -1;
    hipDeviceProp_t prop;
    if (check_hip(hipGetDeviceProperties(&prop, dev), "hipGetDeviceProperties")) return -1;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail("libkascade_hip is built for gfx950 only; device is %s", prop.gcnArchName);
    g_cu_count = prop.multiProcessorCount;
    float* ptr;
    return noalloc_scratch(&ptr);   // this device's copy of the scratch array
}

int kascade_decode_reuse_call(const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                              const int32_t* topk_indices, const int32_t* head_mapping,
                              float* glse, float* Output_partial, kascade_half* Output, int batch,
                              int kv_seqlen, int topk, int num_split, int32_t* sync_counters,
                              void* stream) {
    return kascade_decode_reuse_paged_call(Q, K, V, nullptr, topk_indices, head_mapping, 0.f, glse,
                                           Output_partial, Output, batch, kv_seqlen, topk,
                                           num_split, nullptr, 0, 1, nullptr, nullptr, nullptr, sync_counters,
                                           nullptr, stream);
}

}  // extern "C"
namespace {
int decode_reuse_paged_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K,
                                    const kascade_half* V, const int32_t* cache_seqlens,
                                    const int32_t* topk_indices, const int32_t* head_mapping,
                                    float topk_percent, float* glse, float* Output_partial,
                                    kascade_half* Output, int batch, int kv_stride_tokens,
                                    int topk, int num_split, const int32_t* block_table,
                                    int max_pages, int page_size, const kascade_strides* kv_strides,
                                    const kascade_half* k_new, const kascade_half* v_new,
                                    int32_t* sync_counters, float* log_sum, void* stream) {
    REQUIRE(Q && K && V && topk_indices && head_mapping && glse && Output_partial && Output,
            "decode_reuse: null pointer argument");
    REQUIRE(batch > 0 && topk > 0 && num_split > 0, "decode_reuse: batch, topk, num_split must be > 0");
    REQUIRE(batch <= 65535, "decode_reuse: batch exceeds grid limit");
    REQUIRE(block_table || kv_stride_tokens > 0, "decode_reuse: kv_stride_tokens must be > 0");
    REQUIRE(!(topk_percent > 0.f) || cache_seqlens, "decode_reuse: topk_percent needs cache_seqlens");
    REQUIRE(aligned16(Q) && aligned16(K) && aligned16(V), "decode_reuse: Q/K/V must be 16-byte aligned");
    int shift;
    if (check_paging(block_table, max_pages, page_size, &shift)) return -1;
    DecodeParams p{};
    p.Q = H(Q); p.K = H(K); p.V = H(V);
    p.seqlens = cache_seqlens; p.idx = topk_indices; p.head_map = head_mapping;
    p.block_table = block_table; p.glse = glse; p.opart = Output_partial; p.scores = nullptr;
    p.max_pages = max_pages; p.page_shift = shift; p.kv_stride_tokens = kv_stride_tokens;
    if (set_kv_strides(p, sh, kv_strides, block_table, kv_stride_tokens)) return -1;
    if (set_append(p, k_new, v_new, K, V)) return -1;
    p.topk = topk; p.topk_percent = topk_percent; p.scores_stride = 0; p.num_split = num_split;
    p.rows_per_split = rows_per_split(topk, num_split);
    p.B = batch;
    p.counters = sync_counters; p.out = H(Output); p.row_sums = log_sum;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (check_hip(launch_decode_split(p, true, true, false, s), "decode_reuse split")) return -1;
    if (sync_counters) return 0;   // the split kernel's last workgroups have combined
    return check_hip(launch_decode_combine(glse, Output_partial, E(Output), log_sum, batch, sh.H(), num_split, true, sh.D, sh.elem, s), "decode_reuse combine");
}
}  // namespace
extern "C" {

int kascade_decode_reuse_paged_call(const kascade_half* Q, const kascade_half* K,
                                    const kascade_half* V, const int32_t* cache_seqlens,
                                    const int32_t* topk_indices, const int32_t* head_mapping,
                                    float topk_percent, float* glse, float* Output_partial,
                                    kascade_half* Output, int batch, int kv_stride_tokens,
                                    int topk, int num_split, const int32_t* block_table,
                                    int max_pages, int page_size, const kascade_strides* kv_strides,
                                    const kascade_half* k_new, const kascade_half* v_new,
                                    int32_t* sync_counters, float* log_sum, void* stream) {
    return decode_reuse_paged_impl(kRefShape, Q, K, V, cache_seqlens, topk_indices, head_mapping, topk_percent, glse, Output_partial, Output, batch, kv_stride_tokens, topk, num_split, block_table, max_pages, page_size, kv_strides, k_new, v_new, sync_counters, log_sum, stream);
}

int kascade_decode_reuse_paged_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K,
                                    const kascade_half* V, const int32_t* cache_seqlens,
                                    const int32_t* topk_indices, const int32_t* head_mapping,
                                    float topk_percent, float* glse, float* Output_partial,
                                    kascade_half* Output, int batch, int kv_stride_tokens,
                                    int topk, int num_split, const int32_t* block_table,
                                    int max_pages, int page_size, const kascade_strides* kv_strides,
                                    const kascade_half* k_new, const kascade_half* v_new,
                                    int32_t* sync_counters, float* log_sum, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return decode_reuse_paged_impl(sh, Q, K, V, cache_seqlens, topk_indices, head_mapping, topk_percent, glse, Output_partial, Output, batch, kv_stride_tokens, topk, num_split, block_table, max_pages, page_size, kv_strides, k_new, v_new, sync_counters, log_sum, stream);
}

}  // extern "C"
namespace {
int decode_reuse_rows_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K_pages,
                                   const kascade_half* V_pages, const int32_t* cache_seqlens,
                                   const int32_t* cache_rows, const int32_t* head_mapping,
                                   float topk_percent, float* glse, float* Output_partial,
                                   kascade_half* Output, int batch, int topk, int num_split,
                                   const int32_t* block_table, int max_pages, int page_size,
                                   int num_pages, const kascade_half* k_new,
                                   const kascade_half* v_new, int32_t* sync_counters, float* log_sum, void* stream) {
    REQUIRE(Q && K_pages && V_pages && cache_rows && head_mapping && glse && Output_partial && Output &&
                block_table, "decode_reuse_rows: null pointer argument");
    REQUIRE(batch > 0 && topk > 0 && num_split > 0, "decode_reuse_rows: batch, topk, num_split must be > 0");
    REQUIRE(batch <= 65535, "decode_reuse_rows: batch exceeds grid limit");
    REQUIRE(!(topk_percent > 0.f) || cache_seqlens, "decode_reuse_rows: topk_percent needs cache_seqlens");
    REQUIRE(!k_new || cache_seqlens, "decode_reuse_rows: the fused append needs cache_seqlens");
    REQUIRE(aligned16(Q) && aligned16(K_pages) && aligned16(V_pages),
            "decode_reuse_rows: Q/K/V must be 16-byte aligned");
    int shift;
    if (check_paging(block_table, max_pages, page_size, &shift)) return -1;
    REQUIRE(num_pages > 0 && (long long)num_pages * page_size < (1LL << 31),
            "decode_reuse_rows: num_pages out of range");
    DecodeParams p{};
    p.Q = H(Q); p.K = H(K_pages); p.V = H(V_pages);
    p.seqlens = cache_seqlens; p.idx = cache_rows; p.head_map = head_mapping;
    p.idx_physical = 1; p.max_row = num_pages * page_size - 1;
    p.block_table = block_table; p.glse = glse; p.opart = Output_partial; p.scores = nullptr;
    p.max_pages = max_pages; p.page_shift = shift; p.kv_stride_tokens = 0;
    if (set_kv_strides(p, sh, nullptr, block_table, 0)) return -1;
    if (set_append(p, k_new, v_new, K_pages, V_pages)) return -1;
    p.topk = topk; p.topk_percent = topk_percent; p.scores_stride = 0; p.num_split = num_split;
    p.rows_per_split = rows_per_split(topk, num_split);
    p.B = batch;
    p.counters = sync_counters; p.out = H(Output); p.row_sums = log_sum;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (check_hip(launch_decode_split(p, true, true, false, s), "decode_reuse_rows split")) return -1;
    if (sync_counters) return 0;
    return check_hip(launch_decode_combine(glse, Output_partial, E(Output), log_sum, batch, sh.H(), num_split, true, sh.D, sh.elem, s), "decode_reuse_rows combine");
}
}  // namespace
extern "C" {

int kascade_decode_reuse_rows_call(const kascade_half* Q, const kascade_half* K_pages,
                                   const kascade_half* V_pages, const int32_t* cache_seqlens,
                                   const int32_t* cache_rows, const int32_t* head_mapping,
                                   float topk_percent, float* glse, float* Output_partial,
                                   kascade_half* Output, int batch, int topk, int num_split,
                                   const int32_t* block_table, int max_pages, int page_size,
                                   int num_pages, const kascade_half* k_new,
                                   const kascade_half* v_new, int32_t* sync_counters, float* log_sum, void* stream) {
    return decode_reuse_rows_impl(kRefShape, Q, K_pages, V_pages, cache_seqlens, cache_rows, head_mapping, topk_percent, glse, Output_partial, Output, batch, topk, num_split, block_table, max_pages, page_size, num_pages, k_new, v_new, sync_counters, log_sum, stream);
}

int kascade_decode_reuse_rows_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K_pages,
                                   const kascade_half* V_pages, const int32_t* cache_seqlens,
                                   const int32_t* cache_rows, const int32_t* head_mapping,
                                   float topk_percent, float* glse, float* Output_partial,
                                   kascade_half* Output, int batch, int topk, int num_split,
                                   const int32_t* block_table, int max_pages, int page_size,
                                   int num_pages, const kascade_half* k_new,
                                   const kascade_half* v_new, int32_t* sync_counters, float* log_sum, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return decode_reuse_rows_impl(sh, Q, K_pages, V_pages, cache_seqlens, cache_rows, head_mapping, topk_percent, glse, Output_partial, Output, batch, topk, num_split, block_table, max_pages, page_size, num_pages, k_new, v_new, sync_counters, log_sum, stream);
}

int kascade_decode_reuse_paged_noalloc_call(const kascade_half* Q, const kascade_half* K,
                                            const kascade_half* V, const int32_t* cache_seqlens,
                                            const int32_t* topk_indices, const int32_t* head_mapping,
                                            float topk_percent, kascade_half* Output, int batch,
                                            int kv_stride_tokens, int topk, int num_split,
                                            const int32_t* block_table, int max_pages, int page_size,
                                            const kascade_strides* kv_strides,
                                            const kascade_half* k_new, const kascade_half* v_new,
                                            void* stream) {
    REQUIRE(batch > 0 && num_split > 0, "decode_reuse_noalloc: batch, num_split must be > 0");
    REQUIRE((long long)batch * num_split <= kNoAllocUnits,
            "decode_reuse_noalloc: batch * num_split = %lld exceeds the built-in scratch (%d); "
            "use kascade_decode_reuse_paged_call with caller-provided scratch",
            (long long)batch * num_split, kNoAllocUnits);
    float* base;
    if (noalloc_scratch(&base)) return -1;
    float* glse = base;                                           // [batch,32,num_split]
    float* opart = base + (size_t)kNoAllocUnits * kHeads;         // [batch,32,num_split,128]
    return decode_reuse_paged_impl(kRefShape, Q, K, V, cache_seqlens, topk_indices, head_mapping,
                                           topk_percent, glse, opart, Output, batch,
                                           kv_stride_tokens, topk, num_split, block_table, max_pages,
                                           page_size, kv_strides, k_new, v_new, nullptr, nullptr, stream);
}

}  // extern "C"
namespace {
int decode_dense_paged_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K,
                                    const kascade_half* V, const int32_t* cache_seqlens,
                                    float* glse, float* Output_partial, kascade_half* Output,
                                    int batch, int kv_stride_tokens, int num_split,
                                    const int32_t* block_table, int max_pages, int page_size,
                                    const kascade_strides* kv_strides, const kascade_half* k_new,
                                    const kascade_half* v_new, int32_t* sync_counters,
                                    void* stream) {
    REQUIRE(Q && K && V && glse && Output_partial && Output, "decode_dense: null pointer argument");
    REQUIRE(batch > 0 && num_split > 0, "decode_dense: batch, num_split must be > 0");
    REQUIRE(batch <= 65535, "decode_dense: batch exceeds grid limit");
    REQUIRE(cache_seqlens || kv_stride_tokens > 0, "decode_dense: need cache_seqlens or kv_stride_tokens");
    REQUIRE(block_table || kv_stride_tokens > 0, "decode_dense: kv_stride_tokens must be > 0");
    REQUIRE(aligned16(Q) && aligned16(K) && aligned16(V), "decode_dense: Q/K/V must be 16-byte aligned");
    int shift;
    if (check_paging(block_table, max_pages, page_size, &shift)) return -1;
    DecodeParams p{};
    p.Q = H(Q); p.K = H(K); p.V = H(V);
    p.seqlens = cache_seqlens; p.block_table = block_table; p.glse = glse; p.opart = Output_partial;
    p.max_pages = max_pages; p.page_shift = shift; p.kv_stride_tokens = kv_stride_tokens;
    if (set_kv_strides(p, sh, kv_strides, block_table, kv_stride_tokens)) return -1;
    if (set_append(p, k_new, v_new, K, V)) return -1;
    p.num_split = num_split; p.B = batch;
    const long long max_rows = kv_stride_tokens > 0 ? kv_stride_tokens : (long long)max_pages * page_size;
    p.rows_per_split = rows_per_split(max_rows, num_split);
    p.counters = sync_counters; p.out = H(Output);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (check_hip(launch_decode_split(p, false, true, false, s), "decode_dense split")) return -1;
    if (sync_counters) return 0;
    return check_hip(launch_decode_combine(glse, Output_partial, E(Output), nullptr, batch, sh.H(), num_split, true, sh.D, sh.elem, s), "decode_dense combine");
}
}  // namespace
extern "C" {

int kascade_decode_dense_paged_call(const kascade_half* Q, const kascade_half* K,
                                    const kascade_half* V, const int32_t* cache_seqlens,
                                    float* glse, float* Output_partial, kascade_half* Output,
                                    int batch, int kv_stride_tokens, int num_split,
                                    const int32_t* block_table, int max_pages, int page_size,
                                    const kascade_strides* kv_strides, const kascade_half* k_new,
                                    const kascade_half* v_new, int32_t* sync_counters,
                                    void* stream) {
    return decode_dense_paged_impl(kRefShape, Q, K, V, cache_seqlens, glse, Output_partial, Output, batch, kv_stride_tokens, num_split, block_table, max_pages, page_size, kv_strides, k_new, v_new, sync_counters, stream);
}

int kascade_decode_dense_paged_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K,
                                    const kascade_half* V, const int32_t* cache_seqlens,
                                    float* glse, float* Output_partial, kascade_half* Output,
                                    int batch, int kv_stride_tokens, int num_split,
                                    const int32_t* block_table, int max_pages, int page_size,
                                    const kascade_strides* kv_strides, const kascade_half* k_new,
                                    const kascade_half* v_new, int32_t* sync_counters,
                                    void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return decode_dense_paged_impl(sh, Q, K, V, cache_seqlens, glse, Output_partial, Output, batch, kv_stride_tokens, num_split, block_table, max_pages, page_size, kv_strides, k_new, v_new, sync_counters, stream);
}

}  // extern "C"
namespace {
int decode_recompute_paged_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K,
                                        const kascade_half* V, const int32_t* cache_seqlens,
                                        float* glse, float* Output_partial, float* row_sums,
                                        float* scores, kascade_half* Output,
                                        kascade_half* aggregated_scores, int batch,
                                        int kv_stride_tokens, int scores_stride, int num_split,
                                        int with_output, const int32_t* block_table,
                                        int max_pages, int page_size,
                                        const kascade_strides* kv_strides,
                                        const kascade_half* k_new, const kascade_half* v_new,
                                        int32_t* sync_counters, void* stream) {
    REQUIRE(Q && K && glse && row_sums && scores && aggregated_scores,
            "decode_recompute: null pointer argument");
    REQUIRE(!with_output || (V && Output && Output_partial),
            "decode_recompute: with_output needs V, Output and Output_partial");
    REQUIRE(batch > 0 && num_split > 0 && scores_stride > 0,
            "decode_recompute: batch, num_split, scores_stride must be > 0");
    REQUIRE(scores_stride % 8 == 0, "decode_recompute: scores_stride must be a multiple of 8");
    REQUIRE(batch <= 65535, "decode_recompute: batch exceeds grid limit");
    REQUIRE(cache_seqlens || (kv_stride_tokens > 0 && kv_stride_tokens <= scores_stride),
            "decode_recompute: without cache_seqlens need 0 < kv_stride_tokens <= scores_stride");
    REQUIRE(block_table || kv_stride_tokens > 0, "decode_recompute: kv_stride_tokens must be > 0");
    REQUIRE(aligned16(Q) && aligned16(K) && (!with_output || aligned16(V)),
            "decode_recompute: Q/K/V must be 16-byte aligned");
    REQUIRE(aligned16(scores) && aligned16(aggregated_scores),
            "decode_recompute: scores buffers must be 16-byte aligned");
    int shift;
    if (check_paging(block_table, max_pages, page_size, &shift)) return -1;
    DecodeParams p{};
    p.Q = H(Q); p.K = H(K); p.V = with_output ? H(V) : H(K);
    p.seqlens = cache_seqlens; p.block_table = block_table; p.glse = glse; p.opart = Output_partial;
    p.scores = scores; p.scores_stride = scores_stride;
    p.max_pages = max_pages; p.page_shift = shift; p.kv_stride_tokens = kv_stride_tokens;
    if (set_kv_strides(p, sh, kv_strides, block_table, kv_stride_tokens)) return -1;
    if (set_append(p, k_new, v_new, K, V)) return -1;
    p.num_split = num_split; p.B = batch;
    long long max_rows = kv_stride_tokens > 0 ? kv_stride_tokens : (long long)max_pages * page_size;
    if (max_rows > scores_stride) max_rows = scores_stride;
    p.rows_per_split = rows_per_split(max_rows, num_split);
    p.counters = sync_counters; p.out = H(Output); p.row_sums = row_sums;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (check_hip(launch_decode_split(p, false, with_output != 0, true, s), "decode_recompute split"))
        return -1;
    // the kernels cut every sequence length down to this (decode_split_kernel's safe_len)
    long long len_cap = block_table ? (long long)max_pages * page_size : (long long)kv_stride_tokens;
    if (len_cap > scores_stride) len_cap = scores_stride;
    // Without an output the only thing left to merge is the log-sums, which the aggregate
    // launch does for itself: no combine launch.
    const bool merge_in_aggregate = !sync_counters && !with_output;
    if (!sync_counters && with_output &&
        check_hip(launch_decode_combine(glse, Output_partial, E(Output), row_sums, batch, sh.H(), num_split, true, sh.D, sh.elem, s), "decode_recompute combine"))
        return -1;
    return check_hip(launch_decode_aggregate(scores, merge_in_aggregate ? nullptr : row_sums,
                                             merge_in_aggregate ? glse : nullptr, num_split, row_sums,
                                             cache_seqlens, H(aggregated_scores), batch, sh.G, sh.gs, scores_stride,
                                             kv_stride_tokens, (int)len_cap, s),
                     "decode_recompute aggregate");
}
}  // namespace
extern "C" {

int kascade_decode_recompute_paged_call(const kascade_half* Q, const kascade_half* K,
                                        const kascade_half* V, const int32_t* cache_seqlens,
                                        float* glse, float* Output_partial, float* row_sums,
                                        float* scores, kascade_half* Output,
                                        kascade_half* aggregated_scores, int batch,
                                        int kv_stride_tokens, int scores_stride, int num_split,
                                        int with_output, const int32_t* block_table,
                                        int max_pages, int page_size,
                                        const kascade_strides* kv_strides,
                                        const kascade_half* k_new, const kascade_half* v_new,
                                        int32_t* sync_counters, void* stream) {
    return decode_recompute_paged_impl(kRefShape, Q, K, V, cache_seqlens, glse, Output_partial, row_sums, scores, Output, aggregated_scores, batch, kv_stride_tokens, scores_stride, num_split, with_output, block_table, max_pages, page_size, kv_strides, k_new, v_new, sync_counters, stream);
}

int kascade_decode_recompute_paged_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K,
                                        const kascade_half* V, const int32_t* cache_seqlens,
                                        float* glse, float* Output_partial, float* row_sums,
                                        float* scores, kascade_half* Output,
                                        kascade_half* aggregated_scores, int batch,
                                        int kv_stride_tokens, int scores_stride, int num_split,
                                        int with_output, const int32_t* block_table,
                                        int max_pages, int page_size,
                                        const kascade_strides* kv_strides,
                                        const kascade_half* k_new, const kascade_half* v_new,
                                        int32_t* sync_counters, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return decode_recompute_paged_impl(sh, Q, K, V, cache_seqlens, glse, Output_partial, row_sums, scores, Output, aggregated_scores, batch, kv_stride_tokens, scores_stride, num_split, with_output, block_table, max_pages, page_size, kv_strides, k_new, v_new, sync_counters, stream);
}

int64_t kascade_topk_workspace_bytes(int rows, int64_t row_len) {
    return topk_split_workspace_bytes(rows, row_len);
}

int kascade_topk_call(const kascade_half* scores, int32_t* out_idx, int rows, int64_t row_stride,
                      int uniform_len, const int32_t* valid_len, const int32_t* n_sel, int period,
                      int k, int fill_value, void* workspace, void* stream) {
    return kascade_topk_rows_call(scores, out_idx, rows, row_stride, uniform_len, valid_len, n_sel,
                                  period, k, fill_value, workspace, nullptr, nullptr, 0, 1, 1, stream);
}

int kascade_topk_rows_call(const kascade_half* scores, int32_t* out_idx, int rows, int64_t row_stride,
                           int uniform_len, const int32_t* valid_len, const int32_t* n_sel, int period,
                           int k, int fill_value, void* workspace, int32_t* out_rows,
                           const int32_t* block_table, int max_pages, int page_size,
                           int rows_per_sequence, void* stream) {
    REQUIRE(scores && out_idx, "topk: null pointer argument");
    TopkRows tr{};
    if (out_rows) {
        REQUIRE(block_table && rows_per_sequence > 0, "topk: out_rows needs a block table and rows_per_sequence > 0");
        int shift;
        if (check_paging(block_table, max_pages, page_size, &shift)) return -1;
        REQUIRE((long long)max_pages * page_size >= uniform_len,
                "topk: block table shorter than the rows it is to translate");
        tr.out_rows = out_rows; tr.block_table = block_table; tr.max_pages = max_pages;
        tr.page_shift = shift; tr.rows_per_seq = rows_per_sequence;
    }
    REQUIRE(rows >= 0 && k > 0 && row_stride > 0, "topk: rows >= 0, k > 0, row_stride > 0 required");
    REQUIRE(uniform_len >= 0 && uniform_len <= row_stride,
            "topk: uniform_len must be within [0, row_stride]");
    REQUIRE(!(valid_len || n_sel) || period > 0, "topk: period must be > 0 with per-row arrays");
    if (period <= 0) period = 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // rows of up to 131072 entries that start 16-byte aligned fit one workgroup's registers: one
    // launch; longer (or unaligned long) rows go to several workgroups per row, four launches
    const bool one_workgroup = uniform_len + (row_stride % 8 != 0 ? 7 : 0) <= topk_max_register_row() &&
                               (reinterpret_cast<uintptr_t>(scores) & 15) == 0;
    if (!one_workgroup && workspace && topk_split_workspace_bytes(rows, uniform_len) > 0)
        return check_hip(launch_topk_split(H(scores), out_idx, rows, row_stride, uniform_len,
                                           uniform_len, valid_len, n_sel, period, k, fill_value,
                                           workspace, &tr, s), "topk (split)");
    return check_hip(launch_topk(H(scores), out_idx, rows, row_stride, uniform_len, valid_len, n_sel,
                                 period, k, fill_value, &tr, s), "topk");
}

namespace {
inline long long sorted_list_bytes(int rows, int k) {
    return (topk_sort_workspace_bytes(rows, k) + 255) / 256 * 256;
}
}  // namespace

int64_t kascade_topk_sorted_workspace_bytes(int rows, int64_t row_len, int k) {
    if (rows < 0 || k < 0) return 0;
    return sorted_list_bytes(rows, k) + topk_split_workspace_bytes(rows, row_len);
}

int kascade_topk_sorted_call(const kascade_half* scores, int32_t* out_idx, int rows, int64_t row_stride,
                             int uniform_len, const int32_t* valid_len, int period, int k,
                             void* workspace, void* stream) {
    REQUIRE(k > 0 && k <= uniform_len, "topk_sorted: 0 < k <= uniform_len required (as torch.topk)");
    REQUIRE(rows >= 0, "topk_sorted: rows >= 0 required");
    REQUIRE(workspace || kascade_topk_sorted_workspace_bytes(rows, uniform_len, k) == 0,
            "topk_sorted: workspace of kascade_topk_sorted_workspace_bytes() bytes required");
    char* ws = static_cast<char*>(workspace);
    void* split_ws = topk_split_workspace_bytes(rows, uniform_len) > 0 ? ws + sorted_list_bytes(rows, k) : nullptr;
    // the k largest of every row in position order (all valid positions, then the first positions
    // past the row's end, when a row holds fewer than k), then the reordering by score
    if (kascade_topk_call(scores, out_idx, rows, row_stride, uniform_len, valid_len, nullptr, period, k, 0,
                          split_ws, stream))
        return -1;
    if (period <= 0) period = 1;
    return check_hip(launch_topk_sort_rows(H(scores), out_idx, ws, rows, row_stride, uniform_len, valid_len,
                                           period, k, static_cast<hipStream_t>(stream)), "topk_sorted");
}

}  // extern "C"
namespace {
int prefill_dense_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                               float* log_sum, kascade_half* Output, int batch, int seq_len,
                               kascade_strides q_strides, kascade_strides kv_strides,
                               int with_output, void* stream) {
    REQUIRE(Q && K, "prefill_dense: null pointer argument");
    REQUIRE(!with_output || (V && Output), "prefill_dense: with_output needs V and Output");
    REQUIRE(with_output || log_sum, "prefill_dense: nothing to compute (no Output, no log_sum)");
    REQUIRE(batch > 0 && seq_len > 0 && batch <= 65535, "prefill_dense: bad batch/seq_len");
    REQUIRE(aligned16(Q) && aligned16(K) && (!with_output || (aligned16(V) && aligned16(Output))),
            "prefill_dense: tensors must be 16-byte aligned");
    if (check_strides(q_strides, "Q") || check_strides(kv_strides, "K/V")) return -1;
    PrefillParams p{};
    p.G = sh.G; p.head_dim = sh.D; p.elem = sh.elem; p.gs = sh.gs;
    p.Q = H(Q); p.K = H(K); p.V = with_output ? H(V) : H(K); p.log_sum = log_sum; p.O = H(Output);
    p.q_sb = q_strides.b; p.q_sl = q_strides.l; p.q_sh = q_strides.h;
    p.k_sb = kv_strides.b; p.k_sl = kv_strides.l; p.k_sh = kv_strides.h;
    p.B = batch; p.L = seq_len; p.Lq = seq_len; p.T = (seq_len + kTile - 1) / kTile;
    return check_hip(launch_prefill_attn(p, false, with_output != 0, (with_output || sh.D != 128) ? 1 : 2,
                                         static_cast<hipStream_t>(stream)), "prefill_dense");
}
}  // namespace
extern "C" {

int kascade_prefill_dense_call(const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                               float* log_sum, kascade_half* Output, int batch, int seq_len,
                               kascade_strides q_strides, kascade_strides kv_strides,
                               int with_output, void* stream) {
    return prefill_dense_impl(kRefShape, Q, K, V, log_sum, Output, batch, seq_len, q_strides, kv_strides, with_output, stream);
}

int kascade_prefill_dense_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                               float* log_sum, kascade_half* Output, int batch, int seq_len,
                               kascade_strides q_strides, kascade_strides kv_strides,
                               int with_output, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return prefill_dense_impl(sh, Q, K, V, log_sum, Output, batch, seq_len, q_strides, kv_strides, with_output, stream);
}

}  // extern "C"
namespace {
int prefill_aggregate_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K,
                                   const float* log_sum, kascade_half* aggregate_scores, int batch,
                                   int seq_len, kascade_strides q_strides,
                                   kascade_strides kv_strides, int fill_invalid, void* stream) {
    REQUIRE(Q && K && log_sum && aggregate_scores, "prefill_aggregate: null pointer argument");
    REQUIRE(batch > 0 && seq_len > 0 && batch <= 65535, "prefill_aggregate: bad batch/seq_len");
    REQUIRE(aligned16(Q) && aligned16(K), "prefill_aggregate: Q/K must be 16-byte aligned");
    if (check_strides(q_strides, "Q") || check_strides(kv_strides, "K")) return -1;
    PrefillParams p{};
    p.G = sh.G; p.head_dim = sh.D; p.elem = sh.elem; p.gs = sh.gs;
    p.Q = H(Q); p.K = H(K); p.V = H(K); p.log_sum_in = log_sum; p.agg = H(aggregate_scores);
    p.q_sb = q_strides.b; p.q_sl = q_strides.l; p.q_sh = q_strides.h;
    p.k_sb = kv_strides.b; p.k_sl = kv_strides.l; p.k_sh = kv_strides.h;
    p.B = batch; p.L = seq_len; p.Lq = seq_len; p.T = (seq_len + kTile - 1) / kTile; p.fill_invalid = fill_invalid;
    return check_hip(launch_prefill_aggregate(p, static_cast<hipStream_t>(stream)),
                     "prefill_aggregate");
}
}  // namespace
extern "C" {

int kascade_prefill_aggregate_call(const kascade_half* Q, const kascade_half* K,
                                   const float* log_sum, kascade_half* aggregate_scores, int batch,
                                   int seq_len, kascade_strides q_strides,
                                   kascade_strides kv_strides, int fill_invalid, void* stream) {
    return prefill_aggregate_impl(kRefShape, Q, K, log_sum, aggregate_scores, batch, seq_len, q_strides, kv_strides, fill_invalid, stream);
}

int kascade_prefill_aggregate_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K,
                                   const float* log_sum, kascade_half* aggregate_scores, int batch,
                                   int seq_len, kascade_strides q_strides,
                                   kascade_strides kv_strides, int fill_invalid, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return prefill_aggregate_impl(sh, Q, K, log_sum, aggregate_scores, batch, seq_len, q_strides, kv_strides, fill_invalid, stream);
}

}  // extern "C"
namespace {
int prefill_aggregate_range_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K,
                                         const float* log_sum, kascade_half* aggregate_scores,
                                         int batch, int q_start, int q_len,
                                         kascade_strides q_strides, kascade_strides kv_strides,
                                         int fill_invalid, void* stream) {
    REQUIRE(Q && K && log_sum && aggregate_scores, "prefill_aggregate_range: null pointer argument");
    REQUIRE(batch > 0 && q_len > 0 && batch <= 65535, "prefill_aggregate_range: bad batch/q_len");
    REQUIRE(q_start >= 0 && q_start % kTile == 0, "prefill_aggregate_range: q_start must be a multiple of 32");
    REQUIRE((long long)q_start + q_len < (1LL << 31), "prefill_aggregate_range: q_start + q_len out of range");
    REQUIRE(aligned16(Q) && aligned16(K), "prefill_aggregate_range: Q/K must be 16-byte aligned");
    if (check_strides(q_strides, "Q") || check_strides(kv_strides, "K")) return -1;
    PrefillParams p{};
    p.G = sh.G; p.head_dim = sh.D; p.elem = sh.elem; p.gs = sh.gs;
    p.Q = H(Q); p.K = H(K); p.V = H(K); p.log_sum_in = log_sum; p.agg = H(aggregate_scores);
    p.q_sb = q_strides.b; p.q_sl = q_strides.l; p.q_sh = q_strides.h;
    p.k_sb = kv_strides.b; p.k_sl = kv_strides.l; p.k_sh = kv_strides.h;
    p.B = batch; p.L = q_start + q_len; p.Lq = q_len; p.q_start = q_start;
    p.T = (q_len + kTile - 1) / kTile; p.fill_invalid = fill_invalid;
    return check_hip(launch_prefill_aggregate(p, static_cast<hipStream_t>(stream)),
                     "prefill_aggregate_range");
}
}  // namespace
extern "C" {

int kascade_prefill_aggregate_range_call(const kascade_half* Q, const kascade_half* K,
                                         const float* log_sum, kascade_half* aggregate_scores,
                                         int batch, int q_start, int q_len,
                                         kascade_strides q_strides, kascade_strides kv_strides,
                                         int fill_invalid, void* stream) {
    return prefill_aggregate_range_impl(kRefShape, Q, K, log_sum, aggregate_scores, batch, q_start, q_len, q_strides, kv_strides, fill_invalid, stream);
}

int kascade_prefill_aggregate_range_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K,
                                         const float* log_sum, kascade_half* aggregate_scores,
                                         int batch, int q_start, int q_len,
                                         kascade_strides q_strides, kascade_strides kv_strides,
                                         int fill_invalid, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return prefill_aggregate_range_impl(sh, Q, K, log_sum, aggregate_scores, batch, q_start, q_len, q_strides, kv_strides, fill_invalid, stream);
}

}  // extern "C"
namespace {
int prefill_reuse_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                               const int32_t* topk_indices, const int32_t* head_mapping,
                               float topk_percent, kascade_half* Output, int batch, int seq_len,
                               int max_topk_num, int rolling, kascade_strides q_strides,
                               kascade_strides kv_strides, float* log_sum, void* stream) {
    REQUIRE(Q && K && V && topk_indices && head_mapping && Output,
            "prefill_reuse: null pointer argument");
    REQUIRE(batch > 0 && seq_len > 0 && batch <= 65535, "prefill_reuse: bad batch/seq_len");
    REQUIRE(max_topk_num > 0, "prefill_reuse: max_topk_num must be > 0");
    REQUIRE(!rolling || topk_percent > 0.f, "prefill_reuse: rolling needs topk_percent > 0");
    REQUIRE(aligned16(Q) && aligned16(K) && aligned16(V) && aligned16(Output),
            "prefill_reuse: tensors must be 16-byte aligned");
    if (check_strides(q_strides, "Q") || check_strides(kv_strides, "K/V")) return -1;
    PrefillParams p{};
    p.G = sh.G; p.head_dim = sh.D; p.elem = sh.elem; p.gs = sh.gs;
    p.Q = H(Q); p.K = H(K); p.V = H(V); p.idx = topk_indices; p.head_map = head_mapping;
    p.O = H(Output); p.log_sum = log_sum;
    p.q_sb = q_strides.b; p.q_sl = q_strides.l; p.q_sh = q_strides.h;
    p.k_sb = kv_strides.b; p.k_sl = kv_strides.l; p.k_sh = kv_strides.h;
    p.B = batch; p.L = seq_len; p.Lq = seq_len; p.T = (seq_len + kTile - 1) / kTile;
    p.max_topk = max_topk_num; p.rolling = rolling; p.topk_percent = topk_percent;
    return check_hip(launch_prefill_attn(p, true, true, 1, static_cast<hipStream_t>(stream)),
                     "prefill_reuse");
}
}  // namespace
extern "C" {

int kascade_prefill_reuse_call(const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                               const int32_t* topk_indices, const int32_t* head_mapping,
                               float topk_percent, kascade_half* Output, int batch, int seq_len,
                               int max_topk_num, int rolling, kascade_strides q_strides,
                               kascade_strides kv_strides, float* log_sum, void* stream) {
    return prefill_reuse_impl(kRefShape, Q, K, V, topk_indices, head_mapping, topk_percent, Output, batch, seq_len, max_topk_num, rolling, q_strides, kv_strides, log_sum, stream);
}

int kascade_prefill_reuse_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K, const kascade_half* V,
                               const int32_t* topk_indices, const int32_t* head_mapping,
                               float topk_percent, kascade_half* Output, int batch, int seq_len,
                               int max_topk_num, int rolling, kascade_strides q_strides,
                               kascade_strides kv_strides, float* log_sum, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return prefill_reuse_impl(sh, Q, K, V, topk_indices, head_mapping, topk_percent, Output, batch, seq_len, max_topk_num, rolling, q_strides, kv_strides, log_sum, stream);
}

}  // extern "C"
namespace {
int paged_kv_append_impl(const Shape& sh, kascade_half* K_pages, kascade_half* V_pages,
                                 const kascade_half* k_new, const kascade_half* v_new,
                                 const int32_t* start_pos, const int32_t* block_table, int batch,
                                 int n_new, int max_pages, int page_size,
                                 kascade_strides new_strides, const int32_t* n_new_rows, void* stream) {
    REQUIRE(K_pages && V_pages && k_new && v_new && start_pos && block_table,
            "paged_kv_append: null pointer argument");
    REQUIRE(batch > 0 && n_new >= 0, "paged_kv_append: bad batch/n_new");
    int shift;
    if (check_paging(block_table, max_pages, page_size, &shift)) return -1;
    REQUIRE(new_strides.b % 8 == 0 && new_strides.l % 8 == 0 && new_strides.h % 8 == 0,
            "paged_kv_append: strides must be multiples of 8 elements");
    REQUIRE(aligned16(K_pages) && aligned16(V_pages) && aligned16(k_new) && aligned16(v_new),
            "paged_kv_append: tensors must be 16-byte aligned");
    return check_hip(launch_paged_kv_append(H(K_pages), H(V_pages), H(k_new), H(v_new), start_pos,
                                            block_table, batch, n_new, n_new_rows, max_pages, shift,
                                            new_strides.b, new_strides.l, new_strides.h, sh.G, sh.D,
                                            static_cast<hipStream_t>(stream)),
                     "paged_kv_append");
}
}  // namespace
extern "C" {

int kascade_paged_kv_append_call(kascade_half* K_pages, kascade_half* V_pages,
                                 const kascade_half* k_new, const kascade_half* v_new,
                                 const int32_t* start_pos, const int32_t* block_table, int batch,
                                 int n_new, int max_pages, int page_size,
                                 kascade_strides new_strides, const int32_t* n_new_rows, void* stream) {
    return paged_kv_append_impl(kRefShape, K_pages, V_pages, k_new, v_new, start_pos, block_table, batch, n_new, max_pages, page_size, new_strides, n_new_rows, stream);
}

int kascade_paged_kv_append_shaped_call(const kascade_shape* shape, kascade_half* K_pages, kascade_half* V_pages,
                                 const kascade_half* k_new, const kascade_half* v_new,
                                 const int32_t* start_pos, const int32_t* block_table, int batch,
                                 int n_new, int max_pages, int page_size,
                                 kascade_strides new_strides, const int32_t* n_new_rows, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return paged_kv_append_impl(sh, K_pages, V_pages, k_new, v_new, start_pos, block_table, batch, n_new, max_pages, page_size, new_strides, n_new_rows, stream);
}

}  // extern "C"
namespace {
int rope_append_impl(const Shape& sh, const kascade_half* q_in, const kascade_strides* q_strides,
                                   const kascade_half* k_in, const kascade_half* v_in,
                                   const kascade_strides* kv_strides, const float* cos_sin,
                                   int max_pos, const kascade_half* q_norm_weight,
                                   const kascade_half* k_norm_weight, float norm_eps,
                                   const int32_t* start_pos, int pos_offset, kascade_half* q_out,
                                   kascade_half* K_pages, kascade_half* V_pages,
                                   const int32_t* block_table, int max_pages, int page_size,
                                   int batch, int n_new, void* stream) {
    REQUIRE(q_in && k_in && v_in && cos_sin && start_pos && q_out && K_pages && V_pages && block_table,
            "rope_append: null pointer argument");
    REQUIRE(batch > 0 && n_new >= 0 && max_pos > 0, "rope_append: bad batch/n_new/max_pos");
    REQUIRE((long long)batch * n_new < (1LL << 31), "rope_append: too many tokens for one launch");
    REQUIRE(norm_eps >= 0.f, "rope_append: norm_eps must not be negative");
    int shift;
    if (check_paging(block_table, max_pages, page_size, &shift)) return -1;
    RopeAppendParams p{};
    const kascade_strides qs = q_strides ? *q_strides
        : kascade_strides{(long long)n_new * sh.H() * sh.D, (long long)sh.H() * sh.D, sh.D};
    const kascade_strides ks = kv_strides ? *kv_strides
        : kascade_strides{(long long)n_new * sh.G * sh.D, (long long)sh.G * sh.D, sh.D};
    if (check_strides(qs, "q_in") || check_strides(ks, "k_in/v_in")) return -1;
    REQUIRE(aligned16(q_in) && aligned16(k_in) && aligned16(v_in) && aligned16(q_out) &&
                aligned16(K_pages) && aligned16(V_pages) && aligned16(cos_sin) &&
                aligned16(q_norm_weight) && aligned16(k_norm_weight),
            "rope_append: tensors must be 16-byte aligned");
    p.q_in = E(q_in); p.k_in = E(k_in); p.v_in = E(v_in);
    p.cos_sin = cos_sin; p.q_weight = E(q_norm_weight); p.k_weight = E(k_norm_weight);
    p.start_pos = start_pos; p.q_out = E(q_out); p.Kp = E(K_pages); p.Vp = E(V_pages);
    p.block_table = block_table;
    p.q_sb = qs.b; p.q_sl = qs.l; p.q_sh = qs.h;
    p.kv_sb = ks.b; p.kv_sl = ks.l; p.kv_sh = ks.h;
    p.eps = norm_eps; p.pos_offset = pos_offset; p.batch = batch; p.n_new = n_new;
    p.max_pages = max_pages; p.page_shift = shift; p.max_pos = max_pos;
    p.G = sh.G; p.head_dim = sh.D; p.elem = sh.elem; p.gs = sh.gs;
    return check_hip(launch_rope_append(p, static_cast<hipStream_t>(stream)), "rope_append");
}
}  // namespace
extern "C" {

int kascade_rope_append_paged_call(const kascade_half* q_in, const kascade_strides* q_strides,
                                   const kascade_half* k_in, const kascade_half* v_in,
                                   const kascade_strides* kv_strides, const float* cos_sin,
                                   int max_pos, const kascade_half* q_norm_weight,
                                   const kascade_half* k_norm_weight, float norm_eps,
                                   const int32_t* start_pos, int pos_offset, kascade_half* q_out,
                                   kascade_half* K_pages, kascade_half* V_pages,
                                   const int32_t* block_table, int max_pages, int page_size,
                                   int batch, int n_new, void* stream) {
    return rope_append_impl(kRefShape, q_in, q_strides, k_in, v_in, kv_strides, cos_sin, max_pos, q_norm_weight, k_norm_weight, norm_eps, start_pos, pos_offset, q_out, K_pages, V_pages, block_table, max_pages, page_size, batch, n_new, stream);
}

int kascade_rope_append_paged_shaped_call(const kascade_shape* shape, const kascade_half* q_in, const kascade_strides* q_strides,
                                   const kascade_half* k_in, const kascade_half* v_in,
                                   const kascade_strides* kv_strides, const float* cos_sin,
                                   int max_pos, const kascade_half* q_norm_weight,
                                   const kascade_half* k_norm_weight, float norm_eps,
                                   const int32_t* start_pos, int pos_offset, kascade_half* q_out,
                                   kascade_half* K_pages, kascade_half* V_pages,
                                   const int32_t* block_table, int max_pages, int page_size,
                                   int batch, int n_new, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return rope_append_impl(sh, q_in, q_strides, k_in, v_in, kv_strides, cos_sin, max_pos, q_norm_weight, k_norm_weight, norm_eps, start_pos, pos_offset, q_out, K_pages, V_pages, block_table, max_pages, page_size, batch, n_new, stream);
}

int kascade_decode_budgets_shaped_call(const kascade_shape* shape, int32_t* cache_seqlens, int advance,
                                       float topk_percent, int batch, int32_t* valid_len_rows,
                                       int32_t* n_sel_rows, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    REQUIRE(cache_seqlens, "decode_budgets: null pointer argument");
    REQUIRE(batch > 0 && batch <= 65535, "decode_budgets: bad batch");
    REQUIRE(topk_percent >= 0.f && topk_percent <= 100.f, "decode_budgets: topk_percent out of range");
    return check_hip(launch_decode_budgets(cache_seqlens, advance, topk_percent, batch, sh.G, valid_len_rows,
                                           n_sel_rows, static_cast<hipStream_t>(stream)),
                     "decode_budgets");
}

int kascade_decode_budgets_call(int32_t* cache_seqlens, int advance, float topk_percent, int batch,
                                int32_t* valid_len_rows, int32_t* n_sel_rows, void* stream) {
    const kascade_shape ref{kRefShape.G, kRefShape.D, KASCADE_F16, kRefShape.gs};
    return kascade_decode_budgets_shaped_call(&ref, cache_seqlens, advance, topk_percent, batch,
                                              valid_len_rows, n_sel_rows, stream);
}

// ---- chunked prefill over the paged cache ----

}  // extern "C"
namespace {
int chunk_params(PrefillParams& p, const Shape& sh, const kascade_half* Q, int batch,
                        int q_start, int q_len, kascade_strides q_strides,
                        const int32_t* block_table, int max_pages, int page_size, int num_pages,
                        const int32_t* q_start_rows, const int32_t* q_len_rows) {
    REQUIRE(block_table, "prefill_chunk: block_table is required");
    REQUIRE(batch > 0 && batch <= 65535 && q_len > 0, "prefill_chunk: bad batch/q_len");
    REQUIRE(q_start >= 0 && q_start % kTile == 0, "prefill_chunk: q_start must be a multiple of 32");
    REQUIRE(aligned16(Q), "prefill_chunk: Q must be 16-byte aligned");
    if (check_strides(q_strides, "Q")) return -1;
    int shift;
    if (check_paging(block_table, max_pages, page_size, &shift)) return -1;
    REQUIRE(page_size >= 4, "prefill_chunk: page_size must be at least 4");
    REQUIRE(num_pages > 0 && (long long)num_pages * page_size < (1LL << 31),
            "prefill_chunk: num_pages out of range");
    REQUIRE((long long)max_pages * page_size >= (long long)q_start + q_len,
            "prefill_chunk: block table shorter than q_start + q_len");
    p.G = sh.G; p.head_dim = sh.D; p.elem = sh.elem; p.gs = sh.gs;
    p.Q = E(Q);
    p.q_sb = q_strides.b; p.q_sl = q_strides.l; p.q_sh = q_strides.h;
    p.B = batch; p.L = q_start + q_len; p.Lq = q_len; p.q_start = q_start;
    p.T = (q_len + kTile - 1) / kTile;
    p.block_table = block_table; p.max_pages = max_pages; p.page_shift = shift;
    p.num_pages = num_pages;
    REQUIRE(q_start_rows || !q_len_rows, "prefill_chunk: q_len_rows comes with q_start_rows");
    p.q_start_rows = q_start_rows; p.q_len_rows = q_len_rows;
    return 0;
}

int prefill_chunk_dense_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K_pages,
                                     const kascade_half* V_pages, float* log_sum,
                                     kascade_half* Output, int batch, int q_start, int q_len,
                                     kascade_strides q_strides, const int32_t* block_table,
                                     int max_pages, int page_size, int num_pages, int with_output, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows,
                                     void* stream) {
    REQUIRE(Q && K_pages, "prefill_chunk_dense: null pointer argument");
    REQUIRE(!with_output || (V_pages && Output), "prefill_chunk_dense: with_output needs V and Output");
    REQUIRE(with_output || log_sum, "prefill_chunk_dense: nothing to compute (no Output, no log_sum)");
    REQUIRE(aligned16(K_pages) && (!with_output || (aligned16(V_pages) && aligned16(Output))),
            "prefill_chunk_dense: tensors must be 16-byte aligned");
    PrefillParams p{};
    if (chunk_params(p, sh, Q, batch, q_start, q_len, q_strides, block_table, max_pages,
                     page_size, num_pages, q_start_rows, q_len_rows))
        return -1;
    p.K = E(K_pages); p.V = with_output ? E(V_pages) : E(K_pages);
    p.log_sum = log_sum; p.O = E(Output);
    return check_hip(launch_prefill_attn(p, false, with_output != 0, 1,
                                         static_cast<hipStream_t>(stream)), "prefill_chunk_dense");
}

int prefill_chunk_aggregate_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K_pages,
                                         const float* log_sum, kascade_half* aggregate_scores,
                                         int batch, int q_start, int q_len,
                                         kascade_strides q_strides, const int32_t* block_table,
                                         int max_pages, int page_size, int num_pages,
                                         int fill_invalid, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows, void* stream) {
    REQUIRE(Q && K_pages && log_sum && aggregate_scores,
            "prefill_chunk_aggregate: null pointer argument");
    REQUIRE(aligned16(K_pages), "prefill_chunk_aggregate: K must be 16-byte aligned");
    PrefillParams p{};
    if (chunk_params(p, sh, Q, batch, q_start, q_len, q_strides, block_table, max_pages,
                     page_size, num_pages, q_start_rows, q_len_rows))
        return -1;
    p.K = E(K_pages); p.V = E(K_pages); p.log_sum_in = log_sum; p.agg = H(aggregate_scores);
    p.fill_invalid = fill_invalid;
    return check_hip(launch_prefill_aggregate(p, static_cast<hipStream_t>(stream)),
                     "prefill_chunk_aggregate");
}

int prefill_chunk_reuse_impl(const Shape& sh, const kascade_half* Q, const kascade_half* K_pages,
                                     const kascade_half* V_pages, const int32_t* physical_rows,
                                     const int32_t* head_mapping, float topk_percent,
                                     kascade_half* Output, int batch, int q_start, int q_len,
                                     int max_topk_num, int rolling, kascade_strides q_strides,
                                     const int32_t* block_table, int max_pages, int page_size,
                                     int num_pages, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows, float* log_sum, void* stream) {
    REQUIRE(Q && K_pages && V_pages && physical_rows && head_mapping && Output,
            "prefill_chunk_reuse: null pointer argument");
    REQUIRE(max_topk_num > 0, "prefill_chunk_reuse: max_topk_num must be > 0");
    REQUIRE(!rolling || topk_percent > 0.f, "prefill_chunk_reuse: rolling needs topk_percent > 0");
    REQUIRE(aligned16(K_pages) && aligned16(V_pages) && aligned16(Output),
            "prefill_chunk_reuse: tensors must be 16-byte aligned");
    PrefillParams p{};
    if (chunk_params(p, sh, Q, batch, q_start, q_len, q_strides, block_table, max_pages,
                     page_size, num_pages, q_start_rows, q_len_rows))
        return -1;
    p.K = E(K_pages); p.V = E(V_pages); p.idx = physical_rows; p.head_map = head_mapping;
    p.O = E(Output); p.log_sum = log_sum;
    p.max_topk = max_topk_num; p.rolling = rolling; p.topk_percent = topk_percent;
    return check_hip(launch_prefill_attn(p, true, true, 1, static_cast<hipStream_t>(stream)),
                     "prefill_chunk_reuse");
}
}  // namespace
extern "C" {

int kascade_prefill_chunk_dense_call(const kascade_half* Q, const kascade_half* K_pages,
                                     const kascade_half* V_pages, float* log_sum,
                                     kascade_half* Output, int batch, int q_start, int q_len,
                                     kascade_strides q_strides, const int32_t* block_table,
                                     int max_pages, int page_size, int num_pages, int with_output, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows,
                                     void* stream) {
    return prefill_chunk_dense_impl(kRefShape, Q, K_pages, V_pages, log_sum, Output, batch, q_start, q_len, q_strides, block_table, max_pages, page_size, num_pages, with_output, q_start_rows, q_len_rows, stream);
}

int kascade_prefill_chunk_dense_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K_pages,
                                     const kascade_half* V_pages, float* log_sum,
                                     kascade_half* Output, int batch, int q_start, int q_len,
                                     kascade_strides q_strides, const int32_t* block_table,
                                     int max_pages, int page_size, int num_pages, int with_output, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows,
                                     void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return prefill_chunk_dense_impl(sh, Q, K_pages, V_pages, log_sum, Output, batch, q_start, q_len, q_strides, block_table, max_pages, page_size, num_pages, with_output, q_start_rows, q_len_rows, stream);
}

int kascade_prefill_chunk_aggregate_call(const kascade_half* Q, const kascade_half* K_pages,
                                         const float* log_sum, kascade_half* aggregate_scores,
                                         int batch, int q_start, int q_len,
                                         kascade_strides q_strides, const int32_t* block_table,
                                         int max_pages, int page_size, int num_pages,
                                         int fill_invalid, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows, void* stream) {
    return prefill_chunk_aggregate_impl(kRefShape, Q, K_pages, log_sum, aggregate_scores, batch, q_start, q_len, q_strides, block_table, max_pages, page_size, num_pages, fill_invalid, q_start_rows, q_len_rows, stream);
}

int kascade_prefill_chunk_aggregate_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K_pages,
                                         const float* log_sum, kascade_half* aggregate_scores,
                                         int batch, int q_start, int q_len,
                                         kascade_strides q_strides, const int32_t* block_table,
                                         int max_pages, int page_size, int num_pages,
                                         int fill_invalid, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return prefill_chunk_aggregate_impl(sh, Q, K_pages, log_sum, aggregate_scores, batch, q_start, q_len, q_strides, block_table, max_pages, page_size, num_pages, fill_invalid, q_start_rows, q_len_rows, stream);
}

int kascade_prefill_chunk_reuse_call(const kascade_half* Q, const kascade_half* K_pages,
                                     const kascade_half* V_pages, const int32_t* physical_rows,
                                     const int32_t* head_mapping, float topk_percent,
                                     kascade_half* Output, int batch, int q_start, int q_len,
                                     int max_topk_num, int rolling, kascade_strides q_strides,
                                     const int32_t* block_table, int max_pages, int page_size,
                                     int num_pages, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows, float* log_sum, void* stream) {
    return prefill_chunk_reuse_impl(kRefShape, Q, K_pages, V_pages, physical_rows, head_mapping, topk_percent, Output, batch, q_start, q_len, max_topk_num, rolling, q_strides, block_table, max_pages, page_size, num_pages, q_start_rows, q_len_rows, log_sum, stream);
}

int kascade_prefill_chunk_reuse_shaped_call(const kascade_shape* shape, const kascade_half* Q, const kascade_half* K_pages,
                                     const kascade_half* V_pages, const int32_t* physical_rows,
                                     const int32_t* head_mapping, float topk_percent,
                                     kascade_half* Output, int batch, int q_start, int q_len,
                                     int max_topk_num, int rolling, kascade_strides q_strides,
                                     const int32_t* block_table, int max_pages, int page_size,
                                     int num_pages, const int32_t* q_start_rows,
                                     const int32_t* q_len_rows, float* log_sum, void* stream) {
    Shape sh;
    if (get_shape(shape, &sh)) return -1;
    return prefill_chunk_reuse_impl(sh, Q, K_pages, V_pages, physical_rows, head_mapping, topk_percent, Output, batch, q_start, q_len, max_topk_num, rolling, q_strides, block_table, max_pages, page_size, num_pages, q_start_rows, q_len_rows, log_sum, stream);
}

int kascade_translate_indices_call(const int32_t* token_idx, int32_t* physical_rows,
                                   const int32_t* block_table, int batch, int64_t per_sequence,
                                   int max_pages, int page_size, int kv_len, void* stream) {
    REQUIRE(token_idx && physical_rows && block_table, "translate_indices: null pointer argument");
    REQUIRE(batch > 0 && batch <= 65535 && per_sequence >= 0 && kv_len > 0,
            "translate_indices: bad batch/per_sequence/kv_len");
    int shift;
    if (check_paging(block_table, max_pages, page_size, &shift)) return -1;
    REQUIRE((long long)max_pages * page_size >= kv_len,
            "translate_indices: block table shorter than kv_len");
    return check_hip(launch_translate_indices(token_idx, physical_rows, block_table, batch,
                                              per_sequence, max_pages, shift, kv_len,
                                              static_cast<hipStream_t>(stream)),
                     "translate_indices");
}

// ---- the reference's argument lists, verbatim ----

int kascade_ref_decode_reuse_call(kascade_half* Q, kascade_half* K, kascade_half* V,
                                  int* topk_indices, int* head_mapping, float* glse,
                                  float* Output_partial, kascade_half* Output, int batch,
                                  int kv_seqlen, int topk, void* stream) {
    return kascade_decode_reuse_call(Q, K, V, topk_indices, head_mapping, glse, Output_partial, Output,
                                     batch, kv_seqlen, topk, kRefNumSplit, nullptr, stream);
}

int kascade_ref_decode_reuse_kvcache_call(kascade_half* Q, kascade_half* K, kascade_half* V,
                                          int* cache_seqlens, int* topk_indices, int* head_mapping,
                                          float topk_percent, float* glse, float* Output_partial,
                                          kascade_half* Output, int batch, int max_cache_seqlen,
                                          int topk, void* stream) {
    return kascade_decode_reuse_paged_call(Q, K, V, cache_seqlens, topk_indices, head_mapping,
                                           topk_percent, glse, Output_partial, Output, batch,
                                           max_cache_seqlen, topk, kRefNumSplit, nullptr, 0, 1, nullptr,
                                           nullptr, nullptr, nullptr, nullptr, stream);
}

int kascade_ref_prefill_aggregate_call(kascade_half* Q, kascade_half* K, float* log_sum,
                                       kascade_half* aggregate_scores, int batch, int seq_len,
                                       void* stream) {
    return kascade_prefill_aggregate_call(Q, K, log_sum, aggregate_scores, batch, seq_len,
                                          contiguous_strides(seq_len, kHeads), contiguous_strides(seq_len, kGroups),
                                          0, stream);
}

int kascade_ref_prefill_reuse_rolling_call(kascade_half* Q, kascade_half* K, kascade_half* V,
                                           int* topk_indices, int* head_mapping,
                                           float topk_percent, kascade_half* Output, int batch,
                                           int seq_len, int max_topk_num, void* stream) {
    return kascade_prefill_reuse_call(Q, K, V, topk_indices, head_mapping, topk_percent, Output, batch,
                                      seq_len, max_topk_num, 1, contiguous_strides(seq_len, kHeads),
                                      contiguous_strides(seq_len, kGroups), nullptr, stream);
}

int kascade_ref_prefill_reuse_call(kascade_half* Q, kascade_half* K, kascade_half* V,
                                   int* topk_indices, int* head_mapping, float topk_percent,
                                   kascade_half* Output, int batch, int seq_len, int topk_num,
                                   void* stream) {
    return kascade_prefill_reuse_call(Q, K, V, topk_indices, head_mapping, topk_percent, Output, batch,
                                      seq_len, topk_num, 0, contiguous_strides(seq_len, kHeads),
                                      contiguous_strides(seq_len, kGroups), nullptr, stream);
}

// ---- diagnostics ----

int kascade_diag_stream_read_call(const void* src, int64_t bytes, void* sink, void* stream) {
    REQUIRE(src && sink, "diag_stream_read: null pointer argument");
    REQUIRE(bytes >= 16 && aligned16(src) && aligned16(sink), "diag_stream_read: need >= 16 bytes, 16-byte aligned");
    const int cus = g_cu_count > 0 ? g_cu_count : 256;
    return check_hip(launch_diag_stream_read(src, bytes, sink, cus * 32, static_cast<hipStream_t>(stream)),
                     "diag_stream_read");
}

int kascade_diag_gather_rows_call(const void* rows_a, const void* rows_b, const int32_t* row_ids,
                                  int64_t n_rows, int64_t row_stride_bytes, void* sink, void* stream) {
    REQUIRE(rows_a && row_ids && sink, "diag_gather_rows: null pointer argument");
    REQUIRE(n_rows > 0 && row_stride_bytes >= 256 && row_stride_bytes % 16 == 0,
            "diag_gather_rows: n_rows > 0 and a row stride of at least 256 bytes, multiple of 16, required");
    REQUIRE(aligned16(rows_a) && (!rows_b || aligned16(rows_b)) && aligned16(sink),
            "diag_gather_rows: arrays must be 16-byte aligned");
    return check_hip(launch_diag_gather_rows(rows_a, rows_b, row_ids, n_rows, 128, row_stride_bytes, sink,
                                             static_cast<hipStream_t>(stream)), "diag_gather_rows");
}

}  // extern "C"
