// stub_kernels.cpp -- a host-only stand-in for libaixhip_kernels.so (include/aixhip_kernels.h) for the sanitizer
// builds of the device's host code (the counterpart of the reference's ASan / TSan configurations,
// CMakeLists.txt:25, 47-53).  Memory comes from the host heap under a settable budget, events complete after a
// settable number of queries, every compute entry point only counts its call: what runs under the sanitizers is
// DeviceHIP's own bookkeeping -- block table, buckets, limbo, cooling lists, the planner and the source generator.
// TEST INFRASTRUCTURE ONLY; never linked into the product.
#include "aixhip_kernels.h"

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <string>

struct aixk_module { std::string entry; };
struct aixk_ctx {
    size_t budget{SIZE_MAX}, held{0}; int event_delay{0}; uint64_t launches{0}, allocs{0}, frees{0}, syncs{0}, hits{0}, misses{0};
    std::string log;                                       // what was launched, in order: "name;name;..." (generated kernels by their entry)
    std::deque<aixk_module> modules;
};
struct aixk_event { int countdown{0}; bool recorded{false}; };

static thread_local char g_error[256] = "";
static std::atomic<long long> g_held_everywhere{0};        // bytes handed out and not yet returned, over all contexts
static std::atomic<int> g_fail_matmuls{0};                 // the next n matmul calls report AIXK_ENOMEM

extern "C" {

// test controls (not part of the product ABI)
void stub_set_budget(aixk_ctx* c, size_t bytes) { c->budget = bytes; }
void stub_set_event_delay(aixk_ctx* c, int queries) { c->event_delay = queries; }
size_t stub_held(aixk_ctx* c) { return c->held; }
uint64_t stub_launches(aixk_ctx* c) { return c->launches; }
uint64_t stub_allocs(aixk_ctx* c) { return c->allocs; }
uint64_t stub_frees(aixk_ctx* c) { return c->frees; }
uint64_t stub_syncs(aixk_ctx* c) { return c->syncs; }
long long stub_held_everywhere(void) { return g_held_everywhere.load(); }
void stub_fail_next_matmuls(int n) { g_fail_matmuls = n; }
const char* stub_log(aixk_ctx* c) { return c->log.c_str(); }
void stub_log_clear(aixk_ctx* c) { c->log.clear(); }

const char* aixk_last_error(void) { return g_error; }
size_t aixk_dtype_size(int dtype) { static const size_t sz[9] = {8, 4, 2, 2, 8, 4, 2, 1, 1}; return dtype >= 0 && dtype < 9 ? sz[dtype] : 0; }
int32_t aixk_create(int, aixk_ctx** out) { *out = new aixk_ctx(); return AIXK_OK; }
int32_t aixk_destroy(aixk_ctx* c) { delete c; return AIXK_OK; }
int32_t aixk_info(aixk_ctx*, aixk_device_info* out)
{
    std::memset(out, 0, sizeof(*out));
    std::snprintf(out->name, sizeof(out->name), "stub");
    out->compute_units = 256; out->large_bar = 1; out->wavefront = 64; out->total_mem = 1ull << 30;
    return AIXK_OK;
}
int32_t aixk_alloc(aixk_ctx* c, size_t bytes, int, void** out)
{
    if (c->held + bytes > c->budget) { std::snprintf(g_error, sizeof(g_error), "stub: out of memory (%zu held, %zu asked)", c->held, bytes); return AIXK_ENOMEM; }
    void* p = nullptr;
    if (posix_memalign(&p, 256, bytes + sizeof(size_t) * 32) != 0) return AIXK_ENOMEM;
    *(size_t*)p = bytes;                                   // size header in front of the 256-byte aligned block
    c->held += bytes; ++c->allocs; g_held_everywhere += (long long)bytes;
    *out = (char*)p + 256;
    return AIXK_OK;
}
int32_t aixk_free(aixk_ctx* c, void* ptr, int)
{
    if (!ptr) return AIXK_OK;
    void* base = (char*)ptr - 256;
    c->held -= *(size_t*)base; ++c->frees; g_held_everywhere -= (long long)*(size_t*)base;
    std::free(base);
    return AIXK_OK;
}
int32_t aixk_copy_in(aixk_ctx* c, void* d, const void* s, size_t n) { ++c->launches; std::memcpy(d, s, n); return AIXK_OK; }
int32_t aixk_copy_out(aixk_ctx* c, void* d, const void* s, size_t n) { ++c->launches; std::memcpy(d, s, n); return AIXK_OK; }
int32_t aixk_copy_dev(aixk_ctx* c, void* d, const void* s, size_t n) { ++c->launches; std::memmove(d, s, n); return AIXK_OK; }
int32_t aixk_zero(aixk_ctx* c, void* d, size_t n) { ++c->launches; std::memset(d, 0, n); return AIXK_OK; }
int32_t aixk_sync(aixk_ctx* c) { ++c->syncs; return AIXK_OK; }

#define STUB_OP(name, ...) int32_t name(aixk_ctx* c, __VA_ARGS__) { ++c->launches; c->log += #name ";"; return AIXK_OK; }
STUB_OP(aixk_binary, int, const aixhip_tensor*, const aixhip_tensor*, const aixhip_tensor*)
STUB_OP(aixk_unary, int, const aixhip_tensor*, const aixhip_tensor*)
STUB_OP(aixk_fill, const void*, int, const aixhip_tensor*)
STUB_OP(aixk_fill_min, const aixhip_tensor*)
STUB_OP(aixk_cast, const void*, int, void*, int, uint64_t)
STUB_OP(aixk_contiguous, const aixhip_tensor*, const aixhip_tensor*)
STUB_OP(aixk_transpose, const aixhip_tensor*, const aixhip_tensor*, uint64_t, uint64_t)
STUB_OP(aixk_slice_set, const aixhip_tensor*, const aixhip_tensor*, uint64_t, uint64_t, uint64_t, uint64_t)
STUB_OP(aixk_slice_set_many, const aixk_slice_item*, uint32_t)
STUB_OP(aixk_slice_set_init, const aixhip_tensor*, const aixhip_tensor*, uint64_t, uint64_t, uint64_t, uint64_t, uint64_t)
STUB_OP(aixk_tri, int, const aixhip_tensor*, const aixhip_tensor*, int64_t)
STUB_OP(aixk_index_select, const aixhip_tensor*, const aixhip_tensor*, const aixhip_tensor*, uint64_t)
STUB_OP(aixk_index_add, const aixhip_tensor*, const aixhip_tensor*, const aixhip_tensor*, uint64_t)
STUB_OP(aixk_reduce_all, int, const aixhip_tensor*, const aixhip_tensor*)
STUB_OP(aixk_reduce_all_noalloc, int, const aixhip_tensor*, const aixhip_tensor*)
STUB_OP(aixk_reduce_to, int, const aixhip_tensor*, const aixhip_tensor*)
STUB_OP(aixk_reduce_to_init, int, const aixhip_tensor*, const aixhip_tensor*, uint64_t)
STUB_OP(aixk_argmax_to, int, const aixhip_tensor*, const aixhip_tensor*, uint64_t)
STUB_OP(aixk_argmax_onehot_many, const aixk_argmax_item*, uint32_t)
STUB_OP(aixk_sum_columns_many, const aixk_colsum_item*, uint32_t)
STUB_OP(aixk_sum_partials, const void*, uint64_t, const aixhip_tensor*, uint64_t)
STUB_OP(aixk_sum_partials_many, const aixk_partials_item*, uint32_t)
int32_t aixk_matmul(aixk_ctx* c, const aixhip_tensor*, const aixhip_tensor*, const aixhip_tensor*)
{
    if (g_fail_matmuls > 0) { --g_fail_matmuls; std::snprintf(g_error, sizeof(g_error), "stub: matmul workspace"); return AIXK_ENOMEM; }
    ++c->launches; c->log += "aixk_matmul;";
    return AIXK_OK;
}
STUB_OP(aixk_matmul_batched, const aixhip_tensor*, const aixhip_tensor*, const aixhip_tensor*)
int32_t aixk_matmul_grouped(aixk_ctx* c, const aixhip_tensor* a, const aixhip_tensor* b, const aixhip_tensor* out, uint32_t count)
{
    for (uint32_t i = 0; i < count; ++i) { const int32_t rc = aixk_matmul(c, a + i, b + i, out + i); if (rc != AIXK_OK) return rc; }
    return AIXK_OK;
}

int32_t aixk_rtc_get(aixk_ctx* c, const char*, const char*, const char* entry, aixk_module** out, int32_t* was_cached)
{
    ++c->misses;
    c->modules.push_back(aixk_module{entry ? entry : ""});
    *out = &c->modules.back();
    if (was_cached) *was_cached = 0;
    return AIXK_OK;
}
int32_t aixk_rtc_launch(aixk_ctx* c, aixk_module* m, uint32_t, uint32_t, const void*, size_t) { ++c->launches; c->log += m->entry + ";"; return AIXK_OK; }
STUB_OP(aixk_fill_many, const aixk_fill_item*, uint32_t)
int32_t aixk_rtc_launch_many(aixk_ctx* c, aixk_module* m, uint32_t, const void*, size_t, size_t, uint32_t) { ++c->launches; c->log += m->entry + "*;"; return AIXK_OK; }
const char* aixk_rtc_prelude(void) { return ""; }
// captures: the stub "graph" is the stretch of the launch log recorded between begin and end; a launch appends it again
struct aixk_graph { std::string log; uint64_t nodes{0}; };
static thread_local size_t g_capture_from = 0;
static thread_local uint64_t g_capture_launches = 0;
static thread_local bool g_capturing = false;
int32_t aixk_capture_begin(aixk_ctx* c) { if (g_capturing) return AIXK_EINVAL; g_capturing = true; g_capture_from = c->log.size(); g_capture_launches = c->launches; return AIXK_OK; }
int32_t aixk_capture_end(aixk_ctx* c, aixk_graph** out)
{
    if (!g_capturing) return AIXK_EINVAL;
    g_capturing = false;
    *out = new aixk_graph{c->log.substr(g_capture_from), c->launches - g_capture_launches};
    return AIXK_OK;
}
int32_t aixk_capture_abort(aixk_ctx*) { g_capturing = false; return AIXK_OK; }
int32_t aixk_graph_launch(aixk_ctx* c, aixk_graph* g) { c->launches += g->nodes; c->log += g->log; return AIXK_OK; }
int32_t aixk_graph_nodes(aixk_graph* g, uint64_t* n) { *n = g->nodes; return AIXK_OK; }
int32_t aixk_graph_destroy(aixk_ctx*, aixk_graph* g) { delete g; return AIXK_OK; }
int32_t aixk_rtc_stats(aixk_ctx* c, uint64_t* hits, uint64_t* misses) { *hits = c->hits; *misses = c->misses; return AIXK_OK; }

int32_t aixk_event_create(aixk_ctx*, aixk_event** out) { *out = new aixk_event(); return AIXK_OK; }
int32_t aixk_event_record(aixk_ctx* c, aixk_event* e) { e->recorded = true; e->countdown = c->event_delay; return AIXK_OK; }
int32_t aixk_event_query(aixk_ctx*, aixk_event* e, int32_t* done) { *done = e->recorded && e->countdown-- <= 0; return AIXK_OK; }
int32_t aixk_event_elapsed_ms(aixk_ctx*, aixk_event*, aixk_event*, float* ms) { *ms = 0.f; return AIXK_OK; }
int32_t aixk_event_destroy(aixk_ctx*, aixk_event* e) { delete e; return AIXK_OK; }

} // extern "C"
