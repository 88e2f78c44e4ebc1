// runtime.hip -- context, memory, ordering, timing and the hipRTC kernel cache.

#include "common.hpp"

#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <sys/stat.h>
#include <unistd.h>

#include <hip/hiprtc.h>

#include <vector>

namespace aixk {

static thread_local char g_error[1024] = "";

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

// The text of aix_device.h, embedded at build time (see the Makefile rule for prelude.inc).
static const char kPrelude[] = {
#include "prelude.inc"
    , 0};

namespace {
__global__ void zero_k(uint4* __restrict__ p, uint64_t n16, unsigned char* __restrict__ tail, unsigned ntail)
{
    const uint4 z = make_uint4(0, 0, 0, 0);
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * blockDim.x) p[i] = z;
    if (blockIdx.x == 0 && threadIdx.x < ntail) tail[threadIdx.x] = 0;
}
} // namespace

} // namespace aixk

using namespace aixk;

namespace aixk {
// The ring is used in two halves.  Moving on to a half records an event behind the work that used the other half and
// waits for the event that was recorded when this half was left the last time: by then every copy out of it and every
// kernel reading its device twin has finished.  The wait only ever blocks a host that is a whole half (hundreds of
// grouped launches) ahead of the GPU.
int table_slot(aixk_ctx* ctx, size_t bytes, void** host, const void** dev)
{
    bytes = (bytes + 255) & ~(size_t)255;
    if (ctx->capturing) {
        // the launch that reads this table will run again at every replay: the table gets memory of its own for as long
        // as the graph lives (the ring's slots are written over a few hundred launches later)
        void *d = nullptr, *h = nullptr;
        AIXK_HIP(hipMalloc(&d, bytes));
        if (hipHostMalloc(&h, bytes, hipHostMallocDefault) != hipSuccess) { (void)hipFree(d); return fail(AIXK_ENOMEM, "no pinned memory for a captured table of %zu bytes", bytes); }
        ctx->capturing->tables.emplace_back(d, h);
        *host = h; *dev = d;
        return AIXK_OK;
    }
    if (!ctx->table_host) {
        ctx->table_bytes = 1u << 20;
        AIXK_HIP(hipHostMalloc((void**)&ctx->table_host, ctx->table_bytes, hipHostMallocDefault));
        AIXK_HIP(hipMalloc((void**)&ctx->table_dev, ctx->table_bytes));
        AIXK_HIP(hipEventCreateWithFlags(&ctx->table_lap[0], hipEventDisableTiming));
        AIXK_HIP(hipEventCreateWithFlags(&ctx->table_lap[1], hipEventDisableTiming));
        AIXK_HIP(hipEventRecord(ctx->table_lap[0], ctx->stream));
        AIXK_HIP(hipEventRecord(ctx->table_lap[1], ctx->stream));
    }
    const size_t half = ctx->table_bytes / 2;
    if (bytes > half) return fail(AIXK_EINVAL, "table of %zu bytes exceeds the ring", bytes);
    if (ctx->table_used + bytes > half) {
        AIXK_HIP(hipEventRecord(ctx->table_lap[ctx->table_half], ctx->stream));      // behind everything that used this half
        ctx->table_half ^= 1;
        AIXK_HIP(hipEventSynchronize(ctx->table_lap[ctx->table_half]));              // the half we return to is idle
        ctx->table_used = 0;
    }
    const size_t at = (size_t)ctx->table_half * half + ctx->table_used;
    ctx->table_used += bytes;
    *host = ctx->table_host + at;
    *dev = ctx->table_dev + at;
    return AIXK_OK;
}

int table_upload(aixk_ctx* ctx, const void* host, const void* dev, size_t bytes)
{
    if (ctx->capturing) {
        // written now, on a stream of its own (the main stream only records), and complete before this call returns: the
        // captured launch finds it in place at every replay and no copy node enters the graph
        AIXK_HIP(hipMemcpyAsync(const_cast<void*>(dev), host, bytes, hipMemcpyHostToDevice, ctx->side));
        AIXK_HIP(hipStreamSynchronize(ctx->side));
        return AIXK_OK;
    }
    AIXK_HIP(hipMemcpyAsync(const_cast<void*>(dev), host, bytes, hipMemcpyHostToDevice, ctx->stream));
    return AIXK_OK;
}

size_t stream_store_min_bytes()
{
    static const size_t value = [] {
        const char* e = std::getenv("AIXHIP_STREAM_STORE_MIN_BYTES");
        return e && *e ? (size_t)std::strtoull(e, nullptr, 10) : (size_t)AIXK_STREAM_STORE_MIN_BYTES;
    }();
    return value;
}
} // namespace aixk

extern "C" {

const char* aixk_last_error(void) { return g_error; }

size_t aixk_dtype_size(int dtype)
{
    static const size_t sz[AIXK_DTYPE_COUNT] = {8, 4, 2, 2, 8, 4, 2, 1, 1};
    return (dtype >= 0 && dtype < AIXK_DTYPE_COUNT) ? sz[dtype] : 0;
}

int32_t aixk_create(int device_index, aixk_ctx** out)
{
    AIXK_REQUIRE(out != nullptr, "create: null out pointer");
    int count = 0;
    AIXK_HIP(hipGetDeviceCount(&count));
    if (count <= 0) return fail(AIXK_EHIP, "no HIP device is visible to this process");
    AIXK_REQUIRE(device_index >= 0 && device_index < count, "create: device index %d out of range (%d devices)", device_index, count);
    AIXK_HIP(hipSetDevice(device_index));
    aixk_ctx* ctx = new aixk_ctx();
    ctx->device = device_index;
    const int32_t rc = [ctx, device_index]() -> int32_t {
        AIXK_HIP(hipGetDeviceProperties(&ctx->prop, device_index));
        ctx->cus = ctx->prop.multiProcessorCount > 0 ? ctx->prop.multiProcessorCount : 256;
        AIXK_HIP(hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking));
        if (const char* dir = std::getenv("AIXHIP_KERNEL_CACHE_DIR"); dir && *dir) {
            ctx->rtc_disk_dir = dir;
            while (ctx->rtc_disk_dir.size() > 1 && ctx->rtc_disk_dir.back() == '/') ctx->rtc_disk_dir.pop_back();
            for (size_t at = 1; at <= ctx->rtc_disk_dir.size(); ++at)          // mkdir -p; an unusable directory only costs the cache
                if (at == ctx->rtc_disk_dir.size() || ctx->rtc_disk_dir[at] == '/') (void)mkdir(ctx->rtc_disk_dir.substr(0, at).c_str(), 0777);
        }
        ctx->scratch_bytes = 64u << 20;
        AIXK_HIP(hipMalloc(&ctx->scratch, ctx->scratch_bytes));
        AIXK_HIP(hipMalloc((void**)&ctx->counter, 256));
        AIXK_HIP(hipMemset(ctx->counter, 0, 256));
        return aixk::resolve_static_scratch(ctx);
    }();
    if (rc != AIXK_OK) {                              // nothing of a half-built context survives
        if (ctx->counter) (void)hipFree(ctx->counter);
        if (ctx->scratch) (void)hipFree(ctx->scratch);
        if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return rc;
    }
    *out = ctx;
    return AIXK_OK;
}

int32_t aixk_destroy(aixk_ctx* ctx)
{
    if (!ctx) return AIXK_OK;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    for (auto& kv : ctx->rtc) {
        if (kv.second->m.module) (void)hipModuleUnload(kv.second->m.module);
        delete kv.second;
    }
    if (ctx->table_host) {
        (void)hipHostFree(ctx->table_host);
        (void)hipFree(ctx->table_dev);
        (void)hipEventDestroy(ctx->table_lap[0]);
        (void)hipEventDestroy(ctx->table_lap[1]);
    }
    (void)hipFree(ctx->scratch);
    (void)hipFree(ctx->counter);
    for (void* ws : ctx->gemm_ws) if (ws) (void)hipFree(ws);
    if (ctx->capturing) (void)aixk_capture_abort(ctx);
    if (ctx->side) (void)hipStreamDestroy(ctx->side);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return AIXK_OK;
}

int32_t aixk_info(aixk_ctx* ctx, aixk_device_info* out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(out != nullptr, "info: null out pointer");
    std::memset(out, 0, sizeof(*out));
    std::snprintf(out->name, sizeof(out->name), "%s", ctx->prop.name);
    std::snprintf(out->arch, sizeof(out->arch), "%s", ctx->prop.gcnArchName);
    out->compute_units = ctx->prop.multiProcessorCount;
    out->clock_khz = ctx->prop.clockRate;
    out->large_bar = ctx->prop.isLargeBar;
    out->wavefront = ctx->prop.warpSize;
    out->total_mem = ctx->prop.totalGlobalMem;
    out->lds_per_block = ctx->prop.sharedMemPerBlock;
    return AIXK_OK;
}

int32_t aixk_alloc(aixk_ctx* ctx, size_t bytes, int kind, void** out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(out != nullptr, "alloc: null out pointer");
    const size_t padded = ((bytes ? bytes : 1) + 255) & ~(size_t)255;   // tail lanes of 16-byte kernels stay inside
    void* p = nullptr;
    hipError_t e;
    switch (kind) {
        case 0: e = hipMalloc(&p, padded); break;
        case 1:
            e = hipMallocManaged(&p, padded, hipMemAttachGlobal);
            if (e == hipSuccess) {
                (void)hipMemAdvise(p, padded, hipMemAdviseSetPreferredLocation, ctx->device);
                (void)hipMemAdvise(p, padded, hipMemAdviseSetCoarseGrain, ctx->device);
                (void)hipMemPrefetchAsync(p, padded, ctx->device, ctx->stream);
                (void)hipGetLastError();
            }
            break;
        case 2: e = hipHostMalloc(&p, padded, hipHostMallocDefault); break;
        default: return fail(AIXK_EINVAL, "alloc: unknown memory kind %d", kind);
    }
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(AIXK_ENOMEM, "alloc of %zu bytes (kind %d) failed: %s", padded, kind, hipGetErrorString(e));
    }
    *out = p;
    return AIXK_OK;
}

int32_t aixk_free(aixk_ctx* ctx, void* ptr, int kind)
{
    AIXK_TRY(set_device(ctx));
    if (!ptr) return AIXK_OK;
    if (kind == 2) AIXK_HIP(hipHostFree(ptr));
    else AIXK_HIP(hipFree(ptr));
    return AIXK_OK;
}

int32_t aixk_copy_in(aixk_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes)
{
    AIXK_TRY(set_device(ctx));
    if (bytes == 0) return AIXK_OK;
    AIXK_REQUIRE(dst_dev && src_host, "copy_in: null pointer");
    AIXK_REQUIRE(!ctx->capturing, "copy_in: no transfers from host memory inside a capture");
    // pageable source: the runtime stages it before returning, so the caller may reuse it
    AIXK_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    AIXK_HIP(hipStreamSynchronize(ctx->stream));
    return AIXK_OK;
}

int32_t aixk_copy_out(aixk_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes)
{
    AIXK_TRY(set_device(ctx));
    if (bytes == 0) return AIXK_OK;
    AIXK_REQUIRE(dst_host && src_dev, "copy_out: null pointer");
    AIXK_REQUIRE(!ctx->capturing, "copy_out: no transfers to host memory inside a capture");
    AIXK_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    AIXK_HIP(hipStreamSynchronize(ctx->stream));
    return AIXK_OK;
}

int32_t aixk_copy_dev(aixk_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes)
{
    AIXK_TRY(set_device(ctx));
    if (bytes == 0) return AIXK_OK;
    AIXK_REQUIRE(dst_dev && src_dev, "copy_dev: null pointer");
    AIXK_HIP(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, ctx->stream));
    return AIXK_OK;
}

int32_t aixk_zero(aixk_ctx* ctx, void* dst_dev, size_t bytes)
{
    AIXK_TRY(set_device(ctx));
    if (bytes == 0) return AIXK_OK;
    AIXK_REQUIRE(dst_dev != nullptr, "zero: null pointer");
    // A kernel rather than hipMemsetAsync, so that callers may capture this stream in a graph.
    unsigned char* p = (unsigned char*)dst_dev;
    const size_t head = ((uintptr_t)p & 15u) ? 16 - ((uintptr_t)p & 15u) : 0;
    if (head >= bytes) {
        hipLaunchKernelGGL(zero_k, dim3(1), dim3(kBlock), 0, ctx->stream, (uint4*)nullptr, (uint64_t)0, p, (unsigned)bytes);
    } else {
        if (head) hipLaunchKernelGGL(zero_k, dim3(1), dim3(kBlock), 0, ctx->stream, (uint4*)nullptr, (uint64_t)0, p, (unsigned)head);
        const size_t body = bytes - head, n16 = body / 16, ntail = body % 16;
        hipLaunchKernelGGL(zero_k, dim3(grid_for(n16 + 1, kBlock, (unsigned)ctx->cus * 16u)), dim3(kBlock), 0, ctx->stream,
                           (uint4*)(p + head), (uint64_t)n16, p + head + n16 * 16, (unsigned)ntail);
    }
    AIXK_HIP(hipGetLastError());
    return AIXK_OK;
}

int32_t aixk_sync(aixk_ctx* ctx)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(!ctx->capturing, "sync: nothing runs while the stream is being captured");
    AIXK_HIP(hipStreamSynchronize(ctx->stream));
    return AIXK_OK;
}

// ---- hipRTC -----------------------------------------------------------------------------------
const char* aixk_rtc_prelude(void) { return kPrelude; }

// Code objects on disk.  A generated kernel takes 30-150 ms to compile and a model's first step compiles dozens of them;
// with AIXHIP_KERNEL_CACHE_DIR set, each code object is also written to <dir>/<128-bit name>.aixk and a later process
// loads it instead of compiling.  The name is a hash of everything the code depends on: the device header, the source,
// the target, the compiler's options and the compiler's version.  A file is header + size + hash of the payload + payload,
// written under a temporary name and renamed, so a reader never sees half a file and a damaged one is ignored (the kernel
// is compiled and the file replaced).
namespace {

uint64_t fnv1a(const void* data, size_t n, uint64_t h)
{
    const unsigned char* p = (const unsigned char*)data;
    for (size_t i = 0; i < n; ++i) { h ^= p[i]; h *= 0x100000001b3ull; }
    return h;
}

const char kDiskMagic[8] = {'A', 'I', 'X', 'K', 'C', 'O', '0', '1'};

std::string disk_name(const aixk_ctx* ctx, const char* source, const char* arch, const char* const* opts, int nopts)
{
    int major = 0, minor = 0;
    (void)hiprtcVersion(&major, &minor);
    uint64_t h[2] = {0xcbf29ce484222325ull, 0x84222325cbf29ce4ull};
    for (uint64_t& x : h) {
        x = fnv1a(kPrelude, std::strlen(kPrelude), x);
        x = fnv1a(source, std::strlen(source) + 1, x);
        x = fnv1a(arch, std::strlen(arch) + 1, x);
        for (int i = 0; i < nopts; ++i) x = fnv1a(opts[i], std::strlen(opts[i]) + 1, x);
        x = fnv1a(&major, sizeof major, x);
        x = fnv1a(&minor, sizeof minor, x);
        x = fnv1a(&x, sizeof x, x);                      // the two lanes start apart and stay apart
    }
    char name[40];
    std::snprintf(name, sizeof name, "%016llx%016llx.aixk", (unsigned long long)h[0], (unsigned long long)h[1]);
    return ctx->rtc_disk_dir + "/" + name;
}

bool disk_load(const std::string& path, std::vector<char>& code)
{
    std::FILE* f = std::fopen(path.c_str(), "rb");
    if (!f) return false;
    char magic[8];
    uint64_t size = 0, hash = 0;
    bool ok = std::fread(magic, 1, 8, f) == 8 && std::memcmp(magic, kDiskMagic, 8) == 0 && std::fread(&size, 8, 1, f) == 1 &&
              std::fread(&hash, 8, 1, f) == 1 && size > 0 && size < (1ull << 30);
    if (ok) {
        code.resize(size);
        ok = std::fread(code.data(), 1, size, f) == size && std::fgetc(f) == EOF && fnv1a(code.data(), size, 0xcbf29ce484222325ull) == hash;
    }
    std::fclose(f);
    if (!ok) code.clear();
    return ok;
}

bool disk_store(const std::string& path, const std::vector<char>& code)
{
    static std::atomic<unsigned> serial{0};                  // two contexts of one process may store the same kernel at once
    const std::string tmp = path + ".tmp." + std::to_string((long)getpid()) + "." + std::to_string(serial.fetch_add(1));
    std::FILE* f = std::fopen(tmp.c_str(), "wb");
    if (!f) return false;
    const uint64_t size = code.size(), hash = fnv1a(code.data(), code.size(), 0xcbf29ce484222325ull);
    bool ok = std::fwrite(kDiskMagic, 1, 8, f) == 8 && std::fwrite(&size, 8, 1, f) == 1 && std::fwrite(&hash, 8, 1, f) == 1 &&
              std::fwrite(code.data(), 1, code.size(), f) == code.size();
    ok = (std::fclose(f) == 0) && ok;
    if (ok) ok = std::rename(tmp.c_str(), path.c_str()) == 0;
    if (!ok) (void)std::remove(tmp.c_str());
    return ok;
}

} // namespace

int32_t aixk_rtc_get(aixk_ctx* ctx, const char* key, const char* source, const char* entry, aixk_module** out, int32_t* was_cached)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(key && source && entry && out, "rtc_get: null argument");
    auto it = ctx->rtc.find(key);
    if (it != ctx->rtc.end()) {
        ++ctx->rtc_hits;
        *out = it->second;
        if (was_cached) *was_cached = 1;
        return AIXK_OK;
    }
    ++ctx->rtc_misses;
    if (was_cached) *was_cached = 0;

    std::string arch = std::string("--offload-arch=") + (ctx->prop.gcnArchName[0] ? ctx->prop.gcnArchName : "gfx950");
    // IEEE arithmetic: no contraction (a*b+c stays two roundings), no fast-math, correctly rounded
    // division and square root, no packed-f32 instruction selection.
    const char* opts[] = {arch.c_str(), "-O3", "-std=c++17", "-ffp-contract=off", "-fno-fast-math",
                          "-fhip-fp32-correctly-rounded-divide-sqrt",
                          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    const int nopts = (int)(sizeof(opts) / sizeof(opts[0]));

    // a code object an earlier process left on disk
    const std::string disk_path = ctx->rtc_disk_dir.empty() ? std::string() : disk_name(ctx, source, arch.c_str(), opts, nopts);
    if (!disk_path.empty()) {
        std::vector<char> kept;
        if (disk_load(disk_path, kept)) {
            aixk_module* mod = new aixk_module();
            hipError_t e = hipModuleLoadData(&mod->m.module, kept.data());
            if (e == hipSuccess) e = hipModuleGetFunction(&mod->m.fn, mod->m.module, entry);
            if (e == hipSuccess) {
                ++ctx->rtc_disk_hits;
                ctx->rtc.emplace(key, mod);
                *out = mod;
                return AIXK_OK;
            }
            if (mod->m.module) (void)hipModuleUnload(mod->m.module);     // not loadable here: compile, and replace the file
            delete mod;
            (void)hipGetLastError();
        }
    }

    hiprtcProgram prog;
    const char* header_names[] = {"aix_device.h"};
    const char* header_texts[] = {kPrelude};
    hiprtcResult r = hiprtcCreateProgram(&prog, source, "aix_fused.hip", 1, header_texts, header_names);
    if (r != HIPRTC_SUCCESS) return fail(AIXK_EHIP, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
    r = hiprtcCompileProgram(prog, nopts, opts);
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, '\0');
        if (n) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        return fail(AIXK_EHIP, "hipRTC compile failed (%s): %.800s", hiprtcGetErrorString(r), log.c_str());
    }
    size_t code_size = 0;
    hiprtcGetCodeSize(prog, &code_size);
    std::vector<char> code(code_size);
    hiprtcGetCode(prog, code.data());
    hiprtcDestroyProgram(&prog);

    aixk_module* mod = new aixk_module();
    hipError_t e = hipModuleLoadData(&mod->m.module, code.data());
    if (e == hipSuccess) e = hipModuleGetFunction(&mod->m.fn, mod->m.module, entry);
    if (e != hipSuccess) {
        if (mod->m.module) (void)hipModuleUnload(mod->m.module);
        delete mod;
        return fail(AIXK_EHIP, "loading the compiled kernel '%s' failed: %s", entry, hipGetErrorString(e));
    }
    ctx->rtc.emplace(key, mod);
    *out = mod;
    if (!disk_path.empty() && disk_store(disk_path, code)) ++ctx->rtc_disk_stores;     // a cache that cannot be written is no error
    return AIXK_OK;
}

int32_t aixk_rtc_disk_stats(aixk_ctx* ctx, uint64_t* loaded, uint64_t* stored)
{
    AIXK_REQUIRE(ctx != nullptr, "rtc_disk_stats: null context");
    if (loaded) *loaded = ctx->rtc_disk_hits;
    if (stored) *stored = ctx->rtc_disk_stores;
    return AIXK_OK;
}

int32_t aixk_rtc_launch_many(aixk_ctx* ctx, aixk_module* mod, uint32_t block_x, const void* table, size_t table_bytes,
                             size_t starts_offset, uint32_t count)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(mod && mod->m.fn, "rtc_launch_many: null kernel");
    AIXK_REQUIRE(table && count > 0 && block_x > 0 && block_x <= 1024, "rtc_launch_many: bad arguments");
    AIXK_REQUIRE(starts_offset % 4 == 0 && starts_offset + ((size_t)count + 1) * 4 <= table_bytes && table_bytes <= (256u << 10),
                 "rtc_launch_many: table of %zu bytes, starts at %zu, %u blocks", table_bytes, starts_offset, count);
    const uint32_t* starts = (const uint32_t*)((const char*)table + starts_offset);
    for (uint32_t k = 0; k < count; ++k) AIXK_REQUIRE(starts[k] < starts[k + 1], "rtc_launch_many: empty or unordered share %u", k);
    AIXK_REQUIRE(starts[0] == 0, "rtc_launch_many: the first share starts at workgroup %u", starts[0]);
    void* host = nullptr;
    const void* dev = nullptr;
    AIXK_TRY(aixk::table_slot(ctx, table_bytes, &host, &dev));
    std::memcpy(host, table, table_bytes);
    AIXK_TRY(aixk::table_upload(ctx, host, dev, table_bytes));
    struct { uint64_t table; uint64_t starts; uint32_t count; uint32_t pad; } args{(uint64_t)(uintptr_t)dev, (uint64_t)(uintptr_t)dev + starts_offset, count, 0};
    size_t size = sizeof(args);
    void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
    AIXK_HIP(hipModuleLaunchKernel(mod->m.fn, starts[count], 1, 1, block_x, 1, 1, 0, ctx->stream, nullptr, config));
    return AIXK_OK;
}

int32_t aixk_rtc_launch(aixk_ctx* ctx, aixk_module* mod, uint32_t grid_x, uint32_t block_x, const void* args, size_t args_bytes)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(mod && mod->m.fn, "rtc_launch: null kernel");
    AIXK_REQUIRE(grid_x > 0 && block_x > 0 && block_x <= 1024, "rtc_launch: bad launch shape %u x %u", grid_x, block_x);
    AIXK_REQUIRE(args != nullptr || args_bytes == 0, "rtc_launch: null argument block");
    size_t size = args_bytes;
    void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, const_cast<void*>(args), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
    AIXK_HIP(hipModuleLaunchKernel(mod->m.fn, grid_x, 1, 1, block_x, 1, 1, 0, ctx->stream, nullptr, config));
    return AIXK_OK;
}

// ---- a stretch of the stream as a graph ----------------------------------------------------------------------------
int32_t aixk_capture_begin(aixk_ctx* ctx)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(!ctx->capturing, "capture_begin: a capture is already open on this context");
    if (!ctx->side) AIXK_HIP(hipStreamCreateWithFlags(&ctx->side, hipStreamNonBlocking));
    AIXK_HIP(hipStreamSynchronize(ctx->stream));
    // relaxed: the thread may go on calling hipMalloc and copying on other streams while this one records
    AIXK_HIP(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeRelaxed));
    ctx->capturing = new aixk_graph();
    return AIXK_OK;
}

int32_t aixk_capture_end(aixk_ctx* ctx, aixk_graph** out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(ctx->capturing && out, "capture_end: no capture is open on this context");
    aixk_graph* g = ctx->capturing;
    ctx->capturing = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &g->graph);
    if (e == hipSuccess && !g->graph) e = hipErrorInvalidValue;
    if (e == hipSuccess) e = hipGraphInstantiate(&g->exec, g->graph, nullptr, nullptr, 0);
    size_t nodes = 0;
    if (e == hipSuccess) e = hipGraphGetNodes(g->graph, nullptr, &nodes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        aixk_graph_destroy(ctx, g);
        return fail(AIXK_EHIP, "capture_end: %s", hipGetErrorString(e));
    }
    g->nodes = nodes;
    *out = g;
    return AIXK_OK;
}

int32_t aixk_capture_abort(aixk_ctx* ctx)
{
    if (!ctx || !ctx->capturing) return AIXK_OK;
    (void)hipSetDevice(ctx->device);
    aixk_graph* g = ctx->capturing;
    ctx->capturing = nullptr;
    (void)hipStreamEndCapture(ctx->stream, &g->graph);
    (void)hipGetLastError();
    return aixk_graph_destroy(ctx, g);
}

int32_t aixk_graph_launch(aixk_ctx* ctx, aixk_graph* g)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(g && g->exec, "graph_launch: null graph");
    AIXK_REQUIRE(!ctx->capturing, "graph_launch: a capture is open on this context");
    AIXK_HIP(hipGraphLaunch(g->exec, ctx->stream));
    return AIXK_OK;
}

int32_t aixk_graph_nodes(aixk_graph* g, uint64_t* nodes)
{
    AIXK_REQUIRE(g && nodes, "graph_nodes: null argument");
    *nodes = g->nodes;
    return AIXK_OK;
}

int32_t aixk_graph_destroy(aixk_ctx* ctx, aixk_graph* g)
{
    if (!g) return AIXK_OK;
    if (ctx) { (void)hipSetDevice(ctx->device); (void)hipStreamSynchronize(ctx->stream); }     // a replay may still be running
    if (g->exec) (void)hipGraphExecDestroy(g->exec);
    if (g->graph) (void)hipGraphDestroy(g->graph);
    for (auto& t : g->tables) { (void)hipFree(t.first); (void)hipHostFree(t.second); }
    delete g;
    return AIXK_OK;
}

int32_t aixk_rtc_stats(aixk_ctx* ctx, uint64_t* hits, uint64_t* misses)
{
    AIXK_REQUIRE(ctx != nullptr, "null context");
    if (hits) *hits = ctx->rtc_hits;
    if (misses) *misses = ctx->rtc_misses;
    return AIXK_OK;
}

// ---- timing -----------------------------------------------------------------------------------
int32_t aixk_event_create(aixk_ctx* ctx, aixk_event** out)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(out != nullptr, "event_create: null out pointer");
    aixk_event* ev = new aixk_event();
    hipError_t e = hipEventCreate(&ev->ev);
    if (e != hipSuccess) { delete ev; return fail(AIXK_EHIP, "hipEventCreate: %s", hipGetErrorString(e)); }
    *out = ev;
    return AIXK_OK;
}

int32_t aixk_event_record(aixk_ctx* ctx, aixk_event* ev)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(ev != nullptr, "event_record: null event");
    AIXK_REQUIRE(!ctx->capturing, "event_record: no events inside a capture");
    AIXK_HIP(hipEventRecord(ev->ev, ctx->stream));
    return AIXK_OK;
}

int32_t aixk_event_query(aixk_ctx* ctx, aixk_event* ev, int32_t* done)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(ev && done, "event_query: null argument");
    const hipError_t e = hipEventQuery(ev->ev);
    if (e == hipSuccess) { *done = 1; return AIXK_OK; }
    if (e == hipErrorNotReady) { (void)hipGetLastError(); *done = 0; return AIXK_OK; }
    return fail(AIXK_EHIP, "hipEventQuery: %s", hipGetErrorString(e));
}

int32_t aixk_event_elapsed_ms(aixk_ctx* ctx, aixk_event* start, aixk_event* stop, float* ms)
{
    AIXK_TRY(set_device(ctx));
    AIXK_REQUIRE(start && stop && ms, "event_elapsed: null argument");
    AIXK_HIP(hipEventSynchronize(stop->ev));
    AIXK_HIP(hipEventElapsedTime(ms, start->ev, stop->ev));
    return AIXK_OK;
}

int32_t aixk_event_destroy(aixk_ctx* ctx, aixk_event* ev)
{
    if (!ev) return AIXK_OK;
    if (ctx) (void)hipSetDevice(ctx->device);
    (void)hipEventDestroy(ev->ev);
    delete ev;
    return AIXK_OK;
}

} // extern "C"
