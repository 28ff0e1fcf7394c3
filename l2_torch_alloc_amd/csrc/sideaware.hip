// sideaware.so for MI355X: device contexts, the kernel registry and launcher, and the C ABI.
// Declarations and the reference interface each entry point replaces: include/sideaware.h.
#include <hip/hip_runtime.h>

#include <array>
#include <atomic>
#include <cctype>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/sideaware.h"
#include "hip_backing.h"
#include "launch_plan.h"
#include "pool.h"
#include "rtc.h"

namespace sideaware {

// ---------------------------------------------------------------------------------------------
// Source text compiled at run time
// ---------------------------------------------------------------------------------------------

static const char* kKernelTemplate =
#include "elementwise_kernel.generated.inc"
    ;

// Kernel id 0: a bit-exact copy, four bytes per element so that sixteen bytes make one vector.
// The source is marked evict (read once, with the streaming hint) and UNROLLED is left at 1: one
// workgroup moves one 4 KiB chunk.  The destination is written plainly while it fits the Infinity
// Cache, so the next kernel finds it there, and with the streaming hint beyond that.
static const char* kMemcpyHeader = R"SA_HDR(
#define KERNEL_NAME sideaware_copy
typedef int o0;
typedef int i0;
struct unused {};
typedef unused o1, o2, o3, i1, i2, i3;

constexpr bool reverse_order = false;
constexpr bool input_evict[4] = {true, false, false, false};

__device__ __forceinline__ void elementwise_op(size_t element_idx, int sideband,
                                               o0 &out0, o1 &out1, o2 &out2, o3 &out3,
                                               const i0 &in0, const i1 &in1, const i2 &in2, const i3 &in3) {
    out0 = in0;
}
)SA_HDR";

// ---------------------------------------------------------------------------------------------
// Errors: recorded, printed, never thrown
// ---------------------------------------------------------------------------------------------

static std::mutex g_err_mu;
static std::string g_last_error;
static std::string g_last_error_snapshot;

static void set_error(const char* fmt, ...) {
    char buf[2048];
    va_list ap;
    va_start(ap, fmt);
    std::vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    std::fprintf(stderr, "sideaware: %s\n", buf);
    std::lock_guard<std::mutex> g(g_err_mu);
    g_last_error = buf;
}

// ---------------------------------------------------------------------------------------------
// Tuning
// ---------------------------------------------------------------------------------------------

struct Tuning {
    long long stripe_bytes = 16384;  // ownership stripe of an XCD (power of two; shrunk for small arrays)
    long long slot_run = 1;          // tiles a workgroup takes in a row; 0 = one contiguous block each
    long long one_shot = 1;          // 1: one workgroup per tile unless the caller fixes the groups
    long long cache_bytes = 256ll << 20;   // arrays larger than this are compiled to stream in both directions
    long long nt_store = 2;          // nontemporal stores: 0 never, 1 always, 2 only for arrays beyond the Infinity Cache
    long long groups_cap = 8;        // upper bound on default workgroups per CU
    long long wg_threads = 256;
};
static Tuning g_tune;
static std::atomic<unsigned> g_tune_generation{0};
static std::mutex g_tune_mu;

static long long env_ll(const char* name, long long fallback) {
    const char* v = std::getenv(name);
    return v && *v ? std::atoll(v) : fallback;
}

static void load_tuning_from_env_once() {
    static std::once_flag once;
    std::call_once(once, [] {
        g_tune.stripe_bytes = env_ll("SIDEAWARE_STRIPE_BYTES", g_tune.stripe_bytes);
        g_tune.slot_run = env_ll("SIDEAWARE_SLOT_RUN", g_tune.slot_run);
        g_tune.one_shot = env_ll("SIDEAWARE_ONE_SHOT", g_tune.one_shot);
        g_tune.cache_bytes = env_ll("SIDEAWARE_CACHE_BYTES", g_tune.cache_bytes);
        g_tune.nt_store = env_ll("SIDEAWARE_NT_STORE", g_tune.nt_store);
        g_tune.groups_cap = env_ll("SIDEAWARE_GROUPS_CAP", g_tune.groups_cap);
        g_tune.wg_threads = env_ll("SIDEAWARE_WG_THREADS", g_tune.wg_threads);
    });
}

static long long* tune_slot(const char* key) {
    if (!key) return nullptr;
    if (!std::strcmp(key, "stripe_bytes")) return &g_tune.stripe_bytes;
    if (!std::strcmp(key, "slot_run")) return &g_tune.slot_run;
    if (!std::strcmp(key, "one_shot")) return &g_tune.one_shot;
    if (!std::strcmp(key, "cache_bytes")) return &g_tune.cache_bytes;
    if (!std::strcmp(key, "nt_store")) return &g_tune.nt_store;
    if (!std::strcmp(key, "groups_cap")) return &g_tune.groups_cap;
    if (!std::strcmp(key, "wg_threads")) return &g_tune.wg_threads;
    return nullptr;
}

// ---------------------------------------------------------------------------------------------
// Device context
// ---------------------------------------------------------------------------------------------

constexpr int kMaxCUs = 1024;
constexpr int kDefaultXcds = 8;       // MI355X, used when no device is there to ask
constexpr int kDefaultCUs = 256;

// Reads the id of the XCD (the "XCC" of the ISA documents) a workgroup is running on.
__global__ void sa_probe_xcd(unsigned char* wg_xcd) {
    if (threadIdx.x == 0) {
        unsigned int xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        wg_xcd[blockIdx.x] = (unsigned char)(xcc & 0xf);
    }
}

struct ScopedDevice {
    int prev = -1;
    bool switched = false;
    explicit ScopedDevice(int want) {
        if (hipGetDevice(&prev) == hipSuccess && prev != want) switched = hipSetDevice(want) == hipSuccess;
    }
    ~ScopedDevice() {
        if (switched) (void)hipSetDevice(prev);
    }
};

struct DeviceContext {
    int device = -1;
    bool ready = false;
    int num_cus = 0;
    int num_xcds = 1;
    int cus_per_xcd = 0;
    bool dealing_verified = false;
    int cus_on_xcd[16] = {0};
    unsigned char cpu_side_index[kMaxCUs] = {0};
    unsigned char* gpu_side_index = nullptr;
    int side_summary[5] = {0};
    std::unique_ptr<HipBacking> backing;
    std::unique_ptr<Pool> pool;
    std::once_flag once;

    void initialize();
};

static int g_num_devices = -1;
static std::once_flag g_devices_once;
static std::vector<std::unique_ptr<DeviceContext>> g_contexts;

static int stripe_hash_mask(int num_xcds) {
    // the address bits that select the owning XCD of a byte: log2(num_xcds) bits above the stripe
    long long stripe = g_tune.stripe_bytes;
    long long mask = 0;
    for (long long x = 1; x < num_xcds; x <<= 1) mask |= stripe * x;
    return (int)(mask & 0x7fffffff);
}

// Settings may arrive before the first device call: they are kept here, applied to every
// context that exists, and replayed on contexts created later.
static std::mutex g_config_mu;
static size_t g_pending_threshold = 0;
static bool g_have_pending_threshold = false;
static size_t g_pending_trim[2] = {0, 0};
static bool g_have_pending_trim = false;
static size_t g_pending_limit = 0;
static bool g_have_pending_limit = false;
static size_t g_pending_arena = 0;
static bool g_have_pending_arena = false;

static void apply_config(Pool* pool) {
    std::lock_guard<std::mutex> g(g_config_mu);
    if (g_have_pending_threshold) pool->set_large_threshold(g_pending_threshold);
    if (g_have_pending_trim) pool->set_trim_thresholds(g_pending_trim[0], g_pending_trim[1]);
    if (g_have_pending_limit) pool->set_reserve_limit(g_pending_limit);
    if (g_have_pending_arena) pool->set_arena_bytes(g_pending_arena);
}

void DeviceContext::initialize() {
    ScopedDevice guard(device);
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || v <= 0) {
        set_error("device %d: cannot read the CU count", device);
        return;
    }
    num_cus = v > kMaxCUs ? kMaxCUs : v;
    v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeNumberOfXccs, device) != hipSuccess || v <= 0) {
        (void)hipGetLastError();
        v = 1;
    }
    num_xcds = v > 16 ? 16 : v;
    if (num_cus % num_xcds != 0) num_xcds = 1;
    cus_per_xcd = num_cus / num_xcds;

    // One workgroup per CU-sized slot; each reports the XCD it landed on.
    if (hipMalloc((void**)&gpu_side_index, kMaxCUs) != hipSuccess) {
        set_error("device %d: hipMalloc of the XCD table failed", device);
        return;
    }
    (void)hipMemset(gpu_side_index, 0xff, kMaxCUs);
    hipLaunchKernelGGL(sa_probe_xcd, dim3(num_cus), dim3(64), 0, 0, gpu_side_index);
    unsigned char seen[kMaxCUs];
    if (hipMemcpy(seen, gpu_side_index, num_cus, hipMemcpyDeviceToHost) != hipSuccess) {
        set_error("device %d: XCD probe failed: %s", device, hipGetErrorString(hipGetLastError()));
        return;
    }
    dealing_verified = true;
    int rank[16] = {0};
    for (int i = 0; i < num_cus; i++) {
        int x = seen[i] < num_xcds ? seen[i] : i % num_xcds;
        if (seen[i] != i % num_xcds) dealing_verified = false;
        cpu_side_index[i] = (unsigned char)(((rank[x]++ & 0x1f) << 3) | (x & 7));
        cus_on_xcd[x]++;
    }
    (void)hipMemcpy(gpu_side_index, cpu_side_index, num_cus, hipMemcpyHostToDevice);

    int fewest = cus_on_xcd[0];
    for (int x = 1; x < num_xcds; x++) fewest = cus_on_xcd[x] < fewest ? cus_on_xcd[x] : fewest;
    side_summary[0] = num_cus;
    side_summary[1] = cus_on_xcd[0];
    side_summary[2] = num_xcds > 1 ? cus_on_xcd[1] : 0;
    side_summary[3] = fewest;
    side_summary[4] = stripe_hash_mask(num_xcds) | (1 << 21);

    backing = std::make_unique<HipBacking>(device);
    pool = std::make_unique<Pool>(backing.get());
    // The reference trims its cache from 16 GiB down to 2 GiB on an 80 GB part
    // (sideaware.cu:421-422); keep those proportions of whatever this device holds.
    size_t free_bytes = 0, total_bytes = 0;
    if (hipMemGetInfo(&free_bytes, &total_bytes) == hipSuccess && total_bytes > (80ull << 30)) {
        pool->set_trim_thresholds(total_bytes / 5, total_bytes / 40);
    }
    apply_config(pool.get());
    ready = true;
}

static DeviceContext* get_context(int device = -1) {
    load_tuning_from_env_once();
    std::call_once(g_devices_once, [] {
        int n = 0;
        if (hipGetDeviceCount(&n) != hipSuccess) {
            (void)hipGetLastError();
            n = 0;
        }
        g_num_devices = n;
        for (int i = 0; i < n; i++) {
            g_contexts.push_back(std::make_unique<DeviceContext>());
            g_contexts.back()->device = i;
        }
    });
    if (g_num_devices <= 0) {
        set_error("no HIP device is visible");
        return nullptr;
    }
    if (device < 0) {
        if (g_num_devices == 1) device = 0;
        else if (hipGetDevice(&device) != hipSuccess) device = 0;
    }
    if (device >= g_num_devices) {
        set_error("device %d does not exist (%d visible)", device, g_num_devices);
        return nullptr;
    }
    DeviceContext* ctx = g_contexts[device].get();
    std::call_once(ctx->once, [ctx] { ctx->initialize(); });
    if (!ctx->ready) {
        set_error("device %d failed to initialise", device);
        return nullptr;
    }
    return ctx;
}

// ---------------------------------------------------------------------------------------------
// Kernel registry: header text -> id, and per (id, device, variant) the compiled function
// ---------------------------------------------------------------------------------------------

constexpr int kMaxDevices = 16;
constexpr int kVariants = 8;

struct CompiledKernel {
    hipModule_t module = nullptr;
    hipFunction_t fn = nullptr;
    int vgprs = 0, sgprs = 0;
    int occupancy = 0;          // workgroups per CU the hardware can hold
    int tile_vectors = 0;       // from the module's sideaware_kernel_meta
    int owner_is_o0 = 0;
    bool failed = false;
    unsigned generation = 0;
};

struct KernelEntry {
    std::string header;         // fixed at registration
    int default_groups = 0;     // fixed at registration; 0: decide from occupancy
    // Guards function_name and compiled[]: a first-use compile of one op (hundreds of
    // milliseconds) does not hold up launches of the others.
    std::mutex mu;
    std::string function_name = "sideaware_elementwise";   // or the header's `#define KERNEL_NAME x`
    // [device * kVariants + variant]; variant = wide_index | beyond_cache << 1 | in_place << 2.
    // Fixed size: launches keep pointers into it while other threads compile other variants.
    std::array<CompiledKernel, kMaxDevices * kVariants> compiled;
};

static std::mutex g_kernels_mu;
static std::vector<std::unique_ptr<KernelEntry>> g_kernels;
static std::unordered_map<std::string, int> g_header_to_id;

// Finds `#define KERNEL_NAME identifier` in an op header.
static std::string kernel_name_of(const std::string& header) {
    const std::string key = "#define KERNEL_NAME";
    size_t pos = header.find(key);
    if (pos == std::string::npos) return "sideaware_elementwise";
    pos += key.size();
    while (pos < header.size() && (header[pos] == ' ' || header[pos] == '\t')) pos++;
    size_t end = pos;
    while (end < header.size() && (std::isalnum((unsigned char)header[end]) || header[end] == '_')) end++;
    return end > pos ? header.substr(pos, end - pos) : "sideaware_elementwise";
}

static void ensure_builtin_locked() {
    if (!g_kernels.empty()) return;
    auto e = std::make_unique<KernelEntry>();
    e->header = kMemcpyHeader;
    e->function_name = kernel_name_of(e->header);
    g_kernels.push_back(std::move(e));
}

static std::string config_block(int variant, int num_xcds, int num_cus) {
    load_tuning_from_env_once();
    std::string s;
    s += "#define SA_NUM_XCD " + std::to_string(num_xcds) + "\n";
    s += "#define SA_WG_THREADS " + std::to_string(g_tune.wg_threads) + "\n";
    s += "#define SA_NT_STORE " + std::to_string(g_tune.nt_store) + "\n";
    // Names the reference injects (sideaware.cu:789-794); kept so headers that mention them compile.
    s += "#define MAX_SM " + std::to_string(num_cus) + "\n";
    s += "#define HASH " + std::to_string((stripe_hash_mask(num_xcds) | (1 << 21)) / 16) + "\n";
    s += "#define SA_BEYOND_CACHE " + std::to_string((variant >> 1) & 1) + "\n";
    s += "#define SA_IN_PLACE " + std::to_string((variant >> 2) & 1) + "\n";
    s += (variant & 1) ? "using size_type = long long;\nconstexpr bool aligned_2MiB = false;\n"
                       : "using size_type = int;\nconstexpr bool aligned_2MiB = true;\n";
    return s;
}

static std::string full_source(const std::string& header, int variant, int num_xcds, int num_cus) {
    return config_block(variant, num_xcds, num_cus) + "\n" + header + "\n" + kKernelTemplate;
}

// Returns the compiled function for (id, variant) on ctx's device, building it on first use
// (sideaware.cu:772-813).  Null after a failed compile; the failure is reported once.
static KernelEntry* find_entry(int kernel_id) {
    std::lock_guard<std::mutex> g(g_kernels_mu);
    ensure_builtin_locked();
    if (kernel_id < 0 || kernel_id >= (int)g_kernels.size()) {
        set_error("kernel id %d was never created", kernel_id);
        return nullptr;
    }
    return g_kernels[kernel_id].get();      // entries are never removed
}

static CompiledKernel* get_kernel(DeviceContext* ctx, int kernel_id, int variant, KernelEntry** entry = nullptr) {
    KernelEntry* found = find_entry(kernel_id);
    if (entry) *entry = found;
    if (!found) return nullptr;
    KernelEntry& e = *found;
    std::lock_guard<std::mutex> g(e.mu);
    if (ctx->device >= kMaxDevices) {
        set_error("device %d is beyond the %d devices this build keeps kernels for", ctx->device, kMaxDevices);
        return nullptr;
    }
    CompiledKernel& k = e.compiled[(size_t)ctx->device * kVariants + (size_t)(variant & (kVariants - 1))];
    unsigned gen = g_tune_generation.load();
    if (k.generation != gen) {
        if (k.module) (void)hipModuleUnload(k.module);
        k = CompiledKernel();
        k.generation = gen;
    }
    if (k.fn) return &k;
    if (k.failed) return nullptr;

    CompileResult r = compile_for_gfx950(full_source(e.header, variant, ctx->num_xcds, ctx->num_cus));
    if (!r.log.empty()) std::fprintf(stderr, "sideaware: compiler log for kernel %d:\n%s\n", kernel_id, r.log.c_str());
    if (!r.ok) {
        k.failed = true;
        set_error("kernel %d (variant %d) failed to compile", kernel_id, variant);
        return nullptr;
    }
    ScopedDevice guard(ctx->device);
    hipError_t err = hipModuleLoadData(&k.module, r.code.data());
    if (err != hipSuccess && r.from_disk_cache) {
        // a cached code object the runtime refuses (damaged file, another driver): build it again
        (void)hipGetLastError();
        k.module = nullptr;
        r = compile_for_gfx950(full_source(e.header, variant, ctx->num_xcds, ctx->num_cus), "gfx950",
                               /*use_disk_cache=*/false);
        err = r.ok ? hipModuleLoadData(&k.module, r.code.data()) : hipErrorInvalidImage;
    }
    if (err == hipSuccess) {
        // The module itself says what its entry point is called: the header text may not (a
        // header that is only `#include "file"`, example_llmc_rope.cu:138).
        char name[128] = {0};
        hipDeviceptr_t name_ptr = nullptr;
        size_t name_bytes = 0;
        if (hipModuleGetGlobal(&name_ptr, &name_bytes, k.module, "sideaware_kernel_name") == hipSuccess &&
            name_bytes > 1 && name_bytes < sizeof name &&
            hipMemcpyDtoH(name, name_ptr, name_bytes) == hipSuccess && name[0]) {
            e.function_name = name;               // e.mu is held
        } else {
            (void)hipGetLastError();
        }
        err = hipModuleGetFunction(&k.fn, k.module, e.function_name.c_str());
    }
    if (err != hipSuccess) {
        k.failed = true;
        k.fn = nullptr;
        set_error("kernel %d (variant %d) failed to load: %s", kernel_id, variant, hipGetErrorString(err));
        (void)hipGetLastError();
        return nullptr;
    }
    // The instantiation says how many vectors make a tile and which array's address defines
    // ownership; the launch planner needs both.
    {
        hipDeviceptr_t meta_ptr = nullptr;
        size_t meta_bytes = 0;
        int meta[4] = {0, 0, 0, 0};
        err = hipModuleGetGlobal(&meta_ptr, &meta_bytes, k.module, "sideaware_kernel_meta");
        if (err == hipSuccess && meta_bytes >= sizeof meta) err = hipMemcpyDtoH(meta, meta_ptr, sizeof meta);
        if (err != hipSuccess || meta[0] <= 0) {
            k.failed = true;
            k.fn = nullptr;
            set_error("kernel %d (variant %d): cannot read its tile size: %s", kernel_id, variant, hipGetErrorString(err));
            (void)hipGetLastError();
            return nullptr;
        }
        k.tile_vectors = meta[0];
        k.owner_is_o0 = meta[2];
    }
    (void)hipFuncGetAttribute(&k.vgprs, HIP_FUNC_ATTRIBUTE_NUM_REGS, k.fn);
    int occ = 0;
    if (hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&occ, k.fn, (int)g_tune.wg_threads, 0) != hipSuccess) {
        (void)hipGetLastError();
        occ = 0;
    }
    k.occupancy = occ;
    return &k;
}

static int register_header(const char* header, int default_groups) {
    std::lock_guard<std::mutex> g(g_kernels_mu);
    ensure_builtin_locked();
    if (!header || !*header) return 0;
    std::string text(header);
    auto it = g_header_to_id.find(text);
    if (it != g_header_to_id.end()) return it->second;
    auto e = std::make_unique<KernelEntry>();
    e->header = text;
    e->function_name = kernel_name_of(text);
    e->default_groups = default_groups > 0 ? default_groups : 0;
    g_kernels.push_back(std::move(e));
    int id = (int)g_kernels.size() - 1;
    g_header_to_id.emplace(std::move(text), id);
    return id;
}

}  // namespace sideaware

using namespace sideaware;

// =============================================================================================
// C ABI
// =============================================================================================
#pragma GCC visibility push(default)
extern "C" {

// ---- allocation -------------------------------------------------------------------------------

void* sideaware_malloc_auto(size_t size, int device, sideaware_stream_t stream) {
    DeviceContext* ctx = get_context(device);
    if (!ctx) return nullptr;
    return ctx->pool->allocate(size, stream, /*always_large=*/false);
}

void sideaware_free_auto(void* ptr, size_t size, int device, sideaware_stream_t stream) {
    (void)size;
    if (!ptr) return;
    DeviceContext* ctx = get_context(device);
    if (!ctx) return;
    ctx->pool->deallocate(ptr, stream);
}

int sideaware_malloc_async(void** dev_ptr, size_t size, sideaware_stream_t stream) {
    if (!dev_ptr) return (int)hipErrorInvalidValue;
    *dev_ptr = nullptr;
    DeviceContext* ctx = get_context();
    if (!ctx) return (int)hipErrorNoDevice;
    *dev_ptr = ctx->pool->allocate(size, stream, /*always_large=*/true);
    return *dev_ptr ? (int)hipSuccess : (int)hipErrorOutOfMemory;
}

int sideaware_free_async(void* ptr, sideaware_stream_t stream) {
    if (!ptr) return (int)hipSuccess;
    DeviceContext* ctx = get_context();
    if (!ctx) return (int)hipErrorNoDevice;
    return ctx->pool->deallocate(ptr, stream) == 0 ? (int)hipSuccess : (int)hipErrorInvalidValue;
}

int sideaware_malloc(void** dev_ptr, size_t size) {
    DeviceContext* ctx = get_context();
    if (!ctx) {
        if (dev_ptr) *dev_ptr = nullptr;
        return (int)hipErrorNoDevice;
    }
    ctx->backing->sync_device();
    return sideaware_malloc_async(dev_ptr, size, nullptr);
}

int sideaware_free(void* ptr) {
    DeviceContext* ctx = get_context();
    if (!ctx) return (int)hipErrorNoDevice;
    ctx->backing->sync_device();
    return sideaware_free_async(ptr, nullptr);
}

size_t sideaware_release_unused(void) {
    size_t total = 0;
    for (auto& c : g_contexts) {
        if (c && c->ready) total += c->pool->release_unused();
    }
    return total;
}

// ---- kernels ----------------------------------------------------------------------------------

int sideaware_create_kernel_advanced(const char* header, bool precompile, int default_num_groups) {
    int id = register_header(header, default_num_groups);
    if (precompile) {
        if (DeviceContext* ctx = get_context()) {
            for (int v = 0; v <= 4; v++) get_kernel(ctx, id, v);     // both index widths x both size classes, and in place
        }
    }
    return id;
}

int sideaware_create_kernel(const char* header) {
    return sideaware_create_kernel_advanced(header, false, 0);
}

void sideaware_elementwise(int kernel_id, size_t num_bytes,
                           void* out0, void* out1, void* out2, void* out3,
                           const void* in0, const void* in1, const void* in2, const void* in3,
                           void* sideband_memory, int sideband_value,
                           int parallel_groups, int forced_per_side,
                           int device, sideaware_stream_t stream) {
    if (num_bytes == 0 || (out0 == nullptr && in0 == nullptr)) return;
    DeviceContext* ctx = get_context(device);
    if (!ctx) return;
    if ((uintptr_t)out0 % 16 || (uintptr_t)in0 % 16 || num_bytes % 16) {
        set_error("elementwise: out0 (%p), in0 (%p) and num_bytes (%zu) must be multiples of 16",
                  out0, in0, num_bytes);
        return;
    }

    // Lazily compiled instantiations per op.  Index width: 32-bit below 2 GiB, 64-bit from there on (the
    // reference also sends bases that are not 2 MiB-aligned to its 64-bit variant,
    // sideaware.cu:1386-1388; here the base only shifts the planner's b0, whatever its alignment).
    // Cache class: arrays whose result fits the Infinity Cache (written plainly, so the next kernel
    // finds it there) and larger ones (everything streams).
    // In place (o0 written over i0) is a class of its own below the cache size: see the template's
    // notes on cache policy.  Beyond it everything streams already.
    const int wide = num_bytes >= (2ull << 30) ? 1 : 0;
    const int beyond = num_bytes > (unsigned long long)g_tune.cache_bytes ? 2 : 0;
    const int in_place = (!beyond && out0 != nullptr && out0 == in0) ? 4 : 0;
    const int variant = wide | beyond | in_place;

    KernelEntry* entry = nullptr;
    CompiledKernel* k = get_kernel(ctx, kernel_id, variant, &entry);
    if (!k) return;
    const int default_groups = entry->default_groups;
    // Workgroups per XCD.  The caller's parallel_groups / forced_per_side, or the header's
    // default, fix a persistent grid of (CUs per XCD) x groups; otherwise the tuning decides
    // between one workgroup per tile and a persistent grid sized from the kernel's occupancy.
    int per_xcd = ctx->cus_per_xcd;
    if (forced_per_side > 0 && forced_per_side < per_xcd) per_xcd = forced_per_side;
    int groups = parallel_groups > 0 ? parallel_groups : default_groups;
    long long slots_wanted;
    if (groups > 0 || forced_per_side > 0 || !g_tune.one_shot) {
        if (groups <= 0) {
            groups = k->occupancy > 0 ? k->occupancy : 4;
            if (groups > g_tune.groups_cap) groups = (int)g_tune.groups_cap;
        }
        slots_wanted = (long long)per_xcd * groups;
    } else {
        slots_wanted = 0;
    }

    const long long num_vectors = (long long)(num_bytes / 16);
    // The ownership stripe: the tuned size, shrunk for arrays too short to give every XCD at least
    // ~32 stripes of it (one XCD can be a stripe ahead of another).
    unsigned long long stripe = (unsigned long long)g_tune.stripe_bytes;
    while (stripe > 4096 && stripe * 32 * ctx->num_xcds > num_bytes) stripe >>= 1;
    const uint64_t base = (uint64_t)(uintptr_t)(k->owner_is_o0 ? out0 : in0);
    LaunchPlan plan = plan_launch(base, num_vectors, k->tile_vectors, ctx->num_xcds, stripe,
                                  g_tune.slot_run, slots_wanted);
    const unsigned grid = plan.grid;

    long long nv64 = num_vectors, ft64 = plan.full_tiles, b064 = plan.b0, uc64 = plan.u_count, run64 = plan.run;
    int nv32 = (int)num_vectors, ft32 = (int)plan.full_tiles, b032 = (int)plan.b0, uc32 = (int)plan.u_count,
        run32 = (int)plan.run;
    int* mem = (int*)sideband_memory;
    void* args[17];
    args[0] = wide ? (void*)&nv64 : (void*)&nv32;
    args[1] = &out0;
    args[2] = &out1;
    args[3] = &out2;
    args[4] = &out3;
    args[5] = &in0;
    args[6] = &in1;
    args[7] = &in2;
    args[8] = &in3;
    args[9] = &mem;
    args[10] = &sideband_value;
    args[11] = wide ? (void*)&ft64 : (void*)&ft32;
    args[12] = wide ? (void*)&b064 : (void*)&b032;
    args[13] = wide ? (void*)&uc64 : (void*)&uc32;
    args[14] = wide ? (void*)&run64 : (void*)&run32;
    args[15] = &plan.r;
    args[16] = &plan.tail_block;

    ScopedDevice guard(ctx->device);
    hipError_t err = hipModuleLaunchKernel(k->fn, grid, 1, 1, (unsigned)g_tune.wg_threads, 1, 1, 0,
                                           (hipStream_t)stream, args, nullptr);
    if (err != hipSuccess) {
        set_error("elementwise: launch of kernel %d failed: %s", kernel_id, hipGetErrorString(err));
        (void)hipGetLastError();
    }
}

void sideaware_one_to_one(int kernel_id, size_t num_bytes, void* out0, const void* in0,
                          int device, sideaware_stream_t stream) {
    sideaware_elementwise(kernel_id, num_bytes, out0, nullptr, nullptr, nullptr, in0, nullptr, nullptr, nullptr,
                          nullptr, 0, 0, 0, device, stream);
}

void sideaware_memcpy(void* out, const void* in, size_t num_bytes, int device, sideaware_stream_t stream) {
    sideaware_elementwise(0, num_bytes, out, nullptr, nullptr, nullptr, in, nullptr, nullptr, nullptr,
                          nullptr, 0, 0, 0, device, stream);
}

// ---- configuration ----------------------------------------------------------------------------

void sideaware_compression(bool enable) { (void)enable; }

void sideaware_alloc_threshold(size_t threshold) {
    {
        std::lock_guard<std::mutex> g(g_config_mu);
        g_pending_threshold = threshold;
        g_have_pending_threshold = true;
    }
    for (auto& c : g_contexts) if (c && c->ready) apply_config(c->pool.get());
}

void sideaware_prealloc_config(int extra_required, int extra_alloc) {
    (void)extra_required;
    (void)extra_alloc;
}

void sideaware_free_mapped_thresholds(size_t start_threshold, size_t end_threshold) {
    {
        std::lock_guard<std::mutex> g(g_config_mu);
        g_pending_trim[0] = start_threshold;
        g_pending_trim[1] = end_threshold;
        g_have_pending_trim = true;
    }
    for (auto& c : g_contexts) if (c && c->ready) apply_config(c->pool.get());
}

void sideaware_reserve_limit(size_t bytes) {
    {
        std::lock_guard<std::mutex> g(g_config_mu);
        g_pending_limit = bytes;
        g_have_pending_limit = true;
    }
    for (auto& c : g_contexts) if (c && c->ready) apply_config(c->pool.get());
}

void sideaware_arena_bytes(size_t bytes) {
    {
        std::lock_guard<std::mutex> g(g_config_mu);
        g_pending_arena = bytes;
        g_have_pending_arena = true;
    }
    for (auto& c : g_contexts) if (c && c->ready) apply_config(c->pool.get());
}

void sideaware_write_sass(const char* filename) { set_isa_dump_file(filename ? filename : ""); }

// ---- queries ----------------------------------------------------------------------------------

void sideaware_fill_side_index(unsigned char* gpu_array) {
    DeviceContext* ctx = get_context();
    if (!ctx || !gpu_array) return;
    if (hipMemcpy(gpu_array, ctx->gpu_side_index, ctx->num_cus, hipMemcpyDeviceToDevice) != hipSuccess) {
        set_error("fill_side_index: copy failed: %s", hipGetErrorString(hipGetLastError()));
    }
}

const char* sideaware_gpu_side_index(void) {
    DeviceContext* ctx = get_context();
    return ctx ? (const char*)ctx->gpu_side_index : nullptr;
}

const char* sideaware_cpu_side_index(void) {
    DeviceContext* ctx = get_context();
    return ctx ? (const char*)ctx->cpu_side_index : nullptr;
}

const int* sideaware_sm_side_summary(void) {
    static int none[5] = {0, 0, 0, 0, 0};
    DeviceContext* ctx = get_context();
    if (!ctx) return none;
    ctx->side_summary[4] = stripe_hash_mask(ctx->num_xcds) | (1 << 21);
    return ctx->side_summary;
}

int sideaware_num_sms(void) { DeviceContext* c = get_context(); return c ? c->side_summary[0] : 0; }
int sideaware_num_sm_side0(void) { DeviceContext* c = get_context(); return c ? c->side_summary[1] : 0; }
int sideaware_num_sm_side1(void) { DeviceContext* c = get_context(); return c ? c->side_summary[2] : 0; }
int sideaware_min_sm_per_side(void) { DeviceContext* c = get_context(); return c ? c->side_summary[3] : 0; }
int sideaware_hash_mask(void) {
    DeviceContext* c = get_context();
    return c ? (stripe_hash_mask(c->num_xcds) | (1 << 21)) : 0;
}

// ---- additions --------------------------------------------------------------------------------

int sideaware_num_xcds(void) { DeviceContext* c = get_context(); return c ? c->num_xcds : 0; }
int sideaware_xcd_dealing_verified(void) { DeviceContext* c = get_context(); return c && c->dealing_verified ? 1 : 0; }

const char* sideaware_last_error(void) {
    std::lock_guard<std::mutex> g(g_err_mu);
    g_last_error_snapshot = g_last_error;
    return g_last_error_snapshot.c_str();
}

void sideaware_clear_error(void) {
    std::lock_guard<std::mutex> g(g_err_mu);
    g_last_error.clear();
}

int sideaware_compile_check(const char* header, int variant, char* log, size_t log_capacity) {
    std::string hdr = header && *header ? header : kMemcpyHeader;
    CompileResult r = compile_for_gfx950(full_source(hdr, variant & (kVariants - 1), kDefaultXcds, kDefaultCUs));
    if (log && log_capacity) {
        std::snprintf(log, log_capacity, "%s", r.log.c_str());
    }
    return r.ok ? 0 : 1;
}

const char* sideaware_kernel_source(void) { return kKernelTemplate; }
const char* sideaware_memcpy_header(void) { return kMemcpyHeader; }

const char* sideaware_config_block(int variant) {
    static std::mutex mu;
    static std::string text[kVariants];
    std::lock_guard<std::mutex> g(mu);
    const int v = variant & (kVariants - 1);
    text[v] = config_block(v, kDefaultXcds, kDefaultCUs);
    return text[v].c_str();
}

int sideaware_kernel_info(int kernel_id, int variant, int* out) {
    DeviceContext* ctx = get_context();
    if (!ctx || !out) return 1;
    KernelEntry* entry = nullptr;
    CompiledKernel* k = get_kernel(ctx, kernel_id, variant & (kVariants - 1), &entry);
    if (!k) return 1;
    int groups = entry->default_groups;
    if (groups <= 0) {
        groups = k->occupancy > 0 ? k->occupancy : 4;
        if (groups > g_tune.groups_cap) groups = (int)g_tune.groups_cap;
    }
    out[0] = k->vgprs;
    out[1] = k->sgprs;
    out[2] = k->occupancy;
    out[3] = groups;
    return 0;
}

int sideaware_alloc_stats(unsigned long long* out, int capacity) {
    DeviceContext* ctx = get_context();
    if (!ctx || !out) return 0;
    PoolStats s = ctx->pool->stats();
    const uint64_t* f = (const uint64_t*)&s;
    int n = capacity < kPoolStatsFields ? capacity : kPoolStatsFields;
    for (int i = 0; i < n; i++) out[i] = f[i];
    return n;
}

int sideaware_tune(const char* key, long long value) {
    load_tuning_from_env_once();
    std::lock_guard<std::mutex> g(g_tune_mu);
    long long* slot = tune_slot(key);
    if (!slot) return 1;
    if (!std::strcmp(key, "wg_threads") && (value < 64 || value > 1024 || (value & (value - 1)))) return 1;
    if (!std::strcmp(key, "stripe_bytes") && (value < 4096 || value > (1ll << 30) || (value & (value - 1)))) return 1;
    if (!std::strcmp(key, "slot_run") && (value < 0 || value > (1 << 20))) return 1;
    if (*slot != value) {
        *slot = value;
        const bool compiled_in = !std::strcmp(key, "nt_store") || !std::strcmp(key, "wg_threads");
        if (compiled_in) g_tune_generation++;      // compiled kernels are rebuilt on their next use
    }
    return 0;
}

long long sideaware_tune_get(const char* key) {
    load_tuning_from_env_once();
    std::lock_guard<std::mutex> g(g_tune_mu);
    long long* slot = tune_slot(key);
    return slot ? *slot : -1;
}

}  // extern "C"
#pragma GCC visibility pop
