#include "runtime.hpp"

#include <dlfcn.h>

#include <hip/hiprtc.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sys/stat.h>
#include <unistd.h>

namespace dsc {

namespace {
thread_local std::string g_last_error;
}

void set_error(const std::string& msg) { g_last_error = msg; }
const std::string& last_error() { return g_last_error; }
int fail(int status, const std::string& msg) {
    g_last_error = msg;
    return status;
}

#define HIP_TRY(expr)                                                                                     \
    do {                                                                                                  \
        hipError_t e_ = (expr);                                                                           \
        if (e_ != hipSuccess) return fail(DSC_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_)); \
    } while (0)

// ---------------------------------------------------------------------------------------------- heap

DeviceHeap::~DeviceHeap() {
    for (auto& c : chunks_)
        if (c.base) (void)hipFree(c.base);
}

void DeviceHeap::add_free(int chunk, size_t offset, size_t size) {
    free_by_size_[chunks_[chunk].io].emplace(size, std::make_pair(chunk, offset));
}

void DeviceHeap::remove_free(int chunk, size_t offset, size_t size) {
    auto& by_size = free_by_size_[chunks_[chunk].io];
    auto range = by_size.equal_range(size);
    for (auto it = range.first; it != range.second; ++it) {
        if (it->second.first == chunk && it->second.second == offset) {
            by_size.erase(it);
            return;
        }
    }
}

uint64_t DeviceHeap::alloc_io(size_t bytes, size_t need) {
    auto& by_size = free_by_size_[1];
    auto range = by_size.equal_range(need);
    auto best = by_size.end();
    for (auto it = range.first; it != range.second; ++it)
        if (best == by_size.end() ||
            chunks_[it->second.first].blocks[it->second.second].stamp < chunks_[best->second.first].blocks[best->second.second].stamp)
            best = it;
    int ci = -1;
    size_t off = 0;
    uint64_t stamp = 0;
    if (best != by_size.end()) {
        ci = best->second.first;
        off = best->second.second;
        by_size.erase(best);
        Block& b = chunks_[ci].blocks[off];
        b.is_free = false;
        stamp = b.stamp;
    } else {
        for (int i = 0; i < (int)chunks_.size() && ci < 0; ++i)
            if (chunks_[i].io && chunks_[i].size - chunks_[i].tail >= need) ci = i;
        if (ci < 0) {
            Chunk c;
            c.io = true;
            c.size = std::max(kIoChunkBytes, need);
            void* p = nullptr;
            if (hipMalloc(&p, c.size) != hipSuccess) {
                (void)hipGetLastError();
                return 0;
            }
            c.base = static_cast<char*>(p);
            chunks_.push_back(std::move(c));
            ci = (int)chunks_.size() - 1;
        }
        Chunk& c = chunks_[ci];
        off = c.tail;
        c.tail += need;
        c.blocks[off] = Block{need, false, 0};
    }
    const uint64_t h = next_handle_++;
    live_[h] = Live{ci, off, bytes, stamp};
    live_bytes_ += (int64_t)need;
    return h;
}

uint64_t DeviceHeap::alloc(size_t bytes, bool io) {
    const size_t need = std::max(kAlign, (bytes + kAlign - 1) / kAlign * kAlign);
    if (io) return alloc_io(bytes, need);
    auto& by_size = free_by_size_[0];
    auto it = by_size.lower_bound(need);
    if (it == by_size.end()) {
        Chunk c;
        c.size = std::max(kChunkBytes, need);
        void* p = nullptr;
        if (hipMalloc(&p, c.size) != hipSuccess) {
            (void)hipGetLastError();
            // a smaller chunk may still fit
            c.size = need;
            if (hipMalloc(&p, c.size) != hipSuccess) {
                (void)hipGetLastError();
                return 0;
            }
        }
        c.base = static_cast<char*>(p);
        c.blocks[0] = Block{c.size, true, 0};
        chunks_.push_back(std::move(c));
        add_free((int)chunks_.size() - 1, 0, chunks_.back().size);
        it = by_size.lower_bound(need);
    }
    const int ci = it->second.first;
    const size_t off = it->second.second;
    const size_t have = it->first;
    by_size.erase(it);
    Chunk& c = chunks_[ci];
    const uint64_t stamp = c.blocks[off].stamp;
    c.blocks[off] = Block{need, false, stamp};
    if (have > need) {
        c.blocks[off + need] = Block{have - need, true, stamp};
        add_free(ci, off + need, have - need);
    }
    const uint64_t h = next_handle_++;
    live_[h] = Live{ci, off, bytes, stamp};
    live_bytes_ += (int64_t)need;
    return h;
}

bool DeviceHeap::free(uint64_t handle) {
    auto lit = live_.find(handle);
    if (lit == live_.end()) return false;
    const int ci = lit->second.chunk;
    size_t off = lit->second.offset;
    uint64_t stamp = std::max(lit->second.stamp, clock ? *clock : 0);
    live_.erase(lit);
    Chunk& c = chunks_[ci];
    auto it = c.blocks.find(off);
    size_t size = it->second.size;
    live_bytes_ -= (int64_t)size;
    if (c.io) {  // recycled whole, by size
        it->second = Block{size, true, stamp};
        add_free(ci, off, size);
        return true;
    }
    // coalesce with the next range, then with the previous one
    auto next = std::next(it);
    if (next != c.blocks.end() && next->second.is_free) {
        remove_free(ci, next->first, next->second.size);
        size += next->second.size;
        stamp = std::max(stamp, next->second.stamp);
        c.blocks.erase(next);
    }
    if (it != c.blocks.begin()) {
        auto prev = std::prev(it);
        if (prev->second.is_free) {
            remove_free(ci, prev->first, prev->second.size);
            size += prev->second.size;
            stamp = std::max(stamp, prev->second.stamp);
            off = prev->first;
            c.blocks.erase(it);
            it = prev;
        }
    }
    it->second = Block{size, true, stamp};
    add_free(ci, off, size);
    return true;
}

bool DeviceHeap::info(uint64_t handle, void** ptr, size_t* bytes) const {
    auto it = live_.find(handle);
    if (it == live_.end()) return false;
    if (ptr) *ptr = chunks_[it->second.chunk].base + it->second.offset;
    if (bytes) *bytes = it->second.bytes;
    return true;
}

uint64_t DeviceHeap::stamp_of(uint64_t handle) const {
    auto it = live_.find(handle);
    return it == live_.end() ? 0 : it->second.stamp;
}

void DeviceHeap::touch(uint64_t handle, uint64_t stamp) {
    auto it = live_.find(handle);
    if (it != live_.end() && it->second.stamp < stamp) it->second.stamp = stamp;
}

void DeviceHeap::stats(int64_t* live, int64_t* live_bytes, int64_t* arena_bytes) const {
    if (live) *live = (int64_t)live_.size();
    if (live_bytes) *live_bytes = live_bytes_;
    if (arena_bytes) {
        int64_t total = 0;
        for (auto& c : chunks_) total += (int64_t)c.size;
        *arena_bytes = total;
    }
}

// ------------------------------------------------------------------------------------------- context

Context::~Context() {
    if (offline) return;
    if (copy_stream) (void)hipStreamSynchronize(copy_stream);
    if (stream) (void)hipStreamSynchronize(stream);
    for (auto& m : marks) (void)hipEventDestroy(m.second);
    for (auto& cp : copies)
        if (cp.own) (void)hipEventDestroy(cp.own);
    for (auto& kv : pinned) (void)hipHostFree(const_cast<char*>(kv.first));
    if (copy_stream) (void)hipStreamDestroy(copy_stream);
    for (auto& kv : kernels)
        if (kv.second->module) (void)hipModuleUnload(kv.second->module);
    for (auto& p : profile) {
        (void)hipEventDestroy(p.start);
        (void)hipEventDestroy(p.stop);
    }
    for (auto e : event_pool) (void)hipEventDestroy(e);
    for (auto& kv : fences) (void)hipEventDestroy(kv.second.event);
    for (auto e : fence_pool) (void)hipEventDestroy(e);
    for (int i = 0; i < kStagingRegions; ++i) {
        if (staging_done[i]) (void)hipEventDestroy(staging_done[i]);
        if (staging[i]) (void)hipHostFree(staging[i]);
    }
    if (seed_cell) (void)hipFree(seed_cell);
    if (stream) (void)hipStreamDestroy(stream);
}

// --------------------------------------------------------------------------------------------- hipRTC

namespace {

CacheStats g_cache_stats;

uint64_t fnv1a(const std::string& s, uint64_t seed) {
    uint64_t h = seed;
    for (unsigned char c : s) {
        h ^= c;
        h *= 1099511628211ull;
    }
    return h;
}

// Directory of the on-disk code-object cache ("" = disabled).  DSC_CACHE_DIR overrides; "off" disables.
std::string cache_dir() {
    const char* env = std::getenv("DSC_CACHE_DIR");
    std::string dir;
    if (env) {
        if (std::string(env) == "off") return "";
        dir = env;
    } else {
        const char* home = std::getenv("HOME");
        if (!home) return "";
        dir = std::string(home) + "/.cache";
        ::mkdir(dir.c_str(), 0755);
        dir += "/descent_amd";
    }
    ::mkdir(dir.c_str(), 0755);
    struct stat st;
    if (::stat(dir.c_str(), &st) != 0 || !S_ISDIR(st.st_mode)) return "";
    return dir;
}

// What a cached object depends on besides its source: the target, the compile options, the compiler (hipRTC) and
// runtime versions, and the layout of the cache file itself.
std::string cache_salt(const std::string& arch) {
    std::string salt = arch;
    for (auto& o : compile_options()) salt += "|" + o;
    int rtc_major = 0, rtc_minor = 0, runtime = 0;
    (void)hiprtcVersion(&rtc_major, &rtc_minor);
    if (hipRuntimeGetVersion(&runtime) != hipSuccess) (void)hipGetLastError();
    salt += "|hiprtc " + std::to_string(rtc_major) + "." + std::to_string(rtc_minor) + "|hip " + std::to_string(runtime) + "|file v2";
    return salt;
}

std::string cache_path(const std::string& source, const std::string& arch) {
    const std::string dir = cache_dir();
    if (dir.empty()) return "";
    const std::string salt = cache_salt(arch);
    char name[64];
    std::snprintf(name, sizeof name, "%016llx%016llx.co", (unsigned long long)fnv1a(source + salt, 1469598103934665603ull),
                  (unsigned long long)fnv1a(salt + source, 0x9e3779b97f4a7c15ull));
    return dir + "/" + name;
}

// Cache file = 24-byte header (magic, payload length, FNV-1a of the payload) + the code object.  A file is used only
// if the header matches what follows it and the payload is an AMDGPU ELF image; anything else (a truncated write, a
// file from another tool, bit rot) is deleted and counted as rejected.
constexpr char kCacheMagic[8] = {'D', 'S', 'C', 'C', 'O', 'B', 'J', '2'};
constexpr size_t kCacheHeader = 24;

uint64_t fnv1a_bytes(const char* p, size_t n) {
    uint64_t h = 1469598103934665603ull;
    for (size_t i = 0; i < n; ++i) {
        h ^= (unsigned char)p[i];
        h *= 1099511628211ull;
    }
    return h;
}

bool plausible_code_object(const char* p, size_t n) {
    // ELF64 little-endian, e_machine EM_AMDGPU (224), section header table inside the file
    if (n < 64 || std::memcmp(p, "\177ELF", 4) != 0 || p[4] != 2 || p[5] != 1) return false;
    uint16_t machine, shentsize, shnum;
    uint64_t shoff;
    std::memcpy(&machine, p + 18, 2);
    std::memcpy(&shoff, p + 40, 8);
    std::memcpy(&shentsize, p + 58, 2);
    std::memcpy(&shnum, p + 60, 2);
    if (machine != 224) return false;
    return shoff <= n && (uint64_t)shentsize * shnum <= n - shoff;
}

bool read_cache_file(const std::string& path, std::vector<char>* code) {
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    std::vector<char> all((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
    uint64_t length = 0, hash = 0;
    bool ok = all.size() > kCacheHeader && std::memcmp(all.data(), kCacheMagic, 8) == 0;
    if (ok) {
        std::memcpy(&length, all.data() + 8, 8);
        std::memcpy(&hash, all.data() + 16, 8);
        ok = length == all.size() - kCacheHeader && hash == fnv1a_bytes(all.data() + kCacheHeader, (size_t)length) &&
             plausible_code_object(all.data() + kCacheHeader, (size_t)length);
    }
    if (!ok) {
        f.close();
        std::remove(path.c_str());
        ++g_cache_stats.rejected;
        return false;
    }
    code->assign(all.begin() + kCacheHeader, all.end());
    return true;
}

void write_cache_file(const std::string& path, const std::vector<char>& code) {
    const std::string tmp = path + ".tmp" + std::to_string((long long)::getpid());
    std::ofstream f(tmp, std::ios::binary);
    if (!f) return;
    const uint64_t length = code.size(), hash = fnv1a_bytes(code.data(), code.size());
    f.write(kCacheMagic, 8);
    f.write(reinterpret_cast<const char*>(&length), 8);
    f.write(reinterpret_cast<const char*>(&hash), 8);
    f.write(code.data(), (std::streamsize)code.size());
    f.close();
    if (!f || std::rename(tmp.c_str(), path.c_str()) != 0) std::remove(tmp.c_str());
}

}  // namespace

const CacheStats& cache_stats() { return g_cache_stats; }

void drop_cached_object(const std::string& source, const std::string& arch) {
    const std::string path = cache_path(source, arch);
    if (path.empty()) return;
    if (std::remove(path.c_str()) == 0) ++g_cache_stats.rejected;
}

int compile_source(const std::string& source, const std::string& arch, std::vector<char>* code, std::string* log, bool* from_cache) {
    if (from_cache) *from_cache = false;
    const std::string path = cache_path(source, arch);
    if (!path.empty() && read_cache_file(path, code)) {
        ++g_cache_stats.hits;
        if (from_cache) *from_cache = true;
        return DSC_OK;
    }
    ++g_cache_stats.compiles;
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, source.c_str(), "dsc_kernel.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS)
        return fail(DSC_ERR_COMPILE, "hiprtcCreateProgram failed");
    std::vector<std::string> opts;
    opts.push_back("--offload-arch=" + arch);
    for (auto& o : compile_options()) opts.push_back(o);
    std::vector<const char*> copts;
    for (auto& o : opts) copts.push_back(o.c_str());
    hiprtcResult r = hiprtcCompileProgram(prog, (int)copts.size(), copts.data());
    size_t log_size = 0;
    hiprtcGetProgramLogSize(prog, &log_size);
    std::string text(log_size, '\0');
    if (log_size) hiprtcGetProgramLog(prog, &text[0]);
    if (log) *log = text;
    if (r != HIPRTC_SUCCESS) {
        hiprtcDestroyProgram(&prog);
        return fail(DSC_ERR_COMPILE, std::string("hipRTC: ") + hiprtcGetErrorString(r) + "\n" + text);
    }
    size_t code_size = 0;
    hiprtcGetCodeSize(prog, &code_size);
    code->resize(code_size);
    hiprtcGetCode(prog, code->data());
    hiprtcDestroyProgram(&prog);
    if (!path.empty()) write_cache_file(path, *code);
    return DSC_OK;
}

namespace {

// Loads a code object and looks up the entry point.
hipError_t load_module(const std::vector<char>& code, const std::string& entry, hipModule_t* module, hipFunction_t* function, const char** what) {
    *what = "hipModuleLoadData";
    hipError_t e = hipModuleLoadData(module, code.data());
    if (e != hipSuccess) return e;
    *what = "hipModuleGetFunction";
    e = hipModuleGetFunction(function, *module, entry.c_str());
    if (e != hipSuccess) {
        (void)hipModuleUnload(*module);
        *module = nullptr;
    }
    return e;
}

}  // namespace

Kernel* get_kernel(Context* ctx, const FusedKernel& fk, int* status) {
    const std::string key = fk.key();
    auto it = ctx->kernels.find(key);
    if (it != ctx->kernels.end()) {
        *status = DSC_OK;
        return it->second.get();
    }
    auto k = std::make_unique<Kernel>();
    k->fused = fk;
    std::string err = generate(fk, &k->gen);
    if (!err.empty()) {
        *status = fail(err.find("too large") != std::string::npos ? DSC_ERR_UNSUPPORTED : DSC_ERR_INVALID, err);
        return nullptr;
    }
    k->label = label_name(fk.main.raw());
    if (!fk.row_stages.empty())
        k->label = "RowFused [" + std::to_string((long long)fk.row_m) + ", " + std::to_string((long long)fk.row_n) + "] (" +
                   std::to_string(fk.row_stages.size()) + " clusters)";
    if (fk.dgrad.on) {
        const auto& c = fk.dgrad;
        char text[160];
        std::snprintf(text, sizeof text, "%s [%lld, %lld, %lld, %lld] %lldx%lld taps, %lld groups", c.wgrad_only ? "ConvFilterGrad" : c.wgrad ? "ConvBackward" : "ConvDataGrad", (long long)c.img,
                      (long long)(c.oh + c.fh - 1 - 2 * c.pad_h), (long long)(c.ow + c.fw - 1 - 2 * c.pad_w), (long long)(c.g * c.c),
                      (long long)c.fh, (long long)c.fw, (long long)c.g);
        k->label = text;
    }
    if (fk.cfwd.on) {
        const auto& c = fk.cfwd;
        char text[160];
        std::snprintf(text, sizeof text, "ConvForward [%lld, %lld, %lld, %lld] %lldx%lld taps, %lld groups", (long long)c.img, (long long)c.oh,
                      (long long)c.ow, (long long)(c.g * matmul_dims(fk.main.raw()).n), (long long)c.fh, (long long)c.fw, (long long)c.g);
        k->label = text;
    }
    if (fk.has_epilogue) k->label += " + " + label_name(fk.epilogue.raw());
    if (!fk.virtuals.empty()) k->label += " <" + std::to_string(fk.virtuals.size()) + " fused producers>";
    if (!fk.parts.empty()) {
        k->label = "Multi (" + std::to_string(fk.parts.size()) + " kernels:";
        for (auto& part : fk.parts)
            k->label += " " + std::string(part.dgrad.on ? (part.dgrad.wgrad_only ? "ConvFilterGrad" : part.dgrad.wgrad ? "ConvBackward" : "ConvDataGrad") : part.cfwd.on ? "ConvForward" : part.row_stages.empty() ? label_name(part.main.raw()) : "RowFused") + ";";
        k->label += ")";
    }
    k->reference_groups = reference_group_count(fk.main.raw());
    if (const char* dump = std::getenv("DSC_DUMP_DIR")) {  // debugging aid: one source file per generated kernel
        std::ofstream f(std::string(dump) + "/kernel_" + std::to_string(ctx->kernels.size()) + ".hip");
        if (f) f << "// " << k->label << "\n// " << k->gen.note << "\n" << k->gen.source;
    }
    std::vector<char> code;
    std::string log;
    bool from_cache = false;
    int rc = compile_source(k->gen.source, ctx->arch, &code, &log, &from_cache);
    if (rc != DSC_OK) {
        *status = rc;
        return nullptr;
    }
    if (ctx->offline) {
        Kernel* raw_offline = k.get();
        ctx->kernels[key] = std::move(k);
        *status = DSC_OK;
        return raw_offline;
    }
    const char* what = "";
    hipError_t e = load_module(code, k->gen.entry, &k->module, &k->function, &what);
    if (e != hipSuccess && from_cache) {
        // the cached object passed the file checks and the runtime still refuses it: drop it and compile afresh, once
        (void)hipGetLastError();
        drop_cached_object(k->gen.source, ctx->arch);
        rc = compile_source(k->gen.source, ctx->arch, &code, &log, &from_cache);
        if (rc != DSC_OK) {
            *status = rc;
            return nullptr;
        }
        e = load_module(code, k->gen.entry, &k->module, &k->function, &what);
    }
    if (e != hipSuccess) {
        *status = fail(DSC_ERR_HIP, std::string(what) + ": " + hipGetErrorString(e));
        return nullptr;
    }
    if (k->gen.persistent_ok) {
        // as many workgroups as the device holds at once (a multiple of the 8 XCDs), never more than the units
        int per_cu = 0;
        e = hipModuleOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, k->function, (int)k->gen.block, 0);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            per_cu = 0;
        }
        const int64_t resident = (int64_t)per_cu * ctx->caps.compute_units / 8 * 8;
        if (resident >= 8 && resident < (int64_t)k->gen.grid) k->gen.grid = (unsigned)resident;
    }
    Kernel* raw = k.get();
    ctx->kernels[key] = std::move(k);
    *status = DSC_OK;
    return raw;
}

int set_seed(Context* ctx, uint32_t rand_seed) {
    if (ctx->seed_known && ctx->seed_value == rand_seed) return DSC_OK;
    HIP_TRY(hipMemsetD32Async(reinterpret_cast<hipDeviceptr_t>(ctx->seed_cell), (int)rand_seed, 1, ctx->stream));
    ctx->seed_value = rand_seed;
    ctx->seed_known = true;
    return DSC_OK;
}

hipEvent_t take_plain_event(Context* ctx) {
    hipEvent_t ev = nullptr;
    if (!ctx->fence_pool.empty()) {
        ev = ctx->fence_pool.back();
        ctx->fence_pool.pop_back();
        return ev;
    }
    if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return ev;
}

int load_markers(Context* ctx) {
    if (ctx->range_push && ctx->range_pop) return DSC_OK;
    static void* roctx = [] {
        void* h = dlopen("librocprofiler-sdk-roctx.so.1", RTLD_NOW | RTLD_GLOBAL);
        if (!h) h = dlopen("librocprofiler-sdk-roctx.so", RTLD_NOW | RTLD_GLOBAL);
        if (!h) h = dlopen("libroctx64.so.4", RTLD_NOW | RTLD_GLOBAL);
        return h;
    }();
    if (!roctx) return fail(DSC_ERR_UNSUPPORTED, "no ROCTx library (librocprofiler-sdk-roctx.so, libroctx64.so) could be loaded");
    ctx->range_push = reinterpret_cast<int (*)(const char*)>(dlsym(roctx, "roctxRangePushA"));
    ctx->range_pop = reinterpret_cast<int (*)()>(dlsym(roctx, "roctxRangePop"));
    if (!ctx->range_push || !ctx->range_pop) {
        ctx->range_push = nullptr;
        ctx->range_pop = nullptr;
        return fail(DSC_ERR_UNSUPPORTED, "the ROCTx library lacks roctxRangePushA / roctxRangePop");
    }
    return DSC_OK;
}

int enable_async_io(Context* ctx) {
    if (ctx->async_io) return DSC_OK;
    if (ctx->offline) return fail(DSC_ERR_NO_DEVICE, "overlapped I/O without a device");
    if (!ctx->copy_stream) HIP_TRY(hipStreamCreate(&ctx->copy_stream));
    // stamps were not kept up to date until now: start from an idle stream
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    ctx->work_done = ctx->work_seq;
    ctx->async_io = true;
    return DSC_OK;
}

namespace {
// marks whose event has fired are dropped; the last one dropped says how far the compute stream has come
void prune_marks(Context* ctx) {
    while (!ctx->marks.empty()) {
        const hipError_t e = hipEventQuery(ctx->marks.front().second);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return;
        }
        ctx->work_done = std::max(ctx->work_done, ctx->marks.front().first);
        ctx->fence_pool.push_back(ctx->marks.front().second);
        ctx->marks.pop_front();
    }
}
}  // namespace

int mark_stream(Context* ctx) {
    prune_marks(ctx);
    if (ctx->work_done >= ctx->work_seq) return DSC_OK;
    if (!ctx->marks.empty() && ctx->marks.back().first >= ctx->work_seq) return DSC_OK;
    hipEvent_t ev = take_plain_event(ctx);
    if (!ev) return fail(DSC_ERR_HIP, "hipEventCreate failed");
    const hipError_t e = hipEventRecord(ev, ctx->stream);
    if (e != hipSuccess) {
        ctx->fence_pool.push_back(ev);
        return fail(DSC_ERR_HIP, std::string("hipEventRecord: ") + hipGetErrorString(e));
    }
    ctx->marks.emplace_back(ctx->work_seq, ev);
    return DSC_OK;
}

int copy_stream_wait(Context* ctx, uint64_t stamp) {
    if (stamp <= ctx->work_done) return DSC_OK;
    prune_marks(ctx);
    if (stamp <= ctx->work_done) return DSC_OK;
    if (ctx->marks.empty() || ctx->marks.back().first < stamp) {
        const int rc = mark_stream(ctx);
        if (rc != DSC_OK) return rc;
        if (stamp <= ctx->work_done) return DSC_OK;
    }
    // The host waits, not the copy stream: memory that an upload reuses was last read two runs ago when buffers
    // alternate, so this only holds back a host that is further ahead than that -- and a queue of copies that each
    // wait in the copy stream for a compute event has measured slower than uploads on the compute stream itself.
    for (auto& m : ctx->marks) {
        if (m.first >= stamp) {
            HIP_TRY(hipEventSynchronize(m.second));
            prune_marks(ctx);
            return DSC_OK;
        }
    }
    return fail(DSC_ERR_INVALID, "no mark covers a buffer's last use");
}

int join_copies(Context* ctx) {
    if (ctx->copies.empty()) return DSC_OK;
    for (auto& cp : ctx->copies) {
        hipEvent_t ev = cp.own;
        if (!ev) {
            auto it = ctx->fences.find(cp.fence);
            if (it == ctx->fences.end()) continue;  // waited for and retired: the copy has finished
            ev = it->second.event;
        }
        // a copy that has already finished needs no barrier in the compute queue
        if (hipEventQuery(ev) != hipSuccess) {
            (void)hipGetLastError();
            HIP_TRY(hipStreamWaitEvent(ctx->stream, ev, 0));
        }
        if (cp.own) ctx->fence_pool.push_back(cp.own);
        cp.own = nullptr;
    }
    ctx->copies.clear();
    return DSC_OK;
}

int launch_kernel(Context* ctx, Kernel* k, void* const* device_ptrs, int n, uint32_t rand_seed) {
    if (ctx->offline || !k->function) return fail(DSC_ERR_NO_DEVICE, "kernel launch without a device");
    if (n != k->gen.n_buffers)
        return fail(DSC_ERR_INVALID, "kernel '" + k->label + "' takes " + std::to_string(k->gen.n_buffers) + " buffers, got " +
                                         std::to_string(n));
    // 256 pointers are 2 KiB of the 4 KiB a kernel's arguments may take; a launch shared by many chains binds the most
    void* ptr_values[256];
    void* args[258];
    if (n > 256) return fail(DSC_ERR_UNSUPPORTED, "more than 256 buffers bound to one kernel");
    for (int i = 0; i < n; ++i) {
        ptr_values[i] = device_ptrs[i];
        args[i] = &ptr_values[i];
    }
    void* seed_ptr = ctx->seed_through_cell ? ctx->seed_cell : nullptr;
    uint32_t seed_value = rand_seed;
    args[n] = &seed_ptr;
    args[n + 1] = &seed_value;
    hipEvent_t start = nullptr, stop = nullptr;
    if (ctx->profiling) {
        auto take = [&](hipEvent_t* ev) -> hipError_t {
            if (!ctx->event_pool.empty()) {
                *ev = ctx->event_pool.back();
                ctx->event_pool.pop_back();
                return hipSuccess;
            }
            return hipEventCreate(ev);
        };
        HIP_TRY(take(&start));
        HIP_TRY(take(&stop));
        HIP_TRY(hipEventRecord(start, ctx->stream));
    }
    if (ctx->range_push) (void)ctx->range_push(k->label.c_str());
    const hipError_t launched = hipModuleLaunchKernel(k->function, k->gen.grid, 1, 1, k->gen.block, 1, 1, 0, ctx->stream, args, nullptr);
    if (ctx->range_pop) (void)ctx->range_pop();
    if (launched != hipSuccess) return fail(DSC_ERR_HIP, "hipModuleLaunchKernel '" + k->label + "': " + hipGetErrorString(launched));
    ++ctx->work_seq;
    if (ctx->profiling) {
        HIP_TRY(hipEventRecord(stop, ctx->stream));
        ctx->profile.push_back(ProfileEntry{start, stop, k});
    }
    return DSC_OK;
}

}  // namespace dsc
