#include "runtime.hpp"

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

void DeviceHeap::add_free(int chunk, size_t offset, size_t size) { free_by_size_.emplace(size, std::make_pair(chunk, offset)); }

void DeviceHeap::remove_free(int chunk, size_t offset, size_t size) {
    auto range = free_by_size_.equal_range(size);
    for (auto it = range.first; it != range.second; ++it) {
        if (it->second.first == chunk && it->second.second == offset) {
            free_by_size_.erase(it);
            return;
        }
    }
}

uint64_t DeviceHeap::alloc(size_t bytes) {
    const size_t need = std::max(kAlign, (bytes + kAlign - 1) / kAlign * kAlign);
    auto it = free_by_size_.lower_bound(need);
    if (it == free_by_size_.end()) {
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
        c.blocks[0] = Block{c.size, true};
        chunks_.push_back(std::move(c));
        add_free((int)chunks_.size() - 1, 0, chunks_.back().size);
        it = free_by_size_.lower_bound(need);
    }
    const int ci = it->second.first;
    const size_t off = it->second.second;
    const size_t have = it->first;
    free_by_size_.erase(it);
    Chunk& c = chunks_[ci];
    c.blocks[off] = Block{need, false};
    if (have > need) {
        c.blocks[off + need] = Block{have - need, true};
        add_free(ci, off + need, have - need);
    }
    const uint64_t h = next_handle_++;
    live_[h] = Live{ci, off, bytes};
    live_bytes_ += (int64_t)need;
    return h;
}

bool DeviceHeap::free(uint64_t handle) {
    auto lit = live_.find(handle);
    if (lit == live_.end()) return false;
    const int ci = lit->second.chunk;
    size_t off = lit->second.offset;
    live_.erase(lit);
    Chunk& c = chunks_[ci];
    auto it = c.blocks.find(off);
    size_t size = it->second.size;
    live_bytes_ -= (int64_t)size;
    // coalesce with the next range, then with the previous one
    auto next = std::next(it);
    if (next != c.blocks.end() && next->second.is_free) {
        remove_free(ci, next->first, next->second.size);
        size += next->second.size;
        c.blocks.erase(next);
    }
    if (it != c.blocks.begin()) {
        auto prev = std::prev(it);
        if (prev->second.is_free) {
            remove_free(ci, prev->first, prev->second.size);
            size += prev->second.size;
            off = prev->first;
            c.blocks.erase(it);
            it = prev;
        }
    }
    it->second = Block{size, true};
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
    if (stream) (void)hipStreamSynchronize(stream);
    for (auto& kv : kernels)
        if (kv.second->module) (void)hipModuleUnload(kv.second->module);
    for (auto& p : profile) {
        (void)hipEventDestroy(p.start);
        (void)hipEventDestroy(p.stop);
    }
    for (auto e : event_pool) (void)hipEventDestroy(e);
    for (auto& kv : fences) (void)hipEventDestroy(kv.second);
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

std::string cache_path(const std::string& source, const std::string& arch) {
    const std::string dir = cache_dir();
    if (dir.empty()) return "";
    std::string salt = arch;
    for (auto& o : compile_options()) salt += "|" + o;
    char name[64];
    std::snprintf(name, sizeof name, "%016llx%016llx.co", (unsigned long long)fnv1a(source + salt, 1469598103934665603ull),
                  (unsigned long long)fnv1a(salt + source, 0x9e3779b97f4a7c15ull));
    return dir + "/" + name;
}

}  // namespace

int compile_source(const std::string& source, const std::string& arch, std::vector<char>* code, std::string* log) {
    const std::string path = cache_path(source, arch);
    if (!path.empty()) {
        std::ifstream f(path, std::ios::binary);
        if (f) {
            code->assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
            if (!code->empty()) return DSC_OK;
        }
    }
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
    if (!path.empty()) {
        const std::string tmp = path + ".tmp" + std::to_string((long long)::getpid());
        std::ofstream f(tmp, std::ios::binary);
        if (f) {
            f.write(code->data(), (std::streamsize)code->size());
            f.close();
            if (std::rename(tmp.c_str(), path.c_str()) != 0) std::remove(tmp.c_str());
        }
    }
    return DSC_OK;
}

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
        std::snprintf(text, sizeof text, "ConvDataGrad [%lld, %lld, %lld, %lld] %lldx%lld taps, %lld groups", (long long)c.img,
                      (long long)(c.oh + c.fh - 1 - 2 * c.pad_h), (long long)(c.ow + c.fw - 1 - 2 * c.pad_w), (long long)(c.g * c.c),
                      (long long)c.fh, (long long)c.fw, (long long)c.g);
        k->label = text;
    }
    if (fk.has_epilogue) k->label += " + " + label_name(fk.epilogue.raw());
    if (!fk.virtuals.empty()) k->label += " <" + std::to_string(fk.virtuals.size()) + " fused producers>";
    if (!fk.parts.empty()) {
        k->label = "Multi (" + std::to_string(fk.parts.size()) + " kernels:";
        for (auto& part : fk.parts)
            k->label += " " + std::string(part.dgrad.on ? "ConvDataGrad" : part.row_stages.empty() ? label_name(part.main.raw()) : "RowFused") + ";";
        k->label += ")";
    }
    k->reference_groups = reference_group_count(fk.main.raw());
    if (const char* dump = std::getenv("DSC_DUMP_DIR")) {  // debugging aid: one source file per generated kernel
        std::ofstream f(std::string(dump) + "/kernel_" + std::to_string(ctx->kernels.size()) + ".hip");
        if (f) f << "// " << k->label << "\n// " << k->gen.note << "\n" << k->gen.source;
    }
    std::vector<char> code;
    std::string log;
    int rc = compile_source(k->gen.source, ctx->arch, &code, &log);
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
    hipError_t e = hipModuleLoadData(&k->module, code.data());
    if (e != hipSuccess) {
        *status = fail(DSC_ERR_HIP, std::string("hipModuleLoadData: ") + hipGetErrorString(e));
        return nullptr;
    }
    e = hipModuleGetFunction(&k->function, k->module, k->gen.entry.c_str());
    if (e != hipSuccess) {
        *status = fail(DSC_ERR_HIP, std::string("hipModuleGetFunction: ") + hipGetErrorString(e));
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

int launch_kernel(Context* ctx, Kernel* k, void* const* device_ptrs, int n, uint32_t rand_seed) {
    if (ctx->offline || !k->function) return fail(DSC_ERR_NO_DEVICE, "kernel launch without a device");
    if (n != k->gen.n_buffers)
        return fail(DSC_ERR_INVALID, "kernel '" + k->label + "' takes " + std::to_string(k->gen.n_buffers) + " buffers, got " +
                                         std::to_string(n));
    void* ptr_values[64];
    void* args[66];
    if (n > 64) return fail(DSC_ERR_UNSUPPORTED, "more than 64 buffers bound to one kernel");
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
    HIP_TRY(hipModuleLaunchKernel(k->function, k->gen.grid, 1, 1, k->gen.block, 1, 1, 0, ctx->stream, args, nullptr));
    if (ctx->profiling) {
        HIP_TRY(hipEventRecord(stop, ctx->stream));
        ctx->profile.push_back(ProfileEntry{start, stop, k});
    }
    return DSC_OK;
}

}  // namespace dsc
