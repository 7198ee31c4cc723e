// Device runtime behind the C ABI: context + stream, arena heap, pinned staging, hipRTC kernel cache,
// event profiler.  Replaces the reference's Vulkan device layer (src/device/*.rs).
#pragma once

#include "codegen.hpp"

#include <hip/hip_runtime.h>

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

namespace dsc {

void set_error(const std::string& msg);
const std::string& last_error();
int fail(int status, const std::string& msg);

// Sub-allocator over large hipMalloc'd chunks (reference: BufferHeap over 256 MiB Vulkan chunks,
// device/buffer_heap.rs:29-110, with the free-list heap of device/heap.rs).  Best fit over an ordered set of
// free ranges, split on allocation, coalescing with both neighbours on free, 256-byte alignment.
class DeviceHeap {
  public:
    static constexpr size_t kAlign = 256;
    static constexpr size_t kChunkBytes = size_t(1) << 30;  // sized for 288 GB of HBM: few, large chunks

    ~DeviceHeap();
    // returns 0 when the device cannot provide the memory
    uint64_t alloc(size_t bytes);
    bool free(uint64_t handle);
    bool info(uint64_t handle, void** ptr, size_t* bytes) const;
    void stats(int64_t* live, int64_t* live_bytes, int64_t* arena_bytes) const;

  private:
    struct Block {
        size_t size;
        bool is_free;
    };
    struct Chunk {
        char* base = nullptr;
        size_t size = 0;
        std::map<size_t, Block> blocks;  // by offset
    };
    struct Live {
        int chunk;
        size_t offset;
        size_t bytes;  // requested size
    };
    std::vector<Chunk> chunks_;
    std::multimap<size_t, std::pair<int, size_t>> free_by_size_;  // size -> (chunk, offset)
    std::unordered_map<uint64_t, Live> live_;
    uint64_t next_handle_ = 1;
    int64_t live_bytes_ = 0;

    void add_free(int chunk, size_t offset, size_t size);
    void remove_free(int chunk, size_t offset, size_t size);
};

struct Kernel {
    FusedKernel fused;
    Generated gen;
    std::string label;
    hipModule_t module = nullptr;
    hipFunction_t function = nullptr;
    int64_t reference_groups = 0;
};

struct ProfileEntry {
    hipEvent_t start, stop;
    const Kernel* kernel;
};

struct Context {
    int device = 0;
    bool offline = false;  // no GPU: kernels are generated and compiled, never loaded or launched
    hipStream_t stream = nullptr;
    std::string arch;
    dsc_caps caps{};
    DeviceHeap heap;

    // pinned staging ring (reference: 2 x 4 MiB host-visible regions gated by fences, device/staging.rs:337-338)
    static constexpr int kStagingRegions = 2;
    static constexpr size_t kStagingBytes = size_t(16) << 20;
    char* staging[kStagingRegions] = {nullptr, nullptr};
    hipEvent_t staging_done[kStagingRegions] = {nullptr, nullptr};
    bool staging_busy[kStagingRegions] = {false, false};
    int staging_next = 0;

    // Launches take the rand seed by value.  While `seed_through_cell` is set (a schedule capturing or replaying a
    // HIP graph) they are given this one device word instead, which set_seed fills before the graph runs.
    bool seed_through_cell = false;
    uint32_t* seed_cell = nullptr;
    uint32_t seed_value = 0;
    bool seed_known = false;

    std::unordered_map<std::string, std::unique_ptr<Kernel>> kernels;  // by FusedKernel::key()

    // fences: id -> event recorded on the stream; ids at or below `fence_retired` are known to have finished
    std::map<uint64_t, hipEvent_t> fences;
    std::vector<hipEvent_t> fence_pool;
    uint64_t fence_next = 1, fence_retired = 0;

    bool profiling = false;
    std::vector<ProfileEntry> profile;
    std::vector<hipEvent_t> event_pool;

    ~Context();
};

// Compiles (or fetches) the kernel for a fused descriptor.  Returns nullptr and sets the error on failure.
Kernel* get_kernel(Context* ctx, const FusedKernel& fk, int* status);
int launch_kernel(Context* ctx, Kernel* k, void* const* device_ptrs, int n, uint32_t rand_seed);
// Makes `rand_seed` the seed seen by launches enqueued after this call.
int set_seed(Context* ctx, uint32_t rand_seed);
// hipRTC compile without a device.
int compile_source(const std::string& source, const std::string& arch, std::vector<char>* code, std::string* log);

}  // namespace dsc
