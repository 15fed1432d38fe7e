// Devices, memory, streams, host<->device copies.
// Replaces the reference's src/cuda/mem.cu, src/cuda/streams.cu and
// src/cuda/exc.cuh; cited per function in include/tannic_hip.h.
#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "common.hpp"

namespace th {

static thread_local std::string g_last_error;

void set_error(const char* what, const char* file, int line, hipError_t code) {
    char buf[512];
    std::snprintf(buf, sizeof buf, "HIP error at %s:%d code=%d(%s) in '%s'", file, line, static_cast<int>(code),
                  hipGetErrorString(code), what);
    g_last_error = buf;
}

void set_error_text(const char* text) { g_last_error = text; }

// Per-device LIFO pool of streams (src/cuda/streams.cu:23-38).  With one host
// thread the pool hands the same stream back every time, so consecutive
// operator calls are ordered; a mutex makes concurrent callers safe, which the
// reference's pool is not.
class Streams {
   public:
    static Streams& instance() {
        static Streams s;
        return s;
    }
    hipStream_t pop(int device) {
        std::lock_guard<std::mutex> lock(mutex_);
        if (device < 0) return nullptr;
        if (static_cast<size_t>(device) >= pools_.size()) pools_.resize(device + 1);
        auto& pool = pools_[device];
        if (!pool.empty()) {
            hipStream_t s = pool.back();
            pool.pop_back();
            return s;
        }
        hipStream_t s = nullptr;
        // default flags: ordered against the legacy stream like the reference's
        // cudaStreamCreate; default priority
        if (hipStreamCreate(&s) != hipSuccess) return nullptr;
        return s;
    }
    void put(int device, hipStream_t s) {
        std::lock_guard<std::mutex> lock(mutex_);
        if (device < 0) return;
        if (static_cast<size_t>(device) >= pools_.size()) pools_.resize(device + 1);
        pools_[device].push_back(s);
    }

   private:
    std::mutex mutex_;
    std::vector<std::vector<hipStream_t>> pools_;
};

// Keep freed blocks in the device's pool instead of returning them to the
// driver: the front end allocates one temporary per operator node.
static void retain_pool_memory(int device) {
    static std::mutex m;
    static std::vector<bool> done;
    std::lock_guard<std::mutex> lock(m);
    if (static_cast<size_t>(device) >= done.size()) done.resize(device + 1, false);
    if (done[device]) return;
    done[device] = true;
    hipMemPool_t pool;
    if (hipDeviceGetDefaultMemPool(&pool, device) == hipSuccess) {
        uint64_t threshold = UINT64_MAX;
        (void)hipMemPoolSetAttribute(pool, hipMemPoolAttrReleaseThreshold, &threshold);
    }
    (void)hipGetLastError();
}

// Work scratch of the kernels (partial results, rearranged weights, flags).
// Blocks are kept per stream and handed out again to later calls on the SAME
// stream: stream order already separates the kernels of the earlier call from
// those of the later one, so no allocation and no free sits on the hot path.
struct ScratchBlock {
    void* ptr;
    size_t size;
    hipStream_t stream;
    int device;
    int pins = 0;      // recorded graphs whose kernels hold this address: never freed while one of them lives
};

// A recorded sequence of backend calls (a HIP graph) and the memory its kernels address.  Tensor blocks allocated while
// recording belong to the recording until it is destroyed: released, they wait in `idle` for the recording's own later
// requests and never reach the blocks kept for everybody, so no tensor outside the graph can share an address with one
// of its temporaries.
struct Recording {
    uint64_t id = 0;
    int device = 0;
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    bool capturing = false;
    std::vector<void*> scratch;
};
static Recording* g_capturing = nullptr;   // at most one at a time, guarded by g_scratch_mutex and g_mem_mutex alike (set with both held)
static std::mutex g_scratch_mutex;
static std::vector<ScratchBlock> g_scratch_free, g_scratch_live;
static size_t g_scratch_cached = 0;
constexpr size_t kScratchCacheLimit = size_t(2) << 30;

void release_idle_memory();   // defined below, next to the kept tensor blocks

// Whether some stream is being recorded right now: memory must not go back to the driver then (a stream-ordered free on
// the capturing stream would become a node of the graph, a wait for the device would end the capture).
static bool recording_open() {
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    return g_capturing && g_capturing->capturing;
}

// With g_scratch_mutex held: a block handed out while `stream` is being recorded is addressed by the graph's kernels.
static void pin_for_recording(ScratchBlock& b, hipStream_t stream) {
    if (!g_capturing || !g_capturing->capturing || g_capturing->stream != stream) return;
    for (void* seen : g_capturing->scratch)
        if (seen == b.ptr) return;
    g_capturing->scratch.push_back(b.ptr);
    b.pins += 1;
}

std::atomic<uint64_t> g_counters[kCounters];
void count(Counter which, uint64_t value, bool set) {
    if (set) g_counters[which].store(value, std::memory_order_relaxed);
    else g_counters[which].fetch_add(value, std::memory_order_relaxed);
}

int scratch_acquire(void** ptr, size_t nbytes, hipStream_t stream) {
    count(kCounterScratchAcquired, 1);
    int device = 0;
    TH_TRY(hipGetDevice(&device));
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        size_t best = g_scratch_free.size();
        for (size_t i = 0; i < g_scratch_free.size(); ++i) {
            const ScratchBlock& b = g_scratch_free[i];
            if (b.stream == stream && b.device == device && b.size >= nbytes && (best == g_scratch_free.size() || b.size < g_scratch_free[best].size)) best = i;
        }
        if (best != g_scratch_free.size()) {
            ScratchBlock b = g_scratch_free[best];
            g_scratch_free.erase(g_scratch_free.begin() + best);
            g_scratch_cached -= b.size;
            pin_for_recording(b, stream);
            g_scratch_live.push_back(b);
            *ptr = b.ptr;
            return TANNIC_SUCCESS;
        }
    }
    const size_t size = ((nbytes + 0xFFFF) & ~size_t(0xFFFF)) ? ((nbytes + 0xFFFF) & ~size_t(0xFFFF)) : 0x10000;
    hipError_t err = hipMalloc(ptr, size);
    if (err == hipErrorOutOfMemory && !recording_open()) {
        // Idle memory the library itself holds may be all that is missing: the cached scratch blocks and the tensor
        // blocks kept for reuse go back to the driver (once every stream has passed their last use), then one more try.
        // Not while a recording is open: the frees would be issued on, and the wait would break, the capturing stream.
        (void)hipGetLastError();
        release_idle_memory();
        err = hipMalloc(ptr, size);
    }
    if (err != hipSuccess) {
        set_error("hipMalloc (kernel scratch)", __FILE__, __LINE__, err);
        return TANNIC_ERROR;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    ScratchBlock fresh{*ptr, size, stream, device};
    pin_for_recording(fresh, stream);
    g_scratch_live.push_back(fresh);
    return TANNIC_SUCCESS;
}

int scratch_release(void* ptr, hipStream_t stream) {
    ScratchBlock block{nullptr, 0, stream, 0};
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        for (size_t i = 0; i < g_scratch_live.size(); ++i)
            if (g_scratch_live[i].ptr == ptr) {
                block = g_scratch_live[i];
                g_scratch_live.erase(g_scratch_live.begin() + i);
                break;
            }
        if (block.ptr && (block.pins > 0 || g_scratch_cached + block.size <= kScratchCacheLimit)) {
            g_scratch_free.push_back(block);
            g_scratch_cached += block.size;
            return TANNIC_SUCCESS;
        }
    }
    // over the cache limit (or unknown pointer): the block came from hipMalloc, so it goes back with hipFree, once the
    // stream has passed the kernels that used it
    TH_TRY(hipStreamSynchronize(stream));
    TH_TRY(hipFree(ptr));
    return TANNIC_SUCCESS;
}

bool refuses_while_recording(hipStream_t stream, const char* call) {
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (!g_capturing || !g_capturing->capturing || (stream && g_capturing->stream != stream)) return false;
    }
    std::string text = std::string(call) + ": waits for the stream, which is being recorded into a graph; end the recording first";
    set_error_text(text.c_str());
    return true;
}

}  // namespace th

using namespace th;

extern "C" {

const char* tannic_hip_last_error(void) { return g_last_error.c_str(); }

const char* tannic_hip_arch(void) { return "gfx950"; }

int tannic_hip_get_device_count(void) {
    int count = 0;
    hipError_t err = hipGetDeviceCount(&count);
    if (err != hipSuccess) {
        set_error("hipGetDeviceCount", __FILE__, __LINE__, err);
        return -1;
    }
    return count;
}

int tannic_hip_set_device(int id) {
    TH_TRY(hipSetDevice(id));
    return TANNIC_SUCCESS;
}

// The front end allocates a destination per operator node and drops it soon after.  A released block is kept,
// tagged with the stream it was allocated and released on, and handed to the next request of a fitting size on that
// SAME stream: the stream's order already separates the old user's kernels from the new user's, so neither a
// stream-ordered free nor an allocation has to be queued between two kernels.  Requests that find no block, and
// blocks that push the kept total over the limit, go to hipMallocAsync / hipFreeAsync.
namespace {
struct MemBlock {
    size_t size;
    hipStream_t stream;
    int device;
    uint64_t recording = 0;   // the recorded graph that owns the block (0: nobody)
    bool plain = false;       // from hipMalloc (allocated while a stream was being recorded), not from the stream-ordered pool
};
struct FreeBlock {
    void* ptr;
    MemBlock info;
};
std::mutex g_mem_mutex;
std::unordered_map<void*, MemBlock> g_mem_live;
std::vector<FreeBlock> g_mem_free;     // oldest first
size_t g_mem_kept = 0;
std::unordered_map<uint64_t, std::vector<FreeBlock>> g_recording_idle;   // per living recording: its released blocks
uint64_t g_recording_ids = 0;

// Returns a block to the driver: stream-ordered for the pool's blocks; a hipMalloc block once its stream has passed it.
void free_block(const FreeBlock& f) {
    hipError_t err;
    if (f.info.plain) {
        err = hipStreamSynchronize(f.info.stream);
        if (err == hipSuccess) err = hipFree(f.ptr);
    } else {
        err = hipFreeAsync(f.ptr, f.info.stream);
    }
    if (err != hipSuccess) set_error(f.info.plain ? "hipFree" : "hipFreeAsync", __FILE__, __LINE__, err);
}

bool fits(const MemBlock& b, size_t size) { return b.size >= size && b.size <= size + size / 4; }
constexpr size_t kMemKeepLimit = size_t(48) << 30;

size_t block_size(size_t nbytes) {
    if (nbytes == 0) nbytes = 1;
    const size_t grain = nbytes < (size_t(1) << 20) ? 512 : (size_t(2) << 20);
    return (nbytes + grain - 1) / grain * grain;
}

// Gives every tensor block kept for reuse back to the pool (stream-ordered: each after its stream's last use of it).
void release_kept_blocks() {
    std::vector<FreeBlock> all;
    {
        std::lock_guard<std::mutex> lock(g_mem_mutex);
        all.swap(g_mem_free);
        g_mem_kept = 0;
    }
    for (const FreeBlock& f : all) free_block(f);
    (void)hipGetLastError();
}
}  // namespace

}  // extern "C"

// Everything idle the library holds goes back to the driver: the kept tensor blocks, the pool's cached memory and the
// cached scratch blocks.  Called when an allocation outside the pool fails for lack of memory.
void th::release_idle_memory() {
    release_kept_blocks();
    (void)hipDeviceSynchronize();
    int device = 0;
    hipMemPool_t pool;
    if (hipGetDevice(&device) == hipSuccess && hipDeviceGetDefaultMemPool(&pool, device) == hipSuccess) (void)hipMemPoolTrimTo(pool, 0);
    std::vector<ScratchBlock> idle;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        for (const ScratchBlock& b : g_scratch_free) {
            if (b.pins == 0) idle.push_back(b);
        }
        g_scratch_free.erase(std::remove_if(g_scratch_free.begin(), g_scratch_free.end(), [](const ScratchBlock& b) { return b.pins == 0; }), g_scratch_free.end());
        g_scratch_cached = 0;
        for (const ScratchBlock& b : g_scratch_free) g_scratch_cached += b.size;
    }
    for (const ScratchBlock& b : idle) (void)hipFree(b.ptr);
    (void)hipGetLastError();
}

extern "C" {

void* tannic_hip_allocate(const tannic_device_t* device, size_t nbytes) {
    count(kCounterMemoryCalls, 1);
    if (!device || tannic_hip_set_device(device->id) != TANNIC_SUCCESS) return nullptr;
    retain_pool_memory(device->id);
    Streams& streams = Streams::instance();
    hipStream_t stream = streams.pop(device->id);
    streams.put(device->id, stream);
    const size_t size = block_size(nbytes);
    uint64_t recording = 0;
    {
        std::lock_guard<std::mutex> lock(g_mem_mutex);
        if (g_capturing && g_capturing->capturing && g_capturing->stream == stream && g_capturing->device == device->id) {
            // the recording's own released blocks first: their addresses are already private to it
            recording = g_capturing->id;
            std::vector<FreeBlock>& idle = g_recording_idle[recording];
            size_t best = idle.size();
            for (size_t i = 0; i < idle.size(); ++i)
                if (fits(idle[i].info, size) && (best == idle.size() || idle[i].info.size < idle[best].info.size)) best = i;
            if (best != idle.size()) {
                const FreeBlock f = idle[best];
                idle.erase(idle.begin() + best);
                g_mem_live[f.ptr] = f.info;
                return f.ptr;
            }
        }
        size_t best = g_mem_free.size();
        for (size_t i = 0; i < g_mem_free.size(); ++i) {
            const MemBlock& b = g_mem_free[i].info;
            if (b.device != device->id || b.stream != stream || !fits(b, size)) continue;
            if (best == g_mem_free.size() || b.size < g_mem_free[best].info.size) best = i;
        }
        if (best != g_mem_free.size()) {
            FreeBlock f = g_mem_free[best];
            g_mem_free.erase(g_mem_free.begin() + best);
            g_mem_kept -= f.info.size;
            f.info.recording = recording;
            g_mem_live[f.ptr] = f.info;
            return f.ptr;
        }
    }
    void* ptr = nullptr;
    // A stream-ordered allocation on a stream that is being recorded would become a node of the graph: take the block
    // from hipMalloc instead (the recording owns it from here on).
    hipError_t err = recording ? hipMalloc(&ptr, size) : hipMallocAsync(&ptr, size, stream);
    if (err != hipSuccess && !recording) {
        // give the kept blocks back and try once more
        release_kept_blocks();
        err = hipMallocAsync(&ptr, size, stream);
    }
    if (err != hipSuccess) {
        set_error(recording ? "hipMalloc (while recording)" : "hipMallocAsync", __FILE__, __LINE__, err);
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_mem_mutex);
    g_mem_live[ptr] = MemBlock{size, stream, device->id, recording, recording != 0};
    return ptr;
}

void* tannic_hip_deallocate(const tannic_device_t* device, void* address) {
    count(kCounterMemoryCalls, 1);
    if (!device || !address) return nullptr;
    if (tannic_hip_set_device(device->id) != TANNIC_SUCCESS) return nullptr;
    Streams& streams = Streams::instance();
    hipStream_t stream = streams.pop(device->id);
    streams.put(device->id, stream);
    std::vector<FreeBlock> evict;
    bool kept = false;
    FreeBlock released{address, MemBlock{0, stream, device->id}};
    {
        std::lock_guard<std::mutex> lock(g_mem_mutex);
        auto it = g_mem_live.find(address);
        if (it != g_mem_live.end()) {
            MemBlock info = it->second;
            g_mem_live.erase(it);
            auto owner = info.recording ? g_recording_idle.find(info.recording) : g_recording_idle.end();
            if (owner != g_recording_idle.end()) {
                // the graph's kernels address this block for as long as the recording lives
                owner->second.push_back(FreeBlock{address, info});
                return nullptr;
            }
            info.recording = 0;
            released.info = info;
            // only a block released on the stream it lives on can be reused without waiting
            if (info.stream == stream && info.device == device->id && info.size <= kMemKeepLimit) {
                g_mem_free.push_back(FreeBlock{address, info});
                g_mem_kept += info.size;
                kept = true;
                // (over the limit the oldest kept blocks go back to the driver - later, if a recording is open now: see recording_open)
                const bool recording_now = g_capturing && g_capturing->capturing;
                while (!recording_now && g_mem_kept > kMemKeepLimit && !g_mem_free.empty()) {
                    evict.push_back(g_mem_free.front());
                    g_mem_kept -= g_mem_free.front().info.size;
                    g_mem_free.erase(g_mem_free.begin());
                }
            }
        }
    }
    for (const FreeBlock& f : evict) free_block(f);
    if (!kept) {
        if (released.info.plain) {
            free_block(released);
        } else {
            hipError_t err = hipFreeAsync(address, stream);
            if (err != hipSuccess) set_error("hipFreeAsync", __FILE__, __LINE__, err);
        }
    }
    return nullptr;
}

int tannic_hip_copy_from_host(const tannic_device_t* device, const void* host, void* dev, size_t nbytes) {
    if (!device) return TANNIC_NULL_ALLOCATOR;
    if (nbytes == 0) return TANNIC_SUCCESS;
    if (!host || !dev) { set_error_text("copy_from_host: null address"); return TANNIC_ERROR; }
    TH_TRY(hipSetDevice(device->id));
    Streams& streams = Streams::instance();
    hipStream_t stream = streams.pop(device->id);
    if (refuses_while_recording(stream, "copy_from_host")) {
        streams.put(device->id, stream);
        return TANNIC_ERROR;
    }
    hipError_t err = hipMemcpyAsync(dev, host, nbytes, hipMemcpyHostToDevice, stream);
    // callers pass temporaries (one element of an initializer list): the source
    // must be consumed before returning
    if (err == hipSuccess) err = hipStreamSynchronize(stream);
    streams.put(device->id, stream);
    TH_TRY(err);
    return TANNIC_SUCCESS;
}

int tannic_hip_copy_device_to_host(const tannic_device_t* device, const void* dev, void* host, size_t nbytes) {
    if (!device) return TANNIC_NULL_ALLOCATOR;
    if (nbytes == 0) return TANNIC_SUCCESS;
    if (!host || !dev) { set_error_text("copy_device_to_host: null address"); return TANNIC_ERROR; }
    TH_TRY(hipSetDevice(device->id));
    Streams& streams = Streams::instance();
    hipStream_t stream = streams.pop(device->id);
    if (refuses_while_recording(stream, "copy_device_to_host")) {
        streams.put(device->id, stream);
        return TANNIC_ERROR;
    }
    hipError_t err = hipMemcpyAsync(host, dev, nbytes, hipMemcpyDeviceToHost, stream);
    if (err == hipSuccess) err = hipStreamSynchronize(stream);
    streams.put(device->id, stream);
    TH_TRY(err);
    return TANNIC_SUCCESS;
}

int tannic_hip_compare_from_host(const tannic_device_t* device, const void* host, const void* dev, size_t nbytes) {
    if (!device || (nbytes && (!host || !dev))) return -1;
    void* buffer = std::malloc(nbytes ? nbytes : 1);
    if (!buffer) return -1;
    int rc = tannic_hip_copy_device_to_host(device, dev, buffer, nbytes);
    int equal = rc == TANNIC_SUCCESS ? (std::memcmp(host, buffer, nbytes) == 0 ? 1 : 0) : -1;
    std::free(buffer);
    return equal;
}

int tannic_hip_copy(const tannic_tensor_t* src, tannic_tensor_t* dst, size_t nbytes, tannic_stream_t s) {
    if (!src || !dst) return TANNIC_ERROR;
    if (nbytes == 0) return TANNIC_SUCCESS;
    if (!src->address || !dst->address) {
        set_error_text("copy: a tensor without storage");
        return TANNIC_ERROR;
    }
    hipStream_t stream = as_stream(s);
    const bool src_dev = src->environment.kind == TANNIC_DEVICE;
    const bool dst_dev = dst->environment.kind == TANNIC_DEVICE;
    if (src_dev != dst_dev && refuses_while_recording(stream, "copy between host and device")) return TANNIC_ERROR;
    if (!src_dev && dst_dev) {
        TH_TRY(hipMemcpyAsync(dst->address, src->address, nbytes, hipMemcpyHostToDevice, stream));
        // pageable sources behave like the reference's blocking cudaMemcpy
        if (src->environment.resource.host.traits != TANNIC_PINNED) TH_TRY(hipStreamSynchronize(stream));
    } else if (src_dev && !dst_dev) {
        TH_TRY(hipMemcpyAsync(dst->address, src->address, nbytes, hipMemcpyDeviceToHost, stream));
        if (dst->environment.resource.host.traits != TANNIC_PINNED) TH_TRY(hipStreamSynchronize(stream));
    } else if (src_dev && dst_dev) {
        TH_TRY(hipMemcpyAsync(dst->address, src->address, nbytes, hipMemcpyDeviceToDevice, stream));
    } else {
        std::memmove(dst->address, src->address, nbytes);   // host to host: the front end never asks, a caller of the C ABI may
    }
    return TANNIC_SUCCESS;
}

tannic_stream_t tannic_hip_pop_stream(const tannic_device_t* device) {
    tannic_stream_t s;
    s.address = reinterpret_cast<uintptr_t>(Streams::instance().pop(device ? device->id : 0));
    return s;
}

void tannic_hip_put_stream(const tannic_device_t* device, tannic_stream_t stream) {
    Streams::instance().put(device ? device->id : 0, as_stream(stream));
}

int tannic_hip_stream_synchronize(tannic_stream_t stream) {
    if (refuses_while_recording(as_stream(stream), "stream_synchronize")) return TANNIC_ERROR;
    TH_TRY(hipStreamSynchronize(as_stream(stream)));
    return TANNIC_SUCCESS;
}

int tannic_hip_device_synchronize(void) {
    if (refuses_while_recording(nullptr, "device_synchronize")) return TANNIC_ERROR;
    TH_TRY(hipDeviceSynchronize());
    return TANNIC_SUCCESS;
}

void* tannic_hip_graph_begin(const tannic_device_t* device) {
    if (!device || tannic_hip_set_device(device->id) != TANNIC_SUCCESS) return nullptr;
    Streams& streams = Streams::instance();
    hipStream_t stream = streams.pop(device->id);
    streams.put(device->id, stream);      // the next backend call pops this same stream
    std::scoped_lock lock(g_scratch_mutex, g_mem_mutex);
    if (g_capturing) {
        set_error_text("graph_begin: another recording is open; end it first");
        return nullptr;
    }
    hipError_t err = hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed);
    if (err != hipSuccess) {
        set_error("hipStreamBeginCapture", __FILE__, __LINE__, err);
        return nullptr;
    }
    Recording* r = new Recording;
    r->id = ++g_recording_ids;
    r->device = device->id;
    r->stream = stream;
    r->capturing = true;
    g_recording_idle[r->id];
    g_capturing = r;
    return r;
}

void tannic_hip_counters(uint64_t out[3]) {
    for (int i = 0; i < th::kCounters; ++i) out[i] = th::g_counters[i].load(std::memory_order_relaxed);
}

tannic_stream_t tannic_hip_graph_stream(void* recording) {
    tannic_stream_t handle{};
    handle.address = recording ? reinterpret_cast<uintptr_t>(static_cast<Recording*>(recording)->stream) : 0;
    return handle;
}

int tannic_hip_graph_end(void* recording) {
    Recording* r = static_cast<Recording*>(recording);
    if (!r || !r->capturing) {
        set_error_text("graph_end: not an open recording");
        return TANNIC_ERROR;
    }
    {
        std::scoped_lock lock(g_scratch_mutex, g_mem_mutex);
        r->capturing = false;
        if (g_capturing == r) g_capturing = nullptr;
    }
    TH_TRY(hipSetDevice(r->device));
    hipError_t err = hipStreamEndCapture(r->stream, &r->graph);
    if (err != hipSuccess || !r->graph) {
        // a call that cannot be recorded (a wait for the stream, a copy to pageable host memory) has ended the capture
        set_error("hipStreamEndCapture", __FILE__, __LINE__, err);
        r->graph = nullptr;
        (void)hipGetLastError();
        return TANNIC_ERROR;
    }
    err = hipGraphInstantiate(&r->exec, r->graph, nullptr, nullptr, 0);
    if (err != hipSuccess) {
        set_error("hipGraphInstantiate", __FILE__, __LINE__, err);
        r->exec = nullptr;
        return TANNIC_ERROR;
    }
    return TANNIC_SUCCESS;
}

int tannic_hip_graph_launch(void* recording) {
    Recording* r = static_cast<Recording*>(recording);
    if (!r || !r->exec) {
        set_error_text("graph_launch: the recording was not ended successfully");
        return TANNIC_ERROR;
    }
    TH_TRY(hipSetDevice(r->device));
    TH_TRY(hipGraphLaunch(r->exec, r->stream));
    return TANNIC_SUCCESS;
}

void tannic_hip_graph_destroy(void* recording) {
    Recording* r = static_cast<Recording*>(recording);
    if (!r) return;
    (void)hipSetDevice(r->device);
    if (r->capturing) {
        // abandoned while open: close the capture and drop what it holds
        {
            std::scoped_lock lock(g_scratch_mutex, g_mem_mutex);
            r->capturing = false;
            if (g_capturing == r) g_capturing = nullptr;
        }
        hipGraph_t partial = nullptr;
        (void)hipStreamEndCapture(r->stream, &partial);
        if (partial) (void)hipGraphDestroy(partial);
        (void)hipGetLastError();
    }
    (void)hipStreamSynchronize(r->stream);     // no replay is still running when the memory changes hands
    if (r->exec) (void)hipGraphExecDestroy(r->exec);
    if (r->graph) (void)hipGraphDestroy(r->graph);
    std::vector<FreeBlock> idle;
    {
        std::scoped_lock lock(g_scratch_mutex, g_mem_mutex);
        for (void* ptr : r->scratch) {
            for (ScratchBlock& b : g_scratch_free)
                if (b.ptr == ptr && b.pins > 0) b.pins -= 1;
            for (ScratchBlock& b : g_scratch_live)
                if (b.ptr == ptr && b.pins > 0) b.pins -= 1;
        }
        auto it = g_recording_idle.find(r->id);
        if (it != g_recording_idle.end()) {
            idle.swap(it->second);
            g_recording_idle.erase(it);    // blocks of this recording that are still live are ordinary blocks from now on
        }
        // its released blocks join the blocks kept for everybody
        for (FreeBlock& f : idle) {
            f.info.recording = 0;
            g_mem_free.push_back(f);
            g_mem_kept += f.info.size;
        }
    }
    (void)hipGetLastError();
    delete r;
}

void* tannic_hip_event_create(void) {
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}

void tannic_hip_event_destroy(void* event) {
    if (event) (void)hipEventDestroy(static_cast<hipEvent_t>(event));
}

int tannic_hip_event_record(void* event, tannic_stream_t stream) {
    TH_TRY(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)));
    return TANNIC_SUCCESS;
}

float tannic_hip_event_elapsed_ms(void* start, void* stop) {
    float ms = -1.0f;
    if (hipEventSynchronize(static_cast<hipEvent_t>(stop)) != hipSuccess) return -1.0f;
    if (hipEventElapsedTime(&ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)) != hipSuccess) return -1.0f;
    return ms;
}

}  // extern "C"
