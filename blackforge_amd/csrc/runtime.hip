// Devices, streams, events and the per-device memory pool.
//
// The pool replaces the reference's exact-byte-size free lists (device_pool.cu:29-65) with size
// classes: requests are rounded up to a class (four classes per power of two, 512 B minimum, 2 MiB
// granularity above 64 MiB) so that tensors of nearby sizes share blocks and a 288 GB card is not
// fragmented by one free list per distinct shape.  As in the reference, released blocks stay cached
// for the life of the process unless bf_hip_pool_trim() is called.
#include "common.hpp"

#include <algorithm>
#include <map>
#include <mutex>
#include <thread>
#include <unordered_map>
#include <vector>

namespace bf {

namespace {
thread_local std::string g_lastError;
}

void setLastError(const std::string& message) { g_lastError = message; }

int failInvalid(const char* function, const std::string& message) {
    g_lastError = std::string(function) + ": " + message;
    return BF_ERR_INVALID_ARGUMENT;
}

int failRuntime(const char* function, hipError_t error, const char* file, int line) {
    g_lastError = std::string(file) + ":" + std::to_string(line) + ": " + function + ": HIP error: " +
                  hipGetErrorString(error);
    return BF_ERR_RUNTIME;
}

hipStream_t g_defaultStream = nullptr;
hipStream_t g_currentStream = nullptr;
bool g_currentStreamKnown = false;

void switchStream(hipStream_t next) {
    if (capturing()) return;
    if (g_currentStreamKnown && next != g_currentStream) {
        // one event per device, recorded again at every switch: only the latest record matters to the waiter
        static std::unordered_map<int, hipEvent_t> fences;
        int dev = 0;
        if (hipGetDevice(&dev) == hipSuccess) {
            hipEvent_t& fence = fences[dev];
            if (fence == nullptr && hipEventCreateWithFlags(&fence, hipEventDisableTiming) != hipSuccess) fence = nullptr;
            // a failure here (a stream that no longer exists) leaves the old stream's work unordered with the new one's:
            // fall back to waiting for the whole device
            if (fence == nullptr || hipEventRecord(fence, g_currentStream) != hipSuccess || hipStreamWaitEvent(next, fence, 0) != hipSuccess) {
                (void)hipGetLastError();
                (void)hipDeviceSynchronize();
            }
        }
    }
    g_currentStream = next;
    g_currentStreamKnown = true;
}

int computeUnits() {
    static std::unordered_map<int, int> cache;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    auto it = cache.find(dev);
    if (it != cache.end()) return it->second;
    int cus = 256;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cus = 256;
    cache[dev] = cus;
    return cus;
}

size_t deviceMemoryBytes() {
    static std::unordered_map<int, size_t> cache;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    auto it = cache.find(dev);
    if (it != cache.end()) return it->second;
    size_t freeBytes = 0, totalBytes = 0;
    if (hipMemGetInfo(&freeBytes, &totalBytes) != hipSuccess) { (void)hipGetLastError(); totalBytes = 0; }
    cache[dev] = totalBytes;
    return totalBytes;
}

namespace {
struct DescriptorTable {
    std::vector<unsigned char> host;
    void* device = nullptr;
    size_t capacity = 0;
};
std::map<std::pair<int, int>, DescriptorTable>& descriptorTables() {
    static std::map<std::pair<int, int>, DescriptorTable> tables;
    return tables;
}
}  // namespace

int uploadPrivateTable(const void* hostBytes, size_t bytes, const void** devicePtr);

int allowDynamicSharedMemory(const void* kernel, size_t bytes) {
    if (bytes <= 48 * 1024) return BF_OK;
    int dev = 0;
    BF_HIP_TRY(hipGetDevice(&dev));
    static std::map<std::pair<const void*, int>, size_t> granted;
    size_t& have = granted[{kernel, dev}];
    if (have >= bytes) return BF_OK;
    BF_HIP_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, int(bytes)));
    have = bytes;
    return BF_OK;
}

int uploadDescriptorTable(int slot, const void* hostBytes, size_t bytes, hipStream_t stream, const void** devicePtr) {
    int dev = 0;
    BF_HIP_TRY(hipGetDevice(&dev));
    if (capturing()) return uploadPrivateTable(hostBytes, bytes, devicePtr);
    DescriptorTable& t = descriptorTables()[{dev, slot}];
    const auto* src = static_cast<const unsigned char*>(hostBytes);
    bool same = t.device != nullptr && t.host.size() == bytes && std::equal(src, src + bytes, t.host.begin());
    if (!same) {
        // kernels still reading the old table must finish before it is overwritten or freed
        BF_HIP_TRY(hipStreamSynchronize(stream));
        if (bytes > t.capacity) {
            if (t.device) BF_HIP_TRY(hipFree(t.device));
            t.device = nullptr;
            size_t cap = bytes < 4096 ? 4096 : bytes * 2;
            BF_HIP_TRY(hipMalloc(&t.device, cap));
            t.capacity = cap;
        }
        BF_HIP_TRY(hipMemcpy(t.device, hostBytes, bytes, hipMemcpyHostToDevice));
        t.host.assign(src, src + bytes);
    }
    *devicePtr = t.device;
    return BF_OK;
}

namespace {

size_t sizeClass(size_t bytes) {
    constexpr size_t kMin = 512;
    constexpr size_t kLarge = size_t(64) << 20;
    constexpr size_t kLargeStep = size_t(2) << 20;
    if (bytes <= kMin) return kMin;
    if (bytes > kLarge) return (bytes + kLargeStep - 1) / kLargeStep * kLargeStep;
    size_t pow2 = kMin;
    while (pow2 < bytes) pow2 <<= 1;   // smallest power of two >= bytes
    size_t quarter = pow2 >> 3;        // classes at 5/8, 6/8, 7/8, 8/8 of pow2
    for (size_t c = (pow2 >> 1) + quarter; c < pow2; c += quarter)
        if (bytes <= c) return c;
    return pow2;
}

struct DevicePool {
    std::unordered_map<size_t, std::vector<void*>> freeLists;
    bf_pool_stats stats{};
};

std::unordered_map<int, DevicePool>& pools() {
    static std::unordered_map<int, DevicePool> registry;
    return registry;
}

// The memory of one captured graph.  Every block acquired while the capture runs belongs to the arena: when it is
// released (during the capture or later, by whoever holds it) it goes to the arena's own free lists, where only the
// same capture can take it again, and it reaches the device's general free lists only when the graph is destroyed.
// A replay therefore never finds one of its buffers in somebody else's hands, and bf_hip_pool_trim cannot free them.
struct CaptureArena {
    int device = 0;
    hipStream_t stream = nullptr;
    std::thread::id thread;   // the host thread that records: nobody else may take pool memory meanwhile
    std::unordered_map<size_t, std::vector<void*>> freeLists;
    std::vector<std::pair<void*, size_t>> blocks;   // (pointer, size class) of every block taken during the capture
    std::vector<void*> tables;                      // descriptor tables of recorded launches (hipMalloc, not pool blocks)
};
CaptureArena* g_capture = nullptr;                               // the capture in progress
std::unordered_map<void*, CaptureArena*>& arenaOwners() {        // block -> arena, for arenas that still exist
    static std::unordered_map<void*, CaptureArena*> owners;
    return owners;
}
// non-blocking stream of the capturing device, for copies that must not touch a capturing stream (one per device)
hipStream_t g_utilityStream = nullptr;
std::unordered_map<int, hipStream_t>& utilityStreams() {
    static std::unordered_map<int, hipStream_t> streams;
    return streams;
}

struct CapturedGraph {
    hipGraphExec_t exec = nullptr;
    CaptureArena* arena = nullptr;
};

// hipMalloc with one retry after returning every cached block to the driver: size classes above 64 MiB are 2 MiB
// apart, so a process that has seen many shapes can hold most of the card in free lists that fit nothing new.
hipError_t mallocWithTrim(void** ptr, size_t bytes, DevicePool& pool) {
    hipError_t err = hipMalloc(ptr, bytes);
    if (err != hipErrorOutOfMemory || capturing()) return err;
    (void)hipGetLastError();
    if (hipDeviceSynchronize() != hipSuccess) return err;
    for (auto& entry : pool.freeLists) {
        std::vector<void*> kept;   // a block the driver refuses to take back stays on its free list
        for (void* p : entry.second) {
            if (hipFree(p) == hipSuccess) pool.stats.bytes_from_driver -= entry.first;
            else { (void)hipGetLastError(); kept.push_back(p); }
        }
        entry.second.swap(kept);
    }
    return hipMalloc(ptr, bytes);
}

void retireArena(CaptureArena* arena) {
    DevicePool& pool = pools()[arena->device];
    for (const auto& block : arena->blocks) arenaOwners().erase(block.first);
    for (auto& entry : arena->freeLists)
        for (void* p : entry.second) pool.freeLists[entry.first].push_back(p);
    for (void* table : arena->tables) (void)hipFree(table);
    delete arena;
}

}  // namespace

bool capturing() { return g_capture != nullptr; }

// A descriptor table for kernels that are being recorded: memory of its own, written now (on a stream that has nothing
// to do with the capturing one) and never again, so that replays read what the recording saw.  It must not come from
// the pool: a block that recorded kernels used as a temporary earlier in the capture and released would be rewritten
// by those kernels on every replay, under the table.
int uploadPrivateTable(const void* hostBytes, size_t bytes, const void** devicePtr) {
    void* block = nullptr;
    BF_HIP_TRY(hipMalloc(&block, bytes < 256 ? 256 : bytes));
    g_capture->tables.push_back(block);   // freed with the graph
    BF_HIP_TRY(hipMemcpyAsync(block, hostBytes, bytes, hipMemcpyHostToDevice, g_utilityStream));
    BF_HIP_TRY(hipStreamSynchronize(g_utilityStream));
    *devicePtr = block;
    return BF_OK;
}

namespace {
__global__ void fillZeroKernel(uint32_t* dst, size_t words) {
    size_t stride = size_t(gridDim.x) * blockDim.x;
    for (size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x; i < words; i += stride) dst[i] = 0u;
}
__global__ void fillZeroBytesKernel(unsigned char* dst, size_t bytes) {
    size_t i = size_t(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < bytes) dst[i] = 0;
}

}  // namespace
}  // namespace bf

using namespace bf;

extern "C" {

const char* bf_hip_last_error(void) { return g_lastError.c_str(); }
const char* bf_hip_version(void) { return "blackforge-hip 0.1 (gfx950)"; }

int bf_hip_device_count(int* count) {
    BF_REQUIRE(count != nullptr, "count is NULL");
    int n = 0;
    hipError_t err = hipGetDeviceCount(&n);
    if (err != hipSuccess) {  // no driver / no device: the reference returns an empty list
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return BF_OK;
}

int bf_hip_device_props(int index, bf_device_props* props) {
    BF_REQUIRE(props != nullptr, "props is NULL");
    hipDeviceProp_t p;
    BF_HIP_TRY(hipGetDeviceProperties(&p, index));
    snprintf(props->name, sizeof(props->name), "%s", p.name);
    snprintf(props->arch, sizeof(props->arch), "%s", p.gcnArchName);
    props->compute_units = p.multiProcessorCount;
    props->clock_khz = p.clockRate;
    props->wavefront_size = p.warpSize;
    props->lds_bytes_per_block = static_cast<int>(p.sharedMemPerBlock);
    props->total_memory = p.totalGlobalMem;
    return BF_OK;
}

int bf_hip_set_device(int index) {
    int n = 0;
    bf_hip_device_count(&n);
    BF_REQUIRE(index >= 0 && index < n, "device index " + std::to_string(index) + " out of range (" +
                                            std::to_string(n) + " devices)");
    int before = index;
    (void)hipGetDevice(&before);
    BF_HIP_TRY(hipSetDevice(index));
    if (before != index) {   // the stream last used is a per-device fact (pools are per device): park it, fetch the other device's
        static std::unordered_map<int, std::pair<hipStream_t, bool>> parked;
        parked[before] = {g_currentStream, g_currentStreamKnown};
        const auto it = parked.find(index);
        g_currentStream = it != parked.end() ? it->second.first : nullptr;
        g_currentStreamKnown = it != parked.end() && it->second.second;
    }
    return BF_OK;
}

int bf_hip_get_device(int* index) {
    BF_REQUIRE(index != nullptr, "index is NULL");
    BF_HIP_TRY(hipGetDevice(index));
    return BF_OK;
}

int bf_hip_synchronize(void) {
    BF_HIP_TRY(hipDeviceSynchronize());
    return BF_OK;
}

int bf_hip_stream_create(bf_stream_t* stream) {
    BF_REQUIRE(stream != nullptr, "stream is NULL");
    hipStream_t s;
    // blocking with respect to the default stream, so the synchronous copies of fromHost/toHost stay
    // ordered with work enqueued on this stream
    BF_HIP_TRY(hipStreamCreate(&s));
    *stream = s;
    return BF_OK;
}
int bf_hip_stream_destroy(bf_stream_t stream) {
    if (stream == nullptr) return BF_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (g_currentStreamKnown && g_currentStream == s) {
        // its queued work may still use pool blocks that are free again on the host: it finishes before the stream goes,
        // and the next stream has nothing to be ordered behind
        BF_HIP_TRY(hipStreamSynchronize(s));
        g_currentStreamKnown = false;
    }
    BF_HIP_TRY(hipStreamDestroy(s));
    return BF_OK;
}
int bf_hip_stream_synchronize(bf_stream_t stream) {
    BF_HIP_TRY(hipStreamSynchronize(asStream(stream)));
    return BF_OK;
}
int bf_hip_event_create(bf_event_t* event) {
    BF_REQUIRE(event != nullptr, "event is NULL");
    hipEvent_t e;
    BF_HIP_TRY(hipEventCreate(&e));
    *event = e;
    return BF_OK;
}
int bf_hip_event_destroy(bf_event_t event) {
    if (event) BF_HIP_TRY(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return BF_OK;
}
int bf_hip_event_record(bf_event_t event, bf_stream_t stream) {
    BF_HIP_TRY(hipEventRecord(static_cast<hipEvent_t>(event), asStream(stream)));
    return BF_OK;
}
int bf_hip_event_synchronize(bf_event_t event) {
    BF_HIP_TRY(hipEventSynchronize(static_cast<hipEvent_t>(event)));
    return BF_OK;
}
int bf_hip_event_elapsed_ms(bf_event_t start, bf_event_t stop, float* ms) {
    BF_REQUIRE(ms != nullptr, "ms is NULL");
    BF_HIP_TRY(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
    return BF_OK;
}

int bf_hip_pool_acquire(size_t bytes, void** ptr) {
    BF_REQUIRE(ptr != nullptr, "ptr is NULL");
    *ptr = nullptr;
    if (bytes == 0) return BF_OK;
    int dev = 0;
    BF_HIP_TRY(hipGetDevice(&dev));
    if (g_capture != nullptr && g_capture->thread != std::this_thread::get_id())
        return failInvalid(__func__, "another host thread is recording a graph: its pool memory belongs to the recording");
    DevicePool& pool = pools()[dev];
    size_t cls = sizeClass(bytes);
    std::vector<void*>* list = &pool.freeLists[cls];
    if (g_capture != nullptr && !g_capture->freeLists[cls].empty()) list = &g_capture->freeLists[cls];
    if (!list->empty()) {
        *ptr = list->back();
        list->pop_back();
    } else {
        BF_HIP_TRY(mallocWithTrim(ptr, cls, pool));
        pool.stats.bytes_from_driver += cls;
        pool.stats.driver_allocations += 1;
    }
    if (g_capture != nullptr && arenaOwners().emplace(*ptr, g_capture).second) g_capture->blocks.emplace_back(*ptr, cls);
    pool.stats.bytes_in_use += cls;
    pool.stats.acquires += 1;
    return BF_OK;
}

int bf_hip_pool_release(void* ptr, size_t bytes) {
    if (ptr == nullptr) return BF_OK;
    int dev = 0;
    BF_HIP_TRY(hipGetDevice(&dev));
    DevicePool& pool = pools()[dev];
    size_t cls = sizeClass(bytes);
    const auto owner = arenaOwners().find(ptr);
    if (owner != arenaOwners().end()) owner->second->freeLists[cls].push_back(ptr);
    else pool.freeLists[cls].push_back(ptr);
    pool.stats.bytes_in_use -= cls < pool.stats.bytes_in_use ? cls : pool.stats.bytes_in_use;
    return BF_OK;
}

int bf_hip_pool_stats(bf_pool_stats* stats) {
    BF_REQUIRE(stats != nullptr, "stats is NULL");
    int dev = 0;
    BF_HIP_TRY(hipGetDevice(&dev));
    *stats = pools()[dev].stats;
    return BF_OK;
}

int bf_hip_pool_trim(void) {
    int dev = 0;
    BF_HIP_TRY(hipGetDevice(&dev));
    BF_HIP_TRY(hipDeviceSynchronize());
    DevicePool& pool = pools()[dev];
    for (auto& entry : pool.freeLists) {
        for (void* p : entry.second) {
            BF_HIP_TRY(hipFree(p));
            pool.stats.bytes_from_driver -= entry.first;
        }
        entry.second.clear();
    }
    return BF_OK;
}

int bf_hip_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    if (bytes == 0) return BF_OK;
    BF_REQUIRE(dst && src, "NULL pointer");
    BF_HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
    return BF_OK;
}
int bf_hip_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    if (bytes == 0) return BF_OK;
    BF_REQUIRE(dst && src, "NULL pointer");
    BF_HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
    return BF_OK;
}
int bf_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, bf_stream_t stream) {
    if (bytes == 0) return BF_OK;
    BF_REQUIRE(dst && src, "NULL pointer");
    BF_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, asStream(stream)));
    return BF_OK;
}

int bf_hip_capture_begin(bf_stream_t stream) {
    BF_REQUIRE(stream != nullptr, "a capture needs a stream made by bf_hip_stream_create");
    BF_REQUIRE(g_capture == nullptr, "a capture is already in progress");
    int dev = 0;
    BF_HIP_TRY(hipGetDevice(&dev));
    hipStream_t& utility = utilityStreams()[dev];
    if (utility == nullptr) BF_HIP_TRY(hipStreamCreateWithFlags(&utility, hipStreamNonBlocking));
    g_utilityStream = utility;
    BF_HIP_TRY(hipDeviceSynchronize());   // nothing of the eager work before may still be in flight on another stream
    BF_HIP_TRY(hipStreamBeginCapture(static_cast<hipStream_t>(stream), hipStreamCaptureModeRelaxed));
    g_capture = new CaptureArena;
    g_capture->device = dev;
    g_capture->stream = static_cast<hipStream_t>(stream);
    g_capture->thread = std::this_thread::get_id();
    g_defaultStream = g_capture->stream;
    g_currentStream = g_capture->stream;   // the device is idle: nothing to be ordered behind
    g_currentStreamKnown = true;
    return BF_OK;
}

int bf_hip_capture_end(bf_graph_t* graph) {
    BF_REQUIRE(g_capture != nullptr, "no capture in progress");
    CaptureArena* arena = g_capture;
    dropCaptureWeightImages();   // while releases still go to the arena
    g_capture = nullptr;
    g_defaultStream = nullptr;
    hipGraph_t recorded = nullptr;
    hipError_t err = hipStreamEndCapture(arena->stream, &recorded);
    hipGraphExec_t exec = nullptr;
    if (err == hipSuccess && graph != nullptr) err = hipGraphInstantiate(&exec, recorded, nullptr, nullptr, 0);
    if (recorded != nullptr) (void)hipGraphDestroy(recorded);
    if (err != hipSuccess || graph == nullptr) {   // failed, or the caller abandons the capture (graph == NULL)
        (void)hipGetLastError();
        retireArena(arena);
        if (graph != nullptr) *graph = nullptr;
        if (err != hipSuccess) return failRuntime(__func__, err, __FILE__, __LINE__);
        return BF_OK;
    }
    *graph = new CapturedGraph{exec, arena};
    return BF_OK;
}

int bf_hip_graph_launch(bf_graph_t graph, bf_stream_t stream) {
    BF_REQUIRE(graph != nullptr, "graph is NULL");
    BF_REQUIRE(g_capture == nullptr, "a graph cannot be launched into a capture");
    BF_HIP_TRY(hipGraphLaunch(static_cast<CapturedGraph*>(graph)->exec, asStream(stream)));
    noteGraphLaunched();
    return BF_OK;
}

int bf_hip_graph_destroy(bf_graph_t graph) {
    if (graph == nullptr) return BF_OK;
    CapturedGraph* g = static_cast<CapturedGraph*>(graph);
    BF_HIP_TRY(hipDeviceSynchronize());   // a replay still running keeps using the arena's blocks
    if (g->exec != nullptr) (void)hipGraphExecDestroy(g->exec);
    retireArena(g->arena);
    delete g;
    return BF_OK;
}

int bf_hip_fill_zero(void* dst, size_t bytes, bf_stream_t stream) {
    if (bytes == 0) return BF_OK;
    BF_REQUIRE(dst != nullptr, "NULL pointer");
    BF_REQUIRE((reinterpret_cast<uintptr_t>(dst) & 3u) == 0, "dst must be 4-byte aligned");
    size_t words = bytes / 4;
    if (words) {
        unsigned grid = gridFor(words, size_t(kBlock) * 4);
        fillZeroKernel<<<grid, kBlock, 0, asStream(stream)>>>(static_cast<uint32_t*>(dst), words);
        BF_LAUNCH_CHECK();
    }
    size_t tail = bytes - words * 4;
    if (tail) {
        fillZeroBytesKernel<<<1, 64, 0, asStream(stream)>>>(static_cast<unsigned char*>(dst) + words * 4, tail);
        BF_LAUNCH_CHECK();
    }
    return BF_OK;
}

}  // extern "C"
