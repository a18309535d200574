// Optional per-kernel timing with hipEvents (diagnostics for bench.py and profiling scripts).
// Stands for the reference's ad-hoc cudaEvent phase breakdown (sentinel/NeuralNet/Cuda/CudaLanguageModel.cu:4203-4211).
// Off by default; while on, every kernel launch is bracketed by two events on its own stream, so calls
// made with timing on must not be captured into a graph.
#include "flash_common.h"

#include <atomic>
#include <cstring>
#include <mutex>
#include <vector>

namespace sentinel_hip {
namespace {

struct Record {
    const char* name;
    hipEvent_t start;
    hipEvent_t stop;
};

std::mutex g_mutex;
std::atomic<bool> g_enabled{false};  // read without the lock on every launch
std::vector<Record> g_records;
std::vector<hipEvent_t> g_pool;

hipEvent_t take_event() {
    if (!g_pool.empty()) {
        hipEvent_t e = g_pool.back();
        g_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}

}  // namespace

KernelTimer::KernelTimer(const char* name, hipStream_t stream) : name_(name), stream_(stream), start_(nullptr) {
    if (!g_enabled.load(std::memory_order_relaxed)) return;  // timing off: no lock, no host state touched
    std::lock_guard<std::mutex> lock(g_mutex);
    start_ = take_event();
    if (start_) (void)hipEventRecord(start_, stream_);
}

KernelTimer::~KernelTimer() {
    if (!start_) return;
    std::lock_guard<std::mutex> lock(g_mutex);
    hipEvent_t stop = take_event();
    if (!stop) {
        g_pool.push_back(start_);
        return;
    }
    (void)hipEventRecord(stop, stream_);
    g_records.push_back(Record{name_, start_, stop});
}

int timing_set_enabled(int enabled) {
    std::lock_guard<std::mutex> lock(g_mutex);
    const int before = g_enabled.load() ? 1 : 0;
    g_enabled.store(enabled != 0);
    return before;
}

int timing_collect(const char** names, float* total_ms, int* launches, int capacity) {
    std::lock_guard<std::mutex> lock(g_mutex);
    int distinct = 0;
    for (const Record& r : g_records) {
        float ms = 0.0f;
        if (hipEventSynchronize(r.stop) != hipSuccess || hipEventElapsedTime(&ms, r.start, r.stop) != hipSuccess) ms = 0.0f;
        g_pool.push_back(r.start);
        g_pool.push_back(r.stop);
        int slot = -1;
        for (int i = 0; i < distinct && i < capacity; ++i)
            if (std::strcmp(names[i], r.name) == 0) slot = i;
        if (slot < 0) {
            if (distinct >= capacity) continue;
            slot = distinct++;
            names[slot] = r.name;
            total_ms[slot] = 0.0f;
            launches[slot] = 0;
        }
        total_ms[slot] += ms;
        launches[slot] += 1;
    }
    g_records.clear();
    return distinct;
}

}  // namespace sentinel_hip
