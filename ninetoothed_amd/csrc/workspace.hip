#include "workspace.h"

#include <map>
#include <mutex>
#include <tuple>

#include "../../include/ninetoothed_hip.h"

namespace nt {
namespace {

struct Buffer {
    void *data = nullptr;
    size_t bytes = 0;
};

std::recursive_mutex g_mutex;
std::map<std::tuple<int, hipStream_t, int>, Buffer> g_buffers;

}  // namespace

WorkspaceLease::WorkspaceLease(hipStream_t stream) : stream_(stream), device_(0) {
    g_mutex.lock();
    (void)hipGetDevice(&device_);
}

WorkspaceLease::~WorkspaceLease() { g_mutex.unlock(); }

void *WorkspaceLease::get(WorkspacePurpose purpose, size_t bytes) {
    Buffer &buffer = g_buffers[std::make_tuple(device_, stream_, (int)purpose)];
    if (buffer.bytes >= bytes && buffer.data != nullptr) return buffer.data;
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream_, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return nullptr;
    }
    if (buffer.data != nullptr) {
        // hipFree waits for the device: nothing still reads the old buffer afterwards
        (void)hipFree(buffer.data);
        buffer = Buffer();
    }
    void *data = nullptr;
    const size_t rounded = (bytes + 255) & ~(size_t)255;
    if (hipMalloc(&data, rounded) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    buffer.data = data;
    buffer.bytes = rounded;
    return data;
}

}  // namespace nt

extern "C" void nt_release_workspaces(void) {
    std::lock_guard<std::recursive_mutex> lock(nt::g_mutex);
    for (auto &entry : nt::g_buffers) {
        if (entry.second.data != nullptr) (void)hipFree(entry.second.data);
    }
    nt::g_buffers.clear();
}
