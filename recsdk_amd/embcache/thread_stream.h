// Shared by the HIP-backed Embcache classes: the calling thread's stream and copies on it.
// EmbcacheManager computes the swap info of its tables from worker threads (embcache_manager.cpp:89-185); with a
// stream per thread the tables' kernels and copies run side by side on the device, where the null stream would queue
// them.  Every member function waits for its stream before it returns, so an object may be used from a different
// thread on every call.  The streams live as long as the process.
#ifndef RECSDK_EMBCACHE_THREAD_STREAM_H
#define RECSDK_EMBCACHE_THREAD_STREAM_H

#include <cstddef>
#include <stdexcept>
#include <string>

#include <hip/hip_runtime_api.h>

namespace recsdk_embcache {

inline hipStream_t ThreadStream()
{
    thread_local hipStream_t stream = nullptr;
    if (stream == nullptr && hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        stream = nullptr;   // the null stream still works
    }
    return stream;
}

inline void CheckHip(hipError_t e, const char* who, const char* what)
{
    if (e != hipSuccess) {
        throw std::runtime_error(std::string(who) + " (HIP): " + what + ": " + hipGetErrorString(e));
    }
}

// host -> device, complete on return
inline void CopyUp(void* dst, const void* src, size_t bytes, const char* who)
{
    if (bytes != 0) {
        CheckHip(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ThreadStream()), who, "hipMemcpyAsync");
        CheckHip(hipStreamSynchronize(ThreadStream()), who, "hipStreamSynchronize");
    }
}

// device -> host, complete on return (and with it everything issued on the thread's stream before)
inline void CopyDown(void* dst, const void* src, size_t bytes, const char* who)
{
    if (bytes != 0) {
        CheckHip(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ThreadStream()), who, "hipMemcpyAsync");
    }
    CheckHip(hipStreamSynchronize(ThreadStream()), who, "hipStreamSynchronize");
}

}  // namespace recsdk_embcache

#endif  // RECSDK_EMBCACHE_THREAD_STREAM_H
