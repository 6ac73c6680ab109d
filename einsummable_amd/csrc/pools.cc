#include "pools.h"

#include "kernel_manager.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <string>

namespace es
{

namespace
{
void check(hipError_t err, const char* what)
{
    if (err != hipSuccess) {
        throw km_error(km_status::device, std::string(what) + ": " + hipGetErrorString(err));
    }
}
}  // namespace

workspace_pool_t::~workspace_pool_t()
{
    for (auto const& b : free_) (void)hipFree(b.first);
    for (auto const& b : out_) (void)hipFree(b.first);
}

void* workspace_pool_t::acquire(uint64_t bytes, uint64_t* got)
{
    std::lock_guard<std::mutex> lock(mu_);
    for (size_t i = 0; i != free_.size(); ++i) {
        if (free_[i].second >= bytes) {
            auto b = free_[i];
            free_.erase(free_.begin() + long(i));
            out_.push_back(b);
            if (got) *got = b.second;
            return b.first;
        }
    }
    check(hipSetDevice(device_), "hipSetDevice");
    void* p = nullptr;
    check(hipMalloc(&p, std::max<uint64_t>(bytes, 256)), "workspace pool: hipMalloc");
    out_.push_back({p, std::max<uint64_t>(bytes, 256)});
    if (got) *got = out_.back().second;
    return p;
}

void workspace_pool_t::release(void* ptr)
{
    std::lock_guard<std::mutex> lock(mu_);
    for (size_t i = 0; i != out_.size(); ++i) {
        if (out_[i].first == ptr) {
            free_.push_back(out_[i]);
            out_.erase(out_.begin() + long(i));
            return;
        }
    }
    throw km_error(km_status::invalid, "workspace pool: release of a block it did not give out");
}

int workspace_pool_t::n_blocks() const
{
    std::lock_guard<std::mutex> lock(mu_);
    return int(free_.size() + out_.size());
}

stream_pool_t::stream_pool_t(int device, int n_streams) : device_(device)
{
    if (n_streams < 1 || n_streams > 64) {
        throw km_error(km_status::invalid, "stream pool: between 1 and 64 streams");
    }
    check(hipSetDevice(device_), "hipSetDevice");
    for (int i = 0; i != n_streams; ++i) {
        hipStream_t s;
        // default priority; non-blocking, so that work on the null stream does not order them
        check(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreateWithFlags");
        all_.push_back(s);
    }
    free_ = all_;
}

stream_pool_t::~stream_pool_t()
{
    for (hipStream_t s : all_) (void)hipStreamDestroy(s);
}

hipStream_t stream_pool_t::try_acquire()
{
    std::lock_guard<std::mutex> lock(mu_);
    if (free_.empty()) return nullptr;
    hipStream_t s = free_.back();
    free_.pop_back();
    return s;
}

void stream_pool_t::release(hipStream_t s)
{
    std::lock_guard<std::mutex> lock(mu_);
    if (std::find(all_.begin(), all_.end(), s) == all_.end() ||
        std::find(free_.begin(), free_.end(), s) != free_.end()) {
        throw km_error(km_status::invalid, "stream pool: release of a stream that is not out");
    }
    free_.push_back(s);
}

}  // namespace es
