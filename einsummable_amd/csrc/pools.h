// The two resource pools an event loop needs to drive exec nodes one by one: device
// workspaces and streams.  Same behaviour as the reference's managers
// (src/engine/gpu/workspace.cc:48-91: the first free block that is large enough, else a new
// allocation, blocks returned for reuse and freed at the end; src/engine/gpu/stream_pool.cc:
// a fixed set of streams per device, try-acquire returns nothing when all are out).
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <mutex>
#include <utility>
#include <vector>

namespace es
{

class workspace_pool_t
{
public:
    explicit workspace_pool_t(int device) : device_(device) {}
    ~workspace_pool_t();
    workspace_pool_t(workspace_pool_t const&) = delete;
    workspace_pool_t& operator=(workspace_pool_t const&) = delete;

    // a block of at least `bytes` (its real size in *got); throws km_error when the device
    // is out of memory
    void* acquire(uint64_t bytes, uint64_t* got);
    // hands a block back; throws km_error for a pointer the pool did not give out
    void release(void* ptr);
    // blocks the pool has allocated so far, free or not
    int n_blocks() const;

private:
    int                                     device_;
    mutable std::mutex                      mu_;
    std::vector<std::pair<void*, uint64_t>> free_, out_;
};

class stream_pool_t
{
public:
    stream_pool_t(int device, int n_streams);
    ~stream_pool_t();
    stream_pool_t(stream_pool_t const&) = delete;
    stream_pool_t& operator=(stream_pool_t const&) = delete;

    // a free stream, or null when all are out
    hipStream_t try_acquire();
    void        release(hipStream_t s);

private:
    int                      device_;
    std::mutex               mu_;
    std::vector<hipStream_t> all_, free_;
};

}  // namespace es
