// The library's own workspace in device memory (see static_workspace.hip).
#pragma once
#include <cstdint>

namespace es
{

constexpr uint64_t STATIC_WORKSPACE_BYTES = 64ull << 20;

// Looks up, once per device and with that device current, where the workspace lies on it.
// Throws km_error.  Called by the kernel manager's constructor.
void* static_workspace_init(int device);

// The address found by static_workspace_init, or null before it ran for this device.
void* static_workspace(int device);

}  // namespace es
