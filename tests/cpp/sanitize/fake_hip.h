// fake_hip.h -- controls of the host stand-in for the HIP runtime (fake_hip.cpp). Test infrastructure only.
#pragma once

#include <functional>

// Number of devices hipGetDevice / hipSetDevice believe in (default 1; 0 makes hipGetDevice fail).
void fake_hip_set_device_count(int n);
// hipMalloc / hipHostMalloc / stream / event objects that exist right now: 0 after everything has been given back.
long fake_hip_live_allocations();
// Called at the top of every hipGetDevice (the first runtime call of a file-store transfer that meets a device iov):
// lets a test know that a put or get is inside the library. Empty function = no hook.
void fake_hip_on_get_device(std::function<void()> fn);
// Queues `job` on a stream of the stand-in, behind whatever was queued before: how the stand-ins of the library's
// kernel entry points (sanitize_host.cpp) do their work "on the device", in stream order.
void fake_hip_enqueue(void *stream, std::function<void()> job);
