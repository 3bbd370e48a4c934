// What the stand-in runtime (fake_hip.cpp) offers beyond the HIP calls it replaces: a way to put host code on one of its
// streams, which is how the stand-in kernels (fake_kernels.cpp) and the test's own producers and consumers "launch".
#pragma once

#include <hip/hip_runtime_api.h>

#include <functional>

// Runs `work` on `stream`, in order with everything queued there before; on the null stream at once, in the calling thread.
void fake_enqueue(hipStream_t stream, std::function<void()> work);
