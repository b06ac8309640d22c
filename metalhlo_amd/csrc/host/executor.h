// Host executor: walks a parsed function in program order and issues one kernel
// launch per op on one HIP stream (no host synchronisation between ops; one
// stream synchronisation at the end).  Mirrors the role of the reference's
// IntegratedExecutor (Sources/MetalHLOCore/Runtime/IntegratedExecutor.swift:150-270)
// with explicit device allocations in place of its unified buffer.
#pragma once
#include <hip/hip_runtime.h>

#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "hlo.h"

namespace mhlo {

struct ExecError : std::runtime_error { using std::runtime_error::runtime_error; };
struct InputMismatch : std::runtime_error { using std::runtime_error::runtime_error; };
struct NoDevice : std::runtime_error { using std::runtime_error::runtime_error; };
struct BufferError : std::runtime_error { using std::runtime_error::runtime_error; };

// Size-bucketed free list in front of hipMalloc: intermediate tensors of one
// execution are reused by the next instead of being allocated again.
class DevicePool {
public:
    ~DevicePool();
    void* alloc(size_t bytes);
    void release(void* p, size_t bytes);
private:
    std::mutex mu_;
    std::multimap<size_t, void*> free_;
};

struct DeviceMem {
    DevicePool* pool = nullptr;
    void* ptr = nullptr;
    size_t bytes = 0;
    ~DeviceMem() { if (pool && ptr) pool->release(ptr, bytes); }
};

struct DeviceTensor {
    TensorType type;
    std::shared_ptr<DeviceMem> mem;   // may be shared by reshapes
    void* data() const { return mem ? mem->ptr : nullptr; }
};

struct Client {
    int device = -1;          // -1: created without a device (host-only operations)
    std::string device_name;
    hipStream_t stream = nullptr;
    DevicePool pool;
    DeviceTensor allocate(const TensorType& t);
};

struct Executable {
    Client* client = nullptr;
    Function fn;
    int opt_level = 2;
    std::vector<DeviceTensor> constants;   // per op index (empty when the op is not a constant)
    // statistics (milliseconds), CInterface.swift:63-96
    int64_t exec_count = 0;
    double total_ms = 0, last_ms = 0;
    std::mutex mu;
};

// Validates every op against what the kernels cover (throws UnsupportedOp) and
// uploads constants when the client has a device.
void compile(Executable& exe);

// Runs the function.  `encode_s` = host time to issue all launches, `gpu_s` =
// time from first launch to stream completion.
std::vector<DeviceTensor> execute(Executable& exe, const std::vector<DeviceTensor>& inputs,
                                  double* encode_s, double* gpu_s);

}  // namespace mhlo
