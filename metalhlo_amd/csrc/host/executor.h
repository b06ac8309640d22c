// Host executor: walks a parsed function in program order and issues one kernel
// launch per op on one HIP stream (no host synchronisation between ops; one
// stream synchronisation at the end).  Mirrors the role of the reference's
// IntegratedExecutor (Sources/MetalHLOCore/Runtime/IntegratedExecutor.swift:150-270)
// with explicit device allocations in place of its unified buffer.
#pragma once
#include <hip/hip_runtime.h>

#include <map>
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

// Placement of every device allocation one execution makes (results of operations and the
// temporaries inside them) in one arena, from the lifetimes a dry run of the program records
// at compile time: slots whose lifetimes overlap never share bytes, offsets are multiples of
// 256.  The role of the reference's StaticMemoryPlanner
// (Sources/MetalHLOCore/Memory/StaticMemoryPlanner.swift:144-250).
struct ArenaPlan {
    struct Slot {
        size_t bytes = 0;        // rounded up to 256
        int begin = 0, end = 0;  // allocation / release time of the dry run
        size_t offset = 0;
        bool escapes = false;    // returned to the caller
    };
    std::vector<Slot> slots;     // in allocation order
    size_t core_bytes = 0;       // arena for the slots that do not escape
    size_t full_bytes = 0;       // ... plus the escaping ones behind them (graph replay needs fixed addresses)
    size_t sum_bytes = 0;        // what one allocation per non-escaping slot takes
    bool valid = false;
    int clock = 0;
};

struct DeviceMem {
    DevicePool* pool = nullptr;
    void* ptr = nullptr;
    size_t bytes = 0;
    ArenaPlan* recorder = nullptr;   // dry run: note the release time of slot `slot`
    int slot = -1;
    bool replay_result = false;      // result buffer of a captured graph: the graph keeps one reference, the caller gets the other
    ~DeviceMem() {
        if (recorder) recorder->slots[slot].end = recorder->clock++;
        else if (pool && ptr) pool->release(ptr, bytes);
    }
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
    // Held while the stream is being captured into a graph, and by every other thread that
    // enqueues work on the stream (the PJRT plugin's transfers): work enqueued from another thread
    // during a capture would become part of the graph instead of running.
    std::mutex stream_mu;
    // Graphs are captured on a stream of their own (created at the first capture, non-blocking), never on
    // `stream`: the launches of a capture do not run, so which stream records them is immaterial to
    // the replays, and the events that other threads wait for on `stream` (the PJRT plugin's
    // transfer completions) then never belong to a stream that is capturing -- waiting for such an
    // event invalidates the capture.  `capture_broken`: a capture failed and left that stream in the
    // capturing state; this client captures nothing further (every execution is eager).
    hipStream_t capture_stream = nullptr;
    bool capture_broken = false;
    ~Client() { if (capture_stream && !capture_broken) (void)hipStreamDestroy(capture_stream); }
    DevicePool pool;
    DeviceTensor allocate(const TensorType& t);
};

struct Executable {
    Client* client = nullptr;
    Function fn;
    int opt_level = 2;
    std::vector<DeviceTensor> constants;   // per op index (empty when the op is not a constant)
    size_t batched_converts = 0;           // leading ops: f32 -> 16-bit converts of arguments, run as one batch
    // statistics (milliseconds), CInterface.swift:63-96
    int64_t exec_count = 0;
    double total_ms = 0, last_ms = 0;
    std::mutex mu;
    // arena and captured graphs (one execution at a time per executable while they are in use)
    ArenaPlan plan;
    void* arena = nullptr;
    size_t arena_size = 0;
    std::mutex run_mu;
    struct CapturedGraph {
        std::vector<const void*> inputs;                     // device addresses the graph was captured with
        hipGraphExec_t exec = nullptr;
        std::vector<std::pair<const void*, TensorType>> returns;   // where each result lies after a replay (arena form)
        // Direct form: the graph writes its results into buffers of their own, which are handed to the
        // caller as they are (no copy out of the arena).  A replay needs all of them back, i.e. released
        // by the caller of the previous one; otherwise that execution runs eagerly.
        std::vector<DeviceTensor> results;
    };
    std::vector<CapturedGraph> graphs;
    int64_t graph_captures = 0, graph_replays = 0, eager_runs = 0;
    bool graph_failed = false;
    // Device time of every operation of the last profiled execution (METALHLO_PROFILE_GPU=1 or a call of
    // mhlo_execute_with_profile): microseconds between the HIP events recorded in front of and
    // behind the operation's launches on the client's stream.
    struct OpTime { std::string name; std::string shape; double us = 0; };
    std::vector<OpTime> last_profile;
    bool profile_next = false;             // set by mhlo_execute_with_profile for one execution
    ~Executable();
};

// Validates every op against what the kernels cover (throws UnsupportedOp), uploads constants
// when the client has a device, and plans the arena.
void compile(Executable& exe);

// Runs the function.  `encode_s` = host time to issue all launches, `gpu_s` =
// time from first launch to stream completion.
// Memory: intermediates live in the executable's arena (METALHLO_ARENA=0: one pool block per
// value instead); results are always fresh buffers the caller owns.
// Launches: METALHLO_HIP_GRAPH=1 (default at optimisation level 3 for programs of sixteen or
// more launches; =0 switches it off) captures the op list into a
// HIP graph on the second execution and replays it while the input addresses stay the same
// (up to eight address sets are kept); results are then copied out of the arena.
// Per-dispatch timing (the role of METALHLO_PROFILE_GPU / METALHLO_DEBUG_DISPATCH in the reference,
// Runtime/MetalExecutor.swift:289-316, Runtime/IntegratedExecutor.swift:411-478): with
// METALHLO_PROFILE_GPU=1, or for the one execution after exe.profile_next is set, the program runs
// eagerly with a HIP event pair around every operation; the times land in exe.last_profile and,
// with the environment variable, one line per operation goes to stderr.
std::vector<DeviceTensor> execute(Executable& exe, const std::vector<DeviceTensor>& inputs,
                                  double* encode_s, double* gpu_s);

}  // namespace mhlo
