// PJRT plugin (C API 0.90) over the C++ host: GetPjrtApi() returns the function table
// declared in include/pjrt_abi.h.  Behaviour follows the reference plugin
// (Sources/PJRTMetalHLO): platform "metalhlo" / version "0.1.0", one device (id 0), one
// memory space "device" (PJRTTopology.swift:106-107, PJRTClient.swift:42-50);
// Compile takes StableHLO text (MLIR bytecode is converted by a jaxlib subprocess when one
// is available, as PJRTExecutable.swift:23-239 does, else refused); Execute is synchronous
// and single-device (PJRTExecutable.swift:2020-2098); a serialized executable is
// `u32 1 | u64 length | MLIR text` and loading it recompiles (:342-359, :2148-2208).
// Differences: buffers are explicit device allocations and H2D / D2H are asynchronous
// (the reference copies eagerly into unified memory and returns complete events,
// PJRTBuffer.swift:98-148): a host buffer is staged into pinned memory during the call (so
// done_with_host_buffer is complete at return) and DMA'd with hipMemcpyAsync on the client's
// stream; a download DMAs into pinned memory and a completion thread, woken by the HIP event
// recorded behind the copy, moves the bytes to the caller's destination and completes the
// PJRT event (Await blocks, OnReady callbacks run on that thread).  Transfers above 256 MiB
// take the synchronous path.  Device attributes describe the GPU (architecture, CU count) instead of the ANE;
// the fingerprint is a stable FNV-1a hash of the program text.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include <atomic>
#include <algorithm>
#include <chrono>
#include <condition_variable>
#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "../../../include/mhip.h"
#include "../../../include/pjrt_abi.h"
#include "../host/executor.h"

using namespace mhlo;

// ---- opaque objects --------------------------------------------------------------------
struct PJRT_Error {
    PJRT_Error_Code code;
    std::string message;
};

// Completion state, shared between the PJRT_Event handles given out for it and the transfer
// that completes it (a handle may be destroyed first).
struct EventState {
    std::mutex mu;
    std::condition_variable cv;
    bool ready = true;
    PJRT_Error_Code code = PJRT_Error_Code_OK;
    std::string message;
    std::vector<std::pair<PJRT_Event_OnReadyCallback, void*>> waiting;
};

struct PJRT_Event {
    std::shared_ptr<EventState> state = std::make_shared<EventState>();
};

// Pinned staging memory and the thread that finishes transfers.  A transfer records a HIP event
// behind its hipMemcpyAsync and queues {event, finish}; the thread waits for the events in queue
// order (= stream order) and runs `finish` (copy out of the staging block, release it, complete
// the PJRT event).
struct TransferEngine {
    static constexpr size_t kStageMax = (size_t)256 << 20;
    struct Task { hipEvent_t done; std::function<void()> finish; };
    std::mutex mu;
    std::condition_variable cv;
    std::deque<Task> queue;
    std::multimap<size_t, void*> free_blocks;      // pinned, by capacity
    std::vector<hipEvent_t> free_events;
    std::thread worker;
    bool running = false, stop = false;

    static size_t capacity(size_t bytes) { size_t b = 4096; while (b < bytes) b <<= 1; return b; }
    void* stage(size_t bytes) {
        const size_t cap = capacity(bytes);
        {
            std::lock_guard<std::mutex> g(mu);
            auto it = free_blocks.find(cap);
            if (it != free_blocks.end()) { void* p = it->second; free_blocks.erase(it); return p; }
        }
        void* p = nullptr;
        if (hipHostMalloc(&p, cap, hipHostMallocDefault) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
        return p;
    }
    void unstage(void* p, size_t bytes) {
        std::lock_guard<std::mutex> g(mu);
        free_blocks.emplace(capacity(bytes), p);
    }
    void start() {
        running = true;
        worker = std::thread([this] {
            (void)hipSetDevice(0);
            for (;;) {
                Task t;
                {
                    std::unique_lock<std::mutex> g(mu);
                    cv.wait(g, [this] { return stop || !queue.empty(); });
                    if (queue.empty()) return;          // stop requested and nothing left
                    t = std::move(queue.front());
                    queue.pop_front();
                }
                (void)hipEventSynchronize(t.done);
                t.finish();
                std::lock_guard<std::mutex> g(mu);
                free_events.push_back(t.done);
            }
        });
    }
    // `finish` runs on the completion thread once everything queued on `stream` so far is done.
    // False (nothing queued, `finish` not run) when no event can be recorded.
    bool after(hipStream_t stream, std::function<void()> finish) {
        if (!running) return false;
        hipEvent_t e = nullptr;
        {
            std::lock_guard<std::mutex> g(mu);
            if (!free_events.empty()) { e = free_events.back(); free_events.pop_back(); }
        }
        if (!e && hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) { (void)hipGetLastError(); return false; }
        if (hipEventRecord(e, stream) != hipSuccess) {
            (void)hipGetLastError();
            std::lock_guard<std::mutex> g(mu);
            free_events.push_back(e);
            return false;
        }
        {
            std::lock_guard<std::mutex> g(mu);
            queue.push_back(Task{e, std::move(finish)});
        }
        cv.notify_one();
        return true;
    }
    void shutdown() {
        if (running) {
            { std::lock_guard<std::mutex> g(mu); stop = true; }
            cv.notify_all();
            worker.join();                               // drains the queue first
            running = false;
        }
        for (auto& kv : free_blocks) (void)hipHostFree(kv.second);
        free_blocks.clear();
        for (auto e : free_events) (void)hipEventDestroy(e);
        free_events.clear();
    }
};

struct PJRT_DeviceDescription {
    int id = 0;
    std::string kind, debug_string, to_string;
    std::string arch;
    std::vector<PJRT_NamedValue> attributes;   // point into the strings / values above
    int64_t compute_units = 0;
};

struct PJRT_Memory {
    PJRT_Client* client = nullptr;
    int id = 0;
    std::string kind = "device", debug_string = "MetalHLO device memory 0", to_string = "DEVICE_0";
};

struct PJRT_Device {
    PJRT_Client* client = nullptr;
    PJRT_DeviceDescription description;
};

struct PJRT_TopologyDescription {
    std::string platform_name = "metalhlo", platform_version = "0.1.0";
    std::vector<PJRT_DeviceDescription*> descriptions;
    std::unique_ptr<PJRT_DeviceDescription> owned;   // standalone topologies own their description
};

struct PJRT_Client {
    Client host;
    std::string platform_name = "metalhlo", platform_version = "0.1.0";
    PJRT_Device device;
    PJRT_Memory memory;
    std::vector<PJRT_Device*> devices;
    std::vector<PJRT_Memory*> memories;
    PJRT_TopologyDescription topology;
    TransferEngine transfers;
};

struct PJRT_Buffer {
    PJRT_Client* client = nullptr;
    DeviceTensor tensor;
    std::shared_ptr<EventState> ready;         // the upload that fills it, while in flight (null: ready)
    std::vector<int64_t> dims;
    bool deleted = false;
    std::atomic<int> external_refs{0};
    std::mutex mu;
};

namespace {

// What a compiled program needs, shared by PJRT_Executable and PJRT_LoadedExecutable.
struct Program {
    Executable exe;
    std::string mlir, name, fingerprint;
    std::vector<PJRT_Buffer_Type> out_types;
    std::vector<int64_t> out_dims;             // all outputs back to back
    std::vector<size_t> out_ranks;
    std::vector<const char*> out_memory_kinds;
    std::vector<size_t> out_memory_kind_sizes;
};

}  // namespace

struct PJRT_Executable {
    std::shared_ptr<Program> program;
};

struct PJRT_LoadedExecutable {
    PJRT_Client* client = nullptr;
    std::shared_ptr<Program> program;
    bool deleted = false;
};

struct PJRT_SerializedExecutable {
    std::string bytes;
};
struct PJRT_DeviceAssignmentSerialized {
    std::string bytes;
};

namespace {

PJRT_Error* make_error(PJRT_Error_Code code, const std::string& msg) { return new PJRT_Error{code, msg}; }
PJRT_Error* invalid(const std::string& msg) { return make_error(PJRT_Error_Code_INVALID_ARGUMENT, msg); }
PJRT_Error* unimplemented(const char* what) {
    return make_error(PJRT_Error_Code_UNIMPLEMENTED, std::string(what) + " is not implemented by the MetalHLO HIP plugin");
}
#define REQUIRE_ARGS(args, name) \
    if (!(args)) return invalid(std::string(name) + ": args is null")
#define REQUIRE(field, name) \
    if (!(field)) return invalid(std::string(name) + " is null")

// Runs `body`, translating the host's exceptions into PJRT errors.
PJRT_Error* guarded(const std::function<void()>& body) {
    try {
        body();
        return nullptr;
    } catch (const ParseError& e) { return invalid(std::string("Parse failed: ") + e.what());
    } catch (const UnsupportedOp& e) { return make_error(PJRT_Error_Code_UNIMPLEMENTED, std::string("Unsupported operation: ") + e.what());
    } catch (const InputMismatch& e) { return invalid(e.what());
    } catch (const NoDevice& e) { return make_error(PJRT_Error_Code_FAILED_PRECONDITION, e.what());
    } catch (const BufferError& e) { return make_error(PJRT_Error_Code_RESOURCE_EXHAUSTED, e.what());
    } catch (const ExecError& e) { return make_error(PJRT_Error_Code_INTERNAL, std::string("Execution failed: ") + e.what());
    } catch (const std::bad_alloc&) { return make_error(PJRT_Error_Code_RESOURCE_EXHAUSTED, "out of host memory");
    } catch (const std::exception& e) { return make_error(PJRT_Error_Code_INTERNAL, e.what()); }
}

int to_dtype(PJRT_Buffer_Type t) {
    switch (t) {
        case PJRT_Buffer_Type_PRED: return I1;
        case PJRT_Buffer_Type_S8: return I8;
        case PJRT_Buffer_Type_S16: return I16;
        case PJRT_Buffer_Type_S32: return I32;
        case PJRT_Buffer_Type_S64: return I64;
        case PJRT_Buffer_Type_U8: return UI8;
        case PJRT_Buffer_Type_U16: return UI16;
        case PJRT_Buffer_Type_U32: return UI32;
        case PJRT_Buffer_Type_U64: return UI64;
        case PJRT_Buffer_Type_F16: return F16;
        case PJRT_Buffer_Type_F32: return F32;
        case PJRT_Buffer_Type_F64: return F64;
        case PJRT_Buffer_Type_BF16: return BF16;
        default: return -1;
    }
}
PJRT_Buffer_Type from_dtype(int d) {
    switch (d) {
        case I1: return PJRT_Buffer_Type_PRED;
        case I8: return PJRT_Buffer_Type_S8;
        case I16: return PJRT_Buffer_Type_S16;
        case I32: return PJRT_Buffer_Type_S32;
        case I64: return PJRT_Buffer_Type_S64;
        case UI8: return PJRT_Buffer_Type_U8;
        case UI16: return PJRT_Buffer_Type_U16;
        case UI32: return PJRT_Buffer_Type_U32;
        case UI64: return PJRT_Buffer_Type_U64;
        case F16: return PJRT_Buffer_Type_F16;
        case F32: return PJRT_Buffer_Type_F32;
        case F64: return PJRT_Buffer_Type_F64;
        case BF16: return PJRT_Buffer_Type_BF16;
        default: return PJRT_Buffer_Type_INVALID;
    }
}

PJRT_NamedValue named_string(const char* name, const std::string& v) {
    PJRT_NamedValue n;
    memset(&n, 0, sizeof(n));
    n.struct_size = sizeof(n);
    n.name = name;
    n.name_size = strlen(name);
    n.type = PJRT_NamedValue_kString;
    n.string_value = v.c_str();
    n.value_size = v.size();
    return n;
}
PJRT_NamedValue named_int(const char* name, int64_t v) {
    PJRT_NamedValue n;
    memset(&n, 0, sizeof(n));
    n.struct_size = sizeof(n);
    n.name = name;
    n.name_size = strlen(name);
    n.type = PJRT_NamedValue_kInt64;
    n.int64_value = v;
    n.value_size = 1;
    return n;
}

void describe_device(PJRT_DeviceDescription& d, const Client& host) {
    d.id = 0;
    char arch[128] = {0};
    int cus = 0;
    if (host.device >= 0) mhip_device_info(host.device, &cus, nullptr, arch, sizeof(arch));
    d.arch = arch[0] ? arch : "none";
    d.compute_units = cus;
    d.kind = host.device >= 0 ? host.device_name : "host-only";
    d.debug_string = "MetalHLO HIP device 0: " + d.kind;
    d.to_string = "MetalHloDevice(id=0)";
    d.attributes.clear();
    d.attributes.push_back(named_string("gfx_arch", d.arch));
    d.attributes.push_back(named_int("compute_units", d.compute_units));
}

std::string fnv1a_hex(const std::string& s) {
    uint64_t h = 1469598103934665603ull;
    for (unsigned char c : s) { h ^= c; h *= 1099511628211ull; }
    char buf[17];
    snprintf(buf, sizeof(buf), "%016llx", (unsigned long long)h);
    return buf;
}

bool is_bytecode(const char* code, size_t n) {
    return n >= 4 && (unsigned char)code[0] == 0x4D && (unsigned char)code[1] == 0x4C && (unsigned char)code[2] == 0xEF &&
           (unsigned char)code[3] == 0x52;
}

// MLIR bytecode -> text through jaxlib's MLIR bindings in a subprocess (the reference does the
// same; there is no offline decoder).  METALHLO_PYTHON names the interpreter (default python3).
bool bytecode_to_text(const char* code, size_t n, std::string* text, std::string* why) {
    char in_path[] = "/tmp/mhlo_pjrt_XXXXXX";
    const int fd = mkstemp(in_path);
    if (fd < 0) { *why = "cannot create a temporary file"; return false; }
    const bool wrote = write(fd, code, n) == (ssize_t)n;
    close(fd);
    if (!wrote) { unlink(in_path); *why = "cannot write a temporary file"; return false; }
    const char* py = getenv("METALHLO_PYTHON");
    const std::string cmd = std::string(py && py[0] ? py : "python3") +
        " -c \"import sys\nfrom jaxlib.mlir import ir\nfrom jaxlib.mlir.dialects import stablehlo\n"
        "b = open(sys.argv[1], 'rb').read()\nc = ir.Context()\nstablehlo.register_dialect(c)\n"
        "try:\n    m = stablehlo.deserialize_portable_artifact(c, b)\nexcept Exception:\n    m = ir.Module.parse(b, c)\n"
        "sys.stdout.write(m.operation.get_asm(large_elements_limit=None))\" " + in_path + " 2>/dev/null";
    FILE* p = popen(cmd.c_str(), "r");
    if (!p) { unlink(in_path); *why = "cannot start the converter"; return false; }
    char buf[65536];
    size_t got;
    while ((got = fread(buf, 1, sizeof(buf), p)) > 0) text->append(buf, got);
    const int rc = pclose(p);
    unlink(in_path);
    if (rc != 0 || text->empty()) {
        *why = "MLIR bytecode needs jaxlib's MLIR bindings to be converted to text and no working converter was found "
               "(set METALHLO_PYTHON to an interpreter that has jaxlib, or pass textual StableHLO)";
        return false;
    }
    return true;
}

PJRT_Error* build_program(PJRT_Client* client, const std::string& text, std::shared_ptr<Program>* out) {
    auto prog = std::make_shared<Program>();
    PJRT_Error* err = guarded([&] {
        prog->exe.client = &client->host;
        // METALHLO_OPT_LEVEL = O0 | O1 | O2 | O3, default O2 (PJRTExecutable.swift:1755-1765)
        const char* lvl = getenv("METALHLO_OPT_LEVEL");
        prog->exe.opt_level = !lvl ? 2 : !strcmp(lvl, "O0") ? 0 : !strcmp(lvl, "O1") ? 1 : !strcmp(lvl, "O3") ? 3 : 2;
        // METALHLO_DUMP_MLIR = <directory>: the program as received, mlir_<lines>_<time>.txt (:1701-1706)
        if (const char* dir = getenv("METALHLO_DUMP_MLIR")) {
            const long lines = (long)std::count(text.begin(), text.end(), '\n') + 1;
            const std::string path = std::string(dir) + "/mlir_" + std::to_string(lines) + "_" +
                                     std::to_string(std::chrono::steady_clock::now().time_since_epoch().count()) + ".txt";
            if (FILE* f = fopen(path.c_str(), "w")) { fwrite(text.data(), 1, text.size(), f); fclose(f); }
        }
        prog->exe.fn = build_function(text, prog->exe.opt_level);
        compile(prog->exe);
    });
    if (err) return err;
    prog->mlir = text;
    prog->name = prog->exe.fn.name.empty() ? "main" : prog->exe.fn.name;
    prog->fingerprint = fnv1a_hex(text);
    for (const TensorType& t : prog->exe.fn.result_types) {
        prog->out_types.push_back(from_dtype(t.dtype));
        prog->out_ranks.push_back(t.shape.size());
        for (int64_t d : t.shape) prog->out_dims.push_back(d);
        prog->out_memory_kinds.push_back("device");
        prog->out_memory_kind_sizes.push_back(6);
    }
    *out = prog;
    return nullptr;
}

PJRT_Event* complete_event() { return new PJRT_Event(); }

// ---- errors ------------------------------------------------------------------------------
void Error_Destroy(PJRT_Error_Destroy_Args* a) { if (a) delete a->error; }
void Error_Message(PJRT_Error_Message_Args* a) {
    if (!a) return;
    a->message = a->error ? a->error->message.c_str() : "";
    a->message_size = a->error ? a->error->message.size() : 0;
}
PJRT_Error* Error_GetCode(PJRT_Error_GetCode_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Error_GetCode");
    REQUIRE(a->error, "error");
    a->code = a->error->code;
    return nullptr;
}

// ---- plugin ------------------------------------------------------------------------------
PJRT_Error* Plugin_Initialize(PJRT_Plugin_Initialize_Args* a) { REQUIRE_ARGS(a, "PJRT_Plugin_Initialize"); return nullptr; }
PJRT_Error* Plugin_Attributes(PJRT_Plugin_Attributes_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Plugin_Attributes");
    static const std::string version = "0.1.0";
    static const PJRT_NamedValue attrs[] = {named_int("xla_version", 2), named_int("stablehlo_current_version", 1),
                                            named_string("plugin_version", version)};
    a->attributes = attrs;
    a->num_attributes = sizeof(attrs) / sizeof(attrs[0]);
    return nullptr;
}

// ---- events ------------------------------------------------------------------------------
PJRT_Error* Event_Destroy(PJRT_Event_Destroy_Args* a) { REQUIRE_ARGS(a, "PJRT_Event_Destroy"); delete a->event; return nullptr; }
PJRT_Error* Event_IsReady(PJRT_Event_IsReady_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Event_IsReady");
    REQUIRE(a->event, "event");
    std::lock_guard<std::mutex> lock(a->event->state->mu);
    a->is_ready = a->event->state->ready;
    return nullptr;
}
PJRT_Error* status_of(EventState& st) {      // st.mu held by the caller
    return st.code == PJRT_Error_Code_OK ? nullptr : make_error(st.code, st.message);
}
PJRT_Error* Event_Error(PJRT_Event_Error_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Event_Error");
    REQUIRE(a->event, "event");
    std::lock_guard<std::mutex> lock(a->event->state->mu);
    if (!a->event->state->ready) return make_error(PJRT_Error_Code_FAILED_PRECONDITION, "the event is not ready yet");
    return status_of(*a->event->state);
}
PJRT_Error* Event_Await(PJRT_Event_Await_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Event_Await");
    REQUIRE(a->event, "event");
    EventState& st = *a->event->state;
    std::unique_lock<std::mutex> lock(st.mu);
    if (!st.cv.wait_for(lock, std::chrono::seconds(300), [&] { return st.ready; }))
        return make_error(PJRT_Error_Code_DEADLINE_EXCEEDED, "the transfer did not complete within 300 s");
    return status_of(st);
}
PJRT_Error* Event_OnReady(PJRT_Event_OnReady_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Event_OnReady");
    REQUIRE(a->event, "event");
    REQUIRE(a->callback, "callback");
    EventState& st = *a->event->state;
    PJRT_Error* status = nullptr;
    {
        std::lock_guard<std::mutex> lock(st.mu);
        if (!st.ready) {                        // runs on the completion thread when the transfer ends
            st.waiting.emplace_back(a->callback, a->user_arg);
            return nullptr;
        }
        status = status_of(st);
    }
    a->callback(status, a->user_arg);           // already complete: inline on the calling thread; the callback owns the error
    return nullptr;
}

// Marks a pending event complete, wakes the waiters and runs the callbacks registered so far.
void complete(const std::shared_ptr<EventState>& st, PJRT_Error_Code code = PJRT_Error_Code_OK, const std::string& message = "") {
    std::vector<std::pair<PJRT_Event_OnReadyCallback, void*>> run;
    {
        std::lock_guard<std::mutex> lock(st->mu);
        st->ready = true;
        st->code = code;
        st->message = message;
        run.swap(st->waiting);
    }
    st->cv.notify_all();
    for (auto& cb : run) cb.first(code == PJRT_Error_Code_OK ? nullptr : make_error(code, message), cb.second);
}
std::shared_ptr<EventState> pending_state() {
    auto st = std::make_shared<EventState>();
    st->ready = false;
    return st;
}
PJRT_Event* event_for(const std::shared_ptr<EventState>& st) {
    PJRT_Event* e = new PJRT_Event();
    if (st) e->state = st;
    return e;
}

// ---- client ------------------------------------------------------------------------------
PJRT_Error* Client_Create(PJRT_Client_Create_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_Create");
    const int n = mhip_device_count();
    const char* allow = getenv("METALHLO_ALLOW_NO_DEVICE");
    if (n <= 0 && !(allow && allow[0] == '1')) return make_error(PJRT_Error_Code_FAILED_PRECONDITION, "No HIP device found");
    PJRT_Client* c = new PJRT_Client();
    if (n > 0) {
        c->host.device = 0;
        if (hipSetDevice(0) != hipSuccess || hipStreamCreate(&c->host.stream) != hipSuccess) {
            delete c;
            return make_error(PJRT_Error_Code_INTERNAL, "cannot initialise HIP device 0");
        }
        hipDeviceProp_t p;
        c->host.device_name = hipGetDeviceProperties(&p, 0) == hipSuccess && p.name[0] ? std::string(p.name) : std::string("AMD GPU");
        char arch[128] = {0};
        int cus = 0;
        mhip_device_info(0, &cus, nullptr, arch, sizeof(arch));
        c->host.device_name += std::string(" (") + arch + ", " + std::to_string(cus) + " CUs)";
        const char* sync = getenv("METALHLO_PJRT_SYNC_TRANSFERS");
        if (!(sync && sync[0] == '1')) c->transfers.start();
    } else {
        c->host.device_name = "none (host-only client)";
    }
    c->device.client = c;
    describe_device(c->device.description, c->host);
    c->memory.client = c;
    c->devices = {&c->device};
    c->memories = {&c->memory};
    c->topology.descriptions = {&c->device.description};
    a->client = c;
    return nullptr;
}
PJRT_Error* Client_Destroy(PJRT_Client_Destroy_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_Destroy");
    if (a->client) {
        if (a->client->host.stream) (void)hipStreamSynchronize(a->client->host.stream);
        a->client->transfers.shutdown();          // finishes what is still queued, then frees the staging memory
        if (a->client->host.stream) (void)hipStreamDestroy(a->client->host.stream);
        delete a->client;
    }
    return nullptr;
}
PJRT_Error* Client_PlatformName(PJRT_Client_PlatformName_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_PlatformName");
    REQUIRE(a->client, "client");
    a->platform_name = a->client->platform_name.c_str();
    a->platform_name_size = a->client->platform_name.size();
    return nullptr;
}
PJRT_Error* Client_ProcessIndex(PJRT_Client_ProcessIndex_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_ProcessIndex");
    REQUIRE(a->client, "client");
    a->process_index = 0;
    return nullptr;
}
PJRT_Error* Client_PlatformVersion(PJRT_Client_PlatformVersion_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_PlatformVersion");
    REQUIRE(a->client, "client");
    a->platform_version = a->client->platform_version.c_str();
    a->platform_version_size = a->client->platform_version.size();
    return nullptr;
}
PJRT_Error* Client_TopologyDescription(PJRT_Client_TopologyDescription_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_TopologyDescription");
    REQUIRE(a->client, "client");
    a->topology = &a->client->topology;
    return nullptr;
}
PJRT_Error* Client_Devices(PJRT_Client_Devices_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_Devices");
    REQUIRE(a->client, "client");
    a->devices = a->client->devices.data();
    a->num_devices = a->client->devices.size();
    return nullptr;
}
PJRT_Error* Client_AddressableDevices(PJRT_Client_AddressableDevices_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_AddressableDevices");
    REQUIRE(a->client, "client");
    a->addressable_devices = a->client->devices.data();
    a->num_addressable_devices = a->client->devices.size();
    return nullptr;
}
PJRT_Error* Client_LookupDevice(PJRT_Client_LookupDevice_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_LookupDevice");
    REQUIRE(a->client, "client");
    if (a->id != 0) return make_error(PJRT_Error_Code_NOT_FOUND, "no device with id " + std::to_string(a->id));
    a->device = &a->client->device;
    return nullptr;
}
PJRT_Error* Client_LookupAddressableDevice(PJRT_Client_LookupAddressableDevice_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_LookupAddressableDevice");
    REQUIRE(a->client, "client");
    if (a->local_hardware_id != 0)
        return make_error(PJRT_Error_Code_NOT_FOUND, "no addressable device with local hardware id " + std::to_string(a->local_hardware_id));
    a->addressable_device = &a->client->device;
    return nullptr;
}
PJRT_Error* Client_AddressableMemories(PJRT_Client_AddressableMemories_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_AddressableMemories");
    REQUIRE(a->client, "client");
    a->addressable_memories = a->client->memories.data();
    a->num_addressable_memories = a->client->memories.size();
    return nullptr;
}
PJRT_Error* Client_Compile(PJRT_Client_Compile_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_Compile");
    REQUIRE(a->client, "client");
    REQUIRE(a->program, "program");
    REQUIRE(a->program->code, "program code");
    const std::string format(a->program->format ? a->program->format : "mlir", a->program->format ? a->program->format_size : 4);
    if (format != "mlir")
        return invalid("program format '" + format + "' is not supported: pass StableHLO as 'mlir'");
    std::string text;
    if (is_bytecode(a->program->code, a->program->code_size)) {
        std::string why;
        if (!bytecode_to_text(a->program->code, a->program->code_size, &text, &why)) return make_error(PJRT_Error_Code_UNIMPLEMENTED, why);
    } else {
        text.assign(a->program->code, a->program->code_size);
    }
    std::shared_ptr<Program> prog;
    if (PJRT_Error* err = build_program(a->client, text, &prog)) return err;
    a->executable = new PJRT_LoadedExecutable{a->client, prog, false};
    return nullptr;
}
PJRT_Error* Client_DefaultDeviceAssignment(PJRT_Client_DefaultDeviceAssignment_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_DefaultDeviceAssignment");
    REQUIRE(a->client, "client");
    const int64_t need = (int64_t)a->num_replicas * a->num_partitions;
    if (a->num_replicas < 0 || a->num_partitions < 0 || (size_t)need > a->default_assignment_size)
        return invalid("default_assignment holds " + std::to_string(a->default_assignment_size) + " entries, " + std::to_string(need) + " needed");
    if (need > 1) return make_error(PJRT_Error_Code_UNIMPLEMENTED, "one device only: replicas x partitions must be 1");
    if (need > 0) { REQUIRE(a->default_assignment, "default_assignment"); a->default_assignment[0] = 0; }
    return nullptr;
}
PJRT_Error* Client_BufferFromHostBuffer(PJRT_Client_BufferFromHostBuffer_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Client_BufferFromHostBuffer");
    REQUIRE(a->client, "client");
    if (a->num_dims > 0) REQUIRE(a->dims, "dims");
    const int dt = to_dtype(a->type);
    if (dt < 0) return invalid("element type " + std::to_string((int)a->type) + " is not supported (F16, F32, F64, BF16, PRED, S8-S64, U8-U64)");
    TensorType t;
    t.dtype = dt;
    for (size_t i = 0; i < a->num_dims; i++) {
        if (a->dims[i] < 0) return invalid("negative dimension");
        t.shape.push_back(a->dims[i]);
    }
    if (a->byte_strides && a->num_byte_strides) {           // dense row-major only
        if (a->num_byte_strides != a->num_dims) return invalid("byte_strides must have one entry per dimension");
        int64_t expect = dtype_bytes(dt);
        for (size_t i = a->num_dims; i-- > 0;) {
            if (t.shape[i] > 1 && a->byte_strides[i] != expect)
                return make_error(PJRT_Error_Code_UNIMPLEMENTED, "only dense row-major host buffers are supported");
            expect *= t.shape[i];
        }
    }
    if (t.bytes() > 0) REQUIRE(a->data, "data");
    PJRT_Client* c = a->client;
    PJRT_Buffer* b = nullptr;
    PJRT_Error* err = guarded([&] {
        DeviceTensor d = c->host.allocate(t);
        std::shared_ptr<EventState> ready;
        const size_t n = t.bytes();
        void* staged = n && n <= TransferEngine::kStageMax && c->transfers.running ? c->transfers.stage(n) : nullptr;
        if (staged) {
            // the caller's memory is read here and never again; the DMA runs behind this call
            memcpy(staged, a->data, n);
            std::lock_guard<std::mutex> stream_lock(c->host.stream_mu);     // not into a graph capture
            if (hipMemcpyAsync(d.data(), staged, n, hipMemcpyHostToDevice, c->host.stream) != hipSuccess) {
                (void)hipGetLastError();
                c->transfers.unstage(staged, n);
                throw BufferError("host to device copy failed");
            }
            ready = pending_state();
            TransferEngine* eng = &c->transfers;
            auto finish = [eng, staged, n, ready] { eng->unstage(staged, n); complete(ready); };
            if (!c->transfers.after(c->host.stream, finish)) {
                (void)hipStreamSynchronize(c->host.stream);
                finish();
            }
        } else if (n) {
            std::lock_guard<std::mutex> stream_lock(c->host.stream_mu);
            if (hipMemcpyAsync(d.data(), a->data, n, hipMemcpyHostToDevice, c->host.stream) != hipSuccess ||
                hipStreamSynchronize(c->host.stream) != hipSuccess) {
                (void)hipGetLastError();
                throw BufferError("host to device copy failed");
            }
        }
        b = new PJRT_Buffer();
        b->client = c;
        b->tensor = d;
        b->dims = t.shape;
        b->ready = ready;
    });
    if (err) return err;
    a->buffer = b;
    a->done_with_host_buffer = complete_event();          // staged or copied: the host buffer is free
    return nullptr;
}

// ---- device descriptions, devices, memories ------------------------------------------------
PJRT_Error* DeviceDescription_Id(PJRT_DeviceDescription_Id_Args* a) {
    REQUIRE_ARGS(a, "PJRT_DeviceDescription_Id"); REQUIRE(a->device_description, "device_description");
    a->id = a->device_description->id;
    return nullptr;
}
PJRT_Error* DeviceDescription_ProcessIndex(PJRT_DeviceDescription_ProcessIndex_Args* a) {
    REQUIRE_ARGS(a, "PJRT_DeviceDescription_ProcessIndex"); REQUIRE(a->device_description, "device_description");
    a->process_index = 0;
    return nullptr;
}
PJRT_Error* DeviceDescription_Attributes(PJRT_DeviceDescription_Attributes_Args* a) {
    REQUIRE_ARGS(a, "PJRT_DeviceDescription_Attributes"); REQUIRE(a->device_description, "device_description");
    a->attributes = a->device_description->attributes.data();
    a->num_attributes = a->device_description->attributes.size();
    return nullptr;
}
PJRT_Error* DeviceDescription_Kind(PJRT_DeviceDescription_Kind_Args* a) {
    REQUIRE_ARGS(a, "PJRT_DeviceDescription_Kind"); REQUIRE(a->device_description, "device_description");
    a->device_kind = a->device_description->kind.c_str();
    a->device_kind_size = a->device_description->kind.size();
    return nullptr;
}
PJRT_Error* DeviceDescription_DebugString(PJRT_DeviceDescription_DebugString_Args* a) {
    REQUIRE_ARGS(a, "PJRT_DeviceDescription_DebugString"); REQUIRE(a->device_description, "device_description");
    a->debug_string = a->device_description->debug_string.c_str();
    a->debug_string_size = a->device_description->debug_string.size();
    return nullptr;
}
PJRT_Error* DeviceDescription_ToString(PJRT_DeviceDescription_ToString_Args* a) {
    REQUIRE_ARGS(a, "PJRT_DeviceDescription_ToString"); REQUIRE(a->device_description, "device_description");
    a->to_string = a->device_description->to_string.c_str();
    a->to_string_size = a->device_description->to_string.size();
    return nullptr;
}
PJRT_Error* Device_GetDescription(PJRT_Device_GetDescription_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Device_GetDescription"); REQUIRE(a->device, "device");
    a->device_description = &a->device->description;
    return nullptr;
}
PJRT_Error* Device_IsAddressable(PJRT_Device_IsAddressable_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Device_IsAddressable"); REQUIRE(a->device, "device");
    a->is_addressable = true;
    return nullptr;
}
PJRT_Error* Device_LocalHardwareId(PJRT_Device_LocalHardwareId_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Device_LocalHardwareId"); REQUIRE(a->device, "device");
    a->local_hardware_id = 0;
    return nullptr;
}
PJRT_Error* Device_AddressableMemories(PJRT_Device_AddressableMemories_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Device_AddressableMemories"); REQUIRE(a->device, "device");
    a->memories = a->device->client->memories.data();
    a->num_memories = a->device->client->memories.size();
    return nullptr;
}
PJRT_Error* Device_DefaultMemory(PJRT_Device_DefaultMemory_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Device_DefaultMemory"); REQUIRE(a->device, "device");
    a->memory = &a->device->client->memory;
    return nullptr;
}
PJRT_Error* Device_MemoryStats(PJRT_Device_MemoryStats_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Device_MemoryStats"); REQUIRE(a->device, "device");
    if (a->device->client->host.device < 0) return make_error(PJRT_Error_Code_FAILED_PRECONDITION, "the client has no device");
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) { (void)hipGetLastError(); return make_error(PJRT_Error_Code_INTERNAL, "hipMemGetInfo failed"); }
    PJRT_Device* dev = a->device;
    const size_t sz = a->struct_size;
    PJRT_Extension_Base* ext = a->extension_start;
    memset(a, 0, sizeof(*a));
    a->struct_size = sz;
    a->extension_start = ext;
    a->device = dev;
    a->bytes_in_use = (int64_t)(total_b - free_b);
    a->bytes_limit = (int64_t)total_b;
    a->bytes_limit_is_set = true;
    return nullptr;
}
PJRT_Error* Memory_Id(PJRT_Memory_Id_Args* a) { REQUIRE_ARGS(a, "PJRT_Memory_Id"); REQUIRE(a->memory, "memory"); a->id = a->memory->id; return nullptr; }
PJRT_Error* Memory_Kind(PJRT_Memory_Kind_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Memory_Kind"); REQUIRE(a->memory, "memory");
    a->kind = a->memory->kind.c_str();
    a->kind_size = a->memory->kind.size();
    return nullptr;
}
PJRT_Error* Memory_Kind_Id(PJRT_Memory_Kind_Id_Args* a) { REQUIRE_ARGS(a, "PJRT_Memory_Kind_Id"); REQUIRE(a->memory, "memory"); a->kind_id = 0; return nullptr; }
PJRT_Error* Memory_DebugString(PJRT_Memory_DebugString_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Memory_DebugString"); REQUIRE(a->memory, "memory");
    a->debug_string = a->memory->debug_string.c_str();
    a->debug_string_size = a->memory->debug_string.size();
    return nullptr;
}
PJRT_Error* Memory_ToString(PJRT_Memory_ToString_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Memory_ToString"); REQUIRE(a->memory, "memory");
    a->to_string = a->memory->to_string.c_str();
    a->to_string_size = a->memory->to_string.size();
    return nullptr;
}
PJRT_Error* Memory_AddressableByDevices(PJRT_Memory_AddressableByDevices_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Memory_AddressableByDevices"); REQUIRE(a->memory, "memory");
    a->devices = a->memory->client->devices.data();
    a->num_devices = a->memory->client->devices.size();
    return nullptr;
}

// ---- executables -----------------------------------------------------------------------------
#define EXE(a, name) REQUIRE_ARGS(a, name); REQUIRE(a->executable, "executable"); Program& p = *a->executable->program
PJRT_Error* Executable_Destroy(PJRT_Executable_Destroy_Args* a) { REQUIRE_ARGS(a, "PJRT_Executable_Destroy"); delete a->executable; return nullptr; }
PJRT_Error* Executable_Name(PJRT_Executable_Name_Args* a) {
    EXE(a, "PJRT_Executable_Name");
    a->executable_name = p.name.c_str();
    a->executable_name_size = p.name.size();
    return nullptr;
}
PJRT_Error* Executable_NumReplicas(PJRT_Executable_NumReplicas_Args* a) { EXE(a, "PJRT_Executable_NumReplicas"); (void)p; a->num_replicas = 1; return nullptr; }
PJRT_Error* Executable_NumPartitions(PJRT_Executable_NumPartitions_Args* a) { EXE(a, "PJRT_Executable_NumPartitions"); (void)p; a->num_partitions = 1; return nullptr; }
PJRT_Error* Executable_NumOutputs(PJRT_Executable_NumOutputs_Args* a) { EXE(a, "PJRT_Executable_NumOutputs"); a->num_outputs = p.out_types.size(); return nullptr; }
PJRT_Error* Executable_SizeOfGeneratedCodeInBytes(PJRT_Executable_SizeOfGeneratedCodeInBytes_Args* a) {
    EXE(a, "PJRT_Executable_SizeOfGeneratedCodeInBytes");
    a->size_in_bytes = (int64_t)p.mlir.size();             // no machine code is generated per program: the kernels are prebuilt
    return nullptr;
}
PJRT_Error* Executable_GetCostAnalysis(PJRT_Executable_GetCostAnalysis_Args* a) {
    EXE(a, "PJRT_Executable_GetCostAnalysis"); (void)p;
    a->num_properties = 0;
    a->properties = nullptr;
    return nullptr;
}
PJRT_Error* Executable_OutputMemoryKinds(PJRT_Executable_OutputMemoryKinds_Args* a) {
    EXE(a, "PJRT_Executable_OutputMemoryKinds");
    a->num_outputs = p.out_memory_kinds.size();
    a->memory_kinds = p.out_memory_kinds.data();
    a->memory_kind_sizes = p.out_memory_kind_sizes.data();
    return nullptr;
}
PJRT_Error* Executable_OptimizedProgram(PJRT_Executable_OptimizedProgram_Args* a) { REQUIRE_ARGS(a, "PJRT_Executable_OptimizedProgram"); return unimplemented("PJRT_Executable_OptimizedProgram"); }
void free_serialized(PJRT_SerializedExecutable* s) { delete s; }
PJRT_Error* Executable_Serialize(PJRT_Executable_Serialize_Args* a) {
    EXE(a, "PJRT_Executable_Serialize");
    auto* s = new PJRT_SerializedExecutable();
    const uint32_t version = 1;
    const uint64_t len = p.mlir.size();
    s->bytes.append(reinterpret_cast<const char*>(&version), 4);
    s->bytes.append(reinterpret_cast<const char*>(&len), 8);
    s->bytes.append(p.mlir);
    a->serialized_bytes = s->bytes.data();
    a->serialized_bytes_size = s->bytes.size();
    a->serialized_executable = s;
    a->serialized_executable_deleter = free_serialized;
    return nullptr;
}
PJRT_Error* Executable_OutputElementTypes(PJRT_Executable_OutputElementTypes_Args* a) {
    EXE(a, "PJRT_Executable_OutputElementTypes");
    a->output_types = p.out_types.data();
    a->num_output_types = p.out_types.size();
    return nullptr;
}
PJRT_Error* Executable_OutputDimensions(PJRT_Executable_OutputDimensions_Args* a) {
    EXE(a, "PJRT_Executable_OutputDimensions");
    a->num_outputs = p.out_ranks.size();
    a->dims = p.out_dims.data();
    a->dim_sizes = p.out_ranks.data();
    return nullptr;
}
PJRT_Error* Executable_Fingerprint(PJRT_Executable_Fingerprint_Args* a) {
    EXE(a, "PJRT_Executable_Fingerprint");
    a->executable_fingerprint = p.fingerprint.c_str();
    a->executable_fingerprint_size = p.fingerprint.size();
    return nullptr;
}
PJRT_Error* Executable_GetCompiledMemoryStats(PJRT_Executable_GetCompiledMemoryStats_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Executable_GetCompiledMemoryStats");
    REQUIRE(a->executable, "executable");
    // the reference leaves this unimplemented; here the memory plan made at compile time answers it
    const Executable& exe = a->executable->program->exe;
    int64_t args = 0, outs = 0;
    for (auto& t : exe.fn.arg_types) args += (int64_t)t.bytes();
    for (auto& t : exe.fn.result_types) outs += (int64_t)t.bytes();
    a->generated_code_size_in_bytes = 0;               // the kernels are prebuilt: nothing is generated per program
    a->argument_size_in_bytes = args;
    a->output_size_in_bytes = outs;
    a->alias_size_in_bytes = 0;
    a->temp_size_in_bytes = (int64_t)exe.plan.core_bytes;   // the arena all intermediates share
    a->host_generated_code_size_in_bytes = a->host_argument_size_in_bytes = a->host_output_size_in_bytes = 0;
    a->host_alias_size_in_bytes = a->host_temp_size_in_bytes = 0;
    a->peak_memory_in_bytes = args + outs + (int64_t)exe.plan.core_bytes;
    a->total_size_in_bytes = a->peak_memory_in_bytes;
    return nullptr;
}

PJRT_Error* LoadedExecutable_Destroy(PJRT_LoadedExecutable_Destroy_Args* a) { REQUIRE_ARGS(a, "PJRT_LoadedExecutable_Destroy"); delete a->executable; return nullptr; }
PJRT_Error* LoadedExecutable_GetExecutable(PJRT_LoadedExecutable_GetExecutable_Args* a) {
    REQUIRE_ARGS(a, "PJRT_LoadedExecutable_GetExecutable"); REQUIRE(a->loaded_executable, "loaded_executable");
    a->executable = new PJRT_Executable{a->loaded_executable->program};
    return nullptr;
}
PJRT_Error* LoadedExecutable_AddressableDevices(PJRT_LoadedExecutable_AddressableDevices_Args* a) {
    REQUIRE_ARGS(a, "PJRT_LoadedExecutable_AddressableDevices"); REQUIRE(a->executable, "executable");
    a->addressable_devices = a->executable->client->devices.data();
    a->num_addressable_devices = a->executable->client->devices.size();
    return nullptr;
}
PJRT_Error* LoadedExecutable_Delete(PJRT_LoadedExecutable_Delete_Args* a) {
    REQUIRE_ARGS(a, "PJRT_LoadedExecutable_Delete"); REQUIRE(a->executable, "executable");
    a->executable->deleted = true;
    return nullptr;
}
PJRT_Error* LoadedExecutable_IsDeleted(PJRT_LoadedExecutable_IsDeleted_Args* a) {
    REQUIRE_ARGS(a, "PJRT_LoadedExecutable_IsDeleted"); REQUIRE(a->executable, "executable");
    a->is_deleted = a->executable->deleted;
    return nullptr;
}
PJRT_Error* LoadedExecutable_Fingerprint(PJRT_LoadedExecutable_Fingerprint_Args* a) {
    REQUIRE_ARGS(a, "PJRT_LoadedExecutable_Fingerprint"); REQUIRE(a->executable, "executable");
    a->executable_fingerprint = a->executable->program->fingerprint.c_str();
    a->executable_fingerprint_size = a->executable->program->fingerprint.size();
    return nullptr;
}
void free_assignment(PJRT_DeviceAssignmentSerialized* d) { delete d; }
PJRT_Error* LoadedExecutable_GetDeviceAssignment(PJRT_LoadedExecutable_GetDeviceAssignment_Args* a) {
    REQUIRE_ARGS(a, "PJRT_LoadedExecutable_GetDeviceAssignment"); REQUIRE(a->executable, "executable");
    // DeviceAssignmentProto{replica_count: 1, computation_count: 1, computation_devices: [{replica_device_ids: [0]}]}
    static const unsigned char proto[] = {0x08, 0x01, 0x10, 0x01, 0x1A, 0x02, 0x08, 0x00};
    auto* d = new PJRT_DeviceAssignmentSerialized();
    d->bytes.assign(reinterpret_cast<const char*>(proto), sizeof(proto));
    a->serialized_bytes = d->bytes.data();
    a->serialized_bytes_size = d->bytes.size();
    a->serialized_device_assignment = d;
    a->serialized_device_assignment_deleter = free_assignment;
    return nullptr;
}
PJRT_Error* Executable_DeserializeAndLoad(PJRT_Executable_DeserializeAndLoad_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Executable_DeserializeAndLoad");
    REQUIRE(a->client, "client");
    REQUIRE(a->serialized_executable, "serialized_executable");
    const char* s = a->serialized_executable;
    const size_t n = a->serialized_executable_size;
    if (n < 12) return invalid("serialized executable is truncated (" + std::to_string(n) + " bytes, header needs 12)");
    uint32_t version;
    uint64_t len;
    memcpy(&version, s, 4);
    memcpy(&len, s + 4, 8);
    if (version != 1) return invalid("serialized executable has version " + std::to_string(version) + ", expected 1");
    if (len > n - 12) return invalid("serialized executable is truncated: header announces " + std::to_string(len) + " bytes of program, " +
                                     std::to_string(n - 12) + " present");
    std::shared_ptr<Program> prog;
    if (PJRT_Error* err = build_program(a->client, std::string(s + 12, (size_t)len), &prog)) return err;
    a->loaded_executable = new PJRT_LoadedExecutable{a->client, prog, false};
    return nullptr;
}
PJRT_Error* LoadedExecutable_Execute(PJRT_LoadedExecutable_Execute_Args* a) {
    REQUIRE_ARGS(a, "PJRT_LoadedExecutable_Execute");
    REQUIRE(a->executable, "executable");
    if (a->executable->deleted) return make_error(PJRT_Error_Code_FAILED_PRECONDITION, "the executable was deleted");
    if (a->num_devices != 1) return make_error(PJRT_Error_Code_UNIMPLEMENTED, "execution on " + std::to_string(a->num_devices) + " devices: one device only");
    if (a->num_args > 0) { REQUIRE(a->argument_lists, "argument_lists"); REQUIRE(a->argument_lists[0], "argument_lists[0]"); }
    Program& p = *a->executable->program;
    if (!p.out_types.empty()) { REQUIRE(a->output_lists, "output_lists"); REQUIRE(a->output_lists[0], "output_lists[0]"); }
    std::vector<DeviceTensor> inputs;
    for (size_t i = 0; i < a->num_args; i++) {
        PJRT_Buffer* b = a->argument_lists[0][i];
        if (!b) return invalid("argument " + std::to_string(i) + " is null");
        if (b->deleted) return invalid("argument " + std::to_string(i) + " was deleted");
        inputs.push_back(b->tensor);
    }
    std::vector<DeviceTensor> outputs;
    PJRT_Error* err = guarded([&] {
        double encode_s = 0, gpu_s = 0;
        outputs = execute(p.exe, inputs, &encode_s, &gpu_s);
        if (getenv("METALHLO_PROFILE_PJRT"))
            fprintf(stderr, "[metalhlo pjrt] %s: encode %.3f ms, gpu %.3f ms\n", p.name.c_str(), encode_s * 1e3, gpu_s * 1e3);
    });
    if (err) return err;
    for (size_t i = 0; i < outputs.size(); i++) {
        PJRT_Buffer* b = new PJRT_Buffer();
        b->client = a->executable->client;
        b->tensor = outputs[i];
        b->dims = outputs[i].type.shape;
        a->output_lists[0][i] = b;
    }
    if (a->device_complete_events) a->device_complete_events[0] = complete_event();
    return nullptr;
}

// ---- buffers -----------------------------------------------------------------------------------
#define BUF(a, name) REQUIRE_ARGS(a, name); REQUIRE(a->buffer, "buffer"); PJRT_Buffer& b = *a->buffer
PJRT_Error* Buffer_Destroy(PJRT_Buffer_Destroy_Args* a) { REQUIRE_ARGS(a, "PJRT_Buffer_Destroy"); delete a->buffer; return nullptr; }
PJRT_Error* Buffer_ElementType(PJRT_Buffer_ElementType_Args* a) { BUF(a, "PJRT_Buffer_ElementType"); a->type = from_dtype(b.tensor.type.dtype); return nullptr; }
PJRT_Error* Buffer_Dimensions(PJRT_Buffer_Dimensions_Args* a) { BUF(a, "PJRT_Buffer_Dimensions"); a->dims = b.dims.data(); a->num_dims = b.dims.size(); return nullptr; }
PJRT_Error* Buffer_UnpaddedDimensions(PJRT_Buffer_UnpaddedDimensions_Args* a) {
    BUF(a, "PJRT_Buffer_UnpaddedDimensions");
    a->unpadded_dims = b.dims.data();
    a->num_dims = b.dims.size();
    return nullptr;
}
PJRT_Error* Buffer_DynamicDimensionIndices(PJRT_Buffer_DynamicDimensionIndices_Args* a) {
    BUF(a, "PJRT_Buffer_DynamicDimensionIndices"); (void)b;
    a->dynamic_dim_indices = nullptr;
    a->num_dynamic_dims = 0;
    return nullptr;
}
PJRT_Error* Buffer_GetMemoryLayout(PJRT_Buffer_GetMemoryLayout_Args* a) { REQUIRE_ARGS(a, "PJRT_Buffer_GetMemoryLayout"); return unimplemented("PJRT_Buffer_GetMemoryLayout"); }
PJRT_Error* Buffer_OnDeviceSizeInBytes(PJRT_Buffer_OnDeviceSizeInBytes_Args* a) {
    BUF(a, "PJRT_Buffer_OnDeviceSizeInBytes");
    a->on_device_size_in_bytes = b.tensor.type.bytes();
    return nullptr;
}
PJRT_Error* Buffer_Device(PJRT_Buffer_Device_Args* a) { BUF(a, "PJRT_Buffer_Device"); a->device = &b.client->device; return nullptr; }
PJRT_Error* Buffer_Memory(PJRT_Buffer_Memory_Args* a) { BUF(a, "PJRT_Buffer_Memory"); a->memory = &b.client->memory; return nullptr; }
PJRT_Error* Buffer_Delete(PJRT_Buffer_Delete_Args* a) {
    BUF(a, "PJRT_Buffer_Delete");
    std::lock_guard<std::mutex> lock(b.mu);
    b.deleted = true;
    b.tensor.mem.reset();                                   // the device memory goes back to the pool now
    return nullptr;
}
PJRT_Error* Buffer_IsDeleted(PJRT_Buffer_IsDeleted_Args* a) { BUF(a, "PJRT_Buffer_IsDeleted"); a->is_deleted = b.deleted; return nullptr; }
// Device to host; *event completes when `dst` holds the bytes.
PJRT_Error* copy_to_host(PJRT_Buffer& b, void* dst, size_t offset, size_t bytes, PJRT_Event** event) {
    if (b.deleted) return make_error(PJRT_Error_Code_FAILED_PRECONDITION, "the buffer was deleted");
    *event = nullptr;
    if (bytes == 0) { *event = complete_event(); return nullptr; }
    PJRT_Client* c = b.client;
    const char* src = static_cast<const char*>(b.tensor.data()) + offset;
    void* staged = bytes <= TransferEngine::kStageMax && c->transfers.running ? c->transfers.stage(bytes) : nullptr;
    std::lock_guard<std::mutex> stream_lock(c->host.stream_mu);     // not into a graph capture
    if (staged) {
        if (hipMemcpyAsync(staged, src, bytes, hipMemcpyDeviceToHost, c->host.stream) != hipSuccess) {
            (void)hipGetLastError();
            c->transfers.unstage(staged, bytes);
            return make_error(PJRT_Error_Code_INTERNAL, "device to host copy failed");
        }
        auto st = pending_state();
        TransferEngine* eng = &c->transfers;
        const DeviceTensor keep = b.tensor;      // the device memory outlives the buffer handle until the copy ends
        auto finish = [eng, staged, dst, bytes, st, keep] {
            memcpy(dst, staged, bytes);
            eng->unstage(staged, bytes);
            complete(st);
        };
        if (!c->transfers.after(c->host.stream, finish)) {
            (void)hipStreamSynchronize(c->host.stream);
            finish();
        }
        *event = event_for(st);
        return nullptr;
    }
    if (hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, c->host.stream) != hipSuccess ||
        hipStreamSynchronize(c->host.stream) != hipSuccess) {
        (void)hipGetLastError();
        return make_error(PJRT_Error_Code_INTERNAL, "device to host copy failed");
    }
    *event = complete_event();
    return nullptr;
}
PJRT_Error* Buffer_ToHostBuffer(PJRT_Buffer_ToHostBuffer_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Buffer_ToHostBuffer");
    REQUIRE(a->src, "src");
    PJRT_Buffer& b = *a->src;
    const size_t need = b.tensor.type.bytes();
    if (!a->dst) { a->dst_size = need; return nullptr; }    // size query
    if (a->dst_size < need)
        return invalid("dst_size (" + std::to_string(a->dst_size) + ") is smaller than the buffer (" + std::to_string(need) + " bytes)");
    return copy_to_host(b, a->dst, 0, need, &a->event);
}
PJRT_Error* Buffer_CopyRawToHost(PJRT_Buffer_CopyRawToHost_Args* a) {
    BUF(a, "PJRT_Buffer_CopyRawToHost");
    REQUIRE(a->dst, "dst");
    const int64_t total = (int64_t)b.tensor.type.bytes();
    if (a->offset < 0 || a->transfer_size < 0 || a->offset + a->transfer_size > total)
        return make_error(PJRT_Error_Code_OUT_OF_RANGE, "offset + transfer_size exceeds the buffer (" + std::to_string(total) + " bytes)");
    return copy_to_host(b, a->dst, (size_t)a->offset, (size_t)a->transfer_size, &a->event);
}
PJRT_Error* clone_buffer(PJRT_Buffer& b, PJRT_Buffer** out) {
    if (b.deleted) return make_error(PJRT_Error_Code_FAILED_PRECONDITION, "the buffer was deleted");
    PJRT_Buffer* nb = nullptr;
    PJRT_Error* err = guarded([&] {
        DeviceTensor d = b.client->host.allocate(b.tensor.type);
        const size_t n = b.tensor.type.bytes();
        std::lock_guard<std::mutex> stream_lock(b.client->host.stream_mu);
        if (n && (hipMemcpyAsync(d.data(), b.tensor.data(), n, hipMemcpyDeviceToDevice, b.client->host.stream) != hipSuccess ||
                  hipStreamSynchronize(b.client->host.stream) != hipSuccess)) {
            (void)hipGetLastError();
            throw BufferError("device to device copy failed");
        }
        nb = new PJRT_Buffer();
        nb->client = b.client;
        nb->tensor = d;
        nb->dims = b.dims;
    });
    if (err) return err;
    *out = nb;
    return nullptr;
}
PJRT_Error* Buffer_CopyToDevice(PJRT_Buffer_CopyToDevice_Args* a) {
    BUF(a, "PJRT_Buffer_CopyToDevice");
    REQUIRE(a->dst_device, "dst_device");
    return clone_buffer(b, &a->dst_buffer);
}
PJRT_Error* Buffer_CopyToMemory(PJRT_Buffer_CopyToMemory_Args* a) {
    BUF(a, "PJRT_Buffer_CopyToMemory");
    REQUIRE(a->dst_memory, "dst_memory");
    return clone_buffer(b, &a->dst_buffer);
}
PJRT_Error* Buffer_IsOnCpu(PJRT_Buffer_IsOnCpu_Args* a) { BUF(a, "PJRT_Buffer_IsOnCpu"); (void)b; a->is_on_cpu = false; return nullptr; }
PJRT_Error* Buffer_ReadyEvent(PJRT_Buffer_ReadyEvent_Args* a) {
    BUF(a, "PJRT_Buffer_ReadyEvent");
    a->event = event_for(b.ready);              // pending while the upload that fills the buffer is in flight
    return nullptr;
}
PJRT_Error* Buffer_UnsafePointer(PJRT_Buffer_UnsafePointer_Args* a) { REQUIRE_ARGS(a, "PJRT_Buffer_UnsafePointer"); return unimplemented("PJRT_Buffer_UnsafePointer"); }
PJRT_Error* Buffer_IncreaseExternalReferenceCount(PJRT_Buffer_IncreaseExternalReferenceCount_Args* a) {
    BUF(a, "PJRT_Buffer_IncreaseExternalReferenceCount");
    b.external_refs++;
    return nullptr;
}
PJRT_Error* Buffer_DecreaseExternalReferenceCount(PJRT_Buffer_DecreaseExternalReferenceCount_Args* a) {
    BUF(a, "PJRT_Buffer_DecreaseExternalReferenceCount");
    if (b.external_refs.load() <= 0) return make_error(PJRT_Error_Code_FAILED_PRECONDITION, "the external reference count is already zero");
    b.external_refs--;
    return nullptr;
}
PJRT_Error* Buffer_OpaqueDeviceMemoryDataPointer(PJRT_Buffer_OpaqueDeviceMemoryDataPointer_Args* a) {
    REQUIRE_ARGS(a, "PJRT_Buffer_OpaqueDeviceMemoryDataPointer");
    return unimplemented("PJRT_Buffer_OpaqueDeviceMemoryDataPointer");
}

// ---- topology ----------------------------------------------------------------------------------
PJRT_Error* TopologyDescription_Create(PJRT_TopologyDescription_Create_Args* a) {
    REQUIRE_ARGS(a, "PJRT_TopologyDescription_Create");
    auto* t = new PJRT_TopologyDescription();
    t->owned.reset(new PJRT_DeviceDescription());
    Client none;                                            // a description that needs no device
    none.device_name = "MI355X (gfx950)";
    describe_device(*t->owned, none);
    t->owned->kind = none.device_name;
    t->descriptions = {t->owned.get()};
    a->topology = t;
    return nullptr;
}
PJRT_Error* TopologyDescription_Destroy(PJRT_TopologyDescription_Destroy_Args* a) {
    REQUIRE_ARGS(a, "PJRT_TopologyDescription_Destroy");
    if (a->topology && a->topology->owned) delete a->topology;   // a client's own topology goes with the client
    return nullptr;
}
PJRT_Error* TopologyDescription_PlatformName(PJRT_TopologyDescription_PlatformName_Args* a) {
    REQUIRE_ARGS(a, "PJRT_TopologyDescription_PlatformName"); REQUIRE(a->topology, "topology");
    a->platform_name = a->topology->platform_name.c_str();
    a->platform_name_size = a->topology->platform_name.size();
    return nullptr;
}
PJRT_Error* TopologyDescription_PlatformVersion(PJRT_TopologyDescription_PlatformVersion_Args* a) {
    REQUIRE_ARGS(a, "PJRT_TopologyDescription_PlatformVersion"); REQUIRE(a->topology, "topology");
    a->platform_version = a->topology->platform_version.c_str();
    a->platform_version_size = a->topology->platform_version.size();
    return nullptr;
}
PJRT_Error* TopologyDescription_GetDeviceDescriptions(PJRT_TopologyDescription_GetDeviceDescriptions_Args* a) {
    REQUIRE_ARGS(a, "PJRT_TopologyDescription_GetDeviceDescriptions"); REQUIRE(a->topology, "topology");
    a->descriptions = a->topology->descriptions.data();
    a->num_descriptions = a->topology->descriptions.size();
    return nullptr;
}
PJRT_Error* TopologyDescription_Attributes(PJRT_TopologyDescription_Attributes_Args* a) {
    REQUIRE_ARGS(a, "PJRT_TopologyDescription_Attributes"); REQUIRE(a->topology, "topology");
    a->attributes = nullptr;
    a->num_attributes = 0;
    return nullptr;
}

PJRT_Api* make_api() {
    PJRT_Api* api = new PJRT_Api();
    memset(api, 0, sizeof(*api));
    api->struct_size = sizeof(PJRT_Api);
    api->pjrt_api_version.struct_size = sizeof(PJRT_Api_Version);
    api->pjrt_api_version.major_version = PJRT_API_MAJOR;
    api->pjrt_api_version.minor_version = PJRT_API_MINOR;
#define SET(group, fn) api->PJRT_##group##_##fn = group##_##fn
    SET(Error, Destroy); SET(Error, Message); SET(Error, GetCode);
    SET(Plugin, Initialize); SET(Plugin, Attributes);
    SET(Event, Destroy); SET(Event, IsReady); SET(Event, Error); SET(Event, Await); SET(Event, OnReady);
    SET(Client, Create); SET(Client, Destroy); SET(Client, PlatformName); SET(Client, ProcessIndex); SET(Client, PlatformVersion);
    SET(Client, Devices); SET(Client, AddressableDevices); SET(Client, LookupDevice); SET(Client, LookupAddressableDevice);
    SET(Client, AddressableMemories); SET(Client, Compile); SET(Client, DefaultDeviceAssignment); SET(Client, BufferFromHostBuffer);
    SET(Client, TopologyDescription);
    SET(DeviceDescription, Id); SET(DeviceDescription, ProcessIndex); SET(DeviceDescription, Attributes); SET(DeviceDescription, Kind);
    SET(DeviceDescription, DebugString); SET(DeviceDescription, ToString);
    SET(Device, GetDescription); SET(Device, IsAddressable); SET(Device, LocalHardwareId); SET(Device, AddressableMemories);
    SET(Device, DefaultMemory); SET(Device, MemoryStats);
    SET(Memory, Id); SET(Memory, Kind); SET(Memory, Kind_Id); SET(Memory, DebugString); SET(Memory, ToString); SET(Memory, AddressableByDevices);
    SET(Executable, Destroy); SET(Executable, Name); SET(Executable, NumReplicas); SET(Executable, NumPartitions); SET(Executable, NumOutputs);
    SET(Executable, SizeOfGeneratedCodeInBytes); SET(Executable, GetCostAnalysis); SET(Executable, OutputMemoryKinds);
    SET(Executable, OptimizedProgram); SET(Executable, Serialize); SET(Executable, OutputElementTypes); SET(Executable, OutputDimensions);
    SET(Executable, Fingerprint); SET(Executable, GetCompiledMemoryStats); SET(Executable, DeserializeAndLoad);
    SET(LoadedExecutable, Destroy); SET(LoadedExecutable, GetExecutable); SET(LoadedExecutable, AddressableDevices); SET(LoadedExecutable, Delete);
    SET(LoadedExecutable, IsDeleted); SET(LoadedExecutable, Execute); SET(LoadedExecutable, Fingerprint); SET(LoadedExecutable, GetDeviceAssignment);
    SET(Buffer, Destroy); SET(Buffer, ElementType); SET(Buffer, Dimensions); SET(Buffer, UnpaddedDimensions); SET(Buffer, DynamicDimensionIndices);
    SET(Buffer, GetMemoryLayout); SET(Buffer, OnDeviceSizeInBytes); SET(Buffer, Device); SET(Buffer, Memory); SET(Buffer, Delete);
    SET(Buffer, IsDeleted); SET(Buffer, CopyToDevice); SET(Buffer, ToHostBuffer); SET(Buffer, IsOnCpu); SET(Buffer, ReadyEvent);
    SET(Buffer, UnsafePointer); SET(Buffer, IncreaseExternalReferenceCount); SET(Buffer, DecreaseExternalReferenceCount);
    SET(Buffer, OpaqueDeviceMemoryDataPointer); SET(Buffer, CopyToMemory); SET(Buffer, CopyRawToHost);
    SET(TopologyDescription, Create); SET(TopologyDescription, Destroy); SET(TopologyDescription, PlatformName);
    SET(TopologyDescription, PlatformVersion); SET(TopologyDescription, GetDeviceDescriptions); SET(TopologyDescription, Attributes);
#undef SET
    return api;
}

}  // namespace

extern "C" const PJRT_Api* GetPjrtApi(void) {
    static const PJRT_Api* api = make_api();                // built once, never freed (PJRTApi.swift:158-162)
    return api;
}
