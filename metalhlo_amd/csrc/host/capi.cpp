// The mhlo_* C API (include/metalhlo.h) over the parser and the executor.
// Behaviour follows Sources/CMetalHLO/CInterface.swift: NULL checks with the same
// argument names in the messages (:245-297), status mapping (:137-158), defaults
// (:873-882), statistics in milliseconds (:63-96), timing outputs in seconds.
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <new>
#include <string>

#include "../../../include/metalhlo.h"
#include "../../../include/mhip.h"
#include "executor.h"

using namespace mhlo;

namespace {

thread_local std::string g_error;
thread_local bool g_has_error = false;

MHLOStatusCode set_error(MHLOStatusCode code, const std::string& msg) {
    g_error = msg;
    g_has_error = true;
    return code;
}
void clear_error() { g_has_error = false; g_error.clear(); }

struct BufferHandle { Client* client; DeviceTensor t; };

bool valid_dtype(int t) { return t >= MHLO_F16 && t <= MHLO_UI64; }

// Runs `body`, translating the host's exceptions into status codes.
template <typename F>
MHLOStatusCode guarded(F&& body) {
    try {
        clear_error();
        body();
        return MHLO_OK;
    } catch (const ParseError& e) { return set_error(MHLO_ERROR_PARSE_FAILED, std::string("Parse failed: ") + e.what());
    } catch (const UnsupportedOp& e) { return set_error(MHLO_ERROR_UNSUPPORTED_OP, std::string("Unsupported operation: ") + e.what());
    } catch (const InputMismatch& e) { return set_error(MHLO_ERROR_INPUT_MISMATCH, e.what());
    } catch (const NoDevice& e) { return set_error(MHLO_ERROR_NO_DEVICE, e.what());
    } catch (const BufferError& e) { return set_error(MHLO_ERROR_BUFFER_FAILED, e.what());
    } catch (const ExecError& e) { return set_error(MHLO_ERROR_EXECUTION_FAILED, std::string("Execution failed: ") + e.what());
    } catch (const std::bad_alloc&) { return set_error(MHLO_ERROR_BUFFER_FAILED, "out of host memory");
    } catch (const std::exception& e) { return set_error(MHLO_ERROR_COMPILATION_FAILED, e.what()); }
}

MHLOStatusCode compile_text(MHLOClientRef client, const std::string& text, const MHLOCompileConfig* cfg,
                            MHLOExecutableRef* out) {
    Executable* exe = nullptr;
    MHLOStatusCode st = guarded([&] {
        exe = new Executable();
        exe->client = static_cast<Client*>(client);
        exe->opt_level = cfg ? (int)cfg->optimization_level : (int)MHLO_OPT_O2;
        // O0 runs the module as written; every other level recognises the fused patterns
        // (Sources/MetalHLO/CompilationConfig.swift:232-263 enables the fusion passes from O1)
        exe->fn = build_function(text, exe->opt_level);
        compile(*exe);
    });
    if (st != MHLO_OK) { delete exe; return st; }
    *out = exe;
    return MHLO_OK;
}

MHLOStatusCode type_query(const TensorType& t, int64_t* shape, int32_t* rank, MHLOElementType* et) {
    if (shape) for (size_t i = 0; i < t.shape.size(); i++) shape[i] = t.shape[i];
    if (rank) *rank = (int32_t)t.shape.size();
    if (et) *et = (MHLOElementType)t.dtype;
    return MHLO_OK;
}

MHLOStatusCode run(MHLOExecutableRef executable, const MHLOBufferRef* inputs, int32_t num_inputs,
                   MHLOBufferRef* out_outputs, int32_t* out_num_outputs, double* enc, double* gpu, double* total) {
    if (!executable) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "executable is null");
    if (!out_outputs) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "out_outputs is null");
    if (!out_num_outputs) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "out_num_outputs is null");
    if (num_inputs < 0 || (num_inputs > 0 && !inputs)) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "inputs is null");
    Executable& exe = *static_cast<Executable*>(executable);
    std::vector<DeviceTensor> in;
    for (int32_t i = 0; i < num_inputs; i++) {
        if (!inputs[i]) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "input buffer " + std::to_string(i) + " is null");
        in.push_back(static_cast<BufferHandle*>(inputs[i])->t);
    }
    std::vector<DeviceTensor> outs;
    double e = 0, g = 0;
    const auto t0 = std::chrono::steady_clock::now();
    MHLOStatusCode st = guarded([&] { outs = execute(exe, in, &e, &g); });
    const double wall = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    if (st != MHLO_OK) return st;
    for (size_t i = 0; i < outs.size(); i++) out_outputs[i] = new BufferHandle{exe.client, outs[i]};
    *out_num_outputs = (int32_t)outs.size();
    {
        std::lock_guard<std::mutex> lk(exe.mu);
        exe.exec_count++;
        exe.last_ms = wall * 1e3;
        exe.total_ms += wall * 1e3;
    }
    if (enc) *enc = e;
    if (gpu) *gpu = g;
    if (total) *total = wall;
    return MHLO_OK;
}

}  // namespace

extern "C" {

const char* mhlo_version(void) { return "0.2.0"; }

const char* mhlo_get_last_error(void) { return g_has_error ? g_error.c_str() : nullptr; }
void mhlo_clear_error(void) { clear_error(); }

size_t mhlo_element_type_size(MHLOElementType type) {
    if (!valid_dtype(type) || type == MHLO_I1) return 0;
    return (size_t)dtype_bytes(type);
}

MHLOStatusCode mhlo_client_create(MHLOClientRef* out_client) {
    if (!out_client) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "out_client is null");
    const int n = mhip_device_count();
    // METALHLO_ALLOW_NO_DEVICE=1: a client without a GPU, for parsing / validation
    // only (compile works, buffers and execution report MHLO_ERROR_NO_DEVICE).
    const char* allow = getenv("METALHLO_ALLOW_NO_DEVICE");
    if (n <= 0 && !(allow && allow[0] == '1')) return set_error(MHLO_ERROR_NO_DEVICE, "No HIP device found");
    clear_error();
    Client* c = new Client();
    if (n > 0) {
        c->device = 0;
        if (hipSetDevice(0) != hipSuccess || hipStreamCreate(&c->stream) != hipSuccess) {
            delete c;
            return set_error(MHLO_ERROR_UNSUPPORTED_DEVICE, "cannot initialise HIP device 0");
        }
        char arch[128] = {0};
        int cus = 0;
        mhip_device_info(0, &cus, nullptr, arch, sizeof(arch));
        hipDeviceProp_t p;
        c->device_name = hipGetDeviceProperties(&p, 0) == hipSuccess ? std::string(p.name) : std::string("HIP device");
        c->device_name += std::string(" (") + arch + ", " + std::to_string(cus) + " CUs)";
    } else {
        c->device_name = "none (host-only client)";
    }
    *out_client = c;
    return MHLO_OK;
}

void mhlo_client_destroy(MHLOClientRef client) {
    if (!client) return;
    Client* c = static_cast<Client*>(client);
    if (c->stream) { (void)hipStreamSynchronize(c->stream); (void)hipStreamDestroy(c->stream); }
    delete c;
}

char* mhlo_client_device_name(MHLOClientRef client) {
    if (!client) return nullptr;
    return strdup(static_cast<Client*>(client)->device_name.c_str());
}

void mhlo_compile_config_init(MHLOCompileConfig* out_config) {
    if (!out_config) return;
    out_config->optimization_level = MHLO_OPT_O2;
    out_config->enable_caching = true;
    out_config->enable_debug_info = false;
    out_config->device_policy = MHLO_DEVICE_GPU_ONLY;
}

bool mhlo_ane_available(void) { return false; }

MHLOStatusCode mhlo_compile(MHLOClientRef client, const char* mlir_text, MHLOExecutableRef* out_executable) {
    if (!client) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "client is null");
    if (!mlir_text) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "mlir_text is null");
    if (!out_executable) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "out_executable is null");
    return compile_text(client, mlir_text, nullptr, out_executable);
}

MHLOStatusCode mhlo_compile_n(MHLOClientRef client, const char* mlir_text, size_t mlir_length,
                              MHLOExecutableRef* out_executable) {
    if (!client) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "client is null");
    if (!mlir_text) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "mlir_text is null");
    if (!out_executable) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "out_executable is null");
    return compile_text(client, std::string(mlir_text, mlir_length), nullptr, out_executable);
}

MHLOStatusCode mhlo_compile_with_config(MHLOClientRef client, const char* mlir_text,
                                        const MHLOCompileConfig* config, MHLOExecutableRef* out_executable) {
    if (!client) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "client is null");
    if (!mlir_text) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "mlir_text is null");
    if (!out_executable) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "out_executable is null");
    if (config && (config->optimization_level < MHLO_OPT_O0 || config->optimization_level > MHLO_OPT_O3))
        return set_error(MHLO_ERROR_INVALID_ARGUMENT, "optimization_level out of range");
    return compile_text(client, mlir_text, config, out_executable);
}

void mhlo_executable_destroy(MHLOExecutableRef executable) { delete static_cast<Executable*>(executable); }

int32_t mhlo_executable_input_count(MHLOExecutableRef executable) {
    return executable ? (int32_t)static_cast<Executable*>(executable)->fn.arg_types.size() : 0;
}
int32_t mhlo_executable_output_count(MHLOExecutableRef executable) {
    return executable ? (int32_t)static_cast<Executable*>(executable)->fn.returns.size() : 0;
}

MHLOStatusCode mhlo_executable_input_type(MHLOExecutableRef executable, int32_t index, int64_t* out_shape,
                                          int32_t* out_rank, MHLOElementType* out_element_type) {
    if (!executable) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "executable is null");
    const Function& fn = static_cast<Executable*>(executable)->fn;
    if (index < 0 || index >= (int32_t)fn.arg_types.size()) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "input index out of range");
    clear_error();
    return type_query(fn.arg_types[index], out_shape, out_rank, out_element_type);
}

MHLOStatusCode mhlo_executable_output_type(MHLOExecutableRef executable, int32_t index, int64_t* out_shape,
                                           int32_t* out_rank, MHLOElementType* out_element_type) {
    if (!executable) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "executable is null");
    const Function& fn = static_cast<Executable*>(executable)->fn;
    if (index < 0 || index >= (int32_t)fn.returns.size()) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "output index out of range");
    clear_error();
    TensorType t;
    if (index < (int32_t)fn.result_types.size()) t = fn.result_types[index];
    else {
        for (auto& op : fn.ops) if (op.result == fn.returns[index]) t = op.out;
        for (size_t i = 0; i < fn.arg_ids.size(); i++) if (fn.arg_ids[i] == fn.returns[index]) t = fn.arg_types[i];
    }
    return type_query(t, out_shape, out_rank, out_element_type);
}

MHLOStatusCode mhlo_executable_get_stats(MHLOExecutableRef executable, MHLOExecutionStats* out_stats) {
    if (!executable) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "executable is null");
    if (!out_stats) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "out_stats is null");
    Executable& exe = *static_cast<Executable*>(executable);
    std::lock_guard<std::mutex> lk(exe.mu);
    out_stats->execution_count = exe.exec_count;
    out_stats->total_execution_time_ms = exe.total_ms;
    out_stats->last_execution_time_ms = exe.last_ms;
    out_stats->average_execution_time_ms = exe.exec_count ? exe.total_ms / (double)exe.exec_count : 0.0;
    return MHLO_OK;
}

void mhlo_executable_reset_stats(MHLOExecutableRef executable) {
    if (!executable) return;
    Executable& exe = *static_cast<Executable*>(executable);
    std::lock_guard<std::mutex> lk(exe.mu);
    exe.exec_count = 0;
    exe.total_ms = exe.last_ms = 0;
}

static MHLOStatusCode make_buffer(MHLOClientRef client, const void* data, size_t data_size, const int64_t* shape,
                                  int32_t rank, MHLOElementType et, MHLOBufferRef* out, bool init) {
    if (!client) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "client is null");
    if (init && !data) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "data is null");
    if (rank < 0 || (rank > 0 && !shape)) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "shape is null");
    if (!out) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "out_buffer is null");
    if (!valid_dtype(et)) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "unknown element type");
    TensorType t;
    t.dtype = et;
    for (int32_t i = 0; i < rank; i++) {
        if (shape[i] < 0) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "negative dimension");
        t.shape.push_back(shape[i]);
    }
    if (init && data_size < t.bytes())
        return set_error(MHLO_ERROR_BUFFER_FAILED, "data_size (" + std::to_string(data_size) + ") is smaller than the tensor (" +
                                                        std::to_string(t.bytes()) + " bytes)");
    Client* c = static_cast<Client*>(client);
    BufferHandle* h = nullptr;
    MHLOStatusCode st = guarded([&] {
        DeviceTensor d = c->allocate(t);
        if (init && t.bytes()) {
            // explicit host -> device copy on the client's stream (the reference relies on unified memory)
            std::lock_guard<std::mutex> stream_lock(c->stream_mu);      // not into another thread's graph capture
            if (hipMemcpyAsync(d.data(), data, t.bytes(), hipMemcpyHostToDevice, c->stream) != hipSuccess ||
                hipStreamSynchronize(c->stream) != hipSuccess) {
                (void)hipGetLastError();
                throw BufferError("host to device copy failed");
            }
        }
        h = new BufferHandle{c, d};
    });
    if (st != MHLO_OK) return st;
    *out = h;
    return MHLO_OK;
}

MHLOStatusCode mhlo_buffer_create(MHLOClientRef client, const void* data, size_t data_size, const int64_t* shape,
                                  int32_t rank, MHLOElementType element_type, MHLOBufferRef* out_buffer) {
    return make_buffer(client, data, data_size, shape, rank, element_type, out_buffer, true);
}

MHLOStatusCode mhlo_buffer_create_uninitialized(MHLOClientRef client, const int64_t* shape, int32_t rank,
                                                MHLOElementType element_type, MHLOBufferRef* out_buffer) {
    return make_buffer(client, nullptr, 0, shape, rank, element_type, out_buffer, false);
}

void mhlo_buffer_destroy(MHLOBufferRef buffer) { delete static_cast<BufferHandle*>(buffer); }

void mhlo_buffer_shape(MHLOBufferRef buffer, int64_t* out_shape, int32_t* out_rank) {
    if (!buffer) { if (out_rank) *out_rank = 0; return; }
    const TensorType& t = static_cast<BufferHandle*>(buffer)->t.type;
    if (out_shape) for (size_t i = 0; i < t.shape.size(); i++) out_shape[i] = t.shape[i];
    if (out_rank) *out_rank = (int32_t)t.shape.size();
}

int32_t mhlo_buffer_rank(MHLOBufferRef buffer) {
    return buffer ? (int32_t)static_cast<BufferHandle*>(buffer)->t.type.shape.size() : 0;
}

MHLOElementType mhlo_buffer_element_type(MHLOBufferRef buffer) {
    return buffer ? (MHLOElementType)static_cast<BufferHandle*>(buffer)->t.type.dtype : MHLO_F32;
}

size_t mhlo_buffer_byte_count(MHLOBufferRef buffer) {
    return buffer ? static_cast<BufferHandle*>(buffer)->t.type.bytes() : 0;
}

MHLOStatusCode mhlo_buffer_to_host(MHLOBufferRef buffer, void* out_data, size_t data_size) {
    if (!buffer) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "buffer is null");
    if (!out_data) return set_error(MHLO_ERROR_INVALID_ARGUMENT, "out_data is null");
    BufferHandle* h = static_cast<BufferHandle*>(buffer);
    const size_t need = h->t.type.bytes();
    if (data_size < need)
        return set_error(MHLO_ERROR_TRANSFER_FAILED, "Output buffer too small: need " + std::to_string(need) + " bytes, got " +
                                                          std::to_string(data_size));
    clear_error();
    if (need == 0) return MHLO_OK;
    std::lock_guard<std::mutex> stream_lock(h->client->stream_mu);      // not into another thread's graph capture
    if (hipMemcpyAsync(out_data, h->t.data(), need, hipMemcpyDeviceToHost, h->client->stream) != hipSuccess ||
        hipStreamSynchronize(h->client->stream) != hipSuccess) {
        (void)hipGetLastError();
        return set_error(MHLO_ERROR_TRANSFER_FAILED, "device to host copy failed");
    }
    return MHLO_OK;
}

MHLOStatusCode mhlo_execute(MHLOExecutableRef executable, const MHLOBufferRef* inputs, int32_t num_inputs,
                            MHLOBufferRef* out_outputs, int32_t* out_num_outputs) {
    return run(executable, inputs, num_inputs, out_outputs, out_num_outputs, nullptr, nullptr, nullptr);
}

MHLOStatusCode mhlo_execute_with_timing(MHLOExecutableRef executable, const MHLOBufferRef* inputs, int32_t num_inputs,
                                        MHLOBufferRef* out_outputs, int32_t* out_num_outputs, double* out_encode_time,
                                        double* out_gpu_time, double* out_total_time) {
    return run(executable, inputs, num_inputs, out_outputs, out_num_outputs, out_encode_time, out_gpu_time, out_total_time);
}

MHLOStatusCode mhlo_execute_with_profile(MHLOExecutableRef executable, const MHLOBufferRef* inputs, int32_t num_inputs,
                                         MHLOBufferRef* out_outputs, int32_t* out_num_outputs,
                                         MHLOExecutionProfile* out_profile) {
    double enc = 0, gpu = 0, total = 0;
    // this execution is timed operation by operation (mhlo_ext_executable_profile returns the list)
    if (executable) static_cast<Executable*>(executable)->profile_next = true;
    MHLOStatusCode st = run(executable, inputs, num_inputs, out_outputs, out_num_outputs, &enc, &gpu, &total);
    if (st == MHLO_OK && out_profile) {
        out_profile->partition_count = 1;
        out_profile->gpu_partition_count = 1;
        out_profile->ane_partition_count = 0;
        out_profile->gpu_time_ms = gpu * 1e3;
        out_profile->ane_time_ms = 0;
        out_profile->transfer_time_ms = 0;
        out_profile->total_time_ms = total * 1e3;
        out_profile->used_ane = false;
    }
    return st;
}

void mhlo_free_string(const char* str) { free(const_cast<char*>(str)); }

// Extension (no counterpart in the reference's header): the operations an
// executable runs after pattern recognition, in program order, separated by
// commas; custom calls appear as their target name.  Caller frees with
// mhlo_free_string.
char* mhlo_ext_executable_ops(MHLOExecutableRef executable) {
    if (!executable) { set_error(MHLO_ERROR_INVALID_ARGUMENT, "executable is null"); return nullptr; }
    const Executable* exe = static_cast<const Executable*>(executable);
    std::string out;
    for (const Op& op : exe->fn.ops) {
        if (!out.empty()) out += ",";
        out += op.name == "custom_call" ? op.target : op.name;
    }
    return strdup(out.c_str());
}

// Extension (not in the reference's header): the memory plan and launch statistics of an
// executable as "key=value" pairs separated by commas: arena_bytes (the planned arena for
// intermediates), slots, unshared_bytes (one allocation per intermediate would take this),
// result_bytes, overlaps (pairs of slots alive at the same time whose bytes intersect: 0 in a
// sound plan), graph_captures, graph_replays, eager_runs.  Caller frees with mhlo_free_string.
char* mhlo_ext_executable_plan(MHLOExecutableRef executable) {
    if (!executable) { set_error(MHLO_ERROR_INVALID_ARGUMENT, "executable is null"); return nullptr; }
    Executable* exe = static_cast<Executable*>(executable);
    std::lock_guard<std::mutex> lk(exe->run_mu);
    const ArenaPlan& p = exe->plan;
    size_t overlaps = 0;
    for (size_t i = 0; i < p.slots.size(); i++)
        for (size_t j = i + 1; j < p.slots.size(); j++) {
            const ArenaPlan::Slot &a = p.slots[i], &b = p.slots[j];
            overlaps += a.begin <= b.end && b.begin <= a.end && a.offset < b.offset + b.bytes && b.offset < a.offset + a.bytes;
        }
    std::string out = "planned=" + std::to_string(p.valid ? 1 : 0) + ",arena_bytes=" + std::to_string(p.core_bytes) +
                      ",slots=" + std::to_string(p.slots.size()) + ",unshared_bytes=" + std::to_string(p.sum_bytes) +
                      ",result_bytes=" + std::to_string(p.full_bytes - p.core_bytes) + ",overlaps=" + std::to_string(overlaps) +
                      ",graph_captures=" + std::to_string(exe->graph_captures) +
                      ",graph_replays=" + std::to_string(exe->graph_replays) + ",eager_runs=" + std::to_string(exe->eager_runs);
    return strdup(out.c_str());
}

// Extension: the device time of every operation of the last profiled execution (the one made by
// mhlo_execute_with_profile, or any execution under METALHLO_PROFILE_GPU=1), one
// "<operation> <result shape> <microseconds>" line per launch group in program order.  The reference
// prints the same breakdown from METALHLO_PROFILE_GPU / METALHLO_DEBUG_DISPATCH
// (Runtime/MetalExecutor.swift:289-316, Runtime/IntegratedExecutor.swift:411-478).  Empty string when
// no execution was profiled.  Caller frees with mhlo_free_string.
char* mhlo_ext_executable_profile(MHLOExecutableRef executable) {
    if (!executable) { set_error(MHLO_ERROR_INVALID_ARGUMENT, "executable is null"); return nullptr; }
    Executable* exe = static_cast<Executable*>(executable);
    std::lock_guard<std::mutex> lk(exe->run_mu);
    std::string out;
    char buf[64];
    for (auto& t : exe->last_profile) {
        snprintf(buf, sizeof buf, " %.1f\n", t.us);
        out += t.name + " " + t.shape + buf;
    }
    return strdup(out.c_str());
}

}  // extern "C"
