/* metalhlo.h — the `mhlo_*` C API, served by the gfx950 host in this repository.
 *
 * Same symbols, enums and struct layouts as the reference's
 * Sources/CMetalHLO/include/metalhlo.h (cited per declaration), so a program
 * built against that header links against libCMetalHLO.so here unchanged.
 * Device work goes through the kernel C-ABI in mhip.h.
 *
 * Conventions (reference: Sources/CMetalHLO/CInterface.swift:112-134,245-297):
 * every fallible call returns an MHLOStatusCode and leaves a message readable
 * with mhlo_get_last_error(); a NULL argument is MHLO_ERROR_INVALID_ARGUMENT;
 * handles are opaque pointers owned by the caller until the matching
 * *_destroy.  The error slot is per thread here (process-global there).
 */
#ifndef METALHLO_H
#define METALHLO_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Everything declared here is the library's public surface: the library itself is built with
 * hidden visibility, and only these names (and the two mhlo_ext_* extensions) are exported. */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

/* metalhlo.h:23 — static string, never freed. */
const char* mhlo_version(void);

/* metalhlo.h:29-31 */
typedef void* MHLOClientRef;
typedef void* MHLOExecutableRef;
typedef void* MHLOBufferRef;

/* metalhlo.h:37-49 */
typedef enum {
    MHLO_OK = 0,
    MHLO_ERROR_NO_DEVICE = 1,
    MHLO_ERROR_UNSUPPORTED_DEVICE = 2,
    MHLO_ERROR_PARSE_FAILED = 3,
    MHLO_ERROR_UNSUPPORTED_OP = 4,
    MHLO_ERROR_COMPILATION_FAILED = 5,
    MHLO_ERROR_BUFFER_FAILED = 6,
    MHLO_ERROR_INPUT_MISMATCH = 7,
    MHLO_ERROR_EXECUTION_FAILED = 8,
    MHLO_ERROR_TRANSFER_FAILED = 9,
    MHLO_ERROR_INVALID_ARGUMENT = 10,
} MHLOStatusCode;

/* metalhlo.h:53,56 — message owned by the library; NULL when no error is pending. */
const char* mhlo_get_last_error(void);
void mhlo_clear_error(void);

/* metalhlo.h:62-76 */
typedef enum {
    MHLO_F16 = 0,
    MHLO_F32 = 1,
    MHLO_F64 = 2,
    MHLO_BF16 = 3,
    MHLO_I1 = 4,
    MHLO_I8 = 5,
    MHLO_I16 = 6,
    MHLO_I32 = 7,
    MHLO_I64 = 8,
    MHLO_UI8 = 9,
    MHLO_UI16 = 10,
    MHLO_UI32 = 11,
    MHLO_UI64 = 12,
} MHLOElementType;

/* metalhlo.h:79 — bytes per element; 0 for I1 (buffers hold one byte per i1 element). */
size_t mhlo_element_type_size(MHLOElementType type);

/* metalhlo.h:88-96 — client on HIP device 0 (MHLO_ERROR_NO_DEVICE without one).
 * mhlo_client_device_name returns a malloc'd string; release with mhlo_free_string. */
MHLOStatusCode mhlo_client_create(MHLOClientRef* out_client);
void mhlo_client_destroy(MHLOClientRef client);
char* mhlo_client_device_name(MHLOClientRef client);

/* metalhlo.h:103-128 — accepted for source compatibility.  The optimisation
 * level is recorded; the device policy has no meaning on a single GPU and is ignored. */
typedef enum {
    MHLO_OPT_O0 = 0,
    MHLO_OPT_O1 = 1,
    MHLO_OPT_O2 = 2,
    MHLO_OPT_O3 = 3,
} MHLOOptimizationLevel;

typedef enum {
    MHLO_DEVICE_GPU_ONLY = 0,
    MHLO_DEVICE_ANE_ONLY = 1,
    MHLO_DEVICE_AUTO = 2,
    MHLO_DEVICE_PREFER_ANE = 3,
    MHLO_DEVICE_PREFER_GPU = 4,
} MHLODevicePolicy;

typedef struct {
    MHLOOptimizationLevel optimization_level; /* default MHLO_OPT_O2 */
    bool enable_caching;                      /* default true */
    bool enable_debug_info;                   /* default false */
    MHLODevicePolicy device_policy;           /* default MHLO_DEVICE_GPU_ONLY */
} MHLOCompileConfig;

/* metalhlo.h:132,136 */
void mhlo_compile_config_init(MHLOCompileConfig* out_config);
bool mhlo_ane_available(void); /* always false here */

/* metalhlo.h:148-178 — StableHLO MLIR text in, executable out.  NULL config = defaults. */
MHLOStatusCode mhlo_compile(MHLOClientRef client, const char* mlir_text,
                            MHLOExecutableRef* out_executable);
MHLOStatusCode mhlo_compile_n(MHLOClientRef client, const char* mlir_text, size_t mlir_length,
                              MHLOExecutableRef* out_executable);
MHLOStatusCode mhlo_compile_with_config(MHLOClientRef client, const char* mlir_text,
                                        const MHLOCompileConfig* config,
                                        MHLOExecutableRef* out_executable);

/* metalhlo.h:181-211 — out_shape / out_rank / out_element_type may each be NULL. */
void mhlo_executable_destroy(MHLOExecutableRef executable);
int32_t mhlo_executable_input_count(MHLOExecutableRef executable);
int32_t mhlo_executable_output_count(MHLOExecutableRef executable);
MHLOStatusCode mhlo_executable_input_type(MHLOExecutableRef executable, int32_t index,
                                          int64_t* out_shape, int32_t* out_rank,
                                          MHLOElementType* out_element_type);
MHLOStatusCode mhlo_executable_output_type(MHLOExecutableRef executable, int32_t index,
                                           int64_t* out_shape, int32_t* out_rank,
                                           MHLOElementType* out_element_type);

/* metalhlo.h:215-238 — times in milliseconds. */
typedef struct {
    int64_t execution_count;
    double total_execution_time_ms;
    double last_execution_time_ms;
    double average_execution_time_ms;
} MHLOExecutionStats;

MHLOStatusCode mhlo_executable_get_stats(MHLOExecutableRef executable,
                                         MHLOExecutionStats* out_stats);
void mhlo_executable_reset_stats(MHLOExecutableRef executable);

/* metalhlo.h:254-310 — mhlo_buffer_create copies `data_size` bytes to the device;
 * mhlo_buffer_to_host fails with MHLO_ERROR_TRANSFER_FAILED when `data_size` is
 * smaller than the tensor. */
MHLOStatusCode mhlo_buffer_create(MHLOClientRef client, const void* data, size_t data_size,
                                  const int64_t* shape, int32_t rank,
                                  MHLOElementType element_type, MHLOBufferRef* out_buffer);
MHLOStatusCode mhlo_buffer_create_uninitialized(MHLOClientRef client, const int64_t* shape,
                                                int32_t rank, MHLOElementType element_type,
                                                MHLOBufferRef* out_buffer);
void mhlo_buffer_destroy(MHLOBufferRef buffer);
void mhlo_buffer_shape(MHLOBufferRef buffer, int64_t* out_shape, int32_t* out_rank);
int32_t mhlo_buffer_rank(MHLOBufferRef buffer);
MHLOElementType mhlo_buffer_element_type(MHLOBufferRef buffer);
size_t mhlo_buffer_byte_count(MHLOBufferRef buffer);
MHLOStatusCode mhlo_buffer_to_host(MHLOBufferRef buffer, void* out_data, size_t data_size);

/* metalhlo.h:324-346 — `out_outputs` is a caller-allocated array with room for
 * mhlo_executable_output_count() handles; each returned buffer is the caller's
 * to destroy.  Timing outputs are in SECONDS and may be NULL. */
MHLOStatusCode mhlo_execute(MHLOExecutableRef executable, const MHLOBufferRef* inputs,
                            int32_t num_inputs, MHLOBufferRef* out_outputs,
                            int32_t* out_num_outputs);
MHLOStatusCode mhlo_execute_with_timing(MHLOExecutableRef executable, const MHLOBufferRef* inputs,
                                        int32_t num_inputs, MHLOBufferRef* out_outputs,
                                        int32_t* out_num_outputs, double* out_encode_time,
                                        double* out_gpu_time, double* out_total_time);

/* metalhlo.h:354-388 — always one GPU partition, no ANE. */
typedef struct {
    int32_t partition_count;
    int32_t gpu_partition_count;
    int32_t ane_partition_count;
    double gpu_time_ms;
    double ane_time_ms;
    double transfer_time_ms;
    double total_time_ms;
    bool used_ane;
} MHLOExecutionProfile;

MHLOStatusCode mhlo_execute_with_profile(MHLOExecutableRef executable,
                                         const MHLOBufferRef* inputs, int32_t num_inputs,
                                         MHLOBufferRef* out_outputs, int32_t* out_num_outputs,
                                         MHLOExecutionProfile* out_profile);

/* metalhlo.h:397 */
void mhlo_free_string(const char* str);

/* Extension, not part of the reference's header: the operations an executable runs
 * after pattern recognition, in program order, comma-separated (custom calls by their
 * target name).  Returns a malloc'd string; release with mhlo_free_string. */
char* mhlo_ext_executable_ops(MHLOExecutableRef executable);

/* Extension, not part of the reference's header: the memory plan and launch statistics of an
 * executable, "key=value" pairs separated by commas: planned (0/1), arena_bytes (one arena
 * holds every intermediate; lifetimes that do not overlap share bytes), slots, unshared_bytes
 * (what one allocation per intermediate would take), result_bytes, overlaps (pairs of slots
 * alive together whose bytes intersect; 0 in a sound plan), graph_captures, graph_replays,
 * eager_runs.  The plan plays the part of the reference's StaticMemoryPlanner
 * (Sources/MetalHLOCore/Memory/StaticMemoryPlanner.swift:144-250).  Returns a malloc'd
 * string; release with mhlo_free_string. */
char* mhlo_ext_executable_plan(MHLOExecutableRef executable);

/* Extension: per-operation device time of the last profiled execution (mhlo_execute_with_profile
 * profiles the execution it makes; METALHLO_PROFILE_GPU=1 profiles every execution and also prints
 * the lines to stderr): one "<operation> <result shape> <microseconds>" line per operation in
 * program order, measured with HIP events around the operation's launches on an eager run.  The
 * counterpart of the reference's METALHLO_PROFILE_GPU / METALHLO_DEBUG_DISPATCH output
 * (Runtime/MetalExecutor.swift:289-316, IntegratedExecutor.swift:411-478).  Returns a malloc'd
 * string (empty when nothing was profiled); release with mhlo_free_string. */
char* mhlo_ext_executable_profile(MHLOExecutableRef executable);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif

#ifdef __cplusplus
}
#endif
#endif /* METALHLO_H */
