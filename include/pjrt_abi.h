/* PJRT C API, version 0.90: the part of the binary interface that libPJRTMetalHLO.so
 * implements, restated for building the plugin and its tests.
 *
 * Replaces: Sources/PJRTMetalHLO (PJRTApi.swift:23-173 builds the table and exports
 * GetPjrtApi) compiled against Sources/CPJRTApi/include/pjrt_c_api.h (the OpenXLA header the
 * reference vendors) and pjrt_metal_types.h:24-37.  A program built against the OpenXLA
 * header binds to this plugin unchanged: every argument struct here has the same fields
 * in the same order, the function table has the same 130 slots in the same order
 * (sizeof(PJRT_Api) == 1064), and tests/test_pjrt_host.py checks both against that header
 * wherever it is available.
 *
 * Conventions of the interface: every entry takes one `*_Args*` whose first two fields are
 * `struct_size` (filled by the caller) and `extension_start`; it returns NULL on success or
 * a PJRT_Error the caller releases with PJRT_Error_Destroy.  Output fields are marked "out".
 * Slots this plugin leaves empty are declared `void*` in the table (the interface allows a
 * NULL slot for a function a plugin does not offer).
 */
#ifndef MHLO_PJRT_ABI_H_
#define MHLO_PJRT_ABI_H_

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PJRT_API_MAJOR 0
#define PJRT_API_MINOR 90

typedef struct PJRT_Extension_Base {
    size_t struct_size;
    int type;                              /* PJRT_Extension_Type */
    struct PJRT_Extension_Base* next;
} PJRT_Extension_Base;

typedef struct PJRT_Api_Version {
    size_t struct_size;
    PJRT_Extension_Base* extension_start;
    int major_version;
    int minor_version;
} PJRT_Api_Version;

/* opaque objects (defined in csrc/pjrt/pjrt.cpp) */
typedef struct PJRT_Error PJRT_Error;
typedef struct PJRT_Event PJRT_Event;
typedef struct PJRT_Client PJRT_Client;
typedef struct PJRT_Device PJRT_Device;
typedef struct PJRT_Memory PJRT_Memory;
typedef struct PJRT_DeviceDescription PJRT_DeviceDescription;
typedef struct PJRT_TopologyDescription PJRT_TopologyDescription;
typedef struct PJRT_Executable PJRT_Executable;
typedef struct PJRT_LoadedExecutable PJRT_LoadedExecutable;
typedef struct PJRT_Buffer PJRT_Buffer;
typedef struct PJRT_ExecuteContext PJRT_ExecuteContext;
typedef struct PJRT_SerializedExecutable PJRT_SerializedExecutable;
typedef struct PJRT_DeviceAssignmentSerialized PJRT_DeviceAssignmentSerialized;

typedef enum {
    PJRT_Error_Code_OK = 0, PJRT_Error_Code_CANCELLED = 1, PJRT_Error_Code_UNKNOWN = 2,
    PJRT_Error_Code_INVALID_ARGUMENT = 3, PJRT_Error_Code_DEADLINE_EXCEEDED = 4,
    PJRT_Error_Code_NOT_FOUND = 5, PJRT_Error_Code_ALREADY_EXISTS = 6,
    PJRT_Error_Code_PERMISSION_DENIED = 7, PJRT_Error_Code_RESOURCE_EXHAUSTED = 8,
    PJRT_Error_Code_FAILED_PRECONDITION = 9, PJRT_Error_Code_ABORTED = 10,
    PJRT_Error_Code_OUT_OF_RANGE = 11, PJRT_Error_Code_UNIMPLEMENTED = 12,
    PJRT_Error_Code_INTERNAL = 13, PJRT_Error_Code_UNAVAILABLE = 14,
    PJRT_Error_Code_DATA_LOSS = 15, PJRT_Error_Code_UNAUTHENTICATED = 16
} PJRT_Error_Code;

typedef enum {
    PJRT_Buffer_Type_INVALID = 0, PJRT_Buffer_Type_PRED, PJRT_Buffer_Type_S8, PJRT_Buffer_Type_S16,
    PJRT_Buffer_Type_S32, PJRT_Buffer_Type_S64, PJRT_Buffer_Type_U8, PJRT_Buffer_Type_U16,
    PJRT_Buffer_Type_U32, PJRT_Buffer_Type_U64, PJRT_Buffer_Type_F16, PJRT_Buffer_Type_F32,
    PJRT_Buffer_Type_F64, PJRT_Buffer_Type_BF16, PJRT_Buffer_Type_C64, PJRT_Buffer_Type_C128
    /* the 8-bit and narrower float / integer types that follow are not accepted here */
} PJRT_Buffer_Type;

typedef enum {
    PJRT_HostBufferSemantics_kImmutableOnlyDuringCall = 0,
    PJRT_HostBufferSemantics_kImmutableUntilTransferCompletes,
    PJRT_HostBufferSemantics_kImmutableZeroCopy,
    PJRT_HostBufferSemantics_kMutableZeroCopy
} PJRT_HostBufferSemantics;

typedef enum {
    PJRT_NamedValue_kString = 0, PJRT_NamedValue_kInt64, PJRT_NamedValue_kInt64List,
    PJRT_NamedValue_kFloat, PJRT_NamedValue_kBool
} PJRT_NamedValue_Type;

typedef struct PJRT_NamedValue {
    size_t struct_size;
    PJRT_Extension_Base* extension_start;
    const char* name;
    size_t name_size;
    PJRT_NamedValue_Type type;
    union {
        const char* string_value;
        int64_t int64_value;
        const int64_t* int64_array_value;
        float float_value;
        bool bool_value;
    };
    size_t value_size;                     /* string length / list length / 1 */
} PJRT_NamedValue;

typedef struct PJRT_Program {
    size_t struct_size;
    PJRT_Extension_Base* extension_start;
    char* code;                            /* StableHLO text (or MLIR bytecode) */
    size_t code_size;
    const char* format;                    /* "mlir" or "hlo" */
    size_t format_size;
} PJRT_Program;

typedef enum { PJRT_Buffer_MemoryLayout_Type_Tiled = 0, PJRT_Buffer_MemoryLayout_Type_Strides } PJRT_Buffer_MemoryLayout_Type;
typedef struct PJRT_Buffer_MemoryLayout_Tiled {
    size_t struct_size;
    PJRT_Extension_Base* extension_start;
    const int64_t* minor_to_major;
    size_t minor_to_major_size;
    const int64_t* tile_dims;
    const size_t* tile_dim_sizes;
    size_t num_tiles;
} PJRT_Buffer_MemoryLayout_Tiled;
typedef struct PJRT_Buffer_MemoryLayout_Strides {
    size_t struct_size;
    PJRT_Extension_Base* extension_start;
    const int64_t* byte_strides;
    size_t num_byte_strides;
} PJRT_Buffer_MemoryLayout_Strides;
typedef struct PJRT_Buffer_MemoryLayout {
    size_t struct_size;
    PJRT_Extension_Base* extension_start;
    union {
        PJRT_Buffer_MemoryLayout_Tiled tiled;
        PJRT_Buffer_MemoryLayout_Strides strides;
    };
    PJRT_Buffer_MemoryLayout_Type type;
} PJRT_Buffer_MemoryLayout;

/* Argument structs: PJRT_ARGS(Name, fields...) declares `struct Name_Args` with the two
 * leading fields every one of them has, and the function type `Name`. */
#define PJRT_ARGS(name, ...)                   \
    typedef struct name##_Args {               \
        size_t struct_size;                    \
        PJRT_Extension_Base* extension_start;  \
        __VA_ARGS__                            \
    } name##_Args;                             \
    typedef PJRT_Error* name(name##_Args* args)
#define PJRT_ARGS_VOID(name, ...)              \
    typedef struct name##_Args {               \
        size_t struct_size;                    \
        PJRT_Extension_Base* extension_start;  \
        __VA_ARGS__                            \
    } name##_Args;                             \
    typedef void name(name##_Args* args)

/* ---- errors ---- */
PJRT_ARGS_VOID(PJRT_Error_Destroy, PJRT_Error* error;);
PJRT_ARGS_VOID(PJRT_Error_Message, const PJRT_Error* error; const char* message; /* out */ size_t message_size; /* out */);
PJRT_ARGS(PJRT_Error_GetCode, const PJRT_Error* error; PJRT_Error_Code code; /* out */);

/* ---- plugin ---- */
typedef struct PJRT_Plugin_Initialize_Args { size_t struct_size; PJRT_Extension_Base* extension_start; } PJRT_Plugin_Initialize_Args;
typedef PJRT_Error* PJRT_Plugin_Initialize(PJRT_Plugin_Initialize_Args* args);
PJRT_ARGS(PJRT_Plugin_Attributes, const PJRT_NamedValue* attributes; /* out */ size_t num_attributes; /* out */);

/* ---- events ---- */
typedef void (*PJRT_Event_OnReadyCallback)(PJRT_Error* error, void* user_arg);
PJRT_ARGS(PJRT_Event_Destroy, PJRT_Event* event;);
PJRT_ARGS(PJRT_Event_IsReady, PJRT_Event* event; bool is_ready; /* out */);
PJRT_ARGS(PJRT_Event_Error, PJRT_Event* event;);
PJRT_ARGS(PJRT_Event_Await, PJRT_Event* event;);
PJRT_ARGS(PJRT_Event_OnReady, PJRT_Event* event; PJRT_Event_OnReadyCallback callback; void* user_arg;);

/* ---- client ---- */
PJRT_ARGS(PJRT_Client_Create,
          const PJRT_NamedValue* create_options; size_t num_options;
          void* kv_get_callback; void* kv_get_user_arg; void* kv_put_callback; void* kv_put_user_arg;
          PJRT_Client* client; /* out */
          void* kv_try_get_callback; void* kv_try_get_user_arg;);
PJRT_ARGS(PJRT_Client_Destroy, PJRT_Client* client;);
PJRT_ARGS(PJRT_Client_PlatformName, PJRT_Client* client; const char* platform_name; /* out */ size_t platform_name_size; /* out */);
PJRT_ARGS(PJRT_Client_ProcessIndex, PJRT_Client* client; int process_index; /* out */);
PJRT_ARGS(PJRT_Client_PlatformVersion, PJRT_Client* client; const char* platform_version; /* out */ size_t platform_version_size; /* out */);
PJRT_ARGS(PJRT_Client_TopologyDescription, PJRT_Client* client; PJRT_TopologyDescription* topology; /* out, owned by the client */);
PJRT_ARGS(PJRT_Client_Devices, PJRT_Client* client; PJRT_Device* const* devices; /* out */ size_t num_devices; /* out */);
PJRT_ARGS(PJRT_Client_AddressableDevices, PJRT_Client* client; PJRT_Device* const* addressable_devices; /* out */ size_t num_addressable_devices; /* out */);
PJRT_ARGS(PJRT_Client_LookupDevice, PJRT_Client* client; int id; PJRT_Device* device; /* out */);
PJRT_ARGS(PJRT_Client_LookupAddressableDevice, PJRT_Client* client; int local_hardware_id; PJRT_Device* addressable_device; /* out */);
PJRT_ARGS(PJRT_Client_AddressableMemories, PJRT_Client* client; PJRT_Memory* const* addressable_memories; /* out */ size_t num_addressable_memories; /* out */);
PJRT_ARGS(PJRT_Client_Compile, PJRT_Client* client; const PJRT_Program* program; const char* compile_options; size_t compile_options_size;
          PJRT_LoadedExecutable* executable; /* out */);
PJRT_ARGS(PJRT_Client_DefaultDeviceAssignment, PJRT_Client* client; int num_replicas; int num_partitions; size_t default_assignment_size;
          int* default_assignment; /* in/out: caller's array */);
PJRT_ARGS(PJRT_Client_BufferFromHostBuffer,
          PJRT_Client* client; const void* data; PJRT_Buffer_Type type; const int64_t* dims; size_t num_dims;
          const int64_t* byte_strides; size_t num_byte_strides; PJRT_HostBufferSemantics host_buffer_semantics;
          PJRT_Device* device; PJRT_Memory* memory; PJRT_Buffer_MemoryLayout* device_layout;
          PJRT_Event* done_with_host_buffer; /* out */ PJRT_Buffer* buffer; /* out */);

/* ---- device descriptions, devices, memories ---- */
PJRT_ARGS(PJRT_DeviceDescription_Id, PJRT_DeviceDescription* device_description; int id; /* out */);
PJRT_ARGS(PJRT_DeviceDescription_ProcessIndex, PJRT_DeviceDescription* device_description; int process_index; /* out */);
PJRT_ARGS(PJRT_DeviceDescription_Attributes, PJRT_DeviceDescription* device_description; size_t num_attributes; /* out */ const PJRT_NamedValue* attributes; /* out */);
PJRT_ARGS(PJRT_DeviceDescription_Kind, PJRT_DeviceDescription* device_description; const char* device_kind; /* out */ size_t device_kind_size; /* out */);
PJRT_ARGS(PJRT_DeviceDescription_DebugString, PJRT_DeviceDescription* device_description; const char* debug_string; /* out */ size_t debug_string_size; /* out */);
PJRT_ARGS(PJRT_DeviceDescription_ToString, PJRT_DeviceDescription* device_description; const char* to_string; /* out */ size_t to_string_size; /* out */);
PJRT_ARGS(PJRT_Device_GetDescription, PJRT_Device* device; PJRT_DeviceDescription* device_description; /* out */);
PJRT_ARGS(PJRT_Device_IsAddressable, PJRT_Device* device; bool is_addressable; /* out */);
PJRT_ARGS(PJRT_Device_LocalHardwareId, PJRT_Device* device; int local_hardware_id; /* out */);
PJRT_ARGS(PJRT_Device_AddressableMemories, PJRT_Device* device; PJRT_Memory* const* memories; /* out */ size_t num_memories; /* out */);
PJRT_ARGS(PJRT_Device_DefaultMemory, PJRT_Device* device; PJRT_Memory* memory; /* out */);
PJRT_ARGS(PJRT_Device_MemoryStats,
          PJRT_Device* device; int64_t bytes_in_use; /* out, as all below */
          int64_t peak_bytes_in_use; bool peak_bytes_in_use_is_set;
          int64_t num_allocs; bool num_allocs_is_set;
          int64_t largest_alloc_size; bool largest_alloc_size_is_set;
          int64_t bytes_limit; bool bytes_limit_is_set;
          int64_t bytes_reserved; bool bytes_reserved_is_set;
          int64_t peak_bytes_reserved; bool peak_bytes_reserved_is_set;
          int64_t bytes_reservable_limit; bool bytes_reservable_limit_is_set;
          int64_t largest_free_block_bytes; bool largest_free_block_bytes_is_set;
          int64_t pool_bytes; bool pool_bytes_is_set;
          int64_t peak_pool_bytes; bool peak_pool_bytes_is_set;);
PJRT_ARGS(PJRT_Memory_Id, PJRT_Memory* memory; int id; /* out */);
PJRT_ARGS(PJRT_Memory_Kind, PJRT_Memory* memory; const char* kind; /* out */ size_t kind_size; /* out */);
PJRT_ARGS(PJRT_Memory_Kind_Id, PJRT_Memory* memory; int kind_id; /* out */);
PJRT_ARGS(PJRT_Memory_DebugString, PJRT_Memory* memory; const char* debug_string; /* out */ size_t debug_string_size; /* out */);
PJRT_ARGS(PJRT_Memory_ToString, PJRT_Memory* memory; const char* to_string; /* out */ size_t to_string_size; /* out */);
PJRT_ARGS(PJRT_Memory_AddressableByDevices, PJRT_Memory* memory; PJRT_Device* const* devices; /* out */ size_t num_devices; /* out */);

/* ---- executables ---- */
PJRT_ARGS(PJRT_Executable_Destroy, PJRT_Executable* executable;);
PJRT_ARGS(PJRT_Executable_Name, PJRT_Executable* executable; const char* executable_name; /* out */ size_t executable_name_size; /* out */);
PJRT_ARGS(PJRT_Executable_NumReplicas, PJRT_Executable* executable; size_t num_replicas; /* out */);
PJRT_ARGS(PJRT_Executable_NumPartitions, PJRT_Executable* executable; size_t num_partitions; /* out */);
PJRT_ARGS(PJRT_Executable_NumOutputs, PJRT_Executable* executable; size_t num_outputs; /* out */);
PJRT_ARGS(PJRT_Executable_SizeOfGeneratedCodeInBytes, PJRT_Executable* executable; int64_t size_in_bytes; /* out */);
PJRT_ARGS(PJRT_Executable_GetCostAnalysis, PJRT_Executable* executable; size_t num_properties; /* out */ const PJRT_NamedValue* properties; /* out */);
PJRT_ARGS(PJRT_Executable_OutputMemoryKinds, PJRT_Executable* executable; size_t num_outputs; /* out */
          const char* const* memory_kinds; /* out */ const size_t* memory_kind_sizes; /* out */);
PJRT_ARGS(PJRT_Executable_OptimizedProgram, PJRT_Executable* executable; PJRT_Program* program;);
PJRT_ARGS(PJRT_Executable_Serialize, const PJRT_Executable* executable; const char* serialized_bytes; /* out */ size_t serialized_bytes_size; /* out */
          PJRT_SerializedExecutable* serialized_executable; /* out: backing store */
          void (*serialized_executable_deleter)(PJRT_SerializedExecutable* exec); /* out */);
PJRT_ARGS(PJRT_Executable_OutputElementTypes, PJRT_Executable* executable; PJRT_Buffer_Type* output_types; /* out */ size_t num_output_types; /* out */);
PJRT_ARGS(PJRT_Executable_OutputDimensions, PJRT_Executable* executable; size_t num_outputs; /* out */
          const int64_t* dims; /* out: all outputs' dimensions back to back */ const size_t* dim_sizes; /* out: rank of each output */);
PJRT_ARGS(PJRT_Executable_Fingerprint, PJRT_Executable* executable; const char* executable_fingerprint; /* out */ size_t executable_fingerprint_size; /* out */);
PJRT_ARGS(PJRT_Executable_GetCompiledMemoryStats,
          PJRT_Executable* executable; int64_t generated_code_size_in_bytes; int64_t argument_size_in_bytes;
          int64_t output_size_in_bytes; int64_t alias_size_in_bytes; int64_t temp_size_in_bytes;
          int64_t host_generated_code_size_in_bytes; int64_t host_argument_size_in_bytes; int64_t host_output_size_in_bytes;
          int64_t host_alias_size_in_bytes; int64_t host_temp_size_in_bytes; int64_t peak_memory_in_bytes; int64_t total_size_in_bytes;);

PJRT_ARGS(PJRT_LoadedExecutable_Destroy, PJRT_LoadedExecutable* executable;);
PJRT_ARGS(PJRT_LoadedExecutable_GetExecutable, PJRT_LoadedExecutable* loaded_executable; PJRT_Executable* executable; /* out: caller destroys */);
PJRT_ARGS(PJRT_LoadedExecutable_AddressableDevices, PJRT_LoadedExecutable* executable; PJRT_Device* const* addressable_devices; /* out */
          size_t num_addressable_devices; /* out */);
PJRT_ARGS(PJRT_LoadedExecutable_Delete, PJRT_LoadedExecutable* executable;);
PJRT_ARGS(PJRT_LoadedExecutable_IsDeleted, PJRT_LoadedExecutable* executable; bool is_deleted; /* out */);
PJRT_ARGS(PJRT_LoadedExecutable_Fingerprint, PJRT_LoadedExecutable* executable; const char* executable_fingerprint; /* out */
          size_t executable_fingerprint_size; /* out */);
PJRT_ARGS(PJRT_LoadedExecutable_GetDeviceAssignment, PJRT_LoadedExecutable* executable; const char* serialized_bytes; /* out */
          size_t serialized_bytes_size; /* out */ PJRT_DeviceAssignmentSerialized* serialized_device_assignment; /* out */
          void (*serialized_device_assignment_deleter)(PJRT_DeviceAssignmentSerialized* da); /* out */);
PJRT_ARGS(PJRT_Executable_DeserializeAndLoad, PJRT_Client* client; const char* serialized_executable; size_t serialized_executable_size;
          PJRT_LoadedExecutable* loaded_executable; /* out */
          const char* overridden_serialized_compile_options; size_t overridden_serialized_compile_options_size;);

typedef struct PJRT_ExecuteOptions {
    size_t struct_size;
    PJRT_Extension_Base* extension_start;
    void** send_callbacks;
    void** recv_callbacks;
    size_t num_send_ops;
    size_t num_recv_ops;
    int launch_id;
    const int64_t* non_donatable_input_indices;
    size_t num_non_donatable_input_indices;
    PJRT_ExecuteContext* context;
    const char* call_location;
    size_t num_tasks;
    int* task_ids;
    int64_t* incarnation_ids;
} PJRT_ExecuteOptions;
PJRT_ARGS(PJRT_LoadedExecutable_Execute,
          PJRT_LoadedExecutable* executable; PJRT_ExecuteOptions* options;
          PJRT_Buffer* const* const* argument_lists;   /* [num_devices][num_args] */
          size_t num_devices; size_t num_args;
          PJRT_Buffer** const* output_lists;           /* [num_devices][num_outputs], filled with new buffers */
          PJRT_Event** device_complete_events;         /* [num_devices] or NULL; filled with new events */
          PJRT_Device* execute_device;);

/* ---- buffers ---- */
PJRT_ARGS(PJRT_Buffer_Destroy, PJRT_Buffer* buffer;);
PJRT_ARGS(PJRT_Buffer_ElementType, PJRT_Buffer* buffer; PJRT_Buffer_Type type; /* out */);
PJRT_ARGS(PJRT_Buffer_Dimensions, PJRT_Buffer* buffer; const int64_t* dims; /* out */ size_t num_dims; /* out */);
PJRT_ARGS(PJRT_Buffer_UnpaddedDimensions, PJRT_Buffer* buffer; const int64_t* unpadded_dims; /* out */ size_t num_dims; /* out */);
PJRT_ARGS(PJRT_Buffer_DynamicDimensionIndices, PJRT_Buffer* buffer; const size_t* dynamic_dim_indices; /* out */ size_t num_dynamic_dims; /* out */);
PJRT_ARGS(PJRT_Buffer_GetMemoryLayout, PJRT_Buffer* buffer; PJRT_Buffer_MemoryLayout layout; /* out */);
PJRT_ARGS(PJRT_Buffer_ToHostBuffer, PJRT_Buffer* src; PJRT_Buffer_MemoryLayout* host_layout; void* dst; /* NULL: only report dst_size */
          size_t dst_size; /* in/out */ PJRT_Event* event; /* out */);
PJRT_ARGS(PJRT_Buffer_OnDeviceSizeInBytes, PJRT_Buffer* buffer; size_t on_device_size_in_bytes; /* out */);
PJRT_ARGS(PJRT_Buffer_Delete, PJRT_Buffer* buffer;);
PJRT_ARGS(PJRT_Buffer_IsDeleted, PJRT_Buffer* buffer; bool is_deleted; /* out */);
PJRT_ARGS(PJRT_Buffer_CopyRawToHost, PJRT_Buffer* buffer; void* dst; int64_t offset; int64_t transfer_size; PJRT_Event* event; /* out */);
PJRT_ARGS(PJRT_Buffer_CopyToDevice, PJRT_Buffer* buffer; PJRT_Device* dst_device; PJRT_Buffer* dst_buffer; /* out */);
PJRT_ARGS(PJRT_Buffer_CopyToMemory, PJRT_Buffer* buffer; PJRT_Memory* dst_memory; PJRT_Buffer* dst_buffer; /* out */);
PJRT_ARGS(PJRT_Buffer_IsOnCpu, PJRT_Buffer* buffer; bool is_on_cpu; /* out */);
PJRT_ARGS(PJRT_Buffer_Device, PJRT_Buffer* buffer; PJRT_Device* device; /* out */);
PJRT_ARGS(PJRT_Buffer_Memory, PJRT_Buffer* buffer; PJRT_Memory* memory; /* out */);
PJRT_ARGS(PJRT_Buffer_ReadyEvent, PJRT_Buffer* buffer; PJRT_Event* event; /* out: caller destroys */);
PJRT_ARGS(PJRT_Buffer_UnsafePointer, PJRT_Buffer* buffer; uintptr_t buffer_pointer; /* out */);
PJRT_ARGS(PJRT_Buffer_IncreaseExternalReferenceCount, PJRT_Buffer* buffer;);
PJRT_ARGS(PJRT_Buffer_DecreaseExternalReferenceCount, PJRT_Buffer* buffer;);
PJRT_ARGS(PJRT_Buffer_OpaqueDeviceMemoryDataPointer, PJRT_Buffer* buffer; void* device_memory_ptr; /* out */);

/* ---- topology ---- */
PJRT_ARGS(PJRT_TopologyDescription_Create, const char* topology_name; size_t topology_name_size; const PJRT_NamedValue* create_options;
          size_t num_options; PJRT_TopologyDescription* topology; /* out */);
PJRT_ARGS(PJRT_TopologyDescription_Destroy, PJRT_TopologyDescription* topology;);
PJRT_ARGS(PJRT_TopologyDescription_PlatformVersion, PJRT_TopologyDescription* topology; const char* platform_version; /* out */
          size_t platform_version_size; /* out */);
PJRT_ARGS(PJRT_TopologyDescription_PlatformName, const PJRT_TopologyDescription* topology; const char* platform_name; /* out */
          size_t platform_name_size; /* out */);
PJRT_ARGS(PJRT_TopologyDescription_GetDeviceDescriptions, const PJRT_TopologyDescription* topology;
          PJRT_DeviceDescription* const* descriptions; /* out */ size_t num_descriptions; /* out */);
PJRT_ARGS(PJRT_TopologyDescription_Attributes, PJRT_TopologyDescription* topology; const PJRT_NamedValue* attributes; /* out */
          size_t num_attributes; /* out */);

#undef PJRT_ARGS
#undef PJRT_ARGS_VOID

/* The function table.  Slot order is the interface's; `void*` slots are not offered. */
typedef struct PJRT_Api {
    size_t struct_size;
    PJRT_Extension_Base* extension_start;
    PJRT_Api_Version pjrt_api_version;

    PJRT_Error_Destroy* PJRT_Error_Destroy;
    PJRT_Error_Message* PJRT_Error_Message;
    PJRT_Error_GetCode* PJRT_Error_GetCode;
    PJRT_Plugin_Initialize* PJRT_Plugin_Initialize;
    PJRT_Plugin_Attributes* PJRT_Plugin_Attributes;
    PJRT_Event_Destroy* PJRT_Event_Destroy;
    PJRT_Event_IsReady* PJRT_Event_IsReady;
    PJRT_Event_Error* PJRT_Event_Error;
    PJRT_Event_Await* PJRT_Event_Await;
    PJRT_Event_OnReady* PJRT_Event_OnReady;
    PJRT_Client_Create* PJRT_Client_Create;
    PJRT_Client_Destroy* PJRT_Client_Destroy;
    PJRT_Client_PlatformName* PJRT_Client_PlatformName;
    PJRT_Client_ProcessIndex* PJRT_Client_ProcessIndex;
    PJRT_Client_PlatformVersion* PJRT_Client_PlatformVersion;
    PJRT_Client_Devices* PJRT_Client_Devices;
    PJRT_Client_AddressableDevices* PJRT_Client_AddressableDevices;
    PJRT_Client_LookupDevice* PJRT_Client_LookupDevice;
    PJRT_Client_LookupAddressableDevice* PJRT_Client_LookupAddressableDevice;
    PJRT_Client_AddressableMemories* PJRT_Client_AddressableMemories;
    PJRT_Client_Compile* PJRT_Client_Compile;
    PJRT_Client_DefaultDeviceAssignment* PJRT_Client_DefaultDeviceAssignment;
    PJRT_Client_BufferFromHostBuffer* PJRT_Client_BufferFromHostBuffer;
    PJRT_DeviceDescription_Id* PJRT_DeviceDescription_Id;
    PJRT_DeviceDescription_ProcessIndex* PJRT_DeviceDescription_ProcessIndex;
    PJRT_DeviceDescription_Attributes* PJRT_DeviceDescription_Attributes;
    PJRT_DeviceDescription_Kind* PJRT_DeviceDescription_Kind;
    PJRT_DeviceDescription_DebugString* PJRT_DeviceDescription_DebugString;
    PJRT_DeviceDescription_ToString* PJRT_DeviceDescription_ToString;
    PJRT_Device_GetDescription* PJRT_Device_GetDescription;
    PJRT_Device_IsAddressable* PJRT_Device_IsAddressable;
    PJRT_Device_LocalHardwareId* PJRT_Device_LocalHardwareId;
    PJRT_Device_AddressableMemories* PJRT_Device_AddressableMemories;
    PJRT_Device_DefaultMemory* PJRT_Device_DefaultMemory;
    PJRT_Device_MemoryStats* PJRT_Device_MemoryStats;
    PJRT_Memory_Id* PJRT_Memory_Id;
    PJRT_Memory_Kind* PJRT_Memory_Kind;
    PJRT_Memory_DebugString* PJRT_Memory_DebugString;
    PJRT_Memory_ToString* PJRT_Memory_ToString;
    PJRT_Memory_AddressableByDevices* PJRT_Memory_AddressableByDevices;
    PJRT_Executable_Destroy* PJRT_Executable_Destroy;
    PJRT_Executable_Name* PJRT_Executable_Name;
    PJRT_Executable_NumReplicas* PJRT_Executable_NumReplicas;
    PJRT_Executable_NumPartitions* PJRT_Executable_NumPartitions;
    PJRT_Executable_NumOutputs* PJRT_Executable_NumOutputs;
    PJRT_Executable_SizeOfGeneratedCodeInBytes* PJRT_Executable_SizeOfGeneratedCodeInBytes;
    PJRT_Executable_GetCostAnalysis* PJRT_Executable_GetCostAnalysis;
    PJRT_Executable_OutputMemoryKinds* PJRT_Executable_OutputMemoryKinds;
    PJRT_Executable_OptimizedProgram* PJRT_Executable_OptimizedProgram;
    PJRT_Executable_Serialize* PJRT_Executable_Serialize;
    PJRT_LoadedExecutable_Destroy* PJRT_LoadedExecutable_Destroy;
    PJRT_LoadedExecutable_GetExecutable* PJRT_LoadedExecutable_GetExecutable;
    PJRT_LoadedExecutable_AddressableDevices* PJRT_LoadedExecutable_AddressableDevices;
    PJRT_LoadedExecutable_Delete* PJRT_LoadedExecutable_Delete;
    PJRT_LoadedExecutable_IsDeleted* PJRT_LoadedExecutable_IsDeleted;
    PJRT_LoadedExecutable_Execute* PJRT_LoadedExecutable_Execute;
    PJRT_Executable_DeserializeAndLoad* PJRT_Executable_DeserializeAndLoad;
    PJRT_LoadedExecutable_Fingerprint* PJRT_LoadedExecutable_Fingerprint;
    PJRT_Buffer_Destroy* PJRT_Buffer_Destroy;
    PJRT_Buffer_ElementType* PJRT_Buffer_ElementType;
    PJRT_Buffer_Dimensions* PJRT_Buffer_Dimensions;
    PJRT_Buffer_UnpaddedDimensions* PJRT_Buffer_UnpaddedDimensions;
    PJRT_Buffer_DynamicDimensionIndices* PJRT_Buffer_DynamicDimensionIndices;
    PJRT_Buffer_GetMemoryLayout* PJRT_Buffer_GetMemoryLayout;
    PJRT_Buffer_OnDeviceSizeInBytes* PJRT_Buffer_OnDeviceSizeInBytes;
    PJRT_Buffer_Device* PJRT_Buffer_Device;
    PJRT_Buffer_Memory* PJRT_Buffer_Memory;
    PJRT_Buffer_Delete* PJRT_Buffer_Delete;
    PJRT_Buffer_IsDeleted* PJRT_Buffer_IsDeleted;
    PJRT_Buffer_CopyToDevice* PJRT_Buffer_CopyToDevice;
    PJRT_Buffer_ToHostBuffer* PJRT_Buffer_ToHostBuffer;
    PJRT_Buffer_IsOnCpu* PJRT_Buffer_IsOnCpu;
    PJRT_Buffer_ReadyEvent* PJRT_Buffer_ReadyEvent;
    PJRT_Buffer_UnsafePointer* PJRT_Buffer_UnsafePointer;
    PJRT_Buffer_IncreaseExternalReferenceCount* PJRT_Buffer_IncreaseExternalReferenceCount;
    PJRT_Buffer_DecreaseExternalReferenceCount* PJRT_Buffer_DecreaseExternalReferenceCount;
    PJRT_Buffer_OpaqueDeviceMemoryDataPointer* PJRT_Buffer_OpaqueDeviceMemoryDataPointer;
    void* PJRT_CopyToDeviceStream_Destroy;
    void* PJRT_CopyToDeviceStream_AddChunk;
    void* PJRT_CopyToDeviceStream_TotalBytes;
    void* PJRT_CopyToDeviceStream_GranuleSize;
    void* PJRT_CopyToDeviceStream_CurrentBytes;
    PJRT_TopologyDescription_Create* PJRT_TopologyDescription_Create;
    PJRT_TopologyDescription_Destroy* PJRT_TopologyDescription_Destroy;
    PJRT_TopologyDescription_PlatformName* PJRT_TopologyDescription_PlatformName;
    PJRT_TopologyDescription_PlatformVersion* PJRT_TopologyDescription_PlatformVersion;
    PJRT_TopologyDescription_GetDeviceDescriptions* PJRT_TopologyDescription_GetDeviceDescriptions;
    void* PJRT_TopologyDescription_Serialize;
    PJRT_TopologyDescription_Attributes* PJRT_TopologyDescription_Attributes;
    void* PJRT_Compile;
    PJRT_Executable_OutputElementTypes* PJRT_Executable_OutputElementTypes;
    PJRT_Executable_OutputDimensions* PJRT_Executable_OutputDimensions;
    PJRT_Buffer_CopyToMemory* PJRT_Buffer_CopyToMemory;
    void* PJRT_Client_CreateViewOfDeviceBuffer;
    PJRT_Executable_Fingerprint* PJRT_Executable_Fingerprint;
    PJRT_Client_TopologyDescription* PJRT_Client_TopologyDescription;
    PJRT_Executable_GetCompiledMemoryStats* PJRT_Executable_GetCompiledMemoryStats;
    PJRT_Memory_Kind_Id* PJRT_Memory_Kind_Id;
    void* PJRT_ExecuteContext_Create;
    void* PJRT_ExecuteContext_Destroy;
    PJRT_Buffer_CopyRawToHost* PJRT_Buffer_CopyRawToHost;
    void* PJRT_AsyncHostToDeviceTransferManager_Destroy;
    void* PJRT_AsyncHostToDeviceTransferManager_TransferData;
    void* PJRT_Client_CreateBuffersForAsyncHostToDevice;
    void* PJRT_AsyncHostToDeviceTransferManager_RetrieveBuffer;
    void* PJRT_AsyncHostToDeviceTransferManager_Device;
    void* PJRT_AsyncHostToDeviceTransferManager_BufferCount;
    void* PJRT_AsyncHostToDeviceTransferManager_BufferSize;
    void* PJRT_AsyncHostToDeviceTransferManager_SetBufferError;
    void* PJRT_AsyncHostToDeviceTransferManager_AddMetadata;
    void* PJRT_Client_DmaMap;
    void* PJRT_Client_DmaUnmap;
    void* PJRT_Client_CreateUninitializedBuffer;
    void* PJRT_Client_UpdateGlobalProcessInfo;
    void* PJRT_TopologyDescription_Deserialize;
    void* PJRT_Client_CreateAliasBuffer;
    void* PJRT_Client_FulfillAliasBuffer;
    PJRT_LoadedExecutable_GetDeviceAssignment* PJRT_LoadedExecutable_GetDeviceAssignment;
    void* PJRT_Client_CreateErrorBuffer;
    void* PJRT_AsyncHostToDeviceTransferManager_TransferLiteral;
    void* PJRT_Buffer_CopyRawToHostFuture;
    void* PJRT_Device_PoisonExecution;
    void* PJRT_Device_CreateAsyncTrackingEvent;
    void* PJRT_AsyncTrackingEvent_Destroy;
    void* PJRT_Executable_GetCompileOptions;
    void* PJRT_Buffer_DonateWithControlDependency;
    void* PJRT_Event_Create;
    void* PJRT_Event_Set;
} PJRT_Api;

/* The one exported symbol (PJRTApi.swift:170-173): the table lives for the whole process. */
/* The one exported symbol of the plugin (it is built with hidden visibility). */
#if defined(__GNUC__)
__attribute__((visibility("default")))
#endif
const PJRT_Api* GetPjrtApi(void);

#ifdef __cplusplus
}
#endif
#endif  /* MHLO_PJRT_ABI_H_ */
