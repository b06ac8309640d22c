// Compile-time comparison of include/pjrt_abi.h with the OpenXLA PJRT C API header
// (given with -DPJRT_REFERENCE_HEADER="<path>").  It only has to compile: every check is
// a static_assert.  tests/test_pjrt_host.py builds it when such a header is available.
#include <cstddef>
#include PJRT_REFERENCE_HEADER
namespace mine {
#include "pjrt_abi.h"
}

#define SAME_SIZE(T) static_assert(sizeof(mine::T) == sizeof(::T), "size of " #T)
#define SAME_FIELD(T, f) static_assert(offsetof(mine::T, f) == offsetof(::T, f) && sizeof(((mine::T*)0)->f) == sizeof(((::T*)0)->f), #T "." #f)
#define SAME_SLOT(f) static_assert(offsetof(mine::PJRT_Api, f) == offsetof(::PJRT_Api, f), "table slot " #f);

SAME_SIZE(PJRT_Api); SAME_SIZE(PJRT_Extension_Base); SAME_SIZE(PJRT_Api_Version); SAME_SIZE(PJRT_NamedValue); SAME_SIZE(PJRT_Program);
SAME_SIZE(PJRT_Buffer_MemoryLayout); SAME_SIZE(PJRT_ExecuteOptions);
SAME_FIELD(PJRT_NamedValue, type); SAME_FIELD(PJRT_NamedValue, int64_value); SAME_FIELD(PJRT_NamedValue, value_size);
SAME_FIELD(PJRT_Program, code_size); SAME_FIELD(PJRT_Program, format); SAME_FIELD(PJRT_Program, format_size);
SAME_FIELD(PJRT_Buffer_MemoryLayout, type); SAME_FIELD(PJRT_Buffer_MemoryLayout, strides);
SAME_FIELD(PJRT_ExecuteOptions, launch_id); SAME_FIELD(PJRT_ExecuteOptions, context); SAME_FIELD(PJRT_ExecuteOptions, incarnation_ids);

// enum values used across the boundary
static_assert((int)mine::PJRT_Error_Code_UNIMPLEMENTED == (int)::PJRT_Error_Code_UNIMPLEMENTED, "");
static_assert((int)mine::PJRT_Error_Code_INVALID_ARGUMENT == (int)::PJRT_Error_Code_INVALID_ARGUMENT, "");
static_assert((int)mine::PJRT_Buffer_Type_PRED == (int)::PJRT_Buffer_Type_PRED && (int)mine::PJRT_Buffer_Type_S64 == (int)::PJRT_Buffer_Type_S64 &&
              (int)mine::PJRT_Buffer_Type_U64 == (int)::PJRT_Buffer_Type_U64 && (int)mine::PJRT_Buffer_Type_F16 == (int)::PJRT_Buffer_Type_F16 &&
              (int)mine::PJRT_Buffer_Type_F64 == (int)::PJRT_Buffer_Type_F64 && (int)mine::PJRT_Buffer_Type_BF16 == (int)::PJRT_Buffer_Type_BF16 &&
              (int)mine::PJRT_Buffer_Type_C128 == (int)::PJRT_Buffer_Type_C128, "buffer types");
static_assert((int)mine::PJRT_NamedValue_kBool == (int)::PJRT_NamedValue_kBool, "");
static_assert((int)mine::PJRT_HostBufferSemantics_kMutableZeroCopy == (int)::PJRT_HostBufferSemantics_kMutableZeroCopy, "");

// argument structs: size, and the offset of every field the plugin reads or writes
#define A1(T, a) SAME_SIZE(T); SAME_FIELD(T, a)
#define A2(T, a, b) A1(T, a); SAME_FIELD(T, b)
#define A3(T, a, b, c) A2(T, a, b); SAME_FIELD(T, c)
#define A4(T, a, b, c, d) A3(T, a, b, c); SAME_FIELD(T, d)
#define A5(T, a, b, c, d, e) A4(T, a, b, c, d); SAME_FIELD(T, e)
A1(PJRT_Error_Destroy_Args, error); A3(PJRT_Error_Message_Args, error, message, message_size); A2(PJRT_Error_GetCode_Args, error, code);
SAME_SIZE(PJRT_Plugin_Initialize_Args); A2(PJRT_Plugin_Attributes_Args, attributes, num_attributes);
A1(PJRT_Event_Destroy_Args, event); A2(PJRT_Event_IsReady_Args, event, is_ready); A1(PJRT_Event_Error_Args, event); A1(PJRT_Event_Await_Args, event);
A3(PJRT_Event_OnReady_Args, event, callback, user_arg);
A5(PJRT_Client_Create_Args, create_options, num_options, client, kv_try_get_callback, kv_try_get_user_arg); A1(PJRT_Client_Destroy_Args, client);
A3(PJRT_Client_PlatformName_Args, client, platform_name, platform_name_size); A2(PJRT_Client_ProcessIndex_Args, client, process_index);
A3(PJRT_Client_PlatformVersion_Args, client, platform_version, platform_version_size); A2(PJRT_Client_TopologyDescription_Args, client, topology);
A3(PJRT_Client_Devices_Args, client, devices, num_devices); A3(PJRT_Client_AddressableDevices_Args, client, addressable_devices, num_addressable_devices);
A3(PJRT_Client_LookupDevice_Args, client, id, device); A3(PJRT_Client_LookupAddressableDevice_Args, client, local_hardware_id, addressable_device);
A3(PJRT_Client_AddressableMemories_Args, client, addressable_memories, num_addressable_memories);
A5(PJRT_Client_Compile_Args, client, program, compile_options, compile_options_size, executable);
A5(PJRT_Client_DefaultDeviceAssignment_Args, client, num_replicas, num_partitions, default_assignment_size, default_assignment);
A5(PJRT_Client_BufferFromHostBuffer_Args, client, data, type, dims, num_dims); A5(PJRT_Client_BufferFromHostBuffer_Args, byte_strides, num_byte_strides, host_buffer_semantics, device, memory);
A3(PJRT_Client_BufferFromHostBuffer_Args, device_layout, done_with_host_buffer, buffer);
A2(PJRT_DeviceDescription_Id_Args, device_description, id); A2(PJRT_DeviceDescription_ProcessIndex_Args, device_description, process_index);
A3(PJRT_DeviceDescription_Attributes_Args, device_description, num_attributes, attributes); A3(PJRT_DeviceDescription_Kind_Args, device_description, device_kind, device_kind_size);
A3(PJRT_DeviceDescription_DebugString_Args, device_description, debug_string, debug_string_size); A3(PJRT_DeviceDescription_ToString_Args, device_description, to_string, to_string_size);
A2(PJRT_Device_GetDescription_Args, device, device_description); A2(PJRT_Device_IsAddressable_Args, device, is_addressable); A2(PJRT_Device_LocalHardwareId_Args, device, local_hardware_id);
A3(PJRT_Device_AddressableMemories_Args, device, memories, num_memories); A2(PJRT_Device_DefaultMemory_Args, device, memory);
A5(PJRT_Device_MemoryStats_Args, device, bytes_in_use, peak_bytes_in_use_is_set, bytes_limit, bytes_limit_is_set); A2(PJRT_Device_MemoryStats_Args, peak_pool_bytes, peak_pool_bytes_is_set);
A2(PJRT_Memory_Id_Args, memory, id); A3(PJRT_Memory_Kind_Args, memory, kind, kind_size); A2(PJRT_Memory_Kind_Id_Args, memory, kind_id);
A3(PJRT_Memory_DebugString_Args, memory, debug_string, debug_string_size); A3(PJRT_Memory_ToString_Args, memory, to_string, to_string_size);
A3(PJRT_Memory_AddressableByDevices_Args, memory, devices, num_devices);
A1(PJRT_Executable_Destroy_Args, executable); A3(PJRT_Executable_Name_Args, executable, executable_name, executable_name_size);
A2(PJRT_Executable_NumReplicas_Args, executable, num_replicas); A2(PJRT_Executable_NumPartitions_Args, executable, num_partitions); A2(PJRT_Executable_NumOutputs_Args, executable, num_outputs);
A2(PJRT_Executable_SizeOfGeneratedCodeInBytes_Args, executable, size_in_bytes); A3(PJRT_Executable_GetCostAnalysis_Args, executable, num_properties, properties);
A4(PJRT_Executable_OutputMemoryKinds_Args, executable, num_outputs, memory_kinds, memory_kind_sizes); A2(PJRT_Executable_OptimizedProgram_Args, executable, program);
A5(PJRT_Executable_Serialize_Args, executable, serialized_bytes, serialized_bytes_size, serialized_executable, serialized_executable_deleter);
A3(PJRT_Executable_OutputElementTypes_Args, executable, output_types, num_output_types); A4(PJRT_Executable_OutputDimensions_Args, executable, num_outputs, dims, dim_sizes);
A3(PJRT_Executable_Fingerprint_Args, executable, executable_fingerprint, executable_fingerprint_size); A2(PJRT_Executable_GetCompiledMemoryStats_Args, executable, total_size_in_bytes);
A1(PJRT_LoadedExecutable_Destroy_Args, executable); A2(PJRT_LoadedExecutable_GetExecutable_Args, loaded_executable, executable);
A3(PJRT_LoadedExecutable_AddressableDevices_Args, executable, addressable_devices, num_addressable_devices); A1(PJRT_LoadedExecutable_Delete_Args, executable);
A2(PJRT_LoadedExecutable_IsDeleted_Args, executable, is_deleted); A3(PJRT_LoadedExecutable_Fingerprint_Args, executable, executable_fingerprint, executable_fingerprint_size);
A5(PJRT_LoadedExecutable_GetDeviceAssignment_Args, executable, serialized_bytes, serialized_bytes_size, serialized_device_assignment, serialized_device_assignment_deleter);
A5(PJRT_Executable_DeserializeAndLoad_Args, client, serialized_executable, serialized_executable_size, loaded_executable, overridden_serialized_compile_options_size);
A5(PJRT_LoadedExecutable_Execute_Args, executable, options, argument_lists, num_devices, num_args); A3(PJRT_LoadedExecutable_Execute_Args, output_lists, device_complete_events, execute_device);
A1(PJRT_Buffer_Destroy_Args, buffer); A2(PJRT_Buffer_ElementType_Args, buffer, type); A3(PJRT_Buffer_Dimensions_Args, buffer, dims, num_dims);
A3(PJRT_Buffer_UnpaddedDimensions_Args, buffer, unpadded_dims, num_dims); A3(PJRT_Buffer_DynamicDimensionIndices_Args, buffer, dynamic_dim_indices, num_dynamic_dims);
A2(PJRT_Buffer_GetMemoryLayout_Args, buffer, layout); A5(PJRT_Buffer_ToHostBuffer_Args, src, host_layout, dst, dst_size, event);
A2(PJRT_Buffer_OnDeviceSizeInBytes_Args, buffer, on_device_size_in_bytes); A1(PJRT_Buffer_Delete_Args, buffer); A2(PJRT_Buffer_IsDeleted_Args, buffer, is_deleted);
A5(PJRT_Buffer_CopyRawToHost_Args, buffer, dst, offset, transfer_size, event); A3(PJRT_Buffer_CopyToDevice_Args, buffer, dst_device, dst_buffer);
A3(PJRT_Buffer_CopyToMemory_Args, buffer, dst_memory, dst_buffer); A2(PJRT_Buffer_IsOnCpu_Args, buffer, is_on_cpu); A2(PJRT_Buffer_Device_Args, buffer, device);
A2(PJRT_Buffer_Memory_Args, buffer, memory); A2(PJRT_Buffer_ReadyEvent_Args, buffer, event); A2(PJRT_Buffer_UnsafePointer_Args, buffer, buffer_pointer);
A1(PJRT_Buffer_IncreaseExternalReferenceCount_Args, buffer); A1(PJRT_Buffer_DecreaseExternalReferenceCount_Args, buffer);
A2(PJRT_Buffer_OpaqueDeviceMemoryDataPointer_Args, buffer, device_memory_ptr);
A5(PJRT_TopologyDescription_Create_Args, topology_name, topology_name_size, create_options, num_options, topology); A1(PJRT_TopologyDescription_Destroy_Args, topology);
A3(PJRT_TopologyDescription_PlatformVersion_Args, topology, platform_version, platform_version_size); A3(PJRT_TopologyDescription_PlatformName_Args, topology, platform_name, platform_name_size);
A3(PJRT_TopologyDescription_GetDeviceDescriptions_Args, topology, descriptions, num_descriptions); A3(PJRT_TopologyDescription_Attributes_Args, topology, attributes, num_attributes);

// every slot of the table
#define SLOTS(X) X(PJRT_Error_Destroy) X(PJRT_Error_Message) X(PJRT_Error_GetCode) X(PJRT_Plugin_Initialize) X(PJRT_Plugin_Attributes) \
  X(PJRT_Event_Destroy) X(PJRT_Event_IsReady) X(PJRT_Event_Error) X(PJRT_Event_Await) X(PJRT_Event_OnReady) X(PJRT_Client_Create) X(PJRT_Client_Destroy) \
  X(PJRT_Client_PlatformName) X(PJRT_Client_ProcessIndex) X(PJRT_Client_PlatformVersion) X(PJRT_Client_Devices) X(PJRT_Client_AddressableDevices) \
  X(PJRT_Client_LookupDevice) X(PJRT_Client_LookupAddressableDevice) X(PJRT_Client_AddressableMemories) X(PJRT_Client_Compile) \
  X(PJRT_Client_DefaultDeviceAssignment) X(PJRT_Client_BufferFromHostBuffer) X(PJRT_DeviceDescription_Id) X(PJRT_DeviceDescription_ProcessIndex) \
  X(PJRT_DeviceDescription_Attributes) X(PJRT_DeviceDescription_Kind) X(PJRT_DeviceDescription_DebugString) X(PJRT_DeviceDescription_ToString) \
  X(PJRT_Device_GetDescription) X(PJRT_Device_IsAddressable) X(PJRT_Device_LocalHardwareId) X(PJRT_Device_AddressableMemories) X(PJRT_Device_DefaultMemory) \
  X(PJRT_Device_MemoryStats) X(PJRT_Memory_Id) X(PJRT_Memory_Kind) X(PJRT_Memory_DebugString) X(PJRT_Memory_ToString) X(PJRT_Memory_AddressableByDevices) \
  X(PJRT_Executable_Destroy) X(PJRT_Executable_Name) X(PJRT_Executable_NumReplicas) X(PJRT_Executable_NumPartitions) X(PJRT_Executable_NumOutputs) \
  X(PJRT_Executable_SizeOfGeneratedCodeInBytes) X(PJRT_Executable_GetCostAnalysis) X(PJRT_Executable_OutputMemoryKinds) X(PJRT_Executable_OptimizedProgram) \
  X(PJRT_Executable_Serialize) X(PJRT_LoadedExecutable_Destroy) X(PJRT_LoadedExecutable_GetExecutable) X(PJRT_LoadedExecutable_AddressableDevices) \
  X(PJRT_LoadedExecutable_Delete) X(PJRT_LoadedExecutable_IsDeleted) X(PJRT_LoadedExecutable_Execute) X(PJRT_Executable_DeserializeAndLoad) \
  X(PJRT_LoadedExecutable_Fingerprint) X(PJRT_Buffer_Destroy) X(PJRT_Buffer_ElementType) X(PJRT_Buffer_Dimensions) X(PJRT_Buffer_UnpaddedDimensions) \
  X(PJRT_Buffer_DynamicDimensionIndices) X(PJRT_Buffer_GetMemoryLayout) X(PJRT_Buffer_OnDeviceSizeInBytes) X(PJRT_Buffer_Device) X(PJRT_Buffer_Memory) \
  X(PJRT_Buffer_Delete) X(PJRT_Buffer_IsDeleted) X(PJRT_Buffer_CopyToDevice) X(PJRT_Buffer_ToHostBuffer) X(PJRT_Buffer_IsOnCpu) X(PJRT_Buffer_ReadyEvent) \
  X(PJRT_Buffer_UnsafePointer) X(PJRT_Buffer_IncreaseExternalReferenceCount) X(PJRT_Buffer_DecreaseExternalReferenceCount) \
  X(PJRT_Buffer_OpaqueDeviceMemoryDataPointer) X(PJRT_CopyToDeviceStream_Destroy) X(PJRT_CopyToDeviceStream_AddChunk) X(PJRT_CopyToDeviceStream_TotalBytes) \
  X(PJRT_CopyToDeviceStream_GranuleSize) X(PJRT_CopyToDeviceStream_CurrentBytes) X(PJRT_TopologyDescription_Create) X(PJRT_TopologyDescription_Destroy) \
  X(PJRT_TopologyDescription_PlatformName) X(PJRT_TopologyDescription_PlatformVersion) X(PJRT_TopologyDescription_GetDeviceDescriptions) \
  X(PJRT_TopologyDescription_Serialize) X(PJRT_TopologyDescription_Attributes) X(PJRT_Compile) X(PJRT_Executable_OutputElementTypes) \
  X(PJRT_Executable_OutputDimensions) X(PJRT_Buffer_CopyToMemory) X(PJRT_Client_CreateViewOfDeviceBuffer) X(PJRT_Executable_Fingerprint) \
  X(PJRT_Client_TopologyDescription) X(PJRT_Executable_GetCompiledMemoryStats) X(PJRT_Memory_Kind_Id) X(PJRT_ExecuteContext_Create) \
  X(PJRT_ExecuteContext_Destroy) X(PJRT_Buffer_CopyRawToHost) X(PJRT_AsyncHostToDeviceTransferManager_Destroy) \
  X(PJRT_AsyncHostToDeviceTransferManager_TransferData) X(PJRT_Client_CreateBuffersForAsyncHostToDevice) \
  X(PJRT_AsyncHostToDeviceTransferManager_RetrieveBuffer) X(PJRT_AsyncHostToDeviceTransferManager_Device) \
  X(PJRT_AsyncHostToDeviceTransferManager_BufferCount) X(PJRT_AsyncHostToDeviceTransferManager_BufferSize) \
  X(PJRT_AsyncHostToDeviceTransferManager_SetBufferError) X(PJRT_AsyncHostToDeviceTransferManager_AddMetadata) X(PJRT_Client_DmaMap) \
  X(PJRT_Client_DmaUnmap) X(PJRT_Client_CreateUninitializedBuffer) X(PJRT_Client_UpdateGlobalProcessInfo) X(PJRT_TopologyDescription_Deserialize) \
  X(PJRT_Client_CreateAliasBuffer) X(PJRT_Client_FulfillAliasBuffer) X(PJRT_LoadedExecutable_GetDeviceAssignment) X(PJRT_Client_CreateErrorBuffer) \
  X(PJRT_AsyncHostToDeviceTransferManager_TransferLiteral) X(PJRT_Buffer_CopyRawToHostFuture) X(PJRT_Device_PoisonExecution) \
  X(PJRT_Device_CreateAsyncTrackingEvent) X(PJRT_AsyncTrackingEvent_Destroy) X(PJRT_Executable_GetCompileOptions) \
  X(PJRT_Buffer_DonateWithControlDependency) X(PJRT_Event_Create) X(PJRT_Event_Set)
SLOTS(SAME_SLOT)

int main() { return 0; }
