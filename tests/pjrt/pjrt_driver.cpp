// Drives libPJRTMetalHLO.so through its function table the way a PJRT client does (dlopen,
// GetPjrtApi, argument structs with struct_size set).  Usage: pjrt_driver <plugin.so> host|gpu
// Prints one "ok <case>" line per case; the first failed check prints "FAIL ..." and exits 1.
// The cases restate Tests/PJRTMetalHLOTests/PJRTPluginTests.swift (table version and slots
// :160-180, error lifecycle :182-207, events :209-235, platform and device :237-261, host
// round trip :263-285, compile + execute add :287-318, serialize / deserialize :406-467);
// case_async_transfers has no counterpart there (the reference's transfers complete inside
// the call): it covers the asynchronous uploads and downloads of this plugin.
#include <dlfcn.h>
#include <execinfo.h>
#include <signal.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <string>
#include <thread>
#include <vector>

#include "pjrt_abi.h"

static const PJRT_Api* api;
typedef const PJRT_Api* (*GetApi)(void);
static GetApi get_api;

#define CHECK(cond)                                                                  \
    do {                                                                             \
        if (!(cond)) {                                                               \
            printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);                   \
            exit(1);                                                                 \
        }                                                                            \
    } while (0)
#define ARGS(T, name) \
    T name;           \
    memset(&name, 0, sizeof(name)); \
    name.struct_size = sizeof(name)

static PJRT_Error_Code code_of(PJRT_Error* e, std::string* msg = nullptr) {
    if (!e) return PJRT_Error_Code_OK;
    ARGS(PJRT_Error_GetCode_Args, c);
    c.error = e;
    CHECK(api->PJRT_Error_GetCode(&c) == nullptr);
    ARGS(PJRT_Error_Message_Args, m);
    m.error = e;
    api->PJRT_Error_Message(&m);
    CHECK(m.message != nullptr && m.message_size > 0 && strlen(m.message) == m.message_size);
    if (msg) msg->assign(m.message, m.message_size);
    ARGS(PJRT_Error_Destroy_Args, d);
    d.error = e;
    api->PJRT_Error_Destroy(&d);
    return c.code;
}
#define OK(call)                                                                                   \
    do {                                                                                           \
        std::string ok_msg;                                                                        \
        const PJRT_Error_Code ok_code = code_of(call, &ok_msg);                                    \
        if (ok_code != PJRT_Error_Code_OK) {                                                       \
            printf("FAIL %s:%d: %s -> code %d: %s\n", __FILE__, __LINE__, #call, (int)ok_code, ok_msg.c_str()); \
            fflush(stdout);                                                                        \
            exit(1);                                                                               \
        }                                                                                          \
    } while (0)

static const char* kAdd =
    "module @add {\n  func.func @main(%a: tensor<4xf32>, %b: tensor<4xf32>) -> tensor<4xf32> {\n"
    "    %0 = stablehlo.add %a, %b : tensor<4xf32>\n    return %0 : tensor<4xf32>\n  }\n}\n";
static const char* kSoftmax =
    "func.func @main(%x: tensor<2x4xf32>) -> tensor<2x4xf32> {\n"
    "  %0 = stablehlo.custom_call @fused_softmax(%x) {backend_config = \"{\\\"axis\\\": -1}\"} : (tensor<2x4xf32>) -> tensor<2x4xf32>\n"
    "  return %0 : tensor<2x4xf32>\n}\n";

static PJRT_Client* make_client() {
    ARGS(PJRT_Client_Create_Args, a);
    OK(api->PJRT_Client_Create(&a));
    CHECK(a.client != nullptr);
    return a.client;
}
static void destroy_client(PJRT_Client* c) {
    ARGS(PJRT_Client_Destroy_Args, a);
    a.client = c;
    OK(api->PJRT_Client_Destroy(&a));
}
static PJRT_Error* compile(PJRT_Client* c, const std::string& code, const char* format, PJRT_LoadedExecutable** out) {
    ARGS(PJRT_Program, prog);
    prog.code = const_cast<char*>(code.data());
    prog.code_size = code.size();
    prog.format = format;
    prog.format_size = strlen(format);
    ARGS(PJRT_Client_Compile_Args, a);
    a.client = c;
    a.program = &prog;
    PJRT_Error* e = api->PJRT_Client_Compile(&a);
    *out = a.executable;
    return e;
}
static void destroy_loaded(PJRT_LoadedExecutable* e) {
    ARGS(PJRT_LoadedExecutable_Destroy_Args, a);
    a.executable = e;
    OK(api->PJRT_LoadedExecutable_Destroy(&a));
}
static void destroy_event(PJRT_Event* e) {
    ARGS(PJRT_Event_Destroy_Args, a);
    a.event = e;
    OK(api->PJRT_Event_Destroy(&a));
}
static void destroy_buffer(PJRT_Buffer* b) {
    ARGS(PJRT_Buffer_Destroy_Args, a);
    a.buffer = b;
    OK(api->PJRT_Buffer_Destroy(&a));
}

// ---- cases that need no device -----------------------------------------------------------
static void case_table() {
    CHECK(api->struct_size == sizeof(PJRT_Api) && sizeof(PJRT_Api) == 1064);
    CHECK(api->pjrt_api_version.major_version == 0 && api->pjrt_api_version.minor_version == 90);
    CHECK(api->pjrt_api_version.struct_size == sizeof(PJRT_Api_Version));
    CHECK(api->PJRT_Error_Destroy && api->PJRT_Error_Message && api->PJRT_Error_GetCode && api->PJRT_Plugin_Initialize &&
          api->PJRT_Plugin_Attributes && api->PJRT_Event_Destroy && api->PJRT_Event_IsReady && api->PJRT_Event_Await &&
          api->PJRT_Event_OnReady && api->PJRT_Client_Create && api->PJRT_Client_Destroy && api->PJRT_Client_Compile &&
          api->PJRT_Client_BufferFromHostBuffer && api->PJRT_Client_Devices && api->PJRT_LoadedExecutable_Execute &&
          api->PJRT_Buffer_ToHostBuffer && api->PJRT_Executable_Serialize && api->PJRT_Executable_DeserializeAndLoad &&
          api->PJRT_Client_TopologyDescription && api->PJRT_Executable_Fingerprint && api->PJRT_LoadedExecutable_GetDeviceAssignment);
    CHECK(api->PJRT_Event_Set == nullptr && api->PJRT_Compile == nullptr);      // slots the plugin does not offer stay NULL
    CHECK(get_api() == api);                                // one table for the whole process
    ARGS(PJRT_Plugin_Initialize_Args, init);
    OK(api->PJRT_Plugin_Initialize(&init));
    ARGS(PJRT_Plugin_Attributes_Args, at);
    OK(api->PJRT_Plugin_Attributes(&at));
    CHECK(at.num_attributes >= 2 && at.attributes != nullptr);
    bool has_xla = false;
    for (size_t i = 0; i < at.num_attributes; i++) has_xla |= std::string(at.attributes[i].name, at.attributes[i].name_size) == "xla_version";
    CHECK(has_xla);
    printf("ok table\n");
}
static void case_errors(PJRT_Client* c) {
    std::string msg;
    ARGS(PJRT_Client_LookupDevice_Args, l);
    l.client = c;
    l.id = 5;
    CHECK(code_of(api->PJRT_Client_LookupDevice(&l), &msg) == PJRT_Error_Code_NOT_FOUND);
    CHECK(msg.find("5") != std::string::npos);
    CHECK(code_of(api->PJRT_Client_LookupDevice(nullptr)) == PJRT_Error_Code_INVALID_ARGUMENT);
    ARGS(PJRT_Client_PlatformName_Args, p);
    CHECK(code_of(api->PJRT_Client_PlatformName(&p)) == PJRT_Error_Code_INVALID_ARGUMENT);   // client is null
    ARGS(PJRT_Buffer_Dimensions_Args, d);
    CHECK(code_of(api->PJRT_Buffer_Dimensions(&d)) == PJRT_Error_Code_INVALID_ARGUMENT);
    ARGS(PJRT_Buffer_UnsafePointer_Args, u);
    CHECK(code_of(api->PJRT_Buffer_UnsafePointer(&u)) == PJRT_Error_Code_UNIMPLEMENTED);
    printf("ok errors\n");
}
static void case_platform(PJRT_Client* c) {
    ARGS(PJRT_Client_PlatformName_Args, n);
    n.client = c;
    OK(api->PJRT_Client_PlatformName(&n));
    CHECK(std::string(n.platform_name, n.platform_name_size) == "metalhlo");
    ARGS(PJRT_Client_PlatformVersion_Args, v);
    v.client = c;
    OK(api->PJRT_Client_PlatformVersion(&v));
    CHECK(std::string(v.platform_version, v.platform_version_size) == "0.1.0");
    ARGS(PJRT_Client_ProcessIndex_Args, pi);
    pi.client = c;
    pi.process_index = 7;
    OK(api->PJRT_Client_ProcessIndex(&pi));
    CHECK(pi.process_index == 0);
    ARGS(PJRT_Client_Devices_Args, ds);
    ds.client = c;
    OK(api->PJRT_Client_Devices(&ds));
    CHECK(ds.num_devices == 1 && ds.devices[0] != nullptr);
    ARGS(PJRT_Client_AddressableDevices_Args, ad);
    ad.client = c;
    OK(api->PJRT_Client_AddressableDevices(&ad));
    CHECK(ad.num_addressable_devices == 1 && ad.addressable_devices[0] == ds.devices[0]);
    ARGS(PJRT_Client_LookupDevice_Args, l);
    l.client = c;
    OK(api->PJRT_Client_LookupDevice(&l));
    CHECK(l.device == ds.devices[0]);
    ARGS(PJRT_Device_GetDescription_Args, gd);
    gd.device = ds.devices[0];
    OK(api->PJRT_Device_GetDescription(&gd));
    ARGS(PJRT_DeviceDescription_Id_Args, id);
    id.device_description = gd.device_description;
    id.id = 9;
    OK(api->PJRT_DeviceDescription_Id(&id));
    CHECK(id.id == 0);
    ARGS(PJRT_DeviceDescription_Kind_Args, k);
    k.device_description = gd.device_description;
    OK(api->PJRT_DeviceDescription_Kind(&k));
    CHECK(k.device_kind_size > 0);
    ARGS(PJRT_DeviceDescription_Attributes_Args, at);
    at.device_description = gd.device_description;
    OK(api->PJRT_DeviceDescription_Attributes(&at));
    CHECK(at.num_attributes == 2 && std::string(at.attributes[0].name, at.attributes[0].name_size) == "gfx_arch");
    ARGS(PJRT_Device_IsAddressable_Args, ia);
    ia.device = ds.devices[0];
    OK(api->PJRT_Device_IsAddressable(&ia));
    CHECK(ia.is_addressable);
    ARGS(PJRT_Device_DefaultMemory_Args, dm);
    dm.device = ds.devices[0];
    OK(api->PJRT_Device_DefaultMemory(&dm));
    ARGS(PJRT_Memory_Kind_Args, mk);
    mk.memory = dm.memory;
    OK(api->PJRT_Memory_Kind(&mk));
    CHECK(std::string(mk.kind, mk.kind_size) == "device");
    ARGS(PJRT_Memory_AddressableByDevices_Args, mad);
    mad.memory = dm.memory;
    OK(api->PJRT_Memory_AddressableByDevices(&mad));
    CHECK(mad.num_devices == 1 && mad.devices[0] == ds.devices[0]);
    ARGS(PJRT_Client_AddressableMemories_Args, am);
    am.client = c;
    OK(api->PJRT_Client_AddressableMemories(&am));
    CHECK(am.num_addressable_memories == 1 && am.addressable_memories[0] == dm.memory);
    int assign[1] = {42};
    ARGS(PJRT_Client_DefaultDeviceAssignment_Args, da);
    da.client = c;
    da.num_replicas = 1;
    da.num_partitions = 1;
    da.default_assignment_size = 1;
    da.default_assignment = assign;
    OK(api->PJRT_Client_DefaultDeviceAssignment(&da));
    CHECK(assign[0] == 0);
    da.num_replicas = 2;
    da.default_assignment_size = 1;
    CHECK(code_of(api->PJRT_Client_DefaultDeviceAssignment(&da)) == PJRT_Error_Code_INVALID_ARGUMENT);
    // topology: the client's own, and a standalone one
    ARGS(PJRT_Client_TopologyDescription_Args, ct);
    ct.client = c;
    OK(api->PJRT_Client_TopologyDescription(&ct));
    ARGS(PJRT_TopologyDescription_GetDeviceDescriptions_Args, tdd);
    tdd.topology = ct.topology;
    OK(api->PJRT_TopologyDescription_GetDeviceDescriptions(&tdd));
    CHECK(tdd.num_descriptions == 1 && tdd.descriptions[0] == gd.device_description);
    ARGS(PJRT_TopologyDescription_Create_Args, tc);
    OK(api->PJRT_TopologyDescription_Create(&tc));
    ARGS(PJRT_TopologyDescription_PlatformName_Args, tn);
    tn.topology = tc.topology;
    OK(api->PJRT_TopologyDescription_PlatformName(&tn));
    CHECK(std::string(tn.platform_name, tn.platform_name_size) == "metalhlo");
    ARGS(PJRT_TopologyDescription_Destroy_Args, td);
    td.topology = tc.topology;
    OK(api->PJRT_TopologyDescription_Destroy(&td));
    printf("ok platform\n");
}
static void case_compile(PJRT_Client* c) {
    PJRT_LoadedExecutable* le = nullptr;
    std::string msg;
    CHECK(code_of(compile(c, "this is not mlir", "mlir", &le), &msg) == PJRT_Error_Code_INVALID_ARGUMENT);
    CHECK(code_of(compile(c, "func.func @main(%a: tensor<4xf32>) -> tensor<4xf32> {\n  %0 = stablehlo.cholesky %a : tensor<4xf32>\n  return %0 : tensor<4xf32>\n}\n",
                          "mlir", &le), &msg) == PJRT_Error_Code_UNIMPLEMENTED);
    CHECK(msg.find("cholesky") != std::string::npos);
    CHECK(code_of(compile(c, kAdd, "hlo", &le)) == PJRT_Error_Code_INVALID_ARGUMENT);
    setenv("METALHLO_PYTHON", "/nonexistent/python", 1);     // no converter: bytecode is refused with a clear message
    CHECK(code_of(compile(c, std::string("ML\xEFR\x01garbage", 12), "mlir", &le), &msg) == PJRT_Error_Code_UNIMPLEMENTED);
    CHECK(msg.find("jaxlib") != std::string::npos);
    // a converter that answers: the plugin hands it the bytecode in a file (last argument) and
    // compiles the text it prints.  This stand-in checks the magic of that file and prints a
    // three-input module, so the executable below can only come from its output.
    {
        char path[] = "/tmp/pjrt_fake_converter_XXXXXX";
        const int fd = mkstemp(path);
        CHECK(fd >= 0);
        const char* script =
            "#!/bin/sh\nfor last; do :; done\n"
            "[ \"$(head -c 2 \"$last\")\" = ML ] || exit 3\n"
            "cat <<'EOT'\nmodule @from_bytecode {\n  func.func @main(%a: tensor<4xf32>, %b: tensor<4xf32>, %c: tensor<4xf32>) -> tensor<4xf32> {\n"
            "    %0 = stablehlo.add %a, %b : tensor<4xf32>\n    %1 = stablehlo.multiply %0, %c : tensor<4xf32>\n"
            "    return %1 : tensor<4xf32>\n  }\n}\nEOT\n";
        CHECK(write(fd, script, strlen(script)) == (ssize_t)strlen(script));
        close(fd);
        CHECK(chmod(path, 0700) == 0);
        setenv("METALHLO_PYTHON", path, 1);
        PJRT_LoadedExecutable* from_bc = nullptr;
        OK(compile(c, std::string("ML\xEFR\x01garbage", 12), "mlir", &from_bc));
        ARGS(PJRT_LoadedExecutable_GetExecutable_Args, g2);
        g2.loaded_executable = from_bc;
        OK(api->PJRT_LoadedExecutable_GetExecutable(&g2));
        ARGS(PJRT_Executable_OutputElementTypes_Args, ot);
        ot.executable = g2.executable;
        OK(api->PJRT_Executable_OutputElementTypes(&ot));
        CHECK(ot.num_output_types == 1 && ot.output_types[0] == PJRT_Buffer_Type_F32);
        ARGS(PJRT_Executable_Serialize_Args, se);
        se.executable = g2.executable;
        OK(api->PJRT_Executable_Serialize(&se));
        CHECK(std::string(se.serialized_bytes, se.serialized_bytes_size).find("@from_bytecode") != std::string::npos);
        se.serialized_executable_deleter(se.serialized_executable);
        ARGS(PJRT_Executable_Destroy_Args, de);
        de.executable = g2.executable;
        OK(api->PJRT_Executable_Destroy(&de));
        destroy_loaded(from_bc);
        // a converter that fails is reported like a missing one
        unlink(path);
        setenv("METALHLO_PYTHON", "/bin/false", 1);
        CHECK(code_of(compile(c, std::string("ML\xEFR\x01garbage", 12), "mlir", &from_bc), &msg) == PJRT_Error_Code_UNIMPLEMENTED);
        unsetenv("METALHLO_PYTHON");
    }
    OK(compile(c, kAdd, "mlir", &le));
    CHECK(le != nullptr);
    ARGS(PJRT_LoadedExecutable_GetExecutable_Args, ge);
    ge.loaded_executable = le;
    OK(api->PJRT_LoadedExecutable_GetExecutable(&ge));
    ARGS(PJRT_Executable_Name_Args, nm);
    nm.executable = ge.executable;
    OK(api->PJRT_Executable_Name(&nm));
    CHECK(std::string(nm.executable_name, nm.executable_name_size) == "main");
    ARGS(PJRT_Executable_NumOutputs_Args, no);
    no.executable = ge.executable;
    OK(api->PJRT_Executable_NumOutputs(&no));
    CHECK(no.num_outputs == 1);
    ARGS(PJRT_Executable_NumReplicas_Args, nr);
    nr.executable = ge.executable;
    OK(api->PJRT_Executable_NumReplicas(&nr));
    ARGS(PJRT_Executable_NumPartitions_Args, np);
    np.executable = ge.executable;
    OK(api->PJRT_Executable_NumPartitions(&np));
    CHECK(nr.num_replicas == 1 && np.num_partitions == 1);
    // memory statistics come from the plan made at compile time: two 16-byte arguments, one
    // 16-byte result, no intermediates for a single add
    ARGS(PJRT_Executable_GetCompiledMemoryStats_Args, cm);
    cm.executable = ge.executable;
    OK(api->PJRT_Executable_GetCompiledMemoryStats(&cm));
    CHECK(cm.argument_size_in_bytes == 32 && cm.output_size_in_bytes == 16 && cm.temp_size_in_bytes == 0);
    CHECK(cm.peak_memory_in_bytes == 48 && cm.generated_code_size_in_bytes == 0 && cm.host_temp_size_in_bytes == 0);
    ARGS(PJRT_Executable_OutputElementTypes_Args, ot);
    ot.executable = ge.executable;
    OK(api->PJRT_Executable_OutputElementTypes(&ot));
    CHECK(ot.num_output_types == 1 && ot.output_types[0] == PJRT_Buffer_Type_F32);
    ARGS(PJRT_Executable_OutputDimensions_Args, od);
    od.executable = ge.executable;
    OK(api->PJRT_Executable_OutputDimensions(&od));
    CHECK(od.num_outputs == 1 && od.dim_sizes[0] == 1 && od.dims[0] == 4);
    ARGS(PJRT_Executable_OutputMemoryKinds_Args, omk);
    omk.executable = ge.executable;
    OK(api->PJRT_Executable_OutputMemoryKinds(&omk));
    CHECK(omk.num_outputs == 1 && std::string(omk.memory_kinds[0], omk.memory_kind_sizes[0]) == "device");
    ARGS(PJRT_Executable_Fingerprint_Args, fp);
    fp.executable = ge.executable;
    OK(api->PJRT_Executable_Fingerprint(&fp));
    const std::string fp1(fp.executable_fingerprint, fp.executable_fingerprint_size);
    CHECK(fp1.size() == 16);
    ARGS(PJRT_LoadedExecutable_Fingerprint_Args, lfp);
    lfp.executable = le;
    OK(api->PJRT_LoadedExecutable_Fingerprint(&lfp));
    CHECK(fp1 == std::string(lfp.executable_fingerprint, lfp.executable_fingerprint_size));
    ARGS(PJRT_LoadedExecutable_GetDeviceAssignment_Args, gda);
    gda.executable = le;
    OK(api->PJRT_LoadedExecutable_GetDeviceAssignment(&gda));
    const unsigned char proto[] = {0x08, 0x01, 0x10, 0x01, 0x1A, 0x02, 0x08, 0x00};
    CHECK(gda.serialized_bytes_size == 8 && memcmp(gda.serialized_bytes, proto, 8) == 0);
    gda.serialized_device_assignment_deleter(gda.serialized_device_assignment);
    // serialize: u32 1 | u64 length | text; loading it gives the same program; damaged input is refused
    ARGS(PJRT_Executable_Serialize_Args, se);
    se.executable = ge.executable;
    OK(api->PJRT_Executable_Serialize(&se));
    const std::string bytes(se.serialized_bytes, se.serialized_bytes_size);
    se.serialized_executable_deleter(se.serialized_executable);
    uint32_t version;
    uint64_t len;
    memcpy(&version, bytes.data(), 4);
    memcpy(&len, bytes.data() + 4, 8);
    CHECK(version == 1 && len == strlen(kAdd) && bytes.size() == 12 + len && bytes.substr(12) == kAdd);
    ARGS(PJRT_Executable_DeserializeAndLoad_Args, dl);
    dl.client = c;
    dl.serialized_executable = bytes.data();
    dl.serialized_executable_size = bytes.size();
    OK(api->PJRT_Executable_DeserializeAndLoad(&dl));
    ARGS(PJRT_LoadedExecutable_Fingerprint_Args, lfp2);
    lfp2.executable = dl.loaded_executable;
    OK(api->PJRT_LoadedExecutable_Fingerprint(&lfp2));
    CHECK(fp1 == std::string(lfp2.executable_fingerprint, lfp2.executable_fingerprint_size));
    destroy_loaded(dl.loaded_executable);
    dl.serialized_executable_size = bytes.size() - 5;
    CHECK(code_of(api->PJRT_Executable_DeserializeAndLoad(&dl), &msg) == PJRT_Error_Code_INVALID_ARGUMENT && msg.find("truncated") != std::string::npos);
    dl.serialized_executable_size = 7;
    CHECK(code_of(api->PJRT_Executable_DeserializeAndLoad(&dl)) == PJRT_Error_Code_INVALID_ARGUMENT);
    std::string bad = bytes;
    bad[0] = 2;
    dl.serialized_executable = bad.data();
    dl.serialized_executable_size = bad.size();
    CHECK(code_of(api->PJRT_Executable_DeserializeAndLoad(&dl), &msg) == PJRT_Error_Code_INVALID_ARGUMENT && msg.find("version") != std::string::npos);
    // more than one device is refused before anything runs
    ARGS(PJRT_LoadedExecutable_Execute_Args, ex);
    ex.executable = le;
    ex.num_devices = 2;
    CHECK(code_of(api->PJRT_LoadedExecutable_Execute(&ex)) == PJRT_Error_Code_UNIMPLEMENTED);
    ARGS(PJRT_LoadedExecutable_Delete_Args, del);
    del.executable = le;
    OK(api->PJRT_LoadedExecutable_Delete(&del));
    ARGS(PJRT_LoadedExecutable_IsDeleted_Args, isd);
    isd.executable = le;
    OK(api->PJRT_LoadedExecutable_IsDeleted(&isd));
    CHECK(isd.is_deleted);
    ex.num_devices = 1;
    CHECK(code_of(api->PJRT_LoadedExecutable_Execute(&ex)) == PJRT_Error_Code_FAILED_PRECONDITION);
    ARGS(PJRT_Executable_Destroy_Args, de);
    de.executable = ge.executable;
    OK(api->PJRT_Executable_Destroy(&de));
    destroy_loaded(le);
    printf("ok compile\n");
}
static void case_no_device_buffers(PJRT_Client* c) {
    const float x[4] = {1, 2, 3, 4};
    const int64_t dims[1] = {4};
    ARGS(PJRT_Client_BufferFromHostBuffer_Args, b);
    b.client = c;
    b.data = x;
    b.type = PJRT_Buffer_Type_F32;
    b.dims = dims;
    b.num_dims = 1;
    CHECK(code_of(api->PJRT_Client_BufferFromHostBuffer(&b)) == PJRT_Error_Code_FAILED_PRECONDITION);
    b.type = (PJRT_Buffer_Type)14;                          // C64
    CHECK(code_of(api->PJRT_Client_BufferFromHostBuffer(&b)) == PJRT_Error_Code_INVALID_ARGUMENT);
    printf("ok no_device_buffers\n");
}

// ---- cases on the GPU ------------------------------------------------------------------------
static int callbacks = 0;
static void on_ready(PJRT_Error* e, void* user) {
    CHECK(e == nullptr && user == &callbacks);
    callbacks++;
}
static PJRT_Buffer* upload(PJRT_Client* c, const void* data, PJRT_Buffer_Type t, const std::vector<int64_t>& dims) {
    ARGS(PJRT_Client_BufferFromHostBuffer_Args, b);
    b.client = c;
    b.data = data;
    b.type = t;
    b.dims = dims.data();
    b.num_dims = dims.size();
    b.host_buffer_semantics = PJRT_HostBufferSemantics_kImmutableOnlyDuringCall;
    OK(api->PJRT_Client_BufferFromHostBuffer(&b));
    CHECK(b.buffer != nullptr && b.done_with_host_buffer != nullptr);
    ARGS(PJRT_Event_IsReady_Args, r);
    r.event = b.done_with_host_buffer;
    OK(api->PJRT_Event_IsReady(&r));
    CHECK(r.is_ready);
    destroy_event(b.done_with_host_buffer);
    return b.buffer;
}
static void download(PJRT_Buffer* b, void* dst, size_t bytes) {
    ARGS(PJRT_Buffer_ToHostBuffer_Args, q);
    q.src = b;
    OK(api->PJRT_Buffer_ToHostBuffer(&q));                 // size query
    CHECK(q.dst_size == bytes);
    ARGS(PJRT_Buffer_ToHostBuffer_Args, t);
    t.src = b;
    t.dst = dst;
    t.dst_size = bytes;
    OK(api->PJRT_Buffer_ToHostBuffer(&t));
    CHECK(t.event != nullptr);
    ARGS(PJRT_Event_Await_Args, aw);
    aw.event = t.event;
    OK(api->PJRT_Event_Await(&aw));
    destroy_event(t.event);
}
static void await_and_destroy(PJRT_Event* e) {
    CHECK(e != nullptr);
    ARGS(PJRT_Event_Await_Args, aw);
    aw.event = e;
    OK(api->PJRT_Event_Await(&aw));
    ARGS(PJRT_Event_IsReady_Args, r);
    r.event = e;
    OK(api->PJRT_Event_IsReady(&r));
    CHECK(r.is_ready);
    destroy_event(e);
}
static void case_round_trip(PJRT_Client* c) {
    const float x[6] = {1.5f, -2.f, 3.25f, 4.f, 5.f, -6.75f};
    PJRT_Buffer* b = upload(c, x, PJRT_Buffer_Type_F32, {2, 3});
    ARGS(PJRT_Buffer_ElementType_Args, et);
    et.buffer = b;
    OK(api->PJRT_Buffer_ElementType(&et));
    CHECK(et.type == PJRT_Buffer_Type_F32);
    ARGS(PJRT_Buffer_Dimensions_Args, d);
    d.buffer = b;
    OK(api->PJRT_Buffer_Dimensions(&d));
    CHECK(d.num_dims == 2 && d.dims[0] == 2 && d.dims[1] == 3);
    ARGS(PJRT_Buffer_OnDeviceSizeInBytes_Args, sz);
    sz.buffer = b;
    OK(api->PJRT_Buffer_OnDeviceSizeInBytes(&sz));
    CHECK(sz.on_device_size_in_bytes == 24);
    ARGS(PJRT_Buffer_IsOnCpu_Args, cpu);
    cpu.buffer = b;
    OK(api->PJRT_Buffer_IsOnCpu(&cpu));
    CHECK(!cpu.is_on_cpu);
    float y[6] = {0};
    download(b, y, sizeof(y));
    CHECK(memcmp(x, y, sizeof(x)) == 0);
    // too small a destination, a raw slice, a device-side copy
    ARGS(PJRT_Buffer_ToHostBuffer_Args, small);
    small.src = b;
    small.dst = y;
    small.dst_size = 8;
    CHECK(code_of(api->PJRT_Buffer_ToHostBuffer(&small)) == PJRT_Error_Code_INVALID_ARGUMENT);
    float part[2] = {0};
    ARGS(PJRT_Buffer_CopyRawToHost_Args, raw);
    raw.buffer = b;
    raw.dst = part;
    raw.offset = 8;
    raw.transfer_size = 8;
    OK(api->PJRT_Buffer_CopyRawToHost(&raw));
    await_and_destroy(raw.event);                          // the bytes are in `part` once the event completes
    CHECK(part[0] == 3.25f && part[1] == 4.f);
    raw.offset = 20;
    CHECK(code_of(api->PJRT_Buffer_CopyRawToHost(&raw)) == PJRT_Error_Code_OUT_OF_RANGE);
    ARGS(PJRT_Buffer_Device_Args, bd);
    bd.buffer = b;
    OK(api->PJRT_Buffer_Device(&bd));
    ARGS(PJRT_Buffer_CopyToDevice_Args, cp);
    cp.buffer = b;
    cp.dst_device = bd.device;
    OK(api->PJRT_Buffer_CopyToDevice(&cp));
    float z[6] = {0};
    download(cp.dst_buffer, z, sizeof(z));
    CHECK(memcmp(x, z, sizeof(x)) == 0);
    destroy_buffer(cp.dst_buffer);
    // events: ready, awaitable, callback runs once
    ARGS(PJRT_Buffer_ReadyEvent_Args, re);
    re.buffer = b;
    OK(api->PJRT_Buffer_ReadyEvent(&re));
    ARGS(PJRT_Event_OnReady_Args, orr);
    orr.event = re.event;
    orr.callback = on_ready;
    orr.user_arg = &callbacks;
    OK(api->PJRT_Event_OnReady(&orr));
    CHECK(callbacks == 1);
    ARGS(PJRT_Event_Error_Args, ee);
    ee.event = re.event;
    OK(api->PJRT_Event_Error(&ee));
    destroy_event(re.event);
    // delete releases the memory but keeps the handle
    ARGS(PJRT_Buffer_Delete_Args, del);
    del.buffer = b;
    OK(api->PJRT_Buffer_Delete(&del));
    ARGS(PJRT_Buffer_IsDeleted_Args, isd);
    isd.buffer = b;
    OK(api->PJRT_Buffer_IsDeleted(&isd));
    CHECK(isd.is_deleted);
    ARGS(PJRT_Buffer_ToHostBuffer_Args, gone);
    gone.src = b;
    gone.dst = y;
    gone.dst_size = sizeof(y);
    CHECK(code_of(api->PJRT_Buffer_ToHostBuffer(&gone)) == PJRT_Error_Code_FAILED_PRECONDITION);
    destroy_buffer(b);
    // strided host data is refused, dense strides are fine, i64 round trip
    const int64_t v[4] = {-1, 2, 1ll << 40, 7};
    const int64_t dims[2] = {2, 2}, dense[2] = {16, 8}, strided[2] = {8, 16};
    ARGS(PJRT_Client_BufferFromHostBuffer_Args, hb);
    hb.client = c;
    hb.data = v;
    hb.type = PJRT_Buffer_Type_S64;
    hb.dims = dims;
    hb.num_dims = 2;
    hb.byte_strides = strided;
    hb.num_byte_strides = 2;
    CHECK(code_of(api->PJRT_Client_BufferFromHostBuffer(&hb)) == PJRT_Error_Code_UNIMPLEMENTED);
    hb.byte_strides = dense;
    OK(api->PJRT_Client_BufferFromHostBuffer(&hb));
    destroy_event(hb.done_with_host_buffer);
    int64_t w[4] = {0};
    download(hb.buffer, w, sizeof(w));
    CHECK(memcmp(v, w, sizeof(v)) == 0);
    destroy_buffer(hb.buffer);
    ARGS(PJRT_Client_Devices_Args, ds);
    ds.client = c;
    OK(api->PJRT_Client_Devices(&ds));
    ARGS(PJRT_Device_MemoryStats_Args, ms);
    ms.device = ds.devices[0];
    OK(api->PJRT_Device_MemoryStats(&ms));
    CHECK(ms.bytes_limit_is_set && ms.bytes_limit > (1ll << 30) && ms.bytes_in_use > 0 && ms.device == ds.devices[0]);
    printf("ok round_trip\n");
}
// Transfers in flight: uploads return once the host bytes are staged (the source may change
// right away), downloads return a pending event; data is right after Await, also when the
// source buffer handle is destroyed first; OnReady callbacks registered on pending events run
// exactly once; an execution queued behind uploads that nobody awaited sees their data.
static std::atomic<int> async_callbacks{0};
static void on_async_ready(PJRT_Error* e, void* user) {
    CHECK(e == nullptr && user == &async_callbacks);
    async_callbacks++;
}
static void case_async_transfers(PJRT_Client* c) {
    const int kBuffers = 48;
    const size_t kElems = 256 * 1024;                      // 1 MiB of f32 each
    std::vector<std::vector<float>> src(kBuffers, std::vector<float>(kElems)), dst(kBuffers, std::vector<float>(kElems, -1.f));
    std::vector<PJRT_Buffer*> bufs;
    for (int i = 0; i < kBuffers; i++) {
        for (size_t j = 0; j < kElems; j++) src[i][j] = (float)(i * 1000003 % 977) + (float)(j % 4093) * 0.25f;
        bufs.push_back(upload(c, src[i].data(), PJRT_Buffer_Type_F32, {(int64_t)kElems}));
        src[i][0] = -12345.f;                               // done_with_host_buffer was complete: the upload no longer reads this
        src[i][kElems - 1] = -54321.f;
    }
    std::vector<PJRT_Event*> events;
    int pending = 0;
    for (int i = 0; i < kBuffers; i++) {
        ARGS(PJRT_Buffer_ToHostBuffer_Args, t);
        t.src = bufs[i];
        t.dst = dst[i].data();
        t.dst_size = kElems * sizeof(float);
        OK(api->PJRT_Buffer_ToHostBuffer(&t));
        CHECK(t.event != nullptr);
        ARGS(PJRT_Event_IsReady_Args, r);
        r.event = t.event;
        OK(api->PJRT_Event_IsReady(&r));
        pending += !r.is_ready;
        ARGS(PJRT_Event_OnReady_Args, cb);
        cb.event = t.event;
        cb.callback = on_async_ready;
        cb.user_arg = &async_callbacks;
        OK(api->PJRT_Event_OnReady(&cb));
        events.push_back(t.event);
        if (i % 2 == 0) { destroy_buffer(bufs[i]); bufs[i] = nullptr; }   // the copy in flight keeps the memory
    }
    for (auto e : events) await_and_destroy(e);
    for (int spin = 0; spin < 5000 && async_callbacks.load() < kBuffers; spin++) usleep(1000);
    CHECK(async_callbacks.load() == kBuffers);
    for (int i = 0; i < kBuffers; i++) {
        CHECK(dst[i][0] == (float)(i * 1000003 % 977) && dst[i][kElems - 1] == (float)(i * 1000003 % 977) + (float)((kElems - 1) % 4093) * 0.25f);
        for (size_t j = 1; j + 1 < kElems; j++) CHECK(dst[i][j] == src[i][j]);
    }
    printf("  %d of %d downloads were still pending when ToHostBuffer returned\n", pending, kBuffers);
    for (auto b : bufs) if (b) destroy_buffer(b);
    // ReadyEvent of a large upload: awaitable, ready afterwards; raw slices of it
    const size_t big = 16u << 20;                           // 64 MiB
    std::vector<float> host(big);
    for (size_t j = 0; j < big; j++) host[j] = (float)(j % 65521);
    PJRT_Buffer* bb = upload(c, host.data(), PJRT_Buffer_Type_F32, {(int64_t)big});
    ARGS(PJRT_Buffer_ReadyEvent_Args, re);
    re.buffer = bb;
    OK(api->PJRT_Buffer_ReadyEvent(&re));
    await_and_destroy(re.event);
    float tailv[4] = {0};
    ARGS(PJRT_Buffer_CopyRawToHost_Args, raw);
    raw.buffer = bb;
    raw.dst = tailv;
    raw.offset = (int64_t)((big - 4) * sizeof(float));
    raw.transfer_size = sizeof(tailv);
    OK(api->PJRT_Buffer_CopyRawToHost(&raw));
    await_and_destroy(raw.event);
    for (int j = 0; j < 4; j++) CHECK(tailv[j] == (float)((big - 4 + j) % 65521));
    destroy_buffer(bb);
    // an execution right behind two uploads nobody waited for
    const char* add_big =
        "module { func.func @main(%a: tensor<1048576xf32>, %b: tensor<1048576xf32>) -> (tensor<1048576xf32>) {\n"
        "  %0 = stablehlo.add %a, %b : tensor<1048576xf32>\n  return %0 : tensor<1048576xf32>\n} }\n";
    PJRT_LoadedExecutable* le = nullptr;
    OK(compile(c, add_big, "mlir", &le));
    std::vector<float> x(1048576), y(1048576), z(1048576, 0.f);
    for (size_t j = 0; j < x.size(); j++) { x[j] = (float)(j % 1021); y[j] = (float)(j % 509) * 0.5f; }
    PJRT_Buffer* in[2] = {upload(c, x.data(), PJRT_Buffer_Type_F32, {1048576}), upload(c, y.data(), PJRT_Buffer_Type_F32, {1048576})};
    PJRT_Buffer* const* lists[1] = {in};
    PJRT_Buffer* out[1] = {nullptr};
    PJRT_Buffer** out_lists[1] = {out};
    PJRT_Event* done[1] = {nullptr};
    ARGS(PJRT_ExecuteOptions, opts);
    ARGS(PJRT_LoadedExecutable_Execute_Args, ex);
    ex.executable = le;
    ex.options = &opts;
    ex.argument_lists = lists;
    ex.num_devices = 1;
    ex.num_args = 2;
    ex.output_lists = out_lists;
    ex.device_complete_events = done;
    OK(api->PJRT_LoadedExecutable_Execute(&ex));
    await_and_destroy(done[0]);
    download(out[0], z.data(), z.size() * sizeof(float));
    for (size_t j = 0; j < z.size(); j++) CHECK(z[j] == x[j] + y[j]);
    destroy_buffer(out[0]);
    destroy_buffer(in[0]);
    destroy_buffer(in[1]);
    destroy_loaded(le);
    printf("ok async_transfers\n");
}

static std::vector<float> run1(PJRT_LoadedExecutable* le, std::vector<PJRT_Buffer*> in, size_t n_out) {
    PJRT_Buffer* const* lists[1] = {in.data()};
    PJRT_Buffer* outs[1] = {nullptr};
    PJRT_Buffer** out_lists[1] = {outs};
    PJRT_Event* done[1] = {nullptr};
    ARGS(PJRT_ExecuteOptions, opt);
    ARGS(PJRT_LoadedExecutable_Execute_Args, ex);
    ex.executable = le;
    ex.options = &opt;
    ex.argument_lists = lists;
    ex.num_devices = 1;
    ex.num_args = in.size();
    ex.output_lists = out_lists;
    ex.device_complete_events = done;
    OK(api->PJRT_LoadedExecutable_Execute(&ex));
    CHECK(outs[0] != nullptr && done[0] != nullptr);
    ARGS(PJRT_Event_IsReady_Args, r);
    r.event = done[0];
    OK(api->PJRT_Event_IsReady(&r));
    CHECK(r.is_ready);
    destroy_event(done[0]);
    std::vector<float> y(n_out);
    download(outs[0], y.data(), n_out * sizeof(float));
    destroy_buffer(outs[0]);
    return y;
}
static void case_execute(PJRT_Client* c) {
    PJRT_LoadedExecutable* le = nullptr;
    OK(compile(c, kAdd, "mlir", &le));
    const float a[4] = {1, 2, 3, 4}, b[4] = {10, 20, 30, 40};
    PJRT_Buffer* ba = upload(c, a, PJRT_Buffer_Type_F32, {4});
    PJRT_Buffer* bb = upload(c, b, PJRT_Buffer_Type_F32, {4});
    std::vector<float> y = run1(le, {ba, bb}, 4);
    CHECK(y[0] == 11 && y[1] == 22 && y[2] == 33 && y[3] == 44);
    // wrong argument count / shape -> INVALID_ARGUMENT, nothing crashes
    {
        PJRT_Buffer* one[1] = {ba};
        PJRT_Buffer* const* lists[1] = {one};
        PJRT_Buffer* outs[1] = {nullptr};
        PJRT_Buffer** out_lists[1] = {outs};
        ARGS(PJRT_LoadedExecutable_Execute_Args, ex);
        ex.executable = le;
        ex.argument_lists = lists;
        ex.num_devices = 1;
        ex.num_args = 1;
        ex.output_lists = out_lists;
        CHECK(code_of(api->PJRT_LoadedExecutable_Execute(&ex)) == PJRT_Error_Code_INVALID_ARGUMENT);
    }
    // serialize -> deserialize -> execute gives the same numbers
    ARGS(PJRT_LoadedExecutable_GetExecutable_Args, ge);
    ge.loaded_executable = le;
    OK(api->PJRT_LoadedExecutable_GetExecutable(&ge));
    ARGS(PJRT_Executable_Serialize_Args, se);
    se.executable = ge.executable;
    OK(api->PJRT_Executable_Serialize(&se));
    ARGS(PJRT_Executable_DeserializeAndLoad_Args, dl);
    dl.client = c;
    dl.serialized_executable = se.serialized_bytes;
    dl.serialized_executable_size = se.serialized_bytes_size;
    OK(api->PJRT_Executable_DeserializeAndLoad(&dl));
    se.serialized_executable_deleter(se.serialized_executable);
    std::vector<float> y2 = run1(dl.loaded_executable, {ba, bb}, 4);
    CHECK(y2 == y);
    destroy_loaded(dl.loaded_executable);
    ARGS(PJRT_Executable_Destroy_Args, de);
    de.executable = ge.executable;
    OK(api->PJRT_Executable_Destroy(&de));
    destroy_loaded(le);
    destroy_buffer(ba);
    destroy_buffer(bb);
    // a fused kernel through the plugin: softmax rows [1,2,3,4] and [1,1,1,1]
    OK(compile(c, kSoftmax, "mlir", &le));
    const float x[8] = {1, 2, 3, 4, 1, 1, 1, 1};
    PJRT_Buffer* bx = upload(c, x, PJRT_Buffer_Type_F32, {2, 4});
    std::vector<float> s = run1(le, {bx}, 8);
    const double z = exp(1.0) + exp(2.0) + exp(3.0) + exp(4.0);
    for (int i = 0; i < 4; i++) {
        CHECK(fabs(s[i] - exp(1.0 + i) / z) < 1e-6);
        CHECK(fabs(s[4 + i] - 0.25) < 1e-6);
    }
    destroy_buffer(bx);
    destroy_loaded(le);
    printf("ok execute\n");
}

// Executions that are replayed as a HIP graph (METALHLO_HIP_GRAPH=1: the second execution captures the
// client's stream, later ones replay) while a second thread keeps uploading and downloading on
// the same client: a capture holds the stream lock that every transfer takes, so no transfer is
// recorded into a graph or left without its completion event.  Every result of both threads is
// checked.  Without graph replay the case is the same traffic on the eager path.
static void case_execute_while_transferring(PJRT_Client* c) {
    std::string prog = "func.func @main(%x: tensor<256xf32>) -> tensor<256xf32> {\n  %c = stablehlo.constant dense<1.0> : tensor<256xf32>\n";
    std::string cur = "%x";
    for (int i = 0; i < 24; i++) {           // a chain long enough for the replay threshold
        prog += "  %v" + std::to_string(i) + " = stablehlo.add " + cur + ", %c : tensor<256xf32>\n";
        cur = "%v" + std::to_string(i);
    }
    prog += "  return " + cur + " : tensor<256xf32>\n}\n";
    PJRT_LoadedExecutable* le = nullptr;
    OK(compile(c, prog, "mlir", &le));
    std::atomic<bool> stop{false};
    std::atomic<int> round_trips{0};
    std::thread mover([&] {
        std::vector<float> src(4096), dst(4096);
        for (int it = 0; !stop.load(); it++) {
            for (size_t i = 0; i < src.size(); i++) src[i] = (float)(it * 7 + (int)i);
            PJRT_Buffer* b = upload(c, src.data(), PJRT_Buffer_Type_F32, {4096});
            download(b, dst.data(), dst.size() * sizeof(float));
            destroy_buffer(b);
            CHECK(dst == src);
            round_trips++;
        }
    });
    std::vector<float> x(256);
    for (int it = 0; it < 40; it++) {
        for (int i = 0; i < 256; i++) x[i] = (float)(it + i);
        PJRT_Buffer* bx = upload(c, x.data(), PJRT_Buffer_Type_F32, {256});
        std::vector<float> y = run1(le, {bx}, 256);
        for (int i = 0; i < 256; i++) CHECK(y[i] == x[i] + 24.f);
        destroy_buffer(bx);
    }
    while (round_trips.load() < 8) usleep(1000);
    stop = true;
    mover.join();
    destroy_loaded(le);
    printf("ok execute_while_transferring\n");
}

// Two programs executed from two threads on ONE client with graph replay on: while one thread's
// second execution captures the client's stream, the other thread's launches must not be recorded
// into that graph (they would never run and its results would be stale).  Every enqueue of an
// execution happens under the client's stream lock; each thread checks every result, with inputs
// that change from one execution to the next so that a launch that did not run is seen.
static void case_two_programs_two_threads(PJRT_Client* c) {
    auto chain = [](int n, const char* op, const char* cst) {
        std::string prog = std::string("func.func @main(%x: tensor<512xf32>) -> tensor<512xf32> {\n  %c = stablehlo.constant dense<") + cst + "> : tensor<512xf32>\n";
        std::string cur = "%x";
        for (int i = 0; i < n; i++) {
            prog += "  %v" + std::to_string(i) + " = stablehlo." + op + " " + cur + ", %c : tensor<512xf32>\n";
            cur = "%v" + std::to_string(i);
        }
        return prog + "  return " + cur + " : tensor<512xf32>\n}\n";
    };
    PJRT_LoadedExecutable *la = nullptr, *lb = nullptr;
    OK(compile(c, chain(24, "add", "1.0"), "mlir", &la));
    OK(compile(c, chain(20, "subtract", "2.0"), "mlir", &lb));
    std::atomic<int> failures{0};
    auto worker = [&](PJRT_LoadedExecutable* le, float delta, int seed) {
        std::vector<float> x(512);
        for (int it = 0; it < 30; it++) {
            for (int i = 0; i < 512; i++) x[i] = (float)(seed + 3 * it + i);
            // a fresh input buffer every other execution: new addresses force new captures while
            // the other thread is launching
            PJRT_Buffer* bx = upload(c, x.data(), PJRT_Buffer_Type_F32, {512});
            for (int rep = 0; rep < 2; rep++) {
                std::vector<float> y = run1(le, {bx}, 512);
                for (int i = 0; i < 512; i++)
                    if (y[i] != x[i] + delta) failures++;
            }
            destroy_buffer(bx);
        }
    };
    std::thread ta(worker, la, 24.f, 1), tb(worker, lb, -40.f, 1000);
    ta.join();
    tb.join();
    CHECK(failures.load() == 0);
    destroy_loaded(la);
    destroy_loaded(lb);
    printf("ok two_programs_two_threads\n");
}

// A crash inside the plugin names its call chain (module + offset per frame) before the process ends.
static void on_crash(int sig) {
    void* frames[48];
    const int n = backtrace(frames, 48);
    const char msg[] = "FAIL: fatal signal, call chain:\n";
    (void)!write(1, msg, sizeof msg - 1);
    backtrace_symbols_fd(frames, n, 1);
    signal(sig, SIG_DFL);
    raise(sig);
}

int main(int argc, char** argv) {
    signal(SIGSEGV, on_crash);
    signal(SIGABRT, on_crash);
    setvbuf(stdout, nullptr, _IONBF, 0);       // every "ok" line reaches a pipe even when a later case crashes
    if (argc < 3) { printf("usage: pjrt_driver <plugin.so> host|gpu\n"); return 2; }
    void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
    if (!lib) { printf("FAIL dlopen: %s\n", dlerror()); return 1; }
    get_api = (GetApi)dlsym(lib, "GetPjrtApi");
    if (!get_api) { printf("FAIL GetPjrtApi is not exported\n"); return 1; }
    api = get_api();
    CHECK(api != nullptr);
    const bool gpu = strcmp(argv[2], "gpu") == 0;
    if (!gpu) setenv("METALHLO_ALLOW_NO_DEVICE", "1", 1);
    case_table();
    PJRT_Client* c = make_client();
    case_errors(c);
    case_platform(c);
    case_compile(c);
    if (gpu) {
        case_round_trip(c);
        case_execute(c);
        case_async_transfers(c);
        case_execute_while_transferring(c);
        case_two_programs_two_threads(c);
    } else {
        case_no_device_buffers(c);
    }
    destroy_client(c);
    printf("ok all\n");
    return 0;
}
