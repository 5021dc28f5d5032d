"""ctypes driver for a PJRT plugin shared library.

Walks the same C-API call sequence jaxlib's PJRT client walks
(`GetPjrtApi` -> `PJRT_Plugin_Initialize` -> `PJRT_Client_Create` ->
`PJRT_Client_BufferFromHostBuffer` -> `PJRT_Client_Compile` ->
`PJRT_LoadedExecutable_Execute` -> `PJRT_Buffer_ToHostBuffer`) and offers the small
slice of `xla_client`'s Python surface that the reference's raw-client test uses
(reference: tests/test_ops.py:260-281: `client.compile_and_load(text, devices)`,
`client.buffer_from_pyval(x)`, `exe.execute([buf])`).  Struct layouts mirror
include/pjrt_c_api.h.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import List, Optional, Sequence

import numpy as np

_P = C.c_void_p
_SZ = C.c_size_t


def _args(name, fields):
    return type(name, (C.Structure,), {"_fields_": [("struct_size", _SZ), ("extension_start", _P)] + fields})


# ---- argument structs (field order as in include/pjrt_c_api.h) ---------------------------------
Error_Destroy_Args = _args("Error_Destroy_Args", [("error", _P)])
Error_Message_Args = _args("Error_Message_Args", [("error", _P), ("message", C.c_char_p), ("message_size", _SZ)])
Error_GetCode_Args = _args("Error_GetCode_Args", [("error", _P), ("code", C.c_int)])
Plugin_Initialize_Args = _args("Plugin_Initialize_Args", [])
Event_Args = _args("Event_Args", [("event", _P)])
Event_IsReady_Args = _args("Event_IsReady_Args", [("event", _P), ("is_ready", C.c_bool)])
Event_Error_Args = _args("Event_Error_Args", [("event", _P)])
OnReadyCallback = C.CFUNCTYPE(None, _P, _P)      # void (*)(PJRT_Error* error, void* user_arg); the callback owns the error
Event_OnReady_Args = _args("Event_OnReady_Args", [("event", _P), ("callback", OnReadyCallback), ("user_arg", _P)])
Buffer_CopyToDevice_Args = _args("Buffer_CopyToDevice_Args", [("buffer", _P), ("dst_device", _P), ("dst_buffer", _P)])
LoadedExecutable_GetDeviceAssignment_Args = _args("LoadedExecutable_GetDeviceAssignment_Args", [
    ("executable", _P), ("serialized_bytes", _P), ("serialized_bytes_size", _SZ), ("serialized_device_assignment", _P),
    ("serialized_device_assignment_deleter", C.CFUNCTYPE(None, _P))])
Plugin_Attributes_Args = _args("Plugin_Attributes_Args", [("attributes", _P), ("num_attributes", _SZ)])
Client_Create_Args = _args("Client_Create_Args", [
    ("create_options", _P), ("num_options", _SZ), ("kv_get_callback", _P), ("kv_get_user_arg", _P),
    ("kv_put_callback", _P), ("kv_put_user_arg", _P), ("client", _P), ("kv_try_get_callback", _P),
    ("kv_try_get_user_arg", _P)])
Client_Str_Args = _args("Client_Str_Args", [("client", _P), ("value", C.c_char_p), ("value_size", _SZ)])
Client_Devices_Args = _args("Client_Devices_Args", [("client", _P), ("devices", C.POINTER(_P)), ("num_devices", _SZ)])


class Program(C.Structure):
    _fields_ = [("struct_size", _SZ), ("extension_start", _P), ("code", C.c_char_p), ("code_size", _SZ),
                ("format", C.c_char_p), ("format_size", _SZ)]


Client_Compile_Args = _args("Client_Compile_Args", [
    ("client", _P), ("program", C.POINTER(Program)), ("compile_options", C.c_char_p), ("compile_options_size", _SZ),
    ("executable", _P)])
Executable_Serialize_Args = _args("Executable_Serialize_Args", [
    ("executable", _P), ("serialized_bytes", _P), ("serialized_bytes_size", _SZ), ("serialized_executable", _P),
    ("serialized_executable_deleter", C.CFUNCTYPE(None, _P))])
Executable_DeserializeAndLoad_Args = _args("Executable_DeserializeAndLoad_Args", [
    ("client", _P), ("serialized_executable", C.c_char_p), ("serialized_executable_size", _SZ), ("loaded_executable", _P),
    ("overridden_serialized_compile_options", C.c_char_p), ("overridden_serialized_compile_options_size", _SZ)])
BufferFromHostBuffer_Args = _args("BufferFromHostBuffer_Args", [
    ("client", _P), ("data", _P), ("type", C.c_int), ("dims", C.POINTER(C.c_int64)), ("num_dims", _SZ),
    ("byte_strides", C.POINTER(C.c_int64)), ("num_byte_strides", _SZ), ("host_buffer_semantics", C.c_int),
    ("device", _P), ("memory", _P), ("device_layout", _P), ("done_with_host_buffer", _P), ("buffer", _P)])
Device_GetDescription_Args = _args("Device_GetDescription_Args", [("device", _P), ("device_description", _P)])
DeviceDescription_Str_Args = _args("DeviceDescription_Str_Args", [("device_description", _P), ("value", C.c_char_p), ("value_size", _SZ)])
Device_MemoryStats_Args = _args("Device_MemoryStats_Args", [
    ("device", _P), ("bytes_in_use", C.c_int64),
    ("peak_bytes_in_use", C.c_int64), ("peak_bytes_in_use_is_set", C.c_bool),
    ("num_allocs", C.c_int64), ("num_allocs_is_set", C.c_bool),
    ("largest_alloc_size", C.c_int64), ("largest_alloc_size_is_set", C.c_bool),
    ("bytes_limit", C.c_int64), ("bytes_limit_is_set", C.c_bool),
    ("bytes_reserved", C.c_int64), ("bytes_reserved_is_set", C.c_bool),
    ("peak_bytes_reserved", C.c_int64), ("peak_bytes_reserved_is_set", C.c_bool),
    ("bytes_reservable_limit", C.c_int64), ("bytes_reservable_limit_is_set", C.c_bool),
    ("largest_free_block_bytes", C.c_int64), ("largest_free_block_bytes_is_set", C.c_bool),
    ("pool_bytes", C.c_int64), ("pool_bytes_is_set", C.c_bool),
    ("peak_pool_bytes", C.c_int64), ("peak_pool_bytes_is_set", C.c_bool)])
LoadedExecutable_Args = _args("LoadedExecutable_Args", [("executable", _P)])
LoadedExecutable_GetExecutable_Args = _args("LoadedExecutable_GetExecutable_Args", [("loaded_executable", _P), ("executable", _P)])
Executable_NumOutputs_Args = _args("Executable_NumOutputs_Args", [("executable", _P), ("num_outputs", _SZ)])
Executable_OutputElementTypes_Args = _args("Executable_OutputElementTypes_Args", [("executable", _P), ("output_types", C.POINTER(C.c_int)), ("num_output_types", _SZ)])
Executable_OutputDimensions_Args = _args("Executable_OutputDimensions_Args", [("executable", _P), ("num_outputs", _SZ), ("dims", C.POINTER(C.c_int64)), ("dim_sizes", C.POINTER(_SZ))])


class NamedValue(C.Structure):
    class _U(C.Union):
        _fields_ = [("string_value", C.c_char_p), ("int64_value", C.c_int64), ("int64_array_value", _P),
                    ("float_value", C.c_float), ("bool_value", C.c_bool)]
    _anonymous_ = ("u",)
    _fields_ = [("struct_size", _SZ), ("extension_start", _P), ("name", C.c_char_p), ("name_size", _SZ),
                ("type", C.c_int), ("u", _U), ("value_size", _SZ)]


Executable_GetCostAnalysis_Args = _args("Executable_GetCostAnalysis_Args", [("executable", _P), ("num_properties", _SZ), ("properties", C.POINTER(NamedValue))])


class ExecuteOptions(C.Structure):
    _fields_ = [("struct_size", _SZ), ("extension_start", _P), ("send_callbacks", _P), ("recv_callbacks", _P),
                ("num_send_ops", _SZ), ("num_recv_ops", _SZ), ("launch_id", C.c_int),
                ("non_donatable_input_indices", _P), ("num_non_donatable_input_indices", _SZ), ("context", _P)]


Execute_Args = _args("Execute_Args", [
    ("executable", _P), ("options", C.POINTER(ExecuteOptions)), ("argument_lists", C.POINTER(C.POINTER(_P))),
    ("num_devices", _SZ), ("num_args", _SZ), ("output_lists", C.POINTER(C.POINTER(_P))),
    ("device_complete_events", C.POINTER(_P)), ("execute_device", _P)])
Buffer_Args = _args("Buffer_Args", [("buffer", _P)])
Buffer_ElementType_Args = _args("Buffer_ElementType_Args", [("buffer", _P), ("type", C.c_int)])
Buffer_Dimensions_Args = _args("Buffer_Dimensions_Args", [("buffer", _P), ("dims", C.POINTER(C.c_int64)), ("num_dims", _SZ)])
Buffer_ToHostBuffer_Args = _args("Buffer_ToHostBuffer_Args", [("src", _P), ("host_layout", _P), ("dst", _P), ("dst_size", _SZ), ("event", _P)])
Buffer_ReadyEvent_Args = _args("Buffer_ReadyEvent_Args", [("buffer", _P), ("event", _P)])
Buffer_OpaqueDeviceMemoryDataPointer_Args = _args("Buffer_OpaqueDeviceMemoryDataPointer_Args", [("buffer", _P), ("device_memory_ptr", _P)])
Buffer_IsDeleted_Args = _args("Buffer_IsDeleted_Args", [("buffer", _P), ("is_deleted", C.c_bool)])


class ApiVersion(C.Structure):
    _fields_ = [("struct_size", _SZ), ("extension_start", _P), ("major_version", C.c_int), ("minor_version", C.c_int)]


# function-table entries in declaration order (include/pjrt_c_api.h, struct PJRT_Api)
API_ENTRIES = [
    "PJRT_Error_Destroy", "PJRT_Error_Message", "PJRT_Error_GetCode", "PJRT_Plugin_Initialize", "PJRT_Plugin_Attributes",
    "PJRT_Event_Destroy", "PJRT_Event_IsReady", "PJRT_Event_Error", "PJRT_Event_Await", "PJRT_Event_OnReady",
    "PJRT_Client_Create", "PJRT_Client_Destroy", "PJRT_Client_PlatformName", "PJRT_Client_ProcessIndex",
    "PJRT_Client_PlatformVersion", "PJRT_Client_Devices", "PJRT_Client_AddressableDevices", "PJRT_Client_LookupDevice",
    "PJRT_Client_LookupAddressableDevice", "PJRT_Client_AddressableMemories", "PJRT_Client_Compile",
    "PJRT_Client_DefaultDeviceAssignment", "PJRT_Client_BufferFromHostBuffer",
    "PJRT_DeviceDescription_Id", "PJRT_DeviceDescription_ProcessIndex", "PJRT_DeviceDescription_Attributes",
    "PJRT_DeviceDescription_Kind", "PJRT_DeviceDescription_DebugString", "PJRT_DeviceDescription_ToString",
    "PJRT_Device_GetDescription", "PJRT_Device_IsAddressable", "PJRT_Device_LocalHardwareId",
    "PJRT_Device_AddressableMemories", "PJRT_Device_DefaultMemory", "PJRT_Device_MemoryStats",
    "PJRT_Memory_Id", "PJRT_Memory_Kind", "PJRT_Memory_DebugString", "PJRT_Memory_ToString", "PJRT_Memory_AddressableByDevices",
    "PJRT_Executable_Destroy", "PJRT_Executable_Name", "PJRT_Executable_NumReplicas", "PJRT_Executable_NumPartitions",
    "PJRT_Executable_NumOutputs", "PJRT_Executable_SizeOfGeneratedCodeInBytes", "PJRT_Executable_GetCostAnalysis",
    "PJRT_Executable_OutputMemoryKinds", "PJRT_Executable_OptimizedProgram", "PJRT_Executable_Serialize",
    "PJRT_LoadedExecutable_Destroy", "PJRT_LoadedExecutable_GetExecutable", "PJRT_LoadedExecutable_AddressableDevices",
    "PJRT_LoadedExecutable_Delete", "PJRT_LoadedExecutable_IsDeleted", "PJRT_LoadedExecutable_Execute",
    "PJRT_Executable_DeserializeAndLoad", "PJRT_LoadedExecutable_Fingerprint",
    "PJRT_Buffer_Destroy", "PJRT_Buffer_ElementType", "PJRT_Buffer_Dimensions", "PJRT_Buffer_UnpaddedDimensions",
    "PJRT_Buffer_DynamicDimensionIndices", "PJRT_Buffer_GetMemoryLayout", "PJRT_Buffer_OnDeviceSizeInBytes",
    "PJRT_Buffer_Device", "PJRT_Buffer_Memory", "PJRT_Buffer_Delete", "PJRT_Buffer_IsDeleted", "PJRT_Buffer_CopyToDevice",
    "PJRT_Buffer_ToHostBuffer", "PJRT_Buffer_IsOnCpu", "PJRT_Buffer_ReadyEvent", "PJRT_Buffer_UnsafePointer",
    "PJRT_Buffer_IncreaseExternalReferenceCount", "PJRT_Buffer_DecreaseExternalReferenceCount",
    "PJRT_Buffer_OpaqueDeviceMemoryDataPointer",
    "PJRT_CopyToDeviceStream_Destroy", "PJRT_CopyToDeviceStream_AddChunk", "PJRT_CopyToDeviceStream_TotalBytes",
    "PJRT_CopyToDeviceStream_GranuleSize", "PJRT_CopyToDeviceStream_CurrentBytes",
    "PJRT_TopologyDescription_Create", "PJRT_TopologyDescription_Destroy", "PJRT_TopologyDescription_PlatformName",
    "PJRT_TopologyDescription_PlatformVersion", "PJRT_TopologyDescription_GetDeviceDescriptions",
    "PJRT_TopologyDescription_Serialize", "PJRT_TopologyDescription_Attributes", "PJRT_Compile",
    "PJRT_Executable_OutputElementTypes", "PJRT_Executable_OutputDimensions", "PJRT_Buffer_CopyToMemory",
    "PJRT_Client_CreateViewOfDeviceBuffer", "PJRT_Executable_Fingerprint", "PJRT_Client_TopologyDescription",
    "PJRT_Executable_GetCompiledMemoryStats", "PJRT_Memory_Kind_Id", "PJRT_ExecuteContext_Create",
    "PJRT_ExecuteContext_Destroy", "PJRT_Buffer_CopyRawToHost", "PJRT_AsyncHostToDeviceTransferManager_Destroy",
    "PJRT_AsyncHostToDeviceTransferManager_TransferData", "PJRT_Client_CreateBuffersForAsyncHostToDevice",
    "PJRT_AsyncHostToDeviceTransferManager_RetrieveBuffer", "PJRT_AsyncHostToDeviceTransferManager_Device",
    "PJRT_AsyncHostToDeviceTransferManager_BufferCount", "PJRT_AsyncHostToDeviceTransferManager_BufferSize",
    "PJRT_AsyncHostToDeviceTransferManager_SetBufferError", "PJRT_AsyncHostToDeviceTransferManager_AddMetadata",
    "PJRT_Client_DmaMap", "PJRT_Client_DmaUnmap", "PJRT_Client_CreateUninitializedBuffer",
    "PJRT_Client_UpdateGlobalProcessInfo", "PJRT_TopologyDescription_Deserialize", "PJRT_Client_CreateAliasBuffer",
    "PJRT_Client_FulfillAliasBuffer", "PJRT_LoadedExecutable_GetDeviceAssignment", "PJRT_Client_CreateErrorBuffer",
    "PJRT_AsyncHostToDeviceTransferManager_TransferLiteral", "PJRT_Buffer_CopyRawToHostFuture",
    "PJRT_Device_PoisonExecution", "PJRT_Device_CreateAsyncTrackingEvent", "PJRT_AsyncTrackingEvent_Destroy",
    "PJRT_Executable_GetCompileOptions", "PJRT_Buffer_DonateWithControlDependency", "PJRT_Event_Create", "PJRT_Event_Set",
    "PJRT_Device_GetAttributes", "PJRT_Client_Load", "PJRT_LoadedExecutable_AddressableDeviceLogicalIds",
    "PJRT_Buffer_Bitcast", "PJRT_Error_ForEachPayload", "PJRT_TopologyDescription_Fingerprint",
    "PJRT_Executable_ParameterMemoryKinds",
]

# entries the reference leaves NULL (src/pjrt_plugin/pjrt_api.cc:351-392); every other one must be set
NULL_ENTRIES = {
    "PJRT_Client_CreateViewOfDeviceBuffer", "PJRT_Memory_Kind_Id", "PJRT_ExecuteContext_Create", "PJRT_ExecuteContext_Destroy",
    "PJRT_Buffer_CopyRawToHost", "PJRT_AsyncHostToDeviceTransferManager_Destroy",
    "PJRT_AsyncHostToDeviceTransferManager_TransferData", "PJRT_Client_CreateBuffersForAsyncHostToDevice",
    "PJRT_AsyncHostToDeviceTransferManager_RetrieveBuffer", "PJRT_AsyncHostToDeviceTransferManager_Device",
    "PJRT_AsyncHostToDeviceTransferManager_BufferCount", "PJRT_AsyncHostToDeviceTransferManager_BufferSize",
    "PJRT_AsyncHostToDeviceTransferManager_SetBufferError", "PJRT_AsyncHostToDeviceTransferManager_AddMetadata",
    "PJRT_Client_DmaMap", "PJRT_Client_DmaUnmap", "PJRT_Client_CreateUninitializedBuffer", "PJRT_Client_UpdateGlobalProcessInfo",
    "PJRT_TopologyDescription_Deserialize", "PJRT_Client_CreateAliasBuffer", "PJRT_Client_FulfillAliasBuffer",
    "PJRT_Client_CreateErrorBuffer", "PJRT_AsyncHostToDeviceTransferManager_TransferLiteral", "PJRT_Buffer_CopyRawToHostFuture",
    "PJRT_Device_PoisonExecution", "PJRT_Device_CreateAsyncTrackingEvent", "PJRT_AsyncTrackingEvent_Destroy",
    "PJRT_Buffer_DonateWithControlDependency", "PJRT_Event_Create", "PJRT_Event_Set", "PJRT_Device_GetAttributes",
    "PJRT_Client_Load", "PJRT_LoadedExecutable_AddressableDeviceLogicalIds", "PJRT_Buffer_Bitcast",
    "PJRT_Executable_ParameterMemoryKinds",
}


class Api(C.Structure):
    _fields_ = [("struct_size", _SZ), ("extension_start", _P), ("pjrt_api_version", ApiVersion)] + [(n, _P) for n in API_ENTRIES]


# PJRT_Buffer_Type <-> numpy (bf16 travels as uint16 bit patterns tagged with the BF16 code)
PRED, S8, S16, S32, S64, U8, U16, U32, U64, F16, F32, F64, BF16 = range(1, 14)
_NP_TO_PJRT = {np.dtype(np.bool_): PRED, np.dtype(np.int8): S8, np.dtype(np.int16): S16, np.dtype(np.int32): S32,
               np.dtype(np.int64): S64, np.dtype(np.uint8): U8, np.dtype(np.uint16): U16, np.dtype(np.uint32): U32,
               np.dtype(np.uint64): U64, np.dtype(np.float16): F16, np.dtype(np.float32): F32, np.dtype(np.float64): F64}
_PJRT_TO_NP = {v: k for k, v in _NP_TO_PJRT.items()}
_PJRT_TO_NP[BF16] = np.dtype(np.uint16)
MLIR_TO_PJRT = {"i1": PRED, "i8": S8, "i16": S16, "i32": S32, "i64": S64, "ui8": U8, "ui16": U16, "ui32": U32, "ui64": U64,
                "f16": F16, "f32": F32, "f64": F64, "bf16": BF16}


class PjrtError(RuntimeError):
    def __init__(self, message, code):
        super().__init__(message)
        self.code = code


def default_library_path() -> str:
    env = os.environ.get("MI355X_PJRT_LIBRARY_PATH")
    if env:
        return env
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), "libpjrt_plugin_mi355x.so")


class Plugin:
    """Loaded shared library + its PJRT_Api table."""

    def __init__(self, path: Optional[str] = None):
        self.path = path or default_library_path()
        if not os.path.exists(self.path):
            raise FileNotFoundError(f"PJRT plugin library not found at {self.path}; build it with __graft_entry__.build()")
        self.lib = C.CDLL(self.path)
        self.lib.GetPjrtApi.restype = C.POINTER(Api)
        self.api = self.lib.GetPjrtApi().contents

    def fn(self, name, argtype, restype=_P):
        ptr = getattr(self.api, name)
        if not ptr:
            raise PjrtError(f"{name} is NULL in the plugin's table", 12)
        return C.CFUNCTYPE(restype, C.POINTER(argtype))(ptr)

    def call(self, name, args):
        args.struct_size = C.sizeof(args)
        err = self.fn(name, type(args))(C.byref(args))
        if err:
            self.raise_error(err)
        return args

    def raise_error(self, err):
        m = Error_Message_Args(error=err)
        m.struct_size = C.sizeof(m)
        self.fn("PJRT_Error_Message", Error_Message_Args, None)(C.byref(m))
        msg = C.string_at(m.message, m.message_size).decode("utf-8", "replace")
        g = Error_GetCode_Args(error=err)
        g.struct_size = C.sizeof(g)
        self.fn("PJRT_Error_GetCode", Error_GetCode_Args)(C.byref(g))
        d = Error_Destroy_Args(error=err)
        d.struct_size = C.sizeof(d)
        self.fn("PJRT_Error_Destroy", Error_Destroy_Args, None)(C.byref(d))
        raise PjrtError(msg, g.code)


class ScatterDesc(C.Structure):
    """mi355x_scatter_desc of include/mi355x_noalloc.h."""
    _fields_ = [("num_updates", C.c_int64), ("row_elems", C.c_int64), ("operand_rows", C.c_int64), ("kind", C.c_int),
                ("dtype", C.c_int), ("index_bytes", C.c_int)]


SCATTER_KINDS = {"add": 0, "set": 1, "mul": 2, "min": 3, "max": 4}
SCATTER_DTYPES = {"f32": 0, "bf16": 1, "i32": 2, "ui32": 3}


def scatter_rows_noalloc(plugin: Plugin, result_ptr: int, indices_ptr: int, updates_ptr: int, *, num_updates: int, row_elems: int,
                         operand_rows: int, kind: str = "add", dtype: str = "f32", index_bytes: int = 4, stream: int = 0) -> None:
    """mi355x_scatter_rows_noalloc (include/mi355x_noalloc.h): ordered row scatter into `result_ptr` in place, enqueued
    on `stream`, using the library's fixed workspace.  Raises PjrtError with the entry point's message on failure."""
    fn = plugin.lib.mi355x_scatter_rows_noalloc
    fn.restype = C.c_int
    fn.argtypes = [C.POINTER(ScatterDesc), _P, _P, _P, _P, C.c_char_p, _SZ]
    d = ScatterDesc(num_updates, row_elems, operand_rows, SCATTER_KINDS[kind], SCATTER_DTYPES[dtype], index_bytes)
    err = C.create_string_buffer(256)
    rc = fn(C.byref(d), result_ptr or None, indices_ptr or None, updates_ptr or None, stream or None, err, len(err))
    if rc != 0:
        raise PjrtError(err.value.decode("utf-8", "replace"), rc)


class Buffer:
    def __init__(self, client: "Client", handle):
        self.client = client
        self.handle = handle

    @property
    def _p(self):
        return self.client.plugin

    def dtype_code(self) -> int:
        return self._p.call("PJRT_Buffer_ElementType", Buffer_ElementType_Args(buffer=self.handle)).type

    def shape(self):
        a = self._p.call("PJRT_Buffer_Dimensions", Buffer_Dimensions_Args(buffer=self.handle))
        return tuple(a.dims[i] for i in range(a.num_dims))

    def device_pointer(self) -> int:
        """Device address of the buffer's memory (PJRT_Buffer_OpaqueDeviceMemoryDataPointer)."""
        a = self._p.call("PJRT_Buffer_OpaqueDeviceMemoryDataPointer", Buffer_OpaqueDeviceMemoryDataPointer_Args(buffer=self.handle))
        return int(a.device_memory_ptr or 0)

    def block_until_ready(self):
        a = self._p.call("PJRT_Buffer_ReadyEvent", Buffer_ReadyEvent_Args(buffer=self.handle))
        self._p.call("PJRT_Event_Await", Event_Args(event=a.event))
        self._p.call("PJRT_Event_Destroy", Event_Args(event=a.event))
        return self

    def to_numpy(self) -> np.ndarray:
        """Raw element type of the buffer; bf16 comes back as uint16 bit patterns."""
        q = self._p.call("PJRT_Buffer_ToHostBuffer", Buffer_ToHostBuffer_Args(src=self.handle, dst=None))
        out = np.empty(self.shape(), dtype=_PJRT_TO_NP[self.dtype_code()])
        assert out.nbytes == q.dst_size, (out.nbytes, q.dst_size)
        a = self._p.call("PJRT_Buffer_ToHostBuffer", Buffer_ToHostBuffer_Args(src=self.handle, dst=out.ctypes.data, dst_size=out.nbytes))
        if a.event:
            self._p.call("PJRT_Event_Await", Event_Args(event=a.event))
            self._p.call("PJRT_Event_Destroy", Event_Args(event=a.event))
        return out

    def copy_to_device(self) -> "Buffer":
        a = self._p.call("PJRT_Buffer_CopyToDevice", Buffer_CopyToDevice_Args(buffer=self.handle, dst_device=self.client.devices[0]))
        return Buffer(self.client, a.dst_buffer)

    def mark_deleted(self):
        """PJRT_Buffer_Delete: the device memory goes back to the allocator, the handle stays until destroyed."""
        self._p.call("PJRT_Buffer_Delete", Buffer_Args(buffer=self.handle))

    def is_deleted(self) -> bool:
        return bool(self._p.call("PJRT_Buffer_IsDeleted", Buffer_IsDeleted_Args(buffer=self.handle)).is_deleted)

    def delete(self):
        if self.handle:
            self._p.call("PJRT_Buffer_Destroy", Buffer_Args(buffer=self.handle))
            self.handle = None

    def __del__(self):
        try:
            self.delete()
        except Exception:
            pass


class LoadedExecutable:
    def __init__(self, client: "Client", handle):
        self.client = client
        self.handle = handle
        p = client.plugin
        self.exe = p.call("PJRT_LoadedExecutable_GetExecutable", LoadedExecutable_GetExecutable_Args(loaded_executable=handle)).executable
        self.num_outputs = p.call("PJRT_Executable_NumOutputs", Executable_NumOutputs_Args(executable=self.exe)).num_outputs

    def output_types(self):
        p = self.client.plugin
        t = p.call("PJRT_Executable_OutputElementTypes", Executable_OutputElementTypes_Args(executable=self.exe))
        d = p.call("PJRT_Executable_OutputDimensions", Executable_OutputDimensions_Args(executable=self.exe))
        out, k = [], 0
        for i in range(d.num_outputs):
            n = d.dim_sizes[i]
            out.append((tuple(d.dims[k + j] for j in range(n)), t.output_types[i]))
            k += n
        return out

    def execute(self, buffers: Sequence[Buffer], return_event: bool = False, donate: bool = False):
        """Outputs of one PJRT_LoadedExecutable_Execute; with `return_event` also the device-complete PJRT_Event
        handle, which the caller then destroys.  Unless `donate` is set every input is listed as non-donatable, so
        arguments the program marks as donated (tf.aliasing_output / jax.buffer_donor) stay valid."""
        p = self.client.plugin
        n = len(buffers)
        arg_arr = (_P * max(n, 1))(*[b.handle for b in buffers])
        arg_lists = (C.POINTER(_P) * 1)(C.cast(arg_arr, C.POINTER(_P)))
        out_arr = (_P * max(self.num_outputs, 1))()
        out_lists = (C.POINTER(_P) * 1)(C.cast(out_arr, C.POINTER(_P)))
        events = (_P * 1)()
        opts = ExecuteOptions()
        opts.struct_size = C.sizeof(opts)
        keep = (C.c_int64 * max(n, 1))(*range(n))
        if not donate:
            opts.non_donatable_input_indices = C.cast(keep, _P)
            opts.num_non_donatable_input_indices = n
        a = Execute_Args(executable=self.handle, options=C.pointer(opts), argument_lists=arg_lists, num_devices=1, num_args=n,
                         output_lists=out_lists, device_complete_events=events, execute_device=None)
        p.call("PJRT_LoadedExecutable_Execute", a)
        outs = [Buffer(self.client, out_arr[i]) for i in range(self.num_outputs)]
        if return_event:
            return outs, events[0]
        if events[0]:
            p.call("PJRT_Event_Destroy", Event_Args(event=events[0]))
        return outs

    def device_assignment_bytes(self) -> bytes:
        a = self.client.plugin.call("PJRT_LoadedExecutable_GetDeviceAssignment", LoadedExecutable_GetDeviceAssignment_Args(executable=self.handle))
        data = C.string_at(a.serialized_bytes, a.serialized_bytes_size)
        if a.serialized_device_assignment_deleter:
            a.serialized_device_assignment_deleter(a.serialized_device_assignment)
        return data

    def serialize(self) -> bytes:
        """PJRT_Executable_Serialize: bytes that `Client.deserialize_and_load` turns back into a loaded executable."""
        a = self.client.plugin.call("PJRT_Executable_Serialize", Executable_Serialize_Args(executable=self.exe))
        data = C.string_at(a.serialized_bytes, a.serialized_bytes_size)
        if a.serialized_executable_deleter:
            a.serialized_executable_deleter(a.serialized_executable)
        return data

    def cost_analysis(self) -> dict:
        a = self.client.plugin.call("PJRT_Executable_GetCostAnalysis", Executable_GetCostAnalysis_Args(executable=self.exe))
        out = {}
        for i in range(a.num_properties):
            nv = a.properties[i]
            out[C.string_at(nv.name, nv.name_size).decode()] = float(nv.float_value)
        return out

    def delete(self):
        if self.handle:
            self.client.plugin.call("PJRT_LoadedExecutable_Destroy", LoadedExecutable_Args(executable=self.handle))
            self.handle = None

    def __del__(self):
        try:
            self.delete()
        except Exception:
            pass


class Client:
    def __init__(self, plugin: Optional[Plugin] = None):
        self.plugin = plugin or Plugin()
        self.plugin.call("PJRT_Plugin_Initialize", Plugin_Initialize_Args())
        self.handle = self.plugin.call("PJRT_Client_Create", Client_Create_Args()).client
        d = self.plugin.call("PJRT_Client_AddressableDevices", Client_Devices_Args(client=self.handle))
        self.devices = [d.devices[i] for i in range(d.num_devices)]

    @property
    def platform(self) -> str:
        a = self.plugin.call("PJRT_Client_PlatformName", Client_Str_Args(client=self.handle))
        return C.string_at(a.value, a.value_size).decode()

    @property
    def platform_version(self) -> str:
        a = self.plugin.call("PJRT_Client_PlatformVersion", Client_Str_Args(client=self.handle))
        return C.string_at(a.value, a.value_size).decode()

    def device_kind(self) -> str:
        dd = self.plugin.call("PJRT_Device_GetDescription", Device_GetDescription_Args(device=self.devices[0])).device_description
        a = self.plugin.call("PJRT_DeviceDescription_Kind", DeviceDescription_Str_Args(device_description=dd))
        return C.string_at(a.value, a.value_size).decode()

    def memory_stats(self) -> dict:
        a = self.plugin.call("PJRT_Device_MemoryStats", Device_MemoryStats_Args(device=self.devices[0]))
        return {"bytes_in_use": a.bytes_in_use, "peak_bytes_in_use": a.peak_bytes_in_use, "num_allocs": a.num_allocs,
                "largest_alloc_size": a.largest_alloc_size, "bytes_limit": a.bytes_limit, "bytes_reserved": a.bytes_reserved}

    def plugin_attributes(self) -> dict:
        a = self.plugin.call("PJRT_Plugin_Attributes", Plugin_Attributes_Args())
        out = {}
        arr = C.cast(a.attributes, C.POINTER(NamedValue))
        for i in range(a.num_attributes):
            nv = arr[i]
            name = C.string_at(nv.name, nv.name_size).decode()
            if nv.type == 0:
                out[name] = C.string_at(nv.string_value, nv.value_size).decode()
            elif nv.type == 1:
                out[name] = int(nv.int64_value)
            elif nv.type == 2:
                out[name] = [C.cast(nv.int64_array_value, C.POINTER(C.c_int64))[k] for k in range(nv.value_size)]
            elif nv.type == 3:
                out[name] = float(nv.float_value)
            else:
                out[name] = bool(nv.bool_value)
        return out

    def compile_and_load(self, text, devices=None) -> LoadedExecutable:
        code = text.encode() if isinstance(text, str) else bytes(text)
        prog = Program(code=code, code_size=len(code), format=b"mlir", format_size=4)
        prog.struct_size = C.sizeof(prog)
        a = Client_Compile_Args(client=self.handle, program=C.pointer(prog), compile_options=None, compile_options_size=0)
        self.plugin.call("PJRT_Client_Compile", a)
        return LoadedExecutable(self, a.executable)

    def deserialize_and_load(self, data: bytes) -> LoadedExecutable:
        a = Executable_DeserializeAndLoad_Args(client=self.handle, serialized_executable=data, serialized_executable_size=len(data),
                                               overridden_serialized_compile_options=None, overridden_serialized_compile_options_size=0)
        self.plugin.call("PJRT_Executable_DeserializeAndLoad", a)
        return LoadedExecutable(self, a.loaded_executable)

    def buffer_from_pyval(self, x, dtype_code: Optional[int] = None) -> Buffer:
        arr = np.asarray(x)
        code = dtype_code if dtype_code is not None else _NP_TO_PJRT[arr.dtype]
        dims = (C.c_int64 * max(arr.ndim, 1))(*arr.shape)
        strides = (C.c_int64 * max(arr.ndim, 1))(*arr.strides)
        keep = arr  # keep the host array alive during the call
        a = BufferFromHostBuffer_Args(client=self.handle, data=keep.ctypes.data if keep.size else None, type=code, dims=dims,
                                      num_dims=arr.ndim, byte_strides=strides, num_byte_strides=arr.ndim,
                                      host_buffer_semantics=0, device=self.devices[0], memory=None, device_layout=None)
        self.plugin.call("PJRT_Client_BufferFromHostBuffer", a)
        if a.done_with_host_buffer:
            self.plugin.call("PJRT_Event_Await", Event_Args(event=a.done_with_host_buffer))
            self.plugin.call("PJRT_Event_Destroy", Event_Args(event=a.done_with_host_buffer))
        return Buffer(self, a.buffer)


_client: Optional[Client] = None


def get_client() -> Client:
    """Process-wide client (the plugin's client is a singleton, as in the reference)."""
    global _client
    if _client is None:
        _client = Client()
    return _client
