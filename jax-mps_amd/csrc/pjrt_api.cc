// The PJRT C API surface of the plugin: one exported symbol, GetPjrtApi, and the
// function table behind it.  Same populated / NULL entries as the reference's table
// (src/pjrt_plugin/pjrt_api.cc:232-393); same ownership rules (caller frees errors,
// events and buffers; the client is a process-wide singleton; output arrays are
// allocated by the caller).  No C++ exception crosses this boundary.
#include <condition_variable>
#include <cstring>
#include <deque>
#include <functional>
#include <mutex>
#include <thread>

#include "../../include/pjrt_c_api.h"
#include "runtime.h"

using namespace mi355;

// ------------------------------------------------------------ opaque types
struct PJRT_Error {
  std::string message;
  PJRT_Error_Code code;
};

struct PJRT_DeviceDescription {
  int id = 0;
  std::string kind = "MI355X";
  std::string debug = "MI355X:0";
  std::string str = "Mi355xDevice(id=0)";
};
struct PJRT_Memory {
  int id = 0;
  std::string kind = "device";
  std::string debug = "MI355X_HBM:0";
  PJRT_Device* device = nullptr;
};
struct PJRT_Device {
  PJRT_DeviceDescription desc;
  PJRT_Memory* memory = nullptr;
  PJRT_Client* client = nullptr;
};
struct PJRT_TopologyDescription {
  PJRT_DeviceDescription* desc = nullptr;
};
struct PJRT_Client {
  PJRT_Device device;
  PJRT_Memory memory;
  PJRT_TopologyDescription topology;
  PJRT_Device* devices[1];
  PJRT_Memory* memories[1];
  PJRT_DeviceDescription* descs[1];
  std::string platformVersion;
};

struct PJRT_Event {
  mi355_event_t ev = nullptr;   // null: already complete
  std::string error;
  ~PJRT_Event() { if (ev) mi355_event_destroy(ev); }
};

struct PJRT_Buffer {
  std::shared_ptr<DeviceBuffer> buf;
  PJRT_Client* client = nullptr;
  std::vector<int64_t> dims;
};

struct PJRT_Executable {
  std::shared_ptr<Executable> exe;
  std::vector<PJRT_Buffer_Type> outTypes;
  std::vector<int64_t> outDims;
  std::vector<size_t> outDimSizes;
  std::vector<const char*> outMemKinds;
  std::vector<size_t> outMemKindSizes;
  std::vector<PJRT_NamedValue> cost;
  std::vector<std::string> costNames;
  std::string fingerprint;
  std::string source;            // program text as compiled (what Serialize hands out)
  bool ownedByLoaded = false;
};
struct PJRT_SerializedExecutable {
  std::string bytes;
};
struct PJRT_LoadedExecutable {
  PJRT_Executable* executable = nullptr;
  PJRT_Client* client = nullptr;
  bool deleted = false;
};

namespace {

constexpr const char* kPlatformName = "mi355x";
constexpr const char* kPlatformVersion = "0.1.0";
constexpr const char* kExecutableName = "mi355x_executable";

// One lock for everything that touches device state (reference: pjrt_mutex.h:11-14).
std::recursive_mutex& apiMutex() {
  static std::recursive_mutex m;
  return m;
}

PJRT_Error* makeError(const std::string& msg, PJRT_Error_Code code = PJRT_Error_Code_INTERNAL) {
  return new PJRT_Error{msg, code};
}
PJRT_Error* unimplemented(const char* what) {
  return makeError(std::string(what) + " is not implemented by the MI355X plugin", PJRT_Error_Code_UNIMPLEMENTED);
}

template <typename F>
PJRT_Error* guard(F&& f) {
  try {
    return f();
  } catch (const CompileError& e) {
    return makeError(e.what(), PJRT_Error_Code_INVALID_ARGUMENT);
  } catch (const std::exception& e) {
    return makeError(e.what(), PJRT_Error_Code_INTERNAL);
  } catch (...) {
    return makeError("unknown C++ exception", PJRT_Error_Code_INTERNAL);
  }
}

// dtype maps (reference: mlx_buffer.cc:14-87, type_utils.cc:5-41).  F64 and complex are rejected.
DType fromPjrt(PJRT_Buffer_Type t) {
  switch (t) {
    case PJRT_Buffer_Type_PRED: return DType::Pred;
    case PJRT_Buffer_Type_S8: return DType::S8;
    case PJRT_Buffer_Type_S16: return DType::S16;
    case PJRT_Buffer_Type_S32: return DType::S32;
    case PJRT_Buffer_Type_S64: return DType::S64;
    case PJRT_Buffer_Type_U8: return DType::U8;
    case PJRT_Buffer_Type_U16: return DType::U16;
    case PJRT_Buffer_Type_U32: return DType::U32;
    case PJRT_Buffer_Type_U64: return DType::U64;
    case PJRT_Buffer_Type_F16: return DType::F16;
    case PJRT_Buffer_Type_F32: return DType::F32;
    case PJRT_Buffer_Type_BF16: return DType::BF16;
    default: return DType::Invalid;
  }
}
PJRT_Buffer_Type toPjrt(DType d) {
  switch (d) {
    case DType::Pred: return PJRT_Buffer_Type_PRED;
    case DType::S8: return PJRT_Buffer_Type_S8;
    case DType::S16: return PJRT_Buffer_Type_S16;
    case DType::S32: return PJRT_Buffer_Type_S32;
    case DType::S64: return PJRT_Buffer_Type_S64;
    case DType::U8: return PJRT_Buffer_Type_U8;
    case DType::U16: return PJRT_Buffer_Type_U16;
    case DType::U32: return PJRT_Buffer_Type_U32;
    case DType::U64: return PJRT_Buffer_Type_U64;
    case DType::F16: return PJRT_Buffer_Type_F16;
    case DType::F32: return PJRT_Buffer_Type_F32;
    case DType::F64: return PJRT_Buffer_Type_F64;
    case DType::BF16: return PJRT_Buffer_Type_BF16;
    case DType::Token: return PJRT_Buffer_Type_TOKEN;
    default: return PJRT_Buffer_Type_INVALID;
  }
}

PJRT_Event* readyEvent() { return new PJRT_Event(); }
PJRT_Event* streamEvent() {
  auto* e = new PJRT_Event();
  if (mi355_event_create(&e->ev, 0) != 0 || mi355_event_record(e->ev, Device::get().stream()) != 0) {
    e->error = mi355_last_error();
  }
  return e;
}

// Fires OnReady callbacks in FIFO order on one background thread (reference: pjrt_event.cc:28-78).
class CompletionService {
 public:
  static CompletionService& get() {
    static CompletionService* s = new CompletionService();
    return *s;
  }
  void post(std::function<void()> fn) {
    {
      std::lock_guard<std::mutex> lk(mu_);
      q_.push_back(std::move(fn));
    }
    cv_.notify_one();
  }

 private:
  CompletionService() {
    std::thread([this] {
      while (true) {
        std::function<void()> fn;
        {
          std::unique_lock<std::mutex> lk(mu_);
          cv_.wait(lk, [this] { return !q_.empty(); });
          fn = std::move(q_.front());
          q_.pop_front();
        }
        fn();
      }
    }).detach();
  }
  std::mutex mu_;
  std::condition_variable cv_;
  std::deque<std::function<void()>> q_;
};

PJRT_Client* theClient() {
  static PJRT_Client* c = nullptr;
  static std::once_flag once;
  static std::string error;
  std::call_once(once, [] {
    try {
      Device& dev = Device::get();
      auto* cl = new PJRT_Client();
      cl->device.client = cl;
      cl->device.memory = &cl->memory;
      cl->memory.device = &cl->device;
      cl->topology.desc = &cl->device.desc;
      cl->devices[0] = &cl->device;
      cl->memories[0] = &cl->memory;
      cl->descs[0] = &cl->device.desc;
      cl->platformVersion = std::string(kPlatformVersion) + " (" + dev.name() + ", " + dev.arch() + ")";
      c = cl;
    } catch (const std::exception& e) {
      error = e.what();
    }
  });
  if (!c) throw RuntimeError(error.empty() ? "client creation failed" : error);
  return c;
}

// ------------------------------------------------------------------ errors
void Error_Destroy(PJRT_Error_Destroy_Args* a) { delete a->error; }
void Error_Message(PJRT_Error_Message_Args* a) {
  a->message = a->error->message.c_str();
  a->message_size = a->error->message.size();
}
PJRT_Error* Error_GetCode(PJRT_Error_GetCode_Args* a) {
  a->code = a->error->code;
  return nullptr;
}
PJRT_Error* Error_ForEachPayload(PJRT_Error_ForEachPayload_Args*) { return nullptr; }

// ------------------------------------------------------------------ plugin
PJRT_Error* Plugin_Initialize(PJRT_Plugin_Initialize_Args*) { return nullptr; }
// The StableHLO versions whose portable artifacts the bytecode reader accepts: jaxlib serialises a module for
// min(its own version, stablehlo_current_version) and refuses a plugin whose current version is below its minimum.
// The reader goes by op names with any version suffix and ignores attributes it has no use for, so the range is wide.
// (The reference advertises nothing, pjrt_client.cc:42-46, and lets MLIR's own reader take whatever jaxlib writes.)
PJRT_Error* Plugin_Attributes(PJRT_Plugin_Attributes_Args* a) {
  static const int64_t current[3] = {1, 9, 0}, minimum[3] = {0, 9, 0};
  static PJRT_NamedValue attrs[2];
  static std::once_flag once;
  std::call_once(once, [] {
    memset(attrs, 0, sizeof attrs);
    const char* names[2] = {"stablehlo_current_version", "stablehlo_minimum_version"};
    const int64_t* values[2] = {current, minimum};
    for (int k = 0; k < 2; ++k) {
      attrs[k].struct_size = sizeof(PJRT_NamedValue);
      attrs[k].name = names[k];
      attrs[k].name_size = strlen(names[k]);
      attrs[k].type = PJRT_NamedValue_kInt64List;
      attrs[k].int64_array_value = values[k];
      attrs[k].value_size = 3;
    }
  });
  a->attributes = attrs;
  a->num_attributes = 2;
  return nullptr;
}

// ------------------------------------------------------------------ events
PJRT_Error* Event_Destroy(PJRT_Event_Destroy_Args* a) {
  delete a->event;
  return nullptr;
}
PJRT_Error* Event_IsReady(PJRT_Event_IsReady_Args* a) {
  return guard([&]() -> PJRT_Error* {
    a->is_ready = true;
    if (a->event->ev) {
      int r = 0;
      if (mi355_event_query(a->event->ev, &r) != 0) return makeError(mi355_last_error());
      a->is_ready = r != 0;
    }
    return nullptr;
  });
}
PJRT_Error* Event_Error(PJRT_Event_Error_Args* a) {
  if (!a->event->error.empty()) return makeError(a->event->error);
  return nullptr;
}
PJRT_Error* Event_Await(PJRT_Event_Await_Args* a) {
  return guard([&]() -> PJRT_Error* {
    if (a->event->ev && mi355_event_sync(a->event->ev) != 0) return makeError(mi355_last_error());
    if (!a->event->error.empty()) return makeError(a->event->error);
    return nullptr;
  });
}
PJRT_Error* Event_OnReady(PJRT_Event_OnReady_Args* a) {
  return guard([&]() -> PJRT_Error* {
    PJRT_Event* e = a->event;
    auto cb = a->callback;
    void* arg = a->user_arg;
    int ready = 1;
    if (e->ev) mi355_event_query(e->ev, &ready);
    if (ready) {
      cb(e->error.empty() ? nullptr : makeError(e->error), arg);   // the callback owns the error
      return nullptr;
    }
    // the event may be destroyed by the caller before it fires: wait on a private event
    mi355_event_t priv = nullptr;
    if (mi355_event_create(&priv, 0) != 0 || mi355_event_record(priv, Device::get().stream()) != 0)
      return makeError(mi355_last_error());
    std::string err = e->error;
    CompletionService::get().post([priv, cb, arg, err] {
      std::string msg = err;
      if (mi355_event_sync(priv) != 0) msg = mi355_last_error();
      mi355_event_destroy(priv);
      cb(msg.empty() ? nullptr : makeError(msg), arg);
    });
    return nullptr;
  });
}

// ------------------------------------------------------------------ client
PJRT_Error* Client_Create(PJRT_Client_Create_Args* a) {
  return guard([&]() -> PJRT_Error* {
    std::lock_guard<std::recursive_mutex> lk(apiMutex());
    a->client = theClient();
    return nullptr;
  });
}
PJRT_Error* Client_Destroy(PJRT_Client_Destroy_Args*) { return nullptr; }   // process-wide singleton
PJRT_Error* Client_PlatformName(PJRT_Client_PlatformName_Args* a) {
  a->platform_name = kPlatformName;
  a->platform_name_size = strlen(kPlatformName);
  return nullptr;
}
PJRT_Error* Client_ProcessIndex(PJRT_Client_ProcessIndex_Args* a) {
  a->process_index = 0;
  return nullptr;
}
PJRT_Error* Client_PlatformVersion(PJRT_Client_PlatformVersion_Args* a) {
  a->platform_version = a->client->platformVersion.c_str();
  a->platform_version_size = a->client->platformVersion.size();
  return nullptr;
}
PJRT_Error* Client_TopologyDescription(PJRT_Client_TopologyDescription_Args* a) {
  a->topology = &a->client->topology;
  return nullptr;
}
PJRT_Error* Client_Devices(PJRT_Client_Devices_Args* a) {
  a->devices = a->client->devices;
  a->num_devices = 1;
  return nullptr;
}
PJRT_Error* Client_AddressableDevices(PJRT_Client_AddressableDevices_Args* a) {
  a->addressable_devices = a->client->devices;
  a->num_addressable_devices = 1;
  return nullptr;
}
PJRT_Error* Client_LookupDevice(PJRT_Client_LookupDevice_Args* a) {
  if (a->id != 0) return makeError("no device with id " + std::to_string(a->id), PJRT_Error_Code_NOT_FOUND);
  a->device = &a->client->device;
  return nullptr;
}
PJRT_Error* Client_LookupAddressableDevice(PJRT_Client_LookupAddressableDevice_Args* a) {
  if (a->local_hardware_id != 0) return makeError("no device with local hardware id " + std::to_string(a->local_hardware_id), PJRT_Error_Code_NOT_FOUND);
  a->addressable_device = &a->client->device;
  return nullptr;
}
PJRT_Error* Client_AddressableMemories(PJRT_Client_AddressableMemories_Args* a) {
  a->addressable_memories = a->client->memories;
  a->num_addressable_memories = 1;
  return nullptr;
}
PJRT_Error* Client_DefaultDeviceAssignment(PJRT_Client_DefaultDeviceAssignment_Args* a) {
  if (a->num_replicas * a->num_partitions > 1) return makeError("the MI355X plugin drives exactly one device", PJRT_Error_Code_INVALID_ARGUMENT);
  for (size_t i = 0; i < a->default_assignment_size; ++i) a->default_assignment[i] = 0;
  return nullptr;
}

void fillExecutableMetadata(PJRT_Executable* e) {
  const CompiledProgram& p = e->exe->program();
  static const char* kDevice = "device";
  for (auto& o : p.outputs) {
    e->outTypes.push_back(toPjrt(o.type.dt));
    e->outDimSizes.push_back(o.type.dims.size());
    for (auto d : o.type.dims) e->outDims.push_back(d);
    e->outMemKinds.push_back(kDevice);
    e->outMemKindSizes.push_back(6);
  }
  char fp[64];
  snprintf(fp, sizeof fp, "mi355x-%d-ops-%d-steps-%lld", p.numOps, p.numSteps, (long long)p.arenaBytes);
  e->fingerprint = fp;
}

// text -> plan -> loaded executable (shared by Compile and DeserializeAndLoad)
PJRT_LoadedExecutable* compileAndLoad(PJRT_Client* client, const char* code, size_t size) {
  auto module = parseStableHLOText(code, size);
  auto prog = compileProgram(std::move(module));
  auto* ex = new PJRT_Executable();
  try {
    ex->exe = std::make_shared<Executable>(std::move(prog));
  } catch (...) {
    delete ex;
    throw;
  }
  ex->source.assign(code, size);
  ex->ownedByLoaded = true;
  fillExecutableMetadata(ex);
  auto* le = new PJRT_LoadedExecutable();
  le->executable = ex;
  le->client = client;
  return le;
}

PJRT_Error* Client_Compile(PJRT_Client_Compile_Args* a) {
  return guard([&]() -> PJRT_Error* {
    std::lock_guard<std::recursive_mutex> lk(apiMutex());
    if (!a->program || !a->program->code) return makeError("null program", PJRT_Error_Code_INVALID_ARGUMENT);
    std::string format(a->program->format ? a->program->format : "", a->program->format ? a->program->format_size : 0);
    if (format != "mlir") return makeError("unsupported program format '" + format + "' (expected 'mlir')", PJRT_Error_Code_INVALID_ARGUMENT);
    a->executable = compileAndLoad(a->client, a->program->code, a->program->code_size);
    return nullptr;
  });
}

// host -> device (reference: mlx_buffer.cc:104-267): dense row-major on device; strided host layouts are repacked
PJRT_Error* Client_BufferFromHostBuffer(PJRT_Client_BufferFromHostBuffer_Args* a) {
  return guard([&]() -> PJRT_Error* {
    std::lock_guard<std::recursive_mutex> lk(apiMutex());
    DType dt = fromPjrt(a->type);
    if (dt == DType::Invalid) return makeError("unsupported buffer element type " + std::to_string((int)a->type) + " (f64, complex and sub-byte types are not supported)", PJRT_Error_Code_INVALID_ARGUMENT);
    TensorType t;
    t.dt = dt;
    for (size_t i = 0; i < a->num_dims; ++i) t.dims.push_back(a->dims[i]);
    size_t bytes = t.bytes();
    if (bytes > 0 && !a->data) return makeError("null host data pointer", PJRT_Error_Code_INVALID_ARGUMENT);
    Device& dev = Device::get();
    auto buf = std::make_shared<DeviceBuffer>();
    buf->type = t;
    buf->ptr = dev.alloc(std::max<size_t>(bytes, 4));
    if (bytes > 0) {
      const void* src = a->data;
      std::vector<char> packed;
      size_t esz = dtypeSize(dt);
      bool dense = true;
      if (a->byte_strides && a->num_byte_strides == a->num_dims) {
        int64_t expect = (int64_t)esz;
        for (int d = (int)a->num_dims - 1; d >= 0; --d) {
          if (a->dims[d] != 1 && a->byte_strides[d] != expect) dense = false;
          expect *= a->dims[d];
        }
      }
      if (!dense) {
        for (size_t d = 0; d < a->num_dims; ++d)
          if (a->byte_strides[d] < 0) return makeError("negative host byte strides are not supported", PJRT_Error_Code_INVALID_ARGUMENT);
        packed.resize(bytes);
        std::vector<int64_t> idx(a->num_dims, 0);
        int64_t n = t.numel();
        for (int64_t i = 0; i < n; ++i) {
          int64_t off = 0;
          for (size_t d = 0; d < a->num_dims; ++d) off += idx[d] * a->byte_strides[d];
          memcpy(packed.data() + i * esz, (const char*)a->data + off, esz);
          for (int d = (int)a->num_dims - 1; d >= 0; --d) {
            if (++idx[d] < a->dims[d]) break;
            idx[d] = 0;
          }
        }
        src = packed.data();
      }
      if (mi355_memcpy_h2d(buf->ptr, src, bytes, dev.stream()) != 0) return makeError(mi355_last_error());
      dev.sync();   // the host buffer may be reused as soon as we return
    }
    auto* pb = new PJRT_Buffer();
    pb->buf = std::move(buf);
    pb->client = a->client;
    pb->dims = t.dims;
    a->buffer = pb;
    a->done_with_host_buffer = readyEvent();
    return nullptr;
  });
}

// --------------------------------------------------------- device / memory
PJRT_Error* DeviceDescription_Id(PJRT_DeviceDescription_Id_Args* a) { a->id = a->device_description->id; return nullptr; }
PJRT_Error* DeviceDescription_ProcessIndex(PJRT_DeviceDescription_ProcessIndex_Args* a) { a->process_index = 0; return nullptr; }
PJRT_Error* DeviceDescription_Attributes(PJRT_DeviceDescription_Attributes_Args* a) { a->attributes = nullptr; a->num_attributes = 0; return nullptr; }
PJRT_Error* DeviceDescription_Kind(PJRT_DeviceDescription_Kind_Args* a) {
  a->device_kind = a->device_description->kind.c_str();
  a->device_kind_size = a->device_description->kind.size();
  return nullptr;
}
PJRT_Error* DeviceDescription_DebugString(PJRT_DeviceDescription_DebugString_Args* a) {
  a->debug_string = a->device_description->debug.c_str();
  a->debug_string_size = a->device_description->debug.size();
  return nullptr;
}
PJRT_Error* DeviceDescription_ToString(PJRT_DeviceDescription_ToString_Args* a) {
  a->to_string = a->device_description->str.c_str();
  a->to_string_size = a->device_description->str.size();
  return nullptr;
}
PJRT_Error* Device_GetDescription(PJRT_Device_GetDescription_Args* a) { a->device_description = &a->device->desc; return nullptr; }
PJRT_Error* Device_IsAddressable(PJRT_Device_IsAddressable_Args* a) { a->is_addressable = true; return nullptr; }
PJRT_Error* Device_LocalHardwareId(PJRT_Device_LocalHardwareId_Args* a) { a->local_hardware_id = 0; return nullptr; }
PJRT_Error* Device_AddressableMemories(PJRT_Device_AddressableMemories_Args* a) {
  a->memories = a->device->client->memories;
  a->num_memories = 1;
  return nullptr;
}
PJRT_Error* Device_DefaultMemory(PJRT_Device_DefaultMemory_Args* a) { a->memory = a->device->memory; return nullptr; }
PJRT_Error* Device_MemoryStats(PJRT_Device_MemoryStats_Args* a) {
  return guard([&]() -> PJRT_Error* {
    Device& d = Device::get();
    a->bytes_in_use = d.bytesInUse();
    a->peak_bytes_in_use = d.peakBytesInUse(); a->peak_bytes_in_use_is_set = true;
    a->num_allocs = d.numAllocs(); a->num_allocs_is_set = true;
    a->largest_alloc_size = d.largestAlloc(); a->largest_alloc_size_is_set = true;
    a->bytes_limit = (int64_t)d.totalMemory(); a->bytes_limit_is_set = true;
    a->bytes_reserved = d.bytesReserved(); a->bytes_reserved_is_set = true;
    a->peak_bytes_reserved = 0; a->peak_bytes_reserved_is_set = false;
    a->bytes_reservable_limit = 0; a->bytes_reservable_limit_is_set = false;
    a->largest_free_block_bytes = 0; a->largest_free_block_bytes_is_set = false;
    a->pool_bytes = d.bytesReserved(); a->pool_bytes_is_set = true;
    a->peak_pool_bytes = 0; a->peak_pool_bytes_is_set = false;
    return nullptr;
  });
}
PJRT_Error* Memory_Id(PJRT_Memory_Id_Args* a) { a->id = a->memory->id; return nullptr; }
PJRT_Error* Memory_Kind(PJRT_Memory_Kind_Args* a) { a->kind = a->memory->kind.c_str(); a->kind_size = a->memory->kind.size(); return nullptr; }
PJRT_Error* Memory_DebugString(PJRT_Memory_DebugString_Args* a) { a->debug_string = a->memory->debug.c_str(); a->debug_string_size = a->memory->debug.size(); return nullptr; }
PJRT_Error* Memory_ToString(PJRT_Memory_ToString_Args* a) { a->to_string = a->memory->debug.c_str(); a->to_string_size = a->memory->debug.size(); return nullptr; }
PJRT_Error* Memory_AddressableByDevices(PJRT_Memory_AddressableByDevices_Args* a) {
  a->devices = a->memory->device->client->devices;
  a->num_devices = 1;
  return nullptr;
}

// --------------------------------------------------------------- executables
PJRT_Error* Executable_Destroy(PJRT_Executable_Destroy_Args* a) {
  std::lock_guard<std::recursive_mutex> lk(apiMutex());
  if (a->executable && !a->executable->ownedByLoaded) delete a->executable;
  return nullptr;
}
PJRT_Error* Executable_Name(PJRT_Executable_Name_Args* a) {
  a->executable_name = kExecutableName;
  a->executable_name_size = strlen(kExecutableName);
  return nullptr;
}
PJRT_Error* Executable_NumReplicas(PJRT_Executable_NumReplicas_Args* a) { a->num_replicas = 1; return nullptr; }
PJRT_Error* Executable_NumPartitions(PJRT_Executable_NumPartitions_Args* a) { a->num_partitions = 1; return nullptr; }
PJRT_Error* Executable_NumOutputs(PJRT_Executable_NumOutputs_Args* a) {
  a->num_outputs = a->executable->exe->program().outputs.size();
  return nullptr;
}
PJRT_Error* Executable_SizeOfGeneratedCodeInBytes(PJRT_Executable_SizeOfGeneratedCodeInBytes_Args* a) {
  int64_t n = 0;
  for (auto& k : a->executable->exe->program().kernels) n += (int64_t)k.source.size();
  a->size_in_bytes = n;
  return nullptr;
}
// Static plan figures plus, when MI355X_TIMING is set, measured per-kind step times
// (HIP events on the compute stream): "<kind>.count/.time_ms/.flops/.bytes".
PJRT_Error* Executable_GetCostAnalysis(PJRT_Executable_GetCostAnalysis_Args* a) {
  return guard([&]() -> PJRT_Error* {
    std::lock_guard<std::recursive_mutex> lk(apiMutex());
    PJRT_Executable* e = a->executable;
    e->cost.clear();
    e->costNames.clear();
    std::vector<std::pair<std::string, double>> vals;
    const CompiledProgram& p = e->exe->program();
    vals.emplace_back("steps", p.numSteps);
    vals.emplace_back("ops", p.numOps);
    vals.emplace_back("fused_kernels", (double)p.kernels.size());
    vals.emplace_back("arena_bytes", (double)p.arenaBytes);
    vals.emplace_back("compile_seconds", e->exe->compileSeconds);
    vals.emplace_back("loop.host_syncs", (double)e->exe->loopHostSyncs());
    vals.emplace_back("plan.graph_launches", (double)e->exe->planGraphLaunches());
    for (auto& kv : e->exe->timings()) {
      vals.emplace_back(kv.first + ".count", (double)kv.second.count);
      vals.emplace_back(kv.first + ".time_ms", kv.second.ms);
      vals.emplace_back(kv.first + ".flops", kv.second.flops);
      vals.emplace_back(kv.first + ".bytes", kv.second.bytes);
    }
    e->costNames.reserve(vals.size());
    for (auto& v : vals) e->costNames.push_back(v.first);
    for (size_t i = 0; i < vals.size(); ++i) {
      PJRT_NamedValue nv;
      memset(&nv, 0, sizeof nv);
      nv.struct_size = sizeof(PJRT_NamedValue);
      nv.name = e->costNames[i].c_str();
      nv.name_size = e->costNames[i].size();
      nv.type = PJRT_NamedValue_kFloat;
      nv.float_value = (float)vals[i].second;
      nv.value_size = 1;
      e->cost.push_back(nv);
    }
    a->num_properties = e->cost.size();
    a->properties = e->cost.data();
    return nullptr;
  });
}
PJRT_Error* Executable_OutputMemoryKinds(PJRT_Executable_OutputMemoryKinds_Args* a) {
  a->num_outputs = a->executable->outMemKinds.size();
  a->memory_kinds = a->executable->outMemKinds.data();
  a->memory_kind_sizes = a->executable->outMemKindSizes.data();
  return nullptr;
}
PJRT_Error* Executable_OptimizedProgram(PJRT_Executable_OptimizedProgram_Args*) { return unimplemented("PJRT_Executable_OptimizedProgram"); }
// A serialized executable is the program text behind a small header: loading it again replans
// (milliseconds) and finds every generated kernel in the on-disk code-object cache, so nothing
// is recompiled.  The reference leaves both entry points unimplemented (pjrt_executable.cc:101-107,
// 269-271); with them JAX's persistent compilation cache works.
constexpr char kSerialMagic[] = "MI355X-PJRT-EXE\x01";
PJRT_Error* Executable_Serialize(PJRT_Executable_Serialize_Args* a) {
  return guard([&]() -> PJRT_Error* {
    if (!a->executable) return makeError("null executable", PJRT_Error_Code_INVALID_ARGUMENT);
    auto* out = new PJRT_SerializedExecutable();
    out->bytes.assign(kSerialMagic, sizeof(kSerialMagic) - 1);
    uint64_t n = a->executable->source.size();
    out->bytes.append((const char*)&n, sizeof n);
    out->bytes += a->executable->source;
    a->serialized_executable = out;
    a->serialized_bytes = out->bytes.data();
    a->serialized_bytes_size = out->bytes.size();
    a->serialized_executable_deleter = [](PJRT_SerializedExecutable* p) { delete p; };
    return nullptr;
  });
}
PJRT_Error* Executable_OutputElementTypes(PJRT_Executable_OutputElementTypes_Args* a) {
  a->output_types = a->executable->outTypes.data();
  a->num_output_types = a->executable->outTypes.size();
  return nullptr;
}
PJRT_Error* Executable_OutputDimensions(PJRT_Executable_OutputDimensions_Args* a) {
  a->num_outputs = a->executable->outDimSizes.size();
  a->dims = a->executable->outDims.data();
  a->dim_sizes = a->executable->outDimSizes.data();
  return nullptr;
}
PJRT_Error* Executable_Fingerprint(PJRT_Executable_Fingerprint_Args* a) {
  a->executable_fingerprint = a->executable->fingerprint.c_str();
  a->executable_fingerprint_size = a->executable->fingerprint.size();
  return nullptr;
}
PJRT_Error* Executable_GetCompiledMemoryStats(PJRT_Executable_GetCompiledMemoryStats_Args*) { return unimplemented("PJRT_Executable_GetCompiledMemoryStats"); }
PJRT_Error* Executable_GetCompileOptions(PJRT_Executable_GetCompileOptions_Args*) { return unimplemented("PJRT_Executable_GetCompileOptions"); }
PJRT_Error* Executable_DeserializeAndLoad(PJRT_Executable_DeserializeAndLoad_Args* a) {
  return guard([&]() -> PJRT_Error* {
    std::lock_guard<std::recursive_mutex> lk(apiMutex());
    const size_t head = sizeof(kSerialMagic) - 1 + sizeof(uint64_t);
    if (!a->serialized_executable || a->serialized_executable_size < head || memcmp(a->serialized_executable, kSerialMagic, sizeof(kSerialMagic) - 1) != 0)
      return makeError("not an executable serialized by this plugin", PJRT_Error_Code_INVALID_ARGUMENT);
    uint64_t n = 0;
    memcpy(&n, a->serialized_executable + sizeof(kSerialMagic) - 1, sizeof n);
    if (n != a->serialized_executable_size - head) return makeError("serialized executable is truncated", PJRT_Error_Code_INVALID_ARGUMENT);
    a->loaded_executable = compileAndLoad(a->client, a->serialized_executable + head, (size_t)n);
    return nullptr;
  });
}

PJRT_Error* LoadedExecutable_Destroy(PJRT_LoadedExecutable_Destroy_Args* a) {
  std::lock_guard<std::recursive_mutex> lk(apiMutex());
  if (a->executable) {
    delete a->executable->executable;
    delete a->executable;
  }
  return nullptr;
}
PJRT_Error* LoadedExecutable_GetExecutable(PJRT_LoadedExecutable_GetExecutable_Args* a) {
  a->executable = a->loaded_executable->executable;
  return nullptr;
}
PJRT_Error* LoadedExecutable_AddressableDevices(PJRT_LoadedExecutable_AddressableDevices_Args* a) {
  a->addressable_devices = a->executable->client->devices;
  a->num_addressable_devices = 1;
  return nullptr;
}
PJRT_Error* LoadedExecutable_Delete(PJRT_LoadedExecutable_Delete_Args* a) { a->executable->deleted = true; return nullptr; }
PJRT_Error* LoadedExecutable_IsDeleted(PJRT_LoadedExecutable_IsDeleted_Args* a) { a->is_deleted = a->executable->deleted; return nullptr; }
PJRT_Error* LoadedExecutable_Fingerprint(PJRT_LoadedExecutable_Fingerprint_Args* a) {
  a->executable_fingerprint = a->executable->executable->fingerprint.c_str();
  a->executable_fingerprint_size = a->executable->executable->fingerprint.size();
  return nullptr;
}
// xla.DeviceAssignmentProto{replica_count=1, computation_count=1, computation_devices=[{replica_device_ids=[0]}]}
// hand-encoded (reference links protobuf for these nine bytes: pjrt_executable.cc:290-313)
PJRT_Error* LoadedExecutable_GetDeviceAssignment(PJRT_LoadedExecutable_GetDeviceAssignment_Args* a) {
  static const unsigned char kProto[] = {0x08, 0x01, 0x10, 0x01, 0x1a, 0x03, 0x0a, 0x01, 0x00};
  auto* blob = new std::string((const char*)kProto, sizeof kProto);
  a->serialized_bytes = blob->data();
  a->serialized_bytes_size = blob->size();
  a->serialized_device_assignment = blob;
  a->serialized_device_assignment_deleter = [](void* p) { delete (std::string*)p; };
  return nullptr;
}

// reference: pjrt_executable.cc:178-258
PJRT_Error* LoadedExecutable_Execute(PJRT_LoadedExecutable_Execute_Args* a) {
  return guard([&]() -> PJRT_Error* {
    std::lock_guard<std::recursive_mutex> lk(apiMutex());
    if (!a->executable || a->executable->deleted) return makeError("executable was deleted", PJRT_Error_Code_FAILED_PRECONDITION);
    if (a->num_devices != 1) return makeError("the MI355X plugin executes on exactly one device", PJRT_Error_Code_INVALID_ARGUMENT);
    std::vector<DeviceBuffer*> ins;
    for (size_t i = 0; i < a->num_args; ++i) {
      PJRT_Buffer* b = a->argument_lists[0][i];
      if (!b || !b->buf) return makeError("null input buffer at argument " + std::to_string(i), PJRT_Error_Code_INVALID_ARGUMENT);
      ins.push_back(b->buf.get());
    }
    // every input may be donated except those the caller lists (they have other holders); which of them the
    // program actually takes is its own declaration (tf.aliasing_output / jax.buffer_donor on the argument)
    std::vector<bool> mayDonate(ins.size(), true);
    if (a->options && a->options->non_donatable_input_indices)
      for (size_t k = 0; k < a->options->num_non_donatable_input_indices; ++k) {
        int64_t i = a->options->non_donatable_input_indices[k];
        if (i >= 0 && (size_t)i < mayDonate.size()) mayDonate[(size_t)i] = false;
      }
    for (size_t i = 0; i < ins.size(); ++i)
      if (a->argument_lists[0][i]->buf.use_count() > 1) mayDonate[i] = false;
    auto outs = a->executable->executable->exe->execute(ins, &mayDonate);
    for (size_t i = 0; i < outs.size(); ++i) {
      auto* pb = new PJRT_Buffer();
      pb->dims = outs[i]->type.dims;
      pb->buf = std::move(outs[i]);
      pb->client = a->executable->client;
      a->output_lists[0][i] = pb;
    }
    if (a->device_complete_events) a->device_complete_events[0] = streamEvent();
    return nullptr;
  });
}

// ------------------------------------------------------------------- buffers
PJRT_Error* Buffer_Destroy(PJRT_Buffer_Destroy_Args* a) {
  std::lock_guard<std::recursive_mutex> lk(apiMutex());
  delete a->buffer;
  return nullptr;
}
PJRT_Error* Buffer_ElementType(PJRT_Buffer_ElementType_Args* a) { a->type = toPjrt(a->buffer->buf->type.dt); return nullptr; }
PJRT_Error* Buffer_Dimensions(PJRT_Buffer_Dimensions_Args* a) {
  a->dims = a->buffer->dims.data();
  a->num_dims = a->buffer->dims.size();
  return nullptr;
}
PJRT_Error* Buffer_UnpaddedDimensions(PJRT_Buffer_UnpaddedDimensions_Args* a) {
  a->unpadded_dims = a->buffer->dims.data();
  a->num_dims = a->buffer->dims.size();
  return nullptr;
}
PJRT_Error* Buffer_DynamicDimensionIndices(PJRT_Buffer_DynamicDimensionIndices_Args* a) {
  a->dynamic_dim_indices = nullptr;
  a->num_dynamic_dims = 0;
  return nullptr;
}
PJRT_Error* Buffer_GetMemoryLayout(PJRT_Buffer_GetMemoryLayout_Args* a) {
  memset(&a->layout, 0, sizeof a->layout);
  a->layout.struct_size = sizeof(PJRT_Buffer_MemoryLayout);
  a->layout.type = PJRT_Buffer_MemoryLayout_Type_Strides;
  return nullptr;
}
PJRT_Error* Buffer_OnDeviceSizeInBytes(PJRT_Buffer_OnDeviceSizeInBytes_Args* a) {
  a->on_device_size_in_bytes = a->buffer->buf->type.bytes();
  return nullptr;
}
PJRT_Error* Buffer_Device(PJRT_Buffer_Device_Args* a) { a->device = &a->buffer->client->device; return nullptr; }
PJRT_Error* Buffer_Memory(PJRT_Buffer_Memory_Args* a) { a->memory = &a->buffer->client->memory; return nullptr; }
// Marks the buffer deleted and gives its memory back to the allocator now (work already enqueued that reads it is
// ordered before any reuse, because every use is ordered on the main stream: side-stream work is joined before Execute returns or fails); the handle lives on until Buffer_Destroy.
// The reference only sets the flag (mlx_buffer.cc:290-296) and lets MLX's reference counting free the array.
PJRT_Error* Buffer_Delete(PJRT_Buffer_Delete_Args* a) {
  return guard([&]() -> PJRT_Error* {
    std::lock_guard<std::recursive_mutex> lk(apiMutex());
    DeviceBuffer* b = a->buffer->buf.get();
    if (!b->deleted) {
      b->deleted = true;
      if (b->ptr && a->buffer->buf.use_count() == 1) {
        Device::get().release(b->ptr);
        b->ptr = nullptr;
      }
    }
    return nullptr;
  });
}
PJRT_Error* Buffer_IsDeleted(PJRT_Buffer_IsDeleted_Args* a) { a->is_deleted = a->buffer->buf->deleted; return nullptr; }

PJRT_Error* copyBuffer(PJRT_Buffer* src, PJRT_Buffer** dst) {
  return guard([&]() -> PJRT_Error* {
    std::lock_guard<std::recursive_mutex> lk(apiMutex());
    if (src->buf->deleted) return makeError("buffer was deleted", PJRT_Error_Code_FAILED_PRECONDITION);
    Device& dev = Device::get();
    auto nb = std::make_shared<DeviceBuffer>();
    nb->type = src->buf->type;
    size_t bytes = std::max<size_t>(nb->type.bytes(), 4);
    nb->ptr = dev.alloc(bytes);
    if (mi355_memcpy_d2d(nb->ptr, src->buf->ptr, nb->type.bytes(), dev.stream()) != 0) return makeError(mi355_last_error());
    auto* pb = new PJRT_Buffer();
    pb->buf = std::move(nb);
    pb->client = src->client;
    pb->dims = src->dims;
    *dst = pb;
    return nullptr;
  });
}
PJRT_Error* Buffer_CopyToDevice(PJRT_Buffer_CopyToDevice_Args* a) { return copyBuffer(a->buffer, &a->dst_buffer); }
PJRT_Error* Buffer_CopyToMemory(PJRT_Buffer_CopyToMemory_Args* a) { return copyBuffer(a->buffer, &a->dst_buffer); }

// device -> host (reference: mlx_buffer.cc:298-335).  dst == NULL only reports the size.
PJRT_Error* Buffer_ToHostBuffer(PJRT_Buffer_ToHostBuffer_Args* a) {
  return guard([&]() -> PJRT_Error* {
    std::lock_guard<std::recursive_mutex> lk(apiMutex());
    DeviceBuffer* b = a->src->buf.get();
    if (b->deleted) return makeError("buffer was deleted", PJRT_Error_Code_FAILED_PRECONDITION);
    size_t bytes = b->type.bytes();
    if (!a->dst) {
      a->dst_size = bytes;
      a->event = nullptr;
      return nullptr;
    }
    if (a->dst_size < bytes) return makeError("destination holds " + std::to_string(a->dst_size) + " bytes, buffer needs " + std::to_string(bytes), PJRT_Error_Code_INVALID_ARGUMENT);
    Device& dev = Device::get();
    if (bytes > 0) {
      if (mi355_memcpy_d2h(a->dst, b->ptr, bytes, dev.stream()) != 0) return makeError(mi355_last_error());
      dev.sync();
    }
    a->event = readyEvent();
    return nullptr;
  });
}
PJRT_Error* Buffer_IsOnCpu(PJRT_Buffer_IsOnCpu_Args* a) { a->is_on_cpu = false; return nullptr; }
PJRT_Error* Buffer_ReadyEvent(PJRT_Buffer_ReadyEvent_Args* a) {
  return guard([&]() -> PJRT_Error* {
    std::lock_guard<std::recursive_mutex> lk(apiMutex());
    a->event = streamEvent();   // everything queued so far includes the producer of this buffer
    return nullptr;
  });
}
PJRT_Error* Buffer_UnsafePointer(PJRT_Buffer_UnsafePointer_Args* a) { a->buffer_pointer = (uintptr_t)a->buffer->buf->ptr; return nullptr; }
PJRT_Error* Buffer_IncreaseExternalReferenceCount(PJRT_Buffer_IncreaseExternalReferenceCount_Args*) { return nullptr; }
PJRT_Error* Buffer_DecreaseExternalReferenceCount(PJRT_Buffer_DecreaseExternalReferenceCount_Args*) { return nullptr; }
PJRT_Error* Buffer_OpaqueDeviceMemoryDataPointer(PJRT_Buffer_OpaqueDeviceMemoryDataPointer_Args* a) { a->device_memory_ptr = a->buffer->buf->ptr; return nullptr; }

PJRT_Error* CopyToDeviceStream_Destroy(PJRT_CopyToDeviceStream_Destroy_Args*) { return nullptr; }
PJRT_Error* CopyToDeviceStream_AddChunk(PJRT_CopyToDeviceStream_AddChunk_Args*) { return unimplemented("PJRT_CopyToDeviceStream_AddChunk"); }
PJRT_Error* CopyToDeviceStream_TotalBytes(PJRT_CopyToDeviceStream_TotalBytes_Args* a) { a->total_bytes = 0; return nullptr; }
PJRT_Error* CopyToDeviceStream_GranuleSize(PJRT_CopyToDeviceStream_GranuleSize_Args* a) { a->granule_size_in_bytes = 0; return nullptr; }
PJRT_Error* CopyToDeviceStream_CurrentBytes(PJRT_CopyToDeviceStream_CurrentBytes_Args* a) { a->current_bytes = 0; return nullptr; }

// ------------------------------------------------------------------ topology
PJRT_Error* TopologyDescription_Create(PJRT_TopologyDescription_Create_Args* a) {
  return guard([&]() -> PJRT_Error* {
    a->topology = &theClient()->topology;
    return nullptr;
  });
}
PJRT_Error* TopologyDescription_Destroy(PJRT_TopologyDescription_Destroy_Args*) { return nullptr; }
PJRT_Error* TopologyDescription_PlatformName(PJRT_TopologyDescription_PlatformName_Args* a) {
  a->platform_name = kPlatformName;
  a->platform_name_size = strlen(kPlatformName);
  return nullptr;
}
PJRT_Error* TopologyDescription_PlatformVersion(PJRT_TopologyDescription_PlatformVersion_Args* a) {
  a->platform_version = kPlatformVersion;
  a->platform_version_size = strlen(kPlatformVersion);
  return nullptr;
}
PJRT_Error* TopologyDescription_GetDeviceDescriptions(PJRT_TopologyDescription_GetDeviceDescriptions_Args* a) {
  a->descriptions = &a->topology->desc;
  a->num_descriptions = 1;
  return nullptr;
}
PJRT_Error* TopologyDescription_Serialize(PJRT_TopologyDescription_Serialize_Args*) { return unimplemented("PJRT_TopologyDescription_Serialize"); }
PJRT_Error* TopologyDescription_Attributes(PJRT_TopologyDescription_Attributes_Args* a) { a->attributes = nullptr; a->num_attributes = 0; return nullptr; }
PJRT_Error* TopologyDescription_Fingerprint(PJRT_TopologyDescription_Fingerprint_Args* a) {
  static const char* fp = "mi355x-1x1";
  a->fingerprint = fp;
  a->fingerprint_size = strlen(fp);
  return nullptr;
}
PJRT_Error* Compile(PJRT_Compile_Args*) { return unimplemented("PJRT_Compile (ahead-of-time compilation without a client)"); }

// Profiler extension: present in the chain so that jaxlib does not dereference NULL; every
// operation reports "not supported" (reference: pjrt_profiler.cc:61-111).
struct ProfilerApi {
  size_t struct_size;
  void* priv;
  PJRT_Error* (*error_destroy)(void*);
  PJRT_Error* (*error_message)(void*);
  PJRT_Error* (*error_get_code)(void*);
  PJRT_Error* (*create)(void*);
  PJRT_Error* (*destroy)(void*);
  PJRT_Error* (*start)(void*);
  PJRT_Error* (*stop)(void*);
  PJRT_Error* (*collect_data)(void*);
};
PJRT_Error* profilerUnsupported(void*) { return makeError("profiling is not supported by the MI355X plugin", PJRT_Error_Code_UNIMPLEMENTED); }
struct ProfilerExtension {
  PJRT_Extension_Base base;
  ProfilerApi* profiler_api;
  int64_t traceme_context_id;
};
ProfilerApi g_profilerApi = {sizeof(ProfilerApi), nullptr, profilerUnsupported, profilerUnsupported, profilerUnsupported,
                             profilerUnsupported, profilerUnsupported, profilerUnsupported, profilerUnsupported, profilerUnsupported};
ProfilerExtension g_profilerExt = {{sizeof(ProfilerExtension), PJRT_Extension_Type_Profiler, nullptr}, &g_profilerApi, 0};

const PJRT_Api* buildApi() {
  static PJRT_Api api;
  memset(&api, 0, sizeof api);
  api.struct_size = sizeof(PJRT_Api);
  api.extension_start = &g_profilerExt.base;
  api.pjrt_api_version.struct_size = sizeof(PJRT_Api_Version);
  api.pjrt_api_version.major_version = PJRT_API_MAJOR;
  api.pjrt_api_version.minor_version = PJRT_API_MINOR;
#define SET(name, fn) api.PJRT_##name = fn
  SET(Error_Destroy, Error_Destroy); SET(Error_Message, Error_Message); SET(Error_GetCode, Error_GetCode);
  SET(Plugin_Initialize, Plugin_Initialize); SET(Plugin_Attributes, Plugin_Attributes);
  SET(Event_Destroy, Event_Destroy); SET(Event_IsReady, Event_IsReady); SET(Event_Error, Event_Error);
  SET(Event_Await, Event_Await); SET(Event_OnReady, Event_OnReady);
  SET(Client_Create, Client_Create); SET(Client_Destroy, Client_Destroy); SET(Client_PlatformName, Client_PlatformName);
  SET(Client_ProcessIndex, Client_ProcessIndex); SET(Client_PlatformVersion, Client_PlatformVersion);
  SET(Client_Devices, Client_Devices); SET(Client_AddressableDevices, Client_AddressableDevices);
  SET(Client_LookupDevice, Client_LookupDevice); SET(Client_LookupAddressableDevice, Client_LookupAddressableDevice);
  SET(Client_AddressableMemories, Client_AddressableMemories); SET(Client_Compile, Client_Compile);
  SET(Client_DefaultDeviceAssignment, Client_DefaultDeviceAssignment);
  SET(Client_BufferFromHostBuffer, Client_BufferFromHostBuffer);
  SET(DeviceDescription_Id, DeviceDescription_Id); SET(DeviceDescription_ProcessIndex, DeviceDescription_ProcessIndex);
  SET(DeviceDescription_Attributes, DeviceDescription_Attributes); SET(DeviceDescription_Kind, DeviceDescription_Kind);
  SET(DeviceDescription_DebugString, DeviceDescription_DebugString); SET(DeviceDescription_ToString, DeviceDescription_ToString);
  SET(Device_GetDescription, Device_GetDescription); SET(Device_IsAddressable, Device_IsAddressable);
  SET(Device_LocalHardwareId, Device_LocalHardwareId); SET(Device_AddressableMemories, Device_AddressableMemories);
  SET(Device_DefaultMemory, Device_DefaultMemory); SET(Device_MemoryStats, Device_MemoryStats);
  SET(Memory_Id, Memory_Id); SET(Memory_Kind, Memory_Kind); SET(Memory_DebugString, Memory_DebugString);
  SET(Memory_ToString, Memory_ToString); SET(Memory_AddressableByDevices, Memory_AddressableByDevices);
  SET(Executable_Destroy, Executable_Destroy); SET(Executable_Name, Executable_Name);
  SET(Executable_NumReplicas, Executable_NumReplicas); SET(Executable_NumPartitions, Executable_NumPartitions);
  SET(Executable_NumOutputs, Executable_NumOutputs);
  SET(Executable_SizeOfGeneratedCodeInBytes, Executable_SizeOfGeneratedCodeInBytes);
  SET(Executable_GetCostAnalysis, Executable_GetCostAnalysis); SET(Executable_OutputMemoryKinds, Executable_OutputMemoryKinds);
  SET(Executable_OptimizedProgram, Executable_OptimizedProgram); SET(Executable_Serialize, Executable_Serialize);
  SET(LoadedExecutable_Destroy, LoadedExecutable_Destroy); SET(LoadedExecutable_GetExecutable, LoadedExecutable_GetExecutable);
  SET(LoadedExecutable_AddressableDevices, LoadedExecutable_AddressableDevices);
  SET(LoadedExecutable_Delete, LoadedExecutable_Delete); SET(LoadedExecutable_IsDeleted, LoadedExecutable_IsDeleted);
  SET(LoadedExecutable_Execute, LoadedExecutable_Execute); SET(Executable_DeserializeAndLoad, Executable_DeserializeAndLoad);
  SET(LoadedExecutable_Fingerprint, LoadedExecutable_Fingerprint);
  SET(Buffer_Destroy, Buffer_Destroy); SET(Buffer_ElementType, Buffer_ElementType); SET(Buffer_Dimensions, Buffer_Dimensions);
  SET(Buffer_UnpaddedDimensions, Buffer_UnpaddedDimensions); SET(Buffer_DynamicDimensionIndices, Buffer_DynamicDimensionIndices);
  SET(Buffer_GetMemoryLayout, Buffer_GetMemoryLayout); SET(Buffer_OnDeviceSizeInBytes, Buffer_OnDeviceSizeInBytes);
  SET(Buffer_Device, Buffer_Device); SET(Buffer_Memory, Buffer_Memory); SET(Buffer_Delete, Buffer_Delete);
  SET(Buffer_IsDeleted, Buffer_IsDeleted); SET(Buffer_CopyToDevice, Buffer_CopyToDevice);
  SET(Buffer_ToHostBuffer, Buffer_ToHostBuffer); SET(Buffer_IsOnCpu, Buffer_IsOnCpu); SET(Buffer_ReadyEvent, Buffer_ReadyEvent);
  SET(Buffer_UnsafePointer, Buffer_UnsafePointer);
  SET(Buffer_IncreaseExternalReferenceCount, Buffer_IncreaseExternalReferenceCount);
  SET(Buffer_DecreaseExternalReferenceCount, Buffer_DecreaseExternalReferenceCount);
  SET(Buffer_OpaqueDeviceMemoryDataPointer, Buffer_OpaqueDeviceMemoryDataPointer);
  SET(CopyToDeviceStream_Destroy, CopyToDeviceStream_Destroy); SET(CopyToDeviceStream_AddChunk, CopyToDeviceStream_AddChunk);
  SET(CopyToDeviceStream_TotalBytes, CopyToDeviceStream_TotalBytes);
  SET(CopyToDeviceStream_GranuleSize, CopyToDeviceStream_GranuleSize);
  SET(CopyToDeviceStream_CurrentBytes, CopyToDeviceStream_CurrentBytes);
  SET(TopologyDescription_Create, TopologyDescription_Create); SET(TopologyDescription_Destroy, TopologyDescription_Destroy);
  SET(TopologyDescription_PlatformName, TopologyDescription_PlatformName);
  SET(TopologyDescription_PlatformVersion, TopologyDescription_PlatformVersion);
  SET(TopologyDescription_GetDeviceDescriptions, TopologyDescription_GetDeviceDescriptions);
  SET(TopologyDescription_Serialize, TopologyDescription_Serialize);
  SET(TopologyDescription_Attributes, TopologyDescription_Attributes);
  SET(Compile, Compile);
  SET(Executable_OutputElementTypes, Executable_OutputElementTypes); SET(Executable_OutputDimensions, Executable_OutputDimensions);
  SET(Buffer_CopyToMemory, Buffer_CopyToMemory); SET(Executable_Fingerprint, Executable_Fingerprint);
  SET(Client_TopologyDescription, Client_TopologyDescription);
  SET(Executable_GetCompiledMemoryStats, Executable_GetCompiledMemoryStats);
  SET(LoadedExecutable_GetDeviceAssignment, LoadedExecutable_GetDeviceAssignment);
  SET(Executable_GetCompileOptions, Executable_GetCompileOptions);
  SET(Error_ForEachPayload, Error_ForEachPayload);
  SET(TopologyDescription_Fingerprint, TopologyDescription_Fingerprint);
#undef SET
  return &api;
}

}  // namespace

extern "C" __attribute__((visibility("default"))) const PJRT_Api* GetPjrtApi(void) {
  static const PJRT_Api* api = buildApi();
  return api;
}
