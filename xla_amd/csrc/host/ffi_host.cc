// Native side of the FFI host: replays prepared call frames without going back to Python
// between calls, the way a thunk sequence re-invokes a custom call every step with only the
// buffer pointers changing (xla/backends/gpu/runtime/custom_call_thunk.cc:305-336,546-575).
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include <ctype.h>

#include "xla_ffi_abi.h"
#include "xla_ffi_record_abi.h"

#define HOST_EXPORT extern "C" __attribute__((visibility("default")))

// Calls handlers[i](frames[i]) for i in [0, n), `rounds` times over.  Stops at the first error
// and returns it (the caller owns it, as XLA would); *failed_at receives round*n + i.
HOST_EXPORT XLA_FFI_Error* xla_amd_host_replay(XLA_FFI_Handler* const* handlers,
                                               XLA_FFI_CallFrame* const* frames, int64_t n,
                                               int64_t rounds, int64_t* failed_at) {
  for (int64_t r = 0; r < rounds; ++r) {
    for (int64_t i = 0; i < n; ++i) {
      if (XLA_FFI_Error* e = handlers[i](frames[i])) {
        if (failed_at) *failed_at = r * n + i;
        return e;
      }
    }
  }
  if (failed_at) *failed_at = -1;
  return nullptr;
}

// ---- a native XLA_FFI_Api table: what xla/ffi/ffi_api.cc:668-706 provides inside XLA, reduced
// to what the handlers of this library call (errors, stream, registration).
#include <stdarg.h>
#include <stdio.h>

#include <map>
#include <mutex>
#include <string>
#include <utility>

struct XLA_FFI_Error {
  XLA_FFI_Error_Code code;
  std::string message;
};

namespace {

struct Registration {
  XLA_FFI_Metadata metadata;
  XLA_FFI_Handler_Bundle bundle;
};

// One registry per process, keyed by (target, canonical platform), like the static handler map
// of xla/ffi/ffi_registry.cc:40-43: XLA_FFI_Handler_Register carries no context, and handlers
// registered from static initialisers (XLA_FFI_REGISTER_HANDLER) must land somewhere.
struct Registry {
  std::mutex mu;
  std::map<std::pair<std::string, std::string>, Registration> map;
};
Registry& StaticRegistry() {
  static Registry* r = new Registry();
  return *r;
}

struct HostState {
  XLA_FFI_Api api;
  void* stream = nullptr;
  // what a command-buffer recording attaches to the invoke context (custom_call_thunk.cc:610-618):
  // a record extension whose function table only implements request_stream_capture
  XLA_FFI_RecordApi record_api{};
  XLA_FFI_RecordFrame record_frame{};
  XLA_FFI_Record_Extension record_extension{};
  bool recording = false;
  int stream_capture_requests = 0;
};

// xla/service/platform_util.cc:64-91 as a ROCm build resolves it.
std::string CanonicalPlatformName(std::string platform) {
  for (char& c : platform) c = (char)tolower((unsigned char)c);
  if (platform == "cpu") return "host";
  if (platform == "gpu") return "rocm";
  if (platform == "oneapi") return "sycl";
  return platform;
}

XLA_FFI_Error* InvalidArgument(const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  return new XLA_FFI_Error{XLA_FFI_Error_Code_INVALID_ARGUMENT, buf};
}

// ctx of every frame built for this host points at the HostState
XLA_FFI_Error* ErrorCreate(XLA_FFI_Error_Create_Args* a) { return new XLA_FFI_Error{a->errc, a->message}; }
void ErrorGetDetails(XLA_FFI_Error_GetDetails_Args* a) {
  a->message = a->error->message.c_str();
  a->errc = a->error->code;
}
void ErrorDestroy(XLA_FFI_Error_Destroy_Args* a) { delete a->error; }
XLA_FFI_Error* StreamGet(XLA_FFI_Stream_Get_Args* a) {
  if (!a->ctx) return new XLA_FFI_Error{XLA_FFI_Error_Code_INVALID_ARGUMENT, "XLA FFI GPU context is not available"};
  a->stream = reinterpret_cast<HostState*>(a->ctx)->stream;
  return nullptr;
}

XLA_FFI_Error* FindExtension(XLA_FFI_InvokeContext_FindExtension_Args* a) {
  a->extension = nullptr;
  if (!a->ctx) return new XLA_FFI_Error{XLA_FFI_Error_Code_INVALID_ARGUMENT, "no invoke context"};
  HostState* h = reinterpret_cast<HostState*>(a->ctx);
  if (h->recording && a->extension_type == XLA_FFI_Extension_Record) a->extension = &h->record_extension.extension_base;
  return nullptr;  // not found: a null extension, no error (ffi_api.cc XLA_FFI_InvokeContext_FindExtension)
}
XLA_FFI_Error* RequestStreamCapture(XLA_FFI_RecordContext* ctx) {
  ++reinterpret_cast<HostState*>(ctx)->stream_capture_requests;
  return nullptr;
}

// The registration-time handshake of xla/ffi/invoke.cc:174-233: a call frame that carries nothing
// but a metadata extension; the handler fills in the API version it was built against and its
// traits and returns without doing any work.
XLA_FFI_Error* GetMetadata(const XLA_FFI_Api* api, XLA_FFI_Handler* handler, XLA_FFI_Metadata* metadata) {
  *metadata = XLA_FFI_Metadata{};
  metadata->struct_size = XLA_FFI_Metadata_STRUCT_SIZE;
  metadata->api_version.struct_size = XLA_FFI_Api_Version_STRUCT_SIZE;
  XLA_FFI_Metadata_Extension ext{};
  ext.extension_base.struct_size = XLA_FFI_Metadata_Extension_STRUCT_SIZE;
  ext.extension_base.type = XLA_FFI_Extension_Metadata;
  ext.metadata = metadata;
  XLA_FFI_CallFrame frame{};
  frame.struct_size = XLA_FFI_CallFrame_STRUCT_SIZE;
  frame.extension_start = &ext.extension_base;
  frame.api = api;
  frame.ctx = nullptr;
  frame.stage = XLA_FFI_ExecutionStage_EXECUTE;
  frame.args.struct_size = XLA_FFI_Args_STRUCT_SIZE;
  frame.rets.struct_size = XLA_FFI_Rets_STRUCT_SIZE;
  frame.attrs.struct_size = XLA_FFI_Attrs_STRUCT_SIZE;
  return (*handler)(&frame);
}

bool SameMetadata(const XLA_FFI_Metadata& a, const XLA_FFI_Metadata& b) {
  return a.api_version.major_version == b.api_version.major_version &&
         a.api_version.minor_version == b.api_version.minor_version && a.traits == b.traits &&
         a.state_type_id.type_id == b.state_type_id.type_id;
}
bool SameBundle(const XLA_FFI_Handler_Bundle& a, const XLA_FFI_Handler_Bundle& b) {
  return a.instantiate == b.instantiate && a.prepare == b.prepare && a.initialize == b.initialize &&
         a.execute == b.execute && a.record == b.record;
}

const XLA_FFI_Api* g_registering_api = nullptr;  // the table handed to the metadata query

// RegisterHandler of xla/ffi/ffi_registry.cc:87-158, rule for rule: canonical platform, an execute
// stage is required, the handler's API version must lie in [0.1, this API's], explicit traits are
// OR-ed into the handler's own, and a second registration of the same key is accepted only when it
// is the very same handler with the same metadata.
XLA_FFI_Error* HandlerRegister(XLA_FFI_Handler_Register_Args* a) {
  const std::string name(a->name.ptr, a->name.len), platform(a->platform.ptr, a->platform.len);
  const std::string canonical = CanonicalPlatformName(platform);
  if (!a->bundle.execute)
    return InvalidArgument("FFI handler for %s on a platform %s must provide an execute implementation",
                           name.c_str(), platform.c_str());
  XLA_FFI_Metadata metadata;
  if (XLA_FFI_Error* e = GetMetadata(g_registering_api, a->bundle.execute, &metadata)) return e;
  const std::pair<int, int> version{metadata.api_version.major_version, metadata.api_version.minor_version};
  const std::pair<int, int> lo{0, 1}, hi{XLA_FFI_API_MAJOR, XLA_FFI_API_MINOR};
  if (version < lo || version > hi)
    return InvalidArgument(
        "XLA FFI handler registration for %s on platform %s (canonical %s) failed because the handler's API "
        "version (%d.%d) is incompatible with the framework's API version (%d.%d). Minimum supported API "
        "version is (%d.%d).",
        name.c_str(), platform.c_str(), canonical.c_str(), version.first, version.second, hi.first, hi.second,
        lo.first, lo.second);
  metadata.traits |= a->traits;
  if (a->bundle.instantiate) {
    XLA_FFI_Metadata im;
    if (XLA_FFI_Error* e = GetMetadata(g_registering_api, a->bundle.instantiate, &im)) return e;
    metadata.state_type_id = im.state_type_id;
  }
  Registry& reg = StaticRegistry();
  std::lock_guard<std::mutex> lock(reg.mu);
  auto [it, emplaced] = reg.map.try_emplace({name, canonical}, Registration{metadata, a->bundle});
  if (!emplaced) {
    if (!SameMetadata(it->second.metadata, metadata))
      return InvalidArgument("Duplicate FFI handler registration for %s on platform %s (canonical %s) with different metadata",
                             name.c_str(), platform.c_str(), canonical.c_str());
    if (!SameBundle(it->second.bundle, a->bundle))
      return InvalidArgument("Duplicate FFI handler registration for %s on platform %s (canonical %s) with different bundle addresses",
                             name.c_str(), platform.c_str(), canonical.c_str());
  }
  return nullptr;
}
template <typename Args>
XLA_FFI_Error* Unimplemented(Args*) {
  return new XLA_FFI_Error{XLA_FFI_Error_Code_UNIMPLEMENTED, "not implemented by this host"};
}

}  // namespace

HOST_EXPORT void* xla_amd_host_create(void) {
  HostState* h = new HostState();
  XLA_FFI_Api& t = h->api;
  t.struct_size = XLA_FFI_Api_STRUCT_SIZE;
  t.extension_start = nullptr;
  t.api_version = XLA_FFI_Api_Version{XLA_FFI_Api_Version_STRUCT_SIZE, nullptr, XLA_FFI_API_MAJOR, XLA_FFI_API_MINOR};
  t.internal_api = nullptr;
  t.XLA_FFI_Error_Create = ErrorCreate;
  t.XLA_FFI_Error_GetDetails = ErrorGetDetails;
  t.XLA_FFI_Error_Destroy = ErrorDestroy;
  t.XLA_FFI_Handler_Register = HandlerRegister;
  t.XLA_FFI_Stream_Get = StreamGet;
  t.XLA_FFI_Type_Register = Unimplemented<XLA_FFI_Type_Register_Args>;
  t.XLA_FFI_InvokeContext_Get = Unimplemented<XLA_FFI_InvokeContext_Get_Args>;
  t.XLA_FFI_State_Set = Unimplemented<XLA_FFI_State_Set_Args>;
  t.XLA_FFI_State_Get = Unimplemented<XLA_FFI_State_Get_Args>;
  t.XLA_FFI_DeviceMemory_Allocate = Unimplemented<XLA_FFI_DeviceMemory_Allocate_Args>;
  t.XLA_FFI_DeviceMemory_Free = Unimplemented<XLA_FFI_DeviceMemory_Free_Args>;
  t.XLA_FFI_ThreadPool_Schedule = Unimplemented<XLA_FFI_ThreadPool_Schedule_Args>;
  t.XLA_FFI_ThreadPool_NumThreads = Unimplemented<XLA_FFI_ThreadPool_NumThreads_Args>;
  t.XLA_FFI_Future_Create = Unimplemented<XLA_FFI_Future_Create_Args>;
  t.XLA_FFI_Future_SetAvailable = Unimplemented<XLA_FFI_Future_SetAvailable_Args>;
  t.XLA_FFI_Future_SetError = Unimplemented<XLA_FFI_Future_SetError_Args>;
  t.XLA_FFI_RunId_Get = Unimplemented<XLA_FFI_RunId_Get_Args>;
  t.XLA_FFI_DeviceOrdinal_Get = Unimplemented<XLA_FFI_DeviceOrdinal_Get_Args>;
  t.XLA_FFI_InvokeContext_FindExtension = FindExtension;
  h->record_api.request_stream_capture = RequestStreamCapture;
  h->record_frame.record_ctx = reinterpret_cast<XLA_FFI_RecordContext*>(h);
  h->record_frame.api = &h->record_api;
  h->record_frame.action = XLA_FFI_RecordAction_Create;
  h->record_extension.extension_base.struct_size = XLA_FFI_Record_Extension_STRUCT_SIZE;
  h->record_extension.extension_base.id =
      XLA_FFI_ExtensionId{XLA_FFI_Extension_Record, XLA_FFI_Extension_Record_MajorVersion, XLA_FFI_Extension_Record_MinorVersion};
  h->record_extension.extension_base.next = nullptr;
  h->record_extension.record_frame = &h->record_frame;
  if (!g_registering_api) g_registering_api = &h->api;  // any host's table serves the metadata query
  return h;
}

HOST_EXPORT void xla_amd_host_destroy(void* host) { delete reinterpret_cast<HostState*>(host); }
HOST_EXPORT const XLA_FFI_Api* xla_amd_host_api(void* host) { return &reinterpret_cast<HostState*>(host)->api; }
HOST_EXPORT void xla_amd_host_set_stream(void* host, void* stream) { reinterpret_cast<HostState*>(host)->stream = stream; }

// While `on`, frames of this host find a record extension on their invoke context, as a custom call
// finds one while XLA records it into a command buffer.  Returns how often a handler has asked
// for stream capture so far.
HOST_EXPORT int xla_amd_host_set_recording(void* host, int on) {
  HostState* h = reinterpret_cast<HostState*>(host);
  h->recording = on != 0;
  return h->stream_capture_requests;
}

// Copies the error's message into buf (NUL-terminated), destroys it and returns its code.
HOST_EXPORT int xla_amd_host_take_error(XLA_FFI_Error* err, char* buf, size_t n) {
  if (!err) return 0;
  int code = err->code;
  if (buf && n) {
    size_t len = err->message.size() < n - 1 ? err->message.size() : n - 1;
    memcpy(buf, err->message.data(), len);
    buf[len] = 0;
  }
  delete err;
  return code;
}

// Runs `register_fn(api)` (e.g. xla_amd_register_handlers) against the process-wide registry.
HOST_EXPORT XLA_FFI_Error* xla_amd_host_register(void* host, XLA_FFI_Error* (*register_fn)(const XLA_FFI_Api*)) {
  return register_fn(&reinterpret_cast<HostState*>(host)->api);
}

// Looks a handler up by (target, platform) the way the registry does (xla/ffi/ffi_registry.cc:160-186):
// the platform name is canonicalised first.  Returns the execute stage, or null.
HOST_EXPORT XLA_FFI_Handler* xla_amd_host_find_handler(void* host, const char* name, const char* platform) {
  (void)host;
  Registry& reg = StaticRegistry();
  std::lock_guard<std::mutex> lock(reg.mu);
  auto it = reg.map.find({name, CanonicalPlatformName(platform)});
  return it == reg.map.end() ? nullptr : it->second.bundle.execute;
}

// Traits the registry holds for a handler (its own OR-ed with those given at registration), -1 if
// it is not registered.
HOST_EXPORT int64_t xla_amd_host_handler_traits(void* host, const char* name, const char* platform) {
  (void)host;
  Registry& reg = StaticRegistry();
  std::lock_guard<std::mutex> lock(reg.mu);
  auto it = reg.map.find({name, CanonicalPlatformName(platform)});
  return it == reg.map.end() ? -1 : (int64_t)it->second.metadata.traits;
}
