// Native side of the FFI host: replays prepared call frames without going back to Python
// between calls, the way a thunk sequence re-invokes a custom call every step with only the
// buffer pointers changing (xla/backends/gpu/runtime/custom_call_thunk.cc:305-336,546-575).
#include <stddef.h>
#include <stdint.h>
#include <string.h>
#include <ctype.h>

#include "xla_ffi_abi.h"

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
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

struct XLA_FFI_Error {
  XLA_FFI_Error_Code code;
  std::string message;
};

namespace {

struct Registration {
  std::string name, platform;
  XLA_FFI_Handler_Bundle bundle;
  XLA_FFI_Handler_Traits traits;
};

struct HostState {
  XLA_FFI_Api api;
  void* stream = nullptr;
  std::vector<Registration> registry;
};

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
HostState* g_registering = nullptr;  // Handler_Register carries no ctx; set around the call
XLA_FFI_Error* HandlerRegister(XLA_FFI_Handler_Register_Args* a) {
  if (!g_registering) return new XLA_FFI_Error{XLA_FFI_Error_Code_FAILED_PRECONDITION, "no host is registering"};
  if (!a->bundle.execute) return new XLA_FFI_Error{XLA_FFI_Error_Code_INVALID_ARGUMENT, "execute handler is required"};
  Registration r{std::string(a->name.ptr, a->name.len), std::string(a->platform.ptr, a->platform.len), a->bundle, a->traits};
  for (char& c : r.platform) c = (char)tolower(c);
  g_registering->registry.push_back(r);
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
  t.XLA_FFI_InvokeContext_FindExtension = Unimplemented<XLA_FFI_InvokeContext_FindExtension_Args>;
  return h;
}

HOST_EXPORT void xla_amd_host_destroy(void* host) { delete reinterpret_cast<HostState*>(host); }
HOST_EXPORT const XLA_FFI_Api* xla_amd_host_api(void* host) { return &reinterpret_cast<HostState*>(host)->api; }
HOST_EXPORT void xla_amd_host_set_stream(void* host, void* stream) { reinterpret_cast<HostState*>(host)->stream = stream; }

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

// Runs `register_fn(api)` (e.g. xla_amd_register_handlers) against this host's registry.
HOST_EXPORT XLA_FFI_Error* xla_amd_host_register(void* host, XLA_FFI_Error* (*register_fn)(const XLA_FFI_Api*)) {
  static std::mutex mu;
  std::lock_guard<std::mutex> lock(mu);
  g_registering = reinterpret_cast<HostState*>(host);
  XLA_FFI_Error* e = register_fn(&g_registering->api);
  g_registering = nullptr;
  return e;
}

// Looks a handler up by (target, platform) the way the registry does (xla/ffi/ffi_registry.cc:160-175).
HOST_EXPORT XLA_FFI_Handler* xla_amd_host_find_handler(void* host, const char* name, const char* platform) {
  for (const Registration& r : reinterpret_cast<HostState*>(host)->registry)
    if (r.name == name && r.platform == platform) return r.bundle.execute;
  return nullptr;
}
