/*
 * Binary interface of XLA's typed FFI, version 0.4, restated from scratch for a
 * library that is built without an XLA checkout.  Only the layout is shared
 * with XLA (struct field order, enum values, function-table order): those are
 * the ABI and cannot differ.  The interface restated is
 * xla/ffi/api/c_api.h:28-859; every struct below names the lines it mirrors.
 *
 * Inside an XLA build include "xla/ffi/api/c_api.h" *before* this file: the
 * guard below is XLA's own, so this file then contributes nothing and the
 * handlers compile against the real header.  tests/test_ffi_boundary.py
 * compares sizeof/offsetof and the enum values with the real header when an
 * XLA tree is present; tests/test_ffi_reference_headers.py registers and
 * decodes through the real api.h / ffi.h.
 */
#ifndef XLA_FFI_API_C_API_H_
#define XLA_FFI_API_C_API_H_
#define XLA_AMD_USING_RESTATED_FFI_ABI 1

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* size of a struct up to and including `last` -- what XLA stores in struct_size */
#define XLA_FFI_STRUCT_SIZE(type, last) (offsetof(type, last) + sizeof(((type*)0)->last))
#define XLA_AMD_SIZED(type, last) \
  typedef struct type type;       \
  enum { type##_STRUCT_SIZE = XLA_FFI_STRUCT_SIZE(type, last) }

#define XLA_FFI_API_MAJOR 0
#define XLA_FFI_API_MINOR 4

typedef struct XLA_FFI_Api XLA_FFI_Api;
typedef struct XLA_FFI_InternalApi XLA_FFI_InternalApi;
typedef struct XLA_FFI_Error XLA_FFI_Error;
typedef struct XLA_FFI_Future XLA_FFI_Future;
typedef struct XLA_FFI_InvokeContext XLA_FFI_InvokeContext;
typedef XLA_FFI_InvokeContext XLA_FFI_ExecutionContext;

/* ---- extension chain (c_api.h:70-110) ---- */
typedef enum { XLA_FFI_Extension_Metadata = 1 } XLA_FFI_InternalExtension_Type;

typedef struct XLA_FFI_InternalExtension {
  size_t struct_size;
  XLA_FFI_InternalExtension_Type type;
  struct XLA_FFI_InternalExtension* next;
} XLA_FFI_InternalExtension;
enum { XLA_FFI_InternalExtension_STRUCT_SIZE = XLA_FFI_STRUCT_SIZE(XLA_FFI_InternalExtension, next) };

typedef struct XLA_FFI_ExtensionId {
  int64_t extension_type;
  int32_t major_version;
  int32_t minor_version;
} XLA_FFI_ExtensionId;

typedef struct XLA_FFI_Extension XLA_FFI_Extension;
struct XLA_FFI_Extension {
  size_t struct_size;
  XLA_FFI_ExtensionId id;
  const XLA_FFI_Extension* next;
};

/* ---- version handshake (c_api.h:112-150) ---- */
struct XLA_FFI_Api_Version {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  int major_version;
  int minor_version;
};
XLA_AMD_SIZED(XLA_FFI_Api_Version, minor_version);

/* ---- errors: absl::StatusCode numbering (c_api.h:159-231) ---- */
typedef enum {
  XLA_FFI_Error_Code_OK = 0,
  XLA_FFI_Error_Code_CANCELLED = 1,
  XLA_FFI_Error_Code_UNKNOWN = 2,
  XLA_FFI_Error_Code_INVALID_ARGUMENT = 3,
  XLA_FFI_Error_Code_DEADLINE_EXCEEDED = 4,
  XLA_FFI_Error_Code_NOT_FOUND = 5,
  XLA_FFI_Error_Code_ALREADY_EXISTS = 6,
  XLA_FFI_Error_Code_PERMISSION_DENIED = 7,
  XLA_FFI_Error_Code_RESOURCE_EXHAUSTED = 8,
  XLA_FFI_Error_Code_FAILED_PRECONDITION = 9,
  XLA_FFI_Error_Code_ABORTED = 10,
  XLA_FFI_Error_Code_OUT_OF_RANGE = 11,
  XLA_FFI_Error_Code_UNIMPLEMENTED = 12,
  XLA_FFI_Error_Code_INTERNAL = 13,
  XLA_FFI_Error_Code_UNAVAILABLE = 14,
  XLA_FFI_Error_Code_DATA_LOSS = 15,
  XLA_FFI_Error_Code_UNAUTHENTICATED = 16
} XLA_FFI_Error_Code;

struct XLA_FFI_Error_Create_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  const char* message;
  XLA_FFI_Error_Code errc;
};
XLA_AMD_SIZED(XLA_FFI_Error_Create_Args, errc);
typedef XLA_FFI_Error* XLA_FFI_Error_Create(XLA_FFI_Error_Create_Args* args);

struct XLA_FFI_Error_GetDetails_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_Error* error;
  const char* message;     /* out */
  XLA_FFI_Error_Code errc; /* out */
};
XLA_AMD_SIZED(XLA_FFI_Error_GetDetails_Args, errc);
typedef void XLA_FFI_Error_GetDetails(XLA_FFI_Error_GetDetails_Args* args);

struct XLA_FFI_Error_Destroy_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_Error* error;
};
XLA_AMD_SIZED(XLA_FFI_Error_Destroy_Args, error);
typedef void XLA_FFI_Error_Destroy(XLA_FFI_Error_Destroy_Args* args);

/* ---- element types: equal to xla::PrimitiveType (c_api.h:233-266) ---- */
typedef enum {
  XLA_FFI_DataType_INVALID = 0,
  XLA_FFI_DataType_PRED = 1,
  XLA_FFI_DataType_S8 = 2,
  XLA_FFI_DataType_S16 = 3,
  XLA_FFI_DataType_S32 = 4,
  XLA_FFI_DataType_S64 = 5,
  XLA_FFI_DataType_U8 = 6,
  XLA_FFI_DataType_U16 = 7,
  XLA_FFI_DataType_U32 = 8,
  XLA_FFI_DataType_U64 = 9,
  XLA_FFI_DataType_F16 = 10,
  XLA_FFI_DataType_F32 = 11,
  XLA_FFI_DataType_F64 = 12,
  XLA_FFI_DataType_C64 = 15,
  XLA_FFI_DataType_BF16 = 16,
  XLA_FFI_DataType_TOKEN = 17,
  XLA_FFI_DataType_C128 = 18,
  XLA_FFI_DataType_F8E5M2 = 19,
  XLA_FFI_DataType_F8E4M3FN = 20,
  XLA_FFI_DataType_S4 = 21,
  XLA_FFI_DataType_U4 = 22,
  XLA_FFI_DataType_F8E4M3B11FNUZ = 23,
  XLA_FFI_DataType_F8E5M2FNUZ = 24,
  XLA_FFI_DataType_F8E4M3FNUZ = 25,
  XLA_FFI_DataType_S2 = 26,
  XLA_FFI_DataType_U2 = 27,
  XLA_FFI_DataType_F8E4M3 = 28,
  XLA_FFI_DataType_F8E3M4 = 29,
  XLA_FFI_DataType_S1 = 30,
  XLA_FFI_DataType_U1 = 31,
  XLA_FFI_DataType_F4E2M1FN = 32,
  XLA_FFI_DataType_F8E8M0FNU = 33
} XLA_FFI_DataType;

/* ---- operands (c_api.h:268-345) ---- */
struct XLA_FFI_Buffer {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_DataType dtype;
  void* data;    /* device pointer; sub-byte types are packed */
  int64_t rank;
  int64_t* dims; /* logical HLO dimensions, no strides */
};
XLA_AMD_SIZED(XLA_FFI_Buffer, dims);

typedef enum { XLA_FFI_ArgType_BUFFER = 1 } XLA_FFI_ArgType;
typedef enum { XLA_FFI_RetType_BUFFER = 1 } XLA_FFI_RetType;

typedef enum {
  XLA_FFI_AttrType_ARRAY = 1,
  XLA_FFI_AttrType_DICTIONARY = 2,
  XLA_FFI_AttrType_SCALAR = 3,
  XLA_FFI_AttrType_STRING = 4
} XLA_FFI_AttrType;

typedef struct XLA_FFI_ByteSpan {
  const char* ptr;
  size_t len;
} XLA_FFI_ByteSpan;

typedef struct XLA_FFI_Scalar {
  XLA_FFI_DataType dtype;
  void* value;
} XLA_FFI_Scalar;

typedef struct XLA_FFI_Array {
  XLA_FFI_DataType dtype;
  size_t size;
  void* data;
} XLA_FFI_Array;

typedef struct XLA_FFI_TypeId {
  int64_t type_id;
} XLA_FFI_TypeId;

typedef struct XLA_FFI_TypeInfo {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  void (*deleter)(void* object);
} XLA_FFI_TypeInfo;

/* ---- async results (c_api.h:380-420); unused by this library ---- */
struct XLA_FFI_Future_Create_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_Future* future;
};
typedef struct XLA_FFI_Future_Create_Args XLA_FFI_Future_Create_Args;
typedef XLA_FFI_Error* XLA_FFI_Future_Create(XLA_FFI_Future_Create_Args* args);
struct XLA_FFI_Future_SetAvailable_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_Future* future;
};
typedef struct XLA_FFI_Future_SetAvailable_Args XLA_FFI_Future_SetAvailable_Args;
typedef XLA_FFI_Error* XLA_FFI_Future_SetAvailable(XLA_FFI_Future_SetAvailable_Args* args);
struct XLA_FFI_Future_SetError_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_Future* future;
  XLA_FFI_Error* error;
};
typedef struct XLA_FFI_Future_SetError_Args XLA_FFI_Future_SetError_Args;
typedef XLA_FFI_Error* XLA_FFI_Future_SetError(XLA_FFI_Future_SetError_Args* args);

/* ---- call frame (c_api.h:449-517) ---- */
typedef enum {
  XLA_FFI_ExecutionStage_INSTANTIATE = 0,
  XLA_FFI_ExecutionStage_PREPARE = 1,
  XLA_FFI_ExecutionStage_INITIALIZE = 2,
  XLA_FFI_ExecutionStage_EXECUTE = 3,
  XLA_FFI_ExecutionStage_RECORD = 4
} XLA_FFI_ExecutionStage;

struct XLA_FFI_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  int64_t size;
  XLA_FFI_ArgType* types;
  void** args;
};
XLA_AMD_SIZED(XLA_FFI_Args, args);

struct XLA_FFI_Rets {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  int64_t size;
  XLA_FFI_RetType* types;
  void** rets;
};
XLA_AMD_SIZED(XLA_FFI_Rets, rets);

/* names are sorted; attrs[i] points at XLA_FFI_Scalar / XLA_FFI_ByteSpan /
 * XLA_FFI_Array / XLA_FFI_Attrs according to types[i] */
struct XLA_FFI_Attrs {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  int64_t size;
  XLA_FFI_AttrType* types;
  XLA_FFI_ByteSpan** names;
  void** attrs;
};
XLA_AMD_SIZED(XLA_FFI_Attrs, attrs);

struct XLA_FFI_CallFrame {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  const XLA_FFI_Api* api;
  XLA_FFI_InvokeContext* ctx;
  XLA_FFI_ExecutionStage stage;
  XLA_FFI_Args args;
  XLA_FFI_Rets rets;
  XLA_FFI_Attrs attrs;
  XLA_FFI_Future* future; /* out; not counted in struct_size */
};
XLA_AMD_SIZED(XLA_FFI_CallFrame, attrs);

typedef XLA_FFI_Error* XLA_FFI_Handler(XLA_FFI_CallFrame* call_frame);

/* ---- registration (c_api.h:519-560) ---- */
typedef struct XLA_FFI_Handler_Bundle {
  XLA_FFI_Handler* instantiate;
  XLA_FFI_Handler* prepare;
  XLA_FFI_Handler* initialize;
  XLA_FFI_Handler* execute; /* the only required one */
  XLA_FFI_Handler* record;
} XLA_FFI_Handler_Bundle;

enum XLA_FFI_Handler_TraitsBits { XLA_FFI_HANDLER_TRAITS_COMMAND_BUFFER_COMPATIBLE = 1u << 0 };
typedef uint32_t XLA_FFI_Handler_Traits;

struct XLA_FFI_Handler_Register_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_ByteSpan name;
  XLA_FFI_ByteSpan platform;
  XLA_FFI_Handler_Bundle bundle;
  XLA_FFI_Handler_Traits traits;
};
XLA_AMD_SIZED(XLA_FFI_Handler_Register_Args, traits);
typedef XLA_FFI_Error* XLA_FFI_Handler_Register(XLA_FFI_Handler_Register_Args* args);

struct XLA_FFI_Type_Register_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_ByteSpan name;
  XLA_FFI_TypeId* type_id;
  const XLA_FFI_TypeInfo* type_info;
};
typedef struct XLA_FFI_Type_Register_Args XLA_FFI_Type_Register_Args;
typedef XLA_FFI_Error* XLA_FFI_Type_Register(XLA_FFI_Type_Register_Args* args);

/* ---- context services (c_api.h:580-790) ---- */
struct XLA_FFI_InvokeContext_FindExtension_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  int64_t extension_type;
  const XLA_FFI_Extension* extension;
};
typedef struct XLA_FFI_InvokeContext_FindExtension_Args XLA_FFI_InvokeContext_FindExtension_Args;
typedef XLA_FFI_Error* XLA_FFI_InvokeContext_FindExtension(
    XLA_FFI_InvokeContext_FindExtension_Args* args);

struct XLA_FFI_InvokeContext_Get_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  XLA_FFI_TypeId* type_id;
  void* data;
};
typedef struct XLA_FFI_InvokeContext_Get_Args XLA_FFI_InvokeContext_Get_Args;
typedef XLA_FFI_Error* XLA_FFI_InvokeContext_Get(XLA_FFI_InvokeContext_Get_Args* args);

struct XLA_FFI_State_Set_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  XLA_FFI_ExecutionStage stage;
  XLA_FFI_TypeId* type_id;
  void* state;
};
typedef struct XLA_FFI_State_Set_Args XLA_FFI_State_Set_Args;
typedef XLA_FFI_Error* XLA_FFI_State_Set(XLA_FFI_State_Set_Args* args);

struct XLA_FFI_State_Get_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  XLA_FFI_ExecutionStage stage;
  XLA_FFI_TypeId* type_id;
  void* state;
};
typedef struct XLA_FFI_State_Get_Args XLA_FFI_State_Get_Args;
typedef XLA_FFI_Error* XLA_FFI_State_Get(XLA_FFI_State_Get_Args* args);

/* the platform stream the custom call must enqueue on: hipStream_t on ROCm */
struct XLA_FFI_Stream_Get_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  void* stream; /* out */
};
XLA_AMD_SIZED(XLA_FFI_Stream_Get_Args, stream);
typedef XLA_FFI_Error* XLA_FFI_Stream_Get(XLA_FFI_Stream_Get_Args* args);

struct XLA_FFI_DeviceMemory_Allocate_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  size_t size;
  size_t alignment;
  void* data; /* out */
};
XLA_AMD_SIZED(XLA_FFI_DeviceMemory_Allocate_Args, data);
typedef XLA_FFI_Error* XLA_FFI_DeviceMemory_Allocate(XLA_FFI_DeviceMemory_Allocate_Args* args);

struct XLA_FFI_DeviceMemory_Free_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  size_t size;
  void* data;
};
XLA_AMD_SIZED(XLA_FFI_DeviceMemory_Free_Args, data);
typedef XLA_FFI_Error* XLA_FFI_DeviceMemory_Free(XLA_FFI_DeviceMemory_Free_Args* args);

typedef void XLA_FFI_Task(void* data);
struct XLA_FFI_ThreadPool_Schedule_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  XLA_FFI_Task* task;
  void* data;
};
typedef struct XLA_FFI_ThreadPool_Schedule_Args XLA_FFI_ThreadPool_Schedule_Args;
typedef XLA_FFI_Error* XLA_FFI_ThreadPool_Schedule(XLA_FFI_ThreadPool_Schedule_Args* args);

struct XLA_FFI_ThreadPool_NumThreads_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  int64_t* num_threads;
};
typedef struct XLA_FFI_ThreadPool_NumThreads_Args XLA_FFI_ThreadPool_NumThreads_Args;
typedef XLA_FFI_Error* XLA_FFI_ThreadPool_NumThreads(XLA_FFI_ThreadPool_NumThreads_Args* args);

struct XLA_FFI_RunId_Get_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  int64_t run_id;
};
typedef struct XLA_FFI_RunId_Get_Args XLA_FFI_RunId_Get_Args;
typedef XLA_FFI_Error* XLA_FFI_RunId_Get(XLA_FFI_RunId_Get_Args* args);

struct XLA_FFI_DeviceOrdinal_Get_Args {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  XLA_FFI_InvokeContext* ctx;
  int32_t device_ordinal;
};
XLA_AMD_SIZED(XLA_FFI_DeviceOrdinal_Get_Args, device_ordinal);
typedef XLA_FFI_Error* XLA_FFI_DeviceOrdinal_Get(XLA_FFI_DeviceOrdinal_Get_Args* args);

/* ---- metadata query answered by every handler (c_api.h:795-813) ---- */
struct XLA_FFI_Metadata {
  size_t struct_size;
  struct XLA_FFI_Api_Version api_version;
  XLA_FFI_Handler_Traits traits;
  XLA_FFI_TypeId state_type_id;
};
XLA_AMD_SIZED(XLA_FFI_Metadata, traits);

struct XLA_FFI_Metadata_Extension {
  XLA_FFI_InternalExtension extension_base;
  XLA_FFI_Metadata* metadata;
};
XLA_AMD_SIZED(XLA_FFI_Metadata_Extension, metadata);

/* ---- function table handed to the handler in every call frame (c_api.h:821-851) ---- */
struct XLA_FFI_Api {
  size_t struct_size;
  XLA_FFI_InternalExtension* extension_start;
  struct XLA_FFI_Api_Version api_version;
  const XLA_FFI_InternalApi* internal_api;
  XLA_FFI_Error_Create* XLA_FFI_Error_Create;
  XLA_FFI_Error_GetDetails* XLA_FFI_Error_GetDetails;
  XLA_FFI_Error_Destroy* XLA_FFI_Error_Destroy;
  XLA_FFI_Handler_Register* XLA_FFI_Handler_Register;
  XLA_FFI_Stream_Get* XLA_FFI_Stream_Get;
  XLA_FFI_Type_Register* XLA_FFI_Type_Register;
  XLA_FFI_InvokeContext_Get* XLA_FFI_InvokeContext_Get;
  XLA_FFI_State_Set* XLA_FFI_State_Set;
  XLA_FFI_State_Get* XLA_FFI_State_Get;
  XLA_FFI_DeviceMemory_Allocate* XLA_FFI_DeviceMemory_Allocate;
  XLA_FFI_DeviceMemory_Free* XLA_FFI_DeviceMemory_Free;
  XLA_FFI_ThreadPool_Schedule* XLA_FFI_ThreadPool_Schedule;
  XLA_FFI_ThreadPool_NumThreads* XLA_FFI_ThreadPool_NumThreads;
  XLA_FFI_Future_Create* XLA_FFI_Future_Create;
  XLA_FFI_Future_SetAvailable* XLA_FFI_Future_SetAvailable;
  XLA_FFI_Future_SetError* XLA_FFI_Future_SetError;
  XLA_FFI_RunId_Get* XLA_FFI_RunId_Get;
  XLA_FFI_DeviceOrdinal_Get* XLA_FFI_DeviceOrdinal_Get;
  XLA_FFI_InvokeContext_FindExtension* XLA_FFI_InvokeContext_FindExtension;
};
enum { XLA_FFI_Api_STRUCT_SIZE = XLA_FFI_STRUCT_SIZE(struct XLA_FFI_Api, XLA_FFI_InvokeContext_FindExtension) };

#ifdef __cplusplus
}
#endif
#endif /* XLA_FFI_API_C_API_H_ */
