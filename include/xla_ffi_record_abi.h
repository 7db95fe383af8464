/*
 * The part of XLA's FFI record extension (xla/ffi/api/record_c_api.h:40-222, extension version
 * 0.1) that a handler needs in order to answer the RECORD stage by asking for stream capture:
 * the extension id, the record function table (order is the ABI), the record frame and the
 * extension struct.  Layout only; restated from scratch like xla_ffi_abi.h, whose guard
 * convention it follows: inside an XLA build include "xla/ffi/api/record_c_api.h" first and this
 * file contributes nothing.
 */
#ifndef XLA_FFI_API_RECORD_C_API_H_
#define XLA_FFI_API_RECORD_C_API_H_

#include <stddef.h>
#include <stdint.h>

#include "xla_ffi_abi.h"

#ifdef __cplusplus
extern "C" {
#endif

#define XLA_FFI_Extension_Record 128 /* record_c_api.h:43 */
#define XLA_FFI_Extension_Record_MajorVersion 0
#define XLA_FFI_Extension_Record_MinorVersion 1

typedef struct XLA_FFI_RecordContext XLA_FFI_RecordContext; /* opaque, record_c_api.h:54 */
typedef struct XLA_FFI_Command XLA_FFI_Command;             /* opaque, record_c_api.h:58 */

typedef enum XLA_FFI_RecordAction { /* record_c_api.h:60-63 */
  XLA_FFI_RecordAction_Create = 0,
  XLA_FFI_RecordAction_Update = 1,
} XLA_FFI_RecordAction;

typedef enum XLA_FFI_SourceFormat { XLA_FFI_SourceFormat_PTX = 0, XLA_FFI_SourceFormat_CUBIN = 1 } XLA_FFI_SourceFormat;
typedef struct XLA_FFI_Dim3 { int32_t x, y, z; } XLA_FFI_Dim3;
typedef struct XLA_FFI_LaunchDims { XLA_FFI_Dim3 grid, block, cluster; } XLA_FFI_LaunchDims;
typedef enum XLA_FFI_KernelArgType { XLA_FFI_KernelArgType_DevicePtr = 0, XLA_FFI_KernelArgType_HostValue = 1 } XLA_FFI_KernelArgType;
typedef struct XLA_FFI_KernelArg {
  const void* arg_address;
  int64_t size;
  XLA_FFI_KernelArgType type;
} XLA_FFI_KernelArg;
typedef struct XLA_FFI_KernelArgs {
  const XLA_FFI_KernelArg* args;
  int64_t num_args;
} XLA_FFI_KernelArgs;

/* record_c_api.h:142-198: six entries, in this order */
typedef struct XLA_FFI_RecordApi {
  XLA_FFI_Error* (*create_launch)(XLA_FFI_RecordContext* ctx, const char* kernel_name, const void* kernel_data,
                                  int64_t kernel_size, XLA_FFI_SourceFormat format, XLA_FFI_LaunchDims launch_dims,
                                  uint32_t shared_mem_bytes, int32_t uses_pdl, const XLA_FFI_KernelArgs* args,
                                  const XLA_FFI_Command* const* dependencies, uint32_t num_dependencies,
                                  const XLA_FFI_Command** out_command);
  XLA_FFI_Error* (*update_launch)(XLA_FFI_RecordContext* ctx, const XLA_FFI_Command* command,
                                  const XLA_FFI_KernelArgs* args);
  XLA_FFI_Error* (*create_memcpy_d2d)(XLA_FFI_RecordContext* ctx, void* dst, void* src, int64_t size,
                                      const XLA_FFI_Command* const* dependencies, uint32_t num_dependencies,
                                      const XLA_FFI_Command** out_command);
  XLA_FFI_Error* (*update_memcpy_d2d)(XLA_FFI_RecordContext* ctx, const XLA_FFI_Command* command, void* dst,
                                      void* src, int64_t size);
  XLA_FFI_Error* (*request_stream_capture)(XLA_FFI_RecordContext* ctx);
  XLA_FFI_Error* (*create_empty_command)(XLA_FFI_RecordContext* ctx, const XLA_FFI_Command* const* dependencies,
                                         uint32_t num_dependencies, const XLA_FFI_Command** out_command);
} XLA_FFI_RecordApi;

typedef struct XLA_FFI_RecordFrame { /* record_c_api.h:205-212 */
  XLA_FFI_RecordContext* record_ctx;
  const XLA_FFI_RecordApi* api;
  XLA_FFI_RecordAction action;
  const XLA_FFI_Command** commands;
  int64_t* num_commands;
  int64_t max_commands;
} XLA_FFI_RecordFrame;

typedef struct XLA_FFI_Record_Extension { /* record_c_api.h:215-218 */
  XLA_FFI_Extension extension_base;
  XLA_FFI_RecordFrame* record_frame;
} XLA_FFI_Record_Extension;
enum { XLA_FFI_Record_Extension_STRUCT_SIZE = XLA_FFI_STRUCT_SIZE(XLA_FFI_Record_Extension, record_frame) };

#ifdef __cplusplus
}
#endif
#endif /* XLA_FFI_API_RECORD_C_API_H_ */
