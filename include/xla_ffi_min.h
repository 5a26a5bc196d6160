/*
 * xla_ffi_min.h — the part of XLA's typed-FFI C ABI (xla/ffi/api/c_api.h) that the custom-call
 * handlers in this library touch, restated by hand because jaxlib's headers are not available
 * where this library is built.  Field order follows the upstream header as of the XLA revision
 * the reference plugin pins (xla/workspace.bzl of the reference).  It could not be compared with
 * the real header here: a host that has it should build with -DXMK_HAVE_XLA_FFI_H and
 * xla/ffi/api/c_api.h on the include path, which replaces this file (see xmk_ffi.h).
 *
 * The handlers registered by the reference (xla/service/gpu/sycl_custom_call.cc:207-226) are
 * C++ functions behind XLA_FFI_DEFINE_HANDLER; what crosses the ABI is one
 * `XLA_FFI_Error* handler(XLA_FFI_CallFrame*)` per custom-call target, which is what this
 * library exports (see xmk_ffi.h).
 */
#ifndef XMK_XLA_FFI_MIN_H_
#define XMK_XLA_FFI_MIN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct XLA_FFI_Api XLA_FFI_Api;
typedef struct XLA_FFI_Error XLA_FFI_Error;
typedef struct XLA_FFI_ExecutionContext XLA_FFI_ExecutionContext;
typedef struct XLA_FFI_InternalApi XLA_FFI_InternalApi;
typedef struct XLA_FFI_Future XLA_FFI_Future;

typedef enum { XLA_FFI_Extension_Metadata = 1 } XLA_FFI_Extension_Type;

typedef struct XLA_FFI_Extension_Base {
  size_t struct_size;
  XLA_FFI_Extension_Type type;
  struct XLA_FFI_Extension_Base* next;
} XLA_FFI_Extension_Base;

typedef struct XLA_FFI_Api_Version {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  int major_version;
  int minor_version;
} XLA_FFI_Api_Version;

#define XLA_FFI_API_MAJOR 0
#define XLA_FFI_API_MINOR 1

/* = absl::StatusCode */
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

/* = xla::PrimitiveType */
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
  XLA_FFI_DataType_BF16 = 16,
  XLA_FFI_DataType_F8E5M2 = 19,
  XLA_FFI_DataType_F8E4M3FN = 20
} XLA_FFI_DataType;

typedef struct XLA_FFI_Buffer {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_DataType dtype;
  void* data;
  int64_t rank;
  int64_t* dims; /* length == rank */
} XLA_FFI_Buffer;

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

typedef enum {
  XLA_FFI_ExecutionStage_INSTANTIATE = 0,
  XLA_FFI_ExecutionStage_PREPARE = 1,
  XLA_FFI_ExecutionStage_INITIALIZE = 2,
  XLA_FFI_ExecutionStage_EXECUTE = 3
} XLA_FFI_ExecutionStage;

typedef struct XLA_FFI_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  int64_t size;
  XLA_FFI_ArgType* types; /* length == size */
  void** args;            /* length == size; XLA_FFI_Buffer* for BUFFER */
} XLA_FFI_Args;

typedef struct XLA_FFI_Rets {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  int64_t size;
  XLA_FFI_RetType* types;
  void** rets;
} XLA_FFI_Rets;

/* Attributes are sorted by name. */
typedef struct XLA_FFI_Attrs {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  int64_t size;
  XLA_FFI_AttrType* types;
  XLA_FFI_ByteSpan** names;
  void** attrs; /* XLA_FFI_Scalar* / XLA_FFI_Array* / XLA_FFI_ByteSpan* / XLA_FFI_Attrs* */
} XLA_FFI_Attrs;

typedef struct XLA_FFI_CallFrame {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  const XLA_FFI_Api* api;
  XLA_FFI_ExecutionContext* ctx;
  XLA_FFI_ExecutionStage stage;
  XLA_FFI_Args args;
  XLA_FFI_Rets rets;
  XLA_FFI_Attrs attrs;
  XLA_FFI_Future* future;
} XLA_FFI_CallFrame;

typedef XLA_FFI_Error* XLA_FFI_Handler(XLA_FFI_CallFrame* call_frame);

typedef uint32_t XLA_FFI_Handler_Traits;

typedef struct XLA_FFI_Metadata {
  size_t struct_size;
  XLA_FFI_Api_Version api_version;
  XLA_FFI_Handler_Traits traits;
} XLA_FFI_Metadata;

typedef struct XLA_FFI_Metadata_Extension {
  XLA_FFI_Extension_Base extension_base;
  XLA_FFI_Metadata* metadata;
} XLA_FFI_Metadata_Extension;

typedef struct XLA_FFI_Error_Create_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  const char* message;
  XLA_FFI_Error_Code errc;
} XLA_FFI_Error_Create_Args;
typedef XLA_FFI_Error* XLA_FFI_Error_Create(XLA_FFI_Error_Create_Args* args);

typedef struct XLA_FFI_Error_GetMessage_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_Error* error;
  const char* message; /* out */
} XLA_FFI_Error_GetMessage_Args;
typedef void XLA_FFI_Error_GetMessage(XLA_FFI_Error_GetMessage_Args* args);

typedef struct XLA_FFI_Error_Destroy_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_Error* error;
} XLA_FFI_Error_Destroy_Args;
typedef void XLA_FFI_Error_Destroy(XLA_FFI_Error_Destroy_Args* args);

typedef struct XLA_FFI_Handler_Bundle {
  XLA_FFI_Handler* instantiate; /* optional */
  XLA_FFI_Handler* prepare;     /* optional */
  XLA_FFI_Handler* initialize;  /* optional */
  XLA_FFI_Handler* execute;     /* required */
} XLA_FFI_Handler_Bundle;

typedef struct XLA_FFI_Handler_Register_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_ByteSpan name;     /* custom-call target */
  XLA_FFI_ByteSpan platform; /* "SYCL" in the reference (sycl_custom_call.cc:37), "ROCM" on this GPU */
  XLA_FFI_Handler_Bundle bundle;
  XLA_FFI_Handler_Traits traits;
} XLA_FFI_Handler_Register_Args;
typedef XLA_FFI_Error* XLA_FFI_Handler_Register(XLA_FFI_Handler_Register_Args* args);

typedef struct XLA_FFI_Stream_Get_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_ExecutionContext* ctx;
  void* stream; /* out: the platform stream, a hipStream_t here */
} XLA_FFI_Stream_Get_Args;
typedef XLA_FFI_Error* XLA_FFI_Stream_Get(XLA_FFI_Stream_Get_Args* args);

/* Scratch device memory from the executor's allocator, the C face of ffi::ScratchAllocator
 * (what the reference's handlers bind with Ctx<ffi::ScratchAllocator>, sycl_custom_call.cc:207-221). */
typedef struct XLA_FFI_DeviceMemory_Allocate_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_ExecutionContext* ctx;
  size_t size;
  size_t alignment;
  void* data; /* out */
} XLA_FFI_DeviceMemory_Allocate_Args;
typedef XLA_FFI_Error* XLA_FFI_DeviceMemory_Allocate(XLA_FFI_DeviceMemory_Allocate_Args* args);

typedef struct XLA_FFI_DeviceMemory_Free_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_ExecutionContext* ctx;
  size_t size;
  void* data;
} XLA_FFI_DeviceMemory_Free_Args;
typedef XLA_FFI_Error* XLA_FFI_DeviceMemory_Free(XLA_FFI_DeviceMemory_Free_Args* args);

/* Leading part of the function table.  The four entries between Stream_Get and
 * DeviceMemory_Allocate are not used here and kept as opaque pointers; entries after
 * DeviceMemory_Free are omitted.  A caller's table may be shorter: check struct_size before
 * touching anything past Stream_Get. */
struct XLA_FFI_Api {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_Api_Version api_version;
  XLA_FFI_InternalApi* internal_api;
  XLA_FFI_Error_Create* XLA_FFI_Error_Create;
  XLA_FFI_Error_GetMessage* XLA_FFI_Error_GetMessage;
  XLA_FFI_Error_Destroy* XLA_FFI_Error_Destroy;
  XLA_FFI_Handler_Register* XLA_FFI_Handler_Register;
  XLA_FFI_Stream_Get* XLA_FFI_Stream_Get;
  void* XLA_FFI_TypeId_Register;
  void* XLA_FFI_ExecutionContext_Get;
  void* XLA_FFI_State_Set;
  void* XLA_FFI_State_Get;
  XLA_FFI_DeviceMemory_Allocate* XLA_FFI_DeviceMemory_Allocate;
  XLA_FFI_DeviceMemory_Free* XLA_FFI_DeviceMemory_Free;
};

#ifdef __cplusplus
}
#endif
#endif /* XMK_XLA_FFI_MIN_H_ */
