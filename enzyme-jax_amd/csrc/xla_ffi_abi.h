/* Subset of the XLA FFI C ABI (xla/ffi/api/c_api.h) that the handlers in
 * ffi_handlers.cc touch.
 *
 * The header itself is third-party (XLA at the commit JAX pins; the reference
 * gets it through Bazel, third_party/xla/workspace.bzl:13-22) and is not part
 * of this tree, so the structures are restated here from the public layout:
 * every struct starts with {size_t struct_size; XLA_FFI_Extension_Base*
 * extension_start}, enumerators carry their public values.  Field names that
 * the reference itself dereferences (src/enzyme_ad/jax/gpu.cc:44-63,96-151)
 * are marked [ref].  Handlers check `struct_size` before using any field past
 * that verified subset, and fail with an error instead of reading beyond a
 * smaller struct.  This restatement has not been compiled against a real XLA.
 */
#ifndef EMI_XLA_FFI_ABI_H_
#define EMI_XLA_FFI_ABI_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XLA_FFI_API_MAJOR 0
#define XLA_FFI_API_MINOR 1

typedef struct XLA_FFI_Api XLA_FFI_Api;
typedef struct XLA_FFI_InternalApi XLA_FFI_InternalApi;
typedef struct XLA_FFI_Error XLA_FFI_Error;                       /* nullptr == success [ref] */
typedef struct XLA_FFI_ExecutionContext XLA_FFI_ExecutionContext;
typedef struct XLA_FFI_Future XLA_FFI_Future;

typedef enum { XLA_FFI_Extension_Metadata = 1 } XLA_FFI_Extension_Type;   /* [ref] */

typedef struct XLA_FFI_Extension_Base {
  size_t struct_size;
  XLA_FFI_Extension_Type type;                                    /* [ref] */
  struct XLA_FFI_Extension_Base* next;
} XLA_FFI_Extension_Base;

typedef struct XLA_FFI_Api_Version {                              /* 4-field init [ref] gpu.cc:102-107 */
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  int major_version;
  int minor_version;
} XLA_FFI_Api_Version;

typedef uint32_t XLA_FFI_Handler_Traits;

typedef struct XLA_FFI_Metadata {
  size_t struct_size;
  XLA_FFI_Api_Version api_version;                                /* [ref] */
  XLA_FFI_Handler_Traits traits;
} XLA_FFI_Metadata;

typedef struct XLA_FFI_Metadata_Extension {
  XLA_FFI_Extension_Base extension_base;
  XLA_FFI_Metadata* metadata;                                     /* [ref] */
} XLA_FFI_Metadata_Extension;

typedef enum {
  XLA_FFI_Error_Code_OK = 0,
  XLA_FFI_Error_Code_INVALID_ARGUMENT = 3,
  XLA_FFI_Error_Code_UNIMPLEMENTED = 12,
  XLA_FFI_Error_Code_INTERNAL = 13                                /* [ref] */
} XLA_FFI_Error_Code;

typedef struct XLA_FFI_Error_Create_Args {                        /* [ref] gpu.cc:144-149 */
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  const char* message;
  XLA_FFI_Error_Code errc;
} XLA_FFI_Error_Create_Args;

typedef enum {                                                    /* = xla::PrimitiveType */
  XLA_FFI_DataType_INVALID = 0, XLA_FFI_DataType_PRED = 1, XLA_FFI_DataType_S8 = 2, XLA_FFI_DataType_S16 = 3,
  XLA_FFI_DataType_S32 = 4, XLA_FFI_DataType_S64 = 5, XLA_FFI_DataType_U8 = 6, XLA_FFI_DataType_U16 = 7,
  XLA_FFI_DataType_U32 = 8, XLA_FFI_DataType_U64 = 9, XLA_FFI_DataType_F16 = 10, XLA_FFI_DataType_F32 = 11,
  XLA_FFI_DataType_F64 = 12, XLA_FFI_DataType_C64 = 15, XLA_FFI_DataType_BF16 = 16, XLA_FFI_DataType_TOKEN = 17,
  XLA_FFI_DataType_C128 = 18
} XLA_FFI_DataType;

typedef struct XLA_FFI_Buffer {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_DataType dtype;
  void* data;                                                     /* [ref] */
  int64_t* dims;
  int64_t rank;
} XLA_FFI_Buffer;

typedef enum { XLA_FFI_ArgType_BUFFER = 1 } XLA_FFI_ArgType;
typedef enum { XLA_FFI_RetType_BUFFER = 1 } XLA_FFI_RetType;
typedef enum {
  XLA_FFI_AttrType_ARRAY = 1, XLA_FFI_AttrType_DICTIONARY = 2, XLA_FFI_AttrType_SCALAR = 3,
  XLA_FFI_AttrType_STRING = 4                                     /* [ref] */
} XLA_FFI_AttrType;
typedef enum {
  XLA_FFI_ExecutionStage_INSTANTIATE = 0, XLA_FFI_ExecutionStage_PREPARE = 1,
  XLA_FFI_ExecutionStage_INITIALIZE = 2,                          /* [ref] */
  XLA_FFI_ExecutionStage_EXECUTE = 3
} XLA_FFI_ExecutionStage;

typedef struct XLA_FFI_ByteSpan { const char* ptr; size_t len; } XLA_FFI_ByteSpan;       /* ptr [ref] */
typedef struct XLA_FFI_Scalar { XLA_FFI_DataType dtype; void* value; } XLA_FFI_Scalar;
typedef struct XLA_FFI_Array { XLA_FFI_DataType dtype; size_t size; void* data; } XLA_FFI_Array;

typedef struct XLA_FFI_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  int64_t size;                                                   /* [ref] */
  XLA_FFI_ArgType* types;
  void** args;                                                    /* [ref] */
} XLA_FFI_Args;

typedef struct XLA_FFI_Rets {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  int64_t size;
  XLA_FFI_RetType* types;
  void** rets;
} XLA_FFI_Rets;

typedef struct XLA_FFI_Attrs {                                    /* sorted by name */
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  int64_t size;                                                   /* [ref] */
  XLA_FFI_AttrType* types;                                        /* [ref] */
  XLA_FFI_ByteSpan** names;
  void** attrs;                                                   /* [ref] */
} XLA_FFI_Attrs;

typedef struct XLA_FFI_CallFrame {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;                        /* [ref] */
  const XLA_FFI_Api* api;                                         /* [ref] */
  XLA_FFI_ExecutionContext* ctx;                                  /* [ref] */
  XLA_FFI_ExecutionStage stage;
  XLA_FFI_Args args;
  XLA_FFI_Rets rets;
  XLA_FFI_Attrs attrs;
  XLA_FFI_Future* future;
} XLA_FFI_CallFrame;

typedef XLA_FFI_Error* XLA_FFI_Handler(XLA_FFI_CallFrame* call_frame);                  /* [ref] gpu.cc:35,95 */

typedef struct XLA_FFI_Handler_Bundle {                           /* [ref] gpu.cc:160-168 */
  XLA_FFI_Handler* instantiate;
  XLA_FFI_Handler* prepare;
  XLA_FFI_Handler* initialize;
  XLA_FFI_Handler* execute;
} XLA_FFI_Handler_Bundle;

typedef struct XLA_FFI_Handler_Register_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_ByteSpan name;
  XLA_FFI_ByteSpan platform;
  XLA_FFI_Handler_Bundle bundle;
  XLA_FFI_Handler_Traits traits;
} XLA_FFI_Handler_Register_Args;

typedef struct XLA_FFI_Stream_Get_Args {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_ExecutionContext* ctx;
  void* stream;                                                   /* out: hipStream_t on the ROCM platform */
} XLA_FFI_Stream_Get_Args;

typedef struct XLA_FFI_Error_GetMessage_Args XLA_FFI_Error_GetMessage_Args;
typedef struct XLA_FFI_Error_Destroy_Args XLA_FFI_Error_Destroy_Args;

struct XLA_FFI_Api {
  size_t struct_size;
  XLA_FFI_Extension_Base* extension_start;
  XLA_FFI_Api_Version api_version;
  XLA_FFI_InternalApi* internal_api;                              /* [ref] */
  XLA_FFI_Error* (*XLA_FFI_Error_Create)(XLA_FFI_Error_Create_Args*);                    /* [ref] */
  void (*XLA_FFI_Error_GetMessage)(XLA_FFI_Error_GetMessage_Args*);
  void (*XLA_FFI_Error_Destroy)(XLA_FFI_Error_Destroy_Args*);
  XLA_FFI_Error* (*XLA_FFI_Handler_Register)(XLA_FFI_Handler_Register_Args*);
  XLA_FFI_Error* (*XLA_FFI_Stream_Get)(XLA_FFI_Stream_Get_Args*);
  /* further entries (type ids, execution state, device memory, thread pool) are not used */
};

#ifdef __cplusplus
}
#endif
#endif /* EMI_XLA_FFI_ABI_H_ */
