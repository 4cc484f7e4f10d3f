/*
 * Tensor handle types of the tinyflow C-ABI.
 *
 * These three types are the binary contract between the ctypes binding and
 * libc_runtime_api.so; their layout is fixed by the reference
 * (reference: src/dlarray.h:21-52, mirrored by pycode/tinyflow/ndarray.py:8-36):
 *
 *   DLContext  { int device_id; int device_type }            8 bytes
 *   DLArray    { void* data; DLContext ctx; int ndim; int64_t* shape }   32 bytes
 *
 * A DLArray is always a dense, row-major block of 32-bit floats; it carries no
 * strides and no dtype (reference: src/c_runtime_api.cc:72-80 sizes every array
 * as 4 bytes per element).
 */
#ifndef TINYFLOW_AMD_DLARRAY_H_
#define TINYFLOW_AMD_DLARRAY_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* device_type values sent by the binding: cpu() -> 1, gpu() -> 2. */
typedef enum {
  kCPU = 1,
  kGPU = 2,
} DLDeviceType;

typedef struct {
  int device_id;
  DLDeviceType device_type;
} DLContext;

typedef struct {
  void *data;      /* device pointer (kGPU) or pinned host pointer (kCPU), 256-byte aligned */
  DLContext ctx;
  int ndim;
  int64_t *shape;  /* ndim entries, owned by the library for arrays it allocated */
} DLArray;

typedef DLArray *DLArrayHandle;

/* NULL (synchronous copy) or a pointer to a cell holding the stream
 * (reference: src/c_runtime_api.cc:148-158 dereferences it once). */
typedef void *DLStreamHandle;

#ifdef __cplusplus
}
#endif
#endif /* TINYFLOW_AMD_DLARRAY_H_ */
