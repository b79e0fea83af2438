/*
 * Minimal DLPack tensor descriptors (ABI of DLPack v0.x / v1 "unversioned" structs), restated from the
 * public DLPack specification so that this library has no build-time dependency on a framework.
 * Only the structs the C-ABI of sqattn.h needs are declared.  If <dlpack/dlpack.h> was included
 * first, its definitions are used instead.
 */
#ifndef SQ_DLPACK_H_
#define SQ_DLPACK_H_

#include <stdint.h>

#ifndef DLPACK_DLPACK_H_
#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  kDLCPU = 1,
  kDLCUDA = 2,
  kDLCUDAHost = 3,
  kDLROCM = 10,
  kDLROCMHost = 11,
} DLDeviceType;

typedef struct {
  int32_t device_type; /* a DLDeviceType */
  int32_t device_id;
} DLDevice;

typedef enum {
  kDLInt = 0,
  kDLUInt = 1,
  kDLFloat = 2,
  kDLOpaqueHandle = 3,
  kDLBfloat = 4,
} DLDataTypeCode;

typedef struct {
  uint8_t code; /* a DLDataTypeCode */
  uint8_t bits;
  uint16_t lanes;
} DLDataType;

typedef struct {
  void* data;
  DLDevice device;
  int32_t ndim;
  DLDataType dtype;
  int64_t* shape;
  int64_t* strides; /* in elements; NULL means compact row-major */
  uint64_t byte_offset;
} DLTensor;

typedef struct DLManagedTensor {
  DLTensor dl_tensor;
  void* manager_ctx;
  void (*deleter)(struct DLManagedTensor* self);
} DLManagedTensor;

#ifdef __cplusplus
}
#endif
#endif /* DLPACK_DLPACK_H_ */

#endif /* SQ_DLPACK_H_ */
