/* The HIP runtime entry points the shim calls, declared by hand so that the Clang importer does not
 * have to digest the HIP headers.  Signatures as in <hip/hip_runtime_api.h>; hipError_t is an enum
 * whose success value is 0, hipStream_t an opaque pointer. */
#ifndef CDFLASHHIP_HIP_MIN_H
#define CDFLASHHIP_HIP_MIN_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

int hipMalloc(void** ptr, size_t size);
int hipFree(void* ptr);
int hipMemcpy(void* dst, const void* src, size_t size_bytes, int kind); /* kind 1 = host to device, 2 = device to host */
int hipMemsetAsync(void* dst, int value, size_t size_bytes, void* stream);
int hipStreamSynchronize(void* stream);
const char* hipGetErrorString(int error);

#ifdef __cplusplus
}
#endif
#endif
