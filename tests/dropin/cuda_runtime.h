// Test-local stand-in for <cuda_runtime.h>: the handful of runtime calls the reference's model.cpp makes itself
// (model.cpp:42, 59-79, 94, 102-116, 349, 361, 369), forwarded to section C of lpp.h.  Not part of the library.
#pragma once
#include "lpp.h"
enum { cudaMemcpyHostToDevice, cudaMemcpyDeviceToHost, cudaMemcpyDeviceToDevice };
enum { cudaHostAllocDefault = 0 };
#define cudaMalloc(p, n) lpp_malloc((void**)(p), (n))
#define cudaFree(p) lpp_free(p)
#define cudaHostAlloc(p, n, flags) lpp_malloc_host((void**)(p), (n))
#define cudaFreeHost(p) lpp_free_host(p)
#define cudaMemset(p, v, n) lpp_memset((p), (v), (n))
#define cudaMemcpy(d, s, n, kind)                                       \
    ((kind) == cudaMemcpyHostToDevice   ? lpp_memcpy_h2d((d), (s), (n)) \
     : (kind) == cudaMemcpyDeviceToHost ? lpp_memcpy_d2h((d), (s), (n)) \
                                        : lpp_memcpy_d2d((d), (s), (n)))
