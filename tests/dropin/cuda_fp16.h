// Test-local stand-in for <cuda_fp16.h>: lpp_kernels_compat.h already names the 16-bit storage type __half.
#pragma once
