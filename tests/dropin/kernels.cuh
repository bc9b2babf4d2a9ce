// What a Lighter++ tree puts in place of its src/kernels.cuh to build against liblpp_hip.so: one include.
#pragma once
#include "lpp_kernels_compat.h"
