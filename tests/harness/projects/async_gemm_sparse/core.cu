#pragma once

#include <hip/hip_runtime.h>
#include <iostream>

// Role split and ring of the async_gemm launcher.  A grid-search driver rewrites the lines below that start with
// "#define <NAME>" (same mechanism as the reference's projects/async_gemm_sparse/core.cu:29-40).
#define A_PRODUCERS 1
#define B_PRODUCERS 4
#define CONSUMERS 3
#define B_LANES 2
#define QSIZE 6
