#pragma once

#include <hip/hip_runtime.h>
#include <iostream>

// Tunables of the fastpath.  A grid-search driver rewrites the lines below that start with
// "#define <NAME>_" (same names and mechanism as the reference's projects/skinny_gemm/core.cu:29-38).
#define B_LANES_ 1
#define QSIZE_ 8
#define OP_M_ 8
#define OPS_ 4

#define A_PRODUCERS_ 0
#define B_PRODUCERS_ 0
#define CONSUMERS_ 1

#define SK_ 1
