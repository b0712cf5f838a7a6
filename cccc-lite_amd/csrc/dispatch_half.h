// FP8 weights against IEEE-half activations (the reference's other 16-bit route,
// cccc/cublas_real.h:921-938): launches the half instantiations of the dot2 GEMV (up to 4 tokens
// per pass) or of the matrix-core GEMM.  Preconditions as for the BF16 kernels (K-major operands,
// K % 16 == 0, ldw % 16 == 0, 16-byte aligned pointers, ldx % 8 == 0); returns the kernel family name.
#pragma once
#include "linear_args.h"
#include "runtime.h"

namespace ccq
{
// `scratch` as in gemm_mfma; returns nullptr when a fixed scratch buffer was too small (nothing launched).
const char* half_linear(const LinearArgs& a, int w_type, SplitScratch* scratch = nullptr);
}
