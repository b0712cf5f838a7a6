// The BLAS face of the HIP build for the quantized path.  The reference's Rocblas has no quantized
// overload (cccc/rocblas_real.h:454-478 only types the operands by the output dtype); this is the
// unified dispatcher the CUDA build has (cccc/cublas_real.h:855-881), forwarding to the kernel
// library's hip_quant_gemm.
#pragma once
#include "types.h"

namespace cccc
{

class Rocblas
{
public:
    static bool isQuantized(DataType dt) { return dt == FP8_E4M3 || dt == FP8_E5M2 || dt == FP4_E2M1; }

    // Bytes per element; FP4 reports 1 and callers halve byte strides themselves, as in the reference
    // (cccc/cublas_real.h:859-871).
    static size_t elemBytes(DataType dt)
    {
        switch (dt)
        {
        case DOUBLE: return 8;
        case FLOAT: return 4;
        case HALF:
        case BFLOAT16: return 2;
        default: return 1;
        }
    }

    // Column-major C = alpha * op(A) * op(B) + beta * C with typed operands.  Returns the kernel
    // library's code (0 ok, 1 runtime error, -1 unsupported) and remembers it in lastStatus().
    int gemm(MatrixTransType TransA, MatrixTransType TransB, int M, int N, int K, float alpha,
             const void* A, DataType typeA, int lda, float invScaleA,
             const void* B, DataType typeB, int ldb, float invScaleB,
             float beta, void* C, DataType typeC, int ldc, float act_scale = 0.0f,
             const uint8_t* blk_scA = nullptr, const uint8_t* blk_scB = nullptr);

    int lastStatus() const { return last_status_; }

private:
    int last_status_ = 0;
};

}    // namespace cccc
