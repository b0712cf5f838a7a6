// Scalar type tags of the host mirror.  Values are the reference's (cccc/types.h:24-34,
// cccc/blas_types.h:10-14) because they cross the C-ABI as plain ints.
#pragma once
#include <cstddef>
#include <cstdint>

namespace cccc
{

enum DataType
{
    FLOAT = 0,
    DOUBLE = 1,
    HALF = 2,
    BFLOAT16 = 3,
    FP8_E4M3 = 4,    // 1 byte per element
    FP8_E5M2 = 5,    // 1 byte per element
    FP4_E2M1 = 6,    // two elements per byte, low nibble = even element
    CURRENT = 65535,
};

enum MatrixTransType
{
    MATRIX_NO_TRANS = 0,
    MATRIX_TRANS = 1,
};

}    // namespace cccc
