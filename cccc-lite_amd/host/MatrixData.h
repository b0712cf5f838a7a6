// Device storage with the quantization state the reference keeps per storage
// (cccc/MatrixData.h:10-27): per-tensor dequant multiplier, FP4 block scales (one E4M3 byte per
// fp4_block_size_ elements), static activation scale.
#pragma once
#include "GpuControl.h"
#include "types.h"
#include <cstdint>

namespace cccc
{

struct MatrixData
{
    GpuControl* gpu_ = nullptr;
    void* data_ = nullptr;
    int64_t occupy_data_size_ = 0;    // elements (FP4: packed bytes, as the reference sizes it)
    DataType data_type_ = FLOAT;
    float quant_scale_ = 1.0f;
    void* block_scale_data_ = nullptr;
    int64_t block_scale_count_ = 0;
    static constexpr unsigned int fp4_block_size_ = 16;
    float input_scale_ = 0.0f;
    // Load-time repacked (tiled) copy of an FP8 weight, or of an FP4 weight and its block scales, for the matrix-core GEMV; owned here, registered
    // with the kernel library under the key data_.  No counterpart in the reference.
    void* tiled_data_ = nullptr;
    static inline bool repack_weights = true;    // global switch
    bool allow_repack_ = true;                    // per storage (e.g. off for weights only the row-major SwiGLU pair kernel reads)

    MatrixData() = default;
    ~MatrixData() { release(); }
    MatrixData(const MatrixData&) = delete;
    MatrixData& operator=(const MatrixData&) = delete;

    void setGpu(GpuControl* gpu) { gpu_ = gpu; }
    DataType getDataType() const { return data_type_; }
    static size_t getDataTypeSize(DataType dt) { return Rocblas::elemBytes(dt); }
    size_t sizeInByte() const { return (size_t)occupy_data_size_ * getDataTypeSize(data_type_); }

    // (Re)allocates when the byte size grows or `force` is set; contents are not kept.
    void* resize(int64_t size, DataType data_type, bool force = false);
    void release();

    // Builds / drops the tiled copy for a [n_out][K] FP8 weight (or FP4 weight with block scales) stored in data_.
    void prepareTiled(int n_out, int K);
    void releaseTiled();

    void setBlockScaleFromHost(const void* src, int64_t n_scales);
    void getBlockScaleToHost(void* dst) const;
    void* allocBlockScaleGpu(int64_t n_scales);
};

}    // namespace cccc
