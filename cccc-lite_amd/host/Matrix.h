// Column-major tensor of the host mirror, dims (W, H, C, N) with W fastest, shallow-copy views over
// shared storage: the part of the reference's Matrix (cccc/Matrix.h, cccc/Matrix.cpp) that the
// quantized linear path touches, HIP only.
#pragma once
#include <cstdio>
#include "MatrixData.h"
#include <memory>
#include <vector>

namespace cccc
{

class Matrix
{
public:
    Matrix() = default;
    Matrix(int w, int h, int c, int n, DataType dt, GpuControl* gpu = nullptr);
    Matrix(const std::vector<int>& dim, DataType dt, GpuControl* gpu = nullptr);

    // A view of the same storage with other dims (element count must not grow).
    Matrix view(int w, int h, int c, int n) const;
    // Rows [row0, row0 + n_rows) of a (W x H) matrix as a (W x n_rows) matrix on the same storage -- for a linear
    // weight stored [n_out][K] these are output features row0 .. row0 + n_rows - 1 with their block scales.  This is
    // how several projections that share an input (q, k, v; gate, up) can live in ONE storage that a single GEMV
    // reads while each keeps a tensor of its own (the reference's view mechanics: cccc/MatrixOp.cpp:1370-1396).
    // An empty Matrix when the range does not fit or the matrix is not 2-D.
    Matrix rowsView(int row0, int n_rows) const;

    int getWidth() const { return width_; }
    int getHeight() const { return height_; }
    int getChannel() const { return channel_; }
    int getNumber() const { return number_; }
    int getRow() const { return row_; }
    int64_t getDataSize() const { return (int64_t)row_ * number_; }
    DataType getDataType() const { return shared_data_ ? shared_data_->data_type_ : FLOAT; }
    GpuControl* gpu() const { return shared_data_ ? shared_data_->gpu_ : nullptr; }
    void* data() const { return data_; }

    float getQuantScale() const { return shared_data_->quant_scale_; }
    void setQuantScale(float s) { shared_data_->quant_scale_ = s; }
    const void* getBlockScaleData() const
    {
        return shared_data_->block_scale_data_ ? (const uint8_t*)shared_data_->block_scale_data_ + scale_offset_ : nullptr;
    }
    // Block scales this tensor owns: all of the storage's, or, for a row view, those of its own rows
    int64_t getBlockScaleCount() const
    {
        if (!rows_view_) { return shared_data_->block_scale_count_; }
        return shared_data_->block_scale_data_ ? (getDataSize() + fp4BlockSize() - 1) / fp4BlockSize() : 0;
    }
    // Uploads the FP4 block scales; a [K x n_out] linear weight then gets its tiled copy (codes + scales).  A row view
    // does neither: the scale array and the tiled copy belong to the whole storage, under the storage's own dims.
    void setBlockScaleFromHost(const void* src, int64_t n_scales)
    {
        if (rows_view_)
        {
            fprintf(stderr, "cccc host: setBlockScaleFromHost on a row view is refused (upload the scales through the storage that owns them)\n");
            return;
        }
        shared_data_->setBlockScaleFromHost(src, n_scales);
        if (number_ == 1 && channel_ == 1 && getDataType() == FP4_E2M1) { shared_data_->prepareTiled(height_, width_); }
    }
    void getBlockScaleToHost(void* dst) const
    {
        if (!rows_view_) { shared_data_->getBlockScaleToHost(dst); }
        else if (getBlockScaleCount() > 0) { GpuControl::copyDeviceToHost(dst, getBlockScaleData(), (size_t)getBlockScaleCount()); }
    }
    static unsigned int fp4BlockSize() { return MatrixData::fp4_block_size_; }
    void prepareTiled() { if (shared_data_ && !rows_view_ && number_ == 1 && channel_ == 1) { shared_data_->prepareTiled(height_, width_); } }
    bool isRowsView() const { return rows_view_; }
    void setAllowRepack(bool allow) { if (shared_data_) { shared_data_->allow_repack_ = allow; } }
    bool hasTiled() const { return shared_data_ && shared_data_->tiled_data_ != nullptr; }
    float getInputScale() const { return shared_data_ ? shared_data_->input_scale_ : 0.0f; }
    void setInputScale(float s) { if (shared_data_) { shared_data_->input_scale_ = s; } }
    // Re-allocates the storage for the same dims with another element type (contents are not kept).
    void retype(DataType dt);

    // Raw byte transfers between host memory and this tensor's storage.
    int copyFromHost(const void* src, size_t bytes);
    int copyToHost(void* dst, size_t bytes) const;

    // Re-types the storage to a 1-byte (FP8) or packed-nibble (FP4) weight and uploads the file
    // bytes as they are (cccc/Matrix.cpp:357-375).  `n` is the byte count to upload.
    void loadQuantizedDirect(const uint8_t* host_data, int64_t n, float scale, DataType fp8_dt = FP8_E4M3);

    // In-place BF16 -> quantized conversion on the device (cccc/Matrix.cpp:301-355): FP4 gets
    // per-block E4M3 scales and quant_scale_ = 1; FP8 gets one per-tensor scale absmax / max_code.
    void quantizeWeights(DataType target_dt);

    // R = a * op(A) * op(B) + r * R (cccc/Matrix.cpp:1107-1157) and its per-batch form
    // (cccc/Matrix.cpp:1162-1268).  Quantized operands go through Rocblas::gemm(unified).
    // Return the last status of the BLAS face (0 ok).
    static int mul(const Matrix& A, const Matrix& B, Matrix& R, float a = 1, float r = 0,
                   MatrixTransType ta = MATRIX_NO_TRANS, MatrixTransType tb = MATRIX_NO_TRANS);
    static int mulBatched(const Matrix& A, const Matrix& B, Matrix& R,
                          MatrixTransType ta = MATRIX_NO_TRANS, MatrixTransType tb = MATRIX_NO_TRANS, float a = 1, float r = 0);

private:
    void setDim(int w, int h, int c, int n);

    std::shared_ptr<MatrixData> shared_data_;
    void* data_ = nullptr;
    int64_t scale_offset_ = 0;    // first block scale of this view within the storage's scale array
    bool rows_view_ = false;      // made by rowsView(): a row range of a larger storage
    int width_ = 0, height_ = 0, channel_ = 0, number_ = 0, row_ = 0;
};

}    // namespace cccc
