// Implementation of the host mirror (GpuControl, Rocblas, MatrixData, Matrix), HIP only.
#include "Matrix.h"
#include "../../include/cccc_hip_quant.h"
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdio>

namespace cccc
{

// ------------------------------------------------------------------ GpuControl

static thread_local GpuControl* current_gpu_ = nullptr;

GpuControl::GpuControl(int device_id) : device_id_(device_id)
{
    rocblas_owner_ = std::make_unique<Rocblas>();
    rocblas_ = rocblas_owner_.get();
}

GpuControl::~GpuControl()
{
    std::lock_guard<std::mutex> lock(mutex_);
    for (auto& kv : malloc_map_) { (void)hipFree(kv.first); }
    malloc_map_.clear();
}

GpuControl* GpuControl::select(int device_id)
{
    static std::mutex table_mutex;
    static std::map<int, std::unique_ptr<GpuControl>> table;
    std::lock_guard<std::mutex> lock(table_mutex);
    auto& slot = table[device_id];
    if (!slot) { slot = std::make_unique<GpuControl>(device_id); }
    slot->setAsCurrent();
    return slot.get();
}

GpuControl* GpuControl::getCurrentGpu() { return current_gpu_; }

void GpuControl::setAsCurrent()
{
    if (current_gpu_ != this)
    {
        (void)hipSetDevice(device_id_);
        current_gpu_ = this;
    }
}

int GpuControl::malloc(void** p, size_t bytes)
{
    setAsCurrent();
    *p = nullptr;
    if (bytes == 0) { return 0; }
    const hipError_t err = hipMalloc(p, bytes);
    if (err != hipSuccess)
    {
        fprintf(stderr, "hipMalloc of %zu bytes failed: %s\n", bytes, hipGetErrorString(err));
        *p = nullptr;
        return 1;
    }
    std::lock_guard<std::mutex> lock(mutex_);
    malloc_map_[*p] = bytes;
    return 0;
}

int GpuControl::free(void* p)
{
    if (!p) { return 0; }
    {
        std::lock_guard<std::mutex> lock(mutex_);
        auto it = malloc_map_.find(p);
        if (it == malloc_map_.end()) { return 1; }    // not ours: refuse
        malloc_map_.erase(it);
    }
    return hipFree(p) == hipSuccess ? 0 : 1;
}

size_t GpuControl::allocatedBytes() const
{
    std::lock_guard<std::mutex> lock(mutex_);
    size_t total = 0;
    for (auto& kv : malloc_map_) { total += kv.second; }
    return total;
}

// The reference reads and writes device memory with blocking copies behind kernels on the null stream
// (cccc/MatrixData.cpp:155-165).  Here the kernels of a host thread may run on a stream of its own
// (hip_quant_set_stream), possibly one the null stream does not order with, so every blocking copy of the mirror first
// waits for that stream: the copy then sees what the launches before it wrote, and overwrites nothing they still read.
static bool drain_launch_stream()
{
    hipStream_t s = (hipStream_t)hip_quant_get_stream();
    return s == nullptr || hipStreamSynchronize(s) == hipSuccess;
}

int GpuControl::copyHostToDevice(void* dst, const void* src, size_t bytes)
{
    return drain_launch_stream() && hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice) == hipSuccess ? 0 : 1;
}
int GpuControl::copyDeviceToHost(void* dst, const void* src, size_t bytes)
{
    return drain_launch_stream() && hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost) == hipSuccess ? 0 : 1;
}
int GpuControl::copyDeviceToDevice(void* dst, const void* src, size_t bytes)
{
    return drain_launch_stream() && hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice) == hipSuccess ? 0 : 1;
}

// ------------------------------------------------------------------ Rocblas

int Rocblas::gemm(MatrixTransType TransA, MatrixTransType TransB, int M, int N, int K, float alpha,
                  const void* A, DataType typeA, int lda, float invScaleA,
                  const void* B, DataType typeB, int ldb, float invScaleB,
                  float beta, void* C, DataType typeC, int ldc, float act_scale,
                  const uint8_t* blk_scA, const uint8_t* blk_scB)
{
    last_status_ = hip_quant_gemm((int)TransA, (int)TransB, M, N, K, alpha, A, (int)typeA, lda, invScaleA,
                                  B, (int)typeB, ldb, invScaleB, beta, C, (int)typeC, ldc, act_scale,
                                  blk_scA, blk_scB, MatrixData::fp4_block_size_);
    return last_status_;
}

// ------------------------------------------------------------------ MatrixData

void* MatrixData::resize(int64_t size, DataType data_type, bool force)
{
    releaseTiled();
    const size_t want = (size_t)size * getDataTypeSize(data_type);
    if (force || want > sizeInByte() || !data_)
    {
        if (data_ && gpu_) { gpu_->free(data_); }
        data_ = nullptr;
        if (gpu_ && want) { gpu_->malloc(&data_, want); }
    }
    occupy_data_size_ = size;
    data_type_ = data_type;
    return data_;
}

void MatrixData::prepareTiled(int n_out, int K)
{
    releaseTiled();
    if (!repack_weights || !allow_repack_ || !gpu_ || !data_ || !Rocblas::isQuantized(data_type_)) { return; }
    const bool fp4 = data_type_ == FP4_E2M1;
    // an FP4 weight is tiled together with its block scales: nothing to do until they have arrived
    if (fp4 && (!block_scale_data_ || K % 32 != 0 || block_scale_count_ < ((int64_t)n_out * K + fp4_block_size_ - 1) / fp4_block_size_)) { return; }
    const unsigned long long bytes = hip_quant_tiled_size((int)data_type_, n_out, K);
    if (bytes == 0 || gpu_->malloc(&tiled_data_, (size_t)bytes) != 0) { tiled_data_ = nullptr; return; }
    const int rc = fp4 ? hip_quant_weight_prepare_fp4(data_, block_scale_data_, fp4_block_size_, n_out, K, tiled_data_)
                       : hip_quant_weight_prepare(data_, (int)data_type_, n_out, K, K, tiled_data_);
    if (rc != 0)
    {
        gpu_->free(tiled_data_);
        tiled_data_ = nullptr;
    }
}

void MatrixData::releaseTiled()
{
    if (tiled_data_)
    {
        hip_quant_weight_release(data_);
        (void)hipDeviceSynchronize();
        if (gpu_) { gpu_->free(tiled_data_); }
        tiled_data_ = nullptr;
    }
}

void MatrixData::release()
{
    releaseTiled();
    if (gpu_)
    {
        if (data_) { gpu_->free(data_); }
        if (block_scale_data_) { gpu_->free(block_scale_data_); }
    }
    data_ = nullptr;
    block_scale_data_ = nullptr;
    block_scale_count_ = 0;
    occupy_data_size_ = 0;
}

void* MatrixData::allocBlockScaleGpu(int64_t n_scales)
{
    if (block_scale_data_ && gpu_) { gpu_->free(block_scale_data_); }
    block_scale_data_ = nullptr;
    block_scale_count_ = 0;
    if (gpu_ && n_scales > 0 && gpu_->malloc(&block_scale_data_, (size_t)n_scales) == 0) { block_scale_count_ = n_scales; }
    return block_scale_data_;
}

void MatrixData::setBlockScaleFromHost(const void* src, int64_t n_scales)
{
    releaseTiled();    // a tiled FP4 copy holds the old scales
    if (allocBlockScaleGpu(n_scales)) { GpuControl::copyHostToDevice(block_scale_data_, src, (size_t)n_scales); }
}

void MatrixData::getBlockScaleToHost(void* dst) const
{
    if (block_scale_data_ && block_scale_count_ > 0) { GpuControl::copyDeviceToHost(dst, block_scale_data_, (size_t)block_scale_count_); }
}

// ------------------------------------------------------------------ Matrix

void Matrix::setDim(int w, int h, int c, int n)
{
    width_ = w;
    height_ = h;
    channel_ = c;
    number_ = n;
    row_ = w * h * c;
}

Matrix::Matrix(int w, int h, int c, int n, DataType dt, GpuControl* gpu)
{
    setDim(w, h, c, n);
    shared_data_ = std::make_shared<MatrixData>();
    shared_data_->setGpu(gpu ? gpu : GpuControl::getCurrentGpu());
    const int64_t elems = getDataSize();
    shared_data_->resize(dt == FP4_E2M1 ? (elems + 1) / 2 : elems, dt);
    data_ = shared_data_->data_;
}

Matrix::Matrix(const std::vector<int>& dim, DataType dt, GpuControl* gpu) :
    Matrix(dim.size() > 0 ? dim[0] : 1, dim.size() > 1 ? dim[1] : 1, dim.size() > 2 ? dim[2] : 1, dim.size() > 3 ? dim[3] : 1, dt, gpu)
{
}

Matrix Matrix::view(int w, int h, int c, int n) const
{
    Matrix m = *this;
    if ((int64_t)w * h * c * n <= getDataSize()) { m.setDim(w, h, c, n); }
    return m;
}

Matrix Matrix::rowsView(int row0, int n_rows) const
{
    if (!shared_data_ || channel_ != 1 || number_ != 1 || row0 < 0 || n_rows <= 0 || row0 + n_rows > height_) { return Matrix(); }
    const int64_t first = (int64_t)row0 * width_;                       // first element of the range
    const DataType dt = getDataType();
    if (dt == FP4_E2M1 && (first % 2 != 0 || first % fp4BlockSize() != 0)) { return Matrix(); }
    Matrix m = *this;
    m.setDim(width_, n_rows, 1, 1);
    m.data_ = (char*)data_ + (dt == FP4_E2M1 ? first / 2 : first * (int64_t)Rocblas::elemBytes(dt));
    m.scale_offset_ = scale_offset_ + (dt == FP4_E2M1 ? first / fp4BlockSize() : 0);
    m.rows_view_ = rows_view_ || n_rows != height_;
    return m;
}

int Matrix::copyFromHost(const void* src, size_t bytes)
{
    if (!shared_data_ || bytes > shared_data_->sizeInByte()) { return 1; }
    shared_data_->releaseTiled();    // a tiled copy of the old bytes must not outlive them; prepareTiled() builds a new one
    return GpuControl::copyHostToDevice(data_, src, bytes);
}

int Matrix::copyToHost(void* dst, size_t bytes) const
{
    if (!shared_data_ || bytes > shared_data_->sizeInByte()) { return 1; }
    return GpuControl::copyDeviceToHost(dst, data_, bytes);
}

void Matrix::retype(DataType dt)
{
    if (!shared_data_ || !gpu()) { return; }
    gpu()->setAsCurrent();
    const int64_t n = dt == FP4_E2M1 ? (getDataSize() + 1) / 2 : getDataSize();
    shared_data_->resize(n, dt, true);
    data_ = shared_data_->data_;
}

void Matrix::loadQuantizedDirect(const uint8_t* host_data, int64_t n, float scale, DataType fp8_dt)
{
    if (!gpu()) { return; }
    gpu()->setAsCurrent();
    // a storage of another type, or one too small for the upload, is replaced
    shared_data_->releaseTiled();    // whatever tiled copy exists belongs to the bytes about to be replaced
    if (getDataType() != fp8_dt || (size_t)n > shared_data_->sizeInByte()) { shared_data_->resize(n, fp8_dt, true); }
    GpuControl::copyHostToDevice(shared_data_->data_, host_data, (size_t)n);
    shared_data_->quant_scale_ = scale;
    data_ = shared_data_->data_;
    // a [K x n_out] linear weight (one batch): keep an MI355X-friendly tiled copy next to the file bytes
    if (number_ == 1 && channel_ == 1 && (int64_t)width_ * height_ == n) { shared_data_->prepareTiled(height_, width_); }
}

void Matrix::quantizeWeights(DataType target_dt)
{
    if (!gpu() || (getDataType() != BFLOAT16 && getDataType() != HALF)) { return; }
    if (getWidth() < 64 || getHeight() < 64) { return; }
    const int64_t n = getDataSize();
    if (n <= 0 || !Rocblas::isQuantized(target_dt)) { return; }
    gpu()->setAsCurrent();

    MatrixData float_buf;
    float_buf.setGpu(gpu());
    float_buf.resize(n, FLOAT);
    hip_convert(data_, getDataType(), float_buf.data_, FLOAT, (unsigned int)n, 1.0f);

    if (target_dt == FP4_E2M1)
    {
        const unsigned int block = MatrixData::fp4_block_size_;
        const int64_t n_blocks = (n + block - 1) / block;
        shared_data_->resize((n + 1) / 2, target_dt, true);
        void* d_scales = shared_data_->allocBlockScaleGpu(n_blocks);
        hip_float_to_fp4_blockscale(float_buf.data_, shared_data_->data_, d_scales, (unsigned int)n, block);
        shared_data_->quant_scale_ = 1.0f;
    }
    else
    {
        float max_abs = 0.0f;
        void* d_max = nullptr;
        gpu()->malloc(&d_max, sizeof(float));
        hip_absmax(float_buf.data_, FLOAT, (unsigned int)n, d_max);
        GpuControl::copyDeviceToHost(&max_abs, d_max, sizeof(float));
        gpu()->free(d_max);
        max_abs = std::fabs(max_abs);
        const float max_code = target_dt == FP8_E4M3 ? 448.0f : 57344.0f;
        const float fwd_scale = (max_abs > 1e-10f) ? (max_code / max_abs) : 1.0f;
        shared_data_->quant_scale_ = (max_abs > 1e-10f) ? (max_abs / max_code) : 1.0f;
        shared_data_->resize(n, target_dt, true);
        hip_convert(float_buf.data_, FLOAT, shared_data_->data_, target_dt, (unsigned int)n, fwd_scale);
    }
    (void)hipDeviceSynchronize();    // float_buf is freed on return
    data_ = shared_data_->data_;
    if (number_ == 1 && channel_ == 1) { shared_data_->prepareTiled(height_, width_); }
}

// The operand extents a column-major GEMM will touch, checked against what the tensors hold before
// anything is launched (a shape mistake must come back as an error code, not as a device fault).
static bool gemm_extents_fit(MatrixTransType ta, MatrixTransType tb, long long M, long long N, long long K,
                             long long lda, long long ldb, long long ldc, long long sizeA, long long sizeB, long long sizeC)
{
    const long long rowsA = (ta == MATRIX_NO_TRANS) ? M : K, colsA = (ta == MATRIX_NO_TRANS) ? K : M;
    const long long rowsB = (tb == MATRIX_NO_TRANS) ? K : N, colsB = (tb == MATRIX_NO_TRANS) ? N : K;
    if (M < 0 || N < 0 || K < 0 || lda < rowsA || ldb < rowsB || ldc < M) { return false; }
    if (M == 0 || N == 0) { return true; }
    if (K > 0 && ((colsA - 1) * lda + rowsA > sizeA || (colsB - 1) * ldb + rowsB > sizeB)) { return false; }
    return (N - 1) * ldc + M <= sizeC;
}

int Matrix::mul(const Matrix& A, const Matrix& B, Matrix& R, float a, float r, MatrixTransType ta, MatrixTransType tb)
{
    const int m = R.row_;
    const int n = R.number_;
    const int lda = A.row_;
    const int k = (ta == MATRIX_TRANS) ? A.row_ : A.number_;
    const int ldb = B.row_;
    if (!gemm_extents_fit(ta, tb, m, n, k, lda, ldb, m, A.getDataSize(), B.getDataSize(), R.getDataSize()))
    {
        fprintf(stderr, "Matrix::mul: operand shapes do not fit (m=%d n=%d k=%d lda=%d ldb=%d)\n", m, n, k, lda, ldb);
        return -1;
    }
    float act_scale = 0.0f;
    if (Rocblas::isQuantized(B.getDataType()) && !Rocblas::isQuantized(A.getDataType())) { act_scale = B.getInputScale(); }
    else if (Rocblas::isQuantized(A.getDataType()) && !Rocblas::isQuantized(B.getDataType())) { act_scale = A.getInputScale(); }
    const uint8_t* blk_scA = (A.getDataType() == FP4_E2M1) ? (const uint8_t*)A.getBlockScaleData() : nullptr;
    const uint8_t* blk_scB = (B.getDataType() == FP4_E2M1) ? (const uint8_t*)B.getBlockScaleData() : nullptr;
    return R.gpu()->rocblas_->gemm(ta, tb, m, n, k, a, A.data(), A.getDataType(), lda, A.getQuantScale(),
                                   B.data(), B.getDataType(), ldb, B.getQuantScale(), r, R.data(), R.getDataType(), m,
                                   act_scale, blk_scA, blk_scB);
}

int Matrix::mulBatched(const Matrix& A, const Matrix& B, Matrix& R, MatrixTransType ta, MatrixTransType tb, float a, float r)
{
    const int M = (ta == MATRIX_NO_TRANS) ? A.width_ : A.height_;
    const int K = (ta == MATRIX_NO_TRANS) ? A.height_ : A.width_;
    const int N = (tb == MATRIX_NO_TRANS) ? B.height_ : B.width_;
    const int batch = A.number_;
    const int lda = (ta == MATRIX_NO_TRANS) ? M : K;
    const int ldb = (tb == MATRIX_NO_TRANS) ? K : N;
    const int ldc = M;
    const long long strideA = (long long)M * K, strideB = (long long)K * N, strideC = (long long)M * N;
    const DataType tA = A.getDataType(), tB = B.getDataType(), tC = R.getDataType();
    if (batch < 1 || B.number_ != batch || R.number_ != batch ||
        !gemm_extents_fit(ta, tb, M, N, K, lda, ldb, ldc, A.row_, B.row_, R.row_))
    {
        fprintf(stderr, "Matrix::mulBatched: operand shapes do not fit (M=%d N=%d K=%d batch=%d)\n", M, N, K, batch);
        return -1;
    }
    int status = 0;
    for (int b = 0; b < batch; b++)
    {
        const long long byteA = (tA == FP4_E2M1) ? strideA / 2 : strideA * (long long)Rocblas::elemBytes(tA);
        const long long byteB = (tB == FP4_E2M1) ? strideB / 2 : strideB * (long long)Rocblas::elemBytes(tB);
        const long long byteC = strideC * (long long)Rocblas::elemBytes(tC);
        float act_scale = 0.0f;
        if (Rocblas::isQuantized(tB) && !Rocblas::isQuantized(tA)) { act_scale = B.getInputScale(); }
        else if (Rocblas::isQuantized(tA) && !Rocblas::isQuantized(tB)) { act_scale = A.getInputScale(); }
        const uint8_t* blk_scA = nullptr;
        if (tA == FP4_E2M1 && A.getBlockScaleData()) { blk_scA = (const uint8_t*)A.getBlockScaleData() + b * strideA / (long long)fp4BlockSize(); }
        const uint8_t* blk_scB = nullptr;
        if (tB == FP4_E2M1 && B.getBlockScaleData()) { blk_scB = (const uint8_t*)B.getBlockScaleData() + b * strideB / (long long)fp4BlockSize(); }
        const int rc = R.gpu()->rocblas_->gemm(ta, tb, M, N, K, a,
                                               (const char*)A.data() + b * byteA, tA, lda, A.getQuantScale(),
                                               (const char*)B.data() + b * byteB, tB, ldb, B.getQuantScale(),
                                               r, (char*)R.data() + b * byteC, tC, ldc, act_scale, blk_scA, blk_scB);
        if (rc != 0) { status = rc; }
    }
    return status;
}

}    // namespace cccc
