// Reader of cccc's weight container ("CFG_BIN INI") and the named-weight loading rules on top of it.
//
// Container, as scripts/convert_weights.py:54-83 writes it (the reading side lives in the reference's
// un-vendored mlcc library, INIReaderBin):
//     bytes 0..31   "CFG_BIN INI" padded with zeros
//     bytes 32..39  little-endian uint64: length L of the index text
//     L bytes       ASCII lines  "<key> = <offset>,<length>\n"   (offsets relative to the data area)
//     rest          data area
// Keys of a model file: "weight_<dtype>_<name>" with dtype in {fp8_e4m3, fp8e4m3, fp8, bf16, bfloat16,
// float, half, fp8_e5m2, fp4_e2m1} (cccc/Net.cpp:238-248), the legacy "weight_<name>" (FP8_E4M3),
// "scale_<name>" / "input_scale_<name>" (one float32), "blockscale_<name>" (FP4: one E4M3 byte per
// 16 elements, or legacy float32 per block).  Loading follows Net::loadNamedWeights
// (cccc/Net.cpp:1324-1527).  The file is memory-mapped, never read whole.
#pragma once
#include "Matrix.h"
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace cccc
{

// Host-side scalar conversions the loader needs, exposed for tests.
uint8_t floatToE4m3Truncated(float f);
uint16_t halfBitsToBf16Truncated(uint16_t h);

class WeightFile
{
public:
    WeightFile() = default;
    ~WeightFile();
    WeightFile(const WeightFile&) = delete;
    WeightFile& operator=(const WeightFile&) = delete;

    // 0 ok; -1 cannot open / map; -2 not a CFG_BIN INI file; -3 malformed index; -4 an entry lies outside the file
    int parseFile(const std::string& filename);
    void close();

    bool has_value(const std::string& key) const { return index_.count(key) != 0; }
    // Bytes of an entry ({nullptr, 0} when absent); valid while the file is open.
    std::pair<const uint8_t*, size_t> get_value(const std::string& key) const;
    const std::vector<std::string>& keys() const { return order_; }
    float loadFloat(const std::string& key, float default_val = 0.0f) const;

    struct WeightKey
    {
        std::string source;    // weight name
        std::string key;       // key of its bytes in the file
        DataType dt = CURRENT;
        bool is_quant = false;
        bool valid() const { return !source.empty(); }
    };
    // Typed quantized key first, then the legacy "weight_<name>" (FP8_E4M3), then a typed plain key
    // (cccc/Net.cpp:1376-1396).
    WeightKey resolve(const std::string& name) const;

    // Loads the weight `name` into m (cccc/Net.cpp:1429-1518): quantized bytes through
    // loadQuantizedDirect with scale_<name>, FP4 block scales (E4M3 bytes or legacy float32; surplus
    // bytes beyond elements / 16 are ignored), plain weights copied as they are (HALF converted to
    // BF16 by truncation when m is BF16; otherwise m takes the file's dtype).
    // 0 loaded; 1 not in the file; -1 byte count does not fit the tensor.
    int loadNamed(Matrix& m, const std::string& name) const;

    // Loads several quantized linear weights that share their input width into ONE storage, row ranges in the
    // order given (m is K x sum of their rows): the file bytes are uploaded unchanged, one after the other, FP4 block
    // scales likewise, and the storage gets one tiled copy.  A GEMV on m then serves all of them in one launch and
    // Matrix::rowsView hands each projection its own tensor.  All members must have the same data type and the same
    // per-tensor scale (the one GEMM call has one).  0 ok; 1 a name is missing; -1 sizes, types or scales do not fit.
    int loadNamedGroup(Matrix& m, const std::vector<std::string>& names) const;

private:
    struct Entry
    {
        uint64_t offset, length;
    };
    int fd_ = -1;
    const uint8_t* map_ = nullptr;
    size_t map_bytes_ = 0;
    const uint8_t* data_ = nullptr;    // start of the data area
    size_t data_bytes_ = 0;
    std::unordered_map<std::string, Entry> index_;
    std::vector<std::string> order_;
};

// Writer of the same container: what the reference's INIReaderBin::set_value / save do for
// Net::saveNamedWeights (cccc/Net.cpp:1235-1314), in the byte layout of scripts/convert_weights.py:54-83.
// Entries are written in the order they were added.  A tensor entry is not buffered on the host: its bytes
// are copied from the device in slabs while the file is written.
class WeightFileWriter
{
public:
    void set_value(const std::string& key, const void* bytes, size_t n);
    void set_value(const std::string& key, const std::string& text) { set_value(key, text.data(), text.size()); }
    // n bytes of device memory, read when save() runs (the memory must stay valid until then)
    void set_device_value(const std::string& key, const void* device_ptr, size_t n);
    // Bytes written, or -1 (cannot create / short write / device copy failed).
    long long save(const std::string& filename) const;

private:
    struct Entry
    {
        std::string key;
        std::vector<uint8_t> host;
        const void* device = nullptr;
        size_t bytes = 0;
    };
    std::vector<Entry> entries_;
};

// "weight_<dtype>_<name>" suffix of a data type (cccc/Net.cpp:222-235); empty for types without one.
const char* weightTypeSuffix(DataType dt);

// One named weight as Net::saveNamedWeights stores it (cccc/Net.cpp:1274-1303): the raw bytes under
// "weight_<dtype>_<name>", "scale_<name>" (one float32) when the per-tensor scale is not 1, and
// "blockscale_<name>" (one E4M3 byte per 16 elements) for FP4.  An FP4 blob is sized as the converter sizes it,
// (elements + 1) / 2 bytes (scripts/convert_weights.py:363-365); the reference's own writer reserves one byte
// per element there (cccc/Net.cpp:1284), of which only the first half is data.
void addNamedWeight(WeightFileWriter& w, const std::string& name, const Matrix& m);

}    // namespace cccc
