#include "WeightFile.h"
#include <cstdio>
#include <cstring>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace cccc
{

namespace
{

const char kMagic[] = "CFG_BIN INI";

// suffix order of cccc/Net.cpp:238-248: the first match wins
const std::pair<const char*, DataType> kTypedWeightSuffixes[] = {
    { "fp8_e4m3", FP8_E4M3 }, { "fp8e4m3", FP8_E4M3 }, { "fp8", FP8_E4M3 }, { "bf16", BFLOAT16 }, { "bfloat16", BFLOAT16 },
    { "float", FLOAT },       { "half", HALF },        { "fp8_e5m2", FP8_E5M2 }, { "fp4_e2m1", FP4_E2M1 },
};

size_t typeBytes(DataType dt) { return dt == FLOAT ? 4 : dt == DOUBLE ? 8 : (dt == HALF || dt == BFLOAT16) ? 2 : 1; }

std::string trim(const std::string& s)
{
    size_t a = 0, b = s.size();
    while (a < b && (s[a] == ' ' || s[a] == '\t' || s[a] == '\r')) { a++; }
    while (b > a && (s[b - 1] == ' ' || s[b - 1] == '\t' || s[b - 1] == '\r')) { b--; }
    return s.substr(a, b - a);
}

bool parseU64(const std::string& s, uint64_t& out)
{
    if (s.empty() || s.size() > 19) { return false; }
    uint64_t v = 0;
    for (char c : s)
    {
        if (c < '0' || c > '9') { return false; }
        v = v * 10 + (uint64_t)(c - '0');
    }
    out = v;
    return true;
}

// IEEE half -> float -> BF16 by dropping the low 16 bits: the host conversion of cccc/types.h:43-48
uint16_t halfToBf16Truncated(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0)
    {
        if (man == 0) { bits = sign; }
        else
        {
            int e = -1;
            uint32_t m = man;
            do { e++; m <<= 1; } while (!(m & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((m & 0x3FFu) << 13);
        }
    }
    else if (exp == 31) { bits = sign | 0x7F800000u | (man << 13); }
    else { bits = sign | ((exp + 112) << 23) | (man << 13); }
    return (uint16_t)(bits >> 16);
}

}    // namespace

// float -> FP8_E4M3 byte as the reference's host type encodes it (cccc/types.h:92-137): mantissa
// truncated, |x| >= 512 and Inf saturate to 448 (0x7E), [480, 512) lands on 448 as well (the NaN
// code point is avoided), NaN -> 0x7F without sign, subnormals m * 2^-9.  Used for legacy float32
// block scales.
uint8_t floatToE4m3Truncated(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) { return 0x7F; }
    const uint8_t sign = (uint8_t)((u >> 31) << 7);
    const int exp = (int)((u >> 23) & 0xFFu) - 127;
    const uint32_t man = u & 0x7FFFFFu;
    if (exp > 8) { return (uint8_t)(sign | 0x7E); }
    if (exp < -6)                                            // below the smallest normal 2^-6
    {
        const int shift = 14 - exp;
        return shift >= 32 ? sign : (uint8_t)(sign | (((man | 0x800000u) >> shift) & 7u));
    }
    uint32_t m3 = man >> 20;
    if (exp == 8 && m3 == 7) { m3 = 6; }
    return (uint8_t)(sign | ((uint32_t)(exp + 7) << 3) | m3);
}

uint16_t halfBitsToBf16Truncated(uint16_t h) { return halfToBf16Truncated(h); }

WeightFile::~WeightFile() { close(); }

void WeightFile::close()
{
    if (map_) { munmap((void*)map_, map_bytes_); }
    if (fd_ >= 0) { ::close(fd_); }
    map_ = data_ = nullptr;
    map_bytes_ = data_bytes_ = 0;
    fd_ = -1;
    index_.clear();
    order_.clear();
}

int WeightFile::parseFile(const std::string& filename)
{
    close();
    fd_ = ::open(filename.c_str(), O_RDONLY);
    if (fd_ < 0) { return -1; }
    struct stat st;
    if (fstat(fd_, &st) != 0 || st.st_size < 40)
    {
        close();
        return st.st_size < 40 ? -2 : -1;
    }
    map_bytes_ = (size_t)st.st_size;
    void* p = mmap(nullptr, map_bytes_, PROT_READ, MAP_PRIVATE, fd_, 0);
    if (p == MAP_FAILED)
    {
        map_bytes_ = 0;
        close();
        return -1;
    }
    map_ = (const uint8_t*)p;
    if (std::memcmp(map_, kMagic, sizeof(kMagic) - 1) != 0)
    {
        close();
        return -2;
    }
    uint64_t ini_len = 0;
    for (int i = 7; i >= 0; i--) { ini_len = (ini_len << 8) | map_[32 + i]; }
    if (ini_len > map_bytes_ - 40)
    {
        close();
        return -3;
    }
    data_ = map_ + 40 + ini_len;
    data_bytes_ = map_bytes_ - 40 - (size_t)ini_len;
    const std::string ini((const char*)map_ + 40, (size_t)ini_len);
    size_t pos = 0;
    while (pos < ini.size())
    {
        size_t eol = ini.find('\n', pos);
        if (eol == std::string::npos) { eol = ini.size(); }
        const std::string line = trim(ini.substr(pos, eol - pos));
        pos = eol + 1;
        if (line.empty() || line[0] == '[' || line[0] == ';' || line[0] == '#') { continue; }
        const size_t eq = line.find('=');
        const size_t comma = line.find(',', eq == std::string::npos ? 0 : eq);
        Entry e{};
        if (eq == std::string::npos || comma == std::string::npos || !parseU64(trim(line.substr(eq + 1, comma - eq - 1)), e.offset)
            || !parseU64(trim(line.substr(comma + 1)), e.length))
        {
            close();
            return -3;
        }
        if (e.offset > data_bytes_ || e.length > data_bytes_ - e.offset)
        {
            close();
            return -4;
        }
        const std::string key = trim(line.substr(0, eq));
        if (!index_.count(key)) { order_.push_back(key); }
        index_[key] = e;
    }
    return 0;
}

std::pair<const uint8_t*, size_t> WeightFile::get_value(const std::string& key) const
{
    auto it = index_.find(key);
    if (it == index_.end()) { return { nullptr, 0 }; }
    return { data_ + it->second.offset, (size_t)it->second.length };
}

float WeightFile::loadFloat(const std::string& key, float default_val) const
{
    auto [p, n] = get_value(key);
    float v = default_val;
    if (p && n >= sizeof(float)) { std::memcpy(&v, p, sizeof(float)); }
    return v;
}

WeightFile::WeightKey WeightFile::resolve(const std::string& name) const
{
    std::string typed;
    DataType tdt = CURRENT;
    for (auto& [sfx, dt] : kTypedWeightSuffixes)
    {
        const std::string key = std::string("weight_") + sfx + "_" + name;
        if (has_value(key))
        {
            typed = key;
            tdt = dt;
            break;
        }
    }
    const bool is_q = Rocblas::isQuantized(tdt);
    if (!typed.empty() && is_q) { return { name, typed, tdt, true }; }
    const std::string old_key = "weight_" + name;
    if (has_value(old_key)) { return { name, old_key, FP8_E4M3, true }; }
    if (!typed.empty()) { return { name, typed, tdt, false }; }
    return {};
}

int WeightFile::loadNamed(Matrix& m, const std::string& name) const
{
    const WeightKey wk = resolve(name);
    if (!wk.valid()) { return 1; }
    auto [bytes, n_bytes] = get_value(wk.key);
    if (!bytes || n_bytes == 0) { return 1; }
    const int64_t elems = m.getDataSize();
    if (wk.is_quant)
    {
        const int64_t want = wk.dt == FP4_E2M1 ? (elems + 1) / 2 : elems;
        // the reference's own writer sizes FP4 blobs by the element count (cccc/Net.cpp:1284): only the packed half is data
        if ((int64_t)n_bytes < want || ((int64_t)n_bytes != want && !(wk.dt == FP4_E2M1 && (int64_t)n_bytes == elems))) { return -1; }
        m.loadQuantizedDirect(bytes, want, loadFloat("scale_" + wk.source, 1.0f), wk.dt);
        const float input_scale = loadFloat("input_scale_" + wk.source);
        if (input_scale > 0.0f) { m.setInputScale(input_scale); }
        if (wk.dt == FP4_E2M1)
        {
            auto [bs, bs_bytes] = get_value("blockscale_" + wk.source);
            if (bs && bs_bytes)
            {
                const unsigned block = Matrix::fp4BlockSize();
                const int64_t n_blocks = (elems + block - 1) / block;
                if ((int64_t)bs_bytes < n_blocks) { return -1; }
                if ((int64_t)bs_bytes / n_blocks >= 4)       // legacy float32 per block
                {
                    std::vector<uint8_t> codes((size_t)n_blocks);
                    for (int64_t i = 0; i < n_blocks; i++)
                    {
                        float f;
                        std::memcpy(&f, bs + 4 * i, 4);
                        codes[i] = floatToE4m3Truncated(f);
                    }
                    m.setBlockScaleFromHost(codes.data(), n_blocks);
                }
                else { m.setBlockScaleFromHost(bs, n_blocks); }
            }
        }
        return 0;
    }
    if (wk.dt == HALF && m.getDataType() == BFLOAT16 && (int64_t)n_bytes == elems * 2)
    {
        std::vector<uint16_t> buf((size_t)elems);
        for (int64_t i = 0; i < elems; i++)
        {
            uint16_t h;
            std::memcpy(&h, bytes + 2 * i, 2);
            buf[i] = halfToBf16Truncated(h);
        }
        return m.copyFromHost(buf.data(), buf.size() * 2) == 0 ? 0 : -1;
    }
    if ((int64_t)n_bytes != elems * (int64_t)typeBytes(wk.dt)) { return -1; }
    if (m.getDataType() != wk.dt) { m.retype(wk.dt); }
    return m.copyFromHost(bytes, n_bytes) == 0 ? 0 : -1;
}

int WeightFile::loadNamedGroup(Matrix& m, const std::vector<std::string>& names) const
{
    const int K = m.getWidth();
    const int64_t elems = m.getDataSize();
    if (names.empty() || K <= 0 || m.getChannel() != 1 || m.getNumber() != 1) { return -1; }
    DataType dt = CURRENT;
    float scale = 1.0f;
    std::vector<uint8_t> codes, scales;
    for (const std::string& name : names)
    {
        const WeightKey wk = resolve(name);
        if (!wk.valid()) { return 1; }
        auto [bytes, n_bytes] = get_value(wk.key);
        if (!wk.is_quant || !bytes || n_bytes == 0) { return -1; }
        const float s = loadFloat("scale_" + wk.source, 1.0f);
        if (dt == CURRENT) { dt = wk.dt; scale = s; }
        else if (wk.dt != dt || s != scale) { return -1; }
        const int64_t per_row = dt == FP4_E2M1 ? K / 2 : K;              // bytes per row
        if (dt == FP4_E2M1 && K % (2 * (int)Matrix::fp4BlockSize()) != 0) { return -1; }
        // whole rows only; an FP4 blob sized by elements (the reference's own writer) carries its data in the first half
        int64_t data_bytes = (int64_t)n_bytes;
        if (dt == FP4_E2M1 && data_bytes % (2 * per_row) == 0 && has_value("blockscale_" + wk.source) &&
            (int64_t)get_value("blockscale_" + wk.source).second * (int64_t)Matrix::fp4BlockSize() == data_bytes)
        {
            data_bytes /= 2;
        }
        if (data_bytes % per_row != 0) { return -1; }
        codes.insert(codes.end(), bytes, bytes + data_bytes);
        if (dt == FP4_E2M1)
        {
            auto [bs, bs_bytes] = get_value("blockscale_" + wk.source);
            const int64_t n_blocks = data_bytes * 2 / (int64_t)Matrix::fp4BlockSize();
            if (!bs || (int64_t)bs_bytes < n_blocks) { return -1; }
            scales.insert(scales.end(), bs, bs + n_blocks);
        }
    }
    const int64_t want = dt == FP4_E2M1 ? elems / 2 : elems;
    if ((int64_t)codes.size() != want) { return -1; }
    m.loadQuantizedDirect(codes.data(), want, scale, dt);
    if (dt == FP4_E2M1) { m.setBlockScaleFromHost(scales.data(), (int64_t)scales.size()); }
    return 0;
}

// ------------------------------------------------------------------ writer

void WeightFileWriter::set_value(const std::string& key, const void* bytes, size_t n)
{
    Entry e;
    e.key = key;
    e.host.assign((const uint8_t*)bytes, (const uint8_t*)bytes + n);
    e.bytes = n;
    entries_.push_back(std::move(e));
}

void WeightFileWriter::set_device_value(const std::string& key, const void* device_ptr, size_t n)
{
    Entry e;
    e.key = key;
    e.device = device_ptr;
    e.bytes = n;
    entries_.push_back(std::move(e));
}

long long WeightFileWriter::save(const std::string& filename) const
{
    std::string index;
    uint64_t offset = 0;
    for (const Entry& e : entries_)
    {
        index += e.key + " = " + std::to_string(offset) + "," + std::to_string(e.bytes) + "\n";
        offset += e.bytes;
    }
    FILE* f = std::fopen(filename.c_str(), "wb");
    if (!f) { return -1; }
    uint8_t head[40] = {};
    std::memcpy(head, kMagic, sizeof(kMagic) - 1);
    const uint64_t index_len = index.size();
    for (int i = 0; i < 8; i++) { head[32 + i] = (uint8_t)(index_len >> (8 * i)); }
    bool ok = std::fwrite(head, 1, sizeof(head), f) == sizeof(head) && std::fwrite(index.data(), 1, index.size(), f) == index.size();
    std::vector<uint8_t> slab;
    for (const Entry& e : entries_)
    {
        if (!ok) { break; }
        if (!e.device)
        {
            ok = e.bytes == 0 || std::fwrite(e.host.data(), 1, e.bytes, f) == e.bytes;
            continue;
        }
        const size_t kSlab = (size_t)64 << 20;
        slab.resize(e.bytes < kSlab ? e.bytes : kSlab);
        for (size_t done = 0; ok && done < e.bytes; done += kSlab)
        {
            const size_t n = e.bytes - done < kSlab ? e.bytes - done : kSlab;
            ok = GpuControl::copyDeviceToHost(slab.data(), (const uint8_t*)e.device + done, n) == 0 && std::fwrite(slab.data(), 1, n, f) == n;
        }
    }
    ok = (std::fclose(f) == 0) && ok;
    return ok ? (long long)(sizeof(head) + index.size() + offset) : -1;
}

const char* weightTypeSuffix(DataType dt)
{
    switch (dt)
    {
    case BFLOAT16: return "bf16";
    case FLOAT: return "float";
    case HALF: return "half";
    case DOUBLE: return "double";
    case FP8_E4M3: return "fp8_e4m3";
    case FP8_E5M2: return "fp8_e5m2";
    case FP4_E2M1: return "fp4_e2m1";
    default: return "";
    }
}

void addNamedWeight(WeightFileWriter& w, const std::string& name, const Matrix& m)
{
    const DataType dt = m.getDataType();
    const size_t n_bytes = dt == FP4_E2M1 ? (size_t)((m.getDataSize() + 1) / 2) : (size_t)m.getDataSize() * typeBytes(dt);
    const std::string suffix = weightTypeSuffix(dt);
    w.set_device_value(suffix.empty() ? "weight_" + name : "weight_" + suffix + "_" + name, m.data(), n_bytes);
    const float scale = m.getQuantScale();
    if (scale != 1.0f) { w.set_value("scale_" + name, &scale, sizeof(float)); }
    if (m.getBlockScaleData() && m.getBlockScaleCount() > 0)
    {
        w.set_device_value("blockscale_" + name, m.getBlockScaleData(), (size_t)m.getBlockScaleCount());
    }
}

}    // namespace cccc
