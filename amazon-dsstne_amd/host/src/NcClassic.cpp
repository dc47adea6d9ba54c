// NcClassic.cpp — classic NetCDF (CDF-1/2/5) header parsing and writing.  File layout per the NetCDF classic format
// specification: magic, numrecs, dim_list, gatt_list, var_list, then the variables' data, everything big-endian and
// padded to 4-byte boundaries; CDF-5 widens counts, sizes and offsets to 64 bits and adds the unsigned types.
#include "NcClassic.h"

#include <cstdio>
#include <cstring>
#include <fstream>

namespace ncc {

size_t typeSize(int t)
{
    switch (t) {
    case NC_BYTE: case NC_CHAR: case NC_UBYTE: return 1;
    case NC_SHORT: case NC_USHORT: return 2;
    case NC_INT: case NC_FLOAT: case NC_UINT: return 4;
    case NC_DOUBLE: case NC_INT64: case NC_UINT64: return 8;
    default: throw Error("unknown NetCDF type " + std::to_string(t));
    }
}

static void swapInPlace(uint8_t* p, size_t elemSize, uint64_t count)
{
    if (elemSize == 1) return;
    for (uint64_t i = 0; i < count; i++, p += elemSize)
        for (size_t a = 0, b = elemSize - 1; a < b; a++, b--) std::swap(p[a], p[b]);
}

template <typename T> static T rawAs(const uint8_t* p, int type, size_t i)
{
    switch (type) {
    case NC_BYTE: return (T)((const int8_t*)p)[i];
    case NC_CHAR: case NC_UBYTE: return (T)((const uint8_t*)p)[i];
    case NC_SHORT: { int16_t v; memcpy(&v, p + 2 * i, 2); return (T)v; }
    case NC_USHORT: { uint16_t v; memcpy(&v, p + 2 * i, 2); return (T)v; }
    case NC_INT: { int32_t v; memcpy(&v, p + 4 * i, 4); return (T)v; }
    case NC_UINT: { uint32_t v; memcpy(&v, p + 4 * i, 4); return (T)v; }
    case NC_FLOAT: { float v; memcpy(&v, p + 4 * i, 4); return (T)v; }
    case NC_DOUBLE: { double v; memcpy(&v, p + 8 * i, 8); return (T)v; }
    case NC_INT64: { int64_t v; memcpy(&v, p + 8 * i, 8); return (T)v; }
    case NC_UINT64: { uint64_t v; memcpy(&v, p + 8 * i, 8); return (T)v; }
    default: throw Error("unknown NetCDF type " + std::to_string(type));
    }
}

std::string Attribute::asString() const
{
    if (type != NC_CHAR) throw Error("attribute " + name + " is not text");
    std::string s((const char*)raw.data(), (size_t)count);
    while (!s.empty() && s.back() == '\0') s.pop_back();
    return s;
}

double Attribute::asDouble(size_t i) const
{
    if (type == NC_CHAR || i >= count) throw Error("attribute " + name + " is not numeric or too short");
    return rawAs<double>(raw.data(), type, i);
}

uint64_t Attribute::asUInt64(size_t i) const
{
    if (type == NC_CHAR || i >= count) throw Error("attribute " + name + " is not numeric or too short");
    return rawAs<uint64_t>(raw.data(), type, i);
}

namespace {

struct Cursor {
    std::ifstream& in;
    int version;
    const std::string& fname;
    uint64_t fileSize;   // no count in the header can exceed what the file holds

    void bytes(void* dst, size_t n)
    {
        in.read((char*)dst, (std::streamsize)n);
        if (!in) throw Error(fname + ": truncated NetCDF header");
    }
    uint32_t u32()
    {
        uint8_t b[4];
        bytes(b, 4);
        return ((uint32_t)b[0] << 24) | ((uint32_t)b[1] << 16) | ((uint32_t)b[2] << 8) | b[3];
    }
    uint64_t u64()
    {
        uint64_t hi = u32();
        return (hi << 32) | u32();
    }
    uint64_t count() { return version == 5 ? u64() : u32(); }   // NON_NEG
    uint64_t offset() { return version == 1 ? u32() : u64(); }
    std::string name()
    {
        uint64_t n = count();
        if (n > (1u << 20) || n > fileSize) throw Error(fname + ": implausible name length");
        std::string s((size_t)n, '\0');
        if (n) bytes(&s[0], (size_t)n);
        skipPad(n);
        return s;
    }
    void skipPad(uint64_t n)
    {
        uint8_t pad[4];
        size_t r = (size_t)((4 - (n & 3)) & 3);
        if (r) bytes(pad, r);
    }
    Attribute attribute()
    {
        Attribute a;
        a.name = name();
        a.type = (int)u32();
        a.count = count();
        size_t es = typeSize(a.type);
        if (a.count > fileSize / es) throw Error(fname + ": an attribute claims more values than the file holds");
        a.raw.resize((size_t)(a.count * es));
        if (!a.raw.empty()) bytes(a.raw.data(), a.raw.size());
        skipPad(a.count * es);
        swapInPlace(a.raw.data(), es, a.count);
        return a;
    }
    // tag + nelems, or ABSENT (zero tag, zero count)
    uint64_t listHeader(uint32_t expectTag)
    {
        uint32_t tag = u32();
        uint64_t n = count();
        if (tag == 0 && n == 0) return 0;
        if (tag != expectTag) throw Error(fname + ": malformed NetCDF header (list tag " + std::to_string(tag) + ")");
        return n;
    }
};

}  // namespace

bool isHdf5File(const std::string& fname)
{
    std::ifstream in(fname, std::ios::binary);
    char sig[8] = {0};
    in.read(sig, 8);
    static const char hdf5[8] = {'\x89', 'H', 'D', 'F', '\r', '\n', '\x1a', '\n'};
    return in && memcmp(sig, hdf5, 8) == 0;
}

Reader::Reader(const std::string& fname) : _fname(fname), _version(0)
{
    std::ifstream in(fname, std::ios::binary);
    if (!in) throw Error(fname + ": cannot open");
    char magic[4] = {0};
    in.read(magic, 4);
    if (!in || magic[0] != 'C' || magic[1] != 'D' || magic[2] != 'F' || (magic[3] != 1 && magic[3] != 2 && magic[3] != 5)) {
        if (isHdf5File(fname)) {
            in.close();
            _version = 4;
            parseHdf5(fname, _dims, _dimByName, _atts, _attOrder, _vars, _varByName);
            return;
        }
        throw Error(fname + ": neither a classic NetCDF file nor a NetCDF-4 (HDF5) one");
    }
    _version = magic[3];
    in.seekg(0, std::ios::end);
    const uint64_t fileSize = (uint64_t)in.tellg();
    in.seekg(4);
    Cursor c{in, _version, _fname, fileSize};
    c.count();   // numrecs: no record variables are used
    // (a list of n entries takes at least 8 n bytes of header)
    auto plausible = [&](uint64_t n, const char* what) {
        if (n > fileSize / 8) throw Error(_fname + ": the header claims more " + what + " than the file could hold");
        return n;
    };
    uint64_t ndims = plausible(c.listHeader(0x0A), "dimensions");
    for (uint64_t i = 0; i < ndims; i++) {
        Dimension d;
        d.name = c.name();
        d.length = c.count();
        _dimByName[d.name] = _dims.size();
        _dims.push_back(d);
    }
    uint64_t natts = plausible(c.listHeader(0x0C), "attributes");
    for (uint64_t i = 0; i < natts; i++) {
        Attribute a = c.attribute();
        if (!_atts.count(a.name)) _attOrder.push_back(a.name);
        _atts[a.name] = a;
    }
    uint64_t nvars = plausible(c.listHeader(0x0B), "variables");
    for (uint64_t i = 0; i < nvars; i++) {
        Variable v;
        v.name = c.name();
        uint64_t nd = plausible(c.count(), "dimensions of a variable");
        v.count = 1;
        for (uint64_t j = 0; j < nd; j++) {
            uint64_t id = _version == 5 ? c.u64() : c.u32();
            if (id >= _dims.size()) throw Error(_fname + ": variable " + v.name + " uses an unknown dimension");
            v.dimIds.push_back((uint32_t)id);
            const uint64_t len = _dims[(size_t)id].length;
            if (len != 0 && v.count > (1ull << 62) / len) throw Error(_fname + ": variable " + v.name + " has an implausible size");
            v.count *= len;
        }
        uint64_t nva = plausible(c.listHeader(0x0C), "attributes of a variable");
        for (uint64_t j = 0; j < nva; j++) c.attribute();
        v.type = (int)c.u32();
        c.count();   // vsize
        v.begin = c.offset();
        _varByName[v.name] = _vars.size();
        _vars.push_back(v);
    }
}

const Attribute& Reader::att(const std::string& name) const
{
    auto it = _atts.find(name);
    if (it == _atts.end()) throw Error(_fname + ": missing attribute " + name);
    return it->second;
}

uint64_t Reader::dim(const std::string& name) const
{
    auto it = _dimByName.find(name);
    if (it == _dimByName.end()) throw Error(_fname + ": missing dimension " + name);
    return _dims[it->second].length;
}

const Variable& Reader::var(const std::string& name) const
{
    auto it = _varByName.find(name);
    if (it == _varByName.end()) throw Error(_fname + ": missing variable " + name);
    return _vars[it->second];
}

void Reader::readRaw(const Variable& v, std::vector<uint8_t>& raw) const
{
    if (!v.unsupported.empty()) throw Error(_fname + ": variable " + v.name + " cannot be read: " + v.unsupported);
    std::ifstream in(_fname, std::ios::binary);
    if (!in) throw Error(_fname + ": cannot open");
    in.seekg(0, std::ios::end);
    const uint64_t fileSize = (uint64_t)in.tellg();
    size_t es = typeSize(v.type);
    // What a variable may claim: no more than the file can hold where its values are stored in one piece; for a chunked
    // variable no more than its chunks hold (DSSTNE writes every value, so every chunk exists); a variable that was declared
    // and never written reads as zeros, up to 256 MiB of them.
    uint64_t limit = (fileSize + v.inlineData.size() + 8) / es;
    if (v.hdf5 && v.chunked) {
        limit = 0;
        for (const Variable::Extent& e : v.extents) {
            if (e.count > fileSize) throw Error(_fname + ": variable " + v.name + " has a chunk larger than the file");
            limit += e.count;
        }
    } else if (v.hdf5 && !v.compact && v.begin == ~0ull)
        limit = (1ull << 28) / es;
    if (v.count > limit) throw Error(_fname + ": variable " + v.name + " claims more data than the file holds");
    raw.assign((size_t)(v.count * es), 0);
    auto readAt = [&](uint64_t offset, uint8_t* dst, uint64_t bytes) {
        if (offset > fileSize || bytes > fileSize - offset) throw Error(_fname + ": variable " + v.name + " is truncated");
        in.seekg((std::streamoff)offset);
        if (bytes) in.read((char*)dst, (std::streamsize)bytes);
        if (!in) throw Error(_fname + ": variable " + v.name + " is truncated");
    };
    if (!v.hdf5) {
        readAt(v.begin, raw.data(), raw.size());
        swapInPlace(raw.data(), es, v.count);
        return;
    }
    if (v.compact) {
        if (v.inlineData.size() < raw.size()) throw Error(_fname + ": variable " + v.name + " is truncated");
        memcpy(raw.data(), v.inlineData.data(), raw.size());
    } else if (v.chunked) {
        for (const Variable::Extent& e : v.extents) {
            if (e.first >= v.count) continue;
            const uint64_t n = std::min(e.count, v.count - e.first);   // the last chunk may reach beyond the variable
            if (e.first * es > raw.size() || n * es > raw.size() - e.first * es) throw Error(_fname + ": variable " + v.name + " has a chunk outside its extent");
            readAt(e.offset, raw.data() + e.first * es, n * es);
        }
    } else if (v.begin != ~0ull) {
        readAt(v.begin, raw.data(), raw.size());
    }
    if (!v.littleEndian) swapInPlace(raw.data(), es, v.count);
}

template <typename T> void Reader::read(const std::string& name, std::vector<T>& out) const
{
    const Variable& v = var(name);
    std::vector<uint8_t> raw;
    readRaw(v, raw);
    out.resize((size_t)v.count);
    for (size_t i = 0; i < out.size(); i++) out[i] = rawAs<T>(raw.data(), v.type, i);
}

template void Reader::read<float>(const std::string&, std::vector<float>&) const;
template void Reader::read<double>(const std::string&, std::vector<double>&) const;
template void Reader::read<uint32_t>(const std::string&, std::vector<uint32_t>&) const;
template void Reader::read<int32_t>(const std::string&, std::vector<int32_t>&) const;
template void Reader::read<uint64_t>(const std::string&, std::vector<uint64_t>&) const;
template void Reader::read<int64_t>(const std::string&, std::vector<int64_t>&) const;
template void Reader::read<char>(const std::string&, std::vector<char>&) const;
template void Reader::read<unsigned char>(const std::string&, std::vector<unsigned char>&) const;

// ---------------------------------------------------------------------------------------------------------------- writer

void Writer::putAttRaw(const std::string& name, int type, uint64_t count, const void* data)
{
    Attribute a;
    a.name = name;
    a.type = type;
    a.count = count;
    a.raw.assign((const uint8_t*)data, (const uint8_t*)data + count * typeSize(type));
    for (auto& e : _atts)
        if (e.name == name) {
            e = a;
            return;
        }
    _atts.push_back(a);
}

void Writer::putAttString(const std::string& name, const std::string& value) { putAttRaw(name, NC_CHAR, value.size(), value.data()); }
void Writer::putAttUInt(const std::string& name, uint32_t v) { putAttRaw(name, NC_UINT, 1, &v); }
void Writer::putAttInt(const std::string& name, int32_t v) { putAttRaw(name, NC_INT, 1, &v); }
void Writer::putAttUInt64(const std::string& name, uint64_t v) { putAttRaw(name, NC_UINT64, 1, &v); }
void Writer::putAttFloat(const std::string& name, float v) { putAttRaw(name, NC_FLOAT, 1, &v); }

uint32_t Writer::addDim(const std::string& name, uint64_t length)
{
    _dims.push_back(Dimension{name, length});
    return (uint32_t)_dims.size() - 1;
}

void Writer::addVar(const std::string& name, int type, uint32_t dimId, const void* data)
{
    _vars.push_back(PendingVar{name, type, dimId, data});
}

namespace {
struct Out {
    std::vector<uint8_t> buf;
    int version = 5;
    void cnt(uint64_t v)   // NON_NEG: 64-bit in CDF-5, 32-bit before
    {
        if (version == 5) u64(v); else u32((uint32_t)v);
    }
    void u32(uint32_t v)
    {
        for (int s = 24; s >= 0; s -= 8) buf.push_back((uint8_t)(v >> s));
    }
    void u64(uint64_t v)
    {
        u32((uint32_t)(v >> 32));
        u32((uint32_t)v);
    }
    void pad()
    {
        while (buf.size() & 3) buf.push_back(0);
    }
    void name(const std::string& s)
    {
        cnt(s.size());
        buf.insert(buf.end(), s.begin(), s.end());
        pad();
    }
    void values(int type, uint64_t count, const uint8_t* hostData)
    {
        size_t es = typeSize(type);
        size_t at = buf.size();
        buf.insert(buf.end(), hostData, hostData + count * es);
        swapInPlace(buf.data() + at, es, count);
        pad();
    }
};
}  // namespace

void Writer::write(const std::string& fname)
{
    // header size depends on the offsets only through fixed-width fields, so build it once with placeholder offsets
    if (_version != 5)
        for (auto& a : _atts)
            if (a.type > NC_DOUBLE) throw Error(fname + ": attribute " + a.name + " needs the CDF-5 container (unsigned / 64-bit type)");
    auto build = [&](const std::vector<uint64_t>& begins) {
        Out o;
        o.version = _version;
        o.buf = {'C', 'D', 'F', (uint8_t)_version};
        o.cnt(0);   // numrecs
        if (_dims.empty()) { o.u32(0); o.cnt(0); } else {
            o.u32(0x0A); o.cnt(_dims.size());
            for (auto& d : _dims) { o.name(d.name); o.cnt(d.length); }
        }
        if (_atts.empty()) { o.u32(0); o.cnt(0); } else {
            o.u32(0x0C); o.cnt(_atts.size());
            for (auto& a : _atts) { o.name(a.name); o.u32((uint32_t)a.type); o.cnt(a.count); o.values(a.type, a.count, a.raw.data()); }
        }
        if (_vars.empty()) { o.u32(0); o.cnt(0); } else {
            o.u32(0x0B); o.cnt(_vars.size());
            for (size_t i = 0; i < _vars.size(); i++) {
                auto& v = _vars[i];
                if (_version != 5 && v.type > NC_DOUBLE) throw Error(fname + ": variable " + v.name + " needs the CDF-5 container");
                o.name(v.name);
                o.cnt(1); o.cnt(v.dimId);
                o.u32(0); o.cnt(0);   // no variable attributes
                o.u32((uint32_t)v.type);
                uint64_t vsize = _dims[v.dimId].length * typeSize(v.type);
                o.cnt((vsize + 3) & ~3ull);
                o.u64(begins[i]);     // 64-bit offsets in CDF-2 and CDF-5
            }
        }
        return o.buf;
    };
    std::vector<uint64_t> begins(_vars.size(), 0);
    std::vector<uint8_t> header = build(begins);
    uint64_t pos = header.size();
    for (size_t i = 0; i < _vars.size(); i++) {
        begins[i] = pos;
        pos += ((_dims[_vars[i].dimId].length * typeSize(_vars[i].type)) + 3) & ~3ull;
    }
    header = build(begins);
    std::ofstream out(fname, std::ios::binary | std::ios::trunc);
    if (!out) throw Error(fname + ": cannot create");
    out.write((const char*)header.data(), (std::streamsize)header.size());
    std::vector<uint8_t> chunk;
    for (auto& v : _vars) {
        size_t es = typeSize(v.type);
        uint64_t count = _dims[v.dimId].length;
        const uint8_t* src = (const uint8_t*)v.data;
        const uint64_t step = (1u << 20);
        for (uint64_t at = 0; at < count; at += step) {
            uint64_t n = std::min(step, count - at);
            chunk.assign(src + at * es, src + (at + n) * es);
            swapInPlace(chunk.data(), es, n);
            out.write((const char*)chunk.data(), (std::streamsize)chunk.size());
        }
        static const char zeros[4] = {0, 0, 0, 0};
        size_t r = (size_t)((4 - ((count * es) & 3)) & 3);
        if (r) out.write(zeros, (std::streamsize)r);
    }
    if (!out) throw Error(fname + ": write failed");
}

}  // namespace ncc
