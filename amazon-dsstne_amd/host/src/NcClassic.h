// NcClassic.h — minimal reader/writer for classic-model NetCDF files (CDF-1, CDF-2 and CDF-5 on-disk formats).
//
// Network and dataset files keep the reference's attribute, dimension and variable names.  The reference writes them
// through netcdf-cxx4 as NetCDF-4 (an HDF5 container); this build reads and writes the classic container, whose CDF-5
// variant carries the same unsigned 32/64-bit types.  `nccopy -k cdf5 in.nc out.nc` converts a reference file.
// Only fixed-size variables and global attributes are supported (that is all DSSTNE files contain).
#ifndef DSSTNE_AMD_NCCLASSIC_H
#define DSSTNE_AMD_NCCLASSIC_H

#include <cstdint>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace ncc {

enum Type { NC_BYTE = 1, NC_CHAR = 2, NC_SHORT = 3, NC_INT = 4, NC_FLOAT = 5, NC_DOUBLE = 6, NC_UBYTE = 7, NC_USHORT = 8, NC_UINT = 9,
            NC_INT64 = 10, NC_UINT64 = 11 };

size_t typeSize(int t);

struct Error : public std::runtime_error {
    explicit Error(const std::string& m) : std::runtime_error(m) {}
};

struct Attribute {
    std::string name;
    int type;
    uint64_t count;
    std::vector<uint8_t> raw;   // host byte order

    std::string asString() const;
    double asDouble(size_t i = 0) const;
    uint64_t asUInt64(size_t i = 0) const;
};

struct Dimension {
    std::string name;
    uint64_t length;
};

struct Variable {
    std::string name;
    int type;
    std::vector<uint32_t> dimIds;
    uint64_t count;     // product of the dimension lengths
    uint64_t begin;     // file offset of the data
};

class Reader {
public:
    explicit Reader(const std::string& fname);
    int version() const { return _version; }
    bool hasAtt(const std::string& name) const { return _atts.count(name) != 0; }
    const Attribute& att(const std::string& name) const;
    bool hasDim(const std::string& name) const { return _dimByName.count(name) != 0; }
    uint64_t dim(const std::string& name) const;
    bool hasVar(const std::string& name) const { return _varByName.count(name) != 0; }
    const Variable& var(const std::string& name) const;
    // Reads a whole variable, converting its stored type to T.
    template <typename T> void read(const std::string& name, std::vector<T>& out) const;

private:
    std::string _fname;
    int _version;
    std::vector<Dimension> _dims;
    std::map<std::string, size_t> _dimByName;
    std::map<std::string, Attribute> _atts;
    std::vector<Variable> _vars;
    std::map<std::string, size_t> _varByName;
    void readRaw(const Variable& v, std::vector<uint8_t>& raw) const;
};

// Writes CDF-5 by default; setVersion(2) selects the older 64-bit-offset container (signed types only).
class Writer {
public:
    void setVersion(int version) { _version = (version == 2) ? 2 : 5; }
    void putAttString(const std::string& name, const std::string& value);
    void putAttUInt(const std::string& name, uint32_t v);
    void putAttInt(const std::string& name, int32_t v);
    void putAttUInt64(const std::string& name, uint64_t v);
    void putAttFloat(const std::string& name, float v);
    uint32_t addDim(const std::string& name, uint64_t length);
    // data must stay alive until write() returns
    void addVar(const std::string& name, int type, uint32_t dimId, const void* data);
    void write(const std::string& fname);

private:
    struct PendingVar {
        std::string name;
        int type;
        uint32_t dimId;
        const void* data;
    };
    int _version = 5;
    std::vector<Attribute> _atts;
    std::vector<Dimension> _dims;
    std::vector<PendingVar> _vars;
    void putAttRaw(const std::string& name, int type, uint64_t count, const void* data);
};

bool isHdf5File(const std::string& fname);

}  // namespace ncc

#endif
