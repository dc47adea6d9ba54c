// NcClassic.h — minimal reader/writer for NetCDF files: the classic containers (CDF-1, CDF-2, CDF-5) are read and written,
// NetCDF-4 files (an HDF5 container, what the reference writes through netcdf-cxx4) are read (NcHdf5.cpp).
//
// Network and dataset files keep the reference's attribute, dimension and variable names.  Files written here use the CDF-5
// container, which carries the same unsigned 32/64-bit types.  Only fixed-size variables and global attributes are supported
// (that is all DSSTNE files contain).
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
    int type = 0;
    std::vector<uint32_t> dimIds;   // classic container only
    uint64_t count = 0;  // product of the dimension lengths
    uint64_t begin = 0;  // file offset of the data (contiguous storage); ~0: nothing was ever written (reads as zeros)
    // NetCDF-4 (HDF5) container only
    struct Extent {
        uint64_t first;    // index of the chunk's first element
        uint64_t count;    // elements stored in the chunk
        uint64_t offset;   // file offset
    };
    bool hdf5 = false;
    bool littleEndian = false;
    bool compact = false;             // the data sits in the object header: inlineData
    bool chunked = false;             // the data sits in the chunks listed in extents (absent chunks read as zeros)
    std::vector<uint8_t> inlineData;
    std::vector<Extent> extents;
    std::string unsupported;          // why the variable's data cannot be read (its presence and size still can)
};

class Reader {
public:
    explicit Reader(const std::string& fname);
    int version() const { return _version; }   // 1, 2, 5: classic containers; 4: NetCDF-4 (HDF5)
    bool hasAtt(const std::string& name) const { return _atts.count(name) != 0; }
    const Attribute& att(const std::string& name) const;
    bool hasDim(const std::string& name) const { return _dimByName.count(name) != 0; }
    uint64_t dim(const std::string& name) const;
    bool hasVar(const std::string& name) const { return _varByName.count(name) != 0; }
    const Variable& var(const std::string& name) const;
    // Everything the file holds, in the file's order.
    std::vector<std::string> attNames() const { return _attOrder; }
    const std::vector<Dimension>& dims() const { return _dims; }
    const std::vector<Variable>& vars() const { return _vars; }
    // A whole variable as stored, in host byte order.
    void readBytes(const std::string& name, std::vector<uint8_t>& raw) const { readRaw(var(name), raw); }
    // Reads a whole variable, converting its stored type to T.
    template <typename T> void read(const std::string& name, std::vector<T>& out) const;

private:
    std::string _fname;
    int _version;
    std::vector<Dimension> _dims;
    std::map<std::string, size_t> _dimByName;
    std::map<std::string, Attribute> _atts;
    std::vector<std::string> _attOrder;
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
// Fills the tables of a Reader from a NetCDF-4 (HDF5) file (NcHdf5.cpp).
void parseHdf5(const std::string& fname, std::vector<Dimension>& dims, std::map<std::string, size_t>& dimByName,
               std::map<std::string, Attribute>& atts, std::vector<std::string>& attOrder, std::vector<Variable>& vars,
               std::map<std::string, size_t>& varByName);

}  // namespace ncc

#endif
