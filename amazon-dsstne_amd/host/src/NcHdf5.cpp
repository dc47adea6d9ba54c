// NcHdf5.cpp — read-only access to NetCDF-4 files, i.e. the HDF5 container the reference writes through netcdf-cxx4
// (NcFile(fname, NcFile::replace), engine/NNNetwork.cpp:1933, engine/NNTypes.cpp:2175, utils/NetCDFhelper.cpp:345).
//
// Only what such files contain is understood, parsed straight from the bytes per the HDF5 File Format Specification (version 3):
//   * superblock versions 0-3; object headers version 1 (with continuation blocks) and version 2 ("OHDR" / "OCHK");
//   * the root group only, old style (symbol table message: version 1 B-tree of "SNOD" nodes + local heap) or new style (link
//     messages in the header, or "dense" links in a fractal heap indexed by a version 2 B-tree);
//   * attributes in header messages (versions 1-3) or dense (fractal heap + version 2 B-tree); fixed-point, floating-point and
//     fixed-length string types of either byte order, scalar or one-dimensional; attributes of other types (the dimension
//     scales' reference lists) are skipped;
//   * datasets with compact, contiguous or chunked (version 1 B-tree index, no filters) layout, layout message versions 3 and 4;
//   * the NetCDF-4 conventions on top: a dataset whose CLASS attribute is "DIMENSION_SCALE" is a dimension (its length is the
//     dataset's extent; a NAME starting with "This is a netCDF dimension but not a netCDF variable" means it is nothing else),
//     every other dataset a variable, root attributes whose names start with "_NC" or "_nc" are the library's own.
// Anything else (compression filters, other chunk indexes, variable-length data, sub-groups) ends in an ncc::Error that says what
// was met.  Checksums are not verified.
#include <cstring>
#include <fstream>
#include <functional>
#include <set>

#include "NcClassic.h"

namespace ncc {

namespace {

constexpr uint64_t kUndef = ~0ull;

struct File {
    std::ifstream in;
    std::string fname;
    uint64_t size = 0;
    unsigned O = 8, L = 8;   // size of offsets / lengths
    uint64_t base = 0;

    explicit File(const std::string& f) : in(f, std::ios::binary), fname(f)
    {
        if (!in) throw Error(f + ": cannot open");
        in.seekg(0, std::ios::end);
        size = (uint64_t)in.tellg();
    }
    [[noreturn]] void fail(const std::string& what) const { throw Error(fname + ": HDF5: " + what); }
    std::vector<uint8_t> bytes(uint64_t at, uint64_t n)
    {
        if (at > size || n > size - at) fail("a structure at offset " + std::to_string(at) + " (" + std::to_string(n) + " bytes) lies beyond the end of the file");
        std::vector<uint8_t> b((size_t)n);
        in.clear();
        in.seekg((std::streamoff)at);
        if (n) in.read((char*)b.data(), (std::streamsize)n);
        if (!in) fail("read error at offset " + std::to_string(at));
        return b;
    }
};

// A bounds-checked little-endian cursor over a byte block.
struct Cur {
    const uint8_t* p;
    size_t n, at;
    const File& f;
    Cur(const std::vector<uint8_t>& b, const File& file, size_t start = 0) : p(b.data()), n(b.size()), at(start), f(file) {}
    Cur(const uint8_t* ptr, size_t len, const File& file) : p(ptr), n(len), at(0), f(file) {}
    void need(size_t k) const
    {
        if (k > n - std::min(at, n) || at > n) f.fail("a structure is shorter than its fields");
    }
    uint64_t u(unsigned bytes)
    {
        need(bytes);
        uint64_t v = 0;
        for (unsigned i = 0; i < bytes; i++) v |= (uint64_t)p[at + i] << (8 * i);
        at += bytes;
        return v;
    }
    uint8_t u8() { return (uint8_t)u(1); }
    uint16_t u16() { return (uint16_t)u(2); }
    uint32_t u32() { return (uint32_t)u(4); }
    uint64_t off() { uint64_t v = u(f.O); return (f.O < 8 && v == ((1ull << (8 * f.O)) - 1)) ? kUndef : v; }
    uint64_t len() { return u(f.L); }
    void skip(size_t k) { need(k); at += k; }
    void align8(size_t from) { size_t r = (at - from) & 7; if (r) skip(8 - r); }
    bool sig(const char* s)
    {
        need(4);
        bool ok = memcmp(p + at, s, 4) == 0;
        at += 4;
        return ok;
    }
    const uint8_t* here() const { return p + at; }
    size_t left() const { return at < n ? n - at : 0; }
    // Moves to an absolute position taken from fields of the file; a position beyond the block is an error, not a cursor.
    void seek(size_t to)
    {
        if (to > n) f.fail("a structure is shorter than its fields");
        at = to;
    }
};

struct Msg {
    unsigned type;
    unsigned flags;
    std::vector<uint8_t> data;
};

struct TypeInfo {
    int nc = 0;           // ncc::Type, 0 = not representable
    unsigned size = 0;    // bytes per element (string: its length)
    bool little = true;
    bool isString = false;
};

struct SpaceInfo {
    bool null = false;
    std::vector<uint64_t> dims;   // empty = scalar
    uint64_t count() const
    {
        if (null) return 0;
        uint64_t c = 1;
        for (uint64_t d : dims) c *= d;
        return c;
    }
};

struct Parser {
    File f;
    explicit Parser(const std::string& fname) : f(fname) {}

    uint64_t rootHeader = kUndef;
    uint64_t chunkEntries_ = 0;   // entries of chunk B-tree nodes visited so far, all variables together

    void superblock()
    {
        uint64_t at = 0;
        std::vector<uint8_t> b;
        for (;; at = at ? at * 2 : 512) {
            if (at + 8 > f.size) f.fail("no HDF5 superblock");
            b = f.bytes(at, 8);
            if (memcmp(b.data(), "\x89HDF\r\n\x1a\n", 8) == 0) break;
        }
        b = f.bytes(at, std::min<uint64_t>(f.size - at, 128));
        Cur c(b, f, 8);
        const unsigned version = c.u8();
        if (version <= 1) {
            c.skip(4);               // free-space version, root entry version, reserved, shared header version
            f.O = c.u8();
            f.L = c.u8();
            c.skip(1);
            c.skip(4);               // group leaf node K, group internal node K
            c.skip(4);               // consistency flags
            if (version == 1) c.skip(4);
            if ((f.O != 4 && f.O != 8) || (f.L != 4 && f.L != 8)) f.fail("offsets of " + std::to_string(f.O) + " bytes");
            f.base = c.off();
            c.off();                 // free-space info
            c.off();                 // end of file
            c.off();                 // driver info
            c.off();                 // root entry: link name offset
            rootHeader = c.off();
        } else if (version <= 3) {
            f.O = c.u8();
            f.L = c.u8();
            c.skip(1);
            if ((f.O != 4 && f.O != 8) || (f.L != 4 && f.L != 8)) f.fail("offsets of " + std::to_string(f.O) + " bytes");
            f.base = c.off();
            c.off();                 // superblock extension
            c.off();                 // end of file
            rootHeader = c.off();
        } else
            f.fail("superblock version " + std::to_string(version));
        if (f.base == kUndef) f.base = 0;
        f.base += 0;
        if (rootHeader == kUndef) f.fail("no root group");
    }

    uint64_t abs(uint64_t rel) const { return rel + f.base; }

    // ---- object headers ---------------------------------------------------------------------------------------------------
    std::vector<Msg> objectHeader(uint64_t addr)
    {
        std::vector<Msg> msgs;
        std::vector<uint8_t> head = f.bytes(abs(addr), std::min<uint64_t>(f.size - abs(addr), 64));
        if (head.size() >= 4 && memcmp(head.data(), "OHDR", 4) == 0)
            headerV2(addr, msgs);
        else
            headerV1(addr, msgs);
        return msgs;
    }

    void headerV1(uint64_t addr, std::vector<Msg>& msgs)
    {
        std::vector<uint8_t> h = f.bytes(abs(addr), 16);
        Cur c(h, f);
        if (c.u8() != 1) f.fail("object header at " + std::to_string(addr) + " has an unknown version");
        c.skip(1);
        unsigned nmsgs = c.u16();
        c.skip(4);
        uint64_t size = c.u32();
        std::vector<std::pair<uint64_t, uint64_t>> blocks{{abs(addr) + 16, size}};
        std::set<uint64_t> seen;
        for (size_t bi = 0; bi < blocks.size() && msgs.size() < nmsgs + 64u; bi++) {
            if (!seen.insert(blocks[bi].first).second) f.fail("object header continuation loop");
            std::vector<uint8_t> b = f.bytes(blocks[bi].first, blocks[bi].second);
            Cur m(b, f);
            while (m.left() >= 8) {
                Msg msg;
                msg.type = m.u16();
                unsigned sz = m.u16();
                msg.flags = m.u8();
                m.skip(3);
                if (sz > m.left()) f.fail("object header message overruns its block");
                msg.data.assign(m.here(), m.here() + sz);
                m.skip(sz);
                if (msg.type == 0x10) {
                    Cur k(msg.data, f);
                    uint64_t o = k.off(), l = k.len();
                    blocks.push_back({abs(o), l});
                } else if (msg.type != 0)
                    msgs.push_back(std::move(msg));
            }
        }
    }

    void headerV2(uint64_t addr, std::vector<Msg>& msgs)
    {
        std::vector<uint8_t> h = f.bytes(abs(addr), std::min<uint64_t>(f.size - abs(addr), 64));
        Cur c(h, f, 4);
        if (c.u8() != 2) f.fail("object header at " + std::to_string(addr) + " has an unknown version");
        const unsigned flags = c.u8();
        if (flags & 0x20) c.skip(16);
        if (flags & 0x10) c.skip(4);
        const uint64_t size0 = c.u(1u << (flags & 3));
        const bool order = (flags & 0x04) != 0;
        std::vector<std::pair<uint64_t, uint64_t>> blocks{{abs(addr) + c.at, size0}};   // message area (without the checksum)
        std::set<uint64_t> seen;
        for (size_t bi = 0; bi < blocks.size(); bi++) {
            if (!seen.insert(blocks[bi].first).second) f.fail("object header continuation loop");
            std::vector<uint8_t> b = f.bytes(blocks[bi].first, blocks[bi].second);
            Cur m(b, f);
            while (m.left() >= (order ? 6u : 4u)) {
                Msg msg;
                msg.type = m.u8();
                unsigned sz = m.u16();
                msg.flags = m.u8();
                if (order) m.skip(2);
                if (sz > m.left()) f.fail("object header message overruns its block");
                msg.data.assign(m.here(), m.here() + sz);
                m.skip(sz);
                if (msg.type == 0x10) {
                    Cur k(msg.data, f);
                    uint64_t o = k.off(), l = k.len();
                    if (l < 8) f.fail("object header continuation too short");
                    std::vector<uint8_t> s4 = f.bytes(abs(o), 4);
                    if (memcmp(s4.data(), "OCHK", 4) != 0) f.fail("object header continuation without signature");
                    blocks.push_back({abs(o) + 4, l - 8});
                } else if (msg.type != 0)
                    msgs.push_back(std::move(msg));
            }
        }
    }

    // ---- messages ------------------------------------------------------------------------------------------------------------
    TypeInfo datatype(Cur& c)
    {
        TypeInfo t;
        const unsigned cv = c.u8();
        const unsigned cls = cv & 15;
        const unsigned b0 = c.u8();
        c.skip(2);
        t.size = c.u32();
        switch (cls) {
        case 0: {   // fixed point
            t.little = (b0 & 1) == 0;
            const bool sgn = (b0 & 8) != 0;
            c.skip(4);
            if (t.size == 1) t.nc = sgn ? NC_BYTE : NC_UBYTE;
            else if (t.size == 2) t.nc = sgn ? NC_SHORT : NC_USHORT;
            else if (t.size == 4) t.nc = sgn ? NC_INT : NC_UINT;
            else if (t.size == 8) t.nc = sgn ? NC_INT64 : NC_UINT64;
            break;
        }
        case 1:   // floating point
            t.little = (b0 & 1) == 0;
            c.skip(12);
            if (t.size == 4) t.nc = NC_FLOAT;
            else if (t.size == 8) t.nc = NC_DOUBLE;
            break;
        case 3:   // fixed-length string
            t.nc = NC_CHAR;
            t.isString = true;
            break;
        default: break;   // not representable: the caller skips the attribute or refuses the variable
        }
        return t;
    }

    SpaceInfo dataspace(Cur& c)
    {
        SpaceInfo s;
        const unsigned version = c.u8();
        const unsigned rank = c.u8();
        const unsigned flags = c.u8();
        if (version == 1)
            c.skip(5);
        else if (version == 2) {
            const unsigned type = c.u8();
            if (type == 2) s.null = true;
        } else
            f.fail("dataspace message version " + std::to_string(version));
        if (rank > 32) f.fail("dataspace of rank " + std::to_string(rank));
        for (unsigned i = 0; i < rank; i++) s.dims.push_back(c.len());
        if (flags & 1) c.skip((size_t)rank * f.L);
        // the element count must stay a number that sizes and offsets can be computed from (16-byte elements at most)
        uint64_t product = 1;
        for (uint64_t d : s.dims) {
            if (d != 0 && product > (1ull << 58) / d) f.fail("a dataspace of more than 2^58 elements");
            product *= d;
        }
        return s;
    }

    // An attribute message; returns false when its type cannot be represented (the attribute is skipped).
    bool attributeMessage(const uint8_t* p, size_t n, Attribute& a)
    {
        Cur c(p, n, f);
        const unsigned version = c.u8();
        if (version < 1 || version > 3) f.fail("attribute message version " + std::to_string(version));
        const unsigned flags = c.u8();
        const unsigned nameSize = c.u16(), typeSize_ = c.u16(), spaceSize = c.u16();
        if (version == 3) c.skip(1);
        if (version >= 2 && (flags & 3)) return false;   // shared datatype or dataspace: not written for these files
        const size_t start = c.at;
        (void)start;
        c.need(nameSize);
        std::string name((const char*)c.here(), nameSize);
        while (!name.empty() && name.back() == '\0') name.pop_back();
        c.skip(nameSize);
        if (version == 1) c.skip((8 - (nameSize & 7)) & 7);
        size_t at = c.at;
        TypeInfo t = datatype(c);
        c.seek(at + typeSize_ + (version == 1 ? (8 - (typeSize_ & 7)) & 7 : 0));
        at = c.at;
        SpaceInfo s = dataspace(c);
        c.seek(at + spaceSize + (version == 1 ? (8 - (spaceSize & 7)) & 7 : 0));
        if (t.nc == 0 || s.dims.size() > 1) return false;
        a.name = name;
        a.type = t.nc;
        const uint64_t elems = s.count();
        if (t.isString) {
            // a text attribute is one fixed-length string (several of them are joined)
            a.count = elems * t.size;
            if (a.count > c.left()) f.fail("attribute " + name + " is longer than its message");
            a.raw.assign(c.here(), c.here() + a.count);
            while (a.count && a.raw[(size_t)a.count - 1] == 0) {
                a.raw.pop_back();
                a.count--;
            }
            return true;
        }
        a.count = elems;
        if (elems > c.left() / t.size) f.fail("attribute " + name + " is longer than its message");
        a.raw.assign(c.here(), c.here() + elems * t.size);
        if (!t.little)
            for (uint64_t i = 0; i < elems; i++)
                for (size_t x = 0, y = t.size - 1; x < y; x++, y--) std::swap(a.raw[i * t.size + x], a.raw[i * t.size + y]);
        return true;
    }

    // ---- local heap, version 1 B-trees, symbol table nodes ---------------------------------------------------------------------------
    void symbolTable(uint64_t btree, uint64_t heap, std::vector<std::pair<std::string, uint64_t>>& links)
    {
        std::vector<uint8_t> hh = f.bytes(abs(heap), 8 + 2 * f.L + f.O);
        Cur h(hh, f);
        if (!h.sig("HEAP")) f.fail("local heap signature");
        h.skip(4);
        const uint64_t dataSize = h.len();
        h.len();
        const uint64_t dataAddr = h.off();
        std::vector<uint8_t> names = f.bytes(abs(dataAddr), dataSize);
        std::function<void(uint64_t, int)> node = [&](uint64_t addr, int depth) {
            if (depth > 32) f.fail("group B-tree too deep");
            std::vector<uint8_t> hd = f.bytes(abs(addr), 8 + 2 * f.O);
            Cur c(hd, f);
            if (!c.sig("TREE")) {
                f.fail("group B-tree signature");
            }
            const unsigned type = c.u8(), level = c.u8(), used = c.u16();
            if (type != 0) f.fail("group B-tree of the wrong type");
            std::vector<uint8_t> body = f.bytes(abs(addr) + 8 + 2 * f.O, (uint64_t)used * (f.L + f.O) + f.L);
            Cur b(body, f);
            for (unsigned i = 0; i < used; i++) {
                b.len();   // key
                const uint64_t child = b.off();
                if (level > 0)
                    node(child, depth + 1);
                else {
                    std::vector<uint8_t> sh = f.bytes(abs(child), 8);
                    Cur s(sh, f);
                    if (!s.sig("SNOD")) f.fail("symbol table node signature");
                    s.skip(2);
                    const unsigned nsym = s.u16();
                    std::vector<uint8_t> eb = f.bytes(abs(child) + 8, (uint64_t)nsym * (2 * f.O + 24));
                    Cur e(eb, f);
                    for (unsigned k = 0; k < nsym; k++) {
                        const uint64_t nameOff = e.off();
                        const uint64_t hdr = e.off();
                        e.skip(24);
                        if (nameOff >= names.size()) f.fail("link name outside the local heap");
                        const char* s0 = (const char*)names.data() + nameOff;
                        links.push_back({std::string(s0, strnlen(s0, names.size() - (size_t)nameOff)), hdr});
                    }
                }
            }
        };
        node(btree, 0);
    }

    // ---- fractal heap + version 2 B-tree (dense links and attributes) ------------------------------------------------------------------
    struct FractalHeap {
        unsigned idLen = 0, flags = 0, maxHeapBits = 0, width = 0, curRows = 0, offBytes = 0, lenBytes = 0;
        uint64_t startSize = 0, maxDirect = 0, rootAddr = kUndef, maxManaged = 0;
        bool filtered = false;
        std::vector<std::pair<uint64_t, std::pair<uint64_t, uint64_t>>> blocks;   // heap offset -> (file address, size) of direct blocks
    };

    static unsigned log2u(uint64_t v)   // ceiling
    {
        unsigned b = 0;
        while (b < 63 && (1ull << b) < v) b++;
        return b;
    }
    static unsigned floorLog2(uint64_t v)
    {
        unsigned b = 0;
        while (v >>= 1) b++;
        return b;
    }

    FractalHeap openHeap(uint64_t addr)
    {
        FractalHeap h;
        std::vector<uint8_t> b = f.bytes(abs(addr), std::min<uint64_t>(f.size - abs(addr), 512));
        Cur c(b, f);
        if (!c.sig("FRHP")) f.fail("fractal heap signature");
        if (c.u8() != 0) f.fail("fractal heap version");
        h.idLen = c.u16();
        const unsigned filterLen = c.u16();
        h.flags = c.u8();
        h.maxManaged = c.u32();
        c.len();   // next huge id
        c.off();   // huge objects' B-tree
        c.len();   // free space
        c.off();   // free space manager
        c.len();   // managed space
        c.len();   // allocated managed space
        c.len();   // direct block allocation iterator
        c.len();   // managed objects
        c.len(); c.len();   // huge size, count
        c.len(); c.len();   // tiny size, count
        h.width = c.u16();
        h.startSize = c.len();
        h.maxDirect = c.len();
        h.maxHeapBits = c.u16();
        c.u16();   // starting rows of the root indirect block
        h.rootAddr = c.off();
        h.curRows = c.u16();
        h.filtered = filterLen != 0;
        if (h.filtered) f.fail("a filtered fractal heap (compressed attribute or link storage)");
        if (h.width == 0 || h.startSize == 0 || h.maxHeapBits > 64) f.fail("fractal heap parameters");
        h.offBytes = (h.maxHeapBits + 7) / 8;
        // length field of a managed object's ID: the lesser of the bytes that address a byte of the largest direct block and the
        // bytes that hold the largest managed object's size
        h.lenBytes = std::min((floorLog2(h.maxDirect) + 7) / 8, floorLog2(h.maxManaged) / 8 + 1);
        if (h.rootAddr == kUndef) return h;
        if (h.curRows == 0)
            h.blocks.push_back({0, {h.rootAddr, h.startSize}});
        else
            indirect(h, h.rootAddr, 0, h.curRows, 0);
        return h;
    }

    uint64_t rowSize(const FractalHeap& h, unsigned row) const { return row < 2 ? h.startSize : h.startSize << (row - 1); }

    void indirect(FractalHeap& h, uint64_t addr, uint64_t heapOff, unsigned rows, int depth)
    {
        if (depth > 8) f.fail("fractal heap too deep");
        const unsigned maxDirectRows = log2u(h.maxDirect) - log2u(h.startSize) + 2;
        uint64_t nDirect = 0, nIndirect = 0;
        for (unsigned r = 0; r < rows; r++) (r < maxDirectRows ? nDirect : nIndirect) += h.width;
        const uint64_t headLen = 5 + f.O + h.offBytes;
        std::vector<uint8_t> b = f.bytes(abs(addr), headLen + (nDirect + nIndirect) * f.O);
        Cur c(b, f);
        if (!c.sig("FHIB")) f.fail("fractal heap indirect block signature");
        c.skip(1 + f.O + h.offBytes);
        uint64_t off = heapOff;
        for (unsigned r = 0; r < rows; r++) {
            const uint64_t sz = rowSize(h, r);
            for (unsigned k = 0; k < h.width; k++) {
                const uint64_t child = c.off();
                if (r < maxDirectRows) {
                    if (child != kUndef) h.blocks.push_back({off, {child, sz}});
                } else if (child != kUndef) {
                    // an indirect child covering `sz` of heap space: as many rows as fit
                    unsigned childRows = log2u(sz) - log2u(h.startSize * h.width) + 1;
                    indirect(h, child, off, childRows, depth + 1);
                }
                off += sz;
            }
        }
    }

    // The object a heap ID names.
    std::vector<uint8_t> heapObject(const FractalHeap& h, const uint8_t* id, size_t idLen)
    {
        if (idLen < 1) f.fail("empty heap ID");
        const unsigned type = (id[0] >> 4) & 3;
        if (type == 2) {   // tiny: the object sits in the ID itself
            size_t n = (size_t)(id[0] & 15) + 1;
            if (1 + n > idLen) f.fail("tiny heap object longer than its ID");
            return std::vector<uint8_t>(id + 1, id + 1 + n);
        }
        if (type != 0) f.fail("a 'huge' fractal heap object (an attribute of more than a few kilobytes)");
        if (1 + h.offBytes + h.lenBytes > idLen) f.fail("heap ID too short");
        uint64_t off = 0, len = 0;
        for (unsigned i = 0; i < h.offBytes; i++) off |= (uint64_t)id[1 + i] << (8 * i);
        for (unsigned i = 0; i < h.lenBytes; i++) len |= (uint64_t)id[1 + h.offBytes + i] << (8 * i);
        for (const auto& blk : h.blocks)
            if (off >= blk.first && off - blk.first < blk.second.second) {
                if (len > blk.second.second - (off - blk.first)) f.fail("heap object crosses its block");
                return f.bytes(abs(blk.second.first) + (off - blk.first), len);
            }
        f.fail("heap object outside every direct block");
    }

    // Every record of a version 2 B-tree, in order.
    void btree2(uint64_t addr, unsigned expectType, const std::function<void(const uint8_t*, unsigned)>& record)
    {
        std::vector<uint8_t> hb = f.bytes(abs(addr), 4 + 2 + 4 + 2 + 2 + 2 + f.O + 2 + f.L + 4);
        Cur c(hb, f);
        if (!c.sig("BTHD")) f.fail("version 2 B-tree signature");
        if (c.u8() != 0) f.fail("version 2 B-tree version");
        const unsigned type = c.u8();
        if (type != expectType) f.fail("version 2 B-tree of type " + std::to_string(type) + " where " + std::to_string(expectType) + " was expected");
        const uint64_t nodeSize = c.u32();
        const unsigned recSize = c.u16();
        const unsigned depth = c.u16();
        c.skip(2);
        const uint64_t root = c.off();
        const unsigned rootRecs = c.u16();
        if (root == kUndef || rootRecs == 0) return;
        if (recSize == 0 || nodeSize < 32 || depth > 16) f.fail("version 2 B-tree parameters");
        // sizes of the "number of records" fields, level by level
        auto bytesFor = [](uint64_t v) { unsigned b = 0; do { b++; v >>= 8; } while (v); return b; };
        std::vector<uint64_t> maxRec(depth + 1), cumMax(depth + 1);
        std::vector<unsigned> cumBytes(depth + 1);
        maxRec[0] = (nodeSize - 10) / recSize;
        cumMax[0] = maxRec[0];
        cumBytes[0] = 0;
        const unsigned nrecBytes = bytesFor(maxRec[0]);   // one width for every level: that of a full leaf's count
        for (unsigned u = 1; u <= depth; u++) {
            const unsigned ptr = f.O + nrecBytes + cumBytes[u - 1];
            maxRec[u] = (nodeSize - 10 - ptr) / (recSize + ptr);
            cumMax[u] = (maxRec[u] + 1) * cumMax[u - 1] + maxRec[u];
            cumBytes[u] = bytesFor(cumMax[u]);
        }
        std::function<void(uint64_t, unsigned, unsigned)> node = [&](uint64_t at, unsigned nrec, unsigned level) {
            std::vector<uint8_t> nb = f.bytes(abs(at), nodeSize);
            Cur n(nb, f);
            if (!n.sig(level ? "BTIN" : "BTLF")) f.fail("version 2 B-tree node signature");
            n.skip(2);
            if ((uint64_t)nrec * recSize > n.left()) f.fail("version 2 B-tree node overfull");
            const uint8_t* recs = n.here();
            n.skip((size_t)nrec * recSize);
            if (level == 0) {
                for (unsigned i = 0; i < nrec; i++) record(recs + (size_t)i * recSize, recSize);
                return;
            }
            std::vector<std::pair<uint64_t, unsigned>> children;
            for (unsigned i = 0; i <= nrec; i++) {
                const uint64_t child = n.off();
                const unsigned cn = (unsigned)n.u(nrecBytes);
                if (level > 1) n.skip(cumBytes[level - 1]);
                children.push_back({child, cn});
            }
            for (unsigned i = 0; i <= nrec; i++) {
                node(children[i].first, children[i].second, level - 1);
                if (i < nrec) record(recs + (size_t)i * recSize, recSize);
            }
        };
        node(root, rootRecs, depth);
    }

    // ---- objects ---------------------------------------------------------------------------------------------------------------------------
    void attributesOf(const std::vector<Msg>& msgs, std::vector<Attribute>& out)
    {
        for (const Msg& m : msgs) {
            if (m.type == 0x0C) {
                if (m.flags & 2) continue;   // shared message: not written for these files
                Attribute a;
                if (attributeMessage(m.data.data(), m.data.size(), a)) out.push_back(std::move(a));
            } else if (m.type == 0x15) {
                Cur c(m.data, f);
                if (c.u8() != 0) f.fail("attribute info message version");
                const unsigned flags = c.u8();
                if (flags & 1) c.skip(2);
                const uint64_t heapAddr = c.off();
                const uint64_t nameTree = c.off();
                if (heapAddr == kUndef || nameTree == kUndef) continue;
                FractalHeap h = openHeap(heapAddr);
                btree2(nameTree, 8, [&](const uint8_t* rec, unsigned recSize) {
                    if (recSize < 9) f.fail("attribute index record too short");
                    if (rec[8] & 2) return;   // a shared attribute message
                    std::vector<uint8_t> obj = heapObject(h, rec, 8);
                    Attribute a;
                    if (attributeMessage(obj.data(), obj.size(), a)) out.push_back(std::move(a));
                });
            }
        }
    }

    void linkMessage(const uint8_t* p, size_t n, std::vector<std::pair<std::string, uint64_t>>& links)
    {
        Cur c(p, n, f);
        if (c.u8() != 1) f.fail("link message version");
        const unsigned flags = c.u8();
        unsigned type = 0;
        if (flags & 8) type = c.u8();
        if (flags & 4) c.skip(8);
        if (flags & 16) c.skip(1);
        const uint64_t nameLen = c.u(1u << (flags & 3));
        c.need((size_t)nameLen);
        std::string name((const char*)c.here(), (size_t)nameLen);
        c.skip((size_t)nameLen);
        if (type != 0) return;   // soft and external links: not part of a NetCDF-4 file's data model
        links.push_back({name, c.off()});
    }

    void linksOf(const std::vector<Msg>& msgs, std::vector<std::pair<std::string, uint64_t>>& links)
    {
        for (const Msg& m : msgs) {
            if (m.type == 0x11) {
                Cur c(m.data, f);
                const uint64_t btree = c.off(), heap = c.off();
                symbolTable(btree, heap, links);
            } else if (m.type == 0x06) {
                linkMessage(m.data.data(), m.data.size(), links);
            } else if (m.type == 0x02) {
                Cur c(m.data, f);
                if (c.u8() != 0) f.fail("link info message version");
                const unsigned flags = c.u8();
                if (flags & 1) c.skip(8);
                const uint64_t heapAddr = c.off();
                const uint64_t nameTree = c.off();
                if (heapAddr == kUndef || nameTree == kUndef) continue;
                FractalHeap h = openHeap(heapAddr);
                btree2(nameTree, 5, [&](const uint8_t* rec, unsigned recSize) {
                    if (recSize < 4 + h.idLen) f.fail("link index record too short");
                    std::vector<uint8_t> obj = heapObject(h, rec + 4, h.idLen);
                    linkMessage(obj.data(), obj.size(), links);
                });
            }
        }
    }

    // Chunk addresses of a one-dimensional chunked dataset (version 1 B-tree, node type 1).
    void chunkTree(uint64_t addr, unsigned dimensionality, unsigned elemSize, std::vector<Variable::Extent>& out, int depth = 0)
    {
        if (depth > 32) f.fail("chunk B-tree too deep");
        std::vector<uint8_t> hd = f.bytes(abs(addr), 8 + 2 * f.O);
        Cur c(hd, f);
        if (!c.sig("TREE")) f.fail("chunk B-tree signature");
        const unsigned type = c.u8(), level = c.u8(), used = c.u16();
        if (type != 1) f.fail("chunk B-tree of the wrong type");
        const uint64_t keyLen = 8 + 8ull * dimensionality;
        // every entry of a real index occupies its own bytes of the file: more entries than the file has room for means the
        // tree's pointers run in a circle
        chunkEntries_ += used;
        if (chunkEntries_ > f.size / (keyLen + f.O) + 1) f.fail("chunk B-tree with more entries than the file can hold");
        std::vector<uint8_t> body = f.bytes(abs(addr) + 8 + 2 * f.O, used * (keyLen + f.O) + keyLen);
        Cur b(body, f);
        for (unsigned i = 0; i < used; i++) {
            const uint64_t bytes = b.u32();
            const uint32_t mask = b.u32();
            const uint64_t first = b.u(8);
            b.skip(8 * (dimensionality - 1));
            const uint64_t child = b.off();
            if (level > 0)
                chunkTree(child, dimensionality, elemSize, out, depth + 1);
            else {
                if (mask != 0) f.fail("a filtered chunk");
                out.push_back(Variable::Extent{first, bytes / elemSize, abs(child)});
            }
        }
    }

    void run(std::vector<Dimension>& dims, std::map<std::string, size_t>& dimByName, std::map<std::string, Attribute>& atts,
             std::vector<std::string>& attOrder, std::vector<Variable>& vars, std::map<std::string, size_t>& varByName)
    {
        superblock();
        std::vector<Msg> root = objectHeader(rootHeader);
        std::vector<Attribute> ra;
        attributesOf(root, ra);
        for (Attribute& a : ra)
            if (a.name.compare(0, 3, "_NC") != 0 && a.name.compare(0, 3, "_nc") != 0) {
                if (!atts.count(a.name)) attOrder.push_back(a.name);
                const std::string name = a.name;
                atts[name] = std::move(a);
            }
        std::vector<std::pair<std::string, uint64_t>> links;
        linksOf(root, links);
        for (const auto& link : links) {
            std::vector<Msg> msgs = objectHeader(link.second);
            const Msg *mt = nullptr, *ms = nullptr, *ml = nullptr;
            bool filtered = false;
            for (const Msg& m : msgs) {
                if (m.type == 0x03) mt = &m;
                else if (m.type == 0x01) ms = &m;
                else if (m.type == 0x08) ml = &m;
                else if (m.type == 0x0B) filtered = true;
            }
            if (!mt || !ms || !ml) continue;   // a group or a named datatype: not something DSSTNE writes
            std::vector<Attribute> da;
            attributesOf(msgs, da);
            bool scale = false, dimOnly = false;
            for (const Attribute& a : da) {
                if (a.name == "CLASS" && a.type == NC_CHAR && a.asString() == "DIMENSION_SCALE") scale = true;
                if (a.name == "NAME" && a.type == NC_CHAR && a.asString().compare(0, 52, "This is a netCDF dimension but not a netCDF variable") == 0)
                    dimOnly = true;
            }
            Cur cs(ms->data, f);
            SpaceInfo space = dataspace(cs);
            if (scale) {
                Dimension d;
                d.name = link.first;
                d.length = space.dims.empty() ? 1 : space.dims[0];
                dimByName[d.name] = dims.size();
                dims.push_back(d);
                if (dimOnly) continue;
            }
            Cur ct(mt->data, f);
            TypeInfo type = datatype(ct);
            Variable v;
            v.name = link.first;
            v.type = type.nc;
            v.count = space.count();
            v.littleEndian = type.little;
            v.hdf5 = true;
            v.begin = kUndef;
            if (type.nc == 0 || type.isString) {
                v.unsupported = "its values are of a type other than integers and floating-point numbers";
            } else if (filtered) {
                v.unsupported = "it is stored with a compression filter";
            } else {
                Cur cl(ml->data, f);
                const unsigned version = cl.u8();
                if (version != 3 && version != 4) f.fail("data layout message version " + std::to_string(version) + " (variable " + v.name + ")");
                const unsigned cls = cl.u8();
                if (cls == 0) {
                    const unsigned n = cl.u16();
                    cl.need(n);
                    v.inlineData.assign(cl.here(), cl.here() + n);
                    v.compact = true;
                } else if (cls == 1) {
                    const uint64_t a = cl.off();
                    cl.len();
                    v.begin = (a == kUndef) ? kUndef : abs(a);
                } else if (cls == 2 && version == 3) {
                    const unsigned dimensionality = cl.u8();
                    const uint64_t tree = cl.off();
                    if (dimensionality != 2) {
                        v.unsupported = "it is chunked in more than one dimension";
                    } else {
                        v.chunked = true;
                        if (tree != kUndef) chunkTree(tree, dimensionality, type.size, v.extents);
                    }
                } else
                    v.unsupported = "its chunks are indexed in a way this reader does not know (written with a newer HDF5 file format)";
            }
            varByName[v.name] = vars.size();
            vars.push_back(std::move(v));
        }
    }
};

}  // namespace

void parseHdf5(const std::string& fname, std::vector<Dimension>& dims, std::map<std::string, size_t>& dimByName,
               std::map<std::string, Attribute>& atts, std::vector<std::string>& attOrder, std::vector<Variable>& vars,
               std::map<std::string, size_t>& varByName)
{
    Parser p(fname);
    p.run(dims, dimByName, atts, attOrder, vars, varByName);
}

}  // namespace ncc
