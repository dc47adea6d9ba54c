// nc_dump — prints everything ncc::Reader finds in a NetCDF file (classic or NetCDF-4) in a canonical text form: dimensions,
// global attributes with their values, variables with type, element count and every value.  The tests compare the dumps of a
// classic file and of the same content in NetCDF-4 containers of several layouts.
//
//   nc_dump file.nc                          the dump
//   nc_dump --sweep file.nc first last tmp   damages one byte at a time (every offset in [first, last), four values each), writes
//                                            the copy to `tmp`, and reads everything in it; prints how many copies still read and
//                                            how many ended in an error.  Meant for the sanitizer build: a read outside a buffer
//                                            aborts the program there.
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <string>
#include <vector>

#include "NcClassic.h"

static void printValues(int type, const uint8_t* p, uint64_t count)
{
    for (uint64_t i = 0; i < count; i++) {
        switch (type) {
        case ncc::NC_BYTE: printf(" %d", ((const int8_t*)p)[i]); break;
        case ncc::NC_UBYTE: printf(" %u", p[i]); break;
        case ncc::NC_SHORT: { int16_t v; memcpy(&v, p + 2 * i, 2); printf(" %d", v); break; }
        case ncc::NC_USHORT: { uint16_t v; memcpy(&v, p + 2 * i, 2); printf(" %u", v); break; }
        case ncc::NC_INT: { int32_t v; memcpy(&v, p + 4 * i, 4); printf(" %d", v); break; }
        case ncc::NC_UINT: { uint32_t v; memcpy(&v, p + 4 * i, 4); printf(" %u", v); break; }
        case ncc::NC_INT64: { int64_t v; memcpy(&v, p + 8 * i, 8); printf(" %" PRId64, v); break; }
        case ncc::NC_UINT64: { uint64_t v; memcpy(&v, p + 8 * i, 8); printf(" %" PRIu64, v); break; }
        case ncc::NC_FLOAT: { uint32_t v; memcpy(&v, p + 4 * i, 4); printf(" f%08x", v); break; }
        case ncc::NC_DOUBLE: { uint64_t v; memcpy(&v, p + 8 * i, 8); printf(" d%016" PRIx64, v); break; }
        default: printf(" ?"); break;
        }
    }
}

// Reads every dimension, attribute and variable of a file; 0 = read, 1 = refused with an error.
static int readAll(const char* path)
{
    try {
        ncc::Reader nc(path);
        uint64_t sum = nc.dims().size();
        for (const auto& n : nc.attNames()) sum += nc.att(n).raw.size();
        for (const auto& v : nc.vars()) {
            std::vector<uint8_t> raw;
            nc.readBytes(v.name, raw);
            for (uint8_t b : raw) sum += b;
        }
        return sum == ~0ull ? 1 : 0;
    } catch (const std::exception&) {
        return 1;
    }
}

static int sweep(const char* path, size_t first, size_t last, const char* tmp)
{
    FILE* f = fopen(path, "rb");
    if (!f) return 2;
    std::vector<uint8_t> data;
    uint8_t buf[65536];
    for (size_t n; (n = fread(buf, 1, sizeof buf, f)) > 0;) data.insert(data.end(), buf, buf + n);
    fclose(f);
    last = std::min(last, data.size());
    size_t ok = 0, refused = 0;
    for (size_t at = first; at < last; at++) {
        const uint8_t orig = data[at];
        const uint8_t values[4] = {0x00, 0xFF, (uint8_t)(orig ^ 0x80), (uint8_t)(orig + 1)};
        for (uint8_t v : values) {
            if (v == orig) continue;
            data[at] = v;
            FILE* o = fopen(tmp, "wb");
            if (!o || fwrite(data.data(), 1, data.size(), o) != data.size()) return 2;
            fclose(o);
            (readAll(tmp) ? refused : ok)++;
        }
        data[at] = orig;
    }
    printf("sweep %s [%zu, %zu): %zu copies still read, %zu refused\n", path, first, last, ok, refused);
    return 0;
}

int main(int argc, char** argv)
{
    if (argc == 6 && strcmp(argv[1], "--sweep") == 0) return sweep(argv[2], strtoull(argv[3], nullptr, 10), strtoull(argv[4], nullptr, 10), argv[5]);
    if (argc < 2) {
        fprintf(stderr, "usage: nc_dump file.nc\n");
        return 2;
    }
    try {
        ncc::Reader nc(argv[1]);
        fprintf(stderr, "container %d\n", nc.version());
        std::vector<ncc::Dimension> dims = nc.dims();
        std::sort(dims.begin(), dims.end(), [](const ncc::Dimension& a, const ncc::Dimension& b) { return a.name < b.name; });
        for (const auto& d : dims) printf("dim %s %" PRIu64 "\n", d.name.c_str(), d.length);
        std::vector<std::string> names = nc.attNames();
        std::sort(names.begin(), names.end());
        for (const auto& n : names) {
            const ncc::Attribute& a = nc.att(n);
            if (a.type == ncc::NC_CHAR)
                printf("att %s text \"%s\"\n", n.c_str(), a.asString().c_str());
            else {
                printf("att %s type %d count %" PRIu64 ":", n.c_str(), a.type, a.count);
                printValues(a.type, a.raw.data(), a.count);
                printf("\n");
            }
        }
        std::vector<std::string> vnames;
        for (const auto& v : nc.vars()) vnames.push_back(v.name);
        std::sort(vnames.begin(), vnames.end());
        for (const auto& n : vnames) {
            const ncc::Variable& v = nc.var(n);
            std::vector<uint8_t> raw;
            nc.readBytes(n, raw);
            printf("var %s type %d count %" PRIu64 ":", n.c_str(), v.type, v.count);
            printValues(v.type, raw.data(), v.count);
            printf("\n");
        }
    } catch (const std::exception& e) {
        printf("error: %s\n", e.what());
        return 1;
    }
    return 0;
}
