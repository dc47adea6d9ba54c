// classic_to_nc4 — writes the content of a classic NetCDF file (CDF-1/2/5, read with this repository's own ncc::Reader) as a
// NetCDF-4 file, i.e. an HDF5 container laid out the way the netCDF-C library lays it out, through the HDF5 library itself.
//
// TEST INFRASTRUCTURE: it makes the fixtures under tests/golden/nc4/ that pin the product's own HDF5 parser (NcHdf5.cpp) against
// bytes written by the real HDF5 library.  It needs an HDF5 installation (headers + libhdf5 + libhdf5_hl) and is only built
// when the fixtures are regenerated (see Makefile in this directory); nothing in the product or in the tests links to it.
//
// What netCDF-C does for a NetCDF-4 file, restated from its published file-format description ("NetCDF-4 format", appendix of
// the NetCDF Users Guide):
//   * creation order of links and attributes is tracked and indexed on the root group and on every dataset;
//   * a dimension is a one-dimensional dataset (a "dimension scale") named after the dimension, of type IEEE float big-endian,
//     whose NAME attribute is "This is a netCDF dimension but not a netCDF variable." followed by the length in a 10-character
//     field, with an integer attribute _Netcdf4Dimid; nothing is ever written into it;
//   * a variable is a dataset of the little-endian file type of its NetCDF type whose dimension scales are attached
//     (DIMENSION_LIST on the variable, REFERENCE_LIST on the scale);
//   * a text attribute is a scalar attribute of a fixed-length string type, a numeric attribute a one-dimensional one;
//   * the root group carries a text attribute _NCProperties.
//
// usage: classic_to_nc4 in.nc out.nc earliest|v18|latest|plain [chunk-elements]
//   earliest: superblock 0; object headers and the root group are still the new-style ones (version 2 headers, link messages or
//             a fractal heap), because tracking creation order needs them (what netCDF-C >= 4.4.1 writes);
//   plain:    as earliest, but without creation-order tracking: version 1 object headers and an old-style root group (B-tree of
//             symbol nodes + local heap) — not what netCDF-C writes, but what other HDF5 writers of the same content produce;
//   v18:      HDF5 1.8's newest structures: superblock 2, version 2 object headers, dense link and attribute storage
//             (what netCDF-C < 4.4.1 wrote);
//   latest:   this HDF5 library's newest structures (superblock 3, version 4 layout messages);
//   chunk-elements: variables are chunked in pieces of that many elements instead of contiguous.
#include <hdf5.h>
#include <hdf5_hl.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "NcClassic.h"

#define CHECK(x)                                                                  \
    do {                                                                          \
        if ((x) < 0) {                                                            \
            fprintf(stderr, "classic_to_nc4: %s failed (line %d)\n", #x, __LINE__); \
            exit(1);                                                              \
        }                                                                         \
    } while (0)

static hid_t fileType(int t)
{
    switch (t) {
    case ncc::NC_BYTE: return H5T_STD_I8LE;
    case ncc::NC_UBYTE: return H5T_STD_U8LE;
    case ncc::NC_SHORT: return H5T_STD_I16LE;
    case ncc::NC_USHORT: return H5T_STD_U16LE;
    case ncc::NC_INT: return H5T_STD_I32LE;
    case ncc::NC_UINT: return H5T_STD_U32LE;
    case ncc::NC_INT64: return H5T_STD_I64LE;
    case ncc::NC_UINT64: return H5T_STD_U64LE;
    case ncc::NC_FLOAT: return H5T_IEEE_F32LE;
    case ncc::NC_DOUBLE: return H5T_IEEE_F64LE;
    default: fprintf(stderr, "classic_to_nc4: type %d\n", t); exit(1);
    }
}

static void putTextAtt(hid_t obj, const char* name, const std::string& text)
{
    hid_t type = H5Tcopy(H5T_C_S1);
    CHECK(H5Tset_size(type, text.size() ? text.size() : 1));
    CHECK(H5Tset_strpad(type, H5T_STR_NULLTERM));
    hid_t space = H5Screate(text.size() ? H5S_SCALAR : H5S_NULL);
    hid_t att = H5Acreate2(obj, name, type, space, H5P_DEFAULT, H5P_DEFAULT);
    CHECK(att);
    if (text.size()) CHECK(H5Awrite(att, type, text.data()));
    H5Aclose(att); H5Sclose(space); H5Tclose(type);
}

int main(int argc, char** argv)
{
    if (argc < 4) {
        fprintf(stderr, "usage: classic_to_nc4 in.nc out.nc earliest|v18|latest|plain [chunk-elements]\n");
        return 2;
    }
    const std::string mode = argv[3];
    const hsize_t chunk = argc > 4 ? (hsize_t)atoll(argv[4]) : 0;
    ncc::Reader in(argv[1]);

    hid_t fapl = H5Pcreate(H5P_FILE_ACCESS);
    CHECK(H5Pset_fclose_degree(fapl, H5F_CLOSE_STRONG));
    const bool track = mode != "plain";
    const unsigned order = track ? (H5P_CRT_ORDER_TRACKED | H5P_CRT_ORDER_INDEXED) : 0;
    if (mode == "earliest" || mode == "plain") CHECK(H5Pset_libver_bounds(fapl, H5F_LIBVER_EARLIEST, H5F_LIBVER_V18));
    else if (mode == "v18") CHECK(H5Pset_libver_bounds(fapl, H5F_LIBVER_V18, H5F_LIBVER_V18));
    else CHECK(H5Pset_libver_bounds(fapl, H5F_LIBVER_LATEST, H5F_LIBVER_LATEST));
    hid_t fcpl = H5Pcreate(H5P_FILE_CREATE);
    CHECK(H5Pset_obj_track_times(fcpl, 0));
    CHECK(H5Pset_link_creation_order(fcpl, order));
    CHECK(H5Pset_attr_creation_order(fcpl, order));
    hid_t file = H5Fcreate(argv[2], H5F_ACC_TRUNC, fcpl, fapl);
    CHECK(file);
    hid_t root = H5Gopen2(file, "/", H5P_DEFAULT);
    CHECK(root);
    putTextAtt(root, "_NCProperties", "version=1|netcdflibversion=4.4.1|hdf5libversion=1.8.17");

    // global attributes, in the file's order
    for (const std::string& name : in.attNames()) {
        const ncc::Attribute& a = in.att(name);
        if (a.type == ncc::NC_CHAR) {
            putTextAtt(root, name.c_str(), std::string((const char*)a.raw.data(), (size_t)a.count));
            continue;
        }
        hsize_t n = a.count;
        hid_t space = H5Screate_simple(1, &n, NULL);
        hid_t att = H5Acreate2(root, name.c_str(), fileType(a.type), space, H5P_DEFAULT, H5P_DEFAULT);
        CHECK(att);
        hid_t mem = H5Tget_native_type(fileType(a.type), H5T_DIR_ASCEND);
        CHECK(H5Awrite(att, mem, a.raw.data()));
        H5Tclose(mem); H5Aclose(att); H5Sclose(space);
    }

    // dimensions: dimension scales without a variable
    std::vector<hid_t> scales;
    int dimid = 0;
    for (const ncc::Dimension& d : in.dims()) {
        hsize_t len = d.length;
        hid_t space = H5Screate_simple(1, &len, &len);
        hid_t dcpl = H5Pcreate(H5P_DATASET_CREATE);
        CHECK(H5Pset_obj_track_times(dcpl, 0));
        CHECK(H5Pset_attr_creation_order(dcpl, order));
        hid_t ds = H5Dcreate2(root, d.name.c_str(), H5T_IEEE_F32BE, space, H5P_DEFAULT, dcpl, H5P_DEFAULT);
        CHECK(ds);
        char label[128];
        snprintf(label, sizeof(label), "This is a netCDF dimension but not a netCDF variable.%10d", (int)d.length);
        CHECK(H5DSset_scale(ds, label));
        hid_t sspace = H5Screate(H5S_SCALAR);
        hid_t att = H5Acreate2(ds, "_Netcdf4Dimid", H5T_NATIVE_INT, sspace, H5P_DEFAULT, H5P_DEFAULT);
        CHECK(att);
        CHECK(H5Awrite(att, H5T_NATIVE_INT, &dimid));
        H5Aclose(att); H5Sclose(sspace);
        H5Pclose(dcpl); H5Sclose(space);
        scales.push_back(ds);
        dimid++;
    }

    // variables
    for (const ncc::Variable& v : in.vars()) {
        std::vector<hsize_t> shape;
        for (uint32_t id : v.dimIds) shape.push_back(in.dims()[id].length);
        hid_t space = H5Screate_simple((int)shape.size(), shape.data(), NULL);
        hid_t dcpl = H5Pcreate(H5P_DATASET_CREATE);
        CHECK(H5Pset_obj_track_times(dcpl, 0));
        CHECK(H5Pset_attr_creation_order(dcpl, order));
        if (chunk && shape.size() == 1 && shape[0] > 0) {
            hsize_t c = chunk < shape[0] ? chunk : shape[0];
            CHECK(H5Pset_chunk(dcpl, 1, &c));
        } else
            CHECK(H5Pset_layout(dcpl, H5D_CONTIGUOUS));
        hid_t ds = H5Dcreate2(root, v.name.c_str(), fileType(v.type), space, H5P_DEFAULT, dcpl, H5P_DEFAULT);
        CHECK(ds);
        hid_t mem = H5Tget_native_type(fileType(v.type), H5T_DIR_ASCEND);
        std::vector<uint8_t> raw;
        in.readBytes(v.name, raw);
        if (!raw.empty()) CHECK(H5Dwrite(ds, mem, H5S_ALL, H5S_ALL, H5P_DEFAULT, raw.data()));
        for (size_t i = 0; i < v.dimIds.size(); i++) CHECK(H5DSattach_scale(ds, scales[v.dimIds[i]], (unsigned)i));
        H5Tclose(mem); H5Dclose(ds); H5Pclose(dcpl); H5Sclose(space);
    }
    for (hid_t s : scales) H5Dclose(s);
    H5Gclose(root);
    H5Pclose(fcpl); H5Pclose(fapl);
    CHECK(H5Fclose(file));
    return 0;
}
