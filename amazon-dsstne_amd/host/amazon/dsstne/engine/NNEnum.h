// NNEnum.h — dataset enumerations shared with files written by the reference (ordinals of engine/NNEnum.h:9-47).
#ifndef DSSTNE_AMD_NNENUM_H
#define DSSTNE_AMD_NNENUM_H

#include <cstdint>
#include <stdexcept>

namespace NNDataSetEnums {

enum Attributes {
    Sparse = 1,
    Boolean = 2,
    Compressed = 4,
    Recurrent = 8,
    Mutable = 16,
    SparseIgnoreZero = 32,
    Indexed = 64,
    Weighted = 128
};

enum Kind { Numeric = 0, Image = 1, Audio = 2 };

enum Sharding { None = 0, Model = 1, Data = 2 };

enum DataType { UInt = 0, Int = 1, LLInt = 2, ULLInt = 3, Float = 4, Double = 5, RGB8 = 6, RGB16 = 7, UChar = 8, Char = 9 };

template <typename T> inline DataType getDataType() { throw std::runtime_error("Default data type not defined"); }
template <> inline DataType getDataType<uint32_t>() { return UInt; }
template <> inline DataType getDataType<int32_t>() { return Int; }
template <> inline DataType getDataType<int64_t>() { return LLInt; }
template <> inline DataType getDataType<uint64_t>() { return ULLInt; }
template <> inline DataType getDataType<float>() { return Float; }
template <> inline DataType getDataType<double>() { return Double; }
template <> inline DataType getDataType<char>() { return Char; }
template <> inline DataType getDataType<unsigned char>() { return UChar; }

}  // namespace NNDataSetEnums

#endif
