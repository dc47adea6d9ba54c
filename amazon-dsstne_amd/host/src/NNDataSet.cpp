// NNDataSet.cpp — host side of the dataset classes: construction, validated loading, upload, and dispatch to the device
// kernels.  Behaviour follows the reference's engine/NNTypes.cpp (constructors :469-581, loaders :583-778, accessors
// :780-1000, single-process Shard :1835-1950, 2152-2158) and the dispatch in engine/NNTypes.h:478-545.
#include <algorithm>
#include <sstream>
#include <stdexcept>

#include <cstring>
#include "NcClassic.h"
#include "amazon/dsstne/engine/NNTypes.h"

using namespace std;

NNDataSetDimensions::NNDataSetDimensions() : NNDataSetDimensions(1, 1, 1) {}

NNDataSetDimensions::NNDataSetDimensions(uint32_t width, uint32_t height, uint32_t length)
    : _dimensions(0), _width(width), _height(height), _length(length)
{
    // only extents above 1 count: (1) is 0-D, (2) is 1-D (tst/amazon/dsstne/engine/TestNNDataSetDimensions.cpp:18-28)
    _dimensions = (width > 1 ? 1 : 0) + (height > 1 ? 1 : 0) + (length > 1 ? 1 : 0);
}

template <typename T> static NNDataSetBase* createTyped(const NNDataSetDescriptor& d)
{
    if (d._attributes & NNDataSetEnums::Sparse) return new NNDataSet<T>(d._examples, d._sparseDensity, d._dim, false, d._name);
    return new NNDataSet<T>(d._examples, d._dim, d._name);
}

NNDataSetBase* createNNDataSet(const NNDataSetDescriptor& descriptor)
{
    using NNDataSetEnums::DataType;
    if (!NNDataSetDescriptor::isSupported(descriptor._attributes)) {
        stringstream msg;
        msg << "Unsupported attributes " << descriptor._attributes << " for dataset " << descriptor._name;
        throw std::runtime_error(msg.str());
    }
    switch (descriptor._dataType) {
    case DataType::UInt: return createTyped<uint32_t>(descriptor);
    case DataType::Int: return createTyped<int>(descriptor);
    case DataType::Float: return createTyped<float>(descriptor);
    case DataType::Double: return createTyped<double>(descriptor);
    case DataType::Char: return createTyped<char>(descriptor);
    case DataType::UChar:
    case DataType::RGB8: return createTyped<uint8_t>(descriptor);
    default: {
        stringstream msg;
        msg << "Unsupported data type: " << descriptor._dataType << ". DataType must be one of: UInt, Int, Float, Double, Char, UChar, RGB8";
        throw std::runtime_error(msg.str());
    }
    }
}

NNDataSetBase::NNDataSetBase()
    : _name(""), _dataType(NNDataSetEnums::DataType::Float), _attributes(0), _examples(0), _uniqueExamples(0), _localExamples(0),
      _dimensions(0), _width(0), _height(0), _length(0), _stride(0), _sharding(NNDataSetEnums::Sharding::None), _minX(0), _maxX(0),
      _sparseDataSize(0), _sparseDensity(0), _bDenoising(false), _bDirty(true), _bStreaming(false), _bIndexed(false), _batch(0)
{
}

NNDataSetBase::NNDataSetBase(const string& name, NNDataSetEnums::DataType dataType, uint32_t examples, uint32_t uniqueExamples,
                             const NNDataSetDimensions& datasetDim)
    : _name(name), _dataType(dataType), _attributes(0), _examples(examples), _uniqueExamples(uniqueExamples), _localExamples(examples),
      _dimensions(datasetDim._dimensions), _width(datasetDim._width), _height(datasetDim._height), _length(datasetDim._length), _stride(0),
      _sharding(NNDataSetEnums::Sharding::None), _minX(0), _maxX(0), _sparseDataSize(0), _sparseDensity(0), _bDenoising(false),
      _bDirty(true), _bStreaming(false), _bIndexed(false), _batch(0)
{
}

NNDataSetBase::~NNDataSetBase()
{
    if (dsx_is_initialized()) {
        dsx_marker_destroy(_sparseSet._uploaded);
        for (auto& set : _parkedSparse) dsx_marker_destroy(set._state._uploaded);
    }
}

NNDataSetDimensions NNDataSetBase::GetDimensions() { return NNDataSetDimensions(_width, _height, _length); }

// ------------------------------------------------------------------------------------------------------------ construction

template <typename T>
NNDataSet<T>::NNDataSet(uint32_t examples, const NNDataSetDimensions& dim, const string& name)
    : NNDataSetBase(name, NNDataSetEnums::getDataType<T>(), examples, examples, dim)
{
    _sparseDensity = 1.0f;
    _stride = _width * _height * _length;
    _vData.resize((size_t)_stride * _examples);
    _pbData.reset(new GpuBuffer<T>(_vData.size(), false, _bStreaming));
}

template <typename T>
NNDataSet<T>::NNDataSet(uint32_t examples, uint32_t uniqueExamples, const NNDataSetDimensions& dim, const string& name)
    : NNDataSetBase(name, NNDataSetEnums::getDataType<T>(), examples, uniqueExamples, dim)
{
    _sparseDensity = 1.0f;
    _stride = _width * _height * _length;
    _attributes = NNDataSetEnums::Attributes::Indexed;
    _bIndexed = true;
    // _vData holds the unique rows, _vIndex the row number of every example
    _vData.resize((size_t)_stride * _uniqueExamples);
    _vIndex.resize(_examples, 0);
    _pbData.reset(new GpuBuffer<T>(_vData.size(), false, _bStreaming));
    _pbIndex.reset(new GpuBuffer<uint32_t>(_vIndex.size(), false, _bStreaming));
}

template <typename T>
NNDataSet<T>::NNDataSet(uint32_t examples, NNFloat sparseDensity, const NNDataSetDimensions& dim, bool isWeighted, const string& name)
    : NNDataSet(examples, examples, (size_t)(((double)(dim._width * dim._height * dim._length * examples)) * sparseDensity), dim, false,
                isWeighted, name)
{
    // the per-example stride of sparse data is end - start, so _stride stays 0
    _attributes = NNDataSetEnums::Attributes::Sparse;
    if (isWeighted) _attributes |= NNDataSetEnums::Attributes::Weighted;
}

template <typename T>
NNDataSet<T>::NNDataSet(uint32_t examples, uint32_t uniqueExamples, size_t sparseDataSize, const NNDataSetDimensions& dim, bool isIndexed,
                        bool isWeighted, const string& name)
    : NNDataSetBase(name, NNDataSetEnums::getDataType<T>(), examples, uniqueExamples, dim)
{
    _attributes = NNDataSetEnums::Attributes::Sparse;
    _sparseDataSize = sparseDataSize;
    _vSparseStart.resize(_uniqueExamples, 0);
    _vSparseEnd.resize(_uniqueExamples, 0);
    _vSparseData.resize(_sparseDataSize);
    _vSparseIndex.resize(_sparseDataSize, 0);

    // evenly spaced placeholder rows until real data is loaded (engine/NNTypes.cpp:540-554)
    if (_uniqueExamples > 0) {
        size_t sparseStride = (_sparseDataSize + _uniqueExamples - 1) / _uniqueExamples;
        // (clamped to the allocation: the rounded-up stride would otherwise run the last rows past the end of the buffers,
        // and these placeholder rows are what the priming prediction of DsstneContext reads)
        _vSparseStart[0] = 0;
        _vSparseEnd[0] = std::min<uint64_t>(sparseStride, _sparseDataSize);
        for (uint32_t i = 1; i < _uniqueExamples; ++i) {
            _vSparseStart[i] = _vSparseEnd[i - 1];
            _vSparseEnd[i] = std::min<uint64_t>(_vSparseStart[i] + sparseStride, _sparseDataSize);
        }
    }

    _pbSparseStart.reset(new GpuBuffer<uint64_t>(_vSparseStart.size(), false, _bStreaming));
    _pbSparseEnd.reset(new GpuBuffer<uint64_t>(_vSparseEnd.size(), false, _bStreaming));
    _pbSparseData.reset(new GpuBuffer<T>(_vSparseData.size(), false, _bStreaming));
    _pbSparseIndex.reset(new GpuBuffer<uint32_t>(_vSparseIndex.size(), false, _bStreaming));

    if (isIndexed) {
        _attributes |= NNDataSetEnums::Attributes::Indexed;
        _bIndexed = true;
        _vIndex.resize(_examples, 0);
        _pbIndex.reset(new GpuBuffer<uint32_t>(_vIndex.size(), false, _bStreaming));
    }
    if (isWeighted) {
        _attributes |= NNDataSetEnums::Attributes::Weighted;
        _vDataWeight.resize(_examples);
        _pbDataWeight.reset(new GpuBuffer<NNFloat>(_vDataWeight.size(), false, _bStreaming));
    }
}

template <typename T> NNDataSet<T>::~NNDataSet() {}

// ----------------------------------------------------------------------------------------------------------------- loading

template <typename T> void NNDataSet<T>::LoadDenseData(const void* srcData)
{
    CopyDenseData(srcData);
    _pbData->Upload(_vData.data());
}

template <typename T> void NNDataSet<T>::CopyDenseData(const void* srcData)
{
    if (_attributes & NNDataSetEnums::Attributes::Sparse) throw std::runtime_error("Cannot set dense data on a sparse NNDataSet");
    const T* src = static_cast<const T*>(srcData);
    copy(src, src + _vData.size(), _vData.data());
}

template <typename T> void NNDataSet<T>::checkSparseLoad(const uint64_t start0, const uint64_t dataLength) const
{
    if (!(_attributes & NNDataSetEnums::Attributes::Sparse)) throw std::runtime_error("Cannot set sparse data on a non sparse NNDataSet");
    if (start0 != 0) throw std::runtime_error("Sparse data should be zero indexed; srcSparseStart[0] != 0");
    if (dataLength > _vSparseData.size() || dataLength > _vSparseIndex.size()) {
        stringstream msg;
        msg << "Not enough space to store sparse data. Allocated: " << _vSparseData.size() << " Required: " << dataLength;
        throw std::length_error(msg.str());
    }
}

template <typename T> void NNDataSet<T>::uploadSparse()
{
    { void* marker = _sparseSet._uploaded; _sparseSet = SparseSetState(); _sparseSet._uploaded = marker; }   // the uploads below are ordered on every lane
    // The buffers were sized at construction (or by Shard); batches loaded later reuse them without reallocation.
    _pbSparseStart->Upload(_vSparseStart.data());
    _pbSparseEnd->Upload(_vSparseEnd.data());
    _pbSparseIndex->Upload(_vSparseIndex.data());
    if (_pbSparseData) _pbSparseData->Upload(_vSparseData.data());
    _bSparseHostStale = false;
}

template <typename T>
void NNDataSet<T>::CopySparseData(const uint64_t* srcSparseStart, const uint64_t* srcSparseEnd, const void* srcSparseData,
                                  const uint32_t* srcSparseIndex)
{
    if (!(_attributes & NNDataSetEnums::Attributes::Sparse)) throw std::runtime_error("Cannot set sparse data on a non sparse NNDataSet");
    checkSparseLoad(srcSparseStart[0], srcSparseEnd[_uniqueExamples - 1]);
    const uint64_t dataLength = srcSparseEnd[_uniqueExamples - 1];
    const T* src = static_cast<const T*>(srcSparseData);
    memcpy(_vSparseStart.data(), srcSparseStart, _uniqueExamples * sizeof(uint64_t));
    memcpy(_vSparseEnd.data(), srcSparseEnd, _uniqueExamples * sizeof(uint64_t));
    if (src) memcpy(_vSparseData.data(), src, dataLength * sizeof(T));   // (no values: a Boolean set, whose kernels never read them)
    memcpy(_vSparseIndex.data(), srcSparseIndex, dataLength * sizeof(uint32_t));
    _bSparseHostStale = false;
}

// The device arrays hold the latest load; the host vectors are brought up to date from them (everything queued is waited for).
template <typename T> void NNDataSet<T>::SyncSparseHostCopy()
{
    if (!_bSparseHostStale) return;
    _bSparseHostStale = false;
    dsxFatal(dsx_sync(), "NNDataSet::SyncSparseHostCopy");
    auto fetch = [](auto& vec, auto& buf) {
        if (!buf || vec.empty()) return;
        const size_t n = std::min<size_t>(vec.size(), buf->_length);
        dsxFatal(dsx_memcpy_d2h(vec.data(), buf->_pDevData, n * sizeof(vec[0])), "NNDataSet::SyncSparseHostCopy");
    };
    fetch(_vSparseStart, _pbSparseStart);
    fetch(_vSparseEnd, _pbSparseEnd);
    fetch(_vSparseIndex, _pbSparseIndex);
    if (!(_attributes & NNDataSetEnums::Attributes::Boolean)) fetch(_vSparseData, _pbSparseData);
}

// Queues the copies of one batch's arrays to the device, only as long as the batch's data (the buffers may be larger).  They go
// to the set of device arrays that the kernels in flight do not read, on the lane the next PredictBatch will use, and are
// ordered against that lane only.  False (and nothing done) when the device arrays are missing or too small.
template <typename T>
bool NNDataSet<T>::uploadSparseDirect(const uint64_t* srcSparseStart, const uint64_t* srcSparseEnd, const void* srcSparseData,
                                      const uint32_t* srcSparseIndex)
{
    const uint64_t dataLength = srcSparseEnd[_uniqueExamples - 1];
    const bool direct = _pbSparseStart && _pbSparseEnd && _pbSparseIndex && _pbSparseStart->_length >= _uniqueExamples &&
                        _pbSparseIndex->_length >= dataLength && (!_pbSparseData || _pbSparseData->_length >= dataLength);
    if (!direct) return false;
    {
        const int selected = dsx_get_lane();
        const int target = (s_nextLane >= 0 && s_nextLane < DSX_MAX_LANES) ? s_nextLane : 0;
        if (target != _sparseLane) {   // park the arrays of the lane that loaded last, take out the target lane's
            ParkedSparseSet& mine = _parkedSparse[_sparseLane];
            mine._pbSparseStart.swap(_pbSparseStart);
            mine._pbSparseEnd.swap(_pbSparseEnd);
            mine._pbSparseIndex.swap(_pbSparseIndex);
            mine._state = _sparseSet;
            _parkedSparseData[_sparseLane].swap(_pbSparseData);
            ParkedSparseSet& next = _parkedSparse[target];
            if (!next._pbSparseStart || next._pbSparseStart->_length < mine._pbSparseStart->_length ||
                next._pbSparseIndex->_length < mine._pbSparseIndex->_length) {   // first use, or the arrays have grown since (Shard)
                next._pbSparseStart.reset(new GpuBuffer<uint64_t>(mine._pbSparseStart->_length, false, _bStreaming));
                next._pbSparseEnd.reset(new GpuBuffer<uint64_t>(mine._pbSparseEnd->_length, false, _bStreaming));
                next._pbSparseIndex.reset(new GpuBuffer<uint32_t>(mine._pbSparseIndex->_length, false, _bStreaming));
                if (_parkedSparseData[_sparseLane]) _parkedSparseData[target].reset(new GpuBuffer<T>(_parkedSparseData[_sparseLane]->_length, false, _bStreaming));
                next._state = SparseSetState();
                next._state._orderedLanes = 0;   // nothing has been loaded into it yet
            }
            _pbSparseStart.swap(next._pbSparseStart);
            _pbSparseEnd.swap(next._pbSparseEnd);
            _pbSparseIndex.swap(next._pbSparseIndex);
            _pbSparseData.swap(_parkedSparseData[target]);
            _sparseSet = next._state;
            _sparseLane = target;
        }
        if (target != selected) dsxFatal(dsx_set_lane(target), "NNDataSet::LoadSparseData");
        if (_sparseSet._readLanes & ~(1u << target)) dsxFatal(dsx_lane_wait_other(), "NNDataSet::LoadSparseData");   // readers on other lanes
        // The load before the last went into this set: once its copies are through, the device is at most two batches behind.
        // (A host that queues dozens of batches ahead makes the runtime stall in bursts of 150-200 us: measured 105-137 us per
        // batch of 1024 instead of 102.)
        if (!_sparseSet._uploaded) dsxFatal(dsx_marker_create(&_sparseSet._uploaded), "NNDataSet::LoadSparseData");
        else dsxFatal(dsx_marker_wait(_sparseSet._uploaded), "NNDataSet::LoadSparseData");
        {
            const bool values = _pbSparseData && srcSparseData;
            void* const dst[4] = {_pbSparseStart->_pDevData, _pbSparseEnd->_pDevData, _pbSparseIndex->_pDevData, values ? _pbSparseData->_pDevData : NULL};
            const void* const src[4] = {srcSparseStart, srcSparseEnd, srcSparseIndex, srcSparseData};
            const size_t bytes[4] = {_uniqueExamples * sizeof(uint64_t), _uniqueExamples * sizeof(uint64_t), dataLength * sizeof(uint32_t), dataLength * sizeof(T)};
            dsxFatal(dsx_memcpy_h2d_unordered_many(values ? 4 : 3, dst, src, bytes), "NNDataSet::LoadSparseData");
        }
        _sparseSet._uploadLane = target;
        _sparseSet._readLanes = 0;
        _sparseSet._orderedLanes = 1u << target;
        dsxFatal(dsx_marker_record(_sparseSet._uploaded), "NNDataSet::LoadSparseData");
        if (target != selected) dsxFatal(dsx_set_lane(selected), "NNDataSet::LoadSparseData");
    }
    return true;
}

template <typename T>
void NNDataSet<T>::LoadSparseData(const uint64_t* srcSparseStart, const uint64_t* srcSparseEnd, const void* srcSparseData,
                                  const uint32_t* srcSparseIndex)
{
    if (!(_attributes & NNDataSetEnums::Attributes::Sparse)) throw std::runtime_error("Cannot set sparse data on a non sparse NNDataSet");
    checkSparseLoad(srcSparseStart[0], srcSparseEnd[_uniqueExamples - 1]);
    if (!srcSparseData && !(_attributes & NNDataSetEnums::Attributes::Boolean)) throw std::runtime_error("NNDataSet::LoadSparseData: no values for a data set that is not Boolean");
    // Straight from the caller's arrays.  The host vectors are not filled here (that copy is a tenth of a request's round trip,
    // and the forward pass never reads them): they are marked stale and fetched back when something reads them.
    if (uploadSparseDirect(srcSparseStart, srcSparseEnd, srcSparseData, srcSparseIndex)) {
        _bSparseHostStale = true;
        return;
    }
    CopySparseData(srcSparseStart, srcSparseEnd, srcSparseData, srcSparseIndex);
    uploadSparse();
}

template <typename T>
void NNDataSet<T>::CopySparseData(const long* srcSparseStart, const long* srcSparseEnd, const void* srcSparseData, const long* srcSparseIndex)
{
    if (!(_attributes & NNDataSetEnums::Attributes::Sparse)) throw std::runtime_error("Cannot set sparse data on a non sparse NNDataSet");
    checkSparseLoad((uint64_t)srcSparseStart[0], (uint64_t)srcSparseEnd[_uniqueExamples - 1]);
    const uint64_t dataLength = (uint64_t)srcSparseEnd[_uniqueExamples - 1];
    const T* src = static_cast<const T*>(srcSparseData);
    for (uint32_t i = 0; i < _uniqueExamples; ++i) {
        _vSparseStart[i] = (uint64_t)srcSparseStart[i];
        _vSparseEnd[i] = (uint64_t)srcSparseEnd[i];
    }
    for (uint64_t i = 0; i < dataLength; ++i) {
        if (src) _vSparseData[i] = src[i];
        _vSparseIndex[i] = (uint32_t)srcSparseIndex[i];
    }
}

// (the arrays of a language without unsigned types are converted into the host vectors, which then are the source)
template <typename T>
void NNDataSet<T>::LoadSparseData(const long* srcSparseStart, const long* srcSparseEnd, const void* srcSparseData, const long* srcSparseIndex)
{
    if (!srcSparseData && !(_attributes & NNDataSetEnums::Attributes::Boolean)) throw std::runtime_error("NNDataSet::LoadSparseData: no values for a data set that is not Boolean");
    CopySparseData(srcSparseStart, srcSparseEnd, srcSparseData, srcSparseIndex);
    if (!uploadSparseDirect(_vSparseStart.data(), _vSparseEnd.data(), srcSparseData ? _vSparseData.data() : NULL, _vSparseIndex.data())) uploadSparse();
}

template <typename T> void NNDataSet<T>::LoadIndexedData(const uint32_t* srcIndexedData)
{
    if (!(_attributes & NNDataSetEnums::Attributes::Indexed)) throw std::runtime_error("Cannot set indexed data on a non indexed NNDataSet");
    copy(srcIndexedData, srcIndexedData + _vIndex.size(), _vIndex.data());
    _pbIndex->Upload(_vIndex.data());
}

template <typename T> void NNDataSet<T>::LoadDataWeight(const NNFloat* srcWeightData)
{
    if (!(_attributes & NNDataSetEnums::Attributes::Weighted)) throw std::runtime_error("Cannot set weight data on a non weighted NNDataSet");
    copy(srcWeightData, srcWeightData + _vDataWeight.size(), _vDataWeight.data());
    _pbDataWeight->Upload(_vDataWeight.data());
}

// --------------------------------------------------------------------------------------------------------------- accessors

static void fatalAccess(const char* msg)
{
    printf("%s\n", msg);
    getGpu().Shutdown();
    exit(-1);
}

template <typename T> T NNDataSet<T>::GetDataPoint(uint32_t n, uint32_t x, uint32_t y, uint32_t z)
{
    if (_attributes & NNDataSetEnums::Sparse) fatalAccess("NNDataSet::GetDataPoint: attempt to read non-sparse data from sparse data set.");
    if (n >= _examples) fatalAccess("NNDataSet::GetDataPoint: illegal example index.");
    if (_bIndexed) n = _vIndex[n];
    if ((x >= _width) || (y >= _height) || (z >= _length)) fatalAccess("NNDataSet::GetDataPoint: illegal datapoint coordinates.");
    return _vData[((size_t)n * _stride) + x + _width * (y + z * _height)];
}

template <typename T> bool NNDataSet<T>::SetDataPoint(T v, uint32_t n, uint32_t x, uint32_t y, uint32_t z)
{
    if (_attributes & NNDataSetEnums::Sparse) fatalAccess("NNDataSet::SetDataPoint: attempt to read non-sparse data from sparse data set.");
    if (n >= _examples) fatalAccess("NNDataSet::SetDataPoint: illegal example index.");
    if (_bIndexed) n = _vIndex[n];
    if ((x >= _width) || (y >= _height) || (z >= _length)) fatalAccess("NNDataSet::SetDataPoint: illegal datapoint coordinates.");
    _vData[((size_t)n * _stride) + x + _width * (y + z * _height)] = v;
    return true;
}

template <typename T> uint64_t NNDataSet<T>::GetSparseDataPoints(uint32_t n)
{
    if (!(_attributes & NNDataSetEnums::Sparse)) fatalAccess("NNDataSet::GetSparseDataPoints: attempt to read sparse data from non-sparse data set.");
    if (n >= _examples) fatalAccess("NNDataSet::GetSparseDataPoints: illegal example index.");
    SyncSparseHostCopy();
    if (_bIndexed) n = _vIndex[n];
    return _vSparseEnd[n] - _vSparseStart[n];
}

template <typename T> uint32_t NNDataSet<T>::GetSparseIndex(uint32_t n, uint32_t i)
{
    if (!(_attributes & NNDataSetEnums::Sparse)) fatalAccess("NNDataSet::GetSparseIndex: attempt to read sparse data from non-sparse data set.");
    if (n >= _examples) fatalAccess("NNDataSet::GetSparseIndex: illegal example index.");
    SyncSparseHostCopy();
    if (_bIndexed) n = _vIndex[n];
    if (i >= _vSparseEnd[n] - _vSparseStart[n]) fatalAccess("NNDataSet::GetSparseIndex: Sparse index out of range.");
    return _vSparseIndex[_vSparseStart[n] + i];
}

template <typename T> bool NNDataSet<T>::SetSparseIndex(uint32_t n, uint32_t i, uint32_t v)
{
    if (!(_attributes & NNDataSetEnums::Sparse)) fatalAccess("NNDataSet::SetSparseIndex: attempt to read sparse data from non-sparse data set.");
    if (n >= _examples) fatalAccess("NNDataSet::SetSparseIndex: illegal example index.");
    SyncSparseHostCopy();
    if (_bIndexed) n = _vIndex[n];
    if (i >= _vSparseEnd[n] - _vSparseStart[n]) fatalAccess("NNDataSet::SetSparseIndex: Sparse index out of range.");
    _vSparseIndex[_vSparseStart[n] + i] = v;
    _bDirty = true;
    return true;
}

template <typename T> T NNDataSet<T>::GetSparseDataPoint(uint32_t n, uint32_t i)
{
    if (!(_attributes & NNDataSetEnums::Sparse)) fatalAccess("NNDataSet::GetSparseDataPoint: attempt to read sparse data from non-sparse data set.");
    if (n >= _examples) fatalAccess("NNDataSet::GetSparseDataPoint: illegal example index.");
    SyncSparseHostCopy();
    if (_bIndexed) n = _vIndex[n];
    if (i >= _vSparseEnd[n] - _vSparseStart[n]) fatalAccess("NNDataSet::GetSparseDataPoint: Sparse index out of range.");
    return _vSparseData[_vSparseStart[n] + i];
}

template <typename T> bool NNDataSet<T>::SetSparseDataPoint(uint32_t n, uint32_t i, T v)
{
    if (!(_attributes & NNDataSetEnums::Sparse)) fatalAccess("NNDataSet::SetSparseDataPoint: attempt to read sparse data from non-sparse data set.");
    if (n >= _examples) fatalAccess("NNDataSet::SetSparseDataPoint: illegal example index.");
    SyncSparseHostCopy();
    if (_bIndexed) n = _vIndex[n];
    if (i >= _vSparseEnd[n] - _vSparseStart[n]) fatalAccess("NNDataSet::SetSparseDataPoint: Sparse index out of range.");
    _vSparseData[_vSparseStart[n] + i] = v;
    _bDirty = true;
    return true;
}

// ---------------------------------------------------------------------------------------------------------- device residency

// One process: "sharding" only (re)creates the device copies of the host vectors (engine/NNTypes.cpp:1940-1950, 2152-2158).
template <typename T> bool NNDataSet<T>::Shard(NNDataSetEnums::Sharding sharding)
{
    if (sharding == _sharding) return true;
    SyncSparseHostCopy();
    UnShard();
    _sharding = sharding;
    _minX = 0;
    _maxX = _width;
    _localExamples = _examples;
    if (_attributes & NNDataSetEnums::Sparse) {
        _pbSparseStart.reset(new GpuBuffer<uint64_t>(_vSparseStart.size(), false, _bStreaming));
        _pbSparseEnd.reset(new GpuBuffer<uint64_t>(_vSparseEnd.size(), false, _bStreaming));
        _pbSparseIndex.reset(new GpuBuffer<uint32_t>(_vSparseIndex.size(), false, _bStreaming));
        _pbSparseStart->Upload(_vSparseStart.data());
        _pbSparseEnd->Upload(_vSparseEnd.data());
        _pbSparseIndex->Upload(_vSparseIndex.data());
        if (!(_attributes & NNDataSetEnums::Boolean)) {
            _pbSparseData.reset(new GpuBuffer<T>(_vSparseData.size(), false, _bStreaming));
            _pbSparseData->Upload(_vSparseData.data());
        }
    } else {
        _pbData.reset(new GpuBuffer<T>(_vData.size(), false, _bStreaming));
        _pbData->Upload(_vData.data());
    }
    if (_attributes & NNDataSetEnums::Indexed) {
        _pbIndex.reset(new GpuBuffer<uint32_t>(_vIndex.size(), false, _bStreaming));
        _pbIndex->Upload(_vIndex.data());
    }
    if (_attributes & NNDataSetEnums::Weighted) {
        _pbDataWeight.reset(new GpuBuffer<NNFloat>(_vDataWeight.size(), false, _bStreaming));
        _pbDataWeight->Upload(_vDataWeight.data());
    }
    return true;
}

template <typename T> bool NNDataSet<T>::UnShard()
{
    _sharding = NNDataSetEnums::Sharding::None;
    return true;
}

template <typename T> bool NNDataSet<T>::SetDenoising(bool flag)
{
    if (flag) printf("NNDataSet::SetDenoising: denoising is a training feature and is not available in this build.\n");
    _bDenoising = false;
    return !flag;
}

int NNDataSetBase::s_nextLane = 0;

void NNDataSetBase::NoteSparseRead()
{
    const uint32_t lane = 1u << dsx_get_lane();
    if (_sparseSet._uploadLane >= 0 && !(_sparseSet._orderedLanes & lane)) {   // loaded on another lane: run after that copy
        dsxFatal(dsx_lane_wait_other(), "NNDataSetBase::NoteSparseRead");
        _sparseSet._orderedLanes |= lane;
    }
    _sparseSet._readLanes |= lane;
}

// ------------------------------------------------------------------------------------------------------------- device work

template <typename T> bool NNDataSet<T>::LoadInputUnit(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pUnit)
{
    const uint32_t* pIndex = (_attributes & NNDataSetEnums::Indexed) ? _pbIndex->_pDevData : NULL;
    dsxFatal(dsx_load_input_unit((uint32_t)_dataType, position, batch, stride, pUnit, pIndex, _pbData->_pDevData), "NNDataSet::LoadInputUnit");
    return true;
}

template <typename T> bool NNDataSet<T>::LoadSparseInputUnit(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pUnit)
{
    NoteSparseRead();
    dsxFatal(dsx_load_sparse_input_unit(_attributes, (uint32_t)_dataType, position, batch, stride, pUnit, _pbIndex ? _pbIndex->_pDevData : NULL,
                                        _pbSparseStart->_pDevData, _pbSparseEnd->_pDevData, _pbSparseIndex->_pDevData,
                                        _pbDataWeight ? _pbDataWeight->_pDevData : NULL, _pbSparseData ? _pbSparseData->_pDevData : NULL),
             "NNDataSet::LoadSparseInputUnit");
    return true;
}

template <typename T>
bool NNDataSet<T>::CalculateSparseZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, NNFloat* pUnit, NNFloat beta)
{
    NoteSparseRead();
    dsxFatal(dsx_sparse_z(_attributes, (uint32_t)_dataType, position, batch, stride, pWeight, _pbIndex ? _pbIndex->_pDevData : NULL,
                          _pbSparseStart->_pDevData, _pbSparseEnd->_pDevData, _pbSparseIndex->_pDevData,
                          _pbDataWeight ? _pbDataWeight->_pDevData : NULL, _pbSparseData ? _pbSparseData->_pDevData : NULL, pUnit, beta),
             "NNDataSet::CalculateSparseZ");
    return true;
}

template <typename T>
bool NNDataSet<T>::CalculateSparseLayer(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, NNFloat* pBias,
                                        Activation activation, NNFloat slope, NNFloat alpha, NNFloat lambda, NNFloat* pUnit)
{
    NoteSparseRead();
    dsx_act_params p = {slope, alpha, lambda};
    dsxFatal(dsx_sparse_layer_forward(_attributes, (uint32_t)_dataType, position, batch, stride, pWeight, _pbIndex ? _pbIndex->_pDevData : NULL,
                                      _pbSparseStart->_pDevData, _pbSparseEnd->_pDevData, _pbSparseIndex->_pDevData,
                                      _pbDataWeight ? _pbDataWeight->_pDevData : NULL, _pbSparseData ? _pbSparseData->_pDevData : NULL, pBias,
                                      (uint32_t)activation, &p, pUnit),
             "NNDataSet::CalculateSparseLayer");
    return true;
}

// ---------------------------------------------------------------------------------------------------------------- file I/O

namespace {

template <typename T> int ncTypeOf();
template <> int ncTypeOf<uint32_t>() { return ncc::NC_UINT; }
template <> int ncTypeOf<int32_t>() { return ncc::NC_INT; }
template <> int ncTypeOf<int64_t>() { return ncc::NC_INT64; }
template <> int ncTypeOf<uint64_t>() { return ncc::NC_UINT64; }
template <> int ncTypeOf<float>() { return ncc::NC_FLOAT; }
template <> int ncTypeOf<double>() { return ncc::NC_DOUBLE; }
template <> int ncTypeOf<char>() { return ncc::NC_BYTE; }
template <> int ncTypeOf<unsigned char>() { return ncc::NC_UBYTE; }

struct DataSetWriterHook {
    virtual ~DataSetWriterHook() {}
};

}  // namespace

// Writes dataset number n with the names the reference reader expects (engine/NNTypes.cpp:1090-1350).
template <typename T> static void writeDataSet(ncc::Writer& nc, NNDataSet<T>& d, uint32_t n)
{
    const string s = std::to_string(n);
    d.SyncSparseHostCopy();
    nc.putAttString("name" + s, d._name);
    nc.putAttUInt("attributes" + s, d._attributes);
    nc.putAttUInt("kind" + s, 0);
    nc.putAttUInt("dataType" + s, (uint32_t)d._dataType);
    nc.putAttUInt("dimensions" + s, d._dimensions);
    nc.putAttUInt("width" + s, d._width);
    if (d._dimensions > 1) nc.putAttUInt("height" + s, d._height);
    if (d._dimensions > 2) nc.putAttUInt("length" + s, d._length);
    const uint32_t uniqueDim = nc.addDim("uniqueExamplesDim" + s, d._uniqueExamples);
    const uint32_t examplesDim = nc.addDim("examplesDim" + s, d._examples);
    if (d._attributes & NNDataSetEnums::Sparse) {
        const uint32_t sparseDim = nc.addDim("sparseDataDim" + s, d._vSparseIndex.size());
        nc.addVar("sparseStart" + s, ncc::NC_UINT64, uniqueDim, d._vSparseStart.data());
        nc.addVar("sparseEnd" + s, ncc::NC_UINT64, uniqueDim, d._vSparseEnd.data());
        nc.addVar("sparseIndex" + s, ncc::NC_UINT, sparseDim, d._vSparseIndex.data());
        if (!(d._attributes & NNDataSetEnums::Boolean)) nc.addVar("sparseData" + s, ncTypeOf<T>(), sparseDim, d._vSparseData.data());
    } else {
        const uint32_t dataDim = nc.addDim("dataDim" + s, d._vData.size());
        nc.addVar("data" + s, ncTypeOf<T>(), dataDim, d._vData.data());
    }
    if (d._attributes & NNDataSetEnums::Weighted) nc.addVar("dataWeight" + s, ncc::NC_FLOAT, uniqueDim, d._vDataWeight.data());
    if (d._attributes & NNDataSetEnums::Indexed) nc.addVar("index" + s, ncc::NC_UINT, examplesDim, d._vIndex.data());
}

template <typename T> bool NNDataSet<T>::SaveNetCDF(const string& fname)
{
    try {
        ncc::Writer nc;
        nc.putAttUInt("datasets", 1);
        writeDataSet<T>(nc, *this, 0);
        nc.write(fname);
    } catch (std::exception& e) {
        printf("NNDataSet::SaveNetCDF: %s\n", e.what());
        return false;
    }
    return true;
}

#define DSX_FOR_EACH_TYPE(X) X(uint32_t) X(int32_t) X(int64_t) X(uint64_t) X(float) X(double) X(char) X(unsigned char)

bool SaveNetCDF(const string& fname, vector<NNDataSetBase*> vDataSet)
{
    try {
        ncc::Writer nc;
        nc.putAttUInt("datasets", (uint32_t)vDataSet.size());
        for (uint32_t i = 0; i < vDataSet.size(); i++) {
            NNDataSetBase* b = vDataSet[i];
            bool done = false;
#define DSX_TRY(T)                                                       \
    if (!done)                                                           \
        if (auto* p = dynamic_cast<NNDataSet<T>*>(b)) {                  \
            writeDataSet<T>(nc, *p, i);                                  \
            done = true;                                                 \
        }
            DSX_FOR_EACH_TYPE(DSX_TRY)
#undef DSX_TRY
            if (!done) throw std::runtime_error("unknown dataset type");
        }
        nc.write(fname);
    } catch (std::exception& e) {
        printf("SaveNetCDF: %s\n", e.what());
        return false;
    }
    return true;
}

// Reads dataset n of an open file into a new NNDataSet<T> (engine/NNTypes.cpp:1081-1358).
template <typename T> static NNDataSetBase* readDataSet(const ncc::Reader& nc, uint32_t n)
{
    const string s = std::to_string(n);
    const string name = nc.att("name" + s).asString();
    const uint32_t attributes = (uint32_t)nc.att("attributes" + s).asUInt64();
    const uint32_t examples = (uint32_t)nc.dim("examplesDim" + s);
    const uint32_t uniqueExamples = nc.hasDim("uniqueExamplesDim" + s) ? (uint32_t)nc.dim("uniqueExamplesDim" + s) : examples;
    const uint32_t dimensions = (uint32_t)nc.att("dimensions" + s).asUInt64();
    const uint32_t width = (uint32_t)nc.att("width" + s).asUInt64();
    const uint32_t height = dimensions > 1 ? (uint32_t)nc.att("height" + s).asUInt64() : 1;
    const uint32_t length = dimensions > 2 ? (uint32_t)nc.att("length" + s).asUInt64() : 1;
    const NNDataSetDimensions dim(width, height, length);
    const bool indexed = attributes & NNDataSetEnums::Indexed;
    const bool weighted = attributes & NNDataSetEnums::Weighted;
    NNDataSet<T>* d;
    if (attributes & NNDataSetEnums::Sparse) {
        const uint64_t sparseSize = nc.dim("sparseDataDim" + s);
        d = new NNDataSet<T>(examples, uniqueExamples, (size_t)sparseSize, dim, indexed, weighted, name);
        nc.read<uint64_t>("sparseStart" + s, d->_vSparseStart);   // legacy files hold uint32 offsets; read() widens them
        nc.read<uint64_t>("sparseEnd" + s, d->_vSparseEnd);
        nc.read<uint32_t>("sparseIndex" + s, d->_vSparseIndex);
        if (!(attributes & NNDataSetEnums::Boolean)) nc.read<T>("sparseData" + s, d->_vSparseData);
        d->_sparseDensity = (NNFloat)((double)sparseSize / ((double)uniqueExamples * (double)width * height * length));
    } else {
        d = indexed ? new NNDataSet<T>(examples, uniqueExamples, dim, name) : new NNDataSet<T>(examples, dim, name);
        nc.read<T>("data" + s, d->_vData);
    }
    d->_attributes = attributes;   // Boolean (and the other stored bits) come only from the file (engine/NNTypes.cpp:1118-1123)
    d->_dimensions = dimensions;
    if (weighted) nc.read<NNFloat>("dataWeight" + s, d->_vDataWeight);
    if (indexed) nc.read<uint32_t>("index" + s, d->_vIndex);
    // device copies are (re)created from the host vectors when the dataset is attached to a layer (Shard)
    d->_sharding = NNDataSetEnums::Sharding::None;
    return d;
}

vector<NNDataSetBase*> LoadNetCDF(const string& fname)
{
    vector<NNDataSetBase*> v;
    try {
        ncc::Reader nc(fname);
        const uint32_t datasets = (uint32_t)nc.att("datasets").asUInt64();
        for (uint32_t i = 0; i < datasets; i++) {
            const string s = std::to_string(i);
            // the reference's generator writes "dataType<n>", its SaveNetCDF writes "datatype<n>": accept both
            const string key = nc.hasAtt("dataType" + s) ? "dataType" + s : "datatype" + s;
            const uint32_t dataType = (uint32_t)nc.att(key).asUInt64();
            NNDataSetBase* d = NULL;
            switch (dataType) {
            case NNDataSetEnums::UInt: d = readDataSet<uint32_t>(nc, i); break;
            case NNDataSetEnums::Int: d = readDataSet<int64_t>(nc, i); break;   // engine/NNTypes.cpp:2550-2552 maps stored Int to long
            case NNDataSetEnums::LLInt: d = readDataSet<int64_t>(nc, i); break;
            case NNDataSetEnums::ULLInt: d = readDataSet<uint64_t>(nc, i); break;
            case NNDataSetEnums::Float: d = readDataSet<float>(nc, i); break;
            case NNDataSetEnums::Double: d = readDataSet<double>(nc, i); break;
            case NNDataSetEnums::UChar: d = readDataSet<unsigned char>(nc, i); break;
            case NNDataSetEnums::Char: d = readDataSet<char>(nc, i); break;
            default:
                printf("LoadNetCDF: invalid data type in binary input file %s.\n", fname.c_str());
                getGpu().Shutdown();
                exit(-1);
            }
            v.push_back(d);
        }
    } catch (std::exception& e) {
        printf("LoadNetCDF: %s\n", e.what());
        for (auto p : v) delete p;
        v.clear();
        getGpu().Shutdown();
        exit(-1);
    }
    return v;
}

#define DSX_INSTANTIATE(T) template class NNDataSet<T>;
DSX_FOR_EACH_TYPE(DSX_INSTANTIATE)
#undef DSX_INSTANTIATE
