// NNTypes.h — engine-wide enumerations and the dataset classes of the inference path.
//
// Mirrors the public surface of the reference's engine/NNTypes.h: NNDataSetDimensions, NNDataSetDescriptor,
// createNNDataSet, NNDataSetBase (public fields of :199-243) and NNDataSet<T> with its four public constructors and the
// Load*/Copy* entry points (:425-476).  Training-only members (denoising, transposed sparse matrices, error and delta
// dispatch) are not part of this build.
#ifndef DSSTNE_AMD_NNTYPES_H
#define DSSTNE_AMD_NNTYPES_H

#include "GpuTypes.h"
#include "NNEnum.h"
#include "NNDefs.h"

class NNLayer;
class NNWeight;
class NNNetwork;
struct NNDataSetBase;

struct NNDataSetDimensions {
    uint32_t _dimensions;   // number of extents greater than 1
    uint32_t _width;
    uint32_t _height;
    uint32_t _length;

    NNDataSetDimensions();
    NNDataSetDimensions(uint32_t width, uint32_t height = 1, uint32_t length = 1);
};

struct NNDataSetDescriptor {
    string _name;
    NNDataSetEnums::DataType _dataType;
    uint32_t _attributes;
    NNDataSetDimensions _dim;
    uint32_t _examples;
    float _sparseDensity;

    // Only plain dense and plain sparse datasets can be created from a descriptor.
    static bool isSupported(uint32_t attributes) { return (attributes & ~(uint32_t)NNDataSetEnums::Sparse) == 0; }
};

// Caller owns the returned dataset.
NNDataSetBase* createNNDataSet(const NNDataSetDescriptor& descriptor);

struct NNDataSetBase {
    string _name;
    NNDataSetEnums::DataType _dataType;
    uint32_t _attributes;
    uint32_t _examples;
    uint32_t _uniqueExamples;
    uint32_t _localExamples;
    uint32_t _dimensions;
    uint32_t _width;
    uint32_t _height;
    uint32_t _length;
    uint32_t _stride;
    NNDataSetEnums::Sharding _sharding;
    uint32_t _minX;
    uint32_t _maxX;
    uint64_t _sparseDataSize;
    NNFloat _sparseDensity;
    vector<uint64_t> _vSparseStart;
    unique_ptr<GpuBuffer<uint64_t>> _pbSparseStart;
    vector<uint64_t> _vSparseEnd;
    unique_ptr<GpuBuffer<uint64_t>> _pbSparseEnd;
    vector<uint32_t> _vSparseIndex;
    unique_ptr<GpuBuffer<uint32_t>> _pbSparseIndex;
    vector<NNFloat> _vDataWeight;
    unique_ptr<GpuBuffer<NNFloat>> _pbDataWeight;
    vector<uint32_t> _vIndex;
    unique_ptr<GpuBuffer<uint32_t>> _pbIndex;

    bool _bDenoising;
    bool _bDirty;
    bool _bStreaming;
    bool _bIndexed;
    uint32_t _batch;

    // No counterpart in the reference (one set of arrays, blocking uploads).  Sparse data that arrives batch by batch
    // (LoadSparseData) goes to the set of device arrays that belongs to the lane the next PredictBatch will use, which no
    // kernel of another lane reads: the copy overlaps with the batches before it.  _pbSparseStart / End / Index / Data above
    // always name the set that holds the latest load (it belongs to lane _sparseLane); kernels launched earlier keep reading
    // the set they were given.  The other lanes' sets are parked here.
    struct SparseSetState {
        int _uploadLane = -1;                 // lane whose stream carries the set's last unordered upload (-1: ordered on every lane)
        uint32_t _readLanes = 0;              // lanes that have launched readers of the set since that upload
        uint32_t _orderedLanes = 0xffffffffu; // lanes that are known to run after that upload
        void* _uploaded = NULL;               // marker behind that upload: the next load into this set waits for it on the host, which
                                              // keeps a caller that streams batches a few batches ahead of the device and no more
    };
    struct ParkedSparseSet {
        unique_ptr<GpuBuffer<uint64_t>> _pbSparseStart;
        unique_ptr<GpuBuffer<uint64_t>> _pbSparseEnd;
        unique_ptr<GpuBuffer<uint32_t>> _pbSparseIndex;
        SparseSetState _state;
    };
    ParkedSparseSet _parkedSparse[DSX_MAX_LANES];
    SparseSetState _sparseSet;
    int _sparseLane = 0;
    // Call before launching a kernel that reads the _pbSparse* arrays on the selected lane.
    void NoteSparseRead();
    // The lane the next PredictBatch will run on (kept by NNNetwork); a wrong value costs a wait between the lanes, no more.
    static int s_nextLane;
    // No counterpart in the reference (which fills the host vectors first and uploads them): a LoadSparseData that goes
    // straight to the device arrays leaves _vSparseStart / End / Index / Data behind, and the accessors below, Shard and
    // SaveNetCDF fetch them back before they read them.  Code that reads the vectors itself calls SyncSparseHostCopy() first.
    bool _bSparseHostStale = false;
    virtual void SyncSparseHostCopy() = 0;

    NNDataSetBase();
    virtual ~NNDataSetBase() = 0;
    NNDataSetDimensions GetDimensions();
    uint32_t GetExamples() { return _examples; }
    uint32_t GetUniqueExamples() { return _uniqueExamples; }

    virtual void RefreshState(uint32_t batch) = 0;
    virtual bool Shard(NNDataSetEnums::Sharding sharding) = 0;
    virtual bool UnShard() = 0;
    virtual bool SetDenoising(bool flag) = 0;
    virtual bool SaveNetCDF(const string& fname) = 0;

    // Device-side consumers used by NNLayer (engine/NNTypes.h:478-545)
    virtual bool LoadInputUnit(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pUnit) = 0;
    virtual bool LoadSparseInputUnit(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pUnit) = 0;
    virtual bool CalculateSparseZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, NNFloat* pUnit,
                                  NNFloat beta = (NNFloat)0.0) = 0;
    // Bias initialisation + sparse Z + activation of a layer fed only by this dataset, as one kernel.
    virtual bool CalculateSparseLayer(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, NNFloat* pBias,
                                      Activation activation, NNFloat slope, NNFloat alpha, NNFloat lambda, NNFloat* pUnit) = 0;

    virtual void LoadDenseData(const void* srcData) = 0;
    virtual void CopyDenseData(const void* srcData) = 0;
    virtual void LoadSparseData(const uint64_t* srcSparseStart, const uint64_t* srcSparseEnd, const void* srcSparseData,
                                const uint32_t* srcSparseIndex) = 0;
    virtual void CopySparseData(const uint64_t* srcSparseStart, const uint64_t* srcSparseEnd, const void* srcSparseData,
                                const uint32_t* srcSparseIndex) = 0;
    // long* overloads for language bindings without unsigned types (JNI)
    virtual void LoadSparseData(const long* srcSparseStart, const long* srcSparseEnd, const void* srcSparseData,
                                const long* srcSparseIndex) = 0;
    virtual void CopySparseData(const long* srcSparseStart, const long* srcSparseEnd, const void* srcSparseData,
                                const long* srcSparseIndex) = 0;
    virtual void LoadIndexedData(const uint32_t* srcIndexedData) = 0;
    virtual void LoadDataWeight(const NNFloat* srcWeightData) = 0;

protected:
    NNDataSetBase(const string& name, NNDataSetEnums::DataType dataType, uint32_t examples, uint32_t uniqueExamples,
                  const NNDataSetDimensions& datasetDim);
};

template <typename T> class NNDataSet : public NNDataSetBase {
public:
    friend class NNNetwork;
    friend class NNLayer;
    friend vector<NNDataSetBase*> LoadNetCDF(const string& fname);
    friend bool SaveNetCDF(const string& fname, vector<NNDataSetBase*> vDataSet);

    vector<T> _vData;
    unique_ptr<GpuBuffer<T>> _pbData;
    vector<T> _vSparseData;
    unique_ptr<GpuBuffer<T>> _pbSparseData;
    unique_ptr<GpuBuffer<T>> _parkedSparseData[DSX_MAX_LANES];   // see _parkedSparse

    // dense
    NNDataSet(uint32_t examples, const NNDataSetDimensions& dim, const string& name = "");
    // dense, indexed
    NNDataSet(uint32_t examples, uint32_t uniqueExamples, const NNDataSetDimensions& dim, const string& name = "");
    // sparse (optionally weighted) with room for examples * width * height * length * sparseDensity non-zeros
    NNDataSet(uint32_t examples, NNFloat sparseDensity, const NNDataSetDimensions& dim, bool isWeighted = false, const string& name = "");
    // sparse (optionally indexed / weighted) with room for sparseDataSize non-zeros
    NNDataSet(uint32_t examples, uint32_t uniqueExamples, size_t sparseDataSize, const NNDataSetDimensions& dim, bool isIndexed = false,
              bool isWeighted = false, const string& name = "");
    ~NNDataSet();

    void LoadDenseData(const void* srcData) override;
    void CopyDenseData(const void* srcData) override;
    void LoadSparseData(const uint64_t* srcSparseStart, const uint64_t* srcSparseEnd, const void* srcSparseData,
                        const uint32_t* srcSparseIndex) override;
    void CopySparseData(const uint64_t* srcSparseStart, const uint64_t* srcSparseEnd, const void* srcSparseData,
                        const uint32_t* srcSparseIndex) override;
    void LoadSparseData(const long* srcSparseStart, const long* srcSparseEnd, const void* srcSparseData, const long* srcSparseIndex) override;
    void CopySparseData(const long* srcSparseStart, const long* srcSparseEnd, const void* srcSparseData, const long* srcSparseIndex) override;
    void LoadIndexedData(const uint32_t* srcIndexedData) override;
    void LoadDataWeight(const NNFloat* srcWeightData) override;
    void SyncSparseHostCopy() override;

    void RefreshState(uint32_t batch) override {}
    bool Shard(NNDataSetEnums::Sharding sharding) override;
    bool UnShard() override;
    bool SetDenoising(bool flag) override;
    bool SaveNetCDF(const string& fname) override;
    bool LoadInputUnit(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pUnit) override;
    bool LoadSparseInputUnit(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pUnit) override;
    bool CalculateSparseZ(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, NNFloat* pUnit, NNFloat beta) override;
    bool CalculateSparseLayer(uint32_t position, uint32_t batch, uint32_t stride, NNFloat* pWeight, NNFloat* pBias, Activation activation,
                              NNFloat slope, NNFloat alpha, NNFloat lambda, NNFloat* pUnit) override;

    T GetDataPoint(uint32_t n, uint32_t x, uint32_t y = 0, uint32_t z = 0);
    bool SetDataPoint(T v, uint32_t n, uint32_t x, uint32_t y = 0, uint32_t z = 0);
    uint64_t GetSparseDataPoints(uint32_t n);
    uint32_t GetSparseIndex(uint32_t n, uint32_t i);
    bool SetSparseIndex(uint32_t n, uint32_t i, uint32_t v);
    T GetSparseDataPoint(uint32_t n, uint32_t i);
    bool SetSparseDataPoint(uint32_t n, uint32_t i, T v);

private:
    void checkSparseLoad(const uint64_t start0, const uint64_t dataLength) const;
    void uploadSparse();
    bool uploadSparseDirect(const uint64_t* srcSparseStart, const uint64_t* srcSparseEnd, const void* srcSparseData,
                            const uint32_t* srcSparseIndex);
};

// Dataset files (same attribute and variable names as the reference writes, engine/NNTypes.cpp:1081-1358).
vector<NNDataSetBase*> LoadNetCDF(const string& fname);
bool SaveNetCDF(const string& fname, vector<NNDataSetBase*> vDataSet);

#include "NNWeight.h"
#include "NNLayer.h"
#include "NNNetwork.h"
#include "kernels.h"

#endif
