// Dataset and buffer behaviour on the device, following the assertions of the reference's own unit tests
// tst/amazon/dsstne/engine/TestNNDataSet.cpp:58-349 and TestGpuBuffer.cpp:31-68.
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>

#include "amazon/dsstne/engine/NNTypes.h"
#include "check.h"

static NNDataSetDimensions datasetDim = NNDataSetDimensions(128, 1, 1);
static const uint32_t examples = 32;
static const uint32_t uniqueExamples = 16;
static const double sparseDensity = 0.1;
static const size_t stride = 128;
static const size_t dataLength = stride * examples;

static void testCreate()
{
    {
        NNDataSet<uint32_t> d(32, datasetDim);
        CHECK(d._stride == 128 && !d._bIndexed && !d._bStreaming && d._dimensions == 1);
        CHECK(d._attributes == NNDataSetEnums::None);
        CHECK(d._dataType == NNDataSetEnums::DataType::UInt);
        CHECK(d._width == 128 && d._height == 1 && d._length == 1);
        CHECK(d._examples == 32 && d._uniqueExamples == 32 && d._localExamples == 32 && d._sparseDataSize == 0);
    }
    {
        NNDataSet<uint32_t> d(examples, uniqueExamples, datasetDim);
        CHECK(d._stride == 128 && d._bIndexed && d._attributes == NNDataSetEnums::Indexed);
        CHECK(d._examples == examples && d._uniqueExamples == uniqueExamples && d._localExamples == examples && d._sparseDataSize == 0);
    }
    {
        NNDataSet<int> d(examples, sparseDensity, datasetDim, false);
        CHECK(d._stride == 0 && !d._bIndexed && d._attributes == NNDataSetEnums::Sparse);
        CHECK(d._dataType == NNDataSetEnums::DataType::Int);
        CHECK(d._uniqueExamples == examples && d._sparseDataSize == (uint64_t)(128.0 * 0.1 * 32.0));
    }
    {
        NNDataSet<int> d(examples, sparseDensity, datasetDim, true);
        CHECK(d._attributes == (NNDataSetEnums::Sparse | NNDataSetEnums::Weighted));
        CHECK(d._sparseDataSize == (uint64_t)(128.0 * 0.1 * 32.0));
    }
    {
        size_t sparseDataSize = 128 * uniqueExamples / 10;
        NNDataSet<long> d(examples, uniqueExamples, sparseDataSize, datasetDim, true, false);
        CHECK(d._bIndexed && d._attributes == (NNDataSetEnums::Sparse | NNDataSetEnums::Indexed));
        CHECK(d._dataType == NNDataSetEnums::DataType::LLInt);
        CHECK(d._uniqueExamples == uniqueExamples && d._sparseDataSize == sparseDataSize);
    }
    {
        size_t sparseDataSize = 128 * uniqueExamples / 10;
        NNDataSet<long> d(examples, uniqueExamples, sparseDataSize, datasetDim, true, true);
        CHECK(d._attributes == (NNDataSetEnums::Sparse | NNDataSetEnums::Indexed | NNDataSetEnums::Weighted));
    }
    {
        NNDataSet<NNFloat> f(examples, datasetDim);
        NNDataSet<double> d(examples, datasetDim);
        NNDataSet<unsigned char> uc(examples, datasetDim);
        NNDataSet<char> c(examples, datasetDim);
        NNDataSet<uint32_t> u(examples, datasetDim);
        NNDataSet<uint64_t> ul(examples, datasetDim);
        NNDataSet<int32_t> i(examples, datasetDim);
        NNDataSet<int64_t> l(examples, datasetDim);
        CHECK(c._dataType == NNDataSetEnums::Char && uc._dataType == NNDataSetEnums::UChar && ul._dataType == NNDataSetEnums::ULLInt);
    }
}

static void testLoadDense()
{
    NNDataSet<uint32_t> dataset(examples, datasetDim);
    std::vector<uint32_t> src(dataLength);
    for (size_t i = 0; i < dataLength; ++i) src[i] = (uint32_t)i;
    dataset.LoadDenseData(src.data());
    for (size_t i = 0; i < examples; ++i)
        for (size_t j = 0; j < stride; ++j) CHECK_EQ((uint32_t)(i * stride + j), dataset.GetDataPoint(i, j));
    std::vector<uint32_t> back(dataLength);
    dataset._pbData->Download(back.data());
    CHECK(back == src);   // the device copy holds the same rows
    checkThrows<std::runtime_error>("dense data on a sparse dataset", [&] {
        NNDataSet<uint32_t> s(examples, sparseDensity, datasetDim, false);
        s.LoadDenseData(src.data());
    });
}

static void testLoadSparse()
{
    NNDataSet<NNFloat> dataset(examples, sparseDensity, datasetDim, false);
    NNDataSetDimensions dim = dataset.GetDimensions();
    size_t sparseDataSize = (size_t)(((double)dim._height * dim._width * dim._length) * examples * sparseDensity);
    std::vector<uint64_t> sparseStart(examples), sparseEnd(examples);
    std::vector<NNFloat> sparseData(sparseDataSize);
    std::vector<uint32_t> sparseIndex(sparseDataSize);
    size_t sparseExampleSize = (sparseDataSize + examples - 1) / examples;
    sparseStart[0] = 0;
    sparseEnd[0] = sparseDataSize - (sparseExampleSize * (examples - 1));
    for (uint32_t i = 1; i < examples; i++) {
        sparseStart[i] = sparseEnd[i - 1];
        sparseEnd[i] = sparseStart[i] + sparseExampleSize;
    }
    for (uint32_t i = 0; i < sparseDataSize; ++i) {
        sparseData[i] = i + 1;
        sparseIndex[i] = i;
    }
    dataset.LoadSparseData(sparseStart.data(), sparseEnd.data(), sparseData.data(), sparseIndex.data());
    CHECK_EQ(sparseEnd[0], dataset.GetSparseDataPoints(0));
    for (uint32_t i = 0; i < sparseEnd[0]; ++i) {
        CHECK_EQ((NNFloat)i + 1, dataset.GetSparseDataPoint(0, i));
        CHECK_EQ(i, dataset.GetSparseIndex(0, i));
    }
    std::vector<uint32_t> back(dataset._pbSparseIndex->_length);
    dataset._pbSparseIndex->Download(back.data());
    CHECK(std::equal(sparseIndex.begin(), sparseIndex.end(), back.begin()));

    // the long* overloads used by language bindings without unsigned types
    std::vector<long> ls(sparseStart.begin(), sparseStart.end()), le(sparseEnd.begin(), sparseEnd.end()), li(sparseIndex.begin(), sparseIndex.end());
    NNDataSet<NNFloat> viaLong(examples, sparseDensity, datasetDim, false);
    viaLong.LoadSparseData(ls.data(), le.data(), sparseData.data(), li.data());
    dataset.SyncSparseHostCopy();   // (loaded straight to the device: the host vectors follow on request)
    viaLong.SyncSparseHostCopy();
    CHECK(viaLong._vSparseIndex == dataset._vSparseIndex && viaLong._vSparseEnd == dataset._vSparseEnd);

    // A load that went straight to the device leaves the host vectors stale until something reads them: a second load with
    // other numbers, then SaveNetCDF (which reads them) and LoadNetCDF must give back the second load, not the first.
    {
        NNDataSet<NNFloat> second(examples, sparseDensity, datasetDim, false);
        second._name = "second";
        second.LoadSparseData(sparseStart.data(), sparseEnd.data(), sparseData.data(), sparseIndex.data());
        std::vector<NNFloat> data2(sparseData);
        std::vector<uint32_t> index2(sparseIndex);
        for (size_t i = 0; i < data2.size(); i++) {
            data2[i] = (NNFloat)(1000 + i);
            index2[i] = (uint32_t)((i * 7) % 128);
        }
        second.LoadSparseData(sparseStart.data(), sparseEnd.data(), data2.data(), index2.data());
        CHECK(second._bSparseHostStale);
        const char* tmp = getenv("TMPDIR");
        const std::string file = std::string(tmp && tmp[0] ? tmp : "/tmp") + "/dsx_stale_host_copy.nc";
        CHECK(second.SaveNetCDF(file));
        CHECK(!second._bSparseHostStale);
        std::vector<NNDataSetBase*> back2 = LoadNetCDF(file);
        CHECK(back2.size() == 1);
        if (back2.size() == 1) {
            NNDataSet<NNFloat>* r = dynamic_cast<NNDataSet<NNFloat>*>(back2[0]);
            CHECK(r != NULL);
            if (r) {
                CHECK(std::equal(index2.begin(), index2.end(), r->_vSparseIndex.begin()));
                CHECK(std::equal(data2.begin(), data2.end(), r->_vSparseData.begin()));
                CHECK(r->_vSparseEnd == std::vector<uint64_t>(sparseEnd.begin(), sparseEnd.end()));
            }
        }
        for (auto* d : back2) delete d;
        remove(file.c_str());
    }

    checkThrows<std::length_error>("sparse overflow", [&] {
        NNDataSet<NNFloat> d(examples, sparseDensity, datasetDim, false);
        std::vector<uint64_t> s(examples, 0), e(examples, 0);
        NNFloat one[1] = {0};
        uint32_t idx[1] = {0};
        e[examples - 1] = sparseDataSize + 1;
        d.LoadSparseData(s.data(), e.data(), one, idx);
    });
    checkThrows<std::runtime_error>("sparse start not zero", [&] {
        NNDataSet<NNFloat> d(examples, sparseDensity, datasetDim, false);
        std::vector<uint64_t> s(examples, 0), e(examples, 0);
        NNFloat one[1] = {0};
        uint32_t idx[1] = {0};
        s[0] = 1;
        e[examples - 1] = sparseDataSize + 1;
        d.LoadSparseData(s.data(), e.data(), one, idx);
    });
    checkThrows<std::runtime_error>("sparse data on a dense dataset", [&] {
        NNDataSet<NNFloat> d(examples, datasetDim);
        std::vector<uint64_t> s(examples, 0), e(examples, 0);
        NNFloat one[1] = {0};
        uint32_t idx[1] = {0};
        d.LoadSparseData(s.data(), e.data(), one, idx);
    });
}

static void testIndexedAndWeights()
{
    {
        NNDataSet<NNFloat> dataset(examples, uniqueExamples, datasetDim);
        std::vector<uint32_t> indexed(examples);
        for (uint32_t i = 0; i < examples; ++i) indexed[i] = i % uniqueExamples;
        dataset.LoadIndexedData(indexed.data());
        for (uint32_t i = 0; i < examples; ++i) CHECK_EQ(i % uniqueExamples, dataset._vIndex[i]);
    }
    checkThrows<std::runtime_error>("indexed data on a plain dataset", [&] {
        NNDataSet<NNFloat> d(examples, datasetDim);
        std::vector<uint32_t> indexed(examples);
        d.LoadIndexedData(indexed.data());
    });
    {
        NNDataSet<uint32_t> dataset(examples, sparseDensity, datasetDim, true);
        std::vector<NNFloat> w(examples);
        for (uint32_t i = 0; i < examples; ++i) w[i] = (NNFloat)i;
        dataset.LoadDataWeight(w.data());
        for (uint32_t i = 0; i < examples; ++i) CHECK_EQ((NNFloat)i, dataset._vDataWeight[i]);
    }
    checkThrows<std::runtime_error>("weights on an unweighted dataset", [&] {
        NNDataSet<uint32_t> d(examples, sparseDensity, datasetDim, false);
        std::vector<NNFloat> w(examples);
        d.LoadDataWeight(w.data());
    });
    {
        NNDataSetDescriptor desc;
        desc._name = "bad";
        desc._dataType = NNDataSetEnums::DataType::Float;
        desc._attributes = NNDataSetEnums::Sparse | NNDataSetEnums::Indexed;
        desc._dim = datasetDim;
        desc._examples = 4;
        desc._sparseDensity = 0.1f;
        checkThrows<std::runtime_error>("unsupported descriptor attributes", [&] { delete createNNDataSet(desc); });
        desc._attributes = NNDataSetEnums::Sparse;
        NNDataSetBase* d = createNNDataSet(desc);
        CHECK(d->_attributes == NNDataSetEnums::Sparse && d->_dataType == NNDataSetEnums::Float && d->_examples == 4);
        delete d;
    }
}

static void testGpuBufferResize()
{
    size_t length = 1024;
    GpuBuffer<uint32_t> buff(length, false, true);   // managed: host-dereferenceable
    for (size_t i = 0; i < length; ++i) CHECK_EQ(0u, buff._pDevData[i]);
    for (size_t i = 0; i < length; ++i) buff._pDevData[i] = (uint32_t)i;
    buff.Resize(length);
    for (uint32_t i = 0; i < length; ++i) CHECK_EQ(i, buff._pDevData[i]);
    buff.Resize(length - 1);
    for (uint32_t i = 0; i < length; ++i) CHECK_EQ(i, buff._pDevData[i]);
    CHECK_EQ(buff.GetLength(), length);
    buff.Resize(length + 1);
    bool isSame = true;
    for (uint32_t i = 0; i < length; ++i) isSame &= (buff._pDevData[i] == i);
    CHECK(!isSame);
    CHECK_EQ(buff.GetLength(), length + 1);
    CHECK_EQ(buff.GetSize(), (length + 1) * sizeof(uint32_t));

    GpuBuffer<float> shadowed(16, true);
    for (int i = 0; i < 16; i++) shadowed._pSysData[i] = i * 0.5f;
    shadowed.Upload();
    for (int i = 0; i < 16; i++) shadowed._pSysData[i] = -1;
    shadowed.Download();
    for (int i = 0; i < 16; i++) CHECK_EQ(shadowed._pSysData[i], i * 0.5f);
    int gpuKiB = 0, cpuKiB = 0;
    getGpu().GetMemoryUsage(&gpuKiB, &cpuKiB);
    CHECK(gpuKiB >= 4);
}

int main(int argc, char** argv)
{
    getGpu().Startup(argc, argv);
    testCreate();
    testLoadDense();
    testLoadSparse();
    testIndexedAndWeights();
    testGpuBufferResize();
    getGpu().Shutdown();
    return finish("test_dataset_gpu");
}
