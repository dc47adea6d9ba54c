// Host-only checks (no GPU): dataset dimensions, network/dataset file round trips, filter parsing and application,
// CPU top-K, KNN text reader and merge.  Mirrors tst/amazon/dsstne/engine/TestNNDataSetDimensions.cpp and the parsing
// tests of tst/unittests.
#include <cmath>
#include <fstream>
#include <map>
#include <sstream>
#include <unordered_map>

#include "amazon/dsstne/engine/NNTypes.h"
#include "amazon/dsstne/knn/KnnExactGpu.h"
#include "amazon/dsstne/utils/Filters.h"
#include "amazon/dsstne/utils/NetCDFhelper.h"
#include "amazon/dsstne/utils/Utils.h"
#include "Json.h"
#include "NcClassic.h"
#include "check.h"

using namespace std;

static void testDimensions()
{
    NNDataSetDimensions zero_d(1), one_d(2), two_d(2, 2), three_d(2, 2, 2);
    CHECK_EQ(0U, zero_d._dimensions);
    CHECK_EQ(1U, one_d._dimensions);
    CHECK_EQ(2U, two_d._dimensions);
    CHECK_EQ(3U, three_d._dimensions);
    NNDataSetDimensions dflt;
    CHECK(dflt._width == 1 && dflt._height == 1 && dflt._length == 1 && dflt._dimensions == 0);
}

static NNNetworkDescriptor sampleDescriptor()
{
    NNNetworkDescriptor nd;
    nd._name = "roundtrip";
    nd._kind = NNNetwork::Kind::AutoEncoder;
    nd._errorFunction = ErrorFunction::ScaledMarginalCrossEntropy;
    nd._SMCE_zeroScale = 0.25f;
    nd._checkpoint_interval = 7;
    const char* names[] = {"Input", "Hidden", "Output"};
    const uint32_t widths[] = {6, 3, 6};
    for (int i = 0; i < 3; i++) {
        NNLayerDescriptor ld;
        ld._name = names[i];
        ld._kind = i == 0 ? NNLayer::Kind::Input : (i == 2 ? NNLayer::Kind::Output : NNLayer::Kind::Hidden);
        ld._Nx = widths[i];
        ld._activation = i == 1 ? Activation::LeakyRectifiedLinear : Activation::Sigmoid;
        ld._RELUSlope = 0.125f;
        ld._ELUAlpha = 1.5f;
        ld._SELULambda = 1.25f;
        ld._attributes = i == 0 ? NNLayer::Attributes::Sparse : NNLayer::Attributes::None;
        ld._dataSet = i == 1 ? "" : "data";
        if (i > 0) ld._vSource.push_back(names[i - 1]);
        if (i == 2) ld._vSkip.push_back("Input");
        nd._vLayerDescriptor.push_back(ld);
    }
    NNWeightDescriptor w0;
    w0._inputLayer = "Input";
    w0._outputLayer = "Hidden";
    w0._width = 3;
    w0._height = 6;
    for (int i = 0; i < 18; i++) w0._vWeight.push_back(0.5f * i - 3);
    w0._vBias = {0.1f, -0.2f, 0.3f};
    nd._vWeightDescriptor.push_back(w0);
    NNWeightDescriptor w1;
    w1._inputLayer = "Hidden";
    w1._outputLayer = "Output";
    w1._width = 6;
    w1._height = 3;
    w1._bShared = true;
    w1._bTransposed = true;
    w1._sourceInputLayer = "Input";
    w1._sourceOutputLayer = "Hidden";
    w1._vBias = {1, 2, 3, 4, 5, 6};
    nd._vWeightDescriptor.push_back(w1);
    return nd;
}

static void testNetworkFileRoundTrip(const string& dir)
{
    NNNetworkDescriptor nd = sampleDescriptor();
    const string f = dir + "/net.nc";
    CHECK(SaveNNNetworkDescriptorNetCDF(f, nd));
    NNNetworkDescriptor rd;
    CHECK(LoadNNNetworkDescriptorNetCDF(f, rd));
    CHECK_EQ(rd._name, nd._name);
    CHECK_EQ(rd._kind, nd._kind);
    CHECK_EQ(rd._errorFunction, nd._errorFunction);
    CHECK_EQ(rd._SMCE_zeroScale, 0.25f);
    CHECK_EQ(rd._checkpoint_interval, 7);
    CHECK_EQ(rd._checkpoint_name, string("checkpoint"));
    CHECK_EQ(rd._vLayerDescriptor.size(), (size_t)3);
    CHECK_EQ(rd._vLayerDescriptor[1]._activation, Activation::LeakyRectifiedLinear);
    CHECK_EQ(rd._vLayerDescriptor[1]._RELUSlope, 0.125f);
    CHECK_EQ(rd._vLayerDescriptor[0]._attributes, (uint32_t)NNLayer::Attributes::Sparse);
    CHECK_EQ(rd._vLayerDescriptor[2]._vSource.size(), (size_t)1);
    CHECK_EQ(rd._vLayerDescriptor[2]._vSource[0], string("Hidden"));
    CHECK_EQ(rd._vLayerDescriptor[2]._vSkip[0], string("Input"));
    CHECK_EQ(rd._vLayerDescriptor[2]._dataSet, string("data"));
    CHECK_EQ(rd._vWeightDescriptor.size(), (size_t)2);
    CHECK(rd._vWeightDescriptor[0]._vWeight == nd._vWeightDescriptor[0]._vWeight);
    CHECK(rd._vWeightDescriptor[0]._vBias == nd._vWeightDescriptor[0]._vBias);
    CHECK_EQ(rd._vWeightDescriptor[0]._width, (uint64_t)3);
    CHECK_EQ(rd._vWeightDescriptor[0]._height, (uint64_t)6);
    CHECK(rd._vWeightDescriptor[1]._bShared && rd._vWeightDescriptor[1]._bTransposed);
    CHECK_EQ(rd._vWeightDescriptor[1]._sourceOutputLayer, string("Hidden"));
    CHECK(rd._vWeightDescriptor[1]._vWeight.empty());
    CHECK(rd._vWeightDescriptor[1]._vBias == nd._vWeightDescriptor[1]._vBias);
    // unreadable inputs are reported, not fatal, at the descriptor level
    NNNetworkDescriptor bad;
    CHECK(!LoadNNNetworkDescriptorNetCDF(dir + "/does-not-exist.nc", bad));
    ofstream(dir + "/garbage.nc") << "this is not a NetCDF file";
    CHECK(!LoadNNNetworkDescriptorNetCDF(dir + "/garbage.nc", bad));
    ofstream h(dir + "/hdf5.nc", ios::binary);
    h.write("\x89HDF\r\n\x1a\n", 8);
    h.close();
    CHECK(!LoadNNNetworkDescriptorNetCDF(dir + "/hdf5.nc", bad));
}

static void testFilters(const string& dir)
{
    unordered_map<string, unsigned int> items = {{"a", 0}, {"b", 1}, {"c", 2}, {"d", 3}};
    unordered_map<string, unsigned int> samples = {{"u0", 0}, {"u1", 1}, {"u2", 2}};
    {
        ofstream f(dir + "/filter.txt");
        f << "u0\ta:c,0.5:zzz\n";       // a -> 0 (no value), c -> 0.5, unknown item ignored
        f << "nobody\tb\n";            // unknown sample ignored
        f << "u2\td,2\n";
    }
    unique_ptr<FilterConfig> fc(loadFilters(dir + "/filter.txt", dir + "/recs.txt", items, samples));
    CHECK_EQ(fc->getOutputFileName(), dir + "/recs.txt");
    float row0[4] = {1, 1, 1, 1}, row1[4] = {1, 1, 1, 1}, row2[4] = {1, 1, 1, 1};
    fc->applySamplesFilter(row0, 0, 0, 4);
    fc->applySamplesFilter(row1, 1, 0, 4);   // no filter for u1: untouched
    fc->applySamplesFilter(row2, 2, 0, 4);
    CHECK(row0[0] == 0 && row0[1] == 1 && row0[2] == 0.5f && row0[3] == 1);
    CHECK(row1[0] == 1 && row1[1] == 1 && row1[2] == 1 && row1[3] == 1);
    CHECK(row2[3] == 2);
    // offset / width window (utils/Filters.cpp:49-67): only indexes inside [offset, offset + width) are touched
    float part[2] = {1, 1};
    fc->applySamplesFilter(part, 0, 2, 2);   // covers items 2, 3
    CHECK(part[0] == 0.5f && part[1] == 1);
    // a path that does not exist yields an empty filter set (listFiles reports it), not an exception
    SamplesFilter none;
    none.loadFilter(items, samples, dir + "/no-such-filter");
    CHECK_EQ(none.samples(), (size_t)3);
    float keep[4] = {1, 2, 3, 4};
    none.applyFilter(keep, 1, 0, 4);
    CHECK(keep[0] == 1 && keep[3] == 4);
}

static void testTopKsort()
{
    float keys[8] = {0.5f, 0.9f, 0.1f, 0.9f, 0.3f, 0.7f, 0.9f, 0.2f};
    float tk[4];
    unsigned int tv[4];
    topKsort<float, unsigned int>(keys, NULL, 8, tk, tv, 4);
    CHECK(tk[0] == 0.9f && tk[1] == 0.9f && tk[2] == 0.9f && tk[3] == 0.7f);
    CHECK(tv[0] == 1 && tv[1] == 3 && tv[2] == 6 && tv[3] == 5);   // equal keys: lower position first
    float vals[8] = {8, 7, 6, 5, 4, 3, 2, 1}, tvf[3];
    topKsort<float, float>(keys, vals, 8, tk, tvf, 3);
    CHECK(tvf[0] == 7 && tvf[1] == 5 && tvf[2] == 2);
}

// The reference's own case (tst/unittests/TestUtils.cpp:10-17) and the helpers beside it.
static void testUtils(const string& dir)
{
    CHECK(isNetCDFfile("network.nc"));
    CHECK(!isNetCDFfile("network.nic"));
    CHECK(!isNetCDFfile("network"));
    CHECK(isNetCDFfile("a.b/net.v2.nc") && !isNetCDFfile("net.nc.bak"));
    vector<string> parts = {"head"};
    vector<string>& same = split("a,b,,c", ',', parts);
    CHECK(&same == &parts && parts.size() == 5 && parts[0] == "head" && parts[3] == "" && parts[4] == "c");
    CHECK(split("x:y", ':').size() == 2 && split("", ':').empty());
    const string file = dir + "/utils_probe.txt";
    FILE* f = fopen(file.c_str(), "w");
    fputs("x\n", f);
    fclose(f);
    CHECK(isDirectory(dir) && !isFile(dir));
    CHECK(isFile(file) && !isDirectory(file));
    CHECK(!isFile(dir + "/no_such_entry") && !isDirectory(dir + "/no_such_entry"));
    for (int i = 0; i < 200; i++) {
        const int r = rand(3, 5);
        const float x = rand(-1.0f, 2.0f);
        CHECK(r >= 3 && r <= 5);
        CHECK(x >= -1.0f && x <= 2.0f);
    }
    CHECK(rand(7, 7) == 7);
    CHECK(INPUT_DATASET_SUFFIX == "_input" && OUTPUT_DATASET_SUFFIX == "_output" && FIXED_SEED == 12134ul);
}

static void testKnnHost(const string& dir)
{
    {
        ofstream f(dir + "/vectors.txt");
        f << "k0\t1.0 2.0 3.0\n";
        f << "k1\t-1 0.5 4\n";
    }
    uint32_t rows = 0;
    int cols = 0;
    TextFileDataReader::findDataDimensions(dir + "/vectors.txt", rows, cols);
    CHECK_EQ(rows, 2u);
    CHECK_EQ(cols, 3);
    TextFileDataReader r(dir + "/vectors.txt");
    string key;
    float v[3];
    CHECK(r.readRow(&key, v));
    CHECK(key == "k0" && v[0] == 1 && v[1] == 2 && v[2] == 3);
    CHECK(r.readRow(&key, v));
    CHECK(key == "k1" && v[0] == -1 && v[1] == 0.5f && v[2] == 4);
    CHECK(!r.readRow(&key, v));

    using namespace astdl::knn;
    // two "devices", batch 1, width 3: strict '<' keeps the lower device on ties (knn/KnnExactGpu.cu:183)
    float s0[3] = {0.9f, 0.5f, 0.1f}, s1[3] = {0.9f, 0.7f, 0.2f};
    uint32_t i0[3] = {0, 1, 2}, i1[3] = {0, 1, 2};
    vector<float*> as = {s0, s1};
    vector<uint32_t*> ai = {i0, i1};
    vector<vector<string>> keys = {{"a0", "a1", "a2"}, {"b0", "b1", "b2"}};
    float out[3];
    string outk[3];
    mergeKnn(3, 1, 3, 2, as, ai, keys, out, outk);
    CHECK(out[0] == 0.9f && out[1] == 0.9f && out[2] == 0.7f);
    CHECK(outk[0] == "a0" && outk[1] == "b0" && outk[2] == "b1");
    CHECK(getDataTypeFromString("fp32") == DataType::FP32 && getDataTypeString(DataType::FP16) == "fp16");
    CHECK(getDataTypeFromString("fp32-split") == DataType::FP32Split && getDataTypeString(DataType::FP32Split) == "fp32-split");
    checkThrows<std::invalid_argument>("bad data type", [] { getDataTypeFromString("int8"); });
}

// --dump-network file: prints what LoadNNNetworkDescriptorNetCDF sees, for comparison with an independent writer.
static int dumpNetwork(const string& file)
{
    NNNetworkDescriptor nd;
    if (!LoadNNNetworkDescriptorNetCDF(file, nd)) return 1;
    printf("name=%s kind=%d errorFunction=%d layers=%zu weights=%zu\n", nd._name.c_str(), (int)nd._kind, (int)nd._errorFunction,
           nd._vLayerDescriptor.size(), nd._vWeightDescriptor.size());
    for (auto& l : nd._vLayerDescriptor)
        printf("layer %s kind=%d Nx=%u activation=%d attributes=%u dataSet=%s sources=%zu\n", l._name.c_str(), (int)l._kind, l._Nx,
               (int)l._activation, l._attributes, l._dataSet.c_str(), l._vSource.size());
    for (auto& w : nd._vWeightDescriptor) {
        double sw = 0, sb = 0;
        for (size_t i = 0; i < w._vWeight.size(); i++) sw += (double)w._vWeight[i] * (double)(i + 1);
        for (size_t i = 0; i < w._vBias.size(); i++) sb += (double)w._vBias[i] * (double)(i + 1);
        printf("weight %s->%s width=%lu height=%lu shared=%d nweights=%zu wsum=%.9g bsum=%.9g\n", w._inputLayer.c_str(),
               w._outputLayer.c_str(), (unsigned long)w._width, (unsigned long)w._height, (int)w._bShared, w._vWeight.size(), sw, sb);
    }
    return 0;
}

// --write-cdf2 file: a small CDF-2 file from this build's writer, to be read back by an independent reader.
static int writeCdf2(const string& file)
{
    ncc::Writer nc;
    nc.setVersion(2);
    nc.putAttString("title", "written by NcClassic");
    nc.putAttInt("answer", 42);
    nc.putAttFloat("ratio", 0.375f);
    static float fv[5] = {1.5f, -2.25f, 3.0f, 1e-3f, 7.0f};
    static int32_t iv[3] = {-7, 0, 123456789};
    static double dv[2] = {3.141592653589793, -1e100};
    uint32_t d5 = nc.addDim("five", 5), d3 = nc.addDim("three", 3), d2 = nc.addDim("two", 2);
    nc.addVar("fv", ncc::NC_FLOAT, d5, fv);
    nc.addVar("iv", ncc::NC_INT, d3, iv);
    nc.addVar("dv", ncc::NC_DOUBLE, d2, dv);
    nc.write(file);
    return 0;
}

// ---- index files and sample text (the cases of tst/unittests/TestNetCDFhelper.cpp, plus the sample parser) ------------------
static void testLoadIndex()
{
    const std::map<string, unsigned int> valid = {{"110510", 26743}, {"120372", 26744}, {"abc", 7}, {"x y", 0}};
    auto feed = [&](stringstream& in) {
        for (const auto& e : valid) in << e.first << "\t" << e.second << "\n";
    };
    {   // valid input
        stringstream in, out;
        feed(in);
        unordered_map<string, unsigned int> idx;
        CHECK(loadIndex(idx, in, out));
        CHECK(out.str().find("Error") == string::npos);
        CHECK_EQ(idx.size(), valid.size());
        for (const auto& e : valid) CHECK(idx.count(e.first) && idx[e.first] == e.second);
    }
    {   // a whole entry twice
        stringstream in, out;
        feed(in);
        in << valid.begin()->first << "\t" << valid.begin()->second << "\n";
        unordered_map<string, unsigned int> idx;
        CHECK(!loadIndex(idx, in, out));
        CHECK(out.str().find("Error") != string::npos);
    }
    {   // a label twice with another index
        stringstream in, out;
        feed(in);
        in << valid.begin()->first << "\t123\n";
        unordered_map<string, unsigned int> idx;
        CHECK(!loadIndex(idx, in, out));
        CHECK(out.str().find("Error") != string::npos);
    }
    for (const char* bad : {"\t123\n", "123\n", "110510\t123\t121017\n"}) {   // no label; no tab; an extra tab
        stringstream in(bad), out;
        unordered_map<string, unsigned int> idx;
        CHECK(!loadIndex(idx, in, out));
        CHECK(out.str().find("Error") != string::npos);
    }
}

static void testParseSamplesAndDatasetFile(const string& dir)
{
    unordered_map<string, unsigned int> features = {{"f0", 0}, {"f1", 1}, {"f2", 2}};
    unordered_map<string, unsigned int> samples;
    const string text =
        "s0\tf1,3.5:f2\n"
        "\n"                      // empty line: ignored
        "no tab on this line\n"   // malformed: skipped with a warning
        "s1\tf0,2,9:unknown,1:f2,0.25:\n"   // a third field is ignored (warning), an unknown feature is dropped, an empty tuple is skipped
        "s2\t\n"                 // a sample without data points
        "s0\tf0,1.5\n";          // the same sample again: the last line wins
    {
        stringstream in(text), out;
        bool fu = false, su = false;
        std::map<unsigned int, vector<unsigned int>> sig;
        std::map<unsigned int, vector<float>> val;
        CHECK(parseSamples(in, false, features, samples, fu, su, sig, val, out));
        CHECK(!fu && su);
        CHECK_EQ(features.size(), 3u);
        CHECK_EQ(samples.size(), 3u);
        CHECK(samples["s0"] == 0 && samples["s1"] == 1 && samples["s2"] == 2);
        CHECK(sig[0] == vector<unsigned int>({0}) && val[0] == vector<float>({1.5f}));
        CHECK(sig[1] == vector<unsigned int>({0, 2}) && val[1] == vector<float>({2.0f, 0.25f}));
        CHECK(sig[2].empty());
        CHECK(out.str().find("Warning") != string::npos);
    }
    {   // with feature updates an unknown feature gets the next index
        stringstream in("s9\tnew,1:f1\n"), out;
        bool fu = false, su = false;
        std::map<unsigned int, vector<unsigned int>> sig;
        std::map<unsigned int, vector<float>> val;
        unordered_map<string, unsigned int> f2 = features, s2;
        CHECK(parseSamples(in, true, f2, s2, fu, su, sig, val, out));
        CHECK(fu && f2["new"] == 3);
        CHECK(sig[0] == vector<unsigned int>({3, 1}) && val[0] == vector<float>({1.0f, 0.0f}));
    }
    // file -> CSR in sample-index order -> dataset file -> read back
    const string samplesFile = dir + "/samples.txt";
    {
        ofstream f(samplesFile);
        f << "b\tf2,1:f0,1\n" << "a\tf1,7\n";
    }
    unordered_map<string, unsigned int> sidx = {{"a", 0}};   // "a" is known: it stays row 0 although it comes second
    vector<unsigned int> vs, ve, vi;
    vector<float> vd;
    stringstream out;
    CHECK(generateNetCDFIndexes(samplesFile, false, dir + "/features.idx", dir + "/samples.idx", features, sidx, vs, ve, vi, vd, out));
    CHECK(vs == vector<unsigned int>({0, 1}) && ve == vector<unsigned int>({1, 3}));
    CHECK(vi == vector<unsigned int>({1, 2, 0}) && vd == vector<float>({7.0f, 1.0f, 1.0f}));
    CHECK(fileExists(dir + "/samples.idx") && !fileExists(dir + "/features.idx"));   // only the index that changed is exported
    unordered_map<string, unsigned int> reread;
    CHECK(loadIndexFromFile(reread, dir + "/samples.idx", out) && reread.size() == 2 && reread["b"] == 1);
    CHECK_EQ(roundUpMaxIndex(3), 128u);
    CHECK_EQ(roundUpMaxIndex(128), 128u);
    CHECK_EQ(roundUpMaxIndex(129), 256u);
    for (int analog = 0; analog < 2; analog++) {
        const string nc = dir + (analog ? "/analog.nc" : "/boolean.nc");
        if (analog) writeNetCDFFile(vs, ve, vi, vd, nc, "gl_input", (unsigned int)features.size());
        else writeNetCDFFile(vs, ve, vi, nc, "gl_input", (unsigned int)features.size());
        ncc::Reader r(nc);
        CHECK_EQ(r.att("datasets").asUInt64(), 1u);
        CHECK(r.att("name0").asString() == "gl_input");
        CHECK_EQ(r.att("attributes0").asUInt64(), analog ? (uint64_t)NNDataSetEnums::Sparse : (uint64_t)(NNDataSetEnums::Sparse | NNDataSetEnums::Boolean));
        CHECK_EQ(r.att("dataType0").asUInt64(), analog ? (uint64_t)NNDataSetEnums::Float : (uint64_t)NNDataSetEnums::UInt);
        CHECK_EQ(r.att("width0").asUInt64(), 128u);
        CHECK_EQ(r.dim("examplesDim0"), 2u);
        vector<uint64_t> s64;
        r.read<uint64_t>("sparseEnd0", s64);   // stored as 32-bit offsets, widened on reading
        CHECK(s64 == vector<uint64_t>({1, 3}));
        CHECK_EQ(r.hasVar("sparseData0"), analog != 0);
    }
}


static void testJsonReader()
{
    json::Value v;
    string err;
    CHECK(json::parse("{ \"a\" : [1, 2.5e1, -3], // note\n \"b\" : { \"c\" : \"x\\n\\u00e9\\\"\" }, /* c */ \"d\" : true, \"e\" : null, \"f\" : false }", v, err));
    CHECK(v.isObject() && v.members().size() == 5);
    CHECK(v.members()[0].first == "a" && v.members()[4].first == "f");   // file order is kept
    const json::Value* a = v.find("a");
    CHECK(a && a->isArray() && a->size() == 3);
    CHECK_EQ((*a)[1].asDouble(), 25.0);
    CHECK_EQ((*a)[2].asInt(), (int64_t)-3);
    CHECK(v.find("b")->find("c")->asString() == "x\n\xc3\xa9\"");
    CHECK(v.find("d")->asBool() && !v.find("f")->asBool() && v.find("e")->isNull());
    CHECK(v.find("zzz") == nullptr);
    CHECK_EQ(v.find("d")->size(), (size_t)1);            // a scalar reads as an array of one
    CHECK(&(*v.find("d"))[0] == v.find("d"));
    bool threw = false;
    try { v.find("a")->asString(); } catch (std::runtime_error&) { threw = true; }
    CHECK(threw);
    CHECK(json::parse("[]", v, err) && v.isArray() && v.size() == 0);
    CHECK(json::parse(" 7 ", v, err) && v.asInt() == 7);
    for (const char* bad : {"{", "{\"a\" 1}", "[1,]", "{\"a\":1,}", "\"abc", "tru", "{\"a\":1} x", "/* open", "[1 2]", "{'a':1}", ""}) {
        err.clear();
        CHECK(!json::parse(bad, v, err));
        CHECK(err.find("line ") == 0);
    }
    CHECK(!json::parse("{\n\n  \"a\" : ?\n}", v, err) && err.find("line 3, column 9") == 0);
    CHECK(json::lower("ReLU Max") == "relu max");
}

static const NNWeightDescriptor* findWeight(const NNNetworkDescriptor& nd, const string& in, const string& out)
{
    for (auto& w : nd._vWeightDescriptor)
        if (w._inputLayer == in && w._outputLayer == out) return &w;
    return nullptr;
}

static void testNetworkDefinitions(const string& dir, const string& golden)
{
    const vector<NNDataSetBase*> none;
    {   // data file of the reference's tests: tst/test_data/validate_L2_LRelu_02.json
        NNNetworkDescriptor nd;
        CHECK(LoadNNNetworkDescriptorJSON(golden + "/validate_L2_LRelu_02.json", nd, none));
        CHECK(nd._name == "L2 1d regression");
        CHECK_EQ((int)nd._kind, (int)NNNetwork::Kind::FeedForward);
        CHECK_EQ((int)nd._errorFunction, (int)ErrorFunction::L2);
        CHECK(!nd._bShuffleIndices);
        CHECK_EQ(nd._vLayerDescriptor.size(), (size_t)3);
        if (nd._vLayerDescriptor.size() != 3) return;   // fixture directory wrong or file unreadable: reported above
        const NNLayerDescriptor& in = nd._vLayerDescriptor[0];
        const NNLayerDescriptor& hid = nd._vLayerDescriptor[1];
        const NNLayerDescriptor& out = nd._vLayerDescriptor[2];
        CHECK(in._name == "Input" && in._kind == NNLayer::Kind::Input && in._Nx == 2 && in._dataSet == "input");
        CHECK(in._attributes == NNLayer::Attributes::Sparse);
        CHECK(hid._name == "Hidden" && hid._kind == NNLayer::Kind::Hidden && hid._activation == Activation::LeakyRectifiedLinear);
        CHECK_EQ(hid._RELUSlope, 0.5f);
        CHECK(hid._vSource == vector<string>({"Input"}));
        CHECK(out._kind == NNLayer::Kind::Output && out._activation == Activation::Linear && out._dataSet == "output");
        CHECK(out._vSource == vector<string>({"Input"}));      // the output reads the input, not the hidden layer
        CHECK_EQ(nd._vWeightDescriptor.size(), (size_t)2);
        CHECK(findWeight(nd, "Input", "Hidden") && findWeight(nd, "Input", "Output") && !findWeight(nd, "Hidden", "Output"));
        CHECK(nd._vWeightDescriptor[0]._vWeight.empty() && !nd._vWeightDescriptor[0]._bShared);
        // layers without a slope of their own take the network's (default 0.0... is stored, never NaN)
        CHECK(!std::isnan(out._RELUSlope) && !std::isnan(out._ELUAlpha) && !std::isnan(out._SELULambda));
    }
    {   // the MovieLens sample definition sizes two layers from data sets, which are not there
        NNNetworkDescriptor nd;
        CHECK(!LoadNNNetworkDescriptorJSON(golden + "/movielens_config.json", nd, none));
    }
    {
        NNNetworkDescriptor nd;
        CHECK(LoadNNNetworkDescriptorJSON(golden + "/tied_autoencoder.json", nd, none));
        CHECK(nd._name == "tied autoencoder" && nd._kind == NNNetwork::Kind::AutoEncoder && nd._errorFunction == ErrorFunction::CrossEntropy);
        CHECK(nd._bShuffleIndices);
        CHECK_EQ(nd._RELUSlope, 0.125f);
        CHECK_EQ(nd._ELUAlpha, 1.5f);
        CHECK_EQ(nd._decay, 0.25f);
        CHECK_EQ(nd._deltaBoost_one, 30.0f);
        CHECK_EQ(nd._deltaBoost_zero, 2.0f);
        CHECK_EQ(nd._LRN_k, 3.0f);
        CHECK_EQ(nd._LRN_n, 7u);
        CHECK_EQ(nd._LRN_alpha, 0.5f);
        CHECK_EQ(nd._LRN_beta, 0.25f);
        CHECK_EQ(nd._maxout_k, 4u);
        CHECK_EQ(nd._vLayerDescriptor.size(), (size_t)5);
        const auto& L = nd._vLayerDescriptor;
        CHECK(L[0]._name == "Input0" && L[0]._kind == NNLayer::Kind::Input && L[0]._Nx == 96 && (L[0]._attributes & NNLayer::Attributes::Sparse));
        CHECK(L[1]._name == "Enc" && L[1]._kind == NNLayer::Kind::Hidden && L[1]._vSource == vector<string>({"Input0"}));
        CHECK(L[1]._weightInit == Gaussian && L[1]._weightInitScale == 0.01f && L[1]._biasInit == 0.5f);
        CHECK_EQ(L[1]._RELUSlope, 0.125f);                       // network default
        CHECK(L[2]._activation == Activation::ExponentialLinear && L[2]._ELUAlpha == 0.75f && L[2]._pDropout == 0.5f);
        CHECK(L[2]._vSkip == vector<string>({"Enc"}) && L[2]._dimensions == 1 && L[2]._Nx == 32);
        CHECK(L[2]._weightInit == Constant);
        CHECK(L[3]._kind == NNLayer::Kind::Hidden && L[3]._vSource == vector<string>({"Input0", "Enc"}) && L[3]._weightNorm == 2.0f);
        CHECK_EQ(L[3]._ELUAlpha, 1.5f);
        CHECK(L[4]._kind == NNLayer::Kind::Output && L[4]._name == "Out" && L[4]._dataSet == "out");
        CHECK_EQ(nd._vWeightDescriptor.size(), (size_t)6);
        const NNWeightDescriptor* tied = findWeight(nd, "Mid", "Out");
        CHECK(tied && tied->_bShared && tied->_bTransposed && tied->_sourceInputLayer == "Input0" && tied->_sourceOutputLayer == "Enc");
        const NNWeightDescriptor* side = findWeight(nd, "Side", "Out");
        CHECK(side && !side->_bShared);
        CHECK(findWeight(nd, "Enc", "Side") && findWeight(nd, "Enc", "Side")->_norm == 2.0f);
        // the descriptor survives the binary network format (weights stay empty)
        NNNetworkDescriptor back;
        CHECK(SaveNNNetworkDescriptorNetCDF(dir + "/tied.nc", nd) && LoadNNNetworkDescriptorNetCDF(dir + "/tied.nc", back));
        CHECK(back._vLayerDescriptor.size() == 5 && back._vLayerDescriptor[2]._vSkip == vector<string>({"Enc"}));
        CHECK(back._vWeightDescriptor.size() == 6 && back._vWeightDescriptor[4]._bTransposed);
    }
    // what the loader refuses, one definition each
    struct Case { const char* what; const char* text; };
    const Case refused[] = {
        {"old version", "{\"Version\": 0.5, \"Layers\": [{\"N\": 2}, {\"N\": 2}]}"},
        {"unknown network key", "{\"Layers\": [{\"N\": 2}, {\"N\": 2}], \"Colour\": 1}"},
        {"unknown network kind", "{\"Kind\": \"Recurrent\", \"Layers\": [{\"N\": 2}, {\"N\": 2}]}"},
        {"unknown error function", "{\"ErrorFunction\": \"L3\", \"Layers\": [{\"N\": 2}, {\"N\": 2}]}"},
        {"unknown layer key", "{\"Layers\": [{\"N\": 2}, {\"N\": 2, \"Colour\": 1}]}"},
        {"activation on an input layer", "{\"Layers\": [{\"N\": 2, \"Activation\": \"Relu\"}, {\"N\": 2}]}"},
        {"data set on a hidden layer", "{\"Layers\": [{\"N\": 2}, {\"N\": 2, \"DataSet\": \"x\"}, {\"N\": 2}]}"},
        {"source on an input layer", "{\"Layers\": [{\"N\": 2, \"Source\": \"x\"}, {\"N\": 2}]}"},
        {"auto on a hidden layer", "{\"Layers\": [{\"N\": 2}, {\"N\": \"auto\"}, {\"N\": 2}]}"},
        {"auto without its data set", "{\"Layers\": [{\"N\": \"auto\", \"DataSet\": \"nowhere\"}, {\"N\": 2}]}"},
        {"duplicate layer name", "{\"Layers\": [{\"Name\": \"a\", \"N\": 2}, {\"Name\": \"a\", \"N\": 2}]}"},
        {"five dimensions", "{\"Layers\": [{\"N\": [1, 2, 3, 4, 5]}, {\"N\": 2}]}"},
        {"unknown activation", "{\"Layers\": [{\"N\": 2}, {\"N\": 2, \"Activation\": \"Swish\"}]}"},
        {"unknown layer kind", "{\"Layers\": [{\"N\": 2}, {\"N\": 2, \"Kind\": \"Middle\"}]}"},
        {"unknown layer type", "{\"Layers\": [{\"N\": 2}, {\"N\": 2, \"Type\": \"Dense\"}]}"},
        {"unknown weight scheme", "{\"Layers\": [{\"N\": 2}, {\"N\": 2, \"WeightInit\": {\"Scheme\": \"He\"}}]}"},
        {"unknown weight init field", "{\"Layers\": [{\"N\": 2}, {\"N\": 2, \"WeightInit\": {\"Gain\": 1}}]}"},
        {"unknown shared weight field", "{\"Layers\": [{\"N\": 2}, {\"N\": 2}, {\"N\": 2, \"SharedWeights\": {\"Transpose\": true}}]}"},
        {"shared weight without its source", "{\"Layers\": [{\"N\": 2}, {\"N\": 2}, {\"N\": 2, \"SharedWeights\": {\"InputLayer\": \"nope\"}}]}"},
        {"unknown penalty parameter", "{\"SparsenessPenalty\": {\"q\": 1}, \"Layers\": [{\"N\": 2}, {\"N\": 2}]}"},
        {"not JSON", "{\"Layers\": [{\"N\": 2}, {\"N\": 2}]"},
    };
    for (auto& c : refused) {
        const string f = dir + "/refused.json";
        { ofstream o(f); o << c.text; }
        NNNetworkDescriptor nd;
        if (LoadNNNetworkDescriptorJSON(f, nd, none)) {
            printf("FAILED: definition with %s was accepted\n", c.what);
            CHECK(false);
        } else
            CHECK(true);
    }
    {   // defaults: kinds by position, names by kind and position, Sigmoid, Xavier, chain of sources, multi-dimensional N
        const string f = dir + "/defaults.json";
        { ofstream o(f); o << "{\"Layers\": [{\"N\": [4, 3, 2]}, {\"N\": 5}, {\"N\": 6, \"Sparse\": false}], \"Denoising\": {\"p\": 0.25},"
                              " \"SparsenessPenalty\": {\"p\": 0.1, \"beta\": 0.5}}"; }
        NNNetworkDescriptor nd;
        CHECK(LoadNNNetworkDescriptorJSON(f, nd, none));
        const auto& L = nd._vLayerDescriptor;
        CHECK(L.size() == 3 && L[0]._name == "Input0" && L[1]._name == "Hidden1" && L[2]._name == "Output2");
        CHECK(L[0]._Nx == 4 && L[0]._Ny == 3 && L[0]._Nz == 2 && L[0]._dimensions == 3);
        CHECK(L[1]._activation == Activation::Sigmoid && L[1]._weightInit == Xavier && L[1]._vSource == vector<string>({"Input0"}));
        CHECK(L[2]._vSource == vector<string>({"Hidden1"}) && L[2]._attributes == NNLayer::Attributes::None);
        CHECK(nd._bDenoising && nd._bSparsenessPenalty);
        CHECK(!(L[0]._attributes & NNLayer::Attributes::Denoising));   // only sparse input layers are denoised
        CHECK_EQ(nd._vWeightDescriptor.size(), (size_t)2);
    }
    {   // a single layer object instead of an array, a convolutional entry with a kernel (parsed, not built)
        const string f = dir + "/conv.json";
        { ofstream o(f); o << "{\"Layers\": [{\"N\": [8, 8, 3]}, {\"Type\": \"Convolutional\", \"N\": 16, \"Kernel\": [3, 3], \"KernelStride\": 2},"
                              " {\"Type\": \"Pooling\", \"Function\": \"Max\", \"Kernel\": [2, 2]}, {\"N\": 10, \"Activation\": \"SoftMax\"}]}"; }
        NNNetworkDescriptor nd;
        CHECK(LoadNNNetworkDescriptorJSON(f, nd, none));
        const auto& L = nd._vLayerDescriptor;
        CHECK(L[1]._type == NNLayer::Type::Convolutional && L[1]._kernelX == 3 && L[1]._kernelY == 3 && L[1]._kernelDimensions == 2);
        CHECK(L[1]._kernelStrideX == 2 && L[1]._kernelStrideY == 1 && !L[1]._bDimensionsProvided);
        CHECK(L[2]._type == NNLayer::Type::Pooling && L[2]._poolingFunction == PoolingFunction::Max);
        CHECK_EQ(nd._vWeightDescriptor.size(), (size_t)2);       // pooling layers have no weights
        CHECK(L[3]._activation == Activation::SoftMax);
    }
}

int main(int argc, char** argv)
{
    if (argc > 2 && string(argv[1]) == "--dump-network") return dumpNetwork(argv[2]);
    if (argc > 2 && string(argv[1]) == "--write-cdf2") return writeCdf2(argv[2]);
    const string dir = argc > 1 ? argv[1] : "/tmp";
    const string golden = argc > 2 ? argv[2] : "tests/golden/ldl";
    testDimensions();
    testNetworkFileRoundTrip(dir);
    testFilters(dir);
    testTopKsort();
    testUtils(dir);
    testKnnHost(dir);
    testLoadIndex();
    testParseSamplesAndDatasetFile(dir);
    testJsonReader();
    testNetworkDefinitions(dir, golden);
    return finish("test_host_cpu");
}
