// DataReader.h — row source for the KNN item table (reference: knn/DataReader.h:23-64).
#ifndef DSSTNE_AMD_KNN_DATAREADER_H
#define DSSTNE_AMD_KNN_DATAREADER_H

#include <cstdint>
#include <fstream>
#include <string>

class DataReader {
public:
    // Parses the next row into *key and vector[0 .. columns); false at end of data.
    virtual bool readRow(std::string* key, float* vector) = 0;
    uint32_t getRows() const { return rows; }
    int getColumns() const { return columns; }
    virtual ~DataReader() {}

protected:
    uint32_t rows = 0;
    int columns = 0;
};

// Text file with one "key<kv-delimiter>v0<vec-delimiter>v1..." line per item.
class TextFileDataReader : public DataReader {
public:
    TextFileDataReader(const std::string& fileName, char keyValueDelimiter = '\t', char vectorDelimiter = ' ');
    bool readRow(std::string* key, float* vector) override;
    static void findDataDimensions(const std::string& fileName, uint32_t& rows, int& columns, char keyValueDelimiter = '\t',
                                   char vectorDelimiter = ' ');
    ~TextFileDataReader();

private:
    std::string fileName;
    std::fstream fileStream;
    char keyValueDelimiter;
    char vectorDelimiter;
};

// In-memory rows (row-major [rows][columns]) with generated or supplied keys.
class ArrayDataReader : public DataReader {
public:
    ArrayDataReader(const float* data, uint32_t rows, int columns, const std::string* keys = nullptr);
    bool readRow(std::string* key, float* vector) override;

private:
    const float* data;
    const std::string* keys;
    uint32_t next;
};

#endif
