// Utils.h — small host helpers of the prediction tools (reference: utils/Utils.h): string splitting, index files and the
// CPU top-K used to cross-check the device kernel.
#ifndef DSSTNE_AMD_UTILS_H
#define DSSTNE_AMD_UTILS_H

#include <chrono>
#include <cstdlib>
#include <string>
#include <unordered_map>
#include <vector>

// Names that the tools agree on (reference: utils/Utils.h:24-27): the suffixes of a generated data set's name, the
// extension isNetCDFfile looks for and the seed of the reproducible runs.
const std::string INPUT_DATASET_SUFFIX = "_input";
const std::string OUTPUT_DATASET_SUFFIX = "_output";
const std::string NETCDF_FILE_EXTENTION = ".nc";
const unsigned long FIXED_SEED = 12134ull;

// Command-line helpers of the tools (reference: utils/Utils.cpp:42-95).  A flag's value is the argument that follows it.
char* getCmdOption(char** begin, char** end, const std::string& option);
bool cmdOptionExists(char** begin, char** end, const std::string& option);
// Prints the message and the usage and exits with status 1 when the flag is missing.
std::string getRequiredArgValue(int argc, char** argv, std::string flag, std::string message, void (*usage)());
std::string getOptionalArgValue(int argc, char** argv, std::string flag, std::string defaultValue);
bool isArgSet(int argc, char** argv, std::string flag);

template <typename Clock, typename Duration1, typename Duration2>
double elapsed_seconds(std::chrono::time_point<Clock, Duration1> start, std::chrono::time_point<Clock, Duration2> end)
{
    return std::chrono::duration_cast<std::chrono::duration<double>>(end - start).count();
}

// Pieces of s between delim characters; the three-argument form appends to elems and returns it.
std::vector<std::string>& split(const std::string& s, char delim, std::vector<std::string>& elems);
std::vector<std::string> split(const std::string& s, char delim);
bool fileExists(const std::string& fileName);
// True when the name's last extension is ".nc" (reference: utils/Utils.cpp:114-123); the file is not opened.
bool isNetCDFfile(const std::string& filename);
// True iff the path exists and is a directory / a regular file (reference: utils/Utils.cpp:147-157; a path that does
// not exist is neither, where the reference reads an unset stat buffer).
bool isDirectory(const std::string& dirname);
bool isFile(const std::string& filename);
// Files of a directory (or the file itself when dirname is a file), sorted by name.  Returns 0 on success.
int listFiles(const std::string& dirname, const bool recursive, std::vector<std::string>& files);

// "label<TAB>index" lines -> label->index map and index->label vector (reference: utils/NetCDFhelper.cpp loadIndex).
bool loadIndexFile(const std::string& fileName, std::unordered_map<std::string, unsigned int>& labelToIndex,
                   std::vector<std::string>& indexToLabel);

// Top-k of keys[0..size) (values default to positions), sorted by key (or by value) descending; equal keys keep the
// lower position first.
template <typename Tkey, typename Tval>
void topKsort(Tkey* keys, Tval* vals, const int size, Tkey* topKkeys, Tval* topKvals, const int topK, const bool sortByKey = true);

// Uniform draws from the C library's generator, both ends included (reference: utils/Utils.h:120-128).
inline int rand(int min, int max) { return std::rand() % (max - min + 1) + min; }
inline float rand(float min, float max) { return min + ((float)std::rand() / (float)RAND_MAX) * (max - min); }

#endif
