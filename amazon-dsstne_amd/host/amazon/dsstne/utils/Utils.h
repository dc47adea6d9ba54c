// Utils.h — small host helpers of the prediction tools (reference: utils/Utils.h): string splitting, index files and the
// CPU top-K used to cross-check the device kernel.
#ifndef DSSTNE_AMD_UTILS_H
#define DSSTNE_AMD_UTILS_H

#include <chrono>
#include <string>
#include <unordered_map>
#include <vector>

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

std::vector<std::string> split(const std::string& s, char delim);
bool fileExists(const std::string& fileName);
// Files of a directory (or the file itself when dirname is a file), sorted by name.  Returns 0 on success.
int listFiles(const std::string& dirname, const bool recursive, std::vector<std::string>& files);

// "label<TAB>index" lines -> label->index map and index->label vector (reference: utils/NetCDFhelper.cpp loadIndex).
bool loadIndexFile(const std::string& fileName, std::unordered_map<std::string, unsigned int>& labelToIndex,
                   std::vector<std::string>& indexToLabel);

// Top-k of keys[0..size) (values default to positions), sorted by key (or by value) descending; equal keys keep the
// lower position first.
template <typename Tkey, typename Tval>
void topKsort(Tkey* keys, Tval* vals, const int size, Tkey* topKkeys, Tval* topKvals, const int topK, const bool sortByKey = true);

#endif
