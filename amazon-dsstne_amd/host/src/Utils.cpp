// Utils.cpp — host helpers (reference: utils/Utils.cpp:93-250).
#include "amazon/dsstne/utils/Utils.h"

#include <dirent.h>
#include <sys/stat.h>

#include <algorithm>
#include <fstream>
#include <iostream>
#include <sstream>

using namespace std;

char* getCmdOption(char** begin, char** end, const string& option)
{
    char** it = find(begin, end, option);
    return (it != end && it + 1 != end) ? *(it + 1) : nullptr;
}

bool cmdOptionExists(char** begin, char** end, const string& option) { return find(begin, end, option) != end; }

string getRequiredArgValue(int argc, char** argv, string flag, string message, void (*usage)())
{
    char* value = getCmdOption(argv, argv + argc, flag);
    if (!value) {   // missing flag, or a flag without a value after it
        cout << "Error: Missing required argument: " << flag << ": " << message << endl;
        if (usage) usage();
        exit(1);
    }
    return string(value);
}

string getOptionalArgValue(int argc, char** argv, string flag, string defaultValue)
{
    char* value = getCmdOption(argv, argv + argc, flag);
    return value ? string(value) : defaultValue;
}

bool isArgSet(int argc, char** argv, string flag) { return cmdOptionExists(argv, argv + argc, flag); }

vector<string>& split(const string& s, char delim, vector<string>& elems)
{
    stringstream ss(s);
    string item;
    while (getline(ss, item, delim)) elems.push_back(item);
    return elems;
}

vector<string> split(const string& s, char delim)
{
    vector<string> out;
    split(s, delim, out);
    return out;
}

bool isNetCDFfile(const string& filename)
{
    const size_t dot = filename.find_last_of('.');
    return dot != string::npos && filename.compare(dot, string::npos, NETCDF_FILE_EXTENTION) == 0;
}

bool isDirectory(const string& dirname)
{
    struct stat st;
    return stat(dirname.c_str(), &st) == 0 && S_ISDIR(st.st_mode);
}

bool isFile(const string& filename)
{
    struct stat st;
    return stat(filename.c_str(), &st) == 0 && S_ISREG(st.st_mode);
}

bool fileExists(const string& fileName)
{
    struct stat st;
    return stat(fileName.c_str(), &st) == 0;
}

int listFiles(const string& dirname, const bool recursive, vector<string>& files)
{
    struct stat st;
    if (stat(dirname.c_str(), &st) != 0) {
        cout << "Unable to read " << dirname << endl;
        return 1;
    }
    if (!S_ISDIR(st.st_mode)) {
        files.push_back(dirname);
        return 0;
    }
    DIR* dir = opendir(dirname.c_str());
    if (!dir) return 1;
    struct dirent* ent;
    while ((ent = readdir(dir)) != NULL) {
        const string name = ent->d_name;
        if (name == "." || name == "..") continue;
        const string path = dirname + "/" + name;
        if (stat(path.c_str(), &st) != 0) continue;
        if (S_ISDIR(st.st_mode)) {
            if (recursive) listFiles(path, recursive, files);
        } else {
            files.push_back(path);
        }
    }
    closedir(dir);
    sort(files.begin(), files.end());
    return 0;
}

bool loadIndexFile(const string& fileName, unordered_map<string, unsigned int>& labelToIndex, vector<string>& indexToLabel)
{
    ifstream in(fileName);
    if (!in) {
        cout << "Error: Failed to open index file " << fileName << endl;
        return false;
    }
    string line;
    while (getline(in, line)) {
        size_t tab = line.find('\t');
        if (tab == string::npos) continue;
        const string label = line.substr(0, tab);
        const unsigned int index = (unsigned int)stoul(line.substr(tab + 1));
        labelToIndex[label] = index;
        if (indexToLabel.size() <= index) indexToLabel.resize(index + 1);
        indexToLabel[index] = label;
    }
    return true;
}

template <typename Tkey, typename Tval>
void topKsort(Tkey* keys, Tval* vals, const int size, Tkey* topKkeys, Tval* topKvals, const int topK, const bool sortByKey)
{
    if (!keys || !topKkeys || !topKvals) {
        cout << "null input array" << endl;
        exit(0);
    }
    struct Item {
        Tkey key;
        Tval val;
        int pos;
    };
    vector<Item> data(size);
    for (int i = 0; i < size; i++) data[i] = Item{keys[i], vals ? vals[i] : (Tval)i, i};
    const int m = min(topK, size);
    auto byKey = [](const Item& a, const Item& b) { return a.key > b.key || (a.key == b.key && a.pos < b.pos); };
    auto byVal = [](const Item& a, const Item& b) { return a.val > b.val || (a.val == b.val && a.pos < b.pos); };
    if (sortByKey)
        partial_sort(data.begin(), data.begin() + m, data.end(), byKey);
    else
        partial_sort(data.begin(), data.begin() + m, data.end(), byVal);
    for (int i = 0; i < m; i++) {
        topKkeys[i] = data[i].key;
        topKvals[i] = data[i].val;
    }
}

template void topKsort<float, unsigned int>(float*, unsigned int*, const int, float*, unsigned int*, const int, const bool);
template void topKsort<float, float>(float*, float*, const int, float*, float*, const int, const bool);
