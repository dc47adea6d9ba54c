// ref_shim.cpp — TEST INFRASTRUCTURE.  C-ABI binding over the reference's own CPU top-K routine, topKsort
// (utils/Utils.cpp:207-250), so that tests can call the real reference code from Python.  This file contains no
// reference source: it is compiled together with /root/reference/src/amazon/dsstne/utils/Utils.cpp, taken where it
// lies, by oracle/Makefile into oracle/_ref/libref_utils.so.
#include <cstdint>
#include "Utils.h"

extern "C" {

// topKsort<float, unsigned int>(keys, NULL, size, topKkeys, topKvals, topK, sortByKey = true):
// values default to the element position, result ordered by key descending (tie order unspecified).
void ref_topksort_f32_u32(float* keys, int size, float* top_keys, unsigned int* top_vals, int top_k)
{
    topKsort<float, unsigned int>(keys, nullptr, size, top_keys, top_vals, top_k, true);
}

// topKsort<float, float>(keys, vals, ...): explicit float payloads.
void ref_topksort_f32_f32(float* keys, float* vals, int size, float* top_keys, float* top_vals, int top_k)
{
    topKsort<float, float>(keys, vals, size, top_keys, top_vals, top_k, true);
}

}
