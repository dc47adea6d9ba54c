// GpuTypes.h — process-wide device context and typed device buffers for the MI355X build.
//
// Public surface follows the reference's engine/GpuTypes.h (GpuContext at :317-390, GpuBuffer<T> at :392-625, getGpu()),
// restricted to what the single-GPU inference path uses.  All device work goes through the C ABI of libdsx_hip.so
// (include/dsx.h); this header contains no HIP or CUDA types.
#ifndef DSSTNE_AMD_GPUTYPES_H
#define DSSTNE_AMD_GPUTYPES_H

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <map>
#include <memory>
#include <string>
#include <tuple>
#include <vector>

#include "dsx.h"

using std::cout;
using std::endl;
using std::map;
using std::ostream;
using std::string;
using std::tuple;
using std::unique_ptr;
using std::vector;

// engine/GpuTypes.h:87-97: single precision is the only live precision mode
typedef float NNFloat;

class NNNetwork;

// Reports a failed device call the way RTERROR does (engine/GpuTypes.h:248-254): message, shutdown, exit(-1).
void dsxFatal(int status, const char* what);

struct GpuContext {
    int _id;                    // rank of this process: always 0 (one GPU, one process)
    int _numprocs;              // always 1
    int _device;
    bool _bStarted;
    bool _bCPUValidate;
    unsigned long _randomSeed;
    NNNetwork* _pNetwork;
    int _warpSize;              // 64 on CDNA
    int _threadsPerBlock;
    long long _totalGPUMemory;  // bytes held by GpuBuffers
    long long _totalCPUMemory;

    GpuContext();
    ~GpuContext();
    void Startup(int argc, char** argv);
    void Shutdown();
    void SetRandomSeed(unsigned long seed);
    void CopyConstants();
    void SetNeuralNetwork(NNNetwork* pNetwork);
    void SetCPUValidate(bool bCPUValidate);
    void GetMemoryUsage(int* gpuMemory, int* cpuMemory);
};

GpuContext& getGpu();

template <typename T> struct GpuBuffer {
    size_t _length;
    bool _bSysMem;
    bool _bManaged;
    T* _pSysData;
    T* _pDevData;

    GpuBuffer(int length, bool bSysMem = false, bool bManaged = false) : GpuBuffer((size_t)length, bSysMem, bManaged) {}
    GpuBuffer(unsigned int length, bool bSysMem = false, bool bManaged = false) : GpuBuffer((size_t)length, bSysMem, bManaged) {}
    GpuBuffer(unsigned long long int length, bool bSysMem = false, bool bManaged = false) : GpuBuffer((size_t)length, bSysMem, bManaged) {}
    GpuBuffer(size_t length, bool bSysMem = false, bool bManaged = false)
        : _length(length), _bSysMem(bSysMem), _bManaged(bManaged), _pSysData(NULL), _pDevData(NULL)
    {
        Allocate();
    }
    GpuBuffer(const GpuBuffer&) = delete;
    GpuBuffer& operator=(const GpuBuffer&) = delete;
    virtual ~GpuBuffer() { Deallocate(); }

    // Device memory is zero-filled; a managed buffer is host-dereferenceable and shadows itself (_pSysData == _pDevData).
    void Allocate()
    {
        if (_bManaged) _bSysMem = true;
        void* p = NULL;
        const size_t bytes = _length * sizeof(T);
        if (_bManaged) {
            dsxFatal(dsx_malloc_managed(&p, bytes), "GpuBuffer::Allocate failed (managed)");
            _pDevData = (T*)p;
            _pSysData = _pDevData;
        } else {
            dsxFatal(dsx_malloc(&p, bytes), "GpuBuffer::Allocate failed");
            _pDevData = (T*)p;
            if (_bSysMem) {
                _pSysData = new T[_length ? _length : 1];
                memset((void*)_pSysData, 0, bytes);
                getGpu()._totalCPUMemory += bytes;
            }
        }
        getGpu()._totalGPUMemory += bytes;
    }

    // Grows only; contents are lost when it grows.
    void Resize(size_t length)
    {
        if (length > _length) {
            Deallocate();
            _length = length;
            Allocate();
        }
    }

    void Deallocate()
    {
        const size_t bytes = _length * sizeof(T);
        if (_pDevData) {
            if (dsx_is_initialized()) dsxFatal(dsx_free(_pDevData), "GpuBuffer::Deallocate failed");
            getGpu()._totalGPUMemory -= bytes;
        }
        if (_bSysMem && !_bManaged && _pSysData) {
            delete[] _pSysData;
            getGpu()._totalCPUMemory -= bytes;
        }
        _pSysData = NULL;
        _pDevData = NULL;
        _length = 0;
    }

    void Upload(const T* pBuff = NULL) const
    {
        if (pBuff)
            dsxFatal(dsx_memcpy_h2d(_pDevData, pBuff, _length * sizeof(T)), "GpuBuffer::Upload failed");
        else if (_bSysMem && !_bManaged)
            dsxFatal(dsx_memcpy_h2d(_pDevData, _pSysData, _length * sizeof(T)), "GpuBuffer::Upload failed");
    }

    void Download(T* pBuff = NULL)
    {
        if (pBuff)
            dsxFatal(dsx_memcpy_d2h(pBuff, _pDevData, _length * sizeof(T)), "GpuBuffer::Download failed");
        else if (_bSysMem && !_bManaged)
            dsxFatal(dsx_memcpy_d2h(_pSysData, _pDevData, _length * sizeof(T)), "GpuBuffer::Download failed");
        else if (_bManaged)
            dsxFatal(dsx_sync(), "GpuBuffer::Download failed (sync)");
    }

    void Copy(T* pBuff) { dsxFatal(dsx_memcpy_d2d(_pDevData, pBuff, _length * sizeof(T)), "GpuBuffer::Copy failed"); }

    size_t GetLength() { return _length; }
    size_t GetSize() { return _length * sizeof(T); }
};

#endif
