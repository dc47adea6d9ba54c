// GpuTypes.cpp — the process-wide device context (reference: engine/GpuTypes.cpp:62-406 Startup, 434-472 Shutdown,
// 475-498 SetNeuralNetwork, 408-414 CopyConstants, 501-516 SetRandomSeed, 520-525 GetMemoryUsage), one process, one GPU.
#include "amazon/dsstne/engine/GpuTypes.h"

static GpuContext gpu;

GpuContext& getGpu() { return gpu; }

void dsxFatal(int status, const char* what)
{
    if (status == DSX_OK) return;
    printf("%s: %s\n", what, dsx_last_error());
    fflush(stdout);
    getGpu().Shutdown();
    exit(-1);
}

GpuContext::GpuContext()
    : _id(0), _numprocs(1), _device(0), _bStarted(false), _bCPUValidate(false), _randomSeed(0), _pNetwork(NULL), _warpSize(64),
      _threadsPerBlock(256), _totalGPUMemory(0), _totalCPUMemory(0)
{
}

GpuContext::~GpuContext() {}

void GpuContext::Startup(int argc, char** argv)
{
    (void)argc;
    (void)argv;
    if (_bStarted) return;
    const char* dev = getenv("DSSTNE_DEVICE");
    _device = dev ? atoi(dev) : 0;
    int rc = dsx_init(_device);
    if (rc != DSX_OK) {
        printf("GpuContext::Startup: %s\n", dsx_last_error());
        fflush(stdout);
        exit(-1);
    }
    dsx_device_info info;
    if (dsx_get_device_info(&info) == DSX_OK) {
        printf("GpuContext::Startup: Process 0 out of 1 initialized on device %d: %s (%s), %d CUs, %.1f GiB HBM.\n", _device, info.name,
               info.arch, info.compute_units, (double)info.hbm_bytes / (1024.0 * 1024.0 * 1024.0));
        _warpSize = info.wavefront_size;
    }
    _bStarted = true;
}

void GpuContext::Shutdown()
{
    if (!_bStarted) return;
    _bStarted = false;
    _pNetwork = NULL;
    dsx_shutdown();
    printf("GpuContext::Shutdown: Process 0 out of 1 finalized.\n");
}

void GpuContext::SetRandomSeed(unsigned long seed)
{
    // Weights are always supplied in this build, so the seed only has to be remembered.
    _randomSeed = seed;
    printf("GpuContext::SetRandomSeed: Random seed set to %lu.\n", seed);
}

void GpuContext::CopyConstants() {}   // kernels take their parameters as arguments; there are no constant blocks to refresh

void GpuContext::SetNeuralNetwork(NNNetwork* pNetwork) { _pNetwork = pNetwork; }

void GpuContext::SetCPUValidate(bool bCPUValidate) { _bCPUValidate = bCPUValidate; }

void GpuContext::GetMemoryUsage(int* gpuMemory, int* cpuMemory)
{
    if (gpuMemory) *gpuMemory = (int)(_totalGPUMemory / 1024ll);
    if (cpuMemory) *cpuMemory = (int)(_totalCPUMemory / 1024ll);
}
