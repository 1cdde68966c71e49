// Kernels for the module checks of shim_app: built as a code object file (--genco) and
// loaded with hipModuleLoad at run time.
#include <hip/hip_runtime.h>

extern "C" __global__ void ModScale(uint32_t *p, uint32_t factor, uint32_t count)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) p[i] *= factor;
}

extern "C" __global__ void ModShift(uint32_t *p, unsigned short add, uint32_t count)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) p[i] += add;
}
