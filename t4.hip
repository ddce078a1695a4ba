#include <hip/hip_runtime.h>
__global__ void k(unsigned short* p, unsigned short v){
  __hip_atomic_store(p+threadIdx.x, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
