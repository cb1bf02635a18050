// bind_core, init_cuda and SizedGPUBuffer (reference src/util/util.cpp, src/util/gpu_util.cpp).
#include <sched.h>
#include <algorithm>
#include "util/common.h"
#include "util/gpu_util.h"

void bind_core(int core_id) {
    cpu_set_t mask;
    CPU_ZERO(&mask);
    CPU_SET(core_id, &mask);
    if (sched_setaffinity(0, sizeof(mask), &mask) != 0) std::fprintf(stderr, "Failed to bind core %d\n", core_id);
}

namespace foo {
namespace util {

void init_cuda() { ASSERT_CUDA_ERROR(gp_init(0)); }

SizedGPUBuffer::SizedGPUBuffer(size_t size) : size_(size) { ASSERT_CUDA_ERROR(gp_malloc(&ptr_, size)); }
SizedGPUBuffer::~SizedGPUBuffer() { gp_free(ptr_); }
void SizedGPUBuffer::from_vector(std::vector<float> &vec) { gp_memcpy_h2d(ptr_, vec.data(), std::min(size_, vec.size() * sizeof(float))); }
void SizedGPUBuffer::to_vector(std::vector<float> &vec) {
    vec.resize(size_ / sizeof(float));
    gp_memcpy_d2h(vec.data(), ptr_, size_);
}

}  // namespace util
}  // namespace foo
