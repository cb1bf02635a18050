// GPU* vocabulary of the reference (include/util/gpu_util.h:74-162) expressed over the C ABI of
// libgpreempt_hip.so.  There is one backend (HIP on gfx950) and no CUDA/HIP switch: host code
// never includes a HIP header, it only sees opaque handles and plain pointers.
#pragma once
#include <cstddef>
#include <string>
#include <vector>
#include "gpreempt_hip.h"
#include "util/common.h"

typedef void *GPUdeviceptr;
typedef gp_stream GPUstream;
typedef gp_graph GPUgraphExec;
typedef int GPUresult;
#define GPU_SUCCESS 0

inline const char *GPUGetErrorString(GPUresult) { return gp_last_error(); }

// Stream / memory calls the reference's clients and tests use directly
// (src/cuda-clients/blpclient.cpp:121-133, src/tests/test-dnn-blp.cpp:13-22).
inline GPUresult GPUStreamCreate(GPUstream *s, unsigned /*flags*/) { return gp_stream_create(0, s); }
inline GPUresult GPUStreamCreateWithPriority(GPUstream *s, unsigned /*flags*/, int priority) { return gp_stream_create(priority, s); }
inline GPUresult GPUStreamDestroy(GPUstream s) { return gp_stream_destroy(s); }
inline GPUresult GPUStreamSynchronize(GPUstream s) { return gp_stream_sync(s); }
inline GPUresult GPUMemAlloc(GPUdeviceptr *p, size_t bytes) { return gp_malloc(p, bytes); }
inline GPUresult GPUMemFree(GPUdeviceptr p) { return gp_free(p); }
inline GPUresult GPUMemHostAlloc(void **p, size_t bytes, unsigned /*flags*/) { return gp_host_alloc(p, bytes); }
inline GPUresult GPUMemFreeHost(void *p) { return gp_host_free(p); }
inline GPUresult GPUMemcpyHtoD(GPUdeviceptr d, const void *h, size_t n) { return gp_memcpy_h2d(d, h, n); }
inline GPUresult GPUMemcpyDtoH(void *h, GPUdeviceptr d, size_t n) { return gp_memcpy_d2h(h, d, n); }
inline GPUresult GPUMemcpyHtoDAsync(GPUdeviceptr d, const void *h, size_t n, GPUstream s) { return gp_memcpy_h2d_async(d, h, n, s); }
inline GPUresult GPUMemcpyDtoHAsync(void *h, GPUdeviceptr d, size_t n, GPUstream s) { return gp_memcpy_d2h_async(h, d, n, s); }
inline GPUresult GPUMemcpyDtoDAsync(GPUdeviceptr d, GPUdeviceptr s_, size_t n, GPUstream s) { return gp_memcpy_d2d_async(d, s_, n, s); }
#define CU_MEMHOSTALLOC_PORTABLE 0u

// exit on failure (reference gpu_util.h:143-151)
#define ASSERT_CUDA_ERROR(cmd)                                                                  \
    do {                                                                                        \
        GPUresult gp_e_ = (cmd);                                                                \
        if (gp_e_ != GPU_SUCCESS) {                                                             \
            std::fprintf(stderr, "GPU error %d: %s at %s:%d\n", gp_e_, gp_last_error(), __FILE__, __LINE__); \
            std::exit(EXIT_FAILURE);                                                            \
        }                                                                                       \
    } while (0)

// print and return Status::Fail (reference gpu_util.h:153-162)
#define CUDA_RETURN_STATUS(cmd)                                                                 \
    do {                                                                                        \
        GPUresult gp_e_ = (cmd);                                                                \
        if (gp_e_ != GPU_SUCCESS) {                                                             \
            std::cout << "GPU error: " << gp_e_ << " " << gp_last_error() << " at " << __FILE__ << ":" << __LINE__ << std::endl; \
            return Status::Fail;                                                                \
        }                                                                                       \
    } while (0)

namespace foo {
namespace util {

// Selects device 0 for the calling thread; idempotent, called once per client thread
// (reference src/util/gpu_util.cpp:14-25).
void init_cuda();

class SizedGPUBuffer {
public:
    explicit SizedGPUBuffer(size_t size);
    ~SizedGPUBuffer();
    SizedGPUBuffer(const SizedGPUBuffer &) = delete;
    SizedGPUBuffer &operator=(const SizedGPUBuffer &) = delete;
    GPUdeviceptr ptr() const { return ptr_; }
    size_t size() const { return size_; }
    void from_vector(std::vector<float> &vec);
    void to_vector(std::vector<float> &vec);

private:
    GPUdeviceptr ptr_ = nullptr;
    size_t size_ = 0;
};

}  // namespace util
}  // namespace foo
