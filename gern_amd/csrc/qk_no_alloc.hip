// gern_qk_softmax_run_no_alloc (include/gern_pipelines.h): gern_qk_softmax_run
// for callers that may not allocate device memory.  The memory through which
// the workgroups of the tile kernel exchange row statistics (gernels/qk_tiles.h)
// comes from a device array of this library instead of the pipeline's own
// allocation.  Every GPU holds its own copy of the array, at its own address,
// from the moment the array is first looked up (when the first tile-kernel
// pipeline is created on that GPU) until the process ends.
#include "gern_pipelines.h"

#include <hip/hip_runtime.h>

#include <mutex>
#include <string>

// csrc/pipelines.cpp (internal to the library)
extern "C" {
__attribute__((visibility("hidden"))) int gern_detail_qk_softmax_run(gern_pipeline p, const uint16_t *Q, const uint16_t *K, float *S,
                                                                     int64_t M, int64_t N, float scale, void *scratch, void *stream,
                                                                     const char *who);
__attribute__((visibility("hidden"))) int gern_detail_fail(const char *message);
__attribute__((visibility("hidden"))) void *gern_detail_qk_shared_of(gern_pipeline p);
}

namespace {

// State and entries of the exchange; zero when the code object is loaded,
// which is the state the exchange starts from, and left consistent by every
// launch (a launch tags what it writes with its own number and never relies
// on the contents left by another).
static __device__ __align__(256) unsigned char scratch[GERN_QK_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex lookup_mutex;
void *device_address[kMaxDevices];  // of `scratch`, per GPU; null until looked up

// The address of this GPU's copy of the array.  `scratch` itself is only a
// handle on the host: it names the symbol for hipGetSymbolAddress and is never
// passed anywhere else.
int scratchOfCurrentDevice(void **out) {
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) {
        return gern_detail_fail((std::string("gern_qk_softmax_run_no_alloc: hipGetDevice: ") + hipGetErrorString(err)).c_str());
    }
    if (device < 0 || device >= kMaxDevices) {
        return gern_detail_fail("gern_qk_softmax_run_no_alloc: device index out of range");
    }
    std::lock_guard<std::mutex> lock(lookup_mutex);
    if (device_address[device] == nullptr) {
        void *ptr = nullptr;
        err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess || ptr == nullptr) {
            return gern_detail_fail((std::string("gern_qk_softmax_run_no_alloc: hipGetSymbolAddress: ") + hipGetErrorString(err)).c_str());
        }
        device_address[device] = ptr;
    }
    *out = device_address[device];
    return 0;
}

}  // namespace

// For gern_qk_softmax_create (csrc/pipelines.cpp): set-up, once per GPU, with that GPU current.
extern "C" __attribute__((visibility("hidden"))) int gern_detail_qk_shared_scratch(void **out) {
    return scratchOfCurrentDevice(out);
}

// The run itself looks nothing up: the address was found when the pipeline was created.
extern "C" int gern_qk_softmax_run_no_alloc(gern_pipeline p, const uint16_t *Q, const uint16_t *K, float *S, int64_t M, int64_t N,
                                            float scale, void *stream) {
    void *ptr = gern_detail_qk_shared_of(p);
    if (ptr == nullptr) {
        return 1;
    }
    return gern_detail_qk_softmax_run(p, Q, K, S, M, N, scale, ptr, stream, "gern_qk_softmax_run_no_alloc");
}
