// xrt_linear_static: the matrix product of xrt_linear for callers that cannot allocate device memory.
//
// Products of 17 to 64 rows (and some wider ones with few tiles) are split along k: their tiles write
// float32 partial sums to a workspace and a second kernel adds them up. xrt_linear takes that workspace
// from its caller. Here it is a fixed array in device memory that the library itself holds, one copy on
// every GPU the library is used on, from the first call on that GPU until the process ends. The entry
// point calls no hipMalloc, hipFree or other allocating routine.
//
// All calls on one GPU share that GPU's array. Nothing in it has to start at zero: the tiles of a product
// write every partial sum that its second kernel reads, so what an earlier call left is never read. Two
// calls that overlap on one GPU (different streams) would write the same array at once and race: a caller
// keeps its calls on a GPU in one stream, or orders them itself.
#include <mutex>

#include "common.h"
#include "xrt_hip.h"

#define XRT_STATIC_MAX_DEVICES 64

static __device__ __align__(256) float scratch[XRT_LINEAR_STATIC_FLOATS];

// The address of `scratch` on each device. In host code the array's name is only a handle for
// hipGetSymbolAddress, not a device address; kernels get the pointer kept here.
static float* scratch_on_device[XRT_STATIC_MAX_DEVICES];
static std::mutex scratch_lock;

static int scratch_pointer(float** pointer) {
    int device = -1;
    hipError_t status = hipGetDevice(&device);
    XRT_REQUIRE(status == hipSuccess, "linear (static): no current device: %s", hipGetErrorString(status));
    XRT_REQUIRE(device >= 0 && device < XRT_STATIC_MAX_DEVICES, "linear (static): device %d is beyond the %d that are kept",
                device, XRT_STATIC_MAX_DEVICES);
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (scratch_on_device[device] == nullptr) {
        float* address = nullptr;
        status = hipGetSymbolAddress((void**)&address, HIP_SYMBOL(scratch));
        XRT_REQUIRE(status == hipSuccess && address != nullptr, "linear (static): the scratch array has no address on device %d: %s",
                    device, hipGetErrorString(status));
        scratch_on_device[device] = address;
    }
    *pointer = scratch_on_device[device];
    return 0;
}

extern "C" long xrt_linear_static_floats(void) { return (long)XRT_LINEAR_STATIC_FLOATS; }

extern "C" int xrt_linear_static(const void* a, const void* w, int dtype, void* out, int out_dtype, int M, int N,
                                 int K, int mode, void* stream) {
    XRT_REQUIRE(M >= 0 && N > 0 && K > 0, "linear (static): bad sizes M=%d N=%d K=%d", M, N, K);
    XRT_REQUIRE(mode >= 0 && mode <= 2, "linear (static): unknown mode %d", mode);
    XRT_REQUIRE(a && w && out, "linear (static): null operand");
    const long need = xrt_linear_workspace(a, w, dtype, M, N, K, mode);
    XRT_REQUIRE(need <= (long)XRT_LINEAR_STATIC_FLOATS,
                "linear (static): M=%d N=%d K=%d mode %d splits into %ld floats of partial sums, the fixed buffer holds %ld",
                M, N, K, mode, need, (long)XRT_LINEAR_STATIC_FLOATS);
    float* workspace = nullptr;
    if (need > 0 && scratch_pointer(&workspace) != 0) return 1;
    return xrt_linear(a, w, dtype, out, out_dtype, M, N, K, mode, workspace, need, stream);
}
