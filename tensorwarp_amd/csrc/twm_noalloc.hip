// twm_gemm_tw_marlin_m1_noalloc: the GEMV on the reference's arrays for callers that cannot allocate (code under
// HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It needs no context: the split-K
// scratch that twm_gemm_tw_marlin_m1 takes from its context lives here in a file-scope device array, one copy per
// GPU, held until the process ends.  The call allocates nothing and frees nothing.
#include "../../include/twmarlin.h"
#include "twm_internal.h"

#include <mutex>

using namespace twm;

namespace {

// f32 partial sums followed by the arrival counters.  The default plan splits K only on matrices of at most 64
// sub-tiles of 16 columns (N <= 1024) and never into more ranges than bring the workgroups to 256, so splits x padded
// N <= 4096 floats and at most 64 counters are ever used, whatever the shape; a split that would not fit is reduced.
constexpr size_t kPartialBytes = 64u << 10;
constexpr uint32_t kCounters = 256;
// the largest shape the entry point takes
constexpr uint32_t kMaxN = 1u << 20, kMaxK = 1u << 20;

}  // namespace

// (No `used` attribute here: the compiler gives a static device variable that host code names a global symbol in the
// code object, which is what hipGetSymbolAddress looks up; with the attribute the symbol stays local and the lookup
// aborts inside the runtime.)
static __device__ __align__(256) unsigned char scratch[kPartialBytes + kCounters * sizeof(unsigned)];

namespace {

// In host code the array's name is a stand-in, not a device address; each GPU holds its own copy at its own
// address, which hipGetSymbolAddress returns with that GPU current.
constexpr int kMaxDevices = 64;
void *g_scratch_ptr[kMaxDevices];
std::mutex g_scratch_mutex;

}  // namespace

// Device address of `scratch` on the current device, looked up once per device; nullptr with the error text set.
void *twm::noalloc_scratch_for_current_device(const char *who)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        api_fail(TWM_DEVICE_ERROR, "%s: no current HIP device (%s)", who,
                 e != hipSuccess ? hipGetErrorString(e) : "ordinal out of range");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            api_fail(TWM_DEVICE_ERROR, "%s: hipGetSymbolAddress(scratch) on device %d: %s", who, dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}

extern "C" int twm_gemm_tw_marlin_m1_noalloc(void *hip_stream, const float *a_dev, const uint8_t *packed_dev,
                                             const uint16_t *scales_dev, float *c_dev, uint32_t n, uint32_t k)
{
    const char *who = "twm_gemm_tw_marlin_m1_noalloc";
    if (int rc = check_kn(who, k, n)) return rc;
    if (n > kMaxN) return api_fail(TWM_SHAPE_ERROR, "%s: N = %u is beyond the %u columns this entry point takes", who, n, kMaxN);
    if (k > kMaxK) return api_fail(TWM_SHAPE_ERROR, "%s: K = %u is beyond the depth of %u this entry point takes", who, k, kMaxK);
    unsigned char *base = (unsigned char *)noalloc_scratch_for_current_device(who);
    if (!base) return TWM_DEVICE_ERROR;
    // the default plan of twm_gemm_tw_marlin_m1 (no context, hence no options); the counters a split launch uses are
    // cleared first by a fill kernel, because the array keeps whatever the last call on this GPU left in it
    const M1Env env = {(hipStream_t)hip_stream, 0, 0, 0, 0, (float *)base, kPartialBytes,
                       (unsigned *)(base + kPartialBytes), kCounters, true};
    return m1_dispatch(env, who, a_dev, packed_dev, scales_dev, c_dev, n, k);
}

// Testing aid: every byte of the current GPU's scratch (partial sums and counters) set to `value` on hip_stream, so
// that a test can show that a call does not depend on what earlier calls left there.  Not for capture (a memset node).
extern "C" int twm_noalloc_scratch_fill(void *hip_stream, int value)
{
    const char *who = "twm_noalloc_scratch_fill";
    unsigned char *base = (unsigned char *)noalloc_scratch_for_current_device(who);
    if (!base) return TWM_DEVICE_ERROR;
    hipError_t e = hipMemsetAsync(base, value & 0xFF, sizeof scratch, (hipStream_t)hip_stream);
    if (e != hipSuccess) return api_fail(TWM_DEVICE_ERROR, "%s: %s", who, hipGetErrorString(e));
    return TWM_OK;
}
