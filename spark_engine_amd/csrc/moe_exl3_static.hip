// spark_exl3_moe without a workspace argument: the exchange words of the single-launch kernel live in an array of the library's
// own, so the call allocates nothing and the caller passes inputs and outputs only.
#include "moe_exl3.hpp"
#include "runtime.hpp"
#include "exl3_decode.hpp"
#include <atomic>

namespace spk {

namespace {
constexpr size_t SCRATCH_BYTES = (size_t)16 << 20;        // the largest single-launch call it takes (the 512-expert top-10 layer at 8 rows needs 5.3 MB)
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
std::atomic<void*> g_scratch_ptr[MAX_DEVICES] = {};       // per device: every GPU holds its own copy of the array at its own address (two
                                                          // host threads that set up the same device store the same address)
}  // namespace

// the array's device address on the current device, resolved once per device (the name `scratch` itself is a host-side stand-in)
int exl3_static_setup()
{
    int dev = -1;
    hipError_t rc = hipGetDevice(&dev);
    if (rc != hipSuccess) return (int)rc;
    if (dev < 0 || dev >= MAX_DEVICES) return -6;
    if (g_scratch_ptr[dev].load()) return 0;
    void* ptr = nullptr;
    rc = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (rc != hipSuccess) return (int)rc;
    if (!ptr) return -6;
    g_scratch_ptr[dev].store(ptr);
    return 0;
}

// spark_exl3_moe for callers that cannot allocate or pass a workspace (code under graph capture, serving loops, harnesses that
// forbid hipMalloc).  Same arguments without ws; decode sizes only (the single-launch path: at most 8 rows, uniform 4-bit table).
// Returns -5 when the shape is not one the single-launch path takes, -7 when its exchange words exceed the array (16 MiB).  Every
// call first puts the words it will use into their idle state with a fill kernel (no memset node: safe to capture), so nothing is
// assumed of what the last call left.  All calls on one GPU share the array: calls that overlap on one GPU (two streams) race.
extern "C" __attribute__((visibility("default"))) int spark_exl3_moe_static(const void* x, int xtype, int64_t ldx, int R, const void* idx, int itype, const void* w,
                                                                              int wtype, const void* tab, const void* add, void* out, int H, int I, int E, int topk,
                                                                              int codebook, int act, hipStream_t st)
{
    const Exl3Cfg c{E, topk, H, I, codebook, act, xtype, wtype, itype};
    if (R < 1 || E < 1 || topk < 1 || H < 128 || I < 128 || H % 128 || I % 128 || (ldx & 1) || (codebook != CB_MCG && codebook != CB_MUL1)) return -1;
    if (!exl3_fused_ok(c, R)) return -5;
    if (exl3_fused_ws_bytes(c, R) > SCRATCH_BYTES) return -7;
    if (const int v = routes_check(idx, itype != 0, R, topk, E, st)) return v > 0 ? -6 : -8;         // opt-in host check of the routes
    const int rs = exl3_static_setup();
    if (rs) return rs;
    int dev = 0;
    (void)hipGetDevice(&dev);
    return exl3_fused_launch(c, x, ldx, R, idx, w, tab, add, out, g_scratch_ptr[dev].load(), 0, st);
}

// The error flag of the library's own array after the last spark_exl3_moe_static call on the current device (every call clears it as
// it starts): waits for the stream, then 0 = every wait of that call was served, 1 = a wait expired or the routes broke the contract
// (the rows concerned hold NaN), negative = the array is not set up or the read failed.  Synchronises: never on a capturing stream.
extern "C" __attribute__((visibility("default"))) int spark_exl3_moe_static_status(hipStream_t st)
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES || !g_scratch_ptr[dev].load()) return -1;
    if (hipStreamSynchronize(st) != hipSuccess) return -2;
    int flag = 0;
    if (hipMemcpy(&flag, g_scratch_ptr[dev].load(), sizeof(flag), hipMemcpyDeviceToHost) != hipSuccess) return -3;
    return flag != 0 ? 1 : 0;
}

}  // namespace spk
