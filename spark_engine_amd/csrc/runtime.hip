// Host-side state shared by the single-launch expert kernels: the one-time workgroup placement check, the table of workspaces
// their owner has prepared, and the read-out of a workspace's bounded-wait flag.
#include "runtime.hpp"

#include <atomic>
#include <cstdlib>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace spk {
namespace {

constexpr int NXCD = 8, PROBE_BLOCKS = 1024;
// where the placement check leaves each workgroup's XCC_ID: library memory, so the check allocates nothing
__device__ int g_probe[PROBE_BLOCKS];

// the XCD a workgroup runs on (XCC_ID, hardware register 20)
__global__ void xcd_probe_kernel(int* out)
{
    if (threadIdx.x == 0) out[blockIdx.x] = __builtin_amdgcn_s_getreg((31 << 11) | 20) & 0xf;
}

std::atomic<int> g_placement{-1};      // -1 not checked yet, 0 check failed, 1 workgroup b of a 1-D grid runs on XCD b % 8.  One value for the
                                       // process: the property belongs to the GPU model and the runtime, and every GPU of a node is the same model
std::mutex g_mu, g_probe_mu;
std::unordered_map<const void*, size_t> g_prepared;       // workspace base -> bytes its owner prepared

}  // namespace

// Checks once per process that workgroup b of a 1-D grid runs on XCD b % 8 (eight distinct XCDs).  Synchronises the device: call
// it outside stream capture (the workspace initialisation does).  Until it has run the single-launch kernels exchange through
// device-coherent accesses only.
int xcd_placement_check()
{
    if (g_placement >= 0) return g_placement;
    std::lock_guard<std::mutex> lk(g_probe_mu);            // two host threads: one runs the check, the other finds its result
    if (g_placement >= 0) return g_placement;
    int* d = nullptr;
    if (hipGetSymbolAddress((void**)&d, HIP_SYMBOL(g_probe)) != hipSuccess) return g_placement = 0;
    xcd_probe_kernel<<<PROBE_BLOCKS, 64>>>(d);
    int h[PROBE_BLOCKS];
    bool ok = hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost) == hipSuccess;
    for (int i = 0; ok && i < PROBE_BLOCKS; ++i) ok = h[i] == h[i % NXCD];
    for (int i = 0; ok && i < NXCD; ++i)
        for (int j = 0; j < i; ++j) ok = ok && h[i] != h[j];
    return g_placement = ok ? 1 : 0;
}
int xcd_placement() { return g_placement; }
void xcd_placement_reset() { g_placement = -1; }

void ws_note_prepared(const void* ws, size_t bytes)
{
    std::lock_guard<std::mutex> lk(g_mu);
    g_prepared[ws] = bytes;
}
bool ws_is_prepared(const void* ws, size_t need)
{
    std::lock_guard<std::mutex> lk(g_mu);
    const auto it = g_prepared.find(ws);
    return it != g_prepared.end() && it->second >= need;
}
void ws_forget(const void* ws)
{
    std::lock_guard<std::mutex> lk(g_mu);
    g_prepared.erase(ws);
}

namespace {
int g_validate = -1;                   // -1 = not decided yet (the environment decides at the first call), 0 off, 1 on
}
bool routes_checked()
{
    if (g_validate < 0) {
        const char* e = std::getenv("SPARK_VALIDATE_ROUTES");
        g_validate = e && e[0] == '1' ? 1 : 0;
    }
    return g_validate == 1;
}
int routes_check(const void* idx, bool idx64, int R, int topk, int E, hipStream_t st)
{
    if (!routes_checked()) return 0;
    if (!idx || R < 1 || topk < 1 || E < 1) return 1;
    if (hipStreamSynchronize(st) != hipSuccess) return -2;
    const size_t n = (size_t)R * topk;
    std::vector<long long> v(n);
    if (idx64) {
        if (hipMemcpy(v.data(), idx, n * 8, hipMemcpyDeviceToHost) != hipSuccess) return -3;
    } else {
        std::vector<int> t(n);
        if (hipMemcpy(t.data(), idx, n * 4, hipMemcpyDeviceToHost) != hipSuccess) return -3;
        for (size_t i = 0; i < n; ++i) v[i] = t[i];
    }
    for (int r = 0; r < R; ++r)
        for (int k = 0; k < topk; ++k) {
            const long long e = v[(size_t)r * topk + k];
            if (e < 0 || e >= E) return 1;
            for (int j = 0; j < k; ++j)
                if (v[(size_t)r * topk + j] == e) return 1;
        }
    return 0;
}

}  // namespace spk

// ---- the stream floor: what this GPU needs to READ a number of bytes with nothing else to do.  Non-temporal 16-byte loads, eight in
// flight a thread, over exactly `bytes` (rounded down to 16), one 4-byte store a wave: the time no kernel that must fetch those bytes
// from memory can beat, measured the way the layer kernels are (the benchmark records it into the same graph of instances).  The
// shape - 512 workgroups of 1024 threads walking the bytes with the grid's stride, all resident at once - is the fastest of the
// shapes tried at 2 MB .. 326 MB (15.9 MB: 4.0 us against 6.1 for 256-thread workgroups that read eight pieces a thread and end).
namespace spk {
namespace {
constexpr int SR_THREADS = 1024, SR_BLOCKS = 512;
__global__ __launch_bounds__(SR_THREADS) void stream_read_kernel(const uint4* __restrict__ p, int64_t n16, uint32_t* __restrict__ out)
{
    const int64_t stride = (int64_t)gridDim.x * SR_THREADS;
    int64_t i = (int64_t)blockIdx.x * SR_THREADS + threadIdx.x;
    uint32_t acc = 0u;
    for (; i + 7 * stride < n16; i += 8 * stride) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = ld_stream16(p + i + u * stride);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < n16; i += stride) { const uint4 v = ld_stream16(p + i); acc ^= v.x ^ v.y ^ v.z ^ v.w; }
    acc ^= __float_as_uint(lane_xor<32>(__uint_as_float(acc), threadIdx.x & 63));
    if ((threadIdx.x & 63) == 0) out[(blockIdx.x * (SR_THREADS / 64) + (threadIdx.x >> 6)) & 1023] = acc;
}
}  // namespace
}  // namespace spk
// src: device memory of `bytes` bytes (16-byte aligned), out: device memory of 4096 bytes
SPARK_API int spark_debug_stream_read(const void* src, size_t bytes, void* out, hipStream_t st)
{
    if (!src || !out || bytes < 16 || ((uintptr_t)src & 15)) return 1;
    spk::stream_read_kernel<<<spk::SR_BLOCKS, spk::SR_THREADS, 0, st>>>((const uint4*)src, (int64_t)(bytes / 16), (uint32_t*)out);
    return spk::launch_status();
}

// diagnostics: 1 = check every call's routes on the host before launching (see routes_check), 0 = off, negative = as the environment says
SPARK_API void spark_debug_validate_routes(int on) { spk::g_validate = on < 0 ? -1 : on ? 1 : 0; }

// The bounded-wait flag of a single-launch workspace (its first word): waits for the stream's work, then 0 = every wait of every call
// so far was served, 1 = a wait expired (the call that hit it stored nothing for the rows concerned and the workspace holds stale
// words: prepare it again before the next call), negative = the read failed.  Synchronises: a diagnostic, never on a captured stream.
SPARK_API int spark_moe_ws_status(const void* ws, hipStream_t st)
{
    if (!ws) return -1;
    if (hipStreamSynchronize(st) != hipSuccess) return -2;
    int flag = 0;
    if (hipMemcpy(&flag, ws, sizeof(flag), hipMemcpyDeviceToHost) != hipSuccess) return -3;
    if (flag != 0) spk::ws_forget(ws);                     // no longer known as prepared: the next call that may prepare it does so itself
    return flag != 0 ? 1 : 0;
}
// The owner of a prepared workspace is about to free it (or hand it to other code): calls through the reference-named entry points
// with this pointer prepare it again themselves from now on.
SPARK_API void spark_moe_ws_release(const void* ws) { spk::ws_forget(ws); }
// diagnostics: what the placement check found (1 = workgroup b of a 1-D grid runs on XCD b % 8, 0 = it does not, -1 = not checked yet)
SPARK_API int spark_debug_placement(void) { return spk::xcd_placement(); }
