// Routed EXL3 experts in ONE launch for decode-sized calls (R <= 16 rows, R * topk <= 256 pairs).
//
// The multi-kernel path (moe_exl3.hip) needs seven dependent launches for a layer that moves 16 MB: launch gaps and the
// chain of cold first loads cost far more than the weight stream.  Here one grid holds both weight streams:
//   A blocks: (item, 128-column block of I | gate or up, K slice).  Transform the slice of x (x * suh, Hadamard, fp16)
//       into LDS, stream and decode the slice's k-tiles, write FP32 partials; the last block of an (item, column block)
//       group sums the slices, finishes gate and up (Hadamard, svh), applies the activation and the down input
//       transform and publishes that block of xh2; a per-item counter tells the B blocks when all of xh2 is there.
//   B blocks: (128-column block of H | item, K slice).  Issue and DECODE their down-projection tiles first (they do not
//       depend on stage 1), then wait for the item's counter, dot with xh2, finish (Hadamard, svh); the block that
//       completes a token row's last expert does the weighted slot-order sum for its 128 columns.
//
// XCD-aware placement.  MI355X has 8 XCDs with one L2 each, and workgroup b runs on XCD b % 8 (checked once per process
// by reading XCC_ID).  Block ids are laid out so that every exchange but one stays inside one XCD: the 2 * S1 blocks of
// an (item, column block) group share an XCD, and so do all B blocks of one output column block (their experts' outputs
// meet in the final sum).  Inside an XCD data moves through the shared L2 with ordinary stores, L1-bypassing loads and
// L2 atomics.  Only xh2 crosses XCDs, through device-coherent stores / loads (slow: they go to memory), once per item.
// If the placement check fails, every exchange uses the device-coherent form.
//
// Blocks are dispatched in id order and all A blocks precede all B blocks, so every A block is resident or done before a
// B block can start waiting; A blocks never wait.  Waits are bounded: on expiry the block sets an error flag and skips
// its work, and every block still runs to its end, so the grid always drains.  The last block to finish clears the
// counters for the next call.  A producer block waits until every wave's stores are acknowledged (s_waitcnt vmcnt(0),
// a workgroup fence does not wait for global stores), then one thread bumps the counter.
//
// Items are distinct experts in order of first appearance; rows of the per-pair buffers are the pair indices r * topk + k.
// Semantics: reference engine-rs/shim/moe_exl3.cuh:204-228,272-285,935-956,1019-1064,1084-1112,1380-1410.
#include "moe_exl3.hpp"
#include "exl3_decode.hpp"

namespace spk {
namespace {

long long* g_trace = nullptr;
#define TRACE(i) do { if (a.trace && tid == 0) a.trace[(int64_t)bid * 8 + (i)] = wall_clock64(); } while (0)

constexpr int FW = 4;                 // waves per block
constexpr int TW = 8;                 // k-tiles per wave (all loaded up front)
constexpr int KTB = FW * TW;          // k-tiles per block = K slice of 512
constexpr int PF_MAX = 256, RF_MAX = 16;
constexpr int SPIN_MAX = 400000;
constexpr int SMAX = 8;               // K slices per product (K <= 4096)
constexpr int NXCD = 8;

struct FArgs {
    const void* x; int64_t ldx; const void* idx; const void* w; const uint64_t* tab; const float* add; float* out;
    float* part1; uint16_t* xh2; float* part2; float* yd; int* cnt;
    int R, P, Gmax, S1, S2, NB1, NB2, nA, nB, ncnt, bpgA, bpgB, local;
    Exl3Cfg c;
    long long* trace;                 // optional per-block timestamps (diagnostics), 8 per block
};
// counter layout: [0] XCDs done, [1] error flag (sticky), [2..9] blocks done per XCD, then cnt1 [Gmax][NB1], ready [Gmax],
// cnt2 [Gmax][NB2], cnt3 [R][NB2]
__device__ __forceinline__ int* cnt1_of(const FArgs& a) { return a.cnt + 2 + NXCD; }
__device__ __forceinline__ int* ready_of(const FArgs& a) { return cnt1_of(a) + a.Gmax * a.NB1; }
__device__ __forceinline__ int* cnt2_of(const FArgs& a) { return ready_of(a) + a.Gmax; }
__device__ __forceinline__ int* cnt3_of(const FArgs& a) { return cnt2_of(a) + a.Gmax * a.NB2; }

// ---- device-coherent (cross-XCD) accesses
__device__ __forceinline__ int ld_acquire(const int* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint64_t ld_dev64(const void* p) { return __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_dev64(void* p, uint64_t v) { __hip_atomic_store((uint64_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint32_t ld_dev32(const void* p) { return __hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_dev32(void* p, uint32_t v) { __hip_atomic_store((uint32_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// ---- XCD-local accesses: an ordinary store reaches the XCD's L2 (the L1 is write-through); a load with sc0 misses the
// L1 and reads that L2.  Eight 8-byte loads are issued together and waited for once.
__device__ __forceinline__ void ld_l2x8(const void* const (&p)[8], uint64_t (&o)[8])
{
    asm volatile(
        "global_load_dwordx2 %0, %8, off sc0\n\tglobal_load_dwordx2 %1, %9, off sc0\n\tglobal_load_dwordx2 %2, %10, off sc0\n\t"
        "global_load_dwordx2 %3, %11, off sc0\n\tglobal_load_dwordx2 %4, %12, off sc0\n\tglobal_load_dwordx2 %5, %13, off sc0\n\t"
        "global_load_dwordx2 %6, %14, off sc0\n\tglobal_load_dwordx2 %7, %15, off sc0\n\ts_waitcnt vmcnt(0)"
        : "=&v"(o[0]), "=&v"(o[1]), "=&v"(o[2]), "=&v"(o[3]), "=&v"(o[4]), "=&v"(o[5]), "=&v"(o[6]), "=&v"(o[7])
        : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7])
        : "memory");
}
// up to 8 pairs of floats from 8 addresses (slots >= n repeat slot 0 and are ignored), XCD-local or device-coherent
__device__ __forceinline__ void gather8(bool local, const float* const (&p)[8], int n, float (&lo)[8], float (&hi)[8])
{
    uint64_t o[8];
    if (local) {
        const void* q[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = i < n ? p[i] : p[0];
        ld_l2x8(q, o);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = i < n ? ld_dev64(p[i]) : 0;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) { lo[i] = __uint_as_float((uint32_t)o[i]); hi[i] = __uint_as_float((uint32_t)(o[i] >> 32)); }
}
__device__ __forceinline__ void put2(bool local, float* p, float v0, float v1)
{
    const uint64_t u = (uint64_t)__float_as_uint(v0) | ((uint64_t)__float_as_uint(v1) << 32);
    if (local) *(uint64_t*)p = u; else st_dev64(p, u);
}
// all of this wave's stores have been acknowledged (then __syncthreads() covers the block)
__device__ __forceinline__ void stores_done() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// counter bump that publishes the block's data: one thread, after stores_done() + __syncthreads() of every wave
__device__ __forceinline__ int bump(bool local, int* p)
{
    return local ? __hip_atomic_fetch_add(p, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)     // executes in the XCD's L2
                 : __hip_atomic_fetch_add(p, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct Group { int e, n; };
// item g of the call: expert and its pair rows (ascending), or n = 0 when the call has fewer items.  All threads call.
__device__ __forceinline__ Group find_item(const FArgs& a, int g, int* sidx, unsigned char* isf, int* rows, int* misc)
{
    const int P = a.P, tid = threadIdx.x;
    if (a.R == 1) {                                       // every pair is its own item
        if (g >= P) return Group{0, 0};
        if (tid == 0) rows[0] = g;
        __syncthreads();
        return Group{exl3_ld_idx(a.idx, a.c.itype, g), 1};
    }
    if (tid == 0) { misc[0] = -1; misc[1] = 0; }
    for (int p = tid; p < P; p += blockDim.x) sidx[p] = exl3_ld_idx(a.idx, a.c.itype, p);
    __syncthreads();
    for (int p = tid; p < P; p += blockDim.x) {           // first occurrence of its expert?
        const int e = sidx[p];
        bool first = true;
        for (int q = 0; q < p; ++q) first &= sidx[q] != e;
        isf[p] = first;
    }
    __syncthreads();
    for (int p = tid; p < P; p += blockDim.x)
        if (isf[p]) {
            int before = 0;
            for (int q = 0; q < p; ++q) before += isf[q];
            if (before == g) misc[0] = sidx[p];
        }
    __syncthreads();
    const int e = misc[0];
    if (e < 0) return Group{0, 0};
    for (int p = tid; p < P; p += blockDim.x)
        if (sidx[p] == e) {
            int slot = 0;
            for (int q = 0; q < p; ++q) slot += sidx[q] == e;
            rows[slot] = p;
            atomicAdd(&misc[1], 1);
        }
    __syncthreads();
    return Group{e, misc[1]};
}

template <int CBK, int MR>
__global__ __launch_bounds__(64 * FW) void fused_kernel(const FArgs a)
{
    __shared__ __align__(16) uint16_t xs[MR][KTB * 16];   // this block's K slice of the transformed activations (fp16)
    __shared__ float red[FW][MR][128];
    __shared__ int sidx[PF_MAX], rows[RF_MAX], misc[4];
    __shared__ unsigned char isf[PF_MAX];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bid = blockIdx.x;
    const bool isA = bid < a.nA, local = a.local != 0;
    const Exl3Cfg& c = a.c;
    // ---- block id -> work.  Group q lives on XCD q % 8: bid = ((q / 8) * bpg + j) * 8 + q % 8, j = position in the group.
    int g = -1, t = 0, nb = 0, s = 0, K, N;
    {
        const int b = isA ? bid : bid - a.nA, xcd = b % NXCD, li = b / NXCD;
        if (isA) {
            const int j = li % a.bpgA, q = (li / a.bpgA) * NXCD + xcd;      // q = g * NB1 + nb1, j = t * S1 + s
            if (q < a.Gmax * a.NB1) { g = q / a.NB1; nb = q % a.NB1; t = j / a.S1; s = j % a.S1; }
            K = c.H; N = c.I;
        } else {
            const int j = li % a.bpgB, q = (li / a.bpgB) * NXCD + xcd;      // q = nb2, j = g * S2 + s
            if (q < a.NB2) { nb = q; g = j / a.S2; s = j % a.S2; }
            K = c.I; N = c.H;
        }
    }
    TRACE(0);
    Group grp{0, 0};
    if (g >= 0) grp = find_item(a, g, sidx, isf, rows, misc);
    TRACE(1);
    bool alive = grp.n > 0;
    if (alive) {
        const int Kt = K / 16, Nt = N / 16;
        const int kt0 = s * KTB, kt1 = min(Kt, kt0 + KTB), nkt = kt1 - kt0;
        const int nblk = (nkt + 7) / 8;                   // 128-blocks of K in this slice
        const uint32_t* tr = (const uint32_t*)a.tab[(int64_t)(isA ? t : 2) * c.E + grp.e];
        // ---- issue this wave's tile loads: k-tiles kt0 + wave + FW i
        uint4 wr[TW];
#pragma unroll
        for (int i = 0; i < TW; ++i) {
            const int kt = kt0 + wave + FW * i;
            wr[i] = make_uint4(0u, 0u, 0u, 0u);
            if (kt < kt1) wr[i] = ld_stream16(tr + ((int64_t)kt * Nt + nb * 8) * 32 + lane * 4);
        }
        TRACE(2);
        const int src = tile_prev_lane(lane);
        const int ncol = nb * 128 + 2 * lane;             // this lane's two columns in the finishing steps
        float acc[MR][2];
#pragma unroll
        for (int r = 0; r < MR; ++r) { acc[r][0] = 0.f; acc[r][1] = 0.f; }
        if (isA) {
            // ---- scales of the finishing step, fetched early (any block of the group may be its last)
            const uint16_t* suh = (const uint16_t*)a.tab[(int64_t)(3 + t) * c.E + grp.e];
            const uint16_t* svg = (const uint16_t*)a.tab[(int64_t)6 * c.E + grp.e];
            const uint16_t* svu = (const uint16_t*)a.tab[(int64_t)7 * c.E + grp.e];
            const uint16_t* sud = (const uint16_t*)a.tab[(int64_t)5 * c.E + grp.e];
            const float sg0 = f16_bits_to_f32(svg[ncol]), sg1 = f16_bits_to_f32(svg[ncol + 1]);
            const float su0 = f16_bits_to_f32(svu[ncol]), su1 = f16_bits_to_f32(svu[ncol + 1]);
            const float sd0 = f16_bits_to_f32(sud[ncol]), sd1 = f16_bits_to_f32(sud[ncol + 1]);
            // ---- transform the slice of x into LDS: wave per (row, 128-block)
            for (int u = wave; u < grp.n * nblk; u += FW) {
                const int r = u / nblk, kb = u % nblk;
                const int k = kt0 * 16 + kb * 128 + 2 * lane;
                const int64_t srow = rows[r] / c.topk;
                float v0 = exl3_ld_x(a.x, c.xtype, srow * a.ldx + k) * f16_bits_to_f32(suh[k]);
                float v1 = exl3_ld_x(a.x, c.xtype, srow * a.ldx + k + 1) * f16_bits_to_f32(suh[k + 1]);
                fwht128(v0, v1, lane);
                *(uint32_t*)&xs[r][kb * 128 + 2 * lane] = (uint32_t)f32_to_f16_bits(v0) | ((uint32_t)f32_to_f16_bits(v1) << 16);
            }
            __syncthreads();
            TRACE(3);
#pragma unroll
            for (int i = 0; i < TW; ++i) {
                const int kt = kt0 + wave + FW * i;
                if (kt < kt1) {
                    h2 wd[4][4];
                    decode_tile32<CBK>(wr[i], __shfl(wr[i].w, src, 64), wd);
#pragma unroll
                    for (int r = 0; r < MR; ++r) {
                        if (r >= grp.n) break;
                        dot_tile32(wd, (const uint32_t*)&xs[r][(kt - kt0) * 16], acc[r][0], acc[r][1]);
                    }
                }
            }
            TRACE(5);
            // ---- sum the waves in wave order, publish the partial of this (matrix, K slice) inside the XCD
            const int j = lane >> 3, m = lane & 7;
#pragma unroll
            for (int r = 0; r < MR; ++r) { red[wave][r][16 * j + m] = acc[r][0]; red[wave][r][16 * j + m + 8] = acc[r][1]; }
            __syncthreads();
            float* part = a.part1 + ((int64_t)(s * 2 + t) * a.P) * N;
            for (int i = tid; i < grp.n * 64; i += 64 * FW) {
                const int r = i >> 6, col = (i & 63) * 2;
                float v0 = red[0][r][col], v1 = red[0][r][col + 1];
#pragma unroll
                for (int w = 1; w < FW; ++w) { v0 += red[w][r][col]; v1 += red[w][r][col + 1]; }
                put2(local, &part[(int64_t)rows[r] * N + nb * 128 + col], v0, v1);
            }
            stores_done();
            __syncthreads();
            if (tid == 0) misc[3] = bump(local, cnt1_of(a) + g * a.NB1 + nb) == 2 * a.S1 - 1;
            __syncthreads();
            TRACE(6);
            if (misc[3]) {
                // ---- last block of the group: finish gate and up, activation, down input transform -> xh2 (device-coherent)
                for (int r = wave; r < grp.n; r += FW) {
                    float gl[8], gh[8], ul[8], uh[8];
                    const float* pg[8]; const float* pu[8];
#pragma unroll
                    for (int ss = 0; ss < 8; ++ss) {
                        const int s2 = ss < a.S1 ? ss : 0;
                        pg[ss] = a.part1 + ((int64_t)(s2 * 2 + 0) * a.P + rows[r]) * c.I + ncol;
                        pu[ss] = a.part1 + ((int64_t)(s2 * 2 + 1) * a.P + rows[r]) * c.I + ncol;
                    }
                    gather8(local, pg, a.S1, gl, gh);
                    gather8(local, pu, a.S1, ul, uh);
                    float g0 = 0.f, g1 = 0.f, u0 = 0.f, u1 = 0.f;
#pragma unroll
                    for (int ss = 0; ss < 8; ++ss) if (ss < a.S1) { g0 += gl[ss]; g1 += gh[ss]; u0 += ul[ss]; u1 += uh[ss]; }
                    fwht128(g0, g1, lane);
                    fwht128(u0, u1, lane);
                    float v0 = exl3_act(c.act, g0 * sg0, u0 * su0) * sd0;
                    float v1 = exl3_act(c.act, g1 * sg1, u1 * su1) * sd1;
                    fwht128(v0, v1, lane);
                    st_dev32(a.xh2 + (int64_t)rows[r] * c.I + ncol, (uint32_t)f32_to_f16_bits(v0) | ((uint32_t)f32_to_f16_bits(v1) << 16));
                }
                stores_done();
                __syncthreads();
                if (tid == 0) bump(false, ready_of(a) + g);
            }
        } else {
            // ---- decode first and fetch the finishing scales (independent of stage 1), then wait for the item's xh2
            h2 wd[TW][4][4];
#pragma unroll
            for (int i = 0; i < TW; ++i) decode_tile32<CBK>(wr[i], __shfl(wr[i].w, src, 64), wd[i]);
            const uint16_t* svd = (const uint16_t*)a.tab[(int64_t)8 * c.E + grp.e];
            const float svd0 = f16_bits_to_f32(svd[ncol]), svd1 = f16_bits_to_f32(svd[ncol + 1]);
            asm volatile("" :: "v"(svd0), "v"(svd1));
            TRACE(3);
            if (tid == 0) {
                const int* rdy = ready_of(a) + g;
                int spins = 0;
                while (ld_acquire(rdy) < a.NB1 && spins < SPIN_MAX) { __builtin_amdgcn_s_sleep(2); ++spins; }
                misc[2] = spins < SPIN_MAX;
                if (spins >= SPIN_MAX) atomicExch(&a.cnt[1], 1);
            }
            __syncthreads();
            TRACE(4);
            alive = misc[2] != 0;
            if (alive) {
                for (int u = tid; u < grp.n * (nkt * 8); u += 64 * FW) {      // 2 fp16 per thread-step
                    const int r = u / (nkt * 8), q = u % (nkt * 8);
                    *(uint32_t*)&xs[r][q * 2] = ld_dev32((const uint32_t*)(a.xh2 + (int64_t)rows[r] * c.I + kt0 * 16) + q);
                }
                __syncthreads();
#pragma unroll
                for (int i = 0; i < TW; ++i) {
                    const int kt = kt0 + wave + FW * i;
                    if (kt < kt1) {
#pragma unroll
                        for (int r = 0; r < MR; ++r) {
                            if (r >= grp.n) break;
                            dot_tile32(wd[i], (const uint32_t*)&xs[r][(kt - kt0) * 16], acc[r][0], acc[r][1]);
                        }
                    }
                }
                TRACE(5);
                const int j = lane >> 3, m = lane & 7;
#pragma unroll
                for (int r = 0; r < MR; ++r) { red[wave][r][16 * j + m] = acc[r][0]; red[wave][r][16 * j + m + 8] = acc[r][1]; }
                __syncthreads();
                bool last = true;
                if (a.S2 > 1) {
                    float* part = a.part2 + ((int64_t)s * a.P) * N;
                    for (int i = tid; i < grp.n * 64; i += 64 * FW) {
                        const int r = i >> 6, col = (i & 63) * 2;
                        float v0 = red[0][r][col], v1 = red[0][r][col + 1];
#pragma unroll
                        for (int w = 1; w < FW; ++w) { v0 += red[w][r][col]; v1 += red[w][r][col + 1]; }
                        put2(local, &part[(int64_t)rows[r] * N + nb * 128 + col], v0, v1);
                    }
                    stores_done();
                    __syncthreads();
                    if (tid == 0) misc[3] = bump(local, cnt2_of(a) + g * a.NB2 + nb) == a.S2 - 1;
                    __syncthreads();
                    last = misc[3] != 0;
                }
                TRACE(6);
                if (last) {
                    // ---- finish the down product: yd[pair] = had128(sum of slices) * svh; wave per row
                    for (int r = wave; r < grp.n; r += FW) {
                        float v0 = 0.f, v1 = 0.f;
                        if (a.S2 > 1) {
                            float pl[8], ph[8];
                            const float* pp[8];
#pragma unroll
                            for (int ss = 0; ss < 8; ++ss) pp[ss] = a.part2 + ((int64_t)(ss < a.S2 ? ss : 0) * a.P + rows[r]) * c.H + ncol;
                            gather8(local, pp, a.S2, pl, ph);
#pragma unroll
                            for (int ss = 0; ss < 8; ++ss) if (ss < a.S2) { v0 += pl[ss]; v1 += ph[ss]; }
                        } else {
#pragma unroll
                            for (int w = 0; w < FW; ++w) { v0 += red[w][r][2 * lane]; v1 += red[w][r][2 * lane + 1]; }
                        }
                        fwht128(v0, v1, lane);
                        put2(local, a.yd + (int64_t)rows[r] * c.H + ncol, v0 * svd0, v1 * svd1);
                    }
                    stores_done();
                    __syncthreads();
                    // ---- rows whose last expert just arrived: weighted slot-order sum of this column block
                    if (tid < grp.n) {
                        const int r = rows[tid] / c.topk;
                        sidx[tid] = bump(local, cnt3_of(a) + r * a.NB2 + nb) == c.topk - 1 ? r : -1;
                    }
                    __syncthreads();
                    for (int i = wave; i < grp.n; i += FW) {
                        const int r = sidx[i];
                        if (r < 0) continue;
                        float a0 = 0.f, a1 = 0.f;
                        for (int k0 = 0; k0 < c.topk; k0 += 8) {                // 8 experts' outputs requested together
                            float yl[8], yh[8];
                            const float* py[8];
                            const int nk = min(8, c.topk - k0);
#pragma unroll
                            for (int k = 0; k < 8; ++k) py[k] = a.yd + (int64_t)(r * c.topk + k0 + (k < nk ? k : 0)) * c.H + ncol;
                            gather8(local, py, nk, yl, yh);
#pragma unroll
                            for (int k = 0; k < 8; ++k)
                                if (k < nk) {
                                    const float wk = exl3_ld_w(a.w, c.wtype, r * c.topk + k0 + k);
                                    a0 += wk * yl[k]; a1 += wk * yh[k];
                                }
                        }
                        const float b0 = a.add ? a.add[(int64_t)r * c.H + ncol] : 0.f, b1 = a.add ? a.add[(int64_t)r * c.H + ncol + 1] : 0.f;
                        a.out[(int64_t)r * c.H + ncol] = b0 + a0;
                        a.out[(int64_t)r * c.H + ncol + 1] = b1 + a1;
                    }
                }
            }
        }
    }
    // ---- every block ends here: the last block of an XCD reports to the device-wide counter, the last of those clears
    // the counters for the next call (nothing else is running then)
    __syncthreads();
    TRACE(7);
    if (tid == 0) {
        const int xcd = bid % NXCD, mine = ((int)gridDim.x - xcd + NXCD - 1) / NXCD;   // blocks with this id % 8
        bool fin = false;
        if (bump(local, a.cnt + 2 + xcd) == mine - 1) fin = bump(false, a.cnt) == NXCD - 1;
        misc[0] = fin;
    }
    __syncthreads();
    if (misc[0]) {
        for (int i = tid; i < a.ncnt; i += 64 * FW) if (i != 1) a.cnt[i] = 0;
    }
}

__global__ void zero_kernel(int* p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}
// the XCD a workgroup runs on (XCC_ID, hardware register 20)
__global__ void xcd_probe_kernel(int* out)
{
    if (threadIdx.x == 0) out[blockIdx.x] = __builtin_amdgcn_s_getreg((31 << 11) | 20) & 0xf;
}

struct FPlan { int P, Gmax, S1, S2, NB1, NB2, nA, nB, ncnt, bpgA, bpgB; size_t cnt, part1, xh2, part2, yd, total; };
FPlan fplan(const Exl3Cfg& c, int R)
{
    FPlan p;
    p.P = R * c.topk;
    p.Gmax = p.P < c.E ? p.P : c.E;
    p.S1 = (c.H / 16 + KTB - 1) / KTB;
    p.S2 = (c.I / 16 + KTB - 1) / KTB;
    p.NB1 = c.I / 128; p.NB2 = c.H / 128;
    p.bpgA = 2 * p.S1; p.bpgB = p.Gmax * p.S2;
    const int QA = (p.Gmax * p.NB1 + NXCD - 1) / NXCD * NXCD, QB = (p.NB2 + NXCD - 1) / NXCD * NXCD;   // groups, padded to the XCD count
    p.nA = QA * p.bpgA;
    p.nB = QB * p.bpgB;
    p.ncnt = 2 + NXCD + p.Gmax * p.NB1 + p.Gmax + p.Gmax * p.NB2 + R * p.NB2;
    size_t o = 0;
    auto take = [&](size_t n) { const size_t q = o; o += align256(n); return q; };
    p.cnt = take(4 * (size_t)p.ncnt);
    p.part1 = take(4 * (size_t)p.S1 * 2 * p.P * c.I);
    p.xh2 = take(2 * (size_t)p.P * c.I);
    p.part2 = take(4 * (size_t)p.S2 * p.P * c.H);
    p.yd = take(4 * (size_t)p.P * c.H);
    p.total = o;
    return p;
}

template <int CBK>
void launch(const FArgs& a, int maxrows, hipStream_t st)
{
    const dim3 grid(a.nA + a.nB), blk(64 * FW);
    if (maxrows <= 1) fused_kernel<CBK, 1><<<grid, blk, 0, st>>>(a);
    else if (maxrows <= 2) fused_kernel<CBK, 2><<<grid, blk, 0, st>>>(a);
    else if (maxrows <= 4) fused_kernel<CBK, 4><<<grid, blk, 0, st>>>(a);
    else if (maxrows <= 8) fused_kernel<CBK, 8><<<grid, blk, 0, st>>>(a);
    else fused_kernel<CBK, 16><<<grid, blk, 0, st>>>(a);
}

int g_xcd_local = -1;                 // -1 unknown, 0 placement check failed, 1 workgroup b runs on XCD b % 8

}  // namespace

bool exl3_fused_ok(const Exl3Cfg& c, int R)
{
    return R >= 1 && R <= RF_MAX && R * c.topk <= PF_MAX && c.H <= SMAX * KTB * 16 && c.I <= SMAX * KTB * 16;
}
size_t exl3_fused_ws_bytes(const Exl3Cfg& c, int R) { return fplan(c, R).total; }

// Checks once per process that workgroup b of a 1-D grid runs on XCD b % 8 (synchronises: call outside stream capture,
// e.g. from the workspace initialisation).  Until it has run, the single-launch path uses device-coherent exchanges only.
int exl3_xcd_probe()
{
    if (g_xcd_local >= 0) return g_xcd_local;
    constexpr int NB = 1024;
    int* d = nullptr;
    if (hipMalloc(&d, NB * sizeof(int)) != hipSuccess) return g_xcd_local = 0;
    xcd_probe_kernel<<<NB, 64>>>(d);
    int h[NB];
    const bool copied = hipMemcpy(h, d, sizeof(h), hipMemcpyDeviceToHost) == hipSuccess;
    (void)hipFree(d);
    bool ok = copied;
    for (int i = 0; ok && i < NB; ++i) ok = h[i] == h[i % NXCD];
    for (int i = 0; ok && i < NXCD; ++i)
        for (int j = 0; j < i; ++j) ok = ok && h[i] != h[j];
    return g_xcd_local = ok ? 1 : 0;
}

int exl3_fused_launch(const Exl3Cfg& c, const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out, void* ws,
                      int clean, hipStream_t st)
{
    const FPlan p = fplan(c, R);
    char* b = (char*)ws;
    FArgs a;
    a.x = x; a.ldx = ldx; a.idx = idx; a.w = w; a.tab = (const uint64_t*)tab; a.add = (const float*)add; a.out = (float*)out;
    a.cnt = (int*)(b + p.cnt); a.part1 = (float*)(b + p.part1); a.xh2 = (uint16_t*)(b + p.xh2); a.part2 = (float*)(b + p.part2); a.yd = (float*)(b + p.yd);
    a.R = R; a.P = p.P; a.Gmax = p.Gmax; a.S1 = p.S1; a.S2 = p.S2; a.NB1 = p.NB1; a.NB2 = p.NB2; a.nA = p.nA; a.nB = p.nB; a.ncnt = p.ncnt;
    a.bpgA = p.bpgA; a.bpgB = p.bpgB;
    a.local = g_xcd_local == 1;
    a.c = c;
    a.trace = g_trace;
    if (!clean) zero_kernel<<<(p.ncnt + 255) / 256, 256, 0, st>>>(a.cnt, p.ncnt);
    if (c.cbk == CB_MCG) launch<CB_MCG>(a, R, st);
    else launch<CB_MUL1>(a, R, st);
    return launch_status();
}

// diagnostics: device buffer of 8 timestamps (100 MHz) per block of the next launches, or null
extern "C" __attribute__((visibility("default"))) void spark_debug_exl3_trace(long long* buf) { g_trace = buf; }
// diagnostics: force the exchange mode of the single-launch path (1 XCD-local, 0 device-coherent, -1 probe again)
extern "C" __attribute__((visibility("default"))) void spark_debug_exl3_local(int v) { g_xcd_local = v; }

}  // namespace spk
