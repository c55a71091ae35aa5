// Routed EXL3 experts in ONE launch for decode-sized calls (R <= 8 rows, R * topk <= 128 pairs).
//
// The multi-kernel path (moe_exl3.hip) needs seven dependent launches for a layer that moves 16 MB: launch gaps and the
// chain of cold first loads cost far more than the weight stream.  Here one grid holds both weight streams:
//   A blocks: (item, 128-column block of I | gate or up, K slice).  Transform the slice of x (x * suh, Hadamard, fp16)
//       into LDS while the slice's k-tiles stream in, decode, dot, write FP32 partials.  The last block of an
//       (item, column block) group in launch order is its finisher: it takes the other blocks' partials, finishes gate
//       and up (Hadamard, svh), applies the activation and the down input transform and hands that block of xh2 to
//       every down-projection block of the item.
//   B blocks: (128-column block of H | item, K slice of 256).  Issue and DECODE their down-projection tiles first (they do not
//       depend on stage 1), then take the item's xh2, dot, and finish their own slice (the Hadamard transform is linear, so
//       every slice is transformed on its own): Hadamard, svh, the pair's route weight.
//   C blocks: (128-column block of H | token row).  They hold no weights: they wait for the topk * S2 finished slices of
//       their row and add them in (slot, slice) order, four waves a share each, then the waves' sums in wave order.
//
// Exchange without counters: every exchanged 32-bit word of the workspace is EMPTY (all ones) between uses.  A producer
// simply stores its value (a value that happens to be all ones, one particular NaN, is stored as another NaN); the one
// consumer of a word polls until it is no longer EMPTY, then stores EMPTY back.  No fence, no acknowledged-store wait and
// no atomic lies on the critical path: one store and one load per hop.  Every word has exactly one consumer (xh2 is
// written once per consuming column block for that reason), so the workspace is all EMPTY again when the kernel ends.
//
// XCD-aware placement.  MI355X has 8 XCDs with one L2 each, and workgroup b runs on XCD b % 8 (checked once per process
// by reading XCC_ID).  Block ids are laid out so that every exchange but one stays inside one XCD: the 2 * S1 blocks of
// an (item, column block) group share an XCD, and so do all B and C blocks of one output column block (their experts'
// outputs meet in the final sum).  Inside an XCD data moves through the shared L2 with ordinary stores and L1-bypassing loads.
// Only xh2 crosses XCDs, through device-coherent stores / loads.  If the placement check fails, every exchange uses the
// device-coherent form.
//
// Order.  Every A block comes before every B block: a B block that waits for its item must not hold a slot an A block could
// use (interleaving the two stages item by item was measured 17 % slower at one row and 46 % at four).
// Progress.  Blocks are dispatched in id order and a block only ever waits for blocks with lower ids (A before B before C,
// the finisher is the last block of its group), so whatever a block waits for is resident or done.  Waits are bounded: on expiry the block sets an error flag and skips its work, and every
// block still runs to its end, so the grid always drains (the workspace must then be initialised again).
//
// Items are distinct experts in order of first appearance; rows of the per-pair buffers are the pair indices r * topk + k.
// Semantics: reference engine-rs/shim/moe_exl3.cuh:204-228,272-285,935-956,1019-1064,1084-1112,1380-1410.
#include "moe_exl3.hpp"
#include "exl3_decode.hpp"
#include "runtime.hpp"
#include <type_traits>

namespace spk {
namespace {

long long* g_trace = nullptr;
#ifdef SPK_EXL3_TRACE
#define TRACE(i) do { if (a.trace && tid == 0) a.trace[(int64_t)bid * 16 + (i)] = wall_clock64(); } while (0)
#else
#define TRACE(i) do { } while (0)
#endif

constexpr int FW = 4;                 // waves per block
constexpr int TWB = 4;                // k-tiles per wave of a stage-2 block (all loaded and decoded up front): K slice of 256.  Eight would
                                      // spare the split of I = 512 in two slices but need 155 registers: three blocks per CU instead of four
constexpr int TWMAX = 8;              // most k-tiles per wave of a stage-1 block (4 or 8, chosen per shape)
constexpr int PF_MAX = 128, RF_MAX = 8;            // more rows go through the grouped GEMM (faster from 9 rows on)
constexpr int SPIN_MAX = 200000;
constexpr int EMAX_F = 1024;           // most experts of a layer on this path
constexpr int SMAX = 8;               // K slices per product (K <= 4096)
constexpr int NXCD = 8;
constexpr int HEAD = 256;             // bytes at the start of the workspace: [0] error flag (sticky)
constexpr uint32_t EMPTY = 0xffffffffu;
constexpr uint64_t EMPTY2 = ~0ull;

struct FArgs {
    const void* x; int64_t ldx; const void* idx; const void* w; const uint64_t* tab; const float* add; float* out;
    float* part1;                     // [S1][2][P][I] gate / up partial sums per K slice
    uint32_t* xh2;                    // [NB2][P][I / 2] packed fp16 pairs: one copy of the down input per consuming column block
    float* part2;                     // [S2][P][H] per pair and K slice of the down product: finished (Hadamard, svh) and weighted
    int* err;
    int R, P, Gmax, S1, VS, S2, NB1, NB2, nA, nB, nC, bpgA, bpgB, local;     // S1 / S2 = blocks along K of stage 1 / 2; VS = K slices of stage 1 (NH per block)
    Exl3Cfg c;
    long long* trace;                 // optional per-block timestamps (diagnostics), 8 per block
};

// ---- device-coherent (cross-XCD) accesses
__device__ __forceinline__ uint64_t ld_dev64(const void* p) { return __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_dev64(void* p, uint64_t v) { __hip_atomic_store((uint64_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint32_t ld_dev32(const void* p) { return __hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_dev32(void* p, uint32_t v) { __hip_atomic_store((uint32_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// ---- XCD-local accesses: an ordinary store reaches the XCD's L2 (the L1 is write-through).  An ordinary or sc0 load may be
// served from the CU's L1 once the line is there, so a consumer that polls with it spins on a stale line (measured); a
// non-temporal load is not kept in the L1 and reads the L2 every time (measured: 0.3 us from store to observation).
__device__ __forceinline__ uint64_t ld_l2(const float* p)
{
    return __builtin_nontemporal_load((const __attribute__((address_space(1))) uint64_t*)(uintptr_t)p);
}
__device__ __forceinline__ uint32_t fbits(float v) { const uint32_t u = __float_as_uint(v); return u == EMPTY ? 0x7fc00000u : u; }
// producer side: two adjacent words
template <bool local> __device__ __forceinline__ void put2(float* p, float v0, float v1)
{
    const uint64_t u = (uint64_t)fbits(v0) | ((uint64_t)fbits(v1) << 32);
    if (local) *(uint64_t*)p = u; else st_dev64(p, u);
}
// consumer side, whole wave: waits until the n (<= NMAX) word pairs at p[] all hold data, returns them and leaves the words
// EMPTY again (n >= 1).  Slots >= n are ignored.  All requests of a round are in flight together.  The outcome is the same for
// every lane; false = the wait expired.
template <bool local, int NMAX>
__device__ __forceinline__ bool take(float* const (&p)[NMAX], int n, float (&lo)[NMAX], float (&hi)[NMAX])
{
    uint64_t o[NMAX];
    int spins = 0;
    for (;;) {
        asm volatile("" ::: "memory");                     // the words change under us: load them again every round
#pragma unroll
        for (int i = 0; i < NMAX; ++i) o[i] = local ? ld_l2(p[i < n ? i : 0]) : ld_dev64(p[i < n ? i : 0]);   // straight-line: all in flight together
        bool ok = true;
#pragma unroll
        for (int i = 0; i < NMAX; ++i) ok = ok && o[i] != EMPTY2;
        if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
        if (++spins >= SPIN_MAX) return false;
        __builtin_amdgcn_s_sleep(1);
    }
#pragma unroll
    for (int i = 0; i < NMAX; ++i) {                       // slots >= n repeat slot 0: no branches
        if (local) *(uint64_t*)p[i < n ? i : 0] = EMPTY2; else st_dev64(p[i < n ? i : 0], EMPTY2);
    }
#pragma unroll
    for (int i = 0; i < NMAX; ++i) { lo[i] = __uint_as_float((uint32_t)o[i]); hi[i] = __uint_as_float((uint32_t)(o[i] >> 32)); }
    return true;
}
// the two activations k, k + 1 of a row (k even) as raw words: both loads are valid for every element type
__device__ __forceinline__ void ld_x2_raw(const void* x, int xtype, int64_t i, uint32_t& r0, uint32_t& r1)
{
    const char* b = (const char*)x + i * (xtype == X_F32 ? 4 : 2);
    r0 = *(const uint32_t*)b;
    r1 = *(const uint32_t*)(xtype == X_F32 ? b + 4 : b);
}
__device__ __forceinline__ void cvt_x2(int xtype, uint32_t r0, uint32_t r1, float& v0, float& v1)
{
    if (xtype == X_F32) { v0 = __uint_as_float(r0); v1 = __uint_as_float(r1); }
    else if (xtype == X_F16) { v0 = f16_bits_to_f32((uint16_t)r0); v1 = f16_bits_to_f32((uint16_t)(r0 >> 16)); }
    else { v0 = __uint_as_float(r0 << 16); v1 = __uint_as_float(r0 & 0xffff0000u); }
}

__device__ __forceinline__ int ld_idx_k(const void* idx, int itype, int i) { return itype ? (int)ld_k((const int64_t*)idx, i) : ld_k((const int*)idx, i); }

struct Group { int e, n; };
// item g of the call: expert and its pair rows (ascending) in rows[], or n = 0 when the call has fewer items.  All threads
// call; wave 0 works the item out (one barrier).
// cap: the rows this kernel instance's arrays hold per item (MR); an item beyond it is cut there and the error flag raised.
__device__ __forceinline__ Group find_item(const FArgs& a, int g, int* owner, int* rows, int* misc, int cap)
{
    const int P = a.P, tid = threadIdx.x;
    if (a.R == 1) {                                       // every pair is its own item
        if (g >= P) return Group{0, 0};
        const int e = clamp_expert(ld_idx_k(a.idx, a.c.itype, g), a.c.E);      // on its way while the block meets at the barrier
        if (tid == 0) rows[0] = g;
        __syncthreads();
        return Group{e, 1};
    }
    if (tid < 64) {
        WaveItems<PF_MAX / 64> wi;
        wave_items_init(wi, P, tid, owner, [&](int p) { return clamp_expert(exl3_ld_idx(a.idx, a.c.itype, p), a.c.E); });
        int n = 0;
        bool over;
        const int e = wave_items_pick(wi, g, tid, rows, n, cap, over);
        if (tid == 0) { misc[0] = e; misc[1] = n; if (over) atomicExch(a.err, 1); }
    }
    __syncthreads();
    return misc[0] < 0 ? Group{0, 0} : Group{__builtin_amdgcn_readfirstlane(misc[0]), __builtin_amdgcn_readfirstlane(misc[1])};
}

// MIXED: the kernel for tables with per-expert rows.  The experts' trellis widths (3..6 bits) come from row 9 of the table (reference
// moe_exl3.cuh:239-252); a block works on one expert, so the width is uniform over the block and selects one of four instances of the
// weight stream and its decode.  With c.varw row 10 holds the experts' own intermediate widths (such tables always carry row 9 too).
// Uniform 4-bit tables run the plain instance, which has none of this in it.
template <int CBK, int MR, int TWA, int NH, bool LOCAL, bool MIXED>
__global__ __launch_bounds__(64 * FW, 4) void fused_kernel(const FArgs a)
{
    __shared__ __align__(16) uint16_t xs[MR][FW * TWMAX * 16];   // this block's K slice of the transformed activations (fp16)
    __shared__ float red[FW][MR][128];
    __shared__ int rows[RF_MAX], misc[4];
    __shared__ int owner[EMAX_F];                         // one int per expert id: scratch of the item lookup
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bid = blockIdx.x;
    const bool isA = bid < a.nA, isC = bid >= a.nA + a.nB;
    const Exl3Cfg& c = a.c;
    // ---- block id -> work.  Group q lives on XCD q % 8: bid = ((q / 8) * bpg + j) * 8 + q % 8, j = position in the group.
    int g = -1, t = 0, nb = 0, s = 0, K, N;
    {
        const int b = isA ? bid : isC ? bid - a.nA - a.nB : bid - a.nA, xcd = b % NXCD, li = b / NXCD;
        if (isC) {
            const int q = (li / a.R) * NXCD + xcd;                          // q = nb2, t = token row
            if (q < a.NB2) { nb = q; t = li % a.R; s = 1; }                 // s = 1: this block has work
            K = c.I; N = c.H;
        } else if (isA) {
            const int j = li % a.bpgA, q = (li / a.bpgA) * NXCD + xcd;      // q = g * NB1 + nb1, j = t * S1 + s
            if (q < a.Gmax * a.NB1) { g = q / a.NB1; nb = q % a.NB1; t = j / a.S1; s = j % a.S1; }
            K = c.H; N = c.I;
        } else {
            const int j = li % a.bpgB, q = (li / a.bpgB) * NXCD + xcd;      // q = nb2, j = g * S2 + s
            if (q < a.NB2) { nb = q; g = j / a.S2; s = j % a.S2; }
            K = c.I; N = c.H;
        }
    }
    if (isA) __builtin_amdgcn_s_setprio(2);               // stage 1 is the critical path: its waves issue first
    TRACE(0);
    // Warm this XCD's L2 with the expert table while the routing indices are on their way: the table lookup that follows
    // them is a dependent access and would otherwise go to memory.  The blocks of an XCD cover the table once.
    uint32_t warm = 0;                                     // one word of each pointer is enough to bring its line in
    {
        const int64_t i = (int64_t)(bid / NXCD) * (64 * FW) + tid;
        if (i < (int64_t)9 * c.E) warm = *(const uint32_t*)(a.tab + i);
    }
    if (tid == 0) misc[2] = 1;
    Group grp{0, 0};
    if (g >= 0) grp = find_item(a, g, owner, rows, misc, MR);
    // The summing blocks look at the workspace's error flag as they start: it is sticky, so a wait that expired in an EARLIER call (which
    // left words of the workspace behind that are not idle) turns every later call's output into NaN until the workspace is prepared
    // again, instead of sums of stale words.  The load is in flight while the block waits for its slices.
    int stale = 0;
    if (isC && s) stale = __hip_atomic_load(a.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // Experts with their own intermediate width (row 10 of the table, reference moe_exl3.cuh:63-67,132-136): fewer column blocks in
    // gate / up (the blocks past the width have no work and their group exchanges nothing), fewer k-tiles in down; the exchange
    // buffers keep the strides of the widest expert.
    if constexpr (MIXED) {
        if (c.varw && grp.n > 0 && !isC) {
            const int we = (int)ld_k(a.tab, 10 * c.E + grp.e);
            if (isA) { N = we; if (nb * 128 >= we) grp.n = 0; }
            else K = we;
        }
    }
    TRACE(1);
    if (isC) {
        if (s) {
            // ---- the row's topk * S2 finished slices, T words per lane pair, dealt to the waves in chunks of at most 8
            const int ncol = nb * 128 + 2 * lane;
            const int T = c.topk * a.S2, chunk = min(8, (T + FW - 1) / FW);
            const float b0 = a.add ? a.add[(int64_t)t * c.H + ncol] : 0.f, b1 = a.add ? a.add[(int64_t)t * c.H + ncol + 1] : 0.f;
            float a0 = 0.f, a1 = 0.f;
            bool ok = true;
            for (int q0 = wave * chunk; q0 < T; q0 += FW * chunk) {
                const int n = min(chunk, T - q0);
                float yl[8], yh[8];
                float* py[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int q = q0 + (i < n ? i : 0);                     // slot q = (k, slice), k major
                    py[i] = a.part2 + ((int64_t)(q % a.S2) * a.P + t * c.topk + q / a.S2) * c.H + ncol;
                }
                ok = take<LOCAL, 8>(py, n, yl, yh) && ok;
#pragma unroll
                for (int i = 0; i < 8; ++i) if (i < n) { a0 += yl[i]; a1 += yh[i]; }
            }
            TRACE(4);
            red[wave][0][2 * lane] = a0; red[wave][0][2 * lane + 1] = a1;
            __syncthreads();
            if (!ok && lane == 0) atomicExch(a.err, 1);
            misc[3] = 1;
            __syncthreads();
            if (!ok || stale) misc[3] = 0;                // any wave's wait expired, or the workspace was not idle when the call began
            __syncthreads();
            if (wave == 0) {
                float v0 = red[0][0][2 * lane], v1 = red[0][0][2 * lane + 1];
#pragma unroll
                for (int w = 1; w < FW; ++w) { v0 += red[w][0][2 * lane]; v1 += red[w][0][2 * lane + 1]; }
                // a failed call must not leave the caller's old bytes in out, where a caller that only looks at the return code would
                // take them for a result: every column this block owns becomes NaN (every upstream failure ends here as an expired wait)
                if (!misc[3]) { v0 = __uint_as_float(0x7fc00000u); v1 = v0; }
                if (c.obf16) *(uint32_t*)((uint16_t*)a.out + (int64_t)t * c.H + ncol) = (uint32_t)f32_to_bf16(b0 + v0) | ((uint32_t)f32_to_bf16(b1 + v1) << 16);
                else { a.out[(int64_t)t * c.H + ncol] = b0 + v0; a.out[(int64_t)t * c.H + ncol + 1] = b1 + v1; }
            }
            TRACE(6);
        }
    } else if (grp.n > 0) {
      auto body = [&](auto bits_c) {
        constexpr int BITS = decltype(bits_c)::value;
        const int Kt = K / 16, Nt = N / 16;
        const int ktb = FW * (isA ? TWA : TWB);           // k-tiles per block
        const int kt0 = s * ktb, kt1 = min(Kt, kt0 + ktb), nkt = kt1 - kt0;
        const int nblk = (nkt + 7) / 8;                   // 128-blocks of K in this slice
        const uint32_t* tr = (const uint32_t*)ld_k(a.tab, (isA ? t : 2) * c.E + grp.e);
        const int src = tile_prev_lane(lane);
        const int ncol = nb * 128 + 2 * lane;             // this lane's two columns in the finishing steps
        const int j8 = lane >> 3, m8 = lane & 7;
        // products on the matrix unit, four token rows per instruction: acc[h][c][i] = row 4h + i, column m8 (c = 0) or m8 + 8
        constexpr int MH = (MR + 3) / 4;
        v4f acc[MH][2];
#pragma unroll
        for (int h = 0; h < MH; ++h) { acc[h][0] = v4f{0.f, 0.f, 0.f, 0.f}; acc[h][1] = v4f{0.f, 0.f, 0.f, 0.f}; }
        const int xrow = min(lane & 3, MR - 1);           // the token row whose activations this lane feeds (rows past the item's are ignored)
        if (isA) {
            const bool finisher = t == 1 && s == a.S1 - 1;
            // ---- the slice of x and its sign vector first (the transform overlaps the weight stream), then the tiles
            const uint16_t* suh = (const uint16_t*)ld_k(a.tab, (3 + t) * c.E + grp.e);
            uint32_t xr0, xr1, sr;
            const int unit0 = wave;                       // first (row, 128-block) unit of this wave
            {
                // no branch around these loads (a wave without a unit fetches unit 0 again): their wait must not land
                // ahead of the tile loads
                const int uu = unit0 < grp.n * nblk ? unit0 : 0;
                const int r = uu / nblk, kb = uu % nblk, k = kt0 * 16 + kb * 128 + 2 * lane;
                ld_x2_raw(a.x, c.xtype, (int64_t)(rows[r] / c.topk) * a.ldx + k, xr0, xr1);
                sr = *(const uint32_t*)(suh + k);
            }
            typename TileRegs<BITS>::type wr[TWA];
#pragma unroll
            for (int i = 0; i < TWA; ++i) {
                const int kt = min(kt0 + wave + FW * i, kt1 - 1);          // past the slice: a valid tile again, unused (no branch around a load)
                wr[i] = ld_tile_regs<BITS>(tr + ((int64_t)kt * Nt + nb * 8) * (8 * BITS) + lane * BITS);
            }
            TRACE(2);
            // ---- scales of the finishing step (the finisher only)
            uint32_t sgr = 0u, sur = 0u, sdr = 0u;         // fp16 pairs as loaded: three registers across the products instead of six
            if (finisher) {
                const uint16_t* svg = (const uint16_t*)ld_k(a.tab, 6 * c.E + grp.e);
                const uint16_t* svu = (const uint16_t*)ld_k(a.tab, 7 * c.E + grp.e);
                const uint16_t* sud = (const uint16_t*)ld_k(a.tab, 5 * c.E + grp.e);
                sgr = *(const uint32_t*)(svg + ncol); sur = *(const uint32_t*)(svu + ncol); sdr = *(const uint32_t*)(sud + ncol);   // ncol is even
            }
            // ---- transform the slice of x into LDS: wave per (row, 128-block)
            for (int u = unit0; u < grp.n * nblk; u += FW) {
                const int r = u / nblk, kb = u % nblk;
                if (u != unit0) {
                    const int k = kt0 * 16 + kb * 128 + 2 * lane;
                    ld_x2_raw(a.x, c.xtype, (int64_t)(rows[r] / c.topk) * a.ldx + k, xr0, xr1);
                    sr = *(const uint32_t*)(suh + k);
                }
                float v0, v1;
                cvt_x2(c.xtype, xr0, xr1, v0, v1);
                v0 *= f16_bits_to_f32((uint16_t)sr); v1 *= f16_bits_to_f32((uint16_t)(sr >> 16));
                fwht128(v0, v1, lane);
                *(uint32_t*)&xs[r][kb * 128 + 2 * lane] = (uint32_t)f32_to_f16_bits(v0) | ((uint32_t)f32_to_f16_bits(v1) << 16);
            }
            __syncthreads();
            TRACE(3);
            // A block of eight k-tiles per wave keeps one sum per half (NH = 2): a K slice is always sixteen k-tiles summed in the
            // same order, whatever the block size, so a row's bits do not depend on the block size a call's grid asks for.
            v4f acc2[NH == 2 ? MH : 1][2];
#pragma unroll
            for (int h = 0; h < (NH == 2 ? MH : 1); ++h) { acc2[h][0] = v4f{0.f, 0.f, 0.f, 0.f}; acc2[h][1] = v4f{0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
            for (int i = 0; i < TWA; ++i) {
                const int kt = kt0 + wave + FW * i;
                if (kt < kt1) {
                    h2 wd[4][4];
                    decode_tile_regs<CBK, BITS>(wr[i], __shfl(tile_last_word<BITS>(wr[i]), src, 64), wd);
#pragma unroll
                    for (int h = 0; h < MH; ++h) {
                        h4 xq[4];
                        ld_xq(&xs[min(4 * h + xrow, MR - 1)][(kt - kt0) * 16], xq);
                        if (NH == 2 && i >= 4) mfma_tile32(wd, xq, acc2[h][0], acc2[h][1]);
                        else mfma_tile32(wd, xq, acc[h][0], acc[h][1]);
                    }
                }
            }
            TRACE(5);
            // ---- per K slice: sum the waves in wave order; every block but the finisher hands the slice over inside the XCD, the
            // finisher keeps its own slices in LDS (where the activations were: every wave is past them after the first barrier)
            float* ownl = (float*)&xs[0][0];              // [NH][MR][128]
            const int nh = NH == 1 ? 1 : min(NH, (nkt + 15) / 16);          // K slices of this block that hold k-tiles
#pragma unroll
            for (int hf = 0; hf < NH; ++hf) {
                if (hf < nh) {
                    if (hf) __syncthreads();              // the previous slice's sums have been read
#pragma unroll
                    for (int r = 0; r < MR; ++r) {
                        red[wave][r][16 * j8 + m8] = (NH == 2 && hf ? acc2 : acc)[r >> 2][0][r & 3];
                        red[wave][r][16 * j8 + m8 + 8] = (NH == 2 && hf ? acc2 : acc)[r >> 2][1][r & 3];
                    }
                    __syncthreads();
                    float* part = a.part1 + ((int64_t)((s * NH + hf) * 2 + t) * a.P) * c.I;   // strides of the widest expert
                    for (int i = tid; i < grp.n * 64; i += 64 * FW) {
                        const int r = i >> 6, col = (i & 63) * 2;
                        float v0 = red[0][r][col], v1 = red[0][r][col + 1];
#pragma unroll
                        for (int w = 1; w < FW; ++w) { v0 += red[w][r][col]; v1 += red[w][r][col + 1]; }
                        if (!finisher) put2<LOCAL>(&part[(int64_t)rows[r] * c.I + nb * 128 + col], v0, v1);
                        else { ownl[(hf * MR + r) * 128 + col] = v0; ownl[(hf * MR + r) * 128 + col + 1] = v1; }
                    }
                }
            }
            if (!finisher) {
                TRACE(6);
            } else if (grp.n == 1) {
                __syncthreads();                          // the own slices are in place and the waves' sums are free
                // ---- finisher of a one-row item, spread over the block (a lone wave's instruction chain is the cost here):
                // wave 0 sums and transforms gate, wave 1 up; then every wave applies the activation and the down input
                // transform itself and stores its share of the copies of xh2.  Same arithmetic as the general form below.
                float* fin = &red[0][0][0];               // [2][128]
                const int r0 = rows[0];
                if (wave < 2) {
                    const int n = wave == 0 ? a.VS : a.VS - nh;            // this block holds the last up slices itself
                    float pl[SMAX], ph[SMAX];
                    float* pp[SMAX];
#pragma unroll
                    for (int ss = 0; ss < SMAX; ++ss) pp[ss] = a.part1 + ((int64_t)((ss < n ? ss : 0) * 2 + wave) * a.P + r0) * c.I + ncol;
                    bool good = true;
                    if (n > 0) good = take<LOCAL, SMAX>(pp, n, pl, ph);
                    TRACE(4);
                    float v0 = 0.f, v1 = 0.f;
#pragma unroll
                    for (int ss = 0; ss < SMAX; ++ss) if (ss < n) { v0 += pl[ss]; v1 += ph[ss]; }
                    if (wave == 1) {
#pragma unroll
                        for (int hf = 0; hf < NH; ++hf) if (hf < nh) { v0 += ownl[hf * MR * 128 + 2 * lane]; v1 += ownl[hf * MR * 128 + 2 * lane + 1]; }
                    }
                    fwht128(v0, v1, lane);
                    *(float2*)&fin[wave * 128 + 2 * lane] = make_float2(v0, v1);
                    if (!good) misc[2] = 0;
                }
                __syncthreads();
                if (misc[2]) {
                    const float2 gg = *(const float2*)&fin[2 * lane], uu = *(const float2*)&fin[128 + 2 * lane];
                    const float sg0 = f16_bits_to_f32((uint16_t)sgr), sg1 = f16_bits_to_f32((uint16_t)(sgr >> 16));
                    const float su0 = f16_bits_to_f32((uint16_t)sur), su1 = f16_bits_to_f32((uint16_t)(sur >> 16));
                    const float sd0 = f16_bits_to_f32((uint16_t)sdr), sd1 = f16_bits_to_f32((uint16_t)(sdr >> 16));
                    float v0 = exl3_act(c.act, gg.x * sg0, uu.x * su0) * sd0;
                    float v1 = exl3_act(c.act, gg.y * sg1, uu.y * su1) * sd1;
                    fwht128(v0, v1, lane);
                    uint32_t pk = (uint32_t)f32_to_f16_bits(v0) | ((uint32_t)f32_to_f16_bits(v1) << 16);
                    if (pk == EMPTY) pk = 0x7e007e00u;
                    for (int q = wave; q < a.NB2; q += FW) st_dev32(a.xh2 + ((int64_t)q * a.P + r0) * (c.I / 2) + (ncol >> 1), pk);
                } else if (tid == 0) atomicExch(a.err, 1);
                TRACE(6);
            } else {
                // ---- finisher: gate and up sums in slice order, Hadamard, svh, activation, down input transform -> xh2
                __syncthreads();                          // the own slices are in place
                bool good = true;
                for (int r = wave; r < grp.n; r += FW) {
                    // gate slices 0 .. VS-1 and up slices 0 .. VS-nh-1 (this block holds the last up slices itself), one round of requests
                    float pl[2 * SMAX], ph[2 * SMAX];
                    float* pp[2 * SMAX];
#pragma unroll
                    for (int ss = 0; ss < 2 * SMAX; ++ss) {
                        const int tt = ss < a.VS ? 0 : 1, s2 = ss < a.VS ? ss : (ss - a.VS < a.VS - nh ? ss - a.VS : 0);
                        pp[ss] = a.part1 + ((int64_t)(s2 * 2 + tt) * a.P + rows[r]) * c.I + ncol;
                    }
                    good = take<LOCAL, 2 * SMAX>(pp, 2 * a.VS - nh, pl, ph) && good;
                    TRACE(4);
                    float g0 = 0.f, g1 = 0.f, u0 = 0.f, u1 = 0.f;
#pragma unroll
                    for (int ss = 0; ss < 2 * SMAX; ++ss) {
                        if (ss < a.VS) { g0 += pl[ss]; g1 += ph[ss]; }
                        else if (ss < 2 * a.VS - nh) { u0 += pl[ss]; u1 += ph[ss]; }
                    }
#pragma unroll
                    for (int hf = 0; hf < NH; ++hf)           // this block's own slices of up, last in order
                        if (hf < nh) { u0 += ownl[(hf * MR + r) * 128 + 2 * lane]; u1 += ownl[(hf * MR + r) * 128 + 2 * lane + 1]; }
                    fwht128(g0, g1, lane);
                    fwht128(u0, u1, lane);
                    const float sg0 = f16_bits_to_f32((uint16_t)sgr), sg1 = f16_bits_to_f32((uint16_t)(sgr >> 16));
                    const float su0 = f16_bits_to_f32((uint16_t)sur), su1 = f16_bits_to_f32((uint16_t)(sur >> 16));
                    const float sd0 = f16_bits_to_f32((uint16_t)sdr), sd1 = f16_bits_to_f32((uint16_t)(sdr >> 16));
                    float v0 = exl3_act(c.act, g0 * sg0, u0 * su0) * sd0;
                    float v1 = exl3_act(c.act, g1 * sg1, u1 * su1) * sd1;
                    fwht128(v0, v1, lane);
                    uint32_t pk = (uint32_t)f32_to_f16_bits(v0) | ((uint32_t)f32_to_f16_bits(v1) << 16);
                    if (pk == EMPTY) pk = 0x7e007e00u;
                    if (good)
                        for (int q = 0; q < a.NB2; ++q) st_dev32(a.xh2 + ((int64_t)q * a.P + rows[r]) * (c.I / 2) + (ncol >> 1), pk);
                }
                TRACE(6);
                if (!good && lane == 0) atomicExch(a.err, 1);
            }
        } else {
            if constexpr (MIXED) {
                if (nkt <= 0) {
                    // a K slice wholly past the expert's own width: its share of every pair's output is zero (the summing block
                    // waits for a word from every slice)
                    for (int r = wave; r < grp.n; r += FW) put2<LOCAL>(a.part2 + ((int64_t)s * a.P + rows[r]) * c.H + ncol, 0.f, 0.f);
                    return;
                }
            }
            // ---- issue the tile loads, decode and fetch the finishing scales (independent of stage 1), then take xh2
            typename TileRegs<BITS>::type wr[TWB];
#pragma unroll
            for (int i = 0; i < TWB; ++i) {
                const int kt = min(kt0 + wave + FW * i, kt1 - 1);          // past the slice: a valid tile again, unused (no branch around a load)
                wr[i] = ld_tile_regs<BITS>(tr + ((int64_t)kt * Nt + nb * 8) * (8 * BITS) + lane * BITS);
            }
            TRACE(2);
            const uint16_t* svd = (const uint16_t*)ld_k(a.tab, 8 * c.E + grp.e);
            const float svd0 = f16_bits_to_f32(svd[ncol]), svd1 = f16_bits_to_f32(svd[ncol + 1]);
            // route weights of the pairs this wave finishes (rows wave, wave + FW, ...), fetched long before they are needed
            float wk[(MR + FW - 1) / FW];
#pragma unroll
            for (int j = 0; j < (MR + FW - 1) / FW; ++j) wk[j] = exl3_ld_w(a.w, c.wtype, rows[wave + FW * j < grp.n ? wave + FW * j : 0]);
            h2 wd[TWB][4][4];
#pragma unroll
            for (int i = 0; i < TWB; ++i) {
                decode_tile_regs<CBK, BITS>(wr[i], __shfl(tile_last_word<BITS>(wr[i]), src, 64), wd[i]);
#pragma unroll
                for (int q = 0; q < 16; ++q) asm volatile("" : "+v"(wd[i][q >> 2][q & 3]));   // decoded now, not after the wait
            }
            asm volatile("" :: "v"(svd0), "v"(svd1));
#pragma unroll
            for (int j = 0; j < (MR + FW - 1) / FW; ++j) asm volatile("" :: "v"(wk[j]));
            TRACE(3);
            uint32_t* xc = a.xh2 + ((int64_t)nb * a.P) * (c.I / 2) + kt0 * 8;         // this column block's copy, this K slice
            // One round per row: a wave watches whole rows of the slice (two words per lane, at most 128 words per row), so the
            // data arrives with the poll that sees it complete; the other waves sleep at the barrier meanwhile.
            __builtin_amdgcn_s_setprio(3);                // from here on this block is the critical path
            bool good = true;
            {
                constexpr int RW = (MR + FW - 1) / FW;    // rows per wave
                uint32_t* p[RW];
#pragma unroll
                for (int j = 0; j < RW; ++j) {
                    const int r = wave + FW * j;          // past the item's rows: this wave's first row again (never another wave's)
                    p[j] = xc + (int64_t)rows[r < grp.n ? r : (wave < grp.n ? wave : 0)] * (c.I / 2) + (lane < nkt * 4 ? 2 * lane : 0);
                }
                if (wave < grp.n) {
                    uint64_t v[RW];
                    int spins = 0;
                    for (;;) {
                        asm volatile("" ::: "memory");
                        bool ok = true;
#pragma unroll
                        for (int j = 0; j < RW; ++j) v[j] = ld_dev64(p[j]);
#pragma unroll
                        for (int j = 0; j < RW; ++j) ok = ok && (uint32_t)v[j] != EMPTY && (uint32_t)(v[j] >> 32) != EMPTY;
                        if (__builtin_amdgcn_ballot_w64(!ok) == 0) break;
                        if (++spins >= SPIN_MAX) { good = false; break; }
                        __builtin_amdgcn_s_sleep(2);
                    }
#pragma unroll
                    for (int j = 0; j < RW; ++j) {
                        const int r = wave + FW * j;
                        if (r < grp.n && lane < nkt * 4) {
                            if (good) st_dev64(p[j], EMPTY2);
                            *(uint64_t*)&xs[r][4 * lane] = v[j];
                        }
                    }
                }
            }
            if (!good) misc[2] = 0;
            __syncthreads();
            TRACE(4);
            if (misc[2]) {
#pragma unroll
                for (int i = 0; i < TWB; ++i) {
                    const int kt = kt0 + wave + FW * i;
                    if (kt < kt1) {
#pragma unroll
                        for (int h = 0; h < MH; ++h) {
                            h4 xq[4];
                            ld_xq(&xs[min(4 * h + xrow, MR - 1)][(kt - kt0) * 16], xq);
                            mfma_tile32(wd[i], xq, acc[h][0], acc[h][1]);
                        }
                    }
                }
                TRACE(5);
#pragma unroll
                for (int r = 0; r < MR; ++r) { red[wave][r][16 * j8 + m8] = acc[r >> 2][0][r & 3]; red[wave][r][16 * j8 + m8 + 8] = acc[r >> 2][1][r & 3]; }
                __syncthreads();
                // ---- finish this slice of the down product (the transform is linear: slice by slice): Hadamard, svh, route
                // weight; wave per pair row.  The C block of the token row adds the slices.
#pragma unroll
                for (int j = 0; j < (MR + FW - 1) / FW; ++j) {
                    const int r = wave + FW * j;
                    if (r < grp.n) {
                        float o0 = red[0][r][2 * lane], o1 = red[0][r][2 * lane + 1];
#pragma unroll
                        for (int w = 1; w < FW; ++w) { o0 += red[w][r][2 * lane]; o1 += red[w][r][2 * lane + 1]; }
                        fwht128(o0, o1, lane);
                        put2<LOCAL>(a.part2 + ((int64_t)s * a.P + rows[r]) * c.H + ncol, o0 * svd0 * wk[j], o1 * svd1 * wk[j]);
                    }
                }
                TRACE(6);
            } else if (tid == 0) atomicExch(a.err, 1);
        }
      };
      if constexpr (!MIXED) body(std::integral_constant<int, 4>{});
      else {
        switch ((int)ld_k(a.tab, 9 * c.E + grp.e)) {
            case 3: body(std::integral_constant<int, 3>{}); break;
            case 4: body(std::integral_constant<int, 4>{}); break;
            case 5: body(std::integral_constant<int, 5>{}); break;
            case 6: body(std::integral_constant<int, 6>{}); break;
            default: if (tid == 0) atomicExch(a.err, 1);      // a width the format does not have: nothing stored, the flag raised
        }
      }
    }
    asm volatile("" :: "v"(warm));                         // the warming load is complete before the wave ends
    TRACE(7);
#ifdef SPK_EXL3_TRACE
    // where the block ran: XCC_ID (register 20) and HW_ID (register 4: CU, shader array, shader engine)
    if (a.trace && tid == 0) a.trace[(int64_t)bid * 16 + 8] = ((long long)(__builtin_amdgcn_s_getreg((31 << 11) | 20) & 0xf) << 32) | (uint32_t)__builtin_amdgcn_s_getreg((31 << 11) | 4);
#endif
}

// every exchanged word EMPTY, the error flag clear
__global__ void fill_kernel(uint32_t* p, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = i < HEAD / 4 ? 0u : EMPTY;
}
int g_force_twa = 0;                  // diagnostics: 4 or 8 forces the k-tiles per wave of a stage-1 block, 0 = by shape
struct FPlan { int P, Gmax, twa, nh, S1, VS, S2, NB1, NB2, nA, nB, nC, bpgA, bpgB; size_t part1, xh2, part2, total; };
FPlan fplan(const Exl3Cfg& c, int R)
{
    FPlan p;
    p.P = R * c.topk;
    p.Gmax = p.P < c.E ? p.P : c.E;
    // The K slices (and with them the order of summation) depend on the shape only, never on R: a row's bits must not depend on
    // the batch.  Where K allows 8 slices of sixteen k-tiles, a slice is sixteen k-tiles; finer stage-1 blocks (one slice each)
    // balance the CUs better while the grid is small, larger blocks (two slices each, summed apart) turn over less when it is not.
    const bool fine = c.H / 16 <= SMAX * FW * 4;
    p.twa = fine && (int64_t)p.Gmax * (c.I / 128) * 2 * (c.H / 16 / (FW * 4)) <= 1536 ? 4 : 8;   // measured: C2 at two rows (1280 blocks) is faster fine, at four (2560) coarse
    if (g_force_twa == 8 || (g_force_twa == 4 && fine)) p.twa = g_force_twa;
    p.nh = p.twa == 8 && fine ? 2 : 1;
    p.S1 = (c.H / 16 + FW * p.twa - 1) / (FW * p.twa);
    p.VS = p.nh == 2 ? (c.H / 16 + FW * 4 - 1) / (FW * 4) : p.S1;
    p.S2 = (c.I / 16 + FW * TWB - 1) / (FW * TWB);
    p.NB1 = c.I / 128; p.NB2 = c.H / 128;
    p.bpgA = 2 * p.S1; p.bpgB = p.Gmax * p.S2;
    const int QA = (p.Gmax * p.NB1 + NXCD - 1) / NXCD * NXCD, QB = (p.NB2 + NXCD - 1) / NXCD * NXCD;   // groups, padded to the XCD count
    p.nA = QA * p.bpgA;
    p.nB = QB * p.bpgB;
    p.nC = QB * R;
    size_t o = HEAD;
    auto take = [&](size_t n) { const size_t q = o; o += align256(n); return q; };
    p.part1 = take(4 * (size_t)p.VS * 2 * p.P * c.I);
    p.xh2 = take(4 * (size_t)p.NB2 * p.P * (c.I / 2));
    p.part2 = take(4 * (size_t)p.S2 * p.P * c.H);
    p.total = o;
    return p;
}

template <int CBK, int TWA, int NH, bool LOCAL, bool MIXED>
void launch3(const FArgs& a, int maxrows, hipStream_t st)
{
    const dim3 grid(a.nA + a.nB + a.nC), blk(64 * FW);
    if (maxrows <= 1) fused_kernel<CBK, 1, TWA, NH, LOCAL, MIXED><<<grid, blk, 0, st>>>(a);
    else if (maxrows <= 2) fused_kernel<CBK, 2, TWA, NH, LOCAL, MIXED><<<grid, blk, 0, st>>>(a);
    else if (maxrows <= 4) fused_kernel<CBK, 4, TWA, NH, LOCAL, MIXED><<<grid, blk, 0, st>>>(a);
    else fused_kernel<CBK, 8, TWA, NH, LOCAL, MIXED><<<grid, blk, 0, st>>>(a);
}
template <int CBK, bool LOCAL, bool MIXED>
void launch2(const FArgs& a, int twa, int nh, int maxrows, hipStream_t st)
{
    if (twa == 4) launch3<CBK, 4, 1, LOCAL, MIXED>(a, maxrows, st);
    else if (nh == 2) launch3<CBK, 8, 2, LOCAL, MIXED>(a, maxrows, st);
    else launch3<CBK, 8, 1, LOCAL, MIXED>(a, maxrows, st);
}
template <int CBK, bool MIXED>
void launch(const FArgs& a, int twa, int nh, int maxrows, hipStream_t st)
{
    if (a.local) launch2<CBK, true, MIXED>(a, twa, nh, maxrows, st); else launch2<CBK, false, MIXED>(a, twa, nh, maxrows, st);
}

int g_force_local = -1;               // diagnostics: 1 / 0 force the XCD-local / the device-coherent exchange, -1 = by the placement check

}  // namespace

bool exl3_fused_ok(const Exl3Cfg& c, int R)
{
    return R >= 1 && R <= RF_MAX && c.E <= EMAX_F && c.topk <= 16 && R * c.topk <= PF_MAX && c.H <= SMAX * FW * TWMAX * 16 && c.I <= SMAX * FW * TWB * 16;
}
size_t exl3_fused_ws_bytes(const Exl3Cfg& c, int R) { return fplan(c, R).total; }

// Every exchanged word of a workspace EMPTY and its error flag clear (any size: the whole buffer is filled).
int exl3_fused_ws_prepare(void* ws, size_t bytes, hipStream_t st)
{
    const int64_t n = (int64_t)(bytes / 4);
    if (n > 0) fill_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>((uint32_t*)ws, n);
    return launch_status();
}

int exl3_fused_launch(const Exl3Cfg& c, const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out, void* ws,
                      int clean, hipStream_t st)
{
    const FPlan p = fplan(c, R);
    char* b = (char*)ws;
    FArgs a;
    a.x = x; a.ldx = ldx; a.idx = idx; a.w = w; a.tab = (const uint64_t*)tab; a.add = (const float*)add; a.out = (float*)out;
    a.err = (int*)b; a.part1 = (float*)(b + p.part1); a.xh2 = (uint32_t*)(b + p.xh2); a.part2 = (float*)(b + p.part2);
    a.R = R; a.P = p.P; a.Gmax = p.Gmax; a.S1 = p.S1; a.VS = p.VS; a.S2 = p.S2; a.NB1 = p.NB1; a.NB2 = p.NB2; a.nA = p.nA; a.nB = p.nB; a.nC = p.nC;
    a.bpgA = p.bpgA; a.bpgB = p.bpgB;
    a.local = g_force_local >= 0 ? g_force_local : xcd_placement() == 1;
    a.c = c;
    a.trace = g_trace;
    if (!clean && !ws_is_prepared(ws, p.total)) {          // idle exchange words: promised by the caller or known from the workspace's own *_ws_init call
        const int rc = exl3_fused_ws_prepare(ws, p.total, st);
        if (rc) return rc;
    }
    if (c.mixed || c.varw) { if (c.cbk == CB_MCG) launch<CB_MCG, true>(a, p.twa, p.nh, R, st); else launch<CB_MUL1, true>(a, p.twa, p.nh, R, st); }
    else if (c.cbk == CB_MCG) launch<CB_MCG, false>(a, p.twa, p.nh, R, st);
    else launch<CB_MUL1, false>(a, p.twa, p.nh, R, st);
    return launch_status();
}

// diagnostics: device buffer of 8 timestamps (100 MHz) per block of the next launches, or null
extern "C" __attribute__((visibility("default"))) void spark_debug_exl3_trace(long long* buf) { g_trace = buf; }
// diagnostics: force the k-tiles per wave of a stage-1 block (4 or 8; 0 = chosen by shape)
extern "C" __attribute__((visibility("default"))) void spark_debug_exl3_twa(int v) { g_force_twa = v; }
// diagnostics: force the exchange mode of the single-launch path (1 XCD-local, 0 device-coherent, -1 as the placement check found)
extern "C" __attribute__((visibility("default"))) void spark_debug_exl3_local(int v) { g_force_local = v; }

}  // namespace spk
