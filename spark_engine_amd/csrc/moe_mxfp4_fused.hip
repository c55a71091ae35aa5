// Routed MXFP4 experts (gate / up, SwiGLU, act_quant, down, weighted sum) in ONE launch for decode-sized calls:
// R <= 8 token rows, topk + shared <= 16 experts per row.
//
// The several-kernel path (moe_mxfp4.hip) spends more time in launch gaps and tiny kernels (activation quantisation,
// grouping, combine) than the batch-1 weight stream takes.  Here one grid holds both weight streams:
//   U blocks: (item, 32 features of I).  8 waves split K as in up_kernel (same summation order, so the values are the
//       same bits): each wave quantises its K groups of the token rows itself (act_quant per 32, into LDS), streams the 32
//       gate and 32 up rows, exact products on the bf16 MFMA, LDS reduction in wave order, SwiGLU * route weight, act_quant of the 32
//       features; the 32 code bytes + scale of every item row go to every stage-2 column block's own copy of h.
//   D blocks: (64 output columns | item).  Stream their down-projection rows into registers first (raw MXFP4 is the MFMA
//       operand, nothing to decode), then take the item's h, MFMA as in down_kernel (same order), hand the per-pair
//       outputs over inside the XCD; for every token row the block of the row's last item in launch order adds
//       them up: (add + shared experts) + (routed experts in slot order), the reference's order.
//
// Block order.  Work is laid out in groups of GS blocks: block i of group g first does stage-1 unit i of item g, then
// stage-2 unit i of item g - 1 (group 0 has no stage 2, the last group no stage 1).  A block issues its stage-2 weight loads
// the moment its stage-1 registers are free, so the weight stream never pauses for a block to retire and another to start,
// and the last item's stage-2 blocks hold their weights long before its h arrives.
//
// Exchange without counters: every exchanged 32-bit word of the workspace is EMPTY (all ones) between uses; a producer
// stores its value (an all-ones value is altered to another NaN pattern), the single consumer of the word polls until it
// is not EMPTY and stores EMPTY back.  h crosses XCDs (device-coherent stores and loads), the per-pair outputs stay in
// one XCD's L2 (workgroup b runs on XCD b % 8; all D blocks of a column block share an XCD).  A block only waits for blocks
// with lower ids; waits are bounded and an expiry raises an error flag while every block still runs to its end.
//
// Semantics: reference engine-rs/shim/ds41_moe.cu:1-24, ds41_mx.cu:129-317, engine-rs/src/ds41/kern.rs:1116-1133.
#include "moe_mxfp4.hpp"
#include "runtime.hpp"
#include <type_traits>

namespace spk {
namespace mx {
namespace {

constexpr int NW = 8, NT = 64 * NW;
constexpr int RMAX = 8, TTMAX = 16, PMAXF = RMAX * TTMAX;
constexpr int DC = 64;                 // output columns of a stage-2 block
constexpr int NXCD = 8, HEAD = 256, SPIN_MAX = 200000;
constexpr uint32_t EMPTY = 0xffffffffu;
constexpr uint64_t EMPTY2 = ~0ull;
constexpr int RED_BYTES = NW * 4 * 4 * 64 * 4;
constexpr size_t XBF_BYTES = 44 * 1024;                   // most bytes of activation rows staged as bf16 (four rows of hidden width 5120)

long long* g_trace = nullptr;
#ifdef SPK_MX_TRACE
#define TRACE(i) do { if (a.trace && tid == 0) a.trace[(int64_t)bid * 16 + (i)] = wall_clock64(); } while (0)
#else
#define TRACE(i) do { } while (0)
#endif

struct MArgs {
    const void* x;                     // bf16 [R, H] (QUANT) or E4M3 [R, H]
    const uint8_t* xs;                 // UE8M0 [R, H / 32] (not QUANT)
    const int64_t* idx; const float* rw;
    WMat w1, w3, w2;
    const float* add; float* y;
    uint32_t* hc;                      // [NBD][P][I / 4]  act-quantised intermediate, code words, one copy per column block
    uint32_t* hsw;                     // [NBD][P][I / 32] its scales, one word each
    float* yd;                         // [P][H] per-pair outputs
    int* err;
    long long* trace;                  // optional per-block time stamps (diagnostic builds), 16 per block
    int R, TT, topk, E, P, Gmax, H, I, NJ, NBD, GS;        // GS = blocks per group (a multiple of 8)
    int obf16;                         // y is bf16 [R, H] (the binary32 result rounded to nearest even)
};

__device__ __forceinline__ uint32_t ld_dev32(const void* p) { return __hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ uint64_t ld_dev64(const void* p) { return __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_dev32(void* p, uint32_t v) { __hip_atomic_store((uint32_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void st_dev64(void* p, uint64_t v) { __hip_atomic_store((uint64_t*)p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
// four words with one device-coherent vector store (p 16-byte aligned): every word arrives whole, the four not necessarily together,
// which is all a consumer that checks every word needs; a quarter of the write transactions of four st_dev32
__device__ __forceinline__ void st_dev128(void* p, const v4i& v)
{
    asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
// a non-temporal load is not kept in the CU's L1: a poll reads the XCD's L2 every time
__device__ __forceinline__ uint32_t ld_l2(const float* p)
{
    return __builtin_nontemporal_load((const __attribute__((address_space(1))) uint32_t*)(uintptr_t)p);
}

__device__ __forceinline__ int pair_expert(const MArgs& a, int p)
{
    const int r = p / a.TT, k = p % a.TT;
    return k < a.topk ? clamp_expert((int)a.idx[(int64_t)r * a.topk + k], a.E) : a.E + (k - a.topk);
}
// the same for a pair index that is uniform over the wave: the index comes through the scalar cache
__device__ __forceinline__ int pair_expert_k(const MArgs& a, int p)
{
    const int r = p / a.TT, k = p % a.TT;
    return k < a.topk ? clamp_expert((int)ld_k(a.idx, r * a.topk + k), a.E) : a.E + (k - a.topk);
}
struct Group { int e, n; };      // an item: expert and number of pairs (rows), the pairs ascending in a rows[] array

template <int LAYOUT, bool QUANT, bool LOCAL>
__global__ __launch_bounds__(NT, 4) void mx_fused_kernel(const MArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ int sidx[PMAXF], rowsU[RMAX], rowsD[RMAX], comb[RMAX], misc[4], gsel[4];
    __shared__ float amx[NW][16];
    __shared__ __align__(16) uint32_t hbw[16][8];          // the block's 32 code bytes per item row
    __shared__ uint32_t he[16];
    float (*red)[4][4][64] = (float (*)[4][4][64])smem;    // [wave][tile][v][lane]
    unsigned char* extra = smem + RED_BYTES;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, rg = lane >> 4;
    const int bid = blockIdx.x;
    const int grpi = bid / a.GS, bi = bid % a.GS;          // GS % 8 == 0: column block bi runs on XCD bi % 8 in every group
    const int H = a.H, I = a.I;
    TRACE(0);
    __builtin_amdgcn_s_setprio(2);
    const bool hasU = grpi < a.Gmax && bi < a.NJ;
    // both items of this block up front (the stage-2 loads must not wait for an index lookup later), worked out by one wave
    Group gu{0, 0}, gd{0, 0};
    const bool wantU = hasU, wantD = grpi >= 1 && bi < a.NBD;
    if (a.R == 1) {                                        // every pair is its own item
        if (wantU && grpi < a.P) gu = Group{pair_expert_k(a, grpi), 1};
        if (wantD && grpi - 1 < a.P) gd = Group{pair_expert_k(a, grpi - 1), 1};
        if (tid == 0) { rowsU[0] = grpi; rowsD[0] = grpi - 1; }
        __syncthreads();
    } else {
        if (wave == 0) {
            WaveItems<PMAXF / 64> wi;
            wave_items_init(wi, a.P, lane, (int*)smem, [&](int p) { return pair_expert(a, p); });
#pragma unroll
            for (int j = 0; j < PMAXF / 64; ++j) if (lane + 64 * j < a.P) sidx[lane + 64 * j] = wi.e[j];
            int nu = 0, nd = 0;
            bool ou = false, od = false;                   // an item never holds more rows than the call unless a token row names an expert twice
            const int eu = wantU ? wave_items_pick(wi, grpi, lane, rowsU, nu, a.R, ou) : -1;
            const int ed = wantD ? wave_items_pick(wi, grpi - 1, lane, rowsD, nd, a.R, od) : -1;
            if (lane == 0) { gsel[0] = eu; gsel[1] = nu; gsel[2] = ed; gsel[3] = nd; if (ou || od) atomicExch(a.err, 1); }
        }
        __syncthreads();
        gu = Group{gsel[0], gsel[0] >= 0 ? gsel[1] : 0};
        gd = Group{gsel[2], gsel[2] >= 0 ? gsel[3] : 0};
    }
    TRACE(1);
    if (gu.n > 0) {
        // ================================================================ stage 1
        const Group grp = gu;
        const int* rows = rowsU;
        const int jb = bi, j0 = jb * 32;
        const int steps = H >> 7, nkg = (steps + 3) >> 2;
        // route weight of this lane's item row, requested ahead of the weight rows
        float wgt = 0.f;
        if (c < grp.n) { const int pr = rows[c], k = pr % a.TT; wgt = k < a.topk ? a.rw[(int64_t)(pr / a.TT) * a.topk + k] : 1.0f; }
        unsigned char* xql = extra;                        // [n][H] E4M3 codes of the item's token rows
        unsigned char* xsl = extra + (size_t)a.R * H;      // [n][H / 32] scales
        // activations of this wave's K groups into LDS: act_quant per 32 (reference engine-rs/src/ds41/ops.rs:26-35, 4 lanes x 8
        // elements per block) of bf16 rows, or (COPY) the caller's codes and scales as they are
        auto stage_x = [&](auto copy) {
            constexpr bool COPY = decltype(copy)::value;
            for (int kg = wave; kg < nkg; kg += NW)
                for (int r = 0; r < grp.n; ++r) {
                    const int k = kg * 512 + lane * 8;
                    if (k >= H) continue;
                    const int tok = rows[r] / a.TT;
                    if constexpr (COPY) {
                        *(uint2*)(xql + (size_t)r * H + k) = *(const uint2*)((const uint8_t*)a.x + (int64_t)tok * H + k);
                        if ((lane & 3) == 0) xsl[(size_t)r * (H >> 5) + (k >> 5)] = a.xs[(int64_t)tok * (H >> 5) + (k >> 5)];
                    } else {
                        const uint4 raw = *(const uint4*)((const uint16_t*)a.x + (int64_t)tok * H + k);
                        const uint32_t rw4[4] = {raw.x, raw.y, raw.z, raw.w};
                        float v[8];
                        float am = 0.f;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            v[2 * i] = __uint_as_float(rw4[i] << 16); v[2 * i + 1] = __uint_as_float(rw4[i] & 0xffff0000u);
                            am = fmaxf(am, fmaxf(fabsf(v[2 * i]), fabsf(v[2 * i + 1])));
                        }
                        am = fmaxf(am, lane_xor<1>(am, lane));
                        am = fmaxf(am, lane_xor<2>(am, lane));
                        const uint32_t e = aq_scale(am);
                        *(uint2*)(xql + (size_t)r * H + k) = make_uint2(aq_word4(v[0], v[1], v[2], v[3], e), aq_word4(v[4], v[5], v[6], v[7], e));
                        if ((lane & 3) == 0) xsl[(size_t)r * (H >> 5) + (k >> 5)] = (unsigned char)e;
                    }
                }
        };
        const bool valid = c < grp.n;
        const int rc = valid ? c : 0;
        const int pair = rows[rc];
        if (nkg <= NW || nkg > NW + 2) {
            // ---- wave w walks K groups w, w + 8, ... of the four tiles (gate, gate + 16, up, up + 16); normally one K group, loaded
            // before the wave stages that K group's activations
            v4i A[4][4];
            GrpScale sr[4];                                // requested here, turned into operands right before the multiplies
            uint32_t sa[4];
            {
                const int kg = min(wave, nkg - 1);
                grp_load<LAYOUT>(a.w1, grp.e, j0, kg, lane, A[0], sr[0]);
                // The other three tiles are requested once the first has arrived.  Measured, not derived: with every request of every
                // block issued at once the memory system serves them by fair share and the exchanges queue behind all of it; holding
                // three quarters back by one round trip (C3, same box, alternating runs): 27.1 -> 26.5 us at one row, 46.5 / 74.5
                // unchanged at two / four; two and two 26.7 / 46.7 / 74.5, three and one 26.6 / 47.4 / 75.5, none 27.1 / 46.5 / 74.6.
#pragma unroll
                for (int s = 0; s < 4; ++s) asm volatile("" : "+v"(A[0][s]));
                grp_load<LAYOUT>(a.w1, grp.e, j0 + 16, kg, lane, A[1], sr[1]);
                grp_load<LAYOUT>(a.w3, grp.e, j0, kg, lane, A[2], sr[2]);
                grp_load<LAYOUT>(a.w3, grp.e, j0 + 16, kg, lane, A[3], sr[3]);
            }
            if (QUANT) stage_x(std::false_type{});         // read back by this wave only: no barrier
            TRACE(2);
            const uint8_t* xr = QUANT ? xql + (size_t)rc * H : (const uint8_t*)a.x + (int64_t)(pair / a.TT) * H;
            const uint8_t* xsr = QUANT ? xsl + (size_t)rc * (H >> 5) : a.xs + (int64_t)(pair / a.TT) * (H >> 5);
            v4f acc[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) { acc[t] = v4f{0.f, 0.f, 0.f, 0.f}; asm volatile("" : "+v"(acc[t])); }
            for (int kg = wave; kg < nkg; kg += NW) {
                if (kg != wave) {
                    grp_load<LAYOUT>(a.w1, grp.e, j0, kg, lane, A[0], sr[0]);
                    grp_load<LAYOUT>(a.w1, grp.e, j0 + 16, kg, lane, A[1], sr[1]);
                    grp_load<LAYOUT>(a.w3, grp.e, j0, kg, lane, A[2], sr[2]);
                    grp_load<LAYOUT>(a.w3, grp.e, j0 + 16, kg, lane, A[3], sr[3]);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) grp_fix<LAYOUT>(A[t], sr[t], lane, sa[t]);
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const int step = kg * 4 + s;
                    if (step >= steps) break;
                    const XOp xo = load_x(xr, xsr, step, lane);
#pragma unroll
                    for (int t = 0; t < 4; ++t) acc[t] = mfma_exact_step(s, A[t][s], xo, acc[t], sa[t]);
                }
            }
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int v = 0; v < 4; ++v) red[wave][t][v][lane] = acc[t][v];
        } else {
            // ---- nine or ten K groups (hidden width up to 5120): the (tile, K group) units are dealt so that every wave streams
            // four or five of them at once.  Wave w owns tile w % 4 and the sums of slots q, q + 2, q + 4, q + 6 (q = w / 4); slot
            // s is K group s followed, in the same accumulator, by K group s + 8: the order in which a wave that walks K groups
            // w, w + 8 adds them, so the sums are the same bits.
            const int t = wave & 3, q = wave >> 2;
            const bool tail = q + NW < nkg;
            const WMat& m = t < 2 ? a.w1 : a.w3;
            const int row0 = j0 + 16 * (t & 1);
            // Here a wave multiplies one tile with four or five K groups, so converting its activations itself would cost as many
            // converts again as its weights do: where the rows fit, the block stages them as finished bf16 operands (thread = half a
            // 32-block of a row, 16 values: act_quant or the caller's codes, then code x 2^scale; the two halves are lane neighbours),
            // else as codes.  The same values either way.  The first round of pieces is requested AHEAD of the weight rows: a wave's
            // loads return in issue order, so pieces requested behind them would arrive with the last weight row, and the barrier
            // below would hold every wave's multiplies until the slowest wave's weights were there.
            const bool xbf = (size_t)a.R * (2 * H + 16) <= XBF_BYTES;
            const int xbs = 2 * H + 16;                    // row stride of the bf16 rows
            const int nh = H >> 4, npieces = grp.n * nh;
            struct XPiece { uint4 a, b; uint32_t sb; int r, hb; bool live; };
            auto piece_fetch = [&](int u0) {
                XPiece p;
                p.live = u0 + tid < npieces;               // a round's spare threads load the last piece again and store nothing
                const int u = p.live ? u0 + tid : npieces - 1;
                // (the first round ahead of the weight requests without a division: more than 256 pieces a row in this branch, 512 threads)
                p.r = u0 == 0 ? (u >= nh ? 1 : 0) : u / nh; p.hb = u - p.r * nh;
                const int tok = rows[p.r] / a.TT;
                if constexpr (!QUANT) {
                    p.a = *(const uint4*)((const uint8_t*)a.x + (int64_t)tok * H + p.hb * 16);
                    p.b = p.a;
                    p.sb = a.xs[(int64_t)tok * (H >> 5) + (p.hb >> 1)];
                } else {
                    const uint4* px = (const uint4*)((const uint16_t*)a.x + (int64_t)tok * H + p.hb * 16);
                    p.a = px[0]; p.b = px[1]; p.sb = 0u;
                }
                return p;
            };
            auto piece_put = [&](const XPiece& p) {
                uint4 cw;
                uint32_t sb;
                if constexpr (!QUANT) { cw = p.a; sb = p.sb; }
                else {
                    const uint4 r0 = p.a, r1 = p.b;
                    auto lo16 = [](uint32_t w) { return __uint_as_float(w << 16); };
                    auto hi16 = [](uint32_t w) { return __uint_as_float(w & 0xffff0000u); };
                    auto amax8 = [&](const uint4& q4) {
                        return fmaxf(fmaxf(fmaxf(fabsf(lo16(q4.x)), fabsf(hi16(q4.x))), fmaxf(fabsf(lo16(q4.y)), fabsf(hi16(q4.y)))),
                                     fmaxf(fmaxf(fabsf(lo16(q4.z)), fabsf(hi16(q4.z))), fmaxf(fabsf(lo16(q4.w)), fabsf(hi16(q4.w)))));
                    };
                    float am = fmaxf(amax8(r0), amax8(r1));
                    am = fmaxf(am, lane_xor<1>(am, lane));
                    sb = aq_scale(am);
                    cw = make_uint4(aq_word4(lo16(r0.x), hi16(r0.x), lo16(r0.y), hi16(r0.y), sb), aq_word4(lo16(r0.z), hi16(r0.z), lo16(r0.w), hi16(r0.w), sb),
                                    aq_word4(lo16(r1.x), hi16(r1.x), lo16(r1.y), hi16(r1.y), sb), aq_word4(lo16(r1.z), hi16(r1.z), lo16(r1.w), hi16(r1.w), sb));
                }
                const float sc = e8m0_to_f32(sb & 0xffu);
                const uint32_t w[4] = {cw.x, cw.y, cw.z, cw.w};
                unsigned char* d = extra + (size_t)p.r * xbs + p.hb * 32;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    bf2 v[4];
                    v[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j], sc, false); v[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j], sc, true);
                    v[2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j + 1], sc, false); v[3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j + 1], sc, true);
                    uint4 w4; __builtin_memcpy(&w4, v, 16);
                    if (p.live) *(uint4*)(d + 16 * j) = w4;
                }
            };
            const XPiece first = piece_fetch(0);           // (no branch around it: valid addresses whichever way the rows are staged)
            v4i A[5][4];
            GrpScale sa[5];                                // all five requested at once; each becomes an operand when its unit is multiplied
            grp_load<LAYOUT>(m, grp.e, row0, q, lane, A[0], sa[0]);
            if (tail) grp_load<LAYOUT>(m, grp.e, row0, q + NW, lane, A[4], sa[4]);
            // The other three units are requested once these have arrived.  Measured, not derived (the memory system serves everything
            // requested at once by fair share, and the exchanges queue behind all of it): all five at once 35.6 us per layer at one
            // row of the hidden-5120 shape against 33.9 this way; the first alone and then four 34.6.
#pragma unroll
            for (int s = 0; s < 4; ++s) asm volatile("" : "+v"(A[0][s]));
            if (tail) {
#pragma unroll
                for (int s = 0; s < 4; ++s) asm volatile("" : "+v"(A[4][s]));
            }
            grp_load<LAYOUT>(m, grp.e, row0, q + 2, lane, A[1], sa[1]);
            grp_load<LAYOUT>(m, grp.e, row0, q + 4, lane, A[2], sa[2]);
            grp_load<LAYOUT>(m, grp.e, row0, q + 6, lane, A[3], sa[3]);
            if (xbf) {
                piece_put(first);
                for (int u0 = NT; u0 < npieces; u0 += NT) piece_put(piece_fetch(u0));
            } else stage_x(std::integral_constant<bool, !QUANT>{});
            __syncthreads();                               // a wave multiplies K groups that other waves staged
            TRACE(2);
            const uint8_t* xr = xql + (size_t)rc * H;
            const uint8_t* xsr = xsl + (size_t)rc * (H >> 5);
            const unsigned char* xb = extra + (size_t)rc * xbs + 64 * rg;
            auto unit = [&](v4i (&Au)[4], const GrpScale& sru, int kg, v4f acc) {
                uint32_t sau;
                grp_fix<LAYOUT>(Au, sru, lane, sau);
                if (xbf) {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const int step = kg * 4 + s;
                        if (step >= steps) break;
                        const float sc = e8m0_to_f32((sau >> (8 * s)) & 0xffu);
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            bf8v b;
                            { const uint4 w4 = *(const uint4*)(xb + step * 256 + 16 * j); __builtin_memcpy(&b, &w4, 16); }
                            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_operand((uint32_t)Au[s][j], sc), b, acc, 0, 0, 0);
                        }
                    }
                } else {
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const int step = kg * 4 + s;
                        if (step >= steps) break;
                        acc = mfma_exact_step(s, Au[s], load_x(xr, xsr, step, lane), acc, sau);
                    }
                }
                return acc;
            };
            auto put = [&](int slot, const v4f& acc) {
#pragma unroll
                for (int v = 0; v < 4; ++v) red[slot][t][v][lane] = acc[v];
            };
            v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
            asm volatile("" : "+v"(acc));
            acc = unit(A[0], sa[0], q, acc);
            if (tail) acc = unit(A[4], sa[4], q + NW, acc);
            put(q, acc);
#pragma unroll
            for (int j = 1; j < 4; ++j) {
                acc = v4f{0.f, 0.f, 0.f, 0.f};
                asm volatile("" : "+v"(acc));
                acc = unit(A[j], sa[j], q + 2 * j, acc);
                put(q + 2 * j, acc);
            }
        }
        TRACE(3);
        __syncthreads();
        TRACE(4);
        // epilogue: thread (wave = (tp, v), lane = (c, rg)) owns feature j0 + 16 tp + 4 rg + v of column c
        const int tp = wave >> 2, v = wave & 3;
        float gsum = 0.f, usum = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) { gsum += red[w][tp][v][lane]; usum += red[w][2 + tp][v][lane]; }
        const float gt = fminf(bf16_round(gsum), 10.f);
        const float up = fminf(fmaxf(bf16_round(usum), -10.f), 10.f);
        const float yv = bf16_round(silu(gt) * up * wgt);
        float am = fabsf(yv);
        am = fmaxf(am, lane_xor<16>(am, lane));
        am = fmaxf(am, lane_xor<32>(am, lane));
        if (rg == 0) amx[wave][c] = am;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < NW; ++w) am = fmaxf(am, amx[w][c]);
        const uint32_t e = aq_scale(am);
        ((unsigned char*)hbw[c])[16 * tp + 4 * rg + v] = (unsigned char)aq_byte(yv, e);
        if (wave == 0 && rg == 0) he[c] = e;
        __syncthreads();
        // ---- hand the rows' 32 codes + scale to every column block's copy of h (device-coherent: the readers sit on all XCDs)
        // eight threads per column block (one code word each) and one thread per column block for the scale word, row after row:
        // no index arithmetic beyond shifts on the way out
        for (int cc = 0; cc < grp.n; ++cc) {
            const int pr = rows[cc];
            const uint4 w4 = *(const uint4*)&hbw[cc][4 * (tid & 1)];            // thread = (column block, half of the row's 32 code bytes)
            const v4i v = v4i{(int)(w4.x == EMPTY ? 0xffffff7fu : w4.x), (int)(w4.y == EMPTY ? 0xffffff7fu : w4.y), (int)(w4.z == EMPTY ? 0xffffff7fu : w4.z),
                              (int)(w4.w == EMPTY ? 0xffffff7fu : w4.w)};
            for (int q = tid >> 1; q < a.NBD; q += NT / 2) st_dev128(a.hc + ((int64_t)q * a.P + pr) * (I >> 2) + jb * 8 + 4 * (tid & 1), v);
            for (int q = tid; q < a.NBD; q += NT) st_dev32(a.hsw + ((int64_t)q * a.P + pr) * (I >> 5) + jb, he[cc]);
        }
        TRACE(5);
    }
    // ==================================================================== stage 2
    if (gd.n == 0) return;
    const Group grp = gd;
    const int* rows = rowsD;
    const int nb = bi, g = grpi - 1;
    const int sub = wave >> 2, kw = wave & 3;              // 32-column half of the block, K group within a round
    const int n0 = nb * DC + sub * 32;
    const int steps = I >> 7, nkg = (steps + 3) >> 2;
    v4i A[2][4];
    GrpScale sr[2];
    uint32_t sa[2];
    {
        const int kg = min(kw, nkg - 1);
        grp_load<LAYOUT>(a.w2, grp.e, n0, kg, lane, A[0], sr[0]);
        grp_load<LAYOUT>(a.w2, grp.e, n0 + 16, kg, lane, A[1], sr[1]);
    }
    TRACE(6);
    __builtin_amdgcn_s_setprio(0);                         // waiting: the stage-1 waves of the CU's other block go first
    // token rows of this item that this block sums: those whose other experts all belong to earlier items
    if (a.R == 1) { if (tid == 0) comb[0] = g == a.P - 1; }
    else {
        if (tid < grp.n) comb[tid] = 1;
        __syncthreads();
        const int fo = rows[0];
        for (int u = tid; u < grp.n * a.TT; u += NT) {
            const int i = u / a.TT, k = u % a.TT, e = sidx[(rows[i] / a.TT) * a.TT + k];
            bool seen = false;
            for (int q = 0; q <= fo; ++q) seen |= sidx[q] == e;
            if (!seen) comb[i] = 0;
        }
    }
    if (tid == 0) misc[2] = 1;
    __syncthreads();
    // the residual of the token row this wave sums later, requested ahead of the wait (a late request would queue behind
    // the other blocks' weight rows)
    float base = 0.f;
    if (wave < grp.n && comb[wave] && a.add) base = a.add[(int64_t)(rows[wave] / a.TT) * H + nb * DC + lane];
    // The summing waves look at the workspace's error flag as they start: it is sticky, so a wait that expired in an EARLIER call (which
    // left words behind that are not idle) turns every later call's output into NaN until the workspace is prepared again.
    int stale = 0;
    if (wave < grp.n && comb[wave]) stale = __hip_atomic_load(a.err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // a failed call must not leave the caller's old bytes in y: the columns this wave owns become NaN
    auto poison = [&]() {
        if (wave < grp.n && comb[wave]) {
            const int64_t o = (int64_t)(rows[wave] / a.TT) * H + nb * DC + lane;
            if (a.obf16) ((uint16_t*)a.y)[o] = 0x7fc0u; else a.y[o] = __uint_as_float(0x7fc00000u);
        }
    };
    // B operands of a round in LDS: [kw][step][g4][row < n] x (8 code words + 1 scale word), written by the waves of half 0
    uint32_t* hl = (uint32_t*)extra;
    const bool valid = c < grp.n;
    const int rc = valid ? c : 0;
    v4f acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) { acc[t] = v4f{0.f, 0.f, 0.f, 0.f}; asm volatile("" : "+v"(acc[t])); }
    for (int rd = 0; rd * 4 < nkg; ++rd) {
        const int kg = rd * 4 + kw;
        const bool have = kg < nkg;
        if (rd > 0) {
            __syncthreads();                               // the previous round's operands have been read
            if (have) {
                grp_load<LAYOUT>(a.w2, grp.e, n0, kg, lane, A[0], sr[0]);
                grp_load<LAYOUT>(a.w2, grp.e, n0 + 16, kg, lane, A[1], sr[1]);
            }
        }
        if (sub == 0 && have) {
            // cheap wait first (one scale word per 32-block of the K group, first row), then every word of this lane
            const int nblk = min(16, (I >> 5) - kg * 16);
            int spins = 0;
            for (;;) {
                const uint32_t v = lane < nblk ? ld_dev32(a.hsw + ((int64_t)nb * a.P + rows[0]) * (I >> 5) + kg * 16 + lane) : 0u;
                if (__builtin_amdgcn_ballot_w64(v == EMPTY) == 0 || ++spins >= SPIN_MAX) break;
                __builtin_amdgcn_s_sleep(16);
            }
            if (valid) {
                const int64_t row = (int64_t)nb * a.P + rows[c];
                uint32_t* pc = a.hc + row * (I >> 2);
                uint32_t* ps = a.hsw + row * (I >> 5);
                uint64_t w[4][4];
                uint32_t sw[4];
                bool ok = false;
                for (spins = 0; spins < SPIN_MAX && !ok; ++spins) {
                    ok = true;
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        const int step = min(kg * 4 + s, steps - 1);
                        w[s][0] = ld_dev64(pc + step * 32 + rg * 4); w[s][1] = ld_dev64(pc + step * 32 + rg * 4 + 2);
                        w[s][2] = ld_dev64(pc + step * 32 + 16 + rg * 4); w[s][3] = ld_dev64(pc + step * 32 + 16 + rg * 4 + 2);
                        sw[s] = ld_dev32(ps + step * 4 + rg);
                    }
#pragma unroll
                    for (int s = 0; s < 4; ++s) {
                        ok = ok && sw[s] != EMPTY;
#pragma unroll
                        for (int i = 0; i < 4; ++i) ok = ok && (uint32_t)w[s][i] != EMPTY && (uint32_t)(w[s][i] >> 32) != EMPTY;
                    }
                    if (!ok) __builtin_amdgcn_s_sleep(1);
                }
                if (!ok) misc[2] = 0;
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const int step = kg * 4 + s;
                    if (step < steps && ok) {
                        st_dev64(pc + step * 32 + rg * 4, EMPTY2); st_dev64(pc + step * 32 + rg * 4 + 2, EMPTY2);
                        st_dev64(pc + step * 32 + 16 + rg * 4, EMPTY2); st_dev64(pc + step * 32 + 16 + rg * 4 + 2, EMPTY2);
                        st_dev32(ps + step * 4 + rg, EMPTY);
                    }
                    uint32_t* o = hl + (((kw * 4 + s) * 4 + rg) * RMAX + c) * 9;
#pragma unroll
                    for (int i = 0; i < 4; ++i) { o[2 * i] = (uint32_t)w[s][i]; o[2 * i + 1] = (uint32_t)(w[s][i] >> 32); }
                    o[8] = sw[s];
                }
            }
        }
        __syncthreads();
        TRACE(7);
        if (rd == 0) __builtin_amdgcn_s_setprio(3);        // from here on this block is the critical path
        if (have && misc[2]) {
            grp_fix<LAYOUT>(A[0], sr[0], lane, sa[0]);
            grp_fix<LAYOUT>(A[1], sr[1], lane, sa[1]);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int step = kg * 4 + s;
                if (step >= steps) break;
                const uint32_t* o = hl + (((kw * 4 + s) * 4 + rg) * RMAX + rc) * 9;
                const v8i b = v8i{(int)o[0], (int)o[1], (int)o[2], (int)o[3], (int)o[4], (int)o[5], (int)o[6], (int)o[7]};
                const uint32_t sb = o[8];
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[t] = mfma_group_step(s, A[t][s], b, acc[t], sa[t], sb);
            }
        }
    }
    TRACE(8);
    if (!misc[2]) { if (tid == 0) atomicExch(a.err, 1); poison(); return; }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wave][t][v][lane] = acc[t][v];
    __syncthreads();
    // thread (wave = (sub, v), lane) sums element v of both tiles over the four K waves of its half, in wave order
    if (valid) {
        const int v = kw;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < 4; ++w) s += red[sub * 4 + w][t][v][lane];
            uint32_t u = __float_as_uint(s);
            if (u == EMPTY) u = 0x7fc00000u;
            float* p = a.yd + (int64_t)rows[c] * H + n0 + 16 * t + 4 * rg + v;
            if (LOCAL) *(uint32_t*)p = u; else st_dev32(p, u);
        }
    }
    TRACE(9);
    // ---- the token rows this block sums: wave i takes item row i, lane = column
    if (wave < grp.n && comb[wave]) {
        const int tok = rows[wave] / a.TT, col = nb * DC + lane;
        float* py[TTMAX];
#pragma unroll
        for (int k = 0; k < TTMAX; ++k) py[k] = a.yd + (int64_t)(tok * a.TT + (k < a.TT ? k : 0)) * H + col;
        uint32_t o[TTMAX];
        int spins = 0;
        bool ok;
        for (;;) {
            asm volatile("" ::: "memory");
#pragma unroll
            for (int k = 0; k < TTMAX; ++k) o[k] = LOCAL ? ld_l2(py[k]) : ld_dev32(py[k]);
            ok = true;
#pragma unroll
            for (int k = 0; k < TTMAX; ++k) ok = ok && o[k] != EMPTY;
            if (__builtin_amdgcn_ballot_w64(!ok) == 0) { ok = true; break; }
            if (++spins >= SPIN_MAX) { ok = false; break; }
            __builtin_amdgcn_s_sleep(1);
        }
        if (ok && !stale) {
#pragma unroll
            for (int k = 0; k < TTMAX; ++k) { if (LOCAL) *(uint32_t*)py[k] = EMPTY; else st_dev32(py[k], EMPTY); }
            float accs = base;                             // add + shared experts, then the routed experts in slot order
#pragma unroll
            for (int k = 0; k < TTMAX; ++k) if (k >= a.topk && k < a.TT) accs += __uint_as_float(o[k]);
            float s = 0.f;
#pragma unroll
            for (int k = 0; k < TTMAX; ++k) if (k < a.topk) s += __uint_as_float(o[k]);
            if (a.obf16) ((uint16_t*)a.y)[(int64_t)tok * H + col] = f32_to_bf16(accs + s);
            else a.y[(int64_t)tok * H + col] = accs + s;
        } else { poison(); if (lane == 0) atomicExch(a.err, 1); }
    }
    TRACE(10);
}

__global__ void fill_kernel(uint32_t* p, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = i < HEAD / 4 ? 0u : EMPTY;
}

struct FPlan { int TT, ET, P, Gmax, NJ, NBD, GS, nblocks; size_t hc, hsw, yd, total, lds; };
FPlan fplan(int R, int H, int I, int topk, int E, int n_shared)
{
    FPlan p;
    p.TT = topk + n_shared; p.ET = E + n_shared;
    p.P = R * p.TT;
    p.Gmax = p.P < p.ET ? p.P : p.ET;
    p.NJ = I / 32; p.NBD = H / DC;
    p.GS = ((p.NJ > p.NBD ? p.NJ : p.NBD) + NXCD - 1) / NXCD * NXCD;
    p.nblocks = (p.Gmax + 1) * p.GS;
    size_t o = HEAD;
    auto take = [&](size_t n) { const size_t q = o; o += align256(n); return q; };
    p.hc = take((size_t)p.NBD * p.P * I);
    p.hsw = take((size_t)p.NBD * p.P * (I / 32) * 4);
    p.yd = take((size_t)p.P * H * 4);
    p.total = o;
    const size_t xb = (size_t)R * (2 * H + 16);           // nine or ten K groups: the rows as bf16 where they fit
    const size_t lu = ((H + 511) / 512 > NW && (H + 511) / 512 <= NW + 2 && xb <= XBF_BYTES) ? xb : (size_t)R * H + (size_t)R * (H / 32), ld = (size_t)16 * 4 * RMAX * 9 * 4;
    p.lds = RED_BYTES + ((lu > ld ? lu : ld) + 15) / 16 * 16;
    return p;
}

int g_force_local = -1;               // diagnostics: 1 / 0 force the same-XCD / the device-coherent exchange, -1 = by the placement check

template <int LAYOUT, bool QUANT>
int launch(const MArgs& a, const FPlan& p, hipStream_t st)
{
    const dim3 grid(p.nblocks), blk(NT);
    if (g_force_local >= 0 ? g_force_local == 1 : xcd_placement() == 1) {
        static bool attr = false;
        if (!attr) { (void)hipFuncSetAttribute((const void*)mx_fused_kernel<LAYOUT, QUANT, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024); attr = true; }
        mx_fused_kernel<LAYOUT, QUANT, true><<<grid, blk, p.lds, st>>>(a);
    } else {
        static bool attr = false;
        if (!attr) { (void)hipFuncSetAttribute((const void*)mx_fused_kernel<LAYOUT, QUANT, false>, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024); attr = true; }
        mx_fused_kernel<LAYOUT, QUANT, false><<<grid, blk, p.lds, st>>>(a);
    }
    return launch_status();
}

}  // namespace

bool mx_fused_ok(int R, int H, int I, int topk, int E, int n_shared)
{
    if (R < 1 || R > RMAX || topk + n_shared > TTMAX || H % DC || I % 128 || H % 128) return false;
    const FPlan p = fplan(R, H, I, topk, E, n_shared);
    return p.lds <= 96 * 1024;
}
size_t mx_fused_ws_bytes(int R, int H, int I, int topk, int E, int n_shared) { return fplan(R, H, I, topk, E, n_shared).total; }

// every exchanged word of a workspace idle, its error flag clear
int mx_fused_ws_prepare(void* ws, size_t bytes, hipStream_t st)
{
    const int64_t n = (int64_t)(bytes / 4);
    if (n > 0) fill_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>((uint32_t*)ws, n);
    return launch_status();
}

// x: bf16 [R, H] when xs == nullptr (quantised inside), else E4M3 [R, H] with scales xs.  clean = the workspace is idle
// (prepared once and only used by this path since).
int mx_fused_launch(const void* x, const void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1, const void* w3, const void* s3,
                    const void* w2, const void* s2, int layout, int H, int I, int topk, int E, int n_shared, const float* add, float* y, void* ws, int clean,
                    hipStream_t st, int obf16)
{
    const FPlan p = fplan(R, H, I, topk, E, n_shared);
    char* b = (char*)ws;
    MArgs a;
    a.x = x; a.xs = (const uint8_t*)xs; a.idx = idx; a.rw = rw;
    const int64_t ET = E + n_shared;
    a.w1 = WMat{(const uint8_t*)w1, (const uint8_t*)s1, I, H, ET * I / 8}; a.w3 = WMat{(const uint8_t*)w3, (const uint8_t*)s3, I, H, ET * I / 8};
    a.w2 = WMat{(const uint8_t*)w2, (const uint8_t*)s2, H, I, ET * H / 8};
    a.add = add; a.y = y;
    a.hc = (uint32_t*)(b + p.hc); a.hsw = (uint32_t*)(b + p.hsw); a.yd = (float*)(b + p.yd); a.err = (int*)b;
    a.R = R; a.TT = p.TT; a.topk = topk; a.E = E; a.P = p.P; a.Gmax = p.Gmax; a.H = H; a.I = I; a.NJ = p.NJ; a.NBD = p.NBD; a.GS = p.GS;
    a.trace = g_trace;
    a.obf16 = obf16;
    if (!clean && !ws_is_prepared(ws, p.total)) {          // idle exchange words: promised by the caller or known from the workspace's own *_ws_init call
        const int rc = mx_fused_ws_prepare(ws, p.total, st);
        if (rc) return rc;
    }
    const bool quant = xs == nullptr;
    switch (layout) {
        case L_T16: return quant ? launch<L_T16, true>(a, p, st) : launch<L_T16, false>(a, p, st);
        case L_NATURAL: return quant ? launch<L_NATURAL, true>(a, p, st) : launch<L_NATURAL, false>(a, p, st);
        case L_PACK8: return quant ? launch<L_PACK8, true>(a, p, st) : launch<L_PACK8, false>(a, p, st);
        case L_MX8: return quant ? launch<L_MX8, true>(a, p, st) : launch<L_MX8, false>(a, p, st);
        case L_MX8S2: return quant ? launch<L_MX8S2, true>(a, p, st) : launch<L_MX8S2, false>(a, p, st);
    }
    return 1;
}

// diagnostics: device buffer of 16 time stamps (100 MHz) per block of the next launches, or null (recorded by builds with
// -DSPK_MX_TRACE only)
extern "C" __attribute__((visibility("default"))) void spark_debug_mx_trace(long long* buf) { g_trace = buf; }
// diagnostics: force the exchange mode of the single-launch path (1 same-XCD through L2, 0 device-coherent, -1 as the placement check found)
extern "C" __attribute__((visibility("default"))) void spark_debug_mx_local(int v) { g_force_local = v; }

}  // namespace mx
}  // namespace spk
