// Routed MXFP4 experts (DeepSeek-style MoE layer) for gfx950.
//
//   y[r] = add[r] + sum_shared expert_s(x[r]) + sum_k (slot order) w2_e . q(bf16(silu(min(bf16(w1_e . xq_r), 10)) *
//          clamp(bf16(w3_e . xq_r), +-10) * rw[r][k]))          e = idx[r][k], q = act_quant (E4M3 + UE8M0 per 32)
//
// Semantics: reference engine-rs/shim/ds41_moe.cu:1-24 and ds41_mx.cu:1-16,95-317,1436-1523 (ds41_moe_mx_ex),
// reference engine-rs/src/ds41/kern.rs:1116-1133 (moe_ref).
//
// MI355X design.  A lane's piece of the weight stream is 16 contiguous bytes = the 32 E2M1 codes of one scale block of one row.
// The down product runs on the block-scaled matrix unit, v_mfma_scale_f32_16x16x128_f8f6f4, with A = 16 weight rows in E2M1 (one
// E8M0 scale per lane = per row and 32-block, exactly the stored format) and B = up to 16 token rows in E4M3 with their UE8M0
// scales: the packed weights go from the 128-bit load straight into the instruction.  That instruction aligns the products of a
// 32-block to the block's largest and drops what lies about 14 bits under it (1e-5 of a sum), which is harmless for the down
// product but not for gate / up, whose sums are rounded to bf16 and quantised: those run on v_mfma_f32_16x16x32_bf16 with both
// operands converted exactly (moe_mxfp4.hpp: mfma_exact_step), four instructions per 128-wide step, dword j of the same 16 bytes
// feeding instruction j.
// Operand layout measured on gfx950: A/B lane l = row/column l % 16, K group g = l / 16.  An E2M1 operand holds
// k = 32 g + e (nibble e of its 16 bytes); an E4M3 operand holds k = 16 g + e in registers 0-3 and k = 64 + 16 g + e in
// registers 4-7; the scale byte of lane l applies to logical block g (k in [32 g, 32 g + 32)); D lane l = column l % 16,
// rows 4 (l / 16) + {0..3}.  v_mfma_f32_16x16x32_bf16: lane l = row/column l % 16, k = 8 (l / 16) + {0..7}, D as above.
//
// Weight storage ("T16" records, written once by spark_mxfp4_prepack): per 16 rows and 512-wide K group one record of
// 4352 bytes = 4 steps x (64 lanes x 16 bytes of codes) + 64 lanes x 4 scale bytes (byte s = step s).  A wave streams a
// record with four 16-byte loads and one 4-byte load per lane, all contiguous.
#include "moe_mxfp4.hpp"
#include "runtime.hpp"
#include <cstdlib>

using namespace spk;
using namespace spk::mx;

namespace {

struct Item { int e, off, n, pad; };

#ifdef SPK_MX_TRACE
__device__ long long* g_gtrace = nullptr;     // 16 stamps per block of up_res_kernel
#define GTRACE(i) do { if (g_gtrace && threadIdx.x == 0) { const int64_t bb = (int64_t)blockIdx.y * gridDim.x + blockIdx.x; if (bb < 32768) g_gtrace[bb * 16 + (i)] = wall_clock64(); } } while (0)
#else
#define GTRACE(i) do { } while (0)
#endif

constexpr int EMAXG = 2048;            // experts the grouping kernel can hold
constexpr int UP_WAVES = 8, DN_WAVES = 4;



// ---------------------------------------------------------------- grouping of the (row, expert) pairs by expert
// Pairs per row: topk routed (idx, rw) followed by n_shared shared experts (ids E .. E + n_shared - 1, weight 1).
// Items = at most GR compact rows of one expert.  One workgroup.  reference ds41_mx.cu:95-125.
__global__ __launch_bounds__(1024) void group_kernel(const int64_t* __restrict__ idx, const float* __restrict__ rw, int R, int topk, int n_shared, int E,
                                                    int GR, int* __restrict__ G, Item* __restrict__ items, int* __restrict__ pairmap, int* __restrict__ prow,
                                                    float* __restrict__ pw, int* __restrict__ counters, int ncounters, int* __restrict__ geoff,
                                                    int* __restrict__ gfill)
{
    __shared__ int cnt[EMAXG], fill[EMAXG], eoff[EMAXG], ioff[EMAXG];
    __shared__ int wsum[2][16];
    const int ET = E + n_shared, TT = topk + n_shared, P = R * TT, tid = threadIdx.x;
    for (int i = tid; i < ncounters; i += 1024) counters[i] = 0;
    for (int e = tid; e < ET; e += 1024) { cnt[e] = 0; fill[e] = 0; }
    __syncthreads();
    // eight pairs per thread at a time: their index loads are in flight together (one workgroup has no other latency hiding)
    for (int p0 = tid; p0 < P; p0 += 8 * 1024) {
        int ev[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int p = min(p0 + u * 1024, P - 1), r = p / TT, k = p % TT;
            ev[u] = k < topk ? clamp_expert((int)idx[(int64_t)r * topk + k], E) : E + (k - topk);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (p0 + u * 1024 < P) atomicAdd(&cnt[ev[u]], 1);
    }
    __syncthreads();
    // exclusive scans of rows and items over the experts (two experts per thread)
    int c0 = 0, c1 = 0;
    if (2 * tid < ET) c0 = cnt[2 * tid];
    if (2 * tid + 1 < ET) c1 = cnt[2 * tid + 1];
    const int n0 = (c0 + GR - 1) / GR, n1 = (c1 + GR - 1) / GR;
    int rs = c0 + c1, is = n0 + n1;
    const int lane = tid & 63, wv = tid >> 6;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int a = __shfl_up(rs, o, 64), b = __shfl_up(is, o, 64);
        if (lane >= o) { rs += a; is += b; }
    }
    if (lane == 63) { wsum[0][wv] = rs; wsum[1][wv] = is; }
    __syncthreads();
    int rbase = 0, ibase = 0;
    for (int w = 0; w < wv; ++w) { rbase += wsum[0][w]; ibase += wsum[1][w]; }
    const int rex = rbase + rs - (c0 + c1), iex = ibase + is - (n0 + n1);
    if (2 * tid < ET) { eoff[2 * tid] = rex; ioff[2 * tid] = iex; }
    if (2 * tid + 1 < ET) { eoff[2 * tid + 1] = rex + c0; ioff[2 * tid + 1] = iex + n0; }
    if (tid == 1023) *G = ibase + is;
    __syncthreads();
    for (int e = tid; e < ET; e += 1024) {
        const int c = cnt[e];
        for (int j = 0; j * GR < c; ++j) items[ioff[e] + j] = Item{e, eoff[e] + j * GR, min(GR, c - j * GR), 0};
        if (geoff) { geoff[e] = eoff[e]; gfill[e] = 0; }
    }
    if (geoff) return;                                     // a large call: scatter_kernel hands out the rows, over many CUs
    for (int p0 = tid; p0 < P; p0 += 8 * 1024) {
        int ev[8];
        float wv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int p = min(p0 + u * 1024, P - 1), r = p / TT, k = p % TT;
            ev[u] = k < topk ? clamp_expert((int)idx[(int64_t)r * topk + k], E) : E + (k - topk);
            wv[u] = k < topk ? rw[(int64_t)r * topk + k] : 1.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int p = p0 + u * 1024;
            if (p < P) {
                const int pos = eoff[ev[u]] + atomicAdd(&fill[ev[u]], 1);
                pairmap[p] = pos;
                prow[pos] = p;
                pw[pos] = wv[u];
            }
        }
    }
}

// The second sweep of a large call: one workgroup's scattered stores go through one CU's memory pipeline (most of that kernel's
// 34 us at 14336 pairs); here a workgroup per 1024 pairs ranks them per expert in LDS, reserves each expert's rows with one atomic on
// the fill counts in memory, and stores.
__global__ __launch_bounds__(1024) void scatter_kernel(const int64_t* __restrict__ idx, const float* __restrict__ rw, int R, int topk, int n_shared, int E,
                                                      const int* __restrict__ geoff, int* __restrict__ gfill, int* __restrict__ pairmap, int* __restrict__ prow,
                                                      float* __restrict__ pw)
{
    __shared__ int lcnt[EMAXG], lbase[EMAXG];
    const int ET = E + n_shared, TT = topk + n_shared, P = R * TT, tid = threadIdx.x, p = (int)blockIdx.x * 1024 + tid;
    for (int e = tid; e < ET; e += 1024) lcnt[e] = 0;
    __syncthreads();
    int ev = 0, rank = 0;
    float wv = 1.0f;
    if (p < P) {
        const int r = p / TT, k = p % TT;
        ev = k < topk ? clamp_expert((int)idx[(int64_t)r * topk + k], E) : E + (k - topk);
        if (k < topk) wv = rw[(int64_t)r * topk + k];
        rank = atomicAdd(&lcnt[ev], 1);
    }
    __syncthreads();
    for (int e = tid; e < ET; e += 1024) { const int n = lcnt[e]; lbase[e] = n ? geoff[e] + atomicAdd(&gfill[e], n) : 0; }
    __syncthreads();
    if (p < P) {
        const int pos = lbase[ev] + rank;
        pairmap[p] = pos;
        prow[pos] = p;
        pw[pos] = wv;
    }
}

// ---------------------------------------------------------------- gate / up + SwiGLU + act_quant -> hq [P, I], hs [P, I/32]
// grid (I / 32, Gmax), 8 waves: wave w takes K groups w, w + 8, ... of the 32 gate and 32 up rows j0 .. j0 + 31 for the
// item's rows (16 per MFMA column group); the partial tiles are summed through LDS in wave order.
template <int LAYOUT>
__global__ __launch_bounds__(64 * UP_WAVES) void up_kernel(const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, WMat w1, WMat w3, int H, int I, int TT,
                                                           const int* __restrict__ G, const Item* __restrict__ items, const int* __restrict__ prow,
                                                           const float* __restrict__ pw, uint8_t* __restrict__ hq, uint8_t* __restrict__ hs)
{
    __shared__ float red[UP_WAVES][4][4][64];      // [wave][tile: g0 g1 u0 u1][v][lane]
    __shared__ float amx[UP_WAVES][16];
    if ((int)blockIdx.y >= *G) return;
    const Item it = items[blockIdx.y];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, rg = lane >> 4;
    const int j0 = blockIdx.x * 32;
    const int steps = H >> 7, nkg = (steps + 3) >> 2;
    // a wave with one K group keeps its weight rows in registers for every group of 16 item rows: an item's weights are
    // streamed once however many token rows it has
    const bool resident = nkg <= UP_WAVES;
    v4i a[4][4];
    uint32_t sa[4];
    if (resident && wave < nkg) {
        load_group<LAYOUT>(w1, it.e, j0, wave, lane, a[0], sa[0]);
        load_group<LAYOUT>(w1, it.e, j0 + 16, wave, lane, a[1], sa[1]);
        load_group<LAYOUT>(w3, it.e, j0, wave, lane, a[2], sa[2]);
        load_group<LAYOUT>(w3, it.e, j0 + 16, wave, lane, a[3], sa[3]);
    }
    for (int cg = 0; cg * 16 < it.n; ++cg) {
        const int rr = cg * 16 + c;                // compact row of this lane's column within the item
        const bool valid = rr < it.n;
        const int pos = it.off + (valid ? rr : 0);
        const int tok = prow[pos] / TT;
        const uint8_t* xr = xq + (int64_t)tok * H;
        const uint8_t* xsr = xs + (int64_t)tok * (H >> 5);
        v4f acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) { acc[t] = v4f{0.f, 0.f, 0.f, 0.f}; asm volatile("" : "+v"(acc[t])); }
        for (int kg = wave; kg < nkg; kg += UP_WAVES) {
            if (!resident) {
                load_group<LAYOUT>(w1, it.e, j0, kg, lane, a[0], sa[0]);
                load_group<LAYOUT>(w1, it.e, j0 + 16, kg, lane, a[1], sa[1]);
                load_group<LAYOUT>(w3, it.e, j0, kg, lane, a[2], sa[2]);
                load_group<LAYOUT>(w3, it.e, j0 + 16, kg, lane, a[3], sa[3]);
            }
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int step = kg * 4 + s;
                if (step >= steps) break;
                const XOp xo = load_x(xr, xsr, step, lane);
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[t] = mfma_exact_step(s, a[t][s], xo, acc[t], sa[t]);
            }
        }
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][t][v][lane] = acc[t][v];
        __syncthreads();
        // epilogue: thread (wave = (tp, v), lane = (c, rg)) owns feature j0 + 16 tp + 4 rg + v of column c
        const int tp = wave >> 2, v = wave & 3;
        float gsum = 0.f, usum = 0.f;
#pragma unroll
        for (int w = 0; w < UP_WAVES; ++w) { gsum += red[w][tp][v][lane]; usum += red[w][2 + tp][v][lane]; }
        const float wgt = valid ? pw[pos] : 0.f;
        const float gt = fminf(bf16_round(gsum), 10.f);
        const float up = fminf(fmaxf(bf16_round(usum), -10.f), 10.f);
        const float yv = bf16_round(silu(gt) * up * wgt);
        float am = fabsf(yv);
        am = fmaxf(am, __shfl_xor(am, 16, 64));
        am = fmaxf(am, __shfl_xor(am, 32, 64));
        if (rg == 0) amx[wave][c] = am;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < UP_WAVES; ++w) am = fmaxf(am, amx[w][c]);
        const uint32_t e = aq_scale(am);
        if (valid) {
            hq[(int64_t)pos * I + j0 + 16 * tp + 4 * rg + v] = (uint8_t)aq_byte(yv, e);
            if (wave == 0 && rg == 0) hs[(int64_t)pos * (I >> 5) + (j0 >> 5)] = (uint8_t)e;
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------- down: out [P, H] = h . w2_e^T
// grid (H / 32, Gmax), 4 waves: wave w takes K groups w, w + 4, ... of output rows n0 .. n0 + 31.
template <int LAYOUT>
__global__ __launch_bounds__(64 * DN_WAVES) void down_kernel(const uint8_t* __restrict__ hq, const uint8_t* __restrict__ hs, WMat w2, int H, int I,
                                                             const int* __restrict__ G, const Item* __restrict__ items, float* __restrict__ out)
{
    __shared__ float red[DN_WAVES][2][4][64];
    if ((int)blockIdx.y >= *G) return;
    const Item it = items[blockIdx.y];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15;
    const int n0 = blockIdx.x * 32;
    const int steps = I >> 7, nkg = (steps + 3) >> 2;
    const bool resident = nkg <= DN_WAVES;         // one K group per wave: its weight rows stay in registers for all item rows
    v4i a[2][4];
    uint32_t sa[2];
    if (resident && wave < nkg) {
        load_group<LAYOUT>(w2, it.e, n0, wave, lane, a[0], sa[0]);
        load_group<LAYOUT>(w2, it.e, n0 + 16, wave, lane, a[1], sa[1]);
    }
    for (int cg = 0; cg * 16 < it.n; ++cg) {
        const int rr = cg * 16 + c;
        const int pos = it.off + (rr < it.n ? rr : 0);
        const uint8_t* hr = hq + (int64_t)pos * I;
        const uint8_t* hsr = hs + (int64_t)pos * (I >> 5);
        v4f acc[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) { acc[t] = v4f{0.f, 0.f, 0.f, 0.f}; asm volatile("" : "+v"(acc[t])); }
        for (int kg = wave; kg < nkg; kg += DN_WAVES) {
            if (!resident) {
                load_group<LAYOUT>(w2, it.e, n0, kg, lane, a[0], sa[0]);
                load_group<LAYOUT>(w2, it.e, n0 + 16, kg, lane, a[1], sa[1]);
            }
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int step = kg * 4 + s;
                if (step >= steps) break;
                v8i b; uint32_t sb;
                load_b(hr, hsr, step, lane, b, sb);
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[t] = mfma_group_step(s, a[t][s], b, acc[t], sa[t], sb);
            }
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][t][v][lane] = acc[t][v];
        __syncthreads();
        // thread (wave = v, lane) sums both tiles' element v
        const int v = wave, rg = lane >> 4;
        if (rr < it.n) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < DN_WAVES; ++w) s += red[w][t][v][lane];
                out[(int64_t)pos * H + n0 + 16 * t + 4 * rg + v] = s;
            }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------- the same two products for shapes whose K groups all fit the
// block's waves (one K group per wave): the weight rows stay in registers for every group of 16 item rows, and the loop is
// software-pipelined - the next row group's activations (and the row bookkeeping of the one after) are requested right after
// this group's MFMAs have consumed their operands, so their latency hides behind the reduction and the epilogue.  Same MFMA
// and summation order as up_kernel / down_kernel: the same bits.
template <int LAYOUT>
__global__ __launch_bounds__(64 * UP_WAVES, 4) void up_res_kernel(const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, WMat w1, WMat w3, int H, int I,
                                                                  int TT, const int* __restrict__ G, const Item* __restrict__ items,
                                                                  const int* __restrict__ prow, const float* __restrict__ pw, uint8_t* __restrict__ hq,
                                                                  uint8_t* __restrict__ hs)
{
    __shared__ float red[UP_WAVES][4][4][64];      // [wave][tile: g0 g1 u0 u1][v][lane]
    __shared__ float amx[UP_WAVES][16];
    if ((int)blockIdx.y >= *G) return;
    GTRACE(0);
    const Item it = items[blockIdx.y];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, rg = lane >> 4;
    const int j0 = blockIdx.x * 32;
    const int steps = H >> 7, nkg = (steps + 3) >> 2;
    const bool active = wave < nkg;
    const int kg = active ? wave : 0;
    // rows past the item's end repeat its last row (no branch around a load); their results are not stored
    int pos = it.off + min(c, it.n - 1);
    int tok = prow[pos] / TT;
    float wgt = pw[pos];
    int posn = it.off + min(16 + c, it.n - 1);
    int tokn = prow[posn] / TT;
    float wgtn = pw[posn];
    v4i a[4][4];
    uint32_t sa[4];
    load_group<LAYOUT>(w1, it.e, j0, kg, lane, a[0], sa[0]);
    load_group<LAYOUT>(w1, it.e, j0 + 16, kg, lane, a[1], sa[1]);
    load_group<LAYOUT>(w3, it.e, j0, kg, lane, a[2], sa[2]);
    load_group<LAYOUT>(w3, it.e, j0 + 16, kg, lane, a[3], sa[3]);
    GTRACE(1);
    const int ncg = (it.n + 15) >> 4;
    for (int cg = 0; cg < ncg; ++cg) {
        v4f acc[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) { acc[t] = v4f{0.f, 0.f, 0.f, 0.f}; asm volatile("" : "+v"(acc[t])); }
        if (active) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                if (kg * 4 + s >= steps) break;
                const XOp xo = load_x(xq + (int64_t)tok * H, xs + (int64_t)tok * (H >> 5), kg * 4 + s, lane);
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[t] = mfma_exact_step(s, a[t][s], xo, acc[t], sa[t]);
            }
        }
        if (cg < 3) GTRACE(2 + cg * 4);
        // the next row group's operands, and the rows of the one after
        const int pos2 = it.off + min((cg + 2) * 16 + c, it.n - 1);
        const int tok2 = prow[pos2] / TT;
        const float wgt2 = pw[pos2];
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][t][v][lane] = acc[t][v];
        if (cg < 3) GTRACE(3 + cg * 4);
        __syncthreads();
        if (cg < 3) GTRACE(4 + cg * 4);
        // epilogue: thread (wave = (tp, v), lane = (c, rg)) owns feature j0 + 16 tp + 4 rg + v of column c
        const bool valid = cg * 16 + c < it.n;
        const int tp = wave >> 2, v = wave & 3;
        float gsum = 0.f, usum = 0.f;
#pragma unroll
        for (int w = 0; w < UP_WAVES; ++w) { gsum += red[w][tp][v][lane]; usum += red[w][2 + tp][v][lane]; }
        const float gt = fminf(bf16_round(gsum), 10.f);
        const float up = fminf(fmaxf(bf16_round(usum), -10.f), 10.f);
        const float yv = bf16_round(silu(gt) * up * (valid ? wgt : 0.f));
        float am = fabsf(yv);
        am = fmaxf(am, __shfl_xor(am, 16, 64));
        am = fmaxf(am, __shfl_xor(am, 32, 64));
        if (rg == 0) amx[wave][c] = am;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < UP_WAVES; ++w) am = fmaxf(am, amx[w][c]);
        const uint32_t e = aq_scale(am);
        if (valid) {
            hq[(int64_t)pos * I + j0 + 16 * tp + 4 * rg + v] = (uint8_t)aq_byte(yv, e);
            if (wave == 0 && rg == 0) hs[(int64_t)pos * (I >> 5) + (j0 >> 5)] = (uint8_t)e;
        }
        __syncthreads();
        pos = posn; tok = tokn; wgt = wgtn; posn = pos2; tokn = tok2; wgtn = wgt2;
    }
}

template <int LAYOUT>
__global__ __launch_bounds__(64 * DN_WAVES) void down_res_kernel(const uint8_t* __restrict__ hq, const uint8_t* __restrict__ hs, WMat w2, int H, int I,
                                                                 const int* __restrict__ G, const Item* __restrict__ items, float* __restrict__ out)
{
    __shared__ float red[DN_WAVES][2][4][64];
    if ((int)blockIdx.y >= *G) return;
    const Item it = items[blockIdx.y];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15;
    const int n0 = blockIdx.x * 32;
    const int steps = I >> 7, nkg = (steps + 3) >> 2;
    const bool active = wave < nkg;
    const int kg = active ? wave : 0;
    v4i a[2][4];
    uint32_t sa[2];
    load_group<LAYOUT>(w2, it.e, n0, kg, lane, a[0], sa[0]);
    load_group<LAYOUT>(w2, it.e, n0 + 16, kg, lane, a[1], sa[1]);
    v8i b[4];
    uint32_t sb[4];
    {
        const int pos = it.off + min(c, it.n - 1);
#pragma unroll
        for (int s = 0; s < 4; ++s) load_b(hq + (int64_t)pos * I, hs + (int64_t)pos * (I >> 5), min(kg * 4 + s, steps - 1), lane, b[s], sb[s]);
    }
    const int ncg = (it.n + 15) >> 4;
    for (int cg = 0; cg < ncg; ++cg) {
        const int rr = cg * 16 + c;
        const int pos = it.off + min(rr, it.n - 1);
        v4f acc[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) { acc[t] = v4f{0.f, 0.f, 0.f, 0.f}; asm volatile("" : "+v"(acc[t])); }
        if (active) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                if (kg * 4 + s >= steps) break;
#pragma unroll
                for (int t = 0; t < 2; ++t) acc[t] = mfma_group_step(s, a[t][s], b[s], acc[t], sa[t], sb[s]);
            }
        }
        {
            const int posn = it.off + min(rr + 16, it.n - 1);      // the next row group's operands
#pragma unroll
            for (int s = 0; s < 4; ++s) load_b(hq + (int64_t)posn * I, hs + (int64_t)posn * (I >> 5), min(kg * 4 + s, steps - 1), lane, b[s], sb[s]);
        }
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int v = 0; v < 4; ++v) red[wave][t][v][lane] = acc[t][v];
        __syncthreads();
        // thread (wave = v, lane) sums both tiles' element v
        const int v = wave, rg = lane >> 4;
        if (rr < it.n) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
                float sm = 0.f;
#pragma unroll
                for (int w = 0; w < DN_WAVES; ++w) sm += red[w][t][v][lane];
                out[(int64_t)pos * H + n0 + 16 * t + 4 * rg + v] = sm;
            }
        }
        __syncthreads();
    }
}

// ---------------------------------------------------------------- prefill: grouped GEMM over 32-row items (T16 records)
// Many rows per expert make the products above re-read every item's activation rows once per 32 output features and write the
// intermediate in single bytes; both cost more than the weight stream.  Here a block owns 32 item rows x 128 output features
// for the whole K range: the item's activation rows go through LDS one K group (512) at a time, double-buffered and shared by
// the 8 waves (wave = 16 features, both matrices, two 16-row tiles), the weight records stream straight from memory into the
// MFMA A operand through a four-step register ring that is refilled as soon as a step's MFMAs are issued, and results leave in
// whole 128-byte lines.  Each K group accumulates from zero and the groups are added in order: the values are the same bits as
// up_kernel / down_kernel and the single-launch kernel produce (reference engine-rs/shim/ds41_mx.cu:694-932 keeps the same
// property between its grouped GEMM and its decode kernels).  Gate / up: the exact bf16 form, the activation rows staged as finished
// bf16 operands (xb_put); down: the block-scaled instruction on staged codes.
constexpr int GT_ROWS = 32;            // rows of a GEMM item
constexpr int GT_XS = 528;             // LDS stride of a staged row: one K group (512 bytes) + 16: conflict-free 16-byte reads down a column
constexpr int GT_FEAT = 128;           // output features / columns of a block

// The A operand of a 16-row tile, one K group (four steps) at a time, for the layouts the grouped GEMM takes.  ATile holds this
// lane's base addresses; codes(kg, s) is the 16-byte load of step s (default cache policy, not a streaming load: an expert's
// other 32-row items - neighbours in launch order, on the same XCD - read the same bytes and find them in the L2; measured
// 1.45 -> 1.25 ms on the 2048-token workload), fix() turns what was loaded into the operand, scales(kg) is the K group's scale
// dword (byte s = this lane's K block of step s).
//   T16: records of 4352 bytes, already in operand order.
//   PACK8 / MX8 (reference engine-rs/src/ds41/kern.rs moe_pack / moe_pack_mx): tiles of 8 rows, [K / 128][8][64 bytes] codes and
//   [K / 128][8][4] scales.  MX8 keeps a row's 64 bytes as 4 x 4 dwords [q][b] and the lane of K block g needs column b = g: the
//   four lanes of a row (16 apart) load one q-row each and transpose with two rounds of row swaps.  The scale dword is gathered
//   the same way: lane (row, g) loads the four block scales of step g and the four lanes transpose 4 x 4 bytes.  MX8S2: the
//   codes of MX8 with the scales in the lossless 2-bit coding (a base byte per row + four 2-bit offsets per step, or raw words).
template <int LAYOUT, bool GEN> struct ATile {
    const uint8_t* w;
    const uint8_t* sc;                 // tile layouts: the scale bytes of this lane's row of the tile, step 0 (MX8S2: its code byte)
    const uint8_t* raw;                // MX8S2: the tile's raw scale words when it has them (else null)
    uint32_t base4;                    // MX8S2: the row's base scale in all four bytes
    int steps, g;                      // 128-wide K steps of the matrix (the last K group may hold fewer than four); lane / 16
    uint32_t lo;                       // T16: the lane's offset inside a step's 1024 code bytes (a quarter of it inside the scale bytes)
    static constexpr bool MXT = LAYOUT == L_MX8 || LAYOUT == L_MX8S2;       // 4 x 4 dword order inside a row's 64 bytes
    // an address that is the same in every lane, pinned to scalar registers: the compiler then keeps scalar base + lane offset apart
    // (left alone it folds the lane offset into a 64-bit pointer per lane and stream, and those spill beside the weight ring)
    typedef const __attribute__((address_space(1))) uint8_t* GPtr;          // (an integer turned pointer must say that it is global memory)
    __device__ __forceinline__ static GPtr uniform(const uint8_t* p)
    {
        uint64_t b = (uint64_t)p;
        asm volatile("" : "+s"(b));
        return (GPtr)b;
    }
    __device__ __forceinline__ ATile(const WMat& m, int64_t row0, int lane)          // row0: first row of the tile in the stacked matrix
    {
        steps = m.K >> 7; g = lane >> 4;
        if constexpr (LAYOUT == L_T16) {
            // the tile's first record is the same address for the whole wave (row0 is uniform): kept apart from the lane's offset so that
            // the loads address it as scalar base + 32-bit lane offset (one register a lane instead of a 64-bit pointer per stream)
            w = m.w + (row0 >> 4) * (int64_t)((steps + 3) >> 2) * REC;      // a ragged last K group is a whole record, zero filled
            sc = w + 4096; lo = (uint32_t)lane * 16u;
        } else {
            const int64_t row = row0 + (lane & 15), t8 = row >> 3;
            const int r8 = (int)(row & 7);
            w = m.w + t8 * steps * 512 + r8 * 64 + g * 16;
            if constexpr (LAYOUT == L_MX8S2) {
                // the lossless 2-bit coding (reference engine-rs/shim/ds41_mx.cu:64-91): desc [T][16], codes [T][S][8], raw [n_raw][S][8][4]
                const uint32_t* d = (const uint32_t*)(m.s + t8 * 16);
                const uint8_t* code = m.s + m.tiles8 * 16;
                const int ri = (int)d[2];
                base4 = ((d[r8 >> 2] >> (8 * (r8 & 3))) & 0xffu) * 0x01010101u;
                sc = code + t8 * steps * 8 + r8;
                raw = ri >= 0 ? code + m.tiles8 * steps * 8 + (int64_t)ri * steps * 32 + r8 * 4 : nullptr;
            } else sc = m.s + t8 * steps * 32 + r8 * 4;
        }
    }
    // GEN: steps past the matrix (the tail of a ragged last K group) read the last step again: a valid address, multiplied by zeros
    __device__ __forceinline__ v4i codes(int kg, int s) const
    {
        if constexpr (LAYOUT == L_T16) {
            return *(const __attribute__((address_space(1))) v4i*)(uniform(w + (int64_t)kg * REC) + s * 1024 + lo);
        }
        const uint8_t* p = w + (int64_t)(GEN ? min(kg * 4 + s, steps - 1) : kg * 4 + s) * 512;
        const uint4 v = *(const uint4*)p;
        return v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
    }
    __device__ __forceinline__ static v4i fix(const v4i& v)
    {
        if constexpr (!MXT) return v;
        else {
            const auto a02 = __builtin_amdgcn_permlane32_swap((uint32_t)v.x, (uint32_t)v.z, false, false);
            const auto a13 = __builtin_amdgcn_permlane32_swap((uint32_t)v.y, (uint32_t)v.w, false, false);
            const auto b01 = __builtin_amdgcn_permlane16_swap(a02[0], a13[0], false, false);
            const auto b23 = __builtin_amdgcn_permlane16_swap(a02[1], a13[1], false, false);
            return v4i{(int)b01[0], (int)b01[1], (int)b23[0], (int)b23[1]};
        }
    }
    __device__ __forceinline__ uint32_t scales_raw(int kg) const
    {
        if constexpr (LAYOUT == L_T16) return *(const __attribute__((address_space(1))) uint32_t*)(uniform(sc + (int64_t)kg * REC) + (lo >> 2));
        else {
            const int step = GEN ? min(kg * 4 + g, steps - 1) : kg * 4 + g;   // this lane fetches the four block scales of step g of the K group
            if constexpr (LAYOUT == L_MX8S2) {
                // both forms are requested whatever the tile has (no load behind a branch): a tile without raw words reads its code
                // byte's word a second time
                const uint8_t* cp = sc + (int64_t)step * 8;
                const uint32_t cb = *cp;
                const uint32_t rw = *(const uint32_t*)(raw ? raw + (int64_t)step * 32 : (const uint8_t*)((uintptr_t)cp & ~(uintptr_t)3));
                const uint32_t coded = base4 + ((cb & 3u) | ((cb & 0xcu) << 6) | ((cb & 0x30u) << 12) | ((cb & 0xc0u) << 18));
                return raw ? rw : coded;
            } else return *(const uint32_t*)(sc + (int64_t)step * 32);
        }
    }
    // what scales_raw() loaded -> byte s = the scale of this lane's K block in step s
    __device__ __forceinline__ static uint32_t scales_fix(uint32_t d, int lane)
    {
        if constexpr (LAYOUT == L_T16) return d;
        else {
            // lane (row, g) holds M[g][b] = scale(step g, block b) and wants M[s][g] in byte s: a 4 x 4 byte transpose over the four
            // lanes of the row, 2 x 2 blocks first (partner g ^ 2), then inside the blocks (partner g ^ 1)
            const int g = lane >> 4;
            const uint32_t p = __float_as_uint(lane_xor<32>(__uint_as_float(d), lane));
            // __builtin_amdgcn_perm(hi, lo, sel): result byte i = byte sel[i] of the 8 bytes {hi, lo} (0-3 lo, 4-7 hi)
            const uint32_t n = (g & 2) ? __builtin_amdgcn_perm(d, p, 0x07060302u) : __builtin_amdgcn_perm(p, d, 0x05040100u);
            const uint32_t q = __float_as_uint(lane_xor<16>(__uint_as_float(n), lane));
            return (g & 1) ? __builtin_amdgcn_perm(n, q, 0x07030501u) : __builtin_amdgcn_perm(q, n, 0x06020400u);
        }
    }
};
constexpr bool gemm_layout(int layout) { return layout == L_T16 || layout == L_PACK8 || layout == L_MX8 || layout == L_MX8S2; }

// Activation rows of a K group on their way into LDS: thread (row, 32-byte chunk) fetches its chunk, threads 0..31 also the row's
// 16 scale bytes.  In a ragged last K group (K not a multiple of 512; K >= 512) the chunks past the row's end come out as zero codes
// (fetched from the group's first chunk: a valid address) and the scale bytes past the end repeat valid ones, so the steps past
// the end multiply by exact zeros and no load or matrix instruction sits behind a branch.
// GEN = false (K a multiple of 512): plain loads and stores.  What is loaded is touched only when it is stored into LDS, an
// iteration later: a select right after the load would wait for it (and for every older load of the wave: the weight ring).
struct XStage { uint4 x0, x1, xsc; bool in; int d; };
// xrow / xsrow: the start of the thread's activation row and of the row whose scales it carries; sch: its chunk; K: row length
template <bool GEN>
__device__ __forceinline__ XStage x_fetch(const uint8_t* xrow, const uint8_t* xsrow, int kg, int sch, int K)
{
    XStage r;
    if constexpr (GEN) {
        r.in = kg * 512 + sch * 32 < K;
        const uint8_t* p = xrow + kg * 512 + (r.in ? sch * 32 : 0);
        r.x0 = *(const uint4*)p;
        r.x1 = *(const uint4*)(p + 16);
        // the K group's 16 scale bytes: one 16-byte load that ends inside the row, moved down by whole words where it had to start early
        const int nsb = K >> 5, off = min(kg * 16, nsb - 16);
        r.d = (kg * 16 - off) >> 2;
        r.xsc = *(const uint4*)(xsrow + off);
    } else {
        const uint8_t* p = xrow + kg * 512 + sch * 32;
        r.in = true; r.d = 0;
        r.x0 = *(const uint4*)p;
        r.x1 = *(const uint4*)(p + 16);
        r.xsc = *(const uint4*)(xsrow + kg * 16);
    }
    return r;
}
// the fetched chunk and (threads 0 .. GT_ROWS - 1) the row's scale bytes into the staging buffers
template <bool GEN>
__device__ __forceinline__ void x_put(const XStage& r, unsigned char* xdst, unsigned char* sdst, bool scales)
{
    if constexpr (GEN) {
        const uint32_t m = r.in ? ~0u : 0u;
        *(uint4*)xdst = make_uint4(r.x0.x & m, r.x0.y & m, r.x0.z & m, r.x0.w & m);
        *(uint4*)(xdst + 16) = make_uint4(r.x1.x & m, r.x1.y & m, r.x1.z & m, r.x1.w & m);
        if (scales) {
            const uint32_t a = r.xsc.x, b = r.xsc.y, c = r.xsc.z, e = r.xsc.w;
            const uint32_t o0 = r.d == 0 ? a : r.d == 1 ? b : r.d == 2 ? c : e;
            const uint32_t o1 = r.d == 0 ? b : r.d == 1 ? c : e;
            const uint32_t o2 = r.d == 0 ? c : e;
            *(uint4*)sdst = make_uint4(o0, o1, o2, e);
        }
    } else {
        *(uint4*)xdst = r.x0;
        *(uint4*)(xdst + 16) = r.x1;
        if (scales) *(uint4*)sdst = r.xsc;
    }
}

// Visit order of the K groups of a product with more K groups than the decode kernels have waves along K (W = 8 for gate / up, 4 for
// down): the decode kernels' wave j walks K groups j, j + W, j + 2W, ... in one accumulator and the W sums are added in wave order.
// So the groups are visited slot by slot: visit i is K group kg, `fresh` says that it starts a sum from zero and `last` that its sum
// is complete.  Up to W K groups: 0, 1, 2, ..., each its own sum.
struct KVisit { int kg; bool fresh, last; };
// GEN = false: at most 2 W K groups for W = 8 (the sums of two K groups, slots 0 .. nkg - 9, visited first), at most W for W = 4
template <bool GEN, int W>
__device__ __forceinline__ KVisit k_visit(int i, int nkg)
{
    if constexpr (GEN) {
        const int q = nkg / W, r = nkg % W;                // slots 0 .. r - 1 hold q + 1 K groups, the others q
        int j, t, len;
        if (i < r * (q + 1)) { j = i / (q + 1); t = i % (q + 1); len = q + 1; }
        else { const int i2 = i - r * (q + 1), qq = max(q, 1); j = r + i2 / qq; t = i2 % qq; len = q; }     // (q = 0: every visit is in the first case)
        return KVisit{j + t * W, t == 0, t == len - 1};
    } else if constexpr (W == DN_WAVES) return KVisit{i, true, true};
    else {
        const int nl = nkg > W ? nkg - W : 0;
        if (i < 2 * nl) return KVisit{(i >> 1) + W * (i & 1), (i & 1) == 0, (i & 1) != 0};
        return KVisit{i - nl, true, true};
    }
}

// The gate / up operand of the grouped GEMM is staged as bf16: thread (row, 32-block) converts its block's 32 E4M3 codes with the
// block's UE8M0 scale (exact) and writes 64 bytes, so that the eight waves read finished B operands of v_mfma_f32_16x16x32_bf16
// (16 bytes a lane and instruction) instead of each converting the same codes again.  GT_XB: the row stride, 16 bytes over a multiple
// of 256: the 16-byte reads of 16 rows at one column cover every bank once.
constexpr int GT_XB = 1024 + 16;
struct XStageB { uint4 x0, x1; uint32_t sb; bool in; };
template <bool GEN>
__device__ __forceinline__ XStageB xb_fetch(const uint8_t* xrow, const uint8_t* xsrow, int kg, int sch, int K)
{
    XStageB r;
    r.in = !GEN || kg * 512 + sch * 32 < K;
    const int off = r.in ? sch : 0;                        // past the row's end: the group's first block again (a valid address), stored as zeros
    const uint8_t* p = xrow + kg * 512 + off * 32;
    r.x0 = *(const uint4*)p;
    r.x1 = *(const uint4*)(p + 16);
    r.sb = xsrow[kg * 16 + off];
    return r;
}
__device__ __forceinline__ void xb_put(const XStageB& r, unsigned char* dst)
{
    // eight codes (two dwords) at a time: converted and stored before the next eight, so that few registers are live beside the K loop's
    const uint32_t m = r.in ? ~0u : 0u;
    const float sc = e8m0_to_f32(r.sb & 0xffu);
    const uint32_t w[8] = {r.x0.x & m, r.x0.y & m, r.x0.z & m, r.x0.w & m, r.x1.x & m, r.x1.y & m, r.x1.z & m, r.x1.w & m};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        bf2 v[4];
        v[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j], sc, false); v[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j], sc, true);
        v[2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j + 1], sc, false); v[3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j + 1], sc, true);
        uint4 o; __builtin_memcpy(&o, v, 16);
        *(uint4*)(dst + 16 * j) = o;
        __builtin_amdgcn_sched_barrier(0);
    }
}

// One block of the gate / up GEMM for an item of NRT 16-row tiles.  The kernel below runs the instance of the item's tile count: each
// instance is a region of its own for the register allocator (one K loop with a run-time tile count put a branch into every step;
// two K loops sharing their surroundings spilled beside the weight ring).
template <int LAYOUT, bool GEN, int NRT>
__device__ __forceinline__ void up_gemm_block(const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, const WMat& w1, const WMat& w3, int H, int I, int TT,
                                              const Item it, const int* __restrict__ prow, const float* __restrict__ pw, uint8_t* __restrict__ hq,
                                              uint8_t* __restrict__ hs, unsigned char* gsm, int* toks, float* wgts, float (*amx)[2][16], unsigned char (*hes)[4])
{
    unsigned char* const xl = gsm;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), c = lane & 15, rg = lane >> 4;
    const int f0 = blockIdx.x * GT_FEAT;
    const int steps = H >> 7, nkg = (steps + 3) >> 2;      // the last K group may hold fewer than four steps
    if (tid < GT_ROWS) {
        const int pos = it.off + min(tid, it.n - 1);
        toks[tid] = prow[pos] / TT;
        wgts[tid] = tid < it.n ? pw[pos] : 0.f;
    }
    // the wave's weight rows: 16 gate and 16 up rows, the first K group visited (K group 0) first
    const ATile<LAYOUT, GEN> t1(w1, (int64_t)it.e * I + f0 + 16 * wave, lane), t3(w3, (int64_t)it.e * I + f0 + 16 * wave, lane);
    v4i a[2][4];
    uint32_t sa[2];
#pragma unroll
    for (int s = 0; s < 4; ++s) { a[0][s] = t1.codes(0, s); a[1][s] = t3.codes(0, s); }
    sa[0] = t1.scales_raw(0); sa[1] = t3.scales_raw(0);
    const int kg1 = k_visit<GEN, UP_WAVES>(min(1, nkg - 1), nkg).kg;
    __syncthreads();
    // staging: thread = (row, 32-block) of a K group
    const int srow = tid >> 4, sch = tid & 15;
    const uint8_t* xrow = xq + (int64_t)toks[srow] * H;
    const uint8_t* xsrow = xs + (int64_t)toks[srow] * (H >> 5);
    unsigned char* const xdst = xl + srow * GT_XB + sch * 64;
    XStageB xf = xb_fetch<GEN>(xrow, xsrow, 0, sch, H);
    xb_put(xf, xdst);
    xf = xb_fetch<GEN>(xrow, xsrow, kg1, sch, H);
    __syncthreads();
    v4f tot[2][NRT];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int rt = 0; rt < NRT; ++rt) tot[m][rt] = v4f{0.f, 0.f, 0.f, 0.f};
    const unsigned char* const bbase = xl + c * GT_XB + 64 * rg;
    // The K loop in two instances, for items of one and of two 16-row tiles: no branch inside a K group, so that the compiler
    // schedules a K group's 16-byte operand reads, converts and matrix instructions as one block (with a branch around the second
    // row tile's instructions every read waited for its data right in front of its matrix instruction).
    {
        v4f cur[2][NRT];
        for (int i = 0; i < nkg; ++i) {
            const KVisit vis = k_visit<GEN, UP_WAVES>(i, nkg);
            const int buf = i & 1, kn = k_visit<GEN, UP_WAVES>(min(i + 1, nkg - 1), nkg).kg;
            const uint32_t san0 = t1.scales_raw(kn), san1 = t3.scales_raw(kn);
            const uint32_t sc0 = ATile<LAYOUT, GEN>::scales_fix(sa[0], lane), sc1 = ATile<LAYOUT, GEN>::scales_fix(sa[1], lane);
            if (vis.fresh) {
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int rt = 0; rt < NRT; ++rt) cur[m][rt] = v4f{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int rt = 0; rt < NRT; ++rt) asm volatile("" : "+v"(cur[m][rt]));
            const unsigned char* bp = bbase + buf * (GT_ROWS * GT_XB);
            // B operands one step ahead of their matrix instructions: step t = (s, j) reads the operands of step t + 1 first
            auto read_b = [&](int t, bf8v (&b)[NRT]) {
#pragma unroll
                for (int rt = 0; rt < NRT; ++rt) {
                    const uint4 v = *(const uint4*)(bp + rt * (16 * GT_XB) + (t >> 2) * 256 + 16 * (t & 3));
                    __builtin_memcpy(&b[rt], &v, 16);
                }
            };
            constexpr bool AHEAD = NRT == 1 || LAYOUT == L_T16;    // (the tile layouts with two row tiles have no registers left for the second set of operands)
            bf8v bq[AHEAD ? 2 : 1][NRT];
            if constexpr (AHEAD) read_b(0, bq[0]);
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const v4i a0 = ATile<LAYOUT, GEN>::fix(a[0][s]), a1 = ATile<LAYOUT, GEN>::fix(a[1][s]);
                const float f0s = e8m0_to_f32((sc0 >> (8 * s)) & 0xffu), f1s = e8m0_to_f32((sc1 >> (8 * s)) & 0xffu);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int t = 4 * s + j;
                    if constexpr (AHEAD) { if (t < 15) read_b(t + 1, bq[(t + 1) & 1]); }
                    else read_b(t, bq[0]);                 // requested ahead of the step's converts
                    __builtin_amdgcn_sched_barrier(0);
                    const bf8v w0 = a_operand((uint32_t)a0[j], f0s), w1v = a_operand((uint32_t)a1[j], f1s);
#pragma unroll
                    for (int rt = 0; rt < NRT; ++rt) {
                        cur[0][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, bq[AHEAD ? (t & 1) : 0][rt], cur[0][rt], 0, 0, 0);
                        cur[1][rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1v, bq[AHEAD ? (t & 1) : 0][rt], cur[1][rt], 0, 0, 0);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
                a[0][s] = t1.codes(kn, s);                 // the ring slot is free again: the same step of the next K group
                a[1][s] = t3.codes(kn, s);
            }
            if (vis.last) {
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int rt = 0; rt < NRT; ++rt) tot[m][rt] += cur[m][rt];
            }
            sa[0] = san0; sa[1] = san1;
            // the next K group of the rows into the other buffer (nobody reads it before the barrier), the one after into registers
            xb_put(xf, xdst + (buf ^ 1) * (GT_ROWS * GT_XB));
            xf = xb_fetch<GEN>(xrow, xsrow, k_visit<GEN, UP_WAVES>(min(i + 2, nkg - 1), nkg).kg, sch, H);
            __syncthreads();
        }
    }
    // ---- SwiGLU * route weight, act_quant per 32 features (this wave's 16 and its neighbour's), 128 code bytes + 4 scales per row
    unsigned char (*hbuf)[GT_FEAT + 16] = (unsigned char (*)[GT_FEAT + 16])gsm;     // the staging buffers are free: the loop ended on a barrier
    float yv[NRT][4];
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
        const float wgt = wgts[rt * 16 + c];
        float am = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float gt = fminf(bf16_round(tot[0][rt][i]), 10.f);
            const float up = fminf(fmaxf(bf16_round(tot[1][rt][i]), -10.f), 10.f);
            yv[rt][i] = bf16_round(silu(gt) * up * wgt);
            am = fmaxf(am, fabsf(yv[rt][i]));
        }
        am = fmaxf(am, __shfl_xor(am, 16, 64));
        am = fmaxf(am, __shfl_xor(am, 32, 64));
        if (rg == 0) amx[wave][rt][c] = am;
    }
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < NRT; ++rt) {
        const uint32_t e = aq_scale(fmaxf(amx[wave][rt][c], amx[wave ^ 1][rt][c]));
        *(uint32_t*)&hbuf[rt * 16 + c][16 * wave + 4 * rg] = aq_word4(yv[rt][0], yv[rt][1], yv[rt][2], yv[rt][3], e);
        if (rg == 0 && (wave & 1) == 0) hes[rt * 16 + c][wave >> 1] = (unsigned char)e;
    }
    __syncthreads();
    if (tid < 256) {
        const int row = tid >> 3, ch = tid & 7;
        if (row < it.n) *(uint4*)(hq + (int64_t)(it.off + row) * I + f0 + ch * 16) = *(const uint4*)&hbuf[row][ch * 16];
    } else if (tid < 256 + GT_ROWS) {
        const int row = tid - 256;
        if (row < it.n) *(uint32_t*)(hs + (int64_t)(it.off + row) * (I >> 5) + (f0 >> 5)) = *(const uint32_t*)hes[row];
    }
}
template <int LAYOUT, bool GEN>
__global__ __launch_bounds__(512, 4) void up_gemm_kernel(const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, WMat w1, WMat w3, int H, int I, int TT,
                                                         const int* __restrict__ G, const Item* __restrict__ items, const int* __restrict__ prow,
                                                         const float* __restrict__ pw, uint8_t* __restrict__ hq, uint8_t* __restrict__ hs)
{
    extern __shared__ __align__(16) unsigned char gsm[];  // xl [2][GT_ROWS * GT_XB], then the epilogue's hbuf [GT_ROWS][GT_FEAT + 16] over it
    __shared__ int toks[GT_ROWS];
    __shared__ float wgts[GT_ROWS];
    __shared__ float amx[8][2][16];
    __shared__ __align__(4) unsigned char hes[GT_ROWS][4];
    const Item it = items[blockIdx.y];             // requested together with the item count (entries past it hold anything)
    if ((int)blockIdx.y >= *G) return;
    if (it.n > 16) up_gemm_block<LAYOUT, GEN, 2>(xq, xs, w1, w3, H, I, TT, it, prow, pw, hq, hs, gsm, toks, wgts, amx, hes);
    else up_gemm_block<LAYOUT, GEN, 1>(xq, xs, w1, w3, H, I, TT, it, prow, pw, hq, hs, gsm, toks, wgts, amx, hes);
}
constexpr size_t UP_GEMM_LDS = (size_t)2 * GT_ROWS * GT_XB;

constexpr int GT_COLS = 256;           // output columns of a down-projection block: two 16-column tiles per wave
template <int LAYOUT, bool GEN>
__global__ __launch_bounds__(512, 4) void down_gemm_kernel(const uint8_t* __restrict__ hq, const uint8_t* __restrict__ hs, WMat w2, int H, int I,
                                                           const int* __restrict__ G, const Item* __restrict__ items, float* __restrict__ out, int col0, int ldo,
                                                           int ob16)
{
    // ob16: the pairs' outputs are stored as bf16 (the binary32 sums rounded to nearest even; reference engine-rs/shim/ds41_mx.cu:1245-1255,
    // DS41_MOE_PAIR_BF16): out is then uint16 [P, ldo]
    // col0 / ldo: this launch covers output columns [col0, col0 + ldo) and out has ldo columns per row (a column pass of a call
    // whose per-pair outputs would not fit the cap on that buffer; one pass: col0 = 0, ldo = H)
    __shared__ __align__(16) unsigned char xl[2][GT_ROWS * GT_XS];
    __shared__ __align__(16) unsigned char xsl[2][GT_ROWS * 16];
    const Item it = items[blockIdx.y];             // requested together with the item count (entries past it hold anything)
    if ((int)blockIdx.y >= *G) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), c = lane & 15, rg = lane >> 4;
    const int n0 = col0 + blockIdx.x * GT_COLS + 32 * wave;
    const int steps = I >> 7, nkg = (steps + 3) >> 2;      // the last K group may hold fewer than four steps
    const int nrt = (it.n + 15) >> 4;
    const ATile<LAYOUT, GEN> ta(w2, (int64_t)it.e * H + n0, lane), tb(w2, (int64_t)it.e * H + n0 + 16, lane);
    v4i a[2][4];
    uint32_t sa[2];
#pragma unroll
    for (int s = 0; s < 4; ++s) { a[0][s] = ta.codes(0, s); a[1][s] = tb.codes(0, s); }
    sa[0] = ta.scales_raw(0); sa[1] = tb.scales_raw(0);
    const int srow = tid >> 4, sch = tid & 15;
    const uint8_t* xrow = hq + (int64_t)(it.off + min(srow, it.n - 1)) * I;
    const uint8_t* xsrow = hs + (int64_t)(it.off + min(tid & (GT_ROWS - 1), it.n - 1)) * (I >> 5);
    unsigned char* const xdst = &xl[0][srow * GT_XS + sch * 32];
    XStage xf = x_fetch<GEN>(xrow, xsrow, 0, sch, I);
    x_put<GEN>(xf, xdst, &xsl[0][(tid & (GT_ROWS - 1)) * 16], tid < GT_ROWS);
    xf = x_fetch<GEN>(xrow, xsrow, k_visit<GEN, DN_WAVES>(min(1, nkg - 1), nkg).kg, sch, I);
    __syncthreads();
    v4f tot[2][2];
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) tot[m][rt] = v4f{0.f, 0.f, 0.f, 0.f};
    v4f cur[2][2];
    for (int i = 0; i < nkg; ++i) {
        const KVisit vis = k_visit<GEN, DN_WAVES>(i, nkg);
        const int kg = vis.kg, buf = i & 1, kn = k_visit<GEN, DN_WAVES>(min(i + 1, nkg - 1), nkg).kg;
        const uint32_t san0 = ta.scales_raw(kn), san1 = tb.scales_raw(kn);
        const uint32_t sc0 = ATile<LAYOUT, GEN>::scales_fix(sa[0], lane), sc1 = ATile<LAYOUT, GEN>::scales_fix(sa[1], lane);
        if (vis.fresh) {
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) cur[m][rt] = v4f{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) asm volatile("" : "+v"(cur[m][rt]));
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const v4i a0 = ATile<LAYOUT, GEN>::fix(a[0][s]), a1 = ATile<LAYOUT, GEN>::fix(a[1][s]);
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                if (rt < nrt) {
                    const unsigned char* bp = &xl[buf][(rt * 16 + c) * GT_XS + s * 128 + 16 * rg];
                    const uint4 lo = *(const uint4*)bp, hi = *(const uint4*)(bp + 64);
                    const v8i b = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
                    const uint32_t sb = *(const uint32_t*)&xsl[buf][(rt * 16 + c) * 16 + s * 4] >> (8 * rg);
                    cur[0][rt] = mfma_group_step(s, a0, b, cur[0][rt], sc0, sb);
                    cur[1][rt] = mfma_group_step(s, a1, b, cur[1][rt], sc1, sb);
                }
            }
            a[0][s] = ta.codes(kn, s);
            a[1][s] = tb.codes(kn, s);
        }
        if (vis.last) {
#pragma unroll
            for (int m = 0; m < 2; ++m)
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) tot[m][rt] += cur[m][rt];
        }
        sa[0] = san0; sa[1] = san1;
        x_put<GEN>(xf, xdst + (buf ^ 1) * (GT_ROWS * GT_XS), &xsl[buf ^ 1][(tid & (GT_ROWS - 1)) * 16], tid < GT_ROWS);
        xf = x_fetch<GEN>(xrow, xsrow, k_visit<GEN, DN_WAVES>(min(i + 2, nkg - 1), nkg).kg, sch, I);
        __syncthreads();
    }
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
        const int row = rt * 16 + c;
        if (row < it.n) {
#pragma unroll
            for (int m = 0; m < 2; ++m) {
                // written once, read once by the sum over the pairs: a streaming store leaves the caches to the weight stream
                if (ob16)
                    *(uint2*)((uint16_t*)out + (int64_t)(it.off + row) * ldo + (n0 - col0) + 16 * m + 4 * rg) =
                        make_uint2((uint32_t)f32_to_bf16(tot[m][rt][0]) | ((uint32_t)f32_to_bf16(tot[m][rt][1]) << 16),
                                   (uint32_t)f32_to_bf16(tot[m][rt][2]) | ((uint32_t)f32_to_bf16(tot[m][rt][3]) << 16));
                else
                    st_stream16(out + (int64_t)(it.off + row) * ldo + (n0 - col0) + 16 * m + 4 * rg,
                                make_uint4(__float_as_uint(tot[m][rt][0]), __float_as_uint(tot[m][rt][1]), __float_as_uint(tot[m][rt][2]), __float_as_uint(tot[m][rt][3])));
            }
        }
    }
}

// y[r] = (add[r] + sum of the shared experts' outputs) + (sum_k routed out[pairmap[r, k]], k ascending)
// reference ds41_mx.cu:302-317
__global__ __launch_bounds__(256) void combine_kernel(const float* __restrict__ out, const int* __restrict__ pairmap, const float* __restrict__ add,
                                                      float* __restrict__ y, int nr, int H, int topk, int n_shared, int col0, int ldo, int obf16, int pb16)
{
    // columns [col0, col0 + ldo) of y; out has ldo columns per row (one pass: col0 = 0, ldo = H); pb16: the pairs' outputs are bf16
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int h4 = ldo >> 2;
    if (i >= (int64_t)nr * h4) return;
    const int r = (int)(i / h4), col = (int)(i % h4) * 4, TT = topk + n_shared;
    float4 acc = add ? *(const float4*)(add + (int64_t)r * H + col0 + col) : make_float4(0.f, 0.f, 0.f, 0.f);
    // the pairs' outputs are read once: streaming loads
    auto pair4 = [&](int k) {
        const int64_t o = (int64_t)pairmap[r * TT + k] * ldo + col;
        if (pb16) {
            const uint2 v = *(const uint2*)((const uint16_t*)out + o);
            return make_float4(__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u), __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u));
        }
        const uint4 v = ld_stream16(out + o);
        return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
    };
    for (int k = topk; k < TT; ++k) { const float4 v = pair4(k); acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w; }
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k = 0; k < topk; ++k) { const float4 v = pair4(k); s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w; }
    acc.x += s.x; acc.y += s.y; acc.z += s.z; acc.w += s.w;
    if (obf16) *(uint2*)((uint16_t*)y + (int64_t)r * H + col0 + col) = make_uint2((uint32_t)f32_to_bf16(acc.x) | ((uint32_t)f32_to_bf16(acc.y) << 16),
                                                                                   (uint32_t)f32_to_bf16(acc.z) | ((uint32_t)f32_to_bf16(acc.w) << 16));
    else *(float4*)(y + (int64_t)r * H + col0 + col) = acc;
}

// ---------------------------------------------------------------- natural layout -> T16 records
// w [rows_total, K/2], s [rows_total, K/32] (rows_total % 16 == 0, K % 128 == 0); one thread per (tile, K group, lane).
__global__ __launch_bounds__(256) void prepack_kernel(const uint8_t* __restrict__ w, const uint8_t* __restrict__ s, uint8_t* __restrict__ out, int64_t tiles, int K)
{
    const int steps = K >> 7, nkg = (steps + 3) >> 2;
    const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= tiles * nkg * 64) return;
    const int lane = (int)(gid & 63);
    const int64_t rec = gid >> 6;
    const int kg = (int)(rec % nkg);
    const int64_t tile = rec / nkg, row = tile * 16 + (lane & 15);
    const int g = lane >> 4;
    uint8_t* o = out + rec * REC;
    uint32_t sc4 = 0x7f7f7f7fu;
    for (int st = 0; st < 4; ++st) {
        const int step = kg * 4 + st;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (step < steps) {
            v = *(const uint4*)(w + row * (K >> 1) + step * 64 + g * 16);
            sc4 = (sc4 & ~(0xffu << (8 * st))) | ((uint32_t)s[row * (K >> 5) + step * 4 + g] << (8 * st));
        }
        *(uint4*)(o + st * 1024 + lane * 16) = v;
    }
    *(uint32_t*)(o + 4096 + lane * 4) = sc4;
}

// ---------------------------------------------------------------- host side
// rows per item: 32 for the grouped GEMM, which takes every call of more than 8 rows that it can (T16 records or the 8-row tile
// layouts, K a multiple of 128 and at least 512 - the reference's per-rank intermediate width is 768 -, at most sixteen K groups
// for gate / up and eight for down, visited in the decode kernels' order of summation; measured against the kernels below at 9-16 rows: 2-7 % faster on T16 records, 1.8x on the tile layouts at hidden
// width 5120); otherwise 16 up to 16 rows and up to 512 beyond (one pass over the expert's weights per item)
inline int gr_of(int R, bool gemm) { return gemm ? GT_ROWS : R <= 16 ? 16 : 512; }
// Most rows of a call that the single launch takes where the grouped GEMM could take it too.  Measured on both (same bits either
// way), us per call single launch / grouped GEMM.  T16 records, H 4096, I 2048: 1 row 22 / 43, 2 rows 42 / 48, 4 rows 68 / 80,
// 8 rows 127 / 122: the single launch up to 8 rows.  The reference's 8-row tile layouts, H 5120: I 768: 22 / 40, 39 / 43, 67 / 51,
// 121 / 87; I 2048: 28 / 48, 51 / 56, 96 / 96, 182 / 159: the single launch up to 2 rows, up to 4 from I = 1536 on.
int g_fused_rows = -1;                  // diagnostics: 0..8 overrides the rule for every layout
inline int fused_rows(int layout, int I) { return g_fused_rows >= 0 ? g_fused_rows : layout == L_T16 ? 8 : I >= 1536 ? 4 : 2; }
inline bool gemm_ok(int layout, int R, int H, int I)
{
    return gemm_layout(layout) && R > fused_rows(layout, I) && H >= 512 && I >= 512 && (H + 511) / 512 <= 2 * UP_WAVES && (I + 511) / 512 <= 2 * DN_WAVES && I % GT_FEAT == 0 && H % GT_COLS == 0;
}
inline int gmax_of(int R, int TT, int ET, bool gemm)
{
    const int64_t P = (int64_t)R * TT;
    return (int)((P < ET ? P : ET) + P / gr_of(R, gemm) + 1);
}
struct WsLayout {
    size_t G, items, pairmap, prow, pw, hq, hs, out, total;
};
// np: column passes of the down product + sum (the per-pair output buffer then holds H / np columns)
inline WsLayout ws_layout(int R, int H, int I, int TT, int ET, int np = 1)
{
    const size_t P = (size_t)R * TT;
    WsLayout l;
    size_t o = 0;
    l.G = o; o += align256(16 + 64 * 4 + 2 * 4 * (size_t)EMAXG);     // G + a few counters + the experts' row offsets and fill counts of a large call
    l.items = o; o += align256(sizeof(Item) * (size_t)gmax_of(R, TT, ET, true));     // the finer of the two item sizes
    l.pairmap = o; o += align256(4 * P);
    l.prow = o; o += align256(4 * P);
    l.pw = o; o += align256(4 * P);
    l.hq = o; o += align256(P * I);
    l.hs = o; o += align256(P * I / 32);
    l.out = o; o += align256(4 * P * H / np);
    l.total = o;
    return l;
}

template <int LAYOUT>
int moe_launch(const uint8_t* xq, const uint8_t* xs, int R, const int64_t* idx, const float* rw, const uint8_t* w1, const uint8_t* s1, const uint8_t* w3,
               const uint8_t* s3, const uint8_t* w2, const uint8_t* s2, int H, int I, int topk, int E, int n_shared, const float* add, float* y, void* ws,
               int skip_combine, hipStream_t st, int np = 1, int obf16 = 0, int pb16 = 0)
{
    const bool gemm = gemm_ok(LAYOUT, R, H, I);
    if (pb16 && !gemm) return 1;                              // bf16 pair outputs belong to the grouped GEMM
    if (np > 1 && (!gemm || skip_combine)) return 1;          // column passes belong to the grouped GEMM and sum as they go
    const int TT = topk + n_shared, ET = E + n_shared, GR = gr_of(R, gemm), Gm = gmax_of(R, TT, ET, gemm);
    const WsLayout l = ws_layout(R, H, I, TT, ET, np);
    char* base = (char*)ws;
    int* G = (int*)(base + l.G);
    Item* items = (Item*)(base + l.items);
    int* pairmap = (int*)(base + l.pairmap);
    int* prow = (int*)(base + l.prow);
    float* pw = (float*)(base + l.pw);
    uint8_t* hq = (uint8_t*)(base + l.hq);
    uint8_t* hs = (uint8_t*)(base + l.hs);
    float* out = (float*)(base + l.out);
    if ((int64_t)R * TT > 4096) {
        int *geoff = G + 4 + 64, *gfill = geoff + EMAXG;
        group_kernel<<<1, 1024, 0, st>>>(idx, rw, R, topk, n_shared, E, GR, G, items, pairmap, prow, pw, G + 4, 64, geoff, gfill);
        scatter_kernel<<<(unsigned)(((int64_t)R * TT + 1023) / 1024), 1024, 0, st>>>(idx, rw, R, topk, n_shared, E, geoff, gfill, pairmap, prow, pw);
    } else
        group_kernel<<<1, 1024, 0, st>>>(idx, rw, R, topk, n_shared, E, GR, G, items, pairmap, prow, pw, G + 4, 64, nullptr, nullptr);
    const WMat m1{w1, s1, I, H, (int64_t)ET * I / 8}, m3{w3, s3, I, H, (int64_t)ET * I / 8}, m2{w2, s2, H, I, (int64_t)ET * H / 8};
    if constexpr (gemm_layout(LAYOUT)) {
        if (gemm) {
            // the plain forms take K in whole 512-wide groups (gate / up: at most sixteen, down: at most four); a ragged last K group or a
            // longer down product runs the general forms (clamped loads, zero codes past the end, the visit order worked out per group)
            const bool genu = H % 512 != 0, gend = I % 512 != 0 || I / 512 > DN_WAVES;
            static bool attr = false;                      // 65 KB of staging a block: beyond the default cap on dynamic LDS
            if (!attr) {
                (void)hipFuncSetAttribute((const void*)up_gemm_kernel<LAYOUT, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)UP_GEMM_LDS);
                (void)hipFuncSetAttribute((const void*)up_gemm_kernel<LAYOUT, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)UP_GEMM_LDS);
                attr = true;
            }
            if (genu) up_gemm_kernel<LAYOUT, true><<<dim3(I / GT_FEAT, Gm), 512, UP_GEMM_LDS, st>>>(xq, xs, m1, m3, H, I, TT, G, items, prow, pw, hq, hs);
            else up_gemm_kernel<LAYOUT, false><<<dim3(I / GT_FEAT, Gm), 512, UP_GEMM_LDS, st>>>(xq, xs, m1, m3, H, I, TT, G, items, prow, pw, hq, hs);
            const int hn = H / np;
            const int64_t n4 = (int64_t)R * (hn / 4);
            for (int ps = 0; ps < np; ++ps) {
                // a pass = the down product of hn output columns, then (with more than one pass) their weighted sum, before the next
                // pass writes over the buffer; every output's products and sums are those of the one-pass call
                if (gend) down_gemm_kernel<LAYOUT, true><<<dim3(hn / GT_COLS, Gm), 512, 0, st>>>(hq, hs, m2, H, I, G, items, out, ps * hn, hn, pb16);
                else down_gemm_kernel<LAYOUT, false><<<dim3(hn / GT_COLS, Gm), 512, 0, st>>>(hq, hs, m2, H, I, G, items, out, ps * hn, hn, pb16);
                if (np > 1) combine_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, st>>>(out, pairmap, add, y, R, H, topk, n_shared, ps * hn, hn, obf16, pb16);
            }
            if (np > 1) return launch_status();
        }
    }
    if (!gemm) {
    if (((H >> 7) + 3) >> 2 <= UP_WAVES) up_res_kernel<LAYOUT><<<dim3(I / 32, Gm), 64 * UP_WAVES, 0, st>>>(xq, xs, m1, m3, H, I, TT, G, items, prow, pw, hq, hs);
    else up_kernel<LAYOUT><<<dim3(I / 32, Gm), 64 * UP_WAVES, 0, st>>>(xq, xs, m1, m3, H, I, TT, G, items, prow, pw, hq, hs);
    if (((I >> 7) + 3) >> 2 <= DN_WAVES) down_res_kernel<LAYOUT><<<dim3(H / 32, Gm), 64 * DN_WAVES, 0, st>>>(hq, hs, m2, H, I, G, items, out);
    else down_kernel<LAYOUT><<<dim3(H / 32, Gm), 64 * DN_WAVES, 0, st>>>(hq, hs, m2, H, I, G, items, out);
    }
    if (!skip_combine) {
        const int64_t n4 = (int64_t)R * (H / 4);
        combine_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, st>>>(out, pairmap, add, y, R, H, topk, n_shared, 0, H, obf16, pb16);
    }
    return launch_status();
}

inline bool shapes_ok(int R, int H, int I, int topk, int E, int n_shared)
{
    return R >= 1 && H >= 128 && I >= 128 && H % 128 == 0 && I % 128 == 0 && topk >= 1 && n_shared >= 0 && E >= 1 && E + n_shared <= EMAXG;
}

int g_s2 = 0;          // scale blobs handed to the ds41_moe_mx* symbols are 2-bit coded (reference ds41_mx.cu:1304)

#ifdef SPK_MX_TRACE
}  // namespace
extern "C" __attribute__((visibility("default"))) void spark_debug_mx_gemm_trace(long long* buf) { (void)hipMemcpyToSymbol(HIP_SYMBOL(g_gtrace), &buf, sizeof(buf)); }
namespace {
#endif
}  // namespace

// ================================================================ C ABI: runtime-sized entry points (no reference counterpart symbol)

// bytes of one stacked matrix [rows_total, K] in T16 records
SPARK_API size_t spark_mxfp4_packed_bytes(long long rows_total, int K)
{
    if (rows_total < 16 || rows_total % 16 || K < 128 || K % 128) return 0;
    return (size_t)(rows_total / 16) * ((K / 128 + 3) / 4) * REC;
}
// natural layout (w [rows_total, K/2], s [rows_total, K/32], device) -> T16 records (device)
SPARK_API int spark_mxfp4_prepack(const void* w, const void* s, void* packed, long long rows_total, int K, hipStream_t st)
{
    if (rows_total < 16 || rows_total % 16 || K < 128 || K % 128) return 1;
    const int64_t tiles = rows_total / 16, n = tiles * ((K / 128 + 3) / 4) * 64;
    prepack_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>((const uint8_t*)w, (const uint8_t*)s, (uint8_t*)packed, tiles, K);
    return launch_status();
}
// the single-launch path's workspace follows the several-kernel path's (they never share bytes)
// The single-launch path's region comes first in a spark_mxfp4_moe* workspace and has one size per shape (that of the most rows the
// path takes), so calls of any size can share a workspace without writing over its idle exchange words.
static size_t fused_cap(int H, int I, int topk, int E, int n_shared)
{
    for (int r = 8; r >= 1; --r)
        if (mx_fused_ok(r, H, I, topk, E, n_shared)) return mx_fused_ws_bytes(r, H, I, topk, E, n_shared);
    return 0;
}
// Which path a call of this shape takes (a host-side query: nothing is launched): 0 = the single launch, 1 = the grouped GEMM, 2 = the
// several-kernel path, -1 = a shape no entry point takes.  layout: 0 T16 records, 1 checkpoint layout, 2 / 3 / 4 the reference's
// moe_pack / moe_pack_mx / moe_pack_mx + 2-bit coded scales tile layouts (the ds41_* entry points).
SPARK_API int spark_mxfp4_moe_path(int layout, int R, int H, int I, int topk, int E, int n_shared)
{
    if (!shapes_ok(R, H, I, topk, E, n_shared) || layout < L_T16 || layout > L_MX8S2) return -1;
    if (gemm_ok(layout, R, H, I)) return 1;
    return mx_fused_ok(R, H, I, topk, E, n_shared) ? 0 : 2;
}
SPARK_API size_t spark_mxfp4_moe_ws_bytes(int R, int H, int I, int topk, int E, int n_shared)
{
    if (!shapes_ok(R, H, I, topk, E, n_shared)) return 0;
    return fused_cap(H, I, topk, E, n_shared) + ws_layout(R, H, I, topk + n_shared, E + n_shared).total;     // grows with R
}
// Prepares a workspace once after allocation (every exchanged word idle) and runs the one-time placement check, which synchronises
// the device: call it outside stream capture.  From then on decode-sized calls that use this workspace - spark_mxfp4_moe_x with or
// without flags bit 0, spark_mxfp4_moe(_q), ds41_moe_mx(_ex), ds41_moe - skip their own preparing launch;
// spark_moe_ws_release(ws) before the memory is freed or reused.
SPARK_API int spark_mxfp4_moe_ws_init(void* ws, size_t bytes, hipStream_t st)
{
    xcd_placement_check();
    if (!ws || bytes == 0) return 0;
    const int rc = mx_fused_ws_prepare(ws, bytes, st);
    if (rc == 0) ws_note_prepared(ws, bytes);
    return rc;
}
namespace {
inline void* fused_ws(void* ws, int R, int H, int I, int topk, int E, int n_shared)
{
    (void)R; (void)H; (void)I; (void)topk; (void)E; (void)n_shared;
    return ws;                                     // first in the workspace, one size per shape (fused_cap)
}
}  // namespace
// xq [R, H] E4M3 + xs [R, H/32] UE8M0 (act_quant of x); idx int64 / rw f32 [R, topk]; stacked weights of E + n_shared
// experts: layout 0 = T16 records (s* unused), 1 = natural [E, rows, K/2] + [E, rows, K/32]; the n_shared experts after
// the E routed ones run on every row with weight 1; add [R, H] f32 or null; y [R, H] f32.
SPARK_API int spark_mxfp4_moe_q(const void* xq, const void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1, const void* w3,
                                const void* s3, const void* w2, const void* s2, int layout, int H, int I, int topk, int E, int n_shared, const float* add,
                                float* y, void* ws, hipStream_t st)
{
    if (!shapes_ok(R, H, I, topk, E, n_shared) || (layout != L_T16 && layout != L_NATURAL)) return 1;
    if (const int v = routes_check(idx, true, R, topk, E, st)) return v > 0 ? 6 : 8;              // opt-in host check of the routes
    if (mx_fused_ok(R, H, I, topk, E, n_shared) && !gemm_ok(layout, R, H, I))
        return mx_fused_launch(xq, xs, R, idx, rw, w1, s1, w3, s3, w2, s2, layout, H, I, topk, E, n_shared, add, y, fused_ws(ws, R, H, I, topk, E, n_shared), 0, st);
    if (layout == L_T16)
        return moe_launch<L_T16>((const uint8_t*)xq, (const uint8_t*)xs, R, idx, rw, (const uint8_t*)w1, nullptr, (const uint8_t*)w3, nullptr, (const uint8_t*)w2,
                                 nullptr, H, I, topk, E, n_shared, add, y, (char*)ws + fused_cap(H, I, topk, E, n_shared), 0, st);
    return moe_launch<L_NATURAL>((const uint8_t*)xq, (const uint8_t*)xs, R, idx, rw, (const uint8_t*)w1, (const uint8_t*)s1, (const uint8_t*)w3,
                                 (const uint8_t*)s3, (const uint8_t*)w2, (const uint8_t*)s2, H, I, topk, E, n_shared, add, y, (char*)ws + fused_cap(H, I, topk, E, n_shared), 0, st);
}
extern "C" int ds41_act_quant_fp8(const void* x, void* q, void* s, long long numel, hipStream_t st);
// x bf16 [R, H]: act_quant per 32 first (scratch xq, xs from the caller: R*H and R*H/32 bytes, used beyond 8 rows), then the experts
SPARK_API int spark_mxfp4_moe(const void* x, void* xq, void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1, const void* w3,
                              const void* s3, const void* w2, const void* s2, int layout, int H, int I, int topk, int E, int n_shared, const float* add, float* y,
                              void* ws, hipStream_t st)
{
    if (!shapes_ok(R, H, I, topk, E, n_shared) || (layout != L_T16 && layout != L_NATURAL)) return 1;
    if (const int v = routes_check(idx, true, R, topk, E, st)) return v > 0 ? 6 : 8;              // opt-in host check of the routes
    if (mx_fused_ok(R, H, I, topk, E, n_shared) && !gemm_ok(layout, R, H, I))
        return mx_fused_launch(x, nullptr, R, idx, rw, w1, s1, w3, s3, w2, s2, layout, H, I, topk, E, n_shared, add, y, fused_ws(ws, R, H, I, topk, E, n_shared), 0, st);
    const int rc = ds41_act_quant_fp8(x, xq, xs, (long long)R * H, st);
    if (rc) return rc;
    return spark_mxfp4_moe_q(xq, xs, R, idx, rw, w1, s1, w3, s3, w2, s2, layout, H, I, topk, E, n_shared, add, y, ws, st);
}
// The decode entry: x bf16 [R, H] with xs null (quantised inside the kernel) or E4M3 with scales xs; R <= 8, topk + n_shared <= 16.
// flags bit 0: ws was prepared by spark_mxfp4_moe_ws_init and has only been used by this entry point since (one launch in all);
// flags bit 1: use the several-kernel path (xs must be given).  flags bit 4 (16): y is bf16 [R, H], the binary32 result rounded to nearest even.
SPARK_API int spark_mxfp4_moe_x(const void* x, const void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1, const void* w3,
                                const void* s3, const void* w2, const void* s2, int layout, int H, int I, int topk, int E, int n_shared, const float* add, float* y,
                                void* ws, int flags, hipStream_t st)
{
    if (!shapes_ok(R, H, I, topk, E, n_shared) || (layout != L_T16 && layout != L_NATURAL)) return 1;
    if (const int v = routes_check(idx, true, R, topk, E, st)) return v > 0 ? 6 : 8;              // opt-in host check of the routes
    const int obf16 = (flags & 16) ? 1 : 0;
    if (flags & 2) {
        if (!xs) return 1;
        if (layout == L_T16)
            return moe_launch<L_T16>((const uint8_t*)x, (const uint8_t*)xs, R, idx, rw, (const uint8_t*)w1, nullptr, (const uint8_t*)w3, nullptr,
                                     (const uint8_t*)w2, nullptr, H, I, topk, E, n_shared, add, y, (char*)ws + fused_cap(H, I, topk, E, n_shared), 0, st, 1, obf16);
        return moe_launch<L_NATURAL>((const uint8_t*)x, (const uint8_t*)xs, R, idx, rw, (const uint8_t*)w1, (const uint8_t*)s1, (const uint8_t*)w3,
                                     (const uint8_t*)s3, (const uint8_t*)w2, (const uint8_t*)s2, H, I, topk, E, n_shared, add, y, (char*)ws + fused_cap(H, I, topk, E, n_shared), 0, st,
                                     1, obf16);
    }
    if (!mx_fused_ok(R, H, I, topk, E, n_shared)) return 1;
    return mx_fused_launch(x, xs, R, idx, rw, w1, s1, w3, s3, w2, s2, layout, H, I, topk, E, n_shared, add, y, fused_ws(ws, R, H, I, topk, E, n_shared), flags & 1, st, obf16);
}

// diagnostics: where the several-kernel path (flags bit 1 of spark_mxfp4_moe_x, and every call of more than 8 rows) left the
// act-quantised intermediate of its last call in a spark_mxfp4_moe* workspace: codes hq [P, I] and scale bytes hs [P, I / 32] in
// grouped order, prow [P] = the pair (row * (topk + n_shared) + slot) of each grouped row.  Tests compare them with the oracle's.
SPARK_API int spark_debug_mx_ws_h(void* ws, int R, int H, int I, int topk, int E, int n_shared, void** hq, void** hs, int** prow)
{
    if (!shapes_ok(R, H, I, topk, E, n_shared)) return 1;
    const WsLayout l = ws_layout(R, H, I, topk + n_shared, E + n_shared);
    char* base = (char*)ws + fused_cap(H, I, topk, E, n_shared);
    *hq = base + l.hq; *hs = base + l.hs; *prow = (int*)(base + l.prow);
    return 0;
}

// ================================================================ C ABI: the reference's symbols (hidden size 5120)
// reference ds41_mx.cu:1303-1523, ds41_moe.cu:257-292; Rust declarations engine-rs/src/ds41/kern.rs:5-80.
namespace {
constexpr int DS41_H = 5120;
// The several-kernel region of a ds41_* workspace follows the single-launch region (one size per shape), so that decode calls and
// prefill calls can share a workspace without the latter writing over the former's idle exchange words.
inline char* ds41_region(void* ws, int I, int topk, int E) { return (char*)ws + fused_cap(DS41_H, I, topk, E, 0); }
}

SPARK_API void ds41_moe_mx_set_s2(int on) { g_s2 = on; }
SPARK_API int ds41_moe_mx_get_s2() { return g_s2; }
SPARK_API void ds41_moe_gr16_max(int) {}                       // row-count switch of the reference's item size: one kernel family here
namespace {
size_t g_out_cap = 0;                  // bytes; 0 = not set yet
// The reference caps the per-pair output buffer of a prefill-sized call (512 MiB, DS41_MOE_OUT_MB; reference ds41_mx.cu:1416-1425):
// beyond it the down product and the weighted sum run in 2 or 4 column passes over a buffer of H / passes columns.  The same rule for
// the calls the grouped GEMM takes, whatever their scale layout (the scales' coding does not change a call's row count).
int ds41_rule_passes(int R, int topk)
{
    if (!g_out_cap) {
        const char* e = std::getenv("DS41_MOE_OUT_MB");
        const long mb = e ? std::atol(e) : 0;
        g_out_cap = (size_t)(mb > 0 ? mb : 512) << 20;
    }
    if (R <= 8) return 1;
    const size_t P = (size_t)R * topk;
    int n = 1;
    while (4 * P * DS41_H / n > g_out_cap && n < 4 && (DS41_H / (2 * n)) % GT_COLS == 0) n *= 2;
    return n;
}
// the passes a call really runs in: intermediate widths the grouped GEMM does not take run in one pass over a whole buffer
int ds41_passes(int R, int I, int topk) { return gemm_ok(L_MX8, R, DS41_H, I) ? ds41_rule_passes(R, topk) : 1; }
size_t ds41_ws_total(int R, int I, int topk, int E)
{
    if (!shapes_ok(R, DS41_H, I, topk, E, 0)) return 0;
    return fused_cap(DS41_H, I, topk, E, 0) + ws_layout(R, DS41_H, I, topk, E, ds41_passes(R, I, topk)).total;
}
}  // namespace
// diagnostics: the cap on the per-pair output buffer in bytes (0 = back to DS41_MOE_OUT_MB / 512 MiB)
SPARK_API void spark_debug_mx_out_cap(size_t bytes) { g_out_cap = bytes; }
// diagnostics: the most rows the single launch takes where the grouped GEMM could take the call too (negative: the rule per layout)
SPARK_API void spark_debug_mx_fused_rows(int rows) { g_fused_rows = rows < 0 ? -1 : rows > 8 ? 8 : rows; }
SPARK_API int ds41_moe_mx_col_passes(int R, int topk, int E) { (void)E; return R < 1 || topk < 1 ? 1 : ds41_rule_passes(R, topk); }
namespace {
int g_pair_b16 = -1;                   // -1 = not decided yet (DS41_MOE_PAIR_BF16 in the environment decides at the first call), 0 off, 1 on
// reference ds41_mx.cu:1245-1255: with DS41_MOE_PAIR_BF16=1 (off by default there and here) the prefill-sized calls (more than 64
// rows, the grouped GEMM) keep every pair's down output as bf16 - the binary32 sum rounded once - instead of binary32: half the bytes
// the down product writes and the sum over the pairs reads; the sums over the pairs stay binary32 in the same order
bool pair_b16_on(int R, int I)
{
    if (g_pair_b16 < 0) { const char* e = std::getenv("DS41_MOE_PAIR_BF16"); g_pair_b16 = e && e[0] == '1' ? 1 : 0; }
    return g_pair_b16 == 1 && R > 64 && gemm_ok(L_MX8, R, DS41_H, I);
}
}  // namespace
// diagnostics: 1 / 0 switch the bf16 pair outputs on / off, negative = as the environment says (read again at the next call)
SPARK_API void spark_debug_mx_pair_b16(int on) { g_pair_b16 = on < 0 ? -1 : on ? 1 : 0; }
// whether a call's pair outputs (ds41_moe_mx_ws_ptrs) are bf16; the intermediate width does not enter the reference's signature:
// answered for widths the grouped GEMM takes (every width the reference uses)
SPARK_API int ds41_moe_mx_pair_b16(int R, int topk, int E) { (void)topk; (void)E; return pair_b16_on(R, 2048) ? 1 : 0; }
SPARK_API size_t ds41_moe_mx_ws_bytes(int R, int I, int topk, int E) { return ds41_ws_total(R, I, topk, E); }
SPARK_API size_t ds41_moe_ws_bytes(int R, int I, int topk, int E)
{
    const size_t t = ds41_ws_total(R, I, topk, E);
    return t ? t + align256((size_t)R * DS41_H) + align256((size_t)R * DS41_H / 32) : 0;
}
// weights in the reference's "mx" tile layout (kern.rs:728-734 moe_pack_mx), raw scales [tiles][K/128][8][4]
SPARK_API int ds41_moe_mx_ex(const void* xq, const void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1, const void* w3,
                             const void* s3, const void* w2, const void* s2, int I, const float* add, float* y, void* ws, int topk, int E, int skip_combine,
                             hipStream_t st)
{
    if (R < 1 || I % 128 != 0 || E > 384 || topk < 1) return 1;
    if (skip_combine && ds41_rule_passes(R, topk) > 1) return 1;     // column passes sum as they go (reference ds41_mx.cu:1445)
    if (const int v = routes_check(idx, true, R, topk, E, st)) return v > 0 ? 6 : 8;              // opt-in host check of the routes
    // decode sizes: the whole layer in one launch, straight from the reference's tile layout (same bits as the kernels below)
    if (!skip_combine && mx_fused_ok(R, DS41_H, I, topk, E, 0) && !gemm_ok(L_MX8, R, DS41_H, I))
        return mx_fused_launch(xq, xs, R, idx, rw, w1, s1, w3, s3, w2, s2, g_s2 ? L_MX8S2 : L_MX8, DS41_H, I, topk, E, 0, add, y, ws, 0, st);
    const int np = ds41_passes(R, I, topk), pb = pair_b16_on(R, I) ? 1 : 0;
    if (g_s2)                                                  // s1 / s3 / s2 are 2-bit coded scale blobs
        return moe_launch<L_MX8S2>((const uint8_t*)xq, (const uint8_t*)xs, R, idx, rw, (const uint8_t*)w1, (const uint8_t*)s1, (const uint8_t*)w3,
                                   (const uint8_t*)s3, (const uint8_t*)w2, (const uint8_t*)s2, DS41_H, I, topk, E, 0, add, y, ds41_region(ws, I, topk, E), skip_combine, st, np,
                                   0, pb);
    return moe_launch<L_MX8>((const uint8_t*)xq, (const uint8_t*)xs, R, idx, rw, (const uint8_t*)w1, (const uint8_t*)s1, (const uint8_t*)w3, (const uint8_t*)s3,
                             (const uint8_t*)w2, (const uint8_t*)s2, DS41_H, I, topk, E, 0, add, y, ds41_region(ws, I, topk, E), skip_combine, st, np, 0, pb);
}
SPARK_API int ds41_moe_mx(const void* xq, const void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1, const void* w3,
                          const void* s3, const void* w2, const void* s2, int I, const float* add, float* y, void* ws, int topk, int E, hipStream_t st)
{
    return ds41_moe_mx_ex(xq, xs, R, idx, rw, w1, s1, w3, s3, w2, s2, I, add, y, ws, topk, E, 0, st);
}
SPARK_API int ds41_moe_mx_combine_rows(void* ws, int R, int I, int topk, int E, const float* add, float* y, int r0, int nr, hipStream_t st)
{
    if (r0 < 0 || nr < 1 || r0 + nr > R || ds41_passes(R, I, topk) > 1) return 1;
    const WsLayout l = ws_layout(R, DS41_H, I, topk, E);
    const char* base = ds41_region(ws, I, topk, E);
    const int* pairmap = (const int*)(base + l.pairmap);
    const float* out = (const float*)(base + l.out);
    const int64_t n4 = (int64_t)nr * (DS41_H / 4);
    combine_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, st>>>(out, pairmap + (int64_t)r0 * topk, add ? add + (int64_t)r0 * DS41_H : nullptr,
                                                                 y + (int64_t)r0 * DS41_H, nr, DS41_H, topk, 0, 0, DS41_H, 0, pair_b16_on(R, I) ? 1 : 0);
    return launch_status();
}
SPARK_API int ds41_moe_mx_combine(void* ws, int R, int I, int topk, int E, const float* add, float* y, hipStream_t st)
{
    return ds41_moe_mx_combine_rows(ws, R, I, topk, E, add, y, 0, R, st);
}
SPARK_API int ds41_moe_mx_ws_ptrs(void* ws, int R, int I, int topk, int E, float** out, int** pairmap)
{
    const WsLayout l = ws_layout(R, DS41_H, I, topk, E);
    char* base = ds41_region(ws, I, topk, E);
    *pairmap = (int*)(base + l.pairmap);
    *out = (float*)(base + l.out);
    return 0;
}
// reference ds41_moe.cu:266-291: xq is the act-quantized input as BF16 values; weights in the moe_pack tile layout
// (kern.rs:718-726).  The BF16 values are re-encoded as E4M3 + UE8M0 (exactly: act_quant is idempotent) in the tail of ws.
SPARK_API int ds41_moe(const void* xq, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1, const void* w3, const void* s3,
                       const void* w2, const void* s2, int I, const float* add, float* y, void* ws, int topk, int E, hipStream_t st)
{
    if (R < 1 || I % 128 != 0 || E > 384 || topk < 1) return 1;
    if (const int v = routes_check(idx, true, R, topk, E, st)) return v > 0 ? 6 : 8;              // opt-in host check of the routes
    // decode sizes: one launch; the kernel re-encodes the BF16 values itself (act_quant of act-quantised values is exact)
    if (mx_fused_ok(R, DS41_H, I, topk, E, 0) && !gemm_ok(L_PACK8, R, DS41_H, I))
        return mx_fused_launch(xq, nullptr, R, idx, rw, w1, s1, w3, s3, w2, s2, L_PACK8, DS41_H, I, topk, E, 0, add, y, ws, 0, st);
    char* tail = (char*)ws + ds41_ws_total(R, I, topk, E);
    uint8_t* q = (uint8_t*)tail;
    uint8_t* qs = (uint8_t*)(tail + align256((size_t)R * DS41_H));
    const int rc = ds41_act_quant_fp8(xq, q, qs, (long long)R * DS41_H, st);
    if (rc) return rc;
    return moe_launch<L_PACK8>(q, qs, R, idx, rw, (const uint8_t*)w1, (const uint8_t*)s1, (const uint8_t*)w3, (const uint8_t*)s3, (const uint8_t*)w2,
                               (const uint8_t*)s2, DS41_H, I, topk, E, 0, add, y, ds41_region(ws, I, topk, E), 0, st, ds41_passes(R, I, topk));
}
