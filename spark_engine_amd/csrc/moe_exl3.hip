// Routed EXL3 (4-bit trellis) experts for gfx950: Qwen-style (mul1 codebook) and GLM-style (mcg codebook, clamped SwiGLU).
//
//   out[r] = add[r] + sum_k (slot order) w[r][k] * ( act(x_r @ Wg_e, x_r @ Wu_e) @ Wd_e ),   e = idx[r][k]
//   x @ W = had128( had128(x * suh) @ inner ) * svh                       (reference qwen_exl3.cuh:4-7)
//
// Semantics: reference engine-rs/shim/moe_exl3.cuh:1-13,204-228,272-285,935-1112,1512-1691 (moex::experts),
// qwen_moe.cu:112-116, glm_moe.cu:10-14.  Expert table tab[9][E] of device pointers: gate_tr, up_tr, down_tr,
// gate_suh, up_suh, down_suh, gate_svh, up_svh, down_svh (moe_exl3.cuh:8-9).
//
// MI355X design of the weight stream (the hot loop).  The reference decodes a tile into a 32-lane tensor-core fragment.
// Here a wave64 takes eight adjacent 16x16 tiles (128 output columns of one k-tile, 1 KiB contiguous) per 128-bit load:
// lane (j = lane / 8, m = lane % 8) holds words 4m..4m+3 of tile j = sequence positions 32m..32m+31 = all 16 k rows of
// columns m and m + 8 of that tile.  So a lane owns two output columns outright: no cross-lane reduction over K, only
// the three trailing nibbles of the previous word come from the neighbour lane.  States are cut out of the 64-bit
// window with alignbit / bfe, decoded two at a time (packed fp16 codebook arithmetic) and accumulated with
// v_dot2_f32_f16 against the Hadamard-transformed activations, which are wave-uniform and arrive as scalar loads.
#include "moe_exl3.hpp"
#include "exl3_decode.hpp"
#include "runtime.hpp"

using namespace spk;

namespace {

constexpr int EMAX = 1024;            // experts (one grouping thread each)
constexpr int PMAX = 1024;            // routed pairs per call (decode / verify chains)
constexpr int GV_WAVES = 4;

typedef Exl3Cfg Cfg;
__device__ __forceinline__ float ld_x(const void* x, int xtype, int64_t i) { return exl3_ld_x(x, xtype, i); }
__device__ __forceinline__ int ld_idx(const void* idx, int itype, int i) { return exl3_ld_idx(idx, itype, i); }
__device__ __forceinline__ float ld_w(const void* w, int wtype, int i) { return exl3_ld_w(w, wtype, i); }
__device__ __forceinline__ float act_fn(int act, float a, float u) { return exl3_act(act, a, u); }

// ---------------------------------------------------------------- grouping: pairs -> items of at most GR rows of one expert
// One workgroup for any call size: experts are counted with LDS atomics, a wave-level scan lays out the experts' row ranges and
// items, and a second sweep hands every pair its compact row.  pairmap[p] = compact row of pair p; ppair[row] = p; pexp[row] =
// the row's expert.  The rows of an expert come in no particular order (every row is computed on its own).
// (semantics of the reference's count / scan / fill kernels, moe_exl3.cuh:141-200,961-1014)
constexpr int EBIG = 1024;             // experts the grouping holds
__global__ __launch_bounds__(1024) void group_pairs_kernel(const void* __restrict__ idx, int itype, int R, int topk, int E, int GR, int* __restrict__ G,
                                                           int* __restrict__ gexp, int* __restrict__ goff, int* __restrict__ gcnt, int* __restrict__ pairmap,
                                                           int* __restrict__ ppair, int* __restrict__ pexp, int* __restrict__ geoff, int* __restrict__ gfill)
{
    __shared__ int cnt[EBIG], fill[EBIG], eoff[EBIG];
    __shared__ int wsum[2][16];
    const int tid = threadIdx.x, P = R * topk;
    if (tid < E) { cnt[tid] = 0; fill[tid] = 0; }
    __syncthreads();
    // the first KEEP x 1024 pairs stay in registers between the two sweeps (all their loads in flight at once: 2048 tokens of top-10
    // are 20 a thread); a larger call reads the rest again in the second sweep
    constexpr int KEEP = 24;
    int ev[KEEP];
#pragma unroll
    for (int u = 0; u < KEEP; ++u) ev[u] = clamp_expert(ld_idx(idx, itype, min(tid + u * 1024, P - 1)), E);
#pragma unroll
    for (int u = 0; u < KEEP; ++u) if (tid + u * 1024 < P) atomicAdd(&cnt[ev[u]], 1);
    for (int p0 = tid + KEEP * 1024; p0 < P; p0 += 8 * 1024) {
        int ew[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) ew[u] = clamp_expert(ld_idx(idx, itype, min(p0 + u * 1024, P - 1)), E);
#pragma unroll
        for (int u = 0; u < 8; ++u) if (p0 + u * 1024 < P) atomicAdd(&cnt[ew[u]], 1);
    }
    __syncthreads();
    const int c = tid < E ? cnt[tid] : 0, nit = (c + GR - 1) / GR;
    int rs = c, is = nit;
    const int lane = tid & 63, wv = tid >> 6;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int a = __shfl_up(rs, o, 64), b = __shfl_up(is, o, 64);
        if (lane >= o) { rs += a; is += b; }
    }
    if (lane == 63) { wsum[0][wv] = rs; wsum[1][wv] = is; }
    __syncthreads();
    int rb = 0, ib = 0;
    for (int w = 0; w < wv; ++w) { rb += wsum[0][w]; ib += wsum[1][w]; }
    if (tid == 1023) *G = ib + is;
    if (tid < E) {
        eoff[tid] = rb + rs - c;
        for (int j = 0; j * GR < c; ++j) { const int it = ib + is - nit + j; gexp[it] = tid; goff[it] = rb + rs - c + j * GR; gcnt[it] = min(GR, c - j * GR); }
    }
    if (geoff) {                                           // a large call: the rows are handed out by scatter_pairs_kernel, over many CUs
        if (tid < E) { geoff[tid] = rb + rs - c; gfill[tid] = 0; }
        return;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < KEEP; ++u) {
        const int p = tid + u * 1024;
        if (p < P) {
            const int pos = eoff[ev[u]] + atomicAdd(&fill[ev[u]], 1);
            pairmap[p] = pos; ppair[pos] = p; pexp[pos] = ev[u];
        }
    }
    for (int p0 = tid + KEEP * 1024; p0 < P; p0 += 8 * 1024) {
        int ew[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) ew[u] = clamp_expert(ld_idx(idx, itype, min(p0 + u * 1024, P - 1)), E);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int p = p0 + u * 1024;
            if (p < P) {
                const int pos = eoff[ew[u]] + atomicAdd(&fill[ew[u]], 1);
                pairmap[p] = pos; ppair[pos] = p; pexp[pos] = ew[u];
            }
        }
    }
}

// The second sweep of a large call: one workgroup's stores to 2 P scattered words go through one CU's memory pipeline (17 of that
// kernel's 27 us at 20480 pairs); here a workgroup per 1024 pairs.  It ranks its pairs per expert in LDS, reserves each expert's
// rows with one atomic on the fill counts in memory (an atomic per pair has 40 waiting in line per expert), and stores.
__global__ __launch_bounds__(1024) void scatter_pairs_kernel(const void* __restrict__ idx, int itype, int P, int E, const int* __restrict__ geoff,
                                                             int* __restrict__ gfill, int* __restrict__ pairmap, int* __restrict__ ppair, int* __restrict__ pexp)
{
    __shared__ int lcnt[EBIG], lbase[EBIG];
    const int tid = threadIdx.x, p = (int)blockIdx.x * 1024 + tid;
    if (tid < E) lcnt[tid] = 0;
    __syncthreads();
    const int e = p < P ? clamp_expert(ld_idx(idx, itype, p), E) : 0;
    const int rank = p < P ? atomicAdd(&lcnt[e], 1) : 0;
    __syncthreads();
    if (tid < E) { const int n = lcnt[tid]; lbase[tid] = n ? geoff[tid] + atomicAdd(&gfill[tid], n) : 0; }
    __syncthreads();
    if (p < P) {
        const int pos = lbase[e] + rank;
        pairmap[p] = pos; ppair[pos] = p; pexp[pos] = e;
    }
}

// ---------------------------------------------------------------- xh[t][row][K] = fp16(had128(x[token of row] * suh_t[e])), t = gate, up
// reference moe_exl3.cuh:204-228 (had_grouped_kernel).  Wave per (t, row), sixteen lanes per 128-block with eight values each (16-byte
// accesses: a wave writes 1 KB per store), up to sixteen blocks of the row with their loads in flight together.  VEC: x rows start
// on 16-byte boundaries; else the activations are read two at a time.
template <bool VEC>
__global__ __launch_bounds__(256) void had_rows_kernel(const void* __restrict__ x, int xtype, int64_t ldx, const uint64_t* __restrict__ tab, int E,
                                                       int suh_slot0, int T, int P, int topk, const int* __restrict__ ppair, const int* __restrict__ pexp, int K,
                                                       uint16_t* __restrict__ xh)
{
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63, blk = lane >> 4, l16 = lane & 15;
    const int row = (int)(wave % P), t = (int)(wave / P);
    if (t >= T) return;
    const uint16_t* suh = (const uint16_t*)tab[(int64_t)(suh_slot0 + t) * E + pexp[row]];
    const int64_t src = ppair[row] / topk;
    uint16_t* dst = xh + ((int64_t)t * P + row) * K;
    const int nbk = K / 128;
    for (int kb0 = 0; kb0 < nbk; kb0 += 16) {
        float v[4][8];
        uint4 sv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = min(kb0 + 4 * u + blk, nbk - 1) * 128 + l16 * 8;
            if (xtype == X_F32) {
                const float* xp = (const float*)x + src * ldx + k;
                if (VEC) { const float4 a = *(const float4*)xp, b = *(const float4*)(xp + 4); v[u][0] = a.x; v[u][1] = a.y; v[u][2] = a.z; v[u][3] = a.w; v[u][4] = b.x; v[u][5] = b.y; v[u][6] = b.z; v[u][7] = b.w; }
                else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) { const float2 a = *(const float2*)(xp + 2 * i); v[u][2 * i] = a.x; v[u][2 * i + 1] = a.y; }
                }
            } else {
                const uint16_t* xp = (const uint16_t*)x + src * ldx + k;
                uint32_t w4[4];
                if (VEC) { const uint4 a = *(const uint4*)xp; w4[0] = a.x; w4[1] = a.y; w4[2] = a.z; w4[3] = a.w; }
                else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) w4[i] = *(const uint32_t*)(xp + 2 * i);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (xtype == X_F16) { v[u][2 * i] = f16_bits_to_f32((uint16_t)w4[i]); v[u][2 * i + 1] = f16_bits_to_f32((uint16_t)(w4[i] >> 16)); }
                    else { v[u][2 * i] = __uint_as_float(w4[i] << 16); v[u][2 * i + 1] = __uint_as_float(w4[i] & 0xffff0000u); }
                }
            }
            sv[u] = ld_8h(suh + k);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int kb = kb0 + 4 * u + blk;
            const uint32_t s4[4] = {sv[u].x, sv[u].y, sv[u].z, sv[u].w};
#pragma unroll
            for (int i = 0; i < 4; ++i) { v[u][2 * i] *= f16_bits_to_f32((uint16_t)s4[i]); v[u][2 * i + 1] *= f16_bits_to_f32((uint16_t)(s4[i] >> 16)); }
            fwht128_x8(v[u], lane);          // every lane takes part (a block past the end works on the last block again and stores nothing)
            if (kb < nbk) {
                uint4 o;
                o.x = (uint32_t)f32_to_f16_bits(v[u][0]) | ((uint32_t)f32_to_f16_bits(v[u][1]) << 16);
                o.y = (uint32_t)f32_to_f16_bits(v[u][2]) | ((uint32_t)f32_to_f16_bits(v[u][3]) << 16);
                o.z = (uint32_t)f32_to_f16_bits(v[u][4]) | ((uint32_t)f32_to_f16_bits(v[u][5]) << 16);
                o.w = (uint32_t)f32_to_f16_bits(v[u][6]) | ((uint32_t)f32_to_f16_bits(v[u][7]) << 16);
                st_stream16(dst + kb * 128 + l16 * 8, o);
            }
        }
    }
}

// ---------------------------------------------------------------- what follows a product: done by the kernel that made it
// A wave holds one row of 128 columns, two per lane.  Gate / up sums -> the down product's input; down sums -> the pair's output.
// The order of operations is the reference's (moe_exl3.cuh:935-956,1019-1064): Hadamard, channel scale, activation, sign vector,
// Hadamard, binary16; and Hadamard, channel scale, route weight.
struct GateUpScales { float g0, g1, u0, u1, d0, d1; };
__device__ __forceinline__ GateUpScales gate_up_scales(const uint64_t* __restrict__ tab, int E, int e, int n)
{
    const uint16_t* svg = (const uint16_t*)tab[(int64_t)6 * E + e];
    const uint16_t* svu = (const uint16_t*)tab[(int64_t)7 * E + e];
    const uint16_t* sud = (const uint16_t*)tab[(int64_t)5 * E + e];
    const uint32_t a = *(const uint32_t*)(svg + n), b = *(const uint32_t*)(svu + n), c = *(const uint32_t*)(sud + n);
    return GateUpScales{f16_bits_to_f32((uint16_t)a), f16_bits_to_f32((uint16_t)(a >> 16)), f16_bits_to_f32((uint16_t)b), f16_bits_to_f32((uint16_t)(b >> 16)),
                        f16_bits_to_f32((uint16_t)c), f16_bits_to_f32((uint16_t)(c >> 16))};
}
__device__ __forceinline__ uint32_t down_input(float g0, float g1, float u0, float u1, const GateUpScales& s, int act, int lane)
{
    fwht128(g0, g1, lane);
    fwht128(u0, u1, lane);
    float v0 = act_fn(act, g0 * s.g0, u0 * s.u0) * s.d0;
    float v1 = act_fn(act, g1 * s.g1, u1 * s.u1) * s.d1;
    fwht128(v0, v1, lane);
    return (uint32_t)f32_to_f16_bits(v0) | ((uint32_t)f32_to_f16_bits(v1) << 16);
}
// the same for eight columns a lane (sixteen lanes a 128-block)
__device__ __forceinline__ uint4 down_input_x8(float (&g)[8], float (&u)[8], const uint64_t* __restrict__ tab, int E, int e, int n, int act, int lane)
{
    const uint4 sg = ld_8h((const uint16_t*)tab[(int64_t)6 * E + e] + n), su = ld_8h((const uint16_t*)tab[(int64_t)7 * E + e] + n),
                sd = ld_8h((const uint16_t*)tab[(int64_t)5 * E + e] + n);
    const uint32_t g4[4] = {sg.x, sg.y, sg.z, sg.w}, u4[4] = {su.x, su.y, su.z, su.w}, d4[4] = {sd.x, sd.y, sd.z, sd.w};
    fwht128_x8(g, lane);
    fwht128_x8(u, lane);
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int sh = (i & 1) * 16;
        v[i] = act_fn(act, g[i] * f16_bits_to_f32((uint16_t)(g4[i >> 1] >> sh)), u[i] * f16_bits_to_f32((uint16_t)(u4[i >> 1] >> sh))) * f16_bits_to_f32((uint16_t)(d4[i >> 1] >> sh));
    }
    fwht128_x8(v, lane);
    uint4 o;
    o.x = (uint32_t)f32_to_f16_bits(v[0]) | ((uint32_t)f32_to_f16_bits(v[1]) << 16);
    o.y = (uint32_t)f32_to_f16_bits(v[2]) | ((uint32_t)f32_to_f16_bits(v[3]) << 16);
    o.z = (uint32_t)f32_to_f16_bits(v[4]) | ((uint32_t)f32_to_f16_bits(v[5]) << 16);
    o.w = (uint32_t)f32_to_f16_bits(v[6]) | ((uint32_t)f32_to_f16_bits(v[7]) << 16);
    return o;
}
__device__ __forceinline__ float2 pair_output(float o0, float o1, float sv0, float sv1, float wk, int lane)
{
    fwht128(o0, o1, lane);
    return make_float2(wk * (o0 * sv0), wk * (o1 * sv1));
}

// ---------------------------------------------------------------- the weight stream of items of up to 16 rows (calls of up to 64 rows
// that the single-launch path and the grouped GEMM do not take: tables with per-expert widths, the forced comparison path)
// Workgroup = (128 columns, item), all of K: the four waves interleave over the k-tiles (two in flight each) and are summed through
// LDS in wave order, so the block holds finished sums and does what follows the product itself - no partial sums leave the chip.
//   STAGE 1: gate, then up, over the same rows; -> xh2 [P][I] binary16 (the down product's input)
//   STAGE 2: down; -> pout [P][H] binary32, the pair's finished and weighted output
// MIXED: the experts' trellis widths come from row 9 of the table (3..6 bits, reference moe_exl3.cuh:239-252): a k-tile's 16 x 128
// strip is decoded into LDS with the generic state extraction and multiplied in binary32, thread = column x (even | odd rows).
// vw: row 10 of the table holds the expert's own intermediate width (reference moe_exl3.cuh:63-67,132-136).
template <int CBK, int MR>
__device__ __forceinline__ void tile_fma(const uint4 w, uint32_t prev, const uint32_t* __restrict__ xrow, int64_t ldx32, int rows, float (&acc)[MR][2])
{
    h2 wd[4][4];
    decode_tile32<CBK>(w, prev, wd);
#pragma unroll
    for (int r = 0; r < MR; ++r) {
        if (r >= rows) break;
        dot_tile32(wd, xrow + r * ldx32, acc[r][0], acc[r][1]);   // 8 packed fp16 pairs of this k-tile (wave-uniform address)
    }
}
// sums[r][128]: rows x this block's 128 columns of x[rows][Ke] @ inner[Ke][128 nb ..], Ke = k-tiles kt1 * 16
template <int CBK, int MR, bool MIXED>
__device__ __forceinline__ void item_product(const uint16_t* __restrict__ xrows, int K, const uint32_t* __restrict__ tr, int bits, int Nt, int nb, int kt1, int rows,
                                             float (*red)[MR][128], float (*sums)[128], uint16_t* wl, uint32_t* tw)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if constexpr (!MIXED) {
        float acc[MR][2];
#pragma unroll
        for (int r = 0; r < MR; ++r) { acc[r][0] = 0.f; acc[r][1] = 0.f; }
        const int src = tile_prev_lane(lane);
        const uint32_t* xbase = (const uint32_t*)xrows;    // rows K fp16 = K / 2 words apart
        for (int kt = wave; kt < kt1; kt += 2 * GV_WAVES) {
            const int ktb = kt + GV_WAVES;
            const uint4 wa = ld_stream16(tr + ((int64_t)kt * Nt + nb * 8) * 32 + lane * 4);
            uint4 wb = make_uint4(0u, 0u, 0u, 0u);
            if (ktb < kt1) wb = ld_stream16(tr + ((int64_t)ktb * Nt + nb * 8) * 32 + lane * 4);
            tile_fma<CBK, MR>(wa, __shfl(wa.w, src, 64), xbase + kt * 8, K / 2, rows, acc);
            if (ktb < kt1) tile_fma<CBK, MR>(wb, __shfl(wb.w, src, 64), xbase + ktb * 8, K / 2, rows, acc);
        }
        const int j = lane >> 3, m = lane & 7;
#pragma unroll
        for (int r = 0; r < MR; ++r) { red[wave][r][16 * j + m] = acc[r][0]; red[wave][r][16 * j + m + 8] = acc[r][1]; }
        __syncthreads();
        for (int i = tid; i < rows * 128; i += 64 * GV_WAVES) {
            const int r = i >> 7, c = i & 127;
            float v = red[0][r][c];
#pragma unroll
            for (int w = 1; w < GV_WAVES; ++w) v += red[w][r][c];
            sums[r][c] = v;
        }
    } else {
        const int col = tid & 127, half = tid >> 7, nw = 8 * bits;
        float acc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = 0.f;
        if (bits >= 3 && bits <= 6)
            for (int kt = 0; kt < kt1; ++kt) {
                __syncthreads();
                for (int i = tid; i < 8 * nw; i += 256) tw[(i / nw) * 48 + i % nw] = tr[((int64_t)kt * Nt + nb * 8 + i / nw) * nw + i % nw];
                __syncthreads();
                for (int i = tid; i < 8 * 256; i += 256) {
                    const int tl = i >> 8, p = i & 255;
                    int row, c;
                    tile_pos(p, row, c);
                    const _Float16 v = cb_decode<CBK>(tile_state(tw + tl * 48, bits, p));
                    uint16_t hb; __builtin_memcpy(&hb, &v, 2);
                    wl[row * 128 + tl * 16 + c] = hb;
                }
                __syncthreads();
                float wv[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) wv[r] = f16_bits_to_f32(wl[r * 128 + col]);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int m = 2 * i + half;
                    if (m < rows) {
                        const uint16_t* xr = xrows + (int64_t)m * K + kt * 16;
                        float a = acc[i];
#pragma unroll
                        for (int r = 0; r < 16; ++r) a = __builtin_fmaf(f16_bits_to_f32(xr[r]), wv[r], a);
                        acc[i] = a;
                    }
                }
            }
#pragma unroll
        for (int i = 0; i < 8; ++i) { const int m = 2 * i + half; if (m < rows) sums[m][col] = acc[i]; }
    }
    __syncthreads();
}

template <int CBK, int MR, bool MIXED, int STAGE>
__global__ __launch_bounds__(64 * GV_WAVES) void item_kernel(const uint16_t* __restrict__ xh, const uint64_t* __restrict__ tab, int E, const int* __restrict__ G,
                                                             const int* __restrict__ gexp, const int* __restrict__ goff, const int* __restrict__ gcnt, int P, int K,
                                                             int N, int act, int vw, const int* __restrict__ ppair, const void* __restrict__ w, int wtype,
                                                             uint16_t* __restrict__ xh2, float* __restrict__ pout)
{
    constexpr int SR = MIXED ? 16 : MR;
    __shared__ float red[MIXED ? 1 : GV_WAVES][MR][128];
    __shared__ float sums[STAGE == 1 ? 2 : 1][SR][128];
    __shared__ uint16_t wl[MIXED ? 16 * 128 : 8];
    __shared__ uint32_t tw[MIXED ? 8 * 48 : 8];
    const int g = blockIdx.y, nb = blockIdx.x;
    if (g >= *G) return;
    // the host asks the grouping for items of at most this instance's rows (gr_of_rows), so the bound never bites; it stays as the
    // guarantee that the arrays below cannot be overrun whatever the grouping wrote
    const int rows = min(gcnt[g], SR), e = gexp[g], row0 = goff[g];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int bits_raw = MIXED ? (int)tab[(int64_t)9 * E + e] : 4;
    // a width the format does not have (row 9 outside 3..6): the expert contributes nothing - its products run over no k-tiles, so its
    // rows are finished and stored as zeros like any others (nothing downstream reads memory nobody wrote)
    const bool bits_ok = bits_raw >= 3 && bits_raw <= 6;
    const int bits = bits_ok ? bits_raw : 4;
    // vw: the expert's own intermediate width replaces N (gate / up) or K (down); strides keep N / K
    const int we = vw ? (int)tab[(int64_t)10 * E + e] : 0;
    const int Ne = vw && STAGE == 1 ? we : N, Ke = !bits_ok ? 0 : vw && STAGE == 2 ? we : K;
    if (nb * 128 >= Ne) return;
    const int n = nb * 128 + 2 * lane;
    if constexpr (STAGE == 1) {
        const GateUpScales sc = gate_up_scales(tab, E, e, n);
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const uint32_t* tr = (const uint32_t*)tab[(int64_t)t * E + e];
            item_product<CBK, MR, MIXED>(xh + ((int64_t)t * P + row0) * K, K, tr, bits, Ne / 16, nb, Ke / 16, rows, red, sums[t], wl, tw);
        }
        for (int r = wave; r < rows; r += GV_WAVES) {
            const float2 gg = *(const float2*)&sums[0][r][2 * lane], uu = *(const float2*)&sums[1][r][2 * lane];
            *(uint32_t*)(xh2 + (int64_t)(row0 + r) * N + n) = down_input(gg.x, gg.y, uu.x, uu.y, sc, act, lane);
        }
    } else {
        const uint16_t* svd = (const uint16_t*)tab[(int64_t)8 * E + e];
        const uint32_t sv = *(const uint32_t*)(svd + n);
        const uint32_t* tr = (const uint32_t*)tab[(int64_t)2 * E + e];
        item_product<CBK, MR, MIXED>(xh + (int64_t)row0 * K, K, tr, bits, N / 16, nb, Ke / 16, rows, red, sums[0], wl, tw);
        for (int r = wave; r < rows; r += GV_WAVES) {
            const float2 oo = *(const float2*)&sums[0][r][2 * lane];
            const float wk = ld_w(w, wtype, ppair[row0 + r]);
            *(float2*)(pout + (int64_t)(row0 + r) * N + n) = pair_output(oo.x, oo.y, f16_bits_to_f32((uint16_t)sv), f16_bits_to_f32((uint16_t)(sv >> 16)), wk, lane);
        }
    }
}

// ---------------------------------------------------------------- out[r] = add[r] + sum_k pout[pairmap[r, k]], k ascending (the pairs arrive
// finished and weighted); thread = four columns of a token row
__global__ __launch_bounds__(256) void sum_pairs_kernel(const float* __restrict__ pout, const int* __restrict__ pairmap, const float* __restrict__ add,
                                                        float* __restrict__ out, int R, int H, int topk, int obf16)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int h4 = H >> 2;
    if (i >= (int64_t)R * h4) return;
    const int r = (int)(i / h4), col = (int)(i % h4) * 4;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k = 0; k < topk; ++k) {
        const uint4 v = ld_stream16(pout + (int64_t)pairmap[r * topk + k] * H + col);       // read once
        acc.x += __uint_as_float(v.x); acc.y += __uint_as_float(v.y); acc.z += __uint_as_float(v.z); acc.w += __uint_as_float(v.w);
    }
    if (add) { const float4 b = *(const float4*)(add + (int64_t)r * H + col); acc.x = b.x + acc.x; acc.y = b.y + acc.y; acc.z = b.z + acc.z; acc.w = b.w + acc.w; }
    if (obf16) *(uint2*)((uint16_t*)out + (int64_t)r * H + col) = make_uint2((uint32_t)f32_to_bf16(acc.x) | ((uint32_t)f32_to_bf16(acc.y) << 16),
                                                                              (uint32_t)f32_to_bf16(acc.z) | ((uint32_t)f32_to_bf16(acc.w) << 16));
    else *(float4*)(out + (int64_t)r * H + col) = acc;
}

// ================================================================ prefill: grouped GEMM over 64-row items
// With many rows per expert the item kernels above decode every weight once per 16 rows; here a block owns 64 item rows x 128 output
// columns for the whole K range and decodes each weight once: every wave decodes the tiles of its own 32 columns straight into the
// operands of v_mfma_f32_16x16x32_f16 (weights = A, activations = B; binary32 accumulate; gemm_pass below), the item's transformed
// activation rows are staged in LDS, and the next chunk's loads are in flight during the decode and the multiplies.  The down
// product is finished in the same block: its sums go through LDS, 32 rows at a time, to the wave-per-row routine above.  Gate and
// up stay two blocks (blockIdx.z) that write their sums, and a small kernel turns them into the down product's input: one block
// doing both passes and the transforms measured slower (313 us against 206 + 49 for 2048 tokens of the 512-expert layer: the
// transforms are vector-ALU work, and so is the decode that bounds this kernel).
// reference moe_exl3.cuh:520-1370 (gux_kernel, gemm_grouped_kernel): decode once, tensor-core multiply.
constexpr int PG_ROWS = 64;            // rows of a prefill item
constexpr int PG_KT = 4;              // k-tiles per chunk of the grouped GEMM

typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
// eight halfs from LDS at an 8-byte boundary (rows are 8 bytes apart in their phase: two 8-byte reads)
__device__ __forceinline__ v8h ld_v8h(const uint16_t* p)
{
    const uint2 lo = *(const uint2*)p, hi = *(const uint2*)(p + 4);
    const uint4 u = make_uint4(lo.x, lo.y, hi.x, hi.y);
    v8h r;
    __builtin_memcpy(&r, &u, 16);
    return r;
}

// acc[rt][nt] += rows (64) x this wave's 32 columns over all of K; smem = the activation buffers
// xstride: halfs between activation rows (the widest expert's K where experts have their own intermediate widths)
// A wave owns two column tiles and decodes them itself, straight into matrix operands: its lane (c = lane % 16, q = lane / 16) holds
// the tile of k-tile q of the chunk and column tile c / 8 of its two, words m = c % 8 - all 16 k of tile columns m and m + 8.  A
// decoded lane's rows 0..7 (8..15) of one column are exactly one operand of the 32-deep instruction, whose k runs over the four
// lanes q = 0..3 of a column: one instruction multiplies rows 0..7 of the chunk's four k-tiles, the next rows 8..15, for tile columns
// m (accumulator 0) and again for m + 8 (accumulator 1); the activation operand follows the same k.  Output row i of accumulator nt
// is column 16 (i / 8) + i % 8 + 8 nt of the wave's 32 (gemm_col below).  No weight passes through LDS; the activation rows are
// staged in two buffers in turn, one barrier a chunk.
__device__ __forceinline__ int gemm_col(int q, int nt) { return (q >> 1) * 16 + (q & 1) * 4 + nt * 8; }      // first of the lane's four columns
template <int CBK, int KT, int BITS>
__device__ __forceinline__ void gemm_pass(const uint16_t* __restrict__ xrows, int64_t xstride, int rows, int K, const uint32_t* __restrict__ tr, int Nt, int nb,
                                          unsigned char* smem, v4f (&acc)[4][2])
{
    static_assert(KT == 4, "a chunk is the four k-tiles of the four lane groups");
    constexpr int LD = KT * 16 + 4;                     // halfs per LDS row: the chunk + 4 (8-byte operand reads down a column of rows hit distinct banks)
    constexpr int XV = KT / 2;                          // 16-byte loads per thread of the activation stage (a quarter of the chunk)
    uint16_t* xl = (uint16_t*)smem;                     // [2][64 rows][k of the chunk]
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), c = lane & 15, q = lane >> 4;
    const int nrt = (rows + 15) >> 4, nch = K / (16 * KT);
    const int srow = tid >> 2, spart = tid & 3;         // staging role: thread = (row, quarter of the chunk's K)
    constexpr int TWORDS = 8 * BITS;                    // words of a 16 x 16 tile
    const uint16_t* xsrc = xrows + (int64_t)min(srow, rows - 1) * xstride + spart * (XV * 8);
    const uint32_t* wsrc = tr + ((int64_t)q * Nt + nb * 8 + 2 * wave + (c >> 3)) * TWORDS + (c & 7) * BITS;
    const int src = tile_prev_lane(lane);
    uint4 xa[XV];
#pragma unroll
    for (int i = 0; i < XV; ++i) xa[i] = *(const uint4*)(xsrc + i * 8);
    TileW<BITS> wt = ld_tile<BITS>(wsrc);
#pragma unroll
    for (int i = 0; i < XV; ++i) {
        uint2* d = (uint2*)&xl[srow * LD + spart * (XV * 8) + i * 8];
        d[0] = make_uint2(xa[i].x, xa[i].y); d[1] = make_uint2(xa[i].z, xa[i].w);
    }
    __syncthreads();
    for (int ch = 0; ch < nch; ++ch) {
        const uint16_t* xb = xl + (ch & 1) * (PG_ROWS * LD);
        // ---- the next chunk's loads, in flight during the decode and the multiplies (past the end: the last chunk again, unused)
        const int cn = min(ch + 1, nch - 1);
#pragma unroll
        for (int i = 0; i < XV; ++i) xa[i] = *(const uint4*)(xsrc + cn * (16 * KT) + i * 8);
        const TileW<BITS> wn = ld_tile<BITS>(wsrc + (int64_t)cn * KT * Nt * TWORDS);
        // ---- this chunk's tile into operands: [column m | m + 8][rows 0..7 | 8..15]
        h2 wd[4][4];
        decode_tile32b<CBK, BITS>(wt, __shfl(wt.w[BITS - 1], src, 64), wd);
        v8h a[2][2];
#pragma unroll
        for (int cc = 0; cc < 2; ++cc)
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                uint32_t u[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) __builtin_memcpy(&u[j], &wd[j][2 * cc + hh], 4);
                __builtin_memcpy(&a[cc][hh], u, 16);
            }
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            if (rt < nrt) {
                const v8h b0 = ld_v8h(&xb[(rt * 16 + c) * LD + 16 * q]), b1 = ld_v8h(&xb[(rt * 16 + c) * LD + 16 * q + 8]);
                acc[rt][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[0][0], b0, acc[rt][0], 0, 0, 0);
                acc[rt][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[1][0], b0, acc[rt][1], 0, 0, 0);
                acc[rt][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[0][1], b1, acc[rt][0], 0, 0, 0);
                acc[rt][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[1][1], b1, acc[rt][1], 0, 0, 0);
            }
        }
        // ---- the next chunk's activation rows into the other buffer (its last readers passed the barrier below a chunk ago)
        {
            uint16_t* xn = xl + ((ch + 1) & 1) * (PG_ROWS * LD);
#pragma unroll
            for (int i = 0; i < XV; ++i) {
                uint2* d = (uint2*)&xn[srow * LD + spart * (XV * 8) + i * 8];
                d[0] = make_uint2(xa[i].x, xa[i].y); d[1] = make_uint2(xa[i].z, xa[i].w);
            }
        }
        wt = wn;
        __syncthreads();
    }
}

// grid (N / 128, Gmax, STAGE 1 ? 2 : 1), 4 waves.  STAGE 1: xh [2][P][K] fp16 (rows = compact pair rows) -> part [2][P][N] binary32, gate and up
// sums (blockIdx.z); STAGE 2: xh [P][K] -> pout [P][N] binary32, the pairs' finished and weighted outputs.
// MIXED: the expert's trellis width (3..6 bits) comes from row 9 of the table and selects the instance of the weight stream and decode;
// vw: row 10 holds the expert's own intermediate width (its N in stage 1, its K in stage 2; the buffers keep the strides N / K).
template <int CBK, int KT, int STAGE, bool MIXED>
__global__ __launch_bounds__(256, 6) void gemm_kernel(const uint16_t* __restrict__ xh, const uint64_t* __restrict__ tab, int E, const int* __restrict__ G,
                                                   const int* __restrict__ gexp, const int* __restrict__ goff, const int* __restrict__ gcnt, int P, int K, int N,
                                                   const int* __restrict__ ppair, const void* __restrict__ w, int wtype, float* __restrict__ part,
                                                   float* __restrict__ pout, int vw)
{
    constexpr int LD = KT * 16 + 4;
    constexpr int CHUNK_BYTES = 2 * PG_ROWS * LD * 2, EP_BYTES = STAGE == 2 ? 32 * 128 * 4 : 0;         // the epilogue reuses the activation buffers
    __shared__ __align__(16) unsigned char smem[CHUNK_BYTES > EP_BYTES ? CHUNK_BYTES : EP_BYTES];
    const int g = blockIdx.y, nb = blockIdx.x, t = STAGE == 1 ? blockIdx.z : 2;
    if (g >= *G) return;
    const int rows = gcnt[g], e = gexp[g], row0 = goff[g];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), c = lane & 15, q = lane >> 4;
    const int we = vw ? (int)tab[(int64_t)10 * E + e] : 0;
    const int Ne = vw && STAGE == 1 ? we : N, Ke = vw && STAGE == 2 ? we : K;
    if (nb * 128 >= Ne) return;
    v4f acc[4][2];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) acc[rt][nt] = v4f{0.f, 0.f, 0.f, 0.f};
    {
        const uint16_t* xrows = xh + ((int64_t)(STAGE == 1 ? t : 0) * P + row0) * K;
        const uint32_t* tr = (const uint32_t*)tab[(int64_t)t * E + e];
        if constexpr (!MIXED) gemm_pass<CBK, KT, 4>(xrows, K, rows, Ke, tr, Ne / 16, nb, smem, acc);
        else {
            switch ((int)tab[(int64_t)9 * E + e]) {
                case 3: gemm_pass<CBK, KT, 3>(xrows, K, rows, Ke, tr, Ne / 16, nb, smem, acc); break;
                case 4: gemm_pass<CBK, KT, 4>(xrows, K, rows, Ke, tr, Ne / 16, nb, smem, acc); break;
                case 5: gemm_pass<CBK, KT, 5>(xrows, K, rows, Ke, tr, Ne / 16, nb, smem, acc); break;
                case 6: gemm_pass<CBK, KT, 6>(xrows, K, rows, Ke, tr, Ne / 16, nb, smem, acc); break;
                default: break;                                 // a width the format does not have: the expert contributes nothing, zeros are stored
            }
        }
    }
    // D: lane = row c of the row tile, four columns from gemm_col(q, nt) on of the wave's 32
    if constexpr (STAGE == 1) {
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) {
            const int row = rt * 16 + c;
            if (row < rows) {
#pragma unroll
                for (int nt = 0; nt < 2; ++nt)
                    *(float4*)(part + ((int64_t)t * P + row0 + row) * N + nb * 128 + wave * 32 + gemm_col(q, nt)) = make_float4(acc[rt][nt][0], acc[rt][nt][1], acc[rt][nt][2], acc[rt][nt][3]);
            }
        }
    } else {
        // ---- finished in place, 32 rows at a time through LDS: Hadamard, channel scale, route weight; sixteen lanes a row with eight
        // columns each (the butterflies of pair_output in the same order: the same bits), four rows a wave instruction
        const int rr = lane >> 4, l16 = lane & 15, n = nb * 128 + 8 * l16;
        const uint4 sv4 = ld_8h((const uint16_t*)tab[(int64_t)8 * E + e] + n);
        const uint32_t svw[4] = {sv4.x, sv4.y, sv4.z, sv4.w};
        float* ep = (float*)smem;                           // [32 rows][128 columns]
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            if (hf * 32 >= rows) break;
#pragma unroll
            for (int r2 = 0; r2 < 2; ++r2)
#pragma unroll
                for (int nt = 0; nt < 2; ++nt)
                    *(float4*)&ep[(r2 * 16 + c) * 128 + wave * 32 + gemm_col(q, nt)] =
                        make_float4(acc[2 * hf + r2][nt][0], acc[2 * hf + r2][nt][1], acc[2 * hf + r2][nt][2], acc[2 * hf + r2][nt][3]);
            __syncthreads();
#pragma unroll
            for (int it = 0; it < 2; ++it) {
                const int r = wave * 8 + it * 4 + rr;           // every lane takes part in the exchanges; rows past the item's end store nothing
                const bool live = hf * 32 + r < rows;
                const float4 v0 = *(const float4*)&ep[r * 128 + 8 * l16], v1 = *(const float4*)&ep[r * 128 + 8 * l16 + 4];
                float v[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
                const float wk = live ? ld_w(w, wtype, ppair[row0 + hf * 32 + r]) : 0.f;
                fwht128_x8(v, lane);
                float o[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) o[i] = wk * (v[i] * f16_bits_to_f32((uint16_t)(svw[i >> 1] >> (16 * (i & 1)))));
                if (live) {
                    float* dst = pout + (int64_t)(row0 + hf * 32 + r) * N + n;
                    *(float4*)dst = make_float4(o[0], o[1], o[2], o[3]);
                    *(float4*)(dst + 4) = make_float4(o[4], o[5], o[6], o[7]);
                }
            }
            __syncthreads();
        }
    }
}

// gate / up sums of the grouped GEMM -> the down product's input: wave per (compact row, four 128-blocks of columns), sixteen lanes a
// block with eight columns each
__global__ __launch_bounds__(256) void down_input_kernel(const float* __restrict__ part, const uint64_t* __restrict__ tab, int E, int P, int I, int act,
                                                         const int* __restrict__ pexp, uint16_t* __restrict__ xh2, int vw)
{
    const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63, nb = I / 128, wpr = (nb + 3) / 4;
    const int row = (int)(wave / wpr), blk = (int)(wave % wpr) * 4 + (lane >> 4);
    if (row >= P) return;
    const int e = pexp[row];
    const int width = vw ? (int)tab[(int64_t)10 * E + e] : I;                // past the expert's own width nothing was summed
    const int n = min(blk, nb - 1) * 128 + (lane & 15) * 8;
    const float* gp = part + (int64_t)row * I + n;
    const float* up = part + ((int64_t)P + row) * I + n;
    // the sums are read once and the result is read by the next kernel only: streaming loads and store
    const uint4 g0 = ld_stream16(gp), g1 = ld_stream16(gp + 4), u0 = ld_stream16(up), u1 = ld_stream16(up + 4);
    float g[8] = {__uint_as_float(g0.x), __uint_as_float(g0.y), __uint_as_float(g0.z), __uint_as_float(g0.w),
                  __uint_as_float(g1.x), __uint_as_float(g1.y), __uint_as_float(g1.z), __uint_as_float(g1.w)};
    float u[8] = {__uint_as_float(u0.x), __uint_as_float(u0.y), __uint_as_float(u0.z), __uint_as_float(u0.w),
                  __uint_as_float(u1.x), __uint_as_float(u1.y), __uint_as_float(u1.z), __uint_as_float(u1.w)};
    const uint4 o = down_input_x8(g, u, tab, E, e, n, act, lane);            // every lane takes part; blocks past the end store nothing
    if (blk < nb && blk * 128 < width) st_stream16(xh2 + (int64_t)row * I + n, o);
}

// ---------------------------------------------------------------- host side
// One workspace layout for both row ranges: the grouping arrays, the transformed inputs of gate and up, the down input, the pairs' outputs.
struct Plan { int P, Gmax; size_t G, gexp, goff, gcnt, geoff, gfill, pairmap, ppair, pexp, xh1, xh2, pout, part, total; };
inline Plan plan(const Cfg& c, int R, int GR)
{
    Plan p;
    p.P = R * c.topk;
    p.Gmax = (p.P < c.E ? p.P : c.E) + p.P / GR + 1;    // items: an expert's rows go GR to an item (the last one short)
    size_t o = 0;
    auto take = [&](size_t n) { const size_t q = o; o += align256(n); return q; };
    p.G = take(16);
    p.gexp = take(4 * (size_t)p.Gmax); p.goff = take(4 * (size_t)p.Gmax); p.gcnt = take(4 * (size_t)p.Gmax);
    p.geoff = take(4 * (size_t)EBIG); p.gfill = take(4 * (size_t)EBIG);
    p.pairmap = take(4 * (size_t)p.P); p.ppair = take(4 * (size_t)p.P); p.pexp = take(4 * (size_t)p.P);
    p.xh1 = take(2 * (size_t)p.P * c.H * 2);
    p.xh2 = take((size_t)p.P * c.I * 2);
    p.pout = take(4 * (size_t)p.P * c.H);
    p.part = take(GR == PG_ROWS ? 4 * (size_t)2 * p.P * c.I : 0);      // gate / up sums of the grouped GEMM
    p.total = o;
    return p;
}
constexpr int GR_ITEM = 16;            // most rows of an item of the item kernels
// Rows of an item for a call of R rows = the row count of the kernel instance the call runs (1, 2, 4, 8, 16).  With valid routes an
// expert has at most R rows anyway; a token row that names an expert twice then gives that expert a second item instead of an item
// larger than the instance's arrays, and its pairs are all multiplied and summed.
inline int gr_of_rows(int R, bool mixed) { return mixed || R > 8 ? GR_ITEM : R <= 1 ? 1 : R <= 2 ? 2 : R <= 4 ? 4 : 8; }
inline bool cfg_ok(const Cfg& c, int R)
{
    return R >= 1 && c.E >= 1 && c.E <= EMAX && c.topk >= 1 && c.topk <= 64 && (int64_t)R * c.topk <= PMAX && R <= 64 && c.H >= 128 && c.I >= 128 &&
           c.H % 128 == 0 && c.I % 128 == 0 && (c.cbk == CB_MCG || c.cbk == CB_MUL1);
}

// The single-launch path's region comes first in a workspace and has one size per shape (that of the most rows the path takes),
// so calls of any size can share a workspace without writing over its idle exchange words.
inline size_t fused_cap(const Cfg& c)
{
    for (int r = 8; r >= 1; --r)
        if (exl3_fused_ok(c, r)) return exl3_fused_ws_bytes(c, r);
    return 0;
}

template <int CBK, bool MIXED, int STAGE, class... A>
void launch_items(int maxrows, dim3 grid, hipStream_t st, A... a)
{
    const dim3 blk(64 * GV_WAVES);
    if (MIXED) { item_kernel<CBK, 16, MIXED, STAGE><<<grid, blk, 0, st>>>(a...); return; }
    // one instantiation per row-count class of the call (items never hold more rows than the call has)
    if (maxrows <= 1) item_kernel<CBK, 1, false, STAGE><<<grid, blk, 0, st>>>(a...);
    else if (maxrows <= 2) item_kernel<CBK, 2, false, STAGE><<<grid, blk, 0, st>>>(a...);
    else if (maxrows <= 4) item_kernel<CBK, 4, false, STAGE><<<grid, blk, 0, st>>>(a...);
    else if (maxrows <= 8) item_kernel<CBK, 8, false, STAGE><<<grid, blk, 0, st>>>(a...);
    else item_kernel<CBK, 16, false, STAGE><<<grid, blk, 0, st>>>(a...);
}

// flags: bit 0 = the workspace is prepared (once, then only used by these calls);
//        bit 1 = force the item kernels; bit 2 = mixed trellis widths (table row 9 = bits per expert);
//        bit 3 = every expert has its own intermediate width (table row 10, a multiple of 128 up to I)
int experts(const Cfg& c, const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out, void* ws,
            int flags, hipStream_t st)
{
    if (!cfg_ok(c, R) || (ldx & 1)) return -1;       // rows start on even elements (two activations per access)
    const bool mixed = (flags & 4) != 0;             // the table has a row 9 with every expert's trellis width (3..6 bits)
    const bool varw = (flags & 8) != 0;              // and a row 10 with every expert's intermediate width (reference moe_exl3.cuh:63-67,132-136)
    if (!(flags & 2) && exl3_fused_ok(c, R)) {
        Cfg cf = c;
        cf.mixed = mixed ? 1 : 0;
        cf.varw = varw ? 1 : 0;
        return exl3_fused_launch(cf, x, ldx, R, idx, w, tab, add, out, ws, flags & 1, st);
    }
    const int gr = gr_of_rows(R, mixed);
    const Plan p = plan(c, R, gr);
    char* b = (char*)ws + fused_cap(c);              // the two paths never share workspace bytes
    int* G = (int*)(b + p.G);
    int *gexp = (int*)(b + p.gexp), *goff = (int*)(b + p.goff), *gcnt = (int*)(b + p.gcnt);
    int *pairmap = (int*)(b + p.pairmap), *ppair = (int*)(b + p.ppair), *pexp = (int*)(b + p.pexp);
    uint16_t* xh1 = (uint16_t*)(b + p.xh1);
    uint16_t* xh2 = (uint16_t*)(b + p.xh2);
    float* pout = (float*)(b + p.pout);
    const uint64_t* tb = (const uint64_t*)tab;
    const int maxrows = R < GR_ITEM ? R : GR_ITEM, vw = varw ? 1 : 0;
    group_pairs_kernel<<<1, 1024, 0, st>>>(idx, c.itype, R, c.topk, c.E, gr, G, gexp, goff, gcnt, pairmap, ppair, pexp, nullptr, nullptr);
    const int64_t waves = (int64_t)2 * p.P;
    // x rows on 16-byte boundaries (every layout the callers have): whole 16-byte reads
    if ((uintptr_t)x % 16 == 0 && ldx % (c.xtype == X_F32 ? 4 : 8) == 0)
        had_rows_kernel<true><<<(unsigned)((waves + 3) / 4), 256, 0, st>>>(x, c.xtype, ldx, tb, c.E, 3, 2, p.P, c.topk, ppair, pexp, c.H, xh1);
    else
        had_rows_kernel<false><<<(unsigned)((waves + 3) / 4), 256, 0, st>>>(x, c.xtype, ldx, tb, c.E, 3, 2, p.P, c.topk, ppair, pexp, c.H, xh1);
    const dim3 g1(c.I / 128, p.Gmax), g2(c.H / 128, p.Gmax);
#define ITEMS(CB, MX)                                                                                                                                   \
    do {                                                                                                                                                \
        launch_items<CB, MX, 1>(maxrows, g1, st, (const uint16_t*)xh1, tb, c.E, (const int*)G, (const int*)gexp, (const int*)goff, (const int*)gcnt, p.P, c.H, c.I, \
                                c.act, vw, (const int*)ppair, w, c.wtype, xh2, pout);                                                                  \
        launch_items<CB, MX, 2>(maxrows, g2, st, (const uint16_t*)xh2, tb, c.E, (const int*)G, (const int*)gexp, (const int*)goff, (const int*)gcnt, p.P, c.I, c.H, \
                                c.act, vw, (const int*)ppair, w, c.wtype, xh2, pout);                                                                  \
    } while (0)
    if (c.cbk == CB_MCG) { if (mixed) ITEMS(CB_MCG, true); else ITEMS(CB_MCG, false); }
    else { if (mixed) ITEMS(CB_MUL1, true); else ITEMS(CB_MUL1, false); }
#undef ITEMS
    const int64_t n4 = (int64_t)R * (c.H / 4);
    sum_pairs_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, st>>>(pout, pairmap, (const float*)add, (float*)out, R, c.H, c.topk, c.obf16);
    return launch_status();
}

// ---- more than 8 rows of a uniform 4-bit table: grouped GEMM over 64-row items
inline bool big_ok(const Cfg& c, int R)
{
    return R > 8 && c.E >= 1 && c.E <= EBIG && c.topk >= 1 && c.topk <= 64 && (int64_t)R * c.topk < (1ll << 24) && c.H >= 128 && c.I >= 128 &&
           c.H % 128 == 0 && c.I % 128 == 0 && (c.cbk == CB_MCG || c.cbk == CB_MUL1);
}
int experts_big(const Cfg& c, const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out, void* ws,
                int flags, hipStream_t st)
{
    const bool mixed = (flags & 4) != 0;
    const int vw = (flags & 8) ? 1 : 0;
    const Plan p = plan(c, R, PG_ROWS);
    char* b = (char*)ws + fused_cap(c);
    int* G = (int*)(b + p.G);
    int *gexp = (int*)(b + p.gexp), *goff = (int*)(b + p.goff), *gcnt = (int*)(b + p.gcnt);
    int *pairmap = (int*)(b + p.pairmap), *ppair = (int*)(b + p.ppair), *pexp = (int*)(b + p.pexp);
    uint16_t* xh1 = (uint16_t*)(b + p.xh1);
    uint16_t* xh2 = (uint16_t*)(b + p.xh2);
    float* pout = (float*)(b + p.pout);
    const uint64_t* tb = (const uint64_t*)tab;
    if (p.P > 4096) {
        int *geoff = (int*)(b + p.geoff), *gfill = (int*)(b + p.gfill);
        group_pairs_kernel<<<1, 1024, 0, st>>>(idx, c.itype, R, c.topk, c.E, PG_ROWS, G, gexp, goff, gcnt, pairmap, ppair, pexp, geoff, gfill);
        scatter_pairs_kernel<<<(unsigned)((p.P + 1023) / 1024), 1024, 0, st>>>(idx, c.itype, p.P, c.E, geoff, gfill, pairmap, ppair, pexp);
    } else
        group_pairs_kernel<<<1, 1024, 0, st>>>(idx, c.itype, R, c.topk, c.E, PG_ROWS, G, gexp, goff, gcnt, pairmap, ppair, pexp, nullptr, nullptr);
    const int64_t waves = (int64_t)2 * p.P;
    // x rows on 16-byte boundaries (every layout the callers have): whole 16-byte reads
    if ((uintptr_t)x % 16 == 0 && ldx % (c.xtype == X_F32 ? 4 : 8) == 0)
        had_rows_kernel<true><<<(unsigned)((waves + 3) / 4), 256, 0, st>>>(x, c.xtype, ldx, tb, c.E, 3, 2, p.P, c.topk, ppair, pexp, c.H, xh1);
    else
        had_rows_kernel<false><<<(unsigned)((waves + 3) / 4), 256, 0, st>>>(x, c.xtype, ldx, tb, c.E, 3, 2, p.P, c.topk, ppair, pexp, c.H, xh1);
    float* part = (float*)(b + p.part);
    const dim3 g1(c.I / 128, p.Gmax, 2), g2(c.H / 128, p.Gmax);
    const int64_t wv = (int64_t)p.P * ((c.I / 128 + 3) / 4);
#define GEMM(CB, STAGE, MX, GRID, XH, KK, NN) \
    gemm_kernel<CB, PG_KT, STAGE, MX><<<GRID, 256, 0, st>>>(XH, tb, c.E, G, gexp, goff, gcnt, p.P, KK, NN, ppair, w, c.wtype, part, pout, vw)
#define GEMM_STAGE(STAGE, GRID, XH, KK, NN)                                                                        \
    do {                                                                                                           \
        if (c.cbk == CB_MCG) { if (mixed) GEMM(CB_MCG, STAGE, true, GRID, XH, KK, NN); else GEMM(CB_MCG, STAGE, false, GRID, XH, KK, NN); } \
        else { if (mixed) GEMM(CB_MUL1, STAGE, true, GRID, XH, KK, NN); else GEMM(CB_MUL1, STAGE, false, GRID, XH, KK, NN); }               \
    } while (0)
    GEMM_STAGE(1, g1, xh1, c.H, c.I);
    down_input_kernel<<<(unsigned)((wv + 3) / 4), 256, 0, st>>>(part, tb, c.E, p.P, c.I, c.act, pexp, xh2, vw);
    GEMM_STAGE(2, g2, xh2, c.I, c.H);
#undef GEMM_STAGE
#undef GEMM
    const int64_t n4 = (int64_t)R * (c.H / 4);
    sum_pairs_kernel<<<(unsigned)((n4 + 255) / 256), 256, 0, st>>>(pout, pairmap, (const float*)add, (float*)out, R, c.H, c.topk, c.obf16);
    return launch_status();
}

// Calls the grouped GEMM does not take (tables with per-expert trellis or intermediate widths, the forced several-kernel
// path) with more rows than one pass takes (64 rows, 1024 pairs) run pass after pass over row ranges: a row's result does not
// depend on the other rows of a call, so the values are those of one big call.  The passes share the workspace.
inline int rows_per_pass(const Cfg& c) { const int byp = PMAX / c.topk; return byp < 64 ? byp : 64; }
int experts_rows(const Cfg& c, const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out, void* ws,
                 int flags, hipStream_t st)
{
    if (R < 1 || c.topk < 1 || c.topk > 64) return -1;
    if (const int v = routes_check(idx, c.itype != 0, R, c.topk, c.E, st)) return v > 0 ? -6 : -8;    // opt-in host check of the routes
    const int RC = rows_per_pass(c);
    if (!(flags & 2) && big_ok(c, R)) return experts_big(c, x, ldx, R, idx, w, tab, add, out, ws, flags, st);     // more than 8 rows: grouped GEMM
    if (R <= RC) return experts(c, x, ldx, R, idx, w, tab, add, out, ws, flags, st);
    const size_t xsz = c.xtype == X_F32 ? 4 : 2, isz = c.itype ? 8 : 4, wsz = c.wtype ? 2 : 4;
    for (int r0 = 0; r0 < R; r0 += RC) {
        const int n = R - r0 < RC ? R - r0 : RC;
        const int rc = experts(c, (const char*)x + (size_t)r0 * ldx * xsz, ldx, n, (const char*)idx + (size_t)r0 * c.topk * isz,
                               (const char*)w + (size_t)r0 * c.topk * wsz, tab, add ? (const float*)add + (size_t)r0 * c.H : nullptr,
                               (char*)out + (size_t)r0 * c.H * (c.obf16 ? 2 : 4), ws, flags, st);
        if (rc) return rc;
    }
    return 0;
}

const Cfg QWEN{512, 10, 2560, 640, CB_MUL1, 0, X_F32, 0, 0};
const Cfg GLM{288, 8, 4096, 1024, CB_MCG, 1, X_F16, 1, 1};
const Cfg GLM3{288, 8, 4096, 768, CB_MCG, 1, X_F16, 1, 1};        // TP3: experts 640 or 768 wide, I = the widest (strides)

}  // namespace

// ================================================================ C ABI

// Runtime-sized entry (no reference counterpart symbol): x [R, H] of xtype (0 f32, 1 f16, 2 bf16), row stride ldx;
// idx [R, topk] int32 (itype 0) or int64 (1); w [R, topk] f32 (wtype 0) or f16 (1); tab u64 [9][E]; codebook 2 = mul1,
// 1 = mcg; act 0 = silu(g) u, 1 = clamped; add / out f32 [R, H].  Any R: up to 8 rows in one launch, more as a grouped GEMM (or, for tables the GEMM does not take, as passes of 64 rows).
// flags bit 0: the workspace was zeroed by spark_exl3_moe_ws_init and only used by this entry since (saves a launch);
// bit 1: use the several-kernel path even where the single-launch path or the grouped GEMM applies.
// Which path a call of this shape and these flags takes (a host-side query: nothing is launched): 0 = the single launch, 1 = the
// grouped GEMM, 2 = the item kernels (pass after pass beyond 64 rows), -1 = a shape no entry point takes.
SPARK_API int spark_exl3_moe_path(int R, int H, int I, int E, int topk, int flags)
{
    const Cfg c{E, topk, H, I, CB_MUL1, 0, 0, 0, 0};
    if (R < 1 || topk < 1 || topk > 64) return -1;
    if (!(flags & 2) && big_ok(c, R)) return 1;
    const int RC = rows_per_pass(c);
    if (!cfg_ok(c, R < RC ? R : RC)) return -1;
    return !(flags & 2) && R <= RC && exl3_fused_ok(c, R) ? 0 : 2;
}
SPARK_API size_t spark_exl3_moe_ws_bytes(int R, int H, int I, int E, int topk)
{
    const Cfg c{E, topk, H, I, CB_MUL1, 0, 0, 0, 0};
    if (R < 1 || topk < 1 || topk > 64) return 0;
    const int RC = rows_per_pass(c);
    const int n = R < RC ? R : RC;                   // rows of the largest pass
    if (!cfg_ok(c, n)) return 0;
    size_t need = plan(c, n, GR_ITEM).total;
    { const size_t v = plan(c, n, gr_of_rows(n, false)).total; if (v > need) need = v; }     // uniform tables group by the instance's row count
    if (big_ok(c, R)) { const size_t v = plan(c, R, PG_ROWS).total; if (v > need) need = v; }
    return fused_cap(c) + need;                      // grows with R: a caller may size once for its largest call
}
// Prepares a workspace once after allocation (every exchanged word idle) and runs the one-time placement check, which synchronises
// the device: call it outside stream capture.  From then on calls that use this workspace - spark_exl3_moe with or without flags
// bit 0, qwen_moe_experts, glm_moe*_experts - run the decode sizes as one launch; spark_moe_ws_release(ws) before the memory is
// freed or reused.  With ws null only the one-time set-up runs (placement check, address of the library's own scratch array).
SPARK_API int spark_exl3_moe_ws_init(void* ws, size_t bytes, hipStream_t st)
{
    xcd_placement_check();
    const int rs = exl3_static_setup();
    if (rs) return rs;
    if (!ws || bytes == 0) return 0;
    const int rc = exl3_fused_ws_prepare(ws, bytes, st);
    if (rc == 0) ws_note_prepared(ws, bytes);
    return rc;
}
SPARK_API int spark_exl3_moe(const void* x, int xtype, int64_t ldx, int R, const void* idx, int itype, const void* w, int wtype, const void* tab,
                             const void* add, void* out, void* ws, int H, int I, int E, int topk, int codebook, int act, int flags, hipStream_t st)
{
    const Cfg c{E, topk, H, I, codebook, act, xtype, wtype, itype, (flags & 16) ? 1 : 0};
    return experts_rows(c, x, ldx, R, idx, w, tab, add, out, ws, flags, st);
}
// reference qwen_moe.cu:112-116: x f32 [R, 2560], idx i32 / w f32 [R, 10], tab u64 [9][512], out f32 [R, 2560]; S is the
// reference's K-slice hint (the slice count is chosen from the shape here)
SPARK_API size_t qwen_moe_ws_bytes(int R, int S) { (void)S; return spark_exl3_moe_ws_bytes(R, QWEN.H, QWEN.I, QWEN.E, QWEN.topk); }
SPARK_API int qwen_moe_experts(const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out, void* ws, int S,
                               hipStream_t st)
{
    (void)S;
    return experts_rows(QWEN, x, ldx, R, idx, w, tab, add, out, ws, 0, st);
}
// reference glm_moe.cu:6-24: x f16 [R, 4096], idx i64 / w f16 [R, 8], tab u64 [10|11][288] (rows 0-8 as above), mcg codebook,
// clamped SwiGLU.  suh0 (shared gate/up input scales) is a prefill shortcut and is not needed.  kmask = bit K set for every
// trellis width K present: 1 << 4 runs the 4-bit kernels, anything else reads every expert's width from row 9 of the table.
SPARK_API size_t glm_moe_ws_bytes(int R, int S) { (void)S; return spark_exl3_moe_ws_bytes(R, GLM.H, GLM.I, GLM.E, GLM.topk); }
SPARK_API int glm_moe_experts(const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out, void* ws, int S,
                              const void* suh0, int kmask, hipStream_t st)
{
    (void)S; (void)suh0;
    if (kmask <= 0 || (kmask & ~0x78)) return -4;              // widths 3..6 only
    return experts_rows(GLM, x, ldx, R, idx, w, tab, add, out, ws, kmask == (1 << 4) ? 0 : 4, st);
}
// reference glm_moe.cu:17-24 (moex::GlmMoe3, moe_exl3.cuh:63-67): GLM under a three-way split, every expert 768 or 640 wide (6 or
// 5 of its 128-wide Hadamard blocks); tab u64 [11][288]: rows 0-8 as above, row 9 the trellis width in bits, row 10 the
// expert's intermediate width.  Intermediates keep the stride of the widest expert (768).
SPARK_API size_t glm_moe3_ws_bytes(int R, int S) { (void)S; return spark_exl3_moe_ws_bytes(R, GLM3.H, GLM3.I, GLM3.E, GLM3.topk); }
SPARK_API int glm_moe3_experts(const void* x, int64_t ldx, int R, const void* idx, const void* w, const void* tab, const void* add, void* out, void* ws, int S,
                               int kmask, hipStream_t st)
{
    (void)S;
    if (kmask <= 0 || (kmask & ~0x78)) return -4;
    return experts_rows(GLM3, x, ldx, R, idx, w, tab, add, out, ws, 8 | (kmask == (1 << 4) ? 0 : 4), st);
}
