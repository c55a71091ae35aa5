// Shared pieces of the MXFP4 expert kernels: weight layouts, the A / B operand loads, the exact gate / up step on the bf16 MFMA and
// the block-scaled MFMA step of the down product.
//
// Operand layout of v_mfma_scale_f32_16x16x128_f8f6f4 measured on gfx950: A/B lane l = row/column l % 16, K group g = l / 16.
// An E2M1 operand holds k = 32 g + e (nibble e of its 16 bytes); an E4M3 operand holds k = 16 g + e in registers 0-3 and
// k = 64 + 16 g + e in registers 4-7; the scale byte of lane l applies to logical block g (k in [32 g, 32 g + 32)); D lane l =
// column l % 16, rows 4 (l / 16) + {0..3}.
#pragma once
#include "common.hpp"

namespace spk {
namespace mx {

constexpr int REC = 4352;              // bytes per T16 record

// L_MX8S2: the codes of L_MX8 with the scales in the reference's lossless 2-bit coding (engine-rs/shim/ds41_mx.cu:64-91,
// engine-rs/src/ds41/kern.rs:747-770): one blob per matrix of T = experts * rows / 8 tiles and S = K / 128 steps =
// desc [T][16] (bytes 0-7 the rows' base scales, bytes 8-11 an int32 index into raw or -1), codes [T][S][8 rows] (four 2-bit
// offsets per byte, block b in bits 2b..2b+1), raw [n_raw][S][8][4] (tiles with a row whose scales span more than 3).
enum Layout { L_T16 = 0, L_NATURAL = 1, L_PACK8 = 2, L_MX8 = 3, L_MX8S2 = 4 };

struct WMat {                          // one stacked weight matrix [E, rows, K]
    const uint8_t* w;
    const uint8_t* s;
    int rows, K;                       // per expert
    int64_t tiles8;                    // experts * rows / 8 (locates the sections of a 2-bit coded scale blob)
};

// ---- A operand: the 4 steps of K group kg of the 16 rows starting at row0 (row0 % 16 == 0) of expert e
template <int LAYOUT>
__device__ __forceinline__ void load_group(const WMat& m, int e, int row0, int kg, int lane, v4i (&c)[4], uint32_t& sc4)
{
    const int r = lane & 15, g = lane >> 4, steps = m.K >> 7, nkg = (steps + 3) >> 2;
    if constexpr (LAYOUT == L_T16) {
        const int64_t tile = ((int64_t)e * m.rows + row0) >> 4;
        const uint8_t* rec = m.w + (tile * nkg + kg) * REC;
#pragma unroll
        for (int s = 0; s < 4; ++s) { const uint4 v = ld_stream16(rec + s * 1024 + lane * 16); c[s] = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w}; }
        sc4 = __builtin_nontemporal_load((const uint32_t*)(rec + 4096 + lane * 4));
    } else {
        sc4 = 0x7f7f7f7fu;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int step = kg * 4 + s;
            c[s] = v4i{0, 0, 0, 0};
            if (step >= steps) continue;
            const int64_t row = (int64_t)e * m.rows + row0 + r;
            uint32_t sb;
            if constexpr (LAYOUT == L_NATURAL) {
                const uint4 v = ld_stream16(m.w + row * (m.K >> 1) + step * 64 + g * 16);
                c[s] = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
                sb = m.s[row * (m.K >> 5) + step * 4 + g];
            } else if constexpr (LAYOUT == L_PACK8) {      // [rows/8][K/128][8][4][16], scales [rows/8][K/128][8][4]
                const int64_t t8 = row >> 3;
                const uint4 v = ld_stream16(m.w + (t8 * steps + step) * 512 + (row & 7) * 64 + g * 16);
                c[s] = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
                sb = m.s[(t8 * steps + step) * 32 + (row & 7) * 4 + g];
            } else {                                        // L_MX8 / L_MX8S2: [rows/8][K/128][8][4 q][4 b][4]
                const int64_t t8 = row >> 3;
                const int r8 = (int)(row & 7);
                // the row's 64 bytes of a step are 4 x 4 dwords [q][b] and the lane of K block g needs column b = g: the four lanes
                // of a row (16 apart) load one q-row each with a 16-byte load and transpose with two rounds of row swaps
                const uint4 v = ld_stream16(m.w + (t8 * steps + step) * 512 + r8 * 64 + g * 16);
                const auto a02 = __builtin_amdgcn_permlane32_swap(v.x, v.z, false, false);
                const auto a13 = __builtin_amdgcn_permlane32_swap(v.y, v.w, false, false);
                const auto b01 = __builtin_amdgcn_permlane16_swap(a02[0], a13[0], false, false);
                const auto b23 = __builtin_amdgcn_permlane16_swap(a02[1], a13[1], false, false);
                c[s] = v4i{(int)b01[0], (int)b01[1], (int)b23[0], (int)b23[1]};
                if constexpr (LAYOUT == L_MX8) sb = m.s[(t8 * steps + step) * 32 + r8 * 4 + g];
                else {
                    const uint32_t* d = (const uint32_t*)(m.s + t8 * 16);
                    const uint8_t* code = m.s + m.tiles8 * 16;
                    const uint8_t* raw = code + m.tiles8 * steps * 8;
                    const int ri = (int)d[2];
                    if (ri >= 0) sb = raw[((int64_t)ri * steps + step) * 32 + r8 * 4 + g];
                    else sb = ((d[r8 >> 2] >> (8 * (r8 & 3))) & 0xffu) + ((code[(t8 * steps + step) * 8 + r8] >> (2 * g)) & 3u);
                }
            }
            sc4 = (sc4 & ~(0xffu << (8 * s))) | (sb << (8 * s));
        }
    }
}

// ---- The same operand in two steps, for code that keeps several K groups in flight: grp_load only requests (nothing it loads is
// touched, so a second request does not wait for the first to arrive - load_group above builds the scale word from byte loads and
// transposes the MX8 codes on the spot, which makes every call a round trip to memory), grp_fix turns what arrived into the operand
// right before the matrix instructions.  Steps past the matrix (a ragged last K group) fetch the last step again: unused.
struct GrpScale { uint32_t v0, v1, base4; bool has_raw; };      // v0: the scale dword as loaded (MX8S2: the code byte); v1, base4, has_raw: MX8S2 only
template <int LAYOUT>
__device__ __forceinline__ void grp_load(const WMat& m, int e, int row0, int kg, int lane, v4i (&c)[4], GrpScale& sr)
{
    const int r = lane & 15, g = lane >> 4, steps = m.K >> 7, nkg = (steps + 3) >> 2;
    sr.v1 = 0u; sr.base4 = 0u; sr.has_raw = false;
    if constexpr (LAYOUT == L_T16) {
        const int64_t tile = ((int64_t)e * m.rows + row0) >> 4;
        const uint8_t* rec = m.w + (tile * nkg + kg) * REC;
#pragma unroll
        for (int s = 0; s < 4; ++s) { const uint4 v = ld_stream16(rec + s * 1024 + lane * 16); c[s] = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w}; }
        sr.v0 = __builtin_nontemporal_load((const uint32_t*)(rec + 4096 + lane * 4));
    } else {
        // Addresses = a wave-uniform part (expert, tile row, K group: 64-bit, on the scalar unit) + this lane's 32-bit offset.  The
        // 16 rows start on a multiple of 16, so lane row r sits in 8-row tile r / 8 of the two, at row r % 8 of it.
        const int eu = __builtin_amdgcn_readfirstlane(e), row0u = __builtin_amdgcn_readfirstlane(row0), kgu = __builtin_amdgcn_readfirstlane(kg);
        const int64_t row_u = (int64_t)eu * m.rows + row0u;
        const int r8 = r & 7, th = r >> 3;
        const int sstep = min(kgu * 4 + g, steps - 1);      // this lane fetches the four block scales of step g of the K group
        if constexpr (LAYOUT == L_NATURAL) {
            const uint8_t* wu = m.w + row_u * (m.K >> 1);
            const uint32_t lo = (uint32_t)r * (uint32_t)(m.K >> 1) + g * 16;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int step = min(kgu * 4 + s, steps - 1);
                const uint4 v = ld_stream16(wu + step * 64 + lo);
                c[s] = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
            }
            sr.v0 = *(const uint32_t*)(m.s + row_u * (m.K >> 5) + ((uint32_t)r * (uint32_t)(m.K >> 5) + sstep * 4));
        } else {
            const int64_t t8u = row_u >> 3;                 // the first of the two 8-row tiles
            const uint8_t* wu = m.w + t8u * steps * 512;    // PACK8: [rows/8][K/128][8][4][16]; MX8: [rows/8][K/128][8][4 q][4 b][4]
            const uint32_t lo = (uint32_t)(th * steps) * 512u + r8 * 64 + g * 16;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const int step = min(kgu * 4 + s, steps - 1);
                const uint4 v = ld_stream16(wu + step * 512 + lo);
                c[s] = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
            }
            if constexpr (LAYOUT == L_MX8S2) {
                // the tile's descriptor first (a dependent address: the only wait in here)
                const uint32_t* d = (const uint32_t*)(m.s + (t8u + th) * 16);
                const uint8_t* code = m.s + m.tiles8 * 16;
                const int ri = (int)d[2];
                sr.base4 = ((d[r8 >> 2] >> (8 * (r8 & 3))) & 0xffu) * 0x01010101u;
                sr.has_raw = ri >= 0;
                const uint8_t* raw = code + m.tiles8 * steps * 8 + (int64_t)(ri >= 0 ? ri : 0) * steps * 32;
                const uint8_t* cp = code + t8u * steps * 8 + (uint32_t)((th * steps + sstep) * 8 + r8);
                sr.v0 = *cp;
                // both forms are requested whatever the tile has: a tile without raw words reads its code byte's word a second time
                sr.v1 = *(const uint32_t*)(sr.has_raw ? raw + (uint32_t)(sstep * 32 + r8 * 4) : (const uint8_t*)((uintptr_t)cp & ~(uintptr_t)3));
            } else sr.v0 = *(const uint32_t*)(m.s + t8u * steps * 32 + (uint32_t)((th * steps + sstep) * 32 + r8 * 4));
        }
    }
}
// -> c[s] = the A operand of step s, sc4 byte s = the scale of this lane's K block in step s
template <int LAYOUT>
__device__ __forceinline__ void grp_fix(v4i (&c)[4], const GrpScale& sr, int lane, uint32_t& sc4)
{
    if constexpr (LAYOUT == L_T16) { sc4 = sr.v0; return; }
    else {
        if constexpr (LAYOUT == L_MX8 || LAYOUT == L_MX8S2) {
            // the row's 64 bytes of a step are 4 x 4 dwords [q][b] and the lane of K block g needs column b = g: the four lanes of a
            // row (16 apart) hold one q-row each and transpose with two rounds of row swaps
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const auto a02 = __builtin_amdgcn_permlane32_swap((uint32_t)c[s].x, (uint32_t)c[s].z, false, false);
                const auto a13 = __builtin_amdgcn_permlane32_swap((uint32_t)c[s].y, (uint32_t)c[s].w, false, false);
                const auto b01 = __builtin_amdgcn_permlane16_swap(a02[0], a13[0], false, false);
                const auto b23 = __builtin_amdgcn_permlane16_swap(a02[1], a13[1], false, false);
                c[s] = v4i{(int)b01[0], (int)b01[1], (int)b23[0], (int)b23[1]};
            }
        }
        uint32_t d = sr.v0;
        if constexpr (LAYOUT == L_MX8S2) {
            const uint32_t cb = sr.v0;
            const uint32_t coded = sr.base4 + ((cb & 3u) | ((cb & 0xcu) << 6) | ((cb & 0x30u) << 12) | ((cb & 0xc0u) << 18));
            d = sr.has_raw ? sr.v1 : coded;
        }
        // lane (row, g) holds M[g][b] = scale(step g, block b) and wants M[s][g] in byte s: a 4 x 4 byte transpose over the four lanes of
        // the row, 2 x 2 blocks first (partner g ^ 2), then inside the blocks (partner g ^ 1)
        const int g = lane >> 4;
        const uint32_t pp = __float_as_uint(lane_xor<32>(__uint_as_float(d), lane));
        // __builtin_amdgcn_perm(hi, lo, sel): result byte i = byte sel[i] of the 8 bytes {hi, lo} (0-3 lo, 4-7 hi)
        const uint32_t n = (g & 2) ? __builtin_amdgcn_perm(d, pp, 0x07060302u) : __builtin_amdgcn_perm(pp, d, 0x05040100u);
        const uint32_t q = __float_as_uint(lane_xor<16>(__uint_as_float(n), lane));
        sc4 = (g & 1) ? __builtin_amdgcn_perm(n, q, 0x07030501u) : __builtin_amdgcn_perm(q, n, 0x06020400u);
    }
}

// ---- B operand of one step: E4M3 bytes of row `q` (row stride K) + its UE8M0 scales (row stride K/32)
__device__ __forceinline__ void load_b(const uint8_t* __restrict__ q, const uint8_t* __restrict__ qs, int step, int lane, v8i& b, uint32_t& sb)
{
    const int g = lane >> 4;
    const uint4 lo = *(const uint4*)(q + step * 128 + 16 * g);
    const uint4 hi = *(const uint4*)(q + step * 128 + 64 + 16 * g);
    b = v8i{(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
    sb = qs[step * 4 + g];
}

// ---- gate / up products, exact.  The block-scaled instruction below aligns the products of a 32-block to the block's largest and
// drops what lies more than about 14 bits under it; the activation quantiser behind the gate / up sums turns some of those 1e-5
// differences into a flipped E4M3 step of the intermediate.  The reference forms these products exactly (engine-rs/shim/
// ds41_moe.cu:8-10: E2M1 through a table into bf16, bf16 MMA, binary32 sums), so gate / up run on v_mfma_f32_16x16x32_bf16:
// E2M1 x 2^sw and E4M3 x 2^sx convert to bf16 exactly (scales inside the hardware convert), every product is exact in
// binary32 and the sums are binary32.  A 128-wide step is four instructions; instruction j takes, in lane group g, the k
// 32 g + 8 j .. + 7 of the step from both operands (the contraction index may be dealt to the instructions in any order as long as
// both operands agree), i.e. dword j of the lane's 16 code bytes as they are streamed: no data crosses lanes.
typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf8v __attribute__((ext_vector_type(8)));
struct XOp { bf8v b[4]; };             // the B operands of a step's four instructions
// E4M3 bytes lo / hi = k 32 g .. + 15 / + 16 .. + 31 of the step for this lane's token row, sb = the block's UE8M0 byte
__device__ __forceinline__ XOp x_operand(const uint4& lo, const uint4& hi, uint32_t sb)
{
    const float sc = e8m0_to_f32(sb & 0xffu);
    const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    XOp r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        bf2 v[4];
        v[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j], sc, false); v[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j], sc, true);
        v[2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j + 1], sc, false); v[3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w[2 * j + 1], sc, true);
        __builtin_memcpy(&r.b[j], v, 16);
    }
    return r;
}
// row q (E4M3, row stride K) + its UE8M0 scales qs (row stride K / 32): the lane's 32 bytes of the step are neighbours
__device__ __forceinline__ XOp load_x(const uint8_t* __restrict__ q, const uint8_t* __restrict__ qs, int step, int lane)
{
    const int g = lane >> 4;
    const uint4 lo = *(const uint4*)(q + step * 128 + 32 * g), hi = *(const uint4*)(q + step * 128 + 32 * g + 16);
    return x_operand(lo, hi, qs[step * 4 + g]);
}
// eight E2M1 codes (one dword of the stream, low nibble first) x the block's scale -> the A operand of one instruction
__device__ __forceinline__ bf8v a_operand(uint32_t w, float sc)
{
    bf2 v[4];
    v[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 0); v[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 1);
    v[2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 2); v[3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 3);
    bf8v av;
    __builtin_memcpy(&av, v, 16);
    return av;
}
// a: the lane's 16 code bytes of step s (block g of 16 weight rows), sa4 byte s: that block's E8M0 scale
__device__ __forceinline__ v4f mfma_exact_step(int s, const v4i& a, const XOp& x, v4f acc, uint32_t sa4)
{
    const float sc = e8m0_to_f32((sa4 >> (8 * s)) & 0xffu);
    const uint32_t w[4] = {(uint32_t)a.x, (uint32_t)a.y, (uint32_t)a.z, (uint32_t)a.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_operand(w[j], sc), x.b[j], acc, 0, 0, 0);
    return acc;
}

template <int OPSEL>
__device__ __forceinline__ v4f mfma_step(const v4i& a, const v8i& b, v4f acc, uint32_t sa, uint32_t sb)
{
    const v8i a8 = v8i{a.x, a.y, a.z, a.w, 0, 0, 0, 0};
    return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a8, b, acc, 4 /*A: E2M1*/, 0 /*B: E4M3*/, OPSEL, (int)sa, 0, (int)sb);
}
__device__ __forceinline__ v4f mfma_group_step(int s, const v4i& a, const v8i& b, v4f acc, uint32_t sa4, uint32_t sb)
{
    switch (s) {
        case 0: return mfma_step<0>(a, b, acc, sa4, sb);
        case 1: return mfma_step<1>(a, b, acc, sa4, sb);
        case 2: return mfma_step<2>(a, b, acc, sa4, sb);
        default: return mfma_step<3>(a, b, acc, sa4, sb);
    }
}

// ---- the single-launch decode path (moe_mxfp4_fused.hip): R <= 8 token rows, topk + shared <= 16
bool mx_fused_ok(int R, int H, int I, int topk, int E, int n_shared);
size_t mx_fused_ws_bytes(int R, int H, int I, int topk, int E, int n_shared);
int mx_fused_ws_prepare(void* ws, size_t bytes, hipStream_t st);
// x: bf16 [R, H] when xs is null (quantised inside), else E4M3 [R, H] with its scales xs.  clean: the exchanged words of ws are
// idle (prepared once and only used by this path since); otherwise one more launch prepares them first.
int mx_fused_launch(const void* x, const void* xs, int R, const int64_t* idx, const float* rw, const void* w1, const void* s1, const void* w3, const void* s3,
                    const void* w2, const void* s2, int layout, int H, int I, int topk, int E, int n_shared, const float* add, float* y, void* ws, int clean,
                    hipStream_t st, int obf16 = 0);

}  // namespace mx
}  // namespace spk
