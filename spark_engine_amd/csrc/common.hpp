// Shared device helpers for the gfx950 (CDNA4, wave64) kernels of the quantized MoE expert path.
// Everything here is written for one target: no other architecture is supported.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define SPARK_API extern "C" __attribute__((visibility("default")))

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));

namespace spk {

constexpr int WAVE = 64;

// A load whose address is the same for the whole wave, through the scalar cache: it does not queue behind the vector
// loads (weight bursts) of the CU's other blocks, which cost a dependent lookup 1 - 2 us.  Only for memory the kernel
// never writes (routing indices, route weights, the expert table).
template <class T> __device__ __forceinline__ T ld_k(const T* p, int i)
{
    return *(const __attribute__((address_space(4))) T*)(uintptr_t)(p + __builtin_amdgcn_readfirstlane(i));
}

// ---- number formats (bit-exact, software: the bytes must match the CPU reference of the same rule) ----
__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7f800000u) == 0x7f800000u && (u & 0x7fffffu)) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float bf16_round(float f) { return bf16_to_f32(f32_to_bf16(f)); }
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { _Float16 v; __builtin_memcpy(&v, &h, 2); return (float)v; }
// binary32 -> fp16 bits, round to nearest even.  The argument is made opaque first: otherwise the compiler folds a multiply that
// produced it into the conversion (one rounding of the exact product instead of the reference's two roundings: a different fp16
// value when the binary32 product is a tie).
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f)
{
    asm volatile("" : "+v"(f));
    _Float16 v = (_Float16)f; uint16_t h; __builtin_memcpy(&h, &v, 2); return h;
}
// E8M0 scale byte -> 2^(b-127) from the exponent bits (byte 0 gives 0.0)
__device__ __forceinline__ float e8m0_to_f32(uint32_t b) { return __uint_as_float(b << 23); }
// OCP E4M3 (fn) -> binary32.  Exponent and mantissa are dropped into binary32 and rescaled by 2^120, which also maps the
// subnormal codes exactly; done with integer arithmetic so that it does not depend on the denormal mode.
__device__ __forceinline__ float e4m3_to_f32(uint32_t b)
{
    const uint32_t s = (b & 0x80u) << 24, em = b & 0x7fu;
    if ((em >> 3) == 0) return __uint_as_float(s | __float_as_uint((float)(em & 7u) * 0.001953125f));
    return __uint_as_float(s | ((em << 20) + (120u << 23)));
}
// binary32 (already clamped to [-448, 448]) -> E4M3 code, round to nearest even
__device__ __forceinline__ uint32_t f32_to_e4m3(float f)
{
    const uint32_t u = __float_as_uint(f), s = (u >> 24) & 0x80u, a = u & 0x7fffffffu;
    const float af = __uint_as_float(a);
    if (af >= 448.0f) return s | 0x7eu;
    const int e = (int)(a >> 23) - 127;
    if (e < -6) return s | (uint32_t)__builtin_rintf(af * 512.0f);   // units of 2^-9, ties to even; 8 = smallest normal
    const uint32_t m = a & 0x7fffffu;
    uint32_t q = m >> 20;
    const uint32_t rem = m & 0xfffffu;
    q += (rem > 0x80000u || (rem == 0x80000u && (q & 1u))) ? 1u : 0u;
    uint32_t r = ((uint32_t)(e + 7) << 3) + q;
    return s | (r > 0x7eu ? 0x7eu : r);
}
// act_quant: UE8M0 scale byte of a 32-block from its absolute maximum, and the E4M3 byte of one value under it
__device__ __forceinline__ uint32_t aq_scale(float amax)
{
    amax = fmaxf(amax, 1e-4f);
    const uint32_t bits = __float_as_uint(amax * (1.0f / 448.0f));
    return ((bits >> 23) & 0xffu) + ((bits & 0x7fffffu) != 0u ? 1u : 0u);
}
// 1 / 2^(e - 127) as binary32: multiplying by it is the division by the scale, bit for bit (a power of two; 2^-127 is a
// denormal, the reciprocal of the scale byte 255 - infinity - is 0)
__device__ __forceinline__ float aq_inv(uint32_t e) { return __uint_as_float(e < 254u ? (254u - e) << 23 : (e == 254u ? 0x00400000u : 0u)); }
__device__ __forceinline__ float aq_clamp(float v, float inv) { return fminf(fmaxf(v * inv, -448.f), 448.f); }
// The encode is the hardware's (v_cvt_pk_fp8_f32: OCP E4M3, round to nearest even, denormal codes included; it turns what lies
// beyond the format into NaN, which the clamp in front excludes): the same bytes as f32_to_e4m3 above, which every binary16
// input of act_quant checks.
__device__ __forceinline__ uint32_t aq_byte(float v, uint32_t e)
{
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(aq_clamp(v, aq_inv(e)), 0.f, 0, false) & 0xffu;
}
// four values under one scale -> four code bytes, v0 in the low byte
__device__ __forceinline__ uint32_t aq_word4(float v0, float v1, float v2, float v3, uint32_t e)
{
    const float inv = aq_inv(e);
    const int lo = __builtin_amdgcn_cvt_pk_fp8_f32(aq_clamp(v0, inv), aq_clamp(v1, inv), 0, false);
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(aq_clamp(v2, inv), aq_clamp(v3, inv), lo, true);
}
__device__ __forceinline__ float silu(float g) { return g / (1.0f + expf(-g)); }

// ---- wave64 cross-lane primitives ----
// value of lane (lane ^ mask) for mask < 64
__device__ __forceinline__ float xor_f(float v, int mask) { return __shfl_xor(v, mask, 64); }
__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int o = 32; o; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// The value lane ^ M holds, without LDS traffic: DPP quad permutes and row mirrors inside a row of 16 lanes (xor 4 = reverse
// the quad then mirror the half row, xor 8 = mirror the half row then the row), the gfx950 row / half-wave swaps beyond.
template <int CTRL> __device__ __forceinline__ float dpp_mov_f32(float v)
{
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, false));
}
template <int M> __device__ __forceinline__ float lane_xor(float v, int lane)
{
    static_assert(M == 1 || M == 2 || M == 4 || M == 8 || M == 16 || M == 32, "one bit");
    if constexpr (M == 1) return dpp_mov_f32<0xB1>(v);                        // quad_perm [1,0,3,2]
    else if constexpr (M == 2) return dpp_mov_f32<0x4E>(v);                   // quad_perm [2,3,0,1]
    else if constexpr (M == 4) return dpp_mov_f32<0x141>(dpp_mov_f32<0x1B>(v));   // quad_perm [3,2,1,0], row_half_mirror
    else if constexpr (M == 8) return dpp_mov_f32<0x128>(v);                  // row_ror:8 (lane i of a row of 16 reads lane i + 8 mod 16 = i ^ 8)
    else if constexpr (M == 16) {
        // vdst' = rows (0, 0, 2, 2) of v, src' = rows (1, 1, 3, 3)
        const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        return __uint_as_float((lane & 16) ? r[0] : r[1]);
    } else {
        // vdst' = the lower half twice, src' = the upper half twice
        const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
        return __uint_as_float((lane & 32) ? r[0] : r[1]);
    }
}
// butterfly sum over the wave, partners 32, 16, ..., 1 apart in that order (every lane ends with the total)
__device__ __forceinline__ float wave_sum(float v)
{
    const int lane = threadIdx.x & 63;
    v += lane_xor<32>(v, lane); v += lane_xor<16>(v, lane); v += lane_xor<8>(v, lane);
    v += lane_xor<4>(v, lane); v += lane_xor<2>(v, lane); v += lane_xor<1>(v, lane);
    return v;
}
template <int M> __device__ __forceinline__ void fwht_stage(float& v0, float& v1, int lane)
{
    // (a + b, a - b) with the lower lane holding a: upper lanes negate their own value first, then both add
    const uint32_t sign = (lane & M) ? 0x80000000u : 0u;
    const float o0 = lane_xor<M>(v0, lane), o1 = lane_xor<M>(v1, lane);
    v0 = o0 + __uint_as_float(__float_as_uint(v0) ^ sign);
    v1 = o1 + __uint_as_float(__float_as_uint(v1) ^ sign);
}
// 128-point normalized Walsh-Hadamard over values held 2 per lane (lane l: elements 2l, 2l+1), binary32, butterflies
// h = 1, 2, ..., 64 with (a + b, a - b), lower index first, then one multiply: the operation order of a serial FWHT.
__device__ __forceinline__ void fwht128(float& v0, float& v1, int lane)
{
    { const float a = v0 + v1, b = v0 - v1; v0 = a; v1 = b; }
    fwht_stage<1>(v0, v1, lane); fwht_stage<2>(v0, v1, lane); fwht_stage<4>(v0, v1, lane);
    fwht_stage<8>(v0, v1, lane); fwht_stage<16>(v0, v1, lane); fwht_stage<32>(v0, v1, lane);
    v0 *= 0.08838834764831845f;
    v1 *= 0.08838834764831845f;
}

// The same transform over values held 8 per lane by 16 neighbouring lanes (lane l of the sixteen: elements 8 l .. 8 l + 7), four
// transforms a wave: the same butterflies in the same order (h = 1, 2, 4 inside the lane, 8 .. 64 across lanes), so the same bits.
template <int CTRL> __device__ __forceinline__ float dpp_mov_f32_all(float v)       // every lane has a source lane: no fill value to set up
{
    return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, true));
}
template <int M> __device__ __forceinline__ void fwht_stage8(float (&v)[8], int lane)
{
    static_assert(M == 1 || M == 2 || M == 4 || M == 8, "inside a row of 16 lanes");
    const uint32_t sign = (lane & M) ? 0x80000000u : 0u;
    float sv[8];                                           // all eight sign flips first: the exchanges then read registers written long before
#pragma unroll
    for (int i = 0; i < 8; ++i) sv[i] = __uint_as_float(__float_as_uint(v[i]) ^ sign);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float o;
        if constexpr (M == 1) o = dpp_mov_f32_all<0xB1>(v[i]);
        else if constexpr (M == 2) o = dpp_mov_f32_all<0x4E>(v[i]);
        else if constexpr (M == 4) o = dpp_mov_f32_all<0x141>(dpp_mov_f32_all<0x1B>(v[i]));
        else o = dpp_mov_f32_all<0x128>(v[i]);
        v[i] = o + sv[i];
    }
}
__device__ __forceinline__ void fwht128_x8(float (&v)[8], int lane)
{
#pragma unroll
    for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) if (!(i & h)) { const float a = v[i] + v[i + h], b = v[i] - v[i + h]; v[i] = a; v[i + h] = b; }
    }
    fwht_stage8<1>(v, lane); fwht_stage8<2>(v, lane); fwht_stage8<4>(v, lane); fwht_stage8<8>(v, lane);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] *= 0.08838834764831845f;
}
// eight binary16 values from an address that is a multiple of 4 (one 16-byte access where it is a multiple of 16)
__device__ __forceinline__ uint4 ld_8h(const uint16_t* p)
{
    if (((uintptr_t)p & 15) == 0) return *(const uint4*)p;
    const uint32_t* q = (const uint32_t*)p;
    return make_uint4(q[0], q[1], q[2], q[3]);
}

// ---- the items of a routed call, worked out by ONE wave.  Items are the call's distinct experts in order of first appearance;
// an item's pairs are the (row, slot) pairs routed to its expert, ascending.  Lane l holds pairs l, l + 64, ... (NJ per lane).
// owner: LDS scratch with one int per expert id.  No barrier inside: LDS operations of one wave execute in order.
template <int NJ> struct WaveItems { int e[NJ]; bool first[NJ]; int rank[NJ]; };
__device__ __forceinline__ int lanes_below(uint64_t m) { return (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u)); }
template <int NJ, class F> __device__ __forceinline__ void wave_items_init(WaveItems<NJ>& w, int P, int lane, int* owner, F expert_of)
{
#pragma unroll
    for (int j = 0; j < NJ; ++j) { const int p = lane + 64 * j; w.e[j] = p < P ? expert_of(p) : -1; }
#pragma unroll
    for (int j = 0; j < NJ; ++j) if (w.e[j] >= 0) owner[w.e[j]] = 0x7fffffff;
#pragma unroll
    for (int j = 0; j < NJ; ++j) if (w.e[j] >= 0) atomicMin(&owner[w.e[j]], lane + 64 * j);
    int base = 0;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        w.first[j] = w.e[j] >= 0 && owner[w.e[j]] == lane + 64 * j;      // the first pair of its expert
        const uint64_t m = __builtin_amdgcn_ballot_w64(w.first[j]);
        w.rank[j] = base + lanes_below(m);
        base += __builtin_popcountll(m);
    }
}
// item g: its expert (or -1 when the call has fewer items), its pairs in rows[0 .. n).  cap: the entries rows[] has; an item with more
// pairs than that (only possible when a token row names an expert twice, which the routes' contract excludes) keeps its first cap
// pairs, n stops at cap and `over` is set: the caller raises the workspace's error flag instead of writing past its arrays.
template <int NJ> __device__ __forceinline__ int wave_items_pick(const WaveItems<NJ>& w, int g, int lane, int* rows, int& n, int cap, bool& over)
{
    over = false;
    int eg = -1;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const uint64_t m = __builtin_amdgcn_ballot_w64(w.first[j] && w.rank[j] == g);
        if (m) eg = __shfl(w.e[j], __builtin_ctzll(m), 64);
    }
    n = 0;
    if (eg < 0) return -1;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
        const bool hit = w.e[j] == eg;
        const uint64_t m = __builtin_amdgcn_ballot_w64(hit);
        if (hit && n + lanes_below(m) < cap) rows[n + lanes_below(m)] = lane + 64 * j;
        n += __builtin_popcountll(m);
    }
    if (n > cap) { n = cap; over = true; }
    return eg;
}

// 16-byte streaming load (weights are read once: keep them out of the way of reused data)
__device__ __forceinline__ uint4 ld_stream16(const void* p)
{
    typedef const __attribute__((address_space(1))) v4i* gptr;   // global memory: a plain global_load, never a flat one
    const v4i v = __builtin_nontemporal_load((gptr)(uintptr_t)p);
    return make_uint4((uint32_t)v.x, (uint32_t)v.y, (uint32_t)v.z, (uint32_t)v.w);
}

// 16 bytes written once and read by a later kernel: a store that does not displace what the writing kernel still reads
__device__ __forceinline__ void st_stream16(void* p, uint4 v)
{
    typedef __attribute__((address_space(1))) v4i* gptr;
    __builtin_nontemporal_store(v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w}, (gptr)(uintptr_t)p);
}

// A routing index as the kernels use it: forced into [0, E - 1], so that an index far outside the table cannot become an address far
// outside the weights.  Valid routes are unchanged.  The kernels' contract is the reference's - every index in range and the experts
// of one token row distinct (an item then never holds more rows than the call).  Routes that break it (NaN logits in a caller's router,
// indices read before the router has written them) stay inside the kernels' arrays all the same: the clamp bounds the index, the
// single-launch kernels cap an item's rows at what their arrays hold (wave_items_pick) and raise the workspace's error flag, and the
// rows concerned come out as NaN.
__device__ __forceinline__ int clamp_expert(int e, int E) { return min(max(e, 0), E - 1); }

inline int launch_status() { return (int)hipGetLastError(); }
inline size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

}  // namespace spk
