// Dense FP8 (E4M3, one binary32 scale per 128 x 128 block) GEMV on weights packed once at load into the matrix unit's operand
// order, for 1-16 activation rows.  The format and the product are those of reference/ds41/kernel.py:96-119 (fp8_gemm, block
// 128); the packing plays the part moe_pack plays for the experts (reference engine-rs/src/ds41/kern.rs:718-770): done once when
// the weights are loaded, never per call.
//
// Packed layout ("T16"): the matrix is cut into tiles of 16 rows x 128 k, 2048 bytes each, tile (nt, kb) at
// ((nt * k / 128) + kb) * 2048.  A tile is two halves of 64 lanes x 16 bytes; lane (i = lane % 16, g = lane / 16) of half h
// holds W[16 nt + i][128 kb + 64 h + 8 g .. + 8] followed by W[16 nt + i][128 kb + 64 h + 32 + 8 g .. + 8]: the A operands
// of two v_mfma_f32_16x16x32_bf16 steps (after the exact E4M3 -> bf16 convert), so a wave reads 1 KB of consecutive bytes per
// load instruction and nothing has to be transposed.  With the row-major matrix the same operand order asks one instruction for
// 64-byte pieces of 16 rows, which reads a third slower than whole lines, and the lane-wise dot-product kernel that reads whole
// lines pays for every further activation row on the vector ALU (dot products and the fold of 16 row sums across lanes); here
// the convert is the only vector-ALU work per weight and the cost does not depend on the number of activation rows.
#include "common.hpp"
#include "fp8_packed.hpp"

using namespace spk;

namespace {

typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf8v __attribute__((ext_vector_type(8)));
constexpr int T16_TILE = 2048;         // bytes of a tile: 16 rows x 128 k
constexpr int T16_SPAN = 8;            // tiles (128-wide K blocks) of a wave
constexpr int T16_WAVES = 8;           // waves of a workgroup: K up to 8192

// one thread per 16 bytes of the packed matrix
__global__ __launch_bounds__(256) void fp8_t16_pack_kernel(const uint8_t* __restrict__ w, uint8_t* __restrict__ out, int n, int k)
{
    const int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (u >= (int64_t)n * k / 16) return;
    const int lane = (int)(u & 63), h = (int)((u >> 6) & 1), nkb = k >> 7;
    const int64_t tile = u >> 7;
    const int kb = (int)(tile % nkb), i = lane & 15, g = lane >> 4;
    const int64_t nt = tile / nkb;
    const uint8_t* src = w + (nt * 16 + i) * (int64_t)k + kb * 128 + 64 * h + 8 * g;
    const uint2 a = *(const uint2*)src, b = *(const uint2*)(src + 32);
    *(uint4*)(out + u * 16) = make_uint4(a.x, a.y, b.x, b.y);
}

// Workgroup = one tile row (16 weight rows), wave = T16_SPAN K blocks of it.  A wave's loads return in the order it issued them, so
// everything small goes first: the wave's own span of the activation rows (up to MX rows x 1024 k, staged in a wave-private LDS
// area: no workgroup barrier before the first multiply) and its block scales, then all of its weight loads at once; the matrix
// instructions of a K block start when that block's two loads have arrived.  A K block is four matrix instructions summed from
// zero and added with its block scale, the waves' sums are added through LDS in wave order.
// Lane (j = lane % 16, g = lane / 16) supplies activation row j as the B operand (rows past m repeat the last one: a column of
// the product depends on its own activation row only, and those columns are not stored) and receives rows 4 g .. 4 g + 3 of
// column j.
constexpr int T16_XLD = T16_SPAN * 128 + 8;        // bf16 per staged activation row: 16-byte reads of neighbouring rows start 16 bytes apart
// E8: the scales are E8M0 bytes per 32 rows x 32 k (the format of ds41_fp8_gemv, reference engine-rs/shim/ds41.cu:28-73) instead of
// binary32 per 128 x 128: a matrix instruction covers exactly one scale block of 32 k, so each of a K block's four instructions
// starts from zero and is added with its own power of two.
template <int MX, bool E8>
__global__ __launch_bounds__(64 * T16_WAVES) void fp8_t16_gemv_kernel(const uint16_t* __restrict__ x, int64_t xs, const uint8_t* __restrict__ wt,
                                                                       const void* __restrict__ scp, float* __restrict__ y, int m, int n, int k)
{
    extern __shared__ __align__(16) uint16_t t16_x[];     // [wave][MX][T16_XLD]
    __shared__ float red[T16_WAVES][16][16];              // [wave][activation row][tile row]
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nw = blockDim.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int nt = blockIdx.x, n0 = nt * 16, nkb = k >> 7;
    const int kb0 = wave * T16_SPAN, nb = min(T16_SPAN, nkb - kb0);          // 1 .. T16_SPAN by the launch
    // the span's activations: 16-byte pieces, piece c = lane + 64 u of the MX x (T16_SPAN * 16) pieces of the wave's rows
    uint16_t* xw = t16_x + (size_t)wave * (MX * T16_XLD);
    // (left to itself the compiler sinks these loads below the weight loads, next to the LDS writes, where each one waits for the
    // whole weight span: a scheduling fence keeps them ahead, and the compiler counts the wait before the writes itself - loads
    // return in issue order, so the writes wait for everything but the 2 * T16_SPAN weight loads)
    v4i xt[2 * MX];
#pragma unroll
    for (int u = 0; u < 2 * MX; ++u) {
        const int c = lane + 64 * u, r = min(c >> 7, m - 1), col = min(c & 127, nb * 16 - 1) * 8;
        const uint16_t* xp = x + (int64_t)r * xs + kb0 * 128 + col;
        xt[u] = *(const v4i*)xp;
    }
    // the span's scales, one K block per lane (lanes 0-7): a binary32 factor, or the four E8M0 bytes of the block's steps
    float scv = 0.f;
    uint32_t scw = 0u;
    if constexpr (E8) scw = ((const uint32_t*)((const uint8_t*)scp + (int64_t)(n0 >> 5) * (k >> 5)))[kb0 + min(lane & 7, nb - 1)];
    else scv = ((const float*)scp)[(int64_t)(n0 >> 7) * nkb + kb0 + min(lane & 7, nb - 1)];
    const uint8_t* wp = wt + ((int64_t)nt * nkb + kb0) * T16_TILE + lane * 16;
    __builtin_amdgcn_sched_barrier(0);
    // (past a short span's end the last K block is requested again: the same lines, nothing is used)
    uint4 p[T16_SPAN][2];
#pragma unroll
    for (int b = 0; b < T16_SPAN; ++b) {
        const int bb = min(b, nb - 1);
        p[b][0] = ld_stream16(wp + bb * T16_TILE); p[b][1] = ld_stream16(wp + bb * T16_TILE + 1024);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < 2 * MX; ++u) {
        const int c = lane + 64 * u;
        *(v4i*)(xw + (c >> 7) * T16_XLD + (c & 127) * 8) = xt[u];
    }
    __builtin_amdgcn_wave_barrier();                       // the area belongs to this wave: its LDS operations execute in order
    asm volatile("" ::: "memory");
    const uint16_t* xr = xw + min(j, m - 1) * T16_XLD + 8 * g;
    v4f tot = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int b = 0; b < T16_SPAN; ++b) {
        if (b < nb) {
            v4f cur = v4f{0.f, 0.f, 0.f, 0.f};
            const uint32_t sdw = E8 ? (uint32_t)__builtin_amdgcn_readlane((int)scw, b) : 0u;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const uint32_t pw[4] = {p[b][h].x, p[b][h].y, p[b][h].z, p[b][h].w};
                bf2 wv[8];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    wv[2 * q + 0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(pw[q], 1.0f, false);
                    wv[2 * q + 1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(pw[q], 1.0f, true);
                }
                const uint4 x0 = *(const uint4*)(xr + b * 128 + 64 * h), x1 = *(const uint4*)(xr + b * 128 + 64 * h + 32);
                bf8v a0, a1, b0, b1;
                __builtin_memcpy(&a0, &wv[0], 16); __builtin_memcpy(&a1, &wv[4], 16);
                __builtin_memcpy(&b0, &x0, 16); __builtin_memcpy(&b1, &x1, 16);
                if constexpr (E8) {
                    const v4f zero = v4f{0.f, 0.f, 0.f, 0.f};
                    const v4f c0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, zero, 0, 0, 0);
                    const v4f c1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1, zero, 0, 0, 0);
                    const float s0 = e8m0_to_f32((sdw >> (16 * h)) & 0xffu), s1 = e8m0_to_f32((sdw >> (16 * h + 8)) & 0xffu);
#pragma unroll
                    for (int v = 0; v < 4; ++v) { tot[v] = __builtin_fmaf(c0[v], s0, tot[v]); tot[v] = __builtin_fmaf(c1[v], s1, tot[v]); }
                } else {
                    cur = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, cur, 0, 0, 0);
                    cur = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b1, cur, 0, 0, 0);
                }
            }
            if constexpr (!E8) {
                const float s = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(scv), b));
#pragma unroll
                for (int v = 0; v < 4; ++v) tot[v] = __builtin_fmaf(cur[v], s, tot[v]);
            }
        }
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][j][4 * g + v] = tot[v];
    __syncthreads();
    for (int t = threadIdx.x; t < 16 * m; t += (int)blockDim.x) {       // a workgroup may have a single wave
        const int r = t >> 4, i = t & 15;
        float v = red[0][r][i];
        for (int u = 1; u < nw; ++u) v += red[u][r][i];
        y[(int64_t)r * n + n0 + i] = v;
    }
}

// The bf16-activation kernel (fp8_t16_gemv_kernel) on the ROW-MAJOR matrix, for spark_fp8_block128_gemv / ds41_fp8_gemv with two or
// more activation rows and for ds41_fp8_gemv_mx_q.  A load instruction reads 256 bytes of each of four rows (lane l: row 4 i +
// l / 16, bytes 16 (l % 16) of a 256-wide chunk; whole lines side by side: the operand's own order, 64-byte pieces of 16 rows,
// reads a third slower), all sixteen loads of the wave's span in flight at once, and a chunk goes through a wave-private LDS tile
// into the operand order right before its eight matrix instructions (a lane's operand: 8 bytes of its row at k = 32 s + 8 g).
// The last tile of a matrix whose row count is not a multiple of 16 reads its last row again and stores the rows there are.
// XMODE: how the activations arrive.  0: bf16 rows (stride xs; rpg > 0: a block-diagonal weight, the tile's group reads its own k
// inputs).  1: act-quantised rows, E4M3 codes aq [m, k] with E8M0 scales as_ [m, k / 32] (ds41_act_quant_fp8's output).
// 2: bf16 rows to quantise here, by the wave for its own span, by the rule of act_quant (the codes and scales ds41_act_quant_fp8
// would write: the same result as with codes given); a lane takes 16 neighbouring values, two lanes share a block of 32.
// In modes 1 and 2 the wave stages code x 2^(scale - 127) as bf16, which is exact (four significant bits), so the product is the
// one of ds41_fp8_gemv on the dequantised activations: bf16 x bf16 products are exact in binary32 and the sums come out 1e-7 from
// the exact value.  (The scaled f8f6f4 matrix instruction takes codes and scale bytes as they are and saves the converts, but its
// 128-deep sums measured 1.3e-5 .. 3e-5 from the exact value relative to the largest output, over the reference's own threshold
// for this product, kern.rs:1863-1867.)
// LOOP: K beyond eight spans a workgroup; a wave's next span is nw spans further on.
constexpr int RM_TS = 256 + 16;        // row stride of a wave's transpose tile: 16-byte reads down its 16 rows hit distinct banks
// CH: 256-wide chunks of a wave's span (1, 2 or 4: a wave has 4 CH weight loads in flight); up to 16 waves a workgroup for the
// shorter spans, 8 for the longest (whose instances need more than 128 registers).
template <int CH> constexpr int rm_waves() { return CH == 4 ? 8 : 16; }
template <int CH> constexpr size_t rm_dyn() { return (size_t)(CH == 4 ? 150 : 140) * 1024; }     // dynamic LDS beside the 8 / 16 KB of wave sums
template <int MX, bool E8, bool LOOP, int XMODE, int CH>
__global__ __launch_bounds__(64 * rm_waves<CH>()) void fp8_rm_gemv_kernel(const uint16_t* __restrict__ x, int64_t xs, const uint8_t* __restrict__ aq,
                                                                            const uint8_t* __restrict__ as_, const uint8_t* __restrict__ w,
                                                                            const void* __restrict__ scp, void* __restrict__ y, int ob16, int m, int n, int k, int rpg)
{
    static_assert(XMODE == 0 || E8, "act-quantised activations go with E8M0 weight scales");
    static_assert(CH == 1 || CH == 2 || CH == 4, "chunks of a span");
    constexpr int SPAN = 2 * CH;                           // 128-wide K blocks of a wave's span
    constexpr int XLD = SPAN * 128 + 8;                    // bf16 per staged activation row: 16-byte reads of neighbouring rows start 16 bytes apart
    static_assert(XMODE == 0 ? MX * SPAN >= 4 : MX * SPAN >= 8, "every lane stages at least one piece");
    extern __shared__ __align__(16) unsigned char t16q_x[];          // [wave][MX * XLD bf16 + 16 * RM_TS tile]
    __shared__ float red[rm_waves<CH>()][16][16];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nw = blockDim.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int nt = blockIdx.x, n0 = nt * 16, nkb = k >> 7;
    unsigned char* base = t16q_x + (size_t)wave * (MX * XLD * 2 + 16 * RM_TS);
    uint16_t* xw = (uint16_t*)base;
    unsigned char* tw = base + MX * XLD * 2;
    const int lr = lane >> 4, lc = (lane & 15) * 16;
    const uint16_t* xr = xw + min(j, m - 1) * XLD + 8 * g;
    v4f tot = v4f{0.f, 0.f, 0.f, 0.f}, tot2 = v4f{0.f, 0.f, 0.f, 0.f};
    int64_t xoff = 0;                                                // a block-diagonal weight: the tile's group reads its own k inputs
    if constexpr (XMODE == 0) xoff = rpg ? (int64_t)(n0 / rpg) * k : 0;
    int kb0 = wave * SPAN;
    do {
    const int nb = min(SPAN, nkb - kb0);                   // an even count by the launch (k a multiple of 256)
    constexpr int NU = XMODE == 0 ? MX * SPAN / 4 : MX * SPAN / 8;     // pieces a lane stages: 8 bf16 values / 16 codes or values each
    constexpr int PR = XMODE == 0 ? SPAN * 16 : SPAN * 8;             // pieces of a row's span
    v4i xt[XMODE == 2 ? 2 * NU : NU];
    int sb[XMODE == 1 ? NU : 1];
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        // piece c = lane + 64 u: row c / PR, position c % PR of the span (a piece past a short span's end reads the span's last
        // piece again, a row past m the last row: neither is used)
        const int c = lane + 64 * u, r = min(c / PR, m - 1), pc = min(c % PR, nb * (PR / SPAN) - 1);
        if constexpr (XMODE == 0) {
            const uint16_t* xp = x + xoff + (int64_t)r * xs + kb0 * 128 + pc * 8;
            xt[u] = *(const v4i*)xp;
        } else if constexpr (XMODE == 1) {
            const uint8_t* xp = aq + (int64_t)r * k + kb0 * 128 + pc * 16;
            const uint8_t* sp = as_ + (int64_t)r * (k >> 5) + kb0 * 4 + (pc >> 1);          // the scale byte of the piece's block of 32
            xt[u] = *(const v4i*)xp;
            sb[u] = *sp;
        } else {
            const uint16_t* xp = x + (int64_t)r * xs + kb0 * 128 + pc * 16;
            xt[2 * u] = *(const v4i*)xp;
            xt[2 * u + 1] = *(const v4i*)(xp + 8);
        }
    }
    float scv = 0.f;
    uint32_t scw = 0u;
    if constexpr (E8) scw = ((const uint32_t*)((const uint8_t*)scp + (int64_t)(n0 >> 5) * (k >> 5)))[kb0 + min(lane & (SPAN - 1), nb - 1)];
    else scv = ((const float*)scp)[(int64_t)(n0 >> 7) * nkb + kb0 + min(lane & (SPAN - 1), nb - 1)];
    const uint8_t* wp[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) wp[i] = w + (int64_t)min(n0 + lr + 4 * i, n - 1) * k + kb0 * 128 + lc;
    __builtin_amdgcn_sched_barrier(0);
    uint4 p[CH][4];
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
        const int cc = min(ch, (nb >> 1) - 1);            // past a short span's end: the last chunk again, unused
#pragma unroll
        for (int i = 0; i < 4; ++i) p[ch][i] = ld_stream16(wp[i] + cc * 256);
    }
    // The activation and scale loads stay ahead of the weight loads (a wave's loads return in issue order: staging then waits for
    // everything but the 4 CH weight loads, and the compiler counts that wait itself); nothing moves across the two fences.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < NU; ++u) {
        const int c = lane + 64 * u;
        if constexpr (XMODE == 0) {
            *(v4i*)(xw + (c / PR) * XLD + (c % PR) * 8) = xt[u];
        } else {
            uint32_t cw[4], e;
            if constexpr (XMODE == 1) {
                cw[0] = (uint32_t)xt[u].x; cw[1] = (uint32_t)xt[u].y; cw[2] = (uint32_t)xt[u].z; cw[3] = (uint32_t)xt[u].w;
                e = (uint32_t)sb[u] & 0xffu;
            } else {
                // act_quant of the piece's 16 values: the block maximum over the two lanes of a 32-block, one scale per block
                const uint32_t xu[8] = {(uint32_t)xt[2 * u].x, (uint32_t)xt[2 * u].y, (uint32_t)xt[2 * u].z, (uint32_t)xt[2 * u].w,
                                        (uint32_t)xt[2 * u + 1].x, (uint32_t)xt[2 * u + 1].y, (uint32_t)xt[2 * u + 1].z, (uint32_t)xt[2 * u + 1].w};
                float v[16], am = 0.f;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    v[2 * i] = __uint_as_float(xu[i] << 16); v[2 * i + 1] = __uint_as_float(xu[i] & 0xffff0000u);
                    am = fmaxf(am, fmaxf(fabsf(v[2 * i]), fabsf(v[2 * i + 1])));
                }
                am = fmaxf(am, lane_xor<1>(am, lane));
                e = aq_scale(am);
#pragma unroll
                for (int i = 0; i < 4; ++i) cw[i] = aq_word4(v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3], e);
            }
            // code x 2^(e - 127) as bf16: exact
            const float sc = e8m0_to_f32(e);
            bf2 o[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                o[2 * i] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(cw[i], sc, false);
                o[2 * i + 1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(cw[i], sc, true);
            }
            v4i s0, s1;
            __builtin_memcpy(&s0, &o[0], 16); __builtin_memcpy(&s1, &o[4], 16);
            uint16_t* dst = xw + (c / PR) * XLD + (c % PR) * 16;
            *(v4i*)dst = s0; *(v4i*)(dst + 8) = s1;
        }
    }
    __builtin_amdgcn_wave_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int ch = 0; ch < CH; ++ch) {
        if (2 * ch < nb) {
#pragma unroll
            for (int i = 0; i < 4; ++i) *(uint4*)(tw + (4 * i + lr) * RM_TS + lc) = p[ch][i];
            __builtin_amdgcn_wave_barrier();               // the tile belongs to this wave: its LDS operations execute in order
            asm volatile("" ::: "memory");
            uint2 aw[8];
#pragma unroll
            for (int s8 = 0; s8 < 8; ++s8) aw[s8] = *(const uint2*)(tw + j * RM_TS + 32 * s8 + 8 * g);
            __builtin_amdgcn_wave_barrier();
            asm volatile("" ::: "memory");
#pragma unroll
            for (int hb = 0; hb < 2; ++hb) {               // the chunk's two 128-wide K blocks
                const int b = 2 * ch + hb;
                v4f cur = v4f{0.f, 0.f, 0.f, 0.f};
                const uint32_t sdw = E8 ? (uint32_t)__builtin_amdgcn_readlane((int)scw, b) : 0u;
#pragma unroll
                for (int st = 0; st < 4; ++st) {
                    const uint2 a2 = aw[4 * hb + st];
                    // E8M0 weight scales go into the convert (a power of two: the scaled weight is still exact in bf16), and the
                    // matrix instructions add up in two accumulators in turn
                    const float ws = E8 ? e8m0_to_f32((sdw >> (8 * st)) & 0xffu) : 1.0f;
                    bf2 wv[4];
                    wv[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(a2.x, ws, false); wv[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(a2.x, ws, true);
                    wv[2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(a2.y, ws, false); wv[3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(a2.y, ws, true);
                    const uint4 xq = *(const uint4*)(xr + b * 128 + 32 * st);
                    bf8v a0, b0;
                    __builtin_memcpy(&a0, &wv[0], 16); __builtin_memcpy(&b0, &xq, 16);
                    if constexpr (E8) {
                        if (st & 1) tot2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, tot2, 0, 0, 0);
                        else tot = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, tot, 0, 0, 0);
                    } else {
                        cur = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, cur, 0, 0, 0);
                    }
                }
                if constexpr (!E8) {
                    const float sc = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(scv), b));
#pragma unroll
                    for (int v = 0; v < 4; ++v) tot[v] = __builtin_fmaf(cur[v], sc, tot[v]);
                }
            }
        }
    }
    if constexpr (LOOP) { __builtin_amdgcn_wave_barrier(); asm volatile("" ::: "memory"); }     // the staged span is read before the next one is written
    kb0 += nw * SPAN;
    } while (LOOP && kb0 < nkb);
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][j][4 * g + v] = tot[v] + tot2[v];
    __syncthreads();
    for (int t = threadIdx.x; t < 16 * m; t += (int)blockDim.x) {
        const int r = t >> 4, i = t & 15;
        if (n0 + i >= n) continue;
        float v = red[0][r][i];
        for (int u = 1; u < nw; ++u) v += red[u][r][i];
        const int64_t o = (int64_t)r * n + n0 + i;
        if (ob16) ((uint16_t*)y)[o] = f32_to_bf16(v); else ((float*)y)[o] = v;
    }
}

}  // namespace

// ================================================================ C ABI

// w E4M3 [n, k] row-major -> out [n * k] bytes in the T16 order; n a multiple of 16, k of 128.  Once per weight matrix, at load.
SPARK_API int spark_fp8_t16_pack(const void* w, void* out, int n, int k, hipStream_t st)
{
    if (!w || !out || n < 16 || n % 16 != 0 || k < 128 || k % 128 != 0) return 1;
    const int64_t units = (int64_t)n * k / 16;
    fp8_t16_pack_kernel<<<(unsigned)((units + 255) / 256), 256, 0, st>>>((const uint8_t*)w, (uint8_t*)out, n, k);
    return launch_status();
}
// y f32 [m, n] = x bf16 [m, k] (row stride k) times the packed matrix, scales f32 [ceil(n / 128), k / 128] as for
// spark_fp8_block128_gemv; m 1..16 (more than eight rows: two launches), n a multiple of 16, k a multiple of 128 up to 8192.
namespace {
template <bool E8>
int launch_t16_gemv(const void* x, const void* wt, const void* scales, float* y, int m, int n, int k, hipStream_t st)
{
    const int nkb = k / 128, nw = (nkb + T16_SPAN - 1) / T16_SPAN;
    if (nw > T16_WAVES) return 1;
    static const bool attr = hipFuncSetAttribute((const void*)fp8_t16_gemv_kernel<8, E8>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 T16_WAVES * 8 * T16_XLD * 2) == hipSuccess &&
                             hipFuncSetAttribute((const void*)fp8_t16_gemv_kernel<4, E8>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 T16_WAVES * 4 * T16_XLD * 2) == hipSuccess;
    if (!attr) return (int)hipErrorInvalidValue;
    // one, two, up to four or up to eight rows per launch (the staged rows a wave requests), more in two launches: a row's value
    // does not depend on the rows beside it
    for (int r0 = 0; r0 < m; r0 += 8) {
        const int mm = m - r0 < 8 ? m - r0 : 8, mx = mm <= 1 ? 1 : mm <= 2 ? 2 : mm <= 4 ? 4 : 8;
        const uint16_t* xp = (const uint16_t*)x + (int64_t)r0 * k;
        float* yp = y + (int64_t)r0 * n;
        const size_t lds = (size_t)nw * mx * T16_XLD * 2;
        const dim3 grid(n / 16), block(64 * nw);
        if (mx == 1) fp8_t16_gemv_kernel<1, E8><<<grid, block, lds, st>>>(xp, (int64_t)k, (const uint8_t*)wt, scales, yp, mm, n, k);
        else if (mx == 2) fp8_t16_gemv_kernel<2, E8><<<grid, block, lds, st>>>(xp, (int64_t)k, (const uint8_t*)wt, scales, yp, mm, n, k);
        else if (mx == 4) fp8_t16_gemv_kernel<4, E8><<<grid, block, lds, st>>>(xp, (int64_t)k, (const uint8_t*)wt, scales, yp, mm, n, k);
        else fp8_t16_gemv_kernel<8, E8><<<grid, block, lds, st>>>(xp, (int64_t)k, (const uint8_t*)wt, scales, yp, mm, n, k);
    }
    return launch_status();
}
}  // namespace
SPARK_API int spark_fp8_block128_gemv_t16(const void* x, const void* wt, const float* scales, float* y, int m, int n, int k, hipStream_t st)
{
    if (!x || !wt || !scales || !y || m < 1 || m > 16 || n < 16 || n % 16 != 0 || k < 128 || k % 128 != 0) return 1;
    return launch_t16_gemv<false>(x, wt, scales, y, m, n, k, st);
}
// The same on a matrix with E8M0 scales per 32 x 32 ([n / 32, k / 32] bytes, the format of ds41_fp8_gemv: reference
// engine-rs/shim/ds41.cu:28-73), packed by spark_fp8_t16_pack like the block-128 matrix; n a multiple of 32.
SPARK_API int spark_fp8_e8m0_gemv_t16(const void* x, const void* wt, const void* scales, float* y, int m, int n, int k, hipStream_t st)
{
    if (!x || !wt || !scales || !y || m < 1 || m > 16 || n < 32 || n % 32 != 0 || k < 128 || k % 128 != 0) return 1;
    return launch_t16_gemv<true>(x, wt, scales, y, m, n, k, st);
}
// The row-major kernel's launch: 1 when the shape is not this kernel's (the caller goes on to its other kernels), else the launch
// status.  k a multiple of 256, any n; rows in passes of as many as fit beside the tiles in LDS.
int g_rm_ch = 0;                       // diagnostics: chunks of a wave's span (1, 2, 4), 0 = by the shape
namespace {
template <bool E8, int XMODE, int CH, bool LOOP>
int rm_launch_ch(const uint16_t* x, int64_t xs, const uint8_t* aq, const uint8_t* as_, const void* w, const void* scales, void* y, int ob16, int m, int n, int k, int rpg,
                 hipStream_t st)
{
    constexpr int SPAN = 2 * CH, XLD = SPAN * 128 + 8, MXMIN = XMODE == 0 ? (CH == 1 ? 2 : 1) : 8 / SPAN;
    const int nkb = k / 128, spans = (nkb + SPAN - 1) / SPAN, nw = spans < rm_waves<CH>() ? spans : rm_waves<CH>();
    if (!LOOP && spans > nw) return 1;
    const auto need = [&](int mx) { return (size_t)nw * (mx * XLD * 2 + 16 * RM_TS); };
    constexpr size_t RM_DYN = rm_dyn<CH>();
    // rows per pass: sixteen coded rows where they fit beside the tiles (K up to 3328, and 4096 on four-chunk spans), else eight, else four
    const int per = XMODE == 1 && need(16) <= RM_DYN ? 16 : need(8) <= RM_DYN ? 8 : 4;
    const unsigned grid = (unsigned)((n + 15) / 16);
#define RMK(MXX)                                                                                                                                 \
    do {                                                                                                                                         \
        static const bool attr = hipFuncSetAttribute((const void*)fp8_rm_gemv_kernel<MXX, E8, LOOP, XMODE, CH>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RM_DYN) == hipSuccess; \
        if (!attr) return (int)hipErrorInvalidValue;                                                                                             \
        fp8_rm_gemv_kernel<MXX, E8, LOOP, XMODE, CH><<<grid, 64 * nw, need(MXX), st>>>(xp, xs, qp, sp, (const uint8_t*)w, scales, yp, ob16, mm, n, k, rpg); \
    } while (0)
    for (int r0 = 0; r0 < m; r0 += per) {
        const int mm = m - r0 < per ? m - r0 : per;
        int mx = mm <= 2 ? 2 : mm <= 4 ? 4 : mm <= 8 ? 8 : 16;
        if (mx < MXMIN) mx = MXMIN;
        const uint16_t* xp = x ? x + (int64_t)r0 * xs : nullptr;
        const uint8_t* qp = aq ? aq + (int64_t)r0 * k : nullptr;
        const uint8_t* sp = as_ ? as_ + (int64_t)r0 * (k / 32) : nullptr;
        void* yp = ob16 ? (void*)((uint16_t*)y + (int64_t)r0 * n) : (void*)((float*)y + (int64_t)r0 * n);
        if (mx == 2) { if constexpr (MXMIN <= 2) RMK(2); }
        else if (mx == 4) RMK(4);
        else if (mx == 8) RMK(8);
        else { if constexpr (XMODE == 1) RMK(16); }
    }
#undef RMK
    return launch_status();
}
template <bool E8, int XMODE>
int rm_launch(const uint16_t* x, int64_t xs, const uint8_t* aq, const uint8_t* as_, const void* w, const void* scales, void* y, int ob16, int m, int n, int k, int rpg,
              hipStream_t st)
{
    // Chunks of a wave's span.  Short spans give a workgroup more waves, each with less to do once its loads are back: one chunk
    // up to K = 1024, two up to 8192 (1280 x 5120: 5.1 -> 4.5 us, 5120 x 3072: 5.9 -> 5.7).  Four where the matrix has more tiles
    // than one a CU and K is 4096 and more (fewer, longer waves leave room for more workgroups on a CU: 25600 x 6144 31.7 -> 27.3
    // us, 7168 x 4096 7.5 -> 7.3), where eight staged rows fit beside four-chunk spans only (K 5632 .. 7424), and beyond 8192,
    // where the waves take further spans in turn.  The choice does not look at the row count: a row's value must not depend on it.
    const int chunks = k / 256, tiles = (n + 15) / 16;
    int ch = chunks <= 4 ? 1 : chunks <= 32 ? 2 : 4;
    if (ch == 2 && tiles > 256 && chunks >= 16) ch = 4;
    if (ch == 2 && (size_t)((chunks + 1) / 2) * (8 * (4 * 128 + 8) * 2 + 16 * RM_TS) > rm_dyn<2>() &&
        (size_t)((chunks + 3) / 4) * (8 * (8 * 128 + 8) * 2 + 16 * RM_TS) <= rm_dyn<4>()) ch = 4;
    if (g_rm_ch == 1 || g_rm_ch == 2 || g_rm_ch == 4) ch = g_rm_ch;
    if (ch == 1 && chunks <= 16) return rm_launch_ch<E8, XMODE, 1, false>(x, xs, aq, as_, w, scales, y, ob16, m, n, k, rpg, st);
    if (ch <= 2 && chunks <= 32) return rm_launch_ch<E8, XMODE, 2, false>(x, xs, aq, as_, w, scales, y, ob16, m, n, k, rpg, st);
    if (chunks <= 32) return rm_launch_ch<E8, XMODE, 4, false>(x, xs, aq, as_, w, scales, y, ob16, m, n, k, rpg, st);
    return rm_launch_ch<E8, XMODE, 4, true>(x, xs, aq, as_, w, scales, y, ob16, m, n, k, rpg, st);
}
}  // namespace
SPARK_API void spark_debug_rm_span(int ch) { g_rm_ch = ch; }

// ds41_fp8_gemv_mx_q: activations as codes (aq, as_; any row count up to 32) or as bf16 rows to quantise inside (x, up to 16 rows)
int spk::fp8q_rowmajor_launch(const void* x, const void* aq, const void* as_, const void* w, const void* ws, void* y, int m, int n, int k, int ob16, hipStream_t st)
{
    if (!w || !ws || !y || m < 1 || m > 32 || n < 1 || k < 256 || k % 256 != 0) return 1;
    if (aq) return as_ ? rm_launch<true, 1>(nullptr, 0, (const uint8_t*)aq, (const uint8_t*)as_, w, ws, y, ob16, m, n, k, 0, st) : 1;
    if (!x) return 1;
    return rm_launch<true, 2>((const uint16_t*)x, k, nullptr, nullptr, w, ws, y, ob16, m, n, k, 0, st);
}

// spark_fp8_block128_gemv / ds41_fp8_gemv (e8: E8M0 scales per 32 x 32, else binary32 per 128 x 128), bf16 activations used as given;
// m 1..8; rpg > 0: a block-diagonal weight in groups of rpg rows (a multiple of 16: a tile lies inside one group), group t reading
// the input elements [t k, +k) of its row.
int spk::fp8_rowmajor_launch(const void* x, int64_t xs, const void* w, const void* scales, float* y, int m, int n, int k, int e8, int rpg, hipStream_t st)
{
    if (!x || !w || !scales || !y || m < 1 || m > 8 || n < 1 || k < 256 || k % 256 != 0 || xs % 8 != 0 || rpg < 0 || rpg % 16 != 0) return 1;
    if (xs < (rpg ? (int64_t)((n + rpg - 1) / rpg) * k : (int64_t)k)) return 1;
    if (e8) return rm_launch<true, 0>((const uint16_t*)x, xs, nullptr, nullptr, w, scales, y, 0, m, n, k, rpg, st);
    return rm_launch<false, 0>((const uint16_t*)x, xs, nullptr, nullptr, w, scales, y, 0, m, n, k, rpg, st);
}
