// Weight-only FP8 (E4M3) GEMV with ONE binary32 scale per output row, for 1-32 activation rows: the format of the reference's GLM
// dense / shared-expert projections (engine-rs/shim/fp8.cu:13-22 fp8_gemv, :110-178 the entry points; quantiser
// engine-rs/src/dense_fp8.rs:59-62: scale = row amax / 448).
//
//   y[r, n] = (sum_k a(x[r, k]) * e4m3(w[n, k])) * scale[n]        a = round to binary16 (glm53_fp8_dense_cuda) or to bf16
//                                                                  (glm53_fp8_bf16_cuda); products exact, binary32 sums
//
// MI355X design.  The matrix is row-major as the reference hands it over.  Workgroup = 16 weight rows, its waves take 512-wide spans
// of K in turn.  A load instruction reads 256 bytes of each of four rows (whole lines; the matrix unit's own operand order, 64-byte
// pieces of 16 rows, reads a third slower), and a 256-wide chunk goes through a wave-private LDS tile into the operand order right
// before its eight matrix instructions.  E4M3 converts exactly to binary16 and to bf16, the activations are rounded once to the same
// type when the wave stages its span of them (wave-private LDS: no workgroup barrier before the first multiply), so every product is
// exact in binary32 on v_mfma_f32_16x16x32_f16 / _bf16 and the convert is the only vector-ALU work per weight, whatever the number of
// activation rows.  The row scale multiplies the finished sum.  A row's value does not depend on the rows beside it.
// K that is not a multiple of 256 (the reference takes multiples of 64) runs a plain wave-per-row kernel.
#include "common.hpp"

using namespace spk;

namespace {

typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf8v __attribute__((ext_vector_type(8)));
typedef _Float16 h8v __attribute__((ext_vector_type(8)));

constexpr int RS_WAVES = 16;           // most waves of a workgroup
constexpr int RS_SPAN = 4;             // 128-wide K blocks of a wave's span (two 256-wide chunks)
constexpr int RS_XLD = RS_SPAN * 128 + 8;      // 16-bit values per staged activation row: 16-byte reads of neighbouring rows start 16 bytes apart
constexpr int RS_TS = 256 + 16;        // row stride of a wave's transpose tile: 16-byte reads down its 16 rows hit distinct banks

__device__ __forceinline__ uint32_t pack16(float a, float b, bool f16)
{
    if (f16) { const h2 v = h2{(_Float16)a, (_Float16)b}; uint32_t u; __builtin_memcpy(&u, &v, 4); return u; }
    return (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
}

// MX: activation rows staged (rows past m repeat the last one; their columns are not stored).  F16: binary16 arithmetic, else bf16.
// XF32: x is binary32 [m, xs] and is rounded here, else 16-bit rows of the arithmetic's type used as given.
template <int MX, bool F16, bool XF32>
__global__ __launch_bounds__(64 * RS_WAVES) void fp8_rowscale_gemv_kernel(const void* __restrict__ xv, int64_t xs, const uint8_t* __restrict__ w,
                                                                          const float* __restrict__ scale, float* __restrict__ y, int oround, int m, int n, int k)
{
    extern __shared__ __align__(16) unsigned char rs_smem[];         // [wave][MX * RS_XLD 16-bit values + 16 * RS_TS tile]
    __shared__ float red[RS_WAVES][16][16];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nw = blockDim.x >> 6;
    const int j = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16, nkb = k >> 7;
    unsigned char* base = rs_smem + (size_t)wave * (MX * RS_XLD * 2 + 16 * RS_TS);
    uint16_t* xw = (uint16_t*)base;
    unsigned char* tw = base + MX * RS_XLD * 2;
    const int lr = lane >> 4, lc = (lane & 15) * 16;
    const uint16_t* xr = xw + min(j, MX - 1) * RS_XLD + 8 * g;
    v4f tot = v4f{0.f, 0.f, 0.f, 0.f}, tot2 = v4f{0.f, 0.f, 0.f, 0.f};
    constexpr int PR = RS_SPAN * 16;                       // pieces of 8 values in a row's span
    constexpr int NU = MX * PR / 64;                       // pieces a lane stages
    for (int kb0 = wave * RS_SPAN; kb0 < nkb; kb0 += nw * RS_SPAN) {
        const int nb = min(RS_SPAN, nkb - kb0);            // 2 or 4 (k is a multiple of 256)
        // the span's weight loads, all in flight at once
        uint4 p[2][4];
#pragma unroll
        for (int ch = 0; ch < 2; ++ch) {
            const int cc = min(ch, (nb >> 1) - 1);        // past a short span's end: the last chunk again, unused
#pragma unroll
            for (int i = 0; i < 4; ++i) p[ch][i] = ld_stream16(w + (int64_t)min(n0 + lr + 4 * i, n - 1) * k + kb0 * 128 + cc * 256 + lc);
        }
        // the wave's span of the activation rows: piece c = lane + 64 u is row c / PR, position c % PR (a piece past a short span's
        // end reads the span's last piece again, a row past m the last row: neither is used)
#pragma unroll
        for (int u = 0; u < NU; ++u) {
            const int c = lane + 64 * u, r = min(c / PR, m - 1), pc = min(c % PR, nb * 16 - 1);
            uint4 v;
            if constexpr (XF32) {
                const float* xp = (const float*)xv + (int64_t)r * xs + kb0 * 128 + pc * 8;
                const float4 a = *(const float4*)xp, b = *(const float4*)(xp + 4);
                v = make_uint4(pack16(a.x, a.y, F16), pack16(a.z, a.w, F16), pack16(b.x, b.y, F16), pack16(b.z, b.w, F16));
            } else v = *(const uint4*)((const uint16_t*)xv + (int64_t)r * xs + kb0 * 128 + pc * 8);
            *(uint4*)(xw + (c / PR) * RS_XLD + (c % PR) * 8) = v;
        }
        __builtin_amdgcn_wave_barrier();                   // the staged rows and the tile belong to this wave: its LDS operations execute in order
        asm volatile("" ::: "memory");
#pragma unroll
        for (int ch = 0; ch < 2; ++ch) {
            if (2 * ch < nb) {
#pragma unroll
                for (int i = 0; i < 4; ++i) *(uint4*)(tw + (4 * i + lr) * RS_TS + lc) = p[ch][i];
                __builtin_amdgcn_wave_barrier();
                asm volatile("" ::: "memory");
                uint2 aw[8];                               // this lane's operand pieces: 8 bytes of row j at k = 32 s + 8 g
#pragma unroll
                for (int s8 = 0; s8 < 8; ++s8) aw[s8] = *(const uint2*)(tw + j * RS_TS + 32 * s8 + 8 * g);
                __builtin_amdgcn_wave_barrier();
                asm volatile("" ::: "memory");
#pragma unroll
                for (int s8 = 0; s8 < 8; ++s8) {
                    const uint4 xq = *(const uint4*)(xr + (2 * ch) * 128 + 32 * s8);
                    v4f& acc = (s8 & 1) ? tot2 : tot;     // two accumulators in turn: no instruction waits for the one before it
                    if constexpr (F16) {
                        h2 wv[4];
                        wv[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(aw[s8].x, 1.0f, false); wv[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(aw[s8].x, 1.0f, true);
                        wv[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(aw[s8].y, 1.0f, false); wv[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(aw[s8].y, 1.0f, true);
                        h8v a0, b0;
                        __builtin_memcpy(&a0, &wv[0], 16); __builtin_memcpy(&b0, &xq, 16);
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, b0, acc, 0, 0, 0);
                    } else {
                        bf2 wv[4];
                        wv[0] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(aw[s8].x, 1.0f, false); wv[1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(aw[s8].x, 1.0f, true);
                        wv[2] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(aw[s8].y, 1.0f, false); wv[3] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(aw[s8].y, 1.0f, true);
                        bf8v a0, b0;
                        __builtin_memcpy(&a0, &wv[0], 16); __builtin_memcpy(&b0, &xq, 16);
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b0, acc, 0, 0, 0);
                    }
                }
            }
        }
        __builtin_amdgcn_wave_barrier();                   // the staged span is read before the next one is written
        asm volatile("" ::: "memory");
    }
    // D: lane (j, g) holds column j (activation row) of tile rows 4 g .. 4 g + 3
#pragma unroll
    for (int v = 0; v < 4; ++v) red[wave][j][4 * g + v] = tot[v] + tot2[v];
    __syncthreads();
    for (int t = threadIdx.x; t < 16 * m; t += (int)blockDim.x) {
        const int r = t >> 4, i = t & 15;
        if (n0 + i >= n) continue;
        float v = red[0][r][i];
        for (int u = 1; u < nw; ++u) v += red[u][r][i];
        v *= scale[n0 + i];
        if (oround) v = f16_bits_to_f32(f32_to_f16_bits(v));      // the binary32 product first, then its rounding: two roundings, as the reference's
        y[(int64_t)r * n + n0 + i] = v;
    }
}

// Any K that is a multiple of 8: a wave per weight row, a lane 8 neighbouring k at a time, binary32 fused multiply-adds as the
// reference's own kernel does them (fp8.cu:13-22), the 64 lane sums folded by the wave's butterfly.
template <bool F16, bool XF32>
__global__ __launch_bounds__(256) void fp8_rowscale_plain_kernel(const void* __restrict__ xv, int64_t xs, const uint8_t* __restrict__ w, const float* __restrict__ scale,
                                                                 float* __restrict__ y, int oround, int m, int n, int k)
{
    const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    for (int r = 0; r < m; ++r) {
        float sum = 0.f;
        for (int col = lane * 8; col < k; col += 512) {
            const uint2 pw = *(const uint2*)(w + (int64_t)row * k + col);
            float xf[8];
            if constexpr (XF32) {
                const float* xp = (const float*)xv + (int64_t)r * xs + col;
#pragma unroll
                for (int i = 0; i < 8; ++i) xf[i] = F16 ? (float)(_Float16)xp[i] : bf16_round(xp[i]);
            } else {
                const uint16_t* xp = (const uint16_t*)xv + (int64_t)r * xs + col;
#pragma unroll
                for (int i = 0; i < 8; ++i) xf[i] = F16 ? f16_bits_to_f32(xp[i]) : bf16_to_f32(xp[i]);
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) sum = __builtin_fmaf(xf[i], e4m3_to_f32(((i < 4 ? pw.x : pw.y) >> (8 * (i & 3))) & 0xffu), sum);
        }
        sum = wave_sum(sum);
        if (lane == 0) {
            sum *= scale[row];
            y[(int64_t)r * n + row] = oround ? f16_bits_to_f32(f32_to_f16_bits(sum)) : sum;
        }
    }
}

template <bool F16, bool XF32>
int rowscale_launch(const void* x, int64_t xs, const void* w, const float* scale, float* y, int m, int n, int k, int oround, hipStream_t st)
{
    if (k % 256 != 0) {
        fp8_rowscale_plain_kernel<F16, XF32><<<(unsigned)((n + 3) / 4), 256, 0, st>>>(x, xs, (const uint8_t*)w, scale, y, oround, m, n, k);
        return launch_status();
    }
    const int spans = (k / 128 + RS_SPAN - 1) / RS_SPAN, nw = spans < RS_WAVES ? spans : RS_WAVES;
    const unsigned grid = (unsigned)((n + 15) / 16);
    const auto need = [&](int mx) { return (size_t)nw * (mx * RS_XLD * 2 + 16 * RS_TS); };
    constexpr size_t RS_DYN = 140 * 1024;                  // dynamic LDS beside the 16 KB of wave sums
#define RSK(MXX)                                                                                                                              \
    do {                                                                                                                                      \
        static const bool attr = hipFuncSetAttribute((const void*)fp8_rowscale_gemv_kernel<MXX, F16, XF32>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                                     (int)RS_DYN) == hipSuccess;                                                              \
        if (!attr) return (int)hipErrorInvalidValue;                                                                                          \
        fp8_rowscale_gemv_kernel<MXX, F16, XF32><<<grid, 64 * nw, need(MXX), st>>>(xp, xs, (const uint8_t*)w, scale, yp, oround, mm, n, k);   \
    } while (0)
    // eight rows a launch where eight staged spans a wave fit the LDS beside the tiles (K up to 5632), else four; more rows in further
    // launches: a row's value does not depend on the rows beside it
    const int per = need(8) <= RS_DYN ? 8 : 4;
    for (int r0 = 0; r0 < m; r0 += per) {
        const int mm = m - r0 < per ? m - r0 : per;
        const void* xp = XF32 ? (const void*)((const float*)x + (int64_t)r0 * xs) : (const void*)((const uint16_t*)x + (int64_t)r0 * xs);
        float* yp = y + (int64_t)r0 * n;
        if (mm <= 1) RSK(1);
        else if (mm <= 2) RSK(2);
        else if (mm <= 4) RSK(4);
        else RSK(8);
    }
#undef RSK
    return launch_status();
}

}  // namespace

// ================================================================ C ABI: the reference's symbols (engine-rs/shim/fp8.cu:110-178)
// x binary32 [m, k], rounded to binary16 inside; w E4M3 [n, k]; scales binary32 [n]; y binary32 [m, n] (rounded: each output rounded to
// binary16).  m 1..16, n and k multiples of 64, else 1 (the reference's cudaErrorInvalidValue).  scratch, mode and split_override
// choose among the reference's kernels (its split-K forms need the scratch): one kernel family here, K split by the shape, so they
// are accepted and ignored.
SPARK_API int glm53_fp8_dense_cuda(const float* x, const void* w, const float* scales, float* y, float* scratch, int m, int n, int k, int rounded, int mode,
                                   int split_override, hipStream_t st)
{
    (void)scratch; (void)mode; (void)split_override;
    if (m < 1 || m > 16 || n % 64 || k % 64 || n < 64 || k < 64) return (int)hipErrorInvalidValue;
    return rowscale_launch<true, true>(x, k, w, scales, y, m, n, k, rounded != 0, st);
}
// the same with the activations rounded to bf16 and no output rounding; splits (1, 2, 4, 8 or 16: the reference's K split) is
// checked and otherwise ignored
SPARK_API int glm53_fp8_bf16_cuda(const float* x, const void* w, const float* scales, float* y, float* scratch, int m, int n, int k, int splits, hipStream_t st)
{
    (void)scratch;
    if (m < 1 || m > 16 || n % 64 || k % 64 || n < 64 || k < 64 || !(splits == 1 || splits == 2 || splits == 4 || splits == 8 || splits == 16)) return (int)hipErrorInvalidValue;
    return rowscale_launch<false, true>(x, k, w, scales, y, m, n, k, 0, st);
}
// bf16 activations read as they are, 2..32 rows, n a multiple of 16 (reference fp8.cu:133-141)
SPARK_API int glm53_fp8_bf16_skinny_cuda(const void* x_bf16, const void* w, const float* scales, float* y, int m, int n, int k, hipStream_t st)
{
    if (m < 2 || m > 32 || n % 16 || k % 64 || n < 16 || k < 64) return (int)hipErrorInvalidValue;
    return rowscale_launch<false, false>(x_bf16, k, w, scales, y, m, n, k, 0, st);
}
