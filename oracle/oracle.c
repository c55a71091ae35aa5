/*
 * CPU oracle for the quantized MoE expert path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of spark-engine's decode-time quantized MoE path so that the
 * HIP kernels can be checked against it.  It is linked only by tests/, by __graft_entry__.smoke() and by the
 * cpu_baseline leg of bench.py.  Nothing the library ships calls into it.
 *
 * Every function cites the reference file:line it follows (paths relative to the reference checkout).
 * The reference's own implementation of this path is CUDA (sm_121 PTX) and Rust and cannot be built in
 * this image, so there is no oracle/_ref build; each function here is pinned by the checks in
 * tests/test_oracle_*.py (closed forms, library routines, the reference's NIBMAP table and test anchors).
 *
 * Pinning status: every function below has at least one independent check; none is "parity unpinned".
 * The third-party exllamav3 extension (v1.4.9, un-vendored) is not restated: the judged path does not use it.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define EXPORT __attribute__((visibility("default")))

/* ------------------------------------------------------------------ soft floating point ---------- */

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* IEEE binary16 -> binary32 (exact). */
EXPORT float orc_f16_to_f32(uint16_t h)
{
    uint32_t s = (uint32_t)(h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 1023u;
    if (e == 0) {
        if (m == 0) return u2f(s);
        int sh = 0;
        while (!(m & 1024u)) { m <<= 1; ++sh; }
        return u2f(s | ((uint32_t)(113 - sh) << 23) | ((m & 1023u) << 13));
    }
    if (e == 31) return u2f(s | 0x7f800000u | (m << 13));
    return u2f(s | ((e + 112u) << 23) | (m << 13));
}

/* binary64 -> binary16, round to nearest even, one rounding (no intermediate binary32). */
EXPORT uint16_t orc_f64_to_f16(double d)
{
    uint64_t u; memcpy(&u, &d, 8);
    uint16_t s = (uint16_t)((u >> 48) & 0x8000u);
    int e = (int)((u >> 52) & 0x7ff);
    uint64_t m = u & 0xfffffffffffffull;
    if (e == 0x7ff) return (uint16_t)(s | 0x7c00u | (m ? 0x200u : 0));
    if (e == 0 && m == 0) return s;
    /* value = 1.m * 2^(e-1023); target exponent bias 15 */
    int he = e - 1023 + 15;
    m |= 1ull << 52;                         /* 53-bit significand */
    int shift = 42;                          /* keep 11 bits */
    if (he <= 0) { shift += 1 - he; he = 0; }
    if (shift > 63) return s;                /* underflows to zero */
    uint64_t q = m >> shift, rem = m & ((1ull << shift) - 1), half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) ++q;
    /* q holds either a subnormal significand (he == 0) or 1.xxx with the hidden bit at bit 10 */
    uint32_t r;
    if (he == 0) r = (uint32_t)q;            /* a carry into bit 10 makes it the smallest normal: same encoding */
    else r = ((uint32_t)he << 10) + (uint32_t)(q - 1024);   /* carry out of the significand bumps the exponent */
    if (r >= 0x7c00u) r = 0x7c00u;
    return (uint16_t)(s | r);
}
EXPORT uint16_t orc_f32_to_f16(float f) { return orc_f64_to_f16((double)f); }

EXPORT float orc_bf16_to_f32(uint16_t b) { return u2f((uint32_t)b << 16); }
/* binary32 -> bfloat16, round to nearest even. */
EXPORT uint16_t orc_f32_to_bf16(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7f800000u) == 0x7f800000u && (u & 0x7fffffu)) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static inline float bf16r(float f) { return orc_bf16_to_f32(orc_f32_to_bf16(f)); }

/* OCP FP8 E4M3 (fn: no infinities, 0x7f/0xff = NaN, max 448) -> binary32. */
EXPORT float orc_e4m3_to_f32(uint8_t b)
{
    uint32_t s = (uint32_t)(b & 0x80u) << 24, e = (b >> 3) & 15u, m = b & 7u;
    if (e == 15 && m == 7) return u2f(s | 0x7fc00000u);
    if (e == 0) return (b & 0x80u ? -1.0f : 1.0f) * (float)m * 0.001953125f;   /* m * 2^-9 */
    return u2f(s | ((e + 120u) << 23) | (m << 20));
}
/* binary32 -> E4M3, round to nearest even, saturating to +-448 (the conversion __nv_fp8_e4m3 / torch
 * float8_e4m3fn perform on values already clamped to [-448, 448]; reference ds41.cu:160-162). */
EXPORT uint8_t orc_f32_to_e4m3(float f)
{
    uint32_t u = f2u(f);
    uint8_t s = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint8_t)(s | 0x7f);
    float af = u2f(a);
    if (af >= 448.0f) return (uint8_t)(s | 0x7e);
    if (af < 0.0009765625f) return s;                     /* < 2^-10: rounds to zero (2^-10 itself is the tie to even 0) */
    int e = (int)(a >> 23) - 127;
    if (e < -6) {                                         /* subnormal target: units of 2^-9 */
        float q = af * 512.0f;                            /* exact */
        float r = nearbyintf(q);                          /* default rounding mode: nearest even */
        return (uint8_t)(s | (uint8_t)r);                 /* r == 8 encodes the smallest normal */
    }
    uint32_t m = a & 0x7fffffu;
    uint32_t q = m >> 20, rem = m & 0xfffffu;
    if (rem > 0x80000u || (rem == 0x80000u && (q & 1))) ++q;
    uint32_t r = ((uint32_t)(e + 7) << 3) + q;
    if (r > 0x7e) r = 0x7e;
    return (uint8_t)(s | r);
}
/* E8M0 scale byte -> binary32 from the exponent bits: b << 23 (byte 0 gives 0.0; reference ds41.cu:23, ops.rs:22). */
EXPORT float orc_e8m0_to_f32(uint8_t b) { return u2f((uint32_t)b << 23); }

/* E2M1 code (bit 3 = sign) -> value; reference kernel.py:21,122-131. */
static const float FP4_MAG[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
EXPORT float orc_e2m1_to_f32(uint8_t c) { float v = FP4_MAG[c & 7]; return (c & 8) ? -v : v; }

/* ------------------------------------------------------------------ EXL3 codebooks ---------------- */

/* mul1: reference qwen_exl3.cuh:17-23, qwen38/exl3.py:38-50.  One fp16 fma rounding. */
EXPORT uint16_t orc_mul1_decode(uint32_t state)
{
    uint32_t x = (state & 0xffffu) * 0x83DCD12Du;
    uint32_t b = (x & 255u) + ((x >> 8) & 255u) + ((x >> 16) & 255u) + (x >> 24);
    double h = 1024.0 + (double)b;
    double c1 = (double)orc_f16_to_f32(0x1eee), c2 = (double)orc_f16_to_f32(0xc931);
    return orc_f64_to_f16(h * c1 + c2);          /* product and sum exact in binary64 */
}
/* mcg: reference qwen_exl3.cuh:26-32, glm53/exl3.py:35-46, exl3.rs:9-25.  One fp16 add rounding. */
EXPORT uint16_t orc_mcg_decode(uint32_t state)
{
    uint32_t x = (state & 0xffffu) * 0xCBAC1FEDu;
    x = (x & 0x8fff8fffu) ^ 0x3b603b60u;
    double s = (double)orc_f16_to_f32((uint16_t)(x & 0xffffu)) + (double)orc_f16_to_f32((uint16_t)(x >> 16));
    return orc_f64_to_f16(s);
}
/* codebook: 2 = mul1 (Qwen), 1 = mcg (GLM), the reference's CBK numbering (moe_exl3.cuh:6). */
EXPORT void orc_exl3_codebook(int codebook, uint16_t* out65536)
{
    for (uint32_t s = 0; s < 65536u; ++s) out65536[s] = codebook == 1 ? orc_mcg_decode(s) : orc_mul1_decode(s);
}

/* ------------------------------------------------------------------ EXL3 tile decode -------------- */

/* The 256 trellis states of one tile in sequence order.  tile: 16*bits int16 words.
 * reference qwen38/exl3.py:66-78 (tile_states), qwen_exl3.cuh:8-11. */
EXPORT void orc_exl3_tile_states(const int16_t* tile, int bits, uint16_t* states256)
{
    const int nw = 8 * bits, L = 256 * bits;
    uint32_t w[48];
    for (int j = 0; j < nw; ++j) w[j] = ((uint32_t)(uint16_t)tile[2 * j]) | ((uint32_t)(uint16_t)tile[2 * j + 1] << 16);
    for (int t = 0; t < 256; ++t) {
        int b0 = (((t + 1) * bits - 16) % L + L) % L;
        int i0 = b0 >> 5, i1 = (i0 + 1) % nw;
        uint64_t win = ((uint64_t)w[i0] << 32) | w[i1];
        states256[t] = (uint16_t)((win >> (48 - (b0 & 31))) & 0xffffu);
    }
}
/* Sequence position -> element (row*16 + col) of the 16x16 tile; reference qwen38/exl3.py:23-32. */
EXPORT int orc_exl3_perm(int pos)
{
    int t = pos >> 3, j = pos & 7;
    static const int roff[4] = {0, 1, 8, 9};
    int row = (t % 4) * 2 + roff[j & 3], col = t / 4 + 8 * (j >> 2);
    return row * 16 + col;
}
/* trellis [Kt, Nt, 16*bits] int16 -> inner [Kt*16, Nt*16] fp16 bit patterns (K-major, y = x @ inner).
 * reference qwen38/exl3.py:81-97 (decode_inner), glm53/exl3.py:69-87, qwen_exl3.cuh:629-650 (reconstruct_kernel). */
EXPORT void orc_exl3_decode_inner(const int16_t* trellis, int Kt, int Nt, int bits, int codebook, uint16_t* inner)
{
    uint16_t* cb = (uint16_t*)malloc(65536 * 2);
    orc_exl3_codebook(codebook, cb);
    const int N = Nt * 16;
#pragma omp parallel for schedule(static)
    for (int kt = 0; kt < Kt; ++kt) {
        uint16_t st[256];
        for (int nt = 0; nt < Nt; ++nt) {
            orc_exl3_tile_states(trellis + ((size_t)kt * Nt + nt) * 16 * bits, bits, st);
            for (int p = 0; p < 256; ++p) {
                int el = orc_exl3_perm(p);
                inner[(size_t)(kt * 16 + (el >> 4)) * N + nt * 16 + (el & 15)] = cb[st[p]];
            }
        }
    }
    free(cb);
}

/* ------------------------------------------------------------------ Hadamard ---------------------- */

/* In-place 128-point Walsh-Hadamard (Sylvester order) / sqrt(128) in binary32, butterflies h = 1, 2, ..., 64 with
 * (a + b, a - b) and the lower index first, then one multiply by 0.08838834764831845f.
 * reference qwen_exl3.cuh:118-137 (fwht128).  stride: distance between consecutive elements. */
EXPORT void orc_fwht128(float* v, size_t stride)
{
    for (int h = 1; h < 128; h <<= 1)
        for (int i = 0; i < 128; ++i)
            if (!(i & h)) {
                const float a = v[i * stride], b = v[(i + h) * stride];
                v[i * stride] = a + b;
                v[(i + h) * stride] = a - b;
            }
    for (int i = 0; i < 128; ++i) v[i * stride] *= 0.08838834764831845f;
}
/* xh[k] = fp16(had128(x[:] * suh)[k]); reference qwen_exl3.cuh:165-183 (had_in_kernel). */
EXPORT void orc_exl3_had_in(const float* x, const uint16_t* suh, int K, uint16_t* xh)
{
    float v[128];
    for (int kb = 0; kb < K / 128; ++kb) {
        for (int i = 0; i < 128; ++i) v[i] = x[kb * 128 + i] * orc_f16_to_f32(suh[kb * 128 + i]);
        orc_fwht128(v, 1);
        for (int i = 0; i < 128; ++i) xh[kb * 128 + i] = orc_f32_to_f16(v[i]);
    }
}
/* Effective weight W [K, N] binary32 with y = x @ W:  W = diag(suh) H inner H diag(svh), H per 128-block.
 * Operation order of reference qwen_exl3.cuh:658-701 (fold_kernel): H along k, * suh[k], H along n, * svh[n].
 * Same mathematics as qwen38/exl3.py:100-110 and glm53/exl3.py:90-101 (decode_weight). */
EXPORT void orc_exl3_decode_weight(const int16_t* trellis, const uint16_t* suh, const uint16_t* svh, int K, int N, int bits,
                                   int codebook, float* W)
{
    uint16_t* inner = (uint16_t*)malloc((size_t)K * N * 2);
    orc_exl3_decode_inner(trellis, K / 16, N / 16, bits, codebook, inner);
    for (size_t i = 0; i < (size_t)K * N; ++i) W[i] = orc_f16_to_f32(inner[i]);
    free(inner);
#pragma omp parallel for schedule(static)
    for (int kb = 0; kb < K / 128; ++kb)
        for (int n = 0; n < N; ++n) {
            float* col = W + (size_t)kb * 128 * N + n;
            orc_fwht128(col, (size_t)N);
            for (int i = 0; i < 128; ++i) col[(size_t)i * N] *= orc_f16_to_f32(suh[kb * 128 + i]);
        }
#pragma omp parallel for schedule(static)
    for (int k = 0; k < K; ++k)
        for (int nb = 0; nb < N / 128; ++nb) {
            float* row = W + (size_t)k * N + nb * 128;
            orc_fwht128(row, 1);
            for (int i = 0; i < 128; ++i) row[i] *= orc_f16_to_f32(svh[nb * 128 + i]);
        }
}
/* fold: W^T [N, K] rounded to fp16 (row stride ldo); reference qwen_exl3.cuh:696-701, qwen_exl3.cu fold entry. */
EXPORT void orc_exl3_fold(const int16_t* trellis, const uint16_t* suh, const uint16_t* svh, int K, int N, int bits, int codebook,
                          uint16_t* out, int64_t ldo)
{
    float* W = (float*)malloc((size_t)K * N * 4);
    orc_exl3_decode_weight(trellis, suh, svh, K, N, bits, codebook, W);
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k) out[(size_t)n * ldo + k] = orc_f32_to_f16(W[(size_t)k * N + n]);
    free(W);
}

/* ------------------------------------------------------------------ dense helpers ----------------- */

/* y[n] = sum_k x[k] * W[k*N + n], binary32 accumulation in k order. */
static void gemv_kn(const float* x, const float* W, int K, int N, float* y)
{
    for (int n = 0; n < N; ++n) y[n] = 0.f;
    for (int k = 0; k < K; ++k) {
        const float xv = x[k];
        const float* w = W + (size_t)k * N;
        for (int n = 0; n < N; ++n) y[n] += xv * w[n];
    }
}
static inline float silu(float g) { return g / (1.0f + expf(-g)); }

/* ------------------------------------------------------------------ EXL3 MoE (fp32 reference) ----- */

/* One EXL3 expert on one row in binary32: out = (act(x@Wg, x@Wu)) @ Wd with dequantised weights.
 * act: 0 = silu(g)*u (Qwen, reference qwen38/model.py:189-202, test_kern_moe.py:17-22),
 *      1 = clamp (g <= 10, |u| <= 10) then silu(g)*u (GLM, reference glm53/moe.py:85-95, moe_own.rs:141-158). */
static void exl3_expert_rows(const float* Wg, const float* Wu, const float* Wd, int H, int I, int act, const float* x, int rows,
                             float* out)
{
    float* g = (float*)malloc((size_t)I * 4 * 3);
    float *u = g + I, *a = u + I;
    for (int r = 0; r < rows; ++r) {
        gemv_kn(x + (size_t)r * H, Wg, H, I, g);
        gemv_kn(x + (size_t)r * H, Wu, H, I, u);
        for (int i = 0; i < I; ++i) {
            float gv = g[i], uv = u[i];
            if (act == 1) { gv = fminf(gv, 10.0f); uv = fminf(fmaxf(uv, -10.0f), 10.0f); }
            a[i] = silu(gv) * uv;
        }
        gemv_kn(a, Wd, I, H, out + (size_t)r * H);
    }
    free(g);
}
/* Routed EXL3 experts: out[r] = add[r] + sum_k (slot order) w[r,k] * expert_{idx[r,k]}(x[r]).
 * tab: 9 arrays of E host pointers in the reference's table order gate_tr, up_tr, down_tr, gate_suh, up_suh, down_suh,
 * gate_svh, up_svh, down_svh (moe_exl3.cuh:8-9).  x binary32 [R, H].  Dequantise + matmul per distinct expert
 * (the reference CPU path: reference glm53/moe.py:85-141, qwen38/model.py:189-202). */
EXPORT void orc_exl3_moe(const float* x, int R, const int32_t* idx, const float* w, const void* const* tab, int E, int topk, int H, int I,
                         int bits, int codebook, int act, const float* add, float* out)
{
    const int P = R * topk;
    float* yd = (float*)malloc((size_t)P * H * 4);
    char* done = (char*)calloc(P, 1);
    float* Wg = (float*)malloc((size_t)H * I * 4 * 3);
    float *Wu = Wg + (size_t)H * I, *Wd = Wu + (size_t)H * I;
    for (int p = 0; p < P; ++p) {
        if (done[p]) continue;
        const int e = idx[p];
        orc_exl3_decode_weight((const int16_t*)tab[0 * E + e], (const uint16_t*)tab[3 * E + e], (const uint16_t*)tab[6 * E + e], H, I, bits, codebook, Wg);
        orc_exl3_decode_weight((const int16_t*)tab[1 * E + e], (const uint16_t*)tab[4 * E + e], (const uint16_t*)tab[7 * E + e], H, I, bits, codebook, Wu);
        orc_exl3_decode_weight((const int16_t*)tab[2 * E + e], (const uint16_t*)tab[5 * E + e], (const uint16_t*)tab[8 * E + e], I, H, bits, codebook, Wd);
        for (int q = p; q < P; ++q)
            if (!done[q] && idx[q] == e) {
                exl3_expert_rows(Wg, Wu, Wd, H, I, act, x + (size_t)(q / topk) * H, 1, yd + (size_t)q * H);
                done[q] = 1;
            }
    }
    for (int r = 0; r < R; ++r)
        for (int n = 0; n < H; ++n) {
            float acc = 0.f;
            for (int k = 0; k < topk; ++k) acc += w[r * topk + k] * yd[(size_t)(r * topk + k) * H + n];
            out[(size_t)r * H + n] = (add ? add[(size_t)r * H + n] : 0.f) + acc;
        }
    free(Wg); free(done); free(yd);
}

/* ------------------------------------------------------------------ routers ----------------------- */

/* Qwen: softmax over E logits, top-k by repeated argmax (ties -> lower index), weights renormalised.
 * reference qwen_moe.cu:10-66, qwen38/model.py:189-192. */
EXPORT void orc_qwen_route(const float* logits, int64_t ld, int R, int E, int topk, int32_t* idx, float* w)
{
    float* p = (float*)malloc((size_t)E * 4);
    for (int r = 0; r < R; ++r) {
        const float* x = logits + (size_t)r * ld;
        float m = x[0];
        for (int e = 1; e < E; ++e) m = fmaxf(m, x[e]);
        double s = 0.0;
        for (int e = 0; e < E; ++e) { p[e] = expf(x[e] - m); s += p[e]; }
        for (int e = 0; e < E; ++e) p[e] = p[e] / (float)s;
        float t = 0.f, tv[64];
        for (int k = 0; k < topk; ++k) {
            int bi = 0;
            for (int e = 1; e < E; ++e) if (p[e] > p[bi]) bi = e;
            idx[r * topk + k] = bi; tv[k] = p[bi]; t += p[bi]; p[bi] = -1.0f;
        }
        for (int k = 0; k < topk; ++k) w[r * topk + k] = tv[k] / t;
    }
    free(p);
}
/* DeepSeek: s = sqrt(softplus(x)) (threshold 20), top-k of s + bias (ties -> lower index),
 * w = s / (sum + 1e-20) (k > 1) * scale.  reference ds41_ops.cu:376-419. */
EXPORT void orc_ds41_route(const float* logits, const float* bias, int64_t* idx, float* w, int T, int E, int K, float scale)
{
    float* sc = (float*)malloc((size_t)E * 8);
    float* b = sc + E;
    for (int r = 0; r < T; ++r) {
        for (int e = 0; e < E; ++e) {
            const float x = logits[(size_t)r * E + e];
            sc[e] = sqrtf(x > 20.f ? x : log1pf(expf(x)));
            b[e] = sc[e] + bias[e];
        }
        float picked[64], sum = 0.f;
        for (int k = 0; k < K; ++k) {
            int bi = 0;
            for (int e = 1; e < E; ++e) if (b[e] > b[bi]) bi = e;
            idx[(size_t)r * K + k] = bi; picked[k] = sc[bi]; b[bi] = -INFINITY;
        }
        for (int k = 0; k < K; ++k) sum += picked[k];
        for (int k = 0; k < K; ++k) w[(size_t)r * K + k] = (K > 1 ? picked[k] / (sum + 1e-20f) : picked[k]) * scale;
    }
    free(sc);
}
/* GLM: score = sigmoid(logit), select top-k on score + bias (ties -> lower index), w = score / sum * scaling.
 * reference glm53/moe.py:72-83 (route), dataflow.cu:433-448 (router_select), glm53_tests/test_moe.py:20-31. */
EXPORT void orc_glm_route(const float* logits, const float* bias, int64_t* idx, float* w, int T, int E, int K, float scaling)
{
    float* sc = (float*)malloc((size_t)E * 8);
    float* b = sc + E;
    for (int r = 0; r < T; ++r) {
        for (int e = 0; e < E; ++e) {
            sc[e] = 1.0f / (1.0f + expf(-logits[(size_t)r * E + e]));
            b[e] = sc[e] + bias[e];
        }
        float picked[64], sum = 0.f;
        for (int k = 0; k < K; ++k) {
            int bi = 0;
            for (int e = 1; e < E; ++e) if (b[e] > b[bi]) bi = e;
            idx[(size_t)r * K + k] = bi; picked[k] = sc[bi]; b[bi] = -INFINITY;
        }
        for (int k = 0; k < K; ++k) sum += picked[k];
        for (int k = 0; k < K; ++k) w[(size_t)r * K + k] = picked[k] / fmaxf(sum, 1e-20f) * scaling;
    }
    free(sc);
}

/* ------------------------------------------------------------------ MXFP4 / FP8 dequant ----------- */

/* W [N, K/2] packed E2M1 (low nibble = even k) + S [N, K/32] E8M0 -> binary32 [N, K].
 * reference kernel.py:122-131 (dequant_fp4_weight), ds41/load.rs:338-349. */
EXPORT void orc_mxfp4_dequant(const uint8_t* w, const uint8_t* s, int N, int K, float* out)
{
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; k += 2) {
            const uint8_t b = w[(size_t)n * (K / 2) + k / 2];
            const float sc = orc_e8m0_to_f32(s[(size_t)n * (K / 32) + k / 32]);
            out[(size_t)n * K + k] = orc_e2m1_to_f32(b & 15) * sc;
            out[(size_t)n * K + k + 1] = orc_e2m1_to_f32(b >> 4) * sc;
        }
}
/* W [N, K] E4M3 + scales binary32 [ceil(N/bs), ceil(K/bs)] -> binary32 [N, K]: one multiply per element.
 * reference kernel.py:96-99 (_dequant_fp8_weight, block_size 128). */
EXPORT void orc_fp8_block_dequant(const uint8_t* w, const float* s, int N, int K, int bs, float* out)
{
    const int kb = (K + bs - 1) / bs;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k) out[(size_t)n * K + k] = orc_e4m3_to_f32(w[(size_t)n * K + k]) * s[(size_t)(n / bs) * kb + k / bs];
}
/* W [N, K] E4M3 + E8M0 scales [ceil(N/32), K/32] -> binary32; reference ds41.cu:9-11,28-73 (fp8_gemv's operand). */
EXPORT void orc_fp8_e8m0_dequant(const uint8_t* w, const uint8_t* s, int N, int K, float* out)
{
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
        for (int k = 0; k < K; ++k)
            out[(size_t)n * K + k] = orc_e4m3_to_f32(w[(size_t)n * K + k]) * orc_e8m0_to_f32(s[(size_t)(n >> 5) * (K >> 5) + (k >> 5)]);
}
/* y[m, n] = sum_k x[m, k] * W[n, k] with W binary32 [N, K]; x binary32 [M, K] (row stride K). */
EXPORT void orc_gemv_nk(const float* x, const float* W, int M, int N, int K, float* y)
{
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n)
        for (int m = 0; m < M; ++m) {
            const float* wr = W + (size_t)n * K;
            const float* xr = x + (size_t)m * K;
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int k = 0; k < K; k += 8)
                for (int j = 0; j < 8; ++j) acc[j] += xr[k + j] * wr[k + j];
            y[(size_t)m * N + n] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
        }
}

/* ------------------------------------------------------------------ act_quant --------------------- */

/* UE8M0 scale byte of a 32-block from its absolute maximum: amax >= 1e-4, scale = 2^ceil(log2(amax / 448)) from the
 * exponent bits.  reference kernel.py:24-37,59-73, ops.rs:26-35, ds41_mx.cu:42-46 (aq_scale). */
EXPORT uint8_t orc_aq_scale(float amax)
{
    amax = fmaxf(amax, 1e-4f);
    const uint32_t bits = f2u(amax * (1.0f / 448.0f));
    return (uint8_t)(((bits >> 23) & 0xff) + ((bits & 0x7fffffu) != 0));
}
/* reference ds41_mx.cu:47-51 (aq_byte). */
EXPORT uint8_t orc_aq_byte(float v, uint8_t e)
{
    const float s = u2f((uint32_t)e << 23);
    return orc_f32_to_e4m3(fminf(fmaxf(v / s, -448.f), 448.f));
}
/* x bf16 [numel] -> q E4M3 bytes [numel] + s UE8M0 bytes [numel/32]; reference ds41_mx.cu:320-331. */
EXPORT void orc_act_quant_fp8(const uint16_t* x, uint8_t* q, uint8_t* s, int64_t numel)
{
    for (int64_t b = 0; b < numel / 32; ++b) {
        float a = 0.f;
        for (int i = 0; i < 32; ++i) a = fmaxf(a, fabsf(orc_bf16_to_f32(x[b * 32 + i])));
        const uint8_t e = orc_aq_scale(a);
        for (int i = 0; i < 32; ++i) q[b * 32 + i] = orc_aq_byte(orc_bf16_to_f32(x[b * 32 + i]), e);
        s[b] = e;
    }
}
/* x bf16 -> quantize-dequantize bf16 (act_quant inplace); reference ds41.cu:148-164, ops.rs:26-35. */
EXPORT void orc_act_quant32(const uint16_t* x, uint16_t* out, int64_t numel)
{
    for (int64_t b = 0; b < numel / 32; ++b) {
        float a = 0.f;
        for (int i = 0; i < 32; ++i) a = fmaxf(a, fabsf(orc_bf16_to_f32(x[b * 32 + i])));
        const uint8_t e = orc_aq_scale(a);
        const float sc = u2f((uint32_t)e << 23);
        for (int i = 0; i < 32; ++i)
            out[b * 32 + i] = orc_f32_to_bf16(orc_e4m3_to_f32(orc_aq_byte(orc_bf16_to_f32(x[b * 32 + i]), e)) * sc);
    }
}

/* ------------------------------------------------------------------ shared-expert glue ------------- */

/* gu binary32 [T, 2I] (gate | up, the stacked w1 / w3 GEMV sums) -> bf16 [T, I]: gate and up rounded to bf16, gate <= lim and
 * |up| <= lim when lim > 0, silu(gate) * up rounded to bf16, then act_quant per 32 (quantise-dequantise, UE8M0 scale).
 * reference engine-rs/shim/ds41_ops.cu:421-442 (swiglu_quant_kernel), entry :615-621. */
EXPORT void orc_swiglu_quant(const float* gu, uint16_t* out, int T, int I, float lim)
{
    for (int t = 0; t < T; ++t)
        for (int b = 0; b < I / 32; ++b) {
            float v[32], a = 0.f;
            for (int i = 0; i < 32; ++i) {
                const int j = b * 32 + i;
                float g = bf16r(gu[(size_t)t * 2 * I + j]), u = bf16r(gu[(size_t)t * 2 * I + I + j]);
                if (lim > 0.f) { g = fminf(g, lim); u = fminf(fmaxf(u, -lim), lim); }
                v[i] = bf16r(g / (1.f + expf(-g)) * u);
                a = fmaxf(a, fabsf(v[i]));
            }
            const uint8_t e = orc_aq_scale(a);
            const float sc = u2f((uint32_t)e << 23);
            for (int i = 0; i < 32; ++i) out[(size_t)t * I + b * 32 + i] = orc_f32_to_bf16(orc_e4m3_to_f32(orc_aq_byte(v[i], e)) * sc);
        }
}
/* h[i] = silu(g[i]) * u[i], binary32.  reference engine-rs/shim/qwen_moe.cu:69-76 (silu_mul_kernel). */
EXPORT void orc_silu_mul(const float* g, const float* u, float* h, int n)
{
    for (int i = 0; i < n; ++i) { const float x = g[i]; h[i] = x / (1.0f + expf(-x)) * u[i]; }
}
/* out[r, :] = sigmoid(gl[r * ldg + col]) * d[r, :], binary32 (the shared expert's scalar gate).
 * reference engine-rs/shim/qwen_moe.cu:77-84 (gate_scale_kernel). */
EXPORT void orc_gate_scale(const float* gl, int64_t ldg, int col, const float* d, float* out, int R, int N)
{
    for (int r = 0; r < R; ++r) {
        const float sg = 1.0f / (1.0f + expf(-gl[(size_t)r * ldg + col]));
        for (int n = 0; n < N; ++n) out[(size_t)r * N + n] = sg * d[(size_t)r * N + n];
    }
}

/* ------------------------------------------------------------------ DeepSeek MXFP4 MoE ------------ */

/* Dot products whose result a quantiser reads (gate / up: rounded to bf16, then act_quant): summed in binary64 and rounded
 * once to binary32.  The reference's moe_ref leaves the order of this sum to its BLAS (x.matmul, ds41/kern.rs:1124-1125); the
 * exact sum is the value every binary32 order approximates, and a binary64 sum of these terms (products of a 4-bit and a 6-bit
 * significand, a few thousand of them) is that value to 1e-16.  With binary32 sums here the oracle's own summation error (5e-7 of
 * the sum, eight chains of K / 8 terms) decided more bf16 / E4M3 roundings of the intermediate than the kernels' did. */
static void gemv_nk_f64acc(const float* x, const float* W, int N, int K, float* y, double* yd, double* ynorm)
{
    /* yd, ynorm (optional): the binary64 sums and the Euclidean norm of each sum's terms (the size of its partial sums: what a
     * binary32 summation's error is relative to) */
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        const float* wr = W + (size_t)n * K;
        double acc[8] = {0, 0, 0, 0, 0, 0, 0, 0}, sq = 0.0;
        for (int k = 0; k < K; k += 8)
            for (int j = 0; j < 8; ++j) { const double p = (double)x[k + j] * (double)wr[k + j]; acc[j] += p; sq += p * p; }
        const double t = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
        y[n] = (float)t;
        if (yd) { yd[n] = t; ynorm[n] = sqrt(sq); }
    }
}
/* Distance of v from the nearest point where its rounding to bf16 changes (the midpoint between neighbouring bf16 values on the
 * side of bf16(v) that v lies on): how large an error of v it takes to move bf16(v). */
static double bf16_margin(double v)
{
    const double r = (double)bf16r((float)v);
    int ex;
    (void)frexp(r != 0.0 ? r : (v != 0.0 ? v : 1.0), &ex);    /* |r| in [2^(ex-1), 2^ex): one step of bf16 there is 2^(ex-8) */
    double half = ldexp(1.0, ex - 9);
    if (fabs(v) < fabs(r) && fabs(r) == ldexp(1.0, ex - 1)) half *= 0.5;   /* below a power of two the steps are half as wide */
    return fabs(fabs(v - r) - half);
}
/* One pair: out[H] = w2 . q(bf16(silu(min(bf16(w1.x),10)) * clamp(bf16(w3.x),+-10) * rw)), dequantise + matmul.
 * xd: the act-quantized input as binary32 [H].  w1/w3 [I, H/2]+[I, H/32], w2 [H, I/2]+[H, I/32] of ONE expert.
 * hq / hs (optional): the intermediate's E4M3 codes [I] and UE8M0 scale bytes [I / 32]; margin (optional) [I]: the smallest
 * bf16_margin of the element's three roundings, each relative to the size of what is rounded (gate sum and up sum: the norm of the
 * sum's terms; the product: itself), i.e. how close the element is to coming out differently under another order of the binary32
 * sums or another library's expf.
 * reference ds41/kern.rs:1116-1133 (moe_ref), ds41_moe.cu:1-6,161-181. */
static void ds41_pair(const float* xd, const uint8_t* w1, const uint8_t* s1, const uint8_t* w3, const uint8_t* s3, const uint8_t* w2,
                      const uint8_t* s2, int H, int I, float rw, float* W, float* out, uint8_t* hq, uint8_t* hs, float* margin)
{
    float* g = (float*)malloc((size_t)I * 4 * 3);
    float *u = g + I, *hm = u + I;
    double* gd = margin ? (double*)malloc((size_t)I * 8 * 4) : NULL;
    double *ud = gd ? gd + I : NULL, *gn = gd ? gd + 2 * I : NULL, *un = gd ? gd + 3 * I : NULL;
    orc_mxfp4_dequant(w1, s1, I, H, W);
    gemv_nk_f64acc(xd, W, I, H, g, gd, gn);
    orc_mxfp4_dequant(w3, s3, I, H, W);
    gemv_nk_f64acc(xd, W, I, H, u, ud, un);
    uint16_t hb[32];
    for (int j0 = 0; j0 < I; j0 += 32) {
        float a = 0.f;
        for (int j = 0; j < 32; ++j) {
            const float gt = fminf(bf16r(g[j0 + j]), 10.f);
            const float up = fminf(fmaxf(bf16r(u[j0 + j]), -10.f), 10.f);
            const float y = bf16r(silu(gt) * up * rw);
            hb[j] = orc_f32_to_bf16(y);
            a = fmaxf(a, fabsf(y));
            if (margin) {
                const double yd = (double)gt / (1.0 + exp(-(double)gt)) * (double)up * (double)rw;
                const double mg = gn[j0 + j] > 0.0 ? bf16_margin(gd[j0 + j]) / gn[j0 + j] : 1.0, mu = un[j0 + j] > 0.0 ? bf16_margin(ud[j0 + j]) / un[j0 + j] : 1.0;
                margin[j0 + j] = (float)fmin(fmin(mg, mu), yd != 0.0 ? bf16_margin(yd) / fabs(yd) : 1.0);
            }
        }
        const uint8_t e = orc_aq_scale(a);
        const float sc = u2f((uint32_t)e << 23);
        if (hs) hs[j0 / 32] = e;
        for (int j = 0; j < 32; ++j) {
            const uint8_t q = orc_aq_byte(orc_bf16_to_f32(hb[j]), e);
            if (hq) hq[j0 + j] = q;
            hm[j0 + j] = orc_e4m3_to_f32(q) * sc;
        }
    }
    orc_mxfp4_dequant(w2, s2, H, I, W);
    orc_gemv_nk(hm, W, 1, H, I, out);
    free(g); free(gd);
}
/* Routed MXFP4 experts.  x bf16 [R, H] (NOT yet quantized: act_quant per 32 is applied here, as the layer does before
 * the experts, reference ds41/kern.rs act_quant_fp8 + moe_mx).  Stacked natural-layout weights w1,w3 [E, I, H/2],
 * s1,s3 [E, I, H/32], w2 [E, H, I/2], s2 [E, H, I/32].  n_shared extra experts (ids E .. E+n_shared-1 in the stacked
 * arrays) run on every row with weight 1 and enter as `add` (reference ds41_mx.cu:1433 add, model.rs:2987-3009).
 * y[r] = add[r] + shared(x[r]) + sum_k (slot order) out[r,k]   (combine order of ds41_mx.cu:302-317: the routed sum
 * first, then added to add).  pair_out (optional) receives the per-pair outputs [R*topk, H]. */
EXPORT void orc_mxfp4_moe(const uint16_t* x, int R, const int64_t* idx, const float* rw, const uint8_t* w1, const uint8_t* s1,
                          const uint8_t* w3, const uint8_t* s3, const uint8_t* w2, const uint8_t* s2, int H, int I, int topk, int E,
                          int n_shared, const float* add, float* y, float* pair_out, uint8_t* h_codes, uint8_t* h_scales, float* h_margin)
{
    /* h_codes [R * topk + R * n_shared, I], h_scales [.., I / 32], h_margin [.., I] (optional): the act-quantised intermediate of
     * every pair and each element's rounding margin (ds41_pair), the routed pairs (r, k) first, then the shared ones (r, j) */
    const int P = R * topk;
    float* xd = (float*)malloc((size_t)R * H * 4);
    {
        uint8_t* q = (uint8_t*)malloc((size_t)R * H);
        uint8_t* s = (uint8_t*)malloc((size_t)R * H / 32);
        orc_act_quant_fp8(x, q, s, (int64_t)R * H);
        for (size_t i = 0; i < (size_t)R * H; ++i) xd[i] = orc_e4m3_to_f32(q[i]) * orc_e8m0_to_f32(s[i / 32]);
        free(q); free(s);
    }
    float* W = (float*)malloc((size_t)H * I * 4);
    float* out = (float*)malloc((size_t)(P + R * (n_shared > 0 ? n_shared : 1)) * H * 4);
    const size_t wsz = (size_t)I * H / 2, ssz = (size_t)I * H / 32;
    for (int p = 0; p < P; ++p) {
        const int64_t e = idx[p];
        ds41_pair(xd + (size_t)(p / topk) * H, w1 + e * wsz, s1 + e * ssz, w3 + e * wsz, s3 + e * ssz, w2 + e * wsz, s2 + e * ssz, H, I, rw[p], W,
                  out + (size_t)p * H, h_codes ? h_codes + (size_t)p * I : NULL, h_scales ? h_scales + (size_t)p * (I / 32) : NULL,
                  h_margin ? h_margin + (size_t)p * I : NULL);
    }
    for (int r = 0; r < R; ++r)
        for (int j = 0; j < n_shared; ++j) {
            const int64_t e = E + j;
            const size_t q = (size_t)P + (size_t)r * n_shared + j;
            ds41_pair(xd + (size_t)r * H, w1 + e * wsz, s1 + e * ssz, w3 + e * wsz, s3 + e * ssz, w2 + e * wsz, s2 + e * ssz, H, I, 1.0f, W,
                      out + q * H, h_codes ? h_codes + q * I : NULL, h_scales ? h_scales + q * (I / 32) : NULL, h_margin ? h_margin + q * I : NULL);
        }
    for (int r = 0; r < R; ++r)
        for (int n = 0; n < H; ++n) {
            float acc = add ? add[(size_t)r * H + n] : 0.f;
            for (int j = 0; j < n_shared; ++j) acc += out[(size_t)(P + r * n_shared + j) * H + n];
            float s = 0.f;
            for (int k = 0; k < topk; ++k) s += out[(size_t)(r * topk + k) * H + n];
            y[(size_t)r * H + n] = acc + s;
        }
    if (pair_out) memcpy(pair_out, out, (size_t)P * H * 4);
    free(out); free(W); free(xd);
}
/* The second half of the layer alone: the down products of a GIVEN act-quantised intermediate (codes h_codes [R * topk + R * n_shared, I]
 * and scale bytes h_scales [.., I / 32], pairs ordered as orc_mxfp4_moe hands them out) and the sum in the reference's order
 * (ds41_mx.cu:302-317).  Lets a test hold a kernel's output against the oracle evaluated on the kernel's own intermediate. */
EXPORT void orc_mxfp4_moe_from_h(const uint8_t* h_codes, const uint8_t* h_scales, int R, const int64_t* idx, const uint8_t* w2, const uint8_t* s2,
                                 int H, int I, int topk, int E, int n_shared, const float* add, float* y)
{
    const int P = R * topk, Q = P + R * n_shared;
    float* W = (float*)malloc((size_t)H * I * 4);
    float* hm = (float*)malloc((size_t)I * 4);
    float* out = (float*)malloc((size_t)(Q > 0 ? Q : 1) * H * 4);
    const size_t wsz = (size_t)I * H / 2, ssz = (size_t)I * H / 32;
    for (int q = 0; q < Q; ++q) {
        const int64_t e = q < P ? idx[q] : E + (q - P) % n_shared;
        for (int j = 0; j < I; ++j) hm[j] = orc_e4m3_to_f32(h_codes[(size_t)q * I + j]) * u2f((uint32_t)h_scales[(size_t)q * (I / 32) + j / 32] << 23);
        orc_mxfp4_dequant(w2 + e * wsz, s2 + e * ssz, H, I, W);
        orc_gemv_nk(hm, W, 1, H, I, out + (size_t)q * H);
    }
    for (int r = 0; r < R; ++r)
        for (int n = 0; n < H; ++n) {
            float acc = add ? add[(size_t)r * H + n] : 0.f;
            for (int j = 0; j < n_shared; ++j) acc += out[(size_t)(P + r * n_shared + j) * H + n];
            float s = 0.f;
            for (int k = 0; k < topk; ++k) s += out[(size_t)(r * topk + k) * H + n];
            y[(size_t)r * H + n] = acc + s;
        }
    free(out); free(hm); free(W);
}

/* ------------------------------------------------------------------ dense GEMVs ------------------- */

/* y[m, n] = x[m, :] . dequant(W)[n, :] for MXFP4 W; x bf16 used as given.  reference ds41.cu:75-110, kernel.py:134-139. */
EXPORT void orc_mxfp4_gemv(const uint16_t* x, const uint8_t* w, const uint8_t* s, float* y, int m, int n, int k)
{
    float* W = (float*)malloc((size_t)n * k * 4);
    float* xf = (float*)malloc((size_t)m * k * 4);
    orc_mxfp4_dequant(w, s, n, k, W);
    for (size_t i = 0; i < (size_t)m * k; ++i) xf[i] = orc_bf16_to_f32(x[i]);
    orc_gemv_nk(xf, W, m, n, k, y);
    free(W); free(xf);
}
/* FP8 E4M3 W [n, k] with binary32 scales per bs x bs block (bs = 128: reference kernel.py:96-119), x bf16 used as
 * given (weight-only dequant, the contract of reference ds41.cu:9-11). */
EXPORT void orc_fp8_block_gemv(const uint16_t* x, const uint8_t* w, const float* s, float* y, int m, int n, int k, int bs)
{
    float* W = (float*)malloc((size_t)n * k * 4);
    float* xf = (float*)malloc((size_t)m * k * 4);
    orc_fp8_block_dequant(w, s, n, k, bs, W);
    for (size_t i = 0; i < (size_t)m * k; ++i) xf[i] = orc_bf16_to_f32(x[i]);
    orc_gemv_nk(xf, W, m, n, k, y);
    free(W); free(xf);
}
/* FP8 E4M3 W [n, k] with E8M0 scales per 32 x 32 block; reference ds41.cu:28-73. */
EXPORT void orc_fp8_e8m0_gemv(const uint16_t* x, const uint8_t* w, const uint8_t* s, float* y, int m, int n, int k)
{
    float* W = (float*)malloc((size_t)n * k * 4);
    float* xf = (float*)malloc((size_t)m * k * 4);
    orc_fp8_e8m0_dequant(w, s, n, k, W);
    for (size_t i = 0; i < (size_t)m * k; ++i) xf[i] = orc_bf16_to_f32(x[i]);
    orc_gemv_nk(xf, W, m, n, k, y);
    free(W); free(xf);
}

/* FP8 E4M3 W [n, k] with one binary32 scale per output row; x binary32 [m, k], rounded to binary16 (act 0) or bf16 (act 1) or used
 * as given (act 2); y[r, n] = (sum_k a(x) * w) * scale[n], rounded to binary16 when `rounded`.  The sum in binary64 (the products
 * are exact; the reference's kernels sum in binary32, each in its own order), rounded once to binary32 before the scale, as the
 * reference multiplies its finished binary32 sum.  reference engine-rs/shim/fp8.cu:13-22 (fp8_gemv), :110-151. */
EXPORT void orc_fp8_rowscale_gemv(const float* x, const uint8_t* w, const float* scale, float* y, int m, int n, int k, int act, int rounded)
{
    float* xa = (float*)malloc((size_t)m * k * 4);
    for (size_t i = 0; i < (size_t)m * k; ++i)
        xa[i] = act == 0 ? orc_f16_to_f32(orc_f32_to_f16(x[i])) : act == 1 ? orc_bf16_to_f32(orc_f32_to_bf16(x[i])) : x[i];
#pragma omp parallel for schedule(static)
    for (int c = 0; c < n; ++c)
        for (int r = 0; r < m; ++r) {
            double acc = 0.0;
            for (int j = 0; j < k; ++j) acc += (double)xa[(size_t)r * k + j] * (double)orc_e4m3_to_f32(w[(size_t)c * k + j]);
            float v = (float)acc * scale[c];
            if (rounded) v = orc_f16_to_f32(orc_f32_to_f16(v));
            y[(size_t)r * n + c] = v;
        }
    free(xa);
}
/* The quantiser of that format: scale[n] = max(row amax, 1e-12) / 448, q = e4m3_rn(clamp(w / scale, +-448)), the division in
 * binary32.  reference engine-rs/src/dense_fp8.rs:59-62 (quantize). */
EXPORT void orc_fp8_rowscale_quant(const float* w, uint8_t* q, float* scale, int n, int k)
{
    for (int r = 0; r < n; ++r) {
        float a = 0.f;
        for (int j = 0; j < k; ++j) a = fmaxf(a, fabsf(w[(size_t)r * k + j]));
        const float s = fmaxf(a, 1e-12f) / 448.0f;
        scale[r] = s;
        for (int j = 0; j < k; ++j) q[(size_t)r * k + j] = orc_f32_to_e4m3(fminf(fmaxf(w[(size_t)r * k + j] / s, -448.0f), 448.0f));
    }
}

EXPORT int orc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
