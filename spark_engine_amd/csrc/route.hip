// Routers: top-k selection over expert scores, ties to the lower expert id.
//   Qwen   softmax top-k                    reference engine-rs/shim/qwen_moe.cu:10-66,88-100
//   DS41   sqrt(softplus) + bias top-k       reference engine-rs/shim/ds41_ops.cu:376-419,609-614
//   GLM    sigmoid + bias top-k, fused GEMV  reference engine-rs/shim/dataflow.cu:370-546
#include "common.hpp"

using namespace spk;

namespace {

constexpr int ROUTE_EMAX = 1024;   // experts per row (16 per lane of one wave)
constexpr int ROUTE_KMAX = 16;

// ---- wave64 all-reduce with DPP (no LDS traffic): butterflies inside each row of 16 lanes, then the four row results are
// read back as scalars.  The result is wave-uniform.
template <int CTRL> __device__ __forceinline__ uint32_t dpp_u32(uint32_t v) { return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false); }
template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) { return __uint_as_float(dpp_u32<CTRL>(__float_as_uint(v))); }
constexpr int DPP_XOR1 = 0xB1, DPP_XOR2 = 0x4E, DPP_ROR4 = 0x124, DPP_ROR8 = 0x128;   // quad_perm [1,0,3,2], [2,3,0,1]; row_ror:4, row_ror:8
__device__ __forceinline__ uint32_t wave_umax(uint32_t v)
{
    v = max(v, dpp_u32<DPP_XOR1>(v)); v = max(v, dpp_u32<DPP_XOR2>(v));
    v = max(v, dpp_u32<DPP_ROR4>(v)); v = max(v, dpp_u32<DPP_ROR8>(v));
    const uint32_t a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16), c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return max(max(a, b), max(c, d));
}
__device__ __forceinline__ float readlane_f(float v, int l) { return __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), l)); }
// fixed summation tree: the result is the same on every lane and from call to call
__device__ __forceinline__ float wave_fsum(float v)
{
    v += dpp_f32<DPP_XOR1>(v); v += dpp_f32<DPP_XOR2>(v);
    v += dpp_f32<DPP_ROR4>(v); v += dpp_f32<DPP_ROR8>(v);
    const float a = readlane_f(v, 0), b = readlane_f(v, 16), c = readlane_f(v, 32), d = readlane_f(v, 48);
    return (a + b) + (c + d);
}
// order-preserving map of a float to an unsigned integer (-0 treated as +0)
__device__ __forceinline__ uint32_t fkey(float f)
{
    const uint32_t u = __float_as_uint(f + 0.0f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// One wave per row; lane l holds experts l * PER .. l * PER + PER - 1 in registers.  MODE 0: softmax (weights renormalised
// over the picks); 1: sqrt(softplus) + bias; 2: sigmoid + bias.  sel = value compared, score = value that becomes the
// weight.  K rounds of argmax: the largest key by a DPP reduction, then the lowest lane holding it (a ballot) and that
// lane's lowest expert with it: ties go to the lower expert id.
// score and selection key of one expert for the bias modes (1: sqrt(softplus), 2: sigmoid)
template <int MODE> __device__ __forceinline__ void bias_score(float v, float b, float& score, uint32_t& key)
{
    score = MODE == 1 ? sqrtf(v > 20.f ? v : log1pf(expf(v))) : 1.f / (1.f + expf(-v));
    const float sel = score + b;
    key = sel != sel ? 1u : max(fkey(sel), 1u);          // a NaN never wins over a number; -inf still ranks above "absent"
}

// pre = scores and keys of all lane * PER + i already worked out (LDS arrays of 64 * PER entries), or null
template <int MODE, int PER, typename IT>
__device__ __forceinline__ void route_row(const float* __restrict__ x, const float* __restrict__ bias, IT* __restrict__ idx,
                                          float* __restrict__ w, int E, int K, float scale, int lane, const float* pre_score = nullptr,
                                          const uint32_t* pre_key = nullptr)
{
    float score[PER];
    uint32_t key[PER];                                   // 0 = not a candidate (absent, taken, or NaN)
    const int e0 = lane * PER;
    if (MODE != 0 && pre_score) {
#pragma unroll
        for (int i = 0; i < PER; ++i) { score[i] = pre_score[e0 + i]; key[i] = pre_key[e0 + i]; }
    } else if (MODE == 0) {
        float xv[PER], m = -INFINITY;
#pragma unroll
        for (int i = 0; i < PER; ++i) { xv[i] = e0 + i < E ? x[e0 + i] : -INFINITY; m = fmaxf(m, xv[i]); }
        // wave maximum through the ordered keys
        {
            const uint32_t km = wave_umax(fkey(m));
            m = __uint_as_float((km & 0x80000000u) ? (km & 0x7fffffffu) : ~km);
        }
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) { score[i] = e0 + i < E ? expf(xv[i] - m) : 0.f; s += score[i]; }
        s = wave_fsum(s);
#pragma unroll
        for (int i = 0; i < PER; ++i) { score[i] = score[i] / s; key[i] = e0 + i < E ? fkey(score[i]) : 0u; }
    } else {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            score[i] = 0.f; key[i] = 0u;
            if (e0 + i < E) bias_score<MODE>(x[e0 + i], bias[e0 + i], score[i], key[i]);
        }
    }
    float mine = 0.f, sum = 0.f;                          // lane k keeps pick k
    int mine_id = 0;
    if constexpr (PER == 4 || PER == 8) {
        // Every lane sorts its own candidates once (a fixed compare-exchange network on 64-bit words: key above, PER - 1 - i below,
        // so equal keys keep the lower expert first); a round is then the wave's largest head, the lowest lane that holds it, and
        // that lane dropping its head.  A third of the instructions per round of scanning the lane's candidates every round,
        // and the same picks: same keys, ties to the lowest lane and there to the lowest i.
        uint64_t q[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) q[i] = ((uint64_t)key[i] << 32) | (uint32_t)(PER - 1 - i);
        auto cx = [&](int i, int j) {                      // larger first
            const bool sw = q[j] > q[i];
            const uint64_t hi = sw ? q[j] : q[i], lo = sw ? q[i] : q[j];
            q[i] = hi; q[j] = lo;
        };
        if constexpr (PER == 8) {
            cx(0, 1); cx(2, 3); cx(4, 5); cx(6, 7); cx(0, 2); cx(1, 3); cx(4, 6); cx(5, 7); cx(1, 2); cx(5, 6); cx(0, 4); cx(3, 7);
            cx(1, 5); cx(2, 6); cx(1, 4); cx(3, 6); cx(2, 4); cx(3, 5); cx(3, 4);
        } else {
            cx(0, 1); cx(2, 3); cx(0, 2); cx(1, 3); cx(1, 2);
        }
        uint32_t mine_key = 0u;
        for (int k = 0; k < K; ++k) {
            const uint32_t bk = (uint32_t)(q[0] >> 32);
            const uint32_t wk = wave_umax(bk);
            const uint64_t bal = __builtin_amdgcn_ballot_w64(bk == wk);
            const int wl = __builtin_ctzll(bal);           // lowest lane = lowest expert ids
            const int wi = PER - 1 - __builtin_amdgcn_readlane((int)(uint32_t)q[0], wl);
            if (lane == k) { mine_key = wk; mine_id = wl * PER + wi; }
            const bool win = lane == wl;
#pragma unroll
            for (int i = 0; i + 1 < PER; ++i) q[i] = win ? q[i + 1] : q[i];
            q[PER - 1] = win ? 0ull : q[PER - 1];
        }
        // the pick's score: the key read backwards (softmax: the key orders the score itself), else the expert's score again
        if (MODE == 0) mine = __uint_as_float((mine_key & 0x80000000u) ? (mine_key & 0x7fffffffu) : ~mine_key);
        else if (lane < K) {
            if (pre_score) mine = pre_score[mine_id];
            else { uint32_t ky; bias_score<MODE>(x[mine_id], bias[mine_id], mine, ky); }
        }
        for (int k = 0; k < K; ++k) sum += readlane_f(mine, k);          // in pick order
    } else {
        for (int k = 0; k < K; ++k) {
            uint32_t bk = 0u; int bi = 0;
#pragma unroll
            for (int i = PER - 1; i >= 0; --i) if (key[i] >= bk) { bk = key[i]; bi = i; }   // lowest i among equals
            const uint32_t wk = wave_umax(bk);
            const uint64_t bal = __builtin_amdgcn_ballot_w64(bk == wk);
            const int wl = __builtin_ctzll(bal);               // lowest lane = lowest expert ids
            const int wi = __builtin_amdgcn_readlane(bi, wl);
            float sc = 0.f;
#pragma unroll
            for (int i = 0; i < PER; ++i) if (lane == wl && i == wi) { sc = score[i]; key[i] = 0u; }
            sc = readlane_f(sc, wl);
            sum += sc;
            if (lane == k) { mine = sc; mine_id = wl * PER + wi; }
        }
    }
    if (lane < K) {
        idx[lane] = (IT)mine_id;
        if (MODE == 0) w[lane] = mine / sum;
        else if (MODE == 1) w[lane] = (K > 1 ? mine / (sum + 1e-20f) : mine) * scale;
        else w[lane] = (mine / fmaxf(sum, 1e-20f)) * scale;
    }
}

template <int MODE, int PER, typename IT>
__global__ __launch_bounds__(64) void route_kernel(const float* __restrict__ logits, int64_t ld, const float* __restrict__ bias, IT* __restrict__ idx,
                                                   float* __restrict__ w, int T, int E, int K, float scale)
{
    const int row = blockIdx.x;
    route_row<MODE, PER, IT>(logits + (int64_t)row * ld, bias, idx + (int64_t)row * K, w + (int64_t)row * K, E, K, scale, threadIdx.x);
}
// The bias modes spend most of their time in the transcendental functions (softplus, sqrt: ~70 instructions an expert, eight or
// sixteen experts a lane).  Four waves share that part, one expert per thread and round, and hand the scores to the first wave
// through LDS; the selection is the one-wave routine above.  Same functions on the same inputs: the same bits.
template <int MODE, int PER, typename IT>
__global__ __launch_bounds__(256) void route_kernel_mw(const float* __restrict__ logits, int64_t ld, const float* __restrict__ bias, IT* __restrict__ idx,
                                                       float* __restrict__ w, int T, int E, int K, float scale)
{
    __shared__ float s_score[64 * PER];
    __shared__ uint32_t s_key[64 * PER];
    const int row = blockIdx.x;
    const float* x = logits + (int64_t)row * ld;
    for (int e = threadIdx.x; e < 64 * PER; e += 256) {
        float sc = 0.f; uint32_t ky = 0u;
        if (e < E) bias_score<MODE>(x[e], bias[e], sc, ky);
        s_score[e] = sc; s_key[e] = ky;
    }
    __syncthreads();
    if (threadIdx.x < 64)
        route_row<MODE, PER, IT>(x, bias, idx + (int64_t)row * K, w + (int64_t)row * K, E, K, scale, threadIdx.x, s_score, s_key);
}
template <int MODE, typename IT>
void launch_route(const float* logits, int64_t ld, const float* bias, IT* idx, float* w, int T, int E, int K, float scale, hipStream_t st)
{
    if constexpr (MODE != 0) {
        if (E <= 256) route_kernel_mw<MODE, 4, IT><<<T, 256, 0, st>>>(logits, ld, bias, idx, w, T, E, K, scale);
        else if (E <= 512) route_kernel_mw<MODE, 8, IT><<<T, 256, 0, st>>>(logits, ld, bias, idx, w, T, E, K, scale);
        else route_kernel_mw<MODE, 16, IT><<<T, 256, 0, st>>>(logits, ld, bias, idx, w, T, E, K, scale);
        return;
    }
    if (E <= 256) route_kernel<MODE, 4, IT><<<T, 64, 0, st>>>(logits, ld, bias, idx, w, T, E, K, scale);
    else if (E <= 512) route_kernel<MODE, 8, IT><<<T, 64, 0, st>>>(logits, ld, bias, idx, w, T, E, K, scale);
    else route_kernel<MODE, 16, IT><<<T, 64, 0, st>>>(logits, ld, bias, idx, w, T, E, K, scale);
}

// GLM router logits: partial[(r*E + e)*2 + half] = sum over half of K of h[r, k] * W[e, k], binary32 fma.
// One wave per (expert, half); lane strides of 4 elements.
template <typename WT>
__global__ __launch_bounds__(256) void glm_logits_kernel(const float* __restrict__ h, const WT* __restrict__ w, float* __restrict__ partial, int rows,
                                                         int experts, int k)
{
    const int wv = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (wv >= experts * 2) return;
    const int e = wv >> 1, half = wv & 1, span = k / 2, start = half * span;
    const WT* wr = w + (int64_t)e * k + start;
    for (int r0 = 0; r0 < rows; r0 += 8) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int c = lane * 4; c < span; c += 256) {
            float wf[4];
            if constexpr (sizeof(WT) == 2) { for (int j = 0; j < 4; ++j) wf[j] = bf16_to_f32(((const uint16_t*)wr)[c + j]); }
            else { for (int j = 0; j < 4; ++j) wf[j] = ((const float*)wr)[c + j]; }
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                if (r0 + r >= rows) break;
                const float* xr = h + (int64_t)(r0 + r) * k + start + c;
                float a = acc[r];
                for (int j = 0; j < 4; ++j) a = __builtin_fmaf(xr[j], wf[j], a);
                acc[r] = a;
            }
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            if (r0 + r >= rows) break;
            const float s = wave_sum(acc[r]);
            if (lane == 0) partial[((int64_t)(r0 + r) * experts + e) * 2 + half] = s;
        }
    }
}
__global__ __launch_bounds__(64) void glm_select_kernel(const float* __restrict__ partial, const float* __restrict__ bias, long long* __restrict__ ids,
                                                        float* __restrict__ weights, int experts, int K, float scaling)
{
    __shared__ float lg[320];
    const int r = blockIdx.x, lane = threadIdx.x;
    for (int e = lane; e < experts; e += 64) lg[e] = partial[((int64_t)r * experts + e) * 2] + partial[((int64_t)r * experts + e) * 2 + 1];
    __syncthreads();
    route_row<2, 5, long long>(lg, bias, ids + (int64_t)r * K, weights + (int64_t)r * K, experts, K, scaling, lane);
}

}  // namespace

// ================================================================ C ABI

// logits f32 [R, ld >= E] -> idx i32 [R, topk], w f32 [R, topk]; runtime expert count and top-k
SPARK_API int spark_softmax_route(const void* logits, int64_t ld, int R, int E, int topk, void* idx, void* w, hipStream_t st)
{
    if (R < 1) return 0;
    if (E < 1 || E > ROUTE_EMAX || topk < 1 || topk > ROUTE_KMAX || topk > E || ld < E) return 1;
    launch_route<0, int>((const float*)logits, ld, nullptr, (int*)idx, (float*)w, R, E, topk, 1.0f, st);
    return launch_status();
}
// reference qwen_moe.cu:88-100: 512 experts, top-10
SPARK_API int qwen_moe_route(const void* logits, int R, void* idx, void* w, hipStream_t st)
{
    return spark_softmax_route(logits, 512, R, 512, 10, idx, w, st);
}
SPARK_API int qwen_moe_route_ld(const void* logits, int64_t ld, int R, void* idx, void* w, hipStream_t st)
{
    return spark_softmax_route(logits, ld, R, 512, 10, idx, w, st);
}
// reference ds41_ops.cu:609-614; the expert and top-k limits are wider here (E <= 1024, K <= 16)
SPARK_API int ds41_route(const float* logits, const float* bias, int64_t* idx, float* w, int T, int E, int K, float scale, hipStream_t st)
{
    if (T < 1) return 0;
    if (E < 1 || E > ROUTE_EMAX || K > ROUTE_KMAX || K < 1 || K > E) return 1;
    launch_route<1, long long>(logits, E, bias, (long long*)idx, w, T, E, K, scale, st);
    return launch_status();
}
// sigmoid + bias selection on ready logits f32 [T, E]
SPARK_API int spark_sigmoid_route(const float* logits, const float* bias, int64_t* idx, float* w, int T, int E, int K, float scaling, hipStream_t st)
{
    if (T < 1) return 0;
    if (E < 1 || E > ROUTE_EMAX || K > ROUTE_KMAX || K < 1 || K > E) return 1;
    launch_route<2, long long>(logits, E, bias, (long long*)idx, w, T, E, K, scaling, st);
    return launch_status();
}
// reference dataflow.cu:519-546: h f32 [rows, k], w f32 or bf16 [experts, k], partial f32 [rows, experts, 2] scratch
SPARK_API int glm53_router_split() { return 2; }
SPARK_API int glm53_router_fused_cuda(const float* h, const void* w, int w_bf16, const float* bias, float* partial, long long* ids, float* weights,
                                      int rows, int experts, int k, float scaling, hipStream_t st)
{
    if (rows < 1 || rows > 32 || experts < 8 || experts > 320 || k % 256) return (int)hipErrorInvalidValue;
    const unsigned g = (unsigned)((experts * 2 + 3) / 4);
    if (w_bf16) glm_logits_kernel<uint16_t><<<g, 256, 0, st>>>(h, (const uint16_t*)w, partial, rows, experts, k);
    else glm_logits_kernel<float><<<g, 256, 0, st>>>(h, (const float*)w, partial, rows, experts, k);
    glm_select_kernel<<<rows, 64, 0, st>>>(partial, bias, ids, weights, experts, 8, scaling);
    return launch_status();
}
