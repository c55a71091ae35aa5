// Routers: top-k selection over expert scores, ties to the lower expert id.
//   Qwen   softmax top-k                    reference engine-rs/shim/qwen_moe.cu:10-66,88-100
//   DS41   sqrt(softplus) + bias top-k       reference engine-rs/shim/ds41_ops.cu:376-419,609-614
//   GLM    sigmoid + bias top-k, fused GEMV  reference engine-rs/shim/dataflow.cu:370-546
#include "common.hpp"

using namespace spk;

namespace {

constexpr int ROUTE_EMAX = 1024;   // experts per row a wave can hold (16 per lane)
constexpr int ROUTE_KMAX = 16;

// wave-wide argmax of (value, id): larger value wins, equal values go to the lower id
__device__ __forceinline__ void wave_argmax(float& v, int& id)
{
#pragma unroll
    for (int o = 32; o; o >>= 1) {
        const float ov = __shfl_xor(v, o, 64);
        const int oi = __shfl_xor(id, o, 64);
        if (ov > v || (ov == v && oi < id)) { v = ov; id = oi; }
    }
}

// One wave per row.  MODE 0: softmax (weights renormalised over the picks); 1: sqrt(softplus) + bias;
// 2: sigmoid + bias.  sel = value compared, score = value that becomes the weight.
template <int MODE, typename IT>
__device__ __forceinline__ void route_row(const float* __restrict__ x, const float* __restrict__ bias, IT* __restrict__ idx,
                                          float* __restrict__ w, int E, int K, float scale, int lane)
{
    constexpr int PER = ROUTE_EMAX / 64;
    float score[PER], sel[PER];
    if (MODE == 0) {
        float m = -INFINITY;
#pragma unroll
        for (int i = 0; i < PER; ++i) { const int e = lane + 64 * i; score[i] = e < E ? x[e] : -INFINITY; m = fmaxf(m, score[i]); }
        m = wave_max(m);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) { const int e = lane + 64 * i; score[i] = e < E ? expf(score[i] - m) : 0.f; s += score[i]; }
        s = wave_sum(s);
#pragma unroll
        for (int i = 0; i < PER; ++i) { const int e = lane + 64 * i; score[i] = score[i] / s; sel[i] = e < E ? score[i] : -INFINITY; }
    } else {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = lane + 64 * i;
            if (e < E) {
                const float v = x[e];
                score[i] = MODE == 1 ? sqrtf(v > 20.f ? v : log1pf(expf(v))) : 1.f / (1.f + expf(-v));
                sel[i] = score[i] + bias[e];
                if (sel[i] != sel[i]) sel[i] = -INFINITY;      // a NaN never wins
            } else { score[i] = 0.f; sel[i] = -INFINITY; }
        }
    }
    float picked[ROUTE_KMAX];
    int pid[ROUTE_KMAX];
#pragma unroll
    for (int k = 0; k < ROUTE_KMAX; ++k) {
        if (k >= K) break;
        float bv = -INFINITY, bs = 0.f;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < PER; ++i) { const int e = lane + 64 * i; if (e < E && (sel[i] > bv || (sel[i] == bv && e < bi))) { bv = sel[i]; bi = e; bs = score[i]; } }
        wave_argmax(bv, bi);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) if (lane + 64 * i == bi) { s = score[i]; sel[i] = -INFINITY; }
        (void)bs;
        picked[k] = __shfl(s, bi & 63, 64);
        pid[k] = bi;
    }
    if (lane == 0) {
        float sum = 0.f;
#pragma unroll
        for (int k = 0; k < ROUTE_KMAX; ++k) if (k < K) sum += picked[k];
#pragma unroll
        for (int k = 0; k < ROUTE_KMAX; ++k) {
            if (k >= K) break;
            idx[k] = (IT)pid[k];
            if (MODE == 0) w[k] = picked[k] / sum;
            else if (MODE == 1) w[k] = (K > 1 ? picked[k] / (sum + 1e-20f) : picked[k]) * scale;
            else w[k] = (picked[k] / fmaxf(sum, 1e-20f)) * scale;
        }
    }
}

template <int MODE, typename IT>
__global__ __launch_bounds__(256) void route_kernel(const float* __restrict__ logits, int64_t ld, const float* __restrict__ bias, IT* __restrict__ idx,
                                                    float* __restrict__ w, int T, int E, int K, float scale)
{
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= T) return;
    route_row<MODE, IT>(logits + (int64_t)row * ld, bias, idx + (int64_t)row * K, w + (int64_t)row * K, E, K, scale, lane);
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
    __shared__ float lg[ROUTE_EMAX];
    const int r = blockIdx.x, lane = threadIdx.x;
    for (int e = lane; e < experts; e += 64) lg[e] = partial[((int64_t)r * experts + e) * 2] + partial[((int64_t)r * experts + e) * 2 + 1];
    __syncthreads();
    route_row<2, long long>(lg, bias, ids + (int64_t)r * K, weights + (int64_t)r * K, experts, K, scaling, lane);
}

}  // namespace

// ================================================================ C ABI

// logits f32 [R, ld >= E] -> idx i32 [R, topk], w f32 [R, topk]; runtime expert count and top-k
SPARK_API int spark_softmax_route(const void* logits, int64_t ld, int R, int E, int topk, void* idx, void* w, hipStream_t st)
{
    if (R < 1) return 0;
    if (E < 1 || E > ROUTE_EMAX || topk < 1 || topk > ROUTE_KMAX || topk > E || ld < E) return 1;
    route_kernel<0, int><<<(R + 3) / 4, 256, 0, st>>>((const float*)logits, ld, nullptr, (int*)idx, (float*)w, R, E, topk, 1.0f);
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
    route_kernel<1, long long><<<(T + 3) / 4, 256, 0, st>>>(logits, E, bias, (long long*)idx, w, T, E, K, scale);
    return launch_status();
}
// sigmoid + bias selection on ready logits f32 [T, E]
SPARK_API int spark_sigmoid_route(const float* logits, const float* bias, int64_t* idx, float* w, int T, int E, int K, float scaling, hipStream_t st)
{
    if (T < 1) return 0;
    if (E < 1 || E > ROUTE_EMAX || K > ROUTE_KMAX || K < 1 || K > E) return 1;
    route_kernel<2, long long><<<(T + 3) / 4, 256, 0, st>>>(logits, E, bias, (long long*)idx, w, T, E, K, scaling);
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
