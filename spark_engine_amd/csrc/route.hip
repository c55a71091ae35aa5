// Routers: top-k selection over expert scores, ties to the lower expert id.
//   Qwen   softmax top-k                    reference engine-rs/shim/qwen_moe.cu:10-66,88-100
//   DS41   sqrt(softplus) + bias top-k       reference engine-rs/shim/ds41_ops.cu:376-419,609-614
//   GLM    sigmoid + bias top-k, fused GEMV  reference engine-rs/shim/dataflow.cu:370-546
#include "common.hpp"

using namespace spk;

namespace {

constexpr int ROUTE_EMAX = 1024;   // experts per row (one thread each)
constexpr int ROUTE_KMAX = 16;

// One workgroup per row, one thread per expert.  MODE 0: softmax (weights renormalised over the picks);
// 1: sqrt(softplus) + bias; 2: sigmoid + bias.  sel = value compared, score = value that becomes the weight.
// Selection by rank: expert e is pick number #{j : sel[j] > sel[e] or (sel[j] == sel[e] and j < e)}, which is the order
// repeated argmax with ties to the lower id produces, found in one parallel pass over LDS instead of K serial rounds.
template <int MODE, typename IT>
__device__ __forceinline__ void route_row(const float* __restrict__ x, const float* __restrict__ bias, IT* __restrict__ idx,
                                          float* __restrict__ w, int E, int K, float scale)
{
    __shared__ __align__(16) float ssel[ROUTE_EMAX];
    __shared__ float red[16], pick_s[ROUTE_KMAX];
    __shared__ int pick_i[ROUTE_KMAX];
    const int e = threadIdx.x, lane = e & 63, wv = e >> 6, nw = blockDim.x >> 6;
    const bool on = e < E;
    float score = 0.f, sel = -INFINITY;
    if (MODE == 0) {
        const float xv = on ? x[e] : -INFINITY;
        float m = wave_max(xv);
        if (lane == 0) red[wv] = m;
        __syncthreads();
        m = red[0];
        for (int i = 1; i < nw; ++i) m = fmaxf(m, red[i]);
        __syncthreads();
        const float p = on ? expf(xv - m) : 0.f;
        float s = wave_sum(p);
        if (lane == 0) red[wv] = s;
        __syncthreads();
        s = 0.f;
        for (int i = 0; i < nw; ++i) s += red[i];
        score = p / s;
        sel = on ? score : -INFINITY;
    } else if (on) {
        const float v = x[e];
        score = MODE == 1 ? sqrtf(v > 20.f ? v : log1pf(expf(v))) : 1.f / (1.f + expf(-v));
        sel = score + bias[e];
        if (sel != sel) sel = -INFINITY;               // a NaN never wins
    }
    ssel[e] = sel;
    __syncthreads();
    int rank = 0;
    const int E4 = (E + 3) & ~3;                        // blockDim.x >= E4: the tail entries hold -inf
    for (int j = 0; j < E4; j += 4) {
        const float4 o = *(const float4*)&ssel[j];
        rank += (o.x > sel || (o.x == sel && j < e)) + (o.y > sel || (o.y == sel && j + 1 < e)) + (o.z > sel || (o.z == sel && j + 2 < e)) +
                (o.w > sel || (o.w == sel && j + 3 < e));
    }
    if (on && rank < K) { pick_i[rank] = e; pick_s[rank] = score; }
    __syncthreads();
    if (e < K) {
        float sum = 0.f;
        for (int k = 0; k < K; ++k) sum += pick_s[k];
        idx[e] = (IT)pick_i[e];
        if (MODE == 0) w[e] = pick_s[e] / sum;
        else if (MODE == 1) w[e] = (K > 1 ? pick_s[e] / (sum + 1e-20f) : pick_s[e]) * scale;
        else w[e] = (pick_s[e] / fmaxf(sum, 1e-20f)) * scale;
    }
}

template <int MODE, typename IT>
__global__ __launch_bounds__(ROUTE_EMAX) void route_kernel(const float* __restrict__ logits, int64_t ld, const float* __restrict__ bias, IT* __restrict__ idx,
                                                           float* __restrict__ w, int T, int E, int K, float scale)
{
    const int row = blockIdx.x;
    route_row<MODE, IT>(logits + (int64_t)row * ld, bias, idx + (int64_t)row * K, w + (int64_t)row * K, E, K, scale);
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
__global__ __launch_bounds__(ROUTE_EMAX) void glm_select_kernel(const float* __restrict__ partial, const float* __restrict__ bias, long long* __restrict__ ids,
                                                                float* __restrict__ weights, int experts, int K, float scaling)
{
    __shared__ float lg[ROUTE_EMAX];
    const int r = blockIdx.x, e = threadIdx.x;
    if (e < experts) lg[e] = partial[((int64_t)r * experts + e) * 2] + partial[((int64_t)r * experts + e) * 2 + 1];
    __syncthreads();
    route_row<2, long long>(lg, bias, ids + (int64_t)r * K, weights + (int64_t)r * K, experts, K, scaling);
}

inline int route_threads(int E) { return (E + 63) & ~63; }

}  // namespace

// ================================================================ C ABI

// logits f32 [R, ld >= E] -> idx i32 [R, topk], w f32 [R, topk]; runtime expert count and top-k
SPARK_API int spark_softmax_route(const void* logits, int64_t ld, int R, int E, int topk, void* idx, void* w, hipStream_t st)
{
    if (R < 1) return 0;
    if (E < 1 || E > ROUTE_EMAX || topk < 1 || topk > ROUTE_KMAX || topk > E || ld < E) return 1;
    route_kernel<0, int><<<R, route_threads(E), 0, st>>>((const float*)logits, ld, nullptr, (int*)idx, (float*)w, R, E, topk, 1.0f);
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
    route_kernel<1, long long><<<T, route_threads(E), 0, st>>>(logits, E, bias, (long long*)idx, w, T, E, K, scale);
    return launch_status();
}
// sigmoid + bias selection on ready logits f32 [T, E]
SPARK_API int spark_sigmoid_route(const float* logits, const float* bias, int64_t* idx, float* w, int T, int E, int K, float scaling, hipStream_t st)
{
    if (T < 1) return 0;
    if (E < 1 || E > ROUTE_EMAX || K > ROUTE_KMAX || K < 1 || K > E) return 1;
    route_kernel<2, long long><<<T, route_threads(E), 0, st>>>(logits, E, bias, (long long*)idx, w, T, E, K, scaling);
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
    glm_select_kernel<<<rows, route_threads(experts), 0, st>>>(partial, bias, ids, weights, experts, 8, scaling);
    return launch_status();
}
