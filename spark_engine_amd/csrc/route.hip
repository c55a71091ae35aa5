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

// MODE 0: softmax (weights renormalised over the picks); 1: sqrt(softplus) + bias; 2: sigmoid + bias.  The selection compares
// score + bias (softmax: the score), the weight comes from the score.  Ties go to the lower expert id.
// score and selection key of one expert for the bias modes (1: sqrt(softplus), 2: sigmoid)
template <int MODE> __device__ __forceinline__ void bias_score(float v, float b, float& score, uint32_t& key)
{
    score = MODE == 1 ? sqrtf(v > 20.f ? v : log1pf(expf(v))) : 1.f / (1.f + expf(-v));
    const float sel = score + b;
    key = sel != sel ? 1u : max(fkey(sel), 1u);          // a NaN never wins over a number; -inf still ranks above "absent"
}

// Four waves per row: thread t holds experts t * PER .. t * PER + PER - 1 (PER = 1, 2 or 4), so scoring, sorting and the rounds
// work on a quarter of the candidates each and a lone wave's chain of dependent instructions is half as long.  Every wave picks the
// K best of its own 64 * PER experts (every thread sorts its candidates once; a round is the wave's largest head by a DPP reduction,
// the lowest lane that holds it - a ballot - and that lane dropping its head); the 4 K picks meet in LDS as 64-bit words (key above, the
// complement of the expert id below: a larger word is a better pick, equal keys go to the lower id) and each finds its rank among
// them by counting the picks of the other waves that beat it - a wave's own picks are already in order.  Ranks 0 .. K - 1 are the
// row's picks in order: the same picks as one wave's K rounds over all experts, because every one of the row's K best is among
// the K best of its wave.
// Whatever the logits hold (NaNs, infinities), a row's picks are K different experts in [0, E): present experts have keys >= 1,
// absent ones 0, K <= E, and a pick leaves its thread's list when it is taken.
template <int MODE, int PER, typename IT>
__device__ __forceinline__ void route_block(const float* __restrict__ x, const float* __restrict__ bias, IT* __restrict__ idx, float* __restrict__ wr, int E,
                                            int K, float scale)
{
    __shared__ uint32_t s_max[4];
    __shared__ float s_sum[4];
    __shared__ float s_score[MODE != 0 ? 256 * PER : 1];
    __shared__ uint64_t s_cand[4][ROUTE_KMAX];
    __shared__ uint32_t s_pkey[ROUTE_KMAX];
    __shared__ int s_pid[ROUTE_KMAX];
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int e0 = tid * PER;
    uint32_t key[PER];                                   // 0 = not a candidate (absent)
    if constexpr (MODE == 0) {
        float xv[PER], score[PER], m = -INFINITY;
#pragma unroll
        for (int i = 0; i < PER; ++i) { const float v = x[min(e0 + i, E - 1)]; xv[i] = e0 + i < E ? v : -INFINITY; m = fmaxf(m, xv[i]); }
        const uint32_t kw = wave_umax(fkey(m));
        if (lane == 0) s_max[wv] = kw;
        __syncthreads();
        const uint32_t km = max(max(s_max[0], s_max[1]), max(s_max[2], s_max[3]));
        m = __uint_as_float((km & 0x80000000u) ? (km & 0x7fffffffu) : ~km);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) { score[i] = e0 + i < E ? expf(xv[i] - m) : 0.f; s += score[i]; }
        s = wave_fsum(s);
        if (lane == 0) s_sum[wv] = s;
        __syncthreads();
        s = (s_sum[0] + s_sum[1]) + (s_sum[2] + s_sum[3]);   // fixed order: the same bits on every call
#pragma unroll
        for (int i = 0; i < PER; ++i) key[i] = e0 + i < E ? max(fkey(score[i] / s), 1u) : 0u;      // a present expert is always a candidate
    } else {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = min(e0 + i, E - 1);
            float sc; uint32_t ky;
            bias_score<MODE>(x[e], bias[e], sc, ky);
            key[i] = e0 + i < E ? ky : 0u;
            s_score[e0 + i] = e0 + i < E ? sc : 0.f;
        }
    }
    // the wave's K best, best first: lane k keeps pick k
    uint64_t q[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) q[i] = ((uint64_t)key[i] << 32) | (uint32_t)(PER - 1 - i);
    auto cx = [&](int i, int j) {                          // larger first
        const bool sw = q[j] > q[i];
        const uint64_t hi = sw ? q[j] : q[i], lo = sw ? q[i] : q[j];
        q[i] = hi; q[j] = lo;
    };
    if constexpr (PER == 2) cx(0, 1);
    if constexpr (PER == 4) { cx(0, 1); cx(2, 3); cx(0, 2); cx(1, 3); cx(1, 2); }
    uint64_t mine = 0ull;
    for (int k = 0; k < K; ++k) {
        const uint32_t bk = (uint32_t)(q[0] >> 32);
        const uint32_t wk = wave_umax(bk);
        const uint64_t bal = __builtin_amdgcn_ballot_w64(bk == wk);
        const int wl = __builtin_ctzll(bal);               // lowest lane = lowest expert ids
        const int wi = PER - 1 - __builtin_amdgcn_readlane((int)(uint32_t)q[0], wl);
        if (lane == k) mine = ((uint64_t)wk << 32) | (uint32_t)~(uint32_t)((wv * 64 + wl) * PER + wi);
        const bool win = lane == wl;
#pragma unroll
        for (int i = 0; i + 1 < PER; ++i) q[i] = win ? q[i + 1] : q[i];
        q[PER - 1] = win ? 0ull : q[PER - 1];
    }
    if (lane < ROUTE_KMAX) s_cand[wv][lane] = lane < K ? mine : 0ull;
    __syncthreads();
    if (wv == 0) {
        const int lw = lane >> 4, lk = lane & 15;           // ROUTE_KMAX = 16 picks of each of the four waves: one per lane
        const uint64_t c = s_cand[lw][lk];
        int rank = lk;
        for (int k3 = 0; k3 < K; ++k3) {
#pragma unroll
            for (int j = 1; j < 4; ++j) rank += s_cand[(lw + j) & 3][k3] > c ? 1 : 0;
        }
        if (lk < K && rank < K) { s_pkey[rank] = (uint32_t)(c >> 32); s_pid[rank] = (int)~(uint32_t)c; }
    }
    __syncthreads();
    if (wv == 0) {
        float pick = 0.f, sum = 0.f;
        int id = 0;
        if (lane < K) {
            id = min(max(s_pid[lane], 0), E - 1);
            const uint32_t ky = s_pkey[lane];
            // the pick's score: the key read backwards (softmax: the key orders the score itself), else the expert's score
            pick = MODE == 0 ? __uint_as_float((ky & 0x80000000u) ? (ky & 0x7fffffffu) : ~ky) : s_score[id];
        }
        for (int k = 0; k < K; ++k) sum += readlane_f(pick, k);          // in pick order
        if (lane < K) {
            idx[lane] = (IT)id;
            if (MODE == 0) wr[lane] = pick / sum;
            else if (MODE == 1) wr[lane] = (K > 1 ? pick / (sum + 1e-20f) : pick) * scale;
            else wr[lane] = (pick / fmaxf(sum, 1e-20f)) * scale;
        }
    }
}
template <int MODE, int PER, typename IT>
__global__ __launch_bounds__(256) void route_kernel4(const float* __restrict__ logits, int64_t ld, const float* __restrict__ bias, IT* __restrict__ idx,
                                                     float* __restrict__ w, int T, int E, int K, float scale)
{
    const int row = blockIdx.x;
    route_block<MODE, PER, IT>(logits + (int64_t)row * ld, bias, idx + (int64_t)row * K, w + (int64_t)row * K, E, K, scale);
}
template <int MODE, typename IT>
void launch_route(const float* logits, int64_t ld, const float* bias, IT* idx, float* w, int T, int E, int K, float scale, hipStream_t st)
{
    static_assert(ROUTE_KMAX == 16 && ROUTE_EMAX == 1024, "route_kernel4: 4 x 16 picks in one wave, at most 4 experts a thread");
    if (E <= 256) route_kernel4<MODE, 1, IT><<<T, 256, 0, st>>>(logits, ld, bias, idx, w, T, E, K, scale);
    else if (E <= 512) route_kernel4<MODE, 2, IT><<<T, 256, 0, st>>>(logits, ld, bias, idx, w, T, E, K, scale);
    else route_kernel4<MODE, 4, IT><<<T, 256, 0, st>>>(logits, ld, bias, idx, w, T, E, K, scale);
}

// GLM router logits: partial[(r*E + e)*2 + half] = sum over half of K of h[r, k] * W[e, k], binary32 fma.
// One workgroup per expert, eight waves: four per half, each a quarter of the half (one wave per (expert, half), 576 waves that
// walk 2048 k each, took 5 us for 288 x 4096); a lane strides 4 elements, the quarters are added through LDS in wave order.
template <typename WT>
__global__ __launch_bounds__(512) void glm_logits_kernel(const float* __restrict__ h, const WT* __restrict__ w, float* __restrict__ partial, int rows,
                                                         int experts, int k)
{
    __shared__ float red[8][32];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int e = blockIdx.x, half = wave >> 2, span = k / 2, sub = span / 4, start = half * span + (wave & 3) * sub;
    const WT* wr = w + (int64_t)e * k + start;
    for (int r0 = 0; r0 < rows; r0 += 8) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int c = lane * 4; c < sub; c += 256) {
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
            if (lane == 0) red[wave][r0 + r] = s;
        }
    }
    __syncthreads();
    for (int t = threadIdx.x; t < rows * 2; t += 512) {
        const int r = t >> 1, hf = t & 1;
        const float v = ((red[4 * hf][r] + red[4 * hf + 1][r]) + red[4 * hf + 2][r]) + red[4 * hf + 3][r];
        partial[((int64_t)r * experts + e) * 2 + hf] = v;
    }
}
__global__ __launch_bounds__(256) void glm_select_kernel(const float* __restrict__ partial, const float* __restrict__ bias, long long* __restrict__ ids,
                                                         float* weights, int experts, int K, float scaling, uint16_t* __restrict__ wh)
{
    // wh (may be null): the binary16 copy of the row's weights, round to nearest even, for the expert entry points that take them so
    __shared__ float lg[320];
    const int r = blockIdx.x;
    for (int e = threadIdx.x; e < experts; e += 256) lg[e] = partial[((int64_t)r * experts + e) * 2] + partial[((int64_t)r * experts + e) * 2 + 1];
    __syncthreads();
    route_block<2, 2, long long>(lg, bias, ids + (int64_t)r * K, weights + (int64_t)r * K, experts, K, scaling);
    if (wh) {
        __threadfence_block();
        __syncthreads();                                   // the row's weights are written: the same values, rounded once
        if ((int)threadIdx.x < K) wh[(int64_t)r * K + threadIdx.x] = f32_to_f16_bits(__hip_atomic_load(weights + (int64_t)r * K + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
    }
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
    if (w_bf16) glm_logits_kernel<uint16_t><<<experts, 512, 0, st>>>(h, (const uint16_t*)w, partial, rows, experts, k);
    else glm_logits_kernel<float><<<experts, 512, 0, st>>>(h, (const float*)w, partial, rows, experts, k);
    glm_select_kernel<<<rows, 256, 0, st>>>(partial, bias, ids, weights, experts, 8, scaling, nullptr);
    return launch_status();
}
// reference dataflow.cu:549-574 (GLM53_ROUTER_HALF_W=1): the same, and wh [rows, 8] receives the binary16 rounding of the weights
// that glm_moe_experts takes (the reference otherwise converts them in a launch of its own)
SPARK_API int glm53_router_fused_h_cuda(const float* h, const void* w, int w_bf16, const float* bias, float* partial, long long* ids, float* weights,
                                        void* wh, int rows, int experts, int k, float scaling, hipStream_t st)
{
    if (rows < 1 || rows > 32 || experts < 8 || experts > 320 || k % 256 || !wh) return (int)hipErrorInvalidValue;
    if (w_bf16) glm_logits_kernel<uint16_t><<<experts, 512, 0, st>>>(h, (const uint16_t*)w, partial, rows, experts, k);
    else glm_logits_kernel<float><<<experts, 512, 0, st>>>(h, (const float*)w, partial, rows, experts, k);
    glm_select_kernel<<<rows, 256, 0, st>>>(partial, bias, ids, weights, experts, 8, scaling, (uint16_t*)wh);
    return launch_status();
}
