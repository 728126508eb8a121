// Feed-forwards without a gate projection, act(x Wup^T) Wdown^T, dense or as a mixture of experts.
//
// The router: scores = softmax over all experts of the 32-bit logits; the `top` largest are chosen (of equal scores the
// lower index first); an expert's weight is its score, as it is or divided by the chosen scores' sum.  The experts' up
// matrices lie one under the other and their down matrices side by side, so that the experts of a token are a dense
// feed-forward of experts * ff hidden units whose activations are multiplied by the expert's weight, zero for the
// experts that were not chosen: the activation kernel below applies act and that weight in one pass.
#include "common.h"

#define ROUTE_MAX_EXPERTS 1024

// One wave a token.  weights [T, E] 32-bit: the chosen experts' weights, zero elsewhere.
__global__ __launch_bounds__(64) void route_topk_kernel(const float* __restrict__ logits, int ld, float* __restrict__ weights, int ldw,
                                                         int E, int top, int renormalize) {
    int t = blockIdx.x, lane = threadIdx.x;
    constexpr int PER = ROUTE_MAX_EXPERTS / 64;
    float z[PER];
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        int e = lane + 64 * i;
        z[i] = e < E ? logits[(size_t)t * ld + e] : -INFINITY;
        mx = fmaxf(mx, z[i]);
    }
    mx = wave_max(mx);
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        z[i] = (lane + 64 * i) < E ? expf(z[i] - mx) : -1.0f;       // (scores are >= 0: -1 marks what is not there or taken)
        sum += fmaxf(z[i], 0.0f);
    }
    float inv = 1.0f / wave_sum(sum);
    float keep[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) keep[i] = 0.0f;
    float chosen_sum = 0.0f;
    for (int r = 0; r < top; ++r) {
        float best = -1.0f;
        int at = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (z[i] > best) { best = z[i]; at = lane + 64 * i; }      // ascending index within a lane: the first of equals stays
        // the wave's best: the largest score, of equal scores the lowest index
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) {
            float ob = __shfl_xor(best, d, 64);
            int oa = __shfl_xor(at, d, 64);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
        if (best < 0.0f) break;
        chosen_sum += best * inv;
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (lane + 64 * i == at) { keep[i] = z[i] * inv; z[i] = -1.0f; }
    }
    float norm = renormalize ? 1.0f / chosen_sum : 1.0f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        int e = lane + 64 * i;
        if (e < E) weights[(size_t)t * ldw + e] = keep[i] * norm;
    }
}

extern "C" int llmrs_route_topk(hipStream_t stream, const float* logits, int ld, float* weights, int ldw, int n_tokens, int E, int top,
                                int renormalize) {
    LLMRS_REQUIRE(logits && weights && E > 0 && top > 0 && top <= E && ld >= E && ldw >= E, "route_topk: bad arguments");
    LLMRS_REQUIRE(E <= ROUTE_MAX_EXPERTS, "route_topk: %d experts exceed %d", E, ROUTE_MAX_EXPERTS);
    if (n_tokens <= 0) return 0;
    route_topk_kernel<<<n_tokens, 64, 0, stream>>>(logits, ld, weights, ldw, E, top, renormalize);
    LLMRS_LAUNCH_CHECK("route_topk");
    return 0;
}

// out[t, c] = act(up[t, c]) * (weights ? weights[t, c / ff] : 1), act = relu(x)^2 (kind 0); up 32-bit sums, out in the
// activation type (one rounding).
template <class T>
__global__ void act_weight_kernel(const float* __restrict__ up, int ldu, const float* __restrict__ weights, int ldw, int ff, int n,
                                  long total, T* __restrict__ out, int ldo) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    long t = i / n;
    int c = (int)(i - t * n);
    float x = fmaxf(up[(size_t)t * ldu + c], 0.0f);
    float y = x * x;
    if (weights) y *= weights[(size_t)t * ldw + c / ff];
    out[(size_t)t * ldo + c] = from_f32<T>(y);
}

extern "C" int llmrs_act_weight(hipStream_t stream, int dtype, const float* up, int ldu, const float* weights, int ldw, int ff,
                                int n_tokens, int n, int kind, void* out, int ldo) {
    LLMRS_REQUIRE(up && out && n > 0 && ldu >= n && ldo >= n && ff > 0 && n % ff == 0, "act_weight: bad arguments");
    LLMRS_REQUIRE(kind == 0, "act_weight: unknown activation %d (0: squared relu)", kind);
    LLMRS_REQUIRE(!weights || ldw >= n / ff, "act_weight: the weights' rows are too short");
    long total = (long)n_tokens * n;
    if (total <= 0) return 0;
    LLMRS_REQUIRE(ceil_div(total, 256) <= 0x7fffffff, "act_weight: too many elements for one launch");
    int blocks = ceil_div(total, 256);
    if (dtype == LLMRS_F32)
        act_weight_kernel<float><<<blocks, 256, 0, stream>>>(up, ldu, weights, ldw, ff, n, total, (float*)out, ldo);
    else if (dtype == LLMRS_BF16)
        act_weight_kernel<bf16><<<blocks, 256, 0, stream>>>(up, ldu, weights, ldw, ff, n, total, (bf16*)out, ldo);
    else
        return llmrs_fail("act_weight: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("act_weight");
    return 0;
}
