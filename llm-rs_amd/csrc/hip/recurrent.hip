// Recurrent mixers: a gated recurrence whose gates read only the current token (minGRU), and a selective
// state-space scan with its short causal convolution.  Each request's state lives in 32-bit in the row of its slot
// and is carried from step to step; an entry's tokens are walked in order from the state the step before left.
// Everything that enters a recurrence is 32-bit: gates, decays, step sizes, exponentials and the state itself.
//
// A step's entries are given as on every kernel of the engine: q_starts [n_entries + 1] (where each entry's tokens
// start among the step's rows) and slots [n_entries] (the state row of each entry's request).
#include "common.h"

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_f32(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// ---- minGRU ---------------------------------------------------------------------------------------------------
// sums: [T, ld] 32-bit, per token the projections' sums (gate | candidate | output gate), each W wide.
//   z = sigmoid(sums_z + bias_z);  u = sums_c + bias_c;  c = u + 1/2 where u >= 0, sigmoid(u) elsewhere
//   s <- (1 - z) s + z c;  out = s * silu(sums_g)
// One thread for each (entry, channel).
template <class T>
__global__ void mingru_scan_kernel(const float* __restrict__ sums, int ld, const float* __restrict__ bias_z,
                                   const float* __restrict__ bias_c, float* __restrict__ state, long state_stride,
                                   const int* __restrict__ q_starts, const int* __restrict__ slots, int W,
                                   T* __restrict__ out, int ldo) {
    int c = blockIdx.x * blockDim.x + threadIdx.x, e = blockIdx.y;
    if (c >= W) return;
    int t0 = q_starts[e], t1 = q_starts[e + 1];
    float* sp = state + (size_t)slots[e] * state_stride + c;
    float s = *sp, bz = bias_z ? bias_z[c] : 0.0f, bc = bias_c ? bias_c[c] : 0.0f;
    for (int t = t0; t < t1; ++t) {
        const float* row = sums + (size_t)t * ld;
        float z = sigmoid_f32(row[c] + bz);
        float u = row[W + c] + bc;
        float cand = u >= 0.0f ? u + 0.5f : sigmoid_f32(u);
        s = (1.0f - z) * s + z * cand;
        out[(size_t)t * ldo + c] = from_f32<T>(s * silu_f32(row[2 * W + c]));
    }
    *sp = s;
}

// ---- short causal convolution -------------------------------------------------------------------------------------
// y[t, c] = silu(bias[c] + sum_j taps[c, j] * x[t - (K - 1 - j), c]): the last tap weighs the current token.  Inputs
// from before the step's first token come from the request's state (its last K - 1 inputs, oldest first), which is
// zero at the start of a sequence.  x: the first C columns of `sums` [T, ld], 32-bit.
template <class T>
__global__ void causal_conv_silu_kernel(const float* __restrict__ sums, int ld, const float* __restrict__ taps,
                                        const float* __restrict__ bias, const float* __restrict__ state, long state_stride,
                                        const int* __restrict__ q_starts, const int* __restrict__ slots,
                                        const int* __restrict__ token_entry, int C, int K, T* __restrict__ out, int ldo) {
    int c = blockIdx.x * blockDim.x + threadIdx.x, t = blockIdx.y;
    if (c >= C) return;
    int e = token_entry[t];
    int i = t - q_starts[e];                    // the token's place in its entry
    const float* sp = state + (size_t)slots[e] * state_stride;
    float acc = bias ? bias[c] : 0.0f;
    for (int j = 0; j < K; ++j) {
        int back = K - 1 - j;                   // how many tokens before this one
        float x = i - back >= 0 ? sums[(size_t)(t - back) * ld + c] : sp[(size_t)(K - 1 + i - back) * C + c];
        acc = fmaf(taps[(size_t)c * K + j], x, acc);
    }
    out[(size_t)t * ldo + c] = from_f32<T>(silu_f32(acc));
}

// After the convolution: the state becomes the last K - 1 inputs of (old state, this step's inputs).
__global__ void causal_conv_state_kernel(const float* __restrict__ sums, int ld, float* __restrict__ state, long state_stride,
                                         const int* __restrict__ q_starts, const int* __restrict__ slots, int C, int K) {
    int c = blockIdx.x * blockDim.x + threadIdx.x, e = blockIdx.y;
    if (c >= C) return;
    int t0 = q_starts[e], n = q_starts[e + 1] - t0;
    float* sp = state + (size_t)slots[e] * state_stride;
    for (int m = 0; m < K - 1; ++m) {           // ascending: a row is read before a lower one overwrites nothing it needs
        int i = n - (K - 1) + m;                // place in the entry of what row m holds afterwards
        sp[(size_t)m * C + c] = i >= 0 ? sums[(size_t)(t0 + i) * ld + c] : sp[(size_t)(m + n) * C + c];
    }
}

// ---- selective scan -----------------------------------------------------------------------------------------------
// Per channel c and state n, with step = softplus(dt[t, c] + dt_bias[c]) and A[c, n] < 0:
//   S[c, n] <- exp(step A[c, n]) S[c, n] + step x[t, c] B[t, n];   y = sum_n S[c, n] C[t, n] + D[c] x[t, c]
//   out[t, c] = y * silu(gate[t, c])
// One thread for each (entry, channel) holds NS states in registers; a channel with more states is walked in
// passes of NS, the partial y of earlier passes waiting in `ypart` [T, C] 32-bit.
struct ScanArgs {
    const float* dt; int ld_dt;          // [T, C] sums of the step projection, 32-bit
    const float* dt_bias;                // [C]
    const float* A;                      // [C, N], negative
    const float* D;                      // [C]
    const float* gate; int ld_gate;      // [T, C] 32-bit (the projection's second half)
    float* state; long state_stride;     // [slots][C][N]
    float* ypart;                        // [T, C], needed when N > NS
    int C, N;
};

template <class T, int NS>
__global__ void selective_scan_kernel(const T* __restrict__ x, int ldx, const T* __restrict__ bc, int ldbc, int off_b,
                                      int off_c, const int* __restrict__ q_starts, const int* __restrict__ slots,
                                      T* __restrict__ out, int ldo, ScanArgs a) {
    int c = blockIdx.x * blockDim.x + threadIdx.x, e = blockIdx.y;
    if (c >= a.C) return;
    int t0 = q_starts[e], t1 = q_starts[e + 1];
    float* sp = a.state + (size_t)slots[e] * a.state_stride + (size_t)c * a.N;
    float bias = a.dt_bias ? a.dt_bias[c] : 0.0f, Dc = a.D[c];
    for (int n0 = 0; n0 < a.N; n0 += NS) {
        bool first = n0 == 0, last = n0 + NS >= a.N;
        float S[NS], Ac[NS];
#pragma unroll
        for (int n = 0; n < NS; ++n) {
            bool in = n0 + n < a.N;
            S[n] = in ? sp[n0 + n] : 0.0f;
            Ac[n] = in ? a.A[(size_t)c * a.N + n0 + n] : 0.0f;
        }
        for (int t = t0; t < t1; ++t) {
            float step = softplus_f32(a.dt[(size_t)t * a.ld_dt + c] + bias);
            float xv = to_f32(x[(size_t)t * ldx + c]);
            float sx = step * xv;
            const T* Bt = bc + (size_t)t * ldbc + off_b + n0;
            const T* Ct = bc + (size_t)t * ldbc + off_c + n0;
            float y = 0.0f;
#pragma unroll
            for (int n = 0; n < NS; ++n) {
                if (n0 + n < a.N) {
                    S[n] = fmaf(expf(step * Ac[n]), S[n], sx * to_f32(Bt[n]));
                    y = fmaf(S[n], to_f32(Ct[n]), y);
                }
            }
            if (!first) y += a.ypart[(size_t)t * a.C + c];
            if (!last) { a.ypart[(size_t)t * a.C + c] = y; continue; }
            y = fmaf(Dc, xv, y);
            out[(size_t)t * ldo + c] = from_f32<T>(y * silu_f32(a.gate[(size_t)t * a.ld_gate + c]));
        }
#pragma unroll
        for (int n = 0; n < NS; ++n)
            if (n0 + n < a.N) sp[n0 + n] = S[n];
    }
}

static bool entries_ok(const int* q_starts, const int* slots, int n_entries) { return q_starts && slots && n_entries >= 0 && n_entries <= 65535; }

extern "C" int llmrs_mingru_scan(hipStream_t stream, int dtype, const float* sums, int ld, const float* bias_z,
                                 const float* bias_c, float* state, long state_stride, const int* q_starts, const int* slots,
                                 int n_entries, int W, void* out, int ldo) {
    LLMRS_REQUIRE(W > 0 && ld >= 3 * W && ldo >= W && state_stride >= W, "mingru_scan: bad sizes");
    LLMRS_REQUIRE(entries_ok(q_starts, slots, n_entries), "mingru_scan: bad entries");
    if (n_entries == 0) return 0;
    dim3 grid(ceil_div(W, 64), n_entries);
    if (dtype == LLMRS_F32)
        mingru_scan_kernel<float><<<grid, 64, 0, stream>>>(sums, ld, bias_z, bias_c, state, state_stride, q_starts, slots, W, (float*)out, ldo);
    else if (dtype == LLMRS_BF16)
        mingru_scan_kernel<bf16><<<grid, 64, 0, stream>>>(sums, ld, bias_z, bias_c, state, state_stride, q_starts, slots, W, (bf16*)out, ldo);
    else
        return llmrs_fail("mingru_scan: unknown dtype %d", dtype);
    LLMRS_LAUNCH_CHECK("mingru_scan");
    return 0;
}

// The convolution of a step's tokens and then the new state.  state: [slots][K - 1][C] at state_stride floats a slot.
extern "C" int llmrs_causal_conv_silu(hipStream_t stream, int dtype, const float* sums, int ld, const float* taps,
                                      const float* bias, float* state, long state_stride, const int* q_starts,
                                      const int* slots, const int* token_entry, int n_entries, int n_tokens, int C, int K,
                                      void* out, int ldo) {
    LLMRS_REQUIRE(C > 0 && K >= 1 && ld >= C && ldo >= C && state_stride >= (long)(K - 1) * C, "causal_conv: bad sizes");
    LLMRS_REQUIRE(entries_ok(q_starts, slots, n_entries) && token_entry && n_tokens >= 0 && n_tokens <= 65535 * 32, "causal_conv: bad entries");
    if (n_tokens == 0) return 0;
    LLMRS_REQUIRE(n_tokens <= 65535, "causal_conv: %d tokens are too many for one launch", n_tokens);
    dim3 grid(ceil_div(C, 64), n_tokens);
    if (dtype == LLMRS_F32)
        causal_conv_silu_kernel<float><<<grid, 64, 0, stream>>>(sums, ld, taps, bias, state, state_stride, q_starts, slots, token_entry, C, K, (float*)out, ldo);
    else if (dtype == LLMRS_BF16)
        causal_conv_silu_kernel<bf16><<<grid, 64, 0, stream>>>(sums, ld, taps, bias, state, state_stride, q_starts, slots, token_entry, C, K, (bf16*)out, ldo);
    else
        return llmrs_fail("causal_conv: unknown dtype %d", dtype);
    if (K > 1)
        causal_conv_state_kernel<<<dim3(ceil_div(C, 64), n_entries), 64, 0, stream>>>(sums, ld, state, state_stride, q_starts, slots, C, K);
    LLMRS_LAUNCH_CHECK("causal_conv");
    return 0;
}

// x: [T, ldx] the convolution's output; bc: [T, ldbc] with B at column off_b and C at off_c, N wide each; both and
// `out` in `dtype`.  ypart: [T, C] 32-bit, needed only when N > 64.
extern "C" int llmrs_selective_scan(hipStream_t stream, int dtype, const void* x, int ldx, const void* bc, int ldbc, int off_b,
                                    int off_c, const float* dt, int ld_dt, const float* dt_bias, const float* A, const float* D,
                                    const float* gate, int ld_gate, float* state, long state_stride, float* ypart,
                                    const int* q_starts, const int* slots, int n_entries, int C, int N, void* out, int ldo) {
    LLMRS_REQUIRE(C > 0 && N > 0 && ldx >= C && ld_dt >= C && ld_gate >= C && ldo >= C && state_stride >= (long)C * N, "selective_scan: bad sizes");
    LLMRS_REQUIRE(off_b >= 0 && off_c >= 0 && ldbc >= off_b + N && ldbc >= off_c + N, "selective_scan: B and C do not fit their rows");
    LLMRS_REQUIRE(entries_ok(q_starts, slots, n_entries), "selective_scan: bad entries");
    LLMRS_REQUIRE(N <= 64 || ypart != nullptr, "selective_scan: %d states a channel need room for partial sums", N);
    if (n_entries == 0) return 0;
    ScanArgs a{dt, ld_dt, dt_bias, A, D, gate, ld_gate, state, state_stride, ypart, C, N};
    dim3 grid(ceil_div(C, 64), n_entries);
#define SCAN(T, NS) selective_scan_kernel<T, NS><<<grid, 64, 0, stream>>>((const T*)x, ldx, (const T*)bc, ldbc, off_b, off_c, q_starts, slots, (T*)out, ldo, a)
#define BY_STATES(T) do { if (N <= 8) SCAN(T, 8); else if (N <= 16) SCAN(T, 16); else if (N <= 32) SCAN(T, 32); else SCAN(T, 64); } while (0)
    if (dtype == LLMRS_F32) BY_STATES(float);
    else if (dtype == LLMRS_BF16) BY_STATES(bf16);
    else return llmrs_fail("selective_scan: unknown dtype %d", dtype);
#undef BY_STATES
#undef SCAN
    LLMRS_LAUNCH_CHECK("selective_scan");
    return 0;
}
