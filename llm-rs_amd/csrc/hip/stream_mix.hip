// A residual stream kept as several copies ("streams") that small matrices mix, and the RMS norm in groups that
// reads them.
//
// The streams lie as [n_streams][T][D], 32-bit.  A sublayer reads one vector per token,
//     u[t, :] = sum_s w_in[s] * X[s][t, :]            (w_in null: every weight 1, the plain sum)
// normed in groups: D is cut into `groups` equal consecutive parts, each part p becomes p / sqrt(mean(p^2) + eps),
// and the whole is multiplied by the norm's weight.  What the sublayer gives, y[t, :], goes back into every stream
// together with a mix of the old streams:
//     X'[r][t, :] = sum_s mix[s, r] * X[s][t, :] + w_out[r] * y[t, :]
// All sums are 32-bit and in a fixed order (streams ascending; a group's squares in an order that depends on D, the
// group count and the block size only), so a token's row does not depend on the batch it is in.
#include "common.h"

#define MAX_STREAMS 16
#define MAX_NORM_GROUPS 64

struct StreamWeights {
    float w[MAX_STREAMS];
};

// One block per output row.  The combined row lives in LDS between the sums of squares and the scaling.
template <class T>
__global__ void group_rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ x, size_t stream_stride, int n_streams,
                                     const float* __restrict__ w_in, const float* __restrict__ weight,
                                     const int* __restrict__ rows, int D, int groups, float eps,
                                     float* __restrict__ zero, float* __restrict__ combined) {
    extern __shared__ float row[];           // [D], then [groups] inverse roots, then [16] partial sums
    float* inv = row + D;
    float* partial = inv + groups;
    int r = rows ? rows[blockIdx.x] : blockIdx.x;
    const float* src = x + (size_t)r * D;
    bool plain = n_streams == 1 && w_in == nullptr;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float v[MAX_STREAMS];                   // (every stream's value is asked for before the first is used)
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s) v[s] = s < n_streams ? src[(size_t)s * stream_stride + d] : 0.0f;
        float u = plain ? v[0] : (w_in ? w_in[0] : 1.0f) * v[0];
#pragma unroll
        for (int s = 1; s < MAX_STREAMS; ++s)
            if (s < n_streams) u = fmaf(w_in ? w_in[s] : 1.0f, v[s], u);
        row[d] = u;
    }
    __syncthreads();
    int gs = D / groups, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    for (int g = 0; g < groups; ++g) {
        float ss = 0.0f;
        for (int d = threadIdx.x; d < gs; d += blockDim.x) {
            float v = row[g * gs + d];
            ss = fmaf(v, v, ss);
        }
        ss = wave_sum(ss);
        if ((threadIdx.x & 63) == 0) partial[wave] = ss;
        __syncthreads();
        if (threadIdx.x == 0) {
            float total = 0.0f;
            for (int i = 0; i < nwaves; ++i) total += partial[i];
            inv[g] = 1.0f / sqrtf(total / (float)gs + eps);
        }
        __syncthreads();
    }
    T* dst = out + (size_t)blockIdx.x * D;
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        dst[d] = from_f32<T>(row[d] * inv[d / gs] * weight[d]);
        if (zero) zero[(size_t)blockIdx.x * D + d] = 0.0f;
        if (combined) combined[(size_t)blockIdx.x * D + d] = row[d];
    }
}

// X'[r] = sum_s mix[s][r] X[s] + w_out[r] y, in place: a thread reads one feature of every stream, then writes them.
__global__ void streams_mix_kernel(float* __restrict__ x, size_t stream_stride, int n_streams, const float* __restrict__ mix,
                                   const float* __restrict__ w_out, const float* __restrict__ y, size_t n) {
    __shared__ float m[MAX_STREAMS * MAX_STREAMS + MAX_STREAMS];
    for (int i = threadIdx.x; i < n_streams * n_streams; i += blockDim.x) m[i] = mix[i];
    for (int i = threadIdx.x; i < n_streams; i += blockDim.x) m[MAX_STREAMS * MAX_STREAMS + i] = w_out[i];
    __syncthreads();
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float old[MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < MAX_STREAMS; ++s) old[s] = s < n_streams ? x[(size_t)s * stream_stride + i] : 0.0f;
    float yy = y[i];
#pragma unroll
    for (int r = 0; r < MAX_STREAMS; ++r) {
        if (r < n_streams) {
            float v = m[r] * old[0];
#pragma unroll
            for (int s = 1; s < MAX_STREAMS; ++s)
                if (s < n_streams) v = fmaf(m[s * n_streams + r], old[s], v);
            x[(size_t)r * stream_stride + i] = fmaf(m[MAX_STREAMS * MAX_STREAMS + r], yy, v);
        }
    }
}

// Every stream starts as a copy of the first.
__global__ void streams_copy_first_kernel(float* __restrict__ x, size_t stream_stride, int n_streams, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float v = x[i];
    for (int s = 1; s < n_streams; ++s) x[(size_t)s * stream_stride + i] = v;
}

// out[i, :] = weight * groupnorm(sum_s w_in[s] x[s][rows[i] or i, :]) in the type `dtype` says.
// zero: if given, [n_rows, D] 32-bit that is cleared on the way (room for a sublayer to add its result into);
// combined: if given, [n_rows, D] 32-bit that gets the combined rows before the norm.
extern "C" int llmrs_group_rmsnorm(hipStream_t stream, int dtype, void* out, const float* x, long stream_stride, int n_streams,
                                   const float* w_in, const float* weight, const int* rows, int n_rows, int D, int groups,
                                   float eps, float* zero, float* combined) {
    LLMRS_REQUIRE(n_rows >= 0 && D > 0, "group_rmsnorm: bad sizes rows=%d D=%d", n_rows, D);
    LLMRS_REQUIRE(eps > 0.0f, "group_rmsnorm: eps must be positive, got %g", eps);
    LLMRS_REQUIRE(groups > 0 && groups <= MAX_NORM_GROUPS && D % groups == 0, "group_rmsnorm: %d features do not fall into %d equal groups (at most %d)", D, groups, MAX_NORM_GROUPS);
    LLMRS_REQUIRE(n_streams >= 1 && n_streams <= MAX_STREAMS, "group_rmsnorm: %d streams (at most %d)", n_streams, MAX_STREAMS);
    LLMRS_REQUIRE(D <= 15360, "group_rmsnorm: rows of %d features do not fit the block's memory", D);
    if (n_rows == 0) return 0;
    if (dtype != LLMRS_F32 && dtype != LLMRS_BF16) return llmrs_fail("group_rmsnorm: unknown dtype %d", dtype);
    int threads = D > 4096 ? 1024 : 256;
    size_t lds = (size_t)(D + groups + 16) * sizeof(float);
    if (dtype == LLMRS_F32)
        group_rmsnorm_kernel<float><<<n_rows, threads, lds, stream>>>((float*)out, x, (size_t)stream_stride, n_streams, w_in, weight,
                                                                      rows, D, groups, eps, zero, combined);
    else
        group_rmsnorm_kernel<bf16><<<n_rows, threads, lds, stream>>>((bf16*)out, x, (size_t)stream_stride, n_streams, w_in, weight,
                                                                     rows, D, groups, eps, zero, combined);
    LLMRS_LAUNCH_CHECK("group_rmsnorm");
    return 0;
}

// x: [n_streams][n] with stream_stride floats between streams; mix: [n_streams][n_streams] indexed [from][to];
// w_out: [n_streams]; y: [n].
extern "C" int llmrs_streams_mix(hipStream_t stream, float* x, long stream_stride, int n_streams, const float* mix,
                                 const float* w_out, const float* y, long n) {
    LLMRS_REQUIRE(n_streams >= 1 && n_streams <= MAX_STREAMS, "streams_mix: %d streams (at most %d)", n_streams, MAX_STREAMS);
    LLMRS_REQUIRE(n >= 0 && stream_stride >= n, "streams_mix: bad sizes");
    if (n == 0) return 0;
    streams_mix_kernel<<<ceil_div(n, 256), 256, 0, stream>>>(x, (size_t)stream_stride, n_streams, mix, w_out, y, (size_t)n);
    LLMRS_LAUNCH_CHECK("streams_mix");
    return 0;
}

extern "C" int llmrs_streams_copy_first(hipStream_t stream, float* x, long stream_stride, int n_streams, long n) {
    LLMRS_REQUIRE(n_streams >= 1 && n >= 0 && stream_stride >= n, "streams_copy_first: bad sizes");
    if (n == 0 || n_streams == 1) return 0;
    streams_copy_first_kernel<<<ceil_div(n, 256), 256, 0, stream>>>(x, (size_t)stream_stride, n_streams, (size_t)n);
    LLMRS_LAUNCH_CHECK("streams_copy_first");
    return 0;
}
