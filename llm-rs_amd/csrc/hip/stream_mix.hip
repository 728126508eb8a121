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

__device__ __forceinline__ void store4(float* p, const float (&v)[4]) { *(float4*)p = make_float4(v[0], v[1], v[2], v[3]); }
__device__ __forceinline__ void store4(bf16* p, const float (&v)[4]) {
    typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
    bf16x4_t t;
#pragma unroll
    for (int j = 0; j < 4; ++j) t[j] = (bf16)v[j];
    *(bf16x4_t*)p = t;
}

// One block per output row.  The combined row lives in LDS between the sums of squares and the scaling.
// MIX: what a sublayer gave (y) goes into the streams first, as streams_mix_kernel does it and with the same sums in
// the same order; the row that is normed is combined from the new streams, which are written back on the way.
// SMAX: a bound of n_streams that the loops over streams are unrolled to.  A thread takes four neighbouring
// features at a time where rows are a multiple of four long (`wide`), else one.
template <class T, bool MIX, int SMAX>
__global__ void group_rmsnorm_kernel(T* __restrict__ out, float* __restrict__ x, size_t stream_stride, int n_streams,
                                     const float* __restrict__ w_in, const float* __restrict__ weight,
                                     const int* __restrict__ rows, int D, int groups, float eps,
                                     float* zero, float* __restrict__ combined,
                                     const float* __restrict__ mix, const float* __restrict__ w_out, const float* y, int wide) {
    extern __shared__ float row[];           // [D], then [groups] inverse roots, then [16] partial sums, then the mix
    float* inv = row + D;
    float* partial = inv + groups;
    float* m = partial + 16;                 // [MAX_STREAMS * MAX_STREAMS] mix, [MAX_STREAMS] w_out
    int r = rows ? rows[blockIdx.x] : blockIdx.x;
    float* src = x + (size_t)r * D;
    if (MIX) {
        for (int i = threadIdx.x; i < n_streams * n_streams; i += blockDim.x) m[i] = mix[i];
        for (int i = threadIdx.x; i < n_streams; i += blockDim.x) m[MAX_STREAMS * MAX_STREAMS + i] = w_out[i];
        __syncthreads();
    }
    bool plain = n_streams == 1 && w_in == nullptr;
    int each = wide ? 4 : 1;
    for (int d = threadIdx.x * each; d < D; d += blockDim.x * each) {
        float v[SMAX][4];                       // (every stream's values are asked for before the first is used)
#pragma unroll
        for (int s = 0; s < SMAX; ++s) {
            v[s][0] = v[s][1] = v[s][2] = v[s][3] = 0.0f;
            if (s < n_streams) {
                if (wide) load4(src + (size_t)s * stream_stride + d, v[s]);
                else v[s][0] = src[(size_t)s * stream_stride + d];
            }
        }
        if (MIX) {
            float yy[4] = {0.0f, 0.0f, 0.0f, 0.0f}, old[SMAX][4];
            if (wide) load4(y + (size_t)r * D + d, yy);
            else yy[0] = y[(size_t)r * D + d];
#pragma unroll
            for (int s = 0; s < SMAX; ++s)
#pragma unroll
                for (int j = 0; j < 4; ++j) old[s][j] = v[s][j];
#pragma unroll
            for (int to = 0; to < SMAX; ++to) {
                if (to < n_streams) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        float nv = m[to] * old[0][j];
#pragma unroll
                        for (int s = 1; s < SMAX; ++s)
                            if (s < n_streams) nv = fmaf(m[s * n_streams + to], old[s][j], nv);
                        v[to][j] = fmaf(m[MAX_STREAMS * MAX_STREAMS + to], yy[j], nv);
                    }
                    if (wide) store4(src + (size_t)to * stream_stride + d, v[to]);
                    else src[(size_t)to * stream_stride + d] = v[to][0];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float u = plain ? v[0][j] : (w_in ? w_in[0] : 1.0f) * v[0][j];
#pragma unroll
            for (int s = 1; s < SMAX; ++s)
                if (s < n_streams) u = fmaf(w_in ? w_in[s] : 1.0f, v[s][j], u);
            if (j < each) row[d + j] = u;
        }
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
    for (int d = threadIdx.x * each; d < D; d += blockDim.x * each) {
        float o[4], c[4], z[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int dj = j < each ? d + j : d;
            c[j] = row[dj];
            o[j] = c[j] * inv[dj / gs] * weight[dj];
        }
        if (wide) {
            store4(dst + d, o);
            if (zero) store4(zero + (size_t)blockIdx.x * D + d, z);
            if (combined) store4(combined + (size_t)blockIdx.x * D + d, c);
        } else {
            dst[d] = from_f32<T>(o[0]);
            if (zero) zero[(size_t)blockIdx.x * D + d] = 0.0f;
            if (combined) combined[(size_t)blockIdx.x * D + d] = c[0];
        }
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
// mix, w_out, y: if given (all three; no `rows` then), x <- streams_mix(x, mix, w_out, y) first, in the same launch;
// y may be the memory that `zero` clears.
extern "C" int llmrs_group_rmsnorm(hipStream_t stream, int dtype, void* out, float* x, long stream_stride, int n_streams,
                                   const float* w_in, const float* weight, const int* rows, int n_rows, int D, int groups,
                                   float eps, float* zero, float* combined, const float* mix, const float* w_out, const float* y) {
    LLMRS_REQUIRE(n_rows >= 0 && D > 0, "group_rmsnorm: bad sizes rows=%d D=%d", n_rows, D);
    LLMRS_REQUIRE(eps > 0.0f, "group_rmsnorm: eps must be positive, got %g", eps);
    LLMRS_REQUIRE(groups > 0 && groups <= MAX_NORM_GROUPS && D % groups == 0, "group_rmsnorm: %d features do not fall into %d equal groups (at most %d)", D, groups, MAX_NORM_GROUPS);
    LLMRS_REQUIRE(n_streams >= 1 && n_streams <= MAX_STREAMS, "group_rmsnorm: %d streams (at most %d)", n_streams, MAX_STREAMS);
    LLMRS_REQUIRE(D <= 15000, "group_rmsnorm: rows of %d features do not fit the block's memory", D);
    LLMRS_REQUIRE(mix == nullptr || (w_out != nullptr && y != nullptr && rows == nullptr), "group_rmsnorm: a mix needs its weights and every row in place");
    if (n_rows == 0) return 0;
    if (dtype != LLMRS_F32 && dtype != LLMRS_BF16) return llmrs_fail("group_rmsnorm: unknown dtype %d", dtype);
    int wide = D % 4 == 0 && stream_stride % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)y & 15) == 0
               && ((uintptr_t)zero & 15) == 0 && ((uintptr_t)combined & 15) == 0;
    int threads = D > 8192 ? 1024 : D > 2048 ? 512 : 256;
    size_t lds = (size_t)(D + groups + 16 + MAX_STREAMS * MAX_STREAMS + MAX_STREAMS) * sizeof(float);
#define NORM(T, MIX, SMAX) group_rmsnorm_kernel<T, MIX, SMAX><<<n_rows, threads, lds, stream>>>((T*)out, x, (size_t)stream_stride, n_streams, w_in, weight, \
                                                                                          rows, D, groups, eps, zero, combined, mix, w_out, y, wide)
#define BY_STREAMS(T, MIX) do { if (n_streams <= 4) NORM(T, MIX, 4); else NORM(T, MIX, MAX_STREAMS); } while (0)
    if (dtype == LLMRS_F32) { if (mix) BY_STREAMS(float, true); else BY_STREAMS(float, false); }
    else { if (mix) BY_STREAMS(bf16, true); else BY_STREAMS(bf16, false); }
#undef BY_STREAMS
#undef NORM
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
