// Layer norm over the float32 residual stream, fused with the residual sum:
//   v = residual + delta_a + delta_b        (each delta: absent, one array of the activations' type, or float32
//                                            partial sums that are added in order; the sum in float32)
//   y1 = (v - mean) / sqrt(var + eps) * w1 + b1,   y2 = the same with w2, b2 (optional)
// mean and variance (the mean of the squared deviations) in float32, from the row held in registers.  Two
// deltas are what a block leaves whose mixer and feed-forward read the same stream; two outputs are what such a
// block asks for: its two norms differ in weight and bias only, so the statistics are computed once.
#include "common.h"
#include "api.h"

namespace {

constexpr int kMaxPer = 4;  // groups of V values a thread holds

template <typename T>
struct Delta {
    const void* p;
    int parts;  // 0: one array of T; n >= 1: n float32 arrays
};

template <typename T, int V>
__device__ __forceinline__ void add_delta(float (&v)[V], const Delta<T>& d, int64_t at, int64_t plane) {
    if (!d.p) return;
    if (d.parts == 0) {
        const T* x = static_cast<const T*>(d.p) + at;
#pragma unroll
        for (int i = 0; i < V; ++i) v[i] += to_float(x[i]);
    } else {
        const float* x = static_cast<const float*>(d.p) + at;
        for (int s = 0; s < d.parts; ++s) {
#pragma unroll
            for (int i = 0; i < V; ++i) v[i] += x[s * plane + i];
        }
    }
}

template <typename T, int V>
__device__ __forceinline__ void store_row(T* out, const float (&y)[V]) {
#pragma unroll
    for (int i = 0; i < V; ++i) out[i] = from_float<T>(y[i]);
}

template <typename T, int V>
__global__ __launch_bounds__(1024) void layer_norm_kernel(float* __restrict__ residual, Delta<T> da, Delta<T> db,
                                                          const float* __restrict__ w1, const float* __restrict__ b1,
                                                          T* __restrict__ out1, const float* __restrict__ w2,
                                                          const float* __restrict__ b2, T* __restrict__ out2,
                                                          const int32_t* __restrict__ rows, int hidden, float eps,
                                                          int write_back, int64_t plane) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const int64_t row = rows ? rows[r] : r;
    float* res = residual + row * hidden;
    const int groups = hidden / V;
    float v[kMaxPer][V];
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < kMaxPer; ++k) {
        const int g = threadIdx.x + k * blockDim.x;
        if (g < groups) {
#pragma unroll
            for (int i = 0; i < V; ++i) v[k][i] = res[g * V + i];
            add_delta<T, V>(v[k], da, row * hidden + g * V, plane);
            add_delta<T, V>(v[k], db, row * hidden + g * V, plane);
            if (write_back) {
#pragma unroll
                for (int i = 0; i < V; ++i) res[g * V + i] = v[k][i];
            }
#pragma unroll
            for (int i = 0; i < V; ++i) sum += v[k][i];
        }
    }
    const float mean = block_sum(sum, scratch) / static_cast<float>(hidden);
    float sq = 0.f;
#pragma unroll
    for (int k = 0; k < kMaxPer; ++k) {
        const int g = threadIdx.x + k * blockDim.x;
        if (g < groups) {
#pragma unroll
            for (int i = 0; i < V; ++i) {
                v[k][i] -= mean;
                sq = fmaf(v[k][i], v[k][i], sq);
            }
        }
    }
    const float inv = 1.0f / sqrtf(block_sum(sq, scratch) / static_cast<float>(hidden) + eps);
#pragma unroll
    for (int k = 0; k < kMaxPer; ++k) {
        const int g = threadIdx.x + k * blockDim.x;
        if (g < groups) {
            float y[V];
#pragma unroll
            for (int i = 0; i < V; ++i) y[i] = fmaf(v[k][i] * inv, w1[g * V + i], b1[g * V + i]);
            store_row<T, V>(out1 + static_cast<int64_t>(r) * hidden + g * V, y);
            if (out2) {
#pragma unroll
                for (int i = 0; i < V; ++i) y[i] = fmaf(v[k][i] * inv, w2[g * V + i], b2[g * V + i]);
                store_row<T, V>(out2 + static_cast<int64_t>(r) * hidden + g * V, y);
            }
        }
    }
}

}  // namespace

extern "C" int fsie_layer_norm(float* residual, const void* delta_a, int parts_a, const void* delta_b, int parts_b,
                               const float* w1, const float* b1, void* out1, const float* w2, const float* b2, void* out2,
                               const int32_t* rows, int n_rows, int hidden, float eps, int dtype, int write_back,
                               int total_rows, hipStream_t stream) {
    FSIE_REQUIRE(n_rows >= 0 && hidden > 0 && total_rows >= 0, "layer_norm: bad sizes rows=%d hidden=%d", n_rows, hidden);
    FSIE_REQUIRE(residual && w1 && b1 && out1, "layer_norm: missing operand");
    FSIE_REQUIRE(!out2 || (w2 && b2), "layer_norm: a second output needs its weight and bias");
    FSIE_REQUIRE(parts_a >= 0 && parts_a <= FSIE_GEMM_MAX_SPLITS && parts_b >= 0 && parts_b <= FSIE_GEMM_MAX_SPLITS,
                 "layer_norm: at most %d partial sums a delta", FSIE_GEMM_MAX_SPLITS);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "layer_norm: unknown dtype %d", dtype);
    FSIE_REQUIRE(!(rows && write_back), "layer_norm: chosen rows are not written back");
    if (n_rows == 0) return 0;
    const int vec = hidden % 4 == 0 ? 4 : 1;
    const int groups = hidden / vec;
    const int threads = groups <= 256 * kMaxPer ? 256 : 1024;
    FSIE_REQUIRE(groups <= threads * kMaxPer, "layer_norm: hidden %d is wider than the kernel holds (%d)", hidden,
                 1024 * kMaxPer * vec);
    const int64_t plane = static_cast<int64_t>(total_rows) * hidden;
#define FSIE_LN(T, V)                                                                                              \
    layer_norm_kernel<T, V><<<n_rows, threads, 0, stream>>>(residual, Delta<T>{delta_a, parts_a}, Delta<T>{delta_b, parts_b}, \
                                                            w1, b1, static_cast<T*>(out1), w2, b2, static_cast<T*>(out2),  \
                                                            rows, hidden, eps, write_back, plane)
    if (dtype == FSIE_F32) {
        if (vec == 4) FSIE_LN(float, 4); else FSIE_LN(float, 1);
    } else {
        if (vec == 4) FSIE_LN(bf16_t, 4); else FSIE_LN(bf16_t, 1);
    }
#undef FSIE_LN
    FSIE_CHECK_LAUNCH("layer_norm");
    return 0;
}
