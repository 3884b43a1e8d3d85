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

// V consecutive values as floats: one 16-byte (float32) or 8-byte (bfloat16) load where V = 4
template <int V>
__device__ __forceinline__ void load_values(const float* p, float (&f)[V]) {
    if constexpr (V == 4) {
        const float4 v = *reinterpret_cast<const float4*>(p);
        f[0] = v.x, f[1] = v.y, f[2] = v.z, f[3] = v.w;
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) f[i] = p[i];
    }
}
template <int V>
__device__ __forceinline__ void load_values(const bf16_t* p, float (&f)[V]) {
    if constexpr (V == 4) {
        const uint2 v = *reinterpret_cast<const uint2*>(p);
        f[0] = __uint_as_float(v.x << 16), f[1] = __uint_as_float(v.x & 0xffff0000u);
        f[2] = __uint_as_float(v.y << 16), f[3] = __uint_as_float(v.y & 0xffff0000u);
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) f[i] = to_float(p[i]);
    }
}

// Partial sums are asked for eight at a time and added in order: a loop that waits for each slice in turn
// costs a trip to memory a slice.
template <typename T, int V>
__device__ __forceinline__ void add_delta(float (&v)[V], const Delta<T>& d, int64_t at, int64_t plane) {
    if (!d.p) return;
    if (d.parts == 0) {
        float f[V];
        load_values<V>(static_cast<const T*>(d.p) + at, f);
#pragma unroll
        for (int i = 0; i < V; ++i) v[i] += f[i];
        return;
    }
    const float* x = static_cast<const float*>(d.p) + at;
    for (int s0 = 0; s0 < d.parts; s0 += 8) {
        float f[8][V];
#pragma unroll
        for (int j = 0; j < 8; ++j) load_values<V>(x + min(s0 + j, d.parts - 1) * plane, f[j]);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (s0 + j < d.parts) {
#pragma unroll
                for (int i = 0; i < V; ++i) v[i] += f[j][i];
            }
        }
    }
}

template <typename T, int V>
__device__ __forceinline__ void store_row(T* out, const float (&y)[V]) {
    if constexpr (V == 4 && sizeof(T) == 2) {
        uint2 w;
        w.x = pack2_bf16(y[0], y[1]);
        w.y = pack2_bf16(y[2], y[3]);
        *reinterpret_cast<uint2*>(out) = w;
    } else if constexpr (V == 4) {
        *reinterpret_cast<float4*>(out) = float4{y[0], y[1], y[2], y[3]};
    } else {
#pragma unroll
        for (int i = 0; i < V; ++i) out[i] = from_float<T>(y[i]);
    }
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
            load_values<V>(res + g * V, v[k]);
            add_delta<T, V>(v[k], da, row * hidden + g * V, plane);
            add_delta<T, V>(v[k], db, row * hidden + g * V, plane);
            if (write_back) store_row<float, V>(res + g * V, v[k]);
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
            float y[V], w[V], b[V];
            load_values<V>(w1 + g * V, w);
            load_values<V>(b1 + g * V, b);
#pragma unroll
            for (int i = 0; i < V; ++i) y[i] = fmaf(v[k][i] * inv, w[i], b[i]);
            store_row<T, V>(out1 + static_cast<int64_t>(r) * hidden + g * V, y);
            if (out2) {
                load_values<V>(w2 + g * V, w);
                load_values<V>(b2 + g * V, b);
#pragma unroll
                for (int i = 0; i < V; ++i) y[i] = fmaf(v[k][i] * inv, w[i], b[i]);
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
    const bool aligned = ((reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(delta_a) |
                           reinterpret_cast<uintptr_t>(delta_b) | reinterpret_cast<uintptr_t>(w1) | reinterpret_cast<uintptr_t>(b1) |
                           reinterpret_cast<uintptr_t>(w2) | reinterpret_cast<uintptr_t>(b2) | reinterpret_cast<uintptr_t>(out1) |
                           reinterpret_cast<uintptr_t>(out2)) & 15) == 0;
    const int vec = hidden % 4 == 0 && aligned ? 4 : 1;
    const int groups = hidden / vec;
    // few rows (decoding): a thread a group, up to 1,024 threads, so that a compute unit has many waves asking
    // memory at once; many rows: 256 threads with several groups each
    int threads = groups <= 256 * kMaxPer ? 256 : 1024;
    if (n_rows <= 128) threads = groups >= 1024 ? 1024 : (groups + 63) / 64 * 64;
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
