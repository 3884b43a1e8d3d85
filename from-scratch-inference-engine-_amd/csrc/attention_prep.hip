// What stands between the fused projection and attention when the heads are normalised, only partly rotated,
// or have values of another size than their keys: one kernel a step and layer.
//
// proj [tokens][stride] holds of every token q (heads * dim from q_off), k (kv_heads * dim from k_off),
// v (kv_heads * vdim from v_off) and, optionally, one gate logit a head (from g_off).  Per token:
//   q, k heads: RMS norm over dim with a weight shared by the heads (q_weight / k_weight, or none), then the
//               first 2 * pairs values turned, value i with value i + pairs, by the step's cosines and sines
//               cos_sin [tokens][pairs][2]; all of it float32
//   v:          (1 - mix) v + mix * v_other where another layer's values of the same token are given
//   gate:       sigmoid of the logits, float32 [tokens][heads]
// q goes to q_out [tokens][heads * D] and k, v into the pools at slots[t], heads of D >= max(dim, vdim) values,
// zeros behind the dim (or vdim) that are used: the attention kernels take one head size for keys and values.
// A second kernel brings attention's result [tokens][heads * D] back to [tokens][heads * vdim], times the gate.
#include "common.h"
#include "api.h"

namespace {

constexpr int kThreads = 256;

// value j of a head's run x[0 .. dim) after norm (factor `scale`, weight w or none) and rotation
template <typename T>
__device__ __forceinline__ float normed_turned(const T* __restrict__ x, int j, float scale, const float* __restrict__ w,
                                               int pairs, const float2* __restrict__ cs) {
    const float a = w ? (to_float(x[j]) * scale) * w[j] : to_float(x[j]);
    if (j >= 2 * pairs) return a;
    const int jp = j < pairs ? j + pairs : j - pairs;
    const float b = w ? (to_float(x[jp]) * scale) * w[jp] : to_float(x[jp]);
    const float2 t = cs[j < pairs ? j : j - pairs];
    return j < pairs ? fmaf(a, t.x, -(b * t.y)) : fmaf(a, t.x, b * t.y);
}

template <typename T>
__global__ __launch_bounds__(kThreads) void attention_prep_kernel(
    const T* __restrict__ proj, int64_t stride, int q_off, int k_off, int v_off, int g_off, int heads, int kv_heads, int dim,
    int vdim, int D, const float* __restrict__ q_weight, const float* __restrict__ k_weight, float eps, int pairs,
    const float2* __restrict__ cos_sin, const T* __restrict__ v_other, int64_t v_other_stride, const float* __restrict__ mix,
    T* __restrict__ q_out, float* __restrict__ gate, const int32_t* __restrict__ slots, T* __restrict__ k_pool,
    T* __restrict__ v_pool, int page_size, int64_t pool_slots) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const T* row = proj + static_cast<int64_t>(t) * stride;
    const float2* cs = cos_sin + static_cast<int64_t>(t) * pairs;
    const int64_t slot = slots ? slots[t] : -1;
    const bool store = k_pool && slot >= 0 && slot < pool_slots;
    const int64_t page = store ? slot / page_size : 0;
    const int off = store ? static_cast<int>(slot - page * page_size) : 0;
    // a wave a head: the query heads, then the key heads
    for (int h = wave; h < heads + kv_heads; h += kThreads / 64) {
        const bool is_q = h < heads;
        const T* x = row + (is_q ? q_off + h * dim : k_off + (h - heads) * dim);
        const float* w = is_q ? q_weight : k_weight;
        float scale = 1.f;
        if (w) {
            float sum = 0.f;
            for (int j = lane; j < dim; j += 64) sum = fmaf(to_float(x[j]), to_float(x[j]), sum);
            scale = 1.0f / sqrtf(wave_sum(sum) / static_cast<float>(dim) + eps);
        }
        if (is_q) {
            T* o = q_out + (static_cast<int64_t>(t) * heads + h) * D;
            for (int j = lane; j < D; j += 64) o[j] = from_float<T>(j < dim ? normed_turned(x, j, scale, w, pairs, cs) : 0.f);
        } else if (store) {
            const int g = h - heads;
            T* o = k_pool + ((page * kv_heads + g) * page_size + off) * D;
            for (int j = lane; j < D; j += 64) o[j] = from_float<T>(j < dim ? normed_turned(x, j, scale, w, pairs, cs) : 0.f);
        }
    }
    if (store) {
        const float lam = (v_other && mix) ? mix[0] : 0.f;
        for (int e = threadIdx.x; e < kv_heads * D; e += kThreads) {
            const int g = e / D, j = e - g * D;
            float v = 0.f;
            if (j < vdim) {
                v = to_float(row[v_off + g * vdim + j]);
                if (v_other) v = fmaf(lam, to_float(v_other[static_cast<int64_t>(t) * v_other_stride + g * vdim + j]), (1.0f - lam) * v);
            }
            v_pool[((page * kv_heads + g) * D + j) * page_size + off] = from_float<T>(v);
        }
    }
    if (gate) {
        for (int h = threadIdx.x; h < heads; h += kThreads)
            gate[static_cast<int64_t>(t) * heads + h] = 1.0f / (1.0f + expf(-to_float(row[g_off + h])));
    }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void gate_heads_kernel(const T* __restrict__ x, int D, const float* __restrict__ gate,
                                                              T* __restrict__ y, int heads, int vdim, int64_t total) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
    if (e >= total) return;
    const int64_t th = e / vdim;  // token * heads + head
    const int j = static_cast<int>(e - th * vdim);
    const float g = gate ? gate[th] : 1.f;
    y[e] = from_float<T>(to_float(x[th * D + j]) * g);
}

}  // namespace

extern "C" int fsie_attention_prep(const void* proj, int64_t stride, int q_off, int k_off, int v_off, int g_off, int heads,
                                   int kv_heads, int dim, int vdim, int D, const float* q_weight, const float* k_weight,
                                   float eps, int pairs, const float* cos_sin, const void* v_other, int64_t v_other_stride,
                                   const float* mix, void* q_out, float* gate, const int32_t* slots, void* k_pool,
                                   void* v_pool, int page_size, int64_t pool_slots, int n_tokens, int dtype,
                                   hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0 && D >= dim && D >= vdim,
                 "attention_prep: bad sizes heads=%d kv=%d dim=%d vdim=%d D=%d", heads, kv_heads, dim, vdim, D);
    FSIE_REQUIRE(pairs >= 0 && 2 * pairs <= dim && (pairs == 0 || cos_sin), "attention_prep: %d rotated pairs in heads of %d",
                 pairs, dim);
    FSIE_REQUIRE(proj && q_out, "attention_prep: missing operand");
    FSIE_REQUIRE(!k_pool || (v_pool && slots && page_size > 0 && pool_slots > 0), "attention_prep: bad page geometry");
    FSIE_REQUIRE(!v_other || mix, "attention_prep: values to mix in come with their weight");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "attention_prep: unknown dtype %d", dtype);
    if (n_tokens == 0) return 0;
#define FSIE_PREP(T)                                                                                                     \
    attention_prep_kernel<T><<<n_tokens, kThreads, 0, stream>>>(                                                         \
        static_cast<const T*>(proj), stride, q_off, k_off, v_off, g_off, heads, kv_heads, dim, vdim, D, q_weight, k_weight, \
        eps, pairs, reinterpret_cast<const float2*>(cos_sin), static_cast<const T*>(v_other), v_other_stride, mix,       \
        static_cast<T*>(q_out), gate, slots, static_cast<T*>(k_pool), static_cast<T*>(v_pool), page_size, pool_slots)
    if (dtype == FSIE_F32) FSIE_PREP(float); else FSIE_PREP(bf16_t);
#undef FSIE_PREP
    FSIE_CHECK_LAUNCH("attention_prep");
    return 0;
}

// y[t][h][0 .. vdim) = x[t][h][0 .. vdim) * gate[t][h] (gate null: 1), x's heads D values apart
extern "C" int fsie_gate_heads(const void* x, int D, const float* gate, void* y, int n_tokens, int heads, int vdim, int dtype,
                               hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && heads > 0 && vdim > 0 && D >= vdim, "gate_heads: bad sizes");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "gate_heads: unknown dtype %d", dtype);
    const int64_t total = static_cast<int64_t>(n_tokens) * heads * vdim;
    if (total == 0) return 0;
    const unsigned grid = static_cast<unsigned>(ceil_div64(total, kThreads));
    if (dtype == FSIE_F32)
        gate_heads_kernel<float><<<grid, kThreads, 0, stream>>>(static_cast<const float*>(x), D, gate, static_cast<float*>(y),
                                                                heads, vdim, total);
    else
        gate_heads_kernel<bf16_t><<<grid, kThreads, 0, stream>>>(static_cast<const bf16_t*>(x), D, gate, static_cast<bf16_t*>(y),
                                                                 heads, vdim, total);
    FSIE_CHECK_LAUNCH("gate_heads");
    return 0;
}
