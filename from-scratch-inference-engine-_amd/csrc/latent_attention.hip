// Attention through a latent: what stands around the attention kernels when keys and values of all
// heads are made from one cached vector a token.
//
// A layer caches, per token, the normed latent c [kv_rank] and one rotated key part [rot_dim] shared by
// all heads, as one row of `width` values (the rest zeros) in a cache of ONE kv head: keys row-major,
// values transposed, as the attention kernels read them.  Head h's key is [W_uk,h c | rotated part] and
// its value W_uv,h c; with q~_h = W_uk,h^T q_h the score q_h . (W_uk,h c) equals q~_h . c, and the sum of
// weights times values is W_uv,h (sum of weights times c).  So attention runs over the cached rows
// themselves, every head reading the same keys, with queries [q~_h | rotated q part] of `width` values,
// and W_uv,h is applied to its result.  The kernels here: what is written into the cache
// (fsie_latent_prep), the rotation of pairs of neighbours (fsie_rope_pairs), and the product with a
// matrix of its own for every head (fsie_head_gemm).
#include "common.h"
#include "api.h"

namespace {

constexpr int kThreads = 256;

// Element j of a run of `width` values of which the first 2 * |pairs| are turned by the angles whose cosines
// and sines are cs[i]; the rest passes.  pairs > 0: the pairs are neighbours (2i, 2i + 1); pairs < 0: value i
// goes with value i + |pairs|.
template <typename T>
__device__ __forceinline__ float rotated_neighbour(const T* __restrict__ run, int j, int pairs, const float2* __restrict__ cs) {
    const float x = to_float(run[j]);
    const int n = pairs < 0 ? -pairs : pairs;
    if (j >= 2 * n) return x;
    if (pairs < 0) {
        const bool low = j < n;
        const float2 t = cs[low ? j : j - n];
        const float other = to_float(run[low ? j + n : j - n]);
        return low ? fmaf(x, t.x, -(other * t.y)) : fmaf(x, t.x, other * t.y);
    }
    const float2 t = cs[j >> 1];
    const float other = to_float(run[j ^ 1]);
    return (j & 1) ? fmaf(x, t.x, other * t.y) : fmaf(x, t.x, -(other * t.y));
}

// One workgroup a token.  proj [tokens][stride] holds, of every token: the query latent (q_rank values
// from dq_off), the key/value latent and the shared key part (kv_rank + rot_dim values from dkv_off), and
// one gate a head (from g_off).
//   cq[t]   = RMS norm of the query latent, weight q_weight                       (type T)
//   gate[t] = sigmoid of the gates                                                 (float32)
//   cache row of the token (if the layer keeps a cache): [RMS norm of the latent, weight kv_weight |
//             shared key part, its first 2 * pairs values rotated | zeros up to width]
template <typename T>
__global__ __launch_bounds__(kThreads) void latent_prep_kernel(
    const T* __restrict__ proj, int64_t stride, int dq_off, int q_rank, int dkv_off, int kv_rank, int rot_dim, int pairs,
    int g_off, int heads, const float* __restrict__ q_weight, const float* __restrict__ kv_weight, float eps,
    const float2* __restrict__ cos_sin, T* __restrict__ cq, float* __restrict__ gate, const int32_t* __restrict__ slots,
    T* __restrict__ k_pool, T* __restrict__ v_pool, int width, int page_size, int64_t pool_slots) {
    __shared__ float scratch[16];
    const int t = blockIdx.x;
    const T* row = proj + static_cast<int64_t>(t) * stride;
    {
        const T* x = row + dq_off;
        float sum = 0.f;
        for (int j = threadIdx.x; j < q_rank; j += kThreads) sum += to_float(x[j]) * to_float(x[j]);
        const float scale = 1.0f / sqrtf(block_sum(sum, scratch) / static_cast<float>(q_rank) + eps);
        T* dst = cq + static_cast<int64_t>(t) * q_rank;
        for (int j = threadIdx.x; j < q_rank; j += kThreads) dst[j] = from_float<T>((to_float(x[j]) * scale) * q_weight[j]);
    }
    for (int h = threadIdx.x; h < heads; h += kThreads)
        gate[static_cast<int64_t>(t) * heads + h] = 1.0f / (1.0f + expf(-to_float(row[g_off + h])));
    if (!k_pool) return;  // the layer reads another layer's cache
    const T* x = row + dkv_off;
    float sum = 0.f;
    for (int j = threadIdx.x; j < kv_rank; j += kThreads) sum += to_float(x[j]) * to_float(x[j]);
    const float scale = 1.0f / sqrtf(block_sum(sum, scratch) / static_cast<float>(kv_rank) + eps);
    const int64_t slot = slots[t];
    if (slot < 0 || slot >= pool_slots) return;
    const int64_t page = slot / page_size;
    const int off = static_cast<int>(slot - page * page_size);
    const float2* cs = cos_sin + static_cast<int64_t>(t) * (pairs < 0 ? -pairs : pairs);
    for (int j = threadIdx.x; j < width; j += kThreads) {
        float v = 0.f;
        if (j < kv_rank) v = (to_float(x[j]) * scale) * kv_weight[j];
        else if (j < kv_rank + rot_dim) v = rotated_neighbour(x + kv_rank, j - kv_rank, pairs, cs);
        const T stored = from_float<T>(v);
        k_pool[slot * width + j] = stored;
        v_pool[(page * width + j) * page_size + off] = stored;
    }
}

// out[t][out_off + h * out_hs + j] for j < out_width: the run in[t][in_off + h * in_hs + (0 .. width)] with
// its first 2 * pairs values rotated as pairs of neighbours, then zeros.
template <typename T>
__global__ __launch_bounds__(kThreads) void rope_pairs_kernel(const T* __restrict__ in, int64_t in_stride, int in_off, int in_hs,
                                                              T* __restrict__ out, int64_t out_stride, int out_off, int out_hs,
                                                              int heads, int width, int pairs, int out_width,
                                                              const float2* __restrict__ cos_sin) {
    const int t = blockIdx.x;
    const float2* cs = cos_sin + static_cast<int64_t>(t) * (pairs < 0 ? -pairs : pairs);
    for (int e = threadIdx.x; e < heads * out_width; e += kThreads) {
        const int h = e / out_width, j = e - h * out_width;
        const float v = j < width ? rotated_neighbour(in + static_cast<int64_t>(t) * in_stride + in_off + h * in_hs, j, pairs, cs) : 0.f;
        out[static_cast<int64_t>(t) * out_stride + out_off + h * out_hs + j] = from_float<T>(v);
    }
}

// y[t][h][n] = (sum over k of x[t][h][k] * w[h][n][k]) * (gate ? gate[t][h] : 1): a tile of 32 tokens by 64
// outputs of one head a workgroup, 32 values of k a pass through LDS, float32 sums.
constexpr int kTileM = 32, kTileN = 64, kTileK = 32;
template <typename T>
__global__ __launch_bounds__(kThreads) void head_gemm_kernel(const T* __restrict__ x, int64_t x_stride, int x_off, int x_hs,
                                                             const T* __restrict__ w, T* __restrict__ y, int64_t y_stride,
                                                             int y_off, int y_hs, const float* __restrict__ gate,
                                                             int n_tokens, int heads, int N, int K) {
    __shared__ float xs[kTileM][kTileK + 1];
    __shared__ float ws[kTileN][kTileK + 1];
    const int h = blockIdx.z, n0 = blockIdx.x * kTileN, t0 = blockIdx.y * kTileM;
    const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;
    const T* wh = w + static_cast<int64_t>(h) * N * K;
    float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
    for (int k0 = 0; k0 < K; k0 += kTileK) {
        __syncthreads();
        for (int e = tid; e < kTileM * kTileK; e += kThreads) {
            const int r = e / kTileK, c = e - r * kTileK;
            const int t = t0 + r, k = k0 + c;
            xs[r][c] = (t < n_tokens && k < K) ? to_float(x[static_cast<int64_t>(t) * x_stride + x_off + h * x_hs + k]) : 0.f;
        }
        for (int e = tid; e < kTileN * kTileK; e += kThreads) {
            const int r = e / kTileK, c = e - r * kTileK;
            const int n = n0 + r, k = k0 + c;
            ws[r][c] = (n < N && k < K) ? to_float(wh[static_cast<int64_t>(n) * K + k]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < kTileK; ++kk) {
            const float a0 = xs[2 * ty][kk], a1 = xs[2 * ty + 1][kk];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float b = ws[tx + 16 * j][kk];
                acc[0][j] = fmaf(a0, b, acc[0][j]);
                acc[1][j] = fmaf(a1, b, acc[1][j]);
            }
        }
    }
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const int t = t0 + 2 * ty + a;
        if (t >= n_tokens) continue;
        const float g = gate ? gate[static_cast<int64_t>(t) * heads + h] : 1.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx + 16 * j;
            if (n < N) y[static_cast<int64_t>(t) * y_stride + y_off + h * y_hs + n] = from_float<T>(acc[a][j] * g);
        }
    }
}

// The same product on the matrix cores, bfloat16 operands and float32 sums (v_mfma_f32_16x16x32_bf16): both x's
// and w's rows run along K, which is what the instruction's operands want of a lane (eight neighbouring K
// values of one row), so both are read from memory as they lie, no staging.  w is the first operand: a lane
// then ends with four neighbouring outputs of one token, one 8-byte store.  A wave computes MT tiles of
// sixteen tokens by four tiles of sixteen outputs; the four waves of a workgroup are next to each other along N.
// Rows must start at multiples of eight values (16 bytes) and K must be one.
typedef __bf16 hg_bf16x8 __attribute__((ext_vector_type(8)));
typedef float hg_floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned hg_u32x4 __attribute__((ext_vector_type(4)));
union HgFrag {
    hg_u32x4 u;
    hg_bf16x8 v;
};

template <int MT>
__global__ __launch_bounds__(kThreads) void head_gemm_mfma_kernel(const bf16_t* __restrict__ x, int64_t x_stride, int x_off,
                                                                  int x_hs, const bf16_t* __restrict__ w,
                                                                  bf16_t* __restrict__ y, int64_t y_stride, int y_off,
                                                                  int y_hs, const float* __restrict__ gate, int n_tokens,
                                                                  int heads, int N, int K) {
    const int h = blockIdx.z, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * 4 + wave) * 64, t0 = blockIdx.y * (16 * MT);
    if (n0 >= N) return;
    const int r = lane & 15, kq = (lane >> 4) * 8;
    const bf16_t* wh = w + static_cast<int64_t>(h) * N * K;
    const bf16_t* wrow[4];
    bool wok[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const int n = n0 + 16 * a + r;
        wok[a] = n < N;
        wrow[a] = wh + static_cast<int64_t>(min(n, N - 1)) * K + kq;
    }
    const bf16_t* xrow[MT];
    bool xok[MT];
#pragma unroll
    for (int b = 0; b < MT; ++b) {
        const int t = t0 + 16 * b + r;
        xok[b] = t < n_tokens;
        xrow[b] = x + static_cast<int64_t>(min(t, n_tokens - 1)) * x_stride + x_off + h * x_hs + kq;
    }
    hg_floatx4 acc[4][MT];
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int b = 0; b < MT; ++b) acc[a][b] = hg_floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const hg_u32x4 zero = {0u, 0u, 0u, 0u};
    for (int k0 = 0; k0 < K; k0 += 32) {
        const bool kok = k0 + kq < K;  // K is a multiple of eight: a lane's eight values are all inside or all outside
        HgFrag wf[4], xf[MT];
#pragma unroll
        for (int a = 0; a < 4; ++a) wf[a].u = (kok && wok[a]) ? *reinterpret_cast<const hg_u32x4*>(wrow[a] + k0) : zero;
#pragma unroll
        for (int b = 0; b < MT; ++b) xf[b].u = (kok && xok[b]) ? *reinterpret_cast<const hg_u32x4*>(xrow[b] + k0) : zero;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
#pragma unroll
            for (int b = 0; b < MT; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[a].v, xf[b].v, acc[a][b], 0, 0, 0);
        }
    }
    // lane: the outputs 4 (lane / 16) .. + 3 of a tile of sixteen, of the token lane % 16 of a tile
    const int nq = (lane >> 4) * 4;
#pragma unroll
    for (int b = 0; b < MT; ++b) {
        const int t = t0 + 16 * b + r;
        if (t >= n_tokens) continue;
        const float g = gate ? gate[static_cast<int64_t>(t) * heads + h] : 1.0f;
        bf16_t* dst = y + static_cast<int64_t>(t) * y_stride + y_off + h * y_hs;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int n = n0 + 16 * a + nq;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (n + i < N) dst[n + i] = from_float<bf16_t>(acc[a][b][i] * g);
            }
        }
    }
}

}  // namespace

extern "C" int fsie_latent_prep(const void* proj, int64_t stride, int dq_off, int q_rank, int dkv_off, int kv_rank,
                                int rot_dim, int rot_pairs, int g_off, int heads, const float* q_weight,
                                const float* kv_weight, float eps, const float* cos_sin, void* cq, float* gate,
                                const int32_t* slots, void* k_pool, void* v_pool, int width, int page_size,
                                int64_t pool_slots, int n_tokens, int dtype, hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && q_rank > 0 && kv_rank > 0 && rot_dim >= 0 && heads >= 0, "latent_prep: bad sizes");
    FSIE_REQUIRE(2 * abs(rot_pairs) <= rot_dim, "latent_prep: %d rotated pairs do not fit %d values", rot_pairs, rot_dim);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "latent_prep: unknown dtype %d", dtype);
    FSIE_REQUIRE(proj && q_weight && cq && (gate || heads == 0), "latent_prep: missing operand");
    FSIE_REQUIRE(dq_off >= 0 && dq_off + q_rank <= stride && g_off >= 0 && g_off + heads <= stride,
                 "latent_prep: the columns do not fit a row of %lld", static_cast<long long>(stride));
    const bool writes = k_pool != nullptr;
    if (writes) {
        FSIE_REQUIRE(v_pool && slots && kv_weight && (rot_pairs == 0 || cos_sin), "latent_prep: missing operand of the cache write");
        FSIE_REQUIRE(dkv_off >= 0 && dkv_off + kv_rank + rot_dim <= stride, "latent_prep: the latent's columns do not fit a row");
        FSIE_REQUIRE(width >= kv_rank + rot_dim && page_size > 0 && pool_slots > 0, "latent_prep: bad cache geometry");
        FSIE_REQUIRE(reinterpret_cast<uintptr_t>(cos_sin) % 8 == 0, "latent_prep: the cosines and sines must be 8-byte aligned");
    }
    if (n_tokens == 0) return 0;
#define FSIE_PREP(T)                                                                                                     \
    latent_prep_kernel<T><<<n_tokens, kThreads, 0, stream>>>(                                                            \
        static_cast<const T*>(proj), stride, dq_off, q_rank, dkv_off, kv_rank, rot_dim, rot_pairs, g_off, heads, q_weight, \
        kv_weight, eps, reinterpret_cast<const float2*>(cos_sin), static_cast<T*>(cq), gate, slots, static_cast<T*>(k_pool), \
        static_cast<T*>(v_pool), width, page_size, pool_slots)
    if (dtype == FSIE_F32) FSIE_PREP(float);
    else FSIE_PREP(bf16_t);
#undef FSIE_PREP
    FSIE_CHECK_LAUNCH("latent_prep");
    return 0;
}

extern "C" int fsie_rope_pairs(const void* in, int64_t in_stride, int in_off, int in_hs, void* out, int64_t out_stride,
                               int out_off, int out_hs, int heads, int width, int rot_pairs, int out_width,
                               const float* cos_sin, int n_tokens, int dtype, hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && heads > 0 && width >= 0 && out_width >= width && 2 * abs(rot_pairs) <= width,
                 "rope_pairs: bad sizes heads=%d width=%d pairs=%d out_width=%d", heads, width, rot_pairs, out_width);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "rope_pairs: unknown dtype %d", dtype);
    FSIE_REQUIRE(in && out && (rot_pairs == 0 || cos_sin) && reinterpret_cast<uintptr_t>(cos_sin) % 8 == 0, "rope_pairs: missing operand");
    FSIE_REQUIRE(in_off >= 0 && out_off >= 0 && in_off + (heads - 1) * in_hs + width <= in_stride &&
                     out_off + (heads - 1) * out_hs + out_width <= out_stride,
                 "rope_pairs: the heads do not fit the rows");
    if (n_tokens == 0 || out_width == 0) return 0;
    if (dtype == FSIE_F32) {
        rope_pairs_kernel<float><<<n_tokens, kThreads, 0, stream>>>(static_cast<const float*>(in), in_stride, in_off, in_hs,
                                                                  static_cast<float*>(out), out_stride, out_off, out_hs, heads,
                                                                  width, rot_pairs, out_width, reinterpret_cast<const float2*>(cos_sin));
    } else {
        rope_pairs_kernel<bf16_t><<<n_tokens, kThreads, 0, stream>>>(static_cast<const bf16_t*>(in), in_stride, in_off, in_hs,
                                                                   static_cast<bf16_t*>(out), out_stride, out_off, out_hs, heads,
                                                                   width, rot_pairs, out_width, reinterpret_cast<const float2*>(cos_sin));
    }
    FSIE_CHECK_LAUNCH("rope_pairs");
    return 0;
}

// x [n_tokens][x_stride]: head h's K values start at column x_off + h * x_hs; w [heads][N][K]; y likewise
// with N values a head from y_off + h * y_hs; gate (or null) float32 [n_tokens][heads].
extern "C" int fsie_head_gemm(const void* x, int64_t x_stride, int x_off, int x_hs, const void* w, void* y, int64_t y_stride,
                              int y_off, int y_hs, const float* gate, int n_tokens, int heads, int N, int K, int dtype,
                              hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && heads > 0 && heads <= 65535 && N > 0 && K > 0, "head_gemm: bad sizes T=%d heads=%d N=%d K=%d",
                 n_tokens, heads, N, K);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "head_gemm: unknown dtype %d", dtype);
    FSIE_REQUIRE(x && w && y, "head_gemm: missing operand");
    FSIE_REQUIRE(x_off >= 0 && y_off >= 0 && x_off + (heads - 1) * x_hs + K <= x_stride && y_off + (heads - 1) * y_hs + N <= y_stride,
                 "head_gemm: the heads do not fit the rows");
    if (n_tokens == 0) return 0;
    const int row_tiles = (n_tokens + kTileM - 1) / kTileM;
    FSIE_REQUIRE(row_tiles <= 65535, "head_gemm: %d tokens are more than one launch takes", n_tokens);
    const dim3 grid((N + kTileN - 1) / kTileN, row_tiles, heads);
    const bool aligned = K % 8 == 0 && x_stride % 8 == 0 && x_off % 8 == 0 && x_hs % 8 == 0 &&
                         reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
    if (dtype == FSIE_BF16 && aligned) {
        const bool two = n_tokens > 16;
        const int token_tiles = (n_tokens + (two ? 32 : 16) - 1) / (two ? 32 : 16);
        FSIE_REQUIRE(token_tiles <= 65535, "head_gemm: %d tokens are more than one launch takes", n_tokens);
        const dim3 mgrid((N + 255) / 256, token_tiles, heads);
        if (two) {
            head_gemm_mfma_kernel<2><<<mgrid, kThreads, 0, stream>>>(static_cast<const bf16_t*>(x), x_stride, x_off, x_hs,
                                                                    static_cast<const bf16_t*>(w), static_cast<bf16_t*>(y),
                                                                    y_stride, y_off, y_hs, gate, n_tokens, heads, N, K);
        } else {
            head_gemm_mfma_kernel<1><<<mgrid, kThreads, 0, stream>>>(static_cast<const bf16_t*>(x), x_stride, x_off, x_hs,
                                                                    static_cast<const bf16_t*>(w), static_cast<bf16_t*>(y),
                                                                    y_stride, y_off, y_hs, gate, n_tokens, heads, N, K);
        }
    } else if (dtype == FSIE_F32) {
        head_gemm_kernel<float><<<grid, kThreads, 0, stream>>>(static_cast<const float*>(x), x_stride, x_off, x_hs,
                                                             static_cast<const float*>(w), static_cast<float*>(y), y_stride,
                                                             y_off, y_hs, gate, n_tokens, heads, N, K);
    } else {
        head_gemm_kernel<bf16_t><<<grid, kThreads, 0, stream>>>(static_cast<const bf16_t*>(x), x_stride, x_off, x_hs,
                                                              static_cast<const bf16_t*>(w), static_cast<bf16_t*>(y), y_stride,
                                                              y_off, y_hs, gate, n_tokens, heads, N, K);
    }
    FSIE_CHECK_LAUNCH("head_gemm");
    return 0;
}
