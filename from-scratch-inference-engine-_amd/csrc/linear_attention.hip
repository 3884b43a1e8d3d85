// Gated linear attention: a recurrent state per request and head, S [dim][vdim] in float32,
//   S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
// with a decay per key channel alpha = sigmoid(z)^(1/tau).  One kernel serves portions of prompts and
// single decoded tokens: it walks the tokens of a request's portion in order, from the state that the
// request's slot holds, and leaves the state there for the next step.  Everything that enters the
// recurrence is float32 (decays, their logarithms, the state, the sums); q, k and v come in the
// activations' type as the projections left them.
#include "common.h"
#include "api.h"

#include <math.h>

namespace {

constexpr int kGlaWaves = 16;  // wave w owns the key channels [w ROWS, (w + 1) ROWS), lane = value column
constexpr int kGlaThreads = 64 * kGlaWaves;
constexpr int kGlaCols = 64;

// log(sigmoid(z)) without overflow: min(z, 0) - log(1 + exp(-|z|))
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// grid = (requests of the step, heads, ceil(vdim / 64)).  A workgroup of sixteen waves keeps its [dim][64]
// slice of the state in registers (ROWS values a thread: few, so that a token costs a wave only 3 ROWS
// instructions and the sixteen waves hide each other's waits), takes the portion's tokens in tiles of TT
// through LDS (q scaled, k, and the decays already as numbers in (0, 1), read by every lane of a wave at
// the same address), and adds the waves' shares of every o_t through LDS in the order of the waves.
template <typename T, int ROWS, int TT>
__global__ __launch_bounds__(kGlaThreads) void gla_scan_kernel(
    const T* __restrict__ proj, int64_t proj_stride, int q_off, int k_off, int v_off, const float* __restrict__ z,
    float* __restrict__ state, const int32_t* __restrict__ q_starts, const int32_t* __restrict__ seq_slots,
    float* __restrict__ out, int heads, int dim, int vdim, float q_scale, float inv_tau, int n_slots) {
    constexpr int DP = kGlaWaves * ROWS;
    constexpr int VW = ROWS % 4 == 0 ? 4 : 2;  // values of a shared-memory load (ROWS is 2, 4, 8 or 16)
    typedef float Vec __attribute__((ext_vector_type(VW)));
    __shared__ __attribute__((aligned(16))) float qs[TT][DP], ks[TT][DP], as[TT][DP];
    __shared__ float part[kGlaWaves][TT][kGlaCols];
    const int seq = blockIdx.x, h = blockIdx.y;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = blockIdx.z * kGlaCols + lane;
    const int lo = q_starts[seq], hi = q_starts[seq + 1];
    const int slot = seq_slots[seq];
    if (hi <= lo || slot < 0 || slot >= n_slots) return;  // the same for the whole workgroup
    const bool col_ok = col < vdim;

    float* my_state = state + ((static_cast<int64_t>(slot) * heads + h) * dim) * vdim + col;
    float S[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int i = wave * ROWS + r;
        S[r] = (col_ok && i < dim) ? my_state[static_cast<int64_t>(i) * vdim] : 0.f;
    }

    // The inputs of the next tile are asked for before the present one is worked on, and wait in registers:
    // a tile costs a few hundred cycles of arithmetic, a trip to memory several times that.
    constexpr int EPT = (TT * DP + kGlaThreads - 1) / kGlaThreads;
    float rq[EPT], rk[EPT], rz[EPT], v_next[TT];
    auto fetch = [&](int t0) {
        const int nt = min(TT, hi - t0);
#pragma unroll
        for (int u = 0; u < EPT; ++u) {
            const int e = tid + u * kGlaThreads;
            const int tt = e / DP, i = e - tt * DP;
            rq[u] = 0.f, rk[u] = 0.f, rz[u] = INFINITY;  // a channel or token that does not exist: q = k = 0, decay 1
            if (tt < nt && i < dim) {
                const T* row = proj + static_cast<int64_t>(t0 + tt) * proj_stride + h * dim + i;
                rq[u] = to_float(row[q_off]);
                rk[u] = to_float(row[k_off]);
                rz[u] = z[(static_cast<int64_t>(t0 + tt) * heads + h) * dim + i];
            }
        }
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            v_next[tt] = (tt < nt && col_ok)
                             ? to_float(proj[static_cast<int64_t>(t0 + tt) * proj_stride + v_off + h * vdim + col]) : 0.f;
        }
    };
    fetch(lo);
    for (int t0 = lo; t0 < hi; t0 += TT) {
        const int nt = min(TT, hi - t0);
        __syncthreads();  // the last tile's shares have been added up, its q, k and decays are no longer read
#pragma unroll
        for (int u = 0; u < EPT; ++u) {
            const int e = tid + u * kGlaThreads;
            if (e < TT * DP) {
                const int tt = e / DP, i = e - tt * DP;
                qs[tt][i] = rq[u] * q_scale;
                ks[tt][i] = rk[u];
                as[tt][i] = expf(inv_tau * log_sigmoid(rz[u]));
            }
        }
        float v[TT];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) v[tt] = v_next[tt];
        __syncthreads();
        if (t0 + TT < hi) fetch(t0 + TT);
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            if (tt < nt) {  // the same for the whole workgroup
                // this wave's channels of the token: every lane reads the same addresses, VW values a load
                float a[ROWS], k[ROWS], q[ROWS];
#pragma unroll
                for (int r = 0; r < ROWS; r += VW) {
                    *reinterpret_cast<Vec*>(&a[r]) = *reinterpret_cast<const Vec*>(&as[tt][wave * ROWS + r]);
                    *reinterpret_cast<Vec*>(&k[r]) = *reinterpret_cast<const Vec*>(&ks[tt][wave * ROWS + r]);
                    *reinterpret_cast<Vec*>(&q[r]) = *reinterpret_cast<const Vec*>(&qs[tt][wave * ROWS + r]);
                }
                float o = 0.f;
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    S[r] = fmaf(a[r], S[r], k[r] * v[tt]);
                    o = fmaf(S[r], q[r], o);
                }
                part[wave][tt][lane] = o;
            }
        }
        __syncthreads();
        for (int e = tid; e < nt * kGlaCols; e += kGlaThreads) {
            const int tt = e >> 6, c = e & 63;
            const int cc = blockIdx.z * kGlaCols + c;
            if (cc < vdim) {
                float o = part[0][tt][c];
#pragma unroll
                for (int w = 1; w < kGlaWaves; ++w) o += part[w][tt][c];
                out[(static_cast<int64_t>(t0 + tt) * heads + h) * vdim + cc] = o;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int i = wave * ROWS + r;
        if (col_ok && i < dim) my_state[static_cast<int64_t>(i) * vdim] = S[r];
    }
}

}  // namespace

// proj [n_tokens][proj_stride]: of every token the q heads (heads x dim) from column q_off, the k heads
// from k_off, the v heads (heads x vdim) from v_off.  z [n_tokens][heads * dim] float32: the decays before
// the sigmoid.  state [n_slots][heads][dim][vdim] float32.  Request s of the step owns the tokens
// q_starts[s] .. q_starts[s + 1] and the slot seq_slots[s] (a slot outside the table: the request is
// skipped).  out [n_tokens][heads * vdim] float32.  q is multiplied by q_scale; alpha = sigmoid(z)^inv_tau.
extern "C" int fsie_gla_scan(const void* proj, int64_t proj_stride, int q_off, int k_off, int v_off, const float* z,
                             float* state, const int32_t* q_starts, const int32_t* seq_slots, int n_seqs, float* out,
                             int heads, int dim, int vdim, float q_scale, float inv_tau, int n_slots, int dtype,
                             hipStream_t stream) {
    FSIE_REQUIRE(n_seqs >= 0 && heads > 0 && dim > 0 && vdim > 0 && n_slots > 0, "gla_scan: bad sizes");
    FSIE_REQUIRE(dim <= 256, "gla_scan: %d key channels a head are more than the kernel takes (256)", dim);
    FSIE_REQUIRE(heads <= 65535 && (vdim + kGlaCols - 1) / kGlaCols <= 65535, "gla_scan: too many heads or columns");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "gla_scan: unknown dtype %d", dtype);
    FSIE_REQUIRE(proj && z && state && q_starts && seq_slots && out, "gla_scan: missing operand");
    FSIE_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + heads * dim <= proj_stride &&
                     k_off + heads * dim <= proj_stride && v_off + heads * vdim <= proj_stride,
                 "gla_scan: the q, k and v columns do not fit a row of %lld", static_cast<long long>(proj_stride));
    if (n_seqs == 0) return 0;
    const dim3 grid(n_seqs, heads, (vdim + kGlaCols - 1) / kGlaCols);
#define FSIE_GLA_LAUNCH(T, ROWS, TT)                                                                                  \
    gla_scan_kernel<T, ROWS, TT><<<grid, kGlaThreads, 0, stream>>>(static_cast<const T*>(proj), proj_stride, q_off, k_off, \
                                                                   v_off, z, state, q_starts, seq_slots, out, heads, dim, \
                                                                   vdim, q_scale, inv_tau, n_slots)
#define FSIE_GLA_BY_DIM(T)                        \
    if (dim <= 32) FSIE_GLA_LAUNCH(T, 2, 8);      \
    else if (dim <= 64) FSIE_GLA_LAUNCH(T, 4, 8); \
    else if (dim <= 128) FSIE_GLA_LAUNCH(T, 8, 8); \
    else FSIE_GLA_LAUNCH(T, 16, 8)
    if (dtype == FSIE_F32) {
        FSIE_GLA_BY_DIM(float);
    } else {
        FSIE_GLA_BY_DIM(bf16_t);
    }
#undef FSIE_GLA_BY_DIM
#undef FSIE_GLA_LAUNCH
    FSIE_CHECK_LAUNCH("gla_scan");
    return 0;
}
