// Gated linear attention: a recurrent state per request and head, S [dim][vdim] in float32,
//   S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,   o_t = S_t^T q_t,
// with a decay per key channel alpha = sigmoid(z)^(1/tau).  One pair of kernels serves portions of prompts
// and single decoded tokens: the tokens of a request's portion are walked in order, from the state that the
// request's slot holds, and the state is left there for the next step.  Everything that enters the
// recurrence is float32 (decays, their logarithms, the state, the sums); q, k and v come in the
// activations' type as the projections left them.
//
// The walk is bound by arithmetic: every state element costs three instructions a token, on the vector
// units, in float32.  So the state of a head is spread over as many waves as the sizes give: a workgroup of
// sixteen waves holds [rows of one split][64 value columns], wave w a few consecutive key channels of it,
// lane = value column.  What a wave needs of a token besides v (its channels' decay, k and scaled q) is
// the same in all its lanes: a first kernel lays these out in float32 ([token][head][padded channel], the
// padding with decay 1 and k = q = 0), and the walk reads them with addresses that are uniform over the
// wave, which the compiler turns into scalar loads: no lane-wide traffic for them at all.
#include "common.h"
#include "api.h"

#include <math.h>

namespace {

constexpr int kGlaWaves = 16;
constexpr int kGlaThreads = 64 * kGlaWaves;
constexpr int kGlaCols = 64;
constexpr int kGlaTokens = 8;  // tokens whose shares of o are added up at once

// log(sigmoid(z)) without overflow: min(z, 0) - log(1 + exp(-|z|))
__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// A workgroup barrier that waits for this wave's shared-memory traffic only.  __syncthreads also waits for
// the wave's loads and stores of global memory, and the walk has both in flight at every barrier (the next
// tokens' v on their way in, the last tokens' o on their way out): with it every tile of tokens paid two
// trips to memory, ten times its arithmetic.  What the waves exchange here goes through shared memory alone.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// prep [3][tokens][heads][dp]: scaled q, k, decay.
template <typename T>
__global__ void gla_prep_kernel(const T* __restrict__ proj, int64_t proj_stride, int q_off, int k_off,
                                const float* __restrict__ z, float* __restrict__ prep, int64_t total, int heads, int dim,
                                int dp, float q_scale, float inv_tau) {
    const int64_t e = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (e >= total) return;
    const int i = static_cast<int>(e % dp);
    const int64_t th = e / dp;
    const int h = static_cast<int>(th % heads);
    const int64_t t = th / heads;
    float q = 0.f, k = 0.f, a = 1.f;
    if (i < dim) {
        const T* row = proj + t * proj_stride + h * dim + i;
        q = to_float(row[q_off]) * q_scale;
        k = to_float(row[k_off]);
        a = expf(inv_tau * log_sigmoid(z[(t * heads + h) * dim + i]));
    }
    prep[e] = q;
    prep[total + e] = k;
    prep[2 * total + e] = a;
}

// grid = (requests of the step, heads, column blocks * row splits).  out [row splits][tokens][heads * vdim]:
// every split's share of o, for the consumer to add in order.
template <typename T, int ROWS>
__global__ __launch_bounds__(kGlaThreads) void gla_scan_kernel(
    const T* __restrict__ proj, int64_t proj_stride, int v_off, const float* __restrict__ prep, int64_t prep_plane,
    float* __restrict__ state, const int32_t* __restrict__ q_starts, const int32_t* __restrict__ seq_slots,
    float* __restrict__ out, int64_t out_plane, int heads, int dim, int vdim, int dp, int row_splits, int n_slots) {
    constexpr int TT = kGlaTokens;
    __shared__ float part[kGlaWaves][TT][kGlaCols];
    const int seq = blockIdx.x, h = blockIdx.y;
    const int split = blockIdx.z % row_splits, col_block = blockIdx.z / row_splits;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same in all lanes: what depends on it alone is scalar
    const int col = col_block * kGlaCols + lane;
    const int lo = q_starts[seq], hi = q_starts[seq + 1];
    const int slot = seq_slots[seq];
    if (hi <= lo || slot < 0 || slot >= n_slots) return;  // the same for the whole workgroup
    const bool col_ok = col < vdim;
    const int row0 = (split * kGlaWaves + wave) * ROWS;  // this wave's first key channel

    float* my_state = state + ((static_cast<int64_t>(slot) * heads + h) * dim) * vdim + col;
    float S[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) S[r] = (col_ok && row0 + r < dim) ? my_state[static_cast<int64_t>(row0 + r) * vdim] : 0.f;

    const float* qp = prep + static_cast<int64_t>(h) * dp + row0;
    const float* kp = qp + prep_plane;
    const float* ap = kp + prep_plane;
    const int64_t token_stride = static_cast<int64_t>(heads) * dp;
    float* mine = out + split * out_plane;

    for (int t0 = lo; t0 < hi; t0 += TT) {
        const int nt = min(TT, hi - t0);
        float v[TT];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            v[tt] = (tt < nt && col_ok)
                        ? to_float(proj[static_cast<int64_t>(t0 + tt) * proj_stride + v_off + h * vdim + col]) : 0.f;
        }
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
            if (tt < nt) {  // the same for the whole workgroup
                const int64_t at = static_cast<int64_t>(t0 + tt) * token_stride;
                float o = 0.f;
#pragma unroll
                for (int r = 0; r < ROWS; ++r) {
                    S[r] = fmaf(ap[at + r], S[r], kp[at + r] * v[tt]);
                    o = fmaf(S[r], qp[at + r], o);
                }
                part[wave][tt][lane] = o;
            }
        }
        lds_barrier();
        for (int e = tid; e < nt * kGlaCols; e += kGlaThreads) {
            const int tt = e >> 6, c = e & 63;
            const int cc = col_block * kGlaCols + c;
            if (cc < vdim) {
                float o = part[0][tt][c];
#pragma unroll
                for (int w = 1; w < kGlaWaves; ++w) o += part[w][tt][c];
                mine[(static_cast<int64_t>(t0 + tt) * heads + h) * vdim + cc] = o;
            }
        }
        lds_barrier();  // the shares have been read: the next tile may overwrite them
    }
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        if (col_ok && row0 + r < dim) my_state[static_cast<int64_t>(row0 + r) * vdim] = S[r];
    }
}

// Key channels a wave holds and the splits of a head's channels over workgroups: as many splits (1, 2, 4)
// as still leave a wave four channels, while the workgroups of one request number fewer than 128.  A
// function of the layer's sizes alone, never of the step.
void gla_shape(int heads, int dim, int vdim, int* rows, int* splits) {
    const int col_blocks = (vdim + kGlaCols - 1) / kGlaCols;
    int s = 1;
    while (s < 4 && dim >= kGlaWaves * 2 * s * 4 && heads * col_blocks * s < 128) s *= 2;
    const int per_wave = (dim + kGlaWaves * s - 1) / (kGlaWaves * s);
    int r = 1;
    while (r < per_wave) r *= 2;
    *rows = r;
    *splits = s;
}

}  // namespace

// Sizes of the two work arrays of fsie_gla_scan for a layer of these sizes: floats of `prep` a token, and the
// planes of `out` (row splits).
extern "C" int fsie_gla_scan_shape(int heads, int dim, int vdim, int* prep_floats_per_token, int* out_planes) {
    FSIE_REQUIRE(heads > 0 && dim > 0 && dim <= 256 && vdim > 0, "gla_scan_shape: bad sizes");
    int rows, splits;
    gla_shape(heads, dim, vdim, &rows, &splits);
    *prep_floats_per_token = 3 * heads * kGlaWaves * splits * rows;
    *out_planes = splits;
    return 0;
}

// proj [n_tokens][proj_stride]: of every token the q heads (heads x dim) from column q_off, the k heads
// from k_off, the v heads (heads x vdim) from v_off.  z [n_tokens][heads * dim] float32: the decays before
// the sigmoid.  state [n_slots][heads][dim][vdim] float32.  Request s of the step owns the tokens
// q_starts[s] .. q_starts[s + 1] and the slot seq_slots[s] (a slot outside the table: the request is
// skipped).  q is multiplied by q_scale; alpha = sigmoid(z)^inv_tau.  prep: work array of n_tokens *
// prep_floats_per_token floats; out: out_planes arrays [n_tokens][heads * vdim] float32 whose sum, in order,
// is o (fsie_gla_scan_shape gives both numbers).
extern "C" int fsie_gla_scan(const void* proj, int64_t proj_stride, int q_off, int k_off, int v_off, const float* z,
                             float* state, const int32_t* q_starts, const int32_t* seq_slots, int n_seqs, int n_tokens,
                             float* prep, float* out, int heads, int dim, int vdim, float q_scale, float inv_tau,
                             int n_slots, int dtype, hipStream_t stream) {
    FSIE_REQUIRE(n_seqs >= 0 && n_tokens >= 0 && heads > 0 && dim > 0 && vdim > 0 && n_slots > 0, "gla_scan: bad sizes");
    FSIE_REQUIRE(dim <= 256, "gla_scan: %d key channels a head are more than the kernel takes (256)", dim);
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "gla_scan: unknown dtype %d", dtype);
    FSIE_REQUIRE(proj && z && state && q_starts && seq_slots && out && prep, "gla_scan: missing operand");
    FSIE_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + heads * dim <= proj_stride &&
                     k_off + heads * dim <= proj_stride && v_off + heads * vdim <= proj_stride,
                 "gla_scan: the q, k and v columns do not fit a row of %lld", static_cast<long long>(proj_stride));
    if (n_seqs == 0 || n_tokens == 0) return 0;
    int rows, splits;
    gla_shape(heads, dim, vdim, &rows, &splits);
    const int dp = kGlaWaves * splits * rows;
    const int col_blocks = (vdim + kGlaCols - 1) / kGlaCols;
    FSIE_REQUIRE(heads <= 65535 && col_blocks * splits <= 65535, "gla_scan: too many heads or columns");
    const int64_t plane = static_cast<int64_t>(n_tokens) * heads * dp;
    const int64_t out_plane = static_cast<int64_t>(n_tokens) * heads * vdim;
    const unsigned prep_grid = static_cast<unsigned>(ceil_div64(plane, 256));
    const dim3 grid(n_seqs, heads, col_blocks * splits);
#define FSIE_GLA_LAUNCH(T, ROWS)                                                                                       \
    gla_scan_kernel<T, ROWS><<<grid, kGlaThreads, 0, stream>>>(static_cast<const T*>(proj), proj_stride, v_off, prep, plane, \
                                                               state, q_starts, seq_slots, out, out_plane, heads, dim, vdim, \
                                                               dp, splits, n_slots)
#define FSIE_GLA_BY_ROWS(T)                                                                                          \
    gla_prep_kernel<T><<<prep_grid, 256, 0, stream>>>(static_cast<const T*>(proj), proj_stride, q_off, k_off, z, prep, \
                                                      plane, heads, dim, dp, q_scale, inv_tau);                      \
    if (rows == 1) FSIE_GLA_LAUNCH(T, 1);                                                                            \
    else if (rows == 2) FSIE_GLA_LAUNCH(T, 2);                                                                       \
    else if (rows == 4) FSIE_GLA_LAUNCH(T, 4);                                                                       \
    else if (rows == 8) FSIE_GLA_LAUNCH(T, 8);                                                                       \
    else FSIE_GLA_LAUNCH(T, 16)
    if (dtype == FSIE_F32) {
        FSIE_GLA_BY_ROWS(float);
    } else {
        FSIE_GLA_BY_ROWS(bf16_t);
    }
#undef FSIE_GLA_BY_ROWS
#undef FSIE_GLA_LAUNCH
    FSIE_CHECK_LAUNCH("gla_scan");
    return 0;
}
