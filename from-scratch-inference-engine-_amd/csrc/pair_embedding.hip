// Token embedding times a constant plus a hashed embedding of the pair (previous token, token):
//   x[t] = table[id_t] * scale + pairs[(id_{t-1} * mul_prev + id_t * mul_cur) mod buckets]
// and pairs[buckets] (the table's last row) for a request's first token.  The token before a portion's first
// one is what the request's state slot holds from the step before: last[slot] = that id + 1, 0 = none (a slot is
// zeroed when a request starts).  A second, tiny kernel stores the portion's last id for the next step: it runs
// after the rows are written, so no block reads a slot that another has already overwritten.
#include "common.h"
#include "api.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void pair_embedding_kernel(const T* __restrict__ table, const T* __restrict__ pairs,
                                                             const int32_t* __restrict__ ids,
                                                             const int32_t* __restrict__ q_starts,
                                                             const int32_t* __restrict__ seq_slots, int n_seqs,
                                                             const int32_t* __restrict__ last, int n_slots,
                                                             float* __restrict__ out, int hidden, int vocab, int buckets,
                                                             int64_t mul_prev, int64_t mul_cur, float scale) {
    __shared__ int64_t s_rows[2];
    const int t = blockIdx.x;
    if (threadIdx.x == 0) {
        // the request of this row: the last one whose first row is not beyond it
        int lo = 0, hi = n_seqs - 1;
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (q_starts[mid] <= t) lo = mid; else hi = mid - 1;
        }
        int prev = -1;
        if (t > q_starts[lo]) {
            prev = ids[t - 1];
        } else {
            const int slot = seq_slots[lo];
            if (slot >= 0 && slot < n_slots) prev = last[slot] - 1;
        }
        int id = ids[t];
        id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
        int64_t row = buckets;
        if (prev >= 0) {
            row = (static_cast<int64_t>(prev) * mul_prev + static_cast<int64_t>(id) * mul_cur) % buckets;
            if (row < 0) row += buckets;
        }
        s_rows[0] = id;
        s_rows[1] = row;
    }
    __syncthreads();
    const T* a = table + s_rows[0] * hidden;
    const T* b = pairs + s_rows[1] * hidden;
    float* o = out + static_cast<int64_t>(t) * hidden;
    for (int j = threadIdx.x; j < hidden; j += blockDim.x) o[j] = fmaf(to_float(a[j]), scale, to_float(b[j]));
}

__global__ void store_last_token_kernel(const int32_t* __restrict__ ids, const int32_t* __restrict__ q_starts,
                                        const int32_t* __restrict__ seq_slots, int n_seqs, int32_t* __restrict__ last,
                                        int n_slots) {
    const int s = blockIdx.x * blockDim.x + threadIdx.x;
    if (s >= n_seqs) return;
    const int slot = seq_slots[s];
    const int end = q_starts[s + 1];
    if (slot >= 0 && slot < n_slots && end > q_starts[s]) last[slot] = ids[end - 1] + 1;
}

}  // namespace

extern "C" int fsie_pair_embedding(const void* table, const void* pairs, int dtype, const int32_t* ids,
                                   const int32_t* q_starts, const int32_t* seq_slots, int n_seqs, int32_t* last,
                                   int n_slots, float* out, int n_tokens, int hidden, int vocab, int buckets,
                                   int64_t mul_prev, int64_t mul_cur, float scale, hipStream_t stream) {
    FSIE_REQUIRE(n_tokens >= 0 && n_seqs >= 0 && hidden > 0 && vocab > 0 && buckets > 0 && n_slots > 0,
                 "pair_embedding: bad sizes T=%d requests=%d hidden=%d vocab=%d buckets=%d", n_tokens, n_seqs, hidden, vocab,
                 buckets);
    FSIE_REQUIRE(table && pairs && ids && q_starts && seq_slots && last && out, "pair_embedding: missing operand");
    FSIE_REQUIRE(dtype == FSIE_F32 || dtype == FSIE_BF16, "pair_embedding: unknown dtype %d", dtype);
    if (n_tokens == 0 || n_seqs == 0) return 0;
    if (dtype == FSIE_F32)
        pair_embedding_kernel<float><<<n_tokens, 256, 0, stream>>>(static_cast<const float*>(table), static_cast<const float*>(pairs),
                                                                   ids, q_starts, seq_slots, n_seqs, last, n_slots, out, hidden,
                                                                   vocab, buckets, mul_prev, mul_cur, scale);
    else
        pair_embedding_kernel<bf16_t><<<n_tokens, 256, 0, stream>>>(static_cast<const bf16_t*>(table), static_cast<const bf16_t*>(pairs),
                                                                    ids, q_starts, seq_slots, n_seqs, last, n_slots, out, hidden,
                                                                    vocab, buckets, mul_prev, mul_cur, scale);
    FSIE_CHECK_LAUNCH("pair_embedding");
    store_last_token_kernel<<<(n_seqs + 63) / 64, 64, 0, stream>>>(ids, q_starts, seq_slots, n_seqs, last, n_slots);
    FSIE_CHECK_LAUNCH("store_last_token");
    return 0;
}
