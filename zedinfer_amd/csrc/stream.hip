// What happens to the residual stream between the sublayers of some designs, and what enters it at the start.
//
//   zi_embedding_sum   x[t] = table[id_t] + pair[hash(id_{t-1}, id_t)] + sinusoid(position_t), float32.  The pair
//                      table is looked up by (id_{t-1} * mul_prev + id_t * mul_cur) mod buckets, its last row
//                      (number `buckets`) for a sequence's first token; the token before an entry's first one comes
//                      from the request's state slot, and the entry's last token goes there.
//   zi_token_shift     y[t] = h[t] + (h[t-1] - h[t]) * w, per channel, zeros before a sequence's first token; the
//                      row before an entry's first one comes from the request's state slot (float32), and the
//                      entry's last row goes there.
//   zi_stream_reenter  resid += (pending terms) + again[t] + row, for designs that feed the embedding output (or a
//                      learned row) into the stream again at a later layer.
//
// A state slot is read and rewritten by one workgroup (the one of the entry's first token), so a step needs one
// launch whatever its entries bring.  A row's values depend on the row, its predecessor and the tables only.
#include "zi_common.h"
#include "zi_api.h"

template <typename TW, typename TP>
__global__ void __launch_bounds__(256)
embedding_sum_kernel(float* __restrict__ out, const TW* __restrict__ table, const TP* __restrict__ pair,
                     const int32_t* __restrict__ ids, const int32_t* __restrict__ pos, const int32_t* __restrict__ tok_seq,
                     const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_len,
                     const int32_t* __restrict__ entry_slot, int32_t* __restrict__ state, int64_t state_stride,
                     const double* __restrict__ freq, int H, int V, int buckets, int64_t mul_prev, int64_t mul_cur) {
    const int64_t row = blockIdx.x;
    const int id = ids[row];
    const bool ok = id >= 0 && id < V;
    const int p = pos[row];
    const TP* prow = nullptr;
    if (pair) {
        const int e = tok_seq[row], first = entry_start[e];
        int32_t* slot = state + (int64_t)entry_slot[e] * state_stride;
        int prev;
        if (row == first) {
            prev = *slot;
            __syncthreads();        // every thread has read the slot before one rewrites it
            if (threadIdx.x == 0) *slot = ids[first + entry_len[e] - 1];
        } else {
            prev = ids[row - 1];
        }
        int64_t r = buckets;
        if (p > 0) {
            r = ((int64_t)prev * mul_prev + (int64_t)id * mul_cur) % buckets;
            if (r < 0) r += buckets;
        }
        prow = pair + r * H;
    }
    const TW* src = table + (int64_t)(ok ? id : 0) * H;
    float* dst = out + row * H;
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
        float v = ok ? zi_load(src + j) : NAN;
        if (prow) v += zi_load(prow + j);
        if (freq) {
            // the angle and its sine in double: the argument grows with the position
            const double a = (double)p * freq[j >> 1];
            v += (float)((j & 1) ? cos(a) : sin(a));
        }
        dst[j] = v;
    }
}

// `pair` [buckets + 1][hidden] or null; `freq` (double [ceil(hidden / 2)]: channel j turns with freq[j / 2], even
// channels take the sine, odd ones the cosine) or null; `state` int32 [slots][state_stride], needed with `pair`.
extern "C" int zi_embedding_sum(float* out, const void* table, int table_dt, const void* pair, int pair_dt,
                                const int32_t* ids, const int32_t* pos, const int32_t* tok_seq,
                                const int32_t* entry_start, const int32_t* entry_len, const int32_t* entry_slot,
                                int32_t* state, int64_t state_stride, const double* freq, int n, int hidden, int vocab,
                                int buckets, int64_t mul_prev, int64_t mul_cur, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && hidden > 0 && vocab > 0, "embedding_sum: bad sizes n=%d hidden=%d vocab=%d", n, hidden, vocab);
    ZI_REQUIRE(!pair || (buckets > 0 && state && state_stride >= 1 && tok_seq && entry_start && entry_len && entry_slot),
               "embedding_sum: the pair table needs buckets, the entries and a state slot");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(table_dt, TW, ZI_DISPATCH_DTYPE(pair ? pair_dt : table_dt, TP, {
        embedding_sum_kernel<TW, TP><<<n, 256, 0, stream>>>(out, (const TW*)table, (const TP*)pair, ids, pos, tok_seq,
                                                            entry_start, entry_len, entry_slot, state, state_stride, freq,
                                                            hidden, vocab, buckets, mul_prev, mul_cur);
    }));
    return zi_check_launch("embedding_sum");
}

template <typename TX, typename TW, typename TO>
__global__ void __launch_bounds__(256)
token_shift_kernel(TO* __restrict__ out, int64_t ldo, const TX* __restrict__ x, int64_t ldx, const TW* __restrict__ w,
                   float* __restrict__ state, int64_t state_stride, const int32_t* __restrict__ tok_seq,
                   const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ entry_start,
                   const int32_t* __restrict__ entry_len, const int32_t* __restrict__ entry_slot, int H) {
    const int64_t row = blockIdx.x;
    const int e = tok_seq[row], first = entry_start[e];
    const TX* cur = x + row * ldx;
    TO* dst = out + row * ldo;
    if (row != first) {
        const TX* prev = cur - ldx;
        for (int j = threadIdx.x; j < H; j += blockDim.x) {
            const float h = zi_load(cur + j);
            zi_store(dst + j, h + (zi_load(prev + j) - h) * zi_load(w + j));
        }
        return;
    }
    // an entry's first row: its predecessor is the request's slot (nothing before position 0), which this
    // workgroup then rewrites with the entry's last row; a thread reads and writes its own channels only
    float* slot = state + (int64_t)entry_slot[e] * state_stride;
    const bool start = tok_pos[row] == 0;
    const TX* last = x + (int64_t)(first + entry_len[e] - 1) * ldx;
    for (int j = threadIdx.x; j < H; j += blockDim.x) {
        const float h = zi_load(cur + j);
        const float before = start ? 0.f : slot[j];
        slot[j] = zi_load(last + j);
        zi_store(dst + j, h + (before - h) * zi_load(w + j));
    }
}

extern "C" int zi_token_shift(void* out, int out_dt, int64_t ldo, const void* x, int x_dt, int64_t ldx, const void* w,
                              int w_dt, float* state, int64_t state_stride, const int32_t* tok_seq,
                              const int32_t* tok_pos, const int32_t* entry_start, const int32_t* entry_len,
                              const int32_t* entry_slot, int n, int hidden, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && hidden > 0 && ldx >= hidden && ldo >= hidden && state_stride >= hidden,
               "token_shift: bad sizes n=%d hidden=%d", n, hidden);
    ZI_REQUIRE(out != x, "token_shift: the result cannot overwrite its input (a row reads the one before it)");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(x_dt, TX, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
        token_shift_kernel<TX, TW, TO><<<n, 256, 0, stream>>>((TO*)out, ldo, (const TX*)x, ldx, (const TW*)w, state,
                                                              state_stride, tok_seq, tok_pos, entry_start, entry_len,
                                                              entry_slot, hidden);
    })));
    return zi_check_launch("token_shift");
}

template <typename TD, typename TR>
__global__ void __launch_bounds__(256)
stream_reenter_kernel(float* __restrict__ resid, const TD* __restrict__ delta, int splits, int64_t split_stride,
                      const float* __restrict__ again, const TR* __restrict__ row, int64_t total, int H) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
        float v = resid[i];
        for (int s = 0; s < splits; ++s) v += zi_load(delta + s * split_stride + i);
        if (again) v += again[i];
        if (row) v += zi_load(row + i % H);
        resid[i] = v;
    }
}

// resid [n][hidden] float32, in place.  `delta`: `splits` terms [n][hidden] of type delta_dt, split_stride apart
// (added first, in rising order), or null; `again` float32 [n][hidden] or null; `row` [hidden] or null.
extern "C" int zi_stream_reenter(float* resid, const void* delta, int delta_dt, int splits, int64_t split_stride,
                                 const float* again, const void* row, int row_dt, int n, int hidden,
                                 hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && hidden > 0 && splits >= 0, "stream_reenter: bad sizes");
    if (n == 0) return 0;
    if (!delta) splits = 0;
    const int64_t total = (int64_t)n * hidden;
    const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    ZI_DISPATCH_DTYPE(splits ? delta_dt : ZI_F32, TD, ZI_DISPATCH_DTYPE(row ? row_dt : ZI_F32, TR, {
        stream_reenter_kernel<TD, TR><<<blocks, 256, 0, stream>>>(resid, (const TD*)delta, splits, split_stride, again,
                                                                  (const TR*)row, total, hidden);
    }));
    return zi_check_launch("stream_reenter");
}
