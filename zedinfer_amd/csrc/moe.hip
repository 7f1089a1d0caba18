// Mixture of experts, all on the device: nothing of a step's routing is seen by the host, so a step's launches
// are the same whatever the tokens choose (a step can be recorded and replayed).
//
//   zi_moe_route    z [n][E] float32 router logits -> s = softmax(z); choice = s + correction; the `top` experts
//                   of largest choice (the lowest index among equals), weights s * scale
//   zi_moe_route_table  the experts of a token are read from a table by its id, equal weights
//   zi_moe_group    the (token, choice) pairs sorted by expert: offsets, the order and its inverse, and the list
//                   of row tiles (expert, first row, rows) that the products walk
//   zi_moe_linear   out[row] = act(W[expert of row] . x[source of row]) for every row of the sorted order
//   zi_moe_combine  out[t] = sum_k weight[t][k] * y[place of (t, k)], float32, k in rising order
//
// A row's sums depend on its own values and its expert's weights only, never on where in the order it stands.
#include "zi_common.h"
#include "zi_api.h"

#define MOE_MAX_EXPERTS 1024
#define MOE_PER_LANE (MOE_MAX_EXPERTS / ZI_WAVE)

template <int PER>
__global__ void __launch_bounds__(256)
moe_route_kernel(int32_t* __restrict__ idx, float* __restrict__ wt, const float* __restrict__ z,
                 const float* __restrict__ correction, int n, int E, int top, float scale) {
    const int lane = threadIdx.x % ZI_WAVE;
    const int t = blockIdx.x * (blockDim.x / ZI_WAVE) + threadIdx.x / ZI_WAVE;
    if (t >= n) return;
    float s[PER], choice[PER];
    float m = -INFINITY;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = lane + i * ZI_WAVE;
        s[i] = e < E ? z[(int64_t)t * E + e] : -INFINITY;
        m = fmaxf(m, s[i]);
    }
    m = zi_wave_max(m);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = lane + i * ZI_WAVE;
        s[i] = e < E ? expf(s[i] - m) : 0.f;
        sum += s[i];
    }
    sum = zi_wave_sum(sum);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = lane + i * ZI_WAVE;
        s[i] = s[i] / sum;
        choice[i] = e < E ? s[i] + correction[e] : -INFINITY;
    }
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY, best_s = 0.f;
        int best_e = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = lane + i * ZI_WAVE;
            if (e < E && (choice[i] > best || (choice[i] == best && e < best_e))) {
                best = choice[i];
                best_e = e;
                best_s = s[i];
            }
        }
#pragma unroll
        for (int o = ZI_WAVE / 2; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, ZI_WAVE), os = __shfl_xor(best_s, o, ZI_WAVE);
            const int oe = __shfl_xor(best_e, o, ZI_WAVE);
            if (ob > best || (ob == best && oe < best_e)) {
                best = ob;
                best_e = oe;
                best_s = os;
            }
        }
        if (lane == 0) {
            idx[(int64_t)t * top + k] = best_e;
            wt[(int64_t)t * top + k] = best_s * scale;
        }
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (lane + i * ZI_WAVE == best_e) choice[i] = -INFINITY;
    }
}

extern "C" int zi_moe_route(int32_t* idx, float* wt, const float* z, const float* correction, int n, int experts,
                            int top, float scale, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && experts > 0 && experts <= MOE_MAX_EXPERTS && top > 0 && top <= experts,
               "moe_route: bad sizes (experts %d, top %d; at most %d experts)", experts, top, MOE_MAX_EXPERTS);
    if (n == 0) return 0;
    const int blocks = (n + 3) / 4;
#define ZI_MOE_ROUTE(PER) moe_route_kernel<PER><<<blocks, 256, 0, stream>>>(idx, wt, z, correction, n, experts, top, scale)
    if (experts <= ZI_WAVE) ZI_MOE_ROUTE(1);
    else if (experts <= 2 * ZI_WAVE) ZI_MOE_ROUTE(2);
    else if (experts <= 4 * ZI_WAVE) ZI_MOE_ROUTE(4);
    else ZI_MOE_ROUTE(MOE_PER_LANE);
#undef ZI_MOE_ROUTE
    return zi_check_launch("moe_route");
}

// The other router: the `top` largest logits themselves are chosen (the lowest index among equals) and the weights
// are the softmax over the chosen logits only.  z [n][E] float32; `bias` [E] (or null) is added to it first.
template <int PER>
__global__ void __launch_bounds__(256)
moe_route_top_kernel(int32_t* __restrict__ idx, float* __restrict__ wt, const float* __restrict__ z,
                     const float* __restrict__ bias, int n, int E, int top) {
    const int lane = threadIdx.x % ZI_WAVE;
    const int t = blockIdx.x * (blockDim.x / ZI_WAVE) + threadIdx.x / ZI_WAVE;
    if (t >= n) return;
    float choice[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = lane + i * ZI_WAVE;
        choice[i] = e < E ? z[(int64_t)t * E + e] + (bias ? bias[e] : 0.f) : -INFINITY;
    }
    float first = 0.f, sum = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int best_e = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = lane + i * ZI_WAVE;
            if (e < E && (choice[i] > best || (choice[i] == best && e < best_e))) {
                best = choice[i];
                best_e = e;
            }
        }
#pragma unroll
        for (int o = ZI_WAVE / 2; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, ZI_WAVE);
            const int oe = __shfl_xor(best_e, o, ZI_WAVE);
            if (ob > best || (ob == best && oe < best_e)) {
                best = ob;
                best_e = oe;
            }
        }
        if (k == 0) first = best;      // the largest of all: the softmax's maximum
        const float p = expf(best - first);
        sum += p;
        if (lane == 0) {
            idx[(int64_t)t * top + k] = best_e;
            wt[(int64_t)t * top + k] = p;
        }
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (lane + i * ZI_WAVE == best_e) choice[i] = -INFINITY;
    }
    if (lane == 0)
        for (int k = 0; k < top; ++k) wt[(int64_t)t * top + k] /= sum;
}

extern "C" int zi_moe_route_top(int32_t* idx, float* wt, const float* z, const float* bias, int n, int experts, int top,
                                hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && experts > 0 && experts <= MOE_MAX_EXPERTS && top > 0 && top <= experts,
               "moe_route_top: bad sizes (experts %d, top %d; at most %d experts)", experts, top, MOE_MAX_EXPERTS);
    if (n == 0) return 0;
    const int blocks = (n + 3) / 4;
#define ZI_MOE_ROUTE(PER) moe_route_top_kernel<PER><<<blocks, 256, 0, stream>>>(idx, wt, z, bias, n, experts, top)
    if (experts <= ZI_WAVE) ZI_MOE_ROUTE(1);
    else if (experts <= 2 * ZI_WAVE) ZI_MOE_ROUTE(2);
    else if (experts <= 4 * ZI_WAVE) ZI_MOE_ROUTE(4);
    else ZI_MOE_ROUTE(MOE_PER_LANE);
#undef ZI_MOE_ROUTE
    return zi_check_launch("moe_route_top");
}

// Experts named by a table instead of a router: token id v uses the experts table[v][0 .. top), each with the
// weight 1 / top.  An id outside the table, or an entry that names no expert, gives expert 0 with weight NaN so
// that the fault shows.
__global__ void __launch_bounds__(256)
moe_route_table_kernel(int32_t* __restrict__ idx, float* __restrict__ wt, const int32_t* __restrict__ ids,
                       const int32_t* __restrict__ table, int pairs, int vocab, int E, int top) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= pairs) return;
    const int id = ids[i / top];
    const int e = (id >= 0 && id < vocab) ? table[(int64_t)id * top + i % top] : -1;
    const bool ok = e >= 0 && e < E;
    idx[i] = ok ? e : 0;
    wt[i] = ok ? 1.f / (float)top : NAN;
}

extern "C" int zi_moe_route_table(int32_t* idx, float* wt, const int32_t* ids, const int32_t* table, int n, int vocab,
                                  int experts, int top, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && vocab > 0 && experts > 0 && experts <= MOE_MAX_EXPERTS && top > 0 && top <= experts,
               "moe_route_table: bad sizes (experts %d, top %d; at most %d experts)", experts, top, MOE_MAX_EXPERTS);
    if (n == 0) return 0;
    const int pairs = n * top;
    moe_route_table_kernel<<<(pairs + 255) / 256, 256, 0, stream>>>(idx, wt, ids, table, pairs, vocab, experts, top);
    return zi_check_launch("moe_route_table");
}

// One workgroup sorts the M = n * top pairs by expert (a counting sort; within an expert the order is the order
// of arrival, which no result depends on).  plan: [0] = number of row tiles, then [1 + 3 i ...] = (expert, first
// row, rows) of tile i; order[place] = pair, place_of[pair] = place.
__global__ void __launch_bounds__(1024)
moe_group_kernel(int32_t* __restrict__ plan, int32_t* __restrict__ order, int32_t* __restrict__ place_of,
                 const int32_t* __restrict__ idx, int M, int E, int tile_rows) {
    __shared__ int count[MOE_MAX_EXPERTS], first[MOE_MAX_EXPERTS], tile0[MOE_MAX_EXPERTS], cursor[MOE_MAX_EXPERTS];
    for (int e = threadIdx.x; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < M; i += blockDim.x) {
        const int e = idx[i];
        if ((unsigned)e < (unsigned)E) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, tiles = 0;
        for (int e = 0; e < E; ++e) {
            first[e] = at;
            tile0[e] = tiles;
            at += count[e];
            tiles += (count[e] + tile_rows - 1) / tile_rows;
        }
        plan[0] = tiles;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x) {
        cursor[e] = first[e];
        for (int r = 0, i = tile0[e]; r < count[e]; r += tile_rows, ++i) {
            plan[1 + 3 * i] = e;
            plan[2 + 3 * i] = first[e] + r;
            plan[3 + 3 * i] = count[e] - r < tile_rows ? count[e] - r : tile_rows;
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < M; i += blockDim.x) {
        const int e = idx[i];
        if ((unsigned)e >= (unsigned)E) continue;
        const int at = atomicAdd(&cursor[e], 1);
        order[at] = i;
        place_of[i] = at;
    }
}

extern "C" int zi_moe_group(int32_t* plan, int32_t* order, int32_t* place_of, const int32_t* idx, int pairs,
                            int experts, int tile_rows, hipStream_t stream) {
    ZI_REQUIRE(pairs >= 0 && experts > 0 && experts <= MOE_MAX_EXPERTS && tile_rows > 0, "moe_group: bad sizes");
    moe_group_kernel<<<1, 1024, 0, stream>>>(plan, order, place_of, idx, pairs, experts, tile_rows);
    return zi_check_launch("moe_group");
}

#define MOE_ACT_NONE 0
#define MOE_ACT_GELU_ERF 1

__device__ __forceinline__ void moe_store4(float* p, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
__device__ __forceinline__ void moe_store4(zi_bf16* p, float a, float b, float c, float d) {
    uint2 v;
    v.x = zi_pack_bf16x2(a, b);
    v.y = zi_pack_bf16x2(c, d);
    *reinterpret_cast<uint2*>(p) = v;
}

__device__ __forceinline__ float moe_act(float z, int act) {
    return act == MOE_ACT_GELU_ERF ? 0.5f * z * (1.f + erff(z * 0.70710678118654752440f)) : z;
}

// The plain product: a workgroup of 256 threads makes 16 rows x 64 columns, k in blocks of 32 through LDS.
#define MOE_TM 16
#define MOE_TN 64
#define MOE_KC 32

template <typename TX, typename TW, typename TO>
__global__ void __launch_bounds__(256)
moe_linear_kernel(TO* __restrict__ out, int64_t ldo, const TX* __restrict__ x, int64_t ldx, const TW* __restrict__ w,
                  const int32_t* __restrict__ plan, const int32_t* __restrict__ source, int source_div, int N, int K,
                  int act) {
    __shared__ float xs[MOE_TM][MOE_KC + 1], ws[MOE_TN][MOE_KC + 1];
    __shared__ int src[MOE_TM];
    const int tile = blockIdx.y;
    if (tile >= plan[0]) return;
    const int e = plan[1 + 3 * tile], r0 = plan[2 + 3 * tile], rows = plan[3 + 3 * tile];
    const int n0 = blockIdx.x * MOE_TN;
    if (threadIdx.x < MOE_TM) {
        const int r = r0 + (threadIdx.x < rows ? threadIdx.x : 0);
        src[threadIdx.x] = source ? source[r] / source_div : r;
    }
    const TW* we = w + (int64_t)e * N * K;
    const int c = threadIdx.x % MOE_TN, rg = threadIdx.x / MOE_TN;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += MOE_KC) {
        __syncthreads();
        for (int i = threadIdx.x; i < MOE_TM * MOE_KC; i += 256) {
            const int r = i / MOE_KC, kk = i % MOE_KC;
            xs[r][kk] = k0 + kk < K ? zi_load(x + (int64_t)src[r] * ldx + k0 + kk) : 0.f;
        }
        for (int i = threadIdx.x; i < MOE_TN * MOE_KC; i += 256) {
            const int cc = i / MOE_KC, kk = i % MOE_KC;
            ws[cc][kk] = (n0 + cc < N && k0 + kk < K) ? zi_load(we + (int64_t)(n0 + cc) * K + k0 + kk) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < MOE_KC; ++kk) {
            const float wv = ws[c][kk];
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] += xs[rg * 4 + i][kk] * wv;
        }
    }
    if (n0 + c >= N) return;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = rg * 4 + i;
        if (r < rows) zi_store(out + (int64_t)(r0 + r) * ldo + n0 + c, moe_act(acc[i], act));
    }
}

// The same on the matrix cores (bfloat16 operands, float32 sums): a wavefront makes 16 columns of RT tiles of 16
// rows; the expert's weight rows are the first operand (lane: row l % 16, eight k from 8 (l / 16)), the tokens'
// rows the second, so a lane ends with four neighbouring columns of one row.  Operands come straight from memory:
// the weights are read once per tile of rows.
typedef __attribute__((ext_vector_type(8))) __bf16 moe_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float moe_f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned moe_u32x4_t;
union moe_pack {
    moe_u32x4_t u;
    moe_bf16x8_t b;
};

template <typename TO, int RT, int CT>      // a wavefront makes RT tiles of 16 rows x CT tiles of 16 columns
__global__ void __launch_bounds__(256)
moe_linear_mfma_kernel(TO* __restrict__ out, int64_t ldo, const zi_bf16* __restrict__ x, int64_t ldx,
                       const zi_bf16* __restrict__ w, const int32_t* __restrict__ plan,
                       const int32_t* __restrict__ source, int source_div, int N, int K, int act) {
    const int tile = blockIdx.y;
    if (tile >= plan[0]) return;
    const int e = plan[1 + 3 * tile], r0 = plan[2 + 3 * tile], rows = plan[3 + 3 * tile];
    const int lane = threadIdx.x % ZI_WAVE, wave = threadIdx.x / ZI_WAVE;
    const int r = lane % 16, j = lane / 16;
    const int n0 = (blockIdx.x * 4 + wave) * 16 * CT;
    if (n0 >= N) return;
    const zi_bf16* wrow[CT];
#pragma unroll
    for (int c = 0; c < CT; ++c) {
        const int wn = n0 + 16 * c + r < N ? n0 + 16 * c + r : N - 1;
        wrow[c] = w + ((int64_t)e * N + wn) * K;
    }
    const zi_bf16* xrow[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int rr = t * 16 + r < rows ? t * 16 + r : 0;
        xrow[t] = x + (int64_t)(source ? source[r0 + rr] / source_div : r0 + rr) * ldx;
    }
    moe_f32x4_t acc[RT][CT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int c = 0; c < CT; ++c) acc[t][c] = (moe_f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll 2
    for (int k0 = 0; k0 < K; k0 += 32) {
        const int k = k0 + 8 * j;
        const bool in = k < K;      // K is a multiple of 8: a piece of eight lies inside or outside
        const int kc = in ? k : 0;
        const unsigned mask = 0u - (unsigned)in;
        moe_pack a[CT], b[RT];
#pragma unroll
        for (int c = 0; c < CT; ++c) a[c].u = *reinterpret_cast<const moe_u32x4_t*>(wrow[c] + kc) & mask;
#pragma unroll
        for (int t = 0; t < RT; ++t) b[t].u = *reinterpret_cast<const moe_u32x4_t*>(xrow[t] + kc) & mask;
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
            for (int c = 0; c < CT; ++c)
                acc[t][c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[c].b, b[t].b, acc[t][c], 0, 0, 0);
    }
    // a lane holds four consecutive columns of a row: one store of 16 (float32) or 8 bytes (bfloat16) where the rows
    // allow it
    const bool whole = ldo % 4 == 0 && ((uintptr_t)out % 16) == 0;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int row = t * 16 + r;
        if (row >= rows) continue;
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            const int n = n0 + 16 * c + 4 * j;
            TO* dst = out + (int64_t)(r0 + row) * ldo + n;
            if (whole && n + 3 < N) {
                moe_store4(dst, moe_act(acc[t][c][0], act), moe_act(acc[t][c][1], act), moe_act(acc[t][c][2], act),
                           moe_act(acc[t][c][3], act));
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (n + i < N) zi_store(dst + i, moe_act(acc[t][c][i], act));
            }
        }
    }
}

extern "C" int zi_moe_linear(void* out, int out_dt, int64_t ldo, const void* x, int x_dt, int64_t ldx, const void* w,
                             int w_dt, const int32_t* plan, const int32_t* source, int source_div, int max_tiles,
                             int tile_rows, int N, int K, int act, hipStream_t stream) {
    ZI_REQUIRE(max_tiles >= 0 && max_tiles <= 65535 && N > 0 && K > 0 && ldx >= K && ldo >= N && source_div > 0,
               "moe_linear: bad sizes");
    ZI_REQUIRE(act == MOE_ACT_NONE || act == MOE_ACT_GELU_ERF, "moe_linear: unknown activation %d", act);
    if (max_tiles == 0) return 0;
    const dim3 grid((N + MOE_TN - 1) / MOE_TN, max_tiles);
    const bool cores = x_dt == ZI_BF16 && w_dt == ZI_BF16 && K % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x % 16) == 0 &&
                       ((uintptr_t)w % 16) == 0 && (tile_rows == 16 || tile_rows == 32 || tile_rows == 64);
    // tiles of 64 rows (many rows an expert: prompts): a wavefront makes 64 columns of them, so that an operand of
    // the tokens serves four of the weights'; smaller tiles (decoded tokens) are bound by the weights' stream
#define ZI_MOE_CORES(RT, CT)                                                                                       \
    moe_linear_mfma_kernel<TO, RT, CT><<<dim3((N + 64 * CT - 1) / (64 * CT), max_tiles), 256, 0, stream>>>(         \
        (TO*)out, ldo, (const zi_bf16*)x, ldx, (const zi_bf16*)w, plan, source, source_div, N, K, act)
    if (cores) {
        ZI_DISPATCH_DTYPE(out_dt, TO, {
            if (tile_rows == 16) ZI_MOE_CORES(1, 1);
            else if (tile_rows == 32) ZI_MOE_CORES(2, 2);
            else ZI_MOE_CORES(4, 4);
        });
        return zi_check_launch("moe_linear");
    }
#undef ZI_MOE_CORES
    ZI_REQUIRE(tile_rows == MOE_TM, "moe_linear: the plain product walks tiles of %d rows, not %d", MOE_TM, tile_rows);
    ZI_DISPATCH_DTYPE(x_dt, TX, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
        moe_linear_kernel<TX, TW, TO><<<grid, 256, 0, stream>>>((TO*)out, ldo, (const TX*)x, ldx, (const TW*)w, plan,
                                                                 source, source_div, N, K, act);
    })));
    return zi_check_launch("moe_linear");
}

__global__ void __launch_bounds__(256)
moe_combine_kernel(float* __restrict__ out, const float* __restrict__ y, const float* __restrict__ wt,
                   const int32_t* __restrict__ place_of, int top, int H) {
    const int64_t t = blockIdx.x;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) acc += wt[t * top + k] * y[(int64_t)place_of[t * top + k] * H + c];
        out[t * H + c] = acc;
    }
}

extern "C" int zi_moe_combine(float* out, const float* y, const float* wt, const int32_t* place_of, int n, int top,
                              int hidden, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && top > 0 && hidden > 0, "moe_combine: bad sizes");
    if (n == 0) return 0;
    moe_combine_kernel<<<n, 256, 0, stream>>>(out, y, wt, place_of, top, hidden);
    return zi_check_launch("moe_combine");
}

// ---- a router of independent scores --------------------------------------------------------------------------
// s = sigmoid(z); the `top` experts with the largest s are chosen (the lowest index among equals); their weights are
// the scores themselves, not renormalised.  z [n][ld] float32 of which the first E columns are the experts'.
template <int PER>
__global__ void __launch_bounds__(256)
moe_route_sigmoid_kernel(int32_t* __restrict__ idx, float* __restrict__ wt, const float* __restrict__ z, int64_t ld,
                         int n, int E, int top) {
    const int lane = threadIdx.x % ZI_WAVE;
    const int t = blockIdx.x * (blockDim.x / ZI_WAVE) + threadIdx.x / ZI_WAVE;
    if (t >= n) return;
    float choice[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const int e = lane + i * ZI_WAVE;
        choice[i] = e < E ? 1.f / (1.f + expf(-z[(int64_t)t * ld + e])) : -INFINITY;
    }
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int best_e = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = lane + i * ZI_WAVE;
            if (e < E && (choice[i] > best || (choice[i] == best && e < best_e))) {
                best = choice[i];
                best_e = e;
            }
        }
#pragma unroll
        for (int o = ZI_WAVE / 2; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, ZI_WAVE);
            const int oe = __shfl_xor(best_e, o, ZI_WAVE);
            if (ob > best || (ob == best && oe < best_e)) {
                best = ob;
                best_e = oe;
            }
        }
        if (lane == 0) {
            idx[(int64_t)t * top + k] = best_e;
            wt[(int64_t)t * top + k] = best;
        }
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (lane + i * ZI_WAVE == best_e) choice[i] = -INFINITY;
    }
}

extern "C" int zi_moe_route_sigmoid(int32_t* idx, float* wt, const float* z, int64_t ld, int n, int experts, int top,
                                    hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && experts > 0 && experts <= MOE_MAX_EXPERTS && top > 0 && top <= experts && ld >= experts,
               "moe_route_sigmoid: bad sizes (experts %d, top %d; at most %d experts)", experts, top, MOE_MAX_EXPERTS);
    if (n == 0) return 0;
    const int blocks = (n + 3) / 4;
#define ZI_MOE_ROUTE(PER) moe_route_sigmoid_kernel<PER><<<blocks, 256, 0, stream>>>(idx, wt, z, ld, n, experts, top)
    if (experts <= ZI_WAVE) ZI_MOE_ROUTE(1);
    else if (experts <= 2 * ZI_WAVE) ZI_MOE_ROUTE(2);
    else if (experts <= 4 * ZI_WAVE) ZI_MOE_ROUTE(4);
    else ZI_MOE_ROUTE(MOE_PER_LANE);
#undef ZI_MOE_ROUTE
    return zi_check_launch("moe_route_sigmoid");
}

// The gated middle of experts whose INPUT carries the routing weight: an expert is linear up to its activation, so
// gate (w x) = w gate(x) and up (w x) = w up(x): out = silu(w g) * (w u) for row r of the grouped pairs, w the weight
// of the pair that stands at place r (wt[order[r]]).  gu [pairs][2 ff] float32 (gate, then up).
template <typename TO>
__global__ void __launch_bounds__(256)
moe_weighted_glu_kernel(TO* __restrict__ out, int64_t ldo, const float* __restrict__ gu, int64_t ld,
                        const float* __restrict__ wt, const int32_t* __restrict__ order, int pairs, int ff) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)pairs * ff) return;
    const int64_t r = i / ff, c = i % ff;
    const float w = wt[order[r]];
    const float g = w * gu[r * ld + c], u = w * gu[r * ld + ff + c];
    zi_store(out + r * ldo + c, g / (1.f + expf(-g)) * u);
}

extern "C" int zi_moe_weighted_glu(void* out, int out_dt, int64_t ldo, const float* gu, int64_t ld, const float* wt,
                                   const int32_t* order, int pairs, int ff, hipStream_t stream) {
    ZI_REQUIRE(pairs >= 0 && ff > 0 && ld >= 2 * (int64_t)ff && ldo >= ff, "moe_weighted_glu: bad sizes");
    if (pairs == 0) return 0;
    const int64_t total = (int64_t)pairs * ff;
    ZI_DISPATCH_DTYPE(out_dt, TO, {
        moe_weighted_glu_kernel<TO><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>((TO*)out, ldo, gu, ld, wt, order,
                                                                                         pairs, ff);
    });
    return zi_check_launch("moe_weighted_glu");
}

// out [n][H] = sum over a token's `top` pairs of y[place_of[pair]] (each counts once: the weight went into the
// expert's input) + sigmoid(gate[t * ld_gate]) * shared[t], where shared is the sum of `splits` float32 terms
// (`split_stride` apart) or null.
__global__ void __launch_bounds__(256)
moe_sum_shared_kernel(float* __restrict__ out, const float* __restrict__ y, const int32_t* __restrict__ place_of,
                      const float* __restrict__ shared, int splits, int64_t split_stride, const float* __restrict__ gate,
                      int64_t ld_gate, int top, int H) {
    const int64_t t = blockIdx.x;
    const float gs = (shared && gate) ? 1.f / (1.f + expf(-gate[t * ld_gate])) : 1.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) acc += y[(int64_t)place_of[t * top + k] * H + c];
        if (shared) {
            float sv = shared[t * H + c];
            for (int s = 1; s < splits; ++s) sv += shared[s * split_stride + t * H + c];
            acc += gs * sv;
        }
        out[t * H + c] = acc;
    }
}

extern "C" int zi_moe_sum_shared(float* out, const float* y, const int32_t* place_of, const float* shared, int splits,
                                 int64_t split_stride, const float* gate, int64_t ld_gate, int n, int top, int hidden,
                                 hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && top > 0 && hidden > 0 && splits >= 1, "moe_sum_shared: bad sizes");
    if (n == 0) return 0;
    moe_sum_shared_kernel<<<n, 256, 0, stream>>>(out, y, place_of, shared, splits, split_stride, gate, ld_gate, top, hidden);
    return zi_check_launch("moe_sum_shared");
}
