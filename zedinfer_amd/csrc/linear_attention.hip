// Linear attention with a decayed matrix state per head, token by token:
//
//     S_t = diag(a_t) S_{t-1} + k_t v_t^T        (S: dim x vdim, float32, zero at a sequence's start)
//     o_t = S_t^T q_t
//
// The decay a_t is a factor for every ROW of S (a key channel): either given per token and channel (gated linear
// attention), or one constant per head (a fixed geometric decay).  q, k and v are float32 rows of a projection; an
// activation (SiLU) and a scale of q may be applied as they are loaded.
//
//   zi_lowrank_decay     a = sigmoid(W2 u + b)^(1/tau) for u = W1 h given as float32 rows: exp(logsigmoid(z) / tau)
//   zi_linear_attention  the recurrence over the tokens of every entry, state in the request's slot
//   zi_gate_heads        y = x * act(gate) * scale over heads that may be padded in x
//
// The recurrence runs token by token in prompts too: a token's sums are made in the same order whatever the cut of
// the prompt into steps, so portions, batches and whole prompts agree to the last bit.
#include "zi_common.h"
#include "zi_api.h"

#define LA_COLS 4                       // columns of S a wavefront holds
#define LA_PARTS (ZI_WAVE / LA_COLS)    // lanes that share a column: lane (c, p) holds rows p, p + 16, ...

__device__ __forceinline__ float la_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float la_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }

template <typename TW>
__global__ void __launch_bounds__(256)
lowrank_decay_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ u, int64_t ldu,
                     const TW* __restrict__ w2, const TW* __restrict__ bias, int C, int rank, float inv_tau) {
    extern __shared__ float us[];
    const int64_t t = blockIdx.x;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) us[i] = u[t * ldu + i];
    __syncthreads();
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
        float z = bias ? zi_load(bias + c) : 0.f;
        const TW* wr = w2 + (int64_t)c * rank;
        for (int i = 0; i < rank; ++i) z += zi_load(wr + i) * us[i];
        // log sigmoid(z) = min(z, 0) - log1p(exp(-|z|)), exact for large |z| too
        const float ls = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
        out[t * ldo + c] = expf(ls * inv_tau);
    }
}

// out [n][C] float32 (row stride ldo); u [n][rank] float32 (row stride ldu); w2 [C][rank], bias [C] or null.
extern "C" int zi_lowrank_decay(float* out, int64_t ldo, const float* u, int64_t ldu, const void* w2, const void* bias,
                                int w_dt, int n, int channels, int rank, float tau, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && channels > 0 && rank > 0 && rank <= 8192 && ldo >= channels && ldu >= rank && tau > 0.f,
               "lowrank_decay: bad sizes");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(w_dt, TW, {
        lowrank_decay_kernel<TW><<<n, 256, rank * sizeof(float), stream>>>(out, ldo, u, ldu, (const TW*)w2,
                                                                           (const TW*)bias, channels, rank, 1.f / tau);
    });
    return zi_check_launch("lowrank_decay");
}

// One wavefront per (entry, head, LA_COLS columns of S).  R rows a lane.  The next token's operands are asked
// for before the present token is worked on.
template <int R>
__global__ void __launch_bounds__(ZI_WAVE)
linear_attention_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ q, const float* __restrict__ k,
                        const float* __restrict__ v, int64_t ld, const float* __restrict__ decay, int64_t ld_decay,
                        const float* __restrict__ head_decay, float* __restrict__ state, int64_t state_stride,
                        const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_len,
                        const int32_t* __restrict__ entry_past, const int32_t* __restrict__ entry_slot, int heads,
                        int dim, int vdim, int act, float qscale) {
    const int lane = threadIdx.x, c = lane / LA_PARTS, p = lane % LA_PARTS;
    const int head = blockIdx.y, e = blockIdx.z;
    const int col = blockIdx.x * LA_COLS + c;
    const bool live = col < vdim;
    const int colc = live ? col : vdim - 1;
    const int t0 = entry_start[e], len = entry_len[e];
    float* S_ = state + (int64_t)entry_slot[e] * state_stride + (int64_t)head * dim * vdim;
    const bool fresh = entry_past[e] == 0;      // a sequence's first tokens: the state is zero whatever the slot holds
    float S[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = r * LA_PARTS + p;
        S[r] = (!fresh && row < dim) ? S_[(int64_t)row * vdim + colc] : 0.f;
    }
    const float hd = head_decay ? head_decay[head] : 1.f;
    const int64_t qk_at = (int64_t)head * dim, v_at = (int64_t)head * vdim + colc;
    float kq[R], qq[R], aq[R], vq;
    auto load = [&](int t, float* kk, float* qv, float* av, float& vv) {
        const int64_t base = (int64_t)t * ld;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = r * LA_PARTS + p;
            const bool in = row < dim;
            kk[r] = in ? k[base + qk_at + row] : 0.f;
            qv[r] = in ? q[base + qk_at + row] : 0.f;
            av[r] = decay ? (in ? decay[(int64_t)t * ld_decay + qk_at + row] : 0.f) : hd;
        }
        vv = v[base + v_at];
    };
    if (len > 0) load(t0, kq, qq, aq, vq);
    for (int i = 0; i < len; ++i) {
        float kn[R], qn[R], an[R], vn = 0.f;
        if (i + 1 < len) load(t0 + i + 1, kn, qn, an, vn);
        float vv = vq;
        if (act) vv = la_silu(vv);
        float acc = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float kk = kq[r], qv = qq[r];
            if (act) {
                kk = la_silu(kk);
                qv = la_silu(qv);
            }
            S[r] = aq[r] * S[r] + kk * vv;
            acc += S[r] * (qv * qscale);
        }
#pragma unroll
        for (int o = LA_PARTS / 2; o > 0; o >>= 1) acc += __shfl_xor(acc, o, ZI_WAVE);
        if (p == 0 && live) out[(int64_t)(t0 + i) * ldo + (int64_t)head * vdim + col] = acc;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            kq[r] = kn[r];
            qq[r] = qn[r];
            aq[r] = an[r];
        }
        vq = vn;
    }
    if (live && len > 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = r * LA_PARTS + p;
            if (row < dim) S_[(int64_t)row * vdim + col] = S[r];
        }
    }
}

// out [n][heads*vdim] float32 (row stride ldo).  q, k [n][heads*dim] and v [n][heads*vdim]: float32, one row stride
// `ld` (columns of one projection).  decay [n][heads*dim] float32 (row stride ld_decay) or null; head_decay [heads]
// or null (then 1).  state [slots][state_stride] float32, of which this layer's heads*dim*vdim floats start at the
// pointer given.  act 1: SiLU of q, k and v as they are read.  q is multiplied by qscale.
extern "C" int zi_linear_attention(float* out, int64_t ldo, const float* q, const float* k, const float* v, int64_t ld,
                                   const float* decay, int64_t ld_decay, const float* head_decay, float* state,
                                   int64_t state_stride, const int32_t* entry_start, const int32_t* entry_len,
                                   const int32_t* entry_past, const int32_t* entry_slot, int entries, int heads,
                                   int dim, int vdim, int act, float qscale, hipStream_t stream) {
    ZI_REQUIRE(entries >= 0 && entries <= 65535 && heads > 0 && heads <= 65535 && dim > 0 && vdim > 0,
               "linear_attention: bad sizes");
    ZI_REQUIRE(dim <= 512, "linear_attention: dim %d is more than the 512 rows a wavefront holds", dim);
    ZI_REQUIRE(state_stride >= (int64_t)heads * dim * vdim, "linear_attention: the state row is too short");
    ZI_REQUIRE(ldo >= (int64_t)heads * vdim && ld >= (int64_t)heads * dim && ld >= (int64_t)heads * vdim &&
               (!decay || ld_decay >= (int64_t)heads * dim), "linear_attention: row stride too small");
    ZI_REQUIRE(act == 0 || act == 1, "linear_attention: unknown activation %d", act);
    if (entries == 0) return 0;
    const dim3 grid((vdim + LA_COLS - 1) / LA_COLS, heads, entries);
#define ZI_LA(R)                                                                                                    \
    linear_attention_kernel<R><<<grid, ZI_WAVE, 0, stream>>>(out, ldo, q, k, v, ld, decay, ld_decay, head_decay,    \
                                                             state, state_stride, entry_start, entry_len, entry_past, \
                                                             entry_slot, heads, dim, vdim, act, qscale)
    if (dim <= 32) ZI_LA(2);
    else if (dim <= 64) ZI_LA(4);
    else if (dim <= 128) ZI_LA(8);
    else if (dim <= 256) ZI_LA(16);
    else ZI_LA(32);
#undef ZI_LA
    return zi_check_launch("linear_attention");
}

#define GATE_SIGMOID 0
#define GATE_SILU 1

template <typename TX, typename TO>
__global__ void __launch_bounds__(256)
gate_heads_kernel(TO* __restrict__ out, int64_t ldo, const TX* __restrict__ x, int64_t ldx, int x_head,
                  const float* __restrict__ gate, int64_t ld_gate, int width, int head, int act, float scale) {
    const int64_t t = blockIdx.x;
    for (int j = threadIdx.x; j < width; j += blockDim.x) {
        const float g = gate[t * ld_gate + j];
        const float a = act == GATE_SILU ? la_silu(g) : la_sigmoid(g);
        const float xv = zi_load(x + t * ldx + (int64_t)(j / head) * x_head + j % head);
        zi_store(out + t * ldo + j, xv * a * scale);
    }
}

// out [n][width] = x * act(gate) * scale; x holds heads of x_head >= head values of which the first `head` count
// (x[t][(j / head) * x_head + j % head]); gate float32 [n][width] (row stride ld_gate).
extern "C" int zi_gate_heads(void* out, int out_dt, int64_t ldo, const void* x, int x_dt, int64_t ldx, int x_head,
                             const float* gate, int64_t ld_gate, int n, int width, int head, int act, float scale,
                             hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && width > 0 && head > 0 && width % head == 0 && x_head >= head && ldo >= width &&
               ld_gate >= width && ldx >= (int64_t)(width / head) * x_head, "gate_heads: bad sizes");
    ZI_REQUIRE(act == GATE_SIGMOID || act == GATE_SILU, "gate_heads: unknown activation %d", act);
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(x_dt, TX, ZI_DISPATCH_DTYPE(out_dt, TO, {
        gate_heads_kernel<TX, TO><<<n, 256, 0, stream>>>((TO*)out, ldo, (const TX*)x, ldx, x_head, gate, ld_gate, width,
                                                         head, act, scale);
    }));
    return zi_check_launch("gate_heads");
}
