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
#define LA_PARTS (ZI_WAVE / LA_COLS)    // lanes that share a column: lane (c, p) holds rows p * R .. p * R + R - 1
#define LA_WAVES 4                      // wavefronts of a workgroup: they share the staged tokens
#define LA_WCOLS (LA_COLS * LA_WAVES)   // columns of S a workgroup holds

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

// x of the lane that `CTRL` names within this lane's row of 16 lanes (quad permutations, mirrors)
template <int CTRL>
__device__ __forceinline__ float la_dpp(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
// the sum over the 16 lanes of a row, in every one of them
__device__ __forceinline__ float la_row_sum(float x) {
    x += la_dpp<0xB1>(x);       // quad_perm [1, 0, 3, 2]
    x += la_dpp<0x4E>(x);       // quad_perm [2, 3, 0, 1]
    x += la_dpp<0x141>(x);      // row_half_mirror
    x += la_dpp<0x140>(x);      // row_mirror
    return x;
}

// where element e of a staged row lies: 16 bytes are skipped every 64 floats, so that the 16-byte reads of the
// sixteen lanes of a row (lane p reads R consecutive floats from p * R) fall into different banks
__device__ __forceinline__ constexpr int la_place(int e) { return e + (e >> 6) * 4; }

// A workgroup of LA_WAVES wavefronts per (entry, head, LA_WCOLS columns of S); a wavefront holds LA_COLS of
// them, lane (c, p) rows p * R .. p * R + R - 1 of column c in registers.  k, q (and the decays) of TC tokens at a
// time lie in LDS, activated and scaled as they are put there (once, not by every lane that reads them); the next
// TC tokens are asked for before the present ones are worked on and go into the other buffer afterwards, so no
// token waits for memory.  Nothing but the state's own multiply-add chains one token to the next: the read-outs
// of a chunk's tokens are summed over the lanes together, after the chunk.
template <int R, int TC, bool GATED>
__global__ void __launch_bounds__(LA_WAVES* ZI_WAVE)
linear_attention_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ q, const float* __restrict__ k,
                        const float* __restrict__ v, int64_t ld, const float* __restrict__ decay, int64_t ld_decay,
                        const float* __restrict__ head_decay, float* __restrict__ state, int64_t state_stride,
                        const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_len,
                        const int32_t* __restrict__ entry_past, const int32_t* __restrict__ entry_slot, int heads,
                        int dim, int vdim, int act, float qscale, int share, int decay_heads) {
    constexpr int D = LA_PARTS * R;               // rows the lanes of a column hold
    constexpr int DP = la_place(D);               // floats of a staged row
    constexpr int NSEG = GATED ? 3 : 2;           // k, q (, decay)
    constexpr int THREADS = LA_WAVES * ZI_WAVE;
    constexpr int PSEG = TC * D / THREADS;        // values of k (or q, or the decay) of a chunk a thread stages
    constexpr int PRE = NSEG * PSEG;
    static_assert(PSEG * THREADS == TC * D, "a chunk's rows divide evenly over the threads");
    static_assert(TC <= LA_PARTS && TC * LA_WCOLS <= THREADS, "a chunk's read-outs are written by the lanes of a row");
    __shared__ __attribute__((aligned(16))) float rows[2][TC][NSEG][DP];
    __shared__ float vs[2][TC][LA_WCOLS];
    const int tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int c = lane / LA_PARTS, p = lane % LA_PARTS;
    const int head = blockIdx.y, e = blockIdx.z;
    const int col0 = blockIdx.x * LA_WCOLS, col = col0 + wave * LA_COLS + c;
    const bool live = col < vdim;
    const int colc = live ? col : vdim - 1;
    const int t0 = entry_start[e], len = entry_len[e];
    if (len <= 0) return;
    float* S_ = state + (int64_t)entry_slot[e] * state_stride + (int64_t)head * dim * vdim;
    const bool fresh = entry_past[e] == 0;      // a sequence's first tokens: the state is zero whatever the slot holds
    float S[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = p * R + r;
        S[r] = (!fresh && row < dim) ? S_[(int64_t)row * vdim + colc] : 0.f;
    }
    const float hd = head_decay ? head_decay[head] : 1.f;
    // `share` heads in a row read the same q and k; a decay of one number a (token, head) is staged for every row
    const int64_t qk_at = (int64_t)(head / share) * dim, v_at = (int64_t)head * vdim;

    // global -> registers: the chunk of tokens from `base` on.  Every load is issued, from addresses clamped into
    // the entry; what a thread must not use is zeroed when it goes to LDS.
    float pre[PRE], vpre;
    unsigned ok_bits = 0;
    bool v_ok = false;
    auto fetch = [&](int base) __attribute__((always_inline)) {
        const int n_in = len - base;      // tokens of the chunk (more than TC: all TC; none or fewer past the end)
        const int tb = t0 + (base < len ? base : len - 1);
        ok_bits = 0;
#pragma unroll
        for (int seg = 0; seg < NSEG; ++seg) {      // which array a pass reads is known when the loop is unrolled
            const float* src = seg == 0 ? k : (seg == 1 ? q : decay);
            const int64_t stride = seg == 2 ? ld_decay : ld;
#pragma unroll
            for (int u = 0; u < PSEG; ++u) {
                const int idx = u * THREADS + tid, tt = idx / D, d = idx % D;
                const bool ok = tt < n_in && d < dim;
                const int64_t at = seg == 2 ? (decay_heads ? (int64_t)head : (int64_t)head * dim + (ok ? d : 0))
                                            : qk_at + (ok ? d : 0);
                pre[seg * PSEG + u] = src[(int64_t)(tb + (ok ? tt : 0)) * stride + at];
                ok_bits |= (unsigned)ok << (seg * PSEG + u);
            }
        }
        const int tt = tid / LA_WCOLS, cc = tid % LA_WCOLS;
        v_ok = tid < TC * LA_WCOLS && tt < n_in && col0 + cc < vdim;
        vpre = v[(int64_t)(tb + (v_ok ? tt : 0)) * ld + v_at + (v_ok ? col0 + cc : 0)];
    };
    auto stash = [&](int b) __attribute__((always_inline)) {
#pragma unroll
        for (int seg = 0; seg < NSEG; ++seg)
#pragma unroll
            for (int u = 0; u < PSEG; ++u) {
                const int idx = u * THREADS + tid, tt = idx / D, d = idx % D;
                float x = ((ok_bits >> (seg * PSEG + u)) & 1u) ? pre[seg * PSEG + u] : 0.f;
                if (seg < 2 && act) x = la_silu(x);
                if (seg == 1) x *= qscale;
                rows[b][tt][seg][la_place(d)] = x;
            }
        if (tid < TC * LA_WCOLS) {
            const float x = v_ok ? vpre : 0.f;
            vs[b][tid / LA_WCOLS][tid % LA_WCOLS] = act ? la_silu(x) : x;
        }
    };
    auto work = [&](int base, int b) __attribute__((always_inline)) {
        const int n_in = len - base;
        float accs[TC];
#pragma unroll
        for (int tt = 0; tt < TC; ++tt) {
            accs[tt] = 0.f;
            if (tt < n_in) {
                float kk[R], qq[R], aa[R];
                const float* kr = &rows[b][tt][0][la_place(p * R)];
                const float* qr = &rows[b][tt][1][la_place(p * R)];
                const float* ar = &rows[b][tt][NSEG - 1][la_place(p * R)];
                if constexpr (R == 2) {
                    const float2 k2 = *reinterpret_cast<const float2*>(kr), q2 = *reinterpret_cast<const float2*>(qr);
                    kk[0] = k2.x; kk[1] = k2.y; qq[0] = q2.x; qq[1] = q2.y;
                    if constexpr (GATED) {
                        const float2 a2 = *reinterpret_cast<const float2*>(ar);
                        aa[0] = a2.x; aa[1] = a2.y;
                    }
                } else {
#pragma unroll
                    for (int r4 = 0; r4 < R; r4 += 4) {
                        const float4 k4 = *reinterpret_cast<const float4*>(kr + r4), q4 = *reinterpret_cast<const float4*>(qr + r4);
                        kk[r4] = k4.x; kk[r4 + 1] = k4.y; kk[r4 + 2] = k4.z; kk[r4 + 3] = k4.w;
                        qq[r4] = q4.x; qq[r4 + 1] = q4.y; qq[r4 + 2] = q4.z; qq[r4 + 3] = q4.w;
                        if constexpr (GATED) {
                            const float4 a4 = *reinterpret_cast<const float4*>(ar + r4);
                            aa[r4] = a4.x; aa[r4 + 1] = a4.y; aa[r4 + 2] = a4.z; aa[r4 + 3] = a4.w;
                        }
                    }
                }
                const float vv = vs[b][tt][wave * LA_COLS + c];
                float acc = 0.f;
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    S[r] = (GATED ? aa[r] : hd) * S[r] + kk[r] * vv;
                    acc += S[r] * qq[r];
                }
                accs[tt] = acc;
            }
        }
        float mine = 0.f;
#pragma unroll
        for (int tt = 0; tt < TC; ++tt) {
            const float total = la_row_sum(accs[tt]);
            if (p == tt) mine = total;
        }
        // lane (c, p) writes token p's read-out of column c
        if (live && p < TC && p < n_in) out[(int64_t)(t0 + base + p) * ldo + (int64_t)head * vdim + col] = mine;
    };
    fetch(0);
    stash(0);
    __syncthreads();
    int cur = 0;
    for (int base = 0; base < len; base += TC, cur ^= 1) {
        fetch(base + TC);
        work(base, cur);
        stash(cur ^ 1);
        __syncthreads();
    }
    if (live) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int row = p * R + r;
            if (row < dim) S_[(int64_t)row * vdim + col] = S[r];
        }
    }
}

// The same recurrence for steps in which every entry brings ONE token: a workgroup per (entry, head) streams the
// head's matrix through once, a wavefront a row at a time (64 consecutive columns a load: whole lines of memory),
// the rows dealt out over the four wavefronts; the read-out's four partial sums are added in the wavefronts' order.
// Its sums add up in another order than the kernel's above, so a token decoded alone and the same token inside a
// portion agree within rounding, not to the bit.
#define LA_STEP_MAX_DIM 512
__global__ void __launch_bounds__(LA_WAVES* ZI_WAVE)
linear_attention_step_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ q, const float* __restrict__ k,
                             const float* __restrict__ v, int64_t ld, const float* __restrict__ decay, int64_t ld_decay,
                             const float* __restrict__ head_decay, float* __restrict__ state, int64_t state_stride,
                             const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_len,
                             const int32_t* __restrict__ entry_past, const int32_t* __restrict__ entry_slot, int dim,
                             int vdim, int act, float qscale, int share, int decay_heads) {
    __shared__ float ks[LA_STEP_MAX_DIM], qs[LA_STEP_MAX_DIM], as[LA_STEP_MAX_DIM];
    __shared__ float part[LA_WAVES][ZI_WAVE];
    const int head = blockIdx.x, e = blockIdx.y, tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    if (entry_len[e] != 1) return;
    const int64_t t = entry_start[e];
    const bool fresh = entry_past[e] == 0;
    float* S = state + (int64_t)entry_slot[e] * state_stride + (int64_t)head * dim * vdim;
    const float hd = head_decay ? head_decay[head] : 1.f;
    const float at = (decay && decay_heads) ? decay[t * ld_decay + head] : hd;
    for (int d = tid; d < dim; d += LA_WAVES * ZI_WAVE) {
        float kk = k[t * ld + (int64_t)(head / share) * dim + d], qq = q[t * ld + (int64_t)(head / share) * dim + d];
        if (act) {
            kk = la_silu(kk);
            qq = la_silu(qq);
        }
        ks[d] = kk;
        qs[d] = qq * qscale;
        as[d] = (decay && !decay_heads) ? decay[t * ld_decay + (int64_t)head * dim + d] : at;
    }
    __syncthreads();
    for (int c0 = 0; c0 < vdim; c0 += ZI_WAVE) {
        const int col = c0 + lane;
        const bool live = col < vdim;
        const int cc = live ? col : vdim - 1;
        float vv = v[t * ld + (int64_t)head * vdim + cc];
        if (act) vv = la_silu(vv);
        float acc = 0.f;
        int row = wave;
        for (; row + 7 * LA_WAVES < dim; row += 8 * LA_WAVES) {      // eight rows' loads in flight
            float sv[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) sv[u] = fresh ? 0.f : S[(int64_t)(row + u * LA_WAVES) * vdim + cc];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int r = row + u * LA_WAVES;
                sv[u] = as[r] * sv[u] + ks[r] * vv;
                acc += sv[u] * qs[r];
                if (live) S[(int64_t)r * vdim + col] = sv[u];
            }
        }
        for (; row < dim; row += LA_WAVES) {
            float sv = fresh ? 0.f : S[(int64_t)row * vdim + cc];
            sv = as[row] * sv + ks[row] * vv;
            acc += sv * qs[row];
            if (live) S[(int64_t)row * vdim + col] = sv;
        }
        part[wave][lane] = acc;
        __syncthreads();
        if (wave == 0 && live) {
            float total = part[0][lane];
#pragma unroll
            for (int w = 1; w < LA_WAVES; ++w) total += part[w][lane];
            out[t * ldo + (int64_t)head * vdim + col] = total;
        }
        __syncthreads();
    }
}

// out [n][heads*vdim] float32 (row stride ldo).  q, k [n][(heads/share)*dim] and v [n][heads*vdim]: float32, one row
// stride `ld` (columns of one projection); `share` heads in a row read the same q and k.  decay float32 (row stride
// ld_decay): [n][heads*dim], or with `decay_heads` [n][heads], one factor a (token, head); or null; head_decay
// [heads] or null (then 1).  state [slots][state_stride] float32, of which this layer's heads*dim*vdim floats start at
// the pointer given.  act 1: SiLU of q, k and v as they are read.  q is multiplied by qscale.  single_tokens: the
// caller says that every entry brings one token (entries that do not are left alone): the kernel that streams a head's
// matrix through once takes the step.
extern "C" int zi_linear_attention_grouped(float* out, int64_t ldo, const float* q, const float* k, const float* v,
                                           int64_t ld, const float* decay, int64_t ld_decay, const float* head_decay,
                                           float* state, int64_t state_stride, const int32_t* entry_start,
                                           const int32_t* entry_len, const int32_t* entry_past,
                                           const int32_t* entry_slot, int entries, int heads, int dim, int vdim, int act,
                                           float qscale, int share, int decay_heads, int single_tokens,
                                           hipStream_t stream) {
    ZI_REQUIRE(entries >= 0 && entries <= 65535 && heads > 0 && heads <= 65535 && dim > 0 && vdim > 0,
               "linear_attention: bad sizes");
    ZI_REQUIRE(share > 0 && heads % share == 0, "linear_attention: %d heads do not share q and k in runs of %d", heads, share);
    ZI_REQUIRE(dim <= 512, "linear_attention: dim %d is more than the 512 rows a wavefront holds", dim);
    ZI_REQUIRE(state_stride >= (int64_t)heads * dim * vdim, "linear_attention: the state row is too short");
    ZI_REQUIRE(ldo >= (int64_t)heads * vdim && ld >= (int64_t)(heads / share) * dim && ld >= (int64_t)heads * vdim &&
               (!decay || ld_decay >= (int64_t)heads * (decay_heads ? 1 : dim)), "linear_attention: row stride too small");
    ZI_REQUIRE(!decay_heads || decay, "linear_attention: a decay a head and token must be given");
    ZI_REQUIRE(act == 0 || act == 1, "linear_attention: unknown activation %d", act);
    if (entries == 0) return 0;
    if (single_tokens) {
        linear_attention_step_kernel<<<dim3(heads, entries), LA_WAVES * ZI_WAVE, 0, stream>>>(
            out, ldo, q, k, v, ld, decay, ld_decay, head_decay, state, state_stride, entry_start, entry_len, entry_past,
            entry_slot, dim, vdim, act, qscale, share, decay_heads);
        return zi_check_launch("linear_attention_step");
    }
    const dim3 grid((vdim + LA_WCOLS - 1) / LA_WCOLS, heads, entries);
#define ZI_LA(R, TC)                                                                                                 \
    if (decay)                                                                                                       \
        linear_attention_kernel<R, TC, true><<<grid, LA_WAVES * ZI_WAVE, 0, stream>>>(                               \
            out, ldo, q, k, v, ld, decay, ld_decay, head_decay, state, state_stride, entry_start, entry_len,         \
            entry_past, entry_slot, heads, dim, vdim, act, qscale, share, decay_heads);                              \
    else                                                                                                             \
        linear_attention_kernel<R, TC, false><<<grid, LA_WAVES * ZI_WAVE, 0, stream>>>(                              \
            out, ldo, q, k, v, ld, decay, ld_decay, head_decay, state, state_stride, entry_start, entry_len,         \
            entry_past, entry_slot, heads, dim, vdim, act, qscale, share, decay_heads)
    if (dim <= 32) { ZI_LA(2, 16); }
    else if (dim <= 64) { ZI_LA(4, 16); }
    else if (dim <= 128) { ZI_LA(8, 16); }
    else if (dim <= 256) { ZI_LA(16, 8); }
    else { ZI_LA(32, 4); }
#undef ZI_LA
    return zi_check_launch("linear_attention");
}

extern "C" int zi_linear_attention(float* out, int64_t ldo, const float* q, const float* k, const float* v, int64_t ld,
                                   const float* decay, int64_t ld_decay, const float* head_decay, float* state,
                                   int64_t state_stride, const int32_t* entry_start, const int32_t* entry_len,
                                   const int32_t* entry_past, const int32_t* entry_slot, int entries, int heads,
                                   int dim, int vdim, int act, float qscale, hipStream_t stream) {
    return zi_linear_attention_grouped(out, ldo, q, k, v, ld, decay, ld_decay, head_decay, state, state_stride,
                                       entry_start, entry_len, entry_past, entry_slot, entries, heads, dim, vdim, act,
                                       qscale, 1, 0, 0, stream);
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
