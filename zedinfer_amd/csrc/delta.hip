// The gated delta rule: a recurrent mixer whose state per head is a matrix S [dim][vdim], float32.
//
//   for every token, per head:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//
// with q, k unit vectors (q also times dim^-1/2), beta in (0, 1) and the decay g in (0, 1).  q, k and v come out
// of a short causal convolution over time (per channel, `taps` taps, the last one the current token's) and SiLU.
// A request's state is S and, for the convolution, the last taps - 1 rows that entered it; both live in one
// float32 row per request slot: [heads][dim][vdim] first, then [taps - 1][channels].
//
// Everything here is float32 arithmetic.  Three launches a step: `zi_delta_prepare` (convolution, SiLU, unit
// vectors, beta, g, for every token at once), `zi_delta_conv_state` (the new tail of the convolution's input),
// `zi_delta_rule` (the recurrence, token by token within an entry, entries and heads and columns in parallel).
#include "zi_common.h"
#include "zi_api.h"

__device__ __forceinline__ float delta_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float delta_softplus(float z) { return z > 30.f ? z : log1pf(expf(z)); }

// proj [n][ld]: columns [q (kvh*dim) | k (kvh*dim) | v (heads*vdim) | gate (heads*vdim) | b (heads) | a (heads)].
// One workgroup per (token, unit): a unit is one head of q or k (its dim channels, and their unit length), or 256
// channels of v; the first unit of a token also makes its beta and g.
#define DELTA_UNIT 256

__device__ __forceinline__ float delta_conv(const float* __restrict__ proj, int64_t ld, const float* __restrict__ conv_w,
                                            const float* __restrict__ tail, int t, int local, int c, int C, int taps) {
    float y = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int li = local - (taps - 1) + j;
        const float x = li >= 0 ? proj[(int64_t)(t - local + li) * ld + c] : tail[(int64_t)(li + taps - 1) * C + c];
        y += conv_w[(int64_t)c * taps + j] * x;
    }
    return delta_silu(y);
}

__global__ void __launch_bounds__(DELTA_UNIT)
delta_prepare_kernel(float* __restrict__ qk, float* __restrict__ v, float* __restrict__ beta_g,
                     const float* __restrict__ proj, int64_t ld, const float* __restrict__ conv_w,
                     const float* __restrict__ a_log, const float* __restrict__ dt_bias, const float* __restrict__ state,
                     int64_t state_stride, int64_t conv_off, const int32_t* __restrict__ tok_seq,
                     const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_slot, int heads,
                     int kvh, int dim, int vdim, int taps) {
    __shared__ float red[16];
    const int t = blockIdx.x, unit = blockIdx.y, e = tok_seq[t];
    const int local = t - entry_start[e];
    const int qkc = 2 * kvh * dim, C = qkc + heads * vdim;
    const float* tail = state + (int64_t)entry_slot[e] * state_stride + conv_off;      // [taps - 1][C]
    if (unit < 2 * kvh) {
        // dim may exceed the workgroup: a thread takes channels threadIdx.x, threadIdx.x + 256, ...
        float x[2] = {0.f, 0.f}, ss = 0.f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int d = threadIdx.x + i * DELTA_UNIT;
            if (d < dim) x[i] = delta_conv(proj, ld, conv_w, tail, t, local, unit * dim + d, C, taps);
            ss += x[i] * x[i];
        }
        ss = zi_block_sum(ss, red);
        const float r = (1.f / sqrtf(ss + 1e-6f)) * (unit < kvh ? 1.f / sqrtf((float)dim) : 1.f);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int d = threadIdx.x + i * DELTA_UNIT;
            if (d < dim) qk[(int64_t)t * qkc + unit * dim + d] = x[i] * r;
        }
    } else {
        const int c = (unit - 2 * kvh) * DELTA_UNIT + threadIdx.x;
        if (c < heads * vdim) v[(int64_t)t * heads * vdim + c] = delta_conv(proj, ld, conv_w, tail, t, local, qkc + c, C, taps);
    }
    if (unit == 0) {
        const float* row = proj + (int64_t)t * ld + C + heads * vdim;      // b, then a
        for (int h = threadIdx.x; h < heads; h += blockDim.x) {
            beta_g[(int64_t)t * 2 * heads + h] = 1.f / (1.f + expf(-row[h]));
            const float step = delta_softplus(row[heads + h] + dt_bias[h]);
            beta_g[(int64_t)t * 2 * heads + heads + h] = expf(-expf(a_log[h]) * step);
        }
    }
}

extern "C" int zi_delta_prepare(float* qk, float* v, float* beta_g, const float* proj, int64_t ld, int n,
                                const void* conv_w, const void* a_log, const void* dt_bias, int w_dt, const float* state,
                                int64_t state_stride, int64_t conv_off, const int32_t* tok_seq, const int32_t* entry_start,
                                const int32_t* entry_slot, int heads, int kvh, int dim, int vdim, int taps,
                                hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && heads > 0 && kvh > 0 && heads % kvh == 0 && dim > 0 && vdim > 0 && taps >= 1,
               "delta_prepare: bad sizes");
    ZI_REQUIRE(w_dt == ZI_F32, "delta_prepare: the convolution's taps, A_log and dt_bias are float32");
    ZI_REQUIRE(dim <= 2 * DELTA_UNIT, "delta_prepare: dim %d is more than %d", dim, 2 * DELTA_UNIT);
    const int64_t C = 2LL * kvh * dim + (int64_t)heads * vdim;
    ZI_REQUIRE(ld >= C + (int64_t)heads * vdim + 2 * heads, "delta_prepare: row stride too small");
    ZI_REQUIRE(state_stride >= conv_off + (int64_t)(taps - 1) * C, "delta_prepare: the state row is too short");
    const int units = 2 * kvh + (heads * vdim + DELTA_UNIT - 1) / DELTA_UNIT;
    ZI_REQUIRE(units <= 65535, "delta_prepare: too many channels");
    if (n == 0) return 0;
    delta_prepare_kernel<<<dim3(n, units), DELTA_UNIT, 0, stream>>>(
        qk, v, beta_g, proj, ld, (const float*)conv_w, (const float*)a_log, (const float*)dt_bias, state, state_stride,
        conv_off, tok_seq, entry_start, entry_slot, heads, kvh, dim, vdim, taps);
    return zi_check_launch("delta_prepare");
}

// The convolution's new tail: the last taps - 1 rows of the sequence so far, from this step's rows and, where the
// entry brought fewer, from the old tail.  A thread reads all it needs of the old tail before it writes.
#define DELTA_MAX_TAPS 16

__global__ void __launch_bounds__(256)
delta_conv_state_kernel(float* __restrict__ state, int64_t state_stride, int64_t conv_off,
                        const float* __restrict__ proj, int64_t ld, const int32_t* __restrict__ entry_start,
                        const int32_t* __restrict__ entry_len, const int32_t* __restrict__ entry_slot, int C, int taps) {
    const int e = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int start = entry_start[e], len = entry_len[e];
    float* tail = state + (int64_t)entry_slot[e] * state_stride + conv_off;
    float keep[DELTA_MAX_TAPS];
#pragma unroll
    for (int k = 0; k < DELTA_MAX_TAPS; ++k) {
        if (k >= taps - 1) break;
        const int li = len - (taps - 1) + k;
        float x = 0.f;
        if (li >= 0) x = proj[(int64_t)(start + li) * ld + c];
        else x = tail[(int64_t)(li + taps - 1) * C + c];
        keep[k] = x;
    }
#pragma unroll
    for (int k = 0; k < DELTA_MAX_TAPS; ++k) {
        if (k >= taps - 1) break;
        tail[(int64_t)k * C + c] = keep[k];
    }
}

extern "C" int zi_delta_conv_state(float* state, int64_t state_stride, int64_t conv_off, const float* proj, int64_t ld,
                                   const int32_t* entry_start, const int32_t* entry_len, const int32_t* entry_slot,
                                   int entries, int channels, int taps, hipStream_t stream) {
    ZI_REQUIRE(entries >= 0 && entries <= 65535 && channels > 0 && taps >= 1 && taps - 1 <= DELTA_MAX_TAPS,
               "delta_conv_state: bad sizes (at most %d taps)", DELTA_MAX_TAPS + 1);
    ZI_REQUIRE(ld >= channels && state_stride >= conv_off + (int64_t)(taps - 1) * channels,
               "delta_conv_state: a row is too short");
    if (entries == 0 || taps == 1) return 0;
    delta_conv_state_kernel<<<dim3((channels + 255) / 256, entries), 256, 0, stream>>>(
        state, state_stride, conv_off, proj, ld, entry_start, entry_len, entry_slot, channels, taps);
    return zi_check_launch("delta_conv_state");
}

// The recurrence.  One wavefront per (entry, head, 8 columns of S): lane (col, part) = 8 col + part holds the R rows
// part R ... part R + R - 1 of column col, so a dot product over dim is an eighth of it in every lane and three
// exchanges among 8 neighbouring lanes (data-parallel-primitive moves, no trip through LDS).  (Sixteen parts and 4
// columns a wavefront were measured too: a prompt of 2,048 tokens 1.07 against 1.22 ms a layer, but decoded tokens
// 23 against 14 us, the state then being read in pieces of 16 bytes.)
// With S the state before the token, the token's read-out needs no second pass over the updated state:
//     a = S^T k,  b = S^T q   (two dot products over the same registers, reduced together)
//     u = beta (v - g a);     o = g b + (k . q) u;     S <- g S + k u^T
// which is the rule's S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q with the products regrouped.  k . q
// does not depend on the state: it is made when the tokens are put into LDS.  The order of all additions is fixed
// by dim alone.  q, k, v, beta and g of TOKS tokens at a time lie in LDS; the next TOKS tokens' are requested
// before the present ones are worked on and put into the other LDS buffer afterwards, so no token waits for memory.
#define DELTA_COLS 8
#define DELTA_PARTS 8
#define DELTA_TOKS 8

// x of the lane that `ctrl` names within this lane's row of 16 (quad permutations, mirrors)
template <int CTRL>
__device__ __forceinline__ float delta_dpp(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true));
}
// the sum over the 8 lanes of a half row, in every one of them: neighbours, pairs of neighbours, the other quad of
// the half (lane 7 - i)
__device__ __forceinline__ float delta_row_sum(float x) {
    x += delta_dpp<0xB1>(x);       // quad_perm [1, 0, 3, 2]
    x += delta_dpp<0x4E>(x);       // quad_perm [2, 3, 0, 1]
    x += delta_dpp<0x141>(x);      // row_half_mirror
    return x;
}

template <int R>      // rows a lane holds: dim <= 8 R; R is a multiple of 4
__global__ void __launch_bounds__(ZI_WAVE)
delta_rule_kernel(float* __restrict__ out, const float* __restrict__ qk, const float* __restrict__ v,
                  const float* __restrict__ beta_g, float* __restrict__ state, int64_t state_stride,
                  const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_len,
                  const int32_t* __restrict__ entry_slot, int heads, int kvh, int dim, int vdim) {
    constexpr int D = DELTA_PARTS * R, PRE = DELTA_TOKS * D * 2 / ZI_WAVE;
    __shared__ __attribute__((aligned(16))) float qks[2][2][DELTA_TOKS][D];      // [buffer][q, k][token][d]
    __shared__ float vs[2][DELTA_TOKS][DELTA_COLS];
    __shared__ float bg[2][DELTA_TOKS][2];
    __shared__ float kq[2][DELTA_TOKS];
    const int e = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
    const int col0 = blockIdx.x * DELTA_COLS, col = col0 + lane / DELTA_PARTS, part = lane % DELTA_PARTS;
    const bool live = col < vdim;
    const int kh = h / (heads / kvh), qkc = 2 * kvh * dim;
    const int start = entry_start[e], len = entry_len[e];
    float* S = state + (int64_t)entry_slot[e] * state_stride + (int64_t)h * dim * vdim;
    float s[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int d = part * R + i;
        s[i] = (live && d < dim) ? S[(int64_t)d * vdim + col] : 0.f;
    }
    float pre[PRE], pre_v = 0.f, pre_bg = 0.f;
    // request the tokens t0 .. t0 + TOKS - 1 of the entry (those past its end, and rows past dim: zeros)
    auto request = [&](int t0) {
#pragma unroll
        for (int i = 0; i < PRE; ++i) {
            const int idx = lane + ZI_WAVE * i, which = idx / (DELTA_TOKS * D), tt = (idx / D) % DELTA_TOKS, d = idx % D;
            pre[i] = (t0 + tt < len && d < dim) ? qk[(int64_t)(start + t0 + tt) * qkc + (which * kvh + kh) * dim + d] : 0.f;
        }
        if (lane < DELTA_TOKS * DELTA_COLS) {
            const int tt = lane / DELTA_COLS, c = col0 + lane % DELTA_COLS;
            pre_v = (t0 + tt < len && c < vdim) ? v[((int64_t)(start + t0 + tt) * heads + h) * vdim + c] : 0.f;
        }
        if (lane < 2 * DELTA_TOKS)
            pre_bg = t0 + lane / 2 < len ? beta_g[(int64_t)(start + t0 + lane / 2) * 2 * heads + (lane % 2) * heads + h] : 0.f;
    };
    auto put = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PRE; ++i) (&qks[buf][0][0][0])[lane + ZI_WAVE * i] = pre[i];
        if (lane < DELTA_TOKS * DELTA_COLS) (&vs[buf][0][0])[lane] = pre_v;
        if (lane < 2 * DELTA_TOKS) (&bg[buf][0][0])[lane] = pre_bg;
        __syncthreads();
        // k . q of the TOKS tokens: eight lanes a token
        const int tt = lane / 8, sub = lane % 8;
        float acc = 0.f;
        for (int d = sub; d < D; d += 8) acc += qks[buf][0][tt][d] * qks[buf][1][tt][d];
        acc += __shfl_xor(acc, 1, ZI_WAVE);
        acc += __shfl_xor(acc, 2, ZI_WAVE);
        acc += __shfl_xor(acc, 4, ZI_WAVE);
        if (sub == 0) kq[buf][tt] = acc;
    };
    request(0);
    put(0);
    __syncthreads();
    int buf = 0;
    for (int t0 = 0; t0 < len; t0 += DELTA_TOKS, buf ^= 1) {
        const int cnt = len - t0 < DELTA_TOKS ? len - t0 : DELTA_TOKS;
        if (t0 + DELTA_TOKS < len) request(t0 + DELTA_TOKS);
        // a token's k, q and scalars are read from LDS into registers while the token before it is worked on
        // (1.00 against 1.13 ms for a layer's 2,048 tokens)
        struct Tok {
            float4 k[R / 4], q[R / 4];
            float beta, g, kq, v;
        };
        auto fetch = [&](Tok& x, int tt) {
            const float4* kk = reinterpret_cast<const float4*>(&qks[buf][1][tt][part * R]);
            const float4* qq = reinterpret_cast<const float4*>(&qks[buf][0][tt][part * R]);
#pragma unroll
            for (int i = 0; i < R / 4; ++i) {
                x.k[i] = kk[i];
                x.q[i] = qq[i];
            }
            x.beta = bg[buf][tt][0];
            x.g = bg[buf][tt][1];
            x.kq = kq[buf][tt];
            x.v = vs[buf][tt][lane / DELTA_PARTS];
        };
        auto work = [&](const Tok& x, int tt) {
            float a0 = 0.f, a1 = 0.f, b0 = 0.f, b1 = 0.f;
#pragma unroll
            for (int i = 0; i < R / 4; ++i) {
                a0 += s[4 * i] * x.k[i].x;
                a1 += s[4 * i + 1] * x.k[i].y;
                a0 += s[4 * i + 2] * x.k[i].z;
                a1 += s[4 * i + 3] * x.k[i].w;
                b0 += s[4 * i] * x.q[i].x;
                b1 += s[4 * i + 1] * x.q[i].y;
                b0 += s[4 * i + 2] * x.q[i].z;
                b1 += s[4 * i + 3] * x.q[i].w;
            }
            const float a = delta_row_sum(a0 + a1), b = delta_row_sum(b0 + b1);
            const float u = x.beta * (x.v - x.g * a);
            if (live && part == 0) out[((int64_t)(start + t0 + tt) * heads + h) * vdim + col] = x.g * b + x.kq * u;
#pragma unroll
            for (int i = 0; i < R / 4; ++i) {
                s[4 * i] = x.g * s[4 * i] + x.k[i].x * u;
                s[4 * i + 1] = x.g * s[4 * i + 1] + x.k[i].y * u;
                s[4 * i + 2] = x.g * s[4 * i + 2] + x.k[i].z * u;
                s[4 * i + 3] = x.g * s[4 * i + 3] + x.k[i].w * u;
            }
        };
        Tok even, odd;
        fetch(even, 0);
#pragma unroll
        for (int tt = 0; tt < DELTA_TOKS; tt += 2) {
            if (tt + 1 < cnt) fetch(odd, tt + 1);
            if (tt < cnt) work(even, tt);
            if (tt + 2 < cnt) fetch(even, tt + 2);
            if (tt + 1 < cnt) work(odd, tt + 1);
        }
        if (t0 + DELTA_TOKS < len) put(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int d = part * R + i;
        if (live && d < dim) S[(int64_t)d * vdim + col] = s[i];
    }
}

extern "C" int zi_delta_rule(float* out, const float* qk, const float* v, const float* beta_g, float* state,
                             int64_t state_stride, const int32_t* entry_start, const int32_t* entry_len,
                             const int32_t* entry_slot, int entries, int heads, int kvh, int dim, int vdim,
                             hipStream_t stream) {
    ZI_REQUIRE(entries >= 0 && entries <= 65535 && heads > 0 && heads <= 65535 && kvh > 0 && heads % kvh == 0 && dim > 0 &&
               vdim > 0, "delta_rule: bad sizes");
    ZI_REQUIRE(dim <= 256, "delta_rule: dim %d is more than the 256 rows a wavefront holds", dim);
    ZI_REQUIRE(state_stride >= (int64_t)heads * dim * vdim, "delta_rule: the state row is too short");
    if (entries == 0) return 0;
    const dim3 grid((vdim + DELTA_COLS - 1) / DELTA_COLS, heads, entries);
#define ZI_DELTA_RULE(R)                                                                                         \
    delta_rule_kernel<R><<<grid, ZI_WAVE, 0, stream>>>(out, qk, v, beta_g, state, state_stride, entry_start,      \
                                                       entry_len, entry_slot, heads, kvh, dim, vdim)
    if (dim <= 32) ZI_DELTA_RULE(4);
    else if (dim <= 64) ZI_DELTA_RULE(8);
    else if (dim <= 128) ZI_DELTA_RULE(16);
    else ZI_DELTA_RULE(32);
#undef ZI_DELTA_RULE
    return zi_check_launch("delta_rule");
}

// o [rows][vdim] (a row per token and head) divided by its root mean square, times a weight [vdim], times
// an activation of a gate read from gate[token][head * vdim + e] with row stride ld_gate (act 0: SiLU, 1: sigmoid),
// times `scale`; the result goes to out[token][head * vdim + e] with row stride ldo.  A wavefront per row.
template <typename TO, typename TW>
__global__ void __launch_bounds__(256)
gated_rmsnorm_kernel(TO* __restrict__ out, int64_t ldo, const float* __restrict__ o, const TW* __restrict__ w,
                     const float* __restrict__ gate, int64_t ld_gate, int rows, int heads, int vdim, float eps, int act,
                     float scale) {
    const int lane = threadIdx.x % ZI_WAVE;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x / ZI_WAVE) + threadIdx.x / ZI_WAVE;
    if (row >= rows) return;
    const float* orow = o + row * vdim;
    float ss = 0.f;
    for (int j = lane; j < vdim; j += ZI_WAVE) ss += orow[j] * orow[j];
    ss = zi_wave_sum(ss);
    const float rstd = 1.f / sqrtf(ss / (float)vdim + eps);
    const float* grow = gate + (row / heads) * ld_gate + (row % heads) * vdim;
    TO* dst = out + (row / heads) * ldo + (row % heads) * vdim;
    for (int j = lane; j < vdim; j += ZI_WAVE) {
        const float g = grow[j];
        const float a = act == 1 ? 1.f / (1.f + expf(-g)) : delta_silu(g);
        zi_store(dst + j, orow[j] * rstd * zi_load(w + j) * a * scale);
    }
}

extern "C" int zi_gated_rmsnorm_act(void* out, int out_dt, int64_t ldo, const float* o, const void* w, int w_dt,
                                    const float* gate, int64_t ld_gate, int n, int heads, int vdim, float eps, int act,
                                    float scale, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && heads > 0 && vdim > 0 && eps > 0.f && ld_gate >= (int64_t)heads * vdim &&
               ldo >= (int64_t)heads * vdim, "gated_rmsnorm: bad sizes");
    ZI_REQUIRE(act == 0 || act == 1, "gated_rmsnorm: unknown gate activation %d", act);
    if (n == 0) return 0;
    const int rows = n * heads;
    ZI_DISPATCH_DTYPE(out_dt, TO, ZI_DISPATCH_DTYPE(w_dt, TW, {
        gated_rmsnorm_kernel<TO, TW><<<(rows + 3) / 4, 256, 0, stream>>>((TO*)out, ldo, o, (const TW*)w, gate, ld_gate,
                                                                         rows, heads, vdim, eps, act, scale);
    }));
    return zi_check_launch("gated_rmsnorm");
}

extern "C" int zi_gated_rmsnorm(void* out, int out_dt, const float* o, const void* w, int w_dt, const float* gate,
                                int64_t ld_gate, int n, int heads, int vdim, float eps, hipStream_t stream) {
    return zi_gated_rmsnorm_act(out, out_dt, (int64_t)heads * vdim, o, w, w_dt, gate, ld_gate, n, heads, vdim, eps, 0, 1.f,
                                stream);
}
