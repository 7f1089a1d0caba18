// A selective state-space mixer with one decay a head and token (the state-space-duality form), around the
// linear-attention kernel: what comes before the recurrence and what comes after it.
//
// The stacked input projection of a token is [z: inner | x: inner | B: groups*N | C: groups*N | dt: heads], float32,
// inner = heads * vdim.  x, B and C pass a short causal convolution per channel (weights [channels][taps], the last
// tap weighs the token itself, with a bias) and SiLU; rows before an entry's first token come from the tail kept in
// the request's state slot (its first (taps - 1) * channels floats, zero for a fresh request; `zi_conv_tail` moves
// it on afterwards).  dt <- softplus(dt + dt_bias).  The recurrence of head h,
//     S_t = exp(-exp(A_log_h) dt_t) S_{t-1} + dt_t B_t x_t^T,   y_t = S_t^T C_t + D_h x_t,
// is `zi_linear_attention_grouped` with keys B, queries C (heads of a group share them), values dt_t x_t and one
// decay a (token, head).  `zi_ssm_prepare` leaves, for every token, the row
//     [x: inner | B: groups*N | C: groups*N | dt x: inner | decay: heads]
// and `zi_ssm_finish` makes (y + D x) * silu(z), divides every one of `norm_groups` equal parts of it by its root
// mean square, and multiplies by a gain a channel.  Everything here is float32 but the last store.
#include "zi_common.h"
#include "zi_api.h"

#define SSM_THREADS 256
#define SSM_MAX_TAPS 16

__device__ __forceinline__ float ssm_silu(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float ssm_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

__global__ void __launch_bounds__(SSM_THREADS)
ssm_prepare_kernel(float* __restrict__ out, int64_t ldo, const float* __restrict__ proj, int64_t ld,
                   const float* __restrict__ conv_w, const float* __restrict__ conv_b, const float* __restrict__ dt_bias,
                   const float* __restrict__ a_log, const float* __restrict__ state, int64_t state_stride,
                   const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ entry_start,
                   const int32_t* __restrict__ entry_slot, int heads, int vdim, int gn2, int taps) {
    const int t = blockIdx.x;
    const int e = tok_seq[t];
    const int local = t - entry_start[e];
    const int inner = heads * vdim, C = inner + gn2;
    const float* tail = state + (int64_t)entry_slot[e] * state_stride;
    const float* row = proj + (int64_t)t * ld;
    float* orow = out + (int64_t)t * ldo;
    // (a token's channels are dealt out over the workgroups of its row of the launch)
    for (int c = blockIdx.y * SSM_THREADS + threadIdx.x; c < C; c += gridDim.y * SSM_THREADS) {
        float acc = conv_b ? conv_b[c] : 0.f;
        for (int j = 0; j < taps; ++j) {
            const int li = local - (taps - 1) + j;
            const float u = li >= 0 ? proj[(int64_t)(t - local + li) * ld + inner + c]
                                    : tail[(int64_t)(li + taps - 1) * C + c];
            acc += conv_w[(int64_t)c * taps + j] * u;
        }
        const float x = ssm_silu(acc);
        orow[c] = x;
        if (c < inner) {
            const int h = c / vdim;
            const float dt = ssm_softplus(row[2 * inner + gn2 + h] + dt_bias[h]);
            orow[C + c] = dt * x;
        }
    }
    for (int h = blockIdx.y * SSM_THREADS + threadIdx.x; h < heads; h += gridDim.y * SSM_THREADS) {
        const float dt = ssm_softplus(row[2 * inner + gn2 + h] + dt_bias[h]);
        orow[C + inner + h] = expf(-expf(a_log[h]) * dt);
    }
}

// out [n][2 inner + gn2 + heads] float32 (row stride ldo); proj [n][2 inner + gn2 + heads] float32 (row stride ld);
// gn2 = 2 * groups * N; conv_w [inner + gn2][taps], conv_b [inner + gn2] (or null), dt_bias, a_log [heads]: float32.
// state [slots][state_stride] float32, the convolution's tail first.
extern "C" int zi_ssm_prepare(float* out, int64_t ldo, const float* proj, int64_t ld, int n, const float* conv_w,
                              const float* conv_b, const float* dt_bias, const float* a_log, const float* state,
                              int64_t state_stride, const int32_t* tok_seq, const int32_t* entry_start,
                              const int32_t* entry_slot, int heads, int vdim, int gn2, int taps, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && heads > 0 && vdim > 0 && gn2 >= 0 && taps >= 1 && taps <= SSM_MAX_TAPS, "ssm_prepare: bad sizes");
    const int64_t inner = (int64_t)heads * vdim, width = 2 * inner + gn2 + heads;
    ZI_REQUIRE(ld >= width && ldo >= width, "ssm_prepare: a row is too short");
    ZI_REQUIRE(state_stride >= (int64_t)(taps - 1) * (inner + gn2), "ssm_prepare: the state row is too short");
    if (n == 0) return 0;
    // few tokens: a workgroup for every 256 channels of a token, so that a step of decoded tokens fills more of the chip
    const int64_t C = inner + gn2;
    int per_token = n >= 1024 ? 1 : (int)((C + SSM_THREADS - 1) / SSM_THREADS);
    if (per_token > 64) per_token = 64;
    ssm_prepare_kernel<<<dim3(n, per_token), SSM_THREADS, 0, stream>>>(out, ldo, proj, ld, conv_w, conv_b, dt_bias, a_log, state,
                                                      state_stride, tok_seq, entry_start, entry_slot, heads, vdim, gn2,
                                                      taps);
    return zi_check_launch("ssm_prepare");
}

template <typename TO>
__global__ void __launch_bounds__(SSM_THREADS)
ssm_finish_kernel(TO* __restrict__ out, int64_t ldo, const float* __restrict__ y, int64_t ldy,
                  const float* __restrict__ x, int64_t ldx, const float* __restrict__ z, int64_t ldz,
                  const float* __restrict__ skip, const float* __restrict__ gain, int vdim, int part, float eps) {
    __shared__ float scratch[16];
    const int64_t t = blockIdx.x;
    const int c0 = blockIdx.y * part;
    float ss = 0.f;
    for (int i = threadIdx.x; i < part; i += SSM_THREADS) {
        const int c = c0 + i;
        const float g = (y[t * ldy + c] + skip[c / vdim] * x[t * ldx + c]) * ssm_silu(z[t * ldz + c]);
        ss += g * g;
    }
    ss = zi_block_sum(ss, scratch);
    const float r = 1.f / sqrtf(ss / (float)part + eps);
    for (int i = threadIdx.x; i < part; i += SSM_THREADS) {
        const int c = c0 + i;
        const float g = (y[t * ldy + c] + skip[c / vdim] * x[t * ldx + c]) * ssm_silu(z[t * ldz + c]);
        zi_store(out + t * ldo + c, g * r * gain[c]);
    }
}

// out [n][inner] = norm_parts((y + skip_h x) * silu(z)) * gain; y, x, z float32 rows of `inner` values (row strides
// ldy, ldx, ldz); skip [heads], gain [inner] float32; the norm runs over each of `parts` equal parts of a row.
extern "C" int zi_ssm_finish(void* out, int out_dt, int64_t ldo, const float* y, int64_t ldy, const float* x, int64_t ldx,
                             const float* z, int64_t ldz, const float* skip, const float* gain, int n, int heads, int vdim,
                             int parts, float eps, hipStream_t stream) {
    const int64_t inner = (int64_t)heads * vdim;
    ZI_REQUIRE(n >= 0 && heads > 0 && vdim > 0 && parts > 0 && parts <= 65535 && inner % parts == 0, "ssm_finish: bad sizes");
    ZI_REQUIRE(ldo >= inner && ldy >= inner && ldx >= inner && ldz >= inner && eps > 0.f, "ssm_finish: a row is too short");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(out_dt, TO, {
        ssm_finish_kernel<TO><<<dim3(n, parts), SSM_THREADS, 0, stream>>>((TO*)out, ldo, y, ldy, x, ldx, z, ldz, skip, gain,
                                                                         vdim, (int)(inner / parts), eps);
    });
    return zi_check_launch("ssm_finish");
}
