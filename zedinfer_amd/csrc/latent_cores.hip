// Latent attention on the matrix cores (bfloat16 cache, float32 scores and sums; see latent.hip for what is
// computed).  A row is one (token, head); all heads of a token meet the same latents, and neighbouring tokens
// nearly the same, so a workgroup takes 16 rows a wavefront of ONE entry (rows in the order token, head) and walks
// the keys its rows see in blocks of 32:
//
//   stage    the block's latents and key parts, [32][rank + rot], from the pages into LDS, rows padded by 16
//            bytes; the latents once more transposed, [rank][32], for the second product.  Neighbouring lanes take
//            neighbouring keys, so that the transposed copy's 2-byte stores fall into neighbouring LDS banks (with
//            neighbouring pieces of one key a lane, all 64 stores of an instruction met in one bank: 694 against
//            381 us for a layer's 2,048 tokens)
//   scores   S[key][row] = K . Q^T   v_mfma_f32_16x16x32_bf16: first operand the keys' rows from LDS, second the
//            queries, held in registers for the whole walk (KS operands a lane)
//   softmax  a lane holds 8 of a row's 32 scores, the row's other 24 are in 3 lanes: two lane exchanges; running
//            maximum and sum in float32, base e
//   values   O[dim][row] += C^T . P   the same instruction, contraction over the block's keys in the order in
//            which the lanes hold P (keys 4j..4j+3 and 16+4j..16+4j+3 for lane group j), the transposed latents
//            read in that order: no exchange of P between lanes
//
// A tile's keys can be cut into chunks over blockIdx.y (decoded tokens: few rows, many keys); the chunks leave
// (maximum, sum, unnormalised O) per row and a second kernel merges them.  The cut is a launch parameter that
// depends on the window and the head count only.  Which tile a workgroup owns it finds itself from the step's
// entry lengths, so the launch is sized by tokens and entries alone.
#include "zi_common.h"
#include "zi_api.h"

typedef __attribute__((ext_vector_type(8))) __bf16 la_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float la_f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned la_u32x4_t;
typedef __attribute__((ext_vector_type(2))) unsigned la_u32x2_t;
union la_pack {
    la_u32x4_t u;
    la_bf16x8_t b;
    la_u32x2_t h[2];
    unsigned w[4];
};

#define LA_BK 32      // keys a block
#define LA_PAD 8      // elements of padding of an LDS row
#define LA_EMPTY -1e30f
#define LA_BATCH 6     // requests a thread has in flight while it stages a block

// SPLIT: all WAVES wavefronts share one tile of 16 rows (decoded tokens): they stage together, each makes the
// scores again (cheap) and every WAVES-th tile of 16 latent dims of the second product.
template <int WAVES, int NT, int KS, bool SPLIT>      // rank <= 16 NT, rank + rot <= 32 KS
__global__ void __launch_bounds__(WAVES* ZI_WAVE)
latent_attention_cores_kernel(float* __restrict__ out, float* __restrict__ partial, const float* __restrict__ qa,
                              const zi_bf16* __restrict__ c_cache, const zi_bf16* __restrict__ kr_cache,
                              const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_len,
                              const int32_t* __restrict__ entry_past, const int32_t* __restrict__ block_tables,
                              int entries, int max_pages, int num_pages, int heads, int rank, int rot, int page_size,
                              int window, float scale, int chunk_keys, int total_rows) {
    constexpr int ROWS = SPLIT ? 16 : WAVES * 16, OT = SPLIT ? (NT + WAVES - 1) / WAVES : NT, KD = KS * 32, KP = KD + LA_PAD, RD = NT * 16, CP = LA_BK + LA_PAD;
    __shared__ __attribute__((aligned(16))) uint16_t krow[LA_BK * KP];
    __shared__ __attribute__((aligned(16))) uint16_t ct[RD * CP];
    int tile = blockIdx.x, e = 0;
    for (; e < entries; ++e) {
        const int tiles = (entry_len[e] * heads + ROWS - 1) / ROWS;
        if (tile < tiles) break;
        tile -= tiles;
    }
    if (e >= entries) return;      // the launch is sized for the worst case: the whole workgroup leaves
    const int len = entry_len[e], past = entry_past[e], start = entry_start[e];
    const int erows = len * heads, row0 = tile * ROWS;
    const int lane = threadIdx.x % ZI_WAVE, wave = threadIdx.x / ZI_WAVE, r = lane % 16, j = lane / 16;
    const int32_t* bt = block_tables + (int64_t)e * max_pages;
    const int qw = rank + rot;

    // the tile's keys, and this workgroup's chunk of them
    const int last_row = (row0 + ROWS < erows ? row0 + ROWS : erows) - 1;
    const int pos_first = past + row0 / heads, pos_last = past + last_row / heads;
    const int kmin = (window > 0 && pos_first - window + 1 > 0) ? pos_first - window + 1 : 0;
    int k_lo = kmin, k_hi = pos_last;
    if (chunk_keys > 0) {
        k_lo = kmin + (int)blockIdx.y * chunk_keys;
        if (k_lo + chunk_keys - 1 < k_hi) k_hi = k_lo + chunk_keys - 1;
    }

    // this lane's row
    const int row = row0 + (SPLIT ? 0 : wave * 16) + r;
    const bool row_ok = row < erows;
    const int rc = row_ok ? row : last_row;
    const int tok = start + rc / heads, head = rc % heads, pos = past + rc / heads;
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const int64_t grow = (int64_t)tok * heads + head;

    la_pack q[KS];
    {
        const float* qr = qa + grow * qw;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int d = ks * 32 + 8 * j;
            if (d < qw) {      // rank + rot is a multiple of 8: a piece of eight lies inside or outside
                const float4 a = *reinterpret_cast<const float4*>(qr + d), b = *reinterpret_cast<const float4*>(qr + d + 4);
                q[ks].w[0] = zi_pack_bf16x2(a.x, a.y);
                q[ks].w[1] = zi_pack_bf16x2(a.z, a.w);
                q[ks].w[2] = zi_pack_bf16x2(b.x, b.y);
                q[ks].w[3] = zi_pack_bf16x2(b.z, b.w);
            } else {
                q[ks].u = (la_u32x4_t){0u, 0u, 0u, 0u};
            }
        }
    }

    float m = LA_EMPTY, l = 0.f;
    la_f32x4_t o[OT];      // tile tq of this wavefront is the latent dims 16 t ..., t = tq (SPLIT: tq WAVES + wave)
#pragma unroll
    for (int t = 0; t < OT; ++t) o[t] = (la_f32x4_t){0.f, 0.f, 0.f, 0.f};

    constexpr int G = KD / 8;      // pieces of eight of a staged key
    for (int kb = k_lo; kb <= k_hi; kb += LA_BK) {
        __syncthreads();
        // requests in batches of LA_BATCH a thread, all of a batch before the first is put into LDS
        for (int i0 = threadIdx.x; i0 < LA_BK * G; i0 += WAVES * ZI_WAVE * LA_BATCH) {
            la_pack val[LA_BATCH];
#pragma unroll
            for (int u = 0; u < LA_BATCH; ++u) {
                const int i = i0 + u * WAVES * ZI_WAVE;
                const int key = i % LA_BK, d = ((i / LA_BK) % G) * 8, kp = kb + key;      // neighbouring lanes, neighbouring keys
                // addresses are clamped, not guarded (a load under a branch would make every load before it
                // wait), and what was read for a place that does not exist is masked
                const bool want = i < LA_BK * G && kp <= k_hi && d < qw;
                const int kc = kp <= k_hi ? kp : k_hi, dc = d < qw ? d : 0;
                const int pi = kc / page_size;
                const int page = bt[pi < max_pages ? pi : max_pages - 1];
                const bool held = (unsigned)page < (unsigned)num_pages;
                const int64_t slot = (int64_t)(held ? page : 0) * page_size + kc % page_size;
                const zi_bf16* src = dc < rank ? c_cache + slot * rank + dc : kr_cache + slot * rot + (dc - rank);
                const unsigned mask = 0u - (unsigned)(want && held);
                val[u].u = *reinterpret_cast<const la_u32x4_t*>(src) & mask;
            }
#pragma unroll
            for (int u = 0; u < LA_BATCH; ++u) {
                const int i = i0 + u * WAVES * ZI_WAVE;
                if (i >= LA_BK * G) break;
                const int key = i % LA_BK, d = (i / LA_BK) * 8;
                *reinterpret_cast<la_u32x4_t*>(&krow[key * KP + d]) = val[u].u;
                if (d < RD) {
                    const unsigned keep = d < rank ? 0xffffffffu : 0u;      // the key parts are no values
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        const unsigned w = val[u].w[x] & keep;
                        ct[(d + 2 * x) * CP + key] = (uint16_t)(w & 0xffffu);
                        ct[(d + 2 * x + 1) * CP + key] = (uint16_t)(w >> 16);
                    }
                }
            }
        }
        __syncthreads();

        la_f32x4_t s[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            s[h] = (la_f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                la_pack a;
                a.u = *reinterpret_cast<const la_u32x4_t*>(&krow[(h * 16 + r) * KP + ks * 32 + 8 * j]);
                s[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, q[ks].b, s[h], 0, 0, 0);
            }
        }
        // lane (r, j) holds, of row r, the keys kb + 16 h + 4 j + x
        bool ok[2][4];
        float mb = LA_EMPTY;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int kp = kb + 16 * h + 4 * j + x;
                ok[h][x] = row_ok && kp >= lo && kp <= pos && kp <= k_hi;
                s[h][x] *= scale;
                if (ok[h][x]) mb = fmaxf(mb, s[h][x]);
            }
        mb = fmaxf(mb, __shfl_xor(mb, 16, ZI_WAVE));
        mb = fmaxf(mb, __shfl_xor(mb, 32, ZI_WAVE));
        const float m_new = fmaxf(m, mb);
        const float corr = expf(m - m_new);
        float p[2][4], sum = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                p[h][x] = ok[h][x] ? expf(s[h][x] - m_new) : 0.f;
                sum += p[h][x];
            }
        sum += __shfl_xor(sum, 16, ZI_WAVE);
        sum += __shfl_xor(sum, 32, ZI_WAVE);
        l = l * corr + sum;
        m = m_new;
        la_pack pb;
        pb.w[0] = zi_pack_bf16x2(p[0][0], p[0][1]);
        pb.w[1] = zi_pack_bf16x2(p[0][2], p[0][3]);
        pb.w[2] = zi_pack_bf16x2(p[1][0], p[1][1]);
        pb.w[3] = zi_pack_bf16x2(p[1][2], p[1][3]);
#pragma unroll
        for (int tq = 0; tq < OT; ++tq) {
            const int t = SPLIT ? tq * WAVES + wave : tq;
            if (t * 16 < rank) {
                o[tq] *= corr;
                la_pack a;
                a.h[0] = *reinterpret_cast<const la_u32x2_t*>(&ct[(t * 16 + r) * CP + 4 * j]);
                a.h[1] = *reinterpret_cast<const la_u32x2_t*>(&ct[(t * 16 + r) * CP + 16 + 4 * j]);
                o[tq] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, pb.b, o[tq], 0, 0, 0);
            }
        }
    }
    // lane (r, j) holds, of row r, the dims 16 t + 4 j + x
    if (!row_ok) return;
    if (gridDim.y == 1) {
        const float inv = 1.f / l;
        float* orow = out + grow * rank;
#pragma unroll
        for (int tq = 0; tq < OT; ++tq)
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int d = 16 * (SPLIT ? tq * WAVES + wave : tq) + 4 * j + x;
                if (d < rank) orow[d] = o[tq][x] * inv;
            }
    } else {
        float* prow = partial + ((int64_t)blockIdx.y * total_rows + grow) * (rank + 2);
        if (j == 0 && (!SPLIT || wave == 0)) {
            prow[0] = m;
            prow[1] = l;
        }
#pragma unroll
        for (int tq = 0; tq < OT; ++tq)
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int d = 16 * (SPLIT ? tq * WAVES + wave : tq) + 4 * j + x;
                if (d < rank) prow[2 + d] = o[tq][x];
            }
    }
}

// out[row] = sum_c O_c exp(m_c - M) / sum_c l_c exp(m_c - M), chunks in rising order.
__global__ void __launch_bounds__(256)
latent_attention_merge_kernel(float* __restrict__ out, const float* __restrict__ partial, int chunks, int total_rows,
                              int rank) {
    const int64_t row = blockIdx.x;
    float M = LA_EMPTY;
    for (int c = 0; c < chunks; ++c) M = fmaxf(M, partial[((int64_t)c * total_rows + row) * (rank + 2)]);
    float L = 0.f;
    for (int c = 0; c < chunks; ++c) {
        const float* p = partial + ((int64_t)c * total_rows + row) * (rank + 2);
        L += p[1] * expf(p[0] - M);
    }
    const float inv = 1.f / L;
    for (int d = threadIdx.x; d < rank; d += blockDim.x) {
        float acc = 0.f;
        for (int c = 0; c < chunks; ++c) {
            const float* p = partial + ((int64_t)c * total_rows + row) * (rank + 2);
            acc += p[2 + d] * expf(p[0] - M);
        }
        out[row * rank + d] = acc * inv;
    }
}

extern "C" int zi_latent_attention_cores_supported(int dt, int rank, int rot) {
    return dt == ZI_BF16 && rank > 0 && rank % 8 == 0 && rot >= 0 && rot % 8 == 0 && rank <= 512 && rank + rot <= 576;
}

// Rows of a tile for `waves` wavefronts, and the most tiles a step of n tokens in `entries` entries has.
extern "C" int zi_latent_attention_cores_tiles(int n, int entries, int heads, int waves) {
    const int rows = 16 * waves;
    return (int)(((int64_t)n * heads + rows - 1) / rows) + entries;
}

extern "C" int zi_latent_attention_cores(float* out, float* partial, int64_t partial_floats, const float* qa,
                                         const void* c_cache, const void* kr_cache, const int32_t* entry_start,
                                         const int32_t* entry_len, const int32_t* entry_past, const int32_t* block_tables,
                                         int entries, int n, int max_pages, int num_pages, int heads, int rank, int rot,
                                         int page_size, int window, float scale, int waves, int chunk_keys, int chunks,
                                         hipStream_t stream) {
    ZI_REQUIRE(zi_latent_attention_cores_supported(ZI_BF16, rank, rot), "latent_attention_cores: rank %d, rot %d not taken",
               rank, rot);
    ZI_REQUIRE(n >= 0 && entries > 0 && heads > 0 && page_size > 0 && max_pages > 0 && num_pages > 0 && window >= 0,
               "latent_attention_cores: bad sizes");
    ZI_REQUIRE(waves == 1 || waves == 4, "latent_attention_cores: 1 or 4 wavefronts a workgroup");
    ZI_REQUIRE(chunks >= 1 && chunks <= 65535 && (chunks == 1) == (chunk_keys == 0) && chunk_keys >= 0,
               "latent_attention_cores: bad cut (%d chunks of %d keys)", chunks, chunk_keys);
    if (chunks > 1) {
        // every key a tile's rows see lies in one of the chunks
        const int tokens_in_tile = (16 * waves + heads - 1) / heads + 1;
        // (without a window the caller sees to it that the chunks reach the last key of every entry)
        ZI_REQUIRE(window == 0 || (int64_t)chunks * chunk_keys >= (int64_t)window + tokens_in_tile,
                   "latent_attention_cores: %d chunks of %d keys do not cover a window of %d", chunks, chunk_keys, window);
        ZI_REQUIRE(partial && partial_floats >= (int64_t)chunks * n * heads * (rank + 2),
                   "latent_attention_cores: the workspace is too small");
    }
    if (n == 0) return 0;
    const int total_rows = n * heads;
    const dim3 grid(zi_latent_attention_cores_tiles(n, entries, heads, waves), chunks);
#define ZI_LA_LAUNCH(W, NT, KS)                                                                                       \
    latent_attention_cores_kernel<4, NT, KS, W == 1><<<grid, 4 * ZI_WAVE, 0, stream>>>(                                \
        out, partial, qa, (const zi_bf16*)c_cache, (const zi_bf16*)kr_cache, entry_start, entry_len, entry_past,       \
        block_tables, entries, max_pages, num_pages, heads, rank, rot, page_size, window, scale, chunk_keys, total_rows)
#define ZI_LA_SIZES(W)                                                       \
    do {                                                                     \
        if (rank <= 128 && rank + rot <= 192) ZI_LA_LAUNCH(W, 8, 6);         \
        else if (rank <= 256 && rank + rot <= 320) ZI_LA_LAUNCH(W, 16, 10);  \
        else ZI_LA_LAUNCH(W, 32, 18);                                        \
    } while (0)
    if (waves == 1) ZI_LA_SIZES(1);
    else ZI_LA_SIZES(4);
#undef ZI_LA_SIZES
#undef ZI_LA_LAUNCH
    int rc = zi_check_launch("latent_attention_cores");
    if (rc != 0 || chunks == 1) return rc;
    latent_attention_merge_kernel<<<total_rows, 256, 0, stream>>>(out, partial, chunks, total_rows, rank);
    return zi_check_launch("latent_attention_merge");
}

// ---- a product per head on the matrix cores ---------------------------------------------------------------------
// out[t][h][i] = sum_k w[h][i][k] x[t][h][k]: w bfloat16 [heads][N][K] (k runs fastest), x float32 with row stride
// ldx and head stride xs (rounded to bfloat16 as it is loaded), out float32 or bfloat16 with row stride ldo and head
// stride os.  One wavefront per (16 tokens, head, 16 outputs); operands straight from memory.  It carries the
// queries through W_uk (w = W_uk of the head, transposed at load) and the attended latents through W_uv.
template <typename TO>
__global__ void __launch_bounds__(ZI_WAVE)
headwise_linear_cores_kernel(TO* __restrict__ out, int64_t ldo, int os, const float* __restrict__ x, int64_t ldx, int xs,
                             const zi_bf16* __restrict__ w, int n, int N, int K) {
    const int t0 = blockIdx.x * 16, h = blockIdx.y, n0 = blockIdx.z * 16;
    const int lane = threadIdx.x, r = lane % 16, j = lane / 16;
    const zi_bf16* wrow = w + ((int64_t)h * N + (n0 + r < N ? n0 + r : N - 1)) * K;
    const float* xrow = x + (int64_t)(t0 + r < n ? t0 + r : n - 1) * ldx + (int64_t)h * xs;
    la_f32x4_t acc = (la_f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int k0 = 0; k0 < K; k0 += 32) {
        const int k = k0 + 8 * j;
        const bool in = k < K;      // K is a multiple of 8
        const int kc = in ? k : 0;
        const unsigned mask = 0u - (unsigned)in;
        la_pack a, b;
        a.u = *reinterpret_cast<const la_u32x4_t*>(wrow + kc) & mask;
        const float4 lo = *reinterpret_cast<const float4*>(xrow + kc), hi = *reinterpret_cast<const float4*>(xrow + kc + 4);
        b.w[0] = zi_pack_bf16x2(lo.x, lo.y) & mask;
        b.w[1] = zi_pack_bf16x2(lo.z, lo.w) & mask;
        b.w[2] = zi_pack_bf16x2(hi.x, hi.y) & mask;
        b.w[3] = zi_pack_bf16x2(hi.z, hi.w) & mask;
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, b.b, acc, 0, 0, 0);
    }
    if (t0 + r >= n) return;
    TO* orow = out + (int64_t)(t0 + r) * ldo + (int64_t)h * os + n0 + 4 * j;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        if (n0 + 4 * j + i < N) zi_store(orow + i, acc[i]);
}

extern "C" int zi_headwise_linear_supported(int w_dt, int K, int64_t ldx, int xs) {
    return w_dt == ZI_BF16 && K > 0 && K % 8 == 0 && ldx % 4 == 0 && xs % 4 == 0;
}

extern "C" int zi_headwise_linear(void* out, int out_dt, int64_t ldo, int os, const float* x, int64_t ldx, int xs,
                                  const void* w, int n, int heads, int N, int K, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && heads > 0 && heads <= 65535 && N > 0 && (N + 15) / 16 <= 65535, "headwise_linear: bad sizes");
    ZI_REQUIRE(zi_headwise_linear_supported(ZI_BF16, K, ldx, xs) && ((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0,
               "headwise_linear: K %d, row stride %lld, head stride %d or an address is not aligned", K, (long long)ldx, xs);
    ZI_REQUIRE(xs >= K && os >= N && ldx >= (int64_t)(heads - 1) * xs + K && ldo >= (int64_t)(heads - 1) * os + N,
               "headwise_linear: strides too small");
    if (n == 0) return 0;
    const dim3 grid((n + 15) / 16, heads, (N + 15) / 16);
    ZI_DISPATCH_DTYPE(out_dt, TO, {
        headwise_linear_cores_kernel<TO><<<grid, ZI_WAVE, 0, stream>>>((TO*)out, ldo, os, x, ldx, xs, (const zi_bf16*)w, n, N, K);
    });
    return zi_check_launch("headwise_linear");
}

// qa[t][h][rank + ...] = the rotated part of every head's query, turned in neighbouring pairs.
template <typename T>
__global__ void latent_query_rot_kernel(float* __restrict__ qa, const T* __restrict__ q, int64_t ldq,
                                        const float* __restrict__ table, int n, int heads, int dim, int rank, int rot) {
    const int half = rot / 2;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)n * heads * half) return;
    const int p = (int)(i % half), h = (int)((i / half) % heads);
    const int64_t t = i / ((int64_t)half * heads);
    const T* qr = q + t * ldq + (int64_t)h * (dim + rot) + dim + 2 * p;
    const float u = zi_load(qr), v = zi_load(qr + 1);
    const float c = table[(t * half + p) * 2], s = table[(t * half + p) * 2 + 1];
    float* o = qa + (t * heads + h) * (rank + rot) + rank + 2 * p;
    o[0] = u * c - v * s;
    o[1] = v * c + u * s;
}

extern "C" int zi_latent_query_rot(float* qa, const void* q, int dt, int64_t ldq, const float* table, int n, int heads,
                                   int dim, int rank, int rot, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && heads > 0 && dim > 0 && rank > 0 && rot >= 0 && rot % 2 == 0 && ldq >= (int64_t)heads * (dim + rot),
               "latent_query_rot: bad sizes");
    const int64_t total = (int64_t)n * heads * (rot / 2);
    if (total == 0) return 0;
    ZI_REQUIRE(table, "latent_query_rot: no table of angles");
    ZI_DISPATCH_DTYPE(dt, T, {
        latent_query_rot_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>(qa, (const T*)q, ldq, table, n, heads,
                                                                                         dim, rank, rot);
    });
    return zi_check_launch("latent_query_rot");
}
