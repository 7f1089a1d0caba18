// Grouped-query softmax attention under a sliding window, with the positions before the window seen as one mean
// key and one mean value for every whole block of `pool` positions.
//
// Position i sees position j when 0 <= i - j < window, and block b (positions bP .. bP + P - 1) when
// bP + P - 1 <= i - window; positions that have left the window and whose block is not yet whole behind it are not
// seen.  Tokens and blocks share one softmax.  Keys have `dim` values a head, values `vdim`.
//
// Two caches, each found through a block table of its own:
//   tokens: keys [page][slot][kv_head][dim], values [page][slot][kv_head][vdim], in the activation type; pages of
//           positions that the window has passed may be gone (-1 in the table) and are never read;
//   blocks: mean keys [page][slot][kv_head][dim] and mean values [page][slot][kv_head][vdim], float32; block b lies
//           at index b of its sequence (page b / page_size of the blocks' table).
// A block's means are made from the token cache (what it holds: normed, turned, rounded to its type) when the
// block's last token has been stored, in the order of the positions, so they do not depend on how a prompt was cut.
//
// Kernels: `zi_norm_rope_store` (per head: optional RMS norm of q and k with a gain, split-half rotation of their
// first R dims by a table of (cos, sin), optional rotation of the whole value by a second table; queries out, keys
// and values into the token cache), `zi_pool_blocks`, `zi_pooled_attention` (a workgroup of four wavefronts per
// (token, head): a lane scores one key, wavefronts take runs of 64 keys in turn and are merged at the end; the
// head's result is turned back by the query's own position when values are rotated).  All arithmetic is float32.
#include "zi_common.h"
#include "zi_api.h"

#define PA_MAX_D 512
#define PA_ACC (PA_MAX_D / ZI_WAVE)
#define PA_WAVES 4
#define PB_ACC (2 * PA_MAX_D / ZI_WAVE)      // values of a key and a value a lane of the blocks' kernel sums

// ---- norm, rotation, store ---------------------------------------------------------------------------------
// One wavefront per (token, unit): units 0 .. nh-1 are the query heads, nh .. nh+nkv-1 the key/value heads.
template <typename T>
__global__ void __launch_bounds__(ZI_WAVE)
norm_rope_store_kernel(T* __restrict__ q_out, int64_t ldq, T* __restrict__ kcache, T* __restrict__ vcache,
                       const float* __restrict__ proj, int64_t ld, int splits, int64_t split_stride,
                       const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
                       const float* __restrict__ table, int rot, const float* __restrict__ vtable,
                       const int32_t* __restrict__ slots, int64_t cache_slots, int nh, int nkv, int dim, int vdim) {
    __shared__ float xs[PA_MAX_D];
    const int t = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const bool is_q = unit < nh;
    const int g = is_q ? unit : unit - nh;
    const int64_t slot = slots ? slots[t] : -1;
    const bool stores = slot >= 0 && slot < cache_slots && kcache;
    if (!is_q && !stores) return;
    // q or k: sum the partial sums, norm, turn
    const int64_t at = is_q ? (int64_t)unit * dim : (int64_t)nh * dim + (int64_t)g * dim;
    const float* row = proj + (int64_t)t * ld + at;
    float ss = 0.f;
    for (int i = lane; i < dim; i += ZI_WAVE) {
        float v = row[i];
        for (int s = 1; s < splits; ++s) v += row[s * split_stride + i];
        xs[i] = v;
        ss += v * v;
    }
    const float* gain = is_q ? q_gain : k_gain;
    if (gain) {
        ss = zi_wave_sum(ss);
        const float r = 1.f / sqrtf(ss / (float)dim + eps);
        for (int i = lane; i < dim; i += ZI_WAVE) xs[i] = xs[i] * r * gain[i];
    }
    __syncthreads();
    T* dst = is_q ? q_out + (int64_t)t * ldq + (int64_t)unit * dim : kcache + (slot * nkv + g) * dim;
    const int half = rot / 2;
    for (int i = lane; i < dim; i += ZI_WAVE) {
        float v = xs[i];
        if (i < rot) {
            const int pr = i < half ? i : i - half;
            const float c = table[((int64_t)t * half + pr) * 2], s = table[((int64_t)t * half + pr) * 2 + 1];
            v = i < half ? xs[i] * c - xs[i + half] * s : xs[i] * c + xs[i - half] * s;
        }
        zi_store(dst + i, v);
    }
    if (is_q) return;
    // the value of this key/value head
    __syncthreads();
    const float* vrow = proj + (int64_t)t * ld + (int64_t)(nh + nkv) * dim + (int64_t)g * vdim;
    for (int i = lane; i < vdim; i += ZI_WAVE) {
        float v = vrow[i];
        for (int s = 1; s < splits; ++s) v += vrow[s * split_stride + i];
        xs[i] = v;
    }
    __syncthreads();
    T* vdst = vcache + (slot * nkv + g) * vdim;
    const int vh = vdim / 2;
    for (int i = lane; i < vdim; i += ZI_WAVE) {
        float v = xs[i];
        if (vtable) {
            const int pr = i < vh ? i : i - vh;
            const float c = vtable[((int64_t)t * vh + pr) * 2], s = vtable[((int64_t)t * vh + pr) * 2 + 1];
            v = i < vh ? xs[i] * c - xs[i + vh] * s : xs[i] * c + xs[i - vh] * s;
        }
        zi_store(vdst + i, v);
    }
}

// proj [n][nh*dim + nkv*dim + nkv*vdim] float32 (row stride ld; `splits` partial sums `split_stride` apart);
// q_gain, k_gain [dim] float32 or null (no norm); table [n][rot/2][2] (cos, sin) or null when rot == 0; vtable
// [n][vdim/2][2] or null (values are stored as they are); slots [n] or null (nothing is stored); the caches hold
// cache_slots = pages * page_size rows.
extern "C" int zi_norm_rope_store(void* q_out, int dt, int64_t ldq, void* kcache, void* vcache, const float* proj,
                                  int64_t ld, int splits, int64_t split_stride, const float* q_gain, const float* k_gain,
                                  float eps, const float* table, int rot, const float* vtable, const int32_t* slots,
                                  int64_t cache_slots, int n, int nh, int nkv, int dim, int vdim, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && nh > 0 && nkv > 0 && nh + nkv <= 65535 && dim > 0 && vdim > 0 && dim <= PA_MAX_D && vdim <= PA_MAX_D,
               "norm_rope_store: bad sizes (heads %d/%d, dim %d, vdim %d)", nh, nkv, dim, vdim);
    ZI_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dim && (rot == 0 || table), "norm_rope_store: %d rotated dims of %d", rot, dim);
    ZI_REQUIRE(!vtable || vdim % 2 == 0, "norm_rope_store: values of an odd size cannot be rotated");
    ZI_REQUIRE(ld >= (int64_t)(nh + nkv) * dim + (int64_t)nkv * vdim && ldq >= (int64_t)nh * dim && splits >= 1 && eps > 0.f,
               "norm_rope_store: a row is too short");
    ZI_REQUIRE(!kcache || (vcache && slots && cache_slots > 0), "norm_rope_store: a cache without slots");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(dt, T, {
        norm_rope_store_kernel<T><<<dim3(n, nh + nkv), ZI_WAVE, 0, stream>>>(
            (T*)q_out, ldq, (T*)kcache, (T*)vcache, proj, ld, splits, split_stride, q_gain, k_gain, eps, table, rot, vtable,
            slots, cache_slots, nh, nkv, dim, vdim);
    });
    return zi_check_launch("norm_rope_store");
}

// ---- the blocks' means -------------------------------------------------------------------------------------
// One workgroup of four wavefronts per (token, key/value head); a token whose position does not end a block has pool
// slot -1 and its workgroup leaves at once.  The block's rows in the cache are looked up 64 positions at a time (a
// thread each); the wavefronts take the positions in turn (wavefront w: w, w + 4, ...), a lane the dims lane, lane +
// 64, ..., with the loads of eight positions in flight and no load under a branch; the four partial sums are added in
// the wavefronts' order.  The order of the additions depends on the block's length alone.
template <typename T>
__global__ void __launch_bounds__(PA_WAVES* ZI_WAVE)
pool_blocks_kernel(float* __restrict__ kpool, float* __restrict__ vpool, const T* __restrict__ kcache,
                   const T* __restrict__ vcache, const int32_t* __restrict__ pool_slots, int64_t pool_rows,
                   const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                   const int32_t* __restrict__ block_tables, int max_pages, int num_pages, int page_size, int nkv,
                   int dim, int vdim, int pool) {
    __shared__ int64_t rows[ZI_WAVE];
    __shared__ float parts[PA_WAVES][2 * PA_MAX_D];
    const int t = blockIdx.x, g = blockIdx.y, tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int64_t ps = pool_slots[t];
    if (ps < 0 || ps >= pool_rows) return;
    const int p = tok_pos[t];
    if (p + 1 < pool) return;
    const int32_t* bt = block_tables + (int64_t)tok_seq[t] * max_pages;
    const float inv = 1.f / (float)pool;
    if constexpr (sizeof(T) == 2) {
        // bfloat16 rows whose widths are multiples of 8: a thread loads 16 bytes (8 dims) of a position at a time, so a
        // block of 64 positions is two loads a thread, all in flight together; the positions are dealt out over the
        // threads that share a piece of 8 dims (thread: piece tid % pieces, positions tid / pieces, + groups, ...), the
        // groups' partial sums are added in the groups' order
        const int pieces = (dim + vdim) / 8;
        if (dim % 8 == 0 && vdim % 8 == 0 && pieces <= PA_WAVES * ZI_WAVE && ((uintptr_t)kcache % 16) == 0 &&
            ((uintptr_t)vcache % 16) == 0) {
            const int groups = PA_WAVES * ZI_WAVE / pieces;      // at most 2 * PA_MAX_D / 8 = 128 pieces: at least 2 groups
            const int piece = tid % pieces, grp = tid / pieces;
            const bool works = grp < groups;
            const bool key = piece * 8 < dim;
            const T* base = key ? kcache + piece * 8 : vcache + (piece * 8 - dim);
            const int64_t stride = key ? dim : vdim;
            float a8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            bool hole = false;
            for (int j0 = p - pool + 1; j0 <= p; j0 += ZI_WAVE) {
                const int cnt = p - j0 + 1 < ZI_WAVE ? p - j0 + 1 : ZI_WAVE;
                __syncthreads();
                if (tid < cnt) {
                    const int j = j0 + tid, pi = j / page_size;
                    const int page = pi < max_pages ? bt[pi] : -1;
                    rows[tid] = (unsigned)page < (unsigned)num_pages ? ((int64_t)page * page_size + j % page_size) * nkv + g : -1;
                }
                __syncthreads();
                if (works) {
                    for (int jj = grp; jj < cnt; jj += 4 * groups) {
                        uint4 x[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int at = jj + u * groups;
                            const int64_t r = rows[at < cnt ? at : jj];
                            hole |= r < 0;
                            x[u] = *reinterpret_cast<const uint4*>(base + (r < 0 ? 0 : r) * stride);
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            if (jj + u * groups >= cnt) continue;
                            a8[0] += __uint_as_float(x[u].x << 16); a8[1] += __uint_as_float(x[u].x & 0xffff0000u);
                            a8[2] += __uint_as_float(x[u].y << 16); a8[3] += __uint_as_float(x[u].y & 0xffff0000u);
                            a8[4] += __uint_as_float(x[u].z << 16); a8[5] += __uint_as_float(x[u].z & 0xffff0000u);
                            a8[6] += __uint_as_float(x[u].w << 16); a8[7] += __uint_as_float(x[u].w & 0xffff0000u);
                        }
                    }
                }
            }
            // parts as [group][dim]: groups * (dim + vdim) <= 256 * 8 floats
            float* flat = &parts[0][0];
            if (works) {
#pragma unroll
                for (int i = 0; i < 8; ++i) flat[(int64_t)grp * pieces * 8 + piece * 8 + i] = hole ? NAN : a8[i];
            }
            __syncthreads();
            for (int i = tid; i < pieces * 8; i += PA_WAVES * ZI_WAVE) {
                float total = flat[i];
                for (int w = 1; w < groups; ++w) total += flat[(int64_t)w * pieces * 8 + i];
                if (i < dim) kpool[(ps * nkv + g) * dim + i] = total * inv;
                else vpool[(ps * nkv + g) * vdim + (i - dim)] = total * inv;
            }
            return;
        }
    }
    float acc[PB_ACC];
#pragma unroll
    for (int a = 0; a < PB_ACC; ++a) acc[a] = 0.f;
    const int width = dim + vdim;
    bool hole = false;      // a position without a page is never scheduled: it shows as NaN
    for (int j0 = p - pool + 1; j0 <= p; j0 += ZI_WAVE) {
        const int cnt = p - j0 + 1 < ZI_WAVE ? p - j0 + 1 : ZI_WAVE;
        __syncthreads();
        if (tid < cnt) {
            const int j = j0 + tid, pi = j / page_size;
            const int page = pi < max_pages ? bt[pi] : -1;
            rows[tid] = (unsigned)page < (unsigned)num_pages ? ((int64_t)page * page_size + j % page_size) * nkv + g : -1;
        }
        __syncthreads();
#pragma unroll
        for (int a = 0; a < PB_ACC; ++a) {
            const int i = lane + a * ZI_WAVE;
            if (i < width) {
                const bool key = i < dim;
                const T* base = key ? kcache + i : vcache + (i - dim);
                const int64_t stride = key ? dim : vdim;
                int jj = wave;
                for (; jj + 7 * PA_WAVES < cnt; jj += 8 * PA_WAVES) {
                    float x[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) {
                        const int64_t r = rows[jj + u * PA_WAVES];
                        hole |= r < 0;
                        x[u] = zi_load(base + (r < 0 ? 0 : r) * stride);
                    }
#pragma unroll
                    for (int u = 0; u < 8; ++u) acc[a] += x[u];
                }
                for (; jj < cnt; jj += PA_WAVES) {
                    const int64_t r = rows[jj];
                    hole |= r < 0;
                    acc[a] += zi_load(base + (r < 0 ? 0 : r) * stride);
                }
            }
        }
    }
#pragma unroll
    for (int a = 0; a < PB_ACC; ++a) {
        const int i = lane + a * ZI_WAVE;
        if (i < width) parts[wave][i] = hole ? NAN : acc[a];
    }
    __syncthreads();
    for (int i = tid; i < width; i += PA_WAVES * ZI_WAVE) {
        float total = parts[0][i];
#pragma unroll
        for (int w = 1; w < PA_WAVES; ++w) total += parts[w][i];
        if (i < dim) kpool[(ps * nkv + g) * dim + i] = total * inv;
        else vpool[(ps * nkv + g) * vdim + (i - dim)] = total * inv;
    }
}

extern "C" int zi_pool_blocks(float* kpool, float* vpool, int64_t pool_rows, const void* kcache, const void* vcache,
                              int dt, const int32_t* pool_slots, const int32_t* tok_seq, const int32_t* tok_pos,
                              const int32_t* block_tables, int max_pages, int num_pages, int page_size, int n, int nkv,
                              int dim, int vdim, int pool, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && nkv > 0 && nkv <= 65535 && dim > 0 && vdim > 0 && pool > 0 && page_size > 0 && max_pages > 0 &&
                   num_pages > 0 && pool_rows > 0, "pool_blocks: bad sizes");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(dt, T, {
        pool_blocks_kernel<T><<<dim3(n, nkv), PA_WAVES * ZI_WAVE, 0, stream>>>(kpool, vpool, (const T*)kcache, (const T*)vcache,
                                                                    pool_slots, pool_rows, tok_seq, tok_pos, block_tables,
                                                                    max_pages, num_pages, page_size, nkv, dim, vdim, pool);
    });
    return zi_check_launch("pool_blocks");
}

// ---- attention ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float pa_dot(const float* __restrict__ row, const float* __restrict__ qs, int d) {
    float dot = 0.f;
    if ((d & 3) == 0 && ((uintptr_t)row & 15) == 0) {
        for (int x = 0; x < d; x += 4) {
            const float4 k4 = *reinterpret_cast<const float4*>(row + x);
            dot += qs[x] * k4.x + qs[x + 1] * k4.y + qs[x + 2] * k4.z + qs[x + 3] * k4.w;
        }
    } else {
        for (int x = 0; x < d; ++x) dot += qs[x] * row[x];
    }
    return dot;
}
__device__ __forceinline__ float pa_dot(const zi_bf16* __restrict__ row, const float* __restrict__ qs, int d) {
    float dot = 0.f;
    if ((d & 7) == 0 && ((uintptr_t)row & 15) == 0) {
        for (int x = 0; x < d; x += 8) {
            const uint4 k8 = *reinterpret_cast<const uint4*>(row + x);
            dot += qs[x] * __uint_as_float(k8.x << 16) + qs[x + 1] * __uint_as_float(k8.x & 0xffff0000u) +
                   qs[x + 2] * __uint_as_float(k8.y << 16) + qs[x + 3] * __uint_as_float(k8.y & 0xffff0000u) +
                   qs[x + 4] * __uint_as_float(k8.z << 16) + qs[x + 5] * __uint_as_float(k8.z & 0xffff0000u) +
                   qs[x + 6] * __uint_as_float(k8.w << 16) + qs[x + 7] * __uint_as_float(k8.w & 0xffff0000u);
        }
    } else {
        for (int x = 0; x < d; ++x) dot += qs[x] * zi_load(row + x);
    }
    return dot;
}

template <typename T>
__global__ void __launch_bounds__(PA_WAVES* ZI_WAVE)
pooled_attention_kernel(T* __restrict__ out, int64_t ldo, const T* __restrict__ q, int64_t ldq,
                        const T* __restrict__ kcache, const T* __restrict__ vcache, const float* __restrict__ kpool,
                        const float* __restrict__ vpool, const int32_t* __restrict__ tok_seq,
                        const int32_t* __restrict__ tok_pos, const int32_t* __restrict__ block_tables, int max_pages,
                        int num_pages, int page_size, const int32_t* __restrict__ pool_tables, int pool_max_pages,
                        int pool_num_pages, int pool_page_size, int nh, int nkv, int dim, int vdim, int window, int pool,
                        float scale, const float* __restrict__ vtable, const int32_t* __restrict__ entry_len, int long_len) {
    // (the tokens of entries of long_len tokens and more are another kernel's)
    if (entry_len && entry_len[tok_seq[blockIdx.x]] >= long_len) return;
    __shared__ float qs[PA_MAX_D];
    __shared__ float ps[PA_WAVES][ZI_WAVE];
    __shared__ int64_t vat[PA_WAVES][ZI_WAVE];
    __shared__ float merged[PA_WAVES][PA_MAX_D + 2];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & (ZI_WAVE - 1), wave = tid / ZI_WAVE;
    const int g = h / (nh / nkv);
    const int p = tok_pos[t];
    const int32_t* bt = block_tables + (int64_t)tok_seq[t] * max_pages;
    const int32_t* pt = pool_tables ? pool_tables + (int64_t)tok_seq[t] * pool_max_pages : nullptr;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    // blocks wholly before the window: b P + P - 1 <= p - window
    const int blocks = (pt && pool > 0 && window > 0 && p - window + 1 >= pool) ? (p - window + 1) / pool : 0;
    const int count = blocks + (p - lo + 1);

    const T* qr = q + (int64_t)t * ldq + (int64_t)h * dim;
    for (int j = tid; j < dim; j += PA_WAVES * ZI_WAVE) qs[j] = zi_load(qr + j);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[PA_ACC];
#pragma unroll
    for (int i = 0; i < PA_ACC; ++i) acc[i] = 0.f;

    for (int base = wave * ZI_WAVE; base < count; base += PA_WAVES * ZI_WAVE) {
        const int at = base + lane;
        bool valid = at < count;
        float s = -INFINITY;
        int64_t vrow = -1;      // >= 0: a token's value row; <= -2: block row -(vrow + 2)
        if (valid) {
            if (at < blocks) {
                const int pi = at / pool_page_size;
                const int page = pi < pool_max_pages ? pt[pi] : -1;
                if ((unsigned)page >= (unsigned)pool_num_pages) {
                    valid = false;
                } else {
                    const int64_t r = ((int64_t)page * pool_page_size + at % pool_page_size) * nkv + g;
                    s = pa_dot(kpool + r * dim, qs, dim) * scale;
                    vrow = -(r + 2);
                }
            } else {
                const int j = lo + (at - blocks);
                const int pi = j / page_size;
                const int page = pi < max_pages ? bt[pi] : -1;
                if ((unsigned)page >= (unsigned)num_pages) {
                    valid = false;      // a hole in the table: the host never schedules this; stay in bounds
                } else {
                    const int64_t r = ((int64_t)page * page_size + j % page_size) * nkv + g;
                    s = pa_dot(kcache + r * dim, qs, dim) * scale;
                    vrow = r;
                }
            }
        }
        const float mt = zi_wave_max(s);
        const float m_new = fmaxf(m, mt);
        const float pj = (valid && m_new > -INFINITY) ? expf(s - m_new) : 0.f;
        const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
        l = l * corr + zi_wave_sum(pj);
        ps[wave][lane] = pj;
        vat[wave][lane] = valid ? vrow : -1;
        __builtin_amdgcn_wave_barrier();
        const int cnt = (count - base < ZI_WAVE) ? count - base : ZI_WAVE;
#pragma unroll
        for (int i = 0; i < PA_ACC; ++i) acc[i] *= corr;
        for (int jj = 0; jj < cnt; ++jj) {
            const float pw = ps[wave][jj];
            const int64_t vr = vat[wave][jj];
            if (vr == -1) continue;
            if (vr >= 0) {
                const T* vv = vcache + vr * vdim;
#pragma unroll
                for (int i = 0; i < PA_ACC; ++i) {
                    const int x = lane + i * ZI_WAVE;
                    if (x < vdim) acc[i] += pw * zi_load(vv + x);
                }
            } else {
                const float* vv = vpool + (-(vr + 2)) * vdim;
#pragma unroll
                for (int i = 0; i < PA_ACC; ++i) {
                    const int x = lane + i * ZI_WAVE;
                    if (x < vdim) acc[i] += pw * vv[x];
                }
            }
        }
        m = m_new;
        __builtin_amdgcn_wave_barrier();
    }
    // the wavefronts' parts, merged in their order
#pragma unroll
    for (int i = 0; i < PA_ACC; ++i) {
        const int x = lane + i * ZI_WAVE;
        if (x < vdim) merged[wave][x] = acc[i];
    }
    if (lane == 0) {
        merged[wave][PA_MAX_D] = m;
        merged[wave][PA_MAX_D + 1] = l;
    }
    __syncthreads();
    float mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < PA_WAVES; ++w) mm = fmaxf(mm, merged[w][PA_MAX_D]);
    float ll = 0.f, f[PA_WAVES];
#pragma unroll
    for (int w = 0; w < PA_WAVES; ++w) {
        const float mw = merged[w][PA_MAX_D];
        f[w] = mw == -INFINITY ? 0.f : expf(mw - mm);
        ll += merged[w][PA_MAX_D + 1] * f[w];
    }
    const float inv = 1.f / ll;
    __syncthreads();
    for (int x = tid; x < vdim; x += PA_WAVES * ZI_WAVE) {
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < PA_WAVES; ++w) o += merged[w][x] * f[w];
        qs[x] = o * inv;      // the query is no longer needed
    }
    __syncthreads();
    T* orow = out + (int64_t)t * ldo + (int64_t)h * vdim;
    const int vh = vdim / 2;
    for (int x = tid; x < vdim; x += PA_WAVES * ZI_WAVE) {
        float o = qs[x];
        if (vtable) {       // turn back by the query's position: the angle's sign changes
            const int pr = x < vh ? x : x - vh;
            const float c = vtable[((int64_t)t * vh + pr) * 2], s = vtable[((int64_t)t * vh + pr) * 2 + 1];
            o = x < vh ? qs[x] * c + qs[x + vh] * s : qs[x] * c - qs[x - vh] * s;
        }
        zi_store(orow + x, o);
    }
}

// out [n][nh*vdim], q [n][nh*dim] in the caches' type `dt`.  Token cache: kcache, vcache with `num_pages` pages of
// `page_size` rows, found through block_tables [entries][max_pages]; block cache: kpool, vpool (float32) with
// pool_num_pages pages of pool_page_size rows through pool_tables [entries][pool_max_pages] (null, or pool == 0: no
// blocks, a plain window; window == 0: all positions, no blocks).  vtable [n][vdim/2][2] or null: the (cos, sin) of
// every token's position over the value's pairs, by which a head's result is turned back.  entry_len (or null) and
// long_len: the tokens of entries that bring long_len tokens or more are left out (the matrix-core kernel takes them).
extern "C" int zi_pooled_attention(void* out, int64_t ldo, const void* q, int64_t ldq, int dt, const void* kcache,
                                   const void* vcache, const float* kpool, const float* vpool, const int32_t* tok_seq,
                                   const int32_t* tok_pos, const int32_t* block_tables, int max_pages, int num_pages,
                                   int page_size, const int32_t* pool_tables, int pool_max_pages, int pool_num_pages,
                                   int pool_page_size, int n, int nh, int nkv, int dim, int vdim, int window, int pool,
                                   float scale, const float* vtable, const int32_t* entry_len, int long_len,
                                   hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0 && nh <= 65535 && dim > 0 && vdim > 0 && dim <= PA_MAX_D &&
                   vdim <= PA_MAX_D, "pooled_attention: bad sizes (heads %d/%d, dim %d, vdim %d)", nh, nkv, dim, vdim);
    ZI_REQUIRE(page_size > 0 && max_pages > 0 && num_pages > 0 && window >= 0 && pool >= 0, "pooled_attention: bad cache sizes");
    ZI_REQUIRE(!pool_tables || pool == 0 || (kpool && vpool && pool_max_pages > 0 && pool_num_pages > 0 && pool_page_size > 0),
               "pooled_attention: blocks without a cache of their means");
    ZI_REQUIRE(ldq >= (int64_t)nh * dim && ldo >= (int64_t)nh * vdim, "pooled_attention: a row is too short");
    ZI_REQUIRE(!vtable || vdim % 2 == 0, "pooled_attention: values of an odd size cannot be turned");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(dt, T, {
        pooled_attention_kernel<T><<<dim3(n, nh), PA_WAVES * ZI_WAVE, 0, stream>>>(
            (T*)out, ldo, (const T*)q, ldq, (const T*)kcache, (const T*)vcache, kpool, vpool, tok_seq, tok_pos, block_tables,
            max_pages, num_pages, page_size, pool > 0 ? pool_tables : nullptr, pool_max_pages, pool_num_pages,
            pool_page_size, nh, nkv, dim, vdim, window, pool, scale, vtable, entry_len, long_len);
    });
    return zi_check_launch("pooled_attention");
}
