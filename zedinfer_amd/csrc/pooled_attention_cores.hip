// Windowed attention over tokens and means of blocks (see pooled_attention.hip for what is computed and for the two
// caches) on the matrix cores, for portions of prompts: bfloat16, keys of 32, 64, 96 or 128 values a head, values of a
// multiple of 16 up to 128.
//
// A workgroup of four wavefronts takes up to 64 rows: the query heads of one key/value head for a run of consecutive
// tokens of one entry (row = token * heads_in_group + head), so that a staged block of keys serves every head of the
// group.  It walks the items its rows can see, first the blocks' means and then the positions from the first row's
// window on, 32 items at a time: the items' keys go into LDS as they lie ([item][dim], rows padded), their values
// transposed ([vdim][item]).  Per wavefront (16 rows): S^T = K Q^T with `v_mfma_f32_16x16x32_bf16` (a lane then holds
// the scores of ONE row for eight items), the visibility of every (row, item), a running maximum and sum in base 2,
// and O^T += V^T P^T, where P^T is the matrix operand straight from the lanes' scores: the items are contracted in the
// order in which the lanes hold them, and the transposed values are read in that order.  The blocks' float32 means are
// rounded to bfloat16 as they are staged.  At the end the rows pass LDS once more, are turned back by their
// positions when values are stored turned, and leave in bfloat16.
#include "zi_common.h"
#include "zi_api.h"

#define PC_ROWS 64
#define PC_ITEMS 32
#define PC_THREADS 256
#define PC_VT_STRIDE 36      // elements of a row of the transposed values: 8 rows apart are 16 banks apart

typedef __attribute__((ext_vector_type(8))) __bf16 pc_bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float pc_f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t pc_u32x4_t;
union pc_pack {
    pc_u32x4_t u;
    pc_bf16x8_t b;
    uint16_t h[8];
};

template <int DK32, int DV16>
__global__ void __launch_bounds__(PC_THREADS)
pooled_attention_cores_kernel(zi_bf16* __restrict__ out, int64_t ldo, const zi_bf16* __restrict__ q, int64_t ldq,
                              const zi_bf16* __restrict__ kcache, const zi_bf16* __restrict__ vcache,
                              const float* __restrict__ kpool, const float* __restrict__ vpool,
                              const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_len,
                              const int32_t* __restrict__ entry_past, const int32_t* __restrict__ block_tables,
                              int max_pages, int num_pages, int page_size, const int32_t* __restrict__ pool_tables,
                              int pool_max_pages, int pool_num_pages, int pool_page_size, int nh, int nkv, int window,
                              int pool, float scale_log2, const float* __restrict__ vtable, int long_len,
                              int chunk_blocks, float* __restrict__ partial, int total_rows) {
    constexpr int DIM = 32 * DK32, VD = 16 * DV16, KS = DIM + 8;
    __shared__ __attribute__((aligned(16))) uint16_t ks[PC_ITEMS][KS];
    __shared__ __attribute__((aligned(16))) uint16_t vt[VD][PC_VT_STRIDE];
    __shared__ __attribute__((aligned(16))) float os[PC_ROWS][VD + 1];
    const int e = blockIdx.z, g = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int len = entry_len[e];
    const int group = nh / nkv;
    const int tq_tile = PC_ROWS / group;           // tokens a tile holds
    // chunk_blocks > 0: the short entries (fewer than long_len tokens: one tile), their items cut into chunks of
    // chunk_blocks blocks over blockIdx.x, the chunks' unnormalised results left in `partial`; else the long ones,
    // a tile a workgroup
    const bool split = chunk_blocks > 0;
    if (split ? (len >= long_len || len <= 0) : len < long_len) return;
    const int tq0 = split ? 0 : blockIdx.x * tq_tile;
    if (tq0 >= len) return;
    const int tq_n = len - tq0 < tq_tile ? len - tq0 : tq_tile;
    const int past = entry_past[e], t0 = entry_start[e] + tq0;
    const int p_first = past + tq0, p_last = p_first + tq_n - 1;
    const int32_t* bt = block_tables + (int64_t)e * max_pages;
    const int32_t* pt = pool_tables ? pool_tables + (int64_t)e * pool_max_pages : nullptr;
    const bool pooled = pt && pool > 0 && window > 0;
    const int nb_max = (pooled && p_last - window + 1 >= pool) ? (p_last - window + 1) / pool : 0;
    const int lo_min = (window > 0 && p_first - window + 1 > 0) ? p_first - window + 1 : 0;
    const int n_tok = p_last - lo_min + 1;

    // this lane's row: the scores it holds are those of row r
    const int r = 16 * wave + (lane & 15), j = lane >> 4;
    const int r_tok = r / group, r_head = r % group;
    const bool r_ok = r_tok < tq_n && r < tq_tile * group;
    const int p_r = p_first + (r_ok ? r_tok : 0);
    const int lo_r = (window > 0 && p_r - window + 1 > 0) ? p_r - window + 1 : 0;
    const int nb_r = (pooled && p_r - window + 1 >= pool) ? (p_r - window + 1) / pool : 0;

    // the row's query as the second operand of K Q^T: lane (row, j) holds dims 32 s + 8 j .. + 8
    pc_pack qreg[DK32];
    {
        const zi_bf16* qr = q + (int64_t)(t0 + (r_ok ? r_tok : 0)) * ldq + (int64_t)(g * group + r_head) * DIM + 8 * j;
#pragma unroll
        for (int s = 0; s < DK32; ++s) qreg[s].u = *reinterpret_cast<const pc_u32x4_t*>(qr + 32 * s);
    }
    pc_f32x4_t acc_o[DV16];
#pragma unroll
    for (int v = 0; v < DV16; ++v) acc_o[v] = (pc_f32x4_t){0.f, 0.f, 0.f, 0.f};
    float m_run = -1e30f, l_run = 0.f;

    const int blocks_pool = (nb_max + PC_ITEMS - 1) / PC_ITEMS, blocks_tok = (n_tok + PC_ITEMS - 1) / PC_ITEMS;
    const int blk_first = split ? blockIdx.x * chunk_blocks : 0;
    const int blk_end = split && blk_first + chunk_blocks < blocks_pool + blocks_tok ? blk_first + chunk_blocks
                                                                                     : blocks_pool + blocks_tok;
    for (int blk = blk_first; blk < blk_end; ++blk) {
        const bool pool_phase = blk < blocks_pool;
        const int base = pool_phase ? blk * PC_ITEMS : (blk - blocks_pool) * PC_ITEMS;
        const int n_items = pool_phase ? nb_max : n_tok;
        __syncthreads();      // the block before has been read
        // ---- stage the items' keys as they lie and their values transposed
        constexpr int KP = DIM / 8, VP = VD / 8;
        for (int c = tid; c < PC_ITEMS * KP; c += PC_THREADS) {
            const int item = c / KP, piece = c % KP, a = base + item;
            pc_pack x;
            x.u = (pc_u32x4_t){0u, 0u, 0u, 0u};
            if (a < n_items) {
                if (pool_phase) {
                    const int pi = a / pool_page_size;
                    const int page = pi < pool_max_pages ? pt[pi] : -1;
                    if ((unsigned)page < (unsigned)pool_num_pages) {
                        const float* src = kpool + (((int64_t)page * pool_page_size + a % pool_page_size) * nkv + g) * DIM + 8 * piece;
                        const float4 lo4 = *reinterpret_cast<const float4*>(src), hi4 = *reinterpret_cast<const float4*>(src + 4);
                        x.u[0] = zi_pack_bf16x2(lo4.x, lo4.y); x.u[1] = zi_pack_bf16x2(lo4.z, lo4.w);
                        x.u[2] = zi_pack_bf16x2(hi4.x, hi4.y); x.u[3] = zi_pack_bf16x2(hi4.z, hi4.w);
                    }
                } else {
                    const int pos = lo_min + a, pi = pos / page_size;
                    const int page = pi < max_pages ? bt[pi] : -1;
                    if ((unsigned)page < (unsigned)num_pages)
                        x.u = *reinterpret_cast<const pc_u32x4_t*>(
                            kcache + (((int64_t)page * page_size + pos % page_size) * nkv + g) * DIM + 8 * piece);
                }
            }
            *reinterpret_cast<pc_u32x4_t*>(&ks[item][8 * piece]) = x.u;
        }
        for (int c = tid; c < PC_ITEMS * VP; c += PC_THREADS) {
            const int item = c % PC_ITEMS, piece = c / PC_ITEMS, a = base + item;
            pc_pack x;
            x.u = (pc_u32x4_t){0u, 0u, 0u, 0u};
            if (a < n_items) {
                if (pool_phase) {
                    const int pi = a / pool_page_size;
                    const int page = pi < pool_max_pages ? pt[pi] : -1;
                    if ((unsigned)page < (unsigned)pool_num_pages) {
                        const float* src = vpool + (((int64_t)page * pool_page_size + a % pool_page_size) * nkv + g) * VD + 8 * piece;
                        const float4 lo4 = *reinterpret_cast<const float4*>(src), hi4 = *reinterpret_cast<const float4*>(src + 4);
                        x.u[0] = zi_pack_bf16x2(lo4.x, lo4.y); x.u[1] = zi_pack_bf16x2(lo4.z, lo4.w);
                        x.u[2] = zi_pack_bf16x2(hi4.x, hi4.y); x.u[3] = zi_pack_bf16x2(hi4.z, hi4.w);
                    }
                } else {
                    const int pos = lo_min + a, pi = pos / page_size;
                    const int page = pi < max_pages ? bt[pi] : -1;
                    if ((unsigned)page < (unsigned)num_pages)
                        x.u = *reinterpret_cast<const pc_u32x4_t*>(
                            vcache + (((int64_t)page * page_size + pos % page_size) * nkv + g) * VD + 8 * piece);
                }
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) vt[8 * piece + i][item] = x.h[i];
        }
        __syncthreads();
        // ---- scores of this wavefront's 16 rows against the 32 items: lane (row, j) gets items 16 kt + 4 j + i
        pc_f32x4_t sc[2];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt) {
            sc[kt] = (pc_f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < DK32; ++s) {
                pc_pack a;
                a.u = *reinterpret_cast<const pc_u32x4_t*>(&ks[16 * kt + (lane & 15)][32 * s + 8 * j]);
                sc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, qreg[s].b, sc[kt], 0, 0, 0);
            }
        }
        float sv[8];
        bool vis[8];
        float mx = -1e30f;
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int a = base + 16 * kt + 4 * j + i;
                bool ok = r_ok && a < n_items;
                if (pool_phase) ok = ok && a < nb_r;
                else ok = ok && lo_min + a >= lo_r && lo_min + a <= p_r;
                vis[4 * kt + i] = ok;
                sv[4 * kt + i] = ok ? sc[kt][i] * scale_log2 : -1e30f;
                mx = fmaxf(mx, sv[4 * kt + i]);
            }
        mx = fmaxf(mx, __shfl_xor(mx, 16, ZI_WAVE));
        mx = fmaxf(mx, __shfl_xor(mx, 32, ZI_WAVE));
        const float m_new = fmaxf(m_run, mx);
        const float corr = exp2f(m_run - m_new);
        float psum = 0.f;
        float pv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            pv[i] = vis[i] ? exp2f(sv[i] - m_new) : 0.f;
            psum += pv[i];
        }
        l_run = l_run * corr + psum;      // this lane's share of the row's sum; the four shares are added at the end
        m_run = m_new;
        pc_pack pb;
        pb.u[0] = zi_pack_bf16x2(pv[0], pv[1]); pb.u[1] = zi_pack_bf16x2(pv[2], pv[3]);
        pb.u[2] = zi_pack_bf16x2(pv[4], pv[5]); pb.u[3] = zi_pack_bf16x2(pv[6], pv[7]);
#pragma unroll
        for (int v = 0; v < DV16; ++v) {
            // the transposed values in the lanes' order of items: 4 j .. 4 j + 3, then 16 + 4 j .. 16 + 4 j + 3
            const uint16_t* vrow = &vt[16 * v + (lane & 15)][0];
            const uint2 first = *reinterpret_cast<const uint2*>(vrow + 4 * j), second = *reinterpret_cast<const uint2*>(vrow + 16 + 4 * j);
            pc_pack a;
            a.u = (pc_u32x4_t){first.x, first.y, second.x, second.y};
#pragma unroll
            for (int i = 0; i < 4; ++i) acc_o[v][i] *= corr;
            acc_o[v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.b, pb.b, acc_o[v], 0, 0, 0);
        }
    }
    // ---- the rows: normalise, through LDS, turn back, store
    float l_row = l_run;
    l_row += __shfl_xor(l_row, 16, ZI_WAVE);
    l_row += __shfl_xor(l_row, 32, ZI_WAVE);
    if (split) {
        // this chunk's share of the row: (maximum in base-2 units, sum, unnormalised result); a chunk without
        // items leaves a share that counts nothing
        if (r_ok) {
            float* dst = partial + ((int64_t)blockIdx.x * total_rows + (int64_t)(t0 + r_tok) * nh + g * group + r_head) * (VD + 2);
            if (j == 0) {
                dst[0] = m_run;
                dst[1] = l_row;
            }
#pragma unroll
            for (int v = 0; v < DV16; ++v)
#pragma unroll
                for (int i = 0; i < 4; ++i) dst[2 + 16 * v + 4 * j + i] = acc_o[v][i];
        }
        return;
    }
    const float inv = l_row > 0.f ? 1.f / l_row : 0.f;
#pragma unroll
    for (int v = 0; v < DV16; ++v)
#pragma unroll
        for (int i = 0; i < 4; ++i) os[r][16 * v + 4 * j + i] = acc_o[v][i] * inv;
    __syncthreads();
    const int rows = tq_n * group;
    constexpr int VH = VD / 2;
    for (int c = tid; c < rows * VD; c += PC_THREADS) {
        const int row = c / VD, x = c % VD;
        const int tok = row / group, head = row % group;
        float o = os[row][x];
        if (vtable) {
            const int pr = x < VH ? x : x - VH;
            const float cs = vtable[((int64_t)(t0 + tok) * VH + pr) * 2], sn = vtable[((int64_t)(t0 + tok) * VH + pr) * 2 + 1];
            o = x < VH ? os[row][x] * cs + os[row][x + VH] * sn : os[row][x] * cs - os[row][x - VH] * sn;
        }
        zi_store(out + (int64_t)(t0 + tok) * ldo + (int64_t)(g * group + head) * VD + x, o);
    }
}

// The rows of the short entries from their chunks' shares, in rising order of the chunks; turned back where values
// are stored turned.  One workgroup per (token, head); tokens of long entries are left alone.
__global__ void __launch_bounds__(128)
pooled_attention_merge_kernel(zi_bf16* __restrict__ out, int64_t ldo, const float* __restrict__ partial, int chunks,
                              int total_rows, int nh, int vd, const float* __restrict__ vtable,
                              const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ entry_len, int long_len) {
    __shared__ float os[128];
    const int t = blockIdx.x, h = blockIdx.y;
    const int len = entry_len[tok_seq[t]];
    if (len >= long_len) return;
    const int64_t row = (int64_t)t * nh + h;
    float M = -1e30f;
    for (int c = 0; c < chunks; ++c) M = fmaxf(M, partial[((int64_t)c * total_rows + row) * (vd + 2)]);
    float L = 0.f;
    for (int c = 0; c < chunks; ++c) {
        const float* p = partial + ((int64_t)c * total_rows + row) * (vd + 2);
        L += p[1] * exp2f(p[0] - M);
    }
    const int x = threadIdx.x;
    if (x < vd) {
        float o = 0.f;
        for (int c = 0; c < chunks; ++c) {
            const float* p = partial + ((int64_t)c * total_rows + row) * (vd + 2);
            o += p[2 + x] * exp2f(p[0] - M);
        }
        os[x] = L > 0.f ? o / L : 0.f;
    }
    __syncthreads();
    if (x < vd) {
        float o = os[x];
        const int vh = vd / 2;
        if (vtable) {
            const int pr = x < vh ? x : x - vh;
            const float cs = vtable[((int64_t)t * vh + pr) * 2], sn = vtable[((int64_t)t * vh + pr) * 2 + 1];
            o = x < vh ? os[x] * cs + os[x + vh] * sn : os[x] * cs - os[x - vh] * sn;
        }
        zi_store(out + (int64_t)t * ldo + (int64_t)h * vd + x, o);
    }
}

extern "C" int zi_pooled_attention_cores_supported(int dt, int nh, int nkv, int dim, int vdim) {
    return dt == ZI_BF16 && nkv > 0 && nh % nkv == 0 && nh / nkv <= PC_ROWS && (dim == 32 || dim == 64 || dim == 96 || dim == 128) &&
           vdim % 16 == 0 && vdim >= 16 && vdim <= 128;
}

// The entries of at least `long_len` tokens of this step; `max_len` is the most tokens an entry brings (it sizes the
// launch).  Everything else as zi_pooled_attention.  With chunks > 0 instead the entries of FEWER than long_len tokens
// (long_len - 1 tokens times the heads of a group must fit 64 rows): every entry's items are cut into `chunks` chunks
// of chunk_blocks blocks of 32 (the caller sees to it that they cover the items of every such entry), whose shares go
// through `partial` (chunks * n * nh * (vdim + 2) floats) and a second kernel; tok_seq [n] names every token's entry.
extern "C" int zi_pooled_attention_cores(void* out, int64_t ldo, const void* q, int64_t ldq, const void* kcache,
                                         const void* vcache, const float* kpool, const float* vpool,
                                         const int32_t* entry_start, const int32_t* entry_len, const int32_t* entry_past,
                                         int entries, int max_len, const int32_t* block_tables, int max_pages, int num_pages,
                                         int page_size, const int32_t* pool_tables, int pool_max_pages, int pool_num_pages,
                                         int pool_page_size, int nh, int nkv, int dim, int vdim, int window, int pool,
                                         float scale, const float* vtable, int long_len, int chunks, int chunk_blocks,
                                         float* partial, int64_t partial_floats, const int32_t* tok_seq, int n,
                                         hipStream_t stream) {
    ZI_REQUIRE(zi_pooled_attention_cores_supported(ZI_BF16, nh, nkv, dim, vdim), "pooled_attention_cores: sizes it does not take "
               "(heads %d/%d, dim %d, vdim %d)", nh, nkv, dim, vdim);
    ZI_REQUIRE(entries >= 0 && entries <= 65535 && nkv <= 65535 && max_len >= 0 && page_size > 0 && max_pages > 0 && num_pages > 0 &&
               window >= 0 && pool >= 0 && long_len >= 1, "pooled_attention_cores: bad sizes");
    ZI_REQUIRE(!pool_tables || pool == 0 || (kpool && vpool && pool_max_pages > 0 && pool_num_pages > 0 && pool_page_size > 0),
               "pooled_attention_cores: blocks without a cache of their means");
    ZI_REQUIRE(ldq >= (int64_t)nh * dim && ldo >= (int64_t)nh * vdim && ldq % 8 == 0 && ((uintptr_t)q % 16) == 0 &&
               ((uintptr_t)kcache % 16) == 0 && ((uintptr_t)vcache % 16) == 0, "pooled_attention_cores: rows must be 16-byte aligned");
    const int tq_tile = PC_ROWS / (nh / nkv);
    const bool split = chunks > 0;
    if (split) {
        ZI_REQUIRE(chunk_blocks > 0 && chunks <= 65535 && long_len - 1 <= tq_tile && tok_seq && n >= 0,
                   "pooled_attention_cores: a bad cut (%d chunks of %d blocks, entries below %d tokens)", chunks, chunk_blocks, long_len);
        ZI_REQUIRE(partial && partial_floats >= (int64_t)chunks * n * nh * (vdim + 2), "pooled_attention_cores: the workspace is too small");
        if (entries == 0 || n == 0) return 0;
    } else if (entries == 0 || max_len < long_len) {
        return 0;
    }
    const dim3 grid(split ? chunks : (max_len + tq_tile - 1) / tq_tile, nkv, entries);
    const int total_rows = n * nh;
    const float scale_log2 = scale * 1.4426950408889634f;
#define ZI_PC(DK32, DV16)                                                                                              \
    pooled_attention_cores_kernel<DK32, DV16><<<grid, PC_THREADS, 0, stream>>>(                                        \
        (zi_bf16*)out, ldo, (const zi_bf16*)q, ldq, (const zi_bf16*)kcache, (const zi_bf16*)vcache, kpool, vpool,      \
        entry_start, entry_len, entry_past, block_tables, max_pages, num_pages, page_size, pool > 0 ? pool_tables : nullptr, \
        pool_max_pages, pool_num_pages, pool_page_size, nh, nkv, window, pool, scale_log2, vtable, long_len,           \
        split ? chunk_blocks : 0, partial, total_rows)
#define ZI_PC_V(DK32)                                   \
    switch (vdim / 16) {                                \
        case 1: ZI_PC(DK32, 1); break;                  \
        case 2: ZI_PC(DK32, 2); break;                  \
        case 3: ZI_PC(DK32, 3); break;                  \
        case 4: ZI_PC(DK32, 4); break;                  \
        case 5: ZI_PC(DK32, 5); break;                  \
        case 6: ZI_PC(DK32, 6); break;                  \
        case 7: ZI_PC(DK32, 7); break;                  \
        default: ZI_PC(DK32, 8); break;                 \
    }
    switch (dim / 32) {
        case 1: ZI_PC_V(1); break;
        case 2: ZI_PC_V(2); break;
        case 3: ZI_PC_V(3); break;
        default: ZI_PC_V(4); break;
    }
#undef ZI_PC_V
#undef ZI_PC
    const int rc = zi_check_launch("pooled_attention_cores");
    if (rc != 0 || !split) return rc;
    pooled_attention_merge_kernel<<<dim3(n, nh), 128, 0, stream>>>((zi_bf16*)out, ldo, partial, chunks, total_rows, nh, vdim,
                                                                  vtable, tok_seq, entry_len, long_len);
    return zi_check_launch("pooled_attention_merge");
}
