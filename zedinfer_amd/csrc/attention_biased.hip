// What stands between the projections and the attention kernels of a softmax mixer without rotation whose values
// are normed: zi_normed_kv_store takes float32 rows of one projection (q | k | v somewhere in them), writes the
// queries in the storage type with heads of the cache's size, the keys into the paged cache, and the values, each
// head divided by its root mean square (no gain), into the transposed value cache.  Heads of the cache hold
// d >= dim, vdim values, the rest zero (they change no score and no output).
#include "zi_common.h"
#include "zi_api.h"

template <typename T>
__global__ void __launch_bounds__(256)
normed_kv_store_kernel(T* __restrict__ q_out, int64_t ldq, T* __restrict__ kcache, T* __restrict__ vcache,
                       const float* __restrict__ proj, int64_t ld, int q_at, int k_at, int v_at,
                       const int32_t* __restrict__ slots, int64_t cache_slots, int nh, int nkv, int dim, int vdim, int d,
                       int page_size, float eps, int norm_values) {
    const int64_t t = blockIdx.x;
    const float* row = proj + t * ld;
    for (int j = threadIdx.x; j < nh * d; j += blockDim.x) {
        const int h = j / d, x = j % d;
        zi_store(q_out + t * ldq + j, x < dim ? row[q_at + h * dim + x] : 0.f);
    }
    const int slot = slots ? slots[t] : -1;
    if (!kcache || slot < 0 || slot >= cache_slots) return;      // a token without a place in the cache stores nothing
    const int64_t page = slot / page_size, off = slot % page_size;
    for (int j = threadIdx.x; j < nkv * d; j += blockDim.x) {
        const int g = j / d, x = j % d;
        zi_store(kcache + ((page * nkv + g) * page_size + off) * d + x, x < dim ? row[k_at + g * dim + x] : 0.f);
    }
    const int lane = threadIdx.x % ZI_WAVE, wave = threadIdx.x / ZI_WAVE, waves = blockDim.x / ZI_WAVE;
    for (int g = wave; g < nkv; g += waves) {
        const float* vr = row + v_at + g * vdim;
        float rstd = 1.f;
        if (norm_values) {
            float ss = 0.f;
            for (int x = lane; x < vdim; x += ZI_WAVE) ss += vr[x] * vr[x];
            ss = zi_wave_sum(ss);
            rstd = 1.f / sqrtf(ss / (float)vdim + eps);
        }
        for (int x = lane; x < d; x += ZI_WAVE)
            zi_store(vcache + ((page * nkv + g) * d + x) * page_size + off, x < vdim ? vr[x] * rstd : 0.f);
    }
}

// proj [n][ld] float32 with the queries [nh*dim] at column q_at, the keys [nkv*dim] at k_at, the values [nkv*vdim]
// at v_at.  q_out [n][nh*d]; kcache [pages][nkv][page_size][d], vcache [pages][nkv][d][page_size] (both null: only
// the queries are written); slots [n], negative: the token stores nothing.
extern "C" int zi_normed_kv_store(void* q_out, int dt, int64_t ldq, void* kcache, void* vcache, const float* proj,
                                  int64_t ld, int q_at, int k_at, int v_at, const int32_t* slots, int64_t cache_slots,
                                  int n, int nh, int nkv, int dim, int vdim, int d, int page_size, float eps,
                                  int norm_values, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && nh > 0 && nkv > 0 && dim > 0 && vdim > 0 && d >= dim && d >= vdim && page_size > 0,
               "normed_kv_store: bad sizes");
    ZI_REQUIRE(q_at >= 0 && k_at >= 0 && v_at >= 0 && ld >= q_at + nh * dim && ld >= k_at + nkv * dim &&
               ld >= v_at + nkv * vdim && ldq >= (int64_t)nh * d, "normed_kv_store: the columns do not fit the rows");
    ZI_REQUIRE((kcache == nullptr) == (vcache == nullptr) && (!kcache || slots), "normed_kv_store: caches need slots");
    ZI_REQUIRE(!norm_values || eps > 0.f, "normed_kv_store: eps must be positive");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(dt, T, {
        normed_kv_store_kernel<T><<<n, 256, 0, stream>>>((T*)q_out, ldq, (T*)kcache, (T*)vcache, proj, ld, q_at, k_at, v_at,
                                                         slots, cache_slots, nh, nkv, dim, vdim, d, page_size, eps,
                                                         norm_values);
    });
    return zi_check_launch("normed_kv_store");
}
