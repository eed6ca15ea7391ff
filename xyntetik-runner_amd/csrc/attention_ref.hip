// Attention over the paged cache with 32-bit arithmetic only: the attention of the
// true 32-bit path, for prompt portions and decoded tokens alike, any head size up
// to 256.  One wave per (token, query head).
//
// For the token at position p of its request and query head h (key/value head
// h / (H/Hk), contiguous groups): s_t = (q . K_t) * scale for t in [lo, p], causal by
// the loop bound, lo = max(0, p - window + 1) for a windowed layer
// (src/model.c:3553-3573, :6326); softmax with the maximum taken out
// (src/model.c:3409-3415); out = sum_t p_t V_t (:3576-3587).  The
// softmax runs over blocks of 64 keys with a running maximum and sum, which gives the
// same value up to rounding.
#include "common.h"

#define AR_MAX_D 256

template <typename T>
__global__ __launch_bounds__(64) void k_attention_ref(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kc, const T* __restrict__ vc,
    const int* __restrict__ positions, const int* __restrict__ req_of_token,
    const int* __restrict__ block_table, int table_stride, int H, int Hk, int D, int page_shift,
    int page_mask, int page_size, float scale, int window) {
    __shared__ float qs[AR_MAX_D];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[t];
    const int req = req_of_token[t];
    const int kvh = h / (H / Hk);
    const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    const T* qrow = q + ((size_t)t * H + h) * D;
    for (int d = lane; d < D; d += 64) qs[d] = ld<T>(qrow, d);
    __syncthreads();
    const int* bt = block_table + (size_t)req * table_stride;

    float m = -INFINITY, l = 0.f;
    float acc[AR_MAX_D / 64];
#pragma unroll
    for (int dd = 0; dd < AR_MAX_D / 64; ++dd) acc[dd] = 0.f;

    for (int k0 = lo; k0 <= pos; k0 += 64) {
        const int key = k0 + lane;
        const bool valid = key <= pos;
        float s = -INFINITY;
        if (valid) {
            const int page = bt[key >> page_shift];
            const int off = key & page_mask;
            const T* kr = kc + (((size_t)page * Hk + kvh) * page_size + off) * D;
            float dot = 0.f;
            for (int d = 0; d < D; ++d) dot = fmaf(qs[d], ld<T>(kr, d), dot);
            s = dot * scale;
        }
        const float mn = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - mn) : 0.f;
        const float corr = expf(m - mn);
        l = l * corr + wave_sum(p);
#pragma unroll
        for (int dd = 0; dd < AR_MAX_D / 64; ++dd) acc[dd] *= corr;
        const int nk = (pos - k0 + 1) < 64 ? (pos - k0 + 1) : 64;
        for (int j = 0; j < nk; ++j) {
            const float pj = __shfl(p, j, 64);
            const int kj = k0 + j;
            const int page = bt[kj >> page_shift];
            const int off = kj & page_mask;
            const T* vb = vc + ((size_t)page * Hk + kvh) * D * page_size + off;
#pragma unroll
            for (int dd = 0; dd < AR_MAX_D / 64; ++dd) {
                const int d = lane + 64 * dd;
                if (d < D) acc[dd] = fmaf(pj, ld<T>(vb, (size_t)d * page_size), acc[dd]);
            }
        }
        m = mn;
    }
    T* orow = out + ((size_t)t * H + h) * D;
#pragma unroll
    for (int dd = 0; dd < AR_MAX_D / 64; ++dd) {
        const int d = lane + 64 * dd;
        if (d < D) st<T>(orow, d, acc[dd] / l);
    }
}

extern "C" int xr_attention_ref(void* out, const void* q, const void* k_cache, const void* v_cache,
                                const int* positions, const int* req_of_token, const int* block_table,
                                int table_stride, int T, int H, int Hk, int D, int page_size, float scale,
                                int window, int dtype, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && H > 0 && Hk > 0 && D > 0, "attention: bad sizes T=%d H=%d Hk=%d D=%d", T, H, Hk, D);
    XR_REQUIRE(H % Hk == 0, "attention: %d query heads are not a multiple of %d key/value heads", H, Hk);
    XR_REQUIRE(D <= AR_MAX_D, "attention: head size %d exceeds %d", D, AR_MAX_D);
    int shift = ilog2_exact(page_size);
    XR_REQUIRE(shift >= 0, "attention: page size %d is not a power of two", page_size);
    XR_REQUIRE(window >= 0, "attention: window %d is negative", window);
    if (T == 0) return XR_OK;
    dim3 grid(T, H);
    if (dtype == XR_F32)
        k_attention_ref<float><<<grid, 64, 0, stream>>>((float*)out, (const float*)q, (const float*)k_cache,
                                                        (const float*)v_cache, positions, req_of_token, block_table,
                                                        table_stride, H, Hk, D, shift, page_size - 1, page_size, scale, window);
    else if (dtype == XR_BF16)
        k_attention_ref<bf16_t><<<grid, 64, 0, stream>>>((bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache,
                                                         (const bf16_t*)v_cache, positions, req_of_token, block_table,
                                                         table_stride, H, Hk, D, shift, page_size - 1, page_size, scale, window);
    else { xr_set_error("attention: bad dtype %d", dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("attention_ref");
    return XR_OK;
}
