// Element-wise and row-wise kernels of the forward pass, for float and bfloat16
// storage: embedding gather, RMSNorm, rotary position encoding fused with the
// write of keys and values into cache pages, SiLU-gate, residual add, fill.
// All arithmetic is 32-bit float; only loads and stores see the storage type.
#include "common.h"

// ---------------------------------------------------------------- embedding
// x[t] = table[id_t]; an id outside [0, V) reads row 0
// (src/model.c:6148-6162).
template <typename TW>
__global__ void k_embedding(float* __restrict__ out, const TW* __restrict__ table,
                            const int* __restrict__ ids, int E, int V, float scale) {
    int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 || id >= V) id = 0;
    const TW* row = table + (size_t)id * E;
    float* o = out + (size_t)t * E;
    for (int i = threadIdx.x; i < E; i += blockDim.x) o[i] = ld<TW>(row, i) * scale;
}

// The same from a bfloat16 table in the matrix kernels' packed order (blocks of 16 rows x 32
// columns, 1 KB each, [row group][column block][row][column]): a model that ties its output
// head to the embedding then keeps the table once, in the order the head's product reads it.
__global__ void k_embedding_packed(float* __restrict__ out, const bf16_t* __restrict__ table,
                                   const int* __restrict__ ids, int E, int V, float scale) {
    int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 || id >= V) id = 0;
    const size_t kblocks = (size_t)((E + 31) / 32);
    const bf16_t* grp = table + (size_t)(id >> 4) * kblocks * 512 + (id & 15) * 32;
    float* o = out + (size_t)t * E;
    for (int i = threadIdx.x; i < E; i += blockDim.x) o[i] = bf16_to_f32(grp[(size_t)(i >> 5) * 512 + (i & 31)]) * scale;
}

extern "C" int xr_embedding(float* out, const void* table, const int* ids, int T, int E, int V,
                            float scale, int table_dtype, int packed, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && E > 0 && V > 0, "embedding: bad sizes T=%d E=%d V=%d", T, E, V);
    XR_REQUIRE(table_dtype == XR_F32 || table_dtype == XR_BF16, "embedding: bad dtype %d", table_dtype);
    XR_REQUIRE(!packed || table_dtype == XR_BF16, "embedding: a packed table is bfloat16");
    if (T == 0) return XR_OK;
    if (packed)
        k_embedding_packed<<<T, 256, 0, stream>>>(out, (const bf16_t*)table, ids, E, V, scale);
    else if (table_dtype == XR_F32)
        k_embedding<float><<<T, 256, 0, stream>>>(out, (const float*)table, ids, E, V, scale);
    else
        k_embedding<bf16_t><<<T, 256, 0, stream>>>(out, (const bf16_t*)table, ids, E, V, scale);
    XR_CHECK_LAUNCH("embedding");
    return XR_OK;
}

// ---------------------------------------------------------------- RMSNorm
// y_i = x_i * r * w_i with r = 1/sqrt(mean(x^2) + eps): eps inside the root, added to
// the mean; multiply order (x*r)*w (src/model.c:3386-3392).
template <typename TO, typename TW>
__global__ void k_rmsnorm(TO* __restrict__ out, const float* __restrict__ x, const TW* __restrict__ w,
                          const int* __restrict__ rows, int E, int ldx, float eps) {
    __shared__ float part[4];
    int r = blockIdx.x;
    int src = rows ? rows[r] : r;
    const float* xr = x + (size_t)src * ldx;
    float ss = 0.f;
    for (int i = threadIdx.x; i < E; i += blockDim.x) {
        float v = xr[i];
        ss += v * v;
    }
    ss = wave_sum(ss);
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) part[wave] = ss;
    __syncthreads();
    float tot = part[0] + part[1] + part[2] + part[3];
    float rinv = 1.0f / sqrtf(tot / (float)E + eps);
    TO* o = out + (size_t)r * E;
    if (w) {
        for (int i = threadIdx.x; i < E; i += blockDim.x) st<TO>(o, i, xr[i] * rinv * ld<TW>(w, i));
    } else {
        for (int i = threadIdx.x; i < E; i += blockDim.x) st<TO>(o, i, xr[i] * rinv);
    }
}

// Rows whose width is a multiple of 4 (up to 4 * 256 * RN_MAXV): every thread keeps its
// float4 pieces in registers between the sum and the scaling, and writes 4 values at a time.
#define RN_MAXV 8
template <typename TO> __device__ inline void st4(TO* p, size_t i, float a, float b, float c, float d);
template <> __device__ inline void st4<float>(float* p, size_t i, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(p + i) = make_float4(a, b, c, d);
}
template <> __device__ inline void st4<bf16_t>(bf16_t* p, size_t i, float a, float b, float c, float d) {
    uint2 w;
    w.x = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
    w.y = (uint32_t)f32_to_bf16(c) | ((uint32_t)f32_to_bf16(d) << 16);
    *reinterpret_cast<uint2*>(p + i) = w;
}

template <typename TO, typename TW, int NV>
__global__ __launch_bounds__(256) void k_rmsnorm_v4(TO* __restrict__ out, const float* __restrict__ x,
                                                    const TW* __restrict__ w, const int* __restrict__ rows,
                                                    int E, int ldx, float eps) {
    __shared__ float part[4];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)src * ldx);
    const int n4 = E >> 2;
    float4 v[NV];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = threadIdx.x + i * 256;
        v[i] = c < n4 ? xr[c] : make_float4(0.f, 0.f, 0.f, 0.f);
        ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    }
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float tot = part[0] + part[1] + part[2] + part[3];
    const float rinv = 1.0f / sqrtf(tot / (float)E + eps);
    TO* o = out + (size_t)r * E;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int c = threadIdx.x + i * 256;
        if (c >= n4) continue;
        float w0 = 1.f, w1 = 1.f, w2 = 1.f, w3 = 1.f;
        if (w) { w0 = ld<TW>(w, 4 * c); w1 = ld<TW>(w, 4 * c + 1); w2 = ld<TW>(w, 4 * c + 2); w3 = ld<TW>(w, 4 * c + 3); }
        st4<TO>(o, (size_t)4 * c, v[i].x * rinv * w0, v[i].y * rinv * w1, v[i].z * rinv * w2, v[i].w * rinv * w3);
    }
}

extern "C" int xr_rmsnorm(void* out, const float* x, const void* w, const int* rows, int R, int E,
                          int ldx, float eps, int out_dtype, int w_dtype, hipStream_t stream) {
    XR_REQUIRE(R >= 0 && E > 0 && ldx >= E, "rmsnorm: bad sizes R=%d E=%d ldx=%d", R, E, ldx);
    XR_REQUIRE(eps >= 0.f, "rmsnorm: eps %g is negative", eps);
    XR_REQUIRE((out_dtype == XR_F32 || out_dtype == XR_BF16) && (w_dtype == XR_F32 || w_dtype == XR_BF16),
               "rmsnorm: bad dtypes out=%d w=%d", out_dtype, w_dtype);
    if (R == 0) return XR_OK;
    const bool vec = E % 4 == 0 && ldx % 4 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0 &&
                     E <= 4 * 256 * RN_MAXV;
#define RN(TO, TW)                                                                                              \
    do {                                                                                                        \
        if (!vec) k_rmsnorm<TO, TW><<<R, 256, 0, stream>>>((TO*)out, x, (const TW*)w, rows, E, ldx, eps);        \
        else if (E <= 4 * 256 * 2) k_rmsnorm_v4<TO, TW, 2><<<R, 256, 0, stream>>>((TO*)out, x, (const TW*)w, rows, E, ldx, eps); \
        else if (E <= 4 * 256 * 4) k_rmsnorm_v4<TO, TW, 4><<<R, 256, 0, stream>>>((TO*)out, x, (const TW*)w, rows, E, ldx, eps); \
        else k_rmsnorm_v4<TO, TW, RN_MAXV><<<R, 256, 0, stream>>>((TO*)out, x, (const TW*)w, rows, E, ldx, eps); \
    } while (0)
    if (out_dtype == XR_F32 && w_dtype == XR_F32) RN(float, float);
    else if (out_dtype == XR_F32 && w_dtype == XR_BF16) RN(float, bf16_t);
    else if (out_dtype == XR_BF16 && w_dtype == XR_F32) RN(bf16_t, float);
    else RN(bf16_t, bf16_t);
#undef RN
    XR_CHECK_LAUNCH("rmsnorm");
    return XR_OK;
}

// ---------------------------------------------------------------- rotary + cache write
// Rotation of pair index j of a head by a = pos * inv_freq[j]:
//   (x0, x1) -> (x0*c - x1*s, x0*s + x1*c), c = cos(a)*mscale, s = sin(a)*mscale
// (src/model.c:3514-3532).  Half-split pairs (j, j + rot/2) are what
// un-permuted checkpoints need; interleaved pairs (2j, 2j+1) are the other option.
// Keys are cached rotated, values as they are (src/model.c:6300-6311).
// Cache layout per layer: K [page][kv_head][slot][d], V [page][kv_head][d][slot].
struct RopeArgs {
    const float* q_in;      // [T, in_stride] 32-bit
    const float* k_in;
    const float* v_in;
    int in_stride;
    void* q_out;            // [T, H*D] storage type
    void* k_cache;
    void* v_cache;
    const int* positions;   // [T]
    const int* req_of_token;// [T]
    const int* block_table; // [B, table_stride]
    int table_stride;
    const float* inv_freq;  // [rot/2] or null
    int T, H, Hk, D, rot, interleaved;
    float mscale;
    int page_shift, page_mask, page_size;
    int heads_per_block;
    int paired;             // queries and keys come in paired order (paired_col)
};

// 8 values of one channel at 8 consecutive positions of a page: 16 or 32 bytes side by side in
// the transposed value cache.
template <typename T> __device__ inline void store8(T* dst, const float* v);
template <> __device__ inline void store8<float>(float* dst, const float* v) {
    *reinterpret_cast<float4*>(dst) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(dst + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
template <> __device__ inline void store8<bf16_t>(bf16_t* dst, const float* v) {
    *reinterpret_cast<uint4*>(dst) = make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]),
                                                pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7]));
}

// A workgroup takes a token and some of its heads (heads_per_block, a wave a head at a time):
// query heads are rotated into q_out, key heads rotated into their page, value heads written
// to theirs.  The cosines and sines of the token's angles are computed once per workgroup into
// LDS and serve every head (the exact cosf/sinf of 64 angles for each of 40 heads was what the
// kernel's time went to).  Values are cached transposed ([channel][position]), so a token
// alone writes one element every page_size: where the step brings the 8 positions of an
// aligned group of a page (prompt portions), the wave of the group's first token writes all 8
// side by side for each channel and the other seven leave their values to it.
template <typename T>
__global__ __launch_bounds__(256) void k_rope_kv_write(RopeArgs a) {
    __shared__ float cs[2][128];
    const int t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int pos = a.positions[t];
    const int D = a.D, half = a.rot >> 1;
    for (int j = threadIdx.x; j < half; j += 256) {
        const float ang = (float)pos * a.inv_freq[j];
        cs[0][j] = cosf(ang) * a.mscale;
        cs[1][j] = sinf(ang) * a.mscale;
    }
    __syncthreads();
    const int h_begin = blockIdx.y * a.heads_per_block;
    const int h_end = min(a.H + a.Hk, h_begin + a.heads_per_block);
    // query heads, four at a time per wave: the loads of all four are on their way before the
    // first is used (one head at a time, a wave waited out a memory latency per head)
    const int hq_end = min(h_end, a.H);
    for (int hb = h_begin + wave * 4; hb < hq_end; hb += 16) {
        const float* src[4];
        T* dst[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int hs = hb + u < hq_end ? hb + u : hb;
            src[u] = a.q_in + (size_t)t * a.in_stride + (size_t)hs * D;
            dst[u] = (T*)a.q_out + ((size_t)t * a.H + hs) * D;
        }
        for (int j = lane; j < half; j += 64) {
            const int i0 = a.interleaved ? 2 * j : j;
            const int i1 = a.interleaved ? 2 * j + 1 : j + half;
            const int c0 = a.paired ? paired_col(i0, a.rot) : i0, c1 = a.paired ? paired_col(i1, a.rot) : i1;
            float x0[4], x1[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) { x0[u] = src[u][c0]; x1[u] = src[u][c1]; }
            const float c = cs[0][j], sn = cs[1][j];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (hb + u < hq_end) {
                    st<T>(dst[u], i0, x0[u] * c - x1[u] * sn);
                    st<T>(dst[u], i1, x0[u] * sn + x1[u] * c);
                }
        }
        for (int i = a.rot + lane; i < D; i += 64) {
            float x[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) x[u] = src[u][i];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (hb + u < hq_end) st<T>(dst[u], i, x[u]);
        }
    }
    for (int hs = max(h_begin, a.H) + wave; hs < h_end; hs += 4) {
        const int kvh = hs - a.H;
        const int req = a.req_of_token[t];
        PageRef pr = page_of(a.block_table, a.table_stride, req, pos, a.page_shift, a.page_mask);
        const float* ks = a.k_in + (size_t)t * a.in_stride + (size_t)kvh * D;
        const float* vs = a.v_in + (size_t)t * a.in_stride + (size_t)kvh * D;
        T* kd = (T*)a.k_cache + (((size_t)pr.page * a.Hk + kvh) * a.page_size + pr.off) * D;
        T* vd = (T*)a.v_cache + ((size_t)pr.page * a.Hk + kvh) * D * a.page_size + pr.off;
        for (int j = lane; j < half; j += 64) {
            const int i0 = a.interleaved ? 2 * j : j;
            const int i1 = a.interleaved ? 2 * j + 1 : j + half;
            const float x0 = ks[a.paired ? paired_col(i0, a.rot) : i0], x1 = ks[a.paired ? paired_col(i1, a.rot) : i1];
            const float c = cs[0][j], sn = cs[1][j];
            st<T>(kd, i0, x0 * c - x1 * sn);
            st<T>(kd, i1, x0 * sn + x1 * c);
        }
        for (int i = a.rot + lane; i < D; i += 64) st<T>(kd, i, ks[i]);
        // the aligned group of 8 positions this token belongs to: whole in this step?  (A request's
        // tokens of a step are consecutive rows at consecutive positions.)
        const int lead = t - (pos & 7);
        const bool whole = a.page_size >= 8 && lead >= 0 && lead + 7 < a.T && a.req_of_token[lead] == req &&
                           a.req_of_token[lead + 7] == req && a.positions[lead] == pos - (pos & 7);
        if (!whole) {
            for (int i = lane; i < D; i += 64) st<T>(vd, (size_t)i * a.page_size, vs[i]);
        } else if ((pos & 7) == 0) {
            for (int i = lane; i < D; i += 64) {
                float v[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = vs[(size_t)j * a.in_stride + i];
                store8<T>(vd + (size_t)i * a.page_size, v);
            }
        }
    }
}

extern "C" int xr_rope_kv_write(const float* q_in, const float* k_in, const float* v_in, int in_stride,
                                void* q_out, void* k_cache, void* v_cache, const int* positions,
                                const int* req_of_token, const int* block_table, int table_stride,
                                const float* inv_freq, int T, int H, int Hk, int D, int rot,
                                int interleaved, float mscale, int page_size, int dtype, int paired,
                                hipStream_t stream) {
    XR_REQUIRE(T >= 0 && H >= 0 && Hk >= 0 && D > 0, "rope_kv_write: bad sizes T=%d H=%d Hk=%d D=%d", T, H, Hk, D);
    XR_REQUIRE(rot >= 0 && rot <= D && (rot % 2) == 0, "rope_kv_write: rotary width %d must be even and at most head_dim %d", rot, D);
    XR_REQUIRE(rot == 0 || inv_freq, "rope_kv_write: rotary width %d without a frequency table", rot);
    int shift = ilog2_exact(page_size);
    XR_REQUIRE(Hk == 0 || shift >= 0, "rope_kv_write: page size %d is not a power of two", page_size);
    XR_REQUIRE(Hk == 0 || (k_in && v_in && k_cache && v_cache && block_table && req_of_token),
               "rope_kv_write: keys and values to cache but a null operand");
    XR_REQUIRE(H == 0 || (q_in && q_out), "rope_kv_write: queries but a null operand");
    XR_REQUIRE(dtype == XR_F32 || dtype == XR_BF16, "rope_kv_write: bad dtype %d", dtype);
    if (T == 0 || H + Hk == 0) return XR_OK;
    RopeArgs a;
    a.q_in = q_in; a.k_in = k_in; a.v_in = v_in; a.in_stride = in_stride;
    a.q_out = q_out; a.k_cache = k_cache; a.v_cache = v_cache;
    a.positions = positions; a.req_of_token = req_of_token;
    a.block_table = block_table; a.table_stride = table_stride; a.inv_freq = inv_freq;
    a.T = T; a.H = H; a.Hk = Hk; a.D = D; a.rot = rot; a.interleaved = interleaved; a.mscale = mscale;
    a.page_shift = shift < 0 ? 0 : shift; a.page_mask = page_size - 1; a.page_size = page_size;
    XR_REQUIRE(rot <= 256, "rope_kv_write: rotary width %d exceeds 256", rot);
    XR_REQUIRE(!paired || (!interleaved && rot % 16 == 0), "rope_kv_write: paired order needs pairs (j, j + width/2) and a rotary width (%d) that is a multiple of 16", rot);
    a.paired = paired ? 1 : 0;
    // all heads of a token in one workgroup when there are tokens enough to fill the chip, else
    // fewer heads each, down to one a wave
    int groups = (1024 + T - 1) / T;
    const int max_groups = (H + Hk + 3) / 4;
    groups = groups < 1 ? 1 : (groups > max_groups ? max_groups : groups);
    a.heads_per_block = (H + Hk + groups - 1) / groups;
    dim3 grid(T, (H + Hk + a.heads_per_block - 1) / a.heads_per_block);
    if (dtype == XR_F32) k_rope_kv_write<float><<<grid, 256, 0, stream>>>(a);
    else k_rope_kv_write<bf16_t><<<grid, 256, 0, stream>>>(a);
    XR_CHECK_LAUNCH("rope_kv_write");
    return XR_OK;
}

// ---------------------------------------------------------------- gate
// h = act(g) * u; act = SiLU: g / (1 + exp(-g)) (src/model.c:4451-4452,
// src/kernels.cu:2868-2874).  gu row = [gate(F) | up(F)].
template <typename TI, typename TO>
__global__ void k_gate_mul(TO* __restrict__ out, const TI* __restrict__ gu, int F, int ld_gu, size_t n, int act) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    size_t t = i / F;
    int c = (int)(i - t * F);
    float g = ld<TI>(gu, t * ld_gu + c);
    float u = ld<TI>(gu, t * ld_gu + F + c);
    st<TO>(out, i, gate_act<false>(act, g) * u);
}

extern "C" int xr_gate_mul(void* out, const void* gu, int T, int F, int ld_gu, int dtype, int act, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && F > 0 && ld_gu >= 2 * F, "gate_mul: bad sizes T=%d F=%d ld=%d", T, F, ld_gu);
    XR_REQUIRE(act >= 0 && act < XR_ACT_COUNT, "gate_mul: unknown activation code %d", act);
    size_t n = (size_t)T * F;
    if (n == 0) return XR_OK;
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == XR_F32) k_gate_mul<float, float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)gu, F, ld_gu, n, act);
    else if (dtype == XR_BF16) k_gate_mul<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)gu, F, ld_gu, n, act);
    else { xr_set_error("gate_mul: bad dtype %d", dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("gate_mul");
    return XR_OK;
}

// ---------------------------------------------------------------- residual add
template <typename TY>
__global__ void k_add(float* __restrict__ x, const TY* __restrict__ y, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = x[i] + ld<TY>(y, i);
}

extern "C" int xr_add(float* x, const void* y, size_t n, int y_dtype, hipStream_t stream) {
    if (n == 0) return XR_OK;
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (y_dtype == XR_F32) k_add<float><<<blocks, 256, 0, stream>>>(x, (const float*)y, n);
    else if (y_dtype == XR_BF16) k_add<bf16_t><<<blocks, 256, 0, stream>>>(x, (const bf16_t*)y, n);
    else { xr_set_error("add: bad dtype %d", y_dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("add");
    return XR_OK;
}

// ---------------------------------------------------------------- fill (32-bit words)
__global__ void k_fill_rows(uint32_t* __restrict__ base, const int* __restrict__ rows, size_t row_words,
                            uint32_t value) {
    int r = rows ? rows[blockIdx.y] : blockIdx.y;
    if (r < 0) return;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < row_words) base[(size_t)r * row_words + i] = value;
}

// Sets rows[r] (or rows 0..n_rows-1) of a [*, row_words] array of 32-bit words to `value`.
extern "C" int xr_fill_rows(void* base, const int* rows, int n_rows, size_t row_words, uint32_t value,
                            hipStream_t stream) {
    if (n_rows <= 0 || row_words == 0) return XR_OK;
    dim3 grid((unsigned)((row_words + 255) / 256), n_rows);
    k_fill_rows<<<grid, 256, 0, stream>>>((uint32_t*)base, rows, row_words, value);
    XR_CHECK_LAUNCH("fill_rows");
    return XR_OK;
}

// ---------------------------------------------------------------- dtype conversion
template <typename TI, typename TO>
__global__ void k_convert(TO* __restrict__ out, const TI* __restrict__ in, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) st<TO>(out, i, ld<TI>(in, i));
}

extern "C" int xr_convert(void* out, const void* in, size_t n, int in_dtype, int out_dtype, hipStream_t stream) {
    if (n == 0) return XR_OK;
    unsigned blocks = (unsigned)((n + 255) / 256);
    if (in_dtype == XR_F32 && out_dtype == XR_BF16) k_convert<float, bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const float*)in, n);
    else if (in_dtype == XR_BF16 && out_dtype == XR_F32) k_convert<bf16_t, float><<<blocks, 256, 0, stream>>>((float*)out, (const bf16_t*)in, n);
    else if (in_dtype == XR_F32 && out_dtype == XR_F32) k_convert<float, float><<<blocks, 256, 0, stream>>>((float*)out, (const float*)in, n);
    else if (in_dtype == XR_BF16 && out_dtype == XR_BF16) k_convert<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)out, (const bf16_t*)in, n);
    else { xr_set_error("convert: bad dtypes %d -> %d", in_dtype, out_dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("convert");
    return XR_OK;
}

// ---------------------------------------------------------------- memory yardstick
// What the memory system delivers to a kernel that does nothing but read: every workgroup
// streams a range of its own with 16-byte loads marked as streaming, eight of them in flight
// a lane, and leaves the XOR of its words (so the loads cannot be dropped, and a test can
// check that every word was read once).  The benchmark reports a decode step's bytes per second
// as a fraction of this figure beside the fraction of the nominal peak.
typedef uint32_t xr_u32x4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void k_stream_read(const xr_u32x4* __restrict__ src, size_t n16, uint32_t* __restrict__ sink) {
    const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t begin = (size_t)blockIdx.x * per;
    const size_t end = begin + per < n16 ? begin + per : n16;
    xr_u32x4 acc = {0u, 0u, 0u, 0u};
    size_t i = begin + threadIdx.x;
    for (; i + 7 * 256 < end; i += 8 * 256) {
        xr_u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i + u * 256);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u];
    }
    for (; i < end; i += 256) acc ^= __builtin_nontemporal_load(src + i);
    uint32_t x = acc.x ^ acc.y ^ acc.z ^ acc.w;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x ^= __shfl_xor(x, o, 64);
    __shared__ uint32_t part[4];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = x;
    __syncthreads();
    if (threadIdx.x == 0) sink[blockIdx.x] = part[0] ^ part[1] ^ part[2] ^ part[3];
}

// sink: [blocks] words; the XOR of all of them is the XOR of the buffer's 32-bit words.
extern "C" int xr_stream_read(const void* src, size_t bytes, uint32_t* sink, int blocks, hipStream_t stream) {
    XR_REQUIRE(src && sink && blocks > 0 && blocks <= 65535, "stream_read: bad operands (%d workgroups)", blocks);
    XR_REQUIRE(bytes % 16 == 0 && ((uintptr_t)src % 16) == 0, "stream_read: the buffer must be a multiple of 16 bytes long and aligned so");
    k_stream_read<<<blocks, 256, 0, stream>>>((const xr_u32x4*)src, bytes / 16, sink);
    XR_CHECK_LAUNCH("stream_read");
    return XR_OK;
}
