// Plain matrix product out[M,N] = a[M,K] * w[N,K]^T (+ bias) with 32-bit FMA only:
// the matrix product of the true 32-bit path, and the yardstick of the MFMA kernels.
// Weights are [n_out][n_in] row-major as the reference keeps them
// (src/model.c:193-205).  A row's result does not depend on the rows beside it, but the order
// of its sum over k depends on how many rows the product has: with more than 16 rows the tile
// kernel below sums in ascending order in two levels, with up to 16 the kernel further down
// (k_gemv_ref) gives every lane every 64th group of four columns and adds the lanes' sums in a
// tree.  A token's 32-bit result therefore differs in its last bits between a step of 16 rows and
// one of 17 (both stay within 1e-6 of the exact product at K = 14,336).
// The tile kernel's two levels: runs of RBK * RB_FOLD = 128 columns are summed by FMA, and the runs'
// sums are added up with a compensated (Kahan) sum.  One running 32-bit sum over the 14,336
// columns of a wide feed-forward loses about 1e-5 of the result to rounding, which at such
// widths is as much as a real fault may be; summed this way a product is about ten times closer
// to the exact one, so the 32-bit path can be held to the tolerance that small models are.
#include "common.h"

#define RBM 64
#define RBN 64
#define RBK 16
#define RB_FOLD 8

template <typename TI, typename TO, bool ACC>
__global__ __launch_bounds__(256) void k_gemm_ref(TO* __restrict__ out, const TI* __restrict__ a,
                                                   const TI* __restrict__ w, const float* __restrict__ bias,
                                                   int M, int N, int K, int lda, int ldo) {
    __shared__ float As[RBK][RBM + 4];
    __shared__ float Ws[RBK][RBN + 4];
    int m0 = blockIdx.y * RBM, n0 = blockIdx.x * RBN;
    int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    float acc[4][4], tot[4][4], lost[4][4];      // the run's sum, the sum of the runs, what that sum has lost
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = tot[i][j] = lost[i][j] = 0.f;
#define FOLD_RUN()                                                   \
    _Pragma("unroll") for (int i = 0; i < 4; ++i)                    \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) {              \
            const float y = acc[i][j] - lost[i][j];                  \
            const float t = tot[i][j] + y;                           \
            lost[i][j] = (t - tot[i][j]) - y;                        \
            tot[i][j] = t;                                           \
            acc[i][j] = 0.f;                                         \
        }

    int slice = 0;
    for (int k0 = 0; k0 < K; k0 += RBK, ++slice) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            int idx = threadIdx.x + e * 256;
            int r = idx >> 4, kk = idx & 15;
            int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
            As[kk][r] = (gm < M && gk < K) ? ld<TI>(a, (size_t)gm * lda + gk) : 0.f;
            Ws[kk][r] = (gn < N && gk < K) ? ld<TI>(w, (size_t)gn * K + gk) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < RBK; ++kk) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
        if (slice % RB_FOLD == RB_FOLD - 1) { FOLD_RUN() }
    }
    FOLD_RUN()
#undef FOLD_RUN
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int gm = m0 + ty * 4 + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int gn = n0 + tx * 4 + j;
            if (gn >= N) continue;
            float v = tot[i][j];
            if (bias) v += bias[gn];
            size_t o = (size_t)gm * ldo + gn;
            if (ACC) v += ld<TO>(out, o);
            st<TO>(out, o, v);
        }
    }
}

// Up to 16 rows of 32-bit operands (decoded tokens): the product is bound by how fast the weights
// arrive, and the tile kernel above, 64 weight rows a workgroup, leaves most of the chip idle then
// (a decode step of the Llama-3.1-8B shape took 136 ms).  Here a wave takes 8 weight rows: a lane
// sums, for every row of `a` and each of them, the columns 4 l .. 4 l + 3 (mod 256) in ascending
// order by FMA, and the lanes' sums are added in a fixed tree.  A row's result does not depend
// on the rows beside it; it differs from the tile kernel's by the order of the sum only.
template <int MT, typename TO, bool ACC>
__global__ __launch_bounds__(256) void k_gemv_ref(TO* __restrict__ out, const float* __restrict__ a,
                                                   const float* __restrict__ w, const float* __restrict__ bias,
                                                   int M, int N, int K, int lda, int ldo) {
    constexpr int COLS = 8;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = (blockIdx.x * 4 + wave) * COLS;
    if (n0 >= N) return;
    float acc[COLS][MT];
#pragma unroll
    for (int c = 0; c < COLS; ++c)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[c][m] = 0.f;
    for (int k = lane * 4; k < K; k += 256) {
        float4 av[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m)
            av[m] = m < M ? *reinterpret_cast<const float4*>(a + (size_t)m * lda + k) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
            const int n = n0 + c;
            const float4 wv = n < N ? *reinterpret_cast<const float4*>(w + (size_t)n * K + k) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                float t = acc[c][m];
                t = fmaf(av[m].x, wv.x, t);
                t = fmaf(av[m].y, wv.y, t);
                t = fmaf(av[m].z, wv.z, t);
                t = fmaf(av[m].w, wv.w, t);
                acc[c][m] = t;
            }
        }
    }
#pragma unroll
    for (int c = 0; c < COLS; ++c)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float v = acc[c][m];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
            const int n = n0 + c;
            if (lane == 0 && m < M && n < N) {
                if (bias) v += bias[n];
                const size_t at = (size_t)m * ldo + n;
                if (ACC) v += ld<TO>(out, at);
                st<TO>(out, at, v);
            }
        }
}

template <int MT>
static void launch_gemv_ref(void* out, const float* a, const float* w, const float* bias, int M, int N, int K,
                            int lda, int ldo, int out_dtype, int accumulate, hipStream_t stream) {
    const unsigned blocks = (unsigned)((N + 31) / 32);
    if (out_dtype == XR_BF16) k_gemv_ref<MT, bf16_t, false><<<blocks, 256, 0, stream>>>((bf16_t*)out, a, w, bias, M, N, K, lda, ldo);
    else if (accumulate) k_gemv_ref<MT, float, true><<<blocks, 256, 0, stream>>>((float*)out, a, w, bias, M, N, K, lda, ldo);
    else k_gemv_ref<MT, float, false><<<blocks, 256, 0, stream>>>((float*)out, a, w, bias, M, N, K, lda, ldo);
}

// accumulate != 0: out (float) += product.
extern "C" int xr_gemm_ref(void* out, const void* a, const void* w, const float* bias, int M, int N, int K,
                           int lda, int ldo, int in_dtype, int out_dtype, int accumulate, hipStream_t stream) {
    XR_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    XR_REQUIRE(lda >= K && ldo >= N, "gemm: row strides lda=%d ldo=%d are shorter than K=%d N=%d", lda, ldo, K, N);
    XR_REQUIRE(!accumulate || out_dtype == XR_F32, "gemm: accumulation needs a 32-bit output");
    if (M == 0) return XR_OK;
    if (M <= 16 && in_dtype == XR_F32 && (out_dtype == XR_F32 || out_dtype == XR_BF16) && K % 4 == 0 && lda % 4 == 0 &&
        ((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0) {
        const float* af = (const float*)a;
        const float* wf = (const float*)w;
        if (M == 1) launch_gemv_ref<1>(out, af, wf, bias, M, N, K, lda, ldo, out_dtype, accumulate, stream);
        else if (M <= 4) launch_gemv_ref<4>(out, af, wf, bias, M, N, K, lda, ldo, out_dtype, accumulate, stream);
        else if (M <= 8) launch_gemv_ref<8>(out, af, wf, bias, M, N, K, lda, ldo, out_dtype, accumulate, stream);
        else launch_gemv_ref<16>(out, af, wf, bias, M, N, K, lda, ldo, out_dtype, accumulate, stream);
        XR_CHECK_LAUNCH("gemv_ref");
        return XR_OK;
    }
    dim3 grid((N + RBN - 1) / RBN, (M + RBM - 1) / RBM);
#define G(TI, TO, ACC) k_gemm_ref<TI, TO, ACC><<<grid, 256, 0, stream>>>((TO*)out, (const TI*)a, (const TI*)w, bias, M, N, K, lda, ldo)
    if (in_dtype == XR_F32 && out_dtype == XR_F32) { if (accumulate) G(float, float, true); else G(float, float, false); }
    else if (in_dtype == XR_BF16 && out_dtype == XR_F32) { if (accumulate) G(bf16_t, float, true); else G(bf16_t, float, false); }
    else if (in_dtype == XR_BF16 && out_dtype == XR_BF16) G(bf16_t, bf16_t, false);
    else if (in_dtype == XR_F32 && out_dtype == XR_BF16) G(float, bf16_t, false);
    else { xr_set_error("gemm: bad dtypes in=%d out=%d", in_dtype, out_dtype); return XR_BAD_ARG; }
#undef G
    XR_CHECK_LAUNCH("gemm_ref");
    return XR_OK;
}
