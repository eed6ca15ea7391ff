// Shared declarations of the gfx950 kernel library.
//
// Every entry point is extern "C", takes raw device pointers and a HIP stream,
// checks its operands on the host, launches, and returns 0 or a negative code;
// xr_last_error() gives the text of the last failure on the calling thread.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#define XR_OK 0
#define XR_BAD_ARG -1
#define XR_LAUNCH -2

// dtype codes shared with the Python side
#define XR_F32 0
#define XR_BF16 1

#define XR_WAVE 64

typedef uint16_t bf16_t;   // storage only; arithmetic is float

extern "C" const char* xr_last_error();
void xr_set_error(const char* fmt, ...);

#define XR_REQUIRE(cond, ...)                 \
    do {                                      \
        if (!(cond)) {                        \
            xr_set_error(__VA_ARGS__);        \
            return XR_BAD_ARG;                \
        }                                     \
    } while (0)

#define XR_CHECK_LAUNCH(name)                                                   \
    do {                                                                        \
        hipError_t e_ = hipGetLastError();                                      \
        if (e_ != hipSuccess) {                                                 \
            xr_set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
            return XR_LAUNCH;                                                   \
        }                                                                       \
    } while (0)

// ---- bfloat16 <-> float, round to nearest even --------------------------------
__host__ __device__ inline float bf16_to_f32(bf16_t h) {
    union { uint32_t u; float f; } c;
    c.u = ((uint32_t)h) << 16;
    return c.f;
}

__host__ __device__ inline bf16_t f32_to_bf16(float f) {
    union { uint32_t u; float f; } c;
    c.f = f;
    uint32_t u = c.u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);   // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}

// two floats -> two bfloat16 in one word (low half first), round to nearest even, one
// v_cvt_pk_bf16_f32 on gfx950
#if defined(__HIP_DEVICE_COMPILE__)
typedef __bf16 xr_bf16x2 __attribute__((ext_vector_type(2)));
typedef float xr_f32x2 __attribute__((ext_vector_type(2)));
__device__ inline uint32_t pack_bf16x2(float lo, float hi) {
    xr_f32x2 v = {lo, hi};
    union { xr_bf16x2 b; uint32_t u; } c;
    c.b = __builtin_convertvector(v, xr_bf16x2);
    return c.u;
}
#else   // the host pass only has to parse the callers
__host__ __device__ inline uint32_t pack_bf16x2(float lo, float hi) {
    return (uint32_t)f32_to_bf16(lo) | ((uint32_t)f32_to_bf16(hi) << 16);
}
#endif

// Activations of a gated feed-forward, act(gate) * up, by the code the Python side passes.
// Another activation is another code and another case below; every kernel that applies the
// gate (the products' epilogues and k_gate_mul) takes the code as an argument.
#define XR_ACT_SILU 0
#define XR_ACT_COUNT 1
#if defined(__HIP_DEVICE_COMPILE__)
// FAST: with the hardware's 2^x and reciprocal (1 ulp each)
template <bool FAST> __device__ inline float gate_act(int act, float g) {
    switch (act) {
    default:    // XR_ACT_SILU: g / (1 + exp(-g)) (src/model.c:4451-4452)
        return FAST ? g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g * -1.44269504f))
                    : g / (1.0f + expf(-g));
    }
}
#else
template <bool FAST> __host__ __device__ inline float gate_act(int, float g) { return g; }   // the host pass only parses the callers
#endif

template <typename T> __device__ inline float ld(const T* p, size_t i);
template <> __device__ inline float ld<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ inline float ld<bf16_t>(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }

template <typename T> __device__ inline void st(T* p, size_t i, float v);
template <> __device__ inline void st<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ inline void st<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

// ---- wave (64 lanes) reductions -------------------------------------------------
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Page lookup: logical position of a request -> element offset pieces.
struct PageRef {
    int page;
    int off;
};
__device__ inline PageRef page_of(const int* __restrict__ block_table, int table_stride, int req,
                                  int pos, int page_shift, int page_mask) {
    PageRef r;
    r.page = block_table[(size_t)req * table_stride + (pos >> page_shift)];
    r.off = pos & page_mask;
    return r;
}

// "Paired order" of a head's channels: where a rotation pairs channel j with j + rot/2, the
// product that makes queries and keys may have its weight rows ordered so that both lie in
// one group of 16 columns: channel j < rot/2 at column (j/8)*16 + j%8, its partner 8 further
// (rot a multiple of 16); channels from rot on stay where they are.
__host__ __device__ inline int paired_col(int d, int rot) {
    if (d >= rot) return d;
    const int half = rot >> 1, hi = d >= half ? 1 : 0, j = hi ? d - half : d;
    return (j >> 3) * 16 + hi * 8 + (j & 7);
}

static inline int ilog2_exact(int v) {   // -1 if v is not a power of two
    if (v <= 0 || (v & (v - 1))) return -1;
    int s = 0;
    while ((1 << s) < v) ++s;
    return s;
}
