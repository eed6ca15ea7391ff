// Sampling on the device: one workgroup per row of logits.
//
// temp <= 0: the first index of the maximum, logits untouched
// (src/sample.c:169-172).  temp > 0, in the reference's order
// (src/sample.c:148-166, :86-127, :302-328):
//   repeat penalty over the recent window (each occurrence counts; exempt ids skipped;
//   a positive logit is divided, another multiplied), z = logit / temp, candidates in
//   the total order "z descending, then id ascending", top-k (softmax over the k kept),
//   top-p (smallest prefix with mass >= top_p, renormalised), min-p (drop p < min_p *
//   p_best, renormalised), then the roulette walk: first candidate whose cumulative
//   mass exceeds the draw r.
// Every cut keeps a prefix of that total order, so the kernel never sorts: it finds
// each boundary by a radix selection over the 56-bit key (32 bits of z, 24 bits of id),
// counting candidates or adding their mass.  Mass is exp(z - z_max) in 40-bit fixed
// point, added with integer atomics, so the result does not depend on the order in
// which lanes arrive.
#include "common.h"
#include "no_alloc.h"

#include <mutex>

#define SM_THREADS 1024
#define SM_FIX 1099511627776.0   // 2^40

struct SampleArgs {
    int* out;
    float* logits;
    int ld, V;
    const float* temp;
    const int* top_k;
    const float* top_p;
    const float* min_p;
    const float* repeat_penalty;
    const float* draw;
    const int* recent;      // [W, recent_cap]
    const int* n_recent;    // [W]
    int recent_cap;
    const int* exempt;
    int n_exempt;
    const float* greedy_part;   // [W, GREEDY_SPLITS, 2] (value, index bits) from k_greedy_partial, or null
};

#define GREEDY_SPLITS 32

// The greedy pick's first pass for rows without temperature: a row's logits are read by
// GREEDY_SPLITS workgroups instead of one (one workgroup reads 128k logits in 60 us, bound by
// its loads' latency), each leaving the maximum of its range and the first index that has it.
__global__ __launch_bounds__(256) void k_greedy_partial(const float* logits, int ld, int V, const float* temp, float* part) {
    const int r = blockIdx.x, sp = blockIdx.y;
    if (temp[r] > 0.f) return;
    const int chunk = ((V + GREEDY_SPLITS - 1) / GREEDY_SPLITS + 3) & ~3;
    const int lo = sp * chunk, hi = lo + chunk < V ? lo + chunk : V;
    const float* row = logits + (size_t)r * ld;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
        float v = row[i];
        if (v > best || (v == best && i < bi)) { best = v; bi = i; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        float ob = __shfl_xor(best, o, 64);
        int oi = __shfl_xor(bi, o, 64);
        if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    __shared__ float sb[4];
    __shared__ int si[4];
    if ((threadIdx.x & 63) == 0) { sb[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w)
            if (sb[w] > best || (sb[w] == best && si[w] < bi)) { best = sb[w]; bi = si[w]; }
        float* p = part + ((size_t)r * GREEDY_SPLITS + sp) * 2;
        p[0] = best;
        p[1] = __int_as_float(bi);
    }
}

__device__ inline uint32_t order_key32(float z) {
    if (z != z) return 0xFFFFFFFFu;          // NaN sorts last
    if (z == 0.f) z = 0.f;                   // -0 and +0 are one value
    uint32_t u = __float_as_uint(z);
    u = (u >> 31) ? ~u : (u | 0x80000000u);  // ascending with z
    return ~u;                               // ascending key = descending z
}

__device__ inline unsigned long long order_key(float z, int id) {
    return ((unsigned long long)order_key32(z) << 24) | (unsigned long long)(uint32_t)id;
}

struct RowView {
    const float* row;
    int V;
    float inv_t;      // candidates carry logit / temp
    float temp;
    float zmax;
    unsigned long long limit;   // keep key <= limit
    float min_e;                // keep exp(z - zmax) >= min_e
};

__device__ inline bool row_item(const RowView& rv, int i, unsigned long long& key, unsigned long long& mass) {
    float z = rv.row[i] / rv.temp;
    key = order_key(z, i);
    float e = expf(z - rv.zmax);
    if (!(e >= rv.min_e) || key > rv.limit) return false;
    mass = (unsigned long long)((double)e * SM_FIX);
    return true;
}

__device__ unsigned long long block_sum_u64(unsigned long long v, unsigned long long* sh) {
    // sh has SM_THREADS / 64 entries
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    unsigned long long t = 0;
    for (int w = 0; w < SM_THREADS / 64; ++w) t += sh[w];
    return t;
}

// Mass (by_mass) or number of the kept candidates.
__device__ unsigned long long kept_total(const RowView& rv, bool by_mass, unsigned long long* sh) {
    unsigned long long acc = 0;
    for (int i = threadIdx.x; i < rv.V; i += SM_THREADS) {
        unsigned long long key, mass;
        if (row_item(rv, i, key, mass)) acc += by_mass ? mass : 1ull;
    }
    return block_sum_u64(acc, sh);
}

// Smallest key B among the kept candidates with F(B) > target, where F(B) is the mass
// (by_mass) or the number of kept candidates with key <= B.  If no key reaches the
// target the largest kept key is returned.
__device__ unsigned long long radix_select(const RowView& rv, bool by_mass, unsigned long long target,
                                           unsigned long long* hist, unsigned long long* sh2) {
    unsigned long long prefix = 0, remaining = target;
    for (int shift = 48; shift >= 0; shift -= 8) {
        __syncthreads();
        if (threadIdx.x < 256) hist[threadIdx.x] = 0;
        __syncthreads();
        for (int i = threadIdx.x; i < rv.V; i += SM_THREADS) {
            unsigned long long key, mass;
            if (!row_item(rv, i, key, mass)) continue;
            if ((key >> (shift + 8)) != (prefix >> (shift + 8))) continue;
            unsigned long long w = by_mass ? mass : 1ull;
            if (w) atomicAdd(&hist[(key >> shift) & 255ull], w);
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            unsigned long long cum = 0;
            int sel = -1, last = -1;
            for (int d = 0; d < 256; ++d) {
                unsigned long long h = hist[d];
                if (!h) continue;
                last = d;
                if (cum + h > remaining) { sel = d; break; }
                cum += h;
            }
            if (sel < 0) {            // ran off the end: stay in the last kept bin
                sel = last < 0 ? 0 : last;
                remaining = last < 0 ? 0 : hist[sel] - 1;
            } else {
                remaining -= cum;
            }
            sh2[0] = prefix | ((unsigned long long)sel << shift);
            sh2[1] = remaining;
        }
        __syncthreads();
        prefix = sh2[0];
        remaining = sh2[1];
    }
    return prefix;
}

__global__ __launch_bounds__(SM_THREADS) void k_sample(SampleArgs a) {
    __shared__ unsigned long long hist[256];
    __shared__ unsigned long long sh[SM_THREADS / 64];
    __shared__ unsigned long long sh2[2];
    __shared__ float shf[SM_THREADS / 64];
    __shared__ int shi[SM_THREADS / 64];
    const int r = blockIdx.x;
    float* row = a.logits + (size_t)r * a.ld;
    const int V = a.V;
    const float temp = a.temp[r];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;

    if (!(temp > 0.f)) {
        // greedy: first index of the maximum, over the logits or over the ranges' results
        float best = -INFINITY;
        int bi = 0x7fffffff;
        if (a.greedy_part) {
            if (threadIdx.x < GREEDY_SPLITS) {
                const float* p = a.greedy_part + ((size_t)r * GREEDY_SPLITS + threadIdx.x) * 2;
                best = p[0];
                bi = __float_as_int(p[1]);
            }
        } else {
            for (int i = threadIdx.x; i < V; i += SM_THREADS) {
                float v = row[i];
                if (v > best || (v == best && i < bi)) { best = v; bi = i; }
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            float ob = __shfl_xor(best, o, 64);
            int oi = __shfl_xor(bi, o, 64);
            if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
        }
        if (lane == 0) { shf[wave] = best; shi[wave] = bi; }
        __syncthreads();
        if (threadIdx.x == 0) {
            for (int w = 1; w < SM_THREADS / 64; ++w)
                if (shf[w] > best || (shf[w] == best && shi[w] < bi)) { best = shf[w]; bi = shi[w]; }
            a.out[r] = bi == 0x7fffffff ? 0 : bi;
        }
        return;
    }

    // repeat penalty, in the window's order
    const float rp = a.repeat_penalty ? a.repeat_penalty[r] : 1.f;
    if (rp != 1.f && a.recent && threadIdx.x == 0) {
        const int n = a.n_recent[r];
        const int* rec = a.recent + (size_t)r * a.recent_cap;
        for (int i = 0; i < n && i < a.recent_cap; ++i) {
            int tok = rec[i];
            if (tok < 0 || tok >= V) continue;
            bool ex = false;
            for (int k = 0; k < a.n_exempt; ++k) ex = ex || (a.exempt[k] == tok);
            if (ex) continue;
            float v = row[tok];
            row[tok] = v > 0.f ? v / rp : v * rp;
        }
    }
    __syncthreads();

    // maximum of z
    float zm = -INFINITY;
    for (int i = threadIdx.x; i < V; i += SM_THREADS) {
        float z = row[i] / temp;
        if (z > zm) zm = z;
    }
    zm = wave_max(zm);
    if (lane == 0) shf[wave] = zm;
    __syncthreads();
    zm = shf[0];
    for (int w = 1; w < SM_THREADS / 64; ++w) zm = fmaxf(zm, shf[w]);

    RowView rv;
    rv.row = row; rv.V = V; rv.temp = temp; rv.inv_t = 1.f / temp; rv.zmax = zm;
    rv.limit = ~0ull; rv.min_e = 0.f;

    const int tk = a.top_k ? a.top_k[r] : 0;
    if (tk > 0 && tk < V) rv.limit = radix_select(rv, false, (unsigned long long)(tk - 1), hist, sh2);
    const float tp = a.top_p ? a.top_p[r] : 1.f;
    if (tp < 1.f) {
        unsigned long long s_k = kept_total(rv, true, sh);
        unsigned long long want = (unsigned long long)((double)(tp > 0.f ? tp : 0.f) * (double)s_k);
        rv.limit = radix_select(rv, true, want > 0 ? want - 1 : 0, hist, sh2);
    }
    const float mp = a.min_p ? a.min_p[r] : 0.f;
    if (mp > 0.f) rv.min_e = mp < 1.f ? mp : 1.f;
    unsigned long long s_keep = kept_total(rv, true, sh);
    double u = (double)a.draw[r];
    unsigned long long target = (unsigned long long)(u * (double)s_keep);
    if (s_keep > 0 && target >= s_keep) target = s_keep - 1;
    unsigned long long pick = radix_select(rv, true, target, hist, sh2);
    if (threadIdx.x == 0) a.out[r] = (int)(pick & 0xFFFFFFull);
}

static int sample_launch(int* out, float* logits, int W, int V, int ld, const float* temp, const int* top_k,
                         const float* top_p, const float* min_p, const float* repeat_penalty,
                         const float* draw, const int* recent, const int* n_recent, int recent_cap,
                         const int* exempt, int n_exempt, float* greedy_ws, hipStream_t stream) {
    XR_REQUIRE(W >= 0 && V > 0 && ld >= V, "sample: bad sizes W=%d V=%d ld=%d", W, V, ld);
    XR_REQUIRE(V <= (1 << 24), "sample: vocabulary %d exceeds 2^24", V);
    XR_REQUIRE(out && logits && temp && draw, "sample: null operand");
    XR_REQUIRE(!recent || (n_recent && recent_cap > 0), "sample: a recent window without its length");
    if (W == 0) return XR_OK;
    SampleArgs a;
    a.out = out; a.logits = logits; a.ld = ld; a.V = V; a.temp = temp; a.top_k = top_k; a.top_p = top_p;
    a.min_p = min_p; a.repeat_penalty = repeat_penalty; a.draw = draw; a.recent = recent;
    a.n_recent = n_recent; a.recent_cap = recent_cap; a.exempt = exempt; a.n_exempt = exempt ? n_exempt : 0;
    a.greedy_part = greedy_ws;
    if (greedy_ws) {        // [W, GREEDY_SPLITS, 2] floats
        k_greedy_partial<<<dim3(W, GREEDY_SPLITS), 256, 0, stream>>>(logits, ld, V, temp, greedy_ws);
        XR_CHECK_LAUNCH("greedy_partial");
    }
    k_sample<<<W, SM_THREADS, 0, stream>>>(a);
    XR_CHECK_LAUNCH("sample");
    return XR_OK;
}

extern "C" int xr_sample(int* out, float* logits, int W, int V, int ld, const float* temp, const int* top_k,
                         const float* top_p, const float* min_p, const float* repeat_penalty,
                         const float* draw, const int* recent, const int* n_recent, int recent_cap,
                         const int* exempt, int n_exempt, float* greedy_ws, hipStream_t stream) {
    return sample_launch(out, logits, W, V, ld, temp, top_k, top_p, min_p, repeat_penalty, draw, recent, n_recent,
                         recent_cap, exempt, n_exempt, greedy_ws, stream);
}

// ------------------------------------------------------------------------------ no allocation
// The same pick with the first pass's work area in an array of the library's own (no_alloc.h).
// In host code the array's name is only a handle: its device address is asked for once per
// device and kept, and the kernels get that address as they get the caller's work area above.
#define XR_MAX_DEVICES 64
static __device__ __align__(256) float scratch[(size_t)XR_SAMPLE_STATIC_MAX_ROWS * GREEDY_SPLITS * 2];
static float* scratch_ptr[XR_MAX_DEVICES];       // the array's address on each device, once resolved
static std::mutex scratch_lock;

static int scratch_on_current_device(float** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) (void)hipGetLastError();
    XR_REQUIRE(e == hipSuccess, "sample_static: no current device: %s", hipGetErrorString(e));
    XR_REQUIRE(dev >= 0 && dev < XR_MAX_DEVICES, "sample_static: device %d is beyond the %d this library keeps an address for", dev, XR_MAX_DEVICES);
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (!scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) (void)hipGetLastError();
        XR_REQUIRE(e == hipSuccess && p, "sample_static: the work area's address on device %d: %s", dev, hipGetErrorString(e));
        scratch_ptr[dev] = (float*)p;
    }
    *ptr = scratch_ptr[dev];
    return XR_OK;
}

extern "C" int xr_sample_static_init() {
    float* p = nullptr;
    return scratch_on_current_device(&p);
}

extern "C" int xr_sample_static(int* out, float* logits, int W, int V, int ld, const float* temp, const int* top_k,
                                const float* top_p, const float* min_p, const float* repeat_penalty,
                                const float* draw, const int* recent, const int* n_recent, int recent_cap,
                                const int* exempt, int n_exempt, hipStream_t stream) {
    XR_REQUIRE(W <= XR_SAMPLE_STATIC_MAX_ROWS, "sample_static: %d rows, the library's work area holds %d (use xr_sample with a work area of the caller's)",
               W, XR_SAMPLE_STATIC_MAX_ROWS);
    float* ws = nullptr;
    const int rc = scratch_on_current_device(&ws);
    if (rc != XR_OK) return rc;
    return sample_launch(out, logits, W, V, ld, temp, top_k, top_p, min_p, repeat_penalty, draw, recent, n_recent,
                         recent_cap, exempt, n_exempt, ws, stream);
}
