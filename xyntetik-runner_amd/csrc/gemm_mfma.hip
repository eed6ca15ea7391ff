// bfloat16 matrix products on the gfx950 matrix cores, 32-bit accumulation:
//   out[M,N] = a[M,K] * w[N,K]^T (+ bias)        (weights [n_out][n_in], row-major)
// Two kernels share the epilogues:
//   * k_gemm_tile_async: more than 16 rows (prompt portions, large batches).  A workgroup
//     computes a BM x BN tile; both operands are copied from memory straight into LDS in
//     64-wide K slices (16-byte chunks, XOR-swizzled so that fragment reads do not collide),
//     several slices ahead, and fed to v_mfma_f32_32x32x16_bf16.  With few tiles K is split
//     over workgroups and k_gemm_finish adds the parts in a fixed order.  Three main loops:
//     four waves with the order of their instructions written out (what serves, where K is
//     whole slices), and two with eight waves for the rest.
//   * k_gemm_skinny: M <= 16 (decoding).  The product is bound by reading the weights
//     once, so each wave streams 16 weight rows straight from memory into MFMA fragments
//     (v_mfma_f32_16x16x32_bf16, weights as the A operand, tokens as the B operand) with
//     many loads in flight, and the waves of a workgroup split K among themselves.
// Weights come row-major or packed for these kernels (k_pack_weight): blocks of 16 rows x 32
// columns, 1 KB each, in the order the lanes of a wave read them, so that one load instruction
// of a wave reads one contiguous kilobyte instead of 64 bytes from each of 16 rows.  Measured on MI355X
// at 8 rows: 101 -> 86 us for the four products of a layer of the 8B shape.
// Epilogues: store (float or bfloat16), add into a float output (the residual stream),
// and SwiGLU: with w = [gate rows; up rows] the kernel writes silu(gate) * up, so the
// [M, 2F] intermediate never reaches memory (src/model.c:6399-6404).
// Up to 64 rows two more things ride on a product, in the skinny kernel's epilogue (up to 16
// rows) or in the kernel that adds up a split product's K ranges: the RMSNorm that follows a
// product into the residual stream (src/model.c:3386-3392), and for the
// q/k/v product the rotation of queries and keys and the write of keys and values to their
// pages (RopeFuse), so that a decode step launches 6 kernels a layer.
// The reference's float-weight "GEMM" is a multi-column matvec (src/kernels.cu:116-144);
// its tensor-core kernels (:856) exist for quantised weights only.
#include <type_traits>

#include "common.h"
#include "async_copy.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define EPI_STORE 0
#define EPI_ACCUM 1
#define EPI_GATED 2     // w = [gate rows; up rows]: act(gate) * up, act = GemmArgs.act

// Rotation and cache write in the epilogue of the skinny kernel (on: q_out not null).  The
// product's columns are [query heads | key heads | value heads], each head D wide; what would
// be its output row is rotated and stored like k_rope_kv_write does, and nothing else is
// written.  With pairs (j, j + rot/2) the weight rows must be in paired order (see
// paired_col in common.h), so that both halves of a pair lie in one group of 16 columns.
struct RopeFuse {
    const int* positions;      // [M]
    const int* req_of_token;   // [M]
    const int* block_table;    // [requests, table_stride]
    int table_stride;
    const float* inv_freq;     // [rot/2] or null
    int H, Hk, D, rot, interleaved;
    float mscale;
    int page_shift, page_mask, page_size;
    bf16_t* q_out;             // [M, H*D]
    bf16_t* k_cache;
    bf16_t* v_cache;
    const float2* cs;          // [M][rot/2] (cosine, sine) of each row's angles, times mscale: set where the tile kernel rotates
};

struct GemmArgs {
    const bf16_t* a;   // [M, lda]
    const bf16_t* w;   // [N or 2N, K] row-major, or packed (see k_pack_weight)
    int w_packed;
    const float* bias; // [N] (or [2N] for SwiGLU) or null
    void* out;         // [M, ldo]
    int M, N, K, lda, ldo;
    int out_bf16;      // storage of out
    int epi;
    int act;           // the gate's activation (XR_ACT_*), with EPI_GATED
    int m_fast;        // tile order of the asynchronous kernel: 1 = consecutive workgroups share a weight tile, 2 = by XCD
    int splits;        // > 1: K is cut into this many ranges, each workgroup writes raw sums to `partial`
    int k_per_split;   // columns per range (a multiple of 64)
    float* partial;    // [splits][M][rows of w]
    int raw;           // 1: raw sums go to `partial` also when K is whole (an epilogue of k_gemm_finish is wanted)
    int norm_whole;    // 1: k_gemm_finish_norm writes the whole norm of the updated rows to xg
    int col0, col1;    // the tile kernel computes output columns col0 .. col1-1 (col0 a multiple of the tile's width)
    int vec_out;       // 1: the tile kernel may write 4 columns a lane (widths and row strides are multiples of 4, bases 16-byte aligned)
    // RMSNorm folded into the skinny kernel (all null or zero: off).
    // Before: `a` holds rows x*weight that are not yet divided by their root mean square; ss_in
    // [n_ss][16] holds partial sums of x^2 per row, and the product's row t is scaled by
    // rsqrt(sum_p ss_in[p][t] * ss_inv_width + ss_eps) (exact: the scale is one factor per row).
    const float* ss_in;
    int n_ss;
    float ss_inv_width, ss_eps;
    // After (with EPI_ACCUM): the updated output row times norm_w goes to xg [M][N], and
    // the sums of squares of columns 16p .. 16p+15 of the updated rows go to ss_out[p][16].
    const void* norm_w;
    int norm_w_bf16;
    bf16_t* xg;
    float* ss_out;
    RopeFuse rope;     // rotation and cache write in place of the output (on: rope.q_out not null)
};

// what a caller passes to have the product's row rotated and cached (see RopeFuse)
struct XrGemmRope {
    const int* positions;
    const int* req_of_token;
    const int* block_table;
    int table_stride;
    const float* inv_freq;
    int H, Hk, D, rot, interleaved;
    float mscale;
    int page_size;
    void* q_out;
    void* k_cache;
    void* v_cache;
    const void* cs_table;   // [M][rot/2] (cosine, sine) pairs made by xr_rope_table for these rows, or null: the product makes its own
};

// what a caller passes to fold a norm into a product of at most 16 rows (see GemmArgs)
struct XrGemmNorm {
    const float* ss_in;
    int n_ss;
    float ss_inv_width, ss_eps;
    const void* norm_w;
    int norm_w_bf16;
    void* xg;
    float* ss_out;
    int ss_out_rows;   // in: partial rows that ss_out has room for; out: partial rows written
};

__device__ inline uint4 ldg16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
// streaming load: the weights of a decode step are read once and must not push the
// activations out of the caches
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ inline uint4 ldg16_stream(const bf16_t* p) {
    u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ inline bf16x8 as_bf16x8(uint4 v) {
    union { uint4 u; bf16x8 b; } c;
    c.u = v;
    return c.b;
}
// zero unless ok, word by word (a select between two 16-byte objects goes through memory)
__device__ inline uint4 keep_if(bool ok, uint4 v) {
    return make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
}
__device__ inline void store_out(const GemmArgs& g, int m, int n, float v) {
    size_t o = (size_t)m * g.ldo + n;
    if (g.epi == EPI_ACCUM) {
        float* p = (float*)g.out;
        p[o] = p[o] + v;
    } else if (g.out_bf16) {
        ((bf16_t*)g.out)[o] = f32_to_bf16(v);
    } else {
        ((float*)g.out)[o] = v;
    }
}

// One element of a projection's result, column nn of row tok, to where it belongs: queries and
// keys rotated (`partner` is the value 8 columns away in paired order, or 1 with interleaved
// pairs), queries to their buffer, keys and values to their pages; formulas as in k_rope_kv_write.
__device__ inline void rope_store(const RopeFuse& rp, int tok, int nn, float val, float partner) {
    const int Q = rp.H * rp.D, KV = rp.Hk * rp.D;
    const int sec = nn < Q ? 0 : (nn < Q + KV ? 1 : 2);
    const int rel = nn - (sec == 0 ? 0 : (sec == 1 ? Q : Q + KV));
    const int hs = rel / rp.D, c = rel - hs * rp.D;
    const int pos = rp.positions[tok];
    int d = c;
    float o = val;
    if (sec < 2 && c < rp.rot) {
        int j, hi;
        if (rp.interleaved) { j = c >> 1; hi = c & 1; }
        else { hi = (c >> 3) & 1; j = (c >> 4) * 8 + (c & 7); d = j + hi * (rp.rot >> 1); }
        const float ang = (float)pos * rp.inv_freq[j];
        const float cs = cosf(ang) * rp.mscale, sn = sinf(ang) * rp.mscale;
        const float x0 = hi ? partner : val, x1 = hi ? val : partner;
        o = hi ? x0 * sn + x1 * cs : x0 * cs - x1 * sn;
    }
    if (sec == 0) {
        rp.q_out[((size_t)tok * rp.H + hs) * rp.D + d] = f32_to_bf16(o);
        return;
    }
    const PageRef pr = page_of(rp.block_table, rp.table_stride, rp.req_of_token[tok], pos, rp.page_shift, rp.page_mask);
    if (sec == 1)
        rp.k_cache[(((size_t)pr.page * rp.Hk + hs) * rp.page_size + pr.off) * rp.D + d] = f32_to_bf16(o);
    else
        rp.v_cache[(((size_t)pr.page * rp.Hk + hs) * rp.D + d) * rp.page_size + pr.off] = f32_to_bf16(o);
}

// NT side-by-side 32x32 tiles in the accumulator layout of v_mfma_f32_32x32x16 (a lane holds one
// column and 16 rows) go to rows m_base.., columns col_base.. of a row-major matrix through the
// wave's own LDS area, so that a lane then holds 4 consecutive columns of one row: a store
// instruction writes whole 128-byte runs instead of 2 or 4 bytes a lane.  (Measured on a
// 256x256 tile with bfloat16 output: 21 us of a tile's 137 us went to 128 two-byte stores a
// lane and their addresses.)  mode: 0 store float, 1 add into float, 2 store bfloat16.
// A wave's LDS accesses are served in order, so it needs no barrier for an area of its own.
constexpr int STAGE_FLOATS = 32 * (64 + 4);      // a wave's area: 32 rows of 64 columns, rows 16 bytes apart in the banks
// What write_tiles will add to (mode 1), fetched ahead: a lane's 4 floats of each of its 4 NT rows.
// The stores of one tile and the loads of the next may be the same memory for all the compiler
// knows, so loads left inside write_tiles wait for each store before them, one trip to memory
// after the other (measured: the down product of 2,048 rows 240 us against 194 without adding).
template <int NT>
__device__ inline void load_old(float4 (&old)[4 * NT], const void* dst, int ld, int m_base, int M, int col_base, int col_end, int lane) {
    constexpr int CPR = 8 * NT, RPI = 64 / CPR;
    const int ch = lane % CPR, col = col_base + ch * 4;
    const float* const dst32 = (const float*)dst + ((size_t)m_base * ld + col_base);
    const uint32_t lane_off = (uint32_t)((lane / CPR) * ld + ch * 4);
#pragma unroll
    for (int it = 0; it < 4 * NT; ++it) {
        const int m = m_base + it * RPI + lane / CPR;
        old[it] = (m < M && col < col_end) ? *reinterpret_cast<const float4*>(dst32 + lane_off + (uint32_t)(it * RPI * ld)) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
}

template <int NT>
__device__ inline void write_tiles(float* stage, const f32x16 (&t)[NT], void* dst, int ld, int mode,
                                   int m_base, int M, int col_base, int col_end, int lane, const float4* old = nullptr) {
    constexpr int SW = 32 * NT, LD = SW + 4, CPR = SW / 4, RPI = 64 / CPR;
    const int lr = lane & 31, lg = lane >> 5;
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int e = 0; e < 16; ++e) stage[((e / 4) * 8 + lg * 4 + (e % 4)) * LD + n * 32 + lr] = t[n][e];
    // one address for the tile's corner, which all lanes share, and a 32-bit offset per lane from it
    const int ch = lane % CPR, col = col_base + ch * 4;
    const size_t corner = (size_t)m_base * ld + col_base;
    bf16_t* const dst16 = (bf16_t*)dst + corner;
    float* const dst32 = (float*)dst + corner;
    const uint32_t lane_off = (uint32_t)((lane / CPR) * ld + ch * 4);
#pragma unroll
    for (int it = 0; it < 32 / RPI; ++it) {
        const int row = it * RPI + lane / CPR, m = m_base + row;
        const float4 x = *reinterpret_cast<const float4*>(stage + row * LD + ch * 4);
        if (m >= M || col >= col_end) continue;
        const uint32_t o = lane_off + (uint32_t)(it * RPI * ld);
        if (mode == 2) {
            uint2 v;
            v.x = pack_bf16x2(x.x, x.y);
            v.y = pack_bf16x2(x.z, x.w);
            *reinterpret_cast<uint2*>(dst16 + o) = v;
        } else {
            float4* q = reinterpret_cast<float4*>(dst32 + o);
            float4 y = x;
            if (mode == 1) { const float4 o4 = old ? old[it] : *q; y.x += o4.x; y.y += o4.y; y.z += o4.z; y.w += o4.w; }
            *q = y;
        }
    }
    __builtin_amdgcn_sched_barrier(0);               // (tile by tile: no tile's addresses wait in registers for another's stores)
}

// The cosines and sines a product of many rows needs to rotate its own result, once for all
// its tiles: the same formulas as rope_store (src/model.c:3514-3532).
__global__ __launch_bounds__(256) void k_rope_table(float2* cs, const int* positions, const float* inv_freq,
                                                    int M, int half, float mscale) {
    const int q = blockIdx.x * 256 + threadIdx.x;
    if (q >= M * half) return;
    const int m = q / half, j = q - m * half;
    const float ang = (float)positions[m] * inv_freq[j];
    cs[q] = make_float2(cosf(ang) * mscale, sinf(ang) * mscale);
}

// The tile kernel's way of doing what rope_store does: NT side-by-side 32x32 accumulator tiles
// of the [query heads | key heads | value heads] product go through the wave's LDS area, and a
// lane then has 4 consecutive columns of a row and, 8 columns away (paired order) or beside
// them (interleaved pairs), their partners.  Queries and keys leave rotated, 4 channels a
// store; values, cached transposed, leave 8 positions of a channel at a time where the rows
// bring an aligned group of 8 positions of one request, else one by one.
template <int NT>
__device__ inline void rope_tiles(float* stage, const f32x16 (&t)[NT], const RopeFuse& rp,
                                  int m_base, int M, int col_base, int N, int lane) {
    constexpr int SW = 32 * NT, LD = SW + 4, CPR = SW / 4, RPI = 64 / CPR;
    const int lr = lane & 31, lg = lane >> 5;
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int e = 0; e < 16; ++e) stage[((e / 4) * 8 + lg * 4 + (e % 4)) * LD + n * 32 + lr] = t[n][e];
    const int Q = rp.H * rp.D, KV = rp.Hk * rp.D, half = rp.rot >> 1;
    // values: the tiles hold columns of one section only where sections begin at multiples of 32 * NT;
    // so every (8 rows, column) or (row, 4 columns) item asks for its own section
    const int ch = lane % CPR, col = col_base + ch * 4;
    if (col < Q + KV && col < N) {
        const int sec = col < Q ? 0 : 1;
        const int rel = col - (sec ? Q : 0);
        const int hs = rel / rp.D, c = rel - hs * rp.D;
        constexpr int ITS = 32 / RPI;
        const int hi = (c >> 3) & 1, j0 = (c >> 4) * 8 + (c & 7);           // (paired order)
        // what the rows' stores need from memory first (cosines and sines, the keys' places), then
        // the arithmetic and the stores, four rows of the lane at a time (all eight are more
        // registers than the eight-wave 256x256 kernel has): a load behind a store waits for that
        // store, since they may be the same memory for all the compiler knows, and one trip to
        // memory after the other was most of this function's time
        constexpr int HB = ITS < 4 ? ITS : 4;
        static_assert(ITS % HB == 0, "the lane's rows come in fours");
#pragma unroll
        for (int it0 = 0; it0 < ITS; it0 += HB) {
        float2 f[HB][4];
        size_t kdst[HB];
#pragma unroll
        for (int it = it0; it < it0 + HB; ++it) {
            const int m = m_base + it * RPI + lane / CPR;
            if (m >= M) continue;
            if (c < rp.rot) {
                const float2* cs = rp.cs + (size_t)m * half;
                if (rp.interleaved) {
#pragma unroll
                    for (int e = 0; e < 4; e += 2)
                        if (c + e < rp.rot) f[it - it0][e] = cs[(c + e) >> 1];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) f[it - it0][e] = cs[j0 + e];
                }
            }
            if (sec == 1) {
                const PageRef pr = page_of(rp.block_table, rp.table_stride, rp.req_of_token[m], rp.positions[m], rp.page_shift, rp.page_mask);
                kdst[it - it0] = (((size_t)pr.page * rp.Hk + hs) * rp.page_size + pr.off) * rp.D;
            }
        }
#pragma unroll
        for (int it = it0; it < it0 + HB; ++it) {
            const int row = it * RPI + lane / CPR, m = m_base + row;
            if (m >= M) continue;
            const float4 x = *reinterpret_cast<const float4*>(stage + row * LD + ch * 4);
            float o[4] = {x.x, x.y, x.z, x.w};
            int d0 = c;
            if (c < rp.rot) {
                if (rp.interleaved) {
#pragma unroll
                    for (int e = 0; e < 4; e += 2)
                        if (c + e < rp.rot) {
                            const float x0 = o[e], x1 = o[e + 1];
                            o[e] = x0 * f[it - it0][e].x - x1 * f[it - it0][e].y;
                            o[e + 1] = x0 * f[it - it0][e].y + x1 * f[it - it0][e].x;
                        }
                } else {
                    const float4 y = *reinterpret_cast<const float4*>(stage + row * LD + (ch ^ 2) * 4);
                    const float pv[4] = {y.x, y.y, y.z, y.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float x0 = hi ? pv[e] : o[e], x1 = hi ? o[e] : pv[e];
                        o[e] = hi ? x0 * f[it - it0][e].y + x1 * f[it - it0][e].x : x0 * f[it - it0][e].x - x1 * f[it - it0][e].y;
                    }
                    d0 = j0 + hi * half;
                }
            }
            const uint2 w = make_uint2(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]));
            if (sec == 0) *reinterpret_cast<uint2*>(rp.q_out + ((size_t)m * rp.H + hs) * rp.D + d0) = w;
            else *reinterpret_cast<uint2*>(rp.k_cache + kdst[it - it0] + d0) = w;
        }
        }
    }
    if (col_base + SW > Q + KV && KV > 0) {
        // value columns: items are (group of 8 rows, column)
        for (int q = lane; q < 4 * SW; q += 64) {
            const int grp = q / SW, cc = q - grp * SW, vcol = col_base + cc;
            const int m8 = m_base + grp * 8;
            if (vcol < Q + KV || vcol >= N || m8 >= M) continue;
            const int rel = vcol - Q - KV, hs = rel / rp.D, d = rel - hs * rp.D;
            const int pos = rp.positions[m8], req = rp.req_of_token[m8];
            const bool whole = rp.page_size >= 8 && (pos & 7) == 0 && m8 + 7 < M && rp.req_of_token[m8 + 7] == req &&
                               rp.positions[m8 + 7] == pos + 7;
            if (whole) {
                const PageRef pr = page_of(rp.block_table, rp.table_stride, req, pos, rp.page_shift, rp.page_mask);
                float v[8];
#pragma unroll
                for (int r = 0; r < 8; ++r) v[r] = stage[(grp * 8 + r) * LD + cc];
                *reinterpret_cast<uint4*>(rp.v_cache + (((size_t)pr.page * rp.Hk + hs) * rp.D + d) * rp.page_size + pr.off) =
                    make_uint4(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7]));
            } else {
                for (int r = 0; r < 8 && m8 + r < M; ++r) {
                    const int p = rp.positions[m8 + r];
                    const PageRef pr = page_of(rp.block_table, rp.table_stride, rp.req_of_token[m8 + r], p, rp.page_shift, rp.page_mask);
                    rp.v_cache[(((size_t)pr.page * rp.Hk + hs) * rp.D + d) * rp.page_size + pr.off] = f32_to_bf16(stage[(grp * 8 + r) * LD + cc]);
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------ tile kernel
// Row r (0..BN-1) of the weight tile of workgroup bx -> row of w.  Plain: n0 + r.  SwiGLU:
// each wave's 32-column MFMA tiles alternate gate, up, gate, up ... so that the two values
// of one output column meet in the same lane and register.
template <int BN, int WN>
__device__ inline int w_row_of(int r, int bx, int N, int epi, int& out_col) {
    if (epi != EPI_GATED) {
        out_col = bx * BN + r;
        return out_col;
    }
    const int wn = r / WN, t = (r % WN) / 32, c = r % 32;
    out_col = bx * (BN / 2) + (wn * (WN / 64) + t / 2) * 32 + c;
    return (t & 1) ? N + out_col : out_col;
}

// WARPS_M x WARPS_N waves share a BM x BN tile; a wave owns (BM/WARPS_M) x (BN/WARPS_N) of it
// as 32x32 MFMA tiles.  The operands are copied from memory straight into LDS
// (global_load_lds_dwordx4: every lane names a 16-byte source, the wave's 64 pieces land
// side by side in LDS) with STAGES K-slices in flight: while the matrix cores work on slice
// kt, slices kt+1 .. kt+STAGES-1 are on their way, with no registers and no LDS-write
// instructions spent on them.  A lane whose piece lies outside the matrices reads from a
// block of zeros instead, so every slice issues the same number of loads and one counter
// wait (vmcnt) tells when a slice has landed.  Three main loops (PIPE): in the plain one (0) a
// k-step reads its fragments and multiplies; in the second (1) the fragments of k-step ks+1 (also
// the next slice's first) are read into a second set of registers before the products of k-step ks
// are issued; the third (2) is the second with the order of its instructions written out, slot by
// slot, for waves that have a SIMD to themselves (described where it stands).
// Measured on MI355X (8192 x 28672 x 4096, random data): a compute unit is given its operands
// at up to 50 bytes a cycle from L2 and reads LDS at 190, the matrix cores alone do 1.8 PFLOP/s
// (the clock falls from 2.4 to 1.8-2.0 GHz under them); a 256x256 tile spent 115 us in its loop
// and 21 us storing its result two bytes a lane, with nothing else on its compute unit to hide
// that (128 KB of LDS: one workgroup at a time).  So results leave through LDS, 4 columns a lane
// (write_tiles: 21 -> 6 us, 1.0 -> 1.14 PFLOP/s), and PIPE gives another 3-5% on all tiles but
// 256x192.
// Where chunk c of row r lies within the row in LDS: at c ^ swz(r).  A fragment read takes
// one column of 32 rows; LDS serves 16 lanes of 16 bytes a cycle from 64 banks of 4 bytes, so
// 16 consecutive rows must fall into 16 different 16-byte bank groups.  Two rows of 128 bytes
// (8 chunks) fill the banks, so the shift counts pairs of rows.  (The counter of LDS bank
// conflicts reads zero with this, and half the active cycles with a shift by the row number.)
// (Rows of 64 bytes, 4 chunks: four rows fill the banks, and the shift counts fours of rows.)
template <int CH> __device__ inline int swz(int r) {
    static_assert(CH == 8 || CH == 4, "rows of 8 or of 4 chunks");
    return CH == 8 ? (r >> 1) & 7 : (r >> 2) & 3;
}

// f(integral_constant<int, I>) for I = FROM .. TO-1, each call with its index a constant
template <int FROM, int TO, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (FROM < TO) {
        f(std::integral_constant<int, FROM>{});
        static_for<FROM + 1, TO>(f);
    }
}

// waits until at most `slices` slices of LOADS copies each are still on their way (a number the
// unrolled loops around the call make a constant)
template <int LOADS> __device__ inline void wait_slices(int slices) {
    static_assert(LOADS * 3 < 64, "the counter holds 6 bits");
    if (slices <= 0) wait_vmcnt<0>();
    else if (slices == 1) wait_vmcnt<LOADS>();
    else if (slices == 2) wait_vmcnt<LOADS * 2>();
    else wait_vmcnt<LOADS * 3>();
}

template <int BM, int BN, int WARPS_M, int WARPS_N, int STAGES, int PIPE = 0, int BK = 64>
__device__ __forceinline__ void gemm_tile(const GemmArgs& g, const int item, uint4* lds) {
    constexpr int WAVES = WARPS_M * WARPS_N;
    constexpr int CH = BK / 8, RPL = 64 / CH;           // chunks of a row; rows that one load instruction covers
    constexpr int KS = BK / 16;                         // k-steps of a slice
    static_assert(BK == 64 || BK == 32, "slices of 64 or of 32 columns");
    constexpr int WM = BM / WARPS_M, WN = BN / WARPS_N;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int ROWS = BM + BN;                       // rows of one stage: activations, then weights
    constexpr int LOADS = ROWS / RPL / WAVES;           // load instructions per wave and stage
    static_assert(ROWS % (RPL * WAVES) == 0, "stage does not divide among waves");
    static_assert(LOADS * STAGES < 64, "too many loads in flight for the counter");
    constexpr int BUF = ROWS * CH;                      // chunks per stage
                                                        // lds: [STAGES][BUF]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // (the same in all lanes: what follows from it stays in scalar registers)
    const int wm0 = (wave / WARPS_N) * WM, wn0 = (wave % WARPS_N) * WN;
    // Workgroups are numbered along M first (m_fast) or along N first.  Consecutive
    // workgroups go to different XCDs, so with 8 row tiles each XCD keeps one activation tile
    // in its L2 while the weight tile of the moment is fetched once from memory for all.
    const int tiles_m = (g.M + BM - 1) / BM;
    constexpr int BN_OUT_S = BN / 2;
    const int bn_out = g.epi == EPI_GATED ? BN_OUT_S : BN;
    const int tiles_n = (g.col1 - g.col0 + bn_out - 1) / bn_out;
    const int tile_ = __builtin_amdgcn_readfirstlane(item / g.splits), split_ = __builtin_amdgcn_readfirstlane(item % g.splits);
    // (the divisions are done in vector registers; their results go back to scalar ones)
    // m_fast 2 (at most 8 row tiles): workgroup i runs on XCD i % 8, and each XCD takes every 8th
    // column tile with all its row tiles, row tiles first, so a weight tile is fetched from memory by
    // one XCD alone, and the XCD's 32 workgroups of a moment share 4 weight tiles and the activation
    // tiles in its L2.  (Where the column tiles are no multiple of 8 the launch has workgroups for 8
    // equal shares, and those of a share's missing column leave at once.)  (Measured on the 8B shape's prompt
    // step of 2,048 rows against m_fast 1: 29.4 -> 27.9 ms.  With 32 row tiles, in groups of 8 x 4
    // tiles an XCD, it lost: 8192 x 28672 x 4096 in 1,776 us against 1,456.)
    int bm_v, bn_v;
    if (g.m_fast == 2) {
        const int l = tile_ >> 3;
        bm_v = l % tiles_m;
        bn_v = (l / tiles_m) * 8 + (tile_ & 7);
        if (bn_v >= tiles_n) return;
    } else {
        bm_v = g.m_fast ? tile_ % tiles_m : tile_ / tiles_n;
        bn_v = g.m_fast ? tile_ / tiles_m : tile_ % tiles_n;
    }
    const int bm_ = __builtin_amdgcn_readfirstlane(bm_v);
    const int bx = __builtin_amdgcn_readfirstlane(g.col0 / bn_out + bn_v);
    const int k_begin = split_ * g.k_per_split;
    const int k_end = (k_begin + g.k_per_split) < g.K ? (k_begin + g.k_per_split) : g.K;
    const int m0 = bm_ * BM;
    const int n_rows = g.epi == EPI_GATED ? 2 * g.N : g.N;
    const bf16_t* zero_src = reinterpret_cast<const bf16_t*>(xr_zero_chunk);

    // The pieces this lane fetches for every stage: where each begins (or a block of zeros, for
    // a row that does not exist) and how far on the same piece of the next slice lies.  Every
    // slice is copied once and in order, so the pointers simply move on; only a slice that is
    // not whole (the last, if K is no multiple of 64, and the empty ones after it that keep the
    // count of copies in flight the same) looks at columns, lane by lane.
    const bf16_t* src[LOADS];
    int src_step[LOADS];                                          // elements from slice to slice; 0: the row does not exist
    const size_t kblocks = (size_t)((g.K + 31) / 32);
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int row = (i * WAVES + wave) * RPL + lane / CH;     // row of the stage
        const int c = (lane % CH) ^ swz<CH>(row);                 // the chunk that belongs in this LDS place
        const bf16_t* p = nullptr;
        int step = BK;
        if (row < BM) {
            const int m = m0 + row;
            if (m < g.M) p = g.a + (size_t)m * g.lda + c * 8;
        } else {
            int oc;
            const int n = w_row_of<BN, WN>(row - BM, bx, g.N, g.epi, oc);
            const bool ok = oc < g.N && n < n_rows;
            if (g.w_packed) {
                // row n % 16 of group n / 16; a slice of 64 columns is 2 blocks, chunk c the
                // (c % 4)-th of its row in block c / 4; a slice further on is 2 blocks = 1024 elements on,
                // so one copy instruction of a wave (8 rows) reads two runs of 512 bytes (a slice of 32
                // columns is one block, and a copy instruction reads all 1024 bytes of it)
                if (ok) p = g.w + (size_t)(n >> 4) * kblocks * 512 + (c >> 2) * 512 + (n & 15) * 32 + (c & 3) * 8;
                step = BK * 16;
            } else if (ok) {
                p = g.w + (size_t)n * g.K + c * 8;
            }
        }
        src_step[i] = p ? step : 0;
        src[i] = p ? p + (size_t)k_begin * (step / BK) : zero_src;
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds;
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane(lds_base + (uint32_t)(wave * 64 * 16));
    const int nk_whole = (k_end - k_begin) / BK;                  // slices that lie within the range entirely
// the copies PART, PART + PARTS, .. of slice KT: spread over the k-steps of the slice before, so
// that no wave has to push a whole slice into the memory pipeline at once
#define ASYNC_ISSUE_PART(KT, PART, PARTS)                                                            \
    {                                                                                                \
        const uint32_t dst_ = lds_wave + (uint32_t)(((KT) % STAGES) * BUF * 16);                     \
        if ((KT) < nk_whole) {                                                                       \
            _Pragma("unroll") for (int i = (PART); i < LOADS; i += (PARTS)) {                        \
                lds_dma16(src[i], dst_ + i * WAVES * 64 * 16);                                       \
                src[i] += src_step[i];                                                               \
            }                                                                                        \
        } else {                                                                                     \
            const int k0_ = k_begin + (KT) * BK;                                                     \
            _Pragma("unroll") for (int i = (PART); i < LOADS; i += (PARTS)) {                        \
                const int c_ = ((lane % CH) ^ swz<CH>((i * WAVES + wave) * RPL + lane / CH)) * 8;    \
                const bf16_t* p_ = (src_step[i] && k0_ + c_ < k_end) ? src[i] : zero_src;            \
                lds_dma16(p_, dst_ + i * WAVES * 64 * 16);                                           \
                src[i] += src_step[i];                                                               \
            }                                                                                        \
        }                                                                                            \
    }
#define ASYNC_ISSUE(KT) ASYNC_ISSUE_PART(KT, 0, 1)

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const int nk = (k_end - k_begin + BK - 1) / BK;
    const int lr = lane & 31, lg = lane >> 5;
    if constexpr (PIPE == 2) {
        // The order of instructions is written out: a k-step is TM*TN slots, each one product
        // followed by at most Q other instructions (a fragment read for the next k-step, a copy of
        // a later slice), and nothing moves from slot to slot.  Every slice is whole here (the
        // host sees to it), rows that do not exist are read from a row that does (their results
        // are never stored), so a copy is a base that all lanes share, which moves on from slice
        // to slice in scalar registers, and a fixed offset per lane.
        constexpr int LA = BM / (RPL * WAVES);                    // the first LA copies of a slice bring activations
        static_assert(BM % (RPL * WAVES) == 0 && LA < LOADS, "a copy instruction would straddle the operands");
        static_assert(KS % 2 == 0, "the two sets of fragments alternate");
        constexpr int SLOTS = TM * TN, READS = TM + TN;
        // copies issued in one k-step: one every other slot, or what brings a slice's copies out in KS-1 k-steps
        constexpr int DPK = SLOTS / 2 > (LOADS + KS - 2) / (KS - 1) ? SLOTS / 2 : (LOADS + KS - 2) / (KS - 1);
        constexpr int DOFF = SLOTS / DPK > 1 ? SLOTS / DPK - 1 : 0;               // (copies in the slots between the reads)
        constexpr int DSTEPS = (LOADS + DPK - 1) / DPK;           // k-steps that issue a slice's copies
        static_assert(DSTEPS <= KS, "a slice's copies must be out before the next barrier");
        uint32_t off[LOADS];
        int oc0;
        const int n_base = w_row_of<BN, WN>(0, bx, g.N, g.epi, oc0);
#pragma unroll
        for (int i = 0; i < LOADS; ++i) {
            const int row = (i * WAVES + wave) * RPL + lane / CH;
            const int c = (lane % CH) ^ swz<CH>(row);
            if (i < LA) {
                const int m = m0 + row < g.M ? row : g.M - 1 - m0;
                off[i] = (uint32_t)(m * g.lda + c * 8) * 2u;
            } else {
                int oc;
                int n = w_row_of<BN, WN>(row - BM, bx, g.N, g.epi, oc);
                if (!(oc < g.N && n < n_rows)) n = n_base;
                off[i] = g.w_packed ? (uint32_t)(((n >> 4) - (n_base >> 4)) * (int)kblocks * 512 + (c >> 2) * 512 + (n & 15) * 32 + (c & 3) * 8) * 2u
                                    : (uint32_t)((n - n_base) * g.K + c * 8) * 2u;
            }
        }
        const bf16_t* a_nxt = g.a + (size_t)m0 * g.lda + k_begin;
        const bf16_t* w_nxt = g.w_packed ? g.w + (size_t)(n_base >> 4) * kblocks * 512 + (size_t)k_begin * 16
                                         : g.w + (size_t)n_base * g.K + k_begin;
        const int w_step = g.w_packed ? BK * 16 : BK;
        bf16x8 af[2][TM], wf[2][TN];
#define LONE_COPY(DI, DST)                                                                           \
    lds_dma16_base((DI) < LA ? a_nxt : w_nxt, off[DI], lds_wave + (uint32_t)((DST) * BUF * 16 + (DI) * WAVES * 64 * 16));
// one k-step: the products of fragment set F; if RD, the reads of k-step RD_KS of the slice in
// buffer RD_BUF into the other set; if PART >= 0, copies PART*DPK .. of the next slice into buffer DST
#define LONE_KSTEP(F, RD, RD_BUF, RD_KS, PART, DST)                                                  \
    {                                                                                                \
        const uint4* A_ = lds + (RD_BUF) * BUF;                                                      \
        const uint4* W_ = A_ + BM * CH;                                                              \
        const int c_ = (RD_KS) * 2 + lg;                                                             \
        _Pragma("unroll") for (int t = 0; t < SLOTS; ++t) {                                          \
            acc[t / TN][t % TN] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[F][t / TN], wf[F][t % TN], acc[t / TN][t % TN], 0, 0, 0); \
            _Pragma("unroll") for (int q = 0; q < READS; ++q) {             /* read q in slot q SLOTS / READS */ \
                if ((RD) && q * SLOTS / READS == t) {                                                \
                    if (q < TM) {                                                                    \
                        const int r = wm0 + q * 32 + lr;                                             \
                        af[(F) ^ 1][q] = as_bf16x8(A_[r * CH + (c_ ^ swz<CH>(r))]);                  \
                    } else {                                                                         \
                        const int r = wn0 + (q - TM) * 32 + lr;                                      \
                        wf[(F) ^ 1][q - TM] = as_bf16x8(W_[r * CH + (c_ ^ swz<CH>(r))]);             \
                    }                                                                                \
                }                                                                                    \
            }                                                                                        \
            _Pragma("unroll") for (int d = 0; d < DPK; ++d) {               /* copy d in slot d SLOTS / DPK (+ DOFF) */ \
                if ((PART) >= 0 && d * SLOTS / DPK + DOFF == t) {                                    \
                    const int di = (PART) * DPK + d;                                                 \
                    if (di < LOADS) LONE_COPY(di, DST)                                               \
                }                                                                                    \
            }                                                                                        \
            __builtin_amdgcn_sched_barrier(0);                                                       \
        }                                                                                            \
        if ((PART) == DSTEPS - 1) { a_nxt += BK; w_nxt += w_step; }                                                 \
    }
// the last k-step of the slice in buffer SB, behind the barrier that frees this buffer and
// certifies the next slice, and the other k-steps of the slice after it
#define LONE_ROUND(SB, SBN, COPY, WAITN)                                                             \
    {                                                                                                \
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");                                           \
        wait_slices<LOADS>(WAITN);                                                                   \
        __builtin_amdgcn_s_barrier();                                                                \
        __builtin_amdgcn_sched_barrier(0);                                                           \
        LONE_KSTEP((KS - 1) & 1, true, SBN, 0, (COPY) ? 0 : -1, SB)                                  \
        _Pragma("unroll") for (int ks = 0; ks < KS - 1; ++ks)                                        \
            LONE_KSTEP(ks & 1, true, SBN, ks + 1, (COPY) && ks + 1 < DSTEPS ? ks + 1 : -1, SB)       \
    }
#pragma unroll
        for (int st = 0; st < STAGES; ++st) {
#pragma unroll
            for (int i = 0; i < LOADS; ++i) LONE_COPY(i, st)
            a_nxt += BK;
            w_nxt += w_step;
        }
        wait_vmcnt<LOADS * (STAGES - 1)>();              // slice 0 has landed
        __builtin_amdgcn_s_barrier();
        {
            const uint4* A_ = lds;
            const uint4* W_ = A_ + BM * CH;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int r = wm0 + i * 32 + lr;
                af[0][i] = as_bf16x8(A_[r * CH + (lg ^ swz<CH>(r))]);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int r = wn0 + j * 32 + lr;
                wf[0][j] = as_bf16x8(W_[r * CH + (lg ^ swz<CH>(r))]);
            }
        }
#pragma unroll
        for (int ks = 0; ks < KS - 1; ++ks) LONE_KSTEP(ks & 1, true, 0, ks + 1, -1, 0)
        int sb = 0;                                      // the buffer of slice s
        for (int s_ = 0; s_ < nk - STAGES; ++s_) {
            const int sbn = sb + 1 == STAGES ? 0 : sb + 1;
            LONE_ROUND(sb, sbn, true, STAGES - 2)
            sb = sbn;
        }
#pragma unroll
        for (int r_ = 0; r_ < STAGES - 1; ++r_) {        // the slices after which nothing is copied
            const int sbn = sb + 1 == STAGES ? 0 : sb + 1;
            LONE_ROUND(sb, sbn, false, STAGES - 2 - r_)
            sb = sbn;
        }
        LONE_KSTEP((KS - 1) & 1, false, 0, 0, -1, 0)
#undef LONE_ROUND
#undef LONE_KSTEP
#undef LONE_COPY
    } else if constexpr (PIPE == 1) {
        // The fragments of k-step ks+1 are read into a second set of registers before the
        // products of k-step ks are issued, also across the edge of a slice.  A buffer is free
        // for the slice STAGES further on as soon as every wave has left its slice (the barrier
        // in the last k-step), and the copies begin right there: a third at once, a third in
        // each of the next two k-steps, so that the last of them are two k-steps old when waited for.
#pragma unroll
        for (int st = 0; st < STAGES; ++st) ASYNC_ISSUE(st)
        wait_vmcnt<LOADS * (STAGES - 1)>();              // slice 0 has landed
        __builtin_amdgcn_s_barrier();
        bf16x8 af[2][TM], wf[2][TN];
#define READ_FRAGS(BUFI, KS, F)                                                                      \
    {                                                                                                \
        const uint4* A_ = lds + (BUFI) * BUF;                                                        \
        const uint4* W_ = A_ + BM * CH;                                                              \
        const int c_ = (KS) * 2 + lg;                                                                \
        _Pragma("unroll") for (int i = 0; i < TM; ++i) {                                             \
            const int r = wm0 + i * 32 + lr;                                                         \
            af[F][i] = as_bf16x8(A_[r * CH + (c_ ^ swz<CH>(r))]);                                    \
        }                                                                                            \
        _Pragma("unroll") for (int j = 0; j < TN; ++j) {                                             \
            const int r = wn0 + j * 32 + lr;                                                         \
            wf[F][j] = as_bf16x8(W_[r * CH + (c_ ^ swz<CH>(r))]);                                    \
        }                                                                                            \
    }
        READ_FRAGS(0, 0, 0)
        constexpr int PARTS = KS > 2 ? 3 : KS;
        for (int kt = 0; kt < nk; ++kt) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if (ks < KS - 1) {
                    if (ks < PARTS - 1 && kt > 0) ASYNC_ISSUE_PART(kt + STAGES - 1, ks + 1, PARTS)
                    READ_FRAGS(kt % STAGES, ks + 1, (ks + 1) & 1)
                } else {
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // this wave no longer reads slice kt ...
                    wait_vmcnt<LOADS * (STAGES - 2)>();                  // ... and its share of slice kt+1 has landed
                    __builtin_amdgcn_s_barrier();
                    ASYNC_ISSUE_PART(kt + STAGES, 0, PARTS)              // into the buffer of slice kt
                    READ_FRAGS((kt + 1) % STAGES, 0, 0)
                }
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[ks & 1][i], wf[ks & 1][j], acc[i][j], 0, 0, 0);
            }
        }
#undef READ_FRAGS
    } else {
#pragma unroll
    for (int st = 0; st < STAGES - 1; ++st) ASYNC_ISSUE(st)
    for (int kt = 0; kt < nk; ++kt) {
        // slice kt has landed when at most the STAGES-2 younger slices are still in flight
        wait_vmcnt<LOADS * (STAGES - 2)>();
        __builtin_amdgcn_s_barrier();                    // for every wave; and slice kt-1 is no longer read
        const uint4* A = lds + (kt % STAGES) * BUF;
        const uint4* W = A + BM * CH;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            // a quarter of the copies of slice kt+STAGES-1, into the buffer that slice kt-1 used
            // (zeros past the end)
            ASYNC_ISSUE_PART(kt + STAGES - 1, ks, BK / 16)
            bf16x8 af[TM], wf[TN];
            const int c = ks * 2 + lg;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int r = wm0 + i * 32 + lr;
                af[i] = as_bf16x8(A[r * CH + (c ^ swz<CH>(r))]);
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int r = wn0 + j * 32 + lr;
                wf[j] = as_bf16x8(W[r * CH + (c ^ swz<CH>(r))]);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
        }
    }
    }
#undef ASYNC_ISSUE
#undef ASYNC_ISSUE_PART
    wait_vmcnt<0>();                                     // the trailing loads of zeros
    // What the write-out derives from the lane's number is computed here, from a copy the compiler
    // cannot trace back: values kept in registers through the loop were spilled, and a reload
    // between the stores waits for every store before it (one counter for loads and stores).
    int lane_after = lane;
    asm volatile("" : "+v"(lane_after));
    {
    const int lane = lane_after, lr = lane & 31, lg = lane >> 5;

    // where 4 columns a lane may be written, the results go through LDS, each wave through an area
    // of its own, once no wave reads operands there any more
    static_assert((size_t)STAGES * ROWS * CH * 16 >= (size_t)WAVES * STAGE_FLOATS * 4, "no room for the waves' output areas");
    float* stage = reinterpret_cast<float*>(lds) + wave * STAGE_FLOATS;
    constexpr int NTP = TN % 2 == 0 ? 2 : 1;             // tiles written together
    const bool rotate = g.rope.cs != nullptr;
    if (g.vec_out || rotate) __builtin_amdgcn_s_barrier();

    if (g.splits > 1 || g.raw) {
        // raw sums of this K range, by weight row: the epilogue belongs to k_gemm_finish
        const int ldp = g.epi == EPI_GATED ? 2 * g.N : g.N;
        float* part = g.partial + (size_t)split_ * g.M * ldp;
        if (g.vec_out && g.epi != EPI_GATED) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; j += NTP) {
                    f32x16 t[NTP];
#pragma unroll
                    for (int n = 0; n < NTP; ++n) t[n] = acc[i][j + n];
                    write_tiles<NTP>(stage, t, part, ldp, 0, m0 + wm0 + i * 32, g.M, bx * BN + wn0 + j * 32, g.N, lane);
                }
            return;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                int oc;
                const int n = w_row_of<BN, WN>(wn0 + j * 32 + lr, bx, g.N, g.epi, oc);
                if (oc >= g.N || n >= ldp) continue;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    int m = m0 + wm0 + i * 32 + (e / 4) * 8 + lg * 4 + (e % 4);
                    if (m < g.M) part[(size_t)m * ldp + n] = acc[i][j][e];
                }
            }
        return;
    }
    if (g.epi == EPI_GATED) {
        if (g.vec_out) {
            constexpr int TO = TN / 2, NTO = TO % 2 == 0 && TO > 0 ? 2 : 1;     // output tiles of a wave's row, and how many go together
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int jo = 0; jo < TO; jo += NTO) {
                    f32x16 t[NTO];
                    int oc0 = 0;
#pragma unroll
                    for (int n = 0; n < NTO; ++n) {
                        int oc;
                        w_row_of<BN, WN>(wn0 + (jo + n) * 64 + lr, bx, g.N, g.epi, oc);
                        if (n == 0) oc0 = oc - lr;
                        const bool in = oc < g.N;
                        const float bg = g.bias && in ? g.bias[oc] : 0.f, bu = g.bias && in ? g.bias[g.N + oc] : 0.f;
#pragma unroll
                        for (int e = 0; e < 16; ++e)
                            t[n][e] = gate_act<true>(g.act, acc[i][(jo + n) * 2][e] + bg) * (acc[i][(jo + n) * 2 + 1][e] + bu);
                    }
                    write_tiles<NTO>(stage, t, g.out, g.ldo, g.out_bf16 ? 2 : 0, m0 + wm0 + i * 32, g.M, oc0, g.N, lane);
                }
            return;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j + 1 < TN; j += 2) {
                int oc;
                w_row_of<BN, WN>(wn0 + j * 32 + lr, bx, g.N, g.epi, oc);
                if (oc >= g.N) continue;
                float bg = g.bias ? g.bias[oc] : 0.f, bu = g.bias ? g.bias[g.N + oc] : 0.f;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    int m = m0 + wm0 + i * 32 + (e / 4) * 8 + lg * 4 + (e % 4);
                    if (m < g.M) store_out(g, m, oc, gate_act<true>(g.act, acc[i][j][e] + bg) * (acc[i][j + 1][e] + bu));
                }
            }
        return;
    }
    if (g.vec_out || rotate) {
        // (tile by tile through a recursion of templates: a loop that the compiler declines to unroll,
        // as it does one with 16 rotations in it, would index the accumulators at run time, and
        // they would live in memory)
        const bool adding = !rotate && g.epi == EPI_ACCUM;
        float4 old[2][4 * NTP];                     // what the tiles of this round and of the next are added to
        if (adding) load_old<NTP>(old[0], g.out, g.ldo, m0 + wm0, g.M, bx * BN + wn0, g.N, lane);
        static_for<0, TM * (TN / NTP)>([&](auto idx) {
            constexpr int i = decltype(idx)::value / (TN / NTP), j = decltype(idx)::value % (TN / NTP) * NTP;
            constexpr int nxt = decltype(idx)::value + 1, ni = nxt / (TN / NTP), nj = nxt % (TN / NTP) * NTP;
            if (adding && nxt < TM * (TN / NTP))
                load_old<NTP>(old[nxt & 1], g.out, g.ldo, m0 + wm0 + ni * 32, g.M, bx * BN + wn0 + nj * 32, g.N, lane);
            f32x16 t[NTP];
#pragma unroll
            for (int n = 0; n < NTP; ++n) {
                const int col = bx * BN + wn0 + (j + n) * 32 + lr;
                const float b = g.bias && col < g.N ? g.bias[col] : 0.f;
#pragma unroll
                for (int e = 0; e < 16; ++e) t[n][e] = acc[i][j + n][e] + b;
            }
            if (rotate)
                rope_tiles<NTP>(stage, t, g.rope, m0 + wm0 + i * 32, g.M, bx * BN + wn0 + j * 32, g.N, lane);
            else
                write_tiles<NTP>(stage, t, g.out, g.ldo, g.epi == EPI_ACCUM ? 1 : (g.out_bf16 ? 2 : 0),
                                 m0 + wm0 + i * 32, g.M, bx * BN + wn0 + j * 32, g.N, lane, adding ? old[decltype(idx)::value & 1] : nullptr);
        });
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            int n = bx * BN + wn0 + j * 32 + lr;
            if (n >= g.N) continue;
            float b = g.bias ? g.bias[n] : 0.f;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                int m = m0 + wm0 + i * 32 + (e / 4) * 8 + lg * 4 + (e % 4);
                if (m < g.M) store_out(g, m, n, acc[i][j][e] + b);
            }
        }
    }
}

// One workgroup a tile and K range.  (Workgroups that stay and take every 256th tile were measured
// too, with the tiles assigned in turn or taken from a counter: no faster, and what the compiler then
// keeps in registers from tile to tile it spills.)
template <int BM, int BN, int WARPS_M, int WARPS_N, int STAGES, int PIPE = 0, int BK = 64>
__global__ __launch_bounds__(64 * WARPS_M * WARPS_N) void k_gemm_tile_async(GemmArgs g) {
    extern __shared__ uint4 lds[];
    gemm_tile<BM, BN, WARPS_M, WARPS_N, STAGES, PIPE, BK>(g, (int)blockIdx.x, lds);
}

// Sums the K ranges of a split product in a fixed order and applies the epilogue.
__global__ __launch_bounds__(256) void k_gemm_finish(GemmArgs g) {
    const int ldp = g.epi == EPI_GATED ? 2 * g.N : g.N;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const bool ok = idx < (size_t)g.M * g.N;
    if (!ok && !g.rope.q_out) return;
    const int m = ok ? (int)(idx / g.N) : 0, n = ok ? (int)(idx % g.N) : 0;
    const size_t step = (size_t)g.M * ldp;
    const float* p = g.partial + (size_t)m * ldp + n;
    float v = 0.f, u = 0.f;
    // eight ranges at a time, all their loads on their way before the first is added (one load
    // and one wait a range cost a memory latency each: 8 us for the 8 ranges of a small product);
    // the order of the sum is the ranges' order as before
    for (int s0 = 0; s0 < g.splits; s0 += 8) {
        float part[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) part[i] = s0 + i < g.splits ? p[(size_t)(s0 + i) * step] : 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) v += part[i];
    }
    if (g.rope.q_out) {
        // (N is a multiple of 16 here, so the 16 columns of a group are 16 lanes side by side)
        const float val = v + (g.bias ? g.bias[n] : 0.f);
        const float partner = __shfl_xor(val, g.rope.interleaved ? 1 : 8);
        if (ok) rope_store(g.rope, m, n, val, partner);
    } else if (g.epi == EPI_GATED) {
        for (int s0 = 0; s0 < g.splits; s0 += 8) {
            float part[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) part[i] = s0 + i < g.splits ? p[(size_t)(s0 + i) * step + g.N] : 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) u += part[i];
        }
        const float bg = g.bias ? g.bias[n] : 0.f, bu = g.bias ? g.bias[g.N + n] : 0.f;
        store_out(g, m, n, gate_act<false>(g.act, v + bg) * (u + bu));
    } else {
        store_out(g, m, n, v + (g.bias ? g.bias[n] : 0.f));
    }
}

// The same for a product that adds into the 32-bit residual stream and is followed by an
// RMSNorm: a workgroup takes a whole row, so it can also sum the squares of the updated row
// (threads, then waves, in a fixed order) and write the normed row, times the norm's weight,
// to xg.  N is a multiple of 4.
__global__ __launch_bounds__(1024) void k_gemm_finish_norm(GemmArgs g) {
    __shared__ float wave_sq[16];
    __shared__ float rstd_s;
    const int m = blockIdx.x, tid = threadIdx.x;
    const size_t step = (size_t)g.M * g.N;
    float* xrow = (float*)g.out + (size_t)m * g.ldo;
    float sq = 0.f;
    for (int n = tid * 4; n < g.N; n += 1024 * 4) {
        const float* p = g.partial + (size_t)m * g.N + n;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int s0 = 0; s0 < g.splits; s0 += 8) {          // eight ranges' loads on their way at a time, summed in order
            float4 part[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                part[i] = s0 + i < g.splits ? *reinterpret_cast<const float4*>(p + (size_t)(s0 + i) * step) : make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int i = 0; i < 8; ++i) { v.x += part[i].x; v.y += part[i].y; v.z += part[i].z; v.w += part[i].w; }
        }
        if (g.bias) { v.x += g.bias[n]; v.y += g.bias[n + 1]; v.z += g.bias[n + 2]; v.w += g.bias[n + 3]; }
        float4 x = *reinterpret_cast<const float4*>(xrow + n);
        x.x += v.x; x.y += v.y; x.z += v.z; x.w += v.w;
        *reinterpret_cast<float4*>(xrow + n) = x;
        sq += x.x * x.x + x.y * x.y + x.z * x.z + x.w * x.w;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
    if ((tid & 63) == 0) wave_sq[tid >> 6] = sq;
    __syncthreads();
    if (tid == 0) {
        float t = 0.f;
        for (int w = 0; w < 16; ++w) t += wave_sq[w];
        rstd_s = rsqrtf(t * g.ss_inv_width + g.ss_eps);
    }
    __syncthreads();
    const float rstd = rstd_s;
    for (int n = tid * 4; n < g.N; n += 1024 * 4) {
        const float4 x = *reinterpret_cast<const float4*>(xrow + n);     // what this thread wrote above
        float w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = g.norm_w_bf16 ? bf16_to_f32(((const bf16_t*)g.norm_w)[n + i]) : ((const float*)g.norm_w)[n + i];
        uint2 o;
        o.x = pack_bf16x2(x.x * rstd * w[0], x.y * rstd * w[1]);
        o.y = pack_bf16x2(x.z * rstd * w[2], x.w * rstd * w[3]);
        *reinterpret_cast<uint2*>(g.xg + (size_t)m * g.N + n) = o;
    }
}

// (what a launcher answers when its kernel does not take the product and another one must)
#define XR_NOT_TAKEN -1000

template <int BM, int BN, int WM_, int WN_, int ST, int PIPE = 0, int BK = 64>
static int launch_tile_async(GemmArgs g, hipStream_t stream) {
    if (g.epi == EPI_GATED && (BN / WN_ / 32) % 2) {
        xr_set_error("gemm: a %dx%d tile cannot pair gate and up columns", BM, BN);
        return XR_BAD_ARG;
    }
    size_t smem = (size_t)ST * (BM + BN) * (BK / 8) * 16;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)k_gemm_tile_async<BM, BN, WM_, WN_, ST, PIPE, BK>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) {
            (void)hipGetLastError();             // or the next launch's check would report this refusal
            xr_set_error("gemm: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
            return XR_LAUNCH;
        }
        attr_set = true;
    }
    int n_out_tile = g.epi == EPI_GATED ? BN / 2 : BN;
    if (g.col1 <= 0 || g.col1 > g.N) g.col1 = g.N;
    if (g.col0 < 0 || g.col0 % n_out_tile || g.col0 >= g.col1 || (g.col1 < g.N && g.col1 % n_out_tile)) {
        xr_set_error("gemm: columns %d..%d do not start at a %d-column tile", g.col0, g.col1, n_out_tile);
        return XR_BAD_ARG;
    }
    unsigned tiles_n = (unsigned)((g.col1 - g.col0 + n_out_tile - 1) / n_out_tile), tiles_m = (unsigned)((g.M + BM - 1) / BM);
    unsigned tiles = tiles_n * tiles_m;
    if (g.m_fast == 2 && (tiles_m > 8 || tiles_n < 8)) g.m_fast = 1;
    if (g.m_fast == 2) tiles = 8 * tiles_m * ((tiles_n + 7) / 8);
    if (g.splits < 1 || !g.partial || g.col0 > 0 || g.col1 < g.N) g.splits = 1;
    if (g.splits > 1) {
        int slices = (g.K + 63) / 64;
        int per = (slices + g.splits - 1) / g.splits;
        g.k_per_split = per * 64;
        g.splits = (slices + per - 1) / per;            // no empty range
    }
    if (g.splits == 1) g.k_per_split = ((g.K + 63) / 64) * 64;
    if (PIPE == 2) {
        // the loop with its instructions in a written order: whole slices only, at least ST of them
        // in every K range, and every lane's piece within 4 GB of the tile's first
        const int last = g.K - (g.splits - 1) * g.k_per_split;
        const size_t span = (size_t)(g.epi == EPI_GATED ? g.N + BN : BN) + 16;
        if (g.K % BK || last < ST * BK || g.k_per_split < ST * BK || (size_t)BM * g.lda * 2 >= (1ull << 32) ||
            span * (size_t)(((g.K + 31) / 32) * 32) * 2 >= (1ull << 32)) {
            return XR_NOT_TAKEN;
        }
    }
    if (g.raw && (!g.partial || g.col0 > 0 || g.col1 < g.N)) {
        xr_set_error("gemm: no room for the raw sums of a product whose epilogue is a kernel of its own");
        return XR_BAD_ARG;
    }
    {
        // 4 columns a lane: every row of the output (and of the raw sums) must begin 16 bytes aligned
        const bool raw_out = g.splits > 1 || g.raw;
        const int ld = raw_out ? (g.epi == EPI_GATED ? 2 * g.N : g.N) : g.ldo;
        const void* base = raw_out ? (const void*)g.partial : (const void*)g.out;
        g.vec_out = g.N % 4 == 0 && ld % 4 == 0 && ((uintptr_t)base % 16) == 0 && (!raw_out || ((size_t)g.M * ld) % 4 == 0);
    }
    k_gemm_tile_async<BM, BN, WM_, WN_, ST, PIPE, BK><<<tiles * g.splits, 64 * WM_ * WN_, smem, stream>>>(g);
    XR_CHECK_LAUNCH("gemm_tile_async");
    if (g.norm_whole) {
        k_gemm_finish_norm<<<(unsigned)g.M, 1024, 0, stream>>>(g);
        XR_CHECK_LAUNCH("gemm_finish_norm");
    } else if (g.splits > 1 || g.raw) {
        size_t n = (size_t)g.M * g.N;
        k_gemm_finish<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(g);
        XR_CHECK_LAUNCH("gemm_finish");
    }
    return XR_OK;
}

// ------------------------------------------------------------------------------ skinny kernel
// MT: 16-token groups (M <= 16*MT).  RT: groups of 16 weight rows per wave.  KSW: waves per
// workgroup; they split K into contiguous slices, so a workgroup owns 16*RT output columns
// and all of K, and no sum crosses workgroups.  A wave issues the weight loads (16 bytes a
// lane, straight into MFMA A fragments) and the activation loads (B fragments, served by
// L2) of U k-steps of 32 before it uses them; with N/(16*RT) workgroups of KSW waves this
// keeps tens of kilobytes in flight on every compute unit.  The slices are summed through
// LDS in a fixed order.
template <int MT, int RT, int KSW, int U, bool SWIGLU, bool NT>
__global__ __launch_bounds__(64 * KSW) void k_gemm_skinny(GemmArgs g) {
    constexpr int NWT = SWIGLU ? 2 : 1;  // weight fragments per row group (gate and up)
    constexpr int MTOK = MT * 16, ROWS = RT * 16, THREADS = 64 * KSW;
    extern __shared__ float red[];       // [KSW][NWT][ROWS][MTOK]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, lq = lane >> 4;
    const int n_base = blockIdx.x * ROWS;
    const int steps_total = (g.K + 31) / 32;
    const int steps_per = (steps_total + KSW - 1) / KSW;
    const int kbeg = wave * steps_per * 32;
    const int kend_ = kbeg + steps_per * 32;
    const int kend = kend_ < g.K ? kend_ : g.K;

    // Row-major: the lane reads row l16 of its group at column 8 * lq of the k-step.  Packed:
    // the wave reads the k-step's block of its group, the lane its 16 bytes of it.
    const size_t kblocks = (size_t)((g.K + 31) / 32);
    const int step_stride = g.w_packed ? 512 : 32;
    const int lane_off = g.w_packed ? (l16 * 4 + lq) * 8 : lq * 8;
    const int dead_off = g.w_packed ? (l16 * 4 + lq) * 8 : 0;      // where a lane whose column does not exist reads
    const bf16_t* wp[NWT][RT];
    bool w_ok[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        int n = n_base + r * 16 + l16;
        w_ok[r] = n < g.N;
        if (g.w_packed) {
            const int n0 = n_base + r * 16;
            const size_t grp = (size_t)(n0 < g.N ? n0 / 16 : 0);
            wp[0][r] = g.w + grp * kblocks * 512;
            if (SWIGLU) wp[NWT - 1][r] = g.w + ((size_t)(g.N / 16) + grp) * kblocks * 512;
        } else {
            wp[0][r] = g.w + (size_t)(w_ok[r] ? n : 0) * g.K;
            if (SWIGLU) wp[NWT - 1][r] = g.w + (size_t)(g.N + (w_ok[r] ? n : 0)) * g.K;
        }
    }
    const bf16_t* ap[MT];
    bool a_ok[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        int tok = i * 16 + l16;
        a_ok[i] = tok < g.M;
        ap[i] = g.a + (size_t)(a_ok[i] ? tok : 0) * g.lda;
    }

    f32x4 acc[NWT][RT][MT];
#pragma unroll
    for (int t = 0; t < NWT; ++t)
#pragma unroll
        for (int r = 0; r < RT; ++r)
#pragma unroll
            for (int i = 0; i < MT; ++i) acc[t][r][i] = f32x4{0.f, 0.f, 0.f, 0.f};

    // the first SS_AHEAD partial sums of squares of a folded norm are copied to LDS meanwhile
    // (no registers are held for them; a wave's copy moves 16 partial rows)
    constexpr int SS_AHEAD = 256;
    float* scale_s = red + KSW * NWT * ROWS * MTOK;       // [16 parts][16 rows]
    float* ss_s = scale_s + 256;                          // [SS_AHEAD][16 rows]
    if (g.ss_in) {
        const int chunks = (g.n_ss < SS_AHEAD ? g.n_ss : SS_AHEAD) * 4;      // pieces of 16 bytes
        const uint32_t ss_lds = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)ss_s;
        for (int c0 = wave * 64; c0 < chunks; c0 += THREADS) {
            const int c = c0 + lane;
            const void* src = c < chunks ? (const void*)((const char*)g.ss_in + (size_t)c * 16) : (const void*)xr_zero_chunk;
            lds_dma16(src, __builtin_amdgcn_readfirstlane(ss_lds + (uint32_t)c0 * 16));
        }
    }

    const uint4 zero = make_uint4(0, 0, 0, 0);
    for (int k0 = kbeg; k0 < kend; k0 += 32 * U) {
        uint4 wreg[U][NWT][RT], areg[U][MT];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = k0 + u * 32 + lq * 8;
            const bool k_ok = k < kend;
            const int ks = k_ok ? k : 0;             // a column that exists; the value is dropped
            const size_t wo = k_ok ? (size_t)((k0 >> 5) + u) * step_stride + lane_off : (size_t)dead_off;
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int t = 0; t < NWT; ++t)
                    wreg[u][t][r] = keep_if(k_ok && w_ok[r], NT ? ldg16_stream(wp[t][r] + wo) : ldg16(wp[t][r] + wo));
#pragma unroll
            for (int i = 0; i < MT; ++i) areg[u][i] = keep_if(k_ok && a_ok[i], ldg16(ap[i] + ks));
        }
        __builtin_amdgcn_sched_barrier(0);      // every load of the batch is issued before the first use
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const bf16x8 af = as_bf16x8(areg[u][i]);
#pragma unroll
                for (int r = 0; r < RT; ++r)
#pragma unroll
                    for (int t = 0; t < NWT; ++t)
                        acc[t][r][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(wreg[u][t][r]), af,
                                                                                acc[t][r][i], 0, 0, 0);
            }
    }

    // acc[t][r][i][e]: weight row r*16 + 4*(lane/16) + e of the workgroup's ROWS, token i*16 + lane%16
#pragma unroll
    for (int t = 0; t < NWT; ++t)
#pragma unroll
        for (int r = 0; r < RT; ++r)
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    red[((wave * NWT + t) * ROWS + r * 16 + lq * 4 + e) * MTOK + i * 16 + l16] = acc[t][r][i][e];
    // the rows' scales, from the partial sums the producer of `a` left: thread (part, tok) of the
    // first 256 sums every 16th partial, each thread of the last loop sums the 16 parts of its
    // row; the order is the same in every instance of this kernel, so a row's scale does not
    // depend on the batch
    if (g.ss_in) {
        wait_vmcnt<0>();
        __syncthreads();                                  // every wave's copies have landed
        if (tid < 256) {
            float s = 0.f;
            const int n_lds = g.n_ss < SS_AHEAD ? g.n_ss : SS_AHEAD;
            for (int p = tid >> 4; p < n_lds; p += 16) s += ss_s[p * 16 + (tid & 15)];
            for (int p = (tid >> 4) + SS_AHEAD; p < g.n_ss; p += 16) s += g.ss_in[p * 16 + (tid & 15)];
            scale_s[tid] = s;
        }
    }
    __syncthreads();
    for (int q = tid; q < ROWS * MTOK; q += THREADS) {
        int col = q % ROWS, tok = q / ROWS;          // consecutive threads write consecutive columns
        int nn = n_base + col;
        const bool ok = tok < g.M && nn < g.N;
        float v[NWT];
#pragma unroll
        for (int t = 0; t < NWT; ++t) {
            float s = 0.f;
#pragma unroll
            for (int k = 0; k < KSW; ++k) s += red[((k * NWT + t) * ROWS + col) * MTOK + tok];
            v[t] = s;
        }
        if (g.ss_in) {
            float ss = 0.f;
#pragma unroll
            for (int p = 0; p < 16; ++p) ss += scale_s[p * 16 + (tok & 15)];
            const float scale = rsqrtf(ss * g.ss_inv_width + g.ss_eps);
#pragma unroll
            for (int t = 0; t < NWT; ++t) v[t] *= scale;
        }
        if (SWIGLU) {
            if (ok) {
                float bg = g.bias ? g.bias[nn] : 0.f, bu = g.bias ? g.bias[g.N + nn] : 0.f;
                store_out(g, tok, nn, gate_act<false>(g.act, v[0] + bg) * (v[NWT - 1] + bu));
            }
        } else if (g.rope.q_out) {
            // rotated and cached (the partner of a pair is 8 lanes away, or 1)
            const float val = v[0] + (ok && g.bias ? g.bias[nn] : 0.f);
            const float partner = __shfl_xor(val, g.rope.interleaved ? 1 : 8);
            if (ok) rope_store(g.rope, tok, nn, val, partner);
        } else if (g.xg) {
            // the rows of the residual stream after this product, their weighted copy for the next
            // product, and the sums of their squares over each 16 columns (16 lanes side by side)
            float xn = 0.f;
            if (ok) {
                float* p = (float*)g.out + (size_t)tok * g.ldo + nn;
                xn = *p + v[0] + (g.bias ? g.bias[nn] : 0.f);
                *p = xn;
                float nw = g.norm_w_bf16 ? bf16_to_f32(((const bf16_t*)g.norm_w)[nn]) : ((const float*)g.norm_w)[nn];
                g.xg[(size_t)tok * g.N + nn] = f32_to_bf16(xn * nw);
            }
            float sq = xn * xn;
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o);
            const int part = blockIdx.x * RT + (col >> 4);
            if ((col & 15) == 0 && tok < 16 && part * 16 < g.N) g.ss_out[part * 16 + tok] = sq;
        } else if (ok) {
            store_out(g, tok, nn, v[0] + (g.bias ? g.bias[nn] : 0.f));
        }
    }
}

static int launch_tile_variant(int variant, const GemmArgs& g, hipStream_t stream) {
    // (the loop that reads its fragments a k-step ahead is the faster one but for the 256x192 tile)
    // Two kernels for the 256x256 and the 256x128 tile: four waves, one a SIMD, each with a quarter of
    // the tile and the order of its instructions written out (PIPE 2), where the product allows it
    // (whole slices of K, enough of them, no rotation), else eight waves and the loop that reads its
    // fragments a k-step ahead.  Measured at 2,048 rows (us, eight waves / four): gate+up 489 / 419,
    // the down product 221 / 194, the output product 69 / 61; 8192 x 28672 x 4096: 1,611 / 1,417.
    // (A product that rotates its result keeps the eight waves unless the four are asked for by name:
    // the rotation is work for the vector units, where four waves with 16 tiles each took 128 us for the
    // q/k/v product of 2,048 rows against 115 in 256x192 tiles with eight.)
    if ((variant == 12 && !g.rope.cs) || variant == 55) {
        const int rc = launch_tile_async<256, 128, 2, 2, 3, 2, 64>(g, stream);
        if (rc != XR_NOT_TAKEN) return rc;
    }
    if (variant == 12) return launch_tile_async<256, 128, 4, 2, 3, 1>(g, stream);
    if ((variant == 14 && !g.rope.cs) || variant == 51) {
        const int rc = launch_tile_async<256, 256, 2, 2, 2, 2, 64>(g, stream);
        if (rc != XR_NOT_TAKEN) return rc;
    }
    if (variant == 14) return launch_tile_async<256, 256, 4, 2, 2, 1>(g, stream);
    if (variant == 112) return launch_tile_async<256, 128, 4, 2, 3, 1>(g, stream);     // (the eight-wave kernels by name, for tests)
    if (variant == 114) return launch_tile_async<256, 256, 4, 2, 2, 1>(g, stream);
    // (four slices in flight: with 65 to 512 rows these products are bound by how fast the weights
    // arrive, and two slices, one of them in use, left a compute unit 32 KB on its way: the down
    // product at 128 rows 46 -> 37 us, gate+up 72 -> 57, q/k/v at 512 rows 65 -> 45)
    // (the written order also where the weights' arrival bounds the kernel: little, 1-2%)
    if ((variant == 17 && !g.rope.cs) || variant == 58) {
        const int rc = launch_tile_async<128, 128, 2, 2, 4, 2, 64>(g, stream);
        if (rc != XR_NOT_TAKEN) return rc;
    }
    if (variant == 17 || variant == 117) return launch_tile_async<128, 128, 2, 2, 4, false>(g, stream);
    if (variant == 51 || variant == 55 || variant == 58) {
        xr_set_error("gemm: the four-wave kernel does not take K %d in %d ranges, lda %d, or a rotation", g.K, g.splits, g.lda);
        return XR_BAD_ARG;
    }
    // (the 256x192 tile with four waves and the rotation, 12 tiles a wave: 27.0 ms for the prompt step
    // of 2,048 rows against 26.8 with eight)
    if (variant == 26) return launch_tile_async<256, 192, 4, 2, 2>(g, stream);
    xr_set_error("gemm: unknown variant %d", variant);
    return XR_BAD_ARG;
}

// returns the number of workgroups, or an error (< 0)
static inline int rc_of(int launched) { return launched < 0 ? launched : XR_OK; }

template <int MT, int RT, int KSW, int U, bool SW, bool NT = false>
static int launch_skinny(const GemmArgs& g, hipStream_t stream) {
    constexpr int NWT = SW ? 2 : 1;
    size_t smem = (size_t)KSW * NWT * RT * 16 * MT * 16 * 4 + 256 * 4 + 256 * 64;    // the sums of the waves, 256 partial scales, 256 rows of partial sums
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)k_gemm_skinny<MT, RT, KSW, U, SW, NT>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) {
            (void)hipGetLastError();             // or the next launch's check would report this refusal
            xr_set_error("gemm: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
            return XR_LAUNCH;
        }
        attr_set = true;
    }
    unsigned blocks = (unsigned)((g.N + 16 * RT - 1) / (16 * RT));
    k_gemm_skinny<MT, RT, KSW, U, SW, NT><<<blocks, 64 * KSW, smem, stream>>>(g);
    XR_CHECK_LAUNCH("gemm_skinny");
    return (int)blocks;
}

// ------------------------------------------------------------------------------ packing
// dst [ceil(N/16)][ceil(K/32)][16 rows][32 columns] from src [N, K] row-major (K a multiple
// of 8): a block is what one v_mfma_f32_16x16x32_bf16 takes as its weight operand, 1 KB that a
// wave reads with one load (lane 16 c + r the 16 bytes of row r, columns 8c .. 8c+7).  Rows
// and columns that do not exist are zeros.  A thread moves one 16-byte chunk.  (Measured: rows
// within a block rather than chunks within a block serve both kernels best.)
__global__ __launch_bounds__(256) void k_pack_weight(bf16_t* dst, const bf16_t* src, int N, int K, size_t chunks) {
    const size_t q = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= chunks) return;
    const size_t kblocks = (size_t)((K + 31) / 32);
    const int c = (int)(q & 3), r = (int)((q >> 2) & 15);
    const size_t blk = q >> 6, grp = blk / kblocks, kb = blk - grp * kblocks;
    const size_t n = grp * 16 + r, k = kb * 32 + c * 8;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (n < (size_t)N && k < (size_t)K) v = *reinterpret_cast<const uint4*>(src + n * K + k);
    *reinterpret_cast<uint4*>(dst + q * 8) = v;
}

extern "C" int xr_pack_weight(void* dst, const void* src, int N, int K, hipStream_t stream) {
    XR_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "pack_weight: %d x %d: the width must be a multiple of 8", N, K);
    XR_REQUIRE(((uintptr_t)dst % 16) == 0 && ((uintptr_t)src % 16) == 0, "pack_weight: buffers must be 16-byte aligned");
    const size_t chunks = (size_t)((N + 15) / 16) * ((K + 31) / 32) * 64;
    k_pack_weight<<<(unsigned)((chunks + 255) / 256), 256, 0, stream>>>((bf16_t*)dst, (const bf16_t*)src, N, K, chunks);
    XR_CHECK_LAUNCH("pack_weight");
    return XR_OK;
}

// The table of a step's rotation angles, [M][half] (cosine, sine) times mscale, that a product of
// many rows takes in XrGemmRope.cs_table: the same for every layer that rotates by the same
// frequencies, so a step makes it once.
extern "C" int xr_rope_table(void* cs, const int* positions, const float* inv_freq, int M, int half, float mscale,
                             hipStream_t stream) {
    XR_REQUIRE(cs && positions && inv_freq && M >= 0 && half > 0, "rope_table: bad operands (M=%d, half=%d)", M, half);
    XR_REQUIRE(((uintptr_t)cs % 8) == 0, "rope_table: the table must be 8-byte aligned");
    if (M == 0) return XR_OK;
    k_rope_table<<<(unsigned)(((size_t)M * half + 255) / 256), 256, 0, stream>>>((float2*)cs, positions, inv_freq, M, half, mscale);
    XR_CHECK_LAUNCH("rope_table");
    return XR_OK;
}

// From this many rows on the q/k/v product has tiles enough with K whole, and its tile kernel rotates
// and caches its own result; with fewer rows the kernel that adds up its K ranges does.
#define XR_ROPE_TILE_ROWS 512
extern "C" int xr_rope_tile_rows() { return XR_ROPE_TILE_ROWS; }

// epi: 0 store, 1 add into float out, 2 gated (w has 2N rows: gate rows then up rows; act: XR_ACT_*).
// variant: 0 = choose by shape; 1 = skinny; 10..20 = tile shapes; 30, 31 = few rows with K split;
//          +1000 = row tiles of one weight tile follow each other.
// w_packed: the weights are in k_pack_weight's order.
// workspace (may be null): room for split products, workspace_bytes long; without it K is not split.
extern "C" int xr_gemm_bf16(void* out, const void* a, const void* w, const float* bias, int M, int N, int K,
                            int lda, int ldo, int out_dtype, int epi, int act, int variant, int w_packed, float* workspace,
                            size_t workspace_bytes, XrGemmNorm* norm, const XrGemmRope* rope, hipStream_t stream) {
    XR_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
    XR_REQUIRE(lda >= K && ldo >= N, "gemm: row strides lda=%d ldo=%d are shorter than K=%d N=%d", lda, ldo, K, N);
    XR_REQUIRE(K % 8 == 0 && lda % 8 == 0, "gemm: the MFMA kernels need K (%d) and the row stride (%d) to be multiples of 8", K, lda);
    XR_REQUIRE(((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm: operands must be 16-byte aligned");
    XR_REQUIRE(epi >= 0 && epi <= 2, "gemm: unknown epilogue %d", epi);
    XR_REQUIRE(epi != EPI_GATED || (act >= 0 && act < XR_ACT_COUNT), "gemm: unknown activation code %d", act);
    XR_REQUIRE(!(w_packed && epi == EPI_GATED && N % 16), "gemm: packed gate and up rows need a width that is a multiple of 16, got %d", N);
    XR_REQUIRE(epi != EPI_ACCUM || out_dtype == XR_F32, "gemm: accumulation needs a 32-bit output");
    XR_REQUIRE(out_dtype == XR_F32 || out_dtype == XR_BF16, "gemm: bad output dtype %d", out_dtype);
    if (M == 0) return XR_OK;
    GemmArgs g;
    g.a = (const bf16_t*)a; g.w = (const bf16_t*)w; g.w_packed = w_packed ? 1 : 0; g.bias = bias; g.out = out;
    g.M = M; g.N = N; g.K = K; g.lda = lda; g.ldo = ldo; g.out_bf16 = out_dtype == XR_BF16; g.epi = epi; g.act = act;
    g.m_fast = 0; g.splits = 1; g.k_per_split = 0; g.partial = workspace; g.col0 = 0; g.col1 = N;
    g.raw = 0; g.norm_whole = 0; g.vec_out = 0;
    bool want_whole_norm = false;      // a norm after a product of more than 16 rows is asked for and possible
    g.ss_in = nullptr; g.n_ss = 0; g.ss_inv_width = 0.f; g.ss_eps = 0.f;
    g.norm_w = nullptr; g.norm_w_bf16 = 0; g.xg = nullptr; g.ss_out = nullptr;
    if (norm) {
        XR_REQUIRE(variant == 0, "gemm: a norm is folded only into a product whose kernel the library chooses");
        XR_REQUIRE(M <= 16 || !norm->ss_in, "gemm: rows that lack their norm's scale: at most 16, got %d", M);
        if (norm->ss_in) {
            XR_REQUIRE(norm->n_ss > 0 && norm->ss_inv_width > 0.f, "gemm: bad partial sums of squares (%d of them)", norm->n_ss);
            g.ss_in = norm->ss_in; g.n_ss = norm->n_ss; g.ss_inv_width = norm->ss_inv_width; g.ss_eps = norm->ss_eps;
        }
        if (norm->xg) {
            XR_REQUIRE(epi == EPI_ACCUM && norm->norm_w, "gemm: the norm after a product needs the accumulating epilogue and a weight");
            XR_REQUIRE(M > 16 || (norm->ss_out && norm->ss_out_rows >= (N + 15) / 16),
                       "gemm: room for %d partial sums of squares, %d needed", norm->ss_out ? norm->ss_out_rows : 0, (N + 15) / 16);
            g.norm_w = norm->norm_w; g.norm_w_bf16 = norm->norm_w_bf16; g.xg = (bf16_t*)norm->xg; g.ss_out = norm->ss_out;
            if (M > 16) {
                // The kernel that adds up the K ranges of a split product takes whole rows and writes the
                // finished norm: always from 17 to 64 rows; above, if the product is split (else the
                // request is declined: ss_out_rows stays as it is and the caller runs the norm's kernel).
                XR_REQUIRE(norm->ss_inv_width > 0.f, "gemm: the norm's width is missing");
                want_whole_norm = N % 4 == 0 && ldo % 4 == 0 && workspace && (size_t)M * N * 4 <= workspace_bytes;
                XR_REQUIRE(want_whole_norm || M > 64, "gemm: the norm after a product of %d rows needs a width (%d) that is a multiple of 4 and a workspace", M, N);
                g.ss_inv_width = norm->ss_inv_width; g.ss_eps = norm->ss_eps;
                if (M <= 64) { g.norm_whole = 1; g.raw = 1; norm->ss_out_rows = -1; }
            }
        }
    }
    g.rope.q_out = nullptr; g.rope.cs = nullptr;
    // many rows: the tile kernel rotates and caches its own result, with the rows' cosines and
    // sines from a table that a small kernel writes into the workspace first; K is then not split
    // from XR_ROPE_TILE_ROWS rows on; below, the kernel that adds up the K ranges rotates and caches
    const bool rope_direct = rope && M >= XR_ROPE_TILE_ROWS;
    if (rope) {
        XR_REQUIRE((variant == 0 || (rope_direct && variant >= 10 && variant < 200)) && epi == EPI_STORE && !(norm && norm->xg),
                   "gemm: rotation and cache write are folded only into a plain product whose kernel the library chooses (or, with many rows, a tile kernel named)");
        if (rope_direct) {
            XR_REQUIRE(rope->cs_table || (workspace && (size_t)M * (rope->rot / 2 + 1) * sizeof(float2) <= workspace_bytes),
                       "gemm: rotation after a product of %d rows needs a workspace for its table", M);
            XR_REQUIRE(((uintptr_t)rope->q_out % 8) == 0 && ((uintptr_t)rope->k_cache % 8) == 0 && ((uintptr_t)rope->v_cache % 16) == 0,
                       "gemm: queries and caches must be 16-byte aligned");
        } else if (M > 16) {
            XR_REQUIRE(workspace && (size_t)M * N * 4 <= workspace_bytes, "gemm: rotation after a product of %d rows needs a workspace", M);
            g.raw = 1;
        }
        XR_REQUIRE(rope->H >= 0 && rope->Hk >= 0 && rope->D > 0 && rope->D % 16 == 0 && N == (rope->H + 2 * rope->Hk) * rope->D,
                   "gemm: %d columns are not %d query and 2 x %d key/value heads of a size (%d) that is a multiple of 16",
                   N, rope->H, rope->Hk, rope->D);
        XR_REQUIRE(rope->rot >= 0 && rope->rot <= rope->D && rope->rot % 2 == 0 && (rope->interleaved || rope->rot % 16 == 0),
                   "gemm: rotary width %d (head size %d): pairs (j, j + width/2) need a multiple of 16", rope->rot, rope->D);
        XR_REQUIRE(rope->rot == 0 || rope->inv_freq, "gemm: rotary width %d without a frequency table", rope->rot);
        const int shift = ilog2_exact(rope->page_size);
        XR_REQUIRE(rope->Hk == 0 || shift >= 0, "gemm: page size %d is not a power of two", rope->page_size);
        XR_REQUIRE(rope->positions && rope->q_out && (rope->Hk == 0 || (rope->k_cache && rope->v_cache && rope->block_table && rope->req_of_token)),
                   "gemm: rotation and cache write with a null operand");
        g.rope.positions = rope->positions; g.rope.req_of_token = rope->req_of_token; g.rope.block_table = rope->block_table;
        g.rope.table_stride = rope->table_stride; g.rope.inv_freq = rope->inv_freq;
        g.rope.H = rope->H; g.rope.Hk = rope->Hk; g.rope.D = rope->D; g.rope.rot = rope->rot; g.rope.interleaved = rope->interleaved;
        g.rope.mscale = rope->mscale; g.rope.page_shift = shift < 0 ? 0 : shift; g.rope.page_mask = rope->page_size - 1;
        g.rope.page_size = rope->page_size;
        g.rope.q_out = (bf16_t*)rope->q_out; g.rope.k_cache = (bf16_t*)rope->k_cache; g.rope.v_cache = (bf16_t*)rope->v_cache;
        if (rope_direct && rope->cs_table) {
            g.rope.cs = (const float2*)rope->cs_table;      // made once for the step, for every layer with this rotation
        } else if (rope_direct) {
            g.rope.cs = (const float2*)workspace;
            const int half = rope->rot / 2;
            if (half > 0) {
                k_rope_table<<<(unsigned)(((size_t)M * half + 255) / 256), 256, 0, stream>>>((float2*)workspace, rope->positions, rope->inv_freq,
                                                                                            M, half, rope->mscale);
                XR_CHECK_LAUNCH("rope_table");
            }
        }
    }
    if (variant >= 2000) { g.m_fast = 2; variant -= 2000; }
    if (variant >= 1000) { g.m_fast = 1; variant -= 1000; }
    const bool sw = epi == EPI_GATED;
    const int w_rows = epi == EPI_GATED ? 2 * N : N;
    // K ranges so that the workgroups make one round on the 256 compute units and no more
    // (measured at 32 and 64 rows: 10 ranges of 32 tiles, two rounds, took 20 us where 8 take 16),
    // if the workspace has room for their sums
    auto pick_splits = [&](int tiles) {
        if (rope_direct) return 1;
        int s = tiles >= 256 ? 1 : 256 / tiles;
        int max_s = K / 256 > 0 ? K / 256 : 1;
        s = s < 1 ? 1 : (s > max_s ? max_s : s);
        while (s > 1 && (size_t)s * M * w_rows * 4 > workspace_bytes) --s;
        return workspace ? s : 1;
    };
    if (variant == 0) {
        if (M <= 16) {
            variant = 1;
        } else if (M <= 64) {
            variant = 31;
        } else {
            // The tile that keeps the chip busiest: larger tiles do more products for a byte that
            // L1 delivers (what bounds this kernel), but their count may fill the 256 compute
            // units badly.  A tile's time is its area over its measured rate with the chip full
            // (relative to 256x256); a launch takes as many of these as its tiles make rounds of
            // 256.  When the last round of the best tile would leave most of the chip idle, the
            // columns of the full rounds go to that tile and the rest to a second launch with a
            // smaller one (3 rounds + 1 of half-size tiles instead of 4).  A tile shape whose tiles
            // are too few for the chip competes with K split among workgroups (below).
            // (The 256 compute units and the tiles' relative rates below are tuning measured on an
            // MI355X with the 8B shape's products, not limits: elsewhere they cost speed only.)
            // (rate: of the tile's products, relative to 256x256; fixed: seconds a round beside them.  At
            // 2,048 rows a round of 256x256 tiles took 107 us with K = 4,096 and 191 with 7,168, one of
            // 256x128 tiles 61 us with K = 4,096 and 194 with 14,336, one of 256x192 tiles 118.)
            struct Cand { int variant, bm, bn; double rate, fixed; };
            const double four = rope_direct ? 0.85 : 1.0;        // (the eight-wave kernels of these tiles, which a rotating product takes)
            const Cand cands[4] = {{14, 256, 256, 1.0 * four, 0.0}, {26, 256, 192, 0.73, 8e-6}, {12, 256, 128, 1.0 * four, 8e-6},
                                   {17, 128, 128, 0.63, 0.0}};
            auto width = [&](const Cand& c) { return sw ? c.bn / 2 : c.bn; };
            auto usable = [&](const Cand& c) { return !(sw && c.variant == 26); };
            auto count = [&](const Cand& c, int cols) { return ((M + c.bm - 1) / c.bm) * ((cols + width(c) - 1) / width(c)); };
            // Times in seconds: a 256x256 tile's products over K columns take 65536 K x 0.4e-12 s at
            // full rate (107 us at K = 4,096, as measured).  A launch whose tiles are too few for the
            // chip (under 160) may split K so that its workgroups make one round; the kernel that then
            // adds the ranges up moves (ranges x their width + 2 x N) x M x 4 bytes at about 4.5 TB/s
            // and costs a launch, and it writes the norm that follows, if one was asked for, which
            // saves that kernel (11 us at 2,048 x 4,096).  Measured against this model at 256 to 1,024
            // rows (us, model / measured): down at 512 rows in 256x128 tiles and 4 ranges 79 / 74-79, in
            // 128x128 and 2 ranges 90 / 94, in 256x256 and 8 ranges 80 / 79; q/k/v at 256 rows in 256x128
            // and 5 ranges 28 / 32, in 128x128 and 2 ranges 31 / 36.
            const double unit = 0.4e-12;
            auto seconds = [&](const Cand& c, int cols) {
                return (double)((count(c, cols) + 255) / 256) * ((double)c.bm * c.bn / c.rate * K * unit + c.fixed);
            };
            auto adding = [&](int ranges) {
                return ((double)ranges * w_rows + 2.0 * N) * M * 4 / 4.5e12 + 3e-6 - (want_whole_norm ? 11e-6 : 0.0);
            };
            int best = 0, best_splits = 1, second = -1, cols_first = N;
            double t_best = 1e30;
            for (int i = 0; i < 4; ++i) {
                if (!usable(cands[i])) continue;
                const int c = count(cands[i], N);
                double t = seconds(cands[i], N);
                int sp = 1;
                if (c < 160 && workspace && !rope_direct) {
                    const int s2 = pick_splits(c);
                    const double ts = (double)cands[i].bm * cands[i].bn / cands[i].rate * ((K + s2 - 1) / s2) * unit + cands[i].fixed + adding(s2);
                    if (s2 >= 2 && ts < t) { t = ts; sp = s2; }
                }
                if (t < t_best) { best = i; best_splits = sp; t_best = t; }
            }
            for (int i = 0; i < 3; ++i) {
                if (!usable(cands[i])) continue;
                const int tm = (M + cands[i].bm - 1) / cands[i].bm, full = count(cands[i], N) / 256;
                const int cols = full * 256 / tm * width(cands[i]);          // the columns of the full rounds
                if (full < 1 || count(cands[i], N) % 256 == 0 || cols <= 0 || cols >= N) continue;
                for (int j = i + 1; j < 4; ++j) {
                    if (!usable(cands[j]) || cols % width(cands[j])) continue;
                    const double t = seconds(cands[i], cols) + seconds(cands[j], N - cols);
                    if (t < 0.92 * t_best) { best = i; best_splits = 1; second = j; cols_first = cols; t_best = t; }   // (a second launch costs a little, too)
                }
            }
            variant = cands[best].variant;
            g.m_fast = 2;                      // (where the tiles' counts allow, else 1: the launcher sees to it)
            if (second >= 0) {
                GemmArgs g2 = g;
                g.col1 = cols_first;
                g2.col0 = cols_first;
                const int rc = launch_tile_variant(variant, g, stream);
                return rc != XR_OK ? rc : launch_tile_variant(cands[second].variant, g2, stream);
            }
            if (best_splits > 1) {
                g.splits = best_splits;
                // the kernel that adds the ranges up takes whole rows and writes the norm that follows
                if (want_whole_norm) { g.norm_whole = 1; norm->ss_out_rows = -1; }
            }
        }
    }
    if (variant == 1) {
        XR_REQUIRE(M <= 64, "gemm: the skinny kernel takes at most 64 rows, got %d", M);
        if (M <= 16) {
            // measured on MI355X with packed weights at M = 1, 8 and 16 (waves per workgroup, loads
            // per batch): the output head, q/k/v, the down product, the output product.  The weights
            // are read once, with loads marked as streaming: that alone gave 3-9% on every one of
            // them (the head of the 8B shape at one row: 1.05 GB in 149 us, 7.1 TB/s).
            int blocks;
            if (sw) blocks = launch_skinny<1, 1, 8, 8, true, true>(g, stream);
            else if (N >= 65536) blocks = M <= 8 ? launch_skinny<1, 1, 8, 8, false, true>(g, stream) : launch_skinny<1, 2, 4, 8, false, true>(g, stream);
            else if (N > 4096 && K <= 8192) blocks = K > 4096 ? launch_skinny<1, 1, 4, 8, false, true>(g, stream) : launch_skinny<1, 1, 4, 4, false, true>(g, stream);
            else blocks = launch_skinny<1, 1, 8, 4, false, true>(g, stream);
            if (blocks < 0) return blocks;
            if (norm) norm->ss_out_rows = (N + 15) / 16;
            return XR_OK;
        }
        if (M <= 32) return rc_of(sw ? launch_skinny<2, 1, 16, 8, true>(g, stream) : launch_skinny<2, 1, 16, 8, false>(g, stream));
        return rc_of(sw ? launch_skinny<4, 2, 8, 4, true>(g, stream) : launch_skinny<4, 2, 8, 4, false>(g, stream));
    }
    if (variant == 30 || variant == 31) {       // few rows: 32 or 64 of them against 128 weight rows, K split
        const int bn_out = sw ? 64 : 128;
        g.splits = pick_splits((N + bn_out - 1) / bn_out);
        if (variant == 30) return launch_tile_async<32, 128, 1, 2, 3>(g, stream);
        // (four slices in flight instead of three: the gate and up product 50.6 -> 47.0 us at 64 rows,
        // the others as before; five, 256 weight rows a tile, or twice the K ranges for two
        // workgroups a compute unit gain nothing or lose)
        // (with the order of instructions written out where the product allows: decode at batch 64 7.43 -> 7.31 ms)
        const int rc = launch_tile_async<64, 128, 2, 2, 4, 2, 64>(g, stream);
        return rc != XR_NOT_TAKEN ? rc : launch_tile_async<64, 128, 2, 2, 4>(g, stream);
    }
    return launch_tile_variant(variant, g, stream);
}
