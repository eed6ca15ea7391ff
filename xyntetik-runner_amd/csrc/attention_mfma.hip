// Paged grouped-query attention on the gfx950 matrix cores, bfloat16 storage, for prompt
// portions and decoded tokens in one launch.  Compiled once per head size (XR_HEAD_DIM,
// a multiple of 16 up to 256).
//
// The formulas are the reference's (src/model.c:3548-3589: scores (q.k)*scale
// over the keys a position may see, softmax with the maximum taken out, weighted values;
// window bound :6326); the arrangement is not.  The query rows that share one key/value
// head -- (token, head-in-group) pairs of one request -- are packed 32 to a block, so the
// 4 heads of a decoded token, or 8 tokens x 4 heads of a prompt portion, read each key
// and value once.  The host lists the work: row blocks with a range of keys each.  Long
// portions go to k_attn_cta (128 rows a workgroup, the tiles shared by its waves), all else
// to k_attn_stream (32 rows a workgroup, the tiles dealt out to its waves); both bring
// the tiles of K and V^T into LDS by asynchronous copies and have a wave compute, for every
// tile of 32 keys, transposed,
//     S^T[key, row] = K[key, :] . Q[row, :]        v_mfma_f32_32x32x16_bf16, A = K tile
//     O^T[d, row]  += V^T[d, key] * P^T[key, row]  A = V^T tile (values are cached transposed)
// so that a lane owns one query row throughout: row maxima and sums are sums over the
// lane's registers and one exchange with the lane 32 places away, and rescaling O^T is a
// multiplication by the lane's own factor.  The key a tile row stands for is permuted so
// that the 8 scores a lane holds for a block of 16 keys are the 8 keys the next MFMA
// wants from it: P^T goes from accumulator to operand without leaving the lane.
// Scores, maxima, sums and the output accumulate in 32-bit; P is rounded to bfloat16
// for the second product.  Items that cover part of a row block's keys write partial
// results that k_attn_merge combines (src/kernels.cu:2171-2270 does this
// with 8 fixed slices for decoding).  Page sizes are powers of two from 16; a key that does
// not exist (past the request's end, or in a page the window has given back) is copied from
// a block of zeros, and the words of V^T past the end in the last tile are masked on use
// (k_attn_cta copies a tile that exists whole where the head size allows, never reads a tile
// it did not copy, and chooses among the scores instead of multiplying them: see there).
#include <type_traits>

#include "common.h"
#include "async_copy.h"

#ifndef XR_HEAD_DIM
#error "compile with -DXR_HEAD_DIM=<head size>"
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int HD = XR_HEAD_DIM;
constexpr int KD = HD / 16;          // k-steps of the score product
constexpr int DB = (HD + 31) / 32;   // 32-row blocks of O^T
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16 up to 256");

#define ITEM_INTS 8                   // req, row0, k_begin, k_end, slot (-1: final), q0, q_len, start
#define ROWS 32
#define JOB_INTS 7                    // req, row0, first slot, slots, distance between slots, q0, q_len (as in the items)

struct AttnArgs {
    const bf16_t* q;        // [T, H, HD]
    const bf16_t* kc;       // [pages, Hk, page_size, HD]
    const bf16_t* vc;       // [pages, Hk, HD, page_size]
    bf16_t* out;            // [T, H, HD]
    const int* items;       // [n_items, ITEM_INTS]; q0: the request's first row, start: its first position
    const int* cta_items;   // [n_cta_items, ITEM_INTS]: the same for 128-row blocks that a whole workgroup takes
    const int* cu_q;        // [B + 1] first row (token) of each request in this step
    const int* starts;      // [B] position of each request's first token of this step
    const int* block_table; // [B, table_stride]
    int table_stride;
    float* part_o;          // [slots, Hk, ROWS, HD]
    float* part_ml;         // [slots, Hk, ROWS, 2]
    int n_items, n_cta_items, H, Hk, page_shift, page_mask, page_size;
    float scale;
    int window;
};

__device__ inline uint4 ldg16(const bf16_t* p) { return *reinterpret_cast<const uint4*>(p); }
__device__ inline bf16x8 as_bf16x8(uint4 v) {
    union { uint4 u; bf16x8 b; } c;
    c.u = v;
    return c.b;
}
__device__ inline uint4 keep_if(bool ok, uint4 v) {     // zero unless ok, word by word
    return make_uint4(ok ? v.x : 0u, ok ? v.y : 0u, ok ? v.z : 0u, ok ? v.w : 0u);
}
__device__ inline uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }

// One tile's softmax step for the lane's row: p[] from s[], the running reference m and sum l,
// and the rescaling of the output accumulators when the reference moved.  A row's scores lie in two
// lanes (32 apart); the maximum is exchanged every tile, the sum l is kept per lane (both lanes
// rescale by the same factor) and the two halves are added once, when the row is finished.  The reference is a
// maximum seen so far, and follows the true maximum only when that has risen by more than
// MAX_SLACK (in units of log2): any reference gives the same quotient sum(p v) / sum(p), terms up
// to 2^8 are no strain on 32-bit sums or on bfloat16 P, and the 64 multiplications a lane owes
// its output when any row of the wave moves its reference become rare (before, nearly every tile
// of a few thousand keys paid them).
// the largest of three in one instruction (fmaxf's promise about signalling NaNs costs a second
// instruction per maximum; a NaN score makes the row's output NaN either way).
// The compiler does not count the wait states an instruction written as assembly owes the matrix
// unit: the first reader of a product's result must be an instruction of the compiler's own (it
// then waits until the whole result is written), and `a` must come from such an instruction.  A
// chain that began with max3 on the accumulator itself read registers the product had not written
// yet: the reference of the running softmax was then some older maximum, which gives the same
// quotient, but a rounding that changed from run to run with the timing of the waves.
__device__ inline float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
// the larger of a lane's value and that of the lane 32 places away, in both lanes: one swap of
// register halves between lanes (gfx950) and one maximum, where an exchange through the LDS
// crossbar made every tile's softmax wait for its round trip
__device__ inline float max_across_halves(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    float o;
    asm("v_max_f32 %0, %1, %2" : "=v"(o) : "v"(__uint_as_float(r[0])), "v"(__uint_as_float(r[1])));
    return o;
}
#define MAX_SLACK 8.0f
#define ATTN_SOFTMAX_STEP(KT, KEND)                                                                  \
        if ((KT) + 32 <= (KEND) && (KT) + 31 <= pos_min && (KT) >= lo_max) {                             \
            float mt = fmaxf(s[0], s[15]);      /* the compiler's own instruction reads s first */       \
            mt = max3(mt, s[1], s[2]);                                                                   \
_Pragma("unroll")                                                                                        \
            for (int e = 3; e < 15; e += 2) mt = max3(mt, s[e], s[e + 1]);                               \
            mt = max_across_halves(mt);                                                                  \
            const float mn = mt * c2 > m + MAX_SLACK ? mt * c2 : m;                                      \
            corr = __builtin_amdgcn_exp2f(m - mn);                                                       \
            float rs = 0.f;                                                                              \
_Pragma("unroll")                                                                                        \
            for (int e = 0; e < 16; ++e) {                                                               \
                p[e] = __builtin_amdgcn_exp2f(fmaf(s[e], c2, -mn));                                      \
                rs += p[e];                                                                              \
            }                                                                                            \
            l = fmaf(l, corr, rs);                                                                       \
            m = mn;                                                                                      \
        } else {                                                                                         \
            float mt = -INFINITY;                                                                        \
_Pragma("unroll")                                                                                        \
            for (int e = 0; e < 16; ++e) {                                                               \
                const int key = (KT) + 16 * (e >> 3) + 8 * lg + (e & 7);                                 \
                const bool ok = row_ok && key <= pos && key >= lo && key < (KEND);                       \
                p[e] = ok ? s[e] * c2 : -INFINITY;                                                       \
                mt = fmaxf(mt, p[e]);                                                                    \
            }                                                                                            \
            mt = max_across_halves(mt);                                                                  \
            const float mn = mt > m + MAX_SLACK ? mt : m;                                                \
            const float mu = mn == -INFINITY ? 0.f : mn;                                                 \
            corr = __builtin_amdgcn_exp2f(m - mu);                                                       \
            float rs = 0.f;                                                                              \
_Pragma("unroll")                                                                                        \
            for (int e = 0; e < 16; ++e) {                                                               \
                p[e] = __builtin_amdgcn_exp2f(p[e] - mu);                                                \
                rs += p[e];                                                                              \
            }                                                                                            \
            l = fmaf(l, corr, rs);                                                                       \
            m = mn;                                                                                      \
        }                                                                                                \
        if (__any(corr != 1.0f)) {                                                                       \
_Pragma("unroll")                                                                                        \
            for (int d = 0; d < DB; ++d)                                                                 \
_Pragma("unroll")                                                                                        \
                for (int e = 0; e < 16; ++e) o[d][e] *= corr;                                            \
        }

// ------------------------------------------------------------------------------ workgroup kernel
// Long prompt portions: a set of 4 waves takes 128 consecutive rows of one request and
// key/value head (wave w the rows row0 + 32 w ..) and a range of keys (a workgroup is one such
// set, or two that halve the range between them: CtaShape::SETS below).  The K tile
// [32 keys][HD] and the V^T tile [HD][32 keys] are copied once into LDS for all four waves,
// by asynchronous copies, two places of a ring of four at a time, into the two that were read
// last (measured at head size 128, a prompt of 2,048 tokens: a barrier and a round of address
// arithmetic every tile with three tiles ahead 73 us, every second tile 71 us), instead of
// once per wave from the caches; each wave then works as above with its fragments read from
// LDS.  A wave skips the tiles that none of its rows can see, but takes part in every copy and
// barrier.
//
// LDS places are 16-byte chunks.  K: row r (key kt + r) has its chunk c at r * KSTR + c',
// c' = c ^ (r mod CK) where CK is a power of two, else c with rows one chunk apart more
// than their length, so that the lanes of a fragment read (32 rows, one column) fall into
// different banks.  V^T: channel d has the 4 chunks of its 32 keys at d * 4 + (c ^ (d/4 mod 4)).
constexpr int CK = HD / 8;                                  // chunks of a key row
constexpr bool CK_POW2 = (CK & (CK - 1)) == 0;
constexpr int KSTR = CK_POW2 ? CK : CK + 1;                 // chunks between key rows
constexpr int NKC = 32 * KSTR;                              // chunks of a K tile
constexpr int NVC = DB * 32 * 4;                            // chunks of a V^T tile
constexpr int CTA_ROWS = 128;
constexpr int CTA_STAGES = 4;                               // places in the ring (filled two at a time)

// Four waves a set, each with one 32-row block, two waves a SIMD.  (Two blocks a wave, 64 rows, one
// wave a SIMD and the output accumulators in the upper half of the register file, so that every K
// and V^T fragment read from LDS serves two products, was built with a loop that finished a tile
// before it began the next: the same bits, and slower, 2,048 rows behind 6,144 keys 447 us against
// 316, because a lone wave has nothing to cover its own waits for LDS and at the barriers.)
//
// Two sets share an item where LDS has room for two rings: the first set takes the first half of the
// item's tiles, the second set the rest, and their results are combined through LDS at the end.  A
// compute unit then has two waves a SIMD from ONE item, and the items, which start longest first,
// follow one another on it: a causal prompt's blocks see 1 to n keys, and with one set an item (two
// items to a unit, a long one beside a short one) the long one ran on alone, one wave a SIMD, for most
// of its time (2,048 tokens, 8 key/value heads: 70 us against 63).
struct CtaShape {
    static constexpr int SET_WAVES = 4;
    static constexpr int SET_THREADS = 64 * SET_WAVES;
    static constexpr int LOADS = (NKC + NVC + SET_THREADS - 1) / SET_THREADS;     // copies per lane and place
    static constexpr int STAGE = LOADS * SET_THREADS;                               // chunks of a place in LDS
    static constexpr int SETS = 2 * CTA_STAGES * STAGE * 16 <= 144 * 1024 ? 2 : 1;
    static constexpr int THREADS = SET_THREADS * SETS;
    static constexpr int RING_BYTES = SETS * CTA_STAGES * STAGE * 16;
    static constexpr int COMBINE_BYTES = SETS == 2 ? 4 * ROWS * (HD + 4 + 2) * 4 : 0;
    static constexpr int LDS_BYTES = RING_BYTES > COMBINE_BYTES ? RING_BYTES : COMBINE_BYTES;
    static_assert(LDS_BYTES <= 160 * 1024, "the tiles do not fit into LDS");
};

// a row block's result: the final output, or the partial result of a key range
__device__ inline void cta_write_out(const AttnArgs& a, const f32x16 (&o)[DB], float m, float l, bool row_ok, int t, int h,
                                     int kvh, int lr, int lg, int slot) {
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    if (!row_ok) return;
    if (slot < 0) {
        bf16_t* op = a.out + ((size_t)t * a.H + h) * HD;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const int dd = d * 32 + e4 * 8 + lg * 4;
                if (dd < HD) {
                    uint2 w = make_uint2(pack2(o[d][e4 * 4 + 0] * inv, o[d][e4 * 4 + 1] * inv),
                                         pack2(o[d][e4 * 4 + 2] * inv, o[d][e4 * 4 + 3] * inv));
                    *reinterpret_cast<uint2*>(op + dd) = w;
                }
            }
        return;
    }
    float* po = a.part_o + (((size_t)slot * a.Hk + kvh) * ROWS + lr) * HD;
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4) {
            const int dd = d * 32 + e4 * 8 + lg * 4;
            if (dd < HD)
                *reinterpret_cast<float4*>(po + dd) = make_float4(o[d][e4 * 4 + 0] * inv, o[d][e4 * 4 + 1] * inv,
                                                                  o[d][e4 * 4 + 2] * inv, o[d][e4 * 4 + 3] * inv);
        }
    if (lg == 0) {
        float* pm = a.part_ml + (((size_t)slot * a.Hk + kvh) * ROWS + lr) * 2;
        pm[0] = m;
        pm[1] = l;
    }
}

// f(integral_constant<int, I>) for I = FROM .. TO-1, each call with its index a constant
template <int FROM, int TO, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (FROM < TO) {
        f(std::integral_constant<int, FROM>{});
        static_for<FROM + 1, TO>(f);
    }
}

__device__ __forceinline__ uint4 lds_read16(uint32_t byte_addr) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 x = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(byte_addr);
    return make_uint4(x[0], x[1], x[2], x[3]);
}

// What a wave's tile loop needs of its lane and of its rows, set up once an item.
struct CtaWave {
    uint32_t kbase;             // LDS byte address of this lane's K fragment of k-step 0 in place 0 of the set's ring
    uint32_t vbase[2];          // and of its V^T fragments of channels 0-31, keys 0-15 and 16-31
    bf16x8 qf[KD];
    float c2;
    int pos, lo, lg;
    bool row_ok;
    int kbeg, kend, nt, seq_len;
    int pos_min, pos_max, lo_min, lo_max;       // the same in every lane, in scalar registers
    __device__ __forceinline__ bool sees(int t) const {          // does any row of the wave see a key of tile t
        const int kt = kbeg + t * 32;
        return t >= 0 && t < nt && !(kt > pos_max || kt + 32 <= lo_min);
    }
    __device__ __forceinline__ bool whole(int t) const {         // does every row see all of it
        const int kt = kbeg + t * 32;
        return kt + 32 <= kend && kt + 31 <= pos_min && kt >= lo_max;
    }
};

// The softmax of a whole tile cut into 18 pieces (the maximum over the lane's scores; the exchange, the
// reference and the factor; the 16 weights) and dealt to the NS product slots of a step by their cost
// in cycles of the vector unit (an exponential is a quarter-rate instruction).
template <int NS> struct CtaPlan {
    static constexpr int WA = 32, WB = 44, WP = 26, TOTAL = WA + WB + 16 * WP;
    static constexpr int slot_of(int piece) {
        const int before = piece == 0 ? 0 : piece == 1 ? WA : WA + WB + (piece - 2) * WP;
        return before * NS / TOTAL;
    }
};

// One step of a wave: the score product of tile v, the softmax of tile v-1 and the value product of
// tile v-2, which do not depend on each other.  K of tile v and V^T of tile v-2 lie in place v mod 4 of
// the ring.  In the middle of an item (cta_step_whole: tile v-1 seen whole by all the wave's rows, tiles
// v and v-2 there) the three are written as NS slots, each one product, the fragment read of the
// product AHEAD slots on and a piece of the softmax, and the compiler keeps the slots apart: the matrix
// unit then works on one tile while the vector unit works on another, in one wave, where the loop that
// finished a tile before it began the next had each unit wait for the other (counters: the matrix unit
// busy 36% of the cycles, the vector unit 40%, both at once 10%).  At an item's edges (cta_step_edge)
// the three run one after the other, each if its tile is there.  The two kinds of step are the bodies
// of loops of their own, not two branches of one loop: where two branches that both write the output
// accumulators meet, the compiler kept a second copy of those 64 registers and spilled.
struct CtaFrags {
    uint32_t kb, vb[2];
    template <int STAGE> __device__ __forceinline__ CtaFrags(const CtaWave& w, int v, std::integral_constant<int, STAGE>) {
        const uint32_t st = (uint32_t)(v & (CTA_STAGES - 1)) * (STAGE * 16);
        kb = w.kbase + st;
        vb[0] = w.vbase[0] + st + NKC * 16;
        vb[1] = w.vbase[1] + st + NKC * 16;
    }
    // (k-step kd of a K row: 32 bytes on, or, where the chunks of a row are swapped about by the
    // row's number, the address with kd's bits flipped: one register for all k-steps)
    template <int K> __device__ __forceinline__ uint4 get() const {
        if constexpr (K < KD) return lds_read16(CK_POW2 ? kb ^ (uint32_t)(K << 5) : kb + (uint32_t)(K << 5));
        else return lds_read16(vb[(K - KD) / DB] + ((K - KD) % DB) * 128 * 16);
    }
};

template <int STAGE>
__device__ __forceinline__ void cta_step_whole(const CtaWave& w, int v, f32x16& s_new, const f32x16& s_cur,
                                               uint4 (&pf_new)[2], const uint4 (&pf_old)[2], f32x16 (&o)[DB], float& m, float& l) {
    constexpr int NS = KD + 2 * DB, AHEAD = 3 < NS ? 3 : NS;
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const CtaFrags f(w, v, std::integral_constant<int, STAGE>{});
    const f32x16& s = s_cur;
    uint4 fr[NS];
    static_for<0, AHEAD>([&](auto kc) { fr[decltype(kc)::value] = f.template get<decltype(kc)::value>(); });
    float mt = 0.f, mn = 0.f, corr = 1.f, rs = 0.f, pe = 0.f;
    uint32_t pk[8];
    __builtin_amdgcn_sched_barrier(0);
    static_for<0, NS>([&](auto kc) {
        constexpr int k = decltype(kc)::value;
        if constexpr (k + AHEAD < NS) fr[k + AHEAD] = f.template get<k + AHEAD>();
        if constexpr (k == 0) s_new = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(fr[k]), w.qf[k], zero, 0, 0, 0);
        else if constexpr (k < KD) s_new = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(fr[k]), w.qf[k], s_new, 0, 0, 0);
        else {
            constexpr int j = (k - KD) / DB, d = (k - KD) % DB;
            o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(fr[k]), as_bf16x8(pf_old[j]), o[d], 0, 0, 0);
        }
        static_for<0, 18>([&](auto pc) {
            constexpr int piece = decltype(pc)::value;
            if constexpr (CtaPlan<NS>::slot_of(piece) == k) {
                if constexpr (piece == 0) {
                    mt = fmaxf(s[0], s[15]);        // the compiler's own instruction reads s first
                    mt = max3(mt, s[1], s[2]);
#pragma unroll
                    for (int e = 3; e < 15; e += 2) mt = max3(mt, s[e], s[e + 1]);
                } else if constexpr (piece == 1) {
                    mt = max_across_halves(mt);
                    mn = mt * w.c2 > m + MAX_SLACK ? mt * w.c2 : m;
                    corr = __builtin_amdgcn_exp2f(m - mn);
                    asm volatile("" : "+v"(corr));
                } else {
                    // (each piece ends in a statement the compiler may not move: it would otherwise
                    // put off all the weights, which nothing in this step reads, to behind the step's
                    // last branch, and the vector unit's work would again follow the matrix unit's)
                    constexpr int e = piece - 2;
                    const float x = __builtin_amdgcn_exp2f(fmaf(s[e], w.c2, -mn));
                    rs += x;
                    asm volatile("" : "+v"(rs));
                    if constexpr (e % 2 == 1) {
                        pk[e / 2] = pack2(pe, x);
                        asm volatile("" : "+v"(pk[e / 2]));
                    } else pe = x;
                }
            }
        });
        __builtin_amdgcn_sched_barrier(0);
    });
    pf_new[0] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
    pf_new[1] = make_uint4(pk[4], pk[5], pk[6], pk[7]);
    l = fmaf(l, corr, rs);
    m = mn;
    if (__any(corr != 1.0f)) {
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int e = 0; e < 16; ++e) o[d][e] *= corr;
    }
}

template <int STAGE>
__device__ __forceinline__ void cta_step_edge(const CtaWave& w, int v, f32x16& s_new, const f32x16& s_cur,
                                              uint4 (&pf_new)[2], const uint4 (&pf_old)[2], f32x16 (&o)[DB], float& m, float& l) {
    constexpr int NS = KD + 2 * DB;
    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    const CtaFrags f(w, v, std::integral_constant<int, STAGE>{});
    const int lg = w.lg;
    if (w.sees(v)) {
        uint4 kf[KD];
        static_for<0, KD>([&](auto kc) { kf[decltype(kc)::value] = f.template get<decltype(kc)::value>(); });
        s_new = zero;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) s_new = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kf[kd]), w.qf[kd], s_new, 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);           // (one after the other: their fragments do not wait in registers side by side)
    if (w.sees(v - 2)) {
        uint4 vf[2 * DB];
        static_for<KD, NS>([&](auto kc) { vf[decltype(kc)::value - KD] = f.template get<decltype(kc)::value>(); });
        const int kt = w.kbeg + (v - 2) * 32;
        if (kt + 32 > w.seq_len) {             // the request's last tile: slots past its end hold old data
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int k8 = kt + 16 * j + 8 * lg;
                uint32_t mk[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    mk[e] = (k8 + 2 * e < w.seq_len ? 0x0000FFFFu : 0u) | (k8 + 2 * e + 1 < w.seq_len ? 0xFFFF0000u : 0u);
#pragma unroll
                for (int d = 0; d < DB; ++d) {
                    uint4& x = vf[j * DB + d];
                    x.x &= mk[0]; x.y &= mk[1]; x.z &= mk[2]; x.w &= mk[3];
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int d = 0; d < DB; ++d)
                o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vf[j * DB + d]), as_bf16x8(pf_old[j]), o[d], 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (w.sees(v - 1)) {
        const f32x16& s = s_cur;
        const int kt = w.kbeg + (v - 1) * 32;
        const bool row_ok = w.row_ok;
        const int pos = w.pos, lo = w.lo, pos_min = w.pos_min, lo_max = w.lo_max;
        const float c2 = w.c2;
        float p[16];
        float corr;
        ATTN_SOFTMAX_STEP(kt, w.kend)
        pf_new[0] = make_uint4(pack2(p[0], p[1]), pack2(p[2], p[3]), pack2(p[4], p[5]), pack2(p[6], p[7]));
        pf_new[1] = make_uint4(pack2(p[8], p[9]), pack2(p[10], p[11]), pack2(p[12], p[13]), pack2(p[14], p[15]));
    }
}

// The kernel.  A place of the ring holds K of tile v beside V^T of tile v-2, which is what step v reads.
__global__ __launch_bounds__(CtaShape::THREADS, 1) void k_attn_cta(AttnArgs a) {
    using SH = CtaShape;
    constexpr int SET_THREADS = SH::SET_THREADS, LOADS = SH::LOADS, STAGE = SH::STAGE, SETS = SH::SETS;
    static_assert(CTA_STAGES == 4, "the steps below name the four places of the ring");
    extern __shared__ uint4 lds_all[];                      // [SETS][CTA_STAGES][STAGE]
    const int tid = threadIdx.x % SET_THREADS, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);                          // within the set
    const int set = __builtin_amdgcn_readfirstlane((int)threadIdx.x / SET_THREADS);
    uint4* lds = lds_all + set * CTA_STAGES * STAGE;
    // Items come longest first, and workgroups start in the order of their numbers: an item's
    // key/value heads are numbered side by side, so that the longest items of every head start
    // first.  (With 8 key/value heads a head's items then also run on one of the 8 dies and share
    // its L2.)
    unsigned wg = blockIdx.x;
    if (SETS == 1 && gridDim.x <= 512 && wg >= (gridDim.x + 1) / 2) wg = gridDim.x - 1 - (wg - (gridDim.x + 1) / 2);
    const int item_no = (int)(wg / (unsigned)a.Hk);
    const int kvh = (int)wg - item_no * a.Hk;
    const int* it = a.cta_items + (size_t)item_no * ITEM_INTS;
    const int req = it[0];
    const int q_len = it[6], start = it[7];
    const int nt_item = (it[3] - it[2] + 31) >> 5;
    const int nt_first = SETS == 2 ? (nt_item + 1) >> 1 : nt_item;
    const int kbeg = it[2] + set * nt_first * 32;
    const int kend = (set == 0 && SETS == 2 && it[2] + nt_first * 32 < it[3]) ? it[2] + nt_first * 32 : it[3];
    const int G = a.H / a.Hk;
    const int seq_len = start + q_len;
    const int* bt = a.block_table + (size_t)req * a.table_stride;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds;

    CtaWave w;
    {
        const int lr = lane & 31, lg = lane >> 5;
        const int rho = it[1] + wave * ROWS + lr;
        const int tok = rho / G, hg = rho - tok * G;
        const bool row_ok = tok < q_len;
        w.row_ok = row_ok;
        w.pos = start + tok;
        w.lo = (a.window > 0 && w.pos - a.window + 1 > 0) ? w.pos - a.window + 1 : 0;
        w.lg = lg;
        const bf16_t* qp = a.q + ((size_t)(row_ok ? it[5] + tok : it[5]) * a.H + kvh * G + hg) * HD + lg * 8;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) w.qf[kd] = as_bf16x8(keep_if(row_ok, ldg16(qp + kd * 16)));
        const int ra = lr >> 3, rg = (lr >> 2) & 1, rb4 = lr & 3;
        const int key_off = 16 * (ra >> 1) + 8 * rg + 4 * (ra & 1) + rb4;
        // (with swapped chunks a row is a power of two long and the ring begins at a multiple of it:
        // the chunk's number within the row is the address's low bits, and k-step kd flips bits of it)
        w.kbase = lds_base + (uint32_t)(key_off * KSTR + (CK_POW2 ? (lg ^ (key_off & (CK - 1))) : lg)) * 16u;
#pragma unroll
        for (int j = 0; j < 2; ++j) w.vbase[j] = lds_base + (uint32_t)(lr * 4 + ((2 * j + lg) ^ ((lr >> 2) & 3))) * 16u;
    }

    // The pieces this lane copies for every place of the ring.  Where every lane's piece exists in every
    // whole tile and a copy instruction brings pieces of keys only or of values only (head sizes 64, 128
    // and 256), a whole tile of an existing page is copied from two bases that all lanes share, each
    // lane adding a fixed 32-bit offset.
    constexpr bool CTA_FAST = CK_POW2 && NKC % SET_THREADS == 0 && NVC % SET_THREADS == 0 && HD % 32 == 0;
    auto piece = [&](int i, int tid_, int& off, int& key, bool& is_k) {
        const int q = i * SET_THREADS + tid_;
        is_k = q < NKC;
        if (q < NKC) {
            const int r = q / KSTR, cs = q - r * KSTR;
            const int c = CK_POW2 ? (cs ^ (r & (CK - 1))) : cs;
            off = r * HD + c * 8;
            key = cs < CK ? r : (1 << 30);                  // the spare chunk of a row stays zero
        } else {
            const int vv = q - NKC, d = vv >> 2, c = (vv & 3) ^ ((d >> 2) & 3);
            off = d * a.page_size + c * 8;
            key = (vv < NVC && d < HD) ? c * 8 : (1 << 30);
        }
    };
    constexpr int N_OFF = CTA_FAST ? LOADS : 1;
    uint32_t fast_off[N_OFF];
    if (CTA_FAST) {
#pragma unroll
        for (int n = 0; n < N_OFF; ++n) {
            int off, key;
            bool is_k;
            piece(n, tid, off, key, is_k);
            fast_off[n] = (uint32_t)off * 2u;
        }
    }
    const bf16_t* __restrict__ kc = a.kc;
    const bf16_t* __restrict__ vc = a.vc;
    // a page's bytes (of all its key/value heads), and this head's part of page 0
    const uint32_t page_bytes = (uint32_t)a.Hk * (uint32_t)a.page_size * (HD * 2);
    const char* const kc_head = reinterpret_cast<const char*>(kc) + (size_t)kvh * a.page_size * (HD * 2);
    const char* const vc_head = reinterpret_cast<const char*>(vc) + (size_t)kvh * a.page_size * (HD * 2);
    const bf16_t* zero_src = reinterpret_cast<const bf16_t*>(xr_zero_chunk);

    // page numbers of the item's keys, one per lane, 64 pages at a time, from the page of the older of
    // the two tiles a place holds (pages hold at least 32 positions: the newer is at most 2 pages on)
    int pages_base = kbeg >> a.page_shift;
    int my_page;
    {
        const int pi = pages_base + lane;
        const bool in = ((long)pi << a.page_shift) < seq_len;
        my_page = bt[in ? pi : 0];
        my_page = in ? my_page : -1;
    }
    const int nt = kend > kbeg ? (kend - kbeg + 31) >> 5 : 0;
    // place u of the ring: K of tile u, V^T of tile u-2 (zeros for tiles that do not exist)
    // (A page number below 0, which the table holds for pages a window has given back, is read as
    // the null page: the host lists no keys from such pages, and a list that did would get wrong
    // values from here, not a fault.)
    // Place u of the ring: K of tile u and V^T of tile u-2.  A tile that does not exist (before the first,
    // past the set's last) is never read and is not copied.  Where every copy instruction brings pieces
    // of keys only or of values only, a tile that exists is copied whole, the slots past the request's
    // end with it: they lie in the tile's page, the scores of their keys are never looked at (the softmax
    // chooses, it does not multiply) and their values are masked where they are used.  Else (a head size
    // with spare chunks in LDS) each piece that exists is copied from where it lies and the others from
    // a block of zeros.
#define STEPS_ISSUE(UI)                                                                                  \
    {                                                                                                    \
        const int u_ = (UI);                                                                             \
        const int ktk_ = kbeg + u_ * 32, ktv_ = ktk_ - 64;                                               \
        const uint32_t dst_ = __builtin_amdgcn_readfirstlane(lds_base + (uint32_t)(((u_ & (CTA_STAGES - 1)) * STAGE + wave * 64) * 16)); \
        const bool k_there_ = u_ < nt && ktk_ < seq_len, v_there_ = u_ >= 2 && u_ - 2 < nt && ktv_ < seq_len; \
        if (k_there_ && (ktk_ >> a.page_shift) - pages_base >= 64) {                                     \
            pages_base = (u_ >= 2 ? ktv_ : ktk_) >> a.page_shift;                                        \
            const int pi = pages_base + lane;                                                            \
            const bool in = ((long)pi << a.page_shift) < seq_len;                                        \
            my_page = bt[in ? pi : 0];                                                                   \
            my_page = in ? my_page : -1;                                                                 \
        }                                                                                                \
        if (CTA_FAST) {                                                                                  \
            if (k_there_) {                                                                              \
                const int pg_ = __builtin_amdgcn_readlane(my_page, (ktk_ >> a.page_shift) - pages_base); \
                const char* kb_ = kc_head + (size_t)(uint32_t)max(pg_, 0) * page_bytes + (uint32_t)(ktk_ & a.page_mask) * (HD * 2); \
                _Pragma("unroll") for (int i = 0; i < LOADS; ++i)                                        \
                    if (i * SET_THREADS < NKC) lds_dma16_base(kb_, fast_off[i % N_OFF], dst_ + i * SET_THREADS * 16); \
            }                                                                                            \
            if (v_there_) {                                                                              \
                const int pg_ = __builtin_amdgcn_readlane(my_page, (ktv_ >> a.page_shift) - pages_base); \
                const char* vb_ = vc_head + (size_t)(uint32_t)max(pg_, 0) * page_bytes + (uint32_t)(ktv_ & a.page_mask) * 2; \
                _Pragma("unroll") for (int i = 0; i < LOADS; ++i)                                        \
                    if (i * SET_THREADS >= NKC) lds_dma16_base(vb_, fast_off[i % N_OFF], dst_ + i * SET_THREADS * 16); \
            }                                                                                            \
        } else {                                                                                         \
            const int pgk_ = k_there_ ? __builtin_amdgcn_readlane(my_page, __builtin_amdgcn_readfirstlane((ktk_ >> a.page_shift) - pages_base)) : -1; \
            const int pgv_ = v_there_ ? __builtin_amdgcn_readlane(my_page, __builtin_amdgcn_readfirstlane((ktv_ >> a.page_shift) - pages_base)) : -1; \
            const size_t pbk_ = (size_t)(pgk_ < 0 ? 0 : pgk_) * a.Hk + kvh;                              \
            const size_t pbv_ = (size_t)(pgv_ < 0 ? 0 : pgv_) * a.Hk + kvh;                              \
            const bf16_t* kb_ = kc + (pbk_ * a.page_size + (ktk_ & a.page_mask)) * HD;                   \
            const bf16_t* vb_ = vc + pbv_ * HD * a.page_size + (ktv_ & a.page_mask);                     \
            _Pragma("unroll") for (int i = 0; i < LOADS; ++i) {                                          \
                int tid_ = tid, off_, key_;                                                              \
                bool isk_;                                                                               \
                asm volatile("" : "+v"(tid_));            /* (worked out here, not kept in registers throughout) */ \
                piece(i, tid_, off_, key_, isk_);                                                        \
                const bool okc_ = isk_ ? (pgk_ >= 0 && ktk_ + key_ < seq_len) : (pgv_ >= 0 && ktv_ + key_ < seq_len); \
                const bf16_t* p_ = okc_ ? (isk_ ? kb_ : vb_) + off_ : zero_src;                          \
                lds_dma16(p_, dst_ + i * SET_THREADS * 16);                                              \
            }                                                                                            \
        }                                                                                                \
    }

    f32x16 o[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[d][e] = 0.f;
    float m = -INFINITY, l = 0.f;           // m in units of log2
    {
        // what the wave's rows can see: keys [lo_min, pos_max]; keys in [lo_max, pos_min] by all
        int pos_min = w.row_ok ? w.pos : 0x7fffffff, lo_max = w.row_ok ? w.lo : 0;
        int pos_max = w.row_ok ? w.pos : -1, lo_min = w.row_ok ? w.lo : 0x7fffffff;
#pragma unroll
        for (int x = 32; x > 0; x >>= 1) {
            pos_min = min(pos_min, __shfl_xor(pos_min, x, 64));
            lo_max = max(lo_max, __shfl_xor(lo_max, x, 64));
            pos_max = max(pos_max, __shfl_xor(pos_max, x, 64));
            lo_min = min(lo_min, __shfl_xor(lo_min, x, 64));
        }
        w.pos_min = __builtin_amdgcn_readfirstlane(pos_min); w.lo_max = __builtin_amdgcn_readfirstlane(lo_max);
        w.pos_max = __builtin_amdgcn_readfirstlane(pos_max); w.lo_min = __builtin_amdgcn_readfirstlane(lo_min);
    }
    w.c2 = a.scale * 1.44269504088896340736f;
    w.kbeg = kbeg; w.kend = kend; w.nt = nt; w.seq_len = seq_len;

    // Step v of a wave touches place v of the ring only, so the places are filled and waited for two
    // at a time as before: at the barrier before steps v and v+1 every wave has done with places v-2
    // and v-1, which then take what steps v+2 and v+3 will read.  A set's tiles take two steps more than
    // it has tiles; both sets go through the loops as often as the first, every wave through the same
    // number of steps, whichever loop it does them in.
    static_assert(LOADS * 2 < 64, "two places' copies are counted at once");
    const int n_steps = nt_first + 2;
    // steps [v1, v2), in pairs: the wave's whole steps.  The steps with a tile v-1 that all rows see
    // whole and tiles v, v-2 that exist are consecutive (each condition holds for a range of v), so
    // both ends are tried and nothing between them.
    auto whole_step = [&](int v) { return w.sees(v) && w.sees(v - 1) && w.sees(v - 2) && w.whole(v - 1); };
    int v1, v2;
    {
        // the first and the last tile that all rows see whole, from the same comparisons as CtaWave::whole
        const int up = min(min(kend - kbeg, min(w.pos_min, kend) + 1 - kbeg), nt * 32);      // (a wave without rows has pos_min at the largest int)
        const int t_last = up >= 32 ? (up >> 5) - 1 : -1;
        const int t_first = w.lo_max > kbeg ? (w.lo_max - kbeg + 31) >> 5 : 0;
        v1 = (max(t_first + 1, 2) + 1) & ~1;
        v2 = min(t_last + 2, n_steps) & ~1;
        while (v1 < v2 && !(whole_step(v1) && whole_step(v1 + 1))) v1 += 2;
        while (v1 < v2 && !(whole_step(v2 - 2) && whole_step(v2 - 1))) v2 -= 2;
        if (v1 >= v2) v1 = v2 = 0;
    }
    f32x16 s_even, s_odd;                    // the scores of the tiles with even and with odd numbers
    uint4 pf_even[2] = {}, pf_odd[2] = {};   // and their weights, rounded, as the value product takes them
    STEPS_ISSUE(0)
    STEPS_ISSUE(1)
#define STEPS_SYNC(V)                                                                                    \
        wait_vmcnt<0>();                                                                                 \
        __builtin_amdgcn_s_barrier();                                                                    \
        STEPS_ISSUE((V) + 2)                                                                             \
        STEPS_ISSUE((V) + 3)
    int v = 0;
    for (; v < v1; v += 2) {
        STEPS_SYNC(v)
        cta_step_edge<STAGE>(w, v, s_even, s_odd, pf_odd, pf_even, o, m, l);
        cta_step_edge<STAGE>(w, v + 1, s_odd, s_even, pf_even, pf_odd, o, m, l);
    }
    for (; v < v2; v += 2) {
        STEPS_SYNC(v)
        cta_step_whole<STAGE>(w, v, s_even, s_odd, pf_odd, pf_even, o, m, l);
        cta_step_whole<STAGE>(w, v + 1, s_odd, s_even, pf_even, pf_odd, o, m, l);
    }
    for (; v < n_steps; v += 2) {
        STEPS_SYNC(v)
        cta_step_edge<STAGE>(w, v, s_even, s_odd, pf_odd, pf_even, o, m, l);
        cta_step_edge<STAGE>(w, v + 1, s_odd, s_even, pf_even, pf_odd, o, m, l);
    }
#undef STEPS_SYNC
#undef STEPS_ISSUE
    wait_vmcnt<0>();                                     // the trailing copies of zeros
    l += __shfl_xor(l, 32, 64);                          // the row's sum from its two lanes

    // (the row's place in the output is worked out again here, from a lane number the compiler cannot
    // trace back, rather than kept in registers through the loop)
    int lane_after = lane;
    asm volatile("" : "+v"(lane_after));
    const int lr = lane_after & 31, lg = lane_after >> 5;
    const int rho = it[1] + wave * ROWS + lr;
    const int tok = rho / G, hg = rho - tok * G;
    const int slot = it[4] < 0 ? -1 : it[4] + wave;
    const bool row_ok = tok < q_len;
    const int t = it[5] + tok, h = kvh * G + hg;
    if (SETS == 2) {
        // the second set hands its rows' maxima, sums and unnormalised outputs to the first
        __syncthreads();                                 // the rings are free
        float* xo = reinterpret_cast<float*>(lds_all);   // [4 row blocks][ROWS][HD + 4]
        float* xml = xo + 4 * ROWS * (HD + 4);           // [4 row blocks][ROWS][2]
        float* mine = xo + (wave * ROWS + lr) * (HD + 4);
        if (set == 1) {
#pragma unroll
            for (int d = 0; d < DB; ++d)
#pragma unroll
                for (int e4 = 0; e4 < 4; ++e4) {
                    const int dd = d * 32 + e4 * 8 + lg * 4;
                    if (dd < HD)
                        *reinterpret_cast<float4*>(mine + dd) = make_float4(o[d][e4 * 4 + 0], o[d][e4 * 4 + 1], o[d][e4 * 4 + 2], o[d][e4 * 4 + 3]);
                }
            if (lg == 0) {
                xml[(wave * ROWS + lr) * 2] = m;
                xml[(wave * ROWS + lr) * 2 + 1] = l;
            }
        }
        __syncthreads();
        if (set == 1) return;
        const float m1 = xml[(wave * ROWS + lr) * 2], l1 = xml[(wave * ROWS + lr) * 2 + 1];
        const float mn = fmaxf(m, m1);
        const float f0 = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m - mn);
        const float f1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m1 - mn);
        l = l * f0 + l1 * f1;
        m = mn;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const int dd = d * 32 + e4 * 8 + lg * 4;
                if (dd < HD) {
                    const float4 x = *reinterpret_cast<const float4*>(mine + dd);
                    o[d][e4 * 4 + 0] = o[d][e4 * 4 + 0] * f0 + x.x * f1;
                    o[d][e4 * 4 + 1] = o[d][e4 * 4 + 1] * f0 + x.y * f1;
                    o[d][e4 * 4 + 2] = o[d][e4 * 4 + 2] * f0 + x.z * f1;
                    o[d][e4 * 4 + 3] = o[d][e4 * 4 + 3] * f0 + x.w * f1;
                }
            }
    }
    cta_write_out(a, o, m, l, row_ok, t, h, kvh, lr, lg, slot);
}

// ------------------------------------------------------------------------------ streaming kernel
// Decoded tokens and short portions: few rows, many keys, bound by how fast the keys and
// values arrive.  A workgroup takes one item (a 32-row block and a range of keys); its waves
// share the rows and take the item's tiles in turn, wave w the tiles w, w + STREAM_WAVES, ..
// Every wave copies its own tiles into a ring of its own in LDS (whole key rows and runs of
// 64 bytes of V^T per lane group, instead of 32 bytes from 32 places per load instruction)
// and reads its fragments from there, so the main loop has no barrier at all.  At the end
// the waves' results are combined through LDS and written as the output or as one partial.
constexpr int STREAM_WAVES = HD <= 128 ? 4 : 2;
constexpr int W_LOADS = (NKC + NVC + 63) / 64;              // copies per lane and tile
constexpr int W_STAGE = W_LOADS * 64;                       // chunks of a wave's tile
// (measured at head size 128, batches of 1 to 64 and contexts of 2k and 8k: 4 waves with 2 tiles
// each, 3 with 3, 2 with 2 to 4 and 1 with 3 or 4 are all within 5% of each other)
constexpr int STREAM_STAGES = W_STAGE * 16 * STREAM_WAVES * 3 <= 96 * 1024 ? 3 : 2;
constexpr int MERGE_STRIDE = HD + 4;                        // floats between rows of the combining buffer
constexpr int STREAM_RING_BYTES = STREAM_WAVES * STREAM_STAGES * W_STAGE * 16;
constexpr int STREAM_MERGE_BYTES = STREAM_WAVES * ROWS * (MERGE_STRIDE + 2) * 4;
constexpr int STREAM_LDS_BYTES = STREAM_RING_BYTES > STREAM_MERGE_BYTES ? STREAM_RING_BYTES : STREAM_MERGE_BYTES;
static_assert(W_LOADS * (STREAM_STAGES - 1) < 64, "too many copies in flight for the counter");
static_assert(STREAM_LDS_BYTES <= 160 * 1024, "the rings do not fit into LDS");

__global__ __launch_bounds__(64 * STREAM_WAVES) void k_attn_stream(AttnArgs a) {
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    // Workgroups start in the order of their numbers and the items come longest first: an item's
    // key/value heads are numbered side by side, so that the longest items of every head start
    // first and the shortest fill the end (numbered head by head, the last head's longest item
    // started among the last and ran on alone: 32 requests of 192 to 2,176 keys with 32 key/value
    // heads took 143 us, now 127).
    const int item_no = (int)(blockIdx.x / (unsigned)a.Hk);
    const int kvh = (int)blockIdx.x - item_no * a.Hk;
    const int* it = a.items + (size_t)item_no * ITEM_INTS;
    const int req = it[0], row0 = it[1], kbeg = it[2], kend = it[3], slot = it[4];
    const int q0 = it[5], q_len = it[6], start = it[7];
    const int G = a.H / a.Hk;
    const int lr = lane & 31, lg = lane >> 5;
    const int seq_len = start + q_len;
    const int* bt = a.block_table + (size_t)req * a.table_stride;

    const int rho = row0 + lr;
    const int tok = rho / G, hg = rho - tok * G;
    const bool row_ok = tok < q_len;
    const int t = q0 + tok, h = kvh * G + hg;
    const int pos = start + tok;
    const int lo = (a.window > 0 && pos - a.window + 1 > 0) ? pos - a.window + 1 : 0;

    bf16x8 qf[KD];
    {
        const bf16_t* qp = a.q + ((size_t)(row_ok ? t : q0) * a.H + h) * HD + lg * 8;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) qf[kd] = as_bf16x8(keep_if(row_ok, ldg16(qp + kd * 16)));
    }
    const int ra = lr >> 3, rg = (lr >> 2) & 1, rb = lr & 3;
    const int key_off = 16 * (ra >> 1) + 8 * rg + 4 * (ra & 1) + rb;

    // the pieces this lane copies for every tile: a key (K: its row, V^T: the first of 8) and
    // an offset from that key's place in its page
    int src_off[W_LOADS], src_key[W_LOADS];
    bool src_is_k[W_LOADS];
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
        const int q = i * 64 + lane;
        src_is_k[i] = q < NKC;
        if (q < NKC) {
            const int r = q / KSTR, cs = q - r * KSTR;
            const int c = CK_POW2 ? (cs ^ (r & (CK - 1))) : cs;
            src_off[i] = c * 8;
            src_key[i] = cs < CK ? r : (1 << 30);           // the spare chunk of a row stays zero
        } else {
            const int v = q - NKC, d = v >> 2, c = (v & 3) ^ ((d >> 2) & 3);
            src_off[i] = d * a.page_size;
            src_key[i] = (v < NVC && d < HD) ? c * 8 : (1 << 30);
        }
    }
    const bf16_t* __restrict__ kc = a.kc;
    const bf16_t* __restrict__ vc = a.vc;
    const bf16_t* zero_src = reinterpret_cast<const bf16_t*>(xr_zero_chunk);
    const uint32_t ring_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)lds +
                                                              (uint32_t)(wave * STREAM_STAGES * W_STAGE * 16));
    const uint4* ring = lds + wave * STREAM_STAGES * W_STAGE;

    int pages_base = kbeg >> a.page_shift;
    int my_page;
    {
        const int pi = pages_base + lane;
        const bool in = ((long)pi << a.page_shift) < seq_len;
        my_page = bt[in ? pi : 0];
        my_page = in ? my_page : -1;
    }
    const int nt = (kend - kbeg + 31) >> 5;
    const int n_mine = nt > wave ? (nt - wave + STREAM_WAVES - 1) / STREAM_WAVES : 0;
    // Copy of this wave's j-th tile (zeros past its last one).  With pages of 32 positions and
    // more a tile lies in one page; with smaller ones every lane looks its own page up.
#define STREAM_ISSUE(J)                                                                                  \
    {                                                                                                    \
        const int j_ = (J);                                                                              \
        const int kt_ = kbeg + (wave + j_ * STREAM_WAVES) * 32;                                          \
        const bool live_ = j_ < n_mine;                                                                  \
        if (live_ && ((kt_ + 31) >> a.page_shift) - pages_base >= 64) {                                  \
            pages_base = kt_ >> a.page_shift;                                                            \
            const int pi = pages_base + lane;                                                            \
            const bool in = ((long)pi << a.page_shift) < seq_len;                                        \
            my_page = bt[in ? pi : 0];                                                                   \
            my_page = in ? my_page : -1;                                                                 \
        }                                                                                                \
        const uint32_t dst_ = __builtin_amdgcn_readfirstlane(ring_base + (uint32_t)((j_ % STREAM_STAGES) * W_STAGE * 16)); \
        if (a.page_size >= 32) {                                                                         \
            int pg_ = -1;                                                                                \
            if (live_) pg_ = __builtin_amdgcn_readlane(my_page, __builtin_amdgcn_readfirstlane((kt_ >> a.page_shift) - pages_base)); \
            const size_t pb_ = (size_t)(pg_ < 0 ? 0 : pg_) * a.Hk + kvh;                                 \
            const int ko_ = kt_ & a.page_mask;                                                           \
            const bf16_t* kb_ = kc + (pb_ * a.page_size + ko_) * HD;                                     \
            const bf16_t* vb_ = vc + pb_ * HD * a.page_size + ko_;                                       \
            _Pragma("unroll") for (int i = 0; i < W_LOADS; ++i) {                                        \
                const bool ok_ = pg_ >= 0 && kt_ + src_key[i] < seq_len;                                 \
                const bf16_t* p_ = ok_ ? (src_is_k[i] ? kb_ + src_key[i] * HD : vb_ + src_key[i]) + src_off[i] : zero_src; \
                lds_dma16(p_, dst_ + i * 64 * 16);                                                       \
            }                                                                                            \
        } else {                                                                                         \
            _Pragma("unroll") for (int i = 0; i < W_LOADS; ++i) {                                        \
                const int key_ = kt_ + src_key[i];                                                       \
                const bool in_ = live_ && key_ < seq_len;                                                \
                const int pg_ = __shfl(my_page, in_ ? (key_ >> a.page_shift) - pages_base : 0, 64);      \
                const bool ok_ = in_ && pg_ >= 0;                                                        \
                const size_t pb_ = (size_t)(ok_ ? pg_ : 0) * a.Hk + kvh;                                 \
                const int ko_ = key_ & a.page_mask;                                                      \
                const bf16_t* p_ = src_is_k[i] ? kc + (pb_ * a.page_size + ko_) * HD + src_off[i]        \
                                               : vc + pb_ * HD * a.page_size + src_off[i] + ko_;         \
                lds_dma16(ok_ ? p_ : zero_src, dst_ + i * 64 * 16);                                      \
            }                                                                                            \
        }                                                                                                \
    }

    f32x16 o[DB];
#pragma unroll
    for (int d = 0; d < DB; ++d)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[d][e] = 0.f;
    float m = -INFINITY, l = 0.f;      // m in units of log2
    const float c2 = a.scale * 1.44269504088896340736f;
    int pos_min = row_ok ? pos : 0x7fffffff, lo_max = row_ok ? lo : 0;
#pragma unroll
    for (int o_ = 32; o_ > 0; o_ >>= 1) {
        pos_min = min(pos_min, __shfl_xor(pos_min, o_, 64));
        lo_max = max(lo_max, __shfl_xor(lo_max, o_, 64));
    }

#pragma unroll
    for (int st = 0; st < STREAM_STAGES - 1; ++st) STREAM_ISSUE(st)
    for (int j = 0; j < n_mine; ++j) {
        wait_vmcnt<W_LOADS * (STREAM_STAGES - 2)>();     // tile j is there
        STREAM_ISSUE(j + STREAM_STAGES - 1)              // into the place of tile j-1, whose fragments are in registers
        const int kt = kbeg + (wave + j * STREAM_WAVES) * 32;
        const uint4* Ks = ring + (j % STREAM_STAGES) * W_STAGE;
        const uint4* Vs = Ks + NKC;
        uint4 kf[KD], vf[2][DB];
#pragma unroll
        for (int kd = 0; kd < KD; ++kd) {
            const int c = 2 * kd + lg;
            kf[kd] = Ks[key_off * KSTR + (CK_POW2 ? (c ^ (key_off & (CK - 1))) : c)];
        }
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
            for (int d = 0; d < DB; ++d) vf[jj][d] = Vs[(d * 32 + lr) * 4 + ((2 * jj + lg) ^ ((lr >> 2) & 3))];
        if (kt + 32 > seq_len) {               // the request's last tile: slots past its end hold old data
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
                const int k8 = kt + 16 * jj + 8 * lg;
                uint32_t mk[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    mk[e] = (k8 + 2 * e < seq_len ? 0x0000FFFFu : 0u) | (k8 + 2 * e + 1 < seq_len ? 0xFFFF0000u : 0u);
#pragma unroll
                for (int d = 0; d < DB; ++d) {
                    vf[jj][d].x &= mk[0]; vf[jj][d].y &= mk[1]; vf[jj][d].z &= mk[2]; vf[jj][d].w &= mk[3];
                }
            }
        }
        f32x16 s;
#pragma unroll
        for (int e = 0; e < 16; ++e) s[e] = 0.f;
#pragma unroll
        for (int kd = 0; kd < KD; ++kd)
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(kf[kd]), qf[kd], s, 0, 0, 0);
        float p[16];
        float corr;
        ATTN_SOFTMAX_STEP(kt, kend)
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
            uint4 pk = make_uint4(pack2(p[8 * jj + 0], p[8 * jj + 1]), pack2(p[8 * jj + 2], p[8 * jj + 3]),
                                  pack2(p[8 * jj + 4], p[8 * jj + 5]), pack2(p[8 * jj + 6], p[8 * jj + 7]));
            const bf16x8 pf = as_bf16x8(pk);
#pragma unroll
            for (int d = 0; d < DB; ++d)
                o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf16x8(vf[jj][d]), pf, o[d], 0, 0, 0);
        }
    }
#undef STREAM_ISSUE
    wait_vmcnt<0>();                                     // the trailing copies of zeros
    l += __shfl_xor(l, 32, 64);                          // the row's sum from its two lanes
    __syncthreads();                                     // the rings are free

    // ---- combine the waves: sum_w 2^(m_w - max) O_w over sum_w 2^(m_w - max) l_w
    float* mo = reinterpret_cast<float*>(lds);           // [waves][ROWS][MERGE_STRIDE] unnormalised outputs
    float* mml = mo + STREAM_WAVES * ROWS * MERGE_STRIDE; // [waves][ROWS][2]
    if (row_ok) {
        float* dst = mo + (wave * ROWS + lr) * MERGE_STRIDE;
#pragma unroll
        for (int d = 0; d < DB; ++d)
#pragma unroll
            for (int e4 = 0; e4 < 4; ++e4) {
                const int dd = d * 32 + e4 * 8 + lg * 4;
                if (dd < HD)
                    *reinterpret_cast<float4*>(dst + dd) = make_float4(o[d][e4 * 4 + 0], o[d][e4 * 4 + 1],
                                                                       o[d][e4 * 4 + 2], o[d][e4 * 4 + 3]);
            }
        if (lg == 0) {
            mml[(wave * ROWS + lr) * 2] = m;
            mml[(wave * ROWS + lr) * 2 + 1] = l;
        }
    }
    __syncthreads();
    const int rows_left = q_len * G - row0;
    const int n_rows = rows_left < ROWS ? rows_left : ROWS;
    for (int idx = tid; idx < n_rows * (HD / 4); idx += 64 * STREAM_WAVES) {
        const int r = idx / (HD / 4), d4 = (idx - r * (HD / 4)) * 4;
        float mx = -INFINITY;
#pragma unroll
        for (int w = 0; w < STREAM_WAVES; ++w) mx = fmaxf(mx, mml[(w * ROWS + r) * 2]);
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        float lsum = 0.f;
#pragma unroll
        for (int w = 0; w < STREAM_WAVES; ++w) {
            const float mw = mml[(w * ROWS + r) * 2], lw = mml[(w * ROWS + r) * 2 + 1];
            const float f = lw > 0.f ? __builtin_amdgcn_exp2f(mw - mx) : 0.f;
            const float4 v = *reinterpret_cast<const float4*>(mo + (w * ROWS + r) * MERGE_STRIDE + d4);
            acc.x += f * v.x; acc.y += f * v.y; acc.z += f * v.z; acc.w += f * v.w;
            lsum += f * lw;
        }
        const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
        const int rr = row0 + r, tk = rr / G, hh = kvh * G + (rr - tk * G);
        if (slot < 0) {
            bf16_t* op = a.out + ((size_t)(q0 + tk) * a.H + hh) * HD + d4;
            *reinterpret_cast<uint2*>(op) = make_uint2(pack2(acc.x * inv, acc.y * inv), pack2(acc.z * inv, acc.w * inv));
        } else {
            float* po = a.part_o + (((size_t)slot * a.Hk + kvh) * ROWS + r) * HD + d4;
            *reinterpret_cast<float4*>(po) = make_float4(acc.x * inv, acc.y * inv, acc.z * inv, acc.w * inv);
            if (d4 == 0) {
                float* pm = a.part_ml + (((size_t)slot * a.Hk + kvh) * ROWS + r) * 2;
                pm[0] = mx;
                pm[1] = lsum;
            }
        }
    }
}

// One merge job: {req, row0, first_slot, n_slots, slot_stride, q0, q_len}.  Slot s holds the normalised output of
// its keys with their maximum m_s (in units of log2) and sum l_s; the whole is
// sum_s w_s O_s / sum_s w_s with w_s = l_s * 2^(m_s - max m).
struct MergeArgs {
    const int* jobs;        // [n_jobs, JOB_INTS]
    const int* cu_q;
    const float* part_o;
    const float* part_ml;
    bf16_t* out;
    int H, Hk;
};

__global__ __launch_bounds__(256) void k_attn_merge(MergeArgs a) {
    const int* job = a.jobs + (size_t)blockIdx.x * JOB_INTS;
    const int row0 = job[1], s0 = job[2], ns = job[3], stride = job[4];
    const int kvh = blockIdx.y;
    const int G = a.H / a.Hk;
    const int q0 = job[5], q_len = job[6];          // (with the job: one dependent read less before the partial results)
    const int n_rows = (q_len * G - row0) < ROWS ? (q_len * G - row0) : ROWS;      // rows of this block that exist
    for (int idx = threadIdx.x; idx < n_rows * (HD / 4); idx += 256) {
        const int r = idx / (HD / 4), d4 = (idx % (HD / 4)) * 4;
        const int rho = row0 + r;
        const int tok = rho / G, hg = rho - tok * G;
        const float* ml = a.part_ml + (((size_t)s0 * a.Hk + kvh) * ROWS + r) * 2;
        const float* po = a.part_o + (((size_t)s0 * a.Hk + kvh) * ROWS + r) * HD + d4;
        const size_t ml_step = (size_t)stride * a.Hk * ROWS * 2, po_step = (size_t)stride * a.Hk * ROWS * HD;
        // 16 slots at a time, all their loads on their way before the first is used (a thread that
        // took the maxima first and then the outputs, four loads at a time, waited out eight memory
        // latencies for the 14 slots of a lone request: 8 us, as long as the attention itself)
        constexpr int MS = 16;
        float mx = -INFINITY;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        float wsum = 0.f;
        for (int sb = 0; sb < ns; sb += MS) {
            float2 mlv[MS];
            float4 pv[MS];
#pragma unroll
            for (int u = 0; u < MS; ++u) {
                const int sc = sb + u < ns ? sb + u : sb;
                mlv[u] = *reinterpret_cast<const float2*>(ml + sc * ml_step);
                pv[u] = *reinterpret_cast<const float4*>(po + sc * po_step);
            }
            float cm = mx;
#pragma unroll
            for (int u = 0; u < MS; ++u)
                if (sb + u < ns) cm = fmaxf(cm, mlv[u].x);
            const float resc = mx == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mx - cm);   // (1 while there is one group only)
            acc.x *= resc; acc.y *= resc; acc.z *= resc; acc.w *= resc;
            wsum *= resc;
            mx = cm;
#pragma unroll
            for (int u = 0; u < MS; ++u) {
                const float w = (sb + u < ns && mlv[u].y > 0.f) ? mlv[u].y * __builtin_amdgcn_exp2f(mlv[u].x - mx) : 0.f;
                acc.x += w * pv[u].x; acc.y += w * pv[u].y; acc.z += w * pv[u].z; acc.w += w * pv[u].w;
                wsum += w;
            }
        }
        const float inv = wsum > 0.f ? 1.0f / wsum : 0.f;
        bf16_t* op = a.out + ((size_t)(q0 + tok) * a.H + kvh * G + hg) * HD + d4;
        *reinterpret_cast<uint2*>(op) = make_uint2(pack2(acc.x * inv, acc.y * inv), pack2(acc.z * inv, acc.w * inv));
    }
}

extern "C" int xr_attn_head_dim() { return HD; }

extern "C" int xr_attention_mfma(void* out, const void* q, const void* k_cache, const void* v_cache,
                                 const int* items, int n_items, int n_cta_items, const int* jobs, int n_jobs,
                                 const int* cu_q,
                                 const int* starts, const int* block_table, int table_stride, float* part_o,
                                 float* part_ml, int H, int Hk, int D, int page_size, float scale, int window,
                                 hipStream_t stream) {
    XR_REQUIRE(D == HD, "attention: this library is compiled for head size %d, got %d", HD, D);
    XR_REQUIRE(H > 0 && Hk > 0 && H % Hk == 0, "attention: %d query heads are not a multiple of %d key/value heads", H, Hk);
    int shift = ilog2_exact(page_size);
    XR_REQUIRE(shift >= 4, "attention: the MFMA kernel needs a page size that is a power of two of at least 16, got %d", page_size);
    XR_REQUIRE(window >= 0, "attention: window %d is negative", window);
    XR_REQUIRE(n_items >= 0 && n_jobs >= 0 && n_cta_items >= 0, "attention: negative work counts");
    XR_REQUIRE((long long)n_cta_items * Hk < (1LL << 31) && (long long)n_items * Hk < (1LL << 31), "attention: %d items of %d key/value heads are more workgroups than a launch takes", n_items + n_cta_items, Hk);
    XR_REQUIRE(n_cta_items == 0 || page_size >= 32, "attention: 128-row items need pages of at least 32 positions, got %d", page_size);
    XR_REQUIRE(n_jobs == 0 || (part_o && part_ml && jobs), "attention: split work without partial buffers");
    if (n_items + n_cta_items == 0) return XR_OK;
    AttnArgs a;
    a.q = (const bf16_t*)q; a.kc = (const bf16_t*)k_cache; a.vc = (const bf16_t*)v_cache; a.out = (bf16_t*)out;
    // the list begins with the items of the workgroup kernel
    a.cta_items = items; a.n_cta_items = n_cta_items; a.items = items + (size_t)n_cta_items * ITEM_INTS; a.cu_q = cu_q; a.starts = starts; a.block_table = block_table; a.table_stride = table_stride;
    a.part_o = part_o; a.part_ml = part_ml; a.n_items = n_items; a.H = H; a.Hk = Hk;
    a.page_shift = shift; a.page_mask = page_size - 1; a.page_size = page_size; a.scale = scale; a.window = window;
    if (n_cta_items > 0) {
        constexpr int smem = CtaShape::LDS_BYTES;
        static bool attr_set = false;
        if (!attr_set) {
            hipError_t e = hipFuncSetAttribute((const void*)k_attn_cta, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
            if (e != hipSuccess) (void)hipGetLastError();     // or the next launch's check would report this refusal
            XR_REQUIRE(e == hipSuccess, "attention: %d bytes of LDS refused: %s", smem, hipGetErrorString(e));
            attr_set = true;
        }
        k_attn_cta<<<dim3((unsigned)n_cta_items * (unsigned)Hk), CtaShape::THREADS, smem, stream>>>(a);
        XR_CHECK_LAUNCH("attention_cta");
    }
    if (n_items > 0) {
        static bool attr_set = false;
        if (!attr_set) {
            hipError_t e = hipFuncSetAttribute((const void*)k_attn_stream, hipFuncAttributeMaxDynamicSharedMemorySize,
                                               STREAM_LDS_BYTES);
            if (e != hipSuccess) (void)hipGetLastError();
            XR_REQUIRE(e == hipSuccess, "attention: %d bytes of LDS refused: %s", STREAM_LDS_BYTES, hipGetErrorString(e));
            attr_set = true;
        }
        k_attn_stream<<<dim3((unsigned)n_items * (unsigned)Hk), 64 * STREAM_WAVES, STREAM_LDS_BYTES, stream>>>(a);
        XR_CHECK_LAUNCH("attention_stream");
    }
    if (n_jobs > 0) {
        MergeArgs mg;
        mg.jobs = jobs; mg.cu_q = cu_q; mg.part_o = part_o; mg.part_ml = part_ml; mg.out = (bf16_t*)out;
        mg.H = H; mg.Hk = Hk;
        k_attn_merge<<<dim3(n_jobs, Hk), 256, 0, stream>>>(mg);
        XR_CHECK_LAUNCH("attention_merge");
    }
    return XR_OK;
}
