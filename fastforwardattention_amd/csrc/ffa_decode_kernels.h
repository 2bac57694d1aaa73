// gfx950 (MI355X, wave64) decode-step kernels of the FastForwardAttention engine, as templates
// over the element type.  Included by one translation unit per element type
// (ffa_decode_f16.hip, ffa_decode_bf16.hip, ffa_decode_f32.hip), which are compiled in parallel.
//
// Data layout in HBM (fixed by the reference, attention.cu:1556-1609):
//   k_cache [B,H,Dh/x,Lmax,x], x = 16/sizeof(T): for one (b,h) and one 16-byte chunk c of
//     the head dimension, the keys are consecutive 16-byte records.  A wavefront whose
//     lane l owns key (tile*64 + l) therefore reads 64 x 16 B = 1 KiB contiguous per
//     load instruction, and a key's whole dot product stays inside one lane.
//   v_cache [B,H,Lmax,Dh]: a row is Dh*sizeof(T) bytes = LPR 16-byte chunks.  Lane l owns
//     chunk (l % LPR) of row (l / LPR) of each group of RPI = 64/LPR consecutive rows, so
//     a load instruction again covers 1 KiB contiguous.
// A 64-key tile is NCH = Dh/x load instructions for K and LPR (= NCH rounded up to a power of
// two; Dh = 80 has 10 or 20 chunks on 16 or 32 lanes) for V.  The probabilities
// computed in the K mapping (one key per lane) reach the V mapping (one row per LPR lanes)
// through a 256-byte LDS stage per wave.
//
// The new token (attention.cu:856-914, :1227-1256) never travels through the tile loops.  Tiles
// cover the cached keys 0 .. tlen-1 only; one wave per (batch, head) pair -- the "token wave" --
// holds the new q, k, v in registers, applies the optional bias and rotary embedding to them,
// folds the new key's score and value into its running softmax state like one more tile of a
// single key, and appends k, v at slot tlen of the caches.  Lanes of a tile that lie beyond the
// last cached key re-read that last key (valid memory, finite values) with weight 0.
//
// Decode kernels (the two-pass pair ffa_scores_kernel / ffa_pruned_pv_kernel is described
// where it is defined):
//   ffa_decode_split_kernel  p == 0.  Grid (b,h,split); every wave walks 64-key tiles with
//     an online softmax, the waves of a workgroup merge (m, l, acc) in LDS, workgroups
//     write partials and the last one to arrive (device-scope counter) merges them.
//   ffa_decode_wg_kernel     any p.  One workgroup per (b,h), all scores staged in LDS so
//     that the global max and sum exist before any V row is touched, which the pruning
//     rule needs (threshold = p * inv_sum, attention.cu:1184-1191).
#pragma once

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include <mutex>
#include <type_traits>

#include "ffa_c_api.h"
#include "ffa_device.h"
#include "ffa_host.h"

namespace ffa {

// What a workgroup needs before it can issue its first cache load travels as leading scalar
// kernel arguments, which the hardware can place in registers while it launches the wave
// (kernel-argument preloading); everything else is fetched from the argument block in memory.
#define HOT_PARAMS_DECL                                                                                      \
    void *hot_k_cache, void *hot_v_cache, const int *hot_seq_lengths, int hot_Lmax, int hot_t, int hot_n_whole, \
        int hot_n_splits, unsigned hot_split_magic, int hot_tiles_per_split, const void *hot_q
#define HOT_PARAMS_USE                                                                                            \
    hot_k_cache, hot_v_cache, hot_seq_lengths, hot_Lmax, hot_t, hot_n_whole, hot_n_splits, hot_split_magic, \
        hot_tiles_per_split, hot_q
#define HOT_PARAMS_OF(P)                                                                                  \
    (P).k_cache, (P).v_cache, (P).seq_lengths, (P).Lmax, (P).t, (P).n_whole, (P).n_splits, (P).split_magic, \
        (P).tiles_per_split, (P).q
__device__ __forceinline__ DecodeParams with_hot_params(const DecodeParams& rest, HOT_PARAMS_DECL) {
    DecodeParams P = rest;
    P.k_cache = hot_k_cache; P.v_cache = hot_v_cache; P.seq_lengths = hot_seq_lengths;
    P.Lmax = hot_Lmax; P.t = hot_t; P.n_whole = hot_n_whole; P.n_splits = hot_n_splits;
    P.split_magic = hot_split_magic; P.tiles_per_split = hot_tiles_per_split; P.q = hot_q;
    return P;
}

// The same for the second kernel of the two-pass path, whose first loads are the pieces' (max, sum)
// and the scores.
#define PV_HOT_PARAMS_DECL                                                                                   \
    float *hot_scores, float *hot_ml, void *hot_v_cache, const int *hot_seq_lengths, int hot_score_stride, \
        int hot_Lmax, int hot_t, int hot_n_splits, unsigned hot_split_magic, int hot_tiles_per_split
#define PV_HOT_PARAMS_USE                                                                                \
    hot_scores, hot_ml, hot_v_cache, hot_seq_lengths, hot_score_stride, hot_Lmax, hot_t, hot_n_splits, \
        hot_split_magic, hot_tiles_per_split
#define PV_HOT_PARAMS_OF(P)                                                                              \
    (P).ws_scores, (P).ws_ml, (P).v_cache, (P).seq_lengths, (P).score_stride, (P).Lmax, (P).t, (P).n_splits, \
        (P).split_magic, (P).tiles_per_split
__device__ __forceinline__ DecodeParams with_pv_hot_params(const DecodeParams& rest, PV_HOT_PARAMS_DECL) {
    DecodeParams P = rest;
    P.ws_scores = hot_scores; P.ws_ml = hot_ml; P.v_cache = hot_v_cache; P.seq_lengths = hot_seq_lengths;
    P.score_stride = hot_score_stride; P.Lmax = hot_Lmax; P.t = hot_t; P.n_splits = hot_n_splits;
    P.split_magic = hot_split_magic; P.tiles_per_split = hot_tiles_per_split;
    return P;
}

// Per-(b) bounds, attention.cu:805-817.  tlen = slot of the new token = number of cached
// keys; first = first unmasked key.  Values are clamped so that a bad seq_lengths entry
// can never produce an out-of-bounds access.
__device__ __forceinline__ void step_bounds(const DecodeParams& P, int b, int& tlen, int& first) {
    tlen = P.t;
    first = 0;
    if (P.seq_lengths != nullptr) {
        const int sl = P.seq_lengths[b];
        if (P.right_or_no_padding) tlen = min(max(sl, 0), P.t);
        else first = max(sl, 0);
    }
}

// (pair, piece) of a workgroup of a split launch: the first n_whole workgroups own one whole
// pair each, the others are n_splits pieces per pair.  The quotient by n_splits comes from a
// multiplication by the host's ceil(2^32 / n_splits) (exact for every workgroup index the
// planner admits): an integer division here would sit in front of every workgroup's first load.
// r / n_splits for r below 2^25 / n_splits (split_magic = 0 stands for n_splits = 1).
__device__ __forceinline__ unsigned pair_of(const DecodeParams& P, unsigned r) {
    const unsigned hi = __umulhi(r, P.split_magic);
    return P.split_magic == 0u ? r : hi;
}

// Branch-free on purpose: with a branch in front of them the compiler fetches the kernel
// arguments in two dependent batches, each a miss of the scalar cache right after a launch.
struct PieceOf {
    int bh, split, n_splits;
    __device__ __forceinline__ PieceOf(const DecodeParams& P, int wg) {
        const bool whole = wg < P.n_whole;
        const unsigned r = (unsigned)(wg - P.n_whole);
        const unsigned pair = pair_of(P, r);
        bh = whole ? wg : P.n_whole + (int)pair;
        split = whole ? 0 : (int)(r - pair * (unsigned)P.n_splits);
        n_splits = whole ? 1 : P.n_splits;
    }
};

// Order in which a workgroup walks its tiles [lo, hi): rotated by an offset that differs from
// workgroup to workgroup.  All workgroups of a launch run the same loop at the same pace over
// caches a fixed stride apart, so without the rotation their loads fall on the same memory
// channels at the same time whenever that stride folds badly onto the channel map (measured:
// 512 pairs x 8192 keys with rows of 8256 slots 166 -> 155 us for the loads alone, rows of
// 2048 slots at 1000 keys 20.0 -> 18.0 us; nothing lost at strides that were good already).
// The result does not depend on the order beyond the rounding of the running sums.
struct TileOrder {
    int lo, n, rot;
    __device__ __forceinline__ TileOrder(int lo_, int hi_, unsigned salt) : lo(lo_), n(max(hi_ - lo_, 0)), rot(0) {
        // A 16-bit hash scaled into [0, n): no integer division.
        rot = (int)((((salt * 2654435761u) >> 16) * (unsigned)n) >> 16);
    }
    // Tile at position idx of the walk, idx in [0, n).
    __device__ __forceinline__ int at(int idx) const {
        const int a = idx + rot;
        return lo + (a >= n ? a - n : a);
    }
};

// ---------------------------------------------------------------------------------------
// The new token.
template <typename T, int DH>
struct Geo {
    static constexpr int X = Elem<T>::X;      // elements per 16 B
    static constexpr int NCH = DH / X;        // 16-byte chunks per key / per V row
    // Lanes per V row: the chunk count rounded up to a power of two (Dh = 80: 10 chunks on
    // 16 lanes, the upper 6 repeat the last chunk and are never stored).
    static constexpr int LPR = NCH <= 8 ? 8 : NCH <= 16 ? 16 : NCH <= 32 ? 32 : 64;
    static constexpr int RPI = kWave / LPR;   // V rows per load instruction
    static constexpr int NVL = LPR;           // V load instructions per 64-key tile (= 64 / RPI)
    static constexpr int ROWW = LPR * X;      // accumulator floats per row group across the wave
    static constexpr int CG = NCH % 8 == 0 ? 8 : 10;  // K loads in flight per group
    static constexpr int VG = 8;                      // V loads in flight per group
    static constexpr bool Q_LDS = NCH > 16;   // q read from LDS when it would not fit SGPRs
    static constexpr int QREG = Q_LDS ? 1 : NCH;
    static_assert(DH % X == 0 && NCH >= 8 && NCH <= kWave && NCH % CG == 0 && NVL % VG == 0,
                  "unsupported head dim");
};

// Pairs of adjacent elements as raw bits (what a load leaves in registers) and widened to fp64
// (the arithmetic of the token transform).
template <typename T> struct PairBits { using type = uint32_t; };
template <> struct PairBits<float> { using type = uint2; };
__device__ __forceinline__ double2 widen_pair(uint32_t bits, uint16_t) {
    const half2_t h = __builtin_bit_cast(half2_t, bits);
    return make_double2((double)(float)h.x, (double)(float)h.y);
}
__device__ __forceinline__ double2 widen_pair(uint32_t bits, bf16_t) {
    return make_double2(bf16_to_float((uint16_t)(bits & 0xffffu)), bf16_to_float((uint16_t)(bits >> 16)));
}
__device__ __forceinline__ double2 widen_pair(uint2 bits, float) {
    return make_double2(__builtin_bit_cast(float, bits.x), __builtin_bit_cast(float, bits.y));
}
__device__ __forceinline__ void store_pair(uint16_t* p, float2 v) {
    half2_t h = {(_Float16)v.x, (_Float16)v.y};
    *reinterpret_cast<half2_t*>(p) = h;
}
__device__ __forceinline__ void store_pair(float* p, float2 v) { p[0] = v.x; p[1] = v.y; }
__device__ __forceinline__ void store_pair(bf16_t* p, float2 v) {
    p[0].bits = float_to_bf16(v.x);
    p[1].bits = float_to_bf16(v.y);
}

// Bias and rotary embedding of the new token (attention.cu:856-882; the pair rotation and its
// angle are decoder_masked_multihead_attention_utils.h:1137-1160): q += q_bias, k += k_bias,
// v += v_bias, then the pairs (2z, 2z+1) below rotary_dim of q and k are rotated by
// pos / base^(2z / rotary_dim).  One lane per pair (two for Dh = 256).
// Arithmetic in fp64 (the angle reaches hundreds of radians, where an fp32 angle is only good to
// 1e-5 and two math libraries no longer agree on its cosine), the result rounded to fp32 and
// then once to T.  The reference does the same sums and products in fp32 (utils.h:1137-1156)
// after adding the bias in T (attention.cu:870-873).
//
// One wave of a workgroup -- the publisher -- computes the angles (an fp64 exp2, sine and cosine
// per pair: some hundreds of instructions) and leaves their cosines and sines in LDS, together
// with the q bias, ahead of a workgroup barrier.  They depend on the position alone, so the
// barrier is reached while the first cache tiles are still on their way.  Every wave that needs
// q' then rotates its own copy of q (a dozen fp64 instructions), which it loaded as the very
// first thing it did: the address of q is among the preloaded kernel arguments, so that load
// leaves before the argument block has been read and returns before the wave's first tile.  The
// wave that appends the token does the same for k and v.
template <typename T, int DH>
struct RawToken {
    static constexpr int N = (DH / 2 + kWave - 1) / kWave;  // pairs per lane
    using Bits = typename PairBits<T>::type;
    Bits q[N], k[N], v[N], qb[N], kb[N], vb[N];
    double sn[N], cs[N];  // sine and cosine of the pair's angle (0 and 1 outside the rotary part)
};

// What the publisher leaves in LDS for the other waves of the workgroup.
template <typename T, int DH, bool XFORM>
struct alignas(16) AngleLds {
    double2 cs_sn[XFORM ? DH / 2 : 1];
    typename PairBits<T>::type q_bias[XFORM ? DH / 2 : 1];  // zero bits when there is none
};

template <typename T, int DH>
__device__ __forceinline__ typename PairBits<T>::type load_pair(const void* base, size_t off) {
    return *reinterpret_cast<const typename PairBits<T>::type*>(static_cast<const char*>(base) + off);
}

// First thing a wave does: its pairs of q.
template <typename T, int DH>
__device__ __forceinline__ void token_load_q(RawToken<T, DH>& r, const DecodeParams& P, int bh, int lane) {
#pragma unroll
    for (int i = 0; i < RawToken<T, DH>::N; ++i) {
        const int z = min(lane + i * kWave, DH / 2 - 1);
        r.q[i] = load_pair<T, DH>(P.q, ((size_t)bh * DH + 2 * z) * sizeof(T));
    }
    __builtin_amdgcn_sched_barrier(0);
}

// The publisher's other loads: the q bias, and with `with_kv` k, v and their biases.
template <typename T, int DH>
__device__ __forceinline__ void token_load_rest(RawToken<T, DH>& r, const DecodeParams& P, int bh, bool with_kv, int lane) {
    using R = RawToken<T, DH>;
    // Everything the transform reads from the argument block, asked for in one batch (the
    // compiler otherwise fetches each field in front of its first use: three round trips in a row).
    asm volatile("" ::"s"(P.H), "s"(P.k), "s"(P.v), "s"(P.q_bias), "s"(P.k_bias), "s"(P.v_bias), "s"(P.rotary_dim),
                 "s"(P.rotary_coef));
    // Every load below is issued whatever is present (an absent operand reads q once more and
    // the value is never looked at): with a fixed number of loads in flight each wait is for the
    // operand it names, not for the last load issued.
    const int h = (P.q_bias || P.k_bias || P.v_bias) ? bh % P.H : 0;  // a division: not in front of the angles for nothing
    const void* qb = P.q_bias ? P.q_bias : P.q;
    const void* kb = P.k_bias ? P.k_bias : P.q;
    const void* vb = P.v_bias ? P.v_bias : P.q;
    const void* k = with_kv ? P.k : P.q;
    const void* v = with_kv ? P.v : P.q;
#pragma unroll
    for (int i = 0; i < R::N; ++i) {
        const int z = min(lane + i * kWave, DH / 2 - 1);
        const size_t e = ((size_t)bh * DH + 2 * z) * sizeof(T), eb = ((size_t)h * DH + 2 * z) * sizeof(T);
        r.qb[i] = load_pair<T, DH>(qb, P.q_bias ? eb : e);
        r.k[i] = load_pair<T, DH>(k, e);
        r.v[i] = load_pair<T, DH>(v, e);
        r.kb[i] = load_pair<T, DH>(kb, P.k_bias ? eb : e);
        r.vb[i] = load_pair<T, DH>(vb, P.v_bias ? eb : e);
    }
    __builtin_amdgcn_sched_barrier(0);
}

// Sine and cosine of an fp64 angle 0 <= a < 2^31, to about one ulp: the quadrant from
// k = rint(a * 2/pi), the remainder by two fused multiply-adds against pi/2 split in two (the first
// is exact: a and k * P1 cancel to a multiple of 2^-52 below 2), then the classic minimax
// polynomials on [-pi/4, pi/4].  Some fifty fp64 instructions without a branch, where the library's
// sincos spends several hundred (its large-argument path, taken by some lanes of every wave, and
// the divergence around it).
__device__ __forceinline__ void sincos_reduced(double a, double* sn, double* cs) {
    const double k = __builtin_rint(a * 0.63661977236758138);          // 2 / pi
    double r = __builtin_fma(-k, 1.5707963267948966, a);               // pi / 2, rounded
    r = __builtin_fma(-k, 6.123233995736766e-17, r);                   // pi / 2 - the above
    const double z = r * r;
    double ps = 1.58969099521155010221e-10;
    ps = __builtin_fma(ps, z, -2.50507602534068634195e-08);
    ps = __builtin_fma(ps, z, 2.75573137070700676789e-06);
    ps = __builtin_fma(ps, z, -1.98412698298579493134e-04);
    ps = __builtin_fma(ps, z, 8.33333333332248946124e-03);
    ps = __builtin_fma(ps, z, -1.66666666666666324348e-01);
    const double s0 = __builtin_fma(r * z, ps, r);
    double pc = -1.13596475577881948265e-11;
    pc = __builtin_fma(pc, z, 2.08757232129817482790e-09);
    pc = __builtin_fma(pc, z, -2.75573143513906633035e-07);
    pc = __builtin_fma(pc, z, 2.48015872894767294178e-05);
    pc = __builtin_fma(pc, z, -1.38888888888741095749e-03);
    pc = __builtin_fma(pc, z, 4.16666666666666019037e-02);
    const double c0 = __builtin_fma(z * z, pc, __builtin_fma(-0.5, z, 1.0));
    const int quadrant = (int)(long long)k & 3;
    const double s1 = (quadrant & 1) ? c0 : s0, c1 = (quadrant & 1) ? s0 : c0;
    *sn = (quadrant & 2) ? -s1 : s1;
    *cs = ((quadrant + 1) & 2) ? -c1 : c1;
}

// Keeps the compiler from looking at a loaded pair before this point.
__device__ __forceinline__ void pin_pair(uint32_t& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void pin_pair(uint2& x) { asm volatile("" : "+v"(x.x), "+v"(x.y)); }

// The angles of the lane's pairs.  They depend on the position alone.  The empty asm statements
// here and in pin_pair are volatile, hence kept in sequence: the angles are complete before the
// first raw pair is looked at.  Left to itself the compiler waits for the loads first and starts
// on the exp2, sine and cosine afterwards.
template <typename T, int DH>
__device__ __forceinline__ void token_angles(RawToken<T, DH>& r, const DecodeParams& P, int pos, int lane) {
    using R = RawToken<T, DH>;
#pragma unroll
    for (int i = 0; i < R::N; ++i) {
        const int z = lane + i * kWave;
        r.sn[i] = 0.0;
        r.cs[i] = 1.0;
        if (z < DH / 2 && 2 * z < P.rotary_dim) {
            const double angle = (double)pos * exp2((double)z * P.rotary_coef);
            sincos_reduced(angle, &r.sn[i], &r.cs[i]);
        }
        asm volatile("" : "+v"(r.sn[i]), "+v"(r.cs[i]));
    }
}

// x (+ bias, when there is one), rotated where `rotate`, rounded to fp32 and then once to T, into
// LDS in element order.
template <typename T, int DH>
__device__ __forceinline__ void token_finish(RawToken<T, DH>& r, const DecodeParams& P, typename RawToken<T, DH>::Bits (&x)[RawToken<T, DH>::N],
                                             typename RawToken<T, DH>::Bits (&bias)[RawToken<T, DH>::N], bool has_bias, bool rotate,
                                             T* dst, int lane) {
    using R = RawToken<T, DH>;
    double2 a[R::N];
#pragma unroll
    for (int i = 0; i < R::N; ++i) {
        pin_pair(x[i]);
        a[i] = widen_pair(x[i], T{});
    }
    if (has_bias) {
#pragma unroll
        for (int i = 0; i < R::N; ++i) {
            pin_pair(bias[i]);
            const double2 ab = widen_pair(bias[i], T{});
            a[i].x += ab.x;
            a[i].y += ab.y;
        }
    }
#pragma unroll
    for (int i = 0; i < R::N; ++i) {
        const int z = lane + i * kWave;
        if (z >= DH / 2) break;
        double2 w = a[i];
        if (rotate && 2 * z < P.rotary_dim) w = make_double2(r.cs[i] * w.x - r.sn[i] * w.y, r.cs[i] * w.y + r.sn[i] * w.x);
        store_pair(dst + 2 * z, make_float2((float)w.x, (float)w.y));
    }
}

// LDS of a workgroup that may transform the token: q' for every wave, k' and v' for the token wave.
template <typename T, int DH>
struct alignas(16) TokenLds {
    uint4 q[Geo<T, DH>::NCH];
    uint4 k[Geo<T, DH>::NCH];
    uint4 v[Geo<T, DH>::NCH];
};

// The transform of a workgroup, first half, called by every wave as the first thing it does
// (callers then issue the loads of their first tile, then call xform_end).  `needs_q`: the wave
// will read q' (tile waves, and the wave that appends the token).  `publisher`: the one wave that
// computes the angles; `with_kv`: it also transforms k and v (it holds the token).
template <typename T, int DH>
__device__ __forceinline__ void xform_begin(RawToken<T, DH>& r, const DecodeParams& P, int bh, int tlen, int first,
                                            bool needs_q, bool publisher, bool with_kv, AngleLds<T, DH, true>& s_ang,
                                            int lane) {
    using R = RawToken<T, DH>;
    if (needs_q) token_load_q<T, DH>(r, P, bh, lane);
    if (publisher) {
        token_load_rest<T, DH>(r, P, bh, with_kv, lane);
        token_angles<T, DH>(r, P, max(tlen - first, 0), lane);
        const bool has_bias = P.q_bias != nullptr;
#pragma unroll
        for (int i = 0; i < R::N; ++i) {
            const int z = lane + i * kWave;
            if (z >= DH / 2) break;
            s_ang.cs_sn[z] = make_double2(r.cs[i], r.sn[i]);
            typename R::Bits bits{};
            if (has_bias) {
                pin_pair(r.qb[i]);
                bits = r.qb[i];
            }
            s_ang.q_bias[z] = bits;
        }
    }
}

// Second half: the barrier behind which the angles wait, then q' (and k', v') into LDS.  Every
// wave that needs q' writes the same values to the same place; a wave reads back only after its
// own stores.
template <typename T, int DH>
__device__ __forceinline__ void xform_end(RawToken<T, DH>& r, const DecodeParams& P, bool needs_q, bool publisher,
                                          bool with_kv, TokenLds<T, DH>& s, AngleLds<T, DH, true>& s_ang, int lane) {
    using R = RawToken<T, DH>;
    __syncthreads();
    if (needs_q) {
#pragma unroll
        for (int i = 0; i < R::N; ++i) {
            const int z = min(lane + i * kWave, DH / 2 - 1);
            const double2 a = s_ang.cs_sn[z];
            r.cs[i] = a.x;
            r.sn[i] = a.y;
            r.qb[i] = s_ang.q_bias[z];
        }
        token_finish<T, DH>(r, P, r.q, r.qb, true, true, reinterpret_cast<T*>(s.q), lane);
    }
    if (publisher && with_kv) {
        token_finish<T, DH>(r, P, r.k, r.kb, P.k_bias != nullptr, true, reinterpret_cast<T*>(s.k), lane);
        token_finish<T, DH>(r, P, r.v, r.vb, P.v_bias != nullptr, false, reinterpret_cast<T*>(s.v), lane);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// q of the pair without a transform, ready for the dot products of the calling wave.  Returns
// true when the dot products are to read q from LDS (s.q): wide heads.  Otherwise q sits in
// SGPR-resident registers (q_reg), loaded straight from memory through scalar loads.  The two
// sources of q are kept apart all the way into the tile code: a register array fed from two
// places costs the plain path its wide scalar loads.
template <typename T, int DH>
__device__ __forceinline__ bool setup_q(const DecodeParams& P, int bh, TokenLds<T, DH>& s, uint4 (&q_reg)[Geo<T, DH>::QREG],
                                        int lane) {
    using G = Geo<T, DH>;
    const uint4* qg = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(P.q) + (size_t)bh * DH * sizeof(T));
    if constexpr (G::Q_LDS) {
        // Every wave stores the same values; a wave reads back only after its own stores.
        if (lane < G::NCH) s.q[lane] = qg[lane];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        return true;
    } else {
#pragma unroll
        for (int c = 0; c < G::NCH; ++c) q_reg[c] = qg[c];
        return false;
    }
}

// The new token in the token wave's registers: lane c < NCH holds 16-byte chunk c of q, k, v
// (after the transform, if any).
struct TokenRegs {
    uint4 q, k, v;
};
template <typename T, int DH, bool XFORM>
__device__ __forceinline__ TokenRegs token_load(const DecodeParams& P, int bh, const TokenLds<T, DH>& s, int lane) {
    constexpr int NCH = Geo<T, DH>::NCH;
    const int c = lane < NCH ? lane : 0;
    TokenRegs r;
    if constexpr (XFORM) {  // the transform has put them in LDS
        r.q = s.q[c];
        r.k = s.k[c];
        r.v = s.v[c];
    } else {
        const size_t off = (size_t)bh * DH * sizeof(T) + (size_t)c * 16;
        r.q = ld16(reinterpret_cast<const char*>(P.q) + off);
        r.k = ld16(reinterpret_cast<const char*>(P.k) + off);
        r.v = ld16(reinterpret_cast<const char*>(P.v) + off);
    }
    return r;
}
// Raw (unscaled) score of the new key: q.k over the NCH lanes that hold chunks.
template <typename T, int DH>
__device__ __forceinline__ float token_score(const TokenRegs& r, int lane) {
    const float part = lane < Geo<T, DH>::NCH ? dot_chunk(r.k, r.q, 0.f, T{}) : 0.f;
    return wave_sum(part);
}
// Append k, v at slot tlen of the pair's own caches (attention.cu:901-914, :1246).
template <typename T, int DH>
__device__ __forceinline__ void token_store(const TokenRegs& r, char* kc_bh, char* vc_bh, int tlen, int Lmax, int lane,
                                            bool through = false) {
    constexpr int NCH = Geo<T, DH>::NCH;
    if (lane < NCH) {
        char* kp = kc_bh + ((size_t)lane * Lmax + tlen) * 16;
        char* vp = vc_bh + ((size_t)tlen * NCH + lane) * 16;
        if (through) {
            st16_through(kp, r.k);
            st16_through(vp, r.v);
        } else {
            st16(kp, r.k);
            st16(vp, r.v);
        }
    }
}

// Beam-search indirection (attention.cu:1003, :1024-1033, :1143, :1195-1202).  Sample b is beam
// b % beam_width of group b / beam_width; its cached key i is read from the caches of the
// group's beam cache_indir[b][i], while the new token is always appended to the sample's own
// caches.  With BEAM = false every method folds to the sample's own caches at compile time.
template <bool BEAM>
struct BeamRows {
    const int* idx = nullptr;  // this sample's row of cache_indir
    int last = 0;              // beam_width - 1
    int own = 0;               // this sample's beam inside its group
    size_t sample_bytes = 0;   // bytes between consecutive samples of a cache
    char* k_group = nullptr;   // head h of the group's first beam
    char* v_group = nullptr;

    __device__ __forceinline__ BeamRows(const DecodeParams& P, int b, int bh, size_t head_bytes) {
        if constexpr (BEAM) {
            own = b % P.beam_width;
            const int first_beam = b - own;
            const size_t off = ((size_t)first_beam * P.H + (bh - b * P.H)) * head_bytes;
            idx = P.cache_indir + (size_t)b * P.Lmax;
            last = P.beam_width - 1;
            sample_bytes = (size_t)P.H * head_bytes;
            k_group = reinterpret_cast<char*>(P.k_cache) + off;
            v_group = reinterpret_cast<char*>(P.v_cache) + off;
        } else {
            k_group = reinterpret_cast<char*>(P.k_cache) + (size_t)bh * head_bytes;
            v_group = reinterpret_cast<char*>(P.v_cache) + (size_t)bh * head_bytes;
        }
    }
    // Source beam of cached key `key` (callers pass one key per lane: a coalesced 4-byte load).
    // A table entry outside [0, beam_width) is clamped, so that it can never address memory
    // outside the group; positions that hold no cached key give 0.
    __device__ __forceinline__ int beam(int key, int tlen) const {
        if constexpr (BEAM) return (key >= 0 && key < tlen) ? min(max(idx[key], 0), last) : 0;
        else return 0;
    }
    __device__ __forceinline__ const char* k_of(int beam) const {
        if constexpr (BEAM) return k_group + (size_t)beam * sample_bytes;
        else return k_group;
    }
    __device__ __forceinline__ const char* v_of(int beam) const {
        if constexpr (BEAM) return v_group + (size_t)beam * sample_bytes;
        else return v_group;
    }
    // Row number of key `key` of beam `beam`, counted from v_group in V rows: what the survivor
    // queue stores.
    __device__ __forceinline__ int v_row(int beam, int key, int rows_per_sample) const {
        if constexpr (BEAM) return beam * rows_per_sample + key;
        else return key;
    }
    // The same for a row of the sample's own cache (the slot the new token was appended to).
    __device__ __forceinline__ int own_row(int key, int rows_per_sample) const {
        if constexpr (BEAM) return own * rows_per_sample + key;
        else return key;
    }
};

// ---------------------------------------------------------------------------------------
// One 64-key tile of q.K^T for the calling wave.  Lane l owns key tile*64+l; lanes beyond the
// last cached key re-read that key and are masked by the caller.
// load_k_group puts CG 16-byte loads in flight, dot_k_group consumes them.
template <int CG>
__device__ __forceinline__ void load_k_group(uint4 (&kv)[CG], const char* kp, size_t kstr, int g) {
#pragma unroll
    for (int c = 0; c < CG; ++c) kv[c] = ld16(kp + (size_t)(g * CG + c) * kstr);
}

template <typename T, int CG, bool Q_LDS>
__device__ __forceinline__ float dot_k_group(const uint4 (&kv)[CG], int g, const uint4* q_reg,
                                             const uint4* q_lds, float s) {
#pragma unroll
    for (int c = 0; c < CG; ++c) {
        uint4 qc;
        if constexpr (Q_LDS) qc = q_lds[g * CG + c];
        else qc = q_reg[g * CG + c];
        s = dot_chunk(kv[c], qc, s, T{});
    }
    return s;
}

// Whole-tile raw dot product (not yet scaled) of cached key `key` (already clamped to a cached
// key), NCH/CG groups, at most two groups of loads in flight.
template <typename T, int NCH, bool Q_LDS>
__device__ __forceinline__ float tile_qk(const char* k_base, int key, int Lmax, const uint4* q_reg,
                                         const uint4* q_lds) {
    const char* kp = k_base + (size_t)key * 16;
    const size_t kstr = (size_t)Lmax * 16;
    constexpr int CG = NCH % 8 == 0 ? 8 : 10;
    float s = 0.f;
#pragma unroll 2
    for (int g = 0; g < NCH / CG; ++g) {
        uint4 kv[CG];
        load_k_group<CG>(kv, kp, kstr, g);
        s = dot_k_group<T, CG, Q_LDS>(kv, g, q_reg, q_lds, s);
    }
    return s;
}

// LDS slot of key k's probability inside a wave's 64-float stage: the V mapping reads, for
// row group rg = lane/LPR, the NVL consecutive floats [rg*NVL, rg*NVL+NVL) = keys j*RPI+rg.
template <int NVL, int RPI>
__device__ __forceinline__ int stage_slot(int k) { return (k % RPI) * NVL + k / RPI; }

// Words exchanged between workgroups of one launch: device-scope relaxed atomics.
__device__ __forceinline__ void publish(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float acquire(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Waits until this lane's outstanding vector memory operations, published stores included,
// have been acknowledged.  A workgroup barrier alone does not: it orders the waves of one CU,
// not their stores on the way to memory.
__device__ __forceinline__ void wait_published() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ---------------------------------------------------------------------------------------
// Survivor queue of the pruning kernels.  A key that the rule drops must cost neither bytes
// nor instructions, so the keys that survive are compacted, per wave, into an LDS queue of
// two 64-entry blocks (weight + cache row each); a block is consumed as soon as it is full,
// by the same V mapping as an ordinary tile: every lane active, every load a surviving row.
// Entry n of the stream sits in block (n >> 6) & 1 at stage_slot(n & 63).  A cache row is a
// V row number counted from `v_base` (BeamRows::v_row / own_row).
struct SurvivorQueue {
    float* w;          // this wave's 128 weights
    int* row;          // this wave's 128 cache rows
    unsigned total;    // survivors pushed so far (wave-uniform)
};

// P.V over one queue block holding `count` >= 1 valid entries (64 unless it is the last one).
template <typename T, int DH>
__device__ __forceinline__ void pv_queue_block(float (&acc)[Elem<T>::X], const SurvivorQueue& q, int block,
                                               int count, const char* v_base, int lane) {
    using G = Geo<T, DH>;
    constexpr int NCH = G::NCH, LPR = G::LPR, RPI = G::RPI, NVL = G::NVL, VG = G::VG;
    const int rg = lane / LPR, dch = min(lane % LPR, NCH - 1);
    const float* pw = q.w + block * kWave + rg * NVL;
    const int* pr = q.row + block * kWave + rg * NVL;
    // Entry 0 of the block (always valid): what the entries past `count` re-read, with weight 0.
    const int row0 = q.row[block * kWave + stage_slot<NVL, RPI>(0)];
#pragma unroll 1
    for (int g = 0; g < NVL / VG; ++g) {
        uint4 vv[VG];
        float pj[VG];
#pragma unroll
        for (int j = 0; j < VG; ++j) {
            // Loads are unconditional (a load under a branch is waited for at the join, one
            // round trip per row).
            const int n = (g * VG + j) * RPI + rg;  // entry number inside the block
            const int r = n < count ? pr[g * VG + j] : row0;
            pj[j] = n < count ? pw[g * VG + j] : 0.f;
            vv[j] = ld16(v_base + ((size_t)r * NCH + dch) * 16);
        }
#pragma unroll
        for (int j = 0; j < VG; ++j) fma_chunk(acc, pj[j], vv[j], T{});
    }
}

// Push this lane's key (cache row `row`) if it survives; consumes a block when one fills up.
template <typename T, int DH>
__device__ __forceinline__ void queue_push(float (&acc)[Elem<T>::X], SurvivorQueue& q, bool keep, float weight,
                                           int row, const char* v_base, int lane) {
    using G = Geo<T, DH>;
    const unsigned long long mask = __builtin_amdgcn_ballot_w64(keep);
    const unsigned before =
        __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
    if (keep) {
        const unsigned n = q.total + before;
        const int slot = ((n >> 6) & 1) * kWave + stage_slot<G::NVL, G::RPI>(n & 63);
        q.w[slot] = weight;
        q.row[slot] = row;
    }
    const unsigned after = q.total + (unsigned)__builtin_popcountll(mask);
    __builtin_amdgcn_wave_barrier();
    if ((after >> 6) != (q.total >> 6))  // wave-uniform: a block has just been completed
        pv_queue_block<T, DH>(acc, q, (q.total >> 6) & 1, kWave, v_base, lane);
    q.total = after;
    __builtin_amdgcn_wave_barrier();
}

template <typename T, int DH>
__device__ __forceinline__ void queue_drain(float (&acc)[Elem<T>::X], SurvivorQueue& q, const char* v_base, int lane) {
    if (q.total & 63) pv_queue_block<T, DH>(acc, q, (q.total >> 6) & 1, q.total & 63, v_base, lane);
}

// ---------------------------------------------------------------------------------------
// The token wave of an online-softmax kernel.  The split kernels run NW tile waves plus this one
// extra wave per workgroup; in the workgroup that owns the pair's last piece it takes the new
// token -- loads q, k, v (with their transform, if any), appends k, v to the caches and enters the
// new key into the workgroup's merge as the running state of a "tile" of one key: max = its
// score, sum = 1, accumulator = v.  It walks no tiles, so none of this sits in front of, between
// or behind the cache loads of the tile waves.  In the other workgroups it only joins the merge
// with an empty state.  The two stores of the append are issued after the workgroup's merge
// barrier, when the tile waves have read all they will read: in the middle of the stream every
// write turns memory channels around under the reads (measured at 320 pairs x 1000 keys: 0.1 us
// per launch for 640 small stores).
template <typename T, int DH, bool XFORM>
__device__ __forceinline__ TokenRegs token_wave_state(const DecodeParams& P, int bh, int tlen, int first,
                                                      TokenLds<T, DH>& s_tok, float& m_run, float& l_run,
                                                      float (&acc)[Elem<T>::X], int lane) {
    constexpr int NCH = Geo<T, DH>::NCH;
    const TokenRegs tok = token_load<T, DH, XFORM>(P, bh, s_tok, lane);
    const float s = token_score<T, DH>(tok, lane);
    if (tlen >= first) {  // else the whole sample is masked up to and including the new slot
        m_run = s * P.scale_log2e;
        l_run = lane == 0 ? 1.f : 0.f;  // per-lane partial sums: the key counts once
        // Lane c < NCH holds chunk c of v: the same lanes that hold chunk c of row group 0 of the acc.
        if (lane < NCH) fma_chunk(acc, 1.f, tok.v, T{});
    }
    return tok;
}

// ---------------------------------------------------------------------------------------
// End of a split-launch workgroup: every wave arrives with its own running (max, sum) and
// its unnormalised accumulators (X floats per lane: chunk lane % LPR of row group lane / LPR).
// Everything meets in LDS: the row groups of a wave are summed by the wave itself, the waves of
// the workgroup after a single barrier; then the output is written (whole pair) or a partial is
// published that the last piece of the pair to arrive merges.
template <typename T, int DH, int NW>
struct MergeLds {
    alignas(16) float part[NW * Geo<T, DH>::RPI][Geo<T, DH>::ROWW];  // [wave, row group][chunk, element]
    float red[NW][DH];                                               // [wave][element]: row groups summed
    float m[NW], l[NW];
};

template <typename T, int DH, int NW>
__device__ __forceinline__ void finish_piece(const DecodeParams& P, int bh, int split, int n_splits,
                                             float (&acc)[Elem<T>::X], float m_run, float l_run,
                                             MergeLds<T, DH, NW>& s) {
    using G = Geo<T, DH>;
    constexpr int X = G::X, LPR = G::LPR, NCH = G::NCH, RPI = G::RPI;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // Stage 1, before the barrier and wave by wave as each one finishes: the RPI row groups of
    // the wave are summed through its own LDS rows (2 wide writes and 64 X / 64 reads per lane,
    // where a butterfly over the lanes takes log2(RPI) x X cross-lane moves).
    l_run = wave_sum(l_run);
    if (lane == 0) { s.m[wave] = m_run; s.l[wave] = l_run; }
    if (lane % LPR < NCH) {
        float* dst = &s.part[wave * RPI + lane / LPR][(lane % LPR) * X];
#pragma unroll
        for (int e = 0; e < X; e += 4) *reinterpret_cast<float4*>(dst + e) = make_float4(acc[e], acc[e + 1], acc[e + 2], acc[e + 3]);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int d = lane; d < DH; d += kWave) {
        float r = 0.f;
#pragma unroll
        for (int g = 0; g < RPI; ++g) r += s.part[wave * RPI + g][d];
        s.red[wave][d] = r;
    }
    __syncthreads();
    // Output elements live in the first ceil(DH / 64) waves; the others are done.
    constexpr int NOUT = (DH + kWave - 1) / kWave < NW ? (DH + kWave - 1) / kWave : NW;
    if (wave >= NOUT) return;

    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, s.m[w]);
    float L = 0.f;
    float wgt[NW];
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        wgt[w] = (s.m[w] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(s.m[w] - M);
        L += wgt[w] * s.l[w];
    }

    T* out = reinterpret_cast<T*>(P.out) + (size_t)bh * DH;
    // Partials of split pairs: n_splits slots of the workspace per pair, each the accumulator
    // followed by (max, sum) and padded to whole 256-byte lines, so that no two workgroups ever
    // write into the same line.
    constexpr int SLOT = DH + kSlotTailFloats;
    const size_t slot0 = (size_t)(bh - P.n_whole) * P.n_splits;
    float* wa = P.ws_acc + (slot0 + split) * SLOT;
    for (int d = tid; d < DH; d += NOUT * 64) {
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) o += wgt[w] * s.red[w][d];
        if (n_splits == 1) store_out(out, d, L > 0.f ? o / L : 0.f);
        else if (P.combine == FFA_COMBINE_FUSED) publish(&wa[d], o);
        else wa[d] = o;
    }
    if (n_splits == 1) return;
    if (P.combine != FFA_COMBINE_FUSED) {
        // A second kernel merges: plain stores would do, the kernel boundary publishes them.
        if (tid == 0) {
            wa[DH] = M;
            wa[DH + 1] = L;
        }
        return;
    }

    // ---- publish the partial; the last wave to arrive merges all splits ----
    // No device-scope fence here: on this part such a fence writes back / invalidates a
    // whole L2 and costs far more than the kernel itself.  Instead every word that crosses
    // workgroups is moved with device-scope atomic accesses, which the hardware performs
    // at the level all XCDs share, so nothing needs flushing.
    // The protocol runs per wave, without further workgroup barriers: the waves that hold
    // output elements (the first ceil(Dh/64)) each publish theirs, wait until the stores have
    // been acknowledged (wait_published), and only then bump the pair's arrival counter; the
    // wave that sees the final count -- n_splits pieces x publishing waves -- knows that
    // every partial of the pair is in memory and merges all of them.
    if (tid == 0) {
        publish(&wa[DH], M);
        publish(&wa[DH + 1], L);
    }
    wait_published();
    unsigned prev = 0;
    if (lane == 0)
        prev = __hip_atomic_fetch_add(&P.ws_cnt[(size_t)bh * kCounterStride], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    prev = __builtin_amdgcn_readfirstlane(prev);
    if (prev != (unsigned)(n_splits * NOUT - 1)) return;
    // Compiler-only barrier: the loads of the merge below must stay behind the counter
    // read-modify-write (in hardware they are ordered by the branch on its returned value).
    __atomic_signal_fence(__ATOMIC_SEQ_CST);

    // Merge: all loads of a batch of splits are issued before any is consumed.
    const float* pa = P.ws_acc + slot0 * SLOT;
    constexpr int MB = 8;
    for (int d = lane; d < DH; d += kWave) {
        float Mg = -INFINITY, o = 0.f, Lg = 0.f;
        for (int s0 = 0; s0 < n_splits; s0 += MB) {
            float ms[MB], ls[MB], as[MB];
#pragma unroll
            for (int j = 0; j < MB; ++j) {
                const int sj = min(s0 + j, n_splits - 1);
                ms[j] = acquire(&pa[(size_t)sj * SLOT + DH]);
                ls[j] = acquire(&pa[(size_t)sj * SLOT + DH + 1]);
                as[j] = acquire(&pa[(size_t)sj * SLOT + d]);
            }
            float Mb = Mg;
#pragma unroll
            for (int j = 0; j < MB; ++j)
                if (s0 + j < n_splits) Mb = fmaxf(Mb, ms[j]);
            const float rescale = (Mg == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(Mg - Mb);
            o *= rescale;
            Lg *= rescale;
#pragma unroll
            for (int j = 0; j < MB; ++j) {
                if (s0 + j < n_splits && ms[j] != -INFINITY) {
                    const float w = __builtin_amdgcn_exp2f(ms[j] - Mb);
                    Lg += w * ls[j];
                    o += w * as[j];
                }
            }
            Mg = Mb;
        }
        if (P.store_through) store_out_through(out, d, Lg > 0.f ? o / Lg : 0.f);
        else store_out(out, d, Lg > 0.f ? o / Lg : 0.f);
    }
    // Ready for the next launch on this stream (kernel boundaries order this store).
    if (lane == 0) __hip_atomic_store(&P.ws_cnt[(size_t)bh * kCounterStride], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------------------
// Sequence-split exact decode (p == 0).
template <typename T, int DH, int NW, bool BEAM, bool XFORM>
__global__ void __launch_bounds__((NW + 1) * 64)
ffa_decode_split_kernel(HOT_PARAMS_DECL, const DecodeParams P_rest) {
    const DecodeParams P = with_hot_params(P_rest, HOT_PARAMS_USE);
    using G = Geo<T, DH>;
    constexpr int X = G::X, NCH = G::NCH, LPR = G::LPR, RPI = G::RPI, NVL = G::NVL;
    constexpr int VG = G::VG;  // V loads kept in flight per group
    constexpr int CG = G::CG;

    __shared__ float s_p[NW][kWave];
    __shared__ MergeLds<T, DH, NW + 1> s_merge;
    __shared__ TokenLds<T, DH> s_tok;
    __shared__ AngleLds<T, DH, XFORM> s_ang;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, and known to be so

    // Work mapping.  The first n_whole workgroups each own a whole (b,h) pair and finish with
    // an LDS merge only; the remaining pairs are cut into n_splits pieces whose partials are
    // merged by the last piece to arrive.  Whole pairs are what the kernel ends on, so the
    // cross-workgroup merges (a chain of memory round trips) finish in their shadow.
    const PieceOf piece(P, (int)blockIdx.x);
    const int bh = piece.bh, split = piece.split, n_splits = piece.n_splits;
    const bool need_b = P.seq_lengths != nullptr || BEAM;
    const int b = need_b ? bh / P.H : 0;

    int tlen, first;
    step_bounds(P, b, tlen, first);

    const size_t head_bytes = (size_t)P.Lmax * DH * sizeof(T);
    char* kc_bh = reinterpret_cast<char*>(P.k_cache) + (size_t)bh * head_bytes;
    char* vc_bh = reinterpret_cast<char*>(P.v_cache) + (size_t)bh * head_bytes;
    const BeamRows<BEAM> beams(P, b, bh, head_bytes);

    // Tiles of cached keys [0, tlen); this piece's share in units of the plan's 64-key tiles.
    const int ntiles = (tlen + kWave - 1) / kWave;
    const int tps = n_splits == 1 ? ntiles : P.tiles_per_split;
    const int tile_lo = max(split * tps, first / kWave);
    const int tile_hi = min(ntiles, (split + 1) * tps);
    const int last_key = tlen - 1;  // >= 0 whenever a tile exists
    // Waves 0 .. NW-1 walk tiles; wave NW is the token wave (token_wave_state).
    const bool token_wave = wave == NW;

    const int rg = lane / LPR, dch = min(lane % LPR, NCH - 1);
    float m_run = -INFINITY, l_run = 0.f;
    float acc[X];
#pragma unroll
    for (int e = 0; e < X; ++e) acc[e] = 0.f;

    // V rows of load group g for this lane: rows tile*64 + (g*VG+j)*RPI + rg, j < VG.  `src` is
    // the source beam of this lane's key of the tile; a row's beam sits in the lane of that key.
    auto load_v_group = [&](uint4 (&vv)[VG], int tile, int g, int src) {
#pragma unroll
        for (int j = 0; j < VG; ++j) {
            const int in_tile = (g * VG + j) * RPI + rg;
            const int row = min(tile * kWave + in_tile, last_key);
            const char* vb = vc_bh;
            if constexpr (BEAM) vb = beams.v_of(__shfl(src, in_tile));
            vv[j] = ld16(vb + ((size_t)row * NCH + dch) * 16);
        }
    };

    // First load groups of one tile: CG chunks of K (lane = key) and VG chunks of V
    // (lane = row group x d-chunk).  V does not depend on the scores, so both go out together.
    const size_t kstr = (size_t)P.Lmax * 16;
    auto load_tile = [&](uint4 (&kv)[CG], uint4 (&vv)[VG], int tile, int src) {
        const int key = min(tile * kWave + lane, last_key);
        load_k_group<CG>(kv, beams.k_of(src) + (size_t)key * 16, kstr, 0);
        load_v_group(vv, tile, 0, src);
    };

    TokenRegs tok;
    const bool has_token = token_wave && split == n_splits - 1;
    if (token_wave) {
        if constexpr (XFORM) {
            // The token wave of EVERY workgroup publishes the angles while the tile waves' first
            // tiles are on their way; where it holds the token it also transforms q, k and v.
            RawToken<T, DH> raw;
            xform_begin<T, DH>(raw, P, bh, tlen, first, /*needs_q=*/has_token, /*publisher=*/true, /*with_kv=*/has_token,
                               s_ang, lane);
            xform_end<T, DH>(raw, P, has_token, true, has_token, s_tok, s_ang, lane);
        }
        if (has_token) tok = token_wave_state<T, DH, XFORM>(P, bh, tlen, first, s_tok, m_run, l_run, acc, lane);
    } else {
    uint4 q_reg[G::QREG];

    // Scores, online softmax and P.V of one tile whose first load groups are in kv / vv.
    // QL: q is read from LDS (wide heads, transformed token) instead of SGPRs.
    auto compute_tile = [&](auto ql, uint4 (&kv)[CG], uint4 (&vv)[VG], int tile, int src) {
        constexpr bool QL = decltype(ql)::value;
        const int key = tile * kWave + lane;
        float s = 0.f;
        if constexpr (NCH > CG) {
            // Rolling groups: as soon as chunk c of a group has been consumed its registers take
            // chunk c of the next group, so a wave has a tile's first CG + VG loads in flight and
            // then tops up one by one.  (Left to itself the compiler hoists a whole second group
            // of K loads above the first dot product: 24 loads in flight per wave cost 5 % at
            // 320 pairs x 1000 keys of fp32.)
            const char* kp = beams.k_of(src) + (size_t)min(key, last_key) * 16;
#pragma unroll
            for (int g = 0; g < NCH / CG; ++g) {
#pragma unroll
                for (int c = 0; c < CG; ++c) {
                    uint4 qc;
                    if constexpr (QL) qc = s_tok.q[g * CG + c];
                    else qc = q_reg[g * CG + c];
                    s = dot_chunk(kv[c], qc, s, T{});
                    if (g + 1 < NCH / CG) kv[c] = ld16(kp + (size_t)((g + 1) * CG + c) * kstr);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        } else {
            s = dot_k_group<T, CG, QL>(kv, 0, q_reg, s_tok.q, 0.f);
        }

        const bool valid = key < tlen && key >= first;
        const float m_new = fmaxf(m_run, wave_max(valid ? s * P.scale_log2e : -INFINITY));
        // m_new == -inf only while every key seen so far is masked: acc, l are still 0.
        const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_run - m_new);
        // One rounding for s*c - m: the rounding of m itself is a common factor of every
        // weight and cancels in the normalisation.
        const float pr = valid ? __builtin_amdgcn_exp2f(fmaf(s, P.scale_log2e, -m_new)) : 0.f;
        l_run = l_run * alpha + pr;
        m_run = m_new;

        __builtin_amdgcn_wave_barrier();
        s_p[wave][stage_slot<G::NVL, RPI>(lane)] = pr;
        __builtin_amdgcn_wave_barrier();

#pragma unroll
        for (int e = 0; e < X; ++e) acc[e] *= alpha;
        const float* pst = &s_p[wave][rg * NVL];
#pragma unroll
        for (int g = 0; g < NVL / VG; ++g) {
            uint4 vn[VG];
            if (g + 1 < NVL / VG) {
                // The next group goes out as a block before this one is consumed (left alone, the
                // compiler may sink each load next to its use: one round trip per pair of loads).
                load_v_group(vn, tile, g + 1, src);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int j = 0; j < VG; ++j) fma_chunk(acc, pst[g * VG + j], vv[j], T{});
            if (g + 1 < NVL / VG) {
                __builtin_amdgcn_sched_barrier(0);  // one group ahead, not more
#pragma unroll
                for (int j = 0; j < VG; ++j) vv[j] = vn[j];
            }
        }
        __builtin_amdgcn_wave_barrier();
    };

    // The scheduling barriers keep the compiler from sinking loads next to their uses to
    // save registers, which would serialise the round trips.  With beam indirection the
    // source beams of a tile are fetched one tile ahead, so that their round trip does not sit
    // in front of the tile's own loads.
    const TileOrder order(tile_lo, tile_hi, (unsigned)(bh * n_splits + split));
    // One loop per source of q, each with a straight-line body (a branch on the source inside
    // the loop lets the compiler hoist code of the tile's arithmetic in between its loads).
    auto walk_tiles = [&](auto ql, int from) {
        int src_next = from < order.n ? beams.beam(min(order.at(from) * kWave + lane, last_key), tlen) : 0;
        for (int idx = from; idx < order.n; idx += NW) {
            const int tile = order.at(idx);
            const int src = src_next;
            if constexpr (BEAM)
                src_next = idx + NW < order.n ? beams.beam(min(order.at(idx + NW) * kWave + lane, last_key), tlen) : 0;
            uint4 kv[CG], vv[VG];
            load_tile(kv, vv, tile, src);
            __builtin_amdgcn_sched_barrier(0);
            compute_tile(ql, kv, vv, tile, src);
        }
    };
    if constexpr (XFORM) {
        // With a transform: the load of q, the loads of the wave's first tile, then the barrier
        // behind which the token wave has left the angles, then q'.
        // (The barrier stands in both branches: behind a join the compiler no longer knows how many
        // loads follow that of q, and waits for all of them before it lets the wave look at q.)
        const bool has_tile = wave < order.n;
        RawToken<T, DH> raw;
        xform_begin<T, DH>(raw, P, bh, tlen, first, /*needs_q=*/has_tile, /*publisher=*/false, false, s_ang, lane);
        if (has_tile) {
            const int tile = order.at(wave);
            const int src = beams.beam(min(tile * kWave + lane, last_key), tlen);
            uint4 kv[CG], vv[VG];
            load_tile(kv, vv, tile, src);
            __builtin_amdgcn_sched_barrier(0);
            xform_end<T, DH>(raw, P, true, false, false, s_tok, s_ang, lane);
            compute_tile(std::true_type{}, kv, vv, tile, src);
            walk_tiles(std::true_type{}, wave + NW);
        } else {
            xform_end<T, DH>(raw, P, false, false, false, s_tok, s_ang, lane);
        }
    } else {
        const bool q_in_lds = setup_q<T, DH>(P, bh, s_tok, q_reg, lane);
        if constexpr (G::Q_LDS) {
            (void)q_in_lds;
            walk_tiles(std::true_type{}, wave);
        } else {
            walk_tiles(std::false_type{}, wave);
        }
    }
    }  // tile waves

    finish_piece<T, DH, NW + 1>(P, bh, split, n_splits, acc, m_run, l_run, s_merge);
    if (has_token) token_store<T, DH>(tok, kc_bh, vc_bh, tlen, P.Lmax, lane, P.store_through != 0);
}

// ---------------------------------------------------------------------------------------
// Sequence-split exact decode with TPK = 2 or 4 lanes per key.  A tile is KPT = 64 / TPK keys:
// lane l works on key l % KPT and on the NK = NCH / TPK chunks [part*NK, part*NK + NK) of the
// head dimension, part = l / KPT; the partial dot products of a key meet through TPK - 1
// cross-lane exchanges.  A load instruction then covers TPK chunk rows of KPT x 16 contiguous
// bytes (K) or still 1 KiB of consecutive V rows.  What this buys: tiles of 8 KiB / 4 KiB
// instead of 16 KiB at Dh = 64 (twice / four times the waves can share a short sequence), and
// at Dh = 256 a tile whose 16 loads are all in flight at once where one lane per key needs
// four dependent groups of loads.  Pieces are cut in units of 64 keys exactly as in
// ffa_decode_split_kernel, with which this kernel shares its epilogue.
template <typename T, int DH, int NW, int TPK, bool BEAM, bool XFORM>
__global__ void __launch_bounds__((NW + 1) * 64)
ffa_decode_split_tpk_kernel(HOT_PARAMS_DECL, const DecodeParams P_rest) {
    const DecodeParams P = with_hot_params(P_rest, HOT_PARAMS_USE);
    using G = Geo<T, DH>;
    constexpr int X = G::X, NCH = G::NCH, LPR = G::LPR, RPI = G::RPI;
    constexpr int KPT = kWave / TPK;   // keys per tile
    constexpr int NK = NCH / TPK;      // K loads per tile and lane
    constexpr int NV = KPT / RPI;      // V loads per tile and lane
    static_assert(TPK == 2 || TPK == 4, "lanes per key");
    static_assert(NCH % TPK == 0 && KPT % RPI == 0 && NK <= 8 && NV <= 8 && NV >= 1, "tile does not fit one load group");

    __shared__ float s_p[NW][KPT];
    __shared__ MergeLds<T, DH, NW + 1> s_merge;
    __shared__ TokenLds<T, DH> s_tok;
    __shared__ AngleLds<T, DH, XFORM> s_ang;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const PieceOf piece(P, (int)blockIdx.x);
    const int bh = piece.bh, split = piece.split, n_splits = piece.n_splits;
    const bool need_b = P.seq_lengths != nullptr || BEAM;
    const int b = need_b ? bh / P.H : 0;
    int tlen, first;
    step_bounds(P, b, tlen, first);

    const size_t head_bytes = (size_t)P.Lmax * DH * sizeof(T);
    char* kc_bh = reinterpret_cast<char*>(P.k_cache) + (size_t)bh * head_bytes;
    char* vc_bh = reinterpret_cast<char*>(P.v_cache) + (size_t)bh * head_bytes;
    const BeamRows<BEAM> beams(P, b, bh, head_bytes);

    const int kl = lane % KPT, part = lane / KPT;

    // Pieces in units of 64 keys (the plan's tiles), walked in tiles of KPT keys.
    const int ntiles64 = (tlen + kWave - 1) / kWave;
    const int tps64 = n_splits == 1 ? ntiles64 : P.tiles_per_split;
    const int ntiles = (tlen + KPT - 1) / KPT;  // cached keys 0..tlen-1
    const int tile_lo = max(split * tps64 * TPK, first / KPT);
    const int tile_hi = min(ntiles, (split + 1) * tps64 * TPK);
    const int last_key = tlen - 1;
    const bool token_wave = wave == NW;  // waves 0 .. NW-1 walk tiles

    const int rg = lane / LPR, dch = min(lane % LPR, NCH - 1);
    float m_run = -INFINITY, l_run = 0.f;
    float acc[X];
#pragma unroll
    for (int e = 0; e < X; ++e) acc[e] = 0.f;

    const size_t kstr = (size_t)P.Lmax * 16;
    auto load_tile = [&](uint4 (&kv)[NK], uint4 (&vv)[NV], int tile, int src) {
        const int key = min(tile * KPT + kl, last_key);
        const char* kp = beams.k_of(src) + ((size_t)(part * NK) * P.Lmax + key) * 16;
#pragma unroll
        for (int i = 0; i < NK; ++i) kv[i] = ld16(kp + (size_t)i * kstr);
#pragma unroll
        for (int j = 0; j < NV; ++j) {
            const int in_tile = j * RPI + rg;
            const int row = min(tile * KPT + in_tile, last_key);
            const char* vb = vc_bh;
            if constexpr (BEAM) vb = beams.v_of(__shfl(src, in_tile));  // lane in_tile < KPT holds that key's beam
            vv[j] = ld16(vb + ((size_t)row * NCH + dch) * 16);
        }
    };

    TokenRegs tok;
    const bool has_token = token_wave && split == n_splits - 1;
    if (token_wave) {
        if constexpr (XFORM) {  // as in ffa_decode_split_kernel
            RawToken<T, DH> raw;
            xform_begin<T, DH>(raw, P, bh, tlen, first, /*needs_q=*/has_token, /*publisher=*/true, /*with_kv=*/has_token,
                               s_ang, lane);
            xform_end<T, DH>(raw, P, has_token, true, has_token, s_tok, s_ang, lane);
        }
        if (has_token) tok = token_wave_state<T, DH, XFORM>(P, bh, tlen, first, s_tok, m_run, l_run, acc, lane);
    } else {
    uint4 q_reg[NK];  // this lane's share of q: chunks [part*NK, part*NK + NK)
    auto compute_tile = [&](uint4 (&kv)[NK], uint4 (&vv)[NV], int tile) {
        const int key = tile * KPT + kl;
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < NK; ++i) s = dot_chunk(kv[i], q_reg[i], s, T{});
#pragma unroll
        for (int off = KPT; off < kWave; off <<= 1) s += __shfl_xor(s, off);

        const bool valid = key < tlen && key >= first;
        const float m_new = fmaxf(m_run, wave_max(valid ? s * P.scale_log2e : -INFINITY));
        const float alpha = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_run - m_new);
        const float pr = valid ? __builtin_amdgcn_exp2f(fmaf(s, P.scale_log2e, -m_new)) : 0.f;
        l_run = l_run * alpha + (part == 0 ? pr : 0.f);  // every key is held by TPK lanes: count it once
        m_run = m_new;

        __builtin_amdgcn_wave_barrier();
        if (part == 0) s_p[wave][stage_slot<NV, RPI>(kl)] = pr;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int e = 0; e < X; ++e) acc[e] *= alpha;
        const float* pst = &s_p[wave][rg * NV];
#pragma unroll
        for (int j = 0; j < NV; ++j) fma_chunk(acc, pst[j], vv[j], T{});
        __builtin_amdgcn_wave_barrier();
    };
    const TileOrder order(tile_lo, tile_hi, (unsigned)(bh * n_splits + split));
    auto walk_tiles = [&](int from) {
        int src_next = from < order.n ? beams.beam(min(order.at(from) * KPT + kl, last_key), tlen) : 0;
        for (int idx = from; idx < order.n; idx += NW) {
            const int tile = order.at(idx);
            const int src = src_next;
            if constexpr (BEAM)
                src_next = idx + NW < order.n ? beams.beam(min(order.at(idx + NW) * KPT + kl, last_key), tlen) : 0;
            uint4 kv[NK], vv[NV];
            load_tile(kv, vv, tile, src);
            __builtin_amdgcn_sched_barrier(0);
            compute_tile(kv, vv, tile);
        }
    };
    if constexpr (XFORM) {
        // As in ffa_decode_split_kernel: q, the first tile's loads, the barrier, q'.
        const bool has_tile = wave < order.n;
        RawToken<T, DH> raw;
        xform_begin<T, DH>(raw, P, bh, tlen, first, /*needs_q=*/has_tile, /*publisher=*/false, false, s_ang, lane);
        if (has_tile) {
            const int tile = order.at(wave);
            const int src = beams.beam(min(tile * KPT + kl, last_key), tlen);
            uint4 kv[NK], vv[NV];
            load_tile(kv, vv, tile, src);
            __builtin_amdgcn_sched_barrier(0);
            xform_end<T, DH>(raw, P, true, false, false, s_tok, s_ang, lane);
#pragma unroll
            for (int i = 0; i < NK; ++i) q_reg[i] = s_tok.q[part * NK + i];
            compute_tile(kv, vv, tile);
            walk_tiles(wave + NW);
        } else {
            xform_end<T, DH>(raw, P, false, false, false, s_tok, s_ang, lane);
        }
    } else {
        uint4 q_full[G::QREG];
        const bool q_in_lds = setup_q<T, DH>(P, bh, s_tok, q_full, lane);
        if (q_in_lds) {
#pragma unroll
            for (int i = 0; i < NK; ++i) q_reg[i] = s_tok.q[part * NK + i];
        } else {
            const char* qg = reinterpret_cast<const char*>(P.q) + (size_t)bh * DH * sizeof(T);
#pragma unroll
            for (int i = 0; i < NK; ++i) q_reg[i] = *reinterpret_cast<const uint4*>(qg + (part * NK + i) * 16);
        }
        walk_tiles(wave);
    }
    }  // tile waves
    finish_piece<T, DH, NW + 1>(P, bh, split, n_splits, acc, m_run, l_run, s_merge);
    if (has_token) token_store<T, DH>(tok, kc_bh, vc_bh, tlen, P.Lmax, lane, P.store_through != 0);
}

// ---------------------------------------------------------------------------------------
// Load floor of a split launch (ffa_load_floor): the grid, the workgroups, the piece mapping, the
// tile order and the addresses of ffa_decode_split_kernel, every 16-byte load of every tile issued
// the same way (at most 16 in flight per wave) -- and nothing else: no arithmetic on the data, no
// merge, no output.  What it takes is what the memory system gives this launch shape; the decode
// kernel's distance from it is the cost of its arithmetic and of its merges.  The loaded words
// are folded with XOR so that the loads cannot be dropped; the fold is stored only if it equals a
// value it never takes.
template <typename T, int DH, int NW>
__global__ void __launch_bounds__((NW + 1) * 64) ffa_load_floor_kernel(HOT_PARAMS_DECL, const DecodeParams P_rest) {
    const DecodeParams P = with_hot_params(P_rest, HOT_PARAMS_USE);
    using G = Geo<T, DH>;
    constexpr int NCH = G::NCH, LPR = G::LPR, RPI = G::RPI, NVL = G::NVL;
    constexpr int GRP = 8;  // loads per group: one group of K and one of V in flight, as in the decode kernel
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const PieceOf piece(P, (int)blockIdx.x);
    const int bh = piece.bh, split = piece.split, n_splits = piece.n_splits;
    int tlen, first;
    step_bounds(P, P.seq_lengths != nullptr ? bh / P.H : 0, tlen, first);
    if (wave == NW || tlen <= 0) return;  // the token wave loads nothing from the caches
    const size_t head_bytes = (size_t)P.Lmax * DH * sizeof(T);
    const char* kc_bh = reinterpret_cast<const char*>(P.k_cache) + (size_t)bh * head_bytes;
    const char* vc_bh = reinterpret_cast<const char*>(P.v_cache) + (size_t)bh * head_bytes;
    const int ntiles = (tlen + kWave - 1) / kWave;
    const int tps = n_splits == 1 ? ntiles : P.tiles_per_split;
    const int tile_lo = max(split * tps, first / kWave);
    const int tile_hi = min(ntiles, (split + 1) * tps);
    const int last_key = tlen - 1;
    const int rg = lane / LPR, dch = min(lane % LPR, NCH - 1);
    const size_t kstr = (size_t)P.Lmax * 16;
    const TileOrder order(tile_lo, tile_hi, (unsigned)(bh * n_splits + split));
    uint4 fold = make_uint4(0u, 0u, 0u, 0u);
    auto take = [&](const uint4& v) { fold.x ^= v.x; fold.y ^= v.y; fold.z ^= v.z; fold.w ^= v.w; };
    for (int idx = wave; idx < order.n; idx += NW) {
        const int tile = order.at(idx);
        const char* kp = kc_bh + (size_t)min(tile * kWave + lane, last_key) * 16;
        constexpr int NG = ((NCH > NVL ? NCH : NVL) + GRP - 1) / GRP;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
            uint4 kv[GRP], vv[GRP];
#pragma unroll
            for (int c = 0; c < GRP; ++c) {
                kv[c] = make_uint4(0u, 0u, 0u, 0u);
                if (g * GRP + c < NCH) kv[c] = ld16(kp + (size_t)(g * GRP + c) * kstr);
            }
#pragma unroll
            for (int j = 0; j < GRP; ++j) {
                vv[j] = make_uint4(0u, 0u, 0u, 0u);
                if (g * GRP + j < NVL) {
                    const int row = min(tile * kWave + (g * GRP + j) * RPI + rg, last_key);
                    vv[j] = ld16(vc_bh + ((size_t)row * NCH + dch) * 16);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int c = 0; c < GRP; ++c) take(kv[c]);
#pragma unroll
            for (int j = 0; j < GRP; ++j) take(vv[j]);
        }
    }
    if (fold.x == 0x9e3779b9u && fold.y == 0x7f4a7c15u && fold.z == 0xf39cc060u && fold.w == 0x5cedc834u)
        *reinterpret_cast<uint4*>(P.out) = fold;
}

// Merge kernel of FFA_COMBINE_KERNEL: one wave per split (b,h) pair, log-sum-exp over its
// partials.
template <typename T, int DH>
__global__ void __launch_bounds__(64) ffa_merge_splits_kernel(const DecodeParams P) {
    const int bh = P.n_whole + blockIdx.x, tid = threadIdx.x;
    constexpr int SLOT = DH + kSlotTailFloats;
    const float* pa = P.ws_acc + (size_t)blockIdx.x * P.n_splits * SLOT;
    float Mg = -INFINITY;
    for (int s = 0; s < P.n_splits; ++s) Mg = fmaxf(Mg, pa[(size_t)s * SLOT + DH]);
    T* out = reinterpret_cast<T*>(P.out) + (size_t)bh * DH;
    for (int d = tid; d < DH; d += 64) {
        float o = 0.f, Lg = 0.f;
        for (int s = 0; s < P.n_splits; ++s) {
            const float ms = pa[(size_t)s * SLOT + DH];
            const float w = (ms == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(ms - Mg);
            Lg += w * pa[(size_t)s * SLOT + DH + 1];
            o += w * pa[(size_t)s * SLOT + d];
        }
        store_out(out, d, Lg > 0.f ? o / Lg : 0.f);
    }
}

// ---------------------------------------------------------------------------------------
// One workgroup per (b,h): exact (p == 0) or pruned (p > 0) decode with LDS-staged scores.
// Dynamic LDS: max((t/64 + 1)*64 scores, NW*64*X merge floats) * 4 bytes.
template <typename T, int DH, int NW, bool BEAM, bool XFORM>
__global__ void __launch_bounds__(NW * 64) ffa_decode_wg_kernel(HOT_PARAMS_DECL, const DecodeParams P_rest) {
    const DecodeParams P = with_hot_params(P_rest, HOT_PARAMS_USE);
    using G = Geo<T, DH>;
    constexpr int X = G::X, NCH = G::NCH, LPR = G::LPR, RPI = G::RPI, NVL = G::NVL, VG = G::VG;
    constexpr int NT = NW * 64;

    extern __shared__ float s_dyn[];
    float* s_sc = s_dyn;
    __shared__ float s_red[NW];
    __shared__ unsigned s_cnt[NW];
    __shared__ TokenLds<T, DH> s_tok;
    // The angles of the token transform are read before the first score is written, the survivor
    // queues are filled after the barriers that follow the last score: one piece of LDS serves
    // both (the dynamic part may take all but 20 KiB of the CU's LDS).
    constexpr size_t kQueueBytes = sizeof(float) * NW * 2 * kWave;
    constexpr size_t kAngleBytes = sizeof(AngleLds<T, DH, XFORM>);
    __shared__ __align__(16) unsigned char s_shared[2 * kQueueBytes > kAngleBytes ? 2 * kQueueBytes : kAngleBytes];
    AngleLds<T, DH, XFORM>& s_ang = *reinterpret_cast<AngleLds<T, DH, XFORM>*>(s_shared);
    float(*s_qw)[2 * kWave] = reinterpret_cast<float(*)[2 * kWave]>(s_shared);
    int(*s_qr)[2 * kWave] = reinterpret_cast<int(*)[2 * kWave]>(s_shared + kQueueBytes);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bh = blockIdx.x;
    const int b = (P.seq_lengths != nullptr || BEAM) ? bh / P.H : 0;  // nobody else asks for it

    int tlen, first;
    step_bounds(P, b, tlen, first);

    const size_t head_bytes = (size_t)P.Lmax * DH * sizeof(T);
    char* kc_bh = reinterpret_cast<char*>(P.k_cache) + (size_t)bh * head_bytes;
    char* vc_bh = reinterpret_cast<char*>(P.v_cache) + (size_t)bh * head_bytes;
    const BeamRows<BEAM> beams(P, b, bh, head_bytes);
    const int rows_per_sample = P.H * P.Lmax;

    const bool token_wave = wave == 0;
    uint4 q_reg[G::QREG];
    bool q_in_lds = true;
    if constexpr (XFORM) {
        RawToken<T, DH> raw;
        xform_begin<T, DH>(raw, P, bh, tlen, first, /*needs_q=*/true, /*publisher=*/token_wave, /*with_kv=*/true, s_ang, lane);
        xform_end<T, DH>(raw, P, true, token_wave, true, s_tok, s_ang, lane);
    } else {
        q_in_lds = setup_q<T, DH>(P, bh, s_tok, q_reg, lane);
    }
    TokenRegs tok;
    if (token_wave) tok = token_load<T, DH, XFORM>(P, bh, s_tok, lane);

    const int ntiles = (tlen + kWave - 1) / kWave;   // tiles of cached keys
    const int nscore = (tlen / kWave + 1) * kWave;   // score slots: keys 0..tlen, padded to 64
    const int tile_lo = min(first / kWave, ntiles);  // tiles below are fully masked
    const int last_key = tlen - 1;
    const bool pruned = P.p > 0.f;

    // ---- phase 1: raw scores to LDS, running max (exp2 domain).  Slot tlen belongs to the
    // token wave; the owner of the tile around it leaves that one slot alone ----
    float mx = -INFINITY;
    const TileOrder order(tile_lo, ntiles, (unsigned)bh);
    for (int idx = wave; idx < order.n; idx += NW) {
        const int tile = order.at(idx);
        const int key = tile * kWave + lane;
        const int ck = min(key, last_key);
        const char* kb = beams.k_of(beams.beam(ck, tlen));
        const float s = q_in_lds ? tile_qk<T, NCH, true>(kb, ck, P.Lmax, q_reg, s_tok.q)
                                 : tile_qk<T, NCH, G::Q_LDS>(kb, ck, P.Lmax, q_reg, s_tok.q);
        const bool valid = key < tlen && key >= first;
        if (key != tlen) s_sc[key] = valid ? s : -INFINITY;  // raw dot product; scaled inside the exp2 below
        mx = fmaxf(mx, valid ? s * P.scale_log2e : -INFINITY);
    }
    if (token_wave) {
        const float s = token_score<T, DH>(tok, lane);
        const bool valid = tlen >= first;
        // With tlen a multiple of 64 no cached tile covers the slots around tlen: fill them too.
        if (lane == 0) s_sc[tlen] = valid ? s : -INFINITY;
        else if (tlen % kWave == 0) s_sc[tlen + lane] = -INFINITY;
        if (valid) mx = fmaxf(mx, s * P.scale_log2e);
        token_store<T, DH>(tok, kc_bh, vc_bh, tlen, P.Lmax, lane);
    }
    mx = wave_max(mx);
    if (lane == 0) s_red[wave] = mx;
    __syncthreads();
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, s_red[w]);
    const bool all_masked = (M == -INFINITY);
    if (all_masked) M = 0.f;
    __syncthreads();  // s_red is reused below

    // ---- phase 2: e_i = exp(s_i - max), sum ----
    float sum = 0.f;
    for (int i = tile_lo * kWave + tid; i < nscore; i += NT) {
        const float sr = s_sc[i];
        // one rounding for s*c - M; masked keys (-inf) give exactly 0
        const float e = (sr == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(fmaf(sr, P.scale_log2e, -M));
        s_sc[i] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    if (lane == 0) s_red[wave] = sum;
    __syncthreads();
    float S = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) S += s_red[w];

    // p == 0: exact softmax, the 1/S factor is applied once at the end.
    // p  > 0: the reference's rule, to the letter (attention.cu:1122-1126, :1184-1191):
    //         inv = 1/(S+1e-6); P_i = T(e_i*inv); thr = T(p*inv); drop i<tlen iff leq(P_i,thr).
    float out_scale = S > 0.f ? 1.f / S : 0.f;
    if (pruned) {
        const float inv = 1.f / (S + 1.e-6f);
        float thr_key;
        (void)round_prob(P.p * inv, T{}, &thr_key);
        unsigned kept = 0;
        for (int i = tile_lo * kWave + tid; i < nscore; i += NT) {
            float key_i;
            const float Pi = round_prob(s_sc[i] * inv, T{}, &key_i);
            const bool in_range = i >= first && i <= tlen;
            const bool drop = !in_range || (i < tlen && key_i <= thr_key);
            s_sc[i] = drop ? -1.f : Pi;
            if (i < tlen) {
                kept += drop ? 0u : 1u;
                if (P.skip_mask) P.skip_mask[(size_t)bh * P.Lmax + i] = drop ? 1 : 0;
            }
        }
        if (P.skip_mask)  // keys of fully masked leading tiles are dropped too
            for (int i = tid; i < min(tile_lo * kWave, tlen); i += NT)
                P.skip_mask[(size_t)bh * P.Lmax + i] = 1;
        if (P.kept_count) {
            kept = wave_sum_u32(kept);
            if (lane == 0) s_cnt[wave] = kept;
        }
        out_scale = 1.f;
    } else {
        if (P.skip_mask)
            for (int i = tid; i < tlen; i += NT)
                P.skip_mask[(size_t)bh * P.Lmax + i] = (i < first) ? 1 : 0;
    }
    __syncthreads();
    if (P.kept_count && tid == 0) {
        unsigned tot = 0;
        if (pruned) {
#pragma unroll
            for (int w = 0; w < NW; ++w) tot += s_cnt[w];
        } else {
            tot = (unsigned)max(tlen - min(first, tlen), 0);
        }
        P.kept_count[bh] = tot;
    }

    // ---- phase 3: P.V over the cached rows.  Pruned: only the surviving rows, compacted per
    // wave.  The new token's row comes from the token wave's registers afterwards ----
    const int rg = lane / LPR, dch = min(lane % LPR, NCH - 1);
    float acc[X];
#pragma unroll
    for (int e = 0; e < X; ++e) acc[e] = 0.f;
    if (pruned) {
        SurvivorQueue sq = {s_qw[wave], s_qr[wave], 0u};
        for (int idx = wave; idx < order.n; idx += NW) {
            const int tile = order.at(idx);
            const int key = tile * kWave + lane;
            const float w = key < tlen ? s_sc[key] : -1.f;
            const int row = beams.v_row(beams.beam(key, tlen), key, rows_per_sample);
            queue_push<T, DH>(acc, sq, w >= 0.f, w, row, beams.v_group, lane);
        }
        queue_drain<T, DH>(acc, sq, beams.v_group, lane);
    } else {
        for (int idx = wave; idx < order.n; idx += NW) {
            const int tile = order.at(idx);
            const int src = beams.beam(min(tile * kWave + lane, last_key), tlen);  // a row's beam sits in its key's lane
#pragma unroll 1
            for (int g = 0; g < NVL / VG; ++g) {
                uint4 vv[VG];
                float pj[VG];
#pragma unroll
                for (int j = 0; j < VG; ++j) {
                    // Unconditional loads (rows past the end re-read the last cached row with
                    // weight 0): a load under a branch would have to be waited for at the
                    // join, one round trip per row.
                    const int in_tile = (g * VG + j) * RPI + rg;
                    const int row = tile * kWave + in_tile;
                    pj[j] = row < tlen ? s_sc[row] : 0.f;
                    const int r = min(row, last_key);
                    const char* vb = vc_bh;
                    if constexpr (BEAM) vb = beams.v_of(__shfl(src, in_tile));
                    vv[j] = ld16(vb + ((size_t)r * NCH + dch) * 16);
                }
#pragma unroll
                for (int j = 0; j < VG; ++j) fma_chunk(acc, pj[j], vv[j], T{});
            }
        }
    }
    if (token_wave) {
        const float w = s_sc[tlen];  // never dropped (a masked sample has weight 0 or -1 there)
        if (lane < NCH) fma_chunk(acc, fmaxf(w, 0.f), tok.v, T{});
    }

    // ---- merge the waves (the score buffer is dead now and is reused) ----
    __syncthreads();
    float* s_acc = s_dyn;
#pragma unroll
    for (int e = 0; e < X; ++e) s_acc[(wave * kWave + lane) * X + e] = acc[e];
    __syncthreads();
    T* out = reinterpret_cast<T*>(P.out) + (size_t)bh * DH;
    for (int d = tid; d < DH; d += NT) {
        float o = 0.f;
        for (int w = 0; w < NW; ++w)
#pragma unroll
            for (int g = 0; g < RPI; ++g) o += s_acc[w * kWave * X + g * G::ROWW + d];
        store_out(out, d, all_masked ? 0.f : o * out_scale);
    }
}

// ---------------------------------------------------------------------------------------
// Two-pass sequence-split path (FFA_LAUNCH_TWO_PASS): any p, any length, n_splits pieces per
// (b,h) pair.  Pass 1 streams K and leaves the raw scores (4 bytes per key) and each piece's
// (max, sum of exp2) in the workspace, and appends the new token; pass 2 folds those into the
// pair's global max and sum -- which the pruning rule needs before it may touch a single V row
// -- then streams only the V rows that survive (the new token's row, appended by pass 1, is
// an ordinary row of the sample's own cache by then).  Weights are normalised globally, hence
// the pieces' partial outputs simply add up (merged by the last piece to arrive).
template <typename T, int DH, int NW, bool BEAM, bool XFORM>
__global__ void __launch_bounds__(NW * 64) ffa_scores_kernel(HOT_PARAMS_DECL, const DecodeParams P_rest) {
    const DecodeParams P = with_hot_params(P_rest, HOT_PARAMS_USE);
    using G = Geo<T, DH>;
    constexpr int NCH = G::NCH;
    __shared__ float s_m[NW], s_l[NW];
    __shared__ TokenLds<T, DH> s_tok;
    __shared__ AngleLds<T, DH, XFORM> s_ang;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const unsigned pair = pair_of(P, blockIdx.x);
    const int bh = (int)pair, split = (int)(blockIdx.x - pair * (unsigned)P.n_splits);
    const int b = (P.seq_lengths != nullptr || BEAM) ? bh / P.H : 0;  // nobody else asks for it
    int tlen, first;
    step_bounds(P, b, tlen, first);

    const size_t head_bytes = (size_t)P.Lmax * DH * sizeof(T);
    char* kc_bh = reinterpret_cast<char*>(P.k_cache) + (size_t)bh * head_bytes;
    char* vc_bh = reinterpret_cast<char*>(P.v_cache) + (size_t)bh * head_bytes;

    const bool token_wave = split == P.n_splits - 1 && wave == 0;
    uint4 q_reg[G::QREG];
    // With a transform, wave 0 of every piece publishes the angles; in the piece that holds the token it
    // also transforms k and v.
    bool q_in_lds = true;
    if constexpr (XFORM) {
        RawToken<T, DH> raw;
        xform_begin<T, DH>(raw, P, bh, tlen, first, /*needs_q=*/true, /*publisher=*/wave == 0, /*with_kv=*/token_wave, s_ang,
                           lane);
        xform_end<T, DH>(raw, P, true, wave == 0, token_wave, s_tok, s_ang, lane);
    } else {
        q_in_lds = setup_q<T, DH>(P, bh, s_tok, q_reg, lane);
    }
    TokenRegs tok;
    if (token_wave) tok = token_load<T, DH, XFORM>(P, bh, s_tok, lane);

    const int ntiles = (tlen + kWave - 1) / kWave;
    const int tile_lo = max(split * P.tiles_per_split, first / kWave);
    const int tile_hi = min(ntiles, (split + 1) * P.tiles_per_split);
    const int last_key = tlen - 1;
    if (split == 0 && tid == 0 && P.kept_count) P.kept_count[bh] = 0u;  // pass 2 accumulates

    // Each lane keeps a running (max, sum of exp2) over its own keys; lanes, then waves, are
    // folded once at the end.  Every 64-key block of the score row up to and including the one
    // of slot tlen is written in full (the token wave owns slot tlen itself).
    const BeamRows<BEAM> beams(P, b, bh, head_bytes);
    float* sc = P.ws_scores + (size_t)bh * P.score_stride;
    float m_run = -INFINITY, l_run = 0.f;
    const TileOrder order(tile_lo, tile_hi, (unsigned)blockIdx.x);
    for (int idx = wave; idx < order.n; idx += NW) {
        const int tile = order.at(idx);
        const int key = tile * kWave + lane;
        const int ck = min(key, last_key);
        const char* kb = beams.k_of(beams.beam(ck, tlen));
        const float s = q_in_lds ? tile_qk<T, NCH, true>(kb, ck, P.Lmax, q_reg, s_tok.q)
                                 : tile_qk<T, NCH, G::Q_LDS>(kb, ck, P.Lmax, q_reg, s_tok.q);
        const bool valid = key < tlen && key >= first;
        if (key != tlen) sc[key] = valid ? s : -INFINITY;  // raw dot product
        if (valid) {
            const float m_new = fmaxf(m_run, s * P.scale_log2e);
            l_run = l_run * __builtin_amdgcn_exp2f(m_run - m_new) +
                    __builtin_amdgcn_exp2f(fmaf(s, P.scale_log2e, -m_new));
            m_run = m_new;
        }
    }
    if (token_wave) {
        const float s = token_score<T, DH>(tok, lane);
        const bool valid = tlen >= first;
        if (lane == 0) {
            sc[tlen] = valid ? s : -INFINITY;
            if (valid) {
                const float m_new = fmaxf(m_run, s * P.scale_log2e);
                l_run = l_run * __builtin_amdgcn_exp2f(m_run - m_new) +
                        __builtin_amdgcn_exp2f(fmaf(s, P.scale_log2e, -m_new));
                m_run = m_new;
            }
        } else if (tlen % kWave == 0) {
            sc[tlen + lane] = -INFINITY;
        }
        token_store<T, DH>(tok, kc_bh, vc_bh, tlen, P.Lmax, lane);
    }
    const float m_w = wave_max(m_run);
    const float l_w = wave_sum(m_run == -INFINITY ? 0.f : l_run * __builtin_amdgcn_exp2f(m_run - m_w));
    if (lane == 0) {
        s_m[wave] = m_w;
        s_l[wave] = l_w;
    }
    __syncthreads();
    if (tid == 0) {
        float M = -INFINITY, L = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) M = fmaxf(M, s_m[w]);
#pragma unroll
        for (int w = 0; w < NW; ++w)
            if (s_m[w] != -INFINITY) L += s_l[w] * __builtin_amdgcn_exp2f(s_m[w] - M);
        float* ml = P.ws_ml + ((size_t)bh * P.n_splits + split) * 2;
        ml[0] = M;
        ml[1] = L;
    }
}

template <typename T, int DH, int NW, bool BEAM>
__global__ void __launch_bounds__(NW * 64) ffa_pruned_pv_kernel(PV_HOT_PARAMS_DECL, const DecodeParams P_rest) {
    const DecodeParams P = with_pv_hot_params(P_rest, PV_HOT_PARAMS_USE);
    using G = Geo<T, DH>;
    constexpr int X = G::X, LPR = G::LPR;
    constexpr int NT = NW * 64;
    __shared__ float s_qw[NW][2 * kWave];
    __shared__ int s_qr[NW][2 * kWave];
    __shared__ float s_acc[NW][DH];
    __shared__ unsigned s_cnt[NW];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const unsigned pair = pair_of(P, blockIdx.x);
    const int bh = (int)pair, split = (int)(blockIdx.x - pair * (unsigned)P.n_splits);
    const int b = (P.seq_lengths != nullptr || BEAM) ? bh / P.H : 0;  // nobody else asks for it
    int tlen, first;
    step_bounds(P, b, tlen, first);

    const size_t head_bytes = (size_t)P.Lmax * DH * sizeof(T);
    const float* sc = P.ws_scores + (size_t)bh * P.score_stride;
    const BeamRows<BEAM> beams(P, b, bh, head_bytes);
    const int rows_per_sample = P.H * P.Lmax;

    // Tiles over keys 0..tlen: the row of slot tlen is in the sample's own cache since pass 1.
    const int ntiles = tlen / kWave + 1;
    const int tile_first = min(first / kWave, ntiles);  // tiles below are fully masked
    const int tile_lo = max(split * P.tiles_per_split, tile_first);
    const int tile_hi = min(ntiles, (split + 1) * P.tiles_per_split);
    const bool pruned = P.p > 0.f;

    // ---- the pair's max and sum from the pieces' (max, sum).  One piece per lane (two when
    // n_splits > 64), all loads in flight at once; every wave of every workgroup of the pair
    // folds them through the same reduction tree, so all arrive at bit-identical M, S ----
    static_assert(kMaxSplits <= 2 * kWave, "two pieces per lane at most");
    // The first tile's scores (and source beams) travel together with the pieces' (max, sum).
    const TileOrder order(tile_lo, tile_hi, (unsigned)blockIdx.x);
    float sr_next = (wave < order.n) ? sc[order.at(wave) * kWave + lane] : -INFINITY;
    int src_next = beams.beam(order.at(wave) * kWave + lane, wave < order.n ? tlen : 0);
    const float* ml = P.ws_ml + (size_t)bh * P.n_splits * 2;
    float m_a = -INFINITY, l_a = 0.f, m_b = -INFINITY, l_b = 0.f;
    if (lane < P.n_splits) {
        m_a = ml[2 * lane];
        l_a = ml[2 * lane + 1];
    }
    if (lane + kWave < P.n_splits) {
        m_b = ml[2 * (lane + kWave)];
        l_b = ml[2 * (lane + kWave) + 1];
    }
    float M = wave_max(fmaxf(m_a, m_b));
    const bool all_masked = (M == -INFINITY);
    if (all_masked) M = 0.f;
    const float S = wave_sum((m_a == -INFINITY ? 0.f : l_a * __builtin_amdgcn_exp2f(m_a - M)) +
                             (m_b == -INFINITY ? 0.f : l_b * __builtin_amdgcn_exp2f(m_b - M)));

    // p == 0: exact softmax weights e_i / S.  p > 0: the reference's rule
    // (attention.cu:1122-1126, :1184-1191), as in ffa_decode_wg_kernel.
    const float inv = pruned ? 1.f / (S + 1.e-6f) : (S > 0.f ? 1.f / S : 0.f);
    float thr_key = 0.f;
    if (pruned) (void)round_prob(P.p * inv, T{}, &thr_key);

    // ---- own tiles: weights (one key per lane) -> survivor queue -> surviving V rows ----
    float acc[X];
#pragma unroll
    for (int e = 0; e < X; ++e) acc[e] = 0.f;
    unsigned kept = 0;
    SurvivorQueue sq = {s_qw[wave], s_qr[wave], 0u};
    for (int idx = wave; idx < order.n; idx += NW) {
        const int key = order.at(idx) * kWave + lane;
        const float sr = sr_next;
        const int src = src_next;
        const int key_next = order.at(idx + NW) * kWave + lane;  // one tile ahead
        sr_next = (idx + NW < order.n) ? sc[key_next] : -INFINITY;
        src_next = beams.beam(key_next, idx + NW < order.n ? tlen : 0);
        const float e = (sr == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(fmaf(sr, P.scale_log2e, -M));
        const bool in_range = key >= first && key <= tlen;
        float w;
        bool drop;
        if (pruned) {
            float key_i;
            w = round_prob(e * inv, T{}, &key_i);
            drop = !in_range || (key < tlen && key_i <= thr_key);
        } else {
            w = e * inv;
            drop = !in_range;
        }
        if (key < tlen) {
            kept += drop ? 0u : 1u;
            if (P.skip_mask) P.skip_mask[(size_t)bh * P.Lmax + key] = drop ? 1 : 0;
        }
        const int row = key < tlen ? beams.v_row(src, key, rows_per_sample) : beams.own_row(tlen, rows_per_sample);
        queue_push<T, DH>(acc, sq, !drop, w, row, beams.v_group, lane);
    }
    queue_drain<T, DH>(acc, sq, beams.v_group, lane);
    if (P.skip_mask && split == 0)  // keys of fully masked leading tiles are dropped too
        for (int i = tid; i < min(tile_first * kWave, tlen); i += NT) P.skip_mask[(size_t)bh * P.Lmax + i] = 1;

    // ---- merge: lanes of a wave, waves of the workgroup, pieces of the pair ----
#pragma unroll
    for (int off = LPR; off < kWave; off <<= 1) {
#pragma unroll
        for (int e = 0; e < X; ++e) acc[e] += __shfl_xor(acc[e], off);
    }
    if (lane < G::NCH) {
#pragma unroll
        for (int e = 0; e < X; ++e) s_acc[wave][lane * X + e] = acc[e];
    }
    kept = wave_sum_u32(kept);
    if (lane == 0) s_cnt[wave] = kept;
    __syncthreads();
    if (P.kept_count && tid == 0) {
        unsigned tot = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w) tot += s_cnt[w];
        if (tot) atomicAdd(&P.kept_count[bh], tot);
    }

    T* out = reinterpret_cast<T*>(P.out) + (size_t)bh * DH;
    float* wa = P.ws_acc + ((size_t)bh * P.n_splits + split) * DH;
    for (int d = tid; d < DH; d += NT) {
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) o += s_acc[w][d];
        if (P.n_splits == 1) store_out(out, d, all_masked ? 0.f : o);
        else publish(&wa[d], o);
    }
    if (P.n_splits == 1) return;

    // Same per-wave publication protocol as finish_piece: the waves that hold output elements
    // publish them, wait for the acknowledgement, bump the pair's arrival counter; the wave
    // that sees the final count (n_splits pieces x publishing waves) sums all partials.
    constexpr int NPUB = (DH + kWave - 1) / kWave < NW ? (DH + kWave - 1) / kWave : NW;
    if (wave >= NPUB) return;
    wait_published();
    unsigned prev = 0;
    if (lane == 0)
        prev = __hip_atomic_fetch_add(&P.ws_cnt[(size_t)bh * kCounterStride], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    prev = __builtin_amdgcn_readfirstlane(prev);
    if (prev != (unsigned)(P.n_splits * NPUB - 1)) return;
    __atomic_signal_fence(__ATOMIC_SEQ_CST);  // compiler-only: keep the merge loads behind the counter
    // All loads of a batch of pieces are issued before any is consumed.
    constexpr int MB = 8;
    for (int d = lane; d < DH; d += kWave) {
        float o = 0.f;
        for (int s0 = 0; s0 < P.n_splits; s0 += MB) {
            float as[MB];
#pragma unroll
            for (int j = 0; j < MB; ++j)
                as[j] = acquire(&P.ws_acc[((size_t)bh * P.n_splits + min(s0 + j, P.n_splits - 1)) * DH + d]);
#pragma unroll
            for (int j = 0; j < MB; ++j)
                if (s0 + j < P.n_splits) o += as[j];
        }
        store_out(out, d, all_masked ? 0.f : o);
    }
    if (lane == 0) __hip_atomic_store(&P.ws_cnt[(size_t)bh * kCounterStride], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---------------------------------------------------------------------------------------
// Host-side dispatch of one element type.
static inline int check_launch() {
    return hipGetLastError() == hipSuccess ? FFA_OK : FFA_ERR_LAUNCH;
}

template <typename T, int DH, int NW, bool BEAM, bool XFORM>
static int launch_split(const DecodeParams& P, hipStream_t st) {
    const int n_split_heads = P.bh_total - P.n_whole;
    const dim3 grid((unsigned)(P.n_whole + n_split_heads * P.n_splits));
    hipLaunchKernelGGL((ffa_decode_split_kernel<T, DH, NW, BEAM, XFORM>), grid, dim3((NW + 1) * 64), 0, st,
                       HOT_PARAMS_OF(P), P);
    if (n_split_heads > 0 && P.n_splits > 1 && P.combine == FFA_COMBINE_KERNEL)
        hipLaunchKernelGGL((ffa_merge_splits_kernel<T, DH>), dim3((unsigned)n_split_heads), dim3(64), 0, st, P);
    return check_launch();
}

template <typename T, int DH, int NW, int TPK, bool BEAM, bool XFORM>
static int launch_split_tpk(const DecodeParams& P, hipStream_t st) {
    using G = Geo<T, DH>;
    // Combinations whose tile fits one group of at most 8 K loads and 8 V loads.
    if constexpr (G::NCH % TPK == 0 && G::NCH / TPK <= 8 && (kWave / TPK) % G::RPI == 0 &&
                  (kWave / TPK) / G::RPI <= 8) {
        const int n_split_heads = P.bh_total - P.n_whole;
        const dim3 grid((unsigned)(P.n_whole + n_split_heads * P.n_splits));
        hipLaunchKernelGGL((ffa_decode_split_tpk_kernel<T, DH, NW, TPK, BEAM, XFORM>), grid, dim3((NW + 1) * 64), 0, st,
                           HOT_PARAMS_OF(P), P);
        if (n_split_heads > 0 && P.n_splits > 1 && P.combine == FFA_COMBINE_KERNEL)
            hipLaunchKernelGGL((ffa_merge_splits_kernel<T, DH>), dim3((unsigned)n_split_heads), dim3(64), 0, st, P);
        return check_launch();
    } else {
        return FFA_ERR_PLAN;
    }
}

template <typename T, int DH, int NW, bool BEAM, bool XFORM>
static int launch_two_pass(const DecodeParams& P, hipStream_t st) {
    const dim3 grid((unsigned)(P.bh_total * P.n_splits));
    hipLaunchKernelGGL((ffa_scores_kernel<T, DH, NW, BEAM, XFORM>), grid, dim3(NW * 64), 0, st, HOT_PARAMS_OF(P), P);
    hipLaunchKernelGGL((ffa_pruned_pv_kernel<T, DH, NW, BEAM>), grid, dim3(NW * 64), 0, st, PV_HOT_PARAMS_OF(P), P);
    return check_launch();
}

template <typename T, int DH, int NW, bool BEAM, bool XFORM>
static int launch_wg(const DecodeParams& P, size_t lds_bytes, hipStream_t st) {
    auto kern = ffa_decode_wg_kernel<T, DH, NW, BEAM, XFORM>;
    if (lds_bytes > 48 * 1024) {
        // Raise the dynamic-LDS ceiling once per instantiation and device (gfx950: 160 KiB per
        // CU).  The attribute is a property of the loaded function, not of a stream, so the
        // call is legal while a stream is being captured.
        static bool raised[kMaxDevices] = {};
        static std::mutex raise_mutex;
        const int dev = current_device();
        if (dev < 0) return FFA_ERR_NO_DEVICE;
        std::lock_guard<std::mutex> lock(raise_mutex);
        if (!raised[dev]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    kMaxDynamicLdsBytes) != hipSuccess) {
                (void)hipGetLastError();
                return FFA_ERR_LAUNCH;
            }
            raised[dev] = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)P.bh_total), dim3(NW * 64), lds_bytes, st, HOT_PARAMS_OF(P), P);
    return check_launch();
}

template <typename T, int DH, int NW>
static int launch_floor(const DecodeParams& P, hipStream_t st) {
    const int n_split_heads = P.bh_total - P.n_whole;
    const dim3 grid((unsigned)(P.n_whole + n_split_heads * P.n_splits));
    hipLaunchKernelGGL((ffa_load_floor_kernel<T, DH, NW>), grid, dim3((NW + 1) * 64), 0, st, HOT_PARAMS_OF(P), P);
    return check_launch();
}

template <typename T, int DH, bool BEAM, bool XFORM>
static int dispatch_waves(const DecodeParams& P, const ffa_launch_plan& plan, hipStream_t st) {
    if (P.floor_probe) {
        if constexpr (!BEAM && !XFORM) {
            if (plan.kind != FFA_LAUNCH_SPLIT || plan.threads_per_key != 1) return FFA_ERR_PLAN;
            switch (plan.waves_per_wg) {
                case 2: return launch_floor<T, DH, 2>(P, st);
                case 4: return launch_floor<T, DH, 4>(P, st);
                case 8: return launch_floor<T, DH, 8>(P, st);
                default: return FFA_ERR_PLAN;
            }
        } else {
            return FFA_ERR_PLAN;
        }
    }
    if (plan.kind == FFA_LAUNCH_SPLIT && plan.threads_per_key > 1) {
        if constexpr (DH == 80) {  // 10 / 20 chunks per key do not divide among 2 or 4 lanes
            return FFA_ERR_PLAN;
        } else {
            const int key = plan.threads_per_key * 100 + plan.waves_per_wg;
            switch (key) {
                case 204: return launch_split_tpk<T, DH, 4, 2, BEAM, XFORM>(P, st);
                case 208: return launch_split_tpk<T, DH, 8, 2, BEAM, XFORM>(P, st);
                case 404: return launch_split_tpk<T, DH, 4, 4, BEAM, XFORM>(P, st);
                case 408: return launch_split_tpk<T, DH, 8, 4, BEAM, XFORM>(P, st);
                default: return FFA_ERR_PLAN;
            }
        }
    }
    if (plan.kind == FFA_LAUNCH_SPLIT) {
        switch (plan.waves_per_wg) {
            case 1: return launch_split<T, DH, 1, BEAM, XFORM>(P, st);
            case 2: return launch_split<T, DH, 2, BEAM, XFORM>(P, st);
            case 3: return launch_split<T, DH, 3, BEAM, XFORM>(P, st);
            case 4: return launch_split<T, DH, 4, BEAM, XFORM>(P, st);
            case 5: return launch_split<T, DH, 5, BEAM, XFORM>(P, st);
            case 6: return launch_split<T, DH, 6, BEAM, XFORM>(P, st);
            case 7: return launch_split<T, DH, 7, BEAM, XFORM>(P, st);
            case 8: return launch_split<T, DH, 8, BEAM, XFORM>(P, st);
            default: return FFA_ERR_PLAN;
        }
    }
    if (plan.kind == FFA_LAUNCH_TWO_PASS) {
        switch (plan.waves_per_wg) {
            case 1: return launch_two_pass<T, DH, 1, BEAM, XFORM>(P, st);
            case 2: return launch_two_pass<T, DH, 2, BEAM, XFORM>(P, st);
            case 4: return launch_two_pass<T, DH, 4, BEAM, XFORM>(P, st);
            case 8: return launch_two_pass<T, DH, 8, BEAM, XFORM>(P, st);
            default: return FFA_ERR_PLAN;
        }
    }
    const size_t lds = wg_dynamic_lds_bytes(P.t, plan.waves_per_wg, (int)sizeof(T));
    switch (plan.waves_per_wg) {
        case 1: return launch_wg<T, DH, 1, BEAM, XFORM>(P, lds, st);
        case 2: return launch_wg<T, DH, 2, BEAM, XFORM>(P, lds, st);
        case 4: return launch_wg<T, DH, 4, BEAM, XFORM>(P, lds, st);
        case 8: return launch_wg<T, DH, 8, BEAM, XFORM>(P, lds, st);
        case 16: return launch_wg<T, DH, 16, BEAM, XFORM>(P, lds, st);
        default: return FFA_ERR_PLAN;
    }
}

template <typename T, bool XFORM>
static int dispatch_head_dim(const DecodeParams& P, int head_dim, const ffa_launch_plan& plan,
                             hipStream_t st) {
    if (P.cache_indir != nullptr) {
        switch (head_dim) {
            case 64: return dispatch_waves<T, 64, true, XFORM>(P, plan, st);
            case 80: return dispatch_waves<T, 80, true, XFORM>(P, plan, st);
            case 128: return dispatch_waves<T, 128, true, XFORM>(P, plan, st);
            case 256: return dispatch_waves<T, 256, true, XFORM>(P, plan, st);
            default: return FFA_ERR_HEAD_DIM;
        }
    }
    switch (head_dim) {
        case 64: return dispatch_waves<T, 64, false, XFORM>(P, plan, st);
        case 80: return dispatch_waves<T, 80, false, XFORM>(P, plan, st);
        case 128: return dispatch_waves<T, 128, false, XFORM>(P, plan, st);
        case 256: return dispatch_waves<T, 256, false, XFORM>(P, plan, st);
        default: return FFA_ERR_HEAD_DIM;
    }
}

}  // namespace ffa
