// Device-side building blocks for the gfx950 decode-attention kernels:
// wave64 DPP reductions, 16-byte chunk dot/fma for fp16 and fp32, fp16 rounding helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ffa {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

// bfloat16 element (1-8-7), carried as its bit pattern like fp16 is carried as uint16_t.
struct bf16_t {
    uint16_t bits;
};
__device__ __forceinline__ float bf16_to_float(uint16_t b) {
    return __builtin_bit_cast(float, (uint32_t)b << 16);
}
// Round-to-nearest-even; NaN stays NaN (quiet).
__device__ __forceinline__ uint16_t float_to_bf16(float f) {
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;

// ---------------------------------------------------------------------------------------
// DPP lane exchange.  ctrl values: quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E,
// row_half_mirror = 0x141, row_mirror = 0x140.  After the four steps every lane of a
// 16-lane row holds that row's reduction; the four rows are merged through readlane.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float x) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}

// __builtin_amdgcn_readlane is typed int -> int: move the bits, not the value.
__device__ __forceinline__ float readlane_f32(float x, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}

__device__ __forceinline__ float wave_max(float x) {
    x = fmaxf(x, dpp_f32<0xB1>(x));
    x = fmaxf(x, dpp_f32<0x4E>(x));
    x = fmaxf(x, dpp_f32<0x141>(x));
    x = fmaxf(x, dpp_f32<0x140>(x));
    const float a = readlane_f32(x, 0), b = readlane_f32(x, 16);
    const float c = readlane_f32(x, 32), d = readlane_f32(x, 48);
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

__device__ __forceinline__ float wave_sum(float x) {
    x += dpp_f32<0xB1>(x);
    x += dpp_f32<0x4E>(x);
    x += dpp_f32<0x141>(x);
    x += dpp_f32<0x140>(x);
    const float a = readlane_f32(x, 0), b = readlane_f32(x, 16);
    const float c = readlane_f32(x, 32), d = readlane_f32(x, 48);
    return (a + b) + (c + d);
}

__device__ __forceinline__ unsigned wave_sum_u32(unsigned x) {
    // counts are < 2^24 per wave-step, exact in the float pipeline
    return (unsigned)wave_sum((float)x);
}

// ---------------------------------------------------------------------------------------
// Element traits: X = elements per 16-byte chunk.
template <typename T> struct Elem;
template <> struct Elem<uint16_t> { static constexpr int X = 8; };
template <> struct Elem<float>    { static constexpr int X = 4; };
template <> struct Elem<bf16_t>   { static constexpr int X = 8; };

// 16-byte accesses to the KV caches carry the non-temporal hint (`nt`): every byte is used
// once per step, and keeping the stream out of the caches' replacement order is worth 9-10 %
// of the step time on MI355X (headline shape 16.9 -> 15.5 us, GPT-J shape 50.9 -> 46.0 us).
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld16(const void* p) {
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st16(void* p, const uint4& v) {
    *reinterpret_cast<uint4*>(p) = v;
}
// The same store written through to memory (`sc0 sc1`): nothing of it stays dirty in the L2.  In a
// launch that consists of split pairs only -- few workgroups, a kernel that ends on a chain of
// small stores -- this shortens the end of the kernel (B = 1 and 2 at 1000 keys: -0.1 us per
// launch); with whole pairs in the launch it costs more than it saves (320 pairs: +0.25 us).
__device__ __forceinline__ void st16_through(void* p, const uint4& v) {
    u32x4_t w = {v.x, v.y, v.z, v.w};
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(p), "v"(w) : "memory");
}
// Streaming store for cache construction (with ld16 on the read side: 8-10 % over plain
// accesses; for the single appended row of a decode step the hint makes no difference).
__device__ __forceinline__ void st16_stream(void* p, const uint4& v) {
    u32x4_t w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, reinterpret_cast<u32x4_t*>(p));
}

// acc += <a, b> over one 16-byte chunk, fp32 accumulation.
__device__ __forceinline__ float dot_chunk(const uint4& a, const uint4& b, float acc, uint16_t) {
    const half2_t* x = reinterpret_cast<const half2_t*>(&a);
    const half2_t* y = reinterpret_cast<const half2_t*>(&b);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2(x[i], y[i], acc, false);
    return acc;
}
__device__ __forceinline__ float dot_chunk(const uint4& a, const uint4& b, float acc, float) {
    const float* x = reinterpret_cast<const float*>(&a);
    const float* y = reinterpret_cast<const float*>(&b);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = fmaf(x[i], y[i], acc);
    return acc;
}

__device__ __forceinline__ float dot_chunk(const uint4& a, const uint4& b, float acc, bf16_t) {
    const bf16x2_t* x = reinterpret_cast<const bf16x2_t*>(&a);
    const bf16x2_t* y = reinterpret_cast<const bf16x2_t*>(&b);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc = __builtin_amdgcn_fdot2_f32_bf16(x[i], y[i], acc, false);
    return acc;
}

// acc[0..X) += p * chunk, fp32 accumulation.
__device__ __forceinline__ void fma_chunk(float (&acc)[8], float p, const uint4& v, uint16_t) {
    const _Float16* h = reinterpret_cast<const _Float16*>(&v);
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = fmaf(p, (float)h[i], acc[i]);
}
__device__ __forceinline__ void fma_chunk(float (&acc)[4], float p, const uint4& v, float) {
    const float* f = reinterpret_cast<const float*>(&v);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = fmaf(p, f[i], acc[i]);
}

__device__ __forceinline__ void fma_chunk(float (&acc)[8], float p, const uint4& v, bf16_t) {
    const uint32_t* w = reinterpret_cast<const uint32_t*>(&v);
#pragma unroll
    for (int i = 0; i < 4; ++i) {   // a bf16 is the upper half of an fp32
        acc[2 * i] = fmaf(p, __builtin_bit_cast(float, w[i] << 16), acc[2 * i]);
        acc[2 * i + 1] = fmaf(p, __builtin_bit_cast(float, w[i] & 0xffff0000u), acc[2 * i + 1]);
    }
}

// Final store of one output element.
__device__ __forceinline__ void store_out(uint16_t* out, int idx, float v) {
    const _Float16 h = (_Float16)v;  // round-to-nearest-even
    out[idx] = __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ void store_out(float* out, int idx, float v) { out[idx] = v; }
__device__ __forceinline__ void store_out(bf16_t* out, int idx, float v) { out[idx].bits = float_to_bf16(v); }
// Written through (see st16_through).
__device__ __forceinline__ void store_out_through(uint16_t* out, int idx, float v) {
    const unsigned bits = __builtin_bit_cast(uint16_t, (_Float16)v);
    asm volatile("global_store_short %0, %1, off sc0 sc1" ::"v"(out + idx), "v"(bits) : "memory");
}
__device__ __forceinline__ void store_out_through(float* out, int idx, float v) {
    asm volatile("global_store_dword %0, %1, off sc0 sc1" ::"v"(out + idx), "v"(v) : "memory");
}
__device__ __forceinline__ void store_out_through(bf16_t* out, int idx, float v) {
    const unsigned bits = float_to_bf16(v);
    asm volatile("global_store_short %0, %1, off sc0 sc1" ::"v"(out + idx), "v"(bits) : "memory");
}

// ---------------------------------------------------------------------------------------
// The reference's pruning predicate.
//   fp32: leq(a, b) = a <= b.
//   fp16: leq(uint16_t a, uint16_t b) = __hle(__half(a), __half(b)), where __half(ushort)
//         converts the integer VALUE of the bit pattern with round-to-nearest-even, so the
//         comparison is between the two bit patterns rounded to 11 significant bits.
// round_prob returns the probability as the kernels will use it (rounded to T); its
// companion `key` is the quantity the predicate compares.
__device__ __forceinline__ float round_prob(float x, uint16_t, float* key) {
    const _Float16 h = (_Float16)x;
    const uint16_t bits = __builtin_bit_cast(uint16_t, h);
    *key = (float)(_Float16)(float)bits;  // numeric value of the pattern, rounded to fp16
    return (float)h;
}
__device__ __forceinline__ float round_prob(float x, float, float* key) {
    *key = x;
    return x;
}
// bf16: the reference never enables its bf16 build, so there is no bit-pattern quirk to follow:
// the probability rounded to bf16 is compared numerically, as the fp32 rule does.
__device__ __forceinline__ float round_prob(float x, bf16_t, float* key) {
    const float r = bf16_to_float(float_to_bf16(x));
    *key = r;
    return r;
}

}  // namespace ffa
