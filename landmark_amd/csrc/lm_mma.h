// Matrix-core operand types and the layout of the packed colour-network weights, shared by
// the colour-network kernels and the appearance gather (which applies basis_mat).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/landmark_hip.h"

namespace lm_mma {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kAppDim = 27;
constexpr int kHidden = 128;
constexpr int kInDim = 150;
constexpr int kSlots1 = 80;  // layer-1 input slots per lane-half

// row of a 32x32 accumulator held in register v of a lane of half h
__host__ __device__ constexpr int row_of(int v, int h) { return 8 * (v / 4) + 4 * h + (v % 4); }

// product channel a lane-half reads for basis slot sigma: W consecutive channels per lane,
// the two halves interleaved so that a sample's pair of lanes covers 2W contiguous channels
__host__ __device__ constexpr int basis_channel(int h, int sigma, int W) {
    return 2 * W * (sigma / W) + W * h + sigma % W;
}

// G  = K slots one lane feeds per MFMA;  CW = consecutive product channels per lane and step
// NP = operand parts (2: hi/lo split);   frag = what one lane holds of an operand
template <int PREC> struct Mma;
template <> struct Mma<LM_MLP_F32> {
    static constexpr int G = 1, CW = 4, NP = 1;
    using elem = float;
    using frag = float;
    __device__ static __forceinline__ floatx16 mma(frag a, frag b, floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ void pack(const float *s, frag *o) { o[0] = s[0]; }
};
template <> struct Mma<LM_MLP_F16> {
    static constexpr int G = 8, CW = 8, NP = 1;
    using elem = _Float16;
    using frag = half8;
    __device__ static __forceinline__ floatx16 mma(frag a, frag b, floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ void pack(const float *s, frag *o) {
#pragma unroll
        for (int i = 0; i < 8; ++i) o[0][i] = (_Float16)s[i];
    }
    // two values -> one register of the operand (per part)
    __device__ static __forceinline__ void pack_pair(float x0, float x1, uint32_t *o) {
        half2v h;
        h[0] = (_Float16)x0;
        h[1] = (_Float16)x1;
        o[0] = __builtin_bit_cast(uint32_t, h);
    }
};
template <> struct Mma<LM_MLP_BF16> {
    static constexpr int G = 8, CW = 8, NP = 1;
    using elem = __bf16;
    using frag = bf16x8;
    __device__ static __forceinline__ floatx16 mma(frag a, frag b, floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    // two values -> one register with one packed conversion (converted one by one, the compiler emits a packed
    // conversion per value and a byte permute per pair)
    __device__ static __forceinline__ void pack_pair(float x0, float x1, uint32_t *o) {
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        typedef float float2v __attribute__((ext_vector_type(2)));
        const float2v v = {x0, x1};
        o[0] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
    __device__ static __forceinline__ void pack(const float *s, frag *o) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        u4 r;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t d;
            pack_pair(s[2 * i], s[2 * i + 1], &d);
            r[i] = d;
        }
        o[0] = __builtin_bit_cast(bf16x8, r);
    }
};
template <> struct Mma<LM_MLP_F16X2> {
    static constexpr int G = 8, CW = 8, NP = 2;
    using elem = _Float16;
    using frag = half8;
    __device__ static __forceinline__ floatx16 mma(frag a, frag b, floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    // x = hi + lo with hi = fp16(x), lo = fp16(x - hi); x - hi is exact in fp32.  Two values per register:
    // one packed conversion gives the hi pair, and one mixed-precision fma per value (the fp16 half of hi as
    // an operand, the result rounded to fp16 into the low or the high half) gives lo: three instructions per
    // pair instead of the seven the compiler makes of the scalar expression (convert, convert back, subtract,
    // convert, per value, plus packing).
    __device__ static __forceinline__ void pack_pair(float x0, float x1, uint32_t *o) {
        half2v h;
        h[0] = (_Float16)x0;
        h[1] = (_Float16)x1;
        const uint32_t hb = __builtin_bit_cast(uint32_t, h);
        uint32_t l;
        asm("v_fma_mixlo_f16 %0, %1, -1.0, %2 op_sel_hi:[1,0,0]" : "=v"(l) : "v"(hb), "v"(x0));
        asm("v_fma_mixhi_f16 %0, %1, -1.0, %2 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(l) : "v"(hb), "v"(x1));
        o[0] = hb;
        o[1] = l;
    }
    __device__ static __forceinline__ void pack(const float *s, frag *o) {
        typedef uint32_t u4 __attribute__((ext_vector_type(4)));
        u4 hi, lo;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t d[2];
            pack_pair(s[2 * i], s[2 * i + 1], d);
            hi[i] = d[0];
            lo[i] = d[1];
        }
        o[0] = __builtin_bit_cast(half8, hi);
        o[1] = __builtin_bit_cast(half8, lo);
    }
};

// ---- layout of the packed weight buffer (offsets in bytes, 256-byte aligned) ----------------
struct PackLayout {
    size_t basis, w1, b1, w2, b2, w3, b3, total;
};
__host__ __device__ inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
inline PackLayout pack_layout(int prec, int K) {
    const size_t E = (prec == LM_MLP_F32 ? 4 : 2) * (prec == LM_MLP_F16X2 ? 2 : 1);
    PackLayout L;
    size_t o = 0;
    L.basis = o; o = align256(o + (size_t)32 * K * E);
    L.w1 = o; o = align256(o + (size_t)4 * kSlots1 * 64 * E);
    L.b1 = o; o = align256(o + 4 * 2 * 16 * sizeof(float));
    L.w2 = o; o = align256(o + (size_t)4 * 64 * 64 * E);
    L.b2 = o; o = align256(o + 4 * 2 * 16 * sizeof(float));
    L.w3 = o; o = align256(o + (size_t)64 * 64 * E);
    L.b3 = o; o = align256(o + 2 * 16 * sizeof(float));
    L.total = o;
    return L;
}

}  // namespace lm_mma
