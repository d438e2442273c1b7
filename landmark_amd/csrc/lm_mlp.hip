// Part 3: positional encoding + colour network (and the basis_mat projection) on the
// matrix cores.
//
// One wave owns 32 samples.  All products are computed "transposed": the weight matrix
// is the A operand (32 output rows per MFMA), the 32 samples are the columns, so the
// 32x32 accumulator of one layer already has the register layout the next layer needs as
// its B operand (lane = sample, registers = features).  Activations therefore never leave
// the register file between the encoding and the three layers.  The order of the K
// dimension is free in a dot product, so the host packs every weight matrix into the exact
// per-lane fragment order the kernel consumes (lm_mlp_pack); layers 1 and 2 are copied to
// LDS once per workgroup and every MFMA reads one contiguous, conflict-free fragment.
//
// Arithmetic modes (accumulation is always fp32):
//   F32    v_mfma_f32_32x32x2_f32
//   F16    v_mfma_f32_32x32x16_f16,  BF16  v_mfma_f32_32x32x16_bf16
//   F16X2  every operand x is split into fp16 parts x = hi + lo; a*b is evaluated as
//          hi*hi + lo*hi + hi*lo with three fp16 MFMAs (products of fp16 numbers are exact
//          in fp32), which keeps ~21 mantissa bits at a quarter of the fp32 MFMA cost.
//
// Register layout of a 32x32 fp32 accumulator (all 32x32 MFMA shapes): lane l holds column
// j = l%32; with h = l/32 its register v (0..15) is row 8*(v/4) + 4*h + v%4.
//
// Row assignment of the network input: rows 0..26 are the 27 appearance features, rows
// 28..30 the view direction, rows 27 and 31 are zero.  Each lane thus owns 16 raw values
// (15 real); the input is built per lane as five groups of 16: raw, sin(raw), cos(raw),
// sin(2 raw), cos(2 raw) = 80 slots, 160 per sample (150 real, the rest meet zero
// weights).  Reference input order it is mapped to: app/models/mlp_render_fea.py:55-65
// with app/tools/utils.py:42-48.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <cmath>
#include <cstring>

#include "lm_common.h"
#include "lm_mma.h"

#ifndef LM_MLP16_THREADS
#define LM_MLP16_THREADS 512
#endif
#ifndef LM_MLP_NCB
#define LM_MLP_NCB 2
#endif
// split-fp16 mode: eight waves with one column block each beat four waves with two (the second wave of a SIMD
// covers the first one's waits for LDS and memory)
#ifndef LM_MLPX2_THREADS
#define LM_MLPX2_THREADS 512
#endif
#ifndef LM_MLPX2_NCB
#define LM_MLPX2_NCB 1
#endif
#ifndef LM_MLPX2_NB
#define LM_MLPX2_NB 1  // split mode: one accumulator block at a time keeps the wave inside 256 registers
#endif
#ifndef LM_MLP16_NB1
#define LM_MLP16_NB1 4  // 16-bit modes with one column block: row blocks per pass
#endif

#ifndef LM_MLP_STREAM
#define LM_MLP_STREAM 1  // 16-bit and split modes: the layers as one stream of matrix steps (colour_layers_stream)
#endif
#ifndef LM_MLP_STREAM_X2
#define LM_MLP_STREAM_X2 0
#endif
#ifndef LM_MLP_PF_X2
#define LM_MLP_PF_X2 1
#endif
#ifndef LM_MLP_PRIO
#define LM_MLP_PRIO 1  // wave priority while it multiplies (its MFMAs go before the other wave's encoding)
#endif
#ifndef LM_MLP_PF
#define LM_MLP_PF 2  // steps a weight fragment is requested ahead of its MFMAs
#endif

namespace {

using namespace lm_mma;

// 16-bit and split modes: 8 waves per workgroup (two per SIMD, 256 registers each); the fp32
// mode needs the full register file of a SIMD per wave
template <int PREC> struct MlpBlock {
    static constexpr int N = (PREC == LM_MLP_F16 || PREC == LM_MLP_BF16) ? LM_MLP16_THREADS
                             : PREC == LM_MLP_F16X2                        ? LM_MLPX2_THREADS
                                                                           : 256;
    // 32-sample column blocks per wave
    static constexpr int NCB = PREC == LM_MLP_F32 ? 1 : (PREC == LM_MLP_F16X2 ? LM_MLPX2_NCB : LM_MLP_NCB);
};

// ---- host-side packing ----------------------------------------------------------------------
// column of the reference's 150-wide input row that feeds slot (h, group, v); -1 = none
inline int input_column(int h, int grp, int v) {
    const int row = row_of(v, h);
    const int F = 2;  // fea_pe = view_pe = 2
    if (row < kAppDim) {
        const int d = row;
        switch (grp) {
            case 0: return d;
            case 1: return kAppDim + 3 + d * F + 0;
            case 2: return kAppDim + 3 + kAppDim * F + d * F + 0;
            case 3: return kAppDim + 3 + d * F + 1;
            default: return kAppDim + 3 + kAppDim * F + d * F + 1;
        }
    }
    if (row >= 28 && row <= 30) {
        const int d = row - 28, base = kAppDim + 3 + 2 * kAppDim * F;
        switch (grp) {
            case 0: return kAppDim + d;
            case 1: return base + d * F + 0;
            case 2: return base + 3 * F + d * F + 0;
            case 3: return base + d * F + 1;
            default: return base + 3 * F + d * F + 1;
        }
    }
    return -1;
}

template <typename E> inline E to_elem(float x);
template <> inline float to_elem<float>(float x) { return x; }
template <> inline _Float16 to_elem<_Float16>(float x) { return (_Float16)x; }
template <> inline __bf16 to_elem<__bf16>(float x) { return (__bf16)x; }

// Writes fragments [block][step][part][lane][G]; value(block, i, h, sigma) gives
// A[row i of the block][slot].  parts = 2 stores (hi, lo) with hi = E(x), lo = E(x - hi).
template <typename E, typename F>
void pack_matrix(E *dst, int n_blocks, int n_slots, int G, int parts, F value) {
    const int steps = n_slots / G;
    for (int fb = 0; fb < n_blocks; ++fb)
        for (int t = 0; t < steps; ++t)
            for (int lane = 0; lane < 64; ++lane)
                for (int e = 0; e < G; ++e) {
                    const int i = lane % 32, h = lane / 32;
                    const float x = value(fb, i, h, t * G + e);
                    const E hi = to_elem<E>(x);
                    const size_t base = (((size_t)fb * steps + t) * parts) * 64;
                    dst[(base + lane) * G + e] = hi;
                    if (parts == 2) dst[(base + 64 + lane) * G + e] = to_elem<E>(x - (float)hi);
                }
}

template <typename E>
void pack_all(int K, int G, int CW, int parts, const PackLayout &L, const float *basis, const float *w1,
              const float *b1, const float *w2, const float *b2, const float *w3, const float *b3, char *out) {
    pack_matrix<E>((E *)(out + L.basis), 1, K / 2, G, parts, [&](int, int i, int h, int s) {
        return i < kAppDim ? basis[(size_t)i * K + basis_channel(h, s, CW)] : 0.0f;
    });
    pack_matrix<E>((E *)(out + L.w1), 4, kSlots1, G, parts, [&](int fb, int i, int h, int s) {
        const int col = input_column(h, s / 16, s % 16);
        return col < 0 ? 0.0f : w1[(size_t)(32 * fb + i) * kInDim + col];
    });
    pack_matrix<E>((E *)(out + L.w2), 4, 64, G, parts, [&](int fb, int i, int h, int s) {
        return w2[(size_t)(32 * fb + i) * kHidden + 32 * (s / 16) + row_of(s % 16, h)];
    });
    pack_matrix<E>((E *)(out + L.w3), 1, 64, G, parts, [&](int, int i, int h, int s) {
        return i < 3 ? w3[(size_t)i * kHidden + 32 * (s / 16) + row_of(s % 16, h)] : 0.0f;
    });
    float *pb1 = (float *)(out + L.b1), *pb2 = (float *)(out + L.b2), *pb3 = (float *)(out + L.b3);
    for (int fb = 0; fb < 4; ++fb)
        for (int h = 0; h < 2; ++h)
            for (int v = 0; v < 16; ++v) {
                pb1[(fb * 2 + h) * 16 + v] = b1 ? b1[32 * fb + row_of(v, h)] : 0.0f;
                pb2[(fb * 2 + h) * 16 + v] = b2 ? b2[32 * fb + row_of(v, h)] : 0.0f;
            }
    for (int h = 0; h < 2; ++h)
        for (int v = 0; v < 16; ++v) pb3[h * 16 + v] = (b3 && row_of(v, h) < 3) ? b3[row_of(v, h)] : 0.0f;
}

// ---- device side ---------------------------------------------------------------------------
__device__ __forceinline__ floatx16 load_bias(const float *b, int idx) {
    floatx16 a;
    const float4 *p = reinterpret_cast<const float4 *>(b + idx * 16);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float4 t = p[i];
        a[4 * i] = t.x; a[4 * i + 1] = t.y; a[4 * i + 2] = t.z; a[4 * i + 3] = t.w;
    }
    return a;
}

// sin and cos of x to float rounding for |x| <= 8192 (three-constant Cody-Waite reduction by
// pi/2, then the minimax polynomials on [-pi/4, pi/4]); callers redo larger arguments with the
// library routines (kSincosMax), outside their hot loop.
constexpr float kSincosMax = 8192.0f;
__device__ __forceinline__ void sincos_f32(float x, float &s, float &c) {
    const float k = rintf(x * 0.636619772367581f);
    float r = fmaf(-k, 1.5703125f, x);
    r = fmaf(-k, 4.837512969970703125e-4f, r);
    r = fmaf(-k, 7.54978995489188216e-8f, r);
    const float r2 = r * r;
    float ps = fmaf(r2, -1.9515295891e-4f, 8.3321608736e-3f);
    ps = fmaf(ps, r2, -1.6666654611e-1f);
    ps = fmaf(ps * r2, r, r);
    float pc = fmaf(r2, 2.443315711809948e-5f, -1.388731625493765e-3f);
    pc = fmaf(pc, r2, 4.166664568298827e-2f);
    pc = fmaf(pc * r2, r2, fmaf(-0.5f, r2, 1.0f));
    const int q = (int)k & 3;
    const float ss = (q & 1) ? pc : ps, cc = (q & 1) ? ps : pc;
    s = (q & 2) ? -ss : ss;
    c = ((q + 1) & 2) ? -cc : cc;
}

// sin and cos through the hardware functions (argument in revolutions) after a two-constant reduction by
// 2 pi: within 4.3e-7 of the exact values for |x| <= 8192 (measured over 2^24 arguments per range), seven
// instructions per value.  Used by the split-fp16 mode, whose products carry about 21 mantissa bits anyway.
__device__ __forceinline__ void sincos_hw(float x, float &s, float &c) {
    const float k = rintf(x * 0.15915494309189535f);
    float r = fmaf(-k, 6.28125f, x);
    r = fmaf(-k, 1.9353071795864769e-3f, r);
    const float t = r * 0.15915494309189535f;
    s = __builtin_amdgcn_sinf(t);
    c = __builtin_amdgcn_cosf(t);
}

// One dense layer on the wave's 32*NCB samples: acc[fb][cb] (+)= W[32*fb .. +32, :] x B[cb]
// for NB row blocks and NCB column blocks of 32 samples.  Every weight fragment read from
// LDS feeds NCB MFMAs (an A fragment is 1 KB per 32-cycle MFMA, which is exactly the LDS
// bandwidth of a CU when nothing is reused).  Steps run outermost so that the NB*NCB
// accumulator chains are independent.  The fragments of step t+PF are requested while
// step t multiplies; scheduling barriers keep the reads ahead of the MFMAs and stop the
// compiler from hoisting every read to the top.
template <int PREC, int NB, int NCB, int T, int PF>
__device__ __forceinline__ void dense_layer(const typename Mma<PREC>::frag *W0, int fb0, unsigned lane,
                                            const typename Mma<PREC>::frag (*b)[T][Mma<PREC>::NP],
                                            floatx16 (*acc)[NCB]) {
    using M = Mma<PREC>;
    using frag = typename M::frag;
    constexpr int NP = M::NP;
    const frag *W = W0 + (size_t)fb0 * T * NP * 64 + lane;
    frag a[T][NB][NP];
#pragma unroll
    for (int t = 0; t < PF && t < T; ++t)
#pragma unroll
        for (int fb = 0; fb < NB; ++fb)
#pragma unroll
            for (int pt = 0; pt < NP; ++pt) a[t][fb][pt] = W[((fb * T + t) * NP + pt) * 64];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (t + PF < T) {
#pragma unroll
            for (int fb = 0; fb < NB; ++fb)
#pragma unroll
                for (int pt = 0; pt < NP; ++pt) a[t + PF][fb][pt] = W[((fb * T + t + PF) * NP + pt) * 64];
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int fb = 0; fb < NB; ++fb)
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                acc[fb][cb] = M::mma(a[t][fb][0], b[cb][t][0], acc[fb][cb]);
                if constexpr (NP == 2) {
                    acc[fb][cb] = M::mma(a[t][fb][1], b[cb][t][0], acc[fb][cb]);
                    acc[fb][cb] = M::mma(a[t][fb][0], b[cb][t][1], acc[fb][cb]);
                }
            }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// max(x, 0) for finite floats as one integer instruction (negative floats are negative integers)
__device__ __forceinline__ float relu_f32(float x) {
    return __builtin_bit_cast(float, max(__builtin_bit_cast(int, x), 0));
}

// relu(acc) of one row block -> G-slot B fragments of the next layer
template <int PREC>
__device__ __forceinline__ void relu_to_frags(const floatx16 &acc, typename Mma<PREC>::frag (*out)[Mma<PREC>::NP]) {
    using M = Mma<PREC>;
    constexpr int G = M::G;
    if constexpr (PREC == LM_MLP_F16) {
        // round first, then clamp two halves per instruction: rounding is monotone and keeps zero, so
        // this equals rounding relu(x)
        float hv[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) hv[v] = acc[v];
#pragma unroll
        for (int u = 0; u < 16 / G; ++u) {
            M::pack(hv + u * G, out[u]);
            const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
            out[u][0] = __builtin_elementwise_max(out[u][0], zero);
        }
    } else {
        float hv[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) hv[v] = relu_f32(acc[v]);
#pragma unroll
        for (int u = 0; u < 16 / G; ++u) M::pack(hv + u * G, out[u]);
    }
}

// raw[cb][16] (the lane's 16 input rows of each of its NCB samples) -> the first layer's B fragments: per lane
// five groups of 16 slots (raw, sin, cos, sin 2x, cos 2x)
template <int PREC, int NCB>
__device__ __forceinline__ void encode_inputs(const float (*raw)[16],
                                              typename Mma<PREC>::frag (*bfrag)[kSlots1 / Mma<PREC>::G][Mma<PREC>::NP]) {
    using M = Mma<PREC>;
    constexpr int G = M::G, T1 = kSlots1 / G;
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        float slots[kSlots1];
        constexpr bool kExact = PREC == LM_MLP_F32 || PREC == LM_MLP_F16X2;
        bool big = false;
        // row 27 / 31 (v = 15) is zero and meets zero weights
        slots[15] = 0.0f; slots[31] = 0.0f; slots[47] = 0.0f; slots[63] = 0.0f; slots[79] = 0.0f;
#pragma unroll
        for (int v = 0; v < 15; ++v) {
            const float x = raw[cb][v];
            float s1, c1;
            if (PREC == LM_MLP_F16X2) {
                sincos_hw(x, s1, c1);
                big |= fabsf(x) > kSincosMax;
            } else if (kExact) {
                sincos_f32(x, s1, c1);
                big |= fabsf(x) > kSincosMax;
            } else {
                s1 = __sinf(x); c1 = __cosf(x);
            }
            const float s2 = 2.0f * s1 * c1;
            const float c2 = fmaf(-2.0f * s1, s1, 1.0f);
            slots[v] = x; slots[16 + v] = s1; slots[32 + v] = c1; slots[48 + v] = s2; slots[64 + v] = c2;
        }
        if (kExact && __builtin_expect(big, 0)) {
            // arguments beyond the fast reduction's range: library routines, rarely if ever taken
#pragma unroll
            for (int v = 0; v < 15; ++v) {
                const float x = raw[cb][v];
                if (fabsf(x) > kSincosMax) {
                    const float s1 = sinf(x), c1 = cosf(x);
                    slots[16 + v] = s1; slots[32 + v] = c1;
                    slots[48 + v] = 2.0f * s1 * c1; slots[64 + v] = fmaf(-2.0f * s1, s1, 1.0f);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < T1; ++t) M::pack(slots + t * G, bfrag[cb][t]);
    }
}

// first-layer B fragments -> rgb in out[cb][0..2] (meaningful on lanes with h == 0)
template <int PREC, int NCB>
__device__ __forceinline__ void colour_layers(const typename Mma<PREC>::frag *w1, const typename Mma<PREC>::frag *w2,
                                              const typename Mma<PREC>::frag *w3, const float *b1, const float *b2,
                                              const float *b3,
                                              const typename Mma<PREC>::frag (*bfrag)[kSlots1 / Mma<PREC>::G][Mma<PREC>::NP],
                                              unsigned lane, float (*out)[3]) {
    using M = Mma<PREC>;
    using frag = typename M::frag;
    constexpr int G = M::G, NP = M::NP;
    constexpr int T1 = kSlots1 / G, T2 = 64 / G;
    // row blocks per pass: NB*NCB accumulators of 16 registers
    constexpr int NB = NCB == 1 ? (PREC == LM_MLP_F16X2 ? LM_MLPX2_NB : (PREC == LM_MLP_F32 ? 4 : LM_MLP16_NB1)) : 2;
    constexpr int PF = G == 1 ? 4 : 1;
    const unsigned h = lane >> 5;
    frag b2frag[NCB][T2][NP];
#pragma unroll
    for (int pass = 0; pass < 4 / NB; ++pass) {
        floatx16 acc[NB][NCB];
#pragma unroll
        for (int fb = 0; fb < NB; ++fb)
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) acc[fb][cb] = load_bias(b1, (pass * NB + fb) * 2 + h);
        dense_layer<PREC, NB, NCB, T1, PF>(w1, pass * NB, lane, bfrag, acc);
#pragma unroll
        for (int fb = 0; fb < NB; ++fb)
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) relu_to_frags<PREC>(acc[fb][cb], &b2frag[cb][(pass * NB + fb) * (16 / G)]);
    }
    frag b3frag[NCB][T2][NP];
#pragma unroll
    for (int pass = 0; pass < 4 / NB; ++pass) {
        floatx16 acc[NB][NCB];
#pragma unroll
        for (int fb = 0; fb < NB; ++fb)
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) acc[fb][cb] = load_bias(b2, (pass * NB + fb) * 2 + h);
        dense_layer<PREC, NB, NCB, T2, PF>(w2, pass * NB, lane, b2frag, acc);
#pragma unroll
        for (int fb = 0; fb < NB; ++fb)
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) relu_to_frags<PREC>(acc[fb][cb], &b3frag[cb][(pass * NB + fb) * (16 / G)]);
    }
    floatx16 acc3[1][NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) acc3[0][cb] = load_bias(b3, h);
    dense_layer<PREC, 1, NCB, T2, (G == 1 ? 8 : 4)>(w3, 0, lane, b3frag, acc3);
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            // sigmoid; the hardware reciprocal is within one unit in the last place, enough for every mode
            const float e = (PREC == LM_MLP_F32 || PREC == LM_MLP_F16X2) ? expf(-acc3[0][cb][k]) : __expf(-acc3[0][cb][k]);
            out[cb][k] = __builtin_amdgcn_rcpf(1.0f + e);
        }
}

// relu of two accumulator values (registers 2 q, 2 q + 1) -> register q % 4 of the next layer's B fragment q / 4
// (per part)
template <int PREC>
__device__ __forceinline__ void relu_pair(const floatx16 &acc, int q, uint32_t (*out)[4]) {
    using M = Mma<PREC>;
    uint32_t d[M::NP];
    if constexpr (PREC == LM_MLP_F16) {
        // round first, then clamp two halves with one instruction (rounding is monotone and keeps zero)
        M::pack_pair(acc[2 * q], acc[2 * q + 1], d);
        const half2v zero = {0, 0};
        d[0] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(half2v, d[0]), zero));
    } else if constexpr (PREC == LM_MLP_BF16) {
        // round first, then clamp both halves with one packed integer maximum: a negative bf16 number is a negative
        // 16-bit integer, a non-negative one keeps its bits
        typedef short short2v __attribute__((ext_vector_type(2)));
        M::pack_pair(acc[2 * q], acc[2 * q + 1], d);
        const short2v zero = {0, 0};
        d[0] = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(short2v, d[0]), zero));
    } else {
        M::pack_pair(relu_f32(acc[2 * q]), relu_f32(acc[2 * q + 1]), d);
    }
#pragma unroll
    for (int pt = 0; pt < M::NP; ++pt) out[pt][q % 4] = d[pt];
}

// The three layers of the 16-bit and split modes as one stream of matrix steps.  A "job" is one block of 32 output
// rows of one layer (4 + 4 + 1 jobs); its NCB accumulators alternate between two register sets, so that the
// conversion of job j's results (relu, round, split) is issued in small groups behind the MFMAs of job j + 1's first
// steps and runs under them: a matrix instruction occupies its pipe for 32 cycles while the wave goes on issuing a
// few ordinary vector instructions.  Once a set's results are converted, the bias of the job after next is read from
// LDS straight into it, half a job before its first MFMA.  The K order of a layer is the order its inputs become
// ready in: the last job of a layer is converted while the next layer's first job multiplies the K slices of the
// earlier jobs.  Weight fragments sit in LDS in exactly this step order (row block, step, part), one pointer walks
// them; they are requested PF steps ahead, across job and layer boundaries.
template <int PREC, int NCB, int PF>
__device__ __forceinline__ void colour_layers_stream(const typename Mma<PREC>::frag *w1, const typename Mma<PREC>::frag *w2,
                                                     const typename Mma<PREC>::frag *w3, const float *b1, const float *b2,
                                                     const float *b3,
                                                     const typename Mma<PREC>::frag (*bfrag)[kSlots1 / Mma<PREC>::G][Mma<PREC>::NP],
                                                     unsigned lane, float (*out)[3]) {
    using M = Mma<PREC>;
    using frag = typename M::frag;
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    constexpr int G = M::G, NP = M::NP;
    static_assert(G == 8, "eight K slots per lane and step");
    constexpr int T1 = kSlots1 / G, T2 = 64 / G;
    constexpr int G1 = 4 * T1, G2 = 4 * T2, GT = G1 + G2 + T2;  // steps of layer 1, layer 2, all
    constexpr int R = PF + 1;                                    // fragment ring
    constexpr int NM = NCB * (NP == 2 ? 3 : 1);                  // MFMAs per step
    const unsigned h = lane >> 5;
    uint32_t hid1[NCB][T2][NP][4], hid2[NCB][T2][NP][4];
    floatx16 acc[2][NCB];
    frag a[R][NP];
    // The fragments of the layers lie one behind the other in LDS (w2 follows w1, w3 follows w2 where it is resident),
    // in the order of the steps: a running offset walks them, advanced once per request and hidden from the compiler,
    // which would otherwise form one address register per fragment beyond the 64 KB an instruction's offset reaches,
    // lift them all out of the tile loop and spill them.
    const bool w3_follows = w3 == w2 + (size_t)G2 * NP * 64;
    typedef const frag __attribute__((address_space(3))) *lds_frag;
    uint32_t walk = (uint32_t)(uintptr_t)(lds_frag)w1 + lane * (uint32_t)sizeof(frag);  // LDS byte address
    uint32_t walk3 = lane;                                                            // fragments of w3 in global memory
    auto request = [&](int g) {  // g is a constant at every call; requests come in the order of g
        if (g < G1 + G2 || w3_follows) {
            const lds_frag p = (lds_frag)(uintptr_t)walk;
#pragma unroll
            for (int pt = 0; pt < NP; ++pt) a[g % R][pt] = p[pt * 64];
            walk += NP * 64 * (uint32_t)sizeof(frag);
            asm volatile("" : "+v"(walk));
        } else {
            const frag *p = w3 + walk3;
#pragma unroll
            for (int pt = 0; pt < NP; ++pt) a[g % R][pt] = p[pt * 64];
            walk3 += NP * 64;
            asm volatile("" : "+v"(walk3));
        }
    };
    auto request_bias = [&](int job) {  // into the accumulators of `job`
        const floatx16 b = load_bias(job < 4 ? b1 : (job < 8 ? b2 : b3), job == 8 ? (int)h : (job & 3) * 2 + (int)h);
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) acc[job & 1][cb] = b;
    };
    request_bias(0);
    static_for<PF>([&](auto gc) { request(decltype(gc)::value); });
    static_for<GT>([&](auto gc) {
        constexpr int g = decltype(gc)::value;
        constexpr int layer = g < G1 ? 0 : (g < G1 + G2 ? 1 : 2);
        constexpr int job = layer == 0 ? g / T1 : (layer == 1 ? 4 + (g - G1) / T2 : 8);
        constexpr int t = layer == 0 ? g % T1 : (g - G1) % T2;
        constexpr int set = job & 1;
        // conversion slots: PPM register pairs behind every MFMA from the second step on, until the previous job's
        // 8 NCB pairs are done
        constexpr int PPM = NP == 2 ? 1 : 2, PAIRS = 8 * NCB;
        constexpr int TC = (PAIRS + PPM * NM - 1) / (PPM * NM);  // steps the conversions take
        constexpr bool converting = job > 0 && t >= 1 && t <= TC;
        if constexpr (g + PF < GT) request(g + PF);
        if constexpr (job < 8 && t == (job == 0 ? 1 : TC + 1)) request_bias(job + 1);
        static_for<NM>([&](auto mc) {
            constexpr int m = decltype(mc)::value, cb = NP == 2 ? m / 3 : m, part = NP == 2 ? m % 3 : 0;
            const frag b = layer == 0 ? bfrag[cb][t][part == 2 ? 1 : 0]
                                      : __builtin_bit_cast(frag, *reinterpret_cast<const u4 *>(layer == 1 ? hid1[cb][t][part == 2 ? 1 : 0] : hid2[cb][t][part == 2 ? 1 : 0]));
            acc[set][cb] = M::mma(a[g % R][part == 1 ? 1 : 0], b, acc[set][cb]);
            // the previous job's results, from the second step on (its last MFMAs have left the pipe by then): a few
            // register pairs behind every MFMA; pair w of the job belongs to B fragment w / 4 = (column block, half)
            if constexpr (converting) {
                __builtin_amdgcn_sched_barrier(0);  // the MFMA first, the conversions in its shadow
                constexpr int slot = (t - 1) * NM + m, prev = job - 1;
                static_for<PPM>([&](auto wc) {
                    constexpr int w = slot * PPM + decltype(wc)::value;
                    if constexpr (w < PAIRS) {
                        constexpr int piece = w / 4, pcb = piece / 2, u = piece % 2;
                        uint32_t(*dst)[4];
                        if constexpr (prev < 4) dst = hid1[pcb][2 * prev + u];
                        else dst = hid2[pcb][2 * (prev - 4) + u];
                        relu_pair<PREC>(acc[set ^ 1][pcb], 4 * u + w % 4, dst);
                    }
                });
                __builtin_amdgcn_sched_barrier(0);
            }
        });
        __builtin_amdgcn_sched_barrier(0);
    });
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
        for (int k = 0; k < 3; ++k) {
            const float e = PREC == LM_MLP_F16X2 ? expf(-acc[0][cb][k]) : __expf(-acc[0][cb][k]);
            out[cb][k] = __builtin_amdgcn_rcpf(1.0f + e);
        }
}

template <int PREC> struct LdsPlan {
    using M = Mma<PREC>;
    static constexpr size_t kW1 = (size_t)4 * kSlots1 * 64 * sizeof(typename M::elem) * M::NP;
    static constexpr size_t kW2 = (size_t)4 * 64 * 64 * sizeof(typename M::elem) * M::NP;
    static constexpr size_t kW3 = (size_t)64 * 64 * sizeof(typename M::elem) * M::NP;
    static constexpr bool kW3InLds = (kW1 + kW2 + kW3) <= 96 * 1024;
    static constexpr size_t kBias = (4 * 2 * 16 + 4 * 2 * 16 + 2 * 16) * sizeof(float);  // b1 | b2 | b3, register order
    static constexpr size_t kWeights = kW1 + kW2 + (kW3InLds ? kW3 : 0);
    static constexpr size_t kQueue = kWeights + kBias;  // the workgroup's tile counter
    // 16-bit modes: every wave owns a staging area that receives its next tile's feature rows (27 floats per row,
    // contiguous in memory) straight from global memory, rounded up to whole 1 KB transfers
    static constexpr bool kStaged = LM_MLP_STREAM && (PREC == LM_MLP_F16 || PREC == LM_MLP_BF16);
    static constexpr size_t kTileBytes = (size_t)32 * MlpBlock<PREC>::NCB * kAppDim * sizeof(float);
    static constexpr size_t kStageWave = (kTileBytes + 1023) / 1024 * 1024;
    static constexpr size_t kStage = kQueue + 16;
    static constexpr size_t kBytes = kStage + (kStaged ? kStageWave * (MlpBlock<PREC>::N / LM_WAVE) : 0);
    static_assert(kBytes <= 160 * 1024, "LDS of a compute unit");
};

template <int PREC>
__device__ __forceinline__ void stage_weights(char *lds, const char *packed, const PackLayout &L) {
    using P = LdsPlan<PREC>;
    const uint4 *s1 = reinterpret_cast<const uint4 *>(packed + L.w1);
    const uint4 *s2 = reinterpret_cast<const uint4 *>(packed + L.w2);
    const uint4 *s3 = reinterpret_cast<const uint4 *>(packed + L.w3);
    uint4 *d = reinterpret_cast<uint4 *>(lds);
    for (size_t i = threadIdx.x; i < P::kW1 / 16; i += blockDim.x) d[i] = s1[i];
    d += P::kW1 / 16;
    for (size_t i = threadIdx.x; i < P::kW2 / 16; i += blockDim.x) d[i] = s2[i];
    d += P::kW2 / 16;
    if (P::kW3InLds)
        for (size_t i = threadIdx.x; i < P::kW3 / 16; i += blockDim.x) d[i] = s3[i];
    // biases: read once per layer and row block by every wave, so they live next to the weights
    float *bl = reinterpret_cast<float *>(lds + P::kWeights);
    const float *b1 = (const float *)(packed + L.b1), *b2 = (const float *)(packed + L.b2), *b3 = (const float *)(packed + L.b3);
    for (unsigned i = threadIdx.x; i < 128; i += blockDim.x) { bl[i] = b1[i]; bl[128 + i] = b2[i]; }
    for (unsigned i = threadIdx.x; i < 32; i += blockDim.x) bl[256 + i] = b3[i];
    if (threadIdx.x == 0) *reinterpret_cast<uint32_t *>(lds + P::kQueue) = blockDim.x / LM_WAVE;  // one tile per wave is dealt at the start
    __syncthreads();
}

// Colour network over a list of rows.
//   MODE 0: feat [M,27] and view [M,3] given per row (isolated network)
//   MODE 1: feat [n,27] per appearance slot, view direction = direction of the slot's ray
template <int PREC, int MODE>
__global__ __launch_bounds__(MlpBlock<PREC>::N) void k_mlp(const char *__restrict__ packed, PackLayout L,
                                                   const float *__restrict__ feat, const float *__restrict__ view,
                                                   uint64_t M_host, const uint32_t *__restrict__ count, uint32_t cap, int S,
                                                   const uint32_t *__restrict__ app_idx, int small,
                                                   float *__restrict__ rgb) {
    extern __shared__ __align__(16) char lds[];
    using Mm = Mma<PREC>;
    using frag = typename Mm::frag;
    using P = LdsPlan<PREC>;
    stage_weights<PREC>(lds, packed, L);
    const frag *w1 = reinterpret_cast<const frag *>(lds);
    const frag *w2 = reinterpret_cast<const frag *>(lds + P::kW1);
    const frag *w3 = P::kW3InLds ? reinterpret_cast<const frag *>(lds + P::kW1 + P::kW2)
                                 : reinterpret_cast<const frag *>(packed + L.w3);
    const float *b1 = reinterpret_cast<const float *>(lds + P::kWeights), *b2 = b1 + 128, *b3 = b1 + 256;
    const unsigned lane = lm_lane(), j = lane & 31u, h = lane >> 5;
    const uint64_t M = MODE == 0 ? M_host : (uint64_t)min(*count, cap);  // the counter keeps counting past the list's capacity
    constexpr int NCB = MlpBlock<PREC>::NCB, TILE = 32 * NCB;
    const uint64_t n_tiles = (M + TILE - 1) / TILE;
    const unsigned wpb = MlpBlock<PREC>::N / LM_WAVE;
    const uint64_t n_waves = (uint64_t)gridDim.x * wpb;
    // The lane's 16 input rows (features, view direction, zeros) of its sample in each column block.  Half h
    // holds rows row_of(v, 0) + 4 h: features up to row 23, then rows 24..26 (features, h = 0) or 28..30 (the
    // view direction, h = 1); rows 27 and 31 are zero.  Two base addresses per lane and compile-time offsets
    // instead of an address per load; when the feature array is below 4 GB (`small`) the bases are 32-bit
    // byte offsets from the array's (scalar) address.
    static_assert(row_of(0, 1) == row_of(0, 0) + 4 && row_of(11, 1) == 23 && row_of(12, 0) == 24 && row_of(12, 1) == 28 &&
                      kAppDim == 27,
                  "input rows per lane half");
    auto fetch = [&](uint64_t tile, float (*raw)[16]) {
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            const uint64_t p = tile * TILE + cb * 32 + j;
            const uint64_t pc = p < M ? p : M - 1;
            const float *vsrc = MODE == 0 ? view + pc * 3 : view + 6 * (size_t)(app_idx[pc] / (uint32_t)S) + 3;
            if (small) {
                const char *base = reinterpret_cast<const char *>(feat);
                const uint32_t body = (uint32_t)pc * (uint32_t)(kAppDim * sizeof(float)) + 16u * h;
#pragma unroll
                for (int v = 0; v < 12; ++v) raw[cb][v] = *reinterpret_cast<const float *>(base + body + 4 * row_of(v, 0));
                if (h) {
#pragma unroll
                    for (int v = 12; v < 15; ++v) raw[cb][v] = vsrc[v - 12];
                } else {
#pragma unroll
                    for (int v = 12; v < 15; ++v) raw[cb][v] = *reinterpret_cast<const float *>(base + body + 4 * (12 + v));
                }
            } else {
                const float *f = feat + pc * kAppDim;
                const float *body = f + 4 * h;
                const float *tail = h ? vsrc : f + 24;
#pragma unroll
                for (int v = 0; v < 12; ++v) raw[cb][v] = body[row_of(v, 0)];
#pragma unroll
                for (int v = 12; v < 15; ++v) raw[cb][v] = tail[v - 12];
            }
            raw[cb][15] = 0.0f;
        }
    };
    constexpr int T1 = kSlots1 / Mm::G;
    float raw[NCB][16];
    // Tiles are dealt to workgroups in rounds of one tile per wave; inside a workgroup a wave takes the group's next
    // tile from a counter in LDS when it has encoded its current one.  The SIMD issues its oldest wave first, so its
    // two waves advance at different speeds, and with a fixed share per wave the slower one would finish alone.
    uint32_t *queue = reinterpret_cast<uint32_t *>(lds + P::kQueue);
    const uint64_t first = (uint64_t)lm_xcd_swizzle(blockIdx.x, gridDim.x) * wpb;
    auto tile_of = [&](uint32_t q) { return (uint64_t)(q / wpb) * n_waves + first + q % wpb; };
    auto claim = [&]() {
        uint32_t q = 0;
        if (lane == 0) q = atomicAdd(queue, 1u);
        return tile_of(__builtin_amdgcn_readfirstlane(q));
    };
    uint64_t tile = tile_of(threadIdx.x / LM_WAVE);
    if constexpr (P::kStaged) {
        // The feature rows of a tile are one contiguous run of global memory: the wave copies it into its staging
        // area with transfers that bypass the registers (16 bytes per lane, 1 KB per instruction; 4-byte transfers
        // when the array is not 16-byte aligned) while the previous tile is multiplied, and every lane picks its
        // 12 or 15 values from LDS when the tile's turn comes.  Only the view direction (three values of the
        // lanes of the upper half) travels through registers.
        char *stage = lds + P::kStage + (threadIdx.x / LM_WAVE) * P::kStageWave;
        const float *stage_f = reinterpret_cast<const float *>(stage);
        const bool wide = (reinterpret_cast<uintptr_t>(feat) & 15u) == 0;
        typedef const void __attribute__((address_space(1))) *gptr;
        typedef void __attribute__((address_space(3))) *lptr;
        float vdir[NCB][3];
        auto request = [&](uint64_t t) {
            // Lanes whose share lies beyond the tile or the array repeat the last valid transfer (into their own
            // part of the staging area, which nobody reads): no lane is switched off, no branch.
            const uint64_t begin = t * P::kTileBytes, left = M * (kAppDim * sizeof(float)) - begin;
            const unsigned span = (unsigned)(left < P::kTileBytes ? left : P::kTileBytes);
            const char *src = reinterpret_cast<const char *>(feat) + begin;
            if (wide) {
                const unsigned last = ((span + 15u) & ~15u) - 16u;
#pragma unroll
                for (unsigned k = 0; k < P::kStageWave / 1024; ++k) {
                    const unsigned off = (k * 64 + lane) * 16;
                    __builtin_amdgcn_global_load_lds((gptr)(src + (off < last ? off : last)), (lptr)(stage + k * 1024), 16, 0, 0);
                }
            } else {
                const unsigned last = span - 4u;
#pragma unroll 1
                for (unsigned k = 0; k < P::kTileBytes / 256; ++k) {
                    const unsigned off = (k * 64 + lane) * 4;
                    __builtin_amdgcn_global_load_lds((gptr)(src + (off < last ? off : last)), (lptr)(stage + k * 256), 4, 0, 0);
                }
            }
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                const uint64_t p = t * TILE + cb * 32 + j;
                const uint64_t pc = p < M ? p : M - 1;
                const float *vsrc = MODE == 0 ? view + pc * 3 : view + 6 * (size_t)(app_idx[pc] / (uint32_t)S) + 3;
#pragma unroll
                for (int k = 0; k < 3; ++k) vdir[cb][k] = vsrc[k];
            }
        };
        if (tile < n_tiles) request(tile);
        float out[NCB][3];
        uint64_t done = ~0ull;  // the tile whose colours wait in `out`
        auto store = [&]() {
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                const uint64_t p = done * TILE + cb * 32 + j;
                if (done != ~0ull && p < M && h == 0) {
                    rgb[p * 3 + 0] = out[cb][0]; rgb[p * 3 + 1] = out[cb][1]; rgb[p * 3 + 2] = out[cb][2];
                }
            }
        };
        while (tile < n_tiles) {
            const uint64_t next = claim();
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the transfers into the staging area have landed
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                const float *r = stage_f + (cb * 32 + j) * kAppDim;
#pragma unroll
                for (int v = 0; v < 12; ++v) raw[cb][v] = r[4 * h + row_of(v, 0)];
#pragma unroll
                for (int v = 12; v < 15; ++v) raw[cb][v] = h ? vdir[cb][v - 12] : r[12 + v];
                raw[cb][15] = 0.0f;
            }
            // the previous tile's colours leave now, so that the wait above never waits for them
            store();
            frag bfrag[NCB][T1][Mm::NP];
            encode_inputs<PREC, NCB>(raw, bfrag);
            // every lane holds its values in registers: the staging area may be overwritten
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            if (next < n_tiles) request(next);
            __builtin_amdgcn_sched_barrier(0);
#if LM_MLP_PRIO
            __builtin_amdgcn_s_setprio(LM_MLP_PRIO);
#endif
            colour_layers_stream<PREC, NCB, LM_MLP_PF>(w1, w2, w3, b1, b2, b3, bfrag, lane, out);
#if LM_MLP_PRIO
            __builtin_amdgcn_s_setprio(0);
#endif
            done = tile;
            tile = next;
        }
        store();
    } else {
        // A tile's inputs are encoded into the first layer's fragments first; the registers that held them then
        // receive the next tile's inputs, which travel while this tile is multiplied.
        if (tile < n_tiles) fetch(tile, raw);
        while (tile < n_tiles) {
            frag bfrag[NCB][T1][Mm::NP];
            encode_inputs<PREC, NCB>(raw, bfrag);
            const uint64_t next = claim();
            if (next < n_tiles) fetch(next, raw);
            float out[NCB][3];
            if constexpr (PREC == LM_MLP_F16X2 && LM_MLP_STREAM_X2) colour_layers_stream<PREC, NCB, LM_MLP_PF_X2>(w1, w2, w3, b1, b2, b3, bfrag, lane, out);
            else colour_layers<PREC, NCB>(w1, w2, w3, b1, b2, b3, bfrag, lane, out);
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb) {
                const uint64_t p = tile * TILE + cb * 32 + j;
                if (p < M && h == 0) {
                    rgb[p * 3 + 0] = out[cb][0]; rgb[p * 3 + 1] = out[cb][1]; rgb[p * 3 + 2] = out[cb][2];
                }
            }
            tile = next;
        }
    }
}

// products [M,K] -> feat [M,27] (stand-alone basis_mat; fragments straight from global memory)
template <int PREC>
__global__ __launch_bounds__(256) void k_basis(const char *__restrict__ packed, PackLayout L, int K,
                                               const float *__restrict__ products, uint64_t M_host,
                                               const uint32_t *__restrict__ count, uint32_t cap, float *__restrict__ feat) {
    const uint64_t M = count ? (uint64_t)min(*count, cap) : M_host;
    using Mm = Mma<PREC>;
    using frag = typename Mm::frag;
    constexpr int G = Mm::G, CW = Mm::CW, NP = Mm::NP;
    const unsigned lane = lm_lane(), j = lane & 31u, h = lane >> 5;
    const uint64_t n_tiles = (M + 31) / 32;
    const uint64_t wave_id = (uint64_t)blockIdx.x * 4 + threadIdx.x / LM_WAVE;
    const uint64_t n_waves = (uint64_t)gridDim.x * 4;
    const frag *A = reinterpret_cast<const frag *>(packed + L.basis);
    for (uint64_t tile = wave_id; tile < n_tiles; tile += n_waves) {
        const uint64_t p = tile * 32 + j;
        const bool live = p < M;
        const float *row = products + (live ? p : M - 1) * (uint64_t)K;
        floatx16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
        const int iters = (K / 2) / CW;
        for (int it = 0; it < iters; ++it) {
            float c[CW];
            const float4 *src = reinterpret_cast<const float4 *>(row + 2 * CW * it + CW * h);
#pragma unroll
            for (int i = 0; i < CW / 4; ++i) {
                float4 t = src[i];
                c[4 * i] = t.x; c[4 * i + 1] = t.y; c[4 * i + 2] = t.z; c[4 * i + 3] = t.w;
            }
#pragma unroll
            for (int u = 0; u < CW / G; ++u) {
                frag b[NP];
                Mm::pack(c + u * G, b);
                const int t = it * (CW / G) + u;
                const frag a0 = A[(t * NP) * 64 + lane];
                acc = Mm::mma(a0, b[0], acc);
                if constexpr (NP == 2) {
                    const frag a1 = A[(t * NP + 1) * 64 + lane];
                    acc = Mm::mma(a1, b[0], acc);
                    acc = Mm::mma(a0, b[1], acc);
                }
            }
        }
        if (live) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = row_of(v, (int)h);
                if (r < kAppDim) feat[p * kAppDim + r] = acc[v];
            }
        }
    }
}

template <int PREC, int MODE>
int launch_mlp(const void *packed, int K, const float *feat, const float *view, uint64_t M, const uint32_t *count,
               uint32_t cap, int S, const uint32_t *app_idx, float *rgb, unsigned grid, hipStream_t stream) {
    const PackLayout L = pack_layout(PREC, K);
    const size_t lds = LdsPlan<PREC>::kBytes;
    // rows the launch can touch: the feature array stays below 4 GB when they number fewer than 2^32 / 108
    const uint64_t rows = MODE == 0 ? M : (uint64_t)cap;
    const int small = rows * (kAppDim * sizeof(float)) < (1ull << 32) ? 1 : 0;
    static thread_local bool configured_on[LM_MAX_DEVICES] = {};  // the attribute belongs to a device's copy of the kernel
    bool &configured = configured_on[lm_current_device()];
    if (!configured) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&k_mlp<PREC, MODE>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) LM_FAIL(LM_ERR_LAUNCH, "k_mlp: cannot reserve %zu bytes of LDS: %s", lds, hipGetErrorString(e));
        configured = true;
    }
    hipLaunchKernelGGL((k_mlp<PREC, MODE>), dim3(grid), dim3(MlpBlock<PREC>::N), lds, stream, (const char *)packed, L, feat, view,
                       M, count, cap, S, app_idx, small, rgb);
    LM_CHECK_LAUNCH("k_mlp");
    return LM_OK;
}

template <int MODE>
int dispatch_mlp(int prec, const void *packed, int K, const float *feat, const float *view, uint64_t M,
                 const uint32_t *count, uint32_t cap, int S, const uint32_t *app_idx, float *rgb, unsigned grid, hipStream_t st) {
    switch (prec) {
        case LM_MLP_F32: return launch_mlp<LM_MLP_F32, MODE>(packed, K, feat, view, M, count, cap, S, app_idx, rgb, grid, st);
        case LM_MLP_F16: return launch_mlp<LM_MLP_F16, MODE>(packed, K, feat, view, M, count, cap, S, app_idx, rgb, grid, st);
        case LM_MLP_BF16: return launch_mlp<LM_MLP_BF16, MODE>(packed, K, feat, view, M, count, cap, S, app_idx, rgb, grid, st);
        default: return launch_mlp<LM_MLP_F16X2, MODE>(packed, K, feat, view, M, count, cap, S, app_idx, rgb, grid, st);
    }
}

}  // namespace

int lm_check_prec(int prec) {
    LM_REQUIRE(prec == LM_MLP_F32 || prec == LM_MLP_F16 || prec == LM_MLP_BF16 || prec == LM_MLP_F16X2,
               "unknown colour-network precision %d", prec);
    return LM_OK;
}
int lm_check_K(int K) {
    LM_REQUIRE(K >= 16 && K % 16 == 0 && K <= 4096, "basis_mat input width %d must be a multiple of 16 in 16..4096", K);
    return LM_OK;
}

extern "C" size_t lm_mlp_packed_bytes(int32_t prec, int32_t K_basis) {
    if (lm_check_prec(prec) || lm_check_K(K_basis)) return 0;
    return pack_layout(prec, K_basis).total;
}

extern "C" int lm_mlp_pack(int32_t prec, int32_t K, const float *basis, const float *w1, const float *b1,
                           const float *w2, const float *b2, const float *w3, const float *b3, void *packed_out) {
    if (int rc = lm_check_prec(prec)) return rc;
    if (int rc = lm_check_K(K)) return rc;
    LM_REQUIRE(basis && w1 && w2 && w3 && packed_out, "null weight pointer");
    const PackLayout L = pack_layout(prec, K);
    memset(packed_out, 0, L.total);
    char *out = (char *)packed_out;
    if (prec == LM_MLP_F32) pack_all<float>(K, 1, 4, 1, L, basis, w1, b1, w2, b2, w3, b3, out);
    else if (prec == LM_MLP_F16) pack_all<_Float16>(K, 8, 8, 1, L, basis, w1, b1, w2, b2, w3, b3, out);
    else if (prec == LM_MLP_BF16) pack_all<__bf16>(K, 8, 8, 1, L, basis, w1, b1, w2, b2, w3, b3, out);
    else pack_all<_Float16>(K, 8, 8, 2, L, basis, w1, b1, w2, b2, w3, b3, out);
    return LM_OK;
}

extern "C" size_t lm_mlp_bias1_offset(int32_t prec, int32_t K_basis) {
    if (lm_check_prec(prec) || lm_check_K(K_basis)) return 0;
    return pack_layout(prec, K_basis).b1;
}

extern "C" int lm_mlp_pack_bias1(const float *b1, float *packed_b1_out) {
    LM_REQUIRE(b1 && packed_b1_out, "null pointer");
    for (int fb = 0; fb < 4; ++fb)
        for (int h = 0; h < 2; ++h)
            for (int v = 0; v < 16; ++v) packed_b1_out[(fb * 2 + h) * 16 + v] = b1[32 * fb + row_of(v, h)];
    return LM_OK;
}

static unsigned mlp_grid(uint64_t M) {
    const uint64_t tiles = (M + 63) / 64, wpb = 4, blocks = (tiles + wpb - 1) / wpb;
    return (unsigned)std::min<uint64_t>(std::max<uint64_t>(blocks, 1), (uint64_t)lm_persistent_blocks(1));
}

extern "C" int lm_mlp(int32_t prec, const void *packed, int32_t K, const float *feat, const float *view, int64_t M,
                      float *rgb, void *stream) {
    if (int rc = lm_check_prec(prec)) return rc;
    if (int rc = lm_check_K(K)) return rc;
    LM_REQUIRE(M >= 0, "negative count");
    if (M == 0) return LM_OK;
    LM_REQUIRE(packed && feat && view && rgb && lm_aligned16(packed), "null or misaligned buffer");
    return dispatch_mlp<0>(prec, packed, K, feat, view, (uint64_t)M, nullptr, 0u, 1, nullptr, rgb, mlp_grid((uint64_t)M),
                           (hipStream_t)stream);
}

// products [M,K] -> feat [M,27]; M from the host, or from *count when count != NULL
int lm_launch_basis(int prec, const void *packed, int K, const float *products, uint64_t M, const uint32_t *count,
                    uint32_t cap, float *feat, hipStream_t st) {
    if (int rc = lm_check_prec(prec)) return rc;
    if (int rc = lm_check_K(K)) return rc;
    LM_REQUIRE(packed && products && feat && lm_aligned16(packed) && lm_aligned16(products), "null or misaligned buffer");
    const PackLayout L = pack_layout(prec, K);
    const uint64_t tiles = (M + 31) / 32;
    const unsigned grid = count ? (unsigned)lm_persistent_blocks(4)
                                : (unsigned)std::min<uint64_t>(std::max<uint64_t>((tiles + 3) / 4, 1), (uint64_t)lm_persistent_blocks(4));
    switch (prec) {
        case LM_MLP_F32: hipLaunchKernelGGL(k_basis<LM_MLP_F32>, dim3(grid), dim3(256), 0, st, (const char *)packed, L, K, products, M, count, cap, feat); break;
        case LM_MLP_F16: hipLaunchKernelGGL(k_basis<LM_MLP_F16>, dim3(grid), dim3(256), 0, st, (const char *)packed, L, K, products, M, count, cap, feat); break;
        case LM_MLP_BF16: hipLaunchKernelGGL(k_basis<LM_MLP_BF16>, dim3(grid), dim3(256), 0, st, (const char *)packed, L, K, products, M, count, cap, feat); break;
        default: hipLaunchKernelGGL(k_basis<LM_MLP_F16X2>, dim3(grid), dim3(256), 0, st, (const char *)packed, L, K, products, M, count, cap, feat); break;
    }
    LM_CHECK_LAUNCH("k_basis");
    return LM_OK;
}

extern "C" int lm_basis(int32_t prec, const void *packed, int32_t K, const float *products, int64_t M, float *feat,
                        void *stream) {
    LM_REQUIRE(M >= 0, "negative count");
    if (M == 0) return LM_OK;
    return lm_launch_basis(prec, packed, K, products, (uint64_t)M, nullptr, 0u, feat, (hipStream_t)stream);
}

// used by lm_render: feat [n_app,27] + ray directions -> rgb [n_app,3]
int lm_launch_app_colour(int prec, const void *packed, int K, int S, const float *feat, const float *rays,
                         const uint32_t *app_idx, const uint32_t *count, uint32_t cap, float *rgb, hipStream_t stream) {
    if (int rc = lm_check_prec(prec)) return rc;
    if (int rc = lm_check_K(K)) return rc;
    LM_REQUIRE(packed && lm_aligned16(packed), "packed colour-network weights are null or misaligned");
    return dispatch_mlp<1>(prec, packed, K, feat, rays, 0, count, cap, S, app_idx, rgb, (unsigned)lm_persistent_blocks(1), stream);
}
