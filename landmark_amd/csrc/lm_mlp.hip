// Part 3: appearance projection (basis_mat) + positional encoding + colour network on the
// matrix cores.
//
// One wave owns 32 samples.  All products are computed "transposed": the weight matrix
// is the A operand (32 output rows per MFMA), the 32 samples are the columns, so the
// 32x32 accumulator of one layer already has the register layout the next layer needs as
// its B operand (lane = sample, registers = features).  Activations therefore never leave
// the register file between basis_mat, the encoding and the three layers.  The order of
// the K dimension is free in a dot product, so the host packs every weight matrix into
// the exact per-lane fragment order the kernel consumes (lm_mlp_pack); a wave reads one
// contiguous fragment per MFMA.
//
// Register layout of a 32x32 fp32 accumulator (all 32x32 MFMA shapes): lane l holds column
// j = l%32; with h = l/32 its register v (0..15) is row 8*(v/4) + 4*h + v%4.
//
// Row assignment after basis_mat: rows 0..26 are the 27 appearance features, rows 28..30
// are overwritten with the view direction, rows 27 and 31 are zero.  Each lane thus owns
// 16 raw values (15 real); the network input is built per lane as five groups of 16:
// raw, sin(raw), cos(raw), sin(2 raw), cos(2 raw) = 80 slots, 160 per sample (150 real,
// the rest meet zero weights).  Reference input order it is mapped to:
// app/models/mlp_render_fea.py:55-65 with app/tools/utils.py:42-48.
#include <hip/hip_fp16.h>

#include <cmath>
#include <cstring>
#include <vector>

#include "lm_common.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

namespace {

constexpr int kAppDim = 27;
constexpr int kHidden = 128;
constexpr int kInDim = 150;
constexpr int kSlots1 = 80;  // per lane-half
constexpr int kBlock = 256;

__host__ __device__ constexpr int row_of(int v, int h) { return 8 * (v / 4) + 4 * h + (v % 4); }

template <int PREC> struct Mma;
template <> struct Mma<LM_MLP_F32> {
    static constexpr int G = 1;   // K slots one lane feeds per MFMA
    static constexpr int CW = 4;  // consecutive product channels a lane reads at once
    using elem = float;
    using frag = float;
    __device__ static __forceinline__ floatx16 mma(frag a, frag b, floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ frag pack(const float *s) { return s[0]; }
};
template <> struct Mma<LM_MLP_F16> {
    static constexpr int G = 8;
    static constexpr int CW = 8;
    using elem = _Float16;
    using frag = half8;
    __device__ static __forceinline__ floatx16 mma(frag a, frag b, floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ frag pack(const float *s) {
        frag f;
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (_Float16)s[i];
        return f;
    }
};
template <> struct Mma<LM_MLP_BF16> {
    static constexpr int G = 8;
    static constexpr int CW = 8;
    using elem = __bf16;
    using frag = bf16x8;
    __device__ static __forceinline__ floatx16 mma(frag a, frag b, floatx16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    __device__ static __forceinline__ frag pack(const float *s) {
        frag f;
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (__bf16)s[i];
        return f;
    }
};

// ---- layout of the packed weight buffer (all offsets in bytes, 256-byte aligned) -----------
struct PackLayout {
    size_t basis, w1, b1, w2, b2, w3, b3, total;
};
inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }
inline PackLayout pack_layout(int prec, int K) {
    const size_t E = prec == LM_MLP_F32 ? 4 : 2;
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

// product channel a lane-half reads for basis slot sigma: W consecutive channels per lane,
// the two halves interleaved so that a sample's pair of lanes reads 2W contiguous floats
__host__ __device__ constexpr int basis_channel(int h, int sigma, int W) { return 2 * W * (sigma / W) + W * h + sigma % W; }

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

// Writes fragments [block][step][lane][G]; value(block, i, h, sigma) gives A[row i of the block][slot]
template <typename E, typename F>
void pack_matrix(E *dst, int n_blocks, int n_slots, int G, F value) {
    const int steps = n_slots / G;
    for (int fb = 0; fb < n_blocks; ++fb)
        for (int t = 0; t < steps; ++t)
            for (int lane = 0; lane < 64; ++lane)
                for (int e = 0; e < G; ++e) {
                    const int i = lane % 32, h = lane / 32;
                    dst[(((size_t)fb * steps + t) * 64 + lane) * G + e] = to_elem<E>(value(fb, i, h, t * G + e));
                }
}

template <typename E>
void pack_all(int K, int G, int CW, const PackLayout &L, const float *basis, const float *w1, const float *b1,
              const float *w2, const float *b2, const float *w3, const float *b3, char *out) {
    pack_matrix<E>((E *)(out + L.basis), 1, K / 2, G, [&](int, int i, int h, int s) {
        return i < kAppDim ? basis[(size_t)i * K + basis_channel(h, s, CW)] : 0.0f;
    });
    pack_matrix<E>((E *)(out + L.w1), 4, kSlots1, G, [&](int fb, int i, int h, int s) {
        const int col = input_column(h, s / 16, s % 16);
        return col < 0 ? 0.0f : w1[(size_t)(32 * fb + i) * kInDim + col];
    });
    pack_matrix<E>((E *)(out + L.w2), 4, 64, G, [&](int fb, int i, int h, int s) {
        return w2[(size_t)(32 * fb + i) * kHidden + 32 * (s / 16) + row_of(s % 16, h)];
    });
    pack_matrix<E>((E *)(out + L.w3), 1, 64, G, [&](int, int i, int h, int s) {
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
// Keeps the compiler from hoisting the weight-fragment loads of later blocks above this
// point (fully unrolled loops would otherwise keep hundreds of fragments live and spill).
#define LM_LOAD_FENCE() asm volatile("" ::: "memory")
// fragments loaded ahead of their MFMAs: one group between two fences
template <int G> struct Group { static constexpr int N = G == 1 ? 16 : 10; };
struct PackPtrs {
    const char *basis, *w1, *w2, *w3;
    const float *b1, *b2, *b3;
};

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

// raw[16] (lane's 16 row values, view direction already inserted) -> rgb of the lane's
// sample in out[0..2] (meaningful on lanes with h == 0)
template <int PREC>
__device__ __forceinline__ void colour_network(const PackPtrs &P, const float *raw, unsigned lane, float *out) {
    using M = Mma<PREC>;
    using frag = typename M::frag;
    constexpr int G = M::G;
    const unsigned h = lane >> 5;
    float slots[kSlots1];
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const float x = raw[v];
        float s1, c1, s2, c2;
        if (PREC == LM_MLP_F32) {
            s1 = sinf(x); c1 = cosf(x);
            const float x2 = x * 2.0f;
            s2 = sinf(x2); c2 = cosf(x2);
        } else {
            s1 = __sinf(x); c1 = __cosf(x);
            s2 = 2.0f * s1 * c1; c2 = 1.0f - 2.0f * s1 * s1;
        }
        slots[v] = x; slots[16 + v] = s1; slots[32 + v] = c1; slots[48 + v] = s2; slots[64 + v] = c2;
    }
    frag bfrag[kSlots1 / G];
#pragma unroll
    for (int t = 0; t < kSlots1 / G; ++t) bfrag[t] = M::pack(slots + t * G);

    // layer 1
    float h1[64];
    {
        const frag *A = reinterpret_cast<const frag *>(P.w1);
        constexpr int T = kSlots1 / G;
#pragma unroll
        for (int fb = 0; fb < 4; ++fb) {
            floatx16 acc = load_bias(P.b1, fb * 2 + h);
#pragma unroll
            for (int t = 0; t < T; ++t) {
                if (t % Group<G>::N == 0) LM_LOAD_FENCE();
                acc = M::mma(A[(fb * T + t) * 64 + lane], bfrag[t], acc);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) h1[fb * 16 + v] = fmaxf(acc[v], 0.0f);
        }
    }
    // layer 2
    constexpr int T2 = 64 / G;
    frag b2frag[T2];
#pragma unroll
    for (int t = 0; t < T2; ++t) b2frag[t] = M::pack(h1 + t * G);
    float h2[64];
    {
        const frag *A = reinterpret_cast<const frag *>(P.w2);
#pragma unroll
        for (int fb = 0; fb < 4; ++fb) {
            floatx16 acc = load_bias(P.b2, fb * 2 + h);
#pragma unroll
            for (int t = 0; t < T2; ++t) {
                if (t % Group<G>::N == 0) LM_LOAD_FENCE();
                acc = M::mma(A[(fb * T2 + t) * 64 + lane], b2frag[t], acc);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) h2[fb * 16 + v] = fmaxf(acc[v], 0.0f);
        }
    }
    // layer 3 (rows 0..2 real)
    {
        const frag *A = reinterpret_cast<const frag *>(P.w3);
        floatx16 acc = load_bias(P.b3, h);
#pragma unroll
        for (int t = 0; t < T2; ++t) {
            if (t % Group<G>::N == 0) LM_LOAD_FENCE();
            acc = M::mma(A[t * 64 + lane], M::pack(h2 + t * G), acc);
        }
#pragma unroll
        for (int k = 0; k < 3; ++k) out[k] = 1.0f / (1.0f + expf(-acc[k]));
    }
}

// basis_mat on 32 samples: products row of the lane's sample -> 16 row values per lane
template <int PREC>
__device__ __forceinline__ floatx16 basis_project(const PackPtrs &P, int K, const float *__restrict__ row, unsigned lane) {
    using M = Mma<PREC>;
    using frag = typename M::frag;
    constexpr int G = M::G, CW = M::CW;
    const unsigned h = lane >> 5;
    const frag *A = reinterpret_cast<const frag *>(P.basis);
    floatx16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
    // per iteration a lane consumes CW consecutive channels = CW/G MFMA steps
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
        for (int u = 0; u < CW / G; ++u) acc = M::mma(A[(it * (CW / G) + u) * 64 + lane], M::pack(c + u * G), acc);
    }
    return acc;
}

__device__ __forceinline__ PackPtrs make_ptrs(const char *packed, PackLayout L) {
    PackPtrs P;
    P.basis = packed + L.basis; P.w1 = packed + L.w1; P.w2 = packed + L.w2; P.w3 = packed + L.w3;
    P.b1 = (const float *)(packed + L.b1); P.b2 = (const float *)(packed + L.b2); P.b3 = (const float *)(packed + L.b3);
    return P;
}

// feat [M,27], view [M,3] -> rgb [M,3]
template <int PREC>
__global__ __launch_bounds__(kBlock) void k_mlp_feat(const char *__restrict__ packed, PackLayout L,
                                                     const float *__restrict__ feat, const float *__restrict__ view,
                                                     uint64_t M, float *__restrict__ rgb) {
    const PackPtrs P = make_ptrs(packed, L);
    const unsigned lane = lm_lane(), j = lane & 31u, h = lane >> 5;
    const uint64_t n_tiles = (M + 31) / 32;
    const uint64_t wave_id = (uint64_t)lm_xcd_swizzle(blockIdx.x, gridDim.x) * (kBlock / LM_WAVE) + threadIdx.x / LM_WAVE;
    const uint64_t n_waves = (uint64_t)gridDim.x * (kBlock / LM_WAVE);
    for (uint64_t tile = wave_id; tile < n_tiles; tile += n_waves) {
        const uint64_t p = tile * 32 + j;
        const bool live = p < M;
        const uint64_t pc = live ? p : M - 1;
        float raw[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = row_of(v, (int)h);
            float x = 0.0f;
            if (row < kAppDim) x = feat[pc * kAppDim + row];
            else if (row >= 28 && row <= 30) x = view[pc * 3 + (row - 28)];
            raw[v] = x;
        }
        float out[3];
        colour_network<PREC>(P, raw, lane, out);
        if (live && h == 0) {
            rgb[p * 3 + 0] = out[0]; rgb[p * 3 + 1] = out[1]; rgb[p * 3 + 2] = out[2];
        }
    }
}

// products [M,K] -> feat [M,27]
template <int PREC>
__global__ __launch_bounds__(kBlock) void k_basis(const char *__restrict__ packed, PackLayout L, int K,
                                                  const float *__restrict__ products, uint64_t M,
                                                  float *__restrict__ feat) {
    const PackPtrs P = make_ptrs(packed, L);
    const unsigned lane = lm_lane(), j = lane & 31u, h = lane >> 5;
    const uint64_t n_tiles = (M + 31) / 32;
    const uint64_t wave_id = (uint64_t)blockIdx.x * (kBlock / LM_WAVE) + threadIdx.x / LM_WAVE;
    const uint64_t n_waves = (uint64_t)gridDim.x * (kBlock / LM_WAVE);
    for (uint64_t tile = wave_id; tile < n_tiles; tile += n_waves) {
        const uint64_t p = tile * 32 + j;
        const bool live = p < M;
        const uint64_t pc = live ? p : M - 1;
        const floatx16 acc = basis_project<PREC>(P, K, products + pc * (uint64_t)K, lane);
        if (live) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = row_of(v, (int)h);
                if (row < kAppDim) feat[p * kAppDim + row] = acc[v];
            }
        }
    }
}

// inside the render: products [n_app,K] + ray directions -> rgb [n_app,3]
template <int PREC>
__global__ __launch_bounds__(kBlock) void k_app_colour(const char *__restrict__ packed, PackLayout L, int K, int S,
                                                       const float *__restrict__ products,
                                                       const float *__restrict__ rays,
                                                       const uint32_t *__restrict__ app_idx,
                                                       const uint32_t *__restrict__ count, float *__restrict__ rgb) {
    const PackPtrs P = make_ptrs(packed, L);
    const unsigned lane = lm_lane(), j = lane & 31u, h = lane >> 5;
    const uint64_t M = *count;
    const uint64_t n_tiles = (M + 31) / 32;
    const uint64_t wave_id = (uint64_t)lm_xcd_swizzle(blockIdx.x, gridDim.x) * (kBlock / LM_WAVE) + threadIdx.x / LM_WAVE;
    const uint64_t n_waves = (uint64_t)gridDim.x * (kBlock / LM_WAVE);
    for (uint64_t tile = wave_id; tile < n_tiles; tile += n_waves) {
        const uint64_t p = tile * 32 + j;
        const bool live = p < M;
        const uint64_t pc = live ? p : M - 1;
        const floatx16 acc = basis_project<PREC>(P, K, products + pc * (uint64_t)K, lane);
        float raw[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) raw[v] = acc[v];
        if (h == 1) {
            const uint32_t r = app_idx[pc] / (uint32_t)S;
            raw[12] = rays[6 * (size_t)r + 3]; raw[13] = rays[6 * (size_t)r + 4]; raw[14] = rays[6 * (size_t)r + 5];
        }
        raw[15] = 0.0f;
        float out[3];
        colour_network<PREC>(P, raw, lane, out);
        if (live && h == 0) {
            rgb[p * 3 + 0] = out[0]; rgb[p * 3 + 1] = out[1]; rgb[p * 3 + 2] = out[2];
        }
    }
}

}  // namespace

static int check_prec(int prec) {
    LM_REQUIRE(prec == LM_MLP_F32 || prec == LM_MLP_F16 || prec == LM_MLP_BF16, "unknown colour-network precision %d", prec);
    return LM_OK;
}
static int check_K(int K) {
    LM_REQUIRE(K >= 16 && K % 16 == 0 && K <= 4096, "basis_mat input width %d must be a multiple of 16 in 16..4096", K);
    return LM_OK;
}

extern "C" size_t lm_mlp_packed_bytes(int32_t prec, int32_t K_basis) {
    if (check_prec(prec) || check_K(K_basis)) return 0;
    return pack_layout(prec, K_basis).total;
}

extern "C" int lm_mlp_pack(int32_t prec, int32_t K, const float *basis, const float *w1, const float *b1,
                           const float *w2, const float *b2, const float *w3, const float *b3, void *packed_out) {
    if (int rc = check_prec(prec)) return rc;
    if (int rc = check_K(K)) return rc;
    LM_REQUIRE(basis && w1 && w2 && w3 && packed_out, "null weight pointer");
    const PackLayout L = pack_layout(prec, K);
    memset(packed_out, 0, L.total);
    char *out = (char *)packed_out;
    if (prec == LM_MLP_F32) pack_all<float>(K, 1, 4, L, basis, w1, b1, w2, b2, w3, b3, out);
    else if (prec == LM_MLP_F16) pack_all<_Float16>(K, 8, 8, L, basis, w1, b1, w2, b2, w3, b3, out);
    else pack_all<__bf16>(K, 8, 8, L, basis, w1, b1, w2, b2, w3, b3, out);
    return LM_OK;
}

#define LM_DISPATCH_PREC(prec, KERNEL, grid, stream, ...)                                                         \
    do {                                                                                                          \
        if ((prec) == LM_MLP_F32)                                                                                 \
            hipLaunchKernelGGL(KERNEL<LM_MLP_F32>, dim3(grid), dim3(kBlock), 0, (hipStream_t)(stream), __VA_ARGS__); \
        else if ((prec) == LM_MLP_F16)                                                                            \
            hipLaunchKernelGGL(KERNEL<LM_MLP_F16>, dim3(grid), dim3(kBlock), 0, (hipStream_t)(stream), __VA_ARGS__); \
        else                                                                                                      \
            hipLaunchKernelGGL(KERNEL<LM_MLP_BF16>, dim3(grid), dim3(kBlock), 0, (hipStream_t)(stream), __VA_ARGS__); \
    } while (0)

static unsigned wave_tile_grid(uint64_t M) {
    const uint64_t tiles = (M + 31) / 32, blocks = (tiles + 3) / 4;
    return (unsigned)std::min<uint64_t>(std::max<uint64_t>(blocks, 1), (uint64_t)lm_persistent_blocks(2));
}

extern "C" int lm_mlp(int32_t prec, const void *packed, int32_t K, const float *feat, const float *view, int64_t M,
                      float *rgb, void *stream) {
    if (int rc = check_prec(prec)) return rc;
    if (int rc = check_K(K)) return rc;
    LM_REQUIRE(M >= 0, "negative count");
    if (M == 0) return LM_OK;
    LM_REQUIRE(packed && feat && view && rgb && lm_aligned16(packed), "null or misaligned buffer");
    const PackLayout L = pack_layout(prec, K);
    LM_DISPATCH_PREC(prec, k_mlp_feat, wave_tile_grid((uint64_t)M), stream, (const char *)packed, L, feat, view, (uint64_t)M, rgb);
    LM_CHECK_LAUNCH("k_mlp_feat");
    return LM_OK;
}

extern "C" int lm_basis(int32_t prec, const void *packed, int32_t K, const float *products, int64_t M, float *feat,
                        void *stream) {
    if (int rc = check_prec(prec)) return rc;
    if (int rc = check_K(K)) return rc;
    LM_REQUIRE(M >= 0, "negative count");
    if (M == 0) return LM_OK;
    LM_REQUIRE(packed && products && feat && lm_aligned16(packed) && lm_aligned16(products), "null or misaligned buffer");
    const PackLayout L = pack_layout(prec, K);
    LM_DISPATCH_PREC(prec, k_basis, wave_tile_grid((uint64_t)M), stream, (const char *)packed, L, (int)K, products, (uint64_t)M, feat);
    LM_CHECK_LAUNCH("k_basis");
    return LM_OK;
}

// used by lm_render
int lm_launch_app_colour(int prec, const void *packed, int K, int S, const float *products, const float *rays,
                         const uint32_t *app_idx, const uint32_t *count, float *rgb, hipStream_t stream) {
    if (int rc = check_prec(prec)) return rc;
    if (int rc = check_K(K)) return rc;
    LM_REQUIRE(packed && lm_aligned16(packed), "packed colour-network weights are null or misaligned");
    const PackLayout L = pack_layout(prec, K);
    const unsigned grid = (unsigned)lm_persistent_blocks(2);
    LM_DISPATCH_PREC(prec, k_app_colour, grid, stream, (const char *)packed, L, K, S, products, rays, app_idx, count, rgb);
    LM_CHECK_LAUNCH("k_app_colour");
    return LM_OK;
}
