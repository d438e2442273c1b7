// Micro-benchmark behind the colour network's instruction schedule: do ordinary vector instructions issue while an
// MFMA occupies the matrix pipe of a SIMD on gfx950, from the same wave and from the SIMD's other wave, and how many
// fit under one 32x32x16 MFMA?  Every variant runs `iters` trips of a loop body on every wave of a grid of one
// workgroup per compute unit.
//   M    NM independent 32x32x16 f16 MFMAs per trip (NA accumulator chains in turn)
//   V    NM * NV independent fp32 fmas (16 chains), or NV x (v_cvt_pk_f16_f32 + v_pk_max_f16): the hidden layers' relu
//   MV   NM x (1 MFMA, NV vector operations) interleaved in one wave, the order pinned with sched_group_barrier
//   M|V  two waves per SIMD, the older one runs M, the younger one V
// Prints one line per variant: milliseconds per launch, ns per trip, ns per MFMA slot, and the shader-clock cycles per
// MFMA slot that the workgroup's first wave (the oldest of its SIMD) counted: the figure that does not move with the clock.
// Build: hipcc --offload-arch=gfx950 -O3 mfma_valu_coissue.hip -o mfma_valu_coissue   (landmark_amd/build.py does it)
// Run:   mfma_valu_coissue [iters]
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

#define MFMA_MASK 0x008
#define VALU_MASK 0x002

template <int NV, int KIND>  // KIND 0: fma, 1: cvt_pk + pk_max (the hidden layers' conversion), 2: 16x16x32 MFMA with fma
__device__ __forceinline__ void valu_ops(float (&v)[16], unsigned (&pk)[8], int m) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int q = (m * NV + j) & 15;
        if (KIND == 1) {
            // one conversion of a pair and one packed max, as the hidden layers' relu does: 2 instructions per j;
            // the packed result becomes the next input of this slot so that nothing is loop invariant
            typedef _Float16 h2 __attribute__((ext_vector_type(2)));
            h2 h; h[0] = (_Float16)v[q]; h[1] = (_Float16)v[(q + 8) & 15];
            const h2 z = {0, 0};
            h = __builtin_elementwise_max(h, z);
            v[q] = __builtin_bit_cast(float, h);
        } else {
            v[q] = fmaf(v[q], 1.0001f, 0.5f);
        }
    }
}

template <int NM, int NV, int MODE, int KIND>  // MODE 0: M only, 1: V only, 2: interleaved
__global__ __launch_bounds__(512) void k(int iters, int split, float *out) {
    floatx16 acc[4];
    for (int k = 0; k < 4; ++k) for (int i = 0; i < 16; ++i) acc[k][i] = 0.f;
    half8 a[4], b;
    for (int k = 0; k < 4; ++k)
        for (int i = 0; i < 8; ++i) { a[k][i] = (_Float16)(threadIdx.x * 0.001f + k * 0.37f + i * 0.01f); b[i] = (_Float16)(0.5f + 0.1f * i); }
    float v[16];
    unsigned pk[8];
    for (int i = 0; i < 16; ++i) v[i] = threadIdx.x * 0.01f + i;
    for (int i = 0; i < 8; ++i) pk[i] = threadIdx.x + i;
    const bool second = threadIdx.x >= blockDim.x / 2;  // waves w and w + n/2 share a SIMD (n = 8: w, w + 4)
    const int mode = split ? (second ? 1 : 0) : MODE;
    const unsigned long long c0 = __builtin_readcyclecounter();
    if (mode == 0) {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int m = 0; m < NM; ++m) acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[m & 3], b, acc[m & 3], 0, 0, 0);
        }
    } else if (mode == 1) {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int m = 0; m < NM; ++m) valu_ops<NV, KIND>(v, pk, m);
        }
    } else {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[m & 3], b, acc[m & 3], 0, 0, 0);
                valu_ops<NV, KIND>(v, pk, m);
            }
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                __builtin_amdgcn_sched_group_barrier(MFMA_MASK, 1, 0);
                if (NV) __builtin_amdgcn_sched_group_barrier(VALU_MASK, KIND == 1 ? 2 * NV : NV, 0);
            }
        }
    }
    const unsigned long long c1 = __builtin_readcyclecounter();
    if (blockIdx.x == 0 && threadIdx.x == 0) reinterpret_cast<unsigned long long *>(out)[1] = c1 - c0;
    float s = 0;
    for (int k = 0; k < 4; ++k) for (int i = 0; i < 16; ++i) s += acc[k][i];
    for (int i = 0; i < 16; ++i) s += v[i];
    for (int i = 0; i < 8; ++i) s += pk[i];
    if (s == 12345.678f) out[0] = s;
}

static float *g_out;
template <typename F> float timeit(F launch, int iters) {
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    launch(iters / 20); hipDeviceSynchronize();
    hipEventRecord(e0); launch(iters); hipEventRecord(e1); hipEventSynchronize(e1);
    float ms; hipEventElapsedTime(&ms, e0, e1);
    hipEventDestroy(e0); hipEventDestroy(e1);
    return ms;
}

template <int NM, int NV, int MODE, int KIND> void run(const char *what, int threads, int split, int iters, int blocks_per_cu) {
    const float ms = timeit([&](int it) {
        hipLaunchKernelGGL((k<NM, NV, MODE, KIND>), dim3(256 * blocks_per_cu), dim3(threads), 0, 0, it, split, g_out);
    }, iters);
    unsigned long long cyc = 0;
    hipMemcpy(&cyc, reinterpret_cast<char *>(g_out) + 8, 8, hipMemcpyDeviceToHost);
    printf("%-44s waves/SIMD %d  NM %2d NV %2d  %8.3f ms  %8.2f ns/trip  %7.2f ns/MFMA-slot  %6.2f shader cycles per MFMA slot of the oldest wave\n", what,
           threads / 256 * blocks_per_cu, NM, NV, ms, ms * 1e6 / iters, ms * 1e6 / iters / NM, (double)cyc / iters / NM);
    fflush(stdout);
}

template <int NA>
__global__ __launch_bounds__(512) void k_chains(int iters, float *out) {
    floatx16 acc[NA];
    for (int k = 0; k < NA; ++k) for (int i = 0; i < 16; ++i) acc[k][i] = 0.f;
    half8 a[4], b;
    for (int k = 0; k < 4; ++k)
        for (int i = 0; i < 8; ++i) { a[k][i] = (_Float16)(threadIdx.x * 0.001f + k * 0.37f + i * 0.01f); b[i] = (_Float16)(0.5f + 0.1f * i); }
    const unsigned long long c0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int m = 0; m < 16; ++m) acc[m % NA] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[m & 3], b, acc[m % NA], 0, 0, 0);
    }
    const unsigned long long c1 = __builtin_readcyclecounter();
    if (blockIdx.x == 0 && threadIdx.x == 0) reinterpret_cast<unsigned long long *>(out)[1] = c1 - c0;
    float s = 0;
    for (int k = 0; k < NA; ++k) for (int i = 0; i < 16; ++i) s += acc[k][i];
    if (s == 12345.678f) out[0] = s;
}

template <int NA> void chains(int threads, int iters) {
    const float ms = timeit([&](int it) { hipLaunchKernelGGL((k_chains<NA>), dim3(256), dim3(threads), 0, 0, it, g_out); }, iters);
    unsigned long long cyc = 0;
    hipMemcpy(&cyc, reinterpret_cast<char *>(g_out) + 8, 8, hipMemcpyDeviceToHost);
    printf("C   chains %d                                   waves/SIMD %d  NM 16 NV  0  %8.3f ms  %8.2f ns/trip  %7.2f ns/MFMA-slot  %6.2f shader cycles per MFMA slot of the oldest wave\n",
           NA, threads / 256, ms, ms * 1e6 / iters, ms * 1e6 / iters / 16, (double)cyc / iters / 16);
    fflush(stdout);
}

int main(int argc, char **argv) {
    const int iters = argc > 1 ? atoi(argv[1]) : 4000;
    hipMalloc(&g_out, 64);
    printf("# one workgroup per CU unless stated; 16 MFMAs (32x32x16 f16, 4 accumulators) per trip\n");
    run<16, 0, 0, 0>("M   MFMA only", 256, 0, iters, 1);
    run<16, 0, 0, 0>("M   MFMA only", 512, 0, iters, 1);
#define ROW(NV) \
    run<16, NV, 1, 0>("V   fma only", 256, 0, iters, 1); \
    run<16, NV, 2, 0>("MV  MFMA + fma interleaved, same wave", 256, 0, iters, 1); \
    run<16, NV, 2, 0>("MV  MFMA + fma interleaved, 2 waves/SIMD", 512, 0, iters, 1); \
    run<16, NV, 0, 0>("M|V one wave MFMA, the SIMD's other wave fma", 512, 1, iters, 1);
    ROW(1) ROW(2) ROW(4) ROW(6) ROW(8) ROW(12) ROW(16)
    printf("# conversion work of the hidden layers: NV x (v_cvt_pk_f16_f32 + v_pk_max_f16) per MFMA\n");
#define ROWC(NV) \
    run<16, NV, 1, 1>("V   cvt+max only", 256, 0, iters, 1); \
    run<16, NV, 2, 1>("MV  MFMA + cvt+max interleaved, same wave", 256, 0, iters, 1); \
    run<16, NV, 2, 1>("MV  MFMA + cvt+max interleaved, 2 waves/SIMD", 512, 0, iters, 1);
    ROWC(1) ROWC(2) ROWC(4)
    printf("# accumulator chains: NA chains in turn, 16 MFMAs per trip (a dependent MFMA on the same accumulator)\n");
    chains<1>(256, iters); chains<2>(256, iters); chains<4>(256, iters); chains<1>(512, iters); chains<4>(512, iters);
    return 0;
}
