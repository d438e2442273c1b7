// Part 4: volume compositing as a per-ray segmented scan.
//
// k_weights: one wave per ray, 64 samples per step.  Each lane recomputes its sample's
// depth with the sampler's own operations, fetches sigma through the bitmap / word-prefix
// (invalid samples have sigma = 0, exactly like the reference's zero-initialised tensor),
// forms alpha, and a multiplicative wave scan yields the transmittance.  Samples whose
// weight exceeds the threshold are appended to the appearance list: one atomic per wave
// step reserves a contiguous slot range, and the (base, bit mask) pair is kept per ray so
// that the final sum runs over a ray's samples in sample order whatever the slot order was.
// k_composite: one thread per ray sums weight * rgb over those slots, adds the white
// background and clamps.
//
// Reference: raw2alpha (app/tools/utils.py:51-64), dists with a zero last interval
// (app/models/gridnerf_sequential.py:457, 531-534), weight threshold (:479, :553) and the
// sums / white background / clamp / depth of :493-504 and :565-576.
#include "lm_common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kRaysPerBlock = kBlock / LM_WAVE;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d);
    return v;
}

__global__ __launch_bounds__(kBlock) void k_weights(lm_geom g, const float *__restrict__ rays, uint64_t N,
                                                    const uint64_t *__restrict__ bitmap,
                                                    const uint32_t *__restrict__ word_prefix,
                                                    const float *__restrict__ sigma, float distance_scale,
                                                    float weight_thres, float term_eps, float *__restrict__ weight_out,
                                                    uint64_t *__restrict__ app_bits, uint32_t *__restrict__ app_base,
                                                    uint32_t *__restrict__ app_idx, float *__restrict__ app_w,
                                                    float *__restrict__ acc_out, float *__restrict__ depth_out,
                                                    uint32_t *__restrict__ app_count) {
    const unsigned lane = lm_lane();
    const uint64_t r = (uint64_t)blockIdx.x * kRaysPerBlock + threadIdx.x / LM_WAVE;
    if (r >= N) return;
    const int S = g.S;
    const int n_steps = (S + 63) / 64;
    float ray[6];
#pragma unroll
    for (int k = 0; k < 6; ++k) ray[k] = rays[6 * r + k];
    const float rp = lm_ray_param(g, ray);
    float T = 1.0f, acc = 0.0f, depth = 0.0f;
    int step = 0;
    for (; step < n_steps; ++step) {
        const int s = step * 64 + (int)lane;
        const bool in = s < S;
        float z = 0.0f, sg = 0.0f, dist = 0.0f;
        if (in) {
            z = lm_sample_z(g, rp, s);
            if (s + 1 < S) dist = lm_sample_z(g, rp, s + 1) - z;
            const uint64_t flat = r * (uint64_t)S + s;
            const uint64_t w = flat >> 6;
            const unsigned b = (unsigned)(flat & 63);
            const uint64_t bits = bitmap[w];
            if ((bits >> b) & 1ull) sg = sigma[word_prefix[w] + (uint32_t)__popcll(bits & ((1ull << b) - 1ull))];
        }
        const float d2 = dist * distance_scale;
        const float alpha = 1.0f - expf(-sg * d2);
        const float x = in ? (1.0f - alpha) + 1e-10f : 1.0f;
        float incl = x;  // inclusive product scan over the wave
#pragma unroll
        for (int d = 1; d < LM_WAVE; d <<= 1) {
            const float y = __shfl_up(incl, d);
            if (lane >= (unsigned)d) incl *= y;
        }
        float excl = __shfl_up(incl, 1);
        if (lane == 0) excl = 1.0f;
        const float wgt = alpha * (T * excl);
        T = T * __shfl(incl, LM_WAVE - 1);
        if (in && weight_out) weight_out[r * (uint64_t)S + s] = wgt;
        acc += wgt;
        depth += wgt * z;
        const bool is_app = in && (wgt > weight_thres);
        const uint64_t abits = __ballot(is_app);
        uint32_t base = 0;
        if (abits) {
            if (lane == 0) base = atomicAdd(app_count, (uint32_t)__popcll(abits));
            base = __shfl(base, 0);
            if (is_app) {
                const uint32_t slot = base + lm_mbcnt(abits);
                app_idx[slot] = (uint32_t)(r * (uint64_t)S + s);
                app_w[slot] = wgt;
            }
        }
        if (lane == 0) {
            app_bits[r * n_steps + step] = abits;
            app_base[r * n_steps + step] = base;
        }
        if (term_eps > 0.0f && T < term_eps) { ++step; break; }
    }
    // steps skipped by early termination hold no appearance samples
    for (; step < n_steps; ++step) {
        if (lane == 0) { app_bits[r * n_steps + step] = 0; app_base[r * n_steps + step] = 0; }
        if (weight_out) {
            const int s = step * 64 + (int)lane;
            if (s < S) weight_out[r * (uint64_t)S + s] = 0.0f;
        }
    }
    acc = wave_sum(acc);
    depth = wave_sum(depth);
    if (lane == 0) { acc_out[r] = acc; depth_out[r] = depth; }
}

__global__ __launch_bounds__(kBlock) void k_composite(uint64_t N, int n_steps, const uint64_t *__restrict__ app_bits,
                                                      const uint32_t *__restrict__ app_base,
                                                      const float *__restrict__ app_w, const float *__restrict__ rgb,
                                                      const float *__restrict__ acc, int white_bg,
                                                      float *__restrict__ rgb_map) {
    const uint64_t r = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (r >= N) return;
    float c0 = 0.0f, c1 = 0.0f, c2 = 0.0f;
    for (int step = 0; step < n_steps; ++step) {
        const uint64_t bits = app_bits[r * n_steps + step];
        const int n = __popcll(bits);
        const uint32_t base = app_base[r * n_steps + step];
        for (int i = 0; i < n; ++i) {
            const float w = app_w[base + i];
            const float *c = rgb + 3 * (size_t)(base + i);
            c0 = fmaf(w, c[0], c0); c1 = fmaf(w, c[1], c1); c2 = fmaf(w, c[2], c2);
        }
    }
    if (white_bg) {
        const float bgd = 1.0f - acc[r];
        c0 += bgd; c1 += bgd; c2 += bgd;
    }
    rgb_map[3 * r + 0] = fminf(fmaxf(c0, 0.0f), 1.0f);
    rgb_map[3 * r + 1] = fminf(fmaxf(c1, 0.0f), 1.0f);
    rgb_map[3 * r + 2] = fminf(fmaxf(c2, 0.0f), 1.0f);
}

__global__ void k_zero_counters(uint32_t *c) {
    if (threadIdx.x < LM_STAT_WORDS) c[threadIdx.x] = 0;
}

}  // namespace

int lm_check_geom(const lm_geom *g);

extern "C" int lm_weights(const lm_geom *geom, const float *rays, int64_t N, const uint64_t *bitmap,
                          const uint32_t *word_prefix, const float *sigma, float distance_scale, float weight_thres,
                          float term_eps, float *weight_out, uint64_t *app_bits, uint32_t *app_base, uint32_t *app_idx,
                          float *app_w, float *acc, float *depth, uint32_t *counters, void *stream) {
    if (int rc = lm_check_geom(geom)) return rc;
    LM_REQUIRE(N >= 0, "negative ray count");
    LM_REQUIRE(counters != nullptr, "counters is null");
    if (N == 0) return LM_OK;
    LM_REQUIRE(rays && bitmap && word_prefix && sigma && app_bits && app_base && app_idx && app_w && acc && depth,
               "null buffer");
    const unsigned grid = (unsigned)(((uint64_t)N + kRaysPerBlock - 1) / kRaysPerBlock);
    hipLaunchKernelGGL(k_weights, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *geom, rays, (uint64_t)N, bitmap,
                       word_prefix, sigma, distance_scale, weight_thres, term_eps, weight_out, app_bits, app_base, app_idx,
                       app_w, acc, depth, counters + LM_STAT_N_APP);
    LM_CHECK_LAUNCH("k_weights");
    return LM_OK;
}

int lm_launch_composite(int64_t N, int S, const uint64_t *app_bits, const uint32_t *app_base, const float *app_w,
                        const float *rgb, const float *acc, int white_bg, float *rgb_map, hipStream_t stream) {
    if (N == 0) return LM_OK;
    const unsigned grid = (unsigned)(((uint64_t)N + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(k_composite, dim3(grid), dim3(kBlock), 0, stream, (uint64_t)N, (S + 63) / 64, app_bits, app_base,
                       app_w, rgb, acc, white_bg, rgb_map);
    LM_CHECK_LAUNCH("k_composite");
    return LM_OK;
}

int lm_launch_zero_counters(uint32_t *counters, hipStream_t stream) {
    hipLaunchKernelGGL(k_zero_counters, dim3(1), dim3(64), 0, stream, counters);
    LM_CHECK_LAUNCH("k_zero_counters");
    return LM_OK;
}
