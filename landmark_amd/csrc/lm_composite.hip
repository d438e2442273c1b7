// Part 4: volume compositing as a per-ray segmented scan over the valid samples only.
//
// k_weights: one lane per ray.  The ray's valid samples are the set bits of its slice of
// the sample bitmap; their densities sit contiguously in the compacted sigma array.  The
// lane walks those bits in sample order and carries the transmittance along, which is
// exactly the sequential product torch.cumprod forms; culled samples have sigma = 0 in the
// reference, i.e. alpha = 0 and a factor (1 - 0 + 1e-10) that rounds to 1.0f, so skipping
// them changes nothing.  Two passes: the first stores the weights of the valid samples and
// counts those above the threshold, a wave-wide prefix sum plus one atomic per wave reserves
// a contiguous slot range per ray in the appearance list, the second pass fills the slots.
// A ray's slots are therefore contiguous and in sample order.
// k_composite: one lane per ray sums weight * rgb over its slots, adds the white
// background and clamps.
// In the whole-chunk render the weights come from the marching kernel (density gather fused with
// the transmittance walk); k_app_slots then builds the appearance list from the stored weights the
// way k_weights' second pass does.  k_weights remains the stage-level form.
//
// Reference: raw2alpha (app/tools/utils.py:51-64), dists with a zero last interval
// (app/models/gridnerf_sequential.py:457, 531-534), weight threshold (:479, :553) and the
// sums / white background / clamp / depth of :493-504 and :565-576.
#include "lm_common.h"

namespace {

constexpr int kBlock = 256;
#ifndef LM_SLOTS_STAGE
#define LM_SLOTS_STAGE 4096
#endif
#ifndef LM_COMPOSITE_STAGE
#define LM_COMPOSITE_STAGE 512
#endif
// list entries a wave moves through LDS: k_app_slots its whole range at once, k_composite a window at a time
constexpr int kSlotsStage = LM_SLOTS_STAGE, kCompositeStage = LM_COMPOSITE_STAGE;

__global__ __launch_bounds__(kBlock) void k_weights(lm_geom g, const float *__restrict__ rays, uint64_t N,
                                                    const uint64_t *__restrict__ bitmap,
                                                    const uint32_t *__restrict__ word_prefix,
                                                    const float *__restrict__ sigma, float distance_scale,
                                                    float weight_thres, float term_eps, float *__restrict__ w_valid,
                                                    float *__restrict__ weight_out, uint32_t *__restrict__ app_first,
                                                    uint32_t *__restrict__ app_cnt, uint32_t *__restrict__ app_idx,
                                                    float *__restrict__ app_w, float *__restrict__ acc_out,
                                                    float *__restrict__ depth_out, uint32_t *__restrict__ app_count) {
    const unsigned lane = lm_lane();
    const uint64_t r = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const bool active = r < N;
    const int S = g.S;
    float acc = 0.0f, depth = 0.0f;
    uint32_t cnt = 0, p_first = 0, p_end = 0;
    float rp = 0.0f;
    const uint64_t flat0 = r * (uint64_t)S;
    if (active) {
        float ray[6];
#pragma unroll
        for (int k = 0; k < 6; ++k) ray[k] = rays[6 * r + k];
        rp = lm_ray_param(g, ray);
        BitWalk it;
        it.start(bitmap, word_prefix, flat0, flat0 + S);
        p_first = it.pos;
        uint32_t p = p_first;
        float T = 1.0f;
        uint64_t flat;
        while (it.next(flat)) {
            const int s = (int)(flat - flat0);
            const float z = lm_sample_z(g, rp, s);
            const float dist = (s + 1 < S) ? lm_sample_z(g, rp, s + 1) - z : 0.0f;
            const float d2 = dist * distance_scale;
            const float alpha = 1.0f - expf(-sigma[p] * d2);
            const float wgt = alpha * T;
            T = T * ((1.0f - alpha) + 1e-10f);
            w_valid[p] = wgt;
            if (weight_out) weight_out[flat] = wgt;
            acc += wgt;
            depth += wgt * z;
            cnt += wgt > weight_thres;
            ++p;
            if (term_eps > 0.0f && T < term_eps) break;
        }
        p_end = p;
    }
    // slot range per ray: exclusive prefix over the wave + one atomic
    uint32_t incl = cnt;
#pragma unroll
    for (int d = 1; d < LM_WAVE; d <<= 1) {
        const uint32_t y = __shfl_up(incl, d);
        if (lane >= (unsigned)d) incl += y;
    }
    const uint32_t total = __shfl(incl, LM_WAVE - 1);
    uint32_t base = 0;
    if (total) {
        if (lane == 0) base = atomicAdd(app_count, total);
        base = __shfl(base, 0);
    }
    if (!active) return;
    uint32_t slot = base + incl - cnt;
    app_first[r] = slot;
    app_cnt[r] = cnt;
    acc_out[r] = acc;
    depth_out[r] = depth;
    if (cnt) {
        BitWalk it;
        it.start(bitmap, word_prefix, flat0, flat0 + S);
        uint64_t flat;
        for (uint32_t p = p_first; p < p_end; ++p) {
            it.next(flat);
            const float wgt = w_valid[p];
            if (wgt > weight_thres) {
                app_idx[slot] = (uint32_t)flat;
                app_w[slot] = wgt;
                ++slot;
            }
        }
    }
}

// The appearance list is laid out wave by wave: the 64 rays a wave handles (consecutive positions of the visiting
// order) own one contiguous range of slots.  k_app_slots and k_composite are one lane per ray, so a lane's slots
// are a short run somewhere in that range: written or read directly, every access of the wave touches 64 different
// cache lines, each of which is visited again a few entries later (partial-line writes reach the memory several
// times over).  Both kernels therefore move the wave's range through LDS (k_app_slots when it has at most STAGE
// entries, k_composite in windows of STAGE): the lanes work on the LDS copy in their own order, the wave copies
// the range to or from memory in whole lines.  A workgroup is one wave.
template <int STAGE>
__global__ __launch_bounds__(LM_WAVE) void k_composite(uint64_t N, const uint32_t *__restrict__ app_first,
                                                       const uint32_t *__restrict__ app_cnt,
                                                       const float *__restrict__ app_w, const float *__restrict__ rgb,
                                                       const float *__restrict__ acc, int white_bg, uint32_t row,
                                                       float *__restrict__ rgb_map) {
    __shared__ float s_w[STAGE];
    __shared__ float s_c[3 * STAGE];
    const unsigned lane = lm_lane();
    const uint64_t o = (uint64_t)blockIdx.x * LM_WAVE + lane;
    const bool live = o < N;
    const uint64_t r = live ? lm_ray_order((uint32_t)o, (uint32_t)N, row) : 0;
    const uint32_t first = live ? app_first[r] : 0u, n = live ? app_cnt[r] : 0u;
    // the slots this wave reads: [lo, hi) over its rays that have any
    uint32_t lo = n ? first : 0xFFFFFFFFu, hi = n ? first + n : 0u;
#pragma unroll
    for (int d = 1; d < LM_WAVE; d <<= 1) {
        lo = min(lo, (uint32_t)__shfl_xor((int)lo, d));
        hi = max(hi, (uint32_t)__shfl_xor((int)hi, d));
    }
    // Windows of STAGE slots over [lo, hi): the wave loads a window in whole lines, every lane adds its slots of
    // that window.  Windows ascend, so a lane's sum keeps the slot order.  A layout whose ranges lie far apart
    // (hi - lo much larger than the slots in use) is read directly instead.
    uint32_t used = n;
#pragma unroll
    for (int d = 1; d < LM_WAVE; d <<= 1) used += (uint32_t)__shfl_xor((int)used, d);
    const bool staged = hi > lo && (uint64_t)(hi - lo) <= 2ull * used + STAGE;
    float c0 = 0.0f, c1 = 0.0f, c2 = 0.0f;
    if (staged) {
        for (uint64_t win = lo; win < hi; win += STAGE) {  // 64-bit: hi may be within STAGE of 2^32
            const uint32_t len = (uint32_t)min((uint64_t)STAGE, hi - win);
            if (win != lo) __builtin_amdgcn_wave_barrier();  // every lane is done with the previous window
            // four loads in flight per lane and array (indices past the window repeat its last entry)
            constexpr int kAhead = 4;
            for (uint32_t i0 = 0; i0 < 3u * len; i0 += kAhead * LM_WAVE) {
                float c[kAhead], w[kAhead];
#pragma unroll
                for (int u = 0; u < kAhead; ++u) {
                    const uint32_t i = i0 + u * LM_WAVE + lane;
                    c[u] = rgb[3 * (size_t)win + min(i, 3u * len - 1u)];
                    if (i0 < len) w[u] = app_w[win + min(i, len - 1u)];
                }
#pragma unroll
                for (int u = 0; u < kAhead; ++u) {
                    const uint32_t i = i0 + u * LM_WAVE + lane;
                    if (i < 3u * len) s_c[i] = c[u];
                    if (i < len) s_w[i] = w[u];
                }
            }
            // LDS operations of one wave complete in order; the fences only pin the compiler
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (n) {
                const uint64_t from = max((uint64_t)first, win), to = min((uint64_t)first + n, win + len);
                // four entries per trip, their LDS reads issued together; the sums stay in slot order
                constexpr int kTrip = 4;
                for (uint64_t q = from; q < to; q += kTrip) {
                    float w[kTrip], c[kTrip][3];
#pragma unroll
                    for (int u = 0; u < kTrip; ++u) {
                        const uint32_t at = (uint32_t)(min(q + u, to - 1) - win);
                        w[u] = s_w[at];
                        c[u][0] = s_c[3 * at]; c[u][1] = s_c[3 * at + 1]; c[u][2] = s_c[3 * at + 2];
                    }
#pragma unroll
                    for (int u = 0; u < kTrip; ++u)
                        if (q + u < to) {
                            c0 = fmaf(w[u], c[u][0], c0); c1 = fmaf(w[u], c[u][1], c1); c2 = fmaf(w[u], c[u][2], c2);
                        }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        }
    } else if (live) {
        // eight slots per trip, all loads issued before the sums (which stay in slot order)
        constexpr int kBatch = 8;
        for (uint32_t i = 0; i < n; i += kBatch) {
            float w[kBatch], c[kBatch][3];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) {
                const uint32_t s = first + (i + u < n ? i + u : n - 1);
                w[u] = app_w[s];
                c[u][0] = rgb[3 * (size_t)s]; c[u][1] = rgb[3 * (size_t)s + 1]; c[u][2] = rgb[3 * (size_t)s + 2];
            }
#pragma unroll
            for (int u = 0; u < kBatch; ++u)
                if (i + u < n) {
                    c0 = fmaf(w[u], c[u][0], c0); c1 = fmaf(w[u], c[u][1], c1); c2 = fmaf(w[u], c[u][2], c2);
                }
        }
    }
    if (!live) return;
    if (white_bg) {
        const float bgd = 1.0f - acc[r];
        c0 += bgd; c1 += bgd; c2 += bgd;
    }
    rgb_map[3 * r + 0] = fminf(fmaxf(c0, 0.0f), 1.0f);
    rgb_map[3 * r + 1] = fminf(fmaxf(c1, 0.0f), 1.0f);
    rgb_map[3 * r + 2] = fminf(fmaxf(c2, 0.0f), 1.0f);
}

// Appearance list from stored weights: a contiguous slot range per ray (wave prefix + one
// atomic), filled in sample order from the weights of the ray's samples [first, p_end).
template <int STAGE>
__global__ __launch_bounds__(LM_WAVE) void k_app_slots(int S, uint64_t N, const uint64_t *__restrict__ bitmap,
                                                       const uint32_t *__restrict__ p_first,
                                                       const uint64_t *__restrict__ word_mask,
                                                       const float *__restrict__ w_valid, float weight_thres,
                                                       uint32_t *__restrict__ app_cnt,
                                                       const uint32_t *__restrict__ p_end,
                                                       uint32_t *__restrict__ app_first, uint32_t *__restrict__ app_idx,
                                                       float *__restrict__ app_w, uint32_t *__restrict__ app_count,
                                                       uint32_t row, uint32_t cap_app, uint32_t *__restrict__ overflow) {
    __shared__ uint32_t s_idx[STAGE];
    __shared__ float s_w[STAGE];
    const unsigned lane = lm_lane();
    const uint64_t o = (uint64_t)blockIdx.x * LM_WAVE + lane;
    const bool live = o < N;
    const uint64_t r = live ? lm_ray_order((uint32_t)o, (uint32_t)N, row) : o;
    const uint32_t cnt = live ? app_cnt[r] : 0;
    uint32_t incl = cnt;
#pragma unroll
    for (int d = 1; d < LM_WAVE; d <<= 1) {
        const uint32_t y = __shfl_up(incl, d);
        if (lane >= (unsigned)d) incl += y;
    }
    const uint32_t total = __shfl(incl, LM_WAVE - 1);
    uint32_t base = 0;
    if (total) {
        if (lane == 0) base = atomicAdd(app_count, total);
        base = __shfl(base, 0);
    }
    uint32_t slot = base + incl - cnt;
    const bool fits = lm_ray_fits(cnt, slot, cap_app, overflow);
    // through LDS when the wave's range is short enough and lies below the capacity as a whole
    const bool staged = total != 0u && total <= (uint32_t)STAGE && (uint64_t)base + total <= (uint64_t)cap_app;
    if (live) {
        app_first[r] = slot;
        if (cnt && !fits) {
            // no room for this ray's samples: it keeps the background colour (and is counted); the slots below the
            // capacity that its range covers still get a sample index of this chunk and weight zero
            app_cnt[r] = 0;
            for (uint32_t i = slot; i < cap_app && i < slot + cnt; ++i) { app_idx[i] = (uint32_t)(r * (uint64_t)S); app_w[i] = 0.0f; }
        } else if (cnt) {
            BitWalk it;
            it.start_at(bitmap, r * (uint64_t)S, (r + 1) * (uint64_t)S, p_first[r], word_mask ? word_mask[r] : ~0ull);
            const uint32_t end = p_end[r], last = slot + cnt;
            uint64_t flat;
            // eight weights per trip so that their loads overlap; the walk over the bitmap stays in order and ends
            // with the ray's last entry
            constexpr int kBatch = 8;
            for (uint32_t p = it.pos; p < end && slot < last; p += kBatch) {
                float wgt[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) wgt[u] = w_valid[p + u < end ? p + u : end - 1];
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    if (p + u >= end) break;
                    it.next(flat);
                    if (wgt[u] > weight_thres && slot < last) {
                        if (staged) {
                            s_idx[slot - base] = (uint32_t)flat;
                            s_w[slot - base] = wgt[u];
                        } else {
                            app_idx[slot] = (uint32_t)flat;
                            app_w[slot] = wgt[u];
                        }
                        ++slot;
                    }
                }
            }
        }
    }
    if (staged) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        for (uint32_t i = lane; i < total; i += LM_WAVE) {
            app_idx[base + i] = s_idx[i];
            app_w[base + i] = s_w[i];
        }
    }
}

__global__ void k_zero_counters(uint32_t *c) {
    if (threadIdx.x < LM_STAT_WORDS) c[threadIdx.x] = 0;
}

}  // namespace

int lm_check_geom(const lm_geom *g);

extern "C" int lm_weights(const lm_geom *geom, const float *rays, int64_t N, const uint64_t *bitmap,
                          const uint32_t *word_prefix, const float *sigma, float distance_scale, float weight_thres,
                          float term_eps, float *w_valid, float *weight_out, uint32_t *app_first, uint32_t *app_cnt,
                          uint32_t *app_idx, float *app_w, float *acc, float *depth, uint32_t *counters, void *stream) {
    if (int rc = lm_check_geom(geom)) return rc;
    LM_REQUIRE(N >= 0, "negative ray count");
    LM_REQUIRE(counters != nullptr, "counters is null");
    if (N == 0) return LM_OK;
    LM_REQUIRE(rays && bitmap && word_prefix && sigma && w_valid && app_first && app_cnt && app_idx && app_w && acc && depth,
               "null buffer");
    const unsigned grid = (unsigned)(((uint64_t)N + kBlock - 1) / kBlock);
    hipLaunchKernelGGL(k_weights, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *geom, rays, (uint64_t)N, bitmap,
                       word_prefix, sigma, distance_scale, weight_thres, term_eps, w_valid, weight_out, app_first, app_cnt,
                       app_idx, app_w, acc, depth, counters + LM_STAT_N_APP);
    LM_CHECK_LAUNCH("k_weights");
    return LM_OK;
}

int lm_launch_composite(int64_t N, const uint32_t *app_first, const uint32_t *app_cnt, const float *app_w,
                        const float *rgb, const float *acc, int white_bg, uint32_t row, float *rgb_map,
                        hipStream_t stream) {
    if (N == 0) return LM_OK;
    const unsigned grid = (unsigned)(((uint64_t)N + LM_WAVE - 1) / LM_WAVE);
    hipLaunchKernelGGL(k_composite<kCompositeStage>, dim3(grid), dim3(LM_WAVE), 0, stream, (uint64_t)N, app_first, app_cnt, app_w, rgb,
                       acc, white_bg, row, rgb_map);
    LM_CHECK_LAUNCH("k_composite");
    return LM_OK;
}

extern "C" int lm_composite_rgb(int64_t N, const uint32_t *app_first, const uint32_t *app_cnt, const float *app_w,
                                const float *rgb, const float *acc, int32_t white_bg, float *rgb_map, void *stream) {
    LM_REQUIRE(N >= 0, "negative ray count");
    if (N == 0) return LM_OK;
    LM_REQUIRE((uint64_t)N < (1ull << 32), "ray count does not fit 32 bits");
    LM_REQUIRE(app_first && app_cnt && app_w && rgb && acc && rgb_map, "null buffer");
    return lm_launch_composite(N, app_first, app_cnt, app_w, rgb, acc, white_bg, 0u, rgb_map, (hipStream_t)stream);
}

int lm_launch_zero_counters(uint32_t *counters, hipStream_t stream) {
    hipLaunchKernelGGL(k_zero_counters, dim3(1), dim3(64), 0, stream, counters);
    LM_CHECK_LAUNCH("k_zero_counters");
    return LM_OK;
}

int lm_launch_app_slots(int S, int64_t N, const uint64_t *bitmap, const uint32_t *p_first, const uint64_t *word_mask,
                        const float *w_valid,
                        float weight_thres, uint32_t *app_cnt, const uint32_t *p_end, uint32_t *app_first,
                        uint32_t *app_idx, float *app_w, uint32_t *app_count, uint32_t row, uint32_t cap_app,
                        uint32_t *overflow, hipStream_t stream) {
    const unsigned grid = (unsigned)(((uint64_t)N + LM_WAVE - 1) / LM_WAVE);
    hipLaunchKernelGGL(k_app_slots<kSlotsStage>, dim3(grid), dim3(LM_WAVE), 0, stream, S, (uint64_t)N, bitmap, p_first, word_mask,
                       w_valid, weight_thres, app_cnt, p_end, app_first, app_idx, app_w, app_count, row, cap_app, overflow);
    LM_CHECK_LAUNCH("k_app_slots");
    return LM_OK;
}
