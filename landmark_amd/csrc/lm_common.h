// Shared declarations of the gfx950 kernels behind include/landmark_hip.h.
#pragma once
#include <utility>
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/landmark_hip.h"

#define LM_WAVE 64
#define LM_XCDS 8  // accelerator dies, each with its own L2; workgroups are dealt to them round robin

// Error plumbing: thread-local message, negative status.
void lm_set_error(const char *fmt, ...);
#define LM_FAIL(code, ...)         \
    do {                           \
        lm_set_error(__VA_ARGS__); \
        return (code);             \
    } while (0)
#define LM_REQUIRE(cond, ...)                               \
    do {                                                    \
        if (!(cond)) LM_FAIL(LM_ERR_INVALID, __VA_ARGS__);  \
    } while (0)
#define LM_CHECK_LAUNCH(name)                                                              \
    do {                                                                                   \
        hipError_t e_ = hipGetLastError();                                                 \
        if (e_ != hipSuccess) LM_FAIL(LM_ERR_LAUNCH, "%s: %s", name, hipGetErrorString(e_)); \
    } while (0)

static inline bool lm_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Launch attributes and device facts are cached per thread and device (index of the current device, clamped)
#define LM_MAX_DEVICES 64
int lm_current_device(void);

// Number of workgroups for grid-stride kernels: enough resident waves to cover every CU
// several times over; 256 CUs in 8 XCDs on MI355X.
int lm_persistent_blocks(int blocks_per_cu);

// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2).  Remap the
// hardware block id so that blocks resident on one XCD own neighbouring tiles.
__device__ __forceinline__ unsigned lm_xcd_swizzle(unsigned bid, unsigned nblocks) {
    const unsigned nx = 8;
    if (nblocks % nx) return bid;
    return (bid % nx) * (nblocks / nx) + bid / nx;
}

// ---------------------------------------------------------------------------------------
// Geometry with the reference's rounding: every product and sum is a separate float
// operation (the translation unit is built with -ffp-contract=off), divisions are IEEE.
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ float lm_ray_param(const lm_geom &g, const float *ray) {
    if (g.sampler == LM_SAMPLER_HULL) {
        float o_z = ray[2] - g.aabb[2];
        float far = -(o_z / ray[5]);
        if (ray[5] >= 0.0f) far = g.far_;
        return far;
    }
    float tmin = -INFINITY;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        float v = ray[3 + k] == 0.0f ? 1e-6f : ray[3 + k];
        float ra = (g.aabb[3 + k] - ray[k]) / v;
        float rb = (g.aabb[k] - ray[k]) / v;
        float m = ra < rb ? ra : rb;
        if (ra != ra || rb != rb) m = NAN;
        if (m > tmin || m != m) tmin = m;
    }
    if (tmin < g.near_) tmin = g.near_;
    if (tmin > g.far_) tmin = g.far_;
    return tmin;
}

__device__ __forceinline__ float lm_sample_z(const lm_geom &g, float ray_param, int s) {
    if (g.sampler == LM_SAMPLER_HULL) {
        float b = ray_param * g.tab_t[s];
        return g.tab_a[s] + b;
    }
    return ray_param + g.tab_a[s];
}

__device__ __forceinline__ void lm_point(const float *ray, float z, float *pt) {
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        float m = ray[3 + k] * z;
        pt[k] = ray[k] + m;
    }
}

__device__ __forceinline__ bool lm_inside(const lm_geom &g, const float *pt) {
    bool out = false;
#pragma unroll
    for (int k = 0; k < 3; ++k) out |= (g.aabb[k] > pt[k]) | (pt[k] > g.aabb[3 + k]);
    return !out;
}

__device__ __forceinline__ void lm_normalise(const lm_geom &g, const float *pt, float *q) {
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        float d = pt[k] - g.aabb[k];
        float m = d * g.inv_aabb[k];
        q[k] = m - 1.0f;
    }
}

// Block of a block-stacked model and the coordinates inside it, with the reference's float
// operations (assign_blocks_to_samples, app/models/gridnerf_parallel.py:300-328; floor_divide and
// remainder as ATen defines them for floats).  q[0], q[1] are replaced; returns the block index.
__device__ __forceinline__ float lm_floor_divide(float a, float b) {
    const float mod = fmodf(a, b);
    float div = (a - mod) / b;
    if (mod != 0.0f && ((b < 0.0f) != (mod < 0.0f))) div = div - 1.0f;
    if (div == 0.0f) return copysignf(0.0f, a / b);
    float fl = floorf(div);
    if (div - fl > 0.5f) fl = fl + 1.0f;
    return fl;
}
__device__ __forceinline__ float lm_remainder(float a, float b) {
    float mod = fmodf(a, b);
    if (mod != 0.0f && ((b < 0.0f) != (mod < 0.0f))) mod = mod + b;
    return mod;
}
__device__ __forceinline__ int lm_block_coords(const lm_geom &g, float *q) {
    const float d1 = (float)g.div1;
    const float xs = (q[0] + 1.0f) / g.blk_w, ys = (q[1] + 1.0f) / g.blk_h;
    const float fx = floorf(xs) * d1;
    const float b = fx + floorf(ys);
    const float bx = lm_floor_divide(b, d1), by = lm_remainder(b, d1);
    const float sz[2] = {g.blk_w, g.blk_h}, bi[2] = {bx, by};
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const float m0 = bi[k] * sz[k];
        const float lo = -1.0f + m0;
        const float m1 = (bi[k] + 1.0f) * sz[k];
        const float hi = -1.0f + m1;
        const float t = (q[k] - lo) * 2.0f;
        const float u = t / (hi - lo);
        q[k] = u - 1.0f;
    }
    // b is integer valued; the clamp keeps the conversion defined for far-away points
    return (int)fminf(fmaxf(b, -1.0f), 1.0e9f);
}

// Trilinear lookup with zero padding and align_corners=True in ATen's operation order
// (corner order tnw, tne, tsw, tse, bnw, bne, bsw, bse; weight = (x)(y)(z) left to right;
// each value*weight rounded before it is added).
__device__ __forceinline__ float lm_alpha_lookup(const lm_geom &g, const float *pt) {
    float c[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        float d = pt[k] - g.vol_aabb_min[k];
        float m = d * g.vol_inv[k];
        c[k] = m - 1.0f;
    }
    const int W = g.vw, H = g.vh, D = g.vd;
    float ix = ((c[0] + 1.0f) / 2.0f) * (float)(W - 1);
    float iy = ((c[1] + 1.0f) / 2.0f) * (float)(H - 1);
    float iz = ((c[2] + 1.0f) / 2.0f) * (float)(D - 1);
    float fx = floorf(ix), fy = floorf(iy), fz = floorf(iz);
    float wx[2] = {(fx + 1.0f) - ix, ix - fx};
    float wy[2] = {(fy + 1.0f) - iy, iy - fy};
    float wz[2] = {(fz + 1.0f) - iz, iz - fz};
    // clamp before the int conversion so that far-away points cannot overflow
    fx = fminf(fmaxf(fx, -2.0f), (float)W);
    fy = fminf(fmaxf(fy, -2.0f), (float)H);
    fz = fminf(fmaxf(fz, -2.0f), (float)D);
    int x0 = (int)fx, y0 = (int)fy, z0 = (int)fz;
    float out = 0.0f;
    if (g.vol_dtype == LM_CELLS) {
        // one byte holds the eight corners of the cell (out-of-range corners are 0 bits); a set
        // corner contributes 1.0f * w = w, added in the same order
        if (x0 < -1 || x0 >= W || y0 < -1 || y0 >= H || z0 < -1 || z0 >= D) return 0.0f;
        const size_t ci = ((size_t)(z0 + 1) * (H + 1) + (y0 + 1)) * (W + 1) + (x0 + 1);
        const unsigned bits = reinterpret_cast<const uint8_t *>(g.vol)[ci];
#pragma unroll
        for (int n = 0; n < 8; ++n)
            if (bits & (1u << n)) out = out + (wx[n & 1] * wy[(n >> 1) & 1]) * wz[n >> 2];
        return out;
    }
#pragma unroll
    for (int zz = 0; zz < 2; ++zz)
#pragma unroll
        for (int yy = 0; yy < 2; ++yy)
#pragma unroll
            for (int xx = 0; xx < 2; ++xx) {
                int x = x0 + xx, y = y0 + yy, z = z0 + zz;
                if (x >= 0 && x < W && y >= 0 && y < H && z >= 0 && z < D) {
                    float w = (wx[xx] * wy[yy]) * wz[zz];
                    const size_t i = ((size_t)z * H + y) * W + x;
                    const float val = g.vol_dtype == LM_U8 ? (float)reinterpret_cast<const uint8_t *>(g.vol)[i]
                                                           : reinterpret_cast<const float *>(g.vol)[i];
                    float t = val * w;
                    out = out + t;
                }
            }
    return out;
}

// lm_alpha_lookup(g, pt) > 0 for a cell table, without forming the sum: every term is a
// product of three weights in [0, 1] (never small enough to underflow: a weight is a difference
// of numbers below 2^24 with spacing >= 2^-24 of their size), so the sum is positive exactly when a
// set corner has three non-zero weights.  The lower weight (f + 1) - i is never zero; the upper
// weight i - f is zero when the coordinate is an integer.
__device__ __forceinline__ bool lm_cells_positive(const lm_geom &g, const float *pt) {
    float c[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        float d = pt[k] - g.vol_aabb_min[k];
        float m = d * g.vol_inv[k];
        c[k] = m - 1.0f;
    }
    const int W = g.vw, H = g.vh, D = g.vd;
    const float ix = ((c[0] + 1.0f) / 2.0f) * (float)(W - 1);
    const float iy = ((c[1] + 1.0f) / 2.0f) * (float)(H - 1);
    const float iz = ((c[2] + 1.0f) / 2.0f) * (float)(D - 1);
    float fx = floorf(ix), fy = floorf(iy), fz = floorf(iz);
    unsigned live = 0xFFu;
    if (ix - fx == 0.0f) live &= 0x55u;  // corners with xx = 1 weigh nothing
    if (iy - fy == 0.0f) live &= 0x33u;
    if (iz - fz == 0.0f) live &= 0x0Fu;
    fx = fminf(fmaxf(fx, -2.0f), (float)W);
    fy = fminf(fmaxf(fy, -2.0f), (float)H);
    fz = fminf(fmaxf(fz, -2.0f), (float)D);
    const int x0 = (int)fx, y0 = (int)fy, z0 = (int)fz;
    if (x0 < -1 || x0 >= W || y0 < -1 || y0 >= H || z0 < -1 || z0 >= D) return false;
    const size_t ci = ((size_t)(z0 + 1) * (H + 1) + (y0 + 1)) * (W + 1) + (x0 + 1);
    return (reinterpret_cast<const uint8_t *>(g.vol)[ci] & live) != 0u;
}

// Sample validity = inside the AABB and (no volume or lookup > threshold)
__device__ __forceinline__ bool lm_sample_valid(const lm_geom &g, const float *pt) {
    bool ok = lm_inside(g, pt);
    if (ok && g.vol) ok = lm_alpha_lookup(g, pt) > g.vol_thre;
    return ok;
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant expression
template <typename F, int... I> __device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F> __device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// ---------------------------------------------------------------------------------------
// wave64 helpers
// ---------------------------------------------------------------------------------------
__device__ __forceinline__ unsigned lm_lane() { return __lane_id(); }
__device__ __forceinline__ unsigned lm_mbcnt(uint64_t mask) {  // set bits of mask below this lane
    return __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
}

// Rays waiting for the marching kernel are kept in four lists by their number of valid samples
// (an upper bound of the work they are), list b at ray_list + b * N, so that the queue can hand
// out the long ones first: a launch then does not end with a few long rays marching alone.
#define LM_RAY_BINS 4
__device__ __forceinline__ int lm_ray_bin(uint32_t n_valid) {
    return n_valid >= 64u ? 0 : (n_valid >= 32u ? 1 : (n_valid >= 12u ? 2 : 3));
}
// append the lanes with `mine` set to their lists (one atomic per wave and non-empty list)
__device__ __forceinline__ void lm_ray_enqueue(bool mine, int bin, uint32_t r, uint32_t *ray_list, uint32_t N,
                                               uint32_t *bins) {
#pragma unroll
    for (int b = 0; b < LM_RAY_BINS; ++b) {
        const uint64_t mask = __ballot(mine && bin == b);
        if (mask == 0) continue;
        uint32_t slot = 0;
        const int first = __ffsll((unsigned long long)mask) - 1;
        if ((int)__lane_id() == first) slot = atomicAdd(bins + b, (uint32_t)__popcll(mask));
        slot = __shfl(slot, first);
        if (mine && bin == b)
            ray_list[(size_t)b * N + slot +
                     __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u))] = r;
    }
}

// A ray that asks for `cnt` entries from position `first` of a list with room for `cap`: true when it has
// entries and they fit.  Rays that do not fit are counted in *overflow (one atomic per wave that has any) and
// are treated by the caller as rays without entries.  Called by all lanes of the wave.
__device__ __forceinline__ bool lm_ray_fits(uint32_t cnt, uint32_t first, uint32_t cap, uint32_t *overflow) {
    const bool over = cnt != 0u && (uint64_t)first + cnt > (uint64_t)cap;
    const uint64_t mask = __ballot(over);
    if (mask != 0ull && (int)__lane_id() == __ffsll((unsigned long long)mask) - 1) atomicAdd(overflow, (uint32_t)__popcll(mask));
    return cnt != 0u && !over;
}

// Visiting order of the whole-chunk render when the rays are image rows of length W (a
// multiple of 8): position o -> ray index, 8 x 8 pixel tiles inside bands of 8 rows; the rays
// behind the last full band keep their order.  A bijection on [0, N).
__device__ __forceinline__ uint32_t lm_ray_order(uint32_t o, uint32_t N, uint32_t W) {
    if (W == 0) return o;
    const uint32_t band = 8u * W;
    const uint32_t full = (N / band) * band;
    if (o >= full) return o;
    const uint32_t b = o / band, t = o - b * band;
    const uint32_t tile = t >> 6, in = t & 63u;
    return b * band + (in >> 3) * W + tile * 8u + (in & 7u);
}

// Iterates the set bits of the sample bitmap in [flat0, flat1): the valid samples of one ray.
// With a word mask (bit i set = the ray has valid samples in its i-th bitmap word, written by the cull of
// the whole-chunk render for rays of up to 64 words) the walk jumps from one non-empty word to the next and
// asks for the word after it at once, so that a long, mostly empty ray costs one memory round trip per
// non-empty word, overlapped with the work on the previous one, instead of one per word.
struct BitWalk {
    const uint64_t *bitmap;
    const uint32_t *prefix;
    uint64_t w, w0, w_last, bits, flat1;
    uint64_t todo, ahead;  // masked walk: words still to visit (relative to w0), the next one's content
    uint32_t pos;
    bool masked;
    __device__ __forceinline__ void start(const uint64_t *bm, const uint32_t *pf, uint64_t flat0, uint64_t flat1_) {
        bitmap = bm; prefix = pf; flat1 = flat1_; masked = false; todo = 0; ahead = 0;
        w = w0 = flat0 >> 6; w_last = (flat1_ - 1) >> 6;
        const uint64_t raw = bm[w];
        const unsigned b0 = (unsigned)(flat0 & 63);
        const uint64_t below = b0 ? ((1ull << b0) - 1ull) : 0ull;
        pos = pf[w] + (uint32_t)__popcll(raw & below);
        bits = mask_tail(raw & ~below, w);
    }
    // same walk when the compact position of the first sample is known (a per-ray table); `mask` as above,
    // ~0 when not known
    __device__ __forceinline__ void start_at(const uint64_t *bm, uint64_t flat0, uint64_t flat1_, uint32_t pos0,
                                             uint64_t mask = ~0ull) {
        bitmap = bm; prefix = nullptr; flat1 = flat1_;
        w = w0 = flat0 >> 6; w_last = (flat1_ - 1) >> 6;
        const unsigned b0 = (unsigned)(flat0 & 63);
        const uint64_t below = b0 ? ((1ull << b0) - 1ull) : 0ull;
        pos = pos0;
        masked = mask != ~0ull && w_last - w0 < 64;
        if (!masked) {
            todo = 0; ahead = 0;
            bits = mask_tail(bm[w] & ~below, w);
            return;
        }
        todo = mask;
        bits = 0;
        if (todo & 1ull) bits = mask_tail(bm[w0] & ~below, w0);
        todo &= ~1ull;
        fetch_ahead();
    }
    __device__ __forceinline__ void fetch_ahead() {
        if (todo) ahead = bitmap[w0 + (uint64_t)(__ffsll((unsigned long long)todo) - 1)];
    }
    __device__ __forceinline__ uint64_t mask_tail(uint64_t x, uint64_t at) const {
        if (at == w_last) {
            const unsigned e = (unsigned)(flat1 & 63);
            if (e) x &= (1ull << e) - 1ull;
        }
        return x;
    }
    // next set bit -> flat index; false when exhausted.  `pos` is the compact position of it.
    __device__ __forceinline__ bool next(uint64_t &flat) {
        while (bits == 0) {
            if (masked) {
                if (todo == 0) return false;
                w = w0 + (uint64_t)(__ffsll((unsigned long long)todo) - 1);
                todo &= todo - 1;
                bits = mask_tail(ahead, w);
                fetch_ahead();
            } else {
                if (w == w_last) return false;
                ++w;
                bits = mask_tail(bitmap[w], w);
            }
        }
        const int b = __ffsll((unsigned long long)bits) - 1;
        bits &= bits - 1;
        flat = w * 64 + (uint64_t)b;
        return true;
    }
};
