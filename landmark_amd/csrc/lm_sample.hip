// Part 1: ray sampling, AABB / occupancy culling and stable compaction.
//
// Samples are numbered ray*S + s.  A wave owns 64 consecutive samples, decides their
// validity, and stores the 64 decisions as one bitmap word (wave ballot).  Compaction is
// a prefix sum over the words' popcounts:
//   k_sample_cull  bitmap words + one popcount per workgroup (4096 samples)
//   k_scan_blocks  exclusive scan of the workgroup counts (one workgroup), total -> counters
//   k_emit         per-word prefix and the ascending list of valid flat indices
// The list order is the row-major order of the reference's boolean-mask indexing
// (app/models/gridnerf_sequential.py:461-465, 472), so indices match it exactly.
//
// The whole-chunk render needs the decisions but no global order of the valid samples; it takes
//   k_cull_rays_setup / k_cull_rays_setup_serial  one lane per (ray, word) or per ray: bitmap, a
//       contiguous range of compact positions per ray, and the rays filed into the marching queue
// which make bit-identical decisions (the same device functions of lm_common.h).
#include <limits.h>

#include <algorithm>

#include "lm_common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kWordsPerBlock = 64;  // 4096 samples per workgroup
constexpr int kWordsPerWave = kWordsPerBlock / (kBlock / LM_WAVE);

__global__ __launch_bounds__(kBlock) void k_sample_cull(lm_geom g, const float *__restrict__ rays, uint64_t total,
                                                        uint64_t n_words, uint64_t *__restrict__ bitmap,
                                                        uint32_t *__restrict__ block_count, float *__restrict__ z_out) {
    __shared__ uint32_t s_cnt[kBlock / LM_WAVE];
    const unsigned lane = lm_lane();
    const unsigned wave = threadIdx.x / LM_WAVE;
    const uint64_t w0 = (uint64_t)blockIdx.x * kWordsPerBlock + (uint64_t)wave * kWordsPerWave;
    uint32_t cnt = 0;
    for (int it = 0; it < kWordsPerWave; ++it) {
        const uint64_t w = w0 + it;
        if (w >= n_words) break;
        const uint32_t base = (uint32_t)(w * 64);  // total < 2^32 is checked by the caller
        const uint32_t flat = base + lane;
        bool ok = false;
        if (flat < total) {
            uint32_t r, s;
            if (g.S % 64 == 0) {
                // a wave never straddles two rays: ray index from wave-uniform values (scalar unit),
                // and the ray's six floats come through scalar loads
                r = (uint32_t)__builtin_amdgcn_readfirstlane((int)(base / (uint32_t)g.S));
                s = base - r * (uint32_t)g.S + lane;
            } else {
                r = flat / (uint32_t)g.S;
                s = flat - r * (uint32_t)g.S;
            }
            float ray[6];
            const float2 *rp = reinterpret_cast<const float2 *>(rays + 6 * (size_t)r);
            float2 a = rp[0], b = rp[1], c = rp[2];
            ray[0] = a.x; ray[1] = a.y; ray[2] = b.x; ray[3] = b.y; ray[4] = c.x; ray[5] = c.y;
            const float z = lm_sample_z(g, lm_ray_param(g, ray), (int)s);
            float pt[3];
            lm_point(ray, z, pt);
            ok = lm_sample_valid(g, pt);
            if (z_out) z_out[flat] = z;
        }
        const uint64_t bits = __ballot(ok);
        if (lane == 0) bitmap[w] = bits;
        cnt += (uint32_t)__popcll(bits);
    }
    if (lane == 0) s_cnt[wave] = cnt;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = 0;
        for (int i = 0; i < kBlock / LM_WAVE; ++i) t += s_cnt[i];
        block_count[blockIdx.x] = t;
    }
}

// Same decisions, one lane per (ray, bitmap word), for S = 64 * WPR with WPR in {1, 2, 4}.  A
// lane walks the 64 samples of its word and keeps the bits in a register; the 64 lanes of a
// wave are 64 neighbouring rays at the same depth, so their occupancy lookups fall into the
// same few cache lines (a wave of 64 samples along one ray touches 64 different ones), and the
// per-ray work (slab test or hull distance) is done once per word instead of once per sample.
// A workgroup covers 256 consecutive words = 4 of the 64-word groups k_scan_blocks counts.
// Bounds of the points of samples s0 .. s0 + n - 1 of one ray: they lie between the first and the last one (the depth
// tables are monotone, and so is o + d * z in z), widened by a margin a hundred times the rounding of the operations
// involved.  lo[k] <= pt[k] <= hi[k] for every sample of the run.  fminf / fmaxf drop NaNs; with FLAG_NAN a NaN anywhere
// on the way makes the bounds NaN (for the cell test, which must make no statement then; the box test needs no flag:
// what its bounds miss fails the per-sample test as well).
template <bool FLAG_NAN>
__device__ __forceinline__ void run_bounds(const lm_geom &g, const float *ray, float rp, int s0, int n, float *lo, float *hi) {
    const float za = lm_sample_z(g, rp, s0), zb = lm_sample_z(g, rp, s0 + n - 1);
    const float zlo = fminf(za, zb), zhi = fmaxf(za, zb);
    // the depth is a sum of two terms bounded by |near| and the ray's parameter (or by the depth itself)
    const float zm = 1e-5f * (fmaxf(fabsf(zlo), fabsf(zhi)) + fabsf(rp) + fabsf(g.near_));
    const bool z_nan = FLAG_NAN && (!(za == za) || !(zb == zb));
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        const float o = ray[k], d = ray[3 + k];
        const float e0 = d * (zlo - zm), e1 = d * (zhi + zm), e2 = d * (zlo + zm), e3 = d * (zhi - zm);
        const float l = o + fminf(fminf(e0, e1), fminf(e2, e3)), h = o + fmaxf(fmaxf(e0, e1), fmaxf(e2, e3));
        const float m = 1e-5f * (fabsf(o) + fmaxf(fabsf(l), fabsf(h))) + 1e-30f;
        const bool bad = FLAG_NAN && (z_nan || !(e0 == e0) || !(e1 == e1) || !(e2 == e2) || !(e3 == e3));
        lo[k] = bad ? NAN : l - m;
        hi[k] = bad ? NAN : h + m;
    }
}

// 1: every point within the bounds fails the box test (it stays on the outer side of one face).  Anything doubtful
// (NaN included) is 0.
__device__ __forceinline__ bool bounds_outside(const lm_geom &g, const float *lo, const float *hi) {
    bool outside = false;
#pragma unroll
    for (int k = 0; k < 3; ++k) outside |= (hi[k] < g.aabb[k]) | (lo[k] > g.aabb[3 + k]);
    return outside;
}

// The coarse level of a cell table (lm_pack_occupancy_coarse): blocks of 8 x 8 x 8 cells, entry b set when a cell of
// blocks b .. b + 1 (per axis) has a bit set.
constexpr int kCoarseShift = 3;
__host__ __device__ inline int coarse_dim(int cells) { return (cells + (1 << kCoarseShift) - 1) >> kCoarseShift; }

// Cell index range of the points within the bounds, per axis, with lm_cells_positive's own float operations: each of
// them is monotone (weakly, rounding included) in the coordinate when vol_inv > 0, so the floor of a point's cell
// coordinate lies between the floors of the bounds'.  Returns 0 when the bounds hold a NaN or the volume is degenerate
// (no statement), 1 with the block range [b0, b1] per axis otherwise; `none` = every index is outside the table
// (all samples are rejected by the lookup itself).
__device__ __forceinline__ bool coarse_range(const lm_geom &g, const float *lo, const float *hi, int *b0, int *b1, bool &none) {
    const int dims[3] = {g.vw, g.vh, g.vd};
    none = false;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        if (!(lo[k] <= hi[k]) || !(g.vol_inv[k] > 0.0f) || dims[k] < 2) return false;
        const float s = (float)(dims[k] - 1);
        float il = (((lo[k] - g.vol_aabb_min[k]) * g.vol_inv[k] - 1.0f) + 1.0f) / 2.0f * s;
        float ih = (((hi[k] - g.vol_aabb_min[k]) * g.vol_inv[k] - 1.0f) + 1.0f) / 2.0f * s;
        if (!(il <= ih)) return false;
        il = fminf(fmaxf(floorf(il), -2.0f), (float)dims[k]);
        ih = fminf(fmaxf(floorf(ih), -2.0f), (float)dims[k]);
        // cell index = floor + 1; indices outside 0 .. dims fail the lookup's range test
        int c0 = (int)il + 1, c1 = (int)ih + 1;
        if (c1 < 0 || c0 > dims[k]) none = true;
        c0 = max(c0, 0);
        c1 = min(c1, dims[k]);
        b0[k] = c0 >> kCoarseShift;
        b1[k] = c1 >> kCoarseShift;
    }
    return true;
}

// 1: no sample of the run can pass the cell lookup (every cell it can fall into is empty, or lies outside the table)
__device__ __forceinline__ bool coarse_empty(const lm_geom &g, const float *lo, const float *hi, int &span) {
    int b0[3], b1[3];
    bool none;
    span = INT_MAX;
    if (!coarse_range(g, lo, hi, b0, b1, none)) return false;
    if (none) return true;
    span = max(max(b1[0] - b0[0], b1[1] - b0[1]), b1[2] - b0[2]);
    if (span > 1) return false;
    const int nx = coarse_dim(g.vw + 1), ny = coarse_dim(g.vh + 1);
    return g.vol_coarse[((size_t)b0[2] * ny + b0[1]) * nx + b0[0]] == 0;
}

// Decisions of samples s0 .. s0 + n - 1 (n <= 64) of one ray, sample s0 + i in bit bit0 + i.
__device__ __forceinline__ uint64_t segment_bits(const lm_geom &g, const float *ray, float rp, int s0, int n, int bit0) {
    // A run whose bounds stay outside the box has no valid sample, and neither has one whose cells are all empty:
    // the bits are zero without visiting the samples.
    const bool cells0 = g.vol && g.vol_dtype == LM_CELLS && g.vol_thre == 0.0f;
    const bool coarse = cells0 && g.vol_coarse;
    bool pieces = false;
    {
        float lo[3], hi[3];
        if (coarse) run_bounds<true>(g, ray, rp, s0, n, lo, hi);
        else run_bounds<false>(g, ray, rp, s0, n, lo, hi);
        if (bounds_outside(g, lo, hi)) return 0ull;
        if (coarse) {
            int span;
            if (coarse_empty(g, lo, hi, span)) return 0ull;
            // quarters of the run have a chance when the whole run spans few blocks
            pieces = n >= 32 && span <= 6;
        }
    }
    uint64_t bits = 0;
    auto visit = [&](int i0, int i1) {
#pragma unroll 4
        for (int i = i0; i < i1; ++i) {
            const float z = lm_sample_z(g, rp, s0 + i);
            float pt[3];
            lm_point(ray, z, pt);
            bool ok;
            if (cells0) ok = lm_inside(g, pt) && lm_cells_positive(g, pt);
            else ok = lm_sample_valid(g, pt);
            bits |= (uint64_t)ok << (bit0 + i);
        }
    };
    if (!pieces) {
        visit(0, n);  // n is a constant for most callers: the loop unrolls without a remainder
    } else {
        const int step = (n + 3) / 4;
        for (int p0 = 0; p0 < n; p0 += step) {
            const int pn = min(step, n - p0);
            float lo[3], hi[3];
            int span;
            run_bounds<true>(g, ray, rp, s0 + p0, pn, lo, hi);
            if (bounds_outside(g, lo, hi) || coarse_empty(g, lo, hi, span)) continue;
            visit(p0, p0 + pn);
        }
    }
    return bits;
}

__device__ __forceinline__ void load_ray(const float *__restrict__ rays, uint64_t r, float *ray) {
    const float2 *rp2 = reinterpret_cast<const float2 *>(rays + 6 * (size_t)r);
    const float2 a = rp2[0], b = rp2[1], c = rp2[2];
    ray[0] = a.x; ray[1] = a.y; ray[2] = b.x; ray[3] = b.y; ray[4] = c.x; ray[5] = c.y;
}

// word j of ray r when S is a multiple of 64
__device__ __forceinline__ uint64_t word_of_ray(const lm_geom &g, const float *__restrict__ rays, uint64_t r, unsigned j) {
    float ray[6];
    load_ray(rays, r, ray);
    return segment_bits(g, ray, lm_ray_param(g, ray), (int)j * 64, 64, 0);
}

template <int WPR>
__global__ __launch_bounds__(kBlock) void k_sample_cull_rays(lm_geom g, const float *__restrict__ rays, uint32_t N,
                                                             uint64_t nb, uint64_t *__restrict__ bitmap,
                                                             uint32_t *__restrict__ block_count) {
    __shared__ uint32_t s_cnt[4];
    const unsigned lane = lm_lane(), wave = threadIdx.x / LM_WAVE;
    if (threadIdx.x < 4) s_cnt[threadIdx.x] = 0;
    __syncthreads();
    constexpr unsigned kRays = kBlock / WPR;  // rays per workgroup
    const unsigned j = wave % WPR;
    const unsigned ray_local = (wave / WPR) * 64 + lane;
    const uint64_t r = (uint64_t)blockIdx.x * kRays + ray_local;
    uint64_t bits = 0;
    if (r < N) {
        bits = word_of_ray(g, rays, r, j);
        bitmap[r * WPR + j] = bits;
    }
    const uint32_t cnt = (uint32_t)__popcll(bits);
    if (cnt) atomicAdd(&s_cnt[(ray_local * WPR + j) / 64], cnt);
    __syncthreads();
    if (threadIdx.x < 4) {
        const uint64_t bi = (uint64_t)blockIdx.x * 4 + threadIdx.x;
        if (bi < nb) block_count[bi] = s_cnt[threadIdx.x];
    }
}

// The same words for the whole-chunk render, which needs no global order of the valid samples:
// every ray gets a contiguous range of compact positions (p_first[r], wave prefix + one atomic on
// n_valid), rays with valid samples are appended to the marching queue's lists, the others get
// their zero results here.  Replaces the scan, the per-word prefix and the list of active rays.
template <int WPR>
__global__ __launch_bounds__(kBlock) void k_cull_rays_setup(lm_geom g, const float *__restrict__ rays, uint32_t N,
                                                            uint32_t row, uint64_t *__restrict__ bitmap, uint32_t *__restrict__ p_first,
                                                            uint32_t *__restrict__ ray_list, uint32_t *__restrict__ bins,
                                                            uint32_t *__restrict__ n_valid, float *__restrict__ acc,
                                                            float *__restrict__ depth, uint32_t *__restrict__ app_cnt,
                                                            uint32_t *__restrict__ p_end, uint32_t cap_valid,
                                                            uint32_t *__restrict__ overflow) {
    __shared__ uint32_t s_cnt[kBlock];
    const unsigned lane = lm_lane(), wave = threadIdx.x / LM_WAVE;
    constexpr unsigned kRays = kBlock / WPR;
    const unsigned j = wave % WPR;
    const unsigned ray_local = (wave / WPR) * 64 + lane;
    const uint64_t o = (uint64_t)blockIdx.x * kRays + ray_local;  // position in the visiting order
    const uint64_t r = o < N ? lm_ray_order((uint32_t)o, N, row) : o;
    uint64_t bits = 0;
    if (r < N) {
        bits = word_of_ray(g, rays, r, j);
        bitmap[r * WPR + j] = bits;
    }
    s_cnt[ray_local * WPR + j] = (uint32_t)__popcll(bits);
    __syncthreads();
    if (j != 0) return;  // whole waves leave: j is wave-uniform
    uint32_t cnt = 0;
#pragma unroll
    for (unsigned jj = 0; jj < (unsigned)WPR; ++jj) cnt += s_cnt[ray_local * WPR + jj];
    uint32_t incl = cnt;
#pragma unroll
    for (int d = 1; d < LM_WAVE; d <<= 1) {
        const uint32_t y = __shfl_up(incl, d);
        if (lane >= (unsigned)d) incl += y;
    }
    const uint32_t total = __shfl(incl, LM_WAVE - 1);
    uint32_t base = 0;
    if (total) {
        if (lane == 0) base = atomicAdd(n_valid, total);
        base = __shfl(base, 0);
    }
    const uint32_t first = base + incl - cnt;
    const bool any = lm_ray_fits(cnt, first, cap_valid, overflow);
    if (r < N) {
        p_first[r] = first;
        if (!any) { acc[r] = 0.0f; depth[r] = 0.0f; app_cnt[r] = 0; p_end[r] = first; }
    }
    lm_ray_enqueue(any && r < N, lm_ray_bin(cnt), (uint32_t)r, ray_list, N, bins);
}

// The same for long rays (three words and more): one lane per ray takes its words one after the other, so a
// word outside the box costs a few instructions and no wave waits at a barrier for a slower one
// (with one lane per word the workgroup lasts as long as its slowest word).  Rays reach the queue
// in a less regular order this way, which costs the march a little; with one or two words per ray
// the kernel above is the better trade.  When a chunk has too few rays to fill the GPU with one lane
// each, LPR neighbouring lanes share a ray and take every LPR-th word of it.
// SEG = 64: a lane's unit of work is a bitmap word; SEG = 16: a quarter of one (chunks with so few rays that even a
// lane per word leaves most of the GPU idle), the words are then put together with atomic ORs.
template <int LPR, int SEG>
__global__ __launch_bounds__(kBlock) void k_cull_rays_setup_serial(lm_geom g, const float *__restrict__ rays, uint32_t N,
                                                                   uint32_t row, uint64_t *__restrict__ bitmap,
                                                                   uint32_t *__restrict__ p_first,
                                                                   uint32_t *__restrict__ ray_list,
                                                                   uint32_t *__restrict__ bins,
                                                                   uint32_t *__restrict__ n_valid, float *__restrict__ acc,
                                                                   float *__restrict__ depth, uint32_t *__restrict__ app_cnt,
                                                                   uint32_t *__restrict__ p_end, uint32_t cap_valid,
                                                                   uint32_t *__restrict__ overflow,
                                                                   uint64_t *__restrict__ word_mask) {
    const unsigned lane = lm_lane();
    const unsigned sub = threadIdx.x % LPR;  // this lane's share of its ray's words
    const uint64_t o = ((uint64_t)blockIdx.x * kBlock + threadIdx.x) / LPR;  // position in the visiting order
    const uint64_t r = o < N ? lm_ray_order((uint32_t)o, N, row) : o;
    uint32_t cnt = 0;
    uint64_t words = 0;  // bit i: the ray has valid samples in its i-th bitmap word (rays of up to 64 words)
    if (r < N) {
        float ray[6];
        load_ray(rays, r, ray);
        const float rp = lm_ray_param(g, ray);
        // the ray's samples are bits [flat0, flat1) of the bitmap: whole words are stored, a first or last word
        // shared with a neighbouring ray is merged into the (zeroed) bitmap
        const uint64_t flat0 = r * (uint64_t)g.S, flat1 = flat0 + (uint64_t)g.S;
        for (uint64_t u = flat0 / SEG + sub; u * SEG < flat1; u += LPR) {
            const uint64_t w = u * SEG / 64;
            const uint64_t lo = u * SEG > flat0 ? u * SEG : flat0, hi = (u + 1) * SEG < flat1 ? (u + 1) * SEG : flat1;
            const uint64_t bits = segment_bits(g, ray, rp, (int)(lo - flat0), (int)(hi - lo), (int)(lo & 63));
            if (hi - lo == 64) bitmap[w] = bits;
            else if (bits) atomicOr(reinterpret_cast<unsigned long long *>(bitmap + w), (unsigned long long)bits);
            cnt += (uint32_t)__popcll(bits);
            if (bits) words |= 1ull << ((w - (flat0 >> 6)) & 63u);
        }
    }
    // the ray's count on all of its lanes; its first lane speaks for it from here on
#pragma unroll
    for (int d = 1; d < LPR; d <<= 1) {
        cnt += __shfl_xor(cnt, d);
        const uint32_t lo = __shfl_xor((uint32_t)words, d), hi = __shfl_xor((uint32_t)(words >> 32), d);
        words |= ((uint64_t)hi << 32) | lo;
    }
    uint32_t incl = sub == 0 ? cnt : 0;
#pragma unroll
    for (int d = 1; d < LM_WAVE; d <<= 1) {
        const uint32_t y = __shfl_up(incl, d);
        if (lane >= (unsigned)d) incl += y;
    }
    const uint32_t total = __shfl(incl, LM_WAVE - 1);
    uint32_t base = 0;
    if (total) {
        if (lane == 0) base = atomicAdd(n_valid, total);
        base = __shfl(base, 0);
    }
    const bool mine = r < N && sub == 0;
    const uint32_t first = base + incl - cnt;
    const bool any = lm_ray_fits(mine ? cnt : 0u, first, cap_valid, overflow);
    if (mine) {
        p_first[r] = first;
        // a ray of more than 64 words cannot be described: all ones = "walk every word"
        word_mask[r] = (((r + 1) * (uint64_t)g.S - 1) >> 6) - ((r * (uint64_t)g.S) >> 6) < 64 ? words : ~0ull;
        if (!any) { acc[r] = 0.0f; depth[r] = 0.0f; app_cnt[r] = 0; p_end[r] = first; }
    }
    lm_ray_enqueue(any && mine, lm_ray_bin(cnt), (uint32_t)r, ray_list, N, bins);
}

// words of the bitmap that two rays share must start at zero (sample counts that are not multiples of 64)
__global__ __launch_bounds__(kBlock) void k_zero_words(uint64_t *__restrict__ p, uint64_t n) {
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (uint64_t)gridDim.x * kBlock) p[i] = 0ull;
}

// exclusive scan of n counts by one workgroup of 1024 threads; total -> *total_out
__global__ __launch_bounds__(1024) void k_scan_blocks(const uint32_t *__restrict__ in, uint32_t *__restrict__ out,
                                                      uint32_t n, uint32_t *__restrict__ total_out) {
    __shared__ uint32_t s_wave[16];
    __shared__ uint32_t s_carry;
    const unsigned lane = lm_lane(), wave = threadIdx.x / LM_WAVE;
    if (threadIdx.x == 0) s_carry = 0;
    __syncthreads();
    for (uint32_t base = 0; base < n; base += 1024) {
        const uint32_t i = base + threadIdx.x;
        const uint32_t v = i < n ? in[i] : 0;
        uint32_t x = v;  // inclusive wave scan
#pragma unroll
        for (int d = 1; d < LM_WAVE; d <<= 1) {
            uint32_t y = __shfl_up(x, d);
            if (lane >= (unsigned)d) x += y;
        }
        if (lane == LM_WAVE - 1) s_wave[wave] = x;
        __syncthreads();
        uint32_t off = s_carry;
        for (unsigned k = 0; k < wave; ++k) off += s_wave[k];
        if (i < n) out[i] = off + x - v;
        __syncthreads();
        if (threadIdx.x == 1023) s_carry = off + x;
        __syncthreads();
    }
    if (threadIdx.x == 0) *total_out = s_carry;
}

__global__ __launch_bounds__(kBlock) void k_emit(const uint64_t *__restrict__ bitmap, uint64_t n_words,
                                                 const uint32_t *__restrict__ block_off,
                                                 uint32_t *__restrict__ word_prefix, uint32_t *__restrict__ valid_idx) {
    __shared__ uint32_t s_pref[kWordsPerBlock];
    const unsigned lane = lm_lane(), wave = threadIdx.x / LM_WAVE;
    const uint64_t wb = (uint64_t)blockIdx.x * kWordsPerBlock;
    if (wave == 0) {
        const uint64_t w = wb + lane;
        const uint32_t v = w < n_words ? (uint32_t)__popcll(bitmap[w]) : 0;
        uint32_t x = v;
#pragma unroll
        for (int d = 1; d < LM_WAVE; d <<= 1) {
            uint32_t y = __shfl_up(x, d);
            if (lane >= (unsigned)d) x += y;
        }
        const uint32_t p = block_off[blockIdx.x] + x - v;
        s_pref[lane] = p;
        if (w < n_words) word_prefix[w] = p;
    }
    __syncthreads();
    for (int it = 0; it < kWordsPerWave; ++it) {
        const unsigned wi = wave * kWordsPerWave + it;
        const uint64_t w = wb + wi;
        if (w >= n_words) break;
        const uint64_t bits = bitmap[w];
        if (valid_idx && ((bits >> lane) & 1ull)) valid_idx[s_pref[wi] + lm_mbcnt(bits)] = (uint32_t)(w * 64 + lane);
    }
}

// coarse level, step 1: any[b] = some cell of block b has a bit set
__global__ __launch_bounds__(256) void k_coarse_any(const uint8_t *__restrict__ cells, int D1, int H1, int W1, uint8_t *__restrict__ any) {
    const int nx = coarse_dim(W1), ny = coarse_dim(H1), nz = coarse_dim(D1);
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)nx * ny * nz) return;
    const int bx = (int)(i % nx), by = (int)((i / nx) % ny), bz = (int)(i / ((size_t)nx * ny));
    unsigned acc = 0;
    for (int z = bz << kCoarseShift; z < min((bz + 1) << kCoarseShift, D1); ++z)
        for (int y = by << kCoarseShift; y < min((by + 1) << kCoarseShift, H1); ++y)
            for (int x = bx << kCoarseShift; x < min((bx + 1) << kCoarseShift, W1); ++x) acc |= cells[((size_t)z * H1 + y) * W1 + x];
    any[i] = acc ? 1 : 0;
}
// step 2: coarse[b] = any over blocks b .. b + 1 along every axis
__global__ __launch_bounds__(256) void k_coarse_dilate(const uint8_t *__restrict__ any, int nz, int ny, int nx, uint8_t *__restrict__ coarse) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)nx * ny * nz) return;
    const int bx = (int)(i % nx), by = (int)((i / nx) % ny), bz = (int)(i / ((size_t)nx * ny));
    unsigned acc = 0;
    for (int z = bz; z < min(bz + 2, nz); ++z)
        for (int y = by; y < min(by + 2, ny); ++y)
            for (int x = bx; x < min(bx + 2, nx); ++x) acc |= any[((size_t)z * ny + y) * nx + x];
    coarse[i] = acc ? 1 : 0;
}

__global__ __launch_bounds__(256) void k_pack_occupancy(const float *__restrict__ vol, int D, int H, int W,
                                                        uint8_t *__restrict__ cells, uint32_t *__restrict__ not_binary) {
    const size_t n = (size_t)(D + 1) * (H + 1) * (W + 1);
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int cx = (int)(i % (W + 1)), cy = (int)((i / (W + 1)) % (H + 1)), cz = (int)(i / ((size_t)(W + 1) * (H + 1)));
    unsigned bits = 0;
    bool bad = false;
    for (int k = 0; k < 8; ++k) {
        const int x = cx - 1 + (k & 1), y = cy - 1 + ((k >> 1) & 1), z = cz - 1 + (k >> 2);
        if (x >= 0 && x < W && y >= 0 && y < H && z >= 0 && z < D) {
            const float v = vol[((size_t)z * H + y) * W + x];
            if (v == 1.0f) bits |= 1u << k;
            else if (v != 0.0f) bad = true;
        }
    }
    cells[i] = (uint8_t)bits;
    if (bad) *not_binary = 1u;  // plain store of the same value from every lane that sees one
}

// updateAlphaMask's pooling step: out[z][y][x] = 1 if the largest clamp(alpha, 0, 1) over the
// 3 x 3 x 3 neighbourhood (cut at the borders) is >= thres, else 0; alpha is [gx][gy][gz].
// box = {min x, y, z, max x, y, z} over the voxels set, count = their number.
__global__ __launch_bounds__(256) void k_alpha_mask_pool(const float *__restrict__ alpha, int gx, int gy, int gz,
                                                         float thres, float *__restrict__ out, int *__restrict__ box,
                                                         unsigned long long *__restrict__ count) {
    const size_t n = (size_t)gx * gy * gz;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    bool set = false;
    int x = 0, y = 0, z = 0;
    if (i < n) {
        x = (int)(i % gx); y = (int)((i / gx) % gy); z = (int)(i / ((size_t)gx * gy));
        float m = -INFINITY;
        for (int dx = -1; dx <= 1; ++dx)
            for (int dy = -1; dy <= 1; ++dy)
                for (int dz = -1; dz <= 1; ++dz) {
                    const int xx = x + dx, yy = y + dy, zz = z + dz;
                    if (xx < 0 || xx >= gx || yy < 0 || yy >= gy || zz < 0 || zz >= gz) continue;
                    float a = alpha[((size_t)xx * gy + yy) * gz + zz];
                    a = fminf(fmaxf(a, 0.0f), 1.0f);
                    m = fmaxf(m, a);
                }
        set = m >= thres;
        out[i] = set ? 1.0f : 0.0f;
    }
    const uint64_t mask = __ballot(set);
    if (mask == 0) return;
    int lo[3] = {set ? x : INT_MAX, set ? y : INT_MAX, set ? z : INT_MAX};
    int hi[3] = {set ? x : -1, set ? y : -1, set ? z : -1};
    for (int off = 32; off > 0; off >>= 1)
#pragma unroll
        for (int d = 0; d < 3; ++d) {
            lo[d] = min(lo[d], __shfl_xor(lo[d], off));
            hi[d] = max(hi[d], __shfl_xor(hi[d], off));
        }
    if (lm_lane() == 0) {
#pragma unroll
        for (int d = 0; d < 3; ++d) {
            atomicMin(box + d, lo[d]);
            atomicMax(box + 3 + d, hi[d]);
        }
        atomicAdd(count, (unsigned long long)__popcll(mask));
    }
}

__global__ void k_alpha_mask_init(int *box, unsigned long long *count) {
    if (threadIdx.x < 3) box[threadIdx.x] = INT_MAX;
    else if (threadIdx.x < 6) box[threadIdx.x] = -1;
    else if (threadIdx.x == 6) *count = 0ull;
}

}  // namespace

static uint64_t n_blocks_for(uint64_t n_words) { return (n_words + kWordsPerBlock - 1) / kWordsPerBlock; }

extern "C" size_t lm_sample_cull_scratch_bytes(int64_t N, int32_t S) {
    if (N <= 0 || S <= 0) return 0;
    const uint64_t n_words = ((uint64_t)N * (uint64_t)S + 63) / 64;
    return (size_t)(n_blocks_for(n_words) * 2 * sizeof(uint32_t) + 256);
}

int lm_check_geom(const lm_geom *g) {
    LM_REQUIRE(g != nullptr, "geom is null");
    LM_REQUIRE(g->S > 0, "S must be positive (got %d)", g->S);
    LM_REQUIRE(g->sampler == LM_SAMPLER_AABB || g->sampler == LM_SAMPLER_HULL, "unknown sampler %d", g->sampler);
    LM_REQUIRE(g->tab_a && g->tab_t, "sampler tables are null");
    if (g->vol) {
        LM_REQUIRE(g->vd > 0 && g->vh > 0 && g->vw > 0, "occupancy volume has an empty dimension");
        LM_REQUIRE(g->vol_dtype == LM_F32 || g->vol_dtype == LM_U8 || g->vol_dtype == LM_CELLS,
                   "occupancy volume dtype %d", g->vol_dtype);
    }
    if (g->div0 != 0 || g->div1 != 0) {
        LM_REQUIRE(g->div0 > 0 && g->div1 > 0 && (int64_t)g->div0 * g->div1 <= 65536, "plane division %d x %d", g->div0,
                   g->div1);
        // One block: the reference maps block b to the coordinate 2 b / (div0 div1 - 1) - 1 = 0 / 0
        // (app/models/gridnerf_parallel.py:333-335) and renders NaN; there is nothing to reproduce.
        if ((int64_t)g->div0 * g->div1 == 1)
            LM_FAIL(LM_ERR_UNSUPPORTED, "plane division 1 x 1: a single block is the plain (unstacked) layout, set div0 = 0");
        LM_REQUIRE(g->blk_w > 0.0f && g->blk_h > 0.0f, "block size must be positive");
    }
    return LM_OK;
}

extern "C" int lm_sample_cull(const lm_geom *geom, const float *rays, int64_t N, uint64_t *bitmap,
                              uint32_t *word_prefix, uint32_t *valid_idx, uint32_t *counters, float *z_out,
                              void *scratch, void *stream) {
    if (int rc = lm_check_geom(geom)) return rc;
    LM_REQUIRE(N >= 0, "negative ray count");
    LM_REQUIRE(counters != nullptr, "counters is null");
    hipStream_t st = (hipStream_t)stream;
    const uint64_t total = (uint64_t)N * (uint64_t)geom->S;
    LM_REQUIRE(total < (1ull << 32), "N*S = %llu does not fit 32-bit sample indices; split the chunk",
               (unsigned long long)total);
    if (N == 0) {
        // an empty chunk is valid (the reference's chunk loop never issues one, but a caller may)
        hipLaunchKernelGGL(k_scan_blocks, dim3(1), dim3(1024), 0, st, (const uint32_t *)nullptr, (uint32_t *)nullptr, 0u,
                           counters + LM_STAT_N_VALID);
        LM_CHECK_LAUNCH("k_scan_blocks");
        return LM_OK;
    }
    LM_REQUIRE(rays && bitmap && word_prefix && scratch, "null buffer");
    LM_REQUIRE((reinterpret_cast<uintptr_t>(rays) & 7u) == 0, "rays must be 8-byte aligned");
    LM_REQUIRE(lm_aligned16(bitmap) && lm_aligned16(scratch), "bitmap and scratch must be 16-byte aligned");
    const uint64_t n_words = (total + 63) / 64;
    const uint64_t nb = n_blocks_for(n_words);
    uint32_t *block_count = (uint32_t *)scratch;
    uint32_t *block_off = block_count + nb;
    const int wpr = geom->S % 64 == 0 ? geom->S / 64 : 0;
    if (!z_out && (wpr == 1 || wpr == 2 || wpr == 4)) {
        const unsigned groups = (unsigned)((n_words + 255) / 256);
#define LM_CULL_RAYS(W_)                                                                                              \
    hipLaunchKernelGGL(k_sample_cull_rays<W_>, dim3(groups), dim3(kBlock), 0, st, *geom, rays, (uint32_t)N, nb, bitmap, \
                       block_count)
        if (wpr == 1) LM_CULL_RAYS(1);
        else if (wpr == 2) LM_CULL_RAYS(2);
        else LM_CULL_RAYS(4);
#undef LM_CULL_RAYS
        LM_CHECK_LAUNCH("k_sample_cull_rays");
    } else {
        hipLaunchKernelGGL(k_sample_cull, dim3((unsigned)nb), dim3(kBlock), 0, st, *geom, rays, total, n_words, bitmap,
                           block_count, z_out);
        LM_CHECK_LAUNCH("k_sample_cull");
    }
    hipLaunchKernelGGL(k_scan_blocks, dim3(1), dim3(1024), 0, st, (const uint32_t *)block_count, block_off,
                       (uint32_t)nb, counters + LM_STAT_N_VALID);
    LM_CHECK_LAUNCH("k_scan_blocks");
    hipLaunchKernelGGL(k_emit, dim3((unsigned)nb), dim3(kBlock), 0, st, (const uint64_t *)bitmap, n_words,
                       (const uint32_t *)block_off, word_prefix, valid_idx);
    LM_CHECK_LAUNCH("k_emit");
    return LM_OK;
}

extern "C" int lm_pack_occupancy(const float *vol, int32_t D, int32_t H, int32_t W, uint8_t *cells, uint32_t *not_binary,
                                 void *stream) {
    LM_REQUIRE(vol && cells && not_binary, "null buffer");
    LM_REQUIRE(D > 0 && H > 0 && W > 0, "empty volume");
    const size_t n = (size_t)(D + 1) * (H + 1) * (W + 1);
    LM_REQUIRE(n < ((size_t)1 << 39), "volume too large");
    hipLaunchKernelGGL(k_pack_occupancy, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, vol, D, H, W,
                       cells, not_binary);
    LM_CHECK_LAUNCH("k_pack_occupancy");
    return LM_OK;
}

// The coarse table and, behind it, the undilated one it is made from (scratch of the build): 2 n bytes.
extern "C" size_t lm_occupancy_coarse_bytes(int32_t D, int32_t H, int32_t W) {
    if (D <= 0 || H <= 0 || W <= 0) return 0;
    return 2 * (size_t)coarse_dim(D + 1) * coarse_dim(H + 1) * coarse_dim(W + 1);
}

extern "C" int lm_pack_occupancy_coarse(const uint8_t *cells, int32_t D, int32_t H, int32_t W, uint8_t *coarse, void *stream) {
    LM_REQUIRE(cells && coarse, "null buffer");
    LM_REQUIRE(D > 0 && H > 0 && W > 0, "empty volume");
    const int nz = coarse_dim(D + 1), ny = coarse_dim(H + 1), nx = coarse_dim(W + 1);
    const size_t n = (size_t)nx * ny * nz;
    uint8_t *any = coarse + n;
    hipLaunchKernelGGL(k_coarse_any, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, cells, D + 1, H + 1, W + 1, any);
    hipLaunchKernelGGL(k_coarse_dilate, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, any, nz, ny, nx, coarse);
    LM_CHECK_LAUNCH("k_coarse_dilate");
    return LM_OK;
}

extern "C" int lm_alpha_mask_pool(const float *alpha, int32_t gx, int32_t gy, int32_t gz, float thres, float *volume,
                                  int32_t *box, uint64_t *count, void *stream) {
    LM_REQUIRE(alpha && volume && box && count, "null buffer");
    LM_REQUIRE(gx > 0 && gy > 0 && gz > 0, "empty lattice %d x %d x %d", gx, gy, gz);
    const size_t n = (size_t)gx * gy * gz;
    LM_REQUIRE(n < ((size_t)1 << 39), "lattice too large");
    hipLaunchKernelGGL(k_alpha_mask_init, dim3(1), dim3(64), 0, (hipStream_t)stream, box,
                       reinterpret_cast<unsigned long long *>(count));
    hipLaunchKernelGGL(k_alpha_mask_pool, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, alpha, gx,
                       gy, gz, thres, volume, box, reinterpret_cast<unsigned long long *>(count));
    LM_CHECK_LAUNCH("k_alpha_mask_pool");
    return LM_OK;
}

// Cull + per-ray set-up for the whole-chunk render: one launch (plus a fill of the bitmap when the sample
// count is not a multiple of 64).
int lm_launch_cull_setup(const lm_geom *geom, const float *rays, int64_t N, uint64_t *bitmap, uint32_t *p_first,
                         uint32_t *ray_list, uint32_t *bins, uint32_t *n_valid, float *acc, float *depth,
                         uint32_t *app_cnt, uint32_t *p_end, uint32_t row, uint32_t cap_valid, uint32_t *overflow,
                         uint64_t *word_mask, hipStream_t st) {
    const int wpr = geom->S % 64 == 0 ? geom->S / 64 : 0;
    LM_REQUIRE((reinterpret_cast<uintptr_t>(rays) & 7u) == 0, "rays must be 8-byte aligned");
#define LM_CULL_SETUP(W_)                                                                                             \
    hipLaunchKernelGGL(k_cull_rays_setup<W_>, dim3((unsigned)(((uint64_t)N * W_ + kBlock - 1) / kBlock)), dim3(kBlock), 0, st, \
                       *geom, rays, (uint32_t)N, row, bitmap, p_first, ray_list, bins, n_valid, acc, depth, app_cnt, p_end,  \
                       cap_valid, overflow)
    // a lane per (ray, word) for 64 and 128 samples, unless the chunk has so few rays that a lane per quarter word
    // is needed to occupy the GPU
    const bool few = (uint64_t)N * (wpr > 0 ? wpr : 1) * 8 <= (uint64_t)lm_persistent_blocks(2) * kBlock;
    if (wpr == 1 && !few) {
        LM_CULL_SETUP(1);
    } else if (wpr == 2 && !few) {
        LM_CULL_SETUP(2);
    } else {
        // one lane per ray when the chunk fills the GPU that way, otherwise 2 .. 16 lanes per ray, which share its
        // words, or quarters of its words when there are fewer words than lanes
        const uint64_t fill = (uint64_t)lm_persistent_blocks(2) * kBlock;
        const int words = (geom->S + 63) / 64;
        int lpr = 1;
        while (lpr < 16 && 2 * lpr <= words && (uint64_t)N * lpr < fill) lpr *= 2;
        const bool quarters = (uint64_t)N * lpr * 2 <= fill && 2 * lpr > words && lpr < 16;
        if (quarters)
            while (lpr < 16 && 2 * lpr <= 4 * words && (uint64_t)N * lpr < fill) lpr *= 2;
        if (wpr == 0 || quarters) {
            const uint64_t n_words = ((uint64_t)N * (uint64_t)geom->S + 63) / 64;
            const unsigned blocks = (unsigned)std::min<uint64_t>((n_words + kBlock - 1) / kBlock, 4096);
            hipLaunchKernelGGL(k_zero_words, dim3(blocks), dim3(kBlock), 0, st, bitmap, n_words);
        }
#define LM_CULL_SERIAL(L_)                                                                                           \
    if (quarters)                                                                                                    \
        hipLaunchKernelGGL((k_cull_rays_setup_serial<L_, 16>), dim3((unsigned)(((uint64_t)N * L_ + kBlock - 1) / kBlock)), \
                           dim3(kBlock), 0, st, *geom, rays, (uint32_t)N, row, bitmap, p_first, ray_list, bins, n_valid,  \
                           acc, depth, app_cnt, p_end, cap_valid, overflow, word_mask);                                 \
    else                                                                                                             \
    hipLaunchKernelGGL((k_cull_rays_setup_serial<L_, 64>), dim3((unsigned)(((uint64_t)N * L_ + kBlock - 1) / kBlock)),     \
                       dim3(kBlock), 0, st, *geom, rays, (uint32_t)N, row, bitmap, p_first, ray_list, bins, n_valid, acc, \
                       depth, app_cnt, p_end, cap_valid, overflow, word_mask)
        switch (lpr) {
            case 1: LM_CULL_SERIAL(1); break;
            case 2: LM_CULL_SERIAL(2); break;
            case 4: LM_CULL_SERIAL(4); break;
            case 8: LM_CULL_SERIAL(8); break;
            default: LM_CULL_SERIAL(16); break;
        }
#undef LM_CULL_SERIAL
    }
#undef LM_CULL_SETUP
    LM_CHECK_LAUNCH("k_cull_rays_setup");
    return LM_OK;
}
