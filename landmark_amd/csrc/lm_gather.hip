// Part 2: bilinear plane x linear line feature gather over channel-last tables.
//
// Four lanes share one sample.  Lane q of the quad owns channels [V*q, V*q+V) of every
// group of 4V channels (V = 4 floats or 8 halves = one 16-byte load), so the quad reads
// 64 contiguous bytes per load instruction and a corner of a 16-channel fp32 plane is one
// such read.  All planes of all resolution levels are walked inside one launch; the
// per-plane partial sums stay in registers.  Work is a grid-stride loop over tiles of 64
// samples so the launch shape does not depend on counts that only exist on the device.
//
// Interpolation follows F.grid_sample(align_corners=True, zeros padding) as the reference
// calls it (app/models/gridnerf_sequential.py:803-812, 851-862): unnormalise
// ((c+1)/2)*(size-1), corners floor/floor+1, out-of-range corners contribute zero.
#include <hip/hip_fp16.h>

#include <algorithm>
#include <type_traits>

#include "lm_common.h"
#include "lm_mma.h"

#ifndef LM_MARCH_NS
#define LM_MARCH_NS 4
#endif
// chunks of up to this many rays march with a wave per ray (too few rays to fill the GPU with a quad each)
#ifndef LM_WAVE_MARCH_RAYS
#define LM_WAVE_MARCH_RAYS 12288
#endif

namespace {

constexpr int kBlock = 256;
constexpr int kQuad = 4;
constexpr int kTile = kBlock / kQuad;  // samples per workgroup iteration
constexpr uint32_t kWaveMarchRays = LM_WAVE_MARCH_RAYS;

struct PlaneSet {
    lm_plane p[LM_MAX_PLANES];
    int n;
    int nblk;  // > 0: block-stacked tables, planes [nblk][H][W][C], lines [Len][nblk][C]
};

// A lane's share of one texel: loaded as it is stored (fetch), converted to float where it is
// used (unpack), so that loads in flight hold the stored width in registers and no conversion
// waits for a load that other work could run under.
template <typename T> struct Vec;
template <> struct Vec<float> {
    using elem = float;
    using raw = float4;
    static constexpr int V = 4;
    __device__ static __forceinline__ raw fetch(const float *p) { return *reinterpret_cast<const float4 *>(p); }
    __device__ static __forceinline__ void unpack(const raw &v, float *o) { o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w; }
};
template <> struct Vec<__half> {
    using elem = __half;
    using raw = uint4;
    static constexpr int V = 8;
    __device__ static __forceinline__ raw fetch(const __half *p) { return *reinterpret_cast<const uint4 *>(p); }
    __device__ static __forceinline__ void unpack(const raw &v, float *o) {
        const __half2 *h = reinterpret_cast<const __half2 *>(&v);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float2 f = __half22float2(h[i]);
            o[2 * i] = f.x; o[2 * i + 1] = f.y;
        }
    }
};
// fp16 tables read four channels (8 bytes) per lane: for 16- and 48-channel planes, where
// 16-byte loads would leave half of a quad idle on the last 16 channels
struct Half4 {};
template <> struct Vec<Half4> {
    using elem = __half;
    using raw = uint2;
    static constexpr int V = 4;
    __device__ static __forceinline__ raw fetch(const __half *p) { return *reinterpret_cast<const uint2 *>(p); }
    __device__ static __forceinline__ void unpack(const raw &v, float *o) {
        const __half2 *h = reinterpret_cast<const __half2 *>(&v);
        const float2 a = __half22float2(h[0]), b = __half22float2(h[1]);
        o[0] = a.x; o[1] = a.y; o[2] = b.x; o[3] = b.y;
    }
};

// fp16 planes of 48 channels (96-byte texels) in the fused appearance gather: six channels (12 bytes) per lane, two load
// instructions per texel and quad instead of three.  The kernel keeps its texture addresser busy 82 % of the time at a
// cost per instruction that depends on the lines touched, not on the bytes (4K city block: 26.7 -> 24.5 ms per frame).
struct Half6 {};
struct __attribute__((aligned(4))) Raw12 {
    uint32_t x, y, z;
};
template <> struct Vec<Half6> {
    using elem = __half;
    using raw = Raw12;
    static constexpr int V = 6;
    __device__ static __forceinline__ raw fetch(const __half *p) { return *reinterpret_cast<const Raw12 *>(p); }
    __device__ static __forceinline__ void unpack(const raw &v, float *o) {
        const __half2 *h = reinterpret_cast<const __half2 *>(&v);
        const float2 a = __half22float2(h[0]), b = __half22float2(h[1]), c = __half22float2(h[2]);
        o[0] = a.x; o[1] = a.y; o[2] = b.x; o[3] = b.y; o[4] = c.x; o[5] = c.y;
    }
};

struct Taps2 {  // bilinear footprint: element offsets of the 4 corners and their weights
    int64_t o00, o01, o10, o11;
    float w00, w01, w10, w11;
};
struct Taps1 {
    int o0, o1;
    float w0, w1;
};

__device__ __forceinline__ float unnorm(float c, int size) { return ((c + 1.0f) / 2.0f) * (float)(size - 1); }

// Corner (y, x) outside the table has weight zero (grid_sample's zeros padding) and is read from
// the nearest texel inside.  A row of the table has fewer than 2^31 elements (checked on the host).
__device__ __forceinline__ Taps2 plane_taps(const lm_plane &pl, float cx, float cy) {
    const float ix = unnorm(cx, pl.W), iy = unnorm(cy, pl.H);
    const float fx = floorf(ix), fy = floorf(iy);
    float wx1 = ix - fx, wx0 = (fx + 1.0f) - ix, wy1 = iy - fy, wy0 = (fy + 1.0f) - iy;
    // clamp in float first: coordinates far outside the table must not overflow the int cast
    const int x0 = (int)fminf(fmaxf(fx, -2.0f), (float)pl.W), y0 = (int)fminf(fmaxf(fy, -2.0f), (float)pl.H);
    const int x1 = x0 + 1, y1 = y0 + 1;
    if ((unsigned)x0 >= (unsigned)pl.W) wx0 = 0.0f;
    if ((unsigned)x1 >= (unsigned)pl.W) wx1 = 0.0f;
    if ((unsigned)y0 >= (unsigned)pl.H) wy0 = 0.0f;
    if ((unsigned)y1 >= (unsigned)pl.H) wy1 = 0.0f;
    const int x0c = min(max(x0, 0), pl.W - 1), x1c = min(max(x1, 0), pl.W - 1);
    const int y0c = min(max(y0, 0), pl.H - 1), y1c = min(max(y1, 0), pl.H - 1);
    const int row = pl.W * pl.C;
    Taps2 t;
    const int dx = x1c != x0c ? pl.C : 0, dy = y1c != y0c ? row : 0;
    t.o00 = (int64_t)y0c * row + x0c * pl.C;
    t.o01 = t.o00 + dx;
    t.o10 = t.o00 + dy;
    t.o11 = t.o10 + dx;
    t.w00 = wx0 * wy0; t.w01 = wx1 * wy0; t.w10 = wx0 * wy1; t.w11 = wx1 * wy1;
    return t;
}

__device__ __forceinline__ Taps1 line_taps(const lm_plane &pl, float c) {
    const float i = unnorm(c, pl.Len);
    const float f = floorf(i);
    float w1 = i - f, w0 = (f + 1.0f) - i;
    int i0 = (int)fminf(fmaxf(f, -2.0f), (float)pl.Len), i1 = i0 + 1;
    if (i0 < 0 || i0 >= pl.Len) w0 = 0.0f;
    if (i1 < 0 || i1 >= pl.Len) w1 = 0.0f;
    i0 = min(max(i0, 0), pl.Len - 1); i1 = min(max(i1, 0), pl.Len - 1);
    Taps1 t;
    t.o0 = i0 * pl.C; t.o1 = i1 * pl.C;
    t.w0 = w0; t.w1 = w1;
    return t;
}

// Queries are float[4]: normalised x, y, z and, for block-stacked tables, the block index as
// integer bits in q[3].  Moves the taps to the block; a block outside the table reads as zero.
__device__ __forceinline__ void block_taps(const lm_plane &pl, int nblk, const float *q, Taps2 &t2, Taps1 &t1) {
    if (nblk <= 0) return;
    const int blk = __float_as_int(q[3]);
    if (blk < 0 || blk >= nblk) {
        t2.w00 = t2.w01 = t2.w10 = t2.w11 = 0.0f;
        t1.w0 = t1.w1 = 0.0f;
        return;
    }
    const int64_t base = (int64_t)blk * pl.H * pl.W * pl.C;
    t2.o00 += base; t2.o01 += base; t2.o10 += base; t2.o11 += base;
    t1.o0 = t1.o0 * nblk + blk * pl.C;
    t1.o1 = t1.o1 * nblk + blk * pl.C;
}

// Sum over the four lanes of a quad, on all four (DPP moves: partner 1 away, then 2 away).
__device__ __forceinline__ float quad_sum(float v) {
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xb1, 0xf, 0xf, false));
    v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4e, 0xf, 0xf, false));
    return v;
}

__device__ __forceinline__ float pick(const float *q, int ax) { return ax == 0 ? q[0] : (ax == 1 ? q[1] : q[2]); }

// products of one plane for the V channels starting at c (lane-private)
template <typename T>
__device__ __forceinline__ void plane_products(const lm_plane &pl, const Taps2 &t2, const Taps1 &t1, int c, float *prod) {
    constexpr int V = Vec<T>::V;
    using E = typename Vec<T>::elem;
    const E *P = reinterpret_cast<const E *>(pl.plane);
    const E *Ln = reinterpret_cast<const E *>(pl.line);
    float a[V], b[V], cc[V], d[V], l0[V], l1[V];
    const typename Vec<T>::raw ra = Vec<T>::fetch(P + t2.o00 + c), rb = Vec<T>::fetch(P + t2.o01 + c),
                               rc = Vec<T>::fetch(P + t2.o10 + c), rd = Vec<T>::fetch(P + t2.o11 + c),
                               r0 = Vec<T>::fetch(Ln + t1.o0 + c), r1 = Vec<T>::fetch(Ln + t1.o1 + c);
    Vec<T>::unpack(ra, a); Vec<T>::unpack(rb, b); Vec<T>::unpack(rc, cc); Vec<T>::unpack(rd, d);
    Vec<T>::unpack(r0, l0); Vec<T>::unpack(r1, l1);
#pragma unroll
    for (int i = 0; i < V; ++i) {
        float pv = a[i] * t2.w00;
        pv = fmaf(b[i], t2.w01, pv);
        pv = fmaf(cc[i], t2.w10, pv);
        pv = fmaf(d[i], t2.w11, pv);
        float lv = fmaf(l1[i], t1.w1, l0[i] * t1.w0);
        prod[i] = pv * lv;
    }
}

// den_w == NULL: plain sum over planes and channels.  Otherwise the reference's
// nonlinear_density: relu(sum of den_w[plane*C + channel] * product) (gridnerf_sequential.py:819-822)
template <typename T>
__device__ __forceinline__ float density_sum(const PlaneSet &ps, const float *q, unsigned qlane,
                                             const float *__restrict__ den_w) {
    constexpr int V = Vec<T>::V;
    float sum = 0.0f;
    int col = 0;
    for (int k = 0; k < ps.n; ++k) {
        const lm_plane pl = ps.p[k];
        Taps2 t2 = plane_taps(pl, pick(q, pl.ax0), pick(q, pl.ax1));
        Taps1 t1 = line_taps(pl, pick(q, pl.axl));
        block_taps(pl, ps.nblk, q, t2, t1);
        for (int c = V * qlane; c < pl.C; c += V * kQuad) {
            float prod[V];
            plane_products<T>(pl, t2, t1, c, prod);
            if (den_w) {
#pragma unroll
                for (int i = 0; i < V; ++i) sum = fmaf(den_w[col + c + i], prod[i], sum);
            } else {
#pragma unroll
                for (int i = 0; i < V; ++i) sum += prod[i];
            }
        }
        col += pl.C;
    }
    sum = quad_sum(sum);
    return den_w ? fmaxf(sum, 0.0f) : sum;
}

// The loads of plane_products and the arithmetic on what they return, as two steps, for callers
// that want several footprints' loads in flight before the first use.
template <typename T> struct Footprint {
    typename Vec<T>::raw a, b, c, d, l0, l1;
};
template <typename T>
__device__ __forceinline__ void footprint_load(const lm_plane &pl, const Taps2 &t2, const Taps1 &t1, int c, Footprint<T> &f) {
    using E = typename Vec<T>::elem;
    const E *P = reinterpret_cast<const E *>(pl.plane);
    const E *Ln = reinterpret_cast<const E *>(pl.line);
    f.a = Vec<T>::fetch(P + t2.o00 + c);
    f.b = Vec<T>::fetch(P + t2.o01 + c);
    f.c = Vec<T>::fetch(P + t2.o10 + c);
    f.d = Vec<T>::fetch(P + t2.o11 + c);
    f.l0 = Vec<T>::fetch(Ln + t1.o0 + c);
    f.l1 = Vec<T>::fetch(Ln + t1.o1 + c);
}
template <typename T>
__device__ __forceinline__ void footprint_products(const Footprint<T> &f, const Taps2 &t2, const Taps1 &t1, float *prod) {
    constexpr int V = Vec<T>::V;
    float a[V], b[V], c[V], d[V], l0[V], l1[V];
    Vec<T>::unpack(f.a, a); Vec<T>::unpack(f.b, b); Vec<T>::unpack(f.c, c); Vec<T>::unpack(f.d, d);
    Vec<T>::unpack(f.l0, l0); Vec<T>::unpack(f.l1, l1);
#pragma unroll
    for (int i = 0; i < V; ++i) {
        float pv = a[i] * t2.w00;
        pv = fmaf(b[i], t2.w01, pv);
        pv = fmaf(c[i], t2.w10, pv);
        pv = fmaf(d[i], t2.w11, pv);
        const float lv = fmaf(l1[i], t1.w1, l0[i] * t1.w0);
        prod[i] = pv * lv;
    }
}

// Value of v on lane n of this lane's quad (n is a constant after unrolling): one DPP move.
__device__ __forceinline__ int quad_lane(int v, int n) {
    switch (n & 3) {
        case 0: return __builtin_amdgcn_update_dpp(0, v, 0x00, 0xf, 0xf, false);
        case 1: return __builtin_amdgcn_update_dpp(0, v, 0x55, 0xf, 0xf, false);
        case 2: return __builtin_amdgcn_update_dpp(0, v, 0xaa, 0xf, 0xf, false);
        default: return __builtin_amdgcn_update_dpp(0, v, 0xff, 0xf, 0xf, false);
    }
}
__device__ __forceinline__ float quad_lane(float v, int n) { return __int_as_float(quad_lane(__float_as_int(v), n)); }
__device__ __forceinline__ int64_t quad_lane(int64_t v, int n) {
    const uint32_t lo = (uint32_t)quad_lane((int)(uint32_t)v, n), hi = (uint32_t)quad_lane((int)(uint32_t)((uint64_t)v >> 32), n);
    return (int64_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ Taps2 quad_lane(const Taps2 &t, int n) {
    Taps2 r;
    // the corners are less than 2^31 elements apart: one 64-bit offset and two 32-bit steps go round
    const int dx = quad_lane((int)(t.o01 - t.o00), n), dy = quad_lane((int)(t.o10 - t.o00), n);
    r.o00 = quad_lane(t.o00, n);
    r.o01 = r.o00 + dx;
    r.o10 = r.o00 + dy;
    r.o11 = r.o10 + dx;
    r.w00 = quad_lane(t.w00, n); r.w01 = quad_lane(t.w01, n); r.w10 = quad_lane(t.w10, n); r.w11 = quad_lane(t.w11, n);
    return r;
}
__device__ __forceinline__ Taps1 quad_lane(const Taps1 &t, int n) {
    Taps1 r;
    r.o0 = quad_lane(t.o0, n); r.o1 = quad_lane(t.o1, n); r.w0 = quad_lane(t.w0, n); r.w1 = quad_lane(t.w1, n);
    return r;
}

// NS samples of a quad at once (the marching kernel's look-ahead).  Lane n of the quad brings
// the coordinates of sample n (lanes NS.. repeat) and works out that sample's footprints, one
// sample per lane instead of every sample on every lane; the footprints then go round the quad
// and each lane loads its quarter of the channels of all NS samples, every load issued before
// the first use, so a ray's chain of dependent memory round trips is NS times shorter.  Same
// operations per sample as density_sum, hence the same bits.  out[n] is valid on all four lanes.
template <typename T, int NS>
__device__ __forceinline__ void density_sum_n(const PlaneSet &ps, const float *q_mine, unsigned qlane,
                                              const float *__restrict__ den_w, float *out) {
    constexpr int V = Vec<T>::V;
    float sum[NS];
#pragma unroll
    for (int n = 0; n < NS; ++n) sum[n] = 0.0f;
    int col = 0;
    for (int k = 0; k < ps.n; ++k) {
        const lm_plane pl = ps.p[k];
        Taps2 m2 = plane_taps(pl, pick(q_mine, pl.ax0), pick(q_mine, pl.ax1));
        Taps1 m1 = line_taps(pl, pick(q_mine, pl.axl));
        block_taps(pl, ps.nblk, q_mine, m2, m1);
        Taps2 t2[NS];
        Taps1 t1[NS];
#pragma unroll
        for (int n = 0; n < NS; ++n) {
            t2[n] = quad_lane(m2, n);
            t1[n] = quad_lane(m1, n);
        }
        for (int c = V * qlane; c < pl.C; c += V * kQuad) {
            Footprint<T> f[NS];
#pragma unroll
            for (int n = 0; n < NS; ++n) footprint_load<T>(pl, t2[n], t1[n], c, f[n]);
            // keep the 6 * NS loads ahead of the first use
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int n = 0; n < NS; ++n) {
                float prod[V];
                footprint_products<T>(f[n], t2[n], t1[n], prod);
                if (den_w) {
#pragma unroll
                    for (int i = 0; i < V; ++i) sum[n] = fmaf(den_w[col + c + i], prod[i], sum[n]);
                } else {
#pragma unroll
                    for (int i = 0; i < V; ++i) sum[n] += prod[i];
                }
            }
        }
        col += pl.C;
    }
#pragma unroll
    for (int n = 0; n < NS; ++n) {
        float v = sum[n];
        v = quad_sum(v);
        out[n] = den_w ? fmaxf(v, 0.0f) : v;
    }
}

// Same sum with a compile-time channel count shared by all planes: the channel groups of a
// plane are unrolled, so a lane has 6 * C / (4 V) independent loads in flight per plane
// instead of 6 (wide planes, e.g. the 64-channel isolated-gather configuration).
template <typename T, int C>
__device__ __forceinline__ float density_sum_fixed(const PlaneSet &ps, const float *q, unsigned qlane,
                                                   const float *__restrict__ den_w) {
    constexpr int V = Vec<T>::V;
    constexpr int NG = (C + V * kQuad - 1) / (V * kQuad);
    float sum = 0.0f;
    for (int k = 0; k < ps.n; ++k) {
        const lm_plane pl = ps.p[k];
        Taps2 t2 = plane_taps(pl, pick(q, pl.ax0), pick(q, pl.ax1));
        Taps1 t1 = line_taps(pl, pick(q, pl.axl));
        block_taps(pl, ps.nblk, q, t2, t1);
        float prod[NG][V];
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            const int c = V * (int)qlane + gi * V * kQuad;
            plane_products<T>(pl, t2, t1, c < C ? c : C - V, prod[gi]);
        }
#pragma unroll
        for (int gi = 0; gi < NG; ++gi) {
            const int c = V * (int)qlane + gi * V * kQuad;
            if (c < C) {
#pragma unroll
                for (int i = 0; i < V; ++i) sum = den_w ? fmaf(den_w[k * C + c + i], prod[gi][i], sum) : sum + prod[gi][i];
            }
        }
    }
    sum = quad_sum(sum);
    return den_w ? fmaxf(sum, 0.0f) : sum;
}

// Plane x line products of the sixteen samples of a wave (four lanes each), written in whole lines: a quad's own stores
// are 64-byte pieces of sixteen different rows per instruction, which reach the memory as partial lines (measured on
// 2^24 random queries of 3 x 64 channels: 16.3 GB written and 86.8 GB read for 12.9 GB of products and 51.5 GB of texels).
// Each plane's products go through a tile in LDS (sixteen rows of C + 4 floats per wave) and leave as runs of C floats
// per sample, a lane storing 16 bytes of a run.  Samples p0 .. p0 + 15 belong to the wave; those at or beyond M are
// computed (from a clamped query) and not stored.  Planes of more than kStageC channels take the direct form.
constexpr int kStageC = 64;
constexpr int kStageRow = kStageC + 4;
template <typename T>
__device__ __forceinline__ void app_store_wave(const PlaneSet &ps, const float *q, uint64_t p0, uint64_t M, int K,
                                               float *__restrict__ out, float *tile) {
    constexpr int V = Vec<T>::V;
    const unsigned lane = lm_lane(), qlane = lane & 3u, qs = lane >> 2;
    int col = 0;
    for (int k = 0; k < ps.n; ++k) {
        const lm_plane pl = ps.p[k];
        Taps2 t2 = plane_taps(pl, pick(q, pl.ax0), pick(q, pl.ax1));
        Taps1 t1 = line_taps(pl, pick(q, pl.axl));
        block_taps(pl, ps.nblk, q, t2, t1);
        const bool staged = pl.C <= kStageC;
        if (staged) {
            // every load of the plane's footprint is issued before the first use: one memory round trip per plane
            constexpr int NG = kStageC / (V * kQuad);
            Footprint<T> fp[NG];
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                const int c = V * (int)qlane + gi * V * kQuad;
                if (c < pl.C) footprint_load<T>(pl, t2, t1, c, fp[gi]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                const int c = V * (int)qlane + gi * V * kQuad;
                if (c >= pl.C) continue;
                float prod[V];
                footprint_products<T>(fp[gi], t2, t1, prod);
#pragma unroll
                for (int i = 0; i < V; i += 4)
                    *reinterpret_cast<float4 *>(tile + qs * kStageRow + c + i) = make_float4(prod[i], prod[i + 1], prod[i + 2], prod[i + 3]);
            }
        } else {
            for (int c = V * qlane; c < pl.C; c += V * kQuad) {
                float prod[V];
                plane_products<T>(pl, t2, t1, c, prod);
#pragma unroll
                for (int i = 0; i < V; i += 4)
                    if (p0 + qs < M)
                        *reinterpret_cast<float4 *>(out + (p0 + qs) * (uint64_t)K + col + c + i) =
                            make_float4(prod[i], prod[i + 1], prod[i + 2], prod[i + 3]);
            }
        }
        if (staged) {
            // LDS operations of one wave complete in order; the fences only pin the compiler
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            const unsigned c4 = (unsigned)pl.C / 4u;  // 16-byte pieces per sample
            for (unsigned idx = lane; idx < 16u * c4; idx += LM_WAVE) {
                const unsigned s_i = idx / c4, f = idx - s_i * c4;
                if (p0 + s_i < M)
                    *reinterpret_cast<float4 *>(out + (p0 + s_i) * (uint64_t)K + col + 4 * f) =
                        *reinterpret_cast<const float4 *>(tile + s_i * kStageRow + 4 * f);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        col += pl.C;
    }
}

// coordinates of list entry `flat` (= ray*S + s): same operations as the sampler
__device__ __forceinline__ void list_coords(const lm_geom &g, const float *__restrict__ rays, uint32_t flat, float *q) {
    const uint32_t r = flat / (uint32_t)g.S;
    const int s = (int)(flat - r * (uint32_t)g.S);
    float ray[6];
    const float2 *rp = reinterpret_cast<const float2 *>(rays + 6 * (size_t)r);
    float2 a = rp[0], b = rp[1], c = rp[2];
    ray[0] = a.x; ray[1] = a.y; ray[2] = b.x; ray[3] = b.y; ray[4] = c.x; ray[5] = c.y;
    const float z = lm_sample_z(g, lm_ray_param(g, ray), s);
    float pt[3];
    lm_point(ray, z, pt);
    lm_normalise(g, pt, q);
    q[3] = __int_as_float(g.div0 > 0 ? lm_block_coords(g, q) : 0);
}

__device__ __forceinline__ float activate(float f, int act, float shift) {
    if (act == LM_ACT_SOFTPLUS) {
        const float x = f + shift;
        return x > 20.0f ? x : log1pf(expf(x));
    }
    return fmaxf(f, 0.0f);
}

// ---- explicit coordinates ----------------------------------------------------------------
template <typename T, int CFIX>  // CFIX > 0: every plane has CFIX channels
__global__ __launch_bounds__(kBlock) void k_density_xyz(PlaneSet ps, const float *__restrict__ den_w,
                                                        const float *__restrict__ xyz, uint64_t M,
                                                        float *__restrict__ out) {
    const unsigned qlane = threadIdx.x & 3u, slot = threadIdx.x >> 2;
    const uint64_t n_tiles = (M + kTile - 1) / kTile;
    for (uint64_t tile = lm_xcd_swizzle(blockIdx.x, gridDim.x); tile < n_tiles; tile += gridDim.x) {
        const uint64_t p = tile * kTile + slot;
        if (p >= M) continue;
        float q[4] = {xyz[3 * p], xyz[3 * p + 1], xyz[3 * p + 2], 0.0f};
        const float s = CFIX > 0 ? density_sum_fixed<T, (CFIX > 0 ? CFIX : 16)>(ps, q, qlane, den_w)
                                 : density_sum<T>(ps, q, qlane, den_w);
        if (qlane == 0) out[p] = s;
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_app_xyz(PlaneSet ps, int K, const float *__restrict__ xyz, uint64_t M,
                                                    float *__restrict__ out) {
    __shared__ __align__(16) float s_tile[kBlock / LM_WAVE][16 * kStageRow];
    const unsigned slot = threadIdx.x >> 2, wave = threadIdx.x / LM_WAVE;
    const uint64_t n_tiles = (M + kTile - 1) / kTile;
    for (uint64_t tile = lm_xcd_swizzle(blockIdx.x, gridDim.x); tile < n_tiles; tile += gridDim.x) {
        const uint64_t p0 = tile * kTile + wave * 16;  // whole waves stay or leave
        if (p0 >= M) continue;
        const uint64_t p = tile * kTile + slot, pc = p < M ? p : M - 1;
        float q[4] = {xyz[3 * pc], xyz[3 * pc + 1], xyz[3 * pc + 2], 0.0f};
        app_store_wave<T>(ps, q, p0, M, K, out, s_tile[wave]);
    }
}

// ---- alpha on a lattice over the AABB (getDenseAlpha / compute_alpha) ------------------------
// Point (i, j, k) = aabb0 * (1 - s) + aabb1 * s with s from three host tables, every product and
// sum rounded on its own like the reference's tensor expression.  A point the existing occupancy
// volume does not see (lookup not > 0) keeps sigma 0.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_dense_alpha(lm_geom g, PlaneSet ps, const float *__restrict__ den_w,
                                                        const float *__restrict__ lin_x,
                                                        const float *__restrict__ lin_y,
                                                        const float *__restrict__ lin_z, int gx, int gy, int gz,
                                                        int act, float shift, float length, float *__restrict__ alpha) {
    const unsigned qlane = threadIdx.x & 3u, slot = threadIdx.x >> 2;
    const uint64_t M = (uint64_t)gx * gy * gz;
    const uint64_t n_tiles = (M + kTile - 1) / kTile;
    for (uint64_t tile = lm_xcd_swizzle(blockIdx.x, gridDim.x); tile < n_tiles; tile += gridDim.x) {
        const uint64_t p = tile * kTile + slot;
        if (p >= M) continue;
        const int k = (int)(p % (uint64_t)gz), j = (int)((p / (uint64_t)gz) % (uint64_t)gy);
        const int i = (int)(p / ((uint64_t)gz * gy));
        const float s[3] = {lin_x[i], lin_y[j], lin_z[k]};
        float pt[3], q[4];
        q[3] = 0.0f;
#pragma unroll
        for (int d = 0; d < 3; ++d) {
            const float a = g.aabb[d] * (1.0f - s[d]);
            const float b = g.aabb[3 + d] * s[d];
            pt[d] = a + b;
        }
        float sigma = 0.0f;
        if (!g.vol || lm_alpha_lookup(g, pt) > 0.0f) {
            lm_normalise(g, pt, q);
            sigma = activate(density_sum<T>(ps, q, qlane, den_w), act, shift);
        }
        if (qlane == 0) alpha[p] = 1.0f - expf((-sigma) * length);
    }
}

// ---- list driven (inside the render) -------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void k_density_list(lm_geom g, PlaneSet ps, const float *__restrict__ den_w,
                                                         const float *__restrict__ rays,
                                                         const uint32_t *__restrict__ list,
                                                         const uint32_t *__restrict__ count, int act, float shift,
                                                         float *__restrict__ sigma) {
    const unsigned qlane = threadIdx.x & 3u, slot = threadIdx.x >> 2;
    const uint64_t M = *count;
    const uint64_t n_tiles = (M + kTile - 1) / kTile;
    for (uint64_t tile = lm_xcd_swizzle(blockIdx.x, gridDim.x); tile < n_tiles; tile += gridDim.x) {
        const uint64_t p = tile * kTile + slot;
        if (p >= M) continue;
        float q[4];
        list_coords(g, rays, list[p], q);
        const float s = density_sum<T>(ps, q, qlane, den_w);
        if (qlane == 0) sigma[p] = activate(s, act, shift);
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void k_app_list(lm_geom g, PlaneSet ps, int K, const float *__restrict__ rays,
                                                     const uint32_t *__restrict__ list,
                                                     const uint32_t *__restrict__ count, uint32_t cap,
                                                     float *__restrict__ out) {
    __shared__ __align__(16) float s_tile[kBlock / LM_WAVE][16 * kStageRow];
    const unsigned slot = threadIdx.x >> 2, wave = threadIdx.x / LM_WAVE;
    const uint64_t M = min(*count, cap);  // the counter keeps counting past the list's capacity
    const uint64_t n_tiles = (M + kTile - 1) / kTile;
    for (uint64_t tile = lm_xcd_swizzle(blockIdx.x, gridDim.x); tile < n_tiles; tile += gridDim.x) {
        const uint64_t p0 = tile * kTile + wave * 16;  // whole waves stay or leave
        if (p0 >= M) continue;
        const uint64_t p = tile * kTile + slot;
        float q[4];
        list_coords(g, rays, list[p < M ? p : M - 1], q);
        app_store_wave<T>(ps, q, p0, M, K, out, s_tile[wave]);
    }
}


// ---- density gather fused with the transmittance march ------------------------------------
// Four lanes (a quad) own one ray at a time and walk its valid samples in order: gather the
// density of the next sample (each lane a quarter of the channels), turn it into alpha and a
// weight, carry the transmittance along.  Quads take rays from a queue of the rays that have
// valid samples and fetch a new one as soon as theirs ends, so the sixteen quads of a wave
// stay busy whatever the rays' lengths.  Two things follow from walking rays in lock step:
// neighbouring rays are at similar depths in the same load instruction, so their corner
// texels share cache lines; and a ray can stop once its transmittance is below term_eps,
// before the density of the samples behind is ever fetched.  With term_eps = 0 the weights
// are those of the separate density + weights kernels, bit for bit (same operations, and the
// transmittance is the same sequential product torch.cumprod forms, app/tools/utils.py:51-64).
template <typename T, int NS>  // NS samples of a ray per round
__global__ __launch_bounds__(kBlock) void k_march(lm_geom g, PlaneSet ps, const float *__restrict__ den_w,
                                                  const float *__restrict__ rays, const uint64_t *__restrict__ bitmap,
                                                  const uint32_t *__restrict__ p_first,
                                                  const uint64_t *__restrict__ word_mask,
                                                  const uint32_t *__restrict__ ray_list,
                                                  const uint32_t *__restrict__ bins, uint32_t n_rays,
                                                  uint32_t *__restrict__ queue,
                                                  int act, float shift, float distance_scale, float weight_thres,
                                                  float term_eps, float *__restrict__ w_valid,
                                                  float *__restrict__ acc_out, float *__restrict__ depth_out,
                                                  uint32_t *__restrict__ app_cnt, uint32_t *__restrict__ p_end_out,
                                                  uint32_t *__restrict__ n_marched) {
    const unsigned lane = lm_lane(), qlane = lane & 3u, leader = lane & ~3u;
    // One cursor per XCD (workgroups go to the XCDs round robin): an XCD takes every n_queues-th
    // granule of consecutive queue entries, so rays that are neighbours on screen march on the
    // same XCD at the same time and meet in its L2.  Granules of 1024 rays when there are many,
    // smaller ones for short queues so that every XCD still gets its share.
    const uint32_t n_queues = gridDim.x < (unsigned)LM_XCDS ? gridDim.x : (unsigned)LM_XCDS;
    const uint32_t my_q = blockIdx.x % n_queues;
    uint32_t *my_queue = queue + my_q;
    uint32_t marched = 0;  // samples whose density this lane's quad gathered (statistics)
    // cumulative sizes of the four ray lists (long rays first)
    const uint32_t end0 = bins[0], end1 = end0 + bins[1], end2 = end1 + bins[2], n_active = end2 + bins[3];
    const int log_n = 31 - __clz((int)(n_active | 1u));
    const uint32_t granule_shift = (uint32_t)(log_n >= 16 ? 10 : log_n >= 10 ? log_n - 6 : 4);
    const int S = g.S;
    bool have = false, done = false;
    uint32_t r = 0, p = 0, cnt = 0;
    uint64_t flat0 = 0;
    float ray[6] = {0, 0, 0, 0, 0, 0}, rp = 0.0f, Tr = 1.0f, acc = 0.0f, depth = 0.0f;
    BitWalk it;
    it.bits = 0; it.w = it.w0 = it.w_last = 0; it.flat1 = 0; it.pos = 0; it.bitmap = bitmap; it.prefix = nullptr;
    it.todo = it.ahead = 0; it.masked = false;
    while (true) {
        // quads without a ray take the next ones from the queue: one atomic per wave and round
        const bool need = !have && !done;
        const uint64_t need_mask = __ballot(need && qlane == 0);
        if (need_mask) {
            const int first = __ffsll((unsigned long long)need_mask) - 1;
            uint32_t base = 0;
            if ((int)lane == first) base = atomicAdd(my_queue, (uint32_t)__popcll(need_mask));
            base = __shfl(base, first);
            if (need) {
                const uint32_t local = base + (uint32_t)__popcll(need_mask & ((1ull << leader) - 1ull));
                const uint32_t idx = ((((local >> granule_shift) * n_queues + my_q)) << granule_shift) + (local & ((1u << granule_shift) - 1u));
                if (idx >= n_active) {
                    done = true;
                } else {
                    r = idx < end0   ? ray_list[idx]
                        : idx < end1 ? ray_list[(size_t)n_rays + (idx - end0)]
                        : idx < end2 ? ray_list[2 * (size_t)n_rays + (idx - end1)]
                                     : ray_list[3 * (size_t)n_rays + (idx - end2)];
                    const float2 *rp2 = reinterpret_cast<const float2 *>(rays + 6 * (size_t)r);
                    const float2 a = rp2[0], b = rp2[1], c = rp2[2];
                    ray[0] = a.x; ray[1] = a.y; ray[2] = b.x; ray[3] = b.y; ray[4] = c.x; ray[5] = c.y;
                    rp = lm_ray_param(g, ray);
                    flat0 = (uint64_t)r * (uint64_t)S;
                    it.start_at(bitmap, flat0, flat0 + S, p_first[r], word_mask ? word_mask[r] : ~0ull);
                    p = it.pos;
                    Tr = 1.0f; acc = 0.0f; depth = 0.0f; cnt = 0;
                    have = true;
                }
            }
        }
        if (!__any(have)) break;
        if (have) {
            // up to NS samples per round: their densities are gathered together, the weights follow in order
            uint64_t flat[NS];
            int n_have = 0;
#pragma unroll
            for (int n = 0; n < NS; ++n) {
                flat[n] = n ? flat[n - 1] : 0;
                if (n_have == n && it.next(flat[n])) n_have = n + 1;
            }
            bool finish = n_have == 0;
            if (!finish) {
                // lane n of the quad prepares sample n: coordinates, footprints, and after the
                // gather its alpha (missing samples repeat the first; their results are unused)
                const int mine = (int)(qlane & (unsigned)(NS - 1));
                uint64_t flat_m = flat[0];
#pragma unroll
                for (int n = 1; n < NS; ++n)
                    if (mine == n && n < n_have) flat_m = flat[n];
                const int s_m = (int)(flat_m - flat0);
                const float z_m = lm_sample_z(g, rp, s_m);
                float q_m[4], f[NS];
                {
                    float pt[3];
                    lm_point(ray, z_m, pt);
                    lm_normalise(g, pt, q_m);
                    q_m[3] = __int_as_float(g.div0 > 0 ? lm_block_coords(g, q_m) : 0);
                }
                density_sum_n<T, NS>(ps, q_m, qlane, den_w, f);
                marched += (uint32_t)n_have;
                float f_m = f[0];
#pragma unroll
                for (int n = 1; n < NS; ++n)
                    if (mine == n) f_m = f[n];
                const float sig = activate(f_m, act, shift);
                const float dist = (s_m + 1 < S) ? lm_sample_z(g, rp, s_m + 1) - z_m : 0.0f;
                const float d2 = dist * distance_scale;
                const float alpha_m = 1.0f - expf(-sig * d2);
                float alpha_n[NS], z_n[NS];
#pragma unroll
                for (int n = 0; n < NS; ++n) {
                    alpha_n[n] = quad_lane(alpha_m, n);
                    z_n[n] = quad_lane(z_m, n);
                }
#pragma unroll
                for (int n = 0; n < NS; ++n) {
                    if (n >= n_have || finish) break;
                    const float alpha = alpha_n[n];
                    const float wgt = alpha * Tr;
                    Tr = Tr * ((1.0f - alpha) + 1e-10f);
                    if (qlane == 0) w_valid[p] = wgt;
                    acc += wgt;
                    depth += wgt * z_n[n];
                    cnt += wgt > weight_thres;
                    ++p;
                    finish = term_eps > 0.0f && Tr < term_eps;
                }
                if (n_have < NS) finish = true;  // the ray's last samples
            }
            if (finish) {
                if (qlane == 0) {
                    acc_out[r] = acc; depth_out[r] = depth; app_cnt[r] = cnt; p_end_out[r] = p;
                }
                have = false;
            }
        }
    }
    if (qlane != 0) marched = 0;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) marched += __shfl_xor(marched, d);
    if (lane == 0 && marched) atomicAdd(n_marched, marched);
}

// ---- the same march with a whole wave per ray ------------------------------------------------
// For chunks with too few rays to fill the GPU with one quad each (a caller that keeps the reference's chunks
// of a few thousand rays), and for their long rays: a launch of the kernel above lasts as long as the longest
// chain of dependent gathers, four samples per round.  Here a wave owns a ray and takes one 64-sample word of
// its bitmap per round: lane j prepares sample j of the word, quad i gathers samples 4i .. 4i+3 (the same
// density_sum_n, quads without a valid sample sit the round out), so a round's 64 densities come back in one
// memory round trip.  The transmittance then runs through the word's valid samples in order, every lane
// computing the same scalars from values read off the owning lanes: the same operations in the same order as
// the quad march, hence the same bits (weights, sums, counts, the sample at which a ray stops), whichever of
// the two kernels a chunk's size selects.
template <typename T>
__global__ __launch_bounds__(kBlock) void k_march_wave(lm_geom g, PlaneSet ps, const float *__restrict__ den_w,
                                                       const float *__restrict__ rays, const uint64_t *__restrict__ bitmap,
                                                       const uint32_t *__restrict__ p_first,
                                                       const uint64_t *__restrict__ word_mask,
                                                       const uint32_t *__restrict__ ray_list,
                                                       const uint32_t *__restrict__ bins, uint32_t n_rays, int act,
                                                       float shift, float distance_scale, float weight_thres, float term_eps,
                                                       float *__restrict__ w_valid, float *__restrict__ acc_out,
                                                       float *__restrict__ depth_out, uint32_t *__restrict__ app_cnt,
                                                       uint32_t *__restrict__ p_end_out, uint32_t *__restrict__ n_marched) {
    const unsigned lane = lm_lane(), qlane = lane & 3u;
    const uint32_t end0 = bins[0], end1 = end0 + bins[1], end2 = end1 + bins[2], n_active = end2 + bins[3];
    const uint32_t n_waves = gridDim.x * (kBlock / LM_WAVE);
    const int S = g.S;
    uint32_t marched = 0;
    // everything that steers a wave is the same on all of its lanes: kept in scalar registers
    auto uniform = [](uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
    auto uniform64 = [&](uint64_t v) { return ((uint64_t)uniform((uint32_t)(v >> 32)) << 32) | uniform((uint32_t)v); };
    for (uint32_t idx = uniform(blockIdx.x * (kBlock / LM_WAVE) + threadIdx.x / LM_WAVE); idx < n_active; idx += n_waves) {
        const uint32_t r = idx < end0   ? ray_list[idx]
                           : idx < end1 ? ray_list[(size_t)n_rays + (idx - end0)]
                           : idx < end2 ? ray_list[2 * (size_t)n_rays + (idx - end1)]
                                        : ray_list[3 * (size_t)n_rays + (idx - end2)];
        float ray[6];
        {
            const float2 *rp2 = reinterpret_cast<const float2 *>(rays + 6 * (size_t)r);
            const float2 a = rp2[0], b = rp2[1], c = rp2[2];
            ray[0] = a.x; ray[1] = a.y; ray[2] = b.x; ray[3] = b.y; ray[4] = c.x; ray[5] = c.y;
        }
        const float rp = lm_ray_param(g, ray);
        const uint64_t flat0 = (uint64_t)r * (uint64_t)S, flat1 = flat0 + (uint64_t)S;
        const uint64_t w0 = flat0 >> 6, w_last = (flat1 - 1) >> 6;
        uint64_t todo = word_mask ? uniform64(word_mask[r]) : ~0ull;  // the ray's non-empty words; all ones: every word
        const bool masked = todo != ~0ull && w_last - w0 < 64;
        uint32_t p = uniform(p_first[r]), cnt = 0;
        float Tr = 1.0f, acc = 0.0f, depth = 0.0f;
        bool finish = false;
        for (uint64_t w = w0; !finish;) {
            if (masked) {
                if (todo == 0) break;
                w = w0 + (uint64_t)(__ffsll((unsigned long long)todo) - 1);
                todo &= todo - 1;
            } else if (w > w_last) {
                break;
            }
            uint64_t bits = uniform64(bitmap[w]);
            if (w == w0 && (flat0 & 63)) bits &= ~((1ull << (flat0 & 63)) - 1ull);  // a neighbouring ray's samples share the word
            if (w == w_last && (flat1 & 63)) bits &= (1ull << (flat1 & 63)) - 1ull;
            if (bits) {
                // lane j prepares sample j of the word; samples that are not valid get the coordinates of the word's
                // first valid one (in range for the tables, results unused)
                const bool mine = (bits >> lane) & 1ull;
                const int j_m = mine ? (int)lane : __ffsll((unsigned long long)bits) - 1;
                const int s_m = (int)(w * 64 + (uint64_t)j_m - flat0);
                const float z_m = lm_sample_z(g, rp, s_m);
                float alpha_m = 0.0f;
                if ((bits >> (lane & ~3u)) & 0xFull) {  // the quad has a valid sample
                    float q_m[4], f[4];
                    {
                        float pt[3];
                        lm_point(ray, z_m, pt);
                        lm_normalise(g, pt, q_m);
                        q_m[3] = __int_as_float(g.div0 > 0 ? lm_block_coords(g, q_m) : 0);
                    }
                    density_sum_n<T, 4>(ps, q_m, qlane, den_w, f);
                    float f_m = f[0];
#pragma unroll
                    for (int n = 1; n < 4; ++n)
                        if ((int)qlane == n) f_m = f[n];
                    const float sig = activate(f_m, act, shift);
                    const float dist = (s_m + 1 < S) ? lm_sample_z(g, rp, s_m + 1) - z_m : 0.0f;
                    const float d2 = dist * distance_scale;
                    alpha_m = 1.0f - expf(-sig * d2);
                }
                marched += (uint32_t)__popcll(bits);
                // the word's valid samples in order; every lane carries the same transmittance and sums
                float w_mine = 0.0f;
                uint32_t done = 0;
                for (uint64_t rem = bits; rem;) {
                    const int j = __ffsll((unsigned long long)rem) - 1;
                    rem &= rem - 1;
                    const float alpha = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(alpha_m), j));
                    const float z = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(z_m), j));
                    const float wgt = alpha * Tr;
                    Tr = Tr * ((1.0f - alpha) + 1e-10f);
                    if ((int)lane == j) w_mine = wgt;
                    acc += wgt;
                    depth += wgt * z;
                    cnt += wgt > weight_thres;
                    ++done;
                    if (term_eps > 0.0f && Tr < term_eps) { finish = true; break; }
                }
                const uint32_t rank = lm_mbcnt(bits);
                if (mine && rank < done) w_valid[p + rank] = w_mine;
                p += done;
            }
            ++w;
        }
        if (lane == 0) {
            acc_out[r] = acc; depth_out[r] = depth; app_cnt[r] = cnt; p_end_out[r] = p;
        }
    }
    if (lane == 0 && marched) atomicAdd(n_marched, marched);
}

// ---- appearance gather fused with basis_mat --------------------------------------------------
// One wave owns 32 appearance samples; lane (j, h) gathers, for sample j, CW consecutive
// channels of every group of 2*CW (the lane pair of a sample covers the group), multiplies
// plane by line and feeds the products straight into the matrix cores as the B operand of
// basis_mat (A = the packed basis fragments, resident in LDS).  The [n, P*L*C] product
// matrix never exists in memory; the kernel writes the 27 projected features per sample.
template <int PREC> struct AppFeatBlock { static constexpr int N = 512; };

// LDS: [basis fragments | one product tile per wave].  A tile is 32 samples x (C + 4) floats.
__host__ __device__ inline size_t app_feat_tile_bytes(int C) { return (size_t)32 * (C + 4) * sizeof(float); }

template <int PREC, typename T, int NU>  // NU = groups of 16 channels per plane (C = 16 * NU)
__global__ __launch_bounds__(AppFeatBlock<PREC>::N) void k_app_feat(lm_geom g, PlaneSet ps, int K,
                                                                   const char *__restrict__ packed, lm_mma::PackLayout L,
                                                                   const float *__restrict__ rays,
                                                                   const uint32_t *__restrict__ list,
                                                                   const uint32_t *__restrict__ count, uint32_t cap,
                                                                   float *__restrict__ feat) {
    using namespace lm_mma;
    using Mm = Mma<PREC>;
    using frag = typename Mm::frag;
    constexpr int NP = Mm::NP;
    constexpr int V = Vec<T>::V;
    constexpr int C = 16 * NU, ROW = C + 4;
    constexpr int NG = (C + V * kQuad - 1) / (V * kQuad);  // 16-byte loads per lane, corner and plane
    constexpr int G = Mm::G, CW = Mm::CW;
    extern __shared__ __align__(16) char lds[];
    const size_t basis_bytes = (size_t)32 * K * sizeof(typename Mm::elem) * NP;  // K MFMA K-slots x 32 rows
    {
        const uint4 *src = reinterpret_cast<const uint4 *>(packed + L.basis);
        uint4 *dst = reinterpret_cast<uint4 *>(lds);
        for (size_t i = threadIdx.x; i < basis_bytes / 16; i += blockDim.x) dst[i] = src[i];
        __syncthreads();
    }
    const frag *A = reinterpret_cast<const frag *>(lds);
    const unsigned lane = lm_lane(), j = lane & 31u, h = lane >> 5;
    const unsigned qlane = lane & 3u, gs = lane >> 2;  // gather role: 4 lanes per sample, 16 samples per pass
    float *tile = reinterpret_cast<float *>(lds + basis_bytes + (threadIdx.x / LM_WAVE) * app_feat_tile_bytes(C));
    const uint64_t M = min(*count, cap);  // the counter keeps counting past the list's capacity
    const uint64_t n_tiles = (M + 31) / 32;
    constexpr unsigned kWaves = AppFeatBlock<PREC>::N / LM_WAVE;
    const uint64_t wave_id = (uint64_t)lm_xcd_swizzle(blockIdx.x, gridDim.x) * kWaves + threadIdx.x / LM_WAVE;
    const uint64_t n_waves = (uint64_t)gridDim.x * kWaves;
    for (uint64_t tile_id = wave_id; tile_id < n_tiles; tile_id += n_waves) {
        // the two samples this lane gathers for (pass 0: tile row gs, pass 1: row 16 + gs)
        float q0[4], q1[4];
        {
            const uint64_t p0 = tile_id * 32 + gs, p1 = p0 + 16;
            list_coords(g, rays, list[p0 < M ? p0 : M - 1], q0);
            list_coords(g, rays, list[p1 < M ? p1 : M - 1], q1);
        }
        floatx16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[v] = 0.0f;
        int t = 0;  // running MFMA step over the concatenated channels
        // Both samples' footprints of a plane are loaded with every load issued before the first use
        // (one memory round trip per plane), and the loads of plane k + 1 are issued before the
        // matrix step of plane k, which then runs under their latency.  Where that many loads in
        // flight would not fit the registers (wide planes), one sample's loads at a time.
        constexpr bool kAhead = 2 * NG * 6 * V <= 144;
        Taps2 t2[2];
        Taps1 t1[2];
        Footprint<T> fp[2][NG];
        auto taps_pass = [&](int k, int pass) {
            const lm_plane &pl = ps.p[k];
            const float *q = pass ? q1 : q0;
            t2[pass] = plane_taps(pl, pick(q, pl.ax0), pick(q, pl.ax1));
            t1[pass] = line_taps(pl, pick(q, pl.axl));
            block_taps(pl, ps.nblk, q, t2[pass], t1[pass]);
        };
        auto load_pass = [&](int k, int pass) {
            const lm_plane &pl = ps.p[k];
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                const int c = V * (int)qlane + gi * V * kQuad;
                if (c < C) footprint_load<T>(pl, t2[pass], t1[pass], c, fp[pass][gi]);
            }
        };
        auto emit_pass = [&](int pass) {
            float *row = tile + (pass * 16 + gs) * ROW;
#pragma unroll
            for (int gi = 0; gi < NG; ++gi) {
                const int c = V * (int)qlane + gi * V * kQuad;
                if (c >= C) continue;
                float prod[V];
                footprint_products<T>(fp[pass][gi], t2[pass], t1[pass], prod);
                if constexpr (V % 4 == 0) {
#pragma unroll
                    for (int i = 0; i < V; i += 4)
                        *reinterpret_cast<float4 *>(row + c + i) = make_float4(prod[i], prod[i + 1], prod[i + 2], prod[i + 3]);
                } else {
#pragma unroll
                    for (int i = 0; i < V; i += 2) *reinterpret_cast<float2 *>(row + c + i) = make_float2(prod[i], prod[i + 1]);
                }
            }
        };
        if (kAhead) { taps_pass(0, 0); taps_pass(0, 1); load_pass(0, 0); load_pass(0, 1); }
        for (int k = 0; k < ps.n; ++k) {
            if (kAhead) {
                __builtin_amdgcn_sched_barrier(0);
                emit_pass(0);
                emit_pass(1);
                __builtin_amdgcn_sched_barrier(0);
                if (k + 1 < ps.n) { taps_pass(k + 1, 0); taps_pass(k + 1, 1); load_pass(k + 1, 0); load_pass(k + 1, 1); }
            } else {
#pragma unroll
                for (int pass = 0; pass < 2; ++pass) {
                    taps_pass(k, pass);
                    load_pass(k, pass);
                    __builtin_amdgcn_sched_barrier(0);
                    emit_pass(pass);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            // LDS operations of one wave complete in order; the fence only pins the compiler
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            // a lane-half reads CW consecutive channels of every 2*CW and feeds them G at a time
            // (the order lm_mlp_pack lays the basis fragments out in)
#pragma unroll
            for (int it = 0; it < C / (2 * CW); ++it) {
                float cw[CW];
                const float4 *src = reinterpret_cast<const float4 *>(tile + j * ROW + 2 * CW * it + CW * (int)h);
#pragma unroll
                for (int i = 0; i < CW / 4; ++i) {
                    const float4 x = src[i];
                    cw[4 * i] = x.x; cw[4 * i + 1] = x.y; cw[4 * i + 2] = x.z; cw[4 * i + 3] = x.w;
                }
#pragma unroll
                for (int u = 0; u < CW / G; ++u, ++t) {
                    frag bf[NP];
                    Mm::pack(cw + u * G, bf);
                    const frag a0 = A[(t * NP) * 64 + lane];
                    acc = Mm::mma(a0, bf[0], acc);
                    if constexpr (NP == 2) {
                        const frag a1 = A[(t * NP + 1) * 64 + lane];
                        acc = Mm::mma(a1, bf[0], acc);
                        acc = Mm::mma(a0, bf[1], acc);
                    }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        const uint64_t p = tile_id * 32 + j;
        if (p < M) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = row_of(v, (int)h);
                if (r < kAppDim) feat[p * kAppDim + r] = acc[v];
            }
        }
    }
}

template <int PREC, typename T>
int launch_app_feat(int nu, const lm_model *m, const PlaneSet &ps, int K, const float *rays, const uint32_t *list,
                    const uint32_t *count, uint32_t cap, float *feat, hipStream_t st) {
    using namespace lm_mma;
    const PackLayout L = pack_layout(PREC, K);
    constexpr int kThreads = AppFeatBlock<PREC>::N;
    const size_t basis = (size_t)32 * K * sizeof(typename Mma<PREC>::elem) * Mma<PREC>::NP;
    const size_t lds = basis + (kThreads / LM_WAVE) * app_feat_tile_bytes(16 * nu);
    if (lds > 160 * 1024) LM_FAIL(LM_ERR_UNSUPPORTED, "basis_mat fragments + tiles (%zu bytes) do not fit LDS", lds);
    const unsigned per_cu = (unsigned)std::max<size_t>(1, std::min<size_t>(2, (size_t)(160 * 1024) / lds));
    const unsigned grid = (unsigned)lm_persistent_blocks((int)per_cu);
#define LM_AF_CASE(NU_)                                                                                            \
    case NU_: {                                                                                                    \
        auto kern = &k_app_feat<PREC, T, NU_>;                                                                     \
        static thread_local size_t reserved_on[LM_MAX_DEVICES] = {}; /* set once per thread, device, kernel, size */ \
        size_t &reserved = reserved_on[lm_current_device()];                                                       \
        if (reserved != lds) {                                                                                     \
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                               \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);              \
            if (e != hipSuccess)                                                                                   \
                LM_FAIL(LM_ERR_LAUNCH, "k_app_feat: LDS reservation failed: %s", hipGetErrorString(e));            \
            reserved = lds;                                                                                        \
        }                                                                                                          \
        hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, st, m->geom, ps, K, (const char *)m->mlp_packed, L, rays, \
                           list, count, cap, feat);                                                                \
        break;                                                                                                     \
    }
    if constexpr (std::is_same<T, Half6>::value) {  // six channels per lane divide 48-channel planes only
        switch (nu) {
            LM_AF_CASE(3)
            default: LM_FAIL(LM_ERR_UNSUPPORTED, "unsupported channel grouping %d", nu);
        }
    } else {
        switch (nu) {
            LM_AF_CASE(1)
            LM_AF_CASE(2)
            LM_AF_CASE(3)
            LM_AF_CASE(4)
            default: LM_FAIL(LM_ERR_UNSUPPORTED, "unsupported channel grouping %d", nu);
        }
    }
#undef LM_AF_CASE
    LM_CHECK_LAUNCH("k_app_feat");
    return LM_OK;
}

}  // namespace

// -------------------------------------------------------------------------------------------
int lm_check_planes(const lm_plane *planes, int32_t n, int *dtype_out, int *K_out) {
    LM_REQUIRE(planes != nullptr, "planes is null");
    LM_REQUIRE(n >= 1 && n <= LM_MAX_PLANES, "n_planes %d out of range 1..%d", n, LM_MAX_PLANES);
    int K = 0;
    for (int k = 0; k < n; ++k) {
        const lm_plane &p = planes[k];
        LM_REQUIRE(p.plane && p.line, "plane %d: null table", k);
        LM_REQUIRE(lm_aligned16(p.plane) && lm_aligned16(p.line), "plane %d: tables must be 16-byte aligned", k);
        LM_REQUIRE(p.H > 0 && p.W > 0 && p.Len > 0, "plane %d: empty table", k);
        LM_REQUIRE(p.C > 0 && (int64_t)p.W * p.C < ((int64_t)1 << 31), "plane %d: a row of more than 2^31 elements", k);
        LM_REQUIRE(p.dtype == planes[0].dtype, "planes must share one storage type");
        LM_REQUIRE(p.dtype == LM_F32 || p.dtype == LM_F16, "plane %d: unknown dtype %d", k, p.dtype);
        const int V = p.dtype == LM_F32 ? 4 : 8;
        LM_REQUIRE(p.C > 0 && p.C % V == 0, "plane %d: channel count %d must be a multiple of %d", k, p.C, V);
        LM_REQUIRE(p.ax0 >= 0 && p.ax0 < 3 && p.ax1 >= 0 && p.ax1 < 3 && p.axl >= 0 && p.axl < 3, "plane %d: bad axis", k);
        K += p.C;
    }
    *dtype_out = planes[0].dtype;
    if (K_out) *K_out = K;
    return LM_OK;
}

static PlaneSet make_set(const lm_plane *planes, int n, const lm_geom *g = nullptr) {
    PlaneSet ps;
    for (int k = 0; k < LM_MAX_PLANES; ++k) ps.p[k] = planes[k < n ? k : 0];
    ps.n = n;
    ps.nblk = g && g->div0 > 0 ? g->div0 * g->div1 : 0;
    return ps;
}

extern "C" int lm_gather_density_xyz(const lm_plane *planes, int32_t n_planes, const float *density_basis,
                                     const float *xyz, int64_t M, float *out, void *stream) {
    int dtype;
    if (int rc = lm_check_planes(planes, n_planes, &dtype, nullptr)) return rc;
    LM_REQUIRE(M >= 0, "negative count");
    if (M == 0) return LM_OK;
    LM_REQUIRE(xyz && out, "null buffer");
    const PlaneSet ps = make_set(planes, n_planes);
    const uint64_t tiles = ((uint64_t)M + kTile - 1) / kTile;
    const unsigned grid = (unsigned)std::min<uint64_t>(tiles, (uint64_t)lm_persistent_blocks(8));
    bool all64 = true;
    for (int k = 0; k < n_planes; ++k) all64 &= planes[k].C == 64;
#define LM_DX(T_, C_)                                                                                               \
    hipLaunchKernelGGL((k_density_xyz<T_, C_>), dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, ps, density_basis, xyz, \
                       (uint64_t)M, out)
    if (dtype == LM_F32) {
        if (all64) LM_DX(float, 64); else LM_DX(float, 0);
    } else {
        if (all64) LM_DX(__half, 64); else LM_DX(__half, 0);
    }
#undef LM_DX
    LM_CHECK_LAUNCH("k_density_xyz");
    return LM_OK;
}

extern "C" int lm_gather_app_xyz(const lm_plane *planes, int32_t n_planes, const float *xyz, int64_t M, float *out,
                                 void *stream) {
    int dtype, K;
    if (int rc = lm_check_planes(planes, n_planes, &dtype, &K)) return rc;
    LM_REQUIRE(M >= 0, "negative count");
    if (M == 0) return LM_OK;
    LM_REQUIRE(xyz && out && lm_aligned16(out), "null or misaligned buffer");
    const PlaneSet ps = make_set(planes, n_planes);
    const uint64_t tiles = ((uint64_t)M + kTile - 1) / kTile;
    const unsigned grid = (unsigned)std::min<uint64_t>(tiles, (uint64_t)lm_persistent_blocks(8));
    if (dtype == LM_F32)
        hipLaunchKernelGGL(k_app_xyz<float>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, ps, K, xyz, (uint64_t)M, out);
    else
        hipLaunchKernelGGL(k_app_xyz<__half>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, ps, K, xyz, (uint64_t)M, out);
    LM_CHECK_LAUNCH("k_app_xyz");
    return LM_OK;
}

int lm_check_geom(const lm_geom *g);

extern "C" int lm_density_valid(const lm_model *m, const float *rays, const uint32_t *valid_idx,
                                const uint32_t *counters, float *sigma, void *stream) {
    LM_REQUIRE(m != nullptr, "model is null");
    if (int rc = lm_check_geom(&m->geom)) return rc;
    int dtype;
    if (int rc = lm_check_planes(m->density, m->n_planes, &dtype, nullptr)) return rc;
    LM_REQUIRE(rays && valid_idx && counters && sigma, "null buffer");
    LM_REQUIRE(m->act == LM_ACT_SOFTPLUS || m->act == LM_ACT_RELU, "unknown activation %d", m->act);
    const PlaneSet ps = make_set(m->density, m->n_planes, &m->geom);
    const unsigned grid = (unsigned)lm_persistent_blocks(8);
    if (dtype == LM_F32)
        hipLaunchKernelGGL(k_density_list<float>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, m->geom, ps,
                           m->density_basis, rays, valid_idx, counters + LM_STAT_N_VALID, m->act, m->density_shift, sigma);
    else
        hipLaunchKernelGGL(k_density_list<__half>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, m->geom, ps,
                           m->density_basis, rays, valid_idx, counters + LM_STAT_N_VALID, m->act, m->density_shift, sigma);
    LM_CHECK_LAUNCH("k_density_list");
    return LM_OK;
}

extern "C" int lm_dense_alpha(const lm_model *m, const float *lin_x, const float *lin_y, const float *lin_z,
                              int32_t gx, int32_t gy, int32_t gz, float length, float *alpha, void *stream) {
    LM_REQUIRE(m != nullptr, "model is null");
    const lm_geom &g = m->geom;
    if (g.vol) {
        LM_REQUIRE(g.vd > 0 && g.vh > 0 && g.vw > 0, "occupancy volume has an empty dimension");
        LM_REQUIRE(g.vol_dtype == LM_F32 || g.vol_dtype == LM_U8 || g.vol_dtype == LM_CELLS, "occupancy volume dtype %d",
                   g.vol_dtype);
    }
    int dtype;
    if (int rc = lm_check_planes(m->density, m->n_planes, &dtype, nullptr)) return rc;
    LM_REQUIRE(gx > 0 && gy > 0 && gz > 0, "empty lattice %d x %d x %d", gx, gy, gz);
    LM_REQUIRE(lin_x && lin_y && lin_z && alpha, "null buffer");
    if (g.div0 > 0)
        LM_FAIL(LM_ERR_UNSUPPORTED, "dense alpha of a block-stacked model: the reference evaluates it per block during "
                                    "training only");
    LM_REQUIRE(m->act == LM_ACT_SOFTPLUS || m->act == LM_ACT_RELU, "unknown activation %d", m->act);
    const PlaneSet ps = make_set(m->density, m->n_planes, &m->geom);
    const uint64_t tiles = ((uint64_t)gx * gy * gz + kTile - 1) / kTile;
    const unsigned grid = (unsigned)std::min<uint64_t>(tiles, (uint64_t)lm_persistent_blocks(8));
    if (dtype == LM_F32)
        hipLaunchKernelGGL(k_dense_alpha<float>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, g, ps, m->density_basis,
                           lin_x, lin_y, lin_z, gx, gy, gz, m->act, m->density_shift, length, alpha);
    else
        hipLaunchKernelGGL(k_dense_alpha<__half>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, g, ps, m->density_basis,
                           lin_x, lin_y, lin_z, gx, gy, gz, m->act, m->density_shift, length, alpha);
    LM_CHECK_LAUNCH("k_dense_alpha");
    return LM_OK;
}

// `count` entries of the list (at most `cap`, the list's capacity) -> products [count, K]
int lm_launch_app_products(const lm_model *m, const float *rays, const uint32_t *app_idx, const uint32_t *count, uint32_t cap,
                           float *products, hipStream_t st) {
    LM_REQUIRE(m != nullptr, "model is null");
    if (int rc = lm_check_geom(&m->geom)) return rc;
    int dtype, K;
    if (int rc = lm_check_planes(m->app, m->n_planes, &dtype, &K)) return rc;
    LM_REQUIRE(rays && app_idx && count && products && lm_aligned16(products), "null or misaligned buffer");
    const PlaneSet ps = make_set(m->app, m->n_planes, &m->geom);
    const unsigned grid = (unsigned)lm_persistent_blocks(8);
    if (dtype == LM_F32)
        hipLaunchKernelGGL(k_app_list<float>, dim3(grid), dim3(kBlock), 0, st, m->geom, ps, K, rays, app_idx, count, cap, products);
    else
        hipLaunchKernelGGL(k_app_list<__half>, dim3(grid), dim3(kBlock), 0, st, m->geom, ps, K, rays, app_idx, count, cap, products);
    LM_CHECK_LAUNCH("k_app_list");
    return LM_OK;
}

extern "C" int lm_app_products(const lm_model *m, const float *rays, const uint32_t *app_idx, const uint32_t *counters,
                               float *products, void *stream) {
    LM_REQUIRE(counters != nullptr, "counters is null");
    return lm_launch_app_products(m, rays, app_idx, counters + LM_STAT_N_APP, UINT32_MAX, products, (hipStream_t)stream);
}

// True when the fused gather + basis_mat kernel covers this model's appearance planes.
int lm_app_feat_supported(const lm_model *m) {
    const int C = m->app[0].C;
    for (int k = 0; k < m->n_planes; ++k)
        if (m->app[k].C != C) return 0;
    return C % 16 == 0 && C >= 16 && C <= 64;
}

int lm_check_prec(int prec);
int lm_check_K(int K);
int lm_launch_app_features(const lm_model *m, const float *rays, const uint32_t *app_idx, const uint32_t *cnt, uint32_t cap,
                           float *feat, hipStream_t st);

// appearance samples (list order) -> feat [n_app, 27] = basis_mat(plane * line products)
extern "C" int lm_app_features(const lm_model *m, const float *rays, const uint32_t *app_idx, const uint32_t *counters,
                               float *feat, void *stream) {
    LM_REQUIRE(counters != nullptr, "counters is null");
    return lm_launch_app_features(m, rays, app_idx, counters + LM_STAT_N_APP, UINT32_MAX, feat, (hipStream_t)stream);
}

int lm_launch_app_features(const lm_model *m, const float *rays, const uint32_t *app_idx, const uint32_t *cnt, uint32_t cap,
                           float *feat, hipStream_t st) {
    LM_REQUIRE(m != nullptr, "model is null");
    if (int rc = lm_check_geom(&m->geom)) return rc;
    int dtype, K;
    if (int rc = lm_check_planes(m->app, m->n_planes, &dtype, &K)) return rc;
    if (int rc = lm_check_prec(m->mlp_prec)) return rc;
    if (int rc = lm_check_K(K)) return rc;
    LM_REQUIRE(rays && app_idx && cnt && feat, "null buffer");
    LM_REQUIRE(m->mlp_packed && lm_aligned16(m->mlp_packed), "packed colour-network weights are null or misaligned");
    if (!lm_app_feat_supported(m))
        LM_FAIL(LM_ERR_UNSUPPORTED, "fused appearance gather needs equal channel counts of 16..64 in steps of 16");
    const PlaneSet ps = make_set(m->app, m->n_planes, &m->geom);
    const int nu = m->app[0].C / 16;
#define LM_AF_GO(PREC_)                                                                                         \
    return dtype == LM_F32 ? launch_app_feat<PREC_, float>(nu, m, ps, K, rays, app_idx, cnt, cap, feat, st)     \
           : nu == 3       ? launch_app_feat<PREC_, Half6>(nu, m, ps, K, rays, app_idx, cnt, cap, feat, st)     \
           : (nu & 1)      ? launch_app_feat<PREC_, Half4>(nu, m, ps, K, rays, app_idx, cnt, cap, feat, st)     \
                           : launch_app_feat<PREC_, __half>(nu, m, ps, K, rays, app_idx, cnt, cap, feat, st)
    switch (m->mlp_prec) {
        case LM_MLP_F32: LM_AF_GO(LM_MLP_F32);
        case LM_MLP_F16: LM_AF_GO(LM_MLP_F16);
        case LM_MLP_BF16: LM_AF_GO(LM_MLP_BF16);
        default: LM_AF_GO(LM_MLP_F16X2);
    }
#undef LM_AF_GO
}

// Density + transmittance march over the rays listed in ray_list (those with valid samples).
int lm_launch_march(const lm_model *m, const float *rays, const uint64_t *bitmap, const uint32_t *p_first,
                    const uint64_t *word_mask, const uint32_t *ray_list, const uint32_t *bins, uint32_t n_rays, uint32_t *queue, float *w_valid,
                    float *acc,
                    float *depth, uint32_t *app_cnt, uint32_t *p_end, uint32_t *n_marched, hipStream_t st) {
    int dtype;
    if (int rc = lm_check_planes(m->density, m->n_planes, &dtype, nullptr)) return rc;
    LM_REQUIRE(m->act == LM_ACT_SOFTPLUS || m->act == LM_ACT_RELU, "unknown activation %d", m->act);
    const PlaneSet ps = make_set(m->density, m->n_planes, &m->geom);
    // as many workgroups as are resident at once (the kernel's register count decides), at most four per CU
    auto resident_grid = [](const void *kernel) {
        // asked once per thread and kernel: the answer depends on the kernel's registers only
        static thread_local const void *known_on[LM_MAX_DEVICES][4] = {};
        static thread_local unsigned grid_on[LM_MAX_DEVICES][4] = {};
        const int dev = lm_current_device();
        const void **known = known_on[dev];
        unsigned *grid = grid_on[dev];
        for (int i = 0; i < 4; ++i)
            if (known[i] == kernel) return grid[i];
        int per_cu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kBlock, 0) != hipSuccess || per_cu < 1) per_cu = 2;
        const unsigned g = (unsigned)lm_persistent_blocks(std::min(per_cu, 4));
        for (int i = 0; i < 4; ++i)
            if (!known[i]) { known[i] = kernel; grid[i] = g; break; }
        return g;
    };
    int c_max = 0;
    for (int k = 0; k < m->n_planes; ++k) c_max = std::max(c_max, (int)m->density[k].C);
    if (n_rays <= kWaveMarchRays) {
        // few rays: a wave per ray, one launch-wide round trip per 64-sample word instead of one per four samples
        const unsigned grid = std::min<unsigned>((n_rays + kBlock / LM_WAVE - 1) / (kBlock / LM_WAVE), (unsigned)lm_persistent_blocks(8));
#define LM_MARCH_WAVE(T_)                                                                                             \
    hipLaunchKernelGGL((k_march_wave<T_>), dim3(grid), dim3(kBlock), 0, st, m->geom, ps, m->density_basis, rays, bitmap, \
                       p_first, word_mask, ray_list, bins, n_rays, m->act, m->density_shift, m->distance_scale,          \
                       m->weight_thres, m->term_eps, w_valid, acc, depth, app_cnt, p_end, n_marched)
        if (dtype == LM_F32) {
            LM_MARCH_WAVE(float);
        } else if (c_max <= 16) {
            LM_MARCH_WAVE(Half4);
        } else {
            LM_MARCH_WAVE(__half);
        }
#undef LM_MARCH_WAVE
        LM_CHECK_LAUNCH("k_march_wave");
        return LM_OK;
    }
#define LM_MARCH(T_, NS_)                                                                                              \
    hipLaunchKernelGGL((k_march<T_, NS_>), dim3(resident_grid(reinterpret_cast<const void *>(&k_march<T_, NS_>))),         \
                       dim3(kBlock), 0, st, m->geom, ps, m->density_basis, rays, bitmap,   \
                       p_first, word_mask, ray_list, bins, n_rays, queue, m->act, m->density_shift, m->distance_scale,            \
                       m->weight_thres, m->term_eps, w_valid, acc, depth, app_cnt, p_end, n_marched)
    // Four samples per round: one per lane of the quad for the footprint arithmetic, 24 loads per lane and plane
    // in flight, half as many dependent round trips per ray as with two (1080p frame, nine fp32 planes: 2.70 ->
    // 2.50 ms although the kernel then holds 223 registers and two waves per SIMD instead of three).
    if (dtype == LM_F32) {
        LM_MARCH(float, LM_MARCH_NS);
    } else if (c_max <= 16) {  // 16-byte loads would leave half of every quad idle
        LM_MARCH(Half4, 4);
    } else {
        LM_MARCH(__half, 4);
    }
#undef LM_MARCH
    LM_CHECK_LAUNCH("k_march");
    return LM_OK;
}
