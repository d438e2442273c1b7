// C-ABI plumbing: error string, launch sizing, table relayout and the whole-chunk render.
#include <stdarg.h>

#include <algorithm>
#include <mutex>

#include "lm_common.h"

static thread_local char g_err[512] = "";

void lm_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char *lm_last_error(void) { return g_err; }
extern "C" int lm_abi_version(void) { return LM_ABI_VERSION; }

int lm_current_device(void) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0) dev = 0;
    return dev < LM_MAX_DEVICES ? dev : LM_MAX_DEVICES - 1;
}

int lm_persistent_blocks(int blocks_per_cu) {
    static thread_local int cus[LM_MAX_DEVICES] = {};  // per device: a thread may switch GPUs between calls
    const int dev = lm_current_device();
    if (cus[dev] == 0) {
        int n = 0;
        cus[dev] = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0 ? n : 256;
    }
    return cus[dev] * blocks_per_cu;
}

// ---- [C,H,W] -> [H,W,C] ---------------------------------------------------------------------
namespace {
template <typename T>
__global__ __launch_bounds__(256) void k_relayout(const T *__restrict__ src, T *__restrict__ dst, int C, uint64_t HW) {
    // 64 texels x 64 channels per tile through LDS: coalesced reads along HW, coalesced writes along C
    __shared__ T tile[64][65];
    const uint64_t t0 = (uint64_t)blockIdx.x * 64;
    const int c0 = blockIdx.y * 64;
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    for (int cc = ty; cc < 64; cc += 4) {
        const int c = c0 + cc;
        const uint64_t t = t0 + tx;
        if (c < C && t < HW) tile[cc][tx] = src[(uint64_t)c * HW + t];
    }
    __syncthreads();
    for (int tt = ty; tt < 64; tt += 4) {
        const uint64_t t = t0 + tt;
        const int c = c0 + tx;
        if (c < C && t < HW) dst[t * C + c] = tile[tx][tt];
    }
}
}  // namespace

extern "C" int lm_relayout_nchw_to_hwc(const void *src, void *dst, int32_t C, int32_t H, int32_t W, int32_t dtype,
                                       void *stream) {
    LM_REQUIRE(src && dst && src != dst, "null or aliased buffer");
    LM_REQUIRE(C > 0 && H > 0 && W > 0, "empty table");
    LM_REQUIRE(dtype == LM_F32 || dtype == LM_F16, "unknown dtype %d", dtype);
    const uint64_t HW = (uint64_t)H * (uint64_t)W;
    const uint64_t bx = (HW + 63) / 64;
    LM_REQUIRE(bx < (1ull << 31), "table too large");
    dim3 grid((unsigned)bx, (unsigned)((C + 63) / 64));
    if (dtype == LM_F32)
        hipLaunchKernelGGL(k_relayout<float>, grid, dim3(256), 0, (hipStream_t)stream, (const float *)src, (float *)dst, C, HW);
    else
        hipLaunchKernelGGL(k_relayout<uint16_t>, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t *)src,
                           (uint16_t *)dst, C, HW);
    LM_CHECK_LAUNCH("k_relayout");
    return LM_OK;
}

// ---- whole chunk -------------------------------------------------------------------------------
int lm_check_geom(const lm_geom *g);
int lm_check_planes(const lm_plane *planes, int32_t n, int *dtype_out, int *K_out);
int lm_app_feat_supported(const lm_model *m);
int lm_launch_app_colour(int prec, const void *packed, int K, int S, const float *feat, const float *rays,
                         const uint32_t *app_idx, const uint32_t *count, uint32_t cap, float *rgb, hipStream_t stream);
int lm_launch_app_features(const lm_model *m, const float *rays, const uint32_t *app_idx, const uint32_t *count, uint32_t cap,
                           float *feat, hipStream_t st);
int lm_launch_app_products(const lm_model *m, const float *rays, const uint32_t *app_idx, const uint32_t *count, uint32_t cap,
                           float *products, hipStream_t st);
int lm_launch_composite(int64_t N, const uint32_t *app_first, const uint32_t *app_cnt, const float *app_w,
                        const float *rgb, const float *acc, int white_bg, uint32_t row, float *rgb_map,
                        hipStream_t stream);
int lm_launch_zero_counters(uint32_t *counters, hipStream_t stream);
int lm_launch_cull_setup(const lm_geom *geom, const float *rays, int64_t N, uint64_t *bitmap, uint32_t *p_first,
                         uint32_t *ray_list, uint32_t *n_active, uint32_t *n_valid, float *acc, float *depth,
                         uint32_t *app_cnt, uint32_t *p_end, uint32_t row, uint32_t cap_valid, uint32_t *overflow,
                         uint64_t *word_mask, hipStream_t st);
int lm_launch_app_slots(int S, int64_t N, const uint64_t *bitmap, const uint32_t *p_first, const uint64_t *word_mask,
                        const float *w_valid,
                        float weight_thres, uint32_t *app_cnt, const uint32_t *p_end, uint32_t *app_first,
                        uint32_t *app_idx, float *app_w, uint32_t *app_count, uint32_t row, uint32_t cap_app,
                        uint32_t *overflow, hipStream_t stream);
int lm_launch_march(const lm_model *m, const float *rays, const uint64_t *bitmap, const uint32_t *p_first,
                    const uint64_t *word_mask, const uint32_t *ray_list, const uint32_t *bins, uint32_t n_rays, uint32_t *queue, float *w_valid, float *acc,
                    float *depth, uint32_t *app_cnt, uint32_t *p_end, uint32_t *n_marched, hipStream_t st);
int lm_launch_basis(int prec, const void *packed, int K, const float *products, uint64_t M, const uint32_t *count,
                    uint32_t cap, float *feat, hipStream_t st);

namespace {
struct Workspace {
    uint64_t *bitmap;
    float *w_valid;
    uint32_t *app_first;
    uint32_t *app_cnt;
    uint32_t *p_first;
    uint32_t *p_end;
    uint64_t *word_mask;  // per ray: which of its bitmap words hold valid samples (sample counts other than 64, 128)
    uint32_t *ray_list;
    uint32_t *app_idx;
    float *app_w;
    float *rgb;
    float *feat;
    float *products;  // only when the fused appearance gather does not cover the model
    float *acc;
    uint32_t *counters;
    uint64_t cap_valid, cap_app;  // room for valid samples and for appearance samples
    size_t total;
};

Workspace carve(char *base, int64_t N, int32_t S, int32_t K, bool need_products, float weight_thres, int64_t want_valid,
                int64_t want_app) {
    Workspace w;
    size_t o = 0;
    auto take = [&](size_t bytes) {
        char *p = base ? base + o : nullptr;
        o = (o + bytes + 255) & ~(size_t)255;
        return p;
    };
    const uint64_t total = (uint64_t)N * (uint64_t)S, n_words = (total + 63) / 64;
    // Every sample may be valid.  A ray's weights are non-negative and sum to at most 1 (+ S * 1e-10 from the
    // reference's cumulative-product guard), so at most 1 / threshold of them exceed the threshold.
    uint64_t per_ray = (uint64_t)S;
    if (weight_thres > 0.0f) per_ray = std::min<uint64_t>(per_ray, (uint64_t)(1.001 / (double)weight_thres) + 2);
    // capacities below the worst case are the caller's choice (lm_model.cap_valid / cap_app); kernels check them
    const uint64_t cap = want_app > 0 ? std::min<uint64_t>((uint64_t)want_app, (uint64_t)N * per_ray) : (uint64_t)N * per_ray;
    w.cap_app = cap;
    w.cap_valid = want_valid > 0 ? std::min<uint64_t>((uint64_t)want_valid, total) : total;
    w.bitmap = (uint64_t *)take(n_words * 8);
    w.w_valid = (float *)take(w.cap_valid * 4);
    w.app_first = (uint32_t *)take((uint64_t)N * 4);
    w.app_cnt = (uint32_t *)take((uint64_t)N * 4);
    w.p_first = (uint32_t *)take((uint64_t)N * 4);
    w.p_end = (uint32_t *)take((uint64_t)N * 4);
    w.word_mask = (uint64_t *)take((uint64_t)N * 8);
    w.ray_list = (uint32_t *)take((uint64_t)N * 4 * LM_RAY_BINS);  // one list per bin of the marching queue
    w.app_idx = (uint32_t *)take(cap * 4);
    w.app_w = (float *)take(cap * 4);
    w.rgb = (float *)take(cap * 12);
    w.feat = (float *)take(cap * 27 * 4);
    w.products = need_products ? (float *)take(cap * (uint64_t)K * 4) : nullptr;
    w.acc = (float *)take((uint64_t)N * 4);
    w.counters = (uint32_t *)take(LM_STAT_WORDS * 4);
    w.total = o;
    return w;
}

int check_model(const lm_model *m, int *K) {
    LM_REQUIRE(m != nullptr, "model is null");
    if (int rc = lm_check_geom(&m->geom)) return rc;
    int dt;
    if (int rc = lm_check_planes(m->density, m->n_planes, &dt, nullptr)) return rc;
    if (int rc = lm_check_planes(m->app, m->n_planes, &dt, K)) return rc;
    const int64_t blocks = m->geom.div0 > 0 ? (int64_t)m->geom.div0 * m->geom.div1 : 1;
    for (int k = 0; k < m->n_planes; ++k)
        for (const lm_plane *pl : {&m->density[k], &m->app[k]}) {
            // line tables are addressed with 32-bit element offsets
            LM_REQUIRE((int64_t)pl->Len * pl->C * blocks < ((int64_t)1 << 31), "plane %d: line table too large", k);
            if (m->geom.div0 > 0)
                LM_REQUIRE(pl->ax0 == 0 && pl->ax1 == 1 && pl->axl == 2,
                           "a block-stacked model has XY planes and z lines only (plane %d)", k);
        }
    return LM_OK;
}

int render_chunk(const lm_model *m, int K, const float *rays, int64_t N, void *workspace, size_t workspace_bytes,
                 float *rgb_map, float *depth_map, uint32_t *counters, void *stream);
}  // namespace

extern "C" size_t lm_render_workspace_bytes(const lm_model *m, int64_t N) {
    int K;
    if (check_model(m, &K) || N <= 0) return 0;
    if (m->cap_valid < 0 || m->cap_app < 0) return 0;
    return carve(nullptr, N, m->geom.S, K, !lm_app_feat_supported(m), m->weight_thres, m->cap_valid, m->cap_app).total;
}

extern "C" int lm_render(const lm_model *m, const float *rays, int64_t N, void *workspace, size_t workspace_bytes,
                         float *rgb_map, float *depth_map, uint32_t *counters, void *stream) {
    int K;
    if (int rc = check_model(m, &K)) return rc;
    return render_chunk(m, K, rays, N, workspace, workspace_bytes, rgb_map, depth_map, counters, stream);
}

// ---- the same render out of a workspace that lives in the library's own image ------------------
// One array per GPU (each device that loads the code object holds its own copy at its own
// address).  In host code the array's name is only a handle for hipGetSymbolAddress: the device
// address is looked up once per device and everything after that uses the pointer.
static __device__ __align__(256) unsigned char scratch[LM_STATIC_WORKSPACE_BYTES];

namespace {
constexpr int kMaxDevices = LM_MAX_DEVICES;
std::mutex g_scratch_lock;
void *g_scratch_ptr[kMaxDevices] = {};

int static_workspace(void **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
        LM_FAIL(LM_ERR_LAUNCH, "lm_render_static: no current device (or device index %d beyond %d)", dev, kMaxDevices - 1);
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (!g_scratch_ptr[dev]) {
        void *ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr)
            LM_FAIL(LM_ERR_LAUNCH, "lm_render_static: address of the built-in workspace on device %d: %s", dev,
                    hipGetErrorString(e));
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return LM_OK;
}
}  // namespace

extern "C" int lm_render_static(const lm_model *m, const float *rays, int64_t N, float *rgb_map, float *depth_map,
                                uint32_t *counters, void *stream) {
    int K;
    if (int rc = check_model(m, &K)) return rc;
    LM_REQUIRE(N >= 0, "negative ray count");
    if (N == 0) return LM_OK;
    LM_REQUIRE(m->cap_valid >= 0 && m->cap_app >= 0, "negative workspace capacity");
    const size_t need = carve(nullptr, N, m->geom.S, K, !lm_app_feat_supported(m), m->weight_thres, m->cap_valid, m->cap_app).total;
    if (need > (size_t)LM_STATIC_WORKSPACE_BYTES)
        LM_FAIL(LM_ERR_WORKSPACE,
                "lm_render_static: %lld rays x %d samples need %zu bytes of workspace, the built-in one has %zu; "
                "render fewer rays per call or use lm_render with a workspace of your own",
                (long long)N, m->geom.S, need, (size_t)LM_STATIC_WORKSPACE_BYTES);
    void *ws = nullptr;
    if (int rc = static_workspace(&ws)) return rc;
    return render_chunk(m, K, rays, N, ws, (size_t)LM_STATIC_WORKSPACE_BYTES, rgb_map, depth_map, counters, stream);
}

namespace {
int render_chunk(const lm_model *m, int K, const float *rays, int64_t N, void *workspace, size_t workspace_bytes,
                 float *rgb_map, float *depth_map, uint32_t *counters, void *stream) {
    LM_REQUIRE(N >= 0, "negative ray count");
    if (N == 0) return LM_OK;
    LM_REQUIRE(rays && rgb_map && depth_map, "null buffer");
    LM_REQUIRE(workspace && lm_aligned16(workspace), "workspace is null or misaligned");
    const int S = m->geom.S;
    LM_REQUIRE((uint64_t)N * (uint64_t)S < (1ull << 32), "N*S does not fit 32-bit sample indices; split the chunk");
    const bool fused = lm_app_feat_supported(m) != 0;
    LM_REQUIRE(m->cap_valid >= 0 && m->cap_app >= 0, "negative workspace capacity");
    Workspace w = carve((char *)workspace, N, S, K, !fused, m->weight_thres, m->cap_valid, m->cap_app);
    if (w.total > workspace_bytes)
        LM_FAIL(LM_ERR_WORKSPACE, "workspace has %zu bytes, %zu needed for N=%lld S=%d K=%d", workspace_bytes, w.total,
                (long long)N, S, K);
    hipStream_t st = (hipStream_t)stream;
    uint32_t *cnt = counters ? counters : w.counters;
    auto mark = [&](int i) {
        if (m->events[i]) (void)hipEventRecord((hipEvent_t)m->events[i], st);
    };
    LM_REQUIRE(m->ray_row >= 0, "negative ray_row");
    const uint32_t row = m->ray_row % 8 == 0 ? (uint32_t)m->ray_row : 0u;  // tiles of 8 x 8 pixels need whole tiles per row
    mark(0);
    if (int rc = lm_launch_zero_counters(cnt, st)) return rc;
    if (int rc = lm_launch_cull_setup(&m->geom, rays, N, w.bitmap, w.p_first, w.ray_list, cnt + LM_STAT_BINS,
                                      cnt + LM_STAT_N_VALID, w.acc, depth_map, w.app_cnt, w.p_end, row, (uint32_t)w.cap_valid,
                                      cnt + LM_STAT_OVERFLOW, w.word_mask, st))
        return rc;
    mark(LM_STAGE_CULL);
    // the cull writes word masks for rays of three bitmap words and more (other sample counts take the kernel
    // with one lane per word, whose rays have one or two words)
    const uint64_t *masks = (S == 64 || S == 128) ? nullptr : w.word_mask;
    if (int rc = lm_launch_march(m, rays, w.bitmap, w.p_first, masks, w.ray_list, cnt + LM_STAT_BINS, (uint32_t)N, cnt + LM_STAT_QUEUE,
                                 w.w_valid, w.acc, depth_map, w.app_cnt, w.p_end, cnt + LM_STAT_N_MARCHED, st))
        return rc;
    mark(LM_STAGE_DENSITY);
    if (int rc = lm_launch_app_slots(S, N, w.bitmap, w.p_first, masks, w.w_valid, m->weight_thres, w.app_cnt, w.p_end,
                                     w.app_first, w.app_idx, w.app_w, cnt + LM_STAT_N_APP, row, (uint32_t)w.cap_app,
                                     cnt + LM_STAT_OVERFLOW, st))
        return rc;
    mark(LM_STAGE_WEIGHTS);
    if (fused) {
        if (int rc = lm_launch_app_features(m, rays, w.app_idx, cnt + LM_STAT_N_APP, (uint32_t)w.cap_app, w.feat, st)) return rc;
    } else {
        // channel counts the fused kernel does not cover: products through memory, then basis_mat
        if (int rc = lm_launch_app_products(m, rays, w.app_idx, cnt + LM_STAT_N_APP, (uint32_t)w.cap_app, w.products, st)) return rc;
        if (int rc = lm_launch_basis(m->mlp_prec, m->mlp_packed, K, w.products, 0, cnt + LM_STAT_N_APP, (uint32_t)w.cap_app, w.feat, st))
            return rc;
    }
    mark(LM_STAGE_APP);
    if (int rc = lm_launch_app_colour(m->mlp_prec, m->mlp_packed, K, S, w.feat, rays, w.app_idx, cnt + LM_STAT_N_APP,
                                      (uint32_t)w.cap_app, w.rgb, st))
        return rc;
    mark(LM_STAGE_COLOUR);
    if (int rc = lm_launch_composite(N, w.app_first, w.app_cnt, w.app_w, w.rgb, w.acc, m->white_bg, row, rgb_map, st)) return rc;
    mark(LM_STAGE_COMPOSITE);
    return LM_OK;
}
}  // namespace
