// The two steps either side of the render path in the serving loop: camera pose -> rays in
// front of it, float rgb -> RGBA8 behind it.
//
// Reference: generate_rays / get_ray_directions_blender_faster / get_rays_with_directions
// (dist_render/dataset/utils.py:57-113) and the tail of model_infer_postprocess
// (dist_render/ddp_infer/nerf_inferer.py:366-370: rgb*255, alpha channel 255, .byte()).
#include "lm_common.h"

namespace {

struct Pose {
    float m[12];  // row-major [3][4] camera-to-world
};

// rays[j*W + i] = (origin, R * (dir_x[i], dir_y[j], -1))
__global__ __launch_bounds__(256) void k_generate_rays(const float *__restrict__ dir_x, const float *__restrict__ dir_y,
                                                       Pose pose, int H, int W, float *__restrict__ rays) {
    const uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (uint64_t)H * W) return;
    const int i = (int)(idx % (uint64_t)W), j = (int)(idx / (uint64_t)W);
    const float dx = dir_x[i], dy = dir_y[j], dz = -1.0f;
    float2 *out = reinterpret_cast<float2 *>(rays + 6 * idx);
    float d[3];
#pragma unroll
    for (int c = 0; c < 3; ++c) d[c] = fmaf(pose.m[4 * c + 2], dz, fmaf(pose.m[4 * c + 1], dy, pose.m[4 * c] * dx));
    out[0] = make_float2(pose.m[3], pose.m[7]);
    out[1] = make_float2(pose.m[11], d[0]);
    out[2] = make_float2(d[1], d[2]);
}

__global__ __launch_bounds__(256) void k_rgba8(const float *__restrict__ rgb, uint64_t N, uint32_t *__restrict__ out) {
    const uint64_t idx = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= N) return;
    uint32_t px = 0xFF000000u;
#pragma unroll
    for (int c = 0; c < 3; ++c) {
        // torch's float -> uint8 conversion truncates toward zero; inputs are in [0, 1]
        const float v = rgb[3 * idx + c] * 255.0f;
        const uint32_t b = (uint32_t)(int)fminf(fmaxf(v, 0.0f), 255.0f);
        px |= b << (8 * c);
    }
    out[idx] = px;
}

}  // namespace

extern "C" int lm_generate_rays(const float *dir_x, const float *dir_y, const float *pose_3x4, int32_t H, int32_t W,
                                float *rays, void *stream) {
    LM_REQUIRE(dir_x && dir_y && pose_3x4 && rays, "null pointer");
    LM_REQUIRE(H > 0 && W > 0, "empty image");
    LM_REQUIRE((reinterpret_cast<uintptr_t>(rays) & 7u) == 0, "rays must be 8-byte aligned");
    Pose p;
    for (int k = 0; k < 12; ++k) p.m[k] = pose_3x4[k];
    const uint64_t n = (uint64_t)H * W;
    hipLaunchKernelGGL(k_generate_rays, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, dir_x, dir_y, p,
                       H, W, rays);
    LM_CHECK_LAUNCH("k_generate_rays");
    return LM_OK;
}

extern "C" int lm_rgba8(const float *rgb, int64_t N, uint8_t *rgba, void *stream) {
    LM_REQUIRE(N >= 0, "negative count");
    if (N == 0) return LM_OK;
    LM_REQUIRE(rgb && rgba, "null pointer");
    LM_REQUIRE((reinterpret_cast<uintptr_t>(rgba) & 3u) == 0, "rgba must be 4-byte aligned");
    hipLaunchKernelGGL(k_rgba8, dim3((unsigned)(((uint64_t)N + 255) / 256)), dim3(256), 0, (hipStream_t)stream, rgb,
                       (uint64_t)N, reinterpret_cast<uint32_t *>(rgba));
    LM_CHECK_LAUNCH("k_rgba8");
    return LM_OK;
}
