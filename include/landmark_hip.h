/* landmark_hip.h -- C ABI of the MI355X (gfx950) GridNeRF render path.
 *
 * Drop-in boundary for the single-GPU render branch of InternLandMark/LandMark.  Every
 * entry point names the reference interface it replaces (paths relative to the
 * reference checkout).  Conventions:
 *   - plain pointers and sizes; all array pointers are DEVICE pointers unless the
 *     parameter is documented as host memory; device pointers must be 16-byte aligned,
 *     except ray arrays ([N,6] floats, any row of a 16-byte aligned array: 8-byte aligned);
 *   - the caller owns every buffer (inputs, outputs and the workspace); the library
 *     allocates no memory.  State it keeps between calls: per calling thread, the error
 *     string and a few per-device caches of device facts and kernel attributes (number of
 *     compute units, resident-workgroup counts, whether a kernel's LDS limit has been
 *     raised), filled on first use and never invalidated; per process, for
 *     lm_render_static only, one built-in device array per GPU and a mutex-guarded table of
 *     those arrays' device addresses.  Nothing of it depends on a model or a call's
 *     arguments, so calls from different threads never interact unless they share buffers;
 *   - every function takes the HIP stream to launch on (`void*` = hipStream_t, NULL =
 *     the null stream) and returns without waiting for the GPU;
 *   - return value: LM_OK (0) or a negative lm_status; lm_last_error() describes the
 *     last failure on the calling thread.  Nothing here calls exit() or abort().
 *
 * Data layout.  Feature planes are channel-last: plane[H][W][C] and line[Len][C]
 * (the reference stores [1,C,H,W] and [1,C,Len,1]; lm_relayout_nchw_to_hwc converts).
 * Samples are addressed by their flat index ray*S + s.  The valid-sample list is the
 * ascending list of flat indices that pass the AABB and occupancy tests: the same
 * order the reference's boolean-mask indexing produces.
 */
#ifndef LANDMARK_HIP_H
#define LANDMARK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Changes whenever a struct, an enum value or the meaning of an argument does (2: 16-word counter block;
 * 3: workspace capacities in lm_model, LM_STAT_OVERFLOW). */
#define LM_ABI_VERSION 4
#define LM_MAX_PLANES 12 /* ndims * len(resMode) */

typedef enum lm_status {
    LM_OK = 0,
    LM_ERR_INVALID = -1,     /* bad argument (null, misaligned, out of range) */
    LM_ERR_UNSUPPORTED = -2, /* valid in the reference, not implemented here */
    LM_ERR_LAUNCH = -3,      /* HIP reported an error at launch */
    LM_ERR_WORKSPACE = -4    /* workspace too small */
} lm_status;

enum { LM_F32 = 0, LM_F16 = 1, LM_U8 = 2, LM_CELLS = 3 }; /* planes: F32 | F16; occupancy: F32 | U8 | CELLS */
enum { LM_SAMPLER_AABB = 0, LM_SAMPLER_HULL = 1 }; /* sampling_opt 0 / 1 */
enum { LM_ACT_SOFTPLUS = 0, LM_ACT_RELU = 1 };     /* fea2denseAct */
/* arithmetic of the colour network's and basis_mat's matrix products (accumulation is
 * always fp32).  F16X2 splits every operand into two fp16 parts (x = hi + lo) and forms
 * hi*hi + lo*hi + hi*lo with three fp16 MFMAs: about 21 mantissa bits, for results that
 * must stay within 1e-4 of an fp32 evaluation.  F16 and F16X2 carry features, plane x line
 * products and hidden activations as fp16 numbers: their magnitudes must stay below 65504
 * (F32 and BF16 have the full float range). */
enum { LM_MLP_F32 = 0, LM_MLP_F16 = 1, LM_MLP_BF16 = 2, LM_MLP_F16X2 = 3 };

/* One feature plane with its line (one entry of density_plane/density_line or
 * app_plane/app_line, app/models/gridnerf_sequential.py:676-718).  ax0/ax1 select the
 * normalised coordinates used as the plane's x (-> W) and y (-> H), axl the line's
 * (matMode / vecMode, gridnerf_sequential.py:106-107). */
typedef struct lm_plane {
    const void *plane; /* [H][W][C] */
    const void *line;  /* [Len][C]  */
    int32_t H, W, Len, C;
    int32_t ax0, ax1, axl;
    int32_t dtype; /* LM_F32 | LM_F16 */
} lm_plane;

/* Ray sampling and occupancy culling parameters.
 * sampler HULL (gridnerf_sequential.py:298-319): z = tab_a[s] + far_ray * tab_t[s] with
 *   tab_t = torch.linspace(0,1,S), tab_a = near*(1-tab_t), far_ray = -((o_z-aabb_min_z)/d_z)
 *   or `far` when d_z >= 0.
 * sampler AABB (gridnerf_sequential.py:260-281): z = t_min + tab_a[s] with
 *   tab_a = stepSize*arange(S), t_min = slab entry clamped to [near, far].
 * The tables are passed in (device memory) because torch.linspace is not reproducible
 * from i/(S-1) in float arithmetic.  inv_aabb = 2/aabbSize and vol_inv = 1/size*2 are
 * computed by the caller in float exactly as the reference does
 * (gridnerf_sequential.py:158-159, alpha_mask.py:20-22). */
typedef struct lm_geom {
    int32_t sampler;
    int32_t S;
    float aabb[6]; /* min xyz, max xyz */
    float near_, far_;
    const float *tab_a; /* [S] */
    const float *tab_t; /* [S] */
    float inv_aabb[3];
    /* occupancy volume (app/models/alpha_mask.py); vol == NULL: no culling */
    /* [vd][vh][vw] float, or uint8 (values a uint8 holds exactly), or the cell table
     * lm_pack_occupancy builds from a 0/1 volume: [vd+1][vh+1][vw+1] bytes, one per trilinear
     * cell, bit (zz*4 + yy*2 + xx) = voxel (z0+zz, y0+yy, x0+xx) is 1.  All three give
     * bit-identical decisions; the cell table needs one load per sample instead of eight. */
    const void *vol;
    int32_t vd, vh, vw;
    int32_t vol_dtype; /* LM_F32 | LM_U8 | LM_CELLS */
    float vol_aabb_min[3];
    float vol_inv[3];
    float vol_thre; /* alpha_mask_filter_thre */
    /* Block-stacked model (the "-merged-stack" checkpoint, gridnerf_branch_parallel.py:465-527,
     * rendered through assign_blocks_to_samples, gridnerf_parallel.py:279-338): the XY extent is
     * cut into div0 x div1 blocks, block b = floor((x+1)/blk_w)*div1 + floor((y+1)/blk_h) of the
     * normalised sample, planes are [B][H][W][C] and lines [Len][B][C] with B = div0*div1, H, W
     * the size of one block, and x, y are re-normalised to the block before the lookup.
     * blk_w = (float)(2.0/div0), blk_h = (float)(2.0/div1).  div0 == 0: one block, plain tables.
     * The reference interpolates over the block axis with a block coordinate that is an integer
     * up to float rounding; here the lookup reads block b alone (difference below 1e-6 relative). */
    int32_t div0, div1;
    float blk_w, blk_h;
    /* Optional coarse level of a cell table (vol_dtype LM_CELLS), built by lm_pack_occupancy_coarse; NULL = none.
     * It lets the culling kernels reject runs of samples that lie in empty space without visiting them; the
     * decisions are the same with and without it. */
    const uint8_t *vol_coarse;
} lm_geom;

/* stages of lm_render, in launch order */
enum {
    LM_STAGE_CULL = 1,      /* sampling + culling + compaction, list of rays with valid samples */
    LM_STAGE_DENSITY = 2,   /* density gather fused with the per-ray transmittance march */
    LM_STAGE_WEIGHTS = 3,   /* appearance list from the stored weights */
    LM_STAGE_APP = 4,       /* appearance gather */
    LM_STAGE_COLOUR = 5,    /* basis_mat + encoding + colour network */
    LM_STAGE_COMPOSITE = 6, /* per-ray colour sum */
    LM_N_STAGES = 6
};

typedef struct lm_model {
    lm_geom geom;
    int32_t n_planes; /* ndims * levels, plane index k = dim * levels + level */
    lm_plane density[LM_MAX_PLANES];
    lm_plane app[LM_MAX_PLANES];
    /* NULL, or basis_den.weight [n_planes * C_d] (device): density feature =
     * relu(sum w * product) instead of the plain sum (nonlinear_density,
     * gridnerf_sequential.py:679-680, 819-822) */
    const float *density_basis;
    int32_t act;         /* LM_ACT_* */
    float density_shift; /* softplus(f + shift) */
    float distance_scale;
    float weight_thres; /* rayMarch_weight_thres */
    int32_t mlp_prec;   /* LM_MLP_* the packed weights were packed for */
    const void *mlp_packed; /* device copy of the buffer written by lm_mlp_pack */
    int32_t white_bg;
    float term_eps; /* > 0: stop marching a ray once transmittance < term_eps */
    /* Hint: the chunk's rays are the pixels of an image stored row by row, ray_row of them per
     * row (the chunk may start anywhere in a row).  lm_render then visits rays in 8 x 8 pixel
     * tiles, so that rays handled together are neighbours in both directions and share more of
     * the tables' cache lines.  Results and their order do not depend on it.  0 or not a
     * multiple of 8: rays are visited in the order given. */
    int32_t ray_row;
    int32_t reserved_;
    /* Workspace capacities of one lm_render call, in samples: room for the chunk's valid samples and for its
     * appearance samples (weight > weight_thres).  0 = the worst case (every sample valid, every ray with
     * min(S, 1 / weight_thres) appearance samples), which cannot overflow; the reference's fused path sizes its
     * buffers for 64 rows per ray instead (dist_render/kernel/cuda_render_extend.py:35-159).  A ray that does
     * not fit is counted in counters[LM_STAT_OVERFLOW] and its output is incomplete: a ray whose valid samples
     * exceed cap_valid is rendered as if it had none (background colour, depth 0); a ray whose appearance samples
     * exceed cap_app keeps the depth and the accumulated opacity of its march but gets no colour from them (rgb =
     * 1 - acc on a white background, 0 otherwise).  Either way the pixel is wrong until the call is repeated: the
     * caller reads the counters, and when OVERFLOW is not zero repeats the call with capacities of at least
     * counters[LM_STAT_N_VALID] and counters[LM_STAT_N_APP] (both keep counting past the capacity; after a
     * valid-sample overflow N_APP is a lower bound and the repeat may report a second, appearance overflow). */
    int64_t cap_valid;
    int64_t cap_app;
    /* Optional timing hooks: hipEvent_t handles created by the caller, or NULL.  lm_render
     * records events[0] before its first kernel and events[i] after stage i on `stream`
     * (LM_STAGE_*); it never waits on them. */
    void *events[LM_N_STAGES + 1];
} lm_model;

/* Counters written by lm_render (device memory, LM_STAT_WORDS x uint32). */
/* N_MARCHED: valid samples whose density was gathered (< N_VALID with early termination);
 * BINS..BINS+3: rays with valid samples, by how many they have (>= 64, >= 32, >= 12, fewer): the
 * marching queue hands out the long rays first; QUEUE..QUEUE+7: internal cursors of that queue,
 * one per XCD.  Two lm_render calls that may run at the same time (different streams) need a
 * counter block and a workspace each. */
/* OVERFLOW: rays dropped because their samples did not fit lm_model.cap_valid / cap_app (0 unless capacities
 * below the worst case were asked for). */
enum { LM_STAT_N_VALID = 0, LM_STAT_N_APP = 1, LM_STAT_N_MARCHED = 2, LM_STAT_OVERFLOW = 3, LM_STAT_BINS = 4, LM_STAT_QUEUE = 8, LM_STAT_WORDS = 16 };

int lm_abi_version(void);
const char *lm_last_error(void);

/* [C,H,W] -> [H,W,C] (and [C,Len] -> [Len,C] with W = 1).  The reference keeps NCHW
 * parameters (gridnerf_sequential.py:703-718); its dynamic-fetching variant re-lays them
 * out channel-last the same way (app/models/gridnerf_elastic_cuda.py:274-303). */
int lm_relayout_nchw_to_hwc(const void *src, void *dst, int32_t C, int32_t H, int32_t W, int32_t dtype,
                            void *stream);

/* Build the cell table of a 0/1 occupancy volume (float [D][H][W]); *not_binary (device
 * uint32, zeroed by the caller) is set to 1 if a voxel is neither 0 nor 1, in which case the
 * table must not be used.  cells: (D+1)*(H+1)*(W+1) bytes.  An internal acceleration
 * structure for AlphaGridMask.sample_alpha (app/models/alpha_mask.py:35-47). */
int lm_pack_occupancy(const float *vol, int32_t D, int32_t H, int32_t W, uint8_t *cells, uint32_t *not_binary,
                      void *stream);

/* Coarse level of a cell table: one byte per block of 8 x 8 x 8 cells, set when any cell of the block or of its
 * upper neighbours (+1 block along every axis) has a bit set, so that one lookup answers for a run of samples that
 * spans at most two blocks per axis.  coarse: lm_occupancy_coarse_bytes(D, H, W) bytes.  No counterpart in the
 * reference: an acceleration structure for AlphaGridMask.sample_alpha (app/models/alpha_mask.py:35-47) at the
 * reference's default of half a grid cell per sample (gridnerf_sequential.py:244-281). */
size_t lm_occupancy_coarse_bytes(int32_t D, int32_t H, int32_t W);
int lm_pack_occupancy_coarse(const uint8_t *cells, int32_t D, int32_t H, int32_t W, uint8_t *coarse, void *stream);

/* Alpha of a segment of length `length` at the gx*gy*gz lattice points
 * aabb0*(1-s) + aabb1*s, s taken from the device tables lin_x[gx], lin_y[gy], lin_z[gz]
 * (the caller's torch.linspace(0,1,g)): getDenseAlpha + compute_alpha
 * (gridnerf_sequential.py:321-349, 401-427).  alpha is [gx][gy][gz] as the reference returns
 * it.  If model->geom.vol is set it is the existing mask: points whose lookup is not > 0 keep
 * sigma 0 (vol_thre is not used here).  Reads geom.aabb / inv_aabb / vol*, the density planes,
 * density_basis, act, density_shift. */
int lm_dense_alpha(const lm_model *model, const float *lin_x, const float *lin_y, const float *lin_z, int32_t gx,
                   int32_t gy, int32_t gz, float length, float *alpha, void *stream);

/* The pooling step of updateAlphaMask (gridnerf_sequential.py:351-384): clamp alpha
 * [gx][gy][gz] to [0,1], transpose to [gz][gy][gx], 3x3x3 max pool (stride 1, padding 1),
 * >= thres -> 1.0f else 0.0f into volume [gz][gy][gx].  box[6] (device int32) receives the
 * smallest and largest x, y, z index of the voxels set (INT_MAX / -1 if none), count their
 * number; the new AABB is the lattice coordinates at those indices. */
int lm_alpha_mask_pool(const float *alpha, int32_t gx, int32_t gy, int32_t gz, float thres, float *volume,
                       int32_t *box, uint64_t *count, void *stream);

/* ---- part 1: sampling + AABB / occupancy culling + stable compaction -----------------
 * Replaces sample_ray / sample_ray_within_hull + AlphaGridMask.sample_alpha + the
 * boolean-mask indexing of GridBaseSequential.forward
 * (gridnerf_sequential.py:244-319, 453-465, 528-541; alpha_mask.py:35-59); prior art
 * SamplerayGridsample.cuda (dist_render/kernel/cuda_kernel/sampleray_gridsample/
 * compute_sampleray_gridsample_cuda.cpp:34-151).
 *   rays        [N,6]  origin, direction
 *   bitmap      [ceil(N*S/64)] uint64, bit (i & 63) of word i>>6 = sample i is valid
 *   word_prefix [ceil(N*S/64)] uint32, number of valid samples before each word
 *   valid_idx   [N*S] uint32 capacity, ascending flat indices of valid samples; may be NULL
 *               (not written) when the caller walks the bitmap instead
 *   counters    [LM_STAT_WORDS] uint32, counters[LM_STAT_N_VALID] = number of valid samples
 *   z_out       optional [N*S] sample depths (NULL to skip)
 *   scratch     lm_sample_cull_scratch_bytes(N,S) bytes
 */
size_t lm_sample_cull_scratch_bytes(int64_t N, int32_t S);
int lm_sample_cull(const lm_geom *geom, const float *rays, int64_t N, uint64_t *bitmap, uint32_t *word_prefix,
                   uint32_t *valid_idx, uint32_t *counters, float *z_out, void *scratch, void *stream);

/* ---- part 2: plane / line feature gather ---------------------------------------------
 * Explicit normalised coordinates (isolated gather):
 *   lm_gather_density_xyz  out[M]        = sum_k sum_c plane_k,c(x) * line_k,c(x), or with
 *                          density_basis != NULL relu(sum_k sum_c w[k*C+c] * plane * line)
 *                          GridNeRF.compute_densityfeature, gridnerf_sequential.py:779-827;
 *                          prior art compute_appfeature.gridsample_sum_xyz_b
 *   lm_gather_app_xyz      out[M, n*C]   = plane_k,c(x) * line_k,c(x), column k*C + c
 *                          GridNeRF.compute_appfeature before basis_mat,
 *                          gridnerf_sequential.py:829-864; prior art gridsample_ew_xyb_bz
 */
int lm_gather_density_xyz(const lm_plane *planes, int32_t n_planes, const float *density_basis, const float *xyz,
                          int64_t M, float *out, void *stream);
int lm_gather_app_xyz(const lm_plane *planes, int32_t n_planes, const float *xyz, int64_t M, float *out,
                      void *stream);

/* ---- part 3: colour network ----------------------------------------------------------
 * MLPRender_Fea.forward (app/models/mlp_render_fea.py:44-68) with positional_encoding
 * (app/tools/utils.py:42-48): rgb = sigmoid(L3(relu(L2(relu(L1([feat|view|PE(feat)|PE(view)])))))).
 * Supported shape: app_dim 27, view_pe = fea_pe = 2 (input 150), hidden 128, encode_app off.
 * lm_mlp_pack (HOST memory in and out) reorders basis_mat [27,K] and the three Linear
 * layers into the matrix-core fragment order the kernels read; biases may be NULL.
 * prior art: pe_concate + gemm_fp16.run x3 (dist_render/kernel/cuda_render_extend.py:461-498).
 */
size_t lm_mlp_packed_bytes(int32_t prec, int32_t K_basis);
int lm_mlp_pack(int32_t prec, int32_t K_basis, const float *basis, const float *w1, const float *b1,
                const float *w2, const float *b2, const float *w3, const float *b3, void *packed_out);
/* The appearance embedding (args.encode_app: MLPRender_Fea gets 48 more inputs between the
 * features and the view direction, mlp_render_fea.py:23-24, 55-58) is constant over a frame,
 * so its product with the first layer folds into that layer's bias: pack the layers with the
 * 48 latent columns of W1 removed, and per frame write  b1 + W1[:, 27:75] @ embedding[app_code]
 * into the packed buffer at lm_mlp_bias1_offset().  lm_mlp_pack_bias1: 128 host floats in
 * natural order -> 128 host floats in the kernel's register order. */
size_t lm_mlp_bias1_offset(int32_t prec, int32_t K_basis);
int lm_mlp_pack_bias1(const float *b1, float *packed_b1_out);
/* feat [M,27] fp32, view [M,3] fp32 -> rgb [M,3] fp32 */
int lm_mlp(int32_t prec, const void *packed, int32_t K_basis, const float *feat, const float *view, int64_t M,
           float *rgb, void *stream);
/* products [M,K] fp32 -> feat [M,27] fp32 : basis_mat(products), gridnerf_sequential.py:871 */
int lm_basis(int32_t prec, const void *packed, int32_t K_basis, const float *products, int64_t M, float *feat,
             void *stream);

/* ---- part 4: compositing -------------------------------------------------------------
 * raw2alpha (app/tools/utils.py:51-64) on sigma scattered by the valid list, the weight
 * threshold (gridnerf_sequential.py:479/553) and the sums of :493-504 / :565-576;
 * prior art compute_beta.cuda + compute_weight.cuda (dist_render/kernel/cuda_kernel/volrend).
 *   sigma       [n_valid] densities of the valid samples, in valid-list order
 *   w_valid     [n_valid] out: their weights (same order)
 *   weight_out  optional [N*S] dense weights; only valid samples are written (NULL to skip)
 *   app_first   [N] uint32: slot of the ray's first sample with weight > thres in app_idx
 *   app_cnt     [N] uint32: number of such samples; a ray's slots are contiguous and in
 *               sample order, the order of rays in the list is not defined
 *   app_idx     [capacity N*S] uint32 flat indices of those samples
 *   app_w       [capacity N*S] float their weights
 *   acc, depth  [N] sum of weights, sum of weight * z
 *   counters    counters[LM_STAT_N_APP] is incremented by the number of listed samples
 */
int lm_weights(const lm_geom *geom, const float *rays, int64_t N, const uint64_t *bitmap,
               const uint32_t *word_prefix, const float *sigma, float distance_scale, float weight_thres,
               float term_eps, float *w_valid, float *weight_out, uint32_t *app_first, uint32_t *app_cnt,
               uint32_t *app_idx, float *app_w, float *acc, float *depth, uint32_t *counters, void *stream);

/* The colour sum of gridnerf_sequential.py:493-502 / :565-574 over the appearance list lm_weights built:
 *   rgb_map[r] = clamp(sum_i app_w[first_r + i] * rgb[first_r + i] + (white_bg ? 1 - acc[r] : 0), 0, 1)
 * with rgb [n_app,3] the colour network's output per list slot (samples outside the list have rgb 0 in
 * the reference and contribute nothing).  prior art: the volrend kernels of dist_render/kernel/cuda_kernel. */
int lm_composite_rgb(int64_t N, const uint32_t *app_first, const uint32_t *app_cnt, const float *app_w, const float *rgb,
                     const float *acc, int32_t white_bg, float *rgb_map, void *stream);

/* ---- whole chunk ---------------------------------------------------------------------
 * GridBaseSequential.forward(rays_chunk, white_bg, is_train=False)
 * (gridnerf_sequential.py:439-658) -> rgb_map [N,3], depth_map [N].
 * workspace: lm_render_workspace_bytes(model, N) bytes of device memory, reusable
 * across calls (the role of MultiBlockParallelCuda.allocate_tensors,
 * dist_render/kernel/cuda_render_extend.py:35-159).  counters: [LM_STAT_WORDS] uint32
 * device memory, may be NULL.  No host synchronisation happens inside. */
size_t lm_render_workspace_bytes(const lm_model *model, int64_t N);
int lm_render(const lm_model *model, const float *rays, int64_t N, void *workspace, size_t workspace_bytes,
              float *rgb_map, float *depth_map, uint32_t *counters, void *stream);

/* lm_render out of a workspace built into the library, for callers that cannot allocate device
 * memory or pass a workspace along: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  No counterpart in the reference (its fused path allocates its buffers
 * with torch, dist_render/kernel/cuda_render_extend.py:35-159).  Same arguments, results and
 * stages as lm_render; the workspace is a LM_STATIC_WORKSPACE_BYTES array in the library's device
 * image (every GPU the library runs on holds one until the process ends).  The call allocates
 * nothing; the array's address is looked up on the first call on a device.  A chunk whose
 * lm_render_workspace_bytes() exceeds the array is refused with LM_ERR_WORKSPACE (80 MiB holds
 * 4096 rays of 128 samples).  All calls on one GPU share the array: calls that overlap on one
 * GPU (different streams or threads) race; everything that must start at zero is cleared by the
 * call's own kernels on `stream`. */
#define LM_STATIC_WORKSPACE_BYTES (80u << 20)
int lm_render_static(const lm_model *model, const float *rays, int64_t N, float *rgb_map, float *depth_map,
                     uint32_t *counters, void *stream);

/* ---- either side of the path in the serving loop ------------------------------------------
 * lm_generate_rays: rays[j*W+i] = (pose[:,3], pose[:,:3] @ (dir_x[i], dir_y[j], -1)), the
 * pinhole rays of dist_render/dataset/utils.py:57-113 (generate_rays).  dir_x [W] and dir_y [H]
 * are the reference's two torch.arange tables (device memory; computed by the caller so they
 * hold the reference's values), pose_3x4 is HOST memory, row-major.
 * lm_rgba8: rgb [N,3] in [0,1] -> [N,4] bytes (r,g,b,255) with torch's truncating float->uint8
 * conversion, the tail of model_infer_postprocess (dist_render/ddp_infer/nerf_inferer.py:366-370). */
int lm_generate_rays(const float *dir_x, const float *dir_y, const float *pose_3x4, int32_t H, int32_t W, float *rays,
                     void *stream);
int lm_rgba8(const float *rgb, int64_t N, uint8_t *rgba, void *stream);

/* Stage-level pieces of lm_render for validation and profiling (same kernels). */
int lm_density_valid(const lm_model *model, const float *rays, const uint32_t *valid_idx,
                     const uint32_t *counters, float *sigma, void *stream);
int lm_app_products(const lm_model *model, const float *rays, const uint32_t *app_idx, const uint32_t *counters,
                    float *products, void *stream);
/* appearance samples (list order) -> feat [n_app,27] = basis_mat(plane*line products): the
 * gather fused with the projection, GridNeRF.compute_appfeature (gridnerf_sequential.py:829-871).
 * Needs a 16-bit matrix mode (not LM_MLP_F32) and equal channel counts per plane of 16, 32, 48 or 64. */
int lm_app_features(const lm_model *model, const float *rays, const uint32_t *app_idx, const uint32_t *counters,
                    float *feat, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LANDMARK_HIP_H */
