/* Scalar C restatement of the GridNeRF render path.  TEST INFRASTRUCTURE ONLY.
 *
 * One sample at a time, one float operation at a time, no vector units, no fused
 * multiply-add (build with -ffp-contract=off).  It serves two purposes:
 *   1. it pins the PyTorch oracle (oracle/gridnerf_oracle.py) from a second, independent
 *      direction: the geometry / occupancy decisions must agree bit for bit, the
 *      interpolated features and colours to float rounding;
 *   2. it states, in plain C, the exact operation order a device kernel has to follow to
 *      reproduce the reference's sample masks.
 * Nothing in the product may link or call it.
 *
 * Reference lines followed (paths relative to the reference checkout):
 *   lmref_sample_z / lmref_point      app/models/gridnerf_sequential.py:260-281, 298-319
 *   lmref_alpha_lookup                app/models/alpha_mask.py:35-59 + ATen grid_sampler_3d
 *                                     (trilinear, zeros padding, align_corners=True)
 *   lmref_bilinear / lmref_linear     F.grid_sample 4-D as called at
 *                                     gridnerf_sequential.py:803-812, 851-862
 *   lmref_render                      gridnerf_sequential.py:448-504 / 523-576,
 *                                     app/tools/utils.py:42-64,
 *                                     app/models/mlp_render_fea.py:44-68
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

typedef struct {
    int sampling_opt;      /* 0: slab entry + fixed step, 1: near .. floor hit */
    int S;                 /* samples per ray */
    float aabb[6];         /* min xyz, max xyz */
    float near, far;
    const float *tab_a;    /* [S] hull: near*(1-t) ; aabb: stepSize*arange */
    const float *tab_t;    /* [S] hull: t = linspace(0,1,S) ; aabb: unused */
    float inv_aabb[3];     /* 2/aabbSize, computed by the caller in float */
    /* occupancy volume; vol == NULL disables it */
    const float *vol;
    int vd, vh, vw;
    float vol_aabb_min[3];
    float vol_inv[3];      /* 1/size*2, computed by the caller in float */
    float vol_thre;
} lmref_geom;

/* per-ray scalar: hull far / slab t_min */
static float ray_param(const lmref_geom *g, const float *ray) {
    if (g->sampling_opt) {
        float o_z = ray[2] - g->aabb[2];
        float far = -(o_z / ray[5]);
        if (ray[5] >= 0.0f) far = g->far;
        return far;
    }
    float tmin = -INFINITY;
    for (int k = 0; k < 3; ++k) {
        float v = ray[3 + k] == 0.0f ? 1e-6f : ray[3 + k];
        float ra = (g->aabb[3 + k] - ray[k]) / v;
        float rb = (g->aabb[k] - ray[k]) / v;
        float m = ra < rb ? ra : rb;
        if (ra != ra || rb != rb) m = NAN;
        if (m > tmin || m != m) tmin = m;
    }
    if (tmin < g->near) tmin = g->near;
    if (tmin > g->far) tmin = g->far;
    return tmin;
}

float lmref_sample_z(const lmref_geom *g, const float *ray, int s) {
    float rp = ray_param(g, ray);
    if (g->sampling_opt) {
        float b = rp * g->tab_t[s];
        return g->tab_a[s] + b;
    }
    return rp + g->tab_a[s];
}

void lmref_point(const float *ray, float z, float *pt) {
    for (int k = 0; k < 3; ++k) {
        float m = ray[3 + k] * z;
        pt[k] = ray[k] + m;
    }
}

static int inside_aabb(const lmref_geom *g, const float *pt) {
    for (int k = 0; k < 3; ++k)
        if (g->aabb[k] > pt[k] || pt[k] > g->aabb[3 + k]) return 0;
    return 1;
}

/* trilinear lookup, value only */
float lmref_alpha_lookup(const lmref_geom *g, const float *pt) {
    float c[3];
    for (int k = 0; k < 3; ++k) {
        float d = pt[k] - g->vol_aabb_min[k];
        float m = d * g->vol_inv[k];
        c[k] = m - 1.0f;
    }
    int W = g->vw, H = g->vh, D = g->vd;
    float ix = ((c[0] + 1.0f) / 2.0f) * (float)(W - 1);
    float iy = ((c[1] + 1.0f) / 2.0f) * (float)(H - 1);
    float iz = ((c[2] + 1.0f) / 2.0f) * (float)(D - 1);
    float fx = floorf(ix), fy = floorf(iy), fz = floorf(iz);
    /* corner names follow ATen: t/b = z, n/s = y, w/e = x */
    float x0 = fx, x1 = fx + 1.0f, y0 = fy, y1 = fy + 1.0f, z0 = fz, z1 = fz + 1.0f;
    float tnw = (x1 - ix) * (y1 - iy) * (z1 - iz);
    float tne = (ix - x0) * (y1 - iy) * (z1 - iz);
    float tsw = (x1 - ix) * (iy - y0) * (z1 - iz);
    float tse = (ix - x0) * (iy - y0) * (z1 - iz);
    float bnw = (x1 - ix) * (y1 - iy) * (iz - z0);
    float bne = (ix - x0) * (y1 - iy) * (iz - z0);
    float bsw = (x1 - ix) * (iy - y0) * (iz - z0);
    float bse = (ix - x0) * (iy - y0) * (iz - z0);
    long xi0 = (long)fx, yi0 = (long)fy, zi0 = (long)fz;
    long xs[2] = {xi0, xi0 + 1}, ys[2] = {yi0, yi0 + 1}, zs[2] = {zi0, zi0 + 1};
    float wts[8] = {tnw, tne, tsw, tse, bnw, bne, bsw, bse};
    float out = 0.0f;
    int n = 0;
    for (int zz = 0; zz < 2; ++zz)
        for (int yy = 0; yy < 2; ++yy)
            for (int xx = 0; xx < 2; ++xx, ++n) {
                long x = xs[xx], y = ys[yy], z = zs[zz];
                if (x >= 0 && x < W && y >= 0 && y < H && z >= 0 && z < D) {
                    float t = g->vol[((size_t)z * H + y) * W + x] * wts[n];
                    out = out + t;
                }
            }
    return out;
}

/* valid[N*S] (0/1), z[N*S]; returns the number of valid samples. */
long lmref_sample_cull(const lmref_geom *g, const float *rays, long N, uint8_t *valid, float *zout) {
    long cnt = 0;
    for (long r = 0; r < N; ++r)
        for (int s = 0; s < g->S; ++s) {
            const float *ray = rays + 6 * r;
            float z = lmref_sample_z(g, ray, s), pt[3];
            lmref_point(ray, z, pt);
            int ok = inside_aabb(g, pt);
            if (ok && g->vol) ok = lmref_alpha_lookup(g, pt) > g->vol_thre;
            valid[r * g->S + s] = (uint8_t)ok;
            if (zout) zout[r * g->S + s] = z;
            cnt += ok;
        }
    return cnt;
}

/* ------------------------------------------------------------------------------------
 * features (reference NCHW layout)
 * ---------------------------------------------------------------------------------- */
typedef struct {
    const float *plane; /* [C,H,W] */
    const float *line;  /* [C,Len]  */
    int C, H, W, Len;
    int ax0, ax1, axl;  /* plane x-coordinate axis, y-coordinate axis, line axis */
} lmref_plane;

static float unnorm(float c, int size) { return ((c + 1.0f) / 2.0f) * (float)(size - 1); }

float lmref_bilinear(const float *img, int H, int W, float cx, float cy) {
    float ix = unnorm(cx, W), iy = unnorm(cy, H);
    float fx = floorf(ix), fy = floorf(iy);
    long x0 = (long)fx, y0 = (long)fy;
    float wx1 = ix - fx, wx0 = (fx + 1.0f) - ix, wy1 = iy - fy, wy0 = (fy + 1.0f) - iy;
    float out = 0.0f;
    if (x0 >= 0 && x0 < W && y0 >= 0 && y0 < H) out += img[y0 * W + x0] * (wx0 * wy0);
    if (x0 + 1 >= 0 && x0 + 1 < W && y0 >= 0 && y0 < H) out += img[y0 * W + x0 + 1] * (wx1 * wy0);
    if (x0 >= 0 && x0 < W && y0 + 1 >= 0 && y0 + 1 < H) out += img[(y0 + 1) * W + x0] * (wx0 * wy1);
    if (x0 + 1 >= 0 && x0 + 1 < W && y0 + 1 >= 0 && y0 + 1 < H) out += img[(y0 + 1) * W + x0 + 1] * (wx1 * wy1);
    return out;
}

float lmref_linear(const float *vec, int Len, float c) {
    /* a [Len,1] image sampled at (x=0, y=c): the x weights are 1 (west) and 0 (east). */
    float i = unnorm(c, Len);
    float f = floorf(i);
    long i0 = (long)f;
    float w1 = i - f, w0 = (f + 1.0f) - i;
    float out = 0.0f;
    if (i0 >= 0 && i0 < Len) out += vec[i0] * w0;
    if (i0 + 1 >= 0 && i0 + 1 < Len) out += vec[i0 + 1] * w1;
    return out;
}

/* products[c] = plane_c(x) * line_c(x) for one plane; returns their sum */
float lmref_plane_products(const lmref_plane *p, const float *xyz, float *products) {
    float sum = 0.0f;
    for (int c = 0; c < p->C; ++c) {
        float pv = lmref_bilinear(p->plane + (size_t)c * p->H * p->W, p->H, p->W, xyz[p->ax0], xyz[p->ax1]);
        float lv = lmref_linear(p->line + (size_t)c * p->Len, p->Len, xyz[p->axl]);
        float v = pv * lv;
        if (products) products[c] = v;
        sum += v;
    }
    return sum;
}

typedef struct {
    lmref_geom geom;
    int n_planes;
    const lmref_plane *density; /* [n_planes] */
    const lmref_plane *app;     /* [n_planes] */
    int app_dim;                /* 27 */
    const float *basis;         /* [app_dim, n_planes*C_a] */
    int view_pe, fea_pe, hidden;
    const float *w1, *b1, *w2, *b2, *w3, *b3; /* biases may be NULL */
    int softplus;
    float density_shift, distance_scale, weight_thres;
    int white_bg;
    const float *basis_den; /* NULL, or [n_planes*C_d]: density = relu(sum w*product) (gridnerf_sequential.py:819-822) */
    const float *latent;    /* NULL, or the frame's appearance embedding row (gridnerf_sequential.py:429-437) */
    int latent_dim;
} lmref_model;

static void pe(const float *x, int n, int F, float *sin_out, float *cos_out) {
    for (int d = 0; d < n; ++d)
        for (int f = 0; f < F; ++f) {
            float q = x[d] * (float)(1 << f);
            sin_out[d * F + f] = sinf(q);
            cos_out[d * F + f] = cosf(q);
        }
}

static void linear(const float *w, const float *b, const float *x, int in, int out, float *y, int relu) {
    for (int o = 0; o < out; ++o) {
        double acc = b ? b[o] : 0.0;
        for (int i = 0; i < in; ++i) acc += (double)w[(size_t)o * in + i] * x[i];
        float v = (float)acc;
        y[o] = (relu && v < 0.0f) ? 0.0f : v;
    }
}

int lmref_mlp_in_dim(const lmref_model *m) {
    return m->app_dim + (m->latent ? m->latent_dim : 0) + 3 + 2 * m->fea_pe * m->app_dim + 2 * m->view_pe * 3;
}

/* rgb[3] of one sample from its app features and view direction */
void lmref_colour(const lmref_model *m, const float *feat, const float *view, float *rgb) {
    float in[512], h1[512], h2[512], o[3];
    int n = 0, A = m->app_dim;
    memcpy(in + n, feat, sizeof(float) * A); n += A;
    if (m->latent) { memcpy(in + n, m->latent, sizeof(float) * m->latent_dim); n += m->latent_dim; }
    memcpy(in + n, view, sizeof(float) * 3); n += 3;
    pe(feat, A, m->fea_pe, in + n, in + n + A * m->fea_pe); n += 2 * A * m->fea_pe;
    pe(view, 3, m->view_pe, in + n, in + n + 3 * m->view_pe); n += 2 * 3 * m->view_pe;
    linear(m->w1, m->b1, in, n, m->hidden, h1, 1);
    linear(m->w2, m->b2, h1, m->hidden, m->hidden, h2, 1);
    linear(m->w3, m->b3, h2, m->hidden, 3, o, 0);
    for (int k = 0; k < 3; ++k) rgb[k] = 1.0f / (1.0f + expf(-o[k]));
}

static void normalise(const lmref_geom *g, const float *pt, float *q) {
    for (int k = 0; k < 3; ++k) {
        float d = pt[k] - g->aabb[k];
        float mm = d * g->inv_aabb[k];
        q[k] = mm - 1.0f;
    }
}

/* Whole render of N rays.  Outputs: rgb_map[N,3], depth_map[N]; optional per-sample
 * valid[N*S], sigma[N*S], weight[N*S], app_mask[N*S]. */
void lmref_render(const lmref_model *m, const float *rays, long N, float *rgb_map, float *depth_map,
                  uint8_t *valid_out, float *sigma_out, float *weight_out, uint8_t *app_out) {
    const lmref_geom *g = &m->geom;
    int S = g->S;
    float *z = (float *)malloc(sizeof(float) * S);
    float *sigma = (float *)malloc(sizeof(float) * S);
    float *prod = (float *)malloc(sizeof(float) * 4096);
    float *feat = (float *)malloc(sizeof(float) * 64);
    for (long r = 0; r < N; ++r) {
        const float *ray = rays + 6 * r;
        for (int s = 0; s < S; ++s) {
            float pt[3], q[3];
            z[s] = lmref_sample_z(g, ray, s);
            lmref_point(ray, z[s], pt);
            int ok = inside_aabb(g, pt);
            if (ok && g->vol) ok = lmref_alpha_lookup(g, pt) > g->vol_thre;
            sigma[s] = 0.0f;
            if (ok) {
                normalise(g, pt, q);
                float f = 0.0f;
                if (m->basis_den) {
                    int Cd = m->density[0].C;
                    for (int k = 0; k < m->n_planes; ++k) {
                        lmref_plane_products(&m->density[k], q, prod);
                        for (int c = 0; c < Cd; ++c) f += m->basis_den[k * Cd + c] * prod[c];
                    }
                    f = f > 0.0f ? f : 0.0f;
                } else
                    for (int k = 0; k < m->n_planes; ++k) f += lmref_plane_products(&m->density[k], q, NULL);
                if (m->softplus) {
                    float x = f + m->density_shift;
                    sigma[s] = x > 20.0f ? x : log1pf(expf(x));
                } else
                    sigma[s] = f > 0.0f ? f : 0.0f;
            }
            if (valid_out) valid_out[r * S + s] = (uint8_t)ok;
            if (sigma_out) sigma_out[r * S + s] = sigma[s];
        }
        float T = 1.0f, acc = 0.0f, depth = 0.0f, col[3] = {0, 0, 0};
        for (int s = 0; s < S; ++s) {
            float dist = (s + 1 < S) ? (z[s + 1] - z[s]) : 0.0f;
            float alpha = 1.0f - expf(-sigma[s] * (dist * m->distance_scale));
            float w = alpha * T;
            T = T * ((1.0f - alpha) + 1e-10f);
            int is_app = w > m->weight_thres;
            if (weight_out) weight_out[r * S + s] = w;
            if (app_out) app_out[r * S + s] = (uint8_t)is_app;
            acc += w;
            depth += w * z[s];
            if (is_app) {
                float pt[3], q[3], rgb[3];
                lmref_point(ray, z[s], pt);
                normalise(g, pt, q);
                int Ca = m->app[0].C, K = m->n_planes * Ca;
                for (int k = 0; k < m->n_planes; ++k) lmref_plane_products(&m->app[k], q, prod + k * Ca);
                linear(m->basis, NULL, prod, K, m->app_dim, feat, 0);
                lmref_colour(m, feat, ray + 3, rgb);
                for (int k = 0; k < 3; ++k) col[k] += w * rgb[k];
            }
        }
        for (int k = 0; k < 3; ++k) {
            float v = col[k];
            if (m->white_bg) v = v + (1.0f - acc);
            rgb_map[3 * r + k] = v < 0.0f ? 0.0f : (v > 1.0f ? 1.0f : v);
        }
        depth_map[r] = depth;
    }
    free(z); free(sigma); free(prod); free(feat);
}
