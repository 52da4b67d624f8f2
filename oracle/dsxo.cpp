/*
 * dsxo.cpp — CPU ORACLE (test infrastructure only; see dsxo.h).
 *
 * Serial restatement of the reference kernels' arithmetic.  Build WITHOUT fast-math and
 * with -ffp-contract=off: the integer outputs (radii, tile counts, keys) depend on every
 * float operation being a separately rounded IEEE-754 binary32 operation in the order the
 * reference writes them.  Two deliberate, documented deviations from the reference text:
 *   * rsqrtf(x) (an approximate GPU instruction, rasterizer_kernels.cu:568,623) is
 *     evaluated as 1.0f / sqrtf(x) so that results are reproducible;
 *   * float -> int conversion saturates and maps NaN to 0, which is what the GPU
 *     conversion instruction does (plain C leaves both undefined).
 * With -fopenmp the per-Gaussian and per-tile loops run in parallel (CPU baseline);
 * without it everything is serial and deterministic (parity oracle).
 */
#include "dsxo.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace
{

constexpr int TILE = 16; /* rasterizer_kernels.cuh:6 */

/* ---------------------------------------------------------------------------------- */
/* helpers                                                                             */
/* ---------------------------------------------------------------------------------- */

inline int32_t f2i(float x)
{
    if(x != x)
        return 0;
    if(x >= 2147483648.0f)
        return INT32_MAX;
    if(x <= -2147483648.0f)
        return INT32_MIN;
    return (int32_t)x;
}

inline float rsqrt_exact(float x)
{
    return 1.0f / sqrtf(x);
}

inline int tiles_x(const dsxo_settings* s)
{
    return (s->image_width + TILE - 1) / TILE;
}
inline int tiles_y(const dsxo_settings* s)
{
    return (s->image_height + TILE - 1) / TILE;
}

struct Rect
{
    int sx, ex, sy, ey;
};

/* rasterizer_kernels.cu:239-247 and :286-292 (identical text) */
inline Rect tile_rect(float px, float py, int32_t radius, const dsxo_settings* s)
{
    const float cx = px / (float)TILE;
    const float cy = py / (float)TILE;
    const float dx = radius / (float)TILE;
    const float dy = radius / (float)TILE;
    const int tx = tiles_x(s);
    const int ty = tiles_y(s);
    Rect r;
    r.sx = std::min(std::max(0, f2i(cx - dx)), tx);
    r.ex = std::min(std::max(0, f2i(cx + dx + 1)), tx);
    r.sy = std::min(std::max(0, f2i(cy - dy)), ty);
    r.ey = std::min(std::max(0, f2i(cy + dy + 1)), ty);
    return r;
}

/* rasterizer_kernels.cu:615-659 */
inline void calc_cov3d(const float* sc, const float* q, float mod, float* out)
{
    float r = q[0], x = q[1], y = q[2], z = q[3];
    const float inv_norm = rsqrt_exact(r * r + x * x + y * y + z * z);
    r = r * inv_norm;
    x = x * inv_norm;
    y = y * inv_norm;
    z = z * inv_norm;
    const float s0 = sc[0] * mod, s1 = sc[1] * mod, s2 = sc[2] * mod;

    const float r00 = 1.0f - 2.0f * (y * y + z * z);
    const float r01 = 2.0f * (x * y - r * z);
    const float r02 = 2.0f * (x * z + r * y);
    const float r10 = 2.0f * (x * y + r * z);
    const float r11 = 1.0f - 2.0f * (x * x + z * z);
    const float r12 = 2.0f * (y * z - r * x);
    const float r20 = 2.0f * (x * z - r * y);
    const float r21 = 2.0f * (y * z + r * x);
    const float r22 = 1.0f - 2.0f * (x * x + y * y);

    const float m00 = s0 * r00, m01 = s1 * r01, m02 = s2 * r02;
    const float m10 = s0 * r10, m11 = s1 * r11, m12 = s2 * r12;
    const float m20 = s0 * r20, m21 = s1 * r21, m22 = s2 * r22;

    out[0] = m00 * m00 + m01 * m01 + m02 * m02;
    out[1] = m00 * m10 + m01 * m11 + m02 * m12;
    out[2] = m00 * m20 + m01 * m21 + m02 * m22;
    out[3] = m10 * m10 + m11 * m11 + m12 * m12;
    out[4] = m10 * m20 + m11 * m21 + m12 * m22;
    out[5] = m20 * m20 + m21 * m21 + m22 * m22;
}

/* rasterizer_kernels.cu:7-24 */
inline int32_t in_frustum(const float* m, const float* P)
{
    const float inv_w = 1.f / (P[12] * m[0] + P[13] * m[1] + P[14] * m[2] + P[15]);
    const float x = inv_w * (P[0] * m[0] + P[1] * m[1] + P[2] * m[2] + P[3]);
    const float y = inv_w * (P[4] * m[0] + P[5] * m[1] + P[6] * m[2] + P[7]);
    const float z = inv_w * (P[8] * m[0] + P[9] * m[1] + P[10] * m[2] + P[11]);
    const float limits = 1.f;
    return x > -limits && x < limits && y > -limits && y < limits && z > 0.1f;
}

/* rasterizer_kernels.cu:174-231 */
inline void calc_cov2d(float fx, float fy, float tanfovx, float tanfovy, const float* v /*view pos*/,
                       const float* V /*view matrix*/, const float* c3, float* out)
{
    const float limx = 1.3f * tanfovx;
    const float limy = 1.3f * tanfovy;
    const float txtz = v[0] / v[2];
    const float tytz = v[1] / v[2];
    const float t[3] = {fminf(limx, fmaxf(-limx, txtz)) * v[2], fminf(limy, fmaxf(-limy, tytz)) * v[2], v[2]};

    const float J[3][3] = {{fx / t[2], 0, -(fx * t[0]) / (t[2] * t[2])},
                           {0, fy / t[2], -(fy * t[1]) / (t[2] * t[2])},
                           {0, 0, 0}};
    const float W[3][3] = {{V[0], V[4], V[8]}, {V[1], V[5], V[9]}, {V[2], V[6], V[10]}};

    float T[3][3] = {{0, 0, 0}, {0, 0, 0}, {0, 0, 0}};
    for(int i = 0; i < 3; ++i)
        for(int j = 0; j < 3; ++j)
            for(int k = 0; k < 3; ++k)
                T[i][j] += W[i][k] * J[j][k];

    const float Vrk[3][3] = {{c3[0], c3[1], c3[2]}, {c3[1], c3[3], c3[4]}, {c3[2], c3[4], c3[5]}};
    float cov[2][2] = {{0, 0}, {0, 0}};
    float temp[3][3] = {{0, 0, 0}, {0, 0, 0}, {0, 0, 0}};
    for(int i = 0; i < 3; ++i)
        for(int j = 0; j < 3; ++j)
            for(int k = 0; k < 3; ++k)
                temp[i][j] += T[k][i] * Vrk[k][j];
    for(int i = 0; i < 2; ++i)
        for(int j = 0; j < 2; ++j)
            for(int k = 0; k < 3; ++k)
                cov[i][j] += temp[i][k] * T[k][j];

    out[0] = cov[0][0] + 0.3f;
    out[1] = cov[0][1];
    out[2] = cov[1][1] + 0.3f;
}

/* rasterizer_kernels.cu:163-172 */
inline int32_t calc_radius(const float* c2, int32_t mask)
{
    const float det = c2[0] * c2[2] - c2[1] * c2[1];
    const float mid = 0.5f * (c2[0] + c2[2]);
    const float diff = mid * mid - det;
    const float lambda1 = mid + sqrtf(fmaxf(0.1f, diff));
    const float lambda2 = mid - sqrtf(fmaxf(0.1f, diff));
    const float keep = (float)(int)(det > 1e-6f && mask > 0);
    return f2i(ceilf(3.0f * sqrtf(fmaxf(lambda1, lambda2))) * keep);
}

/* rasterizer_kernels.cu:433-613 */
inline void sh_to_rgb(int deg, const float* f, const float* mean, const float* campos, float* out)
{
    float rx = 0.0f, ry = 0.0f, rz = 0.0f;
    const float C0 = 0.28209479177387814f;
    rx += C0 * f[0];
    ry += C0 * f[1];
    rz += C0 * f[2];
    if(deg >= 1)
    {
        /* calculate_viewdir :565-571 */
        const float dx = mean[0] - campos[0], dy = mean[1] - campos[1], dz = mean[2] - campos[2];
        const float inv_norm = rsqrt_exact(dx * dx + dy * dy + dz * dz);
        const float vx = dx * inv_norm, vy = dy * inv_norm, vz = dz * inv_norm;

        const float C1 = 0.4886025119029199f;
        rx += C1 * (-vy * f[3] + vz * f[6] - vx * f[9]);
        ry += C1 * (-vy * f[4] + vz * f[7] - vx * f[10]);
        rz += C1 * (-vy * f[5] + vz * f[8] - vx * f[11]);
        if(deg >= 2)
        {
            const float xx = vx * vx, yy = vy * vy, zz = vz * vz;
            const float xy = vx * vy, xz = vx * vz, yz = vy * vz;
            const float C2_0 = 1.0925484305920792f, C2_1 = -1.0925484305920792f, C2_2 = 0.31539156525252005f,
                        C2_3 = -1.0925484305920792f, C2_4 = 0.5462742152960396f;
            rx += C2_0 * xy * f[12] + C2_1 * yz * f[15] + C2_2 * (2.0f * zz - xx - yy) * f[18] + C2_3 * xz * f[21] +
                  C2_4 * (xx - yy) * f[24];
            ry += C2_0 * xy * f[13] + C2_1 * yz * f[16] + C2_2 * (2.0f * zz - xx - yy) * f[19] + C2_3 * xz * f[22] +
                  C2_4 * (xx - yy) * f[25];
            rz += C2_0 * xy * f[14] + C2_1 * yz * f[17] + C2_2 * (2.0f * zz - xx - yy) * f[20] + C2_3 * xz * f[23] +
                  C2_4 * (xx - yy) * f[26];
            if(deg >= 3)
            {
                const float C3_0 = -0.5900435899266435f, C3_1 = 2.890611442640554f, C3_2 = -0.4570457994644658f,
                            C3_3 = 0.3731763325901154f, C3_4 = -0.4570457994644658f, C3_5 = 1.445305721320277f,
                            C3_6 = -0.5900435899266435f;
                for(int c = 0; c < 3; ++c)
                {
                    const float v = C3_0 * vy * (3 * xx - yy) * f[27 + c] + C3_1 * xy * vz * f[30 + c] +
                                    C3_2 * vy * (4 * zz - xx - yy) * f[33 + c] +
                                    C3_3 * vz * (2 * zz - 3 * xx - 3 * yy) * f[36 + c] +
                                    C3_4 * vx * (4 * zz - xx - yy) * f[39 + c] + C3_5 * vz * (xx - yy) * f[42 + c] +
                                    C3_6 * vx * (xx - 3 * yy) * f[45 + c];
                    if(c == 0)
                        rx += v;
                    else if(c == 1)
                        ry += v;
                    else
                        rz += v;
                }
            }
        }
    }
    out[0] = fmaxf(rx + 0.5f, 0.0f);
    out[1] = fmaxf(ry + 0.5f, 0.0f);
    out[2] = fmaxf(rz + 0.5f, 0.0f);
}

/* ---------------------------------------------------------------------------------- */
/* blend forward, templated on the scalar so a double instance serves finite differences */
/* ---------------------------------------------------------------------------------- */

inline float exp_s(float x)
{
    return expf(x);
}
inline double exp_s(double x)
{
    return exp(x);
}

template <typename S> inline S rel_margin(S value, S threshold)
{
    const S d = value > threshold ? value - threshold : threshold - value;
    const S m = threshold > 0 ? threshold : S(1);
    return d / m;
}

} // namespace

/* ---------------------------------------------------------------------------------- */
/* C ABI                                                                               */
/* ---------------------------------------------------------------------------------- */

extern "C" int dsxo_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

extern "C" void dsxo_project_fwd(const dsxo_settings* s, int64_t n, const float* means3d, const float* scales,
                                 const float* quats, const float* shs, const float* cov3d_precomp,
                                 const float* colors_precomp, float* means2d, float* conic, float* rgb,
                                 int32_t* radii, int32_t* tiles_touched, float* cov3d)
{
    /* rasterizer_torch.cu:120-122,144-147 */
    const int max_coeff = (s->max_sh_degree + 1) * (s->max_sh_degree + 1);
    const float focal_y = s->image_height / (2 * s->tanfovy);
    const float focal_x = s->image_width / (2 * s->tanfovx);
    const float c_x = s->image_width / 2.0f;
    const float c_y = s->image_height / 2.0f;

#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for(int64_t i = 0; i < n; ++i)
    {
        float c3[6];
        if(cov3d_precomp)
            memcpy(c3, cov3d_precomp + 6 * i, sizeof(c3));
        else
            calc_cov3d(scales + 3 * i, quats + 4 * i, s->scale_modifier, c3);
        memcpy(cov3d + 6 * i, c3, sizeof(c3));

        const float* m = means3d + 3 * i;
        if(colors_precomp)
            memcpy(rgb + 3 * i, colors_precomp + 3 * i, 3 * sizeof(float));
        else
            sh_to_rgb(s->sh_degree, shs + (int64_t)max_coeff * 3 * i, m, s->campos, rgb + 3 * i);

        int32_t mask = in_frustum(m, s->proj);
        /* project_point :325-330 */
        const float* V = s->view;
        float v[3] = {V[0] * m[0] + V[1] * m[1] + V[2] * m[2] + V[3], V[4] * m[0] + V[5] * m[1] + V[6] * m[2] + V[7],
                      V[8] * m[0] + V[9] * m[1] + V[10] * m[2] + V[11]};
        float c2[3];
        calc_cov2d(focal_x, focal_y, s->tanfovx, s->tanfovy, v, V, c3, c2);
        /* project_to_image :332-337 */
        const float z_inv = 1.f / (v[2] + 1e-6f);
        const float px = focal_x * v[0] * z_inv + c_x;
        const float py = focal_y * v[1] * z_inv + c_y;

        const int32_t radius = calc_radius(c2, mask);
        /* calculate_sizes :233-250 */
        const Rect r = tile_rect(px, py, radius, s);
        const int32_t count = (r.ex - r.sx) * (r.ey - r.sy) * (radius > 0);

        radii[i] = radius;
        tiles_touched[i] = count;
        /* calculate_conic :49-55 */
        const float det = c2[0] * c2[2] - c2[1] * c2[1];
        const float det_inv = 1.0f / (det + 1e-6f);
        conic[3 * i + 0] = c2[2] * det_inv;
        conic[3 * i + 1] = -c2[1] * det_inv;
        conic[3 * i + 2] = c2[0] * det_inv;
        means2d[3 * i + 0] = px;
        means2d[3 * i + 1] = py;
        means2d[3 * i + 2] = v[2];
    }
}

extern "C" int64_t dsxo_offsets(int64_t n, const int32_t* tiles_touched, int32_t* offsets)
{
    int32_t run = 0;
    for(int64_t i = 0; i < n; ++i)
    {
        offsets[i] = run;
        run += tiles_touched[i];
    }
    /* rasterizer_torch.cu:99-104: total = exclusive prefix of the LAST Gaussian */
    return n > 0 ? offsets[n - 1] : 0;
}

extern "C" void dsxo_emit_keys(const dsxo_settings* s, int64_t n, int64_t k, const float* means2d,
                               const int32_t* radii, const int32_t* offsets, int64_t* keys, int32_t* values)
{
    const int tpw = tiles_x(s);
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 4096)
#endif
    for(int64_t i = 0; i < n; ++i)
    {
        /* rasterizer_kernels.cu:275-276 */
        const int64_t start = offsets[i];
        const int64_t end = (i + 1) < n ? offsets[i + 1] : k;
        if(end - start <= 0)
            continue;
        const float px = means2d[3 * i], py = means2d[3 * i + 1];
        int32_t depth_bits;
        memcpy(&depth_bits, means2d + 3 * i + 2, 4);
        const int64_t depth = (int64_t)depth_bits; /* :283, sign-extending */
        const Rect r = tile_rect(px, py, radii[i], s);
        int64_t local = start;
        for(int ty = r.sy; ty < r.ey; ++ty)
            for(int tx = r.sx; tx < r.ex; ++tx, ++local)
            {
                const int64_t tile_index = ty * tpw + tx;
                keys[local] = (int64_t)((uint64_t)tile_index << 32) | depth;
                values[local] = (int32_t)i;
            }
    }
}

extern "C" void dsxo_sort_pairs(int64_t k, int64_t* keys, int32_t* values)
{
    if(k <= 0)
        return;
#ifdef _OPENMP
    /* parallel LSD radix sort (stable), 8-bit digits over the unsigned image of the key;
     * keys emitted by this pipeline are non-negative so this equals the signed order */
    bool nonneg = true;
    for(int64_t i = 0; i < k; ++i)
        if(keys[i] < 0)
        {
            nonneg = false;
            break;
        }
    if(nonneg)
    {
        std::vector<int64_t> k2(k);
        std::vector<int32_t> v2(k);
        int64_t* ka = keys;
        int64_t* kb = k2.data();
        int32_t* va = values;
        int32_t* vb = v2.data();
        uint64_t all_or = 0;
#pragma omp parallel for reduction(| : all_or)
        for(int64_t i = 0; i < k; ++i)
            all_or |= (uint64_t)keys[i];
        const int nt = omp_get_max_threads();
        std::vector<int64_t> hist((size_t)nt * 256);
        for(int shift = 0; shift < 64; shift += 8)
        {
            if(((all_or >> shift) & 0xff) == 0 && (all_or >> shift) == 0)
                break;
            std::fill(hist.begin(), hist.end(), 0);
#pragma omp parallel num_threads(nt)
            {
                const int t = omp_get_thread_num();
                const int64_t lo = k * t / nt, hi = k * (t + 1) / nt;
                int64_t* h = hist.data() + (size_t)t * 256;
                for(int64_t i = lo; i < hi; ++i)
                    h[((uint64_t)ka[i] >> shift) & 0xff]++;
#pragma omp barrier
#pragma omp single
                {
                    int64_t run = 0;
                    for(int d = 0; d < 256; ++d)
                        for(int tt = 0; tt < nt; ++tt)
                        {
                            const int64_t c = hist[(size_t)tt * 256 + d];
                            hist[(size_t)tt * 256 + d] = run;
                            run += c;
                        }
                }
                for(int64_t i = lo; i < hi; ++i)
                {
                    const int64_t dst = h[((uint64_t)ka[i] >> shift) & 0xff]++;
                    kb[dst] = ka[i];
                    vb[dst] = va[i];
                }
            }
            std::swap(ka, kb);
            std::swap(va, vb);
        }
        if(ka != keys)
        {
            memcpy(keys, ka, k * sizeof(int64_t));
            memcpy(values, va, k * sizeof(int32_t));
        }
        return;
    }
#endif
    std::vector<int64_t> perm(k);
    std::iota(perm.begin(), perm.end(), (int64_t)0);
    std::stable_sort(perm.begin(), perm.end(), [&](int64_t a, int64_t b) { return keys[a] < keys[b]; });
    std::vector<int64_t> k2(k);
    std::vector<int32_t> v2(k);
    for(int64_t i = 0; i < k; ++i)
    {
        k2[i] = keys[perm[i]];
        v2[i] = values[perm[i]];
    }
    memcpy(keys, k2.data(), k * sizeof(int64_t));
    memcpy(values, v2.data(), k * sizeof(int32_t));
}

extern "C" void dsxo_tile_ranges(int64_t k, const int64_t* keys, int32_t num_tiles, int32_t* ranges)
{
    /* rasterizer_torch.cu:31-32 */
    for(int32_t i = 0; i <= num_tiles; ++i)
        ranges[i] = 0;
    ranges[num_tiles] = (int32_t)k;
    /* rasterizer_kernels.cu:313-322 */
    for(int64_t i = 0; i + 1 < k; ++i)
    {
        const int32_t cur = (int32_t)(keys[i] >> 32);
        const int32_t nxt = (int32_t)(keys[i + 1] >> 32);
        if(cur != nxt)
            ranges[cur + 1] = (int32_t)(i + 1);
    }
    /* rasterizer_torch.cu:39 */
    int32_t run = ranges[0];
    for(int32_t i = 0; i <= num_tiles; ++i)
    {
        run = std::max(run, ranges[i]);
        ranges[i] = run;
    }
}

namespace
{

/* rasterizer_kernels.cu:341-431 for one pixel; entries [start,end) of the tile's run.
 * Returns nothing; writes C[3], T, last index; counts pairs. */
template <typename S>
inline void blend_pixel(int x, int y, int32_t start, int32_t end, const int32_t* ids, const S* xy, int xy_stride,
                        const S* conic, const S* rgb, const S* opac, S alpha_clamp, S* C, S* T_out, int32_t* last,
                        S* margin, int64_t* walked, int64_t* applied)
{
    S c0 = 0, c1 = 0, c2 = 0, T = 1;
    int32_t curr = 0;
    S mg = S(1e30);
    int64_t nw = 0, na = 0;
    const S alpha_threshold = S(1.0f / 255.0f);
    for(int32_t e = start; e < end; ++e)
    {
        const int32_t g = ids[e];
        ++nw;
        const S dx = x + S(0.5f) - xy[(int64_t)xy_stride * g];
        const S dy = y + S(0.5f) - xy[(int64_t)xy_stride * g + 1];
        const S ca = conic[3 * (int64_t)g], cb = conic[3 * (int64_t)g + 1], cc = conic[3 * (int64_t)g + 2];
        const S power = S(-0.5f) * (ca * dx * dx + cc * dy * dy) - cb * dx * dy;
        const S raw = opac[g] * exp_s(power);
        const S alpha = raw < alpha_clamp ? raw : alpha_clamp;
        if(margin)
        {
            /* sign of power: distance from 0 relative to the size of its terms */
            const S pa = power >= 0 ? power : -power;
            const S t1 = ca * dx * dx, t2 = cc * dy * dy, t3 = cb * dx * dy;
            const S mag = S(0.5f) * ((t1 < 0 ? -t1 : t1) + (t2 < 0 ? -t2 : t2)) + (t3 < 0 ? -t3 : t3);
            mg = std::min(mg, mag > 0 ? pa / mag : S(0));
            /* alpha against 1/255: a rounding difference in the exponent (contraction, term
             * order) is an absolute error of a few mag * 2^-24 there, i.e. a relative one in alpha:
             * the distance from the threshold is counted less a guard band of mag * 1e-6 */
            mg = std::min(mg, rel_margin(raw, alpha_threshold) - mag * S(1e-6));
        }
        if(power >= 0 || alpha < alpha_threshold)
            continue;
        const S Tn = (S(1) - alpha) * T;
        if(margin)
            mg = std::min(mg, rel_margin(Tn, S(0.0001f)));
        if(!(Tn >= S(0.0001f)))
            break; /* is_ok = false: nothing later is evaluated (:386,401) */
        const S vis = alpha * T;
        c0 += vis * rgb[3 * (int64_t)g];
        c1 += vis * rgb[3 * (int64_t)g + 1];
        c2 += vis * rgb[3 * (int64_t)g + 2];
        T = Tn;
        curr = e;
        ++na;
    }
    C[0] = c0;
    C[1] = c1;
    C[2] = c2;
    *T_out = T;
    *last = curr;
    if(margin)
        *margin = mg;
    if(walked)
        *walked = nw;
    if(applied)
        *applied = na;
}

} // namespace

extern "C" void dsxo_blend_fwd(const dsxo_settings* s, const int32_t* ranges, const int32_t* sorted_ids,
                               const float* means2d, const float* conic, const float* rgb, const float* opacities,
                               float* image, float* final_T, int32_t* final_idx, float* margin,
                               dsxo_counters* counters)
{
    const int W = s->image_width, H = s->image_height;
    const int tx = tiles_x(s);
    int64_t walked = 0, applied = 0;
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 16) reduction(+ : walked, applied)
#endif
    for(int y = 0; y < H; ++y)
        for(int x = 0; x < W; ++x)
        {
            const int tile = (y / TILE) * tx + (x / TILE);
            float C[3], T, mg;
            int32_t last;
            int64_t nw, na;
            blend_pixel<float>(x, y, ranges[tile], ranges[tile + 1], sorted_ids, means2d, 3, conic, rgb, opacities,
                               0.999f, C, &T, &last, margin ? &mg : nullptr, &nw, &na);
            const int64_t p = (int64_t)y * W + x;
            image[3 * p] = C[0];
            image[3 * p + 1] = C[1];
            image[3 * p + 2] = C[2];
            final_T[p] = T;
            final_idx[p] = last;
            if(margin)
                margin[p] = mg;
            walked += nw;
            applied += na;
        }
    if(counters)
    {
        counters->pairs_fwd = walked;
        counters->pairs_fwd_applied = applied;
    }
}

extern "C" void dsxo_blend_bwd(const dsxo_settings* s, int64_t n, const int32_t* ranges, const int32_t* sorted_ids,
                               const float* means2d, const float* conic, const float* rgb, const float* opacities,
                               const float* final_T, const int32_t* final_idx, const float* v_out,
                               const float* v_out_alpha, float* v_xy, float* v_conic, float* v_rgb, float* v_opacity,
                               float* g_margin, dsxo_counters* counters)
{
    dsxo_blend_bwd_ex(s, n, ranges, sorted_ids, means2d, conic, rgb, opacities, final_T, final_idx, v_out, v_out_alpha,
                      v_xy, v_conic, v_rgb, v_opacity, g_margin, counters, nullptr);
}

extern "C" void dsxo_blend_bwd_ex(const dsxo_settings* s, int64_t n, const int32_t* ranges, const int32_t* sorted_ids,
                                  const float* means2d, const float* conic, const float* rgb, const float* opacities,
                                  const float* final_T, const int32_t* final_idx, const float* v_out,
                                  const float* v_out_alpha, float* v_xy, float* v_conic, float* v_rgb,
                                  float* v_opacity, float* g_margin, dsxo_counters* counters, float* abs_sums)
{
    const int W = s->image_width, H = s->image_height;
    const int ntx = tiles_x(s), nty = tiles_y(s);
    std::vector<double> acc((size_t)n * 9, 0.0);
    /* sums of the absolute values of the elementary terms of every accumulation: the scale
     * against which a differently ordered float summation may be judged */
    std::vector<double> acc_abs(abs_sums ? (size_t)n * 9 : 0, 0.0);
    if(g_margin)
        for(int64_t i = 0; i < n; ++i)
            g_margin[i] = 1e30f;
    int64_t walked = 0, valid_pairs = 0;
    const float bg0 = s->bg[0], bg1 = s->bg[1], bg2 = s->bg[2];

#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) reduction(+ : walked, valid_pairs)
#endif
    for(int tile = 0; tile < ntx * nty; ++tile)
    {
        const int tile_x0 = (tile % ntx) * TILE, tile_y0 = (tile / ntx) * TILE;
        const int32_t r0 = ranges[tile], r1 = ranges[tile + 1];
        float T[TILE * TILE], Tfin[TILE * TILE], buf[TILE * TILE][3];
        int32_t bin_final[TILE * TILE];
        bool inside[TILE * TILE];
        int32_t max_final = -1;
        for(int t = 0; t < TILE * TILE; ++t)
        {
            const int x = tile_x0 + (t % TILE), y = tile_y0 + (t / TILE);
            inside[t] = x < W && y < H;
            buf[t][0] = buf[t][1] = buf[t][2] = 0.f;
            if(inside[t])
            {
                const int64_t p = (int64_t)y * W + x;
                Tfin[t] = T[t] = final_T[p];
                bin_final[t] = final_idx[p];
                max_final = std::max(max_final, bin_final[t]);
            }
            else
            {
                Tfin[t] = T[t] = 0.f;
                bin_final[t] = 0;
            }
        }
        /* back to front: backward.cu:87-112 */
        for(int32_t e = std::min(r1 - 1, max_final); e >= r0; --e)
        {
            const int32_t g = sorted_ids[e];
            const float mx = means2d[3 * (int64_t)g], my = means2d[3 * (int64_t)g + 1];
            const float opac = opacities[g];
            const float ca = conic[3 * (int64_t)g], cb = conic[3 * (int64_t)g + 1], cc = conic[3 * (int64_t)g + 2];
            const float cr = rgb[3 * (int64_t)g], cg = rgb[3 * (int64_t)g + 1], cbl = rgb[3 * (int64_t)g + 2];
            double l[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
            double la[9] = {0, 0, 0, 0, 0, 0, 0, 0, 0};
            float gm = 1e30f;
            bool any = false;
            for(int t = 0; t < TILE * TILE; ++t)
            {
                if(!inside[t] || e > bin_final[t])
                    continue;
                ++walked;
                const int x = tile_x0 + (t % TILE), y = tile_y0 + (t / TILE);
                const float px = (float)x + 0.5f, py = (float)y + 0.5f;
                const float dx = mx - px, dy = my - py;
                /* :127-134 */
                const float sigma = 0.5f * (ca * dx * dx + cc * dy * dy) + cb * dx * dy;
                const float vis = expf(-sigma);
                const float raw = opac * vis;
                const float alpha = fminf(0.99f, raw);
                {
                    const float mag = 0.5f * (fabsf(ca * dx * dx) + fabsf(cc * dy * dy)) + fabsf(cb * dx * dy);
                    gm = std::min(gm, mag > 0 ? fabsf(sigma) / mag : 0.f);
                    /* as in the forward: the exponent's rounding error scales with mag */
                    gm = std::min(gm, rel_margin(raw, 1.f / 255.f) - mag * 1e-6f);
                }
                if(sigma < 0.f || alpha < 1.f / 255.f)
                    continue;
                ++valid_pairs;
                any = true;
                const int64_t p = (int64_t)y * W + x;
                const float vo0 = v_out[3 * p], vo1 = v_out[3 * p + 1], vo2 = v_out[3 * p + 2];
                const float voa = v_out_alpha ? v_out_alpha[p] : 0.f;
                /* :146-176 */
                const float ra = 1.f / (1.f - alpha);
                T[t] *= ra;
                const float Tc = T[t];
                const float fac = alpha * Tc;
                float v_alpha = 0.f;
                l[0] += (double)(fac * vo0);
                l[1] += (double)(fac * vo1);
                l[2] += (double)(fac * vo2);
                v_alpha += (cr * Tc - buf[t][0] * ra) * vo0;
                v_alpha += (cg * Tc - buf[t][1] * ra) * vo1;
                v_alpha += (cbl * Tc - buf[t][2] * ra) * vo2;
                v_alpha += Tfin[t] * ra * voa;
                v_alpha += -Tfin[t] * ra * bg0 * vo0;
                v_alpha += -Tfin[t] * ra * bg1 * vo1;
                v_alpha += -Tfin[t] * ra * bg2 * vo2;
                const float buf_before[3] = {buf[t][0], buf[t][1], buf[t][2]};
                buf[t][0] += cr * fac;
                buf[t][1] += cg * fac;
                buf[t][2] += cbl * fac;
                const float v_sigma = -opac * vis * v_alpha;
                l[3] += (double)(0.5f * v_sigma * dx * dx);
                l[4] += (double)(v_sigma * dx * dy);
                l[5] += (double)(0.5f * v_sigma * dy * dy);
                l[6] += (double)(v_sigma * (ca * dx + cb * dy));
                l[7] += (double)(v_sigma * (cb * dx + cc * dy));
                l[8] += (double)(vis * v_alpha);
                if(abs_sums)
                {
                    /* the same sums with every elementary term replaced by its absolute value */
                    const double aT = fabs((double)Tc), ara = fabs((double)ra), aTf = fabs((double)Tfin[t]) * ara;
                    const double va = (fabs((double)cr) * aT + fabs((double)buf_before[0]) * ara) * fabs((double)vo0) +
                                      (fabs((double)cg) * aT + fabs((double)buf_before[1]) * ara) * fabs((double)vo1) +
                                      (fabs((double)cbl) * aT + fabs((double)buf_before[2]) * ara) * fabs((double)vo2) +
                                      aTf * (fabs((double)voa) + fabs((double)(bg0 * vo0)) + fabs((double)(bg1 * vo1)) +
                                             fabs((double)(bg2 * vo2)));
                    const double vs = fabs((double)opac) * (double)vis * va;
                    const double adx = fabs((double)dx), ady = fabs((double)dy);
                    la[0] += fabs((double)(fac * vo0));
                    la[1] += fabs((double)(fac * vo1));
                    la[2] += fabs((double)(fac * vo2));
                    la[3] += 0.5 * vs * adx * adx;
                    la[4] += vs * adx * ady;
                    la[5] += 0.5 * vs * ady * ady;
                    la[6] += vs * (fabs((double)ca) * adx + fabs((double)cb) * ady);
                    la[7] += vs * (fabs((double)cb) * adx + fabs((double)cc) * ady);
                    la[8] += (double)vis * va;
                }
            }
            if(g_margin && gm < 1e30f)
            {
#ifdef _OPENMP
#pragma omp critical(dsxo_gm)
#endif
                g_margin[g] = std::min(g_margin[g], gm);
            }
            if(!any)
                continue;
            double* a = acc.data() + (size_t)g * 9;
            for(int c = 0; c < 9; ++c)
            {
#ifdef _OPENMP
#pragma omp atomic
#endif
                a[c] += l[c];
            }
            if(abs_sums)
            {
                double* b = acc_abs.data() + (size_t)g * 9;
                for(int c = 0; c < 9; ++c)
                {
#ifdef _OPENMP
#pragma omp atomic
#endif
                    b[c] += la[c];
                }
            }
        }
    }
    if(abs_sums) /* in the order of the GPU's accumulator record: x y | conic a b c | opacity | r g b */
        for(int64_t i = 0; i < n; ++i)
        {
            const double* b = acc_abs.data() + (size_t)i * 9;
            float* o = abs_sums + 9 * i;
            o[0] = (float)b[6];
            o[1] = (float)b[7];
            o[2] = (float)b[3];
            o[3] = (float)b[4];
            o[4] = (float)b[5];
            o[5] = (float)b[8];
            o[6] = (float)b[0];
            o[7] = (float)b[1];
            o[8] = (float)b[2];
        }
    for(int64_t i = 0; i < n; ++i)
    {
        const double* a = acc.data() + (size_t)i * 9;
        v_rgb[3 * i] = (float)a[0];
        v_rgb[3 * i + 1] = (float)a[1];
        v_rgb[3 * i + 2] = (float)a[2];
        v_conic[3 * i] = (float)a[3];
        v_conic[3 * i + 1] = (float)a[4];
        v_conic[3 * i + 2] = (float)a[5];
        v_xy[2 * i] = (float)a[6];
        v_xy[2 * i + 1] = (float)a[7];
        v_opacity[i] = (float)a[8];
    }
    if(counters)
    {
        counters->pairs_bwd = walked;
        counters->pairs_bwd_valid = valid_pairs;
    }
}

extern "C" void dsxo_sh_bwd(const dsxo_settings* s, int64_t n, int32_t num_bases, const float* means3d,
                            const float* v_rgb, float* v_shs)
{
    const int deg = s->sh_degree;
    const float SH_C0 = 0.28209479177387814f, SH_C1 = 0.4886025119029199f;
    const float SH_C2[] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f, -1.0925484305920792f,
                           0.5462742152960396f};
    const float SH_C3[] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f, 0.3731763325901154f,
                           -0.4570457994644658f, 1.445305721320277f, -0.5900435899266435f};
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for(int64_t i = 0; i < n; ++i)
    {
        float* vc = v_shs + (int64_t)num_bases * 3 * i;
        for(int j = 0; j < num_bases * 3; ++j)
            vc[j] = 0.f;
        const float* v = v_rgb + 3 * i;
        float Y[16];
        int nb = 1;
        Y[0] = SH_C0;
        if(deg >= 1)
        {
            /* sh.cuh:110-120 */
            const float dx = means3d[3 * i] - s->campos[0], dy = means3d[3 * i + 1] - s->campos[1],
                        dz = means3d[3 * i + 2] - s->campos[2];
            const float norm = sqrtf(dx * dx + dy * dy + dz * dz);
            const float x = dx / norm, y = dy / norm, z = dz / norm;
            const float xx = x * x, xy = x * y, xz = x * z, yy = y * y, yz = y * z, zz = z * z;
            Y[1] = -SH_C1 * y;
            Y[2] = SH_C1 * z;
            Y[3] = -SH_C1 * x;
            nb = 4;
            if(deg >= 2)
            {
                Y[4] = SH_C2[0] * xy;
                Y[5] = SH_C2[1] * yz;
                Y[6] = SH_C2[2] * (2.f * zz - xx - yy);
                Y[7] = SH_C2[3] * xz;
                Y[8] = SH_C2[4] * (xx - yy);
                nb = 9;
                if(deg >= 3)
                {
                    Y[9] = SH_C3[0] * y * (3.f * xx - yy);
                    Y[10] = SH_C3[1] * xy * z;
                    Y[11] = SH_C3[2] * y * (4.f * zz - xx - yy);
                    Y[12] = SH_C3[3] * z * (2.f * zz - 3.f * xx - 3.f * yy);
                    Y[13] = SH_C3[4] * x * (4.f * zz - xx - yy);
                    Y[14] = SH_C3[5] * z * (xx - yy);
                    Y[15] = SH_C3[6] * x * (xx - 3.f * yy);
                    nb = 16;
                }
            }
        }
        nb = std::min(nb, (int)num_bases);
        for(int b = 0; b < nb; ++b)
            for(int c = 0; c < 3; ++c)
                vc[3 * b + c] = Y[b] * v[c];
    }
}

namespace
{

/* column-major 3x3 with the semantics of glm::mat3: m[col][row] */
template <typename S> struct M3
{
    S m[3][3];
    S* operator[](int c)
    {
        return m[c];
    }
    const S* operator[](int c) const
    {
        return m[c];
    }
};
template <typename S> inline M3<S> m3(S a, S b, S c, S d, S e, S f, S g, S h, S i)
{
    M3<S> r;
    r.m[0][0] = a, r.m[0][1] = b, r.m[0][2] = c;
    r.m[1][0] = d, r.m[1][1] = e, r.m[1][2] = f;
    r.m[2][0] = g, r.m[2][1] = h, r.m[2][2] = i;
    return r;
}
template <typename S> inline M3<S> mul(const M3<S>& A, const M3<S>& B)
{
    M3<S> R;
    for(int c = 0; c < 3; ++c)
        for(int r = 0; r < 3; ++r)
            R.m[c][r] = A.m[0][r] * B.m[c][0] + A.m[1][r] * B.m[c][1] + A.m[2][r] * B.m[c][2];
    return R;
}
template <typename S> inline M3<S> tr(const M3<S>& A)
{
    M3<S> R;
    for(int c = 0; c < 3; ++c)
        for(int r = 0; r < 3; ++r)
            R.m[c][r] = A.m[r][c];
    return R;
}
template <typename S> inline M3<S> add(const M3<S>& A, const M3<S>& B)
{
    M3<S> R;
    for(int c = 0; c < 3; ++c)
        for(int r = 0; r < 3; ++r)
            R.m[c][r] = A.m[c][r] + B.m[c][r];
    return R;
}

/* helpers.cuh:149-168 */
template <typename S> inline M3<S> quat_to_rotmat(const S* q)
{
    const S w = q[0], x = q[1], y = q[2], z = q[3];
    return m3<S>(S(1) - S(2) * (y * y + z * z), S(2) * (x * y + w * z), S(2) * (x * z - w * y),
                 S(2) * (x * y - w * z), S(1) - S(2) * (x * x + z * z), S(2) * (y * z + w * x),
                 S(2) * (x * z + w * y), S(2) * (y * z - w * x), S(1) - S(2) * (x * x + y * y));
}

} // namespace

extern "C" void dsxo_project_bwd(const dsxo_settings* s, int64_t n, const float* means3d, const float* scales,
                                 const float* quats, const float* conic, const float* cov3d, const int32_t* radii,
                                 const float* v_xy, const float* v_conic, float* v_mean3d, float* v_scale,
                                 float* v_quat, float* v_cov3d, float* v_cov2d)
{
    /* rasterizer_torch.cu:78-81,297-298 */
    const float fovx = 2 * atanf(s->tanfovx);
    const float fovy = 2 * atanf(s->tanfovy);
    const float fx = (float)s->image_width / (2.0f * tanf(fovx / 2.0f));
    const float fy = (float)s->image_height / (2.0f * tanf(fovy / 2.0f));
    const float* V = s->view;
    const float glob = s->scale_modifier;
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for(int64_t i = 0; i < n; ++i)
    {
        float* vm = v_mean3d + 3 * i;
        float* vs = v_scale + 3 * i;
        float* vq = v_quat + 4 * i;
        float* vc3 = v_cov3d + 6 * i;
        float* vc2 = v_cov2d + 3 * i;
        vm[0] = vm[1] = vm[2] = 0.f;
        vs[0] = vs[1] = vs[2] = 0.f;
        vq[0] = vq[1] = vq[2] = vq[3] = 0.f;
        for(int j = 0; j < 6; ++j)
            vc3[j] = 0.f;
        vc2[0] = vc2[1] = vc2[2] = 0.f;
        if(radii[i] <= 0)
            continue; /* backward.cu:239 */

        const float* p = means3d + 3 * i;
        /* transform_4x3 helpers.cuh:107-114 */
        const float pv[3] = {V[0] * p[0] + V[1] * p[1] + V[2] * p[2] + V[3],
                             V[4] * p[0] + V[5] * p[1] + V[6] * p[2] + V[7],
                             V[8] * p[0] + V[9] * p[1] + V[10] * p[2] + V[11]};
        /* project_pix_vjp helpers.cuh:138-147 */
        const float rw = 1.f / (pv[2] + 1e-6f);
        const float vpx = fx * v_xy[2 * i], vpy = fy * v_xy[2 * i + 1];
        const float vv[3] = {vpx * rw, vpy * rw, -(vpx * pv[0] + vpy * pv[1]) * rw * rw};
        /* transform_4x3_rot_only_transposed helpers.cuh:97-104 */
        vm[0] = V[0] * vv[0] + V[4] * vv[1] + V[8] * vv[2];
        vm[1] = V[1] * vv[0] + V[5] * vv[1] + V[9] * vv[2];
        vm[2] = V[2] * vv[0] + V[6] * vv[1] + V[10] * vv[2];
        /* v_depth = 0 (rasterizer_torch.cu:306): backward.cu:256-259 adds zero */

        /* cov2d_to_conic_vjp helpers.cuh:68-79 */
        {
            const float* c = conic + 3 * i;
            const float* g = v_conic + 3 * i;
            /* column-major 2x2: X = [[c0,c1],[c1,c2]], G = [[g0,g1/2],[g1/2,g2]] */
            const float X[2][2] = {{c[0], c[1]}, {c[1], c[2]}};
            const float G[2][2] = {{g[0], g[1] / 2.f}, {g[1] / 2.f, g[2]}};
            float nX[2][2], A[2][2], R[2][2];
            for(int a = 0; a < 2; ++a)
                for(int b = 0; b < 2; ++b)
                    nX[a][b] = -X[a][b];
            for(int col = 0; col < 2; ++col)
                for(int row = 0; row < 2; ++row)
                    A[col][row] = nX[0][row] * G[col][0] + nX[1][row] * G[col][1];
            for(int col = 0; col < 2; ++col)
                for(int row = 0; row < 2; ++row)
                    R[col][row] = A[0][row] * X[col][0] + A[1][row] * X[col][1];
            vc2[0] = R[0][0];
            vc2[1] = R[1][0] + R[0][1];
            vc2[2] = R[1][1];
            /* cov2d_to_compensation_vjp helpers.cuh:81-94 with v_compensation = 0 adds 0 */
        }

        /* project_cov3d_ewa_vjp backward.cu:291-366 */
        {
            const M3<float> Wm = m3<float>(V[0], V[4], V[8], V[1], V[5], V[9], V[2], V[6], V[10]);
            const float t[3] = {Wm[0][0] * p[0] + Wm[1][0] * p[1] + Wm[2][0] * p[2] + V[3],
                                Wm[0][1] * p[0] + Wm[1][1] * p[1] + Wm[2][1] * p[2] + V[7],
                                Wm[0][2] * p[0] + Wm[1][2] * p[1] + Wm[2][2] * p[2] + V[11]};
            const float rz = 1.f / t[2];
            const float rz2 = rz * rz;
            const M3<float> J = m3<float>(fx * rz, 0.f, 0.f, 0.f, fy * rz, 0.f, -fx * t[0] * rz2, -fy * t[1] * rz2, 0.f);
            const float* c3 = cov3d + 6 * i;
            const M3<float> Vm = m3<float>(c3[0], c3[1], c3[2], c3[1], c3[3], c3[4], c3[2], c3[4], c3[5]);
            const M3<float> v_cov = m3<float>(vc2[0], 0.5f * vc2[1], 0.f, 0.5f * vc2[1], vc2[2], 0.f, 0.f, 0.f, 0.f);
            const M3<float> T = mul(J, Wm);
            const M3<float> Tt = tr(T);
            const M3<float> Vt = tr(Vm);
            const M3<float> v_V = mul(mul(Tt, v_cov), T);
            const M3<float> v_T = add(mul(mul(v_cov, T), Vt), mul(mul(tr(v_cov), T), Vm));
            vc3[0] = v_V[0][0];
            vc3[1] = v_V[0][1] + v_V[1][0];
            vc3[2] = v_V[0][2] + v_V[2][0];
            vc3[3] = v_V[1][1];
            vc3[4] = v_V[1][2] + v_V[2][1];
            vc3[5] = v_V[2][2];
            const M3<float> v_J = mul(v_T, tr(Wm));
            const float rz3 = rz2 * rz;
            const float v_t[3] = {-fx * rz2 * v_J[2][0], -fy * rz2 * v_J[2][1],
                                  -fx * rz2 * v_J[0][0] + 2.f * fx * t[0] * rz3 * v_J[2][0] - fy * rz2 * v_J[1][1] +
                                      2.f * fy * t[1] * rz3 * v_J[2][1]};
            vm[0] += v_t[0] * Wm[0][0] + v_t[1] * Wm[0][1] + v_t[2] * Wm[0][2];
            vm[1] += v_t[0] * Wm[1][0] + v_t[1] * Wm[1][1] + v_t[2] * Wm[1][2];
            vm[2] += v_t[0] * Wm[2][0] + v_t[1] * Wm[2][1] + v_t[2] * Wm[2][2];
        }

        /* scale_rot_to_cov3d_vjp backward.cu:370-393 */
        {
            const M3<float> v_V = m3<float>(vc3[0], 0.5f * vc3[1], 0.5f * vc3[2], 0.5f * vc3[1], vc3[3], 0.5f * vc3[4],
                                            0.5f * vc3[2], 0.5f * vc3[4], vc3[5]);
            const float* q = quats + 4 * i;
            const float* sc = scales + 3 * i;
            const M3<float> R = quat_to_rotmat<float>(q);
            M3<float> S = m3<float>(1.f, 0.f, 0.f, 0.f, 1.f, 0.f, 0.f, 0.f, 1.f);
            S[0][0] = glob * sc[0];
            S[1][1] = glob * sc[1];
            S[2][2] = glob * sc[2];
            const M3<float> M = mul(R, S);
            M3<float> v_M = mul(v_V, M);
            for(int c = 0; c < 3; ++c)
                for(int r = 0; r < 3; ++r)
                    v_M[c][r] = 2.f * v_M[c][r];
            /* note: glm evaluates 2.f * v_V first; (2 v_V) M == 2 (v_V M) up to rounding only
             * through exact doubling, so the two orders agree bit for bit */
            vs[0] = (R[0][0] * v_M[0][0] + R[0][1] * v_M[0][1] + R[0][2] * v_M[0][2]) * glob;
            vs[1] = (R[1][0] * v_M[1][0] + R[1][1] * v_M[1][1] + R[1][2] * v_M[1][2]) * glob;
            vs[2] = (R[2][0] * v_M[2][0] + R[2][1] * v_M[2][1] + R[2][2] * v_M[2][2]) * glob;
            const M3<float> v_R = mul(v_M, S);
            /* quat_to_rotmat_vjp helpers.cuh:170-211 */
            const float w = q[0], x = q[1], y = q[2], z = q[3];
            vq[0] = 2.f * (x * (v_R[1][2] - v_R[2][1]) + y * (v_R[2][0] - v_R[0][2]) + z * (v_R[0][1] - v_R[1][0]));
            vq[1] = 2.f * (-2.f * x * (v_R[1][1] + v_R[2][2]) + y * (v_R[0][1] + v_R[1][0]) +
                           z * (v_R[0][2] + v_R[2][0]) + w * (v_R[1][2] - v_R[2][1]));
            vq[2] = 2.f * (x * (v_R[0][1] + v_R[1][0]) - 2.f * y * (v_R[0][0] + v_R[2][2]) +
                           z * (v_R[1][2] + v_R[2][1]) + w * (v_R[2][0] - v_R[0][2]));
            vq[3] = 2.f * (x * (v_R[0][2] + v_R[2][0]) + y * (v_R[1][2] + v_R[2][1]) -
                           2.f * z * (v_R[0][0] + v_R[1][1]) + w * (v_R[0][1] - v_R[1][0]));
        }
    }
}

/* ---------------------------------------------------------------------------------- */
/* whole pipeline                                                                      */
/* ---------------------------------------------------------------------------------- */

struct dsxo_state
{
    int64_t n = 0, k = 0;
    int32_t num_tiles = 0, W = 0, H = 0;
    std::vector<float> means2d, conic, rgb, cov3d, final_T, margin;
    std::vector<int32_t> radii, tiles_touched, offsets, ids, ranges, final_idx, emitted_values;
    std::vector<int64_t> keys, emitted_keys;
    dsxo_counters counters{};
};

static int g_keep_emitted = 0;
extern "C" void dsxo_keep_emitted(int on)
{
    g_keep_emitted = on;
}

extern "C" dsxo_state* dsxo_forward(const dsxo_settings* s, int64_t n, const float* means3d, const float* scales,
                                    const float* quats, const float* opacities, const float* shs,
                                    const float* cov3d_precomp, const float* colors_precomp, float* image,
                                    int32_t* radii)
{
    dsxo_state* st = new dsxo_state();
    st->n = n;
    st->W = s->image_width;
    st->H = s->image_height;
    st->num_tiles = tiles_x(s) * tiles_y(s);
    const int64_t P = (int64_t)st->W * st->H;
    st->means2d.resize(3 * n);
    st->conic.resize(3 * n);
    st->rgb.resize(3 * n);
    st->cov3d.resize(6 * n);
    st->radii.resize(n);
    st->tiles_touched.resize(n);
    st->offsets.resize(n);
    dsxo_project_fwd(s, n, means3d, scales, quats, shs, cov3d_precomp, colors_precomp, st->means2d.data(),
                     st->conic.data(), st->rgb.data(), st->radii.data(), st->tiles_touched.data(), st->cov3d.data());
    st->k = dsxo_offsets(n, st->tiles_touched.data(), st->offsets.data());
    st->keys.resize(st->k);
    st->ids.resize(st->k);
    dsxo_emit_keys(s, n, st->k, st->means2d.data(), st->radii.data(), st->offsets.data(), st->keys.data(),
                   st->ids.data());
    if(g_keep_emitted)
    {
        st->emitted_keys = st->keys;
        st->emitted_values = st->ids;
    }
    dsxo_sort_pairs(st->k, st->keys.data(), st->ids.data());
    st->ranges.resize(st->num_tiles + 1);
    dsxo_tile_ranges(st->k, st->keys.data(), st->num_tiles, st->ranges.data());
    st->final_T.resize(P);
    st->final_idx.resize(P);
    st->margin.resize(P);
    dsxo_blend_fwd(s, st->ranges.data(), st->ids.data(), st->means2d.data(), st->conic.data(), st->rgb.data(),
                   opacities, image, st->final_T.data(), st->final_idx.data(), st->margin.data(), &st->counters);
    if(radii)
        memcpy(radii, st->radii.data(), n * sizeof(int32_t));
    return st;
}

extern "C" int64_t dsxo_state_num_keys(const dsxo_state* st)
{
    return st->k;
}

template <typename T> static void copy_out(T* dst, const std::vector<T>& src)
{
    if(dst && !src.empty())
        memcpy(dst, src.data(), src.size() * sizeof(T));
}

extern "C" void dsxo_state_get(const dsxo_state* st, float* means2d, float* conic, float* rgb,
                               int32_t* tiles_touched, int32_t* offsets, float* cov3d, int64_t* sorted_keys,
                               int32_t* sorted_ids, int32_t* ranges, float* final_T, int32_t* final_idx,
                               float* margin, dsxo_counters* counters)
{
    copy_out(means2d, st->means2d);
    copy_out(conic, st->conic);
    copy_out(rgb, st->rgb);
    copy_out(tiles_touched, st->tiles_touched);
    copy_out(offsets, st->offsets);
    copy_out(cov3d, st->cov3d);
    copy_out(sorted_keys, st->keys);
    copy_out(sorted_ids, st->ids);
    copy_out(ranges, st->ranges);
    copy_out(final_T, st->final_T);
    copy_out(final_idx, st->final_idx);
    copy_out(margin, st->margin);
    if(counters)
        *counters = st->counters;
}

extern "C" void dsxo_state_get_emitted(const dsxo_state* st, int64_t* keys, int32_t* values)
{
    copy_out(keys, st->emitted_keys);
    copy_out(values, st->emitted_values);
}

extern "C" void dsxo_backward(dsxo_state* st, const dsxo_settings* s, int64_t n, int32_t num_bases,
                              const float* means3d, const float* scales, const float* quats, const float* opacities,
                              const float* v_image, float* v_mean3d, float* v_means2d, float* v_shs, float* v_colors,
                              float* v_opacity, float* v_scale, float* v_quat, float* v_cov3d, float* g_margin)
{
    dsxo_backward_ex(st, s, n, num_bases, means3d, scales, quats, opacities, v_image, v_mean3d, v_means2d, v_shs,
                     v_colors, v_opacity, v_scale, v_quat, v_cov3d, g_margin, nullptr);
}

extern "C" void dsxo_backward_ex(dsxo_state* st, const dsxo_settings* s, int64_t n, int32_t num_bases,
                                 const float* means3d, const float* scales, const float* quats,
                                 const float* opacities, const float* v_image, float* v_mean3d, float* v_means2d,
                                 float* v_shs, float* v_colors, float* v_opacity, float* v_scale, float* v_quat,
                                 float* v_cov3d, float* g_margin, float* abs_sums)
{
    std::vector<float> v_xy(2 * n), v_conic(3 * n), v_cov2d(3 * n);
    dsxo_blend_bwd_ex(s, n, st->ranges.data(), st->ids.data(), st->means2d.data(), st->conic.data(), st->rgb.data(),
                      opacities, st->final_T.data(), st->final_idx.data(), v_image, nullptr, v_xy.data(),
                      v_conic.data(), v_colors, v_opacity, g_margin, &st->counters, abs_sums);
    /* rasterizer_torch.cu:292: v_colors *= clamped_colors (all ones) — identity */
    dsxo_sh_bwd(s, n, num_bases, means3d, v_colors, v_shs);
    dsxo_project_bwd(s, n, means3d, scales, quats, st->conic.data(), st->cov3d.data(), st->radii.data(), v_xy.data(),
                     v_conic.data(), v_mean3d, v_scale, v_quat, v_cov3d, v_cov2d.data());
    /* rasterizer_torch.cu:313 */
    for(int64_t i = 0; i < n; ++i)
    {
        v_means2d[3 * i] = v_xy[2 * i];
        v_means2d[3 * i + 1] = v_xy[2 * i + 1];
        v_means2d[3 * i + 2] = 0.f;
    }
}

extern "C" void dsxo_state_free(dsxo_state* st)
{
    delete st;
}

/* ---------------------------------------------------------------------------------- */
/* float64 instances for finite differences                                            */
/* ---------------------------------------------------------------------------------- */

extern "C" double dsxo_blend_loss_f64(int32_t width, int32_t height, const int32_t* ranges,
                                      const int32_t* sorted_ids, int64_t n, const double* xy, const double* conic,
                                      const double* rgb, const double* opac, const double* weights,
                                      const double* bg, double alpha_clamp)
{
    (void)n;
    const int ntx = (width + TILE - 1) / TILE;
    double loss = 0.0;
    for(int y = 0; y < height; ++y)
        for(int x = 0; x < width; ++x)
        {
            const int tile = (y / TILE) * ntx + (x / TILE);
            double C[3], T;
            int32_t last;
            blend_pixel<double>(x, y, ranges[tile], ranges[tile + 1], sorted_ids, xy, 2, conic, rgb, opac, alpha_clamp,
                                C, &T, &last, nullptr, nullptr, nullptr);
            const int64_t p = (int64_t)y * width + x;
            loss += C[0] * weights[3 * p] + C[1] * weights[3 * p + 1] + C[2] * weights[3 * p + 2];
            if(bg) /* composited background: the term backward.cu:160-164 differentiates */
                loss += T * (bg[0] * weights[3 * p] + bg[1] * weights[3 * p + 1] + bg[2] * weights[3 * p + 2]);
        }
    return loss;
}
