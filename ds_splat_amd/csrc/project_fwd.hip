// Stage 1: per-Gaussian projection for gfx950.
//
// One thread per Gaussian, 256 per workgroup (4 wave64).  Each wavefront copies the
// spherical-harmonics rows of its 64 Gaussians (a contiguous 12 KB span at degree 3) into LDS
// with 16-byte coalesced loads and then every lane reads its own row back with an odd LDS
// pitch (conflict free), so the 192-byte AoS rows never produce strided HBM traffic; only
// the columns the active degree needs are fetched, and only the rows of Gaussians whose centre
// passes the frustum test.  The rows go through LDS in three parts of 16 floats (one 64-byte
// sector of each 192-byte row at a time, so every sector is fetched exactly once) and a
// workgroup holds 17 KB of LDS instead of 50 KB: occupancy is no longer bound by LDS.
//
// This translation unit is compiled with floating-point contraction OFF and uses only
// + - * / sqrt on binary32: radii, tile counts and depth keys are integers derived from these
// floats and must not depend on the compiler's choice of fused multiply-adds.
// Behaviour follows cpp/rasterizer_kernels.cu:57-161 of the reference; rsqrtf there (an
// approximate instruction) is evaluated as 1/sqrt so results are reproducible.
#include "dsx_common.h"

#pragma clang fp contract(off)

namespace dsx
{

// Rows pass through LDS in three parts of 16 floats (64 bytes, one sector of the row).
constexpr int kShPart = 16;
constexpr int kShPitch = 17; // floats per row in LDS (odd pitch: conflict-free row reads)

struct ProjectParams
{
    int64_t n;
    const float* means3d;
    const float* scales;
    const float* quats;
    const float* opacities;
    const float* shs;
    const float* cov3d_precomp;
    const float* colors_precomp;
    const float* view;
    const float* proj;
    const float* campos;
    float4* splats;
    int32_t* radii;
    float* cov3d;
    uint32_t* block_sums;
    uint32_t* depth_keys; // optional: depth bits per Gaussian, the key of the depth order
    uint2* rects;         // optional: packed tile rectangle per Gaussian (zero when it emits nothing)
    uint32_t* clear;      // optional: words that the kernel zeroes on the side (counters of the sort that follows)
    int64_t clear_words;
    float focal_x, focal_y, tanfovx, tanfovy, c_x, c_y, scale_modifier;
    int sh_degree, sh_stride; // active degree; floats per shs row
    int ntx, nty;
};

// SH degree 0..3 -> RGB (+0.5, clamped at 0), term order as cpp/rasterizer_kernels.cu:433-554,
// in two steps that add to the same accumulators in the reference's order: degrees 0-2 from
// floats 0..26 of the row, then degree 3 from float 27 (f27) and floats 28..47 (g[0..19]).
struct ShDir
{
    float vx, vy, vz;
};

__device__ __forceinline__ ShDir sh_direction(float3 mean, float3 cam)
{
    const float dx = mean.x - cam.x, dy = mean.y - cam.y, dz = mean.z - cam.z;
    const float inv_norm = 1.0f / sqrtf(dx * dx + dy * dy + dz * dz);
    ShDir d;
    d.vx = dx * inv_norm;
    d.vy = dy * inv_norm;
    d.vz = dz * inv_norm;
    return d;
}

__device__ __forceinline__ void sh_low(int deg, const float* f, ShDir d, float& rx, float& ry, float& rz)
{
    const float C0 = 0.28209479177387814f;
    rx = 0.0f + C0 * f[0];
    ry = 0.0f + C0 * f[1];
    rz = 0.0f + C0 * f[2];
    if(deg >= 1)
    {
        const float vx = d.vx, vy = d.vy, vz = d.vz;
        const float C1 = 0.4886025119029199f;
        rx += C1 * (-vy * f[3] + vz * f[6] - vx * f[9]);
        ry += C1 * (-vy * f[4] + vz * f[7] - vx * f[10]);
        rz += C1 * (-vy * f[5] + vz * f[8] - vx * f[11]);
        if(deg >= 2)
        {
            const float xx = vx * vx, yy = vy * vy, zz = vz * vz;
            const float xy = vx * vy, xz = vx * vz, yz = vy * vz;
            const float A0 = 1.0925484305920792f, A1 = -1.0925484305920792f, A2 = 0.31539156525252005f,
                        A3 = -1.0925484305920792f, A4 = 0.5462742152960396f;
            const float q2 = 2.0f * zz - xx - yy, q4 = xx - yy;
            rx += A0 * xy * f[12] + A1 * yz * f[15] + A2 * q2 * f[18] + A3 * xz * f[21] + A4 * q4 * f[24];
            ry += A0 * xy * f[13] + A1 * yz * f[16] + A2 * q2 * f[19] + A3 * xz * f[22] + A4 * q4 * f[25];
            rz += A0 * xy * f[14] + A1 * yz * f[17] + A2 * q2 * f[20] + A3 * xz * f[23] + A4 * q4 * f[26];
        }
    }
}

// g[j] = float 28 + j of the row
__device__ __forceinline__ void sh_high(float f27, const float* g, ShDir d, float& rx, float& ry, float& rz)
{
    const float vx = d.vx, vy = d.vy, vz = d.vz;
    const float xx = vx * vx, yy = vy * vy, zz = vz * vz;
    const float xy = vx * vy;
    const float B0 = -0.5900435899266435f, B1 = 2.890611442640554f, B2 = -0.4570457994644658f,
                B3 = 0.3731763325901154f, B4 = -0.4570457994644658f, B5 = 1.445305721320277f,
                B6 = -0.5900435899266435f;
    const float t0 = B0 * vy * (3.0f * xx - yy);
    const float t1 = B1 * xy * vz;
    const float t2 = B2 * vy * (4.0f * zz - xx - yy);
    const float t3 = B3 * vz * (2.0f * zz - 3.0f * xx - 3.0f * yy);
    const float t4 = B4 * vx * (4.0f * zz - xx - yy);
    const float t5 = B5 * vz * (xx - yy);
    const float t6 = B6 * vx * (xx - 3.0f * yy);
    rx += t0 * f27 + t1 * g[2] + t2 * g[5] + t3 * g[8] + t4 * g[11] + t5 * g[14] + t6 * g[17];
    ry += t0 * g[0] + t1 * g[3] + t2 * g[6] + t3 * g[9] + t4 * g[12] + t5 * g[15] + t6 * g[18];
    rz += t0 * g[1] + t1 * g[4] + t2 * g[7] + t3 * g[10] + t4 * g[13] + t5 * g[16] + t6 * g[19];
}

// Copies columns [c_begin, c_end) of the wavefront's wanted SH rows into LDS at dst[row * kShPitch
// + (c - c_begin)].  Fast path: 16-byte chunks of 192-byte rows; c_begin and c_end are
// multiples of 4 there.
template <int kMaxChunksPerLane>
__device__ __forceinline__ void stage_sh_columns(const ProjectParams& p, int64_t row0, int rows, uint64_t wanted_rows,
                                                 int c_begin, int c_end, int lane, float* dst)
{
    if(c_end <= c_begin)
        return;
    if(p.sh_stride == 48 && ((uintptr_t)p.shs & 15) == 0)
    {
        const float4* src = reinterpret_cast<const float4*>(p.shs + row0 * 48);
        const int q0 = c_begin >> 2;
        const int per_row = ((c_end + 3) >> 2) - q0; // 16-byte chunks per row in this part
        const int chunks = rows * per_row;
        // all loads are issued before the first LDS write, so their latencies overlap
        float4 v[kMaxChunksPerLane];
        int at[kMaxChunksPerLane];
#pragma unroll
        for(int it = 0; it < kMaxChunksPerLane; ++it)
        {
            const int e = it * 64 + lane;
            const int row = e / per_row;
            const int c4 = e - row * per_row;
            at[it] = -1;
            if(e < chunks && ((wanted_rows >> row) & 1))
            {
                v[it] = src[row * 12 + q0 + c4]; // cached load: the other sectors of the line follow in the next parts
                at[it] = row * kShPitch + c4 * 4;
            }
        }
#pragma unroll
        for(int it = 0; it < kMaxChunksPerLane; ++it)
        {
            if(at[it] >= 0)
            {
                float* d = dst + at[it];
                d[0] = v[it].x;
                d[1] = v[it].y;
                d[2] = v[it].z;
                d[3] = v[it].w;
            }
        }
    }
    else
    {
        const float* src = p.shs + row0 * p.sh_stride;
        const int width = c_end - c_begin;
        const int total = rows * width;
        for(int e = lane; e < total; e += 64)
        {
            const int row = e / width;
            const int c = e - row * width;
            if((wanted_rows >> row) & 1)
                dst[row * kShPitch + c] = src[(int64_t)row * p.sh_stride + c_begin + c];
        }
    }
}

__global__ __launch_bounds__(kProjBlock) void project_fwd_kernel(const ProjectParams p)
{
    __shared__ float sh_lds[4][64 * kShPitch];
    __shared__ uint32_t wave_sums[4];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int64_t i = (int64_t)blockIdx.x * kProjBlock + tid;
    const bool live = i < p.n;

    // housekeeping for the sort that follows: its counters are zeroed here, a word per thread,
    // instead of by a launch of their own
    for(int64_t j = i; j < p.clear_words; j += (int64_t)gridDim.x * kProjBlock)
        p.clear[j] = 0u;

    // frustum test on the centre: strict NDC box, z_ndc > 0.1 (cpp/rasterizer_kernels.cu:7-24).
    // It comes first because a Gaussian that fails it is culled whatever its shape is, nothing
    // downstream reads its colour, and so its SH row (the largest input) is never fetched.
    float3 mean = make_float3(0.f, 0.f, 0.f);
    bool in_frustum = false;
    if(live)
    {
        mean = make_float3(p.means3d[3 * i], p.means3d[3 * i + 1], p.means3d[3 * i + 2]);
        const float* P = p.proj;
        const float inv_w = 1.0f / (P[12] * mean.x + P[13] * mean.y + P[14] * mean.z + P[15]);
        const float nx = inv_w * (P[0] * mean.x + P[1] * mean.y + P[2] * mean.z + P[3]);
        const float ny = inv_w * (P[4] * mean.x + P[5] * mean.y + P[6] * mean.z + P[7]);
        const float nz = inv_w * (P[8] * mean.x + P[9] * mean.y + P[10] * mean.z + P[11]);
        in_frustum = nx > -1.0f && nx < 1.0f && ny > -1.0f && ny < 1.0f && nz > 0.1f;
    }
    const uint64_t wanted_rows = __ballot(in_frustum); // bit r: lane r of this wavefront needs its SH row

    // ---- colours: this wavefront's SH rows through LDS, one 64-byte sector of each row at a time ---
    // (each wavefront owns its part of the LDS array, so wavefront-local ordering is enough)
    const bool use_sh = p.colors_precomp == nullptr;
    float3 rgb = make_float3(0.f, 0.f, 0.f);
    if(use_sh)
    {
        const int64_t row0 = (int64_t)blockIdx.x * kProjBlock + wave * 64;
        const int rows = (int)max((int64_t)0, min((int64_t)64, p.n - row0));
        const int need = (p.sh_degree + 1) * (p.sh_degree + 1) * 3; // floats per row actually used
        float* dst = sh_lds[wave];
        const float* row = dst + lane * kShPitch;
        float rx = 0.f, ry = 0.f, rz = 0.f;
        float f[48]; // the row, collected part by part (registers of parts already used are dead)
#pragma unroll
        for(int part = 0; part < 3; ++part)
        {
            const int c0 = part * kShPart;
            if(c0 < need) // uniform
            {
                if(part > 0)
                {
                    // the wavefront's reads of the previous part are done before it is overwritten
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                }
                stage_sh_columns<4>(p, row0, rows, wanted_rows, c0, min(need, c0 + kShPart), lane, dst);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            }
#pragma unroll
            for(int j = 0; j < kShPart; ++j)
                f[c0 + j] = (in_frustum && c0 + j < need) ? row[j] : 0.0f;
        }
        if(in_frustum)
        {
            ShDir dir = {0.f, 0.f, 0.f};
            if(p.sh_degree >= 1)
                dir = sh_direction(mean, make_float3(p.campos[0], p.campos[1], p.campos[2]));
            sh_low(p.sh_degree, f, dir, rx, ry, rz);
            if(p.sh_degree >= 3)
                sh_high(f[27], f + 28, dir, rx, ry, rz);
        }
        if(in_frustum)
            rgb = make_float3(fmaxf(rx + 0.5f, 0.0f), fmaxf(ry + 0.5f, 0.0f), fmaxf(rz + 0.5f, 0.0f));
    }

    uint32_t count = 0;
    if(live)
    {
        float c3[6];
        if(p.cov3d_precomp)
        {
#pragma unroll
            for(int j = 0; j < 6; ++j)
                c3[j] = p.cov3d_precomp[6 * i + j];
        }
        else
        {
            const float sc[3] = {p.scales[3 * i], p.scales[3 * i + 1], p.scales[3 * i + 2]};
            const float4 q = reinterpret_cast<const float4*>(p.quats)[i];
            cov3d_from_scale_rot(sc, q, p.scale_modifier, c3);
        }
        if(p.cov3d) // optional: the backward can rebuild it from scale and rotation
        {
            float2* o = reinterpret_cast<float2*>(p.cov3d + 6 * i);
            o[0] = make_float2(c3[0], c3[1]);
            o[1] = make_float2(c3[2], c3[3]);
            o[2] = make_float2(c3[4], c3[5]);
        }

        if(!use_sh)
            rgb = make_float3(p.colors_precomp[3 * i], p.colors_precomp[3 * i + 1], p.colors_precomp[3 * i + 2]);

        // view-space position (cpp/rasterizer_kernels.cu:325-330)
        const float* V = p.view;
        const float vx = V[0] * mean.x + V[1] * mean.y + V[2] * mean.z + V[3];
        const float vy = V[4] * mean.x + V[5] * mean.y + V[6] * mean.z + V[7];
        const float vz = V[8] * mean.x + V[9] * mean.y + V[10] * mean.z + V[11];

        // EWA covariance (cpp/rasterizer_kernels.cu:174-231): sums start from 0 and add the
        // three products in index order, zero Jacobian entries included
        const float limx = 1.3f * p.tanfovx;
        const float limy = 1.3f * p.tanfovy;
        const float txtz = vx / vz;
        const float tytz = vy / vz;
        const float t0 = fminf(limx, fmaxf(-limx, txtz)) * vz;
        const float t1 = fminf(limy, fmaxf(-limy, tytz)) * vz;
        const float t2 = vz;
        const float J[3][3] = {{p.focal_x / t2, 0.0f, -(p.focal_x * t0) / (t2 * t2)},
                               {0.0f, p.focal_y / t2, -(p.focal_y * t1) / (t2 * t2)},
                               {0.0f, 0.0f, 0.0f}};
        const float Wm[3][3] = {{V[0], V[4], V[8]}, {V[1], V[5], V[9]}, {V[2], V[6], V[10]}};
        float T[3][3];
#pragma unroll
        for(int a = 0; a < 3; ++a)
#pragma unroll
            for(int b = 0; b < 3; ++b)
            {
                float acc = 0.0f;
#pragma unroll
                for(int k = 0; k < 3; ++k)
                    acc += Wm[a][k] * J[b][k];
                T[a][b] = acc;
            }
        const float S3[3][3] = {{c3[0], c3[1], c3[2]}, {c3[1], c3[3], c3[4]}, {c3[2], c3[4], c3[5]}};
        float tmp[3][3];
#pragma unroll
        for(int a = 0; a < 3; ++a)
#pragma unroll
            for(int b = 0; b < 3; ++b)
            {
                float acc = 0.0f;
#pragma unroll
                for(int k = 0; k < 3; ++k)
                    acc += T[k][a] * S3[k][b];
                tmp[a][b] = acc;
            }
        float cov[2][2];
#pragma unroll
        for(int a = 0; a < 2; ++a)
#pragma unroll
            for(int b = 0; b < 2; ++b)
            {
                float acc = 0.0f;
#pragma unroll
                for(int k = 0; k < 3; ++k)
                    acc += tmp[a][k] * T[k][b];
                cov[a][b] = acc;
            }
        const float ca = cov[0][0] + 0.3f;
        const float cb = cov[0][1];
        const float cc = cov[1][1] + 0.3f;

        // pixel mean (cpp/rasterizer_kernels.cu:332-337)
        const float z_inv = 1.0f / (vz + 1e-6f);
        const float px = p.focal_x * vx * z_inv + p.c_x;
        const float py = p.focal_y * vy * z_inv + p.c_y;

        // radius = ceil(3 sigma_max), zero when culled (cpp/rasterizer_kernels.cu:163-172)
        const float det = ca * cc - cb * cb;
        const float mid = 0.5f * (ca + cc);
        const float diff = mid * mid - det;
        const float root = sqrtf(fmaxf(0.1f, diff));
        const float lambda1 = mid + root;
        const float lambda2 = mid - root;
        const float keep = (det > 1e-6f && in_frustum) ? 1.0f : 0.0f;
        const int radius = f2i_sat(ceilf(3.0f * sqrtf(fmaxf(lambda1, lambda2))) * keep);

        const TileRect r = tile_rect(px, py, radius, p.ntx, p.nty);
        const int tiles = (r.ex - r.sx) * (r.ey - r.sy) * (radius > 0 ? 1 : 0);

        // conic (cpp/rasterizer_kernels.cu:49-55)
        const float det_inv = 1.0f / (det + 1e-6f);
        const float opacity = p.opacities[i];

        float4* rec = p.splats + 3 * i;
        rec[0] = make_float4(px, py, vz, __int_as_float(radius));
        rec[1] = make_float4(cc * det_inv, -cb * det_inv, ca * det_inv, opacity);
        rec[2] = make_float4(rgb.x, rgb.y, rgb.z, __int_as_float(tiles));
        p.radii[i] = radius;

        // the last Gaussian never emits keys (cpp/rasterizer_torch.cu:99-104)
        count = (i == p.n - 1) ? 0u : (uint32_t)tiles;
        if(p.depth_keys)
        {
            // x = sx | sy << 16, y = width | height << 16 | (depth sign) << 31
            // A Gaussian that emits no pair gets the all-ones key: it sorts behind every Gaussian
            // that does (their order among themselves is immaterial) and tells the depth sort that
            // its rectangle is empty without a look at it.
            const uint32_t depth_bits = __float_as_uint(vz);
            p.depth_keys[i] = count ? depth_bits : kNoPairsKey;
            p.rects[i] = count ? make_uint2((uint32_t)r.sx | ((uint32_t)r.sy << 16),
                                            (uint32_t)(r.ex - r.sx) | ((uint32_t)(r.ey - r.sy) << 16) |
                                                (depth_bits & 0x80000000u))
                               : make_uint2(0u, 0u);
        }
    }

    const uint32_t ws = wave_sum_u32(count);
    if(lane == 0)
        wave_sums[wave] = ws;
    __syncthreads();
    if(tid == 0)
        p.block_sums[blockIdx.x] = wave_sums[0] + wave_sums[1] + wave_sums[2] + wave_sums[3];
}

int launch_project_fwd(const dsx_camera& cam, int64_t n, const float* means3d, const float* scales,
                       const float* quats, const float* opacities, const float* shs,
                       const float* cov3d_precomp, const float* colors_precomp, float* splats, int32_t* radii,
                       float* cov3d, uint32_t* block_sums, uint32_t* depth_keys, uint2* rects, hipStream_t stream,
                       uint32_t* clear, int64_t clear_words)
{
    if(n == 0)
        return DSX_OK;
    ProjectParams p;
    p.clear = clear;
    p.clear_words = clear ? clear_words : 0;
    p.n = n;
    p.means3d = means3d;
    p.scales = scales;
    p.quats = quats;
    p.opacities = opacities;
    p.shs = shs;
    p.cov3d_precomp = cov3d_precomp;
    p.colors_precomp = colors_precomp;
    p.view = cam.view;
    p.proj = cam.proj;
    p.campos = cam.campos;
    p.splats = reinterpret_cast<float4*>(splats);
    p.radii = radii;
    p.cov3d = cov3d;
    p.block_sums = block_sums;
    p.depth_keys = depth_keys;
    p.rects = depth_keys ? rects : nullptr;
    // cpp/rasterizer_torch.cu:144-147
    p.focal_y = cam.image_height / (2 * cam.tanfovy);
    p.focal_x = cam.image_width / (2 * cam.tanfovx);
    p.c_x = cam.image_width / 2.0f;
    p.c_y = cam.image_height / 2.0f;
    p.tanfovx = cam.tanfovx;
    p.tanfovy = cam.tanfovy;
    p.scale_modifier = cam.scale_modifier;
    p.sh_degree = cam.sh_degree;
    p.sh_stride = (cam.max_sh_degree + 1) * (cam.max_sh_degree + 1) * 3;
    p.ntx = tiles_x(cam.image_width);
    p.nty = tiles_y(cam.image_height);
    const int64_t blocks = (n + kProjBlock - 1) / kProjBlock;
    {
        DSX_TIMED("project_fwd_kernel", stream);
        hipLaunchKernelGGL(project_fwd_kernel, dim3((unsigned)blocks), dim3(kProjBlock), 0, stream, p);
    }
    DSX_LAUNCH_CHECK();
    return DSX_OK;
}

} // namespace dsx
