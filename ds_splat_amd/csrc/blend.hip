// Stages 4 and 5a for gfx950: per-tile alpha blending, forward (front to back) and backward
// (back to front).  One 256-thread workgroup (4 wave64, each covering 4 pixel rows of 16)
// per 16x16 tile; batches of 256 sorted entries are gathered into LDS as two float4 arrays
// plus one float array, so the inner loop reads each entry with two 128-bit and one 32-bit
// LDS broadcast.
#include "dsx_common.h"

namespace dsx
{

constexpr float kAlphaThreshold = 1.0f / 255.0f;

// exp through the hardware base-2 exponential (the reference is built with fast-math)
__device__ __forceinline__ float fast_exp(float x)
{
    return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
}

// -----------------------------------------------------------------------------------------
// forward: cpp/rasterizer_kernels.cu:341-431
// -----------------------------------------------------------------------------------------
__global__ __launch_bounds__(kTilePixels) void blend_fwd_kernel(const int32_t* __restrict__ ranges,
                                                                const int32_t* __restrict__ ids,
                                                                const float4* __restrict__ splats,
                                                                float* __restrict__ image,
                                                                float* __restrict__ final_T,
                                                                int32_t* __restrict__ final_idx, int W, int H,
                                                                int ntx)
{
    __shared__ float4 s_a[kTilePixels]; // pixel x, pixel y, conic a, conic b
    __shared__ float4 s_b[kTilePixels]; // conic c, opacity, red, green
    __shared__ float s_c[kTilePixels];  // blue

    const int tid = threadIdx.x;
    const int tile = blockIdx.x;
    const int tx = tile % ntx;
    const int ty = tile / ntx;
    const int x = tx * kTile + (tid & 15);
    const int y = ty * kTile + (tid >> 4);
    const bool inside = x < W && y < H;
    const float pxf = (float)x + 0.5f;
    const float pyf = (float)y + 0.5f;

    const int start = ranges[tile];
    const int end = ranges[tile + 1];

    float T = 1.0f, cr = 0.0f, cg = 0.0f, cb = 0.0f;
    int last = 0;
    bool done = !inside;

    for(int b = start; b < end; b += kTilePixels)
    {
        if(__syncthreads_and(done))
            break;
        const int e = b + tid;
        if(e < end)
        {
            const int g = ids[e];
            const float4* rec = splats + 3 * (int64_t)g;
            const float4 q0 = rec[0], q1 = rec[1], q2 = rec[2];
            s_a[tid] = make_float4(q0.x, q0.y, q1.x, q1.y);
            s_b[tid] = make_float4(q1.z, q1.w, q2.x, q2.y);
            s_c[tid] = q2.z;
        }
        __syncthreads();
        const int cnt = min(kTilePixels, end - b);
        if(!done)
        {
            for(int i = 0; i < cnt; ++i)
            {
                const float4 A = s_a[i];
                const float4 B = s_b[i];
                const float dx = pxf - A.x;
                const float dy = pyf - A.y;
                const float power = -0.5f * (A.z * dx * dx + B.x * dy * dy) - A.w * dx * dy;
                const float alpha = fminf(0.999f, B.y * fast_exp(power));
                if(power >= 0.0f || alpha < kAlphaThreshold)
                    continue;
                const float Tn = (1.0f - alpha) * T;
                if(Tn < 0.0001f)
                {
                    done = true;
                    break;
                }
                const float vis = alpha * T;
                cr += vis * B.z;
                cg += vis * B.w;
                cb += vis * s_c[i];
                T = Tn;
                last = b + i;
            }
        }
    }

    if(inside)
    {
        const int64_t pix = (int64_t)y * W + x;
        image[3 * pix] = cr;
        image[3 * pix + 1] = cg;
        image[3 * pix + 2] = cb;
        final_T[pix] = T;
        final_idx[pix] = last;
    }
}

int launch_blend_fwd(const dsx_camera& cam, const int32_t* ranges, const int32_t* sorted_ids, const float* splats,
                     float* image, float* final_T, int32_t* final_idx, hipStream_t stream)
{
    const int ntx = tiles_x(cam.image_width), nty = tiles_y(cam.image_height);
    if(ntx * nty == 0)
        return DSX_OK;
    {
        DSX_TIMED("blend_fwd_kernel", stream);
        hipLaunchKernelGGL(blend_fwd_kernel, dim3(ntx * nty), dim3(kTilePixels), 0, stream, ranges, sorted_ids,
                           reinterpret_cast<const float4*>(splats), image, final_T, final_idx, cam.image_width,
                           cam.image_height, ntx);
    }
    DSX_LAUNCH_CHECK();
    return DSX_OK;
}

// -----------------------------------------------------------------------------------------
// backward: cpp/gsplat/backward.cu:25-202
// -----------------------------------------------------------------------------------------

// Sum over the 64 lanes of a wavefront with data-parallel-primitive adds only (no LDS
// traffic): two quad permutes, two row mirrors, then the row broadcasts.  The total is valid
// in lane 63.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_add(float v)
{
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, kRowMask, 0xf, false);
    return v + __int_as_float(moved);
}

__device__ __forceinline__ float wave_sum_to_lane63(float v)
{
    v = dpp_add<0xB1, 0xf>(v);  // quad_perm [1,0,3,2]
    v = dpp_add<0x4E, 0xf>(v);  // quad_perm [2,3,0,1]
    v = dpp_add<0x141, 0xf>(v); // row_half_mirror
    v = dpp_add<0x140, 0xf>(v); // row_mirror: every lane of a row holds the row sum
    v = dpp_add<0x142, 0xa>(v); // row_bcast:15 into rows 1 and 3
    v = dpp_add<0x143, 0xc>(v); // row_bcast:31 into rows 2 and 3
    return v;
}

constexpr int kGradVals = 9;

__global__ __launch_bounds__(kTilePixels) void blend_bwd_kernel(
    const int32_t* __restrict__ ranges, const int32_t* __restrict__ ids, const float4* __restrict__ splats,
    const float* __restrict__ final_T, const int32_t* __restrict__ final_idx, const float* __restrict__ v_image,
    const float* __restrict__ bg, float* grads, int W, int H, int ntx)
{
    __shared__ float4 s_a[kTilePixels]; // pixel x, pixel y, conic a, conic b
    __shared__ float4 s_b[kTilePixels]; // conic c, opacity, red, green
    __shared__ float s_c[kTilePixels];  // blue
    __shared__ int s_id[kTilePixels];
    __shared__ float s_acc[kTilePixels * kGradVals]; // per-entry sums over the four wavefronts
    __shared__ int s_wave_max[4];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int tile = blockIdx.x;
    const int tx = tile % ntx;
    const int ty = tile / ntx;
    const int x = tx * kTile + (tid & 15);
    const int y = ty * kTile + (tid >> 4);
    const bool inside = x < W && y < H;
    const float pxf = (float)x + 0.5f;
    const float pyf = (float)y + 0.5f;
    const int64_t pix = inside ? (int64_t)y * W + x : 0;

    const float T_final = inside ? final_T[pix] : 0.0f;
    const int bin_final = inside ? final_idx[pix] : -1;
    float vo0 = 0.f, vo1 = 0.f, vo2 = 0.f;
    if(inside)
    {
        vo0 = v_image[3 * pix];
        vo1 = v_image[3 * pix + 1];
        vo2 = v_image[3 * pix + 2];
    }
    // -T_final * bg . v_out  (background term of cpp/gsplat/backward.cu:160-164, times ra later)
    const float bg_term = -T_final * (bg[0] * vo0 + bg[1] * vo1 + bg[2] * vo2);

    const int start = ranges[tile];
    const int end = ranges[tile + 1];

    // last entry any pixel of this wavefront / of this tile blended
    int m = bin_final;
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        m = max(m, __shfl_xor(m, o, DSX_WAVE));
    if(lane == 0)
        s_wave_max[wave] = m;
    __syncthreads();
    const int wave_last = m;
    const int tile_last = max(max(s_wave_max[0], s_wave_max[1]), max(s_wave_max[2], s_wave_max[3]));
    const int hi = min(end - 1, tile_last);

    float T = T_final;
    float buf0 = 0.f, buf1 = 0.f, buf2 = 0.f;

    for(int top = hi; top >= start; top -= kTilePixels)
    {
        __syncthreads(); // previous batch fully consumed (staging and accumulators)
        const int e = top - tid;
        if(e >= start)
        {
            const int g = ids[e];
            const float4* rec = splats + 3 * (int64_t)g;
            const float4 q0 = rec[0], q1 = rec[1], q2 = rec[2];
            s_a[tid] = make_float4(q0.x, q0.y, q1.x, q1.y);
            s_b[tid] = make_float4(q1.z, q1.w, q2.x, q2.y);
            s_c[tid] = q2.z;
            s_id[tid] = g;
        }
#pragma unroll
        for(int j = 0; j < kGradVals; ++j)
            s_acc[j * kTilePixels + tid] = 0.f;
        __syncthreads();
        const int cnt = min(kTilePixels, top - start + 1);
        // entries beyond what any lane of this wavefront blended are skipped outright
        for(int t = max(0, top - wave_last); t < cnt; ++t)
        {
            const int idx = top - t;
            bool valid = idx <= bin_final;
            float alpha = 0.f, vis = 0.f, dx = 0.f, dy = 0.f;
            const float4 A = s_a[t];
            const float4 B = s_b[t];
            if(valid)
            {
                dx = A.x - pxf;
                dy = A.y - pyf;
                const float sigma = 0.5f * (A.z * dx * dx + B.x * dy * dy) + A.w * dx * dy;
                vis = fast_exp(-sigma);
                alpha = fminf(0.99f, B.y * vis);
                if(sigma < 0.0f || alpha < kAlphaThreshold)
                    valid = false;
            }
            if(__ballot(valid) == 0)
                continue;
            float g[kGradVals] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if(valid)
            {
                const float ra = __builtin_amdgcn_rcpf(1.0f - alpha);
                T *= ra;
                const float fac = alpha * T;
                g[6] = fac * vo0;
                g[7] = fac * vo1;
                g[8] = fac * vo2;
                const float blue = s_c[t];
                float v_alpha = (B.z * T - buf0 * ra) * vo0;
                v_alpha += (B.w * T - buf1 * ra) * vo1;
                v_alpha += (blue * T - buf2 * ra) * vo2;
                v_alpha += bg_term * ra;
                buf0 += B.z * fac;
                buf1 += B.w * fac;
                buf2 += blue * fac;
                const float v_sigma = -B.y * vis * v_alpha;
                g[0] = v_sigma * (A.z * dx + A.w * dy);
                g[1] = v_sigma * (A.w * dx + B.x * dy);
                g[2] = 0.5f * v_sigma * dx * dx;
                g[3] = v_sigma * dx * dy;
                g[4] = 0.5f * v_sigma * dy * dy;
                g[5] = vis * v_alpha;
            }
#pragma unroll
            for(int j = 0; j < kGradVals; ++j)
                g[j] = wave_sum_to_lane63(g[j]);
            if(lane == 63)
            {
#pragma unroll
                for(int j = 0; j < kGradVals; ++j)
                    atomicAdd(&s_acc[j * kTilePixels + t], g[j]);
            }
        }
        __syncthreads();
        // one set of global atomics per (tile, entry): thread t flushes entry t
        if(tid < cnt)
        {
            float v[kGradVals];
            bool any = false;
#pragma unroll
            for(int j = 0; j < kGradVals; ++j)
            {
                v[j] = s_acc[j * kTilePixels + tid];
                any = any || v[j] != 0.f;
            }
            if(any)
            {
                float* dst = grads + (int64_t)s_id[tid] * DSX_GRAD_FLOATS;
#pragma unroll
                for(int j = 0; j < kGradVals; ++j)
                    unsafeAtomicAdd(dst + j, v[j]);
            }
        }
    }
}

int launch_blend_bwd(const dsx_camera& cam, int64_t n, const int32_t* ranges, const int32_t* sorted_ids,
                     const float* splats, const float* final_T, const int32_t* final_idx, const float* v_image,
                     float* grads, hipStream_t stream)
{
    int rc = launch_fill_u32(reinterpret_cast<uint32_t*>(grads), n * DSX_GRAD_FLOATS, 0u, stream);
    if(rc)
        return rc;
    const int ntx = tiles_x(cam.image_width), nty = tiles_y(cam.image_height);
    if(ntx * nty == 0 || n == 0)
        return DSX_OK;
    {
        DSX_TIMED("blend_bwd_kernel", stream);
        hipLaunchKernelGGL(blend_bwd_kernel, dim3(ntx * nty), dim3(kTilePixels), 0, stream, ranges, sorted_ids,
                           reinterpret_cast<const float4*>(splats), final_T, final_idx, v_image, cam.bg, grads,
                           cam.image_width, cam.image_height, ntx);
    }
    DSX_LAUNCH_CHECK();
    return DSX_OK;
}

} // namespace dsx
