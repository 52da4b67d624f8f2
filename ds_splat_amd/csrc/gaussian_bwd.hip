// Stages 5b + 5c for gfx950, fused: per-Gaussian backward of the SH colour (v_shs) and of the
// projection (mean, scale, rotation, cov3D) from the screen-space gradients accumulated by the
// blend backward.  Every output is linear in a Gaussian's nine accumulated sums, so a Gaussian
// whose sums are all zero (culled, hidden behind others, or outside every tile that still had
// light to give: the large majority of a dense scene) has all-zero gradients.  The outputs are
// therefore cleared by plain stores (in the whole backward by the blend kernel's wavefronts, each a
// share at its end: that kernel's arithmetic leaves the memory system idle), and this
// kernel reads the 48-byte accumulator rows of a run of Gaussians (or, in the whole backward, the
// byte per Gaussian that the blend backward set when it added a term), packs the ones with a
// non-zero sum in LDS, and works on those only: one thread per such Gaussian, the 192-byte
// v_shs rows assembled in LDS per wavefront and written with 16-byte stores.
// Math follows cpp/gsplat/backward.cu:216-393, cpp/gsplat/helpers.cuh:68-220 and
// cpp/gsplat/sh.cuh:95-186 of the reference; matrices below are indexed [row][col].
#include "dsx_common.h"

#include <atomic>

namespace dsx
{

constexpr int kShPitchB = 49;

struct GaussianBwdParams
{
    int64_t n;
    const float* means3d;
    const float* scales;
    const float* quats;
    const float4* splats;
    const float* cov3d;
    const int32_t* radii;
    const float4* grads;
    const uint8_t* marks; // per Gaussian: did the blend backward add a term? (null: look at the sums)
    const float* view;
    const float* campos;
    float* v_mean3d;
    float* v_means2d;
    float* v_shs;
    float* v_colors;
    float* v_opacity;
    float* v_scale;
    float* v_quat;
    float* v_cov3d;
    float fx, fy, glob;
    int sh_degree, num_bases;
    int conic_in_grads; // the accumulator's places 9..11 hold the conic (the forward put it there)
    int run;            // Gaussians per workgroup: a multiple of the wavefront, at most kBwdListMax
};

__device__ __forceinline__ void mat3_mul(const float (&A)[3][3], const float (&B)[3][3], float (&C)[3][3])
{
#pragma unroll
    for(int r = 0; r < 3; ++r)
#pragma unroll
        for(int c = 0; c < 3; ++c)
            C[r][c] = A[r][0] * B[0][c] + A[r][1] * B[1][c] + A[r][2] * B[2][c];
}

// real SH basis values for degrees <= deg at direction d (cpp/gsplat/sh.cuh:103-155)
__device__ __forceinline__ int sh_basis(int deg, float3 d, float* Y)
{
    Y[0] = 0.28209479177387814f;
    if(deg < 1)
        return 1;
    const float norm = sqrtf(d.x * d.x + d.y * d.y + d.z * d.z);
    const float x = d.x / norm, y = d.y / norm, z = d.z / norm;
    const float C1 = 0.4886025119029199f;
    Y[1] = -C1 * y;
    Y[2] = C1 * z;
    Y[3] = -C1 * x;
    if(deg < 2)
        return 4;
    const float xx = x * x, xy = x * y, xz = x * z, yy = y * y, yz = y * z, zz = z * z;
    Y[4] = 1.0925484305920792f * xy;
    Y[5] = -1.0925484305920792f * yz;
    Y[6] = 0.31539156525252005f * (2.f * zz - xx - yy);
    Y[7] = -1.0925484305920792f * xz;
    Y[8] = 0.5462742152960396f * (xx - yy);
    if(deg < 3)
        return 9;
    Y[9] = -0.5900435899266435f * y * (3.f * xx - yy);
    Y[10] = 2.890611442640554f * xy * z;
    Y[11] = -0.4570457994644658f * y * (4.f * zz - xx - yy);
    Y[12] = 0.3731763325901154f * z * (2.f * zz - 3.f * xx - 3.f * yy);
    Y[13] = -0.4570457994644658f * x * (4.f * zz - xx - yy);
    Y[14] = 1.445305721320277f * z * (xx - yy);
    Y[15] = -0.5900435899266435f * x * (xx - 3.f * yy);
    return 16;
}

// One wavefront per workgroup, each with its own run of Gaussians.  The runs are sized so that all
// workgroups are resident at once whenever the list below can hold a run (12 per CU: at most 168
// VGPRs, 10 KB of LDS): a scene where few Gaussians have work then costs one pass of latency (find the
// few, do them) instead of one per wave of workgroups, and a scene where all have work gives every
// wavefront the same share.
constexpr int kBwdListMax = 2048;  // longest run (its list of Gaussians with work sits in LDS)
constexpr int kBwdRunMin = 256;
constexpr int kBwdResidentPerCu = 12;

// does any of the nine sums of an accumulator row differ from zero? (a NaN does)
__device__ __forceinline__ bool any_sum(const float4& g0, const float4& g1, const float4& g2)
{
    return g0.x != 0.f || g0.y != 0.f || g0.z != 0.f || g0.w != 0.f || g1.x != 0.f || g1.y != 0.f || g1.z != 0.f ||
           g1.w != 0.f || g2.x != 0.f;
}

// what the kernel reads of one Gaussian
struct GaussianBwdInputs
{
    int64_t i; // which Gaussian
    bool live; // (false: this lane has none in this round)
    float4 g0, g1, g2;
    float3 mean;
    int radius;
    float sc[3];
    float4 quat;
    float c3[6];
    float4 conic;
};

// the inputs of entry `at + lane` of the run's list
__device__ __forceinline__ GaussianBwdInputs load_inputs(const GaussianBwdParams& p, int64_t run0,
                                                         const uint16_t* list, int at, int total, int lane)
{
    GaussianBwdInputs in = {};
    in.live = at + lane < total;
    if(!in.live)
        return in;
    const int64_t i = run0 + list[at + lane];
    in.i = i;
    in.g0 = p.grads[3 * i];
    in.g1 = p.grads[3 * i + 1];
    in.g2 = p.grads[3 * i + 2];
    in.mean = make_float3(p.means3d[3 * i], p.means3d[3 * i + 1], p.means3d[3 * i + 2]);
    in.radius = p.radii[i];
    if(p.scales)
    {
        in.sc[0] = p.scales[3 * i];
        in.sc[1] = p.scales[3 * i + 1];
        in.sc[2] = p.scales[3 * i + 2];
        in.quat = reinterpret_cast<const float4*>(p.quats)[i];
    }
    if(p.cov3d)
    {
        const float2* cs = reinterpret_cast<const float2*>(p.cov3d + 6 * i);
        const float2 c01 = cs[0], c23 = cs[1], c45 = cs[2];
        in.c3[0] = c01.x, in.c3[1] = c01.y, in.c3[2] = c23.x, in.c3[3] = c23.y, in.c3[4] = c45.x, in.c3[5] = c45.y;
    }
    // the conic: behind the sums when the forward prepared the accumulator, else from the splat record
    in.conic = p.conic_in_grads ? make_float4(in.g2.y, in.g2.z, in.g2.w, 0.f) : p.splats[3 * i + 1];
    return in;
}

__global__ __launch_bounds__(DSX_WAVE) __attribute__((amdgpu_waves_per_eu(3, 3))) void gaussian_bwd_kernel(const GaussianBwdParams p)
{
    __shared__ float rows[32 * kShPitchB];
    __shared__ uint16_t s_list[kBwdListMax]; // the run's Gaussians with work, in index order

    const int lane = threadIdx.x;
    const int64_t run0 = (int64_t)blockIdx.x * p.run;
    const int run = (int)min((int64_t)p.run, p.n - run0);

    // ---- which Gaussians of the run have anything to propagate --------------------------------
    int total = 0;
    for(int first = 0; first < run; first += 4 * DSX_WAVE)
    {
        bool work[4];
#pragma unroll
        for(int j = 0; j < 4; ++j)
        {
            const int local = first + j * DSX_WAVE + lane;
            const int64_t i = run0 + local;
            work[j] = false;
            if(local < run)
                work[j] = p.marks ? p.marks[i] != 0 : any_sum(p.grads[3 * i], p.grads[3 * i + 1], p.grads[3 * i + 2]);
        }
#pragma unroll
        for(int j = 0; j < 4; ++j)
        {
            const uint64_t mask = __ballot(work[j]);
            if(work[j])
                s_list[total + __popcll(mask & ((1ull << lane) - 1ull))] = (uint16_t)(first + j * DSX_WAVE + lane);
            total += __popcll(mask);
        }
    }
    __syncthreads(); // (one wavefront: orders the LDS writes before the reads)

    // The inputs of a round are fetched one round ahead: the wavefronts of a launch start together
    // and stay in step, all of them waiting for memory or all of them computing.  (Measured with every
    // Gaussian of 3 M having work: 0.273 ms either way; the fetch ahead costs nothing and stays.)
    const int row_floats = p.num_bases * 3;
    GaussianBwdInputs ahead = load_inputs(p, run0, s_list, 0, total, lane);
    for(int first = 0; first < total; first += DSX_WAVE)
    {
        const GaussianBwdInputs in = ahead;
        ahead = load_inputs(p, run0, s_list, first + DSX_WAVE, total, lane);
        const bool live = in.live;
        const int64_t i = in.i;

        float v_rgb[3] = {0.f, 0.f, 0.f};
        const float3 mean = in.mean;
        if(live)
        {
            const float4 g0 = in.g0, g1 = in.g1;
            const float v_x = g0.x, v_y = g0.y;
            const float vc[3] = {g0.z, g0.w, g1.x};
            const float v_o = g1.y;
            v_rgb[0] = g1.z;
            v_rgb[1] = g1.w;
            v_rgb[2] = in.g2.x;

            // straight copies: screen-space mean gradient (z column zero), colour and opacity
            // (every output is optional: a null pointer means that the caller has no use for it)
            if(p.v_means2d)
            {
                p.v_means2d[3 * i] = v_x;
                p.v_means2d[3 * i + 1] = v_y;
                p.v_means2d[3 * i + 2] = 0.f;
            }
            if(p.v_colors)
            {
                p.v_colors[3 * i] = v_rgb[0];
                p.v_colors[3 * i + 1] = v_rgb[1];
                p.v_colors[3 * i + 2] = v_rgb[2];
            }
            if(p.v_opacity)
                p.v_opacity[i] = v_o;

            float vm[3] = {0.f, 0.f, 0.f}, vs[3] = {0.f, 0.f, 0.f}, vq[4] = {0.f, 0.f, 0.f, 0.f};
            float vc3[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            if(in.radius > 0)
            {
                const float* V = p.view;
                const float R[3][3] = {{V[0], V[1], V[2]}, {V[4], V[5], V[6]}, {V[8], V[9], V[10]}};
                const float t[3] = {R[0][0] * mean.x + R[0][1] * mean.y + R[0][2] * mean.z + V[3],
                                    R[1][0] * mean.x + R[1][1] * mean.y + R[1][2] * mean.z + V[7],
                                    R[2][0] * mean.x + R[2][1] * mean.y + R[2][2] * mean.z + V[11]};
                // pixel mean -> view position -> world position
                {
                    const float rw = 1.f / (t[2] + 1e-6f);
                    const float vpx = p.fx * v_x, vpy = p.fy * v_y;
                    const float vv[3] = {vpx * rw, vpy * rw, -(vpx * t[0] + vpy * t[1]) * rw * rw};
#pragma unroll
                    for(int c = 0; c < 3; ++c)
                        vm[c] = R[0][c] * vv[0] + R[1][c] * vv[1] + R[2][c] * vv[2];
                }
                // conic -> cov2d:  v_Sigma = -X G X, X = conic, G = symmetrised v_conic
                float v_cov2d[3];
                {
                    const float4 q1 = in.conic;
                    const float X[2][2] = {{q1.x, q1.y}, {q1.y, q1.z}};
                    const float G[2][2] = {{vc[0], 0.5f * vc[1]}, {0.5f * vc[1], vc[2]}};
                    float M[2][2], N[2][2];
#pragma unroll
                    for(int r = 0; r < 2; ++r)
#pragma unroll
                        for(int c = 0; c < 2; ++c)
                            M[r][c] = X[r][0] * G[0][c] + X[r][1] * G[1][c];
#pragma unroll
                    for(int r = 0; r < 2; ++r)
#pragma unroll
                        for(int c = 0; c < 2; ++c)
                            N[r][c] = M[r][0] * X[0][c] + M[r][1] * X[1][c];
                    v_cov2d[0] = -N[0][0];
                    v_cov2d[1] = -(N[0][1] + N[1][0]);
                    v_cov2d[2] = -N[1][1];
                }
                // EWA projection: cov2d = T Sigma T^T, T = J R (unclamped t, rz = 1/t.z)
                {
                    const float rz = 1.f / t[2];
                    const float rz2 = rz * rz;
                    const float J[2][3] = {{p.fx * rz, 0.f, -p.fx * t[0] * rz2}, {0.f, p.fy * rz, -p.fy * t[1] * rz2}};
                    float T[2][3];
#pragma unroll
                    for(int r = 0; r < 2; ++r)
#pragma unroll
                        for(int c = 0; c < 3; ++c)
                            T[r][c] = J[r][0] * R[0][c] + J[r][1] * R[1][c] + J[r][2] * R[2][c];
                    // the covariance the forward projected: stored by it, or rebuilt here from scale and
                    // rotation with the forward's own routine (same bits; 24 bytes per Gaussian less to
                    // write there and to read here)
                    float c3[6];
                    if(p.cov3d)
                    {
#pragma unroll
                        for(int c = 0; c < 6; ++c)
                            c3[c] = in.c3[c];
                    }
                    else
                        cov3d_from_scale_rot(in.sc, in.quat, p.glob, c3);
                    const float S[3][3] = {{c3[0], c3[1], c3[2]}, {c3[1], c3[3], c3[4]}, {c3[2], c3[4], c3[5]}};
                    const float Gc[2][2] = {{v_cov2d[0], 0.5f * v_cov2d[1]}, {0.5f * v_cov2d[1], v_cov2d[2]}};
                    // GT = Gc T (2x3)
                    float GT[2][3];
#pragma unroll
                    for(int r = 0; r < 2; ++r)
#pragma unroll
                        for(int c = 0; c < 3; ++c)
                            GT[r][c] = Gc[r][0] * T[0][c] + Gc[r][1] * T[1][c];
                    // v_Sigma = T^T Gc T (3x3)
                    float vS[3][3];
#pragma unroll
                    for(int r = 0; r < 3; ++r)
#pragma unroll
                        for(int c = 0; c < 3; ++c)
                            vS[r][c] = T[0][r] * GT[0][c] + T[1][r] * GT[1][c];
                    vc3[0] = vS[0][0];
                    vc3[1] = vS[0][1] + vS[1][0];
                    vc3[2] = vS[0][2] + vS[2][0];
                    vc3[3] = vS[1][1];
                    vc3[4] = vS[1][2] + vS[2][1];
                    vc3[5] = vS[2][2];
                    // v_T = Gc T Sigma^T + Gc^T T Sigma  (2x3); v_J = v_T R^T (2x3)
                    float vT[2][3];
#pragma unroll
                    for(int r = 0; r < 2; ++r)
#pragma unroll
                        for(int c = 0; c < 3; ++c)
                        {
                            const float a = GT[r][0] * S[c][0] + GT[r][1] * S[c][1] + GT[r][2] * S[c][2];
                            const float b = GT[r][0] * S[0][c] + GT[r][1] * S[1][c] + GT[r][2] * S[2][c];
                            vT[r][c] = a + b;
                        }
                    float vJ[2][3];
#pragma unroll
                    for(int r = 0; r < 2; ++r)
#pragma unroll
                        for(int c = 0; c < 3; ++c)
                            vJ[r][c] = vT[r][0] * R[c][0] + vT[r][1] * R[c][1] + vT[r][2] * R[c][2];
                    const float rz3 = rz2 * rz;
                    const float vt[3] = {-p.fx * rz2 * vJ[0][2], -p.fy * rz2 * vJ[1][2],
                                         -p.fx * rz2 * vJ[0][0] + 2.f * p.fx * t[0] * rz3 * vJ[0][2] -
                                             p.fy * rz2 * vJ[1][1] + 2.f * p.fy * t[1] * rz3 * vJ[1][2]};
#pragma unroll
                    for(int c = 0; c < 3; ++c)
                        vm[c] += vt[0] * R[0][c] + vt[1] * R[1][c] + vt[2] * R[2][c];
                }
                // cov3d = (Rq S)(Rq S)^T -> scale, quaternion (raw quaternion, no normalisation)
                if(p.scales != nullptr)
                {
                    const float vV[3][3] = {{vc3[0], 0.5f * vc3[1], 0.5f * vc3[2]},
                                            {0.5f * vc3[1], vc3[3], 0.5f * vc3[4]},
                                            {0.5f * vc3[2], 0.5f * vc3[4], vc3[5]}};
                    const float4 q = in.quat;
                    const float w = q.x, x = q.y, y = q.z, z = q.w;
                    const float Rq[3][3] = {
                        {1.f - 2.f * (y * y + z * z), 2.f * (x * y - w * z), 2.f * (x * z + w * y)},
                        {2.f * (x * y + w * z), 1.f - 2.f * (x * x + z * z), 2.f * (y * z - w * x)},
                        {2.f * (x * z - w * y), 2.f * (y * z + w * x), 1.f - 2.f * (x * x + y * y)}};
                    const float s[3] = {p.glob * in.sc[0], p.glob * in.sc[1], p.glob * in.sc[2]};
                    float M[3][3], vM[3][3], vR[3][3];
#pragma unroll
                    for(int r = 0; r < 3; ++r)
#pragma unroll
                        for(int c = 0; c < 3; ++c)
                            M[r][c] = Rq[r][c] * s[c];
                    mat3_mul(vV, M, vM);
#pragma unroll
                    for(int r = 0; r < 3; ++r)
#pragma unroll
                        for(int c = 0; c < 3; ++c)
                            vM[r][c] *= 2.f;
#pragma unroll
                    for(int c = 0; c < 3; ++c)
                        vs[c] = (Rq[0][c] * vM[0][c] + Rq[1][c] * vM[1][c] + Rq[2][c] * vM[2][c]) * p.glob;
#pragma unroll
                    for(int r = 0; r < 3; ++r)
#pragma unroll
                        for(int c = 0; c < 3; ++c)
                            vR[r][c] = vM[r][c] * s[c];
                    vq[0] = 2.f * (x * (vR[2][1] - vR[1][2]) + y * (vR[0][2] - vR[2][0]) + z * (vR[1][0] - vR[0][1]));
                    vq[1] = 2.f * (-2.f * x * (vR[1][1] + vR[2][2]) + y * (vR[1][0] + vR[0][1]) +
                                   z * (vR[2][0] + vR[0][2]) + w * (vR[2][1] - vR[1][2]));
                    vq[2] = 2.f * (x * (vR[1][0] + vR[0][1]) - 2.f * y * (vR[0][0] + vR[2][2]) +
                                   z * (vR[2][1] + vR[1][2]) + w * (vR[0][2] - vR[2][0]));
                    vq[3] = 2.f * (x * (vR[2][0] + vR[0][2]) + y * (vR[2][1] + vR[1][2]) -
                                   2.f * z * (vR[0][0] + vR[1][1]) + w * (vR[1][0] - vR[0][1]));
                }
            }
            if(p.v_mean3d)
#pragma unroll
                for(int c = 0; c < 3; ++c)
                    p.v_mean3d[3 * i + c] = vm[c];
            if(p.v_scale)
#pragma unroll
                for(int c = 0; c < 3; ++c)
                    p.v_scale[3 * i + c] = vs[c];
            if(p.v_quat)
                reinterpret_cast<float4*>(p.v_quat)[i] = make_float4(vq[0], vq[1], vq[2], vq[3]);
            if(p.v_cov3d)
            {
                float2* o = reinterpret_cast<float2*>(p.v_cov3d + 6 * i);
                o[0] = make_float2(vc3[0], vc3[1]);
                o[1] = make_float2(vc3[2], vc3[3]);
                o[2] = make_float2(vc3[4], vc3[5]);
            }
        }

        // ---- v_shs[b][c] = Y_b(dir) * v_rgb[c], zero above the active degree -------------------
        if(p.v_shs == nullptr)
            continue;
        float Y[16];
        int nb = 0;
        if(live)
        {
            const float3 d = make_float3(mean.x - p.campos[0], mean.y - p.campos[1], mean.z - p.campos[2]);
            nb = min(sh_basis(p.sh_degree, d, Y), p.num_bases);
        }
        // the rows pass through LDS half a wavefront at a time (32 rows: 6 KB, so that twelve
        // workgroups fit a CU) and go out 16 bytes per lane: twelve lanes per row of 48 floats
        const int nrows = min(DSX_WAVE, total - first);
#pragma unroll
        for(int half = 0; half < 2; ++half)
        {
            __syncthreads(); // the rows of the last half have been read
            if(live && (lane >> 5) == half)
            {
                float* r = rows + (lane & 31) * kShPitchB;
#pragma unroll
                for(int b = 0; b < 16; ++b)
                {
                    if(b < p.num_bases)
                    {
                        const float yb = b < nb ? Y[b] : 0.f;
                        r[3 * b] = b < nb ? yb * v_rgb[0] : 0.f;
                        r[3 * b + 1] = b < nb ? yb * v_rgb[1] : 0.f;
                        r[3 * b + 2] = b < nb ? yb * v_rgb[2] : 0.f;
                    }
                }
            }
            __syncthreads();
            const int half_rows = max(0, min(32, nrows - 32 * half));
            const uint16_t* ids = s_list + first + 32 * half;
            if(row_floats == 48 && ((uintptr_t)p.v_shs & 15) == 0)
            {
                const int chunks = half_rows * 12;
#pragma unroll
                for(int j = 0; j < 6; ++j)
                {
                    const int e = j * 64 + lane;
                    if(e < chunks)
                    {
                        const int row = e / 12;
                        const int c4 = e - row * 12;
                        const float* s = rows + row * kShPitchB + c4 * 4;
                        float4* dst = reinterpret_cast<float4*>(p.v_shs + (run0 + ids[row]) * 48);
                        nt_store_f4(dst + c4, make_float4(s[0], s[1], s[2], s[3]));
                    }
                }
            }
            else
            {
                const int count = half_rows * row_floats;
                for(int e = lane; e < count; e += 64)
                {
                    const int row = e / row_floats;
                    const int c = e - row * row_floats;
                    p.v_shs[(run0 + ids[row]) * row_floats + c] = rows[row * kShPitchB + c];
                }
            }
        }
    }
}

// ---- the outputs' zeros as a launch of their own (the stage entry point; the whole backward has
// them written by the blend kernel's wavefronts instead, see zero_share) ---------------------------
__global__ __launch_bounds__(kProjBlock) void zero_outputs_kernel(const ZeroJobs jobs)
{
    zero_share(jobs, blockIdx.x, gridDim.x, threadIdx.x, kProjBlock);
}

int launch_zero_outputs(const ZeroJobs& jobs, hipStream_t stream)
{
    if(!jobs.any)
        return DSX_OK;
    // at least 16 stores per thread, at most eight workgroups per CU
    const int64_t want = (jobs.end[7] + (int64_t)kProjBlock * 16 - 1) / ((int64_t)kProjBlock * 16);
    const unsigned blocks = (unsigned)max((int64_t)1, min(want, (int64_t)2048));
    {
        DSX_TIMED("zero_outputs_kernel", stream);
        hipLaunchKernelGGL(zero_outputs_kernel, dim3(blocks), dim3(kProjBlock), 0, stream, jobs);
    }
    DSX_LAUNCH_CHECK();
    return DSX_OK;
}

// CUs of the current device (asked once per device; 256 if the question fails)
static int compute_units()
{
    constexpr int kMaxDevices = 64;
    static std::atomic<int> known[kMaxDevices] = {};
    int device = 0;
    if(hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices)
        return 256;
    int cus = known[device].load(std::memory_order_relaxed);
    if(cus == 0)
    {
        if(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
        {
            (void)hipGetLastError();
            cus = 256;
        }
        known[device].store(cus, std::memory_order_relaxed);
    }
    return cus;
}

int launch_gaussian_bwd(const dsx_camera& cam, int64_t n, int num_bases, const float* means3d, const float* scales,
                        const float* quats, const float* splats, const float* cov3d, const int32_t* radii,
                        const float* grads, float* v_mean3d, float* v_means2d, float* v_shs, float* v_colors,
                        float* v_opacity, float* v_scale, float* v_quat, float* v_cov3d, hipStream_t stream,
                        bool conic_in_grads, bool outputs_cleared, bool with_marks)
{
    if(n == 0)
        return DSX_OK;
    if(!outputs_cleared)
        if(int rc = launch_zero_outputs(make_zero_jobs(n, num_bases, v_mean3d, v_means2d, v_shs, v_colors, v_opacity,
                                                       v_scale, v_quat, v_cov3d),
                                        stream))
            return rc;
    GaussianBwdParams p;
    p.n = n;
    p.means3d = means3d;
    p.scales = scales;
    p.quats = quats;
    p.splats = reinterpret_cast<const float4*>(splats);
    p.cov3d = cov3d;
    p.radii = radii;
    p.grads = reinterpret_cast<const float4*>(grads);
    p.marks = with_marks ? grad_marks(const_cast<float*>(grads), n) : nullptr;
    p.view = cam.view;
    p.campos = cam.campos;
    p.v_mean3d = v_mean3d;
    p.v_means2d = v_means2d;
    p.v_shs = v_shs;
    p.v_colors = v_colors;
    p.v_opacity = v_opacity;
    p.v_scale = v_scale;
    p.v_quat = v_quat;
    p.v_cov3d = v_cov3d;
    // the reference's backward derives the focal lengths through atan/tan
    // (cpp/rasterizer_torch.cu:78-81,297-298), an ulp-level difference from the forward's
    const float fovx = 2 * atanf(cam.tanfovx);
    const float fovy = 2 * atanf(cam.tanfovy);
    p.fx = (float)cam.image_width / (2.0f * tanf(fovx / 2.0f));
    p.fy = (float)cam.image_height / (2.0f * tanf(fovy / 2.0f));
    p.glob = cam.scale_modifier;
    p.sh_degree = cam.sh_degree;
    p.num_bases = num_bases;
    p.conic_in_grads = conic_in_grads ? 1 : 0;
    // runs that make all workgroups resident at once, if the list can hold such a run
    const int64_t resident = (int64_t)compute_units() * kBwdResidentPerCu;
    const int64_t even = ((n + resident - 1) / resident + DSX_WAVE - 1) / DSX_WAVE * DSX_WAVE;
    p.run = (int)max((int64_t)kBwdRunMin, min(even, (int64_t)kBwdListMax));
    const int64_t blocks = (n + p.run - 1) / p.run;
    {
        DSX_TIMED("gaussian_bwd_kernel", stream);
        hipLaunchKernelGGL(gaussian_bwd_kernel, dim3((unsigned)blocks), dim3(DSX_WAVE), 0, stream, p);
    }
    DSX_LAUNCH_CHECK();
    return DSX_OK;
}

} // namespace dsx
