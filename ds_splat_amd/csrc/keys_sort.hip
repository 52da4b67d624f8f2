// Stages 2 and 3 for gfx950: block-sum scan, tile-key emission, 64-bit LSD radix sort
// (one-sweep: one global histogram pass, then one chained-scan scatter pass per digit) and
// tile-range identification.  Integer work only; everything is HBM-bandwidth bound.
#include "dsx_common.h"

#include <mutex>

namespace dsx
{

// ---------------------------------------------------------------------------------------
// small wave/block primitives
// ---------------------------------------------------------------------------------------

__device__ __forceinline__ uint32_t wave_incl_scan_u32(uint32_t v, int)
{
    return wave_incl_scan_u32(v);
}

// lanes of the wavefront that hold the same (up to 9-bit) digit and are valid; call in uniform
// flow.  Per digit bit: one sign-extending bit extract, one compare (the ballot) and, for each
// half of the lane mask, one three-input boolean op  mask & ~(ballot ^ bit).
__device__ __forceinline__ uint64_t match_digit(uint32_t d, bool valid)
{
    const uint64_t v = __ballot(valid);
    uint32_t lo = (uint32_t)v, hi = (uint32_t)(v >> 32);
#pragma unroll
    for(int b = 0; b < kRadixBitsMax; ++b)
    {
        const uint32_t x = (uint32_t)(((int32_t)(d << (31 - b))) >> 31); // all ones where bit b is set
        const uint64_t m = __ballot(x != 0);
        lo &= ~((uint32_t)m ^ x);
        hi &= ~((uint32_t)(m >> 32) ^ x);
    }
    return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ uint64_t lanemask_lt(int lane)
{
    return (1ull << lane) - 1ull;
}

// Sortable image of a key: negative keys (tile field all ones, produced by negative depths)
// sort first in signed order, so they take tile slot 0 and every real tile moves up by one.
__device__ __forceinline__ uint64_t sortable(int64_t key)
{
    return key < 0 ? ((uint64_t)key & 0xffffffffull) : (uint64_t)key + (1ull << 32);
}

// ---------------------------------------------------------------------------------------
// fill
// ---------------------------------------------------------------------------------------

__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* p, int64_t count, uint32_t value)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for(int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride)
        p[i] = value;
}

int launch_fill_u32(uint32_t* p, int64_t count, uint32_t value, hipStream_t stream)
{
    if(count <= 0)
        return DSX_OK;
    const int64_t blocks = min((int64_t)4096, (count + 255) / 256);
    {
        DSX_TIMED("fill_u32_kernel", stream);
        hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p, count, value);
    }
    DSX_LAUNCH_CHECK();
    return DSX_OK;
}

// ---------------------------------------------------------------------------------------
// exclusive scan of a (short) uint32 array by one workgroup
// ---------------------------------------------------------------------------------------

constexpr int kScanThreads = 1024;
constexpr int kScanItems = 4;

__global__ __launch_bounds__(kScanThreads) void scan_u32_kernel(uint32_t* data, int64_t count, uint32_t* total)
{
    __shared__ __attribute__((aligned(16))) uint32_t wave_tot[kScanThreads / DSX_WAVE];
    __shared__ uint32_t carry_s;
    __shared__ unsigned long long total64; // the true sum: the 32-bit prefixes wrap silently, the total must not
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    if(tid == 0)
    {
        carry_s = 0;
        total64 = 0ull;
    }
    unsigned long long mine64 = 0ull;
    __syncthreads();
    for(int64_t base = 0; base < count; base += kScanThreads * kScanItems)
    {
        const int64_t i0 = base + (int64_t)tid * kScanItems;
        uint32_t v[kScanItems];
        uint32_t sum = 0;
#pragma unroll
        for(int j = 0; j < kScanItems; ++j)
        {
            v[j] = (i0 + j < count) ? data[i0 + j] : 0u;
            sum += v[j];
            mine64 += v[j];
        }
        const uint32_t incl = wave_incl_scan_u32(sum, lane);
        if(lane == 63)
            wave_tot[wave] = incl;
        __syncthreads();
        const uint32_t wave_prefix = sum_of_waves_before<kScanThreads / DSX_WAVE>(wave_tot, wave);
        uint32_t run = carry_s + wave_prefix + incl - sum;
#pragma unroll
        for(int j = 0; j < kScanItems; ++j)
        {
            if(i0 + j < count)
                data[i0 + j] = run;
            run += v[j];
        }
        __syncthreads();
        if(tid == kScanThreads - 1)
            carry_s = run;
        __syncthreads();
    }
    // one LDS atomic per wavefront (1024 same-address atomics would cost more than the scan)
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        mine64 += __shfl_xor(mine64, o, DSX_WAVE);
    if(lane == 0 && mine64)
        atomicAdd(&total64, mine64);
    __syncthreads();
    if(tid == 0)
        *total = total64 > 0xffffffffull ? 0xffffffffu : (uint32_t)total64; // saturates: callers reject counts >= 2^30
}

int launch_scan_u32(int64_t count, uint32_t* data, uint32_t* total, hipStream_t stream)
{
    {
        DSX_TIMED("scan_u32_kernel", stream);
        hipLaunchKernelGGL(scan_u32_kernel, dim3(1), dim3(kScanThreads), 0, stream, data, count, total);
    }
    DSX_LAUNCH_CHECK();
    return DSX_OK;
}

// ---------------------------------------------------------------------------------------
// key emission: one workgroup per 256 Gaussians (the same partition as the projection), one
// thread per OUTPUT key, so stores are contiguous however uneven the per-Gaussian tile counts
// ---------------------------------------------------------------------------------------

__global__ __launch_bounds__(kProjBlock) void emit_keys_kernel(const float4* __restrict__ splats,
                                                               const uint32_t* __restrict__ block_offsets,
                                                               int64_t n, int64_t k, int ntx, int nty,
                                                               int64_t* __restrict__ keys,
                                                               int32_t* __restrict__ values)
{
    __shared__ uint32_t s_off[kProjBlock + 1];
    __shared__ int s_sx[kProjBlock], s_sy[kProjBlock], s_w[kProjBlock], s_depth[kProjBlock];
    __shared__ uint32_t wave_tot[4];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int64_t g0 = (int64_t)blockIdx.x * kProjBlock;
    const int64_t i = g0 + tid;

    uint32_t count = 0;
    if(i < n)
    {
        const float4 q0 = splats[3 * i];
        const int radius = __float_as_int(q0.w);
        const TileRect r = tile_rect(q0.x, q0.y, radius, ntx, nty);
        const int w = r.ex - r.sx;
        count = (uint32_t)(w * (r.ey - r.sy) * (radius > 0 ? 1 : 0));
        if(i == n - 1)
            count = 0; // the last Gaussian never emits (its end index is forced to K)
        s_sx[tid] = r.sx;
        s_sy[tid] = r.sy;
        s_w[tid] = w;
        s_depth[tid] = __float_as_int(q0.z);
    }
    const uint32_t incl = wave_incl_scan_u32(count, lane);
    if(lane == 63)
        wave_tot[wave] = incl;
    __syncthreads();
    uint32_t prefix = 0;
    for(int w = 0; w < wave; ++w)
        prefix += wave_tot[w];
    s_off[tid] = prefix + incl - count;
    if(tid == kProjBlock - 1)
        s_off[kProjBlock] = prefix + incl;
    __syncthreads();

    const uint32_t total = s_off[kProjBlock];
    const int64_t base = block_offsets[blockIdx.x];
    for(uint32_t j = tid; j < total; j += kProjBlock)
    {
        // largest g with s_off[g] <= j
        int lo = 0, hi = kProjBlock;
        while(hi - lo > 1)
        {
            const int mid = (lo + hi) >> 1;
            if(s_off[mid] <= j)
                lo = mid;
            else
                hi = mid;
        }
        const uint32_t r = j - s_off[lo];
        const uint32_t w = (uint32_t)s_w[lo];
        const uint32_t ry = r / w;
        const uint32_t rx = r - ry * w;
        const int64_t tile = (int64_t)(s_sy[lo] + (int)ry) * ntx + (s_sx[lo] + (int)rx);
        const int64_t depth = (int64_t)s_depth[lo]; // sign-extending, as the reference does
        const int64_t out = base + j;
        if(out < k)
        {
            keys[out] = (int64_t)((uint64_t)tile << 32) | depth;
            values[out] = (int32_t)(g0 + lo);
        }
    }
}

int launch_emit_keys(const dsx_camera& cam, int64_t n, int64_t k, const float* splats,
                     const uint32_t* block_offsets, int64_t* keys, int32_t* values, hipStream_t stream)
{
    if(n == 0 || k == 0)
        return DSX_OK;
    const int64_t blocks = (n + kProjBlock - 1) / kProjBlock;
    {
        DSX_TIMED("emit_keys_kernel", stream);
        hipLaunchKernelGGL(emit_keys_kernel, dim3((unsigned)blocks), dim3(kProjBlock), 0, stream,
                           reinterpret_cast<const float4*>(splats), block_offsets, n, k, tiles_x(cam.image_width),
                           tiles_y(cam.image_height), keys, values);
    }
    DSX_LAUNCH_CHECK();
    return DSX_OK;
}

// ---------------------------------------------------------------------------------------
// radix sort
// ---------------------------------------------------------------------------------------

SortWorkspace sort_workspace(int64_t k, int num_tiles)
{
    auto align = [](size_t x) { return (x + 255) & ~(size_t)255; };
    SortWorkspace w;
    w.passes = sort_passes(num_tiles);
    w.tiles = (k + kSortTile - 1) / kSortTile;
    size_t off = 0;
    w.keys_alt = off;
    off = align(off + (size_t)k * 8);
    w.values_alt = off;
    off = align(off + (size_t)k * 4);
    w.global_hist = off;
    off = align(off + (size_t)w.passes * kRadix * 4);
    w.counters = off;
    off = align(off + (size_t)(w.passes + 1) * 4);
    w.status = off;
    off = align(off + (size_t)w.passes * (size_t)w.tiles * kRadix * 4);
    w.bytes = off;
    return w;
}

struct DigitPlan
{
    int passes;
    int shift[kMaxPasses];
    uint32_t mask[kMaxPasses];
};

static DigitPlan digit_plan(int num_tiles)
{
    const SortPlan sp = sort_plan(num_tiles);
    DigitPlan d;
    d.passes = sp.passes;
    for(int p = 0; p < kMaxPasses; ++p)
    {
        d.shift[p] = sp.shift[p];
        d.mask[p] = (1u << sp.bits[p]) - 1u;
    }
    return d;
}

// value of the lane below (lane 0 receives `first`): one DPP move, no LDS traffic
__device__ __forceinline__ uint32_t lane_below(uint32_t v, uint32_t first)
{
    return (uint32_t)__builtin_amdgcn_update_dpp((int)first, (int)v, 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
}

// Histogram of every digit of every key in one read of the keys.  Emission order puts long
// runs of equal digits next to each other (all keys of one Gaussian share their depth bits),
// so each run of equal digits inside a wavefront is collapsed to one LDS atomic by its first
// lane: heads are found with one lane shift and one ballot per digit.
constexpr int kHistThreads = 256;
constexpr int kHistItems = 8;

__global__ __launch_bounds__(kHistThreads) void radix_hist_kernel(const int64_t* __restrict__ keys, int64_t k,
                                                                  const DigitPlan plan,
                                                                  uint32_t* __restrict__ global_hist)
{
    __shared__ uint32_t hist[kMaxPasses * kRadix];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    for(int j = tid; j < plan.passes * kRadix; j += kHistThreads)
        hist[j] = 0;
    __syncthreads();
    const int64_t chunk = (int64_t)kHistThreads * kHistItems;
    const int64_t chunks = (k + chunk - 1) / chunk;
    for(int64_t c = blockIdx.x; c < chunks; c += gridDim.x)
    {
        uint64_t s[kHistItems];
        bool valid[kHistItems];
#pragma unroll
        for(int it = 0; it < kHistItems; ++it)
        {
            const int64_t i = c * chunk + it * kHistThreads + tid;
            valid[it] = i < k;
            s[it] = valid[it] ? sortable(__builtin_nontemporal_load(keys + i)) : 0ull;
        }
#pragma unroll
        for(int it = 0; it < kHistItems; ++it)
        {
            const uint64_t vmask = __ballot(valid[it]); // valid lanes are a prefix of the wavefront
            const int nvalid = __popcll(vmask);
            for(int p = 0; p < plan.passes; ++p)
            {
                const uint32_t d = (uint32_t)(s[it] >> plan.shift[p]) & plan.mask[p];
                const uint32_t below = lane_below(d, ~d);
                const bool head = valid[it] && (lane == 0 || below != d);
                const uint64_t heads = __ballot(head);
                if(head)
                {
                    const uint64_t above = lane == 63 ? 0ull : (heads >> (lane + 1));
                    const int run = above ? __ffsll((unsigned long long)above) : nvalid - lane;
                    atomicAdd(&hist[p * kRadix + d], (uint32_t)run);
                }
            }
        }
    }
    __syncthreads();
    for(int j = tid; j < plan.passes * kRadix; j += kHistThreads)
        if(hist[j])
            atomicAdd(&global_hist[j], hist[j]);
}

// exclusive scan of each pass's 512 bins (one workgroup per pass)
__global__ __launch_bounds__(kRadix) void radix_hist_scan_kernel(uint32_t* global_hist)
{
    __shared__ uint32_t wave_tot[kRadix / DSX_WAVE];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    uint32_t* h = global_hist + blockIdx.x * kRadix;
    const uint32_t v = h[tid];
    const uint32_t incl = wave_incl_scan_u32(v, lane);
    if(lane == 63)
        wave_tot[wave] = incl;
    __syncthreads();
    uint32_t prefix = 0;
    for(int w = 0; w < wave; ++w)
        prefix += wave_tot[w];
    h[tid] = prefix + incl - v;
}

constexpr uint32_t kFlagAggregate = 1u << 30;
constexpr uint32_t kFlagInclusive = 2u << 30;
constexpr uint32_t kFlagMask = 3u << 30;
constexpr uint32_t kValueMask = ~kFlagMask;
constexpr int kSpinLimit = 1 << 18; // bounded wait: a stuck predecessor ends in an error flag, not a hang
#ifndef DSX_LOOK_BATCH
#define DSX_LOOK_BATCH 4
#endif
constexpr int kLookBatch = DSX_LOOK_BATCH; // predecessor statuses fetched per round trip
constexpr int kSortWaves = kSortThreads / DSX_WAVE;

// One digit pass.  Tile = kSortTile consecutive keys, taken in arrival order through a dynamic
// counter so that every tile a workgroup waits for has already started.  Stable ranking:
// wave-local rank by ballot matching (item by item, lane by lane), waves in tile order, tiles
// in chained-scan order (decoupled look-back; thread d owns digit d and fetches several
// predecessors per round trip).  Keys, then values, are reordered through the same LDS buffer
// so that global stores of one digit are contiguous.  Large tiles matter twice: the status
// traffic of the look-back falls with the number of tiles AND with the depth of the walk,
// which itself shrinks when tiles start less often.
constexpr size_t kSortLdsBytes = (size_t)kSortTile * 8 + (size_t)kSortWaves * kRadix * 2 + 2 * kRadix * 4 + 64 + 16;

__global__ __launch_bounds__(kSortThreads) void radix_onesweep_kernel(
    const int64_t* __restrict__ keys_in, const int32_t* __restrict__ vals_in, int64_t* __restrict__ keys_out,
    int32_t* __restrict__ vals_out, int64_t k, int shift, uint32_t mask, const uint32_t* __restrict__ hist_excl,
    uint32_t* status, uint32_t* tile_counter, uint32_t* error_flag)
{
    extern __shared__ __align__(16) unsigned char smem[];
    int64_t* s_keys = reinterpret_cast<int64_t*>(smem); // reused for the values in the second round
    uint16_t(*s_whist)[kRadix] = reinterpret_cast<uint16_t(*)[kRadix]>(smem + (size_t)kSortTile * 8);
    uint32_t* s_digit_start = reinterpret_cast<uint32_t*>(smem + (size_t)kSortTile * 8 + (size_t)kSortWaves * kRadix * 2);
    uint32_t* s_gbase = s_digit_start + kRadix;
    uint32_t* s_wave_tot = s_gbase + kRadix;
    uint32_t& s_tile = s_wave_tot[16];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;

    if(tid == 0)
        s_tile = atomicAdd(tile_counter, 1u);
    for(int j = tid; j < kSortWaves * kRadix; j += kSortThreads)
        (&s_whist[0][0])[j] = 0;
    __syncthreads();
    const int64_t tile = s_tile;
    const int64_t tile_base = tile * kSortTile;
    const int tile_n = (int)min((int64_t)kSortTile, k - tile_base);

    // ---- load (striped inside each wavefront: coalesced, order = (item, lane)) -------------
    int64_t key[kSortItems];
    int32_t val[kSortItems];
    uint32_t pos[kSortItems];
    uint32_t dig[kSortItems];
#pragma unroll
    for(int it = 0; it < kSortItems; ++it)
    {
        const int local = wave * (kSortItems * 64) + it * 64 + lane;
        if(local < tile_n)
        {
            key[it] = __builtin_nontemporal_load(keys_in + tile_base + local);
            val[it] = __builtin_nontemporal_load(vals_in + tile_base + local);
        }
        else
        {
            key[it] = 0;
            val[it] = 0;
        }
    }

    // ---- wave-local stable rank -----------------------------------------------------------
    // plain LDS accesses: a wavefront's LDS instructions execute in program order, and the
    // compiler keeps the load/store order because both may touch the same counter
    uint16_t* wh = s_whist[wave];
#pragma unroll
    for(int it = 0; it < kSortItems; ++it)
    {
        const int local = wave * (kSortItems * 64) + it * 64 + lane;
        const bool valid = local < tile_n;
        const uint32_t d = (uint32_t)(sortable(key[it]) >> shift) & mask;
        dig[it] = d;
        const uint64_t m = match_digit(d, valid);
        const uint32_t below = (uint32_t)__popcll(m & lanemask_lt(lane));
        const uint32_t old = wh[d];
        __builtin_amdgcn_wave_barrier();
        if(valid && below == 0)
            wh[d] = (uint16_t)(old + (uint32_t)__popcll(m));
        __builtin_amdgcn_wave_barrier();
        pos[it] = old + below;
    }
    __syncthreads();

    // ---- per-digit totals of the tile (thread d <-> digit d), wave offsets, digit starts ----
    const bool digit_thread = tid < kRadix; // thread d owns digit d (workgroups may be larger)
    uint32_t total = 0;
    uint32_t* my_status = status + tile * kRadix + (digit_thread ? tid : 0);
    if(digit_thread)
    {
#pragma unroll
        for(int w = 0; w < kSortWaves; ++w)
        {
            const uint32_t c = s_whist[w][tid];
            s_whist[w][tid] = (uint16_t)total;
            total += c;
        }
        // publish this tile's count as soon as it is known
        __hip_atomic_store(my_status, total | (tile == 0 ? kFlagInclusive : kFlagAggregate), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    {
        const uint32_t incl = wave_incl_scan_u32(total, lane);
        if(digit_thread && lane == 63)
            s_wave_tot[wave] = incl;
        __syncthreads();
        if(digit_thread)
        {
            uint32_t prefix = 0;
            for(int w = 0; w < wave; ++w)
                prefix += s_wave_tot[w];
            s_digit_start[tid] = prefix + incl - total;
        }
    }
    __syncthreads();

    // ---- keys into LDS in tile-sorted order ----------------------------------------------
#pragma unroll
    for(int it = 0; it < kSortItems; ++it)
    {
        const int local = wave * (kSortItems * 64) + it * 64 + lane;
        if(local < tile_n)
        {
            const uint32_t d = dig[it];
            pos[it] += s_digit_start[d] + s_whist[wave][d];
            s_keys[pos[it]] = key[it];
        }
    }

    // ---- chained scan over earlier tiles (decoupled look-back), one thread per digit -------
    if(digit_thread)
    {
        uint32_t excl = 0;
        if(tile > 0)
        {
            int64_t t = tile - 1; // next predecessor to account for
            int spins = 0;
            bool done = false;
            while(!done)
            {
                uint32_t v[kLookBatch];
#pragma unroll
                for(int b = 0; b < kLookBatch; ++b)
                {
                    // rows below tile 0 are read as tile 0, whose status is inclusive from the start
                    const int64_t row = t - b > 0 ? t - b : 0;
                    v[b] = __hip_atomic_load(status + row * kRadix + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for(int b = 0; b < kLookBatch; ++b)
                {
                    if(done)
                        break;
                    if((v[b] & kFlagMask) == 0)
                    {
                        // not published yet: poll again from this predecessor
                        if(++spins > kSpinLimit)
                        {
                            *error_flag = 1u;
                            done = true;
                        }
                        else
                            __builtin_amdgcn_s_sleep(1);
                        break;
                    }
                    excl += v[b] & kValueMask;
                    --t;
                    if(v[b] & kFlagInclusive)
                        done = true;
                }
            }
            __hip_atomic_store(my_status, ((excl + total) & kValueMask) | kFlagInclusive, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
        s_gbase[tid] = hist_excl[tid] + excl - s_digit_start[tid];
    }
    __syncthreads();

    // ---- scatter keys: consecutive threads -> consecutive addresses inside a digit's run ----
    uint32_t out[kSortItems];
#pragma unroll
    for(int it = 0; it < kSortItems; ++it)
    {
        const int j = it * kSortThreads + tid;
        if(j < tile_n)
        {
            const int64_t kk = s_keys[j];
            const uint32_t d = (uint32_t)(sortable(kk) >> shift) & mask;
            out[it] = s_gbase[d] + (uint32_t)j;
            keys_out[out[it]] = kk;
        }
    }
    __syncthreads();

    // ---- values through the same buffer, same positions ------------------------------------
    int32_t* s_vals = reinterpret_cast<int32_t*>(s_keys);
#pragma unroll
    for(int it = 0; it < kSortItems; ++it)
    {
        const int local = wave * (kSortItems * 64) + it * 64 + lane;
        if(local < tile_n)
            s_vals[pos[it]] = val[it];
    }
    __syncthreads();
#pragma unroll
    for(int it = 0; it < kSortItems; ++it)
    {
        const int j = it * kSortThreads + tid;
        if(j < tile_n)
            vals_out[out[it]] = s_vals[j];
    }
}

int launch_sort_pairs(int64_t k, int num_tiles, int64_t* keys_a, int32_t* values_a, int64_t* keys_b,
                      int32_t* values_b, void* sort_ws, hipStream_t stream, int64_t** keys_out,
                      int32_t** values_out)
{
    *keys_out = keys_a;
    *values_out = values_a;
    if(k <= 1)
        return DSX_OK;
    if(k >= (1ll << 30))
        return DSX_ERR_TOO_LARGE;
    const SortWorkspace w = sort_workspace(k, num_tiles);
    const DigitPlan plan = digit_plan(num_tiles);
    char* base = static_cast<char*>(sort_ws);
    uint32_t* global_hist = reinterpret_cast<uint32_t*>(base + w.global_hist);
    uint32_t* counters = reinterpret_cast<uint32_t*>(base + w.counters);
    uint32_t* status = reinterpret_cast<uint32_t*>(base + w.status);
    // global_hist, counters and status are adjacent: clear them with one fill
    const int64_t clear_words = (int64_t)((w.bytes - w.global_hist) / 4);
    int rc = launch_fill_u32(global_hist, clear_words, 0u, stream);
    if(rc)
        return rc;
    const int64_t hist_chunks = (k + kHistThreads * kHistItems - 1) / (kHistThreads * kHistItems);
    const int hist_blocks = (int)min((int64_t)2048, hist_chunks);
    {
        DSX_TIMED("radix_hist_kernel", stream);
        hipLaunchKernelGGL(radix_hist_kernel, dim3(hist_blocks), dim3(kHistThreads), 0, stream, keys_a, k, plan,
                           global_hist);
    }
    DSX_LAUNCH_CHECK();
    {
        DSX_TIMED("radix_hist_scan_kernel", stream);
        hipLaunchKernelGGL(radix_hist_scan_kernel, dim3(w.passes), dim3(kRadix), 0, stream, global_hist);
    }
    DSX_LAUNCH_CHECK();
    // more than 64 KB of LDS per workgroup has to be requested explicitly (once per process)
    static std::once_flag lds_once;
    static hipError_t lds_status = hipSuccess;
    std::call_once(lds_once, [] {
        lds_status = hipFuncSetAttribute(reinterpret_cast<const void*>(radix_onesweep_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kSortLdsBytes);
    });
    if(lds_status != hipSuccess)
        return DSX_ERR_RUNTIME;
    int64_t* kin = keys_a;
    int32_t* vin = values_a;
    int64_t* kout = keys_b;
    int32_t* vout = values_b;
    for(int p = 0; p < w.passes; ++p)
    {
        {
            DSX_TIMED("radix_onesweep_kernel", stream);
            hipLaunchKernelGGL(radix_onesweep_kernel, dim3((unsigned)w.tiles), dim3(kSortThreads), kSortLdsBytes, stream, kin,
                               vin, kout, vout, k, plan.shift[p], plan.mask[p], global_hist + p * kRadix,
                               status + (size_t)p * w.tiles * kRadix, counters + p, counters + w.passes);
        }
        DSX_LAUNCH_CHECK();
        int64_t* tk = kin;
        kin = kout;
        kout = tk;
        int32_t* tv = vin;
        vin = vout;
        vout = tv;
    }
    *keys_out = kin;
    *values_out = vin;
    return DSX_OK;
}

// ---------------------------------------------------------------------------------------
// tile ranges
// ---------------------------------------------------------------------------------------

// ranges[j] = number of keys whose tile is below j, by binary search in the sorted keys: one
// thread per tile, about log2(K) dependent loads each, instead of a pass over all K keys.
// Two rules of the reference are kept (cpp/rasterizer_kernels.cu:313-322,
// cpp/rasterizer_torch.cu:31-39): the boundary after the LAST run is never recorded, so tiles
// above the highest occupied tile inherit the START of that run, and ranges[num_tiles] = K.
// Keys with a negative depth carry tile -1 and sort first; ranges[0] skips them.
__global__ __launch_bounds__(256) void ranges_search_kernel(const int64_t* __restrict__ keys, int64_t k,
                                                            int num_tiles, int32_t* __restrict__ ranges)
{
    const int j = blockIdx.x * 256 + threadIdx.x;
    if(j > num_tiles)
        return;
    if(j == num_tiles || k == 0)
    {
        ranges[j] = j == num_tiles ? (int32_t)k : 0;
        return;
    }
    const int64_t last_tile = keys[k - 1] >> 32; // arithmetic shift: -1 for negative keys
    const int64_t target_tile = j < last_tile ? j : last_tile;
    const int64_t target = (int64_t)((uint64_t)target_tile << 32);
    int64_t lo = 0, hi = k; // first index with keys[i] >= target
    while(lo < hi)
    {
        const int64_t mid = (lo + hi) >> 1;
        if(keys[mid] < target)
            lo = mid + 1;
        else
            hi = mid;
    }
    ranges[j] = (int32_t)lo;
}

int launch_tile_ranges(int64_t k, const int64_t* sorted_keys, int num_tiles, int32_t* ranges, hipStream_t stream)
{
    const int count = num_tiles + 1;
    {
        DSX_TIMED("ranges_search_kernel", stream);
        hipLaunchKernelGGL(ranges_search_kernel, dim3((count + 255) / 256), dim3(256), 0, stream, sorted_keys, k,
                           num_tiles, ranges);
    }
    DSX_LAUNCH_CHECK();
    return DSX_OK;
}

} // namespace dsx
