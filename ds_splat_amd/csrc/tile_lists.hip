// Per-tile depth-ordered Gaussian lists without a 64-bit sort of all K keys.
//
// The order the blend kernels need is (tile, depth bits, Gaussian index): the order a stable
// sort of the (tile << 32 | depth) keys produces, because keys are emitted by ascending Gaussian
// index and a Gaussian touches a tile at most once.  The same order falls out of
//   1. a stable sort of the N Gaussians by their 32 depth bits (N is ~10x smaller than K),
//   2. emitting (tile slot, Gaussian) pairs in that depth order,
//   3. a STABLE partition of the K pairs by tile slot alone (2 passes of <= 8 bits).
// Keys with a negative depth carry tile field -1 in the 64-bit scheme and sort first by their
// unsigned depth bits; here they take slot 0 and real tiles move up by one, and the unsigned
// depth order of step 1 keeps their relative order.  HBM traffic: 6 or 8 bytes per pair written
// once and moved twice, instead of 12 bytes moved five times.
#include "dsx_common.h"

#include <algorithm>
#include <mutex>

namespace dsx
{

// One helper stream per device (default priority, created on first use, kept until the process
// ends): work that does not depend on the depth sort runs there, beside the sort's
// latency-bound passes.  Returns nullptr when no stream can be made (the caller then stays on
// its own stream).
static hipStream_t helper_stream()
{
    constexpr int kMaxDevices = 64;
    static std::mutex mutex;
    static hipStream_t streams[kMaxDevices] = {};
    static bool tried[kMaxDevices] = {};
    int device = 0;
    if(hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices)
        return nullptr;
    std::lock_guard<std::mutex> lock(mutex);
    if(!tried[device])
    {
        tried[device] = true;
        hipStream_t s = nullptr;
        if(hipStreamCreateWithFlags(&s, hipStreamNonBlocking) == hipSuccess)
            streams[device] = s;
        else
            (void)hipGetLastError();
    }
    return streams[device];
}

// Bin size of the tile lists: one list per tile below 2048 tiles (a 256 x 256 image has 16 bins of
// 4 x 4, and its 1024 blend wavefronts, four per tile there, would each filter a list sixteen times
// the tile's own); from 2048 tiles on, bins of 4 x 4 tiles (a Gaussian's rectangle then touches a few
// bins instead of a dozen tiles, and emission and partition shrink accordingly), or of 8 x 8 where
// that brings the lists, slot 0 included, down to the 256 that ONE partition pass handles
// (1920 x 1080: 135 lists instead of 510; a 3840 x 2160 image needs two passes either way).
// list_bin != 0 (dsx_camera::list_bin) asks for bins of that many tiles a side instead.
ListGrid list_grid(int image_width, int image_height, int list_bin)
{
    ListGrid g;
    g.ntx = tiles_x(image_width);
    g.nty = tiles_y(image_height);
    int side = list_bin ? list_bin : 1;
    if(!list_bin && g.ntx * g.nty >= 2048)
    {
        auto lists = [&](int64_t b) { return ((g.ntx + b - 1) / b) * ((g.nty + b - 1) / b); };
        side = (slot_bits((int)std::min<int64_t>(lists(4), 1 << 30)) > 8 && slot_bits((int)lists(8)) <= 8) ? 8 : 4;
        // (a bin's slot shares its 32-bit word with the 16-bit tile mask: at most 65534 bins; images beyond
        // that, hundreds of megapixels, get larger bins or, failing that, per-tile lists with 32-bit slots)
        if(lists(side) + 1 > 65535)
            side = lists(8) + 1 <= 65535 ? 8 : 1;
    }
    g.shift = side == 8 ? 3 : (side == 4 ? 2 : (side == 2 ? 1 : 0));
    g.nbx = (g.ntx + side - 1) / side;
    g.nby = (g.nty + side - 1) / side;
    return g;
}

__device__ __forceinline__ uint32_t wave_incl_scan32(uint32_t v, int)
{
    return wave_incl_scan_u32(v);
}

// inclusive max-scan over the 64 lanes with data-parallel-primitive moves only (values >= 0,
// lanes without a source keep 0): four shifts inside each row of 16, then the row broadcasts
template <int kCtrl, int kRowMask>
__device__ __forceinline__ uint32_t dpp_max(uint32_t v)
{
    const uint32_t moved = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, kCtrl, kRowMask, 0xf, false);
    return max(v, moved);
}

__device__ __forceinline__ uint32_t wave_incl_max_scan(uint32_t v)
{
    v = dpp_max<0x111, 0xf>(v); // row_shr:1
    v = dpp_max<0x112, 0xf>(v); // row_shr:2
    v = dpp_max<0x114, 0xf>(v); // row_shr:4
    v = dpp_max<0x118, 0xf>(v); // row_shr:8
    v = dpp_max<0x142, 0xa>(v); // row_bcast:15 into rows 1 and 3
    v = dpp_max<0x143, 0xc>(v); // row_bcast:31 into rows 2 and 3
    return v;
}

// lanes of the wavefront that hold the same (up to 8-bit) digit; uniform flow only
__device__ __forceinline__ uint64_t match_digit8(uint32_t d, int bits)
{
    uint32_t lo = 0xffffffffu, hi = 0xffffffffu;
#pragma unroll
    for(int b = 0; b < kBits32; ++b)
    {
        if(b >= bits) // uniform: digits narrower than 8 bits need fewer rounds
            break;
        uint32_t x = (uint32_t)(((int32_t)(d << (31 - b))) >> 31); // all ones where bit b is set
        asm volatile("" : "+v"(x)); // the ballot tests x itself (one compare), not a second copy of the bit
        const uint64_t m = __ballot(x != 0);
        lo &= ~((uint32_t)m ^ x);
        hi &= ~((uint32_t)(m >> 32) ^ x);
    }
    return ((uint64_t)hi << 32) | lo;
}

// ---------------------------------------------------------------------------------------
// histograms of every digit in one read (run-length merged: neighbouring keys often share a digit)
// ---------------------------------------------------------------------------------------
#ifndef DSX_HIST_BLOCKS
#define DSX_HIST_BLOCKS 512 // few workgroups: each ends with one global atomic per bin, which serialise per address
#endif
// 1024 threads share one LDS histogram: the kernel is bound by latency (3 M keys are few), so
// it wants many wavefronts per CU, while every further workgroup adds a flush of up to 1024
// contended global atomics (256 threads: 0.029 ms, 1024 threads: 0.020 ms at 3 M keys)
constexpr int kHist32Threads = 1024;
constexpr int kHist32Items = 8;

template <typename KeyT>
__global__ __launch_bounds__(kHist32Threads) void hist32_kernel(const KeyT* __restrict__ keys, int64_t count,
                                                                const Digits32 plan,
                                                                uint32_t* __restrict__ global_hist)
{
    __shared__ uint32_t hist[kMaxPasses32 * kBins32];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    for(int j = tid; j < plan.passes * kBins32; j += kHist32Threads)
        hist[j] = 0;
    __syncthreads();
    const int64_t chunk = (int64_t)kHist32Threads * kHist32Items;
    const int64_t chunks = (count + chunk - 1) / chunk;
    uint32_t ones = 0; // all-ones keys of this thread: counted here, added to their bins at the end
    for(int64_t c = blockIdx.x; c < chunks; c += gridDim.x)
    {
        uint32_t s[kHist32Items];
        bool valid[kHist32Items];
#pragma unroll
        for(int it = 0; it < kHist32Items; ++it)
        {
            const int64_t i = c * chunk + it * kHist32Threads + tid;
            valid[it] = i < count;
            s[it] = valid[it] ? (uint32_t)__builtin_nontemporal_load(keys + i) : 0u;
        }
#pragma unroll
        for(int it = 0; it < kHist32Items; ++it)
        {
            // lower digits: plain LDS atomics (values differ from lane to lane).  The most
            // significant digit takes few values (the exponent byte of depths, the high bits of
            // a tile slot): one add per distinct value of the wavefront, after a ballot, because
            // LDS atomics on one address serialise.
            // The all-ones depth keys of Gaussians that emit nothing, a third of a typical scene,
            // share one bin in every digit: each thread counts its own in a register and the
            // wavefront adds the sum to those bins once, at the end (0.026 -> 0.022 ms; a ballot
            // and one add per wavefront and item was slower than letting the atomics serialise).
            if(valid[it] && s[it] == 0xffffffffu)
            {
                ++ones;
                valid[it] = false;
            }
            for(int p = 0; p + 1 < plan.passes; ++p)
                if(valid[it])
                    atomicAdd(&hist[p * kBins32 + ((s[it] >> plan.shift[p]) & plan.mask[p])], 1u);
            {
                const int p = plan.passes - 1;
                const uint32_t d = (s[it] >> plan.shift[p]) & plan.mask[p];
                uint64_t todo = __ballot(valid[it]);
                for(int round = 0; round < 8 && todo; ++round)
                {
                    const int leader = __builtin_ctzll(todo);
                    const uint32_t dl = (uint32_t)__builtin_amdgcn_readlane((int)d, leader);
                    const uint64_t same = __ballot(valid[it] && d == dl) & todo;
                    if(lane == leader)
                        atomicAdd(&hist[p * kBins32 + dl], (uint32_t)__popcll(same));
                    todo &= ~same;
                }
                // more than eight distinct values in the wavefront: the digit is not a
                // concentrated one after all, the rest goes the plain way
                if((todo >> lane) & 1)
                    atomicAdd(&hist[p * kBins32 + d], 1u);
            }
        }
    }
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        ones += __shfl_xor(ones, o, DSX_WAVE);
    if(lane == 0 && ones)
        for(int p = 0; p < plan.passes; ++p)
            atomicAdd(&hist[p * kBins32 + plan.mask[p]], ones);
    __syncthreads();
    for(int j = tid; j < plan.passes * kBins32; j += kHist32Threads)
        if(hist[j])
            atomicAdd(&global_hist[j], hist[j]);
}

// ---------------------------------------------------------------------------------------
// one digit pass (chained scan over tiles, decoupled look-back) for (uint32 key, uint32 value)
// ---------------------------------------------------------------------------------------
constexpr uint32_t kFlagAggregate32 = 1u << 30;
constexpr uint32_t kFlagInclusive32 = 2u << 30;
constexpr uint32_t kFlagMask32 = 3u << 30;
constexpr uint32_t kValueMask32 = ~kFlagMask32;
constexpr int kSpinLimit32 = 1 << 18; // bounded wait: a stuck predecessor ends in an error flag, not a hang
#ifndef DSX_LOOK32
#define DSX_LOOK32 4
#endif
constexpr int kLookBatch32 = DSX_LOOK32;

static_assert(kSortThreads32 >= kBins32, "one thread per digit");
static_assert(kSortThreads32 * kSortItemsMax32 <= 65535, "u16 ranks");

// A tile rectangle as the projection packs it (16-bit fields) in 32 bits: 8 bits each for first
// column, first row, width and height, for images of at most 255 x 255 tiles.  The depth's sign
// takes the first column's place: column 255 does not exist, and what reads the sorted rectangles
// wants only the pair count of a Gaussian behind the camera (all its pairs go to slot 0), so its
// first column and row are not carried.
constexpr int kRect32MaxTiles = 255;
__device__ __forceinline__ uint32_t rect_to_32(uint2 r)
{
    const uint32_t size = ((r.y & 0xffu) << 16) | (((r.y >> 16) & 0xffu) << 24);
    return (r.y >> 31) ? (0xffu | size) : ((r.x & 0xffu) | (((r.x >> 16) & 0xffu) << 8) | size);
}
__device__ __forceinline__ uint2 rect_from_32(uint32_t v)
{
    const bool behind = (v & 0xffu) == 0xffu;
    const uint32_t size = ((v >> 16) & 0xffu) | ((v >> 24) << 16);
    return behind ? make_uint2(0u, size | 0x80000000u) : make_uint2((v & 0xffu) | (((v >> 8) & 0xffu) << 16), size);
}

// What a pass does about the Gaussians' tile rectangles, which the emission wants in depth order.
// Either the last pass gathers them (gather_dst[position] = gather_src[value]; a pair whose key is
// kNoPairsKey gets a zero record without the read): 1.9 M random 8-byte reads that pull 128-byte
// lines.  Or every pass carries the rectangle as a second 32-bit value (kCarry): the first pass
// reads the rectangles in index order, packs them (pack_src), the passes in between move them like
// the values (carry_in -> carry_out), and the last pass unpacks into unpack_dst.
struct RectJob
{
    const uint2* gather_src;
    uint2* gather_dst;
    const uint2* pack_src;
    const uint32_t* carry_in;
    uint32_t* carry_out;
    uint2* unpack_dst;
};

// vals_in == nullptr: the values are the input positions (iota).  keys_out == nullptr: the
// keys are not needed after this pass.  KeyT: uint32_t, or uint16_t for tile slots that fit.
template <typename KeyT, int kSort32Threads, int kSort32Items, bool kCarry>
__global__ __launch_bounds__(kSort32Threads) void onesweep32_kernel(
    const KeyT* __restrict__ keys_in, const uint32_t* __restrict__ vals_in, KeyT* __restrict__ keys_out,
    uint32_t* __restrict__ vals_out, int64_t count, int shift, uint32_t mask, const uint32_t* __restrict__ hist_counts,
    uint32_t* status, uint32_t* tile_counter, uint32_t* error_flag, const RectJob rects)
{
    const uint2* __restrict__ gather_src = rects.gather_src;
    uint2* __restrict__ gather_dst = rects.gather_dst;
    constexpr int kSort32Tile = kSort32Threads * kSort32Items;
    constexpr int kSort32Waves = kSort32Threads / DSX_WAVE;
    __shared__ uint32_t s_keys[kSort32Tile]; // reused for the values in the second round
    __shared__ uint16_t s_whist[kSort32Waves][kBins32];
    __shared__ uint32_t s_digit_start[kBins32];
    __shared__ uint32_t s_gbase[kBins32];
    __shared__ __attribute__((aligned(16))) uint32_t s_wave_tot[kBins32 / DSX_WAVE];
    __shared__ __attribute__((aligned(16))) uint32_t s_hist_tot[kBins32 / DSX_WAVE];
    __shared__ uint32_t s_tile;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;

    if(tid == 0)
        s_tile = atomicAdd(tile_counter, 1u);
    for(int j = tid; j < kSort32Waves * kBins32; j += kSort32Threads)
        (&s_whist[0][0])[j] = 0;
    __syncthreads();
    const int64_t tile = s_tile;
    const int64_t tile_base = tile * kSort32Tile;
    const int tile_n = (int)min((int64_t)kSort32Tile, count - tile_base);
    const int bits = 32 - __builtin_clz(mask); // mask = 2^bits - 1, bits >= 1

    // ---- load the keys (striped inside each wavefront: coalesced, order = (item, lane)) -----
    // Registers are what limits the blocks per compute unit here, so a thread keeps little per
    // item: the key while it is ranked, the rank as 16 bits, the digit as 8 bits; the value is
    // fetched only once the key registers are free.
    uint32_t key[kSort32Items];
    uint32_t pos2[(kSort32Items + 1) / 2]; // two 16-bit positions per register
#pragma unroll
    for(int it = 0; it < kSort32Items; ++it)
    {
        const int local = wave * (kSort32Items * 64) + it * 64 + lane;
        // Places past the end of the input (last tile only) hold all-ones keys: they take the
        // highest digit and, being last in tile order, rank behind every real key, so the real
        // keys' positions are what they would be without them and no phase needs a validity test
        // except the stores (tile position < tile_n).
        key[it] = 0xffffffffu;
        if(local < tile_n)
            key[it] = (uint32_t)__builtin_nontemporal_load(keys_in + tile_base + local);
    }

    // ---- wave-local stable rank ------------------------------------------------------------
    uint16_t* wh = s_whist[wave];
#pragma unroll
    for(int it = 0; it < kSort32Items; ++it)
    {
        const uint32_t d = (key[it] >> shift) & mask;
        const uint64_t m = match_digit8(d, bits);
        const uint32_t below = (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
        const uint32_t old = wh[d];
        __builtin_amdgcn_wave_barrier();
        if(below == 0)
            wh[d] = (uint16_t)(old + (uint32_t)__popcll(m));
        __builtin_amdgcn_wave_barrier();
        if(it & 1)
            pos2[it >> 1] |= (old + below) << 16;
        else
            pos2[it >> 1] = old + below;
        // pin the packed form here and make the key opaque: otherwise the compiler carries each
        // item's digit, histogram address and old count into the next phase in registers of their own
        asm volatile("" : "+v"(pos2[it >> 1]), "+v"(key[it]));
    }
    __syncthreads();

    // ---- per-digit totals of the tile (thread d <-> digit d), wave offsets, digit starts ----
    const bool digit_thread = tid < kBins32; // thread d owns digit d (bins above the mask stay empty)
    uint32_t total = 0;
    uint32_t hist_excl = 0;
    uint32_t* my_status = status + tile * kBins32 + (digit_thread ? tid : 0);
    if(digit_thread)
    {
#pragma unroll
        for(int w = 0; w < kSort32Waves; ++w)
        {
            const uint32_t c = s_whist[w][tid];
            s_whist[w][tid] = (uint16_t)total;
            total += c;
        }
        __hip_atomic_store(my_status, total | (tile == 0 ? kFlagInclusive32 : kFlagAggregate32), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t incl = wave_incl_scan32(total, lane);
        if(lane == 63)
            s_wave_tot[wave] = incl;
        s_gbase[tid] = incl - total; // wave-local exclusive prefix, completed after the barrier
        // the digit's place in the whole output: exclusive scan of the pass's histogram (every
        // tile redoes this 256-entry scan; that is cheaper than a kernel launch of its own)
        const uint32_t hcount = hist_counts[tid];
        const uint32_t hincl = wave_incl_scan32(hcount, lane);
        if(lane == 63)
            s_hist_tot[wave] = hincl;
        hist_excl = hincl - hcount;
    }
    __syncthreads();
    if(digit_thread)
    {
        // totals of the digit wavefronts before this one: two 16-byte reads and selects (a loop over
        // them compiles to dependent 4-byte reads under an exec mask, on every tile's critical path)
        static_assert(kBins32 / DSX_WAVE == 4, "four digit wavefronts");
        const uint4 wt = *reinterpret_cast<const uint4*>(s_wave_tot);
        const uint4 ht = *reinterpret_cast<const uint4*>(s_hist_tot);
        const uint32_t prefix = (wave > 0 ? wt.x : 0u) + (wave > 1 ? wt.y : 0u) + (wave > 2 ? wt.z : 0u);
        const uint32_t hprefix = (wave > 0 ? ht.x : 0u) + (wave > 1 ? ht.y : 0u) + (wave > 2 ? ht.z : 0u);
        s_digit_start[tid] = prefix + s_gbase[tid];
        hist_excl += hprefix;
    }
    __syncthreads();

    // ---- keys into LDS in tile-sorted order ----------------------------------------------
#pragma unroll
    for(int it = 0; it < kSort32Items; ++it)
    {
        const uint32_t d = (key[it] >> shift) & mask;
        const uint32_t p = ((pos2[it >> 1] >> (16 * (it & 1))) & 0xffffu) + s_digit_start[d] + s_whist[wave][d];
        s_keys[p] = key[it];
        pos2[it >> 1] = (it & 1) ? ((pos2[it >> 1] & 0xffffu) | (p << 16)) : ((pos2[it >> 1] & 0xffff0000u) | p);
    }

    // ---- the values: in flight while the chained scan runs ---------------------------------
    uint32_t val[kSort32Items];
#pragma unroll
    for(int it = 0; it < kSort32Items; ++it)
    {
        const int local = wave * (kSort32Items * 64) + it * 64 + lane;
        val[it] = 0;
        if(local < tile_n)
            val[it] = vals_in ? __builtin_nontemporal_load(vals_in + tile_base + local) : (uint32_t)(tile_base + local);
    }
    uint32_t carried[kCarry ? kSort32Items : 1];
    if(kCarry)
    {
#pragma unroll
        for(int it = 0; it < kSort32Items; ++it)
        {
            const int local = wave * (kSort32Items * 64) + it * 64 + lane;
            carried[it] = 0;
            if(local < tile_n)
                carried[it] = rects.pack_src ? rect_to_32(rects.pack_src[tile_base + local])
                                             : __builtin_nontemporal_load(rects.carry_in + tile_base + local);
        }
    }

    // ---- chained scan over earlier tiles (decoupled look-back), one thread per digit -------
    if(digit_thread)
    {
        uint32_t excl = 0;
        if(tile > 0 && (uint32_t)tid <= mask) // bins above the mask are empty in every tile
        {
            int64_t t = tile - 1; // next predecessor to account for
            int spins = 0;
            bool done = false;
            while(!done)
            {
                uint32_t v[kLookBatch32];
#pragma unroll
                for(int b = 0; b < kLookBatch32; ++b)
                {
                    // rows below tile 0 are read as tile 0, whose status is inclusive from the start
                    const int64_t row = t - b > 0 ? t - b : 0;
                    v[b] = __hip_atomic_load(status + row * kBins32 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for(int b = 0; b < kLookBatch32; ++b)
                {
                    if(done)
                        break;
                    if((v[b] & kFlagMask32) == 0)
                    {
                        if(++spins > kSpinLimit32)
                        {
                            *error_flag = 1u;
                            done = true;
                        }
                        else
                            __builtin_amdgcn_s_sleep(1);
                        break;
                    }
                    excl += v[b] & kValueMask32;
                    --t;
                    if(v[b] & kFlagInclusive32)
                        done = true;
                }
            }
            __hip_atomic_store(my_status, ((excl + total) & kValueMask32) | kFlagInclusive32, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
        s_gbase[tid] = hist_excl + excl - s_digit_start[tid];
    }
    __syncthreads();

    // ---- scatter keys: consecutive threads -> consecutive addresses inside a digit's run ----
    uint32_t dig4[(kSort32Items + 3) / 4]; // the digit of the key at tile position it * threads + tid, 8 bits each
    uint32_t no_record = 0;                // bit it: that key is kNoPairsKey (its record is known to be zero)
#pragma unroll
    for(int it = 0; it < kSort32Items; ++it)
    {
        const int j = it * kSort32Threads + tid;
        if((it & 3) == 0)
        {
            __builtin_amdgcn_sched_barrier(0); // four items in flight at a time: registers, not latency, are scarce
            dig4[it >> 2] = 0;
        }
        if(j < tile_n)
        {
            const uint32_t kk = s_keys[j];
            const uint32_t d = (kk >> shift) & mask;
            dig4[it >> 2] |= d << (8 * (it & 3));
            if(gather_src && kk == kNoPairsKey)
                no_record |= 1u << it;
            if(keys_out)
                keys_out[s_gbase[d] + (uint32_t)j] = (KeyT)kk;
        }
    }
    __syncthreads();

    // ---- values through the same buffer, same positions ------------------------------------
#pragma unroll
    for(int it = 0; it < kSort32Items; ++it)
    {
        s_keys[(pos2[it >> 1] >> (16 * (it & 1))) & 0xffffu] = val[it];
    }
    __syncthreads();
#pragma unroll
    for(int it = 0; it < kSort32Items; ++it)
    {
        const int j = it * kSort32Threads + tid;
        if((it & 3) == 0)
            __builtin_amdgcn_sched_barrier(0);
        if(j < tile_n)
        {
            const uint32_t v = s_keys[j];
            const uint32_t out = s_gbase[(dig4[it >> 2] >> (8 * (it & 3))) & 0xffu] + (uint32_t)j;
            vals_out[out] = v;
            // optional: a per-value record follows its value to the sorted position (the random
            // gather overlaps with the scatter traffic of the pass)
            if(gather_src)
                gather_dst[out] = ((no_record >> it) & 1u) ? make_uint2(0u, 0u) : gather_src[v];
        }
    }
    if(kCarry)
    {
        // ---- the carried rectangles through the same buffer, same positions ------------------
        __syncthreads();
#pragma unroll
        for(int it = 0; it < kSort32Items; ++it)
            s_keys[(pos2[it >> 1] >> (16 * (it & 1))) & 0xffffu] = carried[it];
        __syncthreads();
#pragma unroll
        for(int it = 0; it < kSort32Items; ++it)
        {
            const int j = it * kSort32Threads + tid;
            if((it & 3) == 0)
                __builtin_amdgcn_sched_barrier(0);
            if(j < tile_n)
            {
                const uint32_t v = s_keys[j];
                const uint32_t out = s_gbase[(dig4[it >> 2] >> (8 * (it & 3))) & 0xffu] + (uint32_t)j;
                if(rects.unpack_dst)
                    rects.unpack_dst[out] = rect_from_32(v);
                else
                    rects.carry_out[out] = v;
            }
        }
    }
}

Sort32Workspace sort32_workspace(int64_t count, int key_bits, int tile_keys)
{
    auto align = [](size_t x) { return (x + 255) & ~(size_t)255; };
    Sort32Workspace w;
    w.passes = digits32(key_bits).passes;
    w.tiles = (count + tile_keys - 1) / tile_keys;
    size_t off = 0;
    w.hist = off;
    off = align(off + (size_t)w.passes * kBins32 * 4);
    w.counters = off;
    off = align(off + (size_t)(w.passes + 1) * 4);
    w.status = off;
    off = align(off + (size_t)w.passes * (size_t)w.tiles * kBins32 * 4);
    w.bytes = off;
    return w;
}

// zeroes histograms, tile counters and look-back statuses of one sort
// (extra_bytes: memory right behind the workspace that the same fill clears)
static int sort32_clear(int64_t count, int key_bits, int tile_keys, void* sort_ws, hipStream_t stream,
                        size_t extra_bytes = 0)
{
    const Sort32Workspace w = sort32_workspace(count, key_bits, tile_keys);
    return launch_fill_u32(reinterpret_cast<uint32_t*>(static_cast<char*>(sort_ws) + w.hist),
                           (int64_t)((w.bytes + extra_bytes) / 4), 0u, stream);
}

// The digit passes of a sort whose raw digit histograms are in `counts` (the workspace's own
// histogram area when counts is null).
// Ping-pong between (keys_a, vals_a) and (keys_b, vals_b); *keys_out / *vals_out say where the
// result is (keys only when keep_keys).
// gather_src / gather_dst: records that the last pass brings to the values' sorted positions by a
// gather.  carry_a / carry_b (with gather_src and gather_dst): the records travel through the passes
// as packed 32-bit values instead, in ping-pong buffers of their own (the first pass packs them from
// gather_src, the last one unpacks them into gather_dst).
template <typename KeyT, int kThreads, int kItems, bool kCarry = false>
static int sort32_passes(int64_t count, int key_bits, KeyT* keys_a, uint32_t* vals_a, KeyT* keys_b, uint32_t* vals_b,
                         bool iota_values, bool keep_keys, void* sort_ws, const char* label, hipStream_t stream,
                         KeyT** keys_out, uint32_t** vals_out, const uint2* gather_src = nullptr,
                         uint2* gather_dst = nullptr, const uint32_t* counts = nullptr, uint32_t* carry_a = nullptr,
                         uint32_t* carry_b = nullptr)
{
    const Sort32Workspace w = sort32_workspace(count, key_bits, kThreads * kItems);
    const Digits32 plan = digits32(key_bits);
    char* base = static_cast<char*>(sort_ws);
    uint32_t* hist = reinterpret_cast<uint32_t*>(base + w.hist);
    uint32_t* counters = reinterpret_cast<uint32_t*>(base + w.counters);
    uint32_t* status = reinterpret_cast<uint32_t*>(base + w.status);
    const uint32_t* raw = counts ? counts : (const uint32_t*)hist; // the passes scan their histogram themselves
    KeyT* kin = keys_a;
    uint32_t* vin = vals_a;
    KeyT* kout = keys_b;
    uint32_t* vout = vals_b;
    uint32_t* cin = carry_a;
    uint32_t* cout = carry_b;
    for(int p = 0; p < w.passes; ++p)
    {
        const bool last = p == w.passes - 1;
        RectJob job = {};
        if(kCarry)
        {
            job.pack_src = p == 0 ? gather_src : nullptr;
            job.carry_in = cin;
            job.carry_out = cout;
            job.unpack_dst = last ? gather_dst : nullptr;
        }
        else if(last)
        {
            job.gather_src = gather_src;
            job.gather_dst = gather_dst;
        }
        {
            DSX_TIMED(label, stream);
            hipLaunchKernelGGL((onesweep32_kernel<KeyT, kThreads, kItems, kCarry>), dim3((unsigned)w.tiles), dim3(kThreads), 0,
                               stream, (const KeyT*)kin, (const uint32_t*)((p == 0 && iota_values) ? nullptr : vin),
                               (last && !keep_keys) ? (KeyT*)nullptr : kout, vout, count, plan.shift[p], plan.mask[p],
                               raw + p * kBins32, status + (size_t)p * w.tiles * kBins32,
                               counters + p, counters + w.passes, job);
        }
        DSX_LAUNCH_CHECK();
        KeyT* tk = kin;
        kin = kout;
        kout = tk;
        uint32_t* tv = vin;
        vin = vout;
        vout = tv;
        uint32_t* tc = cin;
        cin = cout;
        cout = tc;
    }
    *keys_out = kin;
    *vals_out = vin;
    return DSX_OK;
}

// Stable ascending sort of `count` (key, value) pairs by the low key_bits bits of the key.
int launch_sort32(int64_t count, int key_bits, uint32_t* keys_a, uint32_t* vals_a, uint32_t* keys_b,
                  uint32_t* vals_b, bool iota_values, bool keep_keys, void* sort_ws, hipStream_t stream,
                  uint32_t** keys_out, uint32_t** vals_out, const uint2* gather_src, uint2* gather_dst,
                  bool already_cleared, uint32_t* carry_a, uint32_t* carry_b)
{
    *keys_out = keys_a;
    *vals_out = vals_a;
    if(count <= 0)
        return DSX_OK;
    if(count >= (1ll << 30))
        return DSX_ERR_TOO_LARGE;
    int rc = already_cleared ? DSX_OK : sort32_clear(count, key_bits, sort32_tile_keys(count), sort_ws, stream);
    if(rc)
        return rc;
    const Sort32Workspace w = sort32_workspace(count, key_bits, sort32_tile_keys(count));
    const int64_t chunks = (count + kHist32Threads * kHist32Items - 1) / (kHist32Threads * kHist32Items);
    {
        DSX_TIMED("hist32_kernel", stream);
        hipLaunchKernelGGL(hist32_kernel<uint32_t>, dim3((unsigned)min((int64_t)DSX_HIST_BLOCKS, chunks)), dim3(kHist32Threads), 0,
                           stream, (const uint32_t*)keys_a, count, digits32(key_bits),
                           reinterpret_cast<uint32_t*>(static_cast<char*>(sort_ws) + w.hist));
    }
    DSX_LAUNCH_CHECK();
    const bool carry = carry_a && carry_b && gather_src && gather_dst;
#define DSX_SORT32_ITEMS(ITEMS)                                                                                       \
    case ITEMS:                                                                                                       \
        return carry ? sort32_passes<uint32_t, kSortThreads32, ITEMS, true>(                                          \
                           count, key_bits, keys_a, vals_a, keys_b, vals_b, iota_values, keep_keys, sort_ws,          \
                           "onesweep32_kernel<sort>", stream, keys_out, vals_out, gather_src, gather_dst, nullptr,    \
                           carry_a, carry_b)                                                                          \
                     : sort32_passes<uint32_t, kSortThreads32, ITEMS>(count, key_bits, keys_a, vals_a, keys_b, vals_b, \
                                                                      iota_values, keep_keys, sort_ws,                \
                                                                      "onesweep32_kernel<sort>", stream, keys_out,    \
                                                                      vals_out, gather_src, gather_dst)
    switch(sort32_items(count))
    {
        DSX_SORT32_ITEMS(1);
        DSX_SORT32_ITEMS(2);
        DSX_SORT32_ITEMS(3);
        DSX_SORT32_ITEMS(4);
        DSX_SORT32_ITEMS(6);
        DSX_SORT32_ITEMS(8);
        DSX_SORT32_ITEMS(kSortItemsMax32);
    }
#undef DSX_SORT32_ITEMS
    return DSX_ERR_RUNTIME;
}

// ---------------------------------------------------------------------------------------
// depth order of the Gaussians and the scanned tile counts in that order
// ---------------------------------------------------------------------------------------

OrderLayout order_layout(int64_t n, int image_width, int image_height, int list_bin)
{
    auto align = [](size_t x) { return (x + 255) & ~(size_t)255; };
    OrderLayout o;
    size_t off = 0;
    o.depth_keys = off;
    off = align(off + (size_t)n * 4);
    o.keys_alt = off;
    off = align(off + (size_t)n * 4);
    o.ids_a = off;
    off = align(off + (size_t)n * 4);
    o.ids_b = off;
    off = align(off + (size_t)n * 4);
    o.rects = off;
    off = align(off + (size_t)n * 8);
    o.rects_sorted = off;
    off = align(off + (size_t)n * 8);
    o.rects32 = off;
    off = align(off + (size_t)n * 4);
    o.block_sums = off;
    off = align(off + (size_t)((n + kProjBlock - 1) / kProjBlock + 1) * 4);
    o.slot_hist = off;
    off = align(off + (size_t)kMaxPasses32 * kBins32 * 4);
    o.sort = off;
    off = align(off + sort32_workspace(n, 32, sort32_tile_keys(n)).bytes);
    const ListGrid g = list_grid(image_width, image_height, list_bin);
    o.cover = off;
    off += (size_t)((g.ntx + 1) * (g.nty + 1) + 1) * 4;
    o.bin_cover = off;
    if(g.shift)
        off += (size_t)((g.nbx + 1) * (g.nby + 1) + 1) * 4;
    off = (off + 7) & ~(size_t)7;
    o.key_count = off; // inside the region that is zeroed with the corner grids
    off = align(off + 16);
    o.ranges = off;
    off += (size_t)ranges_layout(g).ready * 4;
    o.bytes = align(off);
    return o;
}

__device__ __forceinline__ uint32_t rect_count(uint2 r)
{
    return (r.y & 0xffffu) * ((r.y >> 16) & 0x7fffu);
}

// The bins a tile rectangle touches: first bin (x, y) and extent, for a rectangle that is not empty.
struct BinRect
{
    uint32_t bx, by, bw, bh;
};
__device__ __forceinline__ BinRect bin_rect(uint2 r, int shift)
{
    const uint32_t sx = r.x & 0xffffu, sy = r.x >> 16;
    const uint32_t w = r.y & 0xffffu, h = (r.y >> 16) & 0x7fffu;
    BinRect b;
    b.bx = sx >> shift;
    b.by = sy >> shift;
    b.bw = ((sx + w - 1u) >> shift) - b.bx + 1u;
    b.bh = ((sy + h - 1u) >> shift) - b.by + 1u;
    return b;
}
// Pairs a Gaussian contributes to the lists: one per bin its rectangle touches (shift = 0: one
// per tile).  A Gaussian with a negative depth is in no bin list; its pairs all sit in slot 0,
// as many as the per-tile lists have, so that slot 0 is the same list whatever the bin size.
__device__ __forceinline__ uint32_t list_count(uint2 r, int shift)
{
    const uint32_t fine = rect_count(r);
    if(shift == 0 || fine == 0 || (r.y >> 31))
        return fine;
    const BinRect b = bin_rect(r, shift);
    return b.bw * b.bh;
}

// Tile count of each run of 256 Gaussians taken in depth order (the last pass of the depth sort
// has already put the rectangles into that order).
__global__ __launch_bounds__(kProjBlock) void ordered_block_sums_kernel(const uint2* __restrict__ rects_sorted,
                                                                       int64_t n, int shift,
                                                                       uint32_t* __restrict__ block_sums)
{
    __shared__ uint32_t wave_sums[kProjBlock / DSX_WAVE];
    const int tid = threadIdx.x;
    const int64_t p = (int64_t)blockIdx.x * kProjBlock + tid;
    uint32_t count = 0;
    if(p < n)
        count = list_count(rects_sorted[p], shift);
    const uint32_t ws = wave_sum_u32(count);
    if((tid & 63) == 0)
        wave_sums[tid >> 6] = ws;
    __syncthreads();
    if(tid == 0)
        block_sums[blockIdx.x] = wave_sums[0] + wave_sums[1] + wave_sums[2] + wave_sums[3];
}

// How many pairs each tile receives, straight from the rectangles (no pair is enumerated):
// a rectangle [sx, ex) x [sy, ey) adds +1, -1, -1, +1 at its four corners of a
// (nty + 1) x (ntx + 1) grid, and the two-dimensional prefix sum of that grid is the number of
// rectangles covering each tile.  Pairs of a Gaussian with a negative depth all sit in slot 0:
// they are counted in the cell after the grid.  From the per-tile counts come the digit
// histograms of the tile partition (and the tile counts themselves).
constexpr int kCoverThreads = 1024;
constexpr int kCoverBlocks = 128;
constexpr int kCoverLdsCells = 14 * 1024;      // grids up to this many cells (56 KB) are held in LDS as they are
constexpr int kCoverLdsCellsLarge = 38 * 1024; // up to 152 KB of the CU's 160 KB, once the kernels are allowed it

// shift > 0: the same for the bins, into a second grid right behind the first (bin_grid); the
// pairs of the bin lists are summed into key_count[1].
__global__ __launch_bounds__(kCoverThreads) void tile_cover_kernel(const uint2* __restrict__ rects, int64_t n, int ntx,
                                                                   int nty, int shift, int nbx, int nby, int use_lds,
                                                                   int32_t* __restrict__ grid,
                                                                   int32_t* __restrict__ bin_grid,
                                                                   unsigned long long* __restrict__ key_count)
{
    extern __shared__ int32_t s_grid[];
    const int tid = threadIdx.x;
    unsigned long long pairs = 0;     // tiles of this thread's rectangles: summed over the launch this is K
    unsigned long long bin_pairs = 0; // the same for the bin lists
    const int pitch = ntx + 1;
    const int cells = pitch * (nty + 1) + 1;
    const int bpitch = nbx + 1;
    const int bcells = shift ? bpitch * (nby + 1) + 1 : 0;
    int32_t* acc = use_lds ? s_grid : grid;
    int32_t* bacc = use_lds ? s_grid + cells : bin_grid;
    if(use_lds)
    {
        for(int j = tid; j < cells + bcells; j += kCoverThreads)
            s_grid[j] = 0;
        __syncthreads();
    }
    for(int64_t g = (int64_t)blockIdx.x * kCoverThreads + tid; g < n; g += (int64_t)gridDim.x * kCoverThreads)
    {
        const uint2 r = rects[g];
        const int w = (int)(r.y & 0xffffu), h = (int)((r.y >> 16) & 0x7fffu);
        if(w == 0 || h == 0)
            continue;
        pairs += (unsigned long long)(w * h);
        if(r.y >> 31)
        {
            atomicAdd(&acc[cells - 1], w * h);
            if(shift)
            {
                atomicAdd(&bacc[bcells - 1], w * h);
                bin_pairs += (unsigned long long)(w * h);
            }
            continue;
        }
        const int sx = (int)(r.x & 0xffffu), sy = (int)(r.x >> 16);
        atomicAdd(&acc[sy * pitch + sx], 1);
        atomicAdd(&acc[sy * pitch + sx + w], -1);
        atomicAdd(&acc[(sy + h) * pitch + sx], -1);
        atomicAdd(&acc[(sy + h) * pitch + sx + w], 1);
        if(shift)
        {
            const BinRect b = bin_rect(r, shift);
            bin_pairs += (unsigned long long)(b.bw * b.bh);
            atomicAdd(&bacc[b.by * bpitch + b.bx], 1);
            atomicAdd(&bacc[b.by * bpitch + b.bx + b.bw], -1);
            atomicAdd(&bacc[(b.by + b.bh) * bpitch + b.bx], -1);
            atomicAdd(&bacc[(b.by + b.bh) * bpitch + b.bx + b.bw], 1);
        }
    }
    if(use_lds)
    {
        __syncthreads();
        for(int j = tid; j < cells; j += kCoverThreads)
            if(s_grid[j])
                atomicAdd(&grid[j], s_grid[j]);
        for(int j = tid; j < bcells; j += kCoverThreads)
            if(s_grid[cells + j])
                atomicAdd(&bin_grid[j], s_grid[cells + j]);
    }
    // the number of pairs of the whole scene (64 bits: it is compared with the 2^30 limit, not wrapped)
    // (one atomic per workgroup: atomics on one address serialise in the L2)
    __shared__ unsigned long long s_pairs[2][kCoverThreads / DSX_WAVE];
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
    {
        pairs += __shfl_xor(pairs, o, DSX_WAVE);
        bin_pairs += __shfl_xor(bin_pairs, o, DSX_WAVE);
    }
    if((tid & 63) == 0)
    {
        s_pairs[0][tid >> 6] = pairs;
        s_pairs[1][tid >> 6] = bin_pairs;
    }
    __syncthreads();
    if(tid < 2)
    {
        unsigned long long total = 0;
        for(int w = 0; w < kCoverThreads / DSX_WAVE; ++w)
            total += s_pairs[tid][w];
        if(total)
            atomicAdd(key_count + tid, total);
    }
}

// One workgroup: 2-D prefix sum of the corner grid (in LDS when the grid fits, else in place in
// global memory, where a few ten thousand cells stay in the L2), then
//  * the digit histograms of slot = tile + 1 (slot 0 = the negative depths),
//  * ranges[j] = number of pairs whose tile is below j, with the two rules of the reference
//    (cpp/rasterizer_kernels.cu:313-322, cpp/rasterizer_torch.cu:31-39): the boundary after
//    the LAST run is never recorded, so tiles above the highest occupied tile inherit the
//    START of that run (all zero when no tile is occupied), and ranges[num_tiles] = K.
// Binned lists: workgroup 0 does the above for the tiles (no histograms: nothing is partitioned by
// tile then) and also records the highest occupied tile; workgroup 1 takes the bins' grid, whose
// ranges are plain prefix sums (the reference's two rules are rules about tiles) and whose
// histograms drive the partition.
struct CountsJob
{
    int32_t* grid;
    int ntx, nty;
    int plain;           // 1: ranges are plain prefix sums, no rule about the last run
    uint32_t* slot_hist; // may be null
    int32_t* ranges;
    int32_t* last;       // may be null: receives the highest occupied tile, -1 if none
    int32_t* header;     // may be null: receives header_value (the bin shift the lists are built for)
    int32_t header_value;
    Digits32 plan;
};
struct CountsJobs
{
    CountsJob job[2];
};

__global__ __launch_bounds__(kCoverThreads) void tile_counts_kernel(const CountsJobs jobs, int use_lds)
{
    const CountsJob& J = jobs.job[blockIdx.x];
    int32_t* const grid = J.grid;
    const int ntx = J.ntx, nty = J.nty;
    const Digits32& plan = J.plan;
    uint32_t* const slot_hist = J.slot_hist;
    int32_t* const ranges = J.ranges;
    extern __shared__ int32_t s_cells[];
    __shared__ uint32_t hist[kMaxPasses32 * kBins32];
    __shared__ __attribute__((aligned(16))) uint32_t wave_tot[kCoverThreads / DSX_WAVE];
    __shared__ uint32_t s_carry;
    __shared__ int s_last;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int pitch = ntx + 1;
    const int cells = pitch * (nty + 1) + 1;
    const uint32_t negatives = (uint32_t)grid[cells - 1];
    int32_t* c = grid;
    if(use_lds)
    {
        for(int j = tid; j < cells; j += kCoverThreads)
            s_cells[j] = grid[j];
        c = s_cells;
    }
    for(int j = tid; j < kMaxPasses32 * kBins32; j += kCoverThreads)
        hist[j] = 0;
    if(tid == 0)
    {
        s_carry = negatives;
        s_last = -1;
    }
    __threadfence_block();
    __syncthreads();
    // along x: one wavefront per row, 64 columns at a time with a carry
    for(int y = wave; y < nty; y += kCoverThreads / DSX_WAVE)
    {
        int32_t carry = 0;
        for(int x0 = 0; x0 < ntx; x0 += DSX_WAVE)
        {
            const int x = x0 + lane;
            const int32_t v = x < ntx ? c[y * pitch + x] : 0;
            const int32_t incl = (int32_t)wave_incl_scan32((uint32_t)v, lane) + carry;
            if(x < ntx)
                c[y * pitch + x] = incl;
            carry = __shfl(incl, 63, DSX_WAVE);
        }
    }
    __threadfence_block();
    __syncthreads();
    // along y: one thread per column
    for(int x = tid; x < ntx; x += kCoverThreads)
    {
        int32_t run = 0;
        for(int y = 0; y < nty; ++y)
        {
            run += c[y * pitch + x];
            c[y * pitch + x] = run; // pairs of tile (x, y)
        }
    }
    __threadfence_block();
    __syncthreads();
    // histograms, exclusive scan over the tiles in row-major order, highest occupied tile
    const int tiles = ntx * nty;
    for(int t0 = 0; t0 < tiles; t0 += kCoverThreads)
    {
        const int t = t0 + tid;
        const uint32_t cnt = t < tiles ? (uint32_t)c[(t / ntx) * pitch + (t % ntx)] : 0u;
        // lanes hold consecutive tiles: the lowest digit differs from lane to lane (plain LDS
        // atomics, no conflicts), a higher digit is constant over long runs (one add per run,
        // after a wavefront sum; same-address LDS atomics would serialise)
        {
            const uint32_t slot = (uint32_t)t + 1u;
            for(int p = 0; slot_hist && p < plan.passes; ++p)
            {
                const uint32_t d = (slot >> plan.shift[p]) & plan.mask[p];
                if(plan.shift[p] == 0)
                {
                    if(cnt)
                        atomicAdd(&hist[p * kBins32 + d], cnt);
                    continue;
                }
                uint64_t todo = __ballot(true);
                while(todo)
                {
                    const int leader = __builtin_ctzll(todo);
                    const uint32_t dl = (uint32_t)__builtin_amdgcn_readlane((int)d, leader);
                    const bool mine = d == dl;
                    const uint32_t sum = wave_sum_u32(mine ? cnt : 0u);
                    if(lane == leader && sum)
                        atomicAdd(&hist[p * kBins32 + dl], sum);
                    todo &= ~__ballot(mine);
                }
            }
            const uint64_t occupied = __ballot(cnt != 0);
            if(occupied && lane == 0)
                atomicMax(&s_last, t0 + wave * DSX_WAVE + 63 - __builtin_clzll(occupied));
        }
        const uint32_t incl = wave_incl_scan32(cnt, lane);
        if(lane == 63)
            wave_tot[wave] = incl;
        __syncthreads();
        const uint32_t prefix = s_carry + sum_of_waves_before<kCoverThreads / DSX_WAVE>(wave_tot, wave);
        if(t < tiles)
            ranges[t] = (int32_t)(prefix + incl - cnt);
        __syncthreads();
        if(tid == kCoverThreads - 1)
            s_carry = prefix + incl;
        __syncthreads();
    }
    __threadfence_block();
    __syncthreads();
    const int last = s_last;
    if(!J.plain)
    {
        const int32_t tail = last >= 0 ? ranges[last] : 0;
        for(int t = tid; t < tiles; t += kCoverThreads)
            if(t > last)
                ranges[t] = tail;
    }
    if(tid == 0)
    {
        ranges[tiles] = (int32_t)s_carry; // K
        if(J.last)
            *J.last = last;
        if(J.header)
            *J.header = J.header_value;
        for(int p = 0; p < plan.passes; ++p)
            atomicAdd(&hist[p * kBins32], negatives);
    }
    __syncthreads();
    if(slot_hist)
        for(int j = tid; j < kMaxPasses32 * kBins32; j += kCoverThreads)
            slot_hist[j] = hist[j];
}

// order: the buffer of order_layout(n) whose depth_keys and rects the projection has written
void depth_order_clear_region(const dsx_camera& cam, int64_t n, void* order, uint32_t** words, int64_t* count)
{
    // the sort's histograms, counters and look-back statuses and, right behind them, the corner grid
    const OrderLayout o = order_layout(n, cam.image_width, cam.image_height, cam.list_bin);
    const Sort32Workspace w = sort32_workspace(n, 32, sort32_tile_keys(n));
    *words = reinterpret_cast<uint32_t*>(static_cast<char*>(order) + o.sort + w.hist);
    *count = (int64_t)((w.bytes + (o.ranges - o.cover)) / 4);
}

// k_host (optional, with k_copied): receives the two pair counts (uint64[2]: per-tile lists, bin lists) as
// soon as the rectangles have been counted; k_copied is recorded behind that copy.
int launch_depth_order(const dsx_camera& cam, int64_t n, void* order, hipStream_t stream, bool already_cleared,
                       void* k_host, hipEvent_t k_copied)
{
    if(n <= 0)
        return DSX_OK;
    const OrderLayout o = order_layout(n, cam.image_width, cam.image_height, cam.list_bin);
    char* base = static_cast<char*>(order);
    uint32_t* keys_a = reinterpret_cast<uint32_t*>(base + o.depth_keys);
    uint32_t* keys_b = reinterpret_cast<uint32_t*>(base + o.keys_alt);
    uint32_t* ids_a = reinterpret_cast<uint32_t*>(base + o.ids_a);
    uint32_t* ids_b = reinterpret_cast<uint32_t*>(base + o.ids_b);
    uint32_t* block_sums = reinterpret_cast<uint32_t*>(base + o.block_sums);
    // one fill zeroes the sort's counters and, right behind them, the corner grid
    int rc = DSX_OK;
    if(!already_cleared)
    {
        uint32_t* words;
        int64_t count;
        depth_order_clear_region(cam, n, order, &words, &count);
        rc = launch_fill_u32(words, count, 0u, stream);
    }
    if(rc)
        return rc;

    // pairs per tile: digit histograms of the tile partition and the tile ranges that the second
    // half of the forward needs.  They depend on the rectangles only, not on the depth order,
    // so they run on the helper stream beside the sort (fork after the fill, join at the end).
    hipStream_t side = helper_stream();
    hipEvent_t fork = nullptr, join = nullptr;
    if(side)
    {
        const bool ok = hipEventCreateWithFlags(&fork, hipEventDisableTiming) == hipSuccess &&
                        hipEventCreateWithFlags(&join, hipEventDisableTiming) == hipSuccess &&
                        hipEventRecord(fork, stream) == hipSuccess && hipStreamWaitEvent(side, fork, 0) == hipSuccess;
        if(!ok)
        {
            (void)hipGetLastError();
            side = nullptr;
        }
    }
    bool k_copy_ok = true;
    {
        hipStream_t cs = side ? side : stream;
        const ListGrid lg = list_grid(cam);
        const RangesLayout rl = ranges_layout(lg);
        const int ntx = lg.ntx, nty = lg.nty;
        const int cells = (ntx + 1) * (nty + 1) + 1;
        const int bcells = lg.shift ? (lg.nbx + 1) * (lg.nby + 1) + 1 : 0;
        int32_t* grid = reinterpret_cast<int32_t*>(base + o.cover);
        int32_t* bin_grid = reinterpret_cast<int32_t*>(base + o.bin_cover);
        int32_t* ranges = reinterpret_cast<int32_t*>(base + o.ranges);
        // The corner grids are privatised in LDS whenever they fit (a 4K image has 32 776 cells =
        // 128 KB: one workgroup per CU); beyond 64 KB a kernel needs its limit raised first.
        // Global atomics are the fallback: correct for any grid, but 24 M same-line atomics
        // at 6 M Gaussians cost 0.6 ms and stall the sort passes that run beside them.
        int use_lds = cells + bcells <= kCoverLdsCells ? 1 : 0;
        if(!use_lds && cells + bcells <= kCoverLdsCellsLarge)
        {
            const int bytes = (cells + bcells) * 4;
            use_lds = hipFuncSetAttribute(reinterpret_cast<const void*>(tile_cover_kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess &&
                              hipFuncSetAttribute(reinterpret_cast<const void*>(tile_counts_kernel),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess
                          ? 1
                          : 0;
            if(!use_lds)
                (void)hipGetLastError();
        }
        const int64_t want = (n + kCoverThreads - 1) / kCoverThreads;
        {
            DSX_TIMED("tile_cover_kernel", cs);
            hipLaunchKernelGGL(tile_cover_kernel, dim3((unsigned)min((int64_t)kCoverBlocks, want)), dim3(kCoverThreads),
                               use_lds ? (size_t)(cells + bcells) * 4 : 0, cs,
                               reinterpret_cast<const uint2*>(base + o.rects), n, ntx, nty, lg.shift, lg.nbx, lg.nby,
                               use_lds, grid, bin_grid, reinterpret_cast<unsigned long long*>(base + o.key_count));
        }
        // both pair counts, 16 bytes: of the per-tile lists (what the reference calls K: the fine ranges
        // and final_idx index that many pairs) and of the bin lists (zero when the lists are per tile)
        if(k_host)
            k_copy_ok = hipMemcpyAsync(k_host, base + o.key_count, 16, hipMemcpyDeviceToHost, cs) == hipSuccess &&
                        hipEventRecord(k_copied, cs) == hipSuccess;
        {
            CountsJobs jobs;
            CountsJob& fine = jobs.job[0];
            fine.grid = grid;
            fine.ntx = ntx;
            fine.nty = nty;
            fine.plain = 0;
            fine.plan = digits32(slot_bits(lg.tiles()));
            fine.slot_hist = lg.shift ? nullptr : reinterpret_cast<uint32_t*>(base + o.slot_hist);
            fine.ranges = ranges + rl.fine;
            fine.last = lg.shift ? ranges + rl.last_tile : nullptr;
            fine.header = ranges + rl.header;
            fine.header_value = lg.shift;
            jobs.job[1] = fine;
            if(lg.shift)
            {
                CountsJob& bins = jobs.job[1];
                bins.grid = bin_grid;
                bins.ntx = lg.nbx;
                bins.nty = lg.nby;
                bins.plain = 1;
                bins.plan = digits32(slot_bits(lg.bins()));
                bins.slot_hist = reinterpret_cast<uint32_t*>(base + o.slot_hist);
                bins.ranges = ranges + rl.bins;
                bins.last = nullptr;
                bins.header = nullptr;
            }
            DSX_TIMED("tile_counts_kernel", cs);
            hipLaunchKernelGGL(tile_counts_kernel, dim3(lg.shift ? 2 : 1), dim3(kCoverThreads),
                               use_lds ? (size_t)cells * 4 : 0, cs, jobs, use_lds);
        }
    }
    bool joined = true;
    if(side)
        joined = hipEventRecord(join, side) == hipSuccess;
    // the caller's stream takes the helper's work back in before this function returns
    auto finish = [&](int status) {
        if(side && joined)
            joined = hipStreamWaitEvent(stream, join, 0) == hipSuccess;
        if(fork)
            (void)hipEventDestroy(fork);
        if(join)
            (void)hipEventDestroy(join);
        return status ? status : (joined ? DSX_OK : DSX_ERR_RUNTIME);
    };
    if(hipGetLastError() != hipSuccess)
        return finish(DSX_ERR_LAUNCH);
    if(!k_copy_ok)
        return finish(DSX_ERR_RUNTIME);

    uint32_t *ko, *vo;
    // 32 key bits = 4 passes: the values (iota in pass 0) go b, a, b, a and end in ids_a
    // the rectangles travel through the passes when they pack into 32 bits (the passes end in
    // rects_sorted, whose first half holds the packed ones of the passes in between), else the last
    // pass gathers them
    const bool carry = tiles_x(cam.image_width) <= kRect32MaxTiles && tiles_y(cam.image_height) <= kRect32MaxTiles;
    rc = launch_sort32(n, 32, keys_a, ids_a, keys_b, ids_b, true, false, base + o.sort, stream, &ko, &vo,
                       reinterpret_cast<const uint2*>(base + o.rects), reinterpret_cast<uint2*>(base + o.rects_sorted),
                       true, carry ? reinterpret_cast<uint32_t*>(base + o.rects_sorted) : nullptr,
                       carry ? reinterpret_cast<uint32_t*>(base + o.rects32) : nullptr);
    if(rc)
        return finish(rc);
    if(vo != ids_a)
        return finish(DSX_ERR_RUNTIME);
    const int64_t blocks = (n + kProjBlock - 1) / kProjBlock;
    {
        DSX_TIMED("ordered_block_sums_kernel", stream);
        hipLaunchKernelGGL(ordered_block_sums_kernel, dim3((unsigned)blocks), dim3(kProjBlock), 0, stream,
                           reinterpret_cast<const uint2*>(base + o.rects_sorted), n,
                           list_grid(cam).shift, block_sums);
    }
    if(hipGetLastError() != hipSuccess)
        return finish(DSX_ERR_LAUNCH);
    return finish(launch_scan_u32(blocks, block_sums, block_sums + blocks, stream));
}

// ---------------------------------------------------------------------------------------
// emission in depth order: a workgroup owns a range of OUTPUT pairs and walks the blocks of 256
// depth-ordered Gaussians that reach into it; one thread per output pair, so the work per
// workgroup is bounded and the stores are contiguous however uneven the tile counts are
// ---------------------------------------------------------------------------------------

#ifndef DSX_EMIT_WINDOWS
#define DSX_EMIT_WINDOWS 4
#endif
constexpr int kEmitWindows = DSX_EMIT_WINDOWS; // windows of 256 outputs per round of the emission
constexpr int kEmitChunkMax = 4096;            // outputs per workgroup: at most this many ...
constexpr int kEmitWorkgroups = 4096;          // ... and fewer when that leaves less than this many workgroups

// kMasks (lists per bin, SlotT = uint32_t): the high half of a pair's slot word says which tiles of the
// bin the Gaussian's rectangle covers, bit x for the columns and bit 8 + y for the rows of the bin
// (a rectangle is the product of a column range and a row range).  The partition sorts by the low bits
// only and carries the rest along; the blend kernels pick a tile's entries out of its bin's list by
// testing the tile's two bits.  Pairs of negative depth (slot 0, one list for the whole image) carry
// all sixteen bits.
template <typename SlotT, bool kMasks>
__global__ __launch_bounds__(kProjBlock) void emit_ordered_kernel(const uint32_t* __restrict__ order,
                                                                  const uint2* __restrict__ rects_sorted,
                                                                  const uint32_t* __restrict__ block_offsets,
                                                                  int64_t n, int64_t k, int ntx, int shift,
                                                                  SlotT* __restrict__ slots, int32_t* __restrict__ ids,
                                                                  const int32_t* __restrict__ ranges_in,
                                                                  int32_t* __restrict__ ranges_out, int range_count,
                                                                  uint32_t* __restrict__ clear, int64_t clear_words,
                                                                  int chunk)
{
    __shared__ uint32_t s_off[kProjBlock + 1];
    // per Gaussian of the block: x = first output, y = slot of the rectangle's first tile (0 for
    // negative depths), z = width (0 marks a negative depth: every pair goes to slot 0), w = id
    __shared__ uint4 s_rec[kProjBlock];
    __shared__ uint2 s_rect[kMasks ? kProjBlock : 1]; // the tile rectangles themselves (for the masks)
    __shared__ __attribute__((aligned(16))) uint32_t wave_tot[kProjBlock / DSX_WAVE];
    __shared__ uint32_t s_mark[kEmitWindows * kProjBlock];
    __shared__ __attribute__((aligned(16))) uint32_t s_wave_max[kEmitWindows][kProjBlock / DSX_WAVE];
    static_assert(kProjBlock == 4 * DSX_WAVE, "four wavefronts per workgroup");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
#pragma unroll
    for(int wdw = 0; wdw < kEmitWindows; ++wdw)
        s_mark[wdw * kProjBlock + tid] = 0;

    // the tile ranges were derived from the rectangles before any pair existed: hand them out
    for(int j = blockIdx.x * kProjBlock + tid; j < range_count; j += gridDim.x * kProjBlock)
        ranges_out[j] = ranges_in[j];
    // housekeeping for the partition that follows: its counters and look-back statuses start at zero
    for(int64_t j = (int64_t)blockIdx.x * kProjBlock + tid; j < clear_words; j += (int64_t)gridDim.x * kProjBlock)
        clear[j] = 0u;

    // This workgroup's share: outputs [o0, o1).  The work is cut by OUTPUTS, not by Gaussians: a
    // block of 256 near Gaussians can own a hundred thousand pairs and a block of far ones a few
    // hundred, and a workgroup that walked a whole heavy block alone set the kernel's time.
    const int64_t o0 = (int64_t)blockIdx.x * chunk;
    const int64_t o1 = min(o0 + chunk, k);
    if(o0 >= o1) // uniform
        return;
    const int64_t blocks = (n + kProjBlock - 1) / kProjBlock;
    // first block of 256 Gaussians (in depth order) whose outputs reach into the share: the largest
    // b with block_offsets[b] <= o0, by a 64-way search (every wavefront does it for itself)
    int64_t first = 0;
    {
        int64_t lo = 0, hi = blocks; // block_offsets[lo] <= o0; the answer lies in [lo, hi)
        while(hi - lo > 1)
        {
            const int64_t step = (hi - lo + 63) / 64;
            const int64_t probe = lo + lane * step;
            const bool ok = probe < hi && (int64_t)block_offsets[probe] <= o0; // true for a prefix of the lanes
            const int reached = __popcll(__ballot(ok)) - 1;                   // lane 0 always holds
            lo += reached * step;
            hi = min(hi, lo + step);
        }
        first = lo;
    }
    for(int64_t blk = first; blk < blocks; ++blk)
    {
        const int64_t base = block_offsets[blk];
        if(base >= o1) // uniform: the share is complete
            break;
        __syncthreads(); // the previous round has finished with the LDS arrays
        const int64_t p = blk * kProjBlock + tid;
        uint32_t count = 0;
        uint4 rec = make_uint4(0u, 0u, 0u, 0u);
        if(p < n)
        {
            // (ntx: lists per row, i.e. bins per row when the lists are binned)
            const uint32_t g = order[p];
            const uint2 r = rects_sorted[p];
            count = list_count(r, shift);
            const bool negative = (r.y >> 31) != 0;
            uint32_t first_x = r.x & 0xffffu, first_y = r.x >> 16, w = r.y & 0xffffu;
            if(shift && count && !negative)
            {
                const BinRect b = bin_rect(r, shift);
                first_x = b.bx;
                first_y = b.by;
                w = b.bw;
            }
            rec.y = negative ? 0u : first_y * (uint32_t)ntx + first_x + 1u;
            rec.z = negative ? 0u : w;
            rec.w = g;
            if(kMasks)
                s_rect[tid] = r;
        }
        const uint32_t incl = wave_incl_scan32(count, lane);
        if(lane == 63)
            wave_tot[wave] = incl;
        __syncthreads();
        const uint32_t prefix = sum_of_waves_before<kProjBlock / DSX_WAVE>(wave_tot, wave);
        rec.x = prefix + incl - count;
        s_off[tid] = rec.x;
        s_rec[tid] = rec;
        if(tid == kProjBlock - 1)
            s_off[kProjBlock] = prefix + incl;
        __syncthreads();

        const uint32_t total = s_off[kProjBlock];
        const uint32_t my_start = s_off[tid];
        // the block's outputs that fall into the share: [ja, jb) of its `total`
        const uint32_t ja = (uint32_t)(max(o0, base) - base);
        const uint32_t jb = (uint32_t)(min(o1, base + (int64_t)total) - base);
        if(jb <= ja) // uniform (an empty block, or one that ends before the share)
            continue;
        // Which Gaussian owns output j?  Every Gaussian that emits marks the output where its run
        // starts with (its index + 1); the owner of j is the largest mark at or before j, i.e. an
        // inclusive max-scan over the outputs (DPP inside the wavefront, LDS across wavefronts
        // and across rounds of 256 outputs).  Costs a dozen VALU instructions per output
        // instead of the eight dependent LDS reads of a binary search.
        // A block of near Gaussians can own tens of thousands of outputs while the workgroup
        // walks them serially, so a round covers kEmitWindows windows of 256 outputs with two
        // barriers in all (the kernel's time is the longest such walk).
        uint32_t carry = 0; // mark of the owner of the last output before the round
        if(ja > 0)          // uniform: the share starts inside the block
        {
            // the last Gaussian whose run starts before ja (starts are monotone in the thread index)
            const uint64_t early = __ballot(count && my_start < ja);
            if(lane == 0)
                s_wave_max[0][wave] = early ? (uint32_t)(wave * DSX_WAVE + 64 - __builtin_clzll(early)) : 0u;
            __syncthreads();
            carry = max(max(s_wave_max[0][0], s_wave_max[0][1]), max(s_wave_max[0][2], s_wave_max[0][3]));
            __syncthreads();
        }
        for(uint32_t j0 = ja; j0 < jb; j0 += kEmitWindows * kProjBlock) // uniform
        {
            if(count && my_start >= j0 && my_start < j0 + kEmitWindows * kProjBlock)
                s_mark[my_start - j0] = (uint32_t)tid + 1u;
            __syncthreads();
            uint32_t m[kEmitWindows];
#pragma unroll
            for(int wdw = 0; wdw < kEmitWindows; ++wdw)
            {
                m[wdw] = s_mark[wdw * kProjBlock + tid];
                s_mark[wdw * kProjBlock + tid] = 0; // ready for the next round (and the next block)
                m[wdw] = wave_incl_max_scan(m[wdw]);
                if(lane == 63)
                    s_wave_max[wdw][wave] = m[wdw];
            }
            __syncthreads();
            uint32_t before = carry; // largest mark before this thread's output of the current window
#pragma unroll
            for(int wdw = 0; wdw < kEmitWindows; ++wdw)
            {
                // the four wavefronts' maxima in one 16-byte read; the earlier wavefronts' count for this one
                static_assert(kProjBlock / DSX_WAVE == 4, "four wavefronts per emission workgroup");
                const uint4 wm = *reinterpret_cast<const uint4*>(s_wave_max[wdw]);
                const uint32_t mine = max(max(before, wave > 0 ? wm.x : 0u), max(wave > 1 ? wm.y : 0u, wave > 2 ? wm.z : 0u));
                const uint32_t owner = max(m[wdw], mine) - 1u; // every output has an owner: never 0 - 1
                before = max(before, max(max(wm.x, wm.y), max(wm.z, wm.w)));
                const uint32_t j = j0 + wdw * kProjBlock + tid;
                if(j < jb)
                {
                    const uint4 own = s_rec[owner]; // one 16-byte LDS read per output
                    const uint32_t r = j - own.x;
                    const uint32_t w = own.z;
                    uint32_t slot = kMasks ? 0xffff0000u : 0u;
                    if(w)
                    {
                        // r / w by a float reciprocal (r < 2^24 tiles per Gaussian), corrected by one step
                        uint32_t ry = (uint32_t)((float)r * __builtin_amdgcn_rcpf((float)w));
                        if(ry * w > r)
                            --ry;
                        else if((ry + 1) * w <= r)
                            ++ry;
                        const uint32_t rx = r - ry * w;
                        slot = own.y + ry * (uint32_t)ntx + rx;
                        if(kMasks)
                        {
                            // the rectangle's columns and rows inside this bin, as bit ranges [lo, hi]
                            const uint2 tr = s_rect[owner];
                            const int side = 1 << shift;
                            const int tsx = (int)(tr.x & 0xffffu), tsy = (int)(tr.x >> 16);
                            const int tw = (int)(tr.y & 0xffffu), th = (int)((tr.y >> 16) & 0x7fffu);
                            const int x0 = (int)(((uint32_t)tsx >> shift) + rx) << shift; // the bin's first column
                            const int y0 = (int)(((uint32_t)tsy >> shift) + ry) << shift;
                            const int xlo = max(tsx - x0, 0), xhi = min(tsx + tw - 1 - x0, side - 1);
                            const int ylo = max(tsy - y0, 0), yhi = min(tsy + th - 1 - y0, side - 1);
                            const uint32_t xm = ((2u << xhi) - 1u) & ~((1u << xlo) - 1u);
                            const uint32_t ym = ((2u << yhi) - 1u) & ~((1u << ylo) - 1u);
                            slot |= (xm | (ym << 8)) << 16;
                        }
                    }
                    slots[base + j] = (SlotT)slot;
                    ids[base + j] = (int32_t)own.w;
                }
            }
            carry = before;
            // (the next round's marks are written after this round's reads of s_wave_max: the
            // barrier after them orders both)
        }
    }
}

// tile slots 0..num_tiles fit 16 bits for every image up to 65534 tiles (4K has 32400)
static bool slots_are_u16(int num_tiles)
{
    return num_tiles + 1 <= 65535;
}

// binned: the slot words are 32 bits (slot in the low half, the tile mask in the high half) and the
// sorted ones end in the caller's buffer, behind the ids
ListsWorkspace lists_workspace(int64_t k, int num_tiles, bool binned)
{
    auto align = [](size_t x) { return (x + 255) & ~(size_t)255; };
    ListsWorkspace w;
    const size_t slot_bytes = (binned || !slots_are_u16(num_tiles)) ? 4 : 2;
    w.passes = digits32(slot_bits(num_tiles)).passes;
    size_t off = 0;
    w.slots_a = off;
    off = align(off + (size_t)k * slot_bytes);
    w.slots_b = off;
    off = align(off + (binned ? 0 : (size_t)k * slot_bytes));
    w.ids_alt = off;
    off = align(off + (size_t)k * 4);
    w.sort = off;
    off += sort32_workspace(k, slot_bits(num_tiles), sort32_tile_keys(k)).bytes;
    w.bytes = align(off);
    return w;
}

// num_tiles: lists that the pairs are partitioned into (tiles, or bins when the lists are binned: kMasks)
template <typename SlotT, bool kMasks>
static int tile_lists_impl(const dsx_camera& cam, int64_t n, int64_t k, int num_tiles, const void* order,
                           int32_t* sorted_ids, int32_t* ranges, void* workspace, hipStream_t stream)
{
    const OrderLayout o = order_layout(n, cam.image_width, cam.image_height, cam.list_bin);
    const char* obase = static_cast<const char*>(order);
    const ListGrid lg = list_grid(cam);
    const RangesLayout rl = ranges_layout(lg);
    // what the depth order left ready: everything but the part that the blend forward writes
    const int ready_words = rl.ready;
    if(k <= 0)
    {
        // no pairs: the ranges are all zero (and no tile is occupied)
        int rc = launch_fill_u32(reinterpret_cast<uint32_t*>(ranges), ready_words, 0u, stream);
        if(rc == DSX_OK && lg.shift)
            rc = launch_fill_u32(reinterpret_cast<uint32_t*>(ranges) + rl.header, 1, (uint32_t)lg.shift, stream);
        if(rc == DSX_OK && lg.shift)
            rc = launch_fill_u32(reinterpret_cast<uint32_t*>(ranges) + rl.last_tile, 1, 0xffffffffu, stream);
        return rc;
    }
    const ListsWorkspace w = lists_workspace(k, num_tiles, kMasks);
    const int bits = slot_bits(num_tiles);
    char* base = static_cast<char*>(workspace);
    uint32_t* ids_final = reinterpret_cast<uint32_t*>(sorted_ids);
    uint32_t* ids_other = reinterpret_cast<uint32_t*>(base + w.ids_alt);
    // ping-pong parity: start so that the last pass lands the ids in the caller's buffer (and, for
    // binned lists, the slot words with their masks right behind them)
    const bool even = (w.passes % 2) == 0;
    uint32_t* vals_a = even ? ids_final : ids_other;
    uint32_t* vals_b = even ? ids_other : ids_final;
    SlotT* slots_final = kMasks ? reinterpret_cast<SlotT*>(ids_final + k) : reinterpret_cast<SlotT*>(base + w.slots_b);
    SlotT* slots_other = reinterpret_cast<SlotT*>(base + w.slots_a);
    SlotT* slots_a = (kMasks && even) ? slots_final : slots_other;
    SlotT* slots_b = (kMasks && even) ? slots_other : slots_final;
    int rc = DSX_OK;
    const Sort32Workspace sw = sort32_workspace(k, bits, sort32_tile_keys(k));
    {
        DSX_TIMED("emit_ordered_kernel", stream);
        // outputs per workgroup: a multiple of 256 between 256 and kEmitChunkMax
        const int64_t want = (k + kEmitWorkgroups - 1) / kEmitWorkgroups;
        const int chunk = (int)min((int64_t)kEmitChunkMax, ((want + kProjBlock - 1) / kProjBlock) * kProjBlock);
        hipLaunchKernelGGL((emit_ordered_kernel<SlotT, kMasks>), dim3((unsigned)((k + chunk - 1) / chunk)),
                           dim3(kProjBlock), 0, stream, reinterpret_cast<const uint32_t*>(obase + o.ids_a),
                           reinterpret_cast<const uint2*>(obase + o.rects_sorted),
                           reinterpret_cast<const uint32_t*>(obase + o.block_sums), n, k,
                           lg.shift ? lg.nbx : lg.ntx, lg.shift, slots_a, reinterpret_cast<int32_t*>(vals_a),
                           reinterpret_cast<const int32_t*>(obase + o.ranges), ranges, ready_words,
                           reinterpret_cast<uint32_t*>(base + w.sort + sw.hist), (int64_t)(sw.bytes / 4), chunk);
    }
    DSX_LAUNCH_CHECK();
    SlotT* ko;
    uint32_t* vo;
    // per-tile lists: the sorted slots themselves are not needed (the ranges are known already);
    // binned lists: they are kept for their masks
    rc = DSX_ERR_RUNTIME;
#define DSX_PARTITION_ITEMS(ITEMS)                                                                                    \
    case ITEMS:                                                                                                       \
        rc = sort32_passes<SlotT, kSortThreads32, ITEMS>(k, bits, slots_a, vals_a, slots_b, vals_b, false, kMasks,     \
                                                         base + w.sort, "onesweep32_kernel<tile partition>", stream,  \
                                                         &ko, &vo, nullptr, nullptr,                                  \
                                                         reinterpret_cast<const uint32_t*>(obase + o.slot_hist));     \
        break
    switch(sort32_items(k))
    {
        DSX_PARTITION_ITEMS(1);
        DSX_PARTITION_ITEMS(2);
        DSX_PARTITION_ITEMS(3);
        DSX_PARTITION_ITEMS(4);
        DSX_PARTITION_ITEMS(6);
        DSX_PARTITION_ITEMS(8);
        DSX_PARTITION_ITEMS(kSortItemsMax32);
    }
#undef DSX_PARTITION_ITEMS
    if(rc)
        return rc;
    if(kMasks && ko != slots_final)
        return DSX_ERR_RUNTIME;
    return vo == ids_final ? DSX_OK : DSX_ERR_RUNTIME;
}

// order: buffer of order_layout(n) after launch_depth_order.  Writes sorted_ids[k] and the ready part
// of ranges (ranges_layout: per-tile ranges and, for binned lists, the last occupied tile and the
// bins' ranges).
int launch_tile_lists(const dsx_camera& cam, int64_t n, int64_t k, const void* order, int32_t* sorted_ids,
                      int32_t* ranges, void* workspace, hipStream_t stream)
{
    const ListGrid lg = list_grid(cam);
    const int num_tiles = lg.lists();
    if(k >= (1ll << 30))
        return DSX_ERR_TOO_LARGE;
    if(n <= 0)
        k = 0;
    if(lg.shift)
    {
        if(num_tiles + 1 > 65535) // (the slot shares its word with the 16-bit mask)
            return DSX_ERR_TOO_LARGE;
        return tile_lists_impl<uint32_t, true>(cam, n, k, num_tiles, order, sorted_ids, ranges, workspace, stream);
    }
    if(slots_are_u16(num_tiles))
        return tile_lists_impl<uint16_t, false>(cam, n, k, num_tiles, order, sorted_ids, ranges, workspace, stream);
    return tile_lists_impl<uint32_t, false>(cam, n, k, num_tiles, order, sorted_ids, ranges, workspace, stream);
}

} // namespace dsx
