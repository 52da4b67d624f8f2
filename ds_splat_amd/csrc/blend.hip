// Stages 4 and 5a for gfx950: per-tile alpha blending, forward (front to back) and backward
// (back to front).  Sorted entries are gathered into LDS in batches as two float4 arrays plus
// one float array, so an entry costs two 128-bit and one 32-bit LDS broadcast read.
#include "dsx_common.h"

#include <atomic>
#include <cstdlib>

namespace dsx
{

constexpr float kAlphaThreshold = 1.0f / 255.0f;

// exp through the hardware base-2 exponential (the reference is built with fast-math).  The factor
// log2(e) is applied to the finished exponent, per pixel: folded into the conic coefficients when an
// entry is staged it would save that multiply, but every term of the quadratic form would carry one
// more rounding, and where the terms are large and cancel (thin, long splats far from their centre)
// the image then moves 1.6 times as far from the reference's as it does now.
__device__ __forceinline__ float fast_exp(float x)
{
    return __builtin_amdgcn_exp2f(x * 1.4426950408889634f);
}

// The exponent of a splat at a pixel, -1/2 (a dx^2 + c dy^2) - b dx dy with d = pixel - mean, in
// ONE fixed sequence of roundings (explicit fused multiply-adds, no contraction left to the
// compiler): the forward and the backward kernel must get the same bits, because both compare the
// resulting alpha with 1/255 on their own.  If they disagreed on a borderline entry, the backward
// would rebuild the transmittance of every entry in front of it from a final value that does
// (or does not) contain its factor: an error of alpha in all their gradients at that pixel.
// (The halves are taken by the caller: a_half = -a/2 and c_half = c/2, exact scalings, so it does
// not matter to the bits whether they are applied per entry or once when the entry is staged.)
struct ExponentX
{
    float ax, bx; // -1/2 a dx^2 and b dx
};
__device__ __forceinline__ ExponentX exponent_x(float a_half, float b, float dx)
{
#pragma clang fp contract(off)
    ExponentX r;
    r.bx = b * dx;
    r.ax = a_half * dx * dx;
    return r;
}
__device__ __forceinline__ float exponent_xy(ExponentX x, float c_half, float dy)
{
#pragma clang fp contract(off)
    const float inner = __builtin_fmaf(c_half, dy, x.bx);
    return __builtin_fmaf(-inner, dy, x.ax);
}

// Can this entry reach alpha >= 1/255 at ANY pixel of the tile?  The exponent's quadratic form
// q(d) = 1/2 (a dx^2 + c dy^2) + b dx dy is convex, so its minimum over the box of pixel
// centres is 0 if the centre lies inside and otherwise sits on one of the four edges, where it
// is a clamped one-dimensional parabola.  An entry is dropped only if opacity * exp(-qmin)
// stays below 0.99/255 (one percent of slack against rounding); whatever fails a comparison
// (NaN, degenerate conic) is kept.  The reference's tile rectangle is the bounding square of a
// 3-sigma circle, so about half of the (tile, entry) pairs a tile walks touch none of its pixels.
__device__ __forceinline__ float edge_min(float a, float b, float c, float u, float v0, float v1)
{
    // minimum over v in [v0, v1] of 1/2 (a u^2 + c v^2) + b u v   (u fixed, c > 0)
    const float v = fminf(v1, fmaxf(v0, -b * u * __builtin_amdgcn_rcpf(c)));
    return 0.5f * (a * u * u + c * v * v) + b * u * v;
}

// (span_y: last row of pixel centres of the box, 15 for a whole tile, 3 for a band of four rows)
__device__ __forceinline__ bool entry_reaches_tile(float mx, float my, float a, float b, float c, float opacity,
                                                   float box_x0, float box_y0, float span_y = 15.0f)
{
    const float dx0 = box_x0 - mx, dx1 = box_x0 + 15.0f - mx;
    const float dy0 = box_y0 - my, dy1 = box_y0 + span_y - my;
    const bool inside = dx0 <= 0.0f && dx1 >= 0.0f && dy0 <= 0.0f && dy1 >= 0.0f;
    float qmin = fminf(fminf(edge_min(a, b, c, dx0, dy0, dy1), edge_min(a, b, c, dx1, dy0, dy1)),
                       fminf(edge_min(c, b, a, dy0, dx0, dx1), edge_min(c, b, a, dy1, dx0, dx1)));
    qmin = inside ? 0.0f : qmin;
    const bool well_formed = a > 0.0f && c > 0.0f;
    const float limit = __logf(opacity * (255.0f / 0.99f)); // ln(opacity / (0.99/255))
    return !(well_formed && qmin > limit);
}

// Pixels per lane of the blend kernels: 4 (one wavefront per tile) when the image has enough tiles
// to occupy the chip (8 wavefronts on each of 1024 SIMDs), else 1 (four wavefronts per tile: more
// instructions in all, but four times as many wavefronts).  Measured crossover (500 K Gaussians,
// 640x480 to 1920x1080): about 5000 tiles for the forward, 1600 for the backward, whose
// one-pixel form also quadruples the atomics.  dsx_set_blend_pixels_per_lane(1 | 4) overrides the
// choice for the whole process (tests run both forms); DSX_BLEND_PIXELS_PER_LANE=1|4 in the
// environment gives the override's initial value and is read once.
static std::atomic<int> g_forced_pixels_per_lane{-1}; // -1: not yet read from the environment, 0: automatic

static int forced_pixels_per_lane()
{
    int v = g_forced_pixels_per_lane.load(std::memory_order_relaxed);
    if(v >= 0)
        return v;
    v = 0;
    if(const char* forced = getenv("DSX_BLEND_PIXELS_PER_LANE"))
        if((forced[0] == '1' || forced[0] == '4') && forced[1] == 0)
            v = forced[0] - '0';
    int expected = -1;
    g_forced_pixels_per_lane.compare_exchange_strong(expected, v, std::memory_order_relaxed);
    return g_forced_pixels_per_lane.load(std::memory_order_relaxed);
}

int set_blend_pixels_per_lane(int pixels)
{
    if(pixels != 0 && pixels != 1 && pixels != 4)
        return DSX_ERR_BAD_ARG;
    g_forced_pixels_per_lane.store(pixels, std::memory_order_relaxed);
    return DSX_OK;
}

static int blend_pixels_per_lane(int num_tiles, int four_from)
{
    const int forced = forced_pixels_per_lane();
    if(forced != 0)
        return forced;
    return num_tiles >= four_from ? 4 : 1;
}
// Binned tile lists (see ListGrid): what a blend kernel needs to find a tile's entries in its
// bin's list.  fine[t] .. fine[t + 1] is the tile's range in the reference's fully sorted key
// array: its length says how many entries of the bin list belong to the tile, and its start turns
// "the i-th entry of the tile" into the index that the reference's final_idx holds.
struct BinLists
{
    const int32_t* fine;      // int32[tiles + 1]
    const int32_t* last_tile; // highest occupied tile (-1: none)
    const int32_t* bins;      // int32[bins + 1]
    int32_t* walk;            // int32[tiles * 8]: per tile and band of four rows, where the forward's scan of the bin list stopped and how many of the tile's entries it had met by then
    int shift, nbx, nty;
};

// Where tile `tile` finds its entries.  The reference never records the end of the LAST run of
// its sorted keys (cpp/rasterizer_kernels.cu:313-322, cpp/rasterizer_torch.cu:31-39), so the pairs
// of the highest occupied tile are walked by the image's last tile instead, and by nobody if that
// is another tile; with no tile occupied at all, the last tile walks the pairs of negative depth
// (slot 0, positions [0, bins[0])), every one of them.  The per-tile ranges carry those rules;
// here they decide whose pairs (src) the tile takes out of which bin's list.
struct TileSource
{
    int start, end; // positions in sorted_ids to scan
    int count;      // entries among them that belong to the tile
    int fine_base;  // index of the tile's first entry in the fully sorted key array
    int sx, sy;     // the tile whose rectangle membership selects the entries; sx < 0: every entry belongs
};
__device__ __forceinline__ TileSource tile_source(const BinLists& L, int tile, int ntx)
{
    TileSource t;
    t.fine_base = L.fine[tile];
    t.count = L.fine[tile + 1] - t.fine_base;
    t.start = t.end = 0;
    t.sx = t.sy = 0;
    if(t.count <= 0)
        return t;
    int src = tile;
    if(tile == ntx * L.nty - 1)
        src = *L.last_tile;
    if(src < 0)
    {
        t.sx = -1;
        t.end = L.bins[0];
        return t;
    }
    t.sx = src % ntx;
    t.sy = src / ntx;
    const int bin = (t.sy >> L.shift) * L.nbx + (t.sx >> L.shift);
    t.start = L.bins[bin];
    t.end = L.bins[bin + 1];
    return t;
}

// Every pair of a bin list carries, in the high half of its key word, which tiles of the bin the
// Gaussian's rectangle covers: bit x for the columns, bit 8 + y for the rows (a rectangle is the
// product of a column range and a row range).  The two bits of the tile this wavefront takes its
// entries for; 0 when every entry belongs (the list of negative depths).
__device__ __forceinline__ uint32_t tile_bits_of(const TileSource& t, int shift)
{
    if(t.sx < 0)
        return 0u;
    const int side = (1 << shift) - 1;
    return (1u << (t.sx & side)) | (256u << (t.sy & side));
}

// number of set bits of a wavefront mask below this lane
__device__ __forceinline__ int bits_below_lane(uint64_t mask)
{
    return (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

constexpr int kFwdFourPixelsFrom = 5000; // tiles
constexpr int kBwdFourPixelsFrom = 1600;

// -----------------------------------------------------------------------------------------
// forward: cpp/rasterizer_kernels.cu:341-431
// -----------------------------------------------------------------------------------------
// One wavefront per 16x16 tile, four pixels per lane (lane l owns column l & 15 of rows
// (l >> 4) + {0, 4, 8, 12}).  Every LDS broadcast read of an entry then feeds 256 pixel
// updates instead of 64, which moves the kernel from the LDS pipe to the VALU, gives each
// lane four independent dependency chains, and needs no workgroup barrier at all.
// Images of few tiles (fewer wavefronts than the chip has slots) take kFwdPix = 1 instead: four
// wavefronts per tile, each with one band of four rows and one pixel per lane; a tile's walk is
// then four times shorter in time, which is what counts when the launch cannot fill the chip.
constexpr int kFwdBatch = 128; // sorted entries staged in LDS per round (two per lane)
constexpr int kScanGroups = 4; // groups of 64 positions of a bin's list whose loads are in flight together

// 8 wavefronts per SIMD (at most 64 VGPRs): all tiles of a 1080p image are resident at once
// kBinned: the entries come out of the list of the tile's bin (BinLists).  The wavefront first
// FILTERS the bin's list: 64 positions at a time it reads the pair's id and key word (two coalesced
// 4-byte loads, the next 64 already in flight), tests the two bits of its tile in the key's mask,
// and packs the ids of its own entries into a queue in LDS (the staging arrays' memory, which is
// free between two rounds) until more than 64 are there or the list ends.  Only those are then gathered,
// tested for reach and staged as with per-tile lists, so a tile pays a dozen instructions per 64
// entries of its bin's list instead of a gather and a rectangle test per entry; a scene whose
// pixels do not saturate early, where every tile reads its bin's whole list, costs a few percent
// more than with per-tile lists instead of twice as much.  final_idx still receives the
// reference's index: the tile's range start plus the entry's rank among the tile's own entries.
template <int kFwdPix, bool kBinned>
__global__ __launch_bounds__(DSX_WAVE) __attribute__((amdgpu_waves_per_eu(8, 8))) void blend_fwd_kernel(const int32_t* __restrict__ ranges,
                                                             const int32_t* __restrict__ ids,
                                                             const float4* __restrict__ splats,
                                                             float* __restrict__ image, float* __restrict__ final_T,
                                                             int32_t* __restrict__ final_idx, int W, int H, int ntx,
                                                             uint32_t last_id, int k,
                                                             const int32_t* __restrict__ header, int header_shift,
                                                             const uint32_t* __restrict__ sort_flag_a,
                                                             const uint32_t* __restrict__ sort_flag_b,
                                                             float4* __restrict__ prep, int64_t prep_count,
                                                             uint8_t* __restrict__ prep_marks,
                                                             const BinLists lists)
{
    __shared__ float4 s_a[kFwdBatch]; // pixel x, pixel y, conic -a/2, conic b
    __shared__ float4 s_b[kFwdBatch]; // conic c/2, opacity, red, green
    __shared__ float s_c[kFwdBatch];  // blue
    // the queue of the tile's own entries (binned lists) lives in s_a between two rounds: up to 128 ids
    int* const s_queue = reinterpret_cast<int*>(s_a);

    const int lane = threadIdx.x;
    const int tile = kFwdPix == 4 ? blockIdx.x : blockIdx.x >> 2;
    const int band = kFwdPix == 4 ? 0 : blockIdx.x & 3; // which four rows of the tile (one-pixel form)
    const int tx = tile % ntx;
    const int ty = tile / ntx;
    const int x = tx * kTile + (lane & 15);
    const int y0 = ty * kTile + 4 * band + (lane >> 4);
    const float pxf = (float)x + 0.5f;
    // first pixel centre and last row of the pixels this wavefront owns
    const float box_x0 = (float)(tx * kTile) + 0.5f, box_y0 = (float)(ty * kTile + 4 * band) + 0.5f;
    const float span_y = kFwdPix == 4 ? 15.0f : 3.0f;

    // The lists are data from the device: positions are taken for what they are only inside
    // sorted_ids[0, k), and a `ranges` buffer that was built for another bin size (its header word,
    // which every layout has in the same place, says which) is not read any further; the image is
    // then NaN, like after a sort that gave up.
    const bool layout_ok = header == nullptr || *header == header_shift;
    int start = 0, end = 0;
    TileSource src = {};
    if(kBinned)
    {
        if(layout_ok)
            src = tile_source(lists, tile, ntx);
        start = src.start;
        end = src.end;
    }
    else if(layout_ok)
    {
        start = ranges[tile];
        end = ranges[tile + 1];
    }
    start = min(max(start, 0), k);
    end = min(max(end, 0), k);

    // A pixel that has stopped (or lies outside the image) gets NaN as its row coordinate: its
    // exponent is then NaN, the test `power < 0` fails whatever the entry holds, and the loop
    // needs no per-pixel flag.  `alive` counts the wavefront's live pixels (a scalar: it is kept
    // from ballots, on the scalar unit, and costs the vector unit nothing).
    float pyf[kFwdPix], T[kFwdPix], cr[kFwdPix], cg[kFwdPix], cb[kFwdPix];
    int last[kFwdPix];
    int alive = 0;
#pragma unroll
    for(int p = 0; p < kFwdPix; ++p)
    {
        const int y = y0 + 4 * p;
        const bool inside = x < W && y < H;
        pyf[p] = inside ? (float)y + 0.5f : __builtin_nanf("");
        alive += __popcll(__builtin_amdgcn_ballot_w64(inside));
        T[p] = 1.0f;
        cr[p] = cg[p] = cb[p] = 0.0f;
        last[p] = 0;
    }

    // per-tile lists: the Gaussian ids of a round are fetched one round ahead: the gather of the
    // splat records then waits for one memory round trip instead of two in a row
    int g_ahead[kFwdBatch / DSX_WAVE];
    // binned lists: the scan of the bin's list
    const uint32_t tile_bits = kBinned ? tile_bits_of(src, lists.shift) << 16 : 0u; // (in the key word's high half)
    const int32_t* const keys = ids + k; // the pairs' key words lie behind the ids (binned lists)
    int scan = start;  // next position of the bin's list to look at
    int seen = 0;      // entries of the tile's own list found so far
    if(!kBinned)
    {
#pragma unroll
        for(int h = 0; h < kFwdBatch / DSX_WAVE; ++h)
        {
            const int e = start + h * DSX_WAVE + lane;
            g_ahead[h] = e < end ? ids[e] : 0;
        }
    }
    int index_base = kBinned ? src.fine_base : start; // what final_idx records for the first entry of the round
    for(int b = start;; b += kFwdBatch)
    {
        if(alive == 0)
            break;
        int batch; // entries of this round
        __syncthreads(); // single wavefront: orders the LDS reads of the last round before these writes
        if(kBinned)
        {
            // Another 64 positions are taken only while all of them would still fit the round, and a
            // tile whose own entries have all been found looks no further.  The loads of four such
            // groups are issued together (the scan is bound by their latency, not by its dozen
            // instructions per group); groups that the round has no room for are read again by the next.
            int count = 0;
            while(count <= kFwdBatch - DSX_WAVE && scan < end && seen < src.count)
            {
                int id[kScanGroups], key[kScanGroups];
#pragma unroll
                for(int j = 0; j < kScanGroups; ++j)
                {
                    const int e = scan + j * DSX_WAVE + lane;
                    id[j] = e < end ? ids[e] : 0;
                    key[j] = e < end ? keys[e] : 0;
                }
#pragma unroll
                for(int j = 0; j < kScanGroups; ++j)
                {
                    if(count <= kFwdBatch - DSX_WAVE && scan < end && seen < src.count) // (uniform)
                    {
                        const bool member = scan + lane < end && (((uint32_t)key[j]) & tile_bits) == tile_bits;
                        const uint64_t m = __ballot(member);
                        if(member)
                            s_queue[count + bits_below_lane(m)] = id[j];
                        const int found = __popcll(m);
                        count += found;
                        seen += found;
                        scan += DSX_WAVE;
                    }
                }
            }
            if(count == 0)
                break;
            __syncthreads();
            batch = count;
#pragma unroll
            for(int h = 0; h < kFwdBatch / DSX_WAVE; ++h)
                g_ahead[h] = h * DSX_WAVE + lane < batch ? s_queue[h * DSX_WAVE + lane] : 0;
            __syncthreads(); // the queue has been read: its memory now takes the staged records
        }
        else
        {
            if(b >= end)
                break;
            batch = min(end - b, kFwdBatch);
        }
        uint64_t todo[kFwdBatch / DSX_WAVE]; // entries of this round that can touch the tile
#pragma unroll
        for(int h = 0; h < kFwdBatch / DSX_WAVE; ++h)
        {
            const int slot = h * DSX_WAVE + lane;
            bool useful = false;
            // (an id is taken for what it is only up to the last Gaussian: lists that a failed sort or a
            // caller's mix-up left in disorder then give a wrong image, not a fetch outside the records)
            const int g = (int)min((uint32_t)g_ahead[h], last_id);
            if(slot < batch)
            {
                const float4* rec = splats + 3 * (int64_t)g;
                const float4 q0 = rec[0], q1 = rec[1], q2 = rec[2];
                s_a[slot] = make_float4(q0.x, q0.y, q1.x * -0.5f, q1.y);
                s_b[slot] = make_float4(q1.z * 0.5f, q1.w, q2.x, q2.y);
                s_c[slot] = q2.z;
                useful = entry_reaches_tile(q0.x, q0.y, q1.x, q1.y, q1.z, q1.w, box_x0, box_y0, span_y);
            }
            todo[h] = __ballot(useful);
        }
        __syncthreads();
        if(!kBinned)
        {
            // the next round's ids: in flight while this round's entries are blended
#pragma unroll
            for(int h = 0; h < kFwdBatch / DSX_WAVE; ++h)
            {
                const int e = b + kFwdBatch + h * DSX_WAVE + lane;
                g_ahead[h] = e < end ? ids[e] : 0;
            }
        }
#pragma unroll
        for(int h = 0; h < kFwdBatch / DSX_WAVE; ++h)
        {
            uint64_t mask = todo[h];
            while(mask != 0)
            {
                if(alive == 0)
                    break;
                const int bit = __builtin_ctzll(mask);
                const int i = h * DSX_WAVE + bit;
                mask &= mask - 1;
                const float4 A = s_a[i];
                const float4 B = s_b[i];
                const float C = s_c[i];
                // what final_idx records for this entry: its position in the sorted key array (binned
                // lists: the tile's range start plus the entry's rank among the tile's own entries)
                const int entry_index = index_base + i;
                const ExponentX ex = exponent_x(A.z, A.w, pxf - A.x);
#pragma unroll
                for(int p = 0; p < kFwdPix; ++p)
                {
                    const float power = exponent_xy(ex, B.x, pyf[p] - A.y);
                    // (a NaN opacity gives alpha = 0.999 here as in the reference: fminf drops the NaN)
                    const float alpha = fminf(0.999f, B.y * fast_exp(power));
                    // the three decisions as wavefront masks (each is its compare's own result register),
                    // combined on the scalar unit and handed back to the lanes as conditions
                    // (1 - alpha) T in one rounding
                    const float Tn = __builtin_fmaf(-alpha, T[p], T[p]);
                    const uint64_t m_pass = __builtin_amdgcn_ballot_w64(power < 0.0f) &
                                            __builtin_amdgcn_ballot_w64(alpha >= kAlphaThreshold);
                    const uint64_t m_low = __builtin_amdgcn_ballot_w64(Tn < 0.0001f);
                    const uint64_t m_stop = m_pass & m_low;
                    const bool stop = __builtin_amdgcn_inverse_ballot_w64(m_stop);
                    const bool apply = __builtin_amdgcn_inverse_ballot_w64(m_pass & ~m_low);
                    const float vis = apply ? alpha * T[p] : 0.0f;
                    cr[p] += vis * B.z;
                    cg[p] += vis * B.w;
                    cb[p] += vis * C;
                    T[p] = apply ? Tn : T[p];
                    last[p] = apply ? entry_index : last[p];
                    pyf[p] = stop ? __builtin_nanf("") : pyf[p];
                    alive -= __popcll(m_stop);
                }
            }
        }
        index_base += batch;
    }

    // A sort pass that gave up waiting on its predecessor (bounded wait, never seen to happen)
    // leaves its flag set and the tile lists wrong: make that loud instead of plausible.
    if(!layout_ok || (sort_flag_a && *sort_flag_a) || (sort_flag_b && *sort_flag_b))
    {
#pragma unroll
        for(int p = 0; p < kFwdPix; ++p)
            cr[p] = cg[p] = cb[p] = __builtin_nanf("");
    }
#pragma unroll
    for(int p = 0; p < kFwdPix; ++p)
    {
        const int y = y0 + 4 * p;
        if(x < W && y < H)
        {
            const int64_t pix = (int64_t)y * W + x;
            image[3 * pix] = cr[p];
            image[3 * pix + 1] = cg[p];
            image[3 * pix + 2] = cb[p];
            final_T[pix] = T[p];
            final_idx[pix] = last[p];
        }
    }
    if(kBinned && layout_ok)
    {
        // for the backward: where this wavefront's scan of the bin's list stopped and how many of the
        // tile's entries it had met by then (everything that any of its pixels blended lies below).
        // The four-pixel form speaks for the whole tile and marks the other three bands as empty.
        int32_t* w = lists.walk + (int64_t)tile * 8;
        const int stopped = min(scan, end);
        if(kFwdPix == 4)
        {
            if(lane < 8)
                w[lane] = lane == 0 ? stopped : (lane == 1 ? seen : (lane & 1 ? 0 : -1));
        }
        else if(lane < 2)
            w[2 * band + lane] = lane == 0 ? stopped : seen;
    }
    // A side job for the memory system, which this kernel leaves idle: every wavefront prepares
    // its share of the backward's gradient accumulator, twelve floats per Gaussian: the nine sums
    // zeroed and, in the three spare places, the conic, which the per-Gaussian backward then has
    // at hand with the sums instead of fetching the splat records for it.  At the end of the
    // kernel, where nothing waits for the stores and the wavefronts arrive spread over time (at
    // the start they would all come at once and hold up the first loads: 0.147 against 0.140 ms).
    if(prep_count > 0)
    {
        static_assert(DSX_GRAD_FLOATS == 12, "three float4 per Gaussian");
        const int64_t share = (prep_count + gridDim.x - 1) / gridDim.x;
        const int64_t g0 = (int64_t)blockIdx.x * share;
        const int64_t g1 = min(g0 + share, prep_count);
        const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
        for(int64_t g = g0 + lane; g < g1; g += DSX_WAVE)
        {
            const float4 q1 = splats[3 * g + 1]; // conic a, b, c, opacity
            prep[3 * g] = zero;
            prep[3 * g + 1] = zero;
            prep[3 * g + 2] = make_float4(0.f, q1.x, q1.y, q1.z);
            if(prep_marks)
                prep_marks[g] = 0; // "no term added yet"
        }
    }
}

// The BinLists view of a `ranges` buffer in ranges_layout(lg) (lists per bin: lg.shift > 0)
static BinLists bin_lists(const ListGrid& lg, int32_t* ranges)
{
    BinLists L = {};
    if(lg.shift)
    {
        const RangesLayout rl = ranges_layout(lg);
        L.fine = ranges + rl.fine;
        L.last_tile = ranges + rl.last_tile;
        L.bins = ranges + rl.bins;
        L.walk = ranges + rl.walk;
        L.shift = lg.shift;
        L.nbx = lg.nbx;
        L.nty = lg.nty;
    }
    return L;
}

// ranges: the `ranges` buffer in ranges_layout(list_grid(cam)) (the kernel also writes its `walk` part
// when the lists are per bin).  check_header: the buffer has its header word, which must name the
// bin size of this call (always so for binned lists; per-tile lists may come as the tiles + 1 words
// of launch_tile_ranges, which have none).  n, k: Gaussians and entries of sorted_ids; ids and list
// positions beyond them are not followed.
int launch_blend_fwd(const dsx_camera& cam, int64_t n, int64_t k, int32_t* ranges, const int32_t* sorted_ids,
                     const float* splats, float* image, float* final_T, int32_t* final_idx, hipStream_t stream,
                     bool check_header, const uint32_t* sort_flag_a, const uint32_t* sort_flag_b,
                     float* prepare_grads, bool prepare_marks)
{
    const ListGrid lg = list_grid(cam);
    const int ntx = lg.ntx, nty = lg.nty;
    if(ntx * nty == 0)
        return prepare_grads ? DSX_ERR_BAD_ARG : DSX_OK; // (no image, no kernel, nothing prepared)
    if(prepare_grads && (((uintptr_t)prepare_grads & 15) != 0 || splats == nullptr))
        return DSX_ERR_BAD_ARG;
    if(n < 0 || k < 0 || k > 0x7fffffffll || (k > 0 && (sorted_ids == nullptr || splats == nullptr || n == 0)))
        return DSX_ERR_BAD_ARG;
    float4* prep = reinterpret_cast<float4*>(prepare_grads);
    const int64_t prep_count = prepare_grads ? n : 0;
    uint8_t* prep_marks = prepare_grads && prepare_marks ? grad_marks(prepare_grads, n) : nullptr;
    const BinLists L = bin_lists(lg, ranges);
    const int32_t* header = (lg.shift || check_header) ? ranges + ranges_layout(lg).header : nullptr;
    // the largest id that the kernel takes from the lists
    const uint32_t last_id = n > 0 ? (uint32_t)(n - 1) : 0u;
    {
        DSX_TIMED("blend_fwd_kernel", stream);
        const bool four = blend_pixels_per_lane(ntx * nty, kFwdFourPixelsFrom) == 4;
        const dim3 grid(four ? ntx * nty : 4 * ntx * nty);
        const float4* sp = reinterpret_cast<const float4*>(splats);
#define DSX_LAUNCH_FWD(PIX, BINNED)                                                                              \
    hipLaunchKernelGGL((blend_fwd_kernel<PIX, BINNED>), grid, dim3(DSX_WAVE), 0, stream, ranges, sorted_ids, sp,   \
                       image, final_T, final_idx, cam.image_width, cam.image_height, ntx, last_id, (int)k, header,  \
                       lg.shift, sort_flag_a, sort_flag_b, prep, prep_count, prep_marks, L)
        if(four && lg.shift)
            DSX_LAUNCH_FWD(4, true);
        else if(four)
            DSX_LAUNCH_FWD(4, false);
        else if(lg.shift)
            DSX_LAUNCH_FWD(1, true);
        else
            DSX_LAUNCH_FWD(1, false);
#undef DSX_LAUNCH_FWD
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

typedef unsigned int dsx_u32x2 __attribute__((ext_vector_type(2)));

template <int kCtrl>
__device__ __forceinline__ float dpp_move(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xf, 0xf, false));
}

// Sums eight per-lane values over the wavefront as a reduce-scatter.  The first two steps use the
// lane-swap instructions, which halve two registers into one at a time: across the halves of
// the wavefront (8 -> 4 registers), across neighbouring rows of 16 (4 -> 2); the third step
// trades between neighbouring lanes (2 -> 1), and three adds over the lanes that differ in bits
// 1, 2 and 3 finish the rows.  18 instructions where a select-and-add scheme over all three
// steps took 32.  Every lane ends up with a total: the one of
// v[4*(lane&1) + 2*((lane>>4)&1) + (lane>>5)].
__device__ __forceinline__ float pair_sum_halves(float a, float b)
{
    // lanes 0..31 get a summed over the two halves, lanes 32..63 get b
    const dsx_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r.x) + __uint_as_float(r.y);
}

__device__ __forceinline__ float pair_sum_rows(float a, float b)
{
    // even rows get a summed over each pair of neighbouring rows, odd rows get b
    const dsx_u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r.x) + __uint_as_float(r.y);
}

__device__ __forceinline__ float wave_sum8_scatter(const float (&v)[8], int lane)
{
    const float s0 = pair_sum_halves(v[0], v[1]);
    const float s1 = pair_sum_halves(v[2], v[3]);
    const float s2 = pair_sum_halves(v[4], v[5]);
    const float s3 = pair_sum_halves(v[6], v[7]);
    const float t0 = pair_sum_rows(s0, s1); // v[2 * row parity + half]
    const float t1 = pair_sum_rows(s2, s3); // v[4 + 2 * row parity + half]
    const bool odd = lane & 1;
    const float keep = odd ? t1 : t0;
    const float send = odd ? t0 : t1;
    float o = keep + dpp_move<0xB1>(send); // quad_perm [1,0,3,2]: the neighbour's share
    o = dpp_add<0x4E, 0xf>(o);             // quad_perm [2,3,0,1]: lanes that differ in bit 1
    o = dpp_add<0x124, 0xf>(o);            // row_ror:4 and
    o = dpp_add<0x128, 0xf>(o);            // row_ror:8: lanes that differ in bits 2 and 3
    return o;
}

constexpr int kBwdBatch = 128; // sorted entries staged in LDS per round (two per lane)

// One wavefront per 16x16 tile, four pixels per lane (same pixel ownership as the forward).
// The per-Gaussian gradients are first summed over a lane's four pixels, then over the
// wavefront with DPP adds, and lane 63 issues ONE set of hardware float atomics per
// (tile, entry).  Compared with four wavefronts of one pixel per lane this does one
// cross-lane reduction per entry instead of four and needs no LDS accumulators or barriers.
// (kBwdPix = 1: four wavefronts per tile with one band of four rows each, as in the forward)
// kBinned: the entries come out of the list of the tile's bin, filtered into a queue as in the forward
// but downwards; the forward left, per tile and band, the bin-list position where its scan stopped and
// the number of the tile's entries it had met by then, from which every entry met on the way down
// gets its index in the sorted key array (final_idx is compared with those).
template <int kBwdPix, bool kBinned>
__global__ __launch_bounds__(DSX_WAVE) void blend_bwd_kernel(
    const int32_t* __restrict__ ranges, const int32_t* __restrict__ ids, const float4* __restrict__ splats,
    const float* __restrict__ final_T, const int32_t* __restrict__ final_idx, const float* __restrict__ v_image,
    const float* __restrict__ bg, float* grads, uint8_t* marks, int W, int H, int ntx, uint32_t last_id, int k,
    const int32_t* __restrict__ header, int header_shift, const BinLists lists, const ZeroJobs zeros)
{
    __shared__ float4 s_a[kBwdBatch]; // pixel x, pixel y, conic -a/2, conic b
    __shared__ float4 s_b[kBwdBatch]; // conic c/2, opacity, red, green
    __shared__ float s_c[kBwdBatch];  // blue
    __shared__ int s_id[kBwdBatch];
    // the queue of the tile's own entries (binned lists) lives in s_a between two rounds, as in the forward
    int* const s_queue = reinterpret_cast<int*>(s_a);

    const int lane = threadIdx.x;
    const int tile = kBwdPix == 4 ? blockIdx.x : blockIdx.x >> 2;
    const int band = kBwdPix == 4 ? 0 : blockIdx.x & 3;
    const int tx = tile % ntx;
    const int ty = tile / ntx;
    const int x = tx * kTile + (lane & 15);
    const int y0 = ty * kTile + 4 * band + (lane >> 4);
    const float pxf = (float)x + 0.5f;
    // first pixel centre and last row of the pixels this wavefront owns
    const float box_x0 = (float)(tx * kTile) + 0.5f, box_y0 = (float)(ty * kTile + 4 * band) + 0.5f;
    const float span_y = kBwdPix == 4 ? 15.0f : 3.0f;
    const float bg0 = bg[0], bg1 = bg[1], bg2 = bg[2];

    // bterm = -T_final * (bg . v_out) - sum over the entries behind of (rgb . v_out) * alpha * T:
    // the three per-channel colour buffers of cpp/gsplat/backward.cu:156-168 only ever appear
    // dotted with v_out, so one scalar carries them
    float pyf[kBwdPix], T[kBwdPix], vo0[kBwdPix], vo1[kBwdPix], vo2[kBwdPix], bterm[kBwdPix];
    int bin_final[kBwdPix];
    int m = -1;
#pragma unroll
    for(int p = 0; p < kBwdPix; ++p)
    {
        const int y = y0 + 4 * p;
        const bool inside = x < W && y < H;
        const int64_t pix = inside ? (int64_t)y * W + x : 0;
        pyf[p] = (float)y + 0.5f;
        const float Tf = inside ? final_T[pix] : 0.0f;
        T[p] = Tf;
        bin_final[p] = inside ? final_idx[pix] : -1;
        vo0[p] = inside ? v_image[3 * pix] : 0.f;
        vo1[p] = inside ? v_image[3 * pix + 1] : 0.f;
        vo2[p] = inside ? v_image[3 * pix + 2] : 0.f;
        bterm[p] = -Tf * (bg0 * vo0[p] + bg1 * vo1[p] + bg2 * vo2[p]);
        m = max(m, bin_final[p]);
    }

    // last entry (as an index in the sorted key array) that any pixel of this wavefront blended
#pragma unroll
    for(int o = 32; o > 0; o >>= 1)
        m = max(m, __shfl_xor(m, o, DSX_WAVE));

    // lists that were built for another bin size than this launch assumes are not read (see the forward)
    const bool layout_ok = header == nullptr || *header == header_shift;
    int start = 0, hi = -1;
    TileSource src = {};
    // binned lists: the scan of the bin's list, downwards from where the forward's scan stopped
    uint32_t my_bits = 0u; // the two bits of this wavefront's tile in a pair's key word (high half)
    int pos = -1;       // next position of the bin's list to look at
    int rank_next = -1; // rank, in the tile's own list, of the next of its entries to be found
    int idx_next = 0;   // index (in the sorted key array) of the next entry that is handed to the blend
    if(kBinned && layout_ok)
    {
        // The forward's scan of the bin's list stopped at position w[0] after meeting w[1] of the
        // tile's entries (the larger of the four bands' figures: both grow together); everything
        // that was blended lies below, and the entries are taken from there downwards.  An entry's
        // index is the tile's range start plus its rank; those above the last blended one (m) are
        // not even queued, so the entries that are handed on have consecutive indices.
        src = tile_source(lists, tile, ntx);
        my_bits = tile_bits_of(src, lists.shift) << 16;
        start = max(src.start, 0);
        const int32_t* w = lists.walk + (int64_t)tile * 8;
        const int stopped = max(max(w[0], w[2]), max(w[4], w[6]));
        const int seen = max(max(w[1], w[3]), max(w[5], w[7]));
        // (positions outside sorted_ids are not followed, as in the forward)
        pos = min(stopped, min(src.end, k)) - 1;
        rank_next = min(seen, src.count) - 1;
        idx_next = min(m, src.fine_base + rank_next);
        if(src.count <= 0 || idx_next < src.fine_base) // nothing of this tile was blended
            pos = start - 1;
    }
    else if(layout_ok)
    {
        start = max(ranges[tile], 0);
        const int end = min(ranges[tile + 1], k);
        hi = min(end - 1, m);
    }

    int g_ahead[kBwdBatch / DSX_WAVE];
    const int32_t* const keys = ids + k; // the pairs' key words lie behind the ids (binned lists)
    if(!kBinned)
    {
        // (ids one round ahead, as in the forward)
#pragma unroll
        for(int h = 0; h < kBwdBatch / DSX_WAVE; ++h)
        {
            const int e = hi - (h * DSX_WAVE + lane);
            g_ahead[h] = e >= start ? ids[e] : 0;
        }
    }
    for(int top = hi;; top -= kBwdBatch)
    {
        int batch;     // entries of this round
        int idx_first; // index (in the sorted key array) of the round's first entry; the others follow downwards
        __syncthreads(); // single wavefront: orders the LDS reads of the last round before these writes
        if(kBinned)
        {
            // (four groups of 64 positions in flight at a time, as in the forward)
            int count = 0;
            while(count <= kBwdBatch - DSX_WAVE && pos >= start && rank_next >= 0)
            {
                int id[kScanGroups], key[kScanGroups];
#pragma unroll
                for(int j = 0; j < kScanGroups; ++j)
                {
                    const int e = pos - j * DSX_WAVE - lane;
                    id[j] = e >= start ? ids[e] : 0;
                    key[j] = e >= start ? keys[e] : 0;
                }
#pragma unroll
                for(int j = 0; j < kScanGroups; ++j)
                {
                    if(count <= kBwdBatch - DSX_WAVE && pos >= start && rank_next >= 0) // (uniform)
                    {
                        const bool member = pos - lane >= start && (((uint32_t)key[j]) & my_bits) == my_bits;
                        const uint64_t mm = __ballot(member);
                        // lower lanes hold higher positions: this entry's rank is the next one less the members before it
                        const int rank = rank_next - bits_below_lane(mm);
                        const bool keep = member && src.fine_base + rank <= m;
                        const uint64_t mk = __ballot(keep);
                        if(keep)
                            s_queue[count + bits_below_lane(mk)] = id[j];
                        count += __popcll(mk);
                        rank_next -= __popcll(mm);
                        pos -= DSX_WAVE;
                    }
                }
            }
            if(count == 0)
                break;
            __syncthreads();
            batch = count;
#pragma unroll
            for(int h = 0; h < kBwdBatch / DSX_WAVE; ++h)
                g_ahead[h] = h * DSX_WAVE + lane < batch ? s_queue[h * DSX_WAVE + lane] : 0;
            __syncthreads(); // the queue has been read: its memory now takes the staged records
            idx_first = idx_next;
            idx_next -= batch;
        }
        else
        {
            if(top < start)
                break;
            batch = min(top - start + 1, kBwdBatch);
            idx_first = top;
        }
        uint64_t todo[kBwdBatch / DSX_WAVE]; // entries of this round that can touch the tile
#pragma unroll
        for(int h = 0; h < kBwdBatch / DSX_WAVE; ++h)
        {
            const int slot = h * DSX_WAVE + lane;
            bool useful = false;
            const int g = (int)min((uint32_t)g_ahead[h], last_id); // (as in the forward)
            if(slot < batch)
            {
                const float4* rec = splats + 3 * (int64_t)g;
                const float4 q0 = rec[0], q1 = rec[1], q2 = rec[2];
                s_a[slot] = make_float4(q0.x, q0.y, q1.x * -0.5f, q1.y);
                s_b[slot] = make_float4(q1.z * 0.5f, q1.w, q2.x, q2.y);
                s_c[slot] = q2.z;
                s_id[slot] = g;
                useful = entry_reaches_tile(q0.x, q0.y, q1.x, q1.y, q1.z, q1.w, box_x0, box_y0, span_y);
            }
            todo[h] = __ballot(useful);
        }
        __syncthreads();
        if(!kBinned)
        {
            // the next round's ids: in flight while this round's entries are blended
#pragma unroll
            for(int h = 0; h < kBwdBatch / DSX_WAVE; ++h)
            {
                const int e = top - kBwdBatch - (h * DSX_WAVE + lane);
                g_ahead[h] = e >= start ? ids[e] : 0;
            }
        }
#pragma unroll
        for(int h = 0; h < kBwdBatch / DSX_WAVE; ++h)
        for(uint64_t mask = todo[h]; mask != 0; mask &= mask - 1)
        {
            const int bit = __builtin_ctzll(mask);
            const int t = h * DSX_WAVE + bit;
            const int idx = idx_first - t; // the entry's index in the sorted key array (scalar unit)
            const float4 A = s_a[t];
            const float4 B = s_b[t];
            // the exponent exactly as the forward computed it (pixel - mean); sigma = -exponent
            const float dxf = pxf - A.x;
            const ExponentX ex = exponent_x(A.z, A.w, dxf);
            float alpha[kBwdPix], vis[kBwdPix], dy[kBwdPix]; // dy = pixel - mean here
            // which lanes' pixel p takes part: wavefront masks (each compare's own result register),
            // combined on the scalar unit
            uint64_t m_valid[kBwdPix];
            uint64_t m_any = 0;
#pragma unroll
            for(int p = 0; p < kBwdPix; ++p)
            {
                dy[p] = pyf[p] - A.y;
                const float power = exponent_xy(ex, B.x, dy[p]);
                vis[p] = fast_exp(power);
                alpha[p] = fminf(0.99f, B.y * vis[p]);
                m_valid[p] = __builtin_amdgcn_ballot_w64(idx <= bin_final[p]) &
                             __builtin_amdgcn_ballot_w64(!(power > 0.0f)) &
                             __builtin_amdgcn_ballot_w64(!(alpha[p] < kAlphaThreshold));
                m_any |= m_valid[p];
            }
            if(m_any == 0)
                continue;
            const float blue = s_c[t];
            float g[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}; // v_x, v_y, v_conic a b c, v_opacity, v_red, v_green
            float g_blue = 0.f;
            // dx is the same for the lane's four pixels, so the five geometric sums are built from
            // three moments over dy of vis * v_alpha (v_sigma without its factor -opacity): S0, S1 (times dy), S2 (times dy^2)
            float S0 = 0.f, S1 = 0.f, S2 = 0.f;
#pragma unroll
            for(int p = 0; p < kBwdPix; ++p)
            {
                if(__builtin_amdgcn_inverse_ballot_w64(m_valid[p]))
                {
                    const float ra = __builtin_amdgcn_rcpf(1.0f - alpha[p]);
                    T[p] *= ra;
                    const float fac = alpha[p] * T[p];
                    g[6] += fac * vo0[p];
                    g[7] += fac * vo1[p];
                    g_blue += fac * vo2[p];
                    const float rv = B.z * vo0[p] + B.w * vo1[p] + blue * vo2[p];
                    const float v_alpha = rv * T[p] + bterm[p] * ra;
                    bterm[p] -= rv * fac;
                    // v_sigma = -opacity * vis * v_alpha: the moments are taken of vis * v_alpha (which is
                    // v_opacity's own term) and the common factor -opacity is applied once per entry
                    const float va = vis[p] * v_alpha;
                    const float vady = va * dy[p];
                    S0 += va;
                    S1 += vady;
                    S2 += vady * dy[p];
                }
            }
            g[5] = S0; // v_opacity
            // the gradients are written with d = mean - pixel: dx = -dxf, and S1 changes sign
            const float dx = -dxf;
            S0 *= -B.y;
            S1 *= B.y;
            // (the staged coefficients are -a/2, b and c/2; A.z * dxf and A.w * dxf are the exponent's own
            // first products)
            {
#pragma clang fp contract(off)
                g[0] = __builtin_fmaf(A.w, S1, (A.z * dxf) * (S0 * 2.0f));    // v_sigma (a dx + b dy)
                g[1] = __builtin_fmaf(B.x, S1 * 2.0f, -((A.w * dxf) * S0)); // v_sigma (b dx + c dy)
            }
            g[2] = 0.5f * dx * dx * S0;
            g[3] = dx * S1;
            g[4] = -0.5f * B.y * S2;
            const float total = wave_sum8_scatter(g, lane);
            g_blue = wave_sum_to_lane63(g_blue);
            // ONE atomic instruction carries all nine sums, each lane its own address: the first
            // two lanes of every row hold the eight totals of the reduce-scatter (every lane holds
            // one), lane 63 the ninth
            if((lane & 14) == 0 || lane == 63)
            {
                const int64_t id = s_id[t];
                float* rec = grads + id * DSX_GRAD_FLOATS;
                const int slot = lane == 63 ? 8 : 4 * (lane & 1) + 2 * ((lane >> 4) & 1) + (lane >> 5);
                unsafeAtomicAdd(rec + slot, lane == 63 ? g_blue : total);
                if(marks)
                    marks[id] = 1; // (all nine lanes store the same byte: no branch of its own)
            }
        }
    }
    // A side job for the memory system, as in the forward: the zeros of the per-Gaussian backward's
    // outputs (that kernel writes only the Gaussians that received a term here), every wavefront a
    // share, at its end, where nothing waits for the stores (3 M Gaussians, 780 MB: the kernel takes
    // 0.275 ms instead of 0.250; a few stores in every round of the walk instead: no better).
    if(zeros.any)
        zero_share(zeros, blockIdx.x, gridDim.x, lane, DSX_WAVE);
}

// ranges, check_header, n, k: as for launch_blend_fwd (the kernel reads the `walk` part that the forward wrote)
int launch_blend_bwd(const dsx_camera& cam, int64_t n, int64_t k, const int32_t* ranges, const int32_t* sorted_ids,
                     const float* splats, const float* final_T, const int32_t* final_idx, const float* v_image,
                     float* grads, hipStream_t stream, bool check_header, bool grads_prepared, bool with_marks,
                     const ZeroJobs* zeros)
{
    if(k < 0 || k > 0x7fffffffll || (k > 0 && sorted_ids == nullptr))
        return DSX_ERR_BAD_ARG;
    // (the marks lie right behind the records, padded to whole words: one fill covers both)
    if(!grads_prepared)
        if(int rc = launch_fill_u32(reinterpret_cast<uint32_t*>(grads),
                                    with_marks ? (int64_t)(grads_bytes(n) / 4) : n * DSX_GRAD_FLOATS, 0u, stream))
            return rc;
    const ListGrid lg = list_grid(cam);
    const int ntx = lg.ntx, nty = lg.nty;
    if(ntx * nty == 0 || n == 0)
        return zeros ? launch_zero_outputs(*zeros, stream) : DSX_OK; // (no tile, no wavefront to store them)
    ZeroJobs Z = {};
    if(zeros)
        Z = *zeros;
    const BinLists L = bin_lists(lg, const_cast<int32_t*>(ranges));
    const int32_t* header = (lg.shift || check_header) ? ranges + ranges_layout(lg).header : nullptr;
    const uint32_t last_id = (uint32_t)(n - 1);
    {
        DSX_TIMED("blend_bwd_kernel", stream);
        const bool four = blend_pixels_per_lane(ntx * nty, kBwdFourPixelsFrom) == 4;
        const dim3 grid(four ? ntx * nty : 4 * ntx * nty);
        const float4* sp = reinterpret_cast<const float4*>(splats);
#define DSX_LAUNCH_BWD(PIX, BINNED)                                                                              \
    hipLaunchKernelGGL((blend_bwd_kernel<PIX, BINNED>), grid, dim3(DSX_WAVE), 0, stream, ranges, sorted_ids, sp,   \
                       final_T, final_idx, v_image, cam.bg, grads, with_marks ? grad_marks(grads, n) : nullptr,       \
                       cam.image_width, cam.image_height, ntx, last_id, (int)k, header, lg.shift, L, Z)
        if(four && lg.shift)
            DSX_LAUNCH_BWD(4, true);
        else if(four)
            DSX_LAUNCH_BWD(4, false);
        else if(lg.shift)
            DSX_LAUNCH_BWD(1, true);
        else
            DSX_LAUNCH_BWD(1, false);
#undef DSX_LAUNCH_BWD
    }
    DSX_LAUNCH_CHECK();
    return DSX_OK;
}

} // namespace dsx
