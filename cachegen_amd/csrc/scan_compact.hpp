// Part of the CacheGen KV codec library for MI355X (gfx950); included by cachegen_hip.hip, which
// is the one translation unit.  Running sums of stream lengths and compaction of the encoder scratch into the payload.
//
// Paths in the comments are relative to LMCache/ in the reference tree:
//   enc_new.cu = third_party/torchac_cuda/torchac_kernel_enc_new.cu
//   dec_new.cu = third_party/torchac_cuda/torchac_kernel_dec_new.cu
//   cal_cdf.cu = third_party/torchac_cuda/cal_cdf.cu
//   encoder.py = lmcache/storage_backend/serde/cachegen_encoder.py
//   decoder.py = lmcache/storage_backend/serde/cachegen_decoder.py
#pragma once

namespace {

// ------------------------------------------------------------------------------------
// Exclusive running sum of the stream lengths (replaces the cumsum of decoder.py:70 and
// the index arithmetic of encoder.py:214-221): per-block sums, a one-block scan of
// those, then a per-block scan with the block's base added.
// ------------------------------------------------------------------------------------
constexpr int kScanThreads = 256;
constexpr int kScanPerThread = 8;
constexpr int kScanTile = kScanThreads * kScanPerThread;

__device__ __forceinline__ int64_t block_exclusive_scan(int64_t v, int64_t *lds, int64_t &total)
{
    const int tid = threadIdx.x;
    lds[tid] = v;
    __syncthreads();
    for (int o = 1; o < kScanThreads; o <<= 1) {
        const int64_t add = tid >= o ? lds[tid - o] : 0;
        __syncthreads();
        lds[tid] += add;
        __syncthreads();
    }
    total = lds[kScanThreads - 1];
    const int64_t incl = lds[tid];
    __syncthreads();
    return incl - v;
}

// The same for a block of 256 threads and 32-bit values, with wavefront shuffles and one
// exchange of the four wavefront totals through `lds` (at least 4 words).
__device__ __forceinline__ int32_t block_exclusive_scan_256(int32_t v, int32_t *lds, int32_t &total)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int32_t incl = v;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int32_t up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
    }
    if (lane == 63) lds[wave] = incl;
    __syncthreads();
    int32_t before = incl - v;
    total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const int32_t t = lds[w];
        if (w < wave) before += t;
        total += t;
    }
    __syncthreads();
    return before;
}

__global__ __launch_bounds__(kScanThreads) void scan_tile_sums_kernel(
    const int32_t *__restrict__ lengths, int64_t n, int32_t clamp, int64_t *__restrict__ sums)
{
    __shared__ int64_t lds[kScanThreads];
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanPerThread;
    int64_t s = 0;
    for (int j = 0; j < kScanPerThread; ++j)
        if (base + j < n) {
            int32_t v = lengths[base + j];
            v = v < 0 ? 0 : (v > clamp ? clamp : v);
            s += v;
        }
    int64_t total;
    block_exclusive_scan(s, lds, total);
    if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// In place, one block: every thread owns a contiguous run of the sums, adds it up, the block
// scans the 256 run totals, and every thread rewrites its run as exclusive running sums.
// Runs are handled 16 values at a time from registers so that the loads are in flight together.
__global__ __launch_bounds__(kScanThreads) void scan_sums_kernel(int64_t *sums, int64_t ntiles)
{
    __shared__ int64_t lds[kScanThreads];
    constexpr int kBatch = 16;
    const int64_t per = (ntiles + kScanThreads - 1) / kScanThreads;
    const int64_t lo = (int64_t)threadIdx.x * per;
    const int64_t hi = lo + per < ntiles ? lo + per : ntiles;
    int64_t mine = 0;
    for (int64_t i0 = lo; i0 < hi; i0 += kBatch) {
        int64_t v[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) v[j] = i0 + j < hi ? sums[i0 + j] : 0;
#pragma unroll
        for (int j = 0; j < kBatch; ++j) mine += v[j];
    }
    int64_t total;
    int64_t run = block_exclusive_scan(mine, lds, total);
    for (int64_t i0 = lo; i0 < hi; i0 += kBatch) {
        int64_t v[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) v[j] = i0 + j < hi ? sums[i0 + j] : 0;
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            if (i0 + j < hi) sums[i0 + j] = run;
            run += v[j];
        }
    }
}

__global__ __launch_bounds__(kScanThreads) void scan_apply_kernel(
    const int32_t *__restrict__ lengths, int64_t n, int32_t clamp,
    const int64_t *__restrict__ sums, int64_t *__restrict__ offsets)
{
    __shared__ int64_t lds[kScanThreads];
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)threadIdx.x * kScanPerThread;
    int32_t v[kScanPerThread];
    int64_t s = 0;
    for (int j = 0; j < kScanPerThread; ++j) {
        int32_t x = base + j < n ? lengths[base + j] : 0;
        x = x < 0 ? 0 : (x > clamp ? clamp : x);
        v[j] = x;
        s += x;
    }
    int64_t total;
    // sums == nullptr: the input is a single tile and this kernel is the whole scan
    int64_t run = (sums ? sums[blockIdx.x] : 0) + block_exclusive_scan(s, lds, total);
    for (int j = 0; j < kScanPerThread; ++j) {
        if (base + j < n) offsets[base + j] = run;
        run += v[j];
        if (base + j == n - 1) offsets[n] = run;
    }
}

// The whole running sum in one launch of one block, for up to kScanSmallMax values (the byte
// counts of the encoder's tiles): every thread owns up to 16 consecutive values, the block scans
// the 1024 thread totals with wavefront shuffles, and every thread writes its run.
constexpr int kScanSmallThreads = 1024;
constexpr int kScanSmallPer = 16;
constexpr int kScanSmallMax = kScanSmallThreads * kScanSmallPer;

__global__ __launch_bounds__(kScanSmallThreads) void scan_small_kernel(
    const int32_t *__restrict__ lengths, int32_t n, int32_t clamp, int64_t *__restrict__ offsets)
{
    __shared__ int64_t wave_totals[kScanSmallThreads / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int per = (n + kScanSmallThreads - 1) / kScanSmallThreads;      // <= kScanSmallPer
    const int lo = tid * per;
    int32_t v[kScanSmallPer];
    int64_t mine = 0;
#pragma unroll
    for (int j = 0; j < kScanSmallPer; ++j) {
        int32_t x = (j < per && lo + j < n) ? lengths[lo + j] : 0;
        x = x < 0 ? 0 : (x > clamp ? clamp : x);
        v[j] = x;
        mine += x;
    }
    // inclusive running sum over the wavefront, then over the 16 wavefront totals
    int64_t incl = mine;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int64_t up = __shfl_up(incl, o, 64);
        if (lane >= o) incl += up;
    }
    if (lane == 63) wave_totals[wave] = incl;
    __syncthreads();
    int64_t before = 0;
    for (int w = 0; w < wave; ++w) before += wave_totals[w];
    int64_t run = before + incl - mine;
#pragma unroll
    for (int j = 0; j < kScanSmallPer; ++j) {
        if (j < per && lo + j < n) {
            offsets[lo + j] = run;
            run += v[j];
            if (lo + j == n - 1) offsets[n] = run;
        }
    }
}

// ------------------------------------------------------------------------------------
// collect_bytes (encoder.py:209-222).  A block owns 256 consecutive streams, i.e. one
// contiguous range of the payload, and assembles it in LDS, 16 KiB at a time: every thread
// copies its own stream from its slot to the stream's place in the range (aligned words
// through a funnel shift, single bytes at the two ends), then the block writes the tile out
// as aligned 32-bit words.  Only the first and last word of a block's range are written
// byte by byte, so neighbouring blocks never write the same byte.  All positions are
// 32-bit offsets from the range's start.
// ------------------------------------------------------------------------------------
constexpr int kCompactStreams = 256;
constexpr int kCompactTile = 16384;

// SCAN: the offsets are not known yet; `offsets` is written here from the streams' lengths and
// the exclusive running sum of the tiles' byte counts, instead of being read.  That sum comes
// from tile_base (a scan launch made it), or, group_sums != null, is added up here: the sums of
// the groups of kTileGroup tiles before this block's group (at most kMaxTileGroups, left by the
// coder) and the counts of the tiles before this one in its group.
template <bool SCAN>
__global__ __launch_bounds__(256) void compact_streams_kernel(
    const uint8_t *__restrict__ slots, int32_t cap, int64_t *__restrict__ offsets,
    const int32_t *__restrict__ lengths, const int64_t *__restrict__ tile_base,
    int64_t nstreams, uint8_t *__restrict__ payload, int64_t payload_cap, int32_t skew, int32_t *status,
    const int32_t *__restrict__ group_sums = nullptr, const int32_t *__restrict__ tile_sums = nullptr)
{
    __shared__ int32_t rel[kCompactStreams + 1];       // stream offsets relative to the block's first byte
    __shared__ __align__(16) uint32_t buf[kCompactTile / 4];
    const int tid = threadIdx.x;
    const int64_t sbase = (int64_t)blockIdx.x * kCompactStreams;
    const int count = (nstreams - sbase < kCompactStreams) ? (int)(nstreams - sbase) : kCompactStreams;
    int64_t o0;
    if (SCAN) {
        int32_t mine = 0;
        if (tid < count) {
            mine = lengths[sbase + tid];
            mine = mine < 0 ? 0 : (mine > cap ? cap : mine);
        }
        int32_t total32;
        if (group_sums) {
            const int g = (int)(blockIdx.x / kTileGroup), r = (int)(blockIdx.x % kTileGroup);
            int32_t part = tid < g ? group_sums[tid] : 0;
            if (tid < r) part += tile_sums[(int64_t)g * kTileGroup + tid];
            int32_t sum;
            block_exclusive_scan_256(part, reinterpret_cast<int32_t *>(buf), sum);     // at most 16384 tiles of 64 KiB: fits
            o0 = sum;
        } else {
            o0 = tile_base[blockIdx.x];
        }
        const int32_t before = block_exclusive_scan_256(mine, reinterpret_cast<int32_t *>(buf), total32);    // buf is free until the copy
        const int64_t total64 = total32;                       // at most 256 streams of `cap` <= 256 bytes
        rel[tid] = before;
        if (tid == 0) rel[kCompactStreams] = total32;
        if (tid < count) offsets[sbase + tid] = o0 + before;
        if (sbase + count == nstreams && tid == 0) offsets[nstreams] = o0 + total64;
        __syncthreads();
        // threads past the last stream carry the total, like the padding of the other form
    } else {
        o0 = offsets[sbase];
        for (int i = tid; i <= kCompactStreams; i += 256)
            rel[i] = (int32_t)(offsets[sbase + (i < count ? i : count)] - o0);
        __syncthreads();
    }
    const int total = rel[count];
    if (o0 + total > payload_cap) {                    // never write past the caller's buffer
        if (tid == 0 && status) atomicOr(status, 2);
        return;
    }
    // x = position in the range + lead: aligned words of the payload are at multiples of 4
    const int lead = (int)((o0 + skew) & 3);
    uint8_t *const dst = payload + o0 - lead;
    const int end = lead + total;
    const int my0 = rel[tid] + lead, my1 = rel[tid + 1] + lead;     // rel[] is padded with the total
    // word k of this thread's stream (see encode_streams_kernel: tiles of kSlotTile streams)
    const uint32_t *const words = reinterpret_cast<const uint32_t *>(slots + sbase * (int64_t)cap) + tid;
    const int kmax = (my1 - my0 - 1) >> 2;             // last word that holds bytes of the stream
    uint8_t *const bytes = reinterpret_cast<uint8_t *>(buf);

    for (int t0 = 0; t0 < end; t0 += kCompactTile) {
        const int t1 = t0 + kCompactTile < end ? t0 + kCompactTile : end;
        const int xs = my0 > t0 ? my0 : t0;
        const int xe = my1 < t1 ? my1 : t1;
        // aligned words j of the range that hold bytes [xs, xe) of this stream, eight at a time:
        // word j is stream bytes 4j - my0 .. +3, i.e. two stream words through a funnel shift
        for (int j = xs >> 2; 4 * j < xe; j += 8) {
            const int q = 4 * j - my0;                 // may be negative for the stream's first word
            const int k = q >> 2;
            const uint32_t sh = (uint32_t)(q & 3) * 8u;
            const int left = ((xe + 3) >> 2) - j;      // words still to produce
            uint32_t wv[9];
#pragma unroll
            for (int u = 0; u < 9; ++u)
                wv[u] = (k + u >= 0 && k + u <= kmax && u <= left) ? words[(k + u) * kSlotTile] : 0u;
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (u >= left) break;
                const uint32_t v = __builtin_amdgcn_alignbit(wv[u + 1], wv[u], sh);
                const int x0 = 4 * (j + u);
                if (x0 >= xs && x0 + 4 <= xe) {
                    buf[(x0 - t0) >> 2] = v;
                } else {
                    for (int c = 0; c < 4; ++c)
                        if (x0 + c >= xs && x0 + c < xe) bytes[x0 + c - t0] = (uint8_t)(v >> (8 * c));
                }
            }
        }
        __syncthreads();
        for (int w = (t0 >> 2) + tid; 4 * w < t1; w += 256) {
            const int x0 = 4 * w;
            const uint32_t v = buf[w - (t0 >> 2)];
            if (x0 >= lead && x0 + 4 <= end) {
                *reinterpret_cast<uint32_t *>(dst + x0) = v;
            } else {
                for (int j = 0; j < 4; ++j)
                    if (x0 + j >= lead && x0 + j < end) dst[x0 + j] = (uint8_t)(v >> (8 * j));
            }
        }
        __syncthreads();
    }
}

__global__ void clear_status_kernel(int32_t *status) { *status = 0; }

}  // namespace
