// Part of the CacheGen KV codec library for MI355X (gfx950); included by cachegen_hip.hip, which
// is the one translation unit.  Per-(row, channel) tables: histogram, running sum, normalisation, staging in LDS; block-to-stream geometry.
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
// Tables (cal_cdf.cu:17-59): one lane per (chunk, row, channel) walks the chunk's tokens
// and counts into its own LDS column hist[bin][lane] (no lane touches another lane's
// counter); the running sum and the normalisation
//   cdf[i] = (uint16)((0xFFFF - max_bins) * cum[i] / cum[max_bins]) + i
// are done per lane in 16-bit wrap-around arithmetic like the reference's uint16
// counters, and the block writes its tables back transposed so stores coalesce.
// ------------------------------------------------------------------------------------

// Row strides of the per-block tables in LDS (entry e of lane c is element e * stride + c).  One
// more than a multiple of 64 banks' worth: the block reads and writes its tables transposed
// (consecutive lanes take consecutive entries of one channel), and with a stride of exactly
// BS elements every lane of a wavefront would hit the same bank.
template <int BS>
struct TableStride {
    static constexpr int k16 = BS + 2;      // 16-bit entries: BS/2 + 1 words
    static constexpr int k32 = BS + 1;      // 32-bit entries
};

// Column of lane c in a block's 16-bit tables: lanes c and c + BS/2 share a 32-bit word (low
// and high half).  The two belong to different wavefronts (for blocks of 128 lanes or more), so
// the lanes of one wavefront never add to the same word in one instruction when they count
// symbols, and their look-ups spread over 64 words instead of 32.
template <int BS>
__device__ __forceinline__ int table_column(int c)
{
    constexpr unsigned kHalf = BS / 2;
    static_assert((kHalf & (kHalf - 1)) == 0, "block size must be a power of two");
    return (int)((((unsigned)c & (kHalf - 1u)) << 1) | ((unsigned)c / kHalf));
}

// Walks i = start, start + step, ... over tables stored one after the other ([channel][lp]) and
// keeps (c, e) = (i / lp, i % lp) up to date with one divide at the start instead of one per step.
struct TableWalk {
    int c, e, dc, de;
    __device__ __forceinline__ TableWalk(int start, int step, int lp)
    {
        c = start / lp;
        e = start - c * lp;
        dc = step / lp;
        de = step - dc * lp;
    }
    __device__ __forceinline__ void next(int lp)
    {
        c += dc;
        e += de;
        if (e >= lp) {
            e -= lp;
            ++c;
        }
    }
};

// Running sum and normalisation of one lane's column col[i * stride], i in [0, lp).
template <int BS>
__device__ __forceinline__ void normalize_column(uint32_t *col, int lp, int max_bins)
{
    constexpr int kS = TableStride<BS>::k32;
    uint32_t running = 0;
    for (int i = 1; i < lp; ++i) {
        running = (running + col[i * kS]) & 0xFFFFu;
        col[i * kS] = running;
    }
    const uint32_t scale = 0xFFFFu - (uint32_t)max_bins;
    for (int i = 0; i < lp; ++i) {
        const uint32_t q = running ? (scale * col[i * kS] / running) & 0xFFFFu : 0u;
        col[i * kS] = (q + (uint32_t)i) & 0xFFFFu;
    }
}

// Write the block's tables tab[entry * stride + lane] to cdf[lane][entry], coalesced.
template <int BS>
__device__ __forceinline__ void write_tables(const uint32_t *tab, uint16_t *cdf, int lp, int64_t ch0, int64_t nc)
{
    const int64_t nvalid = (nc - ch0 < BS) ? (nc - ch0) : BS;
    const int total = (int)nvalid * lp;
    TableWalk w(threadIdx.x, BS, lp);
    for (int i = threadIdx.x; i < total; i += BS, w.next(lp)) {
        cdf[i] = (uint16_t)tab[w.e * TableStride<BS>::k32 + w.c];
    }
}

// Load the block's tables into LDS as tab[entry * stride + lane] (32-bit words).
template <int BS>
__device__ __forceinline__ void stage_tables(uint32_t *tab, const uint16_t *cdf, int lp, int64_t ch0, int64_t nc)
{
    const int64_t nvalid = (nc - ch0 < BS) ? (nc - ch0) : BS;
    const int total = (int)nvalid * lp;
    TableWalk w(threadIdx.x, BS, lp);
    for (int i = threadIdx.x; i < total; i += BS, w.next(lp)) {
        tab[w.e * TableStride<BS>::k32 + w.c] = cdf[i];
    }
}

// The stream kernels keep their tables in LDS as 16-bit entries tab[entry * stride + lane]
// (half the footprint, twice the resident waves).  The end of a table, 2^16, does not fit
// and is substituted where the last symbol's upper bound is read.
template <int BS>
__device__ __forceinline__ void stage_tables16(uint16_t *tab, const uint16_t *cdf, int lp, int64_t ch0, int64_t nc)
{
    const int64_t nvalid = (nc - ch0 < BS) ? (nc - ch0) : BS;
    const int total = (int)nvalid * lp;
    TableWalk w(threadIdx.x, BS, lp);
    // sixteen loads in flight at a time: one trip to memory per sixteen entries of a lane
    constexpr int kBatch = 16;
    for (int i0 = threadIdx.x; i0 < total; i0 += kBatch * BS) {
        uint16_t v[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) v[j] = i0 + j * BS < total ? cdf[i0 + j * BS] : (uint16_t)0;
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            if (i0 + j * BS < total) tab[w.e * TableStride<BS>::k16 + table_column<BS>(w.c)] = v[j];
            w.next(lp);
        }
    }
}

// Copy one lane's own table (lp consecutive 16-bit entries at `mine`) into its LDS column
// col[e * kS]: loads and LDS writes on immediate offsets, sixteen loads in flight; the lanes of a
// wavefront read neighbouring tables, so every cache line is fetched once.
template <int kS>
__device__ __forceinline__ void stage_column16_stride(uint16_t *col, const uint16_t *mine, int lp)
{
    constexpr int kBatch = 16;
    for (int e0 = 0; e0 < lp; e0 += kBatch) {
        uint16_t v[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) v[j] = e0 + j < lp ? mine[e0 + j] : (uint16_t)0;
#pragma unroll
        for (int j = 0; j < kBatch; ++j)
            if (e0 + j < lp) col[(e0 + j) * kS] = v[j];
    }
}

// Write one lane's own table, col[e * kS], e in [0, lp), to its lp consecutive 16-bit entries
// at `mine`, two entries per 32-bit store (a table that starts off a word boundary sends its first
// entry alone).  The lanes of a wavefront write to places lp entries apart; what this costs the
// memory pipeline is hidden behind the vector instructions of the other wavefronts, and a store
// takes no address arithmetic: the LDS reads and the stores use immediate offsets.
template <int kS>
__device__ __forceinline__ void write_column16_stride(const uint16_t *col, uint16_t *mine, int lp)
{
    const int first = (int)((reinterpret_cast<uintptr_t>(mine) >> 1) & 1u);
    if (first) mine[0] = col[0];
    const int rest = lp - first, npairs = rest >> 1;
    const uint16_t *src = col + first * kS;
    uint32_t *dst = reinterpret_cast<uint32_t *>(mine + first);
    constexpr int kBatch = 8;               // pairs in flight
    int i = 0;
    for (; i + kBatch <= npairs; i += kBatch) {
        uint32_t v[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) v[j] = (uint32_t)src[(2 * (i + j)) * kS] | ((uint32_t)src[(2 * (i + j) + 1) * kS] << 16);
#pragma unroll
        for (int j = 0; j < kBatch; ++j) dst[i + j] = v[j];
    }
    for (; i < npairs; ++i) dst[i] = (uint32_t)src[(2 * i) * kS] | ((uint32_t)src[(2 * i + 1) * kS] << 16);
    if (rest & 1) mine[lp - 1] = col[(lp - 1) * kS];
}

// Running sum and normalisation of one lane's 16-bit column of counts (col[e * kS]) when every one of
// `total` tokens was counted (1 <= total <= 65535, uniform over the block): the divide of
// cal_cdf.cu:11-14 becomes a shift or a float estimate corrected exactly.
template <int kS>
__device__ __forceinline__ void normalize_column16_stride(uint16_t *col, int lp, int max_bins, uint32_t total)
{
    const uint32_t scale = 0xFFFFu - (uint32_t)max_bins;
    uint32_t running = 0;
    if ((total & (total - 1)) == 0) {
        const int sh = 31 - __builtin_clz(total);
        for (int i = 0; i < lp; ++i) {
            running += col[i * kS];
            col[i * kS] = (uint16_t)(((scale * running) >> sh) + (uint32_t)i);
        }
    } else {
        const float inv = __fdiv_rn(1.0f, (float)total);
        for (int i = 0; i < lp; ++i) {
            running += col[i * kS];
            const uint32_t x = scale * running;                  // < 2^32, quotient < 2^16
            uint32_t q = (uint32_t)((float)x * inv);
            int32_t rem = (int32_t)(x - q * total);
            if (rem < 0) { q--; rem += (int32_t)total; }
            if (rem >= (int32_t)total) q++;
            col[i * kS] = (uint16_t)(q + (uint32_t)i);
        }
    }
}

// The same two for a block's tables with the row stride of TableStride<BS>.
template <int BS>
__device__ __forceinline__ void write_column16(const uint16_t *col, uint16_t *mine, int lp)
{
    write_column16_stride<TableStride<BS>::k16>(col, mine, lp);
}
template <int BS>
__device__ __forceinline__ void normalize_column16(uint16_t *col, int lp, int max_bins, uint32_t total)
{
    normalize_column16_stride<TableStride<BS>::k16>(col, lp, max_bins, total);
}

struct CdfArgs {
    const uint8_t *sym;     // byte symbols: sym[row*s0 + token*s1 + channel*s2]
    int64_t s0, s1, s2;
    const uint32_t *sym4;   // or packed symbols (see above)
    int64_t nsub;
    // packed symbols: rows of at most 15 symbols hold four bits a symbol, two channels to a word
    // (quantize_pack_kernel); the levels of the rows
    int32_t nibbles;
    const float *key_bins, *value_bins;
    int64_t L;
    uint16_t *cdf;          // [chunk][row][channel][lp]
    int64_t rows, nc;
    int32_t ctiles;
    int32_t max_bins;
    TokenGeom g;
};

template <int BS, bool PACKED>
__global__ __launch_bounds__(BS) void calculate_cdf_kernel(CdfArgs a)
{
    extern __shared__ uint32_t smem[];
    const int tid = threadIdx.x;
    const int lp = a.max_bins + 1;
    int64_t b = blockIdx.x;
    const int ctile = (int)(b % a.ctiles);
    b /= a.ctiles;
    const int64_t row = b % a.rows;
    const int64_t chunk = b / a.rows;
    const int64_t ch = (int64_t)ctile * BS + tid;
    // byte symbols: one 32-bit counter per (entry, lane); packed symbols (the fused path, whose
    // symbols all lie inside the table): 16-bit counters, two lanes to a word, as in the encoder
    constexpr int kS16 = TableStride<BS>::k16, kS32 = TableStride<BS>::k32;
    uint32_t *col = smem + tid;
    uint16_t *tab16 = reinterpret_cast<uint16_t *>(smem);
    const int tcol = table_column<BS>(tid);
    if (PACKED) {
        for (int i = 0; i < lp; ++i) tab16[i * kS16 + tcol] = 0;
        __syncthreads();                     // another lane shares this lane's words
    } else {
        for (int i = 0; i < lp; ++i) col[i * kS32] = 0;
    }

    const int64_t t0 = chunk * a.g.S;
    int64_t t1 = t0 + a.g.S;
    if (t1 > a.g.T) t1 = a.g.T;
    const uint32_t mb = (uint32_t)a.max_bins;
    if (ch < a.nc) {
        if (!PACKED) {
            const uint8_t *p = a.sym + row * a.s0 + ch * a.s2;
            int64_t t = t0;
            for (; t + 8 <= t1; t += 8) {
                uint32_t v[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = p[(t + j) * a.s1];
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (v[j] < mb) atomicAdd(col + (v[j] + 1) * kS32, 1u);      // no value returned: one LDS operation
            }
            for (; t < t1; ++t) {
                const uint32_t v = p[t * a.s1];
                if (v < mb) atomicAdd(col + (v + 1) * kS32, 1u);
            }
        } else {
            uint32_t *const pair = smem + (tcol >> 1);
            const uint32_t one = (tcol & 1) ? 0x10000u : 1u;
            const int64_t sub0 = chunk * a.g.nsc;
            bool narrow = false;                     // uniform over the block
            if (a.nibbles) {
                const int64_t kvi = row / a.L, l = row - kvi * a.L;
                narrow = narrow_alphabet(floorf((kvi ? a.value_bins : a.key_bins)[l] * 0.5f) - 1.0f, lp);
            }
            const int64_t column = narrow ? (ch >> 1) : ch;
            const uint32_t half_shift = narrow ? (uint32_t)(ch & 1) * 16u : 0u;
            const int nsubs = (int)((t1 - t0 + kSub - 1) / kSub);
            for (int sidx = 0; sidx < nsubs; ++sidx) {
                const int64_t left = (t1 - t0) - (int64_t)sidx * kSub;
                const int n = left < kSub ? (int)left : kSub;
                const uint32_t *wp = a.sym4 + ((row * a.nsub + sub0 + sidx) * kWordsPerSub) * a.nc + column;
                const int nwords = (n + 3) >> 2;
                constexpr int kBatch = 16;          // words in flight per lane
                for (int w0 = 0; w0 < nwords; w0 += kBatch) {
                    uint32_t v[kBatch];
#pragma unroll
                    for (int j = 0; j < kBatch; ++j) v[j] = (w0 + j < nwords) ? wp[(int64_t)(w0 + j) * a.nc] : 0u;
                    if (narrow) {
                        // the value 15 stands for a saturated byte: the table's last symbol
#pragma unroll
                        for (int j = 0; j < 4 * kBatch; ++j) {
                            uint32_t s = __builtin_amdgcn_ubfe(v[j >> 2] >> half_shift, (uint32_t)(4 * (j & 3)), 4u);
                            s = s == 15u ? mb - 1u : s;
                            if (w0 * 4 + j < n) atomicAdd(pair + (s + 1) * (kS16 / 2), one);
                        }
                    } else {
#pragma unroll
                        for (int j = 0; j < 4 * kBatch; ++j) {
                            uint32_t s = (v[j >> 2] >> (8 * (j & 3))) & 0xFFu;
                            s = s < mb - 1u ? s : mb - 1u;
                            if (w0 * 4 + j < n) atomicAdd(pair + (s + 1) * (kS16 / 2), one);
                        }
                    }
                }
            }
        }
        if (!PACKED) normalize_column<BS>(col, lp, a.max_bins);
    }
    const int64_t ch0 = (int64_t)ctile * BS;
    uint16_t *dst = a.cdf + ((chunk * a.rows + row) * a.nc + ch0) * lp;
    if (PACKED) {
        __syncthreads();                     // the other lane's atomics on the shared words are done
        if (ch < a.nc) {
            normalize_column16<BS>(tab16 + tcol, lp, a.max_bins, (uint32_t)(t1 - t0));
            write_column16<BS>(tab16 + tcol, dst + (int64_t)tid * lp, lp);
        }
    } else {
        __syncthreads();
        write_tables<BS>(smem, dst, lp, ch0, a.nc);
    }
}

// ------------------------------------------------------------------------------------
// Arithmetic coder.  Shared geometry of the encoder and decoder kernels: a block of BS
// lanes covers BS adjacent channels of one (sub-chunk, row).
// ------------------------------------------------------------------------------------
struct StreamGrid {
    int64_t rows, nc;
    int32_t ctiles;
    TokenGeom g;
};

struct StreamId {
    int64_t sub, row, chunk, t0, ch;
    int n;
    bool active;
};

// The grid is (channel tile, row, sub-chunk): a block reads its place from its index.
template <int BS>
__device__ __forceinline__ StreamId locate(const StreamGrid &sg)
{
    StreamId s;
    s.row = blockIdx.y;
    s.sub = blockIdx.z;
    sub_range(sg.g, s.sub, s.chunk, s.t0, s.n);
    s.ch = (int64_t)blockIdx.x * BS + threadIdx.x;
    s.active = s.ch < sg.nc;
    return s;
}

// The block's number in the order (sub-chunk, row, channel tile), in which tiles of the encoder's
// scratch and their byte counts are laid out.
__device__ __forceinline__ uint32_t linear_block()
{
    return (blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x;
}

}  // namespace
