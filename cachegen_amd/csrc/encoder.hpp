// Part of the CacheGen KV codec library for MI355X (gfx950); included by cachegen_hip.hip, which
// is the one translation unit.  Range encoder: word writer, coder state, encode_streams_kernel.
//
// Paths in the comments are relative to LMCache/ in the reference tree:
//   enc_new.cu = third_party/torchac_cuda/torchac_kernel_enc_new.cu
//   dec_new.cu = third_party/torchac_cuda/torchac_kernel_dec_new.cu
//   cal_cdf.cu = third_party/torchac_cuda/cal_cdf.cu
//   encoder.py = lmcache/storage_backend/serde/cachegen_encoder.py
//   decoder.py = lmcache/storage_backend/serde/cachegen_decoder.py
#pragma once

namespace {

// ---- encoder (enc_new.cu:21-97, 253-307) -------------------------------------------
// The reference's coder emits a bit for every E1/E2 step and counts E3 (underflow) steps as
// pending bits that follow the next emitted bit as its complements (enc_new.cu:86-97,
// 275-305).  That output is the binary expansion of the interval's lower end, written with
// carries: after a total of n renormalisation steps the bits emitted or pending are the
// lower end's first n bits, a pending run 0111..1 being a run of ones that a later carry may
// still turn into 1000..0, and the closing `pending + 2` bits (enc_new.cu:309-317) are the
// next two bits of the lower end plus a quarter of the window.  So the lower end is kept
// here as one long number: its last 32 bits (`low`, the coder's window; bit 31 can differ
// from the reference's, where an underflow step clears it, and nothing reads it) below 64
// bits that are waiting to be written (`out`).  A symbol adds its offset to the number and
// shifts it left by the step count n = clz(low ^ high) + (underflow steps); nothing is
// counted or spliced per symbol.  Words leave at fixed points, once per eight symbols (every
// lane of a wavefront runs the store code whenever one lane has a word ready); a carry out
// of the waiting bits is added to the last word, which is therefore held back one round
// (`cache`), and a word of all ones is only counted (`ones`) until the word after it shows
// whether the carry comes.  n <= 18 for any table whose symbols all have non-zero width,
// because the span stays above 2^30 between symbols.
constexpr int kSlotTile = 256;      // streams per tile of the encoder's scratch
// Tiles whose byte counts the coder's blocks also add up into one sum per group, so that the
// compaction finds a tile's place in the payload from at most kMaxTileGroups group sums and
// kTileGroup - 1 tile counts; calls with more groups run a scan launch over the tile counts.
constexpr int kTileGroup = 64;
constexpr int kMaxTileGroups = 256;

// TILE: the stream's words go to a tile of the scratch (word w of the tile's stream t at the
// tile's word w * kSlotTile + t) through a buffer descriptor that covers exactly the tile: a
// word or byte past the stream's capacity falls outside the descriptor and is dropped by the
// hardware, so nothing is compared or counted per word.
template <bool ALIGNED, bool TILE = false>
struct WordWriter {
    uint8_t *wptr;          // where the next word goes
    int wstride;            // bytes from one word of the stream to the next (4: contiguous)
    int cap;
    int nbytes;             // bytes written so far; -4 before the held-back word's first, empty turn
    __amdgpu_buffer_rsrc_t tile;    // TILE: the block's tile
    uint32_t voff, voff0;           // TILE: byte offset in the tile of the next word, and of the first

    __device__ __forceinline__ void init(uint8_t *dst, int stride, int capacity)
    {
        // the first word stored is the empty held-back word: it goes one word before the
        // stream (TILE: the offset wraps and the hardware drops the store)
        wptr = dst - stride;
        wstride = stride;
        cap = capacity;
        nbytes = -4;
        voff = voff0 = 0;
    }
    __device__ __forceinline__ void init_tile(__amdgpu_buffer_rsrc_t rsrc, uint32_t first)
    {
        tile = rsrc;
        voff0 = first;
        voff = first - kSlotTile * 4;
    }

    __device__ __forceinline__ void store_word(uint32_t word)
    {
        if (TILE) {
            __builtin_amdgcn_raw_buffer_store_b32((int)__builtin_bswap32(word), tile, (int)voff, 0, 0);
            voff += kSlotTile * 4;
            return;
        }
        if (nbytes >= 0) {
            if (__builtin_expect(nbytes + 4 <= cap, 1)) {
                if (ALIGNED) {
                    *reinterpret_cast<uint32_t *>(wptr) = __builtin_bswap32(word);
                } else {
                    wptr[0] = (uint8_t)(word >> 24);
                    wptr[1] = (uint8_t)(word >> 16);
                    wptr[2] = (uint8_t)(word >> 8);
                    wptr[3] = (uint8_t)word;
                }
            } else {
                // the last words of a stream that does not fit its slot: keep what fits
                for (int j = 0; j < 4; ++j)
                    if (nbytes + j < cap) wptr[j] = (uint8_t)(word >> (24 - 8 * j));
            }
        }
        wptr += wstride;
        nbytes += 4;
    }

    // the stream's last `nbits` bits (fewer than 32, left-aligned in `word`), byte by byte
    // (enc_new.cu:42-55); returns the stream length
    __device__ __forceinline__ int finish(uint32_t word, int nbits)
    {
        if (TILE) nbytes = (int)((voff - voff0) / kSlotTile);     // four bytes per word written
        for (int left = nbits, j = 0; left > 0; left -= 8, ++j) {
            if (TILE) __builtin_amdgcn_raw_buffer_store_b8((char)(word >> 24), tile, (int)(voff + j), 0, 0);
            else if (nbytes < cap) wptr[j] = (uint8_t)(word >> 24);
            nbytes++;
            word <<= 8;
        }
        return nbytes;
    }
};

// The coder state is the number described above plus the interval's width less one,
// `span_less_one`: the full range 2^32 (the initial state, and any later interval that is exactly
// a binary fraction) is 2^32 - 1 there, and floor(span * c / 2^16) is the high word of
// span_less_one * (c << 16) + (c << 16) for every span, one 64-bit multiply-add with nothing set
// apart for the full range.  Renormalising by n bits maps span to span << n for E1/E2 and E3
// steps alike.
template <int BS, bool ALIGNED, bool TILE = false>
struct RangeEncoder {
    lds_char *col;          // this lane's table column: entry e at byte e * 2 * TableStride<BS>::k16
    uint32_t smax;          // lp - 2: the largest symbol
    uint32_t span_less_one;
    // the number's last 96 bits: `tail` holds the window (its lower half, called low in the
    // comments) and above it the first 32 of the bits waiting to be written, `out_hi` the rest
    // of them: 63 - room bits wait, and above them there may be a carry (0 or 1) that belongs
    // to the held-back word
    uint64_t tail;
    uint32_t out_hi;
    // counted this way, the subtraction that books a shift borrows exactly when the bits (and
    // the place for a carry above them) do not fit, and that borrow is the test
    uint32_t room;
    uint32_t cache;         // the last complete word, not yet written: a carry may still reach it
    uint32_t ones;          // words of all ones that follow it
    uint32_t plain;         // 0xFFFFFFFF while `ones` is 0, else 0: a word below it is stored the short way
    // the coded symbol's two table entries, each shifted left by 16: only ever written by
    // loads into the upper half, so that the lower halves stay zero
    uint64_t bound_lo, bound_hi;
    WordWriter<ALIGNED, TILE> w;

    __device__ __forceinline__ void init(const uint16_t *column, int lp)
    {
        col = (lds_char *)column;
        bound_lo = 0;
        bound_hi = 0;
        smax = (uint32_t)(lp - 2);
        span_less_one = 0xFFFFFFFFu;
        tail = 0;
        out_hi = 0;
        room = 63;
        cache = 0;
        ones = 0;
        plain = 0xFFFFFFFFu;
    }

    // the held-back word, raised by the carry, and the words of all ones behind it (which the
    // carry turns into zeros); not on the common path
    __device__ __forceinline__ void release(uint32_t carry)
    {
        w.store_word(cache + carry);
        for (; ones; --ones) w.store_word(carry ? 0u : 0xFFFFFFFFu);
        plain = 0xFFFFFFFFu;
    }

    // takes the top 32 waiting bits (and the carry above them); needs at least 32 waiting
    __device__ __forceinline__ void flush_word()
    {
        const uint32_t sh = 31u - room;                 // waiting bits that stay
        const uint32_t out_lo = (uint32_t)(tail >> 32);
        const uint64_t top = (((uint64_t)out_hi << 32) | out_lo) >> sh;
        const uint32_t word = (uint32_t)top, carry = (uint32_t)(top >> 32);
        tail = ((uint64_t)__builtin_amdgcn_ubfe(out_lo, 0u, sh) << 32) | (uint32_t)tail;
        out_hi = 0;
        room += 32u;
        if (__builtin_expect(word < plain, 1)) {
            w.store_word(cache + carry);
            cache = word;
        } else {
            asm volatile("");
            if (carry) {
                release(1u);
                cache = word;
            } else if (word == 0xFFFFFFFFu) {
                ones++;
                plain = 0u;
            } else {
                release(0u);
                cache = word;
            }
        }
    }

    // The two steps below are written out instruction by instruction, on fixed registers
    // (tail in v[56:57], out_hi in v59, v58 as the lower half of the pair that shifts out_hi):
    // the 96-bit add is one carry chain and the 96-bit shift two 64-bit shifts and a move, which
    // the compiler does not find from C (it compares for the carry and shuffles the halves).

    // the number grows by `add` (a carry may run into the waiting bits)
    __device__ __forceinline__ void add_low(uint32_t add)
    {
        asm("v_add_co_u32 v56, vcc, v56, %2\n\t"
            "v_addc_co_u32 v57, vcc, 0, v57, vcc\n\t"
            "v_addc_co_u32 v59, vcc, 0, v59, vcc"
            : "+{v[56:57]}"(tail), "+{v59}"(out_hi)
            : "v"(add)
            : "vcc");
    }

    // the same, then the step count of the interval [low, low + width - 1]: n1 = clz(low ^ high)
    // E1/E2 steps and the E3 run below them, the leading zeros of (~low | high) once the first
    // differing bit is shifted out
    __device__ __forceinline__ int add_and_count(uint32_t add, uint32_t width)
    {
        int n;
        uint32_t t;
        // a carry out of the 64 low bits needs 32 waiting ones: left to a branch that is next to
        // never taken, instead of a third add in every symbol
        uint64_t carry;
        asm("v_add_co_u32 v56, vcc, v56, %4\n\t"
            "v_addc_co_u32 v57, %2, 0, v57, vcc\n\t"
            "v_add3_u32 %1, %5, v56, -1\n\t"
            "v_xor_b32 %0, %1, v56\n\t"
            "v_bitop3_b32 %1, %1, v56, %1 bitop3:0xf3\n\t"
            "v_ffbh_u32 %0, %0\n\t"
            "v_add_lshl_u32 %1, %1, %1, %0\n\t"
            "v_ffbh_u32 %1, %1\n\t"
            "v_add_u32 %0, %0, %1"
            : "=&v"(n), "=&v"(t), "=&s"(carry), "+{v[56:57]}"(tail)
            : "v"(add), "v"(width)
            : "vcc");
        if (__builtin_expect(carry != 0, 0))
            asm("v_addc_co_u32 v59, %0, 0, v59, %0" : "+s"(carry), "+{v59}"(out_hi));
        return n;
    }

    // the number moves left by n <= 31 bits.  ROOM: the caller knows that the bits fit
    template <bool ROOM = false>
    __device__ __forceinline__ void shift(int n)
    {
        uint32_t left;
        if (__builtin_expect(__builtin_usub_overflow(room, (uint32_t)n, &left), 0) && !ROOM) {
            asm volatile("");
            flush_word();                               // more than 32 bits were waiting
            left = room - (uint32_t)n;
        }
        room = left;
        asm("v_mov_b32 v58, v57\n\t"
            "v_lshlrev_b64 v[58:59], %2, v[58:59]\n\t"
            "v_lshlrev_b64 v[56:57], %2, v[56:57]"
            : "+{v[56:57]}"(tail), "+{v59}"(out_hi)
            : "v"(n)
            : "v58");
    }

    // SENTINEL: symbol smax may occur, whose upper bound is 2^16 and not the table's last
    // entry (enc_new.cu:270)
    // FIRST: the symbol directly follows a flush (the first of a group)
    // CLAMP: the symbol may lie outside the table (it is kept inside; symbols that are known to
    // be table symbols skip the compare)
    template <bool SENTINEL, bool FIRST, bool CLAMP = true>
    __device__ __forceinline__ void put_symbol(uint32_t s)
    {
        if (CLAMP) s = s < smax ? s : smax;             // keep table reads inside the table
        constexpr int kRow = 2 * TableStride<BS>::k16;
        // both entries into the upper halves of the lower registers of two pairs whose upper
        // registers stay 0: the pairs are the entries shifted left by 16, as 64-bit values
        asm volatile("ds_read_u16_d16_hi v52, %2\n\tds_read_u16_d16_hi v54, %2 offset:%3\n\ts_waitcnt lgkmcnt(0)"
                     : "+{v[52:53]}"(bound_lo), "+{v[54:55]}"(bound_hi)
                     : "v"(col + s * kRow), "n"(kRow));
        // T(c) = (span * c) >> 16 = high word of span * (c << 16) = high word of
        // span_less_one * (c << 16) + (c << 16): one 64-bit multiply-add, right for the full range
        // (span_less_one = 2^32 - 1) as for every other span, so no case is set apart
        uint64_t prod_lo, prod_hi;
        asm("v_mad_u64_u32 %0, vcc, %2, v52, v[52:53]\n\tv_mad_u64_u32 %1, vcc, %2, v54, v[54:55]"
            : "=&v"(prod_lo), "=&v"(prod_hi)
            : "v"(span_less_one), "{v[52:53]}"(bound_lo), "{v[54:55]}"(bound_hi)
            : "vcc");
        const uint32_t t_lo = (uint32_t)(prod_lo >> 32);
        // the upper bound of symbol smax is 2^16 and not the table's last entry: T(2^16) is the span
        const bool top = SENTINEL && s == smax;
        const uint32_t width = (top ? span_less_one + 1u : (uint32_t)(prod_hi >> 32)) - t_lo;
        const int n = add_and_count(t_lo, width);
        shift<FIRST>(n);
        span_less_one = (width << n) - 1u;
    }

    // one group of symbols is through: write a word if 32 bits are waiting
    __device__ __forceinline__ void end_group()
    {
        if (room <= 31u) flush_word();
    }

    __device__ __forceinline__ int finish()
    {
        // the closing bits (enc_new.cu:309-317): the two bits below `out` of the number plus a
        // quarter of the window
        add_low(0x40000000u);
        shift(2);
        end_group();
        const uint32_t nbits = 63u - room;              // fewer than 32 are left
        const uint32_t out_lo = (uint32_t)(tail >> 32);
        release(out_lo >> nbits);
        return w.finish(nbits ? out_lo << (32u - nbits) : 0u, (int)nbits);
    }
};

struct EncodeArgs {
    uint16_t *cdf;          // [chunk][row][channel][lp]; written when the histogram is fused
    int32_t lp;
    const uint8_t *sym;     // byte symbols: sym[row*s0 + token*s1 + channel*s2]
    int64_t s0, s1, s2;
    const uint32_t *sym4;   // or packed symbols
    int32_t nibbles;        // rows of at most 15 symbols are packed four bits a symbol (quantize_pack_kernel)
    const uint16_t *maxima; // the row maxima [2L, T] and their type, to know the rows that saturate (or null)
    int32_t max_dt;
    int64_t nsub;
    uint8_t *out;           // out[row*o0 + channel*o1 + byte], or the scratch tiles (SLOTS)
    int64_t o0, o1;
    int32_t cap;
    int32_t *lengths;       // [sub][row][channel]
    int32_t *status;        // may be null
    int32_t *tile_sums;     // SLOTS, one block per tile of kSlotTile streams: stored bytes per tile, or null
    int32_t *group_sums;    // with tile_sums, or null: the tile's bytes are also added to the sum of its
                            // group of kTileGroup tiles (zero before the launch)
    const float *key_bins, *value_bins;     // float32 [L] each, or null when the levels are not known
    int64_t L;
    StreamGrid sg;
};


// How a packed word holds its four symbols: kBytes, a byte each (any value; kept inside the
// table where it is used); kNibbles, four bits each, every one a table symbol; kNibblesEscaped,
// four bits each where 15 stands for a saturated byte, i.e. the table's last symbol.
enum { kBytes = 0, kNibbles = 1, kNibblesEscaped = 2 };

template <bool SENTINEL_, int MODE_>
struct CodeTag {
    static constexpr bool SENTINEL = SENTINEL_;
    static constexpr int MODE = MODE_;
};

template <int MODE>
__device__ __forceinline__ uint32_t packed_symbol(uint32_t v, int j, uint32_t smax)
{
    if (MODE == kBytes) return (v >> (8 * j)) & 0xFFu;
    uint32_t s = __builtin_amdgcn_ubfe(v, (uint32_t)(4 * j), 4u);
    if (MODE == kNibblesEscaped) s = s == 15u ? smax : s;
    return s;
}

// PACKED: symbols come from sym4.  FUSE_CDF (PACKED only, one sub-chunk per chunk): the
// block first builds its own tables from the same words and writes them out.
// SLOTS: stream g of the launch is written to out[g * cap ...] (the fused path's scratch).
template <int BS, bool ALIGNED, bool PACKED, bool FUSE_CDF, bool SLOTS, bool TILE = false>
__global__ __launch_bounds__(BS) void encode_streams_kernel(EncodeArgs a)
{
    extern __shared__ uint16_t tab[];
    const int tid = threadIdx.x;
    const StreamId id = locate<BS>(a.sg);
    const int lp = a.lp;
    const int64_t ch0 = id.ch - tid;
    uint16_t *col = tab + table_column<BS>(tid);
    uint16_t *cdf_block = a.cdf + ((id.chunk * a.sg.rows + id.row) * a.sg.nc + ch0) * lp;
    const int nwords = (id.n + 3) >> 2;
    // PACKED: the sub-chunk's words ([word][channel]) are read through a buffer descriptor that
    // ends with its last word row: the lane's channel is the vector offset, the word row the
    // scalar one, and a row past the end (or the offset of a lane without a channel) reads
    // zero, so a load costs no address arithmetic, compare or branch.
    __amdgpu_buffer_rsrc_t symbols_rsrc;
    uint32_t symbols_voff = 0xFFFFFFFCu;
    const uint32_t row_bytes = (uint32_t)a.sg.nc * 4u;
    if (PACKED) {
        const int64_t first = ((id.row * a.nsub + id.sub) * kWordsPerSub) * a.sg.nc;        // uniform over the block
        const uint32_t lo32 = __builtin_amdgcn_readfirstlane((uint32_t)first);
        const uint32_t hi32 = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)first >> 32));
        symbols_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(a.sym4 + (int64_t)(((uint64_t)hi32 << 32) | lo32)), 0,
                                                         (int)((uint32_t)nwords * row_bytes), kBufferWord3);
        if (id.active) symbols_voff = (uint32_t)id.ch * 4u;
    }
    // The row's alphabet (2C + 1 symbols for `bins` levels, encoder.py:44-52): it may leave the
    // table's last symbol unused (then its special upper bound is never needed), and with at
    // most 15 symbols the quantizer may have packed it four bits a symbol, two channels to a
    // word.  A token row whose scale overflowed (a maximum so small that MAX / max is infinite)
    // saturates its bytes to 255, which the reference's coder reads as the table's last symbol:
    // such bytes arrive as the value 15.  All uniform over the block.
    bool sentinel = true;
    int mode = kBytes;
    uint32_t half_shift = 0;
    if (PACKED && a.key_bins) {
        const int64_t kvi = id.row >= a.L ? 1 : 0, l = id.row - kvi * a.L;       // 2L rows: keys, then values
        const float cq = floorf((kvi ? a.value_bins : a.key_bins)[l] * 0.5f) - 1.0f;
        sentinel = !(cq >= 0.0f && 2.0f * cq + 1.0f <= (float)(lp - 2));
        if (a.maxima) {
            int saturates = 0;
            // every token row of the sub-chunk, whatever the block size
            for (int i = tid; i < id.n; i += BS) {
                const uint32_t bits = a.maxima[id.row * a.sg.g.T + id.t0 + i];
                const float m = a.max_dt == CG_DT_BF16 ? load16f<CG_DT_BF16>(bits) : load16f<CG_DT_F16>(bits);
                saturates |= scale_overflows(cq, m);
            }
            if (__syncthreads_or(saturates)) sentinel = true;       // the last symbol does occur
        }
        if (a.nibbles && narrow_alphabet(cq, lp)) {
            mode = sentinel ? kNibblesEscaped : kNibbles;
            if (id.active) symbols_voff = (uint32_t)(id.ch >> 1) * 4u;
            half_shift = (uint32_t)(id.ch & 1) * 16u;
        }
    }

    // Half a sub-chunk (32 words = 128 symbols) at a time is loaded into registers and indexed
    // by the (uniform) loop counter, so the coding loop has no loads to wait for and its stores
    // never hold it up.
    typedef uint32_t words32 __attribute__((ext_vector_type(32)));
    words32 words;
    auto load_half = [&](int h) {
#pragma unroll
        for (int w = 0; w < 32; ++w)
            words[w] = __builtin_amdgcn_raw_buffer_load_b32(symbols_rsrc, (int)symbols_voff,
                                                            (int)((uint32_t)(h * 32 + w) * row_bytes), 0);
    };

    if (FUSE_CDF) {
        for (int i = 0; i < lp; ++i) col[i * TableStride<BS>::k16] = 0;
        __syncthreads();                     // another lane, of another wavefront, shares this lane's words
        if (id.active) {
            const uint32_t smax = (uint32_t)(lp - 2);
            // two lanes share a 32-bit LDS word: each adds to its own half with one atomic that
            // returns nothing (a count is at most 256, so the low half never carries over)
            uint32_t *const pair = reinterpret_cast<uint32_t *>(tab) + (table_column<BS>(tid) >> 1);
            const uint32_t one = (table_column<BS>(tid) & 1) ? 0x10000u : 1u;
            auto count = [&](auto tag) {
                constexpr int MODE = decltype(tag)::MODE;
                for (int h = 0; h * 32 < nwords; ++h) {
                    load_half(h);
                    // uniform; kept in a scalar register so that the loop test is scalar too
                    const int wn = __builtin_amdgcn_readfirstlane(nwords - h * 32 < 32 ? nwords - h * 32 : 32);
#pragma unroll 1
                    for (int w = 0; w < wn; ++w) {
                        const uint32_t v = MODE == kBytes ? words[w] : words[w] >> half_shift;
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            uint32_t s = packed_symbol<MODE>(v, j, smax);
                            if (MODE == kBytes) s = s < smax ? s : smax;
                            if ((h * 32 + w) * 4 + j < id.n) atomicAdd(pair + (s + 1) * (TableStride<BS>::k16 / 2), one);
                        }
                    }
                }
            };
            if (mode == kNibbles) count(CodeTag<false, kNibbles>());
            else if (mode == kNibblesEscaped) count(CodeTag<false, kNibblesEscaped>());
            else count(CodeTag<false, kBytes>());
        }
        __syncthreads();                     // the other lane's counts are all in
        if (id.active) {
            normalize_column16<BS>(col, lp, lp - 1, (uint32_t)id.n);
            write_column16<BS>(col, cdf_block + (int64_t)tid * lp, lp);
        }
    } else {
        // packed symbols: every lane copies its own table (the transposed copy costs a division
        // and a dozen instructions an entry; this one costs the coder under one a symbol)
        if (!PACKED) stage_tables16<BS>(tab, cdf_block, lp, ch0, a.sg.nc);
        else if (id.active) stage_column16_stride<TableStride<BS>::k16>(col, cdf_block + (int64_t)tid * lp, lp);
        __syncthreads();
    }
    if (!id.active) return;

    RangeEncoder<BS, ALIGNED, TILE> enc;
    const int64_t stream = (id.sub * a.sg.rows + id.row) * a.sg.nc + id.ch;
    // SLOTS: the scratch is cut into tiles of kSlotTile streams; word w of a tile's stream t is
    // the tile's word w * kSlotTile + t, so that the words the lanes of a wavefront write, and
    // the words the compaction reads, lie side by side
    if (TILE) {
        // the block is exactly one tile (the host launches this form only then): its number is
        // the tile, tid the stream's place in it
        enc.init(col, lp);
        enc.w.init(nullptr, 0, a.cap);
        enc.w.init_tile(__builtin_amdgcn_make_buffer_rsrc((void *)(a.out + (int64_t)linear_block() * ((int64_t)kSlotTile * a.cap)), 0,
                                                          kSlotTile * a.cap, kBufferWord3),
                        (uint32_t)tid * 4u);
    } else if (SLOTS) {
        enc.init(col, lp);
        enc.w.init(a.out + (stream / kSlotTile) * ((int64_t)kSlotTile * a.cap) + (stream % kSlotTile) * 4, kSlotTile * 4, a.cap);
    } else {
        enc.init(col, lp);
        enc.w.init(a.out + id.row * a.o0 + id.ch * a.o1, 4, a.cap);
    }

    auto code = [&](auto tag) {
        constexpr bool SENTINEL = decltype(tag)::SENTINEL;
        constexpr int MODE = decltype(tag)::MODE;
        // a byte can lie outside the table only where the table's last symbol can occur at all
        // (a saturated row, a table shorter than the row's alphabet, symbols handed in by a caller)
        constexpr bool CLAMP = MODE == kBytes && SENTINEL;
        const uint32_t smax = (uint32_t)(lp - 2);
        if (PACKED) {
            for (int h = 0; h * 32 < nwords; ++h) {
                load_half(h);
                // uniform; kept in a scalar register so that the loop test is scalar too
                const int wn = __builtin_amdgcn_readfirstlane(nwords - h * 32 < 32 ? nwords - h * 32 : 32);
                // two words = eight symbols between two visits of the store code (wn is even
                // except in a sub-chunk's last, partial run of words)
#pragma unroll 1
                for (int w = 0; w < wn; w += 2) {
                    const uint32_t v = MODE == kBytes ? words[w] : words[w] >> half_shift;
                    const int t = (h * 32 + w) * 4;            // first token of the word
                    if (t + 0 < id.n) enc.template put_symbol<SENTINEL, true, CLAMP>(packed_symbol<MODE>(v, 0, smax));
                    if (t + 1 < id.n) enc.template put_symbol<SENTINEL, false, CLAMP>(packed_symbol<MODE>(v, 1, smax));
                    if (t + 2 < id.n) enc.template put_symbol<SENTINEL, false, CLAMP>(packed_symbol<MODE>(v, 2, smax));
                    if (t + 3 < id.n) enc.template put_symbol<SENTINEL, false, CLAMP>(packed_symbol<MODE>(v, 3, smax));
                    if (t + 4 < id.n) {
                        // w + 1 <= 31: wn <= 32
                        const uint32_t u = MODE == kBytes ? words[w + 1] : words[w + 1] >> half_shift;
                        enc.template put_symbol<SENTINEL, false, CLAMP>(packed_symbol<MODE>(u, 0, smax));
                        if (t + 5 < id.n) enc.template put_symbol<SENTINEL, false, CLAMP>(packed_symbol<MODE>(u, 1, smax));
                        if (t + 6 < id.n) enc.template put_symbol<SENTINEL, false, CLAMP>(packed_symbol<MODE>(u, 2, smax));
                        if (t + 7 < id.n) enc.template put_symbol<SENTINEL, false, CLAMP>(packed_symbol<MODE>(u, 3, smax));
                    }
                    enc.end_group();
                }
            }
        } else {
            const uint8_t *sp = a.sym + id.row * a.s0 + id.t0 * a.s1 + id.ch * a.s2;
            uint32_t nxt[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) nxt[j] = (j < id.n) ? sp[(int64_t)j * a.s1] : 0u;
            for (int i0 = 0; i0 < id.n; i0 += 8) {
                uint32_t cur[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) cur[j] = nxt[j];
#pragma unroll
                for (int j = 0; j < 8; ++j) nxt[j] = (i0 + 8 + j < id.n) ? sp[(int64_t)(i0 + 8 + j) * a.s1] : 0u;
#pragma unroll
                for (int j = 0; j < 8; j += 2) {
                    if (i0 + j < id.n) enc.template put_symbol<SENTINEL, true>(cur[j]);
                    if (i0 + j + 1 < id.n) enc.template put_symbol<SENTINEL, false>(cur[j + 1]);
                    enc.end_group();
                }
            }
        }
    };
    if (PACKED && mode == kNibbles) code(CodeTag<false, kNibbles>());
    else if (PACKED && mode == kNibblesEscaped) code(CodeTag<true, kNibblesEscaped>());
    else if (PACKED && !sentinel) code(CodeTag<false, kBytes>());
    else code(CodeTag<true, kBytes>());
    const int len = enc.finish();
    a.lengths[stream] = len;
    if (len > a.cap && a.status) atomicOr(a.status, 1);
    if (SLOTS && a.tile_sums) {
        // every lane of the block is active here (the host asks for tile sums only when a block
        // is exactly one tile): bytes the block's streams occupy in the payload
        __shared__ int32_t wave_sums[BS / 64];
        int32_t v = len < a.cap ? len : a.cap;
#pragma unroll
        for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
        if ((tid & 63) == 0) wave_sums[tid >> 6] = v;
        __syncthreads();
        if (tid == 0) {
            int32_t total = 0;
            for (int w = 0; w < BS / 64; ++w) total += wave_sums[w];
            const uint32_t tile = linear_block();
            a.tile_sums[tile] = total;                            // at most 256 streams of 256 bytes
            if (a.group_sums) __hip_atomic_fetch_add(a.group_sums + tile / kTileGroup, total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace
