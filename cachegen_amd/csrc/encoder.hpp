// Part of the CacheGen KV codec library for MI355X (gfx950); included by cachegen_hip.hip, which
// is the one translation unit.  Range encoder: bit writer, coder state, encode_streams_kernel.
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
// Bits are collected MSB-first in a 64-bit accumulator and leave as big-endian 32-bit words.
// Every lane of a wavefront runs the store code whenever one lane has a word ready, so words
// are written at fixed points, once per eight symbols (per two, for byte symbols), instead of
// whenever a lane's accumulator fills; the accumulator takes the symbols in between (a put
// that would not fit writes a word first).
// The E1/E2 run of a symbol is emitted at once: the n1 = clz(low ^ high) leading bits
// agree, and the pending complements go in after the first of them, which in arithmetic
// is  bits + ((2^pend - 1) << (n1 - 1))  over n1 + pend bits.  The E3 run k is the number
// of positions below those where low has ones and high has zeros.  One combined shift by
// n = n1 + k renormalises low and high; n <= 18 for any table whose symbols all have
// non-zero width, because the span stays above 2^30 between symbols.
constexpr int kSlotTile = 256;      // streams per tile of the encoder's scratch

// TILE: the stream's words go to a tile of the scratch (word w of the tile's stream t at the
// tile's word w * kSlotTile + t) through a buffer descriptor that covers exactly the tile: a
// word or byte past the stream's capacity falls outside the descriptor and is dropped by the
// hardware, so nothing is compared or counted per word.
template <bool ALIGNED, bool TILE = false>
struct BitWriter {
    uint8_t *wptr;          // where the next word goes
    int wstride;            // bytes from one word of the stream to the next (4: contiguous)
    int cap;
    int nbytes;
    __amdgpu_buffer_rsrc_t tile;    // TILE: the block's tile
    uint32_t voff, voff0;           // TILE: byte offset in the tile of the next word, and of the first
    uint64_t acc;           // the low 64 - room bits are waiting to be written; bits above are stale
    // free bits of the accumulator: counted this way, the subtraction that books a put borrows
    // exactly when the bits do not fit, and that borrow is the test
    uint32_t room;

    // the last words of a stream that does not fit its slot: keep what fits
    __device__ __forceinline__ void store_clipped(uint32_t word)
    {
        for (int j = 0; j < 4; ++j)
            if (nbytes + j < cap) wptr[j] = (uint8_t)(word >> (24 - 8 * j));
    }

    __device__ __forceinline__ void store_word(uint32_t word)
    {
        if (TILE) {
            __builtin_amdgcn_raw_buffer_store_b32((int)__builtin_bswap32(word), tile, (int)voff, 0, 0);
            voff += kSlotTile * 4;
            return;
        }
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
            store_clipped(word);
        }
        wptr += wstride;
        nbytes += 4;
    }

    // write one word if 32 bits are waiting
    __device__ __forceinline__ void flush_word()
    {
        if (room <= 32u) {
            store_word((uint32_t)(acc >> (32u - room)));
            room += 32u;
        }
    }

    // append the low m bits of v (v < 2^m), 0 <= m <= 32 (m = 0 needs v = 0).  ROOM: the caller
    // knows that at most 32 bits are waiting (it has just called flush_word), so they fit.
    // `more` (default 0): a second addend, for callers whose value is a sum of two parts that
    // together stay below 2^m; the freshly shifted accumulator has m zero bits at the bottom, so
    // the parts are added in (one three-operand add) instead of summed and then or-ed in
    template <bool ROOM = false>
    __device__ __forceinline__ void put(uint32_t v, int m, uint32_t more = 0)
    {
        uint32_t left;
        if (__builtin_expect(__builtin_usub_overflow(room, (uint32_t)m, &left), 0) && !ROOM) {
            flush_word();                                  // more than 32 bits were waiting
            left = room - (uint32_t)m;
        }
        room = left;
        acc <<= m;
        acc = (acc & 0xFFFFFFFF00000000ull) | (uint32_t)((uint32_t)acc + v + more);
    }

    // one bit, then `count` copies of its complement (any count): the general form of
    // append_bit_and_pending (enc_new.cu:86-97); not on the common path
    __device__ __forceinline__ void bit_and_run(uint32_t bit, uint32_t count)
    {
        uint32_t pv = bit;
        int pm = 1;
        for (;;) {
            put(pv, pm);
            flush_word();
            if (count == 0) break;
            pm = count < 32u ? (int)count : 32;
            pv = bit ? 0u : (pm == 32 ? 0xFFFFFFFFu : ((1u << pm) - 1u));
            count -= (uint32_t)pm;
        }
    }

    // write what is left, the last partial word byte by byte (enc_new.cu:42-55); returns
    // the stream length
    __device__ __forceinline__ int finish()
    {
        flush_word();
        flush_word();
        const int nacc = 64 - (int)room;
        if (TILE) nbytes = (int)((voff - voff0) / kSlotTile);     // four bytes per word written
        if (nacc > 0) {
            uint32_t r = (uint32_t)(acc << (32 - nacc));
            for (int left = nacc, j = 0; left > 0; left -= 8, ++j) {
                if (TILE) __builtin_amdgcn_raw_buffer_store_b8((char)(r >> 24), tile, (int)(voff + j), 0, 0);
                else if (nbytes < cap) wptr[j] = (uint8_t)(r >> 24);
                nbytes++;
                r <<= 8;
            }
        }
        return nbytes;
    }
};

// The coder state is (low, span) with span = high - low + 1 held modulo 2^32: 0 stands for
// the full range 2^32 (the initial state, and any later interval that is exactly a binary
// fraction), where floor(span * c / 2^16) is simply c << 16.  Renormalising by n bits maps
// span to span << n for E1/E2 and E3 steps alike.
template <int BS, bool ALIGNED, bool TILE = false>
struct RangeEncoder {
    lds_char *col;          // this lane's table column: entry e at byte e * 2 * TableStride<BS>::k16
    uint32_t smax;          // lp - 2: the largest symbol
    uint32_t low, span, pend;
    // the coded symbol's two table entries, each shifted left by 16: only ever written by
    // loads into the upper half, so that the lower halves stay zero
    uint32_t bound_lo, bound_hi;
    BitWriter<ALIGNED, TILE> w;

    __device__ __forceinline__ void init(const uint16_t *column, int lp, uint8_t *dst, int wstride, int cap)
    {
        col = (lds_char *)column;
        bound_lo = 0;
        bound_hi = 0;
        smax = (uint32_t)(lp - 2);
        low = 0;
        span = 0;
        pend = 0;
        w.wptr = dst;
        w.wstride = wstride;
        w.cap = cap;
        w.nbytes = 0;
        w.voff = w.voff0 = 0;
        w.acc = 0;
        w.room = 64;
    }

    // SENTINEL: symbol smax may occur, whose upper bound is 2^16 and not the table's last
    // entry (enc_new.cu:270)
    // FIRST: the symbol directly follows a flush_word (the first of a group)
    template <bool SENTINEL, bool FIRST>
    __device__ __forceinline__ void put_symbol(uint32_t s)
    {
        s = s < smax ? s : smax;                        // keep table reads inside the table
        constexpr int kRow = 2 * TableStride<BS>::k16;
        lds_entries_high<kRow>(col + s * kRow, bound_lo, bound_hi);
        // the upper bound of symbol smax is 2^16 and not the table's last entry; shifted left
        // by 16 that is 0 modulo 2^32, and T(2^16) is the span
        const bool top = SENTINEL && s == smax;
        // T(c) = (span * c) >> 16 = high word of span * (c << 16)
        uint32_t t_lo = __umulhi(span, bound_lo);
        uint32_t width = (top ? span : __umulhi(span, bound_hi)) - t_lo;
        if (__builtin_expect(span == 0, 0)) {
            // the full range: T(c) = c << 16.  The empty statement makes the compiler jump over
            // this block when no lane needs it instead of issuing it with every lane masked off.
            asm volatile("");
            t_lo = bound_lo;
            width = (top ? 0u : bound_hi) - bound_lo;
        }
        low += t_lo;
        const uint32_t high = low + width - 1u;

        const int n1 = __builtin_clz(low ^ high);       // low < high always
        // the n1 agreed bits (none if n1 = 0) with the pending complements after the first
        // n1 - 1 is needed below; computed as n1 + 0xFFFFFFFF its carry says whether n1 > 0
        uint32_t n1m1;
        const bool agreed = __builtin_uadd_overflow((uint32_t)n1, 0xFFFFFFFFu, &n1m1);
        const uint32_t pe = agreed ? pend : 0u;
        const int m = n1 + (int)pe;
        if (__builtin_expect(m > 32, 0)) {
            const uint32_t bits = low >> ((32 - n1) & 31);
            w.bit_and_run(bits >> (n1 - 1), pe);
            w.put(bits & ((1u << (n1 - 1)) - 1u), n1 - 1);
        } else {
            const uint32_t bits = __builtin_amdgcn_ubfe(low, (uint32_t)(32 - n1), (uint32_t)n1);
            // ((1 << pe) - 1) << (n1 - 1), pe <= 31 here; with n1 = 0, pe is 0 and so is the mask
            uint32_t fill;
            asm("v_bfm_b32 %0, %1, %2" : "=v"(fill) : "v"(pe), "v"(n1m1));
            w.template put<FIRST>(bits, m, fill);
        }
        // E3 run: leading zeros of (~low | high) below the first differing bit
        const uint32_t z = shift_left_one_more((low & high) | ~low, n1);
        const int k = __builtin_clz(z);
        const int n = n1 + k;
        pend = pend - pe + (uint32_t)k;
        low = (low << n) & 0x7FFFFFFFu;
        span = width << n;
    }

    __device__ __forceinline__ int finish()
    {
        pend += 1;
        w.bit_and_run(low < 0x40000000u ? 0u : 1u, pend);
        return w.finish();
    }
};

struct EncodeArgs {
    uint16_t *cdf;          // [chunk][row][channel][lp]; written when the histogram is fused
    int32_t lp;
    const uint8_t *sym;     // byte symbols: sym[row*s0 + token*s1 + channel*s2]
    int64_t s0, s1, s2;
    const uint32_t *sym4;   // or packed symbols
    int64_t nsub;
    uint8_t *out;           // out[row*o0 + channel*o1 + byte], or the scratch tiles (SLOTS)
    int64_t o0, o1;
    int32_t cap;
    int32_t *lengths;       // [sub][row][channel]
    int32_t *status;        // may be null
    int32_t *tile_sums;     // SLOTS, one block per tile of kSlotTile streams: stored bytes per tile, or null
    const float *key_bins, *value_bins;     // float32 [L] each, or null when the levels are not known
    int64_t L;
    StreamGrid sg;
};


template <bool B>
struct BoolTag {
    static constexpr bool value = B;
};

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
    uint16_t *col = tab + tid;
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
        if (id.active) {
            const uint32_t smax = (uint32_t)(lp - 2);
            // two lanes share a 32-bit LDS word: each adds to its own half with one atomic that
            // returns nothing (a count is at most 256, so the low half never carries over)
            uint32_t *const pair = reinterpret_cast<uint32_t *>(tab) + (tid >> 1);
            const uint32_t one = (tid & 1) ? 0x10000u : 1u;
            for (int h = 0; h * 32 < nwords; ++h) {
                load_half(h);
                // uniform; kept in a scalar register so that the loop test is scalar too
                const int wn = __builtin_amdgcn_readfirstlane(nwords - h * 32 < 32 ? nwords - h * 32 : 32);
#pragma unroll 1
                for (int w = 0; w < wn; ++w) {
                    const uint32_t v = words[w];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        uint32_t s = (v >> (8 * j)) & 0xFFu;
                        s = s < smax ? s : smax;
                        if ((h * 32 + w) * 4 + j < id.n) atomicAdd(pair + (s + 1) * (TableStride<BS>::k16 / 2), one);
                    }
                }
            }
            normalize_column16<BS>(col, lp, lp - 1, (uint32_t)id.n);
        }
        __syncthreads();
        write_tables16<BS>(tab, cdf_block, lp, ch0, a.sg.nc);
    } else {
        stage_tables16<BS>(tab, cdf_block, lp, ch0, a.sg.nc);
        __syncthreads();
    }
    if (!id.active) return;

    RangeEncoder<BS, ALIGNED, TILE> enc;
    const int64_t stream = (id.sub * a.sg.rows + id.row) * a.sg.nc + id.ch;
    // SLOTS: the scratch is cut into tiles of kSlotTile streams; word w of a tile's stream t is
    // the tile's word w * kSlotTile + t, so that the words the lanes of a wavefront write, and
    // the words the compaction reads, lie side by side
    if (TILE) {
        // the block is exactly one tile (the host launches this form only then): blockIdx.x is
        // the tile, tid the stream's place in it
        enc.init(col, lp, nullptr, 0, a.cap);
        enc.w.tile = __builtin_amdgcn_make_buffer_rsrc((void *)(a.out + (int64_t)blockIdx.x * ((int64_t)kSlotTile * a.cap)), 0,
                                                       kSlotTile * a.cap, kBufferWord3);
        enc.w.voff = enc.w.voff0 = (uint32_t)tid * 4u;
    } else if (SLOTS)
        enc.init(col, lp, a.out + (stream / kSlotTile) * ((int64_t)kSlotTile * a.cap) + (stream % kSlotTile) * 4,
                 kSlotTile * 4, a.cap);
    else
        enc.init(col, lp, a.out + id.row * a.o0 + id.ch * a.o1, 4, a.cap);

    // The row's alphabet (2C + 1 symbols for `bins` levels, encoder.py:44-52) may leave the
    // table's last symbol unused; then its special upper bound is never needed.  Uniform
    // over the block.
    bool sentinel = true;
    if (PACKED && a.key_bins) {
        const int64_t kvi = id.row / a.L, l = id.row - kvi * a.L;
        const float cq = floorf((kvi ? a.value_bins : a.key_bins)[l] * 0.5f) - 1.0f;
        sentinel = !(cq >= 0.0f && 2.0f * cq + 1.0f <= (float)(lp - 2));
    }

    auto code = [&](auto tag) {
        constexpr bool SENTINEL = decltype(tag)::value;
        if (PACKED) {
            for (int h = 0; h * 32 < nwords; ++h) {
                load_half(h);
                // uniform; kept in a scalar register so that the loop test is scalar too
                const int wn = __builtin_amdgcn_readfirstlane(nwords - h * 32 < 32 ? nwords - h * 32 : 32);
                // two words = eight symbols between two visits of the store code (wn is even
                // except in a sub-chunk's last, partial run of words)
#pragma unroll 1
                for (int w = 0; w < wn; w += 2) {
                    const uint32_t v = words[w];
                    const int t = (h * 32 + w) * 4;            // first token of the word
                    if (t + 0 < id.n) enc.template put_symbol<SENTINEL, true>(v & 0xFFu);
                    if (t + 1 < id.n) enc.template put_symbol<SENTINEL, false>((v >> 8) & 0xFFu);
                    if (t + 2 < id.n) enc.template put_symbol<SENTINEL, false>((v >> 16) & 0xFFu);
                    if (t + 3 < id.n) enc.template put_symbol<SENTINEL, false>(v >> 24);
                    if (t + 4 < id.n) {
                        const uint32_t u = words[w + 1];       // w + 1 <= 31: wn <= 32
                        enc.template put_symbol<SENTINEL, false>(u & 0xFFu);
                        if (t + 5 < id.n) enc.template put_symbol<SENTINEL, false>((u >> 8) & 0xFFu);
                        if (t + 6 < id.n) enc.template put_symbol<SENTINEL, false>((u >> 16) & 0xFFu);
                        if (t + 7 < id.n) enc.template put_symbol<SENTINEL, false>(u >> 24);
                    }
                    enc.w.flush_word();
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
                    enc.w.flush_word();
                }
            }
        }
    };
    if (PACKED && !sentinel) code(BoolTag<false>());
    else code(BoolTag<true>());
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
            a.tile_sums[blockIdx.x] = total;                  // at most 256 streams of 256 bytes
        }
    }
}

}  // namespace
