// Part of the CacheGen KV codec library for MI355X (gfx950); included by cachegen_hip.hip, which
// is the one translation unit.  Range decoder: bit reader, symbol search, fused dequantisation, decode_streams_kernel.
//
// Paths in the comments are relative to LMCache/ in the reference tree:
//   enc_new.cu = third_party/torchac_cuda/torchac_kernel_enc_new.cu
//   dec_new.cu = third_party/torchac_cuda/torchac_kernel_dec_new.cu
//   cal_cdf.cu = third_party/torchac_cuda/cal_cdf.cu
//   encoder.py = lmcache/storage_backend/serde/cachegen_encoder.py
//   decoder.py = lmcache/storage_backend/serde/cachegen_decoder.py
#pragma once

namespace {

// ---- decoder (dec_new.cu:35-71, 248-302) -------------------------------------------
// The decoder tracks off = value - low, which every renormalisation step maps to
// 2*off + next bit (E1/E2 and E3 alike), and finds the symbol as the largest m with
// T(m) = floor(span*cdf[m] / 2^16) <= off; that is the same m as the reference's search
// of count = ((value-low+1)*2^16 - 1) / span in a strictly increasing table, without the
// 64-bit divide.  For tables of 2^k symbols the search probes with the lower bound
// (span >> 16) * cdf[m] <= T(m) (one multiply), which can only overshoot, and the result
// is then walked back while the exact T(m) exceeds off (almost never).
//
// The stream is read through aligned big-endian words into a 64-bit window of unread bits.
// Every lane of a wavefront runs the refill code whenever one lane needs it, so the window
// is topped up at fixed points, once per four symbols, instead of whenever a lane runs dry:
// after a top-up it holds more than 32 bits, which streams of a few bits per symbol do not
// use up in four symbols; a symbol of a table without zero-width entries consumes at most 18
// (the span stays above 2^30), so the case left (fewer than 18 bits before one of the other
// three symbols) takes an extra top-up.
// Bits past the end of a stream are whatever follows it in memory instead of the reference's
// zeros (dec_new.cu:223-233): the coder's two closing bits place the code value inside
// the final interval for every continuation, so the n symbols that were encoded decode
// identically.  Word loads past the last word of the byte buffer return zeros.

// The most bits one symbol can move for a table without zero-width entries.
constexpr uint32_t kSymbolBits = 18;
// Symbols between two unconditional top-ups of the bit window.
constexpr int kSymbolsPerTopUp = 8;

struct BitReader {
    // Words are fetched with buffer loads: the descriptor (uniform over the wavefront) covers
    // the byte buffer from the wavefront's lowest stream to its last readable word, a lane
    // addresses it with a 32-bit offset, and a load outside it returns zero instead of faulting.
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t pos;            // byte offset inside the descriptor's range of the next word to fetch
    uint64_t win;            // the unread bits of the stream that are loaded, left-aligned, zeros below
    // how many bits `win` holds beyond kSymbolBits, the most one symbol can take: counted this
    // way, the subtraction that consumes a symbol's bits borrows exactly when the window no
    // longer covers another symbol, and that borrow is the test
    uint32_t spare;
    bool short_of_bits;      // the last shift_in left fewer than kSymbolBits
    uint32_t nextw;          // the word after the window, as loaded

    __device__ __forceinline__ uint32_t raw()
    {
        const uint32_t w = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)pos, 0, 0);
        pos += 4;
        return w;
    }

    // position on the stream that begins `begin` bytes after the 4-byte aligned `window`,
    // whose last readable word is at byte offset `last_word`; returns the first 32 bits
    // `lowest`: the smallest `begin` among the wavefront's lanes, the same value in every lane
    __device__ __forceinline__ uint32_t start(const uint8_t *window, int64_t last_word, int64_t begin, int64_t lowest)
    {
        // a start outside the buffer (offsets that are not running sums of stream lengths) is
        // moved inside it: such a stream decodes to garbage, never to a read out of bounds
        const int64_t top = last_word + 3;                                   // last_word is a word's first byte
        begin = begin < 0 ? 0 : (begin > top ? top : begin);
        lowest = lowest < 0 ? 0 : (lowest > top ? top : lowest);
        const uint32_t skip = (uint32_t)begin & 3u;
        const int64_t first_word = begin - skip;
        // the descriptor starts at the word of the wavefront's lowest stream, so every lane's
        // offset from it is its own distance; one that is 4 GiB or more wraps, which reads zeros
        // or some other place inside the buffer
        const int64_t low_word = lowest & ~3ll;
        const uint32_t org_lo = __builtin_amdgcn_readfirstlane((uint32_t)low_word);
        const uint32_t org_hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)low_word >> 32));
        const int64_t origin = (int64_t)(((uint64_t)org_hi << 32) | org_lo);
        const int64_t room = last_word + 4 - origin;                           // >= 4
        rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(window + origin), 0,
                                                 (int)(room > 0xFFFFFFFFll ? 0xFFFFFFFFu : (uint32_t)room), kBufferWord3);
        pos = (uint32_t)(first_word - origin);
        const uint32_t b0 = __builtin_bswap32(raw()), b1 = __builtin_bswap32(raw());
        const uint32_t b2 = __builtin_bswap32(raw());
        nextw = raw();
        const uint32_t s = skip * 8u;
        const uint64_t head = (((uint64_t)b0 << 32) | b1) << s;
        const uint64_t rest = (((uint64_t)b1 << 32) | b2) << s;
        win = rest;
        spare = 64u - kSymbolBits - s;
        short_of_bits = false;
        return (uint32_t)(head >> 32);
    }

    // off = (off << n) | next n bits, 0 <= n <= 31 and n <= spare + kSymbolBits
    __device__ __forceinline__ uint32_t shift_in(uint32_t off, int n)
    {
        // two 64-bit shifts: {off, top word of the window} and the window itself
        const uint64_t pair = (((uint64_t)off << 32) | (uint32_t)(win >> 32)) << n;
        off = (uint32_t)(pair >> 32);
        win <<= n;
        short_of_bits = __builtin_usub_overflow(spare, (uint32_t)n, &spare);
        return off;
    }

    // brings the window to more than 32 bits
    __device__ __forceinline__ void top_up()
    {
        if ((int32_t)spare <= 32 - (int)kSymbolBits) {          // at most 32 bits: the low word is empty
            const uint64_t in = (((uint64_t)__builtin_bswap32(nextw)) << 32) >> ((spare + kSymbolBits) & 63);
            win = (((win >> 32) | (in >> 32)) << 32) | (uint32_t)in;
            spare += 32;
            nextw = raw();
        }
    }
};

enum { SRC_OFFSETS = 0, SRC_PREFIX = 1, SRC_PADDED = 2 };
enum { OUT_SYMBOLS = 0, OUT_F16 = 1, OUT_BF16 = 2 };

struct DecodeArgs {
    const uint16_t *cdf;
    int32_t lp;
    const uint8_t *bytes;       // payload or padded buffer, rounded down to a 4-byte boundary
    uint32_t bytes_skew;        // bytes dropped by that rounding (0..3)
    int64_t last_word;          // byte offset from `bytes` of the last readable word
    const int64_t *offsets;     // SRC_OFFSETS: exclusive sums [nstreams+1]; SRC_PREFIX: inclusive sums
    int64_t p0, p1;             // SRC_PADDED strides
    // OUT_SYMBOLS: out[row*o0 + token*o1 + channel*o2] uint8
    uint8_t *out_sym;
    int64_t o0, o1, o2;
    // OUT_F16 / OUT_BF16: dequantised KV, out[l*ol + kv*okv + token*ot + head*oh + dim]
    uint16_t *out_kv;
    int64_t ol, okv, ot, oh;
    int64_t L;
    int32_t D;
    const uint16_t *maxima;     // [2, L, T]
    int32_t max_dt;
    int32_t delta_group;        // > 0: rows that are not the first of their group hold deltas
    const float *key_bins, *value_bins;
    // blocks from this one on (in launch order) start when no block is left to take a finished
    // one's place: see decode_lane
    uint32_t last_round_first;
    StreamGrid sg;
};

// Tables in LDS for the decoder: entry e of lane c's column is the 16-bit word at byte
// e * kRow + 2 * c.  When the kernel dequantises, every row carries one float behind the
// lanes' entries: (e - C) / C, the quotient of symbol e (decoder.py:28-31).
template <int BS, int OUT>
struct DecodeLayout {
    static constexpr int kRow = OUT == OUT_SYMBOLS ? 2 * BS : 2 * BS + 4;
    static constexpr int kQuot = 2 * BS;          // byte offset of the quotient inside a row
};


__device__ __forceinline__ uint32_t lds_entry(lds_char *p, int byte_offset)
{
    return *(lds_u16 *)(p + byte_offset);
}

// float32 -> bfloat16 bits by the hardware's conversion (round to nearest even, a NaN stays
// a NaN): one instruction on this GPU
__device__ __forceinline__ uint32_t float_to_bf16_bits_hw(float f)
{
    return __builtin_bit_cast(uint16_t, (__bf16)f);
}

struct DecodeLane {
    BitReader rd;
    uint32_t off, low, span;
    lds_char *colp;            // this lane's entry 0
    int lutoff;                // from an entry of this lane to its row's quotient
    // the entries the first two probes of the unrolled search look at (one for the first, one
    // of two for the second), read once per stream: two LDS round trips less per symbol
    uint32_t probe1, probe2_lo, probe2_hi;
    // the decoded symbol's two table entries, each shifted left by 16: only ever written by
    // loads into the upper half, so that the lower halves stay zero
    uint32_t bound_lo, bound_hi;
    uint8_t *osym;
    // dequantised output: one buffer descriptor per block, starting at the block's first token
    // row of its (layer, K/V) slab; a lane adds its channel's byte offset, a token row is
    // reached through the scalar offset
    __amdgpu_buffer_rsrc_t orsrc;
    uint32_t ovoff;
    float anchor;              // reconstructed anchor row value (delta mode)
    int phase;                 // position of the token inside its group (delta mode)
};

// Distance of the unrolled search's first probe from entry 0, in entries.
__host__ __device__ constexpr int first_probe(int log2, int skip) { return log2 >= 2 ? ((1 << log2) >> 1) >> skip : 0; }

// One symbol.  SKIP: how many of the search's first probes are left out because the row's
// alphabet fits the lower 2^(LOG2-SKIP) entries.  SAFE: the last table entry may be decoded
// (its upper bound 2^16 is substituted, dec_new.cu:278) and values may be NaN.
template <int BS, int LOG2, int OUT, int SKIP, bool SAFE>
__device__ __forceinline__ void decode_symbol(const DecodeArgs &a, DecodeLane &s, int lp, int nsteps,
                                              float rm, int i, bool last_symbol)
{
    constexpr int kRow = DecodeLayout<BS, OUT>::kRow;
    constexpr int kStep1 = first_probe(LOG2, SKIP), kStep2 = kStep1 >> 1;
    lds_char *p = s.colp;              // entry of the decoded symbol
    lds_char *const plast = s.colp + (lp - 2) * kRow;
    uint32_t t_lo, width, rel;         // rel = off - t_lo
    float q = 0.0f;                    // (symbol - C) / C
    const bool full_range = s.span == 0;
    const uint32_t sh = s.span >> 16, sl = s.span & 0xFFFFu;
    if (LOG2 >= 2) {
        // largest m with T(m) <= off, probed with the lower bound sh * c <= T(c), which can
        // only overshoot; the first two probes compare entries held in registers
        const bool up1 = mul24(sh, s.probe1) <= s.off;
        p = up1 ? p + kStep1 * kRow : p;
        if (kStep2 >= 1) {
            const uint32_t c2 = up1 ? s.probe2_hi : s.probe2_lo;
            p = (mul24(sh, c2) <= s.off) ? p + kStep2 * kRow : p;
        }
#pragma unroll
        for (int step = kStep2 >> 1; step >= 1; step >>= 1)
            p = (mul24(sh, lds_entry(p, step * kRow)) <= s.off) ? p + step * kRow : p;
        // both bounds and the quotient in one round trip (entry lp - 1 exists, so the upper
        // bound of the last symbol can be read and then replaced)
        if (OUT != OUT_SYMBOLS) q = *(lds_f32 *)(p + s.lutoff);
        lds_entries_high<kRow>(p, s.bound_lo, s.bound_hi);
        // T(c) = (span * c) >> 16 = high word of span * (c << 16) for c < 2^16; the one entry
        // that is 2^16, the upper bound of the last symbol (dec_new.cu:278), gives the span
        t_lo = __umulhi(s.span, s.bound_lo);
        width = ((SAFE && p == plast) ? s.span : __umulhi(s.span, s.bound_hi)) - t_lo;
        // One test for what is left: off - t_lo wraps when the search overshot, and the full
        // range (span 0 modulo 2^32: a stream's first symbol, hardly ever later) gives width 0.
        rel = s.off - t_lo;
        if (__builtin_expect(rel >= width, 0)) {
            if (full_range) {
                // T(m) = cdf[m] << 16, so table values are compared with off >> 16
                const uint32_t key = s.off >> 16;
                p = s.colp;
#pragma unroll
                for (int step = kStep1; step >= 1; step >>= 1)
                    p = (lds_entry(p, step * kRow) <= key) ? p + step * kRow : p;
                const uint32_t c_lo = lds_entry(p, 0);
                const uint32_t c_hi = (SAFE && p == plast) ? 0x10000u : lds_entry(p, kRow);
                t_lo = c_lo << 16;
                width = (c_hi - c_lo) << 16;
            } else {
                // entry 0 is 0 (forced when the tables are staged), so this stops there at the latest
                bool top = SAFE && p == plast;
                uint32_t b_lo = s.bound_lo, b_hi = s.bound_hi;
                while (t_lo > s.off) {
                    p -= kRow;
                    b_hi = b_lo;
                    top = false;
                    b_lo = lds_entry(p, 0) << 16;
                    t_lo = __umulhi(s.span, b_lo);
                }
                width = (top ? s.span : __umulhi(s.span, b_hi)) - t_lo;
            }
            if (OUT != OUT_SYMBOLS) q = *(lds_f32 *)(p + s.lutoff);
            rel = s.off - t_lo;
        }
    } else {
        int lo_i = 0, hi_i = lp - 1;
        for (int step = 0; step < nsteps; ++step) {
            const int mid = (lo_i + hi_i) >> 1;
            const uint32_t c = lds_entry(s.colp, mid * kRow);
            const bool le = mid > 0 && (full_range ? c <= (s.off >> 16) : scale_span(sh, sl, c) <= s.off);
            lo_i = le ? mid : lo_i;
            hi_i = le ? hi_i : mid;
        }
        p = s.colp + lo_i * kRow;
        const uint32_t c_lo = lds_entry(p, 0);
        const uint32_t c_hi = (SAFE && p == plast) ? 0x10000u : lds_entry(p, kRow);
        if (OUT != OUT_SYMBOLS) q = *(lds_f32 *)(p + s.lutoff);
        if (full_range) {
            t_lo = c_lo << 16;
            width = (c_hi - c_lo) << 16;
        } else {
            t_lo = scale_span(sh, sl, c_lo);
            width = scale_span(sh, sl, c_hi) - t_lo;
        }
        rel = s.off - t_lo;
    }
    if (OUT == OUT_SYMBOLS) {
        s.osym[(int64_t)i * a.o1] = (uint8_t)((uint32_t)(p - s.colp) / (uint32_t)kRow);
    } else {
        float v = __fmul_rn(q, rm);
        // the product is rounded to float32 before it is rounded to 16 bits (decoder.py:28-34
        // works in float32): keep the compiler from merging the two into one mixed-precision
        // multiply, which rounds once and turns -0 into +0
        asm volatile("" : "+v"(v));
        if (SAFE && a.delta_group > 0) {             // uniform over the block
            if (s.phase == 0) s.anchor = v;
            else v = __fadd_rn(v, s.anchor);
            s.phase = s.phase + 1 == a.delta_group ? 0 : s.phase + 1;
        }
        uint32_t bits;
        if (OUT == OUT_BF16) bits = float_to_bf16_bits_hw(v);
        else bits = float_to_f16_bits(v);
        __builtin_amdgcn_raw_buffer_store_b16((short)bits, s.orsrc, (int)s.ovoff, (int)((uint32_t)i * (uint32_t)a.ot * 2u), 0);
    }
    if (last_symbol) return;                    // no update after the last symbol
    s.low += t_lo;
    s.off = rel;
    const uint32_t high = s.low + width - 1u;
    const int n1 = __builtin_clz(s.low ^ high);
    // E3 run: positions below the first differing bit where low has 1 and high has 0, i.e.
    // leading zeros of (~low | high) once that bit is shifted out; the run always ends
    // inside the word because the interval is wider than one
    const uint32_t z = shift_left_one_more((s.low & high) | (~s.low & 0xFFFFFFFFu), n1);
    const int n = n1 + __builtin_clz(z);
    // bit 31 of low would be cleared here (the underflow steps subtract a quarter); it is left
    // as it falls: low and high = low + width - 1 then carry the same extra 2^31 modulo 2^32,
    // and only low ^ high and bits below the first differing one are looked at
    s.low <<= n;
    s.span = width << n;
    s.off = s.rd.shift_in(s.off, n);
}

// last_round: the block is one of the launch's last, after which nothing takes the place of a
// finished wavefront.  A wavefront alone on its SIMD cannot go faster than its own dependent
// chain, so the launch ends when the wavefront that started last has run its 256 symbols at that
// pace, while the SIMDs idle more and more (measured: the last 130 us of a 550 us launch, about
// 50 us of issue time lost).  The hardware issues from the oldest wavefront first, which finishes
// the most advanced wavefronts first and leaves the least advanced for the end; these blocks
// raise their wavefronts' priority by the work they have left instead, so that the wavefronts of
// a SIMD finish closer together.
template <int BS, int LOG2, int OUT, int SKIP, bool SAFE>
__device__ __forceinline__ void decode_lane(const DecodeArgs &a, DecodeLane &s, int lp, int n, lds_f32 *rmp, bool last_round)
{
    int nsteps = 0;
    if (LOG2 < 0)
        while ((1 << nsteps) < lp - 1) ++nsteps;
    if (LOG2 >= 2) {
        constexpr int kRow = DecodeLayout<BS, OUT>::kRow;
        constexpr int kStep1 = first_probe(LOG2, SKIP), kStep2 = kStep1 >> 1;
        s.probe1 = lds_entry(s.colp, kStep1 * kRow);
        s.probe2_lo = lds_entry(s.colp, kStep2 * kRow);
        s.probe2_hi = lds_entry(s.colp, (kStep1 + kStep2) * kRow);
        s.bound_lo = 0;
        s.bound_hi = 0;
    }
    // the window is topped up at the head of every group of kGroup symbols and, inside a
    // group, only when a symbol has left it short of bits
    constexpr int kGroup = kSymbolsPerTopUp;
    for (int i0 = 0; i0 < n; i0 += kGroup, rmp += kGroup) {
        if (last_round && (i0 & 63) == 0) {             // uniform over the wavefront
            const int left = (n - i0) >> 6;
            if (left >= 3) __builtin_amdgcn_s_setprio(3);
            else if (left == 2) __builtin_amdgcn_s_setprio(2);
            else if (left == 1) __builtin_amdgcn_s_setprio(1);
            else __builtin_amdgcn_s_setprio(0);
        }
        // the maxima of the group's token rows (the array is padded to a whole group)
        float rm[kGroup];
#pragma unroll
        for (int j = 0; j < kGroup; ++j) rm[j] = OUT != OUT_SYMBOLS ? rmp[j] : 0.0f;
#pragma unroll
        for (int j = 0; j < kGroup; ++j) {
            const int i = i0 + j;
            if (i >= n) break;
            if (j == 0) s.rd.top_up();
            else if (__builtin_expect(s.rd.short_of_bits, 0)) s.rd.top_up();
            decode_symbol<BS, LOG2, OUT, SKIP, SAFE>(a, s, lp, nsteps, rm[j], i, i == n - 1);
        }
    }
}

// LOG2 >= 0: the table has exactly 2^LOG2 symbols (lp = 2^LOG2 + 1) and the search is
// unrolled with immediate LDS offsets; LOG2 < 0: any lp.
template <int BS, int LOG2, int SRC, int OUT>
__global__ __launch_bounds__(BS) void decode_streams_kernel(DecodeArgs a)
{
    extern __shared__ uint32_t smem[];
    constexpr int kRow = DecodeLayout<BS, OUT>::kRow;
    const int tid = threadIdx.x;
    const StreamId id = locate<BS>(a.sg);
    const int lp = LOG2 >= 0 ? (1 << LOG2) + 1 : a.lp;
    char *rows = reinterpret_cast<char *>(smem);
    float *rowmax = reinterpret_cast<float *>(rows + lp * kRow);     // one per token of the sub-chunk
    {
        // Every lane copies its own table (lp consecutive 16-bit entries) into its LDS column:
        // loads and LDS writes with immediate offsets, no address arithmetic per entry; the
        // lanes of a wavefront read neighbouring tables, so each cache line is fetched once.
        // Entry 0 of a table is 0 by construction (cal_cdf.cu:29-49 counts into hist[sym+1]);
        // it is stored as 0 whatever the input holds so that the walk back always ends.
        const uint16_t *mine = a.cdf + ((id.chunk * a.sg.rows + id.row) * a.sg.nc + id.ch) * lp;
        char *column = rows + 2 * tid;
        if (id.active) {
            *reinterpret_cast<uint16_t *>(column) = 0;
            constexpr int kBatch = 16;      // loads in flight per lane
            if (LOG2 >= 0) {
#pragma unroll
                for (int e0 = 1; e0 < lp; e0 += kBatch) {
                    uint16_t v[kBatch];
#pragma unroll
                    for (int j = 0; j < kBatch; ++j)
                        if (e0 + j < lp) v[j] = mine[e0 + j];
#pragma unroll
                    for (int j = 0; j < kBatch; ++j)
                        if (e0 + j < lp) *reinterpret_cast<uint16_t *>(column + (e0 + j) * kRow) = v[j];
                }
            } else {
                for (int e0 = 1; e0 < lp; e0 += kBatch) {
                    uint16_t v[kBatch];
#pragma unroll
                    for (int j = 0; j < kBatch; ++j) v[j] = e0 + j < lp ? mine[e0 + j] : (uint16_t)0;
#pragma unroll
                    for (int j = 0; j < kBatch; ++j)
                        if (e0 + j < lp) *reinterpret_cast<uint16_t *>(column + (e0 + j) * kRow) = v[j];
                }
            }
        }
    }
    int64_t kvi = 0, l = 0;
    int special = 0;                   // a row maximum that is infinite or NaN
    int nsym = lp;                     // symbols the row's alphabet can hold
    if (OUT != OUT_SYMBOLS) {
        kvi = id.row >= a.L ? 1 : 0;             // 2L rows: keys, then values
        l = id.row - kvi * a.L;
        const float bins = (kvi ? a.value_bins : a.key_bins)[l];
        const float cq = floorf(bins * 0.5f) - 1.0f;
        nsym = (cq >= 0.0f && cq < 32768.0f) ? 2 * (int)cq + 1 : lp;
        for (int i = tid; i < lp; i += BS)
            *reinterpret_cast<float *>(rows + i * kRow + DecodeLayout<BS, OUT>::kQuot) =
                __fdiv_rn(__fsub_rn((float)i, cq), cq);
        const uint16_t *mx = a.maxima + id.row * a.sg.g.T + id.t0;
        for (int i = tid; i < id.n; i += BS) {
            const float m = a.max_dt == CG_DT_BF16 ? load16f<CG_DT_BF16>(mx[i]) : load16f<CG_DT_F16>(mx[i]);
            // also rows whose scale overflowed in the quantizer: they hold the table's last symbol
            special |= (__float_as_uint(m) & 0x7FFFFFFFu) >= 0x7F800000u || scale_overflows(cq, m);
            rowmax[i] = m;
        }
    }
    special = __syncthreads_or(special);

    const int64_t stream = (id.sub * a.sg.rows + id.row) * a.sg.nc + id.ch;
    int64_t begin = INT64_MAX;
    if (id.active) {
        if (SRC == SRC_OFFSETS) begin = a.offsets[stream];
        else if (SRC == SRC_PREFIX) begin = stream ? a.offsets[stream - 1] : 0;
        else begin = id.row * a.p0 + id.ch * a.p1;
    }
    // the lowest stream start of the wavefront, taken while all of its lanes are still here
    int64_t lowest = begin;
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const int64_t other = __shfl_xor(lowest, o, 64);
        lowest = other < lowest ? other : lowest;
    }
    if (!id.active) return;

    DecodeLane s;
    s.off = s.rd.start(a.bytes, a.last_word, begin + a.bytes_skew, lowest + a.bytes_skew);
    s.low = 0;
    s.span = 0;                        // span modulo 2^32: 0 is the full range (see RangeEncoder)
    s.colp = (lds_char *)(rows + 2 * tid);
    s.lutoff = DecodeLayout<BS, OUT>::kQuot - 2 * tid;
    s.osym = nullptr;
    s.ovoff = 0;
    s.anchor = 0.0f;
    s.phase = 0;
    if (OUT == OUT_SYMBOLS) {
        s.osym = a.out_sym + id.row * a.o0 + id.t0 * a.o1 + id.ch * a.o2;
    } else {
        const int64_t h = (uint32_t)id.ch / (uint32_t)a.D;     // both fit 32 bits
        const int64_t first_row = l * a.ol + kvi * a.okv + id.t0 * a.ot;             // uniform over the block
        const uint32_t fr_lo = __builtin_amdgcn_readfirstlane((uint32_t)first_row);
        const uint32_t fr_hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)first_row >> 32));
        s.orsrc = __builtin_amdgcn_make_buffer_rsrc((void *)(a.out_kv + (int64_t)(((uint64_t)fr_hi << 32) | fr_lo)), 0,
                                                    (int)0xFFFFFFFFu, kBufferWord3);
        s.ovoff = (uint32_t)((h * a.oh + (id.ch - h * a.D)) * 2);                    // the host checks that this fits
    }
    lds_f32 *rmp = (lds_f32 *)rowmax;

    // all three conditions are uniform over the block
    const bool safe = OUT == OUT_SYMBOLS || LOG2 < 0 || special || a.delta_group > 0 || nsym > lp - 2;
    const bool last_round = linear_block() >= a.last_round_first;
    if (safe) decode_lane<BS, LOG2, OUT, 0, true>(a, s, lp, id.n, rmp, last_round);
    else if (LOG2 > 1 && nsym <= (1 << (LOG2 > 1 ? LOG2 - 1 : 0))) decode_lane<BS, LOG2, OUT, 1, false>(a, s, lp, id.n, rmp, last_round);
    else decode_lane<BS, LOG2, OUT, 0, false>(a, s, lp, id.n, rmp, last_round);
}

}  // namespace
