/*
 * cachegen_oracle.c -- CPU restatement of the CacheGen KV codec arithmetic.
 *
 * THIS FILE IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are
 * compared against (tests/, __graft_entry__.smoke(), bench.py's cpu_baseline
 * leg).  Nothing in the product package may import, link or call it.
 *
 * Every function states the reference lines it restates.  Short names used
 * in the citations (all below LMCache/ in the reference tree):
 *   enc_new.cu  = third_party/torchac_cuda/torchac_kernel_enc_new.cu
 *   dec_new.cu  = third_party/torchac_cuda/torchac_kernel_dec_new.cu
 *   cal_cdf.cu  = third_party/torchac_cuda/cal_cdf.cu
 *   encoder.py  = lmcache/storage_backend/serde/cachegen_encoder.py
 *   decoder.py  = lmcache/storage_backend/serde/cachegen_decoder.py
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   quantize / dequantize : hand known-answers, closed form evaluated with
 *                           torch CPU float32 ops and numpy float16 casts.
 *   calculate_cdf         : hand known-answer, numpy bincount/cumsum with
 *                           Python integers, monotonicity invariants.
 *   encode / decode       : hand known-answers (E1/E2/E3 paths), the
 *                           prefix-code closed form for dyadic CDFs, exact
 *                           rational interval containment, an independent
 *                           bit-serial Python-integer coder, round trips.
 * The reference holds no golden vectors for this path and its CUDA sources
 * cannot be compiled in this image (no nvcc, ATen/CUDA headers), so there is
 * no oracle/_ref build.
 *
 * Build: make -C oracle   (gcc -O2 -ffp-contract=off -fopenmp)
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <math.h>

#define CGO_DT_F16 0
#define CGO_DT_BF16 1

/* ------------------------------------------------------------------------ */
/* 16-bit float formats <-> float32, written out so no compiler support for  */
/* _Float16 is needed.  Conversions to 16 bits round to nearest even, which  */
/* is what torch's .to(float16) / .to(bfloat16) do (decoder.py:171-173).     */
/* ------------------------------------------------------------------------ */
static float bits_to_float(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t float_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

float cgo_half_to_float(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_to_float(sign);
        /* subnormal: value = man * 2^-24 */
        float v = (float)man * (1.0f / 16777216.0f);
        return sign ? -v : v;
    }
    if (exp == 31) return bits_to_float(sign | 0x7F800000u | (man << 13));
    return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

uint16_t cgo_float_to_half(float f)
{
    uint32_t u = float_to_bits(f);
    uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) {                 /* inf / nan */
        if (a == 0x7F800000u) return sign | 0x7C00u;
        return sign | 0x7E00u | (uint16_t)((a >> 13) & 0x3FFu);
    }
    if (a >= 0x477FF000u) return sign | 0x7C00u;   /* >= 65520 rounds to inf */
    if (a < 0x33000001u) return sign;              /* <= 2^-25 rounds to zero */
    int e = (int)(a >> 23) - 127;
    uint32_t man = (a & 0x7FFFFFu) | 0x800000u;     /* 24-bit significand */
    int shift;                                      /* bits dropped from man */
    uint32_t base;
    if (e < -14) { shift = 13 + (-14 - e); base = 0; }
    else { shift = 13; base = (uint32_t)(e + 15) << 10; man &= 0x7FFFFFu; }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return sign | (uint16_t)(base + q);             /* carry into exponent is correct */
}

float cgo_bf16_to_float(uint16_t b) { return bits_to_float((uint32_t)b << 16); }

uint16_t cgo_float_to_bf16(float f)
{
    uint32_t u = float_to_bits(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);  /* quiet nan */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

static float load16(const uint16_t *p, int dt)
{
    return dt == CGO_DT_BF16 ? cgo_bf16_to_float(*p) : cgo_half_to_float(*p);
}
static uint16_t store16(float f, int dt)
{
    return dt == CGO_DT_BF16 ? cgo_float_to_bf16(f) : cgo_float_to_half(f);
}

/* ------------------------------------------------------------------------ */
/* Quantization: torch_quant_vectorized, encoder.py:42-59.                   */
/*   MAX    = bins // 2 - 1                      (float32 per layer)         */
/*   max1   = amax(|x|) over the channels of one (layer, token) row, kept in */
/*            the input's 16-bit dtype (a row with NaNs: see below)          */
/*   factor = MAX / max1                         (float32 divide)            */
/*   sym    = round_half_even(x * factor + MAX)  (float32 mul, then add)     */
/*            cast to int8.  A NaN (all-zero row: 0 * inf) casts to 0.       */
/* x is [nl, nt, nc] with element strides (sl, st, 1); sym is contiguous.    */
/* ------------------------------------------------------------------------ */
void cgo_quantize(const uint16_t *x, int dt, int64_t nl, int64_t nt, int64_t nc,
                  int64_t sl, int64_t st, const float *bins,
                  uint8_t *sym, uint16_t *max_out)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t l = 0; l < nl; l++) {
        for (int64_t t = 0; t < nt; t++) {
            const uint16_t *row = x + l * sl + t * st;
            const float maxq = floorf(bins[l] / 2.0f) - 1.0f;
            /* |x| of a 16-bit float is its bit pattern without the sign, and for patterns
             * that are not NaN the order of the patterns as integers is the order of the
             * values, so amax(|x|) is the largest sign-stripped pattern.  A NaN in the row
             * makes amax NaN (torch propagates it) without saying which payload survives
             * when the row holds several: the rule here is the largest pattern, which is
             * a NaN whenever the row has one (every NaN pattern is above infinity's). */
            uint16_t mbits = 0;
            for (int64_t c = 0; c < nc; c++) {
                const uint16_t a = row[c] & 0x7FFFu;
                if (a > mbits) mbits = a;
            }
            max_out[l * nt + t] = mbits;
            const float mval = load16(&mbits, dt);
            const float factor = maxq / mval;
            uint8_t *out = sym + (l * nt + t) * nc;
            for (int64_t c = 0; c < nc; c++) {
                float v = load16(row + c, dt);
                float p = v * factor;
                float s = p + maxq;
                float r = rintf(s);            /* default rounding mode: half to even */
                out[c] = (r != r) ? 0 : (uint8_t)(int8_t)(int)r;
            }
        }
    }
}

/* ------------------------------------------------------------------------ */
/* Dequantization: do_dequantize, decoder.py:24-34, then the 16-bit cast of  */
/* decoder.py:171-173.  Three separately rounded float32 operations:         */
/*   t = sym - C ; t = t / C ; t = t * max          with C = bins // 2 - 1   */
/* sym [nl, nt, nc] contiguous uint8; maxima [nl, nt] in dtype max_dt; out   */
/* [nl, nt, nc] with strides (ol, ot, 1) in dtype out_dt.                    */
/* ------------------------------------------------------------------------ */
void cgo_dequantize(const uint8_t *sym, int64_t nl, int64_t nt, int64_t nc,
                    const float *bins, const uint16_t *maxima, int max_dt,
                    uint16_t *out, int64_t ol, int64_t ot, int out_dt)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t l = 0; l < nl; l++) {
        for (int64_t t = 0; t < nt; t++) {
            const float cq = floorf(bins[l] / 2.0f) - 1.0f;
            const float m = load16(maxima + l * nt + t, max_dt);
            const uint8_t *s = sym + (l * nt + t) * nc;
            uint16_t *o = out + l * ol + t * ot;
            for (int64_t c = 0; c < nc; c++) {
                float v = (float)s[c];
                v = v - cq;
                v = v / cq;
                v = v * m;
                o[c] = store16(v, out_dt);
            }
        }
    }
}

/* ------------------------------------------------------------------------ */
/* Delta-against-anchor variant of the two functions above.  It has NO         */
/* counterpart in the reference (its snapshot holds no anchor/delta code), so  */
/* there is no parity target: this is the definition the HIP path is checked   */
/* against, pinned by a hand known-answer, by "group = 0 or 1 gives the plain  */
/* functions" and by the reconstruction bound.  Tokens are taken in sub-chunks */
/* of 256; inside a sub-chunk they form groups of `group`; the first row of a  */
/* group (the anchor) is quantized as is, every other row as d = x - x_anchor  */
/* in float32, with max|d| rounded to the 16-bit format (kept finite) and the  */
/* symbols clamped to [0, 2*MAX].  Dequantization adds the anchor's float32    */
/* reconstruction back before the 16-bit cast.                                 */
/* ------------------------------------------------------------------------ */
void cgo_quantize_delta(const uint16_t *x, int dt, int64_t nl, int64_t nt, int64_t nc,
                        int64_t sl, int64_t st, const float *bins, int group,
                        uint8_t *sym, uint16_t *max_out)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t l = 0; l < nl; l++) {
        for (int64_t t = 0; t < nt; t++) {
            const int64_t w = t % 256;
            const int64_t ta = t - (w % group);
            const uint16_t *row = x + l * sl + t * st;
            const uint16_t *arow = x + l * sl + ta * st;
            const float maxq = floorf(bins[l] / 2.0f) - 1.0f;
            float m = 0.0f;
            for (int64_t c = 0; c < nc; c++) {
                float v = load16(row + c, dt);
                float va = (ta == t) ? 0.0f : load16(arow + c, dt);
                float d = fabsf(v - va);
                if (d > m) m = d;               /* NaN differences are ignored, like fmaxf */
            }
            uint16_t m16 = store16(m, dt);
            const uint16_t inf16 = dt == CGO_DT_BF16 ? 0x7F80u : 0x7C00u;
            if (m16 >= inf16) m16 = (uint16_t)(inf16 - 1);
            max_out[l * nt + t] = m16;
            const float factor = maxq / load16(&m16, dt);
            const float top = maxq + maxq;
            uint8_t *out = sym + (l * nt + t) * nc;
            for (int64_t c = 0; c < nc; c++) {
                float v = load16(row + c, dt);
                float va = (ta == t) ? 0.0f : load16(arow + c, dt);
                float d = v - va;
                float p = d * factor;
                float s = p + maxq;
                float r = rintf(s);
                if (r != r) r = 0.0f;
                if (r < 0.0f) r = 0.0f;
                if (r > top) r = top;
                out[c] = (uint8_t)(int)r;
            }
        }
    }
}

void cgo_dequantize_delta(const uint8_t *sym, int64_t nl, int64_t nt, int64_t nc,
                          const float *bins, const uint16_t *maxima, int max_dt, int group,
                          uint16_t *out, int64_t ol, int64_t ot, int out_dt)
{
#pragma omp parallel for schedule(static)
    for (int64_t l = 0; l < nl; l++) {
        const float cq = floorf(bins[l] / 2.0f) - 1.0f;
        for (int64_t c = 0; c < nc; c++) {
            float anchor = 0.0f;
            for (int64_t t = 0; t < nt; t++) {
                const float m = load16(maxima + l * nt + t, max_dt);
                float v = (float)sym[(l * nt + t) * nc + c];
                v = v - cq;
                v = v / cq;
                v = v * m;
                if ((t % 256) % group == 0) anchor = v;
                else v = v + anchor;
                out[l * ol + t * ot + c] = store16(v, out_dt);
            }
        }
    }
}

/* ------------------------------------------------------------------------ */
/* CDF: calculate_cdf_kernel + normalize_cdf_value, cal_cdf.cu:11-14,29-49.  */
/* Per (layer, channel): 16-bit counters hist[sym+1]++ over all tokens, an   */
/* inclusive running sum, then                                               */
/*   cdf[i] = (uint16)((0xFFFF - max_bins) * cum[i] / cum[max_bins]) + i     */
/* in 32-bit unsigned arithmetic with a truncating divide.  The 16-bit       */
/* counters wrap exactly as the reference's do.  sym is [nl, nt, nc] with    */
/* element strides (s0, s1, s2); cdf is [nl, nc, max_bins+1] contiguous.     */
/* ------------------------------------------------------------------------ */
void cgo_calculate_cdf(const uint8_t *sym, int64_t nl, int64_t nt, int64_t nc,
                       int64_t s0, int64_t s1, int64_t s2, int max_bins,
                       uint16_t *cdf)
{
    const int lp = max_bins + 1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t l = 0; l < nl; l++) {
        for (int64_t c = 0; c < nc; c++) {
            uint16_t hist[260];
            for (int i = 0; i <= max_bins; i++) hist[i] = 0;
            for (int64_t t = 0; t < nt; t++) {
                uint8_t v = sym[l * s0 + t * s1 + c * s2];
                if ((int)v + 1 <= max_bins) hist[v + 1]++;   /* out-of-table symbols are a caller error */
            }
            uint16_t running = 0;
            for (int i = 0; i < max_bins; i++) {
                uint16_t v = hist[i + 1];
                hist[i + 1] = (uint16_t)(hist[i + 1] + running);
                running = (uint16_t)(running + v);
            }
            const uint32_t scale = 0xFFFFu - (uint32_t)max_bins;
            uint16_t *o = cdf + (l * nc + c) * lp;
            for (int i = 0; i <= max_bins; i++) {
                uint16_t q = running ? (uint16_t)(scale * (uint32_t)hist[i] / (uint32_t)running) : 0;
                o[i] = (uint16_t)(q + i);
            }
        }
    }
}

/* ------------------------------------------------------------------------ */
/* Bit output of the encoder: spill_reg_to_shared, spill_partial_reg_to_     */
/* shared, add_bits_to_output, append_bit_and_pending (enc_new.cu:21-97).    */
/* Bits enter a 32-bit register MSB-first; a full register is written as 4   */
/* big-endian bytes.  A run of exactly 32 equal bits into an empty register  */
/* is written as 0x00000000 / 0xFFFFFFFF: the reference shifts by 32 there,  */
/* which its hardware clamps to that result.  Bytes past `cap` are counted   */
/* but not stored.                                                           */
/* ------------------------------------------------------------------------ */
typedef struct {
    uint8_t *buf;
    int cap;
    int len;
    uint32_t reg;
    int reg_len;
} bit_sink;

static void sink_byte(bit_sink *s, uint8_t b)
{
    if (s->len < s->cap) s->buf[s->len] = b;
    s->len++;
}

static void sink_run(bit_sink *s, uint32_t bit, uint64_t num)
{
    do {
        int room = 32 - s->reg_len;
        int take = (num < (uint64_t)room) ? (int)num : room;
        if (take == 32) s->reg = bit ? 0xFFFFFFFFu : 0u;
        else s->reg = (s->reg << take) | ((bit << take) - bit);
        num -= (uint64_t)take;
        s->reg_len += take;
        if (s->reg_len == 32) {
            sink_byte(s, (uint8_t)(s->reg >> 24));
            sink_byte(s, (uint8_t)(s->reg >> 16));
            sink_byte(s, (uint8_t)(s->reg >> 8));
            sink_byte(s, (uint8_t)(s->reg));
            s->reg = 0;
            s->reg_len = 0;
        }
    } while (num > 0);
}

static void sink_bit_and_pending(bit_sink *s, uint32_t bit, uint64_t *pending)
{
    sink_run(s, bit, 1);
    sink_run(s, 1u - bit, *pending);
    *pending = 0;
}

static void sink_finish(bit_sink *s)
{
    if (s->reg_len > 0) {
        uint32_t r = s->reg << (32 - s->reg_len);
        int n = s->reg_len;
        while (n > 0) {
            n -= 8;
            sink_byte(s, (uint8_t)(r >> 24));
            r <<= 8;
        }
        s->reg_len = 0;
    }
}

/* ------------------------------------------------------------------------ */
/* One stream of the encoder: encode_with_accessor_kernel, enc_new.cu:       */
/* 253-307.  cdf is one row of `lp` uint16 values; symbol i is sym[i*stride].*/
/* Returns the stream's length in bytes; at most `cap` bytes are stored.     */
/* ------------------------------------------------------------------------ */
int cgo_encode_stream(const uint16_t *cdf, int lp, const uint8_t *sym,
                      int64_t stride, int n, uint8_t *out, int cap)
{
    uint32_t low = 0, high = 0xFFFFFFFFu;
    uint64_t pending = 0;
    const int max_symbol = lp - 2;
    bit_sink s = { out, cap, 0, 0, 0 };

    for (int i = 0; i < n; i++) {
        const int v = sym[(int64_t)i * stride];
        const uint64_t span = (uint64_t)high - (uint64_t)low + 1;
        const uint32_t c_low = cdf[v];
        const uint32_t c_high = (v == max_symbol) ? 0x10000u : cdf[v + 1];
        high = (low - 1u) + (uint32_t)((span * (uint64_t)c_high) >> 16);
        low = low + (uint32_t)((span * (uint64_t)c_low) >> 16);
        for (;;) {
            if (high < 0x80000000u) {
                sink_bit_and_pending(&s, 0, &pending);
                low <<= 1; high <<= 1; high |= 1u;
            } else if (low >= 0x80000000u) {
                sink_bit_and_pending(&s, 1, &pending);
                low <<= 1; high <<= 1; high |= 1u;
            } else if (low >= 0x40000000u && high < 0xC0000000u) {
                pending++;
                low <<= 1; low &= 0x7FFFFFFFu;
                high <<= 1; high |= 0x80000001u;
            } else break;
        }
    }
    pending += 1;
    sink_bit_and_pending(&s, low < 0x40000000u ? 0u : 1u, &pending);
    sink_finish(&s);
    return s.len;
}

/* ------------------------------------------------------------------------ */
/* Symbol search of the decoder: binsearch, dec_new.cu:52-71 (same probes,   */
/* early return on equality).                                                */
/* ------------------------------------------------------------------------ */
static int search_symbol(const uint16_t *cdf, uint16_t target, int max_sym)
{
    int left = 0, right = max_sym + 1;
    while (left + 1 < right) {
        int m = (left + right) / 2;
        uint16_t v = cdf[m];
        if (v < target) left = m;
        else if (v > target) right = m;
        else return m;
    }
    return left;
}

/* ------------------------------------------------------------------------ */
/* One stream of the decoder: decode_prefix_with_accessor_kernel, dec_new.cu */
/* 248-302 (identical loop in decode_with_accessor_kernel, :131-185).  The   */
/* stream is read as if followed by zero bytes (the reference zero-pads each */
/* stream to 256 bytes in shared memory, dec_new.cu:223-233).  The range is  */
/* not updated after the last symbol (:273-275).                             */
/* ------------------------------------------------------------------------ */
void cgo_decode_stream(const uint16_t *cdf, int lp, const uint8_t *bytes, int len,
                       int n, uint8_t *out, int64_t stride)
{
    uint32_t low = 0, high = 0xFFFFFFFFu, value = 0;
    const int max_symbol = lp - 2;
    int pos = 0;                 /* next byte to load into byte_buffer */
    uint8_t byte_buffer;
    int bit_idx = 1;
#define CGO_BYTE(k) ((k) < len ? bytes[(k)] : (uint8_t)0)
    value = ((uint32_t)CGO_BYTE(0) << 24) | ((uint32_t)CGO_BYTE(1) << 16) |
            ((uint32_t)CGO_BYTE(2) << 8) | (uint32_t)CGO_BYTE(3);
    pos = 4;
    byte_buffer = CGO_BYTE(pos);

    for (int i = 0; i < n; i++) {
        const uint64_t span = (uint64_t)high - (uint64_t)low + 1;
        const uint16_t count = (uint16_t)((((uint64_t)value - (uint64_t)low + 1) * 0x10000u - 1) / span);
        const int s = search_symbol(cdf, count, max_symbol);
        out[(int64_t)i * stride] = (uint8_t)s;
        if (i == n - 1) break;
        const uint32_t c_low = cdf[s];
        const uint32_t c_high = (s == max_symbol) ? 0x10000u : cdf[s + 1];
        high = (low - 1u) + (uint32_t)((span * (uint64_t)c_high) >> 16);
        low = low + (uint32_t)((span * (uint64_t)c_low) >> 16);
        for (;;) {
            int shift = 0;
            if (low >= 0x80000000u || high < 0x80000000u) {
                low <<= 1; high <<= 1; high |= 1u;
                shift = 1;
            } else if (low >= 0x40000000u && high < 0xC0000000u) {
                low <<= 1; low &= 0x7FFFFFFFu;
                high <<= 1; high |= 0x80000001u;
                value -= 0x40000000u;
                shift = 1;
            }
            if (!shift) break;
            value = (value << 1) | ((uint32_t)(byte_buffer >> (8 - bit_idx)) & 1u);
            bit_idx++;
            if (bit_idx == 9) { bit_idx = 1; pos++; byte_buffer = CGO_BYTE(pos); }
        }
    }
#undef CGO_BYTE
}

/* ------------------------------------------------------------------------ */
/* Batched forms with the tensor shapes of the reference's entry points.     */
/* ------------------------------------------------------------------------ */

/* encode_cuda_new, enc_new.cu:355-451: cdf [nl, nc, lp] contiguous, sym
 * [nl, nt, nc] with element strides, out [nl, nc, cap] contiguous (bytes past
 * a stream's length are left as they were), lengths [nl, nc] int32. */
void cgo_encode_fast_new(const uint16_t *cdf, int lp, const uint8_t *sym,
                         int64_t nl, int64_t nt, int64_t nc,
                         int64_t s0, int64_t s1, int64_t s2,
                         uint8_t *out, int cap, int32_t *lengths)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t l = 0; l < nl; l++)
        for (int64_t c = 0; c < nc; c++)
            lengths[l * nc + c] = cgo_encode_stream(
                cdf + (l * nc + c) * lp, lp, sym + l * s0 + c * s2, s1, (int)nt,
                out + (l * nc + c) * (int64_t)cap, cap);
}

/* collect_bytes, encoder.py:209-222: concatenate the streams of a padded
 * buffer in (layer, channel) order.  Returns the number of bytes written. */
int64_t cgo_collect_bytes(const uint8_t *padded, int cap, const int32_t *lengths,
                          int64_t nstreams, uint8_t *out)
{
    int64_t pos = 0;
    for (int64_t i = 0; i < nstreams; i++) {
        int n = lengths[i] < cap ? lengths[i] : cap;
        memcpy(out + pos, padded + i * (int64_t)cap, (size_t)n);
        pos += n;
    }
    return pos;
}

/* decode_cuda_prefsum, dec_new.cu:403-479: stream g = l*nc + c occupies
 * bytes [prefix[g-1], prefix[g]) of `bytes` (0 for g = 0); prefix is the
 * INCLUSIVE int64 running sum of the lengths (decoder.py:70).  out is
 * [nl, nt, nc] uint8 with element strides. */
void cgo_decode_fast_prefsum(const uint16_t *cdf, int lp, const uint8_t *bytes,
                             const int64_t *prefix, int64_t nl, int64_t nt, int64_t nc,
                             uint8_t *out, int64_t o0, int64_t o1, int64_t o2)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t l = 0; l < nl; l++)
        for (int64_t c = 0; c < nc; c++) {
            int64_t g = l * nc + c;
            int64_t begin = g ? prefix[g - 1] : 0;
            int64_t end = prefix[g];
            cgo_decode_stream(cdf + g * lp, lp, bytes + begin, (int)(end - begin),
                              (int)nt, out + l * o0 + c * o2, o1);
        }
}

/* decode_cuda_new, dec_new.cu:314-393: streams come from the padded
 * [nl, nc, cap] buffer with raw int32 lengths. */
void cgo_decode_fast_new(const uint16_t *cdf, int lp, const uint8_t *padded, int cap,
                         const int32_t *lengths, int64_t nl, int64_t nt, int64_t nc,
                         uint8_t *out, int64_t o0, int64_t o1, int64_t o2)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t l = 0; l < nl; l++)
        for (int64_t c = 0; c < nc; c++) {
            int64_t g = l * nc + c;
            int n = lengths[g] < cap ? lengths[g] : cap;
            cgo_decode_stream(cdf + g * lp, lp, padded + g * (int64_t)cap, n,
                              (int)nt, out + l * o0 + c * o2, o1);
        }
}

int cgo_max_threads(void);
void cgo_set_threads(int n);
#ifdef _OPENMP
#include <omp.h>
int cgo_max_threads(void) { return omp_get_max_threads(); }
void cgo_set_threads(int n) { omp_set_num_threads(n); }
#else
int cgo_max_threads(void) { return 1; }
void cgo_set_threads(int n) { (void)n; }
#endif
