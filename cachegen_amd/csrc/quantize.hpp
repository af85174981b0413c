// Part of the CacheGen KV codec library for MI355X (gfx950); included by cachegen_hip.hip, which
// is the one translation unit.  Quantization kernels: byte symbols [2L,T,C], packed symbols of the fused path, delta-group variant.
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
// Quantization (encoder.py:42-59): one wavefront per (row of 2L, token).
// Each lane holds up to 8 units of 8 channels (one 128-bit load each) in registers, the
// row maximum of |x| is an integer maximum of the sign-stripped 16-bit patterns (two per
// packed op), and the float32 operations are the reference's, each rounded separately:
//   factor = MAX / max ; sym = rint(x * factor + MAX)
// ------------------------------------------------------------------------------------
constexpr int kMaxUnits = 8;

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b)
{
    typedef unsigned short us2 __attribute__((ext_vector_type(2)));
    us2 x, y;
    __builtin_memcpy(&x, &a, 4);
    __builtin_memcpy(&y, &b, 4);
    us2 z = __builtin_elementwise_max(x, y);
    uint32_t r;
    __builtin_memcpy(&r, &z, 4);
    return r;
}

__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v)
{
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        uint32_t other = (uint32_t)__shfl_xor((int)v, o, 64);
        v = other > v ? other : v;
    }
    return v;
}

template <int DT>
__device__ __forceinline__ uint32_t quant_one(uint32_t bits, float factor, float maxq)
{
    const float v = load16f<DT>(bits);
    const float p = __fmul_rn(v, factor);
    const float s = __fadd_rn(p, maxq);
    float r = __builtin_rintf(s);
    r = (r != r) ? 0.0f : r;          // 0 * inf of an all-zero row: int8 cast of NaN is 0
    return (uint32_t)(int)r & 0xFFu;
}

template <int DT, bool HEADS_CONTIGUOUS>
__global__ __launch_bounds__(256) void quantize_kv_kernel(
    const uint16_t *__restrict__ kv, int64_t L, int64_t T, int D, int64_t sl, int64_t skv,
    int64_t st, int64_t sh, const float *__restrict__ key_bins,
    const float *__restrict__ value_bins, uint8_t *__restrict__ sym,
    uint16_t *__restrict__ maxima, int nunits, int64_t nrows)
{
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= nrows) return;
    const int64_t layer2 = row / T, t = row - layer2 * T;
    const int64_t kvi = layer2 / L, l = layer2 - kvi * L;
    const uint16_t *base = kv + l * sl + kvi * skv + t * st;
    const float bins = (kvi ? value_bins : key_bins)[l];
    const float maxq = floorf(bins * 0.5f) - 1.0f;

    uint4 regs[kMaxUnits];
    uint32_t m = 0;
#pragma unroll
    for (int i = 0; i < kMaxUnits; ++i) {
        const int u = lane + 64 * i;
        if (u < nunits) {
            const int e = u * 8;
            int64_t off;
            if (HEADS_CONTIGUOUS) off = e;
            else { const int h = e / D; off = (int64_t)h * sh + (e - h * D); }
            regs[i] = *reinterpret_cast<const uint4 *>(base + off);
            m = pk_max_u16(m, regs[i].x & 0x7FFF7FFFu);
            m = pk_max_u16(m, regs[i].y & 0x7FFF7FFFu);
            m = pk_max_u16(m, regs[i].z & 0x7FFF7FFFu);
            m = pk_max_u16(m, regs[i].w & 0x7FFF7FFFu);
        }
    }
    m = (m & 0xFFFFu) > (m >> 16) ? (m & 0xFFFFu) : (m >> 16);
    m = wave_max_u32(m);
    if (lane == 0) maxima[row] = (uint16_t)m;
    const float factor = __fdiv_rn(maxq, load16f<DT>(m));

    uint8_t *out = sym + row * ((int64_t)nunits * 8);
#pragma unroll
    for (int i = 0; i < kMaxUnits; ++i) {
        const int u = lane + 64 * i;
        if (u < nunits) {
            const uint32_t w[4] = {regs[i].x, regs[i].y, regs[i].z, regs[i].w};
            uint32_t q[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                q[j] = quant_one<DT>(w[2 * j] & 0xFFFFu, factor, maxq) |
                       (quant_one<DT>(w[2 * j] >> 16, factor, maxq) << 8) |
                       (quant_one<DT>(w[2 * j + 1] & 0xFFFFu, factor, maxq) << 16) |
                       (quant_one<DT>(w[2 * j + 1] >> 16, factor, maxq) << 24);
            }
            *reinterpret_cast<uint2 *>(out + (int64_t)u * 8) = make_uint2(q[0], q[1]);
        }
    }
}

// Any shape / alignment: one wavefront per row, two passes over global memory.
template <int DT>
__global__ __launch_bounds__(256) void quantize_kv_generic_kernel(
    const uint16_t *__restrict__ kv, int64_t L, int64_t T, int D, int C, int64_t sl, int64_t skv,
    int64_t st, int64_t sh, const float *__restrict__ key_bins,
    const float *__restrict__ value_bins, uint8_t *__restrict__ sym,
    uint16_t *__restrict__ maxima, int64_t nrows)
{
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= nrows) return;
    const int64_t layer2 = row / T, t = row - layer2 * T;
    const int64_t kvi = layer2 / L, l = layer2 - kvi * L;
    const uint16_t *base = kv + l * sl + kvi * skv + t * st;
    const float bins = (kvi ? value_bins : key_bins)[l];
    const float maxq = floorf(bins * 0.5f) - 1.0f;
    uint32_t m = 0;
    for (int c = lane; c < C; c += 64) {
        const int h = c / D;
        const uint32_t b = base[(int64_t)h * sh + (c - h * D)] & 0x7FFFu;
        m = b > m ? b : m;
    }
    m = wave_max_u32(m);
    if (lane == 0) maxima[row] = (uint16_t)m;
    const float factor = __fdiv_rn(maxq, load16f<DT>(m));
    uint8_t *out = sym + row * (int64_t)C;
    for (int c = lane; c < C; c += 64) {
        const int h = c / D;
        out[c] = (uint8_t)quant_one<DT>(base[(int64_t)h * sh + (c - h * D)], factor, maxq);
    }
}

// ------------------------------------------------------------------------------------
// Packed symbols of the fused path.  Each (row, sub-chunk) owns a slot of 64 words per
// channel; byte j of word w is the symbol of token 4w + j of the sub-chunk:
//   sym4[((row * nsub + sub) * 64 + w) * C + channel]
// A lane of a stream kernel (one channel) gets four consecutive tokens with one 32-bit
// load and a wave reads 256 contiguous bytes.
// ------------------------------------------------------------------------------------
constexpr int kWordsPerSub = kSub / 4;

constexpr int kMaxLevels = CG_MAX_LEVELS;

struct PackedQuantArgs {
    const uint16_t *kv;
    int64_t L, sl, skv, st, sh;
    int32_t D;
    const float *key_bins, *value_bins;
    // several quantization levels from one read of the tensor (MULTI kernels): level v uses
    // key_bins_lv[v] / value_bins_lv[v] and writes its words level_words * v further on
    int32_t nlevels;
    const float *key_bins_lv[kMaxLevels], *value_bins_lv[kMaxLevels];
    int64_t level_words;
    // status words of the encode call (one per level) that this launch, the first of the call,
    // sets to zero
    int32_t nstatus;
    int32_t *status[kMaxLevels];
    uint32_t *sym4;
    uint16_t *maxima;       // [2L, T]
    int32_t nunits;         // C / 8
    int64_t nsub;
    int32_t nibbles;        // rows of at most 15 symbols are written four bits a symbol (see quantize_pack_kernel)
    int32_t lp, lp_lv[kMaxLevels];          // table length (of every level): the symbols must also fit the table
    int32_t delta_group;    // > 0: tokens of a sub-chunk in groups of this many, see below
    TokenGeom g;
};

// One wavefront quantizes four consecutive tokens of one row (encoder.py:42-59) and
// writes, per channel, one word holding the four symbols: 32 contiguous bytes per lane
// and unit, 2 KB per wave and store pair.
// MULTI: the rows are loaded and their maxima found once, then quantized at each of
// a.nlevels levels (the adaptive-streaming use: run_adaptation.py:63-72 encodes every chunk
// at QUANT_LEVEL 1..3); the maxima do not depend on the level.
__device__ __forceinline__ void clear_statuses(const PackedQuantArgs &a)
{
    if (blockIdx.x == 0 && threadIdx.x < a.nstatus) *a.status[threadIdx.x] = 0;
}

// A row quantized to `maxq` levels either side of zero has the symbols 0 .. 2 maxq: at most
// fifteen of them fit four bits with the value 15 to spare.  Where the caller asks for it
// (a.nibbles) such rows are stored four bits a symbol, word w of channel pair p (channels 2p and
// 2p + 1) of a sub-chunk at sym4[((row * nsub + sub) * 64 + w) * C + p]: half of the bytes.
// The coder does not compare four-bit symbols with the table's end, so the row's alphabet must
// also lie inside a table of `lp` entries (symbols 0 .. lp - 2); the quantizer, the table kernel
// and the coder all decide with this one function.
__device__ __forceinline__ bool narrow_alphabet(float maxq, int lp)
{
    return maxq >= 0.0f && maxq <= 7.0f && 2.0f * maxq <= (float)(lp - 2);
}

// A token row whose maximum is so small that the scale maxq / max is infinite (bfloat16 maxima
// below about 2^-125): every non-zero value of the row saturates, to the byte 255, which the
// coder keeps inside the table as the table's last symbol.  Rows of zeros do not count (0 * inf
// is a NaN, symbol 0).
__device__ __forceinline__ bool scale_overflows(float maxq, float row_max)
{
    return row_max != 0.0f && (__float_as_uint(__fdiv_rn(maxq, row_max)) & 0x7FFFFFFFu) == 0x7F800000u;
}

// The 4 x NU units (128-bit loads of 8 channels) that one lane holds of four consecutive token
// rows, and the rows' maxima (largest sign-stripped 16-bit pattern, over the whole wavefront).
// Rows j >= nvalid and units past the last channel are zeros.
template <bool HEADS_CONTIGUOUS, int NU>
__device__ __forceinline__ void load_four_rows(const uint16_t *base, int64_t st, int64_t sh, int D, int nunits,
                                               int nvalid, int lane, uint4 (&regs)[4][NU], uint32_t (&max_bits)[4])
{
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t m = 0;
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            regs[j][i] = make_uint4(0, 0, 0, 0);
            const int u = lane + 64 * i;
            if (j < nvalid && u < nunits) {
                const int e = u * 8;
                int64_t off;
                if (HEADS_CONTIGUOUS) off = e;
                else { const int h = e / D; off = (int64_t)h * sh + (e - h * D); }
                // read once and never again: loaded past the caches' keep-for-reuse policy
                typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(base + j * st + off));
                regs[j][i] = make_uint4(t.x, t.y, t.z, t.w);
                m = pk_max_u16(m, regs[j][i].x & 0x7FFF7FFFu);
                m = pk_max_u16(m, regs[j][i].y & 0x7FFF7FFFu);
                m = pk_max_u16(m, regs[j][i].z & 0x7FFF7FFFu);
                m = pk_max_u16(m, regs[j][i].w & 0x7FFF7FFFu);
            }
        }
        m = (m & 0xFFFFu) > (m >> 16) ? (m & 0xFFFFu) : (m >> 16);
        max_bits[j] = wave_max_u32(m);
    }
}

// The symbols of one unit: word k holds channel k's four tokens, a byte each.
template <int DT>
__device__ __forceinline__ void quantize_unit(const uint4 (&r)[4], const float (&factor)[4], float maxq, uint32_t (&words)[8])
{
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        uint32_t w = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t src = k < 2 ? r[j].x : k < 4 ? r[j].y : k < 6 ? r[j].z : r[j].w;
            const uint32_t bits = (k & 1) ? (src >> 16) : (src & 0xFFFFu);
            const float v = load16f<DT>(bits);
            const float s = __fadd_rn(__fmul_rn(v, factor[j]), maxq);
            // the conversion itself rounds to nearest even, turns a NaN (0 * inf of an
            // all-zero row) and anything negative into 0 and saturates at 255: the
            // round-half-even, int8 cast and NaN rule of encoder.py:56-57 in one step
            w = __builtin_amdgcn_cvt_pk_u8_f32(s, (uint32_t)j, w);
        }
        words[k] = w;
    }
}

// Four bits a symbol: channels 2k and 2k + 1 share word k of the unit, the even channel's four
// tokens in its lower half.  A saturated byte (255) becomes 15, which no symbol of such a row is:
// the coder gives it its meaning back.
__device__ __forceinline__ uint4 pack_four_bit_words(const uint32_t (&words)[8])
{
    uint32_t half[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        uint32_t e = words[2 * k] & 0x0F0F0F0Fu, o = words[2 * k + 1] & 0x0F0F0F0Fu;
        e |= e >> 4;                                    // bytes 0 and 2 hold two symbols each
        o |= o >> 4;
        half[k] = __builtin_amdgcn_perm(o, e, 0x06040200u);          // e.b0, e.b2, o.b0, o.b2
    }
    return make_uint4(half[0], half[1], half[2], half[3]);
}

template <int DT, bool HEADS_CONTIGUOUS, int NU, bool MULTI = false>
__global__ __launch_bounds__(256) void quantize_pack_kernel(PackedQuantArgs a)
{
    clear_statuses(a);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int64_t b = blockIdx.x;
    const int tq = (int)(b & 15) * 4 + wave;      // word index inside the sub-chunk slot
    b >>= 4;
    const int64_t sub = b % a.nsub;
    const int64_t row = b / a.nsub;
    int64_t chunk, t0;
    int n;
    sub_range(a.g, sub, chunk, t0, n);
    const int tt0 = tq * 4;
    if (tt0 >= n) return;
    const int nvalid = (n - tt0) < 4 ? (n - tt0) : 4;
    const int64_t kvi = row / a.L, l = row - kvi * a.L;
    const uint16_t *base = a.kv + l * a.sl + kvi * a.skv + (t0 + tt0) * a.st;

    uint4 regs[4][NU];
    uint32_t max_bits[4];
    float rowmax[4];
    load_four_rows<HEADS_CONTIGUOUS, NU>(base, a.st, a.sh, a.D, a.nunits, nvalid, lane, regs, max_bits);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (j < nvalid && lane == 0) a.maxima[row * a.g.T + t0 + tt0 + j] = (uint16_t)max_bits[j];
        rowmax[j] = load16f<DT>(max_bits[j]);
    }

    const int64_t C = (int64_t)a.nunits * 8;
    uint32_t *out = a.sym4 + ((row * a.nsub + sub) * kWordsPerSub + tq) * C;
    const int nlevels = MULTI ? a.nlevels : 1;
    for (int lv = 0; lv < nlevels; ++lv, out += a.level_words) {
        const float bins = MULTI ? (kvi ? a.value_bins_lv[lv] : a.key_bins_lv[lv])[l] : (kvi ? a.value_bins : a.key_bins)[l];
        const float maxq = floorf(bins * 0.5f) - 1.0f;
        const bool narrow = a.nibbles && narrow_alphabet(maxq, MULTI ? a.lp_lv[lv] : a.lp);
        float factor[4];
        // rows past the end of the sub-chunk are all zero: 0 * inf = NaN -> symbol byte 0
#pragma unroll
        for (int j = 0; j < 4; ++j) factor[j] = __fdiv_rn(maxq, rowmax[j]);
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            const int u = lane + 64 * i;
            if (u < a.nunits) {
                uint32_t words[8];
                const uint4 r[4] = {regs[0][i], regs[1][i], regs[2][i], regs[3][i]};
                quantize_unit<DT>(r, factor, maxq, words);
                if (narrow) {
                    *reinterpret_cast<uint4 *>(out + (int64_t)u * 4) = pack_four_bit_words(words);
                } else {
                    uint4 *dst = reinterpret_cast<uint4 *>(out + (int64_t)u * 8);
                    dst[0] = make_uint4(words[0], words[1], words[2], words[3]);
                    dst[1] = make_uint4(words[4], words[5], words[6], words[7]);
                }
            }
        }
    }
}

// Delta-against-anchor variant (no counterpart in the reference, off by default).  Inside
// every sub-chunk the tokens form groups of `delta_group`; the first token of a group is its
// anchor and is quantized as above, every other row is replaced by d = x - x_anchor
// (float32) before the same quantization, with the row maximum of |d| rounded to the 16-bit
// input format and symbols clamped to the table.  The decoder adds the reconstructed anchor
// back.  Rows are handled one after the other so that registers hold one row, its anchor
// and the packed result.
template <int DT, bool HEADS_CONTIGUOUS, int NU>
__global__ __launch_bounds__(256) void quantize_pack_delta_kernel(PackedQuantArgs a)
{
    clear_statuses(a);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    int64_t b = blockIdx.x;
    const int tq = (int)(b & 15) * 4 + wave;
    b >>= 4;
    const int64_t sub = b % a.nsub;
    const int64_t row = b / a.nsub;
    int64_t chunk, t0;
    int n;
    sub_range(a.g, sub, chunk, t0, n);
    const int tt0 = tq * 4;
    if (tt0 >= n) return;
    const int nvalid = (n - tt0) < 4 ? (n - tt0) : 4;
    const int64_t kvi = row / a.L, l = row - kvi * a.L;
    const float bins = (kvi ? a.value_bins : a.key_bins)[l];
    const float maxq = floorf(bins * 0.5f) - 1.0f;
    const uint16_t *base = a.kv + l * a.sl + kvi * a.skv + t0 * a.st;     // token 0 of the sub-chunk

    uint32_t words[NU][8];
#pragma unroll
    for (int i = 0; i < NU; ++i)
#pragma unroll
        for (int k = 0; k < 8; ++k) words[i][k] = 0;

    for (int j = 0; j < nvalid; ++j) {
        const int tt = tt0 + j;
        const int ta = tt - tt % a.delta_group;          // the group's anchor
        const bool is_anchor = ta == tt;
        uint4 x[NU], xa[NU];
        float m = 0.0f;
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            x[i] = make_uint4(0, 0, 0, 0);
            xa[i] = make_uint4(0, 0, 0, 0);
            const int u = lane + 64 * i;
            if (u < a.nunits) {
                const int e = u * 8;
                int64_t off;
                if (HEADS_CONTIGUOUS) off = e;
                else { const int h = e / a.D; off = (int64_t)h * a.sh + (e - h * a.D); }
                x[i] = *reinterpret_cast<const uint4 *>(base + tt * a.st + off);
                if (!is_anchor) xa[i] = *reinterpret_cast<const uint4 *>(base + ta * a.st + off);
                const uint32_t xs[4] = {x[i].x, x[i].y, x[i].z, x[i].w};
                const uint32_t as[4] = {xa[i].x, xa[i].y, xa[i].z, xa[i].w};
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const float v = load16f<DT>((k & 1) ? xs[k >> 1] >> 16 : xs[k >> 1] & 0xFFFFu);
                    const float va = is_anchor ? 0.0f : load16f<DT>((k & 1) ? as[k >> 1] >> 16 : as[k >> 1] & 0xFFFFu);
                    m = fmaxf(m, fabsf(__fsub_rn(v, va)));
                }
            }
        }
        m = __uint_as_float(wave_max_u32(__float_as_uint(m)));   // non-negative floats order as integers
        uint32_t m16 = store16f<DT>(m);
        const uint32_t inf16 = DT == CG_DT_BF16 ? 0x7F80u : 0x7C00u;
        if (m16 >= inf16) m16 = inf16 - 1;                        // keep the stored maximum finite
        if (lane == 0) a.maxima[row * a.g.T + t0 + tt] = (uint16_t)m16;
        const float factor = __fdiv_rn(maxq, load16f<DT>(m16));
        const float top = __fadd_rn(maxq, maxq);
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            const uint32_t xs[4] = {x[i].x, x[i].y, x[i].z, x[i].w};
            const uint32_t as[4] = {xa[i].x, xa[i].y, xa[i].z, xa[i].w};
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float v = load16f<DT>((k & 1) ? xs[k >> 1] >> 16 : xs[k >> 1] & 0xFFFFu);
                const float va = is_anchor ? 0.0f : load16f<DT>((k & 1) ? as[k >> 1] >> 16 : as[k >> 1] & 0xFFFFu);
                const float d = __fsub_rn(v, va);
                const float sv = __fadd_rn(__fmul_rn(d, factor), maxq);
                const float r = fminf(fmaxf(__builtin_rintf(sv), 0.0f), top);    // NaN -> 0, clamp to the table
                words[i][k] |= ((uint32_t)(int)r & 0xFFu) << (8 * j);
            }
        }
    }

    const int64_t C = (int64_t)a.nunits * 8;
    uint32_t *out = a.sym4 + ((row * a.nsub + sub) * kWordsPerSub + tq) * C;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
        const int u = lane + 64 * i;
        if (u < a.nunits) {
            uint4 *dst = reinterpret_cast<uint4 *>(out + (int64_t)u * 8);
            dst[0] = make_uint4(words[i][0], words[i][1], words[i][2], words[i][3]);
            dst[1] = make_uint4(words[i][4], words[i][5], words[i][6], words[i][7]);
        }
    }
}

}  // namespace
