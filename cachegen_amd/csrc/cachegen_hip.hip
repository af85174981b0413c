// CacheGen KV codec for MI355X (gfx950): hand-written HIP kernels behind a C ABI.
//
// The codec is HBM/ALU-bound integer work with no dense contraction, so there is
// no MFMA here.  The mapping everywhere is one lane = one (row, channel) stream
// and one wavefront = 64 adjacent channels of one row, which keeps every symbol
// and KV access of a wave on one contiguous segment; per-wave tables live in LDS
// as [entry][lane] 32-bit words so that lanes never collide on a bank.
//
// Paths in the comments are relative to LMCache/ in the reference tree:
//   enc_new.cu = third_party/torchac_cuda/torchac_kernel_enc_new.cu
//   dec_new.cu = third_party/torchac_cuda/torchac_kernel_dec_new.cu
//   cal_cdf.cu = third_party/torchac_cuda/cal_cdf.cu
//   encoder.py = lmcache/storage_backend/serde/cachegen_encoder.py
//   decoder.py = lmcache/storage_backend/serde/cachegen_decoder.py
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "cachegen_hip.h"

// The float32 steps of quantisation and dequantisation are rounded one by one, as eager
// tensor code rounds them: no fused multiply-add anywhere in this file.
#pragma clang fp contract(off)

namespace {

// ------------------------------------------------------------------------------------
// host-side helpers
// ------------------------------------------------------------------------------------
thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char *what)
{
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(CG_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
    return CG_OK;
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

constexpr int kSub = CG_MAX_TOKENS_PER_STREAM;   // tokens per stream (cachegen_basics.py:8)
constexpr int kStreamCap = 256;                  // bytes kept per stream in the fused path

// Token geometry shared by the stream kernels: chunk k covers tokens
// [k*S, min((k+1)*S, T)), and is cut every 256 tokens (encoder.py:279-292).
struct TokenGeom {
    int64_t T;        // tokens in the tensor
    int64_t S;        // tokens per chunk (one table per chunk)
    int32_t nsc;      // sub-chunks in a full chunk = ceil(S / 256)
};

__host__ __device__ inline void sub_range(const TokenGeom &g, int64_t sub, int64_t &chunk,
                                          int64_t &t0, int &n)
{
    chunk = sub / g.nsc;
    const int64_t j = sub - chunk * g.nsc;
    t0 = chunk * g.S + j * kSub;
    int64_t tend = (chunk + 1) * g.S;
    if (tend > g.T) tend = g.T;
    const int64_t left = tend - t0;
    n = left < kSub ? (int)left : kSub;
}

// ------------------------------------------------------------------------------------
// device helpers
// ------------------------------------------------------------------------------------
__device__ __forceinline__ float f16_bits_to_float(uint32_t h)
{
    _Float16 v;
    uint16_t b = (uint16_t)h;
    __builtin_memcpy(&v, &b, 2);
    return (float)v;
}
__device__ __forceinline__ float bf16_bits_to_float(uint32_t h) { return __uint_as_float(h << 16); }

template <int DT>
__device__ __forceinline__ float load16f(uint32_t bits)
{
    return DT == CG_DT_BF16 ? bf16_bits_to_float(bits) : f16_bits_to_float(bits);
}

__device__ __forceinline__ uint32_t float_to_f16_bits(float f)
{
    _Float16 v = (_Float16)f;      // v_cvt_f16_f32, round to nearest even
    uint16_t b;
    __builtin_memcpy(&b, &v, 2);
    return b;
}
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f)
{
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (u >> 16) | 0x40u;
    u += 0x7FFFu + ((u >> 16) & 1u);
    return u >> 16;
}
template <int DT>
__device__ __forceinline__ uint32_t store16f(float f)
{
    return DT == CG_DT_BF16 ? float_to_bf16_bits(f) : float_to_f16_bits(f);
}

// 24-bit multiply, low 32 bits of the product, as an unsigned value (HIP's __umul24 returns
// int, which would turn a following >> into an arithmetic shift).
__device__ __forceinline__ uint32_t mul24(uint32_t a, uint32_t b) { return (uint32_t)__umul24(a, b); }

// floor(span * c / 2^16), the `(span * c) >> precision` of enc_new.cu:272-273 and
// dec_new.cu:280-281, on the full-rate 24-bit multiplier from the span's halves
// (sh = span >> 16, sl = span & 0xffff): span*c = sh*c*2^16 + sl*c.  Valid for every span
// below 2^32 and every c up to and including 2^16 (where it returns the span).
__device__ __forceinline__ uint32_t scale_span(uint32_t sh, uint32_t sl, uint32_t c)
{
    return mul24(sh, c) + (mul24(sl, c) >> 16);
}

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

struct PackedQuantArgs {
    const uint16_t *kv;
    int64_t L, sl, skv, st, sh;
    int32_t D;
    const float *key_bins, *value_bins;
    uint32_t *sym4;
    uint16_t *maxima;       // [2L, T]
    int32_t nunits;         // C / 8
    int64_t nsub;
    int32_t delta_group;    // > 0: tokens of a sub-chunk in groups of this many, see below
    TokenGeom g;
};

// One wavefront quantizes four consecutive tokens of one row (encoder.py:42-59) and
// writes, per channel, one word holding the four symbols: 32 contiguous bytes per lane
// and unit, 2 KB per wave and store pair.
template <int DT, bool HEADS_CONTIGUOUS, int NU>
__global__ __launch_bounds__(256) void quantize_pack_kernel(PackedQuantArgs a)
{
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
    const float bins = (kvi ? a.value_bins : a.key_bins)[l];
    const float maxq = floorf(bins * 0.5f) - 1.0f;
    const uint16_t *base = a.kv + l * a.sl + kvi * a.skv + (t0 + tt0) * a.st;

    uint4 regs[4][NU];
    float factor[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        uint32_t m = 0;
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            regs[j][i] = make_uint4(0, 0, 0, 0);
            const int u = lane + 64 * i;
            if (j < nvalid && u < a.nunits) {
                const int e = u * 8;
                int64_t off;
                if (HEADS_CONTIGUOUS) off = e;
                else { const int h = e / a.D; off = (int64_t)h * a.sh + (e - h * a.D); }
                regs[j][i] = *reinterpret_cast<const uint4 *>(base + j * a.st + off);
                m = pk_max_u16(m, regs[j][i].x & 0x7FFF7FFFu);
                m = pk_max_u16(m, regs[j][i].y & 0x7FFF7FFFu);
                m = pk_max_u16(m, regs[j][i].z & 0x7FFF7FFFu);
                m = pk_max_u16(m, regs[j][i].w & 0x7FFF7FFFu);
            }
        }
        m = (m & 0xFFFFu) > (m >> 16) ? (m & 0xFFFFu) : (m >> 16);
        m = wave_max_u32(m);
        if (j < nvalid && lane == 0) a.maxima[row * a.g.T + t0 + tt0 + j] = (uint16_t)m;
        // rows past the end of the sub-chunk are all zero: 0 * inf = NaN -> symbol byte 0
        factor[j] = __fdiv_rn(maxq, load16f<DT>(m));
    }

    const int64_t C = (int64_t)a.nunits * 8;
    uint32_t *out = a.sym4 + ((row * a.nsub + sub) * kWordsPerSub + tq) * C;
#pragma unroll
    for (int i = 0; i < NU; ++i) {
        const int u = lane + 64 * i;
        if (u < a.nunits) {
            uint32_t words[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                uint32_t w = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t src = k < 2 ? regs[j][i].x : k < 4 ? regs[j][i].y
                                       : k < 6 ? regs[j][i].z : regs[j][i].w;
                    const uint32_t bits = (k & 1) ? (src >> 16) : (src & 0xFFFFu);
                    const float v = load16f<DT>(bits);
                    const float s = __fadd_rn(__fmul_rn(v, factor[j]), maxq);
                    const float r = fmaxf(__builtin_rintf(s), 0.0f);     // NaN -> 0
                    w = __builtin_amdgcn_cvt_pk_u8_f32(r, (uint32_t)j, w);
                }
                words[k] = w;
            }
            uint4 *dst = reinterpret_cast<uint4 *>(out + (int64_t)u * 8);
            dst[0] = make_uint4(words[0], words[1], words[2], words[3]);
            dst[1] = make_uint4(words[4], words[5], words[6], words[7]);
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

// ------------------------------------------------------------------------------------
// Tables (cal_cdf.cu:17-59): one lane per (chunk, row, channel) walks the chunk's tokens
// and counts into its own LDS column hist[bin][lane] (no atomics across lanes, no bank
// conflicts); the running sum and the normalisation
//   cdf[i] = (uint16)((0xFFFF - max_bins) * cum[i] / cum[max_bins]) + i
// are done per lane in 16-bit wrap-around arithmetic like the reference's uint16
// counters, and the block writes its tables back transposed so stores coalesce.
// ------------------------------------------------------------------------------------

// Running sum and normalisation of one lane's column col[i * BS], i in [0, lp).
template <int BS>
__device__ __forceinline__ void normalize_column(uint32_t *col, int lp, int max_bins)
{
    uint32_t running = 0;
    for (int i = 1; i < lp; ++i) {
        running = (running + col[i * BS]) & 0xFFFFu;
        col[i * BS] = running;
    }
    const uint32_t scale = 0xFFFFu - (uint32_t)max_bins;
    for (int i = 0; i < lp; ++i) {
        const uint32_t q = running ? (scale * col[i * BS] / running) & 0xFFFFu : 0u;
        col[i * BS] = (q + (uint32_t)i) & 0xFFFFu;
    }
}

// Write the block's tables tab[entry * BS + lane] to cdf[lane][entry], coalesced.
template <int BS>
__device__ __forceinline__ void write_tables(const uint32_t *tab, uint16_t *cdf, int lp, int64_t ch0, int64_t nc)
{
    const int64_t nvalid = (nc - ch0 < BS) ? (nc - ch0) : BS;
    const int total = (int)nvalid * lp;
    for (int i = threadIdx.x; i < total; i += BS) {
        const int c = i / lp, e = i - c * lp;
        cdf[i] = (uint16_t)tab[e * BS + c];
    }
}

// Load the block's tables into LDS as tab[entry * BS + lane] (32-bit words).
template <int BS>
__device__ __forceinline__ void stage_tables(uint32_t *tab, const uint16_t *cdf, int lp, int64_t ch0, int64_t nc)
{
    const int64_t nvalid = (nc - ch0 < BS) ? (nc - ch0) : BS;
    const int total = (int)nvalid * lp;
    for (int i = threadIdx.x; i < total; i += BS) {
        const int c = i / lp, e = i - c * lp;
        tab[e * BS + c] = cdf[i];
    }
}

// The stream kernels keep their tables in LDS as 16-bit entries tab[entry * BS + lane]
// (half the footprint, twice the resident waves).  The end of a table, 2^16, does not fit
// and is substituted where the last symbol's upper bound is read.
template <int BS>
__device__ __forceinline__ void stage_tables16(uint16_t *tab, const uint16_t *cdf, int lp, int64_t ch0, int64_t nc)
{
    const int64_t nvalid = (nc - ch0 < BS) ? (nc - ch0) : BS;
    const int total = (int)nvalid * lp;
    for (int i = threadIdx.x; i < total; i += BS) {
        const int c = i / lp, e = i - c * lp;
        tab[e * BS + c] = cdf[i];
    }
}

template <int BS>
__device__ __forceinline__ void write_tables16(const uint16_t *tab, uint16_t *cdf, int lp, int64_t ch0, int64_t nc)
{
    const int64_t nvalid = (nc - ch0 < BS) ? (nc - ch0) : BS;
    const int total = (int)nvalid * lp;
    for (int i = threadIdx.x; i < total; i += BS) {
        const int c = i / lp, e = i - c * lp;
        cdf[i] = tab[e * BS + c];
    }
}

// Running sum and normalisation of one lane's 16-bit column of counts when every one of
// `total` tokens was counted (1 <= total <= 65535, uniform over the block): the divide of
// cal_cdf.cu:11-14 becomes a shift or a float estimate corrected exactly.
template <int BS>
__device__ __forceinline__ void normalize_column16(uint16_t *col, int lp, int max_bins, uint32_t total)
{
    const uint32_t scale = 0xFFFFu - (uint32_t)max_bins;
    uint32_t running = 0;
    if ((total & (total - 1)) == 0) {
        const int sh = 31 - __builtin_clz(total);
        for (int i = 0; i < lp; ++i) {
            running += col[i * BS];
            col[i * BS] = (uint16_t)(((scale * running) >> sh) + (uint32_t)i);
        }
    } else {
        const float inv = __fdiv_rn(1.0f, (float)total);
        for (int i = 0; i < lp; ++i) {
            running += col[i * BS];
            const uint32_t x = scale * running;                  // < 2^32, quotient < 2^16
            uint32_t q = (uint32_t)((float)x * inv);
            int32_t rem = (int32_t)(x - q * total);
            if (rem < 0) { q--; rem += (int32_t)total; }
            if (rem >= (int32_t)total) q++;
            col[i * BS] = (uint16_t)(q + (uint32_t)i);
        }
    }
}

struct CdfArgs {
    const uint8_t *sym;     // byte symbols: sym[row*s0 + token*s1 + channel*s2]
    int64_t s0, s1, s2;
    const uint32_t *sym4;   // or packed symbols (see above)
    int64_t nsub;
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
    uint32_t *col = smem + tid;
    for (int i = 0; i < lp; ++i) col[i * BS] = 0;

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
                    if (v[j] < mb) col[(v[j] + 1) * BS]++;
            }
            for (; t < t1; ++t) {
                const uint32_t v = p[t * a.s1];
                if (v < mb) col[(v + 1) * BS]++;
            }
        } else {
            const int64_t sub0 = chunk * a.g.nsc;
            const int nsubs = (int)((t1 - t0 + kSub - 1) / kSub);
            for (int sidx = 0; sidx < nsubs; ++sidx) {
                const int64_t left = (t1 - t0) - (int64_t)sidx * kSub;
                const int n = left < kSub ? (int)left : kSub;
                const uint32_t *wp = a.sym4 + ((row * a.nsub + sub0 + sidx) * kWordsPerSub) * a.nc + ch;
                const int nwords = (n + 3) >> 2;
                for (int w0 = 0; w0 < nwords; w0 += 4) {
                    uint32_t v[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) v[j] = (w0 + j < nwords) ? wp[(int64_t)(w0 + j) * a.nc] : 0u;
#pragma unroll
                    for (int j = 0; j < 16; ++j) {
                        const uint32_t s = (v[j >> 2] >> (8 * (j & 3))) & 0xFFu;
                        if (w0 * 4 + j < n && s < mb) col[(s + 1) * BS]++;
                    }
                }
            }
        }
        normalize_column<BS>(col, lp, a.max_bins);
    }
    __syncthreads();
    const int64_t ch0 = (int64_t)ctile * BS;
    write_tables<BS>(smem, a.cdf + ((chunk * a.rows + row) * a.nc + ch0) * lp, lp, ch0, a.nc);
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

template <int BS>
__device__ __forceinline__ StreamId locate(const StreamGrid &sg)
{
    StreamId s;
    int64_t b = blockIdx.x;
    const int ctile = (int)(b % sg.ctiles);
    b /= sg.ctiles;
    s.row = b % sg.rows;
    s.sub = b / sg.rows;
    sub_range(sg.g, s.sub, s.chunk, s.t0, s.n);
    s.ch = (int64_t)ctile * BS + threadIdx.x;
    s.active = s.ch < sg.nc;
    return s;
}

// ---- encoder (enc_new.cu:21-97, 253-307) -------------------------------------------
// Bits are collected MSB-first in a 64-bit accumulator and leave as big-endian 32-bit words.
// Every lane of a wavefront runs the store code whenever one lane has a word ready, so words
// are written at fixed points, once per two symbols, instead of whenever a lane's
// accumulator fills; the accumulator takes the two symbols in between (a put that would not
// fit writes a word first).
// The E1/E2 run of a symbol is emitted at once: the n1 = clz(low ^ high) leading bits
// agree, and the pending complements go in after the first of them, which in arithmetic
// is  bits + ((2^pend - 1) << (n1 - 1))  over n1 + pend bits.  The E3 run k is the number
// of positions below those where low has ones and high has zeros.  One combined shift by
// n = n1 + k renormalises low and high; n <= 18 for any table whose symbols all have
// non-zero width, because the span stays above 2^30 between symbols.
template <bool ALIGNED>
struct BitWriter {
    uint8_t *wptr;          // where the next word goes
    int wstride;            // bytes from one word of the stream to the next (4: contiguous)
    int cap;
    int nbytes;
    uint64_t acc;           // the low `nacc` bits are waiting to be written; bits above are stale
    int nacc;

    // the last words of a stream that does not fit its slot: keep what fits
    __device__ __forceinline__ void store_clipped(uint32_t word)
    {
        for (int j = 0; j < 4; ++j)
            if (nbytes + j < cap) wptr[j] = (uint8_t)(word >> (24 - 8 * j));
    }

    __device__ __forceinline__ void store_word(uint32_t word)
    {
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
        if (nacc >= 32) {
            store_word((uint32_t)(acc >> (nacc - 32)));
            nacc -= 32;
        }
    }

    // append the low m bits of v (v < 2^m), 0 <= m <= 32 (m = 0 needs v = 0)
    __device__ __forceinline__ void put(uint32_t v, int m)
    {
        if (__builtin_expect(nacc + m > 64, 0)) flush_word();       // more than 32 are waiting then
        acc = (acc << m) | v;
        nacc += m;
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
        if (nacc > 0) {
            uint32_t r = (uint32_t)(acc << (32 - nacc));
            for (int left = nacc, j = 0; left > 0; left -= 8, ++j) {
                if (nbytes < cap) wptr[j] = (uint8_t)(r >> 24);
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
template <int BS, bool ALIGNED>
struct RangeEncoder {
    const uint16_t *col;    // this lane's table column: entry e at col[e * BS]
    uint32_t smax;          // lp - 2: the largest symbol
    uint32_t low, span, pend;
    BitWriter<ALIGNED> w;

    __device__ __forceinline__ void init(const uint16_t *column, int lp, uint8_t *dst, int wstride, int cap)
    {
        col = column;
        smax = (uint32_t)(lp - 2);
        low = 0;
        span = 0;
        pend = 0;
        w.wptr = dst;
        w.wstride = wstride;
        w.cap = cap;
        w.nbytes = 0;
        w.acc = 0;
        w.nacc = 0;
    }

    // SENTINEL: symbol smax may occur, whose upper bound is 2^16 and not the table's last
    // entry (enc_new.cu:270)
    template <bool SENTINEL>
    __device__ __forceinline__ void put_symbol(uint32_t s)
    {
        s = s < smax ? s : smax;                        // keep table reads inside the table
        const uint32_t c_lo = col[s * BS];
        const uint32_t c_next = col[s * BS + BS];
        const uint32_t c_hi = (SENTINEL && s == smax) ? 0x10000u : c_next;
        uint32_t t_lo, width;
        if (__builtin_expect(span == 0, 0)) {
            t_lo = c_lo << 16;
            width = (c_hi - c_lo) << 16;
        } else {
            const uint32_t sh = span >> 16, sl = span & 0xFFFFu;
            t_lo = scale_span(sh, sl, c_lo);
            width = scale_span(sh, sl, c_hi) - t_lo;
        }
        low += t_lo;
        const uint32_t high = low + width - 1u;

        const int n1 = __builtin_clz(low ^ high);       // low < high always
        // the n1 agreed bits (none if n1 = 0) with the pending complements after the first
        const uint32_t pe = n1 > 0 ? pend : 0u;
        const int m = n1 + (int)pe;
        if (__builtin_expect(m > 32, 0)) {
            const uint32_t bits = low >> ((32 - n1) & 31);
            w.bit_and_run(bits >> (n1 - 1), pe);
            w.put(bits & ((1u << (n1 - 1)) - 1u), n1 - 1);
        } else {
            const uint32_t bits = __builtin_amdgcn_ubfe(low, (uint32_t)(32 - n1), (uint32_t)n1);
            const uint32_t fill = ((1u << (pe & 31)) - 1u) << ((n1 - 1) & 31);
            w.put(bits + fill, m);
        }
        // E3 run: leading zeros of (~low | high) below the first differing bit
        const uint32_t z = ((low & high) | ~low) << ((n1 + 1) & 31);
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
    int64_t *tile_sums;     // SLOTS, one block per tile of kSlotTile streams: stored bytes per tile, or null
    const float *key_bins, *value_bins;     // float32 [L] each, or null when the levels are not known
    int64_t L;
    StreamGrid sg;
};

constexpr int kSlotTile = 256;      // streams per tile of the encoder's scratch

template <bool B>
struct BoolTag {
    static constexpr bool value = B;
};

// PACKED: symbols come from sym4.  FUSE_CDF (PACKED only, one sub-chunk per chunk): the
// block first builds its own tables from the same words and writes them out.
// SLOTS: stream g of the launch is written to out[g * cap ...] (the fused path's scratch).
template <int BS, bool ALIGNED, bool PACKED, bool FUSE_CDF, bool SLOTS>
__global__ __launch_bounds__(BS) void encode_streams_kernel(EncodeArgs a)
{
    extern __shared__ uint16_t tab[];
    const int tid = threadIdx.x;
    const StreamId id = locate<BS>(a.sg);
    const int lp = a.lp;
    const int64_t ch0 = id.ch - tid;
    uint16_t *col = tab + tid;
    uint16_t *cdf_block = a.cdf + ((id.chunk * a.sg.rows + id.row) * a.sg.nc + ch0) * lp;
    const uint32_t *wp = nullptr;
    const int nwords = (id.n + 3) >> 2;
    if (PACKED) wp = a.sym4 + ((id.row * a.nsub + id.sub) * kWordsPerSub) * a.sg.nc + id.ch;

    // PACKED: half a sub-chunk (32 words = 128 symbols) at a time is loaded into registers
    // and indexed by the (uniform) loop counter, so the coding loop has no loads to wait
    // for and its stores never hold it up.
    typedef uint32_t words32 __attribute__((ext_vector_type(32)));
    words32 words;
    auto load_half = [&](int h) {
#pragma unroll
        for (int w = 0; w < 32; ++w)
            words[w] = (id.active && h * 32 + w < nwords) ? wp[(int64_t)(h * 32 + w) * a.sg.nc] : 0u;
    };

    if (FUSE_CDF) {
        for (int i = 0; i < lp; ++i) col[i * BS] = 0;
        if (id.active) {
            const uint32_t smax = (uint32_t)(lp - 2);
            for (int h = 0; h * 32 < nwords; ++h) {
                load_half(h);
                const int wn = nwords - h * 32 < 32 ? nwords - h * 32 : 32;
#pragma unroll 1
                for (int w = 0; w < wn; ++w) {
                    const uint32_t v = words[w];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        uint32_t s = (v >> (8 * j)) & 0xFFu;
                        s = s < smax ? s : smax;
                        if ((h * 32 + w) * 4 + j < id.n) col[(s + 1) * BS]++;   // the column is this lane's own
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

    RangeEncoder<BS, ALIGNED> enc;
    const int64_t stream = (id.sub * a.sg.rows + id.row) * a.sg.nc + id.ch;
    // SLOTS: the scratch is cut into tiles of kSlotTile streams; word w of a tile's stream t is
    // the tile's word w * kSlotTile + t, so that the words the lanes of a wavefront write, and
    // the words the compaction reads, lie side by side
    if (SLOTS)
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
                const int wn = nwords - h * 32 < 32 ? nwords - h * 32 : 32;
#pragma unroll 1
                for (int w = 0; w < wn; ++w) {
                    const uint32_t v = words[w];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if ((h * 32 + w) * 4 + j < id.n) enc.template put_symbol<SENTINEL>((v >> (8 * j)) & 0xFFu);
                        if (j & 1) enc.w.flush_word();
                    }
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
                for (int j = 0; j < 8; ++j) {
                    if (i0 + j < id.n) enc.template put_symbol<SENTINEL>(cur[j]);
                    if (j & 1) enc.w.flush_word();
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
            int64_t total = 0;
            for (int w = 0; w < BS / 64; ++w) total += wave_sums[w];
            a.tile_sums[blockIdx.x] = total;
        }
    }
}

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
// is topped up at fixed points, once per two symbols, instead of whenever a lane runs dry:
// after a top-up it holds more than 32 bits, a symbol of a table without zero-width entries
// consumes at most 18 (the span stays above 2^30), and the one case left (fewer than 18 bits
// before the second symbol of a pair) takes an extra top-up.
// Bits past the end of a stream are whatever follows it in memory instead of the reference's
// zeros (dec_new.cu:223-233): the coder's two closing bits place the code value inside
// the final interval for every continuation, so the n symbols that were encoded decode
// identically.  Word loads are clamped to the last word of the byte buffer.
struct BitReader {
    const uint8_t *base;     // the aligned word holding the stream's first byte
    uint32_t last;           // byte offset from `base` of the last word that may be read
    uint32_t pos;            // byte offset from `base` of the next word to fetch
    uint64_t win;            // the next `avail` bits of the stream, left-aligned, zeros below
    int avail;
    uint32_t nextw;          // the word after the window, as loaded

    __device__ __forceinline__ uint32_t raw()
    {
        const uint32_t at = pos < last ? pos : last;
        pos += 4;
        return *reinterpret_cast<const uint32_t *>(base + at);
    }

    // position on the stream that begins `begin` bytes after the 4-byte aligned `window`,
    // whose last readable word is at byte offset `last_word`; returns the first 32 bits
    __device__ __forceinline__ uint32_t start(const uint8_t *window, int64_t last_word, int64_t begin)
    {
        // a start outside the buffer (offsets that are not running sums of stream lengths) is
        // moved inside it: such a stream decodes to garbage, never to a read out of bounds
        begin = begin < 0 ? 0 : (begin > last_word ? last_word : begin);
        const uint32_t skip = (uint32_t)begin & 3u;
        const int64_t first_word = begin - skip;
        base = window + first_word;
        const int64_t room = last_word - first_word;
        last = room < 0 ? 0u : (room > 0xFFFFFFF0ll ? 0xFFFFFFF0u : (uint32_t)room);
        pos = 0;
        const uint32_t b0 = __builtin_bswap32(raw()), b1 = __builtin_bswap32(raw());
        const uint32_t b2 = __builtin_bswap32(raw());
        nextw = raw();
        const uint32_t s = skip * 8u;
        const uint64_t head = (((uint64_t)b0 << 32) | b1) << s;
        const uint64_t rest = (((uint64_t)b1 << 32) | b2) << s;
        win = rest;
        avail = 64 - (int)s;
        return (uint32_t)(head >> 32);
    }

    // off = (off << n) | next n bits, 0 <= n <= 31 and n <= avail
    __device__ __forceinline__ uint32_t shift_in(uint32_t off, int n)
    {
        off = (off << n) | __builtin_amdgcn_ubfe((uint32_t)(win >> 32), (uint32_t)(32 - n), (uint32_t)n);   // n = 0 extracts nothing
        win <<= n;
        avail -= n;
        return off;
    }

    // brings the window to more than 32 bits
    __device__ __forceinline__ void top_up()
    {
        if (avail <= 32) {                      // the low word is empty
            win |= (((uint64_t)__builtin_bswap32(nextw)) << 32) >> (avail & 63);
            avail += 32;
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

typedef __attribute__((address_space(3))) const uint16_t lds_u16;
typedef __attribute__((address_space(3))) const float lds_f32;
typedef __attribute__((address_space(3))) const char lds_char;

__device__ __forceinline__ uint32_t lds_entry(lds_char *p, int byte_offset)
{
    return *(lds_u16 *)(p + byte_offset);
}

// float32 -> bfloat16 bits, round to nearest even, for anything but a NaN
__device__ __forceinline__ uint32_t float_to_bf16_bits_no_nan(float f)
{
    uint32_t u = __float_as_uint(f);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return u >> 16;
}

struct DecodeLane {
    BitReader rd;
    uint32_t off, low, span;
    lds_char *colp;            // this lane's entry 0
    int lutoff;                // from an entry of this lane to its row's quotient
    uint8_t *osym;
    uint16_t *okv;
    float anchor;              // reconstructed anchor row value (delta mode)
    int phase;                 // position of the token inside its group (delta mode)
};

// One symbol.  SKIP: how many of the search's first probes are left out because the row's
// alphabet fits the lower 2^(LOG2-SKIP) entries.  SAFE: the last table entry may be decoded
// (its upper bound 2^16 is substituted, dec_new.cu:278) and values may be NaN.
template <int BS, int LOG2, int OUT, int SKIP, bool SAFE>
__device__ __forceinline__ void decode_symbol(const DecodeArgs &a, DecodeLane &s, int lp, int nsteps,
                                              float rm, int i, bool last_symbol)
{
    constexpr int kRow = DecodeLayout<BS, OUT>::kRow;
    lds_char *p = s.colp;              // entry of the decoded symbol
    lds_char *const plast = s.colp + (lp - 2) * kRow;
    uint32_t t_lo, width;
    if (__builtin_expect(s.span == 0, 0)) {
        // full range: T(m) = cdf[m] << 16, so compare table values with off >> 16
        const uint32_t key = s.off >> 16;
        if (LOG2 >= 0) {
#pragma unroll
            for (int step = ((1 << LOG2) >> 1) >> SKIP; step >= 1; step >>= 1)
                p = (lds_entry(p, step * kRow) <= key) ? p + step * kRow : p;
        } else {
            int lo_i = 0, hi_i = lp - 1;
            for (int step = 0; step < nsteps; ++step) {
                const int mid = (lo_i + hi_i) >> 1;
                const bool le = mid > 0 && lds_entry(s.colp, mid * kRow) <= key;
                lo_i = le ? mid : lo_i;
                hi_i = le ? hi_i : mid;
            }
            p = s.colp + lo_i * kRow;
        }
        const uint32_t c_lo = lds_entry(p, 0);
        const uint32_t c_hi = (SAFE && p == plast) ? 0x10000u : lds_entry(p, kRow);
        t_lo = c_lo << 16;
        width = (c_hi - c_lo) << 16;
    } else {
        const uint32_t sh = s.span >> 16, sl = s.span & 0xFFFFu;
        if (LOG2 >= 0) {
            // probe with the lower bound sh * c <= T(c); it can only overshoot
#pragma unroll
            for (int step = ((1 << LOG2) >> 1) >> SKIP; step >= 1; step >>= 1) {
                const uint32_t t = mul24(sh, lds_entry(p, step * kRow));
                p = (t <= s.off) ? p + step * kRow : p;
            }
            t_lo = scale_span(sh, sl, lds_entry(p, 0));
            // entry 0 is 0 (forced when the tables are staged), so this stops there at the latest
            while (__builtin_expect(t_lo > s.off, 0)) {
                p -= kRow;
                t_lo = scale_span(sh, sl, lds_entry(p, 0));
            }
        } else {
            int lo_i = 0, hi_i = lp - 1;
            for (int step = 0; step < nsteps; ++step) {
                const int mid = (lo_i + hi_i) >> 1;
                const uint32_t t = scale_span(sh, sl, lds_entry(s.colp, mid * kRow));
                const bool le = mid > 0 && t <= s.off;
                lo_i = le ? mid : lo_i;
                hi_i = le ? hi_i : mid;
            }
            p = s.colp + lo_i * kRow;
            t_lo = scale_span(sh, sl, lds_entry(p, 0));
        }
        const uint32_t c_hi = (SAFE && p == plast) ? 0x10000u : lds_entry(p, kRow);
        width = scale_span(sh, sl, c_hi) - t_lo;
    }
    if (OUT == OUT_SYMBOLS) {
        s.osym[(int64_t)i * a.o1] = (uint8_t)((uint32_t)(p - s.colp) / (uint32_t)kRow);
    } else {
        const float q = *(lds_f32 *)(p + s.lutoff);
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
        if (OUT == OUT_BF16) bits = SAFE ? float_to_bf16_bits(v) : float_to_bf16_bits_no_nan(v);
        else bits = float_to_f16_bits(v);
        *s.okv = (uint16_t)bits;
        s.okv += a.ot;
    }
    if (last_symbol) return;                    // no update after the last symbol
    s.low += t_lo;
    s.off -= t_lo;
    const uint32_t high = s.low + width - 1u;
    const int n1 = __builtin_clz(s.low ^ high);
    // E3 run: positions below the first differing bit where low has 1 and high has 0, i.e.
    // leading zeros of (~low | high) once that bit is shifted out; the run always ends
    // inside the word because the interval is wider than one
    const uint32_t z = ((s.low & high) | (~s.low & 0xFFFFFFFFu)) << ((n1 + 1) & 31);   // one bit-field insert
    const int n = n1 + __builtin_clz(z);
    s.low = (s.low << n) & 0x7FFFFFFFu;
    s.span = width << n;
    s.off = s.rd.shift_in(s.off, n);
}

template <int BS, int LOG2, int OUT, int SKIP, bool SAFE>
__device__ __forceinline__ void decode_lane(const DecodeArgs &a, DecodeLane &s, int lp, int n, lds_f32 *rmp)
{
    int nsteps = 0;
    if (LOG2 < 0)
        while ((1 << nsteps) < lp - 1) ++nsteps;
    for (int i0 = 0; i0 < n; i0 += 4, rmp += 4) {
        // the maxima of the next four token rows (the array is padded to a multiple of four)
        float rm[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (OUT != OUT_SYMBOLS) {
#pragma unroll
            for (int j = 0; j < 4; ++j) rm[j] = rmp[j];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = i0 + j;
            if (i >= n) break;
            if ((j & 1) == 0) s.rd.top_up();
            else if (__builtin_expect(s.rd.avail < 18, 0)) s.rd.top_up();
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
    const int64_t ch0 = id.ch - tid;
    {
        // entry 0 of a table is 0 by construction (cal_cdf.cu:29-49 counts into hist[sym+1]);
        // it is stored as 0 whatever the input holds so that the walk back always ends
        const uint16_t *src = a.cdf + ((id.chunk * a.sg.rows + id.row) * a.sg.nc + ch0) * lp;
        const int64_t nvalid = (a.sg.nc - ch0 < BS) ? (a.sg.nc - ch0) : BS;
        const int total = (int)nvalid * lp;
        for (int i = tid; i < total; i += BS) {
            const int c = i / lp, e = i - c * lp;
            *reinterpret_cast<uint16_t *>(rows + e * kRow + 2 * c) = e == 0 ? (uint16_t)0 : src[i];
        }
    }
    int64_t kvi = 0, l = 0;
    int special = 0;                   // a row maximum that is infinite or NaN
    int nsym = lp;                     // symbols the row's alphabet can hold
    if (OUT != OUT_SYMBOLS) {
        kvi = id.row / a.L;
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
            special |= (__float_as_uint(m) & 0x7FFFFFFFu) >= 0x7F800000u;
            rowmax[i] = m;
        }
    }
    special = __syncthreads_or(special);
    if (!id.active) return;

    const int64_t stream = (id.sub * a.sg.rows + id.row) * a.sg.nc + id.ch;
    int64_t begin;
    if (SRC == SRC_OFFSETS) begin = a.offsets[stream];
    else if (SRC == SRC_PREFIX) begin = stream ? a.offsets[stream - 1] : 0;
    else begin = id.row * a.p0 + id.ch * a.p1;

    DecodeLane s;
    s.off = s.rd.start(a.bytes, a.last_word, begin + a.bytes_skew);
    s.low = 0;
    s.span = 0;                        // span modulo 2^32: 0 is the full range (see RangeEncoder)
    s.colp = (lds_char *)(rows + 2 * tid);
    s.lutoff = DecodeLayout<BS, OUT>::kQuot - 2 * tid;
    s.osym = nullptr;
    s.okv = nullptr;
    s.anchor = 0.0f;
    s.phase = 0;
    if (OUT == OUT_SYMBOLS) {
        s.osym = a.out_sym + id.row * a.o0 + id.t0 * a.o1 + id.ch * a.o2;
    } else {
        const int64_t h = id.ch / a.D;
        s.okv = a.out_kv + l * a.ol + kvi * a.okv + id.t0 * a.ot + h * a.oh + (id.ch - h * a.D);
    }
    lds_f32 *rmp = (lds_f32 *)rowmax;

    // all three conditions are uniform over the block
    const bool safe = OUT == OUT_SYMBOLS || LOG2 < 0 || special || a.delta_group > 0 || nsym > lp - 2;
    if (safe) decode_lane<BS, LOG2, OUT, 0, true>(a, s, lp, id.n, rmp);
    else if (LOG2 > 1 && nsym <= (1 << (LOG2 > 1 ? LOG2 - 1 : 0))) decode_lane<BS, LOG2, OUT, 1, false>(a, s, lp, id.n, rmp);
    else decode_lane<BS, LOG2, OUT, 0, false>(a, s, lp, id.n, rmp);
}

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
    int64_t run = sums[blockIdx.x] + block_exclusive_scan(s, lds, total);
    for (int j = 0; j < kScanPerThread; ++j) {
        if (base + j < n) offsets[base + j] = run;
        run += v[j];
        if (base + j == n - 1) offsets[n] = run;
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
// the exclusive running sum of the tiles' byte counts (tile_base), instead of being read.
template <bool SCAN>
__global__ __launch_bounds__(256) void compact_streams_kernel(
    const uint8_t *__restrict__ slots, int32_t cap, int64_t *__restrict__ offsets,
    const int32_t *__restrict__ lengths, const int64_t *__restrict__ tile_base,
    int64_t nstreams, uint8_t *__restrict__ payload, int64_t payload_cap, int32_t skew, int32_t *status)
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
        int64_t *lds = reinterpret_cast<int64_t *>(buf);       // kScanThreads values; buf is free until the copy
        int64_t total64;
        const int32_t before = (int32_t)block_exclusive_scan(mine, lds, total64);
        o0 = tile_base[blockIdx.x];
        rel[tid] = before;
        if (tid == 0) rel[kCompactStreams] = (int32_t)total64;
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

// ------------------------------------------------------------------------------------
// host-side launch helpers
// ------------------------------------------------------------------------------------
// Lanes per block: as many adjacent channels as possible while the per-block table
// (lp words per lane) stays well inside the default dynamic LDS window.
int pick_block(int64_t nc, int lp)
{
    int block = 256;
    if (lp > 80) block = 128;
    while (block > 64 && nc <= block / 2) block /= 2;
    return block;
}

int make_grid(int64_t rows, int64_t nc, int64_t T, int64_t S, int64_t nsub, int block,
              StreamGrid &sg, int64_t &nblocks)
{
    sg.rows = rows;
    sg.nc = nc;
    sg.ctiles = (int32_t)ceil_div(nc, block);
    sg.g.T = T;
    sg.g.S = S;
    sg.g.nsc = (int32_t)ceil_div(S, kSub);
    nblocks = nsub * rows * sg.ctiles;
    if (nblocks <= 0 || nblocks > INT_MAX) return fail(CG_ERR_ARG, "grid of %lld blocks is out of range", (long long)nblocks);
    return CG_OK;
}

// Run `launch` with the block size as a compile-time constant.
#define CG_DISPATCH_BS(block, ...)                      \
    do {                                                \
        if ((block) == 256) { constexpr int BS = 256; __VA_ARGS__; } \
        else if ((block) == 128) { constexpr int BS = 128; __VA_ARGS__; } \
        else { constexpr int BS = 64; __VA_ARGS__; }    \
    } while (0)

int launch_cdf(const uint8_t *sym, const uint32_t *sym4, int64_t nsub, int64_t rows, int64_t T,
               int64_t nc, int64_t s0, int64_t s1, int64_t s2, int max_bins, int64_t S,
               uint16_t *cdf, hipStream_t stream)
{
    const int block = pick_block(nc, max_bins + 1);
    CdfArgs a;
    a.sym = sym;
    a.s0 = s0;
    a.s1 = s1;
    a.s2 = s2;
    a.sym4 = sym4;
    a.nsub = nsub;
    a.cdf = cdf;
    a.rows = rows;
    a.nc = nc;
    a.ctiles = (int32_t)ceil_div(nc, block);
    a.max_bins = max_bins;
    a.g.T = T;
    a.g.S = S;
    a.g.nsc = (int32_t)ceil_div(S, kSub);
    const int64_t nblocks = ceil_div(T, S) * rows * a.ctiles;
    if (nblocks <= 0 || nblocks > INT_MAX) return fail(CG_ERR_ARG, "calculate_cdf: grid out of range");
    const size_t shmem = (size_t)(max_bins + 1) * block * sizeof(uint32_t);
    const dim3 grid((unsigned)nblocks), blk(block);
    if (sym4) CG_DISPATCH_BS(block, (calculate_cdf_kernel<BS, true><<<grid, blk, shmem, stream>>>(a)));
    else CG_DISPATCH_BS(block, (calculate_cdf_kernel<BS, false><<<grid, blk, shmem, stream>>>(a)));
    return check_launch("calculate_cdf");
}

int launch_scan(const int32_t *lengths, int64_t n, int32_t clamp, int64_t *offsets, void *scratch,
                hipStream_t stream)
{
    const int64_t ntiles = ceil_div(n, kScanTile);
    int64_t *sums = static_cast<int64_t *>(scratch);
    scan_tile_sums_kernel<<<dim3((unsigned)ntiles), dim3(kScanThreads), 0, stream>>>(lengths, n, clamp, sums);
    scan_sums_kernel<<<dim3(1), dim3(kScanThreads), 0, stream>>>(sums, ntiles);
    scan_apply_kernel<<<dim3((unsigned)ntiles), dim3(kScanThreads), 0, stream>>>(lengths, n, clamp, sums, offsets);
    return check_launch("scan_lengths");
}

int check_dt(int dt, const char *what)
{
    if (dt != CG_DT_F16 && dt != CG_DT_BF16) return fail(CG_ERR_ARG, "%s: dtype must be CG_DT_F16 or CG_DT_BF16", what);
    return CG_OK;
}

int check_lp(int lp, const char *what)
{
    if (lp < 2 || lp > CG_MAX_LP) return fail(CG_ERR_ARG, "%s: CDF length should be in [2, %d], got %d", what, CG_MAX_LP, lp);
    return CG_OK;
}

bool kv_vectorizable(const void *kv, int64_t D, int64_t C, int64_t sl, int64_t skv, int64_t st, int64_t sh)
{
    return (D % 8 == 0) && (sl % 8 == 0) && (skv % 8 == 0) && (st % 8 == 0) && (sh % 8 == 0) &&
           aligned_to(kv, 16) && (C / 8 <= 64 * kMaxUnits);
}

int launch_quantize(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D,
                    int64_t sl, int64_t skv, int64_t st, int64_t sh, const float *key_bins,
                    const float *value_bins, uint8_t *sym, void *maxima, hipStream_t stream)
{
    const int64_t C = H * D;
    const int64_t nrows = 2 * L * T;
    const int64_t nblocks = ceil_div(nrows, 4);
    if (nblocks > INT_MAX || C > INT_MAX) return fail(CG_ERR_ARG, "quantize: tensor too large for one launch");
    const bool vec = kv_vectorizable(kv, D, C, sl, skv, st, sh) && aligned_to(sym, 8);
    const uint16_t *p = static_cast<const uint16_t *>(kv);
    uint16_t *mx = static_cast<uint16_t *>(maxima);
    dim3 grid((unsigned)nblocks), block(256);
    if (vec) {
        const int nunits = (int)(C / 8);
        const bool contiguous = (sh == D);
#define CG_LAUNCH_Q(DT, HC) quantize_kv_kernel<DT, HC><<<grid, block, 0, stream>>>( \
        p, L, T, (int)D, sl, skv, st, sh, key_bins, value_bins, sym, mx, nunits, nrows)
        if (kv_dt == CG_DT_F16) { if (contiguous) CG_LAUNCH_Q(CG_DT_F16, true); else CG_LAUNCH_Q(CG_DT_F16, false); }
        else { if (contiguous) CG_LAUNCH_Q(CG_DT_BF16, true); else CG_LAUNCH_Q(CG_DT_BF16, false); }
#undef CG_LAUNCH_Q
    } else {
        if (kv_dt == CG_DT_F16)
            quantize_kv_generic_kernel<CG_DT_F16><<<grid, block, 0, stream>>>(
                p, L, T, (int)D, (int)C, sl, skv, st, sh, key_bins, value_bins, sym, mx, nrows);
        else
            quantize_kv_generic_kernel<CG_DT_BF16><<<grid, block, 0, stream>>>(
                p, L, T, (int)D, (int)C, sl, skv, st, sh, key_bins, value_bins, sym, mx, nrows);
    }
    return check_launch("quantize_kv");
}

template <int DT, bool HC>
void launch_quantize_pack_nu(const PackedQuantArgs &a, int64_t nblocks, hipStream_t stream)
{
    const dim3 grid((unsigned)nblocks), block(256);
    if (a.delta_group > 0) {
        if (a.nunits <= 128) quantize_pack_delta_kernel<DT, HC, 2><<<grid, block, 0, stream>>>(a);
        else if (a.nunits <= 256) quantize_pack_delta_kernel<DT, HC, 4><<<grid, block, 0, stream>>>(a);
        else quantize_pack_delta_kernel<DT, HC, 8><<<grid, block, 0, stream>>>(a);
        return;
    }
    if (a.nunits <= 128) quantize_pack_kernel<DT, HC, 2><<<grid, block, 0, stream>>>(a);
    else if (a.nunits <= 256) quantize_pack_kernel<DT, HC, 4><<<grid, block, 0, stream>>>(a);
    else quantize_pack_kernel<DT, HC, 8><<<grid, block, 0, stream>>>(a);
}

int launch_quantize_pack(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D,
                         int64_t sl, int64_t skv, int64_t st, int64_t sh, const float *key_bins,
                         const float *value_bins, uint32_t *sym4, void *maxima, int64_t nsub,
                         int64_t S, int delta_group, hipStream_t stream)
{
    PackedQuantArgs a;
    a.kv = static_cast<const uint16_t *>(kv);
    a.L = L;
    a.sl = sl;
    a.skv = skv;
    a.st = st;
    a.sh = sh;
    a.D = (int32_t)D;
    a.key_bins = key_bins;
    a.value_bins = value_bins;
    a.sym4 = sym4;
    a.maxima = static_cast<uint16_t *>(maxima);
    a.nunits = (int32_t)(H * D / 8);
    a.nsub = nsub;
    a.delta_group = delta_group;
    a.g.T = T;
    a.g.S = S;
    a.g.nsc = (int32_t)ceil_div(S, kSub);
    const int64_t nblocks = 2 * L * nsub * 16;
    if (nblocks > INT_MAX) return fail(CG_ERR_ARG, "quantize: tensor too large for one launch");
    const bool contiguous = (sh == D);
    if (kv_dt == CG_DT_F16) {
        if (contiguous) launch_quantize_pack_nu<CG_DT_F16, true>(a, nblocks, stream);
        else launch_quantize_pack_nu<CG_DT_F16, false>(a, nblocks, stream);
    } else {
        if (contiguous) launch_quantize_pack_nu<CG_DT_BF16, true>(a, nblocks, stream);
        else launch_quantize_pack_nu<CG_DT_BF16, false>(a, nblocks, stream);
    }
    return check_launch("quantize_pack");
}

// Describe the readable byte window [bytes, bytes + nbytes) to the bit reader, which
// loads aligned words at 32-bit offsets from the window's 4-byte-aligned base.
int set_byte_window(DecodeArgs &a, const uint8_t *bytes, int64_t nbytes, const char *what)
{
    if (nbytes <= 0) return fail(CG_ERR_ARG, "%s: empty byte buffer", what);
    const uint32_t skew = (uint32_t)(reinterpret_cast<uintptr_t>(bytes) & 3u);
    a.bytes = bytes - skew;
    a.bytes_skew = skew;
    a.last_word = (skew + nbytes - 1) & ~3ll;
    return CG_OK;
}

size_t decode_shmem(int lp, int block) { return align_up((size_t)lp * block * sizeof(uint16_t), 4) + (size_t)(lp + kSub) * sizeof(float); }

template <int SRC>
int launch_decode_symbols(const DecodeArgs &a, int64_t nblocks, int block, hipStream_t stream)
{
    const dim3 grid((unsigned)nblocks), blk(block);
    const size_t shmem = decode_shmem(a.lp, block);
    CG_DISPATCH_BS(block, (decode_streams_kernel<BS, -1, SRC, OUT_SYMBOLS><<<grid, blk, shmem, stream>>>(a)));
    return check_launch("decode");
}

template <int BS, int OUT>
void launch_decode_kv_log2(const DecodeArgs &a, dim3 grid, size_t shmem, hipStream_t stream)
{
    const dim3 blk(BS);
    switch (a.lp) {
    case 9: decode_streams_kernel<BS, 3, SRC_OFFSETS, OUT><<<grid, blk, shmem, stream>>>(a); break;
    case 17: decode_streams_kernel<BS, 4, SRC_OFFSETS, OUT><<<grid, blk, shmem, stream>>>(a); break;
    case 33: decode_streams_kernel<BS, 5, SRC_OFFSETS, OUT><<<grid, blk, shmem, stream>>>(a); break;
    case 65: decode_streams_kernel<BS, 6, SRC_OFFSETS, OUT><<<grid, blk, shmem, stream>>>(a); break;
    default: decode_streams_kernel<BS, -1, SRC_OFFSETS, OUT><<<grid, blk, shmem, stream>>>(a); break;
    }
}

}  // namespace

// ======================================================================================
// C ABI
// ======================================================================================
extern "C" {

const char *cg_last_error(void) { return g_error; }
int cg_abi_version(void) { return 2; }

int64_t cg_num_chunks(int64_t T, int64_t chunk_tokens)
{
    if (T <= 0 || chunk_tokens <= 0) return 0;
    return ceil_div(T, chunk_tokens);
}

int64_t cg_num_subchunks(int64_t T, int64_t chunk_tokens)
{
    if (T <= 0 || chunk_tokens <= 0) return 0;
    const int64_t nchunks = ceil_div(T, chunk_tokens);
    const int64_t last = T - (nchunks - 1) * chunk_tokens;
    return (nchunks - 1) * ceil_div(chunk_tokens, kSub) + ceil_div(last, kSub);
}

int cg_calculate_cdf(const int8_t *sym, int64_t nl, int64_t nt, int64_t nc, int64_t s0, int64_t s1,
                     int64_t s2, int max_bins, int16_t *cdf, void *stream)
{
    if (!sym || !cdf) return fail(CG_ERR_ARG, "calculate_cdf: null pointer");
    if (nl <= 0 || nt <= 0 || nc <= 0) return fail(CG_ERR_ARG, "calculate_cdf: empty input");
    if (max_bins < 1 || max_bins + 1 > CG_MAX_LP) return fail(CG_ERR_ARG, "Max bins must be less than %d", CG_MAX_LP);
    if (nt > 65535) return fail(CG_ERR_ARG, "calculate_cdf: at most 65535 tokens per table (16-bit counters)");
    return launch_cdf(reinterpret_cast<const uint8_t *>(sym), nullptr, 0, nl, nt, nc, s0, s1, s2, max_bins, nt,
                      reinterpret_cast<uint16_t *>(cdf), static_cast<hipStream_t>(stream));
}

int cg_encode_fast_new(const int16_t *cdf, int lp, const int8_t *sym, int64_t nl, int64_t nt, int64_t nc,
                       int64_t s0, int64_t s1, int64_t s2, uint8_t *out, int64_t cap, int64_t o0,
                       int64_t o1, int32_t *lengths, void *stream)
{
    if (!cdf || (!sym && nt > 0) || !out || !lengths) return fail(CG_ERR_ARG, "encode: null pointer");
    if (int rc = check_lp(lp, "encode")) return rc;
    if (nl <= 0 || nc <= 0 || nt < 0) return fail(CG_ERR_ARG, "encode: empty input");
    if (nt > kSub) return fail(CG_ERR_ARG, "Number of tokens should be less than or equal to %d", kSub);
    if (cap <= 0 || cap > INT_MAX) return fail(CG_ERR_ARG, "encode: bad output buffer length");
    const int block = pick_block(nc, lp);
    EncodeArgs a;
    memset(&a, 0, sizeof(a));
    a.cdf = reinterpret_cast<uint16_t *>(const_cast<int16_t *>(cdf));      // only read here
    a.lp = lp;
    a.sym = reinterpret_cast<const uint8_t *>(sym);
    a.s0 = s0;
    a.s1 = s1;
    a.s2 = s2;
    a.out = out;
    a.o0 = o0;
    a.o1 = o1;
    a.cap = (int32_t)cap;
    a.lengths = lengths;
    a.status = nullptr;
    int64_t nblocks;
    // nt == 0 still writes the two closing bits of every stream
    if (int rc = make_grid(nl, nc, nt ? nt : 1, nt ? nt : 1, 1, block, a.sg, nblocks)) return rc;
    if (nt == 0) a.sg.g.T = 0;
    const size_t shmem = (size_t)lp * block * sizeof(uint16_t);
    const bool aligned = aligned_to(out, 4) && o0 % 4 == 0 && o1 % 4 == 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)nblocks), blk(block);
    if (aligned) CG_DISPATCH_BS(block, (encode_streams_kernel<BS, true, false, false, false><<<grid, blk, shmem, st>>>(a)));
    else CG_DISPATCH_BS(block, (encode_streams_kernel<BS, false, false, false, false><<<grid, blk, shmem, st>>>(a)));
    return check_launch("encode");
}

int cg_decode_fast_new(const int16_t *cdf, int lp, const uint8_t *padded, int64_t cap, int64_t p0,
                       int64_t p1, const int32_t *lengths, int64_t nl, int64_t nt, int64_t nc,
                       uint8_t *out, int64_t o0, int64_t o1, int64_t o2, void *stream)
{
    if (!cdf || !padded || !lengths || !out) return fail(CG_ERR_ARG, "decode: null pointer");
    if (int rc = check_lp(lp, "decode")) return rc;
    if (nl <= 0 || nc <= 0 || nt <= 0) return fail(CG_ERR_ARG, "decode: empty input");
    if (nt > kSub) return fail(CG_ERR_ARG, "Number of tokens should be less than or equal to %d", kSub);
    if (cap <= 0 || cap > INT_MAX) return fail(CG_ERR_ARG, "decode: bad padded buffer length");
    const int block = pick_block(nc, lp);
    DecodeArgs a;
    memset(&a, 0, sizeof(a));
    a.cdf = reinterpret_cast<const uint16_t *>(cdf);
    a.lp = lp;
    if (int rc = set_byte_window(a, padded, (nl - 1) * p0 + (nc - 1) * p1 + cap, "decode")) return rc;
    a.p0 = p0;
    a.p1 = p1;
    a.out_sym = out;
    a.o0 = o0;
    a.o1 = o1;
    a.o2 = o2;
    int64_t nblocks;
    if (int rc = make_grid(nl, nc, nt, nt, 1, block, a.sg, nblocks)) return rc;
    return launch_decode_symbols<SRC_PADDED>(a, nblocks, block, static_cast<hipStream_t>(stream));
}

int cg_decode_fast_prefsum(const int16_t *cdf, int lp, const uint8_t *bytes, int64_t nbytes,
                           const int64_t *prefix, int64_t nl, int64_t nt, int64_t nc, uint8_t *out,
                           int64_t o0, int64_t o1, int64_t o2, void *stream)
{
    if (!cdf || !prefix || !out || !bytes) return fail(CG_ERR_ARG, "decode: null pointer");
    if (int rc = check_lp(lp, "decode")) return rc;
    if (nl <= 0 || nc <= 0 || nt <= 0) return fail(CG_ERR_ARG, "decode: empty input");
    if (nt > kSub) return fail(CG_ERR_ARG, "Number of tokens should be less than or equal to %d", kSub);
    const int block = pick_block(nc, lp);
    DecodeArgs a;
    memset(&a, 0, sizeof(a));
    a.cdf = reinterpret_cast<const uint16_t *>(cdf);
    a.lp = lp;
    if (int rc = set_byte_window(a, bytes, nbytes, "decode")) return rc;
    a.offsets = prefix;
    a.out_sym = out;
    a.o0 = o0;
    a.o1 = o1;
    a.o2 = o2;
    int64_t nblocks;
    if (int rc = make_grid(nl, nc, nt, nt, 1, block, a.sg, nblocks)) return rc;
    return launch_decode_symbols<SRC_PREFIX>(a, nblocks, block, static_cast<hipStream_t>(stream));
}

int cg_quantize_kv(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D, int64_t sl,
                   int64_t skv, int64_t st, int64_t sh, const float *key_bins, const float *value_bins,
                   uint8_t *sym, void *maxima, void *stream)
{
    if (!kv || !key_bins || !value_bins || !sym || !maxima) return fail(CG_ERR_ARG, "quantize: null pointer");
    if (int rc = check_dt(kv_dt, "quantize")) return rc;
    if (L <= 0 || T <= 0 || H <= 0 || D <= 0) return fail(CG_ERR_ARG, "quantize: empty input");
    return launch_quantize(kv, kv_dt, L, T, H, D, sl, skv, st, sh, key_bins, value_bins, sym, maxima,
                           static_cast<hipStream_t>(stream));
}

size_t cg_scan_workspace(int64_t n) { return align_up((size_t)(ceil_div(n > 0 ? n : 1, kScanTile) + 1) * sizeof(int64_t), 256); }

int cg_scan_lengths(const int32_t *lengths, int64_t n, int64_t *offsets, void *scratch,
                    size_t scratch_bytes, void *stream)
{
    if (!lengths || !offsets || !scratch) return fail(CG_ERR_ARG, "scan: null pointer");
    if (n <= 0) return fail(CG_ERR_ARG, "scan: empty input");
    if (scratch_bytes < cg_scan_workspace(n)) return fail(CG_ERR_WORKSPACE, "scan: scratch too small");
    return launch_scan(lengths, n, INT_MAX, offsets, scratch, static_cast<hipStream_t>(stream));
}

size_t cg_encode_kv_workspace(int64_t L, int64_t T, int64_t C, int64_t chunk_tokens)
{
    const int64_t nsub = cg_num_subchunks(T, chunk_tokens);
    const int64_t nstreams = nsub * 2 * L * C;
    size_t total = align_up((size_t)nstreams * kSub, 256);        // symbols: a 256-token slot per stream
    total += (size_t)ceil_div(nstreams, kSlotTile) * kSlotTile * kStreamCap;   // encoder scratch: whole tiles of slots
    total += cg_scan_workspace(nstreams);
    total += align_up((size_t)ceil_div(nstreams, kSlotTile) * sizeof(int64_t), 256);   // bytes per tile of streams
    return total;
}

int cg_encode_kv(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D, int64_t sl,
                 int64_t skv, int64_t st, int64_t sh, const float *key_bins, const float *value_bins,
                 int max_bins, int64_t chunk_tokens, int delta_group, int16_t *cdf, void *maxima,
                 int32_t *lengths, int64_t *offsets, uint8_t *payload, int64_t payload_cap,
                 int32_t *status, void *workspace, size_t workspace_bytes, void *stream)
{
    if (!kv || !key_bins || !value_bins || !cdf || !maxima || !lengths || !offsets || !payload || !status || !workspace)
        return fail(CG_ERR_ARG, "encode_kv: null pointer");
    if (int rc = check_dt(kv_dt, "encode_kv")) return rc;
    if (L <= 0 || T <= 0 || H <= 0 || D <= 0) return fail(CG_ERR_ARG, "encode_kv: empty input");
    if (chunk_tokens <= 0) return fail(CG_ERR_ARG, "encode_kv: chunk_tokens must be positive");
    if (chunk_tokens > 65535) return fail(CG_ERR_ARG, "encode_kv: at most 65535 tokens per chunk (16-bit counters)");
    if (int rc = check_lp(max_bins + 1, "encode_kv")) return rc;
    if (delta_group < 0 || delta_group > kSub) return fail(CG_ERR_ARG, "encode_kv: delta_group must be in [0, %d]", kSub);
    const int64_t C = H * D, rows = 2 * L;
    const int64_t nsub = cg_num_subchunks(T, chunk_tokens);
    const int64_t nstreams = nsub * rows * C;
    if (workspace_bytes < cg_encode_kv_workspace(L, T, C, chunk_tokens)) return fail(CG_ERR_WORKSPACE, "encode_kv: workspace too small");
    if (!aligned_to(workspace, 256)) return fail(CG_ERR_ARG, "encode_kv: workspace must be 256-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int lp = max_bins + 1;

    uint8_t *ws = static_cast<uint8_t *>(workspace);
    uint8_t *symbols = ws;
    ws += align_up((size_t)nstreams * kSub, 256);
    uint8_t *scratch = ws;     // kStreamCap bytes per stream, in tiles of kSlotTile word-interleaved streams
    ws += (size_t)ceil_div(nstreams, kSlotTile) * kSlotTile * kStreamCap;
    void *scan_scratch = ws;
    ws += cg_scan_workspace(nstreams);
    int64_t *tile_sums = reinterpret_cast<int64_t *>(ws);
    uint16_t *tables = reinterpret_cast<uint16_t *>(cdf);

    clear_status_kernel<<<1, 1, 0, s>>>(status);

    const int block = pick_block(C, lp);
    EncodeArgs a;
    memset(&a, 0, sizeof(a));
    a.cdf = tables;
    a.lp = lp;
    a.nsub = nsub;
    a.out = scratch;
    a.cap = kStreamCap;
    a.lengths = lengths;
    a.status = status;
    a.key_bins = key_bins;
    a.value_bins = value_bins;
    a.L = L;
    int64_t nblocks;
    if (int rc = make_grid(rows, C, T, chunk_tokens, nsub, block, a.sg, nblocks)) return rc;
    const size_t shmem = (size_t)lp * block * sizeof(uint16_t);
    const dim3 grid((unsigned)nblocks), blk(block);
    // when every encoder block is exactly one tile of the scratch, the blocks leave their byte
    // counts behind and the compaction computes the stream offsets itself
    const bool fused_scan = block == kSlotTile && C % kSlotTile == 0;
    a.tile_sums = fused_scan ? tile_sums : nullptr;

    const bool packed = kv_vectorizable(kv, D, C, sl, skv, st, sh) && C % 8 == 0;
    if (delta_group > 0 && !packed)
        return fail(CG_ERR_ARG, "encode_kv: delta groups need head sizes and strides that are multiples of 8 and a 16-byte aligned tensor");
    if (packed) {
        // four tokens per word, read by one lane per channel
        uint32_t *sym4 = reinterpret_cast<uint32_t *>(symbols);
        if (int rc = launch_quantize_pack(kv, kv_dt, L, T, H, D, sl, skv, st, sh, key_bins, value_bins, sym4,
                                          maxima, nsub, chunk_tokens, delta_group, s)) return rc;
        a.sym4 = sym4;
        if (chunk_tokens <= kSub) {
            // one sub-chunk per chunk: the encoder builds the tables itself
            CG_DISPATCH_BS(block, (encode_streams_kernel<BS, true, true, true, true><<<grid, blk, shmem, s>>>(a)));
        } else {
            if (int rc = launch_cdf(nullptr, sym4, nsub, rows, T, C, 0, 0, 0, max_bins, chunk_tokens, tables, s)) return rc;
            CG_DISPATCH_BS(block, (encode_streams_kernel<BS, true, true, false, true><<<grid, blk, shmem, s>>>(a)));
        }
    } else {
        // any shape or alignment: byte symbols [2L, T, C]
        if (int rc = launch_quantize(kv, kv_dt, L, T, H, D, sl, skv, st, sh, key_bins, value_bins, symbols, maxima, s)) return rc;
        if (int rc = launch_cdf(symbols, nullptr, 0, rows, T, C, T * C, C, 1, max_bins, chunk_tokens, tables, s)) return rc;
        a.sym = symbols;
        a.s0 = T * C;
        a.s1 = C;
        a.s2 = 1;
        CG_DISPATCH_BS(block, (encode_streams_kernel<BS, true, false, false, true><<<grid, blk, shmem, s>>>(a)));
    }
    if (int rc = check_launch("encode_kv")) return rc;

    const int64_t cblocks = ceil_div(nstreams, kCompactStreams);
    if (cblocks > INT_MAX) return fail(CG_ERR_ARG, "encode_kv: too many streams");
    const int32_t skew = (int32_t)(reinterpret_cast<uintptr_t>(payload) & 3u);
    if (fused_scan) {
        scan_sums_kernel<<<dim3(1), dim3(kScanThreads), 0, s>>>(tile_sums, cblocks);
        compact_streams_kernel<true><<<dim3((unsigned)cblocks), dim3(256), 0, s>>>(
            scratch, kStreamCap, offsets, lengths, tile_sums, nstreams, payload, payload_cap, skew, status);
    } else {
        if (int rc = launch_scan(lengths, nstreams, kStreamCap, offsets, scan_scratch, s)) return rc;
        compact_streams_kernel<false><<<dim3((unsigned)cblocks), dim3(256), 0, s>>>(
            scratch, kStreamCap, offsets, nullptr, nullptr, nstreams, payload, payload_cap, skew, status);
    }
    return check_launch("compact");
}

int cg_decode_kv(const int16_t *cdf, int max_bins, const void *maxima, int max_dt, const int64_t *offsets,
                 const uint8_t *payload, int64_t payload_bytes, const float *key_bins,
                 const float *value_bins, int64_t L, int64_t T, int64_t H, int64_t D,
                 int64_t chunk_tokens, int delta_group, void *out, int out_dt, int64_t ol, int64_t okv,
                 int64_t ot, int64_t oh, void *stream)
{
    if (!cdf || !maxima || !offsets || !key_bins || !value_bins || !out || !payload)
        return fail(CG_ERR_ARG, "decode_kv: null pointer");
    if (int rc = check_dt(max_dt, "decode_kv")) return rc;
    if (int rc = check_dt(out_dt, "decode_kv")) return rc;
    if (L <= 0 || T <= 0 || H <= 0 || D <= 0 || chunk_tokens <= 0) return fail(CG_ERR_ARG, "decode_kv: empty input");
    if (int rc = check_lp(max_bins + 1, "decode_kv")) return rc;
    if (delta_group < 0 || delta_group > kSub) return fail(CG_ERR_ARG, "decode_kv: delta_group must be in [0, %d]", kSub);
    const int64_t C = H * D, rows = 2 * L;
    if (D > INT_MAX) return fail(CG_ERR_ARG, "decode_kv: head size too large");
    const int64_t nsub = cg_num_subchunks(T, chunk_tokens);
    const int block = pick_block(C, max_bins + 1);
    DecodeArgs a;
    memset(&a, 0, sizeof(a));
    a.cdf = reinterpret_cast<const uint16_t *>(cdf);
    a.lp = max_bins + 1;
    if (int rc = set_byte_window(a, payload, payload_bytes, "decode_kv")) return rc;
    a.offsets = offsets;
    a.out_kv = static_cast<uint16_t *>(out);
    a.ol = ol;
    a.okv = okv;
    a.ot = ot;
    a.oh = oh;
    a.L = L;
    a.D = (int32_t)D;
    a.maxima = static_cast<const uint16_t *>(maxima);
    a.max_dt = max_dt;
    a.delta_group = delta_group;
    a.key_bins = key_bins;
    a.value_bins = value_bins;
    int64_t nblocks;
    if (int rc = make_grid(rows, C, T, chunk_tokens, nsub, block, a.sg, nblocks)) return rc;
    const size_t shmem = decode_shmem(a.lp, block);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid((unsigned)nblocks);
    if (out_dt == CG_DT_BF16) CG_DISPATCH_BS(block, (launch_decode_kv_log2<BS, OUT_BF16>(a, grid, shmem, s)));
    else CG_DISPATCH_BS(block, (launch_decode_kv_log2<BS, OUT_F16>(a, grid, shmem, s)));
    return check_launch("decode_kv");
}

}  // extern "C"
