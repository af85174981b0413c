// Part of the CacheGen KV codec library for MI355X (gfx950); included by cachegen_hip.hip, which
// is the one translation unit.  Error reporting, 16-bit float conversions and small device helpers shared by every kernel.
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
    // one sub-chunk per chunk (tables per 256 tokens) needs no division; otherwise both fit 32 bits
    chunk = g.nsc == 1 ? sub : (int64_t)((uint32_t)sub / (uint32_t)g.nsc);
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

// (x + x) << n, i.e. x << (n + 1), in one instruction (n + 1 may be 32: the result is then 0
// if the bit shifted out last is the only one left, which a plain shift by n + 1 cannot express)
__device__ __forceinline__ uint32_t shift_left_one_more(uint32_t x, int n)
{
    uint32_t r;
    asm("v_add_lshl_u32 %0, %1, %1, %2" : "=v"(r) : "v"(x), "v"(n));
    return r;
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

// A compile-time flag as a value, for generic lambdas.
template <bool B>
struct BoolTag {
    static constexpr bool value = B;
};

// Fourth word of a buffer descriptor for raw (untyped, unswizzled) access on gfx9-family
// GPUs: 32-bit data format, everything else off.
constexpr int kBufferWord3 = 0x00020000;

// Pointers into LDS, for loads with immediate offsets.
typedef __attribute__((address_space(3))) const uint16_t lds_u16;
typedef __attribute__((address_space(3))) const float lds_f32;
typedef __attribute__((address_space(3))) const char lds_char;

// Entries at p and p + ROW bytes into the upper halves of `lo` and `hi` (entry << 16), whose
// lower halves must be zero on entry and are zero on return: the hardware either keeps them
// or clears them.  The compiler does not count loads issued from inline assembly, so the wait
// for them is part of it.
template <int ROW>
__device__ __forceinline__ void lds_entries_high(lds_char *p, uint32_t &lo, uint32_t &hi)
{
    asm volatile("ds_read_u16_d16_hi %0, %2\n\tds_read_u16_d16_hi %1, %2 offset:%3\n\ts_waitcnt lgkmcnt(0)"
                 : "+v"(lo), "+v"(hi)
                 : "v"(p), "n"(ROW));
}

}  // namespace
