// Part of the CacheGen KV codec library for MI355X (gfx950); included by cachegen_hip.hip, which
// is the one translation unit.  Tables <-> histogram counts, for containers that store the
// counts instead of the tables.
//
// A table is a function of its histogram (cal_cdf.cu:29-49 in LMCache/third_party/torchac_cuda):
//   cdf[i] = (0xFFFF - max_bins) * cum[i] / n + i,   cum = running sum of the counts, n = tokens
// and for n <= 256 the running sums are recovered from the table exactly, because the scale
// exceeds n: cum[i] = ceil((cdf[i] - i) * n / scale).  A "group" is one (chunk, row): C channels
// that share a token count and, in the ragged form, a number of stored symbols.
#pragma once

namespace {

constexpr int kWireThreads = 256;

__global__ void clear_ints_kernel(int32_t *a, int64_t na, int32_t *b)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < na) a[i] = 0;
    if (i == 0 && b) *b = 0;
}

// One thread per (group, channel).  counts: uint8 [ngroups, C, lp - 1], clamped to 255;
// nsym[g]: one more than the largest symbol that occurs in group g (at least 1);
// inexact: set to 1 if some table is not what the formula gives for any histogram.
__global__ __launch_bounds__(kWireThreads) void tables_to_counts_kernel(
    const uint16_t *__restrict__ cdf, int lp, int64_t C, const int32_t *__restrict__ tokens,
    uint8_t *__restrict__ counts, int32_t *nsym, int32_t *inexact)
{
    const int64_t g = blockIdx.y;
    const int64_t ch = (int64_t)blockIdx.x * kWireThreads + threadIdx.x;
    int last = 1;
    if (ch < C) {
        const uint32_t n = (uint32_t)tokens[g];
        const uint32_t scale = 0xFFFFu - (uint32_t)(lp - 1);
        const uint16_t *t = cdf + (g * C + ch) * lp;
        uint8_t *out = counts + (g * C + ch) * (lp - 1);
        bool exact = t[0] == 0;
        uint32_t prev = 0;
        for (int i = 1; i < lp; ++i) {
            const uint32_t c = t[i];
            const uint32_t q = c - (uint32_t)i;                    // wraps if c < i: caught by the rebuild
            const uint32_t cum = (q * n + scale - 1u) / scale;     // q < 2^16, n <= 256: no overflow
            exact = exact && c >= (uint32_t)i && cum >= prev && cum <= n && (scale * cum) / n + (uint32_t)i == c;
            const uint32_t count = cum >= prev ? cum - prev : 0u;
            out[i - 1] = (uint8_t)(count > 255u ? 255u : count);
            if (count) last = i;
            prev = cum;
        }
        exact = exact && prev == n;
        if (!exact) atomicOr(inexact, 1);
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const int other = __shfl_xor(last, o, 64);
        last = other > last ? other : last;
    }
    if ((threadIdx.x & 63) == 0) atomicMax(nsym + g, last);
}

// Ragged form: group g's channels in turn, nsym[g] counts each, from byte starts[g] on.
__global__ __launch_bounds__(kWireThreads) void pack_counts_kernel(
    const uint8_t *__restrict__ counts, int lp, int64_t C, const int32_t *__restrict__ nsym,
    const int64_t *__restrict__ starts, uint8_t *__restrict__ out)
{
    const int64_t g = blockIdx.y;
    const int64_t ch = (int64_t)blockIdx.x * kWireThreads + threadIdx.x;
    if (ch >= C) return;
    const int k = nsym[g];
    const uint8_t *src = counts + (g * C + ch) * (lp - 1);
    uint8_t *dst = out + starts[g] + ch * k;
    for (int j = 0; j < k; ++j) dst[j] = src[j];
}

// The inverse: ragged counts -> tables.  A count of 256 (one symbol for all n = 256 tokens)
// was stored as 255: the one token missing from the sum goes back to that entry.  invalid is
// set if a channel's counts cannot be completed to its group's token count that way.
__global__ __launch_bounds__(kWireThreads) void counts_to_tables_kernel(
    const uint8_t *__restrict__ data, int64_t data_bytes, int lp, int64_t C,
    const int32_t *__restrict__ tokens, const uint8_t *__restrict__ nsym,
    const int64_t *__restrict__ starts, uint16_t *__restrict__ cdf, int32_t *invalid)
{
    const int64_t g = blockIdx.y;
    const int64_t ch = (int64_t)blockIdx.x * kWireThreads + threadIdx.x;
    if (ch >= C) return;
    const int k = nsym[g];
    const int64_t at = starts[g] + ch * k;
    uint16_t *t = cdf + (g * C + ch) * lp;
    const uint32_t n = (uint32_t)tokens[g];
    const uint32_t scale = 0xFFFFu - (uint32_t)(lp - 1);
    if (k < 1 || k > lp - 1 || at < 0 || at + k > data_bytes) {      // never read outside the section
        atomicOr(invalid, 1);
        for (int i = 0; i < lp; ++i) t[i] = (uint16_t)i;
        return;
    }
    const uint8_t *src = data + at;
    uint32_t sum = 0, full = 0;
    for (int j = 0; j < k; ++j) {
        sum += src[j];
        full += src[j] == 255u;
    }
    const uint32_t missing = n - sum;                               // wraps if the sum is too large
    if (!(missing == 0u || (missing == 1u && full == 1u))) atomicOr(invalid, 1);
    uint32_t cum = 0;
    t[0] = 0;
    for (int i = 1; i < lp; ++i) {
        if (i - 1 < k) {
            const uint32_t c = src[i - 1];
            cum += c + ((c == 255u && missing == 1u) ? 1u : 0u);
        }
        t[i] = (uint16_t)((scale * cum) / (n ? n : 1u) + (uint32_t)i);
    }
}

}  // namespace
