// Part of the CacheGen KV codec library for MI355X (gfx950); included by cachegen_hip.hip, which
// is the one translation unit.  Quantization, row maxima, packed symbols and the tables of every
// chunk in one pass over the tensor.
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
// torch_quant_vectorized (encoder.py:42-59) and calculate_cdf (cal_cdf.cu:17-59) in one kernel:
// a block owns one (row of 2L, chunk) over ALL channels, quantizes its token rows as
// quantize_pack_kernel does (same words to the same places) and counts every symbol, as it is
// made, into 16-bit counters in LDS; at the end it turns the counts into the chunk's tables and
// writes them.  The quantizer is bound by HBM and issues vector instructions a third of the
// time; the count costs it one instruction and one LDS operation a symbol, where a separate
// pass over the symbols (in the coder, or in calculate_cdf_kernel) costs a second read of every
// symbol on a kernel that is bound by instruction issue.
//
// Counters: channel c is unit u = c / 8 (one 128-bit load), channel k = c % 8 of it; unit
// u = lane + 64 i belongs to a lane, and the channel pair (i, k / 2) of all 64 lanes has a
// sub-table of LP rows of 64 words, entry e of the lane's pair in word `lane` of row e, the
// even channel in the lower half.  The byte address of a counter is therefore
//   sub-table + e * 256 + lane * 4,
// which one byte permute builds from the packed symbol word (byte 1 = the symbol, byte 0 = the
// lane's offset), with the sub-table and the `+ 1` of hist[sym + 1] in the LDS instruction's
// immediate offset.  The lanes of a wavefront count into 64 different words.
// ------------------------------------------------------------------------------------
struct QuantTablesArgs {
    const uint16_t *kv;
    int64_t L, sl, skv, st, sh;
    int32_t D;
    const float *key_bins, *value_bins;
    int32_t *status;        // the encode call's status word, set to zero here (first launch of the call)
    int32_t *group_sums;    // ngroups sums the coder's blocks add to, set to zero here (may be null)
    int32_t ngroups;
    uint32_t *sym4;         // packed symbols, as quantize_pack_kernel writes them
    uint16_t *maxima;       // [2L, T]
    uint16_t *cdf;          // [chunk][row][channel][lp]
    int32_t nunits;         // C / 8
    int64_t nsub;
    int32_t nibbles;        // rows of at most 15 symbols are written four bits a symbol
    TokenGeom g;
    // A call with few (row, chunk) pairs and long chunks cuts every chunk into gridDim.z parts of
    // part_tokens tokens (a multiple of 256), one block each: a block then adds its counters to
    // the chunk's words of `partial` (the layout of the LDS counters, zero before the launch)
    // instead of writing tables, and tables_from_partial_kernel turns the sums into the tables.
    int32_t part_tokens;
    uint32_t *partial;      // null: one block per chunk, which writes the chunk's tables itself
};

// Lanes per block.  The counters of 1024 channels (33-entry tables) take 66 KiB, so two blocks
// share a compute unit's LDS; the kernel holds four token rows of all channels in registers,
// which leaves room for 16 wavefronts per compute unit: two blocks of eight, whose clearing and
// table phases overlap with the other block's streaming.  2048 channels need the whole LDS for
// one block, which then has 16 wavefronts itself.
template <int NU>
struct QuantTablesBlock {
    static constexpr int kThreads = NU <= 2 ? 512 : 1024;
};

template <int NU, int LP>
struct CountLayout {
    static constexpr int kPitch = LP * 256;                 // bytes of one sub-table
    static constexpr int kSubTables = NU * 4;
    static constexpr int kBytes = kSubTables * kPitch;
    // a group of sub-tables is reached through the instruction's 16-bit immediate offset; the
    // next group needs its base added to the address
    static constexpr int kReach = (65535 - 256) / kPitch + 1;
    static constexpr int kGroup = kReach >= 8 ? 8 : kReach >= 4 ? 4 : kReach >= 2 ? 2 : 1;
    static_assert((kGroup - 1) * kPitch + 256 <= 65535, "sub-table offset must fit the immediate offset");
    // idx = 4 i + kp: the lane's unit i and the channel pair kp inside it
    __host__ __device__ static constexpr int group_base(int idx) { return idx / kGroup * kGroup * kPitch; }
    __host__ __device__ static constexpr int sub_table(int idx) { return idx % kGroup * kPitch; }
};

typedef __attribute__((address_space(3))) uint32_t lds_word;

// cdf value of a running count (cal_cdf.cu:11-14): (scale * run) / total + entry, the divide as a
// shift (SHIFT: total is a power of two) or as a float estimate corrected exactly.
template <bool SHIFT>
__device__ __forceinline__ uint32_t normalized_entry(uint32_t run, uint32_t entry, uint32_t scale, uint32_t total, int sh, float inv)
{
    const uint32_t x = scale * run;                          // < 2^32, quotient < 2^16
    if (SHIFT) return ((x >> sh) + entry) & 0xFFFFu;
    uint32_t q = (uint32_t)((float)x * inv);
    int32_t rem = (int32_t)(x - q * total);
    if (rem < 0) { q--; rem += (int32_t)total; }
    if (rem >= (int32_t)total) q++;
    return (q + entry) & 0xFFFFu;
}

// The tables of one (row, chunk) from its counters in LDS (every thread of the block, after a
// barrier that follows the last count): `total` tokens were counted, `dst_tables` = the chunk's
// [channel][LP] entries.
template <int NU, int LP, int kThreads>
__device__ __forceinline__ void counts_to_tables(uint32_t *counts, uint32_t total, int nunits, uint16_t *dst_tables)
{
    typedef CountLayout<NU, LP> Layout;
    const int tid = threadIdx.x;
    // One thread per channel pair (the two halves of a counter word).  The 2 LP counts are read
    // in LP reads on immediate offsets; running sums and normalisation (cal_cdf.cu:11-14, 29-49)
    // happen in registers; the pair's two tables, which follow one another in memory, go back to
    // the LDS as LP words in the order of the output, from where the block writes its 2 * LP * C
    // bytes of tables with coalesced 128-bit stores.
    const bool shift = (total & (total - 1)) == 0;
    const int sh = 31 - __builtin_clz(total);
    const float inv = __fdiv_rn(1.0f, (float)total);
    constexpr uint32_t scale = 0xFFFFu - (uint32_t)(LP - 1);
    constexpr int kPairs = Layout::kSubTables * 64;
    static_assert(kPairs % kThreads == 0 || kPairs < kThreads, "");
    constexpr int kRounds = (kPairs + kThreads - 1) / kThreads;
    uint32_t cnt[kRounds][LP];
#pragma unroll
    for (int r = 0; r < kRounds; ++r) {
        const int p = tid + r * kThreads;
        const int idx = p >> 6, ln = p & 63;
        if (p < kPairs) {
            const uint32_t *w = counts + (Layout::group_base(idx) + Layout::sub_table(idx)) / 4 + ln;
#pragma unroll
            for (int e = 0; e < LP; ++e) cnt[r][e] = w[e * 64];
        }
    }
    __syncthreads();                         // every count is in registers: the LDS is free for the tables
#pragma unroll
    for (int r = 0; r < kRounds; ++r) {
        const int p = tid + r * kThreads;
        const int idx = p >> 6, ln = p & 63;
        const int u = ln + 64 * (idx >> 2);
        if (p < kPairs && u < nunits) {
            // the pair's place in the output: channels 8 u + 2 kp and the next, LP words
            uint32_t *dst = counts + ((int64_t)u * 4 + (idx & 3)) * LP;
            auto emit = [&](auto shift_tag) {
                constexpr bool SHIFT = decltype(shift_tag)::value;
                uint32_t ra = 0, rb = 0, pa = 0, pb = 0, b0 = 0;
#pragma unroll
                for (int e = 0; e < LP; ++e) {
                    ra += cnt[r][e] & 0xFFFFu;
                    rb += cnt[r][e] >> 16;
                    const uint32_t va = normalized_entry<SHIFT>(ra, (uint32_t)e, scale, total, sh, inv);
                    const uint32_t vb = normalized_entry<SHIFT>(rb, (uint32_t)e, scale, total, sh, inv);
                    // the sequence A[0..LP), B[0..LP) two entries a word
                    if (e & 1) dst[e >> 1] = pa | (va << 16);                       // A[e-1], A[e]
                    if (e == 0) b0 = vb;
                    else if (!(e & 1)) dst[(LP + e - 1) >> 1] = pb | (vb << 16);    // B[e-1], B[e]
                    if (e == LP - 1) dst[(LP - 1) >> 1] = va | (b0 << 16);          // A[LP-1], B[0]
                    pa = va;
                    pb = vb;
                }
            };
            if (shift) emit(BoolTag<true>());
            else emit(BoolTag<false>());
        }
    }
    __syncthreads();
    // C * LP 16-bit entries = C * LP / 8 quad words (C is a multiple of 8), 16-byte aligned in memory
    uint4 *const tables = reinterpret_cast<uint4 *>(dst_tables);
    const int nquads = nunits * LP;
    for (int q = tid; q < nquads; q += kThreads) tables[q] = reinterpret_cast<const uint4 *>(counts)[q];
}

// LP: the table length, max_bins + 1 (odd).
template <int DT, bool HEADS_CONTIGUOUS, int NU, int LP>
__global__ __launch_bounds__(QuantTablesBlock<NU>::kThreads, 4) void quantize_tables_kernel(QuantTablesArgs a)
{
    static_assert(LP % 2 == 1, "two tables of LP entries are written as LP words");
    constexpr int kThreads = QuantTablesBlock<NU>::kThreads;
    extern __shared__ uint32_t counts[];
    typedef CountLayout<NU, LP> Layout;
    const int tid = threadIdx.x, lane = tid & 63;
    // the same for every lane of a wavefront, and said so: token rows, symbol and maxima
    // addresses that depend on it are then computed once, on the scalar unit
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0) {
        if (tid == 0) *a.status = 0;
        if (a.group_sums && tid < a.ngroups) a.group_sums[tid] = 0;          // ngroups <= kMaxTileGroups < the block's threads
    }
    const int64_t chunk = blockIdx.x, row = blockIdx.y;
    // the block's tokens: the whole chunk, or part blockIdx.z of it (none, past the end of a short last chunk)
    const int part_t0 = (int)blockIdx.z * a.part_tokens;         // 0 when chunks are not cut
    const int64_t t0 = chunk * a.g.S + part_t0;
    int ntok;
    {
        const int64_t chunk_end = (chunk + 1) * a.g.S < a.g.T ? (chunk + 1) * a.g.S : a.g.T;
        const int64_t left = chunk_end - t0;
        ntok = (int)(left < 0 ? 0 : a.partial && left > a.part_tokens ? a.part_tokens : left);
    }
    const int64_t sub0 = chunk * a.g.nsc + (part_t0 >> 8);       // the block's first sub-chunk
    const int64_t kvi = row / a.L, l = row - kvi * a.L;
    const float bins = (kvi ? a.value_bins : a.key_bins)[l];
    const float maxq = floorf(bins * 0.5f) - 1.0f;
    const bool narrow = a.nibbles && narrow_alphabet(maxq, LP);
    // symbols that may lie past the table's last one are kept inside it before they are counted
    const bool fits = maxq >= 0.0f && 2.0f * maxq <= (float)(LP - 2);
    constexpr uint32_t smax = (uint32_t)(LP - 2);
    const int64_t C = (int64_t)a.nunits * 8;

    for (int i = tid; i < Layout::kBytes / 16; i += kThreads)
        reinterpret_cast<uint4 *>(counts)[i] = make_uint4(0, 0, 0, 0);
    __syncthreads();

    const uint32_t lane4 = (uint32_t)lane * 4u;
    const int ngroups = (ntok + 3) >> 2;
    constexpr int kWaves = kThreads / 64;

    // The chunk's token rows through a buffer descriptor at its first row: a unit's byte offset
    // inside a token row is the vector offset (one register per unit; a unit that does not exist
    // gets an offset outside the descriptor and reads zeros), the token row the scalar offset: no
    // 64-bit address arithmetic and no registers per row.
    const int64_t first_row = l * a.sl + kvi * a.skv + t0 * a.st;                // uniform over the block
    const uint32_t fr_lo = __builtin_amdgcn_readfirstlane((uint32_t)first_row);
    const uint32_t fr_hi = __builtin_amdgcn_readfirstlane((uint32_t)((uint64_t)first_row >> 32));
    const __amdgpu_buffer_rsrc_t rows = __builtin_amdgcn_make_buffer_rsrc(
        (void *)(a.kv + (int64_t)(((uint64_t)fr_hi << 32) | fr_lo)), 0, (int)0xFFFFFFF0u, kBufferWord3);
    uint32_t unit_off[NU];
#pragma unroll
    for (int i = 0; i < NU; ++i) {
        const int u = lane + 64 * i, e = u * 8;
        if (HEADS_CONTIGUOUS) unit_off[i] = (uint32_t)e * 2u;
        else { const int h = e / a.D; unit_off[i] = (uint32_t)((h * a.sh + (e - h * a.D)) * 2); }    // the host checks that this fits
        if (u >= a.nunits) unit_off[i] = 0xFFFFFFF0u;
    }
    const uint32_t row_step = (uint32_t)a.st * 2u;

    // the four token rows of group tg: loads only, nothing waits for them here
    auto issue = [&](int tg, uint4 (&regs)[4][NU]) {
        const int left = ntok - tg * 4;                      // token rows that exist from the group's first on
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int i = 0; i < NU; ++i) {
                regs[j][i] = make_uint4(0, 0, 0, 0);
                if (j < left) {
                    // read once by this kernel: loaded past the caches' keep-for-reuse policy
                    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                    const u32x4 t = __builtin_amdgcn_raw_buffer_load_b128(rows, (int)unit_off[i], (int)((uint32_t)(tg * 4 + j) * row_step), 2);
                    regs[j][i] = make_uint4(t.x, t.y, t.z, t.w);
                }
            }
        }
    };

    // maxima, scales and counts of group tg, whose rows are in `regs`
    auto consume = [&](int tg, const uint4 (&regs)[4][NU]) {
        const int tt0 = tg * 4;                              // first token of the group, counted from the block's first
        const int nvalid = ntok - tt0 < 4 ? ntok - tt0 : 4;
        float factor[4];
        bool plain = fits;                                   // uniform over the wavefront
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            uint32_t m = 0;
#pragma unroll
            for (int i = 0; i < NU; ++i) {
                m = pk_max_u16(m, regs[j][i].x & 0x7FFF7FFFu);
                m = pk_max_u16(m, regs[j][i].y & 0x7FFF7FFFu);
                m = pk_max_u16(m, regs[j][i].z & 0x7FFF7FFFu);
                m = pk_max_u16(m, regs[j][i].w & 0x7FFF7FFFu);
            }
            m = (m & 0xFFFFu) > (m >> 16) ? (m & 0xFFFFu) : (m >> 16);
            m = wave_max_u32(m);
            const float mf = load16f<DT>(m);
            factor[j] = __fdiv_rn(maxq, mf);
            if (j < nvalid && lane == 0) a.maxima[row * a.g.T + t0 + tt0 + j] = (uint16_t)m;
            plain = plain && !scale_overflows(maxq, mf);
        }
        const int64_t sub = sub0 + (tt0 >> 8);
        uint32_t *out = a.sym4 + ((row * a.nsub + sub) * kWordsPerSub + ((tt0 & (kSub - 1)) >> 2)) * C;
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            const int u = lane + 64 * i;
            if (u < a.nunits) {
                uint32_t words[8];
                const uint4 r[4] = {regs[0][i], regs[1][i], regs[2][i], regs[3][i]};
                quantize_unit<DT>(r, factor, maxq, words);
                // PLAIN: every byte is a table symbol (no row saturates, the table holds the
                // alphabet); FULL: all four token rows exist
                auto count = [&](auto plain_tag, auto full_tag) {
                    constexpr bool PLAIN = decltype(plain_tag)::value, FULL = decltype(full_tag)::value;
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        const int idx = 4 * i + (k >> 1);
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            if (FULL || j < nvalid) {
                                uint32_t addr;
                                if (PLAIN) {
                                    // byte 0: the lane's word, byte 1: the symbol
                                    addr = __builtin_amdgcn_perm(words[k], lane4, 0x0C0C0000u | ((4u + j) << 8));
                                    if (Layout::group_base(idx)) addr += Layout::group_base(idx);
                                } else {
                                    uint32_t q = (words[k] >> (8 * j)) & 0xFFu;
                                    q = q < smax ? q : smax;
                                    addr = (q << 8) + lane4 + Layout::group_base(idx);
                                }
                                lds_word *p = (lds_word *)(uintptr_t)(addr + Layout::sub_table(idx) + 256);
                                __hip_atomic_fetch_add(p, (k & 1) ? 0x10000u : 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                            }
                        }
                    }
                };
                if (plain && nvalid == 4) count(BoolTag<true>(), BoolTag<true>());
                else if (plain) count(BoolTag<true>(), BoolTag<false>());
                else count(BoolTag<false>(), BoolTag<false>());
                if (narrow) {
                    *reinterpret_cast<uint4 *>(out + (int64_t)u * 4) = pack_four_bit_words(words);
                } else {
                    uint4 *dst = reinterpret_cast<uint4 *>(out + (int64_t)u * 8);
                    dst[0] = make_uint4(words[0], words[1], words[2], words[3]);
                    dst[1] = make_uint4(words[4], words[5], words[6], words[7]);
                }
            }
        }
    };

    if (NU <= 2) {
        // two sets of registers: the next group's rows are on their way while this group's are counted
        uint4 ra[4][NU], rb[4][NU];
        int tg = wave;
        if (tg < ngroups) issue(tg, ra);
        for (; tg < ngroups; tg += 2 * kWaves) {
            if (tg + kWaves < ngroups) issue(tg + kWaves, rb);
            consume(tg, ra);
            if (tg + kWaves < ngroups) {
                if (tg + 2 * kWaves < ngroups) issue(tg + 2 * kWaves, ra);
                consume(tg + kWaves, rb);
            }
        }
    } else {
        // 2048 channels: one set of rows is all the registers hold
        uint4 ra[4][NU];
        for (int tg = wave; tg < ngroups; tg += kWaves) {
            issue(tg, ra);
            consume(tg, ra);
        }
    }

    __syncthreads();
    if (a.partial) {
        // the chunk's other parts add to the same words; what a block has not counted it does not touch
        uint32_t *sums = a.partial + ((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * (Layout::kBytes / 4);
        for (int i = tid; i < Layout::kBytes / 4; i += kThreads) {
            const uint32_t v = counts[i];
            if (v) __hip_atomic_fetch_add(sums + i, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }
    counts_to_tables<NU, LP, kThreads>(counts, (uint32_t)ntok, a.nunits,
                                       a.cdf + (((int64_t)blockIdx.x * gridDim.y + blockIdx.y) * a.nunits * 8) * LP);
}

// Zeroes n quad words (the counters in memory, before the blocks of a launch add to them).
__global__ __launch_bounds__(256) void clear_quads_kernel(uint4 *p, int64_t n)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = make_uint4(0, 0, 0, 0);
}

// The tables of the chunks whose counters quantize_tables_kernel summed in memory: a block per
// (chunk, row) copies the sums into its LDS and goes on as that kernel does at the end of a chunk.
template <int NU, int LP>
__global__ __launch_bounds__(QuantTablesBlock<NU>::kThreads, 4) void tables_from_partial_kernel(
    const uint32_t *__restrict__ partial, uint16_t *cdf, int32_t nunits, TokenGeom g)
{
    constexpr int kThreads = QuantTablesBlock<NU>::kThreads;
    extern __shared__ uint32_t counts[];
    typedef CountLayout<NU, LP> Layout;
    const int tid = threadIdx.x;
    const int64_t chunk = blockIdx.x, row = blockIdx.y;
    const int64_t t0 = chunk * g.S;
    const uint32_t total = (uint32_t)((t0 + g.S < g.T ? t0 + g.S : g.T) - t0);
    const uint4 *src = reinterpret_cast<const uint4 *>(partial + (chunk * gridDim.y + row) * (Layout::kBytes / 4));
    for (int i = tid; i < Layout::kBytes / 16; i += kThreads) reinterpret_cast<uint4 *>(counts)[i] = src[i];
    __syncthreads();
    counts_to_tables<NU, LP, kThreads>(counts, total, nunits, cdf + ((chunk * gridDim.y + row) * (int64_t)nunits * 8) * LP);
}

}  // namespace
